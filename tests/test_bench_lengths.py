"""Synthetic prompt lengths of the offline benchmark (CPU only)."""

import pytest


def test_prompt_lengths_are_drawn_uniformly_and_fixed_by_the_seed():
    from rapid_llm_amd.cli import sample_prompt_lengths

    a = sample_prompt_lengths(2000, 64, 1024, 7)
    assert a == sample_prompt_lengths(2000, 64, 1024, 7) != sample_prompt_lengths(2000, 64, 1024, 8)
    assert min(a) >= 64 and max(a) <= 1024 and min(a) < 80 and max(a) > 1000
    assert abs(sum(a) / len(a) - 544) < 25
    assert sample_prompt_lengths(5, 9, 9, 0) == [9] * 5
    with pytest.raises(ValueError):
        sample_prompt_lengths(3, 10, 5, 0)
