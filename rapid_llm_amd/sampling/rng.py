"""The uniform draw of the sampling kernel, in Python: splitmix64 of (seed, counter).

``counter`` is the number of tokens the request has generated before this draw, so the
i-th output token of a request depends on (seed, i) alone: not on the batch, not on the
step it was drawn in, and not on whether the request was evicted and recomputed.
"""

_MASK = (1 << 64) - 1


def uniform_draw(seed: int, counter: int) -> float:
    """``u`` in [0, 1) with 24 random bits, exactly what ``sample_kernel`` computes."""
    z = ((seed & _MASK) + (counter + 1) * 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    z = z ^ (z >> 31)
    return (z >> 40) / 16777216.0


def derive_seed(engine_seed: int, request_number: int) -> int:
    """Seed of a request that names none: a hash of the engine's seed and its number."""
    z = ((engine_seed & _MASK) * 0xD1342543DE82EF95 + request_number * 0x9E3779B97F4A7C15 + 1) & _MASK
    z = ((z ^ (z >> 32)) * 0xDABA0B6EB09322E3) & _MASK
    return z ^ (z >> 32)
