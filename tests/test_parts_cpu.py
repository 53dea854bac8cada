"""What parts decide on the host, without a device."""

import torch

from rapid_llm_amd.parts.linear import Linear


def _bound(in_features, out_features, dtype):
    linear = Linear(in_features, out_features)
    linear.bind(torch.zeros(out_features, in_features, dtype=dtype))
    return linear


def test_a_product_takes_unscaled_rows_only_if_its_few_row_kernel_runs():
    """A norm leaves its factor to the product behind it only where that product's kernel can
    apply it: bfloat16 weights and a width the kernel's 16-byte reads divide.  A width of 70
    behind an output projection of width 96 once reached the library product with rows that
    nobody had scaled."""
    assert _bound(96, 70, torch.bfloat16).takes_scaled_rows()
    assert not _bound(70, 198, torch.bfloat16).takes_scaled_rows()
    assert not _bound(96, 70, torch.float32).takes_scaled_rows()  # a matrix the checkpoint stores in 32-bit
    assert not Linear(96, 70).takes_scaled_rows()  # nothing bound yet
