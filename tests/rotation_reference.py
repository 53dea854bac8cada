"""A rotation of channel pairs written as a complex product, for the tests of rotations that the
architecture under test does not have (a part of a head, interleaved pairs)."""

import torch


def rotate_pairs(x, positions, rotary_dim, theta, pairing):
    """``x [tokens, heads, d]``: the pair ``(x1, x2)`` of channels is ``x1 + i x2``, multiplied by
    ``e^(i p inv_freq)``.  ``pairing == "half_split"`` pairs channel ``i`` with ``i + rotary_dim / 2``,
    ``"interleaved"`` channel ``2i`` with ``2i + 1``; channels beyond ``rotary_dim`` pass."""
    inv = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    angle = (positions.float()[:, None] * inv[None, :]).double()  # the angle is a float32 product
    unit = torch.polar(torch.ones_like(angle), angle)[:, None, :]
    out = x.double().clone()
    if pairing == "half_split":
        first, second = slice(0, rotary_dim // 2), slice(rotary_dim // 2, rotary_dim)
    elif pairing == "interleaved":
        first, second = slice(0, rotary_dim, 2), slice(1, rotary_dim, 2)
    else:
        raise ValueError(pairing)
    z = torch.complex(out[..., first], out[..., second]) * unit
    out[..., first], out[..., second] = z.real, z.imag
    return out.to(x.dtype)
