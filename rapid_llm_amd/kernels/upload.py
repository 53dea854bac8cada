"""Small host arrays to the device without waiting for the stream.

A copy from ordinary (pageable) host memory makes the host wait until the stream has run
everything queued before it, which would serialise a loop that plans the next step while
the device still runs this one.  Here the array is staged in a pinned buffer of a small
ring and copied asynchronously on the current stream; a buffer is taken again only after the
event recorded behind its last copy has completed.
"""

from __future__ import annotations

import numpy as np
import torch

_RING = 16  # staging buffers per device; a buffer is reused after this many uploads
_MIN_BYTES = 1 << 16


class _Ring:
    def __init__(self, device: torch.device) -> None:
        self.device = device
        self.buffers: list[torch.Tensor | None] = [None] * _RING
        self.events: list[torch.cuda.Event | None] = [None] * _RING
        self.at = 0

    def stage(self, nbytes: int) -> tuple[torch.Tensor, int]:
        i = self.at
        self.at = (i + 1) % _RING
        if self.events[i] is not None:
            self.events[i].synchronize()  # done long ago unless the ring is overrun
        buf = self.buffers[i]
        if buf is None or buf.numel() < nbytes:
            size = max(_MIN_BYTES, 1 << (nbytes - 1).bit_length())
            buf = torch.empty(size, dtype=torch.uint8, pin_memory=True)
            self.buffers[i] = buf
        return buf, i

    def sent(self, i: int) -> None:
        event = self.events[i]
        if event is None:
            event = self.events[i] = torch.cuda.Event()
        event.record()


_rings: dict[torch.device, _Ring] = {}


def _ring(device: torch.device) -> _Ring:
    device = torch.device(device)
    if device.index is None:
        device = torch.device(device.type, torch.cuda.current_device())
    ring = _rings.get(device)
    if ring is None:
        ring = _rings[device] = _Ring(device)
    return ring


def upload(host: np.ndarray, device: torch.device, into: torch.Tensor | None = None) -> torch.Tensor:
    """The array on the device, as a tensor of its dtype and shape (or copied into ``into``,
    which must have them), queued on the current stream; returns without waiting."""
    host = np.ascontiguousarray(host)
    dtype = torch.from_numpy(host[:0].reshape(-1)).dtype
    if into is None:
        into = torch.empty(host.shape, dtype=dtype, device=device)
    elif into.dtype != dtype or tuple(into.shape) != host.shape or not into.is_contiguous():
        raise ValueError(f"upload target {tuple(into.shape)} {into.dtype} does not fit {host.shape} {dtype}")
    nbytes = host.nbytes
    if nbytes == 0:
        return into
    ring = _ring(into.device)
    buf, i = ring.stage(nbytes)
    buf.numpy()[:nbytes] = host.reshape(-1).view(np.uint8)
    into.view(torch.uint8).reshape(-1).copy_(buf[:nbytes], non_blocking=True)
    ring.sent(i)
    return into


def upload_ints(values, device: torch.device, dtype=np.int32) -> torch.Tensor:
    return upload(np.asarray(values, dtype=dtype), device)
