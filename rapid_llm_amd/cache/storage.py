"""Device side of the cache: the page tensors of every layer, the block tables, the state slots.

Layout of one layer's pages (chosen for the attention kernels' matrix-core operands):

* keys   ``K[page, kv_head, slot_in_page, head_dim]``: a key is one contiguous row;
* values ``V[page, kv_head, head_dim, slot_in_page]``: stored transposed, so the positions
  of a page are contiguous for one channel, which is how the ``P @ V`` product reads them.

One page of one group therefore costs ``2 * kv_heads * head_dim * page_size`` elements in
each layer of the group.  (The reference keeps token-granular rows ``[tokens, 2 * kv_heads,
head_dim]``, rapid_llm/executor/kv_cache_manager.py:230-249.)
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from ..kernels.upload import upload, upload_ints
from ..parts.base import CacheNeed
from .manager import CacheManager, GroupSpec


@dataclass
class LayerCache:
    """What one mixer sees of the cache."""

    layer: int
    group_id: int | None  # None: the mixer has no paged cache
    page_size: int
    k: torch.Tensor | None  # [pages, kv_heads, page_size, head_dim]
    v: torch.Tensor | None  # [pages, kv_heads, head_dim, page_size]
    owns_pages: bool  # False: reads another layer's pages and must not write them
    # fixed-size per-request tensors by name, each [max_seqs + 1, *shape], zeroed when a slot
    # is taken (the last row belongs to the filler slot of padded batches)
    states: dict[str, torch.Tensor]

    @property
    def state(self) -> torch.Tensor | None:
        """The mixer's one state tensor (the one it asked for as ``state_shape``)."""
        return self.states.get("state")


def plan_groups(needs: list[CacheNeed]) -> tuple[list[GroupSpec], list[int | None]]:
    """Group layers by what they keep (all keys / a window of w).  Returns the groups and,
    per layer, its group id (``None`` for layers without paged cache).  A layer that shares
    another layer's cache joins that layer's group."""
    keys: dict[int, int] = {}  # window -> group id
    layers_of: dict[int, list[int]] = {}
    group_of: list[int | None] = [None] * len(needs)
    for i, need in enumerate(needs):
        if need.kind != "kv" or need.share_with is not None:
            continue
        gid = keys.setdefault(need.window, len(keys))
        layers_of.setdefault(gid, []).append(i)
        group_of[i] = gid
    for i, need in enumerate(needs):
        if need.kind == "kv" and need.share_with is not None:
            src = need.share_with
            if not 0 <= src < len(needs) or needs[src].kind != "kv" or needs[src].share_with is not None:
                raise ValueError(f"layer {i} shares the cache of layer {src}, which owns none")
            if needs[src].window != need.window:
                raise ValueError(
                    f"layer {i} (window {need.window}) shares the cache of layer {src} "
                    f"(window {needs[src].window}): a shared cache must keep the same positions"
                )
            group_of[i] = group_of[src]
            layers_of[group_of[i]].append(i)
    windows = {gid: w for w, gid in keys.items()}
    groups = [GroupSpec(gid, windows[gid], tuple(layers_of[gid])) for gid in sorted(windows)]
    return groups, group_of


def state_bytes(needs: list[CacheNeed], slots: int, elem: int) -> int:
    """Bytes the per-request state tensors of every layer take for ``slots`` slots."""
    total = 0
    for need in needs:
        for spec in need.state_specs():
            size = getattr(torch, spec.dtype).itemsize if spec.dtype else elem
            total += slots * int(np.prod(spec.shape, dtype=np.int64)) * size
    return total


def page_bytes(needs: list[CacheNeed], group_of: list[int | None], page_size: int, elem: int) -> dict[int, int]:
    """Bytes one page id costs in each group (summed over the group's owning layers)."""
    out: dict[int, int] = {}
    for need, gid in zip(needs, group_of):
        if gid is None or need.share_with is not None:
            continue
        out[gid] = out.get(gid, 0) + 2 * need.num_kv_heads * need.head_dim * page_size * elem
    return out


class DeviceCache:
    def __init__(
        self,
        manager: CacheManager,
        needs: list[CacheNeed],
        group_of: list[int | None],
        dtype: torch.dtype,
        device: torch.device,
    ) -> None:
        self.manager = manager
        self.device = device
        self.dtype = dtype
        P = manager.page_size
        self.layers: list[LayerCache] = []
        for i, need in enumerate(needs):
            k = v = None
            gid = group_of[i]
            owns = False
            if need.kind == "kv" and need.share_with is None:
                pages = manager.pools[gid].num_pages
                # zero-filled once.  Page 0, the null page, is written by rows that only pad a
                # batch (their keys and values land in its first slot) and never read unmasked;
                # nothing is ever read from a page beyond what the masks allow
                k = torch.zeros((pages, need.num_kv_heads, P, need.head_dim), dtype=dtype, device=device)
                v = torch.zeros((pages, need.num_kv_heads, need.head_dim, P), dtype=dtype, device=device)
                owns = True
            states = {
                spec.name: torch.zeros(
                    (manager.max_seqs + 1, *spec.shape),
                    dtype=getattr(torch, spec.dtype) if spec.dtype else dtype, device=device,
                )
                for spec in need.state_specs()
            }
            self.layers.append(LayerCache(i, gid, P, k, v, owns, states))
        for i, need in enumerate(needs):
            if need.kind == "kv" and need.share_with is not None:
                src = self.layers[need.share_with]
                self.layers[i].k, self.layers[i].v = src.k, src.v
        # One row more than there are slots: the filler slot, whose row maps every position to
        # the null page for good.  Rows that only pad a batch to a captured size name it (the
        # reference keeps its last table row for the same purpose,
        # rapid_llm/executor/slot_batch.py:97-100).
        self.filler_slot = manager.max_seqs
        self.tables: dict[int, torch.Tensor] = {
            gid: torch.zeros((tab.shape[0] + 1, tab.shape[1]), dtype=torch.int32, device=device)
            for gid, tab in manager.tables.items()
        }

    def refresh(self) -> None:
        """Bring the device block tables and state slots up to date with the manager: rows
        of slots whose pages changed are copied, state of newly taken slots is cleared.
        Everything is queued on the current stream; the host does not wait."""
        m = self.manager
        if m.dirty_slots:
            slots = sorted(m.dirty_slots)
            index = upload_ints(slots, self.device, np.int64)
            for gid, host in m.tables.items():
                self.tables[gid].index_copy_(0, index, upload(host[slots], self.device))
            m.dirty_slots.clear()
        if m.fresh_slots:
            index = None
            for layer in self.layers:
                for state in layer.states.values():
                    if index is None:
                        index = upload_ints(sorted(m.fresh_slots), self.device, np.int64)
                    state.index_fill_(0, index, 0)
            m.fresh_slots.clear()
