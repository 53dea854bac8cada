"""Device side of the cache: the page tensors of every layer, the block tables, the state slots.

What a layer's pages hold is the mixer's to say: it names its paged tensors, each with a
per-position shape and the place of the page's positions among its axes
(:class:`~rapid_llm_amd.parts.base.PagedSpec`), and finds them here by name.  Nothing in this
file knows of keys, values or heads.  The attention of this package asks for

* keys   ``k[page, kv_head, slot_in_page, head_dim]``: a key is one contiguous row;
* values ``v[page, kv_head, head_dim, slot_in_page]``: stored transposed, so the positions
  of a page are contiguous for one channel, which is how the ``P @ V`` product reads them,

so one page of one group costs ``2 * kv_heads * head_dim * page_size`` elements in each of its
layers of the group.  (The reference keeps token-granular rows ``[tokens, 2 * kv_heads,
head_dim]``, rapid_llm/executor/kv_cache_manager.py:230-249, and a latent row per token for
another mixer, rapid_llm/engine/kv_cache_spec.py:171-188.)
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
    # the mixer's paged tensors by the names it gave them, each
    # [pages, *shape[:slot_axis], page_size, *shape[slot_axis:]]
    pages: dict[str, torch.Tensor]
    owns_pages: bool  # False: reads another layer's pages and must not write them
    # fixed-size per-request tensors by name, each [max_seqs + 1, *shape], zeroed when a slot
    # is taken (the last row belongs to the filler slot of padded batches)
    states: dict[str, torch.Tensor]

    @property
    def k(self) -> torch.Tensor | None:
        """The paged tensor named ``"k"`` (keys ``[pages, kv_heads, page_size, head_dim]`` of the
        layout :meth:`CacheNeed.keys_and_values` asks for)."""
        return self.pages.get("k")

    @property
    def v(self) -> torch.Tensor | None:
        """The paged tensor named ``"v"`` (values ``[pages, kv_heads, head_dim, page_size]``)."""
        return self.pages.get("v")

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
        if need.kind != "paged" or need.share_with is not None:
            continue
        gid = keys.setdefault(need.window, len(keys))
        layers_of.setdefault(gid, []).append(i)
        group_of[i] = gid
    for i, need in enumerate(needs):
        if need.kind == "paged" and need.share_with is not None:
            src = need.share_with
            if not 0 <= src < len(needs) or needs[src].kind != "paged" or needs[src].share_with is not None:
                raise ValueError(f"layer {i} shares the cache of layer {src}, which owns none")
            if needs[src].paged != need.paged:
                raise ValueError(
                    f"layer {i} shares the cache of layer {src} but names other paged tensors: "
                    f"{need.paged} against {needs[src].paged}"
                )
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
    """Bytes one page id costs in each group: every paged tensor of every owning layer of the
    group (``elem``: bytes of an element of the engine's compute type)."""
    out: dict[int, int] = {}
    for need, gid in zip(needs, group_of):
        if gid is None or need.share_with is not None:
            continue
        for spec in need.paged:
            size = getattr(torch, spec.dtype).itemsize if spec.dtype else elem
            out[gid] = out.get(gid, 0) + spec.elements() * page_size * size
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
            paged: dict[str, torch.Tensor] = {}
            gid = group_of[i]
            owns = False
            if need.kind == "paged" and need.share_with is None:
                pages = manager.pools[gid].num_pages
                # zero-filled once.  Page 0, the null page, is written by rows that only pad a
                # batch (what they write lands in its first slot) and never read unmasked;
                # nothing is ever read from a page beyond what the masks allow
                paged = {
                    spec.name: torch.zeros(
                        spec.page_shape(pages, P),
                        dtype=getattr(torch, spec.dtype) if spec.dtype else dtype, device=device,
                    )
                    for spec in need.paged
                }
                owns = True
            states = {
                spec.name: torch.zeros(
                    (manager.max_seqs + 1, *spec.shape),
                    dtype=getattr(torch, spec.dtype) if spec.dtype else dtype, device=device,
                )
                for spec in need.state_specs()
            }
            self.layers.append(LayerCache(i, gid, P, paged, owns, states))
        for i, need in enumerate(needs):
            if need.kind == "paged" and need.share_with is not None:
                self.layers[i].pages = self.layers[need.share_with].pages
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
