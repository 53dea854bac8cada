"""The one step function: a batch of (request, its next tokens) in, logits at the wanted places out.

A step is one forward pass over a flat, unpadded batch: portions of prompts of some
requests beside single decoded tokens of others, cut anywhere.  It runs only the tokens it
is given, reads everything earlier from the cache, writes this step's keys and values into
their pages, and returns float32 logits for the requested rows only.

The reference runs up to three forwards per scheduler step (a padded prefill grid, a
chunked/extend pass, a decode pass; rapid_llm/engine/scheduler.py:964-988) described by
``ModelInput`` spans (rapid_llm/executor/worker.py:69-126).  Here the span description is
kept (a request's tokens cover its cache positions ``[start, start + n)``) and the three
passes are one.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Mapping, Sequence

import numpy as np
import torch

from ..cache.manager import CacheError, CacheManager
from ..cache.storage import DeviceCache, page_bytes, plan_groups, state_bytes
from ..config.engine_config import EngineConfig
from ..config.model_config import read_config_json
from ..config.registry import config_from_dict
from ..kernels import ops
from ..kernels.upload import upload
from ..models.causal_lm import CausalLM
from ..parts.runtime import Runtime
from ..weights.loader import load_model_dir
from ..weights.random_init import random_params
from .feed import fed_token  # noqa: F401  (part of the step function's input convention)

_TORCH_DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32}
# batch sizes decode graphs are captured for; other sizes are padded up with filler rows
GRAPH_BATCHES = (1, 2, 4, 8, 12, 16, 24, 32, 48, 64, 96, 128, 192, 256)


class OutOfPages(CacheError):
    """A step needs more pages (or slots) than are free; nothing was taken."""


@dataclass
class StepEntry:
    """One request's share of a step: its next tokens and the places among them whose
    logits are wanted (indices into ``tokens``; may be empty).  A single token may be given
    as :func:`fed_token` ``(r)``: the token that row ``r`` of the latest sampling chose, which
    the host need not have seen yet."""

    request_id: str
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class StepContext:
    """Everything the parts may read about the batch of one step.  Device tensors are int32."""

    runtime: Runtime
    num_tokens: int
    num_seqs: int
    token_ids: torch.Tensor  # [T]
    positions: torch.Tensor  # [T] absolute position of each token in its request
    token_slot: torch.Tensor  # [T] slot (block-table row, state row) of each token's request
    seq_slots: torch.Tensor  # [n]
    seq_starts: torch.Tensor  # [n] tokens of the request already in the cache
    seq_lens: torch.Tensor  # [n] tokens of the request in this step
    cu_seqlens: torch.Tensor  # [n + 1] offsets of the requests' tokens in the flat batch
    logit_rows: torch.Tensor  # [R] flat token indices whose logits are wanted
    num_logit_rows: int
    block_tables: dict[int, torch.Tensor]  # group id -> [slots, pages per sequence]
    # host copies, for launch decisions (never read by kernels)
    h_seq_slots: list[int] = field(default_factory=list)
    h_seq_starts: list[int] = field(default_factory=list)
    h_seq_lens: list[int] = field(default_factory=list)
    max_position: int = 0
    max_seq_tokens: int = 0  # longest portion in the batch
    fed_tokens: torch.Tensor | None = None  # [rows] what the latest sampling chose (see fed_token)
    # Launch data of the parts' kernels, made on first use and shared by the layers of the step.
    # ``static`` holds what depends only on what a recorded step fixes (the number of rows, one
    # token a request, ``static["context_bound"]``, and in a recorded step
    # ``static["decode_only_tokens"]``): it is kept from the eager run before a recording into the
    # recording itself and lives as long as the graph.  ``extra`` holds anything else of one
    # forward pass and is emptied between the two.
    static: dict[Any, Any] = field(default_factory=dict)
    extra: dict[Any, Any] = field(default_factory=dict)


class ModelRunner:
    """Owns the model, its weights and the cache, and runs steps."""

    def __init__(
        self,
        model: str | Path | Mapping[str, Any],
        engine: EngineConfig | None = None,
        *,
        load_format: str = "auto",
        overrides: Mapping[str, Any] | None = None,
        device: str | torch.device = "cuda",
        weight_norm_std: float = 0.0,
    ) -> None:
        ops.require_gpu()
        self.engine = engine or EngineConfig()
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise ops.KernelError(f"the engine runs on a HIP device only, not on {self.device}")
        self.dtype = _TORCH_DTYPE[self.engine.dtype]

        if isinstance(model, Mapping):
            body, model_dir = dict(model), None
            if load_format == "auto":
                load_format = "random"
        else:
            model_dir = Path(model)
            body = read_config_json(model_dir)
        self.arch, self.config = config_from_dict(body, overrides)
        self.spec = self.arch.build_spec(self.config)
        if self.spec.max_position and self.engine.max_seq_len > self.spec.max_position:
            # rapid_llm/models/config.py:374-378
            raise ValueError(
                f"max_seq_len {self.engine.max_seq_len} exceeds the model's "
                f"max_position_embeddings {self.spec.max_position}"
            )
        self.runtime = Runtime(self.device, self.dtype, self.engine.max_seq_len, self.engine.page_size)
        self.model = CausalLM(self.spec)

        specs = self.model.param_specs()
        if load_format == "random":
            params = random_params(
                specs, self.engine.seed, engine_dtype=self.dtype, device=self.device,
                norm_std=weight_norm_std,
            )
        elif load_format == "auto":
            params = load_model_dir(
                model_dir, specs, engine_dtype=self.dtype, device=self.device,
                ignore_rules=self.spec.ignore_tensors,
            )
        else:
            raise ValueError(f"load_format must be 'auto' or 'random', got {load_format!r}")
        self.params = params
        self.model.bind(params, self.runtime)

        # ---- cache -------------------------------------------------------------
        needs = self.model.cache_needs()
        groups, group_of = plan_groups(needs)
        elem = 4 if self.dtype == torch.float32 else 2
        self.page_bytes = page_bytes(needs, group_of, self.engine.page_size, elem)
        self.state_bytes = state_bytes(needs, self.engine.max_num_seqs + 1, elem)
        num_pages = self._decide_num_pages(groups)
        self.cache = CacheManager(
            groups, num_pages, self.engine.page_size, self.engine.max_num_seqs, self.engine.max_seq_len
        )
        self.device_cache = DeviceCache(self.cache, needs, group_of, self.dtype, self.device)
        self.computed: dict[str, int] = {}
        self.vocab_size = self.spec.vocab_size
        self._graphs: dict[tuple[int, int], tuple] = {}
        # (rows, context bound) -> products of the library that the recorded step holds; a key
        # whose step is not replayed because of them (library_in_graph="eager") is listed too
        self.graph_library_products: dict[tuple[int, int], int] = {}
        # a part that does not promise to be replayable keeps every step eager
        self.graphs_allowed = self.model.replayable()
        # where the sampling kernels leave their choices, one row per sampled request of a
        # step; the next step's embedding reads fed tokens from here
        self.sampled = torch.zeros(max(1, self.engine.max_num_seqs), dtype=torch.int32, device=self.device)
        # the choices of the step before, kept aside while a step's sampling kernels overwrite
        # ``sampled``: a penalised row reads its own newest token from here
        self.sampled_before = torch.zeros_like(self.sampled)

    # ------------------------------------------------------------------ sizing
    def _decide_num_pages(self, groups) -> int:
        e = self.engine
        asked = e.num_pages
        if asked is None and e.max_gpu_num_blocks is not None:
            # the reference's knob counts tokens (README.md:121)
            asked = -(-e.max_gpu_num_blocks // e.page_size) + 1
        if asked is not None:
            # a pool of a given size is made as asked or not at all: say what does not fit
            # before the allocator fails somewhere in the middle of it
            per_page = sum(self.page_bytes.values())
            free, _ = torch.cuda.mem_get_info(self.device)
            if asked * per_page + self.state_bytes > free:
                raise ValueError(
                    f"a cache of {asked} pages of {e.page_size} tokens takes "
                    f"{(asked * per_page + self.state_bytes) >> 20} MiB ({per_page >> 10} KiB a page over the "
                    f"groups' layers) and {free >> 20} MiB are free beside the weights; ask for at most "
                    f"{max(0, free - self.state_bytes) // max(per_page, 1)} pages"
                )
            return asked
        # what is left of the device after the weights, times the utilisation, less what else the
        # engine will allocate (the per-request state tensors, the recorded steps' private
        # buffers, a step's activations), shared by the groups
        # (rapid_llm/executor/kv_cache_manager.py:91-130)
        free, total = torch.cuda.mem_get_info(self.device)
        reserve = self.state_bytes + self._graph_pool_estimate() + (1 << 30)
        budget = free - int(total * (1.0 - e.gpu_memory_utilization)) - reserve
        per_page = sum(self.page_bytes.values()) or 1
        if budget < 2 * per_page:
            raise ValueError(
                f"no memory is left for the cache: {free >> 20} MiB are free, gpu_memory_utilization "
                f"{e.gpu_memory_utilization} keeps {int(total * (1.0 - e.gpu_memory_utilization)) >> 20} MiB back, "
                f"state tensors, recorded steps and activations take {reserve >> 20} MiB, and a page costs "
                f"{per_page >> 10} KiB; lower max_num_seqs or max_seq_len, or give num_pages"
            )
        pages = budget // per_page
        # never more than every slot at full length can use
        cap = e.max_num_seqs * (-(-e.max_seq_len // e.page_size)) + 1
        return int(min(pages, cap))

    def _graph_pool_estimate(self) -> int:
        """Bytes the recorded decode steps may come to hold.  A batch is padded up to the next
        size of the ladder, so every size up to and including the first that holds
        ``max_num_seqs`` may be recorded, in every context bucket; each recording keeps its
        float32 logits, a few rows of activations and what its parts say they keep between
        their kernels (``Part.recorded_step_bytes``; a recording's pool reuses what one layer
        frees for the next, so the largest part counts, twice over)."""
        e = self.engine
        if not (e.use_graph and self.model.replayable()):
            return 0
        most = max(1, min(e.max_num_seqs, GRAPH_BATCHES[-1]))
        sizes = [b for b in GRAPH_BATCHES if b < most] + [next(b for b in GRAPH_BATCHES if b >= most)]
        bounds, bound = [], 512
        while True:
            bounds.append(min(bound, e.max_seq_len))
            if bound >= e.max_seq_len:
                break
            bound *= 2
        widest = max(
            [self.spec.hidden_size]
            + [p.shape[0] for p in self.params.values() if p.dim() == 2 and p.shape[0] != self.spec.vocab_size]
        )
        parts = list(self.model.all_parts())
        total = 0
        for rows in sizes:
            for bound in bounds:
                kept = max((p.recorded_step_bytes(rows, bound, e.page_size) for p in parts), default=0)
                total += rows * 4 * (self.spec.vocab_size + 8 * widest) + 2 * kept
        return total

    # ------------------------------------------------------------------ requests
    def tokens_cached(self, request_id: str) -> int:
        return self.computed.get(request_id, 0)

    def can_run(self, entries: Sequence[StepEntry]) -> bool:
        """Whether ``step(entries)`` would find the slots and pages it needs."""
        new = [e for e in entries if not self.cache.has(e.request_id)]
        if len(new) > self.cache.num_free_slots:
            return False
        need: dict[int, int] = {}
        ps = self.cache.page_size
        for e in entries:
            start = self.computed.get(e.request_id, 0)
            if self.cache.has(e.request_id):
                per = self.cache.pages_needed(e.request_id, start + len(e.tokens), start)
            else:
                per = {}
                for g in self.cache.groups:
                    per[g.group_id] = -(-(start + len(e.tokens)) // ps)
            for gid, n in per.items():
                need[gid] = need.get(gid, 0) + n
        return all(n <= self.cache.num_free_pages(gid) for gid, n in need.items())

    def finish(self, request_id: str) -> None:
        """The request is over: its pages and its slot are given back."""
        if self.cache.has(request_id):
            self.cache.release(request_id)
        self.computed.pop(request_id, None)

    # ------------------------------------------------------------------ the step
    def _prepare(self, entries: Sequence[StepEntry]) -> dict:
        """Check the entries, take the slots and pages they need (all or none), bring the device
        tables up to date; returns what the step knows about its batch on the host."""
        cache = self.cache
        seen = set()
        for e in entries:
            if e.request_id in seen:
                raise ValueError(f"request {e.request_id!r} appears twice in one step")
            seen.add(e.request_id)
            n = len(e.tokens)
            if n < 1:
                raise ValueError(f"request {e.request_id!r} brings no tokens")
            for w in e.want:
                if not 0 <= w < n:
                    raise ValueError(f"request {e.request_id!r} wants place {w} of {n} tokens")
            start = self.computed.get(e.request_id, 0)
            if start + n > self.engine.max_seq_len:
                raise ValueError(
                    f"request {e.request_id!r} would reach {start + n} tokens; max_seq_len is "
                    f"{self.engine.max_seq_len}"
                )
        # slots and pages: all requests of the step or none
        if not self.can_run(entries):
            raise OutOfPages(
                "the step does not fit: "
                f"{cache.num_free_slots} free slots, {cache.num_free_pages()} free pages"
            )
        for e in entries:
            if not cache.has(e.request_id):
                cache.admit(e.request_id)
            start = self.computed.get(e.request_id, 0)
            if not cache.reserve(e.request_id, start + len(e.tokens), start):
                raise CacheError("pages counted as free could not be taken")

        vocab = self.vocab_size
        lens = [len(e.tokens) for e in entries]
        starts = [self.computed.get(e.request_id, 0) for e in entries]
        slots = [cache.slot_of(e.request_id) for e in entries]
        for e in entries:
            lo, hi = min(e.tokens), max(e.tokens)
            if len(e.tokens) == 1 and -self.sampled.numel() <= lo < 0:
                continue  # a fed token: resolved on the device
            if lo < 0 or hi >= vocab:
                raise ValueError(
                    f"request {e.request_id!r} has a token id outside [0, {vocab}): min {lo}, max {hi}"
                )
        self.device_cache.refresh()
        return dict(
            num_tokens=sum(lens),
            num_seqs=len(entries),
            num_logit_rows=sum(len(e.want) for e in entries),
            h_seq_slots=slots,
            h_seq_starts=starts,
            h_seq_lens=lens,
            max_position=max(s + n for s, n in zip(starts, lens)) - 1,
            max_seq_tokens=max(lens),
        )

    @staticmethod
    def _pack(entries: Sequence[StepEntry], meta: dict):
        """One packed int32 upload: ids | positions | token_slot | slots | starts | lens | cu | rows."""
        n_seq, total, n_rows = meta["num_seqs"], meta["num_tokens"], meta["num_logit_rows"]
        lens, starts, slots = meta["h_seq_lens"], meta["h_seq_starts"], meta["h_seq_slots"]
        sizes = [total, total, total, n_seq, n_seq, n_seq, n_seq + 1, n_rows]
        offs = np.concatenate(([0], np.cumsum(sizes)))
        host = np.empty(int(offs[-1]), dtype=np.int32)
        cu = 0
        row = 0
        for i, e in enumerate(entries):
            n = lens[i]
            host[offs[0] + cu : offs[0] + cu + n] = e.tokens
            host[offs[1] + cu : offs[1] + cu + n] = np.arange(starts[i], starts[i] + n)
            host[offs[2] + cu : offs[2] + cu + n] = slots[i]
            for w in e.want:
                host[offs[7] + row] = cu + w
                row += 1
            host[offs[6] + i] = cu
            cu += n
        host[offs[6] + n_seq] = cu
        host[offs[3] : offs[4]] = slots
        host[offs[4] : offs[5]] = starts
        host[offs[5] : offs[6]] = lens
        return host, offs

    def _context(self, dev: torch.Tensor, offs, meta: dict) -> StepContext:
        part = [dev[offs[i] : offs[i + 1]] for i in range(len(offs) - 1)]
        return StepContext(
            runtime=self.runtime,
            token_ids=part[0],
            positions=part[1],
            token_slot=part[2],
            seq_slots=part[3],
            seq_starts=part[4],
            seq_lens=part[5],
            cu_seqlens=part[6],
            logit_rows=part[7],
            block_tables=self.device_cache.tables,
            fed_tokens=self.sampled,
            **meta,
        )

    # ------------------------------------------------------------------ decode graphs
    def _padded_decode(self, meta: dict, token_ids: list[int], rows: int):
        """The packed upload of a step of single tokens, padded to ``rows`` rows with filler
        rows: token 0 at position 0 of the filler slot, whose block-table row is the null page."""
        n = meta["num_seqs"]
        pad = rows - n
        filler = self.device_cache.filler_slot
        ids = np.asarray(token_ids + [0] * pad, dtype=np.int32)
        starts = np.asarray(meta["h_seq_starts"] + [0] * pad, dtype=np.int32)
        slots = np.asarray(meta["h_seq_slots"] + [filler] * pad, dtype=np.int32)
        ones = np.ones(rows, dtype=np.int32)
        arange = np.arange(rows + 1, dtype=np.int32)
        # ids | positions | token_slot | slots | starts | lens | cu | rows  (as _pack lays it out)
        host = np.concatenate([ids, starts, slots, slots, starts, ones, arange, arange[:rows]])
        sizes = [rows, rows, rows, rows, rows, rows, rows + 1, rows]
        offs = np.concatenate(([0], np.cumsum(sizes)))
        padded = dict(
            meta, num_tokens=rows, num_seqs=rows, num_logit_rows=rows,
            h_seq_slots=meta["h_seq_slots"] + [filler] * pad,
            h_seq_starts=meta["h_seq_starts"] + [0] * pad,
            h_seq_lens=[1] * rows,
        )
        return host, offs, padded

    def _graph_step(self, entries, meta) -> torch.Tensor | None:
        """A step of single tokens, all wanted: replayed from a HIP graph (``None``: this shape's
        step holds a product of the library and the engine is told to run such steps eagerly).  Graphs exist for a
        ladder of batch sizes and for context buckets (the next power of two); a batch is
        padded with filler rows to the next size of the ladder, so that a few captures serve
        every batch a scheduler produces.  The graph holds this package's kernels, and the
        library's products where a step has more rows than the package's own products take
        (``graph_library_products`` says how many); its inputs are one static int32 buffer,
        refreshed by a copy on the same stream before each replay.  Launch decisions that
        depend on the context length are made for the bucket's longest context."""
        batch = len(entries)
        rows = next(b for b in GRAPH_BATCHES if b >= batch)
        host, offs, meta = self._padded_decode(meta, [int(e.tokens[0]) for e in entries], rows)
        # the split of the keys over workgroups is fixed at capture and should fit the contexts
        # it serves
        bound = 512
        while bound <= meta["max_position"]:
            bound *= 2
        bound = min(bound, self.engine.max_seq_len)
        key = (rows, bound)
        entry = self._graphs.get(key)
        if entry is None and self.engine.library_in_graph == "eager" and self.graph_library_products.get(key):
            return None  # found out at the first try: this shape's step holds a library product
        if entry is None:
            # One eager run first, on a side stream: kernels get loaded, the allocator warm, and
            # the parts make the launch data they keep in ctx.static.  It runs filler rows only
            # (token 0 at position 0 of the filler slot): a mixer with state of its own must not
            # see a real request's step twice, and what the attention writes goes to the null page.
            blank, _, _ = self._padded_decode(dict(meta, num_seqs=0, h_seq_slots=[], h_seq_starts=[]), [], rows)
            static = torch.zeros(len(host), dtype=torch.int32, device=self.device)
            upload(blank, self.device, into=static)
            filler = [self.device_cache.filler_slot] * rows
            ctx = self._context(
                static, offs, dict(meta, max_position=bound - 1, h_seq_slots=filler, h_seq_starts=[0] * rows)
            )
            ctx.static["decode_only_tokens"] = torch.arange(rows, dtype=torch.int32, device=self.device)
            ctx.static["context_bound"] = bound
            library_before = ops.library_products
            current = torch.cuda.current_stream()
            side = torch.cuda.Stream()
            side.wait_stream(current)
            with torch.cuda.stream(side):
                self.model.forward(ctx, self.device_cache.layers)
            current.wait_stream(side)
            torch.cuda.synchronize()
            # what the parts left in ctx.static (launch data that depends on the step's shape
            # only) was uploaded by that run and is kept: nothing may be copied from the host
            # while the graph is recorded.  Everything else of that run is dropped.
            ctx.extra = {}
            # The eager run told which products of this shape go to the library.  Its kernels
            # are not this package's: some clear a workspace first, and which one runs depends
            # on the rows, the matrix and the library's version.
            library = ops.library_products
            if library != library_before and self.engine.library_in_graph != "record":
                self.graph_library_products[key] = library - library_before
                if self.engine.library_in_graph == "refuse":
                    raise ops.KernelError(
                        f"a decode step of {rows} rows would record {library - library_before} products of "
                        "the library into its graph (library_in_graph='refuse')"
                    )
                return None
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                logits = self.model.forward(ctx, self.device_cache.layers)
            self.graph_library_products[key] = ops.library_products - library
            # the graph's kernel nodes hold raw pointers: everything they point at that was
            # allocated outside the capture (the static inputs, what ctx.static holds) must
            # live as long as the graph does, so the context is kept with it
            entry = (graph, static, logits, ctx)
            self._graphs[key] = entry
        graph, static, logits, _ctx = entry
        upload(host, self.device, into=static)
        graph.replay()
        return logits[:batch]

    @torch.no_grad()
    def step(self, entries: Sequence[StepEntry], use_graph: bool | None = None) -> torch.Tensor:
        """Run one batch; returns float32 logits ``[wanted, vocab]`` in the order of the
        entries and of each entry's ``want``.  Raises :class:`OutOfPages`, with nothing
        changed, when slots or pages do not suffice.  The returned tensor may be reused by
        the next step: read it (sample from it, copy it) before stepping again.
        ``use_graph`` overrides the engine's setting for this one step."""
        if not entries:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        meta = self._prepare(entries)
        if (
            (self.engine.use_graph if use_graph is None else use_graph)
            and self.graphs_allowed
            and len(entries) <= GRAPH_BATCHES[-1]
            and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries)
        ):
            logits = self._graph_step(entries, meta)
        else:
            logits = None
        if logits is None:
            host, offs = self._pack(entries, meta)
            dev = upload(host, self.device)
            logits = self.model.forward(self._context(dev, offs, meta), self.device_cache.layers)
        for e in entries:
            done = self.computed.get(e.request_id, 0) + len(e.tokens)
            self.computed[e.request_id] = done
            self.cache.trim(e.request_id, done)  # pages a window has passed come back now
        return logits
