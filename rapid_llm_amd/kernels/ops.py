"""Call wrappers around the HIP kernels: host-side checks, then one launch on the current stream.

Nothing here computes: every function validates its operands (device, type, contiguity,
shape) and hands raw pointers to the compiled library.  There is no fallback; without a
GPU or without the compiled library these raise.
"""

from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

from . import build
from .upload import upload_ints

F32, BF16 = 0, 1
_TAG = {torch.float32: F32, torch.bfloat16: BF16}

_core: ctypes.CDLL | None = None
_attn: dict[int, ctypes.CDLL] = {}


class KernelError(RuntimeError):
    pass


class Chip:
    """What the launch rules know about the device: its number of compute units, read once on
    the host (the kernels that decide by it are handed the same number), and what follows
    from it.  Without a device the rules are asked about the chip they were measured on."""

    def __init__(self, units: int) -> None:
        if units < 1:
            raise KernelError(f"a chip has at least one compute unit, got {units}")
        self.units = units
        self.first_round = units  # workgroups that start first, one on each compute unit
        self.decode_resident = 3 * units  # decode-attention workgroups the chip holds at a time
        self.prefill_slots = 2 * units  # wave groups of four the prefill kernel keeps at a time


MEASURED_CHIP = Chip(256)  # MI355X
_chips: dict[int, Chip] = {}


def chip() -> Chip:
    """The current device's geometry (the measured chip's where no device is visible)."""
    if not torch.cuda.is_available():
        return MEASURED_CHIP
    dev = torch.cuda.current_device()
    found = _chips.get(dev)
    if found is None:
        found = _chips[dev] = Chip(torch.cuda.get_device_properties(dev).multi_processor_count)
    return found


def require_gpu() -> None:
    if not torch.cuda.is_available():
        raise KernelError(
            "rapid_llm_amd runs its model on a HIP device only (no CPU implementation exists) "
            "and no GPU is visible to this process"
        )


def core() -> ctypes.CDLL:
    global _core
    if _core is None:
        _core = build.load(build.core_library())
    return _core


def attention_lib(head_dim: int) -> ctypes.CDLL:
    lib = _attn.get(head_dim)
    if lib is None:
        lib = build.load(build.attention_library(head_dim))
        if lib.rl_attn_head_dim() != head_dim:
            raise KernelError(f"attention library for head size {head_dim} reports {lib.rl_attn_head_dim()}")
        _attn[head_dim] = lib
    return lib


def _stream() -> ctypes.c_void_p:
    # the raw handle of the current stream of the current device, without the stream object
    # that ``torch.cuda.current_stream()`` builds (2.8 against 0.2 us a call, on every launch)
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def _p(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _tag(dtype: torch.dtype) -> int:
    try:
        return _TAG[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16 tensors, got {dtype}") from None


def _need(t: torch.Tensor, name: str, dtype: torch.dtype | None = None, shape=None) -> None:
    if not t.is_cuda:
        raise KernelError(f"{name} must live on the GPU, is on {t.device}")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous (shape {tuple(t.shape)}, strides {t.stride()})")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, is {t.dtype}")
    if shape is not None:
        have = t.shape
        if len(shape) != len(have):
            raise KernelError(f"{name} must have shape {tuple(shape)}, has {tuple(have)}")
        for want, size in zip(shape, have):
            if want is not None and want != size:
                raise KernelError(f"{name} must have shape {tuple(shape)}, has {tuple(have)}")


def _ok(code: int, what: str) -> None:
    if code != 0:
        reason = {1: "an argument the kernel refuses", 2: "the launch failed"}.get(code, "unknown")
        raise KernelError(f"{what}: error {code} ({reason})")


# --------------------------------------------------------------------------- #


def embed(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, fed: Optional[torch.Tensor] = None) -> None:
    """``out[t] = table[ids[t]]``; an id ``-(r + 1)`` takes ``fed[r]``, the token a sampling
    kernel chose in row ``r`` of the previous step."""
    tokens = ids.numel()
    vocab, hidden = table.shape
    _need(ids, "ids", torch.int32)
    _need(table, "embedding table")
    _need(out, "out", torch.float32, (tokens, hidden))
    if fed is not None:
        _need(fed, "fed", torch.int32)
    _ok(
        core().rl_embed(
            _p(ids), _p(fed), 0 if fed is None else fed.numel(), _p(table), _tag(table.dtype), _p(out),
            tokens, hidden, vocab, _stream(),
        ),
        "rl_embed",
    )


def read_buffer(buf: torch.Tensor, blocks: int = 4096) -> None:
    """Stream a buffer through the compute units once (a measurement of read bandwidth)."""
    if not buf.is_cuda or not buf.is_contiguous():
        raise KernelError("read_buffer takes a contiguous GPU tensor")
    sink = torch.zeros(1, dtype=torch.int32, device=buf.device)
    _ok(
        core().rl_read_buffer(_p(buf), ctypes.c_size_t(buf.numel() * buf.element_size()), _p(sink), blocks, _stream()),
        "rl_read_buffer",
    )


def add_rmsnorm(
    residual: torch.Tensor,
    delta: Optional[torch.Tensor],
    weight: torch.Tensor,
    out: torch.Tensor,
    eps: float,
    rows: Optional[torch.Tensor] = None,
) -> None:
    tokens, hidden = residual.shape
    _need(residual, "residual", torch.float32)
    _need(weight, "norm weight", torch.float32, (hidden,))
    out_rows = tokens if rows is None else rows.numel()
    _need(out, "out", None, (out_rows, hidden))
    if delta is not None:
        _need(delta, "delta", out.dtype, (tokens, hidden))
    if rows is not None:
        _need(rows, "rows", torch.int32)
    _ok(
        core().rl_add_rmsnorm(
            _p(residual), _p(delta), _p(weight), _p(out), _p(rows), out_rows, hidden,
            ctypes.c_float(eps), _tag(out.dtype), _stream(),
        ),
        "rl_add_rmsnorm",
    )


def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    tokens, two_i = gate_up.shape
    if two_i % 2:
        raise KernelError(f"the packed [gate | up] row must have even width, has {two_i}")
    _need(gate_up, "gate_up")
    _need(out, "out", gate_up.dtype, (tokens, two_i // 2))
    _ok(
        core().rl_swiglu(_p(gate_up), _p(out), tokens, two_i // 2, _tag(out.dtype), _stream()),
        "rl_swiglu",
    )


def cast(src: torch.Tensor, dst: torch.Tensor) -> None:
    _need(src, "src")
    _need(dst, "dst")
    if src.numel() != dst.numel():
        raise KernelError(f"cast of {src.numel()} elements into {dst.numel()}")
    _ok(
        core().rl_cast(
            _p(src), _tag(src.dtype), _p(dst), _tag(dst.dtype), ctypes.c_size_t(src.numel()), _stream()
        ),
        "rl_cast",
    )


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> None:
    """``y[r, :] += bias`` in place (``bias`` float32)."""
    rows, cols = y.shape
    _need(y, "y")
    _need(bias, "bias", torch.float32, (cols,))
    _ok(core().rl_add_bias(_p(y), _p(bias), rows, cols, _tag(y.dtype), _stream()), "rl_add_bias")


def rope_table(inv_freq: torch.Tensor, positions: int) -> tuple[torch.Tensor, torch.Tensor]:
    _need(inv_freq, "inv_freq", torch.float32)
    half = inv_freq.numel()
    cos = torch.empty((positions, half), dtype=torch.float32, device=inv_freq.device)
    sin = torch.empty_like(cos)
    _ok(core().rl_rope_table(_p(inv_freq), _p(cos), _p(sin), positions, half, _stream()), "rl_rope_table")
    return cos, sin


# which channels of a head form a rotated pair, as the kernels number them: channel i with
# i + (rotated channels) / 2, or channel 2i with 2i + 1
ROTARY_PAIRINGS = {"half_split": 0, "interleaved": 1}


def qknorm_rope_kvwrite(
    qkv: torch.Tensor,
    q_out: Optional[torch.Tensor],
    k_cache: Optional[torch.Tensor],
    v_cache: Optional[torch.Tensor],
    q_norm_w: Optional[torch.Tensor],
    k_norm_w: Optional[torch.Tensor],
    cos: Optional[torch.Tensor],
    sin: Optional[torch.Tensor],
    positions: torch.Tensor,
    token_slot: torch.Tensor,
    block_table: torch.Tensor,
    page_size: int,
    nq: int,
    nkv: int,
    d: int,
    eps: float,
    max_position: int,
    pairing: str = "half_split",
) -> None:
    """Norm + rotate q and k, write k and v to the cache pages (skipped when the caches
    are ``None``: a layer that reads another layer's cache).  ``q_out`` ``None``: the query
    heads are left as they are (the attention kernels finish them themselves, see
    :func:`attention_prepares_queries`).  ``max_position`` is the
    largest position in the batch, checked against the rotation table and block table.
    The tables' width says how many channels rotate (``2 * cos.shape[1]``, the first of a
    head), ``pairing`` which of them form a pair (:data:`ROTARY_PAIRINGS`)."""
    if pairing not in ROTARY_PAIRINGS:
        raise KernelError(f"rotation pairing {pairing!r} is not one of {sorted(ROTARY_PAIRINGS)}")
    tokens = qkv.shape[0]
    _need(qkv, "qkv", None, (tokens, (nq + 2 * nkv) * d))
    if q_out is not None:
        _need(q_out, "q_out", qkv.dtype, (tokens, nq * d))
    _need(positions, "positions", torch.int32, (tokens,))
    _need(token_slot, "token_slot", torch.int32, (tokens,))
    _need(block_table, "block_table", torch.int32)
    write = k_cache is not None
    if write:
        pages = k_cache.shape[0]
        _need(k_cache, "k_cache", qkv.dtype, (pages, nkv, page_size, d))
        _need(v_cache, "v_cache", qkv.dtype, (pages, nkv, d, page_size))
        if max_position // page_size >= block_table.shape[1]:
            raise KernelError(
                f"position {max_position} needs page {max_position // page_size} of a block "
                f"table with {block_table.shape[1]} columns"
            )
    for w, name in ((q_norm_w, "q_norm weight"), (k_norm_w, "k_norm weight")):
        if w is not None:
            _need(w, name, torch.float32, (d,))
    half = 0
    if cos is not None:
        half = cos.shape[1]
        _need(cos, "cos table", torch.float32, (None, half))
        _need(sin, "sin table", torch.float32, tuple(cos.shape))
        if not 1 <= half <= d // 2:
            raise KernelError(f"rotation tables of {half} pairs do not fit a head of {d} channels")
        if max_position >= cos.shape[0]:
            raise KernelError(
                f"position {max_position} is beyond the rotation table of {cos.shape[0]} positions"
            )
    _ok(
        core().rl_qknorm_rope_kvwrite(
            _p(qkv), _p(q_out), _p(k_cache), _p(v_cache), _p(q_norm_w), _p(k_norm_w), _p(cos),
            _p(sin), _p(positions), _p(token_slot), _p(block_table), block_table.stride(0),
            page_size, tokens, nq, nkv, d, half, ROTARY_PAIRINGS[pairing], ctypes.c_float(eps), int(write),
            _tag(qkv.dtype), _stream(),
        ),
        "rl_qknorm_rope_kvwrite",
    )


def attention_generic(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    out: torch.Tensor,
    positions: torch.Tensor,
    token_slot: torch.Tensor,
    block_table: torch.Tensor,
    page_size: int,
    nq: int,
    nkv: int,
    d: int,
    window: int,
    scale: float,
    max_position: int,
) -> None:
    tokens = q.shape[0]
    pages = k_cache.shape[0]
    _need(q, "q", None, (tokens, nq * d))
    _need(out, "out", q.dtype, (tokens, nq * d))
    _need(k_cache, "k_cache", q.dtype, (pages, nkv, page_size, d))
    _need(v_cache, "v_cache", q.dtype, (pages, nkv, d, page_size))
    _need(positions, "positions", torch.int32, (tokens,))
    _need(token_slot, "token_slot", torch.int32, (tokens,))
    _need(block_table, "block_table", torch.int32)
    if max_position // page_size >= block_table.shape[1]:
        raise KernelError(
            f"position {max_position} needs page {max_position // page_size} of a block table "
            f"with {block_table.shape[1]} columns"
        )
    _ok(
        core().rl_attention_generic(
            _p(q), _p(k_cache), _p(v_cache), _p(out), _p(positions), _p(token_slot),
            _p(block_table), block_table.stride(0), page_size, tokens, nq, nkv, d, window,
            ctypes.c_float(scale), _tag(q.dtype), _stream(),
        ),
        "rl_attention_generic",
    )


def gemm_f32(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> None:
    """``out[M,N] = a[M,K] @ w[N,K]^T`` in true float32.  Rows may be strided (views of wider
    matrices); the inner dimension must be contiguous."""
    for t, name in ((a, "a"), (w, "w"), (out, "out")):
        if not t.is_cuda or t.dtype != torch.float32 or t.dim() != 2 or t.stride(1) != 1:
            raise KernelError(f"gemm_f32 operand {name} must be a float32 GPU matrix with unit inner stride")
    m, k = a.shape
    n, k2 = w.shape
    if k != k2 or out.shape != (m, n):
        raise KernelError(f"gemm_f32 shapes do not agree: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    _ok(
        core().rl_gemm_f32(_p(a), _p(w), _p(out), m, n, k, a.stride(0), w.stride(0), out.stride(0), _stream()),
        "rl_gemm_f32",
    )


def _row_index(row_index: Optional[torch.Tensor]) -> None:
    if row_index is not None:
        _need(row_index, "row_index", torch.int32)
        if row_index.dim() != 1:
            raise KernelError(f"row_index must have one dimension, got {tuple(row_index.shape)}")


def argmax(logits: torch.Tensor, out: torch.Tensor, row_index: Optional[torch.Tensor] = None) -> None:
    """``out[b]`` = arg-max of row ``row_index[b]`` of ``logits`` (row ``b`` without an index)."""
    vocab = logits.shape[1]
    rows = out.shape[0]
    _need(logits, "logits", torch.float32)
    _need(out, "out", torch.int32, (rows,))
    _row_index(row_index)
    if row_index is not None and row_index.shape[0] != rows:
        raise KernelError(f"{row_index.shape[0]} row indices for {rows} outputs")
    if row_index is None and logits.shape[0] != rows:
        raise KernelError(f"{logits.shape[0]} rows of logits for {rows} outputs")
    lib = core()
    slices = lib.rl_argmax_slices(vocab)
    part_v = part_i = None
    if slices > 1 and rows * 4 < slices * 16:  # few wide rows: two stages fill the chip
        part_v = torch.empty((rows, slices), dtype=torch.float32, device=logits.device)
        part_i = torch.empty((rows, slices), dtype=torch.int32, device=logits.device)
    _ok(
        lib.rl_argmax(_p(logits), _p(row_index), _p(out), _p(part_v), _p(part_i), rows, vocab, _stream()),
        "rl_argmax",
    )


_PENALTY_MAX_VOCAB = 40 * 1024 * 8  # one bit per token id in 40 KB of LDS


def _penalty_fits(vocab: int) -> None:
    if vocab > _PENALTY_MAX_VOCAB:
        raise KernelError(
            f"the repetition penalty keeps one bit per token id in 40 KB of LDS: vocabulary "
            f"{vocab} is beyond {_PENALTY_MAX_VOCAB}"
        )


def _fed_tokens(fed: Optional[torch.Tensor], out: Optional[torch.Tensor]) -> None:
    if fed is None:
        return
    _need(fed, "fed", torch.int32)
    if fed.dim() != 1:
        raise KernelError(f"fed tokens must be one-dimensional, are {tuple(fed.shape)}")
    if out is not None and _overlap(fed, out):
        raise KernelError("the fed tokens share memory with the tokens this call chooses")


def _overlap(a: torch.Tensor, b: torch.Tensor) -> bool:
    a0, b0 = a.data_ptr(), b.data_ptr()
    return a0 < b0 + b.numel() * b.element_size() and b0 < a0 + a.numel() * a.element_size()


def sample(
    logits: torch.Tensor,
    row_params: torch.Tensor,
    history: Optional[torch.Tensor],
    out: torch.Tensor,
    out_logprob: Optional[torch.Tensor],
    any_penalty: bool,
    row_index: Optional[torch.Tensor] = None,
    fed: Optional[torch.Tensor] = None,
) -> None:
    """General token selection (penalty, temperature, nucleus, seeded draw), one row per
    workgroup.  ``row_params [rows * 8]`` int32 as the kernel documents them; output row
    ``b`` reads row ``row_index[b]`` of ``logits`` (row ``b`` without an index).  A negative
    entry ``-(r + 1)`` of ``history`` is read as ``fed[r]``; ``fed`` must not share memory
    with ``out``."""
    vocab = logits.shape[1]
    rows = out.shape[0]
    _need(logits, "logits", torch.float32)
    _need(row_params, "row_params", torch.int32, (rows * 8,))
    _need(out, "out", torch.int32, (rows,))
    _row_index(row_index)
    if (row_index.shape[0] if row_index is not None else logits.shape[0]) != rows:
        raise KernelError(f"{rows} outputs do not match the rows to read")
    if out_logprob is not None:
        _need(out_logprob, "out_logprob", torch.float32, (rows,))
    if history is not None:
        _need(history, "history", torch.int32)
    if any_penalty:
        _penalty_fits(vocab)
    _fed_tokens(fed, out)
    _ok(
        core().rl_sample(
            _p(logits), _p(row_index), _p(row_params), _p(history), _p(fed),
            0 if fed is None else fed.shape[0], _p(out), _p(out_logprob), rows, vocab,
            int(bool(any_penalty)), _stream(),
        ),
        "rl_sample",
    )


def logprobs(
    logits: torch.Tensor,
    targets: torch.Tensor,
    k: int,
    row_params: Optional[torch.Tensor] = None,
    history: Optional[torch.Tensor] = None,
    any_penalty: bool = False,
    row_index: Optional[torch.Tensor] = None,
    fed: Optional[torch.Tensor] = None,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Log-probability of ``targets[b]`` and the ``k`` most likely tokens of every row:
    ``(target [rows] float32, top ids [rows, k] int32, top log-probabilities [rows, k]
    float32)``, descending, equal values by ascending id.  With ``row_params`` the
    distribution is the one ``sample`` draws from (penalty, temperature; greedy rows count
    as temperature 1); without, log_softmax of the raw logits.  ``fed`` as for ``sample``."""
    vocab = logits.shape[1]
    rows = targets.shape[0]
    _need(logits, "logits", torch.float32)
    _need(targets, "targets", torch.int32, (rows,))
    _row_index(row_index)
    if (row_index.shape[0] if row_index is not None else logits.shape[0]) != rows:
        raise KernelError(f"{rows} targets do not match the rows to read")
    if not 0 <= k <= vocab:
        raise KernelError(f"top-k width {k} is outside [0, vocabulary {vocab}]")
    if row_params is not None:
        _need(row_params, "row_params", torch.int32, (rows * 8,))
    if history is not None:
        _need(history, "history", torch.int32)
    if any_penalty:
        _penalty_fits(vocab)
        if row_params is None or history is None:
            raise KernelError("a penalty needs row_params and history")
    _fed_tokens(fed, None)
    target_lp = torch.empty(rows, dtype=torch.float32, device=logits.device)
    top_ids = torch.empty((rows, k), dtype=torch.int32, device=logits.device)
    top_lp = torch.empty((rows, k), dtype=torch.float32, device=logits.device)
    _ok(
        core().rl_logprobs(
            _p(logits), _p(row_index), _p(row_params), _p(history), _p(fed),
            0 if fed is None else fed.shape[0], _p(targets), _p(target_lp),
            _p(top_ids if k else None), _p(top_lp if k else None), rows, vocab, k,
            int(bool(any_penalty)), _stream(),
        ),
        "rl_logprobs",
    )
    return target_lp, top_ids, top_lp


def sample_uniform(seed: int, counter: int) -> float:
    """The kernel's own uniform draw, computed by the library on the host."""
    fn = core().rl_sample_uniform
    fn.restype = ctypes.c_float
    return float(fn(ctypes.c_uint(seed & 0xFFFFFFFF), ctypes.c_uint((seed >> 32) & 0xFFFFFFFF), ctypes.c_uint(counter)))


SKINNY_MAX_ROWS = 16  # rows up to which the hand-written bandwidth-bound product is used
def _skinny_tiles(rows: int, out_features: int, plain: bool = False, units: int | None = None) -> int:
    """Weight rows per workgroup of the skinny product, as the kernel's code for them: 1 (16 rows,
    one tile, which leaves the most workgroups), 2 (32 rows) or, for a product that only stores
    its result (``plain``), 3 (24 rows: one tile and a half).

    A compute unit streams at most so fast, so what counts is the most rows a unit gets: the
    rounds of workgroups times their rows.  A matrix of 257 to 1,023 tiles takes 24 rows where
    that gives the fewest (6,144 outputs = 384 tiles: 256 workgroups, one a unit; microseconds at
    1 / 8 / 16 rows of X with 16, 32 and 24 weight rows a workgroup: 11.6 12.3 11.0 / 13.9 12.8
    11.1 / 16.6 14.1 12.0; 5,120 outputs 11.4 11.2 9.8 / 13.1 12.1 10.3 / 16.2 13.7 11.6; but
    7,168 outputs = 448 tiles, where 24 rows make 299 workgroups and a second round, 14.9 15.0
    18.6 / 17.8 15.6 20.4).  Otherwise one tile, except where two were measured faster: from 8
    rows of X on when one tile would leave some units with two workgroups and some with one; and
    with more than 12 rows on matrices of a thousand tiles and more (151,936 outputs: 275 / 244
    at 16 rows, but 216 / 233 at 8)."""
    units = chip().units if units is None else units
    blocks = -(-out_features // 16)
    if plain and units < blocks < 4 * units:
        def most_rows(rows_per_group: int) -> int:
            groups = -(-out_features // rows_per_group)
            return -(-groups // units) * rows_per_group
        if most_rows(24) < min(most_rows(16), most_rows(32)):
            return 3
    if rows >= 8 and units < blocks < 2 * units:
        return 2
    if rows > 12 and blocks >= 4 * units:
        return 2
    return 1


def _scaled_args(scaled, rows: int, k: int) -> tuple:
    """The kernels' arguments for an X whose norm factor is still to be applied."""
    if scaled is None:
        return (None, 0, 0, ctypes.c_float(0.0))
    _need(scaled.partial, "partial sums of squares", torch.float32)
    if scaled.partial.dim() != 2 or scaled.partial.shape[1] != 16 or scaled.size != k or rows > 16:
        raise KernelError(
            f"scaled rows of width {scaled.size} with partials {tuple(scaled.partial.shape)} do not fit "
            f"a product of {rows} rows over {k}"
        )
    return (_p(scaled.partial), scaled.partial.shape[0], scaled.size, ctypes.c_float(scaled.eps))


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, scaled=None) -> torch.Tensor:
    """``x[M,K] @ w[N,K]^T`` with bfloat16 operands and float32 accumulation.  ``scaled``
    (few rows only): the rows of ``x`` still lack their norm's factor, which is applied to
    the result (see ``gemm_bf16_residual``).

    Up to 16 rows (decode) run the hand-written bandwidth-bound kernel, which can write
    float32 directly; so does the kernel for 17 to 64 rows over wide matrices.  Small matrices
    run the one-launch tile product up to 512 rows.  Everything else goes to the library
    product, as the reference's dense products do (``F.linear``); a bfloat16 result is returned
    as is and widened by the caller."""
    _need(x, "x", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    m, k = x.shape
    n = w.shape[0]
    if k != w.shape[1]:
        raise KernelError(f"gemm_bf16 shapes do not agree: x {tuple(x.shape)}, w {tuple(w.shape)}")
    if m <= SKINNY_MAX_ROWS and k % 8 == 0:
        if out_dtype not in (torch.bfloat16, torch.float32):
            raise KernelError(f"gemm_bf16 writes bfloat16 or float32, not {out_dtype}")
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
        nt = _skinny_tiles(m, n, plain=True)
        _ok(
            core().rl_gemm_skinny(
                _p(x), _p(w), _p(out), m, n, k, k, k, n, _tag(out_dtype), nt, *_scaled_args(scaled, m, k), _stream()
            ),
            "rl_gemm_skinny",
        )
        return out
    if scaled is not None:
        raise KernelError(f"scaled rows need the few-row product: {m} rows over {k}")
    if _tile_applies(m, n, k, n):
        out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
        _ok(core().rl_gemm_tile(_p(x), _p(w), _p(out), m, n, k, k, k, n, 0, _stream()), "rl_gemm_tile")
        return out
    plan = rows_plan(m, n, k, swiglu=False)
    if plan is not None:
        wide = torch.float32 if out_dtype == torch.float32 else torch.bfloat16
        out = torch.empty((m, n), dtype=wide, device=x.device)
        _ok(
            core().rl_gemm_rows(_p(x), _p(w), _p(out), m, n, k, k, k, n, 0, _tag(wide), *plan, _stream()),
            "rl_gemm_rows",
        )
        return out
    return library_product(x, w)


# How many products went to the library since the process started.  A step that is recorded into
# a graph is meant to hold this package's kernels only where they exist; whoever records one
# reads the counter before and after.
library_products = 0


def library_product(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``x w^T`` by the library (hipBLASLt behind ``torch.matmul``), as the reference's dense
    products are ``F.linear``: the many-row products of prompt steps, and what no kernel of
    this package takes."""
    global library_products
    library_products += 1
    return torch.matmul(x, w.t())


ROWS_MAX_ROWS = 64  # rows up to which wide matrices run the kernel that keeps X in registers


def rows_plan(m: int, n: int, k: int, swiglu: bool, units: int | None = None) -> tuple[int, int] | None:
    """(result tiles a workgroup holds, workgroups) for the product of 17 to 64 rows over a wide
    matrix with ``n`` result columns (with SwiGLU a tile is a gate and an up tile), ``None`` where
    that kernel does not apply.  A compute unit gets one workgroup with an even share of the
    tiles where a workgroup can hold such a share (the packed gate and up matrices of Qwen3-8B:
    768 pairs, three a unit); a matrix with more tiles than that (the vocabulary) is cut into
    workgroups of the most tiles one holds, which the chip takes in turn."""
    if not (SKINNY_MAX_ROWS < m <= ROWS_MAX_ROWS) or n % 16 or k % 128 or k < 128:
        return None
    if os.environ.get("RAPID_LLM_ROWS_PRODUCT") == "0":  # the library instead, for comparing the two
        return None
    units = chip().units if units is None else units
    tiles = n // 16
    if 2 * tiles < units:  # too few workgroups to stream from
        return None
    holds = ((2, 3, 5) if m <= 48 else (2, 3)) if swiglu else (1, 2, 3, 6)
    share = -(-tiles // min(units, tiles))
    for per in holds:
        if per >= share:
            return per, min(units, tiles)
    if (swiglu and share > 5) or (not swiglu and share < 24):
        # More tiles a compute unit than a workgroup holds (beyond 48 rows a workgroup holds
        # three pairs, and a matrix of up to five pairs a unit is cut into groups of three).  For the packed gate and up matrices
        # of the 32B shape (524 MB, 12.5 tiles a unit) the library's kernel streams at 5.4 TB/s
        # at every row count: 97 to 106 us at 17 to 64 rows against 99 to 136 here in any cut with
        # SwiGLU, 91 against 116 at 32 rows without.  Only for the vocabulary (37 tiles a unit)
        # are its kernels the slower ones (348 us against 294 at 32 rows of the 32B shape).
        return None
    per = holds[-1]
    return per, -(-tiles // per)


def gemm_bf16_residual(
    x: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, norm_weight: torch.Tensor
) -> tuple[torch.Tensor, torch.Tensor]:
    """The few-row product with the residual epilogue: ``residual += x w^T`` (the product
    rounded to bfloat16 first, as a stored result would be) in place; returns
    ``(residual * norm_weight`` as bfloat16, ``partial [workgroups, 16]`` float32``)`` with the
    sums of squares of each workgroup's columns of every row.  A consumer that takes the rows
    as ``scaled`` input finishes the norm."""
    _need(x, "x", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    m, k = x.shape
    n = w.shape[0]
    if k != w.shape[1] or m > SKINNY_MAX_ROWS or k % 8:
        raise KernelError(
            f"gemm_bf16_residual takes up to {SKINNY_MAX_ROWS} rows over a multiple of 8: "
            f"x {tuple(x.shape)}, w {tuple(w.shape)}"
        )
    _need(residual, "residual", torch.float32, (m, n))
    _need(norm_weight, "norm weight", torch.float32, (n,))
    lib = core()
    nt = _skinny_tiles(m, n)
    rows = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    partial = torch.empty((lib.rl_gemm_skinny_parts(n, nt), 16), dtype=torch.float32, device=x.device)
    _ok(
        lib.rl_gemm_skinny_residual(
            _p(x), _p(w), m, n, k, k, k, nt, _p(residual), _p(norm_weight), _p(rows), _p(partial), _stream()
        ),
        "rl_gemm_skinny_residual",
    )
    return rows, partial


TILE_MAX_ROWS = 512  # rows up to which small matrices run the one-launch tile product
_TILE_MAX_WEIGHTS = 7 << 20  # elements of a matrix (14 MB) up to which it is used
_TILE_MIN_COLS = 2048  # fewer columns leave too few workgroups


def _tile_applies(m: int, weight_rows: int, k: int, cols: int) -> bool:
    """Whether the one-launch tile product takes ``m`` rows over a ``[weight_rows, k]`` matrix
    with ``cols`` result columns.  It is for steps of tens to hundreds of rows over matrices of
    a few megabytes, where a kernel's time is its start and its chain of dependent steps, not
    its bytes.  Measured against the library, microseconds at 17 / 64 / 256 rows (the library
    first): 4,096 x 1,024 8.2 / 5.9, 8.7 / 7.8, 9.0 / 8.3; the packed gate and up matrices of
    6,144 x 1,024 with SwiGLU in the epilogue against the library and the activation kernel
    13.4 / 8.2, 13.5 / 10.9, 17.9 / 14.8 (inside a Qwen3-0.6B decode step the library's two
    take 11.5 and 13.8 + 4.6).  From 4,096 x 2,048 on the library is as fast or faster (11.1 /
    11.3, 11.6 / 14.4, 13.1 / 13.8), and matrices of 1,024 rows leave too few workgroups
    (1,024 x 2,048: 8.2 / 9.0, 8.2 / 12.1, 8.6 / 12.3).  Beyond 256 rows the library's kernels
    are the faster ones on the device (512 rows: 10.6 / 12.2, with the activation 20.1 / 19.1;
    1,024 rows: 13.5 / 21.3 and 25.7 / 32.6), but a step of a few hundred tokens of so small a
    model is bound by the host, where a call of the library costs 18 us and one of this kernel
    6: a 512-token prompt of the Qwen3-0.6B shape 5.4 -> 4.2 ms.  Hence up to 512 rows."""
    return (
        SKINNY_MAX_ROWS < m <= TILE_MAX_ROWS
        and k % 128 == 0
        and cols % 4 == 0
        and cols * (weight_rows // cols) >= _TILE_MIN_COLS
        and weight_rows * k <= _TILE_MAX_WEIGHTS
    )


# Rows up to which a product's runs of K may be left to the norm that follows.  Beyond 64 rows the
# kernel runs blocks of 64 rows.  Against the library's product and the plain norm, microseconds
# (the library first): Qwen3-8B output projection 18.7 / 15.2 at 64 rows, 28.1 / 19.9 at 128,
# 36.5 / 24.4 at 192, 27.1 / 30.1 at 256; down projection 40.6 / 30.6, 68.8 / 42.4, 92.6 / 56.4,
# 57.4 / 72.6; the 32B shape's down projection 160 / 65, 184 / 100, 214 / 137, 265 / 180.  The
# library's time jumps between neighbouring row counts (the 8B down projection: 51.8 at 144 rows,
# 78.8 at 160, 55.4 at 176), this kernel's grows with the blocks of 64; from about 200 rows on
# the library's best kernels are the faster ones.  Small matrices (the 0.6B and 1.7B shapes) are
# within a microsecond either way from 144 rows on.
MID_MAX_ROWS = 192
_MID_BLOCK_ROWS = 64  # weight rows per workgroup of the mid-size product
_MID_MAX_BLOCKS = 128  # wider matrices than this many workgroups stay with the library


def mid_runs(n: int, k: int, units: int | None = None) -> int:
    """Runs of K for the mid-size product of an ``[n, k]`` matrix, 0 where it does not apply:
    enough to put a workgroup on every compute unit, at least four chunks of 128 each."""
    units = chip().units if units is None else units
    blocks = -(-n // _MID_BLOCK_ROWS)
    if k % 128 or n % 4 or blocks > _MID_MAX_BLOCKS:
        return 0
    chunks = k // 128
    ks = max(1, min(units // blocks, chunks // 4, 8))
    while ks > 1 and -(-chunks // ks) * (ks - 1) >= chunks:  # every run holds a chunk
        ks -= 1
    return ks


def gemm_bf16_parts(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``x[M,K] @ w[N,K]^T`` for 17 to 192 rows as float32 runs of K, ``[runs, M, N]``: their sum
    is the product.  For products whose result goes into the residual: the norm that follows
    adds the runs (``add_rmsnorm_parts``)."""
    _need(x, "x", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    m, k = x.shape
    n = w.shape[0]
    ks = mid_runs(n, k)
    if k != w.shape[1] or m > MID_MAX_ROWS or ks < 1:
        raise KernelError(f"gemm_bf16_parts does not take x {tuple(x.shape)}, w {tuple(w.shape)}")
    parts = torch.empty((ks, m, n), dtype=torch.float32, device=x.device)
    _ok(core().rl_gemm_mid_parts(_p(x), _p(w), _p(parts), m, n, k, k, k, ks, _stream()), "rl_gemm_mid_parts")
    return parts


def add_rmsnorm_parts(
    residual: torch.Tensor, parts: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, eps: float
) -> None:
    """``residual += bfloat16(sum of parts)`` in place, ``out = norm(residual) * weight``."""
    runs, tokens, hidden = parts.shape
    _need(residual, "residual", torch.float32, (tokens, hidden))
    _need(parts, "parts", torch.float32)
    _need(weight, "norm weight", torch.float32, (hidden,))
    _need(out, "out", torch.bfloat16, (tokens, hidden))
    _ok(
        core().rl_add_rmsnorm_parts(
            _p(residual), _p(parts), runs, _p(weight), _p(out), tokens, hidden, ctypes.c_float(eps), _stream()
        ),
        "rl_add_rmsnorm_parts",
    )


def gemm_bf16_swiglu(x: torch.Tensor, w_gate_up: torch.Tensor, scaled=None) -> torch.Tensor | None:
    """``silu(x Wg^T) * (x Wu^T)`` for the packed ``[gate | up]`` matrix in one kernel: for
    few rows, and for up to 512 rows over a small matrix; ``None`` when the shape is not one a
    fused kernel takes.  ``scaled``: as in ``gemm_bf16``."""
    m, k = x.shape
    two_i = w_gate_up.shape[0]
    if k % 8 or two_i % 2 or x.dtype != torch.bfloat16 or w_gate_up.dtype != torch.bfloat16:
        return None
    if m > SKINNY_MAX_ROWS:
        inter = two_i // 2
        if scaled is not None:
            return None
        _need(x, "x", torch.bfloat16)
        _need(w_gate_up, "w_gate_up", torch.bfloat16, (two_i, k))
        if _tile_applies(m, two_i, k, inter):
            out = torch.empty((m, inter), dtype=torch.bfloat16, device=x.device)
            _ok(core().rl_gemm_tile(_p(x), _p(w_gate_up), _p(out), m, inter, k, k, k, inter, 1, _stream()), "rl_gemm_tile")
            return out
        plan = rows_plan(m, inter, k, swiglu=True)
        if plan is None:
            return None
        out = torch.empty((m, inter), dtype=torch.bfloat16, device=x.device)
        _ok(
            core().rl_gemm_rows(_p(x), _p(w_gate_up), _p(out), m, inter, k, k, k, inter, 1, BF16, *plan, _stream()),
            "rl_gemm_rows",
        )
        return out
    _need(x, "x", torch.bfloat16)
    _need(w_gate_up, "w_gate_up", torch.bfloat16, (two_i, k))
    inter = two_i // 2
    out = torch.empty((m, inter), dtype=torch.bfloat16, device=x.device)
    nt = 2  # one (gate, up) pair of tiles per workgroup
    _ok(
        core().rl_gemm_skinny_swiglu(
            _p(x), _p(w_gate_up), _p(out), m, inter, k, k, k, inter, nt, chip().units,
            *_scaled_args(scaled, m, k), _stream()
        ),
        "rl_gemm_skinny_swiglu",
    )
    return out


class AttentionPlan:
    """Per-step launch data of the matrix-core attention kernels for one group size G
    (query heads per kv head): which requests are single tokens (decode kernel) and how the
    portions of the others are cut into row tiles (prefill kernel)."""

    __slots__ = ("num_decode", "seq_token", "max_decode_ctx", "num_tiles", "tile_info", "tile_keys", "orders",
                 "_prefill_tokens", "_prefill_list", "_decode_order")

    def __init__(self, ctx, group: int, tile_rows: int) -> None:
        self._decode_order = None
        fixed = _static(ctx).get("decode_only_tokens")
        if fixed is not None:
            # a step of single tokens whose index list is already on the device (graphs)
            self.num_decode = fixed.numel()
            self.seq_token = None  # request i is token i: the kernels skip the lookup
            self.max_decode_ctx = max(ctx.h_seq_starts) + 1
            self.num_tiles = 0
            self.tile_info = None
            self.tile_keys = []
            self.orders = {}
            self._prefill_list, self._prefill_tokens = [], None
            return
        dec_tokens: list[int] = []
        self._prefill_list, self._prefill_tokens = [], None
        tile_list: list[tuple[int, int, int, int]] = []
        self.max_decode_ctx = 0
        at = 0
        for start, n in zip(ctx.h_seq_starts, ctx.h_seq_lens):
            if n == 1:
                dec_tokens.append(at)
                self.max_decode_ctx = max(self.max_decode_ctx, start + 1)
            else:
                for row0 in range(0, n * group, tile_rows):
                    tile_list.append((at, start, n, row0))
                self._prefill_list.extend(range(at, at + n))
            at += n
        tiles = [v for t in tile_list for v in t]
        # keys each tile reads: what its workgroups cost
        self.tile_keys = [t[1] + min(t[2], (t[3] + tile_rows) // group) for t in tile_list]
        self.orders = {}
        self.num_decode = len(dec_tokens)
        self.num_tiles = len(tiles) // 4
        device = ctx.token_ids.device
        packed = upload_ints(dec_tokens + tiles, device)
        self.seq_token = packed[: self.num_decode]
        self.tile_info = packed[self.num_decode :]

    def prefill_tokens(self, device) -> torch.Tensor:
        """Indices in the step of the tokens that belong to portions (not single tokens)."""
        if self._prefill_tokens is None:
            self._prefill_tokens = upload_ints(self._prefill_list, device)
        return self._prefill_tokens

    def decode_order(self, ctx) -> torch.Tensor:
        """The step's single-token requests, longest context first, sorted on the device from the
        step's positions (a replayed step has nothing else); made once a step, for every layer."""
        if self._decode_order is None:
            order = torch.empty(self.num_decode, dtype=torch.int32, device=ctx.positions.device)
            _ok(
                core().rl_order_by_length(_p(ctx.positions), _p(self.seq_token), self.num_decode, _p(order), _stream()),
                "rl_order_by_length",
            )
            self._decode_order = order
        return self._decode_order

    def work_order(self, nkv: int, device, resident: int = 1) -> torch.Tensor:
        """Order in which the (tile, kv head) pairs of the prefill kernel are handed out:
        longest first, so that the short ones fill the gaps at the end.  Where a compute unit
        holds two workgroups at a time (``resident == 2``), the first round, one workgroup on
        every unit, takes the longest, and the second round, which joins them on the same
        units, the shortest in ascending order, so that a unit's two workgroups add up alike."""
        order = self.orders.get((nkv, resident))
        if order is None:
            items = sorted(range(self.num_tiles * nkv), key=lambda i: (-self.tile_keys[i // nkv], i))
            if resident == 2:
                round_one = chip().first_round
                first = items[:round_one]
                rest = items[round_one:]
                second = rest[::-1][:round_one]
                middle = rest[: max(0, len(rest) - round_one)]
                items = first + second + middle
            order = upload_ints(items, device)
            self.orders[(nkv, resident)] = order
        return order


# A decode launch splits the keys until it has a workgroup for every compute unit; the fewest
# keys a split is worth (measured at 2,048 keys, 8 kv heads on 256 units: 1 request 128 keys a
# split, 8 requests 512, 64 requests no split; at 512 keys 128 a split for 1 and 8 requests;
# finer splits only add merge work).  A launch of more workgroups than the chip holds at a
# time (``Chip.decode_resident``) hands them out longest request first.
_MIN_SPLIT_KEYS = 128
_MAX_SPLIT_PAGES = 1024  # page ids of one split are staged in LDS
# The prefill kernel cuts its tiles' keys into runs when a launch has fewer workgroups than the
# chip has slots for (``Chip.prefill_slots``) and tiles of at least twice this many keys (a
# portion of one long prompt).
_PREFILL_SPLIT_KEYS = 512
_PREFILL_MAX_SPLITS = 8


def tile_rows_of(lib) -> int:
    return lib.rl_attn_prefill_rows()


_PREFILL_STEP_KEYS = 64  # keys per step of the prefill kernel
# what a step costs more when the two wave groups of a compute unit walk one tile in lockstep
# than when they belong to two tiles and drift apart (measured: 3.17 against 2.83 us)
_PREFILL_PAIRED_COST = 1.12
# a tile that outlasts the others ends alone on its compute unit and steps faster there than
# beside a second workgroup (2,048 tokens behind 2,048: 139 us with one wave group a tile,
# 157 us with two, where whole steps at the shared rate would say 181 against 152)
_PREFILL_ALONE = 0.8
# what cutting the tiles' keys into runs costs, in steps: the runs' partial results are
# written, and read and folded by a second kernel (1,024 tokens from their start: 33 us whole,
# 47 us in two runs)
_PREFILL_MERGE_STEPS = 5


def _prefill_shape(plan: "AttentionPlan", nkv: int, window: int, tile_rows: int,
                   units: int | None = None) -> tuple[int, int]:
    """(wave groups per workgroup, runs the keys of every tile are cut into) for a launch of
    the prefill kernel, from an estimate of the launch's length in steps: the longest tile's
    steps (halved where two wave groups share it, divided where its keys are cut into runs) or
    the steps there are for every slot of the chip, whichever is more.  Few, long tiles (a
    portion of one long prompt) come out with their keys cut into runs, folded by the merge
    kernel; a prompt from its start, whose last rows alone see many keys, with two wave groups
    a tile; a launch with work for every slot with neither."""
    slots = (chip() if units is None else Chip(units)).prefill_slots
    keys = plan.tile_keys
    if window > 0:
        keys = [min(k, window + tile_rows) for k in keys]
    items = plan.num_tiles * nkv
    steps = [-(-k // _PREFILL_STEP_KEYS) for k in keys]
    longest = max(steps)
    share = nkv * sum(steps) / slots  # steps per slot if the work were spread evenly
    best = (max(longest * _PREFILL_ALONE, share), 1, 1)
    paired = max(-(-longest // 2), share) * _PREFILL_PAIRED_COST
    if paired < best[0]:
        best = (paired, 2, 1)
    if items < slots:
        most = min(_PREFILL_MAX_SPLITS, -(-slots // items), max(keys) // _PREFILL_SPLIT_KEYS)
        for nsplit in range(2, most + 1):
            cost = max(-(-longest // nsplit), share) + _PREFILL_MERGE_STEPS
            if cost < best[0]:
                best = (cost, 1, nsplit)
    return best[1], best[2]


def _static(ctx) -> dict:
    """Where launch data that depends on the step's shape alone is kept (``StepContext.static``:
    it survives from the eager run before a recording into the recording)."""
    static = getattr(ctx, "static", None)
    return ctx.extra if static is None else static


def _f32_tiles(ctx, group: int) -> tuple[torch.Tensor, int]:
    """Tiles of 16 (token, head of the group) rows, request by request: ``[tiles, 3]`` int32
    (first token of the request in the step, its tokens, first row of the tile).  A function of
    the requests' token counts alone."""
    key = ("f32_tiles", group)
    store = _static(ctx)
    made = store.get(key)
    if made is None:
        tiles: list[int] = []
        at = 0
        for n in ctx.h_seq_lens:
            for row0 in range(0, n * group, 16):
                tiles += [at, n, row0]
            at += n
        made = (upload_ints(tiles, ctx.token_ids.device), len(tiles) // 3)
        store[key] = made
    return made


def attention_f32(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    out: torch.Tensor,
    ctx,
    block_table: torch.Tensor,
    page_size: int,
    nq: int,
    nkv: int,
    d: int,
    window: int,
    scale: float,
) -> None:
    """float32 attention of every token of the step on the float32 matrix instruction; a
    row's result is the same bit for bit however the step was cut."""
    tokens = q.shape[0]
    pages = k_cache.shape[0]
    _need(q, "q", torch.float32, (tokens, nq * d))
    _need(out, "out", torch.float32, (tokens, nq * d))
    _need(k_cache, "k_cache", torch.float32, (pages, nkv, page_size, d))
    _need(v_cache, "v_cache", torch.float32, (pages, nkv, d, page_size))
    _need(ctx.positions, "positions", torch.int32, (tokens,))
    _need(ctx.token_slot, "token_slot", torch.int32, (tokens,))
    _need(block_table, "block_table", torch.int32)
    if page_size % 4:
        raise KernelError(f"the float32 attention reads four keys of a page at once: page size {page_size}")
    if ctx.max_position // page_size >= block_table.shape[1]:
        raise KernelError(
            f"position {ctx.max_position} needs page {ctx.max_position // page_size} of a block table "
            f"with {block_table.shape[1]} columns"
        )
    if nkv > 65535:
        raise KernelError(f"{nkv} kv heads exceed the launch grid")
    tiles, num_tiles = _f32_tiles(ctx, nq // nkv)
    _ok(
        attention_lib(d).rl_attn_f32(
            _p(q), _p(k_cache), _p(v_cache), _p(out), _p(tiles), num_tiles, _p(ctx.positions),
            _p(ctx.token_slot), _p(block_table), block_table.stride(0), page_size, nq, nkv, window,
            ctypes.c_float(scale), _stream(),
        ),
        "rl_attn_f32",
    )


def paged_attention(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    out: torch.Tensor,
    ctx,
    block_table: torch.Tensor,
    page_size: int,
    nq: int,
    nkv: int,
    d: int,
    window: int,
    scale: float,
    prepare: Optional[tuple] = None,
) -> None:
    """Attention of every token of the step over its request's cached keys.

    Head sizes in steps of 16 run on the matrix cores: float32 on the float32 kernel,
    bfloat16 on the bfloat16 kernels (single tokens go to the split-key decode kernel, portions
    to the tiled prefill kernel).  Other head sizes run the FMA kernel in either type.

    ``prepare`` = ``(q_norm_w, cos, sin, eps)``: ``q`` is the packed [q | k | v] row of every token,
    and the kernels norm and rotate the query heads as they read them (only where
    :func:`attention_prepares_queries` says so)."""
    if prepare is not None and not attention_prepares_queries(q.dtype, d, 0 if prepare[1] is None else prepare[1].shape[1]):
        raise KernelError("the attention kernels do not finish the queries of this head size, type or rotation")
    if q.dtype == torch.float32 and d % 16 == 0:
        attention_f32(q, k_cache, v_cache, out, ctx, block_table, page_size, nq, nkv, d, window, scale)
        return
    if q.dtype != torch.bfloat16 or d % 16:
        attention_generic(
            q, k_cache, v_cache, out, ctx.positions, ctx.token_slot, block_table, page_size,
            nq, nkv, d, window, scale, ctx.max_position,
        )
        return
    tokens = q.shape[0]
    pages = k_cache.shape[0]
    _need(q, "q", torch.bfloat16, (tokens, (nq * d) if prepare is None else (nq + 2 * nkv) * d))
    _need(out, "out", torch.bfloat16, (tokens, nq * d))
    _need(k_cache, "k_cache", torch.bfloat16, (pages, nkv, page_size, d))
    _need(v_cache, "v_cache", torch.bfloat16, (pages, nkv, d, page_size))
    _need(block_table, "block_table", torch.int32)
    if page_size % 4:
        raise KernelError(f"the matrix-core attention kernels need a page size that is a multiple of 4, got {page_size}")
    if ctx.max_position // page_size >= block_table.shape[1]:
        raise KernelError(
            f"position {ctx.max_position} needs page {ctx.max_position // page_size} of a block "
            f"table with {block_table.shape[1]} columns"
        )
    q_norm_w = cos = sin = None
    eps = 0.0
    if prepare is not None:
        q_norm_w, cos, sin, eps = prepare
        if q_norm_w is not None:
            _need(q_norm_w, "q_norm weight", torch.float32, (d,))
        if cos is not None:
            _need(cos, "cos table", torch.float32, (None, d // 2))
            _need(sin, "sin table", torch.float32, tuple(cos.shape))
            if ctx.max_position >= cos.shape[0]:
                raise KernelError(
                    f"position {ctx.max_position} is beyond the rotation table of {cos.shape[0]} positions"
                )
    if ctx.max_position >= (1 << 32) // page_size:
        # the prefill kernel divides positions by the page size with one multiplication
        raise KernelError(f"position {ctx.max_position} is too large for pages of {page_size} tokens")
    lib = attention_lib(d)
    group = nq // nkv
    plan = attention_plan(ctx, group, d)
    if plan.num_tiles:
        groups, nsplit = _prefill_shape(plan, nkv, window, tile_rows_of(lib))
        part_o = part_ml = tokens_list = None
        if nsplit > 1:
            part_o = torch.empty((tokens, nq, nsplit, d), dtype=torch.float32, device=q.device)
            part_ml = torch.empty((tokens, nq, nsplit, 2), dtype=torch.float32, device=q.device)
            tokens_list = plan.prefill_tokens(q.device)
        _ok(
            lib.rl_attn_prefill(
                _p(q), _p(k_cache), _p(v_cache), _p(out), _p(plan.tile_info),
                _p(plan.work_order(nkv, q.device, 2 // groups)), plan.num_tiles,
                _p(ctx.token_slot), _p(block_table), block_table.stride(0), page_size, nq, nkv,
                window, ctypes.c_float(scale), groups, nsplit, _p(part_o), _p(part_ml), _p(tokens_list),
                0 if tokens_list is None else tokens_list.numel(),
                int(prepare is not None), _p(q_norm_w), _p(cos), _p(sin), ctypes.c_float(eps), _stream(),
            ),
            "rl_attn_prefill",
        )
    if plan.num_decode:
        # single tokens beside portions: their keys and values are in the cache already
        fused = None if prepare is None else (q_norm_w, None, cos, sin, None, None, eps)
        _decode_launch(lib, plan, ctx, q, k_cache, v_cache, out, block_table, page_size, nq, nkv, d,
                       window, scale, fused)


def attention_prepares_queries(x_dtype: torch.dtype, d: int, rotary_half: int, pairing: str = "half_split") -> bool:
    """Whether the bfloat16 attention kernels can norm and rotate the query heads themselves, from
    the packed rows: a head size whose rotation pairs stay within a lane, the half-split rotation
    of the whole head or none."""
    if x_dtype != torch.bfloat16 or d % 64 or rotary_half not in (0, d // 2):
        return False
    return not (rotary_half and pairing != "half_split")


def attention_plan(ctx, group: int, d: int) -> AttentionPlan:
    """The step's launch data for one group size, made once and kept with the step."""
    key = ("attention_plan", group)
    plan = ctx.extra.get(key)
    if plan is None:
        plan = AttentionPlan(ctx, group, attention_lib(d).rl_attn_prefill_rows())
        ctx.extra[key] = plan
    return plan


def _decode_launch(lib, plan, ctx, q, k_cache, v_cache, out, block_table, page_size, nq, nkv, d,
                   window, scale, fused) -> None:
    """Split-key decode attention of the step's single tokens.  ``fused`` is ``None`` (``q``
    holds finished queries) or ``(q_norm_w, k_norm_w, cos, sin, k_write, v_write, eps)`` with
    ``q`` the packed [q | k | v] rows."""
    # under a graph the split is laid out for the longest context of the graph's bucket
    span = _static(ctx).get("context_bound", plan.max_decode_ctx)
    pairs, chunk, nsplit = _decode_split(plan.num_decode, nq, nkv, span, page_size, window)
    if plan.num_decode > 65535:
        raise KernelError(f"{plan.num_decode} single-token requests exceed the decode kernel's launch grid")
    # with more workgroups than start at once, the longest requests go first
    order = plan.decode_order(ctx) if pairs * nsplit > chip().decode_resident else None
    part_o = part_ml = None
    if nsplit > 1:
        part_o = torch.empty((plan.num_decode, nq, nsplit, d), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((plan.num_decode, nq, nsplit, 2), dtype=torch.float32, device=q.device)
    qn = kn = cos = sin = kw = vw = None
    eps = 0.0
    if fused is not None:
        qn, kn, cos, sin, kw, vw, eps = fused
    _ok(
        lib.rl_attn_decode(
            _p(q), _p(k_cache), _p(v_cache), _p(out), _p(part_o), _p(part_ml),
            _p(plan.seq_token), _p(order), _p(ctx.positions), _p(ctx.token_slot), _p(block_table),
            block_table.stride(0), page_size, plan.num_decode, nq, nkv, window,
            ctypes.c_float(scale), chunk, nsplit, int(fused is not None), _p(qn), _p(kn), _p(cos),
            _p(sin), _p(kw), _p(vw), ctypes.c_float(eps), _stream(),
        ),
        "rl_attn_decode",
    )


def _decode_split(num_decode: int, nq: int, nkv: int, span: int, page_size: int, window: int,
                  units: int | None = None) -> tuple[int, int, int]:
    """(workgroups before splitting, keys a split, splits) of a decode launch of ``num_decode``
    single tokens over at most ``span`` keys: splits of a multiple of 128 keys, as many as put a
    workgroup on every compute unit, each within what the kernel stages of page ids."""
    units = chip().units if units is None else units
    if window > 0:
        span = min(span, window + 31)
    chunks = (nq // nkv + 15) // 16
    pairs = num_decode * nkv * chunks
    want = max(1, units // pairs)
    chunk = max(_MIN_SPLIT_KEYS, -(-(-(-span // want)) // 128) * 128)
    chunk = min(chunk, max(32, ((_MAX_SPLIT_PAGES - 1) * page_size - 31) // 32 * 32))
    return pairs, chunk, -(-span // chunk)


def decode_scratch_bytes(rows: int, nq: int, nkv: int, d: int, span: int, page_size: int, window: int) -> int:
    """Bytes of split results (float32 outputs, maxima and sums) that a decode launch of
    ``rows`` single tokens over at most ``span`` keys keeps between its two kernels."""
    _, _, nsplit = _decode_split(rows, nq, nkv, span, page_size, window)
    return 0 if nsplit == 1 else rows * nq * nsplit * (d + 2) * 4


def decode_attention_fusable(ctx, x_dtype: torch.dtype, group: int, d: int, rotary_half: int,
                             pairing: str = "half_split") -> bool:
    """Whether the step is one the fused decode kernel takes: bfloat16, single tokens only,
    a head size whose rotation pairs stay within a lane, the half-split rotation of the whole
    head or none."""
    if not attention_prepares_queries(x_dtype, d, rotary_half, pairing):
        return False
    plan = attention_plan(ctx, group, d)
    return plan.num_tiles == 0 and plan.num_decode > 0


def decode_attention_fused(
    qkv: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    out: torch.Tensor,
    ctx,
    block_table: torch.Tensor,
    page_size: int,
    nq: int,
    nkv: int,
    d: int,
    window: int,
    scale: float,
    q_norm_w: Optional[torch.Tensor],
    k_norm_w: Optional[torch.Tensor],
    cos: Optional[torch.Tensor],
    sin: Optional[torch.Tensor],
    eps: float,
    write_cache: bool,
) -> None:
    """Per-head norm, rotation, cache write and split-key attention of a step of single
    tokens in one kernel (plus the merge of the splits).  Same result as
    ``qknorm_rope_kvwrite`` followed by ``paged_attention`` up to rounding."""
    tokens = qkv.shape[0]
    pages = k_cache.shape[0]
    _need(qkv, "qkv", torch.bfloat16, (tokens, (nq + 2 * nkv) * d))
    _need(out, "out", torch.bfloat16, (tokens, nq * d))
    _need(k_cache, "k_cache", torch.bfloat16, (pages, nkv, page_size, d))
    _need(v_cache, "v_cache", torch.bfloat16, (pages, nkv, d, page_size))
    _need(block_table, "block_table", torch.int32)
    if page_size % 4:
        raise KernelError(f"the matrix-core attention kernels need a page size that is a multiple of 4, got {page_size}")
    if ctx.max_position // page_size >= block_table.shape[1]:
        raise KernelError(
            f"position {ctx.max_position} needs page {ctx.max_position // page_size} of a block "
            f"table with {block_table.shape[1]} columns"
        )
    for w, name in ((q_norm_w, "q_norm weight"), (k_norm_w, "k_norm weight")):
        if w is not None:
            _need(w, name, torch.float32, (d,))
    if cos is not None:
        _need(cos, "cos table", torch.float32, (None, d // 2))
        _need(sin, "sin table", torch.float32, tuple(cos.shape))
        if ctx.max_position >= cos.shape[0]:
            raise KernelError(
                f"position {ctx.max_position} is beyond the rotation table of {cos.shape[0]} positions"
            )
    lib = attention_lib(d)
    if not lib.rl_attn_decode_fusable():
        raise KernelError(f"the fused decode kernel needs a head size that is a multiple of 64, got {d}")
    plan = attention_plan(ctx, nq // nkv, d)
    if plan.num_tiles or plan.num_decode != tokens:
        raise KernelError("the fused decode kernel takes steps of single tokens only")
    fused = (q_norm_w, k_norm_w, cos, sin, k_cache if write_cache else None,
             v_cache if write_cache else None, eps)
    _decode_launch(lib, plan, ctx, qkv, k_cache, v_cache, out, block_table, page_size, nq, nkv, d,
                   window, scale, fused)
