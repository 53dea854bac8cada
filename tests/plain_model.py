"""Plain, slow implementation of the Qwen3 dense decoder, used only as the test oracle.

Whole sequences, dense masks, no cache, no paging, one function per part.  It
shares no code with ``rapid_llm_amd``: it reads ``config.json`` with ``json`` and
the weights with ``safetensors.torch.load_file`` under their checkpoint names,
and computes every formula the way the reference states it, with every cast
taken as the identity (all arithmetic in one floating type, float32 by default,
float64 when a tighter oracle is wanted).

Paths in the citations are relative to the reference checkout.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


# --------------------------------------------------------------------------- #
# parts
# --------------------------------------------------------------------------- #


def plain_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``y = x * rsqrt(mean(x^2) + eps) * w`` over the last dimension.

    rapid_llm/kernels/backend/cpu.py:22-29 (``values * rsqrt(values.square().mean(-1) + eps)``
    then ``* weight``); rapid_llm/kernels/ops/layernorm/skip_rmsnorm.py:41-47.
    """
    var = (x * x).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(var + eps) * weight


def plain_inv_freq(head_dim: int, theta: float) -> torch.Tensor:
    """``inv_freq[i] = 1 / theta ** (2i / d)`` in float32.

    rapid_llm/modules/rotary_embedding.py:30-37 (``compute_default_rope``).
    """
    return 1.0 / (float(theta) ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))


def plain_rope_tables(
    positions: torch.Tensor, head_dim: int, theta: float, dtype: torch.dtype = torch.float32
) -> tuple[torch.Tensor, torch.Tensor]:
    """cos / sin of ``outer(position, inv_freq)``: ``[T, d/2]`` each.

    The angle is a float32 product, as in rapid_llm/modules/rotary_embedding.py:194-202
    (``torch.outer(positions, inv_freq)`` with float32 positions); the reference stores
    ``cat(ang, ang)`` and the rotation only reads the first half
    (rapid_llm/kernels/backend/cpu.py:50-51), so only that half is kept here.
    """
    ang = torch.outer(positions.to(torch.float32), plain_inv_freq(head_dim, theta))
    ang = ang.to(torch.float64)
    return ang.cos().to(dtype), ang.sin().to(dtype)


def plain_rope_apply(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Half-split rotation of ``x [T, heads, d]`` with ``cos, sin [T, d/2]``.

    ``x1 = x[..., :d/2]``, ``x2 = x[..., d/2:]``; ``out = cat(x1*c - x2*s, x2*c + x1*s)``.
    rapid_llm/kernels/backend/cpu.py:46-56; rapid_llm/kernels/ops/rope/rope_emb.py:47-82.
    """
    half = x.shape[-1] // 2
    c = cos[:, None, :]
    s = sin[:, None, :]
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)


def plain_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: float,
    window: int | None = None,
    q_positions: torch.Tensor | None = None,
    k_positions: torch.Tensor | None = None,
    hidden: torch.Tensor | None = None,
) -> torch.Tensor:
    """Causal grouped-query attention of one whole sequence, dense mask.

    ``q [Tq, nq, d]``, ``k, v [Tk, nkv, d]``.  Query head ``h`` reads KV head
    ``h // (nq / nkv)`` (rapid_llm/kernels/ops/attention/flashattention2_nopad.py:85;
    ``repeat_interleave`` in rapid_llm/kernels/backend/cpu.py:94-96).  A key at position
    ``j`` is visible to a query at position ``p`` when ``j <= p``
    (rapid_llm/kernels/backend/cpu.py:99) and, under a window of ``w`` positions
    "itself included" (rapid_llm/engine/kv_cache_spec.py:203-205,222), ``p - j < w``.
    Scores are ``(q . k) * scale`` with ``scale = 1/sqrt(d)``
    (rapid_llm/modules/attention.py:62), softmax over the visible keys, then ``P @ V``.
    ``hidden [Tq, Tk]`` (tests of the tests only) marks keys to lose on purpose: what a kernel
    that skips them would compute.
    """
    tq, nq, d = q.shape
    tk, nkv, _ = k.shape
    group = nq // nkv
    if q_positions is None:
        q_positions = torch.arange(tq)
    if k_positions is None:
        k_positions = torch.arange(tk)
    visible = k_positions[None, :] <= q_positions[:, None]
    if window is not None:
        visible &= (q_positions[:, None] - k_positions[None, :]) < window
    if hidden is not None:
        visible = visible & ~hidden
    out = torch.empty_like(q)
    for h in range(nq):
        kh = h // group
        scores = (q[:, h, :] @ k[:, kh, :].T) * scale
        scores = scores.masked_fill(~visible, float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        out[:, h, :] = probs @ v[:, kh, :]
    return out


def plain_swiglu_mlp(
    x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor
) -> torch.Tensor:
    """``down(silu(gate(x)) * up(x))`` with ``silu(z) = z * sigmoid(z)``.

    rapid_llm/modules/mlp.py:67-68; rapid_llm/kernels/ops/activation/swiglu.py:91-121;
    rapid_llm/kernels/ops/activation/activations.py:55-57.
    """
    g = x @ w_gate.T
    u = x @ w_up.T
    return ((g * torch.sigmoid(g)) * u) @ w_down.T


# --------------------------------------------------------------------------- #
# the configuration keys, read with json alone
# --------------------------------------------------------------------------- #


def plain_layer_windows(cfg: dict) -> list[int | None]:
    """Window (or None for all keys) of every layer.

    The reference's Qwen3 never reads the window keys (rapid_llm/models/qwen3.py:16-18);
    the meaning of the keys is the one the checkpoint format documents:
    ``layer_types[i] == "sliding_attention"`` marks a windowed layer; without that list,
    ``use_sliding_window`` turns the window on for the layers from ``max_window_layers``
    upward.  The window itself follows rapid_llm/engine/kv_cache_spec.py:203-205.
    """
    n = cfg["num_hidden_layers"]
    window = cfg.get("sliding_window")
    types = cfg.get("layer_types")
    if types is not None:
        return [window if t == "sliding_attention" else None for t in types]
    if cfg.get("use_sliding_window", False) and window is not None:
        first = cfg.get("max_window_layers", n)
        return [window if i >= first else None for i in range(n)]
    return [None] * n


def plain_rope_theta(cfg: dict) -> float:
    """rapid_llm/models/config.py:317-335: ``rope_theta`` at top level or inside the rope dict."""
    for key in ("rope_parameters", "rope_scaling"):
        sub = cfg.get(key)
        if isinstance(sub, dict) and "rope_theta" in sub:
            return float(sub["rope_theta"])
    return float(cfg.get("rope_theta", 10000.0))


# --------------------------------------------------------------------------- #
# whole model
# --------------------------------------------------------------------------- #


def plain_load(model_dir: str | Path, dtype: torch.dtype = torch.float32) -> tuple[dict, dict]:
    from safetensors.torch import load_file

    model_dir = Path(model_dir)
    cfg = json.loads((model_dir / "config.json").read_text())
    weights = {}
    for shard in sorted(model_dir.glob("*.safetensors")):
        for name, tensor in load_file(str(shard)).items():
            weights[name] = tensor.to(dtype)
    return cfg, weights


def _same(x: torch.Tensor) -> torch.Tensor:
    return x


def plain_block(
    h: torch.Tensor, cfg: dict, w: dict, layer: int, positions: torch.Tensor, window: int | None,
    cast=_same, hide=None,
) -> torch.Tensor:
    """One pre-norm block: ``h += Attn(rms(h)); h += MLP(rms(h))``.

    The reference threads ``(hidden, residual)`` and defers each add into the next norm
    (rapid_llm/models/base.py:231-266,363-375); with exact arithmetic that is this form.
    Inside attention: QKV projection (base.py:121-132), per-head q/k RMSNorm over head_dim
    *before* the rotation (base.py:134-137), rotation (base.py:139-140), attention, output
    projection (base.py:164-165).

    ``cast`` is applied wherever the reference stores an activation in the model's type (the
    residual stream stays as it is); the identity gives exact arithmetic, a round trip through
    bfloat16 shows how far a bfloat16 engine may drift by rounding alone.  ``hide(layer,
    q_positions, k_positions)`` returns keys to lose on purpose (see ``plain_attention``).
    """
    p = f"model.layers.{layer}."
    eps = cfg["rms_norm_eps"]
    nq = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads") or nq
    d = cfg.get("head_dim") or cfg["hidden_size"] // nq
    t = h.shape[0]

    x = cast(plain_rmsnorm(h, w[p + "input_layernorm.weight"], eps))
    q = cast(x @ w[p + "self_attn.q_proj.weight"].T).view(t, nq, d)
    k = cast(x @ w[p + "self_attn.k_proj.weight"].T).view(t, nkv, d)
    v = cast(x @ w[p + "self_attn.v_proj.weight"].T).view(t, nkv, d)
    q = plain_rmsnorm(q, w[p + "self_attn.q_norm.weight"], eps)
    k = plain_rmsnorm(k, w[p + "self_attn.k_norm.weight"], eps)
    cos, sin = plain_rope_tables(positions, d, plain_rope_theta(cfg), h.dtype)
    q = cast(plain_rope_apply(q, cos, sin))
    k = cast(plain_rope_apply(k, cos, sin))
    hidden = hide(layer, positions, positions) if hide is not None else None
    a = cast(plain_attention(q, k, v, 1.0 / math.sqrt(d), window, positions, positions, hidden))
    h = h + cast(a.reshape(t, nq * d) @ w[p + "self_attn.o_proj.weight"].T)

    x = cast(plain_rmsnorm(h, w[p + "post_attention_layernorm.weight"], eps))
    if cast is _same:
        return h + plain_swiglu_mlp(
            x,
            w[p + "mlp.gate_proj.weight"],
            w[p + "mlp.up_proj.weight"],
            w[p + "mlp.down_proj.weight"],
        )
    g = cast(x @ w[p + "mlp.gate_proj.weight"].T)
    u = cast(x @ w[p + "mlp.up_proj.weight"].T)
    act = cast((g * torch.sigmoid(g)) * u)
    return h + cast(act @ w[p + "mlp.down_proj.weight"].T)


def plain_forward(
    cfg: dict, w: dict, token_ids: list[int] | torch.Tensor, position_offset: int = 0,
    cast=_same, hide=None, rows=None,
) -> torch.Tensor:
    """Logits ``[T, V]`` of one whole sequence.

    Embedding is a plain row gather (rapid_llm/modules/vocab_parallel.py:102-103), then the
    blocks, the final norm (rapid_llm/models/base.py:619-621) and the output projection,
    which reuses the embedding table when ``tie_word_embeddings`` is set and the checkpoint
    ships no ``lm_head.weight`` (rapid_llm/models/weights.py:197-214).
    ``position_offset`` shifts every position; it exists for the invariance test.  ``cast`` and
    ``hide`` as in ``plain_block``; ``rows`` (a list of positions) limits the final norm and the
    output projection to those rows, for vocabularies and lengths whose whole product is too
    large to hold.
    """
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    positions = torch.arange(ids.numel()) + position_offset
    h = w["model.embed_tokens.weight"][ids]
    windows = plain_layer_windows(cfg)
    for layer in range(cfg["num_hidden_layers"]):
        h = plain_block(h, cfg, w, layer, positions, windows[layer], cast, hide)
    if rows is not None:
        h = h[torch.as_tensor(rows, dtype=torch.long)]
    h = cast(plain_rmsnorm(h, w["model.norm.weight"], cfg["rms_norm_eps"]))
    head = w.get("lm_head.weight")
    if head is None:
        if not cfg.get("tie_word_embeddings", False):
            raise KeyError("lm_head.weight missing and tie_word_embeddings is false")
        head = w["model.embed_tokens.weight"]
    return h @ head.T


def plain_greedy(cfg: dict, w: dict, prompt: list[int], num_new: int) -> list[int]:
    """Greedy continuation by re-running the whole sequence for every token."""
    ids = list(prompt)
    out = []
    for _ in range(num_new):
        nxt = int(torch.argmax(plain_forward(cfg, w, ids)[-1]))
        out.append(nxt)
        ids.append(nxt)
    return out
