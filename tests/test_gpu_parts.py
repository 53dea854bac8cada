"""Each part the model is put together from, alone against its plain formula; and the seams:
a toy mixer with state of its own and a toy architecture, registered, built and stepped
without a change to the framework; a run order that names a layer twice; a layer that reads
another layer's cache."""

import math
from dataclasses import dataclass

import pytest
import torch

import parity
from rotation_reference import rotate_pairs
from plain_model import (
    plain_attention,
    plain_load,
    plain_rmsnorm,
    plain_rope_apply,
    plain_rope_tables,
    plain_swiglu_mlp,
)
from tiny_configs import TINY, make_model_dir, random_tokens

pytestmark = pytest.mark.gpu

TOL = {"float32": dict(rtol=2e-5, atol=2e-6), "bfloat16": dict(rtol=3e-2, atol=2e-2)}


def _runner(model_dir, dtype, page, **kw):
    from rapid_llm_amd import EngineConfig, ModelRunner

    body = dict(dtype=dtype, max_seq_len=128, page_size=page, num_pages=64, max_num_seqs=4, use_graph=False)
    body.update(kw)
    return ModelRunner(model_dir, EngineConfig(**body))


def _context(runner, entries):
    meta = runner._prepare(entries)
    host, offs = runner._pack(entries, meta)
    dev = torch.from_numpy(host).to(runner.device)
    return runner._context(dev, offs, meta)


@pytest.mark.parametrize("which", ["A", "B", "C", "D"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_parts_alone(tmp_path, which, dtype):
    from rapid_llm_amd import StepEntry
    from rapid_llm_amd.parts.lazy import plain

    cfg, page, seed = TINY[which]
    model_dir = make_model_dir(tmp_path, which, dtype)
    _, w = plain_load(model_dir)
    runner = _runner(model_dir, dtype, page)
    tdt = runner.dtype
    tol = TOL[dtype]
    H, nq, nkv, d = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps = cfg["rms_norm_eps"]
    # two requests in one batch: 11 and 6 tokens
    lens = (11, 6)
    entries = [StepEntry(f"p{i}", random_tokens(n, cfg["vocab_size"], seed + i), [n - 1]) for i, n in enumerate(lens)]
    ctx = _context(runner, entries)
    T = sum(lens)
    gen = torch.Generator().manual_seed(seed)
    model = runner.model

    # ---- embedding: a row gather into the float32 stream --------------------------------
    emb = model.embed.forward(ctx.token_ids, ctx).cpu()
    ids = [t for e in entries for t in e.tokens]
    assert emb.dtype == torch.float32
    torch.testing.assert_close(emb, w["model.embed_tokens.weight"][torch.tensor(ids)], rtol=0, atol=0)

    # ---- norm with the residual add in front of it, whole and on chosen rows -----------------
    block = model.blocks[1]
    residual = torch.randn(T, H, generator=gen)
    delta = torch.randn(T, H, generator=gen).to(tdt)
    res_dev = residual.cuda()
    out = block.mixer_norm.forward(res_dev, delta.cuda(), ctx).cpu().float()
    summed = residual + delta.float()
    torch.testing.assert_close(res_dev.cpu(), summed, rtol=0, atol=0)  # written in place, in float32
    torch.testing.assert_close(out, plain_rmsnorm(summed, w["model.layers.1.input_layernorm.weight"], eps), **tol)
    rows = torch.tensor([T - 1, 2], dtype=torch.int32).cuda()
    picked = model.final_norm.forward(res_dev, None, ctx, rows=rows).cpu().float()
    torch.testing.assert_close(picked, plain_rmsnorm(summed[[T - 1, 2]], w["model.norm.weight"], eps), **tol)

    # ---- feed-forward ----------------------------------------------------------------------
    x = (torch.randn(T, H, generator=gen) * 0.5).to(tdt)
    p = "model.layers.1.mlp."
    # in a step of few bfloat16 rows a part may hand on its last product unfinished: plain() runs it
    got = plain(block.feed_forward.forward(x.cuda(), ctx)).cpu().float()
    want = plain_swiglu_mlp(x.float(), w[p + "gate_proj.weight"], w[p + "up_proj.weight"], w[p + "down_proj.weight"])
    torch.testing.assert_close(got, want, **tol)

    # ---- position tables ---------------------------------------------------------------------
    cos, sin = plain_rope_tables(torch.arange(128), d, cfg["rope_theta"])
    rope = block.mixer.position
    torch.testing.assert_close(rope.cos.cpu(), cos, rtol=0, atol=1e-6)
    torch.testing.assert_close(rope.sin.cpu(), sin, rtol=0, atol=1e-6)

    # ---- the mixer: projection, head norms, rotation, cache write, attention, projection ----
    a = "model.layers.1.self_attn."
    got = plain(block.mixer.forward(x.cuda(), ctx, runner.device_cache.layers[1])).cpu().float()
    window = cfg.get("sliding_window") if cfg.get("layer_types", ["full_attention"] * 3)[1] == "sliding_attention" else None
    want, at = [], 0
    for n in lens:
        xs = x[at : at + n].float()
        q = plain_rmsnorm((xs @ w[a + "q_proj.weight"].T).view(n, nq, d), w[a + "q_norm.weight"], eps)
        k = plain_rmsnorm((xs @ w[a + "k_proj.weight"].T).view(n, nkv, d), w[a + "k_norm.weight"], eps)
        v = (xs @ w[a + "v_proj.weight"].T).view(n, nkv, d)
        c, s = plain_rope_tables(torch.arange(n), d, cfg["rope_theta"])
        o = plain_attention(plain_rope_apply(q, c, s), plain_rope_apply(k, c, s), v, 1 / math.sqrt(d), window)
        want.append(o.reshape(n, nq * d) @ w[a + "o_proj.weight"].T)
        at += n
    torch.testing.assert_close(got, torch.cat(want), **tol)

    # ---- output projection -------------------------------------------------------------------
    h = torch.randn(3, H, generator=gen).to(tdt)
    logits = model.output.forward(h.cuda(), ctx).cpu()
    head = w.get("lm_head.weight", w["model.embed_tokens.weight"])
    assert logits.dtype == torch.float32
    torch.testing.assert_close(logits, h.float() @ head.T, **tol)


# --------------------------------------------------------------------------- #
# a toy architecture defined here: a mixer with state of its own in layer 0, attention in
# layer 1, and a run order that visits layer 1 twice
# --------------------------------------------------------------------------- #
@dataclass(frozen=True)
class ToyConfig:
    hidden: int
    vocab: int
    heads: int
    head_dim: int
    inter: int
    decay: float
    twice: bool = False
    share: bool = False
    experts: int = 0  # > 0: layer 0's feed-forward routes every token to one of so many experts
    period: float = 0.0  # > 0: the toy mixer adds a phase of the position to its input
    toynorm: bool = False  # layer 1 uses a norm defined here, which knows nothing of unfinished products
    ends: bool = False  # an embedding that scales its rows and an output projection that caps its logits
    replay: bool = False  # the toy mixer runs on the device alone and declares itself replayable
    bias: bool = False  # the attention's projections have biases (Qwen3 has none; the part can)
    latent: int = 0  # > 0: layer 0's mixer pages one latent row of so many channels per token, and no values
    rotation: str = "whole"  # "half": a position part defined here rotates the first half of a head; "interleaved"

    @classmethod
    def from_dict(cls, data, overrides=None):
        return cls(data["hidden"], data["vocab"], data["heads"], data["head_dim"], data["inter"],
                   data["decay"], data.get("twice", False), data.get("share", False),
                   data.get("experts", 0), data.get("period", 0.0), data.get("toynorm", False),
                   data.get("ends", False), data.get("replay", False), data.get("bias", False),
                   data.get("latent", 0), data.get("rotation", "whole"))

    def to_dict(self):
        return dict(architectures=["ToyForCausalLM"], hidden=self.hidden, vocab=self.vocab, heads=self.heads,
                    head_dim=self.head_dim, inter=self.inter, decay=self.decay, twice=self.twice,
                    share=self.share, experts=self.experts, period=self.period, toynorm=self.toynorm,
                    ends=self.ends, replay=self.replay, bias=self.bias, latent=self.latent,
                    rotation=self.rotation, torch_dtype="float32")


CAP = 0.3  # the toy output projection's cap: logits = CAP * tanh(h W^T / CAP)


def _phase(positions, period, size):
    """The toy position encoding: a sinusoid of the position, scaled differently per channel."""
    scale = torch.linspace(0.5, 1.5, size, device=positions.device)
    return torch.sin(positions.float()[:, None] * (2 * math.pi / period)) * scale


def _toy_parts():
    from rapid_llm_amd.kernels.upload import upload_ints
    from rapid_llm_amd.parts import (
        EMBEDDINGS, FEED_FORWARDS, MIXERS, NORMS, OUTPUT_PROJECTIONS, POSITION_ENCODINGS, CacheNeed, Embedding,
        FeedForward, Mixer, Norm, OutputProjection, PagedSpec, ParamSpec, PositionEncoding, Source, StateSpec,
    )
    from rapid_llm_amd.parts.linear import Linear

    class ScaledEmbedding(Embedding):
        """Rows of the table times sqrt(hidden), with tensor operations; tokens still on the
        device (negative ids) are looked up in the buffer the sampling kernels write."""

        replayable = True

        def __init__(self, vocab_size, hidden_size, checkpoint_name, name="embed"):
            self.v, self.h, self.checkpoint_name, self.name = vocab_size, hidden_size, checkpoint_name, name

        def param_specs(self):
            return [ParamSpec(self.name + ".weight", (self.v, self.h), "matrix", (Source(self.checkpoint_name, self.v),))]

        def bind(self, params, runtime):
            self.table = params[self.name + ".weight"]

        def forward(self, token_ids, ctx):
            ids = token_ids.long()
            fed = ctx.fed_tokens.long()
            ids = torch.where(ids < 0, fed[(-ids - 1).clamp(min=0, max=fed.numel() - 1)], ids)
            return self.table[ids].float() * math.sqrt(self.h)

    class CappedOutput(OutputProjection):
        replayable = True

        def __init__(self, vocab_size, hidden_size, checkpoint_name, cap, name="output"):
            self.v, self.h, self.checkpoint_name, self.cap, self.name = vocab_size, hidden_size, checkpoint_name, cap, name
            self.proj = Linear(hidden_size, vocab_size)

        def param_specs(self):
            return [ParamSpec(self.name + ".weight", (self.v, self.h), "matrix", (Source(self.checkpoint_name, self.v),))]

        def bind(self, params, runtime):
            self.proj.bind(params[self.name + ".weight"])

        def forward(self, h, ctx):
            return self.cap * torch.tanh(self.proj(h, out_dtype=torch.float32) / self.cap)

    EMBEDDINGS.register("toy_scaled_embedding", ScaledEmbedding, replace=True)
    OUTPUT_PROJECTIONS.register("toy_capped_output", CappedOutput, replace=True)

    class PlainTorchNorm(Norm):
        """The same formula as the built-in norm, written with tensor operations: it declares
        nothing, so whatever its neighbours would leave unfinished reaches it as a tensor."""

        def __init__(self, size, eps, checkpoint_name, name="norm"):
            self.size, self.eps, self.checkpoint_name, self.name = size, eps, checkpoint_name, name

        def param_specs(self):
            return [ParamSpec(self.name + ".weight", (self.size,), "vector",
                              (Source(self.checkpoint_name, self.size),), init="norm")]

        def bind(self, params, runtime):
            self.weight, self.dtype = params[self.name + ".weight"], runtime.dtype

        def forward(self, residual, delta, ctx, rows=None):
            assert delta is None or isinstance(delta, torch.Tensor)
            if delta is not None:
                residual.add_(delta.float())
            x = residual if rows is None else residual[rows.long()]
            return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight).to(self.dtype)

    NORMS.register("toy_plain_norm", PlainTorchNorm, replace=True)

    class PhaseTable(PositionEncoding):
        """Another position encoding: an additive table by absolute position."""

        kind = "toy_phase"

        def __init__(self, size, period):
            self.size, self.period, self.table = size, period, None

        def bind(self, params, runtime):
            pos = torch.arange(runtime.max_seq_len, device=runtime.device)
            self.table = _phase(pos, self.period, self.size)

    class RoutedFF(FeedForward):
        """A feed-forward with routing: the router's logits in float32, the best expert takes
        the token, its output is weighted with the router's probability."""

        def __init__(self, hidden_size, inter, experts, checkpoint_prefix, name="ff"):
            self.h, self.i, self.e, self.prefix, self.name = hidden_size, inter, experts, checkpoint_prefix, name

        def param_specs(self):
            p, n = self.prefix, self.name
            return [
                ParamSpec(n + ".router", (self.e, self.h), "matrix", (Source(p + "router", self.e),)),
                ParamSpec(n + ".w1", (self.e * self.i, self.h), "matrix",
                          tuple(Source(f"{p}e{k}.w1", self.i) for k in range(self.e))),
                ParamSpec(n + ".w2", (self.e * self.h, self.i), "matrix",
                          tuple(Source(f"{p}e{k}.w2", self.h) for k in range(self.e))),
            ]

        def bind(self, params, runtime):
            self.router = params[self.name + ".router"]
            self.w1 = params[self.name + ".w1"].view(self.e, self.i, self.h)
            self.w2 = params[self.name + ".w2"].view(self.e, self.h, self.i)

        def forward(self, x, ctx):
            probs = torch.softmax(x.float() @ self.router.float().T, dim=-1)
            weight, choice = probs.max(dim=-1)
            out = torch.zeros_like(x)
            for k in range(self.e):
                rows = torch.nonzero(choice == k).flatten()
                if rows.numel():
                    y = torch.relu(x[rows] @ self.w1[k].T) @ self.w2[k].T
                    out[rows] = y * weight[rows, None].to(x.dtype)
            return out

    POSITION_ENCODINGS.register("toy_phase", PhaseTable, replace=True)
    FEED_FORWARDS.register("toy_routed", RoutedFF, replace=True)

    class DecayingSum(Mixer):
        """``s_t = decay * s_{t-1} + x_t`` per request, output ``W s_t``: no pages, one vector of
        state per request, carried from step to step in the request's slot."""

        def __init__(self, hidden_size, decay, checkpoint_prefix, position=None, name="mixer"):
            self.h, self.decay, self.prefix, self.name = hidden_size, decay, checkpoint_prefix, name
            self.position = position
            self.proj = Linear(hidden_size, hidden_size)

        def param_specs(self):
            return [ParamSpec(self.name + ".w", (self.h, self.h), "matrix", (Source(self.prefix + "w", self.h),))]

        def bind(self, params, runtime):
            self.proj.bind(params[self.name + ".w"])

        def cache_need(self):
            return CacheNeed("state", state_shape=(self.h,), state_dtype="float32")

        def forward(self, x, ctx, cache):
            out = torch.empty_like(x, dtype=torch.float32)
            at = 0
            for slot, n in zip(ctx.h_seq_slots, ctx.h_seq_lens):
                s = cache.state[slot]
                for t in range(at, at + n):
                    xt = x[t].float()
                    if self.position is not None and getattr(self.position, "table", None) is not None:
                        xt = xt + self.position.table[ctx.positions[t]]
                    s = self.decay * s + xt
                    out[t] = s
                cache.state[slot] = s
                at += n
            return self.proj(out.to(x.dtype))

    MIXERS.register("toy_decaying_sum", DecayingSum, replace=True)

    class DeviceDecayingSum(Mixer):
        """The same recurrence with two state tensors of its own (the sum, and how many tokens
        went into it), run by device operations alone: a step of single tokens updates the slots of
        all its requests at once and may be recorded.  The per-row decay it multiplies with is
        launch data that depends on the number of rows only: it is uploaded once and kept in
        ``ctx.static``, where the recording finds it again."""

        replayable = True
        uploads = 0  # how often the launch data was made (the test counts)

        def __init__(self, hidden_size, decay, checkpoint_prefix, position=None, name="mixer"):
            self.h, self.decay, self.prefix, self.name = hidden_size, decay, checkpoint_prefix, name
            self.proj = Linear(hidden_size, hidden_size)

        def param_specs(self):
            return [ParamSpec(self.name + ".w", (self.h, self.h), "matrix", (Source(self.prefix + "w", self.h),))]

        def bind(self, params, runtime):
            self.proj.bind(params[self.name + ".w"])

        def cache_need(self):
            return CacheNeed("state", states=(StateSpec("sum", (self.h,), "float32"), StateSpec("count", (1,), "int32")))

        def forward(self, x, ctx, cache):
            total, count = cache.states["sum"], cache.states["count"]
            slots = ctx.token_slot.long()
            if ctx.max_seq_tokens == 1:  # fixed for a recorded step
                key = ("toy_decay_rows", x.shape[0])
                rows = ctx.static.get(key)
                if rows is None:
                    type(self).uploads += 1
                    milli = upload_ints([int(round(self.decay * 1000))] * x.shape[0], x.device)
                    rows = ctx.static[key] = (milli.float() / 1000.0)[:, None]
                s = total[slots] * rows + x.float()
                total.index_copy_(0, slots, s)
                count.index_copy_(0, slots, count[slots] + 1)
                return self.proj(s.to(x.dtype))
            out = torch.empty_like(x, dtype=torch.float32)  # portions: never recorded, host lists are fine
            at = 0
            for slot, n in zip(ctx.h_seq_slots, ctx.h_seq_lens):
                s = total[slot]
                for t in range(at, at + n):
                    s = self.decay * s + x[t].float()
                    out[t] = s
                total[slot] = s
                count[slot] += n
                at += n
            return self.proj(out.to(x.dtype))

    MIXERS.register("toy_device_decaying_sum", DeviceDecayingSum, replace=True)

    class LatentMemory(Mixer):
        """A mixer that pages one latent row per token and no values: ``c_t = x_t Wd`` is written
        to the token's place in the request's pages (``[pages, page_size, rank]``, as this mixer
        names it), a token attends over the latents up to its own with ``q_t = x_t Wq``, and the
        mix of latents goes up through ``Wu``.  The cache manager, the device cache and the step
        function see only a paged tensor called "latent"."""

        def __init__(self, hidden_size, rank, checkpoint_prefix, position=None, name="mixer"):
            self.h, self.r, self.prefix, self.name = hidden_size, rank, checkpoint_prefix, name
            self.down, self.query, self.up = Linear(hidden_size, rank), Linear(hidden_size, rank), Linear(rank, hidden_size)

        def param_specs(self):
            p, n = self.prefix, self.name
            return [ParamSpec(n + ".wd", (self.r, self.h), "matrix", (Source(p + "wd", self.r),)),
                    ParamSpec(n + ".wq", (self.r, self.h), "matrix", (Source(p + "wq", self.r),)),
                    ParamSpec(n + ".wu", (self.h, self.r), "matrix", (Source(p + "wu", self.h),))]

        def bind(self, params, runtime):
            self.down.bind(params[self.name + ".wd"])
            self.query.bind(params[self.name + ".wq"])
            self.up.bind(params[self.name + ".wu"])

        def cache_need(self):
            return CacheNeed("paged", paged=(PagedSpec("latent", (self.r,), 0),))

        def forward(self, x, ctx, cache):
            store, size = cache.pages["latent"], cache.page_size
            table = ctx.block_tables[cache.group_id]
            assert store.shape[1:] == (size, self.r) and cache.k is None and cache.v is None
            c, q = self.down(x), self.query(x)
            pos, slots = ctx.positions.long(), ctx.token_slot.long()
            page = table[slots, pos // size].long()
            store[page, pos % size] = c  # this step's latents first, then everything is read back
            out = torch.empty_like(c, dtype=torch.float32)
            at = 0
            for slot, start, n in zip(ctx.h_seq_slots, ctx.h_seq_starts, ctx.h_seq_lens):
                total = start + n
                pages = table[slot, : -(-total // size)].long()
                mem = store[pages].reshape(-1, self.r)[:total].float()
                scores = q[at : at + n].float() @ mem.T / math.sqrt(self.r)
                seen = torch.arange(total, device=x.device)[None, :] <= (start + torch.arange(n, device=x.device))[:, None]
                out[at : at + n] = torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1) @ mem
                at += n
            return self.up(out.to(x.dtype))

    MIXERS.register("toy_latent_memory", LatentMemory, replace=True)

    class HalfHeadRotary(PositionEncoding):
        """A rotation of the first half of a head only, tables made here with tensor operations.
        It says how it is to be applied (``rotary_dim``, ``pairing``); the attention part of the
        package and its kernels do the applying."""

        kind = "toy_half_rotary"
        replayable = True
        pairing = "half_split"

        def __init__(self, head_dim, theta):
            self.head_dim, self.theta, self.rotary_dim = head_dim, theta, head_dim // 2

        def bind(self, params, runtime):
            rot = self.rotary_dim
            inv = 1.0 / (self.theta ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))
            angle = (torch.arange(runtime.max_seq_len).float()[:, None] * inv[None, :]).double()
            self.cos = angle.cos().float().to(runtime.device).contiguous()
            self.sin = angle.sin().float().to(runtime.device).contiguous()

    POSITION_ENCODINGS.register("toy_half_rotary", HalfHeadRotary, replace=True)
    return DeviceDecayingSum


def _toy_spec(cfg: ToyConfig):
    from rapid_llm_amd.models import LayerSpec, ModelSpec, PartSpec, linear_output, token_embedding

    def norm(name):
        return PartSpec("rmsnorm", {"size": cfg.hidden, "eps": 1e-5, "checkpoint_name": name})

    def ff(i):
        return PartSpec("swiglu", {"hidden_size": cfg.hidden, "intermediate_size": cfg.inter,
                                   "checkpoint_prefix": f"l{i}.ff."})

    rope = PartSpec("rope_half_split", {"head_dim": cfg.head_dim, "theta": 100.0})
    if cfg.rotation == "half":
        rope = PartSpec("toy_half_rotary", {"head_dim": cfg.head_dim, "theta": 100.0})
    elif cfg.rotation == "interleaved":
        rope = PartSpec("rope", {"head_dim": cfg.head_dim, "theta": 100.0, "pairing": "interleaved"})

    def attn(i):
        return PartSpec("gqa_attention", {"hidden_size": cfg.hidden, "num_heads": cfg.heads, "num_kv_heads": 1,
                                          "head_dim": cfg.head_dim, "checkpoint_prefix": f"l{i}.attn.",
                                          "qkv_bias": cfg.bias, "o_bias": cfg.bias})

    ff0 = ff(0)
    if cfg.experts:
        ff0 = PartSpec("toy_routed", {"hidden_size": cfg.hidden, "inter": cfg.inter, "experts": cfg.experts,
                                      "checkpoint_prefix": "l0.moe."})
    pos0 = PartSpec("toy_phase", {"size": cfg.hidden, "period": cfg.period}) if cfg.period else PartSpec("none")
    def norm1(name):
        if cfg.toynorm:
            return PartSpec("toy_plain_norm", {"size": cfg.hidden, "eps": 1e-5, "checkpoint_name": name})
        return norm(name)

    mixer0 = PartSpec("toy_device_decaying_sum" if cfg.replay else "toy_decaying_sum",
                      {"hidden_size": cfg.hidden, "decay": cfg.decay, "checkpoint_prefix": "l0.mix."})
    if cfg.latent:
        mixer0 = PartSpec("toy_latent_memory", {"hidden_size": cfg.hidden, "rank": cfg.latent,
                                                "checkpoint_prefix": "l0.mix."})
    layers = [
        LayerSpec(mixer0, ff0, norm("l0.n1"), norm("l0.n2"), position=pos0),
        LayerSpec(attn(1), ff(1), norm1("l1.n1"), norm1("l1.n2"), position=rope),
    ]
    if cfg.share:
        layers.append(LayerSpec(attn(2), ff(2), norm("l2.n1"), norm("l2.n2"), position=rope, share_cache_with=1))
    order = (0, 1, 0, 1) if cfg.twice else None
    embedding, output = token_embedding(cfg.vocab, cfg.hidden, "embed"), linear_output(cfg.vocab, cfg.hidden, "head", False)
    if cfg.ends:
        embedding = PartSpec("toy_scaled_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.hidden,
                                                      "checkpoint_name": "embed"})
        output = PartSpec("toy_capped_output", {"vocab_size": cfg.vocab, "hidden_size": cfg.hidden,
                                                "checkpoint_name": "head", "cap": CAP})
    return ModelSpec(cfg.hidden, cfg.vocab, tuple(layers), norm("final"), embedding, output, run_order=order)


def _toy_plain(w, cfg: ToyConfig, toks):
    """The toy model, whole sequence, in plain torch."""
    t = len(toks)
    h = w["embed"][torch.tensor(toks)]
    if cfg.ends:
        h = h * math.sqrt(cfg.hidden)
    pos = torch.arange(t)

    def ffn(i, h):
        x = plain_rmsnorm(h, w[f"l{i}.n2"], 1e-5)
        if i == 0 and cfg.experts:
            probs = torch.softmax(x @ w["l0.moe.router"].T, dim=-1)
            weight, choice = probs.max(dim=-1)
            y = torch.stack([
                torch.relu(x[j] @ w[f"l0.moe.e{int(choice[j])}.w1"].T) @ w[f"l0.moe.e{int(choice[j])}.w2"].T * weight[j]
                for j in range(t)
            ])
            return h + y
        return h + plain_swiglu_mlp(x, w[f"l{i}.ff.gate_proj.weight"], w[f"l{i}.ff.up_proj.weight"],
                                    w[f"l{i}.ff.down_proj.weight"])

    def rotate(x):
        if cfg.rotation == "whole":
            c, s = plain_rope_tables(pos, cfg.head_dim, 100.0)
            return plain_rope_apply(x, c, s)
        rot = cfg.head_dim // 2 if cfg.rotation == "half" else cfg.head_dim
        return rotate_pairs(x, pos, rot, 100.0, "half_split" if cfg.rotation == "half" else "interleaved")

    def toy(h):
        x = plain_rmsnorm(h, w["l0.n1"], 1e-5)
        if cfg.latent:
            c, q = x @ w["l0.mix.wd"].T, x @ w["l0.mix.wq"].T
            scores = (q @ c.T / math.sqrt(cfg.latent)).masked_fill(pos[None, :] > pos[:, None], float("-inf"))
            return ffn(0, h + (torch.softmax(scores, dim=-1) @ c) @ w["l0.mix.wu"].T)
        s, rows = torch.zeros(cfg.hidden), []
        if cfg.period:
            x = x + _phase(pos, cfg.period, cfg.hidden)
        for j in range(t):
            s = cfg.decay * s + x[j]
            rows.append(s)
        return ffn(0, h + torch.stack(rows) @ w["l0.mix.w"].T)

    def proj(i, which, x):
        y = x @ w[f"l{i}.attn.{which}_proj.weight"].T
        return y + w[f"l{i}.attn.{which}_proj.bias"] if cfg.bias else y

    def kv_of(i, h):
        x = plain_rmsnorm(h, w[f"l{i}.n1"], 1e-5)
        k = rotate(proj(i, "k", x).view(t, 1, cfg.head_dim))
        return k, proj(i, "v", x).view(t, 1, cfg.head_dim)

    def attn(i, h, kv=None):
        x = plain_rmsnorm(h, w[f"l{i}.n1"], 1e-5)
        q = rotate(proj(i, "q", x).view(t, cfg.heads, cfg.head_dim))
        k, v = kv if kv is not None else kv_of(i, h)
        o = plain_attention(q, k, v, cfg.head_dim**-0.5).reshape(t, -1)
        return ffn(i, h + proj(i, "o", o))

    if cfg.twice:
        h = attn(1, toy(h))
        # the second visit of layer 0 starts from fresh state: each place in the order has its own
        h = attn(1, toy(h))
    else:
        h = toy(h)
        kv = kv_of(1, h)
        h = attn(1, h)
        if cfg.share:
            h = attn(2, h, kv)  # reads the keys and values layer 1 wrote
    logits = plain_rmsnorm(h, w["final"], 1e-5) @ w["head"].T
    return CAP * torch.tanh(logits / CAP) if cfg.ends else logits


def _unregister_toys():
    from rapid_llm_amd.config import unregister_architecture
    from rapid_llm_amd.parts import EMBEDDINGS, FEED_FORWARDS, MIXERS, NORMS, OUTPUT_PROJECTIONS, POSITION_ENCODINGS

    unregister_architecture("ToyForCausalLM")
    MIXERS.unregister("toy_decaying_sum")
    MIXERS.unregister("toy_device_decaying_sum")
    MIXERS.unregister("toy_latent_memory")
    POSITION_ENCODINGS.unregister("toy_half_rotary")
    FEED_FORWARDS.unregister("toy_routed")
    POSITION_ENCODINGS.unregister("toy_phase")
    NORMS.unregister("toy_plain_norm")
    EMBEDDINGS.unregister("toy_scaled_embedding")
    OUTPUT_PROJECTIONS.unregister("toy_capped_output")


@pytest.mark.parametrize("variant,dtype", [("plain", "float32"), ("twice", "float32"), ("share", "float32"),
                                           ("routed", "float32"), ("toynorm", "float32"), ("ends", "float32"),
                                           ("replay", "float32"), ("bias", "float32"),
                                           ("latent", "float32"), ("halfrot", "float32"), ("interleaved", "float32"),
                                           ("routed", "bfloat16"), ("toynorm", "bfloat16"), ("twice", "bfloat16"),
                                           ("ends", "bfloat16"), ("bias", "bfloat16"),
                                           ("latent", "bfloat16"), ("halfrot", "bfloat16"), ("interleaved", "bfloat16")])
def test_toy_architecture_registers_builds_and_steps(tmp_path, variant, dtype):
    """In bfloat16 the built-in parts hand unfinished products and unscaled rows to each other
    in steps of few tokens; the toy parts declare nothing and must only ever see tensors."""
    from safetensors.torch import load_file

    from rapid_llm_amd import StepEntry, write_random_model
    from rapid_llm_amd.config import register_architecture

    _toy_parts()
    register_architecture("ToyForCausalLM", ToyConfig, _toy_spec, replace=True)
    try:
        # the other rotations at a head size whose single-token steps would otherwise run the
        # kernel that rotates inside the attention: it must be passed by for them
        other_rotation = {"halfrot": "half", "interleaved": "interleaved"}.get(variant, "whole")
        cfg = ToyConfig(hidden=48, vocab=97, heads=3, head_dim=64 if other_rotation != "whole" else 16, inter=80,
                        decay=0.8, twice=variant == "twice", share=variant == "share",
                        experts=3 if variant == "routed" else 0, period=9.0 if variant == "routed" else 0.0,
                        toynorm=variant == "toynorm", ends=variant == "ends", replay=variant == "replay",
                        bias=variant == "bias", latent=24 if variant == "latent" else 0, rotation=other_rotation)
        folder = write_random_model(cfg.to_dict(), 3, tmp_path / "toy", dtype=dtype)
        weights = {k: v.float() for k, v in load_file(str(folder / "model.safetensors")).items()}
        if variant == "share":  # the sharing layer's own k/v projections exist but are never used
            assert "l2.attn.k_proj.weight" in weights
        runner = _runner(folder, dtype, 8)
        needs = runner.model.cache_needs()
        if variant == "toynorm":
            assert type(runner.model.blocks[1].mixer_norm).__name__ == "PlainTorchNorm"
        assert needs[0].kind == ("paged" if variant == "latent" else "state") and needs[1].kind == "paged"
        if variant == "latent":
            # a page of the shared group costs the latent row and layer 1's keys and values
            elem = 4 if dtype == "float32" else 2
            assert [p.name for p in needs[0].paged] == ["latent"] and runner.device_cache.layers[0].k is None
            assert runner.device_cache.layers[0].pages["latent"].shape[1:] == (8, cfg.latent)
            assert runner.page_bytes == {0: 8 * elem * (cfg.latent + 2 * cfg.head_dim)}
        if variant == "halfrot":
            position = runner.model.blocks[1].mixer.position
            assert type(position).__name__ == "HalfHeadRotary" and position.cos.shape[1] == cfg.head_dim // 4
        if variant == "interleaved":
            assert runner.model.blocks[1].mixer.position.pairing == "interleaved"
        if variant == "bias":
            assert weights["l1.attn.q_proj.bias"].shape == (cfg.heads * cfg.head_dim,)
            assert weights["l1.attn.o_proj.bias"].abs().max() > 0
            assert runner.params["layers.1.mixer.qkv_bias"].dtype == torch.float32
        if variant == "ends":
            assert type(runner.model.embed).__name__ == "ScaledEmbedding"
            assert type(runner.model.output).__name__ == "CappedOutput"
        if variant == "replay":
            states = runner.device_cache.layers[0].states
            assert set(states) == {"sum", "count"} and states["count"].dtype == torch.int32
            assert states["sum"].shape == (5, cfg.hidden) and runner.device_cache.layers[0].state is None
            assert runner.state_bytes == 5 * (cfg.hidden * 4 + 4)
        if variant == "routed":
            assert type(runner.model.blocks[0].feed_forward).__name__ == "RoutedFF"
            assert type(runner.model.blocks[1].feed_forward).__name__ == "SwiGLU"
            assert runner.model.blocks[0].mixer.position.table.shape == (128, cfg.hidden)
        if variant == "share":
            assert needs[2].share_with == 1 and not runner.device_cache.layers[2].owns_pages
            assert runner.device_cache.layers[2].k is runner.device_cache.layers[1].k
        if variant == "twice":
            assert len(runner.device_cache.layers) == 4
            assert runner.device_cache.layers[0].state is not runner.device_cache.layers[2].state
        reqs = {f"t{i}": random_tokens(n, cfg.vocab, 40 + i) for i, n in enumerate((19, 33, 7))}
        want = {rid: _toy_plain(weights, cfg, toks) for rid, toks in reqs.items()}
        # whole, then cut: portions and single tokens of the three requests interleaved
        for cut in ("whole", "cut"):
            got = {rid: [] for rid in reqs}
            if cut == "whole":
                for rid, toks in reqs.items():
                    got[rid].append(runner.step([StepEntry(rid, toks, list(range(len(toks))))]).cpu())
            else:
                done = {rid: 0 for rid in reqs}
                sizes = [5, 1, 2, 9, 1, 3]
                k = 0
                while any(done[r] < len(reqs[r]) for r in reqs):
                    entries = []
                    for rid, toks in reqs.items():
                        if done[rid] >= len(toks):
                            continue
                        n = min(sizes[k % len(sizes)], len(toks) - done[rid])
                        k += 1
                        entries.append(StepEntry(rid, toks[done[rid] : done[rid] + n], list(range(n))))
                        done[rid] += n
                    logits = runner.step(entries).cpu()
                    at = 0
                    for e in entries:
                        got[e.request_id].append(logits[at : at + len(e.tokens)])
                        at += len(e.tokens)
            if variant == "replay":
                counts = runner.device_cache.layers[0].states["count"].cpu()
                for rid, toks in reqs.items():
                    assert int(counts[runner.cache.slot_of(rid)]) == len(toks)
            for rid in reqs:
                if dtype == "float32":
                    torch.testing.assert_close(torch.cat(got[rid]), want[rid], rtol=2e-5, atol=3e-6)
                else:
                    parity.assert_bf16_close(torch.cat(got[rid]), want[rid], f"toy/{variant}/{cut}/{rid}")
                runner.finish(rid)  # the slot's state is cleared for whoever takes it next
        runner.cache.check_invariants()
    finally:
        _unregister_toys()


def test_toy_architecture_generates_through_the_entry_point(tmp_path):
    """The toy model under the scheduler, graphs and pipeline left at their defaults: the toy
    mixer walks host lists and does not declare itself replayable, so every step runs eagerly;
    slots (and with them the mixer's state) pass from finished requests to waiting ones."""
    from safetensors.torch import load_file

    from rapid_llm_amd import LLM, SamplingParams, write_random_model
    from rapid_llm_amd.config import register_architecture

    _toy_parts()
    register_architecture("ToyForCausalLM", ToyConfig, _toy_spec, replace=True)
    try:
        cfg = ToyConfig(hidden=48, vocab=97, heads=3, head_dim=16, inter=80, decay=0.8, period=9.0)
        folder = write_random_model(cfg.to_dict(), 5, tmp_path / "toy", dtype="float32")
        weights = {k: v.float() for k, v in load_file(str(folder / "model.safetensors")).items()}
        llm = LLM(str(folder), dtype="float32", max_seq_len=64, page_size=8, num_pages=24, max_num_seqs=2,
                  max_chunk_size=6, max_num_batched_tokens=16)
        runner = llm.scheduler.runner
        assert not runner.graphs_allowed and runner.engine.use_graph
        prompts = [random_tokens(n, cfg.vocab, 70 + i) for i, n in enumerate((9, 14, 3, 11, 6))]
        new = 7
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_gen_len=new))
        assert not runner._graphs
        for prompt, out in zip(prompts, outs):
            toks = list(prompt)
            for _ in range(new):
                toks.append(int(_toy_plain(weights, cfg, toks)[-1].argmax()))
            assert out.outputs[0].token_ids == toks[len(prompt):]
        runner.cache.check_invariants()
    finally:
        _unregister_toys()


def test_toy_parts_that_declare_themselves_replayable_run_from_graphs(tmp_path):
    """A toy mixer with two state tensors of its own that runs on the device alone, a toy
    embedding and a toy output projection, all declared replayable in this file: the model's
    decode steps are recorded and replayed under the scheduler and the pipeline, tokens fed from
    the device, and the tokens are the plain toy model's.  The mixer's launch data, kept in
    ``ctx.static``, is made once per recorded batch size and not again while recording."""
    from safetensors.torch import load_file

    from rapid_llm_amd import LLM, SamplingParams, write_random_model
    from rapid_llm_amd.config import register_architecture

    mixer_cls = _toy_parts()
    register_architecture("ToyForCausalLM", ToyConfig, _toy_spec, replace=True)
    try:
        cfg = ToyConfig(hidden=48, vocab=97, heads=3, head_dim=16, inter=80, decay=0.8, ends=True, replay=True)
        folder = write_random_model(cfg.to_dict(), 6, tmp_path / "toy", dtype="float32")
        weights = {k: v.float() for k, v in load_file(str(folder / "model.safetensors")).items()}
        llm = LLM(str(folder), dtype="float32", max_seq_len=64, page_size=8, num_pages=40, max_num_seqs=3,
                  max_chunk_size=6, max_num_batched_tokens=64)  # portions of 6: none of a single token
        runner = llm.scheduler.runner
        assert runner.graphs_allowed and llm.scheduler.pipeline
        prompts = [random_tokens(n, cfg.vocab, 90 + i) for i, n in enumerate((9, 14, 3, 11, 6))]
        new = 9
        mixer_cls.uploads = 0
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_gen_len=new))
        sizes = sorted({key[0] for key in runner._graphs})
        assert sizes and set(sizes) <= {1, 2, 4}, sizes
        # one upload per recorded batch size (in the eager run before the recording) and one per
        # eager decode step, of which there is none: every step of single tokens was replayed
        assert mixer_cls.uploads == len(runner._graphs)
        for prompt, out in zip(prompts, outs):
            toks = list(prompt)
            for _ in range(new):
                toks.append(int(_toy_plain(weights, cfg, toks)[-1].argmax()))
            assert out.outputs[0].token_ids == toks[len(prompt):]
        runner.cache.check_invariants()
    finally:
        _unregister_toys()


def test_unknown_part_kinds_are_named():
    from rapid_llm_amd.models import CausalLM, LayerSpec, ModelSpec, PartSpec

    norm = PartSpec("rmsnorm", {"size": 8, "eps": 1e-5, "checkpoint_name": "n"})
    from rapid_llm_amd.models import linear_output, token_embedding

    bad = ModelSpec(8, 10, (LayerSpec(PartSpec("no_such_mixer"), PartSpec("swiglu"), norm, norm),), norm,
                    token_embedding(10, 8, "e"), linear_output(10, 8, "o", False))
    with pytest.raises(ValueError, match="unknown mixer kind 'no_such_mixer'; known: .*gqa_attention"):
        CausalLM(bad)
