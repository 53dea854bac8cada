"""Decode and prefill speed of the engine on one MI355X, random weights, synthetic token ids.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--dtype bfloat16]
                    [--shape NAME] [--batch B] [--prompt-len T] [--context C]
    python bench.py --workload qwen3-0.6b-256 | qwen3-32b-32

A "step" is one decode step of the whole batch through the engine's step function and the
greedy sampling kernel, tokens fed back.  The default run has the layer sizes of
Qwen3-8B (BASELINE.json ``configs[2]``), a batch of 8, every request with a 2,048-token
prompt, context 4,096.  One JSON line is printed: decoded tokens a second (``value``), the
2,048-token prefill (``prefill``), the decode step against the HBM roofline (``roofline``)
and decoding at batch 1 and 64 (``points``, which also holds the true 32-bit path's decode
and prefill speed, measured in a second process).  ``--shape``, ``--prompt-len`` and
``--context`` measure the same at other sizes of the model family and other lengths; the
line then names them in ``metric`` and ``config``.

``points`` also holds the two scheduler workloads of BASELINE.json (``configs[3]``: the
Qwen3-0.6B shape, 256 requests at once, prompts uniform in 64 to 1,024 tokens, 128 tokens each;
``configs[4]``: the Qwen3-32B shape, 32 requests, prompts uniform in 4,096 to 16,384, context
16,384, cache pages from the memory that is free, 128 tokens each): time per output token,
generated tokens a second and the decode step's share of the HBM roofline, each measured in a
process of its own through the continuous-batching scheduler (``--workload NAME`` runs one
alone; ``--no-workloads`` leaves them out).

Metric definitions follow rapid_llm's docs/benchmark_models.md:141-149: decode tok/s is
batch / mean step time; prefill tok/s is prompt tokens / prefill latency; both timed
between device synchronisations after warm-up.
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_GBPS = 8000.0
PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}


def load_shape() -> dict:
    """Layer sizes of BASELINE.json configs[2], parsed from its text."""
    import re

    with open(os.path.join(ROOT, "BASELINE.json")) as fh:
        text = json.load(fh)["configs"][2]

    def num(pattern: str) -> int:
        m = re.search(pattern, text)
        if m is None:
            raise SystemExit(f"BASELINE.json configs[2] does not state {pattern!r}")
        return int(m.group(1).replace(",", ""))

    theta = re.search(r"rope_theta ([0-9.e+]+)", text).group(1)
    eps = re.search(r"rms_norm_eps ([0-9.e+-]+)", text).group(1)
    return dict(
        architectures=["Qwen3ForCausalLM"],
        model_type="qwen3",
        num_hidden_layers=num(r"(\d+) layers"),
        hidden_size=num(r"hidden (\d+)"),
        num_attention_heads=num(r"(\d+) query heads"),
        num_key_value_heads=num(r"(\d+) KV heads"),
        head_dim=num(r"head_dim (\d+)"),
        intermediate_size=num(r"intermediate (\d+)"),
        vocab_size=num(r"vocab (\d+)"),
        rope_theta=float(theta),
        rms_norm_eps=float(eps),
        tie_word_embeddings="untied" not in text,
        max_position_embeddings=40960,
        context=num(r"context (\d+)"),
        prompt_len=num(r"one ([\d,]+)-token prompt"),
    )


# Other members of the model family (layer sizes as their model cards give them), for
# measurements beside the default run's.
FAMILY = {
    "qwen3-0.6b": dict(num_hidden_layers=28, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8,
                       intermediate_size=3072, tie_word_embeddings=True),
    "qwen3-1.7b": dict(num_hidden_layers=28, hidden_size=2048, num_attention_heads=16, num_key_value_heads=8,
                       intermediate_size=6144, tie_word_embeddings=True),
    "qwen3-4b": dict(num_hidden_layers=36, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8,
                     intermediate_size=9728, tie_word_embeddings=True),
    "qwen3-14b": dict(num_hidden_layers=40, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                      intermediate_size=17408, tie_word_embeddings=False),
    "qwen3-32b": dict(num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8,
                      intermediate_size=25600, tie_word_embeddings=False),
}


def weight_bytes(cfg, elem: int) -> int:
    h, i = cfg.hidden_size, cfg.intermediate_size
    per_layer = (cfg.q_size + 2 * cfg.kv_size) * h + h * cfg.q_size + 2 * i * h + h * i
    return (per_layer * cfg.num_hidden_layers + cfg.vocab_size * h) * elem


def kv_bytes_per_token(cfg, elem: int) -> int:
    return 2 * cfg.kv_size * cfg.num_hidden_layers * elem


def prefill_flops(cfg, tokens: int) -> float:
    h, i = cfg.hidden_size, cfg.intermediate_size
    per_layer = (cfg.q_size + 2 * cfg.kv_size) * h + h * cfg.q_size + 2 * i * h + h * i
    linear = 2.0 * tokens * per_layer * cfg.num_hidden_layers + 2.0 * cfg.vocab_size * h  # one logits row
    attn = 2.0 * 2.0 * cfg.q_size * (tokens * (tokens + 1) / 2) * cfg.num_hidden_layers  # causal QK^T and PV
    return linear + attn


def measured_peaks() -> int:
    """Practical peaks of this device, beside the published ones the fractions are quoted
    against: a 4 GiB read by a plain streaming kernel, a 2 GiB library copy, and the library's square
    products of 8,192."""
    import torch

    def timed(fn, n=10) -> float:
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t) / n

    from rapid_llm_amd.kernels import ops

    out = {}
    x = torch.ones(1 << 31, dtype=torch.bfloat16, device="cuda")  # 4 GiB
    out["read_gbps"] = round(
        max(x.numel() * 2 / timed(lambda: ops.read_buffer(x, blocks)) for blocks in (1024, 2048, 4096, 8192, 32768)) / 1e9, 1
    )
    half = x[: 1 << 30]
    y = torch.empty_like(half)
    out["copy_gbps_read_plus_write"] = round(2 * half.numel() * 2 / timed(lambda: y.copy_(half)) / 1e9, 1)
    del x, y, half
    n = 8192
    for name, dtype in (("bf16", torch.bfloat16), ("fp32", torch.float32)):
        a = torch.randn(n, n, device="cuda", dtype=dtype)
        b = torch.randn(n, n, device="cuda", dtype=dtype)
        torch.backends.cuda.matmul.allow_tf32 = False
        out[f"gemm_{name}_tflops"] = round(2 * n**3 / timed(lambda: torch.matmul(a, b.t())) / 1e12, 1)
    # What a kernel of a decode step can hope for: plain reads of the sizes of a layer's four
    # weight matrices (Qwen3-8B: 34, 50, 100 and 201 MB) and of 400 MB, forty in a row replayed
    # from a graph, every one over memory that no earlier one touched.  Microseconds a kernel;
    # the rate is what a product of that size can reach at most, start and end included.
    pool = torch.ones(1 << 30, dtype=torch.bfloat16, device="cuda")  # 2 GiB
    chain = {}
    for mb in (34, 50, 100, 201, 400):
        n = int(mb * 1e6 / 2)
        views = [pool[i * n : (i + 1) * n] for i in range(pool.numel() // n)]
        best = None
        for blocks in (256, 512, 2048):
            graph = torch.cuda.CUDAGraph()
            ops.read_buffer(views[0], blocks)
            torch.cuda.synchronize()
            with torch.cuda.graph(graph):
                for i in range(40):
                    ops.read_buffer(views[i % len(views)], blocks)
            sec = timed(graph.replay, 5) / 40
            best = sec if best is None else min(best, sec)
        chain[f"{mb}MB"] = {"us": round(best * 1e6, 1), "gbps": round(mb * 1e6 / best / 1e9, 1)}
    out["read_chain"] = chain
    out["published"] = {"hbm_gbps": HBM_GBPS, "bf16_tflops": PEAK_TFLOPS["bfloat16"], "fp32_tflops": PEAK_TFLOPS["float32"]}
    print(json.dumps(out), flush=True)
    return 0


# The scheduler workloads of BASELINE.json configs[3] and configs[4].
WORKLOADS = {
    "qwen3-0.6b-256": dict(shape="qwen3-0.6b", requests=256, low=64, high=1024, gen=128, context=2048, key="w06b",
                           passes=2),
    # one pass: its 300,000 prompt tokens take 25 s, and recording the decode graphs in the
    # first steps changes the mean of 127 steps by under 1%
    "qwen3-32b-32": dict(shape="qwen3-32b", requests=32, low=4096, high=16384, gen=128, context=16384 + 128, key="w32b",
                         passes=1),
}


def run_workload(name: str, seed: int = 1234) -> int:
    """One workload through the scheduler; prints one JSON line of its own."""
    import torch

    from rapid_llm_amd.cli import measure_offline, sample_prompt_lengths
    from rapid_llm_amd.engine.llm import build_engine

    w = WORKLOADS[name]
    shape = load_shape()
    shape.pop("context"), shape.pop("prompt_len")
    shape.update(FAMILY[w["shape"]])
    t0 = time.time()
    engine = build_engine(
        shape, load_format="random", dtype="bfloat16", max_seq_len=w["context"], max_num_seqs=w["requests"],
        max_num_batched_tokens=8192, max_chunk_size=8192, page_size=16, seed=seed,
    )
    cfg = engine.runner.config
    torch.cuda.synchronize()
    print(f"[bench] {name}: model ready in {time.time() - t0:.1f} s, "
          f"{engine.cache.capacity_tokens()} tokens of cache", file=sys.stderr, flush=True)
    gen = torch.Generator().manual_seed(seed)
    rows = []
    for it in range(w["passes"]):  # with two, the first records the graphs and warms the allocator
        lengths = sample_prompt_lengths(w["requests"], w["low"], w["high"], seed + it)
        prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist() for n in lengths]
        row = measure_offline(engine, prompts, w["gen"])
        row["mean_prompt"] = sum(lengths) / len(lengths)
        rows.append(row)
        print(f"[bench] {name} pass {it}: {row}", file=sys.stderr, flush=True)
    row = rows[-1]
    tpot = row["tpot_s"]
    mean_ctx = row["mean_prompt"] + w["gen"] / 2.0
    step_bytes = weight_bytes(cfg, 2) + w["requests"] * mean_ctx * kv_bytes_per_token(cfg, 2)
    k = w["key"]
    print(json.dumps({
        f"{k}_tpot_ms": round(tpot * 1e3, 3),
        f"{k}_decode_tok_s": round(w["requests"] / tpot, 1),
        f"{k}_tok_s": round(row["output_tokens"] / row["latency_s"], 1),
        f"{k}_prefill_tok_s": round(row["prompt_tokens"] / row["ttft_s"], 1),
        f"{k}_hbm_frac": round(step_bytes / tpot / 1e9 / HBM_GBPS, 4),
        f"{k}_preemptions": row["preemptions"],
    }), flush=True)
    return 0


def workload_points(names) -> dict:
    """Each workload in a process of its own (the 32B shape needs the whole device)."""
    import subprocess

    out = {}
    for name in names:
        try:
            done = subprocess.run(
                [sys.executable, os.path.abspath(__file__), "--workload", name], capture_output=True, text=True, timeout=900
            )
            out.update(json.loads(done.stdout.strip().splitlines()[-1]))
            print(f"[bench] workload {name}: {done.stdout.strip().splitlines()[-1]}", file=sys.stderr, flush=True)
        except Exception as err:  # the main line must not be lost to a workload
            tail = "" if "done" not in locals() else done.stderr[-800:]
            print(f"[bench] workload {name} gave no result: {err!r} {tail}", file=sys.stderr, flush=True)
    return out


def float32_points(args) -> dict:
    """The same model through the true 32-bit path, in a process of its own (the float32
    weights need their own 33 GB): decode tok/s at the main batch size and prefill tok/s."""
    import subprocess

    cmd = [
        sys.executable, os.path.abspath(__file__), "--dtype", "float32", "--batch", str(args.batch),
        "--steps", "16", "--warmup", "4", "--points", "",
    ]
    if args.layers is not None:
        cmd += ["--layers", str(args.layers)]
    cmd += ["--shape", args.shape]
    if args.prompt_len is not None:
        cmd += ["--prompt-len", str(args.prompt_len)]
    if args.context is not None:
        cmd += ["--context", str(args.context)]
    try:
        done = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        line = json.loads(done.stdout.strip().splitlines()[-1])
        out = {f"fp32_decode_b{args.batch}": line["value"]}
        if line.get("prefill"):
            out["fp32_prefill"] = line["prefill"]["value"]
        print(f"[bench] float32 path: {out}", file=sys.stderr, flush=True)
        return out
    except Exception as err:  # the main line must not be lost to the float32 run
        print(f"[bench] the float32 run gave no result: {err!r}", file=sys.stderr, flush=True)
        return {}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256,
                    help="timed decode steps (BASELINE.json's decode workload: 256 tokens a request)")
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--shape", default="qwen3-8b", choices=["qwen3-8b", *FAMILY],
                    help="layer sizes: qwen3-8b is BASELINE.json configs[2], the others its family's")
    ap.add_argument("--prompt-len", type=int, default=None, help="tokens of every prompt (default 2,048)")
    ap.add_argument("--context", type=int, default=None, help="longest sequence the engine is sized for")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--points", default="1,64", help="other decode batch sizes to measure ('' for none)")
    ap.add_argument("--point-steps", type=int, default=64)
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-pipeline", action="store_true", help="read every step's tokens before queueing the next")
    ap.add_argument("--no-fp32", action="store_true", help="skip the float32 points (a second process)")
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOADS),
                    help="run one scheduler workload of BASELINE.json alone and print its own line")
    ap.add_argument("--no-workloads", action="store_true", help="skip the scheduler workloads (processes of their own)")
    ap.add_argument("--peaks", action="store_true",
                    help="measure what the device reaches with library kernels (a large read, copy and square products) and exit")
    args = ap.parse_args()
    if args.peaks:
        return measured_peaks()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU engine")
        return 2
    if args.workload is not None:
        return run_workload(args.workload)

    import torch

    from rapid_llm_amd import EngineConfig, ModelRunner, StepEntry
    from rapid_llm_amd.engine.feed import fed_token
    from rapid_llm_amd.engine.llm import GpuExecutor
    from rapid_llm_amd.engine.scheduler import SamplingPlan
    from rapid_llm_amd.sampling.sampler import RowSampling, Sampler

    shape = load_shape()
    context, prompt_len = shape.pop("context"), shape.pop("prompt_len")
    if args.shape != "qwen3-8b":
        shape.update(FAMILY[args.shape])
    if args.prompt_len is not None:
        prompt_len = args.prompt_len
        context = max(context, prompt_len + 2048)
    if args.context is not None:
        context = args.context
    room = max(args.steps + args.warmup, args.point_steps + max(2, args.warmup // 2)) + 2
    if prompt_len < 1 or prompt_len + room > context:
        print(f"a prompt of {prompt_len} tokens and {room} decoded ones do not fit a context of {context}")
        return 2
    full_layers = shape["num_hidden_layers"]
    if args.layers is not None:
        shape["num_hidden_layers"] = args.layers
    points = [int(p) for p in args.points.split(",") if p]
    elem = 2 if args.dtype == "bfloat16" else 4

    # batch sizes whose caches do not fit beside the weights are left out, and said so: the
    # pool is made for the largest batch that is measured
    from rapid_llm_amd.config.registry import config_from_dict

    _, sized = config_from_dict(shape)
    per_request = (-(-(prompt_len + room) // 16)) * 16 * kv_bytes_per_token(sized, elem)
    free, _ = torch.cuda.mem_get_info()
    most = int((0.92 * free - weight_bytes(sized, elem)) // per_request)
    if args.batch > most:
        print(f"a batch of {args.batch} requests of {prompt_len + room} tokens does not fit this device "
              f"beside the weights ({most} do)")
        return 2
    for b in [b for b in points if b > most]:
        print(f"[bench] batch {b} left out: {most} requests of {prompt_len + room} tokens fit beside the weights",
              file=sys.stderr, flush=True)
    points = [b for b in points if b <= most]
    max_batch = max([args.batch] + points)

    engine = EngineConfig(
        dtype=args.dtype,
        max_seq_len=context,
        page_size=16,
        num_pages=max_batch * (-(-(prompt_len + room) // 16)) + 1,
        max_num_seqs=max_batch,
        max_num_batched_tokens=8192,
        use_graph=not args.no_graph,
        seed=1234,
    )
    t0 = time.time()
    runner = ModelRunner(shape, engine, load_format="random")
    cfg = runner.config
    torch.cuda.synchronize()
    print(f"[bench] model ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    gen = torch.Generator().manual_seed(7)
    vocab = cfg.vocab_size

    def prompt() -> list[int]:
        return torch.randint(0, vocab, (prompt_len,), generator=gen).tolist()

    def portions(rid: str, toks: list[int]) -> list[StepEntry]:
        """The prompt as the steps that run it: whole if the step's token budget holds it, else
        in portions of that budget; the last one asks for the logits of its last token."""
        budget = engine.max_num_batched_tokens
        cuts = [toks[lo : lo + budget] for lo in range(0, len(toks), budget)]
        return [StepEntry(rid, part, [len(part) - 1] if i == len(cuts) - 1 else []) for i, part in enumerate(cuts)]

    # ---- prefill of one prompt (2,048 tokens unless asked otherwise) ----------
    prefill = None
    if not args.no_prefill:
        times = []
        for i in range(4):
            cuts = portions("p", prompt())
            torch.cuda.synchronize()
            t = time.perf_counter()
            for entry in cuts:
                runner.step([entry])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            runner.finish("p")
        sec = statistics.median(times[1:])
        flops = prefill_flops(cfg, prompt_len)
        prefill = {
            "value": round(prompt_len / sec, 1),
            "tokens": prompt_len,
            "ms": round(sec * 1e3, 3),
            "frac": round(flops / sec / (PEAK_TFLOPS[args.dtype] * 1e12), 4),
        }
        print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)

    # ---- decode ----------------------------------------------------------------
    executor = GpuExecutor(runner, Sampler(runner.device))

    def greedy(rows: int) -> SamplingPlan:
        return SamplingPlan(
            rows=[RowSampling() for _ in range(rows)], logits_rows=list(range(rows)), logprob_ks=[None] * rows
        )

    def decode(batch: int, steps: int, warmup: int) -> tuple[float, float]:
        """Mean seconds per decode step and the mean context length over the timed steps.
        A step is what the engine's loop does for one token of every request: queue the
        forward pass and the choice of the tokens, read the chosen tokens back.  Pipelined
        (the engine's default), the next step is queued, fed from the device, before the
        last one's tokens are read."""
        ids = [f"d{i}" for i in range(batch)]
        tokens = []
        for rid in ids:  # prompts, one request a step
            cuts = portions(rid, prompt())
            for entry in cuts[:-1]:
                executor.execute([entry], greedy(0))
            tokens += executor.execute([cuts[-1]], greedy(1)).token_ids
        plan = greedy(batch)
        fed = [StepEntry(rid, [fed_token(i)], [0]) for i, rid in enumerate(ids)]
        inflight = executor.launch([StepEntry(rid, [tok], [0]) for rid, tok in zip(ids, tokens)], plan)

        def one_step():
            nonlocal inflight
            if args.no_pipeline:
                tokens = inflight.result().token_ids  # the step's one host synchronisation
                inflight = executor.launch([StepEntry(rid, [tok], [0]) for rid, tok in zip(ids, tokens)], plan)
            else:
                queued = executor.launch(fed, plan)
                inflight.result()
                inflight = queued

        for _ in range(warmup):
            one_step()
        inflight.result()
        torch.cuda.synchronize()
        ctx_start = runner.tokens_cached(ids[0]) - 1  # one step is in flight
        t = time.perf_counter()
        for _ in range(steps):
            one_step()
        inflight.result()
        torch.cuda.synchronize()
        sec = (time.perf_counter() - t) / steps
        mean_ctx = ctx_start + (steps - 1) / 2.0 + 1
        for rid in ids:
            runner.finish(rid)
        return sec, mean_ctx

    model_name = "Qwen3-" + args.shape.split("-")[1].upper()
    sec, mean_ctx = decode(args.batch, args.steps, args.warmup)
    step_bytes = weight_bytes(cfg, elem) + args.batch * mean_ctx * kv_bytes_per_token(cfg, elem)
    achieved = step_bytes / sec / 1e9
    result = {
        "metric": f"{model_name} {'bf16' if args.dtype == 'bfloat16' else 'fp32'} decode tok/s (batch {args.batch}, "
                  f"{prompt_len}-token prompts); prefill tok/s at {prompt_len} tokens",
        "value": round(args.batch / sec, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic (uniform random token ids, random N(0,0.02) weights, norm weights 1)",
        "config": {
            "model": f"{model_name} shape",
            "layers": cfg.num_hidden_layers,
            "layers_full": full_layers,
            "hidden": cfg.hidden_size,
            "q_heads": cfg.num_attention_heads,
            "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "intermediate": cfg.intermediate_size,
            "vocab": cfg.vocab_size,
            "rope_theta": cfg.rope_theta,
            "rms_norm_eps": cfg.rms_norm_eps,
            "tied": cfg.tie_word_embeddings,
            "global_batch": args.batch,
            "seq_len": prompt_len,
            "context": context,
            "page_size": engine.page_size,
            "graph": engine.use_graph,
            "pipeline": not args.no_pipeline,
            "parallelism": "single GPU",
        },
        "prefill": prefill,
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_GBPS, 4),
        },
    }
    pts = {}
    for b in points:
        s, _ = decode(b, args.point_steps, max(2, args.warmup // 2))
        pts[f"decode_b{b}"] = round(b / s, 2)
        print(f"[bench] decode batch {b}: {pts[f'decode_b{b}']} tok/s", file=sys.stderr, flush=True)
    if args.dtype == "bfloat16" and not args.no_fp32 and points:
        pts.update(float32_points(args))
    default_run = args.shape == "qwen3-8b" and args.layers is None and args.prompt_len is None and args.context is None
    if args.dtype == "bfloat16" and not args.no_workloads and points and default_run:
        del runner, executor  # the workloads need the device's memory
        torch.cuda.empty_cache()
        pts.update(workload_points(sorted(WORKLOADS)))
    result["points"] = pts
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
