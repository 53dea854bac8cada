"""Command line: ``python -m rapid_llm_amd.cli <command> ...``

Options that the reference's command line has keep their spelling and meaning
(rapid_llm/cli.py:57-165): ``--model-dir`` (or the environment variable
``RAPID_LLM_MODEL_DIR``, :173-186), ``--max-seq-len``, ``--max-gpu-num-blocks``,
``--device``, ``--temperature``, ``--top-p``, ``--max-gen-len``, ``--repetition-penalty``,
``--cuda-graph/--no-cuda-graph``; ``batch`` adds ``--prompts-file``, ``--max-num-seqs``,
``--no-chat-template`` and ``--show-stats`` (:614-701).  Commands:

* ``batch``   run a file of prompts through the continuous-batching engine;
* ``chat``    a read-eval-print loop with streamed output (``/clear``, ``exit``);
* ``bench``   offline generation speed of a model folder with synthetic prompts of exact token
  lengths: TTFT, TPOT, TPS and TGS as the reference defines them (docs/benchmark_models.md:141-149);
* ``init``    write a model folder with random weights from a config.json and a seed;
* ``replay``  feed given token ids step by step and write logits (the same as ``bin/trace_run``).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path


def _common(sub: argparse.ArgumentParser, graph_default: bool) -> None:
    sub.add_argument("--model-dir", help="Checkpoint directory")
    sub.add_argument("--max-seq-len", type=int, default=2048)
    sub.add_argument("--max-gpu-num-blocks", type=int, default=None, help="Cache capacity in tokens")
    sub.add_argument("--device", default="cuda")
    sub.add_argument("--temperature", type=float, default=0.6)
    sub.add_argument("--top-p", type=float, default=0.9)
    sub.add_argument("--max-gen-len", type=int, default=None)
    sub.add_argument(
        "--repetition-penalty", type=float, default=1.1,
        help="Penalise logits of already-generated tokens (1.0 disables it)",
    )
    sub.add_argument(
        "--cuda-graph", action=argparse.BooleanOptionalAction, default=graph_default,
        help="Replay decode steps from captured HIP graphs (default: %(default)s)",
    )
    sub.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    sub.add_argument("--seed", type=int, default=0, help="Seed of the sampling streams")
    sub.add_argument("--load-format", default="auto", choices=["auto", "random"])


def _model_dir(args) -> str:
    model_dir = args.model_dir or os.getenv("RAPID_LLM_MODEL_DIR")
    if not model_dir:
        raise SystemExit("Model directory not provided. Pass --model-dir <path> or set RAPID_LLM_MODEL_DIR.")
    if not Path(model_dir).is_dir():
        raise SystemExit(f"model directory {model_dir!r} does not exist")
    return model_dir


def _sampling(args):
    from .sampling.params import SamplingParams

    return SamplingParams(
        temperature=args.temperature, top_p=args.top_p, max_gen_len=args.max_gen_len,
        repetition_penalty=args.repetition_penalty, stop_on_repeat=True,
    )


def _engine(args, max_num_seqs: int = 32):
    from .engine.llm import build_engine

    return build_engine(
        _model_dir(args), max_seq_len=args.max_seq_len, max_gpu_num_blocks=args.max_gpu_num_blocks,
        device=args.device, use_cuda_graph=args.cuda_graph, dtype=args.dtype,
        max_num_seqs=max_num_seqs, seed=args.seed, load_format=args.load_format,
    )


def _prompter(args, use_template: bool = True):
    """The model folder's chat template (rapid_llm/cli.py:650-652), or ``None``: a folder
    without one, or a base checkpoint, takes its prompts as they are."""
    from .engine.prompting import build_prompter, is_instruct

    model_dir = _model_dir(args)
    prompter = build_prompter(model_dir, use_template)
    if prompter is None and use_template and is_instruct(model_dir) and (Path(model_dir) / "tokenizer.json").is_file():
        print("the model folder has no chat template: prompts go in as they are", file=sys.stderr)
    return prompter


def _parse_prompt(line: str, engine, prompter=None):
    """A line of text, or a list of token ids written as ``[1, 2, 3]`` (models without a
    tokenizer)."""
    line = line.strip()
    if line.startswith("[") and line.endswith("]"):
        return [int(t) for t in json.loads(line)]
    if engine.tokenizer is None:
        raise SystemExit("the model folder has no tokenizer.json: give prompts as lists of token ids")
    return prompter.insert_prompt(line) if prompter is not None else line


def cmd_batch(args) -> int:
    engine = _engine(args, args.max_num_seqs)
    if args.prompts_file is None:
        if engine.tokenizer is None:
            lines = ["[1, 2, 3, 4, 5, 6, 7, 8]", "[9, 8, 7]", "[5, 5, 5, 5, 5, 5]", "[42]"]
        else:
            lines = [
                "Name the largest planet of the solar system.",
                "Write one sentence about rain.",
                "Count from one to five.",
                "What does a compiler do?",
            ]
    else:
        lines = [ln.strip() for ln in Path(args.prompts_file).read_text().splitlines() if ln.strip()]
        if not lines:
            raise SystemExit(f"{args.prompts_file!r} contains no prompts")
    params = _sampling(args)
    prompter = _prompter(args, not args.no_chat_template)
    started = time.perf_counter()
    requests = [engine.add_request(_parse_prompt(ln, engine, prompter), params) for ln in lines]
    engine.run_to_completion()
    elapsed = time.perf_counter() - started
    for index, request in enumerate(requests):
        print(f"--- [{index}] {request.finish_reason} ---")
        print(request.text.strip() if engine.tokenizer is not None else request.output_token_ids)
        print()
    if args.show_stats:
        generated = sum(len(r.output_token_ids) for r in requests)
        t0 = min(r.arrival_time for r in requests)
        ttfts = [(r.first_token_time - t0) * 1000 for r in requests if r.first_token_time is not None]
        print(f"{len(requests)} requests, {generated} tokens in {elapsed:.2f}s")
        print(f"throughput {generated / elapsed:7.1f} tok/s")
        if ttfts:
            print(f"TTFT mean {sum(ttfts) / len(ttfts):7.1f} ms | max {max(ttfts):7.1f} ms")
    return 0


def cmd_chat(args) -> int:
    engine = _engine(args, 1)
    params = _sampling(args)
    prompter = _prompter(args)
    messages: list[dict[str, str]] = []  # the conversation so far, formatted anew every turn
    history = ""  # without a template: the plain text so far
    print("Type a message; '/clear' forgets the conversation, 'exit' leaves.")
    while True:
        try:
            line = input("> ").strip()
        except EOFError:
            break
        if line in ("exit", "quit"):
            break
        if line == "/clear":
            history = ""
            messages = []
            continue
        if not line:
            continue
        prompt = _parse_prompt(line, engine)
        if isinstance(prompt, str):
            if prompter is not None:
                messages.append({"role": "user", "content": prompt})
                prompt = prompter.apply(messages)
            else:
                prompt = history + prompt
        request = engine.add_request(prompt, params)
        while engine.has_unfinished_requests():
            for r in engine.step():
                if r is request and r.delta:
                    print(r.delta, end="", flush=True)
        if engine.tokenizer is None:
            print(request.output_token_ids)
        else:
            print()
            if prompter is not None:
                messages.append({"role": "assistant", "content": request.text})
            else:
                history = prompt + request.text + "\n"
    return 0


def sample_prompt_lengths(count: int, low: int, high: int, seed: int) -> list[int]:
    """``count`` prompt lengths, uniform in ``[low, high]``, fixed by the seed (the reference
    draws ``[input_len * range_ratio, input_len]``, rapid_llm/benchmark/datasets/common.py:52-64)."""
    import random

    if not 1 <= low <= high:
        raise ValueError(f"prompt lengths must satisfy 1 <= low <= high, got {low} and {high}")
    rng = random.Random(seed)
    return [rng.randint(low, high) for _ in range(count)]


def measure_offline(engine, prompts, gen_len: int) -> dict:
    """All prompts submitted at once and run to completion, timed between device
    synchronisations (docs/benchmark_models.md:141-149): TTFT = time until every request has its
    first token, TPOT = (latency - TTFT) / (gen_len - 1), TPS = 1000 / TPOT per request,
    TGS = all output tokens / latency."""
    import torch

    from .sampling.params import SamplingParams

    params = SamplingParams(temperature=0.0, max_gen_len=gen_len, ignore_eos=True)
    before = engine.num_preemptions
    torch.cuda.synchronize()
    start = time.perf_counter()
    requests = [engine.add_request(p, params) for p in prompts]
    ttft = None
    steps = decode_steps = 0
    while engine.has_unfinished_requests():
        engine.step()
        steps += 1
        if ttft is None:
            if all(r.output_token_ids for r in requests):
                torch.cuda.synchronize()
                ttft = time.perf_counter() - start
        else:
            decode_steps += 1
    torch.cuda.synchronize()
    latency = time.perf_counter() - start
    tokens = sum(len(r.output_token_ids) for r in requests)
    return {
        "ttft_s": ttft, "latency_s": latency, "output_tokens": tokens, "steps": steps,
        "decode_steps": decode_steps, "prompt_tokens": sum(len(p) for p in prompts),
        "tpot_s": (latency - ttft) / max(1, gen_len - 1), "preemptions": engine.num_preemptions - before,
    }


def cmd_bench(args) -> int:
    """Offline generation speed with synthetic prompts: uniform random token ids of exactly
    ``--input-len`` tokens, or of lengths uniform in ``[--input-len-min, --input-len-max]``
    (equally ``[input_len * --range-ratio, input_len]``), as the reference's RandomDataset makes
    them (rapid_llm/benchmark/datasets/random.py:70-110)."""
    import random
    import statistics

    engine = _engine(args, args.batch_size)
    vocab = engine.runner.vocab_size
    rng = random.Random(args.seed)
    high = args.input_len_max if args.input_len_max is not None else args.input_len
    low = args.input_len_min if args.input_len_min is not None else max(1, int(high * args.range_ratio))
    rows = []
    for it in range(args.warmup + args.iterations):
        lengths = sample_prompt_lengths(args.batch_size, low, high, args.seed + it)
        prompts = [[rng.randrange(vocab) for _ in range(n)] for n in lengths]
        row = measure_offline(engine, prompts, args.gen_len)
        if it >= args.warmup:
            rows.append(row)
    ttft = statistics.median(r["ttft_s"] for r in rows)
    latency = statistics.median(r["latency_s"] for r in rows)
    tpot = statistics.median(r["tpot_s"] for r in rows)
    print(json.dumps({
        "batch_size": args.batch_size, "input_len_min": low, "input_len_max": high, "gen_len": args.gen_len,
        "ttft_s": round(ttft, 4), "tpot_ms": round(tpot * 1e3, 3),
        "tps": round(1.0 / tpot, 1) if tpot > 0 else None, "tgs": round(rows[0]["output_tokens"] / latency, 1),
        "prefill_tok_s": round(statistics.median(r["prompt_tokens"] / r["ttft_s"] for r in rows), 1),
        "preemptions": sum(r["preemptions"] for r in rows),
    }))
    if args.profile:
        # one more run of the same workload with every step eager and a pair of events around
        # every part: where the device's time goes, by part and by kind of step
        from .engine.timeline import Timeline, instrument

        timeline = Timeline()
        instrument(engine.runner, timeline)
        lengths = sample_prompt_lengths(args.batch_size, low, high, args.seed)
        measure_offline(engine, [[rng.randrange(vocab) for _ in range(n)] for n in lengths], args.gen_len)
        print(timeline.summary(), file=sys.stderr)
    return 0


def cmd_init(args) -> int:
    from .weights.random_init import write_random_model

    body = json.loads(Path(args.config).read_text())
    out = write_random_model(body, args.seed, args.out, dtype=args.dtype, norm_std=args.norm_std)
    print(out)
    return 0


def cmd_replay(args) -> int:
    from .engine.replay import build_replay_runner, run_trace

    runner = build_replay_runner(args.model, args.dtype, args.max_tokens)
    source = sys.stdin if args.trace in (None, "-") else open(args.trace)
    run_trace(runner, iter(source.readline, ""), args.out)
    return 0


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="rapid-llm", description=__doc__.split("\n\n")[0])
    subs = parser.add_subparsers(dest="command", required=True)

    batch = subs.add_parser("batch", help="Run a prompt file through the continuous-batching engine")
    _common(batch, graph_default=True)
    batch.add_argument("--prompts-file", help="One prompt per line: text, or a list of token ids")
    batch.add_argument("--max-num-seqs", type=int, default=32)
    batch.add_argument("--no-chat-template", action="store_true", help="Send prompts verbatim")
    batch.add_argument("--show-stats", action="store_true")
    batch.set_defaults(fn=cmd_batch)

    chat = subs.add_parser("chat", help="Interactive loop with streamed output")
    _common(chat, graph_default=False)
    chat.set_defaults(fn=cmd_chat)

    bench = subs.add_parser("bench", help="Offline generation speed with synthetic prompts")
    _common(bench, graph_default=True)
    bench.add_argument("--batch-size", type=int, default=8)
    bench.add_argument("--input-len", type=int, default=128)
    bench.add_argument("--input-len-min", type=int, default=None, help="shortest prompt (default: input-len * range-ratio)")
    bench.add_argument("--input-len-max", type=int, default=None, help="longest prompt (default: input-len)")
    bench.add_argument("--range-ratio", type=float, default=1.0,
                       help="prompt lengths are uniform in [input-len * ratio, input-len]; 1.0 pins them")
    bench.add_argument("--gen-len", type=int, default=128)
    bench.add_argument("--iterations", type=int, default=3)
    bench.add_argument("--warmup", type=int, default=1)
    bench.add_argument("--profile", action="store_true",
                       help="after the measurement, run the workload once more eagerly and print the "
                            "device time of every part (HIP events) to stderr")
    bench.set_defaults(fn=cmd_bench)

    init = subs.add_parser("init", help="Write a model folder with random weights")
    init.add_argument("--config", required=True, help="a config.json")
    init.add_argument("--out", required=True)
    init.add_argument("--seed", type=int, default=0)
    init.add_argument("--dtype", default=None, choices=["bfloat16", "float32"])
    init.add_argument("--norm-std", type=float, default=0.1)
    init.set_defaults(fn=cmd_init)

    replay = subs.add_parser("replay", help="Feed given tokens step by step and write logits")
    replay.add_argument("--model", required=True)
    replay.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    replay.add_argument("--out", required=True)
    replay.add_argument("--max-tokens", required=True, type=int)
    replay.add_argument("--trace", default="-", help="file of steps, one JSON object a line (default: stdin)")
    replay.set_defaults(fn=cmd_replay)

    args = parser.parse_args(argv)
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
