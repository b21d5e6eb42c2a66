"""Latency under load from the command line, in the manner of the reference's bench_latency.py:8-118.

    python -m mini_engine_amd.cli_latency --model DIR [--num-reqs 240] [--rates 4,8]
                                          [--configs pf,c512,c1024,c2048,c4096,c8192] [--long-frac 0.1]
                                          [--out results/latency.jsonl] [--label NAME]
    python -m mini_engine_amd.cli_latency --random-weights 0.6b ...      (no model folder at hand)

Requests arrive as a Poisson process of `rate` per second (seeded by the rate, so every setting sees
the same arrivals); a share `--long-frac` of them has a long prompt (4,096-7,680 random ids), the rest
a short one (128-512), each wants 128-256 tokens at temperature 0.6 without an end token (reference
bench_latency.py:28-38). For every rate, every setting in --configs serves that workload on one engine
(max_num_seqs 128, max_model_len 8192; reference :98): `pf` is prefill-first with a 16,384 budget, `cN`
is chunked prefill with a budget of N tokens (reference :41-51). Published prefixes are forgotten between
settings, so none starts with another's cache. One JSON row per (rate, setting) is printed and appended
to --out: time to the first token (all, short, long prompts), time between tokens (p50, p99, p99.9,
max), mean time per output token, output tokens a second, steps, preemptions.

Options the reference has keep its names and meanings: --model, --num-reqs, --rates, --configs,
--long-frac, --out, --label. Not taken over: --attn (this engine has one attention path).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile
import time
from dataclasses import dataclass
from datetime import datetime
from random import Random

ENGINE_BUDGET = 16384           # the most any setting asks for; buffers are sized for it once


@dataclass
class Arrival:
    at: float                   # seconds after the start
    prompt: list
    max_tokens: int
    long: bool


def poisson_arrivals(num: int, rate: float, long_frac: float, vocab: int, scale: float = 1.0) -> list:
    """The reference's workload (bench_latency.py:28-38): exponential gaps of mean 1/rate, a long prompt
    with probability long_frac, ids below 10,000 (folded into a smaller vocabulary). `scale` shrinks
    every length, for a model whose max_model_len is short."""
    rng = Random(int(rate * 1000))
    sized = lambda n: max(1, int(n * scale))
    out, clock = [], 0.0
    for _ in range(num):
        clock += rng.expovariate(rate)
        is_long = rng.random() < long_frac
        length = sized(rng.randint(4096, 7680) if is_long else rng.randint(128, 512))
        ids = [rng.randint(0, 10000) % vocab for _ in range(length)]
        out.append(Arrival(clock, ids, sized(rng.randint(128, 256)), is_long))
    return out


def apply_setting(engine, name: str) -> None:
    """`pf`: whole prompts first, 16,384 tokens a step. `c<N>`: chunked prefill under N tokens a step."""
    sched = engine.scheduler
    if name == "pf":
        sched.chunked, sched.token_budget = False, ENGINE_BUDGET
    elif name.startswith("c") and name[1:].isdigit() and 0 < int(name[1:]) <= ENGINE_BUDGET:
        sched.chunked, sched.token_budget = True, int(name[1:])
    else:
        raise ValueError(f"setting {name!r}: expected 'pf' or 'c<tokens>' with at most {ENGINE_BUDGET} tokens")
    if name == "pf" and ENGINE_BUDGET < sched.max_model_len:
        raise ValueError(f"setting 'pf' needs a whole prompt in one step: max_model_len {sched.max_model_len} > {ENGINE_BUDGET}")
    if sched.token_budget < sched.max_live:
        raise ValueError(f"setting {name!r}: the budget must cover one token for each of {sched.max_live} requests")
    engine.manager.forget_prefixes()


def percentile_ms(values, q: float):
    import numpy as np
    return round(float(np.percentile(values, q)) * 1e3, 1) if len(values) else None


def serve(engine, arrivals: list, sampling_params_of) -> dict:
    """Feeds the arrivals at their times, steps the engine in between, and notes when each request's
    tokens come out (reference bench_latency.py:54-96)."""
    import numpy as np
    preempted_before = engine.scheduler.num_preemptions
    due, stamps, came, is_long = 0, {}, {}, {}
    steps = 0
    start = time.perf_counter()
    while due < len(arrivals) or not engine.is_finished():
        now = time.perf_counter() - start
        while due < len(arrivals) and arrivals[due].at <= now:
            a = arrivals[due]
            rid = engine.add_request(a.prompt, sampling_params_of(a))
            came[rid], stamps[rid], is_long[rid] = start + a.at, [], a.long
            due += 1
        if engine.is_finished():                                   # idle until the next arrival
            time.sleep(max(0.0, arrivals[due].at - (time.perf_counter() - start)))
            continue
        _, _, _, emitted = engine.step()
        steps += 1
        t = time.perf_counter()
        for rid in emitted:
            stamps[rid].append(t)
    wall = time.perf_counter() - start

    first = {rid: ts[0] - came[rid] for rid, ts in stamps.items() if ts}
    gaps = np.concatenate([np.diff(ts) for ts in stamps.values() if len(ts) > 1] or [np.zeros(0)])
    per_token = [(ts[-1] - ts[0]) / (len(ts) - 1) for ts in stamps.values() if len(ts) > 1]
    ttft_all = list(first.values())
    ttft_long = [v for rid, v in first.items() if is_long[rid]]
    ttft_short = [v for rid, v in first.items() if not is_long[rid]]
    return {
        "ttft_p50_ms": percentile_ms(ttft_all, 50), "ttft_p99_ms": percentile_ms(ttft_all, 99),
        "ttft_short_p99_ms": percentile_ms(ttft_short, 99),
        "ttft_long_p50_ms": percentile_ms(ttft_long, 50), "ttft_long_p99_ms": percentile_ms(ttft_long, 99),
        "itl_p50_ms": percentile_ms(gaps, 50), "itl_p99_ms": percentile_ms(gaps, 99),
        "itl_p999_ms": percentile_ms(gaps, 99.9),
        "itl_max_ms": round(float(gaps.max()) * 1e3, 1) if len(gaps) else None,
        "tpot_mean_ms": round(float(np.mean(per_token)) * 1e3, 1) if per_token else None,
        "output_tokens": sum(len(ts) for ts in stamps.values()),
        "out_tok_s": round(sum(len(ts) for ts in stamps.values()) / wall, 1), "wall_s": round(wall, 1), "steps": steps,
        "preemptions": engine.scheduler.num_preemptions - preempted_before, "num_long": len(ttft_long),
    }


def main(argv=None) -> int:
    p = argparse.ArgumentParser(prog="python -m mini_engine_amd.cli_latency", description=__doc__,
                                formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("--model", default=None, help="folder with config.json and *.safetensors")
    p.add_argument("--random-weights", default=None, metavar="SIZE",
                   help="write a model folder of this size (tinyA, 0.6b, 8b, 32b) with seeded random weights and use it")
    p.add_argument("--num-reqs", type=int, default=240)
    p.add_argument("--rates", default="4,8", help="arrival rates in requests a second, comma separated")
    p.add_argument("--configs", default="pf,c512,c1024,c2048,c4096,c8192")
    p.add_argument("--long-frac", type=float, default=0.1)
    p.add_argument("--out", default="results/latency.jsonl")
    p.add_argument("--label", default="")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--seed", type=int, default=0, help="seed of the sampler's noise and of random weights")
    p.add_argument("--max-model-len", type=int, default=8192)
    p.add_argument("--max-num-seqs", type=int, default=128)
    p.add_argument("--scale", type=float, default=1.0,
                   help="multiplies every prompt and output length (a tiny model with a short max_model_len)")
    args = p.parse_args(argv)
    if (args.model is None) == (args.random_weights is None):
        p.error("give exactly one of --model and --random-weights")

    import torch
    from . import LLM, SamplingParams

    tmp = None
    path = args.model
    if args.random_weights:
        from .config.sizes import SIZES, model_config
        from .weights.random_init import write_random_model
        if args.random_weights not in SIZES:
            p.error(f"--random-weights must be one of {sorted(SIZES)}")
        tmp = tempfile.TemporaryDirectory()
        cfg, _ = model_config(args.random_weights, None)
        path = write_random_model(cfg, args.seed, tmp.name)
    path = os.path.expanduser(path)

    engine = LLM(path, max_num_seqs=args.max_num_seqs, max_model_len=args.max_model_len,
                 max_num_batched_tokens=ENGINE_BUDGET, dtype=args.dtype, seed=args.seed)
    vocab = engine.model.embedding.vocab_size
    params_of = lambda a: SamplingParams(temperature=0.6, ignore_eos=True, max_tokens=a.max_tokens)
    settings = [s for s in args.configs.split(",") if s]
    if int(7680 * args.scale) + int(256 * args.scale) > engine.scheduler.max_model_len:
        p.error(f"the longest request ({int(7680 * args.scale)} + {int(256 * args.scale)} tokens) exceeds "
                f"max_model_len {engine.scheduler.max_model_len}: lower --scale")
    workload = lambda num, rate: poisson_arrivals(num, rate, args.long_frac, vocab, args.scale)

    apply_setting(engine, "c2048")                   # warm-up: kernels, graphs and library plans
    serve(engine, workload(20, 20.0), params_of)

    os.makedirs(os.path.dirname(args.out) or ".", exist_ok=True)
    for rate in (float(r) for r in args.rates.split(",") if r):
        arrivals = workload(args.num_reqs, rate)
        for name in settings:
            apply_setting(engine, name)
            row = {"engine": "mini_engine_amd", "label": args.label, "config": name, "rate": rate,
                   "num_reqs": args.num_reqs, "long_frac": args.long_frac, **serve(engine, arrivals, params_of),
                   "model": args.random_weights or path, "dtype": args.dtype, "gpu": torch.cuda.get_device_name(0),
                   "torch": torch.__version__, "time": datetime.now().isoformat(timespec="seconds")}
            print(json.dumps(row), flush=True)
            with open(args.out, "a") as f:
                f.write(json.dumps(row) + "\n")
    if tmp is not None:
        tmp.cleanup()
    return 0


if __name__ == "__main__":
    sys.exit(main())
