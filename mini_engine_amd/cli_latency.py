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


@dataclass(frozen=True)
class Setting:
    """How prompts enter the steps: whole prompts first (`pf`), or in portions beside the decoding requests
    under a budget of tokens a step (`c<tokens>`); reference bench_latency.py:41-51 names them so."""

    name: str
    chunked: bool
    budget: int

    @classmethod
    def parse(cls, name: str) -> "Setting":
        if name == "pf":
            return cls(name, False, ENGINE_BUDGET)
        if name[:1] == "c" and name[1:].isdigit() and 0 < int(name[1:]) <= ENGINE_BUDGET:
            return cls(name, True, int(name[1:]))
        raise ValueError(f"setting {name!r}: expected 'pf' or 'c<tokens>' with at most {ENGINE_BUDGET} tokens")

    def check(self, scheduler) -> None:
        if not self.chunked and self.budget < scheduler.max_model_len:
            raise ValueError(f"setting 'pf' needs a whole prompt in one step: max_model_len {scheduler.max_model_len} > {self.budget}")
        if self.budget < scheduler.max_live:
            raise ValueError(f"setting {self.name!r}: the budget must cover one token for each of {scheduler.max_live} requests")

    def switch(self, engine) -> None:
        """Put the engine's scheduler into this setting; what earlier settings left published in the cache is forgotten."""
        self.check(engine.scheduler)
        engine.scheduler.chunked = self.chunked
        engine.scheduler.token_budget = self.budget
        engine.manager.forget_prefixes()


class TokenTimes:
    """When every request came and when each of its tokens left the engine; the latency figures follow from that."""

    def __init__(self):
        self.came: dict = {}
        self.out: dict = {}
        self.long: set = set()

    def request(self, rid, at: float, is_long: bool) -> None:
        self.came[rid] = at
        self.out[rid] = []
        if is_long:
            self.long.add(rid)

    def tokens(self, rids, at: float) -> None:
        for rid in rids:
            self.out[rid].append(at)

    @staticmethod
    def _ms(values, q: float):
        import numpy as np
        return round(float(np.percentile(values, q)) * 1e3, 1) if len(values) else None

    def figures(self) -> dict:
        import numpy as np
        answered = {rid: ts for rid, ts in self.out.items() if ts}
        to_first = {rid: ts[0] - self.came[rid] for rid, ts in answered.items()}
        every = list(to_first.values())
        long = [t for rid, t in to_first.items() if rid in self.long]
        short = [t for rid, t in to_first.items() if rid not in self.long]
        streams = [np.asarray(ts) for ts in answered.values() if len(ts) > 1]
        between = np.concatenate([np.diff(ts) for ts in streams]) if streams else np.zeros(0)
        per_token = [float(ts[-1] - ts[0]) / (len(ts) - 1) for ts in streams]
        ms = self._ms
        return {
            "ttft_p50_ms": ms(every, 50), "ttft_p99_ms": ms(every, 99), "ttft_short_p99_ms": ms(short, 99),
            "ttft_long_p50_ms": ms(long, 50), "ttft_long_p99_ms": ms(long, 99),
            "itl_p50_ms": ms(between, 50), "itl_p99_ms": ms(between, 99), "itl_p999_ms": ms(between, 99.9),
            "itl_max_ms": ms(between, 100),
            "tpot_mean_ms": round(float(np.mean(per_token)) * 1e3, 1) if per_token else None,
            "output_tokens": sum(len(ts) for ts in self.out.values()), "num_long": len(long),
        }


def serve(engine, arrivals: list, sampling_params_of) -> dict:
    """Serves `arrivals` (sorted by time) in real time: a request enters the engine once its time has come, the
    engine steps whenever it holds a request, and sleeps until the next arrival when it holds none. Returns the
    latency figures of the run (the quantities of reference bench_latency.py:78-96)."""
    from collections import deque
    waiting = deque(arrivals)
    times = TokenTimes()
    evictions_at_start = engine.scheduler.num_preemptions
    steps = 0
    t0 = time.perf_counter()
    while True:
        elapsed = time.perf_counter() - t0
        while waiting and waiting[0].at <= elapsed:
            a = waiting.popleft()
            times.request(engine.add_request(a.prompt, sampling_params_of(a)), t0 + a.at, a.long)
        if not engine.is_finished():
            produced = engine.step()[3]
            steps += 1
            times.tokens(produced, time.perf_counter())
        elif waiting:
            pause = waiting[0].at - (time.perf_counter() - t0)
            if pause > 0:
                time.sleep(pause)
        else:
            break
    wall = time.perf_counter() - t0
    row = times.figures()
    row.update(out_tok_s=round(row["output_tokens"] / wall, 1), wall_s=round(wall, 1), steps=steps,
               preemptions=engine.scheduler.num_preemptions - evictions_at_start)
    return row


def sweep(engine, settings: list, rates: list, workload, num_reqs: int, sampling_params_of, emit) -> None:
    """Every setting at every rate, the same arrivals for all settings of a rate; `emit(rate, setting, figures)`
    takes each result as it is ready."""
    for rate in rates:
        arrivals = workload(num_reqs, rate)
        for setting in settings:
            setting.switch(engine)
            emit(rate, setting, serve(engine, arrivals, sampling_params_of))


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
    settings = [Setting.parse(name) for name in args.configs.split(",") if name]
    for setting in settings:
        setting.check(engine.scheduler)
    if int(7680 * args.scale) + int(256 * args.scale) > engine.scheduler.max_model_len:
        p.error(f"the longest request ({int(7680 * args.scale)} + {int(256 * args.scale)} tokens) exceeds "
                f"max_model_len {engine.scheduler.max_model_len}: lower --scale")
    workload = lambda num, rate: poisson_arrivals(num, rate, args.long_frac, vocab, args.scale)

    # before anything is measured: a short, dense run that meets the kernels, graphs and library plans (reference :99-100)
    sweep(engine, [Setting.parse("c2048")], [20.0], workload, 20, params_of, lambda *ignored: None)

    os.makedirs(os.path.dirname(args.out) or ".", exist_ok=True)
    about = {"model": args.random_weights or path, "dtype": args.dtype, "gpu": torch.cuda.get_device_name(0),
             "torch": torch.__version__}

    def emit(rate, setting, figures):
        row = {"engine": "mini_engine_amd", "label": args.label, "config": setting.name, "rate": rate,
               "num_reqs": args.num_reqs, "long_frac": args.long_frac, **figures, **about,
               "time": datetime.now().isoformat(timespec="seconds")}
        text = json.dumps(row)
        print(text, flush=True)
        with open(args.out, "a") as f:
            f.write(text + "\n")

    sweep(engine, settings, [float(r) for r in args.rates.split(",") if r], workload, args.num_reqs, params_of, emit)
    if tmp is not None:
        tmp.cleanup()
    return 0


if __name__ == "__main__":
    sys.exit(main())
