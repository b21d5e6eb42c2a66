"""Decode and prefill throughput of the engine on one MI355X, with the fraction of the roofline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--model-size 0.6b] [--batch 8] [--context 2048]

The default run has the layer sizes of Qwen3-0.6B (28 layers, hidden 1024, 16 query / 8 key heads
of 128, intermediate 3072, vocabulary 151936, tied head) with seeded random weights, bfloat16, a
batch of 8 requests each holding a 2,048-token context. A "step" is one decode step of the whole
batch: the engine's own step function, cache manager and sampler (greedy), from token ids to the
next token ids on the host. As in LLMEngine.step, a step is launched with its input tokens still on
the device while the host fetches the tokens of the step before (--no-run-ahead: one after the
other); all of them reach the host inside the timed span. One JSON line is printed:
  value        decoded tokens per second at the default batch
  prefill      one 2,048-token prompt in one step: tokens/s, ms, fraction of the bf16 MFMA peak
  roofline     bytes the decode step must read (every weight once + the live requests' cache) / time
  points       decode tokens/s at batch 1 and 64
  offline      the reference's offline workload (256 requests) through the scheduler: output tokens/s of the
               second of two passes, and of the first (--offline 0: skip); --mixed-lengths N: the same for N
               requests with nine short prompts to one long under a 2,048-token budget
Peaks: HBM 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s, fp32 157.3 TFLOP/s (MI355X, published).
"""
from __future__ import annotations

import argparse
import json
import sys
import time

HBM_PEAK = 8.0e12
FLOP_PEAK = {"bfloat16": 2.5e15, "float32": 157.3e12}

from mini_engine_amd.config.sizes import SIZES, model_config   # noqa: E402  (the named layer sizes)


def linear_params_per_layer(cfg) -> int:
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim * cfg.hidden_size
    o = cfg.num_attention_heads * cfg.head_dim * cfg.hidden_size
    return qkv + o + 3 * cfg.intermediate_size * cfg.hidden_size


def decode_bytes(cfg, item: int, contexts: list) -> int:
    """Bytes one decode step has to read: every weight it uses once, and the cache of the live requests."""
    weights = cfg.num_hidden_layers * linear_params_per_layer(cfg) + cfg.vocab_size * cfg.hidden_size   # head (tied or not)
    norms = cfg.num_hidden_layers * (2 * cfg.hidden_size + 2 * cfg.head_dim) + cfg.hidden_size
    kv = sum(contexts) * 2 * cfg.num_key_value_heads * cfg.head_dim * cfg.num_hidden_layers
    return weights * item + norms * 4 + kv * item


def prefill_flops(cfg, T: int) -> float:
    lin = 2.0 * T * cfg.num_hidden_layers * linear_params_per_layer(cfg)
    attn = 4.0 * cfg.num_attention_heads * cfg.head_dim * T * (T + 1) / 2 * cfg.num_hidden_layers
    head = 2.0 * cfg.vocab_size * cfg.hidden_size
    return lin + attn + head


class Bench:
    def __init__(self, cfg, dtype: str, page: int, max_batch: int, context: int, gen: int, seed: int = 0,
                 graphs: bool = True, min_pages: int = 0, max_len: int = 0, run_ahead: bool = True):
        import torch
        from mini_engine_amd.cache.manager import CacheManager
        from mini_engine_amd.engine.runner import ModelRunner
        from mini_engine_amd.registry import build_model
        from mini_engine_amd.weights.random_init import fill_random

        self.torch = torch
        self.cfg, self.page, self.context, self.gen = cfg, page, context, gen
        self.run_ahead = run_ahead
        self.dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
        self.max_len = max(context + gen + 64, max_len)
        t0 = time.time()
        self.model = fill_random(build_model(cfg), seed, "cuda", self.dtype, self.max_len)
        print(f"[bench] random weights ready in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)
        pages = max(max_batch * -(-self.max_len // page), min_pages)
        self.manager = CacheManager(pages, page, ModelRunner.windows_of(self.model), enable_prefix_caching=False)
        self.runner = ModelRunner(self.model, self.manager, self.dtype, "cuda", self.max_len, use_graphs=graphs)
        self.gen_ids = torch.Generator().manual_seed(seed)

    def _ids(self, n):
        return self.torch.randint(0, self.cfg.vocab_size, (n,), generator=self.gen_ids).tolist()

    def prefill(self, rid, n, want_last=True, ids=None):
        from mini_engine_amd.engine.runner import StepEntry
        assert self.manager.allocate(rid, 0, n)
        return self.runner.step([StepEntry(rid, ids if ids is not None else self._ids(n), 0, [n - 1] if want_last else [])])

    def time_prefill(self, T: int, reps: int = 3):
        torch = self.torch
        best = None
        for i in range(reps + 1):                          # the first run warms up
            ids = self._ids(T)                             # drawing the prompt is not the engine's work
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            self.prefill(("p", i), T, ids=ids)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            self.manager.free(("p", i))
            if i and (best is None or dt < best):
                best = dt
        return best

    def time_decode(self, batch: int, steps: int, warmup: int):
        """`batch` requests with `context` tokens each in the cache, then warmup + steps decode steps.

        With run_ahead (the engine's default way of decoding, LLMEngine.step) a step is launched with its
        tokens still on the device and the tokens of the step before are fetched behind it; every step's
        tokens reach the host inside the timed span, the last ones before the clock stops."""
        from mini_engine_amd.engine.runner import PENDING, StepEntry
        torch = self.torch
        reqs = [("d", batch, i) for i in range(batch)]
        last = []
        for r in reqs:                                     # real prefill, one request per step
            logits = self.prefill(r, self.context)
            last.append(int(self.runner.sample(logits, [0.0], [(0, 0)])[0]))
        pos = self.context
        temps, keys = [0.0] * batch, [(0, 0)] * batch
        ahead = self.run_ahead and self.runner.graphs is not None and self.runner.graphs.takes(batch)
        in_flight = None

        def one():
            nonlocal last, pos, in_flight
            entries = []
            for r, tok in zip(reqs, last):
                assert self.manager.allocate(r, pos, 1)
                entries.append(StepEntry(r, [PENDING if in_flight is not None else tok], pos, [0]))
            logits = self.runner.step(entries)
            if not ahead:
                last = self.runner.sample(logits, temps, keys)  # token ids on the host: the step is complete
            else:
                launched = self.runner.sample_async(logits, temps, keys, reqs)
                if in_flight is not None:
                    last = in_flight.tokens()              # the tokens of the step before, on the host
                in_flight = launched
            pos += 1

        def drain():
            nonlocal last, in_flight
            if in_flight is not None:
                last = in_flight.tokens()
                in_flight = None

        for _ in range(warmup):
            one()
        drain()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            one()
        drain()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ctx_mid = pos - steps / 2.0                        # mean context length over the timed steps
        for r in reqs:
            self.manager.free(r)
        return dt / steps, ctx_mid


    def offline(self, num_seqs: int, budget: int = 16384, max_model_len: int = 2048):
        """The reference's offline workload (its bench.py:38-48,60-66): `random.seed(0)`, prompts of 100-1024
        random ids below 10000, max_tokens 100-1024, temperature 0.6, ignore_eos, max_num_seqs 256,
        max_model_len 2048, chunked prefill under a 16k budget. Returns (sum of max_tokens / seconds, record)."""
        from random import randint, seed
        seed(0)
        prompts = [[randint(0, 10000) % self.cfg.vocab_size for _ in range(randint(100, 1024))] for _ in range(num_seqs)]
        max_tokens = [randint(100, 1024) for _ in range(num_seqs)]
        rate, record = self.serve(prompts, max_tokens, budget, max_model_len)
        record["reference_a100_tok_s"] = 4205.0
        return rate, record

    def mixed_lengths(self, num_seqs: int, budget: int = 2048, max_model_len: int = 8192):
        """Nine short prompts (128-512 tokens) to one long (4,096-7,680), 128-256 output tokens each, chunked
        prefill under a 2,048 budget: long prompts go through the cache in portions while the others decode
        beside them, so most steps are mixed ones. Same sampling and engine settings as `offline`."""
        from random import randint, random, seed
        seed(0)
        lengths = [randint(4096, 7680) if random() < 0.1 else randint(128, 512) for _ in range(num_seqs)]
        prompts = [[randint(0, 10000) % self.cfg.vocab_size for _ in range(n)] for n in lengths]
        max_tokens = [randint(128, 256) for _ in range(num_seqs)]
        rate, record = self.serve(prompts, max_tokens, budget, max_model_len)
        record["long_prompts"] = sum(n >= 4096 for n in lengths)
        return rate, record

    def serve(self, prompts, max_tokens, budget: int, max_model_len: int):
        """All requests handed to the engine at once (scheduler, sampler and step function as `LLM.generate`
        uses them; temperature 0.6, ignore_eos, at most 256 running). Returns (output tokens / second of the
        second of two passes, record with both)."""
        from types import SimpleNamespace
        from mini_engine_amd.engine.llm_engine import LLMEngine
        from mini_engine_amd.sampling.sampling_params import SamplingParams
        conf = SimpleNamespace(max_num_seqs=256, max_num_batched_tokens=budget, long_prefill_token_threshold=0,
                               enable_chunked_prefill=True, scheduling_policy="fcfs", eos=-1, max_model_len=max_model_len,
                               seed=0, run_ahead=self.run_ahead)
        llm = LLMEngine.from_parts(conf, self.model, self.manager, self.runner)
        sps = [SamplingParams(temperature=0.6, ignore_eos=True, max_tokens=m) for m in max_tokens]
        llm.generate([[1, 2, 3]], SamplingParams(max_tokens=4), use_tqdm=False)
        # The workload runs twice. The first pass, after the reference's one-prompt warm-up (its bench.py:62),
        # still meets every shape for the first time: decode graphs are captured, the library loads its
        # kernels and plans its products. The second pass is the engine in its steady state.
        took = []
        for _ in range(2):
            self.torch.cuda.synchronize()
            t0 = time.perf_counter()
            llm.generate(prompts, sps, use_tqdm=False)
            took.append(time.perf_counter() - t0)
        dt = took[1]
        total = sum(max_tokens)
        return total / dt, {"value": round(total / dt, 1), "unit": "output tokens/s", "seconds": round(dt, 2),
                            "first_pass_value": round(total / took[0], 1), "first_pass_seconds": round(took[0], 2),
                            "requests": len(prompts), "input_tokens": sum(len(p) for p in prompts), "output_tokens": total,
                            "budget": budget, "preemptions": llm.scheduler.num_preemptions}


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--model-size", default="0.6b", choices=sorted(SIZES))
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the size has (both numbers are reported)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048)
    ap.add_argument("--gen", type=int, default=256)
    ap.add_argument("--page", type=int, default=16)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--points", default="1,64", help="extra decode batch sizes, comma separated ('' for none)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--offline", type=int, default=256,
                    help="also run the reference's offline workload with this many requests (0: skip)")
    ap.add_argument("--mixed-lengths", type=int, default=0,
                    help="also run this many requests with nine short prompts to one long under a 2,048 budget (0: skip)")
    ap.add_argument("--no-graphs", action="store_true", help="launch decode kernels one by one instead of replaying HIP graphs")
    ap.add_argument("--no-run-ahead", action="store_true",
                    help="fetch every decode step's tokens before the next step is launched")
    args = ap.parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine runs on a single MI355X, --gpus {args.gpus} is not supported")
        return 2
    if args.steps + args.warmup > args.gen:
        args.gen = args.steps + args.warmup

    import torch
    cfg, full_layers = model_config(args.model_size, args.layers)
    points = [int(p) for p in args.points.split(",") if p]
    off_pages = args.offline * -(-2048 // args.page) if args.offline else 0
    if args.mixed_lengths:      # room for every request at its full length (a tenth of them long): no preemption
        off_pages = max(off_pages, args.mixed_lengths * -(-(768 + 8192 // 8) // args.page))
    bench = Bench(cfg, args.dtype, args.page, max([args.batch] + points), args.context, args.gen, args.seed,
                  graphs=not args.no_graphs, min_pages=off_pages, max_len=8192 if args.mixed_lengths else 2048 if args.offline else 0,
                  run_ahead=not args.no_run_ahead)
    item = 2 if args.dtype == "bfloat16" else 4

    T = args.prefill_tokens
    pre = bench.time_prefill(T)
    prefill = {"value": round(T / pre, 1), "tokens": T, "ms": round(pre * 1e3, 3),
               "frac": round(prefill_flops(cfg, T) / pre / FLOP_PEAK[args.dtype], 4)}
    print(f"[bench] prefill {T} tokens: {pre * 1e3:.2f} ms", file=sys.stderr, flush=True)

    step_s, ctx_mid = bench.time_decode(args.batch, args.steps, args.warmup)
    need = decode_bytes(cfg, item, [ctx_mid] * args.batch)
    roofline = {"bound": "hbm", "achieved": round(need / step_s / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                "frac": round(need / step_s / HBM_PEAK, 4)}
    print(f"[bench] decode batch {args.batch}: {step_s * 1e3:.3f} ms/step", file=sys.stderr, flush=True)
    pts = {}
    for b in points:
        s, _ = bench.time_decode(b, min(args.steps, 64), min(args.warmup, 8))
        pts[f"decode_b{b}"] = round(b / s, 1)
        print(f"[bench] decode batch {b}: {s * 1e3:.3f} ms/step", file=sys.stderr, flush=True)

    offline = None
    if args.offline:
        _, offline = bench.offline(args.offline)
        print(f"[bench] reference offline workload: {offline['value']} output tokens/s", file=sys.stderr, flush=True)

    mixed = None
    if args.mixed_lengths:
        _, mixed = bench.mixed_lengths(args.mixed_lengths)
        print(f"[bench] short and long prompts mixed: {mixed['value']} output tokens/s", file=sys.stderr, flush=True)

    line = {
        "metric": "decode tok/s at batch 1/8/64; prefill tok/s at 2,048 tokens; % roofline",
        "value": round(args.batch / step_s, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: seeded random token ids, seeded random weights",
        "config": {"model": f"Qwen3-{args.model_size} sizes", "layers": cfg.num_hidden_layers, "layers_of_model": full_layers,
                   "hidden": cfg.hidden_size, "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                   "tied": bool(cfg.tie_word_embeddings), "page": args.page, "global_batch": args.batch,
                   "seq_len": args.context, "gen": args.gen, "parallelism": "single GPU",
                   "hip_graphs": not args.no_graphs, "run_ahead": not args.no_run_ahead and not args.no_graphs},
        "prefill": prefill, "roofline": roofline, "points": pts,
    }
    if offline is not None:
        line["offline"] = offline
    if mixed is not None:
        line["mixed_lengths"] = mixed
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
