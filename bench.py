"""Decode and prefill throughput of the engine on one MI355X, with the fraction of the roofline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--model-size 0.6b | --model DIR] [--batch 8] [--context 2048]

The default run has the layer sizes of Qwen3-0.6B (28 layers, hidden 1024, 16 query / 8 key heads
of 128, intermediate 3072, vocabulary 151936, tied head) with seeded random weights, bfloat16, a
batch of 8 requests each holding a 2,048-token context. Everything measured goes through the engine's
entry point: a model folder is written, `LLM(folder, ...)` loads it and sizes its cache pool, requests
are added with `add_request` and run with `step` (scheduler, step function, cache manager, sampler,
decode graphs, steps launched one ahead: what `generate` uses). A "step" is one decode step of the whole
batch; every step's tokens reach the host inside the timed span. One JSON line is printed:
  value        decoded tokens per second at the default batch
  prefill      one 2,048-token prompt in one step: tokens/s, ms, fraction of the bf16 MFMA peak
  roofline     bytes the decode step must read (every weight once + the live requests' cache) / time
  points       decode tokens/s at batch 1 and 64
  8b           the same figures at the Qwen3-8B layer sizes, with the offline workload in it (random weights drawn on
               the device; --second-size '' skips)
  32b          at the Qwen3-32B layer sizes: decode at batch 8, and --third-mixed N requests with nine short prompts
               to one long under a 2,048-token budget, one pass (--third-size '' skips)
  offline      the reference's offline workload (256 requests) through `generate`: output tokens/s of the
               second of two passes, and of the first (--offline 0: skip); --mixed-lengths N: the same for N
               requests with nine short prompts to one long under a 2,048-token budget
`--model DIR` measures the model of a folder (its config.json; its model.safetensors if there is one, else random
weights drawn on the device) in place of a named size. Bytes and flops are counted from the model's declared
parameters, its run order and what its mixers keep per token, not from a configuration's field names.
Peaks: HBM 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s, fp32 157.3 TFLOP/s (MI355X, published).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile
import time

HBM_PEAK = 8.0e12
FLOP_PEAK = {"bfloat16": 2.5e15, "float32": 157.3e12}

from mini_engine_amd.config.sizes import SIZES, model_config   # noqa: E402  (the named layer sizes)


def log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


_ITEM = {"compute": None, "float32": 4, "int32": 4, "stored": None, "bfloat16": 2}


def _spec_bytes(spec, item: int) -> int:
    n = 1
    for d in spec.shape:
        n *= int(d)
    return n * (_ITEM.get(spec.dtype) or item)


def _used_per_call(model) -> dict:
    """How often each layer runs in a step (a run order may name a layer twice)."""
    runs: dict = {}
    for call in model.order:
        runs[call.layer] = runs.get(call.layer, 0) + 1
    return runs


def _matrix_params(model) -> tuple:
    """(matrix elements multiplied per token in the layers, counting a layer once per run; elements of the head's matrix)."""
    runs = _used_per_call(model)
    tied = getattr(model.head, "tied_to", None) is model.embedding
    per_token = head = 0
    for name, _, _, spec in model.named_specs():
        if len(spec.shape) < 2:
            continue
        n = 1
        for d in spec.shape:
            n *= int(d)
        if name.startswith("layers."):
            per_token += n * runs.get(int(name.split(".")[1]), 0)
        elif name.startswith("head.") or (tied and name.startswith("embedding.")):
            head += n
    return per_token, head


def cache_bytes_per_token(model, page: int, dtype) -> list:
    """Per page group: (bytes one cached token costs over all layer calls of the group, the group's window or None)."""
    from mini_engine_amd.cache.pool import page_bytes
    plan = model.cache_plan()
    return [(b / page, need.window) for b, need in zip(page_bytes(plan, page, dtype), plan.group_needs)]


def decode_bytes(model, item: int, contexts: list, page: int, dtype) -> int:
    """Bytes one decode step has to read: every parameter it uses once (the embedding matrix only where it is the
    head's matrix as well: a step gathers a row per request from it), and what the cache holds of the live requests
    (a windowed group at most its window)."""
    tied = getattr(model.head, "tied_to", None) is model.embedding
    weights = sum(_spec_bytes(spec, item) for name, _, _, spec in model.named_specs()
                  if tied or not name.startswith("embedding."))
    kv = 0.0
    for per_token, window in cache_bytes_per_token(model, page, dtype):
        kv += per_token * sum(min(c, window) if window else c for c in contexts)
    return int(weights + kv)


def prefill_flops(model, T: int) -> float:
    """Multiply-adds x 2 of a prompt of T tokens in one step: every matrix of the layers for every token, the scores
    and the weighted sums of every attention call over the keys each token sees, the head for the one row that
    wants logits."""
    per_token, head = _matrix_params(model)
    attn = 0.0
    for call in model.order:
        mixer = getattr(model.layers[call.layer], "mixer", None)
        heads, size = getattr(mixer, "num_heads", None), getattr(mixer, "head_dim", None)
        if heads and size:
            window = getattr(mixer, "window", None)
            seen = sum(min(t + 1, window) if window else t + 1 for t in range(T)) if window else T * (T + 1) / 2
            attn += 4.0 * heads * size * seen
    return 2.0 * T * per_token + attn + 2.0 * head


class Bench:
    """An engine built by `LLM(folder)` and the workloads run on it."""

    def __init__(self, cfg, folder: str, dtype: str, page: int, max_seqs: int, max_len: int, budget: int, seed: int,
                 graphs: bool, run_ahead: bool, random_weights: int | None, kv_blocks: int = -1):
        import torch
        from mini_engine_amd import LLM

        self.torch, self.cfg = torch, cfg
        t0 = time.time()
        self.llm = LLM(folder, dtype=dtype, kvcache_block_size=page, max_num_seqs=max_seqs, max_model_len=max_len,
                       max_num_batched_tokens=budget, seed=seed, use_graphs=graphs, run_ahead=run_ahead,
                       random_weights=random_weights, eos=-1, num_kvcache_blocks=kv_blocks)
        log(f"engine ready in {time.time() - t0:.1f}s: {self.llm.config.num_kvcache_blocks} pages of {page} tokens, "
            f"{self.llm.reserved_bytes >> 20} MiB kept free for the steps' working set")
        self.ids = torch.Generator().manual_seed(seed)

    def _prompt(self, n: int) -> list:
        return self.torch.randint(0, self.cfg.vocab_size, (n,), generator=self.ids).tolist()

    def _drain(self) -> None:
        while not self.llm.is_finished():
            self.llm.step()

    def time_prefill(self, T: int, reps: int = 3, warm: int = 6) -> float:
        """One prompt of T tokens, one generated token: add_request + step, best of `reps` after `warm` untimed runs
        (a step whose shape keeps coming up is replayed as a graph from its sixth appearance on: the steady state
        of a server that is handed prompts of one length)."""
        from mini_engine_amd import SamplingParams
        torch, best = self.torch, None
        for i in range(warm + reps):
            prompt = self._prompt(T)                       # drawing the prompt is not the engine's work
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            self.llm.add_request(prompt, SamplingParams(temperature=0, max_tokens=1, ignore_eos=True))
            finished, num_prefill, _, _ = self.llm.step()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            assert num_prefill == T and len(finished) == 1, "the prompt did not run as one step"
            if i >= warm and (best is None or dt < best):
                best = dt
        return best

    def time_decode(self, batch: int, context: int, steps: int, warmup: int):
        """`batch` requests of `context` prompt tokens each; once all decode, `warmup` untimed steps, then
        `steps` timed ones. Returns (seconds per step, mean context length over the timed steps)."""
        from mini_engine_amd import SamplingParams
        torch, llm = self.torch, self.llm
        slack = 16 + batch * context // max(1, llm.scheduler.token_budget)     # requests admitted early decode while others go in
        sp = SamplingParams(temperature=0, max_tokens=warmup + steps + slack, ignore_eos=True)
        for _ in range(batch):
            llm.add_request(self._prompt(context), sp)
        while True:                                         # prompts go in under the token budget
            _, num_prefill, num_decode, _ = llm.step()
            if num_prefill == 0 and num_decode == batch and not llm.scheduler.waiting:
                break
        for _ in range(warmup):
            llm.step()
        torch.cuda.synchronize()
        live = llm.scheduler.running
        first_ctx = sum(r.in_cache for r in live) / len(live) + 1     # keys a request reads in the first timed step
        t0 = time.perf_counter()
        for _ in range(steps):
            _, num_prefill, num_decode, got = llm.step()
            assert num_prefill == 0 and num_decode == batch and len(got) == batch
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        self._drain()
        return dt / steps, first_ctx + (steps - 1) / 2.0

    def offline(self, num_seqs: int, passes: int = 2):
        """The reference's offline workload (its bench.py:38-48,60-66): `random.seed(0)`, prompts of 100-1024
        random ids below 10000, max_tokens 100-1024, temperature 0.6, ignore_eos, chunked prefill under the
        engine's budget. Returns the record."""
        from random import randint, seed
        seed(0)
        prompts = [[randint(0, 10000) % self.cfg.vocab_size for _ in range(randint(100, 1024))] for _ in range(num_seqs)]
        max_tokens = [randint(100, 1024) for _ in range(num_seqs)]
        record = self.serve(prompts, max_tokens, passes)
        record["reference_a100_tok_s"] = 4205.0
        return record

    def mixed_lengths(self, num_seqs: int, passes: int = 2):
        """Nine short prompts (128-512 tokens) to one long (4,096-7,680), 128-256 output tokens each: long
        prompts go through the cache in portions while the others decode beside them, so most steps are mixed."""
        from random import randint, random, seed
        seed(0)
        lengths = [randint(4096, 7680) if random() < 0.1 else randint(128, 512) for _ in range(num_seqs)]
        prompts = [[randint(0, 10000) % self.cfg.vocab_size for _ in range(n)] for n in lengths]
        max_tokens = [randint(128, 256) for _ in range(num_seqs)]
        record = self.serve(prompts, max_tokens, passes)
        record["long_prompts"] = sum(n >= 4096 for n in lengths)
        return record

    def serve(self, prompts, max_tokens, passes: int = 2):
        """All requests handed to `generate` at once (temperature 0.6, ignore_eos). The workload runs twice: the
        first pass, after the reference's one-prompt warm-up (its bench.py:62), still meets every shape for the
        first time (decode graphs are captured, the library plans its products); the second is the steady state.
        With `passes` 1 the one pass is both."""
        from mini_engine_amd import SamplingParams
        llm = self.llm
        sps = [SamplingParams(temperature=0.6, ignore_eos=True, max_tokens=m) for m in max_tokens]
        llm.generate([[1, 2, 3]], SamplingParams(max_tokens=4), use_tqdm=False)
        took = []
        for _ in range(passes):
            llm.manager.forget_prefixes()                  # the second pass must not find the first one's pages
            self.torch.cuda.synchronize()
            t0 = time.perf_counter()
            llm.generate(prompts, sps, use_tqdm=False)
            took.append(time.perf_counter() - t0)
        total = sum(max_tokens)
        return {"value": round(total / took[-1], 1), "unit": "output tokens/s", "seconds": round(took[-1], 2), "passes": passes,
                "first_pass_value": round(total / took[0], 1), "first_pass_seconds": round(took[0], 2),
                "requests": len(prompts), "input_tokens": sum(len(p) for p in prompts), "output_tokens": total,
                "budget": llm.scheduler.token_budget, "preemptions": llm.scheduler.num_preemptions}


def folder_for(cfg, seed: int, root: str, on_device: bool) -> tuple:
    """(model folder, random_weights option). on_device: the folder holds config.json only and the engine draws
    the weights where they live; otherwise config.json and model.safetensors are written and loaded."""
    from mini_engine_amd.weights.random_init import write_random_model
    os.makedirs(root, exist_ok=True)
    if on_device:
        with open(os.path.join(root, "config.json"), "w") as f:
            json.dump(cfg.to_dict(), f)
        return root, seed
    t0 = time.time()
    write_random_model(cfg, seed, root)
    log(f"model folder written in {time.time() - t0:.1f}s")
    return root, None


def box_rates() -> dict:
    """What this GPU reaches on the plainest work of each kind, beside the published peaks that the fractions are
    taken of: a device copy of 1 GiB (bytes read + written), one-row products over four weights of 201 MB in turn
    (bytes read; the engine's own streaming kernel at the 8B sizes' largest product), and a library product of
    8192^3 in bfloat16."""
    import torch
    from mini_engine_amd.kernels import ops
    dev = torch.device("cuda")

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps

    a = torch.empty(1 << 29, dtype=torch.bfloat16, device=dev).normal_()
    b = torch.empty_like(a)
    copy = timed(lambda: b.copy_(a), 10)
    del b
    size = 24576 * 4096
    weights, row = [a[i * size:(i + 1) * size].view(24576, 4096) for i in range(4)], a[4 * size:4 * size + 4096].view(1, 4096)

    def stream():
        for weight in weights:
            ops.linear(row, weight)

    read = timed(stream, 5)
    del a, weights, row
    x = torch.randn(8192, 8192, device=dev).bfloat16()
    w = torch.randn(8192, 8192, device=dev).bfloat16()
    mm = timed(lambda: ops.library_product(x, w, torch.bfloat16), 10)
    del x, w
    torch.cuda.empty_cache()
    return {"hbm_copy_GBs": round(2 * (1 << 30) / copy / 1e9, 1), "hbm_read_GBs": round(4 * size * 2 / read / 1e9, 1),
            "library_product_bf16_TFLOPs": round(2 * 8192 ** 3 / mm / 1e12, 1)}


def resolve_model(args, size: str, layers, tmp: str) -> tuple:
    """(typed configuration, layers the full model has, label, folder, random_weights option, how the weights came)
    for a named size, or for `--model DIR` (size is then the folder)."""
    from mini_engine_amd.config.model_config import load_model_config
    from mini_engine_amd.registry import build_model
    from mini_engine_amd.weights.loader import checkpoint_files
    if os.path.isdir(size):
        cfg = load_model_config(size)
        label = os.path.basename(os.path.normpath(size))
        full = getattr(cfg, "num_hidden_layers", None)
        if checkpoint_files(size):
            return cfg, full, label, size, None, "the folder's checkpoint"
        return cfg, full, label, size, args.seed, "drawn on the device"
    cfg, full = model_config(size, layers)
    skeleton = build_model(cfg)                              # declared parameters only, no tensors
    params = sum(_spec_bytes(spec, 1) for _, _, _, spec in skeleton.named_specs())
    on_device = args.weights == "device" or (args.weights == "auto" and params > 2e9)
    folder, random_weights = folder_for(cfg, args.seed, os.path.join(tmp, size), on_device)
    return cfg, full, f"Qwen3-{size} sizes", folder, random_weights, "drawn on the device" if on_device else "written folder"


def describe(cfg, label: str, full_layers) -> dict:
    """The sizes of a model as flat keys."""
    get = lambda name: getattr(cfg, name, None)
    return {"model": label, "layers": get("num_hidden_layers"), "layers_of_model": full_layers, "hidden": get("hidden_size"),
            "q_heads": get("num_attention_heads"), "kv_heads": get("num_key_value_heads"), "head_dim": get("head_dim"),
            "intermediate": get("intermediate_size"), "vocab": get("vocab_size"), "tied": bool(get("tie_word_embeddings"))}


def measure(args, size: str, layers, tmp: str, batches: list, steps: int, warmup: int, prefill: bool = True,
            offline: int = 0, mixed: int = 0, serve_passes: int = 2) -> dict:
    """Prefill, decode at `batches` (the first is the headline batch), and the served workloads, at one model."""
    import torch
    cfg, full_layers, label, folder, random_weights, how = resolve_model(args, size, layers, tmp)
    gen = max(args.gen, steps + warmup + 2)
    max_len = max(args.context + gen + 128, args.prefill_tokens + 128, 4096, 8192 if mixed else 0)
    max_seqs = max(batches + ([256] if (offline or mixed) else []))
    budget = max(args.prefill_tokens, 2048 if mixed else 16384, max_seqs)
    bench = Bench(cfg, folder, args.dtype, args.page, max_seqs, max_len, budget, args.seed, not args.no_graphs,
                  not args.no_run_ahead, random_weights, args.kv_blocks)
    model = bench.llm.model
    item = 2 if args.dtype == "bfloat16" else 4
    dtype = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    out = {"cfg": cfg, "full_layers": full_layers, "label": label, "weights": how}

    if prefill:
        T = args.prefill_tokens
        pre = bench.time_prefill(T)
        out["prefill"] = {"value": round(T / pre, 1), "tokens": T, "ms": round(pre * 1e3, 3),
                          "frac": round(prefill_flops(model, T) / pre / FLOP_PEAK[args.dtype], 4)}
        log(f"{label}: prefill {T} tokens: {pre * 1e3:.2f} ms")

    out["decode"] = {}
    for b in batches:
        k, w = (steps, warmup) if b == batches[0] else (min(steps, 64), min(warmup, 8))
        step_s, ctx = bench.time_decode(b, args.context, k, w)
        need = decode_bytes(model, item, [ctx] * b, args.page, dtype)
        out["decode"][b] = {"step_s": step_s, "tok_s": round(b / step_s, 1), "hbm_frac": round(need / step_s / HBM_PEAK, 4),
                            "gbps": round(need / step_s / 1e9, 1)}
        log(f"{label}: decode batch {b}: {step_s * 1e3:.3f} ms/step, {need / step_s / HBM_PEAK:.1%} of HBM")
    if offline:
        out["offline"] = bench.offline(offline, serve_passes)
        log(f"{label}: reference offline workload: {out['offline']['value']} output tokens/s")
    if mixed:
        out["mixed_lengths"] = bench.mixed_lengths(mixed, serve_passes)
        log(f"{label}: short and long prompts mixed: {out['mixed_lengths']['value']} output tokens/s")
    del bench, model
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    return out


def other_size(run: dict, context: int) -> dict:
    """A further model's figures as one flat object."""
    obj = describe(run["cfg"], run["label"], run["full_layers"])
    obj.update(weights=run["weights"], seq_len=context)
    if "prefill" in run:
        obj["prefill"] = run["prefill"]
    for b, d in run["decode"].items():
        obj[f"decode_b{b}"] = d["tok_s"]
        obj[f"decode_b{b}_ms"] = round(d["step_s"] * 1e3, 4)
        obj[f"decode_b{b}_hbm_frac"] = d["hbm_frac"]
    for name in ("offline", "mixed_lengths"):
        if name in run:
            obj[name] = run[name]
    return obj


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--model-size", default="0.6b", choices=sorted(SIZES))
    ap.add_argument("--model", default=None, metavar="DIR",
                    help="measure the model of this folder instead of a named size: its config.json, and its "
                         "model.safetensors if it has one (random weights drawn on the device otherwise)")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the size has (both numbers are reported)")
    ap.add_argument("--second-size", default="8b", help="a second size whose figures go into an object of its own ('' for none)")
    ap.add_argument("--second-layers", type=int, default=None)
    ap.add_argument("--third-size", default="32b", help="a third size: decode at the default batch and the mixed-lengths workload ('' for none)")
    ap.add_argument("--third-mixed", type=int, default=128, help="requests of the third size's mixed-lengths workload (0: skip)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048)
    ap.add_argument("--gen", type=int, default=256)
    ap.add_argument("--page", type=int, default=16)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--points", default="1,64", help="extra decode batch sizes, comma separated ('' for none)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--weights", default="auto", choices=["auto", "folder", "device"],
                    help="folder: write model.safetensors and load it; device: draw the weights on the GPU; "
                         "auto: a folder up to 2 G parameters, the device beyond")
    ap.add_argument("--offline", type=int, default=256,
                    help="also run the reference's offline workload with this many requests, at the first and the second size (0: skip)")
    ap.add_argument("--mixed-lengths", type=int, default=0,
                    help="also run this many requests with nine short prompts to one long under a 2,048 budget (0: skip)")
    ap.add_argument("--kv-blocks", type=int, default=-1,
                    help="pages of the cache pool (-1: sized by the engine from a measured warm-up, as a user's engine is)")
    ap.add_argument("--no-graphs", action="store_true", help="launch decode kernels one by one instead of replaying HIP graphs")
    ap.add_argument("--no-run-ahead", action="store_true",
                    help="fetch every decode step's tokens before the next step is launched")
    args = ap.parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine runs on a single MI355X, --gpus {args.gpus} is not supported")
        return 2

    points = [int(p) for p in args.points.split(",") if p and int(p) != args.batch]
    first = args.model if args.model else args.model_size
    with tempfile.TemporaryDirectory() as tmp:
        main_run = measure(args, first, args.layers, tmp, [args.batch] + points, args.steps, args.warmup,
                           offline=args.offline, mixed=args.mixed_lengths)
        others = {}
        if args.second_size and args.second_size != first:
            others[args.second_size] = measure(args, args.second_size, args.second_layers, tmp, [args.batch] + points,
                                               min(args.steps, 32), min(args.warmup, 4), offline=args.offline)
        if args.third_size and args.third_size not in (first, args.second_size) and args.dtype == "bfloat16":
            others[args.third_size] = measure(args, args.third_size, None, tmp, [args.batch], min(args.steps, 16),
                                              min(args.warmup, 2), prefill=False, mixed=args.third_mixed, serve_passes=1)

    head = main_run["decode"][args.batch]
    config = describe(main_run["cfg"], main_run["label"], main_run["full_layers"])
    config.update(page=args.page, global_batch=args.batch, seq_len=args.context, gen=args.gen, parallelism="single GPU",
                  hip_graphs=not args.no_graphs, run_ahead=not args.no_run_ahead and not args.no_graphs,
                  entry="LLM.add_request/step")
    line = {
        "metric": "decode tok/s at batch 1/8/64; prefill tok/s at 2,048 tokens; % roofline",
        "value": head["tok_s"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(head["step_s"] * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": f"synthetic: seeded random token ids, seeded random weights ({main_run['weights']})",
        "config": config,
        "prefill": main_run["prefill"],
        "roofline": {"bound": "hbm", "achieved": head["gbps"], "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": head["hbm_frac"]},
        "points": {f"decode_b{b}": main_run["decode"][b]["tok_s"] for b in points},
    }
    for name, run in others.items():
        line[name] = other_size(run, args.context)
    for name in ("offline", "mixed_lengths"):
        if name in main_run:
            line[name] = main_run[name]
    if args.dtype == "bfloat16":
        line["box"] = box_rates()
        log(f"this GPU: {line['box']}")
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
