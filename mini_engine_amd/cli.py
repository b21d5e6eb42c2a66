"""Offline throughput from the command line, in the manner of the reference's bench.py:8-90.

    python -m mini_engine_amd.cli --model DIR [--num-seqs 256] [--chunked 1] [--budget 16384]
                                  [--threshold 0] [--out results/bench.jsonl] [--label NAME]
    python -m mini_engine_amd.cli --random-weights 0.6b ...      (no model folder at hand)

Options the reference has keep its names and meanings: --model, --num-seqs, --out, --label,
--chunked (1 = chunked prefill, 0 = prefill-first), --budget (max_num_batched_tokens),
--threshold (long_prefill_token_threshold). The workload is the reference's (bench.py:38-48,60-66):
`random.seed(0)`, prompts of 100-1024 random ids below 10000, max_tokens 100-1024, temperature 0.6,
ignore_eos, max_num_seqs 256, max_model_len 2048, one warm-up generate; the figure is the sum of
max_tokens over the wall time. One JSON row is printed and appended to --out.

With --prompts FILE the workload is the file's instead: one request a line, either a JSON list of token
ids or an object {"prompt": [ids], "max_tokens": n, "temperature": t} (missing fields: --max-output and
--temperature). --tokens-out FILE writes what was generated, one JSON list of token ids a line in the order
of the prompts ("-": standard output, before the row). Ids in, ids out: a model folder needs no tokenizer.
Not taken over: --engine (other engines), --attn unified (this engine has one attention path),
--expect-gpu.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile
import time
from datetime import datetime
from random import randint, seed


def main(argv=None) -> int:
    p = argparse.ArgumentParser(prog="python -m mini_engine_amd.cli", description=__doc__,
                                formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("--model", default=None, help="folder with config.json and *.safetensors")
    p.add_argument("--random-weights", default=None, metavar="SIZE",
                   help="write a model folder of this size (tinyA, 0.6b, 8b, 32b) with seeded random weights and use it")
    p.add_argument("--num-seqs", type=int, default=256)
    p.add_argument("--out", default="results/bench.jsonl")
    p.add_argument("--label", default="")
    p.add_argument("--chunked", type=int, default=1)
    p.add_argument("--budget", type=int, default=16384)
    p.add_argument("--threshold", type=int, default=0)
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--seed", type=int, default=0, help="seed of the sampler's noise and of random weights")
    p.add_argument("--max-model-len", type=int, default=2048)
    p.add_argument("--max-num-seqs", type=int, default=256)
    p.add_argument("--block-size", type=int, default=16, help="kvcache_block_size")
    p.add_argument("--policy", default="fcfs", choices=["fcfs", "priority"])
    p.add_argument("--max-prompt", type=int, default=1024)
    p.add_argument("--max-output", type=int, default=1024)
    p.add_argument("--device", default="cuda")
    p.add_argument("--num-kv-blocks", type=int, default=-1, help="num_kvcache_blocks (-1: sized from free memory)")
    p.add_argument("--prompts", default=None, metavar="FILE", help="requests to run instead of the random workload (JSON lines)")
    p.add_argument("--tokens-out", default=None, metavar="FILE", help="write the generated token ids here, a JSON list a line ('-': stdout)")
    p.add_argument("--temperature", type=float, default=0.6, help="0: greedy")
    p.add_argument("--stop-at-eos", action="store_true", help="end a request at the model's end token (default: ignore it, as the reference's workload)")
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

    vocab_cap = 10000
    if args.prompts:
        prompt_token_ids, max_tokens, temperatures = [], [], []
        with open(args.prompts) as f:
            for number, text in enumerate(f, 1):
                if not text.strip():
                    continue
                rec = json.loads(text)
                if isinstance(rec, list):
                    rec = {"prompt": rec}
                if not (isinstance(rec, dict) and isinstance(rec.get("prompt"), list) and rec["prompt"]
                        and all(isinstance(t, int) for t in rec["prompt"])):
                    p.error(f"{args.prompts}:{number}: expected a list of token ids or an object with one under 'prompt'")
                prompt_token_ids.append(rec["prompt"])
                max_tokens.append(int(rec.get("max_tokens", args.max_output)))
                temperatures.append(float(rec.get("temperature", args.temperature)))
        N = len(prompt_token_ids)
        vocab_cap = None
    else:
        seed(0)
        N = args.num_seqs
        prompt_token_ids = [[randint(0, vocab_cap) for _ in range(randint(min(100, args.max_prompt), args.max_prompt))] for _ in range(N)]
        max_tokens = [randint(min(100, args.max_output), args.max_output) for _ in range(N)]
        temperatures = [args.temperature] * N

    llm = LLM(path, max_num_seqs=args.max_num_seqs, max_model_len=args.max_model_len, max_num_batched_tokens=args.budget,
              enable_chunked_prefill=bool(args.chunked), long_prefill_token_threshold=args.threshold, dtype=args.dtype,
              seed=args.seed, kvcache_block_size=args.block_size, scheduling_policy=args.policy, device=args.device,
              num_kvcache_blocks=args.num_kv_blocks)
    vocab = llm.model.embedding.vocab_size
    if vocab_cap is not None and vocab <= vocab_cap:
        prompt_token_ids = [[t % vocab for t in ids] for ids in prompt_token_ids]
    sps = [SamplingParams(temperature=temp, ignore_eos=not args.stop_at_eos, max_tokens=m)
           for temp, m in zip(temperatures, max_tokens)]

    llm.generate([[1, 2, 3]], SamplingParams(max_tokens=4), use_tqdm=False)      # warm-up
    t = time.time()
    results = llm.generate(prompt_token_ids, sps, use_tqdm=False)
    t = time.time() - t
    if args.tokens_out:
        lines = "".join(json.dumps(r["token_ids"]) + "\n" for r in results)
        if args.tokens_out == "-":
            sys.stdout.write(lines)
        else:
            os.makedirs(os.path.dirname(args.tokens_out) or ".", exist_ok=True)
            with open(args.tokens_out, "w") as f:
                f.write(lines)

    total = sum(len(r["token_ids"]) for r in results)
    row = {
        "engine": "mini_engine_amd", "label": args.label, "gpu": torch.cuda.get_device_name(0) if args.device.startswith("cuda") else args.device, "torch": torch.__version__,
        "model": args.random_weights or path, "dtype": args.dtype, "num_seqs": N,
        "input_tokens": sum(len(x) for x in prompt_token_ids), "output_tokens": total, "time_s": round(t, 2),
        "throughput_tok_s": round(total / t, 1), "chunked": bool(args.chunked), "budget": args.budget,
        "threshold": args.threshold, "preemptions": llm.scheduler.num_preemptions,
        "kv_blocks": llm.config.num_kvcache_blocks, "time": datetime.now().isoformat(timespec="seconds"),
    }
    print(json.dumps(row))
    os.makedirs(os.path.dirname(args.out) or ".", exist_ok=True)
    with open(args.out, "a") as f:
        f.write(json.dumps(row) + "\n")
    if tmp is not None:
        tmp.cleanup()
    return 0


if __name__ == "__main__":
    sys.exit(main())
