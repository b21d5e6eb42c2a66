"""Trace replay: drives the engine's own model, step function, cache manager and kernels with
token ids given from outside, and writes logits. It has no forward pass, cache or loader of
its own, bypasses the scheduler and the sampler, and never looks up cached prefixes (every
token it is given is run).
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np
import torch

from .cache.manager import CacheManager
from .config.model_config import load_model_config
from .engine.runner import ModelRunner, StepEntry
from .weights.loader import load_model

DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}
ROUND = 64     # a request's token count is rounded up to this (or to the page size if larger)


class Replayer:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, page_size: int = 16, device: str = "cuda",
                 poison_cache: bool = False):
        if dtype not in DTYPES:
            raise ValueError(f"--dtype must be one of {sorted(DTYPES)}")
        if page_size > ROUND and page_size % ROUND:
            raise ValueError("page size must divide 64 or be a multiple of it")
        self.page_size = page_size
        round_to = max(ROUND, page_size)
        max_tokens = -(-max_tokens // round_to) * round_to
        cfg = load_model_config(model_dir)
        limit = getattr(cfg, "max_position_embeddings", None)
        self.max_positions = max_tokens if limit is None else min(max_tokens, limit)
        self.model = load_model(model_dir, device, DTYPES[dtype], self.max_positions, cfg)
        plan = self.model.cache_plan()
        slots = 8 if any(s is not None for s in plan.state_needs) else 0
        self.manager = CacheManager(max_tokens // page_size, page_size, ModelRunner.windows_of(self.model),
                                    num_state_slots=slots, enable_prefix_caching=False)
        self.runner = ModelRunner(self.model, self.manager, DTYPES[dtype], device, self.max_positions,
                                  poison_cache=poison_cache)
        self.fed: dict = {}          # request id -> tokens fed so far

    def step(self, entries: list, end: list) -> np.ndarray | None:
        batch = []
        for e in entries:
            rid, tokens, want = e["id"], list(e["tokens"]), list(e.get("want", []))
            start = self.fed.get(rid, 0)
            if not self.manager.allocate(rid, start, len(tokens)):
                raise RuntimeError(f"step needs more cache than --max-tokens allows (request {rid!r}, "
                                   f"{start + len(tokens)} tokens; {self.manager.num_free_pages()} free pages "
                                   f"of {self.page_size} tokens)")
            batch.append(StepEntry(rid, tokens, start, want))
        logits = self.runner.step(batch)
        for e in batch:
            self.fed[e.req] = e.start + len(e.tokens)
        for rid in end:
            if self.manager.holds(rid):
                self.manager.free(rid)
            self.fed.pop(rid, None)
        if logits is None:
            return None
        return logits.float().cpu().numpy()


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__)
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=sorted(DTYPES))
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at a time (each rounded up to a multiple of 64)")
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page")
    args = ap.parse_args(argv)
    os.makedirs(args.out, exist_ok=True)
    print(f"[trace_run] loading {args.model} ({args.dtype}); kernels are compiled on first use", file=sys.stderr, flush=True)
    rep = Replayer(args.model, args.dtype, args.max_tokens, args.page_size)
    print("[trace_run] ready", file=sys.stderr, flush=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        out = rep.step(rec.get("entries", []), rec.get("end", []))
        if out is not None:
            out.astype("<f4").tofile(os.path.join(args.out, f"{rec['step']}.f32"))
        print(f"done {rec['step']}", flush=True)
    return 0
