"""Shared test material: tiny configurations, traces, comparisons."""
from __future__ import annotations

import torch

import plain_qwen3
from mini_engine_amd.config.model_config import Qwen3Config
from mini_engine_amd.weights.random_init import write_random_model

# Tiny configurations that differ in every size and option.
#   A: tied head, page 16, theta 1e4, eps 1e-6, groups of 2, D 16, q width == hidden
#   B: untied, page 8, theta 1e6, eps 1e-5, groups of 3, D 32, q width 192 != hidden 80, no power-of-two sizes
#   C: sliding window of 24 on layers 1 and 3 of 4, groups of 4 (Hkv 1), D 48, vocabulary 300, hidden 72
CONFIGS = {
    "A": dict(architectures=["Qwen3ForCausalLM"], vocab_size=256, hidden_size=64, intermediate_size=128,
              num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
              rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=True, max_position_embeddings=4096),
    "B": dict(architectures=["Qwen3ForCausalLM"], vocab_size=384, hidden_size=80, intermediate_size=224,
              num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=2, head_dim=32,
              rms_norm_eps=1e-5, rope_theta=1000000.0, tie_word_embeddings=False, max_position_embeddings=4096),
    "C": dict(architectures=["Qwen3ForCausalLM"], vocab_size=300, hidden_size=72, intermediate_size=200,
              num_hidden_layers=4, num_attention_heads=4, num_key_value_heads=1, head_dim=48,
              rms_norm_eps=3e-6, rope_theta=50000.0, tie_word_embeddings=False, max_position_embeddings=4096,
              use_sliding_window=True, sliding_window=24,
              layer_types=["full_attention", "sliding_attention", "full_attention", "sliding_attention"]),
    # R: two layers at the layer sizes of Qwen3-0.6B (bfloat16 only: the kernel forms that a real model runs through,
    # which the tiny widths above never reach: products in slices of a long K, wide loads, head size 128)
    "R": dict(architectures=["Qwen3ForCausalLM"], vocab_size=2048, hidden_size=1024, intermediate_size=3072,
              num_hidden_layers=2, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
              rms_norm_eps=1e-6, rope_theta=1000000.0, tie_word_embeddings=True, max_position_embeddings=4096),
}
SEEDS = {"A": 0, "B": 1, "C": 2, "R": 3}
PAGE = {"A": 16, "B": 8, "C": 16, "R": 16}

# float32: the engine against the float64 plain model, relative to the largest logit.
TOL_F32 = 1e-5
# bfloat16 activations (unit roundoff 2^-9 ~ 2e-3, a few dozen roundings per layer, <= 4 layers).
TOL_BF16 = 2e-2


def make_folder(name: str, path: str, store_dtype=torch.bfloat16) -> str:
    cfg = Qwen3Config.from_dict(CONFIGS[name])
    return write_random_model(cfg, SEEDS[name], path, store_dtype)


def random_ids(n: int, vocab: int, seed: int) -> list:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


_plain_cache: dict = {}


def plain_logits(folder: str, ids: list) -> torch.Tensor:
    """float64 logits of the plain implementation at every position (cached per folder/ids)."""
    key = (folder, tuple(ids))
    if key not in _plain_cache:
        if folder not in _plain_cache:
            _plain_cache[folder] = plain_qwen3.read_model_folder(folder, torch.float64)
        cfg, w = _plain_cache[folder]
        _plain_cache[key] = plain_qwen3.logits(cfg, w, ids)
    return _plain_cache[key]


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    got = got.detach().double().cpu()
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert torch.isfinite(got).all(), "engine produced NaN/inf logits"
    return float((got - ref).abs().max() / ref.abs().max())


def first_bad_row(got, ref, tol):
    """Index of the first row whose error exceeds tol (for messages)."""
    err = (got.detach().double().cpu() - ref).abs().amax(dim=-1) / ref.abs().max()
    bad = (err > tol).nonzero()
    return None if bad.numel() == 0 else (int(bad[0]), float(err[int(bad[0])]))


class Driver:
    """Feeds requests through a ModelRunner by explicit cuts, collecting logits per request."""

    def __init__(self, runner, manager):
        self.runner = runner
        self.manager = manager
        self.fed: dict = {}
        self.logits: dict = {}

    def step(self, parts: dict, want_all: bool = True, end=()):
        """parts: {request: tokens to feed now}."""
        from mini_engine_amd.engine.runner import StepEntry

        entries = []
        for rid, toks in parts.items():
            start = self.fed.get(rid, 0)
            assert self.manager.allocate(rid, start, len(toks)), f"out of pages for {rid}"
            entries.append(StepEntry(rid, list(toks), start, list(range(len(toks))) if want_all else []))
        out = self.runner.step(entries)
        k = 0
        for e in entries:
            n = len(e.want)
            if n:
                self.logits.setdefault(e.req, []).append(out[k:k + n].float().cpu())
                k += n
            self.fed[e.req] = e.start + len(e.tokens)
        for rid in end:
            self.manager.free(rid)
            self.fed.pop(rid, None)
        self.manager.check_invariants()

    def result(self, rid) -> torch.Tensor:
        return torch.cat(self.logits[rid])


def cuts_schedule(lengths: dict, pattern: list) -> list:
    """Turn per-request lengths and a cyclic pattern of chunk sizes into a list of steps
    {request: (begin, end)} with up to all requests live, requests rotating through the pattern."""
    pos = {r: 0 for r in lengths}
    steps, i = [], 0
    while any(pos[r] < lengths[r] for r in lengths):
        step = {}
        for j, r in enumerate(lengths):
            if pos[r] >= lengths[r]:
                continue
            n = pattern[(i + j) % len(pattern)]
            if n == 0:
                continue
            n = min(n, lengths[r] - pos[r])
            step[r] = (pos[r], pos[r] + n)
            pos[r] += n
        i += 1
        if step:
            steps.append(step)
    return steps


def assert_greedy_like_plain(folder: str, prompts: list, outputs: list, exact: bool, what: str = "") -> None:
    """outputs[i]: the token ids generated greedily after prompts[i]. Each token must be the plain
    implementation's best next token given what came before it; with exact=False (bfloat16) another
    token passes only where the plain model's logits of the two lie within bfloat16's tolerance."""
    if folder not in _plain_cache:
        _plain_cache[folder] = plain_qwen3.read_model_folder(folder, torch.float64)
    cfg, w = _plain_cache[folder]
    for i, (prompt, out) in enumerate(zip(prompts, outputs)):
        ids = list(prompt)
        for tok in out:
            z = plain_qwen3.logits(cfg, w, ids)[-1]
            best = int(torch.argmax(z))
            if tok != best:
                assert not exact and float(z[best] - z[tok]) <= TOL_BF16 * float(z.abs().max()), \
                    f"{what}: request {i} generated {tok} at position {len(ids)}, the plain implementation gives {best}"
            ids.append(tok)
