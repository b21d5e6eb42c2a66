"""bin/trace_run as a program: the same requests whole, with the last 32 tokens one by one,
in portions of changing size, and mixed with other requests so that pages are used again,
in float32 and in bfloat16, compared with the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def replay(folder, dtype, steps, out_dir, max_tokens, page=16):
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out_dir,
                           "--max-tokens", str(max_tokens), "--page-size", str(page)],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert [l for l in proc.stdout.split("\n") if l] == [f"done {s['step']}" for s in steps]
    return proc


def collect(steps, out_dir, vocab):
    got: dict = {}
    for s in steps:
        n = sum(len(e["want"]) for e in s["entries"])
        path = os.path.join(out_dir, f"{s['step']}.f32")
        if n == 0:
            assert not os.path.exists(path)
            continue
        a = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(n, vocab))
        k = 0
        for e in s["entries"]:
            if e["want"]:
                got.setdefault(e["id"], []).append(a[k:k + len(e["want"])]); k += len(e["want"])
    return {r: torch.cat(v) for r, v in got.items()}


def steps_from_schedule(ids, schedule, ends=True):
    steps = []
    for i, st in enumerate(schedule):
        entries = [{"id": r, "tokens": ids[r][a:b], "want": list(range(b - a))} for r, (a, b) in st.items()]
        end = [r for r, (a, b) in st.items() if ends and b == len(ids[r])]
        steps.append({"step": i, "entries": entries, "end": end})
    return steps


def most_live_tokens(steps) -> int:
    """The --max-tokens a trace needs: the most tokens live requests hold at any time, each request's count
    rounded up to a multiple of 64 (a request is live from its first step to the step that ends it)."""
    fed, most = {}, 0
    for s in steps:
        for e in s["entries"]:
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])
        most = max(most, sum(-(-n // 64) * 64 for n in fed.values()))
        for r in s["end"]:
            fed.pop(r)
    return most


def pages_used_again(folder, steps, max_tokens, page) -> dict:
    """Replays the trace's allocations on a cache manager of the program's size (it hands out pages in a fixed
    order): per request, how many of its pages had belonged to a request that ended before."""
    from mini_engine_amd.cache.manager import CacheManager
    from mini_engine_amd.config.model_config import load_model_config
    from mini_engine_amd.engine.runner import ModelRunner
    from mini_engine_amd.registry import build_model
    manager = CacheManager(max_tokens // page, page, ModelRunner.windows_of(build_model(load_model_config(folder))),
                           enable_prefix_caching=False)
    fed, given_back, again = {}, set(), {}
    for s in steps:
        for e in s["entries"]:
            assert manager.allocate(e["id"], fed.get(e["id"], 0), len(e["tokens"]))
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])
            again[e["id"]] = len(given_back & {p for p in manager.block_table(e["id"]) if p >= 0})
        for r in s["end"]:
            given_back |= {p for p in manager.block_table(r) if p >= 0}
            manager.free(r)
            fed.pop(r)
    return again


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_replay_cuts(folders, tmp_path, dtype, name):
    folder = folders(name)
    V = helpers.CONFIGS[name]["vocab_size"]
    page = helpers.PAGE[name]
    tol = helpers.TOL_F32 if dtype == "float32" else helpers.TOL_BF16
    lens = {"a": 128, "b": 64, "c": 62, "d": 126, "e": 120}
    ids = {r: helpers.random_ids(n, V, 40 + i) for i, (r, n) in enumerate(lens.items())}
    cases = {
        "whole": [{r: (0, lens[r])} for r in ("a", "b")],
        "tail": [{"a": (0, 96)}] + [{"a": (t, t + 1)} for t in range(96, 128)],
        "portions": helpers.cuts_schedule({"a": 128}, [2, 3, 31, 2, 17, 1, 8]),
        # five requests, at most four live, in a pool of exactly what they hold at most: e, which starts when
        # c has ended, cannot be served from pages nobody has used
        "mixed": helpers.cuts_schedule({r: lens[r] for r in ("a", "b", "c", "d")}, [19, 1, 1, 2, 33, 1, 7, 1]),
    }
    for case, schedule in cases.items():
        steps = steps_from_schedule(ids, schedule)
        if case == "mixed":      # e starts once c (the shortest) has ended, taking over its pages
            last_c = max(i for i, st in enumerate(schedule) if "c" in st)
            extra = helpers.cuts_schedule({"e": lens["e"]}, [5, 1, 40, 1])
            for j, st in enumerate(extra):
                i = last_c + 1 + j
                a, b = st["e"]
                entry = {"id": "e", "tokens": ids["e"][a:b], "want": list(range(b - a))}
                if i < len(steps):
                    steps[i]["entries"].append(entry)
                    if b == lens["e"]: steps[i]["end"].append("e")
                else:
                    steps.append({"step": i, "entries": [entry], "end": ["e"] if b == lens["e"] else []})
        max_tokens = most_live_tokens(steps)
        if case == "mixed":
            assert max(len(s["entries"]) for s in steps) == 4
            assert pages_used_again(folder, steps, max_tokens, page)["e"] >= 2, "e was served from pages nobody had used"
        out = str(tmp_path / f"{case}")
        replay(folder, dtype, steps, out, max_tokens=max_tokens, page=page)
        got = collect(steps, out, V)
        for r, g in got.items():
            err = helpers.rel_err(g, helpers.plain_logits(folder, ids[r]))
            assert err <= tol, f"{name} {dtype} {case} request {r}: {err:.3g}"


def test_replay_runs_out_of_cache_loudly(folders, tmp_path):
    folder = folders("A")
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": helpers.random_ids(100, 256, 1), "want": []}], "end": []}]
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out",
                           str(tmp_path / "o"), "--max-tokens", "64"], input=json.dumps(steps[0]) + "\n",
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode != 0 and "max-tokens" in proc.stderr
