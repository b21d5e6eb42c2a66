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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_replay_cuts(folders, tmp_path, dtype, name):
    folder = folders(name)
    V = helpers.CONFIGS[name]["vocab_size"]
    tol = helpers.TOL_F32 if dtype == "float32" else helpers.TOL_BF16
    lens = {"a": 100, "b": 61, "c": 40, "d": 77, "e": 90}
    ids = {r: helpers.random_ids(n, V, 40 + i) for i, (r, n) in enumerate(lens.items())}
    cases = {
        "whole": [{r: (0, lens[r])} for r in ("a", "b")],
        "tail": [{"a": (0, 68)}] + [{"a": (t, t + 1)} for t in range(68, 100)],
        "portions": helpers.cuts_schedule({"a": 100}, [2, 3, 31, 2, 17, 1, 8]),
        # five requests, at most four live, in a pool of 4 x 128 tokens less one request: later ones reuse pages
        "mixed": helpers.cuts_schedule({r: lens[r] for r in ("a", "b", "c", "d")}, [19, 1, 1, 2, 33, 1, 7, 1]),
    }
    for case, schedule in cases.items():
        steps = steps_from_schedule(ids, schedule)
        if case == "mixed":      # e starts once c (the shortest) has ended, taking over its pages
            last_c = max(i for i, st in enumerate(schedule) if "c" in st)
            extra = helpers.cuts_schedule({"e": 90}, [5, 1, 40, 1])
            for j, st in enumerate(extra):
                i = last_c + 1 + j
                a, b = st["e"]
                entry = {"id": "e", "tokens": ids["e"][a:b], "want": list(range(b - a))}
                if i < len(steps):
                    steps[i]["entries"].append(entry)
                    if b == 90: steps[i]["end"].append("e")
                else:
                    steps.append({"step": i, "entries": [entry], "end": ["e"] if b == 90 else []})
        out = str(tmp_path / f"{case}")
        replay(folder, dtype, steps, out, max_tokens=128 * 3 + 64, page=helpers.PAGE[name])
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
