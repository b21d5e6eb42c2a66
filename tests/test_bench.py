"""bench.py: what it counts (bytes a decode step must read, flops of a prompt) from a model's declared parameters and
cache plan, on the CPU; its contract and `--model DIR` on the GPU."""
import json
import os
import subprocess
import sys

import pytest
import torch

import helpers

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_bytes_and_flops_follow_the_model_not_a_configuration():
    from mini_engine_amd.config.sizes import model_config
    from mini_engine_amd.registry import build_model
    cfg, _ = model_config("0.6b")
    model = build_model(cfg)
    # worked out by hand from the published sizes: 28 x (4096 + 1024 + 2 x 3072 + 3072... ) matrices of bfloat16
    per_layer = (4096 * 1024) + (1024 * 2048) + (6144 * 1024) + (1024 * 3072)
    weights = 28 * per_layer + 151936 * 1024                     # tied: the embedding matrix is the head's
    norms = 28 * (2 * 1024 + 2 * 128) + 1024
    per_token = 28 * 2 * 8 * 128 * 2                             # keys and values of 8 heads of 128, bfloat16
    want = weights * 2 + norms * 4 + 8 * 2064 * per_token
    assert bench.decode_bytes(model, 2, [2064] * 8, 16, torch.bfloat16) == want
    flops = 2 * 2048 * 28 * per_layer + 28 * 4 * 16 * 128 * 2048 * 2049 / 2 + 2 * 151936 * 1024
    assert bench.prefill_flops(model, 2048) == flops
    # an untied head counts beside the layers, its embedding (a gather of one row per request) does not
    cfg8, _ = model_config("8b", 2)
    m8 = build_model(cfg8)
    layer8 = 6144 * 4096 + 4096 * 4096 + 24576 * 4096 + 4096 * 12288
    assert bench.decode_bytes(m8, 2, [], 16, torch.bfloat16) == (2 * layer8 + 151936 * 4096) * 2 + (2 * (2 * 4096 + 256) + 4096) * 4


def test_a_window_bounds_what_a_decode_step_reads_and_what_a_prompt_computes():
    from mini_engine_amd.config.model_config import Qwen3Config
    from mini_engine_amd.registry import build_model
    model = build_model(Qwen3Config.from_dict(helpers.CONFIGS["C"]))        # layers 1 and 3 of 4 see 24 keys
    groups = bench.cache_bytes_per_token(model, 16, torch.bfloat16)
    assert sorted(w or 0 for _, w in groups) == [0, 24]
    per_call = 2 * 1 * 48 * 2                                                # keys and values, one head of 48, bfloat16
    weights = bench.decode_bytes(model, 2, [], 16, torch.bfloat16)
    assert bench.decode_bytes(model, 2, [100, 10], 16, torch.bfloat16) - weights == 2 * per_call * (110 + 24 + 10)
    full = 4.0 * 4 * 48 * (50 * 51 / 2)
    windowed = 4.0 * 4 * 48 * sum(min(t + 1, 24) for t in range(50))
    linear = bench.prefill_flops(model, 50) - 2 * (full + windowed)
    assert linear > 0 and abs(linear - bench.prefill_flops(model, 50) + 2 * full + 2 * windowed) < 1e-6


def test_more_than_one_gpu_is_refused_with_one_line(capsys):
    assert bench.main(["--gpus", "2"]) == 2
    out = capsys.readouterr().out.strip().splitlines()
    assert len(out) == 1 and "one GPU" in out[0]


@pytest.mark.gpu
def test_bench_measures_the_model_of_a_folder(folders, tmp_path):
    """`--model DIR`: the folder's own configuration and checkpoint, one JSON line with the contract's keys."""
    folder = folders("B")
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--model", folder, "--steps", "4", "--warmup", "2",
                           "--batch", "2", "--points", "1", "--context", "40", "--gen", "8", "--prefill-tokens", "48",
                           "--page", "8", "--offline", "0", "--second-size", "", "--third-size", ""],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    lines = [l for l in proc.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    row = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in row, key
    cfg = helpers.CONFIGS["B"]
    assert row["config"]["hidden"] == cfg["hidden_size"] and row["config"]["layers"] == cfg["num_hidden_layers"]
    assert row["config"]["vocab"] == cfg["vocab_size"] and len(row["config"]) <= 20
    assert all(not isinstance(v, (dict, list)) for v in row["config"].values())
    assert "checkpoint" in row["data"] and row["value"] > 0 and row["prefill"]["tokens"] == 48
    assert 0 < row["roofline"]["frac"] < 1 and row["roofline"]["bound"] == "hbm" and "decode_b1" in row["points"]
