"""The offline command line (`python -m mini_engine_amd.cli`): the reference's workload row, and a folder and
a prompt file in, generated token ids out."""
import json

import pytest

import helpers
import plain_qwen3


def _prompt_file(tmp_path, vocab):
    prompts = [helpers.random_ids(n, vocab, 600 + n) for n in (3, 19, 41)]
    path = tmp_path / "prompts.jsonl"
    lines = [json.dumps(prompts[0]), json.dumps({"prompt": prompts[1], "max_tokens": 5}),
             json.dumps({"prompt": prompts[2], "temperature": 0.0})]
    path.write_text("\n".join(lines) + "\n")
    return prompts, str(path)


def _check_tokens_against_plain(folder, prompts, out_path, dtype):
    import torch
    cfg, w = plain_qwen3.read_model_folder(folder, torch.float64)
    got = [json.loads(line) for line in open(out_path)]
    assert [len(g) for g in got] == [7, 5, 7]
    for p, g in zip(prompts, got):
        if dtype == "float32":
            assert g == plain_qwen3.greedy_generate(cfg, w, p, len(g))
        else:       # bfloat16 may pick another token only where the two logits lie within its rounding
            ids = list(p)
            for tok in g:
                z = plain_qwen3.logits(cfg, w, ids)[-1]
                best = int(z.argmax())
                assert tok == best or float(z[best] - z[tok]) < 2e-2 * float(z.abs().max())
                ids.append(tok)


def test_prompts_in_tokens_out_on_cpu(folders, plain_backend, tmp_path, capsys):
    from mini_engine_amd import cli
    folder = folders("B")
    prompts, path = _prompt_file(tmp_path, 384)
    out = tmp_path / "o" / "tokens.jsonl"
    rc = cli.main(["--model", folder, "--prompts", path, "--tokens-out", str(out), "--temperature", "0", "--max-output", "7",
                   "--dtype", "float32", "--device", "cpu", "--num-kv-blocks", "64", "--block-size", "8", "--budget", "16",
                   "--max-num-seqs", "4", "--max-model-len", "128", "--out", str(tmp_path / "rows.jsonl")])
    assert rc == 0
    row = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert row["num_seqs"] == 3 and row["output_tokens"] == 19 and row["input_tokens"] == 63 and row["budget"] == 16
    assert json.loads(open(tmp_path / "rows.jsonl").read()) == row
    _check_tokens_against_plain(folder, prompts, out, "float32")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompts_in_tokens_out(folders, tmp_path, capsys, dtype):
    from mini_engine_amd import cli
    folder = folders("B")
    prompts, path = _prompt_file(tmp_path, 384)
    out = tmp_path / "tokens.jsonl"
    rc = cli.main(["--model", folder, "--prompts", path, "--tokens-out", str(out), "--temperature", "0", "--max-output", "7",
                   "--dtype", dtype, "--block-size", "8", "--budget", "16", "--max-num-seqs", "4", "--max-model-len", "128",
                   "--out", str(tmp_path / "rows.jsonl")])
    assert rc == 0
    _check_tokens_against_plain(folder, prompts, out, dtype)


@pytest.mark.gpu
def test_reference_workload_row_with_random_weights(tmp_path, capsys):
    """The reference's offline workload at a tiny size: the row's counts are the workload's (random.seed(0))."""
    from random import randint, seed
    from mini_engine_amd import cli
    rc = cli.main(["--random-weights", "tinyA", "--num-seqs", "6", "--max-prompt", "40", "--max-output", "8",
                   "--max-model-len", "64", "--max-num-seqs", "4", "--budget", "32", "--tokens-out", "-",
                   "--out", str(tmp_path / "bench.jsonl")])
    assert rc == 0
    lines = capsys.readouterr().out.strip().splitlines()
    row = json.loads(lines[-1])
    seed(0)
    prompts = [[randint(0, 10000) for _ in range(randint(40, 40))] for _ in range(6)]
    max_tokens = [randint(8, 8) for _ in range(6)]
    tokens = [json.loads(line) for line in lines[-7:-1]]
    assert [len(t) for t in tokens] == max_tokens and all(0 <= t < 256 for ts in tokens for t in ts)
    assert row["engine"] == "mini_engine_amd" and row["num_seqs"] == 6 and row["output_tokens"] == sum(max_tokens)
    assert row["input_tokens"] == sum(len(p) for p in prompts) and row["throughput_tok_s"] > 0 and row["chunked"] is True
