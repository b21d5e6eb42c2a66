"""The latency command line: its workload, its settings and its bookkeeping, on the CPU with the
plain twins of the kernels; one run through main() on the GPU."""
import json

import pytest

import helpers
from mini_engine_amd import cli_latency
from mini_engine_amd.cache.manager import CacheManager


def test_arrivals_are_seeded_by_the_rate_and_keep_the_reference_ranges():
    a = cli_latency.poisson_arrivals(400, 8.0, 0.1, 151936)
    b = cli_latency.poisson_arrivals(400, 8.0, 0.1, 151936)
    assert [(x.at, x.prompt, x.max_tokens) for x in a] == [(x.at, x.prompt, x.max_tokens) for x in b]
    assert cli_latency.poisson_arrivals(5, 4.0, 0.1, 151936)[0].at != a[0].at          # another rate, other arrivals
    assert all(x.at < y.at for x, y in zip(a, a[1:]))
    assert 0.7 * 400 / 8.0 < a[-1].at < 1.3 * 400 / 8.0                                   # mean gap 1/rate
    for x in a:
        assert (4096 <= len(x.prompt) <= 7680) if x.long else (128 <= len(x.prompt) <= 512)
        assert 128 <= x.max_tokens <= 256 and max(x.prompt) <= 10000
    assert 20 <= sum(x.long for x in a) <= 65                                             # a tenth, give or take
    small = cli_latency.poisson_arrivals(50, 8.0, 0.5, 256, scale=0.01)
    assert all(len(x.prompt) <= 76 and 1 <= x.max_tokens <= 2 and max(x.prompt) < 256 for x in small)


def test_forget_prefixes_makes_the_next_request_start_cold():
    m = CacheManager(8, 4)
    ids = list(range(11))
    assert m.allocate("a", 0, 11)
    m.publish_full_pages("a", ids, 11)
    m.free("a")
    assert m.find_prefix_hit(ids).num_pages == 2
    m.forget_prefixes()
    assert m.find_prefix_hit(ids).num_pages == 0
    m.check_invariants()
    assert m.allocate("b", 0, 11)                      # and the pages serve again, and can be published again
    m.publish_full_pages("b", ids, 11)
    assert m.find_prefix_hit(ids).num_pages == 2
    m.forget_prefixes()                                # while a request holds pages: it publishes from its start again
    m.publish_full_pages("b", ids, 11)
    assert m.find_prefix_hit(ids).num_pages == 2
    m.free("b")
    m.check_invariants()


def _engine(folder, **kw):
    from mini_engine_amd import LLM
    return LLM(folder, dtype="float32", device="cpu", poison_cache=True, kvcache_block_size=8, num_kvcache_blocks=64,
               max_num_seqs=4, max_num_batched_tokens=128, max_model_len=128, **kw)


def test_settings_switch_the_scheduler_and_refuse_what_it_cannot_do(folders, plain_backend):
    llm = _engine(folders("B"))
    Setting = cli_latency.Setting
    assert Setting.parse("c16") == Setting("c16", True, 16) and Setting.parse("pf") == Setting("pf", False, cli_latency.ENGINE_BUDGET)
    Setting.parse("c16").switch(llm)
    assert llm.scheduler.chunked and llm.scheduler.token_budget == 16
    Setting.parse("pf").switch(llm)
    assert not llm.scheduler.chunked and llm.scheduler.token_budget == cli_latency.ENGINE_BUDGET
    for bad in ("c0", "c99999", "x12", "c", "c2"):     # c2: fewer tokens than requests that may decode
        with pytest.raises(ValueError):
            Setting.parse(bad).switch(llm)
    assert not llm.scheduler.chunked and llm.scheduler.token_budget == cli_latency.ENGINE_BUDGET       # a refused setting changes nothing


def test_serving_arrivals_gives_every_request_its_tokens_and_times(folders, plain_backend):
    """Requests arriving over time under a chunked and a prefill-first setting: every request gets all its
    tokens, the figures are consistent with each other, nothing stays held, and both settings sample the
    same number of tokens."""
    from mini_engine_amd import SamplingParams
    llm = _engine(folders("B"))
    arrivals = cli_latency.poisson_arrivals(10, 400.0, 0.3, 384, scale=0.012)      # prompts 1-6 and 49-92, 1-3 tokens out
    arrivals[4].prompt, arrivals[4].long = helpers.random_ids(70, 384, 5), True       # whatever the draw: long ones too
    arrivals[7].prompt, arrivals[7].long = helpers.random_ids(90, 384, 6), True
    for a in arrivals:
        a.max_tokens += 3
    params_of = lambda a: SamplingParams(temperature=0.6, ignore_eos=True, max_tokens=a.max_tokens)
    rows = {}
    for name in ("c16", "pf"):
        cli_latency.Setting.parse(name).switch(llm)
        r = rows[name] = cli_latency.serve(llm, arrivals, params_of)
        assert not llm.manager.held
        llm.manager.check_invariants()
        assert r["num_long"] == sum(a.long for a in arrivals) and r["steps"] > 0 and r["preemptions"] == 0
        assert r["output_tokens"] == sum(a.max_tokens for a in arrivals) and r["out_tok_s"] > 0
        # times are wall-clock: only what holds whatever the machine's speed
        assert 0 <= r["ttft_p50_ms"] <= r["ttft_p99_ms"] and 0 <= r["itl_p50_ms"] <= r["itl_p99_ms"] <= r["itl_max_ms"]
        assert r["ttft_long_p50_ms"] is not None and r["ttft_short_p99_ms"] is not None and r["tpot_mean_ms"] >= 0
    assert rows["c16"]["steps"] >= 90 // 16                  # the longest prompt alone needs that many portions


def test_token_times_give_the_figures_of_a_known_run():
    """Two requests with hand-made times: first tokens after 10 and 30 ms, gaps of 2 ms and 4 ms."""
    t = cli_latency.TokenTimes()
    t.request("a", 100.0, False)
    t.request("b", 100.5, True)
    t.request("c", 101.0, False)                              # never answered: counts nowhere
    t.tokens(["a"], 100.010); t.tokens(["a", "b"], 100.530); t.tokens(["b"], 100.534); t.tokens(["b"], 100.538)
    f = t.figures()
    assert f["output_tokens"] == 5 and f["num_long"] == 1
    assert f["ttft_p50_ms"] == 20.0 and f["ttft_long_p50_ms"] == 30.0 and f["ttft_short_p99_ms"] == 10.0
    assert f["itl_max_ms"] == 520.0 and f["itl_p50_ms"] == 4.0
    assert f["tpot_mean_ms"] == round((520.0 + 4.0) / 2, 1)


@pytest.mark.gpu
def test_command_line_writes_one_row_per_rate_and_setting(tmp_path):
    out = tmp_path / "latency.jsonl"
    rc = cli_latency.main(["--random-weights", "tinyA", "--num-reqs", "12", "--rates", "200,400", "--configs", "pf,c64",
                           "--scale", "0.02", "--max-model-len", "256", "--max-num-seqs", "8", "--out", str(out)])
    assert rc == 0
    rows = [json.loads(line) for line in out.read_text().splitlines()]
    assert [(r["rate"], r["config"]) for r in rows] == [(200.0, "pf"), (200.0, "c64"), (400.0, "pf"), (400.0, "c64")]
    for r in rows:
        assert r["num_reqs"] == 12 and r["out_tok_s"] > 0 and r["ttft_p50_ms"] > 0 and r["preemptions"] == 0
