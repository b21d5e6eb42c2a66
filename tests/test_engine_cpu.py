"""The engine's bookkeeping (model assembly, step function, cache manager, replay, scheduler,
entry point) on the CPU, with the plain twins of the kernels, in float32."""
import io
import json
import os

import pytest
import torch

import engine_cases
import helpers
import plain_qwen3
from mini_engine_amd.cache.manager import CacheManager
from mini_engine_amd.engine.runner import ModelRunner, StepEntry
from mini_engine_amd.weights.loader import load_model


class Env:
    device, dtype, tol = "cpu", torch.float32, helpers.TOL_F32

    def __init__(self, folders, graphs=False, padded_up_to=4096):
        self.folders = folders
        self.models = {}
        self.graphs = graphs           # every step through the fixed layouts (padded; captured where there is a GPU)
        self.padded_up_to = padded_up_to

    def runner(self, name, pages):
        folder = self.folders(name)
        if name not in self.models:
            self.models[name] = load_model(folder, self.device, self.dtype, 512)
        model = self.models[name]
        manager = CacheManager(pages, helpers.PAGE[name], ModelRunner.windows_of(model), enable_prefix_caching=False)
        options = dict(use_graphs=True, mixed_graphs_after=0, mixed_graphs_max_tokens=self.padded_up_to) if self.graphs else {}
        return ModelRunner(model, manager, self.dtype, self.device, 512, poison_cache=True, **options), manager, folder


@pytest.fixture(scope="module")
def env(folders):
    return Env(folders)


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("case", [c for c in engine_cases.ALL if c.__name__ not in ("long_decode",)], ids=lambda c: c.__name__)
def test_cuts_through_padded_layouts(folders, plain_backend, case, name):
    """The same cuts with every step rounded up to a shared layout: padding rows among the single tokens, a
    padding request behind the prompt portions, wider block tables, more rows of logits than wanted."""
    env = Env(folders, graphs=True)
    case(env, name)


@pytest.mark.parametrize("name", ["A", "C"])
def test_padded_layouts_are_used(folders, plain_backend, name):
    engine_cases.padded_layouts_are_used(Env(folders, graphs=True), name, captured=False)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_exactly_sized_layouts_are_used(folders, plain_backend, name):
    engine_cases.exactly_sized_layouts_are_used(Env(folders, graphs=True, padded_up_to=16), name, captured=False)


@pytest.mark.parametrize("name", ["B"])
@pytest.mark.parametrize("case", [engine_cases.changing_portions, engine_cases.mixed_with_reuse], ids=lambda c: c.__name__)
def test_cuts_through_exactly_sized_layouts(folders, plain_backend, case, name):
    case(Env(folders, graphs=True, padded_up_to=16), name)


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("case", [c for c in engine_cases.ALL if c.__name__ not in ("long_decode",)], ids=lambda c: c.__name__)
def test_cuts(env, plain_backend, case, name):
    case(env, name)


def test_runner_refuses_bad_input(env, plain_backend):
    runner, manager, _ = env.runner("A", 4)
    assert manager.allocate("r", 0, 3)
    with pytest.raises(ValueError, match="token id"):
        runner.step([StepEntry("r", [1, 2, 999], 0, [])])
    with pytest.raises(ValueError, match="twice"):
        runner.step([StepEntry("r", [1], 0, []), StepEntry("r", [2], 1, [])])
    with pytest.raises(ValueError, match="wanted place"):
        runner.step([StepEntry("r", [1, 2], 0, [2])])
    with pytest.raises(ValueError, match="limit"):
        runner.step([StepEntry("r", [1], 600, [])])
    with pytest.raises(RuntimeError, match="no page"):
        runner.step([StepEntry("r", list(range(40)), 0, [])])      # only 3 tokens were allocated


def _llm(folder, **kw):
    from mini_engine_amd import LLM
    return LLM(folder, dtype="float32", device="cpu", poison_cache=True, **kw)


def test_generate_greedy_matches_plain(folders, plain_backend):
    """Tiny A: prompts of 5, 17 and 33 tokens, 8 greedy tokens each."""
    from mini_engine_amd import SamplingParams
    folder = folders("A")
    cfg, w = plain_qwen3.read_model_folder(folder, torch.float64)
    prompts = [helpers.random_ids(n, 256, 900 + n) for n in (5, 17, 33)]
    llm = _llm(folder, kvcache_block_size=16, num_kvcache_blocks=12, max_num_seqs=4, max_num_batched_tokens=64, max_model_len=64)
    outs = llm.generate(prompts, SamplingParams(temperature=0, max_tokens=8), use_tqdm=False)
    for p, o in zip(prompts, outs):
        assert o["token_ids"] == plain_qwen3.greedy_generate(cfg, w, p, 8)
    llm.manager.check_invariants()
    assert llm.manager.num_free_pages() == 12


def test_generate_chunked_sampled_is_independent_of_batching_and_preemption(folders, plain_backend):
    """Tiny B: prompts of 1, 9, 24, 40 and 63 tokens, budget 16, temperature 0.8, 12 tokens.
    The same seed must give the same tokens whether requests run together under a tight budget,
    alone, or through a pool so small that requests are preempted and recomputed."""
    from mini_engine_amd import SamplingParams
    folder = folders("B")
    prompts = [helpers.random_ids(n, 384, 950 + n) for n in (1, 9, 24, 40, 63)]
    sp = SamplingParams(temperature=0.8, max_tokens=12, ignore_eos=True)
    common = dict(kvcache_block_size=8, max_num_seqs=16, max_model_len=128, seed=3)
    together = _llm(folder, num_kvcache_blocks=64, max_num_batched_tokens=16, **common)
    out_together = [o["token_ids"] for o in together.generate(prompts, sp, use_tqdm=False)]
    assert all(len(o) == 12 for o in out_together)
    alone = _llm(folder, num_kvcache_blocks=64, max_num_batched_tokens=128, **common)
    for i, p in enumerate(prompts):
        seq = alone.add_request(p, sp, sample_stream=i)
        toks = None
        while not alone.is_finished():
            for sid, t in alone.step()[0]:
                toks = t
        assert toks == out_together[i], f"request {i} differs when run alone"
    tight = _llm(folder, num_kvcache_blocks=21, max_num_batched_tokens=16, enable_prefix_caching=False, **common)
    out_tight = [o["token_ids"] for o in tight.generate(prompts, sp, use_tqdm=False)]
    assert tight.scheduler.num_preemptions > 0, "the pool was large enough that nothing was preempted"
    assert out_tight == out_together
    other_seed = _llm(folder, num_kvcache_blocks=64, max_num_batched_tokens=16, **dict(common, seed=4))
    assert [o["token_ids"] for o in other_seed.generate(prompts, sp, use_tqdm=False)] != out_together


def test_running_one_step_ahead_changes_no_token(folders, plain_backend):
    """Decode steps launched before the step in flight has delivered its tokens: the same tokens as
    step by step, for greedy and sampled requests, with requests that end by max_tokens and by the
    end token at different times (a request that samples its end token has already run one step too
    far; that token is dropped), with and without prefix caching."""
    from mini_engine_amd import SamplingParams
    folder = folders("A")
    prompts = [helpers.random_ids(n, 256, 700 + n) for n in (3, 18, 33, 47)]
    sps = [SamplingParams(temperature=t, max_tokens=m) for t, m in ((0, 9), (0.7, 30), (0, 22), (0.9, 14))]
    kw = dict(kvcache_block_size=16, num_kvcache_blocks=40, max_num_seqs=8, max_num_batched_tokens=64, max_model_len=128, seed=5)
    free_run = [o["token_ids"] for o in _llm(folder, run_ahead=False, eos=-2, **kw).generate(prompts, sps, use_tqdm=False)]
    assert [len(o) for o in free_run] == [9, 30, 22, 14]
    eos = free_run[1][11]                                     # request 1 meets its end token in mid-flight
    want = [o[:o.index(eos) + 1] if eos in o else o for o in free_run]
    assert len(want[1]) < 30
    helpers.assert_greedy_like_plain(folder, prompts[0::2], want[0::2], True, "run ahead")          # the greedy ones
    for caching in (False, True):
        plain = _llm(folder, run_ahead=False, eos=eos, enable_prefix_caching=caching, **kw)
        assert [o["token_ids"] for o in plain.generate(prompts, sps, use_tqdm=False)] == want
        assert plain.steps_run_ahead == 0
        ahead = _llm(folder, run_ahead=True, eos=eos, enable_prefix_caching=caching, **kw)
        assert [o["token_ids"] for o in ahead.generate(prompts, sps, use_tqdm=False)] == want
        assert ahead.steps_run_ahead >= 15
        ahead.manager.check_invariants()
        assert ahead.manager.num_free_pages() == 40 and not ahead.manager.held


@pytest.mark.parametrize("seed", [1, 2, 3, 4])
def test_running_ahead_under_random_traffic(folders, plain_backend, seed):
    """Requests arriving while others decode, a pool so small that requests are preempted, ends by
    max_tokens and by the end token, greedy and sampled: with and without running one step ahead,
    every request gets the same tokens, and nothing is left held."""
    import random
    from mini_engine_amd import SamplingParams
    folder = folders("B")
    rng = random.Random(seed)
    n = 14
    prompts = [helpers.random_ids(rng.randint(1, 50), 384, 100 * seed + i) for i in range(n)]
    sps = [SamplingParams(temperature=rng.choice([0.0, 0.8]), max_tokens=rng.randint(1, 40)) for _ in range(n)]
    arrive = sorted(rng.randint(0, 60) for _ in range(n))      # the step at which a request is added
    kw = dict(kvcache_block_size=8, num_kvcache_blocks=rng.choice([26, 40, 80]), max_num_seqs=6,
              max_num_batched_tokens=rng.choice([16, 48]), max_model_len=128, seed=seed,
              enable_prefix_caching=bool(seed % 2))

    def run(run_ahead, eos):
        llm = _llm(folder, run_ahead=run_ahead, eos=eos, **kw)
        out, ids, step, added = {}, [], 0, 0
        while added < n or not llm.is_finished():
            while added < n and arrive[added] <= step:
                ids.append(llm.add_request(prompts[added], sps[added], sample_stream=added)); added += 1
            if not llm.is_finished():
                for sid, toks in llm.step()[0]:
                    assert sid not in out
                    out[sid] = toks
            step += 1
        llm.manager.check_invariants()
        assert not llm.manager.held and llm.manager.num_free_pages() == kw["num_kvcache_blocks"]
        return [out[i] for i in ids], llm

    free_run, _ = run(False, -2)
    eos = max(set(t for o in free_run for t in o[1:]), key=lambda t: sum(o.count(t) for o in free_run))
    want, plain = run(False, eos)
    got, ahead = run(True, eos)
    assert got == want
    assert any(o[-1] == eos and len(o) < sp.max_tokens for o, sp in zip(want, sps)), "no request met its end token"
    assert plain.steps_run_ahead == 0 and ahead.steps_run_ahead > 0


def test_prefix_hits_give_the_same_tokens(folders, plain_backend):
    from mini_engine_amd import SamplingParams
    folder = folders("A")
    shared = helpers.random_ids(40, 256, 990)
    prompts = [shared + helpers.random_ids(5, 256, 991), shared + helpers.random_ids(9, 256, 992)]
    sp = SamplingParams(temperature=0, max_tokens=6)
    kw = dict(kvcache_block_size=16, num_kvcache_blocks=16, max_num_seqs=4, max_num_batched_tokens=256, max_model_len=128)
    cold = _llm(folder, enable_prefix_caching=False, **kw)
    want = [o["token_ids"] for o in cold.generate(prompts, sp, use_tqdm=False)]
    warm = _llm(folder, **kw)
    first = warm.generate(prompts[:1], sp, use_tqdm=False)[0]["token_ids"]
    sid = warm.add_request(prompts[1], sp)
    seqs = warm.scheduler.waiting
    assert warm.manager.find_prefix_hit(prompts[1]).num_pages == 2          # 32 of the 40 shared tokens
    second = None
    while not warm.is_finished():
        for _, t in warm.step()[0]:
            second = t
    assert [first, second] == want
    helpers.assert_greedy_like_plain(folder, prompts, want, True, "prefix hits")


def test_replay_program_on_cpu(folders, plain_backend, tmp_path, monkeypatch, capsys):
    """bin/trace_run's loop, in process: steps from stdin, <step>.f32 files, `done` lines."""
    from mini_engine_amd import replay
    folder = folders("B")
    a, b = helpers.random_ids(30, 384, 1), helpers.random_ids(12, 384, 2)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:20], "want": [19]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[20:21], "want": [0]}, {"id": "b", "tokens": b[:7], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[7:], "want": [0, 4]}], "end": ["b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": a[21:], "want": list(range(9))}], "end": ["a"]},
    ]
    monkeypatch.setattr("sys.stdin", io.StringIO("\n".join(json.dumps(s) for s in steps) + "\n"))
    real = replay.Replayer
    monkeypatch.setattr(replay, "Replayer", lambda m, d, n, p: real(m, d, n, p, device="cpu", poison_cache=True))
    assert replay.main(["--model", folder, "--dtype", "float32", "--out", str(tmp_path / "o"), "--max-tokens", "128",
                        "--page-size", "8"]) == 0
    assert capsys.readouterr().out.split("\n")[:4] == ["done 0", "done 1", "done 2", "done 3"]
    import numpy as np
    ra, rb = helpers.plain_logits(folder, a), helpers.plain_logits(folder, b)
    def rd(i):
        return torch.from_numpy(np.fromfile(str(tmp_path / "o" / f"{i}.f32"), dtype="<f4").reshape(-1, 384))
    assert helpers.rel_err(rd(0), ra[19:20]) <= helpers.TOL_F32
    assert helpers.rel_err(rd(1), ra[20:21]) <= helpers.TOL_F32
    assert helpers.rel_err(rd(2), rb[[7, 11]]) <= helpers.TOL_F32
    assert helpers.rel_err(rd(3), ra[21:]) <= helpers.TOL_F32


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_padded_decode_layout_without_capture(folders, plain_backend, name):
    """The fixed-layout decode step that HIP graphs replay (batch padded to a bucket, block tables
    kept between steps and patched, rows changing owner), run eagerly on the CPU."""
    V, page, folder = helpers.CONFIGS[name]["vocab_size"], helpers.PAGE[name], folders(name)
    model = load_model(folder, "cpu", torch.float32, 512)
    manager = CacheManager(80, page, ModelRunner.windows_of(model), enable_prefix_caching=False)
    runner = ModelRunner(model, manager, torch.float32, "cpu", 512, poison_cache=True, use_graphs=True)
    lens = {"a": 70, "b": 9, "c": 33, "d": 130, "e": 17}
    ids = {r: helpers.random_ids(n + 24, V, 70 + i) for i, (r, n) in enumerate(lens.items())}
    d = helpers.Driver(runner, manager)
    d.step({r: ids[r][:lens[r]] for r in ("a", "b", "c")})
    pos, live = dict(lens), ["a", "b", "c"]
    for t in range(24):
        if t == 5:
            d.step({"d": ids["d"][:lens["d"]]}); live.append("d")
        if t == 9:
            live.remove("b"); manager.free("b"); d.fed.pop("b")
        if t == 12:
            d.step({"e": ids["e"][:lens["e"]]}); live.insert(0, "e")
        d.step({r: ids[r][pos[r]:pos[r] + 1] for r in live})
        for r in live:
            pos[r] += 1
    assert runner.graphs.replays == 24
    for r in lens:
        got = d.result(r)
        assert helpers.rel_err(got, helpers.plain_logits(folder, ids[r][:got.shape[0]])) <= helpers.TOL_F32, r


@pytest.mark.parametrize("limit", [100, 43])
def test_fixed_layouts_with_a_longest_context_that_is_no_multiple_of_8(folders, plain_backend, limit):
    """The fixed layouts round their block tables up; what they tell the kernels about the longest context must
    not go beyond the engine's limit, which is where the position encoding's table ends (the twins assert it)."""
    V, page, folder = helpers.CONFIGS["A"]["vocab_size"], helpers.PAGE["A"], folders("A")
    model = load_model(folder, "cpu", torch.float32, limit)
    assert model.layers[0].mixer.position.rotary_table().shape[0] == limit
    manager = CacheManager(20, page, ModelRunner.windows_of(model), enable_prefix_caching=False)
    runner = ModelRunner(model, manager, torch.float32, "cpu", limit, poison_cache=True, use_graphs=True,
                         mixed_graphs_after=0, mixed_graphs_max_tokens=4096)
    ids = helpers.random_ids(limit, V, 77)
    d = helpers.Driver(runner, manager)
    d.step({"r": ids[:limit - 6]})
    for t in range(limit - 6, limit):
        d.step({"r": ids[t:t + 1]})
    assert runner.graphs.replays == 6
    assert all(c.context().max_decode_context <= limit for c in runner.graphs.captured.values())
    assert helpers.rel_err(d.result("r"), helpers.plain_logits(folder, ids)) <= helpers.TOL_F32


def test_a_padding_request_longer_than_the_longest_context_is_not_made(folders, plain_backend):
    """Three prompts of 43 tokens under a limit of 64: rounded up to 256 tokens the padding request would hold 126
    tokens, at positions the engine does not have. Such a step runs exactly sized instead."""
    from mini_engine_amd.engine.packing import exact_layout, pack_step
    import numpy as np
    V, page, folder = helpers.CONFIGS["A"]["vocab_size"], helpers.PAGE["A"], folders("A")
    model = load_model(folder, "cpu", torch.float32, 64)
    manager = CacheManager(20, page, ModelRunner.windows_of(model), enable_prefix_caching=False)
    runner = ModelRunner(model, manager, torch.float32, "cpu", 64, poison_cache=True, use_graphs=True,
                         mixed_graphs_after=0, mixed_graphs_max_tokens=4096)
    ids = {r: helpers.random_ids(43, V, 80 + i) for i, r in enumerate("abc")}
    d = helpers.Driver(runner, manager)
    d.step(ids)
    assert runner.mixed_graphs.replays == 0
    d.step({"a": [5, 6]})                      # a small step still takes a padded layout
    assert runner.mixed_graphs.replays == 1
    for r in "abc":
        assert helpers.rel_err(d.result(r)[:43], helpers.plain_logits(folder, ids[r])) <= helpers.TOL_F32, r
    # and the packing itself refuses a padding request whose pages do not fit the layout's tables
    exact = exact_layout([43], [0], [[[0, 1, 2]]], 0, lambda *a: False)
    import dataclasses
    wide = dataclasses.replace(exact, prefill_reqs=2, prefill_tokens=43 + 100)
    with pytest.raises(ValueError, match="padding request"):
        pack_step(wide, np.zeros(wide.segments()[1], dtype=np.int32), [list(range(43))], [0], [[[0, 1, 2]]], [-1], [],
                  page, [9], 0, V)


def test_decode_rows_follow_a_request_that_was_fed_again(folders, plain_backend):
    """Decode steps that continue the one before carry their tables and slots on; a request that gave
    its pages back and was fed again sits at the same positions on other pages, and must be looked up."""
    V, page, folder = helpers.CONFIGS["A"]["vocab_size"], helpers.PAGE["A"], folders("A")
    model = load_model(folder, "cpu", torch.float32, 512)
    manager = CacheManager(80, page, ModelRunner.windows_of(model), enable_prefix_caching=False)
    runner = ModelRunner(model, manager, torch.float32, "cpu", 512, poison_cache=True, use_graphs=True)
    ids = {r: helpers.random_ids(40 + 4 * page + 8, V, 40 + i) for i, r in enumerate(("a", "c", "x"))}
    d = helpers.Driver(runner, manager)
    d.step({"a": ids["a"][:40], "c": ids["c"][:33]})
    pos = {"a": 40, "c": 33}

    def decode(n):
        for _ in range(n):
            d.step({r: ids[r][pos[r]:pos[r] + 1] for r in ("a", "c")})
            for r in pos:
                pos[r] += 1

    decode(2 * page + 3)                                   # across page edges
    carried = runner.graphs.advances
    assert carried >= 2 * page
    before = list(manager.block_table("c"))
    manager.free("c"); d.fed.pop("c")
    d.step({"x": ids["x"][:pos["c"]]}, want_all=False)     # takes the pages c gave back
    d.step({"c": ids["c"][:pos["c"]]}, want_all=False)     # c again, whole, on other pages
    assert manager.block_table("c") != before
    decode(1)
    assert runner.graphs.advances == carried               # not carried on: the tables were read again
    decode(page + 2)
    assert runner.graphs.advances == carried + page + 2
    for r in ("a", "c"):
        got = d.result(r)
        assert helpers.rel_err(got, helpers.plain_logits(folder, ids[r][:got.shape[0]])) <= helpers.TOL_F32, r


def test_decode_layouts_are_dropped_least_recently_used_first(folders, plain_backend):
    """Only so many (batch bucket, context cap) layouts are kept; one that was dropped is built again."""
    V, page, folder = helpers.CONFIGS["A"]["vocab_size"], helpers.PAGE["A"], folders("A")
    model = load_model(folder, "cpu", torch.float32, 512)
    manager = CacheManager(120, page, ModelRunner.windows_of(model), enable_prefix_caching=False)
    runner = ModelRunner(model, manager, torch.float32, "cpu", 512, poison_cache=True, use_graphs=True)
    runner.graphs.max_graphs = 4
    names = [f"r{i}" for i in range(9)]
    ids = {r: helpers.random_ids(40, V, 300 + i) for i, r in enumerate(names)}
    d = helpers.Driver(runner, manager)
    d.step({r: ids[r][:20] for r in names})
    pos = 20
    for count in (1, 2, 3, 5, 9, 1, 9, 2):                 # buckets 1, 2, 4, 8, 16, then some of them again
        d.step({r: ids[r][pos:pos + 1] for r in names[:count]})
        for r in names[count:]:                            # the others keep pace through a step of their own
            d.step({r: ids[r][pos:pos + 1]})
        pos += 1
        assert len(runner.graphs.captured) <= 4
    for r in names:
        got = d.result(r)
        assert helpers.rel_err(got, helpers.plain_logits(folder, ids[r][:got.shape[0]])) <= helpers.TOL_F32, r


def test_toy_architecture_on_cpu(plain_backend):
    """A stateful mixer, a layer run twice, a call that reads another call's cache and an unfused
    position encoding, registered from tests/toy_arch.py, stepped through the real runner."""
    import toy_arch
    toy_arch.run_toy("cpu", torch.float32, 1e-5)


def test_toy_architecture_through_the_engine_on_cpu(plain_backend):
    """The same toy architecture from a written folder through `LLM.generate`: scheduler, state slots and a
    second page group under admission, eviction and finish, the decode steps' fixed layout, steps run ahead."""
    import toy_arch
    toy_arch.run_toy_engine("cpu", "float32", capture=False)


import policy_cases


@pytest.mark.parametrize("case", policy_cases.ALL, ids=lambda c: c.__name__)
def test_policies_with_a_model_on_cpu(folders, plain_backend, case):
    case(_llm, folders, exact=True)


def test_a_part_that_needs_the_host_keeps_its_model_out_of_the_graphs(plain_backend, monkeypatch):
    """A part may declare that its forward reads values on the host (`capturable = False`): a model that
    contains it is never captured, whatever the engine was asked for."""
    import toy_arch
    from mini_engine_amd.registry import build_model
    from mini_engine_amd.weights.random_init import fill_random
    model = fill_random(build_model(toy_arch.ToyConfig.from_dict({"vocab_size": 50, "hidden_size": 40, "eps": 1e-5})),
                        4, "cpu", torch.float32, 64)
    manager = lambda: CacheManager(8, 8, ModelRunner.windows_of(model), num_state_slots=2)
    assert ModelRunner(model, manager(), torch.float32, "cpu", 64, use_graphs=True).graphs is not None
    monkeypatch.setattr(toy_arch.RunningMean, "capturable", False)
    runner = ModelRunner(model, manager(), torch.float32, "cpu", 64, use_graphs=True)
    assert runner.graphs is None and runner.mixed_graphs is None
