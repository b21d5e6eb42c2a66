"""The engine on the GPU with its HIP kernels, in float32 and in bfloat16, against the plain
implementation, under every way of cutting the work; generation through the entry point."""
import pytest
import torch

import engine_cases
import helpers
import plain_qwen3
from mini_engine_amd.cache.manager import CacheManager
from mini_engine_amd.engine.runner import ModelRunner
from mini_engine_amd.weights.loader import load_model

pytestmark = pytest.mark.gpu


class Env:
    device = "cuda"

    def __init__(self, folders, dtype, graphs=False, max_positions=512):
        self.folders, self.dtype, self.max_positions = folders, dtype, max_positions
        self.padded_up_to = 4096
        self.graphs = graphs           # every step through a captured graph of its padded layout
        self.tol = helpers.TOL_F32 if dtype == torch.float32 else helpers.TOL_BF16
        self.models = {}

    def runner(self, name, pages):
        folder = self.folders(name)
        if name not in self.models:
            self.models[name] = load_model(folder, self.device, self.dtype, self.max_positions)
        model = self.models[name]
        manager = CacheManager(pages, helpers.PAGE[name], ModelRunner.windows_of(model), enable_prefix_caching=False)
        options = dict(use_graphs=True, mixed_graphs_after=0, mixed_graphs_max_tokens=self.padded_up_to) if self.graphs else {}
        return ModelRunner(model, manager, self.dtype, self.device, self.max_positions, poison_cache=True, **options), manager, folder


@pytest.fixture(scope="module", params=[torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def env(request, folders):
    return Env(folders, request.param)


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("case", engine_cases.ALL, ids=lambda c: c.__name__)
def test_cuts(env, case, name):
    case(env, name)


@pytest.mark.parametrize("captured", [False, True], ids=["eager", "graphs"])
def test_many_rows_at_the_layer_sizes_of_a_real_model(folders, captured):
    """Two layers at the Qwen3-0.6B layer sizes in bfloat16, batches of 40, 12 and 3 requests, against the plain
    implementation: the tiny configurations never reach the products in slices of a long K, the wide loads, the
    library's products or head size 128 inside the engine."""
    from mini_engine_amd.kernels import ops
    # what the 40 rows of a decode step go through at these sizes: o and down in eight slices by the tiled kernel, gate/up
    # with the gating in that kernel's epilogue; 12 rows: the skinny kernel's split of K; contexts of 90-1,500 keys: partitions
    assert ops.mid_takes(40, 1024, 2048, True) == 8 and ops.mid_takes(40, 1024, 3072, True) == 8
    assert ops.mid_takes(40, 6144, 1024, False) == 1 and ops.choose_ksplit(12, 1024, 2048) > 1
    assert ops.decode_partitions(12, 16, 8, 580)[1] > 1 and ops.decode_partitions(3, 16, 8, 1520)[1] > 1
    engine_cases.many_rows_at_real_layer_sizes(Env(folders, torch.bfloat16, graphs=captured, max_positions=2048))


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("case", [engine_cases.whole, engine_cases.tail_one_by_one, engine_cases.changing_portions,
                                  engine_cases.mixed_with_reuse, engine_cases.wanted_rows_only], ids=lambda c: c.__name__)
def test_cuts_through_captured_steps(env, case, name):
    """The cuts again with every step, prompt portions and mixed ones too, replayed from a captured graph of its
    padded layout (padding rows, a padding request, wider tables, spare logits rows)."""
    graphs = Env(env.folders, env.dtype, graphs=True)
    graphs.models = env.models
    case(graphs, name)


@pytest.mark.parametrize("name", ["A", "C"])
def test_padded_layouts_are_captured_and_replayed(env, name):
    graphs = Env(env.folders, env.dtype, graphs=True)
    graphs.models = env.models
    engine_cases.padded_layouts_are_used(graphs, name, captured=True)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_exactly_sized_layouts_are_captured_and_replayed(env, name):
    graphs = Env(env.folders, env.dtype, graphs=True)
    graphs.models, graphs.padded_up_to = env.models, 16
    engine_cases.exactly_sized_layouts_are_used(graphs, name, captured=True)
    engine_cases.mixed_with_reuse(graphs, name)


def test_hip_libraries_are_the_ones_running(env):
    from mini_engine_amd.kernels import ops
    env.runner("A", 2)
    engine_cases.first_tokens(env, "A")
    assert isinstance(ops.backend(), ops.HipBackend)
    libs = ops.loaded_libraries()
    assert any("libme_core.so" in p for p in libs)
    if env.dtype == torch.bfloat16:
        assert any("libme_attn_d16.so" in p for p in libs)


def _llm(folder, dtype, **kw):
    from mini_engine_amd import LLM
    return LLM(folder, dtype=dtype, poison_cache=True, **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generate_greedy_matches_plain(folders, dtype):
    """Tiny A (prompts of 5, 17 and 33 tokens, 8 greedy tokens each) and untied tiny B. In bfloat16
    a token may differ only where the plain model's two best logits are closer than the tolerance."""
    from mini_engine_amd import SamplingParams
    for name, page in (("A", 16), ("B", 8)):
        folder = folders(name)
        cfg, w = plain_qwen3.read_model_folder(folder, torch.float64)
        V = cfg["vocab_size"]
        prompts = [helpers.random_ids(n, V, 900 + n) for n in (5, 17, 33)]
        llm = _llm(folder, dtype, kvcache_block_size=page, num_kvcache_blocks=24, max_num_seqs=4,
                   max_num_batched_tokens=64, max_model_len=64)
        outs = llm.generate(prompts, SamplingParams(temperature=0, max_tokens=8), use_tqdm=False)
        for p, o in zip(prompts, outs):
            ids = list(p)
            for tok in o["token_ids"]:
                z = plain_qwen3.logits(cfg, w, ids)[-1]
                best = int(torch.argmax(z))
                if tok != best:
                    assert dtype == "bfloat16" and float(z[best] - z[tok]) <= helpers.TOL_BF16 * float(z.abs().max()), \
                        f"{name}: token {tok} instead of {best}"
                ids.append(tok)
        llm.manager.check_invariants()
        assert llm.manager.num_free_pages() == 24


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generate_chunked_sampled_is_independent_of_batching_and_preemption(folders, dtype):
    """Tiny B: prompts of 1, 9, 24, 40 and 63 tokens, budget 16, temperature 0.8, 12 tokens each.
    In float32 the same seed gives the same tokens together, alone, and under preemption."""
    from mini_engine_amd import SamplingParams
    folder = folders("B")
    prompts = [helpers.random_ids(n, 384, 950 + n) for n in (1, 9, 24, 40, 63)]
    sp = SamplingParams(temperature=0.8, max_tokens=12, ignore_eos=True)
    common = dict(kvcache_block_size=8, max_num_seqs=16, max_model_len=128, seed=3)
    together = _llm(folder, dtype, num_kvcache_blocks=64, max_num_batched_tokens=16, **common)
    out_together = [o["token_ids"] for o in together.generate(prompts, sp, use_tqdm=False)]
    assert all(len(o) == 12 for o in out_together)
    again = _llm(folder, dtype, num_kvcache_blocks=64, max_num_batched_tokens=16, **common)
    assert [o["token_ids"] for o in again.generate(prompts, sp, use_tqdm=False)] == out_together
    if dtype == "float32":
        tight = _llm(folder, dtype, num_kvcache_blocks=21, max_num_batched_tokens=16, enable_prefix_caching=False, **common)
        out_tight = [o["token_ids"] for o in tight.generate(prompts, sp, use_tqdm=False)]
        assert tight.scheduler.num_preemptions > 0
        assert out_tight == out_together
        wide = _llm(folder, dtype, num_kvcache_blocks=64, max_num_batched_tokens=128, **common)
        assert [o["token_ids"] for o in wide.generate(prompts, sp, use_tqdm=False)] == out_together


@pytest.mark.parametrize("seed", [11, 12, 13, 14, 15, 16])
def test_random_configurations(tmp_path, seed):
    """Configurations drawn at random (head size, heads and groups, widths and a vocabulary that are no
    powers of two, layers, page size, window, tied or not): a whole prompt, and the same in portions of
    changing size with the last 20 tokens one by one, in float32 and bfloat16, against the plain model."""
    import random
    from mini_engine_amd.config.model_config import Qwen3Config
    from mini_engine_amd.weights.random_init import write_random_model
    rng = random.Random(seed)
    Hkv, L = rng.choice([1, 2, 3, 5]), rng.choice([1, 2, 3])
    vocab, page, window = rng.choice([300, 515, 1000, 2049]), rng.choice([8, 16, 32, 64]), rng.choice([None, 24, 40])
    cfgd = dict(architectures=["Qwen3ForCausalLM"], vocab_size=vocab, hidden_size=rng.choice([72, 88, 136, 200, 264]),
                intermediate_size=rng.choice([120, 200, 328, 520]), num_hidden_layers=L,
                num_attention_heads=Hkv * rng.choice([1, 2, 3, 4, 7]), num_key_value_heads=Hkv,
                head_dim=rng.choice([16, 32, 48, 64, 128]), rms_norm_eps=rng.choice([1e-6, 1e-5]),
                rope_theta=rng.choice([1e4, 1e6]), tie_word_embeddings=rng.random() < 0.5, max_position_embeddings=4096)
    if window:
        cfgd.update(use_sliding_window=True, sliding_window=window,
                    layer_types=[rng.choice(["full_attention", "sliding_attention"]) for _ in range(L)])
    folder = write_random_model(Qwen3Config.from_dict(cfgd), seed, str(tmp_path / "model"), torch.bfloat16)
    n = rng.choice([70, 150, 300])
    ids = helpers.random_ids(n, vocab, seed)
    ref = helpers.plain_logits(folder, ids)
    cuts, pos = [], 0
    while pos < n - 20:
        cuts.append(min(rng.choice([2, 5, 17, 33, 64]), n - 20 - pos)); pos += cuts[-1]
    for dtype, tol in ((torch.float32, helpers.TOL_F32), (torch.bfloat16, helpers.TOL_BF16)):
        model = load_model(folder, "cuda", dtype, 512)
        manager = CacheManager(2 * (-(-n // page) + 2), page, ModelRunner.windows_of(model), enable_prefix_caching=False)
        runner = ModelRunner(model, manager, dtype, "cuda", 512, poison_cache=True, use_graphs=True)
        d = helpers.Driver(runner, manager)
        d.step({"whole": ids}, end=["whole"])
        pos = 0
        for c in cuts + [1] * 20:
            d.step({"cut": ids[pos:pos + c]}); pos += c
        for r in ("whole", "cut"):
            assert helpers.rel_err(d.result(r), ref) <= tol, (cfgd, page, n, dtype, r)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_running_one_step_ahead_changes_no_token(folders, dtype):
    """Decode steps launched with their tokens still on the device (taken from the sampling kernel's
    output between the metadata upload and the graph's replay) give the tokens of steps taken one
    after the other: greedy and sampled requests, ends by max_tokens and by the end token."""
    from mini_engine_amd import SamplingParams
    folder = folders("A")
    prompts = [helpers.random_ids(n, 256, 700 + n) for n in (3, 18, 33, 47)]
    sps = [SamplingParams(temperature=t, max_tokens=m) for t, m in ((0, 9), (0.7, 30), (0, 22), (0.9, 14))]
    kw = dict(kvcache_block_size=16, num_kvcache_blocks=40, max_num_seqs=8, max_num_batched_tokens=64, max_model_len=128, seed=5)
    free_run = [o["token_ids"] for o in _llm(folder, dtype, run_ahead=False, eos=-2, **kw).generate(prompts, sps, use_tqdm=False)]
    eos = free_run[1][11]
    one_by_one = _llm(folder, dtype, run_ahead=False, eos=eos, **kw)
    want = [o["token_ids"] for o in one_by_one.generate(prompts, sps, use_tqdm=False)]
    assert want == [o[:o.index(eos) + 1] if eos in o else o for o in free_run] and len(want[1]) < 30
    ahead = _llm(folder, dtype, run_ahead=True, eos=eos, **kw)
    assert [o["token_ids"] for o in ahead.generate(prompts, sps, use_tqdm=False)] == want
    assert one_by_one.steps_run_ahead == 0 and ahead.steps_run_ahead >= 15
    helpers.assert_greedy_like_plain(folder, prompts[0::2], want[0::2], dtype == "float32", "run ahead")      # the greedy ones
    ahead.manager.check_invariants()
    assert ahead.manager.num_free_pages() == 40 and not ahead.manager.held


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefix_hits_give_the_same_tokens(folders, dtype):
    """A request whose first pages were written by another request (prefix cache hit) starts its
    prompt behind them: its tokens equal those of a run without the cache."""
    from mini_engine_amd import SamplingParams
    folder = folders("A")
    shared = helpers.random_ids(40, 256, 990)
    prompts = [shared + helpers.random_ids(5, 256, 991), shared + helpers.random_ids(9, 256, 992)]
    sp = SamplingParams(temperature=0, max_tokens=6)
    kw = dict(kvcache_block_size=16, num_kvcache_blocks=16, max_num_seqs=4, max_num_batched_tokens=256, max_model_len=128)
    cold = _llm(folder, dtype, enable_prefix_caching=False, **kw)
    want = [o["token_ids"] for o in cold.generate(prompts, sp, use_tqdm=False)]
    warm = _llm(folder, dtype, **kw)
    first = warm.generate(prompts[:1], sp, use_tqdm=False)[0]["token_ids"]
    assert warm.manager.find_prefix_hit(prompts[1]).num_pages == 2          # 32 of the 40 shared tokens
    second = warm.generate(prompts[1:], sp, use_tqdm=False)[0]["token_ids"]
    assert [first, second] == want
    helpers.assert_greedy_like_plain(folder, prompts, want, dtype == "float32", "prefix hits")


def test_float32_logits_do_not_depend_on_the_cut_bitwise(folders):
    """The float32 kernels fix the order of every sum per token, so cuts agree to the last bit."""
    env = Env(folders, torch.float32)
    ids = helpers.random_ids(90, 384, 5)
    runner, manager, folder = env.runner("B", 12)
    d = helpers.Driver(runner, manager); d.step({"r": ids})
    whole = d.result("r")
    runner, manager, folder = env.runner("B", 14)
    d = helpers.Driver(runner, manager)
    other = helpers.random_ids(9, 384, 6)
    d.step({"r": ids[:31], "x": other[:2]}); d.step({"x": other[2:3], "r": ids[31:33]})
    for t in range(33, 90):
        d.step({"r": ids[t:t + 1]})
    assert torch.equal(d.result("r"), whole)


def test_pool_sizing_from_free_memory(folders):
    import gc
    from mini_engine_amd import LLM, SamplingParams
    from mini_engine_amd.cache.pool import page_bytes
    llm = LLM(folders("A"), max_num_seqs=4, max_num_batched_tokens=64, max_model_len=128, gpu_memory_utilization=0.5)
    assert llm.config.num_kvcache_blocks == 4 * 8          # capped by what max_num_seqs requests can hold
    out = llm.generate([[1, 2, 3]], SamplingParams(temperature=0, max_tokens=3), use_tqdm=False)
    assert len(out[0]["token_ids"]) == 3
    # Memory decides, not the cap: 1,024 requests of 4,096 tokens could hold 262,144 pages (1 GiB at this model's
    # 4 KiB a page), and the share of the device the engine may use is set so that about 1,000 MiB are left for them.
    del llm, out
    gc.collect()
    torch.cuda.empty_cache()
    free, total = torch.cuda.mem_get_info()
    share = ((total - free) + (1000 << 20)) / total
    llm = LLM(folders("A"), max_num_seqs=1024, max_num_batched_tokens=1024, max_model_len=4096, gpu_memory_utilization=share)
    pages = llm.config.num_kvcache_blocks
    per_page = sum(page_bytes(llm.model.cache_plan(), 16, torch.bfloat16))
    assert per_page == 2 * 2 * 2 * 16 * 16 * 2              # layers x (keys, values) x kv heads x page x head size x bytes
    assert 150000 < pages < 1024 * 256, pages
    free_now, _ = torch.cuda.mem_get_info()
    in_use = total - free_now                                # weights, workspace, the pool itself
    # what is in use and what is kept free for the steps add up to the share the engine was given: never more, and
    # less only by what the allocator rounds, a library workspace of 64 MiB that a first product may have brought, and
    # what the sizing steps held for a moment on top of what stays (scratch that grew in them: more after other tests
    # of this process have run kernels with large scratch; 257 MiB seen): 384 MiB at most, where wrong arithmetic (a factor
    # of two in a page's bytes, the weights counted twice) is off by the whole pool
    assert in_use + llm.reserved_bytes <= share * total + (8 << 20), (in_use, llm.reserved_bytes, share * total)
    assert in_use + llm.reserved_bytes >= share * total - (384 << 20), (in_use, llm.reserved_bytes, share * total)
    assert pages * per_page <= 1000 << 20


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_decode_graphs_replay_like_eager_steps(folders, dtype, name):
    """Decode steps replayed from HIP graphs give the eager step's logits, on every replay, with
    eager work (prefill of other requests, frees, reused pages) between the replays, batches that
    change size and rows that change owner."""
    env = Env(folders, dtype)
    tol = env.tol
    V = helpers.CONFIGS[name]["vocab_size"]
    page = helpers.PAGE[name]
    folder = folders(name)
    model = load_model(folder, "cuda", dtype, 512)
    manager = CacheManager(80, page, ModelRunner.windows_of(model), enable_prefix_caching=False)
    runner = ModelRunner(model, manager, dtype, "cuda", 512, poison_cache=True, use_graphs=True)
    lens = {"a": 70, "b": 9, "c": 33, "d": 130, "e": 17}
    ids = {r: helpers.random_ids(n + 24, V, 70 + i) for i, (r, n) in enumerate(lens.items())}
    d = helpers.Driver(runner, manager)
    d.step({r: ids[r][:lens[r]] for r in ("a", "b", "c")})             # eager prefill
    pos = dict(lens)
    live = ["a", "b", "c"]
    for t in range(24):
        if t == 5:
            d.step({"d": ids["d"][:lens["d"]]}); live.append("d")       # eager work between replays; bucket 3 -> 4
        if t == 9:
            live.remove("b"); manager.free("b"); d.fed.pop("b")         # rows change owner; bucket 4 -> 3
        if t == 12:
            d.step({"e": ids["e"][:lens["e"]]}); live.insert(0, "e")    # e reuses b's pages
        d.step({r: ids[r][pos[r]:pos[r] + 1] for r in live})
        for r in live:
            pos[r] += 1
    assert runner.graphs.replays >= 24
    for r in lens:
        got = d.result(r)
        err = helpers.rel_err(got, helpers.plain_logits(folder, ids[r][:got.shape[0]]))
        assert err <= tol, f"{name} {r}: {err:.3g}"


@pytest.mark.parametrize("window", [None, 100], ids=["full", "window"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_real_layer_sizes(tmp_path_factory, dtype, window):
    """Qwen3-0.6B's layer sizes (hidden 1024, 16 query / 8 key heads of 128, intermediate 3072, page 16)
    with 2 layers and a vocabulary that is no power of two: a long prompt in portions, then decoding,
    beside a second request, against the plain implementation. `window`: the second layer sees the last 100
    keys only, and the pages behind its window are given back while the first layer keeps all of them."""
    from mini_engine_amd.config.model_config import Qwen3Config
    from mini_engine_amd.weights.random_init import write_random_model
    cfgd = dict(architectures=["Qwen3ForCausalLM"], vocab_size=20011, hidden_size=1024, intermediate_size=3072,
                num_hidden_layers=2, num_attention_heads=16, num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-6,
                rope_theta=1e6, tie_word_embeddings=True, max_position_embeddings=4096)
    if window:
        cfgd.update(use_sliding_window=True, sliding_window=window, layer_types=["full_attention", "sliding_attention"])
    folder = write_random_model(Qwen3Config.from_dict(cfgd), 3, str(tmp_path_factory.mktemp("real")))
    model = load_model(folder, "cuda", dtype, 1024)
    manager = CacheManager(64, 16, ModelRunner.windows_of(model), enable_prefix_caching=False)
    runner = ModelRunner(model, manager, dtype, "cuda", 1024, poison_cache=True, use_graphs=True)
    a, b = helpers.random_ids(300, 20011, 1), helpers.random_ids(70, 20011, 2)
    d = helpers.Driver(runner, manager)
    d.step({"a": a[:200]})
    d.step({"a": a[200:263], "b": b[:64]})
    d.step({"a": a[263:290], "b": b[64:65]})
    for t in range(5):
        d.step({"a": a[290 + t:291 + t], "b": b[65 + t:66 + t]})
    d.step({"a": a[295:]})
    tol = helpers.TOL_F32 if dtype == torch.float32 else helpers.TOL_BF16
    for ids, r in ((a, "a"), (b, "b")):
        got = d.result(r)
        err = helpers.rel_err(got, helpers.plain_logits(folder, ids)[: got.shape[0]])
        assert err <= tol, f"{r}: {err:.3g}"


@pytest.mark.parametrize("hidden,Hq,Hkv,inter", [(4096, 32, 8, 12288), (5120, 64, 8, 25600)], ids=["8b_width", "32b_width"])
def test_wide_layer_sizes_take_the_products_with_partial_sums(tmp_path_factory, hidden, Hq, Hkv, inter):
    """One layer of Qwen3-8B's width (hidden 4096, 32 query / 8 key heads of 128, intermediate 12288) and of
    Qwen3-32B's (hidden 5120, 64 query / 8 key heads: groups of 8, intermediate 25600): o and down are large
    enough for the forms that hand float32 partial sums over slices of K to the norm that follows (the library
    as a strided batch at 300 and 127 rows, the rows kernel at 28 for down, the tiled kernel's slices for o), which the narrow test configurations never
    reach; then decoding; against the plain implementation."""
    from mini_engine_amd.config.model_config import Qwen3Config
    from mini_engine_amd.kernels import ops
    from mini_engine_amd.weights.random_init import write_random_model
    cfgd = dict(architectures=["Qwen3ForCausalLM"], vocab_size=1009, hidden_size=hidden, intermediate_size=inter,
                num_hidden_layers=1, num_attention_heads=Hq, num_key_value_heads=Hkv, head_dim=128, rms_norm_eps=1e-6,
                rope_theta=1e6, tie_word_embeddings=True, max_position_embeddings=4096)
    assert ops.library_splits(300, hidden, Hq * 128) > 1 and ops.library_splits(127, hidden, inter) == 8
    assert ops.rows_takes(28, hidden, inter) and ops.rows_takes(28, hidden, Hq * 128)
    folder = write_random_model(Qwen3Config.from_dict(cfgd), 5, str(tmp_path_factory.mktemp("wide")))
    model = load_model(folder, "cuda", torch.bfloat16, 1024)
    manager = CacheManager(64, 16, ModelRunner.windows_of(model), enable_prefix_caching=False)
    runner = ModelRunner(model, manager, torch.bfloat16, "cuda", 1024, poison_cache=True, use_graphs=True)
    a, b = helpers.random_ids(400, 1009, 1), helpers.random_ids(70, 1009, 2)
    d = helpers.Driver(runner, manager)
    d.step({"a": a[:300]})
    d.step({"a": a[300:363], "b": b[:64]})
    d.step({"a": a[363:390], "b": b[64:65]})
    for t in range(5):
        d.step({"a": a[390 + t:391 + t], "b": b[65 + t:66 + t]})
    d.step({"a": a[395:]})
    for ids, r in ((a, "a"), (b, "b")):
        got = d.result(r)
        err = helpers.rel_err(got, helpers.plain_logits(folder, ids)[: got.shape[0]])
        assert err <= helpers.TOL_BF16, f"{r}: {err:.3g}"


def test_single_token_rows_through_the_prefill_kernel_in_the_engine(folders, monkeypatch):
    """The mixed case of every configuration with the step's single-token rows sent through the prefill kernel
    instead of the decode kernel: a second implementation of decoding under the same cuts, against the plain
    implementation (the reference's `unified` mode, layers/attention.py:66-68)."""
    from mini_engine_amd.kernels import ops
    monkeypatch.setattr(ops, "DECODE_AS_PREFILL", True)
    env = Env(folders, torch.bfloat16)
    for name in ("A", "B", "C"):
        engine_cases.mixed_with_reuse(env, name)
        engine_cases.tail_one_by_one(env, name)
        engine_cases.batch_of_decodes(env, name)

import policy_cases


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", policy_cases.ALL, ids=lambda c: c.__name__)
def test_policies_with_a_model(folders, dtype, case):
    """Priority scheduling, a cap on prompt portions, whole prompts first, 300 requests decoding together and a
    windowed model, each through `LLM.generate` against the plain implementation's greedy tokens."""
    case(lambda folder, **kw: _llm(folder, dtype, **kw), folders, exact=dtype == "float32")
