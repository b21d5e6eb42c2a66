"""Scheduling policies and engine options run with a model through `LLM.generate`, each compared with the
plain implementation's greedy tokens. `make(folder, **options)` builds the engine (on the GPU, or on the CPU
with the plain kernel twins); `exact`: float32 (tokens must be equal) or bfloat16 (near-ties may differ)."""
import helpers


def _greedy(n):
    from mini_engine_amd import SamplingParams
    return SamplingParams(temperature=0, max_tokens=n, ignore_eos=True)


def priority_policy(make, folders, exact):
    """Mixed priorities under a pool so small that the least urgent request is evicted and fed again."""
    folder = folders("B")
    prompts = [helpers.random_ids(n, 384, 300 + n) for n in (24, 9, 40, 17, 33)]
    llm = make(folder, scheduling_policy="priority", kvcache_block_size=8, num_kvcache_blocks=13, max_num_seqs=4,
               max_num_batched_tokens=32, max_model_len=64, enable_prefix_caching=False)
    outs = llm.generate(prompts, _greedy(10), use_tqdm=False, priorities=[2, 0, 1, 0, 2])
    assert llm.scheduler.num_preemptions > 0, "the pool was large enough that nobody was evicted"
    helpers.assert_greedy_like_plain(folder, prompts, [o["token_ids"] for o in outs], exact, "priority")
    llm.manager.check_invariants()
    assert llm.manager.num_free_pages() == 13


def priority_order(make, folders, exact):
    """With room for one request at a time, requests finish in the order of (priority, arrival)."""
    from mini_engine_amd import SamplingParams
    folder = folders("A")
    llm = make(folder, scheduling_policy="priority", kvcache_block_size=16, num_kvcache_blocks=8, max_num_seqs=1,
               max_num_batched_tokens=64, max_model_len=64)
    prompts = [helpers.random_ids(6, 256, 40 + i) for i in range(5)]
    ranks = [3, 1, 2, 1, 0]
    ids = [llm.add_request(p, SamplingParams(temperature=0, max_tokens=3, ignore_eos=True), priority=r)
           for p, r in zip(prompts, ranks)]
    finished, outs = [], {}
    while not llm.is_finished():
        for rid, toks in llm.step()[0]:
            finished.append(rid); outs[rid] = toks
    assert finished == [ids[i] for i in (4, 1, 3, 2, 0)]
    helpers.assert_greedy_like_plain(folder, prompts, [outs[i] for i in ids], exact, "priority order")


def long_prefill_threshold(make, folders, exact):
    """Prompts go in five tokens at a time beside requests that already decode."""
    folder = folders("B")
    prompts = [helpers.random_ids(n, 384, 310 + n) for n in (3, 23, 41, 12)]
    llm = make(folder, long_prefill_token_threshold=5, kvcache_block_size=8, num_kvcache_blocks=40, max_num_seqs=4,
               max_num_batched_tokens=32, max_model_len=64)
    sizes = []
    step = llm.step

    def counting():
        out = step()
        sizes.append(out[1])
        return out
    llm.step = counting
    try:
        outs = llm.generate(prompts, _greedy(9), use_tqdm=False)
    finally:
        del llm.step                    # the wrapper refers to the engine: no reference cycle is left behind
    assert max(sizes) <= 4 * 5 and any(0 < s <= 5 for s in sizes), sizes       # no request ran more than 5 prompt tokens a step
    helpers.assert_greedy_like_plain(folder, prompts, [o["token_ids"] for o in outs], exact, "threshold")


def prefill_first(make, folders, exact):
    """Whole prompts first, decoding only in steps that admit nobody; a pool that forces evictions."""
    folder = folders("A")
    prompts = [helpers.random_ids(n, 256, 320 + n) for n in (15, 31, 16, 47, 14, 30)]
    llm = make(folder, enable_chunked_prefill=False, kvcache_block_size=16, num_kvcache_blocks=6, max_num_seqs=3,
               max_num_batched_tokens=64, max_model_len=64, enable_prefix_caching=False)
    outs = llm.generate(prompts, _greedy(12), use_tqdm=False)
    assert llm.scheduler.num_preemptions > 0
    helpers.assert_greedy_like_plain(folder, prompts, [o["token_ids"] for o in outs], exact, "prefill first")
    assert llm.manager.num_free_pages() == 6


def many_live_requests(make, folders, exact):
    """300 requests decoding together: more rows than any power-of-two layout up to 256 holds."""
    folder = folders("A")
    prompts = [helpers.random_ids(2 + i % 7, 256, 1000 + i) for i in range(300)]
    llm = make(folder, kvcache_block_size=16, num_kvcache_blocks=300, max_num_seqs=300, max_num_batched_tokens=4096,
               max_model_len=16)
    outs = llm.generate(prompts, _greedy(4), use_tqdm=False)
    assert len(llm.scheduler.running) == 0 and llm.runner.graphs.replays >= 3
    assert any(c.bucket == 384 for c in llm.runner.graphs.captured.values())
    helpers.assert_greedy_like_plain(folder, prompts[::13], [o["token_ids"] for o in outs][::13], exact, "300 live")


def windowed_model(make, folders, exact):
    """Tiny C (sliding windows on two of four layers: two page groups) through the scheduler: pages behind the
    window given back while requests run, evictions and feeding again, steps run ahead or not."""
    folder = folders("C")
    prompts = [helpers.random_ids(n, 300, 330 + n) for n in (5, 50, 33, 70, 18)]
    for options in (dict(num_kvcache_blocks=40, max_num_batched_tokens=64),
                    dict(num_kvcache_blocks=11, max_num_batched_tokens=16, run_ahead=True),
                    dict(num_kvcache_blocks=11, max_num_batched_tokens=16, run_ahead=False),
                    dict(num_kvcache_blocks=14, max_num_batched_tokens=128, enable_chunked_prefill=False)):
        llm = make(folder, kvcache_block_size=16, max_num_seqs=4, max_model_len=128, **options)
        outs = llm.generate(prompts, _greedy(16), use_tqdm=False)
        if options["num_kvcache_blocks"] == 11:
            assert llm.scheduler.num_preemptions > 0, "nobody was evicted"
        helpers.assert_greedy_like_plain(folder, prompts, [o["token_ids"] for o in outs], exact, f"windowed {options}")
        llm.manager.check_invariants()
        assert all(llm.manager.num_free_pages(g) == options["num_kvcache_blocks"] for g in range(2))


def eviction_with_prefix_cache(make, folders, exact):
    """Prefix caching on (the engine's default), six requests that share their first three pages, a pool so small
    that requests are evicted: a request that is fed again finds pages of its own tokens (the shared prefix, or what
    it had published itself) and must still give the plain model's tokens. Chunked under two budgets and whole
    prompts first, steps run ahead or not."""
    folder = folders("A")
    shared = helpers.random_ids(48, 256, 340)
    prompts = [shared + helpers.random_ids(n, 256, 341 + n) for n in (5, 20, 9, 30, 14, 3)]
    for options in (dict(max_num_batched_tokens=16), dict(max_num_batched_tokens=64),
                    dict(max_num_batched_tokens=128, enable_chunked_prefill=False)):
        for run_ahead in (True, False):
            llm = make(folder, kvcache_block_size=16, num_kvcache_blocks=10, max_num_seqs=4, max_model_len=128,
                       enable_prefix_caching=True, run_ahead=run_ahead, **options)
            assert llm.manager.prefix_caching
            outs = llm.generate(prompts, _greedy(24), use_tqdm=False)
            what = f"prefix cache + eviction {options} run_ahead={run_ahead}"
            assert llm.scheduler.num_preemptions > 0, f"{what}: nobody was evicted"
            assert llm.scheduler.num_prefix_hits_after_eviction > 0, f"{what}: no request that was fed again found cached pages"
            helpers.assert_greedy_like_plain(folder, prompts, [o["token_ids"] for o in outs], exact, what)
            llm.manager.check_invariants()
            assert llm.manager.num_free_pages() == 10


def sampled_tokens_follow_their_keys(make, folders, exact):
    """Temperature 0.8: output number i of request r is argmax(plain logits / T - log E) with the noise E keyed by
    (seed, r's noise stream, i), the key derived here by the test's own code. A key that left out the seed, the
    request or the output index would give other tokens. Prompts are chunked under a budget of 16 and one request
    brings a seed of its own."""
    import torch
    import kernel_twins
    import plain_qwen3
    from mini_engine_amd import SamplingParams
    folder = folders("B")
    cfg, w = plain_qwen3.read_model_folder(folder, torch.float64)
    prompts = [helpers.random_ids(n, 384, 960 + n) for n in (1, 9, 24, 40)]
    T = 0.8
    sps = [SamplingParams(temperature=T, max_tokens=10, ignore_eos=True, seed=(77 if i == 2 else None)) for i in range(4)]
    llm = make(folder, kvcache_block_size=8, num_kvcache_blocks=64, max_num_seqs=4, max_num_batched_tokens=16,
               max_model_len=128, seed=3)
    outs = [o["token_ids"] for o in llm.generate(prompts, sps, use_tqdm=False)]
    seen_keys = set()
    not_greedy = 0
    for r, (prompt, out) in enumerate(zip(prompts, outs)):
        ids = list(prompt)
        for i, tok in enumerate(out):
            z = plain_qwen3.logits(cfg, w, ids)[-1]
            key = kernel_twins.row_key(77 if r == 2 else 3, r, i)
            seen_keys.add(key)
            keys = torch.tensor([key], dtype=torch.int64).to(torch.int32)      # the words' bits, as the kernel takes them
            score = kernel_twins.sample_scores(z.float()[None, :], torch.tensor([T]), keys)[0].double()
            best = int(score.argmax())
            not_greedy += tok != int(z.argmax())
            # the engine's logits differ from the plain model's within its tolerance; a token other than the best
            # passes only where the two scores lie closer than that
            tol = (helpers.TOL_F32 if exact else helpers.TOL_BF16) * float(z.abs().max()) / T
            assert tok == best or float(score[best] - score[tok]) <= tol, \
                f"request {r}, output {i}: sampled {tok}, the keyed noise on the plain logits gives {best}"
            ids.append(tok)
    assert len(seen_keys) == 40
    assert not_greedy >= 10, "the noise changed next to nothing: the case tests nothing"


ALL = [eviction_with_prefix_cache, sampled_tokens_follow_their_keys, priority_policy, priority_order, long_prefill_threshold, prefill_first, many_live_requests, windowed_model]
