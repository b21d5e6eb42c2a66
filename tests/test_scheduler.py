"""The scheduler's decisions, driven without a model: budget, order, chunking, admission,
what happens when pages run out; and what becomes of requests after a step, through the calls the
engine makes (`advance` when a step is launched, `settle` when its tokens arrive, `release_finished`
once no launched step writes to a request's pages). No GPU."""
import random
from types import SimpleNamespace

import pytest

from mini_engine_amd.cache.manager import CacheManager
from mini_engine_amd.engine.request import Phase, Request
from mini_engine_amd.engine.scheduler import UNKNOWN, Scheduler
from mini_engine_amd.sampling.sampling_params import SamplingParams


def make(pages=64, page=4, seqs=8, budget=16, chunked=True, policy="fcfs", threshold=0, max_len=256, eos=-1):
    cfg = SimpleNamespace(max_num_seqs=seqs, max_num_batched_tokens=budget, long_prefill_token_threshold=threshold,
                          enable_chunked_prefill=chunked, scheduling_policy=policy, eos=eos, max_model_len=max_len)
    m = CacheManager(pages, page)
    return Scheduler(cfg, m), m


def req(n, max_tokens=4, prio=0, base=0, **kw):
    return Request(list(range(base, base + n)), SamplingParams(temperature=0, max_tokens=max_tokens, **kw), prio)


def launch(s):
    """Plan a step and move its requests on, as the engine does when it launches one. Returns what
    `settle` needs later: (sizes, requests that sample, where their tokens go)."""
    batch = s.schedule()
    sizes = [(r.id, r.portion) for r in batch]
    places = [r.in_cache + r.portion for r in batch if r.in_cache + r.portion == len(r.tokens)]
    sampling = s.advance(batch)
    assert len(sampling) == len(places)
    return sizes, sampling, places


def run_step(s, token=7):
    """A step whose tokens arrive before the next one is planned."""
    sizes, sampling, places = launch(s)
    got = s.settle(sampling, [token] * len(sampling), places)
    s.release_finished(sampling)
    s.manager.check_invariants()
    assert all(UNKNOWN not in r.tokens for r in got)
    return sizes


def test_chunks_under_budget_decodes_first():
    s, m = make(budget=16)
    a, b = req(40, base=0), req(10, base=100)
    s.add(a); s.add(b)
    assert run_step(s) == [(a.id, 16)]                      # head of line takes the whole budget
    assert run_step(s) == [(a.id, 16)]
    assert run_step(s) == [(a.id, 8), (b.id, 8)]            # a's rest, then b admitted into what is left
    # now a decodes (1 token) and is scheduled before b's partial prompt
    assert run_step(s) == [(a.id, 1), (b.id, 2)]
    assert run_step(s) == [(a.id, 1), (b.id, 1)]
    assert a.num_generated == 3 and b.num_generated == 2


def test_every_step_respects_budget_and_max_seqs():
    s, m = make(budget=12, seqs=3, pages=200)
    for i in range(7):
        s.add(req(5 + 7 * i, max_tokens=6, base=1000 * i))
    steps = 0
    while not s.is_finished():
        batch = s.schedule()
        assert sum(r.portion for r in batch) <= 12
        assert len(s.running) <= 3
        assert len({r.id for r in batch}) == len(batch)
        kinds = [r.owed == 1 for r in batch if r.in_cache]                  # live ones: decodes before partial prompts
        assert kinds == sorted(kinds, reverse=True)
        places = [r.in_cache + r.portion for r in batch if r.in_cache + r.portion == len(r.tokens)]
        sampling = s.advance(batch)
        s.settle(sampling, [3] * len(sampling), places)
        s.release_finished(sampling)
        m.check_invariants()
        steps += 1
        assert steps < 500
    assert m.num_free_pages() == 200


def test_long_prefill_threshold_caps_a_chunk():
    s, m = make(budget=16, threshold=5)
    a = req(12); s.add(a)
    assert run_step(s) == [(a.id, 5)]
    assert run_step(s) == [(a.id, 5)]
    assert run_step(s) == [(a.id, 2)]


def test_finish_on_max_tokens_and_eos_frees_pages():
    s, m = make(eos=7)
    a = req(3, max_tokens=5); b = req(3, max_tokens=5, base=50, ignore_eos=True)
    s.add(a); s.add(b)
    run_step(s, token=7)                                         # both sample the eos token
    assert a.done and not m.holds(a.id) and a.generated == [7]   # stopped by eos
    assert not b.done                                            # ignore_eos keeps going
    for _ in range(4):
        run_step(s, token=7)
    assert b.done and b.num_generated == 5 and m.num_free_pages() == 64


def test_end_by_max_tokens_is_known_at_launch_and_pages_wait_for_the_token():
    s, m = make()
    a = req(3, max_tokens=2); s.add(a)
    run_step(s, token=5)
    sizes, sampling, places = launch(s)                           # the step that samples a's last token
    assert a.done and a not in s.running and a.tokens[-1] == UNKNOWN
    assert m.holds(a.id)                                          # the step in flight still writes to its pages
    assert s.is_finished()                                        # nothing left to plan
    s.settle(sampling, [9], places)
    s.release_finished(sampling)
    assert a.generated == [5, 9] and not m.holds(a.id) and m.num_free_pages() == 64


def test_end_token_of_a_step_that_ran_ahead_drops_the_token_after_it():
    """Two steps are launched before the first one's tokens arrive (what the engine does while its
    requests only decode). The first token turns out to be the end token: the second step's token is
    dropped, and the pages go back only after the second step."""
    s, m = make(eos=7)
    a, b = req(3, max_tokens=6), req(3, max_tokens=6, base=50)
    s.add(a); s.add(b)
    run_step(s, token=1)
    assert s.next_step_is_plain_decoding()
    _, first, first_places = launch(s)
    assert s.next_step_is_plain_decoding()                        # placeholders do not stop the next plan
    _, second, second_places = launch(s)
    assert a.tokens[-2:] == [UNKNOWN, UNKNOWN]
    got = s.settle(first, [7, 2], first_places)                   # a: end token; b: goes on
    assert got == [a, b] and a.done and a.generated == [1, 7] and a not in s.running
    s.release_finished([])                                        # the engine releases the step before: none
    assert m.holds(a.id)                                          # the second step still writes a's page
    got = s.settle(second, [4, 3], second_places)
    assert got == [b] and a.generated == [1, 7] and b.generated == [1, 2, 3]
    s.release_finished(first)
    assert not m.holds(a.id) and m.holds(b.id)
    m.check_invariants()


def test_admission_errors():
    s, m = make(max_len=32, pages=4, page=4)
    with pytest.raises(ValueError, match="max_model_len"):
        s.add(req(30, max_tokens=8))
    with pytest.raises(ValueError, match="pages"):
        s.add(req(14, max_tokens=8))                              # 22 tokens need 6 pages of 4


def test_out_of_pages_preempts_newest_and_recomputes():
    s, m = make(pages=6, page=4, budget=64, max_len=24)
    a, b = req(8, max_tokens=12, base=0), req(8, max_tokens=12, base=100)
    s.add(a); s.add(b)
    run_step(s)                                                   # both prompts in (2 pages each) -> 9 tokens each
    assert m.num_free_pages() == 2
    for _ in range(4):
        run_step(s)                                               # positions 8..11: 3 pages each, pool full
    assert m.num_free_pages() == 0 and s.num_preemptions == 0
    assert not s.next_step_is_plain_decoding()                    # pages could run out: such a step is not run ahead
    sizes = run_step(s)                                           # a needs a 4th page: b (newest) is preempted
    assert s.num_preemptions == 1 and sizes == [(a.id, 1)]        # nothing new admitted in that step
    assert b.phase is Phase.QUEUED and b.in_cache == 0 and s.waiting[0] is b
    assert not m.holds(b.id)
    # b comes back as one prompt of prompt + generated tokens when there is room
    done = 0
    while not s.is_finished():
        run_step(s); done += 1
        assert done < 100
    assert a.num_generated == 12 and b.num_generated == 12
    assert m.num_free_pages() == 6


def test_lone_request_that_cannot_grow_preempts_itself_then_fails_loudly():
    s, m = make(pages=2, page=4, budget=64, max_len=8)
    a = req(7, max_tokens=1)
    s.add(a)
    m.allocate("squatter", 0, 4)                                  # someone else holds half the pool
    with pytest.raises(RuntimeError, match="nothing schedulable"):
        s.schedule()


def test_head_of_line_blocking_no_overtaking():
    s, m = make(pages=4, page=4, budget=64, max_len=16)
    big, small = req(12, max_tokens=2), req(2, max_tokens=2, base=100)
    m.allocate("squatter", 0, 8)
    s.add(big); s.add(small)
    with pytest.raises(RuntimeError):
        s.schedule()                                              # big does not fit; small may not overtake it
    m.free("squatter")
    assert [r.id for r in s.schedule()] == [big.id, small.id]


def test_priority_policy_orders_waiting_and_picks_victim():
    s, m = make(policy="priority", pages=6, page=4, budget=64, max_len=24)
    lo, hi = req(8, max_tokens=12, prio=5), req(8, max_tokens=12, prio=1, base=100)
    s.add(lo); s.add(hi)
    assert [r.id for r in s.waiting] == [hi.id, lo.id]
    for _ in range(5):
        run_step(s)
    assert s.num_preemptions == 0
    run_step(s)                                                   # out of pages: the least urgent goes
    assert s.num_preemptions == 1 and lo.phase is Phase.QUEUED and hi.phase is Phase.LIVE


def test_priority_queue_stays_sorted_and_stable():
    s, m = make(policy="priority")
    rng = random.Random(3)
    reqs = [req(2, prio=rng.randint(0, 3), base=10 * i) for i in range(20)]
    for r in reqs:
        s.add(r)
    want = sorted(reqs, key=lambda r: (r.priority, r.arrived))
    assert list(s.waiting) == want


def test_prefill_first_policy():
    s, m = make(chunked=False, budget=32, max_len=32)
    a, b, c = req(10), req(20, base=100), req(5, base=200)
    s.add(a); s.add(b); s.add(c)
    assert run_step(s) == [(a.id, 10), (b.id, 20)]                # whole prompts only; c (5 > 2 left) waits
    assert run_step(s) == [(c.id, 5)]                             # prefill goes before any decode
    assert run_step(s) == [(a.id, 1), (b.id, 1), (c.id, 1)]


def test_prefix_hit_shortens_the_prompt():
    s, m = make(pages=32, page=4, budget=64)
    a = req(13, max_tokens=1); s.add(a); run_step(s)              # computes and publishes 3 full pages
    b = Request(list(range(13)) + [77, 78], SamplingParams(temperature=0, max_tokens=1)); s.add(b)
    batch = s.schedule()
    assert batch[0] is b and b.from_prefix == 12 and b.portion == 3
    assert b.in_cache == 12


def test_random_traffic_keeps_every_invariant():
    """Random arrivals, lengths, priorities and end tokens under both policies and both modes, with a pool
    so small that requests are evicted: no page lost or held twice, budget and live limit kept, every
    request ends with the right number of tokens."""
    for seed in range(6):
        rng = random.Random(seed)
        chunked = seed % 2 == 0
        s, m = make(pages=24, page=4, seqs=4, budget=40 if not chunked else 12, chunked=chunked,
                    policy="priority" if seed % 3 == 0 else "fcfs", max_len=40, eos=5)
        todo = [req(rng.randint(1, 24), max_tokens=rng.randint(1, 12), prio=rng.randint(0, 2), base=100 * i,
                    ignore_eos=rng.random() < 0.5) for i in range(14)]
        all_reqs = list(todo)
        steps = 0
        while todo or not s.is_finished():
            while todo and rng.random() < 0.6:
                s.add(todo.pop())
            if s.is_finished():
                continue
            batch = s.schedule()
            assert sum(r.portion for r in batch) <= s.token_budget and len(s.running) <= 4
            places = [r.in_cache + r.portion for r in batch if r.in_cache + r.portion == len(r.tokens)]
            sampling = s.advance(batch)
            s.settle(sampling, [rng.randint(0, 9) for _ in sampling], places)
            s.release_finished(sampling)
            m.check_invariants()
            steps += 1
            assert steps < 2000
        assert m.num_free_pages() == 24
        for r in all_reqs:
            assert r.done and 1 <= r.num_generated <= r.params.max_tokens
            if r.num_generated < r.params.max_tokens:
                assert r.tokens[-1] == 5 and not r.params.ignore_eos


def test_noise_keys_depend_on_seed_request_and_output_index():
    """The sampler's key against the test's own derivation (tests/kernel_twins.py), against SplitMix64's
    published first output for state 0, and: no two of (seed, request, output index) in a small cube share a key."""
    import kernel_twins
    from mini_engine_amd.sampling.sampler import _splitmix64, row_key
    assert _splitmix64(0) == 0xE220A8397B1DCDAF
    seen = set()
    for seed in (0, 3, 2**31, 2**63 + 5):
        for request in (0, 1, 7, 2**40):
            for index in range(6):
                key = row_key(seed, request, index)
                assert key == kernel_twins.row_key(seed, request, index)
                assert all(0 <= word < 2**32 for word in key)
                seen.add(key)
    assert len(seen) == 4 * 4 * 6
