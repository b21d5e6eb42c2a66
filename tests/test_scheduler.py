"""The scheduler's decisions, driven without a model: budget, order, chunking, admission,
what happens when pages run out. No GPU."""
from types import SimpleNamespace

import pytest

from mini_engine_amd.cache.manager import CacheManager
from mini_engine_amd.engine.scheduler import Scheduler
from mini_engine_amd.engine.sequence import Sequence, SequenceStatus
from mini_engine_amd.sampling.sampling_params import SamplingParams


def make(pages=64, page=4, seqs=8, budget=16, chunked=True, policy="fcfs", threshold=0, max_len=256, eos=-1):
    cfg = SimpleNamespace(max_num_seqs=seqs, max_num_batched_tokens=budget, long_prefill_token_threshold=threshold,
                          enable_chunked_prefill=chunked, scheduling_policy=policy, eos=eos, max_model_len=max_len)
    m = CacheManager(pages, page)
    return Scheduler(cfg, m), m


def seq(n, max_tokens=4, prio=0, base=0, **kw):
    return Sequence(list(range(base, base + n)), SamplingParams(temperature=0, max_tokens=max_tokens, **kw), prio)


def run_step(s, token=7):
    batch = s.schedule()
    sizes = [(q.seq_id, q.num_scheduled_tokens) for q in batch]
    s.postprocess(batch, [token if q.samples_this_step else None for q in batch])
    s.manager.check_invariants()
    return sizes


def test_chunks_under_budget_decodes_first():
    s, m = make(budget=16)
    a, b = seq(40, base=0), seq(10, base=100)
    s.add(a); s.add(b)
    assert run_step(s) == [(a.seq_id, 16)]                      # head of line takes the whole budget
    assert run_step(s) == [(a.seq_id, 16)]
    assert run_step(s) == [(a.seq_id, 8), (b.seq_id, 8)]        # a's rest, then b admitted into what is left
    # now a decodes (1 token) and is scheduled before b's partial prompt
    assert run_step(s) == [(a.seq_id, 1), (b.seq_id, 2)]
    assert run_step(s) == [(a.seq_id, 1), (b.seq_id, 1)]
    assert a.num_completion_tokens == 3 and b.num_completion_tokens == 2


def test_every_step_respects_budget_and_max_seqs():
    s, m = make(budget=12, seqs=3, pages=200)
    for i in range(7):
        s.add(seq(5 + 7 * i, max_tokens=6, base=1000 * i))
    steps = 0
    while not s.is_finished():
        batch = s.schedule()
        assert sum(q.num_scheduled_tokens for q in batch) <= 12
        assert len(s.running) <= 3
        assert len({q.seq_id for q in batch}) == len(batch)
        s.postprocess(batch, [3 if q.samples_this_step else None for q in batch])
        m.check_invariants()
        steps += 1
        assert steps < 500
    assert m.num_free_pages() == 200


def test_long_prefill_threshold_caps_a_chunk():
    s, m = make(budget=16, threshold=5)
    a = seq(12); s.add(a)
    assert run_step(s) == [(a.seq_id, 5)]
    assert run_step(s) == [(a.seq_id, 5)]
    assert run_step(s) == [(a.seq_id, 2)]


def test_finish_on_max_tokens_and_eos_frees_pages():
    s, m = make(eos=7)
    a = seq(3, max_tokens=5); b = seq(3, max_tokens=5, base=50, ignore_eos=True)
    s.add(a); s.add(b)
    run_step(s, token=7)                                         # both sample the eos token
    assert a.is_finished and not m.holds(a.seq_id)               # stopped by eos
    assert not b.is_finished                                     # ignore_eos keeps going
    for _ in range(4):
        run_step(s, token=7)
    assert b.is_finished and b.num_completion_tokens == 5 and m.num_free_pages() == 64


def test_admission_errors():
    s, m = make(max_len=32, pages=4, page=4)
    with pytest.raises(ValueError, match="max_model_len"):
        s.add(seq(30, max_tokens=8))
    with pytest.raises(ValueError, match="pages"):
        s.add(seq(14, max_tokens=8))                              # 22 tokens need 6 pages of 4


def test_out_of_pages_preempts_newest_and_recomputes():
    s, m = make(pages=6, page=4, budget=64, max_len=24)
    a, b = seq(8, max_tokens=12, base=0), seq(8, max_tokens=12, base=100)
    s.add(a); s.add(b)
    run_step(s)                                                   # both prompts in (2 pages each) -> 9 tokens each
    assert m.num_free_pages() == 2
    for _ in range(4):
        run_step(s)                                               # positions 8..11: 3 pages each, pool full
    assert m.num_free_pages() == 0 and s.num_preemptions == 0
    sizes = run_step(s)                                           # a needs a 4th page: b (newest) is preempted
    assert s.num_preemptions == 1 and sizes == [(a.seq_id, 1)]    # nothing new admitted in that step
    assert b.status == SequenceStatus.WAITING and b.num_computed_tokens == 0 and s.waiting[0] is b
    assert not m.holds(b.seq_id)
    # b comes back as one prompt of prompt + generated tokens when there is room
    done = 0
    while not s.is_finished():
        run_step(s); done += 1
        assert done < 100
    assert a.num_completion_tokens == 12 and b.num_completion_tokens == 12
    assert m.num_free_pages() == 6


def test_lone_request_that_cannot_grow_preempts_itself_then_fails_loudly():
    s, m = make(pages=2, page=4, budget=64, max_len=8)
    a = seq(7, max_tokens=1)
    s.add(a)
    m.allocate("squatter", 0, 4)                                  # someone else holds half the pool
    with pytest.raises(RuntimeError, match="nothing schedulable"):
        s.schedule()


def test_head_of_line_blocking_no_overtaking():
    s, m = make(pages=4, page=4, budget=64, max_len=16)
    big, small = seq(12, max_tokens=2), seq(2, max_tokens=2, base=100)
    m.allocate("squatter", 0, 8)
    s.add(big); s.add(small)
    with pytest.raises(RuntimeError):
        s.schedule()                                              # big does not fit; small may not overtake it
    m.free("squatter")
    assert [q.seq_id for q in s.schedule()] == [big.seq_id, small.seq_id]


def test_priority_policy_orders_waiting_and_picks_victim():
    s, m = make(policy="priority", pages=6, page=4, budget=64, max_len=24)
    lo, hi = seq(8, max_tokens=12, prio=5), seq(8, max_tokens=12, prio=1, base=100)
    s.add(lo); s.add(hi)
    assert [q.seq_id for q in s.waiting] == [hi.seq_id, lo.seq_id]
    for _ in range(5):
        run_step(s)
    assert s.num_preemptions == 0
    run_step(s)                                                   # out of pages: the least urgent goes
    assert s.num_preemptions == 1 and lo.status == SequenceStatus.WAITING and hi.status == SequenceStatus.RUNNING


def test_prefill_first_policy():
    s, m = make(chunked=False, budget=32, max_len=32)
    a, b, c = seq(10), seq(20, base=100), seq(5, base=200)
    s.add(a); s.add(b); s.add(c)
    assert run_step(s) == [(a.seq_id, 10), (b.seq_id, 20)]        # whole prompts only; c (5 > 2 left) waits
    assert run_step(s) == [(c.seq_id, 5)]                         # prefill goes before any decode
    assert run_step(s) == [(a.seq_id, 1), (b.seq_id, 1), (c.seq_id, 1)]


def test_prefix_hit_shortens_the_prompt():
    s, m = make(pages=32, page=4, budget=64)
    a = seq(13, max_tokens=1); s.add(a); run_step(s)              # computes and publishes 3 full pages
    b = Sequence(list(range(13)) + [77, 78], SamplingParams(temperature=0, max_tokens=1)); s.add(b)
    batch = s.schedule()
    assert batch[0] is b and b.num_cached_tokens == 12 and b.num_scheduled_tokens == 3
    assert b.num_computed_tokens == 12
