"""Admission, chunked prefill under a token budget, decoding, finishing and freeing
(reference engine/scheduler.py:7-173; the policies and their order are the reference's).

What happens when pages run out: a running request that cannot get the pages for its next
tokens makes the scheduler preempt another running request that is not yet part of the step
(FCFS: the one admitted last; priority: the least urgent), i.e. free everything it holds and
put it back at the head of the waiting queue, from where it is later recomputed (prompt and
generated tokens as one prompt, possibly hitting its own still-cached pages). If the
requester is the only candidate left, it is preempted itself. A step in which anything was
preempted admits nothing new. A waiting request that does not fit simply waits
(head-of-line: nothing overtakes it).
"""
from __future__ import annotations

from collections import deque

from ..cache.manager import CacheManager
from .sequence import Sequence, SequenceStatus


class Scheduler:
    def __init__(self, config, manager: CacheManager):
        self.max_num_seqs = config.max_num_seqs
        self.max_num_batched_tokens = config.max_num_batched_tokens
        self.long_prefill_token_threshold = config.long_prefill_token_threshold
        self.enable_chunked_prefill = config.enable_chunked_prefill
        self.policy = config.scheduling_policy
        self.eos = config.eos
        self.max_model_len = config.max_model_len
        self.manager = manager
        self.page_size = manager.page_size
        self.waiting: deque = deque()
        self.running: list = []
        self.num_preemptions = 0

    def is_finished(self) -> bool:
        return not self.waiting and not self.running

    # -- admission ---------------------------------------------------------------------------
    def add(self, seq: Sequence) -> None:
        total = seq.num_prompt_tokens + seq.sampling_params.max_tokens
        if total > self.max_model_len:
            raise ValueError(f"prompt+max_tokens={total} exceeds max_model_len={self.max_model_len}")
        need = self.manager.pages_needed(total)
        for g in range(self.manager.num_groups):
            if need > self.manager.num_pages(g):
                raise ValueError(f"needs {need} cache pages, the pool has {self.manager.num_pages(g)}")
        self._push_waiting(seq)

    @staticmethod
    def _key(seq: Sequence):
        return (seq.priority, seq.arrival_time)

    def _push_waiting(self, seq: Sequence, front: bool = False) -> None:
        if self.policy == "priority":
            i = 0
            while i < len(self.waiting) and self._key(self.waiting[i]) <= self._key(seq):
                i += 1
            self.waiting.insert(i, seq)
        elif front:
            self.waiting.appendleft(seq)
        else:
            self.waiting.append(seq)

    def _cap(self, owed: int, budget: int) -> int:
        n = owed
        if 0 < self.long_prefill_token_threshold < n:
            n = self.long_prefill_token_threshold
        return min(n, budget)

    # -- running out of pages ----------------------------------------------------------------
    def _pick_victim(self, scheduled_ids: set) -> Sequence:
        cands = [s for s in self.running if s.seq_id not in scheduled_ids]
        if self.policy == "priority":
            return max(cands, key=self._key)
        return cands[-1]

    def _preempt(self, seq: Sequence) -> None:
        self.running.remove(seq)
        seq.status = SequenceStatus.WAITING
        seq.num_scheduled_tokens = 0
        self._release(seq)
        self._push_waiting(seq, front=True)
        self.num_preemptions += 1

    def _release(self, seq: Sequence) -> None:
        if self.manager.holds(seq.seq_id):
            self.manager.free(seq.seq_id)
        seq.num_computed_tokens = 0
        seq.num_cached_tokens = 0

    def _allocate_or_preempt(self, seq: Sequence, n: int, scheduled_ids: set) -> bool:
        while not self.manager.allocate(seq.seq_id, seq.num_computed_tokens, n):
            victim = self._pick_victim(scheduled_ids)
            self._preempt(victim)
            if victim is seq:
                return False
        return True

    def _try_start(self, seq: Sequence, budget: int, whole: bool) -> int:
        """Admit the head of the waiting queue with as many tokens as fit; 0 if it has to wait."""
        hit = self.manager.find_prefix_hit(seq.token_ids)
        cached = hit.num_pages * self.page_size
        owed = seq.num_tokens - cached
        n = owed if whole else self._cap(owed, budget)
        if n > budget or n < 1:
            return 0
        if not self.manager.allocate(seq.seq_id, 0, n, hit):
            return 0
        seq.num_computed_tokens = cached
        seq.num_cached_tokens = cached
        return n

    def _start(self, seq: Sequence, n: int, scheduled: list, ids: set) -> None:
        self.waiting.popleft()
        seq.status = SequenceStatus.RUNNING
        seq.num_scheduled_tokens = n
        self.running.append(seq)
        scheduled.append(seq)
        ids.add(seq.seq_id)

    # -- one step's batch --------------------------------------------------------------------
    def schedule(self) -> list:
        scheduled = self._schedule_chunked() if self.enable_chunked_prefill else self._schedule_prefill_first()
        if not scheduled:
            raise RuntimeError("nothing schedulable: the cache pool or the token budget is too small "
                               "for the request at the head of the queue")
        return scheduled

    def _schedule_chunked(self) -> list:
        budget = self.max_num_batched_tokens
        scheduled, ids = [], set()
        preempted = False
        decodes, partials = [], []
        for s in self.running:
            (decodes if len(s.token_ids) - s.num_computed_tokens == 1 else partials).append(s)
        allocate = self.manager.allocate
        for seq in decodes + partials:
            if budget == 0:
                break
            if seq.status != SequenceStatus.RUNNING:     # preempted earlier in this loop
                continue
            owed = len(seq.token_ids) - seq.num_computed_tokens
            n = 1 if owed == 1 else self._cap(owed, budget)
            if not allocate(seq.seq_id, seq.num_computed_tokens, n):     # pages ran out: the slow way
                before = self.num_preemptions
                ok = self._allocate_or_preempt(seq, n, ids)
                preempted |= self.num_preemptions > before
                if not ok:
                    break
            seq.num_scheduled_tokens = n
            budget -= n
            scheduled.append(seq)
            ids.add(seq.seq_id)
        if preempted:
            return scheduled
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs:
            seq = self.waiting[0]
            n = self._try_start(seq, budget, whole=False)
            if n == 0:
                break
            self._start(seq, n, scheduled, ids)
            budget -= n
        return scheduled

    def _schedule_prefill_first(self) -> list:
        budget = self.max_num_batched_tokens
        scheduled, ids = [], set()
        while self.waiting and len(self.running) < self.max_num_seqs:
            seq = self.waiting[0]
            n = self._try_start(seq, budget, whole=True)
            if n == 0:
                break
            self._start(seq, n, scheduled, ids)
            budget -= n
        if scheduled:
            return scheduled
        for seq in list(self.running):
            if seq.status != SequenceStatus.RUNNING:
                continue
            if not self._allocate_or_preempt(seq, seq.num_uncomputed_tokens, ids):
                break
            seq.num_scheduled_tokens = seq.num_uncomputed_tokens
            scheduled.append(seq)
            ids.add(seq.seq_id)
        return scheduled

    # -- after the step ----------------------------------------------------------------------
    def postprocess(self, seqs: list, token_ids: list) -> list:
        """token_ids[i] is the token sampled for seqs[i], or None if it did not sample."""
        emitted = []
        publish = self.manager.publish_full_pages if self.manager.prefix_caching else None
        for seq, token_id in zip(seqs, token_ids):
            seq.num_computed_tokens += seq.num_scheduled_tokens
            seq.num_scheduled_tokens = 0
            sampled = seq.num_computed_tokens == len(seq.token_ids)      # the step reached the end of what is known
            if publish is not None:
                publish(seq.seq_id, seq.token_ids, seq.num_computed_tokens)
            if not sampled:
                continue
            seq.append_token(token_id)
            emitted.append(seq)
            sp = seq.sampling_params
            done = (token_id == self.eos and not sp.ignore_eos) or \
                len(seq.token_ids) - seq.num_prompt_tokens == sp.max_tokens
            if done:
                seq.status = SequenceStatus.FINISHED
                self._release(seq)
                self.running.remove(seq)
        return emitted
