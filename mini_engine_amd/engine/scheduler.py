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

    def next_step_is_plain_decoding(self) -> bool:
        """Whether the next schedule() can only be: every running request decodes one token, nobody
        waits, and pages cannot run out (one new page per request at most). Such a step needs no
        token value and no request's pages back, so it may be launched before the step in flight
        has delivered its tokens."""
        if self.waiting or not self.running or len(self.running) > self.max_num_batched_tokens:
            return False
        need = len(self.running)
        if any(self.manager.num_free_pages(g) < need for g in range(self.manager.num_groups)):
            return False
        return all(len(s.token_ids) - s.num_computed_tokens == 1 for s in self.running)

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
    PLACEHOLDER = -1       # stands in a request's tokens for a sampled token that has not reached the host yet

    def advance(self, seqs: list) -> list:
        """Bookkeeping of a step that has been launched, before its tokens are known: the scheduled
        tokens count as computed; a request whose step reached the end of what is known gets a
        placeholder for the token being sampled, and leaves `running` if that token is its last by
        max_tokens. Returns the requests that sample, in order."""
        samplers = []
        publish = self.manager.publish_full_pages if self.manager.prefix_caching else None
        for seq in seqs:
            seq.num_computed_tokens += seq.num_scheduled_tokens
            seq.num_scheduled_tokens = 0
            if publish is not None:                      # pages whose tokens are all computed and all known
                known = len(seq.token_ids) - (seq.token_ids[-1] == self.PLACEHOLDER)
                publish(seq.seq_id, seq.token_ids, min(seq.num_computed_tokens, known))
            if seq.num_computed_tokens != len(seq.token_ids):
                continue
            seq.token_ids.append(self.PLACEHOLDER)
            samplers.append(seq)
            if len(seq.token_ids) - seq.num_prompt_tokens == seq.sampling_params.max_tokens:
                seq.status = SequenceStatus.FINISHED
                self.running.remove(seq)            # its pages are given back when its token is settled
        return samplers

    def settle(self, samplers: list, token_ids: list, index_of: list) -> list:
        """The sampled tokens have arrived: index_of[i] is where samplers[i]'s placeholder stands.
        Puts them in, publishes full pages, finishes on the end token and frees what finished
        requests hold. A request that an earlier token already finished (it ran one step ahead of
        its end token) is skipped. Returns the requests that got a token."""
        emitted = []
        publish = self.manager.publish_full_pages if self.manager.prefix_caching else None
        for seq, token_id, at in zip(samplers, token_ids, index_of):
            if at >= len(seq.token_ids):                 # cut off behind its end token: this token is not wanted
                continue
            seq.token_ids[at] = int(token_id)
            emitted.append(seq)
            if publish is not None and self.manager.holds(seq.seq_id):
                publish(seq.seq_id, seq.token_ids, min(seq.num_computed_tokens, at + 1))
            if token_id == self.eos and not seq.sampling_params.ignore_eos:
                del seq.token_ids[at + 1:]               # a placeholder of a step that ran ahead
                if seq.status != SequenceStatus.FINISHED:
                    seq.status = SequenceStatus.FINISHED
                    self.running.remove(seq)
        return emitted

    def release_finished(self, seqs: list) -> None:
        """Give back what finished requests among `seqs` hold (once no step that writes to their pages is in flight)."""
        for seq in seqs:
            if seq.status == SequenceStatus.FINISHED and self.manager.holds(seq.seq_id):
                self._release(seq)

    def postprocess(self, seqs: list, token_ids: list) -> list:
        """token_ids[i] is the token sampled for seqs[i], or None if it did not sample."""
        at = {id(s): len(s.token_ids) for s in seqs}
        samplers = self.advance(seqs)
        wanted = {id(s) for s in samplers}
        tokens = [t for s, t in zip(seqs, token_ids) if id(s) in wanted]
        emitted = self.settle(samplers, tokens, [at[id(s)] for s in samplers])
        self.release_finished(samplers)
        return emitted
