"""Which requests run how many tokens in the next step, and what becomes of them afterwards.

The policy is the reference's (engine/scheduler.py:97-155): under chunked prefill a step is filled
from three sources in turn, while the token budget lasts: live requests that owe one token (they
decode), live requests that owe more (their prompt is partly done), and the head of the queue;
without chunked prefill whole prompts are admitted first and only a step that admits nothing
decodes. Under FCFS the queue is served in order of arrival, under "priority" by (priority, arrival).

When pages run out (reference engine/scheduler.py:57-78): a live request that cannot get pages for
its next tokens makes another live request, one not yet in the step, give back everything it holds;
that one returns to the queue (FCFS: to its head) and is later fed again from its first token, its
generated tokens included, possibly finding its own pages still cached. FCFS evicts whoever was
admitted last, "priority" the least urgent. A requester that is the last candidate evicts itself and
the step goes on without it. A step in which anyone was evicted admits nobody. A queued request that
does not fit waits, and nobody overtakes it. A step that could take nobody raises.

After a step is launched its requests are moved on (`advance`) before their sampled tokens are known,
so that the next step can be planned and launched meanwhile; `settle` puts the tokens in when they
arrive, and `release_finished` gives back what ended requests hold once no launched step writes there.
"""
from __future__ import annotations

from collections import deque

from ..cache.manager import CacheManager
from .request import Phase, Request

UNKNOWN = -1       # stands in a request's tokens for a sampled token that has not reached the host yet


class ArrivalOrder:
    """First come, first served; an evicted request goes back to the head of the queue."""

    def enqueue(self, queue: deque, req: Request, returning: bool) -> None:
        if returning:
            queue.appendleft(req)
        else:
            queue.append(req)

    def evict_from(self, candidates: list) -> Request:
        return candidates[-1]                  # live requests are kept in order of admission: the newest


class UrgencyOrder:
    """Lower priority value first, earlier arrival first among equals; the least urgent is evicted."""

    @staticmethod
    def rank(req: Request) -> tuple:
        return req.priority, req.arrived

    def enqueue(self, queue: deque, req: Request, returning: bool) -> None:
        at = sum(1 for other in queue if self.rank(other) <= self.rank(req))     # the queue is kept sorted
        queue.insert(at, req)

    def evict_from(self, candidates: list) -> Request:
        return max(candidates, key=self.rank)


ORDERS = {"fcfs": ArrivalOrder, "priority": UrgencyOrder}


class _Plan:
    """The step being put together."""

    def __init__(self, room: int):
        self.room = room                   # tokens the budget still allows
        self.taken: list = []              # requests, in the order they were taken
        self.members: set = set()          # their ids
        self.evictions = 0

    def take(self, req: Request, n: int) -> None:
        req.portion = n
        self.room -= n
        self.taken.append(req)
        self.members.add(req.id)


class Scheduler:
    def __init__(self, config, manager: CacheManager):
        self.max_live = config.max_num_seqs
        self.token_budget = config.max_num_batched_tokens
        self.portion_cap = config.long_prefill_token_threshold      # 0: prompts are cut by the budget only
        self.chunked = bool(config.enable_chunked_prefill)
        self.order = ORDERS[config.scheduling_policy]()
        self.eos = config.eos
        self.max_model_len = config.max_model_len
        self.manager = manager
        self.page_size = manager.page_size
        self.waiting: deque = deque()
        self.running: list = []
        self.num_preemptions = 0
        self.num_prefix_hits = 0               # admissions that found pages of their tokens already cached
        self.num_prefix_hits_after_eviction = 0    # of those, requests fed again after an eviction

    # -- requests in ---------------------------------------------------------------------------
    def add(self, req: Request) -> None:
        """Queue a request, or refuse one that could never finish (reference engine/scheduler.py:26-33)."""
        most = req.prompt_len + req.params.max_tokens
        if most > self.max_model_len:
            raise ValueError(f"prompt+max_tokens={most} exceeds max_model_len={self.max_model_len}")
        for g in range(self.manager.num_groups):
            need, have = self.manager.pages_needed(most, g), self.manager.num_pages(g)
            if need > have:
                raise ValueError(f"needs {need} cache pages, the pool has {have}")
        self.order.enqueue(self.waiting, req, returning=False)

    def is_finished(self) -> bool:
        return not (self.waiting or self.running)

    # -- planning a step -----------------------------------------------------------------------
    def schedule(self) -> list:
        """The requests of the next step; each one's `portion` says how many of its tokens run."""
        plan = _Plan(self.token_budget)
        if self.chunked:
            self._continue_live(plan)
            if not plan.evictions:
                self._admit(plan, whole_prompts=False)
        else:
            self._admit(plan, whole_prompts=True)
            if not plan.taken:
                self._continue_live(plan)
        if not plan.taken:
            raise RuntimeError("nothing schedulable: the cache pool or the token budget is too small "
                               "for the request at the head of the queue")
        return plan.taken

    def _portion(self, owed: int, room: int) -> int:
        """How much of `owed` tokens runs now (reference engine/scheduler.py:51-55)."""
        if self.portion_cap and owed > self.portion_cap:
            owed = self.portion_cap
        return owed if owed < room else room

    def _continue_live(self, plan: _Plan) -> None:
        """Live requests, those that decode before those whose prompt is under way."""
        turn = sorted(self.running, key=lambda r: r.owed != 1)            # stable: admission order within each kind
        for req in turn:
            if plan.room <= 0:
                return
            if req.phase is not Phase.LIVE:                               # evicted a moment ago by one before it
                continue
            n = self._portion(req.owed, plan.room)
            if not self._pages_for(req, n, plan):
                return
            plan.take(req, n)

    def _pages_for(self, req: Request, n: int, plan: _Plan) -> bool:
        """Pages for the next n tokens of a live request, evicting others if that is what it takes.
        False: it had to evict itself."""
        while not self.manager.allocate(req.id, req.in_cache, n):
            loser = self.order.evict_from([r for r in self.running if r.id not in plan.members])
            self._evict(loser)
            plan.evictions += 1
            if loser is req:
                return False
        return True

    def _evict(self, req: Request) -> None:
        self.running.remove(req)
        self._give_back(req)
        req.phase = Phase.QUEUED
        req.portion = 0
        req.times_evicted += 1
        self.order.enqueue(self.waiting, req, returning=True)
        self.num_preemptions += 1

    def _give_back(self, req: Request) -> None:
        if self.manager.holds(req.id):
            self.manager.free(req.id)
        req.in_cache = req.from_prefix = 0

    def _admit(self, plan: _Plan, whole_prompts: bool) -> None:
        """The head of the queue, again and again, until one does not fit (nobody overtakes it)."""
        while self.waiting and plan.room > 0 and len(self.running) < self.max_live:
            req = self.waiting[0]
            hit = self.manager.find_prefix_hit(req.tokens)
            reused = hit.num_pages * self.page_size
            owed = len(req.tokens) - reused
            n = owed if whole_prompts else self._portion(owed, plan.room)
            if n < 1 or n > plan.room or not self.manager.allocate(req.id, 0, n, hit):
                return
            self.waiting.popleft()
            req.in_cache = req.from_prefix = reused
            if reused:
                self.num_prefix_hits += 1
                self.num_prefix_hits_after_eviction += bool(req.times_evicted)
            req.phase = Phase.LIVE
            self.running.append(req)
            plan.take(req, n)

    def next_step_is_plain_decoding(self) -> bool:
        """Whether the next schedule() can only be: every live request decodes one token, nobody is
        queued, and pages cannot run out (one new page per request at most). Such a step needs no
        token value and no request's pages back, so it may be launched before the step in flight
        has delivered its tokens."""
        live = len(self.running)
        if self.waiting or not live or live > self.token_budget:
            return False
        if any(self.manager.num_free_pages(g) < live for g in range(self.manager.num_groups)):
            return False
        return all(r.owed == 1 for r in self.running)

    # -- after a step --------------------------------------------------------------------------
    def advance(self, reqs: list) -> list:
        """Bookkeeping of a step that has been launched, before its tokens are known: the portions
        count as cached; a request whose portion reached the end of what is known gets a placeholder
        for the token being sampled, and leaves `running` if that token is its last by max_tokens.
        Returns the requests that sample, in order."""
        sampling = []
        publish = self.manager.publish_full_pages if self.manager.prefix_caching else None
        for req in reqs:
            req.in_cache += req.portion
            req.portion = 0
            if publish is not None:                      # pages whose tokens are all cached and all known
                known = len(req.tokens) - (req.tokens[-1] == UNKNOWN)
                publish(req.id, req.tokens, min(req.in_cache, known))
            if req.owed:
                continue
            req.tokens.append(UNKNOWN)
            sampling.append(req)
            if req.num_generated == req.params.max_tokens:
                req.phase = Phase.DONE
                self.running.remove(req)                 # its pages are given back when its token is settled
        return sampling

    def settle(self, sampling: list, token_ids: list, places: list) -> list:
        """The sampled tokens have arrived: places[i] is where sampling[i]'s placeholder stands.
        Puts them in, publishes pages that are now full, ends requests on the end token. A request
        that an earlier token already ended (it ran one step ahead of its end token) is skipped.
        Returns the requests that got a token."""
        got = []
        publish = self.manager.publish_full_pages if self.manager.prefix_caching else None
        for req, token, at in zip(sampling, token_ids, places):
            if at >= len(req.tokens):                    # cut off behind its end token: this token is not wanted
                continue
            req.tokens[at] = int(token)
            got.append(req)
            if publish is not None and self.manager.holds(req.id):
                publish(req.id, req.tokens, min(req.in_cache, at + 1))
            if token == self.eos and not req.params.ignore_eos:
                del req.tokens[at + 1:]                  # a placeholder of a step that ran ahead
                if req.phase is not Phase.DONE:
                    req.phase = Phase.DONE
                    self.running.remove(req)
        return got

    def release_finished(self, reqs: list) -> None:
        """Give back what ended requests among `reqs` hold (once no step that writes to their pages is in flight)."""
        for req in reqs:
            if req.phase is Phase.DONE and self.manager.holds(req.id):
                self._give_back(req)
