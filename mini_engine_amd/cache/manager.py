"""Bookkeeping of the paged key/value cache and of per-request state slots. Pure Python, no torch.

What the reference's BlockManager does (engine/block_manager.py:24-123): a pool of pages,
a block table per request, reference counts, chained xxh64 hashes of full pages for
prefix reuse, oldest-freed-first recycling that evicts a page's hash when it is reused.
Beyond it:

* several **page groups**. Layers with different needs (all keys, or only a trailing
  window of them) have pools and block tables of their own. In a window group the pages
  that the window has passed are given back before new ones are taken; their table
  entries become -1.
* **state slots**: one slot per live request out of a fixed number, for mixers that
  keep state of fixed size. A request holds its slot from its first allocation to `free`.

Prefix reuse is active only when no group has a window and no state slots exist: only
then are a request's pages a pure function of its token prefix.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

import numpy as np
import xxhash


def page_hash(token_ids, prefix: int = -1) -> int:
    """xxh64 of (previous page's hash as 8 little-endian bytes, if any) + int64 token bytes
    (reference engine/block_manager.py:33-39)."""
    h = xxhash.xxh64()
    if prefix != -1:
        h.update(prefix.to_bytes(8, "little"))
    h.update(np.asarray(token_ids, dtype=np.int64).tobytes())
    return h.intdigest()


@dataclass
class PrefixHit:
    num_pages: int = 0
    pages: list = field(default_factory=list)      # per group: page ids of the hit chain


class _Group:
    def __init__(self, num_pages: int, window: int | None):
        self.num_pages = num_pages
        self.window = window
        self.ref = [0] * num_pages
        self.hash = [-1] * num_pages
        self.tokens: list = [None] * num_pages
        self.free: deque = deque(range(num_pages))   # taken from the left, returned to the right
        self.used: set = set()
        self.by_hash: dict = {}

    def take_fresh(self) -> int:
        page = self.free.popleft()
        assert self.ref[page] == 0
        if self.hash[page] != -1 and self.by_hash.get(self.hash[page]) == page:
            del self.by_hash[self.hash[page]]        # its old content can no longer be hit
        self.hash[page] = -1
        self.tokens[page] = None
        self.ref[page] = 1
        self.used.add(page)
        return page

    def touch(self, page: int) -> None:
        if self.ref[page] == 0:
            self.free.remove(page)
            self.used.add(page)
        self.ref[page] += 1

    def release(self, page: int) -> None:
        assert self.ref[page] > 0, f"page {page} released twice"
        self.ref[page] -= 1
        if self.ref[page] == 0:
            self.used.remove(page)
            self.free.append(page)                   # keeps its hash: still hittable until reused


@dataclass
class _Held:
    tables: list                                     # per group: page ids, -1 where given back
    first_live: list                                 # per group: index of the first page still held
    state_slot: int = -1
    num_hashed: int = 0


class CacheManager:
    def __init__(self, num_pages, page_size: int, windows: list | None = None, num_state_slots: int = 0,
                 enable_prefix_caching: bool = True):
        windows = list(windows) if windows is not None else [None]
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(windows)
        if len(num_pages) != len(windows):
            raise ValueError("one page count per group")
        if page_size < 1 or any(n < 0 for n in num_pages):
            raise ValueError("page size must be positive and page counts non-negative")
        self.page_size = page_size
        self.groups = [_Group(n, w) for n, w in zip(num_pages, windows)]
        self.num_state_slots = num_state_slots
        self.free_slots: deque = deque(range(num_state_slots))
        self.held: dict = {}
        self.prefix_caching = bool(enable_prefix_caching and num_state_slots == 0
                                   and all(w is None for w in windows) and len(windows) >= 1)
        self._any_window = any(w is not None for w in windows)
        self.epoch = 0          # counts free() calls: while it stands still no request's pages have changed hands

    # -- queries ---------------------------------------------------------------------------
    @property
    def num_groups(self) -> int:
        return len(self.groups)

    def num_free_pages(self, group: int = 0) -> int:
        return len(self.groups[group].free)

    def num_pages(self, group: int = 0) -> int:
        return self.groups[group].num_pages

    def block_table(self, req, group: int = 0) -> list:
        return self.held[req].tables[group]

    def state_slot(self, req) -> int:
        return self.held[req].state_slot

    def holds(self, req) -> bool:
        return req in self.held

    def pages_needed(self, num_tokens: int, group: int = 0) -> int:
        """Most pages of `group` one request of `num_tokens` tokens can hold at a time when it is
        fed whole in one step (a window bounds it only for requests fed in smaller steps)."""
        return -(-num_tokens // self.page_size)

    # -- prefix reuse ----------------------------------------------------------------------
    def find_prefix_hit(self, token_ids) -> PrefixHit:
        """Longest chain of full pages, from the request's start, whose content is cached in
        every group; never the page that holds the last token, so at least one token is always
        computed (reference engine/block_manager.py:68-78)."""
        if not self.prefix_caching:
            return PrefixHit(0, [[] for _ in self.groups])
        ps = self.page_size
        pages = [[] for _ in self.groups]
        h = -1
        n = 0
        for i in range((len(token_ids) - 1) // ps):
            chunk = list(token_ids[i * ps:(i + 1) * ps])
            h = page_hash(chunk, h)
            found = []
            for g in self.groups:
                page = g.by_hash.get(h, -1)
                if page == -1 or g.tokens[page] != chunk:
                    found = None
                    break
                found.append(page)
            if found is None:
                break
            for gi, page in enumerate(found):
                pages[gi].append(page)
            n += 1
        return PrefixHit(n, pages)

    def publish_full_pages(self, req, token_ids, num_computed: int) -> None:
        """Hash the request's pages that are now completely computed so that others (and the
        request itself after a preemption) can reuse them, also while its prompt is only partly
        done (reference engine/block_manager.py:102-113)."""
        if not self.prefix_caching:
            return
        held = self.held[req]
        ps = self.page_size
        end = num_computed // ps
        for i in range(held.num_hashed, end):
            chunk = list(token_ids[i * ps:(i + 1) * ps])
            prefix = -1
            if i > 0:
                prefix = self.groups[0].hash[held.tables[0][i - 1]]
                assert prefix != -1
            h = page_hash(chunk, prefix)
            for gi, g in enumerate(self.groups):
                page = held.tables[gi][i]
                g.hash[page] = h
                g.tokens[page] = chunk
                g.by_hash[h] = page                  # the newest duplicate wins
        held.num_hashed = max(held.num_hashed, end)

    # -- allocation ------------------------------------------------------------------------
    def _release_behind_window(self, held: _Held, num_computed: int) -> None:
        ps = self.page_size
        for gi, g in enumerate(self.groups):
            if g.window is None:
                continue
            # the next tokens start at position num_computed and see keys >= num_computed - window + 1
            first_needed = max(0, num_computed - g.window + 1)
            table = held.tables[gi]
            i = held.first_live[gi]
            while i < len(table) and (i + 1) * ps <= first_needed:
                g.release(table[i])
                table[i] = -1
                i += 1
            held.first_live[gi] = i

    def allocate(self, req, num_computed: int, num_new: int, hit: PrefixHit | None = None) -> bool:
        """Make room for tokens [num_computed, num_computed + num_new) of `req`; all or nothing.

        A request unknown so far is registered (and gets a state slot if there are any). `hit`
        (only for a request that holds nothing yet) prepends cached pages; the caller then treats
        hit.num_pages * page_size tokens as computed. Pages behind a window are given back first.
        Returns False, changing nothing but that, when pages or slots do not suffice
        (reference engine/block_manager.py:80-100)."""
        ps = self.page_size
        held = self.held.get(req)
        if held is not None and hit is None and not self._any_window:
            # the common call of a decode step: the new token's page is held already
            total = -(-(num_computed + num_new) // ps)
            for table in held.tables:
                if len(table) < total:
                    break
            else:
                return True
        new_req = held is None
        nhit = hit.num_pages if hit else 0
        if nhit:
            assert new_req or all(not t for t in held.tables), "prefix hit for a request that already holds pages"
        if new_req and self.num_state_slots and not self.free_slots:
            return False
        if not new_req:
            self._release_behind_window(held, num_computed)
        computed = num_computed + nhit * ps
        total = -(-(computed + num_new) // ps)
        fresh, free_hits = [], []
        for gi, g in enumerate(self.groups):
            have = 0 if new_req else len(held.tables[gi])
            need = max(0, total - have - nhit)
            # a new request fed far beyond a window would not need its first pages, but it writes
            # all its tokens' keys in this step, so they all need a place
            fh = sum(1 for p in (hit.pages[gi] if nhit else []) if g.ref[p] == 0)
            if need + fh > len(g.free):
                return False
            fresh.append(need)
            free_hits.append(fh)
        if new_req:
            held = _Held([[] for _ in self.groups], [0] * len(self.groups))
            if self.num_state_slots:
                held.state_slot = self.free_slots.popleft()
            self.held[req] = held
        for gi, g in enumerate(self.groups):
            if nhit:
                for page in hit.pages[gi]:
                    g.touch(page)
                    held.tables[gi].append(page)
            for _ in range(fresh[gi]):
                held.tables[gi].append(g.take_fresh())
        if nhit:
            held.num_hashed += nhit
        return True

    def free(self, req) -> None:
        """Give back everything `req` holds: pages in reverse order, so that a request's last
        pages are recycled before its first (which are the likeliest prefix hits), and its
        state slot (reference engine/block_manager.py:115-123)."""
        held = self.held.pop(req)
        self.epoch += 1
        for gi, g in enumerate(self.groups):
            for page in reversed(held.tables[gi]):
                if page != -1:
                    g.release(page)
        if held.state_slot != -1:
            self.free_slots.append(held.state_slot)

    # -- checks (used by tests) ------------------------------------------------------------
    def forget_prefixes(self) -> None:
        """Drops every published prefix: pages keep their owners, but no later request can hit what
        is cached now (a benchmark that replays the same prompts under another setting starts cold;
        the reference builds a new block manager for this, bench_latency.py:51)."""
        for grp in self.groups:
            grp.by_hash.clear()
            for page in range(grp.num_pages):
                grp.hash[page] = -1
                grp.tokens[page] = None
        for held in self.held.values():
            held.num_hashed = 0

    def check_invariants(self) -> None:
        for gi, g in enumerate(self.groups):
            free = list(g.free)
            assert len(set(free)) == len(free), f"group {gi}: a page is in the free list twice"
            assert set(free).isdisjoint(g.used), f"group {gi}: a page is both free and used"
            assert set(free) | g.used == set(range(g.num_pages)), f"group {gi}: a page is lost"
            counts = [0] * g.num_pages
            for held in self.held.values():
                for page in held.tables[gi]:
                    if page != -1:
                        counts[page] += 1
            assert counts == g.ref, f"group {gi}: reference counts {g.ref} != table entries {counts}"
            for page in free:
                assert g.ref[page] == 0
            for h, page in g.by_hash.items():
                assert g.hash[page] == h
        slots = [h.state_slot for h in self.held.values() if h.state_slot != -1]
        assert len(set(slots)) == len(slots), "a state slot is held twice"
        assert set(slots).isdisjoint(self.free_slots)
        assert len(slots) + len(self.free_slots) == self.num_state_slots
