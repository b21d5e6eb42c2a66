"""Decode steps as HIP graphs.

A decode step of a small model is a few hundred short kernels; launched one by one their
launch cost exceeds their run time. For steps in which every request brings exactly one
token, the whole forward pass is captured once per (batch bucket, context cap, contexts equally
long or not) and replayed:
the step's metadata lives in one device array of fixed layout that is rewritten before each
replay. Rows beyond the real batch are padding: context length 0, slot -1 (nothing is
written to any request's page: their slot lies in the pool's spare page, their state row is the spare one), token 0.

The captured work is the same model code and kernels as the eager step; only the launch
mechanism differs. Nothing is cleared with memset nodes inside the graph.
"""
from __future__ import annotations

import gc
import weakref

import numpy as np
import torch

from ..kernels import ops
from .context import GroupStep, StepContext
from .packing import StepLayout, context_of, pack_step, views_of

PENDING = -1      # the runner's marker for a token that is still on the device (runner.PENDING)

CONTEXT_STEP = 1024      # the context cap of a captured graph is a multiple of this


def bucket_of(rows: int) -> int:
    """Rows of the captured layout that holds a step of `rows` requests: powers of two up to 256,
    multiples of 128 beyond."""
    if rows <= 256:
        return 1 << max(0, rows - 1).bit_length()
    return -(-rows // 128) * 128


def _pad4(n: int) -> int:
    return (n + 3) & ~3


class _Captured:
    def __init__(self, runner, bucket: int, ctx_cap: int, even: bool = False):
        self.bucket, self.ctx_cap, self.even = bucket, ctx_cap, even
        # the cap is rounded for the block tables' width; what the kernels are told (and check against the
        # position encoding's table) is never more than the engine's longest context
        self.max_context = min(ctx_cap, runner.max_positions)
        ps = runner.manager.page_size
        self.G = len(runner.plan.group_needs)
        self.MB = -(-ctx_cap // ps)
        B = bucket
        self.seg, n = {}, 0
        for name, size in (("tokens", B), ("positions", B), ("seq_of_token", B), ("context_lens", B), ("cu", B + 1),
                           ("state_slots", B), ("first_chunk", B), ("rows", B), ("take", B)):
            self.seg[name] = (n, size)
            n += _pad4(size)
        for g in range(self.G):
            self.seg[f"slots{g}"] = (n, B); n += _pad4(B)
            self.seg[f"bt{g}"] = (n, B * self.MB); n += _pad4(B * self.MB)
        self.n = n
        self.master = np.zeros(n, dtype=np.int32)            # host copy kept between steps
        self.put("seq_of_token", np.arange(B))
        self.put("cu", np.arange(B + 1))
        self.put("rows", np.arange(B))
        self.spare_state = runner.pool.spare_state_slot
        self.spare_slot = [runner.pool.spare_page(g) * ps for g in range(self.G)]
        self.put("state_slots", self.spare_state)
        for g in range(self.G):
            self.put(f"bt{g}", -1)
            self.put(f"slots{g}", self.spare_slot[g])
        self.row_req = [None] * B                            # which request's table a row holds
        self.row_len = [[0] * B for _ in range(self.G)]      # how many of its entries are written
        self.row_tab = [[None] * B for _ in range(self.G)]   # the manager's table they were copied from
        self.last_starts = None                              # positions of the step before, or None
        self.last_epoch = -1                                 # the cache manager's epoch at that step
        self.on_gpu = runner.device.type == "cuda"
        self.pinned = [torch.empty(n, dtype=torch.int32, pin_memory=self.on_gpu) for _ in range(2)]
        self.events = [None, None]
        self.flip = 0
        self.dev = torch.zeros(n, dtype=torch.int32, device=runner.device)
        self.graph = None

    def put(self, name, values):
        o, size = self.seg[name]
        self.master[o:o + size] = values

    def view(self, name):
        o, size = self.seg[name]
        return self.dev[o:o + size]

    def context(self) -> StepContext:
        B = self.bucket
        return StepContext(
            num_tokens=B, num_seqs=B, num_decodes=B, positions=self.view("positions"),
            seq_of_token=self.view("seq_of_token"), context_lens=self.view("context_lens"),
            cu_seqlens=self.view("cu"), prefill_cu=None, max_decode_context=self.max_context,
            decode_contexts_even=self.even,
            groups=[GroupStep(self.view(f"bt{g}").view(B, self.MB), self.view(f"slots{g}")) for g in range(self.G)],
            state_slots=self.view("state_slots"), first_chunk=self.view("first_chunk"),
            q_lens=[1] * B, starts=[0] * B)

    def upload(self):
        i = self.flip
        self.flip ^= 1
        if self.events[i] is not None:
            self.events[i].synchronize()
        self.pinned[i].numpy()[:] = self.master
        self.dev.copy_(self.pinned[i], non_blocking=True)
        if self.on_gpu:
            ev = torch.cuda.Event()
            ev.record()
            self.events[i] = ev


class DecodeGraphs:
    def __init__(self, runner, max_bucket: int = 256, capture: bool = True, max_graphs: int = 64):
        """Steps of up to `max_bucket` requests go through here. capture=False runs the padded,
        fixed-layout step eagerly every time (no graph): the same metadata path without the capture,
        for machines without a GPU."""
        self.runner = weakref.proxy(runner)      # the runner owns this object: no cycle, so that an engine that
        self.max_bucket = max_bucket             # goes out of use is freed at once, not by a later collection
        self.max_graphs = max(4, max_graphs)     # (bucket, context cap) pairs kept; the one unused for longest goes first
        self.capture = capture
        self.captured: dict = {}
        # One memory pool for all captured graphs: they replay one after the other on one stream, so a
        # graph may reuse what the others' activations occupy. Nothing a graph allocates outlives its
        # capture: the logits, the one result that is read afterwards, go into `self.logits`, one buffer
        # for all layouts (a layout that kept its own would pin 150 MB of the pool at 256 rows).
        self.pool = runner.graph_pool() if capture else None
        self.logits = None
        self.replays = 0
        self.advances = 0        # of those, steps whose tables and slots were carried on from the step before

    def takes(self, num_entries: int) -> bool:
        """Whether a step of this many single-token entries goes through here."""
        r = self.runner
        return ((r.device.type == "cuda" or not self.capture) and num_entries <= self.max_bucket
                and r.vocab_size is not None)

    def eligible(self, entries) -> bool:
        return self.takes(len(entries)) and all(len(e.tokens) == 1 for e in entries)

    def step(self, entries: list):
        """Logits [len(entries), vocab] for a step in which every request brings one token."""
        r = self.runner
        B = len(entries)
        bucket = bucket_of(B)
        need_ctx = max(e.start for e in entries) + 1
        ctx_cap = min(-(-need_ctx // CONTEXT_STEP) * CONTEXT_STEP, -(-r.max_positions // 8) * 8)
        # whether the contexts are equally long is part of the layout: the decode kernel's grid depends on it
        even = ops.decode_contexts_even(B, min(e.start for e in entries) + 1, need_ctx)
        key = (bucket, ctx_cap, even)
        cap = self.captured.pop(key, None)
        if cap is None:
            cap = _Captured(r, bucket, ctx_cap, even)
            while len(self.captured) >= self.max_graphs:      # its last replay lies max_graphs - 1 steps or more back
                del self.captured[next(iter(self.captured))]
        self.captured[key] = cap                              # most recently used last
        ps = r.manager.page_size
        tok = np.zeros(bucket, dtype=np.int64)
        pos = np.zeros(bucket, dtype=np.int64)
        ctx = np.zeros(bucket, dtype=np.int64)
        tok[:B] = [e.tokens[0] for e in entries]
        pos[:B] = [e.start for e in entries]
        ctx[:B] = pos[:B] + 1
        pending = np.flatnonzero(tok[:B] == PENDING)          # tokens still on the device (checked by the runner)
        if pending.size:
            tok[pending] = 0
            row_of = r.last_sampled.row_of
            take = np.full(bucket, -1, dtype=np.int64)       # per row: the row of the last sampling call that holds its token
            take[pending] = [row_of[entries[j].req] for j in pending.tolist()]
            cap.put("take", take)
        if r.vocab_size is not None and (tok.min() < 0 or tok.max() >= r.vocab_size):
            raise ValueError(f"token id outside 0..{r.vocab_size - 1}")
        cap.put("tokens", tok); cap.put("positions", pos); cap.put("context_lens", ctx)
        cap.put("first_chunk", (pos == 0) & (ctx > 0))
        reqs = [e.req for e in entries]
        if r.pool.has_state:
            state = np.full(bucket, cap.spare_state, dtype=np.int64)
            state[:B] = [r.manager.state_slot(q) for q in reqs]
            cap.put("state_slots", state)
            fresh = state[:B][pos[:B] == 0]
            if fresh.size:              # a request whose first token this is starts from empty state (outside the graph)
                r.pool.reset_state(torch.tensor(fresh.tolist(), dtype=torch.long, device=r.device))
        continues = self._continues(cap, reqs, pos, B)
        cap.last_starts = None                       # stays so if what follows raises
        if continues:
            self._advance(cap, entries, pos, B)
            self.advances += 1
        else:
            self._rewrite(cap, entries, B)
            cap.row_req[:B] = reqs
            for j in range(B, bucket):
                cap.row_req[j] = None
        cap.last_starts = pos
        cap.last_epoch = r.manager.epoch
        cap.upload()
        if pending.size:
            self._take_pending(cap, take, B)
        self.replays += 1
        if not self.capture:
            return self._forward(cap)[:B]
        if cap.graph is None and self._capture(cap):
            return self.logits[:B]               # the eager run before the capture was this step
        cap.graph.replay()
        return self.logits[:B]

    def _take_pending(self, cap: _Captured, take, B: int) -> None:
        """Copy the tokens that the last sampling call left on the device into the step's token rows
        (after the upload, before the replay, on the same stream): one small kernel, rows whose `take` is
        negative keep the token that went up with the metadata. `take` went up with the metadata too."""
        ops.take_tokens(cap.view("tokens")[:B], self.runner.last_sampled.out, cap.view("take")[:B])

    def _continues(self, cap: _Captured, reqs: list, pos, B: int) -> bool:
        """Whether this step is the one before with every request one position on: the same
        requests in the same rows, no pages given back by anyone since (a request that was
        preempted and fed again holds other pages at the same positions), no windowed group
        (its tables lose entries as the window moves)."""
        m = self.runner.manager
        if cap.last_starts is None or cap.last_epoch != m.epoch or m._any_window:
            return False
        bucket = cap.bucket
        if cap.row_req[:B] != reqs or (B < bucket and cap.row_req[B] is not None):
            return False
        return bool(np.array_equal(pos[:B], cap.last_starts[:B] + 1))

    def _advance(self, cap: _Captured, entries: list, pos, B: int) -> None:
        """The tables and slots of a step that continues the one before: a row whose new position
        lies in the page of its last one takes the next slot; only rows that enter a page are looked up."""
        r = self.runner
        ps = r.manager.page_size
        entering = np.flatnonzero(pos[:B] % ps == 0)
        for g in range(cap.G):
            o, _ = cap.seg[f"slots{g}"]
            cap.master[o:o + B] += 1
            if entering.size:
                ob, _ = cap.seg[f"bt{g}"]
                bt = cap.master[ob:ob + cap.bucket * cap.MB].reshape(cap.bucket, cap.MB)
                for j in entering.tolist():
                    e = entries[j]
                    t = r.manager.block_table(e.req, g)
                    k = cap.row_len[g][j]
                    if len(t) > k:
                        bt[j, k:len(t)] = t[k:]
                        cap.row_len[g][j] = len(t)
                    page = t[e.start // ps] if e.start // ps < len(t) else -1
                    if page < 0:
                        raise RuntimeError(f"request {e.req!r} has no page for position {e.start} (group {g}); "
                                           f"allocate before stepping")
                    cap.master[o + j] = page * ps

    def _rewrite(self, cap: _Captured, entries: list, B: int) -> None:
        """The tables and slots of every row, from the cache manager's tables."""
        r = self.runner
        ps = r.manager.page_size
        bucket = cap.bucket
        for g in range(cap.G):
            o, _ = cap.seg[f"bt{g}"]
            bt = cap.master[o:o + bucket * cap.MB].reshape(bucket, cap.MB)
            slots = np.full(bucket, cap.spare_slot[g], dtype=np.int64)
            windowed = r.manager.groups[g].window is not None
            for j, e in enumerate(entries):
                t = r.manager.block_table(e.req, g)
                # another table than the row was copied from: another request, or the same one after it
                # gave its pages back and was fed again (same id, same length, other pages)
                if cap.row_tab[g][j] is not t or cap.row_len[g][j] > len(t) or windowed:
                    bt[j, :] = -1
                    cap.row_len[g][j] = 0
                    cap.row_tab[g][j] = t
                k = cap.row_len[g][j]
                if len(t) > k:
                    bt[j, k:len(t)] = t[k:]
                    cap.row_len[g][j] = len(t)
                page = t[e.start // ps] if e.start // ps < len(t) else -1
                if page < 0:
                    raise RuntimeError(f"request {e.req!r} has no page for position {e.start} (group {g}); "
                                       f"allocate before stepping")
                slots[j] = page * ps + e.start % ps
            for j in range(B, bucket):
                if cap.row_req[j] is not None:
                    bt[j, :] = -1
                    cap.row_len[g][j] = 0
                    cap.row_tab[g][j] = None
            cap.put(f"slots{g}", slots)

    def _forward(self, cap: _Captured, out=None):
        r = self.runner
        h, residual = r.model.forward(cap.view("tokens"), cap.context(), r.pool.views, r.pool.states)
        return r.model.logits(h, residual, cap.view("rows"), out=out)

    def _capture(self, cap: _Captured) -> bool:
        """Captures the step; True if the step has thereby run already (see `capture_graph`)."""
        # one eager run first: libraries load, scratch buffers get their size, the caching allocator warms up
        self.logits = self.runner.graph_logits()
        out = self.logits[:cap.bucket]
        cap.graph, ran = capture_graph(self.runner, self.pool, lambda: self._forward(cap, out))
        return ran


def capture_graph(runner, pool, forward):
    """Run `forward` once eagerly, then capture it: (graph, whether the eager run stands as the step's own). The
    eager run comes first so that libraries load, scratch buffers get their size and the caching allocator warms
    up outside the capture. A model without per-request state has then done the step (the same kernels on the same
    buffers as a replay: the logits are where a replay would put them, the cache holds what it would write), and
    the caller need not replay the new graph for it, which is a tenth to a quarter of what a capture costs (0.6B
    sizes, steps of 100-300 tokens: eager run 2.7-3.9 ms, capture 3.2-5.7, first replay 1.0-2.4)."""
    # Cache writes can be repeated, state updates cannot: what the eager run does to the requests'
    # state is taken back, the replay that follows does it for good.
    states = [st for st in runner.pool.states if st is not None]
    kept = [st.clone() for st in states]
    forward()
    for st, was in zip(states, kept):
        st.copy_(was)
    del kept
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    # No garbage collection while the stream is capturing: a collector run that finds an old
    # engine's graphs, events or pinned buffers frees them with calls that a capturing stream
    # refuses, and the process aborts inside a destructor. (torch collects once on entering.)
    collecting = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph, pool=pool):
            forward()
    finally:
        if collecting:
            gc.enable()
    return graph, not states


# ------------------------------------------------------------------------------------------------
# Steps that are not plain decoding: portions of prompts, alone or beside single tokens.

def _round_up(n: int, to: int) -> int:
    return -(-n // to) * to


def _pow2_at_least(n: int) -> int:
    return 1 << max(0, n - 1).bit_length()


# What launching a layer's kernels from Python costs the host, and the rate at which small steps run on the GPU:
# from them follows up to how many tokens a step is bound by the host rather than by the GPU. Measured at
# Qwen3-0.6B sizes (28 layers): an eager step costs the host 3.6-4.4 ms whatever its size; replayed, a prompt of
# 128 tokens takes 2.4 ms and one of 512 tokens 3.2 ms (the GPU's own time: products of so few rows run far below
# the rate of large ones), and a step of 504 prompt tokens beside 8 requests with long contexts 4.1 ms, which is
# what it takes eagerly. A capture costs 12-14 ms, so layouts that do not pay must not be captured at all.
HOST_US_PER_LAYER = 130.0
SMALL_STEP_FLOPS = 1.0e14
# Up to this many times the host-bound size a step is still worth replaying when its layout repeats exactly (the host's
# launches leave gaps between kernels of a few microseconds each): a 2,048-token prompt at the 0.6B sizes 5.40 -> 5.08 ms.
EXACT_LAYOUT_FACTOR = 6


def host_bound_tokens(model) -> int:
    """Up to how many tokens a step of this model is worth replaying from a graph: below, the host's launches
    take longer than the GPU's work; above, the eager step keeps the GPU busy anyway and padding only costs."""
    per_token = 0
    for name, _, _, spec in model.named_specs():
        if len(spec.shape) == 2 and not name.startswith(("embedding.", "head.")):
            per_token += 2 * spec.shape[0] * spec.shape[1]
    per_token *= max(1, len(model.order)) / max(1, len(model.layers))
    if per_token <= 0:
        return 2048
    tokens = HOST_US_PER_LAYER * 1e-6 * len(model.order) / (per_token / SMALL_STEP_FLOPS)
    return int(min(2048, max(64, tokens)))


class _CapturedStep:
    def __init__(self, runner, layout: StepLayout):
        self.layout = layout
        self.n = layout.segments()[1]
        on_gpu = runner.device.type == "cuda"
        self.pinned = [torch.empty(self.n, dtype=torch.int32, pin_memory=on_gpu) for _ in range(2)]
        self.events = [None, None]
        self.flip = 0
        self.dev = torch.zeros(self.n, dtype=torch.int32, device=runner.device)
        self.graph = None
        self.replays = 0

    def staging(self):
        i = self.flip
        self.flip ^= 1
        if self.events[i] is not None:
            self.events[i].synchronize()           # the copy that last used this buffer has finished
        return i, self.pinned[i]


class MixedGraphs:
    """Small steps with prompt portions, padded to a layout shared by many steps and replayed as a graph.

    Launched kernel by kernel from Python, a step costs the host a few milliseconds whatever its size, which
    for small models and short portions is more than the GPU needs. Such a step (up to `max_tokens` tokens: see
    host_bound_tokens) is rounded up to a layout: single-token rows to a bucket, all tokens to a power of two
    (beyond 256 to a multiple of 64, beyond 1,024 of 128: a step that fills a token budget must not grow by half)
    through one padding request, one power-of-two cap for every context and block table, rows that want logits
    to a bucket. The rounding is coarse on purpose: a capture costs about three eager steps, so layouts must be
    few, and a step that the host bounds loses nothing by the padding. A layout that has come up
    `capture_after` times is captured on its next appearance and replayed from then on; larger steps, and
    layouts that come up once, stay eager and exactly sized. The captured work is the model's own forward pass
    over the padded step.

    Steps beyond `max_tokens` and up to `max_exact_tokens` (six times as many: up to there the host's launches
    still leave gaps between the GPU's kernels) take a layout with the step's own token and request counts and
    only the context cap and the rows of logits rounded, if nobody decodes in them: prompts of one length alone, or
    a long prompt's portions under a fixed budget, come up again and again exactly so, and nothing is lost to
    padding when they do not."""

    def __init__(self, runner, max_rows: int, capture: bool = True, capture_after: int = 4, max_graphs: int = 48,
                 max_tokens: int | None = None):
        self.runner = weakref.proxy(runner)
        self.max_rows = max_rows
        self.capture = capture
        self.capture_after = capture_after
        self.max_graphs = max_graphs
        self.max_tokens = host_bound_tokens(runner.model) if max_tokens is None else max_tokens
        self.max_exact_tokens = EXACT_LAYOUT_FACTOR * self.max_tokens
        self.captured: dict = {}
        self.sightings: dict = {}
        self.pool = runner.graph_pool() if capture else None
        self.replays = 0

    def padded(self, exact: StepLayout) -> StepLayout | None:
        r = self.runner
        tokens = exact.decode_rows + exact.prefill_tokens
        if (exact.prefill_reqs == 0 or exact.rows > self.max_rows or tokens >= self.max_exact_tokens or r.vocab_size is None
                or not (r.device.type == "cuda" or not self.capture)):
            return None
        ps = r.manager.page_size
        if tokens >= self.max_tokens:
            # the step's own counts; only what differs from step to step of a repeating pattern is rounded. Only steps
            # in which nobody decodes: a capture holds the GPU for 12-14 ms, which requests that wait for their next
            # token would feel (latency workload, 2,048-token budget: time between tokens p99.9 11.9 -> 20.2 ms with
            # such steps captured too), and their layouts (so many decoding beside so many prompt tokens) seldom
            # come up often enough to earn it back
            if exact.decode_rows:
                return None
            cap = min(max(1024, _pow2_at_least(max(exact.decode_ctx, exact.prefill_ctx))), r.max_positions)
            return StepLayout(
                decode_rows=exact.decode_rows, prefill_reqs=exact.prefill_reqs, prefill_tokens=exact.prefill_tokens,
                rows=bucket_of(exact.rows) if exact.rows else 0,
                max_blocks=tuple(max(mb, -(-cap // ps)) for mb in exact.max_blocks),
                decode_ctx=cap if exact.decode_rows else 0, prefill_ctx=cap, even=exact.even)
        decode_rows = bucket_of(exact.decode_rows) if exact.decode_rows else 0
        need = decode_rows + exact.prefill_tokens + 1
        total = max(32, _pow2_at_least(need)) if need <= 256 else _round_up(need, 64 if need <= 1024 else 128)
        pad = total - decode_rows - exact.prefill_tokens
        if pad > r.max_positions:
            return None       # the padding request would stand at positions the engine does not have: run as it is
        cap = min(max(1024, _pow2_at_least(max(exact.decode_ctx, exact.prefill_ctx, pad))), r.max_positions)
        return StepLayout(
            decode_rows=decode_rows, prefill_reqs=exact.prefill_reqs + 1, prefill_tokens=total - decode_rows,
            rows=bucket_of(exact.rows) if exact.rows else 0,
            max_blocks=tuple(max(mb, -(-cap // ps)) for mb in exact.max_blocks),
            decode_ctx=cap if exact.decode_rows else 0, prefill_ctx=cap, even=exact.even)

    def lookup(self, exact: StepLayout):
        """The captured (or about to be captured) layout that takes this step, or None: run it eagerly."""
        layout = self.padded(exact)
        if layout is None:
            return None
        cap = self.captured.pop(layout, None)
        if cap is None:
            seen = self.sightings.get(layout, 0) + 1
            if seen <= self.capture_after:
                if len(self.sightings) > 4096:
                    self.sightings.clear()
                self.sightings[layout] = seen
                return None
            self.sightings.pop(layout, None)
            cap = _CapturedStep(self.runner, layout)
            while len(self.captured) >= self.max_graphs:        # the one unused for longest goes
                del self.captured[next(iter(self.captured))]
        self.captured[layout] = cap                               # most recently used last
        return cap

    def run(self, cap: _CapturedStep, token_lists, starts, tables, state_slots, rows, names):
        r = self.runner
        layout = cap.layout
        i, host = cap.staging()
        q_lens, first = pack_step(layout, host.numpy(), token_lists, starts, tables, state_slots, rows, r.manager.page_size,
                                  [r.pool.spare_page(g) for g in range(len(layout.max_blocks))], r.pool.spare_state_slot,
                                  r.vocab_size, names)
        cap.dev.copy_(host, non_blocking=True)
        if r.device.type == "cuda":
            ev = torch.cuda.Event()
            ev.record()
            cap.events[i] = ev
        r.zero_fresh_state(state_slots, starts)
        cap.replays += 1
        self.replays += 1
        R = len(rows)
        if not self.capture:
            out = self._forward(cap, None, q_lens, first)
            return out[:R] if R else None
        logits = r.graph_logits()
        ran = False
        if cap.graph is None:
            out = logits[:layout.rows] if layout.rows else None
            cap.graph, ran = capture_graph(r, self.pool, lambda: self._forward(cap, out, q_lens, first))
        if not ran:
            cap.graph.replay()
        return logits[:R] if R else None

    def _forward(self, cap: _CapturedStep, out, q_lens, first):
        r = self.runner
        layout = cap.layout
        tokens, rows = views_of(layout, cap.dev)
        h, residual = r.model.forward(tokens, context_of(layout, cap.dev, q_lens, first), r.pool.views, r.pool.states)
        if not layout.rows:
            return None
        return r.model.logits(h, residual, rows[:layout.rows], out=out)
