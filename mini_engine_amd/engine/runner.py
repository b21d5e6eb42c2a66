"""The step function: one batch of (request, its next tokens) through the model, from the cache.

Reference counterpart: engine/model_runner.py:87-145 (`prepare` + `run`). Differences by
design: the step returns float32 logits at the places the caller names (sampling is a
separate call), the metadata of a step travels to the GPU as one packed int32 array, and
the runner owns the device side of the cache (`CachePool`) while the `CacheManager` it is
given owns the bookkeeping.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..cache.pool import CachePool, page_bytes
from ..kernels import ops
from .packing import context_of, exact_layout, pack_step, views_of


@dataclass
class StepEntry:
    """One request's share of a step: `tokens` are its tokens at positions start..start+n-1
    (start = how many of its tokens are already in the cache); `want` lists the places among
    these tokens whose logits are asked for."""

    req: object
    tokens: list
    start: int
    want: list = field(default_factory=list)


# A decode entry's token may be PENDING: the token that the request sampled in the runner's last
# sample_async() call, which is still on its way to the host. The step takes it from the device,
# so that it can be launched before the host has seen the token (decode steps that run one ahead).
PENDING = -1


class SampledTokens:
    """The token ids of one sampling call, on the device until tokens() fetches them."""

    def __init__(self, out: torch.Tensor, reqs: list | None, host: torch.Tensor | None = None, arrived=None):
        self.out = out
        self.reqs = reqs
        self.row_of = None if reqs is None else {r: i for i, r in enumerate(reqs)}
        self.host = host            # pinned copy, queued right behind the sampling kernel
        self.arrived = arrived      # event behind that copy

    def tokens(self) -> list:
        """Waits for this call's tokens only, not for what was launched after it."""
        if self.host is None:
            return self.out.tolist()
        self.arrived.synchronize()
        return self.host.tolist()


def _pad4(n: int) -> int:
    return (n + 3) & ~3


class ModelRunner:
    def __init__(self, model, manager: CacheManager, dtype: torch.dtype, device, max_positions: int,
                 poison_cache: bool = False, use_graphs: bool = False, max_decode_rows: int = 256,
                 mixed_graphs_after: int | None = 4, mixed_graphs_max_tokens: int | None = None):
        """use_graphs: decode steps are replayed as HIP graphs, and so are small steps with prompt portions
        whose padded shape has come up more than `mixed_graphs_after` times (None: those always run eagerly);
        `mixed_graphs_max_tokens`: up to how many tokens a step counts as small (None: by the model's size)."""
        self.model = model
        self.manager = manager
        self.dtype = dtype
        self.device = torch.device(device)
        self.max_positions = max_positions
        self.plan = model.cache_plan()
        if len(self.plan.group_needs) != manager.num_groups and self.plan.group_needs:
            raise ValueError(f"the model needs {len(self.plan.group_needs)} page groups, "
                             f"the cache manager has {manager.num_groups}")
        self.pool = CachePool(self.plan, [manager.num_pages(g) for g in range(len(self.plan.group_needs))],
                              manager.page_size, manager.num_state_slots, dtype, self.device, poison=poison_cache)
        if self.pool.has_state and manager.num_state_slots < 1:
            raise ValueError("the model keeps per-request state but the cache manager has no state slots")
        self.vocab_size = model.embedding.vocab_size if hasattr(model.embedding, "vocab_size") else None
        self.max_decode_rows = max_decode_rows
        self._graph_pool = None
        self._graph_logits = None
        self.graphs = None              # plain decode steps
        self.mixed_graphs = None        # steps with prompt portions
        if use_graphs and all(part.capturable for part in model.parts()):
            from .graphs import DecodeGraphs, MixedGraphs
            on_gpu = self.device.type == "cuda"
            self.graphs = DecodeGraphs(self, max_bucket=max_decode_rows, capture=on_gpu)
            if mixed_graphs_after is not None:
                self.mixed_graphs = MixedGraphs(self, max_rows=max_decode_rows, capture=on_gpu, capture_after=mixed_graphs_after,
                                                max_tokens=mixed_graphs_max_tokens)
        self._host = [None, None]
        self._events = [None, None]
        self._dev = None
        self._flip = 0
        self.last_sampled: SampledTokens | None = None
        self._sample_host = [None, None]
        self._sample_events = [None, None]
        self._sample_flip = 0
        self._token_host = [None] * 4     # pinned landing places of sampled tokens; a handle is read before 3 more calls
        self._token_flip = 0

    # -- sizing ----------------------------------------------------------------------------
    @staticmethod
    def windows_of(model) -> list:
        return [need.window for need in model.cache_plan().group_needs]

    @staticmethod
    def pages_that_fit(model, page_size: int, dtype: torch.dtype, budget_bytes: int) -> int:
        """Pages per group such that all groups together fit `budget_bytes`."""
        per_page = sum(page_bytes(model.cache_plan(), page_size, dtype))
        return max(0, int(budget_bytes // max(1, per_page)))

    # -- staging ---------------------------------------------------------------------------
    def _staging(self, n: int):
        i = self._flip
        self._flip ^= 1
        on_gpu = self.device.type == "cuda"
        if self._host[i] is None or self._host[i].numel() < n:
            cap = max(n, 4096) * 2
            self._host[i] = torch.empty(cap, dtype=torch.int32, pin_memory=on_gpu)
            self._events[i] = None
        elif self._events[i] is not None:
            self._events[i].synchronize()      # the copy that last used this buffer has finished
        if self._dev is None or self._dev.numel() < n:
            self._dev = torch.empty(max(n, 4096) * 2, dtype=torch.int32, device=self.device)
        return i, self._host[i]

    # -- the step --------------------------------------------------------------------------
    @torch.no_grad()      # not inference_mode: tensors made there cannot be used by a graph capture outside it, ours or the caller's
    def step(self, entries: list) -> torch.Tensor | None:
        """Run the given tokens as one batch. Returns float32 logits [R, vocab] for the wanted
        places, in the order of `entries` and of each entry's `want`; None if nothing is wanted.

        The pages (and state slot) of every request must have been allocated by the caller
        through the cache manager for positions up to start + len(tokens)."""
        if not entries:
            return None
        if len({e.req for e in entries}) != len(entries):
            seen = set()
            for e in entries:
                if e.req in seen:
                    raise ValueError(f"request {e.req!r} appears twice in one step")
                seen.add(e.req)
        most = self.max_positions
        graphs = self.graphs is not None and self.graphs.eligible(entries)
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise ValueError(f"request {e.req!r} brings no tokens")
            if e.tokens[0] == PENDING and not (n == 1 and graphs and self.last_sampled is not None
                                               and self.last_sampled.row_of is not None
                                               and e.req in self.last_sampled.row_of):
                raise ValueError(f"request {e.req!r}: a pending token needs a decode step of single tokens and "
                                 f"the request among those of the last sample_async() call")
            if e.start < 0 or e.start + n > most:
                raise ValueError(f"request {e.req!r}: positions {e.start}..{e.start + n - 1} "
                                 f"exceed the engine's limit of {most} tokens")
            for w in e.want:
                if not 0 <= w < n:
                    raise ValueError(f"request {e.req!r}: wanted place {w} outside its {n} tokens")
        if graphs:
            logits = self.graphs.step(entries)
            wanted = [i for i, e in enumerate(entries) if e.want]
            if not wanted:
                return None
            if len(wanted) == len(entries):
                return logits
            return logits[torch.tensor(wanted, dtype=torch.long, device=self.device)]
        # decodes (one new token) first, the others after, each kept in the caller's order
        order = [i for i, e in enumerate(entries) if len(e.tokens) == 1] + \
                [i for i, e in enumerate(entries) if len(e.tokens) != 1]
        G = self.manager.num_groups if self.plan.group_needs else 0
        tables = [[self.manager.block_table(entries[i].req, g) for i in order] for g in range(G)]
        slots_of = [self.manager.state_slot(entries[i].req) for i in order]
        lens = [len(entries[i].tokens) for i in order]
        cu = np.concatenate(([0], np.cumsum(lens)))
        offset_of = {order[j]: int(cu[j]) for j in range(len(order))}
        rows = [offset_of[i] + w for i, e in enumerate(entries) for w in e.want]      # in the caller's order
        return self._run([entries[i].tokens for i in order], [entries[i].start for i in order], tables, slots_of, rows,
                         names=[entries[i].req for i in order])

    def _run(self, token_lists: list, starts: list, tables: list, slots_of: list, rows: list, names: list | None = None):
        """One pass. Requests in step order (single tokens first): their tokens, first positions, per group
        their block tables, their state slots; `rows`: token rows that want logits. Steps whose padded shape
        has come up before are replayed as graphs (`MixedGraphs`); the others run eagerly, exactly sized."""
        q_lens = [len(t) for t in token_lists]
        layout = exact_layout(q_lens, starts, tables, len(rows), ops.decode_contexts_even)
        if self.mixed_graphs is not None:
            captured = self.mixed_graphs.lookup(layout)
            if captured is not None:
                return self.mixed_graphs.run(captured, token_lists, starts, tables, slots_of, rows, names)
        n = layout.segments()[1]
        buf_i, host = self._staging(n)
        pack_step(layout, host.numpy()[:n], token_lists, starts, tables, slots_of, rows, self.manager.page_size,
                  [self.pool.spare_page(g) for g in range(len(tables))], self.pool.spare_state_slot, self.vocab_size, names)
        dev = self._dev[:n]
        dev.copy_(host[:n], non_blocking=True)
        if self.device.type == "cuda":
            ev = torch.cuda.Event()
            ev.record()
            self._events[buf_i] = ev
        self.zero_fresh_state(slots_of, starts)
        tokens, row_view = views_of(layout, dev)
        h, residual = self.model.forward(tokens, context_of(layout, dev, q_lens, starts), self.pool.views, self.pool.states)
        if not rows:
            return None
        return self.model.logits(h, residual, row_view[:len(rows)])

    def zero_fresh_state(self, slots_of: list, starts: list) -> None:
        """A request whose tokens start at position 0 starts from its mixers' initial state (zeros unless
        a `StateNeed` names another)."""
        if not self.pool.has_state:
            return
        fresh = [s for s, st in zip(slots_of, starts) if st == 0 and s >= 0]
        if fresh:
            self.pool.reset_state(torch.tensor(fresh, dtype=torch.long, device=self.device))

    # -- what the captured graphs share ----------------------------------------------------
    def graph_pool(self):
        """One memory pool for all captured graphs: they replay one after the other on one stream, so a graph
        may reuse what the others' activations occupy."""
        if self._graph_pool is None and self.device.type == "cuda":
            self._graph_pool = torch.cuda.graph_pool_handle()
        return self._graph_pool

    def graph_logits(self) -> torch.Tensor:
        """The one buffer every captured graph writes its logits to ([rows a step can want, vocabulary]); what a
        step returns is a view of it, valid until the next step."""
        if self._graph_logits is None:
            from .graphs import bucket_of
            self._graph_logits = torch.empty((bucket_of(self.max_decode_rows), self.vocab_size), dtype=torch.float32,
                                             device=self.device)
        return self._graph_logits

    # -- sizing by measurement -------------------------------------------------------------
    @torch.no_grad()
    def measure_working_set(self, max_step_tokens: int, max_seqs: int, max_len: int) -> tuple:
        """(bytes the largest step needs beyond what is allocated now, the same for the largest decode step).

        Runs the two largest steps the engine's limits allow, a step of `max_step_tokens` prompt tokens
        and a step in which `max_seqs` requests of `max_len` tokens decode, and reads the allocator's peak
        (reference engine/model_runner.py:59-80 sizes its pool the same way). Every table entry names
        page 0, so one page per group is all the cache this needs; what the steps write and read there
        means nothing."""
        if self.device.type != "cuda":
            return 0, 0
        ps = self.manager.page_size
        G = len(self.plan.group_needs)
        nslots = max(1, self.manager.num_state_slots)

        def run(q_lens, starts, want_last):
            cu = np.concatenate(([0], np.cumsum(q_lens)))
            tables = [[[0] * -(-(s + q) // ps) for s, q in zip(starts, q_lens)] for _ in range(G)]
            rows = [int(cu[j + 1]) - 1 for j in range(len(q_lens))] if want_last else []
            torch.cuda.synchronize(self.device)
            torch.cuda.reset_peak_memory_stats(self.device)
            before = torch.cuda.memory_allocated(self.device)
            out = self._run([[0] * q for q in q_lens], starts, tables, [j % nslots for j in range(len(q_lens))], rows)
            torch.cuda.synchronize(self.device)
            del out
            return torch.cuda.max_memory_allocated(self.device) - before

        m = max(1, min(max_len, max_step_tokens))
        n = max(1, min(max_step_tokens // m, max_seqs))
        prompt_peak = run([m] * n, [0] * n, True)
        decode_peak = run([1] * max_seqs, [max_len - 1] * max_seqs, True)
        torch.cuda.empty_cache()
        return max(prompt_peak, decode_peak), decode_peak

    # -- sampling --------------------------------------------------------------------------
    @torch.no_grad()
    def sample(self, logits: torch.Tensor, temperatures: list, keys: list) -> list:
        """Token ids for float32 logits [S, V]; keys: (k0, k1) 32-bit pairs per row."""
        return self.sample_async(logits, temperatures, keys).tokens()

    @torch.no_grad()
    def sample_async(self, logits: torch.Tensor, temperatures: list, keys: list, reqs: list | None = None) -> SampledTokens:
        """The same without waiting for the result. `reqs` names the request of every row: the next
        step may then give PENDING as the token of any of them."""
        S = logits.shape[0]
        if reqs is not None and len(reqs) != S:
            raise ValueError(f"{len(reqs)} requests named for {S} rows of logits")
        # temperatures and keys travel as one array through pinned memory: a copy from pageable memory
        # would hold the host until the stream has run everything launched before it
        i = self._sample_flip
        self._sample_flip ^= 1
        on_gpu = self.device.type == "cuda"
        if self._sample_host[i] is None or self._sample_host[i].numel() < 3 * S:
            self._sample_host[i] = torch.empty(max(3 * S, 768), dtype=torch.int32, pin_memory=on_gpu)
            self._sample_events[i] = None
        elif self._sample_events[i] is not None:
            self._sample_events[i].synchronize()
        a = self._sample_host[i].numpy()
        a[:S] = np.asarray(temperatures, dtype=np.float32).view(np.int32)
        a[S:3 * S] = np.asarray(keys, dtype=np.uint32).reshape(2 * S).view(np.int32)
        dev = self._sample_host[i][:3 * S].to(self.device, non_blocking=True)
        if on_gpu:
            ev = torch.cuda.Event()
            ev.record()
            self._sample_events[i] = ev
        t = dev[:S].view(torch.float32)
        k = dev[S:].view(S, 2)
        out = ops.sample(logits, t, k)
        host = arrived = None
        if on_gpu:
            # the copy to the host is queued now, before any later step: it arrives when this call's
            # kernels are done, whatever has been launched behind them by then
            j = self._token_flip
            self._token_flip = (j + 1) % len(self._token_host)
            if self._token_host[j] is None or self._token_host[j].numel() < S:
                self._token_host[j] = torch.empty(max(S, 256), dtype=torch.int32, pin_memory=True)
            host = self._token_host[j][:S]
            host.copy_(out, non_blocking=True)
            arrived = torch.cuda.Event()
            arrived.record()
        self.last_sampled = SampledTokens(out, list(reqs) if reqs is not None else None, host, arrived)
        return self.last_sampled
