"""A step's metadata as one int32 array of a fixed layout, and the `StepContext` made of views into it.

The step function packs everything the kernels need to know about a step (token ids, positions, which
request a token belongs to, context lengths, prefix sums, state slots, rows that want logits, and per page
group the cache slots and block tables) into one array that travels to the device in one copy
(reference engine/model_runner.py:87-126 builds a tensor per item). A `StepLayout` fixes the sizes, so the
array's segments lie at offsets that depend on the layout alone: a step may be laid out exactly (every size
is what the step has), or padded up to a layout shared with other steps, which is what lets a captured
graph be replayed for all of them. Padding is made of requests that belong to nobody: rows of one token
with context 0 among the single-token requests, and one request of `pad` tokens at positions 0..pad-1 behind
the others; they write to the pool's spare page and spare state row, and no row of theirs wants logits.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from .context import GroupStep, StepContext


def _pad4(n: int) -> int:
    return (n + 3) & ~3


@dataclass(frozen=True)
class StepLayout:
    decode_rows: int          # requests with one new token (they come first), padding rows included
    prefill_reqs: int         # the other requests, the padding request included
    prefill_tokens: int       # their tokens
    rows: int                 # rows that want logits (at least 1 place is kept)
    max_blocks: tuple         # per page group: columns of the block table
    decode_ctx: int           # no single-token request holds more keys than this
    prefill_ctx: int          # no other request holds more keys than this (0: none)
    even: bool                # the single-token requests' contexts are (nearly) equally long

    @property
    def num_tokens(self) -> int:
        return self.decode_rows + self.prefill_tokens

    @property
    def num_seqs(self) -> int:
        return self.decode_rows + self.prefill_reqs

    def segments(self) -> tuple:
        """({name: (offset, size)}, total size) of the packed array."""
        T, B = self.num_tokens, self.num_seqs
        seg, n = {}, 0
        for name, size in (("tokens", T), ("positions", T), ("seq_of_token", T), ("context_lens", B), ("cu", B + 1),
                           ("prefill_cu", self.prefill_reqs + 1), ("state_slots", B), ("first_chunk", B),
                           ("rows", max(self.rows, 1))):
            seg[name] = (n, size)
            n += _pad4(size)
        for g, mb in enumerate(self.max_blocks):
            seg[f"slots{g}"] = (n, T); n += _pad4(T)
            seg[f"bt{g}"] = (n, B * mb); n += _pad4(B * mb)
        return seg, n


def exact_layout(q_lens: list, starts: list, tables: list, num_rows: int, even) -> StepLayout:
    """The layout that holds this step and nothing more."""
    Dn = sum(1 for q in q_lens if q == 1)
    decode_ctx = max((s + 1 for s, q in zip(starts, q_lens) if q == 1), default=0)
    prefill_ctx = max((s + q for s, q in zip(starts, q_lens) if q != 1), default=0)
    mb = tuple(max(1, max(len(t) for t in group)) for group in tables)
    lo = min((s + 1 for s, q in zip(starts, q_lens) if q == 1), default=0)
    return StepLayout(Dn, len(q_lens) - Dn, sum(q_lens) - Dn, num_rows, mb, decode_ctx, prefill_ctx,
                      bool(Dn) and even(Dn, lo, decode_ctx))


def pack_step(layout: StepLayout, out: np.ndarray, token_lists: list, starts: list, tables: list, state_slots: list,
              rows: list, page_size: int, spare_pages: list, spare_state: int, vocab_size: int | None,
              names: list | None = None) -> tuple:
    """Fill `out` (int32, the layout's size) for the requests given in step order (single tokens first).
    What the layout has beyond them is padding. Returns (new tokens, first position) of every request of the
    padded step, for the host-side copies in `StepContext`."""
    seg, n = layout.segments()
    ps = page_size
    q_lens = [len(t) for t in token_lists]
    Dn = sum(1 for q in q_lens if q == 1)
    Bp = len(q_lens) - Dn
    Tp = sum(q_lens) - Dn
    pad_rows = layout.decode_rows - Dn
    pad_tokens = layout.prefill_tokens - Tp
    pad_req = layout.prefill_reqs - Bp                     # 0 or 1
    if pad_rows < 0 or pad_tokens < 0 or pad_req not in (0, 1) or (pad_tokens > 0) != (pad_req == 1) or len(rows) > max(layout.rows, 0):
        raise ValueError("the step does not fit the layout it is packed into")
    # the padded step, request by request: (tokens, first position, context after the step)
    all_q = [1] * layout.decode_rows + q_lens[Dn:] + [pad_tokens] * pad_req
    all_start = starts[:Dn] + [0] * pad_rows + starts[Dn:] + [0] * pad_req
    all_ctx = [s + 1 for s in starts[:Dn]] + [0] * pad_rows + [s + q for s, q in zip(starts[Dn:], q_lens[Dn:])] + [pad_tokens] * pad_req
    B, T = layout.num_seqs, layout.num_tokens
    cu = np.zeros(B + 1, dtype=np.int64)
    np.cumsum(all_q, out=cu[1:])

    def put(name, values):
        o, size = seg[name]
        out[o:o + size] = values

    tok = np.zeros(T, dtype=np.int64)
    if Dn:
        tok[:Dn] = [t[0] for t in token_lists[:Dn]]
    if Tp:
        tok[layout.decode_rows:layout.decode_rows + Tp] = np.concatenate([np.asarray(t, dtype=np.int64) for t in token_lists[Dn:]])
    if vocab_size is not None and T and (tok.min() < 0 or tok.max() >= vocab_size):
        raise ValueError(f"token id outside 0..{vocab_size - 1}")
    pos = np.concatenate([np.arange(s, s + q, dtype=np.int64) for s, q in zip(all_start, all_q)])
    # where a real request's row sits in the padded step
    place = list(range(Dn)) + list(range(layout.decode_rows, layout.decode_rows + Bp))
    put("tokens", tok)
    put("positions", pos)
    put("seq_of_token", np.repeat(np.arange(B), all_q))
    put("context_lens", all_ctx)
    put("cu", cu)
    put("prefill_cu", cu[layout.decode_rows:] - cu[layout.decode_rows])
    slots = np.full(B, spare_state, dtype=np.int64)
    slots[place] = state_slots
    put("state_slots", slots)
    first = np.zeros(B, dtype=np.int64)
    first[place] = [1 if s == 0 else 0 for s in starts]
    put("first_chunk", first)
    shift = layout.decode_rows - Dn                         # rows of the others lie this much further on
    if rows:
        o, _ = seg["rows"]
        out[o:o + max(layout.rows, 1)] = 0
        out[o:o + len(rows)] = [r if r < Dn else r + shift for r in rows]
    else:
        put("rows", 0)
    for g, mb in enumerate(layout.max_blocks):
        bt = np.full((B, mb), -1, dtype=np.int64)
        slot = np.empty(T, dtype=np.int64)
        spare = spare_pages[g]
        for j, b in enumerate(place):
            t = tables[g][j]
            if len(t) > mb:
                raise ValueError("a block table is longer than the layout allows")
            bt[b, :len(t)] = t
            p = pos[cu[b]:cu[b + 1]]
            pages = bt[b, p // ps] if p[-1] // ps < mb else np.array([-1])
            if (pages < 0).any():
                who = names[j] if names is not None else j
                raise RuntimeError(f"request {who!r} has no page for a position it is "
                                   f"about to write (group {g}); allocate before stepping")
            slot[cu[b]:cu[b + 1]] = pages * ps + p % ps
        if pad_rows:
            slot[Dn:layout.decode_rows] = spare * ps
        if pad_req:
            b = B - 1
            if -(-pad_tokens // ps) > mb:
                raise ValueError(f"the padding request's {pad_tokens} tokens need more than the layout's {mb} block-table columns")
            bt[b, :-(-pad_tokens // ps)] = spare             # every page of the padding request is the spare one
            slot[cu[b]:cu[b + 1]] = spare * ps + pos[cu[b]:cu[b + 1]] % ps
        put(f"slots{g}", slot)
        put(f"bt{g}", bt.reshape(-1))
    return all_q, all_start


def context_of(layout: StepLayout, dev, q_lens: list | None = None, starts: list | None = None) -> StepContext:
    """The `StepContext` whose tensors are views into the packed array `dev` (on the device)."""
    seg, _ = layout.segments()

    def view(name):
        o, size = seg[name]
        return dev[o:o + size]

    B = layout.num_seqs
    return StepContext(
        num_tokens=layout.num_tokens, num_seqs=B, num_decodes=layout.decode_rows, positions=view("positions"),
        seq_of_token=view("seq_of_token"), context_lens=view("context_lens"), cu_seqlens=view("cu"),
        prefill_cu=view("prefill_cu") if layout.prefill_reqs else None, max_decode_context=layout.decode_ctx,
        decode_contexts_even=layout.even, max_prefill_context=layout.prefill_ctx,
        groups=[GroupStep(view(f"bt{g}").view(B, mb), view(f"slots{g}")) for g, mb in enumerate(layout.max_blocks)],
        state_slots=view("state_slots"), first_chunk=view("first_chunk"),
        q_lens=list(q_lens) if q_lens is not None else [], starts=list(starts) if starts is not None else [])


def views_of(layout: StepLayout, dev) -> tuple:
    """(token ids, rows that want logits) as views into the packed array."""
    seg, _ = layout.segments()
    (ot, nt), (orr, nr) = seg["tokens"], seg["rows"]
    return dev[ot:ot + nt], dev[orr:orr + nr]
