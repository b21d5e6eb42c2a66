"""Grouped-query attention over the paged cache (reference models/qwen3.py:12-38,
layers/attention.py:43-76)."""
from __future__ import annotations

from ..kernels import ops
from .base import CacheNeed, Mixer, ParamSpec, PositionEncoding, register_part
from .linear import Linear


@register_part("mixer", "attention")
class Attention(Mixer):
    """q, k, v from one packed product; optional per-head RMSNorm of q and k over the head
    size (applied before the position encoding, not to v); position encoding; causal
    attention of the new tokens over all cached keys of the request (or the last `window`);
    output product.

    Consecutive query heads share a key/value head: kv head = q head // (Hq/Hkv).
    `own_kv=False` builds a mixer with queries only, for a layer call that reads the cache
    another call has written.
    """

    takes_pending_norm = True      # x goes to the packed product and nowhere else

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 scale: float, qk_norm_eps: float | None = None, position: PositionEncoding | None = None,
                 window: int | None = None, own_kv: bool = True):
        super().__init__()
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} key/value heads")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.scale = float(scale)
        self.qk_norm_eps = qk_norm_eps
        self.window = window
        self.own_kv = own_kv
        self.q_size = num_heads * head_dim
        self.kv_size = num_kv_heads * head_dim
        if own_kv:
            self.add_child("qkv", Linear(hidden_size, self.q_size + 2 * self.kv_size,
                                         parts={"q": self.q_size, "k": self.kv_size, "v": self.kv_size}))
        else:
            self.add_child("qkv", Linear(hidden_size, self.q_size, parts={"q": self.q_size}))
        self.add_child("o", Linear(self.q_size, hidden_size))
        if qk_norm_eps is not None:
            self.add_param("q_norm_weight", ParamSpec((head_dim,), init="norm", dtype="float32"))
            if own_kv:
                self.add_param("k_norm_weight", ParamSpec((head_dim,), init="norm", dtype="float32"))
        if position is not None:
            self.add_child("position", position)
        else:
            self.position = None

    def cache_need(self):
        return CacheNeed.keys_and_values(self.num_kv_heads, self.head_dim, self.window)

    def forward(self, x, step, cache, state):
        Hq, Hkv, D = self.num_heads, self.num_kv_heads, self.head_dim
        grp = step.groups[cache.group]
        qkv = self.qkv.forward(x)
        store = self.own_kv and cache.write
        qw = self.q_norm_weight if self.qk_norm_eps is not None else None
        kw = self.k_norm_weight if (self.qk_norm_eps is not None and self.own_kv) else qw
        table = self.position.rotary_table() if self.position is not None else None
        eps = self.qk_norm_eps or 0.0
        if (store and step.num_decodes == step.num_tokens and (self.position is None or table is not None)
                and ops.decode_step_fuses(qkv.dtype, D, cache.page_size)):
            # only single tokens: norm, rotary, cache write and attention in one launch
            o = ops.decode_step_attention(qkv, qw, kw, eps, table, cache.k, cache.v, cache.page_size, grp.block_tables,
                                          step.context_lens, step.max_decode_context, self.scale, self.window,
                                          Hq, Hkv, D, even_contexts=step.decode_contexts_even)
            return self.o.forward(o, allow_partials=True)
        if self.position is None or table is not None:
            # norm + rotary + cache write in one pass
            bound = max(step.max_decode_context, step.max_prefill_context)
            if store:
                ops.qk_norm_rope_store(qkv, qw, kw, eps, table, step.positions, grp.slot_mapping,
                                       cache.k, cache.v, Hq, Hkv, D, cache.page_size, store=True, position_bound=bound)
            else:
                rows = qkv if not self.own_kv else qkv[:, : self.q_size]
                ops.qk_norm_rope_store(rows, qw, kw, eps, table, step.positions, None, None, None,
                                       Hq, 0, D, cache.page_size, store=False, position_bound=bound)
        else:
            # another position encoding: norm in place, the encoding's own apply, then the cache write
            nk = Hkv if self.own_kv else 0
            ops.qk_norm_rope_store(qkv[:, : self.q_size + nk * D], qw, kw, eps, None, step.positions, None, None,
                                   None, Hq, nk, D, cache.page_size, store=False)
            T = qkv.shape[0]
            q3 = qkv[:, : self.q_size].view(T, Hq, D)
            k3 = qkv[:, self.q_size: self.q_size + nk * D].view(T, nk, D)
            self.position.apply(q3, k3, step.positions)
            if store:
                v3 = qkv[:, self.q_size + self.kv_size:].view(T, Hkv, D)
                ops.store_kv(k3, v3, grp.slot_mapping, cache.k, cache.v, cache.page_size)
        q = qkv[:, : self.q_size]
        o = ops.paged_attention(q, cache.k, cache.v, cache.page_size, grp.block_tables, step.context_lens,
                                step.seq_of_token, step.positions, step.prefill_cu, step.num_decodes,
                                step.max_decode_context, self.scale, self.window, Hq, Hkv, D,
                                max_prefill_context=step.max_prefill_context,
                                even_contexts=step.decode_contexts_even)
        return self.o.forward(o, allow_partials=True)
