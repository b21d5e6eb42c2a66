"""The device memory behind the cache manager: pages per group, state tensors per layer call.

Layout of one layer call's pages (differs from the reference's [blocks, block, Hkv, D],
engine/model_runner.py:9-17; chosen for the matrix-core attention kernels):
    K [num_pages, Hkv, page, D]   V [num_pages, Hkv, D, page]
A group's pool stacks the calls that own pages in it: [calls, num_pages, ...].
"""
from __future__ import annotations

import torch

from ..parts.base import CacheView

_STATE_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


def page_bytes(plan, page_size: int, dtype: torch.dtype) -> list:
    """Bytes one page costs in each group (all its layer calls, keys and values)."""
    item = torch.empty((), dtype=dtype).element_size()
    return [2 * len(calls) * need.num_kv_heads * need.head_dim * page_size * item
            for need, calls in zip(plan.group_needs, plan.group_calls)]


class CachePool:
    def __init__(self, plan, num_pages: list, page_size: int, num_state_slots: int, dtype: torch.dtype,
                 device, poison: bool = False):
        self.plan = plan
        self.page_size = page_size
        self.num_pages = list(num_pages)
        self.k, self.v = [], []
        for need, calls, n in zip(plan.group_needs, plan.group_calls, self.num_pages):
            shape_k = (len(calls), n, need.num_kv_heads, page_size, need.head_dim)
            shape_v = (len(calls), n, need.num_kv_heads, need.head_dim, page_size)
            if poison:      # tests: any read of a key nobody wrote shows up as NaN
                self.k.append(torch.full(shape_k, float("nan"), dtype=dtype, device=device))
                self.v.append(torch.full(shape_v, float("nan"), dtype=dtype, device=device))
            else:
                self.k.append(torch.zeros(shape_k, dtype=dtype, device=device))
                self.v.append(torch.zeros(shape_v, dtype=dtype, device=device))
        self.views = []
        for i, g in enumerate(plan.call_group):
            if g is None:
                self.views.append(None)
                continue
            j = plan.call_index_in_group[i]
            self.views.append(CacheView(g, self.k[g][j], self.v[g][j], page_size, write=plan.call_writes[i]))
        self.states = []
        for need in plan.state_needs:
            if need is None:
                self.states.append(None)
            else:
                self.states.append(torch.zeros((max(1, num_state_slots),) + tuple(need.shape),
                                               dtype=_STATE_DTYPES[need.dtype], device=device))

    @property
    def has_state(self) -> bool:
        return any(s is not None for s in self.states)
