"""The device memory behind the cache manager: pages per group, state tensors per layer call.

What a page holds is the mixer's business (`CacheNeed.tensors`); attention's layout is
    K [num_pages, Hkv, page, D]   V [num_pages, Hkv, D, page]
(not the reference's [blocks, block, Hkv, D], engine/model_runner.py:9-17: chosen for the matrix-core
attention kernels). A group's pool stacks the calls that own pages in it: [calls, num_pages + 1, ...].
One page more than the manager hands out, and one state row more than it has slots: spares that belong
to no request, for the padding rows of steps with a fixed layout (they write there, nobody reads it).
"""
from __future__ import annotations

import math

import torch

from ..parts.base import CacheView

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


def _dtype_of(name: str, compute: torch.dtype) -> torch.dtype:
    return compute if name == "compute" else _DTYPES[name]


def page_bytes(plan, page_size: int, dtype: torch.dtype) -> list:
    """Bytes one page costs in each group (all its layer calls, all their tensors)."""
    out = []
    for need, calls in zip(plan.group_needs, plan.group_calls):
        per_call = sum(math.prod(t.sized(page_size)) * torch.empty((), dtype=_dtype_of(t.dtype, dtype)).element_size()
                       for t in need.tensors)
        out.append(len(calls) * per_call)
    return out


class CachePool:
    def __init__(self, plan, num_pages: list, page_size: int, num_state_slots: int, dtype: torch.dtype,
                 device, poison: bool = False):
        self.plan = plan
        self.page_size = page_size
        self.num_pages = list(num_pages)
        self.tensors = []              # per group: name -> [calls, pages + 1, *page shape]
        for need, calls, n in zip(plan.group_needs, plan.group_calls, self.num_pages):
            group = {}
            for t in need.tensors:
                shape = (len(calls), n + 1) + t.sized(page_size)
                dt = _dtype_of(t.dtype, dtype)
                if poison and dt.is_floating_point:      # tests: any read of a place nobody wrote shows up as NaN
                    group[t.name] = torch.full(shape, float("nan"), dtype=dt, device=device)
                else:
                    group[t.name] = torch.zeros(shape, dtype=dt, device=device)
            self.tensors.append(group)
        self.views = []
        for i, g in enumerate(plan.call_group):
            if g is None:
                self.views.append(None)
                continue
            j = plan.call_index_in_group[i]
            self.views.append(CacheView(g, {name: t[j] for name, t in self.tensors[g].items()}, page_size,
                                        write=plan.call_writes[i]))
        self.num_state_slots = max(0, num_state_slots)
        self.states = []
        self.state_initial = []        # per call: None (zeros) or a tensor of one row's shape
        for need in plan.state_needs:
            if need is None:
                self.states.append(None)
                self.state_initial.append(None)
                continue
            dt = _DTYPES[need.dtype]
            st = torch.zeros((self.num_state_slots + 1,) + tuple(need.shape), dtype=dt, device=device)
            first = None
            if need.initial is not None:
                first = torch.as_tensor(need.initial, dtype=dt).to(device).expand(tuple(need.shape)).contiguous()
                st[:] = first
            self.states.append(st)
            self.state_initial.append(first)

    def reset_state(self, slots: torch.Tensor) -> None:
        """Rows `slots` (int64, on the device) of every state tensor back to what a request starts from."""
        for st, first in zip(self.states, self.state_initial):
            if st is None:
                continue
            if first is None:
                st.index_fill_(0, slots, 0)
            else:
                st.index_copy_(0, slots, first.unsqueeze(0).expand((slots.numel(),) + tuple(first.shape)))

    def spare_page(self, group: int) -> int:
        return self.num_pages[group]

    @property
    def spare_state_slot(self) -> int:
        return self.num_state_slots

    @property
    def has_state(self) -> bool:
        return any(s is not None for s in self.states)
