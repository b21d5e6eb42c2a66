"""A decoder assembled from parts: embedding, layers run in a listed order, final norm, head.

Nothing here knows an architecture. An architecture module builds a `DecoderModel`
from its typed config by choosing parts layer by layer, and names where each
parameter is stored in a checkpoint (`weight_sources`).
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ..kernels import ops
from ..parts.base import CacheNeed, LayerCall, Part, StateNeed
from ..parts.block import norm_of


@dataclass
class CachePlan:
    """Which page group each layer call uses, and which calls own pages there."""

    group_needs: list                      # per group: CacheNeed
    group_calls: list                      # per group: indices of the calls that own pages (in run order)
    call_group: list                       # per call: group index or None
    call_index_in_group: list              # per call: which slice of the group's pool it reads/writes
    call_writes: list                      # per call: True if it owns (writes) its slice
    state_needs: list                      # per call: StateNeed or None


@dataclass
class WeightSource:
    """Rows [row_start, row_start + rows) of an engine parameter come from checkpoint tensor `name`."""

    name: str
    row_start: int = 0
    rows: int | None = None                # None: the whole parameter


class DecoderModel(Part):
    def __init__(self, config, embedding: Part, layers: list, order: list, final_norm: Part, head: Part,
                 weight_sources: dict, optional_sources: set | None = None):
        super().__init__()
        self.config = config
        self.add_child("embedding", embedding)
        self.layers = list(layers)
        for i, layer in enumerate(self.layers):
            self.add_child(f"layers.{i}", layer)
        self.order = [c if isinstance(c, LayerCall) else LayerCall(int(c)) for c in order]
        self.add_child("final_norm", final_norm)
        self.add_child("head", head)
        # engine parameter name -> list[WeightSource]
        self.weight_sources = weight_sources
        # checkpoint tensor names that may be present but are not used (e.g. a stored head when tied)
        self.optional_sources = set(optional_sources or ())
        self.device = None
        self.dtype = None
        for i, call in enumerate(self.order):
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"run order entry {i} names layer {call.layer}, the model has {len(self.layers)}")
            if call.cache_of is not None and not 0 <= call.cache_of < i:
                raise ValueError(f"run order entry {i} may only read the cache of an earlier entry, got {call.cache_of}")

    # -- what the cache has to provide ------------------------------------------------------
    def cache_plan(self) -> CachePlan:
        keys: dict = {}
        needs, calls = [], []
        call_group, call_idx, call_writes, states = [], [], [], []
        for i, call in enumerate(self.order):
            layer = self.layers[call.layer]
            need: CacheNeed | None = layer.cache_need() if hasattr(layer, "cache_need") else None
            state: StateNeed | None = layer.state_need() if hasattr(layer, "state_need") else None
            states.append(state)
            if need is None:
                call_group.append(None); call_idx.append(None); call_writes.append(False)
                continue
            if call.cache_of is not None:
                src = call.cache_of
                if call_group[src] is None or not call_writes[src]:
                    raise ValueError(f"run order entry {i} reads the cache of entry {src}, which owns none")
                if need.tensors != needs[call_group[src]].tensors:
                    raise ValueError(f"run order entry {i} and entry {src} disagree on what a page of the cache holds")
                call_group.append(call_group[src]); call_idx.append(call_idx[src]); call_writes.append(False)
                continue
            g = keys.setdefault(need.group_key(), len(needs))
            if g == len(needs):
                needs.append(need); calls.append([])
            call_group.append(g); call_idx.append(len(calls[g])); call_writes.append(True)
            calls[g].append(i)
        return CachePlan(needs, calls, call_group, call_idx, call_writes, states)

    # -- running ----------------------------------------------------------------------------
    def finalize_all(self, device, dtype, max_positions: int) -> None:
        self.device, self.dtype = torch.device(device), dtype
        for part in self.parts():
            part.finalize(self.device, dtype, max_positions)

    def forward(self, token_ids: torch.Tensor, step, caches: list, states: list):
        """token_ids int32 [T] -> (last layer output, residual): both go to `logits`.

        caches[i] / states[i]: the CacheView / state tensor of run-order entry i (or None)."""
        h = self.embedding.forward(token_ids)
        residual = None
        for i, call in enumerate(self.order):
            h, residual = self.layers[call.layer].forward(h, residual, step, caches[i], states[i])
        return h, residual

    def logits(self, h, residual, rows: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """Final norm of (h + residual), then the rows that want logits, then the head: float32
        [len(rows), vocab] (reference models/qwen3.py:91,116-117; layers/embed_head.py:19-23).
        `out`: where the head puts them (`parts.Head.forward(x, out)`)."""
        x, _ = norm_of(self.final_norm, h, residual)
        x = ops.gather_rows(x, rows)
        return self.head.forward(x, out=out)
