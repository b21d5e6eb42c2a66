"""Per-step metadata handed to every part (reference utils/context.py:3-28, built in
engine/model_runner.py:87-126). Passed explicitly instead of through a module global."""
from __future__ import annotations

from dataclasses import dataclass, field

import torch


@dataclass
class GroupStep:
    block_tables: torch.Tensor      # int32 [B, MB] page ids of this group, -1 where none
    slot_mapping: torch.Tensor      # int32 [T] page_id * page_size + offset of each new token


@dataclass
class StepContext:
    num_tokens: int
    num_seqs: int
    num_decodes: int                # requests with exactly one new token; they come first
    positions: torch.Tensor         # int32 [T]
    seq_of_token: torch.Tensor      # int32 [T] index of the token's request in this step
    context_lens: torch.Tensor      # int32 [B] keys visible after this step's write
    cu_seqlens: torch.Tensor        # int32 [B + 1] prefix sums of new-token counts
    prefill_cu: torch.Tensor | None  # int32 [B - Dn + 1] the same for the non-decode requests, from 0
    max_decode_context: int
    max_prefill_context: int = 0     # largest context among the requests with more than one new token
    decode_contexts_even: bool = False   # the decode requests' contexts are (nearly) equally long
    groups: list = field(default_factory=list)       # GroupStep per page group
    state_slots: torch.Tensor | None = None          # int32 [B]
    first_chunk: torch.Tensor | None = None          # int32 [B]: 1 if the request's tokens start at position 0
    # host copies, for parts that decide launches on the host
    q_lens: list = field(default_factory=list)
    starts: list = field(default_factory=list)
