"""One request's state as the scheduler sees it (reference engine/sequence.py:8-75).

The block table lives in the cache manager, keyed by `seq_id`; the page size is the
engine's, not a class-level global (the reference fixes `Sequence.block_size = 16`).
"""
from __future__ import annotations

from enum import Enum
from itertools import count
from time import perf_counter

from ..sampling.sampling_params import SamplingParams


class SequenceStatus(Enum):
    WAITING = 1
    RUNNING = 2
    FINISHED = 3


class Sequence:
    _ids = count()

    def __init__(self, token_ids: list, sampling_params: SamplingParams | None = None, priority: int = 0,
                 sample_stream: int | None = None):
        if not token_ids:
            raise ValueError("a request needs at least one prompt token")
        self.seq_id = next(Sequence._ids)
        self.status = SequenceStatus.WAITING
        self.token_ids = list(token_ids)
        self.num_prompt_tokens = len(self.token_ids)
        self.num_computed_tokens = 0       # tokens whose keys/values are in the cache
        self.num_cached_tokens = 0         # of those, how many came from prefix reuse
        self.num_scheduled_tokens = 0      # tokens to run in the step being built
        self.sampling_params = sampling_params if sampling_params is not None else SamplingParams()
        self.priority = priority           # lower is served first under the priority policy
        self.arrival_time = perf_counter()
        # identity of the request for the sampler's noise: its index among the requests of a
        # generate() call when given, so results do not depend on earlier traffic
        self.sample_stream = self.seq_id if sample_stream is None else sample_stream

    def __len__(self):
        return len(self.token_ids)

    @property
    def num_tokens(self) -> int:
        return len(self.token_ids)

    @property
    def last_token(self) -> int:
        return self.token_ids[-1]

    @property
    def is_finished(self) -> bool:
        return self.status == SequenceStatus.FINISHED

    @property
    def num_completion_tokens(self) -> int:
        return len(self.token_ids) - self.num_prompt_tokens

    @property
    def prompt_token_ids(self) -> list:
        return self.token_ids[:self.num_prompt_tokens]

    @property
    def completion_token_ids(self) -> list:
        return self.token_ids[self.num_prompt_tokens:]

    @property
    def num_uncomputed_tokens(self) -> int:
        return len(self.token_ids) - self.num_computed_tokens

    @property
    def samples_this_step(self) -> bool:
        """The scheduled tokens reach the end of what is known: the step's last logits pick the next token."""
        return self.num_computed_tokens + self.num_scheduled_tokens == len(self.token_ids)

    def append_token(self, token_id: int) -> None:
        self.token_ids.append(int(token_id))
