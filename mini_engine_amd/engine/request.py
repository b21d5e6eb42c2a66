"""What the scheduler knows about one request (reference engine/sequence.py:8-75 keeps the same
facts; the block table lives in the cache manager here, keyed by the request's id, and the page
size is the engine's, not a class-level constant)."""
from __future__ import annotations

import enum
import itertools
import time
from dataclasses import dataclass, field

from ..sampling.sampling_params import SamplingParams


class Phase(enum.Enum):
    QUEUED = "queued"        # waiting for admission, holds nothing
    LIVE = "live"            # admitted: holds pages (and a state slot), takes part in steps
    DONE = "done"            # ended by its end token or by max_tokens


_next_id = itertools.count()


@dataclass(eq=False)
class Request:
    tokens: list                      # prompt, then what was generated; may end in a placeholder (scheduler.UNKNOWN)
    params: SamplingParams = field(default_factory=SamplingParams)
    priority: int = 0                 # lower is served first under the priority policy
    noise_stream: int | None = None   # identity for the sampler's noise; None: the request's id
    id: int = field(init=False)
    prompt_len: int = field(init=False)
    arrived: float = field(init=False)
    phase: Phase = field(init=False, default=Phase.QUEUED)
    in_cache: int = field(init=False, default=0)        # tokens whose keys and values the cache holds
    from_prefix: int = field(init=False, default=0)     # of those, how many another request had left there
    portion: int = field(init=False, default=0)         # tokens it runs in the step being planned
    times_evicted: int = field(init=False, default=0)   # how often it gave everything back and returned to the queue

    def __post_init__(self):
        self.tokens = [int(t) for t in self.tokens]
        if not self.tokens:
            raise ValueError("a request needs at least one prompt token")
        self.id = next(_next_id)
        self.prompt_len = len(self.tokens)
        self.arrived = time.perf_counter()
        if self.noise_stream is None:
            self.noise_stream = self.id

    @property
    def owed(self) -> int:
        """Known tokens not yet in the cache: 1 while decoding, more for a prompt (or a request fed again)."""
        return len(self.tokens) - self.in_cache

    @property
    def num_generated(self) -> int:
        return len(self.tokens) - self.prompt_len

    @property
    def generated(self) -> list:
        return self.tokens[self.prompt_len:]

    @property
    def done(self) -> bool:
        return self.phase is Phase.DONE
