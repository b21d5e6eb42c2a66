"""Greedy and temperature sampling (reference layers/sampler.py:4-11).

The reference draws exponential noise for the whole [S, V] matrix from the global generator,
so a request's tokens depend on who shares its batch. Here the noise is a hash of
(seed, request, output index, vocabulary id): the same request gives the same tokens under any
batching, chunking or preemption.
"""
from __future__ import annotations

_MASK64 = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK64
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK64
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK64
    return x ^ (x >> 31)


def row_key(seed: int, request: int, output_index: int) -> tuple:
    """Two 32-bit words that key the noise of one sampled token."""
    x = _splitmix64(seed & _MASK64)
    x = _splitmix64(x ^ (request & _MASK64))
    x = _splitmix64(x ^ (output_index & _MASK64))
    return x & 0xFFFFFFFF, x >> 32


class Sampler:
    def __init__(self, runner, seed: int = 0):
        self.runner = runner
        self.seed = seed

    def __call__(self, logits, requests: list) -> list:
        """One token per row of float32 logits [S, V]; requests[s] gives temperature, seed, identity
        and how many tokens the request has generated so far."""
        return self.launch(logits, requests).tokens()

    def launch(self, logits, requests: list):
        """The same, not waiting for the tokens: returns the runner's handle, whose tokens() fetches
        them. The next decode step of these requests may be started before that."""
        temps = [r.params.temperature for r in requests]
        keys = [row_key(self.seed if r.params.seed is None else r.params.seed, r.noise_stream, r.num_generated)
                for r in requests]
        return self.runner.sample_async(logits, temps, keys, [r.id for r in requests])
