"""Engine options, with the names, meanings and checks of reference ``config.py:4-29``.

Added beside the reference's fields: ``dtype`` (bfloat16 or a true float32 path),
``seed`` (sampling noise is a function of seed, request and output index),
``enable_prefix_caching``, ``use_graphs``, ``run_ahead`` and ``random_weights``; ``num_kvcache_blocks`` may be given
(the reference always sizes the pool itself, ``engine/model_runner.py:46-48``).
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field, fields

from .model_config import ConfigError, load_model_config

DTYPES = ("bfloat16", "float32")


@dataclass
class EngineConfig:
    model: str
    kvcache_block_size: int = 16
    num_kvcache_blocks: int = -1          # -1: sized from free memory and gpu_memory_utilization
    max_num_seqs: int = 512
    max_num_batched_tokens: int = 16384
    eos: int = -1
    max_model_len: int = 4096
    gpu_memory_utilization: float = 0.9
    enable_chunked_prefill: bool = True
    long_prefill_token_threshold: int = 0
    scheduling_policy: str = "fcfs"
    dtype: str = "bfloat16"
    seed: int = 0
    enable_prefix_caching: bool = True
    use_graphs: bool = True
    run_ahead: bool = True                # launch the next plain decode step before this one's tokens are fetched
    random_weights: int | None = None     # a seed: the folder needs only config.json, weights are drawn on the device
    model_config: object = field(default=None, repr=False)

    @classmethod
    def from_options(cls, model: str, options: dict) -> "EngineConfig":
        """The options this class knows, out of a mapping that may hold others (the reference's entry
        point takes any keyword and passes on what its config knows, engine/llm_engine.py:13-16)."""
        known = {f.name for f in fields(cls)} - {"model"}
        return cls(model, **{name: options[name] for name in options.keys() & known})

    def __post_init__(self):
        self.model = os.path.expanduser(self.model)
        if not os.path.isdir(self.model):
            raise ConfigError(f"model must be a folder with config.json and *.safetensors: {self.model!r}")
        if self.dtype in ("bf16",):
            self.dtype = "bfloat16"
        if self.dtype in ("fp32", "float"):
            self.dtype = "float32"
        if self.dtype not in DTYPES:
            raise ConfigError(f"dtype must be one of {DTYPES}, got {self.dtype!r}")
        if self.max_num_batched_tokens < self.max_num_seqs:
            raise ConfigError("max_num_batched_tokens must be >= max_num_seqs "
                              "(every running request must be able to decode in one step)")
        if self.scheduling_policy not in ("fcfs", "priority"):
            raise ConfigError(f"scheduling_policy must be 'fcfs' or 'priority', got {self.scheduling_policy!r}")
        if self.long_prefill_token_threshold < 0:
            raise ConfigError("long_prefill_token_threshold must be >= 0")
        if self.kvcache_block_size < 1:
            raise ConfigError("kvcache_block_size must be positive")
        if not 0 < self.gpu_memory_utilization <= 1:
            raise ConfigError("gpu_memory_utilization must lie in (0, 1]")
        if self.model_config is None:
            self.model_config = load_model_config(self.model)
        limit = getattr(self.model_config, "max_position_embeddings", None)
        if limit is not None:
            self.max_model_len = min(self.max_model_len, limit)
        if not self.enable_chunked_prefill and self.max_num_batched_tokens < self.max_model_len:
            raise ConfigError("without chunked prefill a whole prompt must fit the token budget: "
                              "max_num_batched_tokens >= max_model_len")
        if self.eos == -1:
            eos = getattr(self.model_config, "eos_token_id", None)
            if eos is not None:
                self.eos = int(eos)
