"""mini_engine_amd: a small, whole inference engine for one decoder architecture on one AMD
MI355X (gfx950) GPU: typed config and registry, safetensors weights, parts assembled into
layers, a paged cache, one step function, a scheduler, sampling, and hand-written HIP kernels.
"""
from . import parts  # noqa: F401  (registers the built-in parts)
from .config.engine_config import EngineConfig  # noqa: F401
from .llm import LLM  # noqa: F401
from .sampling.sampling_params import SamplingParams  # noqa: F401

__all__ = ["LLM", "SamplingParams", "EngineConfig"]
