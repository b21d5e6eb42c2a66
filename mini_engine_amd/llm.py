"""`LLM(model_dir, **engine options).generate(prompts, SamplingParams(...))` (reference llm.py:4-5)."""
from .engine.llm_engine import LLMEngine


class LLM(LLMEngine):
    pass
