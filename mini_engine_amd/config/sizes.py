"""The layer sizes of the Qwen3 dense models that the benchmarks and the command lines name, for runs
with random weights (no model folder at hand). The figures are those of the published config.json
files; a model folder's own config.json always wins where there is one."""
from __future__ import annotations

from .model_config import Qwen3Config

SIZES = {
    # name: (layers, hidden, q heads, kv heads, head_dim, intermediate, vocab, tied)
    "tinyA": (2, 64, 4, 2, 16, 128, 256, True),
    "0.6b": (28, 1024, 16, 8, 128, 3072, 151936, True),
    "1.7b": (28, 2048, 16, 8, 128, 6144, 151936, True),
    "4b": (36, 2560, 32, 8, 128, 9728, 151936, True),
    "8b": (36, 4096, 32, 8, 128, 12288, 151936, False),
    "14b": (40, 5120, 40, 8, 128, 17408, 151936, False),
    "32b": (64, 5120, 64, 8, 128, 25600, 151936, False),
}


def model_config(size: str, layers: int | None = None):
    """(typed configuration of that size with `layers` layers, or all of them; the size's own layer count)."""
    L, h, Hq, Hkv, D, I, V, tied = SIZES[size]
    return Qwen3Config.from_dict(dict(
        architectures=["Qwen3ForCausalLM"], vocab_size=V, hidden_size=h, intermediate_size=I,
        num_hidden_layers=layers or L, num_attention_heads=Hq, num_key_value_heads=Hkv, head_dim=D,
        rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=tied, max_position_embeddings=40960)), L
