"""Qwen3 dense, assembled from parts by its config (reference models/qwen3.py:12-117).

Per layer: RMSNorm -> attention (packed q/k/v, per-head RMSNorm of q and k, rotary, grouped
heads, causal or windowed) -> RMSNorm -> SiLU-gated feed-forward, around a residual stream;
a final RMSNorm; a head that is the embedding matrix when `tie_word_embeddings`.
"""
from __future__ import annotations

from ..config.model_config import Qwen3Config
from ..parts.base import LayerCall, make_part
from ..parts.embedding import LMHead, TokenEmbedding
from ..registry import register_architecture
from .model import DecoderModel, WeightSource


@register_architecture("Qwen3ForCausalLM")
def build_qwen3(cfg: Qwen3Config, checkpoint_names=None) -> DecoderModel:
    """A config without `tie_word_embeddings` is resolved by the checkpoint: the head is the embedding
    matrix exactly when no `lm_head.weight` is stored (untied when there is no checkpoint at all)."""
    tie = cfg.tie_word_embeddings
    if tie is None:
        tie = checkpoint_names is not None and "lm_head.weight" not in checkpoint_names
    h, D = cfg.hidden_size, cfg.head_dim
    Hq, Hkv = cfg.num_attention_heads, cfg.num_key_value_heads
    rotary = make_part("position_encoding", "rotary", head_dim=D, theta=cfg.rope_theta)   # one for all layers
    layers, sources = [], {}
    for i in range(cfg.num_hidden_layers):
        window = cfg.sliding_window if cfg.layer_types[i] == "sliding_attention" else None
        mixer = make_part("mixer", "attention", hidden_size=h, num_heads=Hq, num_kv_heads=Hkv, head_dim=D,
                          scale=D ** -0.5, qk_norm_eps=cfg.rms_norm_eps, position=rotary, window=window)
        ffn = make_part("feed_forward", "swiglu", hidden_size=h, intermediate_size=cfg.intermediate_size)
        layers.append(make_part("block", "pre_norm",
                                norm1=make_part("norm", "rms", size=h, eps=cfg.rms_norm_eps), mixer=mixer,
                                norm2=make_part("norm", "rms", size=h, eps=cfg.rms_norm_eps), feed_forward=ffn))
        # checkpoint names: reference utils/loader.py:25-31 with models/qwen3.py:96-102 (packing)
        ck, me = f"model.layers.{i}.", f"layers.{i}."
        sources[me + "norm1.weight"] = [WeightSource(ck + "input_layernorm.weight")]
        sources[me + "norm2.weight"] = [WeightSource(ck + "post_attention_layernorm.weight")]
        q, kv = Hq * D, Hkv * D
        sources[me + "mixer.qkv.weight"] = [WeightSource(ck + "self_attn.q_proj.weight", 0, q),
                                            WeightSource(ck + "self_attn.k_proj.weight", q, kv),
                                            WeightSource(ck + "self_attn.v_proj.weight", q + kv, kv)]
        sources[me + "mixer.q_norm_weight"] = [WeightSource(ck + "self_attn.q_norm.weight")]
        sources[me + "mixer.k_norm_weight"] = [WeightSource(ck + "self_attn.k_norm.weight")]
        sources[me + "mixer.o.weight"] = [WeightSource(ck + "self_attn.o_proj.weight")]
        I = cfg.intermediate_size
        sources[me + "feed_forward.gate_up.weight"] = [WeightSource(ck + "mlp.gate_proj.weight", 0, I),
                                                       WeightSource(ck + "mlp.up_proj.weight", I, I)]
        sources[me + "feed_forward.down.weight"] = [WeightSource(ck + "mlp.down_proj.weight")]
    embedding = TokenEmbedding(cfg.vocab_size, h)
    head = LMHead(cfg.vocab_size, h, tied_to=embedding if tie else None)
    sources["embedding.weight"] = [WeightSource("model.embed_tokens.weight")]
    sources["final_norm.weight"] = [WeightSource("model.norm.weight")]
    optional = set()
    if tie:
        optional.add("lm_head.weight")      # a stored head is ignored when tied (reference utils/loader.py:23-24)
    else:
        sources["head.weight"] = [WeightSource("lm_head.weight")]
    return DecoderModel(cfg, embedding, layers, [LayerCall(i) for i in range(cfg.num_hidden_layers)],
                        make_part("norm", "rms", size=h, eps=cfg.rms_norm_eps), head, sources, optional)
