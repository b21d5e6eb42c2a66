"""Plain, slow Qwen3 dense: whole sequences, no cache, one function per part.

Written from the reference's formulas (every function cites the file and
lines it follows) and sharing no code with ``mini_engine_amd``: it reads the
raw ``config.json`` dict and the checkpoint tensors by their stored names.
All arithmetic runs in the dtype of the tensors it is given (float32 or
float64 in the tests); nothing is rounded to bfloat16 here.
"""
from __future__ import annotations

import json
import math
import os

import torch


# ---------------------------------------------------------------- parts

def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """reference layers/layernorm.py:11-16: var = mean(x^2) over the last dim,
    y = weight * (x * rsqrt(var + eps)); the weight is a plain multiplier (no 1+w)."""
    var = x.pow(2).mean(-1, keepdim=True)
    return weight * (x * torch.rsqrt(var + eps))


def add_rms_norm(x, residual, weight, eps):
    """reference layers/layernorm.py:19-24: with a residual the sum is formed first,
    normalised, and also returned as the new residual."""
    residual = x + residual
    return rms_norm(residual, weight, eps), residual


def rope_tables(head_dim: int, num_positions: int, theta: float, dtype=torch.float64):
    """reference layers/rotary_embedding.py:11-18: inv_freq[i] = theta^(-2i/D), i < D/2;
    angle[p, i] = p * inv_freq[i]; the tables are cos/sin of cat(angle, angle) -> [P, D]."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=dtype) / head_dim))
    t = torch.arange(num_positions, dtype=dtype)
    freqs = torch.outer(t, inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos(), emb.sin()


def rotate_half(x):
    """reference layers/rotary_embedding.py:5-8: cat(-x[D/2:], x[:D/2])."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor):
    """reference layers/rotary_embedding.py:20-25: x*cos + rotate_half(x)*sin with the
    table rows of the token positions broadcast over heads. x: [T, H, D]."""
    c = cos[positions].unsqueeze(1).to(x.dtype)
    s = sin[positions].unsqueeze(1).to(x.dtype)
    return x * c + rotate_half(x) * s


def causal_attention(q, k, v, scale: float, window: int | None = None, positions=None):
    """Softmax attention of one whole sequence. q: [T, Hq, D], k/v: [T, Hkv, D].

    reference layers/attention.py:54-59 (causal, scale, grouped heads) and :34-35
    (key j is kept iff j <= query position); consecutive query heads share a key
    head: kv head = q head // (Hq/Hkv) (reference csrc/paged_decode.cu:205-212 handles
    the heads of one group together). ``window`` (not in the reference) further keeps
    only keys with position > query position - window.
    """
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    group = Hq // Hkv
    if positions is None:
        positions = torch.arange(T)
    out = torch.empty_like(q)
    i = positions[:, None]
    j = positions[None, :]
    keep = j <= i
    if window is not None:
        keep = keep & (j > i - window)
    for h in range(Hq):
        kh = h // group
        scores = (q[:, h, :] @ k[:, kh, :].T) * scale          # [T, T]
        scores = scores.masked_fill(~keep, float("-inf"))
        p = torch.softmax(scores, dim=-1)
        out[:, h, :] = p @ v[:, kh, :]
    return out


def silu_and_mul(gate, up):
    """reference layers/activation.py:5-7: silu(gate) * up, gate being the first half."""
    return gate * torch.sigmoid(gate) * up


# ---------------------------------------------------------------- the model

def read_model_folder(model_dir: str, dtype=torch.float64):
    """config.json as a raw dict and every stored tensor, converted to ``dtype``."""
    from safetensors import safe_open

    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    weights = {}
    for name in sorted(os.listdir(model_dir)):
        if name.endswith(".safetensors"):
            with safe_open(os.path.join(model_dir, name), "pt", device="cpu") as f:
                for key in f.keys():
                    weights[key] = f.get_tensor(key).to(dtype)
    return cfg, weights


def _theta(cfg: dict) -> float:
    rope = cfg.get("rope_parameters") or {}
    return float(rope.get("rope_theta", cfg.get("rope_theta")))


def _windows(cfg: dict) -> list:
    L = cfg["num_hidden_layers"]
    if not cfg.get("use_sliding_window") or cfg.get("sliding_window") is None:
        return [None] * L
    types = cfg.get("layer_types")
    if types is None:
        first = cfg.get("max_window_layers", L)
        types = ["sliding_attention" if i >= first else "full_attention" for i in range(L)]
    return [cfg["sliding_window"] if t == "sliding_attention" else None for t in types]


def attention_block(cfg, w, prefix, x, positions, cos, sin, window):
    """reference models/qwen3.py:28-38: q/k/v projections (no bias), per-head RMSNorm of
    q and k over head_dim (not v) before rotation, attention with scale head_dim^-0.5
    (:25), output projection."""
    Hq, Hkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps = cfg["rms_norm_eps"]
    T = x.shape[0]
    q = (x @ w[prefix + "q_proj.weight"].T).view(T, Hq, D)
    k = (x @ w[prefix + "k_proj.weight"].T).view(T, Hkv, D)
    v = (x @ w[prefix + "v_proj.weight"].T).view(T, Hkv, D)
    q = rms_norm(q, w[prefix + "q_norm.weight"], eps)
    k = rms_norm(k, w[prefix + "k_norm.weight"], eps)
    q = apply_rope(q, cos, sin, positions)
    k = apply_rope(k, cos, sin, positions)
    o = causal_attention(q, k, v, D ** -0.5, window, positions)
    return o.reshape(T, Hq * D) @ w[prefix + "o_proj.weight"].T


def mlp_block(w, prefix, x):
    """reference models/qwen3.py:42-51: down(silu(gate(x)) * up(x)), no biases."""
    gate = x @ w[prefix + "gate_proj.weight"].T
    up = x @ w[prefix + "up_proj.weight"].T
    return silu_and_mul(gate, up) @ w[prefix + "down_proj.weight"].T


def hidden_states(cfg: dict, w: dict, token_ids, positions=None):
    """reference models/qwen3.py:86-92 and :65-74: embedding; per layer
    (residual add) -> input norm -> attention -> residual add -> post norm -> mlp;
    the last mlp output is added to the residual inside the final norm."""
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    T = ids.shape[0]
    if positions is None:
        positions = torch.arange(T)
    dtype = w["model.embed_tokens.weight"].dtype
    cos, sin = rope_tables(cfg["head_dim"], int(positions.max()) + 1, _theta(cfg), dtype)
    eps = cfg["rms_norm_eps"]
    windows = _windows(cfg)
    h = w["model.embed_tokens.weight"][ids]                     # layers/embed_head.py:10-11
    residual = None
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        if residual is None:
            residual = h
            x = rms_norm(h, w[p + "input_layernorm.weight"], eps)
        else:
            x, residual = add_rms_norm(h, residual, w[p + "input_layernorm.weight"], eps)
        a = attention_block(cfg, w, p + "self_attn.", x, positions, cos, sin, windows[i])
        x, residual = add_rms_norm(a, residual, w[p + "post_attention_layernorm.weight"], eps)
        h = mlp_block(w, p + "mlp.", x)
    x, _ = add_rms_norm(h, residual, w["model.norm.weight"], eps)
    return x


def logits(cfg: dict, w: dict, token_ids, positions=None) -> torch.Tensor:
    """Logits at every position, [T, V]. reference models/qwen3.py:107-117 and
    layers/embed_head.py:19-23: the head is the embedding matrix when tied."""
    x = hidden_states(cfg, w, token_ids, positions)
    tied = cfg.get("tie_word_embeddings")
    if tied is None:
        tied = "lm_head.weight" not in w
    head = w["model.embed_tokens.weight"] if tied else w["lm_head.weight"]
    return x @ head.T


def greedy_generate(cfg: dict, w: dict, prompt, num_tokens: int) -> list:
    """Greedy continuation by recomputing the whole sequence for every token
    (reference layers/sampler.py:6: argmax at temperature 0)."""
    ids = list(prompt)
    out = []
    for _ in range(num_tokens):
        nxt = int(torch.argmax(logits(cfg, w, ids)[-1]))
        out.append(nxt)
        ids.append(nxt)
    return out


def sample_gumbel_reference(logits_row: torch.Tensor, temperature: float, noise_exp: torch.Tensor) -> int:
    """reference layers/sampler.py:5-11: argmax(softmax(logits/T) / E) with E ~ Exp(1);
    temperature 0 is argmax."""
    z = logits_row.to(torch.float64)
    if temperature == 0:
        return int(torch.argmax(z))
    probs = torch.softmax(z / temperature, dim=-1)
    return int(torch.argmax(probs / noise_exp))
