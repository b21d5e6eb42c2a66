"""Pins the plain implementation by what fixes it beside the reference's text: special cases
that reduce to library routines, and invariants, each chosen so that a plausible mistake
(a wrong sign or pairing, a norm in the wrong place, a wrong head grouping) fails it.

The reference publishes no test vectors (its checks are git-ignored, reference .gitignore:10-12),
so none can be used here: parity with its numbers is unpinned, parity with its formulas is
what these tests hold. The model code of installed packages is no source for this repository
(neither read, imported nor run), so no test compares with one; what stands in for it: the
attention scale is the library routine's own default, the rotation's frequencies are literals
worked out by hand, the rotation is a complex product, the window is a band matrix written out.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import helpers
import plain_qwen3 as P

torch.manual_seed(0)
D64 = torch.float64


def test_rms_norm_is_library_rms_norm():
    x = torch.randn(5, 7, 24, dtype=D64)
    w = torch.rand(24, dtype=D64) + 0.5
    got = P.rms_norm(x, w, 1e-5)
    assert torch.allclose(got, F.rms_norm(x, (24,), w, 1e-5), atol=1e-12)
    # weight is a plain multiplier (a "1 + w" convention would double this)
    assert torch.allclose(P.rms_norm(x, torch.ones(24, dtype=D64), 0.0).pow(2).mean(-1),
                          torch.ones(5, 7, dtype=D64), atol=1e-12)
    # eps sits inside the square root, added to the mean of squares
    tiny = torch.full((1, 4), 1e-4, dtype=D64)
    assert torch.allclose(P.rms_norm(tiny, torch.ones(4, dtype=D64), 1e-6),
                          tiny / math.sqrt(1e-8 + 1e-6), atol=1e-12)


def test_add_rms_norm_returns_sum_as_residual():
    x, r = torch.randn(3, 8, dtype=D64), torch.randn(3, 8, dtype=D64)
    w = torch.rand(8, dtype=D64)
    y, res = P.add_rms_norm(x, r, w, 1e-6)
    assert torch.equal(res, x + r)
    assert torch.allclose(y, P.rms_norm(x + r, w, 1e-6))


def test_rope_frequencies_by_hand():
    """The frequencies worked out by hand, not by the formula's own expression. Head size 8, theta 10^4: pair i
    turns by theta^(-2i/8) per position = 1, 1/10, 1/100, 1/1000 (an exponent of i/D, (2i+1)/D or 2i/(D-2) gives
    other numbers); head size 4, theta 10^6: 1 and 1/1000. The cos/sin literals are those of 3, 0.3, 0.03, 0.003."""
    cos, sin = P.rope_tables(8, 4, 10000.0)
    want_cos = [-0.9899924966004454, 0.955336489125606, 0.9995500337489875, 0.9999955000033750]
    want_sin = [0.1411200080598672, 0.29552020666133955, 0.02999550020249566, 0.0029999955000020250]
    assert torch.allclose(cos[3, :4], torch.tensor(want_cos, dtype=D64), atol=1e-14)
    assert torch.allclose(sin[3, :4], torch.tensor(want_sin, dtype=D64), atol=1e-14)
    assert torch.equal(cos[:, :4], cos[:, 4:]) and torch.equal(sin[:, :4], sin[:, 4:])    # both halves carry the same angle
    cos, sin = P.rope_tables(4, 2001, 1e6)
    # one position turns pair 1 by a thousandth of a radian: after 2,000 positions it has turned by 2 radians
    assert torch.allclose(cos[2000, 1], torch.tensor(-0.4161468365471424, dtype=D64), atol=1e-12)
    assert torch.allclose(sin[1, 0], torch.tensor(0.8414709848078965, dtype=D64), atol=1e-14)       # pair 0: one radian


def test_rope_tables_and_pairing():
    Dh, n, theta = 16, 50, 10000.0
    cos, sin = P.rope_tables(Dh, n, theta)
    # the angle of pair i grows linearly with the position, pair 0 by one radian a position, and the pairs'
    # rates form a geometric sequence that ends one step (a factor theta^(2/D)) above 1/theta
    ang = torch.atan2(sin[1, :Dh // 2], cos[1, :Dh // 2])          # position 1: all angles are below pi
    assert torch.allclose(ang[0], torch.tensor(1.0, dtype=D64))
    assert torch.allclose(ang[1:] / ang[:-1], torch.full((Dh // 2 - 1,), theta ** (-2 / Dh), dtype=D64))
    assert torch.allclose(ang[-1] * theta ** (-2 / Dh), torch.tensor(1 / theta, dtype=D64))
    ang = torch.outer(torch.arange(n, dtype=D64), ang)
    assert torch.allclose(cos[:, :Dh // 2], ang.cos()) and torch.allclose(cos[:, Dh // 2:], ang.cos())
    assert torch.allclose(sin[:, Dh // 2:], ang.sin())
    x = torch.randn(n, 3, Dh, dtype=D64)
    pos = torch.arange(n)
    y = P.apply_rope(x, cos, sin, pos)
    # position 0 is the identity
    assert torch.allclose(y[0], x[0])
    # equals a complex multiplication of the pairs (x_i, x_{i+D/2}) by e^{i p theta_i}:
    # an interleaved pairing (x_2i, x_2i+1) or a flipped sign fails this
    z = torch.complex(x[..., :Dh // 2], x[..., Dh // 2:]) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    assert torch.allclose(y[..., :Dh // 2], z.real) and torch.allclose(y[..., Dh // 2:], z.imag)
    # each pair keeps its norm
    assert torch.allclose(y[..., :Dh // 2] ** 2 + y[..., Dh // 2:] ** 2,
                          x[..., :Dh // 2] ** 2 + x[..., Dh // 2:] ** 2)


def test_rope_scores_depend_only_on_distance():
    Dh = 32
    cos, sin = P.rope_tables(Dh, 200, 1e6)
    q, k = torch.randn(1, 1, Dh, dtype=D64), torch.randn(1, 1, Dh, dtype=D64)
    def score(m, n):
        return (P.apply_rope(q, cos, sin, torch.tensor([m])) * P.apply_rope(k, cos, sin, torch.tensor([n]))).sum()
    assert torch.allclose(score(17, 5), score(117, 105), atol=1e-10)
    assert not torch.allclose(score(17, 5), score(17, 6), atol=1e-6)


@pytest.mark.parametrize("Hq,Hkv", [(4, 4), (6, 2), (4, 1), (1, 1)])
def test_attention_is_library_causal_attention(Hq, Hkv):
    T, Dh = 19, 16
    q, k, v = torch.randn(T, Hq, Dh, dtype=D64), torch.randn(T, Hkv, Dh, dtype=D64), torch.randn(T, Hkv, Dh, dtype=D64)
    got = P.causal_attention(q, k, v, 0.37)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                         is_causal=True, scale=0.37, enable_gqa=True)[0].transpose(0, 1)
    assert torch.allclose(got, ref, atol=1e-12)
    got = P.causal_attention(q, k, v, Dh ** -0.5)
    # grouped heads == every kv head repeated for its consecutive query heads
    rep = Hq // Hkv
    full = P.causal_attention(q, k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1), Dh ** -0.5)
    assert torch.allclose(got, full, atol=1e-12)


def test_attention_special_cases():
    Dh = 8
    q, k, v = torch.randn(5, 2, Dh, dtype=D64), torch.randn(5, 1, Dh, dtype=D64), torch.randn(5, 1, Dh, dtype=D64)
    out = P.causal_attention(q, k, v, 0.3)
    # the first token sees only itself: output is its own value row
    assert torch.allclose(out[0, 0], v[0, 0]) and torch.allclose(out[0, 1], v[0, 0])
    # scale 0 -> uniform average of the visible values
    out0 = P.causal_attention(q, k, v, 0.0)
    assert torch.allclose(out0[3, 0], v[:4, 0].mean(0))
    # window w keeps exactly the last w keys, the query's own included
    outw = P.causal_attention(q, k, v, 0.0, window=2)
    assert torch.allclose(outw[4, 0], v[3:5, 0].mean(0))
    # a window as long as the sequence changes nothing
    assert torch.allclose(P.causal_attention(q, k, v, 0.3, window=5), out)
    # the library routine with the band written out: query i sees keys i - w + 1 .. i
    T, w = 23, 6
    q, k, v = torch.randn(T, 2, Dh, dtype=D64), torch.randn(T, 2, Dh, dtype=D64), torch.randn(T, 2, Dh, dtype=D64)
    band = torch.ones(T, T, dtype=torch.bool).tril().triu(-(w - 1))
    assert band[10].nonzero().flatten().tolist() == [5, 6, 7, 8, 9, 10]
    ref = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                         attn_mask=band, scale=0.3)[0].transpose(0, 1)
    assert torch.allclose(P.causal_attention(q, k, v, 0.3, window=w), ref, atol=1e-12)


def test_far_key_dominates():
    """One key scaled to stand out among hundreds must receive (almost) all the weight."""
    T, Dh = 300, 16
    q, k, v = torch.randn(T, 1, Dh, dtype=D64), torch.randn(T, 1, Dh, dtype=D64), torch.randn(T, 1, Dh, dtype=D64)
    k[7, 0] = q[T - 1, 0] * 50
    out = P.causal_attention(q, k, v, Dh ** -0.5)
    assert torch.allclose(out[T - 1, 0], v[7, 0], atol=1e-6)


def test_silu_and_mul_is_library_silu():
    g, u = torch.randn(4, 9, dtype=D64), torch.randn(4, 9, dtype=D64)
    assert torch.allclose(P.silu_and_mul(g, u), F.silu(g) * u, atol=1e-14)


def _folder(tmp_path, name):
    return helpers.make_folder(name, str(tmp_path / name), torch.float32)


def test_model_reduces_to_hand_composition(tmp_path):
    """One layer, written out by hand with library routines only."""
    cfgd = dict(helpers.CONFIGS["B"], num_hidden_layers=1)
    from mini_engine_amd.config.model_config import Qwen3Config
    from mini_engine_amd.weights.random_init import write_random_model
    d = write_random_model(Qwen3Config.from_dict(cfgd), 5, str(tmp_path / "one"), torch.float32)
    cfg, w = P.read_model_folder(d, D64)
    ids = helpers.random_ids(11, cfg["vocab_size"], 3)
    got = P.logits(cfg, w, ids)
    Hq, Hkv, Dh, eps = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["rms_norm_eps"]
    h = F.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    p = "model.layers.0."
    x = F.rms_norm(h, (h.shape[-1],), w[p + "input_layernorm.weight"], eps)
    q = F.linear(x, w[p + "self_attn.q_proj.weight"]).view(-1, Hq, Dh)
    k = F.linear(x, w[p + "self_attn.k_proj.weight"]).view(-1, Hkv, Dh)
    v = F.linear(x, w[p + "self_attn.v_proj.weight"]).view(-1, Hkv, Dh)
    q = F.rms_norm(q, (Dh,), w[p + "self_attn.q_norm.weight"], eps)
    k = F.rms_norm(k, (Dh,), w[p + "self_attn.k_norm.weight"], eps)
    cos, sin = P.rope_tables(Dh, 11, cfg["rope_theta"])
    q, k = P.apply_rope(q, cos, sin, torch.arange(11)), P.apply_rope(k, cos, sin, torch.arange(11))
    # no scale is handed to the library: its default, 1 / sqrt(head size), is what the model's attention must use
    # (reference models/qwen3.py:25 hands head_dim ** -0.5 to its kernels; a scale of 1 / head size, or 1 /
    # sqrt(hidden / heads) where that differs from the head size as it does here (80 / 6), fails this)
    o = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                       is_causal=True, enable_gqa=True)[0].transpose(0, 1)
    res = h + F.linear(o.reshape(11, -1), w[p + "self_attn.o_proj.weight"])
    x = F.rms_norm(res, (res.shape[-1],), w[p + "post_attention_layernorm.weight"], eps)
    m = F.linear(F.silu(F.linear(x, w[p + "mlp.gate_proj.weight"])) * F.linear(x, w[p + "mlp.up_proj.weight"]),
                 w[p + "mlp.down_proj.weight"])
    x = F.rms_norm(m + res, (res.shape[-1],), w["model.norm.weight"], eps)
    ref = F.linear(x, w["lm_head.weight"])
    assert torch.allclose(got, ref, atol=1e-10)


def test_model_is_causal_and_shift_invariant(tmp_path):
    d = _folder(tmp_path, "A")
    cfg, w = P.read_model_folder(d, D64)
    ids = helpers.random_ids(30, cfg["vocab_size"], 1)
    full = P.logits(cfg, w, ids)
    # causality: a prefix gives the same logits
    assert torch.allclose(P.logits(cfg, w, ids[:12]), full[:12], atol=1e-10)
    # only distances count: shifting every position by the same amount changes nothing
    shifted = P.logits(cfg, w, ids, positions=torch.arange(30) + 100)
    assert torch.allclose(shifted, full, atol=1e-9)
    # tied head: the head is the embedding matrix
    assert "lm_head.weight" not in w


def test_window_layers_limit_what_is_seen(tmp_path):
    d = _folder(tmp_path, "C")
    cfg, w = P.read_model_folder(d, D64)
    assert P._windows(cfg) == [None, 24, None, 24]
    cfg_w = dict(cfg, layer_types=["sliding_attention"] * 4)
    ids = helpers.random_ids(60, cfg["vocab_size"], 2)
    ids2 = list(ids)
    ids2[0] = (ids2[0] + 1) % cfg["vocab_size"]
    # with every layer windowed (24) over 4 layers, position 100 > 4*23 cannot see token 0 ...
    a = P.logits(cfg_w, w, ids + ids)[-1]
    b = P.logits(cfg_w, w, ids2 + ids)[-1]
    assert torch.allclose(a, b, atol=1e-9)
    # ... while the mixed model (full layers) does
    assert not torch.allclose(P.logits(cfg, w, ids + ids)[-1], P.logits(cfg, w, ids2 + ids)[-1], atol=1e-9)


def test_sampler_formula():
    """argmax(softmax(z/T)/E) == argmax(z/T - log E); temperature 0 is argmax whatever the noise."""
    z = torch.randn(50, dtype=D64)
    e = torch.empty(50, dtype=D64).exponential_(1.0)
    assert P.sample_gumbel_reference(z, 0.7, e) == int(torch.argmax(z / 0.7 - torch.log(e)))
    assert P.sample_gumbel_reference(z, 0.0, e) == int(torch.argmax(z))


def test_q_and_k_pass_a_norm_and_v_does_not(tmp_path):
    """reference models/qwen3.py:34-35 norms q and k per head and leaves v alone. What that means, whatever the
    code looks like: the block's output does not change when q_proj or k_proj is scaled (an RMS norm forgets
    the scale of its input, up to eps) and is linear in v_proj (the output is a weighted sum of raw values)."""
    d = _folder(tmp_path, "B")
    cfg, w = P.read_model_folder(d, D64)
    p = "model.layers.1.self_attn."
    T = 13
    x = torch.randn(T, cfg["hidden_size"], dtype=D64, generator=torch.Generator().manual_seed(2))
    cos, sin = P.rope_tables(cfg["head_dim"], T, cfg["rope_theta"], D64)
    run = lambda weights: P.attention_block(cfg, weights, p, x, torch.arange(T), cos, sin, None)
    base = run(w)
    for name in ("q_proj.weight", "k_proj.weight"):
        scaled = run({**w, p + name: w[p + name] * 7.0})
        assert float((scaled - base).abs().max()) <= 1e-3 * float(base.abs().max()), name   # eps keeps it from being exact
    assert torch.allclose(run({**w, p + "v_proj.weight": w[p + "v_proj.weight"] * 7.0}), base * 7.0, rtol=1e-12)
    assert not torch.allclose(run({**w, p + "v_proj.weight": w[p + "v_proj.weight"] * 7.0}), base, rtol=1e-2)


def test_gate_goes_through_silu_and_up_does_not(tmp_path):
    """reference layers/activation.py:6-7: silu(first half) * second half, the first half being gate_proj's rows
    (layers/linear.py:29-45). So the feed-forward is linear in up_proj and not in gate_proj."""
    d = _folder(tmp_path, "B")
    cfg, w = P.read_model_folder(d, D64)
    p = "model.layers.0.mlp."
    x = torch.randn(9, cfg["hidden_size"], dtype=D64, generator=torch.Generator().manual_seed(3)) * 4
    base = P.mlp_block(w, p, x)
    assert torch.allclose(P.mlp_block({**w, p + "up_proj.weight": w[p + "up_proj.weight"] * 3.0}, p, x), base * 3.0, rtol=1e-12)
    gate3 = P.mlp_block({**w, p + "gate_proj.weight": w[p + "gate_proj.weight"] * 3.0}, p, x)
    assert not torch.allclose(gate3, base * 3.0, rtol=1e-2)
    # silu(z) -> z for large z: where every gate value is large and positive the block becomes gate * up
    big = {**w, p + "gate_proj.weight": torch.zeros_like(w[p + "gate_proj.weight"])}
    assert torch.equal(P.mlp_block(big, p, x), torch.zeros_like(base))            # silu(0) = 0, whatever up is


def test_layers_that_output_nothing_leave_the_norm_of_the_embedding(tmp_path):
    """reference models/qwen3.py:65-74,91: every layer adds its attention and feed-forward outputs to the
    residual stream, which starts as the embedding, and the final norm takes the last output plus the stream.
    With every o_proj and down_proj zero the logits are therefore head(rms_norm(embedding)): library routines
    only. (A final norm over the last layer's output alone would give zeros; a stream that did not start at the
    embedding would give something else.)"""
    d = _folder(tmp_path, "B")
    cfg, w = P.read_model_folder(d, D64)
    silent = {k: (torch.zeros_like(v) if k.endswith(("o_proj.weight", "down_proj.weight")) else v) for k, v in w.items()}
    ids = helpers.random_ids(17, cfg["vocab_size"], 8)
    h = F.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    want = F.linear(F.rms_norm(h, (h.shape[-1],), w["model.norm.weight"], cfg["rms_norm_eps"]), w["lm_head.weight"])
    assert torch.allclose(P.logits(cfg, silent, ids), want, atol=1e-12)
    # and with only the last feed-forward speaking, its output reaches the logits through the same norm
    last = f"model.layers.{cfg['num_hidden_layers'] - 1}.mlp.down_proj.weight"
    speaking = {**silent, last: w[last]}
    assert not torch.allclose(P.logits(cfg, speaking, ids), want, atol=1e-6)
