"""Configuration, registry, weight loading and its errors, random-weights folders. No GPU."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

import helpers
from mini_engine_amd.config.engine_config import EngineConfig
from mini_engine_amd.config.model_config import ConfigError, Qwen3Config, load_model_config
from mini_engine_amd.registry import architectures, build_model, builder_for
from mini_engine_amd.weights.loader import WeightError, load_model
from mini_engine_amd.weights.random_init import write_random_model


def test_typed_config_reads_its_keys():
    c = Qwen3Config.from_dict(helpers.CONFIGS["B"])
    assert (c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (80, 6, 2, 32)
    assert c.num_attention_heads * c.head_dim != c.hidden_size          # q width need not equal hidden
    assert c.rope_theta == 1e6 and c.rms_norm_eps == 1e-5 and c.tie_word_embeddings is False
    assert c.layer_types == ("full_attention",) * 3 and c.sliding_window is None


def test_rope_theta_nested_or_top_level():
    d = dict(helpers.CONFIGS["A"])
    theta = d.pop("rope_theta")
    d["rope_parameters"] = {"rope_theta": theta, "rope_type": "default"}
    assert Qwen3Config.from_dict(d).rope_theta == theta
    d["rope_parameters"]["rope_type"] = "yarn"
    with pytest.raises(ConfigError, match="yarn"):
        Qwen3Config.from_dict(d)


def test_head_dim_defaults_to_hidden_over_heads_only_when_absent():
    d = dict(helpers.CONFIGS["A"])
    del d["head_dim"]
    assert Qwen3Config.from_dict(d).head_dim == 16


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads", "rms_norm_eps", "rope_theta"])
def test_required_keys(key):
    d = dict(helpers.CONFIGS["A"])
    del d[key]
    with pytest.raises(ConfigError, match=key):
        Qwen3Config.from_dict(d)


def test_rejects_what_the_model_cannot_do():
    for patch, word in ((dict(attention_bias=True), "bias"), (dict(hidden_act="gelu"), "hidden_act"),
                        (dict(num_key_value_heads=3), "multiple"), (dict(head_dim=15), "even")):
        with pytest.raises(ConfigError, match=word):
            Qwen3Config.from_dict(dict(helpers.CONFIGS["A"], **patch))


def test_window_keys():
    c = Qwen3Config.from_dict(helpers.CONFIGS["C"])
    assert c.sliding_window == 24 and c.layer_types[1] == "sliding_attention"
    # use_sliding_window false: the window key is ignored
    d = dict(helpers.CONFIGS["C"], use_sliding_window=False)
    assert Qwen3Config.from_dict(d).sliding_window is None
    # max_window_layers gives the layer types when they are not listed
    d = dict(helpers.CONFIGS["C"]); del d["layer_types"]; d["max_window_layers"] = 3
    assert Qwen3Config.from_dict(d).layer_types == ("full_attention",) * 3 + ("sliding_attention",)
    # round trip through config.json
    assert Qwen3Config.from_dict(c.to_dict()) == c


def test_registry(tmp_path):
    assert "Qwen3ForCausalLM" in architectures()
    with pytest.raises(ConfigError, match="NoSuchLM"):
        builder_for("NoSuchLM")
    d = tmp_path / "m"; d.mkdir()
    (d / "config.json").write_text(json.dumps(dict(helpers.CONFIGS["A"], architectures=["NoSuchLM"])))
    with pytest.raises(ConfigError, match="NoSuchLM"):
        load_model_config(str(d))
    (d / "config.json").write_text(json.dumps({k: v for k, v in helpers.CONFIGS["A"].items() if k != "architectures"}))
    with pytest.raises(ConfigError, match="architectures"):
        load_model_config(str(d))


def test_engine_config_checks(folders):
    d = folders("A")
    c = EngineConfig(d, max_model_len=10 ** 6)
    assert c.max_model_len == 4096                       # clamped to max_position_embeddings
    assert isinstance(c.model_config, Qwen3Config)
    for kw in (dict(max_num_seqs=64, max_num_batched_tokens=32), dict(scheduling_policy="lifo"),
               dict(long_prefill_token_threshold=-1), dict(gpu_memory_utilization=0.0), dict(dtype="float16"),
               dict(enable_chunked_prefill=False, max_num_batched_tokens=512, max_model_len=1024)):
        with pytest.raises(ConfigError):
            EngineConfig(d, **kw)
    with pytest.raises(ConfigError):
        EngineConfig(d + "_missing")


def test_random_folder_is_deterministic_and_loads(tmp_path):
    cfg = Qwen3Config.from_dict(helpers.CONFIGS["B"])
    a = load_file(os.path.join(write_random_model(cfg, 7, str(tmp_path / "a")), "model.safetensors"))
    b = load_file(os.path.join(write_random_model(cfg, 7, str(tmp_path / "b")), "model.safetensors"))
    c = load_file(os.path.join(write_random_model(cfg, 8, str(tmp_path / "c")), "model.safetensors"))
    assert a.keys() == b.keys() and all(torch.equal(a[k], b[k]) for k in a)
    assert any(not torch.equal(a[k], c[k]) for k in a)
    assert all(v.dtype == torch.bfloat16 for v in a.values())
    names = set(a)
    assert "lm_head.weight" in names and "model.layers.2.self_attn.q_norm.weight" in names
    assert abs(float(a["model.layers.0.mlp.up_proj.weight"].float().std()) - 0.02) < 0.002
    nw = a["model.layers.1.self_attn.k_norm.weight"].float()
    assert 0.89 <= float(nw.min()) and float(nw.max()) <= 1.11
    assert load_model_config(str(tmp_path / "a")) == cfg


def test_loader_packs_and_keeps_dtypes(folders):
    d = folders("B")
    m = load_model(d, "cpu", torch.bfloat16, 64)
    raw = load_file(os.path.join(d, "model.safetensors"))
    qkv = m.layers[1].mixer.qkv.weight
    assert qkv.dtype == torch.bfloat16 and qkv.shape == (6 * 32 + 2 * 2 * 32, 80)
    p = "model.layers.1.self_attn."
    assert torch.equal(qkv, torch.cat([raw[p + "q_proj.weight"], raw[p + "k_proj.weight"], raw[p + "v_proj.weight"]]))
    gu = m.layers[0].feed_forward.gate_up.weight
    assert torch.equal(gu, torch.cat([raw["model.layers.0.mlp.gate_proj.weight"], raw["model.layers.0.mlp.up_proj.weight"]]))
    assert m.layers[0].norm1.weight.dtype == torch.float32            # norm weights are held in 32-bit
    assert torch.equal(m.layers[0].norm1.weight, raw["model.layers.0.input_layernorm.weight"].float())
    assert m.head.matrix() is not m.embedding.weight
    m32 = load_model(d, "cpu", torch.float32, 64)
    assert m32.layers[1].mixer.qkv.weight.dtype == torch.float32
    assert torch.equal(m32.layers[1].mixer.qkv.weight, qkv.float())


def test_tied_head_is_the_same_tensor(folders, tmp_path):
    m = load_model(folders("A"), "cpu", torch.bfloat16, 64)
    assert m.head.matrix() is m.embedding.weight
    # a stored lm_head.weight is ignored when tied (reference utils/loader.py:23-24)
    raw = load_file(os.path.join(folders("A"), "model.safetensors"))
    raw["lm_head.weight"] = torch.zeros_like(raw["model.embed_tokens.weight"])
    d = tmp_path / "tied"; d.mkdir()
    save_file(raw, str(d / "model.safetensors"))
    (d / "config.json").write_text(json.dumps(helpers.CONFIGS["A"]))
    m2 = load_model(str(d), "cpu", torch.bfloat16, 64)
    assert m2.head.matrix() is m2.embedding.weight
    # without the key, tying follows whether the checkpoint stores a head
    cfgd = {k: v for k, v in helpers.CONFIGS["A"].items() if k != "tie_word_embeddings"}
    (d / "config.json").write_text(json.dumps(cfgd))
    assert load_model(str(d), "cpu", torch.bfloat16, 64).head.matrix() is not m2.embedding.weight


def test_one_error_lists_missing_unexpected_and_wrong_shapes(folders, tmp_path):
    raw = load_file(os.path.join(folders("B"), "model.safetensors"))
    del raw["model.layers.0.self_attn.k_proj.weight"]
    del raw["model.norm.weight"]
    raw["model.layers.9.mlp.up_proj.weight"] = torch.zeros(3, 3)
    raw["model.layers.1.mlp.down_proj.weight"] = torch.zeros(80, 200, dtype=torch.bfloat16)
    d = tmp_path / "bad"; d.mkdir()
    save_file(raw, str(d / "model.safetensors"))
    (d / "config.json").write_text(json.dumps(helpers.CONFIGS["B"]))
    with pytest.raises(WeightError) as ei:
        load_model(str(d), "cpu", torch.bfloat16, 64)
    msg = str(ei.value)
    assert "missing tensors (2)" in msg and "model.layers.0.self_attn.k_proj.weight" in msg and "model.norm.weight" in msg
    assert "unexpected tensors (1)" in msg and "model.layers.9.mlp.up_proj.weight" in msg
    assert "wrong shapes (1)" in msg and "model.layers.1.mlp.down_proj.weight" in msg and "[80, 224]" in msg
    empty = tmp_path / "empty"; empty.mkdir()
    (empty / "config.json").write_text(json.dumps(helpers.CONFIGS["B"]))
    with pytest.raises(WeightError, match="no .safetensors"):
        load_model(str(empty), "cpu", torch.bfloat16, 64)


def test_float32_checkpoint_keeps_32_bit_norms(tmp_path):
    d = helpers.make_folder("A", str(tmp_path / "f32"), torch.float32)
    raw = load_file(os.path.join(d, "model.safetensors"))
    assert all(v.dtype == torch.float32 for v in raw.values())
    m = load_model(d, "cpu", torch.bfloat16, 64)
    # 32-bit norm weights are not rounded to bfloat16 on the way in
    assert torch.equal(m.final_norm.weight, raw["model.norm.weight"])
    assert m.embedding.weight.dtype == torch.bfloat16
