"""Typed model configurations read from a model folder's ``config.json``.

The reference hands the untyped ``transformers`` config object straight to the
model (reference ``config.py:25``, ``models/qwen3.py:15-23,81-84,107-108``).
Here every architecture has a frozen dataclass whose fields are exactly the
``config.json`` keys it uses; no size or constant of the model lives anywhere
else in the code.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, fields
from typing import Any, Callable


class ConfigError(ValueError):
    """A ``config.json`` that the engine cannot run, with the reason."""


_CONFIG_CLASSES: dict[str, type] = {}


def register_config(architecture: str) -> Callable[[type], type]:
    """Class decorator: ``architecture`` (as spelled in ``architectures[0]``) -> config class."""

    def deco(cls: type) -> type:
        _CONFIG_CLASSES[architecture] = cls
        cls.architecture_name = architecture
        return cls

    return deco


def config_class_for(architecture: str) -> type:
    try:
        return _CONFIG_CLASSES[architecture]
    except KeyError:
        known = ", ".join(sorted(_CONFIG_CLASSES)) or "<none>"
        raise ConfigError(
            f"unknown architecture {architecture!r}; registered architectures: {known}"
        ) from None


def read_config_json(model_dir: str) -> dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{model_dir!r} has no config.json")
    with open(path) as f:
        raw = json.load(f)
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return raw


def architecture_of(raw: dict[str, Any]) -> str:
    archs = raw.get("architectures")
    if not archs or not isinstance(archs, (list, tuple)) or not isinstance(archs[0], str):
        raise ConfigError("config.json must name the model class in 'architectures': [\"...\"]")
    return archs[0]


def load_model_config(model_dir: str):
    """Read ``config.json`` and build the typed config of the architecture it names."""
    raw = read_config_json(model_dir)
    return config_class_for(architecture_of(raw)).from_dict(raw)


def _need(raw: dict, key: str, kind, where: str = "config.json"):
    if key not in raw or raw[key] is None:
        raise ConfigError(f"{where} lacks the required key {key!r}")
    v = raw[key]
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"{where}: {key!r} must be an integer, got {v!r}")
    elif kind is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{where}: {key!r} must be a number, got {v!r}")
        v = float(v)
    return v


@register_config("Qwen3ForCausalLM")
@dataclass(frozen=True)
class Qwen3Config:
    """The ``config.json`` keys of a Qwen3 dense decoder.

    Keys the reference reads: ``models/qwen3.py:15-23`` (heads, head_dim, eps),
    ``:60-62`` (hidden/intermediate), ``:81-84`` (rope theta, positions, vocab,
    layers), ``:107-108`` (tying). ``head_dim`` is read directly, so the query
    width ``num_attention_heads * head_dim`` need not equal ``hidden_size``.

    Beyond the reference: ``sliding_window`` / ``layer_types`` are honoured when
    ``use_sliding_window`` is true (a query at position i then sees keys j with
    ``0 <= i - j < sliding_window`` in layers of type ``"sliding_attention"``);
    the reference ignores those keys and always attends to every earlier key.
    """

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool | None  # None: decided by whether the checkpoint stores lm_head.weight
    max_position_embeddings: int | None
    sliding_window: int | None
    layer_types: tuple[str, ...]
    eos_token_id: int | None = None

    LAYER_TYPES = ("full_attention", "sliding_attention")

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "Qwen3Config":
        hidden = _need(raw, "hidden_size", int)
        heads = _need(raw, "num_attention_heads", int)
        kv_heads = raw.get("num_key_value_heads")
        if kv_heads is None:
            kv_heads = heads
        head_dim = raw.get("head_dim")
        if head_dim is None:
            if hidden % heads:
                raise ConfigError("config.json has no 'head_dim' and hidden_size is not a multiple "
                                  "of num_attention_heads")
            head_dim = hidden // heads
        layers = _need(raw, "num_hidden_layers", int)

        # rope theta: transformers 5 nests it in rope_parameters (reference models/qwen3.py:81);
        # older config.json files carry it at the top level.
        rope = raw.get("rope_parameters") or {}
        scaling = raw.get("rope_scaling") or {}
        theta = rope.get("rope_theta", raw.get("rope_theta", scaling.get("rope_theta")))
        if theta is None:
            raise ConfigError("config.json lacks 'rope_theta' (top level or in 'rope_parameters')")
        for src in (rope, scaling):
            kind = src.get("rope_type", src.get("type", "default"))
            if kind not in (None, "default"):
                raise ConfigError(f"rope scaling of type {kind!r} is not supported (only plain rotary)")
        if raw.get("attention_bias"):
            raise ConfigError("attention_bias=true is not supported: Qwen3 dense has no biases")
        act = raw.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act={act!r} is not supported (the feed-forward is SiLU-gated)")

        window = raw.get("sliding_window") if raw.get("use_sliding_window") else None
        if window is not None:
            if isinstance(window, bool) or not isinstance(window, int) or window < 1:
                raise ConfigError(f"sliding_window must be a positive integer, got {window!r}")
            types = raw.get("layer_types")
            if types is None:
                first = raw.get("max_window_layers", layers)
                types = ["sliding_attention" if i >= first else "full_attention" for i in range(layers)]
        else:
            types = ["full_attention"] * layers
        types = tuple(types)
        if len(types) != layers or any(t not in cls.LAYER_TYPES for t in types):
            raise ConfigError(f"layer_types must hold {layers} entries from {cls.LAYER_TYPES}, got {types!r}")
        if "sliding_attention" not in types:
            window = None

        tie = raw.get("tie_word_embeddings")
        if tie is not None and not isinstance(tie, bool):
            raise ConfigError(f"tie_word_embeddings must be true or false, got {tie!r}")
        eos = raw.get("eos_token_id")
        if isinstance(eos, (list, tuple)):
            eos = eos[0] if eos else None
        cfg = cls(
            vocab_size=_need(raw, "vocab_size", int),
            hidden_size=hidden,
            intermediate_size=_need(raw, "intermediate_size", int),
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=int(kv_heads),
            head_dim=int(head_dim),
            rms_norm_eps=_need(raw, "rms_norm_eps", float),
            rope_theta=float(theta),
            tie_word_embeddings=tie,
            max_position_embeddings=raw.get("max_position_embeddings"),
            sliding_window=window,
            layer_types=types,
            eos_token_id=eos,
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for f in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                  "num_attention_heads", "num_key_value_heads", "head_dim"):
            v = getattr(self, f)
            if not isinstance(v, int) or isinstance(v, bool) or v < 1:
                raise ConfigError(f"{f} must be a positive integer, got {v!r}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads={self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads={self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim={self.head_dim} must be even for rotary pairs")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps!r}")
        if not self.rope_theta > 0:
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta!r}")

    def to_dict(self) -> dict[str, Any]:
        """A ``config.json`` that reads back to an equal config."""
        d: dict[str, Any] = {
            "architectures": [self.architecture_name],
            "model_type": "qwen3",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "hidden_act": "silu",
            "attention_bias": False,
        }
        if self.tie_word_embeddings is not None:
            d["tie_word_embeddings"] = self.tie_word_embeddings
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        if self.sliding_window is not None:
            d["use_sliding_window"] = True
            d["sliding_window"] = self.sliding_window
            d["layer_types"] = list(self.layer_types)
        else:
            d["use_sliding_window"] = False
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        return d

    def flat(self) -> dict[str, Any]:
        """Sizes as a flat dict (for benchmark records)."""
        return {f.name: getattr(self, f.name) for f in fields(self)
                if f.name not in ("layer_types",)}
