"""Seeded random weights: fill a model directly, or write a model folder.

Distributions: matrices (linears, embeddings) ~ N(0, 0.02); norm weights (the per-head
q/k norms too) ~ 1 + U(-0.1, 0.1); a parameter may bring a function of its own (`ParamSpec.init`). Tensors are generated in float32 on the CPU, one
generator seeded once, in sorted order of their checkpoint names, so the values depend
only on (config, seed).
"""
from __future__ import annotations

import json
import os

import torch

from ..registry import build_model


def _checkpoint_tensor_specs(model) -> list:
    """Sorted (checkpoint name, shape, init kind) of every tensor the model loads."""
    specs = {name: spec for name, _, _, spec in model.named_specs()}
    out = {}
    for pname, sources in model.weight_sources.items():
        spec = specs[pname]
        for src in sources:
            rows = spec.shape[0] if src.rows is None else src.rows
            out[src.name] = ((rows,) + tuple(spec.shape[1:]), spec.init, spec.dtype)
    return sorted((n, s, k, d) for n, (s, k, d) in out.items())


def _draw(shape, kind, gen, device) -> torch.Tensor:
    if callable(kind):
        t = kind(tuple(shape), gen, device)
        if tuple(t.shape) != tuple(shape):
            raise ValueError(f"an init function returned shape {tuple(t.shape)} for a parameter of shape {tuple(shape)}")
        return t.to(torch.float32)
    if kind == "matrix":
        return torch.randn(shape, generator=gen, dtype=torch.float32, device=device) * 0.02
    if kind == "norm":
        return 1.0 + (torch.rand(shape, generator=gen, dtype=torch.float32, device=device) * 0.2 - 0.1)
    raise ValueError(f"unknown init kind {kind!r}")


def random_tensors(model, seed: int):
    """Yield (checkpoint name, float32 cpu tensor, dtype policy) in sorted name order."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(seed))
    for name, shape, kind, policy in _checkpoint_tensor_specs(model):
        yield name, _draw(shape, kind, gen, "cpu"), policy


def fill_random(model, seed: int, device, dtype: torch.dtype, max_positions: int, round_to=torch.bfloat16,
                on_device: bool = False):
    """Bind random weights without a folder. Values are first rounded to `round_to` (what a
    written folder would store) so both routes give the same model.

    on_device: every tensor is drawn where it will live, by a generator of that device seeded with
    (seed, the tensor's place in the sorted name order), one tensor at a time: no host copy of the
    model exists at any moment (a 32B model is 65 GB). The values then depend on (config, seed) and
    the kind of device, and differ from those of the host route."""
    from .loader import fill_model

    if on_device and torch.device(device).type != "cpu":
        specs = {name: (i, shape, kind) for i, (name, shape, kind, _) in enumerate(_checkpoint_tensor_specs(model))}
        gen = torch.Generator(device=device)

        def draw(name):
            i, shape, kind = specs[name]
            gen.manual_seed((int(seed) << 20) + i)
            t = _draw(shape, kind, gen, device)
            return t.to(round_to) if round_to is not None else t

        fill_model(model, draw, lambda n: round_to or torch.float32, device, dtype)
    else:
        store = {}
        for name, t, _ in random_tensors(model, seed):
            store[name] = t.to(round_to) if round_to is not None else t
        fill_model(model, store.__getitem__, lambda n: store[n].dtype, device, dtype)
    model.finalize_all(device, dtype, max_positions)
    return model


def write_random_model(model_config, seed: int, out_dir: str, store_dtype: torch.dtype = torch.bfloat16) -> str:
    """Write config.json and model.safetensors for `model_config` with seeded random weights."""
    from safetensors.torch import save_file

    os.makedirs(out_dir, exist_ok=True)
    model = build_model(model_config)
    tensors = {}
    for name, t, policy in random_tensors(model, seed):
        tensors[name] = t.to(torch.float32 if policy == "float32" and store_dtype == torch.float32 else store_dtype).contiguous()
    save_file(tensors, os.path.join(out_dir, "model.safetensors"), metadata={"format": "pt"})
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(model_config.to_dict(), f, indent=2)
    return out_dir
