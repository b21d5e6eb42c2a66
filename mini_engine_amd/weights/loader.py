"""Weights from safetensors, by tensor name (reference utils/loader.py:8-38).

The model names, for every parameter, the checkpoint tensors whose rows it is made
of (packed projections: reference models/qwen3.py:96-102, layers/linear.py:13-22,37-42).
The whole checkpoint is checked against that list before anything is copied, and all
problems are reported in one error: missing tensors, unexpected tensors, wrong shapes.

Storage: matrices in the compute dtype (bfloat16, or float32 on the 32-bit path);
parameters a part declares as "float32" stay 32-bit (norm weights: exact for both
stored forms); "int32" for integer tables; "stored" keeps what the file holds
(bfloat16 stays bfloat16, 32-bit stays 32-bit).
"""
from __future__ import annotations

import os
from glob import glob

import torch

from ..config.model_config import load_model_config
from ..registry import build_model


class WeightError(ValueError):
    """The checkpoint does not fit the model; the message lists every mismatch."""


def checkpoint_files(model_dir: str) -> list:
    files = sorted(glob(os.path.join(model_dir, "*.safetensors")))
    if not files:
        raise WeightError(f"no .safetensors files in {model_dir!r}")
    return files


def checkpoint_index(model_dir: str) -> dict:
    """tensor name -> (file, shape tuple, dtype string) without reading any data."""
    from safetensors import safe_open

    index = {}
    for file in checkpoint_files(model_dir):
        with safe_open(file, "pt", device="cpu") as f:
            for name in f.keys():
                sl = f.get_slice(name)
                index[name] = (file, tuple(sl.get_shape()), str(sl.get_dtype()))
    return index


def _target_dtype(spec_dtype: str, compute: torch.dtype, stored: torch.dtype) -> torch.dtype:
    if spec_dtype == "compute":
        return compute
    if spec_dtype == "float32":
        return torch.float32
    if spec_dtype == "int32":
        return torch.int32
    if spec_dtype == "stored":
        if stored in (torch.float32, torch.float64):
            return torch.float32
        if not stored.is_floating_point:
            return torch.int32
        return torch.bfloat16
    raise ValueError(f"unknown parameter dtype policy {spec_dtype!r}")


def check_checkpoint(model, index: dict) -> None:
    """Raise one WeightError listing missing, unexpected and misshapen tensors."""
    missing, wrong, used = [], [], set()
    specs = {name: spec for name, _, _, spec in model.named_specs()}
    unmapped = sorted(set(specs) - set(model.weight_sources))
    if unmapped:
        raise WeightError(f"the model does not say where these parameters are stored: {unmapped}")
    for pname, sources in model.weight_sources.items():
        spec = specs.get(pname)
        if spec is None:
            raise WeightError(f"weight source given for {pname!r}, which is not a parameter of the model")
        for src in sources:
            rows = spec.shape[0] if src.rows is None else src.rows
            expect = (rows,) + tuple(spec.shape[1:])
            if src.name not in index:
                missing.append(f"{src.name} {list(expect)}")
                continue
            used.add(src.name)
            got = index[src.name][1]
            if tuple(got) != expect:
                wrong.append(f"{src.name}: stored {list(got)}, model needs {list(expect)}")
    unexpected = sorted(set(index) - used - set(model.optional_sources))
    if missing or wrong or unexpected:
        lines = ["checkpoint does not fit the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + "; ".join(sorted(missing)))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + "; ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shapes ({len(wrong)}): " + "; ".join(sorted(wrong)))
        raise WeightError("\n".join(lines))


def fill_model(model, get_tensor, stored_dtype, device, dtype: torch.dtype) -> None:
    """Bind every parameter from `get_tensor(checkpoint name) -> cpu tensor`."""
    owners = {name: (part, local, spec) for name, part, local, spec in model.named_specs()}
    for pname, sources in model.weight_sources.items():
        part, local, spec = owners[pname]
        target = _target_dtype(spec.dtype, dtype, stored_dtype(sources[0].name))
        if len(sources) == 1 and sources[0].rows is None:
            param = get_tensor(sources[0].name).to(device=device, dtype=target).contiguous()
        else:
            param = torch.empty(spec.shape, dtype=target, device=device)
            for src in sources:
                rows = spec.shape[0] if src.rows is None else src.rows
                param.narrow(0, src.row_start, rows).copy_(get_tensor(src.name))
        part.set_param(local, param)


_ST_DTYPES = {"F32": torch.float32, "F64": torch.float64, "BF16": torch.bfloat16, "F16": torch.float16,
              "I32": torch.int32, "I64": torch.int64, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
              "BOOL": torch.bool}


def load_weights(model, model_dir: str, device, dtype: torch.dtype, index: dict | None = None) -> None:
    from safetensors import safe_open

    index = index or checkpoint_index(model_dir)
    check_checkpoint(model, index)
    handles: dict = {}
    try:
        def get(name):
            file = index[name][0]
            if file not in handles:
                handles[file] = safe_open(file, "pt", device="cpu")
            return handles[file].get_tensor(name)

        def stored(name):
            return _ST_DTYPES.get(index[name][2].upper().replace("TORCH.", ""), torch.bfloat16)

        fill_model(model, get, stored, device, dtype)
    finally:
        handles.clear()


def load_model(model_dir: str, device, dtype: torch.dtype, max_positions: int, model_config=None,
               random_weights: int | None = None):
    """config.json -> registry -> model -> weights -> finalize. Returns the ready model.
    `random_weights` (a seed): no checkpoint is read, every tensor is drawn on the device."""
    cfg = model_config or load_model_config(model_dir)
    if random_weights is not None:
        from .random_init import fill_random
        return fill_random(build_model(cfg), random_weights, device, dtype, max_positions, on_device=True)
    index = checkpoint_index(model_dir)
    model = build_model(cfg, checkpoint_names=set(index))
    load_weights(model, model_dir, device, dtype, index)
    model.finalize_all(device, dtype, max_positions)
    return model
