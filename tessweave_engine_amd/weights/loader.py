"""Weights from safetensors by tensor name.

Reference behaviour followed (flow_engine/model.py:114-159): the shard list is
the sorted unique `weight_map` values of model.safetensors.index.json, else the
single model.safetensors; shard names must be bare `*.safetensors` file names;
a tied `lm_head.weight` and any `*rotary_emb.inv_freq` are skipped; unknown,
duplicate, wrongly shaped and missing tensors are errors.

Differences: every problem of a checkpoint is collected into ONE `WeightError`
that lists missing and unexpected tensors and wrong shapes, instead of raising
at the first; tensors go to the device one by one and each part packs its own
(q,k,v rows into one matrix; gate,up rows into one) there.
"""
from __future__ import annotations

import json
from pathlib import Path

import torch

from .spec import MATRIX, VECTOR, TABLE

_TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


class WeightError(ValueError):
    """The checkpoint does not hold exactly the tensors the model needs."""

    def __init__(self, missing=(), unexpected=(), wrong_shape=(), duplicate=(), other=()):
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.wrong_shape = sorted(wrong_shape)        # (name, found, expected)
        self.duplicate = sorted(duplicate)
        self.other = list(other)
        lines = ["checkpoint does not match the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.duplicate:
            lines.append(f"  duplicate ({len(self.duplicate)}): " + ", ".join(self.duplicate))
        for name, found, expected in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(found)}, expected {list(expected)}")
        lines.extend(f"  {text}" for text in self.other)
        super().__init__("\n".join(lines))


def resolve_dtype(dtype):
    if isinstance(dtype, torch.dtype):
        if dtype not in _TORCH_DTYPES.values():
            raise ValueError("dtype must be bfloat16 or float32")
        return dtype
    if dtype not in _TORCH_DTYPES:
        raise ValueError("dtype must be bfloat16 or float32")
    return _TORCH_DTYPES[dtype]


def device_dtype_for(role, stored_dtype, compute_dtype):
    """The precision a tensor of ROLE is held in on the device."""
    if role == TABLE:
        return torch.int32
    if role == VECTOR:
        return torch.float32
    if role == MATRIX:
        return compute_dtype
    raise ValueError(f"unknown tensor role {role!r}")


def shard_names(folder):
    folder = Path(folder)
    index = folder / "model.safetensors.index.json"
    if index.exists():
        names = sorted(set(json.loads(index.read_text())["weight_map"].values()))
    else:
        names = ["model.safetensors"]
    for name in names:
        if Path(name).name != name or not name.endswith(".safetensors"):
            raise WeightError(other=[f"unsafe or unsupported shard file name: {name!r}"])
    return names


def _skipped(key):
    return key.endswith("rotary_emb.inv_freq")


def read_tensors(folder, specs, compute_dtype, device):
    """Read exactly the tensors SPECS names; returns {name: device tensor}.

    Aliases (a tied head's own key) are accepted and skipped, never required.
    """
    from safetensors import safe_open

    folder = Path(folder)
    compute_dtype = resolve_dtype(compute_dtype)
    required = {s.name: s for s in specs if s.optional_alias_of is None}
    aliases = {s.name for s in specs if s.optional_alias_of is not None}
    found, unexpected, duplicate, wrong = {}, [], [], []
    names = shard_names(folder)
    for name in names:
        path = folder / name
        if not path.exists():
            raise WeightError(other=[f"shard {name} does not exist in {folder}"])
        with safe_open(str(path), framework="pt", device="cpu") as shard:
            for key in shard.keys():
                if key in aliases or _skipped(key):
                    continue
                if key not in required:
                    unexpected.append(key)
                    continue
                if key in found:
                    duplicate.append(key)
                    continue
                spec = required[key]
                shape = tuple(shard.get_slice(key).get_shape())
                if shape != spec.shape:
                    wrong.append((key, shape, spec.shape))
                    found[key] = None
                    continue
                found[key] = (name, key)
    missing = [k for k in required if k not in found]
    if missing or unexpected or duplicate or wrong:
        raise WeightError(missing, unexpected, wrong, duplicate)
    tensors = {}
    by_shard = {}
    for key, (name, _) in found.items():
        by_shard.setdefault(name, []).append(key)
    for name, keys in by_shard.items():
        with safe_open(str(folder / name), framework="pt", device="cpu") as shard:
            for key in keys:
                spec = required[key]
                t = shard.get_tensor(key)
                if spec.role == TABLE:
                    if t.dtype.is_floating_point:
                        raise WeightError(other=[f"{key} must hold integers, found {t.dtype}"])
                elif not t.dtype.is_floating_point:
                    raise WeightError(other=[f"{key} must hold floating point values, found {t.dtype}"])
                tensors[key] = t.to(device=device, dtype=device_dtype_for(spec.role, t.dtype, compute_dtype))
    return tensors


def load_model(folder, dtype="bfloat16", device="cuda", **build_options):
    """Model of FOLDER (config.json picks the class) with its weights on DEVICE."""
    from ..config import read_model_config, build_model

    folder = Path(folder).resolve(strict=True)
    config = read_model_config(folder)
    model = build_model(config, **build_options)
    compute_dtype = resolve_dtype(dtype)
    tensors = read_tensors(folder, model.tensor_specs(), compute_dtype, device)
    model.bind(tensors, compute_dtype, torch.device(device))
    return model
