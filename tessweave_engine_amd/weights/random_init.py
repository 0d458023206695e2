"""Random-weights mode: a model folder (config.json, model.safetensors) from a configuration and a seed.

The reference has no such mode; its tests draw random weights by building a
library model under a fixed seed (tests/test_engine.py:15-25). Here every tensor
is drawn by NAME: its generator is seeded from (seed, tensor name), so a
tensor's values do not depend on which other tensors exist or on their order.
Linear, embedding and bias values are N(0, std); norm weights are 1 + N(0, std).
"""
from __future__ import annotations

import hashlib
import json
from pathlib import Path

import torch

from .spec import ONE_PLUS_NORMAL, TABLE
from .loader import device_dtype_for, resolve_dtype

DEFAULT_STD = 0.02


def _tensor_seed(seed, name):
    digest = hashlib.sha256(f"{int(seed)}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & ((1 << 63) - 1)


def draw_tensor(spec, seed, std=DEFAULT_STD, device="cpu", dtype=torch.float32):
    """One tensor of the random-weights mode, as float32 values rounded to DTYPE."""
    if spec.role == TABLE:
        raise ValueError(f"no random initialisation is defined for the integer table {spec.name}")
    generator = torch.Generator(device=device).manual_seed(_tensor_seed(seed, spec.name))
    t = torch.empty(spec.shape, dtype=torch.float32, device=device)
    t.normal_(0.0, std, generator=generator)
    if spec.init == ONE_PLUS_NORMAL:
        t += 1.0
    return t.to(dtype)


def random_tensors(specs, seed, std=DEFAULT_STD, store_dtype=torch.bfloat16, device="cpu"):
    return {s.name: draw_tensor(s, seed, std, device, store_dtype)
            for s in specs if s.optional_alias_of is None}


def write_model_folder(folder, config, seed, std=DEFAULT_STD, store_dtype="bfloat16", device="cpu"):
    """Write config.json and model.safetensors for CONFIG; returns the folder path.

    Values are rounded to STORE_DTYPE before writing, so a float32 run and a
    bfloat16 run of the same folder use the same weight values. DEVICE is where
    the values are drawn: a GPU draws billions of values in a moment, but its
    generator's stream is not the CPU's, so the same seed gives other values there.
    """
    from safetensors.torch import save_file
    from ..config import build_model

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    model = build_model(config)
    tensors = random_tensors(model.tensor_specs(), seed, std, resolve_dtype(store_dtype), device)
    (folder / "config.json").write_text(json.dumps(config.to_dict(), indent=2) + "\n")
    save_file({k: v.contiguous().cpu() for k, v in tensors.items()}, str(folder / "model.safetensors"))
    return folder


def random_model(config, seed, dtype="bfloat16", device="cuda", std=DEFAULT_STD):
    """A model with weights drawn on DEVICE, no files (benchmarks use this).

    The device generator's stream differs from the CPU's, so these values are
    not the ones `write_model_folder` writes for the same seed.
    """
    from ..config import build_model

    compute_dtype = resolve_dtype(dtype)
    device = torch.device(device)
    model = build_model(config)
    tensors = {}
    for spec in model.tensor_specs():
        if spec.optional_alias_of is not None:
            continue
        held = device_dtype_for(spec.role, torch.bfloat16, compute_dtype)
        tensors[spec.name] = draw_tensor(spec, seed, std, device, torch.bfloat16).to(held)
    model.bind(tensors, compute_dtype, device)
    return model
