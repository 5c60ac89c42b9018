"""Random weights: a model folder (config.json, model.safetensors) from a configuration and a seed.

The reference has no such mode; its tests fill in-memory structs with ``std::mt19937(42)`` and
``normal(0, 0.1)``, norm weights 1.0 (/root/reference/tests/test_ops.cpp:797-826,908-937).  Here every
checkpoint tensor the model reads is drawn from its own generator, seeded by (seed, position of the
tensor in the model's table), so tensors can be made one at a time and in any order: matrices, biases and
embedding tables from N(0, std), norm weights 1 or N(1, norm_std).
"""
from __future__ import annotations

import json
import os

import torch

from .safetensors_io import SafetensorsWriter

_FILE_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def random_tensor(index: int, shape, role: str, seed: int, std: float, norm_std: float, dtype: torch.dtype,
                  device="cpu") -> torch.Tensor:
    gen = torch.Generator(device=device)
    gen.manual_seed((seed * 1000003 + index * 7919 + 12345) % (2 ** 63))
    if role == "scale":
        t = torch.ones(shape, dtype=torch.float32, device=device)
        if norm_std > 0:
            t += norm_std * torch.randn(shape, generator=gen, dtype=torch.float32, device=device)
    else:
        t = std * torch.randn(shape, generator=gen, dtype=torch.float32, device=device)
    return t.to(dtype)


def random_tensors(table: dict, seed: int, std: float = 0.02, norm_std: float = 0.0,
                   dtype: torch.dtype = torch.bfloat16, device="cpu"):
    """Yields (name, tensor) for every entry of ``table`` (name -> (shape, role)), in the table's order."""
    for i, (name, (shape, role)) in enumerate(table.items()):
        yield name, random_tensor(i, shape, role, seed, std, norm_std, dtype, device)


def write_random_model(model_dir: str, config_json: dict, table: dict, seed: int, std: float = 0.02,
                       norm_std: float = 0.0, dtype: str = "bfloat16") -> str:
    """Writes ``config.json`` and ``model.safetensors`` into ``model_dir``; returns the folder."""
    os.makedirs(model_dir, exist_ok=True)
    tdtype = _FILE_DTYPES[dtype]
    cfg = dict(config_json)
    cfg["torch_dtype"] = dtype
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=2)
    decl = [(n, tuple(shape), tdtype) for n, (shape, _role) in table.items()]
    with SafetensorsWriter(os.path.join(model_dir, "model.safetensors"), decl,
                           metadata={"format": "pt", "seed": seed, "std": std, "norm_std": norm_std}) as w:
        for name, t in random_tensors(table, seed, std, norm_std, tdtype):
            w.append(name, t)
    return model_dir
