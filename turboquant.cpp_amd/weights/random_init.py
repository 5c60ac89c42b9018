"""Random weights: a model folder (config.json, model.safetensors) from a configuration and a seed.

The reference has no such mode; its tests fill in-memory structs with ``std::mt19937(42)`` and
``normal(0, 0.1)``, norm weights 1.0 (/root/reference/tests/test_ops.cpp:797-826,908-937).  Here every
element of every checkpoint tensor is a function of (seed, position of the tensor in the model's table,
index of the element) alone, so a tensor can be made in pieces, in any order, on the host or on the device,
and comes out the same: a model drawn in the memory of the GPU has the values of the folder written for the
same configuration and seed, and nothing the size of the model is ever held on the host.

The generator: ``key = splitmix64(seed * 2^32 + tensor)``, the two 64-bit words of element ``i`` are the
splitmix64 outputs number ``2 i`` and ``2 i + 1`` of the stream that starts at ``key``, their upper 53 bits give
``u1`` in (0, 1] and ``u2`` in [0, 1), and the value is the Box-Muller normal ``sqrt(-2 ln u1) cos(2 pi u2)``
in float64, scaled and rounded to the tensor's type.  Integer steps are exact everywhere; the logarithm and the
cosine are the math library's, so host and device agree as far as those two agree in float64, which after
rounding to 32 or 16 bits is bit for bit but for about one element in 2^29.  Matrices, biases and embedding
tables are N(0, std); norm weights are 1 or N(1, norm_std).
"""
from __future__ import annotations

import json
import math
import os

import torch

from .safetensors_io import SafetensorsWriter

_FILE_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}
_GAMMA = 0x9E3779B97F4A7C15
_CHUNK = {"cpu": 1 << 22, "cuda": 1 << 27}      # elements drawn at a time: bounds the 64-bit temporaries


def _signed(v: int) -> int:
    v &= (1 << 64) - 1
    return v - (1 << 64) if v >= (1 << 63) else v


def _shr(x: torch.Tensor, n: int) -> torch.Tensor:
    """Logical right shift of 64-bit words kept in int64."""
    return (x >> n) & ((1 << (64 - n)) - 1)


def splitmix64_mix(z: torch.Tensor) -> torch.Tensor:
    """The output function of splitmix64 on int64 tensors holding 64-bit words (products wrap)."""
    z = (z ^ _shr(z, 30)) * _signed(0xBF58476D1CE4E5B9)
    z = (z ^ _shr(z, 27)) * _signed(0x94D049BB133111EB)
    return z ^ _shr(z, 31)


def splitmix64(state: int, n: int) -> int:
    """Output number ``n`` (from 0) of the splitmix64 stream that starts at ``state``, as a Python integer."""
    z = (state + (n + 1) * _GAMMA) & ((1 << 64) - 1)
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & ((1 << 64) - 1)
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & ((1 << 64) - 1)
    return z ^ (z >> 31)


def tensor_key(seed: int, index: int) -> int:
    return splitmix64(((seed & 0xFFFFFFFF) << 32) + index, 0)


def standard_normal(key: int, first: int, count: int, device="cpu") -> torch.Tensor:
    """Elements ``first .. first+count-1`` of the stream of ``key`` as float64 N(0, 1)."""
    i = torch.arange(first, first + count, dtype=torch.int64, device=device)
    base = i * _signed(2 * _GAMMA) + _signed(key + _GAMMA)           # state of output 2 i
    x1 = splitmix64_mix(base)
    x2 = splitmix64_mix(base + _signed(_GAMMA))
    u1 = (_shr(x1, 11) + 1).to(torch.float64) * (2.0 ** -53)
    u2 = _shr(x2, 11).to(torch.float64) * (2.0 ** -53)
    return torch.sqrt(-2.0 * torch.log(u1)) * torch.cos((2.0 * math.pi) * u2)


def random_tensor(index: int, shape, role: str, seed: int, std: float, norm_std: float, dtype: torch.dtype,
                  device="cpu") -> torch.Tensor:
    """The tensor at place ``index`` of a model's table, made on ``device``."""
    numel = 1
    for d in shape:
        numel *= int(d)
    scale, shift = (norm_std, 1.0) if role == "scale" else (std, 0.0)
    out = torch.empty(numel, dtype=dtype, device=device)
    if scale == 0.0:
        out.fill_(shift)
        return out.view(tuple(shape))
    key = tensor_key(seed, index)
    chunk = _CHUNK[torch.device(device).type]
    for first in range(0, numel, chunk):
        n = min(chunk, numel - first)
        v = standard_normal(key, first, n, device) * scale
        if shift:
            v += shift
        out[first:first + n] = v.to(torch.float32).to(dtype)
    return out.view(tuple(shape))


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
