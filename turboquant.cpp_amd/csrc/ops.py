"""Python face of the HIP kernels: one function per kernel, on torch tensors that live on the GPU.

Every function checks on the host that shapes, types and strides are what its kernel and launch
grid assume before anything is launched, and raises :class:`KernelError` with the kernel's name
otherwise.  There is no other implementation behind these functions: without a GPU, or without
the compiled library, they raise.
"""
from __future__ import annotations

import ctypes
import dataclasses
import math
import os
import re

import torch

from . import build as _build


class KernelError(RuntimeError):
    pass


ACT_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# activations of the gate in a gated pair of products: the lines of gates.def, numbered as the kernels number them
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "gates.def"), encoding="utf-8") as _f:
    GATES = {name: i for i, name in enumerate(re.findall(r"^TQ_GATE\((\w+),", _f.read(), re.M))}
_WTYPE = {torch.float32: 0, torch.bfloat16: 1}
_LIBS: dict[str, ctypes.CDLL] = {}

_c_int, _c_i64, _c_f32, _c_ptr = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p

_SIGNATURES = {
    "tq_embed": [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_f32, _c_ptr],
    "tq_softcap": [_c_ptr, _c_i64, _c_f32, _c_ptr],
    "tq_move_rows": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_int, _c_ptr],
    "tq_gated_act": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "tq_head_rmsnorm": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_f32, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "tq_add_rmsnorm": [_c_ptr, _c_ptr, _c_int, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_f32,
                       _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr],
    "tq_rope_kv_write": [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr,
                         _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                         _c_ptr],
    "tq_moe_combine": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_i64, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr],
    "tq_gemm_generic": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_int,
                        _c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "tq_attention_generic": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_i64, _c_int, _c_int,
                             _c_int, _c_int, _c_int, _c_f32, _c_ptr, _c_ptr],
    "tq_router_topk": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                       _c_ptr],
    "tq_moe_align": [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "tq_route": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                 _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr],
    "tq_argmax": [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr],
    "tq_nll": [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr],
    "tq_probs_half": [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "tq_rep_penalty": [_c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_ptr, _c_f32, _c_ptr],
    "tq_sample_topp_scratch": [_c_int],
    "tq_sample_topp": [_c_ptr, _c_int, _c_int, _c_f32, _c_f32, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
}
# entry points that only one of the two libraries has
_OPTIONAL = {
    "tq_gemm_f32": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_int,
                    _c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_ptr],
    "tq_gemm_f32_runs": [_c_int, _c_int, _c_int, _c_int],
    "tq_attention_f32_scratch": [_c_int, _c_int, _c_int, _c_int],
    "tq_attention_f32": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_int, _c_int,
                         _c_int, _c_int, _c_int, _c_f32, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "tq_gemm_mfma": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_int,
                     _c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "tq_gemm_mfma_splits": [_c_int, _c_int, _c_int],
    "tq_gemm_mfma_pair_splits": [_c_int, _c_int, _c_int, _c_int, _c_int, _c_int],
    "tq_gemm_mfma_pair": [_c_ptr, _c_ptr, _c_int, _c_ptr],
    "tq_qkv_rope_write": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr,
                          _c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_ptr],
    "tq_probe_stream": [_c_ptr, _c_i64, _c_int, ctypes.c_uint, _c_ptr, _c_ptr],
    "tq_probe_mfma": [_c_int, _c_int, _c_int, ctypes.c_uint, _c_ptr, _c_ptr],
    "tq_attention_decode_scratch": [_c_int, _c_int, _c_int, _c_int],
    "tq_attention_mfma": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_int, _c_int,
                          _c_int, _c_int, _c_int, _c_f32, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
}


def dtype_name(dtype) -> str:
    if isinstance(dtype, str):
        if dtype in ("float32", "f32", "fp32"):
            return "float32"
        if dtype in ("bfloat16", "bf16"):
            return "bfloat16"
    elif dtype == torch.float32:
        return "float32"
    elif dtype == torch.bfloat16:
        return "bfloat16"
    raise KernelError(f"no kernels for activation type {dtype!r}: float32 and bfloat16 are built")


def library(dtype) -> ctypes.CDLL:
    """The compiled kernels for one activation type; builds them at the first call if they are not there."""
    name = dtype_name(dtype)
    lib = _LIBS.get(name)
    if lib is not None:
        return lib
    if not torch.cuda.is_available():
        raise KernelError("no GPU is visible: the kernels of this library run on gfx950 only and have no CPU form")
    path = _build.find_library(name) or _build.build(name)
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:
        raise KernelError(f"cannot load the kernel library {path}: {e}") from e
    for fn, sig in _SIGNATURES.items():
        f = getattr(lib, fn)
        f.argtypes, f.restype = sig, _c_int
    for fn, sig in _OPTIONAL.items():
        if hasattr(lib, fn):
            f = getattr(lib, fn)
            f.argtypes, f.restype = sig, _c_int
    lib.tq_sample_topp_scratch.restype = _c_i64
    for fn in ("tq_attention_decode_scratch", "tq_attention_f32_scratch"):
        if hasattr(lib, fn):
            getattr(lib, fn).restype = _c_i64
    _LIBS[name] = lib
    return lib


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None) or (lambda dev: torch.cuda.current_stream(dev).cuda_stream)


def has_kernel(dtype, name: str) -> bool:
    return hasattr(library(dtype), name)


def _stream() -> int:
    """The current stream's handle (the raw call: building a stream object for every launch cost 5 us of the host's
    time, a fifth of what a launch took)."""
    return _raw_stream(torch.cuda.current_device())


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _need(cond: bool, kernel: str, what) -> None:
    """``what``: the message, or a function that makes it (so that a check that holds formats nothing)."""
    if not cond:
        raise KernelError(f"{kernel}: {what() if callable(what) else what}")


def _check(t: torch.Tensor, kernel: str, name: str, dtype=None, shape=None) -> None:
    if not (isinstance(t, torch.Tensor) and t.is_cuda):
        raise KernelError(f"{kernel}: {name} must be a GPU tensor")
    if not t.is_contiguous():
        raise KernelError(f"{kernel}: {name} must be contiguous, has strides {t.stride()}")
    if dtype is not None and not (t.dtype in dtype if type(dtype) in (tuple, list) else t.dtype == dtype):
        raise KernelError(f"{kernel}: {name} must be {dtype}, is {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{kernel}: {name} must have shape {tuple(shape)}, has {tuple(t.shape)}")


# Timing by kind of work, as the reference's --profile has it (/root/reference/src/engine/tq_transformer.c:60-93,
# :2995-3020: matmul, moe, attn and the rest): while a profile is open, an event is recorded behind every launch, and
# the time between two events is put down to the kernel between them (the step must run on one stream).
_PROFILE: list | None = None
_KIND = {"gemm": "matmul", "gemm_mfma": "matmul", "gemm_f32": "matmul", "gemm_pair": "matmul", "qkv_rope_write": "matmul",
         "gated_act": "matmul", "attention": "attn", "attention_mfma": "attn", "attention_f32": "attn",
         "router_topk": "moe", "route": "moe", "moe_align": "moe", "moe_combine": "moe"}


def profile_begin() -> None:
    global _PROFILE
    e = torch.cuda.Event(enable_timing=True)
    e.record()
    _PROFILE = [(None, e)]


def profile_end() -> dict:
    """Milliseconds per kind since ``profile_begin`` ("matmul", "moe", "attn", "other"), "total", and "kernels":
    name -> [launches, milliseconds]."""
    global _PROFILE
    marks, _PROFILE = _PROFILE or [], None
    torch.cuda.synchronize()
    out = {"matmul": 0.0, "moe": 0.0, "attn": 0.0, "other": 0.0}
    kernels: dict[str, list] = {}
    for (_, before), ((kind, name), after) in zip(marks, marks[1:]):
        ms = before.elapsed_time(after)
        out[kind] += ms
        row = kernels.setdefault(name, [0, 0.0])
        row[0] += 1
        row[1] += ms
    out["total"] = sum(out.values())
    out["kernels"] = kernels
    return out


def _mark(kind: str, name: str = "vendor product") -> None:
    e = torch.cuda.Event(enable_timing=True)
    e.record()
    _PROFILE.append(((kind, name), e))


def _run(kernel: str, code: int, kind: str | None = None) -> None:
    if code == 0:
        if _PROFILE is not None:
            kind = kind or _KIND.get(kernel, "other")
            _mark(kind, kernel + (" (experts)" if kind == "moe" and kernel.startswith("gemm") else ""))
        return
    if code == -1:
        raise KernelError(f"{kernel}: arguments rejected by the launcher")
    if code == -2:
        raise KernelError(f"{kernel}: size not supported by this kernel")
    raise KernelError(f"{kernel}: HIP error {code} at launch")


# ------------------------------------------------------------------ row-wise kernels
def embed(tokens: torch.Tensor, table: torch.Tensor, act, scale: float = 1.0) -> torch.Tensor:
    """x[t] = table[tokens[t]] (times ``scale``) as float32 [T, H]."""
    k = "embed"
    _check(tokens, k, "tokens", torch.int32)
    _need(tokens.dim() == 1 and table.dim() == 2, k, "tokens [T], table [V, H]")
    _check(table, k, "table", tuple(_WTYPE))
    T, (V, H) = tokens.numel(), table.shape
    x = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _run(k, library(act).tq_embed(_ptr(tokens), _ptr(table), _WTYPE[table.dtype], _ptr(x), T, H, float(scale), _stream()))
    return x


def softcap(logits: torch.Tensor, cap: float, act) -> torch.Tensor:
    """logits <- cap * tanh(logits / cap), in place."""
    k = "softcap"
    _check(logits, k, "logits", torch.float32)
    _need(cap > 0, k, "the cap must be positive")
    _run(k, library(act).tq_softcap(_ptr(logits), logits.numel(), float(cap), _stream()))
    return logits


def gather_rows(src: torch.Tensor, index: torch.Tensor, act) -> torch.Tensor:
    """``src[index]`` along the first dimension (``index`` int32 on the device): the rows of a step's sequences out of
    a tensor that has a row per slot."""
    k = "gather_rows"
    _check(src, k, "src")
    _check(index, k, "index", torch.int32)
    _need(index.dim() == 1 and src.dim() >= 1, k, "index must be [n], src [rows, ...]")
    row_bytes = (src.numel() // max(src.shape[0], 1)) * src.element_size()
    out = torch.empty((index.numel(), *src.shape[1:]), dtype=src.dtype, device=src.device)
    _run(k, library(act).tq_move_rows(_ptr(src), _ptr(index), _ptr(out), index.numel(), row_bytes, 0, _stream()))
    return out


def scatter_rows(dst: torch.Tensor, index: torch.Tensor, rows: torch.Tensor, act) -> None:
    """``dst[index] = rows`` along the first dimension; every index at most once."""
    k = "scatter_rows"
    _check(dst, k, "dst")
    _check(index, k, "index", torch.int32)
    _check(rows, k, "rows", dst.dtype, (index.numel(), *dst.shape[1:]))
    row_bytes = (dst.numel() // max(dst.shape[0], 1)) * dst.element_size()
    _run(k, library(act).tq_move_rows(_ptr(rows), _ptr(index), _ptr(dst), index.numel(), row_bytes, 1, _stream()))


@dataclasses.dataclass
class GatheredSum:
    """A part's output that nobody has summed yet:
    ``out[t] = sum_j weights[t, j] * y[pair_slot[t, j]] + gate[t] * sum_s dense[s, t]`` (j ascending; ``dense``
    and ``gate`` may be None).  The next norm adds it into the residual stream in the pass that normalises;
    ``materialize`` gives it as a float32 [1, T, H] tensor to whoever needs it earlier."""
    y: torch.Tensor                      # float32 [rows, H]
    pair_slot: torch.Tensor              # int32 [T, k]
    weights: torch.Tensor                # float32 [T, k]
    dense: torch.Tensor | None = None    # float32 [S, T, H]
    gate: torch.Tensor | None = None     # float32 [T]

    def materialize(self, act) -> torch.Tensor:
        return moe_combine(self.y, self.pair_slot, self.weights, self.dense, self.gate, act)


def add_rmsnorm(x: torch.Tensor, delta, weight: torch.Tensor, eps: float, act,
                rows: torch.Tensor | None = None, want_act: bool = True, want_f32: bool = False):
    """x += delta (in place, unless ``rows`` picks rows), where delta is None, float32 partial sums [S, T, H] added
    one after the other, or a GatheredSum; returns rmsnorm(x) * weight as (activation-typed or None, float32 or
    None), one row per entry of ``rows`` (all rows if None)."""
    k = "add_rmsnorm"
    _check(x, k, "x", torch.float32)
    _need(x.dim() == 2, k, "x must be [T, H]")
    T, H = x.shape
    _check(weight, k, "weight", tuple(_WTYPE), (H,))
    y = pair_slot = weights = gate = None
    topk = 0
    if isinstance(delta, GatheredSum):
        y, pair_slot, weights, gate, delta = delta.y, delta.pair_slot, delta.weights, delta.gate, delta.dense
        _check(y, k, "y", torch.float32)
        _need(y.dim() == 2 and y.shape[1] == H, k, lambda: f"y must be [rows, {H}]")
        _check(pair_slot, k, "pair_slot", torch.int32)
        _need(pair_slot.dim() == 2 and pair_slot.shape[0] == T, k, lambda: f"pair_slot must be [{T}, k]")
        topk = pair_slot.shape[1]
        _need(1 <= topk <= 64, k, lambda: f"{topk} experts per token is beyond the 64 this kernel takes")
        _check(weights, k, "weights", torch.float32, (T, topk))
        if gate is not None:
            _check(gate, k, "gate", torch.float32, (T,))
    S, stride = 0, 0
    if delta is not None:
        _check(delta, k, "delta", torch.float32)
        _need(delta.dim() == 3 and tuple(delta.shape[1:]) == (T, H), k, lambda: f"delta must be [S, {T}, {H}], is {tuple(delta.shape)}")
        S, stride = delta.shape[0], T * H
    R = T
    if rows is not None:
        _check(rows, k, "rows", torch.int32)
        _need(rows.dim() == 1, k, "rows must be [R]")
        R = rows.numel()
    adt = ACT_DTYPES[dtype_name(act)]
    out = torch.empty((R, H), dtype=adt, device=x.device) if want_act else None
    out32 = torch.empty((R, H), dtype=torch.float32, device=x.device) if want_f32 else None
    _run(k, library(act).tq_add_rmsnorm(_ptr(x), _ptr(delta), S, stride, _ptr(y), _ptr(pair_slot), _ptr(weights), topk,
                                        _ptr(gate), _ptr(weight), _WTYPE[weight.dtype], float(eps), _ptr(rows), R,
                                        _ptr(out), _ptr(out32), H, _stream()))
    return out, out32


def head_rmsnorm(qkv: torch.Tensor, q_weight: torch.Tensor | None, k_weight: torch.Tensor | None, eps: float,
                 num_heads: int, num_kv_heads: int, head_dim: int, act) -> torch.Tensor:
    """RMS norm of every query head (weights ``q_weight`` [hd]) and key head (``k_weight``) of the float32 rows
    ``qkv`` [T, (nh + 2 nkv) * hd], in place; None leaves those heads alone.  Returns ``qkv``."""
    k = "head_rmsnorm"
    _check(qkv, k, "qkv", torch.float32)
    _need(qkv.dim() == 2 and qkv.shape[1] == (num_heads + 2 * num_kv_heads) * head_dim, k,
          lambda: f"qkv must be [T, {(num_heads + 2 * num_kv_heads) * head_dim}]")
    wtype = None
    for name, w in (("q_weight", q_weight), ("k_weight", k_weight)):
        if w is not None:
            _check(w, k, name, tuple(_WTYPE), (head_dim,))
            _need(wtype in (None, w.dtype), k, "q_weight and k_weight must have one type")
            wtype = w.dtype
    if wtype is not None:
        _run(k, library(act).tq_head_rmsnorm(_ptr(qkv), _ptr(q_weight), _ptr(k_weight), _WTYPE[wtype], float(eps),
                                             qkv.shape[0], num_heads, num_kv_heads, head_dim, _stream()))
    return qkv


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor,
                  inv_freq: torch.Tensor, pairing: int, rotary_dim: int, k_pages: torch.Tensor | None,
                  v_pages: torch.Tensor | None, layer_offset: int, page_size: int, page_stride: int,
                  num_heads: int, num_kv_heads: int, head_dim: int, act, runs: dict | None = None,
                  bias: torch.Tensor | None = None) -> torch.Tensor:
    """Rotates queries and keys, returns the queries [T, nh*hd] and writes keys and values into the pages.
    ``bias`` [width] is added to ``qkv`` as it is read, for a product that left its bias out.
    ``k_pages``/``v_pages`` are the flat page pools of the cache group (None: nothing is written, for a
    layer that reads another layer's cache); ``layer_offset`` is the layer's offset inside a page.  ``runs``
    (as for ``attention``) describes the tokens as one run of consecutive positions per sequence; with it the
    values of whole prompts are written by tiles."""
    k = "rope_kv_write"
    T = positions.numel()
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _check(qkv, k, "qkv", torch.float32, (T, width))
    if bias is not None:
        _check(bias, k, "bias", tuple(_WTYPE), (width,))
    _check(positions, k, "positions", torch.int32, (T,))
    _check(seq_of_token, k, "seq_of_token", torch.int32, (T,))
    _check(block_table, k, "block_table", torch.int32)
    _need(block_table.dim() == 2, k, "block_table must be [B, pages]")
    _check(inv_freq, k, "inv_freq", torch.float32)
    _need(inv_freq.numel() * 2 == rotary_dim or rotary_dim == 0, k, lambda: f"inv_freq must hold rotary_dim/2 = {rotary_dim // 2} entries")
    adt = ACT_DTYPES[dtype_name(act)]
    q = torch.empty((T, num_heads * head_dim), dtype=adt, device=qkv.device)
    write = k_pages is not None
    kp = vp = None
    if write:
        _check(k_pages, k, "k_pages", adt)
        _check(v_pages, k, "v_pages", adt)
        _need(layer_offset + num_kv_heads * page_size * head_dim <= page_stride, k, "layer does not fit in a page")
        esz = k_pages.element_size()
        kp, vp = k_pages.data_ptr() + layer_offset * esz, v_pages.data_ptr() + layer_offset * esz
    cu = slots = start = None
    B = max_new = 0
    if runs is not None and write and not runs["decode"]:
        B = runs["slots"].numel()
        cu, slots, start, max_new = runs["cu_seqlens"], runs["slots"], runs["start"], int(runs["max_new"])
        _check(cu, k, "cu_seqlens", torch.int32, (B + 1,))
        _check(slots, k, "slots", torch.int32, (B,))
        _check(start, k, "start", torch.int32, (B,))
        _need(int(runs["max_end"]) <= block_table.shape[1] * page_size, k, "positions reach beyond the page table")
    _run(k, library(act).tq_rope_kv_write(_ptr(qkv), _ptr(bias), _WTYPE[bias.dtype] if bias is not None else 0,
                                          _ptr(positions), _ptr(seq_of_token), _ptr(block_table),
                                          block_table.shape[1], _ptr(inv_freq), pairing, rotary_dim, _ptr(q), kp, vp,
                                          page_size, page_stride, T, num_heads, num_kv_heads, head_dim, int(write),
                                          _ptr(cu), _ptr(slots), _ptr(start), B, max_new, _stream()))
    return q


def qkv_rope_write(a: torch.Tensor, qkv_weight: torch.Tensor, qkv_bias: torch.Tensor | None, positions: torch.Tensor,
                   seq_of_token: torch.Tensor, block_table: torch.Tensor, inv_freq: torch.Tensor, pairing: int,
                   rotary_dim: int, k_pages: torch.Tensor | None, v_pages: torch.Tensor | None, layer_offset: int,
                   page_size: int, page_stride: int, num_heads: int, num_kv_heads: int, head_dim: int, act,
                   runs: dict | None = None) -> torch.Tensor:
    """``gemm(a, qkv_weight, bias=qkv_bias)`` followed by ``rope_kv_write``: the queries [T, nh*hd], keys and
    values in their pages.  Up to 16 tokens in bfloat16, with heads rotated whole in "half" pairing, take one
    launch (the product's workgroups rotate and store what they have summed); anything else is the two calls."""
    k = "qkv_rope_write"
    lib = library(act)
    T, K = a.shape
    fused = (hasattr(lib, "tq_qkv_rope_write") and T <= 16 and pairing == 0 and rotary_dim == head_dim
             and head_dim % 32 == 0 and _use_mfma(act, a, qkv_weight, K)
             and (qkv_bias is None or qkv_bias.dtype in _WTYPE))
    if not fused:
        # the vendor library's product has no bias of its own that costs nothing: the rotation adds it as it reads
        late = qkv_bias is not None and a.dim() == 2 and _vendor_product(act, a, qkv_weight, T, K)
        qkv = gemm(a, qkv_weight, act, bias=None if late else qkv_bias)
        return rope_kv_write(qkv, positions, seq_of_token, block_table, inv_freq, pairing, rotary_dim, k_pages, v_pages,
                             layer_offset, page_size, page_stride, num_heads, num_kv_heads, head_dim, act, runs=runs,
                             bias=qkv_bias if late else None)
    adt = ACT_DTYPES[dtype_name(act)]
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _check(a, k, "a", adt)
    _need(a.stride(1) == 1, k, "a must have unit stride along its rows")
    _check(qkv_weight, k, "qkv_weight", torch.bfloat16, (width, K))
    if qkv_bias is not None:
        _check(qkv_bias, k, "qkv_bias", tuple(_WTYPE), (width,))
    _check(positions, k, "positions", torch.int32, (T,))
    _check(seq_of_token, k, "seq_of_token", torch.int32, (T,))
    _check(block_table, k, "block_table", torch.int32)
    _need(block_table.dim() == 2, k, "block_table must be [B, pages]")
    _check(inv_freq, k, "inv_freq", torch.float32, (head_dim // 2,))
    q = torch.empty((T, num_heads * head_dim), dtype=adt, device=a.device)
    kp = vp = None
    if k_pages is not None:
        _check(k_pages, k, "k_pages", adt)
        _check(v_pages, k, "v_pages", adt)
        _need(layer_offset + num_kv_heads * page_size * head_dim <= page_stride, k, "layer does not fit in a page")
        esz = k_pages.element_size()
        kp, vp = k_pages.data_ptr() + layer_offset * esz, v_pages.data_ptr() + layer_offset * esz
    _run(k, lib.tq_qkv_rope_write(_ptr(a), a.stride(0), _ptr(qkv_weight), _ptr(qkv_bias),
                                  _WTYPE[qkv_bias.dtype] if qkv_bias is not None else 0, T, K, _ptr(positions),
                                  _ptr(seq_of_token), _ptr(block_table), block_table.shape[1], _ptr(inv_freq), _ptr(q),
                                  kp, vp, page_size, page_stride, num_heads, num_kv_heads, head_dim, _stream()))
    return q


def moe_combine(y: torch.Tensor, pair_slot: torch.Tensor, weights: torch.Tensor, shared: torch.Tensor | None,
                shared_gate: torch.Tensor | None, act) -> torch.Tensor:
    """out[t] = sum_j weights[t, j] * y[pair_slot[t, j]] + shared_gate[t] * sum_s shared[s, t]; float32 [1, T, H]."""
    k = "moe_combine"
    _check(y, k, "y", torch.float32)
    T, topk = pair_slot.shape
    H = y.shape[1]
    _check(pair_slot, k, "pair_slot", torch.int32)
    _check(weights, k, "weights", torch.float32, (T, topk))
    S, stride = 0, 0
    if shared is not None:
        _check(shared, k, "shared", torch.float32)
        _need(shared.dim() == 3 and tuple(shared.shape[1:]) == (T, H), k, lambda: f"shared must be [S, {T}, {H}]")
        S, stride = shared.shape[0], T * H
    if shared_gate is not None:
        _check(shared_gate, k, "shared_gate", torch.float32, (T,))
    out = torch.empty((1, T, H), dtype=torch.float32, device=y.device)
    _run(k, library(act).tq_moe_combine(_ptr(y), _ptr(pair_slot), _ptr(weights), topk, _ptr(shared), S, stride,
                                        _ptr(shared_gate), _ptr(out), T, H, _stream()))
    return out


# ------------------------------------------------------------------ matrix products
def _use_mfma(act, a: torch.Tensor, w: torch.Tensor, K: int) -> bool:
    return (dtype_name(act) == "bfloat16" and w.dtype == torch.bfloat16 and K % 8 == 0
            and has_kernel(act, "tq_gemm_mfma"))


EXPERT_16_UPTO, EXPERT_32_UPTO = 5, 10
# Rows per expert on average from which the row order's unit is 128 and 256: never, since units of 64 taken two at a
# time do better wherever the taller units did (see expert_tile_rows); tests lower them to run those kernels.
EXPERT_128_FROM = EXPERT_256_FROM = 1 << 30
TILE_PAIRS = 1024            # added to tile_rows 64: two units of one expert per workgroup (TQ_TILE_PAIRS)
EXPERT_PAIRS_FROM = 48       # rows per expert on average from which units of 64 are taken two at a time


def expert_tile_rows(n_pairs: int, num_experts: int, act, a: torch.Tensor, w: torch.Tensor) -> int:
    """Rows per tile (the padding unit of the row order) that suit a product over experts, by the pairs per expert on
    average.  Up to 5: 16, the streaming kernel, which passes an expert's matrices once per 16 of its rows.  Up to 10,
    where the bfloat16 matrix-core product runs: 32, the same kernel with two row tiles and two column tiles to a wave.
    Beyond: tiles of 64 rows.  Where the borders lie depends on how evenly the router deals: with tokens dealt evenly
    (60 experts of 1,408 x 2,048, 4 per token, both products) units of 16 are best up to 8 rows per expert by 3 to 6 %,
    units of 32 from 10 to 24 by 9 to 13 % (202 us at 16 rows per expert against 270 and 233), tiles of 64 rows beyond;
    with a router of random weights, which gives some experts three times the rows of others, units of 32 are best up
    to 6 rows per expert (64 experts, 8 per token: up to 12) and tiles of 64 rows win by 10 to 18 % from 12 on, since a
    crowded expert's matrices pass the streaming kernel once per unit.  The borders here lose at most 6 % either way (a replayed decode step of 64 sequences, 4.3 rows per expert, is 2 %
    faster with units of 16 than of 32).
    Without the matrix-core product 16 up to 12.  Units of 128 and 256 rows (EXPERT_128_FROM, EXPERT_256_FROM) are
    not chosen: they were 8 to 17 % faster than single tiles of 64 rows from 256 rows per expert on, but units of 64
    taken two at a time (expert_product_rows) are faster than either (60 experts of 1,408 x 2,048, both products:
    396 us against 448 at 205 rows per expert, 492 against 565 at 273, 841 against 949 at 546; 64 experts of
    2,560 x 3,584 at 1,650 rows each: a prompt step of 425 ms against 436 with units of 256)."""
    mfma = _use_mfma(act, a, w, a.shape[1])
    if n_pairs <= (EXPERT_16_UPTO if mfma else 12) * num_experts:
        return 16
    if mfma and n_pairs <= EXPERT_32_UPTO * num_experts:
        return 32
    if mfma and n_pairs >= EXPERT_128_FROM * num_experts:
        return 256 if n_pairs >= EXPERT_256_FROM * num_experts else 128
    return 64


def expert_product_rows(unit: int, n_pairs: int, num_experts: int) -> int:
    """The ``tile_rows`` that a product over experts is called with when the row order has units of ``unit`` rows: from
    48 rows per expert on average, units of 64 two at a time (measured on 60 experts of 1,408 x 2,048, four per
    token, both products together: 251 us against 286 at 68 rows per expert, 260 against 307 at 102, 346 against 360
    at 137; level below; a prompt step of 24 layers: 10.3 ms against 10.9 at 1,024 tokens, 15.8 against 17.0 at
    2,048, 22.3 against 23.7 at 3,072; where the border lies, by such steps: 9.42 ms against 9.73 at 55 rows per
    expert and 9.75 against 10.22 at 60, which already gives many experts a second unit, level at 43 and 47, 7.97
    against 7.81 at 34)."""
    if unit == 64 and n_pairs >= EXPERT_PAIRS_FROM * num_experts:
        return 64 + TILE_PAIRS
    return unit


def _gemm_problem(k: str, a, w, act, bias, w2, out_act, a_rows, tile_group, n_tiles, tile_rows, gather):
    """Checks one product's operands; returns (M, N, K, tile_rows, group stride)."""
    adt = ACT_DTYPES[dtype_name(act)]
    _check(a, k, "a", adt)
    _need(a.dim() == 2, k, "a must be [M, K]")
    K = a.shape[1]
    _check(w, k, "w", tuple(_WTYPE))
    grouped = tile_group is not None
    if grouped:
        _need(w.dim() == 3 and w.shape[2] == K, k, lambda: f"grouped w must be [G, N, {K}], is {tuple(w.shape)}")
        _need(a_rows is not None and n_tiles is not None and tile_rows in (16, 32, 64, 128, 256, 64 + TILE_PAIRS), k,
              "grouped product needs a_rows, n_tiles and tile_rows of 16, 64, 128 or 256")
        if not _use_mfma(act, a, w, a.shape[1]):
            _need(tile_rows % TILE_PAIRS in (16, 64), k, "tiles of 32, 128 and 256 rows are for the bfloat16 matrix-core product")
            tile_rows %= TILE_PAIRS      # pairs of units are that product's too: the others take unit by unit
        _check(a_rows, k, "a_rows", torch.int32)
        _check(tile_group, k, "tile_group", torch.int32)
        _check(n_tiles, k, "n_tiles", torch.int32)
        M = a_rows.numel()
        unit = tile_rows % TILE_PAIRS
        _need(M % unit == 0 and tile_group.numel() >= M // unit, k, "a_rows must hold whole tiles, each with a group")
        _need(tile_rows == unit or (tile_group.numel() >= 2 * (M // unit) and n_tiles.numel() >= 2), k,
              "pairs of tiles need the items behind the row tiles (tile_group [2 M / 64], n_tiles [2])")
        N = w.shape[1]
        gstride = N * K
    else:
        _need(w.dim() == 2 and w.shape[1] == K, k, lambda: f"w must be [N, {K}], is {tuple(w.shape)}")
        N = w.shape[0]
        M = a.shape[0] if a_rows is None else a_rows.numel()
        if a_rows is not None:
            _check(a_rows, k, "a_rows", torch.int32)
        gstride = 0
        if tile_rows is None:
            tile_rows = 16 if M <= 32 else 64
    if w2 is not None:
        _check(w2, k, "w2", w.dtype, tuple(w.shape))
    if bias is not None:
        _check(bias, k, "bias", tuple(_WTYPE), (N,))
    return M, N, K, tile_rows, gstride


# Plain bfloat16 products of many rows may go through the vendor's matrix library (hipBLASLt behind torch.mm), as the
# reference's engine hands its plain products to a BLAS where it has one
# (/root/reference/src/engine/tq_ops.c:296-305): measured on gfx950 it is 25 to 35 % faster than the tile kernel here
# from 512 rows on ([2048, 2048] x [6144, 2048]: 48 against 63 us; 13,199 rows: 282 against 401), slower or equal
# below and where k is long and the rows are not many ([4096, 20480] x [3584, 20480]: 724 against 687 us).  A call
# into the library costs the host twice what a launch here costs, and a step of 512 to 767 rows is as long on the
# host as on the chip (24 layers of 512 tokens: 9.7 ms through the library, 7.9 without), so it starts at 768 rows.
# TQ_PLAIN_PRODUCTS=own keeps every product in this library's kernels.  Products over experts, gated pairs whose
# matrices lie apart, products with a bias that nothing behind them can add, products of few rows, decode steps,
# steps under graph capture and the 32-bit path never leave them.
VENDOR_MIN_ROWS = 768
_VENDOR = os.environ.get("TQ_PLAIN_PRODUCTS", "vendor") != "own"


class own_products:
    """``with own_products(True):`` keeps every product inside in this library's kernels: what a decode step runs
    eagerly must be what its capture will replay, however many sequences it has."""

    def __init__(self, on: bool = True):
        self.on = on

    def __enter__(self):
        global _VENDOR
        self.before = _VENDOR
        if self.on:
            _VENDOR = False

    def __exit__(self, *exc):
        global _VENDOR
        _VENDOR = self.before


def _vendor_product(act, a, w, M: int, K: int) -> bool:
    return (_VENDOR and M >= VENDOR_MIN_ROWS and (K < 16384 or M >= 8192) and dtype_name(act) == "bfloat16"
            and w.dtype == torch.bfloat16 and a.stride(1) == 1 and w.is_contiguous()
            and not torch.cuda.is_current_stream_capturing())


def _vendor_gemm(a, w, out_act: bool) -> torch.Tensor:
    """a w^T by the vendor library: sums in float32, stored as bfloat16 or float32.  It adds no bias: its product
    with one takes a pass more over the result (77 against 48 us), so a product with a bias stays here unless the
    caller has a kernel behind it that adds the bias on its way."""
    out = torch.mm(a, w.t()) if out_act else torch.mm(a, w.t(), out_dtype=torch.float32)
    if _PROFILE is not None:
        _mark("matmul")
    return out


VENDOR_GATED_ROWS = 4096      # rows of a gated pair that go through the vendor library at a time


def side_by_side(first: torch.Tensor, second: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """The two matrices of a gated pair in one piece of memory, the second right behind the first: so laid, ``gemm``
    may hand a pair of many rows to the vendor library as one product over both."""
    both = torch.cat([first, second])
    return both[:first.shape[0]], both[first.shape[0]:]


def _behind(w: torch.Tensor, w2: torch.Tensor) -> bool:
    return (w2.is_contiguous() and w2.untyped_storage().data_ptr() == w.untyped_storage().data_ptr()
            and w2.data_ptr() == w.data_ptr() + w.numel() * w.element_size())


def _vendor_gated(a, w, N: int, K: int, gate: int, act) -> torch.Tensor:
    """f(a w^T) * (a w2^T) with w2 behind w: one product of the vendor library over both matrices into float32, a
    few thousand rows at a time, and the gate's activation in a pass of its own."""
    both = torch.as_strided(w, (2 * N, K), (K, 1))
    M = a.shape[0]
    out = torch.empty((M, N), dtype=ACT_DTYPES[dtype_name(act)], device=a.device)
    lib = library(act)
    for r in range(0, M, VENDOR_GATED_ROWS):
        rows = min(VENDOR_GATED_ROWS, M - r)
        gu = torch.mm(a[r:r + rows], both.t(), out_dtype=torch.float32)
        if _PROFILE is not None:
            _mark("matmul")
        _run("gated_act", lib.tq_gated_act(_ptr(gu), 2 * N, _ptr(out[r:]), rows, N, gate, _stream()))
    return out


def _gate_code(k: str, activation: str) -> int:
    _need(activation in GATES, k, lambda: f"unknown activation {activation!r}; known: {', '.join(sorted(GATES))}")
    return GATES[activation]


def _use_f32(act, a: torch.Tensor, w: torch.Tensor, K: int, gstride: int) -> bool:
    """The float matrix-core product takes float operands whose rows start at multiples of 16 bytes."""
    return (dtype_name(act) == "float32" and w.dtype == torch.float32 and a.dtype == torch.float32 and K % 4 == 0
            and a.stride(0) % 4 == 0 and gstride % 4 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and has_kernel(act, "tq_gemm_f32"))


def gemm(a: torch.Tensor, w: torch.Tensor, act, bias: torch.Tensor | None = None, w2: torch.Tensor | None = None,
         out_act: bool = False, a_rows: torch.Tensor | None = None, tile_group: torch.Tensor | None = None,
         n_tiles: torch.Tensor | None = None, tile_rows: int | None = None, gather: bool = True,
         partial_sums: bool = False, activation: str = "silu") -> torch.Tensor:
    """out[m, n] = sum_k a[row(m), k] * w[g, n, k]  (+ bias[n]);  with ``w2``: f(a w^T) * (a w2^T), f being the
    ``activation`` (silu, gelu_tanh or relu2).

    ``a`` [M, K] activations.  ``w`` [N, K], or [G, N, K] with ``tile_group`` naming the matrix of each tile of
    ``tile_rows`` output rows and ``a_rows`` [P] the row of ``a`` behind each output row (-1: none; with
    ``gather`` false a live output row m reads row m of ``a``).
    Output is float32 unless ``out_act``.  Sums run over k in ascending order whatever M is.
    ``partial_sums`` (plain products into float32 only): the result is [S, M, N], S >= 1 partial sums over runs of
    k that the caller adds up in order, as the next norm does with a part's output; the kernel chooses S.
    """
    k = "gemm"
    adt = ACT_DTYPES[dtype_name(act)]
    grouped = tile_group is not None
    M, N, K, tile_rows, gstride = _gemm_problem(k, a, w, act, bias, w2, out_act, a_rows, tile_group, n_tiles, tile_rows,
                                                gather)
    if partial_sums:
        _need(w2 is None and not out_act and not grouped and a_rows is None, k,
              "partial sums are for plain products into float32")
    lib = library(act)
    gate = _gate_code(k, activation)
    if not grouped and a_rows is None and bias is None and _vendor_product(act, a, w, M, K):
        if w2 is None:
            out = _vendor_gemm(a, w, out_act)
            return out[None] if partial_sums else out
        if out_act and _behind(w, w2):
            return _vendor_gated(a, w, N, K, gate, act)
    if _use_mfma(act, a, w, K) and (bias is None or bias.dtype in _WTYPE):
        splits = lib.tq_gemm_mfma_splits(M, N, K) if partial_sums else 1
        out = torch.empty((splits, M, N) if partial_sums else (M, N), dtype=adt if out_act else torch.float32,
                          device=a.device)
        _run("gemm_mfma", lib.tq_gemm_mfma(_ptr(a), a.stride(0), _ptr(a_rows), int(gather), _ptr(w), _ptr(w2), gstride,
                                           _ptr(tile_group), _ptr(n_tiles), _ptr(bias),
                                           _WTYPE[bias.dtype] if bias is not None else 0, _ptr(out), N, int(out_act),
                                           M, N, K, tile_rows, splits, gate, _stream()), "moe" if grouped else None)
        return out
    if _use_f32(act, a, w, K, gstride) and (w2 is None or w2.data_ptr() % 16 == 0):
        # a narrow matrix times few rows is cut into runs of k: they come back apart if the caller adds them up
        # anyway, else they pass through scratch memory and a second kernel
        runs = lib.tq_gemm_f32_runs(M, N, K, int(grouped or a_rows is not None))
        out = torch.empty((runs, M, N) if partial_sums else (M, N), dtype=torch.float32, device=a.device)
        scratch = None
        if runs > 1 and not partial_sums:
            scratch = torch.empty((runs * (2 if w2 is not None else 1), M, N), dtype=torch.float32, device=a.device)
        _run("gemm_f32", lib.tq_gemm_f32(_ptr(a), a.stride(0), _ptr(a_rows), int(gather), _ptr(w), _ptr(w2), gstride,
                                         _ptr(tile_group), _ptr(n_tiles), _ptr(bias),
                                         _WTYPE[bias.dtype] if bias is not None else 0, _ptr(out), N, M, N, K, tile_rows,
                                         gate, _ptr(scratch), int(partial_sums and runs > 1), _stream()),
             "moe" if grouped else None)
        return out
    out = torch.empty((1, M, N) if partial_sums else (M, N), dtype=adt if out_act else torch.float32, device=a.device)
    _run(k, lib.tq_gemm_generic(_ptr(a), a.stride(0), _ptr(a_rows), int(gather), _ptr(w), _ptr(w2), _WTYPE[w.dtype], gstride,
                                _ptr(tile_group), _ptr(n_tiles), _ptr(bias),
                                _WTYPE[bias.dtype] if bias is not None else 0, _ptr(out), N, int(out_act), M, N, K,
                                tile_rows, gate, _stream()), "moe" if grouped else None)
    return out


def gemm_pair(first: dict, second: dict, act) -> tuple[torch.Tensor, torch.Tensor]:
    """Two products that do not depend on each other; ``first`` and ``second`` hold the arguments of ``gemm``
    (``partial_sums`` only in the second).  Products of few rows of the same kind (both gated or both plain, into
    the same type) go out in one launch, so that the smaller one costs no launch of its own; anything else is two
    calls."""
    k = "gemm_pair"
    keys = ("bias", "w2", "out_act", "a_rows", "tile_group", "n_tiles", "tile_rows", "gather", "partial_sums", "activation")
    probs = []
    _need(not first.get("partial_sums", False), k, "only the second product may leave partial sums")
    for p in (first, second):
        full = {"bias": None, "w2": None, "out_act": False, "a_rows": None, "tile_group": None, "n_tiles": None,
                "tile_rows": None, "gather": True, "partial_sums": False, "activation": "silu"}
        _need(set(p) <= set(full) | {"a", "w"}, k, lambda: f"unknown arguments {sorted(set(p) - set(full) - {'a', 'w'})}")
        full.update(p)
        probs.append(full)
    lib = library(act) if dtype_name(act) == "bfloat16" else None
    fused = lib is not None and hasattr(lib, "tq_gemm_mfma_pair")
    dims = []
    for p in probs:
        M, N, K, tile_rows, gstride = _gemm_problem(k, p["a"], p["w"], act, p["bias"], p["w2"], p["out_act"], p["a_rows"],
                                                    p["tile_group"], p["n_tiles"], p["tile_rows"], p["gather"])
        dims.append((M, N, K, tile_rows, gstride))
        few = (p["tile_group"] is not None and tile_rows == 16) or (p["tile_group"] is None and M <= 16)
        fused = fused and few and _use_mfma(act, p["a"], p["w"], K) and (p["bias"] is None or p["bias"].dtype in _WTYPE)
    fused = fused and (probs[0]["w2"] is None) == (probs[1]["w2"] is None) and probs[0]["out_act"] == probs[1]["out_act"]
    if not fused:
        return tuple(gemm(p["a"], p["w"], act, **{n: p[n] for n in keys}) for p in probs)
    adt = ACT_DTYPES[dtype_name(act)]
    outs, descs = [], []
    splits = 1
    if probs[1]["partial_sums"]:
        p2 = probs[1]
        _need(p2["w2"] is None and not p2["out_act"] and p2["tile_group"] is None and p2["a_rows"] is None, k,
              "partial sums are for plain products into float32")
        splits = lib.tq_gemm_mfma_pair_splits(dims[0][1], dims[0][2], int(probs[0]["tile_group"] is not None),
                                              dims[1][1], dims[1][2], 0)
    for p, (M, N, K, tile_rows, gstride) in zip(probs, dims):
        shape = (splits, M, N) if p["partial_sums"] else (M, N)
        out = torch.empty(shape, dtype=adt if p["out_act"] else torch.float32, device=p["a"].device)
        outs.append(out)
        vals = [_ptr(p["a"]), p["a"].stride(0), _ptr(p["a_rows"]), int(p["gather"]), _ptr(p["w"]), _ptr(p["w2"]), gstride,
                _ptr(p["tile_group"]), _ptr(p["n_tiles"]), _ptr(p["bias"]),
                _WTYPE[p["bias"].dtype] if p["bias"] is not None else 0, _ptr(out), N, int(p["out_act"]), M, N, K, tile_rows,
                _gate_code(k, p["activation"])]
        descs.append((ctypes.c_int64 * 19)(*[0 if v is None else int(v) for v in vals]))
    _run(k, lib.tq_gemm_mfma_pair(descs[0], descs[1], splits, _stream()),
         "moe" if any(p["tile_group"] is not None for p in probs) else None)
    return outs[0], outs[1]


# ------------------------------------------------------------------ attention
def attention(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, layer_offset: int,
              positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor, page_size: int,
              page_stride: int, num_heads: int, num_kv_heads: int, head_dim: int, window: int | None,
              scale: float, act, runs: dict | None = None) -> torch.Tensor:
    """Each token attends to its sequence's cached positions up to its own; returns [T, nh*hd].

    ``seq_of_token`` gives each token's row of ``block_table`` (its slot).  ``runs`` describes the same tokens
    as runs of consecutive positions, one per sequence, for the kernels that work on tiles of tokens:
    ``cu_seqlens`` [B+1], ``slots`` [B], ``start`` [B] (device, int32) and the host numbers ``max_new``,
    ``max_end`` and ``decode`` (every sequence brings one token).  Without it the token-by-token kernel runs."""
    k = "attention"
    adt = ACT_DTYPES[dtype_name(act)]
    T = positions.numel()
    _check(q, k, "q", adt, (T, num_heads * head_dim))
    _check(k_pages, k, "k_pages", adt)
    _check(v_pages, k, "v_pages", adt)
    _check(positions, k, "positions", torch.int32, (T,))
    _check(seq_of_token, k, "seq_of_token", torch.int32, (T,))
    _check(block_table, k, "block_table", torch.int32)
    _need(block_table.dim() == 2, k, "block_table must be [B, pages]")
    _need(num_heads % num_kv_heads == 0, k, "heads must be a multiple of kv heads")
    _need(head_dim <= 512, k, lambda: f"head size {head_dim} is beyond the 512 this kernel takes")
    _need(layer_offset + num_kv_heads * page_size * head_dim <= page_stride, k, "layer does not fit in a page")
    out = torch.empty_like(q)
    esz = k_pages.element_size()
    lib = library(act)
    if (runs is not None and dtype_name(act) == "bfloat16" and hasattr(lib, "tq_attention_mfma")
            and head_dim % 16 == 0 and head_dim <= 256 and page_size % 64 == 0 and page_stride % 8 == 0 and scale > 0):
        B = runs["slots"].numel()
        _check(runs["cu_seqlens"], k, "cu_seqlens", torch.int32, (B + 1,))
        _check(runs["slots"], k, "slots", torch.int32, (B,))
        _check(runs["start"], k, "start", torch.int32, (B,))
        _need(runs["max_end"] <= block_table.shape[1] * page_size, k, "positions reach beyond the page table")
        partial = None
        if runs["decode"]:
            _need(T == B, k, "decoding brings one token per sequence")
            partial = torch.empty((lib.tq_attention_decode_scratch(B, num_heads, head_dim, int(runs["max_end"])),),
                                  dtype=torch.float32, device=q.device)
        _run("attention_mfma", lib.tq_attention_mfma(
            _ptr(q), k_pages.data_ptr() + layer_offset * esz, v_pages.data_ptr() + layer_offset * esz,
            _ptr(block_table), block_table.shape[1], _ptr(runs["cu_seqlens"]), _ptr(runs["slots"]), _ptr(runs["start"]),
            page_size, page_stride, B, num_heads, num_kv_heads, head_dim, int(window or 0), float(scale), _ptr(out),
            _ptr(partial), int(bool(runs["decode"])), int(runs["max_new"]), int(runs["max_end"]), _stream()))
        return out
    if (runs is not None and dtype_name(act) == "float32" and hasattr(lib, "tq_attention_f32") and head_dim % 4 == 0
            and head_dim <= 256 and page_size % 64 == 0 and page_stride % 4 == 0 and layer_offset % 4 == 0):
        B = runs["slots"].numel()
        _check(runs["cu_seqlens"], k, "cu_seqlens", torch.int32, (B + 1,))
        _check(runs["slots"], k, "slots", torch.int32, (B,))
        _check(runs["start"], k, "start", torch.int32, (B,))
        _need(runs["max_end"] <= block_table.shape[1] * page_size, k, "positions reach beyond the page table")
        partial = None
        if runs["decode"]:
            _need(T == B, k, "decoding brings one token per sequence")
            partial = torch.empty((lib.tq_attention_f32_scratch(B, num_heads, head_dim, int(runs["max_end"])),),
                                  dtype=torch.float32, device=q.device)
        _run("attention_f32", lib.tq_attention_f32(
            _ptr(q), k_pages.data_ptr() + layer_offset * esz, v_pages.data_ptr() + layer_offset * esz,
            _ptr(block_table), block_table.shape[1], _ptr(runs["cu_seqlens"]), _ptr(runs["slots"]), _ptr(runs["start"]),
            page_size, page_stride, B, num_heads, num_kv_heads, head_dim, int(window or 0), float(scale), _ptr(out),
            _ptr(partial), int(bool(runs["decode"])), int(runs["max_new"]), int(runs["max_end"]), _stream()))
        return out
    _run(k, lib.tq_attention_generic(_ptr(q), k_pages.data_ptr() + layer_offset * esz,
                                              v_pages.data_ptr() + layer_offset * esz, _ptr(positions),
                                              _ptr(seq_of_token), _ptr(block_table), block_table.shape[1], page_size,
                                              page_stride, T, num_heads, num_kv_heads, head_dim, int(window or 0),
                                              float(scale), _ptr(out), _stream()))
    return out


# ------------------------------------------------------------------ routing
def router_topk(x32: torch.Tensor, router: torch.Tensor, shared_scale: torch.Tensor | None, top_k: int,
                renormalize: bool, act):
    """ids int32 [T, k], weights float32 [T, k], and sigmoid(x . shared_scale) float32 [T] (or None)."""
    k = "router_topk"
    T, H, E, ids, weights, gate, logits = _router_outputs(k, x32, router, shared_scale, top_k)
    _run(k, library(act).tq_router_topk(_ptr(x32), _ptr(router), _ptr(shared_scale), _WTYPE[router.dtype], E, top_k,
                                        int(bool(renormalize)), _ptr(ids), _ptr(weights), _ptr(gate), _ptr(logits),
                                        T, H, _stream()))
    return ids, weights, gate


def _router_outputs(k: str, x32: torch.Tensor, router: torch.Tensor, shared_scale: torch.Tensor | None, top_k: int):
    _check(x32, k, "x", torch.float32)
    _need(x32.dim() == 2, k, "x must be [T, H]")
    T, H = x32.shape
    _check(router, k, "router", tuple(_WTYPE))
    _need(router.dim() == 2 and router.shape[1] == H, k, lambda: f"router must be [E, {H}]")
    E = router.shape[0]
    _need(1 <= top_k <= min(E, 64), k, lambda: f"top_k {top_k} must be within 1..min(E, 64)")
    if shared_scale is not None:
        _check(shared_scale, k, "shared_scale", router.dtype)
        _need(shared_scale.numel() == H, k, lambda: f"shared_scale must hold {H} values")
    ids = torch.empty((T, top_k), dtype=torch.int32, device=x32.device)
    weights = torch.empty((T, top_k), dtype=torch.float32, device=x32.device)
    gate = torch.empty((T,), dtype=torch.float32, device=x32.device) if shared_scale is not None else None
    logits = torch.empty((T, E + (1 if shared_scale is not None else 0)), dtype=torch.float32, device=x32.device)
    return T, H, E, ids, weights, gate, logits


def _align_outputs(T: int, topk: int, num_experts: int, unit: int, dev):
    n_pairs = T * topk
    # every expert with at least one pair wastes at most unit-1 rows
    cap = n_pairs + min(num_experts, n_pairs) * (unit - 1)
    cap = (cap + unit - 1) // unit * unit
    sorted_token = torch.empty((cap,), dtype=torch.int32, device=dev)
    pair_slot = torch.empty((T, topk), dtype=torch.int32, device=dev)
    tile_expert = torch.empty((2 * (cap // unit),), dtype=torch.int32, device=dev)      # row tiles, then items of two
    n_tiles = torch.empty((2,), dtype=torch.int32, device=dev)
    return cap, sorted_token, pair_slot, tile_expert, n_tiles


def route(x32: torch.Tensor, router: torch.Tensor, shared_scale: torch.Tensor | None, top_k: int, renormalize: bool,
          unit: int, act):
    """``router_topk`` followed by ``moe_align`` in one call: (ids, weights, gate, sorted_token, pair_slot,
    tile_expert, n_tiles), with the same results; a handful of tokens takes one kernel less."""
    k = "route"
    T, H, E, ids, weights, gate, logits = _router_outputs(k, x32, router, shared_scale, top_k)
    _need(unit in (16, 32, 64, 128, 256), k, "unit must be 16, 32, 64, 128 or 256")
    cap, sorted_token, pair_slot, tile_expert, n_tiles = _align_outputs(T, top_k, E, unit, x32.device)
    _run(k, library(act).tq_route(_ptr(x32), _ptr(router), _ptr(shared_scale), _WTYPE[router.dtype], E, top_k,
                                  int(bool(renormalize)), _ptr(ids), _ptr(weights), _ptr(gate), _ptr(logits), unit, cap,
                                  _ptr(sorted_token), _ptr(pair_slot), _ptr(tile_expert), _ptr(n_tiles), T, H, _stream()))
    return ids, weights, gate, sorted_token, pair_slot, tile_expert, n_tiles


def moe_align(ids: torch.Tensor, num_experts: int, unit: int, act):
    """Orders the (token, expert) pairs by expert.  Returns sorted_token [cap], pair_slot [T, k],
    tile_expert [cap/unit], n_tiles [1]; each expert's rows start at a multiple of ``unit``."""
    k = "moe_align"
    _check(ids, k, "ids", torch.int32)
    T, topk = ids.shape
    n_pairs = T * topk
    cap, sorted_token, pair_slot, tile_expert, n_tiles = _align_outputs(T, topk, num_experts, unit, ids.device)
    _run(k, library(act).tq_moe_align(_ptr(ids), n_pairs, num_experts, topk, unit, cap, _ptr(sorted_token),
                                      _ptr(pair_slot), _ptr(tile_expert), _ptr(n_tiles), _stream()))
    return sorted_token, pair_slot, tile_expert, n_tiles


# ------------------------------------------------------------------ sampling
def argmax(logits: torch.Tensor, act) -> torch.Tensor:
    k = "argmax"
    _check(logits, k, "logits", torch.float32)
    R, V = logits.shape
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _run(k, library(act).tq_argmax(_ptr(logits), R, V, _ptr(out), _stream()))
    return out


def nll(logits: torch.Tensor, targets: torch.Tensor, act) -> torch.Tensor:
    """-log softmax(logits[r])[targets[r]] per row, float32 [R] (NaN where the target is no token of the vocabulary)."""
    k = "nll"
    _check(logits, k, "logits", torch.float32)
    R, V = logits.shape
    _check(targets, k, "targets", torch.int32, (R,))
    out = torch.empty((R,), dtype=torch.float32, device=logits.device)
    _run(k, library(act).tq_nll(_ptr(logits), R, V, _ptr(targets), _ptr(out), _stream()))
    return out


def probs_half(logits: torch.Tensor, act, want_probs: bool = True,
               base: torch.Tensor | None = None) -> tuple[torch.Tensor | None, torch.Tensor | None]:
    """Each row's probabilities as the reference stores them with ``--save-logits`` (16-bit floats made by its own
    conversion: the mantissa cut, below 2^-14 zero; int16 [R, V], the bit patterns) and, with ``base`` (such rows of
    another run), the KL divergence of ``base`` against this row, float64 [R]
    (/root/reference/tools/quant.c:594-636)."""
    k = "probs_half"
    _check(logits, k, "logits", torch.float32)
    _need(logits.dim() == 2, k, "logits must be [R, V]")
    R, V = logits.shape
    _need(want_probs or base is not None, k, "nothing is asked for")
    probs = torch.empty((R, V), dtype=torch.int16, device=logits.device) if want_probs else None
    kl = None
    if base is not None:
        _check(base, k, "base", torch.int16, (R, V))
        kl = torch.empty((R,), dtype=torch.float64, device=logits.device)
    _run(k, library(act).tq_probs_half(_ptr(logits), R, V, _ptr(probs), _ptr(base), _ptr(kl), _stream()))
    return probs, kl


def rep_penalty(logits: torch.Tensor, recent: torch.Tensor, counts: torch.Tensor, penalty: float, act) -> None:
    k = "rep_penalty"
    _check(logits, k, "logits", torch.float32)
    R, V = logits.shape
    _check(recent, k, "recent", torch.int32)
    _need(recent.dim() == 2 and recent.shape[0] == R, k, lambda: f"recent must be [{R}, window]")
    _check(counts, k, "counts", torch.int32, (R,))
    _run(k, library(act).tq_rep_penalty(_ptr(logits), R, V, _ptr(recent), recent.shape[1], _ptr(counts),
                                        float(penalty), _stream()))


def sample_topp(logits: torch.Tensor, temperature: float, top_p: float, uniforms: torch.Tensor, act) -> torch.Tensor:
    k = "sample_topp"
    _check(logits, k, "logits", torch.float32)
    R, V = logits.shape
    _check(uniforms, k, "uniforms", torch.float32, (R,))
    _need(temperature > 0 and top_p > 0, k, "temperature and top_p must be positive (else use argmax)")
    probs = torch.empty((R, V), dtype=torch.float32, device=logits.device)
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    lib = library(act)
    scratch = torch.empty((lib.tq_sample_topp_scratch(R),), dtype=torch.float32, device=logits.device)
    _run(k, lib.tq_sample_topp(_ptr(logits), R, V, float(temperature), float(top_p), _ptr(uniforms), _ptr(probs),
                               _ptr(scratch), _ptr(out), _stream()))
    return out


# ------------------------------------------------------------------------------------------------ probes
def probe_stream(buf: torch.Tensor, once: bool) -> None:
    """One read of all of ``buf`` (whole lines of 128 bytes per instruction; ``once``: with the read-once hint)."""
    k = "probe_stream"
    _need(buf.is_cuda and buf.is_contiguous(), k, "buf must be a contiguous tensor on the GPU")
    nbytes = buf.numel() * buf.element_size()
    out = torch.zeros((1,), dtype=torch.int32, device=buf.device)
    _run(k, library("bfloat16").tq_probe_stream(_ptr(buf), nbytes, int(once), 0x9e3779b9, _ptr(out), _stream()))


def probe_mfma(shape: int, workgroups: int, iters: int, seed: int, device) -> float:
    """A loop of bfloat16 matrix instructions alone (shape 32: 32x32x16, 16: 16x16x32); returns the number of
    floating-point operations that the launch does."""
    k = "probe_mfma"
    out = torch.empty((workgroups * 512,), dtype=torch.float32, device=device)
    _run(k, library("bfloat16").tq_probe_mfma(shape, workgroups, iters, seed, _ptr(out), _stream()))
    return float(workgroups) * 8 * iters * 196608.0
