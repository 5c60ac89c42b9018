"""The plain C twins of the kernels (``tests/plain_c/plain_kernels.c``), compiled with the host compiler at first use
and called through ctypes on numpy arrays.  No part of the library: only tests load this."""
from __future__ import annotations

import ctypes
import os
import subprocess
import tempfile

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

F, I, L, D, P = ctypes.c_float, ctypes.c_int, ctypes.c_int64, ctypes.c_double, ctypes.c_void_p


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        out = os.path.join(tempfile.mkdtemp(prefix="plain_c_"), "libplain_kernels.so")
        subprocess.check_call(["cc", "-O2", "-shared", "-fPIC", "-o", out, os.path.join(_HERE, "plain_c", "plain_kernels.c"), "-lm"])
        _LIB = ctypes.CDLL(out)
        sig = {
            "pc_embed": [P, P, P, I, I, F],
            "pc_softcap": [P, L, F],
            "pc_move_rows": [P, P, P, I, I, I],
            "pc_moe_combine": [P, P, P, I, P, I, P, P, I, I],
            "pc_add_rmsnorm": [P, P, I, P, F, P, I, P, I, I],
            "pc_head_rmsnorm": [P, P, P, F, I, I, I, I],
            "pc_gated_act": [P, L, P, I, I, I],
            "pc_gemm": [P, L, P, I, P, P, L, P, I, I, P, I, P, I, I, I],
            "pc_rope_kv_write": [P, P, P, P, P, I, P, I, I, P, P, P, L, I, L, I, I, I, I],
            "pc_attention": [P, P, P, P, P, P, I, L, I, L, I, I, I, I, I, F, P],
            "pc_router_topk": [P, P, P, I, I, I, P, P, P, P, I, I],
            "pc_moe_align": [P, I, I, I, I, I, P, P, P, P],
            "pc_argmax": [P, I, I, P],
            "pc_nll": [P, P, I, I, P],
            "pc_rep_penalty": [P, P, P, I, F, I, I],
            "pc_sample_topp": [P, I, F, F, P],
            "pc_sample_topp_u": [P, I, F, F, F],
            "pc_next_uniform": [P],
        }
        for name, args in sig.items():
            getattr(_LIB, name).argtypes = args
            getattr(_LIB, name).restype = None
        _LIB.pc_sample_topp.restype = _LIB.pc_sample_topp_u.restype = I
        _LIB.pc_next_uniform.restype = F
    return _LIB


def f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def i32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.int32))


def ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def embed(tokens, table, scale=1.0):
    tokens, table = i32(tokens), f32(table)
    x = np.empty((tokens.size, table.shape[1]), np.float32)
    lib().pc_embed(ptr(tokens), ptr(table), ptr(x), tokens.size, table.shape[1], scale)
    return x


def softcap(x, cap):
    x = f32(x).copy()
    lib().pc_softcap(ptr(x), x.size, cap)
    return x


def move_rows(src, idx, dst, scatter):
    src, idx = f32(src), i32(idx)
    lib().pc_move_rows(ptr(src), ptr(idx), ptr(dst), idx.size, src.shape[1], int(scatter))
    return dst


def moe_combine(y, pair_slot, weights, shared, gate, T, H):
    y, shared, gate = (None if a is None else f32(a) for a in (y, shared, gate))
    pair_slot, weights = (None if y is None else i32(pair_slot)), (None if y is None else f32(weights))
    out = np.empty((T, H), np.float32)
    lib().pc_moe_combine(ptr(y), ptr(pair_slot), ptr(weights), 0 if y is None else pair_slot.shape[1], ptr(shared),
                         0 if shared is None else shared.shape[0], ptr(gate), ptr(out), T, H)
    return out


def add_rmsnorm(x, delta, w, eps, rows=None):
    """Returns (x after the sum, the normed rows)."""
    x, w = f32(x).copy(), f32(w)
    delta = None if delta is None else f32(delta)
    rows = None if rows is None else i32(rows)
    T, H = x.shape
    out = np.empty((T if rows is None else rows.size, H), np.float32)
    lib().pc_add_rmsnorm(ptr(x), ptr(delta), 0 if delta is None else delta.shape[0], ptr(w), eps, ptr(rows),
                         0 if rows is None else rows.size, ptr(out), T, H)
    return x, out


def head_rmsnorm(qkv, wq, wk, eps, nh, nkv, hd):
    qkv = f32(qkv).copy()
    wq, wk = (None if a is None else f32(a) for a in (wq, wk))
    lib().pc_head_rmsnorm(ptr(qkv), ptr(wq), ptr(wk), eps, qkv.shape[0], nh, nkv, hd)
    return qkv


def gated_act(gu, N, gate):
    gu = f32(gu)
    out = np.empty((gu.shape[0], N), np.float32)
    lib().pc_gated_act(ptr(gu), gu.shape[1], ptr(out), gu.shape[0], N, gate)
    return out


def gemm(a, w, bias=None, w2=None, gate=0, a_rows=None, gather=True, tile_group=None, n_units=0, tile_rows=0):
    a, w = f32(a), f32(w)
    bias, w2 = (None if t is None else f32(t) for t in (bias, w2))
    a_rows, tile_group = (None if t is None else i32(t) for t in (a_rows, tile_group))
    grouped = tile_group is not None
    N, K = (w.shape[1], w.shape[2]) if grouped else w.shape
    M = a.shape[0] if a_rows is None else a_rows.size
    out = np.full((M, N), np.nan, np.float32)
    lib().pc_gemm(ptr(a), a.shape[1], ptr(a_rows), int(gather), ptr(w), ptr(w2), N * K if grouped else 0, ptr(tile_group),
                  n_units, tile_rows, ptr(bias), gate, ptr(out), M, N, K)
    return out


def rope_kv_write(qkv, bias, positions, slot_of_token, table, inv_freq, pairing, rotary_dim, k_pages, v_pages,
                  layer_offset, page_size, page_stride, nh, nkv, hd):
    """Returns the rotated queries; k_pages and v_pages (float32 numpy, flat) are written in place."""
    qkv, positions, slot_of_token, table, inv_freq = f32(qkv), i32(positions), i32(slot_of_token), i32(table), f32(inv_freq)
    bias = None if bias is None else f32(bias)
    T = positions.size
    q = np.empty((T, nh * hd), np.float32)
    lib().pc_rope_kv_write(ptr(qkv), ptr(bias), ptr(positions), ptr(slot_of_token), ptr(table), table.shape[1],
                           ptr(inv_freq), pairing, rotary_dim, ptr(q), ptr(k_pages), ptr(v_pages), layer_offset,
                           page_size, page_stride, T, nh, nkv, hd)
    return q


def attention(q, k_pages, v_pages, positions, slot_of_token, table, layer_offset, page_size, page_stride, nh, nkv, hd,
              window, scale):
    q, positions, slot_of_token, table = f32(q), i32(positions), i32(slot_of_token), i32(table)
    out = np.empty_like(q)
    lib().pc_attention(ptr(q), ptr(k_pages), ptr(v_pages), ptr(positions), ptr(slot_of_token), ptr(table), table.shape[1],
                       layer_offset, page_size, page_stride, positions.size, nh, nkv, hd, window or 0, scale, ptr(out))
    return out


def router_topk(x, wr, shared_w, topk, renorm):
    x, wr = f32(x), f32(wr)
    shared_w = None if shared_w is None else f32(shared_w)
    T, H = x.shape
    E = wr.shape[0]
    ids, weights = np.empty((T, topk), np.int32), np.empty((T, topk), np.float32)
    gate = None if shared_w is None else np.empty((T,), np.float32)
    logits = np.empty((T, E), np.float32)
    lib().pc_router_topk(ptr(x), ptr(wr), ptr(shared_w), E, topk, int(renorm), ptr(ids), ptr(weights), ptr(gate),
                         ptr(logits), T, H)
    return ids, weights, gate, logits


def moe_align(ids, E, unit):
    ids = i32(ids)
    n_pairs, topk = ids.size, ids.shape[1]
    cap = n_pairs + min(E, n_pairs) * (unit - 1)
    cap = (cap + unit - 1) // unit * unit
    sorted_token, pair_slot = np.empty((cap,), np.int32), np.empty(ids.shape, np.int32)
    tile_expert, counts = np.zeros((2 * (cap // unit),), np.int32), np.zeros((2,), np.int32)
    lib().pc_moe_align(ptr(ids), n_pairs, E, topk, unit, cap, ptr(sorted_token), ptr(pair_slot), ptr(tile_expert), ptr(counts))
    return sorted_token, pair_slot, tile_expert, counts


def argmax(logits):
    logits = f32(logits)
    out = np.empty((logits.shape[0],), np.int32)
    lib().pc_argmax(ptr(logits), logits.shape[0], logits.shape[1], ptr(out))
    return out


def nll(logits, targets):
    logits, targets = f32(logits), i32(targets)
    out = np.empty((logits.shape[0],), np.float64)
    lib().pc_nll(ptr(logits), ptr(targets), logits.shape[0], logits.shape[1], ptr(out))
    return out


def rep_penalty(logits, recent, counts, penalty):
    logits, recent, counts = f32(logits).copy(), i32(recent), i32(counts)
    lib().pc_rep_penalty(ptr(logits), ptr(recent), ptr(counts), recent.shape[1], penalty, logits.shape[0], logits.shape[1])
    return logits


def sample_topp(logits, temperature, top_p, state: np.ndarray) -> int:
    """``state``: one uint64 in a numpy array, moved on by the draw."""
    logits = f32(logits)
    return lib().pc_sample_topp(ptr(logits), logits.size, temperature, top_p, ptr(state))


def sample_topp_u(logits, temperature, top_p, uniform: float) -> int:
    logits = f32(logits)
    return lib().pc_sample_topp_u(ptr(logits), logits.size, temperature, top_p, uniform)


def next_uniform(state: np.ndarray) -> float:
    return lib().pc_next_uniform(ptr(state))
