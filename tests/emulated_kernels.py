"""Stand-ins for the HIP kernels, for tests that run where no GPU is.

Each function has the signature and the data contract of its namesake in ``csrc/ops.py`` (packed rows, page
tables indexed by slot, pairs ordered by expert) and computes it with torch on the CPU.  Tests put them in
place of the kernels (``monkeypatch``) to check what surrounds the kernels without a GPU: the cache's
pages and tables, the packing of a step, the order of layers, the generation loop.  They are no part of
the library: the library itself has no CPU path.
"""
from __future__ import annotations

import math

import torch

ACT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def embed(tokens, table, act, scale=1.0):
    return table[tokens.long()].float() * scale


def softcap(logits, cap, act):
    return logits.copy_(cap * torch.tanh(logits / cap))


def add_rmsnorm(x, delta, weight, eps, act, rows=None, want_act=True, want_f32=False):
    if hasattr(delta, "pair_slot"):      # a sum over experts that is still to be done
        delta = moe_combine(delta.y, delta.pair_slot, delta.weights, delta.dense, delta.gate, act)
    v = x if delta is None else x + delta.sum(dim=0)
    if rows is None:
        x.copy_(v)
    else:
        v = v[rows.long()]
    ss = (v * v).sum(dim=-1, keepdim=True) / v.shape[-1] + eps
    o = v * (1.0 / torch.sqrt(ss)) * weight.float()
    return (o.to(ACT[act]) if want_act else None), (o if want_f32 else None)


def _rows_of(table, slot, positions, page_size):
    pages = table[slot, (positions // page_size).long()].long()
    assert (pages >= 0).all(), "a position without a page is read or written"
    return pages, positions % page_size


def rope_kv_write(qkv, positions, slot_of_token, block_table, inv_freq, pairing, rotary_dim, k_pages, v_pages,
                  layer_offset, page_size, page_stride, num_heads, num_kv_heads, head_dim, act, runs=None):
    T = positions.numel()
    x = qkv.view(T, num_heads + 2 * num_kv_heads, head_dim)
    ang = positions.float()[:, None] * inv_freq[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    qk = x[:, :num_heads + num_kv_heads].clone()
    half = rotary_dim // 2
    if pairing == 0:
        a, b = qk[..., :half].clone(), qk[..., half:rotary_dim].clone()
        qk[..., :half], qk[..., half:rotary_dim] = a * cos - b * sin, a * sin + b * cos
    else:
        a, b = qk[..., 0:rotary_dim:2].clone(), qk[..., 1:rotary_dim:2].clone()
        qk[..., 0:rotary_dim:2], qk[..., 1:rotary_dim:2] = a * cos - b * sin, a * sin + b * cos
    q = qk[:, :num_heads].reshape(T, num_heads * head_dim).to(ACT[act])
    if k_pages is not None:
        k, v = qk[:, num_heads:].to(ACT[act]), x[:, num_heads + num_kv_heads:].to(ACT[act])
        for t in range(T):
            p = int(positions[t])
            page = int(block_table[int(slot_of_token[t]), p // page_size])
            assert page >= 0, "a position without a page is written"
            for h in range(num_kv_heads):
                o = page * page_stride + layer_offset + (h * page_size + p % page_size) * head_dim
                k_pages[o:o + head_dim] = k[t, h]
                ov = page * page_stride + layer_offset + h * page_size * head_dim + p % page_size
                v_pages[ov:ov + head_dim * page_size:page_size] = v[t, h]      # values lie [hd][row]
    return q


def attention(q, k_pages, v_pages, layer_offset, positions, slot_of_token, block_table, page_size, page_stride,
              num_heads, num_kv_heads, head_dim, window, scale, act, runs=None):
    T = positions.numel()
    out = torch.empty_like(q)
    qf = q.float().view(T, num_heads, head_dim)
    for t in range(T):
        p, slot = int(positions[t]), int(slot_of_token[t])
        lo = max(0, p - window + 1) if window else 0
        js = torch.arange(lo, p + 1)
        pages = block_table[slot, (js // page_size).long()].long()
        assert (pages >= 0).all(), "a position without a page is read"
        for h in range(num_heads):
            kvh = h // (num_heads // num_kv_heads)
            base = pages * page_stride + layer_offset + (kvh * page_size + js % page_size) * head_dim
            K = k_pages[base[:, None] + torch.arange(head_dim)[None, :]].float()
            vbase = pages * page_stride + layer_offset + kvh * page_size * head_dim + js % page_size
            V = v_pages[vbase[:, None] + page_size * torch.arange(head_dim)[None, :]].float()
            s = (K @ qf[t, h]) * scale
            pr = torch.softmax(s, dim=0)
            out[t, h * head_dim:(h + 1) * head_dim] = (pr @ V).to(out.dtype)
    return out


def gemm(a, w, act, bias=None, w2=None, out_act=False, a_rows=None, tile_group=None, n_tiles=None, tile_rows=None,
         gather=True, partial_sums=False, activation="silu"):
    gate = {"silu": torch.nn.functional.silu, "relu2": lambda v: torch.relu(v) ** 2,
            "gelu_tanh": lambda v: torch.nn.functional.gelu(v, approximate="tanh")}[activation]
    if partial_sums:
        return gemm(a, w, act, bias=bias).unsqueeze(0)
    af = a.float()
    if tile_group is None:
        src = af if a_rows is None else af[a_rows.long()]
        y = src @ w.float().T
        if bias is not None:
            y = y + bias.float()
        if w2 is not None:
            y = gate(y) * (src @ w2.float().T)
    else:
        P, N = a_rows.numel(), w.shape[1]
        tile_rows %= 1024        # (units of 64 taken two at a time give what unit by unit gives)
        y = torch.full((P, N), float("nan"))
        for tile in range(int(n_tiles[0])):
            g = int(tile_group[tile])
            for m in range(tile * tile_rows, (tile + 1) * tile_rows):
                r = int(a_rows[m])
                if r < 0:
                    continue
                row = af[r] if gather else af[m]
                v = w[g].float() @ row
                if w2 is not None:
                    v = gate(v) * (w2[g].float() @ row)
                y[m] = v
    return y.to(ACT[act]) if out_act else y


def router_topk(x32, router, shared_scale, top_k, renormalize, act):
    logits = x32 @ router.float().T
    T, E = logits.shape
    ids = torch.empty((T, top_k), dtype=torch.int32)
    weights = torch.empty((T, top_k), dtype=torch.float32)
    for t in range(T):
        used, chosen = set(), []
        for _ in range(top_k):
            best, bv = -1, -math.inf
            for e in range(E):
                if e not in used and logits[t, e].item() >= bv:
                    best, bv = e, logits[t, e].item()
            used.add(best)
            chosen.append(best)
        ids[t] = torch.tensor(chosen, dtype=torch.int32)
        sel = logits[t, chosen]
        weights[t] = torch.softmax(sel, 0) if renormalize else torch.softmax(logits[t], 0)[chosen]
    gate = None
    if shared_scale is not None:
        gate = torch.sigmoid(x32 @ shared_scale.float().reshape(-1))
    return ids, weights, gate


def moe_align(ids, num_experts, unit, act):
    T, topk = ids.shape
    flat = ids.reshape(-1).tolist()
    n_pairs = len(flat)
    cap = n_pairs + min(num_experts, n_pairs) * (unit - 1)
    cap = (cap + unit - 1) // unit * unit
    sorted_token = torch.full((cap,), -1, dtype=torch.int32)
    pair_slot = torch.empty((T, topk), dtype=torch.int32)
    tile_expert = torch.zeros((2 * (cap // unit),), dtype=torch.int32)      # row tiles, then items of two row tiles
    row = tile = item = 0
    for e in range(num_experts):
        mine = [i for i, x in enumerate(flat) if x == e]
        for j, i in enumerate(mine):
            sorted_token[row + j] = i // topk
            pair_slot.view(-1)[i] = row + j
        nt = -(-len(mine) // unit)
        tile_expert[tile:tile + nt] = e
        for first in range(tile, tile + nt, 2):
            tile_expert[cap // unit + item] = first
            item += 1
        tile += nt
        row += nt * unit
    return sorted_token, pair_slot, tile_expert, torch.tensor([tile, item], dtype=torch.int32)


def moe_combine(y, pair_slot, weights, shared, shared_gate, act):
    T, topk = pair_slot.shape
    out = torch.zeros((T, y.shape[1]))
    for j in range(topk):
        out += weights[:, j:j + 1] * y[pair_slot[:, j].long()]
    if shared is not None:
        sh = shared.sum(dim=0)
        out += sh * (shared_gate[:, None] if shared_gate is not None else 1.0)
    return out.unsqueeze(0)


def argmax(logits, act):
    return torch.argmax(logits, dim=-1).to(torch.int32)


def rep_penalty(logits, recent, counts, penalty, act):
    for r in range(logits.shape[0]):
        for j in range(min(int(counts[r]), recent.shape[1])):
            t = int(recent[r, j])
            if 0 <= t < logits.shape[1]:
                logits[r, t] = logits[r, t] / penalty if logits[r, t] > 0 else logits[r, t] * penalty


def sample_topp(logits, temperature, top_p, uniforms, act):
    out = []
    for r in range(logits.shape[0]):
        l = logits[r]
        mx = l.max()
        keep = l >= mx - 16.0 * temperature
        p = torch.where(keep, torch.exp((l - mx) / temperature), torch.zeros_like(l))
        p = p / p.sum()
        sp, si = torch.sort(p, descending=True, stable=True)
        cum = torch.cumsum(sp, 0)
        n_top = int((cum >= top_p).nonzero()[0]) + 1 if (cum >= top_p).any() else len(sp)
        rr = float(uniforms[r]) * float(cum[n_top - 1])
        hit = (cum[:n_top] >= rr).nonzero()
        out.append(int(si[int(hit[0])]) if len(hit) else int(si[0]))
    return torch.tensor(out, dtype=torch.int32)


def gemm_pair(first, second, act):
    return gemm(first.pop("a"), first.pop("w"), act, **first), gemm(second.pop("a"), second.pop("w"), act, **second)


def route(x32, router, shared_scale, top_k, renormalize, unit, act):
    ids, weights, gate = router_topk(x32, router, shared_scale, top_k, renormalize, act)
    return (ids, weights, gate) + tuple(moe_align(ids, router.shape[0], unit, act))


def head_rmsnorm(qkv, q_weight, k_weight, eps, num_heads, num_kv_heads, head_dim, act):
    x = qkv.view(qkv.shape[0], num_heads + 2 * num_kv_heads, head_dim)
    for lo, hi, w in ((0, num_heads, q_weight), (num_heads, num_heads + num_kv_heads, k_weight)):
        if w is not None:
            h = x[:, lo:hi].float()
            x[:, lo:hi] = h * torch.rsqrt((h * h).mean(-1, keepdim=True) + eps) * w.float()
    return qkv


def expert_tile_rows(n_pairs, num_experts, act, a, w):
    return 16 if n_pairs <= 12 * num_experts else 64


def qkv_rope_write(a, qkv_weight, qkv_bias, positions, seq_of_token, block_table, inv_freq, pairing, rotary_dim, k_pages,
                   v_pages, layer_offset, page_size, page_stride, num_heads, num_kv_heads, head_dim, act, runs=None):
    qkv = gemm(a, qkv_weight, act, bias=qkv_bias)
    return rope_kv_write(qkv, positions, seq_of_token, block_table, inv_freq, pairing, rotary_dim, k_pages, v_pages,
                         layer_offset, page_size, page_stride, num_heads, num_kv_heads, head_dim, act, runs=runs)


def gather_rows(src, index, act):
    return src.index_select(0, index.long())


def scatter_rows(dst, index, rows, act):
    dst.index_copy_(0, index.long(), rows)


def install(monkeypatch):
    """Puts the stand-ins in place of the kernels for one test."""
    from turboquant_cpp_amd.csrc import ops
    for name in ("embed", "add_rmsnorm", "rope_kv_write", "qkv_rope_write", "attention", "gemm", "router_topk", "moe_align", "route", "gemm_pair",
                 "head_rmsnorm", "expert_tile_rows", "moe_combine", "argmax", "rep_penalty", "sample_topp", "softcap", "gather_rows", "scatter_rows"):
        monkeypatch.setattr(ops, name, globals()[name])
