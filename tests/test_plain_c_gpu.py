"""Every kernel entry point of the library beside its plain C twin (tests/plain_c/plain_kernels.c): the same inputs
go to the GPU through the library's Python face and to the C function on the host, in both activation types, at sizes
that are not the engine's (odd widths, head counts and groups, rows that fill no tile, scrambled pages)."""
from __future__ import annotations

import math

import numpy as np
import pytest
import torch

import plain_c_twins as C

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
ACTS = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def ops():
    from turboquant_cpp_amd.csrc import ops as _ops
    for a in ACTS:
        _ops.library(a)
    return _ops


def adt(act):
    return torch.float32 if act == "float32" else torch.bfloat16


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(shape, generator=g)).to(dtype)


def close(got, want, act, scale=1.0):
    """The bound of a kernel against sums in double: rounding of float sums, or of bfloat16 operands and results."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    bound = (2e-5 if act == "float32" else 2e-2) * scale * max(1.0, np.abs(want).max())
    assert np.abs(got - want).max() <= bound, (np.abs(got - want).max(), bound)


def host(t):
    return t.detach().float().cpu().numpy()


@pytest.mark.parametrize("act", ACTS)
def test_embedding_soft_cap_and_rows(ops, act):
    table = rnd((37, 50), adt(act), 1)
    tokens = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32)
    assert np.array_equal(host(ops.embed(tokens.to(DEV), table.to(DEV), act, scale=1.5)), C.embed(tokens, host(table), 1.5))
    x = rnd((3, 77), torch.float32, 2, 40.0)
    close(host(ops.softcap(x.to(DEV).clone(), 30.0, act)), C.softcap(x, 30.0), "float32")
    state = rnd((9, 130), torch.float32, 3)
    idx = torch.tensor([8, 2, 5], dtype=torch.int32)
    assert np.array_equal(host(ops.gather_rows(state.to(DEV), idx.to(DEV), act)),
                          C.move_rows(host(state), idx, np.zeros((3, 130), np.float32), scatter=False))
    rows, dst = rnd((3, 130), torch.float32, 4), state.to(DEV).clone()
    ops.scatter_rows(dst, idx.to(DEV), rows.to(DEV), act)
    assert np.array_equal(host(dst), C.move_rows(host(rows), idx, host(state).copy(), scatter=True))


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("T,H,S", [(1, 50, 0), (5, 136, 2), (3, 2052, 5)])
def test_residual_sum_and_norm(ops, act, T, H, S):
    x, w = rnd((T, H), torch.float32, 5), rnd((H,), adt(act), 6)
    delta = rnd((S, T, H), torch.float32, 7) if S else None
    xd = x.to(DEV).clone()
    got_act, got32 = ops.add_rmsnorm(xd, None if delta is None else delta.to(DEV), w.to(DEV), 1e-5, act, want_f32=True)
    want_x, want = C.add_rmsnorm(x, delta, host(w), 1e-5)
    close(host(xd), want_x, "float32")
    close(host(got32), want, "float32", 4)
    close(host(got_act), want, act)
    rows = torch.tensor([T - 1, 0], dtype=torch.int32)
    xd = x.to(DEV).clone()
    picked, _ = ops.add_rmsnorm(xd, None if delta is None else delta.to(DEV), w.to(DEV), 1e-5, act, rows=rows.to(DEV))
    assert torch.equal(xd.cpu(), x)
    close(host(picked), C.add_rmsnorm(x, delta, host(w), 1e-5, rows=rows)[1], act)


@pytest.mark.parametrize("act", ACTS)
def test_per_head_norm_and_the_gate_of_a_pair(ops, act):
    nh, nkv, hd, T = 5, 1, 48, 7
    qkv, wq, wk = rnd((T, (nh + 2 * nkv) * hd), torch.float32, 8), rnd((hd,), adt(act), 9), rnd((hd,), adt(act), 10)
    got = ops.head_rmsnorm(qkv.to(DEV).clone(), wq.to(DEV), wk.to(DEV), 1e-6, nh, nkv, hd, act)
    close(host(got), C.head_rmsnorm(qkv, host(wq), host(wk), 1e-6, nh, nkv, hd), "float32", 4)
    got = ops.head_rmsnorm(qkv.to(DEV).clone(), None, wk.to(DEV), 1e-6, nh, nkv, hd, act)
    close(host(got), C.head_rmsnorm(qkv, None, host(wk), 1e-6, nh, nkv, hd), "float32", 4)
    if act == "bfloat16":          # the pass behind a pair that came out of one product is the bfloat16 path's
        from turboquant_cpp_amd.csrc.ops import _ptr, _run, _stream, library
        gu = rnd((6, 2 * 88), torch.float32, 11).to(DEV)
        for gate in (0, 1, 2):
            out = torch.empty((6, 88), dtype=torch.bfloat16, device=DEV)
            _run("gated_act", library(act).tq_gated_act(_ptr(gu), 2 * 88, _ptr(out), 6, 88, gate, _stream()))
            close(host(out), C.gated_act(host(gu), 88, gate), act)


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("M,N,K", [(1, 40, 72), (9, 136, 200), (70, 88, 136), (300, 200, 64)])
def test_products(ops, act, M, N, K):
    a, w, w2 = rnd((M, K), adt(act), 12), rnd((N, K), adt(act), 13, 0.2), rnd((N, K), adt(act), 14, 0.2)
    b = rnd((N,), adt(act), 15)
    ad, wd, w2d = a.to(DEV), w.to(DEV), w2.to(DEV)
    s = math.sqrt(K)
    close(host(ops.gemm(ad, wd, act)), C.gemm(host(a), host(w)), act, s / 4)
    close(host(ops.gemm(ad, wd, act, bias=b.to(DEV))), C.gemm(host(a), host(w), bias=host(b)), act, s / 4)
    for name, gate in (("silu", 0), ("gelu_tanh", 1), ("relu2", 2)):
        got = ops.gemm(ad, wd, act, w2=w2d, out_act=True, activation=name)
        close(host(got), C.gemm(host(a), host(w), w2=host(w2), gate=gate), act, s / 2)
    parts = ops.gemm(ad, wd, act, partial_sums=True)
    close(host(parts.sum(0)), C.gemm(host(a), host(w)), act, s / 4)


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("T,E,k,H,I,unit", [(9, 7, 3, 136, 88, 16), (150, 6, 2, 64, 200, 64), (260, 5, 3, 192, 320, 64 + 1024)])
def test_choice_order_and_products_of_experts(ops, act, T, E, k, H, I, unit):
    """The router's choice, the order of pairs, the two products over experts and the weighted sum: each kernel's
    result against its twin's, fed with the same inputs."""
    rows, unit = unit, unit % 1024
    if rows != unit and act != "bfloat16":
        pytest.skip("units two at a time are the bfloat16 matrix-core product's")
    x32 = rnd((T, H), torch.float32, 16)
    wr, sw = rnd((E, H), adt(act), 17), rnd((1, H), adt(act), 18, 0.1)
    for renorm in (True, False):
        ids, weights, gate = ops.router_topk(x32.to(DEV), wr.to(DEV), sw.to(DEV), k, renorm, act)
        c_ids, c_w, c_gate, _ = C.router_topk(x32, host(wr), host(sw).reshape(-1), k, renorm)
        assert np.array_equal(ids.cpu().numpy(), c_ids)
        close(host(weights), c_w, "float32", 4)
        close(host(gate), c_gate, "float32", 4)
    st, slot, te, nt = ops.moe_align(ids, E, unit, act)
    c_st, c_slot, c_te, c_nt = C.moe_align(c_ids, E, unit)
    units, items = c_nt.tolist()
    half = c_te.size // 2
    assert nt.tolist() == [units, items]
    assert np.array_equal(st.cpu().numpy(), c_st) and np.array_equal(slot.cpu().numpy(), c_slot)
    assert np.array_equal(te.cpu().numpy()[:units], c_te[:units])
    assert np.array_equal(te.cpu().numpy()[half:half + items], c_te[half:half + items])
    x = x32.to(adt(act))
    wg, wu, wd = (rnd(s, adt(act), 19 + i, 0.2) for i, s in enumerate(((E, I, H), (E, I, H), (E, H, I))))
    h = ops.gemm(x.to(DEV), wg.to(DEV), act, w2=wu.to(DEV), out_act=True, a_rows=st, tile_group=te, n_tiles=nt, tile_rows=rows)
    c_h = C.gemm(host(x), host(wg), w2=host(wu), a_rows=c_st, tile_group=c_te, n_units=units, tile_rows=unit)
    live = c_st >= 0
    close(host(h)[live], c_h[live], act, math.sqrt(H) / 2)
    y = ops.gemm(h, wd.to(DEV), act, a_rows=st, tile_group=te, n_tiles=nt, tile_rows=rows, gather=False)
    c_y = C.gemm(np.nan_to_num(host(h)), host(wd), a_rows=c_st, gather=False, tile_group=c_te, n_units=units, tile_rows=unit)
    close(host(y)[live], c_y[live], act, math.sqrt(I) / 4)
    shared = rnd((2, T, H), torch.float32, 23)
    y0 = torch.nan_to_num(y)
    got = ops.moe_combine(y0, slot, weights, shared.to(DEV), gate, act)
    want = C.moe_combine(host(y0), c_slot, host(weights), host(shared), host(gate), T, H)
    close(host(got)[0], want, "float32", 4)


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("nh,nkv,hd,window,pairing,rotary", [(3, 1, 48, None, 0, 48), (4, 2, 64, 20, 0, 64), (6, 3, 32, 70, 1, 16),
                                                            (5, 5, 128, None, 0, 128)])
def test_rotation_cache_and_attention(ops, act, nh, nkv, hd, window, pairing, rotary):
    """Prompts of unequal lengths written into scrambled pages and attended to, then one more token each: the
    rotation and the cache write, the kernel for whole prompts, the kernel for single tokens and the plain one, each
    against the twin, which reads the pages that the twin of the write filled."""
    page, layers, layer = 64, 2, 1
    lens = [150, 1, 67]
    n_pages = [-(-(n + 1) // page) for n in lens]
    order = torch.randperm(sum(n_pages) + 3, generator=torch.Generator().manual_seed(24)).tolist()
    table = torch.full((len(lens) + 1, max(n_pages)), -1, dtype=torch.int32)
    slots, at = [3, 1, 2], 0
    for s, n in zip(slots, n_pages):
        table[s, :n] = torch.tensor(order[at:at + n], dtype=torch.int32)
        at += n
    stride, offset = layers * nkv * page * hd, layer * nkv * page * hd
    total = (sum(n_pages) + 3) * stride
    kd, vd = (torch.zeros(total, dtype=adt(act), device=DEV) for _ in range(2))
    kc, vc = (np.zeros(total, np.float32) for _ in range(2))
    from plain_qwen2moe import rope_frequencies
    inv_freq = torch.from_numpy(rope_frequencies(rotary, 10000.0))
    scale = 1.0 / math.sqrt(hd)
    width = (nh + 2 * nkv) * hd
    bias = rnd((width,), torch.float32, 25)

    def step(new, start, seed):
        T = sum(new)
        qkv = rnd((T, width), torch.float32, seed)
        positions = torch.cat([torch.arange(s, s + n) for s, n in zip(start, new)]).to(torch.int32)
        slot_of = torch.cat([torch.full((n,), s) for n, s in zip(new, slots)]).to(torch.int32)
        cu = torch.tensor([0] + list(np.cumsum(new)), dtype=torch.int32)
        runs = dict(cu_seqlens=cu.to(DEV), slots=torch.tensor(slots, dtype=torch.int32, device=DEV),
                    start=torch.tensor(start, dtype=torch.int32, device=DEV), max_new=max(new),
                    max_end=max(s + n for s, n in zip(start, new)), decode=all(n == 1 for n in new))
        args = (positions.to(DEV), slot_of.to(DEV), table.to(DEV))
        q = ops.rope_kv_write(qkv.to(DEV), *args, inv_freq.to(DEV), pairing, rotary, kd, vd, offset, page, stride, nh, nkv,
                              hd, act, runs=runs, bias=bias.to(DEV))
        c_q = C.rope_kv_write(qkv, bias, positions, slot_of, table, inv_freq, pairing, rotary, kc, vc, offset, page, stride,
                              nh, nkv, hd)
        close(host(q), c_q, act, 4)
        want = C.attention(np.asarray(host(q)), kc, vc, positions, slot_of, table, offset, page, stride, nh, nkv, hd, window, scale)
        for how in (runs, None):          # the kernels that work on runs of positions, and the token-by-token one
            got = ops.attention(q, kd, vd, offset, *args, page, stride, nh, nkv, hd, window, scale, act, runs=how)
            close(host(got), want, act, 4)

    step(lens, [0, 0, 0], 26)
    close(host(kd), kc, act, 4)
    close(host(vd), vc, act, 4)
    step([1, 1, 1], lens, 27)


def test_sampling(ops):
    act = "float32"
    R, V = 5, 1031
    logits = rnd((R, V), torch.float32, 28, 3.0)
    assert np.array_equal(ops.argmax(logits.to(DEV), act).cpu().numpy(), C.argmax(logits))
    targets = torch.tensor([7, 0, V - 1, 500, 3], dtype=torch.int32)
    close(host(ops.nll(logits.to(DEV), targets.to(DEV), act)), C.nll(logits, targets), "float32", 4)
    recent = torch.randint(0, V, (R, 12), generator=torch.Generator().manual_seed(29)).to(torch.int32)
    recent[0, :3] = 4                          # a token that occurs three times is penalised three times
    counts = torch.tensor([12, 0, 5, 1, 12], dtype=torch.int32)
    ld = logits.to(DEV).clone()
    ops.rep_penalty(ld, recent.to(DEV), counts.to(DEV), 1.3, act)
    close(host(ld), C.rep_penalty(logits, recent, counts, 1.3), "float32")
    # the draw: the token whose stretch of the running sum holds u * (sum of the kept probabilities); a draw within
    # rounding of a border between two tokens may fall on either, so such draws are left out
    state = np.array([77], np.uint64)
    for temperature, top_p in ((0.7, 0.9), (1.3, 0.5), (1.0, 1.0)):
        u = torch.tensor([C.next_uniform(state) for _ in range(R)], dtype=torch.float32)
        got = ops.sample_topp(logits.to(DEV), temperature, top_p, u.to(DEV), act).cpu().tolist()
        for r in range(R):
            near = {C.sample_topp_u(logits[r], temperature, top_p, float(u[r]) * f) for f in (1 - 1e-4, 1.0, 1 + 1e-4)}
            assert got[r] in near, (temperature, top_p, r, got[r], near)
