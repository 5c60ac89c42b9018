"""The plain C twins of the kernels (tests/plain_c/plain_kernels.c) against the plain model's functions in Python: two
writings of the reference's formulas, in two languages and with different data contracts (whole sequences there;
packed rows, pages and tables, pairs ordered by expert here), that must agree.  Runs on the CPU."""
from __future__ import annotations

import math

import numpy as np
import pytest
import torch

import plain_c_twins as C
import plain_qwen2moe as P


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float64) * scale).to(torch.float32)


def close(got, want, tol=2e-6):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.abs(got - want).max() <= tol * max(1.0, np.abs(want).max()), np.abs(got - want).max()


def test_embedding_soft_cap_and_rows():
    table = rnd(11, 6, seed=1)
    close(C.embed([3, 0, 10], table, 2.5), table[[3, 0, 10]].numpy() * 2.5)
    x = rnd(3, 7, seed=2, scale=40.0)
    close(C.softcap(x, 30.0), 30.0 * np.tanh(x.numpy().astype(np.float64) / 30.0))
    src = rnd(5, 4, seed=3).numpy()
    got = C.move_rows(src, [4, 1], np.zeros((2, 4), np.float32), scatter=False)
    assert np.array_equal(got, src[[4, 1]])
    dst = np.zeros((5, 4), np.float32)
    C.move_rows(src[:2], [3, 0], dst, scatter=True)
    assert np.array_equal(dst[[3, 0]], src[:2]) and not dst[[1, 2, 4]].any()


@pytest.mark.parametrize("T,H,S", [(1, 5, 0), (4, 24, 1), (3, 130, 3)])
def test_residual_sum_and_norm(T, H, S):
    x, w = rnd(T, H, seed=4), rnd(H, seed=5)
    delta = rnd(S, T, H, seed=6) if S else None
    summed, normed = C.add_rmsnorm(x, delta, w, 1e-5)
    want_x = x.double() + (delta.double().sum(0) if S else 0.0)
    close(summed, want_x)
    close(normed, P.rmsnorm(want_x, w.double(), 1e-5))
    rows = [T - 1, 0]
    same_x, picked = C.add_rmsnorm(x, delta, w, 1e-5, rows=rows)
    assert np.array_equal(same_x, x.numpy())          # with rows picked the stream is left alone
    close(picked, P.rmsnorm(want_x, w.double(), 1e-5)[rows])


def test_per_head_norm():
    nh, nkv, hd, T = 3, 1, 8, 4
    qkv, wq, wk = rnd(T, (nh + 2 * nkv) * hd, seed=7), rnd(hd, seed=8), rnd(hd, seed=9)
    got = C.head_rmsnorm(qkv, wq, wk, 1e-6, nh, nkv, hd).reshape(T, nh + 2 * nkv, hd)
    x = qkv.double().reshape(T, nh + 2 * nkv, hd)
    close(got[:, :nh], P.rmsnorm(x[:, :nh], wq.double(), 1e-6))
    close(got[:, nh:nh + nkv], P.rmsnorm(x[:, nh:nh + nkv], wk.double(), 1e-6))
    assert np.array_equal(got[:, nh + nkv:], x[:, nh + nkv:].float().numpy())


def test_products():
    a, w, w2, b = rnd(5, 12, seed=10), rnd(7, 12, seed=11), rnd(7, 12, seed=12), rnd(7, seed=13)
    close(C.gemm(a, w), P.matvec_rows(w.double(), a.double()))
    close(C.gemm(a, w, bias=b), P.matvec_rows(w.double(), a.double()) + b.double())
    gate, up = P.matvec_rows(w.double(), a.double()), P.matvec_rows(w2.double(), a.double())
    close(C.gemm(a, w, w2=w2), P.silu(gate) * up)
    close(C.gated_act(torch.cat([gate, up], dim=1).float(), 7, 0), P.silu(gate) * up)
    close(C.gated_act(torch.cat([gate, up], dim=1).float(), 7, 2), torch.relu(gate) ** 2 * up)


def pages_for(lens, page_size, nkv, hd, layers, seed):
    """Pages handed out in a scrambled order: (table [slots, width], page_stride, number of pages)."""
    need = [-(-n // page_size) for n in lens]
    order = torch.randperm(sum(need) + 2, generator=torch.Generator().manual_seed(seed)).tolist()
    table = np.full((len(lens), max(need)), -1, np.int32)
    at = 0
    for s, n in enumerate(need):
        table[s, :n] = order[at:at + n]
        at += n
    return table, layers * nkv * page_size * hd, sum(need) + 2


@pytest.mark.parametrize("pairing", ["half", "interleaved"])
@pytest.mark.parametrize("rotary", [8, 4])
def test_rotation_cache_and_attention(pairing, rotary):
    """Three sequences of unequal lengths packed into one step, their keys and values written into scrambled pages of
    a cache of two layers, then every token's attention read back from the pages: against the plain functions, which
    take one whole sequence at a time."""
    nh, nkv, hd, page, theta = 4, 2, 8, 4, 10000.0
    lens, window = [9, 1, 6], 5
    table, stride, n_pages = pages_for(lens, page, nkv, hd, 2, seed=14)
    offset = nkv * page * hd          # the second layer of a page
    k_pages, v_pages = (np.zeros((n_pages * stride,), np.float32) for _ in range(2))
    qkv = rnd(sum(lens), (nh + 2 * nkv) * hd, seed=15)
    bias = rnd((nh + 2 * nkv) * hd, seed=16)
    positions = np.concatenate([np.arange(n) for n in lens]).astype(np.int32)
    slot_of = np.concatenate([np.full(n, s) for s, n in enumerate(lens)]).astype(np.int32)
    inv_freq = P.rope_frequencies(rotary, theta)
    q = C.rope_kv_write(qkv, bias, positions, slot_of, table, inv_freq, 0 if pairing == "half" else 1, rotary, k_pages,
                        v_pages, offset, page, stride, nh, nkv, hd)
    got = C.attention(q, k_pages, v_pages, positions, slot_of, table, offset, page, stride, nh, nkv, hd, window,
                      1.0 / math.sqrt(hd))
    at = 0
    for n in lens:
        x = (qkv[at:at + n].double() + bias.double()).reshape(n, nh + 2 * nkv, hd)
        rq = P.rope(x[:, :nh], list(range(n)), theta, pairing, rotary)
        rk = P.rope(x[:, nh:nh + nkv], list(range(n)), theta, pairing, rotary)
        close(q[at:at + n].reshape(n, nh, hd), rq, 3e-6)
        close(got[at:at + n].reshape(n, nh, hd), P.attention(rq, rk, x[:, nh + nkv:], window=window), 3e-6)
        at += n
    assert not k_pages.reshape(n_pages, 2, -1)[:, 0].any()          # the first layer's half of every page is untouched


@pytest.mark.parametrize("renorm", [True, False])
def test_router_choice_and_weights(renorm):
    T, H, E, k = 6, 16, 7, 3
    x, wr, sw = rnd(T, H, seed=17), rnd(E, H, seed=18), rnd(H, seed=19)
    wr[5] = wr[2]                      # two experts that always tie: the higher index wins
    ids, weights, gate, logits = C.router_topk(x, wr, sw, k, renorm)
    for t in range(T):
        want_ids, want_w = P.route(x[t].double(), wr.double(), k, renorm)
        assert ids[t].tolist() == want_ids
        close(weights[t], want_w)
        assert 2 not in ids[t].tolist() or 5 in ids[t].tolist()
    close(gate, 1.0 / (1.0 + torch.exp(-(x.double() @ sw.double()))))
    close(logits, x.double() @ wr.double().T)
    # the reference's own vector (/root/reference/tests/test_gguf_moe.cpp:273-304): experts 3 and 5 of 8
    vec = np.zeros((8, 4), np.float32)
    vec[3, 0], vec[5, 0], vec[0, 0] = 10.0, 8.0, 1.0
    ids, weights, _, _ = C.router_topk(np.eye(1, 4, dtype=np.float32), vec, None, 2, True)
    assert ids[0].tolist() == [3, 5]
    close(weights[0], [0.880797, 0.119203], 1e-6)


def test_experts_through_the_order_of_pairs():
    """The whole feed-forward over experts as the kernels cut it (choice, order of pairs in units of rows, the gated
    product over gathered rows, the second product row for row, the weighted sum with the gated shared expert)
    against the plain model's one function."""
    T, H, E, k, I, Is, unit = 9, 12, 5, 2, 10, 14, 4
    x = rnd(T, H, seed=20)
    w = {"router": rnd(E, H, seed=21).double(), "shared_scale": rnd(1, H, seed=22).double(),
         "experts": [{"gate": rnd(I, H, seed=30 + e).double(), "up": rnd(I, H, seed=40 + e).double(),
                      "down": rnd(H, I, seed=50 + e).double()} for e in range(E)],
         "shared": {"gate": rnd(Is, H, seed=23).double(), "up": rnd(Is, H, seed=24).double(), "down": rnd(H, Is, seed=25).double()}}
    ids, weights, gate, _ = C.router_topk(x, w["router"], w["shared_scale"].reshape(-1), k, False)
    sorted_token, pair_slot, tile_expert, (units, items) = C.moe_align(ids, E, unit)
    # every pair has its row, an expert's rows lie together in order of token, its units are listed two at a time
    assert sorted(pair_slot.reshape(-1).tolist()) == [r for r in range(sorted_token.size) if sorted_token[r] >= 0]
    for t in range(T):
        for j in range(k):
            r = pair_slot[t, j]
            assert sorted_token[r] == t and tile_expert[r // unit] == ids[t, j]
    assert tile_expert[:units].tolist() == sorted(tile_expert[:units].tolist())
    firsts = tile_expert[sorted_token.size // unit:][:items].tolist()
    assert firsts == [u for e in range(E) for u in [i for i in range(units) if tile_expert[i] == e][::2]]
    stack = lambda name: torch.stack([e[name] for e in w["experts"]])
    h = C.gemm(x, stack("gate"), w2=stack("up"), a_rows=sorted_token, tile_group=tile_expert, n_units=units, tile_rows=unit)
    y = C.gemm(np.nan_to_num(h), stack("down"), a_rows=sorted_token, gather=False, tile_group=tile_expert, n_units=units,
               tile_rows=unit)
    hs = C.gemm(x, w["shared"]["gate"], w2=w["shared"]["up"])
    shared = C.gemm(hs, w["shared"]["down"])
    out = C.moe_combine(np.nan_to_num(y), pair_slot, weights, shared[None], gate, T, H)
    close(out, P.moe(x.double(), w, k, False), 5e-6)


def test_sampling():
    logits = rnd(3, 50, seed=26, scale=3.0).numpy()
    assert C.argmax(logits).tolist() == [P.sample_argmax(row) for row in logits]
    flat = np.zeros((1, 9), np.float32)
    assert C.argmax(flat).tolist() == [0]                     # the first maximum wins
    targets = [7, 0, 49]
    want = [-(torch.log_softmax(torch.from_numpy(row).double(), 0)[t]).item() for row, t in zip(logits, targets)]
    close(C.nll(logits, targets), want, 1e-6)
    recent = np.array([[4, 4, 9, -1], [0, 1, 2, 3], [5, 5, 5, 5]], np.int32)
    counts = [3, 0, 4]
    got = C.rep_penalty(logits, recent, counts, 1.3)
    for r in range(3):
        want_row = logits[r].copy()
        P.apply_rep_penalty(want_row, recent[r, :counts[r]].tolist()[::-1], 64, 1.3)
        assert np.array_equal(got[r], want_row)
    # the generator and the draw: the same tokens as the plain model's sampler, draw after draw
    state, rng = np.array([1234], np.uint64), P.PlainRng(1234)
    assert [C.next_uniform(state) for _ in range(5)] == [rng.next() for _ in range(5)]
    state, rng = np.array([99], np.uint64), P.PlainRng(99)
    for step in range(60):
        row = rnd(200, seed=100 + step, scale=2.5).numpy()
        t, p = (0.7, 0.9) if step % 3 else (1.4, 0.5)
        assert C.sample_topp(row, t, p, state) == P.sample_topp(row, t, p, rng), step
    assert C.sample_topp(logits[0], 0.0, 0.9, state) == P.sample_argmax(logits[0])
