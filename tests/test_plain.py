"""Pins of the plain implementation by what fixes each formula beside the reference's text: vectors that the
reference's own tests hold, special cases that reduce to a library routine, and invariants, each chosen so
that a plausible mistake (a wrong sign or pairing, a norm in the wrong place, a wrong head mapping) fails it."""
import copy
import math
import os

import numpy as np
import pytest
import torch

import plain_qwen2moe as P
from tiny_configs import TINY_A, TINY_B

D = torch.float64


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=D)


# ------------------------------------------------------------------------------------------------ products, norm, activation
def test_matvec_is_rows_times_vector():
    """/root/reference/tests/test_ops.cpp:78-108: [[1,2,3],[4,5,6]] . [1,1,1] = [6,15]; identity."""
    w = torch.tensor([[1.0, 2, 3], [4, 5, 6]], dtype=D)
    assert P.matvec_rows(w, torch.ones(3, dtype=D)).tolist() == [6.0, 15.0]
    x = rnd(5, 7)
    assert torch.equal(P.matvec_rows(torch.eye(7, dtype=D), x), x)
    assert torch.allclose(P.matvec_rows(rnd(4, 7, seed=1), x), x @ rnd(4, 7, seed=1).T)


def test_rmsnorm():
    """/root/reference/tests/test_ops.cpp:220-263: the formula, and unit weight gives unit RMS."""
    x, w = rnd(3, 40), rnd(40, seed=1)
    out = P.rmsnorm(x, torch.ones(40, dtype=D), 1e-12)
    assert torch.allclose((out ** 2).mean(-1).sqrt(), torch.ones(3, dtype=D), atol=1e-9)
    assert torch.allclose(P.rmsnorm(7.5 * x, w, 1e-30), P.rmsnorm(x, w, 1e-30))        # scale of x drops out
    ref = x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + 1e-5) * w
    assert torch.allclose(P.rmsnorm(x, w, 1e-5), ref)
    assert torch.equal(P.rmsnorm(torch.zeros(2, 8, dtype=D), w[:8], 1e-6), torch.zeros(2, 8, dtype=D))   # eps is inside the root
    # eps is added to the mean of squares, not to the sum and not to the root
    one = torch.ones(1, 4, dtype=D)
    assert torch.allclose(P.rmsnorm(one, torch.ones(4, dtype=D), 3.0), one / 2.0)


def test_silu_and_softmax():
    """/root/reference/tests/test_ops.cpp:355-463."""
    x = torch.linspace(-6, 6, 25, dtype=D)
    assert torch.allclose(P.silu(x), torch.nn.functional.silu(x)) and P.silu(torch.zeros(1, dtype=D)).item() == 0.0
    assert bool((P.silu(x[x > 0])[1:] > P.silu(x[x > 0])[:-1]).all())
    s = P.softmax(torch.tensor([1000.0, 1000.0, 999.0], dtype=D))
    assert abs(s.sum().item() - 1) < 1e-12 and bool(((s >= 0) & (s <= 1)).all()) and s[0] == s[1] > s[2]
    assert P.softmax(torch.tensor([3.7], dtype=D)).item() == 1.0
    assert torch.allclose(P.softmax(rnd(4, 9)), torch.softmax(rnd(4, 9), -1))


# ------------------------------------------------------------------------------------------------ rotary encoding
@pytest.mark.parametrize("pairing", ["half", "interleaved"])
def test_rope_basics(pairing):
    """/root/reference/tests/test_ops.cpp:269-349: position 0 is the identity, lengths are kept."""
    x = rnd(4, 3, 16)
    assert torch.equal(P.rope(x, [0, 0, 0, 0], 1e4, pairing), x)
    y = P.rope(x, [42, 1, 7, 1000], 1e4, pairing)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1)) and not torch.allclose(y, x)


def test_rope_sign_and_pairs():
    """One pair by hand: (a, b) -> (a cos - b sin, a sin + b cos) with the angle pos * theta^(-2i/d)."""
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0]]], dtype=D)
    f1 = float(np.float32(1.0) / np.power(np.float32(100.0), np.float32(0.5)))          # i = 1: theta^(-2/4)
    a0, a1 = 3.0 * 1.0, float(np.float32(3.0) * np.float32(f1))
    half = P.rope(x, [3], 100.0, "half")[0, 0]            # pairs (x0, x2) and (x1, x3)
    want = [1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
            1 * math.sin(a0) + 3 * math.cos(a0), 2 * math.sin(a1) + 4 * math.cos(a1)]
    assert torch.allclose(half, torch.tensor(want, dtype=D), atol=1e-12)
    inter = P.rope(x, [3], 100.0, "interleaved")[0, 0]    # pairs (x0, x1) and (x2, x3)
    want = [1 * math.cos(a0) - 2 * math.sin(a0), 1 * math.sin(a0) + 2 * math.cos(a0),
            3 * math.cos(a1) - 4 * math.sin(a1), 3 * math.sin(a1) + 4 * math.cos(a1)]
    assert torch.allclose(inter, torch.tensor(want, dtype=D), atol=1e-12)


def test_rope_pairings_are_one_rotation_under_a_permutation():
    hd = 16
    x = rnd(4, 2, hd)
    perm = torch.tensor([i // 2 + (hd // 2) * (i % 2) for i in range(hd)])
    pos = [0, 3, 17, 100]
    assert torch.allclose(P.rope(x[..., perm], pos, 1e4, "interleaved"), P.rope(x, pos, 1e4, "half")[..., perm], atol=1e-12)


def test_rope_scores_depend_on_distance_only():
    q, k = rnd(1, 1, 32, seed=1), rnd(1, 1, 32, seed=2)
    for pairing in ("half", "interleaved"):
        def score(m, n):
            return (P.rope(q, [m], 1e4, pairing) * P.rope(k, [n], 1e4, pairing)).sum().item()
        assert abs(score(9, 4) - score(25, 20)) < 1e-5 and abs(score(9, 4) - score(4, 9)) > 1e-3


def test_partial_rotation_leaves_the_rest_alone():
    x = rnd(2, 1, 16)
    y = P.rope(x, [5, 9], 1e4, "half", rotary_dim=8)
    assert torch.equal(y[..., 8:], x[..., 8:]) and not torch.allclose(y[..., :8], x[..., :8])


# ------------------------------------------------------------------------------------------------ attention
def test_attention_is_the_library_routine_when_nothing_is_special():
    """No window, equal head counts: causal scaled-dot-product attention of the library."""
    q, k, v = rnd(9, 3, 8, seed=1), rnd(9, 3, 8, seed=2), rnd(9, 3, 8, seed=3)
    lib = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                                           is_causal=True).transpose(0, 1)
    assert torch.allclose(P.attention(q, k, v), lib, atol=1e-12)


def test_attention_special_cases():
    q, k, v = rnd(6, 4, 8, seed=1), rnd(6, 2, 8, seed=2), rnd(6, 2, 8, seed=3)
    out = P.attention(q, k, v)
    assert torch.allclose(out[0, :2], v[0, 0].expand(2, 8)) and torch.allclose(out[0, 2:], v[0, 1].expand(2, 8))
    # heads h map to kv head h / (nh / nkv): the same as full heads with each kv head repeated in place
    rep = P.attention(q, k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1))
    assert torch.allclose(out, rep) and not torch.allclose(out, P.attention(q, k.repeat(1, 2, 1), v.repeat(1, 2, 1)))
    # identical keys: the mean of the values so far
    same = P.attention(q, k[:1].expand(6, 2, 8), v)
    assert torch.allclose(same[3, 0], v[:4, 0].mean(0))
    # a window as long as the sequence is no window; a window of one sees only itself; window w sees w positions
    assert torch.allclose(P.attention(q, k, v, window=6), out)
    assert torch.allclose(P.attention(q, k, v, window=1)[:, :2], v[:, :1].expand(6, 2, 8))
    w3 = P.attention(q, k, v, window=3)
    assert torch.allclose(w3[:3], out[:3]) and not torch.allclose(w3[3:], out[3:])
    assert torch.allclose(w3[5], P.attention(q[3:], k[3:], v[3:])[2])
    # causal: later tokens change nothing before them
    assert torch.allclose(P.attention(q[:4], k[:4], v[:4]), out[:4])
    # the scale is 1 / sqrt(head_dim)
    assert torch.allclose(P.attention(q, k, v, scale=1 / math.sqrt(8)), out)
    assert not torch.allclose(P.attention(q, k, v, scale=1.0), out)


# ------------------------------------------------------------------------------------------------ routing and experts
def test_route_reference_vector():
    """/root/reference/tests/test_gguf_moe.cpp:273-304."""
    wr = torch.zeros(8, 4, dtype=D)
    wr[3, 0], wr[5, 0], wr[0, 0] = 10.0, 8.0, 1.0
    x = torch.tensor([1.0, 0, 0, 0], dtype=D)
    ids, w = P.route(x, wr, 2, True)
    assert ids == [3, 5] and abs(w.sum().item() - 1) < 1e-12 and w[0] > w[1]
    assert torch.allclose(w, torch.tensor([0.880797, 0.119203], dtype=D), atol=1e-6)
    ids, w = P.route(x, wr, 2, False)
    assert ids == [3, 5] and torch.allclose(w, torch.softmax(wr[:, 0], 0)[[3, 5]]) and w.sum() < 1


def test_route_ties_and_limits():
    ids, w = P.route(rnd(6), torch.zeros(5, 6, dtype=D), 3, True)
    assert ids == [4, 3, 2] and torch.allclose(w, torch.full((3,), 1 / 3, dtype=D))       # >= : the last index wins
    x, wr = rnd(6, seed=1), rnd(5, 6, seed=2)
    ids, w = P.route(x, wr, 5, True)
    assert torch.allclose(w, torch.softmax(wr @ x, 0)[ids])             # k = E: the whole softmax
    ids_t, w_t = P.route(x, wr, 2, True)
    ids_f, w_f = P.route(x, wr, 2, False)
    assert ids_t == ids_f and torch.allclose(w_t, w_f / w_f.sum())      # renormalised = un-normalised / their sum
    assert P.route_margin(x, wr, 5) == math.inf and P.route_margin(x, wr, 2) > 0


def expert_weights(E, H, I, seed):
    return [{"gate": rnd(I, H, seed=seed + 3 * e), "up": rnd(I, H, seed=seed + 3 * e + 1),
             "down": rnd(H, I, seed=seed + 3 * e + 2)} for e in range(E)]


def test_moe_special_cases():
    H, I = 6, 10
    x = rnd(4, H)
    one = expert_weights(1, H, I, 10)
    dense = P.swiglu_mlp(x, one[0]["gate"], one[0]["up"], one[0]["down"])
    assert torch.allclose(dense, (torch.nn.functional.silu(x @ one[0]["gate"].T) * (x @ one[0]["up"].T)) @ one[0]["down"].T)
    # one expert, top 1, renormalised: the dense layer
    assert torch.allclose(P.moe(x, {"router": rnd(1, H, seed=5), "experts": one}, 1, True), dense)
    # all experts alike: (sum of weights) times the expert
    w = {"router": rnd(4, H, seed=6), "experts": one * 4}
    sums = torch.stack([P.route(x[t], w["router"], 2, False)[1].sum() for t in range(4)])
    assert torch.allclose(P.moe(x, w, 2, False), sums[:, None] * dense)
    assert torch.allclose(P.moe(x, w, 2, True), dense)
    # shared expert with a zero gate vector: exactly half of it; without a gate vector: all of it
    sh = expert_weights(1, H, I, 30)[0]
    base = P.moe(x, w, 2, True)
    shared_out = P.swiglu_mlp(x, sh["gate"], sh["up"], sh["down"])
    assert torch.allclose(P.moe(x, {**w, "shared": sh, "shared_scale": torch.zeros(1, H, dtype=D)}, 2, True), base + 0.5 * shared_out)
    assert torch.allclose(P.moe(x, {**w, "shared": sh}, 2, True), base + shared_out)
    g = rnd(1, H, seed=7)
    assert torch.allclose(P.moe(x, {**w, "shared": sh, "shared_scale": g}, 2, True),
                          base + torch.sigmoid(x @ g[0])[:, None] * shared_out)


# ------------------------------------------------------------------------------------------------ the whole model
def test_layer_kinds_and_windows_follow_the_configuration(model_dirs):
    b = P.PlainQwen2Moe(model_dirs("B"))
    assert [b.layer_is_sparse(l) for l in range(3)] == [False, True, False]
    assert [b.layer_window(l) for l in range(3)] == [None, 24, 24]
    a = P.PlainQwen2Moe(model_dirs("A"))
    assert [a.layer_is_sparse(l) for l in range(2)] == [True, True] and a.layer_window(1) is None


def test_model_is_causal_and_the_window_matters(model_dirs):
    m = P.PlainQwen2Moe(model_dirs("B"))
    toks = list(range(5, 65))
    full = m.logits(toks)
    assert torch.allclose(m.logits(toks[:30]), full[:30], atol=1e-12)
    assert m.min_margins().shape == (30,)
    m.cfg = {**m.cfg, "use_sliding_window": False}
    no_window = m.logits(toks)
    assert torch.allclose(no_window[:24], full[:24], atol=1e-12) and not torch.allclose(no_window[30:], full[30:], atol=1e-6)


def test_tied_head_is_the_embedding(model_dirs, tmp_path):
    from turboquant_cpp_amd.engine.model import write_random_model_dir
    cfg = {**TINY_A, "tie_word_embeddings": True}
    tied = P.PlainQwen2Moe(write_random_model_dir(str(tmp_path / "t"), cfg, seed=0, dtype="float32"))
    assert "lm_head.weight" not in tied.t
    lg = tied.logits([1, 2, 3])
    tied.t["lm_head.weight"] = tied.t["model.embed_tokens.weight"].clone()
    assert torch.equal(tied.logits([1, 2, 3]), lg)


# ------------------------------------------------------------------------------------------------ sampling
def test_sampling_vectors():
    """/root/reference/tests/test_ops.cpp:528-571."""
    assert P.sample_argmax([1.0, 5.0, 3.0, 2.0]) == 1 and P.sample_argmax([-3.0, -1.0, -2.0, -5.0]) == 1
    assert P.sample_argmax([2.0, 7.0, 7.0]) == 1                         # the first maximum
    rng = P.PlainRng(42)
    assert P.sample_topp(np.array([1.0, 5.0, 3.0, 2.0]), 0.001, 0.9, rng) == 1
    assert P.sample_topp(np.array([1.0, 5.0, 3.0, 2.0]), 0.0, 0.9, rng) == 1
    counts = np.bincount([P.sample_topp(np.zeros(4), 1.0, 1.0, rng) for _ in range(1000)], minlength=4)
    assert all(100 < c < 500 for c in counts)
    a = [P.sample_topp(np.arange(20.0) / 4, 0.8, 0.9, P.PlainRng(7)) for _ in range(1)]
    b = [P.sample_topp(np.arange(20.0) / 4, 0.8, 0.9, P.PlainRng(7)) for _ in range(1)]
    assert a == b
    # top-p cuts the tail: with p = 0.5 only the most likely tokens can come
    seen = {P.sample_topp(np.array([5.0, 4.0, 0.0, 0.0, 0.0]), 1.0, 0.5, rng) for _ in range(200)}
    assert seen == {0}


def test_repetition_penalty_counts_every_occurrence():
    """/root/reference/src/engine/tq_generate.c:387-400."""
    l = np.array([2.0, -2.0, 3.0, 1.0], dtype=np.float32)
    P.apply_rep_penalty(l, [0, 1, 0, 9], window=3, penalty=2.0)      # the last three: 1, 0, 9 (9 is out of range)
    assert l.tolist() == [1.0, -4.0, 3.0, 1.0]
    P.apply_rep_penalty(l, [0, 0], window=32, penalty=2.0)
    assert l.tolist() == [0.25, -4.0, 3.0, 1.0]
    P.apply_rep_penalty(l, [0], window=32, penalty=1.0)
    assert l[0] == 0.25


def test_a_near_tie_decided_the_other_way_exchanges_two_experts():
    """``route(..., other_side=(i, j))`` puts the expert of rank j in the place of rank i; ``near_swaps`` lists the
    exchanges by the gap of their logits."""
    router = torch.zeros(6, 4, dtype=torch.float64)
    for e, v in enumerate([5.0, 1.0, 4.0, 3.99, 3.0, 3.98]):
        router[e, 0] = v
    x = torch.tensor([1.0, 0, 0, 0], dtype=torch.float64)
    ids, w = P.route(x, router, 2, True)
    assert ids == [0, 2] and abs(float(w.sum()) - 1) < 1e-12
    ids2, w2 = P.route(x, router, 2, True, other_side=(1, 2))
    assert ids2 == [0, 3] and abs(float(w2[1] / w2[0]) - math.exp(3.99 - 5.0)) < 1e-12
    assert P.route(x, router, 2, True, other_side=(1, 3))[0] == [0, 5]
    assert P.route(x, router, 2, True, other_side=(0, 2))[0] == [3, 2]
    swaps = P.near_swaps(x, router, 2)
    assert [(i, j) for _, i, j in swaps[:2]] == [(1, 2), (1, 3)] and swaps[0][0] < swaps[1][0] < 0.02
