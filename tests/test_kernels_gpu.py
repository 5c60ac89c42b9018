"""Each HIP kernel alone against a plain torch float32 (or float64) computation of the same operation,
at sizes other than the engine's: widths and vocabularies that are no power of two, head sizes in steps
of 16, odd numbers of heads and groups, rows that do not fill a tile."""
import math
import numpy as np

import pytest
import torch

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


def tol(act, scale=1.0):
    return (2e-5 if act == "float32" else 2e-2) * scale


# ------------------------------------------------------------------------------------------------ embed / norm
@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
def test_embed(ops, act, wdtype):
    if act == "float32" and wdtype != torch.float32:
        pytest.skip("the 32-bit path keeps its weights in 32 bits")
    table = rnd((37, 50), wdtype, 1)
    tokens = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32)
    x = ops.embed(tokens.to(DEV), table.to(DEV), act).cpu()
    assert torch.equal(x, table[tokens.long()].float())


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("shape,dtype", [((9, 3), torch.float32), ((40, 5, 130), torch.float32), ((7, 6), torch.bfloat16),
                                         ((5, 4100), torch.int32)])
def test_rows_by_index(ops, act, shape, dtype):
    """Rows gathered out of and scattered into a tensor with a row per slot, as a step takes and puts back the
    fixed-size state of its sequences: bit for bit what indexing gives."""
    g = torch.Generator().manual_seed(5)
    table = (torch.randn(shape, generator=g) * 100).to(dtype)
    index = torch.randperm(shape[0], generator=g)[: max(1, shape[0] // 2)].to(torch.int32)
    got = ops.gather_rows(table.to(DEV), index.to(DEV), act).cpu()
    assert torch.equal(got, table[index.long()])
    rows = (torch.randn((index.numel(), *shape[1:]), generator=g) * 100).to(dtype)
    dev = table.to(DEV)
    ops.scatter_rows(dev, index.to(DEV), rows.to(DEV), act)
    want = table.clone()
    want[index.long()] = rows
    assert torch.equal(dev.cpu(), want)


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("H", [48, 200, 1000])
def test_add_rmsnorm(ops, act, H):
    T, S, eps = 7, 3, 1e-5
    x = rnd((T, H), torch.float32, 2)
    delta = rnd((S, T, H), torch.float32, 3)
    w = rnd((H,), adt(act), 4) + 1
    xd = x.clone().to(DEV)
    out, out32 = ops.add_rmsnorm(xd, delta.to(DEV), w.to(DEV), eps, act, want_f32=True)
    v = x.double() + delta.double().sum(0)
    ref = v * (1.0 / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)) * w.double()
    assert (xd.cpu().double() - v).abs().max() < 1e-5          # the residual stream holds the sum
    assert (out32.cpu().double() - ref).abs().max() < 1e-4
    assert (out.cpu().double() - ref).abs().max() < tol(act, 4)
    # picked rows: x stays as it is, rows may repeat
    rows = torch.tensor([5, 0, 5], dtype=torch.int32)
    xd2 = x.clone().to(DEV)
    out_r, _ = ops.add_rmsnorm(xd2, delta.to(DEV), w.to(DEV), eps, act, rows=rows.to(DEV))
    assert torch.equal(xd2.cpu(), x)
    assert torch.equal(out_r.cpu(), out.cpu()[rows.long()])
    # no pending sum: x is only normalised
    xd3 = x.clone().to(DEV)
    out_n, _ = ops.add_rmsnorm(xd3, None, w.to(DEV), eps, act)
    ref_n = x.double() * (1.0 / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + eps)) * w.double()
    assert (out_n.cpu().double() - ref_n).abs().max() < tol(act, 4)


# ------------------------------------------------------------------------------------------------ products
def ref_gemm(a, w, bias=None, w2=None):
    y = a.double() @ w.double().T
    if bias is not None:
        y = y + bias.double()
    if w2 is not None:
        y = torch.nn.functional.silu(y) * (a.double() @ w2.double().T)
    return y


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("M,N,K", [(5, 33, 50), (1, 50, 72), (5, 130, 200), (16, 64, 64), (17, 33, 136), (40, 257, 264),
                                   (64, 96, 1000), (65, 130, 72), (200, 300, 520), (300, 129, 64), (1130, 7400, 136), (2048, 4096, 72)])
@pytest.mark.parametrize("mode", ["plain", "bias", "gated"])
def test_gemm_dense(ops, act, M, N, K, mode, monkeypatch):
    a = rnd((M, K), adt(act), 10)
    w = rnd((N, K), adt(act), 11, 0.2)
    bias = rnd((N,), adt(act), 12) if mode == "bias" else None
    w2 = rnd((N, K), adt(act), 13, 0.2) if mode == "gated" else None
    # where the vendor library would take the product, this library's own kernel is held to the same bound
    for vendor in (True, False) if ops._vendor_product(act, a.to(DEV), w.to(DEV), M, K) and mode == "plain" else (True,):
        monkeypatch.setattr(ops, "_VENDOR", vendor)
        for out_act in (False, True):
            y = ops.gemm(a.to(DEV), w.to(DEV), act, bias=None if bias is None else bias.to(DEV),
                         w2=None if w2 is None else w2.to(DEV), out_act=out_act).cpu()
            ref = ref_gemm(a, w, bias, w2)
            scale = ref.abs().max().item()
            err = (y.double() - ref).abs().max().item()
            limit = 1e-5 * scale * math.sqrt(K) if act == "float32" else (2e-2 if out_act else 4e-3) * scale
            assert err < limit, (err, scale, vendor)


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("N", [65537, 151936])
@pytest.mark.parametrize("M", [17, 33, 64])
def test_a_few_dozen_rows_times_a_matrix_of_a_vocabulary(ops, act, M, N):
    """17 to 64 rows against a matrix of 65,536 rows and more: the shape of the vocabulary's product in a decode step
    of that many sequences, which takes the tile kernels where narrower matrices take the streaming ones.  Plain and
    as partial sums, against the product in float64 (worked out on the GPU: it is the reference here, not the
    subject)."""
    K = 2048
    a = rnd((M, K), adt(act), 40 + M).to(DEV)
    w = rnd((N, K), adt(act), 41, 0.2).to(DEV)
    ref = a.double() @ w.double().T
    scale = ref.abs().max().item()
    limit = 1e-5 * scale * math.sqrt(K) if act == "float32" else 4e-3 * scale
    y = ops.gemm(a, w, act)
    assert tuple(y.shape) == (M, N) and (y.double() - ref).abs().max().item() < limit
    parts = ops.gemm(a, w, act, partial_sums=True)
    assert tuple(parts.shape[1:]) == (M, N) and (parts.double().sum(0) - ref).abs().max().item() < limit
    # a row's result does not depend on how many rows come with it
    alone = ops.gemm(a[M - 1:], w, act)
    if act == "float32":
        assert (alone[0] - y[M - 1]).abs().max().item() < 1e-5 * scale * math.sqrt(K)
    else:
        assert (alone[0] - y[M - 1]).abs().max().item() < 4e-3 * scale


@pytest.mark.parametrize("M,N,K", [(512, 130, 264), (700, 6144, 2048), (2048, 257, 1000), (8192, 96, 16384), (600, 96, 16384)])
def test_plain_products_of_many_rows(ops, M, N, K, monkeypatch):
    """From VENDOR_MIN_ROWS rows on (512 here, to keep the sizes small) a plain bfloat16 product without bias goes to
    the vendor's library unless k is long and the rows are not many; its result and the own kernel's are the same
    product in another order of sums.  Gated products, products with a bias and the 32-bit path stay;
    TQ_PLAIN_PRODUCTS=own (read at import) keeps all."""
    act = "bfloat16"
    below = rnd((ops.VENDOR_MIN_ROWS - 1, K), adt(act), 13).to(DEV)
    assert not ops._vendor_product(act, below, below, ops.VENDOR_MIN_ROWS - 1, K)       # the border as it ships
    monkeypatch.setattr(ops, "VENDOR_MIN_ROWS", 512)
    a, w = rnd((M, K), adt(act), 14).to(DEV), rnd((N, K), adt(act), 15, 0.2).to(DEV)
    calls = []
    real = torch.mm
    monkeypatch.setattr(torch, "mm", lambda *x, **kw: (calls.append(1), real(*x, **kw))[1])
    taken = ops._vendor_product(act, a, w, M, K)
    assert taken == (K < 16384 or M >= 8192)
    got = ops.gemm(a, w, act, partial_sums=True)
    assert len(calls) == (1 if taken else 0) and got.shape[1:] == (M, N) and got.dtype == torch.float32
    ref = ref_gemm(a.cpu(), w.cpu())
    scale = ref.abs().max().item()
    assert (got.sum(0).cpu().double() - ref).abs().max().item() < 4e-3 * scale
    assert ops.gemm(a, w, act, out_act=True).dtype == torch.bfloat16
    n = len(calls)
    ops.gemm(a, w, act, bias=w[:, 0].contiguous())
    ops.gemm(a, w, act, w2=w, out_act=True)
    ops.gemm(a.float(), w.float(), "float32")
    assert len(calls) == n
    monkeypatch.setattr(ops, "_VENDOR", False)
    own = ops.gemm(a, w, act)
    assert len(calls) == n and (own.cpu().double() - ref).abs().max().item() < 4e-3 * scale


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("activation", ["silu", "gelu_tanh", "relu2"])
@pytest.mark.parametrize("M,N,ld", [(3, 40, 80), (70, 33, 70), (5, 1028, 2056), (9, 10, 21)])
def test_the_gate_applied_afterwards(ops, act, activation, M, N, ld):
    gu = rnd((M, ld), torch.float32, 16, 2.0).to(DEV)
    out = torch.empty((M, N), dtype=adt(act), device=DEV)
    ops._run("gated_act", ops.library(act).tq_gated_act(gu.data_ptr(), ld, out.data_ptr(), M, N, ops.GATES[activation],
                                                        ops._stream()))
    g, u = gu[:, :N].cpu().double(), gu[:, N:2 * N].cpu().double()
    f = {"silu": torch.nn.functional.silu, "relu2": lambda v: torch.relu(v) ** 2,
         "gelu_tanh": lambda v: torch.nn.functional.gelu(v, approximate="tanh")}[activation]
    ref = f(g) * u
    assert (out.cpu().double() - ref).abs().max().item() < (1e-5 if act == "float32" else 8e-3) * ref.abs().max().item()
    assert ops.library(act).tq_gated_act(gu.data_ptr(), 2 * N - 1, out.data_ptr(), M, N, 0, ops._stream()) != 0


@pytest.mark.parametrize("activation", ["silu", "gelu_tanh"])
@pytest.mark.parametrize("M,N,K", [(512, 130, 264), (5000, 96, 72), (700, 1408, 2048)])
def test_gated_pairs_of_many_rows(ops, activation, M, N, K, monkeypatch):
    """A gated pair whose second matrix lies right behind the first goes, from VENDOR_MIN_ROWS rows on (512 here), to
    the vendor's library as one product over both, a few thousand rows at a time, with the gate in a pass of its
    own; matrices that lie apart stay in this library's kernel.  Both are the same function."""
    act = "bfloat16"
    monkeypatch.setattr(ops, "VENDOR_MIN_ROWS", 512)
    a = rnd((M, K), adt(act), 17).to(DEV)
    w, w2 = rnd((N, K), adt(act), 18, 0.2).to(DEV), rnd((N, K), adt(act), 19, 0.2).to(DEV)
    g, u = ops.side_by_side(w, w2)
    assert torch.equal(g, w) and torch.equal(u, w2) and ops._behind(g, u) and not ops._behind(w, w2) and not ops._behind(u, g)
    calls = []
    real = torch.mm
    monkeypatch.setattr(torch, "mm", lambda *x, **kw: (calls.append(x[0].shape[0]), real(*x, **kw))[1])
    monkeypatch.setattr(ops, "VENDOR_GATED_ROWS", 2048)
    got = ops.gemm(a, g, act, w2=u, out_act=True, activation=activation)
    assert calls == [min(2048, M - r) for r in range(0, M, 2048)]
    own = ops.gemm(a, w, act, w2=w2, out_act=True, activation=activation)
    assert len(calls) == -(-M // 2048)
    f = torch.nn.functional.silu if activation == "silu" else lambda v: torch.nn.functional.gelu(v, approximate="tanh")
    ref = f(a.cpu().double() @ w.cpu().double().T) * (a.cpu().double() @ w2.cpu().double().T)
    scale = ref.abs().max().item()
    for y in (got, own):
        assert y.dtype == torch.bfloat16 and (y.cpu().double() - ref).abs().max().item() < 2e-2 * scale
    ops.gemm(a, g, act, w2=u)          # into float32: this library's kernel
    assert len(calls) == -(-M // 2048)


@pytest.mark.parametrize("M,N", [(320, 5632), (384, 5632), (128, 20480), (192, 20480), (260, 20480)])
def test_a_gated_pair_of_a_few_hundred_rows_in_either_tile(ops, M, N):
    """A gated pair with one matrix takes tiles of 64 rows where its workgroups need no more than a compute unit each
    (or where the taller tile would need a second round and the lower fits in one), else tiles of 128: the sizes here
    lie on both sides of both borders, and every one is the same function."""
    act, K = "bfloat16", 136
    a, w, w2 = rnd((M, K), adt(act), 31), rnd((N, K), adt(act), 32, 0.2), rnd((N, K), adt(act), 33, 0.2)
    y = ops.gemm(a.to(DEV), w.to(DEV), act, w2=w2.to(DEV), out_act=True).cpu().double()
    ref = ref_gemm(a, w, None, w2)
    assert (y - ref).abs().max().item() < 2e-2 * ref.abs().max().item()


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("M,N,K,bias", [(300, 200, 2200, True), (129, 130, 4104, False), (70, 64, 1000, False), (9, 40, 4096, True),
                                        (40, 264, 8200, True), (64, 2048, 5632, False), (17, 72, 4096, False), (33, 130, 2112, True),
                                        (50, 96, 400, False), (32, 200, 4096, False)])
def test_gemm_partial_sums(ops, act, M, N, K, bias):
    """A product may come back as partial sums over runs of k ([S, M, N], the bias in the first); however many the
    kernel makes, their sum is the product."""
    a = rnd((M, K), adt(act), 14)
    w = rnd((N, K), adt(act), 15, 0.2)
    b = rnd((N,), adt(act), 16) if bias else None
    y = ops.gemm(a.to(DEV), w.to(DEV), act, bias=None if b is None else b.to(DEV), partial_sums=True).cpu()
    assert y.dim() == 3 and tuple(y.shape[1:]) == (M, N)
    if act == "bfloat16":
        def tile_runs():    # tiles of 64 rows: up to 8 runs of at least 256 while the workgroups are few and the sums small
            tiles, t = -(-M // 64) * -(-N // 128), 1
            while t < 8 and tiles * t * 2 <= 512 and K // (t * 2) >= 256 and t * 2 * M * N * 4 <= 8 << 20:
                t *= 2
            while t > 1 and (t - 1) * (-(-(-(-K // 64)) // t) * 64) >= K:    # no run begins past the end
                t //= 2
            return t

        if M <= 16:
            runs = 1
        elif 32 < M <= 64 and tile_runs() > 1:      # 33 to 64 rows take the tile kernel where it may split k
            runs = tile_runs()
        elif M <= 64:       # few rows of a narrow matrix: runs of at least 128 of k for each of 8 waves, up to 4096 waves
            runs, waves = 1, -(-N // 32) * 8
            while runs < 8 and waves * runs < 4096 and K // (16 * runs) >= 128:
                runs *= 2
        else:
            runs = 1 if K < 2048 else (2 if K < 4096 else 4)
            if M <= 1024:
                runs = max(runs, tile_runs())
        assert y.shape[0] == runs
    ref = ref_gemm(a, w, b, None)
    scale = ref.abs().max().item()
    err = (y.double().sum(0) - ref).abs().max().item()
    assert err < (1e-5 * scale * math.sqrt(K) if act == "float32" else 4e-3 * scale), (err, scale)


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("activation", ["silu", "gelu_tanh", "relu2"])
@pytest.mark.parametrize("M,N,K", [(3, 40, 72), (40, 130, 264), (150, 200, 136), (9, 33, 50)])
def test_gated_products_take_the_activation_as_a_parameter(ops, act, activation, M, N, K):
    """The gate of a gated pair is a parameter of the products' epilogues: every kernel family (few rows, tiles,
    plain multiply-adds where K is no multiple of 4 or 8) with each activation."""
    a, w, w2 = rnd((M, K), adt(act), 22), rnd((N, K), adt(act), 23, 0.3), rnd((N, K), adt(act), 24, 0.3)
    y = ops.gemm(a.to(DEV), w.to(DEV), act, w2=w2.to(DEV), activation=activation).cpu().double()
    g = a.double() @ w.double().T
    gate = {"silu": g / (1 + torch.exp(-g)), "relu2": torch.relu(g) ** 2,
            "gelu_tanh": 0.5 * g * (1 + torch.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g ** 3)))}[activation]
    ref = gate * (a.double() @ w2.double().T)
    assert (y - ref).abs().max() < (1e-5 * math.sqrt(K) if act == "float32" else 4e-3) * ref.abs().max()
    with pytest.raises(ops.KernelError, match="unknown activation"):
        ops.gemm(a.to(DEV), w.to(DEV), act, w2=w2.to(DEV), activation="swish")


@pytest.mark.parametrize("act", ACTS)
def test_gemm_float32_weights_on_the_bfloat16_path(ops, act):
    """A matrix the checkpoint stores in 32 bits stays so and still multiplies."""
    a = rnd((9, 72), adt(act), 20)
    w = rnd((50, 72), torch.float32, 21, 0.2)
    y = ops.gemm(a.to(DEV), w.to(DEV), act).cpu()
    ref = ref_gemm(a, w)
    assert (y.double() - ref).abs().max() < 1e-4 * ref.abs().max() * 10


@pytest.mark.parametrize("act", ACTS)
def test_gemm_rows_do_not_depend_on_the_batch(ops, act):
    """A row's result is the same bits whether it is multiplied alone or among others (same kernel family)."""
    K, N = 264, 130
    a = rnd((16, K), adt(act), 30)
    w = rnd((N, K), adt(act), 31, 0.2)
    full = ops.gemm(a.to(DEV), w.to(DEV), act).cpu()
    for m in (1, 3, 9):
        part = ops.gemm(a[:m].contiguous().to(DEV), w.to(DEV), act).cpu()
        assert torch.equal(part, full[:m])


def test_the_height_of_expert_tiles(ops, monkeypatch):
    """16 up to 5 pairs per expert and 32 up to 10 where the bfloat16 matrix-core product runs (else 16 up to 12), 64
    beyond, which the products take two at a time from 48 rows per expert on; 128 and 256 only where their borders
    are lowered, and only for the bfloat16 matrix-core product."""
    a16, w16 = torch.zeros((1, 64), dtype=torch.bfloat16), torch.zeros((1, 8, 64), dtype=torch.bfloat16)
    a32, w32 = a16.float(), w16.float()
    assert ops.expert_tile_rows(60 * 5, 60, "bfloat16", a16, w16) == 16
    assert ops.expert_tile_rows(60 * 5 + 1, 60, "bfloat16", a16, w16) == 32
    assert ops.expert_tile_rows(60 * 10, 60, "bfloat16", a16, w16) == 32
    assert ops.expert_tile_rows(60 * 10 + 1, 60, "bfloat16", a16, w16) == 64
    assert ops.expert_tile_rows(60 * 12, 60, "float32", a32, w32) == 16
    assert ops.expert_tile_rows(60 * 12 + 1, 60, "float32", a32, w32) == 64
    assert ops.expert_tile_rows(60 * 100000, 60, "bfloat16", a16, w16) == 64
    assert ops.expert_product_rows(64, 60 * 48 - 1, 60) == 64
    assert ops.expert_product_rows(64, 60 * 48, 60) == 64 + ops.TILE_PAIRS
    assert ops.expert_product_rows(16, 60 * 64, 60) == 16 and ops.expert_product_rows(256, 60 * 2000, 60) == 256
    monkeypatch.setattr(ops, "EXPERT_128_FROM", 256)
    monkeypatch.setattr(ops, "EXPERT_256_FROM", 1024)
    assert ops.expert_tile_rows(60 * 256 - 1, 60, "bfloat16", a16, w16) == 64
    assert ops.expert_tile_rows(60 * 256, 60, "bfloat16", a16, w16) == 128
    assert ops.expert_tile_rows(60 * 1024 - 1, 60, "bfloat16", a16, w16) == 128
    assert ops.expert_tile_rows(60 * 1024, 60, "bfloat16", a16, w16) == 256
    assert ops.expert_tile_rows(60 * 1024, 60, "float32", a32, w32) == 64
    assert ops.expert_tile_rows(60 * 256, 60, "float32", a32, w32) == 64
    assert ops.expert_tile_rows(60 * 256, 60, "bfloat16", a16, w32) == 64      # float32 weights: the plain product


@pytest.mark.parametrize("H,I", [(128, 256), (192, 1408), (256, 72)])
def test_units_two_at_a_time_with_a_crowded_expert(ops, H, I):
    """Units of 64 rows taken two at a time when the router sends nearly every token to one expert: that expert has
    many items, its neighbours one row or none, an expert's last unit stands alone where their number is odd, and the
    last column tile is not full (72 columns; a k of 72 falls back to the tile kernel).  Against sums in double, and
    bit for bit what the same units give one by one."""
    act, T, E, k = "bfloat16", 601, 5, 2
    ids = torch.empty((T, k), dtype=torch.int32)
    ids[:, 0] = 3                                  # the crowded expert: ten units, five items
    ids[:, 1] = torch.where(torch.arange(T) % 150 == 0, 1, 4).to(torch.int32)      # expert 1: five rows; 4: the rest
    ids[7, 1], ids[7, 0] = 0, 4                    # expert 0: one row; expert 2: none
    x = rnd((T, H), adt(act), 45)
    wg, wu, wd = rnd((E, I, H), adt(act), 46, 0.2), rnd((E, I, H), adt(act), 47, 0.2), rnd((E, H, I), adt(act), 48, 0.2)
    st, slot, te, nt = ops.moe_align(ids.to(DEV), E, 64, act)
    units, items = nt.tolist()
    assert units == 1 + 1 + 10 + 10 and items == 1 + 1 + 5 + 5
    out = {}
    for rows in (64, 64 + 1024):
        h = ops.gemm(x.to(DEV), wg.to(DEV), act, w2=wu.to(DEV), out_act=True, a_rows=st, tile_group=te, n_tiles=nt, tile_rows=rows)
        y = ops.gemm(h, wd.to(DEV), act, a_rows=st, tile_group=te, n_tiles=nt, tile_rows=rows, gather=False)
        out[rows] = (h.cpu(), y.cpu())
    live = (st >= 0).cpu()
    assert torch.equal(out[64][0][live], out[64 + 1024][0][live]) and torch.equal(out[64][1][live], out[64 + 1024][1][live])
    hc, y = out[64 + 1024]
    for t in (0, 7, 150, 300, 600):
        for j in range(k):
            e, r = int(ids[t, j]), int(slot[t, j])
            href = ref_gemm(x[t:t + 1], wg[e], w2=wu[e])[0]
            assert (hc[r].double() - href).abs().max() < tol(act, 2) * max(1.0, href.abs().max().item())
            yref = hc[r:r + 1].double() @ wd[e].double().T
            assert (y[r].double() - yref[0]).abs().max() < tol(act, 2) * max(1.0, yref.abs().max().item())


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("unit", [16, 32, 64, 128, 256, 64 + 1024])
@pytest.mark.parametrize("T,E,k,H,I", [(1, 5, 2, 72, 40), (9, 7, 3, 136, 88), (150, 6, 2, 64, 200), (700, 3, 2, 64, 136),
                                       (700, 3, 2, 128, 192), (260, 5, 3, 192, 320)])
def test_expert_products(ops, act, unit, T, E, k, H, I):
    """Pairs ordered by expert, the gated product over gathered rows, the second product over rows in place.
    Units of 32, 128 and 256 rows are the bfloat16 matrix-core product's alone (32: the streaming kernel with two row
    tiles to a wave; with 256, the gated pair runs in tiles of
    256 rows and the second product in two tiles of 128 to a unit; 700 tokens give each expert a whole unit and
    a part of one).  64 + 1024: units of 64 that the products take two at a time, by the items that the order lists
    behind its row tiles (where k is no multiple of 64 they fall back to one unit at a time)."""
    rows, unit = unit, unit % 1024
    if rows not in (16, 64) and act != "bfloat16":
        pytest.skip("tiles of 32, 128 and 256 rows and pairs of units are for the bfloat16 matrix-core product")
    g = torch.Generator().manual_seed(40)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    x = rnd((T, H), adt(act), 41)
    wg, wu = rnd((E, I, H), adt(act), 42, 0.2), rnd((E, I, H), adt(act), 43, 0.2)
    wd = rnd((E, H, I), adt(act), 44, 0.2)
    st, slot, tile_e, n_tiles = ops.moe_align(ids.to(DEV), E, unit, act)
    st_c, slot_c, tile_c, (nt, n_items) = st.cpu(), slot.cpu(), tile_e.cpu(), n_tiles.cpu().tolist()
    # the order: every pair has its row, rows of one expert are together and in order of token, tiles are whole
    assert sorted(slot_c.view(-1).tolist()) == [r for r in range(st_c.numel()) if st_c[r] >= 0]
    for t in range(T):
        for j in range(k):
            r = int(slot_c[t, j])
            assert int(st_c[r]) == t and int(tile_c[r // unit]) == int(ids[t, j])
    assert nt == sum(-(-int((ids == e).sum()) // unit) for e in range(E))
    rows_by_expert = [[r for r in range(nt * unit) if st_c[r] >= 0 and tile_c[r // unit] == e] for e in range(E)]
    for mine in rows_by_expert:
        assert [int(st_c[r]) for r in mine] == sorted(int(st_c[r]) for r in mine)
    # the items behind the row tiles: every expert's row tiles two at a time, its last one alone if their number is odd
    items = tile_c[st_c.numel() // unit:][:n_items].tolist()
    expected = []
    for e in range(E):
        mine = [t for t in range(nt) if tile_c[t] == e]
        expected += mine[::2]
    assert items == expected
    h = ops.gemm(x.to(DEV), wg.to(DEV), act, w2=wu.to(DEV), out_act=True, a_rows=st, tile_group=tile_e,
                 n_tiles=n_tiles, tile_rows=rows)
    y = ops.gemm(h, wd.to(DEV), act, a_rows=st, tile_group=tile_e, n_tiles=n_tiles, tile_rows=rows, gather=False).cpu()
    hc = h.cpu()
    for t in range(T):
        for j in range(k):
            e, r = int(ids[t, j]), int(slot_c[t, j])
            href = ref_gemm(x[t:t + 1], wg[e], w2=wu[e])[0]
            assert (hc[r].double() - href).abs().max() < tol(act, 2) * max(1.0, href.abs().max().item())
            yref = hc[r:r + 1].double() @ wd[e].double().T
            assert (y[r].double() - yref[0]).abs().max() < tol(act, 2) * max(1.0, yref.abs().max().item())


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("gated", [True, False])
def test_two_products_in_one_launch(ops, act, gated):
    """A product over experts and a plain product of the same few rows, asked for as a pair: the first gives the
    bits it gives alone (its split of k is its own), the second agrees with the plain formula; more rows, or
    products of different kinds, fall back to two calls with the same results."""
    E, I, H, k, S = 7, 48, 264, 3, 104
    for T in (1, 5, 16, 40):
        x = rnd((T, H), adt(act), 45)
        g = torch.Generator().manual_seed(46)
        ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
        unit = 16 if T <= 16 else 64
        st, slot, te, nt = ops.moe_align(ids.to(DEV), E, unit, act)
        wg, wu = rnd((E, I, H), adt(act), 47, 0.2), rnd((E, I, H), adt(act), 48, 0.2)
        sg, su = rnd((S, H), adt(act), 49, 0.2), rnd((S, H), adt(act), 50, 0.2)
        first = dict(a=x.to(DEV), w=wg.to(DEV), a_rows=st, tile_group=te, n_tiles=nt, tile_rows=unit)
        second = dict(a=x.to(DEV), w=sg.to(DEV))
        if gated:
            first.update(w2=wu.to(DEV), out_act=True)
            second.update(w2=su.to(DEV), out_act=True)
        y1, y2 = ops.gemm_pair(dict(first), dict(second), act)
        a1 = ops.gemm(first.pop("a"), first.pop("w"), act, **first)
        a2 = ops.gemm(second.pop("a"), second.pop("w"), act, **second)
        live = (st >= 0)
        assert torch.equal(y1[live], a1[live])
        ref2 = ref_gemm(x, sg, None, su if gated else None)
        scale = ref2.abs().max().item()
        lim = 1e-5 * scale * math.sqrt(H) if act == "float32" else (2e-2 if gated else 4e-3) * scale
        assert (y2.cpu().double() - ref2).abs().max().item() < lim
        assert (a2.cpu().double() - ref2).abs().max().item() < lim
    # products of different kinds are two calls
    y1, y2 = ops.gemm_pair(dict(a=x.to(DEV), w=sg.to(DEV), w2=su.to(DEV), out_act=True), dict(a=x.to(DEV), w=sg.to(DEV)), act)
    assert y1.dtype == adt(act) and y2.dtype == torch.float32


@pytest.mark.parametrize("act", ACTS)
def test_second_product_of_a_pair_in_runs_of_k(ops, act):
    """The experts' down products (short k) beside a plain product with a long k whose partial sums are wanted
    apart: the second one comes in several runs of k (as many whatever the number of rows),
    their sum is the product, the bias is counted once, and the first product keeps the bits it has alone."""
    E, I, H, k, S = 5, 512, 264, 2, 4104
    shapes = set()
    for T in (1, 7, 16):
        g = torch.Generator().manual_seed(146)
        ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
        st, slot, te, nt = ops.moe_align(ids.to(DEV), E, 16, act)
        h = rnd((st.numel(), I), adt(act), 147)
        hs = rnd((T, S), adt(act), 148)
        wd, sd = rnd((E, H, I), adt(act), 149, 0.2), rnd((H, S), adt(act), 150, 0.2)
        bias = rnd((H,), adt(act), 151)
        first = dict(a=h.to(DEV), w=wd.to(DEV), a_rows=st, tile_group=te, n_tiles=nt, tile_rows=16, gather=False)
        second = dict(a=hs.to(DEV), w=sd.to(DEV), bias=bias.to(DEV), partial_sums=True)
        y1, y2 = ops.gemm_pair(dict(first), dict(second), act)
        a1 = ops.gemm(first.pop("a"), first.pop("w"), act, **first)
        live = (st >= 0)
        assert torch.equal(y1[live], a1[live])
        assert y2.dim() == 3 and y2.shape[1:] == (T, H) and y2.dtype == torch.float32
        shapes.add(y2.shape[0])
        ref2 = ref_gemm(hs, sd, bias, None)
        scale = ref2.abs().max().item()
        lim = 1e-5 * scale * math.sqrt(S) if act == "float32" else 4e-3 * scale
        assert (y2.cpu().double().sum(0) - ref2).abs().max().item() < lim
    # as many runs whatever the number of rows: 8 in bfloat16; in float32 what the plain product's own rule gives
    assert len(shapes) == 1 and (shapes == {8} or act == "float32")


@pytest.mark.parametrize("act", ACTS)
def test_moe_combine(ops, act):
    T, k, H, P, S = 6, 3, 100, 40, 2
    g = torch.Generator().manual_seed(50)
    y = rnd((P, H), torch.float32, 51)
    slot = torch.stack([torch.randperm(P, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    wts = torch.rand((T, k), generator=g)
    shared = rnd((S, T, H), torch.float32, 52)
    gate = torch.rand((T,), generator=g)
    out = ops.moe_combine(y.to(DEV), slot.to(DEV), wts.to(DEV), shared.to(DEV), gate.to(DEV), act).cpu()[0]
    ref = (wts[:, :, None].double() * y[slot.long()].double()).sum(1) + gate[:, None].double() * shared.double().sum(0)
    assert (out.double() - ref).abs().max() < 1e-5
    out2 = ops.moe_combine(y.to(DEV), slot.to(DEV), wts.to(DEV), None, None, act).cpu()[0]
    assert (out2.double() - (wts[:, :, None].double() * y[slot.long()].double()).sum(1)).abs().max() < 1e-5
    # the same sum left to the norm: against the plain formula, for all rows and for chosen rows
    x = rnd((T, H), torch.float32, 53)
    w = rnd((H,), adt(act), 54)
    eps = 1e-5
    for dense, gt in ((shared, gate), (None, None)):
        v = x.double() + (wts[:, :, None].double() * y[slot.long()].double()).sum(1)
        if dense is not None:
            v = v + gt[:, None].double() * dense.double().sum(0)
        want = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * w.double()
        unsummed = ops.GatheredSum(y.to(DEV), slot.to(DEV), wts.to(DEV), None if dense is None else dense.to(DEV),
                                   None if gt is None else gt.to(DEV))
        xs = x.to(DEV).clone()
        got = ops.add_rmsnorm(xs, unsummed, w.to(DEV), eps, act, want_act=False, want_f32=True)[1].cpu()
        assert (got.double() - want).abs().max() < 1e-4 and (xs.cpu().double() - v).abs().max() < 1e-5
        rows = torch.tensor([4, 1], dtype=torch.int32)
        xs = x.to(DEV).clone()
        got = ops.add_rmsnorm(xs, unsummed, w.to(DEV), eps, act, rows=rows.to(DEV), want_act=False, want_f32=True)[1].cpu()
        assert (got.double() - want[rows.long()]).abs().max() < 1e-4 and torch.equal(xs.cpu(), x)


# ------------------------------------------------------------------------------------------------ router
@pytest.mark.parametrize("act", ACTS)
def test_router_reference_vector(ops, act):
    """The vector of /root/reference/tests/test_gguf_moe.cpp:273-304: 8 experts, top 2, x = e0; expert 3 has
    logit 10, expert 5 has 8, expert 0 has 1 -> ids [3, 5], weights softmax([10, 8])."""
    E, H = 8, 4
    wr = torch.zeros((E, H))
    wr[3, 0], wr[5, 0], wr[0, 0] = 10.0, 8.0, 1.0
    x = torch.tensor([[1.0, 0, 0, 0]])
    ids, w, gate = ops.router_topk(x.to(DEV), wr.to(adt(act)).to(DEV), None, 2, True, act)
    assert ids.cpu().tolist() == [[3, 5]] and gate is None
    assert torch.allclose(w.cpu(), torch.tensor([[0.880797, 0.119203]]), atol=1e-5)
    ids, w, _ = ops.router_topk(x.to(DEV), wr.to(adt(act)).to(DEV), None, 2, False, act)
    full = torch.softmax(wr[:, 0], 0)
    assert ids.cpu().tolist() == [[3, 5]]
    assert torch.allclose(w.cpu()[0], full[[3, 5]], atol=1e-6) and w.sum() < 1


@pytest.mark.parametrize("act", ACTS)
def test_router_ties_and_shared_gate(ops, act):
    """Equal logits: the highest index wins (>= in /root/reference/src/engine/tq_moe.c:630-638); a zero shared
    gate vector gives exactly one half."""
    E, H, T = 6, 40, 3
    x = rnd((T, H), torch.float32, 60)
    ids, w, gate = ops.router_topk(x.to(DEV), torch.zeros((E, H), dtype=adt(act)).to(DEV),
                                   torch.zeros((1, H), dtype=adt(act)).to(DEV), 3, True, act)
    assert ids.cpu().tolist() == [[5, 4, 3]] * T
    assert torch.allclose(w.cpu(), torch.full((T, 3), 1 / 3))
    assert torch.equal(gate.cpu(), torch.full((T,), 0.5))


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("E,k,H,renorm", [(5, 5, 72, True), (60, 4, 200, False), (130, 8, 64, True)])
def test_router_random(ops, act, E, k, H, renorm):
    T = 11
    x = rnd((T, H), torch.float32, 61)
    wr = rnd((E, H), adt(act), 62)
    sg = rnd((1, H), adt(act), 63, 0.1)
    ids, w, gate = ops.router_topk(x.to(DEV), wr.to(DEV), sg.to(DEV), k, renorm, act)
    logits = x.double() @ wr.double().T
    top = torch.topk(logits, k, dim=-1)
    assert torch.equal(ids.cpu().long(), top.indices)
    ref = torch.softmax(top.values, -1) if renorm else torch.softmax(logits, -1).gather(1, top.indices)
    assert (w.cpu().double() - ref).abs().max() < 1e-5
    assert (gate.cpu().double() - torch.sigmoid(x.double() @ sg.double()[0])).abs().max() < 1e-5


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("E,k,H,shared", [(60, 4, 2048, True), (64, 8, 3584, True), (5, 2, 72, False), (130, 8, 1000, True),
                                          (17, 3, 4100, True), (8, 2, 70, True)])
def test_router_results_do_not_depend_on_the_number_of_tokens(ops, act, E, k, H, shared):
    """How many tokens a workgroup of the router takes and how many rows a wave takes at a time depend on the number of
    tokens; the order in which a logit is summed does not: choices, weights and the shared expert's gate of a token
    are the same bits in a step of 700 tokens, of 300, and of 7."""
    T = 700
    x = rnd((T, H), torch.float32, 67).to(DEV)
    wr = rnd((E, H), adt(act), 68, 0.3).to(DEV)
    sg = rnd((1, H), adt(act), 69, 0.1).to(DEV) if shared else None
    ids, w, gate = ops.router_topk(x, wr, sg, k, False, act)
    logits = x.cpu().double() @ wr.cpu().double().T
    top = torch.topk(logits, k, dim=-1)
    gap = (top.values[:, -1] - torch.topk(logits, min(k + 1, E), dim=-1).values[:, -1]).abs()
    clear = gap > 1e-3 * logits.abs().max()
    assert clear.sum() > T // 2 and torch.equal(ids.cpu().long()[clear], top.indices[clear])
    for lo, hi in ((0, 300), (300, 307), (693, 700), (400, 655), (0, 256)):
        i2, w2, g2 = ops.router_topk(x[lo:hi].contiguous(), wr, sg, k, False, act)
        assert torch.equal(i2, ids[lo:hi]) and torch.equal(w2, w[lo:hi])
        assert (g2 is None and gate is None) or torch.equal(g2, gate[lo:hi])


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("E,k,H,renorm,shared", [(5, 5, 72, True, True), (60, 4, 2048, False, True), (130, 8, 70, True, False)])
def test_routing_in_one_call(ops, act, E, k, H, renorm, shared):
    """``route`` is router_topk followed by moe_align; up to 16 tokens take a kernel that chooses and orders at
    once: the same results either way, also for a token that sits in a larger batch."""
    big = 21
    x = rnd((big, H), torch.float32, 64).to(DEV)
    wr = rnd((E, H), adt(act), 65).to(DEV)
    sg = rnd((1, H), adt(act), 66, 0.1).to(DEV) if shared else None
    ids_all, w_all, gate_all = ops.router_topk(x, wr, sg, k, renorm, act)
    for T in (1, 3, 16, big):
        for unit in (16, 64):
            got = ops.route(x[:T].contiguous(), wr, sg, k, renorm, unit, act)
            assert torch.equal(got[0], ids_all[:T]) and torch.equal(got[1], w_all[:T])
            assert (got[2] is None) == (not shared) and (not shared or torch.equal(got[2], gate_all[:T]))
            want = ops.moe_align(ids_all[:T].contiguous(), E, unit, act)
            n, items = want[3].tolist()      # tiles and items in use; the entries beyond them are not written
            half = want[2].numel() // 2
            assert torch.equal(got[3], want[0]) and torch.equal(got[4], want[1]) and torch.equal(got[6], want[3])
            assert torch.equal(got[5][:n], want[2][:n]) and torch.equal(got[5][half:half + items], want[2][half:half + items])


@pytest.mark.parametrize("T,E,k,H,unit,skew", [(2048, 60, 4, 128, 64, False), (2500, 60, 4, 128, 64, True), (3000, 5, 3, 72, 16, False),
                                                (1100, 130, 8, 64, 64, False), (40000, 64, 8, 64, 64, True)])
def test_order_by_several_workgroups(ops, T, E, k, H, unit, skew):
    """From 8,192 pairs on ``route`` orders the pairs with several workgroups (three launches, its table in the logits'
    memory) where ``moe_align`` has one workgroup go through them: the same rows, tiles and items, also when most
    tokens choose the same experts and when the last workgroup's waves have nothing left."""
    act = "bfloat16"
    x = rnd((T, H), torch.float32, 71)
    if skew:
        x[: T - T // 7] = x[0] + 0.01 * x[: T - T // 7]      # nearly the same logits for six tokens in seven
    x = x.to(DEV)
    wr = rnd((E, H), adt(act), 72).to(DEV)
    sg = rnd((1, H), adt(act), 73, 0.1).to(DEV)
    assert T * k >= 8192
    ids, w, gate = ops.router_topk(x, wr, sg, k, False, act)
    want = ops.moe_align(ids, E, unit, act)
    got = ops.route(x, wr, sg, k, False, unit, act)
    assert torch.equal(got[0], ids) and torch.equal(got[1], w) and torch.equal(got[2], gate)
    n, items = want[3].tolist()
    half = want[2].numel() // 2
    assert torch.equal(got[3], want[0]) and torch.equal(got[4], want[1]) and torch.equal(got[6], want[3])
    assert torch.equal(got[5][:n], want[2][:n]) and torch.equal(got[5][half:half + items], want[2][half:half + items])
    # and the order is what it says: every pair's row holds its token, rows of an expert ascend with the pair
    st, slot = got[3].cpu().long(), got[4].cpu().long().flatten()
    assert torch.equal(st[slot], torch.arange(T * k) // k)
    flat = ids.cpu().flatten().long()
    order = torch.argsort(flat * (T * k) + torch.arange(T * k))
    assert bool((slot[order][1:] > slot[order][:-1]).all())


# ------------------------------------------------------------------------------------------------ rope + cache + attention
def paged_setup(lens, page_size, nkv, hd, n_layers, act, seed):
    """Pages handed out in a scrambled order, so that a kernel that ignores the table fails."""
    n_pages_seq = [-(-n // page_size) for n in lens]
    total = sum(n_pages_seq) + 3
    perm = torch.randperm(total, generator=torch.Generator().manual_seed(seed)).tolist()
    table = torch.full((len(lens) + 2, max(n_pages_seq) + 1), -1, dtype=torch.int32)
    slots = [len(lens) + 1 - i for i in range(len(lens))]       # slots in reverse order, slot 0 unused
    it = iter(perm)
    for s, n in zip(slots, n_pages_seq):
        for p in range(n):
            table[s, p] = next(it)
    page_stride = n_layers * nkv * page_size * hd
    kp = torch.zeros(total * page_stride, dtype=adt(act))
    vp = torch.zeros(total * page_stride, dtype=adt(act))
    return table, slots, page_stride, kp, vp


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("pairing,rot", [("half", None), ("interleaved", None), ("half", 16)])
def test_rope_kv_write(ops, act, pairing, rot):
    from plain_qwen2moe import rope as plain_rope, rope_frequencies
    nh, nkv, hd, page, layers, layer = 3, 1, 48, 16, 2, 1
    rot = hd if rot is None else rot
    lens = [5, 37]
    table, slots, page_stride, kp, vp = paged_setup(lens, page, nkv, hd, layers, act, 70)
    T = sum(lens)
    qkv = rnd((T, (nh + 2 * nkv) * hd), torch.float32, 71)
    positions = torch.cat([torch.arange(n) for n in lens]).to(torch.int32)
    slot_of = torch.cat([torch.full((n,), s) for n, s in zip(lens, slots)]).to(torch.int32)
    inv_freq = torch.from_numpy(rope_frequencies(rot, 10000.0))
    kd, vd = kp.to(DEV), vp.to(DEV)
    off = layer * nkv * page * hd
    q = ops.rope_kv_write(qkv.to(DEV), positions.to(DEV), slot_of.to(DEV), table.to(DEV), inv_freq.to(DEV),
                          0 if pairing == "half" else 1, rot, kd, vd, off, page, page_stride, nh, nkv, hd, act).cpu()
    x = qkv.view(T, nh + 2 * nkv, hd).double()
    qref = plain_rope(x[:, :nh], positions.tolist(), 10000.0, pairing, rot)
    kref = plain_rope(x[:, nh:nh + nkv], positions.tolist(), 10000.0, pairing, rot)
    assert (q.double().view(T, nh, hd) - qref).abs().max() < tol(act, 4)
    kc, vc = kd.cpu(), vd.cpu()
    for t in range(T):
        p, s = int(positions[t]), int(slot_of[t])
        base = int(table[s, p // page]) * page_stride + off + (p % page) * hd     # kv head 0
        assert (kc[base:base + hd].double() - kref[t, 0]).abs().max() < tol(act, 4)
        vbase = int(table[s, p // page]) * page_stride + off + p % page                # values lie [hd][row]
        assert (vc[vbase:vbase + hd * page:page].double() - x[t, nh + nkv]).abs().max() < tol(act, 4)
    # nothing outside the written rows was touched
    assert int((kc != 0).sum()) <= T * nkv * hd and int((vc != 0).sum()) <= T * nkv * hd


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("bias_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,page", [(3, 1, 48, 64), (2, 2, 18, 64)])
def test_rotation_adds_a_bias_that_the_product_left_out(ops, act, bias_dtype, nh, nkv, hd, page):
    """Given the bias, the rotation kernel reads qkv + bias: queries and pages hold the bits they hold when the
    bias was added beforehand, token by token and by tiles of a run's values."""
    from plain_qwen2moe import rope_frequencies
    starts, news = [0, 37, 5], [150, 100, 9]
    lens = [a + b for a, b in zip(starts, news)]
    table, slots, page_stride, kp, vp = paged_setup(lens, page, nkv, hd, 2, act, 112)
    off = nkv * page * hd
    T = sum(news)
    width = (nh + 2 * nkv) * hd
    qkv = rnd((T, width), torch.float32, 113).to(DEV)
    bias = rnd((width,), bias_dtype, 114).to(DEV)
    positions = torch.cat([torch.arange(a, a + b) for a, b in zip(starts, news)]).to(torch.int32)
    slot_of = torch.cat([torch.full((b,), s) for s, b in zip(slots, news)]).to(torch.int32)
    freqs = torch.from_numpy(rope_frequencies(hd, 1e4))
    cu = torch.tensor([0] + list(torch.tensor(news).cumsum(0)), dtype=torch.int32)
    runs = {"cu_seqlens": cu.to(DEV), "slots": torch.tensor(slots, dtype=torch.int32).to(DEV),
            "start": torch.tensor(starts, dtype=torch.int32).to(DEV), "max_new": max(news), "max_end": max(lens), "decode": False}
    for r in (None, runs):
        got = []
        for late in (True, False):
            kd, vd = kp.to(DEV).clone(), vp.to(DEV).clone()
            q = ops.rope_kv_write(qkv if late else qkv + bias.float(), positions.to(DEV), slot_of.to(DEV), table.to(DEV),
                                  freqs.to(DEV), 0, hd, kd, vd, off, page, page_stride, nh, nkv, hd, act, runs=r,
                                  bias=bias if late else None)
            got.append((q.cpu(), kd.cpu(), vd.cpu()))
        for x, y in zip(*got):
            assert torch.equal(x, y)
        assert not torch.equal(got[0][0], ops.rope_kv_write(qkv, positions.to(DEV), slot_of.to(DEV), table.to(DEV),
                                                            freqs.to(DEV), 0, hd, None, None, off, page, page_stride, nh,
                                                            nkv, hd, act).cpu())
    with pytest.raises(ops.KernelError, match="bias"):
        ops.rope_kv_write(qkv, positions.to(DEV), slot_of.to(DEV), table.to(DEV), freqs.to(DEV), 0, hd, None, None, off, page,
                          page_stride, nh, nkv, hd, act, bias=bias[:-1])


@pytest.mark.parametrize("T", [700])
def test_queries_keys_values_of_a_long_prompt(ops, T, monkeypatch):
    """A long prompt's product of q, k and v goes to the vendor's library without its bias, which the rotation adds:
    queries and pages are those of this library's own product with the bias in it, up to the order of sums."""
    from plain_qwen2moe import rope_frequencies
    act, nh, nkv, hd, H, page = "bfloat16", 6, 2, 64, 264, 64
    monkeypatch.setattr(ops, "VENDOR_MIN_ROWS", 512)
    table, slots, page_stride, kp, vp = paged_setup([T], page, nkv, hd, 1, act, 174)
    a = rnd((T, H), adt(act), 175).to(DEV)
    w = rnd(((nh + 2 * nkv) * hd, H), adt(act), 176, 0.2).to(DEV)
    b = rnd(((nh + 2 * nkv) * hd,), adt(act), 177).to(DEV)
    positions = torch.arange(T, dtype=torch.int32).to(DEV)
    slot_of = torch.full((T,), slots[0], dtype=torch.int32).to(DEV)
    freqs = torch.from_numpy(rope_frequencies(hd, 1e6)).to(DEV)
    out = []
    for vendor in (True, False):
        monkeypatch.setattr(ops, "_VENDOR", vendor)
        kd, vd = kp.to(DEV).clone(), vp.to(DEV).clone()
        q = ops.qkv_rope_write(a, w, b, positions, slot_of, table.to(DEV), freqs, 0, hd, kd, vd, 0, page, page_stride, nh, nkv,
                               hd, act)
        out.append((q.cpu().float(), kd.cpu().float(), vd.cpu().float()))
    scale = out[1][0].abs().max().item()
    for x, y in zip(*out):
        assert (x - y).abs().max().item() <= 1.6e-2 * scale
    nobias = ops.qkv_rope_write(a, w, None, positions, slot_of, table.to(DEV), freqs, 0, hd, None, None, 0, page, page_stride,
                                nh, nkv, hd, act).cpu().float()
    assert (nobias - out[0][0]).abs().max().item() > 0.1 * scale


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("nh,nkv,hd,page", [(3, 1, 48, 64), (4, 2, 128, 128), (2, 2, 16, 64)])
def test_values_of_whole_runs_are_written_by_tiles(ops, act, nh, nkv, hd, page):
    """Told that the tokens are runs of consecutive positions, the kernel writes the values of whole prompts by
    tiles of 64 positions; the pages must hold the same bits as after the token-by-token write, for runs that
    start in the middle of a page, end in the middle of one, span several pages or are a single token."""
    from plain_qwen2moe import rope_frequencies
    starts, news = [0, 37, 64, 130, 5], [150, 100, 64, 1, 9]
    lens = [a + b for a, b in zip(starts, news)]
    table, slots, page_stride, kp, vp = paged_setup(lens, page, nkv, hd, 2, act, 110)
    off = nkv * page * hd
    T = sum(news)
    qkv = rnd((T, (nh + 2 * nkv) * hd), torch.float32, 111)
    positions = torch.cat([torch.arange(a, a + b) for a, b in zip(starts, news)]).to(torch.int32)
    slot_of = torch.cat([torch.full((b,), s) for s, b in zip(slots, news)]).to(torch.int32)
    freqs = torch.from_numpy(rope_frequencies(hd, 1e4))
    cu = torch.tensor([0] + list(torch.tensor(news).cumsum(0)), dtype=torch.int32)
    runs = {"cu_seqlens": cu.to(DEV), "slots": torch.tensor(slots, dtype=torch.int32).to(DEV),
            "start": torch.tensor(starts, dtype=torch.int32).to(DEV), "max_new": max(news), "max_end": max(lens), "decode": False}
    pages = []
    for r in (None, runs):
        kd, vd = kp.to(DEV).clone(), vp.to(DEV).clone()
        q = ops.rope_kv_write(qkv.to(DEV), positions.to(DEV), slot_of.to(DEV), table.to(DEV), freqs.to(DEV), 0, hd, kd, vd,
                              off, page, page_stride, nh, nkv, hd, act, runs=r)
        pages.append((q.cpu(), kd.cpu(), vd.cpu()))
    for a, b in zip(*pages):
        assert torch.equal(a, b)
    assert int((pages[0][2] != 0).sum()) > T * nkv * hd // 2


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("nh,nkv,hd,H,bias,write", [(3, 1, 64, 264, True, True), (16, 16, 128, 2048, True, True), (5, 5, 32, 72, False, True),
                                                    (6, 2, 96, 136, True, False), (4, 2, 48, 136, True, True)])
def test_queries_keys_values_in_one_launch(ops, act, nh, nkv, hd, H, bias, write):
    """The product of q, k, v with rotation and cache write behind it, asked for as one operation: up to 16 tokens
    in bfloat16 go out in one launch (head sizes that are multiples of 32), and queries and pages hold what the
    product followed by the rotation kernel gives; other sizes are those two calls."""
    from plain_qwen2moe import rope_frequencies
    page, layers, layer = 64, 2, 1
    starts, T_each = [3, 70, 0, 129], [1, 1, 1, 1]
    lens = [a + b for a, b in zip(starts, T_each)]
    table, slots, page_stride, kp, vp = paged_setup(lens, page, nkv, hd, layers, act, 170)
    off = layer * nkv * page * hd
    for T in (1, 4):
        positions = torch.tensor(starts[:T], dtype=torch.int32)
        slot_of = torch.tensor(slots[:T], dtype=torch.int32)
        a = rnd((T, H), adt(act), 171)
        w = rnd(((nh + 2 * nkv) * hd, H), adt(act), 172, 0.2)
        b = rnd(((nh + 2 * nkv) * hd,), adt(act), 173) if bias else None
        freqs = torch.from_numpy(rope_frequencies(hd, 1e6))
        out = []
        for fused in (True, False):
            kd, vd = kp.to(DEV).clone(), vp.to(DEV).clone()
            args = (positions.to(DEV), slot_of.to(DEV), table.to(DEV), freqs.to(DEV), 0, hd, kd if write else None,
                    vd if write else None, off, page, page_stride, nh, nkv, hd, act)
            if fused:
                q = ops.qkv_rope_write(a.to(DEV), w.to(DEV), None if b is None else b.to(DEV), *args)
            else:
                q = ops.rope_kv_write(ops.gemm(a.to(DEV), w.to(DEV), act, bias=None if b is None else b.to(DEV)), *args)
            out.append((q.cpu().float(), kd.cpu().float(), vd.cpu().float()))
        scale = out[1][0].abs().max().item()
        lim = 1e-5 * scale if act == "float32" else 1.6e-2 * scale        # two roundings to bfloat16 of sums in another order
        for x, y in zip(*out):
            assert (x - y).abs().max().item() <= lim
        if write:
            assert int((out[0][1] != 0).sum()) > T * nkv * hd // 2 and int((out[0][2] != 0).sum()) > T * nkv * hd // 2
            assert torch.equal(out[0][1] != 0, out[1][1] != 0) or act == "bfloat16"      # the same rows and nothing else
            assert int((out[0][1] != 0).sum()) <= T * nkv * hd and int((out[0][2] != 0).sum()) <= T * nkv * hd
        else:
            assert int((out[0][1] != 0).sum()) == 0 and int((out[0][2] != 0).sum()) == 0


def test_rope_pairings_are_one_rotation(ops):
    """interleaved(P x) = P half(x) for the permutation P that interleaves the two halves."""
    from plain_qwen2moe import rope as plain_rope
    hd = 16
    x = rnd((4, 2, hd), torch.float64, 72)
    perm = torch.tensor([i // 2 + (hd // 2) * (i % 2) for i in range(hd)])    # P x: (x0, x8, x1, x9, ...)
    pos = [0, 3, 17, 100]
    a = plain_rope(x[..., perm], pos, 10000.0, "interleaved")
    b = plain_rope(x, pos, 10000.0, "half")[..., perm]
    assert (a - b).abs().max() < 1e-12


def ref_attention(q, k, v, window, scale):
    from plain_qwen2moe import attention
    return attention(q.double(), k.double(), v.double(), window=window, scale=scale)


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("nh,nkv,hd,window,page", [(4, 4, 16, None, 16), (6, 2, 48, 24, 64), (3, 1, 80, 5, 16),
                                                     (8, 4, 128, None, 64), (5, 5, 32, 1, 16)])
def test_attention_over_pages(ops, act, nh, nkv, hd, window, page):
    """Whole sequences of unequal length in one call, and the last token of each alone (as in decoding),
    against the plain attention."""
    lens = [1, 19, 150]
    layers, layer = 2, 1
    table, slots, page_stride, kp, vp = paged_setup(lens, page, nkv, hd, layers, act, 80)
    off = layer * nkv * page * hd
    scale = 1.0 / math.sqrt(hd)
    qs, ks, vs = [], [], []
    for i, n in enumerate(lens):
        qs.append(rnd((n, nh, hd), adt(act), 81 + i))
        ks.append(rnd((n, nkv, hd), adt(act), 84 + i))
        vs.append(rnd((n, nkv, hd), adt(act), 87 + i))
        for p in range(n):
            for h in range(nkv):
                base = int(table[slots[i], p // page]) * page_stride + off + (h * page + p % page) * hd
                kp[base:base + hd] = ks[i][p, h]
                vbase = int(table[slots[i], p // page]) * page_stride + off + h * page * hd + p % page
                vp[vbase:vbase + hd * page:page] = vs[i][p, h]
    positions = torch.cat([torch.arange(n) for n in lens]).to(torch.int32)
    slot_of = torch.cat([torch.full((n,), s) for n, s in zip(lens, slots)]).to(torch.int32)
    q = torch.cat(qs).reshape(-1, nh * hd)
    kd, vd, td = kp.to(DEV), vp.to(DEV), table.to(DEV)
    out = ops.attention(q.to(DEV), kd, vd, off, positions.to(DEV), slot_of.to(DEV), td, page, page_stride, nh, nkv,
                        hd, window, scale, act).cpu()
    ref = torch.cat([ref_attention(a, b, c, window, scale) for a, b, c in zip(qs, ks, vs)]).reshape(-1, nh * hd)
    assert (out.double() - ref).abs().max() < tol(act, 2)
    last = torch.tensor([sum(lens[:i + 1]) - 1 for i in range(len(lens))])
    out1 = ops.attention(q[last].contiguous().to(DEV), kd, vd, off, positions[last].to(DEV), slot_of[last].to(DEV),
                         td, page, page_stride, nh, nkv, hd, window, scale, act).cpu()
    assert (out1.double() - ref[last]).abs().max() < tol(act, 2)


@pytest.mark.parametrize("act", ACTS)
def test_attention_finds_a_far_key(ops, act):
    """One key among hundreds is made to stand out; its value must come through, whichever page it lies in."""
    nh = nkv = 2
    hd, page, n = 32, 16, 300
    table, slots, page_stride, kp, vp = paged_setup([n], page, nkv, hd, 1, act, 90)
    q = torch.zeros((1, nh, hd))
    q[0, :, 0] = 8.0
    k = rnd((n, nkv, hd), torch.float32, 91, 0.1)
    v = rnd((n, nkv, hd), torch.float32, 92)
    far = 37
    k[far, :, 0] = 40.0
    for p in range(n):
        for h in range(nkv):
            base = int(table[slots[0], p // page]) * page_stride + (h * page + p % page) * hd
            kp[base:base + hd] = k[p, h].to(adt(act))
            vbase = int(table[slots[0], p // page]) * page_stride + h * page * hd + p % page
            vp[vbase:vbase + hd * page:page] = v[p, h].to(adt(act))
    out = ops.attention(q.reshape(1, -1).to(adt(act)).to(DEV), kp.to(DEV), vp.to(DEV), 0,
                        torch.tensor([n - 1], dtype=torch.int32).to(DEV),
                        torch.tensor([slots[0]], dtype=torch.int32).to(DEV), table.to(DEV), page, page_stride, nh,
                        nkv, hd, None, 1.0 / math.sqrt(hd), act).cpu()
    assert (out.float().view(nh, hd) - v[far].to(adt(act)).float()).abs().max() < 1e-2
    # with a window that ends before the far key, it is not seen
    out_w = ops.attention(q.reshape(1, -1).to(adt(act)).to(DEV), kp.to(DEV), vp.to(DEV), 0,
                          torch.tensor([n - 1], dtype=torch.int32).to(DEV),
                          torch.tensor([slots[0]], dtype=torch.int32).to(DEV), table.to(DEV), page, page_stride, nh,
                          nkv, hd, n - 1 - far, 1.0 / math.sqrt(hd), act).cpu()
    assert (out_w.float().view(nh, hd) - v[far].float()).abs().max() > 0.5
    out_w2 = ops.attention(q.reshape(1, -1).to(adt(act)).to(DEV), kp.to(DEV), vp.to(DEV), 0,
                           torch.tensor([n - 1], dtype=torch.int32).to(DEV),
                           torch.tensor([slots[0]], dtype=torch.int32).to(DEV), table.to(DEV), page, page_stride, nh,
                           nkv, hd, n - far, 1.0 / math.sqrt(hd), act).cpu()
    assert (out_w2.float().view(nh, hd) - v[far].to(adt(act)).float()).abs().max() < 1e-2


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("window", [None, 3000])
def test_decoding_over_long_caches(ops, act, window):
    """One token per sequence at positions on both sides of the length at which the split kernel changes the
    length of its runs (4096), of other multiples of 2048 and well beyond, in one batch: the sequences of 3,500 and
    4,095 tokens have more runs (one per 64 positions) than the longest one (one per 192), after which the grid is
    sized.  In each sequence one far key stands out a little, so that a run that is skipped or joined twice shows.
    Against the plain formula for the last token."""
    nh, nkv, hd, page = 6, 2, 64, 64
    lens = [2047, 2048, 2049, 4095, 4097, 6143, 6145, 9001, 130, 3500]
    table, slots, page_stride, kp, vp = paged_setup(lens, page, nkv, hd, 1, act, 95)
    scale = 1.0 / math.sqrt(hd)
    g = torch.Generator().manual_seed(96)
    qs, want = [], []
    kp3, vp3 = kp.view(-1, nkv, page, hd), vp.view(-1, nkv, hd, page)          # [page][kv head][row][hd], values transposed
    for i, n in enumerate(lens):
        q = torch.randn((nh, hd), generator=g).to(adt(act))
        k = (0.5 * torch.randn((n, nkv, hd), generator=g)).to(adt(act))
        v = torch.randn((n, nkv, hd), generator=g).to(adt(act))
        far = (n * 37) // 100
        k[far] = (q.float().view(nkv, nh // nkv, hd)[:, 0] * 0.6).to(adt(act))     # a score that stands out
        pos = torch.arange(n)
        pages = table[slots[i], (pos // page).long()].long()
        kp3[pages, :, pos % page, :] = k
        vp3[pages, :, :, pos % page] = v
        lo = 0 if window is None or n <= window else n - window
        kk, vv = k.double()[lo:], v.double()[lo:]
        out = torch.empty((nh, hd), dtype=torch.float64)
        for h in range(nh):
            kvh = h // (nh // nkv)
            pr = torch.softmax((kk[:, kvh] @ q[h].double()) * scale, dim=0)
            out[h] = pr @ vv[:, kvh]
        qs.append(q)
        want.append(out.reshape(-1))
    B = len(lens)
    positions = torch.tensor([n - 1 for n in lens], dtype=torch.int32)
    runs = {"cu_seqlens": torch.arange(B + 1, dtype=torch.int32).to(DEV), "slots": torch.tensor(slots, dtype=torch.int32).to(DEV),
            "start": positions.to(DEV), "max_new": 1, "max_end": max(lens), "decode": True}
    out = ops.attention(torch.stack(qs).reshape(B, nh * hd).to(DEV), kp.to(DEV), vp.to(DEV), 0, positions.to(DEV),
                        torch.tensor(slots, dtype=torch.int32).to(DEV), table.to(DEV), page, page_stride, nh, nkv, hd,
                        window, scale, act, runs=runs).cpu()
    err = (out.double() - torch.stack(want)).abs().max(dim=1).values
    assert err.max() < (2e-5 if act == "float32" else 2e-2), err
    # each sequence alone gives the same bits: what a run is depends on the token's position only
    for i in (1, 3, 4, 7):
        runs1 = {"cu_seqlens": torch.tensor([0, 1], dtype=torch.int32).to(DEV), "slots": torch.tensor([slots[i]], dtype=torch.int32).to(DEV),
                 "start": positions[i:i + 1].to(DEV), "max_new": 1, "max_end": lens[i], "decode": True}
        alone = ops.attention(qs[i].reshape(1, nh * hd).to(DEV), kp.to(DEV), vp.to(DEV), 0, positions[i:i + 1].to(DEV),
                              torch.tensor([slots[i]], dtype=torch.int32).to(DEV), table.to(DEV), page, page_stride, nh, nkv,
                              hd, window, scale, act, runs=runs1).cpu()
        assert torch.equal(alone[0], out[i])
    # and so does a step with so many waves that the kernel does not fetch tiles ahead (the batch four times over)
    rep = 4
    runs4 = {"cu_seqlens": torch.arange(rep * B + 1, dtype=torch.int32).to(DEV), "slots": torch.tensor(slots * rep, dtype=torch.int32).to(DEV),
             "start": positions.repeat(rep).to(DEV), "max_new": 1, "max_end": max(lens), "decode": True}
    out4 = ops.attention(torch.stack(qs * rep).reshape(rep * B, nh * hd).to(DEV), kp.to(DEV), vp.to(DEV), 0,
                         positions.repeat(rep).to(DEV), torch.tensor(slots * rep, dtype=torch.int32).to(DEV), table.to(DEV), page,
                         page_stride, nh, nkv, hd, window, scale, act, runs=runs4).cpu()
    assert torch.equal(out4, out.repeat(rep, 1))


@pytest.mark.parametrize("hd,nh,nkv", [(128, 16, 16), (128, 28, 4), (64, 8, 8)])
def test_decoding_with_tiles_fetched_ahead_gives_the_same_bits(ops, hd, nh, nkv):
    """A decode step of few waves (up to one per SIMD) runs the form of the kernel that keeps the next tile of keys
    and values in registers; a token's result is the same bits as in a step of many sequences, at positions below and
    beyond 4,096 (runs of one and of three tiles) and with a window."""
    act, page = "bfloat16", 64
    lens = [100, 2500, 4097, 8200]
    table, slots, page_stride, kp, vp = paged_setup(lens, page, nkv, hd, 1, act, 97)
    kp.copy_(rnd((kp.numel(),), adt(act), 98, 0.5))
    vp.copy_(rnd((vp.numel(),), adt(act), 99))
    scale = 1.0 / math.sqrt(hd)
    B, rep = len(lens), 40
    q = rnd((B, nh * hd), adt(act), 100)
    positions = torch.tensor([n - 1 for n in lens], dtype=torch.int32)
    for window in (None, 3000):
        def run(idx):
            n = len(idx)
            runs = {"cu_seqlens": torch.arange(n + 1, dtype=torch.int32).to(DEV),
                    "slots": torch.tensor([slots[i] for i in idx], dtype=torch.int32).to(DEV),
                    "start": positions[idx].to(DEV), "max_new": 1, "max_end": max(lens[i] for i in idx), "decode": True}
            return ops.attention(q[idx].to(DEV), kp.to(DEV), vp.to(DEV), 0, positions[idx].to(DEV), runs["slots"], table.to(DEV), page,
                                 page_stride, nh, nkv, hd, window, scale, act, runs=runs).cpu()
        many = run(list(range(B)) * rep)          # 160 sequences: thousands of waves
        assert many.abs().max() > 0.01
        for i in range(B):
            assert torch.equal(run([i])[0], many[i]) and torch.equal(many[i], many[i + B * (rep - 1)])


# ------------------------------------------------------------------------------------------------ sampling
@pytest.mark.parametrize("V", [10, 1000, 151937])
def test_negative_log_likelihood(ops, V):
    """-log softmax at a given token, per row, against float64; a row with one towering logit (no overflow), and a
    target that is no token (NaN, for the caller to leave out)."""
    logits = rnd((5, V), torch.float32, 98, 3.0)
    logits[1, V // 2] = 300.0
    logits[2] = -1000.0
    targets = torch.tensor([0, V // 2, V - 1, V, -1], dtype=torch.int32)
    out = ops.nll(logits.to(DEV), targets.to(DEV), "float32").cpu().double()
    ref = -torch.log_softmax(logits.double(), dim=-1)
    for r in range(3):
        assert abs(out[r] - ref[r, int(targets[r])]) < 1e-5 * max(1.0, float(ref[r, int(targets[r])])), r
    assert torch.isnan(out[3]) and torch.isnan(out[4])


@pytest.mark.parametrize("V", [10, 1000, 40001])
def test_probabilities_in_16_bits_and_their_divergence(ops, V):
    """A row's probabilities as the reference stores them (/root/reference/tools/quant.c:166-174, :594-602: made in
    double, cut to a float and then to a 16-bit float whose mantissa is cut and whose small values are zero) and the
    divergence of a baseline of such rows against them (:623-631), each against the same formulas in numpy."""
    import numpy as np
    R = 5
    logits = rnd((R, V), torch.float32, 120, 3.0)
    logits[1, 3] = 40.0                                    # one towering logit: everything else is cut to zero
    other = logits + rnd((R, V), torch.float32, 121, 0.3)
    def widen(h):
        h = h.astype(np.uint32)
        e, m = (h >> 10) & 0x1f, h & 0x3ff
        return np.where(e == 0, 0, ((e + 112) << 23) | (m << 13)).astype(np.uint32).view(np.float32)
    def cut(p):
        bits = p.astype(np.float32).view(np.uint32)
        e = ((bits >> 23) & 0xff).astype(np.int64) - 127 + 15
        return np.where(e <= 0, 0, (e.clip(0, 30) << 10) | ((bits >> 13) & 0x3ff)).astype(np.uint16)
    probs, none = ops.probs_half(logits.to(DEV), "float32")
    assert none is None and probs.dtype == torch.int16
    got = probs.cpu().numpy().view(np.uint16)
    l64 = logits.double().numpy()
    p = np.exp((l64 - l64.max(1, keepdims=True)) - np.log(np.exp(l64 - l64.max(1, keepdims=True)).sum(1, keepdims=True)))
    want = cut(p)
    assert (np.abs(got.astype(np.int64) - want.astype(np.int64)) <= 1).all() and (got == want).mean() > 0.999
    assert (got[1] != 0).sum() == 1
    base, _ = ops.probs_half(other.to(DEV), "float32")
    same, kl = ops.probs_half(logits.to(DEV), "float32", want_probs=True, base=base)
    assert torch.equal(same, probs) and kl.dtype == torch.float64
    pb, pc = widen(base.cpu().numpy().view(np.uint16)).astype(np.float64), widen(got).astype(np.float64)
    ref = np.where(pb > 1e-12, pb * (np.log(np.maximum(pb, 1e-300)) - np.log(np.maximum(pc, 1e-20))), 0.0).sum(1)
    assert np.allclose(kl.cpu().numpy(), ref, rtol=1e-9, atol=1e-12)
    zero = ops.probs_half(logits.to(DEV), "float32", want_probs=False, base=probs)[1]
    assert torch.equal(zero, torch.zeros(R, dtype=torch.float64, device=zero.device))
    with pytest.raises(ops.KernelError):
        ops.probs_half(logits.to(DEV), "float32", want_probs=False)


@pytest.mark.parametrize("V", [10, 1000, 151937])
def test_argmax_first_maximum(ops, V):
    logits = rnd((3, V), torch.float32, 100)
    logits[1, V // 3] = logits[1, V - 1] = 50.0          # equal maxima: the first wins
    logits[2, :] = 0.0
    out = ops.argmax(logits.to(DEV), "float32").cpu().tolist()
    assert out == [int(torch.argmax(logits[0])), V // 3, 0]
    # the vectors of /root/reference/tests/test_ops.cpp:528-542
    v = torch.tensor([[1.0, 5.0, 3.0, 2.0], [-3.0, -1.0, -2.0, -5.0]])
    assert ops.argmax(v.to(DEV), "float32").cpu().tolist() == [1, 1]


def test_rep_penalty(ops):
    from plain_qwen2moe import apply_rep_penalty
    V = 50
    logits = rnd((2, V), torch.float32, 110)
    recent = torch.tensor([[3, 7, 3, -1], [49, 0, 1, 2]], dtype=torch.int32)
    counts = torch.tensor([3, 4], dtype=torch.int32)
    d = logits.clone().to(DEV)
    ops.rep_penalty(d, recent.to(DEV), counts.to(DEV), 1.1, "float32")
    ref = logits.numpy().copy()
    apply_rep_penalty(ref[0], [3, 7, 3], 4, 1.1)       # token 3 twice: penalised twice
    apply_rep_penalty(ref[1], [2, 1, 0, 49], 4, 1.1)
    assert (d.cpu() - torch.from_numpy(ref)).abs().max() < 1e-6
    # histories of 100 entries (a thread per entry) and of 200 (one thread walks them), tokens drawn from 20 so that
    # most occur several times; the same bits as the walk in float32
    g = torch.Generator().manual_seed(111)
    for window in (100, 200):
        logits = rnd((3, V), torch.float32, 112)
        recent = torch.randint(0, 20, (3, window), generator=g).to(torch.int32)
        counts = torch.tensor([window, window // 2, 0], dtype=torch.int32)
        d = logits.clone().to(DEV)
        ops.rep_penalty(d, recent.to(DEV), counts.to(DEV), 1.3, "float32")
        ref = logits.numpy().copy()
        for r in range(3):
            n = int(counts[r])
            apply_rep_penalty(ref[r], recent[r, :n].tolist()[::-1], window, 1.3)
        assert torch.equal(d.cpu(), torch.from_numpy(ref)), window


def test_sample_topp_against_plain(ops):
    """Same logits, same uniform draws: the kernel's choice is the plain sorted walk's choice."""
    from plain_qwen2moe import sample_topp

    class Fixed:
        def __init__(self, u):
            self.u = u

        def next(self):
            return self.u

    g = torch.Generator().manual_seed(120)
    # (the last: logits in steps of 1/2, so that many probabilities are equal and the order of indices decides)
    for V, T, P, step in [(4, 0.7, 0.9, 0), (97, 0.7, 0.9, 0), (1000, 1.3, 0.5, 0), (5000, 0.3, 0.95, 0),
                          (300, 0.7, 1.0, 0), (2000, 1.5, 0.97, 0.5)]:
        logits = 3 * torch.randn((16, V), generator=g)
        if step:
            logits = torch.round(logits / step) * step
        u = torch.rand((16,), generator=g)
        got = ops.sample_topp(logits.to(DEV), T, P, u.to(DEV), "float32").cpu().tolist()
        want = [sample_topp(logits[r].numpy(), T, P, Fixed(float(u[r]))) for r in range(16)]
        assert got == want, (V, T, P)


def sorted_walk_in_float64(logits, T, P, u, tol):
    """The reference's walk (/root/reference/src/engine/tq_generate.c:81-156) with every sum in float64: the
    token, and whether the same token comes out when every running sum is off by up to tol of itself (the place
    where top_p is reached may then move, and with it the sum that the draw is scaled by)."""
    l = logits.astype(np.float64)
    p = np.where(l >= l.max() - 16.0 * T, np.exp((l - l.max()) / T), 0.0)
    p /= p.sum()
    order = np.argsort(-p, kind="stable")
    cum = np.cumsum(p[order])

    def first_reaching(x):
        return int(np.argmax(cum >= x)) if (cum >= x).any() else len(cum) - 1

    r = u * cum[first_reaching(P)]
    k = first_reaching(r)
    r_lo = u * cum[first_reaching(P * (1 - tol))] * (1 - tol)
    r_hi = u * cum[first_reaching(P * (1 + tol))] * (1 + tol)
    return int(order[k]), first_reaching(r_lo) == k and first_reaching(r_hi) == k


def test_sample_topp_of_a_long_row(ops):
    """Rows of a real vocabulary's length, a length that is no multiple of 4, lengths that exceed what a workgroup
    loads at once, and logits in steps of 1/2 (many equal probabilities: the order of indices decides).  The plain
    float32 walk adds 100,000 terms one after the other and is itself off by 1e-5 or so there, so the kernel is
    held to the walk in float64 wherever that walk does not turn on 4e-6 of a sum, which is most rows.  (The
    kernel adds at most 20 values in a thread, then 6 + 4 + 32 partial sums: 62 roundings of 2^-24 each at worst.)"""
    g = torch.Generator().manual_seed(121)
    for V, T, P, step in [(151936, 0.7, 0.9, 0), (70001, 1.0, 0.8, 0), (4000, 1.5, 0.97, 0.5), (151936, 1.0, 1.0, 0),
                          (300000, 0.4, 0.95, 0)]:
        logits = 3 * torch.randn((24, V), generator=g)
        if step:
            logits = torch.round(logits / step) * step
        u = torch.rand((24,), generator=g)
        got = ops.sample_topp(logits.to(DEV), T, P, u.to(DEV), "float32").cpu().tolist()
        clear = 0
        for r in range(24):
            want, is_clear = sorted_walk_in_float64(logits[r].numpy(), T, P, float(u[r]), 4e-6)
            if is_clear:
                clear += 1
                assert got[r] == want, (V, T, P, r)
        assert clear >= 18, (V, clear)


def test_sample_topp_distribution(ops):
    """/root/reference/tests/test_ops.cpp:544-571: T = 0.001 is greedy; uniform logits give each of 4 tokens
    between 10 % and 50 % of 1000 draws."""
    from turboquant_cpp_amd.sampling.rng import XorShift64Star
    logits = torch.tensor([[1.0, 5.0, 3.0, 2.0]])
    u = torch.tensor([0.73])
    assert ops.sample_topp(logits.to(DEV), 0.001, 0.9, u.to(DEV), "float32").cpu().tolist() == [1]
    rng = XorShift64Star(42)
    draws = torch.tensor([rng.next_float() for _ in range(1000)])
    out = ops.sample_topp(torch.zeros((1000, 4)).to(DEV), 1.0, 1.0, draws.to(DEV), "float32").cpu()
    counts = torch.bincount(out.long(), minlength=4)
    assert all(100 < int(c) < 500 for c in counts), counts


# ------------------------------------------------------------------------------------------------ tiled attention
@pytest.mark.parametrize("nh,nkv,hd,window,page", [(4, 4, 16, None, 64), (6, 2, 48, 24, 64), (3, 1, 80, 70, 128),
                                                     (16, 16, 128, None, 64), (40, 2, 32, 200, 64), (2, 1, 256, None, 64),
                                                     (5, 5, 96, 1, 64), (8, 2, 64, 100, 64),
                                                     # enough heads for two token groups per wave
                                                     (48, 6, 128, None, 64), (48, 4, 64, 100, 64), (44, 4, 48, 30, 64),
                                                     # head sizes that are a multiple of 4 only (the 32-bit kernels take them)
                                                     (6, 2, 24, 24, 64), (3, 3, 20, None, 64)])
@pytest.mark.parametrize("act", ACTS)
def test_attention_tiled(ops, act, nh, nkv, hd, window, page):
    """The matrix-core kernels of both types (whole runs of tokens, and one token per sequence split over the cache)
    against the plain attention: unequal lengths, a sequence that goes on from a cached prefix, groups of more than
    16 heads."""
    lens = [1, 19, 150, 333]
    layers, layer = 3, 1
    table, slots, page_stride, kp, vp = paged_setup(lens, page, nkv, hd, layers, act, 130)
    off = layer * nkv * page * hd
    scale = 1.0 / math.sqrt(hd)
    qs, ks, vs = [], [], []
    for i, n in enumerate(lens):
        qs.append(rnd((n, nh, hd), adt(act), 131 + i))
        ks.append(rnd((n, nkv, hd), adt(act), 135 + i))
        vs.append(rnd((n, nkv, hd), adt(act), 139 + i))
        for p in range(n):
            for h in range(nkv):
                base = int(table[slots[i], p // page]) * page_stride + off + (h * page + p % page) * hd
                kp[base:base + hd] = ks[i][p, h]
                vbase = int(table[slots[i], p // page]) * page_stride + off + h * page * hd + p % page
                vp[vbase:vbase + hd * page:page] = vs[i][p, h]
    kd, vd, td = kp.to(DEV), vp.to(DEV), table.to(DEV)
    ref = [ref_attention(a, b, c, window, scale).reshape(-1, nh * hd) for a, b, c in zip(qs, ks, vs)]

    def run(first):          # tokens first[i] .. lens[i]-1 of every sequence in one call
        new = [n - f for n, f in zip(lens, first)]
        keep = [i for i, n in enumerate(new) if n > 0]
        positions = torch.cat([torch.arange(first[i], lens[i]) for i in keep]).to(torch.int32)
        slot_of = torch.cat([torch.full((new[i],), slots[i]) for i in keep]).to(torch.int32)
        q = torch.cat([qs[i][first[i]:] for i in keep]).reshape(-1, nh * hd)
        cu = torch.tensor([0] + list(torch.tensor([new[i] for i in keep]).cumsum(0)), dtype=torch.int32)
        runs = {"cu_seqlens": cu.to(DEV), "slots": torch.tensor([slots[i] for i in keep], dtype=torch.int32).to(DEV),
                "start": torch.tensor([first[i] for i in keep], dtype=torch.int32).to(DEV),
                "max_new": max(new), "max_end": max(lens[i] for i in keep), "decode": all(new[i] == 1 for i in keep)}
        out = ops.attention(q.to(DEV), kd, vd, off, positions.to(DEV), slot_of.to(DEV), td, page, page_stride, nh, nkv,
                            hd, window, scale, act, runs=runs).cpu()
        want = torch.cat([ref[i][first[i]:] for i in keep])
        return (out.double() - want).abs().max().item()

    assert run([0, 0, 0, 0]) < tol(act, 2)                       # whole prompts
    assert run([0, 7, 100, 300]) < tol(act, 2)                   # runs that go on from a cached prefix
    assert run([n - 1 for n in lens]) < tol(act, 2)              # one token each: the split kernel
    assert run([1, 18, 149, 200]) < tol(act, 2)                  # mixed: not all single tokens


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("hd", [96, 160, 224, 40])
def test_decoding_reads_nothing_beyond_a_head_that_fills_no_whole_tile(ops, act, hd):
    """One token per sequence with head sizes between the kernels' tile widths (96 lies between 64 and 128): the
    sequence's last page is the pool's last, its kv head the last of the last layer, and what lies behind the pools
    is NaN.  A load that does not stop at the head size reads those and the scores of keys in reach become NaN."""
    nh, nkv, page, layers = 4, 2, 64, 2
    layer = layers - 1
    lens = [70, 129]
    n_pages = sum(-(-n // page) for n in lens)
    page_stride = layers * nkv * page * hd
    table = torch.full((2, 3), -1, dtype=torch.int32)
    table[0, :2] = torch.tensor([1, 0])
    table[1, :3] = torch.tensor([2, 3, n_pages - 1])            # the longer sequence ends in the pool's last page
    slots = [0, 1]
    off = layer * nkv * page * hd
    pools = []
    for seed in (0, 1):
        whole = torch.full((n_pages * page_stride + 65536,), float("nan"), dtype=adt(act))
        whole[:n_pages * page_stride] = 0
        pools.append(whole)
    kp, vp = (w[:n_pages * page_stride] for w in pools)
    scale = 1.0 / math.sqrt(hd)
    qs, ks, vs = [], [], []
    for i, n in enumerate(lens):
        qs.append(rnd((n, nh, hd), adt(act), 231 + i))
        ks.append(rnd((n, nkv, hd), adt(act), 235 + i))
        vs.append(rnd((n, nkv, hd), adt(act), 239 + i))
        for p in range(n):
            for h in range(nkv):
                base = int(table[slots[i], p // page]) * page_stride + off + (h * page + p % page) * hd
                kp[base:base + hd] = ks[i][p, h]
                vbase = int(table[slots[i], p // page]) * page_stride + off + h * page * hd + p % page
                vp[vbase:vbase + hd * page:page] = vs[i][p, h]
    kd, vd = (w.to(DEV)[:n_pages * page_stride] for w in pools)
    ref = [ref_attention(a, b, c, None, scale).reshape(-1, nh * hd) for a, b, c in zip(qs, ks, vs)]
    positions = torch.tensor([n - 1 for n in lens], dtype=torch.int32)
    q = torch.stack([qs[i][-1] for i in range(2)]).reshape(2, nh * hd)
    runs = {"cu_seqlens": torch.tensor([0, 1, 2], dtype=torch.int32).to(DEV),
            "slots": torch.tensor(slots, dtype=torch.int32).to(DEV), "start": positions.to(DEV),
            "max_new": 1, "max_end": max(lens), "decode": True}
    out = ops.attention(q.to(DEV), kd, vd, off, positions.to(DEV), torch.tensor(slots, dtype=torch.int32).to(DEV),
                        table.to(DEV), page, page_stride, nh, nkv, hd, None, scale, act, runs=runs).cpu()
    want = torch.stack([ref[i][-1] for i in range(2)])
    assert torch.isfinite(out).all()
    assert (out.double() - want).abs().max().item() < tol(act, 2)


def test_probes_run(ops):
    """The two kernels behind `bench.py --probe` (a plain read, the matrix instructions alone) do the work they are
    timed for: the read of 256 MiB takes at least as long as the memory's published rate allows and no more than
    twice what it took when measured (4.7 to 6.9 TB/s), and the matrix loop stays below the published peak and above
    two thirds of what it reached (1.85 to 2.45 PFLOP/s).  A kernel whose loop the compiler had emptied, or that read
    a fraction of the buffer, would be too fast; one that had lost its whole-line loads or its unrolling too slow."""
    def seconds(fn):
        fn()
        torch.cuda.synchronize()
        best = 1e9
        for _ in range(3):
            t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0.record()
            fn()
            t1.record()
            torch.cuda.synchronize()
            best = min(best, t0.elapsed_time(t1) * 1e-3)
        return best

    buf = torch.arange(1 << 26, dtype=torch.int32, device=DEV)
    nbytes = buf.numel() * 4
    for once in (False, True):
        rate = nbytes / seconds(lambda: ops.probe_stream(buf, once))
        assert (3.4e12 if once else 2.4e12) < rate < 8.0e12 * 1.05, (once, rate)
    assert ops.probe_mfma(32, 4, 10, 1, DEV) == 4 * 8 * 10 * 196608.0
    for shape in (32, 16):
        flop = [0.0]

        def run():
            flop[0] = ops.probe_mfma(shape, 512, 2000, 12345, DEV)
        t = seconds(run)
        rate = flop[0] / t
        assert 1.2e15 < rate < 2.5e15 * 1.02, (shape, rate)
