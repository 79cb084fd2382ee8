"""Kernel-level parity: each C-ABI entry point against a plain fp32/fp64 PyTorch statement of the
same op on the same seeded inputs.  Tolerances: max rel err (relative to max|ref| of the tensor)
<= 1e-5 for fp32, <= 2e-2 for fp16/bf16 (inputs are pre-rounded to the kernel dtype so the tolerance
measures kernel error only)."""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle
from tests.util import TOL, assert_close, rel_err

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16, torch.bfloat16]
DEV = "cuda:0"


def _ops():
    from terapipe_amd import ops
    return ops


def _rnd(shape, dtype, gen, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("M,E", [(32, 256), (7, 64), (256, 2048), (160, 5120), (33, 12288)])
def test_layernorm_fwd_bwd(dtype, M, E):
    ops = _ops()
    if dtype == torch.float32 and E > 8192 * 2:
        pytest.skip("fp32 rows above 16384 elements are outside the kernel's register cache")
    g = torch.Generator().manual_seed(M * 131 + E)
    x = _rnd((M, E), dtype, g) + 0.3
    gamma = (1 + 0.2 * torch.randn(E, generator=g)).to(dtype)
    beta = _rnd((E,), dtype, g, 0.1)
    dy = _rnd((M, E), dtype, g)
    dres = _rnd((M, E), dtype, g)
    xd, gd, bd, dyd, dresd = [t.to(DEV) for t in (x, gamma, beta, dy, dres)]
    y, mean, rstd = ops.layernorm_fwd(xd, gd, bd)
    x64 = x.double().requires_grad_(True)
    g64, b64 = gamma.double().requires_grad_(True), beta.double().requires_grad_(True)
    yref = F.layer_norm(x64, (E,), g64, b64, 1e-5)
    assert_close(y, yref, dtype, "ln y")
    assert_close(mean, x64.mean(-1), torch.float32, "ln mean", 10)
    yref.backward(dy.double())
    acc = torch.zeros(4, E, dtype=torch.float32, device=DEV)
    dx = ops.layernorm_bwd(dyd, xd, mean, rstd, gd, dresd, acc[0], acc[1], acc[2], acc[3])
    dx_ref = x64.grad + dres.double()
    assert_close(dx, dx_ref, dtype, "ln dx")
    # accumulators are fp32 sums of products of dtype-rounded inputs
    assert_close(acc[0], g64.grad, torch.float32, "ln dgamma", 20)
    assert_close(acc[1], b64.grad, torch.float32, "ln dbeta", 20)
    assert_close(acc[2], dres.double().sum(0), torch.float32, "colsum dres", 20)
    assert_close(acc[3], dx_ref.sum(0), dtype, "colsum dx", 1)
    # without the residual input
    acc.zero_()
    dx2 = ops.layernorm_bwd(dyd, xd, mean, rstd, gd, None, acc[0], acc[1], None, None)
    assert_close(dx2, x64.grad, dtype, "ln dx (no dres)")
    # dx only (no accumulators), parameter gradients by the all-rows reduction
    out = torch.empty_like(xd)
    dx3 = ops.layernorm_bwd(dyd, xd, mean, rstd, gd, dresd, None, None, None, None, out=out)
    assert dx3.data_ptr() == out.data_ptr()
    assert_close(dx3, dx_ref, dtype, "ln dx (no accumulators)")
    if E % 8 == 0:
        acc.zero_()
        ops.ln_param_grads(dyd, xd, mean, rstd, acc[0], acc[1])
        assert_close(acc[0], g64.grad, torch.float32, "ln_param_grads dgamma", 20)
        assert_close(acc[1], b64.grad, torch.float32, "ln_param_grads dbeta", 20)


GEMM_SHAPES = [
    # M, N, K
    (32, 256, 256),     # C1 out_proj
    (32, 768, 256),     # C1 in_proj
    (32, 256, 1024),    # C1 fc2
    (256, 2048, 2048),  # C2 out_proj (split-K)
    (160, 5120, 5120),  # C3 last slice
    (512, 15360, 5120),  # C3 in_proj, large-tile config
    (70, 136, 200),     # ragged everything
    (1, 8, 8),
]


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gemm_nt_nn_tn(dtype, M, N, K):
    ops = _ops()
    from terapipe_amd._lib import TP_GEMM_NN, TP_GEMM_NT, TP_GEMM_TN, TP_EPI_ACCUMULATE
    g = torch.Generator().manual_seed(M + 7 * N + 13 * K)
    sc = 1.0 / math.sqrt(K)
    # NT: C[M,N] = A[M,K] B[N,K]^T
    A, B = _rnd((M, K), dtype, g), _rnd((N, K), dtype, g, sc)
    C = torch.empty(M, N, dtype=dtype, device=DEV)
    ops.gemm(TP_GEMM_NT, A.to(DEV), B.to(DEV), M, N, K, C=C)
    assert_close(C, A.double() @ B.double().t(), dtype, "NT")
    # NN: C[M,N] = A[M,K] B[K,N]
    if N % 8 == 0:
        B2 = _rnd((K, N), dtype, g, sc)
        ops.gemm(TP_GEMM_NN, A.to(DEV), B2.to(DEV), M, N, K, C=C)
        assert_close(C, A.double() @ B2.double(), dtype, "NN")
    # TN: C[M2,N2] = A[K2,M2]^T B[K2,N2] with K2 = M (tokens), M2 = N, N2 = K: the weight-gradient shape
    if K % 8 == 0 and N % 8 == 0:
        dY, X = _rnd((M, N), dtype, g), _rnd((M, K), dtype, g, 1.0 / math.sqrt(M))
        W = torch.empty(N, K, dtype=dtype, device=DEV)
        ops.gemm(TP_GEMM_TN, dY.to(DEV), X.to(DEV), N, K, M, C=W)
        ref = dY.double().t() @ X.double()
        assert_close(W, ref, dtype, "TN")
        ops.gemm(TP_GEMM_TN, dY.to(DEV), X.to(DEV), N, K, M, C=W, epilogue=TP_EPI_ACCUMULATE)
        assert_close(W, 2 * ref, dtype, "TN accumulate")


TILE_CFGS = [0, 2, 3, 5, 6, 7, 8, 10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20] + list(range(21, 44))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("cfg", TILE_CFGS)
def test_gemm_every_tile_configuration(dtype, cfg):
    """Every tile configuration of the 16-bit kernels forced in turn on ragged shapes (rows and columns that
    end inside a tile, k split and unsplit), all three operand layouts, plus one epilogue with column sums."""
    ops = _ops()
    from terapipe_amd import _lib as L
    g = torch.Generator().manual_seed(cfg)
    for (M, N, K) in [(304, 1000, 512), (520, 648, 256), (64, 160, 64)]:
        sc = 1.0 / math.sqrt(K)
        A, B, B2 = _rnd((M, K), dtype, g), _rnd((N, K), dtype, g, sc), _rnd((K, N), dtype, g, sc)
        At = _rnd((K, M), dtype, g)
        R = _rnd((M, N), dtype, g)
        for ks in (1, 2):
            C = torch.zeros(M, N, dtype=dtype, device=DEV)
            ops.gemm(L.TP_GEMM_NT, A.to(DEV), B.to(DEV), M, N, K, C=C, tile_cfg=cfg, ksplit=ks)
            assert_close(C, A.double() @ B.double().t(), dtype, "NT cfg %d split %d %s" % (cfg, ks, (M, N, K)))
            ops.gemm(L.TP_GEMM_NN, A.to(DEV), B2.to(DEV), M, N, K, C=C, tile_cfg=cfg, ksplit=ks)
            assert_close(C, A.double() @ B2.double(), dtype, "NN cfg %d split %d" % (cfg, ks))
            ops.gemm(L.TP_GEMM_TN, At.to(DEV), B2.to(DEV), M, N, K, C=C, tile_cfg=cfg, ksplit=ks)
            assert_close(C, At.double().t() @ B2.double(), dtype, "TN cfg %d split %d" % (cfg, ks))
            acc = torch.zeros(N, dtype=torch.float32, device=DEV)
            ops.gemm(L.TP_GEMM_NT, A.to(DEV), B.to(DEV), M, N, K, C=C, epilogue=L.TP_EPI_RELU_GRAD, aux=R.to(DEV),
                     colsum_acc=acc, tile_cfg=cfg, ksplit=ks)
            ref = (A.double() @ B.double().t()) * (R.double() > 0)
            assert_close(C, ref, dtype, "relu grad cfg %d split %d" % (cfg, ks))
            assert_close(acc, ref.sum(0), dtype, "colsum cfg %d split %d" % (cfg, ks))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
def test_gemm_large_products_take_the_tall_tiles(dtype):
    """Products of 512 rows and more that the plan gives to the 256 x 256 tiles on its own (the LM head's
    shapes in small): many tiles with unsplit k, and few tiles on a long k that is split -- ragged extents,
    against the fp64 product."""
    ops = _ops()
    from terapipe_amd import _lib as L
    g = torch.Generator(device=DEV).manual_seed(91)

    def rnd(r, c, sc=1.0):
        return (torch.randn(r, c, generator=g, device=DEV) * sc).to(dtype)
    # NT, 4 x 50 tiles, unsplit
    A, B = rnd(1000, 192), rnd(12600, 192, 0.1)
    C = torch.empty(1000, 12600, dtype=dtype, device=DEV)
    ops.gemm(L.TP_GEMM_NT, A, B, 1000, 12600, 192, C=C)
    assert_close(C, A.double() @ B.double().t(), dtype, "NT 1000x12600x192")
    # NN, 4 x 13 tiles, k = 8256 split four ways
    A, B = rnd(1000, 8256), rnd(8256, 3104, 0.02)
    d = L.GemmDesc()
    d.op, d.dtype, d.epilogue, d.M, d.N, d.K = L.TP_GEMM_NN, ops.tp_dtype(dtype), L.TP_EPI_STORE, 1000, 3104, 8256
    d.A, d.lda, d.B, d.ldb, d.C, d.ldc = A.data_ptr(), 8256, B.data_ptr(), 3104, A.data_ptr(), 3104
    assert L.load().tp_gemm_splits(d) == 4
    C = torch.empty(1000, 3104, dtype=dtype, device=DEV)
    ops.gemm(L.TP_GEMM_NN, A, B, 1000, 3104, 8256, C=C)
    assert_close(C, A.double() @ B.double(), dtype, "NN 1000x3104x8256")


def _group(ops, L, items, dtype, force_cfg=None):
    """Runs items [(op, A, B, M, N, K)] once through gemm_grouped and once one by one; returns both outputs."""
    Cs_g = [torch.zeros(M, N, dtype=dtype, device=DEV) for (_, _, _, M, N, K) in items]
    Cs_1 = [torch.zeros(M, N, dtype=dtype, device=DEV) for (_, _, _, M, N, K) in items]
    ops.gemm_grouped([(op, A, B, M, N, K, C, L.TP_EPI_STORE) for (op, A, B, M, N, K), C in zip(items, Cs_g)])
    for (op, A, B, M, N, K), C in zip(items, Cs_1):
        ops.gemm(op, A, B, M, N, K, C=C, tile_cfg=force_cfg, ksplit=1 if force_cfg is not None else None)
    return Cs_g, Cs_1


def _group_cfg(L, items, dtype):
    import ctypes
    descs = (L.GemmDesc * len(items))()
    for d, (op, A, B, M, N, K) in zip(descs, items):
        d.op, d.dtype, d.epilogue, d.M, d.N, d.K = op, 1 if dtype == torch.float16 else 2, L.TP_EPI_STORE, M, N, K
        d.A, d.lda, d.B, d.ldb, d.C, d.ldc = A.data_ptr(), A.stride(0), B.data_ptr(), B.stride(0), A.data_ptr(), N
    return L.load().tp_gemm_group_cfg(descs, len(items))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
def test_gemm_grouped_single_launch_matches_member_by_member(dtype):
    """A layer's four weight-gradient products (hidden 2048, FFN 8192, 256 tokens), and a ragged group whose
    extents end inside tiles, through tp_gemm_grouped: the library reports one launch of a 256 x 256 tile
    configuration for them, and every output equals, bit for bit, the same product launched alone with that
    tile configuration (same tiles, same k order) -- and the fp64 product to the 16-bit tolerance."""
    ops = _ops()
    from terapipe_amd import _lib as L
    g = torch.Generator(device=DEV).manual_seed(77)

    def rnd(r, c, sc=1.0):
        return (torch.randn(r, c, generator=g, device=DEV) * sc).to(dtype)
    E, Fd, R = 2048, 8192, 256
    dys = [rnd(R, 3 * E, 0.1), rnd(R, E, 0.1), rnd(R, Fd, 0.1), rnd(R, E, 0.1)]
    xs = [rnd(R, E), rnd(R, E), rnd(R, E), rnd(R, Fd)]
    layer = [(L.TP_GEMM_TN, dy, x, dy.shape[1], x.shape[1], R) for dy, x in zip(dys, xs)]
    ragged = [(L.TP_GEMM_TN, rnd(192, 1000, 0.1), rnd(192, 2000), 1000, 2000, 192),
              (L.TP_GEMM_TN, rnd(192, 304, 0.1), rnd(192, 520), 304, 520, 192),
              (L.TP_GEMM_TN, rnd(192, 3000, 0.1), rnd(192, 4504), 3000, 4504, 192)]
    for tag, items in (("layer", layer), ("ragged", ragged)):
        cfg = _group_cfg(L, items, dtype)
        assert cfg in (2, 19, 20), "%s: the group should run as one launch (got %d)" % (tag, cfg)
        got, want = _group(ops, L, items, dtype, force_cfg=cfg)
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), "%s member %d differs from the product launched alone" % (tag, i)
        op, A, B, M, N, K = items[-1]
        ref = (A.double().t() @ B.double()) if op == L.TP_GEMM_TN else (A.double() @ B.double().t())
        assert_close(got[-1], ref, dtype, tag + " against fp64")


def test_gemm_grouped_falls_back_member_by_member():
    """Groups the single launch does not cover (small products, a k that is not a multiple of 64, five members,
    another operand layout) run member by member with the same results; the accumulate epilogue through the
    single launch."""
    ops = _ops()
    from terapipe_amd import _lib as L
    dtype = torch.float16
    g = torch.Generator(device=DEV).manual_seed(78)

    def rnd(r, c, sc=1.0):
        return (torch.randn(r, c, generator=g, device=DEV) * sc).to(dtype)
    small = [(L.TP_GEMM_TN, rnd(96, 256, 0.1), rnd(96, 512), 256, 512, 96),
             (L.TP_GEMM_TN, rnd(96, 128, 0.1), rnd(96, 64), 128, 64, 96)]
    odd_k = [(L.TP_GEMM_TN, rnd(200, 4096, 0.1), rnd(200, 4096), 4096, 4096, 200),
             (L.TP_GEMM_TN, rnd(200, 512, 0.1), rnd(200, 512), 512, 512, 200)]
    five = [(L.TP_GEMM_NT, rnd(64, 256), rnd(128, 256, 0.1), 64, 128, 256) for _ in range(5)]
    nt = [(L.TP_GEMM_NT, rnd(4096, 128), rnd(4096, 128, 0.1), 4096, 4096, 128),
          (L.TP_GEMM_NT, rnd(520, 128), rnd(264, 128, 0.1), 520, 264, 128)]
    for tag, items in (("small", small), ("odd k", odd_k), ("five", five), ("not TN", nt)):
        assert _group_cfg(L, items, dtype) == 0, tag
        got, want = _group(ops, L, items, dtype)
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), "%s member %d" % (tag, i)
    # accumulate epilogue through the grouped launch: C += product
    items = [(L.TP_GEMM_TN, rnd(128, 4096, 0.1), rnd(128, 4096), 4096, 4096, 128),
             (L.TP_GEMM_TN, rnd(128, 512, 0.1), rnd(128, 768), 512, 768, 128)]
    assert _group_cfg(L, items, dtype) in (2, 19, 20)
    Cs = [torch.ones(M, N, dtype=dtype, device=DEV) for (_, _, _, M, N, K) in items]
    ops.gemm_grouped([(op, A, B, M, N, K, C, L.TP_EPI_ACCUMULATE) for (op, A, B, M, N, K), C in zip(items, Cs)])
    for (op, A, B, M, N, K), C in zip(items, Cs):
        assert_close(C, 1.0 + A.double().t() @ B.double(), dtype, "accumulate")


def _tuned_entries():
    import os
    import re
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "terapipe_amd", "csrc",
                        "gemm_tuned.inc")
    rows = [(m.group(1), int(m.group(2)), int(m.group(3)), int(m.group(4)))
            for m in re.finditer(r"\{TP_GEMM_(NT|NN|TN), (\d+), (\d+), (\d+), \d+, \d+\}", open(path).read())]
    by_weight = {}
    for op, M, N, K in rows:
        by_weight.setdefault((op, N, K) if op != "TN" else (op, M, N), []).append((op, M, N, K))
    return sorted(by_weight.items())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("key,shapes", _tuned_entries(), ids=lambda v: "-".join(map(str, v)) if isinstance(v, tuple) else "")
def test_gemm_measured_plans_at_their_shapes(key, shapes, dtype):
    """Every shape of the measured plan table (the benchmark geometries' own GEMMs, with the tile configuration
    and k-split the table prescribes for them) against the fp32 library product of the same 16-bit operands, in
    both 16-bit types (the table is keyed by extents only: the 175B / 44B entries run in bf16)."""
    ops = _ops()
    from terapipe_amd import _lib as L
    g = torch.Generator(device=DEV).manual_seed(sum(v for v in key if isinstance(v, int)) % 65521)
    op = key[0]
    if op == "TN":
        _, M, N = key
        for (_, _, _, K) in shapes:
            A = (torch.randn(K, M, generator=g, device=DEV) * 0.05).to(dtype)
            B = torch.randn(K, N, generator=g, device=DEV).to(dtype)
            C = torch.empty(M, N, dtype=dtype, device=DEV)
            ops.gemm(L.TP_GEMM_TN, A, B, M, N, K, C=C)
            rows = torch.randperm(M, generator=g, device=DEV)[:1024]
            ref = A[:, rows].float().t() @ B.float()
            assert_close(C[rows], ref.cpu().double(), dtype, "TN %dx%dx%d" % (M, N, K))
        return
    _, N, K = key
    B = (torch.randn((N, K) if op == "NT" else (K, N), generator=g, device=DEV) * K ** -0.5).to(dtype)
    Bf = B.float()
    for (_, M, _, _) in shapes:
        A = torch.randn(M, K, generator=g, device=DEV).to(dtype)
        C = torch.empty(M, N, dtype=dtype, device=DEV)
        ops.gemm(L.TP_GEMM_NT if op == "NT" else L.TP_GEMM_NN, A, B, M, N, K, C=C)
        ref = A.float() @ (Bf.t() if op == "NT" else Bf)
        assert_close(C, ref.cpu().double(), dtype, "%s %dx%dx%d" % (op, M, N, K))


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("M,N,K", [(32, 1024, 256), (256, 8192, 2048), (48, 264, 136)])
def test_gemm_epilogues(dtype, M, N, K):
    ops = _ops()
    from terapipe_amd import _lib as L
    g = torch.Generator().manual_seed(5 * M + N + K)
    sc = 1.0 / math.sqrt(K)
    A, B = _rnd((M, K), dtype, g), _rnd((N, K), dtype, g, sc)
    bias, R = _rnd((N,), dtype, g, 0.5), _rnd((M, N), dtype, g)
    Ad, Bd, bd, Rd = A.to(DEV), B.to(DEV), bias.to(DEV), R.to(DEV)
    base = A.double() @ B.double().t() + bias.double()
    C = torch.empty(M, N, dtype=dtype, device=DEV)
    ops.gemm(L.TP_GEMM_NT, Ad, Bd, M, N, K, C=C, epilogue=L.TP_EPI_BIAS, bias=bd)
    assert_close(C, base, dtype, "bias")
    ops.gemm(L.TP_GEMM_NT, Ad, Bd, M, N, K, C=C, epilogue=L.TP_EPI_BIAS_RELU, bias=bd)
    assert_close(C, base.relu(), dtype, "bias+relu")
    Z = torch.empty_like(C)
    ops.gemm(L.TP_GEMM_NT, Ad, Bd, M, N, K, C=C, epilogue=L.TP_EPI_BIAS_GELU, bias=bd, aux_out=Z)
    assert_close(C, oracle.gelu_erf(base), dtype, "bias+gelu")
    assert_close(Z, base, dtype, "gelu pre-activation")
    ops.gemm(L.TP_GEMM_NT, Ad, Bd, M, N, K, C=C, epilogue=L.TP_EPI_BIAS_RESIDUAL, bias=bd, residual=Rd)
    assert_close(C, base + R.double(), dtype, "bias+residual")
    # activation gradients fused into the data-gradient GEMM, with the bias-gradient column sums
    plain = A.double() @ B.double().t()
    acc = torch.zeros(N, dtype=torch.float32, device=DEV)
    ops.gemm(L.TP_GEMM_NT, Ad, Bd, M, N, K, C=C, epilogue=L.TP_EPI_RELU_GRAD, aux=Rd, colsum_acc=acc)
    ref = plain * (R.double() > 0)
    assert_close(C, ref, dtype, "relu grad")
    assert_close(acc, ref.sum(0), dtype, "relu grad colsum")
    acc.zero_()
    ops.gemm(L.TP_GEMM_NT, Ad, Bd, M, N, K, C=C, epilogue=L.TP_EPI_GELU_GRAD, aux=Rd, colsum_acc=acc)
    z = R.double().requires_grad_(True)
    oracle.gelu_erf(z).sum().backward()
    ref = plain * z.grad
    assert_close(C, ref, dtype, "gelu grad")
    assert_close(acc, ref.sum(0), dtype, "gelu grad colsum")


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("T,B,H,Dh,P,L", [(16, 2, 4, 64, 32, 128), (32, 1, 2, 128, 0, 64), (5, 3, 2, 64, 3, 16),
                                           (16, 2, 4, 80, 32, 128), (40, 1, 3, 96, 7, 64), (24, 2, 5, 16, 9, 40)])
def test_gemm_qkv_scatter(dtype, T, B, H, Dh, P, L):
    ops = _ops()
    from terapipe_amd import _lib as Lb
    E = H * Dh
    g = torch.Generator().manual_seed(T + B + H)
    x, W, b = _rnd((T, B, E), dtype, g), _rnd((3 * E, E), dtype, g, E ** -0.5), _rnd((3 * E,), dtype, g, 0.3)
    q = torch.zeros(B * H, T, Dh, dtype=dtype, device=DEV)
    kc = torch.full((B * H, L, Dh), 7.0, dtype=dtype, device=DEV)
    vc = torch.full((B * H, L, Dh), 7.0, dtype=dtype, device=DEV)
    ops.gemm(Lb.TP_GEMM_NT, x.view(T * B, E).to(DEV), W.to(DEV), T * B, 3 * E, E, epilogue=Lb.TP_EPI_QKV_SCATTER,
             bias=b.to(DEV), qkv=dict(q=q, k_cache=kc, v_cache=vc, batch=B, heads=H, head_dim=Dh, cache_len=P,
                                      cache_rows=L, q_scale=Dh ** -0.5))
    qkv = oracle.linear_col(x.double(), W.double(), b.double())
    qr, kr, vr = oracle.split_qkv(qkv, H)
    assert_close(q, qr * Dh ** -0.5, dtype, "q")
    assert_close(kc[:, P:P + T], kr, dtype, "k rows")
    assert_close(vc[:, P:P + T], vr, dtype, "v rows")
    # rows outside the slice are untouched
    assert (kc[:, :P] == 7).all() and (kc[:, P + T:] == 7).all()
    assert (vc[:, :P] == 7).all() and (vc[:, P + T:] == 7).all()


def _attn_ref(q, kc, vc, B, H, T, P):
    """fp64 restatement through the oracle's attention_core; q, kc, vc are leaf tensors."""
    S = P + T
    mask = oracle.causal_prefix_mask(T, P, torch.float64)
    return oracle.attention_core(q, kc[:, :S], vc[:, :S], mask, T, B)


ATTN_CASES = [
    # T, B, H, Dh, P, L
    (16, 2, 4, 64, 0, 128),
    (16, 2, 4, 64, 112, 128),
    (32, 2, 3, 128, 480, 512),     # single-wave workgroups + split over keys
    (128, 1, 4, 128, 896, 1024),   # four waves, split
    (256, 1, 2, 128, 256, 512),    # multiple query blocks
    (160, 1, 2, 128, 100, 300),    # ragged against every tile size
    (7, 1, 1, 64, 5, 12),
    (1, 1, 1, 64, 0, 1),
    (64, 1, 2, 128, 0, 64),        # two waves
    (32, 2, 48, 128, 2016, 2048),  # benchmark config 5's last slice: 96 (batch, head) pairs, 32 queries, 2048 keys
    (128, 1, 96, 128, 1920, 2048), # config 4's last slice
    (160, 1, 40, 128, 1888, 2048), # config 3's last slice
    # head dimensions other than 64 and 128 (the reference's model table has 80, 96 and 16, transformer_models.py:33-49):
    # the register-staged kernels with the head dimension padded to whole 32-column blocks in LDS, in every dtype
    (16, 2, 4, 80, 112, 128),
    (64, 1, 2, 96, 0, 64),         # no prefix: also pinned against SDPA
    (32, 2, 3, 80, 480, 512),      # split over keys, merged
    (128, 1, 4, 96, 896, 1024),
    (160, 1, 2, 96, 100, 300),     # ragged
    (7, 1, 1, 80, 5, 12),
    (96, 2, 32, 80, 416, 512),     # 64 (batch, head) pairs, several query blocks
    (16, 2, 4, 16, 112, 128),      # head dimension 16: gpt3-175b-megatron's 6144 / 384 (transformer_models.py:49)
    (100, 1, 5, 16, 300, 512),
    (40, 1, 3, 32, 7, 64),
    (128, 2, 2, 32, 896, 1024),
]


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("T,B,H,Dh,P,L", ATTN_CASES)
def test_attn_prefix_fwd_bwd(dtype, T, B, H, Dh, P, L):
    ops = _ops()
    S, E, BH = P + T, H * Dh, B * H
    g = torch.Generator().manual_seed(T * 3 + P)
    q = _rnd((BH, T, Dh), dtype, g, 1.0)          # already "scaled" q as far as the kernel is concerned
    kc, vc = _rnd((BH, L, Dh), dtype, g, Dh ** -0.25), _rnd((BH, L, Dh), dtype, g)
    d_o = _rnd((T, B, E), dtype, g)
    inc_k, inc_v = _rnd((BH, L, Dh), dtype, g), _rnd((BH, L, Dh), dtype, g)
    qd, kd, vd = q.to(DEV), kc.to(DEV), vc.to(DEV)
    o, lse = ops.attn_prefix_fwd(qd, kd, vd, B, H, Dh, T, P, 1.0)
    q64 = q.double().requires_grad_(True)
    k64, v64 = kc.double().requires_grad_(True), vc.double().requires_grad_(True)
    oref = _attn_ref(q64, k64, v64, B, H, T, P)
    assert_close(o, oref, dtype, "attn o")
    s = torch.bmm(q64, k64[:, :S].transpose(1, 2)) + oracle.causal_prefix_mask(T, P, torch.float64)
    assert_close(lse, torch.logsumexp(s, -1), torch.float32, "attn lse", 1e3 if dtype != torch.float32 else 10)
    # both wave counts of the 16-bit forward's 32-query workgroups and its 64-query workgroups (from 64 queries on),
    # whatever the plan picks for this shape
    for variant in (2 | 8, 4 | 8, 16):
        o_v, lse_v = ops.attn_prefix_fwd(qd, kd, vd, B, H, Dh, T, P, 1.0, variant=variant)
        assert_close(o_v, oref, dtype, "attn o, forward variant %d" % variant)
        assert_close(lse_v, torch.logsumexp(s, -1), torch.float32, "attn lse, forward variant %d" % variant,
                     1e3 if dtype != torch.float32 else 10)
    oref.backward(d_o.double())
    # library-routine pin for the no-prefix case
    if P == 0:
        sd = F.scaled_dot_product_attention(q.double(), kc[:, :S].double(), vc[:, :S].double(), is_causal=True, scale=1.0)
        assert_close(o, sd.transpose(0, 1).reshape(T, B, E), dtype, "attn o vs SDPA")

    for gdt in ([dtype] if dtype == torch.float32 else [dtype, torch.float32]):
        for incoming in (False, True):
            gk = inc_k.to(gdt).to(DEV) if incoming else torch.full((BH, L, Dh), 3.0, dtype=gdt, device=DEV)
            gv = inc_v.to(gdt).to(DEV) if incoming else torch.full((BH, L, Dh), 3.0, dtype=gdt, device=DEV)
            dqkv = torch.empty(T * B, 3 * E, dtype=dtype, device=DEV)
            acc = torch.zeros(3 * E, dtype=torch.float32, device=DEV)
            ops.attn_prefix_bwd(qd, kd, vd, o, lse, d_o.to(DEV), dqkv, gk, gv, B, H, Dh, T, P, 0.5,
                                accumulate_prefix=incoming, has_incoming=incoming, zero_slice_rows=incoming,
                                colsum_dqkv_acc=acc)
            dq, dk, dv = oracle.split_qkv(dqkv.view(T, B, 3 * E).double().cpu(), H)
            tag = "[gdt=%s incoming=%s]" % (gdt, incoming)
            assert_close(dq, q64.grad * 0.5, dtype, "dq" + tag)
            ik = inc_k.double() if incoming else torch.zeros(BH, L, Dh, dtype=torch.float64)
            iv = inc_v.double() if incoming else torch.zeros(BH, L, Dh, dtype=torch.float64)
            assert_close(dk, k64.grad[:, P:S] + ik[:, P:S], dtype, "dk slice" + tag)
            assert_close(dv, v64.grad[:, P:S] + iv[:, P:S], dtype, "dv slice" + tag)
            if P > 0:
                assert_close(gk[:, :P], k64.grad[:, :P] + ik[:, :P], dtype, "gk prefix" + tag)
                assert_close(gv[:, :P], v64.grad[:, :P] + iv[:, :P], dtype, "gv prefix" + tag)
            if incoming:
                assert (gk[:, P:S] == 0).all() and (gv[:, P:S] == 0).all(), "slice rows zeroed" + tag
                assert torch.equal(gk[:, S:].cpu(), inc_k.to(gdt)[:, S:]), "rows beyond the slice untouched" + tag
            else:
                assert (gk[:, P:] == 3).all() and (gv[:, P:] == 3).all(), "rows beyond the prefix untouched" + tag
            assert_close(acc, dqkv.double().sum(0), dtype, "dqkv colsum" + tag)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("T,B,H,Dh,P,L,drift", [(128, 1, 4, 128, 896, 1024, 0.0), (160, 1, 4, 128, 352, 512, 0.0),
                                                (32, 2, 3, 64, 480, 512, 0.0), (128, 1, 4, 128, 896, 1024, 0.05),
                                                (64, 2, 2, 64, 448, 512, 0.1)])
def test_attn_peaked_and_drifting_scores(dtype, T, B, H, Dh, P, L, drift):
    """Scores with a standard deviation near 17 (Dh 128) / 12 (Dh 64), so that a row's softmax sits on a few keys and
    its largest score keeps being overtaken along the key range: the forward kernels take exponentials against a
    per-row reference that moves only when a row outgrows it by e^5, and this is the input on which it moves often.
    drift adds a ramp along the key position (later keys score higher), the order in which the reference is
    overtaken tile after tile.  All forward forms against the fp64 restatement, and without the ramp the backward
    too (with it the keys carry a common component of up to 50, which dQ = dS K cancels -- the rows of dS sum to
    zero -- so that the 16-bit rounding of dS alone exceeds the bound on any implementation)."""
    ops = _ops()
    S, E, BH = P + T, H * Dh, B * H
    g = torch.Generator().manual_seed(T + P + Dh)
    q = _rnd((BH, T, Dh), dtype, g, 1.0)
    k32 = torch.randn(BH, L, Dh, generator=g) * 1.5
    if drift:
        # a component along q's mean direction that grows with the key position
        k32 = k32 + drift * torch.arange(L).view(1, L, 1) * torch.sign(q.float().mean(1, keepdim=True))
    kc, vc = k32.to(dtype), _rnd((BH, L, Dh), dtype, g)
    d_o = _rnd((T, B, E), dtype, g)
    qd, kd, vd = q.to(DEV), kc.to(DEV), vc.to(DEV)
    q64 = q.double().requires_grad_(True)
    k64, v64 = kc.double().requires_grad_(True), vc.double().requires_grad_(True)
    oref = _attn_ref(q64, k64, v64, B, H, T, P)
    s = torch.bmm(q64, k64[:, :S].transpose(1, 2)) + oracle.causal_prefix_mask(T, P, torch.float64)
    lse_ref = torch.logsumexp(s, -1)
    o, lse = ops.attn_prefix_fwd(qd, kd, vd, B, H, Dh, T, P, 1.0)
    assert_close(o, oref, dtype, "attn o")
    assert_close(lse, lse_ref, torch.float32, "attn lse", 1e3)
    for variant in (2 | 8, 4 | 8, 16):
        o_v, lse_v = ops.attn_prefix_fwd(qd, kd, vd, B, H, Dh, T, P, 1.0, variant=variant)
        assert_close(o_v, oref, dtype, "attn o, forward variant %d" % variant)
        assert_close(lse_v, lse_ref, torch.float32, "attn lse, forward variant %d" % variant, 1e3)
    if drift:
        return
    oref.backward(d_o.double())
    gk = torch.zeros(BH, L, Dh, dtype=torch.float32, device=DEV)
    gv = torch.zeros(BH, L, Dh, dtype=torch.float32, device=DEV)
    dqkv = torch.empty(T * B, 3 * E, dtype=dtype, device=DEV)
    ops.attn_prefix_bwd(qd, kd, vd, o, lse, d_o.to(DEV), dqkv, gk, gv, B, H, Dh, T, P, 1.0,
                        accumulate_prefix=False, has_incoming=False, zero_slice_rows=False)
    dq, dk, dv = oracle.split_qkv(dqkv.view(T, B, 3 * E).double().cpu(), H)
    assert_close(dq, q64.grad, dtype, "dq")
    assert_close(dk, k64.grad[:, P:S], dtype, "dk slice")
    assert_close(dv, v64.grad[:, P:S], dtype, "dv slice")
    assert_close(gk[:, :P], k64.grad[:, :P], dtype, "gk prefix")
    assert_close(gv[:, :P], v64.grad[:, :P], dtype, "gv prefix")


SUFFIX_CASES = [
    # B, H, Dh, L (cache rows), slices
    (2, 2, 64, 96, [32, 32, 32]),
    (1, 2, 128, 256, [64, 96, 32, 64]),
    (1, 3, 128, 200, [40, 7, 100, 33]),      # ragged: nothing aligned to the 32-row blocks
    (2, 1, 64, 64, [5, 1, 20]),              # caches longer than the sequence
    (1, 2, 128, 512, [128, 128, 128, 128]),
    (2, 48, 128, 1024, [32] * 32),                             # benchmark config 5's heads and slices (half its length)
    (1, 96, 128, 1024, [128] * 8),                             # config 4's
    (1, 40, 128, 2048, [512, 384, 320, 256, 224, 192, 160]),   # config 3's, whole
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("B,H,Dh,L,slices", SUFFIX_CASES)
def test_attn_position_indexed_and_suffix_dkdv(dtype, B, H, Dh, L, slices):
    """The layout a runner uses that keeps every slice: q, lse, delta and dO live in position-indexed
    buffers (as the K/V caches do); each slice's forward and dQ work on views of them (q_bh_rows /
    stat_bh_rows), and dK/dV of a slice's keys come from ONE pass over all later query positions
    (tp_attn_suffix_dkdv) instead of the gradient caches.  Slices run forward in order and backward in
    reverse order, as terapipe.py:182-191 does; the check is the fp64 causal attention over the whole
    sequence through the oracle's attention_core."""
    ops = _ops()
    E, BH, Ltot = H * Dh, B * H, sum(slices)
    g = torch.Generator().manual_seed(Ltot + Dh)
    q = _rnd((BH, L, Dh), dtype, g, 1.0)
    kc, vc = _rnd((BH, L, Dh), dtype, g, Dh ** -0.25), _rnd((BH, L, Dh), dtype, g)
    d_o = _rnd((Ltot, B, E), dtype, g)
    qd, kd, vd, dod = q.to(DEV), kc.to(DEV), vc.to(DEV), d_o.to(DEV)
    o_all = torch.empty(Ltot, B, E, dtype=dtype, device=DEV)
    lse_all = torch.full((BH, L), 123.0, dtype=torch.float32, device=DEV)
    delta_all = torch.full((BH, L), 321.0, dtype=torch.float32, device=DEV)
    P = 0
    for T in slices:
        ops.attn_prefix_fwd(qd[:, P:], kd, vd, B, H, Dh, T, P, 1.0, out=o_all[P:P + T], lse=lse_all[:, P:],
                            q_bh_rows=L, stat_bh_rows=L)
        P += T
    q64 = q[:, :Ltot].double().requires_grad_(True)
    k64, v64 = kc[:, :Ltot].double().requires_grad_(True), vc[:, :Ltot].double().requires_grad_(True)
    oref = _attn_ref(q64, k64, v64, B, H, Ltot, 0)
    assert_close(o_all, oref, dtype, "o, all slices")
    s = torch.bmm(q64, k64.transpose(1, 2)) + oracle.causal_prefix_mask(Ltot, 0, torch.float64)
    assert_close(lse_all[:, :Ltot], torch.logsumexp(s, -1), torch.float32, "lse, all slices", 1e3)
    assert (lse_all[:, Ltot:] == 123).all()
    oref.backward(d_o.double())
    dqkv_all = torch.zeros(Ltot * B, 3 * E, dtype=dtype, device=DEV)
    for i in reversed(range(len(slices))):
        T, P = slices[i], sum(slices[:i])
        dqkv = dqkv_all[P * B:(P + T) * B]
        ops.attn_prefix_bwd(qd[:, P:], kd, vd, o_all[P:P + T], lse_all[:, P:], dod[P:P + T], dqkv, None, None, B, H, Dh,
                            T, P, 0.5, False, False, False, delta=delta_all[:, P:], q_bh_rows=L, stat_bh_rows=L,
                            dq_only=True)
        ops.attn_suffix_dkdv(kd, vd, qd, dod, lse_all, delta_all, dqkv, B, H, Dh, P, T, Ltot)
    delta_ref = (oref.detach() * d_o.double()).view(Ltot, B, H, Dh).sum(-1).permute(1, 2, 0).reshape(BH, Ltot)
    assert_close(delta_all[:, :Ltot], delta_ref, torch.float32, "delta", 1e3)
    assert (delta_all[:, Ltot:] == 321).all()
    dq, dk, dv = oracle.split_qkv(dqkv_all.view(Ltot, B, 3 * E).double().cpu(), H)
    assert_close(dq, q64.grad * 0.5, dtype, "dq")
    assert_close(dk, k64.grad, dtype, "dk over all later queries")
    assert_close(dv, v64.grad, dtype, "dv over all later queries")
    # the two launches of a slice as one (tp_attn_bwd_fused): its dK/dV half takes delta of the slice's own
    # positions from dO and O itself instead of waiting for the dQ half -- same arithmetic, same bits
    # (window: how many slices' delta the dK/dV half takes itself -- its own, or also that of the next two, whose
    # entries in the delta array it then must not read: they are poisoned here)
    for window in (1, 3):
        dqkv_fused = torch.zeros(Ltot * B, 3 * E, dtype=dtype, device=DEV)
        delta_fused = torch.full((BH, L), 321.0, dtype=torch.float32, device=DEV)
        for i in reversed(range(len(slices))):
            T, P = slices[i], sum(slices[:i])
            own_end = sum(slices[:i + window])
            seen = delta_fused.clone()
            seen[:, P:own_end] = float("nan")
            ops.attn_bwd_fused(qd[:, P:], kd, vd, o_all[P:P + T], lse_all[:, P:], dod[P:P + T], dqkv_fused[P * B:(P + T) * B],
                               B, H, Dh, T, P, 0.5, delta_fused[:, P:], qd, dod, lse_all, seen, o_all, Ltot,
                               own_delta_end=own_end, q_bh_rows=L, stat_bh_rows=L)
        assert torch.equal(delta_fused, delta_all), "delta, fused launch, window %d" % window
        assert torch.equal(dqkv_fused, dqkv_all), "dqkv, fused launch, window %d" % window


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("T,B,H,Dh,P,ns", [(32, 2, 3, 128, 480, 2), (40, 1, 2, 64, 200, 3), (128, 1, 4, 128, 896, 5),
                                           (7, 1, 1, 64, 5, 4), (160, 1, 2, 128, 100, 16), (32, 2, 48, 128, 992, 2)])
def test_attn_fwd_keys_shared_by_workgroups(dtype, T, B, H, Dh, P, ns):
    """The 16-bit forward with the key range of every query block forced onto `ns` workgroups whose fp32 partials
    the merge launch weighs together -- what the plan does by itself for calls with few blocks and long key ranges
    (benchmark config 5's later slices in ATTN_CASES).  Shares that come out empty (more workgroups than tiles) and
    ragged last tiles are part of the cases.  Checked against the fp64 attention."""
    ops = _ops()
    S, E, BH = P + T, H * Dh, B * H
    g = torch.Generator().manual_seed(T * 5 + P + ns)
    q = _rnd((BH, T, Dh), dtype, g, 1.0)
    kc, vc = _rnd((BH, S, Dh), dtype, g, Dh ** -0.25), _rnd((BH, S, Dh), dtype, g)
    q64, k64, v64 = q.double(), kc.double(), vc.double()
    oref = _attn_ref(q64, k64, v64, B, H, T, P)
    lse_ref = torch.logsumexp(torch.bmm(q64, k64.transpose(1, 2)) + oracle.causal_prefix_mask(T, P, torch.float64), -1)
    for variant in (2 | 8, 4 | 8, 16):
        o, lse = ops.attn_prefix_fwd(q.to(DEV), kc.to(DEV), vc.to(DEV), B, H, Dh, T, P, 1.0, nsplit=ns, variant=variant)
        assert_close(o, oref, dtype, "o, keys over %d workgroups, variant %d" % (ns, variant))
        assert_close(lse, lse_ref, torch.float32, "lse, keys over %d workgroups, variant %d" % (ns, variant), 1e3)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("M,E,K,ks", [(64, 256, 1024, 2), (37, 512, 4096, 4), (256, 2048, 8192, 2), (5, 64, 512, 1)])
def test_layernorm_consumes_deferred_split_k(dtype, M, E, K, ks):
    """A k-split GEMM with defer_reduce leaves fp32 partial sums; the LayerNorm forward / backward that
    consumes the GEMM's result sums them (+ bias + residual), writes the result tensor and normalises it.
    Bit-identical to GEMM (own reduce) followed by the plain LayerNorm call; without a split (ks = 1) the
    GEMM completes normally and returns the tensor."""
    ops = _ops()
    from terapipe_amd import _lib as Lb
    g = torch.Generator().manual_seed(M + E)
    A, W = _rnd((M, K), dtype, g).to(DEV), _rnd((E, K), dtype, g, K ** -0.5).to(DEV)
    b, r = _rnd((E,), dtype, g, 0.3).to(DEV), _rnd((M, E), dtype, g).to(DEV)
    gm, bt = (_rnd((E,), dtype, g, 0.2) + 1).to(DEV), _rnd((E,), dtype, g, 0.2).to(DEV)
    force = dict(ksplit=ks) if dtype != torch.float32 else {}
    C1 = torch.empty(M, E, dtype=dtype, device=DEV)
    ops.gemm(Lb.TP_GEMM_NT, A, W, M, E, K, C=C1, epilogue=Lb.TP_EPI_BIAS_RESIDUAL, bias=b, residual=r, **force)
    y1, m1, s1 = ops.layernorm_fwd(C1, gm, bt)
    C2 = torch.full((M, E), 9.0, dtype=dtype, device=DEV)
    res = ops.gemm(Lb.TP_GEMM_NT, A, W, M, E, K, C=C2, epilogue=Lb.TP_EPI_BIAS_RESIDUAL, bias=b, residual=r,
                   defer_reduce=True, **force)
    if dtype != torch.float32 and ks > 1:
        assert isinstance(res, ops.PendingReduce) and res.nsplit == ks
        assert (C2 == 9).all(), "the deferred GEMM must not write its result tensor"
    y2, m2, s2 = ops.layernorm_fwd(res, gm, bt)
    assert torch.equal(C1, C2) and torch.equal(y1, y2) and torch.equal(m1, m2) and torch.equal(s1, s2)
    # backward: dy = A W^T as the (deferred) gradient GEMM, x = r
    D1 = torch.empty(M, E, dtype=dtype, device=DEV)
    ops.gemm(Lb.TP_GEMM_NT, A, W, M, E, K, C=D1, **force)
    xm, xs = ops.layernorm_fwd(r, gm, bt)[1:]
    acc1 = [torch.zeros(E, dtype=torch.float32, device=DEV) for _ in range(4)]
    dx1 = ops.layernorm_bwd(D1, r, xm, xs, gm, C1, *acc1)
    D2 = torch.full((M, E), 9.0, dtype=dtype, device=DEV)
    res = ops.gemm(Lb.TP_GEMM_NT, A, W, M, E, K, C=D2, defer_reduce=True, **force)
    acc2 = [torch.zeros(E, dtype=torch.float32, device=DEV) for _ in range(4)]
    dx2 = ops.layernorm_bwd(res, r, xm, xs, gm, C1, *acc2)
    assert torch.equal(D1, D2) and torch.equal(dx1, dx2)
    for a1, a2 in zip(acc1, acc2):
        assert_close(a2, a1, torch.float32, "accumulators", 100)     # atomics: order differs
    dx3 = ops.layernorm_bwd(ops.gemm(Lb.TP_GEMM_NT, A, W, M, E, K, C=D2, defer_reduce=True, **force), r, xm, xs, gm,
                            None, None, None)
    assert torch.equal(dx3, ops.layernorm_bwd(D1, r, xm, xs, gm, None, None, None))


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("M,E,V", [(24, 64, 50257), (7, 256, 1003), (130, 128, 512)])
def test_embedding_lm_head_cross_entropy(dtype, M, E, V):
    """Token ids -> embedding -> (tied) LM head -> per-token cross-entropy -> mean, forward and backward,
    against the oracle's restatements of mpu.VocabParallelEmbedding and mpu.vocab_parallel_cross_entropy."""
    import terapipe_amd as ta
    g = torch.Generator().manual_seed(V + M)
    W = _rnd((V, E), dtype, g, 0.05)
    ids = torch.randint(0, V, (M,), generator=g)
    tgt = torch.randint(0, V, (M,), generator=g)
    ids[0], tgt[-1] = V - 1, V - 1                        # last vocabulary row on both ends
    ids[1] = ids[2]                                       # a repeated id (gradient rows add up)
    emb = ta.VocabParallelEmbedding(V, E, device=DEV, dtype=dtype)
    with torch.no_grad():
        emb.weight.copy_(W.to(DEV))
    x = emb(ids.to(DEV))
    logits = ta.lm_head_logits(x.view(M, E), emb.weight)
    assert logits.shape == (M, (V + 63) // 64 * 64)
    loss = ta.vocab_parallel_cross_entropy(logits, tgt.to(DEV), vocab_size=V)
    scale = _rnd((M,), torch.float32, g).abs() + 0.5
    (loss * scale.to(DEV)).sum().backward()
    W64 = W.double().requires_grad_(True)
    x64 = oracle.embedding(ids, W64)
    loss64 = oracle.vocab_cross_entropy(x64 @ W64.t(), tgt)
    (loss64 * scale.double()).sum().backward()
    assert_close(x, x64, dtype, "embedding")
    assert_close(loss, loss64, torch.float32 if dtype == torch.float32 else dtype, "per-token loss",
                 10 if dtype == torch.float32 else 1)
    assert_close(emb.weight.grad, W64.grad, dtype, "d weight (embedding + LM head)", 3)
    # out-of-range ids give zero rows
    bad = ids.clone(); bad[3] = V + 5
    assert (emb(bad.to(DEV))[3] == 0).all()


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_cross_entropy_vector_and_scalar_paths(dtype):
    """tp_cross_entropy on rows that allow 16-byte accesses (short enough to be held in registers, and longer
    ones) and on rows that do not (odd leading dimension, a padded width that is not a whole number of
    chunks): loss, in-place gradient (softmax - onehot) * scale,
    zeroed padding columns, and a target outside the vocabulary (no onehot, loss without the target term)."""
    ops = _ops()
    g = torch.Generator().manual_seed(5)
    for (M, V, Vpad, ld) in [(9, 50257, 50264, 50264), (9, 50257, 50264, 50265), (5, 1003, 1003, 1003),
                             (6, 1000, 1008, 1024), (3, 7, 8, 8), (3, 70001, 70008, 70008)]:
        z = _rnd((M, V), dtype, g, 3.0)
        tgt = torch.randint(0, V, (M,), generator=g)
        tgt[0] = V - 1
        tgt[1] = V + 3                                   # outside: as a masked target
        buf = torch.full((M, ld), 7.0, dtype=dtype, device=DEV)
        buf[:, :V] = z.to(DEV)
        view = buf[:, :Vpad]
        loss = ops.cross_entropy_(view, tgt.to(DEV), V, grad_scale=0.5)
        z64 = z.double()
        lse = torch.logsumexp(z64, dim=1)
        inside = tgt < V
        want_loss = lse - torch.where(inside, z64.gather(1, tgt.clamp(max=V - 1)[:, None])[:, 0], torch.zeros(M, dtype=torch.float64))
        want_grad = torch.softmax(z64, dim=1)
        for m in range(M):
            if inside[m]:
                want_grad[m, tgt[m]] -= 1.0
        want_grad *= 0.5
        tag = "M=%d V=%d Vpad=%d ld=%d" % (M, V, Vpad, ld)
        assert_close(loss, want_loss, torch.float32 if dtype == torch.float32 else dtype, tag + " loss",
                     10 if dtype == torch.float32 else 1)
        assert_close(buf[:, :V], want_grad, dtype, tag + " gradient", 10 if dtype == torch.float32 else 1)
        assert (buf[:, V:Vpad] == 0).all(), tag + " padding columns"
        assert (buf[:, Vpad:] == 7.0).all(), tag + " columns beyond the padded width are not touched"


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_scale_rows_vector_and_scalar_paths(dtype):
    """tp_scale_rows (x[m, :] *= scale[m]) on rows that allow 16-byte accesses and on rows that do not; columns
    beyond the given width stay as they were."""
    ops = _ops()
    g = torch.Generator().manual_seed(6)
    for (M, N, ld) in [(5, 1024, 1024), (5, 1000, 1032), (4, 1003, 1003), (3, 64, 65)]:
        x = _rnd((M, ld), dtype, g)
        sc = _rnd((M,), torch.float32, g)
        buf = x.to(DEV).clone()
        ops.scale_rows_(buf[:, :N], sc.to(DEV))
        want = x.double().clone()
        want[:, :N] *= sc.double()[:, None]
        assert_close(buf, want, dtype, "M=%d N=%d ld=%d" % (M, N, ld))
        assert torch.equal(buf[:, N:].cpu(), x[:, N:])


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_vec_param_grads_one_launch(dtype):
    """tp_vec_param_grads: the four bias column sums and two LayerNorm pairs of a layer in one launch (ragged row
    count, widths that end inside a 256-column block, a strided view) against fp64 sums; the accumulators are added to."""
    ops = _ops()
    g = torch.Generator().manual_seed(77)
    M, E, Fd = 333, 264, 1048
    dqkv, dh, dz1 = _rnd((M, 3 * E), dtype, g), _rnd((M, E), dtype, g), _rnd((M, Fd), dtype, g)
    wide = _rnd((M, 2 * E), dtype, g)                     # a strided view: the left half of a wider tensor
    dxn, x = _rnd((M, E), dtype, g), _rnd((M, E), dtype, g, 2.0)
    dhn, h = _rnd((M, E), dtype, g), _rnd((M, E), dtype, g, 0.5)
    dev = lambda t: t.to(DEV)
    stats = []
    for t in (x, h):
        mu = t.double().mean(1)
        rs = (t.double().var(1, unbiased=False) + 1e-5).rsqrt()
        stats.append((mu.float().to(DEV), rs.float().to(DEV)))
    accs = [torch.full((n,), 0.5, dtype=torch.float32, device=DEV) for n in (3 * E, E, Fd, E, E, E, E, E)]
    wd = dev(wide)
    ops.vec_param_grads([(dev(dqkv), accs[0]), (dev(dh), accs[1]), (dev(dz1), accs[2]), (wd[:, :E], accs[3]),
                         (dev(dxn), dev(x), stats[0][0], stats[0][1], accs[4], accs[5]),
                         (dev(dhn), dev(h), stats[1][0], stats[1][1], accs[6], accs[7])])
    tol = 1.0 if dtype != torch.float32 else 10.0
    for got, ref, name in ((accs[0], dqkv, "in_proj.bias"), (accs[1], dh, "out_proj.bias"), (accs[2], dz1, "fc1.bias"),
                           (accs[3], wide[:, :E], "fc2.bias (strided)")):
        assert_close(got - 0.5, ref.double().sum(0), torch.float32, name, 1e2 * tol)
    for k, (dy, t) in enumerate(((dxn, x), (dhn, h))):
        mu, rs = stats[k][0].double().cpu(), stats[k][1].double().cpu()
        xhat = (t.double() - mu[:, None]) * rs[:, None]
        assert_close(accs[4 + 2 * k] - 0.5, (dy.double() * xhat).sum(0), torch.float32, "dgamma %d" % k, 1e2 * tol)
        assert_close(accs[5 + 2 * k] - 0.5, dy.double().sum(0), torch.float32, "dbeta %d" % k, 1e2 * tol)


def test_fill_probe_runs_every_mix():
    """The global -> LDS streaming probe behind `bench.py --fill-path`: every hit : miss mix launches, completes and
    leaves its source regions as they were (it only reads)."""
    ops = _ops()
    big = torch.arange(1 << 22, dtype=torch.int32, device=DEV)       # 16 MiB
    small = torch.arange(1 << 18, dtype=torch.int32, device=DEV)     # 1 MiB
    for hpm in (-1, 0, 1, 3, 7):
        for stride in (0, 2048, 10240):
            moved = ops.fill_probe(big, small, hpm, 64, 16, row_stride=stride)
            assert moved == 64 * 4 * 16 * 8192
    torch.cuda.synchronize()
    assert torch.equal(big, torch.arange(1 << 22, dtype=torch.int32, device=DEV))
    assert torch.equal(small, torch.arange(1 << 18, dtype=torch.int32, device=DEV))


def test_error_paths():
    """Bad arguments come back as status codes with a message; nothing is launched."""
    import ctypes
    from terapipe_amd import _lib as L
    lib = L.load()
    d = L.GemmDesc()
    assert lib.tp_gemm(ctypes.byref(d), None, 0, None) != 0
    assert b"tp_gemm" in lib.tp_last_error()
    ops = _ops()
    x = torch.zeros(4, 20, dtype=torch.float16, device=DEV)   # E not a multiple of 8
    w = torch.zeros(20, dtype=torch.float16, device=DEV)
    with pytest.raises(L.TeraPipeHipError):
        ops.layernorm_fwd(x, w, w)
    q = torch.zeros(2, 4, 72, dtype=torch.float16, device=DEV)  # head_dim 72 unsupported
    kc = torch.zeros(2, 8, 72, dtype=torch.float16, device=DEV)
    with pytest.raises(L.TeraPipeHipError, match="head_dim"):
        ops.attn_prefix_fwd(q, kc, kc, 1, 2, 72, 4, 0, 1.0)
    with pytest.raises(L.TeraPipeHipError):
        ops.layernorm_fwd(torch.zeros(4, 64), torch.zeros(64), torch.zeros(64))  # CPU tensors
