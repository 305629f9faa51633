"""Parity of the GEMM kernels (through the C ABI) with the CPU oracle.

Tolerance (bf16 operands, fp32 accumulate): normwise relative error <= 1e-2
against the oracle evaluated in float64 on the same bf16-rounded inputs.  What is
actually left is the final rounding to bf16 (about 2e-3 normwise); with an fp32
result only fp32 accumulation error remains (<= 1e-5).
"""

import numpy as np
import pytest
import torch

from oracle import linear as ol

pytestmark = pytest.mark.gpu

BF16_TOL = 1e-2
F32_TOL = 1e-5


def rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


def bf16_inputs(M, N, K, seed, x_std=1.0, w_std=0.02, g_std=1e-3):
    g = torch.Generator().manual_seed(seed)
    X = (torch.randn(M, K, generator=g) * x_std).bfloat16()
    W = (torch.randn(N, K, generator=g) * w_std).bfloat16()
    dY = (torch.randn(M, N, generator=g) * g_std).bfloat16()
    return X, W, dY


def np64(t):
    return t.float().cpu().numpy().astype(np.float64)


SHAPES = [
    (32, 64, 64), (16, 128, 128), (2, 256, 256),       # the reference's test shapes
    (256, 256, 64), (128, 128, 64), (256, 512, 320),   # exact tiles, 1 and 5 contraction steps
    (100, 72, 40), (33, 8, 8), (1, 8, 16), (257, 264, 72), (130, 136, 520),  # ragged
    (512, 1024, 1024),
]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_three_gemms_match_oracle(M, N, K):
    from axonn_amd import ops

    X, W, dY = bf16_inputs(M, N, K, seed=M * 7 + N * 3 + K)
    yo, _ = ol.linear_forward(np64(X), np64(W).reshape(-1), (N, K))
    bw = ol.linear_backward(np64(X), np64(W).reshape(-1), (N, K), np64(dY))
    Xd, Wd, dYd = X.cuda(), W.cuda(), dY.cuda()
    y, _ = ops.gemm_fwd(Xd, Wd)
    dx = ops.gemm_dgrad(dYd, Wd)
    dw = ops.gemm_wgrad(dYd, Xd)
    dw32 = ops.gemm_wgrad(dYd, Xd, out_dtype=torch.float32)
    assert y.dtype == torch.bfloat16 and y.shape == (M, N)
    assert rel(np64(y), yo) < BF16_TOL
    assert rel(np64(dx), bw["dx"]) < BF16_TOL
    assert rel(np64(dw), bw["dw"].reshape(N, K)) < BF16_TOL
    assert rel(np64(dw32), bw["dw"].reshape(N, K)) < F32_TOL


@pytest.mark.parametrize("M,N,K", [(64, 64, 64), (300, 136, 96), (256, 256, 128)])
@pytest.mark.parametrize("epilogue", ["bias", "bias_gelu", "gelu"])
def test_fused_epilogues_match_oracle(M, N, K, epilogue):
    from axonn_amd import ops

    X, W, _ = bf16_inputs(M, N, K, seed=11, w_std=0.2)
    b = torch.randn(N, generator=torch.Generator().manual_seed(5)) * 0.5
    bias = b if "bias" in epilogue else None
    act = "gelu" if "gelu" in epilogue else None
    yo, zo = ol.linear_forward(np64(X), np64(W).reshape(-1), (N, K),
                               bias=None if bias is None else b.double().numpy(), activation=act)
    y, z = ops.gemm_fwd(X.cuda(), W.cuda(), bias=None if bias is None else b.cuda(),
                        activation=act, save_z=True)
    assert rel(np64(y), yo) < BF16_TOL
    if act:
        assert rel(np64(z), zo) < BF16_TOL
    else:
        assert z is None


@pytest.mark.parametrize("M,N,K", [(64, 64, 64), (300, 136, 96), (512, 768, 128), (4096, 6144, 256)])
@pytest.mark.parametrize("epilogue", ["bias", "bias_gelu"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_forward_with_fp32_result_matches_oracle(M, N, K, epilogue, dtype):
    """The forward whose sum with the fp32 bias stays fp32 (what type promotion makes of the
    reference's `x + bias` under autocast): only fp32 accumulation error is left, on every
    tile shape (register-staged, 128 x 128, whole rounds of 256 x 256 plus a rest)."""
    from axonn_amd import ops

    g = torch.Generator().manual_seed(M + N + K)
    X = torch.randn(M, K, generator=g).to(dtype)
    W = (torch.randn(N, K, generator=g) * 0.2).to(dtype)
    b = torch.randn(N, generator=g) * 0.5
    act = "gelu" if "gelu" in epilogue else None
    yo, zo = ol.linear_forward(np64(X), np64(W).reshape(-1), (N, K), bias=b.double().numpy(),
                               activation=act)
    y, z = ops.gemm_fwd(X.cuda(), W.cuda(), bias=b.cuda(), activation=act, save_z=True, out_f32=True)
    assert y.dtype == torch.float32 and y.shape == (M, N)
    assert rel(np64(y), yo) < F32_TOL
    if act:
        assert z.dtype == dtype and rel(np64(z), zo) < BF16_TOL
    # the 16-bit result of the same call is this one, rounded once
    y16, _ = ops.gemm_fwd(X.cuda(), W.cuda(), bias=b.cuda(), activation=act)
    assert torch.equal(y16, y.to(dtype))
    with pytest.raises(ValueError):
        ops.gemm_fwd(X.cuda(), W.cuda(), out_f32=True)


def test_dgelu_dbias_matches_oracle():
    from axonn_amd import ops

    g = torch.Generator().manual_seed(3)
    M, N = 333, 520
    dY = torch.randn(M, N, generator=g).bfloat16()
    Z = (torch.randn(M, N, generator=g) * 2).bfloat16()
    dz, db = ops.dgelu_dbias(dY.cuda(), Z.cuda(), want_dbias=True)
    want = np64(dY) * ol.dgelu(np64(Z))
    assert rel(np64(dz), want) < BF16_TOL
    # dbias is the column sum of the rounded dZ the weight-gradient kernel reads
    assert rel(db.cpu().numpy(), np64(dz).sum(0)) < 1e-6
    assert rel(db.cpu().numpy(), want.sum(0)) < BF16_TOL
    _, db2 = ops.dgelu_dbias(dY.cuda(), None, want_dbias=True)
    assert rel(db2.cpu().numpy(), np64(dY).sum(0)) < 1e-6
    # fp32 variant
    dz32, db32 = ops.dgelu_dbias(dY.float().cuda(), Z.float().cuda(), want_dbias=True)
    assert rel(dz32.cpu().numpy(), want) < 1e-6 and rel(db32.cpu().numpy(), want.sum(0)) < 1e-5


def test_gelu_and_its_derivative_elementwise_over_the_tails():
    """The kernels evaluate erf by a 5-term rational formula (|error| <= 1.5e-7);
    checked element by element from -12 to 12, not just in norm: the derivative in
    fp32 against the oracle's math.erf, the fused forward epilogue (identity weight,
    so Z = X exactly) to one bf16 rounding of the oracle's value."""
    from axonn_amd import ops

    n = 256 * 256
    z32 = torch.linspace(-12.0, 12.0, n).reshape(256, 256)
    dz, _ = ops.dgelu_dbias(torch.ones_like(z32).cuda(), z32.cuda(), want_dbias=False)
    want = ol.dgelu(z32.double().numpy())
    assert np.max(np.abs(dz.cpu().numpy().astype(np.float64) - want)) < 1e-6
    x = z32.bfloat16()
    eye = torch.eye(256).bfloat16()
    y, z = ops.gemm_fwd(x.cuda(), eye.cuda(), activation="gelu", save_z=True)
    assert torch.equal(z.cpu(), x)
    exact = ol.gelu(np64(x))
    got = np64(y)
    ulp = np.maximum(np.abs(exact), 2.0 ** -126) * 2.0 ** -8   # half a bf16 ulp is 2^-9 relative
    assert np.all(np.abs(got - exact) <= ulp + 5e-7)


def test_dbias_reduction_with_few_bands_and_ragged_columns():
    """Column sums over 1, 3 and 9 row bands of 128 (the reduction splits the
    bands over 4 threads) and a column count that is not a multiple of 64."""
    from axonn_amd import ops

    g = torch.Generator().manual_seed(11)
    for M in (5, 300, 1100):
        dY = torch.randn(M, 72, generator=g).bfloat16()
        _, db = ops.dgelu_dbias(dY.cuda(), None, want_dbias=True)
        assert rel(db.cpu().numpy(), np64(dY).sum(0)) < 1e-6
        acc = torch.ones(72, device="cuda")
        ops.dgelu_dbias(dY.cuda(), None, want_dbias=True, dbias_out=acc, accumulate=True)
        assert rel(acc.cpu().numpy(), 1.0 + np64(dY).sum(0)) < 1e-6


def test_wgrad_accumulates_over_micro_batches():
    """dW += dY^T X over 4 micro-batches equals the weight gradient of the
    concatenated batch (overlap_communication.py:38-47 semantics, in fp32 and in
    the parameter's bf16)."""
    from axonn_amd import ops

    N, K, M = 136, 72, 96
    xs, gs = [], []
    for mb in range(4):
        X, _, dY = bf16_inputs(M, N, K, seed=mb)
        xs.append(X)
        gs.append(dY)
    want = ol.linear_backward(np.concatenate([np64(x) for x in xs]), np.zeros(N * K), (N, K),
                              np.concatenate([np64(g) for g in gs]))["dw"].reshape(N, K)
    acc32 = torch.zeros(N, K, device="cuda")
    acc16 = None
    ref16 = None
    for x, g in zip(xs, gs):
        ops.gemm_wgrad(g.cuda(), x.cuda(), out=acc32, accumulate=True)
        if acc16 is None:
            acc16 = ops.gemm_wgrad(g.cuda(), x.cuda())
        else:
            ops.gemm_wgrad(g.cuda(), x.cuda(), out=acc16, accumulate=True)
        part = ol.linear_backward(np64(x), np.zeros(N * K), (N, K), np64(g))["dw"]
        ref16 = ol.accumulate(ref16, part, "bf16")
    assert rel(acc32.cpu().numpy(), want) < F32_TOL
    assert rel(np64(acc16), want) < BF16_TOL
    assert rel(np64(acc16), ref16.reshape(N, K)) < BF16_TOL


def test_strided_operands_and_leading_dimensions():
    """Row-strided views (ld > row length) go to the kernels without a copy."""
    from axonn_amd import ops

    big = torch.randn(64, 256, generator=torch.Generator().manual_seed(1)).bfloat16().cuda()
    X = big[:, 64:192]  # 64 x 128 view, ld 256, 16-byte aligned start
    W = (torch.randn(72, 128, generator=torch.Generator().manual_seed(2)) * 0.1).bfloat16().cuda()
    y, _ = ops.gemm_fwd(X, W)
    yo, _ = ol.linear_forward(np64(X), np64(W).reshape(-1), (72, 128))
    assert rel(np64(y), yo) < BF16_TOL
    Xo = big[:, 3:131]  # misaligned start: the wrapper copies
    y2, _ = ops.gemm_fwd(Xo, W)
    yo2, _ = ol.linear_forward(np64(Xo), np64(W).reshape(-1), (72, 128))
    assert rel(np64(y2), yo2) < BF16_TOL


def test_unsupported_shapes_raise():
    from axonn_amd import _native as nv
    from axonn_amd import ops

    X = torch.randn(8, 12, device="cuda").bfloat16()
    W = torch.randn(16, 12, device="cuda").bfloat16()
    Y = torch.empty(8, 16, dtype=torch.bfloat16, device="cuda")
    # the entry points take feature counts that are multiples of 8 ...
    with pytest.raises(nv.AxnError, match="multiples of 8") as e:
        nv.call("axn_gemm_fwd", nv.ptr(X), nv.ptr(W), None, nv.ptr(Y), None, 8, 16, 12, 12, 12, 16, 0,
                nv.current_stream())
    assert e.value.code == nv.AXN_ESHAPE
    with pytest.raises(nv.AxnError, match="axn_gemm_fwd_f16: N and K must be multiples of 8"):
        nv.call("axn_gemm_fwd_f16", nv.ptr(X), nv.ptr(W), None, nv.ptr(Y), None, 8, 16, 12, 12, 12, 16, 0,
                nv.current_stream())
    # ... and the tensor-level wrapper pads other shapes with zeros and cuts the result back
    y, _ = ops.gemm_fwd(X, W)
    assert y.shape == (8, 16) and rel(np64(y), np64(X.float() @ W.float().t())) < BF16_TOL
    with pytest.raises(TypeError, match="bf16, fp16 or fp32"):
        ops.gemm_fwd(X.double(), W.double())
    with pytest.raises(TypeError):
        ops.gemm_fwd(X, W.float())


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (5, 7, 3), (64, 48, 40), (130, 70, 257), (66, 130, 8),
                                   (33, 17, 1000), (64, 1024, 4096),
                                   (1030, 1034, 70), (1032, 1040, 72), (2050, 2052, 36), (2048, 2064, 40),
                                   (2049, 2051, 33), (2048, 1030, 1034)])
def test_fp32_gemms_match_oracle(M, N, K):
    """Ragged and whole shapes on each of the fp32 kernel's tiles (16, 32 and 64 rows and
    columns per wave: the last five shapes), with and without the divisibility its vector
    loads and stores need; small outputs with a contraction of 256 or more have four waves
    share a tile (products of (64, 1024, 4096) and (33, 17, 1000)), and so do 1024 to 4095
    of the 32 x 32 tiles with a contraction of 2048 or more (wgrad of the last shape)."""
    from axonn_amd import ops

    g = torch.Generator().manual_seed(M + N + K)
    X, W, dY = torch.randn(M, K, generator=g), torch.randn(N, K, generator=g) * 0.1, torch.randn(M, N, generator=g)
    b = torch.randn(N, generator=g)
    yo, zo = ol.linear_forward(X.double().numpy(), W.double().numpy().reshape(-1), (N, K),
                               bias=b.double().numpy(), activation="gelu")
    bw = ol.linear_backward(X.double().numpy(), W.double().numpy().reshape(-1), (N, K), dY.double().numpy())
    y, z = ops.gemm_fwd(X.cuda(), W.cuda(), bias=b.cuda(), activation="gelu", save_z=True)
    assert rel(y.cpu().numpy(), yo) < F32_TOL and rel(z.cpu().numpy(), zo) < F32_TOL
    assert rel(ops.gemm_dgrad(dY.cuda(), W.cuda()).cpu().numpy(), bw["dx"]) < F32_TOL
    dw = ops.gemm_wgrad(dY.cuda(), X.cuda())
    assert rel(dw.cpu().numpy(), bw["dw"].reshape(N, K)) < F32_TOL
    ops.gemm_wgrad(dY.cuda(), X.cuda(), out=dw, accumulate=True)
    assert rel(dw.cpu().numpy(), 2 * bw["dw"].reshape(N, K)) < F32_TOL


@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (256, 384, 192), (512, 256, 320), (4096, 3072, 128),
                                   (4096, 3072, 320), (4608, 4096, 64),
                                   (4096, 6144, 4096), (4096, 256, 6144), (6144, 4096, 128),
                                   (2304, 2048, 192), (2048, 4096, 64),
                                   (4096, 14336, 128), (128, 14336, 4096), (192, 6144, 4096),
                                   (2048, 12288, 64), (8192, 7168, 320)])
def test_tile_kernels_every_output_block_with_epilogues(M, N, K):
    """Whole-tile shapes on the one-wave-per-SIMD kernel (128 x 128 tiles up to 128
    tiles of 256 x 256 and from 257 to 320 of them, else 256 x 256), checked element by
    element so that a single wrong 16 x 16 accumulator block shows (a block copied out of
    its registers before its last MFMA had finished once passed the normwise checks of
    other shapes).  The last three shapes have 384 large tiles in one of their products:
    one full round of large tiles and a rest of 128 for the small tile, cut along the
    output columns (forward of the first, dgrad of the second) or rows (wgrad of the
    first, forward of the third), with the bias and the saved pre-activation cut too.  The
    two after them have 72 and 128 large tiles in their forward: 256 x 128 tiles throughout.
    The last five have 384 or 896 large tiles in their forward or weight gradient, with 1 to
    64 contraction stages and grids of 8, 16, 32, 48 and 56 tile rows: one and three rounds
    and a rest of 128."""
    from axonn_amd import ops

    g = torch.Generator(device="cuda").manual_seed(M + N + K)
    X = torch.randn(M, K, generator=g, device="cuda").bfloat16()
    W = (torch.randn(N, K, generator=g, device="cuda") * 0.2).bfloat16()
    b = torch.randn(N, generator=g, device="cuda") * 0.5
    dY = torch.randn(M, N, generator=g, device="cuda").bfloat16()
    pre = X.float() @ W.float().t()
    scale = pre.abs().max().item()

    def close(got, want, ulps=1.0):
        return bool(((got.float() - want).abs() <= ulps * 2.0 ** -8 * want.abs() + 1e-3 * scale).all())

    for bias, act in ((None, None), (b, None), (b, "gelu"), (None, "gelu")):
        y, z = ops.gemm_fwd(X, W, bias=bias, activation=act, save_z=act is not None)
        zr = pre + (bias if bias is not None else 0)
        assert close(y, torch.nn.functional.gelu(zr) if act else zr)
        if act:
            assert close(z, zr)
    assert close(ops.gemm_dgrad(dY, W), dY.float() @ W.float())
    dwr = dY.float().t() @ X.float()
    dw = ops.gemm_wgrad(dY, X)
    assert close(dw, dwr)
    dw32 = ops.gemm_wgrad(dY, X, out_dtype=torch.float32)
    assert bool(((dw32 - dwr).abs() <= 1e-4 * dwr.abs().max()).all())
    ops.gemm_wgrad(dY, X, out=dw, accumulate=True)
    assert close(dw, 2 * dwr, ulps=2.0)


# ---- the 256 x 256-tile kernel: few and many contraction stages, all layouts/epilogues ----
@pytest.mark.parametrize("K", [64, 128, 192, 256, 448])
def test_tile256_kernel_short_contractions(K):
    """Shapes of more than 128 whole 256 x 256 tiles take the one-wave-per-SIMD kernel; it
    walks the contraction in stages of 64 and copies two stages ahead, so K = 64 and
    128 exercise the start-up and drain paths alone (1 and 2 stages), 192 and 256 a
    single or two steady-state stages, and 448 the steady state proper."""
    from axonn_amd import ops

    M, N = 4096, 3072
    g = torch.Generator(device="cuda").manual_seed(K)
    X = torch.randn(M, K, generator=g, device="cuda").bfloat16()
    W = (torch.randn(N, K, generator=g, device="cuda") * 0.05).bfloat16()
    b = torch.randn(N, generator=g, device="cuda")
    y, z = ops.gemm_fwd(X, W, bias=b, activation="gelu", save_z=True)
    zr = X.float() @ W.float().t() + b           # fp32 reference of the same op
    assert rel(np64(z), np64(zr)) < BF16_TOL
    assert rel(np64(y), np64(torch.nn.functional.gelu(zr))) < BF16_TOL
    rows = torch.arange(0, M, 97, device="cuda")
    yo, zo = ol.linear_forward(np64(X[rows]), np64(W).reshape(-1), (N, K), bias=np64(b),
                               activation="gelu")
    assert rel(np64(y[rows]), yo) < BF16_TOL and rel(np64(z[rows]), zo) < BF16_TOL


@pytest.mark.parametrize("Kc", [64, 192, 320])
def test_tile256_kernel_backward_layouts(Kc):
    """dgrad (B operand contraction-strided) and wgrad (both operands
    contraction-strided, bf16 and fp32 accumulate) on the 256 x 256-tile kernel."""
    from axonn_amd import ops

    g = torch.Generator(device="cuda").manual_seed(Kc + 1)
    # dgrad: dX[M, K] = dY[M, N] W[N, K], contraction N = Kc, output 4096 x 3072
    dY = torch.randn(4096, Kc, generator=g, device="cuda").bfloat16()
    W = torch.randn(Kc, 3072, generator=g, device="cuda").bfloat16()
    dx = ops.gemm_dgrad(dY, W)
    assert rel(np64(dx), np64(dY.float() @ W.float())) < BF16_TOL
    # wgrad: dW[N, K] = dY[M, N]^T X[M, K], contraction M = Kc, output 3072 x 4096
    dY2 = torch.randn(Kc, 3072, generator=g, device="cuda").bfloat16()
    X2 = torch.randn(Kc, 4096, generator=g, device="cuda").bfloat16()
    ref = dY2.float().t() @ X2.float()
    dw = ops.gemm_wgrad(dY2, X2)
    dw32 = ops.gemm_wgrad(dY2, X2, out_dtype=torch.float32)
    assert rel(np64(dw), np64(ref)) < BF16_TOL
    assert rel(np64(dw32), np64(ref)) < F32_TOL
    ops.gemm_wgrad(dY2, X2, out=dw32, accumulate=True)
    assert rel(np64(dw32), 2 * np64(ref)) < F32_TOL
    rows = torch.arange(0, 3072, 61, device="cuda")
    dwo = np64(dY2[:, rows]).T @ np64(X2)
    assert rel(np64(dw32[rows]), 2 * dwo) < F32_TOL


# ---- full benchmark shapes: size-independent properties + sampled oracle ------
FULL = {
    "qkv": (4096, 6144, 4096), "o": (4096, 4096, 4096), "gate_up": (4096, 14336, 4096),
    "down": (4096, 4096, 14336), "mlp_shard": (8192, 5120, 2560), "skinny": (512, 8192, 3584),
}


@pytest.mark.parametrize("name", sorted(FULL))
def test_full_size_shapes_sampled_oracle_and_properties(name):
    from axonn_amd import ops

    M, N, K = FULL[name]
    g = torch.Generator(device="cuda").manual_seed(0)
    X = torch.randn(M, K, generator=g, device="cuda").bfloat16()
    W = (torch.randn(N, K, generator=g, device="cuda") * 0.02).bfloat16()
    dY = (torch.randn(M, N, generator=g, device="cuda") * 1e-3).bfloat16()
    y, _ = ops.gemm_fwd(X, W)
    dx = ops.gemm_dgrad(dY, W)
    dw = ops.gemm_wgrad(dY, X, out_dtype=torch.float32)
    # (a) oracle on a sample of rows / columns of each result
    rs = np.random.default_rng(1)
    rows = np.sort(rs.choice(M, 48, replace=False))
    nrows = np.sort(rs.choice(N, 48, replace=False))
    ti, tn = torch.from_numpy(rows).cuda(), torch.from_numpy(nrows).cuda()
    Wn, Xn, dYn = np64(W), np64(X[ti]), np64(dY[ti])
    yo, _ = ol.linear_forward(Xn, Wn.reshape(-1), (N, K))
    assert rel(np64(y[ti]), yo) < BF16_TOL
    assert rel(np64(dx[ti]), dYn @ Wn) < BF16_TOL
    dwo = np64(dY[:, tn]).T @ np64(X)   # rows `nrows` of dW
    assert rel(dw[tn].cpu().numpy(), dwo) < 1e-4
    # (b) linearity in the input: f(2x) = 2 f(x) exactly (powers of two commute with rounding)
    y2, _ = ops.gemm_fwd(X * 2, W)
    assert torch.equal(y2, y * 2)
    # (c) <dY, X W^T> = <dY W, X> = <dY^T X, W>: the three kernels agree with each other
    a = float((dY.double() * y.double()).sum())
    yd = float((dx.double() * X.double()).sum())
    wd = float((dw.double() * W.double()).sum())
    scale = float(dY.double().norm() * y.double().norm())
    assert abs(a - yd) < 1e-3 * scale and abs(a - wd) < 1e-3 * scale
    # (d) determinism: the same call gives the same bits
    y3, _ = ops.gemm_fwd(X, W)
    assert torch.equal(y3, y)


def test_operand_of_two_gibibytes_takes_the_64_bit_path():
    """The tile kernels address an operand with 32-bit byte offsets; an operand of
    2 GiB or more must go to the kernel with 64-bit addressing and still be right
    in its last rows."""
    from axonn_amd import ops

    M, K, N = 32768, 32768, 256          # X is exactly 2^31 bytes
    g = torch.Generator(device="cuda").manual_seed(5)
    X = torch.empty(M, K, dtype=torch.bfloat16, device="cuda")
    for r in range(0, M, 4096):          # filled in slabs: no 4 GiB fp32 temporary
        X[r:r + 4096] = torch.randn(4096, K, generator=g, device="cuda").bfloat16()
    W = (torch.randn(N, K, generator=g, device="cuda") * 0.02).bfloat16()
    y, _ = ops.gemm_fwd(X, W)
    rows = torch.cat([torch.arange(0, 64), torch.arange(M // 2 - 32, M // 2 + 32), torch.arange(M - 64, M)]).cuda()
    ref = X[rows].float() @ W.float().t()
    assert rel(np64(y[rows]), np64(ref)) < BF16_TOL
    dY = torch.randn(M, N, generator=g, device="cuda").bfloat16()
    dw = ops.gemm_wgrad(dY, X, out_dtype=torch.float32)       # X as the 2 GiB contraction-strided operand
    cols = torch.arange(K - 128, K, device="cuda")
    refw = dY.float().t() @ X[:, cols].float()
    assert rel(np64(dw[:, cols]), np64(refw)) < 1e-4
    del X
    torch.cuda.empty_cache()


@pytest.mark.parametrize("M,N,K", [(128, 128, 4096), (512, 8192, 3584), (256, 1024, 2048), (384, 512, 1024),
                                   (4096, 256, 512)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_split_contraction_matches_oracle_and_is_deterministic(M, N, K, dtype):
    """Problems with few output tiles run with the contraction cut into 2, 4 or 8 parts
    whose fp32 partial products are added in a fixed order: the same bar as the plain
    kernels (what is left is the final rounding), and bit-identical results on repeats."""
    from axonn_amd import _native as nv
    from axonn_amd import ops

    lib = nv.load()
    g = torch.Generator().manual_seed(M + N + K)
    X = torch.randn(M, K, generator=g).to(dtype)
    W = (torch.randn(N, K, generator=g) * 0.02).to(dtype)
    dY = (torch.randn(M, N, generator=g) * 1e-2).to(dtype)
    split = [lib.axn_gemm_workspace_bytes(op, M, N, K) > 0 for op in (0, 1, 2)]
    assert any(split), "shape chosen to exercise the split path"
    yo, _ = ol.linear_forward(np64(X), np64(W).reshape(-1), (N, K))
    bw = ol.linear_backward(np64(X), np64(W).reshape(-1), (N, K), np64(dY))
    tol = BF16_TOL if dtype == torch.bfloat16 else 1e-3
    Xd, Wd, dYd = X.cuda(), W.cuda(), dY.cuda()
    y, _ = ops.gemm_fwd(Xd, Wd)
    dx = ops.gemm_dgrad(dYd, Wd)
    dw = ops.gemm_wgrad(dYd, Xd)
    dw32 = ops.gemm_wgrad(dYd, Xd, out_dtype=torch.float32)
    assert rel(np64(y), yo) < tol and rel(np64(dx), bw["dx"]) < tol
    assert rel(np64(dw), bw["dw"].reshape(N, K)) < tol
    assert rel(np64(dw32), bw["dw"].reshape(N, K)) < F32_TOL
    # accumulation into an existing fp32 gradient through the reducing pass
    acc = dw32.clone()
    ops.gemm_wgrad(dYd, Xd, out=acc, accumulate=True)
    assert rel(np64(acc), 2 * bw["dw"].reshape(N, K)) < F32_TOL
    acc16 = dw.clone()   # and into a 16-bit gradient: old value + sum, rounded once
    ops.gemm_wgrad(dYd, Xd, out=acc16, accumulate=True)
    assert rel(np64(acc16), np64(dw) + bw["dw"].reshape(N, K)) < tol
    for _ in range(2):
        assert torch.equal(ops.gemm_fwd(Xd, Wd)[0], y) and torch.equal(ops.gemm_dgrad(dYd, Wd), dx)
    # the split result equals the unsplit kernel's up to the order of the fp32 sums
    y_plain = torch.empty_like(y)
    name = "axn_gemm_fwd" if dtype == torch.bfloat16 else "axn_gemm_fwd_f16"
    nv.call(name, nv.ptr(Xd), nv.ptr(Wd), None, nv.ptr(y_plain), None, M, N, K, K, K, N, 0, nv.current_stream())
    assert rel(np64(y), np64(y_plain)) < (4e-3 if dtype == torch.bfloat16 else 5e-4)


def test_split_contraction_output_rows_may_be_strided():
    from axonn_amd import _native as nv

    M, N, K = 128, 256, 2048
    g = torch.Generator(device="cuda").manual_seed(3)
    X = torch.randn(M, K, device="cuda", generator=g).bfloat16()
    W = (torch.randn(N, K, device="cuda", generator=g) * 0.02).bfloat16()
    big = torch.zeros(M, N + 64, device="cuda", dtype=torch.bfloat16)
    nbytes = nv.load().axn_gemm_workspace_bytes(0, M, N, K)
    assert nbytes > 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    nv.call("axn_gemm_fwd_ws", nv.ptr(X), nv.ptr(W), None, nv.ptr(big), None, nv.BF16, M, N, K, K, K, N + 64,
            0, nv.ptr(ws), nbytes, nv.current_stream())
    want = (X.float() @ W.float().t())
    assert rel(np64(big[:, :N]), np64(want)) < BF16_TOL
    assert not big[:, N:].any()


@pytest.mark.parametrize("M,N,K", [(4096, 6144, 4096), (8192, 5120, 2560)])
def test_back_to_back_launches_are_bitwise_reproducible(M, N, K):
    """Seventy-five launches in a row over three operand sets (so that operands come from
    HBM and launches overlap their neighbours' tails), four times: every repeat must give
    the same bits, and the right ones.  A tile read before it has landed, or overwritten
    while still being read, shows here as a repeat that differs."""
    from axonn_amd import _native as nv

    lib, st = nv.load(), nv.current_stream()
    g = torch.Generator(device="cuda").manual_seed(5)
    sets = []
    for _ in range(3):
        X = torch.randn(M, K, generator=g, device="cuda").bfloat16()
        W = (torch.randn(N, K, generator=g, device="cuda") * 0.02).bfloat16()
        dY = (torch.randn(M, N, generator=g, device="cuda") * 1e-3).bfloat16()
        sets.append((X, W, dY, torch.empty(M, N, dtype=torch.bfloat16, device="cuda"),
                     torch.empty(M, K, dtype=torch.bfloat16, device="cuda"),
                     torch.empty(N, K, dtype=torch.bfloat16, device="cuda")))
    first = None
    for _ in range(4):
        for i in range(25):
            X, W, dY, Y, dX, dW = sets[i % 3]
            nv.check(lib.axn_gemm_fwd(X.data_ptr(), W.data_ptr(), None, Y.data_ptr(), None, M, N, K, K, K, N,
                                      0, st))
        for i in range(25):
            X, W, dY, Y, dX, dW = sets[i % 3]
            nv.check(lib.axn_gemm_dgrad(dY.data_ptr(), W.data_ptr(), dX.data_ptr(), M, N, K, N, K, K, st))
        for i in range(25):
            X, W, dY, Y, dX, dW = sets[i % 3]
            nv.check(lib.axn_gemm_wgrad(dY.data_ptr(), X.data_ptr(), dW.data_ptr(), M, N, K, N, K, K, 0,
                                        nv.BF16, st))
        torch.cuda.synchronize()
        got = [t.clone() for t in sets[0][3:]]
        if first is None:
            first = got
            X, W, dY = sets[0][:3]
            for t, want in zip(got, (X.float() @ W.float().t(), dY.float() @ W.float(), dY.float().t() @ X.float())):
                assert float((t.float() - want).norm() / want.norm()) < 3e-3
        for a, b in zip(got, first):
            assert torch.equal(a, b)


@pytest.mark.parametrize("M,N,K", [(512, 512, 512), (4096, 2304, 256), (4096, 6144, 256), (2304, 2048, 192)])
def test_tile_kernels_take_row_strided_operands(M, N, K):
    """Operands that are column slices of wider buffers (leading dimension twice the row
    length) on the 128 x 128-, 256 x 256- and 256 x 128-tile kernels and on a cut problem
    (384 large tiles): the result equals the one from contiguous copies bit for bit."""
    from axonn_amd import ops

    g = torch.Generator(device="cuda").manual_seed(M + N + K)
    Xb = torch.randn(M, 2 * K, device="cuda", generator=g).bfloat16()
    Wb = (torch.randn(N, 2 * K, device="cuda", generator=g) * 0.05).bfloat16()
    dYb = (torch.randn(M, 2 * N, device="cuda", generator=g) * 0.1).bfloat16()
    X, W, dY = Xb[:, K:], Wb[:, :K], dYb[:, N:]
    assert not X.is_contiguous() and X.stride(0) == 2 * K
    Xc, Wc, dYc = X.contiguous(), W.contiguous(), dY.contiguous()
    b = torch.randn(N, device="cuda", generator=g)
    y, z = ops.gemm_fwd(X, W, bias=b, activation="gelu", save_z=True)
    yc, zc = ops.gemm_fwd(Xc, Wc, bias=b, activation="gelu", save_z=True)
    assert torch.equal(y, yc) and torch.equal(z, zc)
    assert torch.equal(ops.gemm_dgrad(dY, W), ops.gemm_dgrad(dYc, Wc))
    assert torch.equal(ops.gemm_wgrad(dY, X, out_dtype=torch.float32),
                       ops.gemm_wgrad(dYc, Xc, out_dtype=torch.float32))
    ref = torch.nn.functional.gelu(Xc.float() @ Wc.float().t() + b)
    assert rel(np64(y), np64(ref)) < BF16_TOL


@pytest.mark.parametrize("tm,tn", [(8, 16), (8, 17), (16, 16), (16, 17), (17, 17), (16, 20), (16, 21),
                                   (12, 24), (20, 20), (16, 33), (5, 13)])
def test_every_launch_rule_boundary(tm, tn):
    """Output sizes of tm x tn large tiles around every threshold of the kernel selection:
    128 tiles (small tile) and 136 (large); 256 (one round); 272 and 320 (a round and a
    rest of 16 / 64 for the small tile); 289 and 288 (no whole tile rows or columns to
    cut: small tile throughout); 336 (rest of 80 on 256 x 128 tiles); 400 (rest of 144:
    not cut); 528 (two rounds and 16); 65 (256 x 128 tiles throughout).  Forward, dgrad
    and wgrad of each, every element against an fp32 product of the same operands."""
    from axonn_amd import ops

    M, N, K = 256 * tm, 256 * tn, 64
    g = torch.Generator(device="cuda").manual_seed(100 * tm + tn)
    X = torch.randn(M, K, device="cuda", generator=g).bfloat16()
    W = (torch.randn(N, K, device="cuda", generator=g) * 0.1).bfloat16()
    y, _ = ops.gemm_fwd(X, W)
    ref = X.float() @ W.float().t()
    assert float((y.float() - ref).abs().max()) <= 2e-2 * float(ref.abs().max())
    # the same tile grids as outputs of dgrad (M x K') and wgrad (N' x K'), contraction 64
    dY = (torch.randn(M, 64, device="cuda", generator=g) * 0.1).bfloat16()     # [M, N''=64]
    W2 = (torch.randn(64, N, device="cuda", generator=g) * 0.1).bfloat16()      # [N''=64, K'=N]
    dx = ops.gemm_dgrad(dY, W2)
    ref = dY.float() @ W2.float()
    assert float((dx.float() - ref).abs().max()) <= 2e-2 * float(ref.abs().max())
    G = (torch.randn(64, M, device="cuda", generator=g) * 0.1).bfloat16()       # [tokens=64, N'=M]
    A = torch.randn(64, N, device="cuda", generator=g).bfloat16()               # [tokens=64, K'=N]
    dw = ops.gemm_wgrad(G, A, out_dtype=torch.float32)
    ref = G.float().t() @ A.float()
    assert float((dw - ref).abs().max()) <= 1e-4 * float(ref.abs().max())


def test_mlp_shard_config_fused_epilogue_four_micro_batches():
    """One GPU's shard of the 12B-style MLP exactly as the configuration states it:
    8192 tokens x 2560 inputs, W shard [5120, 2560] with bias, GELU fused into the forward
    epilogue, backward through dGELU + dbias, dgrad and a weight gradient accumulated over
    4 micro-batches (seeds 0..3) - into a bf16 gradient (the parameter's dtype, as the
    reference accumulates: overlap_communication.py:38-47) and into an fp32 one.  Checked
    against the oracle on sampled rows / columns of every result, the full column sums of
    the bias gradient, and the additivity of dW over micro-batches."""
    from axonn_amd import ops

    M, N, K = 8192, 5120, 2560
    gw = torch.Generator(device="cuda").manual_seed(100)
    W = (torch.randn(N, K, generator=gw, device="cuda") * 0.02).bfloat16()
    b = (torch.randn(N, generator=gw, device="cuda") * 0.1)
    Wn, bn = np64(W), b.double().cpu().numpy()
    rs = np.random.default_rng(7)
    rows = np.sort(rs.choice(M, 40, replace=False))
    nrows = np.sort(rs.choice(N, 40, replace=False))
    ti, tn = torch.from_numpy(rows).cuda(), torch.from_numpy(nrows).cuda()

    dw16 = torch.zeros(N, K, dtype=torch.bfloat16, device="cuda")
    dw32 = torch.zeros(N, K, dtype=torch.float32, device="cuda")
    db = torch.zeros(N, dtype=torch.float32, device="cuda")
    dw_rows_ref = np.zeros((len(nrows), K))          # float64 sum over micro-batches
    dw16_rows_ref = None                             # the reference's bf16 accumulation order
    db_ref = np.zeros(N)
    singles = []
    for mb in range(4):
        g = torch.Generator(device="cuda").manual_seed(mb)
        X = torch.randn(M, K, generator=g, device="cuda").bfloat16()
        dY = (torch.randn(M, N, generator=g, device="cuda") * 1e-3).bfloat16()
        y, z = ops.gemm_fwd(X, W, bias=b, activation="gelu", save_z=True)
        dz, _ = ops.dgelu_dbias(dY, z, want_dbias=True, dbias_out=db, accumulate=True)
        dx = ops.gemm_dgrad(dz, W)
        ops.gemm_wgrad(dz, X, out=dw16, accumulate=True)
        ops.gemm_wgrad(dz, X, out=dw32, accumulate=True)
        # oracle on the sampled token rows
        yo, zo = ol.linear_forward(np64(X[ti]), Wn.reshape(-1), (N, K), bias=bn, activation="gelu")
        assert rel(np64(y[ti]), yo) < BF16_TOL and rel(np64(z[ti]), zo) < BF16_TOL
        # backward from the saved (rounded) pre-activation, as autograd would
        bw = ol.linear_backward(np64(X[ti]), Wn.reshape(-1), (N, K), np64(dY[ti]), z=np64(z[ti]),
                                activation="gelu", has_bias=True)
        assert rel(np64(dz[ti]), bw["dz"]) < BF16_TOL
        assert rel(np64(dx[ti]), np64(dz[ti]) @ Wn) < BF16_TOL
        # rows `nrows` of dW need every token: dZ columns from the kernel's (checked) dZ
        dzc = np64(dz[:, tn])
        part = dzc.T @ np64(X)
        dw_rows_ref += part
        dw16_rows_ref = ol.accumulate(dw16_rows_ref, part, "bf16")
        # bias gradient: column sums of dZ over all tokens, oracle dGELU on the full matrix
        dz_full = np64(dY) * ol.dgelu(np64(z))
        db_ref += dz_full.sum(0)
        if mb < 2:
            singles.append(ops.gemm_wgrad(dz, X, out_dtype=torch.float32))
            if mb == 1:   # additivity: accumulating equals adding the separate gradients
                two = ops.gemm_wgrad(dz, X, out=singles[0].clone(), accumulate=True)
                assert rel(np64(two), np64(singles[0]) + np64(singles[1])) < 1e-6
        del dz_full, dzc
    assert rel(dw32[tn].cpu().numpy(), dw_rows_ref) < 1e-4
    assert rel(np64(dw16[tn]), dw_rows_ref) < BF16_TOL
    # bf16 accumulation rounds after every micro-batch, exactly like the reference's add_
    assert rel(np64(dw16[tn]), dw16_rows_ref) < 4e-3
    assert rel(db.cpu().numpy(), db_ref) < 2e-3


@pytest.mark.parametrize("name", ["down", "mlp_shard", "skinny"])
def test_every_block_of_long_contraction_shapes(name):
    """Element-wise over every 16 x 16 block of the output (the unit a lane group owns) at
    the down projection's contraction of 14336 and at the shard and skinny shapes: the
    largest deviation inside each block stays within bf16 rounding of the fp32 product, so
    a single misplaced fragment cannot hide in a norm."""
    from axonn_amd import ops

    M, N, K = FULL[name]
    g = torch.Generator(device="cuda").manual_seed(9)
    X = torch.randn(M, K, generator=g, device="cuda").bfloat16()
    W = (torch.randn(N, K, generator=g, device="cuda") * 0.02).bfloat16()
    dY = (torch.randn(M, N, generator=g, device="cuda") * 1e-3).bfloat16()

    def blocks_ok(got, ref, tol):
        err = (got.float() - ref).abs()
        r, c = err.shape
        bmax = err.reshape(r // 16, 16, c // 16, 16).amax(dim=(1, 3))
        return float((bmax / ref.abs().max()).max()) <= tol

    assert blocks_ok(ops.gemm_fwd(X, W)[0], X.float() @ W.float().t(), 1e-2)
    assert blocks_ok(ops.gemm_dgrad(dY, W), dY.float() @ W.float(), 1e-2)
    assert blocks_ok(ops.gemm_wgrad(dY, X), dY.float().t() @ X.float(), 1e-2)
    assert blocks_ok(ops.gemm_wgrad(dY, X, out_dtype=torch.float32), dY.float().t() @ X.float(), 1e-4)


@pytest.mark.parametrize("M,N,K", [(8192, 5120, 2560),     # 320 + 200 tiles: one launch for both
                                   (4096, 2560, 2560),     # 160 + 100 tiles: one launch
                                   (4096, 4096, 4096),     # whole rounds: the two launches
                                   (512, 768, 256), (100, 72, 40)])   # small tiles, ragged
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_backward_in_one_call_equals_the_two_calls(M, N, K, dtype):
    """axn_gemm_bwd (dX and dW of one layer; one launch for both where the tile counts
    would leave CUs idle one after the other) against axn_gemm_dgrad and axn_gemm_wgrad:
    bit for bit, with a fresh and an accumulated dW, 16-bit and fp32; and against the oracle
    on sampled rows of the large shapes."""
    from axonn_amd import ops

    g = torch.Generator(device="cuda").manual_seed(M + N)
    X = torch.randn(M, K, device="cuda", generator=g).to(dtype)
    W = (torch.randn(N, K, device="cuda", generator=g) * 0.05).to(dtype)
    dY = (torch.randn(M, N, device="cuda", generator=g) * 0.01).to(dtype)
    dx, dw = ops.gemm_bwd(dY, W, X)
    assert torch.equal(dx, ops.gemm_dgrad(dY, W)) and torch.equal(dw, ops.gemm_wgrad(dY, X))
    for out_dtype in (dtype, torch.float32):
        acc = torch.randn(N, K, device="cuda", generator=g).to(out_dtype)
        twin = acc.clone()
        dx2, _ = ops.gemm_bwd(dY, W, X, out=acc, accumulate=True)
        ops.gemm_wgrad(dY, X, out=twin, accumulate=True)
        assert torch.equal(dx2, dx) and torch.equal(acc, twin)
    rows = torch.randint(0, M, (8,), generator=torch.Generator().manual_seed(1)).tolist()
    want = np64(dY[rows]) @ np64(W)
    assert rel(np64(dx[rows]), want) < BF16_TOL
    cols = torch.randint(0, N, (8,), generator=torch.Generator().manual_seed(2)).tolist()
    want = np64(dY[:, cols]).T @ np64(X)
    assert rel(np64(dw[cols]), want) < BF16_TOL
