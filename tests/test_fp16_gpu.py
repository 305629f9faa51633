"""Parity of the kernels on IEEE half operands (the reference's default mixed precision
is fp16 autocast under a loss scaler) with the CPU oracle, through the C ABI.

The half GEMMs are the bf16 kernels with another MFMA mnemonic and another conversion
in the epilogue, so the tests walk each kernel (256- and 128-wide tiles of the
one-wave-per-SIMD kernel, the register-staged kernel with and without edges), each
storage order and each epilogue once more.  Tolerance: fp16 keeps 11 significant bits,
so against the float64 oracle on the same fp16 inputs the final rounding leaves about
3e-4 normwise; the bar is 1e-3 (ten times tighter than the bf16 bar), 1e-5 with an fp32
result, and elementwise one fp16 rounding where stated.
"""

import numpy as np
import pytest
import torch

from oracle import linear as ol
from oracle import llama as om

pytestmark = pytest.mark.gpu

F16_TOL = 1e-3
F32_TOL = 1e-5


def rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


def np64(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def half_inputs(M, N, K, seed, x_std=1.0, w_std=0.02, g_std=1e-2):
    g = torch.Generator().manual_seed(seed)
    X = (torch.randn(M, K, generator=g) * x_std).half()
    W = (torch.randn(N, K, generator=g) * w_std).half()
    dY = (torch.randn(M, N, generator=g) * g_std).half()
    return X, W, dY


SHAPES = [
    (32, 64, 64), (100, 72, 40), (1, 8, 16), (257, 264, 72),      # register-staged, ragged
    (128, 128, 64), (256, 384, 192), (512, 1024, 1024),           # 128-wide tiles
    (4096, 3072, 128), (2304, 4096, 320),                         # 256-wide tiles
]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_three_half_gemms_match_oracle(M, N, K):
    from axonn_amd import ops

    X, W, dY = half_inputs(M, N, K, seed=M + 3 * N + 7 * K)
    yo, _ = ol.linear_forward(np64(X), np64(W).reshape(-1), (N, K))
    bw = ol.linear_backward(np64(X), np64(W).reshape(-1), (N, K), np64(dY))
    Xd, Wd, dYd = X.cuda(), W.cuda(), dY.cuda()
    y, _ = ops.gemm_fwd(Xd, Wd)
    dx = ops.gemm_dgrad(dYd, Wd)
    dw = ops.gemm_wgrad(dYd, Xd)
    dw32 = ops.gemm_wgrad(dYd, Xd, out_dtype=torch.float32)
    assert y.dtype == dx.dtype == dw.dtype == torch.float16 and dw32.dtype == torch.float32
    assert rel(np64(y), yo) < F16_TOL
    assert rel(np64(dx), bw["dx"]) < F16_TOL
    assert rel(np64(dw), bw["dw"].reshape(N, K)) < F16_TOL
    assert rel(np64(dw32), bw["dw"].reshape(N, K)) < F32_TOL
    # the conversion is to half, not to bfloat16 (2^-8): every output is within one fp16
    # rounding of the float64 value (relative 2^-11) plus the fp32 accumulation error
    excess = np.abs(np64(y) - yo) - 2.0 ** -11 * np.abs(yo)
    assert excess.max() < 1e-5 * np.abs(yo).max()


@pytest.mark.parametrize("M,N,K", [(300, 136, 96), (256, 256, 128), (2304, 4096, 128)])
@pytest.mark.parametrize("epilogue", ["bias", "bias_gelu", "gelu"])
def test_half_epilogues_and_their_backward(M, N, K, epilogue):
    from axonn_amd import ops

    X, W, dY = half_inputs(M, N, K, seed=11, w_std=0.2)
    b = torch.randn(N, generator=torch.Generator().manual_seed(5)) * 0.5
    bias = b if "bias" in epilogue else None
    act = "gelu" if "gelu" in epilogue else None
    yo, zo = ol.linear_forward(np64(X), np64(W).reshape(-1), (N, K),
                               bias=None if bias is None else b.double().numpy(), activation=act)
    y, z = ops.gemm_fwd(X.cuda(), W.cuda(), bias=None if bias is None else b.cuda(),
                        activation=act, save_z=True)
    assert y.dtype == torch.float16
    assert rel(np64(y), yo) < F16_TOL
    if act:
        assert z.dtype == torch.float16 and rel(np64(z), zo) < F16_TOL
        dz, db = ops.dgelu_dbias(dY.cuda(), z, want_dbias=bias is not None)
        want = np64(dY) * ol.dgelu(np64(z))
        assert dz.dtype == torch.float16 and rel(np64(dz), want) < F16_TOL
        if bias is not None:
            # the bias gradient sums what was stored (the rounded dZ), in fp32
            assert rel(np64(db), np64(dz).sum(axis=0)) < F32_TOL


def test_half_wgrad_accumulates():
    from axonn_amd import ops

    M, N, K = 512, 256, 384
    X, W, dY = half_inputs(M, N, K, seed=3)
    bw = ol.linear_backward(np64(X), np64(W).reshape(-1), (N, K), np64(dY))
    acc32 = torch.zeros(N, K, device="cuda")
    acc16 = torch.zeros(N, K, device="cuda", dtype=torch.float16)
    for _ in range(3):
        ops.gemm_wgrad(dY.cuda(), X.cuda(), out=acc32, accumulate=True)
        ops.gemm_wgrad(dY.cuda(), X.cuda(), out=acc16, accumulate=True)
    assert rel(np64(acc32), 3 * bw["dw"].reshape(N, K)) < F32_TOL
    assert rel(np64(acc16), 3 * bw["dw"].reshape(N, K)) < 2 * F16_TOL
    with pytest.raises(TypeError, match="dW must be"):
        ops.gemm_wgrad(dY.cuda(), X.cuda(), out_dtype=torch.bfloat16)
    with pytest.raises(TypeError, match="weight is"):
        ops.gemm_fwd(X.cuda(), W.cuda().bfloat16())


@pytest.mark.parametrize("use_autocast", [False, True])
def test_linear_layer_in_half_precision(use_autocast):
    """The reference's test of the layer (axonn/tests/test_intra_layer_fc.py:18-86) with the
    layer in fp16, or in fp32 under fp16 autocast as its mixed-precision mode runs it."""
    from axonn_amd.intra_layer import Linear

    torch.manual_seed(0)
    B, H, O = 96, 256, 384
    layer = Linear(H, O, fused_activation="gelu").cuda()
    with torch.no_grad():
        layer.bias.copy_(torch.randn(O) * 0.1)
    x = torch.randn(B, H, device="cuda")
    dy = torch.randn(B, O, device="cuda") * 0.1
    if use_autocast:
        xin = x.clone().requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.float16):
            y = layer(xin)
        # the fp32 bias promotes the 16-bit product to fp32, as the reference's `x + bias`
        # does under autocast (axonn/intra_layer/fully_connected.py:348)
        assert y.dtype == torch.float32
        y.backward(dy)
        w_used, x_used, dy_used = layer.weight.detach().half(), x.half(), dy.half()
    else:
        layer = layer.half()
        xin = x.half().requires_grad_(True)
        y = layer(xin)
        y.backward(dy.half())
        w_used, x_used, dy_used = layer.weight.detach(), x.half(), dy.half()
    yo, zo = ol.linear_forward(np64(x_used), np64(w_used), (O, H), bias=np64(layer.bias),
                               activation="gelu")
    bw = ol.linear_backward(np64(x_used), np64(w_used), (O, H), np64(dy_used), z=zo,
                            activation="gelu", has_bias=True)
    assert rel(np64(y), yo) < F16_TOL
    assert rel(np64(xin.grad), bw["dx"]) < 2 * F16_TOL   # dZ is rounded to fp16 before dgrad
    assert rel(np64(layer.weight.grad), bw["dw"]) < 2 * F16_TOL
    assert rel(np64(layer.bias.grad), bw["db"]) < 2 * F16_TOL
    assert layer.weight.grad.dtype == layer.weight.dtype


@pytest.mark.parametrize("M,N", [(37, 520), (256, 1024)])
def test_half_swiglu(M, N):
    from axonn_amd import ops

    g = torch.Generator(device="cuda").manual_seed(M)
    gate, up, dout = (torch.randn(M, N, device="cuda", generator=g).half() for _ in range(3))
    out = ops.swiglu_fwd(gate, up)
    want = om.swiglu_forward(np64(gate), np64(up))
    assert out.dtype == torch.float16
    assert np.allclose(np64(out), want, rtol=2.0 ** -11 + 5e-6, atol=1e-7)
    dg, du = ops.swiglu_bwd(dout, gate, up)
    wg, wu = om.swiglu_backward(np64(dout), np64(gate), np64(up))
    assert np.allclose(np64(dg), wg, rtol=2.0 ** -11 + 5e-6, atol=1e-7)
    assert np.allclose(np64(du), wu, rtol=2.0 ** -11 + 5e-6, atol=1e-7)
