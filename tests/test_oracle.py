"""Pins the CPU oracle (oracle/) before it is trusted as the checker.

The reference holds no golden vectors and no optimizer tests; its layer tests
assert equality with torch.nn.Linear and torch.nn.utils.clip_grad_norm_
(axonn/tests/test_intra_layer_fc.py:77, :167-199).  So every oracle function is
pinned here against (a) the torch library routine the reference delegates to,
(b) closed forms / invariants, (c) brute force on tiny inputs - chosen so that
a dropped term, a wrong sign, a transposed operand or a wrong rounding fails.
"""

import math

import numpy as np
import pytest
import torch

from oracle import linear as ol
from oracle import optim as oo
from oracle import torch_cpu as ot

REF_SHAPES = [(32, 64), (16, 128), (2, 256)]  # test_intra_layer_fc.py:18


# ------------------------------------------------------------------ bf16 -----
def test_bf16_rounding_matches_torch_bitwise():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(20000) * np.logspace(-30, 30, 20000)).astype(np.float32)
    special = np.array([0.0, -0.0, np.inf, -np.inf, 1.00390625, 1.01171875, 1.005859375,
                        3.39e38, 3.4e38, 1e-40, -1e-45, 65504.0], dtype=np.float32)
    x = np.concatenate([x, special])
    want = torch.from_numpy(x).bfloat16().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ol.bf16_bits(x), want)
    assert ol.bf16_bits(np.array([np.nan], dtype=np.float32))[0] == 0x7FC0


def test_bf16_ties_to_even_by_hand():
    # 1 + 2^-8 is exactly half way between 1.0 (even mantissa) and 1 + 2^-7
    assert ol.bf16_round(np.float32(1.0 + 2.0 ** -8)) == 1.0
    # 1 + 3 * 2^-8 is half way between 1 + 2^-7 (odd) and 1 + 2^-6 (even)
    assert ol.bf16_round(np.float32(1.0 + 3 * 2.0 ** -8)) == 1.0 + 2.0 ** -6
    assert np.isinf(ol.bf16_round(np.float32(3.4e38)))


# ------------------------------------------------------------------ GELU -----
def test_gelu_against_math_erf_and_torch():
    z = np.linspace(-6, 6, 241)
    brute = np.array([0.5 * v * (1.0 + math.erf(v / math.sqrt(2.0))) for v in z])
    assert np.allclose(ol.gelu(z), brute, rtol=0, atol=1e-15)
    t = torch.nn.functional.gelu(torch.from_numpy(z)).numpy()
    assert np.allclose(ol.gelu(z), t, rtol=1e-12, atol=1e-15)
    # special values: gelu(0) = 0, gelu(z) -> z for large z, -> 0 for very negative z
    assert ol.gelu(0.0) == 0.0
    assert abs(ol.gelu(10.0) - 10.0) < 1e-12 and abs(ol.gelu(-10.0)) < 1e-12


def test_dgelu_against_autograd_and_finite_differences():
    z = np.linspace(-5, 5, 101)
    zt = torch.from_numpy(z).requires_grad_(True)
    torch.nn.functional.gelu(zt).sum().backward()
    assert np.allclose(ol.dgelu(z), zt.grad.numpy(), rtol=1e-12, atol=1e-14)
    h = 1e-6
    fd = (ol.gelu(z + h) - ol.gelu(z - h)) / (2 * h)
    assert np.allclose(ol.dgelu(z), fd, atol=1e-8)
    assert ol.dgelu(0.0) == 0.5


# ----------------------------------------------------------------- layer -----
@pytest.mark.parametrize("B,H", REF_SHAPES)
@pytest.mark.parametrize("bias", [False, True])
def test_linear_matches_torch_nn_linear(B, H, bias):
    """The reference's own assertion (test_intra_layer_fc.py:55-77, :157-199)."""
    torch.manual_seed(42)
    X = (torch.randn(B, H) * 0.01).double().requires_grad_(True)
    dY = (torch.randn(B, H) * 0.01).double()
    layer = torch.nn.Linear(H, H, bias=bias).double()
    Y = layer(X)
    Y.backward(dY)
    w_flat = ol.extract_local_params_from_full_params(layer.weight.detach().numpy())
    assert w_flat.ndim == 1 and w_flat.size == H * H
    b = layer.bias.detach().numpy() if bias else None
    y, _ = ol.linear_forward(X.detach().numpy(), w_flat, (H, H), bias=b)
    bw = ol.linear_backward(X.detach().numpy(), w_flat, (H, H), dY.numpy(), has_bias=bias)
    assert np.allclose(y, Y.detach().numpy(), rtol=1e-12, atol=1e-15)
    assert np.allclose(bw["dx"], X.grad.numpy(), rtol=1e-12, atol=1e-15)
    assert bw["dw"].ndim == 1  # the reference returns the weight gradient flattened
    assert np.allclose(bw["dw"].reshape(H, H), layer.weight.grad.numpy(), rtol=1e-12, atol=1e-15)
    if bias:
        assert np.allclose(bw["db"], layer.bias.grad.numpy(), rtol=1e-12, atol=1e-15)


def test_linear_brute_force_non_square():
    """Triple loops on a tiny non-square case: catches a transposed operand."""
    rng = np.random.default_rng(1)
    M, K, N = 3, 5, 4
    x, w, g = rng.standard_normal((M, K)), rng.standard_normal((N, K)), rng.standard_normal((M, N))
    y = np.zeros((M, N))
    dx = np.zeros((M, K))
    dw = np.zeros((N, K))
    for i in range(M):
        for j in range(N):
            for k in range(K):
                y[i, j] += x[i, k] * w[j, k]
                dx[i, k] += g[i, j] * w[j, k]
                dw[j, k] += g[i, j] * x[i, k]
    yo, _ = ol.linear_forward(x, w.reshape(-1), (N, K))
    bw = ol.linear_backward(x, w.reshape(-1), (N, K), g)
    assert np.allclose(yo, y) and np.allclose(bw["dx"], dx)
    assert np.allclose(bw["dw"].reshape(N, K), dw)


def test_linear_3d_input_and_skip_bias_add():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((2, 3, 8))
    w = rng.standard_normal((6, 8))
    b = rng.standard_normal(6)
    y, _ = ol.linear_forward(x, w.reshape(-1), (6, 8), bias=b)
    want = torch.nn.functional.linear(torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(b))
    assert y.shape == (2, 3, 6) and np.allclose(y, want.numpy())
    (y2, b2), _ = ol.linear_forward(x, w.reshape(-1), (6, 8), bias=b, skip_bias_add=True)
    assert np.allclose(y2 + b2, y)


def test_fused_gelu_layer_against_autograd():
    torch.manual_seed(5)
    X = torch.randn(7, 12).double().requires_grad_(True)
    lin = torch.nn.Linear(12, 9).double()
    dY = torch.randn(7, 9).double()
    Z = lin(X)
    Y = torch.nn.functional.gelu(Z)
    Y.backward(dY)
    w = lin.weight.detach().numpy().reshape(-1)
    y, z = ol.linear_forward(X.detach().numpy(), w, (9, 12), bias=lin.bias.detach().numpy(),
                             activation="gelu")
    bw = ol.linear_backward(X.detach().numpy(), w, (9, 12), dY.numpy(), z=z, activation="gelu",
                            has_bias=True)
    assert np.allclose(z, Z.detach().numpy()) and np.allclose(y, Y.detach().numpy())
    assert np.allclose(bw["dx"], X.grad.numpy())
    assert np.allclose(bw["dw"].reshape(9, 12), lin.weight.grad.numpy())
    assert np.allclose(bw["db"], lin.bias.grad.numpy())


def test_linearity_and_microbatch_additivity():
    rng = np.random.default_rng(3)
    x1, x2 = rng.standard_normal((4, 6)), rng.standard_normal((4, 6))
    g1, g2 = rng.standard_normal((4, 5)), rng.standard_normal((4, 5))
    w = rng.standard_normal(30)
    y1, _ = ol.linear_forward(x1, w, (5, 6))
    y2, _ = ol.linear_forward(x2, w, (5, 6))
    y12, _ = ol.linear_forward(2 * x1 - 3 * x2, w, (5, 6))
    assert np.allclose(y12, 2 * y1 - 3 * y2)
    # dW over a concatenated batch is the sum of the per-micro-batch dW
    d1 = ol.linear_backward(x1, w, (5, 6), g1)["dw"]
    d2 = ol.linear_backward(x2, w, (5, 6), g2)["dw"]
    dcat = ol.linear_backward(np.concatenate([x1, x2]), w, (5, 6), np.concatenate([g1, g2]))["dw"]
    assert np.allclose(dcat, d1 + d2)


def test_accumulate_rounds_in_param_dtype():
    """overlap_communication.py:38-47: first assignment, then add_ in the
    parameter's dtype."""
    g1 = np.array([1.0, 1.0 + 2.0 ** -9])
    acc = ol.accumulate(None, g1, "bf16")
    want = torch.tensor(g1).to(torch.bfloat16)
    assert np.array_equal(acc, want.double().numpy())
    g2 = np.array([2.0 ** -9, 3.0])
    acc2 = ol.accumulate(acc, g2, "bf16")
    want2 = want.clone().add_(torch.tensor(g2).to(torch.bfloat16))
    assert np.array_equal(acc2, want2.double().numpy())


def test_default_init_bound_is_kaiming_uniform_a_sqrt5():
    torch.manual_seed(0)
    K = 1024
    w = torch.nn.init.kaiming_uniform_(torch.empty(4096, K), a=math.sqrt(5))
    b = ol.default_init_bound(K)
    assert b == 1.0 / math.sqrt(K)
    assert float(w.abs().max()) <= b and float(w.abs().max()) > 0.999 * b
    assert abs(float(w.var()) - b * b / 3.0) < 0.02 * b * b / 3.0


# ----------------------------------------------------------- overflow check --
def test_check_nan_brute_force():
    for dt in ("f32", "f16", "bf16"):
        assert not oo.check_nan(np.array([1.0, -2.0, 3.0]), dt)
        assert oo.check_nan(np.array([1.0, np.inf]), dt)
        assert oo.check_nan(np.array([-np.inf, 1.0]), dt)
        assert oo.check_nan(np.array([np.inf, -np.inf]), dt)  # inf - inf = nan
        assert oo.check_nan(np.array([0.0, np.nan]), dt)
    # the fp16 corner: finite elements whose sum leaves the fp16 range
    x = np.full(4, 30000.0)
    assert not oo.any_nonfinite(x)
    assert oo.check_nan(x, "f16") and not oo.check_nan(x, "f32")
    # and it is what torch's sum does
    assert ot.check_nan(torch.full((4,), 30000.0, dtype=torch.float16))
    assert not ot.check_nan(torch.full((2,), 30000.0, dtype=torch.float16))
    assert not oo.check_nan(np.full(2, 30000.0), "f16")


def test_check_nan_equals_elementwise_when_sum_in_range():
    rng = np.random.default_rng(4)
    for trial in range(50):
        x = rng.standard_normal(64) * 100
        if trial % 3 == 0:
            x[rng.integers(64)] = rng.choice([np.inf, -np.inf, np.nan])
        assert oo.check_nan(x, "bf16") == oo.any_nonfinite(x)
        t = torch.tensor(x, dtype=torch.bfloat16)
        assert ot.check_nan(t) == oo.check_nan(t.double().numpy(), "bf16")


def test_unscale_is_exact_for_power_of_two_scales():
    rng = np.random.default_rng(5)
    g = ol.round_to(rng.standard_normal(100) * 40.0, "f16")
    overflow, (u,) = oo.unscale_gradients([g], "f16", 2.0 ** 16)
    assert not overflow
    t = torch.tensor(g, dtype=torch.float16)
    t.div_(2.0 ** 16)
    assert np.array_equal(u, t.double().numpy())
    # unscaling happens even when an overflow is found (inter_layer.py:455-458)
    g[3] = np.inf
    overflow, (u,) = oo.unscale_gradients([g], "f16", 2.0 ** 16)
    assert overflow and np.isinf(u[3]) and u[0] == g[0] / 2.0 ** 16


# ------------------------------------------------------------- loss scaler ---
def test_loss_scaler_state_machine_table():
    s = oo.LossScaler()
    assert (s.loss_scale, s.max_scale, s.min_scale, s.scaling_window) == (65536.0, 2.0 ** 24, 1024.0, 200)
    assert oo.sync_scale(s, True) is True and s.loss_scale == 32768.0 and s.no_overflow_iters == 0
    for i in range(199):
        assert oo.sync_scale(s, False) is False
        assert s.loss_scale == 32768.0 and s.no_overflow_iters == i + 1
    assert oo.sync_scale(s, False) is False  # the 200th clean step doubles
    assert s.loss_scale == 65536.0 and s.no_overflow_iters == 0
    s = oo.LossScaler(loss_scale=1024.0)
    oo.sync_scale(s, True)
    assert s.loss_scale == 1024.0  # floor
    s = oo.LossScaler(loss_scale=2.0 ** 24, no_overflow_iters=199)
    oo.sync_scale(s, False)
    assert s.loss_scale == 2.0 ** 24  # cap
    s = oo.LossScaler(no_overflow_iters=150)
    oo.sync_scale(s, True)
    assert s.no_overflow_iters == 0  # overflow resets the window


# ------------------------------------------------------------ norm / clip ----
@pytest.mark.parametrize("max_norm", [1e-3, 1.0, 100.0])
def test_clip_matches_torch_clip_grad_norm(max_norm):
    torch.manual_seed(6)
    params = [torch.nn.Parameter(torch.zeros(n)) for n in (5, 17, 64)]
    for p in params:
        p.grad = torch.randn_like(p) * 0.3
    grads = [p.grad.clone().double().numpy() for p in params]
    total = torch.nn.utils.clip_grad_norm_(params, max_norm, foreach=False)
    t, clipped = oo.clip_grad_norm_(grads, max_norm, "f32")
    assert abs(t - float(total)) <= 1e-6 * float(total)
    for c, p in zip(clipped, params):
        assert np.allclose(c, p.grad.double().numpy(), rtol=2e-7, atol=0)
    # closed form
    flat = np.concatenate(grads)
    assert abs(t - math.sqrt(float(np.sum(flat ** 2)))) < 1e-6 * t
    assert oo.clip_coef(2.0, 1.0) == 1.0 / (2.0 + 1e-6) and oo.clip_coef(0.5, 1.0) == 1.0


def test_norm_of_norms_equals_flat_norm():
    rng = np.random.default_rng(7)
    ts = [rng.standard_normal(n) for n in (3, 40, 7)]
    assert abs(oo.get_total_norm(ts) - np.linalg.norm(np.concatenate(ts))) < 1e-12
    assert oo.get_total_norm([]) == 0.0


@pytest.mark.parametrize("p", [float("inf"), float("-inf")])
def test_total_norm_of_infinite_order_matches_torch(p):
    """get_total_norm with p = +inf / -inf against the reference's own expression, the
    torch.norm of the stacked per-tensor torch.norms (gradient_normalization.py:22-25),
    and against the closed form (largest / smallest magnitude); a NaN element gives NaN."""
    rng = np.random.default_rng(11)
    ts = [rng.standard_normal(n) + 0.01 for n in (3, 400, 7, 1)]
    tt = [torch.from_numpy(t) for t in ts]
    want = torch.norm(torch.stack([torch.norm(t, p) for t in tt]), p)
    assert oo.get_total_norm(ts, norm_type=p) == float(want)
    flat = np.abs(np.concatenate(ts))
    assert oo.get_total_norm(ts, norm_type=p) == (flat.max() if p > 0 else flat.min())
    ts[1][17] = np.nan
    assert np.isnan(oo.get_total_norm(ts, norm_type=p))
    assert bool(torch.isnan(torch.norm(torch.from_numpy(ts[1]), p)))


@pytest.mark.parametrize("p", [1.0, 3.0, 0.5, 4.0, 1.5, -1.0, 0.0])
def test_clip_of_any_finite_order_matches_torch(p):
    """The reference hands norm_type to torch.norm per gradient and once more over the
    stacked results (gradient_normalization.py:18-34); torch.nn.utils.clip_grad_norm_
    computes the same quantity, and for p != 0 it equals the p-norm of all elements."""
    torch.manual_seed(60)
    params = [torch.nn.Parameter(torch.zeros(n)) for n in (5, 17, 64)]
    for q in params:
        q.grad = torch.randn_like(q) * 0.3
    params[1].grad[3] = 0.0
    grads = [q.grad.clone().double().numpy() for q in params]
    want = torch.norm(torch.stack([torch.norm(q.grad.detach(), p) for q in params]), p)   # :21-24
    total = torch.nn.utils.clip_grad_norm_(params, 0.05, norm_type=p, foreach=False)
    t, clipped = oo.clip_grad_norm_(grads, 0.05, "f32", norm_type=p)
    assert abs(t - float(want)) <= 2e-6 * abs(float(want))
    assert abs(t - float(total)) <= 2e-6 * abs(float(total))
    for c, q in zip(clipped, params):
        assert np.allclose(c, q.grad.double().numpy(), rtol=1e-6, atol=0)
    flat = np.abs(np.concatenate(grads))
    if p == 0.0:
        assert t == 3.0                       # three gradients with a non-zero element
    elif p > 0:
        assert abs(t - float(np.sum(flat ** p) ** (1.0 / p))) <= 1e-6 * t
    else:
        assert t == 0.0                       # a zero element: |0|^p = inf, inf^(1/p) = 0


# ------------------------------------------------------------------ Adam -----
@pytest.mark.parametrize("wd", [0.0, 0.01])
def test_adam_matches_torch_optim_adam_over_steps(wd):
    torch.manual_seed(8)
    p = torch.nn.Parameter(torch.randn(257) * 0.02)
    opt = torch.optim.Adam([p], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=wd,
                           foreach=False)
    po = p.detach().numpy().copy()
    mo = np.zeros_like(po)
    vo = np.zeros_like(po)
    for step in range(1, 6):
        g = torch.randn(257) * 1e-3
        p.grad = g.clone()
        opt.step()
        po, mo, vo = oo.adam_update(po, g.numpy(), mo, vo, step, weight_decay=wd)
        st = opt.state[p]
        # same float32 operation order as torch: agreement to one ulp of p
        # (torch's CPU kernels may fuse a multiply-add where numpy does not)
        ref = p.detach().numpy()
        assert np.max(np.abs(po - ref)) <= 2.0 ** -23 * np.max(np.abs(ref))
        assert np.max(np.abs(po - ref)) / np.max(np.abs(ref)) <= 1e-6
        assert np.allclose(mo, st["exp_avg"].numpy(), rtol=3e-7, atol=1e-10)
        assert np.allclose(vo, st["exp_avg_sq"].numpy(), rtol=3e-7, atol=1e-15)


def test_adam_step_one_closed_form_and_f64():
    rng = np.random.default_rng(9)
    p = (rng.standard_normal(100) * 0.02).astype(np.float32)
    g = (rng.standard_normal(100) * 1e-3).astype(np.float32)
    z = np.zeros(100, dtype=np.float32)
    p1, m1, v1 = oo.adam_update(p, g, z, z, 1)
    # step 1: m = (1-b1) g, v = (1-b2) g^2, update = -lr * g / (|g| + eps)
    assert np.allclose(m1, 0.1 * g, rtol=1e-6)
    assert np.allclose(v1, 0.001 * g * g, rtol=1e-5)
    want = p.astype(np.float64) - 1e-3 * g.astype(np.float64) / (np.abs(g.astype(np.float64)) + 1e-8)
    assert np.allclose(p1, want, rtol=1e-6)
    p64, m64, v64 = oo.adam_update_f64(p, g, z, z, 1)
    assert np.allclose(p1, p64, rtol=1e-6) and np.allclose(m1, m64, rtol=1e-6)
    # sign: a positive gradient decreases the parameter
    assert np.all(np.sign(p1.astype(np.float64) - p) == -np.sign(g))


def test_bias_corrections_are_python_doubles():
    bc1, bc2 = oo.bias_corrections(3, 0.9, 0.999)
    assert bc1 == 1.0 - 0.9 ** 3 and bc2 == 1.0 - 0.999 ** 3


def test_mixed_precision_step_matches_torch_pipeline():
    torch.manual_seed(10)
    sizes = [33, 7, 129]
    scale = 65536.0
    p32 = [torch.randn(n) * 0.02 for n in sizes]
    m = [torch.zeros(n) for n in sizes]
    v = [torch.zeros(n) for n in sizes]
    g = [(torch.randn(n) * 1e-3 * scale).bfloat16() for n in sizes]
    res = oo.mixed_precision_step(
        [t.float().numpy() for t in g], [t.numpy().copy() for t in p32],
        [t.numpy().copy() for t in m], [t.numpy().copy() for t in v],
        step=1, loss_scale=scale, max_norm=0.01)
    tp = [t.clone() for t in p32]
    tm = [t.clone() for t in m]
    tv = [t.clone() for t in v]
    tres = ot.optimizer_step(g, tp, tm, tv, 1, scale, max_norm=0.01)
    assert res["overflow"] is False and tres["overflow"] is False
    assert abs(res["total_norm"] - tres["total_norm"]) < 1e-6 * tres["total_norm"]
    assert res["clip_coef"] < 1.0
    for a, b in zip(res["p"], tp):
        assert np.allclose(a, b.numpy(), rtol=1e-6, atol=0)
    for a, b in zip(res["p_low"], tres["p_low"]):
        assert np.array_equal(a, b.float().numpy())
    # overflow: nothing changes
    g[1][3] = float("inf")
    res = oo.mixed_precision_step(
        [t.float().numpy() for t in g], [t.numpy() for t in p32], [t.numpy() for t in m],
        [t.numpy() for t in v], step=1, loss_scale=scale, max_norm=0.01)
    assert res["overflow"] is True and res["p_low"] is None
    for a, b in zip(res["p"], p32):
        assert np.array_equal(a, b.numpy())


def test_coalesce_layout():
    a, b, c = np.arange(3.0), np.arange(4.0).reshape(2, 2) + 10, np.array([99.0])
    flat, views = oo.coalesce([a, b, c])
    assert np.array_equal(flat, [0, 1, 2, 10, 11, 12, 13, 99])
    views[1][1, 0] = -1.0  # views alias the flat buffer
    assert flat[5] == -1.0
    t = torch._utils._flatten_dense_tensors([torch.tensor(a), torch.tensor(b) * 0 + torch.tensor(b), torch.tensor(c)])
    assert t.numel() == flat.size
    assert oo.group_offsets([3, 4, 1]) == [0, 3, 7, 8]


def test_torch_cpu_mlp_step_matches_numpy_oracle():
    """The 2-layer MLP configuration, small: the two independent restatements
    agree on loss gradient and on the Adam-updated weights."""
    torch.manual_seed(0)
    B, D, Hd = 8, 16, 32
    w1 = torch.nn.init.kaiming_uniform_(torch.empty(Hd, D), a=math.sqrt(5))
    w2 = torch.nn.init.kaiming_uniform_(torch.empty(D, Hd), a=math.sqrt(5))
    b1, b2 = torch.zeros(Hd), torch.zeros(D)
    x, tgt = torch.randn(B, D), torch.randn(B, D)
    res = ot.mlp_step(x, tgt, w1, b1, w2, b2)
    # numpy oracle, float64
    h, z1 = ol.linear_forward(x.numpy(), w1.numpy().reshape(-1), (Hd, D), bias=b1.numpy(),
                              activation="gelu")
    y, _ = ol.linear_forward(h, w2.numpy().reshape(-1), (D, Hd), bias=b2.numpy())
    dy = 2.0 * (y - tgt.numpy()) / y.size
    bw2 = ol.linear_backward(h, w2.numpy().reshape(-1), (D, Hd), dy, has_bias=True)
    bw1 = ol.linear_backward(x.numpy(), w1.numpy().reshape(-1), (Hd, D), bw2["dx"], z=z1,
                             activation="gelu", has_bias=True)
    assert np.allclose(bw1["dw"].reshape(Hd, D), res["grads"][0].numpy(), rtol=1e-4, atol=1e-7)
    assert np.allclose(bw1["db"], res["grads"][1].numpy(), rtol=1e-4, atol=1e-7)
    assert np.allclose(bw2["dw"].reshape(D, Hd), res["grads"][2].numpy(), rtol=1e-4, atol=1e-7)
    p1, _, _ = oo.adam_update(w1.numpy(), res["grads"][0].numpy(), 0 * w1.numpy(), 0 * w1.numpy(), 1)
    assert np.allclose(p1, res["params"][0].numpy(), rtol=1e-6, atol=0)


# ---- Llama MLP block (oracle/llama.py) ------------------------------------------
def test_silu_swiglu_pinned_by_torch_closed_forms_and_finite_differences():
    from oracle import llama as om

    x = np.linspace(-30.0, 30.0, 2001)
    t = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    y = torch.nn.functional.silu(t)
    y.sum().backward()
    assert np.allclose(om.silu(x), y.detach().numpy(), rtol=1e-13, atol=1e-300)
    assert np.allclose(om.dsilu(x), t.grad.numpy(), rtol=1e-12, atol=1e-15)
    # closed forms: silu(0) = 0, silu'(0) = 1/2, silu(x) - silu(-x) = x, silu -> x / 0 in the tails
    assert om.silu(np.array([0.0]))[0] == 0.0 and om.dsilu(np.array([0.0]))[0] == 0.5
    assert np.allclose(om.silu(x) - om.silu(-x), x, atol=1e-13)
    assert abs(om.silu(np.array([40.0]))[0] - 40.0) < 1e-12 and abs(om.silu(np.array([-745.0]))[0]) < 1e-300
    h = 1e-6
    fd = (om.silu(x + h) - om.silu(x - h)) / (2 * h)
    assert np.allclose(om.dsilu(x), fd, atol=1e-8)
    # swiglu backward against autograd, and a dropped-factor check: dgate must depend on up
    g = torch.randn(7, 16, dtype=torch.float64, requires_grad=True)
    u = torch.randn(7, 16, dtype=torch.float64, requires_grad=True)
    d = torch.randn(7, 16, dtype=torch.float64)
    (torch.nn.functional.silu(g) * u).backward(d)
    dg, du = om.swiglu_backward(d.numpy(), g.detach().numpy(), u.detach().numpy())
    assert np.allclose(dg, g.grad.numpy(), rtol=1e-12) and np.allclose(du, u.grad.numpy(), rtol=1e-12)
    assert not np.allclose(dg, om.swiglu_backward(d.numpy(), g.detach().numpy(), 2 * u.detach().numpy())[0])


def test_llama_mlp_oracle_matches_hugging_face_block_with_autograd():
    """The unpatched Hugging Face LlamaMLP in float64 on the CPU is the library
    routine the oracle's block must equal, forward and backward."""
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaMLP
    from oracle import llama as om

    torch.manual_seed(3)
    H, I, M = 24, 56, 10
    cfg = LlamaConfig(hidden_size=H, intermediate_size=I, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=32)
    mlp = LlamaMLP(cfg).double()
    x = torch.randn(M, H, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(M, H, dtype=torch.float64)
    y = mlp(x)
    y.backward(dy)
    wg, wu, wd = (p.detach().numpy().reshape(-1) for p in
                  (mlp.gate_proj.weight, mlp.up_proj.weight, mlp.down_proj.weight))
    fwd = om.llama_mlp_forward(x.detach().numpy(), wg, wu, wd, H, I)
    bwd = om.llama_mlp_backward(x.detach().numpy(), wg, wu, wd, H, I, dy.numpy(), fwd)
    assert np.allclose(fwd["out"], y.detach().numpy(), rtol=1e-12, atol=1e-14)
    assert np.allclose(bwd["dx"], x.grad.numpy(), rtol=1e-11, atol=1e-14)
    for key, lin in (("dw_gate", mlp.gate_proj), ("dw_up", mlp.up_proj), ("dw_down", mlp.down_proj)):
        assert np.allclose(bwd[key].reshape(lin.weight.shape), lin.weight.grad.numpy(), rtol=1e-11, atol=1e-14)


# ------------------------------------------------------------------ embedding
@pytest.mark.parametrize("padding_idx", [None, 3])
@pytest.mark.parametrize("scale", [False, True])
def test_embedding_oracle_matches_torch_cpu_embedding_and_autograd(padding_idx, scale):
    """torch's CPU F.embedding and its autograd are the library routines the reference
    calls (axonn/intra_layer/embedding.py:164-172); ids repeat heavily (V = 11, T = 60)."""
    from oracle import embedding as oe

    torch.manual_seed(5)
    V, H, T = 11, 8, 60
    W = torch.randn(V, H, requires_grad=True)
    ids = torch.randint(0, V, (4, 15))
    dY = torch.randn(4, 15, H)
    out = torch.nn.functional.embedding(ids, W, padding_idx=padding_idx, scale_grad_by_freq=scale)
    out.backward(dY)
    assert np.array_equal(oe.embedding_forward(ids.numpy(), W.detach().numpy()), out.detach().numpy())
    dW = oe.embedding_backward(ids.numpy(), dY.numpy(), V, padding_idx, scale)
    assert dW.dtype == np.float32
    # torch sums in another order: a few fp32 roundings of sums of up to 12 terms
    assert np.allclose(dW, W.grad.numpy(), rtol=2e-6, atol=2e-6)
    d64 = oe.embedding_backward_f64(ids.numpy(), dY.numpy(), V, padding_idx, scale)
    assert np.allclose(dW, d64, rtol=2e-6, atol=2e-6)
    assert np.allclose(W.grad.numpy(), d64, rtol=2e-6, atol=2e-6)
    if padding_idx is not None:
        assert not dW[padding_idx].any() and (ids == padding_idx).any()


def test_embedding_oracle_closed_forms():
    from oracle import embedding as oe

    rng = np.random.default_rng(0)
    V, H = 9, 4
    W = rng.standard_normal((V, H)).astype(np.float32)
    perm = rng.permutation(V)
    dY = rng.standard_normal((V, H)).astype(np.float32)
    # a permutation of the rows: the gradient is dY put back in place, exactly
    dW = oe.embedding_backward(perm, dY, V)
    assert np.array_equal(dW[perm], dY)
    assert np.array_equal(oe.embedding_forward(perm, W), W[perm])
    # one id repeated: the sequential fp32 sum, term by term
    rep = np.full(7, 2)
    dY7 = rng.standard_normal((7, H)).astype(np.float32)
    acc = np.zeros(H, np.float32)
    for t in range(7):
        acc = acc + dY7[t]
    dW = oe.embedding_backward(rep, dY7, V)
    assert np.array_equal(dW[2], acc) and not dW[[0, 1, 3, 4, 5, 6, 7, 8]].any()
    # scale by frequency: the mean of the rows; the order of summation shows in the last bit only
    dWs = oe.embedding_backward(rep, dY7, V, scale_grad_by_freq=True)
    assert np.allclose(dWs[2], dY7.astype(np.float64).mean(axis=0), rtol=1e-6, atol=1e-7)
    # ids outside the table: zeros forward, skipped backward
    bad = np.array([1, -1, V, 4])
    out = oe.embedding_forward(bad, W)
    assert np.array_equal(out[0], W[1]) and not out[1].any() and not out[2].any()
    dWb = oe.embedding_backward(bad, dY[:4], V)
    assert np.array_equal(dWb[1], dY[0]) and np.array_equal(dWb[4], dY[3]) and dWb.sum() == (dY[0] + dY[3]).sum()
    # accumulate: touched rows get sum + old, the others keep old
    old = rng.standard_normal((V, H)).astype(np.float32)
    acc2 = oe.embedding_backward(np.array([5, 5]), dY[:2], V, accumulate_into=old)
    assert np.array_equal(acc2[5], (dY[0] + dY[1]) + old[5])
    mask = np.ones(V, bool)
    mask[5] = False
    assert np.array_equal(acc2[mask], old[mask])


@pytest.mark.parametrize("norm_type", [1.0, 2.0, 3.0])
def test_embedding_renorm_oracle_matches_torch(norm_type):
    from oracle import embedding as oe

    torch.manual_seed(11)
    V, H = 13, 16
    W = torch.randn(V, H, dtype=torch.float64)
    W[4] *= 0.01  # a row already inside the ball stays as it is
    ids = torch.tensor([[1, 4, 4, 7], [7, 7, 12, 1]])
    ref = W.clone()
    torch.embedding_renorm_(ref, ids, 1.5, norm_type)
    got = oe.embedding_renorm(W.numpy(), ids.numpy(), 1.5, norm_type)
    assert np.allclose(got, ref.numpy(), rtol=1e-12, atol=1e-14)
    untouched = [0, 2, 3, 5, 6, 8, 9, 10, 11]
    assert np.array_equal(got[untouched], W.numpy()[untouched]) and np.array_equal(got[4], W.numpy()[4])
    norms = np.linalg.norm(got[[1, 7, 12]], ord=norm_type, axis=1)
    assert np.all(norms <= 1.5) and np.all(norms > 1.5 * (1 - 1e-6))
