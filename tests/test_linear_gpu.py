"""The Linear module against torch.nn.Linear, as the reference's own tests do
(axonn/tests/test_intra_layer_fc.py: same shapes, seed, 0.01 input scaling, copy
of the weights through load_state_dict, clip norm 1e-3), single process."""

import numpy as np
import pytest
import torch

from oracle import linear as ol

pytestmark = pytest.mark.gpu

REF_SHAPES = [(32, 64), (16, 128), (2, 256)]


def rel(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))


def make_pair(H_in, H_out, bias, dtype, **kw):
    from axonn_amd.intra_layer import Linear

    torch.manual_seed(42)
    seq = torch.nn.Linear(H_in, H_out, bias=bias).cuda()
    layer = Linear(in_features=H_in, out_features=H_out, bias=bias, **kw).cuda()
    layer.load_state_dict(seq.state_dict())      # full checkpoint
    layer.load_state_dict(layer.state_dict())    # sharded checkpoint
    return layer.to(dtype), seq.to(dtype)


@pytest.mark.parametrize("B,H", REF_SHAPES)
@pytest.mark.parametrize("expert_mode", [False, True])
@pytest.mark.parametrize("bias", [False, True])
def test_fw_pass_fp32(B, H, expert_mode, bias):
    from axonn_amd import axonn as ax

    ax.init(G_data=1, G_inter=1, G_intra_r=1, G_intra_c=1, G_intra_d=1)
    layer, seq = make_pair(H, H, bias, torch.float32, expert_mode=expert_mode)
    torch.manual_seed(42)
    X = torch.randn(B, H).cuda() * 0.01
    with torch.no_grad():
        Yp, Ys = layer(X), seq(X)
    # the reference asserts torch.allclose defaults against the same library on
    # the same device; two different fp32 summation orders agree to ~1e-6
    assert torch.allclose(Ys, Yp, rtol=1e-5, atol=1e-7), "FW Pass - output does not match"


@pytest.mark.parametrize("B,H", REF_SHAPES)
@pytest.mark.parametrize("comm_opt_level", [0, 4])
@pytest.mark.parametrize("clip_grad_norm", [-1, 1e-3])
@pytest.mark.parametrize("bias", [False, True])
def test_bw_pass_fp32(B, H, comm_opt_level, clip_grad_norm, bias):
    from axonn_amd.intra_layer import clip_grad_norm_, optimize_communication, sync_gradients

    layer, seq = make_pair(H, H, bias, torch.float32)
    torch.manual_seed(42)
    X = torch.randn(B, H).cuda() * 0.01
    Y_grad = torch.randn(B, H).cuda() * 0.01
    X_local = X.detach().clone().requires_grad_(True)
    with optimize_communication(
        overlap_all_reduce=comm_opt_level >= 1, overlap_reduce_scatter=comm_opt_level >= 2,
        cache_weights=comm_opt_level >= 3, overlap_all_gather=comm_opt_level == 4,
        model_object_for_overlapping_allgathers=layer,
    ):
        Y_local = layer(X_local)
        Y_local.backward(Y_grad)
    sync_gradients(layer)
    Xs = X.detach().clone().requires_grad_(True)
    seq(Xs).backward(Y_grad)
    if clip_grad_norm > 0:
        n1 = clip_grad_norm_(layer.parameters(), max_norm=clip_grad_norm)
        n2 = torch.nn.utils.clip_grad_norm_(seq.parameters(), max_norm=clip_grad_norm)
        assert abs(float(n1) - float(n2)) <= 1e-5 * float(n2)
    assert torch.allclose(X_local.grad, Xs.grad, rtol=1e-5, atol=1e-8), "BW Pass - input grads"
    wg = layer.weight.grad.reshape(layer.local_out_features, layer.local_in_features)
    assert rel(wg, seq.weight.grad) < 1e-5, "BW Pass - weight grads"
    if bias:
        assert rel(layer.bias.grad, seq.bias.grad) < 1e-5, "BW Pass - bias grads"


@pytest.mark.parametrize("B,Hin,Hout", [(64, 128, 256), (50, 72, 136)])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("act", [None, "gelu"])
def test_bf16_layer_matches_oracle(B, Hin, Hout, bias, act):
    layer, seq = make_pair(Hin, Hout, bias, torch.bfloat16, fused_activation=act)
    if bias:
        with torch.no_grad():
            layer.bias.copy_(torch.randn(Hout) * 0.1)
    torch.manual_seed(1)
    X = torch.randn(3, B, Hin).bfloat16().cuda().requires_grad_(True)   # 3-D input
    dY = torch.randn(3, B, Hout).bfloat16().cuda()
    Y = layer(X)
    assert Y.shape == (3, B, Hout) and Y.dtype == torch.bfloat16
    Y.backward(dY)
    n64 = lambda t: t.detach().float().cpu().numpy().astype(np.float64)
    b = n64(layer.bias) if bias else None
    yo, zo = ol.linear_forward(n64(X), n64(layer.weight), (Hout, Hin), bias=b, activation=act)
    bw = ol.linear_backward(n64(X), n64(layer.weight), (Hout, Hin), n64(dY), z=zo, activation=act,
                            has_bias=bias)
    r = lambda a, b_: float(np.linalg.norm(n64(a).reshape(-1) - np.asarray(b_).reshape(-1)) / np.linalg.norm(b_))
    assert r(Y, yo) < 1e-2 and r(X.grad, bw["dx"]) < 1e-2
    assert layer.weight.grad.shape == layer.weight.shape and r(layer.weight.grad, bw["dw"]) < 1e-2
    if bias:
        assert r(layer.bias.grad, bw["db"]) < 1e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("act", [None, "gelu"])
def test_empty_batch_behaves_like_torch(dtype, act):
    """No rows: the output is empty and every gradient is zero, as with torch.nn.Linear."""
    kw = {"fused_activation": act} if act else {}
    layer, seq = make_pair(64, 128, True, dtype, **kw)
    X = torch.empty(0, 64, dtype=dtype, device="cuda", requires_grad=True)
    Xs = X.detach().clone().requires_grad_(True)
    Y = layer(X)
    Ys = seq(Xs)
    if act:
        Ys = torch.nn.functional.gelu(Ys)
    assert Y.shape == Ys.shape == (0, 128) and Y.dtype == Ys.dtype
    Y.sum().backward()
    Ys.sum().backward()
    assert X.grad.shape == Xs.grad.shape == (0, 64)
    assert layer.weight.grad.shape == layer.weight.shape
    assert torch.equal(layer.weight.grad.view_as(seq.weight.grad), seq.weight.grad)   # zeros
    assert torch.equal(layer.bias.grad, seq.bias.grad)
    assert not layer.weight.grad.any() and not layer.bias.grad.any()


def test_skip_bias_add_returns_tuple():
    layer, seq = make_pair(64, 64, True, torch.bfloat16, skip_bias_add=True)
    X = torch.randn(8, 64).bfloat16().cuda()
    out = layer(X)
    assert isinstance(out, tuple) and out[1] is not None
    y, b = out
    assert rel(y + b, seq(X)) < 1e-2


def test_micro_batch_accumulation_into_param_grad():
    """With overlap_reduce_scatter the wgrad kernel adds into weight.grad; four
    micro-batches equal one backward over the concatenated batch."""
    from axonn_amd.intra_layer import optimize_communication

    layer, seq = make_pair(128, 256, True, torch.bfloat16, fused_activation="gelu")
    torch.manual_seed(3)
    xs = [torch.randn(64, 128).bfloat16().cuda() for _ in range(4)]
    gs = [(torch.randn(64, 256) * 0.1).bfloat16().cuda() for _ in range(4)]
    with optimize_communication(overlap_reduce_scatter=True):
        for x, g in zip(xs, gs):
            layer(x).backward(g)
    first = layer.weight.grad.clone()
    fused_ptr = layer.weight.grad.data_ptr()
    layer.zero_grad(set_to_none=True)
    for x, g in zip(xs, gs):   # plain autograd accumulation
        layer(x).backward(g)
    assert rel(first, layer.weight.grad) < 1e-2
    s32 = torch.nn.Linear(128, 256).cuda()
    s32.load_state_dict({"weight": layer.weight.detach().float().view(256, 128),
                         "bias": layer.bias.detach().float()})
    torch.nn.functional.gelu(s32(torch.cat(xs).float())).backward(torch.cat(gs).float())
    assert rel(first.view(256, 128), s32.weight.grad) < 1e-2
    assert rel(layer.bias.grad, s32.bias.grad) < 2e-2
    assert fused_ptr != 0


def test_autocast_bf16_with_fp32_master_weights():
    """fp32 parameters under torch.autocast: kernels run in bf16, gradients come
    back in the parameters' fp32 (custom_fwd/custom_bwd, fully_connected.py:32-54)."""
    layer, seq = make_pair(128, 128, False, torch.float32)
    X = torch.randn(32, 128).cuda().requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        Y = layer(X)
    assert Y.dtype == torch.bfloat16
    Y.float().sum().backward()
    assert layer.weight.grad.dtype == torch.float32 and X.grad.dtype == torch.float32
    Xs = X.detach().clone().requires_grad_(True)
    seq(Xs).sum().backward()
    assert rel(Y, seq(X)) < 1e-2 and rel(X.grad, Xs.grad) < 1e-2
    assert rel(layer.weight.grad.view(128, 128), seq.weight.grad) < 1e-2


@pytest.mark.parametrize("amp_dtype", [torch.bfloat16, torch.float16])
def test_autocast_with_an_fp32_bias_returns_fp32_as_the_reference_does(amp_dtype):
    """fp32 parameters under autocast, with a bias: the reference's product is 16-bit and
    its `x + bias` (fully_connected.py:348) is promoted to fp32 - torch.nn.Linear, whose
    addmm autocast casts as a whole, returns the 16-bit type instead.  Values against
    torch.nn.Linear in fp32 (<= 1e-2), dtypes asserted, gradients in the parameters' fp32."""
    layer, seq = make_pair(128, 256, True, torch.float32)
    with torch.no_grad():
        layer.bias.normal_(0, 0.5)
        seq.bias.copy_(layer.bias)
    torch.manual_seed(1)
    X = torch.randn(64, 128).cuda().requires_grad_(True)
    G = torch.randn(64, 256).cuda()
    with torch.autocast("cuda", dtype=amp_dtype):
        Y = layer(X)
        # the reference's composition, spelled out with torch ops
        want = torch.matmul(X, seq.weight.t()) + seq.bias
    assert want.dtype == torch.float32 and Y.dtype == torch.float32
    Xs = X.detach().clone().requires_grad_(True)
    Ys = seq(Xs)
    assert rel(Y, Ys) < 1e-2 and rel(Y, want) < 1e-2
    Y.backward(G)
    Ys.backward(G)
    assert layer.weight.grad.dtype == torch.float32 and layer.bias.grad.dtype == torch.float32
    assert X.grad.dtype == torch.float32
    assert rel(X.grad, Xs.grad) < 1e-2
    assert rel(layer.weight.grad.view(256, 128), seq.weight.grad) < 1e-2
    assert rel(layer.bias.grad, seq.bias.grad) < 1e-2
    # a 16-bit layer (bias cast with the module) keeps its own type, as `x + bias` does there
    half = layer.to(amp_dtype)
    assert half(X.detach().to(amp_dtype)).dtype == amp_dtype


def test_two_layer_mlp_step_matches_cpu_path():
    """The 2-layer MLP configuration (batch 64, 1024 -> 4096 GELU -> 1024, MSE,
    one Adam step) in fp32 against the torch CPU restatement."""
    import math

    from axonn_amd.intra_layer import Linear
    from axonn_amd.optim import CPUAdam
    from oracle import torch_cpu as ot

    torch.manual_seed(0)
    w1 = torch.nn.init.kaiming_uniform_(torch.empty(4096, 1024), a=math.sqrt(5))
    w2 = torch.nn.init.kaiming_uniform_(torch.empty(1024, 4096), a=math.sqrt(5))
    b1, b2 = torch.zeros(4096), torch.zeros(1024)
    x, tgt = torch.randn(64, 1024), torch.randn(64, 1024)
    want = ot.mlp_step(x, tgt, w1, b1, w2, b2)
    l1 = Linear(1024, 4096, fused_activation="gelu")
    l2 = Linear(4096, 1024)
    l1.load_state_dict({"weight": w1, "bias": b1})
    l2.load_state_dict({"weight": w2, "bias": b2})
    model = torch.nn.Sequential(l1, l2).cuda()
    opt = CPUAdam(model.parameters(), lr=1e-3, betas=(0.9, 0.999), eps=1e-8)
    y = model(x.cuda())
    loss = torch.nn.functional.mse_loss(y, tgt.cuda())
    loss.backward()
    assert abs(float(loss.detach()) - float(want["loss"])) < 1e-5 * float(want["loss"])
    grads = [p.grad.detach().clone() for p in model.parameters()]
    for g, w in zip(grads, want["grads"]):
        assert rel(g.reshape(-1), w.reshape(-1)) < 1e-4
    opt.step()
    # Adam's g / (|g| + eps) amplifies last-bit gradient differences, so the
    # 1e-6 master-weight bound is checked on identical gradients in
    # test_optim_gpu.py; here the step direction and size must agree
    for p, w in zip(model.parameters(), want["params"]):
        assert float((p.detach().cpu().reshape(-1) - w.reshape(-1)).abs().max()) < 2.1e-3
        assert rel(p.reshape(-1), w.reshape(-1)) < 1e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("in_f,out_f", [(64, 10), (50, 24), (27, 13)])
def test_feature_counts_that_are_not_multiples_of_eight(dtype, in_f, out_f):
    """A 16-bit layer takes any shape, as the reference's does (a 10-class head, odd widths):
    forward, input / weight / bias gradients against torch.nn.Linear in float64 on the same
    rounded parameters, also with the weight gradient accumulated by the kernel."""
    from axonn_amd.intra_layer import Linear, optimize_communication

    torch.manual_seed(in_f * 100 + out_f)
    layer = Linear(in_f, out_f).cuda().to(dtype)
    with torch.no_grad():
        layer.bias.copy_(torch.randn(out_f) * 0.1)
    ref = torch.nn.Linear(in_f, out_f).double()
    with torch.no_grad():
        ref.weight.copy_(layer.weight.detach().view(out_f, in_f).double().cpu())
        ref.bias.copy_(layer.bias.detach().double().cpu())
    x = torch.randn(37, in_f, device="cuda").to(dtype).requires_grad_(True)
    xr = x.detach().double().cpu().requires_grad_(True)
    dy = (torch.randn(37, out_f, device="cuda") * 0.1).to(dtype)
    tol = 1e-2 if dtype == torch.bfloat16 else 2e-3

    def rel(a, b):
        return float((a.double().cpu().reshape(-1) - b.reshape(-1)).norm() / b.norm())

    for overlap in (False, True):
        layer.zero_grad()
        x.grad = None
        xr.grad = None
        ref.zero_grad()
        with optimize_communication(overlap_reduce_scatter=overlap):
            y = layer(x)
            y.backward(dy)
        yr = ref(xr)
        yr.backward(dy.double().cpu())
        assert y.shape == (37, out_f)
        assert rel(y, yr.detach()) < tol and rel(x.grad, xr.grad) < tol
        assert rel(layer.weight.grad, ref.weight.grad) < tol
        assert rel(layer.bias.grad, ref.bias.grad) < tol
