"""Oracle (test infrastructure): the hot path written with torch CPU ops.

This is what the reference's calls reduce to on one rank: `input_.matmul(
weight.t())`, `grad_output.matmul(weight)`, `grad_output.t().mm(input_)`
(axonn/intra_layer/fully_connected.py:118, :140, :147-151), `x + bias` (:348),
and for the optimizer `div_(loss_scale)`, the sum-based overflow test, the
gradient clipping and `torch.optim._functional.adam` (axonn/optim.py:157-190,
axonn/inter_layer.py:435-460, axonn/intra_layer/gradient_normalization.py).

Used (a) by bench.py to time the CPU baseline on the host cores next to the GPU
numbers and (b) by the tests as a checker that shares no code with
oracle.linear / oracle.optim.  Never imported by the shipped package.
"""

import time

import torch
import torch.nn.functional as F


def linear_fwd_bwd(x, w, dy, bias=None, gelu=False):
    """One forward + backward of the layer in the dtype of the inputs.
    x [M,K], w [N,K], dy [M,N]; returns dict(y, dx, dw, db)."""
    x = x.detach().clone().requires_grad_(True)
    w = w.detach().clone().requires_grad_(True)
    b = None if bias is None else bias.detach().clone().requires_grad_(True)
    y = x.matmul(w.t())
    if b is not None:
        y = y + b
    if gelu:
        y = F.gelu(y)
    y.backward(dy)
    return {"y": y.detach(), "dx": x.grad, "dw": w.grad, "db": None if b is None else b.grad}


def mlp_step(x, target, w1, b1, w2, b2, lr=1e-3, betas=(0.9, 0.999), eps=1e-8):
    """The 2-layer MLP configuration: Linear -> GELU -> Linear, MSE loss, one
    forward + backward + Adam step.  Returns dict(loss, params after the step,
    grads)."""
    params = [t.detach().clone().requires_grad_(True) for t in (w1, b1, w2, b2)]
    w1, b1, w2, b2 = params
    h = F.gelu(x.matmul(w1.t()) + b1)
    y = h.matmul(w2.t()) + b2
    loss = F.mse_loss(y, target)
    loss.backward()
    grads = [p.grad.detach().clone() for p in params]
    opt = torch.optim.Adam(params, lr=lr, betas=betas, eps=eps, foreach=False)
    opt.step()
    return {"loss": loss.detach(), "params": [p.detach() for p in params], "grads": grads,
            "y": y.detach()}


def check_nan(t):
    s = t.sum()
    return bool((torch.isinf(s) + torch.isnan(s)) > 0)


def optimizer_step(g_lowp, p32, m, v, step, loss_scale, max_norm=0.0, lr=1e-3,
                   betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0,
                   lowp_dtype=torch.bfloat16):
    """Unscale -> overflow check -> clip -> Adam -> cast back, in place on the
    given float32 lists p32, m, v.  Returns dict(overflow, total_norm, p_low)."""
    overflow = False
    for g in g_lowp:
        overflow = overflow or check_nan(g)
    if overflow:
        return {"overflow": True, "total_norm": None, "p_low": None}
    g32 = [g.float().div_(loss_scale) for g in g_lowp]
    total = None
    if max_norm > 0:
        holders = [torch.nn.Parameter(p) for p in p32]
        for h, g in zip(holders, g32):
            h.grad = g
        total = torch.nn.utils.clip_grad_norm_(holders, max_norm, foreach=False)
    else:
        total = torch.norm(torch.stack([torch.norm(g) for g in g32]))
    beta1, beta2 = betas
    steps = [torch.tensor(float(step - 1)) for _ in p32]
    torch.optim._functional.adam(
        list(p32), g32, list(m), list(v), [], steps, foreach=False, amsgrad=False,
        beta1=beta1, beta2=beta2, lr=lr, weight_decay=weight_decay, eps=eps, maximize=False,
    )
    return {"overflow": False, "total_norm": float(total), "p_low": [p.to(lowp_dtype) for p in p32]}


def time_linear_set(shapes, reps=1, dtype=torch.float32, seed=0):
    """Times fwd+bwd of each (M, N, K) on the host cores; returns
    (seconds, flops) summed over the set."""
    g = torch.Generator().manual_seed(seed)
    total_s, total_f = 0.0, 0.0
    for (M, N, K) in shapes:
        x = torch.randn(M, K, generator=g, dtype=dtype)
        w = torch.randn(N, K, generator=g, dtype=dtype) * 0.02
        dy = torch.randn(M, N, generator=g, dtype=dtype) * 1e-3
        linear_fwd_bwd(x, w, dy)  # warm-up (thread pool, page faults)
        t0 = time.perf_counter()
        for _ in range(reps):
            linear_fwd_bwd(x, w, dy)
        total_s += (time.perf_counter() - t0) / reps
        total_f += 6.0 * M * N * K
    return total_s, total_f
