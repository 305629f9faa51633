"""Oracle (test infrastructure) for the mixed-precision optimizer step.

Restates, in numpy, what the reference does between the end of backward and the
updated parameters: overflow check and unscaling (axonn/inter_layer.py:435-460),
the loss-scale state machine (:18-28, :274-302), gradient clipping
(axonn/intra_layer/gradient_normalization.py:18-95), and the Adam update with
low-precision cast-back (axonn/optim.py:157-190, which calls
torch.optim._functional.adam; its non-capturable single-tensor form is restated
in `adam_update`).

The reference has no test for any of this ("parity unpinned" by the reference);
tests/test_oracle.py pins these functions against torch.optim.Adam,
torch.nn.utils.clip_grad_norm_, closed forms and brute force.
"""

from dataclasses import dataclass

import numpy as np

from .linear import round_to

F32 = np.float32


# --------------------------------------------------------- flat buffers ------
def coalesce(tensors):
    """axonn/utils.py:11-30: one flat 1-D buffer, tensors packed back to back in
    order with no padding; returns (flat, views) where views[i] aliases flat."""
    sizes = [int(np.size(t)) for t in tensors]
    flat = np.concatenate([np.asarray(t).reshape(-1) for t in tensors]) if tensors else np.zeros(0)
    views, off = [], 0
    for t, n in zip(tensors, sizes):
        views.append(flat[off:off + n].reshape(np.shape(t)))
        off += n
    return flat, views


def group_offsets(group_sizes):
    """axonn/optim.py:59-65: cumulative element counts of the param groups."""
    off = [0]
    for n in group_sizes:
        off.append(off[-1] + int(n))
    return off


# ------------------------------------------------------- overflow check ------
def check_nan(tensor, dtype):
    """axonn/inter_layer.py:435-445: `s = tensor.sum(); isinf(s) + isnan(s) > 0`.

    `tensor` holds values of storage type `dtype`; torch accumulates a
    low-precision sum in float32 and rounds the result to the tensor's dtype, so
    an fp16 tensor of finite values whose sum exceeds 65504 reports overflow."""
    x = np.asarray(tensor, dtype=np.float64)
    with np.errstate(invalid="ignore", over="ignore"):
        s = round_to(np.sum(x), dtype)
    return bool(np.isinf(s) or np.isnan(s))


def any_nonfinite(tensor):
    """The element-wise criterion; equals check_nan whenever the sum of the
    finite values stays inside the dtype's range."""
    return bool(np.any(~np.isfinite(np.asarray(tensor, dtype=np.float64))))


@dataclass
class LossScaler:
    """axonn/inter_layer.py:18-28."""

    loss_scale: float = 2.0 ** 16
    max_scale: float = 2.0 ** 24
    min_scale: float = 2.0 ** 10
    scaling_window: float = 200
    no_overflow_iters: float = 0


def sync_scale(scaler, local_overflow):
    """axonn/inter_layer.py:274-302 on one rank: halve on overflow (floor
    min_scale) and reset the counter; otherwise count, and after scaling_window
    clean steps double (cap max_scale) and reset.  Returns global_overflow."""
    if local_overflow:
        scaler.loss_scale = max(scaler.loss_scale / 2.0, scaler.min_scale)
        scaler.no_overflow_iters = 0
        return True
    scaler.no_overflow_iters += 1
    if scaler.no_overflow_iters == scaler.scaling_window:
        scaler.loss_scale = min(scaler.loss_scale * 2.0, scaler.max_scale)
        scaler.no_overflow_iters = 0
    return False


def unscale_gradients(grads, dtype, loss_scale):
    """axonn/inter_layer.py:447-460: overflow is checked on the SCALED gradients
    in their own dtype; every gradient is divided in place by the scale (also
    when overflow was found); returns (local_overflow, unscaled grads)."""
    overflow = False
    out = []
    for g in grads:
        overflow = overflow or check_nan(g, dtype)
        with np.errstate(invalid="ignore", over="ignore"):
            out.append(round_to(np.asarray(g, dtype=np.float64) / loss_scale, dtype))
    return overflow, out


# ----------------------------------------------------------- grad norm -------
def _norm(x, norm_type):
    """torch.norm(x, p) of a flat float64 vector: (sum |x|^p)^(1/p); p = 0 counts the
    non-zero elements, p = +inf / -inf are the largest / smallest |x| (NaN if any is)."""
    x = np.abs(np.asarray(x, dtype=np.float64).reshape(-1))
    if norm_type == 0:
        return float(np.count_nonzero(x))
    if norm_type == np.inf:
        return float(np.max(x))
    if norm_type == -np.inf:
        return float(np.min(x))
    with np.errstate(divide="ignore", over="ignore"):
        return float(np.sum(x ** norm_type) ** (1.0 / norm_type))


def get_total_norm(tensors, dtype="f64", norm_type=2.0):
    """gradient_normalization.py:18-34: the norm_type-norm of the stacked per-tensor
    norm_type-norms, each torch.norm returning the tensor's dtype.  The reference passes
    any order through to torch.norm (clip_grad_norm_ refuses inf earlier, :38-39)."""
    if len(tensors) == 0:
        return 0.0
    per = [round_to(_norm(t, norm_type), dtype) for t in tensors]
    return float(round_to(_norm(np.asarray(per), norm_type), dtype))


def clip_coef(total_norm, max_norm):
    """gradient_normalization.py:86-87."""
    c = float(max_norm) / (total_norm + 1e-6)
    return min(c, 1.0) if c == c else c


def clip_grad_norm_(grads, max_norm, dtype="f64", norm_type=2.0):
    """gradient_normalization.py:37-95 on one rank: every process group has one member
    (the all-reduce of norm^p over a group and the 1/p power after it, :74-81, give the
    group's norm back), so the total is the norm over all gradients; every gradient is
    multiplied by the clamped coefficient, also when it is 1.
    Returns (total_norm, clipped grads)."""
    total = get_total_norm(grads, dtype, norm_type)
    c = clip_coef(total, max_norm)
    c = float(round_to(c, "f32"))  # the coefficient is a float32 tensor in torch
    return total, [round_to(np.asarray(g, dtype=np.float64) * c, dtype) for g in grads]


# ----------------------------------------------------------------- Adam ------
def bias_corrections(step, beta1, beta2):
    """Python doubles, as torch/optim/adam.py::_single_tensor_adam computes them."""
    bc1 = 1.0 - beta1 ** step
    bc2 = 1.0 - beta2 ** step
    return bc1, bc2


def adam_update(p, g, m, v, step, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8,
                weight_decay=0.0):
    """One float32 Adam update, operation for operation as torch's
    _single_tensor_adam (amsgrad False, maximize False), which is what
    axonn/optim.py:168-182 invokes.  Inputs are float32 arrays; returns new
    (p, m, v) as float32.  `step` is the 1-based step count."""
    p = np.asarray(p, dtype=F32)
    g = np.asarray(g, dtype=F32)
    m = np.asarray(m, dtype=F32)
    v = np.asarray(v, dtype=F32)
    if weight_decay != 0:
        g = g + F32(weight_decay) * p                      # grad.add(param, alpha=wd)
    m = m + (g - m) * F32(1.0 - beta1)                     # exp_avg.lerp_(grad, 1 - beta1)
    v = v * F32(beta2) + F32(1.0 - beta2) * g * g          # mul_(beta2).addcmul_(g, g, 1-beta2)
    bc1, bc2 = bias_corrections(step, beta1, beta2)
    step_size = lr / bc1
    bc2_sqrt = bc2 ** 0.5
    denom = np.sqrt(v) / F32(bc2_sqrt) + F32(eps)          # (sqrt(v) / bc2_sqrt).add_(eps)
    p = p + F32(-step_size) * (m / denom)                  # addcdiv_(m, denom, value=-step_size)
    return p.astype(F32), m.astype(F32), v.astype(F32)


def adam_update_f64(p, g, m, v, step, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8,
                    weight_decay=0.0):
    """The same recurrences in float64 (the mathematics, free of rounding order)."""
    p, g, m, v = (np.asarray(a, dtype=np.float64) for a in (p, g, m, v))
    if weight_decay != 0:
        g = g + weight_decay * p
    m = beta1 * m + (1.0 - beta1) * g
    v = beta2 * v + (1.0 - beta2) * g * g
    bc1, bc2 = bias_corrections(step, beta1, beta2)
    p = p - (lr / bc1) * m / (np.sqrt(v) / np.sqrt(bc2) + eps)
    return p, m, v


def mixed_precision_step(g_lowp, p32, m, v, step, loss_scale, g_dtype="bf16",
                         p_dtype="bf16", max_norm=0.0, lr=1e-3, beta1=0.9,
                         beta2=0.999, eps=1e-8, weight_decay=0.0):
    """The whole step over lists of tensors, all-or-nothing on overflow (the
    engine's gate, axonn/inter_layer.py:426-432):

      overflow  = OR_i check_nan(g_i)            on the scaled low-precision grads
      g32_i     = float32(g_i) / loss_scale      (optim.py:157-160)
      total     = || all g32 ||_2 ; coef = min(1, max_norm / (total + 1e-6))
      g32_i    *= coef                           (gradient_normalization.py:86-93)
      Adam on (p32_i, m_i, v_i)                  (optim.py:168-182)
      p_low_i   = round(p32_i)                   (optim.py:183-185)

    Returns dict(overflow, total_norm, clip_coef, p, m, v, p_low); on overflow
    p, m, v are returned unchanged and p_low is None."""
    overflow = False
    for g in g_lowp:
        overflow = overflow or check_nan(g, g_dtype)
    with np.errstate(invalid="ignore", over="ignore"):
        g32 = [(np.asarray(g, dtype=F32) / F32(loss_scale)).astype(F32) for g in g_lowp]
        sumsq = float(sum(np.sum(g.astype(np.float64) ** 2) for g in g32))
    total = float(np.sqrt(sumsq))
    coef = 1.0
    if max_norm > 0:
        coef = float(F32(clip_coef(float(F32(total)), max_norm)))
    out = {"overflow": overflow, "total_norm": total, "clip_coef": coef}
    if overflow:
        out.update(p=list(p32), m=list(m), v=list(v), p_low=None)
        return out
    ps, ms, vs, pl = [], [], [], []
    for g, p, mm, vv in zip(g32, p32, m, v):
        g = (g * F32(coef)).astype(F32)
        p2, m2, v2 = adam_update(p, g, mm, vv, step, lr, beta1, beta2, eps, weight_decay)
        ps.append(p2)
        ms.append(m2)
        vs.append(v2)
        pl.append(round_to(p2, p_dtype).astype(F32))
    out.update(p=ps, m=ms, v=vs, p_low=pl)
    return out
