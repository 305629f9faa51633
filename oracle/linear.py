"""Oracle (test infrastructure) for the Linear layer at a 1 x 1 x 1 grid.

Every collective of the reference is the identity when its group has one rank
(axonn/intra_layer/communication.py:24-25, :37-38, :71-72), so the layer reduces
to the three matrix products below.  All arithmetic here is float64 unless a
function says otherwise; rounding to the storage type is explicit.
"""

import math

import numpy as np

try:  # scipy is only a faster erf; math.erf is the definition used for pinning
    from scipy.special import erf as _erf
except ImportError:  # pragma: no cover
    _erf = np.vectorize(math.erf, otypes=[np.float64])

SQRT2 = math.sqrt(2.0)
INV_SQRT_2PI = 1.0 / math.sqrt(2.0 * math.pi)


# ---------------------------------------------------------------- bfloat16 ---
def bf16_bits(x):
    """float32 array -> uint16 bfloat16 bit patterns, round to nearest even.

    Every NaN maps to the canonical quiet NaN 0x7FC0, as torch's conversion does."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    rounding = ((u >> 16) & 1) + np.uint32(0x7FFF)
    out = ((u + rounding) >> 16).astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        out = np.where(nan, np.uint16(0x7FC0), out)
    return out


def bf16_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def bf16_round(x):
    """Rounds a float array to the nearest bfloat16 value, returned as float32."""
    return bf16_to_f32(bf16_bits(np.asarray(x, dtype=np.float32))).reshape(np.shape(x))


def round_to(x, dtype):
    """Rounds float64 values to the storage type named by `dtype`
    ('bf16', 'f16', 'f32', 'f64'); result is float64 for further arithmetic."""
    x = np.asarray(x, dtype=np.float64)
    if dtype == "f64":
        return x
    if dtype == "f32":
        return x.astype(np.float32).astype(np.float64)
    if dtype == "f16":
        return x.astype(np.float32).astype(np.float16).astype(np.float64)
    if dtype == "bf16":
        # double rounding through float32 differs from direct rounding only on
        # exact ties of the float32 result, which random data never hits
        return bf16_round(x.astype(np.float32)).astype(np.float64)
    raise ValueError(dtype)


# --------------------------------------------------------------------- GELU --
def gelu(z):
    """Exact-erf GELU, torch.nn.GELU() default: 0.5 z (1 + erf(z / sqrt 2)).
    The reference's callers place it between two Linears
    (docs/user_guide.rst:118-121)."""
    z = np.asarray(z, dtype=np.float64)
    return 0.5 * z * (1.0 + _erf(z / SQRT2))


def dgelu(z):
    """d gelu / dz = Phi(z) + z phi(z)."""
    z = np.asarray(z, dtype=np.float64)
    return 0.5 * (1.0 + _erf(z / SQRT2)) + z * INV_SQRT_2PI * np.exp(-0.5 * z * z)


# ------------------------------------------------------------------- layer ---
def default_init_bound(in_features):
    """kaiming_uniform_(a=sqrt 5) on [out, in] draws U(-b, b) with
    b = sqrt(2 / (1 + 5)) * sqrt(3 / in) = 1 / sqrt(in)
    (fully_connected.py:91-93)."""
    return 1.0 / math.sqrt(in_features)


def extract_local_params_from_full_params(full):
    """[out, in] -> flat 1-D row-major; Drop is the identity on one rank
    (fully_connected.py:62-70)."""
    return np.ascontiguousarray(full).reshape(-1)


def linear_forward(x, weight_flat, shape, bias=None, skip_bias_add=False,
                   activation=None):
    """Linear.forward + AsyncLinear.forward (fully_connected.py:303-348, :96-121).

    x [..., K]; weight_flat is the 1-D parameter, shape = (N, K).
    Returns (y, z) where z is the pre-activation (== y without activation);
    with skip_bias_add returns ((y, bias), z) as the reference returns a tuple.
    """
    n, k = shape
    x = np.asarray(x, dtype=np.float64)
    w = np.asarray(weight_flat, dtype=np.float64).reshape(n, k)       # :113
    x2 = x.reshape(-1, x.shape[-1])                                    # :309
    z = x2 @ w.T                                                       # :118
    z = z.reshape(*x.shape[:-1], n)                                    # :337
    if bias is None:
        y = z
    elif skip_bias_add:                                                # :345-346
        return (z, np.asarray(bias, dtype=np.float64)), z
    else:
        z = z + np.asarray(bias, dtype=np.float64)                     # :348
        y = z
    if activation == "gelu":
        y = gelu(z)
    elif activation is not None:
        raise ValueError(activation)
    return y, z


def linear_backward(x, weight_flat, shape, grad_out, z=None, activation=None,
                    has_bias=False):
    """AsyncLinear.backward (fully_connected.py:123-187) plus what autograd adds
    for `x + bias` (:348) and a trailing GELU.

    Returns dict(dx, dw (flat, as the reference returns it :153), db)."""
    n, k = shape
    x = np.asarray(x, dtype=np.float64)
    w = np.asarray(weight_flat, dtype=np.float64).reshape(n, k)
    g = np.asarray(grad_out, dtype=np.float64)
    if activation == "gelu":
        g = g * dgelu(np.asarray(z, dtype=np.float64))
    g2 = g.reshape(-1, n)                                              # :148
    x2 = x.reshape(-1, k)                                              # :150
    dx = (g2 @ w).reshape(x.shape)                                     # :140
    dw = (g2.T @ x2).reshape(-1)                                       # :147-153
    out = {"dx": dx, "dw": dw, "dz": g}
    if has_bias:
        out["db"] = g2.sum(axis=0)
    return out


def accumulate(param_grad, grad, dtype):
    """param.grad = grad.to(dtype) the first time, param.grad.add_(grad.to(dtype))
    afterwards, all in the parameter's dtype
    (overlap_communication.py:38-47; autograd's AccumulateGrad does the same)."""
    g = round_to(grad, dtype)
    if param_grad is None:
        return g
    return round_to(np.asarray(param_grad, dtype=np.float64) + g, dtype)
