"""Tensor-level wrappers over the C ABI of libaxn_gfx950.so.

Each function checks dtypes and devices, allocates the outputs with torch,
passes raw pointers, sizes and torch's current HIP stream to the library and
returns.  None of the arithmetic happens here, and nothing here falls back to a
torch op: tensors that are not on a GPU are rejected.
"""

import torch

from . import _native as nv

EPILOGUES = {
    (False, None): nv.EPI_NONE,
    (True, None): nv.EPI_BIAS,
    (True, "gelu"): nv.EPI_BIAS_GELU,
    (False, "gelu"): nv.EPI_GELU,
}


def _require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "axonn_amd kernels run on the GPU only; got a tensor on %s" % t.device
            )


def _rows(t):
    """A 2-D tensor usable by the kernels: unit stride along the last dimension.
    Returns (tensor, leading dimension)."""
    if t.dim() != 2:
        raise ValueError("expected a 2-D tensor, got shape %s" % (tuple(t.shape),))
    if t.stride(1) != 1 or (t.shape[0] > 1 and t.stride(0) < t.shape[1]):
        t = t.contiguous()
    ld = t.stride(0) if t.shape[0] > 1 else t.shape[1]
    return t, ld


def _bf16_ok(t, ld):
    return t.data_ptr() % 16 == 0 and ld % 8 == 0


def _prep_bf16(t):
    t, ld = _rows(t)
    if not _bf16_ok(t, ld):
        t = t.contiguous().clone()
        ld = t.shape[1]
    return t, ld


def _pad8(t, dim):
    """`t` with dimension `dim` (0 or 1) of a 2-D tensor zero-padded up to a multiple of 8."""
    r = (-t.shape[dim]) % 8
    if r == 0:
        return t
    return torch.nn.functional.pad(t, (0, r) if dim == 1 else (0, 0, 0, r))


def _ragged16(dtype, *dims):
    """The 16-bit MFMA kernels move 16-byte vectors: feature counts that are not multiples
    of 8 (a 10-class head, a vocabulary of 50257) run on operands zero-padded to the next
    multiple (zeros add nothing to a product) and the result is cut back."""
    return dtype in _GEMM16 and any(d % 8 for d in dims)


# ------------------------------------------------------------------ GEMMs ----
# 16-bit operand types of the MFMA kernels -> suffix of their entry points
_GEMM16 = {torch.bfloat16: "", torch.float16: "_f16"}
GEMM_FWD, GEMM_DGRAD, GEMM_WGRAD = 0, 1, 2


def _split_workspace(op, M, N, K, device):
    """Workspace for a GEMM whose contraction the library would divide among workgroups
    (few output tiles), or (None, 0)."""
    nbytes = nv.load().axn_gemm_workspace_bytes(op, M, N, K)
    if nbytes == 0:
        return None, 0
    return torch.empty(nbytes, dtype=torch.uint8, device=device), nbytes


def gemm_fwd(x, w, bias=None, activation=None, save_z=False, out_f32=False):
    """Y = act(X W^T + b).  x [M,K], w [N,K]; bf16, fp16 or fp32 (both the same).
    Returns (y, z) with z the saved pre-activation (None unless activation and
    save_z).  out_f32 (16-bit operands with a bias): y is fp32, the sum with the fp32
    bias left unrounded, as type promotion leaves the reference's `x + bias`
    (axonn/intra_layer/fully_connected.py:348) under autocast."""
    _require_gpu(x, w, bias)
    if x.dtype != w.dtype:
        raise TypeError("input is %s but weight is %s" % (x.dtype, w.dtype))
    epi = EPILOGUES[(bias is not None, activation)]
    M, K = x.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise ValueError("weight is %s, input has %d features" % (tuple(w.shape), K))
    if bias is not None:
        bias = bias.float().contiguous()
        if bias.numel() != N:
            raise ValueError("bias has %d elements, expected %d" % (bias.numel(), N))
    want_z = activation is not None and save_z
    if x.dtype not in _GEMM16 and x.dtype != torch.float32:
        raise TypeError("the Linear kernels take bf16, fp16 or fp32 operands, got %s" % x.dtype)
    if M == 0:  # an empty batch: nothing to launch (the library takes M >= 1)
        y = torch.empty((0, N), dtype=x.dtype, device=x.device)
        return y, (torch.empty_like(y) if want_z else None)
    if out_f32 and (bias is None or x.dtype not in _GEMM16):
        raise ValueError("out_f32 is the promotion of a 16-bit product by an fp32 bias")
    if _ragged16(x.dtype, N, K):
        bp = None if bias is None else _pad8(bias.reshape(1, -1), 1).reshape(-1)
        y, z = gemm_fwd(_pad8(x, 1), _pad8(_pad8(w, 1), 0), bp, activation, save_z, out_f32)
        return y[:, :N].contiguous(), (None if z is None else z[:, :N].contiguous())
    if x.dtype in _GEMM16:
        x, ldx = _prep_bf16(x)
        w, ldw = _prep_bf16(w)
        z = torch.empty((M, N), dtype=x.dtype, device=x.device) if want_z else None
        if out_f32:
            y = torch.empty((M, N), dtype=torch.float32, device=x.device)
            nv.call("axn_gemm_fwd_f32out", nv.ptr(x), nv.ptr(w), nv.ptr(bias), nv.ptr(y), nv.ptr(z),
                    nv.dtype_code(x.dtype), M, N, K, ldx, ldw, N, epi, nv.current_stream())
            return y, z
        y = torch.empty((M, N), dtype=x.dtype, device=x.device)
        # (the contraction is only divided for a plain product: an epilogue runs unsplit)
        ws, ws_bytes = _split_workspace(GEMM_FWD, M, N, K, x.device) if epi == nv.EPI_NONE else (None, 0)
        if ws is not None:
            nv.call("axn_gemm_fwd_ws", nv.ptr(x), nv.ptr(w), nv.ptr(bias), nv.ptr(y), nv.ptr(z),
                    nv.dtype_code(x.dtype), M, N, K, ldx, ldw, N, epi, nv.ptr(ws), ws_bytes,
                    nv.current_stream())
            return y, z
        nv.call("axn_gemm_fwd" + _GEMM16[x.dtype], nv.ptr(x), nv.ptr(w), nv.ptr(bias), nv.ptr(y), nv.ptr(z),
                M, N, K, ldx, ldw, N, epi, nv.current_stream())
    elif x.dtype == torch.float32:
        x, w = x.contiguous(), w.contiguous()
        y = torch.empty((M, N), dtype=torch.float32, device=x.device)
        z = torch.empty_like(y) if want_z else None
        nv.call("axn_gemm_fwd_f32", nv.ptr(x), nv.ptr(w), nv.ptr(bias), nv.ptr(y), nv.ptr(z),
                M, N, K, epi, nv.current_stream())
    else:
        raise TypeError("the Linear kernels take bf16, fp16 or fp32 operands, got %s" % x.dtype)
    return y, z


def gemm_dgrad(dy, w):
    """dX = dY W.  dy [M,N], w [N,K]."""
    _require_gpu(dy, w)
    if dy.dtype != w.dtype:
        raise TypeError("grad_output is %s but weight is %s" % (dy.dtype, w.dtype))
    M, N = dy.shape
    K = w.shape[1]
    if dy.dtype not in _GEMM16 and dy.dtype != torch.float32:
        raise TypeError("the Linear kernels take bf16, fp16 or fp32 operands, got %s" % dy.dtype)
    if M == 0:
        return torch.empty((0, K), dtype=dy.dtype, device=dy.device)
    if _ragged16(dy.dtype, N, K):
        return gemm_dgrad(_pad8(dy, 1), _pad8(_pad8(w, 1), 0))[:, :K].contiguous()
    if dy.dtype in _GEMM16:
        dy, lddy = _prep_bf16(dy)
        w, ldw = _prep_bf16(w)
        dx = torch.empty((M, K), dtype=dy.dtype, device=dy.device)
        ws, ws_bytes = _split_workspace(GEMM_DGRAD, M, N, K, dy.device)
        if ws is not None:
            nv.call("axn_gemm_dgrad_ws", nv.ptr(dy), nv.ptr(w), nv.ptr(dx),
                    nv.dtype_code(dy.dtype), M, N, K, lddy, ldw, K, nv.ptr(ws), ws_bytes,
                    nv.current_stream())
            return dx
        nv.call("axn_gemm_dgrad" + _GEMM16[dy.dtype], nv.ptr(dy), nv.ptr(w), nv.ptr(dx), M, N, K, lddy, ldw, K,
                nv.current_stream())
    elif dy.dtype == torch.float32:
        dy, w = dy.contiguous(), w.contiguous()
        dx = torch.empty((M, K), dtype=torch.float32, device=dy.device)
        nv.call("axn_gemm_dgrad_f32", nv.ptr(dy), nv.ptr(w), nv.ptr(dx), M, N, K,
                nv.current_stream())
    else:
        raise TypeError("the Linear kernels take bf16, fp16 or fp32 operands, got %s" % dy.dtype)
    return dx


def gemm_wgrad(dy, x, out=None, accumulate=False, out_dtype=None):
    """dW = dY^T X, optionally accumulated into `out` (dW += ...).  dy [M,N],
    x [M,K]; the result is [N,K] in `out_dtype` (bf16 or fp32 for bf16 operands)."""
    _require_gpu(dy, x, out)
    if dy.dtype != x.dtype:
        raise TypeError("grad_output is %s but input is %s" % (dy.dtype, x.dtype))
    M, N = dy.shape
    K = x.shape[1]
    if out is not None:
        if out.numel() != N * K or not out.is_contiguous():
            raise ValueError("`out` must be a contiguous tensor of %d elements" % (N * K))
        out_dtype = out.dtype
    elif accumulate:
        raise ValueError("accumulate=True needs `out`")
    if out_dtype is None:
        out_dtype = dy.dtype
    if M == 0 and (dy.dtype in _GEMM16 or dy.dtype == torch.float32):
        # an empty batch contributes a zero gradient
        if out is None:
            return torch.zeros((N, K), dtype=out_dtype, device=dy.device)
        return out if accumulate else out.zero_()
    if _ragged16(dy.dtype, N, K):
        # the kernel accumulates into a padded copy of the gradient, which is cut back
        tmp = None
        if out is not None:
            tmp = _pad8(_pad8(out.view(N, K), 1), 0) if accumulate else \
                torch.empty((N + (-N) % 8, K + (-K) % 8), dtype=out.dtype, device=out.device)
        full = gemm_wgrad(_pad8(dy, 1), _pad8(x, 1), out=tmp, accumulate=accumulate, out_dtype=out_dtype)
        if out is None:
            return full[:N, :K].contiguous()
        out.view(N, K).copy_(full[:N, :K])
        return out
    if dy.dtype in _GEMM16:
        if out_dtype not in (dy.dtype, torch.float32):
            raise TypeError("dW must be %s or fp32, got %s" % (dy.dtype, out_dtype))
        dy, lddy = _prep_bf16(dy)
        x, ldx = _prep_bf16(x)
        if out is None:
            out = torch.empty((N, K), dtype=out_dtype, device=dy.device)
        ws, ws_bytes = _split_workspace(GEMM_WGRAD, M, N, K, dy.device)
        if ws is not None:
            nv.call("axn_gemm_wgrad_ws", nv.ptr(dy), nv.ptr(x), nv.ptr(out),
                    nv.dtype_code(dy.dtype), M, N, K, lddy, ldx, K, 1 if accumulate else 0,
                    nv.dtype_code(out_dtype), nv.ptr(ws), ws_bytes, nv.current_stream())
            return out
        nv.call("axn_gemm_wgrad" + _GEMM16[dy.dtype], nv.ptr(dy), nv.ptr(x), nv.ptr(out), M, N, K, lddy, ldx, K,
                1 if accumulate else 0, nv.dtype_code(out_dtype), nv.current_stream())
    elif dy.dtype == torch.float32:
        if out_dtype != torch.float32:
            raise TypeError("fp32 operands give an fp32 dW, got %s" % out_dtype)
        dy, x = dy.contiguous(), x.contiguous()
        if out is None:
            out = torch.empty((N, K), dtype=torch.float32, device=dy.device)
        nv.call("axn_gemm_wgrad_f32", nv.ptr(dy), nv.ptr(x), nv.ptr(out), M, N, K,
                1 if accumulate else 0, nv.current_stream())
    else:
        raise TypeError("the Linear kernels take bf16, fp16 or fp32 operands, got %s" % dy.dtype)
    return out


def gemm_bwd(dy, w, x, out=None, accumulate=False, out_dtype=None):
    """(dX, dW) = (dY W, dY^T X) of one layer, dW optionally accumulated into `out`: the two
    products of AsyncLinear.backward (axonn/intra_layer/fully_connected.py:140, :147-151)
    through ONE entry point, which runs both in a single launch where their tile counts
    would each leave CUs idle in a launch of their own.  Results equal gemm_dgrad and
    gemm_wgrad bit for bit; shapes the joint entry point does not take go through those."""
    _require_gpu(dy, w, x, out)
    M, N = dy.shape
    K = w.shape[1]
    plain16 = (dy.dtype in _GEMM16 and dy.dtype == w.dtype == x.dtype and M > 0
               and not _ragged16(dy.dtype, N, K)
               and nv.load().axn_gemm_workspace_bytes(GEMM_DGRAD, M, N, K) == 0
               and nv.load().axn_gemm_workspace_bytes(GEMM_WGRAD, M, N, K) == 0)
    if not plain16:
        return gemm_dgrad(dy, w), gemm_wgrad(dy, x, out=out, accumulate=accumulate, out_dtype=out_dtype)
    if x.shape != (M, K) or w.shape[0] != N:
        raise ValueError("shapes do not match: dY %s, W %s, X %s" % (tuple(dy.shape), tuple(w.shape),
                                                                     tuple(x.shape)))
    if out is not None:
        if out.numel() != N * K or not out.is_contiguous():
            raise ValueError("`out` must be a contiguous tensor of %d elements" % (N * K))
        out_dtype = out.dtype
    elif accumulate:
        raise ValueError("accumulate=True needs `out`")
    if out_dtype is None:
        out_dtype = dy.dtype
    if out_dtype not in (dy.dtype, torch.float32):
        raise TypeError("dW must be %s or fp32, got %s" % (dy.dtype, out_dtype))
    dy, lddy = _prep_bf16(dy)
    w, ldw = _prep_bf16(w)
    x, ldx = _prep_bf16(x)
    dx = torch.empty((M, K), dtype=dy.dtype, device=dy.device)
    if out is None:
        out = torch.empty((N, K), dtype=out_dtype, device=dy.device)
    nv.call("axn_gemm_bwd", nv.ptr(dy), nv.ptr(w), nv.ptr(x), nv.ptr(dx), nv.ptr(out), nv.dtype_code(dy.dtype),
            M, N, K, lddy, ldw, ldx, K, K, 1 if accumulate else 0, nv.dtype_code(out_dtype),
            nv.current_stream())
    return dx, out


def dgelu_dbias(dy, z=None, want_dbias=True, dbias_out=None, accumulate=False):
    """dZ = dY * gelu'(Z) (when z is given) and dbias = column sums of dZ (fp32).
    Returns (dz, dbias); dz is dy itself when z is None."""
    _require_gpu(dy, z, dbias_out)
    if dy.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise TypeError("bf16, fp16 or fp32 expected, got %s" % dy.dtype)
    if dy.dim() == 2 and dy.shape[1] % 8:   # ragged width: zero-padded columns, results cut back
        N = dy.shape[1]
        acc = None
        if want_dbias and dbias_out is not None:
            acc = _pad8(dbias_out.reshape(1, -1), 1).reshape(-1) if accumulate else \
                torch.empty(N + (-N) % 8, dtype=torch.float32, device=dy.device)
        dz, db = dgelu_dbias(_pad8(dy, 1), None if z is None else _pad8(z, 1), want_dbias, acc,
                             accumulate)
        if db is not None and dbias_out is not None:
            dbias_out.copy_(db[:N])
            db = dbias_out
        elif db is not None:
            db = db[:N].contiguous()
        return (dz[:, :N].contiguous() if z is not None else dy), db
    dy, ld = _rows(dy)
    if dy.data_ptr() % 16 or ld % 8:
        dy = dy.contiguous().clone()
        ld = dy.shape[1]
    M, N = dy.shape
    dz = None
    if M == 0:
        if z is not None and (z.dtype != dy.dtype or z.shape != dy.shape):
            raise ValueError("z must match dy in dtype and shape")
        dbias = None
        if want_dbias:
            dbias = dbias_out if dbias_out is not None else torch.zeros(N, dtype=torch.float32, device=dy.device)
            if dbias_out is not None and not accumulate:
                dbias.zero_()
        return (torch.empty_like(dy) if z is not None else dy), dbias
    if z is not None:
        if z.dtype != dy.dtype or z.shape != dy.shape:
            raise ValueError("z must match dy in dtype and shape")
        if not z.is_contiguous() or ld != N:
            z = z.contiguous()
            dy = dy.contiguous()
            ld = N
        dz = torch.empty_like(dy)
    dbias = None
    ws, ws_bytes = None, 0
    if want_dbias:
        dbias = dbias_out if dbias_out is not None else torch.empty(N, dtype=torch.float32, device=dy.device)
        if dbias.dtype != torch.float32 or dbias.numel() != N:
            raise ValueError("dbias must be fp32 with %d elements" % N)
        ws_bytes = nv.load().axn_dgelu_dbias_workspace_bytes(M, N)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dy.device)
    elif z is None:
        return dy, None
    nv.call("axn_dgelu_dbias", nv.ptr(dy), nv.ptr(z), nv.ptr(dz), nv.dtype_code(dy.dtype),
            nv.ptr(dbias), M, N, ld, 1 if (accumulate and dbias_out is not None) else 0,
            nv.ptr(ws), ws_bytes, nv.current_stream())
    return (dz if dz is not None else dy), dbias


def _same_2d(name, ref, *others):
    for t in others:
        if t.dtype != ref.dtype or t.shape != ref.shape:
            raise ValueError("%s: operands must match in dtype and shape" % name)


def _swiglu_operands(name, tensors):
    ref = tensors[0]
    if ref.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise TypeError("%s: bf16, fp16 or fp32 expected, got %s" % (name, ref.dtype))
    if ref.dim() != 2 or ref.shape[1] % 8:
        raise ValueError("%s: 2-D operands with a multiple of 8 columns expected, got %s"
                         % (name, tuple(ref.shape)))
    _same_2d(name, ref, *tensors[1:])
    out = []
    for t in tensors:
        if not t.is_contiguous() or t.data_ptr() % 16:
            t = t.contiguous().clone()
        out.append(t)
    return out


def swiglu_fwd(gate, up):
    """silu(gate) * up, the activation of the Llama MLP, in one pass."""
    _require_gpu(gate, up)
    gate, up = _swiglu_operands("swiglu_fwd", [gate, up])
    M, N = gate.shape
    out = torch.empty_like(gate)
    if M == 0:
        return out
    nv.call("axn_swiglu_fwd", nv.ptr(gate), nv.ptr(up), nv.ptr(out), nv.dtype_code(gate.dtype),
            M, N, N, nv.current_stream())
    return out


def gemm_swiglu_supported(M, N, K, dtype):
    """Shapes the one-launch gate/up forward takes (see axn_gemm_swiglu_fwd)."""
    return (dtype in _GEMM16 and M > 0 and M % 256 == 0 and N % 128 == 0 and K % 64 == 0
            and M * K * 2 < 2 ** 31 and N * K * 2 < 2 ** 31)


def gemm_swiglu_fwd(x, w_gate, w_up, save=True):
    """silu(X Wg^T) * (X Wu^T) in one launch.  x [M,K], w_gate / w_up [N,K], bf16 or
    fp16.  Returns (h, gate, up); gate and up (the pre-activations, for the backward
    pass) are None unless `save`.  Callers check `gemm_swiglu_supported` first."""
    _require_gpu(x, w_gate, w_up)
    if not (x.dtype == w_gate.dtype == w_up.dtype):
        raise TypeError("operand dtypes differ: %s, %s, %s" % (x.dtype, w_gate.dtype, w_up.dtype))
    if x.dtype not in _GEMM16:
        raise TypeError("gemm_swiglu_fwd takes bf16 or fp16 operands, got %s" % x.dtype)
    M, K = x.shape
    N = w_gate.shape[0]
    if tuple(w_gate.shape) != (N, K) or tuple(w_up.shape) != (N, K):
        raise ValueError("weights are %s and %s, input has %d features"
                         % (tuple(w_gate.shape), tuple(w_up.shape), K))
    x, ldx = _prep_bf16(x)
    w_gate, ldg = _prep_bf16(w_gate)
    w_up, ldu = _prep_bf16(w_up)
    if ldg != ldu:  # one leading dimension for both weights
        w_gate, w_up = w_gate.contiguous(), w_up.contiguous()
        ldg = K
    h = torch.empty((M, N), dtype=x.dtype, device=x.device)
    gate = torch.empty_like(h) if save else None
    up = torch.empty_like(h) if save else None
    nv.call("axn_gemm_swiglu_fwd", nv.ptr(x), nv.ptr(w_gate), nv.ptr(w_up), nv.ptr(h), nv.ptr(gate),
            nv.ptr(up), nv.dtype_code(x.dtype), M, N, K, ldx, ldg, N, nv.current_stream())
    return h, gate, up


def gemm_dgrad_pair_supported(M, N1, N2, K, dtype):
    """Shapes the one-pass two-term input gradient takes (see axn_gemm_dgrad_pair)."""
    return (dtype in _GEMM16 and M > 0 and M % 128 == 0 and K % 128 == 0 and N1 % 64 == 0
            and N1 >= 128 and N2 % 64 == 0 and N2 >= 64 and M * max(N1, N2) * 2 < 2 ** 31
            and (N1 + N2) * K * 2 < 2 ** 31)


def gemm_dgrad_pair(dy1, w1, dy2, w2):
    """dX = dY1 W1 + dY2 W2 with one rounding.  dy_i [M,N_i], w_i [N_i,K].  Shapes the
    one-pass kernel does not take run as two products and an add."""
    _require_gpu(dy1, w1, dy2, w2)
    if not (dy1.dtype == w1.dtype == dy2.dtype == w2.dtype):
        raise TypeError("operand dtypes differ")
    M, N1 = dy1.shape
    N2, K = w2.shape
    if dy2.shape != (M, N2) or w1.shape != (N1, K):
        raise ValueError("shapes do not fit: %s %s %s %s" % (tuple(dy1.shape), tuple(w1.shape),
                                                            tuple(dy2.shape), tuple(w2.shape)))
    if not gemm_dgrad_pair_supported(M, N1, N2, K, dy1.dtype):
        dx = gemm_dgrad(dy1, w1)
        dx += gemm_dgrad(dy2, w2)
        return dx
    dy1, ld1 = _prep_bf16(dy1)
    dy2, ld2 = _prep_bf16(dy2)
    if ld1 != ld2:
        dy1, dy2 = dy1.contiguous(), dy2.contiguous()
        if N1 != N2:  # one leading dimension for both: pad the narrower into a common stride
            dx = gemm_dgrad(dy1, w1)
            dx += gemm_dgrad(dy2, w2)
            return dx
        ld1 = N1
    if M * ld1 * 2 >= 2 ** 31:
        # row-strided operands (column blocks of a wider buffer) can span 2 GiB where dense
        # ones would not: the one-pass kernel addresses an operand with 32-bit offsets
        dx = gemm_dgrad(dy1, w1)
        dx += gemm_dgrad(dy2, w2)
        return dx
    w1, lw1 = _prep_bf16(w1)
    w2, lw2 = _prep_bf16(w2)
    if lw1 != lw2:
        w1, w2 = w1.contiguous(), w2.contiguous()
        lw1 = K
    dx = torch.empty((M, K), dtype=dy1.dtype, device=dy1.device)
    nv.call("axn_gemm_dgrad_pair", nv.ptr(dy1), nv.ptr(w1), nv.ptr(dy2), nv.ptr(w2), nv.ptr(dx),
            nv.dtype_code(dy1.dtype), M, N1, N2, K, ld1, lw1, K, nv.current_stream())
    return dx


def swiglu_bwd(dout, gate, up):
    """(dgate, dup) for out = silu(gate) * up."""
    _require_gpu(dout, gate, up)
    dout, gate, up = _swiglu_operands("swiglu_bwd", [dout, gate, up])
    M, N = gate.shape
    dgate, dup = torch.empty_like(gate), torch.empty_like(up)
    if M == 0:
        return dgate, dup
    nv.call("axn_swiglu_bwd", nv.ptr(dout), nv.ptr(gate), nv.ptr(up), nv.ptr(dgate), nv.ptr(dup),
            nv.dtype_code(gate.dtype), M, N, N, nv.current_stream())
    return dgate, dup


# ------------------------------------------------------------- embedding -----
def _embedding_table(name, w):
    if w.dim() != 2:
        raise ValueError("%s: 2-D table expected, got %s" % (name, tuple(w.shape)))
    per = 16 // w.element_size()
    if w.shape[1] % per:
        raise ValueError("%s: embedding width must be a multiple of %d for %s, got %d"
                         % (name, per, w.dtype, w.shape[1]))
    if w.stride(1) != 1 or w.stride(0) % per or w.data_ptr() % 16:
        raise ValueError("%s: rows must be contiguous and 16-byte aligned" % name)


def _embedding_ids(ids):
    if ids.dtype not in (torch.int64, torch.int32):
        raise TypeError("embedding: int64 or int32 indices expected, got %s" % ids.dtype)
    return ids.reshape(-1).to(torch.int64).contiguous()


def _embedding_workspace(T, V, device):
    nbytes = nv.load().axn_embedding_workspace_bytes(T, V)
    return torch.empty(nbytes, dtype=torch.uint8, device=device), nbytes


def embedding_fwd(ids, weight, status=None):
    """weight[ids]: rows of the table gathered into ids.shape + (H,).  `status`, a
    device int32 scalar, is set to 1 if an id lies outside the table (such a token
    reads as zeros)."""
    _require_gpu(ids, weight)
    _embedding_table("embedding_fwd", weight)
    flat = _embedding_ids(ids)
    V, H = weight.shape
    out = torch.empty((flat.numel(), H), dtype=weight.dtype, device=weight.device)
    nv.call("axn_embedding_fwd", nv.ptr(flat), nv.ptr(weight), nv.ptr(out),
            nv.dtype_code(weight.dtype), flat.numel(), V, H, weight.stride(0), H,
            nv.ptr(status) if status is not None else None, nv.current_stream())
    return out.view(*ids.shape, H)


def embedding_bwd(ids, dy, num_embeddings, padding_idx=None, scale_grad_by_freq=False, out=None,
                  accumulate=False, out_dtype=None):
    """Dense gradient of the table: row v receives the sum of the dy rows of the tokens
    with id v, added in token order (deterministic).  With `out` and accumulate=True the
    sum is added to out."""
    _require_gpu(ids, dy)
    flat = _embedding_ids(ids)
    H = dy.shape[-1]
    dy2 = dy.reshape(-1, H)
    if dy2.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError("embedding_bwd: bf16 or fp32 gradient expected, got %s" % dy2.dtype)
    if dy2.shape[0] != flat.numel():
        raise ValueError("embedding_bwd: %d tokens but %d gradient rows"
                         % (flat.numel(), dy2.shape[0]))
    if dy2.stride(1) != 1 or dy2.stride(0) != H or dy2.data_ptr() % 16:
        dy2 = dy2.contiguous().clone()
    if out is None:
        if accumulate:
            raise ValueError("embedding_bwd: accumulate needs out")
        out = torch.empty((num_embeddings, H), dtype=out_dtype or dy2.dtype, device=dy2.device)
    _embedding_table("embedding_bwd", out)
    if tuple(out.shape) != (num_embeddings, H):
        raise ValueError("embedding_bwd: out is %s, expected %s"
                         % (tuple(out.shape), (num_embeddings, H)))
    ws, nbytes = _embedding_workspace(flat.numel(), num_embeddings, dy2.device)
    nv.call("axn_embedding_bwd", nv.ptr(flat), nv.ptr(dy2), nv.ptr(out), nv.dtype_code(dy2.dtype),
            nv.dtype_code(out.dtype), flat.numel(), num_embeddings, H, H, out.stride(0),
            -1 if padding_idx is None else padding_idx, int(bool(scale_grad_by_freq)),
            int(bool(accumulate)), nv.ptr(ws), nbytes, nv.current_stream())
    return out


def embedding_renorm_(weight, ids, max_norm, norm_type=2.0):
    """In place: every row of the table that ids names and whose norm exceeds max_norm is
    scaled to max_norm (torch.embedding_renorm_)."""
    _require_gpu(ids, weight)
    _embedding_table("embedding_renorm_", weight)
    if weight.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise TypeError("embedding_renorm_: bf16, fp16 or fp32 table expected, got %s" % weight.dtype)
    flat = _embedding_ids(ids)
    V, H = weight.shape
    ws, nbytes = _embedding_workspace(flat.numel(), V, weight.device)
    nv.call("axn_embedding_renorm", nv.ptr(flat), nv.ptr(weight), nv.dtype_code(weight.dtype),
            flat.numel(), V, H, weight.stride(0), float(max_norm), float(norm_type), nv.ptr(ws),
            nbytes, nv.current_stream())
    return weight


# ---------------------------------------------------------- multi-tensor -----
class ScanResult:
    """Device-resident axn_scan_result (32 bytes) with typed views."""

    def __init__(self, device):
        self.buf = torch.zeros(8, dtype=torch.float32, device=device)

    @property
    def sumsq(self):
        return self.buf.view(torch.float64)[0]

    @property
    def total_norm(self):
        return self.buf[2]

    @property
    def clip_coef(self):
        return self.buf[3]

    @property
    def found_inf(self):
        return self.buf.view(torch.int32)[4]

    def ptr(self):
        return nv.ptr(self.buf)


def _check_list(tensors, dtype=None):
    for t in tensors:
        _require_gpu(t)
        if not t.is_contiguous():
            raise ValueError("multi-tensor kernels need contiguous tensors")
        if dtype is not None and t.dtype != dtype:
            raise TypeError("expected %s, got %s" % (dtype, t.dtype))


def mt_scan(grads, inv_scale=1.0, max_norm=0.0, result=None, accumulate=False, norm_type=2.0,
            workspace=True):
    """Overflow flag, sum of |g|^p, p-norm and clip coefficient of a list of gradients of
    ONE dtype, left on the device in a ScanResult (p = +inf / -inf: the largest / smallest
    |g| in place of the sum).  workspace=False takes the entry point
    that keeps its partial results in the library's own device array (no allocation here
    or there; 2-norm only, sizes up to the array's limit)."""
    if len(grads) == 0:
        raise ValueError("empty gradient list")
    dt = grads[0].dtype
    _check_list(grads, dt)
    device = grads[0].device
    if result is None:
        result = ScanResult(device)
        accumulate = False
    norm_type = float(norm_type)
    if norm_type != norm_type:
        raise ValueError("the norm's order is NaN")
    if not workspace:
        if norm_type != 2.0:
            raise ValueError("the entry point without a workspace computes the 2-norm")
        nv.call("axn_mt_scan_noalloc", nv.ptr_array(grads), nv.size_array(grads), len(grads),
                nv.dtype_code(dt), float(inv_scale), float(max_norm), 1 if accumulate else 0,
                result.ptr(), nv.current_stream())
        return result
    total = sum(g.numel() for g in grads)
    ws_bytes = nv.load().axn_mt_scan_workspace_bytes(len(grads), total)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=device)
    if norm_type == 2.0:
        nv.call("axn_mt_scan", nv.ptr_array(grads), nv.size_array(grads), len(grads),
                nv.dtype_code(dt), float(inv_scale), float(max_norm), 1 if accumulate else 0,
                result.ptr(), nv.ptr(ws), ws_bytes, nv.current_stream())
    else:
        nv.call("axn_mt_scan_norm", nv.ptr_array(grads), nv.size_array(grads), len(grads),
                nv.dtype_code(dt), float(inv_scale), float(max_norm), norm_type,
                1 if accumulate else 0, result.ptr(), nv.ptr(ws), ws_bytes, nv.current_stream())
    return result


def mt_adam(grads, params32, exp_avg, exp_avg_sq, params_lowp, hparams, inv_scale=1.0,
            scan=None):
    """One fused Adam pass over the lists; see axn_mt_adam in include/axn.h."""
    n = len(grads)
    if not (len(params32) == len(exp_avg) == len(exp_avg_sq) == n):
        raise ValueError("list lengths differ")
    if n == 0:
        return
    gdt = grads[0].dtype
    _check_list(grads, gdt)
    _check_list(params32, torch.float32)
    _check_list(exp_avg, torch.float32)
    _check_list(exp_avg_sq, torch.float32)
    plow_arr, pdt = None, nv.BF16
    if params_lowp is not None:
        if len(params_lowp) != n:
            raise ValueError("list lengths differ")
        _check_list(params_lowp, params_lowp[0].dtype)
        pdt = nv.dtype_code(params_lowp[0].dtype)
        plow_arr = nv.ptr_array(params_lowp)
    for g, p in zip(grads, params32):
        if g.numel() != p.numel():
            raise ValueError("gradient and parameter sizes differ")
    nv.call("axn_mt_adam", nv.ptr_array(grads), nv.ptr_array(params32), nv.ptr_array(exp_avg),
            nv.ptr_array(exp_avg_sq), plow_arr, nv.size_array(grads), n, nv.dtype_code(gdt),
            pdt, float(inv_scale), scan.ptr() if scan is not None else None,
            hparams, nv.current_stream())


def mt_scale(grads, inv_scale=1.0, scan=None, use_clip=False):
    """In-place g *= inv_scale (* clip coefficient) on a list of ONE dtype."""
    if len(grads) == 0:
        return
    dt = grads[0].dtype
    _check_list(grads, dt)
    nv.call("axn_mt_scale", nv.ptr_array(grads), nv.size_array(grads), len(grads),
            nv.dtype_code(dt), float(inv_scale), scan.ptr() if scan is not None else None,
            1 if use_clip else 0, nv.current_stream())


def adam_hparams(step, lr, beta1, beta2, eps, weight_decay):
    """Host-side scalars of Adam step number `step` (1-based); bias corrections
    in Python doubles as torch computes them."""
    bc1 = 1.0 - beta1 ** step
    bc2 = 1.0 - beta2 ** step
    return nv.AdamHParams(
        lr_over_bc1=lr / bc1,
        inv_sqrt_bc2=1.0 / (bc2 ** 0.5),
        beta1=beta1,
        one_minus_beta1=1.0 - beta1,
        beta2=beta2,
        one_minus_beta2=1.0 - beta2,
        eps=eps,
        weight_decay=weight_decay,
    )
