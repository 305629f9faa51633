"""ctypes binding of libaxn_gfx950.so (the C ABI declared in include/axn.h).

The library holds every kernel of the hot path; this module only marshals
pointers, sizes and the current HIP stream.  There is no fallback: when the
library is missing, loading raises, and every compute entry point needs a GPU.
"""

import ctypes
import os
import threading

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libaxn_gfx950.so")

AXN_OK = 0
AXN_EINVAL = -1
AXN_EALIGN = -2
AXN_ESHAPE = -3
AXN_EHIP = -4
AXN_ELIMIT = -5

BF16, F16, F32 = 0, 1, 2
EPI_NONE, EPI_BIAS, EPI_BIAS_GELU, EPI_GELU = 0, 1, 2, 3

ABI_VERSION = 12

# Every symbol include/axn.h declares: name -> (restype, argtypes)
_c = ctypes
_vp, _i64, _int, _f32, _sz = _c.c_void_p, _c.c_int64, _c.c_int, _c.c_float, _c.c_size_t
_pp, _pi64 = _c.POINTER(_c.c_void_p), _c.POINTER(_c.c_int64)


class AdamHParams(ctypes.Structure):
    """Mirror of axn_adam_hparams."""

    _fields_ = [
        ("lr_over_bc1", _f32),
        ("inv_sqrt_bc2", _f32),
        ("beta1", _f32),
        ("one_minus_beta1", _f32),
        ("beta2", _f32),
        ("one_minus_beta2", _f32),
        ("eps", _f32),
        ("weight_decay", _f32),
    ]


SCAN_RESULT_BYTES = 32  # sizeof(axn_scan_result)

SYMBOLS = {
    "axn_abi_version": (_int, []),
    "axn_last_error": (_c.c_char_p, []),
    "axn_gemm_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _int, _vp]),
    "axn_gemm_dgrad": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp]),
    "axn_gemm_wgrad": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "axn_gemm_fwd_f16": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _int,
                                _vp]),
    "axn_gemm_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                            _int, _int, _vp]),
    "axn_gemm_fwd_f32out": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _i64, _i64,
                                   _int, _vp]),
    "axn_gemm_dgrad_f16": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp]),
    "axn_gemm_wgrad_f16": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int,
                                  _vp]),
    "axn_gemm_workspace_bytes": (_sz, [_int, _i64, _i64, _i64]),
    "axn_gemm_fwd_ws": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _i64, _i64, _int,
                               _vp, _sz, _vp]),
    "axn_gemm_dgrad_ws": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _i64, _i64, _vp, _sz,
                                 _vp]),
    "axn_gemm_wgrad_ws": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _i64, _i64, _int,
                                 _int, _vp, _sz, _vp]),
    "axn_dgelu_dbias": (_int, [_vp, _vp, _vp, _int, _vp, _i64, _i64, _i64, _int, _vp, _sz, _vp]),
    "axn_gemm_swiglu_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _i64, _i64, _vp]),
    "axn_gemm_dgrad_pair": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _vp]),
    "axn_dgelu_dbias_workspace_bytes": (_sz, [_i64, _i64]),
    "axn_swiglu_fwd": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _i64, _vp]),
    "axn_swiglu_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _vp]),
    "axn_embedding_fwd": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _i64, _vp, _vp]),
    "axn_embedding_workspace_bytes": (_sz, [_i64, _i64]),
    "axn_embedding_bwd": (_int, [_vp, _vp, _vp, _int, _int, _i64, _i64, _i64, _i64, _i64, _i64,
                                 _int, _int, _vp, _sz, _vp]),
    "axn_embedding_renorm": (_int, [_vp, _vp, _int, _i64, _i64, _i64, _i64, _f32, _f32, _vp, _sz,
                                    _vp]),
    "axn_gemm_fwd_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "axn_gemm_dgrad_f32": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "axn_gemm_wgrad_f32": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "axn_mt_scan_workspace_bytes": (_sz, [_i64, _i64]),
    "axn_mt_scan": (_int, [_pp, _pi64, _i64, _int, _f32, _f32, _int, _vp, _vp, _sz, _vp]),
    "axn_mt_scan_norm": (_int, [_pp, _pi64, _i64, _int, _f32, _f32, _f32, _int, _vp, _vp, _sz, _vp]),
    "axn_mt_scan_noalloc": (_int, [_pp, _pi64, _i64, _int, _f32, _f32, _int, _vp, _vp]),
    "axn_mt_adam": (_int, [_pp, _pp, _pp, _pp, _pp, _pi64, _i64, _int, _int, _f32, _vp,
                           _c.POINTER(AdamHParams), _vp]),
    "axn_mt_scale": (_int, [_pp, _pi64, _i64, _int, _f32, _vp, _int, _vp]),
}

_lib = None
_probe_lib = None
_lock = threading.Lock()


class AxnError(RuntimeError):
    """A call into libaxn_gfx950.so returned a non-zero status."""

    def __init__(self, code, message):
        super().__init__("libaxn_gfx950 error %d: %s" % (code, message))
        self.code = code


def lib_path():
    return _LIB_PATH


def load():
    """Loads the library once and types its entry points.  Raises if it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(_LIB_PATH):
            raise ImportError(
                "libaxn_gfx950.so is not built (expected at %s); run "
                "`python -m axonn_amd.csrc.build`" % _LIB_PATH
            )
        try:
            # PyTorch ships its own HIP runtime with the same soname; importing it
            # first makes this library bind to the runtime that owns torch's
            # streams and allocations.
            import torch  # noqa: F401
        except ImportError:
            pass
        lib = ctypes.CDLL(_LIB_PATH)
        for name, (restype, argtypes) in SYMBOLS.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.axn_abi_version() != ABI_VERSION:
            raise ImportError(
                "libaxn_gfx950.so has ABI version %d, this package needs %d"
                % (lib.axn_abi_version(), ABI_VERSION)
            )
        _lib = lib
    return _lib


def load_probe():
    """The benchmark-only library of streaming yardsticks (include/axn_probe.h)."""
    global _probe_lib
    if _probe_lib is None:
        path = os.path.join(os.path.dirname(_LIB_PATH), "libaxn_probe_gfx950.so")
        if not os.path.exists(path):
            raise ImportError("libaxn_probe_gfx950.so is not built (expected at %s); run "
                              "`python -m axonn_amd.csrc.build`" % path)
        load()  # binds the HIP runtime torch uses first
        lib = ctypes.CDLL(path)
        lib.axn_probe_stream.restype = _int
        lib.axn_probe_stream.argtypes = [_int, _vp, _vp, _sz, _vp]
        _probe_lib = lib
    return _probe_lib


def check(rc):
    if rc != AXN_OK:
        msg = load().axn_last_error()
        raise AxnError(rc, msg.decode("utf-8", "replace") if msg else "")


def call(name, *args):
    """Calls an int-returning entry point and raises AxnError on failure."""
    check(getattr(load(), name)(*args))


_DTYPE_CODES = {}


def dtype_code(torch_dtype):
    if not _DTYPE_CODES:
        import torch

        _DTYPE_CODES.update({torch.bfloat16: BF16, torch.float16: F16, torch.float32: F32})
    code = _DTYPE_CODES.get(torch_dtype)
    if code is None:
        raise TypeError("unsupported dtype %s (bf16, fp16 or fp32 expected)" % torch_dtype)
    return code


def current_stream():
    """torch's current stream on the current device as a `hipStream_t`."""
    import torch

    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if raw is not None:  # the handle itself, without building a Stream object (5-10 us less per call)
        return ctypes.c_void_p(raw(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(t):
    """Device pointer of a tensor (None -> NULL)."""
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def ptr_array(tensors):
    arr = (ctypes.c_void_p * max(len(tensors), 1))()
    for i, t in enumerate(tensors):
        arr[i] = t.data_ptr()
    return arr


def size_array(tensors):
    arr = (ctypes.c_int64 * max(len(tensors), 1))()
    for i, t in enumerate(tensors):
        arr[i] = t.numel()
    return arr
