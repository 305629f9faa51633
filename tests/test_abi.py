"""The C-ABI shared library: it loads, exports every symbol include/axn.h
declares, and rejects bad arguments with the documented codes before touching
the GPU (so all of this runs on a host without one)."""

import ctypes
import os
import re

import pytest

from axonn_amd import _native as nv

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "axn.h")).read()
    return sorted(set(re.findall(r"AXN_API\s+[\w\s\*]+?\b(axn_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    assert len(names) >= 14
    assert set(names) == set(nv.SYMBOLS), "binding table and header disagree"


def test_library_loads_and_exports_every_declared_symbol():
    lib = ctypes.CDLL(nv.lib_path())
    for name in declared_symbols():
        assert hasattr(lib, name), "libaxn_gfx950.so does not export %s" % name
    assert nv.load().axn_abi_version() == nv.ABI_VERSION


def test_library_is_a_gfx950_code_object():
    blob = open(nv.lib_path(), "rb").read()
    assert b"gfx950" in blob


def test_workspace_queries():
    lib = nv.load()
    assert lib.axn_mt_scan_workspace_bytes(64, 1_300_000_000) >= (1_300_000_000 // 65536 + 64) * 16
    assert lib.axn_mt_scan_workspace_bytes(-1, 5) == 0
    assert lib.axn_dgelu_dbias_workspace_bytes(8192, 5120) == 64 * 5120 * 4
    assert lib.axn_dgelu_dbias_workspace_bytes(0, 8) == 0
    # split contraction: fp32 partial products, only for problems with few 128 x 128 tiles
    assert lib.axn_gemm_workspace_bytes(1, 512, 8192, 3584) == 4 * 512 * 3584 * 4   # dgrad, 112 tiles
    assert lib.axn_gemm_workspace_bytes(0, 512, 8192, 3584) == 2 * 512 * 8192 * 4   # fwd, 128 tiles of 256 x 128, 2 parts
    assert lib.axn_gemm_workspace_bytes(2, 512, 8192, 3584) == 0                    # wgrad, 448 large tiles
    assert lib.axn_gemm_workspace_bytes(0, 4096, 6144, 4096) == 0                   # 384 large tiles: no split
    assert lib.axn_gemm_workspace_bytes(0, 4096, 4096, 4096) == 0                   # one whole round
    assert lib.axn_gemm_workspace_bytes(0, 100, 128, 1024) == 0                     # ragged: no split
    assert lib.axn_gemm_workspace_bytes(0, 128, 128, 512) == 0                      # contraction too short
    assert lib.axn_gemm_workspace_bytes(0, 128, 128, 4096) == 8 * 128 * 128 * 4
    assert lib.axn_gemm_workspace_bytes(3, 128, 128, 4096) == 0 and lib.axn_gemm_workspace_bytes(0, 0, 8, 8) == 0
    # the parts are chosen by estimated time: a short contraction over an output that already has a
    # workgroup for every CU is not split, few tiles take as many parts as still pay for their sums
    assert lib.axn_gemm_workspace_bytes(0, 1024, 4096, 2560) == 0                   # 256 small tiles, 40 stages
    assert lib.axn_gemm_workspace_bytes(0, 256, 2560, 2560) == 4 * 256 * 2560 * 4   # 40 small tiles: 4 parts
    assert lib.axn_gemm_workspace_bytes(0, 512, 4096, 2560) == 2 * 512 * 4096 * 4   # 128 small tiles: 2, not 4
    assert lib.axn_gemm_workspace_bytes(0, 256, 4096, 14336) == 8 * 256 * 4096 * 4  # long contraction: 8
    # embedding: four int32 arrays over the tokens, one over the rows, and the sort's digit
    # counts (17 key bits = two passes of 9 and 8 bits, one count per digit and 512 tokens)
    T, V = 16384, 128256
    need = lib.axn_embedding_workspace_bytes(T, V)
    counts = (512 + 256) * (T // 512) * 4
    assert 4 * T * 4 + V * 4 + counts <= need <= 4 * T * 4 + V * 4 + counts + 4096
    assert lib.axn_embedding_workspace_bytes(0, V) >= V * 4
    assert lib.axn_embedding_workspace_bytes(T, 0) == 0 and lib.axn_embedding_workspace_bytes(-1, V) == 0


def _err():
    return nv.load().axn_last_error().decode()


A = ctypes.c_void_p(0x1000)  # never dereferenced: validation fails first


def test_gemm_argument_errors():
    lib = nv.load()
    f = lib.axn_gemm_fwd
    assert f(None, A, None, A, None, 8, 8, 8, 8, 8, 8, 0, None) == nv.AXN_EINVAL
    assert "null" in _err()
    assert f(A, A, None, A, None, 0, 8, 8, 8, 8, 8, 0, None) == nv.AXN_EINVAL
    assert f(A, A, None, A, None, 8, 12, 8, 8, 8, 16, 0, None) == nv.AXN_ESHAPE
    assert "multiples of 8" in _err()
    assert f(A, A, None, A, None, 8, 8, 8, 4, 8, 8, 0, None) == nv.AXN_EINVAL  # ld < row
    assert f(A, A, None, A, None, 8, 8, 8, 12, 8, 8, 0, None) == nv.AXN_EALIGN  # ld % 8
    assert f(ctypes.c_void_p(0x1004), A, None, A, None, 8, 8, 8, 8, 8, 8, 0, None) == nv.AXN_EALIGN
    assert f(A, A, None, A, None, 8, 8, 8, 8, 8, 8, 7, None) == nv.AXN_EINVAL  # epilogue
    assert f(A, A, None, A, None, 8, 8, 8, 8, 8, 8, nv.EPI_BIAS, None) == nv.AXN_EINVAL
    assert "bias" in _err()
    assert f(A, A, None, A, None, 2 ** 31, 8, 8, 8, 8, 8, 0, None) == nv.AXN_ELIMIT
    assert lib.axn_gemm_dgrad(A, A, None, 8, 8, 8, 8, 8, 8, None) == nv.AXN_EINVAL
    assert lib.axn_gemm_wgrad(A, A, A, 8, 8, 8, 8, 8, 8, 2, nv.BF16, None) == nv.AXN_EINVAL
    assert lib.axn_gemm_wgrad(A, A, A, 8, 8, 8, 8, 8, 8, 0, nv.F16, None) == nv.AXN_EINVAL
    # both gradients in one call: the checks of the two calls
    fb = lib.axn_gemm_bwd
    assert fb(A, A, A, A, A, nv.F32, 8, 8, 8, 8, 8, 8, 8, 8, 0, nv.F32, None) == nv.AXN_EINVAL
    assert fb(A, A, A, A, A, nv.BF16, 8, 8, 8, 8, 8, 8, 8, 8, 2, nv.BF16, None) == nv.AXN_EINVAL
    assert fb(A, A, A, A, A, nv.BF16, 8, 8, 8, 8, 8, 8, 8, 8, 0, nv.F16, None) == nv.AXN_EINVAL
    assert fb(A, A, None, A, A, nv.BF16, 8, 8, 8, 8, 8, 8, 8, 8, 0, nv.BF16, None) == nv.AXN_EINVAL
    assert fb(A, A, A, A, A, nv.BF16, 8, 12, 8, 16, 8, 8, 8, 8, 0, nv.BF16, None) == nv.AXN_ESHAPE
    assert "axn_gemm_bwd" in _err()
    # fp32 result: the promotion of an fp32 bias, so only with a bias epilogue
    fo = lib.axn_gemm_fwd_f32out
    assert fo(A, A, A, A, None, nv.BF16, 8, 8, 8, 8, 8, 8, nv.EPI_NONE, None) == nv.AXN_EINVAL
    assert "BIAS" in _err()
    assert fo(A, A, A, A, None, nv.F32, 8, 8, 8, 8, 8, 8, nv.EPI_BIAS, None) == nv.AXN_EINVAL
    assert fo(A, A, None, A, None, nv.F16, 8, 8, 8, 8, 8, 8, nv.EPI_BIAS, None) == nv.AXN_EINVAL
    assert fo(A, A, A, A, None, nv.BF16, 8, 12, 8, 8, 8, 16, nv.EPI_BIAS, None) == nv.AXN_ESHAPE
    # the fp16 entry points share the checks; dW there is fp16 or fp32, never bf16
    assert lib.axn_gemm_fwd_f16(A, A, None, A, None, 8, 12, 8, 8, 8, 16, 0, None) == nv.AXN_ESHAPE
    assert "axn_gemm_fwd_f16" in _err()
    assert lib.axn_gemm_dgrad_f16(A, None, A, 8, 8, 8, 8, 8, 8, None) == nv.AXN_EINVAL
    assert lib.axn_gemm_wgrad_f16(A, A, A, 8, 8, 8, 8, 8, 8, 0, nv.BF16, None) == nv.AXN_EINVAL
    assert "fp16 or fp32" in _err()
    # split-contraction variants
    ws = lib.axn_gemm_dgrad_ws
    assert ws(A, A, A, nv.F32, 512, 8192, 3584, 8192, 3584, 3584, A, 1 << 30, None) == nv.AXN_EINVAL
    assert ws(A, A, A, nv.BF16, 512, 8192, 3584, 8192, 3584, 3584, A, 1024, None) == nv.AXN_EINVAL
    assert "workspace too small" in _err()
    assert ws(A, A, A, nv.BF16, 512, 8192, 3584, 8192, 3584, 3584, ctypes.c_void_p(0x1008), 1 << 30,
              None) == nv.AXN_EALIGN
    assert ws(A, None, A, nv.BF16, 512, 8192, 3584, 8192, 3584, 3584, A, 1 << 30, None) == nv.AXN_EINVAL
    assert lib.axn_gemm_wgrad_ws(A, A, A, nv.BF16, 8, 8, 8, 8, 8, 8, 0, nv.F16, A, 64, None) == nv.AXN_EINVAL
    assert lib.axn_gemm_fwd_ws(A, A, None, A, None, nv.F16, 8, 12, 8, 8, 8, 16, 0, None, 0, None) == nv.AXN_ESHAPE
    assert lib.axn_gemm_fwd_ws(A, A, None, A, None, nv.F16, 8, 16, 8, 8, 8, 16, 1, None, 0, None) == nv.AXN_EINVAL  # bias missing
    assert lib.axn_gemm_fwd_f32(A, None, None, A, None, 4, 4, 4, 0, None) == nv.AXN_EINVAL
    assert lib.axn_gemm_wgrad_f32(A, A, A, 4, 4, 4, 3, None) == nv.AXN_EINVAL
    assert lib.axn_gemm_dgrad_f32(ctypes.c_void_p(0x1002), A, A, 4, 4, 4, None) == nv.AXN_EALIGN


def test_swiglu_argument_errors():
    lib = nv.load()
    f, b = lib.axn_swiglu_fwd, lib.axn_swiglu_bwd
    assert f(None, A, A, nv.BF16, 8, 8, 8, None) == nv.AXN_EINVAL
    assert f(A, A, A, 7, 8, 8, 8, None) == nv.AXN_EINVAL
    assert f(A, A, A, nv.BF16, 8, 12, 16, None) == nv.AXN_ESHAPE
    assert f(A, A, A, nv.BF16, 8, 8, 4, None) == nv.AXN_EALIGN          # ld < N
    assert f(ctypes.c_void_p(0x1008), A, A, nv.BF16, 8, 8, 8, None) == nv.AXN_EALIGN
    assert b(A, A, A, A, None, nv.BF16, 8, 8, 8, None) == nv.AXN_EINVAL
    assert b(A, A, A, A, A, nv.F32, 0, 8, 8, None) == nv.AXN_EINVAL
    assert "axn_swiglu_bwd" in _err()


def test_gate_up_forward_argument_errors():
    f = nv.load().axn_gemm_swiglu_fwd
    ok = (nv.BF16, 256, 128, 64, 64, 64, 128, None)
    assert f(A, A, None, A, A, A, *ok) == nv.AXN_EINVAL                  # no up weights
    assert f(None, A, A, A, A, A, *ok) == nv.AXN_EINVAL
    assert f(A, A, A, A, A, A, nv.F32, *ok[1:]) == nv.AXN_EINVAL         # 16-bit types only
    assert "bf16 or fp16" in _err()
    assert f(A, A, A, A, ctypes.c_void_p(0x1008), A, *ok) == nv.AXN_EALIGN
    assert f(A, A, A, A, None, None, nv.BF16, 256, 132, 64, 64, 64, 136, None) == nv.AXN_ESHAPE  # N % 8
    # a valid GEMM shape that is not made of whole tiles is refused before any launch
    assert f(A, A, A, A, None, None, nv.BF16, 128, 128, 64, 64, 64, 128, None) == nv.AXN_ESHAPE
    assert "M % 256 == 0" in _err()


def test_dgrad_pair_argument_errors():
    f = nv.load().axn_gemm_dgrad_pair
    tail = (128, 128, 128, 128, 128, 128, None)      # N2, K, lddy, ldw, lddx, stream
    assert f(A, A, None, A, A, nv.BF16, 128, 128, *tail[:-1], None) == nv.AXN_EINVAL   # dY2 missing
    assert f(A, A, A, A, A, nv.F32, 128, 128, *tail) == nv.AXN_EINVAL
    assert f(A, A, A, A, A, nv.BF16, 128, 128, 0, 128, 128, 128, 128, None) == nv.AXN_EINVAL  # N2 = 0
    assert f(A, A, A, A, A, nv.BF16, 128, 128, 12, 128, 128, 128, 128, None) == nv.AXN_ESHAPE  # N2 % 8
    assert f(A, A, A, A, A, nv.BF16, 128, 256, 128, 128, 128, 128, 128, None) == nv.AXN_EINVAL  # lddy < N1
    assert f(A, A, ctypes.c_void_p(0x1008), A, A, nv.BF16, 128, 128, *tail) == nv.AXN_EALIGN
    # valid operands, but the first contraction is shorter than two stages
    assert f(A, A, A, A, A, nv.BF16, 128, 64, 64, 128, 64, 128, 128, None) == nv.AXN_ESHAPE
    assert "gemm_pair" in _err()


def test_embedding_argument_errors():
    lib = nv.load()
    f, b, r = lib.axn_embedding_fwd, lib.axn_embedding_bwd, lib.axn_embedding_renorm
    big = 1 << 30
    assert f(A, None, A, nv.F32, 4, 16, 8, 8, 8, None, None) == nv.AXN_EINVAL
    assert f(None, A, A, nv.F32, 4, 16, 8, 8, 8, None, None) == nv.AXN_EINVAL  # ids missing
    assert f(A, A, A, 7, 4, 16, 8, 8, 8, None, None) == nv.AXN_EINVAL
    assert f(A, A, A, nv.F32, -1, 16, 8, 8, 8, None, None) == nv.AXN_EINVAL
    assert f(A, A, A, nv.F32, 4, 16, 6, 8, 8, None, None) == nv.AXN_ESHAPE      # fp32 rows of 24 bytes
    assert f(A, A, A, nv.BF16, 4, 16, 12, 16, 16, None, None) == nv.AXN_ESHAPE  # bf16 rows of 24 bytes
    assert f(A, A, A, nv.F32, 4, 16, 8, 4, 8, None, None) == nv.AXN_EALIGN      # ldw < H
    assert f(A, A, A, nv.F32, 4, 16, 8, 8, 10, None, None) == nv.AXN_EALIGN
    assert f(A, ctypes.c_void_p(0x1004), A, nv.F32, 4, 16, 8, 8, 8, None, None) == nv.AXN_EALIGN
    assert f(A, A, A, nv.F32, 1 << 31, 16, 8, 8, 8, None, None) == nv.AXN_ELIMIT
    assert "axn_embedding_fwd" in _err()
    assert b(A, A, None, nv.F32, nv.F32, 4, 16, 8, 8, 8, -1, 0, 0, A, big, None) == nv.AXN_EINVAL
    assert b(A, A, A, nv.F16, nv.F32, 4, 16, 8, 8, 8, -1, 0, 0, A, big, None) == nv.AXN_EINVAL
    assert b(A, A, A, nv.BF16, nv.F32, 4, 16, 12, 16, 12, -1, 0, 0, A, big, None) == nv.AXN_ESHAPE
    assert b(A, A, A, nv.F32, nv.F32, 4, 16, 8, 8, 8, 16, 0, 0, A, big, None) == nv.AXN_EINVAL  # padding row
    assert b(A, A, A, nv.F32, nv.F32, 4, 16, 8, 8, 8, -2, 0, 0, A, big, None) == nv.AXN_EINVAL
    assert b(A, A, A, nv.F32, nv.F32, 4, 16, 8, 8, 8, -1, 0, 2, A, big, None) == nv.AXN_EINVAL  # beta
    assert b(A, A, A, nv.F32, nv.F32, 4, 16, 8, 8, 8, -1, 0, 0, A, 64, None) == nv.AXN_EINVAL
    assert "workspace" in _err()
    assert b(A, A, A, nv.F32, nv.F32, 4, 16, 8, 8, 8, -1, 0, 0, None, big, None) == nv.AXN_EINVAL
    assert r(A, None, nv.F32, 4, 16, 8, 8, 1.0, 2.0, A, big, None) == nv.AXN_EINVAL
    assert r(A, A, 7, 4, 16, 8, 8, 1.0, 2.0, A, big, None) == nv.AXN_EINVAL            # unknown dtype
    assert r(A, A, nv.F32, 4, 16, 8, 8, 0.0, 2.0, A, big, None) == nv.AXN_EINVAL
    assert r(A, A, nv.F32, 4, 16, 8, 8, 1.0, -1.0, A, big, None) == nv.AXN_EINVAL
    assert r(A, A, nv.F32, 4, 16, 8, 8, 1.0, 2.0, A, 16, None) == nv.AXN_EINVAL


def test_elementwise_argument_errors():
    lib = nv.load()
    f = lib.axn_dgelu_dbias
    assert f(None, None, None, nv.BF16, A, 8, 8, 8, 0, A, 1024, None) == nv.AXN_EINVAL
    assert f(A, A, None, nv.BF16, A, 8, 8, 8, 0, A, 1024, None) == nv.AXN_EINVAL  # Z without dZ
    assert f(A, None, None, nv.BF16, None, 8, 8, 8, 0, A, 1024, None) == nv.AXN_EINVAL  # nothing to do
    assert f(A, None, None, 7, A, 8, 8, 8, 0, A, 1024, None) == nv.AXN_EINVAL
    assert f(A, None, None, nv.BF16, A, 8, 12, 16, 0, A, 1024, None) == nv.AXN_ESHAPE
    assert f(A, None, None, nv.BF16, A, 8, 8, 8, 0, A, 4, None) == nv.AXN_EINVAL  # workspace too small
    assert "workspace" in _err()


def test_multi_tensor_argument_errors():
    lib = nv.load()
    ptrs = (ctypes.c_void_p * 2)(0x1000, 0x2001)
    sizes = (ctypes.c_int64 * 2)(4, 4)
    res = ctypes.c_void_p(0x3000)
    assert lib.axn_mt_scan(ptrs, sizes, 2, nv.BF16, 1.0, 0.0, 0, res, A, 4096, None) == nv.AXN_EALIGN
    assert "g[1]" in _err()
    sizes[1] = -1
    assert lib.axn_mt_scan(ptrs, sizes, 2, nv.BF16, 1.0, 0.0, 0, res, A, 4096, None) == nv.AXN_EINVAL
    sizes[1] = 0  # empty tensors may carry any pointer
    assert lib.axn_mt_scan(ptrs, sizes, 2, 9, 1.0, 0.0, 0, res, A, 4096, None) == nv.AXN_EINVAL
    assert lib.axn_mt_scan(ptrs, sizes, 2, nv.BF16, 1.0, 0.0, 0, None, A, 4096, None) == nv.AXN_EINVAL
    assert lib.axn_mt_scan(ptrs, sizes, 2, nv.BF16, 1.0, 0.0, 5, res, A, 4096, None) == nv.AXN_EINVAL
    assert lib.axn_mt_scan(ptrs, sizes, 2, nv.BF16, 1.0, 0.0, 0, res, A, 0, None) == nv.AXN_EINVAL
    assert "workspace" in _err()
    hp = nv.AdamHParams()
    assert lib.axn_mt_adam(ptrs, ptrs, ptrs, ptrs, None, sizes, 2, nv.BF16, nv.BF16, 1.0, None,
                           None, None) == nv.AXN_EINVAL
    assert lib.axn_mt_adam(ptrs, None, ptrs, ptrs, None, sizes, 2, nv.BF16, nv.BF16, 1.0, None,
                           hp, None) == nv.AXN_EINVAL
    assert lib.axn_mt_adam(ptrs, ptrs, ptrs, ptrs, ptrs, sizes, 2, nv.BF16, nv.F32, 1.0, None,
                           hp, None) == nv.AXN_EINVAL
    assert lib.axn_mt_scale(ptrs, sizes, 2, nv.BF16, 1.0, None, 1, None) == nv.AXN_EINVAL
    assert "scan" in _err()
    assert lib.axn_mt_scale(ptrs, sizes, -1, nv.BF16, 1.0, None, 0, None) == nv.AXN_EINVAL


def test_scan_variants_argument_errors():
    """The norm's order may be anything but NaN; the entry point without a workspace rejects
    what its built-in array cannot hold before it touches the device."""
    lib = nv.load()
    ptrs = (ctypes.c_void_p * 2)(0x1000, 0x2000)
    sizes = (ctypes.c_int64 * 2)(4, 4)
    res = ctypes.c_void_p(0x3000)
    assert lib.axn_mt_scan_norm(ptrs, sizes, 2, nv.BF16, 1.0, 0.0, float("nan"), 0, res, A, 4096,
                                None) == nv.AXN_EINVAL
    assert "NaN" in _err()
    assert lib.axn_mt_scan_norm(ptrs, sizes, 2, nv.BF16, 1.0, 0.0, 3.0, 0, res, A, 0,
                                None) == nv.AXN_EINVAL          # workspace too small
    assert lib.axn_mt_scan_noalloc(ptrs, sizes, 2, 9, 1.0, 0.0, 0, res, None) == nv.AXN_EINVAL
    assert lib.axn_mt_scan_noalloc(ptrs, sizes, 2, nv.BF16, 1.0, 0.0, 0, None, None) == nv.AXN_EINVAL
    # 65536 chunks of 65536 elements fit the 1 MiB array; three tensors of 2^31 elements do not
    limit = 1048576
    assert lib.axn_mt_scan_workspace_bytes(3, 3 * 2 ** 31) > limit
    ptrs3 = (ctypes.c_void_p * 3)(0x1000, 0x2000, 0x4000)
    sizes3 = (ctypes.c_int64 * 3)(2 ** 31, 2 ** 31, 2 ** 31)
    assert lib.axn_mt_scan_noalloc(ptrs3, sizes3, 3, nv.BF16, 1.0, 0.0, 0, res, None) == nv.AXN_ELIMIT
    assert "scratch" in _err() and "axn_mt_scan" in _err()


def test_probe_library_loads_and_checks_its_arguments():
    """The benchmark-only library (include/axn_probe.h) is built beside the product
    library, exports what its header declares and rejects bad arguments before any launch."""
    text = open(os.path.join(ROOT, "include", "axn_probe.h")).read()
    assert re.findall(r"AXN_PROBE_API\s+int\s+(axn_\w+)\s*\(", text) == ["axn_probe_stream"]
    assert "axn_probe" not in open(os.path.join(ROOT, "include", "axn.h")).read()
    lib = nv.load_probe()
    assert lib.axn_probe_stream(7, A, A, 1024, None) == -1
    assert lib.axn_probe_stream(2, None, A, 1024, None) == -1
    assert lib.axn_probe_stream(1, None, None, 1024, None) == -1
    assert lib.axn_probe_stream(2, ctypes.c_void_p(0x1008), A, 1024, None) == -2
    assert lib.axn_probe_stream(1, None, A, 0, None) == 0     # nothing to do, nothing launched


def test_adam_hparams_struct_layout():
    assert ctypes.sizeof(nv.AdamHParams) == 32
    assert nv.SCAN_RESULT_BYTES == 32


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(nv, "_lib", None)
    monkeypatch.setattr(nv, "_LIB_PATH", "/nonexistent/libaxn_gfx950.so")
    with pytest.raises(ImportError, match="not built"):
        nv.load()
