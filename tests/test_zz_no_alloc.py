"""The gradient scan without a workspace (axn_mt_scan_noalloc: partial results in an
array that is part of the library's device image) against the scan with a caller
workspace (axn_mt_scan): the 32-byte result must be the same bit for bit - overflow flag,
sum of squares, norm, clip coefficient - on two calls in a row, the second on a smaller
input (the array then still holds the first call's partial results), and the size limit
must be refused before anything is launched."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _views(flat, sizes):
    out, off = [], 0
    for n in sizes:
        out.append(flat[off:off + n])
        off += n
    return out


def _scan_pair(grads, inv_scale, max_norm):
    from axonn_amd import _native as nv

    lib = nv.load()
    dev = grads[0].device
    n = len(grads)
    ptrs, sizes = nv.ptr_array(grads), nv.size_array(grads)
    total = sum(g.numel() for g in grads)
    ws_bytes = lib.axn_mt_scan_workspace_bytes(n, total)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    want = torch.full((8,), -1.0, dtype=torch.float32, device=dev)
    got = torch.full((8,), -2.0, dtype=torch.float32, device=dev)
    st = nv.current_stream()
    code = nv.dtype_code(grads[0].dtype)
    nv.check(lib.axn_mt_scan(ptrs, sizes, n, code, inv_scale, max_norm, 0, want.data_ptr(),
                             ws.data_ptr(), ws_bytes, st))
    nv.check(lib.axn_mt_scan_noalloc(ptrs, sizes, n, code, inv_scale, max_norm, 0, got.data_ptr(),
                                     st))
    torch.cuda.synchronize()
    return got, want


def test_scan_without_workspace_equals_scan_with_workspace():
    from axonn_amd import _native as nv

    g = torch.Generator(device="cuda").manual_seed(3)
    # first call: 40 M bf16 gradients in 9 ragged tensors (about 620 chunks of 64 K)
    sizes1 = [5_000_001, 17, 9_999_999, 70_001, 3, 12_345_679, 1, 8_000_000, 4_584_299]
    flat1 = (torch.randn(sum(sizes1), generator=g, device="cuda") * 65.536).bfloat16()
    got, want = _scan_pair(_views(flat1, sizes1), 1.0 / 65536.0, 1.0)
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    assert int(want.view(torch.int32)[4]) == 0 and float(want[2]) > 0.0
    ref = float(torch.sqrt(((flat1.double() / 65536.0) ** 2).sum()))
    assert abs(float(got[2]) - ref) <= 1e-6 * ref
    # second call, smaller input, fp16 with an overflow in its last tensor
    sizes2 = [100_003, 5, 65_536]
    flat2 = torch.randn(sum(sizes2), generator=g, device="cuda").half()
    flat2[-1] = float("inf")
    got2, want2 = _scan_pair(_views(flat2, sizes2), 1.0 / 1024.0, 0.0)
    assert torch.equal(got2.view(torch.int32), want2.view(torch.int32))
    assert int(got2.view(torch.int32)[4]) == 1
    # third: smaller again and finite - nothing of the earlier calls may leak into it
    flat3 = torch.randn(1000, generator=g, device="cuda")
    got3, want3 = _scan_pair([flat3], 1.0, 0.5)
    assert torch.equal(got3.view(torch.int32), want3.view(torch.int32))
    assert int(got3.view(torch.int32)[4]) == 0
    assert abs(float(got3[2]) - float(flat3.double().norm())) <= 1e-6 * float(flat3.norm())
    # accumulate = 1 combines with what the result holds, as axn_mt_scan does
    lib, st = nv.load(), nv.current_stream()
    acc = got3.clone()
    nv.check(lib.axn_mt_scan_noalloc(nv.ptr_array([flat3]), nv.size_array([flat3]), 1, nv.F32, 1.0, 0.5,
                                     1, acc.data_ptr(), st))
    torch.cuda.synchronize()
    assert abs(float(acc.view(torch.float64)[0]) - 2 * float(got3.view(torch.float64)[0])) \
        <= 1e-12 * float(acc.view(torch.float64)[0])


def test_scan_without_workspace_refuses_what_its_array_cannot_hold():
    from axonn_amd import _native as nv

    lib = nv.load()
    t = torch.zeros(16, dtype=torch.bfloat16, device="cuda")
    res = torch.zeros(8, dtype=torch.float32, device="cuda")
    ptrs = (ctypes.c_void_p * 3)(t.data_ptr(), t.data_ptr(), t.data_ptr())
    sizes = (ctypes.c_int64 * 3)(2 ** 31, 2 ** 31, 2 ** 31)     # sizes only: nothing is launched
    rc = lib.axn_mt_scan_noalloc(ptrs, sizes, 3, nv.BF16, 1.0, 0.0, 0, res.data_ptr(),
                                 nv.current_stream())
    assert rc == nv.AXN_ELIMIT
    assert b"scratch" in lib.axn_last_error()
    torch.cuda.synchronize()
    assert not res.any()
