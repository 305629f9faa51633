"""Parity of the embedding kernels (row gather, dense weight gradient, max_norm) and of
the Embedding layer with the CPU oracle, through the C ABI.

Bars: the forward moves rows verbatim - bit-exact.  The fp32 weight gradient adds its
terms in ascending token order in fp32, as the oracle does - bit-exact, also with
repeated ids, padding_idx, accumulation and bf16 gradients (exact in fp32); a bf16
result is the fp32 sum rounded once - bit-exact as well.  With scale_grad_by_freq each
term enters through one fused multiply-add; the oracle imitates that through float64,
which can differ in rare ties: 1 ulp (rtol 2e-7).  max_norm sums a row across lanes in
another order than the float64 oracle: rtol 2e-6 in fp32, one rounding in bf16.

Shapes follow the reference's own test of the layer (axonn/tests/test_intra_layer_emb.py:
B in {2, 4, 8}, S in {1024, 2048}, H in {1024, 2048}, V in {50304, 32000, 128256}); the
largest of them runs against the oracle too (its sums take about a second in numpy).
"""

import numpy as np
import pytest
import torch

from axonn_amd import _native as nv
from oracle import embedding as oe

pytestmark = pytest.mark.gpu


def host(t):
    return t.detach().float().cpu().numpy()


def bf16_round(a):
    return torch.from_numpy(np.asarray(a, np.float32)).bfloat16().float().numpy()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,V,H", [(1, 1, 8), (7, 5, 24), (300, 1000, 520), (4096, 32000, 1024)])
def test_forward_gathers_rows_verbatim(dtype, T, V, H):
    from axonn_amd import ops

    g = torch.Generator(device="cuda").manual_seed(T + V)
    W = torch.randn(V, H, device="cuda", generator=g).to(dtype)
    ids = torch.randint(0, V, (T,), device="cuda", generator=g)
    out = ops.embedding_fwd(ids, W)
    assert out.shape == (T, H) and out.dtype == dtype
    want = oe.embedding_forward(ids.cpu().numpy(), host(W))
    assert np.array_equal(host(out), want)


def test_forward_keeps_the_index_shape_and_takes_strided_tables_and_int32_ids():
    from axonn_amd import ops

    torch.manual_seed(0)
    big = torch.randn(40, 64, device="cuda")
    W = big[:, 16:48]  # 40 x 32 view, row stride 64, 16-byte aligned
    ids = torch.randint(0, 40, (3, 5, 2), device="cuda", dtype=torch.int32)
    out = ops.embedding_fwd(ids, W)
    assert out.shape == (3, 5, 2, 32)
    assert torch.equal(out, W[ids.long()])
    empty = ops.embedding_fwd(torch.zeros(0, dtype=torch.long, device="cuda"), W)
    assert empty.shape == (0, 32)


def test_ids_outside_the_table_read_zeros_and_raise_the_status_word():
    from axonn_amd import ops

    W = torch.randn(16, 8, device="cuda")
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    good = torch.tensor([0, 15, 3], device="cuda")
    ops.embedding_fwd(good, W, status=status)
    assert int(status) == 0
    bad = torch.tensor([0, 16, -1, 3], device="cuda")
    out = ops.embedding_fwd(bad, W, status=status)
    assert int(status) == 1
    assert np.array_equal(host(out), oe.embedding_forward(bad.cpu().numpy(), host(W)))
    # backward skips them
    dy = torch.randn(4, 8, device="cuda")
    dW = ops.embedding_bwd(bad, dy, 16)
    assert np.array_equal(host(dW), oe.embedding_backward(bad.cpu().numpy(), host(dy), 16))


@pytest.mark.parametrize("dy_dtype,dw_dtype", [(torch.float32, torch.float32),
                                               (torch.bfloat16, torch.float32),
                                               (torch.bfloat16, torch.bfloat16),
                                               (torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("T,V,H", [(1, 1, 8), (64, 5, 24), (1000, 300, 520), (4096, 32000, 1024)])
def test_backward_equals_the_sequential_sum_bit_for_bit(dy_dtype, dw_dtype, T, V, H):
    from axonn_amd import ops

    g = torch.Generator(device="cuda").manual_seed(T * 3 + V)
    ids = torch.randint(0, V, (T,), device="cuda", generator=g)
    dy = (torch.randn(T, H, device="cuda", generator=g) * 0.01).to(dy_dtype)
    dW = ops.embedding_bwd(ids, dy, V, out_dtype=dw_dtype)
    assert dW.shape == (V, H) and dW.dtype == dw_dtype
    want = oe.embedding_backward(ids.cpu().numpy(), host(dy), V)
    if dw_dtype == torch.bfloat16:
        want = bf16_round(want)
    assert np.array_equal(host(dW), want)


@pytest.mark.parametrize("T,V", [(700, 3), (513, 1023), (5000, 1024), (40000, 70000), (3000, (1 << 21) + 5),
                                 (100000, 200), ((1 << 18) + 77, 5000), (300000, 1 << 20)])
def test_backward_over_every_shape_of_the_sort(T, V):
    """The token positions are sorted by id with the library's own radix sort: one pass
    (up to 10 key bits), two (11 to 20) and three (21 and more), token counts that end
    inside a segment, both segment lengths (128 slots up to 2^18 tokens, 512 beyond), and ids
    drawn from a few hot rows so that runs cross segments.  The row sums depend on the order of their terms: equal to the sequential
    loop bit for bit means every row's tokens came out in ascending order."""
    from axonn_amd import ops

    g = torch.Generator(device="cuda").manual_seed(T + V)
    ids = torch.randint(0, V, (T,), device="cuda", generator=g)
    hot = torch.randint(0, V, (7,), device="cuda", generator=g)
    pick = torch.randint(0, 7, (T,), device="cuda", generator=g)
    ids = torch.where(torch.rand(T, device="cuda", generator=g) < 0.3, hot[pick], ids)
    ids[-1] = V - 1
    ids[0] = 0
    dy = torch.randn(T, 8, device="cuda", generator=g)
    dW = ops.embedding_bwd(ids, dy, V)
    want = oe.embedding_backward(ids.cpu().numpy(), host(dy), V)
    assert np.array_equal(host(dW), want)


def test_backward_padding_row_repeated_ids_and_determinism():
    """A tenth of the tokens name one row, another tenth the padding row; the sum of 400
    terms depends on its order, and the kernel's order is the token order."""
    from axonn_amd import ops

    torch.manual_seed(4)
    T, V, H = 4000, 64, 136
    ids = torch.randint(0, V, (T,), device="cuda")
    ids[::10] = 7
    ids[5::10] = 9
    dy = torch.randn(T, H, device="cuda")
    dW = ops.embedding_bwd(ids, dy, V, padding_idx=9)
    want = oe.embedding_backward(ids.cpu().numpy(), host(dy), V, padding_idx=9)
    assert np.array_equal(host(dW), want)
    assert not host(dW)[9].any()
    # the order matters at this length: a reversed sum differs somewhere
    rev = oe.embedding_backward(ids.cpu().numpy()[::-1], host(dy)[::-1], V, padding_idx=9)
    assert not np.array_equal(rev, want)
    for _ in range(3):
        assert torch.equal(ops.embedding_bwd(ids, dy, V, padding_idx=9), dW)


def test_backward_accumulates_into_an_existing_gradient():
    from axonn_amd import ops

    torch.manual_seed(6)
    T, V, H = 500, 200, 64
    ids = torch.randint(0, V, (T,), device="cuda")
    ids[ids == 11] = 12  # row 11 receives nothing: it must keep its old value
    dy = torch.randn(T, H, device="cuda")
    old = torch.randn(V, H, device="cuda")
    acc = old.clone()
    ops.embedding_bwd(ids, dy, V, padding_idx=3, out=acc, accumulate=True)
    want = oe.embedding_backward(ids.cpu().numpy(), host(dy), V, padding_idx=3, accumulate_into=host(old))
    assert np.array_equal(host(acc), want)
    assert torch.equal(acc[11], old[11]) and torch.equal(acc[3], old[3])
    # no tokens at all: beta = 0 clears the gradient, beta = 1 leaves it
    none = torch.zeros(0, dtype=torch.long, device="cuda")
    assert not ops.embedding_bwd(none, torch.zeros(0, H, device="cuda"), V).any()
    keep = old.clone()
    ops.embedding_bwd(none, torch.zeros(0, H, device="cuda"), V, out=keep, accumulate=True)
    assert torch.equal(keep, old)


@pytest.mark.parametrize("dy_dtype", [torch.float32, torch.bfloat16])
def test_backward_scaled_by_frequency(dy_dtype):
    from axonn_amd import ops

    torch.manual_seed(8)
    T, V, H = 3000, 97, 72
    ids = torch.randint(0, V, (T,), device="cuda")
    dy = torch.randn(T, H, device="cuda").to(dy_dtype)
    dW = ops.embedding_bwd(ids, dy, V, padding_idx=0, scale_grad_by_freq=True, out_dtype=torch.float32)
    want = oe.embedding_backward(ids.cpu().numpy(), host(dy), V, padding_idx=0, scale_grad_by_freq=True)
    assert np.allclose(host(dW), want, rtol=2e-7, atol=1e-9)
    exact = oe.embedding_backward_f64(ids.cpu().numpy(), host(dy), V, padding_idx=0, scale_grad_by_freq=True)
    assert np.allclose(host(dW), exact, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("norm_type", [1.0, 2.0, 3.0])
def test_max_norm_scales_each_named_row_once(dtype, norm_type):
    from axonn_amd import ops

    torch.manual_seed(9)
    V, H = 300, 264
    W = torch.randn(V, H, device="cuda").to(dtype)
    W[5] *= 0.001
    ids = torch.randint(0, 40, (8, 50), device="cuda")  # rows 40.. are never named
    ids[0, :10] = 5
    before = host(W).copy()
    ops.embedding_renorm_(W, ids, 2.0, norm_type)
    want = oe.embedding_renorm(before, ids.cpu().numpy(), 2.0, norm_type)
    if dtype == torch.float32:
        assert np.allclose(host(W), want, rtol=2e-6, atol=1e-9)
    elif dtype == torch.float16:
        assert np.allclose(host(W), want, rtol=2 ** -11 + 1e-5, atol=1e-7)
    else:
        # the scaled row is rounded to bf16 once; the scale itself carries fp32 rounding
        assert np.allclose(host(W), want, rtol=2 ** -8 + 1e-5, atol=1e-9)
    assert np.array_equal(host(W)[40:], before[40:]) and np.array_equal(host(W)[5], before[5])


@pytest.mark.parametrize("B,S,H,V", [(2, 1024, 1024, 50304), (8, 2048, 2048, 128256)])
def test_layer_matches_torch_embedding_at_the_reference_test_shapes(B, S, H, V):
    """What axonn/tests/test_intra_layer_emb.py checks on its grid, on the 1 x 1 x 1 grid:
    the layer loaded from torch.nn.Embedding's state dict gives the same output and the
    same weight gradient (the test's tolerance is torch.allclose's default)."""
    from axonn_amd.intra_layer import Embedding

    torch.manual_seed(42)
    X = torch.randint(0, V, (B, S), device="cuda")
    dY = torch.randn(B, S, H, device="cuda") * 0.01
    layer = Embedding(V, H).cuda()
    seq = torch.nn.Embedding(V, H).cuda()
    layer.load_state_dict(seq.state_dict())
    layer.load_state_dict(layer.state_dict())
    Y = layer(X)
    assert torch.equal(Y, seq(X))
    Y.backward(dY)
    seq(X).backward(dY)
    got = layer.weight.grad.view(V, H)
    assert torch.allclose(got, seq.weight.grad)
    want = oe.embedding_backward(X.cpu().numpy(), host(dY), V)
    assert np.array_equal(host(got), want)


def test_layer_arguments_reach_the_kernels():
    from axonn_amd.intra_layer import Embedding

    torch.manual_seed(1)
    V, H = 120, 32
    layer = Embedding(V, H, padding_idx=2, max_norm=1.0, scale_grad_by_freq=True).cuda()
    seq = torch.nn.Embedding(V, H, padding_idx=2, max_norm=1.0, scale_grad_by_freq=True).cuda()
    layer.load_state_dict(seq.state_dict())
    X = torch.randint(0, 30, (4, 25), device="cuda")
    Y = layer(X)
    Ys = seq(X)
    assert torch.allclose(Y, Ys, rtol=1e-6, atol=1e-7)
    assert torch.allclose(layer.weight.view(V, H), seq.weight, rtol=1e-6, atol=1e-7)  # renormalised in place
    dY = torch.randn(4, 25, H, device="cuda")
    Y.backward(dY)
    Ys.backward(dY)
    assert torch.allclose(layer.weight.grad.view(V, H), seq.weight.grad, rtol=1e-5, atol=1e-6)
    assert not layer.weight.grad.view(V, H)[2].any()
    # bf16 table: gradient in bf16
    lb = Embedding(V, H).cuda().bfloat16()
    out = lb(X)
    out.backward(dY.bfloat16())
    assert out.dtype == torch.bfloat16 and lb.weight.grad.dtype == torch.bfloat16
    want = bf16_round(oe.embedding_backward(X.cpu().numpy(), host(dY.bfloat16()), V))
    assert np.array_equal(host(lb.weight.grad.view(V, H)), want)


def test_bad_arguments_raise_before_any_launch():
    from axonn_amd import ops

    W = torch.randn(16, 8, device="cuda")
    ids = torch.zeros(4, dtype=torch.long, device="cuda")
    with pytest.raises(ValueError, match="multiple of 4"):
        ops.embedding_fwd(ids, torch.randn(16, 6, device="cuda"))
    with pytest.raises(TypeError, match="indices"):
        ops.embedding_fwd(ids.float(), W)
    with pytest.raises(ValueError, match="gradient rows"):
        ops.embedding_bwd(ids, torch.randn(5, 8, device="cuda"), 16)
    with pytest.raises(nv.AxnError, match="padding_idx"):
        ops.embedding_bwd(ids, torch.randn(4, 8, device="cuda"), 16, padding_idx=16)
    with pytest.raises(nv.AxnError, match="max_norm"):
        ops.embedding_renorm_(W, ids, -1.0)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.embedding_fwd(ids.cpu(), W.cpu())


def test_table_of_more_than_two_to_the_31_elements():
    """Row offsets are 64-bit: a 2^18 x 8192 bf16 table (4 GiB) with ids in its last rows."""
    from axonn_amd import ops

    V, H, T = 1 << 18, 8192, 96
    g = torch.Generator(device="cuda").manual_seed(7)
    W = torch.empty(V, H, device="cuda", dtype=torch.bfloat16)
    W[-4096:].normal_(generator=g)
    ids = torch.randint(V - 4096, V, (T,), device="cuda", generator=g)
    ids[:8] = V - 1
    out = ops.embedding_fwd(ids, W)
    assert torch.equal(out, W[ids])
    dy = torch.randn(T, H, device="cuda", generator=g).bfloat16()
    dW = ops.embedding_bwd(ids, dy, V, out_dtype=torch.float32)
    rows = torch.unique(ids)
    base = V - 4096
    want = oe.embedding_backward((ids - base).cpu().numpy(), host(dy), 4096)
    assert np.array_equal(host(dW[base:]), want)
    assert not dW[:base:4099].any() and len(rows) > 50
    del W, dW
    torch.cuda.empty_cache()
