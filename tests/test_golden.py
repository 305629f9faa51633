"""Oracle and HIP path against the committed golden fixtures
(tests/golden/*.npz, written by tests/golden/make_golden.py from torch's own
routines on the reference's test shapes)."""

import os

import numpy as np
import pytest
import torch

from oracle import linear as ol
from oracle import optim as oo


@pytest.fixture(scope="module")
def lin(golden_dir):
    return np.load(os.path.join(golden_dir, "linear_f64.npz"))


@pytest.fixture(scope="module")
def opt(golden_dir):
    return np.load(os.path.join(golden_dir, "optimizer_f32.npz"))


SHAPES = [(32, 64), (16, 128), (2, 256)]


def _f64(bits):
    return ol.bf16_to_f32(bits).astype(np.float64)


@pytest.mark.parametrize("idx", [0, 1, 2])
def test_oracle_linear_reproduces_golden(lin, idx):
    B, H = SHAPES[idx]
    X, W, dY = _f64(lin[f"c{idx}_X"]), _f64(lin[f"c{idx}_W"]), _f64(lin[f"c{idx}_dY"])
    b = lin[f"c{idx}_b"].astype(np.float64)
    y, _ = ol.linear_forward(X, W.reshape(-1), (H, H), bias=b)
    bw = ol.linear_backward(X, W.reshape(-1), (H, H), dY, has_bias=True)
    assert np.allclose(y, lin[f"c{idx}_Y"], rtol=1e-12, atol=1e-16)
    assert np.allclose(bw["dx"], lin[f"c{idx}_dX"], rtol=1e-12, atol=1e-16)
    dw = bw["dw"].reshape(H, H)
    assert np.allclose(dw, lin[f"c{idx}_dW"], rtol=1e-6, atol=1e-12)  # stored in float32
    assert np.allclose(dw.sum(1), lin[f"c{idx}_dW_rowsum"], rtol=1e-11, atol=1e-16)
    assert np.allclose(dw.sum(0), lin[f"c{idx}_dW_colsum"], rtol=1e-11, atol=1e-16)
    assert np.allclose(bw["db"], lin[f"c{idx}_db"], rtol=1e-12, atol=1e-16)


def test_oracle_gelu_layer_reproduces_golden(lin):
    X, W, dY = _f64(lin["g_X"]), _f64(lin["g_W"]), _f64(lin["g_dY"])
    b = lin["g_b"].astype(np.float64)
    y, z = ol.linear_forward(X, W.reshape(-1), (56, 40), bias=b, activation="gelu")
    bw = ol.linear_backward(X, W.reshape(-1), (56, 40), dY, z=z, activation="gelu", has_bias=True)
    assert np.allclose(z, lin["g_Z"], rtol=1e-12) and np.allclose(y, lin["g_Y"], rtol=1e-12)
    assert np.allclose(bw["dx"], lin["g_dX"], rtol=1e-11, atol=1e-15)
    assert np.allclose(bw["dw"].reshape(56, 40), lin["g_dW"], rtol=1e-11, atol=1e-15)
    assert np.allclose(bw["db"], lin["g_db"], rtol=1e-11, atol=1e-15)


def test_oracle_bf16_conversion_reproduces_golden(opt):
    assert np.array_equal(ol.bf16_bits(opt["cvt_f32"]), opt["cvt_bf16_bits"].view(np.uint16))


def _split(flat, sizes):
    out, off = [], 0
    for n in sizes:
        out.append(flat[off:off + n].copy())
        off += n
    return out


def test_oracle_optimizer_reproduces_golden(opt):
    sizes = [int(n) for n in opt["sizes"]]
    p = _split(opt["p0"], sizes)
    m = [np.zeros(n, np.float32) for n in sizes]
    v = [np.zeros(n, np.float32) for n in sizes]
    for step in (1, 2, 3):
        g = _split(opt[f"g{step}"], sizes)
        total, clipped = oo.clip_grad_norm_(g, 0.01, "f32")
        assert abs(total - float(opt[f"norm{step}"])) <= 1e-6 * total
        assert np.allclose(np.concatenate(clipped), opt[f"gclip{step}"], rtol=3e-7, atol=0)
        newp, newm, newv = [], [], []
        for gi, pi, mi, vi in zip(_split(opt[f"gclip{step}"], sizes), p, m, v):
            a, b, c = oo.adam_update(pi, gi, mi, vi, step, weight_decay=0.01)
            newp.append(a)
            newm.append(b)
            newv.append(c)
        p, m, v = newp, newm, newv
        ref = opt[f"p{step}"]
        got = np.concatenate(p)
        assert np.max(np.abs(got - ref)) / np.max(np.abs(ref)) <= 1e-6
        assert np.allclose(np.concatenate(m), opt[f"m{step}"], rtol=1e-6, atol=1e-10)
        assert np.allclose(np.concatenate(v), opt[f"v{step}"], rtol=1e-6, atol=1e-15)
        # cast-back: equal bits wherever the fp32 values are equal
        same = got == ref
        assert same.mean() > 0.5
        assert np.array_equal(ol.bf16_bits(got)[same], opt[f"pbf{step}"].view(np.uint16)[same])


# ------------------------------------------------------------------ GPU ------
def _dev_bf16(bits):
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).cuda()


def _rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


@pytest.mark.gpu
@pytest.mark.parametrize("idx", [0, 1, 2])
def test_hip_linear_reproduces_golden(lin, idx):
    """bf16 kernels on the golden inputs: <= 1e-2 relative (bf16 results, fp32
    accumulate); in practice the only error is the final rounding, ~2e-3."""
    from axonn_amd import ops

    X, W, dY = _dev_bf16(lin[f"c{idx}_X"]), _dev_bf16(lin[f"c{idx}_W"]), _dev_bf16(lin[f"c{idx}_dY"])
    b = torch.from_numpy(lin[f"c{idx}_b"]).cuda()
    y, _ = ops.gemm_fwd(X, W, bias=b)
    dx = ops.gemm_dgrad(dY, W)
    dw32 = ops.gemm_wgrad(dY, X, out_dtype=torch.float32)
    dw16 = ops.gemm_wgrad(dY, X)
    _, db = ops.dgelu_dbias(dY, None, want_dbias=True)
    assert _rel(y.float().cpu().numpy(), lin[f"c{idx}_Y"]) < 1e-2
    assert _rel(dx.float().cpu().numpy(), lin[f"c{idx}_dX"]) < 1e-2
    assert _rel(dw16.float().cpu().numpy(), lin[f"c{idx}_dW"]) < 1e-2
    # fp32 output: only fp32 accumulation error is left
    assert _rel(dw32.cpu().numpy(), lin[f"c{idx}_dW"]) < 1e-5
    assert _rel(db.cpu().numpy(), lin[f"c{idx}_db"]) < 1e-5


@pytest.mark.gpu
def test_hip_gelu_layer_reproduces_golden(lin):
    from axonn_amd import ops

    X, W, dY = _dev_bf16(lin["g_X"]), _dev_bf16(lin["g_W"]), _dev_bf16(lin["g_dY"])
    b = torch.from_numpy(lin["g_b"]).cuda()
    y, z = ops.gemm_fwd(X, W, bias=b, activation="gelu", save_z=True)
    assert _rel(z.float().cpu().numpy(), lin["g_Z"]) < 1e-2
    assert _rel(y.float().cpu().numpy(), lin["g_Y"]) < 1e-2
    dz, db = ops.dgelu_dbias(dY, z, want_dbias=True)
    dx = ops.gemm_dgrad(dz, W)
    dw = ops.gemm_wgrad(dz, X, out_dtype=torch.float32)
    assert _rel(dx.float().cpu().numpy(), lin["g_dX"]) < 1e-2
    assert _rel(dw.cpu().numpy(), lin["g_dW"]) < 1e-2
    assert _rel(db.cpu().numpy(), lin["g_db"]) < 1e-2


@pytest.mark.gpu
def test_hip_optimizer_reproduces_golden(opt):
    """fp32 gradients through scan (norm, clip) + Adam with weight decay, three
    steps, on ragged views of flat buffers: master weights within 1e-6."""
    from axonn_amd import ops

    sizes = [int(n) for n in opt["sizes"]]
    total = sum(sizes)
    flat_p = torch.from_numpy(opt["p0"].copy()).cuda()
    flat_m = torch.zeros(total, device="cuda")
    flat_v = torch.zeros(total, device="cuda")
    flat_pl = torch.zeros(total, dtype=torch.bfloat16, device="cuda")

    def views(flat):
        out, off = [], 0
        for n in sizes:
            out.append(flat[off:off + n])
            off += n
        return out

    for step in (1, 2, 3):
        flat_g = torch.from_numpy(opt[f"g{step}"].copy()).cuda()
        scan = ops.mt_scan(views(flat_g), 1.0, 0.01)
        assert int(scan.found_inf.item()) == 0
        assert abs(float(scan.total_norm.item()) - float(opt[f"norm{step}"])) <= 1e-6 * float(opt[f"norm{step}"])
        hp = ops.adam_hparams(step, 1e-3, 0.9, 0.999, 1e-8, 0.01)
        ops.mt_adam(views(flat_g), views(flat_p), views(flat_m), views(flat_v), views(flat_pl), hp,
                    inv_scale=1.0, scan=scan)
        ref = opt[f"p{step}"]
        got = flat_p.cpu().numpy()
        assert np.max(np.abs(got - ref)) / np.max(np.abs(ref)) <= 1e-6
        assert np.allclose(flat_m.cpu().numpy(), opt[f"m{step}"], rtol=1e-5, atol=1e-9)
        assert np.allclose(flat_v.cpu().numpy(), opt[f"v{step}"], rtol=1e-5, atol=1e-14)
        # the low-precision copy is exactly the rounding of the master weights
        want_bits = ol.bf16_bits(got)
        assert np.array_equal(flat_pl.view(torch.int16).cpu().numpy().view(np.uint16), want_bits)


# ------------------------------------------------------------------ embedding
@pytest.fixture(scope="module")
def emb(golden_dir):
    return np.load(os.path.join(golden_dir, "embedding_f64.npz"))


EMB_CASES = [("plain", None, False), ("pad", 5, False), ("freq", 5, True)]


@pytest.mark.parametrize("tag,padding_idx,scale", EMB_CASES)
def test_oracle_embedding_reproduces_golden(emb, tag, padding_idx, scale):
    """The fixture holds torch's float64 results; the oracle adds in fp32 in token order,
    so it agrees to fp32 rounding of sums of at most 8 terms of size 0.01."""
    from oracle import embedding as oe

    V = emb["W"].shape[0]
    assert np.array_equal(oe.embedding_forward(emb["ids"], emb["W"]), emb[tag + "_Y"].astype(np.float32))
    dW = oe.embedding_backward(emb["ids"], emb["dY"], V, padding_idx, scale)
    assert np.allclose(dW, emb[tag + "_dW"], rtol=1e-6, atol=1e-9)
    assert np.allclose(oe.embedding_backward_f64(emb["ids"], emb["dY"], V, padding_idx, scale),
                       emb[tag + "_dW"], rtol=1e-12, atol=1e-15)
    if padding_idx is not None:
        assert (emb["ids"] == padding_idx).any() and not emb[tag + "_dW"][padding_idx].any()


def test_oracle_embedding_renorm_reproduces_golden(emb):
    from oracle import embedding as oe

    got = oe.embedding_renorm(emb["W"], emb["renorm_ids"], 3.0, 2.0)
    assert np.allclose(got, emb["renorm_W"], rtol=1e-12, atol=1e-15)
    assert not np.array_equal(got, emb["W"].astype(np.float64))  # some rows were clipped


@pytest.mark.gpu
@pytest.mark.parametrize("tag,padding_idx,scale", EMB_CASES)
def test_hip_embedding_reproduces_golden(emb, tag, padding_idx, scale):
    from axonn_amd import ops

    V = emb["W"].shape[0]
    ids = torch.from_numpy(emb["ids"]).cuda()
    W = torch.from_numpy(emb["W"]).cuda()
    dY = torch.from_numpy(emb["dY"]).cuda()
    y = ops.embedding_fwd(ids, W)
    assert np.array_equal(y.cpu().numpy(), emb[tag + "_Y"].astype(np.float32))
    dW = ops.embedding_bwd(ids, dY, V, padding_idx=padding_idx, scale_grad_by_freq=scale)
    assert np.allclose(dW.cpu().numpy(), emb[tag + "_dW"], rtol=1e-6, atol=1e-9)


@pytest.mark.gpu
def test_hip_embedding_renorm_reproduces_golden(emb):
    from axonn_amd import ops

    W = torch.from_numpy(emb["W"].copy()).cuda()
    ops.embedding_renorm_(W, torch.from_numpy(emb["renorm_ids"]).cuda(), 3.0, 2.0)
    assert np.allclose(W.cpu().numpy(), emb["renorm_W"], rtol=2e-6, atol=1e-9)
