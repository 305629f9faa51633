"""Writes the golden fixtures in this directory.

The reference ships no golden vectors: its tests assert equality with
torch.nn.Linear / torch.nn.utils.clip_grad_norm_ on seeded random inputs
(axonn/tests/test_intra_layer_fc.py), and it has no optimizer test.  All of the
hot path's arithmetic is delegated to torch, so the fixtures here are produced
by those torch library routines on CPU (float64 for the layer, float32 for the
optimizer, exactly the routines the reference calls), on the reference's own
test shapes and input scaling.  Nothing of the reference is imported or run.

    python tests/golden/make_golden.py
"""

import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def _bf16_exact(t):
    """Rounds to bfloat16-representable values (so the same inputs feed the fp64
    library routine here and the bf16 kernels in the GPU tests without a second
    rounding) and returns (float64 tensor, uint16 bit patterns)."""
    b = t.float().bfloat16()
    return b.double(), b.view(torch.int16).numpy().view(np.uint16)


def linear_cases():
    """Inputs are stored as bfloat16 bit patterns (uint16); outputs are what
    torch.nn.functional.linear + autograd give in float64 on those inputs.  The
    large weight gradients are stored in float32 next to their float64 row and
    column sums."""
    out = {}
    # (B, H) and the 0.01 scaling of axonn/tests/test_intra_layer_fc.py:18,37,112-113
    for idx, (B, H) in enumerate([(32, 64), (16, 128), (2, 256)]):
        torch.manual_seed(42)
        X, Xb = _bf16_exact(torch.randn(B, H) * 0.01)
        dY, dYb = _bf16_exact(torch.randn(B, H) * 0.01)
        ref = torch.nn.Linear(H, H, bias=True)
        W, Wb = _bf16_exact(ref.weight.detach())
        b = ref.bias.detach().double()  # bias stays fp32 in the kernels
        X.requires_grad_(True)
        W.requires_grad_(True)
        b.requires_grad_(True)
        Y = torch.nn.functional.linear(X, W, b)
        Y.backward(dY)
        out[f"c{idx}_X"], out[f"c{idx}_dY"], out[f"c{idx}_W"] = Xb, dYb, Wb
        out[f"c{idx}_b"] = b.detach().float().numpy()
        out[f"c{idx}_Y"] = Y.detach().numpy()
        out[f"c{idx}_dX"] = X.grad.numpy()
        out[f"c{idx}_dW"] = W.grad.float().numpy()
        out[f"c{idx}_dW_rowsum"] = W.grad.sum(1).numpy()
        out[f"c{idx}_dW_colsum"] = W.grad.sum(0).numpy()
        out[f"c{idx}_db"] = b.grad.numpy()
    # bias + exact GELU, a shape that is not a multiple of any tile
    torch.manual_seed(7)
    X, Xb = _bf16_exact(torch.randn(24, 40))
    ref = torch.nn.Linear(40, 56)
    W, Wb = _bf16_exact(ref.weight.detach())
    b = (torch.randn(56) * 0.1).double()
    dY, dYb = _bf16_exact(torch.randn(24, 56))
    X.requires_grad_(True)
    W.requires_grad_(True)
    b.requires_grad_(True)
    Z = torch.nn.functional.linear(X, W, b)
    Y = torch.nn.functional.gelu(Z)
    Y.backward(dY)
    out.update(g_X=Xb, g_dY=dYb, g_W=Wb, g_b=b.detach().float().numpy(),
               g_Z=Z.detach().numpy(), g_Y=Y.detach().numpy(), g_dX=X.grad.numpy(),
               g_dW=W.grad.numpy(), g_db=b.grad.numpy())
    np.savez_compressed(os.path.join(HERE, "linear_f64.npz"), **out)


def optimizer_cases():
    out = {}
    torch.manual_seed(3)
    sizes = [7, 130, 1, 515]  # odd sizes: ragged views into a flat buffer
    params = [torch.nn.Parameter(torch.randn(n) * 0.02) for n in sizes]
    opt = torch.optim.Adam(params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01,
                           foreach=False)
    out["sizes"] = np.array(sizes)
    out["p0"] = torch.cat([p.detach() for p in params]).numpy()
    for step in range(1, 4):
        grads = [torch.randn(n) * 1e-3 for n in sizes]
        for p, g in zip(params, grads):
            p.grad = g.clone()
        total = torch.nn.utils.clip_grad_norm_(params, max_norm=0.01, foreach=False)
        out[f"g{step}"] = torch.cat(grads).numpy()
        out[f"gclip{step}"] = torch.cat([p.grad for p in params]).numpy()
        out[f"norm{step}"] = np.array(float(total))
        opt.step()
        out[f"p{step}"] = torch.cat([p.detach() for p in params]).numpy()
        out[f"m{step}"] = torch.cat([opt.state[p]["exp_avg"] for p in params]).numpy()
        out[f"v{step}"] = torch.cat([opt.state[p]["exp_avg_sq"] for p in params]).numpy()
        out[f"pbf{step}"] = torch.cat([p.detach().bfloat16().view(torch.int16) for p in params]).numpy()
    # float32 -> bfloat16 conversion table incl. ties, subnormals, infinities
    vals = torch.tensor([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 1.005859375, 3.0e38, 3.39e38, 3.4e38,
                         1e-40, -1e-45, float("inf"), float("-inf"), 65504.0, 0.1, -0.3333333],
                        dtype=torch.float32)
    rnd = torch.randn(256) * torch.logspace(-20, 20, 256)
    vals = torch.cat([vals, rnd])
    out["cvt_f32"] = vals.numpy()
    out["cvt_bf16_bits"] = vals.bfloat16().view(torch.int16).numpy()
    np.savez_compressed(os.path.join(HERE, "optimizer_f32.npz"), **out)


def embedding_cases():
    """torch's CPU F.embedding (the call at axonn/intra_layer/embedding.py:164-172) and its
    autograd in float64 on fp32-representable inputs, ids drawn as the reference's test
    draws them (randint over the vocabulary; here a small one, so that ids repeat), with
    each flag of the call exercised once."""
    g = torch.Generator().manual_seed(2024)
    V, H, B, S = 97, 24, 4, 50
    out = {}
    W = torch.randn(V, H, generator=g).double()
    ids = torch.randint(0, V, (B, S), generator=g)
    dY = (torch.randn(B, S, H, generator=g) * 0.01).double()
    out["ids"], out["W"], out["dY"] = ids.numpy(), W.numpy().astype(np.float32), dY.numpy().astype(np.float32)
    for tag, kw in (("plain", {}), ("pad", {"padding_idx": 5}),
                    ("freq", {"padding_idx": 5, "scale_grad_by_freq": True})):
        w = W.clone().requires_grad_(True)
        y = torch.nn.functional.embedding(ids, w, **kw)
        y.backward(dY)
        out[tag + "_Y"] = y.detach().numpy()
        out[tag + "_dW"] = w.grad.numpy()
    w = W.clone()
    torch.nn.functional.embedding(ids[:1, :20], w, max_norm=3.0, norm_type=2.0)
    out["renorm_ids"] = ids[:1, :20].numpy()
    out["renorm_W"] = w.numpy()
    np.savez_compressed(os.path.join(HERE, "embedding_f64.npz"), **out)


if __name__ == "__main__":
    linear_cases()
    optimizer_cases()
    embedding_cases()
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
