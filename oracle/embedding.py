"""Oracle (test infrastructure) for the embedding lookup of the tensor-parallel Embedding.

The reference's layer (axonn/intra_layer/embedding.py:155-177) reshapes its flat weight
shard to [num_embeddings, embedding_dim / G] and calls

    F.embedding(x, weight, padding_idx, max_norm, norm_type, scale_grad_by_freq, sparse)

(:164-172); everything else in its forward is an exchange between ranks that is the
identity on one GPU.  This file restates what that torch call and its autograd compute:

  forward   out[t] = W[ids[t]]
  backward  dW[v]  = sum over tokens t with ids[t] == v of dY[t], nothing for the row
            `padding_idx`; with scale_grad_by_freq every term is divided by the number of
            tokens that name the row (torch: aten/src/ATen/native/Embedding.cpp,
            embedding_dense_backward_cpu)
  max_norm  rows named by ids whose p-norm exceeds max_norm are scaled by
            max_norm / (norm + 1e-7) before the lookup (embedding_renorm_cpu_, same file)

The backward adds in fp32 in ascending token order, one term after the other, which is
the order the HIP kernel promises, so fp32 results are compared bit for bit.

The reference's own tests of this layer (axonn/tests/test_intra_layer_emb.py) compare it
with torch.nn.Embedding on random ids for V in {32000, 50304, 128256}, H in {1024, 2048};
they hold no stored vectors.  Pinned in tests/test_oracle.py by torch's CPU F.embedding
and its autograd (all flags), by permutation / repeated-id closed forms, and by float64
sums.
"""

import numpy as np


def embedding_forward(ids, W):
    """W[ids]; an id outside the table reads as a row of zeros."""
    ids = np.asarray(ids, dtype=np.int64)
    W = np.asarray(W)
    flat = ids.reshape(-1)
    ok = (flat >= 0) & (flat < W.shape[0])
    out = np.zeros((flat.size, W.shape[1]), dtype=W.dtype)
    out[ok] = W[flat[ok]]
    return out.reshape(ids.shape + (W.shape[1],))


def embedding_backward(ids, dY, num_embeddings, padding_idx=None, scale_grad_by_freq=False,
                       accumulate_into=None):
    """Dense fp32 gradient of the table, terms added one by one in token order.

    dY is taken as fp32 values (bf16 inputs are exact in fp32).  With
    scale_grad_by_freq a term enters as fma(dY[t], 1/count, acc) with the reciprocal
    rounded to fp32.  `accumulate_into` (fp32 [V,H]) is added to the rows that
    received terms, after their sum.  Ids outside the table are skipped."""
    ids = np.asarray(ids, dtype=np.int64).reshape(-1)
    dY = np.asarray(dY, dtype=np.float32)
    H = dY.shape[-1]
    dY = dY.reshape(ids.size, H)
    keep = (ids >= 0) & (ids < num_embeddings)
    if padding_idx is not None:
        keep &= ids != padding_idx
    dW = np.zeros((num_embeddings, H), dtype=np.float32)
    if not scale_grad_by_freq:
        # np.add.at is unbuffered: dW[ids[i]] += dY[i] for i = 0, 1, ... in fp32
        np.add.at(dW, ids[keep], dY[keep])
    else:
        counts = np.bincount(ids[(ids >= 0) & (ids < num_embeddings)], minlength=num_embeddings)
        for t in np.nonzero(keep)[0]:
            v = ids[t]
            inv = np.float32(1.0) / np.float32(counts[v])
            # fused multiply-add: exact product and sum in float64, one rounding to fp32
            # (24 + 24 significant bits fit; the float64 sum rounds at 53 bits first,
            # which can differ from a true fma only in exact-tie cases)
            dW[v] = (dY[t].astype(np.float64) * np.float64(inv)
                     + dW[v].astype(np.float64)).astype(np.float32)
    if accumulate_into is not None:
        old = np.asarray(accumulate_into, dtype=np.float32)
        touched = np.zeros(num_embeddings, dtype=bool)
        touched[ids[keep]] = True
        out = old.copy()
        out[touched] = dW[touched] + old[touched]
        return out
    return dW


def embedding_backward_f64(ids, dY, num_embeddings, padding_idx=None, scale_grad_by_freq=False):
    """The same sums in float64, order-free: what every summation order approximates."""
    ids = np.asarray(ids, dtype=np.int64).reshape(-1)
    dY = np.asarray(dY, dtype=np.float64)
    dY = dY.reshape(ids.size, dY.shape[-1])
    keep = (ids >= 0) & (ids < num_embeddings)
    counts = np.bincount(ids[keep], minlength=num_embeddings).astype(np.float64)
    if padding_idx is not None:
        keep &= ids != padding_idx
    dW = np.zeros((num_embeddings, dY.shape[1]), dtype=np.float64)
    np.add.at(dW, ids[keep], dY[keep])
    if scale_grad_by_freq:
        dW /= np.maximum(counts, 1.0)[:, None]
    return dW


def embedding_renorm(W, ids, max_norm, norm_type=2.0):
    """Copy of W (float64) with the rows ids names clipped to norm max_norm."""
    W = np.asarray(W, dtype=np.float64).copy()
    ids = np.asarray(ids, dtype=np.int64).reshape(-1)
    rows = np.unique(ids[(ids >= 0) & (ids < W.shape[0])])
    a = np.abs(W[rows])
    if norm_type == 1.0:
        norm = a.sum(axis=1)
    elif norm_type == 2.0:
        norm = np.sqrt((a * a).sum(axis=1))
    else:
        norm = (a ** norm_type).sum(axis=1) ** (1.0 / norm_type)
    scale = np.where(norm > max_norm, max_norm / (norm + 1e-7), 1.0)
    W[rows] *= scale[:, None]
    return W
