"""Oracle (test infrastructure) for the Llama MLP block built from three Linears.

The reference's Llama patch (axonn/models/transformers/modify_llama.py:76-95)
rebuilds `LlamaMLP` from its Linear and leaves the forward to Hugging Face:

    down_proj(act_fn(gate_proj(x)) * up_proj(x)),   act_fn = SiLU for Llama

(transformers/models/llama/modeling_llama.py, LlamaMLP.forward).  At a 1 x 1 x 1
grid each Linear is the plain product of oracle.linear.  All arithmetic is
float64; `store` names the storage type the layer outputs are rounded to between
the stages ('f64' = none), as they are when the model runs in bf16.

Parity unpinned by the reference itself: it has no test of the patched models.
Pinned in tests/test_oracle.py by torch.nn.functional.silu, autograd, closed
forms and finite differences.
"""

import numpy as np

from .linear import linear_backward, linear_forward, round_to


def sigmoid(x):
    x = np.asarray(x, dtype=np.float64)
    out = np.empty_like(x)
    pos = x >= 0
    out[pos] = 1.0 / (1.0 + np.exp(-x[pos]))
    e = np.exp(x[~pos])
    out[~pos] = e / (1.0 + e)
    return out


def silu(x):
    """x * sigmoid(x), torch.nn.SiLU."""
    x = np.asarray(x, dtype=np.float64)
    return x * sigmoid(x)


def dsilu(x):
    """d silu / dx = s (1 + x (1 - s)), s = sigmoid(x)."""
    x = np.asarray(x, dtype=np.float64)
    s = sigmoid(x)
    return s * (1.0 + x * (1.0 - s))


def swiglu_forward(gate, up):
    return silu(gate) * np.asarray(up, dtype=np.float64)


def swiglu_backward(dout, gate, up):
    """(dgate, dup) of out = silu(gate) * up."""
    dout = np.asarray(dout, dtype=np.float64)
    return dout * np.asarray(up, dtype=np.float64) * dsilu(gate), dout * silu(gate)


def llama_mlp_forward(x, w_gate, w_up, w_down, hidden, intermediate, store="f64"):
    """x [M, hidden]; weights flat 1-D as the Linear holds them.  Returns a dict of
    every stage (gate, up, act, out), each rounded to `store`."""
    g, _ = linear_forward(x, w_gate, (intermediate, hidden))
    u, _ = linear_forward(x, w_up, (intermediate, hidden))
    g, u = round_to(g, store), round_to(u, store)
    a = round_to(swiglu_forward(g, u), store)
    y, _ = linear_forward(a, w_down, (hidden, intermediate))
    return {"gate": g, "up": u, "act": a, "out": round_to(y, store)}


def llama_mlp_backward(x, w_gate, w_up, w_down, hidden, intermediate, dout, fwd, store="f64"):
    """Gradients of the block given the stages `fwd` of llama_mlp_forward."""
    bd = linear_backward(fwd["act"], w_down, (hidden, intermediate), dout)
    da = round_to(bd["dx"], store)
    dg, du = swiglu_backward(da, fwd["gate"], fwd["up"])
    dg, du = round_to(dg, store), round_to(du, store)
    bg = linear_backward(x, w_gate, (intermediate, hidden), dg)
    bu = linear_backward(x, w_up, (intermediate, hidden), du)
    return {
        "dx": round_to(round_to(bg["dx"], store) + round_to(bu["dx"], store), store),
        "dw_gate": bg["dw"], "dw_up": bu["dw"], "dw_down": bd["dw"],
    }
