"""Llama with `axonn_amd.intra_layer.Linear` projections, the counterpart of
axonn/models/transformers/modify_llama.py.

The reference replaces `LlamaAttention.__init__` and `LlamaMLP.__init__` by copies
that build q/k/v/o and gate/up/down from its Linear (:12-95) and leaves the
forward passes to Hugging Face.  Here

* the MLP is rebuilt the same way (`modified_mlp_init`, :76-95), and its forward
  `down_proj(act_fn(gate_proj(x)) * up_proj(x))` additionally runs the activation
  and the product as one kernel (`SwiGLU`, axn_swiglu_fwd / axn_swiglu_bwd) when
  the activation is SiLU - or, for 16-bit layers without bias and whole-tile shapes,
  both projections and the activation as one launch (`GateUpSwiGLU`,
  axn_gemm_swiglu_fwd), with the same results bit for bit;
* the attention projections are swapped after the original constructor has run,
  instead of restating that constructor (:12-73): the constructor's other fields
  changed across transformers releases, the four projections did not.  At a
  1 x 1 x 1 grid the reference's head-count divisions (:65-72) are by 1.
"""

import torch
from transformers.models.llama.modeling_llama import LlamaAttention, LlamaMLP, ACT2FN

from axonn_amd import ops
from axonn_amd.intra_layer import Linear
from axonn_amd.intra_layer.fully_connected import _compute_dtype, _weight_grad

_original_mlp_forward = None


class SwiGLU(torch.autograd.Function):
    """silu(gate) * up with a one-pass backward."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, gate, up):
        shape = gate.shape
        g2, u2 = gate.reshape(-1, shape[-1]), up.reshape(-1, shape[-1])
        ctx.save_for_backward(g2, u2)
        ctx.shape = shape
        return ops.swiglu_fwd(g2, u2).reshape(shape)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_out):
        g2, u2 = ctx.saved_tensors
        d2 = grad_out.reshape(-1, ctx.shape[-1]).to(g2.dtype)
        dgate, dup = ops.swiglu_bwd(d2, g2, u2)
        return dgate.reshape(ctx.shape), dup.reshape(ctx.shape)


def swiglu(gate, up):
    return SwiGLU.apply(gate, up)


class GateUpSwiGLU(torch.autograd.Function):
    """silu(x Wg^T) * (x Wu^T): the two projections and the activation in one launch
    forward; backward is the one-pass SwiGLU backward, the two input-gradient products
    in one pass (added in the accumulators, where autograd would add two rounded
    results), and the two wgrads as one launch."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, x, w_gate, w_up, shape):
        dt = _compute_dtype(x, w_gate.reshape(shape))
        x2 = x.reshape(-1, x.shape[-1]).to(dt)
        needs_grad = any(ctx.needs_input_grad[:3])
        h, gate, up = ops.gemm_swiglu_fwd(x2, w_gate.reshape(shape).to(dt), w_up.reshape(shape).to(dt),
                                          save=needs_grad)
        ctx.save_for_backward(x2, w_gate, w_up, gate, up)
        ctx.shape, ctx.input_shape, ctx.compute_dtype = shape, x.shape, dt
        return h.reshape(*x.shape[:-1], shape[0])

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_out):
        x2, w_gate, w_up, gate, up = ctx.saved_tensors
        dt = ctx.compute_dtype
        d2 = grad_out.reshape(-1, ctx.shape[0]).to(dt)
        n, k = ctx.shape
        # The two weight gradients are two launches: one launch over both outputs measured
        # within +-3 % of them at the Llama-3-8B shape and was dropped.
        dgate, dup = ops.swiglu_bwd(d2, gate, up)
        grad_x = grad_wg = grad_wu = None
        if ctx.needs_input_grad[0]:
            # both products through one set of accumulators, rounded once (two products and
            # an add where the shape does not fit the one-pass kernel)
            grad_x = ops.gemm_dgrad_pair(dgate, w_gate.reshape(ctx.shape).to(dt),
                                         dup, w_up.reshape(ctx.shape).to(dt))
            grad_x = grad_x.reshape(ctx.input_shape)
        if ctx.needs_input_grad[1]:
            grad_wg = _weight_grad(dgate, x2, w_gate)
        if ctx.needs_input_grad[2]:
            grad_wu = _weight_grad(dup, x2, w_up)
        return grad_x, grad_wg, grad_wu, None


def _one_launch_gate_up(mlp, x):
    """The MLP's gate/up pair qualifies for the one-launch forward: SiLU, no biases,
    plain layers on one rank, 16-bit compute type and whole-tile shapes."""
    g, u = mlp.gate_proj, mlp.up_proj
    if not (getattr(mlp, "_axonn_fused_swiglu", False) and x.is_cuda):
        return False
    if g.bias is not None or u.bias is not None or g.fused_activation or u.fused_activation:
        return False
    dt = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled("cuda") else g.weight.dtype
    if not torch.is_autocast_enabled("cuda") and not (x.dtype == g.weight.dtype == u.weight.dtype):
        return False
    tokens = x.numel() // max(x.shape[-1], 1)
    return ops.gemm_swiglu_supported(tokens, g.local_out_features, g.local_in_features, dt)


def modified_mlp_init(self, config):
    super(LlamaMLP, self).__init__()
    self.config = config
    self.hidden_size = config.hidden_size
    self.intermediate_size = config.intermediate_size
    bias = bool(getattr(config, "mlp_bias", False))
    self.gate_proj = Linear(self.hidden_size, self.intermediate_size, bias=bias, use_easy_api=False)
    self.up_proj = Linear(self.hidden_size, self.intermediate_size, bias=bias, use_easy_api=False)
    self.down_proj = Linear(self.intermediate_size, self.hidden_size, bias=bias, use_easy_api=False,
                            transpose=True)
    self.act_fn = ACT2FN[config.hidden_act]
    self._axonn_fused_swiglu = config.hidden_act in ("silu", "swish")


def modified_mlp_forward(self, x):
    if _one_launch_gate_up(self, x):
        shape = (self.gate_proj.local_out_features, self.gate_proj.local_in_features)
        return self.down_proj(GateUpSwiGLU.apply(x, self.gate_proj.weight, self.up_proj.weight, shape))
    gate, up = self.gate_proj(x), self.up_proj(x)
    if getattr(self, "_axonn_fused_swiglu", False) and gate.is_cuda and gate.dtype == up.dtype \
            and gate.dtype in (torch.bfloat16, torch.float16, torch.float32):
        return self.down_proj(swiglu(gate, up))
    return self.down_proj(self.act_fn(gate) * up)


def _make_attention_init(original_init):
    def modified_attention_init(self, config, layer_idx=None):
        original_init(self, config, layer_idx)
        bias = bool(getattr(config, "attention_bias", False))
        for name in ("q_proj", "k_proj", "v_proj", "o_proj"):
            old = getattr(self, name)
            setattr(self, name, Linear(old.in_features, old.out_features, bias=bias,
                                       use_easy_api=False, transpose=(name == "o_proj")))

    return modified_attention_init


def monkey_patch_llama_with_axonn():
    global _original_mlp_forward
    original_inits = LlamaAttention.__init__, LlamaMLP.__init__
    _original_mlp_forward = LlamaMLP.forward
    LlamaAttention.__init__ = _make_attention_init(LlamaAttention.__init__)
    LlamaMLP.__init__ = modified_mlp_init
    LlamaMLP.forward = modified_mlp_forward
    return original_inits


def reverse_monkey_patch_llama_with_axonn(original_attention_init, original_mlp_init):
    global _original_mlp_forward
    LlamaAttention.__init__ = original_attention_init
    LlamaMLP.__init__ = original_mlp_init
    if _original_mlp_forward is not None:
        LlamaMLP.forward = _original_mlp_forward
        _original_mlp_forward = None
