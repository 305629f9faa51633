"""Llama with `axonn_amd.intra_layer.Linear` projections, the counterpart of
axonn/models/transformers/modify_llama.py.

The reference replaces `LlamaAttention.__init__` and `LlamaMLP.__init__` by copies
that build q/k/v/o and gate/up/down from its Linear (:12-95) and leaves the
forward passes to Hugging Face.  Here

* the MLP is rebuilt the same way (`modified_mlp_init`, :76-95), and its forward
  `down_proj(act_fn(gate_proj(x)) * up_proj(x))` additionally runs the activation
  and the product as one kernel (`SwiGLU`, axn_swiglu_fwd / axn_swiglu_bwd) when
  the activation is SiLU;
* the attention projections are swapped after the original constructor has run,
  instead of restating that constructor (:12-73): the constructor's other fields
  changed across transformers releases, the four projections did not.  At a
  1 x 1 x 1 grid the reference's head-count divisions (:65-72) are by 1.
"""

import torch
from transformers.models.llama.modeling_llama import LlamaAttention, LlamaMLP, ACT2FN

from axonn_amd import ops
from axonn_amd.intra_layer import Linear

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
