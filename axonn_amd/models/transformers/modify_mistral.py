"""Mistral with `axonn_amd.intra_layer.Linear` projections, the counterpart of
axonn/models/transformers/modify_mistral.py.

The reference restates `MistralAttention.__init__` and `MistralMLP.__init__` with its
Linear in place of nn.Linear (:12-95).  Mistral's MLP is Llama's (gate / up / down with
SiLU), so it is rebuilt the same way and runs `act_fn(gate) * up` as the one-pass SwiGLU
kernel; the four attention projections are swapped after the original constructor has
run, which keeps the constructor's other fields as the installed transformers release
defines them.
"""

from transformers.models.mistral.modeling_mistral import ACT2FN, MistralAttention, MistralMLP

from axonn_amd.intra_layer import Linear

from .modify_llama import _make_attention_init, modified_mlp_forward

_original_mlp_forward = None


def modified_mlp_init(self, config):
    super(MistralMLP, self).__init__()
    self.config = config
    self.hidden_size = config.hidden_size
    self.intermediate_size = config.intermediate_size
    self.gate_proj = Linear(self.hidden_size, self.intermediate_size, bias=False, use_easy_api=False)
    self.up_proj = Linear(self.hidden_size, self.intermediate_size, bias=False, use_easy_api=False)
    self.down_proj = Linear(self.intermediate_size, self.hidden_size, bias=False, use_easy_api=False,
                            transpose=True)
    self.act_fn = ACT2FN[config.hidden_act]
    self._axonn_fused_swiglu = config.hidden_act in ("silu", "swish")


def monkey_patch_mistral_with_axonn():
    global _original_mlp_forward
    original_inits = MistralAttention.__init__, MistralMLP.__init__
    _original_mlp_forward = MistralMLP.forward
    MistralAttention.__init__ = _make_attention_init(MistralAttention.__init__)
    MistralMLP.__init__ = modified_mlp_init
    MistralMLP.forward = modified_mlp_forward
    return original_inits


def reverse_monkey_patch_mistral_with_axonn(original_attention_init, original_mlp_init):
    global _original_mlp_forward
    MistralAttention.__init__ = original_attention_init
    MistralMLP.__init__ = original_mlp_init
    if _original_mlp_forward is not None:
        MistralMLP.forward = _original_mlp_forward
        _original_mlp_forward = None
