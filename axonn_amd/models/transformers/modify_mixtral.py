"""Mixtral with `axonn_amd.intra_layer.Linear` attention projections, the counterpart of
axonn/models/transformers/modify_mixtral.py.

The reference swaps the four attention projections (:12-75) and the three matrices
w1 / w2 / w3 of every expert, which `MixtralBLockSparseTop2MLP` held as nn.Linear
(:78-97).  Current transformers releases keep all experts of a layer in two 3-D
parameters (`MixtralExperts.gate_up_proj`, `.down_proj`) and multiply through
`nn.functional.linear` on slices of them, so there is no per-expert layer to replace:
the attention projections are swapped, the experts stay as the release defines them,
and where the installed release still has the per-expert class its three matrices are
swapped too.
"""

from transformers.models.mixtral import modeling_mixtral
from transformers.models.mixtral.modeling_mixtral import MixtralAttention

from axonn_amd.intra_layer import Linear

from .modify_llama import _make_attention_init

_EXPERT_CLASS = getattr(modeling_mixtral, "MixtralBlockSparseTop2MLP",
                        getattr(modeling_mixtral, "MixtralBLockSparseTop2MLP", None))


def _make_expert_init(original_init):
    def modified_expert_init(self, *args, **kwargs):
        original_init(self, *args, **kwargs)
        for name in ("w1", "w2", "w3"):
            old = getattr(self, name)
            setattr(self, name, Linear(old.in_features, old.out_features, bias=False,
                                       use_easy_api=False, transpose=(name == "w2")))

    return modified_expert_init


def monkey_patch_mixtral_with_axonn():
    original_expert_init = _EXPERT_CLASS.__init__ if _EXPERT_CLASS is not None else None
    original_inits = MixtralAttention.__init__, original_expert_init
    MixtralAttention.__init__ = _make_attention_init(MixtralAttention.__init__)
    if _EXPERT_CLASS is not None:
        _EXPERT_CLASS.__init__ = _make_expert_init(original_expert_init)
    return original_inits


def reverse_monkey_patch_mixtral_with_axonn(original_attention_init, original_mlp_init):
    MixtralAttention.__init__ = original_attention_init
    if _EXPERT_CLASS is not None and original_mlp_init is not None:
        _EXPERT_CLASS.__init__ = original_mlp_init
