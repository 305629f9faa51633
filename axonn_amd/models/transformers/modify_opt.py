"""OPT with `axonn_amd.intra_layer.Linear` projections, the counterpart of
axonn/models/transformers/modify_opt.py.

The reference restates `OPTAttention.__init__` (k / v / q / out projections, :9-43) and
`OPTDecoderLayer.__init__` (fc1, fc2, :46-74) with its Linear.  Both constructors
changed their signatures across transformers releases while the six projections kept
their names, so here the original constructors run first and the projections are
swapped afterwards; `out_proj` and `fc2` are the transposed layers, as in the
reference.  OPT's activation is ReLU, applied by Hugging Face's forward between fc1
and fc2.
"""

from transformers.models.opt.modeling_opt import OPTAttention, OPTDecoderLayer

from axonn_amd.intra_layer import Linear


def _swap(module, names, transposed):
    for name in names:
        old = getattr(module, name)
        setattr(module, name, Linear(old.in_features, old.out_features, bias=old.bias is not None,
                                     use_easy_api=False, transpose=name in transposed))


def _make_attention_init(original_init):
    def modified_attention_init(self, *args, **kwargs):
        original_init(self, *args, **kwargs)
        _swap(self, ("k_proj", "v_proj", "q_proj", "out_proj"), ("out_proj",))

    return modified_attention_init


def _make_decoder_init(original_init):
    def modified_decoder_init(self, *args, **kwargs):
        original_init(self, *args, **kwargs)  # builds self_attn through the patched OPTAttention
        _swap(self, ("fc1", "fc2"), ("fc2",))

    return modified_decoder_init


def monkey_patch_opt_with_axonn():
    original_inits = OPTAttention.__init__, OPTDecoderLayer.__init__
    OPTAttention.__init__ = _make_attention_init(OPTAttention.__init__)
    OPTDecoderLayer.__init__ = _make_decoder_init(OPTDecoderLayer.__init__)
    return original_inits


def reverse_monkey_patch_opt_with_axonn(original_attention_init, original_mlp_init):
    OPTAttention.__init__ = original_attention_init
    OPTDecoderLayer.__init__ = original_mlp_init
