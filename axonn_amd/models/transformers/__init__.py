"""Swaps the projections of Hugging Face models for `axonn_amd.intra_layer.Linear`,
as `axonn.models.transformers` does (axonn/models/transformers/__init__.py:22-60).
Llama, Mistral, OPT and Mixtral (attention only: current transformers releases keep the
experts in fused 3-D parameters) are covered; a model family is imported when asked for."""

from contextlib import contextmanager

from .modify_llama import (  # noqa: F401
    monkey_patch_llama_with_axonn,
    reverse_monkey_patch_llama_with_axonn,
)


def _lazy(module, family):
    """(patch, unpatch) that import the family's module on first use, so that importing
    this package does not import every model family of transformers."""
    def patch():
        import importlib

        mod = importlib.import_module(__name__ + "." + module)
        return getattr(mod, "monkey_patch_%s_with_axonn" % family)()

    def unpatch(original_attention_init, original_mlp_init):
        import importlib

        mod = importlib.import_module(__name__ + "." + module)
        return getattr(mod, "reverse_monkey_patch_%s_with_axonn" % family)(
            original_attention_init, original_mlp_init)

    return patch, unpatch


modify_dict = {
    "LlamaForCausalLM": (monkey_patch_llama_with_axonn, reverse_monkey_patch_llama_with_axonn),
    "MistralForCausalLM": _lazy("modify_mistral", "mistral"),
    "OPTForCausalLM": _lazy("modify_opt", "opt"),
    "MixtralForCausalLM": _lazy("modify_mixtral", "mixtral"),
}


@contextmanager
def parallelize(model_id_or_config):
    """Models created inside the context get the patched layers.  Takes what the
    reference takes (a model id or path for `AutoConfig.from_pretrained`,
    __init__.py:44) or a config object, which needs no file access."""
    config = model_id_or_config
    if isinstance(model_id_or_config, str):
        from transformers import AutoConfig

        config = AutoConfig.from_pretrained(model_id_or_config)
    architectures = getattr(config, "architectures", None) or ["LlamaForCausalLM"]
    architecture = architectures[0]
    assert architecture in modify_dict, f"{architecture} has not been parallelized within AxoNN"
    monkey_patch_fn, reverse_monkey_patch_fn = modify_dict[architecture]
    original_attention_init, original_mlp_init = monkey_patch_fn()
    try:
        yield None
    finally:
        reverse_monkey_patch_fn(original_attention_init, original_mlp_init)
