"""Host-side logic of the package that needs no GPU: the one-rank grid stub, the
Linear module's parameters and state-dict loader, the loss-scale state machine,
argument checks, and the absence of any CPU fallback."""

import math

import numpy as np
import pytest
import torch

import axonn_amd
from axonn_amd import axonn as ax
from axonn_amd import inter_layer, ops
from axonn_amd.intra_layer import Linear, clip_grad_norm_, optimize_communication
from axonn_amd.intra_layer import communication as comm
from axonn_amd.intra_layer import overlap_communication as oc
from axonn_amd.optim import CPUAdam
from axonn_amd.utils import _coalesce_and_reassign
from oracle import optim as oo


def test_init_accepts_only_the_one_gpu_grid():
    ax.init(G_inter=1, G_data=1, G_intra_r=1, G_intra_c=1, G_intra_d=1)
    assert ax.is_initialized and ax.comm_handle.world_size == 1
    inner, outer, depth = ax.comm_handle.get_intra_layer_groups()
    assert ax.get_world_size(inner) == ax.get_world_size(outer) == ax.get_world_size(depth) == 1
    for kw in ("G_inter", "G_data", "G_intra_r", "G_intra_c", "G_intra_d"):
        with pytest.raises(NotImplementedError):
            ax.init(**{kw: 2})
    with pytest.raises(NotImplementedError):
        ax.comm_handle.get_intra_layer_groups((2, 1, 1))
    ax.init()


def test_linear_parameters_follow_the_reference_layout():
    torch.manual_seed(0)
    layer = Linear(48, 24)
    assert layer.weight.ndim == 1 and layer.weight.numel() == 24 * 48  # flat [out*in]
    assert layer.weight.is_tensor_parallel and not layer.weight.needs_depth_parallel_gradient_sync
    assert layer.bias.shape == (24,) and torch.count_nonzero(layer.bias) == 0
    assert layer.bias.is_tensor_parallel and layer.bias.needs_depth_parallel_gradient_sync
    assert hasattr(layer.weight, "process_group_for_norm_reduction")
    assert (layer.local_in_features, layer.local_out_features) == (48, 24)
    bound = 1.0 / math.sqrt(48)  # kaiming_uniform_(a=sqrt 5)
    assert float(layer.weight.abs().max()) <= bound
    assert Linear(8, 8, bias=False).bias is None
    Linear(8, 8, use_easy_api=True)  # stale keyword arguments are swallowed
    with pytest.raises(ValueError):
        Linear(8, 8, fused_activation="relu")

    def init_ones(w):
        return torch.nn.init.ones_(w)

    assert torch.all(Linear(8, 16, init_method=init_ones).weight == 1)


def test_state_dict_accepts_full_and_sharded_weights():
    torch.manual_seed(1)
    ref = torch.nn.Linear(16, 8)
    layer = Linear(16, 8)
    layer.load_state_dict(ref.state_dict())  # full [out, in] checkpoint
    assert torch.equal(layer.weight.view(8, 16), ref.weight)
    assert torch.equal(layer.bias, ref.bias)
    layer.load_state_dict(layer.state_dict())  # sharded 1-D checkpoint
    assert torch.equal(layer.weight.view(8, 16), ref.weight)
    with pytest.raises(AssertionError, match="neither a full checkpoint nor a sharded"):
        layer.load_state_dict({"weight": torch.zeros(4, 4), "bias": torch.zeros(8)})
    with pytest.raises(AssertionError):
        layer.load_state_dict({"weight": torch.zeros(128), "bias": torch.zeros(3)})


def test_no_cpu_fallback():
    layer = Linear(16, 8)
    with pytest.raises(RuntimeError, match="GPU only"):
        layer(torch.randn(4, 16))
    with pytest.raises(RuntimeError, match="GPU"):
        CPUAdam(layer.parameters())
    p = torch.nn.Parameter(torch.zeros(4))
    p.grad = torch.ones(4)
    with pytest.raises(RuntimeError, match="GPU only"):
        clip_grad_norm_([p], 1.0)
    with pytest.raises(RuntimeError, match="GPU only"):
        inter_layer.check_nan(torch.zeros(4))


def test_communication_primitives_are_identities_on_one_rank():
    x = torch.arange(12.0).reshape(3, 4)
    g = ax._handle().inner_intra_layer_parallel_group
    assert comm._drop(x, 1, g) is x and comm._gather(x, 0, g) is x
    assert comm._reduce_scatter(x, 0, g) is x
    assert torch.equal(comm._all_reduce(x, g), x)
    assert torch.equal(comm.Drop.apply(x, g), x) and torch.equal(comm.Gather.apply(x, g), x)
    with pytest.raises(AssertionError):
        comm._reduce_scatter(x, 1, g)
    with pytest.raises(NotImplementedError):
        comm._gather(x, 0, object())


def test_optimize_communication_flags():
    assert not oc.OVERLAP_REDUCE_SCATTER and not oc.OVERLAP_ALL_REDUCE
    with optimize_communication(overlap_all_reduce=True, overlap_reduce_scatter=True):
        assert oc.OVERLAP_REDUCE_SCATTER and oc.OVERLAP_ALL_REDUCE
        p = torch.nn.Parameter(torch.zeros(3))
        oc.accumulate_later(p, torch.ones(3))
        oc.accumulate_later(p, torch.ones(3) * 2)
    assert not oc.OVERLAP_REDUCE_SCATTER and not oc.OVERLAP_ALL_REDUCE
    assert torch.equal(p.grad, torch.full((3,), 3.0))  # flushed when the context exits
    with pytest.raises(ValueError, match="pass your model"):
        with optimize_communication(overlap_all_gather=True):
            pass


def test_loss_scaler_matches_oracle_on_random_sequences():
    rng = np.random.default_rng(0)
    a, b = inter_layer.LossScaler(), oo.LossScaler()
    assert (a.loss_scale, a.max_scale, a.min_scale, a.scaling_window, a.no_overflow_iters) == (
        b.loss_scale, b.max_scale, b.min_scale, b.scaling_window, b.no_overflow_iters)
    for _ in range(3000):
        ov = bool(rng.random() < 0.004)
        assert inter_layer.sync_scale(a, ov) == oo.sync_scale(b, ov)
        assert (a.loss_scale, a.no_overflow_iters) == (b.loss_scale, b.no_overflow_iters)
    c = inter_layer.LossScaler(loss_scale=2048.0)
    inter_layer.sync_scale(c, True)
    inter_layer.sync_scale(c, True)
    assert c.loss_scale == 1024.0


def test_cpuadam_rejects_bad_hyperparameters():
    p = [torch.nn.Parameter(torch.zeros(2))]
    for kw, msg in ((dict(lr=-1.0), "learning rate"), (dict(eps=-1.0), "epsilon"),
                    (dict(betas=(1.0, 0.9)), "index 0"), (dict(betas=(0.9, 1.5)), "index 1"),
                    (dict(weight_decay=-0.1), "weight_decay")):
        with pytest.raises(ValueError, match=msg):
            CPUAdam(p, **kw)


def test_coalesce_and_reassign_layout():
    ts = [torch.arange(3.0), torch.arange(4.0).reshape(2, 2) + 10, torch.tensor([99.0])]
    flat = _coalesce_and_reassign(ts)
    assert torch.equal(flat, torch.tensor([0, 1, 2, 10, 11, 12, 13, 99.0]))
    flat[5] = -1.0
    assert ts[1][1, 0] == -1.0 and ts[1].shape == (2, 2)  # tensors alias the flat buffer
    assert ts[1].data_ptr() == flat.data_ptr() + 3 * 4    # packed, no padding


def test_adam_hparams_use_double_precision_bias_corrections():
    hp = ops.adam_hparams(3, 1e-3, 0.9, 0.999, 1e-8, 0.01)
    bc1, bc2 = oo.bias_corrections(3, 0.9, 0.999)
    assert hp.lr_over_bc1 == np.float32(1e-3 / bc1)
    assert hp.inv_sqrt_bc2 == np.float32(1.0 / math.sqrt(bc2))
    assert hp.one_minus_beta1 == np.float32(1.0 - 0.9) and hp.weight_decay == np.float32(0.01)


def test_clip_grad_norm_argument_handling():
    with pytest.raises(NotImplementedError):
        clip_grad_norm_([], 1.0, norm_type=float("inf"))
    from axonn_amd.intra_layer.gradient_normalization import get_total_norm

    with pytest.raises(NotImplementedError):
        clip_grad_norm_([], 1.0, norm_type=float("-inf"))
    assert float(get_total_norm([], float("inf"))) == 0.0               # any order, as the reference
    assert float(clip_grad_norm_([], 1.0, norm_type=1.0)) == 0.0        # any finite order is taken
    assert float(get_total_norm([], 3.0)) == 0.0
    assert float(clip_grad_norm_([torch.nn.Parameter(torch.zeros(2))], 1.0)) == 0.0  # no grads


def test_package_exports():
    assert hasattr(axonn_amd, "axonn") and hasattr(axonn_amd, "config")
    from axonn_amd.intra_layer import AsyncLinear, Drop, Gather, no_grad_sync, sync_gradients  # noqa: F401

    assert axonn_amd.config.G_intra == 1


def test_auto_parallelize_swaps_nn_linear_inside_the_context_only():
    import torch.nn as nn

    import axonn_amd.axonn as ax
    from axonn_amd.intra_layer import Linear, auto_parallelize
    from axonn_amd.intra_layer.automatic_parallelism import is_parallelizable_linear

    ax.init(1, 1, 1, 1)
    original = nn.Linear
    with auto_parallelize():
        a = nn.Linear(16, 24)
        b = nn.Linear(16, 8, bias=False, dtype=torch.bfloat16)

        class Net(nn.Module):            # a model declared inside picks the layer up unchanged
            def __init__(self):
                super().__init__()
                self.fc = nn.Linear(8, 8)

        net = Net()
    assert nn.Linear is original and isinstance(nn.Linear(4, 4), original)
    assert isinstance(a, Linear) and a.weight.shape == (16 * 24,) and a.bias is not None
    assert isinstance(b, Linear) and b.bias is None and b.weight.dtype == torch.bfloat16
    assert isinstance(net.fc, Linear)
    assert is_parallelizable_linear(16, 24)
    try:
        with auto_parallelize():
            raise RuntimeError("boom")
    except RuntimeError:
        pass
    assert nn.Linear is original     # restored on error as well


def test_embedding_parameters_state_dict_and_no_cpu_fallback():
    """The reference's layout: a flat [V * H] weight, tags for gradient sync and clipping,
    a loader that takes torch.nn.Embedding's 2-D weight or its own 1-D shard
    (axonn/intra_layer/embedding.py:139-148, :191-222; its test loads both ways,
    axonn/tests/test_intra_layer_emb.py:46-49)."""
    from axonn_amd.intra_layer import Embedding

    torch.manual_seed(2)
    V, H = 50, 16
    layer = Embedding(V, H, padding_idx=-3)
    assert layer.weight.shape == (V * H,) and layer.weight.is_tensor_parallel
    assert layer.weight.needs_depth_parallel_gradient_sync is False
    assert layer.padding_idx == V - 3 and layer.get_output_feature_size() == H
    table = layer.weight.detach().view(V, H)
    assert not table[V - 3].any() and table[0].any() and table[V - 2].any()
    assert abs(float(table.std()) - 1.0) < 0.1  # normal(0, 1) default
    ref = torch.nn.Embedding(V, H)
    layer.load_state_dict(ref.state_dict())
    assert torch.equal(layer.weight.view(V, H), ref.weight)
    layer.load_state_dict(layer.state_dict())
    assert torch.equal(layer.weight.view(V, H), ref.weight)
    with pytest.raises(AssertionError, match="neither a full checkpoint nor a sharded"):
        layer.load_state_dict({"weight": torch.zeros(H, V)})
    with pytest.raises(AssertionError, match="Padding_idx"):
        Embedding(V, H, padding_idx=V)
    with pytest.raises(AssertionError, match="_weight"):
        Embedding(V, H, _weight=torch.zeros(V, H))
    assert Embedding(V, H, _freeze=True).weight.requires_grad is False
    with pytest.raises(RuntimeError, match="GPU only"):
        layer(torch.zeros(2, 3, dtype=torch.long))
    with pytest.raises(NotImplementedError, match="sparse"):
        Embedding(V, H, sparse=True)(torch.zeros(2, 3, dtype=torch.long))


def test_checkpoint_round_trip_under_the_rank_prefix(tmp_path):
    """axonn/checkpoint.py:11-27: one file per tensor-parallel rank, under a folder named
    after its grid coordinates."""
    from axonn_amd import checkpoint

    assert checkpoint.get_prefix_for_checkpoint() == "tp_row_0_col_0_depth_0"
    layer = Linear(16, 8)
    state = {"model": layer.state_dict(), "step": 7}
    checkpoint.save(state, str(tmp_path), "ckpt")
    assert (tmp_path / "tp_row_0_col_0_depth_0" / "ckpt.pt").exists()
    with pytest.raises(ValueError, match="already exists"):
        checkpoint.save(state, str(tmp_path), "ckpt", overwrite=False)
    loaded = checkpoint.load({}, str(tmp_path), "ckpt")
    assert loaded["step"] == 7 and torch.equal(loaded["model"]["weight"], layer.weight)
    other = Linear(16, 8)
    other.load_state_dict(loaded["model"])
    assert torch.equal(other.weight, layer.weight)
    with pytest.raises(AssertionError, match="does not exist"):
        checkpoint.load({}, str(tmp_path / "missing"), "ckpt")


def test_bench_refuses_more_than_one_gpu():
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode != 0
    assert "ONE GPU" in proc.stderr and proc.stdout.strip() == ""


@pytest.mark.parametrize("family,n_linear", [("mistral", 14), ("opt", 12), ("mixtral", 8)])
def test_parallelize_patches_every_family_the_reference_patches(family, n_linear):
    """axonn/models/transformers/__init__.py:22-39 lists OPT, Llama, Mixtral and Mistral;
    models built inside the context get the Linear projections, models built after it
    do not (construction only: no kernel runs on the CPU)."""
    from transformers import MistralConfig, MixtralConfig, OPTConfig
    from transformers.models.mistral.modeling_mistral import MistralForCausalLM
    from transformers.models.mixtral.modeling_mixtral import MixtralForCausalLM
    from transformers.models.opt.modeling_opt import OPTForCausalLM

    from axonn_amd.models.transformers import modify_dict, parallelize

    assert set(modify_dict) == {"OPTForCausalLM", "LlamaForCausalLM", "MixtralForCausalLM", "MistralForCausalLM"}
    ax.init(1, 1, 1, 1)
    common = dict(hidden_size=64, num_attention_heads=4, num_hidden_layers=2, vocab_size=64,
                  max_position_embeddings=32)
    cls, cfg = {
        "mistral": (MistralForCausalLM, MistralConfig(intermediate_size=128, num_key_value_heads=2,
                                                      architectures=["MistralForCausalLM"], **common)),
        "opt": (OPTForCausalLM, OPTConfig(ffn_dim=128, word_embed_proj_dim=64,
                                          architectures=["OPTForCausalLM"], **common)),
        "mixtral": (MixtralForCausalLM, MixtralConfig(intermediate_size=128, num_key_value_heads=2,
                                                      num_local_experts=4,
                                                      architectures=["MixtralForCausalLM"], **common)),
    }[family]
    with parallelize(cfg):
        model = cls(cfg)
    assert sum(isinstance(m, Linear) for m in model.modules()) == n_linear
    assert not any(isinstance(m, Linear) for m in cls(cfg).modules())
    with pytest.raises(AssertionError, match="has not been parallelized"):
        cfg.architectures = ["GPT2LMHeadModel"]
        with parallelize(cfg):
            pass
