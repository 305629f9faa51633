"""Parity of the Llama MLP block (patched Hugging Face LlamaMLP on the kernels)
and of the SwiGLU kernels with the CPU oracle.

Tolerances: the SwiGLU kernels compute in fp32 and round once, so against the
float64 oracle on the same inputs the bf16 result is within one bf16 rounding
(checked elementwise) and the fp32 result within 1e-6 relative.  The block's
outputs and gradients, which pass through three bf16 GEMMs, use the GEMM bar:
normwise 1e-2 against the float64 oracle fed the same bf16 weights and inputs.
"""

import numpy as np
import pytest
import torch

from axonn_amd import _native as nv
from oracle import llama as om

pytestmark = pytest.mark.gpu


def np64(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


@pytest.mark.parametrize("M,N", [(1, 8), (37, 520), (256, 1024)])
def test_swiglu_kernels_match_oracle_elementwise(M, N):
    from axonn_amd import ops

    g = torch.Generator().manual_seed(M * 1000 + N)
    gate = (torch.randn(M, N, generator=g) * 3).bfloat16()
    up = torch.randn(M, N, generator=g).bfloat16()
    dout = torch.randn(M, N, generator=g).bfloat16()
    want = om.swiglu_forward(np64(gate), np64(up))
    out = ops.swiglu_fwd(gate.cuda(), up.cuda())
    assert np.all(np.abs(np64(out) - want) <= 2.0 ** -8 * np.abs(want) + 1e-30)
    wdg, wdu = om.swiglu_backward(np64(dout), np64(gate), np64(up))
    dg, du = ops.swiglu_bwd(dout.cuda(), gate.cuda(), up.cuda())
    assert np.all(np.abs(np64(dg) - wdg) <= 2.0 ** -8 * np.abs(wdg) + 1e-6)
    assert np.all(np.abs(np64(du) - wdu) <= 2.0 ** -8 * np.abs(wdu) + 1e-6)
    # fp32 storage: only the fp32 arithmetic error is left
    o32 = ops.swiglu_fwd(gate.float().cuda(), up.float().cuda())
    assert rel(o32.cpu().numpy(), want) < 1e-6
    dg32, du32 = ops.swiglu_bwd(dout.float().cuda(), gate.float().cuda(), up.float().cuda())
    assert rel(dg32.cpu().numpy(), wdg) < 1e-6 and rel(du32.cpu().numpy(), wdu) < 1e-6


def test_swiglu_tails_and_special_values():
    from axonn_amd import ops

    # the hardware exp / reciprocal pair is good to a few 1e-7 relative; below -88 the
    # exponential overflows and the result is the limit 0 instead of a value under 1e-36
    gate = torch.tensor([[-200.0, -90.0, -30.0, -1e-3, 0.0, 1e-3, 30.0, 200.0]] * 2)
    up = torch.full_like(gate, 1.5)
    out = ops.swiglu_fwd(gate.cuda(), up.cuda()).cpu().numpy()
    want = om.swiglu_forward(gate.numpy(), up.numpy())
    assert np.all(np.isfinite(out)) and np.allclose(out, want, rtol=5e-6, atol=1e-30)
    dg, du = ops.swiglu_bwd(torch.ones_like(gate).cuda(), gate.cuda(), up.cuda())
    wdg, wdu = om.swiglu_backward(np.ones(gate.shape), gate.numpy(), up.numpy())
    assert np.all(np.isfinite(dg.cpu().numpy())) and np.allclose(dg.cpu().numpy(), wdg, rtol=5e-6, atol=1e-30)
    assert np.allclose(du.cpu().numpy(), wdu, rtol=5e-6, atol=1e-30)


def test_swiglu_rejects_bad_arguments():
    from axonn_amd import ops

    a = torch.zeros(4, 12, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.swiglu_fwd(a, a)                       # 12 columns: not a multiple of 8
    b = torch.zeros(4, 16, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.swiglu_fwd(b, b.float())
    with pytest.raises(TypeError):
        ops.swiglu_fwd(b.double(), b.double())
    with pytest.raises(RuntimeError):
        ops.swiglu_fwd(b.cpu(), b.cpu())


@pytest.mark.parametrize("M,H,I", [(48, 64, 160), (512, 256, 768)])
def test_patched_llama_mlp_block_matches_oracle(M, H, I):
    """LlamaMLP built inside `parallelize` has the three projections on the GEMM
    kernels and the fused SwiGLU between them; forward and backward against the
    oracle block with bf16 storage between the stages."""
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaMLP

    import axonn_amd.axonn as ax
    from axonn_amd.intra_layer import Linear
    from axonn_amd.models.transformers import parallelize

    ax.init(1, 1, 1, 1)
    cfg = LlamaConfig(hidden_size=H, intermediate_size=I, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=32)
    original_forward = LlamaMLP.forward
    with parallelize(cfg):
        mlp = LlamaMLP(cfg)
    assert LlamaMLP.forward is original_forward          # the patch is undone on exit
    assert isinstance(mlp.gate_proj, Linear) and mlp.gate_proj.weight.dim() == 1
    from axonn_amd.models.transformers.modify_llama import modified_mlp_forward
    mlp.forward = modified_mlp_forward.__get__(mlp)      # the instance keeps the fused forward
    mlp = mlp.cuda().bfloat16()
    g = torch.Generator(device="cuda").manual_seed(M)
    x = torch.randn(M, H, generator=g, device="cuda").bfloat16().requires_grad_(True)
    dy = (torch.randn(M, H, generator=g, device="cuda") * 0.1).bfloat16()
    y = mlp(x)
    y.backward(dy)
    wg, wu, wd = (np64(p).reshape(-1) for p in (mlp.gate_proj.weight, mlp.up_proj.weight, mlp.down_proj.weight))
    fwd = om.llama_mlp_forward(np64(x), wg, wu, wd, H, I, store="bf16")
    bwd = om.llama_mlp_backward(np64(x), wg, wu, wd, H, I, np64(dy), fwd, store="bf16")
    assert rel(np64(y), fwd["out"]) < 1e-2
    assert rel(np64(x.grad), bwd["dx"]) < 1e-2
    for key, lin in (("dw_gate", mlp.gate_proj), ("dw_up", mlp.up_proj), ("dw_down", mlp.down_proj)):
        assert rel(np64(lin.weight.grad), bwd[key]) < 1e-2
    # and the same block on Hugging Face's own forward (two elementwise kernels of torch)
    with torch.no_grad():
        y_ref = mlp.down_proj(torch.nn.functional.silu(mlp.gate_proj(x)) * mlp.up_proj(x))
    assert rel(np64(y), np64(y_ref)) < 1e-2


def test_patched_attention_projections_are_linear_layers():
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaAttention

    import axonn_amd.axonn as ax
    from axonn_amd.intra_layer import Linear
    from axonn_amd.models.transformers import parallelize

    ax.init(1, 1, 1, 1)
    cfg = LlamaConfig(hidden_size=64, intermediate_size=128, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=32)
    with parallelize(cfg):
        attn = LlamaAttention(cfg, 0)
    for name, shape in (("q_proj", (64, 64)), ("k_proj", (32, 64)), ("v_proj", (32, 64)), ("o_proj", (64, 64))):
        lin = getattr(attn, name)
        assert isinstance(lin, Linear) and lin.weight.numel() == shape[0] * shape[1]
    assert not isinstance(LlamaAttention(cfg, 0).q_proj, Linear)


def test_tiny_llama_model_under_parallelize_matches_its_torch_twin():
    """A 2-layer LlamaForCausalLM built inside `parallelize` (all 7 projections of
    each layer on the GEMM kernels, the fused SwiGLU in the MLP) against the same
    model built from torch.nn.Linear with the same weights: logits, loss and the
    gradients of every projection, bf16 on the GPU, normwise 2e-2 (two models in
    bf16 differ by rounding in every layer; the oracle-level bar is applied to the
    block in the test above)."""
    from transformers import LlamaConfig, LlamaForCausalLM

    import axonn_amd.axonn as ax
    from axonn_amd.intra_layer import Linear
    from axonn_amd.models.transformers import parallelize

    ax.init(1, 1, 1, 1)
    cfg = LlamaConfig(hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=2, vocab_size=128, max_position_embeddings=64,
                      architectures=["LlamaForCausalLM"])
    cfg._attn_implementation = "eager"
    torch.manual_seed(0)
    ref = LlamaForCausalLM(cfg)
    with parallelize(cfg):
        ours = LlamaForCausalLM(cfg)
    n_lin = sum(isinstance(m, Linear) for m in ours.modules())
    assert n_lin == 2 * 7
    missing = ours.load_state_dict(ref.state_dict(), strict=True)   # 2-D weights into the flat parameters
    assert not missing.missing_keys and not missing.unexpected_keys
    ref, ours = ref.cuda().bfloat16(), ours.cuda().bfloat16()
    ids = torch.randint(0, 128, (4, 32), generator=torch.Generator().manual_seed(1)).cuda()
    out_r = ref(input_ids=ids, labels=ids)
    out_o = ours(input_ids=ids, labels=ids)
    assert rel(np64(out_o.logits), np64(out_r.logits)) < 2e-2
    assert abs(out_o.loss.item() - out_r.loss.item()) < 2e-2 * abs(out_r.loss.item())
    out_r.loss.backward()
    out_o.loss.backward()
    for (name, p_r), (_, p_o) in zip(ref.named_parameters(), ours.named_parameters()):
        assert rel(np64(p_o.grad).reshape(-1), np64(p_r.grad).reshape(-1)) < 5e-2, name


def test_auto_parallelize_builds_hugging_face_mlp_on_the_kernels():
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaMLP

    import axonn_amd.axonn as ax
    from axonn_amd.intra_layer import Linear, auto_parallelize

    ax.init(1, 1, 1, 1)
    cfg = LlamaConfig(hidden_size=128, intermediate_size=256, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=32)
    with auto_parallelize():
        mlp = LlamaMLP(cfg)
    assert all(isinstance(getattr(mlp, n), Linear) for n in ("gate_proj", "up_proj", "down_proj"))
    mlp = mlp.cuda().bfloat16()
    x = torch.randn(64, 128, generator=torch.Generator().manual_seed(2)).cuda().bfloat16()
    y = mlp(x)
    wg, wu, wd = (np64(p).reshape(-1) for p in (mlp.gate_proj.weight, mlp.up_proj.weight, mlp.down_proj.weight))
    fwd = om.llama_mlp_forward(np64(x), wg, wu, wd, 128, 256, store="bf16")
    assert rel(np64(y), fwd["out"]) < 1e-2


def _twin_models(family):
    from transformers import MistralConfig, MixtralConfig, OPTConfig
    from transformers.models.mistral.modeling_mistral import MistralForCausalLM
    from transformers.models.mixtral.modeling_mixtral import MixtralForCausalLM
    from transformers.models.opt.modeling_opt import OPTForCausalLM

    common = dict(hidden_size=256, num_attention_heads=4, num_hidden_layers=2, vocab_size=128,
                  max_position_embeddings=64)
    if family == "mistral":
        return MistralForCausalLM, MistralConfig(intermediate_size=512, num_key_value_heads=2,
                                                 architectures=["MistralForCausalLM"], **common), 2 * 7
    if family == "opt":
        # OPT has dropout by default: off, so that the two models see the same function
        return OPTForCausalLM, OPTConfig(ffn_dim=512, word_embed_proj_dim=256, dropout=0.0,
                                         attention_dropout=0.0, layerdrop=0.0,
                                         architectures=["OPTForCausalLM"], **common), 2 * 6
    return MixtralForCausalLM, MixtralConfig(intermediate_size=512, num_key_value_heads=2, num_local_experts=4,
                                             architectures=["MixtralForCausalLM"], **common), 2 * 4


@pytest.mark.parametrize("family", ["mistral", "opt", "mixtral"])
def test_other_model_families_under_parallelize_match_their_torch_twins(family):
    """The reference patches OPT, Mistral and Mixtral as it patches Llama
    (axonn/models/transformers/__init__.py:22-39): a 2-layer model of each family built
    inside `parallelize` against the same model from torch.nn.Linear with the same
    weights; bf16, logits normwise 2e-2, gradients 5e-2, as for Llama above."""
    import axonn_amd.axonn as ax
    from axonn_amd.intra_layer import Linear
    from axonn_amd.models.transformers import parallelize

    ax.init(1, 1, 1, 1)
    cls, cfg, n_expected = _twin_models(family)
    cfg._attn_implementation = "eager"
    torch.manual_seed(0)
    ref = cls(cfg)
    with parallelize(cfg):
        ours = cls(cfg)
    assert sum(isinstance(m, Linear) for m in ours.modules()) == n_expected
    assert not any(isinstance(m, Linear) for m in cls(cfg).modules())   # the patch is undone
    missing = ours.load_state_dict(ref.state_dict(), strict=True)
    assert not missing.missing_keys and not missing.unexpected_keys
    ref, ours = ref.cuda().bfloat16(), ours.cuda().bfloat16()
    ids = torch.randint(0, 128, (4, 32), generator=torch.Generator().manual_seed(1)).cuda()
    out_r = ref(input_ids=ids, labels=ids)
    out_o = ours(input_ids=ids, labels=ids)
    assert rel(np64(out_o.logits), np64(out_r.logits)) < 2e-2
    assert abs(out_o.loss.item() - out_r.loss.item()) < 2e-2 * abs(out_r.loss.item())
    out_r.loss.backward()
    out_o.loss.backward()
    for (name, p_r), (_, p_o) in zip(ref.named_parameters(), ours.named_parameters()):
        if p_r.grad is None:
            assert p_o.grad is None, name
            continue
        assert rel(np64(p_o.grad).reshape(-1), np64(p_r.grad).reshape(-1)) < 5e-2, name


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", [(256, 128, 64), (512, 384, 192), (4096, 1792, 256), (2048, 4096, 128),
                                   (4096, 8192, 64)])
def test_gate_up_forward_in_one_launch_equals_the_three_calls(M, N, K, dtype):
    """axn_gemm_swiglu_fwd against axn_gemm_fwd twice + axn_swiglu_fwd: output and both
    saved pre-activations bit for bit (1, 6, 224, 256 and 1024 workgroups: less than a
    round, one round, four rounds), with a row-strided input; and against float64."""
    from axonn_amd import ops

    g = torch.Generator(device="cuda").manual_seed(M + N + K)
    xb = torch.randn(M, 2 * K, device="cuda", generator=g).to(dtype)
    x = xb[:, K:]
    wg = (torch.randn(N, K, device="cuda", generator=g) * 0.2).to(dtype)
    wu = (torch.randn(N, K, device="cuda", generator=g) * 0.2).to(dtype)
    assert ops.gemm_swiglu_supported(M, N, K, dtype)
    h, gate, up = ops.gemm_swiglu_fwd(x, wg, wu)
    gate_ref, _ = ops.gemm_fwd(x, wg)
    up_ref, _ = ops.gemm_fwd(x, wu)
    assert torch.equal(gate, gate_ref) and torch.equal(up, up_ref)
    assert torch.equal(h, ops.swiglu_fwd(gate_ref, up_ref))
    h2, none_g, none_u = ops.gemm_swiglu_fwd(x, wg, wu, save=False)
    assert none_g is None and none_u is None and torch.equal(h2, h)
    want = om.swiglu_forward(np64(x) @ np64(wg).T, np64(x) @ np64(wu).T)
    assert rel(np64(h), want) < 1e-2


def test_gate_up_forward_rejects_what_it_cannot_run():
    from axonn_amd import ops

    assert not ops.gemm_swiglu_supported(255, 128, 64, torch.bfloat16)
    assert not ops.gemm_swiglu_supported(256, 64, 64, torch.bfloat16)
    assert not ops.gemm_swiglu_supported(256, 128, 32, torch.bfloat16)
    assert not ops.gemm_swiglu_supported(256, 128, 64, torch.float32)
    x = torch.zeros(128, 64, device="cuda", dtype=torch.bfloat16)
    w = torch.zeros(128, 64, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(nv.AxnError, match="M % 256 == 0") as e:
        ops.gemm_swiglu_fwd(x, w, w)
    assert e.value.code == nv.AXN_ESHAPE
    with pytest.raises(TypeError, match="bf16 or fp16"):
        ops.gemm_swiglu_fwd(x.float(), w.float(), w.float())


def test_mlp_with_one_launch_gate_up_equals_the_separate_path(monkeypatch):
    """The patched MLP at a whole-tile shape takes the one-launch gate/up forward; with
    that path switched off it takes three launches.  Output and weight gradients agree bit
    for bit; the input gradient is the sum of two products, which the one-launch path
    adds in the accumulators (one rounding) and autograd adds after rounding each."""
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaMLP

    import axonn_amd.axonn as ax
    from axonn_amd import ops
    from axonn_amd.models.transformers import modify_llama, parallelize

    ax.init(1, 1, 1, 1)
    cfg = LlamaConfig(hidden_size=128, intermediate_size=384, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=32)
    with parallelize(cfg):
        mlp = LlamaMLP(cfg)
    mlp.forward = modify_llama.modified_mlp_forward.__get__(mlp)
    mlp = mlp.cuda().bfloat16()
    g = torch.Generator(device="cuda").manual_seed(5)
    x0 = torch.randn(2, 128, 128, generator=g, device="cuda").bfloat16()     # 256 tokens
    dy = (torch.randn(2, 128, 128, generator=g, device="cuda") * 0.1).bfloat16()

    def run():
        for p in mlp.parameters():
            p.grad = None
        x = x0.clone().requires_grad_(True)
        y = mlp(x)
        y.backward(dy)
        return [y.detach(), x.grad] + [p.grad.clone() for p in mlp.parameters()]

    calls = []
    real = ops.gemm_swiglu_fwd
    monkeypatch.setattr(ops, "gemm_swiglu_fwd", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    fused = run()
    assert calls, "the one-launch path was not taken"
    monkeypatch.setattr(ops, "gemm_swiglu_supported", lambda *a: False)
    n = len(calls)
    separate = run()
    assert len(calls) == n
    for i, (a, b) in enumerate(zip(fused, separate)):
        if i == 1:   # x.grad: one pass and one rounding against two rounded products added
            assert rel(np64(a), np64(b)) < 1e-2
        else:
            assert torch.equal(a, b), i
    # a 3-token input does not qualify and still works
    monkeypatch.undo()
    assert mlp(x0[0, :3]).shape == (3, 128)


def test_gate_up_forward_in_one_launch_at_the_llama_3_8b_shape():
    """4096 tokens, 4096 -> 14336 (1792 workgroups, seven rounds): output and both saved
    pre-activations equal the three separate calls bit for bit, and sampled rows equal the
    float64 oracle."""
    from axonn_amd import ops

    M, N, K = 4096, 14336, 4096
    g = torch.Generator(device="cuda").manual_seed(8)
    x = torch.randn(M, K, device="cuda", generator=g).bfloat16()
    wg = (torch.randn(N, K, device="cuda", generator=g) * 0.02).bfloat16()
    wu = (torch.randn(N, K, device="cuda", generator=g) * 0.02).bfloat16()
    h, gate, up = ops.gemm_swiglu_fwd(x, wg, wu)
    gate_ref, _ = ops.gemm_fwd(x, wg)
    up_ref, _ = ops.gemm_fwd(x, wu)
    assert torch.equal(gate, gate_ref) and torch.equal(up, up_ref)
    assert torch.equal(h, ops.swiglu_fwd(gate_ref, up_ref))
    rows = torch.tensor([0, 255, 256, 1777, 4095], device="cuda")
    want = om.swiglu_forward(np64(x[rows]) @ np64(wg).T, np64(x[rows]) @ np64(wu).T)
    assert rel(np64(h[rows]), want) < 1e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,N1,N2", [(256, 256, 128, 64), (128, 128, 192, 448), (4096, 2304, 192, 128),
                                       (4096, 6144, 128, 128), (6144, 4096, 256, 64), (2304, 2048, 320, 320),
                                       (512, 1024, 2048, 2048)])
def test_two_term_input_gradient_in_one_pass(M, K, N1, N2, dtype):
    """dX = dY1 W1 + dY2 W2 through axn_gemm_dgrad_pair on the 128 x 128, 256 x 256 and
    256 x 128 tiles and on problems cut along the columns and along the rows (384 large
    tiles), the two gradients being column blocks of one buffer (unequal widths, one
    leading dimension): against float64, and within one rounding of the two separate
    products added."""
    from axonn_amd import ops

    g = torch.Generator(device="cuda").manual_seed(M + K + N1 + N2)
    dyb = (torch.randn(M, N1 + N2, device="cuda", generator=g) * 0.1).to(dtype)
    dy1, dy2 = dyb[:, :N1], dyb[:, N1:]
    w1 = (torch.randn(N1, K, device="cuda", generator=g) * 0.1).to(dtype)
    w2 = (torch.randn(N2, K, device="cuda", generator=g) * 0.1).to(dtype)
    assert ops.gemm_dgrad_pair_supported(M, N1, N2, K, dtype)
    dx = ops.gemm_dgrad_pair(dy1, w1, dy2, w2)
    want = dy1.double() @ w1.double() + dy2.double() @ w2.double()
    tol = 1e-2 if dtype == torch.bfloat16 else 1.5e-3
    assert rel(np64(dx), np64(want)) < tol
    err = (dx.double() - want).abs().max() / want.abs().max()
    assert float(err) < (1e-2 if dtype == torch.bfloat16 else 2e-3)
    two = ops.gemm_dgrad(dy1.contiguous(), w1)
    two += ops.gemm_dgrad(dy2.contiguous(), w2)
    assert rel(np64(dx), np64(two)) < tol
    # one pass rounds once: it is at least as close to the exact sum as the added pair
    assert rel(np64(dx), np64(want)) <= rel(np64(two), np64(want)) * 1.05


def test_two_term_input_gradient_falls_back_and_rejects():
    from axonn_amd import ops

    g = torch.Generator(device="cuda").manual_seed(3)
    dy1 = torch.randn(48, 40, device="cuda", generator=g).bfloat16()
    dy2 = torch.randn(48, 24, device="cuda", generator=g).bfloat16()
    w1 = torch.randn(40, 56, device="cuda", generator=g).bfloat16()
    w2 = torch.randn(24, 56, device="cuda", generator=g).bfloat16()
    assert not ops.gemm_dgrad_pair_supported(48, 40, 24, 56, torch.bfloat16)
    dx = ops.gemm_dgrad_pair(dy1, w1, dy2, w2)       # two products and an add
    want = dy1.double() @ w1.double() + dy2.double() @ w2.double()
    assert rel(np64(dx), np64(want)) < 1e-2
    lib = nv.load()
    rc = lib.axn_gemm_dgrad_pair(dy1.data_ptr(), w1.data_ptr(), dy2.data_ptr(), w2.data_ptr(), dx.data_ptr(),
                                 nv.BF16, 48, 40, 24, 56, 40, 56, 56, nv.current_stream())
    assert rc == nv.AXN_ESHAPE and "gemm_pair" in lib.axn_last_error().decode()


def test_mlp_backward_with_accumulating_weight_gradients(monkeypatch):
    """Two micro-batches through the patched MLP under overlap_reduce_scatter (the wgrad
    kernels add into weight.grad): the one-launch paths against the separate ones."""
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaMLP

    import axonn_amd.axonn as ax
    from axonn_amd import ops
    from axonn_amd.intra_layer import optimize_communication
    from axonn_amd.models.transformers import modify_llama, parallelize

    ax.init(1, 1, 1, 1)
    cfg = LlamaConfig(hidden_size=128, intermediate_size=256, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=32)
    with parallelize(cfg):
        mlp = LlamaMLP(cfg)
    mlp.forward = modify_llama.modified_mlp_forward.__get__(mlp)
    mlp = mlp.cuda().bfloat16()
    g = torch.Generator(device="cuda").manual_seed(6)
    xs = [torch.randn(256, 128, generator=g, device="cuda").bfloat16() for _ in range(2)]
    dys = [(torch.randn(256, 128, generator=g, device="cuda") * 0.1).bfloat16() for _ in range(2)]

    def run():
        for p in mlp.parameters():
            p.grad = None
        with optimize_communication(overlap_reduce_scatter=True, model_object_for_overlapping_allgathers=mlp):
            for x, dy in zip(xs, dys):
                mlp(x).backward(dy)
        return [p.grad.clone() for p in mlp.parameters()]

    calls = []
    real = ops.gemm_wgrad
    monkeypatch.setattr(ops, "gemm_wgrad", lambda *a, **k: (calls.append(k.get("accumulate", False)), real(*a, **k))[1])
    # (a layer that also needs its input gradient asks for both through ops.gemm_bwd)
    real_bwd = ops.gemm_bwd
    monkeypatch.setattr(ops, "gemm_bwd", lambda *a, **k: (calls.append(k.get("accumulate", False)), real_bwd(*a, **k))[1])
    fused = run()
    # three weights, two micro-batches: the first assigns, the second accumulates in the kernel
    assert sorted(calls) == [False] * 3 + [True] * 3, calls
    monkeypatch.setattr(ops, "gemm_swiglu_supported", lambda *a: False)
    separate = run()
    for a, b in zip(fused, separate):
        assert rel(np64(a), np64(b)) < 1e-2
