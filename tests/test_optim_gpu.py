"""Parity of the multi-tensor optimizer kernels (through the C ABI) with the CPU
oracle: overflow flag bit-exact, master weights within 1e-6 relative
(max |p - p_ref| / max |p_ref|), skip path bit-identical, low-precision copy
equal to the rounding of the master weights."""

import numpy as np
import pytest
import torch

from oracle import linear as ol
from oracle import optim as oo

pytestmark = pytest.mark.gpu

P_TOL = 1e-6


def flat_views(flat, sizes, start=0):
    out, off = [], start
    for n in sizes:
        out.append(flat[off:off + n])
        off += n
    return out


def make_state(sizes, seed, g_dtype=torch.bfloat16, scale=65536.0, start=0):
    """Flat buffers with every tensor a view at an arbitrary element offset
    (axonn/utils.py:11-30 layout, shifted by `start` to vary the alignment)."""
    g = torch.Generator().manual_seed(seed)
    total = sum(sizes) + start
    P = torch.randn(total, generator=g) * 0.02
    G = (torch.randn(total, generator=g) * 1e-3 * scale).to(g_dtype)
    M = torch.randn(total, generator=g) * 1e-4
    V = torch.rand(total, generator=g) * 1e-7
    return P, G, M, V


def run_oracle(P, G, M, V, sizes, start, step, scale, max_norm, g_dtype, p_dtype="bf16", wd=0.0):
    sl = lambda t: [v.numpy().copy() for v in flat_views(t.float(), sizes, start)]
    return oo.mixed_precision_step(sl(G), sl(P), sl(M), sl(V), step, scale, g_dtype=g_dtype,
                                   p_dtype=p_dtype, max_norm=max_norm, weight_decay=wd)


def run_hip(P, G, M, V, sizes, start, step, scale, max_norm, plow_dtype=torch.bfloat16, wd=0.0):
    from axonn_amd import ops

    Pd, Gd, Md, Vd = P.cuda(), G.cuda(), M.cuda(), V.cuda()
    PL = torch.zeros(P.numel(), dtype=plow_dtype, device="cuda")
    scan = ops.mt_scan(flat_views(Gd, sizes, start), 1.0 / scale, max_norm)
    hp = ops.adam_hparams(step, 1e-3, 0.9, 0.999, 1e-8, wd)
    ops.mt_adam(flat_views(Gd, sizes, start), flat_views(Pd, sizes, start),
                flat_views(Md, sizes, start), flat_views(Vd, sizes, start),
                flat_views(PL, sizes, start), hp, inv_scale=1.0 / scale, scan=scan)
    return Pd, Md, Vd, PL, scan


def check_against_oracle(res, Pd, Md, Vd, PL, scan, sizes, start, lowp="bf16"):
    assert int(scan.found_inf.item()) == int(res["overflow"])
    assert abs(float(scan.total_norm.item()) - res["total_norm"]) <= 1e-5 * res["total_norm"]
    assert abs(float(scan.clip_coef.item()) - res["clip_coef"]) <= 1e-5 * res["clip_coef"]
    got_p = np.concatenate([v.cpu().numpy() for v in flat_views(Pd, sizes, start)])
    ref_p = np.concatenate(res["p"])
    assert np.max(np.abs(got_p - ref_p)) / np.max(np.abs(ref_p)) <= P_TOL
    got_m = np.concatenate([v.cpu().numpy() for v in flat_views(Md, sizes, start)])
    got_v = np.concatenate([v.cpu().numpy() for v in flat_views(Vd, sizes, start)])
    assert np.allclose(got_m, np.concatenate(res["m"]), rtol=1e-5, atol=1e-9)
    assert np.allclose(got_v, np.concatenate(res["v"]), rtol=1e-5, atol=1e-14)
    got_pl = np.concatenate([v.float().cpu().numpy() for v in flat_views(PL, sizes, start)])
    want_pl = ol.round_to(got_p, lowp).astype(np.float32)
    assert np.array_equal(got_pl, want_pl)  # cast-back is exactly the rounding of p


SIZE_SETS = [
    [1], [7], [8], [9], [4099, 1, 33, 16384, 16385, 7, 100000],
    [16384 * 3 + 5, 2, 70001], [300000, 250001],
]


@pytest.mark.parametrize("sizes", SIZE_SETS)
@pytest.mark.parametrize("start", [0, 1, 3])
def test_step_matches_oracle_ragged_layouts(sizes, start):
    P, G, M, V = make_state(sizes, seed=len(sizes) + start, start=start)
    res = run_oracle(P, G, M, V, sizes, start, 3, 65536.0, 1.0, "bf16")
    out = run_hip(P, G, M, V, sizes, start, 3, 65536.0, 1.0)
    check_against_oracle(res, *out, sizes, start)
    # elements outside the views (the `start` prefix) are untouched
    if start:
        assert torch.equal(out[0][:start].cpu(), P[:start])


@pytest.mark.parametrize("count", [2, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 130])
def test_every_row_of_the_tensor_table_is_found(count):
    """The update kernel finds a chunk's tensor in two steps (a quarter of the 64-row table,
    then a row of it): tensor counts on both sides of every quarter, tensors of less than
    one chunk, of exactly one (256 elements), and of several with a ragged end, and more
    tensors than one launch holds."""
    rng = np.random.default_rng(count)
    sizes = [int(rng.choice([1, 5, 255, 256, 1023, 1024, 1025, 2048, 4097, 5000])) for _ in range(count)]
    P, G, M, V = make_state(sizes, seed=100 + count)
    res = run_oracle(P, G, M, V, sizes, 0, 2, 65536.0, 1.0, "bf16")
    out = run_hip(P, G, M, V, sizes, 0, 2, 65536.0, 1.0)
    check_against_oracle(res, *out, sizes, 0)


@pytest.mark.parametrize("g_dtype,name", [(torch.float16, "f16"), (torch.float32, "f32")])
def test_step_other_gradient_dtypes(g_dtype, name):
    sizes = [5001, 17, 40000]
    scale = 1024.0
    P, G, M, V = make_state(sizes, seed=5, g_dtype=g_dtype, scale=scale)
    res = run_oracle(P, G, M, V, sizes, 0, 2, scale, 0.5, name, p_dtype="f16", wd=0.01)
    out = run_hip(P, G, M, V, sizes, 0, 2, scale, 0.5, plow_dtype=torch.float16, wd=0.01)
    check_against_oracle(res, *out, sizes, 0, lowp="f16")


def test_no_clip_and_no_scan():
    from axonn_amd import ops

    sizes = [1000, 3000]
    P, G, M, V = make_state(sizes, seed=6, scale=1.0)
    res = run_oracle(P, G, M, V, sizes, 0, 1, 1.0, 0.0, "bf16")
    Pd, Gd, Md, Vd = P.cuda(), G.cuda(), M.cuda(), V.cuda()
    hp = ops.adam_hparams(1, 1e-3, 0.9, 0.999, 1e-8, 0.0)
    ops.mt_adam(flat_views(Gd, sizes), flat_views(Pd, sizes), flat_views(Md, sizes),
                flat_views(Vd, sizes), None, hp, inv_scale=1.0, scan=None)
    ref = np.concatenate(res["p"])
    assert np.max(np.abs(Pd.cpu().numpy() - ref)) / np.max(np.abs(ref)) <= P_TOL
    assert res["clip_coef"] == 1.0


@pytest.mark.parametrize("bad", [float("inf"), float("-inf"), float("nan")])
@pytest.mark.parametrize("where", [(0, 0), (3, 16383), (6, 99999), (2, 32)])
def test_overflow_skips_the_whole_step(bad, where):
    sizes = SIZE_SETS[4]
    P, G, M, V = make_state(sizes, seed=9)
    t, i = where
    off = sum(sizes[:t]) + i
    G[off] = bad
    res = run_oracle(P, G, M, V, sizes, 0, 2, 65536.0, 1.0, "bf16")
    assert res["overflow"] is True
    Pd, Md, Vd, PL, scan = run_hip(P, G, M, V, sizes, 0, 2, 65536.0, 1.0)
    assert int(scan.found_inf.item()) == 1
    # nothing was written: bit-identical to the state before the step
    assert torch.equal(Pd.cpu(), P) and torch.equal(Md.cpu(), M) and torch.equal(Vd.cpu(), V)
    assert torch.count_nonzero(PL) == 0


def test_overflow_flag_cases_match_reference_semantics():
    """The flag restates `s = tensor.sum(); isinf(s) + isnan(s)` per tensor
    (axonn/inter_layer.py:435-445) - including finite fp16 elements whose sum
    leaves the fp16 range."""
    from axonn_amd import ops

    cases = [
        (torch.float16, [1.0, -2.0, 3.0], False),
        (torch.float16, [30000.0] * 2, False),
        (torch.float16, [30000.0] * 4, True),       # sum 120000 > 65504
        (torch.float16, [30000.0, 30000.0, 30000.0, -30000.0], False),
        (torch.bfloat16, [30000.0] * 4, False),     # bf16 has the range
        (torch.bfloat16, [3.0e38, 3.0e38], True),
        (torch.float32, [3.0e38, 3.0e38], True),
        (torch.float32, [1e30, float("inf"), -float("inf")], True),
        (torch.bfloat16, [0.0, float("nan")], True),
    ]
    for dt, vals, want in cases:
        t = torch.tensor(vals, dtype=dt)
        assert oo.check_nan(t.double().numpy(), {torch.float16: "f16", torch.bfloat16: "bf16",
                                                 torch.float32: "f32"}[dt]) == want
        s = t.sum()
        assert bool(torch.isinf(s) | torch.isnan(s)) == want   # what the reference computes
        scan = ops.mt_scan([t.cuda()], 1.0, 0.0)
        assert int(scan.found_inf.item()) == int(want), (dt, vals)
    # per tensor, not over the list: two tensors of 2 x 30000 do not overflow
    a = torch.full((2,), 30000.0, dtype=torch.float16).cuda()
    assert int(ops.mt_scan([a, a.clone()], 1.0, 0.0).found_inf.item()) == 0


def test_random_flag_agreement():
    from axonn_amd import ops

    rng = np.random.default_rng(0)
    for trial in range(30):
        sizes = [int(n) for n in rng.integers(1, 40000, size=rng.integers(1, 6))]
        G = (torch.randn(sum(sizes)) * 50).bfloat16()
        if trial % 2:
            G[int(rng.integers(sum(sizes)))] = [float("inf"), float("-inf"), float("nan")][trial % 3]
        want = any(oo.check_nan(v.double().numpy(), "bf16") for v in flat_views(G, sizes))
        got = int(ops.mt_scan(flat_views(G.cuda(), sizes), 1.0, 0.0).found_inf.item())
        assert got == int(want)


def test_multi_step_trajectory_against_torch_adam():
    from axonn_amd import ops

    torch.manual_seed(12)
    sizes = [1234, 777, 20001]
    total = sum(sizes)
    p_ref = [torch.nn.Parameter(torch.randn(n) * 0.02) for n in sizes]
    opt = torch.optim.Adam(p_ref, lr=1e-3, foreach=False)
    Pd = torch.cat([p.detach() for p in p_ref]).cuda()
    Md, Vd = torch.zeros(total, device="cuda"), torch.zeros(total, device="cuda")
    PL = torch.zeros(total, dtype=torch.bfloat16, device="cuda")
    for step in range(1, 9):
        G = (torch.randn(total) * 1e-3 * 4096.0).bfloat16()
        for p, g in zip(p_ref, flat_views(G, sizes)):
            p.grad = g.float() / 4096.0
        opt.step()
        Gd = G.cuda()
        scan = ops.mt_scan(flat_views(Gd, sizes), 1.0 / 4096.0, 0.0)
        hp = ops.adam_hparams(step, 1e-3, 0.9, 0.999, 1e-8, 0.0)
        ops.mt_adam(flat_views(Gd, sizes), flat_views(Pd, sizes), flat_views(Md, sizes),
                    flat_views(Vd, sizes), flat_views(PL, sizes), hp, 1.0 / 4096.0, scan)
        ref = torch.cat([p.detach() for p in p_ref]).numpy()
        assert np.max(np.abs(Pd.cpu().numpy() - ref)) / np.max(np.abs(ref)) <= P_TOL


def test_more_tensors_than_one_launch_holds():
    """Lists longer than the per-launch table (64 tensors) are split."""
    sizes = [37 + (i * 13) % 200 for i in range(150)]
    P, G, M, V = make_state(sizes, seed=13)
    res = run_oracle(P, G, M, V, sizes, 0, 1, 65536.0, 1e-3, "bf16")
    out = run_hip(P, G, M, V, sizes, 0, 1, 65536.0, 1e-3)
    check_against_oracle(res, *out, sizes, 0)


def test_unaligned_separate_allocations_take_the_scalar_path():
    """Pointers whose misalignments disagree (g at +1 element, p at +0) cannot
    share one vector phase; the result must still be right."""
    from axonn_amd import ops

    n = 5000
    g = torch.Generator().manual_seed(14)
    Gbuf = (torch.randn(n + 1, generator=g) * 65.0).bfloat16().cuda()
    P = (torch.randn(n, generator=g) * 0.02)
    Pd, Md, Vd = P.cuda(), torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    Gv = Gbuf[1:]
    res = oo.mixed_precision_step([Gv.float().cpu().numpy()], [P.numpy()], [np.zeros(n, np.float32)],
                                  [np.zeros(n, np.float32)], 1, 65536.0, max_norm=1.0)
    scan = ops.mt_scan([Gv], 1.0 / 65536.0, 1.0)
    ops.mt_adam([Gv], [Pd], [Md], [Vd], None, ops.adam_hparams(1, 1e-3, 0.9, 0.999, 1e-8, 0.0),
                1.0 / 65536.0, scan)
    assert np.max(np.abs(Pd.cpu().numpy() - res["p"][0])) / np.max(np.abs(res["p"][0])) <= P_TOL


def test_mt_scale_unscale_and_clip():
    from axonn_amd import ops

    sizes = [1001, 9, 30000]
    G = (torch.randn(sum(sizes)) * 40.0).half()
    Gd = G.cuda()
    ov, un = oo.unscale_gradients([v.double().numpy() for v in flat_views(G, sizes)], "f16", 1024.0)
    ops.mt_scale(flat_views(Gd, sizes), 1.0 / 1024.0)
    assert np.array_equal(Gd.double().cpu().numpy(), np.concatenate(un))  # power of two: exact
    total, clipped = oo.clip_grad_norm_(un, 0.5, "f32")
    scan = ops.mt_scan(flat_views(Gd, sizes), 1.0, 0.5)
    ops.mt_scale(flat_views(Gd, sizes), 1.0, scan=scan, use_clip=True)
    assert abs(float(scan.total_norm.item()) - total) <= 1e-3 * total  # oracle norms are fp16-rounded inputs
    want = ol.round_to(np.concatenate(un) * float(scan.clip_coef.item()), "f16")
    assert np.array_equal(Gd.double().cpu().numpy(), want)


def test_clip_grad_norm_matches_torch():
    from axonn_amd.intra_layer import clip_grad_norm_

    torch.manual_seed(15)
    ps = [torch.nn.Parameter(torch.randn(n).cuda()) for n in (33, 4097, 12)]
    qs = [torch.nn.Parameter(p.detach().clone()) for p in ps]
    for p, q in zip(ps, qs):
        p.grad = torch.randn_like(p)
        q.grad = p.grad.clone()
    n1 = clip_grad_norm_(ps, 1e-3)
    n2 = torch.nn.utils.clip_grad_norm_(qs, 1e-3)
    assert abs(float(n1) - float(n2)) <= 1e-6 * float(n2)
    for p, q in zip(ps, qs):
        assert torch.allclose(p.grad, q.grad, rtol=1e-6, atol=0)
    # mixed dtypes in one list
    g16 = ps[1].grad.bfloat16()
    ps[1] = torch.nn.Parameter(ps[1].detach().bfloat16())
    ps[1].grad = g16
    want = float(torch.sqrt(sum((p.grad.double() ** 2).sum() for p in ps)))
    assert abs(float(clip_grad_norm_(ps, 1e9)) - want) <= 1e-5 * want


def test_cpuadam_class_end_to_end():
    """bf16 model, flat HBM state, clip + static loss scale: three steps equal
    the oracle fed with the same gradients."""
    from axonn_amd.inter_layer import LossScaler
    from axonn_amd.intra_layer import Linear
    from axonn_amd.optim import CPUAdam

    torch.manual_seed(16)
    model = torch.nn.Sequential(Linear(64, 136), Linear(136, 72)).cuda().bfloat16()
    scale = 1024.0
    opt = CPUAdam(model.parameters(), lr=1e-3, max_grad_norm=1.0,
                  loss_scaler=LossScaler(loss_scale=scale), dynamic_loss_scale=False)
    params = list(model.parameters())
    assert all(p.data_ptr() >= opt.model_params_fp16.data_ptr() for p in params)
    assert opt.group_offsets == [0, sum(p.numel() for p in params)]
    p32 = [opt.model_params_fp32[o:o + n].cpu().numpy().copy() for o, n in opt._views]
    m = [np.zeros_like(a) for a in p32]
    v = [np.zeros_like(a) for a in p32]
    for step in (1, 2, 3):
        opt.zero_grad()
        x = torch.randn(40, 64).bfloat16().cuda()
        (model(x).float().pow(2).mean() * scale).backward()
        grads = [p.grad.float().cpu().numpy().copy() for p in params]
        res = oo.mixed_precision_step(grads, p32, m, v, step, scale, max_norm=1.0)
        opt.step()
        assert not opt.last_step_skipped and opt.step_count == step
        p32, m, v = res["p"], res["m"], res["v"]
        got = opt.model_params_fp32.cpu().numpy()
        ref = np.concatenate(p32)
        assert np.max(np.abs(got - ref)) / np.max(np.abs(ref)) <= P_TOL
        # the model's bf16 weights are exactly the rounding of the master weights
        # (and agree with the oracle's wherever the fp32 values agree to the bit)
        for p, (o, n), want in zip(params, opt._views, res["p_low"]):
            mine = p.detach().float().cpu().numpy().reshape(-1)
            assert np.array_equal(mine, ol.bf16_round(got[o:o + n]))
            same = got[o:o + n] == np.concatenate(p32)[o:o + n]
            assert np.array_equal(mine[same], want[same])
        assert abs(float(opt.grad_norm()) - res["total_norm"]) <= 1e-5 * res["total_norm"]


def test_cpuadam_dynamic_loss_scale_skips_and_halves():
    from axonn_amd.optim import CPUAdam

    torch.manual_seed(17)
    w = torch.nn.Parameter((torch.randn(1000) * 0.02).half().cuda())
    opt = CPUAdam([w])
    assert opt.dynamic_loss_scale and opt.loss_scale == 65536.0
    before = opt.model_params_fp32.clone()
    w.grad.copy_(torch.randn(1000).half())
    w.grad[17] = float("inf")
    opt.step()
    assert opt.last_step_skipped and opt.step_count == 0 and opt.loss_scale == 32768.0
    assert torch.equal(opt.model_params_fp32, before) and torch.count_nonzero(opt.exp_avg) == 0
    opt.zero_grad()
    w.grad.copy_((torch.randn(1000) * 3).half())
    opt.step()
    assert not opt.last_step_skipped and opt.step_count == 1
    assert not torch.equal(opt.model_params_fp32, before)
    assert opt.scaler.no_overflow_iters == 1


def test_grad_scaler_engine_unscale_and_gate():
    from axonn_amd.inter_layer import GradScalerEngine

    torch.manual_seed(18)
    model = torch.nn.Linear(16, 16).cuda().half()
    eng = GradScalerEngine(model, computation_dtype=torch.float16)
    for p in model.parameters():
        p.grad = (torch.randn_like(p.float()) * 100).half()
    want = [p.grad.clone().div_(eng.scaler.loss_scale) for p in model.parameters()]
    sgd = torch.optim.SGD(model.parameters(), lr=0.1)
    assert eng.step(sgd) is True
    for p, w in zip(model.parameters(), want):
        assert torch.equal(p.grad, w)           # division by 2^16 in fp16, exact
    next(model.parameters()).grad[0, 0] = float("nan")
    snapshot = [p.detach().clone() for p in model.parameters()]
    assert eng.step(sgd) is False and eng.scaler.loss_scale == 32768.0
    for p, s in zip(model.parameters(), snapshot):
        assert torch.equal(p, s)
    assert eng._check_nan(torch.tensor([1.0, float("inf")]).cuda()) is True
    assert eng._check_nan(torch.tensor([1.0, 2.0]).cuda()) is False


def test_full_size_adam_properties():
    """1.3e9-element configuration scaled to what a test should take (1/16):
    64 ragged tensors; checks a sampled oracle, idempotence of the skip path and
    that one +inf flips the step off."""
    from axonn_amd import ops

    rng = np.random.default_rng(0)
    frac = rng.random(64)
    sizes = np.clip((frac / frac.sum() * 1.3e9 / 16).astype(np.int64), 6250, 3750000) | 1
    sizes = [int(s) for s in sizes]
    total = sum(sizes)
    g = torch.Generator(device="cuda").manual_seed(1)
    P = torch.randn(total, generator=g, device="cuda") * 0.02
    G = (torch.randn(total, generator=g, device="cuda") * 1e-3 * 65536.0).bfloat16()
    M = torch.zeros(total, device="cuda")
    V = torch.zeros(total, device="cuda")
    PL = torch.zeros(total, dtype=torch.bfloat16, device="cuda")
    P0 = P.clone()
    vs = lambda t: flat_views(t, sizes)
    scan = ops.mt_scan(vs(G), 1.0 / 65536.0, 1.0)
    want_norm = float(torch.sqrt(((G.double() / 65536.0) ** 2).sum()))
    assert abs(float(scan.total_norm.item()) - want_norm) <= 1e-6 * want_norm
    hp = ops.adam_hparams(1, 1e-3, 0.9, 0.999, 1e-8, 0.0)
    ops.mt_adam(vs(G), vs(P), vs(M), vs(V), vs(PL), hp, 1.0 / 65536.0, scan)
    idx = torch.from_numpy(rng.choice(total, 20000, replace=False)).cuda()
    coef = float(scan.clip_coef.item())
    gs = (G[idx].float() / 65536.0).cpu().numpy()
    p1, m1, v1 = oo.adam_update(P0[idx].cpu().numpy(), (gs * np.float32(coef)).astype(np.float32),
                                np.zeros(20000, np.float32), np.zeros(20000, np.float32), 1)
    got = P[idx].cpu().numpy()
    assert np.max(np.abs(got - p1)) / np.max(np.abs(p1)) <= P_TOL
    assert torch.equal(PL, P.bfloat16())
    # skip path: one +inf in tensor 17 -> nothing written
    G[sum(sizes[:17]) + 5] = float("inf")
    P1, M1, V1 = P.clone(), M.clone(), V.clone()
    scan = ops.mt_scan(vs(G), 1.0 / 65536.0, 1.0)
    ops.mt_adam(vs(G), vs(P), vs(M), vs(V), vs(PL), ops.adam_hparams(2, 1e-3, 0.9, 0.999, 1e-8, 0.0),
                1.0 / 65536.0, scan)
    assert int(scan.found_inf.item()) == 1
    assert torch.equal(P, P1) and torch.equal(M, M1) and torch.equal(V, V1)


def test_cpuadam_parameter_groups_follow_torch_adam():
    """Two parameter groups with their own lr / betas / weight decay
    (axonn/optim.py:17-26 takes torch's param-group form, :100-150 walks the groups):
    three steps against torch.optim.Adam on fp32 copies fed the same gradients."""
    from axonn_amd.inter_layer import LossScaler
    from axonn_amd.optim import CPUAdam

    torch.manual_seed(21)
    a = torch.nn.Parameter((torch.randn(3001) * 0.05).bfloat16().cuda())
    b = torch.nn.Parameter((torch.randn(517, 8) * 0.05).bfloat16().cuda())
    groups = [{"params": [a], "lr": 1e-3, "weight_decay": 0.0},
              {"params": [b], "lr": 3e-2, "betas": (0.8, 0.95), "weight_decay": 0.05}]
    opt = CPUAdam(groups, loss_scaler=LossScaler(loss_scale=256.0), dynamic_loss_scale=False)
    ra = torch.nn.Parameter(a.detach().float().clone())
    rb = torch.nn.Parameter(b.detach().float().clone())
    ref = torch.optim.Adam([{"params": [ra], "lr": 1e-3, "weight_decay": 0.0},
                            {"params": [rb], "lr": 3e-2, "betas": (0.8, 0.95), "weight_decay": 0.05}],
                           foreach=False)
    assert opt.group_offsets == [0, 3001, 3001 + 517 * 8]
    for _ in range(3):
        opt.zero_grad()
        ga = (torch.randn(3001, device="cuda") * 0.01)
        gb = (torch.randn(517, 8, device="cuda") * 0.01)
        a.grad.copy_((ga * 256.0).bfloat16())
        b.grad.copy_((gb * 256.0).bfloat16())
        ra.grad = a.grad.float() / 256.0     # the same bf16-rounded gradients, unscaled
        rb.grad = b.grad.float() / 256.0
        opt.step()
        ref.step()
        got = opt.model_params_fp32
        want = torch.cat([ra.detach().reshape(-1), rb.detach().reshape(-1)])
        assert float((got - want).abs().max() / want.abs().max()) <= P_TOL
    assert torch.equal(a.detach(), opt.model_params_fp32[:3001].bfloat16())
    assert torch.equal(b.detach().reshape(-1), opt.model_params_fp32[3001:].bfloat16())


def test_cpuadam_overflow_flag_is_per_parameter_not_per_flat_buffer():
    """fp16 gradients whose per-parameter sums stay inside the fp16 range while the sum
    over the whole flat buffer does not: the reference tests each parameter
    (axonn/inter_layer.py:447-460), so the step must be applied and the loss scale kept."""
    from axonn_amd.optim import CPUAdam

    params = [torch.nn.Parameter((torch.randn(1000) * 0.02).half().cuda()) for _ in range(8)]
    opt = CPUAdam(params, lr=1e-3)
    assert opt.dynamic_loss_scale and opt.loss_scale == 65536.0
    for p in params:
        p.grad.fill_(60.0)                   # 1000 x 60 = 60000 per parameter: finite in fp16
    grads = [p.grad.double().cpu().numpy() for p in params]
    overflow, _ = oo.unscale_gradients(grads, "f16", 65536.0)
    assert overflow is False                                     # the reference's flag
    assert oo.check_nan(np.concatenate(grads), "f16") is True    # a whole-buffer sum would trip
    p32 = [opt.model_params_fp32[o:o + n].cpu().numpy().copy() for o, n in opt._views]
    zeros = [np.zeros_like(a) for a in p32]
    res = oo.mixed_precision_step([g.astype(np.float32) for g in grads], p32, zeros, zeros, 1,
                                  65536.0, g_dtype="f16", p_dtype="f16")
    opt.step()
    assert not opt.last_step_skipped and opt.step_count == 1 and opt.loss_scale == 65536.0
    got, ref = opt.model_params_fp32.cpu().numpy(), np.concatenate(res["p"])
    assert np.max(np.abs(got - ref)) / np.max(np.abs(ref)) <= P_TOL
    # a parameter whose own sum leaves the range does trip the flag, as in the reference
    params[3].grad.fill_(70.0)               # 70000 > 65504
    grads = [p.grad.double().cpu().numpy() for p in params]
    assert oo.unscale_gradients(grads, "f16", 65536.0)[0] is True
    before = opt.model_params_fp32.clone()
    opt.step()
    assert opt.last_step_skipped and opt.step_count == 1 and opt.loss_scale == 32768.0
    assert torch.equal(opt.model_params_fp32, before)


def test_cpuadam_large_fp16_buffer_of_finite_gradients_is_not_skipped():
    """Twelve parameters of 40000 fp16 gradients with mean 1: every parameter sums to about
    40000, the flat buffer to about 480000."""
    from axonn_amd.optim import CPUAdam

    torch.manual_seed(31)
    params = [torch.nn.Parameter(torch.zeros(40000 + 3 * i, dtype=torch.float16, device="cuda"))
              for i in range(12)]
    opt = CPUAdam(params, max_grad_norm=1.0)
    for p in params:
        p.grad.copy_((torch.randn(p.numel()) + 1.0).half())
    grads = [p.grad.double().cpu().numpy() for p in params]
    assert oo.unscale_gradients(grads, "f16", 65536.0)[0] is False
    assert abs(float(np.concatenate(grads).sum())) > 4e5
    opt.step()
    assert not opt.last_step_skipped and opt.step_count == 1
    assert opt.scaler.no_overflow_iters == 1 and opt.loss_scale == 65536.0
    want = float(np.sqrt(sum(((g / 65536.0) ** 2).sum() for g in grads)))
    assert abs(float(opt.grad_norm()) - want) <= 1e-5 * want


def test_cpuadam_survives_rebound_gradients():
    """`model.zero_grad()` sets gradients to None by default and backward then makes new
    tensors: the step must still see them (they are copied back into the flat buffer)."""
    from axonn_amd.inter_layer import LossScaler
    from axonn_amd.optim import CPUAdam

    torch.manual_seed(32)
    model = torch.nn.Linear(24, 40).cuda().bfloat16()
    opt = CPUAdam(model.parameters(), lr=1e-2, loss_scaler=LossScaler(loss_scale=1.0),
                  dynamic_loss_scale=False)
    params = list(model.parameters())
    p32 = [opt.model_params_fp32[o:o + n].cpu().numpy().copy() for o, n in opt._views]
    m = [np.zeros_like(a) for a in p32]
    v = [np.zeros_like(a) for a in p32]
    for step in (1, 2):
        model.zero_grad()                       # set_to_none=True: the views are gone
        assert all(p.grad is None for p in params)
        x = torch.randn(16, 24).bfloat16().cuda()
        model(x).float().pow(2).mean().backward()
        grads = [p.grad.float().cpu().numpy().reshape(-1).copy() for p in params]
        res = oo.mixed_precision_step(grads, p32, m, v, step, 1.0, lr=1e-2)
        opt.step()
        p32, m, v = res["p"], res["m"], res["v"]
        got, ref = opt.model_params_fp32.cpu().numpy(), np.concatenate(p32)
        assert np.max(np.abs(got - ref)) / np.max(np.abs(ref)) <= P_TOL
        base = opt.model_grads_fp16.data_ptr()
        assert all(p.grad.data_ptr() == base + o * 2 for p, (o, n) in zip(params, opt._views))
    # a parameter that received no gradient takes a zero gradient
    model.zero_grad()
    params[0].grad = torch.ones_like(params[0])
    opt.step()
    assert torch.count_nonzero(opt.model_grads_fp16[opt._views[1][0]:]) == 0


def test_full_size_adam_config():
    """The optimizer configuration at its full size: 1.3e9 elements in 64 ragged tensors
    packed back to back, bf16 gradients ~ N(0, 1e-3) x 65536, clip norm 1, steps 1 and 2;
    then one +inf in tensor 17.  Checked through a sampled oracle (20000 elements, both
    steps), the exact rounding of the low-precision copy, the norm against a float64 sum,
    and bit-identity of the whole state on the skip path."""
    from axonn_amd import ops

    rng = np.random.default_rng(0)
    frac = rng.random(64)
    sizes = np.clip((frac / frac.sum() * 1.3e9).astype(np.int64), 100000, 60000000) | 1  # odd: ragged
    sizes[np.argmax(sizes)] += 1300000000 - int(sizes.sum())
    sizes = [int(s) for s in sizes]
    total = sum(sizes)
    assert total == 1300000000 and min(sizes) >= 100000
    g = torch.Generator(device="cuda").manual_seed(1)
    P = torch.empty(total, device="cuda").normal_(0, 0.02, generator=g)
    G = torch.empty(total, dtype=torch.bfloat16, device="cuda")
    sumsq = 0.0
    for lo in range(0, total, 1 << 27):        # slabs: no 5 GB fp32 temporary
        hi = min(total, lo + (1 << 27))
        t = torch.empty(hi - lo, device="cuda").normal_(0, 1e-3 * 65536.0, generator=g)
        G[lo:hi] = t.bfloat16()
        sumsq += float(((G[lo:hi].double() / 65536.0) ** 2).sum())
        del t
    M = torch.zeros(total, device="cuda")
    V = torch.zeros(total, device="cuda")
    PL = torch.zeros(total, dtype=torch.bfloat16, device="cuda")
    idx = torch.from_numpy(np.sort(rng.choice(total, 20000, replace=False))).cuda()
    # the sample includes the first and last element of every tensor (the ragged heads and tails)
    edges = np.cumsum([0] + sizes)
    idx = torch.unique(torch.cat([idx, torch.from_numpy(edges[:-1]).cuda(),
                                  torch.from_numpy(edges[1:] - 1).cuda()]))
    p_s, m_s, v_s = P[idx].cpu().numpy(), M[idx].cpu().numpy(), V[idx].cpu().numpy()
    vs = lambda t: flat_views(t, sizes)
    want_norm = float(np.sqrt(sumsq))
    for step in (1, 2):
        scan = ops.mt_scan(vs(G), 1.0 / 65536.0, 1.0)
        assert int(scan.found_inf.item()) == 0
        assert abs(float(scan.total_norm.item()) - want_norm) <= 1e-6 * want_norm
        coef = float(scan.clip_coef.item())
        assert abs(coef - 1.0 / (want_norm + 1e-6)) <= 1e-6 * coef
        ops.mt_adam(vs(G), vs(P), vs(M), vs(V), vs(PL),
                    ops.adam_hparams(step, 1e-3, 0.9, 0.999, 1e-8, 0.0), 1.0 / 65536.0, scan)
        gs = ((G[idx].float() / 65536.0).cpu().numpy() * np.float32(coef)).astype(np.float32)
        p_s, m_s, v_s = oo.adam_update(p_s, gs, m_s, v_s, step)
        got = P[idx].cpu().numpy()
        assert np.max(np.abs(got - p_s)) / np.max(np.abs(p_s)) <= P_TOL
        assert np.allclose(M[idx].cpu().numpy(), m_s, rtol=1e-5, atol=1e-12)
        assert np.allclose(V[idx].cpu().numpy(), v_s, rtol=1e-5, atol=1e-16)
        for lo in range(0, total, 1 << 28):
            hi = min(total, lo + (1 << 28))
            assert torch.equal(PL[lo:hi], P[lo:hi].bfloat16())
    # variant B: one +inf in tensor 17 -> flag set, nothing written
    G[int(edges[17]) + 12345] = float("inf")
    csum = lambda t: t.view(torch.int32).sum(dtype=torch.int64).item()  # wrap-around checksum of the bits
    before = [csum(P), csum(M), csum(V), csum(PL.view(torch.int16).view(torch.int32))]
    Pc = P[: 1 << 24].clone()
    scan = ops.mt_scan(vs(G), 1.0 / 65536.0, 1.0)
    ops.mt_adam(vs(G), vs(P), vs(M), vs(V), vs(PL), ops.adam_hparams(3, 1e-3, 0.9, 0.999, 1e-8, 0.0),
                1.0 / 65536.0, scan)
    assert int(scan.found_inf.item()) == 1
    assert [csum(P), csum(M), csum(V), csum(PL.view(torch.int16).view(torch.int32))] == before
    assert torch.equal(P[: 1 << 24], Pc)


@pytest.mark.parametrize("p", [1.0, 3.0, 0.5, 2.5, 0.0, -1.5])
def test_clip_grad_norm_any_finite_order(p):
    """Orders other than 2 (gradient_normalization.py:18-34 passes norm_type through):
    against the oracle and torch.nn.utils.clip_grad_norm_ on ragged fp32 gradients, and on
    a bf16 / fp32 mix against the float64 closed form."""
    from axonn_amd.intra_layer import clip_grad_norm_
    from axonn_amd.intra_layer.gradient_normalization import get_total_norm

    torch.manual_seed(40)
    ps = [torch.nn.Parameter(torch.randn(n).cuda()) for n in (33, 70001, 12, 4096)]
    qs = [torch.nn.Parameter(p_.detach().clone()) for p_ in ps]
    for a, b in zip(ps, qs):
        a.grad = torch.randn_like(a) * 0.5 + 0.01
        b.grad = a.grad.clone()
    grads = [a.grad.double().cpu().numpy() for a in ps]
    want, clipped = oo.clip_grad_norm_(grads, 0.05, "f32", norm_type=p)
    assert abs(float(get_total_norm([a.grad for a in ps], p)) - want) <= 2e-5 * abs(want)
    got = clip_grad_norm_(ps, 0.05, norm_type=p)
    ref = torch.nn.utils.clip_grad_norm_(qs, 0.05, norm_type=p, foreach=False)
    assert abs(float(got) - want) <= 2e-5 * abs(want)
    assert abs(float(got) - float(ref)) <= 2e-5 * abs(float(ref))
    for a, b, c in zip(ps, qs, clipped):
        assert torch.allclose(a.grad, b.grad, rtol=3e-5, atol=0)
        assert np.allclose(a.grad.double().cpu().numpy(), c, rtol=3e-5, atol=0)
    if p > 0:   # mixed dtypes: one accumulating call per dtype
        gs = [torch.randn(5000).cuda().bfloat16(), torch.randn(333).cuda(), torch.randn(64).cuda().half()]
        flat = np.abs(np.concatenate([g.double().cpu().numpy() for g in gs]))
        w = float(np.sum(flat ** p) ** (1.0 / p))
        assert abs(float(get_total_norm(gs, p)) - w) <= 2e-5 * w


@pytest.mark.parametrize("p", [float("inf"), float("-inf")])
def test_total_norm_of_infinite_order(p):
    """get_total_norm passes +inf and -inf through as the reference's does
    (gradient_normalization.py:18-34): the largest / smallest magnitude over every
    gradient, exact in every dtype, over tensors of several chunks and of mixed dtypes, NaN
    if an element is; clip_grad_norm_ refuses them."""
    from axonn_amd.intra_layer import clip_grad_norm_
    from axonn_amd.intra_layer.gradient_normalization import get_total_norm

    g = torch.Generator(device="cuda").manual_seed(3)
    gs = [torch.randn(n, device="cuda", generator=g) + 0.001 for n in (33, 200001, 12, 4096)]
    want = oo.get_total_norm([t.double().cpu().numpy() for t in gs], norm_type=p)
    ref = torch.norm(torch.stack([torch.norm(t, p) for t in gs]), p)
    assert float(get_total_norm(gs, p)) == want == float(ref)
    mixed = [gs[0].bfloat16(), gs[1], gs[2].half(), gs[3].bfloat16()]
    want = oo.get_total_norm([t.double().cpu().numpy() for t in mixed], norm_type=p)
    assert float(get_total_norm(mixed, p)) == np.float32(want)
    gs[1][150000] = 123.0 if p > 0 else 0.0
    assert float(get_total_norm(gs, p)) == (123.0 if p > 0 else 0.0)
    gs[3][5] = float("nan")
    assert np.isnan(float(get_total_norm(gs, p)))
    with pytest.raises(NotImplementedError):
        clip_grad_norm_([torch.nn.Parameter(gs[0])], 1.0, norm_type=p)


def test_order_zero_counts_gradients_with_a_nonzero_element():
    from axonn_amd.intra_layer.gradient_normalization import get_total_norm

    gs = [torch.zeros(100).cuda(), torch.zeros(70000).cuda(), torch.zeros(9).cuda()]
    assert float(get_total_norm(gs, 0.0)) == 0.0
    gs[1][69999] = -2.0
    gs[2][0] = 1e-30
    assert float(get_total_norm(gs, 0.0)) == 2.0
    want = torch.norm(torch.stack([torch.norm(g, 0.0) for g in gs]), 0.0)
    assert float(want) == 2.0


def test_stream_probes_read_fill_copy():
    """The yardstick kernels of the benchmarks do what they are timed for: a copy equals its
    source (also in place, also over a ragged number of 16-byte vectors), a fill writes zeros
    and nothing behind the given bytes, a read writes nothing."""
    import ctypes

    from axonn_amd import _native as nv

    lib = nv.load_probe()
    stream = nv.current_stream()

    def run(kind, src, dst, nbytes):
        assert lib.axn_probe_stream(kind, src, dst, nbytes, stream) == 0

    for n in (4, 1000, 64 * 4 * 1000 + 12, 1 << 22):   # floats
        g = torch.Generator(device="cuda").manual_seed(n)
        src = torch.randn(n + 8, generator=g, device="cuda")
        dst = torch.full((n + 8,), 7.0, device="cuda")
        nbytes = n * 4
        run(2, src.data_ptr(), dst.data_ptr(), nbytes)
        assert torch.equal(dst[:n], src[:n]) and bool((dst[n:] == 7.0).all())
        keep = src.clone()
        run(2, src.data_ptr(), src.data_ptr(), nbytes)
        assert torch.equal(src, keep)
        sink = torch.full((4,), 3.0, device="cuda")
        run(0, src.data_ptr(), sink.data_ptr(), nbytes)
        assert torch.equal(src, keep) and bool((sink == 3.0).all())
        run(1, None, dst.data_ptr(), nbytes)
        assert bool((dst[:n] == 0.0).all()) and bool((dst[n:] == 7.0).all())
