"""The entry points under HIP graph capture: a captured training step (forward with
the fused epilogue, dgrad, accumulating wgrad, gradient scan, Adam) is replayed several
times, with eager work and synchronisations between the replays, and every replay must
equal the eager step on the same inputs bit for bit.  The library issues no memset, copy,
allocation or synchronisation of its own, so a capture holds kernel nodes only; that
includes the embedding's weight gradient and max_norm, whose sort is the library's own.
"""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _state(seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    n1, n2 = 70001, 4099
    s = {
        "X": torch.randn(384, 256, device="cuda", generator=g).bfloat16(),
        "W": (torch.randn(512, 256, device="cuda", generator=g) * 0.05).bfloat16(),
        "b": torch.randn(512, device="cuda", generator=g) * 0.1,
        "dY": (torch.randn(384, 512, device="cuda", generator=g) * 0.01).bfloat16(),
        "dW": torch.zeros(512, 256, device="cuda"),
        "P": torch.randn(n1 + n2, device="cuda", generator=g) * 0.02,
        "M": torch.zeros(n1 + n2, device="cuda"),
        "V": torch.zeros(n1 + n2, device="cuda"),
        "G": (torch.randn(n1 + n2, device="cuda", generator=g) * 64.0).bfloat16(),
        "PL": torch.zeros(n1 + n2, device="cuda", dtype=torch.bfloat16),
    }
    s["sizes"] = (n1, n2)
    return s


def _views(t, sizes):
    out, off = [], 0
    for n in sizes:
        out.append(t[off:off + n])
        off += n
    return out


def _step(s):
    from axonn_amd import ops

    y, z = ops.gemm_fwd(s["X"], s["W"], bias=s["b"], activation="gelu", save_z=True)
    dz, db = ops.dgelu_dbias(s["dY"], z, want_dbias=True)
    dx = ops.gemm_dgrad(dz, s["W"])
    ops.gemm_wgrad(dz, s["X"], out=s["dW"], accumulate=True)
    v = lambda k: _views(s[k], s["sizes"])  # noqa: E731
    scan = ops.mt_scan(v("G"), inv_scale=1.0 / 64.0, max_norm=1.0)
    ops.mt_adam(v("G"), v("P"), v("M"), v("V"), v("PL"), ops.adam_hparams(3, 1e-3, 0.9, 0.999, 1e-8, 0.01),
                inv_scale=1.0 / 64.0, scan=scan)
    return y, dx, db


MUTATED = ("dW", "P", "M", "V", "PL")


def test_captured_step_replays_like_the_eager_step():
    live = _state(1)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # first launches outside the capture
        warm = {k: (v.clone() if torch.is_tensor(v) else v) for k, v in live.items()}
        _step(warm)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    before_capture = {k: live[k].clone() for k in MUTATED}
    with torch.cuda.graph(graph):
        outs = _step(live)
    for k in MUTATED:  # capturing runs nothing
        assert torch.equal(live[k], before_capture[k]), k

    for replay in range(4):
        fresh = _state(10 + replay)
        for k in ("X", "W", "b", "dY", "G"):  # new inputs at the captured addresses
            live[k].copy_(fresh[k])
        twin = {k: (v.clone() if torch.is_tensor(v) else v) for k, v in live.items()}
        want = _step(twin)          # eager, on copies of the state the replay starts from
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, exp, name in zip(outs, want, ("y", "dx", "db")):
            assert torch.equal(got, exp), (replay, name)
        for k in MUTATED:
            assert torch.equal(live[k], twin[k]), (replay, k)
    assert live["dW"].abs().sum() > 0 and not torch.equal(live["P"], before_capture["P"])


@pytest.mark.parametrize("M,N,K", [(512, 512, 512), (4096, 2304, 256), (256, 1024, 4096)])
def test_captured_tile_kernels_replay_like_eager(M, N, K):
    """The one-wave-per-SIMD kernels (128 x 128 tiles; 256 x 256 tiles; a forward whose
    contraction is split over workgroups through a workspace) under capture: they ask
    for their LDS size with a function attribute at launch time, which must not disturb
    a capture, and every replay equals the eager launch bit for bit."""
    from axonn_amd import ops

    g = torch.Generator(device="cuda").manual_seed(M + N + K)
    X = torch.randn(M, K, device="cuda", generator=g).bfloat16()
    W = (torch.randn(N, K, device="cuda", generator=g) * 0.05).bfloat16()
    dY = (torch.randn(M, N, device="cuda", generator=g) * 0.01).bfloat16()

    def work():
        y, _ = ops.gemm_fwd(X, W)
        return y, ops.gemm_dgrad(dY, W), ops.gemm_wgrad(dY, X, out_dtype=torch.float32)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = work()
    for replay in range(3):
        X.copy_(torch.randn(M, K, device="cuda", generator=g).bfloat16())
        dY.copy_((torch.randn(M, N, device="cuda", generator=g) * 0.01).bfloat16())
        want = work()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, exp, name in zip(outs, want, ("y", "dx", "dw")):
            assert torch.equal(got, exp), (replay, name)


def test_captured_joint_backward_replays_like_eager():
    """axn_gemm_bwd at a shape that runs dX and dW as ONE launch (160 + 100 tiles of 256 x 256)
    under capture: the host's choice of the launch is made at capture time, the replays run
    the same kernel on new operands and must equal the eager call bit for bit."""
    from axonn_amd import ops

    M, N, K = 4096, 2560, 2560
    g = torch.Generator(device="cuda").manual_seed(9)
    X = torch.randn(M, K, device="cuda", generator=g).bfloat16()
    W = (torch.randn(N, K, device="cuda", generator=g) * 0.05).bfloat16()
    dY = (torch.randn(M, N, device="cuda", generator=g) * 0.01).bfloat16()
    acc = torch.zeros(N, K, device="cuda")

    def work(dw):
        dx, _ = ops.gemm_bwd(dY, W, X, out=dw, accumulate=True)
        return dx

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work(torch.zeros_like(acc))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = work(acc)
    assert not acc.any()                      # capturing runs nothing
    twin = torch.zeros_like(acc)
    for replay in range(3):
        X.copy_(torch.randn(M, K, device="cuda", generator=g).bfloat16())
        dY.copy_((torch.randn(M, N, device="cuda", generator=g) * 0.01).bfloat16())
        want = work(twin)                     # eager, accumulating like the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), replay
        assert torch.equal(acc, twin), replay
    assert acc.abs().sum() > 0


def test_captured_embedding_backward_and_renorm_replay_like_eager():
    """The embedding's weight gradient (sort of the token positions, row starts, row sums)
    and the max_norm pass under capture, replayed on new ids and gradients."""
    from axonn_amd import ops

    T, V, H = 3000, 5000, 64
    g = torch.Generator(device="cuda").manual_seed(5)
    ids = torch.randint(0, V, (T,), device="cuda", generator=g)
    dy = torch.randn(T, H, device="cuda", generator=g)
    W = torch.randn(V, H, device="cuda", generator=g)

    def work(table):
        dW = ops.embedding_bwd(ids, dy, V, padding_idx=3)
        ops.embedding_renorm_(table, ids, 1.5)
        return dW

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work(W.clone())
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    live = W.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = work(live)
    for replay in range(3):
        ids.copy_(torch.randint(0, V, (T,), device="cuda", generator=g))
        ids[replay::7] = 11          # a long run that moves from replay to replay
        dy.copy_(torch.randn(T, H, device="cuda", generator=g))
        live.copy_(W)
        twin = W.clone()
        want = work(twin)            # eager
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), replay
        assert torch.equal(live, twin), replay
        assert not torch.equal(live, W)
