"""The library from several host threads at once, each on a stream of its own: the
entry points keep no state between calls (workspaces are the caller's, the last error is
per thread), so concurrent callers get what a lone caller gets, bit for bit.  The
reference's layer is entered from two threads in every training step: forward on the
caller's, backward on the autograd engine's device thread (fully_connected.py:96-187)."""

import threading

import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    n = 50001
    return {
        "X": torch.randn(256, 384, device="cuda", generator=g).bfloat16(),
        "W": (torch.randn(512, 384, device="cuda", generator=g) * 0.05).bfloat16(),
        "b": torch.randn(512, device="cuda", generator=g) * 0.1,
        "dY": (torch.randn(256, 512, device="cuda", generator=g) * 0.01).bfloat16(),
        "P": torch.randn(n, device="cuda", generator=g) * 0.02,
        "G": (torch.randn(n, device="cuda", generator=g) * 64.0).bfloat16(),
        "ids": torch.randint(0, 300, (777,), device="cuda", generator=g),
        "T": torch.randn(300, 64, device="cuda", generator=g),
        "dE": torch.randn(777, 64, device="cuda", generator=g),
    }


def _work(s, rounds):
    from axonn_amd import ops

    dW = torch.zeros(512, 384, device="cuda")
    P, M, V = s["P"].clone(), torch.zeros_like(s["P"]), torch.zeros_like(s["P"])
    PL = torch.zeros_like(P, dtype=torch.bfloat16)
    out = None
    for it in range(rounds):
        y, z = ops.gemm_fwd(s["X"], s["W"], bias=s["b"], activation="gelu", save_z=True)
        dz, db = ops.dgelu_dbias(s["dY"], z, want_dbias=True)
        if it % 2:   # the two gradient products through their own entry points, or through the joint one
            dx = ops.gemm_dgrad(dz, s["W"])
            ops.gemm_wgrad(dz, s["X"], out=dW, accumulate=True)
        else:
            dx, _ = ops.gemm_bwd(dz, s["W"], s["X"], out=dW, accumulate=True)
        scan = ops.mt_scan([s["G"]], inv_scale=1.0 / 64.0, max_norm=1.0)
        ops.mt_adam([s["G"]], [P], [M], [V], [PL], ops.adam_hparams(it + 1, 1e-3, 0.9, 0.999, 1e-8, 0.0),
                    inv_scale=1.0 / 64.0, scan=scan)
        emb = ops.embedding_bwd(s["ids"], s["dE"], 300)
        out = (y, dx, db, emb)
    torch.cuda.current_stream().synchronize()
    return [t.clone() for t in out] + [dW, P, M, V, PL]


def test_concurrent_callers_match_a_lone_caller():
    n_threads, rounds = 4, 12
    inputs = [_inputs(100 + i) for i in range(n_threads)]
    want = [_work(s, rounds) for s in inputs]
    torch.cuda.synchronize()

    got, errors = [None] * n_threads, []
    start = threading.Barrier(n_threads)

    def run(i):
        try:
            stream = torch.cuda.Stream()
            stream.wait_stream(torch.cuda.default_stream())
            with torch.cuda.stream(stream):
                start.wait()
                got[i] = _work(inputs[i], rounds)
        except Exception as e:  # noqa: BLE001 - reported by the asserting thread
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=run, args=(i,)) for i in range(n_threads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for i in range(n_threads):
        for k, (a, b) in enumerate(zip(got[i], want[i])):
            assert torch.equal(a, b), (i, k)


def test_last_error_is_per_thread():
    from axonn_amd import _native as nv

    lib = nv.load()
    X = torch.zeros(8, 8, device="cuda", dtype=torch.bfloat16)
    seen = {}
    gate = threading.Barrier(2)

    def bad(name, n_cols):
        # N = n_cols is not a multiple of 8: rejected before any launch
        rc = lib.axn_gemm_fwd(X.data_ptr(), X.data_ptr(), None, X.data_ptr(), None, 8, n_cols, 8, 8, 8, 8, 0,
                              nv.current_stream())
        gate.wait()   # both threads have failed before either reads its message
        seen[name] = (rc, lib.axn_last_error().decode())

    a = threading.Thread(target=bad, args=("a", 3))
    b = threading.Thread(target=bad, args=("b", 5))
    a.start(), b.start()
    a.join(), b.join()
    assert seen["a"][0] == seen["b"][0] == nv.AXN_ESHAPE
    assert "N=3" in seen["a"][1] and "N=5" in seen["b"][1]
