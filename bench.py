#!/usr/bin/env python3
"""Benchmark of the hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one forward + backward pass over the Llama-3-8B-shaped Linear set
(4096 tokens; QKV 4096->6144, O 4096->4096, gate and up 4096->14336, down
14336->4096; bf16 operands, fp32 accumulate, no bias): 15 GEMMs through the C ABI
of libaxn_gfx950.so - axn_gemm_fwd per layer, then axn_gemm_bwd (dX and dW) per
layer - on operands already resident in HBM.  `value` is
the aggregate TFLOP/s over the set (algorithmic 6 M N K per layer).

The same run also times, outside the main timed region and reported in extra
keys of the one JSON line:
  adam      the mixed-precision Adam step (scan + update) on 1.3e9 parameters in
            64 ragged tensors, GB/s at 30 algorithmic bytes per element, and the
            overflow (skip) variant
  shapes    the 12B-style MLP shard with fused bias + GELU, the skinny
            decode-like shard, the Llama MLP block with the one-pass SwiGLU, and the
            embedding lookup and its weight gradient at the Llama-3 vocabulary
  cpu_baseline  the torch-CPU restatement of the same layer math on the host cores

The calls of every fourth step of the timed region are bracketed by HIP events on the
launch stream; `roofline` reports the kind of call with the largest share of the time.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2516.6   # MI355X dense bf16 MFMA
EVENT_EVERY = 4              # timed steps between two steps whose launches are bracketed by events
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

# HBM bytes per launch (read + written), averaged over the launches of each kernel in
# this workload, from `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` runs of this
# file, scaled by what the same counters read for the 1 GiB copy below
# (profiles/gemm_adam_llama_set_pmc.txt has the runs and the arithmetic).  The
# counters sit between L2 and the fabric, so hits in the memory-side cache are included.
TRAFFIC_BYTES_PER_LAUNCH = {"fwd": 634588622, "bwd": 1246730803}   # bwd: a call = dX and dW of a layer
ADAM_TRAFFIC_BYTES_PER_STEP = 38997215093   # scan + update, 1.3e9 elements: 1.000 x 30 B/element
TRAFFIC_SOURCE = "profiles/gemm_adam_llama_set_pmc.txt"

LLAMA_SET = [  # (name, M, N, K), gate and up are two layers of one shape
    ("qkv", 4096, 6144, 4096),
    ("o", 4096, 4096, 4096),
    ("gate", 4096, 14336, 4096),
    ("up", 4096, 14336, 4096),
    ("down", 4096, 4096, 14336),
]


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-adam", action="store_true")
    ap.add_argument("--no-library-baseline", action="store_true")
    ap.add_argument("--no-extra-shapes", action="store_true")
    ap.add_argument("--adam-elements", type=float, default=1.3e9)
    ap.add_argument("--shapes", default=None,
                    help="comma list of the extra shapes to run (fp16, mlp_shard, skinny, llama_mlp, "
                         "embedding, small_mlp); default: all")
    ap.add_argument("--no-main-set", action="store_true",
                    help="skip the Llama-3-8B-shaped set (value is null): for profiles of the other shapes")
    ap.add_argument("--no-power", action="store_true",
                    help="skip the power / clock telemetry legs (about 6 s)")
    ap.add_argument("--no-launch-events", action="store_true",
                    help="do not bracket every launch with events (no per-kernel figures)")
    return ap.parse_args()


class PowerSampler:
    """Samples the GPU's socket power (hwmon power1_input, microwatts) in a thread while a
    loop runs, and reads the reported per-XCD gfx clocks from `amd-smi metric` once during it.
    Everything is optional: a box that does not expose a value reports null for it."""

    def __init__(self):
        import glob
        self.power_file = self.cap_file = None
        for d in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*")):
            if os.path.exists(os.path.join(d, "power1_input")):
                self.power_file = os.path.join(d, "power1_input")
                cap = os.path.join(d, "power1_cap")
                self.cap_file = cap if os.path.exists(cap) else None
                break

    @staticmethod
    def _read(path):
        try:
            with open(path) as f:
                return int(f.read().strip())
        except (OSError, ValueError):
            return None

    @staticmethod
    def xcd_clocks_mhz():
        import subprocess
        try:
            out = subprocess.run(["amd-smi", "metric", "-g", "0", "--clock", "--json"],
                                 stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True,
                                 timeout=20).stdout
            data = json.loads(out)
            gpu = (data.get("gpu_data") if isinstance(data, dict) else data)[0]
            clk = gpu["clock"]
            vals = []
            for i in range(16):
                c = clk.get("gfx_%d" % i)
                if not c:
                    break
                v = c["clk"]["value"] if isinstance(c["clk"], dict) else c["clk"]
                if isinstance(v, (int, float)):
                    vals.append(int(v))
            return vals or None
        except Exception:   # noqa: BLE001 - telemetry is best effort
            return None

    def measure(self, torch, fn, flops_per_call, seconds=2.5):
        """Runs fn() back to back for `seconds`; returns the rate, the mean socket power over
        the second half of the loop, and the gfx clocks read in the middle of it."""
        import threading
        rows, stop = [], threading.Event()

        def sample():
            while not stop.is_set():
                if self.power_file:
                    rows.append((time.perf_counter(), self._read(self.power_file)))
                time.sleep(0.02)

        clocks = {}

        def read_clocks():
            time.sleep(seconds * 0.5)
            clocks["mhz"] = self.xcd_clocks_mhz()

        th, tc = threading.Thread(target=sample, daemon=True), threading.Thread(target=read_clocks, daemon=True)
        torch.cuda.synchronize()
        th.start()
        tc.start()
        t0 = time.perf_counter()
        calls = 0
        while time.perf_counter() - t0 < seconds:
            for _ in range(4):
                fn()
            calls += 4
            torch.cuda.synchronize()
        t1 = time.perf_counter()
        stop.set()
        th.join()
        tc.join(30)
        late = [w for t, w in rows if w is not None and t >= t0 + 0.5 * (t1 - t0) and t <= t1]
        cap = self._read(self.cap_file) if self.cap_file else None
        mhz = clocks.get("mhz")
        return {"tflops": round(flops_per_call * calls / (t1 - t0) / 1e12, 1),
                "socket_power_w": round(sum(late) / len(late) / 1e6, 1) if late else None,
                "socket_power_cap_w": round(cap / 1e6, 1) if cap else None,
                "power_samples": len(late),
                "gfx_clock_mhz_per_xcd": mhz,
                "gfx_clock_mhz_mean": round(sum(mhz) / len(mhz)) if mhz else None,
                "seconds": round(t1 - t0, 2)}


class Layer:
    def __init__(self, name, M, N, K, seed, torch, bias=False):
        g = torch.Generator(device="cuda").manual_seed(seed)
        self.name, self.M, self.N, self.K = name, M, N, K
        self.X = torch.randn(M, K, generator=g, device="cuda").bfloat16()
        self.W = (torch.randn(N, K, generator=g, device="cuda") * 0.02).bfloat16()
        self.dY = (torch.randn(M, N, generator=g, device="cuda") * 1e-3).bfloat16()
        self.bias = (torch.randn(N, generator=g, device="cuda") * 0.1) if bias else None
        self.Y = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
        self.Z = torch.empty(M, N, dtype=torch.bfloat16, device="cuda") if bias else None
        self.dZ = torch.empty(M, N, dtype=torch.bfloat16, device="cuda") if bias else None
        self.dX = torch.empty(M, K, dtype=torch.bfloat16, device="cuda")
        self.dW = torch.zeros(N, K, dtype=torch.bfloat16, device="cuda")
        self.db = torch.zeros(N, device="cuda") if bias else None
        self.flops = 6.0 * M * N * K


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures the per-GPU hot path on ONE GPU; --gpus %d is not supported "
              "(nothing in this build uses a second GPU)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch

    from axonn_amd import _native as nv

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    lib = nv.load()
    torch.cuda.set_device(0)
    stream = nv.current_stream()

    def fwd(L, epi=nv.EPI_NONE):
        nv.check(lib.axn_gemm_fwd(L.X.data_ptr(), L.W.data_ptr(),
                                  None if L.bias is None else L.bias.data_ptr(), L.Y.data_ptr(),
                                  None if L.Z is None else L.Z.data_ptr(),
                                  L.M, L.N, L.K, L.K, L.K, L.N, epi, stream))

    def bwd(L):
        # dX and dW of a layer through the entry point for both (AsyncLinear.backward): two
        # launches (four where both end in a rest), or one where the library finds that the
        # two tile counts together fill whole rounds (here: the down projection, 896 + 896)
        nv.check(lib.axn_gemm_bwd(L.dY.data_ptr(), L.W.data_ptr(), L.X.data_ptr(), L.dX.data_ptr(),
                                  L.dW.data_ptr(), nv.BF16, L.M, L.N, L.K, L.N, L.K, L.K, L.K, L.K, 0,
                                  nv.BF16, stream))

    selected = None if args.shapes is None else set(args.shapes.split(","))

    def want(name):
        return not args.no_extra_shapes and (selected is None or name in selected)

    main_set = not args.no_main_set
    layers = [Layer(n, M, N, K, i, torch) for i, (n, M, N, K) in enumerate(LLAMA_SET)] if main_set else []
    total_flops = sum(L.flops for L in layers)

    # One plain copy of known size (1 GiB read + 1 GiB written), outside every timed
    # region: the yardstick that scales the FETCH_SIZE / WRITE_SIZE counters of a
    # profiler run of this same command.
    cal = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
    cal_dst = torch.empty_like(cal)
    cal_dst.copy_(cal)
    del cal, cal_dst

    def ev():
        return torch.cuda.Event(enable_timing=True)

    spans = {"fwd": [], "bwd": []}  # (start, end, flops) per call
    # One event between consecutive launches: launch j of a step runs between events j
    # and j + 1, so a span is the kernel plus the gap to the next launch (3-5 us).  Half
    # the event traffic of a start/stop pair per launch, which cost 2.5 % of the step.
    chain = {"last": None}

    def timed(kind, fn, L):
        if chain["last"] is None:
            chain["last"] = ev()
            chain["last"].record()
        fn(L)
        e = ev()
        e.record()
        spans[kind].append((chain["last"], e, L.flops / 3.0 * (2 if kind == "bwd" else 1)))
        chain["last"] = e

    def step(record):
        record = record and not args.no_launch_events
        chain["last"] = None
        for L in layers:
            timed("fwd", fwd, L) if record else fwd(L)
        for L in reversed(layers):
            timed("bwd", bwd, L) if record else bwd(L)

    for _ in range(args.warmup if main_set else 0):
        step(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    # Events bracket the launches of every fourth timed step: recorded on every step they cost
    # 0.7-1.5 % of the step, and the per-kernel averages need no more samples than that.
    for i in range(args.steps if main_set else 0):
        step(i % EVENT_EVERY == 0)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    value = total_flops / (elapsed / args.steps) / 1e12

    roofline = None
    if main_set and not args.no_launch_events:
        kinds = {}
        for kind, lst in spans.items():
            tot_ms = sum(s.elapsed_time(e) for s, e, _ in lst)
            tot_fl = sum(f for _, _, f in lst)
            kinds[kind] = {
                "launches": len(lst), "avg_us": tot_ms / len(lst) * 1e3,
                "tflops": tot_fl / (tot_ms * 1e-3) / 1e12, "total_ms": tot_ms,
            }
        dom = max(kinds, key=lambda k: kinds[k]["total_ms"])
        # template arguments: <tile, A contraction-contiguous, B contraction-contiguous, epilogue, fp32 out>.
        # A call whose output is k x 256 + r large tiles with 0 < r <= 128 is two launches, k rounds
        # of this instance and the rest on 256 x 128 tiles (gemm_bf16_rest_kernel) or, for r <= 64,
        # on its <128, ...> twin; the events bracket the call.
        kernel_names = {"fwd": "gemm_bf16_solo_kernel<256, true, true, 0, false> (Y = X W^T)",
                        "bwd": "axn_gemm_bwd = gemm_bf16_solo_kernel<256, true, false, 0, false> (dX = dY W) + "
                               "gemm_bf16_solo_kernel<256, false, false, 0, false> (dW = dY^T X); for the down "
                               "projection both in one launch (gemm_backward_kernel<false, false>)"}
        roofline = {
            "bound": "mfma", "kernel": kernel_names[dom],
            "achieved": round(kinds[dom]["tflops"], 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
            "frac": round(kinds[dom]["tflops"] / PEAK_BF16_TFLOPS, 4),
            "avg_launch_us": round(kinds[dom]["avg_us"], 1),
            "launches_timed": kinds[dom]["launches"],  # those of every EVENT_EVERY-th timed step
            "flops_per_launch": kinds[dom]["tflops"] * 1e12 * kinds[dom]["avg_us"] * 1e-6,
            "traffic": TRAFFIC_BYTES_PER_LAUNCH.get(dom),
            "traffic_source": TRAFFIC_SOURCE,
            "traffic_counts": "bytes between the 8 XCD-private L2s and the fabric (FETCH_SIZE + WRITE_SIZE), "
                              "reads served by the 256 MB memory-side cache included: each L2 pulls its own "
                              "copy of a shared operand panel, so this bounds HBM bytes from above",
            "algorithmic_bytes_per_launch": round((2 if dom == "bwd" else 1) *
                                                  sum(2.0 * (L[1] * L[3] + L[2] * L[3] + L[1] * L[2])
                                                      for L in LLAMA_SET) / len(LLAMA_SET)),
            "per_kernel": {k: {"avg_us": round(v["avg_us"], 1), "tflops": round(v["tflops"], 1),
                               "frac": round(v["tflops"] / PEAK_BF16_TFLOPS, 4)}
                           for k, v in kinds.items()},
        }
    # The same 15 products through the vendor GEMM library (torch.matmul = hipBLASLt), same
    # operands, same order, timed the same way: a yardstick on this box, not a code path
    # of the library under test.
    library = None
    if main_set and not args.no_library_baseline:
        def library_step():
            for L in layers:
                torch.matmul(L.X, L.W.t(), out=L.Y)
            for L in reversed(layers):
                torch.matmul(L.dY, L.W, out=L.dX)
                torch.matmul(L.dY.t(), L.X, out=L.dW)

        for _ in range(max(args.warmup, 2)):
            library_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            library_step()
        torch.cuda.synchronize()
        lib_elapsed = (time.perf_counter() - t0) / args.steps
        library = {"kind": "torch.matmul (hipBLASLt) on the same operands, fwd + dgrad + wgrad of the 5 layers",
                   "value": round(total_flops / lib_elapsed / 1e12, 2), "unit": "TFLOP/s",
                   "ms_per_step": round(lib_elapsed * 1e3, 4),
                   "ours_over_library": round(value / (total_flops / lib_elapsed / 1e12), 4)}
    # Socket power and reported clocks while the step runs back to back, and while the vendor
    # library runs the same products: the part runs these kernels at its power cap, which
    # is what sets the rate (outside every timed region).
    power = None
    if main_set and not args.no_power:
        sampler = PowerSampler()
        power = {"source": "hwmon power1_input / power1_cap; amd-smi metric --clock (gfx_N clk per XCD)",
                 "gfx_clock_max_mhz": 2400,
                 "this_library": sampler.measure(torch, lambda: step(False), total_flops)}
        if not args.no_library_baseline:
            power["vendor_library"] = sampler.measure(torch, library_step, total_flops)
        # one forward GEMM of whole rounds and a rest (gate projection, 896 tiles) back to back:
        # the kernel alone, and the vendor library's kernel for the same product
        G = layers[2]
        power["forward_gate_4096x14336x4096"] = {
            "this_library": sampler.measure(torch, lambda: fwd(G), G.flops / 3.0, seconds=2.0)}
        if not args.no_library_baseline:
            power["forward_gate_4096x14336x4096"]["vendor_library"] = sampler.measure(
                torch, lambda: torch.matmul(G.X, G.W.t(), out=G.Y), G.flops / 3.0, seconds=2.0)

    def time_loop(fn, n, w=3):
        for _ in range(w):
            fn()
        torch.cuda.synchronize()
        s, e = ev(), ev()
        s.record()
        for _ in range(n):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / n * 1e-3

    shapes = {}
    if main_set and want("fp16"):
        # The same step on fp16 operands (the reference's default autocast type): the same
        # kernels with v_mfma_f32_16x16x32_f16.
        half = [(L.X.half(), L.W.half(), L.dY.half(), torch.empty_like(L.Y, dtype=torch.float16),
                 torch.empty_like(L.dX, dtype=torch.float16), torch.empty_like(L.dW, dtype=torch.float16))
                for L in layers]

        def fp16_step():
            for L, (X, W, dY, Y, dX, dW) in zip(layers, half):
                nv.check(lib.axn_gemm_fwd_f16(X.data_ptr(), W.data_ptr(), None, Y.data_ptr(), None,
                                              L.M, L.N, L.K, L.K, L.K, L.N, nv.EPI_NONE, stream))
            for L, (X, W, dY, Y, dX, dW) in zip(reversed(layers), reversed(half)):
                nv.check(lib.axn_gemm_bwd(dY.data_ptr(), W.data_ptr(), X.data_ptr(), dX.data_ptr(),
                                          dW.data_ptr(), nv.F16, L.M, L.N, L.K, L.N, L.K, L.K, L.K, L.K, 0,
                                          nv.F16, stream))

        t = time_loop(fp16_step, max(args.steps // 2, 3))
        shapes["llama_set_fp16"] = {"ms_per_step": round(t * 1e3, 4),
                                    "tflops": round(total_flops / t / 1e12, 1),
                                    "frac_mfma": round(total_flops / t / 1e12 / PEAK_BF16_TFLOPS, 4)}
        del half
    del layers
    torch.cuda.empty_cache()
    if not args.no_extra_shapes:
        P = lambda t: t.data_ptr()  # noqa: E731
        if want("mlp_shard"):
            # 12B-style MLP shard: bias + GELU fused, dW accumulated over 4 micro-batches
            L = Layer("mlp_shard", 8192, 5120, 2560, 10, torch, bias=True)
            ws_bytes = lib.axn_dgelu_dbias_workspace_bytes(L.M, L.N)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")

            def mlp_shard_step():
                for mb in range(4):
                    fwd(L, nv.EPI_BIAS_GELU)
                    nv.check(lib.axn_dgelu_dbias(L.dY.data_ptr(), L.Z.data_ptr(), L.dZ.data_ptr(),
                                                 nv.BF16, L.db.data_ptr(), L.M, L.N, L.N,
                                                 1 if mb else 0, ws.data_ptr(), ws_bytes, stream))
                    # dX and the accumulated dW through the entry point for both (one launch here:
                    # 320 + 200 tiles of 256 x 256 leave CUs idle one after the other)
                    nv.check(lib.axn_gemm_bwd(L.dZ.data_ptr(), L.W.data_ptr(), L.X.data_ptr(),
                                              L.dX.data_ptr(), L.dW.data_ptr(), nv.BF16, L.M, L.N, L.K,
                                              L.N, L.K, L.K, L.K, L.K, 1 if mb else 0, nv.BF16, stream))

            t = time_loop(mlp_shard_step, max(args.steps // 4, 3)) / 4
            shapes["mlp_shard_8192x5120x2560_bias_gelu"] = {
                "us_per_microbatch": round(t * 1e6, 1), "tflops": round(L.flops / t / 1e12, 1),
                "frac_mfma": round(L.flops / t / 1e12 / PEAK_BF16_TFLOPS, 4)}
            del L, ws
        if want("skinny"):
            # Skinny shard at the ridge of the roofline: its operands (90 MB a set) would stay in
            # the 256 MB memory-side cache from one iteration to the next, so the loop walks over
            # six sets (540 MB) and every GEMM finds its operands in HBM.
            sets = [Layer("skinny", 512, 8192, 3584, 11 + i, torch) for i in range(6)]
            L = sets[0]
            # few output tiles: the entry points that may split the contraction over workgroups
            ws_bytes = max(lib.axn_gemm_workspace_bytes(op, L.M, L.N, L.K) for op in (0, 1, 2))
            ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
            turn = {"i": 0}

            def skinny_step():
                S = sets[turn["i"] % len(sets)]
                turn["i"] += 1
                a = (nv.BF16, S.M, S.N, S.K)
                nv.check(lib.axn_gemm_fwd_ws(S.X.data_ptr(), S.W.data_ptr(), None, S.Y.data_ptr(), None, *a,
                                             S.K, S.K, S.N, nv.EPI_NONE, ws.data_ptr(), ws_bytes, stream))
                nv.check(lib.axn_gemm_dgrad_ws(S.dY.data_ptr(), S.W.data_ptr(), S.dX.data_ptr(), *a,
                                               S.N, S.K, S.K, ws.data_ptr(), ws_bytes, stream))
                nv.check(lib.axn_gemm_wgrad_ws(S.dY.data_ptr(), S.X.data_ptr(), S.dW.data_ptr(), *a,
                                               S.N, S.K, S.K, 0, nv.BF16, ws.data_ptr(), ws_bytes, stream))

            t = time_loop(skinny_step, max(args.steps, 12), w=6)
            nbytes = 6.0 * (L.M * L.K + L.N * L.K + L.M * L.N)
            shapes["skinny_512x8192x3584"] = {
                "us": round(t * 1e6, 1), "tflops": round(L.flops / t / 1e12, 1),
                "frac_mfma": round(L.flops / t / 1e12 / PEAK_BF16_TFLOPS, 4),
                "gbs": round(nbytes / t / 1e9, 1), "frac_hbm": round(nbytes / t / 1e9 / PEAK_HBM_GBS, 4),
                "operands": "cold (6 operand sets in turn)"}
            del L, ws, sets
            torch.cuda.empty_cache()

        if want("llama_mlp"):
            # Llama-3-8B MLP block, 4096 tokens: gate/up/down projections with the one-pass
            # SwiGLU between them, forward + backward (9 GEMMs, 2 elementwise passes, and
            # torch's add of the two input-gradient contributions).
            Mt, H, I = 4096, 4096, 14336
            g = torch.Generator(device="cuda").manual_seed(12)
            x = torch.randn(Mt, H, generator=g, device="cuda").bfloat16()
            wg, wu = ((torch.randn(I, H, generator=g, device="cuda") * 0.02).bfloat16() for _ in range(2))
            wd = (torch.randn(H, I, generator=g, device="cuda") * 0.02).bfloat16()
            dy = (torch.randn(Mt, H, generator=g, device="cuda") * 1e-3).bfloat16()
            bf = dict(dtype=torch.bfloat16, device="cuda")
            gt, up, act = (torch.empty(Mt, I, **bf) for _ in range(3))
            dact, dgt, dup = (torch.empty(Mt, I, **bf) for _ in range(3))
            y, dx1, dx2 = (torch.empty(Mt, H, **bf) for _ in range(3))
            dwg, dwu, dwd = torch.empty(I, H, **bf), torch.empty(I, H, **bf), torch.empty(H, I, **bf)

            def gate_up_three_calls():
                chk = nv.check
                chk(lib.axn_gemm_fwd(P(x), P(wg), None, P(gt), None, Mt, I, H, H, H, I, nv.EPI_NONE, stream))
                chk(lib.axn_gemm_fwd(P(x), P(wu), None, P(up), None, Mt, I, H, H, H, I, nv.EPI_NONE, stream))
                chk(lib.axn_swiglu_fwd(P(gt), P(up), P(act), nv.BF16, Mt, I, I, stream))

            def gate_up_one_launch():
                nv.check(lib.axn_gemm_swiglu_fwd(P(x), P(wg), P(wu), P(act), P(gt), P(up), nv.BF16, Mt, I, H,
                                                 H, H, I, stream))

            def mlp_block_step():
                chk = nv.check
                gate_up_one_launch()
                chk(lib.axn_gemm_fwd(P(act), P(wd), None, P(y), None, Mt, H, I, I, I, H, nv.EPI_NONE, stream))
                chk(lib.axn_gemm_bwd(P(dy), P(wd), P(act), P(dact), P(dwd), nv.BF16, Mt, H, I, H, I, I, I, I, 0,
                                     nv.BF16, stream))
                chk(lib.axn_swiglu_bwd(P(dact), P(gt), P(up), P(dgt), P(dup), nv.BF16, Mt, I, I, stream))
                chk(lib.axn_gemm_dgrad_pair(P(dgt), P(wg), P(dup), P(wu), P(dx1), nv.BF16, Mt, I, I, H, I, H, H,
                                            stream))
                chk(lib.axn_gemm_wgrad(P(dgt), P(x), P(dwg), Mt, I, H, I, H, H, 0, nv.BF16, stream))
                chk(lib.axn_gemm_wgrad(P(dup), P(x), P(dwu), Mt, I, H, I, H, H, 0, nv.BF16, stream))

            t = time_loop(mlp_block_step, max(args.steps // 2, 3))
            fl = 18.0 * Mt * H * I
            t_sw = time_loop(lambda: nv.check(lib.axn_swiglu_fwd(P(gt), P(up), P(act), nv.BF16, Mt, I, I, stream)), 10)
            t_swb = time_loop(lambda: nv.check(lib.axn_swiglu_bwd(P(dact), P(gt), P(up), P(dgt), P(dup), nv.BF16,
                                                                 Mt, I, I, stream)), 10)

            def dgrad_two_calls():
                nv.check(lib.axn_gemm_dgrad(P(dgt), P(wg), P(dx1), Mt, I, H, I, H, H, stream))
                nv.check(lib.axn_gemm_dgrad(P(dup), P(wu), P(dx2), Mt, I, H, I, H, H, stream))
                torch.add(dx1, dx2, out=dx1)

            t_dp1 = time_loop(lambda: nv.check(lib.axn_gemm_dgrad_pair(
                P(dgt), P(wg), P(dup), P(wu), P(dx1), nv.BF16, Mt, I, I, H, I, H, H, stream)), 10)
            t_dp2 = time_loop(dgrad_two_calls, 10)

            t_gu1 = time_loop(gate_up_one_launch, 10)
            t_gu3 = time_loop(gate_up_three_calls, 10)
            shapes["llama_mlp_block_4096x4096x14336_swiglu"] = {
                "us": round(t * 1e6, 1), "tflops": round(fl / t / 1e12, 1),
                "frac_mfma": round(fl / t / 1e12 / PEAK_BF16_TFLOPS, 4),
                "gate_up_swiglu_one_launch_us": round(t_gu1 * 1e6, 1),
                "gate_up_swiglu_three_calls_us": round(t_gu3 * 1e6, 1),
                "gate_up_dgrad_one_pass_us": round(t_dp1 * 1e6, 1),
                "gate_up_dgrad_two_calls_and_add_us": round(t_dp2 * 1e6, 1),
                "swiglu_fwd_gbs": round(6.0 * Mt * I / t_sw / 1e9, 1),
                "swiglu_bwd_gbs": round(10.0 * Mt * I / t_swb / 1e9, 1)}
            del x, wg, wu, wd, dy, gt, up, act, dact, dgt, dup, y, dx1, dx2, dwg, dwu, dwd
            torch.cuda.empty_cache()

        if want("embedding"):
            # Embedding of the Llama-3 vocabulary at the largest shape of the reference's own
            # test of the layer (B 8, S 2048, H 2048, V 128256, fp32): row gather forward and
            # the dense weight gradient (sort of the token positions + one pass that writes
            # every row of dW once).
            Te, He, Ve = 8 * 2048, 2048, 128256
            g = torch.Generator(device="cuda").manual_seed(13)
            table = torch.randn(Ve, He, generator=g, device="cuda")
            ids = torch.randint(0, Ve, (Te,), generator=g, device="cuda")
            dye = torch.randn(Te, He, generator=g, device="cuda") * 1e-3
            oute = torch.empty(Te, He, device="cuda")
            dtab = torch.empty(Ve, He, device="cuda")
            ws_bytes = lib.axn_embedding_workspace_bytes(Te, Ve)
            wse = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
            t_ef = time_loop(lambda: nv.check(lib.axn_embedding_fwd(
                P(ids), P(table), P(oute), nv.F32, Te, Ve, He, He, He, None, stream)), 20)
            t_eb = time_loop(lambda: nv.check(lib.axn_embedding_bwd(
                P(ids), P(dye), P(dtab), nv.F32, nv.F32, Te, Ve, He, He, He, -1, 0, 0, P(wse), ws_bytes,
                stream)), 20)
            fwd_bytes = 8.0 * Te * He + 8.0 * Te            # rows in, rows out, ids
            bwd_bytes = 4.0 * Te * He + 4.0 * Ve * He + 8.0 * Te  # dY in, every dW row out, ids
            shapes["embedding_16384x2048x128256_f32"] = {
                "fwd_us": round(t_ef * 1e6, 1), "fwd_gbs": round(fwd_bytes / t_ef / 1e9, 1),
                "bwd_us": round(t_eb * 1e6, 1), "bwd_gbs": round(bwd_bytes / t_eb / 1e9, 1),
                "bwd_frac_hbm": round(bwd_bytes / t_eb / 1e9 / PEAK_HBM_GBS, 4)}
            del table, ids, dye, oute, dtab, wse
            torch.cuda.empty_cache()

        if want("small_mlp"):
            # The reference's CPU-runnable configuration: batch 64, 1024 -> 4096 GELU -> 1024 in
            # fp32, MSE loss, one Adam step, through the package's modules (launch-bound: a
            # sanity figure, not a roofline target).
            shapes["mlp_64x1024x4096x1024_fp32_train_step"] = small_mlp_step(torch, time_loop)

    adam = None
    if not args.no_adam:
        adam = bench_adam(args, torch, nv, lib, stream, time_loop)

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(torch) if main_set else None
        if adam is not None:
            adam["cpu_baseline"] = cpu_adam_baseline(torch, adam_sizes(int(args.adam_elements)))
        key = "mlp_64x1024x4096x1024_fp32_train_step"
        if key in shapes:
            shapes[key]["cpu_baseline"] = cpu_small_mlp_baseline(torch)

    out = {
        "metric": "Linear fwd+bwd TFLOP/s on the Llama-3-8B-shaped set (Adam step GB/s under 'adam')",
        "value": round(value, 2) if main_set else None, "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4) if main_set else None, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": "llama3-8b-shaped Linear set, 4096 tokens: qkv 4096->6144, o 4096->4096, "
                        "gate+up 4096->14336 (x2), down 14336->4096; fwd+bwd, bf16 in/out, fp32 "
                        "accumulate, no bias; X~N(0,1), W~N(0,0.02), dY~N(0,1e-3)",
            "flops_per_step": total_flops,
            "frac_of_mfma_peak": round(value / PEAK_BF16_TFLOPS, 4) if main_set else None,
        },
        "roofline": roofline,
        "cpu_baseline": cpu,
        "library_baseline": library,
        "power": power,
        "adam": adam,
        "shapes": shapes,
    }
    print(json.dumps(out))


def small_mlp_tensors(torch):
    import math

    torch.manual_seed(0)
    w1 = torch.nn.init.kaiming_uniform_(torch.empty(4096, 1024), a=math.sqrt(5))
    w2 = torch.nn.init.kaiming_uniform_(torch.empty(1024, 4096), a=math.sqrt(5))
    return w1, torch.zeros(4096), w2, torch.zeros(1024), torch.randn(64, 1024), torch.randn(64, 1024)


def small_mlp_step(torch, time_loop):
    from axonn_amd.intra_layer import Linear
    from axonn_amd.optim import CPUAdam

    w1, b1, w2, b2, x, tgt = small_mlp_tensors(torch)
    l1 = Linear(1024, 4096, fused_activation="gelu")
    l2 = Linear(4096, 1024)
    l1.load_state_dict({"weight": w1, "bias": b1})
    l2.load_state_dict({"weight": w2, "bias": b2})
    model = torch.nn.Sequential(l1, l2).cuda()
    opt = CPUAdam(model.parameters(), lr=1e-3, betas=(0.9, 0.999), eps=1e-8)
    x, tgt = x.cuda(), tgt.cuda()

    def train_step():
        opt.zero_grad()
        torch.nn.functional.mse_loss(model(x), tgt).backward()
        opt.step()

    t = time_loop(train_step, 20)
    flops = 2 * 3 * 2.0 * 64 * 1024 * 4096
    return {"us_per_step": round(t * 1e6, 1), "gflops": round(flops / t / 1e9, 1)}


def cpu_small_mlp_baseline(torch):
    from oracle import torch_cpu as ot

    w1, b1, w2, b2, x, tgt = small_mlp_tensors(torch)
    ot.mlp_step(x, tgt, w1, b1, w2, b2)
    reps = 10
    t0 = time.perf_counter()
    for _ in range(reps):
        ot.mlp_step(x, tgt, w1, b1, w2, b2)
    secs = (time.perf_counter() - t0) / reps
    flops = 2 * 3 * 2.0 * 64 * 1024 * 4096
    return {"us_per_step": round(secs * 1e6, 1), "gflops": round(flops / secs / 1e9, 1),
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": "the same step in torch CPU ops, %d timed steps" % reps}


def adam_sizes(total, n=64, seed=0):
    """64 ragged sizes: seeded fractions of the total clipped to [1e5, 6e7] (scaled
    with the total), remainder onto the largest, sizes left odd on purpose."""
    import numpy as np

    scale = total / 1.3e9
    frac = np.random.default_rng(seed).random(n)
    sizes = np.clip((frac / frac.sum() * total).astype(np.int64), int(1e5 * scale), int(6e7 * scale))
    sizes = sizes | 1
    sizes[np.argmax(sizes)] += int(total) - int(sizes.sum())
    return [int(s) for s in sizes]


def bench_adam(args, torch, nv, lib, stream, time_loop):
    import ctypes

    total = int(args.adam_elements)
    sizes = adam_sizes(total)
    total = sum(sizes)
    g = torch.Generator(device="cuda").manual_seed(1)
    P = torch.empty(total, device="cuda").normal_(0, 0.02, generator=g)
    G = torch.empty(total, dtype=torch.bfloat16, device="cuda")
    chunk = 1 << 26
    for o in range(0, total, chunk):  # bf16(N(0, 1e-3) * 65536) without a 5 GB fp32 temporary
        n = min(chunk, total - o)
        G[o:o + n] = (torch.randn(n, generator=g, device="cuda") * (1e-3 * 65536.0)).bfloat16()
    M = torch.zeros(total, device="cuda")
    V = torch.zeros(total, device="cuda")
    PL = torch.empty(total, dtype=torch.bfloat16, device="cuda")

    def arr(t):
        a = (ctypes.c_void_p * len(sizes))()
        off = 0
        for i, n in enumerate(sizes):
            a[i] = t.data_ptr() + off * t.element_size()
            off += n
        return a

    ag, ap, am, av, apl = arr(G), arr(P), arr(M), arr(V), arr(PL)
    asz = (ctypes.c_int64 * len(sizes))(*sizes)
    ws_bytes = lib.axn_mt_scan_workspace_bytes(len(sizes), total)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    res = torch.zeros(8, dtype=torch.float32, device="cuda")
    inv = 1.0 / 65536.0
    state = {"t": 0}

    def hp(t):
        bc1, bc2 = 1 - 0.9 ** t, 1 - 0.999 ** t
        return nv.AdamHParams(1e-3 / bc1, 1.0 / bc2 ** 0.5, 0.9, 1 - 0.9, 0.999, 1 - 0.999, 1e-8, 0.0)

    def scan():
        nv.check(lib.axn_mt_scan(ag, asz, len(sizes), nv.BF16, inv, 1.0, 0, res.data_ptr(),
                                 ws.data_ptr(), ws_bytes, stream))

    def update():
        state["t"] += 1
        nv.check(lib.axn_mt_adam(ag, ap, am, av, apl, asz, len(sizes), nv.BF16, nv.BF16, inv,
                                 res.data_ptr(), hp(state["t"]), stream))

    def full():
        scan()
        update()

    n = max(min(args.steps, 10), 3)
    t_full = time_loop(full, n, 2)
    t_scan = time_loop(scan, n, 1)
    t_upd = time_loop(update, n, 1)
    found = int(res.view(torch.int32)[4].item())
    # overflow variant: one +inf in tensor 17 -> scan only, every write skipped
    off17 = sum(sizes[:17]) + 5
    saved = G[off17].clone()
    G[off17] = float("inf")
    t_skip = time_loop(full, n, 1)
    found_skip = int(res.view(torch.int32)[4].item())
    G[off17] = saved
    out = {
        "elements": total, "tensors": len(sizes), "bytes_per_element": 30,
        "ms_per_step": round(t_full * 1e3, 4),
        "value": round(30.0 * total / t_full / 1e9, 1), "unit": "GB/s",
        "roofline": {"bound": "hbm", "kernel": "mt_adam_kernel + mt_scan_kernel",
                     "achieved": round(30.0 * total / t_full / 1e9, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(30.0 * total / t_full / 1e9 / PEAK_HBM_GBS, 4),
                     "traffic": ADAM_TRAFFIC_BYTES_PER_STEP if total == 1300000000 else None,
                     "traffic_source": TRAFFIC_SOURCE},
        "scan_ms": round(t_scan * 1e3, 4), "scan_gbs": round(2.0 * total / t_scan / 1e9, 1),
        "update_ms": round(t_upd * 1e3, 4), "update_gbs": round(28.0 * total / t_upd / 1e9, 1),
        "found_inf": found,
        "skip_variant": {"ms_per_step": round(t_skip * 1e3, 4), "found_inf": found_skip,
                         "gbs_at_2B_per_element": round(2.0 * total / t_skip / 1e9, 1)},
    }
    del P, G, M, V, PL, ws
    torch.cuda.empty_cache()
    # What plain streams reach on this box, for scale: the runtime's device-to-device
    # copy and a torch elementwise kernel (both 1 read : 1 write, like the update) and a
    # fill (writes only), 4 GiB each.
    a = torch.empty(1 << 30, dtype=torch.float32, device="cuda").normal_()
    b = torch.empty_like(a)
    nb = a.numel() * 4.0
    probe_lib = nv.load_probe()

    def probe(kind, src, dst):
        def run():
            if probe_lib.axn_probe_stream(kind, src.data_ptr(), dst.data_ptr(), int(nb), stream) != 0:
                raise RuntimeError("axn_probe_stream failed")
        return time_loop(run, 5, 2)

    out["hbm_reference_streams"] = {
        "copy_gbs": round(2 * nb / time_loop(lambda: b.copy_(a), 5, 2) / 1e9, 1),
        "elementwise_1r1w_gbs": round(2 * nb / time_loop(lambda: torch.mul(a, 2.0, out=b), 5, 2) / 1e9, 1),
        "fill_gbs": round(nb / time_loop(lambda: b.fill_(1.0), 5, 2) / 1e9, 1),
        # the library's own plain streams in the optimizer kernels' access pattern
        # (libaxn_probe_gfx950.so: 16-byte vectors, one per lane, non-temporal stores)
        "probe_read_gbs": round(nb / probe(0, a, b) / 1e9, 1),
        "probe_fill_gbs": round(nb / probe(1, a, b) / 1e9, 1),
        "probe_copy_gbs": round(2 * nb / probe(2, a, b) / 1e9, 1),
        "probe_copy_in_place_gbs": round(2 * nb / probe(2, a, a) / 1e9, 1),
        "unit": "GB/s",
    }
    del a, b
    torch.cuda.empty_cache()
    if not args.no_library_baseline:
        out["library_baseline"] = adam_library_baseline(torch, sizes, time_loop)
    return out


def adam_library_baseline(torch, sizes, time_loop):
    """torch's own fused multi-tensor Adam on fp32 parameters and fp32 gradients of the
    same 64 sizes, as a yardstick of the box: 16 B read and 12 B written per element, no
    unscale, overflow check, clipping or low-precision copy."""
    g = torch.Generator(device="cuda").manual_seed(2)
    params = []
    for n in sizes:
        p = torch.empty(n, device="cuda").normal_(0, 0.02, generator=g).requires_grad_(True)
        p.grad = torch.empty(n, device="cuda").normal_(0, 1e-3, generator=g)
        params.append(p)
    opt = torch.optim.Adam(params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, fused=True)
    t = time_loop(opt.step, 5, 2)
    total = sum(sizes)
    res = {"kind": "torch.optim.Adam(fused=True), fp32 gradients, same 64 sizes (no unscale, "
                   "overflow check, clip or bf16 copy)",
           "bytes_per_element": 28, "ms_per_step": round(t * 1e3, 4),
           "value": round(28.0 * total / t / 1e9, 1), "unit": "GB/s"}
    del opt, params
    torch.cuda.empty_cache()
    return res


def cpu_baseline(torch):
    """The torch-CPU restatement of the layer math (oracle/torch_cpu.py) on the
    host cores: fp32 fwd+bwd of the O-projection and QKV shapes, a bounded sample
    of the step's 5 layers."""
    from oracle import torch_cpu as ot

    cores = torch.get_num_threads()
    sample = [(M, N, K) for _, M, N, K in LLAMA_SET]
    # time_linear_set returns seconds and flops PER PASS over the set (after one
    # warm-up pass per layer).  A first single pass sizes the sample: about 10 s of
    # timed CPU work, so that with the warm-ups the leg stays under 30 s.
    secs, flops = ot.time_linear_set(sample, reps=1)
    reps = 1
    more = min(int(10.0 / max(secs, 1e-3)), 8)
    if more >= 2:
        secs, flops = ot.time_linear_set(sample, reps=more)
        reps = more
    return {"value": round(flops / secs / 1e12, 4), "unit": "TFLOP/s", "cores": cores,
            "kind": "port",
            "sample": "fp32 torch-CPU fwd+bwd of all 5 layers of the step, %d timed passes "
                      "(%.1f s of CPU work)" % (reps, secs * reps)}


def cpu_adam_baseline(torch, sizes):
    """The torch-CPU restatement of the optimizer step on the benchmark's own tensor list:
    all of it when the host has the memory (about 21 bytes per element for the states, the
    gradients and the step's temporaries), else the first eighth of the list; the sample
    says which.  One untimed step, then two timed."""
    from oracle import torch_cpu as ot

    def available_bytes():
        try:
            import psutil
            return psutil.virtual_memory().available
        except Exception:   # noqa: BLE001
            return 0

    total = sum(sizes)
    avail = available_bytes()
    if avail >= 40 * total:          # 2x headroom over the ~21 B/element the step touches
        used, what = list(sizes), "all %d tensors" % len(sizes)
    elif avail >= 40 * sum(sizes[:len(sizes) // 8]):
        used = list(sizes[:len(sizes) // 8])
        what = "the first %d of the %d tensors (host memory: %.0f GB available)" % (
            len(used), len(sizes), avail / 1e9)
    else:
        used, what = [1 << 24], "one tensor of 2^24 elements (host memory: %.0f GB available)" % (avail / 1e9)
    # values do not matter for the rate: every tensor is tiled from one random block
    g = torch.Generator().manual_seed(0)
    block = 1 << 22
    base_p = torch.randn(block, generator=g) * 0.02
    base_g = (torch.randn(block, generator=g) * 1e-3 * 65536.0).bfloat16()

    def tiled(base, n):
        out = torch.empty(n, dtype=base.dtype)
        k = n // block
        if k:
            out[:k * block].view(k, block).copy_(base.expand(k, block))
        out[k * block:].copy_(base[:n - k * block])
        return out

    ps = [tiled(base_p, n) for n in used]
    gs = [tiled(base_g, n) for n in used]
    ms = [torch.zeros(n) for n in used]
    vs = [torch.zeros(n) for n in used]
    n = sum(used)
    ot.optimizer_step(gs, ps, ms, vs, 1, 65536.0, max_norm=1.0)
    t0 = time.perf_counter()
    reps = 2
    for i in range(reps):
        ot.optimizer_step(gs, ps, ms, vs, i + 2, 65536.0, max_norm=1.0)
    secs = (time.perf_counter() - t0) / reps
    return {"value": round(30.0 * n / secs / 1e9, 2), "unit": "GB/s",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": "torch-CPU unscale + overflow check + clip + Adam + bf16 cast on %s = %d of "
                      "%d elements, %d timed steps of %.2f s" % (what, n, total, reps, secs)}


if __name__ == "__main__":
    main()
