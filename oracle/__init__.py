"""CPU oracle for the hot path: TEST INFRASTRUCTURE, not product code.

A numpy restatement of what the reference (axonn-ai/axonn, pure Python on
torch) computes on the per-GPU hot path at a 1 x 1 x 1 grid:

  oracle.linear   axonn/intra_layer/fully_connected.py (Linear / AsyncLinear)
                  and the deferred gradient accumulation of
                  axonn/intra_layer/overlap_communication.py:33-47
  oracle.optim    axonn/optim.py (CPUAdam.step), the loss scaler and overflow
                  check of axonn/inter_layer.py:18-28, :274-302, :426-460, the
                  gradient clipping of
                  axonn/intra_layer/gradient_normalization.py and the flat
                  buffer layout of axonn/utils.py:11-30
  oracle.torch_cpu  the same path written with torch CPU ops (what the
                  reference's calls reduce to on one rank); used for timing the
                  CPU baseline and as a second, independent checker

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package, and only as the checker.  The shipped package (axonn_amd) never
imports it and has no CPU fallback.

What pins the oracle (tests/test_oracle.py, tests/test_golden.py):
  - GEMM forward/backward, bias: equality with torch.nn.Linear autograd on the
    reference's own test shapes and scaling (axonn/tests/test_intra_layer_fc.py),
    brute-force triple loops on tiny shapes, linearity, micro-batch additivity
  - GELU and its derivative: math.erf, torch.nn.functional.gelu, finite
    differences
  - bf16 rounding: torch's float32 -> bfloat16 conversion incl. ties, infinities
  - overflow check: brute force on tiny vectors, invariant
    "sum-based == any-nonfinite while the sum itself stays in range"
  - gradient norm / clipping: torch.nn.utils.clip_grad_norm_ and the closed form
  - Adam: torch.optim.Adam(foreach=False) over several steps, the step-1 closed
    form, and a float64 evaluation of the same recurrences
  - loss-scale state machine: the transition table of inter_layer.py:281-301

Parity unpinned by any test of the reference itself: the optimizer step, the
loss scaler and the overflow check (the reference has no test for them); they
are pinned by the library routines and closed forms listed above only.
"""
