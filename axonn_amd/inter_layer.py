"""Loss scaling, overflow check and gradient unscaling: the parts of the
reference's training engine that sit on the per-GPU hot path
(axonn/inter_layer.py:18-28 LossScaler, :274-302 _sync_scale, :426-432 the step
gate, :435-445 _check_nan, :447-460 _unscale_gradients).  The pipeline scheduler
and its MPI messaging are not part of this build.
"""

from collections import defaultdict
from dataclasses import dataclass

import torch

from . import ops


@dataclass
class LossScaler:
    """Same fields and defaults as the reference (axonn/inter_layer.py:18-28)."""

    loss_scale: float = 2.0 ** 16
    max_scale: float = 2.0 ** 24
    min_scale: float = 2.0 ** 10
    scaling_window: float = 200
    no_overflow_iters: float = 0


def sync_scale(scaler, local_overflow, verbose=False):
    """Loss-scale state machine (axonn/inter_layer.py:274-302) on one rank;
    returns global_overflow."""
    if local_overflow:
        scaler.loss_scale = max(scaler.loss_scale / 2.0, scaler.min_scale)
        if verbose:
            print(f"overflow detected - reducing loss scale to {scaler.loss_scale}")
        scaler.no_overflow_iters = 0
        return True
    scaler.no_overflow_iters += 1
    if scaler.no_overflow_iters == scaler.scaling_window:
        scaler.loss_scale = min(scaler.loss_scale * 2.0, scaler.max_scale)
        if verbose:
            print(f"increasing loss scale to {scaler.loss_scale}")
        scaler.no_overflow_iters = 0
    return False


def _by_dtype(tensors):
    groups = defaultdict(list)
    for t in tensors:
        groups[t.dtype].append(t)
    return list(groups.values())


def check_nan(tensor):
    """Overflow test of one tensor (axonn/inter_layer.py:435-445): true when the
    tensor's sum, in the tensor's dtype, is inf or nan.  One kernel pass, one
    4-byte read back."""
    result = ops.mt_scan([tensor.detach().reshape(-1)], 1.0, 0.0)
    return bool(result.found_inf.item())


class GradScalerEngine:
    """The mixed-precision tail of `forward_backward_optimizer`
    (axonn/inter_layer.py:426-432): unscale + overflow check, then step unless
    an overflow was seen.  `computation_dtype` float16 turns dynamic loss
    scaling on, as in the reference; bf16 and fp32 step unconditionally."""

    def __init__(self, model, computation_dtype=torch.float16, scaler=None, verbose=False):
        self.model = model
        self.computation_dtype = computation_dtype
        self.scaler = scaler if scaler is not None else LossScaler()
        self.verbose = verbose

    @property
    def loss_scale(self):
        return self.scaler.loss_scale if self.computation_dtype == torch.float16 else 1.0

    def scale_loss(self, loss):
        """axonn/inter_layer.py:240-249: the loss is multiplied by the scale."""
        return loss * self.loss_scale

    def _check_nan(self, tensor):
        return check_nan(tensor)

    def _sync_scale(self, local_overflow):
        assert self.computation_dtype == torch.float16
        return sync_scale(self.scaler, local_overflow, self.verbose)

    @torch.no_grad()
    def _unscale_gradients(self):
        """One scan over all scaled gradients (overflow flag on the device), one
        in-place scaling pass, one 4-byte read back for the host-side state
        machine.  The reference makes a pass and a host sync per parameter."""
        grads = [p.grad for p in self.model.parameters() if p.grad is not None]
        if not grads:
            return self._sync_scale(False)
        result = None
        inv = 1.0 / self.scaler.loss_scale
        for group in _by_dtype(grads):
            result = ops.mt_scan(group, 1.0, 0.0, result=result, accumulate=result is not None)
        for group in _by_dtype(grads):
            ops.mt_scale(group, inv)
        return self._sync_scale(bool(result.found_inf.item()))

    def step(self, optimizer):
        """Returns True when the optimizer stepped."""
        if self.computation_dtype == torch.float16:
            if self._unscale_gradients():
                return False
        optimizer.step()
        return True
