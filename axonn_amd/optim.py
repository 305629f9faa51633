"""Mixed-precision Adam with the reference's `CPUAdam` interface (axonn/optim.py).

The reference keeps fp32 master weights and Adam moments in pinned host memory
and streams them through four GPU staging buffers in 16 M-element buckets,
issuing per bucket two PCIe copies each way, about ten elementwise kernels and a
host synchronisation (optim.py:138-193).  An MI355X holds 288 GB of HBM, so here
the fp32 master weights, both moments, the low-precision weights and the
low-precision gradients all stay resident in flat HBM buffers
(axonn/utils.py:11-30 layout) and one step is two kernels:

  scan   reads the gradients once: overflow flag, sum of squares, clip coefficient
  adam   reads g, p, m, v and writes p, m, v and the low-precision p once,
         skipping every write on the device when the scan saw an overflow

`bucket_size` and `coalescing_factor` are accepted for compatibility and have no
effect.  Behaviour that follows the live training engine rather than this legacy
class (axonn/inter_layer.py:426-432): the step counter advances once per applied
step (the reference advances it twice on torch >= 1.12 and also for skipped
buckets) and an overflow skips the whole step, not single buckets.
"""

import torch
from torch.optim.optimizer import Optimizer

from . import ops
from .inter_layer import LossScaler, sync_scale
from .utils import _coalesce_and_reassign


class CPUAdam(Optimizer):
    """Adam over flat HBM-resident buffers with fp32 master weights.

    `params` are the model's (low-precision or fp32) parameters.  On
    construction they are packed into one flat buffer per param group (their
    `.data` is re-pointed, as the reference's registration step does), an fp32
    master copy and zeroed moments are created, and a flat gradient buffer is
    installed as the parameters' `.grad`, so backward accumulates straight into
    it.

    Extra keyword arguments over the reference: `max_grad_norm` (clip the global
    2-norm inside the step; None = no clipping), `loss_scaler` (a LossScaler;
    default: dynamic scaling for fp16 parameters, scale 1 otherwise) and
    `dynamic_loss_scale` (force the state machine on or off).
    """

    def __init__(
        self,
        params,
        lr=1e-3,
        betas=(0.9, 0.999),
        eps=1e-8,
        weight_decay=0,
        bucket_size=16000000,
        coalescing_factor=4,
        max_grad_norm=None,
        loss_scaler=None,
        dynamic_loss_scale=None,
    ):
        if not 0.0 <= lr:
            raise ValueError("Invalid learning rate: {}".format(lr))
        if not 0.0 <= eps:
            raise ValueError("Invalid epsilon value: {}".format(eps))
        if not 0.0 <= betas[0] < 1.0:
            raise ValueError("Invalid beta parameter at index 0: {}".format(betas[0]))
        if not 0.0 <= betas[1] < 1.0:
            raise ValueError("Invalid beta parameter at index 1: {}".format(betas[1]))
        if not 0.0 <= weight_decay:
            raise ValueError("Invalid weight_decay value: {}".format(weight_decay))
        defaults = dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay)

        self.bucket_size = bucket_size
        self.coalescing_factor = coalescing_factor
        self.max_grad_norm = max_grad_norm

        super(CPUAdam, self).__init__(params, defaults)

        self.calculate_group_offsets()
        self._build_flat_buffers()

        lowp = self._lowp_dtype
        if dynamic_loss_scale is None:
            dynamic_loss_scale = lowp == torch.float16
        self.dynamic_loss_scale = dynamic_loss_scale
        if loss_scaler is None:
            loss_scaler = LossScaler() if dynamic_loss_scale else LossScaler(loss_scale=1.0)
        self.scaler = loss_scaler
        self.step_count = 0
        self.last_step_skipped = False
        self._scan = None

    def __setstate__(self, state):
        super(CPUAdam, self).__setstate__(state)
        for group in self.param_groups:
            group.setdefault("amsgrad", False)

    # -- layout -------------------------------------------------------------
    def calculate_group_offsets(self):
        """Cumulative element counts of the param groups (optim.py:59-65)."""
        self.group_offsets = [0] * (len(self.param_groups) + 1)
        for i in range(1, len(self.group_offsets)):
            group_num_params = 0
            for param in self.param_groups[i - 1]["params"]:
                group_num_params += param.nelement()
            self.group_offsets[i] = self.group_offsets[i - 1] + group_num_params

    def _build_flat_buffers(self):
        all_params = [p for g in self.param_groups for p in g["params"]]
        if len(all_params) == 0:
            raise ValueError("optimizer got an empty parameter list")
        dtypes = {p.dtype for p in all_params}
        if len(dtypes) != 1:
            raise TypeError("all parameters must share one dtype, got %s" % sorted(map(str, dtypes)))
        self._lowp_dtype = all_params[0].dtype
        if self._lowp_dtype not in (torch.bfloat16, torch.float16, torch.float32):
            raise TypeError("parameters must be bf16, fp16 or fp32")
        device = all_params[0].device
        if device.type != "cuda":
            raise RuntimeError("CPUAdam's kernels run on the GPU; move the model to the GPU first")
        with torch.no_grad():
            # flat low-precision weights; every p.data becomes a view into it
            self.model_params_fp16 = _coalesce_and_reassign(all_params)
            total = self.model_params_fp16.numel()
            if self._lowp_dtype == torch.float32:
                # fp32 model: the model weights are the master weights
                self.model_params_fp32 = self.model_params_fp16
            else:
                self.model_params_fp32 = self.model_params_fp16.float()
            self.model_grads_fp16 = torch.zeros(total, dtype=self._lowp_dtype, device=device)
            self.exp_avg = torch.zeros(total, dtype=torch.float32, device=device)
            self.exp_avg_sq = torch.zeros(total, dtype=torch.float32, device=device)
            offset = 0
            self._views = []
            self._params = all_params
            self._grad_views = []   # flat 1-D views, one per parameter: what the scan walks
            self._linked = []       # the `.grad` tensors installed here, one per parameter
            for p in all_params:
                n = p.numel()
                flat_view = self.model_grads_fp16[offset:offset + n]
                p.grad = flat_view.view(p.shape)
                self._linked.append(p.grad)
                self._views.append((offset, n))
                if n:
                    self._grad_views.append(flat_view)
                offset += n
        self._writes_lowp = self._lowp_dtype != torch.float32

    def empty_param_state(self, param):
        """Zeroed Adam state for a slice (optim.py:67-78); states live in HBM."""
        return {
            "step": torch.tensor(0),
            "exp_avg": torch.zeros_like(param, memory_format=torch.preserve_format),
            "exp_avg_sq": torch.zeros_like(param, memory_format=torch.preserve_format),
        }

    def zero_grad(self, set_to_none=False):
        """Zeroes the flat gradient buffer (optim.py:80-81).  Gradients are never
        set to None: they are views into the buffer the step reads."""
        self.model_grads_fp16.zero_()

    # -- step -----------------------------------------------------------------
    @property
    def loss_scale(self):
        return self.scaler.loss_scale

    def _group_slices(self, group_no):
        lo, hi = self.group_offsets[group_no], self.group_offsets[group_no + 1]
        return lo, hi

    def _relink_gradients(self):
        """The step reads the flat gradient buffer; a parameter's `.grad` is a view into
        it.  Code that rebinds `.grad` (`model.zero_grad()` sets it to None by default, a
        cast makes a new tensor) breaks that link without an error: backward would then
        write elsewhere and the step would apply zeros.  A gradient that has moved is
        copied into its slice and the view is installed again; a missing one counts as
        zero: the step runs over the whole flat buffer, as the reference's does
        (axonn/optim.py:157-190), so momentum and weight decay still move that parameter."""
        flat = self.model_grads_fp16
        base, esz = flat.data_ptr(), flat.element_size()
        for i, (p, (offset, n)) in enumerate(zip(self._params, self._views)):
            g = p.grad
            if g is self._linked[i]:   # the view installed by this class: nothing was rebound
                continue
            if g is not None and g.data_ptr() == base + offset * esz and g.numel() == n \
                    and g.dtype == flat.dtype and g.is_contiguous():
                continue
            view = flat[offset:offset + n].view(p.shape)
            if g is None:
                view.zero_()
            else:
                if g.numel() != n:
                    raise RuntimeError("a parameter's gradient changed its size (%d -> %d elements)"
                                       % (n, g.numel()))
                view.copy_(g)
            p.grad = view
            self._linked[i] = p.grad

    @torch.no_grad()
    def step(self, closure=None):
        assert closure is None, "AxoNN CPUAdam does not support closure yet"
        self._relink_gradients()
        inv_scale = 1.0 / self.scaler.loss_scale
        grads = self.model_grads_fp16
        max_norm = float(self.max_grad_norm) if self.max_grad_norm else 0.0
        need_scan = self.dynamic_loss_scale or max_norm > 0.0
        scan = None
        if need_scan:
            # The overflow test is the reference's, per parameter: a tensor's sum, in
            # the gradient dtype, is inf or nan (axonn/inter_layer.py:447-460 walks the
            # parameters; the legacy class walks 16 M-element buckets,
            # axonn/optim.py:158-161).  One sum over the whole flat buffer would trip on
            # fp16 as soon as all scaled gradients together sum past 65504.
            scan = ops.mt_scan(self._grad_views, inv_scale, max_norm, result=self._scan)
            self._scan = scan
        t = self.step_count + 1
        for group_no, group in enumerate(self.param_groups):
            lo, hi = self._group_slices(group_no)
            if hi == lo:
                continue
            beta1, beta2 = group["betas"]
            hp = ops.adam_hparams(t, group["lr"], beta1, beta2, group["eps"],
                                  group["weight_decay"])
            ops.mt_adam(
                [grads[lo:hi]],
                [self.model_params_fp32[lo:hi]],
                [self.exp_avg[lo:hi]],
                [self.exp_avg_sq[lo:hi]],
                [self.model_params_fp16[lo:hi]] if self._writes_lowp else None,
                hp,
                inv_scale=inv_scale,
                scan=scan,
            )
        skipped = False
        if scan is not None:
            skipped = bool(scan.found_inf.item())  # one 4-byte read back per step
        if self.dynamic_loss_scale:
            sync_scale(self.scaler, skipped)
        if not skipped:
            self.step_count = t
        self.last_step_skipped = skipped
        return None

    def grad_norm(self):
        """Global 2-norm of the unscaled gradients seen by the last step (a
        0-dim device tensor), when the step scanned them."""
        return None if self._scan is None else self._scan.total_norm.clone()
