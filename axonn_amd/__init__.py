"""axonn_amd: the per-GPU training hot path of AxoNN, native on AMD MI355X.

The package keeps the reference's Python surface for the one path it covers

    axonn_amd.axonn.init(...)                      (axonn/axonn.py:21-67, 1 x 1 x 1 only)
    axonn_amd.intra_layer.Linear                   (axonn/intra_layer/fully_connected.py)
    axonn_amd.intra_layer.Embedding                (axonn/intra_layer/embedding.py)
    axonn_amd.intra_layer.clip_grad_norm_          (axonn/intra_layer/gradient_normalization.py)
    axonn_amd.intra_layer.optimize_communication   (axonn/intra_layer/overlap_communication.py)
    axonn_amd.optim.CPUAdam                        (axonn/optim.py)
    axonn_amd.inter_layer.LossScaler / GradScalerEngine   (axonn/inter_layer.py:18-28, :274-302, :426-460)
    axonn_amd.checkpoint.save / load               (axonn/checkpoint.py)
    axonn_amd.models.transformers.parallelize      (axonn/models/transformers)

and runs all of its arithmetic in hand-written gfx950 kernels behind the C ABI
of libaxn_gfx950.so (include/axn.h).  There is no CPU or library fallback.
"""

from . import axonn  # noqa: F401
from . import config  # noqa: F401

__version__ = "0.1.0"
