"""MI355X (gfx950) fixed-fan-in sparse output layer: host-side mirror of the reference's op surface.

The directory name contains a hyphen, so import it with
``importlib.import_module("ecml23-sparse_amd")``; the module also registers itself under the
alias ``ecml23_sparse_amd`` for ordinary ``import`` statements afterwards.

Everything here dispatches into ``libffi_hip.so`` (hand-written HIP kernels behind a C ABI).
There is no CPU or PyTorch fallback: if the library is missing, calls raise.
"""
import sys as _sys

_sys.modules.setdefault("ecml23_sparse_amd", _sys.modules[__name__])

from . import _lib  # noqa: E402
from .fixed_fan_in_ops import (  # noqa: E402
    fan_in_sparse_matmul,
    fan_in_sparse_matmul_tp,
    fan_in_sparse_matmul_grad,
    fan_in_sparse_matmul_grad_tp,
    FanInSparseMatmul,
    FanInSparseMatmulTp,
    fan_in_sparse_matmul_bf16,
    fan_in_sparse_topk_bf16,
    topk_scores,
    fan_in_sparse_matmul_bias,
    fan_in_sparse_matmul_tp_bias,
    arrange_connections,
    backward_sparse,
    fan_in_sparse_topk,
    lookup_edited,
)
from . import custom_layer, metrics, optimizer  # noqa: E402
from .optimizer import SparseAdam, SparseOptWrapper, RewireCallback  # noqa: E402
from .metrics import (  # noqa: E402
    SparseHingeLoss,
    SparseSquaredHingeLoss,
    SparseBinaryCrossEntropyLoss,
    PrecisionAtK,
    topk_as_matrix,
    SparsePrecision,
    SparseRecall,
)
from .custom_layer import StratifiedRewireLayerV2, StratifiedRewireLayer, RewireSelector, FixedFractionSelector, FixedMagnitudeSelector  # noqa: E402

__all__ = [
    "fan_in_sparse_matmul",
    "fan_in_sparse_matmul_tp",
    "fan_in_sparse_matmul_grad",
    "fan_in_sparse_matmul_grad_tp",
    "FanInSparseMatmul",
    "FanInSparseMatmulTp",
    "fan_in_sparse_matmul_bf16",
    "fan_in_sparse_topk_bf16",
    "topk_scores",
    "fan_in_sparse_matmul_bias",
    "fan_in_sparse_matmul_tp_bias",
    "arrange_connections",
    "backward_sparse",
    "fan_in_sparse_topk",
    "lookup_edited",
    "StratifiedRewireLayerV2",
    "StratifiedRewireLayer",
    "RewireSelector",
    "FixedFractionSelector",
    "FixedMagnitudeSelector",
    "SparseHingeLoss",
    "SparseSquaredHingeLoss",
    "SparseBinaryCrossEntropyLoss",
    "PrecisionAtK",
    "topk_as_matrix",
    "SparsePrecision",
    "SparseRecall",
    "SparseAdam",
    "SparseOptWrapper",
    "RewireCallback",
]
