"""Single import point mirroring ``flashoptim.optimizers`` of the reference: everything its users and tests
import from there is importable from here under the same name."""

from .adam import FlashAdam, FlashAdamW
from .base import (
    _BITS_TO_BYTES,
    _DTYPE_WIDTHS,
    FlashOptimizer,
    NumericsError,
    _log2_min_expressible_step_size,
)
from .cast import cast_model
from .kernels import (
    _fused_adam_step,
    _fused_momentum_step,
    compute_ecc_bits,
    dequantize,
    quantize,
    reconstruct_fp32_param,
)
from .lion import FlashLion
from .release import GradientReleaseHandle, enable_gradient_release
from .sgd import FlashSGD, FlashSGDW
from .state import QuantizedTensorSpec, _MaybeQuantizedTensor

__all__ = [
    "NumericsError",
    "FlashOptimizer",
    "FlashLion",
    "FlashSGD",
    "FlashSGDW",
    "FlashAdam",
    "FlashAdamW",
    "GradientReleaseHandle",
    "cast_model",
    "compute_ecc_bits",
    "enable_gradient_release",
    "reconstruct_fp32_param",
]
