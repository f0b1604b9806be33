"""flashoptim_amd: MI355X (gfx950) implementation of FlashOptim's fused optimizer-step path.

Drop-in for the reference package's public names (``/root/reference/flashoptim/__init__.py:3-33``).  The
numerical work runs in hand-written HIP kernels (``flashoptim_amd/csrc``) reached through the C ABI of
``flashoptim_amd/lib/libflashoptim_hip.so``; this package is the host-side mirror of the optimizer interface.
"""

from .optimizers import (
    FlashAdam,
    FlashAdamW,
    FlashLion,
    FlashOptimizer,
    FlashSGD,
    FlashSGDW,
    GradientReleaseHandle,
    NumericsError,
    cast_model,
    compute_ecc_bits,
    enable_gradient_release,
    reconstruct_fp32_param,
)

__version__ = "0.1.0"

__all__ = [
    "FlashAdam",
    "FlashAdamW",
    "FlashLion",
    "FlashOptimizer",
    "FlashSGD",
    "FlashSGDW",
    "GradientReleaseHandle",
    "NumericsError",
    "cast_model",
    "compute_ecc_bits",
    "enable_gradient_release",
    "reconstruct_fp32_param",
]
