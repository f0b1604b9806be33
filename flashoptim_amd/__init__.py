"""flashoptim_amd: MI355X (gfx950) implementation of FlashOptim's fused optimizer-step path.

The numerical work runs in hand-written HIP kernels (``flashoptim_amd/csrc``) reached through the C ABI of
``flashoptim_amd/lib/libflashoptim_hip.so``; this package is the host-side mirror of the reference's
optimizer interface.
"""

from .kernels import compute_ecc_bits, dequantize, quantize, reconstruct_fp32_param

__all__ = ["compute_ecc_bits", "dequantize", "quantize", "reconstruct_fp32_param"]
