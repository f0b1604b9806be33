"""ctypes front end of the scalar C restatement (oracle/fo_oracle.c -> oracle/libfo_oracle.so).

TEST INFRASTRUCTURE ONLY (see oracle/torch_oracle.py for the rules and the parity notes).
All functions work on contiguous CPU torch tensors and mutate them in place exactly as the
reference kernels mutate device tensors.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfo_oracle.so")
_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}

_lib: Optional[ctypes.CDLL] = None


def build(force: bool = False) -> str:
    """Compile the C restatement with the Makefile next to this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-B", "-C", _HERE, "libfo_oracle.so"], check=True, capture_output=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i64, i32, f = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
        L.fo_oracle_ecc_join.argtypes = [vp, i32, vp, i32, vp, i64]
        L.fo_oracle_ecc_split.argtypes = [vp, vp, i32, vp, i32, i64]
        L.fo_oracle_quantize.argtypes = [vp, i32, vp, vp, i64, i32, i32, i32]
        L.fo_oracle_dequantize.argtypes = [vp, vp, vp, i64, i32, i32, i32]
        L.fo_oracle_adam_step.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i32, i32, i32, f, f, f, f, f, i32, i32]
        L.fo_oracle_momentum_step.argtypes = [vp, vp, vp, vp, vp, i64, i32, i32, i32, f, f, f, f, i32, i32, i32]
        L.fo_oracle_sgd_plain_step.argtypes = [vp, vp, vp, i64, i32, i32, f, f, i32]
        L.fo_oracle_ecc_invariants.argtypes = [i32, i32, i32, ctypes.POINTER(ctypes.c_int64)]
        L.fo_oracle_ecc_invariants.restype = None
        L.fo_oracle_f32_to_f16.argtypes = [f]
        L.fo_oracle_f32_to_f16.restype = ctypes.c_uint16
        L.fo_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.fo_oracle_f16_to_f32.restype = f
        L.fo_oracle_f32_to_bf16.argtypes = [f]
        L.fo_oracle_f32_to_bf16.restype = ctypes.c_uint16
        for name in ("fo_oracle_ecc_join", "fo_oracle_ecc_split", "fo_oracle_quantize", "fo_oracle_dequantize",
                     "fo_oracle_adam_step", "fo_oracle_momentum_step", "fo_oracle_sgd_plain_step"):
            getattr(L, name).restype = None
        _lib = L
    return _lib


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None:
        return None
    assert t.device.type == "cpu" and t.is_contiguous()
    return t.data_ptr()


def _ecc_bytes(ecc: Optional[torch.Tensor]) -> int:
    if ecc is None:
        return 0
    assert ecc.dtype in (torch.int8, torch.int16)
    return ecc.element_size()


def quantize(x: torch.Tensor, signed: bool = True, sqrt: bool = False, softsign: bool = True):
    x = x.contiguous()
    n = x.numel()
    codes = torch.empty(x.shape, dtype=torch.int8 if signed else torch.uint8)
    scales = torch.empty((n + 31) // 32, dtype=torch.float16)
    lib().fo_oracle_quantize(_ptr(x), _DTYPE_CODE[x.dtype], _ptr(codes), _ptr(scales), n, int(signed), int(sqrt),
                             int(softsign))
    return codes, scales


def dequantize(codes: torch.Tensor, scales: torch.Tensor, signed: bool = True, sqrt: bool = False,
               softsign: bool = True) -> torch.Tensor:
    codes = codes.contiguous()
    assert codes.dtype == (torch.int8 if signed else torch.uint8) and scales.dtype == torch.float16
    out = torch.empty(codes.shape, dtype=torch.float32)
    lib().fo_oracle_dequantize(_ptr(codes), _ptr(scales.contiguous()), _ptr(out), codes.numel(), int(signed),
                               int(sqrt), int(softsign))
    return out


def ecc_join(narrow: torch.Tensor, ecc: torch.Tensor) -> torch.Tensor:
    out = torch.empty(narrow.shape, dtype=torch.float32)
    lib().fo_oracle_ecc_join(_ptr(narrow.contiguous()), _DTYPE_CODE[narrow.dtype], _ptr(ecc.contiguous()),
                             _ecc_bytes(ecc), _ptr(out), narrow.numel())
    return out


def ecc_split(x_f32: torch.Tensor, narrow: torch.Tensor, ecc_dtype: torch.dtype) -> torch.Tensor:
    assert x_f32.dtype == torch.float32
    out = torch.empty(narrow.shape, dtype=ecc_dtype)
    lib().fo_oracle_ecc_split(_ptr(x_f32.contiguous()), _ptr(narrow.contiguous()), _DTYPE_CODE[narrow.dtype],
                              _ptr(out), _ecc_bytes(out), narrow.numel())
    return out


def adam_step(mom, mom_scales, var, var_scales, param, grad, ecc, lr, beta1, beta2, eps, weight_decay, decoupled,
              step, quantized: bool = True) -> None:
    """In place; with quantized=False mom/var are param-dtype tensors and the scales are ignored."""
    assert grad.dtype == param.dtype
    lib().fo_oracle_adam_step(_ptr(mom), _ptr(mom_scales), _ptr(var), _ptr(var_scales), _ptr(param), _ptr(grad),
                              _ptr(ecc), param.numel(), _DTYPE_CODE[param.dtype], _ecc_bytes(ecc), int(quantized),
                              lr, beta1, beta2, eps, weight_decay, int(decoupled), int(step))


def momentum_step(mom, scales, param, grad, ecc, lr, mom_coef, update_coef, weight_decay, decoupled=False,
                  nesterov=False, do_lion=False, quantized: bool = True) -> None:
    assert grad.dtype == param.dtype
    lib().fo_oracle_momentum_step(_ptr(mom), _ptr(scales), _ptr(param), _ptr(grad), _ptr(ecc), param.numel(),
                                  _DTYPE_CODE[param.dtype], _ecc_bytes(ecc), int(quantized), lr, mom_coef,
                                  update_coef, weight_decay, int(decoupled), int(nesterov), int(do_lion))


def sgd_plain_step(param, grad, ecc, lr, weight_decay, decoupled=False) -> None:
    lib().fo_oracle_sgd_plain_step(_ptr(param), _ptr(grad), _ptr(ecc), param.numel(), _DTYPE_CODE[param.dtype],
                                   _ecc_bytes(ecc), lr, weight_decay, int(decoupled))


ECC_INVARIANT_NAMES = (
    "perfect_downcast_8bit", "perfect_downcast_16bit", "16bit_no_worse_zero", "16bit_no_worse_always",
    "8bit_corrects_representable", "16bit_corrects_representable", "16bit_better_in_middle_range",
)


def ecc_invariants(sign: int, exponent: int, narrow_dtype: torch.dtype) -> dict:
    """Exception counts of the seven ECC invariants over all 2**23 mantissas of one binade."""
    counts = (ctypes.c_int64 * 7)()
    lib().fo_oracle_ecc_invariants(sign, exponent, _DTYPE_CODE[narrow_dtype], counts)
    return dict(zip(ECC_INVARIANT_NAMES, [int(c) for c in counts]))
