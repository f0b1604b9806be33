"""ctypes front end of the CPU build of the step kernels' arithmetic (tests/hostmath/hostmath.cpp).

Test infrastructure only.  The functions mirror oracle/c_oracle.py (contiguous CPU torch tensors, mutated in place)
so that a test can run the same inputs through the IEEE restatement of the reference and through the kernels'
own per-element functions.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfo_hostmath.so")
_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
_lib: Optional[ctypes.CDLL] = None


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "hostmath.cpp")
    hdr = os.path.join(_HERE, "..", "..", "flashoptim_amd", "csrc", "fo_math.h")
    stale = os.path.exists(_LIB_PATH) and os.path.getmtime(_LIB_PATH) < max(os.path.getmtime(src), os.path.getmtime(hdr))
    if force or stale or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-B", "-C", _HERE, "libfo_hostmath.so"], check=True, capture_output=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i64, i32, f = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
        L.hm_set_noise.argtypes = [i32]
        L.hm_set_noise.restype = None
        L.hm_adam_step.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i32, i32, i32, f, f, f, f, f, i32, i32, i32, ctypes.POINTER(i64)]
        L.hm_adam_folded_update.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, f, f, f, f, f, i32, i32, vp, vp]
        L.hm_adam_folded_update.restype = None
        L.hm_flow_stats.argtypes = [vp, i32]
        L.hm_flow_stats.restype = None
        L.hm_requantize_wave.argtypes = [vp] * 6
        L.hm_requantize_wave.restype = None
        L.hm_code_over_255.argtypes = [vp]
        L.hm_code_over_255.restype = None
        L.hm_momentum_step.argtypes = [vp, vp, vp, vp, vp, i64, i32, i32, i32, f, f, f, f, i32, i32, i32]
        L.hm_sgd_plain_step.argtypes = [vp, vp, vp, i64, i32, i32, f, f, i32]
        L.hm_div_corrected.argtypes = [vp, vp, vp, i64]
        L.hm_sqrt_corrected.argtypes = [vp, vp, i64]
        L.hm_quantize_group.argtypes = [vp, vp, vp, vp, i64]
        L.hm_quantize_group_from_moments.argtypes = [vp, vp, vp, vp, i64, i32]
        L.hm_quantize_group_from_moments.restype = i64
        L.hm_ecc_join.argtypes = [vp, i32, vp, i32, vp, i64]
        L.hm_ecc_split.argtypes = [vp, vp, i32, vp, i32, i64, i32]
        L.hm_ecc_fraction_table.argtypes = [i32, vp, vp]
        L.hm_ecc_fraction_table.restype = None
        L.hm_softsign_table.argtypes = [vp]
        L.hm_softsign_table.restype = None
        for name in ("hm_div_corrected", "hm_sqrt_corrected", "hm_quantize_group"):
            getattr(L, name).restype = None
        _lib = L
    return _lib


def set_noise(seed: int) -> None:
    """0: the approximate instructions return the correctly rounded value; otherwise they err by one ulp, up or
    down, for about half of their inputs (the pattern depends on `seed`)."""
    lib().hm_set_noise(int(seed))


def _ptr(t):
    if t is None:
        return None
    assert t.device.type == "cpu" and t.is_contiguous()
    return t.data_ptr()


def _ecc_bytes(ecc) -> int:
    return 0 if ecc is None else ecc.element_size()


def adam_step(mom, mom_scales, var, var_scales, param, grad, ecc, lr, beta1, beta2, eps, weight_decay, decoupled, step,
              quantized: bool = True, exact: int = -1) -> int:
    """One Adam step as the kernels compute it.  exact <= 0: what fo_adam_step does for this variant; 1: the
    operation-by-operation update on every element (fo_adam_step_exact).  Returns the number of elements whose
    folded update the guard sent through the operation-by-operation form."""
    flagged = ctypes.c_int64(0)
    rc = lib().hm_adam_step(_ptr(mom), _ptr(mom_scales), _ptr(var), _ptr(var_scales), _ptr(param), _ptr(grad), _ptr(ecc),
                            param.numel(), _DTYPE_CODE[param.dtype], _ecc_bytes(ecc), int(quantized), lr, beta1, beta2,
                            eps, weight_decay, int(decoupled), int(step), int(exact), ctypes.byref(flagged))
    assert rc == 0
    return int(flagged.value)


def adam_folded_update(param, ecc, grad, mom, mom_scales, var, var_scales, lr, beta1, beta2, eps, weight_decay, decoupled, step):
    """The folded Adam update of bf16 parameters with an int8 ECC and quantised states without the repair of the
    flagged elements.  Returns (fp32 results, bool tensor of the elements the guard flags); nothing is changed in
    place."""
    assert param.dtype == torch.bfloat16 and ecc.dtype == torch.int8
    n = param.numel()
    out = torch.empty(n, dtype=torch.float32)
    redo = torch.empty(n, dtype=torch.uint8)
    lib().hm_adam_folded_update(_ptr(mom), _ptr(mom_scales), _ptr(var), _ptr(var_scales), _ptr(param), _ptr(grad), _ptr(ecc), n,
                                lr, beta1, beta2, eps, weight_decay, int(decoupled), int(step), out.data_ptr(), redo.data_ptr())
    return out, redo.bool()


def flow_stats(reset: bool = True) -> dict:
    """What the simulated wavefronts did since the last reset: wavefronts stepped, wave-level questions asked
    (one per verified flow and wavefront, plus one per element position once a flow repairs), how many were answered
    with yes, and how many codes the repairs replaced."""
    out = torch.zeros(4, dtype=torch.int64)
    lib().hm_flow_stats(out.data_ptr(), int(reset))
    return dict(zip(("waves", "questions", "yes", "codes_replaced"), out.tolist()))


def requantize_wave(m: torch.Tensor, v: torch.Tensor):
    """One wavefront (512 first-moment and 512 second-moment values, lane l holding values 8l .. 8l+7, four lanes per
    quantisation group) through the kernels' verified requantisation flows.  Returns (codes of m, codes of v, the
    exact forms' codes of m, of v)."""
    assert m.numel() == 512 and v.numel() == 512 and m.dtype == v.dtype == torch.float32
    out = [torch.empty(512, dtype=torch.uint8) for _ in range(4)]
    lib().hm_requantize_wave(_ptr(m.contiguous()), _ptr(v.contiguous()), *(t.data_ptr() for t in out))
    return out


def code_over_255() -> torch.Tensor:
    """code_over_255(q) of fo_math.h for q = 0 .. 255."""
    out = torch.empty(256, dtype=torch.float32)
    lib().hm_code_over_255(out.data_ptr())
    return out


def momentum_step(mom, scales, param, grad, ecc, lr, mom_coef, update_coef, weight_decay, decoupled=False, nesterov=False,
                  do_lion=False, quantized: bool = True) -> None:
    rc = lib().hm_momentum_step(_ptr(mom), _ptr(scales), _ptr(param), _ptr(grad), _ptr(ecc), param.numel(),
                                _DTYPE_CODE[param.dtype], _ecc_bytes(ecc), int(quantized), lr, mom_coef, update_coef,
                                weight_decay, int(decoupled), int(nesterov), int(do_lion))
    assert rc == 0


def sgd_plain_step(param, grad, ecc, lr, weight_decay, decoupled=False) -> None:
    rc = lib().hm_sgd_plain_step(_ptr(param), _ptr(grad), _ptr(ecc), param.numel(), _DTYPE_CODE[param.dtype],
                                 _ecc_bytes(ecc), lr, weight_decay, int(decoupled))
    assert rc == 0


def div_corrected(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    out = torch.empty_like(a)
    lib().hm_div_corrected(_ptr(a), _ptr(b), _ptr(out), a.numel())
    return out


def sqrt_corrected(x: torch.Tensor) -> torch.Tensor:
    out = torch.empty_like(x)
    lib().hm_sqrt_corrected(_ptr(x), _ptr(out), x.numel())
    return out


def quantize_group(m: torch.Tensor, r: torch.Tensor):
    qm = torch.empty(m.numel(), dtype=torch.int8)
    qv = torch.empty(r.numel(), dtype=torch.uint8)
    lib().hm_quantize_group(_ptr(m), _ptr(r), _ptr(qm), _ptr(qv), m.numel())
    return qm, qv


def quantize_group_from_moments(m: torch.Tensor, v: torch.Tensor, quick: bool):
    """Codes of ONE group (all of m / v) from its moment values: through the quick forms with verification, or through
    the exact forms alone.  Returns (first-moment codes, second-moment codes, number of values that failed the margin
    test and were redone exactly)."""
    qm = torch.empty(m.numel(), dtype=torch.int8)
    qv = torch.empty(v.numel(), dtype=torch.uint8)
    failed = lib().hm_quantize_group_from_moments(_ptr(m), _ptr(v), _ptr(qm), _ptr(qv), m.numel(), int(quick))
    return qm, qv, int(failed)


def ecc_join(narrow: torch.Tensor, ecc: torch.Tensor) -> torch.Tensor:
    out = torch.empty(narrow.shape, dtype=torch.float32)
    assert lib().hm_ecc_join(_ptr(narrow), _DTYPE_CODE[narrow.dtype], _ptr(ecc), ecc.element_size(), _ptr(out), narrow.numel()) == 0
    return out


def ecc_split(x: torch.Tensor, narrow: torch.Tensor, ecc_dtype: torch.dtype, clamp: bool = True) -> torch.Tensor:
    out = torch.empty(narrow.shape, dtype=ecc_dtype)
    assert lib().hm_ecc_split(_ptr(x), _ptr(narrow), _DTYPE_CODE[narrow.dtype], _ptr(out), out.element_size(), narrow.numel(),
                              int(clamp)) == 0
    return out


def ecc_fraction_table(narrow_dtype: torch.dtype):
    """(table entries, arithmetic form) of (q/127) * 2^-(mant+1) for the 256 int8 bytes."""
    t, a = torch.empty(256), torch.empty(256)
    lib().hm_ecc_fraction_table(_DTYPE_CODE[narrow_dtype], _ptr(t), _ptr(a))
    return t, a


def softsign_table() -> torch.Tensor:
    t = torch.empty(256)
    lib().hm_softsign_table(_ptr(t))
    return t
