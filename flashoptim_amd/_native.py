"""ctypes binding of libflashoptim_hip.so (C ABI declared in include/flashoptim_hip.h).

The library is the only implementation of the step math in this package: if it cannot be loaded the
package raises, it never falls back to PyTorch ops.  Calls release the GIL (plain ``ctypes.CDLL``), take
raw ``data_ptr()`` values and the current HIP stream, and return immediately after enqueueing.
"""

from __future__ import annotations

import contextlib
import ctypes
import os
import threading
from typing import Optional

import torch

_LIB_NAME = "libflashoptim_hip.so"
# FLASHOPTIM_HIP_LIBRARY points at an alternative build of the same library (kernel tuning); default: in-tree
_LIB_PATH = os.environ.get("FLASHOPTIM_HIP_LIBRARY") or os.path.join(
    os.path.dirname(os.path.abspath(__file__)), "lib", _LIB_NAME
)

DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
TILE_ELEMS = 4096


class FoTensorDesc(ctypes.Structure):
    """Mirror of ``fo_tensor_desc``."""

    _fields_ = [
        ("param", ctypes.c_void_p),
        ("grad", ctypes.c_void_p),
        ("ecc", ctypes.c_void_p),
        ("mom", ctypes.c_void_p),
        ("mom_scales", ctypes.c_void_p),
        ("var", ctypes.c_void_p),
        ("var_scales", ctypes.c_void_p),
        ("n", ctypes.c_int64),
    ]


class FoChunk(ctypes.Structure):
    """Mirror of ``fo_chunk``."""

    _fields_ = [
        ("tensor", ctypes.c_int32),
        ("first_tile", ctypes.c_int32),
        ("n_tiles", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
    ]


_DIAG_LIB_PATH = os.path.join(os.path.dirname(_LIB_PATH), "libflashoptim_hip_diag.so")

_lock = threading.Lock()
_lib: Optional[ctypes.CDLL] = None
_diag_lib: Optional[ctypes.CDLL] = None

# name -> (restype, argtypes); kept in one table so a test can check it against the header
_vp, _i64, _i32, _f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
SIGNATURES = {
    "fo_version": (_i32, []),
    "fo_last_error": (ctypes.c_char_p, []),
    "fo_device_compute_units": (_i32, [_i32]),
    "fo_adam_step": (_i32, [_vp] * 7 + [_i64, _i32, _i32, _i32] + [_f32] * 5 + [_i32, _i32, _vp]),
    "fo_adam_step_exact": (_i32, [_vp] * 7 + [_i64, _i32, _i32, _i32] + [_f32] * 5 + [_i32, _i32, _vp]),
    "fo_momentum_step": (_i32, [_vp] * 5 + [_i64, _i32, _i32, _i32] + [_f32] * 4 + [_i32, _i32, _i32, _vp]),
    "fo_sgd_plain_step": (_i32, [_vp] * 3 + [_i64, _i32, _i32, _f32, _f32, _i32, _vp]),
    "fo_count_chunks": (_i64, [_vp, _i64, _i32]),
    "fo_build_chunks": (_i64, [_vp, _i64, _i32, _vp, _i64]),
    "fo_multi_adam_step": (_i32, [_vp, _i64, _vp, _i64, _i32, _i32, _i32] + [_f32] * 5 + [_i32, _i32, _vp]),
    "fo_multi_adam_step_exact": (_i32, [_vp, _i64, _vp, _i64, _i32, _i32, _i32] + [_f32] * 5 + [_i32, _i32, _vp]),
    "fo_multi_adam_step_static": (_i32, [_vp, _i64, _i32, _i32, _i32] + [_f32] * 5 + [_i32, _i32, _vp]),
    "fo_multi_momentum_step": (_i32, [_vp, _i64, _vp, _i64, _i32, _i32, _i32] + [_f32] * 4 + [_i32, _i32, _i32, _vp]),
    "fo_multi_sgd_plain_step": (_i32, [_vp, _i64, _vp, _i64, _i32, _i32, _f32, _f32, _i32, _vp]),
    "fo_multi_absmax": (_i32, [_vp, _i64, _vp, _i64, _i32, _vp, _vp]),
    "fo_quantize": (_i32, [_vp, _i32, _vp, _vp, _i64, _i32, _i32, _i32, _vp]),
    "fo_dequantize": (_i32, [_vp, _vp, _vp, _i64, _i32, _i32, _i32, _vp]),
    "fo_ecc_join": (_i32, [_vp, _i32, _vp, _i32, _vp, _i64, _vp]),
    "fo_ecc_split": (_i32, [_vp, _vp, _i32, _vp, _i32, _i64, _vp]),
}
# include/flashoptim_hip_diag.h: exported by the diagnostics build only (libflashoptim_hip_diag.so, which also
# exports everything above)
DIAG_SIGNATURES = {
    "fo_copy_bytes": (_i32, [_vp, _vp, _i64, _vp]),
    "fo_multi_adam_streams_copy": (_i32, [_vp, _i64, _vp, _i64, _i32, _i32, _i32, _vp]),
    "fo_multi_momentum_streams_copy": (_i32, [_vp, _i64, _vp, _i64, _i32, _i32, _i32, _vp]),
    "fo_adam_step_residency": (_i32, [_i32] * 5 + [_vp] * 3),
    "fo_momentum_step_residency": (_i32, [_i32] * 5 + [_vp] * 3),
    "fo_probe_residency": (_i32, [_i32, _vp, _i64, _vp, _vp]),
}


def library_path() -> str:
    return _LIB_PATH


def _load(path: str, signatures: dict) -> ctypes.CDLL:
    if not os.path.exists(path):
        raise RuntimeError(
            f"{path} is missing: flashoptim_amd has no implementation without its HIP "
            "library. Build it with `make -C flashoptim_amd/csrc` (or __graft_entry__.build())."
        )
    handle = ctypes.CDLL(path)
    for name, (restype, argtypes) in signatures.items():
        try:
            fn = getattr(handle, name)
        except AttributeError:
            raise RuntimeError(
                f"{path} does not export {name}: it was built from older sources. Rebuild it with "
                "`make -C flashoptim_amd/csrc`."
            ) from None
        fn.restype = restype
        fn.argtypes = argtypes
    return handle


def lib() -> ctypes.CDLL:
    """Load the HIP library once; raise loudly when it has not been built."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                _lib = _load(_LIB_PATH, SIGNATURES)
    return _lib


def diag_lib() -> ctypes.CDLL:
    """The diagnostics build of the library (measurement kernels and residency queries, for the benchmark and the
    tests; the optimizer path never loads it)."""
    global _diag_lib
    if _diag_lib is None:
        with _lock:
            if _diag_lib is None:
                _diag_lib = _load(_DIAG_LIB_PATH, {**SIGNATURES, **DIAG_SIGNATURES})
    return _diag_lib


def diag_library_path() -> str:
    return _DIAG_LIB_PATH


def check(rc: int, what: str, library: Optional[ctypes.CDLL] = None) -> None:
    """Translate a non-zero native return code into RuntimeError with the message of the library that returned it."""
    if rc != 0:
        msg = (library or lib()).fo_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed (code {rc}): {msg}")


def current_stream_ptr(device: torch.device) -> int:
    """Raw handle of torch's current stream on `device` (what the launches are enqueued on)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    return torch._C._cuda_getCurrentRawStream(index)


_NO_GUARD = contextlib.nullcontext()


def device_guard(device: torch.device):
    """Context that makes `device` current for the HIP calls inside it; free when it already is (the usual case:
    ``torch.cuda.device`` costs several microseconds per launch)."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(device)


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()
