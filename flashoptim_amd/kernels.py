"""Host launch wrappers: plain functions of torch tensors and Python scalars that enqueue the HIP kernels.

This is the boundary the optimizer classes call.  Names, argument order and error behaviour follow the
launch wrappers of the reference (``/root/reference/flashoptim/optimizers.py``, cited as ``ref:``):
``quantize`` (ref:2446), ``dequantize`` (ref:2501), ``reconstruct_fp32_param`` (ref:2835),
``compute_ecc_bits`` (ref:2895), ``_fused_adam_step`` (ref:2203), ``_fused_momentum_step`` (ref:1535).
All of them are asynchronous on the current stream of the tensors' device and mutate their outputs in place.
"""

from __future__ import annotations

from typing import Optional

import torch

from . import _native
from ._native import DTYPE_CODE

GROUP_SIZE = 32

_NUM_MANTISSA_BITS = {torch.float16: 10, torch.bfloat16: 7, torch.float32: 23}


def _require_device(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise NotImplementedError(
            f"{what}: flashoptim_amd only runs on a ROCm GPU; got a {t.dtype} tensor on {t.device} with "
            f"shape {tuple(t.shape)}."
        )


def _require_same_device(ref: torch.Tensor, other: Optional[torch.Tensor], what: str) -> None:
    """The kernels dereference raw addresses: a tensor on another device (or the host) would fault the GPU."""
    if other is not None and other.device != ref.device:
        raise ValueError(f"{what} is on {other.device}, expected {ref.device}.")


def _ecc_bytes(errors: Optional[torch.Tensor]) -> int:
    """Width of the correction term: 0 (none), 1 (int8, 24-bit master) or 2 (int16, 32-bit master);
    same rule as ``_ecc_kernel_params`` (ref:1514-1524)."""
    if errors is None:
        return 0
    width = errors.element_size()
    if width not in (1, 2):
        raise ValueError(f"Errors must have width 1 or 2, not {width}.")
    return width


def _check_group_size(group_size: int) -> None:
    if group_size != GROUP_SIZE:
        raise ValueError(f"group_size is fixed at {GROUP_SIZE} in the HIP kernels; got {group_size}.")


# ------------------------------------------------------------------------------------------ group codec


def quantize(
    x_float: torch.Tensor,
    out_int8: Optional[torch.Tensor] = None,
    out_scales: Optional[torch.Tensor] = None,
    signed: bool = True,
    group_size: int = 32,
    sqrt: bool = False,
    softsign: bool = True,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Group-quantise a floating tensor to 8-bit codes plus one fp16 scale per 32 elements.

    Returns ``(codes, scales)``: codes have the shape of ``x_float`` (int8 when ``signed`` else uint8),
    scales are fp16 ``[ceil(N/32)]`` (ref:2476-2498).
    """
    _check_group_size(group_size)
    _require_device(x_float, "quantize")
    if x_float.dtype not in DTYPE_CODE:
        raise ValueError(f"quantize expects fp32, bf16 or fp16 input, got {x_float.dtype}.")
    x = x_float if x_float.is_contiguous() else x_float.contiguous()
    n = x.numel()
    if out_int8 is None:
        out_int8 = torch.empty_like(x, dtype=torch.int8 if signed else torch.uint8)
    if out_scales is None:
        out_scales = torch.empty((n + GROUP_SIZE - 1) // GROUP_SIZE, device=x.device, dtype=torch.float16)
    if out_int8.numel() != n or not out_int8.is_contiguous() or out_int8.element_size() != 1:
        raise ValueError("out_int8 must be a contiguous 1-byte tensor with as many elements as the input")
    if (out_scales.numel() < (n + GROUP_SIZE - 1) // GROUP_SIZE or out_scales.dtype != torch.float16
            or not out_scales.is_contiguous()):
        raise ValueError("out_scales must be contiguous fp16 with at least ceil(N/32) elements")
    _require_same_device(x, out_int8, "out_int8")
    _require_same_device(x, out_scales, "out_scales")
    if n > 0:
        with _native.device_guard(x.device):
            rc = _native.lib().fo_quantize(
                x.data_ptr(), DTYPE_CODE[x.dtype], out_int8.data_ptr(), out_scales.data_ptr(), n,
                int(signed), int(sqrt), int(softsign), _native.current_stream_ptr(x.device),
            )
        _native.check(rc, "fo_quantize")
    return out_int8, out_scales


def dequantize(
    in_int8: torch.Tensor,
    in_scales: torch.Tensor,
    out_float: Optional[torch.Tensor] = None,
    signed: bool = True,
    group_size: int = 32,
    sqrt: bool = False,
    softsign: bool = True,
) -> torch.Tensor:
    """Inverse of :func:`quantize`; returns fp32 with the shape of the codes (ref:2529-2538)."""
    _check_group_size(group_size)
    _require_device(in_int8, "dequantize")
    if in_int8.dtype != (torch.int8 if signed else torch.uint8):
        raise ValueError(f"codes must be {'int8' if signed else 'uint8'} for signed={signed}, got {in_int8.dtype}.")
    if in_scales.dtype != torch.float16:
        raise ValueError(f"scales must be fp16, got {in_scales.dtype}.")
    codes = in_int8 if in_int8.is_contiguous() else in_int8.contiguous()
    scales = in_scales if in_scales.is_contiguous() else in_scales.contiguous()
    n = codes.numel()
    if scales.numel() < (n + GROUP_SIZE - 1) // GROUP_SIZE:
        raise ValueError("too few scales for the number of codes")
    if out_float is None:
        out_float = torch.empty_like(codes, dtype=torch.float32)
    if out_float.dtype != torch.float32 or out_float.numel() != n or not out_float.is_contiguous():
        raise ValueError("out_float must be a contiguous fp32 tensor with as many elements as the codes")
    _require_same_device(codes, scales, "in_scales")
    _require_same_device(codes, out_float, "out_float")
    if n > 0:
        with _native.device_guard(codes.device):
            rc = _native.lib().fo_dequantize(
                codes.data_ptr(), scales.data_ptr(), out_float.data_ptr(), n, int(signed), int(sqrt),
                int(softsign), _native.current_stream_ptr(codes.device),
            )
        _native.check(rc, "fo_dequantize")
    return out_float


# ------------------------------------------------------------------------------------------------- ECC


def reconstruct_fp32_param(param: torch.Tensor, error_bits: torch.Tensor) -> torch.Tensor:
    """fp32 master weights from a bf16/fp16 parameter and its int8/int16 correction term (ref:2835-2892)."""
    if param.dtype == torch.float32:
        raise ValueError(
            "param is already fp32; ECC reconstruction is only meaningful for narrow dtypes (bf16, fp16). "
            f"Got {param.dtype}."
        )
    if param.dtype not in _NUM_MANTISSA_BITS:
        raise ValueError(f"Unsupported param dtype {param.dtype}; expected one of {list(_NUM_MANTISSA_BITS)}.")
    if error_bits.dtype not in (torch.int8, torch.int16):
        raise ValueError(f"error_bits must be int8 or int16, got {error_bits.dtype}.")
    _require_device(param, "reconstruct_fp32_param")
    if error_bits.numel() != param.numel():
        raise ValueError("error_bits must have as many elements as param")
    _require_same_device(param, error_bits, "error_bits")
    out = torch.empty(param.shape, dtype=torch.float32, device=param.device)
    n = param.numel()
    if n > 0:
        narrow = param.contiguous()
        ecc = error_bits.contiguous()
        with _native.device_guard(param.device):
            rc = _native.lib().fo_ecc_join(
                narrow.data_ptr(), DTYPE_CODE[param.dtype], ecc.data_ptr(), ecc.element_size(), out.data_ptr(), n,
                _native.current_stream_ptr(param.device),
            )
        _native.check(rc, "fo_ecc_join")
    return out


def compute_ecc_bits(
    fp32_param: torch.Tensor, narrow_param: torch.Tensor, master_bytewidth: int = 4
) -> torch.Tensor:
    """Correction term (int8 for 3-byte, int16 for 4-byte masters) such that
    ``reconstruct_fp32_param(narrow_param, result)`` approximates ``fp32_param`` (ref:2895-2970)."""
    if fp32_param.dtype != torch.float32:
        raise ValueError(f"fp32_param must be float32, got {fp32_param.dtype}.")
    if narrow_param.dtype not in (torch.bfloat16, torch.float16):
        raise ValueError(f"narrow_param must be bf16 or fp16, got {narrow_param.dtype}.")
    narrow_bytes = narrow_param.element_size()
    num_err_bytes = master_bytewidth - narrow_bytes
    if num_err_bytes not in (1, 2):
        raise ValueError(
            f"Unsupported dtype combination: master_bytewidth={master_bytewidth} to {narrow_param.dtype} "
            f"({narrow_bytes} bytes). Error byte width {num_err_bytes} must be 1 or 2."
        )
    _require_device(narrow_param, "compute_ecc_bits")
    if fp32_param.numel() != narrow_param.numel():
        raise ValueError("fp32_param and narrow_param must have the same number of elements")
    out = torch.empty(
        narrow_param.shape, dtype=torch.int8 if num_err_bytes == 1 else torch.int16, device=narrow_param.device
    )
    n = narrow_param.numel()
    if n > 0:
        x = fp32_param.to(narrow_param.device).contiguous()
        narrow = narrow_param.contiguous()
        with _native.device_guard(narrow.device):
            rc = _native.lib().fo_ecc_split(
                x.data_ptr(), narrow.data_ptr(), DTYPE_CODE[narrow.dtype], out.data_ptr(), num_err_bytes, n,
                _native.current_stream_ptr(narrow.device),
            )
        _native.check(rc, "fo_ecc_split")
    return out


# ------------------------------------------------------------------------------------------ fused steps


def _check_step_tensors(param: torch.Tensor, grad: torch.Tensor, errors: Optional[torch.Tensor]) -> None:
    """Everything the step kernels assume about param / grad / ECC and cannot check from raw addresses."""
    _require_device(param, "fused step")
    if param.dtype not in DTYPE_CODE:
        raise ValueError(f"Unsupported parameter dtype {param.dtype}.")
    if grad.dtype != param.dtype:
        raise ValueError(f"grad dtype {grad.dtype} must match param dtype {param.dtype}.")
    if grad.numel() != param.numel():
        raise ValueError("grad and param must have the same number of elements")
    if grad.device != param.device:
        raise ValueError("grad and param must be on the same device")
    if not param.is_contiguous() or not grad.is_contiguous():
        raise RuntimeError("the fused kernels need contiguous param and grad tensors")
    if errors is not None:
        if errors.numel() != param.numel():
            raise ValueError("error_bits and param must have the same number of elements")
        if not errors.is_contiguous():
            raise RuntimeError("the fused kernels need a contiguous error_bits tensor")
        _require_same_device(param, errors, "error_bits")


def _check_moment(param: torch.Tensor, values: torch.Tensor, scales: Optional[torch.Tensor], quantized: bool,
                  signed: bool, name: str) -> None:
    """One optimizer state as the step kernels read and write it: 8-bit codes with fp16 group scales, or a tensor
    of the parameter's dtype."""
    n = param.numel()
    if values.numel() != n or not values.is_contiguous():
        raise ValueError(f"{name} must be contiguous with as many elements as param ({n}), got {values.numel()}.")
    _require_same_device(param, values, name)
    if not quantized:
        if values.dtype != param.dtype:
            raise ValueError(f"unquantised {name} must have the parameter's dtype {param.dtype}, got {values.dtype}.")
        return
    if values.dtype != (torch.int8 if signed else torch.uint8):
        raise ValueError(f"quantised {name} must be {'int8' if signed else 'uint8'}, got {values.dtype}.")
    if scales is None or scales.dtype != torch.float16 or not scales.is_contiguous():
        raise ValueError(f"{name} scales must be a contiguous fp16 tensor.")
    if scales.numel() < (n + GROUP_SIZE - 1) // GROUP_SIZE:
        raise ValueError(f"{name} scales hold {scales.numel()} groups, {(n + GROUP_SIZE - 1) // GROUP_SIZE} needed.")
    _require_same_device(param, scales, f"{name} scales")


def _fused_adam_step(
    mom: torch.Tensor,
    mom_scales_f16: torch.Tensor,
    var: torch.Tensor,
    var_scales_f16: torch.Tensor,
    param: torch.Tensor,
    grad: torch.Tensor,
    errors: Optional[torch.Tensor],
    lr: float,
    beta1: float,
    beta2: float,
    eps: float,
    weight_decay: float,
    decoupled: bool,
    step: int,
    quantize_optim_states: bool = True,
    group_size: int = 32,
    exact_update: bool = False,
) -> None:
    """One fused Adam/AdamW step on one contiguous tensor (ref:2203-2251).  ``weight_decay`` is already
    multiplied by lr (or lr/initial_lr) for the decoupled optimizers.

    ``exact_update`` (not in the reference): evaluate the update operation by operation as the reference writes it
    on every element of every variant; every output bit then equals an IEEE evaluation of the reference's formulas.
    The default already does so except for bf16 parameters with an int8 correction term and 2-byte parameters
    without one, whose folded update keeps every master weight within one unit of master precision."""
    _check_group_size(group_size)
    n = param.numel()
    if n == 0:
        return
    _check_step_tensors(param, grad, errors)
    _check_moment(param, mom, mom_scales_f16, quantize_optim_states, True, "mom")
    _check_moment(param, var, var_scales_f16, quantize_optim_states, False, "var")
    ecc_bytes = _ecc_bytes(errors)
    with _native.device_guard(param.device):
        entry = _native.lib().fo_adam_step_exact if exact_update else _native.lib().fo_adam_step
        rc = entry(
            mom.data_ptr(), mom_scales_f16.data_ptr() if quantize_optim_states else None,
            var.data_ptr(), var_scales_f16.data_ptr() if quantize_optim_states else None,
            param.data_ptr(), grad.data_ptr(), _native.ptr(errors), n, DTYPE_CODE[param.dtype], ecc_bytes,
            int(quantize_optim_states), lr, beta1, beta2, eps, weight_decay, int(decoupled), int(step),
            _native.current_stream_ptr(param.device),
        )
    _native.check(rc, "fo_adam_step")


def _fused_momentum_step(
    momentum: torch.Tensor,
    scales_f16: torch.Tensor,
    param: torch.Tensor,
    grad: torch.Tensor,
    errors: Optional[torch.Tensor],
    lr: float,
    mom_coef: float,
    update_coef: float,
    weight_decay: float,
    decoupled: bool = False,
    nesterov: bool = False,
    do_lion: bool = False,
    quantize_optim_states: bool = True,
    group_size: int = 32,
) -> None:
    """One fused SGD/SGDW/Nesterov/Lion step on one contiguous tensor (ref:1535-1579)."""
    _check_group_size(group_size)
    n = param.numel()
    if n == 0:
        return
    _check_step_tensors(param, grad, errors)
    _check_moment(param, momentum, scales_f16, quantize_optim_states, True, "momentum")
    ecc_bytes = _ecc_bytes(errors)
    with _native.device_guard(param.device):
        rc = _native.lib().fo_momentum_step(
            momentum.data_ptr(), scales_f16.data_ptr() if quantize_optim_states else None, param.data_ptr(),
            grad.data_ptr(), _native.ptr(errors), n, DTYPE_CODE[param.dtype], ecc_bytes,
            int(quantize_optim_states), lr, mom_coef, update_coef, weight_decay, int(decoupled), int(nesterov),
            int(do_lion), _native.current_stream_ptr(param.device),
        )
    _native.check(rc, "fo_momentum_step")


def _sgd_plain_step(
    param: torch.Tensor,
    grad: torch.Tensor,
    errors: Optional[torch.Tensor],
    lr: float,
    weight_decay: float,
    decoupled: bool = False,
) -> None:
    """Momentum-free SGD step: the branch the reference evaluates with eager PyTorch ops (ref:1447-1465),
    here one kernel."""
    n = param.numel()
    if n == 0:
        return
    _check_step_tensors(param, grad, errors)
    with _native.device_guard(param.device):
        rc = _native.lib().fo_sgd_plain_step(
            param.data_ptr(), grad.data_ptr(), _native.ptr(errors), n, DTYPE_CODE[param.dtype], _ecc_bytes(errors),
            lr, weight_decay, int(decoupled), _native.current_stream_ptr(param.device),
        )
    _native.check(rc, "fo_sgd_plain_step")


def absmax_many(tensors) -> list:
    """Largest magnitude of every tensor with one launch per (device, dtype); see ``launcher.absmax_many``."""
    from .launcher import absmax_many as _impl

    return _impl(tensors)


def copy_bytes(dst: torch.Tensor, src: torch.Tensor) -> None:
    """Device copy with the step kernels' access shape; a measurement aid (counter calibration, attainable
    streaming rate)."""
    _require_device(src, "copy_bytes")
    _require_same_device(src, dst, "dst")
    nbytes = src.numel() * src.element_size()
    if dst.numel() * dst.element_size() != nbytes:
        raise ValueError("dst and src must have the same size in bytes")
    if not src.is_contiguous() or not dst.is_contiguous():
        raise ValueError("copy_bytes needs contiguous tensors")
    with _native.device_guard(src.device):
        diag = _native.diag_lib()
        rc = diag.fo_copy_bytes(dst.data_ptr(), src.data_ptr(), nbytes, _native.current_stream_ptr(src.device))
    _native.check(rc, "fo_copy_bytes", diag)
