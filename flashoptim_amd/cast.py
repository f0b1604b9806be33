"""``cast_model``: put a model's parameters and buffers into a narrow dtype before training.

Behaviour of ``/root/reference/flashoptim/optimizers.py:2035-2200`` (cited ``ref:``): BatchNorm/InstanceNorm
layers stay fp32 when ``selective``; layers named by fnmatch pattern or given as module objects stay fp32 and
get an input-cast hook (plus an output-cast hook for the "recast" list); tied parameters stay tied.  Host-only
code, no kernels.
"""

from __future__ import annotations

from fnmatch import fnmatch
from typing import Any, Optional, Union

import torch
import torch.nn as nn

LayerSpec = Union[str, nn.Module]

_RUNNING_STAT_NORMS = (
    nn.BatchNorm1d, nn.BatchNorm2d, nn.BatchNorm3d, nn.SyncBatchNorm,
    nn.InstanceNorm1d, nn.InstanceNorm2d, nn.InstanceNorm3d,
)


def _matches_fp32_spec(name: str, module: nn.Module, specs: list[LayerSpec]) -> bool:
    """A module object matches by identity, a string by fnmatch against the full dotted module name."""
    return any((module is s) if isinstance(s, nn.Module) else fnmatch(name, s) for s in specs)


def _fp32_input_cast_hook(module: nn.Module, args: tuple[Any, ...]) -> tuple[Any, ...]:
    del module
    return tuple(a.to(torch.float32) if isinstance(a, torch.Tensor) and a.is_floating_point() else a for a in args)


def _make_output_cast_hook(dtype: torch.dtype):
    def cast_one(o: Any) -> Any:
        return o.to(dtype) if isinstance(o, torch.Tensor) and o.is_floating_point() else o

    def _output_cast_hook(module: nn.Module, input: tuple[Any, ...], output: Any) -> Any:
        del module, input
        if isinstance(output, tuple):
            return tuple(cast_one(o) for o in output)
        return cast_one(output)

    return _output_cast_hook


def cast_model(
    model: nn.Module,
    dtype: torch.dtype = torch.bfloat16,
    selective: bool = True,
    full_precision_layers: Optional[list[LayerSpec]] = None,
    full_precision_recast_layers: Optional[list[LayerSpec]] = None,
) -> None:
    """Cast parameters and floating-point buffers of ``model`` to ``dtype`` in place.

    Args:
        model: module to convert.
        dtype: target dtype (default bf16).
        selective: keep normalisation layers with running statistics (BatchNorm*, InstanceNorm*) in fp32.
        full_precision_layers: modules (objects, or fnmatch patterns on dotted names such as ``"lm_head"`` or
            ``"*.head"``) kept in fp32; their inputs are cast to fp32, their fp32 output is passed on as is.
        full_precision_recast_layers: like ``full_precision_layers`` but the output is cast back to ``dtype``.

    Patterns match the full dotted name: ``"head"`` matches ``model.head`` but not ``model.decoder.head``.
    """
    keep = list(full_precision_layers or [])
    recast = list(full_precision_recast_layers or [])
    fp32_specs = keep + recast

    # names of the tensors owned by (sub)modules that stay fp32
    fp32_params: set[str] = set()
    fp32_buffers: set[str] = set()
    if fp32_specs:
        for mod_name, mod in model.named_modules():
            if _matches_fp32_spec(mod_name, mod, fp32_specs):
                prefix = mod_name + "." if mod_name else ""
                fp32_params.update(prefix + n for n, _ in mod.named_parameters())
                fp32_buffers.update(prefix + n for n, _ in mod.named_buffers())

    name_of_param = {p: n for n, p in model.named_parameters()}
    name_of_buffer = {b: n for n, b in model.named_buffers()}
    converted: dict[Any, torch.Tensor] = {}  # same memory, same view -> one cast tensor, so tied tensors stay tied

    def cast_shared(t: torch.Tensor) -> torch.Tensor:
        if t.numel() == 0:
            return t.data.to(dtype=dtype)  # empty tensors all report address 0 without sharing anything
        key = (t.data.data_ptr(), tuple(t.shape), tuple(t.stride()), t.dtype)
        if key not in converted:
            converted[key] = t.data.to(dtype=dtype)
        return converted[key]

    for module in model.modules():
        if selective and isinstance(module, _RUNNING_STAT_NORMS):
            continue
        for param in module.parameters(recurse=False):
            if name_of_param.get(param, "") not in fp32_params:
                param.data = cast_shared(param)
        for buf in module.buffers(recurse=False):
            if name_of_buffer.get(buf, "") not in fp32_buffers and buf.is_floating_point():
                buf.data = cast_shared(buf)

    if fp32_specs:
        for name, module in model.named_modules():
            wants_recast = _matches_fp32_spec(name, module, recast)
            if (wants_recast or _matches_fp32_spec(name, module, keep)) and not getattr(module, "_has_fp32_input_hook", False):
                module.register_forward_pre_hook(_fp32_input_cast_hook)
                if wants_recast:
                    module.register_forward_hook(_make_output_cast_hook(dtype))
                module._has_fp32_input_hook = True
