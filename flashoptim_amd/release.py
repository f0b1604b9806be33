"""Gradient release: step each parameter as soon as its gradient has been accumulated, then free the gradient.

Interface of ``/root/reference/flashoptim/optimizers.py:2998-3138`` (cited ``ref:``).  The hooks run on the
autograd engine's thread; each one issues a single-tensor HIP launch on that thread's current stream (pointer
extraction plus one kernel launch, no allocation, no synchronisation), so the update interleaves with the rest
of the backward pass.
"""

from __future__ import annotations

import weakref
from dataclasses import dataclass
from typing import Any, Callable, Optional

import torch

from .base import FlashOptimizer


@dataclass
class GradientReleaseHandle:
    """Returned by :func:`enable_gradient_release`; ``remove()`` restores normal ``step`` / ``zero_grad``."""

    _hooks: list
    _optimizer: FlashOptimizer

    def remove(self) -> None:
        for h in self._hooks:
            h.remove()
        self._hooks.clear()
        self._optimizer._gradient_release = False

    @property
    def active(self) -> bool:
        return len(self._hooks) > 0


def _make_hook(p: torch.Tensor, group: dict[str, Any], optimizer: FlashOptimizer,
               pre_step: Optional[Callable[[torch.Tensor, dict[str, Any]], bool]]) -> Callable[[torch.Tensor], None]:
    opt_ref = weakref.ref(optimizer)

    def hook(_p: torch.Tensor) -> None:
        opt = opt_ref()
        if opt is None or p.grad is None:
            return
        if pre_step is not None and not pre_step(p, group):
            return
        opt.step_param(p, group)
        p.grad = None

    return hook


def _register_plain_hooks(model: torch.nn.Module, optimizer: FlashOptimizer, hooks: list,
                          pre_step: Optional[Callable[[torch.Tensor, dict[str, Any]], bool]],
                          param_to_group: dict[int, dict[str, Any]]) -> None:
    # model.parameters() yields a tied tensor once, and a post-accumulate hook fires once per backward after all
    # contributions are summed, so shared parameters are stepped exactly once
    for p in model.parameters():
        if p.requires_grad:
            hooks.append(p.register_post_accumulate_grad_hook(_make_hook(p, param_to_group[id(p)], optimizer, pre_step)))


def enable_gradient_release(
    model: torch.nn.Module,
    optimizer: FlashOptimizer,
    *,
    grad_scaler: Optional["torch.amp.GradScaler"] = None,
    pre_step: Optional[Callable[[torch.Tensor, dict[str, Any]], bool]] = None,
) -> GradientReleaseHandle:
    """Attach hooks that step and free each parameter's gradient during ``backward()``.

    While active ``optimizer.step()`` and ``optimizer.zero_grad()`` warn and do nothing.

    Args:
        model: module whose parameters ``optimizer`` owns.
        optimizer: a :class:`FlashOptimizer`.
        grad_scaler: reserved; anything but ``None`` raises ``NotImplementedError``.
        pre_step: ``(param, group) -> bool`` called before each step; ``False`` skips that parameter.

    Raises:
        TypeError: ``model`` is wrapped in DistributedDataParallel or FullyShardedDataParallel (FSDP1).
        NotImplementedError: ``grad_scaler`` was given.
    """
    if grad_scaler is not None:
        raise NotImplementedError(
            "GradScaler integration with enable_gradient_release is not yet implemented. Per-parameter unscaling "
            "requires multiplying each grad by 1/scale, checking for inf, and skipping steps on inf — this is "
            "planned but not yet available."
        )
    from torch.distributed.fsdp import FullyShardedDataParallel as FSDP
    from torch.nn.parallel import DistributedDataParallel as DDP

    if isinstance(model, FSDP):
        raise TypeError(
            "enable_gradient_release() does not support FullyShardedDataParallel (FSDP1) models. Use FSDP2 "
            "(fully_shard) instead, which is compatible with per-parameter gradient release."
        )
    if isinstance(model, DDP):
        # DDP copies its bucket buffer back into p.grad after the hooks ran, so the gradient cannot be freed
        raise TypeError("enable_gradient_release() does not support DistributedDataParallel (DDP). ")

    param_to_group = {id(p): g for g in optimizer.param_groups for p in g["params"]}
    hooks: list = []
    _register_plain_hooks(model, optimizer, hooks, pre_step, param_to_group)
    optimizer._gradient_release = True
    return GradientReleaseHandle(_hooks=hooks, _optimizer=optimizer)
