"""FlashSGD / FlashSGDW (interface of ``/root/reference/flashoptim/optimizers.py:1348-1511, 1722-1778``)."""

from __future__ import annotations

from collections.abc import Iterable
from typing import Any, Literal, Optional

import torch

from .base import FlashOptimizer
from .state import QuantizedTensorSpec


class FlashSGD(FlashOptimizer):
    """SGD with optional (Nesterov) momentum and L2 regularisation, like ``torch.optim.SGD`` except that the
    momentum buffer starts at zero and ``1 - dampening`` is always applied.

    Args:
        params: parameters or param-group dicts.
        lr: learning rate (default 1e-3).
        momentum: momentum factor (default 0: no state is kept).
        dampening: dampening of the gradient entering the buffer (default 0).
        weight_decay: L2 coefficient (default 0).
        nesterov: Nesterov momentum; needs ``momentum > 0`` and ``dampening == 0``.
        quantize, compress_state_dict, master_weight_bits, check_numerics, fused: see :class:`FlashOptimizer`.
    """

    def __init__(
        self,
        params: Iterable[torch.Tensor],
        lr: float = 0.001,
        momentum: float = 0.0,
        dampening: float = 0.0,
        weight_decay: float = 0.0,
        nesterov: bool = False,
        quantize: bool = True,
        compress_state_dict: bool = False,
        master_weight_bits: Literal[24, 32] | None = 24,
        check_numerics: bool = False,
        fused: bool = True,
    ):
        if nesterov and (momentum <= 0 or dampening != 0):
            raise ValueError("Nesterov momentum requires a momentum and zero dampening")
        if not 0.0 <= weight_decay:
            raise ValueError(f"Invalid weight_decay value: {weight_decay}")
        self._nesterov = nesterov
        self._decoupled = False
        self._decouple_lr = False
        super().__init__(
            params, lr=lr,
            defaults={"lr": lr, "momentum": momentum, "dampening": dampening, "weight_decay": weight_decay},
            quantize=quantize, compress_state_dict=compress_state_dict, master_weight_bits=master_weight_bits,
            check_numerics=check_numerics, fused=fused,
        )

    def _quantized_state_spec(self) -> dict[str, QuantizedTensorSpec]:
        if any(g["momentum"] > 0.0 for g in self.param_groups):
            return {"momentum_buffer": QuantizedTensorSpec(signed=True)}
        return {}

    def _kernel_kind(self, hparams: dict[str, Any]) -> str:
        # without momentum no buffer exists: the momentum-free kernel steps the weights directly (the reference
        # handles this case in eager ops, ref:1447-1465)
        return "plain" if hparams["momentum"] == 0.0 else "momentum"

    def _moment_names(self, kind: str) -> tuple[Optional[str], Optional[str]]:
        return ("momentum_buffer" if kind == "momentum" else None), None

    def _kernel_scalars(self, hparams: dict[str, Any], step: Optional[int]) -> dict[str, Any]:
        lr = float(hparams["lr"])  # schedulers may hand over numpy or 0-dim tensor values
        weight_decay = hparams["weight_decay"]
        if self._decoupled:  # ref:1438-1442
            weight_decay *= (lr / hparams["initial_lr"]) if self._decouple_lr else lr
        if hparams["momentum"] == 0.0:
            return dict(lr=lr, weight_decay=weight_decay, decoupled=self._decoupled)
        return dict(lr=lr, mom_coef=hparams["momentum"], update_coef=1.0 - hparams["dampening"],
                    weight_decay=weight_decay, decoupled=self._decoupled, nesterov=self._nesterov, do_lion=False)


class FlashSGDW(FlashSGD):
    """SGD whose decay multiplies the weights by ``1 - weight_decay * lr`` (``lr / initial_lr`` with
    ``decouple_lr=True``) instead of entering the gradient.  Arguments as :class:`FlashSGD` plus ``decouple_lr``."""

    def __init__(
        self,
        params: Iterable[torch.Tensor],
        lr: float = 0.001,
        momentum: float = 0.0,
        dampening: float = 0.0,
        weight_decay: float = 0.0,
        nesterov: bool = False,
        decouple_lr: bool = False,
        quantize: bool = True,
        compress_state_dict: bool = False,
        master_weight_bits: Optional[Literal[24, 32]] = 24,
        check_numerics: bool = False,
        fused: bool = True,
    ):
        super().__init__(
            params, lr=lr, momentum=momentum, dampening=dampening, weight_decay=weight_decay, nesterov=nesterov,
            quantize=quantize, compress_state_dict=compress_state_dict, master_weight_bits=master_weight_bits,
            check_numerics=check_numerics, fused=fused,
        )
        self._decoupled = True
        self._decouple_lr = decouple_lr
