"""FlashLion (interface of ``/root/reference/flashoptim/optimizers.py:1209-1342``, cited ``ref:``)."""

from __future__ import annotations

from collections.abc import Iterable
from typing import Any, Literal, Optional

import torch

from .base import FlashOptimizer
from .state import QuantizedTensorSpec


class FlashLion(FlashOptimizer):
    """Lion with decoupled weight decay: ``p *= 1 - wd*lr; p -= lr * sign(lerp(m, g, 1-beta1));
    m = lerp(m, g, 1-beta2)``.

    Args:
        params: parameters or param-group dicts.
        lr: learning rate (default 1e-3).
        betas: ``beta1`` interpolates the update, ``beta2`` is the momentum decay (default (0.9, 0.99)).
        weight_decay: decoupled decay coefficient (default 0).
        decouple_lr: scale the decay by ``lr / initial_lr`` instead of ``lr`` (default False).
        quantize, compress_state_dict, master_weight_bits, check_numerics, fused: see :class:`FlashOptimizer`.
    """

    def __init__(
        self,
        params: Iterable[torch.Tensor],
        lr: float = 1e-3,
        betas: tuple[float, float] = (0.9, 0.99),
        weight_decay: float = 0,
        decouple_lr: bool = False,
        quantize: bool = True,
        compress_state_dict: bool = False,
        master_weight_bits: Literal[24, 32] | None = 24,
        check_numerics: bool = False,
        fused: bool = True,
    ):
        for i, beta in enumerate(betas[:2]):
            if not 0.0 <= beta <= 1.0:
                raise ValueError(f"Invalid beta parameter at index {i}: {beta}")
        if not 0.0 <= weight_decay:
            raise ValueError(f"Invalid weight_decay value: {weight_decay}")
        self._decouple_lr = decouple_lr
        super().__init__(
            params=params, lr=lr, defaults={"betas": betas, "weight_decay": weight_decay}, quantize=quantize,
            compress_state_dict=compress_state_dict, master_weight_bits=master_weight_bits,
            check_numerics=check_numerics, fused=fused,
        )

    def _quantized_state_spec(self) -> dict[str, QuantizedTensorSpec]:
        return {"exp_avg": QuantizedTensorSpec(signed=True)}

    def _kernel_kind(self, hparams: dict[str, Any]) -> str:
        return "momentum"

    def _moment_names(self, kind: str) -> tuple[Optional[str], Optional[str]]:
        return "exp_avg", None

    def _kernel_scalars(self, hparams: dict[str, Any], step: Optional[int]) -> dict[str, Any]:
        lr = float(hparams["lr"])  # schedulers may hand over numpy or 0-dim tensor values
        weight_decay = hparams["weight_decay"]  # ref:1290-1294
        weight_decay *= (lr / hparams["initial_lr"]) if self._decouple_lr else lr
        # the kernel's momentum decay is beta2, its update interpolation beta1 (ref:1313-1317)
        return dict(lr=lr, mom_coef=hparams["betas"][1], update_coef=hparams["betas"][0], weight_decay=weight_decay,
                    decoupled=False, nesterov=False, do_lion=True)
