"""FlashAdam / FlashAdamW (interface of ``/root/reference/flashoptim/optimizers.py:1784-2032``, cited ``ref:``)."""

from __future__ import annotations

import os
from collections.abc import Iterable
from typing import Any, Literal, Optional

import torch

from .base import FlashOptimizer
from .state import QuantizedTensorSpec


class FlashAdam(FlashOptimizer):
    """Adam with L2 regularisation folded into the gradient, like ``torch.optim.Adam``.

    Args:
        params: parameters or param-group dicts.
        lr: learning rate (default 1e-3).
        betas: decay rates of the first and second moment (default (0.9, 0.999)).
        eps: added to the denominator (default 1e-8).
        weight_decay: L2 coefficient (default 0).
        quantize, compress_state_dict, master_weight_bits, check_numerics, fused: see :class:`FlashOptimizer`.
        exact_update: keyword-only, not in the reference (default: the ``FLASHOPTIM_EXACT_ADAM`` environment variable,
            else False).  Evaluate the update operation by operation as the reference writes it on every element of
            every variant: all outputs then equal an IEEE evaluation of the reference's formulas bit for bit.  With
            False that already holds for fp32 parameters, 32-bit masters and fp16 parameters with 24-bit masters;
            bf16 parameters with 24-bit masters and 2-byte parameters without master-weight correction fold the
            bias corrections and the learning rate into two constants and redo operation by operation only the
            elements whose update all but cancels the weight: moment codes and scales stay bit-identical, every
            master weight stays within one unit of master precision (the correction code may differ by one step).
    """

    def __init__(
        self,
        params: Iterable[torch.Tensor],
        lr: float = 1e-3,
        betas: tuple[float, float] = (0.9, 0.999),
        eps: float = 1e-8,
        weight_decay: float = 0.0,
        quantize: bool = True,
        compress_state_dict: bool = False,
        master_weight_bits: Literal[24, 32] | None = 24,
        check_numerics: bool = False,
        fused: bool = True,
        *,
        exact_update: Optional[bool] = None,
    ):
        if not 0.0 <= eps:
            raise ValueError(f"Invalid epsilon value: {eps}")
        for i, beta in enumerate(betas[:2]):
            if not 0.0 <= beta <= 1.0:
                raise ValueError(f"Invalid beta parameter at index {i}: {beta}")
        if not 0.0 <= weight_decay:
            raise ValueError(f"Invalid weight_decay value: {weight_decay}")
        self._decoupled = False
        self._decouple_lr = False
        if exact_update is None:
            exact_update = os.environ.get("FLASHOPTIM_EXACT_ADAM", "0").strip().lower() not in ("", "0", "false", "no")
        self._exact_update = bool(exact_update)
        super().__init__(
            params=params, lr=lr, defaults={"betas": betas, "weight_decay": weight_decay, "eps": eps},
            quantize=quantize, compress_state_dict=compress_state_dict, master_weight_bits=master_weight_bits,
            check_numerics=check_numerics, fused=fused,
        )

    def _quantized_state_spec(self) -> dict[str, QuantizedTensorSpec]:
        return {
            "exp_avg": QuantizedTensorSpec(signed=True, softsign=True),                    # int8, softsign
            "exp_avg_sq": QuantizedTensorSpec(signed=False, sqrt=True, softsign=False),    # uint8 of sqrt(v)
        }

    def _ensure_state_initialized(self, p: torch.Tensor, hparams: dict[str, Any]) -> None:
        super()._ensure_state_initialized(p, hparams)
        state = self.state[p]
        if "step" not in state:
            # a CPU fp32 scalar like torch's own optimizers checkpoint it; reading it never syncs the device
            state["step"] = torch.tensor(0, dtype=torch.float32, device="cpu")

    # the kernels take the step number by value (ref:2368-2369): a replayed graph would repeat one step's bias
    # correction while the CPU counters stand still
    _step_number_by_value = True

    def _min_step_size_relative_to_lr(self) -> float:
        # |m| / sqrt(v) has no positive lower bound; assume updates routinely shrink to a tenth of lr
        return 0.1

    def _kernel_kind(self, hparams: dict[str, Any]) -> str:
        return "adam"

    def _moment_names(self, kind: str) -> tuple[Optional[str], Optional[str]]:
        return "exp_avg", "exp_avg_sq"

    def _advance_step(self, param_state: dict[str, Any]) -> Optional[int]:
        param_state["step"] += 1
        return int(param_state["step"].item())

    def _kernel_scalars(self, hparams: dict[str, Any], step: Optional[int]) -> dict[str, Any]:
        lr = float(hparams["lr"])  # schedulers may hand over numpy or 0-dim tensor values
        weight_decay = hparams["weight_decay"]
        if self._decoupled:  # the kernel multiplies the weights by 1 - weight_decay (ref:1894-1898)
            weight_decay *= (lr / hparams["initial_lr"]) if self._decouple_lr else lr
        return dict(lr=lr, beta1=hparams["betas"][0], beta2=hparams["betas"][1], eps=hparams["eps"],
                    weight_decay=weight_decay, decoupled=self._decoupled, step=step, exact_update=self._exact_update)


class FlashAdamW(FlashAdam):
    """AdamW: the decay multiplies the weights by ``1 - weight_decay * lr`` (``lr / initial_lr`` with
    ``decouple_lr=True``) instead of entering the gradient.

    Args:
        weight_decay: decoupled decay coefficient (default 1e-2).
        decouple_lr: scale the decay by ``lr / initial_lr`` instead of ``lr`` (default False).
        Other arguments as :class:`FlashAdam`.
    """

    def __init__(
        self,
        params: Iterable[torch.Tensor],
        lr: float = 1e-3,
        betas: tuple[float, float] = (0.9, 0.999),
        eps: float = 1e-8,
        weight_decay: float = 1e-2,
        decouple_lr: bool = False,
        quantize: bool = True,
        compress_state_dict: bool = False,
        master_weight_bits: Optional[Literal[24, 32]] = 24,
        check_numerics: bool = False,
        fused: bool = True,
        *,
        exact_update: Optional[bool] = None,
    ):
        super().__init__(
            params, lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, quantize=quantize,
            compress_state_dict=compress_state_dict, master_weight_bits=master_weight_bits,
            check_numerics=check_numerics, fused=fused, exact_update=exact_update,
        )
        self._decoupled = True
        self._decouple_lr = decouple_lr
