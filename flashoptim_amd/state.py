"""Optimizer-state container: 8-bit group-quantised codes + fp16 scales, or a plain tensor.

Mirrors the interface of the reference's ``_MaybeQuantizedTensor`` / ``QuantizedTensorSpec``
(``/root/reference/flashoptim/optimizers.py:70-82, 103-285``, cited as ``ref:``) including the state-dict key
names, so checkpoints are interchangeable.  Quantisation and dequantisation are HIP kernels
(:mod:`flashoptim_amd.kernels`).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from .kernels import dequantize, quantize

QUANTIZED_SUFFIX = "::quantized"
SCALES_SUFFIX = "::scales"


@dataclass(frozen=True)
class QuantizedTensorSpec:
    """How one optimizer state is companded before 8-bit quantisation (ref:70-82)."""

    signed: bool = True
    sqrt: bool = False
    softsign: bool = True

    def __post_init__(self) -> None:
        for name in ("signed", "sqrt", "softsign"):
            value = getattr(self, name)
            if not isinstance(value, bool):
                raise ValueError(f"{name} must be bool; got {type(value)}")


class _MaybeQuantizedTensor:
    """One optimizer state of one parameter.

    ``try_quantize=True``: holds ``quantized`` (int8 when signed, uint8 otherwise; parameter shape) and
    ``scales`` (fp16, one per 32 elements).  ``try_quantize=False``: holds ``data`` at ``storage_dtype``.
    """

    def __init__(
        self,
        data: Optional[torch.Tensor],
        try_quantize: bool = True,
        signed: bool = True,
        sqrt: bool = False,
        softsign: bool = True,
        storage_dtype: torch.dtype = torch.float32,
    ):
        self._data: Optional[torch.Tensor] = None
        self._quantized: Optional[torch.Tensor] = None
        self._scales: Optional[torch.Tensor] = None
        # quantisation silently switches off when there is no GPU at all (ref:127)
        self._try_quantize = bool(try_quantize) and torch.cuda.is_available()
        self._signed = signed
        self._sqrt = sqrt
        self._softsign = softsign
        self._storage_dtype = storage_dtype
        if data is not None:
            self.set_data(data)

    # -- accessors ---------------------------------------------------------------------------------
    @property
    def data(self) -> torch.Tensor:
        assert self._data is not None
        return self._data

    @property
    def quantized(self) -> torch.Tensor:
        assert self._quantized is not None
        return self._quantized

    @property
    def scales(self) -> torch.Tensor:
        assert self._scales is not None
        return self._scales

    def is_quantized(self) -> bool:
        return self._data is None

    @property
    def is_cuda(self) -> bool:
        return (self.quantized if self.is_quantized() else self.data).is_cuda

    @property
    def shape(self) -> tuple[int, ...]:
        return tuple((self.quantized if self.is_quantized() else self.data).shape)

    def numel(self) -> int:
        return (self.quantized if self.is_quantized() else self.data).numel()

    def __repr__(self) -> str:
        return f"{type(self).__name__} quantized={self.is_quantized()} signed={self._signed} shape={self.shape}"

    @property
    def kernel_tensor(self) -> torch.Tensor:
        """What the step kernels read and write: the codes, or the plain tensor (ref:265-273)."""
        return self.quantized if self.is_quantized() else self.data

    @property
    def kernel_scales_or_self(self) -> torch.Tensor:
        """The fp16 scales, or the plain tensor as a stand-in the kernels ignore (ref:275-285)."""
        return self.scales if self.is_quantized() else self.kernel_tensor

    # -- value in / out ----------------------------------------------------------------------------
    def set_data(self, data: torch.Tensor) -> None:
        if self._try_quantize:
            if not data.is_cuda:
                raise NotImplementedError(
                    f"Attempting to quantize a non-CUDA {data.dtype} tensor on device {data.device} with shape "
                    f"{tuple(data.shape)}."
                )
            self._data = None
            self._quantized, self._scales = quantize(
                data, signed=self._signed, sqrt=self._sqrt, softsign=self._softsign
            )
        else:
            self._data = data.to(dtype=self._storage_dtype).contiguous()  # the kernels index it flat
            self._quantized = None
            self._scales = None

    @classmethod
    def zeros_like(cls, ref: torch.Tensor, try_quantize: bool = True, signed: bool = True, sqrt: bool = False,
                   softsign: bool = True, storage_dtype: torch.dtype = torch.float32) -> "_MaybeQuantizedTensor":
        """An all-zero state shaped like `ref`, without the temporary tensor and the quantise launch of
        ``set_data(zeros_like(ref))``.  Quantising zeros gives codes 0 and scales fp16(1e-12) = 0 (ref:1006-1013,
        2657-2676), so both forms hold the same bits."""
        self = cls(None, try_quantize=try_quantize, signed=signed, sqrt=sqrt, softsign=softsign, storage_dtype=storage_dtype)
        if self._try_quantize:
            if not ref.is_cuda:
                raise NotImplementedError(
                    f"Attempting to quantize a non-CUDA {ref.dtype} tensor on device {ref.device} with shape "
                    f"{tuple(ref.shape)}."
                )
            self._quantized = torch.zeros(ref.shape, dtype=torch.int8 if signed else torch.uint8, device=ref.device)
            self._scales = torch.zeros((ref.numel() + 31) // 32, dtype=torch.float16, device=ref.device)
        else:
            self._data = torch.zeros(ref.shape, dtype=storage_dtype, device=ref.device)
        return self

    def materialize(self) -> torch.Tensor:
        """The state as a float tensor: fp32 after dequantisation, or the plain tensor itself."""
        if not self.is_quantized():
            return self.data
        return dequantize(self.quantized, self.scales, signed=self._signed, sqrt=self._sqrt, softsign=self._softsign)

    # -- (de)serialisation -------------------------------------------------------------------------
    @staticmethod
    def _quantized_vals_key(name: str) -> str:
        return name + QUANTIZED_SUFFIX

    @staticmethod
    def _quantized_scales_key(name: str) -> str:
        return name + SCALES_SUFFIX

    def state_dict(self, name: str, allow_quantized: bool = False) -> dict[str, torch.Tensor]:
        """``{name::quantized, name::scales}`` for a compressed checkpoint, else ``{name: bf16 tensor}`` which a
        stock torch optimizer can load (ref:159-167)."""
        if allow_quantized and self.is_quantized():
            return {self._quantized_vals_key(name): self.quantized, self._quantized_scales_key(name): self.scales}
        return {name: self.materialize().to(dtype=torch.bfloat16)}

    def load_state_dict(self, d: dict[str, torch.Tensor], name: str) -> None:
        """Accepts the whole per-parameter state dict; only ``name`` and ``name::*`` are looked at (ref:191-210)."""
        mine = {k: v for k, v in d.items() if k == name or k.startswith(name + "::")}
        if name in mine:
            if len(mine) != 1:
                raise ValueError(
                    f"If state dict specifies {name}, it must not specify other keys. Got {list(mine.keys())}"
                )
            self.set_data(mine[name])
            return
        # torch.optim.Optimizer.load_state_dict has cast both tensors to the parameter dtype on the way in
        self._data = None
        codes = mine[self._quantized_vals_key(name)].to(dtype=torch.int8 if self._signed else torch.uint8)
        self._quantized = codes.contiguous()
        self._scales = mine[self._quantized_scales_key(name)].to(dtype=torch.float16).contiguous()

    @classmethod
    def from_state_dict(
        cls,
        d: dict[str, torch.Tensor],
        name: str,
        try_quantize: bool = True,
        signed: bool = True,
        sqrt: bool = False,
        softsign: bool = True,
        storage_dtype: torch.dtype = torch.float32,
    ) -> "_MaybeQuantizedTensor":
        obj = cls(None, try_quantize=try_quantize, signed=signed, sqrt=sqrt, softsign=softsign, storage_dtype=storage_dtype)
        obj.load_state_dict(d, name)
        return obj
