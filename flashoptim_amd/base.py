"""``FlashOptimizer``: the ``torch.optim.Optimizer`` base class of the MI355X FlashOptim implementation.

Same constructor arguments, param-group keys, per-parameter state layout, ``state_dict`` / ``load_state_dict``
format and error behaviour as the reference base class (``/root/reference/flashoptim/optimizers.py:317-1203``,
cited as ``ref:``).  What differs is underneath: subclasses describe a param group's update as a kernel kind plus
fp32 scalars; ``step_param`` executes one parameter with a single-tensor HIP launch, ``step`` groups the
parameters into buckets and issues one multi-tensor launch per bucket, caching the per-parameter host work of a
group whose parameter list and gradient layout did not change.  There is no eager PyTorch implementation of
the update in this package.
"""

from __future__ import annotations

import abc
import math
import os
import warnings
from collections.abc import Iterable
from dataclasses import dataclass
from typing import Any, Callable, Literal, Optional, cast

import torch
import torch.nn as nn

from . import _hostscan, kernels
from .kernels import compute_ecc_bits, reconstruct_fp32_param
from .launcher import BucketPlan, StepTensors
from .state import QuantizedTensorSpec, _MaybeQuantizedTensor

_DTYPE_WIDTHS = {torch.int8: 1, torch.int16: 2, torch.float16: 2, torch.bfloat16: 2, torch.float32: 4}
_EXPONENT_BITS = {torch.float16: 5, torch.bfloat16: 8, torch.float32: 8}
_VALID_MASTER_WEIGHT_BITS = (None, 24, 32)
_BITS_TO_BYTES = {None: 0, 24: 3, 32: 4}


class NumericsError(RuntimeError):
    """The learning rate is too small to change the largest weights at their dtype and master-weight width."""


def _log2_min_expressible_step_size(dtype: torch.dtype, maxabs: float, master_bytewidth: int) -> float:
    """log2 of the smallest step that still moves a value of magnitude ``maxabs`` (ref:291-314).

    A value with exponent e has resolution 2^(e - mantissa_bits); error-correction bytes extend the mantissa;
    a step only needs 0.49 of that resolution to round to the neighbouring value.
    """
    master_bits = max(_DTYPE_WIDTHS[dtype], master_bytewidth) * 8
    mantissa_bits = master_bits - 1 - _EXPONENT_BITS[dtype] + math.log2(0.49)
    return math.floor(math.log2(maxabs)) - mantissa_bits


@dataclass(frozen=True)
class LaunchKey:
    """Everything that must be equal for two tensors to share one multi-tensor launch."""

    kind: str                 # "adam" | "momentum" | "plain"
    dtype: torch.dtype
    ecc_bytes: int
    quantized: bool
    scalars: tuple            # keyword arguments of the kernel wrapper, as a sorted tuple of items
    device: Optional[torch.device] = None   # one launch reaches one device's memory only


@dataclass
class _Bucket:
    """Cached launch state of the tensors of one param group that share a LaunchKey up to the scalars."""

    kind: str
    dtype: torch.dtype
    ecc_bytes: int
    quantized: bool
    params: list                      # the nn.Parameters, in table order
    tensors: list                     # StepTensors with grad=None (state tensors only)
    plan: Optional[BucketPlan]        # multi-tensor tables; None for single-tensor buckets
    step_pool: Optional[torch.Tensor]  # 1-D CPU fp32 tensor whose elements ARE the bucket's `step` scalars (Adam), else None
    step_value: Optional[int]
    step_views: Optional[list] = None  # the 0-dim views of step_pool that were stored as state[p]["step"] (kept alive)
    step_view_ids: Optional[list] = None  # their id()s: one list comparison per step notices a replaced counter object


@dataclass
class _GroupCache:
    epoch: int
    params: list                      # the group's parameter list when the cache was built; keeps `param_ids` unique
    param_ids: list
    signature: Any
    buckets: list
    idle: list                        # non-empty parameters that had no gradient (or are frozen) when the cache was built
    state_len: int                    # len(optimizer.state) then: a cleared or pruned state dict invalidates the cache
    # check_numerics: log2 of the coarsest weight resolution over the group's parameters (None: nothing to check)
    numerics_needed: Optional[float] = None


class FlashOptimizer(torch.optim.Optimizer, abc.ABC):
    """Base class: quantised optimizer states, compressed state dicts, fused HIP steps, ECC master weights and
    gradient release.  See the subclasses for the optimizer-specific arguments.

    Args:
        params: iterable of parameters or of param-group dicts.
        lr: learning rate.
        quantize: keep optimizer states as 8-bit codes with one fp16 scale per 32 elements (~8.5 bits/param).
        compress_state_dict: emit the quantised states in ``state_dict()`` instead of bf16 tensors.
        master_weight_bits: 24 or 32 adds an int8 / int16 correction tensor next to each bf16/fp16 parameter so
            that updates accumulate at 24- / 32-bit precision; ``None`` steps the parameters at their own dtype.
        check_numerics: raise :class:`NumericsError` when ``lr`` cannot move the largest weight of a tensor.
        fused: accepted for signature compatibility.  The fused HIP kernels are the only implementation.

    Raises:
        ValueError: inconsistent or out-of-range hyper-parameters.
        NotImplementedError: no ROCm device is available, or a parameter lives on the CPU.
    """

    def __init__(
        self,
        params: Iterable[torch.Tensor],
        lr: float = 1e-3,
        quantize: bool = True,
        compress_state_dict: bool = False,
        master_weight_bits: Optional[Literal[24, 32]] = 24,
        check_numerics: bool = False,
        fused: bool = True,
        defaults: Optional[dict[str, Any]] = None,
    ):
        if compress_state_dict and not quantize:
            raise ValueError("compress_state_dict=True requires quantize=True")
        if lr < 0.0:
            raise ValueError(f"Invalid learning rate: {lr}")
        if master_weight_bits not in _VALID_MASTER_WEIGHT_BITS:
            raise ValueError(
                f"Master weight bits {master_weight_bits} invalid; must be one of {_VALID_MASTER_WEIGHT_BITS}"
            )
        master_bytewidth = _BITS_TO_BYTES[master_weight_bits]

        if not torch.cuda.is_available():
            # same exception type and order of complaints as the reference (ref:484-493); this package has no
            # CPU implementation at all, so the last case raises as well
            needs = " requires a CUDA device."
            if quantize:
                raise NotImplementedError("Quantization" + needs)
            if compress_state_dict:
                raise NotImplementedError("Quantized state dict" + needs)
            if master_weight_bits is not None:
                raise NotImplementedError("Using error correction bits" + needs)
            if fused:
                raise NotImplementedError("Fused optimizer step" + needs)
            raise NotImplementedError("flashoptim_amd" + needs + " It has no eager CPU implementation.")
        if not fused:
            warnings.warn(
                "fused=False is accepted for compatibility; flashoptim_amd always runs its fused HIP kernels.",
                stacklevel=3,
            )

        self._fused = fused  # kept off the param groups so torch leaves the CPU `step` tensors alone on load
        self._quantize = quantize
        self._master_bytewidth = master_bytewidth
        self._compress_state_dict = compress_state_dict
        self._check_numerics = check_numerics
        self._transient_state: dict[int, dict[str, Any]] = {}  # id(param) -> {"maxabs": ...}; never serialised
        self._gradient_release = False
        self._plan_epoch = 0                       # bumped whenever cached launch plans may be stale
        self._state_ready: set[int] = set()        # id(param) of parameters whose state tensors exist
        self._group_cache: dict[int, _GroupCache] = {}

        group_defaults = dict(defaults or {})
        group_defaults.update(lr=lr, initial_lr=lr, master_bytewidth=master_bytewidth, quantize=quantize)
        super().__init__(params, defaults=group_defaults)

        every_param = [p for g in self.param_groups for p in g["params"]]
        if master_weight_bits is not None and not os.environ.get("FLASHOPTIM_ALLOW_INEFFECTIVE_MASTER_WEIGHT_BITS"):
            if all(p.dtype == torch.float32 for p in every_param):
                raise ValueError(
                    f"master_weight_bits={master_weight_bits} has no effect when all parameters are fp32, since "
                    "fp32 already uses 32 bits. No error correction would be applied in this scenario. Please "
                    "omit master_weight_bits (or set it to None)."
                )
        if master_weight_bits is None and any(p.dtype != torch.float32 for p in every_param):
            warnings.warn(
                "master_weight_bits=None with non-fp32 parameters means pure low-precision training (no error "
                "correction). Optimizer states will be stored at parameter precision. This is numerically "
                "fragile, consider setting master_weight_bits=24 for stable training.",
                stacklevel=2,
            )

    def __repr__(self) -> str:
        lines = [f"{type(self).__name__} (", "FlashOptim Config"]
        for key, value in (
            ("fused", self._fused), ("quantize", self._quantize), ("master_bytewidth", self._master_bytewidth),
            ("compress_state_dict", self._compress_state_dict), ("check_numerics", self._check_numerics),
            ("gradient_release", self._gradient_release),
        ):
            lines.append(f"    {key}: {value}")
        for i, group in enumerate(self.param_groups):
            lines += ["", f"Parameter Group {i}"]
            lines += [f"    {k}: {group[k]}" for k in sorted(group) if k != "params"]
        return "\n".join(lines) + "\n)"

    # ----------------------------------------------------------------------------------- subclass hooks
    @abc.abstractmethod
    def _quantized_state_spec(self) -> dict[str, QuantizedTensorSpec]:
        """Names and companding of the quantisable states, e.g. ``{"exp_avg": ..., "exp_avg_sq": ...}``."""

    @abc.abstractmethod
    def _kernel_kind(self, hparams: dict[str, Any]) -> str:
        """"adam", "momentum" or "plain" (momentum-free SGD) for the tensors of this param group."""

    @abc.abstractmethod
    def _kernel_scalars(self, hparams: dict[str, Any], step: Optional[int]) -> dict[str, Any]:
        """The kernel's scalar arguments for this param group, folded in double like the reference's ``_do_step``
        (decoupled decay times lr, Lion's beta roles, ...)."""

    @abc.abstractmethod
    def _moment_names(self, kind: str) -> tuple[Optional[str], Optional[str]]:
        """State keys of the first and second moment used by `kind` (None where there is none)."""

    def _advance_step(self, param_state: dict[str, Any]) -> Optional[int]:
        """Optimizers with bias correction advance and return their per-parameter step counter here."""
        del param_state
        return None

    def _plan_signature(self, hparams: dict[str, Any]) -> Any:
        """Whatever besides the parameter list decides which kernel a group uses; a change invalidates caches."""
        return self._kernel_kind(hparams)

    def _initial_value_for_state_var(self, param: torch.Tensor, key: str) -> torch.Tensor:
        del key
        return torch.zeros_like(param)

    def _min_step_size_relative_to_lr(self) -> float:
        return 1.0  # sign-based updates (Lion) move every weight by exactly lr

    # True for optimizers whose kernels receive a per-parameter step number as a host value
    _step_number_by_value = False

    def _refuse_graph_capture(self) -> None:
        if self._step_number_by_value and torch.cuda.is_current_stream_capturing():
            raise RuntimeError(
                f"{type(self).__name__} cannot be stepped while a HIP graph is being recorded: its bias correction "
                "depends on the step number, which the kernels receive as a host value."
            )

    # ------------------------------------------------------------------------------ sharded-tensor shims
    @staticmethod
    def _get_tensor_for_stats(tensor: torch.Tensor) -> torch.Tensor:
        return tensor.full_tensor() if hasattr(tensor, "full_tensor") else tensor

    @staticmethod
    def _get_local_tensor(tensor: torch.Tensor) -> torch.Tensor:
        return tensor.to_local() if hasattr(tensor, "to_local") else tensor

    # ------------------------------------------------------------------------------------- numerics check
    def _recompute_stats(self, params: list) -> None:
        """Largest magnitude of every given parameter: one launch per (device, dtype) and one synchronisation per
        device, instead of the reference's ``abs().max().item()`` per tensor (ref:656-673)."""
        tensors = [self._get_tensor_for_stats(p).detach() for p in params]
        for p, maxabs in zip(params, kernels.absmax_many(tensors)):
            self._transient_state.setdefault(id(p), {})["maxabs"] = maxabs
        self._plan_epoch += 1  # cached numerics verdicts are stale

    def _recompute_stats_for_param(self, p: torch.Tensor) -> None:
        self._recompute_stats([p])

    def recompute_param_stats(self) -> None:
        """Refresh the cached largest magnitude of every parameter (used by ``check_numerics``)."""
        self._recompute_stats([p for group in self.param_groups for p in group["params"]])

    def _numerics_needed(self, p: torch.Tensor, master_bytewidth: int) -> Optional[float]:
        maxabs = self._transient_state.get(id(p), {}).get("maxabs", 0)
        if maxabs <= 0 or not math.isfinite(maxabs):
            return None
        return _log2_min_expressible_step_size(dtype=p.dtype, maxabs=maxabs, master_bytewidth=master_bytewidth)

    def _check_param_numerics(self, p: torch.Tensor, lr: float, master_bytewidth: int) -> None:
        if lr == 0.0:
            return
        maxabs = self._transient_state.get(id(p), {}).get("maxabs", 0)
        if maxabs <= 0 or not math.isfinite(maxabs):
            return
        needed = _log2_min_expressible_step_size(dtype=p.dtype, maxabs=maxabs, master_bytewidth=master_bytewidth)
        guaranteed = math.log2(lr * self._min_step_size_relative_to_lr())
        if needed > guaranteed:
            bits = max(_DTYPE_WIDTHS[p.dtype], master_bytewidth) * 8
            raise NumericsError(
                f"Learning rate {lr:.3g} yields steps that may be too small to alter the weights for dtype "
                f"{p.dtype} with master_weight_bits={bits} and weight maximum absolute value {maxabs} (min step "
                f"size {2**guaranteed:.5g} < resolution {2**needed:.5g}). Consider increasing your learning rate, "
                "decreasing your weight magnitudes, or increasing master_weight_bits. Set check_numerics=False to "
                "disable this check. If you're getting this error after loading a checkpoint, you can call "
                "recompute_param_stats() throughout training to fail faster and avoid this surprise."
            )

    # --------------------------------------------------------------------------------- per-parameter plan
    def _ensure_state_initialized(self, p: torch.Tensor, hparams: dict[str, Any]) -> None:
        if self._check_numerics and self._transient_state.get(id(p), {}).get("maxabs") is None:
            self._recompute_stats_for_param(p)
        state = self.state[p]
        local = self._get_local_tensor(p)
        quantize = hparams.get("quantize", self._quantize)
        for key, spec in self._quantized_state_spec().items():
            if key not in state:
                kw = dict(try_quantize=quantize, signed=spec.signed, sqrt=spec.sqrt, softsign=spec.softsign,
                          storage_dtype=local.dtype)
                if type(self)._initial_value_for_state_var is FlashOptimizer._initial_value_for_state_var:
                    state[key] = _MaybeQuantizedTensor.zeros_like(local, **kw)  # zero start: nothing to quantise
                else:
                    state[key] = _MaybeQuantizedTensor(self._initial_value_for_state_var(local, key), **kw)
        extra_bytes = hparams["master_bytewidth"] - _DTYPE_WIDTHS[p.dtype]
        if extra_bytes > 0 and state.get("error_bits") is None:
            state["error_bits"] = torch.zeros_like(local, dtype=torch.int8 if extra_bytes == 1 else torch.int16)

    def _find_group(self, p: torch.Tensor) -> dict[str, Any]:
        for group in self.param_groups:
            if any(q is p for q in group["params"]):
                return group
        raise ValueError(f"Parameter {p.shape} {p.dtype} not managed by this optimizer.")

    def _plan_step(
        self,
        param: torch.Tensor,
        grad: torch.Tensor,
        errors: Optional[torch.Tensor],
        param_state: dict[str, Any],
        hparams: dict[str, Any],
    ) -> tuple[LaunchKey, StepTensors]:
        """Host-side part of one parameter's step: advance counters, fold the hyper-parameters into the kernel
        scalars and name the tensors."""
        if errors is not None and errors.dtype not in (torch.int8, torch.int16):
            raise ValueError("Errors needs to be int8 or int16")
        kind = self._kernel_kind(hparams)
        scalars = self._kernel_scalars(hparams, self._advance_step(param_state))
        mom_name, var_name = self._moment_names(kind)
        mom = param_state[mom_name] if mom_name else None
        var = param_state[var_name] if var_name else None
        key = LaunchKey(kind, param.dtype, 0 if errors is None else errors.element_size(),
                        mom.is_quantized() if mom is not None else False, tuple(sorted(scalars.items())), param.device)
        tensors = StepTensors(
            param=param, grad=grad, ecc=errors,
            mom=None if mom is None else mom.kernel_tensor,
            mom_scales=None if mom is None else mom.kernel_scales_or_self,
            var=None if var is None else var.kernel_tensor,
            var_scales=None if var is None else var.kernel_scales_or_self,
        )
        return key, tensors

    def _plan_param(self, p: torch.Tensor, group: dict[str, Any]) -> Optional[tuple[LaunchKey, StepTensors]]:
        """Everything ``step_param`` does short of launching (ref:699-759)."""
        if id(p) not in self._state_ready or not self.state.get(p):
            self._ensure_state_initialized(p, hparams=group)
            self._state_ready.add(id(p))
        param_state = self.state[p]
        if p.numel() < 1:
            return None  # state exists (checkpoint logic wants it) but there is nothing to update
        if not p.requires_grad or p.grad is None:
            return None
        if self._check_numerics:
            self._check_param_numerics(p, lr=group["lr"], master_bytewidth=group["master_bytewidth"])
        p_local = self._get_local_tensor(p)
        grad_local = self._get_local_tensor(p.grad)
        if not p_local.is_cuda:
            raise NotImplementedError(
                f"FlashOptimizer steps parameters on a ROCm GPU only; got a parameter on {p_local.device}."
            )
        if not p_local.is_contiguous():
            raise RuntimeError(
                f"FlashOptimizer fused kernels require contiguous parameters, but got param with shape "
                f"{p_local.shape} and stride {p_local.stride()}. Call .contiguous() on the parameter or use "
                "fused=False."
            )
        if not grad_local.is_contiguous():
            raise RuntimeError(
                f"FlashOptimizer fused kernels require contiguous gradients, but got grad with shape "
                f"{grad_local.shape} and stride {grad_local.stride()}. Use fused=False for non-contiguous gradients."
            )
        return self._plan_step(p_local, grad_local, param_state.get("error_bits"), param_state, group)

    @staticmethod
    def _launch_single(key: LaunchKey, t: StepTensors) -> None:
        kw = dict(key.scalars)
        if key.kind == "adam":
            kernels._fused_adam_step(t.mom, t.mom_scales, t.var, t.var_scales, t.param, t.grad, t.ecc,
                                     quantize_optim_states=key.quantized, **kw)
        elif key.kind == "momentum":
            kernels._fused_momentum_step(t.mom, t.mom_scales, t.param, t.grad, t.ecc,
                                         quantize_optim_states=key.quantized, **kw)
        else:
            kernels._sgd_plain_step(t.param, t.grad, t.ecc, **kw)

    @torch.no_grad()
    def step_param(self, p: torch.Tensor, group: Optional[dict[str, Any]] = None) -> None:
        """Step one parameter now (its ``.grad`` must be set).  Entry point of the gradient-release hooks.

        Raises:
            RuntimeError: the parameter or its gradient is not contiguous.
            NumericsError: ``check_numerics=True`` and the learning rate cannot move the weights.
        """
        if group is None:
            group = self._find_group(p)
        self._refuse_graph_capture()
        self._plan_epoch += 1  # counters move outside step(): cached bucket state is stale
        plan = self._plan_param(p, group)
        if plan is not None:
            self._launch_single(*plan)

    # -- step(): one multi-tensor launch per bucket, with the host work of an unchanged group cached ------------
    def _step_group_slow(self, index: int, group: dict[str, Any]) -> None:
        """Full per-parameter planning (state creation, checks, counters), then one launch per bucket; leaves a
        cache behind that stays valid while the same parameters have gradients (frozen or unused ones sit out)."""
        if torch.cuda.is_current_stream_capturing() and self._group_cache.get(index) is not None:
            # a cached group fell back to full planning (a parameter, gradient layout or hyper-parameter changed):
            # that builds new launch tables, which a HIP graph cannot record
            raise RuntimeError(
                "step() has to re-plan its launches (a gradient is missing or has a new layout, a parameter was "
                "replaced, or a counter was rewritten), which cannot be recorded into a HIP graph. Run one step "
                "outside the capture with the tensors the graph will use, then capture.")
        planned: dict[LaunchKey, list] = {}
        cacheable = True
        idle = []
        if self._check_numerics:  # one scan for every parameter that has no cached statistic yet
            missing = [p for p in group["params"]
                       if p.grad is not None and self._transient_state.get(id(p), {}).get("maxabs") is None]
            if missing:
                self._recompute_stats(missing)
        for p in group["params"]:
            plan = self._plan_param(p, group)
            if plan is None:
                if p.numel() > 0:
                    idle.append(p)
                continue
            key, tensors = plan
            planned.setdefault(key, []).append((p, tensors))
            if tensors.param is not p:
                cacheable = False  # sharded wrapper: keep the generic path
        buckets = []
        for key, items in planned.items():
            tensors = [t for _, t in items]
            scalars = dict(key.scalars)
            plan = None
            if len(tensors) > 1:
                plan = BucketPlan(key.kind, key.dtype, key.ecc_bytes, key.quantized, tensors)
                plan.launch(**scalars)
            else:
                for t in tensors:
                    self._launch_single(key, t)
            step_pool, step_views = None, None
            if "step" in scalars:
                # the per-parameter CPU `step` scalars become 0-dim views into one tensor, so that the cached path
                # advances all of them with a single in-place add (one add per scalar costs 1.3 us each)
                step_pool = torch.stack([self.state[p]["step"].detach().reshape(()) for p, _ in items])
                step_views = [step_pool[i] for i in range(len(items))]
                for view, (p, _) in zip(step_views, items):
                    self.state[p]["step"] = view
            for t in tensors:
                t.grad = None  # the cache must not keep gradients alive
            buckets.append(_Bucket(key.kind, key.dtype, key.ecc_bytes, key.quantized, [p for p, _ in items], tensors,
                                   plan, step_pool, scalars.get("step"), step_views,
                                   None if step_views is None else list(map(id, step_views))))
        if cacheable and buckets:
            needed = None
            if self._check_numerics:
                each = [self._numerics_needed(p, group["master_bytewidth"]) for b in buckets for p in b.params]
                needed = max((x for x in each if x is not None), default=None)
            self._group_cache[index] = _GroupCache(self._plan_epoch, list(group["params"]), list(map(id, group["params"])),
                                                   self._plan_signature(group), buckets, idle, len(self.state), needed)
        else:
            self._group_cache.pop(index, None)

    def _step_group_fast(self, cache: _GroupCache, group: dict[str, Any]) -> bool:
        """Re-issue the cached launches of a group whose parameters have gradients of the cached layout (and whose
        idle parameters still have none).  Returns False (having changed nothing) when the group must go through
        the full path instead."""
        for p in cache.idle:
            if p.grad is not None and p.requires_grad:
                return False
        moved = []
        for b in cache.buckets:
            if b.step_pool is not None:
                # the counters are live state the caller may have rewritten (a warm restart zeroes them): take the
                # step number from them, and leave counters that no longer agree to the per-parameter path.  A
                # counter OBJECT that was replaced (state[p]["step"] = tensor(0.)) no longer aliases the pool.
                state = self.state
                if [id(state[p].get("step")) for p in b.params] != b.step_view_ids:
                    return False
                lo, hi = torch.aminmax(b.step_pool)
                lo = lo.item()
                if lo != hi.item():
                    return False
                b.step_value = int(lo)
            if b.plan is None:  # single-tensor bucket: launched from the live tensors below
                for p in b.params:
                    g = p.grad
                    if (g is None or not p.requires_grad or g.dtype != b.dtype or g.device != p.device
                            or not g.is_contiguous()):
                        return False
                continue
            plan, i = b.plan, 0
            if _hostscan.scan is not None:
                # the same walk in one C++ loop over the tensor objects (flashoptim_amd/hostscan)
                found = _hostscan.scan(b.params, plan.table_address, plan.n_tensors)
                if found is None:
                    return False
                moved.extend((plan, j, ptr) for j, ptr in found)
                continue
            for p, grad_ptr, param_ptr in zip(b.params, plan.grad_ptrs, plan.param_ptrs):
                g = p.grad
                if g is None or not p.requires_grad:
                    return False
                if p.data_ptr() != param_ptr:
                    return False  # the parameter's storage was replaced (p.data = ..., module.to(...))
                ptr = g.data_ptr()
                if ptr != grad_ptr:
                    if g.dtype != b.dtype or g.device != p.device or not g.is_contiguous() or g.numel() != p.numel():
                        return False
                    moved.append((plan, i, ptr))
                i += 1
        for plan, i, ptr in moved:
            plan.set_grad_ptr(i, ptr)
        for b in cache.buckets:
            if b.step_pool is not None:
                b.step_pool.add_(1)
                b.step_value += 1
            scalars = self._kernel_scalars(group, b.step_value)
            if b.plan is not None:
                b.plan.launch(**scalars)
            else:
                key = LaunchKey(b.kind, b.dtype, b.ecc_bytes, b.quantized, tuple(sorted(scalars.items())))
                for p, t in zip(b.params, b.tensors):
                    t.grad = p.grad
                    self._launch_single(key, t)
                    t.grad = None
        return True

    def _cached_numerics_ok(self, cache: _GroupCache, group: dict[str, Any]) -> bool:
        """check_numerics for a cached group: the weights' resolution is cached, only lr can have moved.  False
        sends the group through the full path, which raises the NumericsError naming the parameter."""
        if not self._check_numerics or cache.numerics_needed is None or group["lr"] == 0.0:
            return True
        return cache.numerics_needed <= math.log2(group["lr"] * self._min_step_size_relative_to_lr())

    @torch.no_grad()
    def step(self, closure: Optional[Callable] = None) -> Optional[torch.Tensor]:
        if self._gradient_release:
            warnings.warn(
                "optimizer.step() is a no-op while enable_gradient_release() is active — parameters are stepped "
                "by gradient hooks.",
                stacklevel=2,
            )
            return None
        self._refuse_graph_capture()
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for index, group in enumerate(self.param_groups):
            cache = self._group_cache.get(index)
            if (
                cache is not None
                and cache.epoch == self._plan_epoch
                and cache.state_len == len(self.state)
                and self._cached_numerics_ok(cache, group)
                and (_hostscan.same_objects(cache.params, group["params"]) if _hostscan.same_objects is not None
                     and type(group["params"]) is list else cache.param_ids == list(map(id, group["params"])))
                and cache.signature == self._plan_signature(group)
                and self._step_group_fast(cache, group)
            ):
                continue
            self._step_group_slow(index, group)
        return loss

    def zero_grad(self, set_to_none: bool = True) -> None:
        if self._gradient_release:
            warnings.warn(
                "optimizer.zero_grad() is a no-op while enable_gradient_release() is active — gradients are freed "
                "by gradient hooks.",
                stacklevel=2,
            )
            return
        super().zero_grad(set_to_none=set_to_none)

    def add_param_group(self, param_group: dict[str, Any]) -> None:
        super().add_param_group(param_group)
        if hasattr(self, "_plan_epoch"):
            self._plan_epoch += 1

    # ------------------------------------------------------------------------------------ (de)serialisation
    def _state_dict_for_param(self, param_number: int, opt_state: dict[int, Any], hparams: dict[str, Any],
                              idx_to_param: dict[int, torch.Tensor]) -> dict[str, Any]:
        """Per-parameter view written to a checkpoint (ref:868-927): quantised states become either their
        codes+scales or a bf16 tensor, and ``error_bits`` is disguised as a tensor of the parameter dtype so
        that ``Optimizer.load_state_dict``'s cast to the parameter dtype is lossless."""
        out = dict(opt_state[param_number])  # shallow copy: self.state must not change
        if isinstance(out.get("step"), torch.Tensor):
            out["step"] = out["step"].clone()  # live counters may be views into a shared pool
        for name in self._quantized_state_spec():
            if name in out:
                holder = out.pop(name)
                assert isinstance(holder, _MaybeQuantizedTensor)
                out.update(holder.state_dict(name=name, allow_quantized=self._compress_state_dict))
        if "error_bits" in out:
            param_dtype = idx_to_param[param_number].dtype
            param_width = _DTYPE_WIDTHS[param_dtype]
            ecc_width = hparams["master_bytewidth"] - param_width
            errs = out["error_bits"]
            if ecc_width == param_width:
                out["error_bits"] = errs.view(dtype=param_dtype)          # same width: reinterpret the bits
            elif ecc_width == 1 and param_width == 2:
                out["error_bits"] = errs.to(dtype=param_dtype)            # int8 -> bf16/fp16 values, exact
            else:
                raise NotImplementedError(
                    f"Cannot save {ecc_width}B error correction tensor for {param_width}B parameter. Non-scalar "
                    "optimizer states must keep the parameter's shape while optim.Optimizer casts them to the "
                    "parameter dtype on load; this combination cannot survive both."
                )
        return out

    def state_dict(self):
        d = super().state_dict()
        idx_to_param: dict[int, torch.Tensor] = {}
        for live, saved in zip(self.param_groups, d["param_groups"]):
            idx_to_param.update(zip(saved["params"], live["params"]))
        state = d["state"]
        for group in d["param_groups"]:
            for idx in group["params"]:
                # torch only lists parameters that already have state
                if idx in state:
                    state[idx] = self._state_dict_for_param(idx, state, group, idx_to_param)
        return d

    def _load_state_for_param(self, param: torch.Tensor, opt_state: dict[torch.Tensor, Any],
                              hparams: dict[str, Any]) -> dict[str, Any]:
        """Inverse of :meth:`_state_dict_for_param` on the already dtype-cast tensors (ref:797-866)."""
        saved = opt_state[param]
        spec = self._quantized_state_spec()
        restored = {k: v for k, v in saved.items() if not any(k == q or k.startswith(q + "::") for q in spec)}
        quantize = hparams.get("quantize", self._quantize)
        for name, s in spec.items():
            if any(k.startswith(name) for k in saved):
                restored[name] = _MaybeQuantizedTensor.from_state_dict(
                    saved, name=name, try_quantize=quantize, signed=s.signed, sqrt=s.sqrt, softsign=s.softsign,
                    storage_dtype=param.dtype,
                )
        master_bytewidth = hparams.get("master_bytewidth")
        if master_bytewidth is None:
            return restored  # the checkpoint was not written by a Flash optimizer: no ECC to restore
        errs = saved.get("error_bits")
        if errs is None:
            return restored
        param_width = _DTYPE_WIDTHS[param.dtype]
        ecc_width = int(master_bytewidth) - param_width
        seen_dtype = errs.dtype
        if ecc_width == 1 and errs.dtype != torch.int8:
            errs = errs.to(dtype=torch.int8)
        elif ecc_width == 2 and errs.dtype != torch.int16:
            errs = errs.view(dtype=torch.int16)
        if param_width + _DTYPE_WIDTHS[errs.dtype] != int(master_bytewidth):
            raise ValueError(
                f"Loading errors of dtype {seen_dtype} for param of dtype {param.dtype} cannot yield "
                f"master_weight_bits={int(master_bytewidth) * 8}."
            )
        restored["error_bits"] = errs
        return restored

    def __getstate__(self) -> dict[str, Any]:
        """For ``copy.deepcopy`` / ``pickle`` of the optimizer object itself: torch keeps ``defaults``, ``state`` and
        ``param_groups``; the scalar configuration of this class and its subclasses travels along."""
        state = super().__getstate__()
        state["_flash_config"] = {k: v for k, v in self.__dict__.items()
                                  if k.startswith("_") and isinstance(v, (bool, int, float, str, type(None)))}
        return state

    def __setstate__(self, state: dict[str, Any]) -> None:
        if "_flash_config" in state:
            # a copied / unpickled optimizer: its states are live containers already, nothing to convert; hooks of
            # the original are not copied, launch caches and statistics are keyed by object identity
            state = dict(state)
            config = state.pop("_flash_config")
            super().__setstate__(state)
            self.__dict__.update(config)
            self._gradient_release = False
            self._plan_epoch = int(config.get("_plan_epoch", 0)) + 1
            self._group_cache = {}
            self._transient_state = {}
            self._state_ready = set()
            return
        opt_state = cast(dict[torch.Tensor, Any], state["state"])
        for group in cast(list[dict[str, Any]], state["param_groups"]):
            for param in group["params"]:
                per_param = opt_state[param]
                for k, v in per_param.items():
                    if isinstance(v, torch.Tensor):
                        per_param[k] = self._get_local_tensor(v)
                opt_state[param] = self._load_state_for_param(param, opt_state, hparams=group)
            # after the per-parameter pass, so that a master_bytewidth found there is known to come from the file
            group.setdefault("master_bytewidth", self._master_bytewidth)
        super().__setstate__(state)
        # state tensors were replaced: cached pointer tables and step counters are stale
        self._plan_epoch = getattr(self, "_plan_epoch", 0) + 1
        self._group_cache = {}
        self._state_ready = set()

    def load_state_dict(self, state_dict: dict[str, Any]) -> None:
        """Also accepts checkpoints of the stock torch optimizers, which may lack ``initial_lr`` (ref:974-986)."""
        super().load_state_dict(state_dict)
        for group in self.param_groups:
            group.setdefault("initial_lr", group["lr"])

    # ------------------------------------------------------------------------------- fp32 export / import
    def get_fp32_model_state_dict(self, model: nn.Module) -> dict[str, torch.Tensor]:
        """The model's state dict in fp32, with ECC-corrected master weights where available (ref:1035-1084)."""
        module = cast(nn.Module, model.module if hasattr(model, "module") else model)
        out = {k: v.detach().float() for k, v in module.state_dict().items()}
        for name, param in module.named_parameters():
            ecc = self.state.get(param, {}).get("error_bits")
            if ecc is not None:
                out[name] = reconstruct_fp32_param(self._get_local_tensor(param.detach()), ecc)
        return out

    def set_fp32_model_state_dict(self, model: nn.Module, fp32_state_dict: dict[str, torch.Tensor]) -> None:
        """Inverse of :meth:`get_fp32_model_state_dict`: narrows into the parameters and recomputes their ECC
        (ref:1086-1147)."""
        module = cast(nn.Module, model.module if hasattr(model, "module") else model)
        self._plan_epoch += 1  # error_bits tensors are replaced below
        for name, param in module.named_parameters():
            if name not in fp32_state_dict:
                continue
            value = fp32_state_dict[name]
            if value.dtype != torch.float32:
                raise ValueError(f"Expected fp32 value for '{name}', got {value.dtype}.")
            local_param = self._get_local_tensor(param.data)
            local_value = self._get_local_tensor(value)
            if local_value.device != local_param.device:
                local_value = local_value.to(local_param.device)
            local_param.copy_(local_value.to(param.dtype))
            state = self.state.get(param, {})
            if "error_bits" in state:
                width = local_param.element_size() + state["error_bits"].element_size()
                state["error_bits"] = compute_ecc_bits(local_value, local_param, master_bytewidth=width)
