"""Multi-tensor launcher: packs many parameter tensors of ragged sizes into one grid.

The reference launches one kernel per tensor from a Python loop (``/root/reference/flashoptim/optimizers.py:
770-785``).  Here ``FlashOptimizer.step`` collects the tensors that share a kernel specialisation and scalar
hyper-parameters into a *bucket* and issues one launch per bucket.  A launch needs two small device tables:

* the chunk table (``fo_chunk``: tensor index, first 4096-element tile, tile count) depends only on the tensor
  lengths; it is built once on the host by ``fo_build_chunks`` and cached;
* the descriptor table (``fo_tensor_desc``: the raw pointers of every tensor) is re-uploaded only when a
  pointer changed since the previous step (gradients are re-allocated by ``zero_grad(set_to_none=True)``,
  although the caching allocator usually hands back the same addresses).  The upload goes through pinned host
  memory with a stream-ordered copy, so ``step`` never synchronises with the device.

Chunks never straddle tensors and start on 4096-element boundaries counted from element 0 of their tensor, so
quantisation groups are exactly those of a per-tensor launch and the result is bit-identical to it.
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass, field
from typing import Optional, Sequence

import torch

from . import _native
from ._native import DTYPE_CODE, FoChunk, FoTensorDesc


@dataclass
class StepTensors:
    """The device tensors of one parameter as the kernels see them (all flat-contiguous)."""

    param: torch.Tensor
    grad: torch.Tensor
    ecc: Optional[torch.Tensor]
    mom: Optional[torch.Tensor]
    mom_scales: Optional[torch.Tensor]
    var: Optional[torch.Tensor] = None
    var_scales: Optional[torch.Tensor] = None

    def pointers(self) -> tuple:
        p = _native.ptr
        return (p(self.param), p(self.grad), p(self.ecc), p(self.mom), p(self.mom_scales), p(self.var), p(self.var_scales))


@dataclass
class _Plan:
    n_tensors: int
    n_chunks: int
    chunks_dev: torch.Tensor           # uint8 view of fo_chunk[n_chunks]
    descs_dev: torch.Tensor            # uint8 view of fo_tensor_desc[n_tensors]
    numels: tuple
    last_pointers: Optional[tuple] = None
    keepalive: list = field(default_factory=list)


class MultiTensorLauncher:
    """Caches the launch tables per (device, tensor-length signature) and issues the multi-tensor kernels."""

    def __init__(self, tiles_per_chunk: int = 0):
        self._tiles_per_chunk = int(tiles_per_chunk)
        self._plans: dict[tuple, _Plan] = {}

    def clear(self) -> None:
        self._plans.clear()

    # ------------------------------------------------------------------------------------------ tables
    def _plan_for(self, tensors: Sequence[StepTensors], device: torch.device, tag: tuple) -> _Plan:
        numels = tuple(t.param.numel() for t in tensors)
        key = (device, tag, numels)
        plan = self._plans.get(key)
        if plan is not None:
            return plan
        lib = _native.lib()
        n = len(numels)
        lens = (ctypes.c_int64 * n)(*numels)
        n_chunks = lib.fo_count_chunks(lens, n, self._tiles_per_chunk)
        if n_chunks < 0:
            _native.check(int(n_chunks), "fo_count_chunks")
        table = (FoChunk * max(n_chunks, 1))()
        built = lib.fo_build_chunks(lens, n, self._tiles_per_chunk, table, n_chunks)
        if built != n_chunks:
            _native.check(int(built) if built < 0 else -1, "fo_build_chunks")
        host = torch.frombuffer(bytearray(bytes(table)), dtype=torch.uint8)[: n_chunks * ctypes.sizeof(FoChunk)]
        chunks_dev = host.to(device)
        descs_dev = torch.empty(max(n, 1) * ctypes.sizeof(FoTensorDesc), dtype=torch.uint8, device=device)
        plan = _Plan(n, int(n_chunks), chunks_dev, descs_dev, numels)
        self._plans[key] = plan
        return plan

    def _refresh_descriptors(self, plan: _Plan, tensors: Sequence[StepTensors]) -> None:
        pointers = tuple(t.pointers() for t in tensors)
        if pointers == plan.last_pointers:
            return
        table = (FoTensorDesc * plan.n_tensors)()
        for d, ptrs, n in zip(table, pointers, plan.numels):
            d.param, d.grad, d.ecc, d.mom, d.mom_scales, d.var, d.var_scales = ptrs
            d.n = n
        staged = torch.frombuffer(bytearray(bytes(table)), dtype=torch.uint8).pin_memory()
        # stream-ordered: launches already queued with the previous table finish before it is overwritten;
        # the pinned staging block is recycled by torch's host allocator only after the copy has run
        plan.descs_dev[: staged.numel()].copy_(staged, non_blocking=True)
        plan.last_pointers = pointers

    # ----------------------------------------------------------------------------------------- launches
    def _prepare(self, tensors: Sequence[StepTensors], tag: tuple):
        device = tensors[0].param.device
        for t in tensors:
            if t.param.device != device:
                raise ValueError("all tensors of one multi-tensor launch must live on one device")
        plan = self._plan_for(tensors, device, tag)
        if plan.n_chunks:
            self._refresh_descriptors(plan, tensors)
        return device, plan

    def adam(self, tensors: Sequence[StepTensors], dtype: torch.dtype, ecc_bytes: int, quantized: bool, lr: float,
             beta1: float, beta2: float, eps: float, weight_decay: float, decoupled: bool, step: int) -> None:
        if not tensors:
            return
        device, plan = self._prepare(tensors, ("adam", dtype, ecc_bytes, quantized))
        if plan.n_chunks == 0:
            return
        with torch.cuda.device(device):
            rc = _native.lib().fo_multi_adam_step(
                plan.descs_dev.data_ptr(), plan.n_tensors, plan.chunks_dev.data_ptr(), plan.n_chunks,
                DTYPE_CODE[dtype], ecc_bytes, int(quantized), lr, beta1, beta2, eps, weight_decay, int(decoupled),
                int(step), _native.current_stream_ptr(device),
            )
        _native.check(rc, "fo_multi_adam_step")

    def momentum(self, tensors: Sequence[StepTensors], dtype: torch.dtype, ecc_bytes: int, quantized: bool, lr: float,
                 mom_coef: float, update_coef: float, weight_decay: float, decoupled: bool, nesterov: bool,
                 do_lion: bool) -> None:
        if not tensors:
            return
        device, plan = self._prepare(tensors, ("momentum", dtype, ecc_bytes, quantized))
        if plan.n_chunks == 0:
            return
        with torch.cuda.device(device):
            rc = _native.lib().fo_multi_momentum_step(
                plan.descs_dev.data_ptr(), plan.n_tensors, plan.chunks_dev.data_ptr(), plan.n_chunks,
                DTYPE_CODE[dtype], ecc_bytes, int(quantized), lr, mom_coef, update_coef, weight_decay,
                int(decoupled), int(nesterov), int(do_lion), _native.current_stream_ptr(device),
            )
        _native.check(rc, "fo_multi_momentum_step")
