"""Multi-tensor launcher: packs many parameter tensors of ragged sizes into one grid.

The reference launches one kernel per tensor from a Python loop (``/root/reference/flashoptim/optimizers.py:
770-785``).  Here ``FlashOptimizer.step`` collects the tensors that share a kernel specialisation and scalar
hyper-parameters into a *bucket* and issues one launch per bucket.  A bucket owns two small device tables:

* the chunk table (``fo_chunk``: tensor index, first 4096-element tile, tile count) depends only on the tensor
  lengths; it is built once on the host by ``fo_build_chunks``;
* the descriptor table (``fo_tensor_desc``: the raw pointers of every tensor).  Parameters and optimizer states
  keep their addresses; gradients are re-allocated by ``zero_grad(set_to_none=True)`` (although the caching
  allocator usually hands back the same addresses), so each step only compares gradient addresses and re-uploads
  the table when one moved.  The upload goes through one pinned staging buffer per bucket with a stream-ordered
  copy: ``step`` never waits for the device (it only waits for the previous upload of the same bucket to have left
  the staging buffer, which has long happened).  The table holds addresses, not tensor references, so a freed
  gradient is not kept alive.  Under HIP graph capture a table cannot be built or re-uploaded (the copy would be
  recorded with the staging buffer's contents of that moment): ``launch`` raises instead, see there.

Chunks never straddle tensors and start on 4096-element boundaries counted from element 0 of their tensor, so
quantisation groups are exactly those of a per-tensor launch and the result is bit-identical to it.
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Optional, Sequence

import torch

from . import _native, kernels
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


def chunk_table(numels: Sequence[int], tiles_per_chunk: int = 0) -> tuple[torch.Tensor, int]:
    """The ``fo_chunk`` table for tensors of these lengths as a host byte tensor, and its entry count."""
    lib = _native.lib()
    n_tensors = len(numels)
    lens = (ctypes.c_int64 * max(n_tensors, 1))(*numels)
    n_chunks = lib.fo_count_chunks(lens, n_tensors, tiles_per_chunk)
    if n_chunks < 0:
        _native.check(int(n_chunks), "fo_count_chunks")
    table = (FoChunk * max(n_chunks, 1))()
    built = lib.fo_build_chunks(lens, n_tensors, tiles_per_chunk, table, n_chunks)
    if built != n_chunks:
        _native.check(int(built) if built < 0 else -1, "fo_build_chunks")
    host = torch.frombuffer(bytearray(bytes(table)), dtype=torch.uint8)[: int(n_chunks) * ctypes.sizeof(FoChunk)]
    return host, int(n_chunks)


def absmax_many(tensors: Sequence[torch.Tensor]) -> list[float]:
    """``float(t.abs().max())`` of every tensor (0 for empty ones): one launch per (device, dtype) and one
    device-to-host copy per device, where the reference synchronises once per tensor
    (``/root/reference/flashoptim/optimizers.py:656-673``).  A tensor holding a NaN reports NaN.  Like the step
    kernels it takes fp32, bf16 and fp16 tensors on a GPU; a non-contiguous tensor is compacted on the device first."""
    out: list[float] = [0.0] * len(tensors)
    groups: dict = {}
    tensors = list(tensors)
    for i, t in enumerate(tensors):
        if t.numel() == 0:
            continue
        if not t.is_cuda:
            raise NotImplementedError(f"absmax_many runs on a ROCm GPU only; got a tensor on {t.device}.")
        if t.dtype not in DTYPE_CODE:
            raise ValueError(f"Unsupported dtype {t.dtype}.")
        if not t.is_contiguous():
            tensors[i] = t = t.contiguous()
        groups.setdefault((t.device, t.dtype), []).append(i)
    pending = []
    for (device, dtype), idx in groups.items():
        table = (FoTensorDesc * len(idx))()
        for d, i in zip(table, idx):
            d.param, d.n = tensors[i].data_ptr(), tensors[i].numel()
        chunks_host, n_chunks = chunk_table([tensors[i].numel() for i in idx], tiles_per_chunk=16)
        with _native.device_guard(device):
            descs = torch.frombuffer(bytearray(bytes(table)), dtype=torch.uint8).to(device)
            chunks = chunks_host.to(device)
            result = torch.zeros(len(idx), dtype=torch.float32, device=device)
            rc = _native.lib().fo_multi_absmax(descs.data_ptr(), len(idx), chunks.data_ptr(), n_chunks, DTYPE_CODE[dtype],
                                               result.data_ptr(), _native.current_stream_ptr(device))
        _native.check(rc, "fo_multi_absmax")
        pending.append((idx, result, descs, chunks))
    for idx, result, _descs, _chunks in pending:  # the tables stay alive until the results are read
        for i, v in zip(idx, result.tolist()):
            out[i] = float(v)
    return out


class BucketPlan:
    """Launch tables of one bucket: tensors that share kernel kind, dtype, ECC width and quantisation."""

    def __init__(self, kind: str, dtype: torch.dtype, ecc_bytes: int, quantized: bool,
                 tensors: Sequence[StepTensors], tiles_per_chunk: int = 0):
        if kind not in ("adam", "momentum", "plain"):
            raise ValueError(f"no multi-tensor kernel for kind {kind!r}")
        self.kind, self.dtype, self.ecc_bytes, self.quantized = kind, dtype, int(ecc_bytes), bool(quantized)
        self.device = tensors[0].param.device
        if any(t.param.device != self.device for t in tensors):
            raise ValueError("all tensors of one multi-tensor launch must live on one device")
        self.n_tensors = len(tensors)
        for t in tensors:  # once per plan: the kernels only see addresses and trust these shapes
            kernels._check_step_tensors(t.param, t.grad, t.ecc)
            if kernels._ecc_bytes(t.ecc) != self.ecc_bytes or t.param.dtype != dtype:
                raise ValueError("every tensor of a bucket must share the parameter dtype and the ECC width")
            if kind != "plain":
                kernels._check_moment(t.param, t.mom, t.mom_scales, self.quantized, True, "mom")
            if kind == "adam":
                kernels._check_moment(t.param, t.var, t.var_scales, self.quantized, False, "var")
        numels = [t.param.numel() for t in tensors]
        p = _native.ptr
        self.table = (FoTensorDesc * self.n_tensors)()
        for d, t, n in zip(self.table, tensors, numels):
            d.param, d.grad, d.ecc, d.mom, d.mom_scales = p(t.param), p(t.grad), p(t.ecc), p(t.mom), p(t.mom_scales)
            d.var, d.var_scales, d.n = p(t.var), p(t.var_scales), n
        # the state tensors must outlive the table that points at them (gradients are tracked by address only)
        self._keepalive = [(t.param, t.ecc, t.mom, t.mom_scales, t.var, t.var_scales) for t in tensors]
        self.grad_ptrs = [d.grad for d in self.table]
        self.param_ptrs = [d.param for d in self.table]
        self.table_address = ctypes.addressof(self.table)  # for the C++ walk over the table (flashoptim_amd/_hostscan.py)

        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError(
                "The launch tables of a multi-tensor step cannot be built while a HIP graph is being captured. Run one "
                "step outside the capture first, with the gradient buffers the graph will use.")
        host, self.n_chunks = chunk_table(numels, tiles_per_chunk)
        self.chunks_dev = host.to(self.device)
        nbytes = self.n_tensors * ctypes.sizeof(FoTensorDesc)
        self.descs_dev = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        # two pinned staging buffers for the life of the plan, used in turn; `_staged[i]` marks the last copy out of
        # buffer i
        self._staging = [torch.empty(nbytes, dtype=torch.uint8).pin_memory() for _ in range(2)]
        self._table_bytes = torch.frombuffer(self.table, dtype=torch.uint8)  # a view of the ctypes table, no copy
        self._staged: list[Optional[torch.cuda.Event]] = [None, None]
        self._next_staging = 0
        self._dirty = True

    def set_grad_ptr(self, index: int, ptr: int) -> None:
        self.table[index].grad = ptr
        self.grad_ptrs[index] = ptr
        self._dirty = True

    def _upload(self) -> None:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError(
                "A gradient of this multi-tensor step moved to another address, so its pointer table has to be "
                "uploaded again, which cannot be recorded into a HIP graph (a replay would copy whatever the staging "
                "buffer holds by then). Run one step outside the capture with the gradient buffers the graph will use "
                "(static gradients, zero_grad(set_to_none=False)), then capture.")
        # The host waits only when the copy out of this buffer, queued two uploads ago, has not run yet: with
        # gradients that move every step the host can therefore run two iterations ahead of the device before it
        # blocks here (a single buffer would tie it to the previous step's copy, which sits behind a whole iteration
        # of queued work).
        i = self._next_staging
        self._next_staging = 1 - i
        if self._staged[i] is not None and not self._staged[i].query():
            self._staged[i].synchronize()
        self._staging[i].copy_(self._table_bytes)
        # stream-ordered: launches already queued with the previous table finish before it is overwritten
        self.descs_dev.copy_(self._staging[i], non_blocking=True)
        if self._staged[i] is None:
            self._staged[i] = torch.cuda.Event()
        self._staged[i].record()
        self._dirty = False

    def launch(self, **scalars) -> None:
        """Enqueue the bucket's kernel on the current stream with the given fp32 scalars."""
        if self.n_chunks == 0:
            return
        with _native.device_guard(self.device):
            if self._dirty:
                self._upload()
            lib = _native.lib()
            head = (self.descs_dev.data_ptr(), self.n_tensors, self.chunks_dev.data_ptr(), self.n_chunks,
                    DTYPE_CODE[self.dtype], self.ecc_bytes, int(self.quantized))
            stream = _native.current_stream_ptr(self.device)
            if self.kind == "adam":
                entry = lib.fo_multi_adam_step_exact if scalars.get("exact_update") else lib.fo_multi_adam_step
                rc = entry(*head, scalars["lr"], scalars["beta1"], scalars["beta2"], scalars["eps"],
                           scalars["weight_decay"], int(scalars["decoupled"]), int(scalars["step"]), stream)
            elif self.kind == "plain":
                rc = lib.fo_multi_sgd_plain_step(*head[:6], scalars["lr"], scalars["weight_decay"],
                                                 int(scalars["decoupled"]), stream)
            else:
                rc = lib.fo_multi_momentum_step(*head, scalars["lr"], scalars["mom_coef"], scalars["update_coef"],
                                                scalars["weight_decay"], int(scalars["decoupled"]),
                                                int(scalars["nesterov"]), int(scalars["do_lion"]), stream)
        _native.check(rc, "fo_multi_sgd_plain_step" if self.kind == "plain" else f"fo_multi_{self.kind}_step")

    def launch_streams_copy(self) -> None:
        """Measurement aid (Adam and momentum buckets; needs the diagnostics build of the library): read every stream
        of the bucket and write it back unchanged with the step kernels' access code, without the step's arithmetic;
        shows what rate the step's access mix can reach."""
        if self.kind not in ("adam", "momentum"):
            raise ValueError("the access-mix copy exists for Adam and momentum buckets only")
        if self.n_chunks == 0:
            return
        with _native.device_guard(self.device):
            if self._dirty:
                self._upload()
            diag = _native.diag_lib()
            entry = getattr(diag, f"fo_multi_{self.kind}_streams_copy")
            rc = entry(self.descs_dev.data_ptr(), self.n_tensors, self.chunks_dev.data_ptr(), self.n_chunks,
                       DTYPE_CODE[self.dtype], self.ecc_bytes, int(self.quantized), _native.current_stream_ptr(self.device))
        _native.check(rc, f"fo_multi_{self.kind}_streams_copy", diag)
