"""fo_multi_adam_step_static: the multi-tensor Adam step whose launch tables live in a static device array.

The entry point is called through the C ABI with a host descriptor array and must give, bit for bit, what the
existing fo_multi_adam_step gives with caller-owned device tables: on two calls in a row (the second with a
smaller list, so stale table entries of the first call lie behind the ones in use), on a list with more tiles than
the static chunk table has entries, and it must refuse a list that is too long.
"""

import ctypes

import pytest
import torch

from flashoptim_amd import _native
from flashoptim_amd._native import DTYPE_CODE, FoTensorDesc
from flashoptim_amd.launcher import BucketPlan, StepTensors
from tests import parity

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HP = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-5, decoupled=True)


def _make(lens, dtype, ecc_dtype, seed):
    g = torch.Generator().manual_seed(seed)
    out = []
    for n in lens:
        out.append(StepTensors(
            param=(torch.randn(n, generator=g) * 0.02).to(dtype).to(DEV),
            grad=(torch.randn(n, generator=g) * 1e-3).to(dtype).to(DEV),
            ecc=None if ecc_dtype is None else torch.zeros(n, dtype=ecc_dtype, device=DEV),
            mom=torch.zeros(n, dtype=torch.int8, device=DEV), mom_scales=torch.zeros((n + 31) // 32, dtype=torch.float16, device=DEV),
            var=torch.zeros(n, dtype=torch.uint8, device=DEV), var_scales=torch.zeros((n + 31) // 32, dtype=torch.float16, device=DEV)))
    return out


def _static_step(tensors, dtype, ecc_bytes, step):
    table = (FoTensorDesc * max(len(tensors), 1))()
    p = _native.ptr
    for d, t in zip(table, tensors):
        d.param, d.grad, d.ecc, d.mom, d.mom_scales = p(t.param), p(t.grad), p(t.ecc), p(t.mom), p(t.mom_scales)
        d.var, d.var_scales, d.n = p(t.var), p(t.var_scales), t.param.numel()
    rc = _native.lib().fo_multi_adam_step_static(table, len(tensors), DTYPE_CODE[dtype], ecc_bytes, 1, HP["lr"], HP["beta1"],
                                                 HP["beta2"], HP["eps"], HP["weight_decay"], 1, step,
                                                 _native.current_stream_ptr(torch.device(DEV)))
    return rc


def _same(a, b):
    for x, y in zip(a, b):
        for name in ("param", "ecc", "mom", "mom_scales", "var", "var_scales"):
            u, v = getattr(x, name), getattr(y, name)
            assert (u is None and v is None) or parity.bits_equal(u, v), f"{name} differs"


@pytest.mark.parametrize("dtype,ecc_dtype", [(torch.bfloat16, torch.int8), (torch.bfloat16, torch.int16), (torch.float32, None)])
def test_static_tables_equal_caller_owned_tables_on_two_calls_in_a_row(dtype, ecc_dtype):
    ecc_bytes = 0 if ecc_dtype is None else torch.empty(0, dtype=ecc_dtype).element_size()
    first = [1, 31, 33, 4096, 4097, 70001, 5, 300000, 0, 12345] + [777] * 60      # more than one staging batch
    second = [9000, 2, 4095]                                                       # smaller: stale entries lie behind it
    for lens, seed in ((first, 1), (second, 2)):
        a, b = _make(lens, dtype, ecc_dtype, seed), _make(lens, dtype, ecc_dtype, seed)
        plan = BucketPlan("adam", dtype, ecc_bytes, True, [t for t in b])
        for step in (1, 2, 3):
            _native.check(_static_step(a, dtype, ecc_bytes, step), "fo_multi_adam_step_static")
            plan.launch(step=step, **HP)
        torch.cuda.synchronize()
        _same(a, b)


def test_more_tiles_than_chunk_entries_and_too_many_tensors():
    # 70 000 tiles > 65 536 chunk entries: the call covers two tiles per work item
    lens = [4096 * 30000 + 17, 4096 * 40000 - 5, 100]
    a, b = _make(lens, torch.bfloat16, torch.int8, 3), _make(lens, torch.bfloat16, torch.int8, 3)
    plan = BucketPlan("adam", torch.bfloat16, 1, True, b)
    for step in (1, 2):
        _native.check(_static_step(a, torch.bfloat16, 1, step), "fo_multi_adam_step_static")
        plan.launch(step=step, **HP)
    torch.cuda.synchronize()
    _same(a, b)
    del a, b, plan
    # a list longer than the static descriptor table is refused with a clear message, before any launch
    tiny = _make([8] * 1025, torch.bfloat16, torch.int8, 4)
    rc = _static_step(tiny, torch.bfloat16, 1, 1)
    assert rc != 0 and b"exceed" in _native.lib().fo_last_error()
    assert _static_step([], torch.bfloat16, 1, 1) == 0


@pytest.mark.parametrize("dtype,ecc_dtype", [(torch.bfloat16, torch.int8), (torch.bfloat16, torch.int16)])
def test_a_captured_static_call_replays_like_the_eager_entry_point(dtype, ecc_dtype):
    """The callers this entry point is for include code under HIP graph capture.  The first call on a device (and
    the first of each kernel variant) takes the address of the static array and plans the residency through host
    API calls that must not run while a stream captures, so one eager call comes first.  After that a call records
    nothing but kernel launches (the table-staging kernels and the step kernel; no copies, no memsets, no
    allocation).  The step number travels by value, so every replay repeats the captured step number: each replay,
    with new gradient values in the same buffers and eager work and synchronisations in between, must equal an
    eager fo_multi_adam_step call with that step number, bit for bit."""
    ecc_bytes = torch.empty(0, dtype=ecc_dtype).element_size()
    lens = [1, 33, 4096, 70001, 12345] + [777] * 50
    a, b = _make(lens, dtype, ecc_dtype, 11), _make(lens, dtype, ecc_dtype, 11)
    plan = BucketPlan("adam", dtype, ecc_bytes, True, b)
    _native.check(_static_step(a, dtype, ecc_bytes, 1), "fo_multi_adam_step_static")   # eager: set-up happens here
    plan.launch(step=1, **HP)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = _static_step(a, dtype, ecc_bytes, 2)
    _native.check(rc, "fo_multi_adam_step_static under capture")
    gen = torch.Generator().manual_seed(12)
    for replay in range(4):
        for x, y in zip(a, b):   # new gradient values, same buffers
            g = (torch.randn(x.grad.numel(), generator=gen) * 1e-3).to(dtype).to(DEV)
            x.grad.copy_(g)
            y.grad.copy_(g)
        torch.cuda.synchronize()
        graph.replay()
        plan.launch(step=2, **HP)
        torch.cuda.synchronize()
        _same(a, b)
