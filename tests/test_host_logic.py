"""CPU tests of the host-side logic: the C ABI surface, the chunk-table builder, constructor validation,
check_numerics' closed form, cast_model and the argument checks of gradient release.  No kernel runs here."""

import ctypes
import math
import os
import re
from collections import OrderedDict

import pytest
import torch
import torch.nn as nn

import flashoptim_amd
from flashoptim_amd import _native
from flashoptim_amd.optimizers import (
    _BITS_TO_BYTES,
    FlashAdam,
    FlashAdamW,
    FlashLion,
    FlashSGD,
    FlashSGDW,
    QuantizedTensorSpec,
    _log2_min_expressible_step_size,
    cast_model,
    enable_gradient_release,
)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NO_GPU = not torch.cuda.is_available()


# ------------------------------------------------------------------------------------------- C ABI


def _declared_symbols(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fo_[a-z0-9_]+)\s*\(", text)))


def _exported_symbols(path):
    import subprocess

    out = subprocess.run(["nm", "-D", "--defined-only", path], capture_output=True, text=True, check=True).stdout
    return sorted(line.split()[-1] for line in out.splitlines() if line.split()[-1].startswith("fo_"))


def test_library_exports_every_declared_symbol():
    """The product library exports exactly what include/flashoptim_hip.h declares (no measurement kernels); the
    diagnostics build exports that plus include/flashoptim_hip_diag.h; the ctypes tables bind exactly those."""
    product, diag = _declared_symbols("flashoptim_hip.h"), _declared_symbols("flashoptim_hip_diag.h")
    assert len(product) >= 15 and len(diag) >= 4 and not set(product) & set(diag)
    lib = _native.lib()
    for name in product:
        assert hasattr(lib, name), f"{name} is declared in include/flashoptim_hip.h but not exported"
    assert _exported_symbols(_native.library_path()) == product
    assert sorted(_native.SIGNATURES) == product
    dlib = _native.diag_lib()
    for name in product + diag:
        assert hasattr(dlib, name), f"{name} is missing from the diagnostics build"
    assert _exported_symbols(_native.diag_library_path()) == sorted(product + diag)
    assert sorted(_native.DIAG_SIGNATURES) == diag


def test_version_and_error_text_without_a_device():
    lib = _native.lib()
    assert lib.fo_version() >= 100
    assert isinstance(lib.fo_last_error(), bytes)
    # argument validation happens before any device work, so it is testable without a GPU
    rc = lib.fo_adam_step(None, None, None, None, None, None, None, -5, 1, 1, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 1, None)
    assert rc == -1 and b"n must be" in lib.fo_last_error()
    rc = lib.fo_adam_step(None, None, None, None, None, None, None, 0, 7, 0, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 1, None)
    assert rc == -1 and b"dtype" in lib.fo_last_error()
    rc = lib.fo_adam_step(None, None, None, None, None, None, None, 0, 0, 1, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 1, None)
    assert rc == -2  # ECC on fp32 parameters
    assert lib.fo_adam_step(None, None, None, None, None, None, None, 0, 1, 1, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 1, None) == 0
    with pytest.raises(RuntimeError, match="code -1"):
        _native.check(-1, "fo_adam_step")
    assert _native.diag_lib().fo_copy_bytes(None, None, 24, None) == -1
    assert lib.fo_ecc_join(None, 0, None, 1, None, 4, None) == -1  # fp32 "narrow" dtype is rejected
    assert lib.fo_ecc_split(None, None, 1, None, 3, 4, None) == -1


def _chunks(numels, tiles_per_chunk=0):
    lib = _native.lib()
    n = len(numels)
    lens = (ctypes.c_int64 * max(n, 1))(*numels)
    count = lib.fo_count_chunks(lens, n, tiles_per_chunk)
    table = (_native.FoChunk * max(count, 1))()
    assert lib.fo_build_chunks(lens, n, tiles_per_chunk, table, count) == count
    return [(c.tensor, c.first_tile, c.n_tiles) for c in table[:count]]


def test_chunk_table_covers_every_tile_once_and_never_straddles_tensors():
    numels = [0, 1, 31, 4096, 4097, 5 * 4096, 1 << 20, 33, 0, (1 << 24) + 5]
    for tpc in (0, 1, 3, 8):
        chunks = _chunks(numels, tpc)
        limit = tpc if tpc > 0 else 4
        seen = {}
        for tensor, first, count in chunks:
            assert 1 <= count <= limit
            tiles = seen.setdefault(tensor, [])
            tiles.extend(range(first, first + count))
        for i, n in enumerate(numels):
            want = list(range((n + 4095) // 4096))
            assert seen.get(i, []) == want, (i, n, tpc)
    assert _chunks([]) == []
    assert _native.lib().fo_count_chunks((ctypes.c_int64 * 1)(-3), 1, 0) < 0


# ------------------------------------------------------------------------------ constructor behaviour


def test_hyperparameter_validation_comes_before_the_device_check():
    p = [nn.Parameter(torch.zeros(4))]
    with pytest.raises(ValueError, match="compress_state_dict=True requires quantize=True"):
        FlashAdamW(p, quantize=False, compress_state_dict=True)
    with pytest.raises(ValueError, match="Invalid learning rate"):
        FlashAdamW(p, lr=-1e-3)
    with pytest.raises(ValueError, match="Master weight bits"):
        FlashAdamW(p, master_weight_bits=16)
    with pytest.raises(ValueError, match="Invalid epsilon"):
        FlashAdam(p, eps=-1.0)
    with pytest.raises(ValueError, match="beta parameter at index 0"):
        FlashAdam(p, betas=(1.5, 0.9))
    with pytest.raises(ValueError, match="beta parameter at index 1"):
        FlashLion(p, betas=(0.9, -0.1))
    with pytest.raises(ValueError, match="weight_decay"):
        FlashLion(p, weight_decay=-1.0)
    with pytest.raises(ValueError, match="Nesterov"):
        FlashSGD(p, nesterov=True, momentum=0.0)
    with pytest.raises(ValueError, match="Nesterov"):
        FlashSGDW(p, nesterov=True, momentum=0.9, dampening=0.1)
    with pytest.raises(ValueError, match="weight_decay"):
        FlashSGD(p, weight_decay=-0.1)


@pytest.mark.skipif(not NO_GPU, reason="needs a machine without a GPU")
def test_no_device_raises_like_the_reference():
    p = [nn.Parameter(torch.zeros(4))]
    with pytest.raises(NotImplementedError, match="Quantization requires a CUDA device"):
        FlashAdamW(p)
    with pytest.raises(NotImplementedError, match="error correction bits"):
        FlashAdamW(p, quantize=False)
    with pytest.raises(NotImplementedError, match="Fused optimizer step"):
        FlashAdamW(p, quantize=False, master_weight_bits=None)
    # there is no eager CPU implementation behind fused=False either
    with pytest.raises(NotImplementedError):
        FlashAdamW(p, quantize=False, master_weight_bits=None, fused=False)
    with pytest.raises(NotImplementedError):
        flashoptim_amd.compute_ecc_bits(torch.zeros(4), torch.zeros(4, dtype=torch.bfloat16), 3)


def test_quantized_tensor_spec_validates_types():
    assert QuantizedTensorSpec() == QuantizedTensorSpec(signed=True, sqrt=False, softsign=True)
    with pytest.raises(ValueError):
        QuantizedTensorSpec(signed=1)
    with pytest.raises(ValueError):
        QuantizedTensorSpec(sqrt="yes")


def test_public_names_match_the_reference_package():
    for name in ("FlashAdam", "FlashAdamW", "FlashLion", "FlashOptimizer", "FlashSGD", "FlashSGDW",
                 "GradientReleaseHandle", "NumericsError", "cast_model", "compute_ecc_bits",
                 "enable_gradient_release", "reconstruct_fp32_param"):
        assert hasattr(flashoptim_amd, name)
    import inspect

    sig = inspect.signature(FlashAdamW.__init__)
    # the reference's parameters in its order; the one addition is keyword-only and defaults to off
    assert list(sig.parameters)[1:] == ["params", "lr", "betas", "eps", "weight_decay", "decouple_lr", "quantize",
                                        "compress_state_dict", "master_weight_bits", "check_numerics", "fused",
                                        "exact_update"]
    assert sig.parameters["exact_update"].kind is inspect.Parameter.KEYWORD_ONLY
    assert sig.parameters["exact_update"].default is None
    assert sig.parameters["weight_decay"].default == 1e-2 and sig.parameters["master_weight_bits"].default == 24
    sig = inspect.signature(FlashLion.__init__)
    assert sig.parameters["betas"].default == (0.9, 0.99) and sig.parameters["weight_decay"].default == 0
    sig = inspect.signature(FlashSGD.__init__)
    assert sig.parameters["lr"].default == 0.001 and sig.parameters["momentum"].default == 0.0


# ------------------------------------------------------------------------------------- check_numerics


@pytest.mark.parametrize("dtype,bits", [(torch.bfloat16, None), (torch.bfloat16, 24), (torch.bfloat16, 32),
                                        (torch.float16, 24), (torch.float32, None)])
@pytest.mark.parametrize("maxabs", [1.0, 1e2, 1e-2])
def test_min_expressible_step_closed_form(dtype, bits, maxabs):
    """Resolution of the master weight at magnitude maxabs: exponent(maxabs) - mantissa bits, where the master
    has 8*max(param bytes, master bytes) bits, one sign bit and the dtype's exponent bits; a step of 0.49 ulp is
    enough to round over."""
    got = _log2_min_expressible_step_size(dtype, maxabs, _BITS_TO_BYTES[bits])
    exp_bits = {torch.bfloat16: 8, torch.float16: 5, torch.float32: 8}[dtype]
    width = {torch.bfloat16: 16, torch.float16: 16, torch.float32: 32}[dtype]
    total = max(width, (bits or 0))
    mant = total - 1 - exp_bits
    assert got == pytest.approx(math.floor(math.log2(maxabs)) - mant - math.log2(0.49))
    # bf16 alone at 1.0: 7 mantissa bits -> a step below 2^-8.03 cannot move it; 24-bit masters gain 8 bits
    if dtype == torch.bfloat16 and maxabs == 1.0:
        assert got == pytest.approx({None: -7, 24: -15, 32: -23}[bits] - math.log2(0.49))


# ------------------------------------------------------------------------------------------ cast_model


def _seq(**layers):
    return nn.Sequential(OrderedDict(layers))


def test_cast_model_plain_and_selective():
    m = nn.Sequential(nn.Linear(16, 32), nn.ReLU(), nn.Linear(32, 10))
    cast_model(m)
    assert all(p.dtype == torch.bfloat16 for p in m.parameters())
    assert m(torch.randn(2, 16, dtype=torch.bfloat16)).shape == (2, 10)

    m = nn.Sequential(nn.Linear(16, 32), nn.LayerNorm(32), nn.BatchNorm1d(32), nn.Linear(32, 10))
    cast_model(m, selective=True)
    assert m[1].weight.dtype == torch.bfloat16      # LayerNorm has no running statistics
    assert m[2].weight.dtype == torch.float32 and m[2].running_mean.dtype == torch.float32
    assert m[2].num_batches_tracked.dtype == torch.int64
    assert m(torch.randn(2, 16, dtype=torch.bfloat16)).shape == (2, 10)

    m = nn.Sequential(nn.BatchNorm2d(3), nn.Flatten(), nn.Linear(3, 10))
    cast_model(m, selective=False)
    assert m[0].weight.dtype == torch.bfloat16 and m[0].running_var.dtype == torch.bfloat16
    assert m[0].num_batches_tracked.dtype == torch.int64  # integer buffers are left alone

    m = nn.Sequential(nn.Linear(4, 4))
    cast_model(m, dtype=torch.float16)
    assert m[0].weight.dtype == torch.float16


@pytest.mark.parametrize("norm,expect_fp32", [
    (nn.BatchNorm1d(8), True), (nn.InstanceNorm1d(8, affine=True), True), (nn.InstanceNorm2d(8, affine=True), True),
    (nn.GroupNorm(2, 8), False), (nn.LayerNorm(8), False), (nn.RMSNorm(8), False),
])
def test_cast_model_selective_norm_types(norm, expect_fp32):
    m = nn.Sequential(nn.Linear(8, 8), norm, nn.Linear(8, 8))
    cast_model(m, selective=True)
    want = torch.float32 if expect_fp32 else torch.bfloat16
    assert all(p.dtype == want for p in m[1].parameters())
    assert all(b.dtype == want for b in m[1].buffers() if b.is_floating_point())
    assert m[0].weight.dtype == torch.bfloat16 and m[2].weight.dtype == torch.bfloat16


def test_cast_model_full_precision_layers():
    m = _seq(backbone=nn.Linear(16, 32), head=nn.Linear(32, 10))
    cast_model(m, full_precision_layers=["head"])
    assert m.head.weight.dtype == torch.float32 and m.backbone.weight.dtype == torch.bfloat16
    assert getattr(m.head, "_has_fp32_input_hook", False) and len(m.head._forward_pre_hooks) == 1
    assert m.head(torch.randn(2, 32, dtype=torch.bfloat16)).dtype == torch.float32   # input upcast by the hook
    assert m(torch.randn(2, 16, dtype=torch.bfloat16)).dtype == torch.float32        # terminal fp32 output kept
    cast_model(m, full_precision_layers=["head"])                                    # idempotent: no second hook
    assert len(m.head._forward_pre_hooks) == 1

    # a module object instead of a pattern
    m = _seq(backbone=nn.Linear(16, 32), head=nn.Linear(32, 10))
    cast_model(m, full_precision_layers=[m.head])
    assert m.head.weight.dtype == torch.float32 and m.backbone.weight.dtype == torch.bfloat16

    # the pattern must match the whole dotted name
    m = _seq(multi_head_attn=nn.Linear(10, 10), head=nn.Linear(10, 5), backbone=nn.Linear(5, 10))
    cast_model(m, full_precision_layers=["head"])
    assert getattr(m.head, "_has_fp32_input_hook", False)
    assert not getattr(m.multi_head_attn, "_has_fp32_input_hook", False)
    assert m.multi_head_attn.weight.dtype == torch.bfloat16


def test_cast_model_nested_patterns_and_multi_input():
    class Nested(nn.Module):
        def __init__(self):
            super().__init__()
            self.encoder = nn.Linear(10, 10)
            self.decoder = nn.ModuleDict({"head": nn.Linear(10, 5), "proj": nn.Linear(10, 3)})

        def forward(self, x):
            return self.decoder["head"](self.encoder(x))

    m = Nested()
    cast_model(m, full_precision_layers=["*.head"])
    assert m.decoder["head"].weight.dtype == torch.float32 and m.decoder["proj"].weight.dtype == torch.bfloat16
    assert m(torch.randn(2, 10, dtype=torch.bfloat16)).dtype == torch.float32
    m = Nested()
    cast_model(m, full_precision_layers=["decoder.*"])
    assert m.decoder["head"].weight.dtype == torch.float32 and m.decoder["proj"].weight.dtype == torch.float32
    assert m.encoder.weight.dtype == torch.bfloat16

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.linear = nn.Linear(8, 8)

        def forward(self, x, mask):
            return self.linear(x) + mask

    class Outer(nn.Module):
        def __init__(self):
            super().__init__()
            self.block = Block()

        def forward(self, x, mask):
            return self.block(x, mask)

    m = Outer()
    cast_model(m, full_precision_layers=["block"])
    out = m(torch.randn(2, 8, dtype=torch.bfloat16), torch.randn(2, 8, dtype=torch.bfloat16))
    assert out.dtype == torch.float32  # every floating-point positional argument was upcast

    m = _seq(embed=nn.Embedding(50, 10))
    cast_model(m, full_precision_layers=["embed"])
    assert m(torch.tensor([0, 1, 2])).dtype == torch.float32  # integer inputs pass through the hook untouched


@pytest.mark.parametrize("target,needs_pre", [(nn.Linear(32, 32), True), (nn.LayerNorm(32), True),
                                              (nn.RMSNorm(32), True), (nn.Embedding(64, 32), False)])
def test_cast_model_recast_layers(target, needs_pre):
    layers = OrderedDict()
    if needs_pre:
        layers["pre"] = nn.Linear(32, 32)
    layers["target"] = target
    layers["post"] = nn.Linear(32, 32)
    m = nn.Sequential(layers)
    cast_model(m, full_precision_recast_layers=["target"])
    assert all(p.dtype == torch.float32 for p in m.target.parameters())
    assert m.post.weight.dtype == torch.bfloat16
    x = torch.randn(4, 32, dtype=torch.bfloat16) if needs_pre else torch.randint(0, 64, (4,))
    out = m(x)
    assert out.dtype == torch.bfloat16 and torch.isfinite(out.float()).all()
    assert len(m.target._forward_hooks) == 1


def test_cast_model_keeps_tied_weights_tied():
    class Tied(nn.Module):
        def __init__(self):
            super().__init__()
            self.embed = nn.Embedding(32, 16)
            self.output = nn.Linear(16, 32, bias=False)
            self.output.weight = self.embed.weight

    m = Tied()
    cast_model(m)
    assert m.embed.weight is m.output.weight and m.embed.weight.dtype == torch.bfloat16

    # tensors that only share storage (two Parameter objects over one buffer) are cast once and still share
    a, b = nn.Linear(4, 4, bias=False), nn.Linear(4, 4, bias=False)
    b.weight = nn.Parameter(a.weight.data)
    m = nn.Sequential(a, b)
    cast_model(m)
    assert a.weight.data_ptr() == b.weight.data_ptr()

    # empty tensors all report address 0 and views of one buffer may start at the same address: neither may be
    # mistaken for a shared tensor
    class Odd(nn.Module):
        def __init__(self):
            super().__init__()
            flat = torch.randn(12)
            self.e1 = nn.Parameter(torch.zeros(0, 4))
            self.e2 = nn.Parameter(torch.zeros(3, 0))
            self.v1 = nn.Parameter(flat.view(3, 4))
            self.v2 = nn.Parameter(flat[:6].view(2, 3))

    m = Odd()
    cast_model(m)
    assert [tuple(p.shape) for p in (m.e1, m.e2, m.v1, m.v2)] == [(0, 4), (3, 0), (3, 4), (2, 3)]
    assert all(p.dtype == torch.bfloat16 for p in m.parameters())


# ------------------------------------------------------------------------------------ gradient release


def test_gradient_release_rejects_grad_scaler_before_anything_else():
    with pytest.raises(NotImplementedError, match="GradScaler"):
        enable_gradient_release(nn.Linear(2, 2), optimizer=None, grad_scaler=object())


def test_packaging_declares_the_reference_entry_points():
    """llm-foundry discovers optimizers through the `llmfoundry_optimizers` entry-point group; the names are the
    reference's (/root/reference/pyproject.toml:47-52) and every target resolves to a class of this package."""
    import importlib
    import os

    import tomli

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with open(os.path.join(root, "pyproject.toml"), "rb") as f:
        points = tomli.load(f)["project"]["entry-points"]["llmfoundry_optimizers"]
    assert sorted(points) == ["flash_adam", "flash_adam_w", "flash_lion", "flash_sgd", "flash_sgd_w"]
    for target in points.values():
        module, _, name = target.partition(":")
        assert issubclass(getattr(importlib.import_module(module), name), torch.optim.Optimizer)


# ------------------------------------------------------------------------------------------- host scan helper


def test_hostscan_module_validates_a_launch_table_like_the_python_walk():
    """flashoptim_amd/lib/_fo_hostscan.so (C++ over the tensor objects): the per-step check of a cached launch plan.
    Unchanged tensors give an empty tuple; gradients that moved are reported with their new address; a missing,
    frozen, strided, resized or re-typed gradient, a parameter on other storage, a non-tensor or a tensor without
    storage make it decline; a list of another length than the table is refused."""
    from flashoptim_amd import _hostscan
    from flashoptim_amd._native import FoTensorDesc

    assert _hostscan.scan is not None, "build it with make -C flashoptim_amd/hostscan"
    n = 50
    params = [torch.nn.Parameter(torch.randn(10)) for _ in range(n)]
    for p in params:
        p.grad = torch.randn(10)
    table = (FoTensorDesc * n)()
    for d, p in zip(table, params):
        d.param, d.grad, d.n = p.data_ptr(), p.grad.data_ptr(), 10
    addr = ctypes.addressof(table)
    assert _hostscan.scan(params, addr, n) == ()
    keep = [p.grad for p in params]                        # keeps the old addresses from being handed out again
    params[7].grad, params[9].grad = torch.randn(10), torch.randn(10)
    assert _hostscan.scan(params, addr, n) == ((7, params[7].grad.data_ptr()), (9, params[9].grad.data_ptr()))
    table[7].grad, table[9].grad = params[7].grad.data_ptr(), params[9].grad.data_ptr()
    assert _hostscan.scan(params, addr, n) == ()

    def declines(change, undo):
        change()
        got = _hostscan.scan(params, addr, n)
        undo()
        return got is None

    p5, g5 = params[5], params[5].grad
    assert declines(lambda: setattr(p5, "grad", None), lambda: setattr(p5, "grad", g5))
    assert declines(lambda: setattr(p5, "grad", torch.randn(20)[::2]), lambda: setattr(p5, "grad", g5))
    assert declines(lambda: setattr(p5, "grad", None) or p5.requires_grad_(False), lambda: (p5.requires_grad_(True), setattr(p5, "grad", g5)))
    old = p5.data
    assert declines(lambda: setattr(p5, "data", torch.randn(10)), lambda: setattr(p5, "data", old))
    assert _hostscan.scan(params, addr, n) == ()
    assert _hostscan.scan(params[:5] + [3], addr, 6) is None
    with pytest.raises(TypeError):
        _hostscan.scan(tuple(params), addr, n)
    with pytest.raises(ValueError):                        # a list that is not the table's length is never walked
        _hostscan.scan(params + params[:1], addr, n)
    # a tensor object libtorch cannot give a data pointer for makes the walk decline instead of ending the process
    meta = torch.nn.Parameter(torch.empty(10, device="meta"))
    meta.grad = torch.empty(10, device="meta")
    assert _hostscan.scan([meta], addr, 1) is None
    assert _hostscan.same_objects(params, list(params)) and not _hostscan.same_objects(params, params[:-1])
    assert not _hostscan.same_objects(params, params[1:] + params[:1])
    del keep
