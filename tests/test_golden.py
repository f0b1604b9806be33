"""Committed vectors (tests/golden/step_vectors.npz, written by tests/golden/make_vectors.py from the C oracle).

CPU: both restatements of the reference's algorithm (oracle/fo_oracle.c, oracle/torch_oracle.py) still reproduce
the committed outputs bit for bit.  GPU: the HIP kernels, fed the committed inputs through the C ABI, land within
the parity tolerances of the committed outputs (bit-exact for the standalone codec and ECC kernels)."""

import os
import sys

import numpy as np
import pytest
import torch

from oracle import c_oracle as C
from oracle import torch_oracle as T
from tests import parity

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_vectors as G  # noqa: E402

DEV = "cuda:0"
VEC = np.load(os.path.join(HERE, "golden", "step_vectors.npz"))

QUANT = {"quant_signed_softsign_f32": (torch.float32, True, False, True),
         "quant_unsigned_sqrt_bf16": (torch.bfloat16, False, True, False),
         "quant_signed_linear_f16": (torch.float16, True, False, False)}
ECCS = {"ecc_bf16_i8": (torch.bfloat16, torch.int8), "ecc_f16_i16": (torch.float16, torch.int16)}


def _get(key, dtype=None):
    a = VEC[key]
    return G.from_np(a, dtype) if dtype is not None else torch.from_numpy(a.copy())


def _opt(name, key, dtype=None):
    full = f"{name}/{key}"
    return _get(full, dtype) if full in VEC.files else None


def _same(a, b):
    return a.dtype == b.dtype and parity.bits_equal(a, b)


# ------------------------------------------------------------------------------------------------ CPU
@pytest.mark.parametrize("name", list(QUANT))
def test_oracles_reproduce_codec_vectors(name):
    dtype, signed, sqrt, softsign = QUANT[name]
    x = _get(f"{name}/x", dtype)
    for quantize, dequantize in ((C.quantize, C.dequantize), (T.quantize_ref, T.dequantize_ref)):
        codes, scales = quantize(x, signed, sqrt, softsign)
        assert _same(codes, _get(f"{name}/codes")) and _same(scales, _get(f"{name}/scales", torch.float16))
        assert _same(dequantize(codes, scales, signed, sqrt, softsign), _get(f"{name}/dequant"))


@pytest.mark.parametrize("name", list(ECCS))
def test_oracles_reproduce_ecc_vectors(name):
    narrow_dt, ecc_dt = ECCS[name]
    x, narrow, ecc = _get(f"{name}/x"), _get(f"{name}/narrow", narrow_dt), _get(f"{name}/ecc")
    assert _same(x.to(narrow_dt), narrow)
    assert _same(C.ecc_split(x, narrow, ecc_dt), ecc) and _same(T.ecc_split_ref(x, narrow, ecc_dt), ecc)
    assert _same(C.ecc_join(narrow, ecc), _get(f"{name}/joined")) and _same(T.ecc_join_ref(narrow, ecc), _get(f"{name}/joined"))


def _adam_inputs(name, dt, quantized):
    dtype = G.DT[dt]
    sd = None if quantized else dtype
    return dict(p=_get(f"{name}/in/p", dtype), g=_get(f"{name}/in/g", dtype), ecc=_opt(name, "in/ecc"),
                m=_get(f"{name}/in/m", sd), ms=_opt(name, "in/ms", torch.float16),
                v=_get(f"{name}/in/v", sd), vs=_opt(name, "in/vs", torch.float16))


def _expected(name, dt, quantized, keys):
    dtype = G.DT[dt]
    sd = None if quantized else dtype
    kinds = dict(p=dtype, ecc=None, m=sd, ms=torch.float16, v=sd, vs=torch.float16)
    return {k: _opt(name, f"out/{k}", kinds[k]) for k in keys}


@pytest.mark.parametrize("name,dt,ec,quantized,decoupled", G.ADAM_CASES)
def test_oracles_reproduce_adam_vectors(name, dt, ec, quantized, decoupled):
    want = _expected(name, dt, quantized, ("p", "ecc", "m", "ms", "v", "vs"))
    hp = G.ADAM_HP
    wd = 0.01 * hp["lr"] if decoupled else 0.01
    a = _adam_inputs(name, dt, quantized)
    C.adam_step(a["m"], a["ms"], a["v"], a["vs"], a["p"], a["g"], a["ecc"], hp["lr"], hp["beta1"], hp["beta2"], hp["eps"], wd,
                decoupled, 3, quantized=quantized)
    for k, w in want.items():
        assert w is None or _same(a[k], w), (name, "C oracle", k)
    b = _adam_inputs(name, dt, quantized)
    mom = T.MomentState(b["m"], b["ms"]) if quantized else T.MomentState(plain=b["m"])
    var = T.MomentState(b["v"], b["vs"]) if quantized else T.MomentState(plain=b["v"])
    T.adam_step_ref(mom, var, b["p"], b["g"], b["ecc"], hp["lr"], hp["beta1"], hp["beta2"], hp["eps"], wd, decoupled, 3)
    for k, w in want.items():
        assert w is None or _same(b[k], w), (name, "torch oracle", k)


def _mom_inputs(name, dt, quantized):
    dtype = G.DT[dt]
    return dict(p=_get(f"{name}/in/p", dtype), g=_get(f"{name}/in/g", dtype), ecc=_get(f"{name}/in/ecc"),
                m=_get(f"{name}/in/m", None if quantized else dtype), ms=_opt(name, "in/ms", torch.float16))


@pytest.mark.parametrize("name,dt,ec,quantized,kw", G.MOM_CASES)
def test_oracles_reproduce_momentum_vectors(name, dt, ec, quantized, kw):
    want = _expected(name, dt, quantized, ("p", "ecc", "m", "ms"))
    a = _mom_inputs(name, dt, quantized)
    C.momentum_step(a["m"], a["ms"], a["p"], a["g"], a["ecc"], quantized=quantized, **kw)
    for k, w in want.items():
        assert w is None or _same(a[k], w), (name, "C oracle", k)
    b = _mom_inputs(name, dt, quantized)
    mom = T.MomentState(b["m"], b["ms"]) if quantized else T.MomentState(plain=b["m"])
    T.momentum_step_ref(mom, b["p"], b["g"], b["ecc"], **kw)
    for k, w in want.items():
        assert w is None or _same(b[k], w), (name, "torch oracle", k)


# ------------------------------------------------------------------------------------------------ GPU
def _dev(t):
    return None if t is None else t.to(DEV)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(QUANT))
def test_hip_codec_matches_vectors(name):
    from flashoptim_amd import kernels as k

    dtype, signed, sqrt, softsign = QUANT[name]
    codes, scales = k.quantize(_get(f"{name}/x", dtype).to(DEV), signed=signed, sqrt=sqrt, softsign=softsign)
    assert _same(codes.cpu(), _get(f"{name}/codes")) and _same(scales.cpu(), _get(f"{name}/scales", torch.float16))
    back = k.dequantize(codes, scales, signed=signed, sqrt=sqrt, softsign=softsign)
    assert _same(back.cpu(), _get(f"{name}/dequant"))


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(ECCS))
def test_hip_ecc_matches_vectors(name):
    from flashoptim_amd import kernels as k

    narrow_dt, ecc_dt = ECCS[name]
    x, narrow = _get(f"{name}/x").to(DEV), _get(f"{name}/narrow", narrow_dt).to(DEV)
    ecc = k.compute_ecc_bits(x, narrow, 3 if ecc_dt == torch.int8 else 4)
    assert _same(ecc.cpu(), _get(f"{name}/ecc"))
    assert _same(k.reconstruct_fp32_param(narrow, ecc).cpu(), _get(f"{name}/joined"))


def _check_step(name, got, want, state_names, exact):
    """Moments, codes and scales: every bit equals the committed vector.  exact: parameters and ECC too (every kernel
    but Adam with the guarded folded update, whose master weights stay within one unit of master precision)."""
    for key in tuple(k for pair in state_names for k in pair):
        if want.get(key) is not None:
            assert parity.bits_equal(got[key], want[key]), f"{name} {key}: bits differ"
    if exact:
        for key in ("p", "ecc"):
            if want.get(key) is not None:
                assert parity.bits_equal(got[key], want[key]), f"{name} {key}: bits differ"
        return
    parity.check_master(got["p"], got["ecc"], want["p"], want["ecc"], name)


@pytest.mark.gpu
@pytest.mark.parametrize("name,dt,ec,quantized,decoupled", G.ADAM_CASES)
def test_hip_adam_step_matches_vectors(name, dt, ec, quantized, decoupled):
    from flashoptim_amd import kernels as k

    want = _expected(name, dt, quantized, ("p", "ecc", "m", "ms", "v", "vs"))
    hp = G.ADAM_HP
    wd = 0.01 * hp["lr"] if decoupled else 0.01
    a = {key: _dev(t) for key, t in _adam_inputs(name, dt, quantized).items()}
    k._fused_adam_step(a["m"], a["ms"], a["v"], a["vs"], a["p"], a["g"], a["ecc"], hp["lr"], hp["beta1"], hp["beta2"], hp["eps"],
                       wd, decoupled, 3, quantize_optim_states=quantized)
    folded = dt != "f32" and (ec == "none" or (dt == "bf16" and ec == "i8"))  # the guarded folded update
    _check_step(name, a, want, (("m", "ms"), ("v", "vs")), exact=not folded)


@pytest.mark.gpu
@pytest.mark.parametrize("name,dt,ec,quantized,kw", G.MOM_CASES)
def test_hip_momentum_step_matches_vectors(name, dt, ec, quantized, kw):
    from flashoptim_amd import kernels as k

    want = _expected(name, dt, quantized, ("p", "ecc", "m", "ms"))
    a = {key: _dev(t) for key, t in _mom_inputs(name, dt, quantized).items()}
    k._fused_momentum_step(a["m"], a["ms"], a["p"], a["g"], a["ecc"], quantize_optim_states=quantized, **kw)
    _check_step(name, a, want, (("m", "ms"),), exact=True)
