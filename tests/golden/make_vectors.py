"""Writes tests/golden/step_vectors.npz: seeded inputs and the outputs the CPU oracle (oracle/fo_oracle.c through
oracle/c_oracle.py) produces for them, for every kernel family of the step path.

The reference ships no golden vectors for this path (its tests are tolerance and invariant tests that need a GPU),
and nothing of the reference is imported or run here.  These vectors freeze the oracle: the CPU suite checks that
both restatements (C and PyTorch) still reproduce them bit for bit, and the GPU suite checks the HIP kernels
against them with the parity tolerances, so a silent change of either side shows up as a diff of this file.

Run from the repository root:  python tests/golden/make_vectors.py
16-bit floats are stored as int16 bit patterns.
"""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import c_oracle as C  # noqa: E402

N = 1024 + 33  # 33 full groups and one group of one element
DT = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}
ECC = {"i8": torch.int8, "i16": torch.int16, "none": None}


def to_np(t: torch.Tensor) -> np.ndarray:
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().copy()
    return t.numpy().copy()


def from_np(a: np.ndarray, dtype: torch.dtype) -> torch.Tensor:
    t = torch.from_numpy(a.copy())
    return t.view(dtype) if dtype in (torch.bfloat16, torch.float16) else t


def rand(seed, scale, n=N):
    return torch.randn(n, generator=torch.Generator().manual_seed(seed)) * scale


ADAM_CASES = [  # name, dtype, ecc, quantized, decoupled
    ("adamw_bf16_i8_q", "bf16", "i8", True, True),
    ("adamw_bf16_i16_q", "bf16", "i16", True, True),
    ("adam_l2_f32_none_q", "f32", "none", True, False),
    ("adamw_f16_i8_plain", "f16", "i8", False, True),
]
MOM_CASES = [  # name, dtype, ecc, quantized, kwargs
    ("lion_bf16_i16_q", "bf16", "i16", True, dict(lr=1e-4, mom_coef=0.99, update_coef=0.9, weight_decay=1e-5, do_lion=True)),
    ("sgd_nesterov_f16_i8_plain", "f16", "i8", False, dict(lr=1e-2, mom_coef=0.9, update_coef=1.0, weight_decay=1e-4, nesterov=True)),
    ("sgdw_bf16_i8_q", "bf16", "i8", True, dict(lr=1e-2, mom_coef=0.9, update_coef=1.0, weight_decay=1e-6, decoupled=True)),
]
ADAM_HP = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8)


def state_for(dtype, quantized, signed):
    if quantized:
        return torch.zeros(N, dtype=torch.int8 if signed else torch.uint8), torch.zeros((N + 31) // 32, dtype=torch.float16)
    return torch.zeros(N, dtype=dtype), None


def main():
    out = {}
    # ---- codec
    x = rand(1, 3.0)
    for name, xx, signed, sqrt, softsign in (("quant_signed_softsign_f32", x, True, False, True),
                                              ("quant_unsigned_sqrt_bf16", x.abs().to(torch.bfloat16), False, True, False),
                                              ("quant_signed_linear_f16", (x * 0.01).to(torch.float16), True, False, False)):
        codes, scales = C.quantize(xx, signed, sqrt, softsign)
        out[f"{name}/x"], out[f"{name}/codes"], out[f"{name}/scales"] = to_np(xx), to_np(codes), to_np(scales)
        out[f"{name}/dequant"] = to_np(C.dequantize(codes, scales, signed, sqrt, softsign))
    # ---- ECC
    for name, narrow_dt, ecc_dt in (("ecc_bf16_i8", torch.bfloat16, torch.int8), ("ecc_f16_i16", torch.float16, torch.int16)):
        xf = rand(2, 1.0) * torch.exp2(torch.randint(-20, 10, (N,), generator=torch.Generator().manual_seed(3)).float())
        narrow = xf.to(narrow_dt)
        ecc = C.ecc_split(xf, narrow, ecc_dt)
        out[f"{name}/x"], out[f"{name}/narrow"], out[f"{name}/ecc"] = to_np(xf), to_np(narrow), to_np(ecc)
        out[f"{name}/joined"] = to_np(C.ecc_join(narrow, ecc))
    # ---- Adam: two warm-up steps build a non-trivial state, the third step is the recorded one
    for name, dt, ec, quantized, decoupled in ADAM_CASES:
        dtype, ecc_dt = DT[dt], ECC[ec]
        p = rand(10, 0.02).to(dtype)
        ecc = None if ecc_dt is None else torch.zeros(N, dtype=ecc_dt)
        (m, ms), (v, vs) = state_for(dtype, quantized, True), state_for(dtype, quantized, False)
        wd = 0.01 * ADAM_HP["lr"] if decoupled else 0.01
        for step in (1, 2, 3):
            g = rand(100 + step, 1e-3).to(dtype)
            if step == 3:
                for key, t in (("p", p), ("ecc", ecc), ("m", m), ("ms", ms), ("v", v), ("vs", vs), ("g", g)):
                    if t is not None:
                        out[f"{name}/in/{key}"] = to_np(t)
            C.adam_step(m, ms, v, vs, p, g, ecc, ADAM_HP["lr"], ADAM_HP["beta1"], ADAM_HP["beta2"], ADAM_HP["eps"], wd,
                        decoupled, step, quantized=quantized)
        for key, t in (("p", p), ("ecc", ecc), ("m", m), ("ms", ms), ("v", v), ("vs", vs)):
            if t is not None:
                out[f"{name}/out/{key}"] = to_np(t)
    # ---- momentum kernels
    for name, dt, ec, quantized, kw in MOM_CASES:
        dtype, ecc_dt = DT[dt], ECC[ec]
        p = rand(20, 0.02).to(dtype)
        ecc = torch.zeros(N, dtype=ecc_dt)
        m, ms = state_for(dtype, quantized, True)
        for step in (1, 2, 3):
            g = rand(200 + step, 1e-3).to(dtype)
            if step == 3:
                for key, t in (("p", p), ("ecc", ecc), ("m", m), ("ms", ms), ("g", g)):
                    if t is not None:
                        out[f"{name}/in/{key}"] = to_np(t)
            C.momentum_step(m, ms, p, g, ecc, quantized=quantized, **kw)
        for key, t in (("p", p), ("ecc", ecc), ("m", m), ("ms", ms)):
            if t is not None:
                out[f"{name}/out/{key}"] = to_np(t)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "step_vectors.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(out)} arrays, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
