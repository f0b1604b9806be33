"""Shared helpers of the parity tests: the checks between the HIP path (or its CPU build) and the CPU oracle.

What the kernels promise (flashoptim_amd/csrc/fo_math.h) and what the tests therefore assert, every step, from
identical inputs, with no allowance beyond the stated bar:
* SGD / SGDW / Nesterov / Lion steps, the momentum-free SGD step, the standalone codec and ECC kernels, and Adam
  wherever the update follows the reference operation by operation -- fp32 parameters, 2-byte parameters with a
  2-byte ECC (32-bit masters), fp16 parameters with a 1-byte ECC, any variant through the `*_exact` entry points:
  every output bit equals the oracle's (`bits_equal`);
* Adam with the guarded folded update -- bf16 parameters with a 1-byte ECC (24-bit masters), bf16 / fp16
  parameters without ECC:
  - moment codes and fp16 group scales: every bit equals the oracle's (the moments are formed operation by
    operation and the requantiser's quick forms are verified value by value);
  - master weights (narrow parameter + ECC code, `master_value`): within one unit of master precision, i.e.
    half-ulp(narrow) / 127 for 24-bit masters and one ulp of the narrow type without ECC (`check_master`);
  - narrow parameters: within one ulp of their dtype.
"""

from __future__ import annotations

import torch

from oracle import torch_oracle as T

CODE_MISMATCH_FRACTION = 1e-4   # the bar of the specification (0.01 % of all elements at +-1); the kernels deliver 0
SCALE_MISMATCH_FRACTION = 1e-3


def check_codes(gpu: torch.Tensor, ref: torch.Tensor, what: str, limit: float = CODE_MISMATCH_FRACTION) -> float:
    """Codes never differ by more than one step and fewer than `limit` of them differ.  Returns the mismatch
    fraction."""
    g = gpu.cpu().to(torch.int32).reshape(-1)
    r = ref.to(torch.int32).reshape(-1)
    if g.numel() == 0:
        return 0.0
    diff = (g - r).abs()
    assert int(diff.max()) <= 1, f"{what}: code differs by {int(diff.max())} steps"
    count = int((diff != 0).sum())
    frac = count / g.numel()
    # tensors shorter than 1/limit: a single flip is tolerated
    assert frac < limit or count <= 1, f"{what}: {frac:.3e} of codes differ"
    return frac


def check_scales(gpu: torch.Tensor, ref: torch.Tensor, what: str) -> float:
    g = gpu.cpu().view(torch.int16).to(torch.int32).reshape(-1)
    r = ref.view(torch.int16).to(torch.int32).reshape(-1)
    diff = (g - r).abs()
    assert int(diff.max() if diff.numel() else 0) <= 1, f"{what}: scale differs by {int(diff.max())} fp16 ulps"
    frac = float((diff != 0).float().mean()) if diff.numel() else 0.0
    assert frac < SCALE_MISMATCH_FRACTION or int((diff != 0).sum()) <= 1, f"{what}: {frac:.3e} of scales differ"
    return frac


def ulp_of(x: torch.Tensor) -> torch.Tensor:
    """ulp of each element in its own dtype (min-normal spacing for zero/subnormal), as float64."""
    mant = {torch.float32: 23, torch.bfloat16: 7, torch.float16: 10}[x.dtype]
    return torch.exp2((T.unbiased_exponent(x) - mant).double())


def master_unit(param: torch.Tensor, ecc) -> torch.Tensor:
    """One unit of master precision at each narrow value: one step of its correction code,
    2^(E - mant - 1) / MAX (ref: /root/reference/flashoptim/optimizers.py:2759-2776), or one ulp of the narrow type
    where there is no code."""
    if ecc is None:
        return ulp_of(param)
    return ulp_of(param) * 0.5 / (127.0 if ecc.dtype == torch.int8 else 32767.0)


def master_value(param: torch.Tensor, ecc) -> torch.Tensor:
    """The master weight a (narrow value, correction code) pair stands for, narrow + code * unit, in float64 (exact to
    2^-53: the pair itself is compared, not one particular fp32 rounding of its reconstruction)."""
    if ecc is None:
        return param.double()
    return param.double() + ecc.double() * master_unit(param, ecc)


def master_difference(param_gpu, ecc_gpu, param_ref, ecc_ref):
    """Per element: (difference of the narrow parameters in ulps of the narrow type, difference of the master weights
    in units of master precision).  Where the two narrow values lie in different binades (one side rounded up to a
    power of two, the other stayed below it) their units differ by a factor of two and the coarser one is the
    measure.  Values that are the same infinity, or NaN on both sides, count as equal."""
    pg = param_gpu.cpu().reshape(-1)
    eg = None if ecc_gpu is None else ecc_gpu.cpu().reshape(-1)
    pr = param_ref.reshape(-1)
    er = None if ecc_ref is None else ecc_ref.reshape(-1)
    zero = torch.zeros((), dtype=torch.float64)
    agree = (pg == pr) | (torch.isnan(pg) & torch.isnan(pr))
    narrow = torch.where(agree, zero, (pg.double() - pr.double()).abs() / torch.maximum(ulp_of(pr), ulp_of(pg)))
    m_ref, m_gpu = master_value(pr, er), master_value(pg, eg)
    agree = (m_gpu == m_ref) | (torch.isnan(m_gpu) & torch.isnan(m_ref))
    master = torch.where(agree, zero, (m_gpu - m_ref).abs() / torch.maximum(master_unit(pr, er), master_unit(pg, eg)))
    return narrow, master


def check_master(param_gpu, ecc_gpu, param_ref, ecc_ref, what: str):
    """Narrow parameter within one ulp of its dtype; master weight within one unit of master precision; no
    allowance beyond the 1e-9 that float64 arithmetic needs.
    Returns (largest master difference in units, fraction of elements whose master weights differ at all)."""
    if param_ref.numel() == 0:
        return 0.0, 0.0
    narrow, master = master_difference(param_gpu, ecc_gpu, param_ref, ecc_ref)
    assert float(narrow.max()) <= 1.0 + 1e-9, f"{what}: narrow parameter off by {float(narrow.max()):.3f} ulps"
    worst = float(master.max())
    assert worst <= 1.0 + 1e-9, f"{what}: master weight off by {worst:.3f} units of master precision"
    return worst, float((master != 0).double().mean())


def bits_equal(a: torch.Tensor, b: torch.Tensor) -> bool:
    if a.dtype != b.dtype or a.shape != b.shape:
        return False
    return torch.equal(a.cpu().contiguous().reshape(-1).view(torch.uint8), b.cpu().contiguous().reshape(-1).view(torch.uint8))
