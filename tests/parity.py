"""Shared helpers of the GPU parity tests: tolerance checks between the HIP path and the CPU oracle.

What the kernels promise (flashoptim_amd/csrc/fo_math.h) and what the tests therefore assert, every step, from
identical inputs:
* SGD / SGDW / Nesterov / Lion steps, the momentum-free SGD step, Adam with fp32 parameters, unquantised states, the
  standalone codec and the standalone ECC kernels: every output bit equals the oracle's (`bits_equal`);
* Adam with fp16 parameters (folded update, unfolded moments): codes and scales bit-exact, master weights and
  narrow parameters as in the next item;
* Adam with bf16 parameters (folded update and moments): the new moments come out of fused multiply-adds and may
  differ from the oracle's by an ulp (the requantiser itself yields the exact forms' codes: its quick forms are
  verified value by value), so
  - 8-bit moment codes never differ by more than +-1 code step and differ on fewer than 0.01 % of the elements
    (measured 1e-6 .. 2.5e-5; exactly 0 on a first step from zero states and in any group that starts from zero,
    where m and v are formed identically);
  - fp16 group scales: equal, or one fp16 ulp apart on fewer than 0.1 % of the groups;
  - master weights (narrow parameter + ECC): within one unit of master precision, i.e. half-ulp(narrow)/127 for
    24-bit, /32767 for 32-bit masters; plus one fp32 ulp (the updated value is rounded to fp32 before it is
    split); plus 2^-19 (16 fp32 ulps) of the size of the update just applied, because the folded update
    m / (sqrt(v) c1 + c2) and the reference's lr (m/bc1) / (sqrt(v/bc2) + eps) round at different places and for
    weights smaller than the step that difference exceeds the weight's own ulp.  `check_master` also returns the
    fraction of elements beyond one unit with no allowance at all, which the tests print;
  - narrow parameters: within one ulp of their dtype.
"""

from __future__ import annotations

import torch

from oracle import torch_oracle as T

CODE_MISMATCH_FRACTION = 1e-4   # 0.01 %, of all elements, on every step
SCALE_MISMATCH_FRACTION = 1e-3
STEP_REL_TOL = 2.0 ** -19       # 16 fp32 ulps of the size of the update (folded Adam update only)


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


def master_value(param: torch.Tensor, ecc) -> torch.Tensor:
    return (param.float() if ecc is None else T.ecc_join_ref(param, ecc)).double()


def check_master(param_gpu, ecc_gpu, param_ref, ecc_ref, what: str, step_size=None):
    """Narrow parameter within one ulp of its dtype; master weight within one unit of master precision plus one
    fp32 ulp plus STEP_REL_TOL of the size of the update just applied (`step_size` = the oracle's update_scale).
    Returns (largest master error as a fraction of the allowance, fraction of elements beyond one unit with no
    allowance)."""
    pg = param_gpu.cpu().reshape(-1)
    eg = None if ecc_gpu is None else ecc_gpu.cpu().reshape(-1)
    pr = param_ref.reshape(-1)
    er = None if ecc_ref is None else ecc_ref.reshape(-1)
    if pr.numel() == 0:
        return 0.0, 0.0
    slack = 0.0 if step_size is None else step_size.reshape(-1).double() * STEP_REL_TOL
    # identical values agree, also where they are the same infinity or both NaN (an update that overflows the
    # narrow dtype overflows it on both sides; inf - inf would otherwise read as a mismatch)
    agree = (pg == pr) | (torch.isnan(pg) & torch.isnan(pr))
    nd = torch.where(agree, torch.zeros((), dtype=torch.float64), (pg.double() - pr.double()).abs())
    assert bool((agree | (nd <= ulp_of(pr) * 1.0000001 + slack)).all()), f"{what}: narrow parameter off by more than one ulp"
    m_ref = master_value(pr, er)
    ulp32 = ulp_of(m_ref.float())
    if er is None:
        allowed = ulp_of(pr) + slack
        unit = ulp_of(pr)
    else:
        # one step of the correction code, plus one fp32 ulp: the updated master is rounded to fp32 before it
        # is split, so two implementations can enter the split one fp32 ulp apart
        unit = ulp_of(pr) * 0.5 / (127.0 if er.dtype == torch.int8 else 32767.0)
        allowed = unit + ulp32 + slack
    m_gpu = master_value(pg, eg)
    agree = (m_gpu == m_ref) | (torch.isnan(m_gpu) & torch.isnan(m_ref))
    md = torch.where(agree, torch.zeros((), dtype=torch.float64), (m_gpu - m_ref).abs())
    allowed = torch.where(agree, torch.ones((), dtype=torch.float64), allowed + torch.zeros_like(md))
    worst = float(torch.where(agree, torch.zeros((), dtype=torch.float64), md / allowed).max())
    assert worst <= 1.0000001, f"{what}: master weight off by {worst:.3f} x the allowance ({float((md / unit).max()):.2f} units)"
    beyond_unit = float((md > unit * 1.0000001).double().mean())
    return worst, beyond_unit


def bits_equal(a: torch.Tensor, b: torch.Tensor) -> bool:
    if a.dtype != b.dtype or a.shape != b.shape:
        return False
    return torch.equal(a.cpu().contiguous().reshape(-1).view(torch.uint8), b.cpu().contiguous().reshape(-1).view(torch.uint8))
