"""Shared helpers of the GPU parity tests: tolerance checks between the HIP path and the CPU oracle.

Tolerances (stated once here, used by every parity test):
* 8-bit moment codes: never more than +-1 code step apart; differing on fewer than 0.01 % of the elements
  outside the rounding-tie band.  The band holds the elements whose exact pre-rounding value x (evaluated in
  float64 from the oracle's fp32 moments) has x + 0.5 within 8 fp32 ulps of an integer: there floor(x + 0.5) is
  decided by sub-ulp rounding noise of the divisions and the square root, which differ between the oracle
  (IEEE), this library (hardware reciprocal/sqrt) and the reference (Triton's approximate divide/sqrt).  For
  generic data the band holds ~1e-5 of the elements; on the first step from an all-zero state with bf16
  gradients it holds up to ~1 % of them, because the values are then ratios of 8-bit mantissas and land on
  rounding boundaries systematically.  Both fractions are reported by the tests;
* fp16 group scales: equal, or one fp16 ulp apart on fewer than 0.1 % of the groups (a scale is the fp16
  rounding of an fp32 absmax; it can only differ when an absmax sits on an fp16 rounding boundary);
* master weights (narrow parameter + ECC, or the fp32 parameter): within one unit of master precision,
  i.e. half-ulp(narrow)/127 for 24-bit, /32767 for 32-bit masters, one fp32 ulp for fp32 parameters; plus one
  fp32 ulp where an ECC split follows the fp32 rounding of the updated value; plus 2^-19 (16 fp32 ulps) of the
  size of the update just applied (its terms taken in magnitude), because the update term goes through a hardware reciprocal and square root
  (approximate ones in the reference as well) and for weights much smaller than the step that error exceeds the
  weight's own ulp;
* narrow parameters: within one ulp of their dtype.
"""

from __future__ import annotations

import torch

from oracle import torch_oracle as T

CODE_MISMATCH_FRACTION = 1e-4   # 0.01 %
SCALE_MISMATCH_FRACTION = 1e-3
STEP_REL_TOL = 2.0 ** -19       # 16 fp32 ulps of the size of the update
TIE_BAND_ULPS = 8.0             # a pre-rounding value this close (in fp32 ulps) to a rounding boundary is a coin-flip


def _tie_band(x64: torch.Tensor) -> torch.Tensor:
    """True where floor(x + 0.5) is decided by rounding noise: x + 0.5 lies within TIE_BAND_ULPS fp32 ulps of an
    integer.  Any two implementations of the same formula whose operations round differently (the reference's
    approximate divide and sqrt included) may land on either side there."""
    b = x64 + 0.5
    dist = (b - torch.round(b)).abs()
    return dist < TIE_BAND_ULPS * 2.0 ** -24 * x64.abs().clamp_min(1.0)


def _groups64(x: torch.Tensor):
    flat = x.reshape(-1).double()
    n = flat.numel()
    pad = (-n) % 32
    if pad:
        flat = torch.cat([flat, flat.new_zeros(pad)])
    return flat.view(-1, 32), n


def near_tie_mom(m_f32: torch.Tensor) -> torch.Tensor:
    """Coin-flip mask for first-moment codes: x = 127 * 2y/(1+|y|), y = m / absmax(group), in float64."""
    g, n = _groups64(m_f32)
    am = g.abs().amax(dim=1, keepdim=True).clamp_min(1e-12)
    y = g / am
    return _tie_band(127.0 * 2.0 * y / (1.0 + y.abs())).reshape(-1)[:n]


def near_tie_var(v_f32: torch.Tensor) -> torch.Tensor:
    """Coin-flip mask for second-moment codes: x = 255 * sqrt(v) / max(group sqrt(v)), in float64."""
    g, n = _groups64(v_f32)
    r = g.sqrt()
    av = r.amax(dim=1, keepdim=True).clamp_min(1e-12)
    return _tie_band(255.0 * r / av).reshape(-1)[:n]


def check_codes(gpu: torch.Tensor, ref: torch.Tensor, what: str, near_tie=None, limit: float = CODE_MISMATCH_FRACTION):
    """Codes never differ by more than one step; outside the coin-flip band fewer than `limit` of them differ.
    Returns (raw mismatch fraction, mismatch fraction outside the band)."""
    g = gpu.cpu().to(torch.int32).reshape(-1)
    r = ref.to(torch.int32).reshape(-1)
    if g.numel() == 0:
        return 0.0, 0.0
    diff = (g - r).abs()
    assert int(diff.max()) <= 1, f"{what}: code differs by {int(diff.max())} steps"
    bad = diff != 0
    raw = float(bad.float().mean())
    if near_tie is not None:
        bad = bad & ~near_tie.reshape(-1)
    count = int(bad.sum())
    frac = count / g.numel()
    # tensors shorter than 1/limit: a single unexplained flip is tolerated
    assert frac < limit or count <= 1, f"{what}: {frac:.3e} of codes differ outside the rounding-tie band (raw {raw:.3e})"
    return raw, frac


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


def check_master(param_gpu, ecc_gpu, param_ref, ecc_ref, what: str, step_size=None) -> float:
    """Narrow parameter within one ulp of its dtype; master weight within one unit of master precision plus
    STEP_REL_TOL of the size of the update just applied (`step_size` = the oracle's update_scale): the
    update term goes through a hardware reciprocal and square root, as it goes through approximate ones in the
    reference, and for weights much smaller than the step that error exceeds the weight's own ulp.
    Returns the largest master error as a fraction of the allowance."""
    pg = param_gpu.cpu().reshape(-1)
    eg = None if ecc_gpu is None else ecc_gpu.cpu().reshape(-1)
    pr = param_ref.reshape(-1)
    er = None if ecc_ref is None else ecc_ref.reshape(-1)
    if pr.numel() == 0:
        return 0.0
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
    return worst


def bits_equal(a: torch.Tensor, b: torch.Tensor) -> bool:
    if a.dtype != b.dtype or a.shape != b.shape:
        return False
    return torch.equal(a.cpu().contiguous().reshape(-1).view(torch.uint8), b.cpu().contiguous().reshape(-1).view(torch.uint8))
