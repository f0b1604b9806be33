"""CPU restatement (pure PyTorch, IEEE fp32, no FMA contraction) of FlashOptim's fused step math.

THIS IS TEST INFRASTRUCTURE.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it.  The product (``flashoptim_amd``) never does:
its only implementation is the HIP library and it raises when that library is missing.

Every function cites the lines of ``/root/reference/flashoptim/optimizers.py`` (abbreviated
``ref:``) it restates.  All arithmetic is fp32 with one rounding per written operation, in the same
order and association as the reference kernels.  Kernel scalars are rounded double -> fp32 first
because Triton passes Python floats as fp32, and ``1.0 - beta`` style expressions are evaluated in
fp32 (ref:1667-1675, ref:2357-2364).

Parity status
-------------
* The reference GPU kernels use Triton's approximate ``fdiv``, fast ``sqrt``, FMA contraction and a
  vendor ``pow(f32, i32)``; no environment available to this project can produce their bit-level
  output and the reference holds no golden vectors for them.  Bit-level parity with the Triton
  kernels is therefore **unpinned**; tolerance-level parity (codes +-1 step on < 0.01 % of
  elements, 1 master-ulp, 1 bf16 ulp) is what the tests check.
* What *is* pinned (tests/test_oracle_*.py): Adam/AdamW/SGD update math against ``torch.optim``
  with codec and ECC bypassed; Lion / SGDW / decouple_lr against the textbook recurrences; the
  group codec and the ECC split/join against hand-derived known answers, the reference tests'
  invariants and brute force over all codes; this file against the independent scalar C restatement
  in ``oracle/fo_oracle.c`` bit for bit.
* ``bias_correction = 1 - beta**step``: the reference evaluates ``pow`` in fp32 with a vendor
  routine (ref:2368-2369).  Here (and in the C restatement and in the HIP library) ``beta**step`` is
  the correctly rounded fp32 value of the power of the fp32 ``beta`` (computed in double), then
  ``1.0f - that`` in fp32.  This can differ from the vendor ``pow`` by an ulp of the power.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

GROUP_SIZE = 32  # ref:1549, 2219, 2451, 2506

_MANTISSA_BITS = {torch.float16: 10, torch.bfloat16: 7, torch.float32: 23}  # ref:54-58
_EXP_BIAS = {torch.float16: 15, torch.bfloat16: 127, torch.float32: 127}  # ref:2691-2699


def f32(x: float) -> float:
    """Round a Python double to fp32 and return it as a (now exactly representable) double."""
    return float(np.float32(x))


def _pow2(k: torch.Tensor) -> torch.Tensor:
    """Exact 2**k (fp32) for an int32 tensor with -126 <= k <= 127, built from the exponent field."""
    if k.numel():
        assert int(k.min()) >= -126 and int(k.max()) <= 127
    return ((k.to(torch.int32) + 127) << 23).view(torch.float32)


def _sqrt_rn(x: torch.Tensor) -> torch.Tensor:
    """Correctly rounded fp32 square root.

    ``torch.sqrt`` on large CPU tensors is routed to a vector math library whose result is not
    always the correctly rounded one (about 0.7 % of elements differ by an ulp), so the root is
    taken in fp64 and rounded once more; for square roots that double rounding is innocuous.
    """
    return torch.sqrt(x.to(torch.float64)).to(torch.float32)


def _group_view(x: torch.Tensor) -> tuple[torch.Tensor, int]:
    """Flatten and zero-pad to whole groups -> [G, 32].  Out-of-range lanes read 0 (ref:2640-2646)."""
    flat = x.reshape(-1)
    n = flat.numel()
    g = (n + GROUP_SIZE - 1) // GROUP_SIZE
    if g * GROUP_SIZE != n:
        flat = torch.cat([flat, flat.new_zeros(g * GROUP_SIZE - n)])
    return flat.view(g, GROUP_SIZE), n


# --------------------------------------------------------------------------------------------
# group codec (ref:2541-2676 standalone kernels; same math inlined at ref:1643-1657, 1697-1716,
# 2314-2348, 2390-2434)
# --------------------------------------------------------------------------------------------


def quantize_groups(
    x_f32: torch.Tensor, signed: bool, sqrt: bool, softsign: bool
) -> tuple[torch.Tensor, torch.Tensor]:
    """fp32 values -> (codes int8|uint8 [n], fp32 absmax per group [G]).

    ref:2647-2671: optional sqrt, absmax clamped at 1e-12, divide by the *fp32* absmax, optional
    softsign ``2x/(1+|x|)``, ``floor(v*OUT_MAX + 0.5)`` and a cast to the integer type.
    """
    assert x_f32.dtype == torch.float32
    groups, n = _group_view(x_f32)
    if sqrt:
        groups = _sqrt_rn(groups)
    # tl.max / tl.maximum (ref:2657-2658) are NaN-ignoring reductions (Triton's default): a NaN element does not
    # poison its group's scale
    mags = groups.abs()
    absmax = torch.where(torch.isnan(mags), torch.zeros_like(mags), mags).amax(dim=1).clamp_min(f32(1e-12))
    normalized = groups / absmax[:, None]
    if softsign:
        transformed = (2.0 * normalized) / (1.0 + normalized.abs())
    else:
        transformed = normalized
    out_max = 127.0 if signed else 255.0
    q = torch.floor(transformed * out_max + 0.5)
    # The cast follows the hardware convention for the values that can occur here (|q| <= OUT_MAX);
    # NaN inputs are outside the parity contract.
    codes = q.to(torch.int32).to(torch.int8 if signed else torch.uint8)
    return codes.reshape(-1)[:n], absmax


def quantize_ref(
    x: torch.Tensor, signed: bool = True, sqrt: bool = False, softsign: bool = True
) -> tuple[torch.Tensor, torch.Tensor]:
    """``quantize`` (ref:2446-2498): codes with x's shape, scales fp16[ceil(N/32)] (RTNE cast on
    store through the fp16 pointer, ref:2676)."""
    codes, absmax = quantize_groups(x.to(torch.float32), signed, sqrt, softsign)
    return codes.view(x.shape), absmax.to(torch.float16)


def dequantize_ref(
    codes: torch.Tensor,
    scales_f16: torch.Tensor,
    signed: bool = True,
    sqrt: bool = False,
    softsign: bool = True,
) -> torch.Tensor:
    """``dequantize`` (ref:2501-2538, kernel ref:2584-2607): ``q/IN_MAX``, inverse softsign
    ``y/(2-|y|)``, times the fp16 scale (upcast), square if sqrt."""
    in_max = 127.0 if signed else 255.0
    groups, n = _group_view(codes.to(torch.float32))
    g = groups.shape[0]
    assert scales_f16.numel() >= g
    transformed = groups / in_max
    if softsign:
        normalized = transformed / (2.0 - transformed.abs())
    else:
        normalized = transformed
    x = normalized * scales_f16.reshape(-1)[:g].to(torch.float32)[:, None]
    if sqrt:
        x = x * x
    return x.reshape(-1)[:n].view(codes.shape)


# --------------------------------------------------------------------------------------------
# ECC split / join (ref:2682-2776)
# --------------------------------------------------------------------------------------------


def unbiased_exponent(x_narrow: torch.Tensor) -> torch.Tensor:
    """ref:2682-2712: biased exponent field of |x|; zero/subnormal use the min-normal exponent."""
    mant = _MANTISSA_BITS[x_narrow.dtype]
    bias = _EXP_BIAS[x_narrow.dtype]
    if x_narrow.dtype == torch.float32:
        bits = x_narrow.abs().view(torch.int32)
    else:
        bits = x_narrow.abs().view(torch.int16).to(torch.int32) & 0xFFFF
    e = bits >> mant
    return torch.where(e == 0, torch.full_like(e, 1 - bias), e - bias)


def _log_scale(x_narrow: torch.Tensor) -> torch.Tensor:
    """ref:2715-2723, 2744, 2769: log2 of half the ulp of the narrow value."""
    return unbiased_exponent(x_narrow) - _MANTISSA_BITS[x_narrow.dtype] - 1


def _ecc_max(ecc_dtype: torch.dtype) -> float:
    return {torch.int8: 127.0, torch.int16: 32767.0}[ecc_dtype]  # ref:1519-1523


def ecc_join_ref(x_narrow: torch.Tensor, ecc: torch.Tensor) -> torch.Tensor:
    """``_apply_error_correction`` / ``reconstruct_fp32_param`` (ref:2759-2776, 2835-2892)."""
    ls = _log_scale(x_narrow)
    h = torch.div(ls, 2, rounding_mode="floor")
    c = ecc.to(torch.float32) / _ecc_max(ecc.dtype)
    # The last product and the sum form one fused multiply-add.  The reference compiles with FP fusion
    # on, and only the fused form stays inside the exception budgets its own invariants test records
    # for the binades 2^-125 .. 2^-113, where c * 2^ls is an fp32 subnormal
    # (/root/reference/test/test_ecc_invariants.py:257-262).  Evaluated in fp64 the product and the sum
    # are exact (at most 8 + 1 + 15 + 24 significant bits), so the single rounding to fp32 is the fma's.
    t = (c * _pow2(h)).to(torch.float64)
    return (t * _pow2(ls - h).to(torch.float64) + x_narrow.to(torch.float64)).to(torch.float32)


def ecc_split_ref(
    x_f32: torch.Tensor, x_narrow: torch.Tensor, ecc_dtype: torch.dtype
) -> torch.Tensor:
    """``_compute_ecc_bits`` / ``compute_ecc_bits`` (ref:2726-2756, 2895-2970)."""
    assert x_f32.dtype == torch.float32
    err = x_f32 - x_narrow.to(torch.float32)
    nls = -_log_scale(x_narrow)
    h = torch.div(nls, 2, rounding_mode="floor")
    en = (err * _pow2(h)) * _pow2(nls - h)
    scaled = en.clamp(-1.0, 1.0) * _ecc_max(ecc_dtype)
    rounded = torch.copysign(torch.floor(scaled.abs() + 0.5), scaled)
    return rounded.to(torch.int32).to(ecc_dtype)


# --------------------------------------------------------------------------------------------
# fused steps
# --------------------------------------------------------------------------------------------


def pow_f32(base_f32: float, step: int) -> float:
    """Correctly rounded fp32 value of base**step (see the module docstring)."""
    return f32(math.pow(base_f32, int(step)))


@dataclass
class MomentState:
    """One optimizer state of one tensor: 8-bit codes + fp16 scales, or a plain tensor at the
    parameter dtype when quantisation is off (ref:2435-2438, 1717-1719)."""

    codes: Optional[torch.Tensor] = None  # int8 / uint8, flat
    scales: Optional[torch.Tensor] = None  # fp16 [G]
    plain: Optional[torch.Tensor] = None  # param dtype, flat

    @property
    def quantized(self) -> bool:
        return self.plain is None

    @staticmethod
    def zeros(n: int, signed: bool, quantized: bool, dtype: torch.dtype) -> "MomentState":
        # State init quantises a zero tensor: codes 0, scale fp16(1e-12) == 0 (ref:1006-1013).
        if quantized:
            g = (n + GROUP_SIZE - 1) // GROUP_SIZE
            return MomentState(
                codes=torch.zeros(n, dtype=torch.int8 if signed else torch.uint8),
                scales=torch.zeros(g, dtype=torch.float16),
            )
        return MomentState(plain=torch.zeros(n, dtype=dtype))

    def clone(self) -> "MomentState":
        c = lambda t: None if t is None else t.clone()
        return MomentState(c(self.codes), c(self.scales), c(self.plain))


def _load_state(s: MomentState, signed: bool, sqrt: bool, softsign: bool) -> torch.Tensor:
    if s.quantized:
        return dequantize_ref(s.codes, s.scales, signed=signed, sqrt=sqrt, softsign=softsign)
    return s.plain.to(torch.float32)


def _store_state(
    s: MomentState, x: torch.Tensor, signed: bool, sqrt: bool, softsign: bool
) -> None:
    if s.quantized:
        codes, absmax = quantize_groups(x, signed, sqrt, softsign)
        s.codes.copy_(codes)
        s.scales[: absmax.numel()].copy_(absmax.to(torch.float16))
    else:
        s.plain.copy_(x.to(s.plain.dtype))


def _read_master(param: torch.Tensor, ecc: Optional[torch.Tensor]) -> torch.Tensor:
    if ecc is not None:
        return ecc_join_ref(param, ecc)  # ref:2300-2307
    return param.to(torch.float32, copy=True)  # ref:2308-2309 (a copy, so the caller keeps the value from before the step)


def _write_master(param: torch.Tensor, ecc: Optional[torch.Tensor], p: torch.Tensor) -> None:
    narrow = p.to(param.dtype)  # RTNE, ref:2377-2378
    param.copy_(narrow)
    if ecc is not None:
        ecc.copy_(ecc_split_ref(p, narrow, ecc.dtype))  # ref:2379-2387


def adam_step_ref(
    mom: MomentState,
    var: MomentState,
    param: torch.Tensor,
    grad: torch.Tensor,
    ecc: Optional[torch.Tensor],
    lr: float,
    beta1: float,
    beta2: float,
    eps: float,
    weight_decay: float,
    decoupled: bool,
    step: int,
) -> dict:
    """``_triton_adam_kernel`` (ref:2255-2438) on flat, contiguous CPU tensors, in place.

    ``weight_decay`` is what the launcher passes: already multiplied by lr (or lr/initial_lr) in
    double for the decoupled optimizers (ref:1894-1898).

    Returns the fp32 intermediates a parity test needs to tell a genuine difference from a rounding
    coin-flip: the master before and after the update and the moments before requantisation.
    """
    lr, b1, b2, eps, wd = f32(lr), f32(beta1), f32(beta2), f32(eps), f32(weight_decay)
    one_m_b1 = f32(np.float32(1.0) - np.float32(b1))
    one_m_b2 = f32(np.float32(1.0) - np.float32(b2))
    one_m_wd = f32(np.float32(1.0) - np.float32(wd))
    bc1 = f32(np.float32(1.0) - np.float32(pow_f32(b1, step)))
    bc2 = f32(np.float32(1.0) - np.float32(pow_f32(b2, step)))

    g = grad.reshape(-1).to(torch.float32)  # ref:2297-2298
    p = _read_master(param.reshape(-1), None if ecc is None else ecc.reshape(-1))
    p_before = p
    if not decoupled:
        g = g + p * wd  # ref:2310-2311
    m = _load_state(mom, signed=True, sqrt=False, softsign=True)  # ref:2325-2343
    v = _load_state(var, signed=False, sqrt=True, softsign=False)  # ref:2326-2348
    m_terms = (m * b1).abs() + (g * one_m_b1).abs()  # magnitude of what is summed into m (for error scales)
    m = m * b1 + g * one_m_b1  # ref:2357
    v = v * b2 + (g * g) * one_m_b2  # ref:2360
    if decoupled:
        p = p * one_m_wd  # ref:2363-2364
    cm = m / bc1  # ref:2370
    cv = v / bc2  # ref:2371
    denom = _sqrt_rn(cv) + eps  # ref:2374
    p = p - (lr * cm) / denom  # ref:2375
    _write_master(param.reshape(-1), None if ecc is None else ecc.reshape(-1), p)
    _store_state(mom, m, signed=True, sqrt=False, softsign=True)  # ref:2390-2434
    _store_state(var, v, signed=False, sqrt=True, softsign=False)
    # update_scale: size of the update with the terms of m taken in magnitude, i.e. what a relative rounding
    # error of the update arithmetic scales with even when those terms cancel
    return {"p_before": p_before, "p_after": p, "m": m, "v": v, "update_scale": (lr * (m_terms / bc1)) / denom}


def momentum_step_ref(
    mom: Optional[MomentState],
    param: torch.Tensor,
    grad: torch.Tensor,
    ecc: Optional[torch.Tensor],
    lr: float,
    mom_coef: float,
    update_coef: float,
    weight_decay: float,
    decoupled: bool = False,
    nesterov: bool = False,
    do_lion: bool = False,
) -> dict:
    """``_triton_momentum_kernel`` (ref:1586-1719), in place.

    Lion: ``mom_coef = beta2``, ``update_coef = beta1`` (ref:1313-1317).  SGD: ``mom_coef =
    momentum``, ``update_coef = 1 - dampening`` (ref:1432-1433).  ``mom is None`` restates the
    momentum-free SGD branch the reference runs in eager PyTorch (ref:1447-1465): same operations
    with the buffer left out.
    """
    lr, mc, uc, wd = f32(lr), f32(mom_coef), f32(update_coef), f32(weight_decay)
    one_m_wd = f32(np.float32(1.0) - np.float32(wd))
    eccf = None if ecc is None else ecc.reshape(-1)

    g = grad.reshape(-1).to(torch.float32)  # ref:1626-1627
    p = _read_master(param.reshape(-1), eccf)  # ref:1628-1638
    p_before = p

    if mom is None:
        # ref:1452-1456: the eager branch skips both decays when weight_decay == 0.
        if not decoupled and weight_decay > 0:
            g = g + p * wd
        if decoupled and weight_decay > 0:
            p = p * one_m_wd
        p = p - g * lr
        _write_master(param.reshape(-1), eccf, p)
        return {"p_before": p_before, "p_after": p, "update_scale": (g * lr).abs()}

    if not do_lion and not decoupled:
        g = g + p * wd  # ref:1639-1640
    m = _load_state(mom, signed=True, sqrt=False, softsign=True)  # ref:1643-1661
    m_terms = (m * mc).abs() + g.abs()
    if do_lion:
        one_m_uc = f32(np.float32(1.0) - np.float32(uc))
        one_m_mc = f32(np.float32(1.0) - np.float32(mc))
        u = (m * uc) + (g * one_m_uc)  # ref:1667
        u = torch.sign(u)  # ref:1668 (0 stays 0)
        m = (m * mc) + (g * one_m_mc)  # ref:1669
        p = p * one_m_wd  # ref:1675
        p = p - u * lr  # ref:1676
    else:
        m = m * mc + g * uc  # ref:1671
        if decoupled:
            p = p * one_m_wd  # ref:1678-1679
        if nesterov:
            p = p - (g + mc * m) * lr  # ref:1680-1681
        else:
            p = p - m * lr  # ref:1682-1683
    _write_master(param.reshape(-1), eccf, p)  # ref:1684-1694
    _store_state(mom, m, signed=True, sqrt=False, softsign=True)  # ref:1697-1719
    scale = torch.full_like(p, lr) if do_lion else (m_terms + g.abs()) * lr
    return {"p_before": p_before, "p_after": p, "m": m, "update_scale": scale}
