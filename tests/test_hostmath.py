"""The step kernels' own arithmetic, checked on the CPU.

flashoptim_amd/csrc/fo_math.h holds the per-element functions the gfx950 kernels call (ECC join / split, the moment
requantiser, the Adam / SGD / Lion element updates).  tests/hostmath compiles the same header for the host, with
stand-ins for the few hardware instructions, and these tests hold it against the independent IEEE restatement of
the reference in oracle/ -- element for element, without a GPU.

The approximate instructions (reciprocal, reciprocal square root) are within one ulp on the hardware and correctly
rounded for 85-90 % of inputs; every test runs with the stand-ins exact and with them erring by an ulp in
pseudo-random directions (`noise`), because the results that are meant to be correctly rounded must not depend on
which way the hardware errs.
"""

import pytest
import torch

from oracle import c_oracle as C
from oracle import torch_oracle as T
from tests import parity
from tests.hostmath import binding as H

NOISE = [0, 1, 7]


@pytest.fixture(autouse=True)
def _reset_noise():
    yield
    H.set_noise(0)


def _rand(n, scale, seed):
    return torch.randn(n, generator=torch.Generator().manual_seed(seed)) * scale


def _bits(t):
    return t.contiguous().view(torch.int32)


# ------------------------------------------------------------------------------------------------ building blocks


@pytest.mark.parametrize("noise", NOISE)
def test_corrected_quotient_is_the_ieee_quotient(noise):
    """q = a * r, one residual correction: equals the correctly rounded a / b whatever the reciprocal instruction
    returns inside its one-ulp bound (up to the rare quotient that lies within 2^-22 ulp of a rounding boundary)."""
    H.set_noise(noise)
    n = 1 << 21
    for seed, (sa, sb) in enumerate([(1.0, 1.0), (1e-3, 3e-5), (1e-20, 1e-12), (3.0, 1e4)]):
        a = _rand(n, sa, 10 + seed)
        b = _rand(n, sb, 20 + seed).abs().clamp_min(1e-12 if sb < 1 else 1e-3)
        got = H.div_corrected(a, b)
        want = a / b
        bad = (_bits(got) != _bits(want))
        assert int((_bits(got) - _bits(want)).abs().max()) <= 1
        assert float(bad.float().mean()) < 5e-6, f"{float(bad.float().mean()):.2e} of quotients not correctly rounded"
    # quotients that are exactly representable, the requantiser's own cases (x / x, 0 / x, k / 2^j)
    x = _rand(4096, 1e-3, 3).abs().clamp_min(1e-12)
    assert torch.equal(H.div_corrected(x, x), torch.ones_like(x))
    assert torch.equal(H.div_corrected(torch.zeros_like(x), x), torch.zeros_like(x))


@pytest.mark.parametrize("noise", NOISE)
def test_corrected_root_is_the_ieee_root(noise):
    H.set_noise(noise)
    n = 1 << 21
    for seed, scale in enumerate([1.0, 1e-6, 1e-12, 1e8]):
        x = (_rand(n, 1.0, 30 + seed) ** 2) * scale
        got = H.sqrt_corrected(x)
        want = x.double().sqrt().float()  # the fp64 root rounded to fp32 is the correctly rounded fp32 root
        bad = _bits(got) != _bits(want)
        assert int((_bits(got) - _bits(want)).abs().max()) <= 1
        assert float(bad.float().mean()) < 5e-6
    # perfect squares and zero are exact
    k = torch.arange(0, 4096, dtype=torch.float32)
    assert torch.equal(H.sqrt_corrected(k * k), k)
    # the first step from a zero state: v = g^2 * (1 - b2) for bf16 gradients
    g = _rand(1 << 18, 1e-3, 5).bfloat16().float()
    v = (g * g) * (1.0 - torch.tensor(0.999, dtype=torch.float32))
    assert torch.equal(H.sqrt_corrected(v), v.double().sqrt().float())


def test_code_tables_hold_the_correctly_rounded_values():
    q = torch.cat([torch.arange(0, 128), torch.arange(-128, 0)]).float()  # value of byte b as int8
    y = q / 127.0
    assert torch.equal(H.softsign_table(), y / (2.0 - y.abs()))                         # ref:2332-2336, op by op
    for dt, mant in ((torch.bfloat16, 7), (torch.float16, 10)):
        table, arithmetic = H.ecc_fraction_table(dt)
        assert torch.equal(table, y * 2.0 ** -(mant + 1))                                # RN(q / 127), scaled exactly
        assert torch.equal(table, arithmetic)                                            # the two-term product form


# ------------------------------------------------------------------------------------------------ requantiser


def _first_step_moments(n, seed, scale=1e-3):
    """m and v after the first step from zero states, for bf16 gradients (ref:2357-2360)."""
    g = _rand(n, scale, seed).bfloat16().float()
    one = torch.tensor(1.0, dtype=torch.float32)
    m = g * (one - torch.tensor(0.9, dtype=torch.float32))
    v = (g * g) * (one - torch.tensor(0.999, dtype=torch.float32))
    return m, v


def _groups(x):
    return x.view(-1, 32)


@pytest.mark.parametrize("noise", NOISE)
def test_requantiser_resolves_exact_ties_like_the_reference(noise):
    """From zero states the moments are a gradient with an 8-bit mantissa times a constant, so the normalised
    values are ratios of small integers and a visible share of them sits EXACTLY on a rounding boundary k + 1/2,
    where the code is decided by how every single operation of the reference's formula rounds.  The kernels'
    requantiser must give the oracle's code for every element.  A round-half-even of a merged formula (what
    these kernels once did) fails this test by two orders of magnitude, which the last assertion shows."""
    H.set_noise(noise)
    n = 1 << 18
    m, v = _first_step_moments(n, 11)
    r = v.double().sqrt().float()
    qm_ref, sm_ref = C.quantize(m, signed=True, sqrt=False, softsign=True)
    qv_ref, sv_ref = C.quantize(v, signed=False, sqrt=True, softsign=False)
    qm = torch.empty(n, dtype=torch.int8)
    qv = torch.empty(n, dtype=torch.uint8)
    for i in range(0, n, 32):
        a, b = H.quantize_group(m[i:i + 32].contiguous(), r[i:i + 32].contiguous())
        qm[i:i + 32], qv[i:i + 32] = a, b
    assert torch.equal(qm, qm_ref) and torch.equal(qv, qv_ref)

    # the data does hold exact ties: second-moment pre-rounding values 255 * |g| / max|g| in exact arithmetic
    g = _groups(m.double())  # proportional to the gradients
    x = 255.0 * g.abs() / g.abs().amax(dim=1, keepdim=True)
    ties = ((x + 0.5) - torch.round(x + 0.5)).abs() < 1e-9
    assert float(ties.double().mean()) > 1e-3

    # what a merged, half-even formula would have produced for the second moment: rne(r * (255 / av))
    rg = _groups(r)
    merged = torch.round(rg * (255.0 / rg.amax(dim=1, keepdim=True).clamp_min(1e-12)))  # torch.round is half-even
    old_rate = float((merged.reshape(-1).to(torch.int32) != qv_ref.to(torch.int32)).double().mean())
    assert old_rate > 1e-3, "the tie data no longer separates half-even from the reference's rounding"


@pytest.mark.parametrize("noise", NOISE)
def test_quick_forms_with_verification_give_the_exact_requantisers_codes(noise):
    """Adam on bf16 parameters requantises through quick forms whose result is trusted only when it lies farther
    than a margin from every rounding boundary; a value that fails is redone with the exact form.  Whatever the
    hardware approximations return within their error bound, the codes must be the exact requantiser's, code for code:
    on continuous values, on first-step values (bf16 gradient times a constant: exact ties in bulk), on lattices of
    a few magnitudes, on sign-like data and across twelve decades of scale.  Continuous values fail the margin test
    at about 4e-4 (that is the price of the check), the adversarial kinds far more often, and none differs."""
    H.set_noise(noise)
    g = torch.Generator().manual_seed(noise + 1)
    rate = {}
    for kind in ("continuous", "first step", "lattice", "signs", "decades"):
        values = failed = 0
        for trial in range(400):
            n = 32 if trial % 3 else 19  # full and ragged groups
            z, y = torch.randn(n, generator=g), torch.randn(n, generator=g)
            if kind == "continuous":
                m, v = z * 1e-3, (y * 1e-3) ** 2
            elif kind == "first step":
                gr = (z * 1e-3).to(torch.bfloat16).float()
                m, v = gr * 0.1, gr * gr * 0.001
            elif kind == "lattice":
                gr = torch.round(z * 2) * 0.125
                m, v = gr * 0.5, gr * gr * 0.05
            elif kind == "signs":
                m = 0.5 * torch.sign(y) * 1.5 + 0.5 * torch.sign(z) * 3.0
                v = torch.full((n,), 0.45) + torch.randint(0, 3, (n,), generator=g).float()
            else:
                m = z * 10.0 ** float(torch.randint(-8, 4, (1,), generator=g))
                v = (y * 10.0 ** float(torch.randint(-8, 4, (1,), generator=g))) ** 2
            m, v = m.float().contiguous(), v.float().contiguous()
            qm_quick, qv_quick, f = H.quantize_group_from_moments(m, v, quick=True)
            qm_exact, qv_exact, _ = H.quantize_group_from_moments(m, v, quick=False)
            assert torch.equal(qm_quick, qm_exact) and torch.equal(qv_quick, qv_exact), f"{kind}, trial {trial}"
            values += 2 * n
            failed += f
        rate[kind] = failed / values
    print("share of values redone exactly:", {k: f"{r:.1e}" for k, r in rate.items()})
    assert rate["continuous"] < 2e-3 and rate["first step"] > rate["continuous"]


# ------------------------------------------------------------------------------------------------ whole steps

VARIANTS = [
    (torch.bfloat16, torch.int8), (torch.bfloat16, torch.int16), (torch.bfloat16, None),
    (torch.float16, torch.int8), (torch.float16, torch.int16), (torch.float32, None),
]


def _adam_state(n, dtype, ecc_dtype, quantized, seed):
    p = _rand(n, 0.02, seed).to(dtype)
    g8 = (n + 31) // 32
    if quantized:
        st = dict(m=torch.zeros(n, dtype=torch.int8), ms=torch.zeros(g8, dtype=torch.float16),
                  v=torch.zeros(n, dtype=torch.uint8), vs=torch.zeros(g8, dtype=torch.float16))
    else:
        st = dict(m=torch.zeros(n, dtype=dtype), ms=None, v=torch.zeros(n, dtype=dtype), vs=None)
    st.update(p=p, e=None if ecc_dtype is None else torch.zeros(n, dtype=ecc_dtype))
    return st


def _clone(st):
    return {k: None if t is None else t.clone() for k, t in st.items()}


def _adam_pair(n, dtype, ecc_dtype, quantized, decoupled, steps, exact=-1, lr=1e-3, seed=1):
    """Yields (step, kernel-math state, oracle state, size of the oracle's update) with both stepped from the
    kernel-math state of the step before, so that every comparison starts from identical inputs."""
    a = _adam_state(n, dtype, ecc_dtype, quantized, seed)
    wd = 0.01 * lr if decoupled else 0.01
    for step in range(1, steps + 1):
        g = _rand(n, 1e-3, 1000 * seed + step).to(dtype)
        b = _clone(a)
        mom = T.MomentState(b["m"], b["ms"]) if quantized else T.MomentState(plain=b["m"])
        var = T.MomentState(b["v"], b["vs"]) if quantized else T.MomentState(plain=b["v"])
        info = T.adam_step_ref(mom, var, b["p"], g, b["e"], lr, 0.9, 0.999, 1e-8, wd, decoupled, step)
        H.adam_step(a["m"], a["ms"], a["v"], a["vs"], a["p"], g, a["e"], lr, 0.9, 0.999, 1e-8, wd, decoupled, step, quantized, exact)
        yield step, a, b, info["update_scale"]


def _all_bits_equal(a, b):
    return all(a[k] is None or parity.bits_equal(a[k], b[k]) for k in a)


@pytest.mark.parametrize("noise", NOISE)
@pytest.mark.parametrize("dtype,ecc_dtype", VARIANTS)
@pytest.mark.parametrize("quantized", [True, False])
def test_adam_step_of_the_kernels_against_the_oracle(noise, dtype, ecc_dtype, quantized):
    """fp32 parameters: every bit of every output equals the oracle's.  bf16 parameters (folded update and moments):
    codes within +-1 on < 0.01 % of elements on every step and identical on the first, scales and master weights
    within the tolerances of tests/parity.py.  fp16 parameters (folded update, unfolded moments): codes and scales
    bit-exact, master weights within tolerance.  Unquantised states bit-exact."""
    H.set_noise(noise)
    for n, decoupled in ((1, True), (33, False), (4097, True), ((1 << 16) + 17, True)):
        for step, a, b, upd in _adam_pair(n, dtype, ecc_dtype, quantized, decoupled, steps=4):
            what = f"adam {dtype} ecc={ecc_dtype} q={quantized} n={n} step={step}"
            if dtype == torch.float32:
                assert _all_bits_equal(a, b), what
                continue
            parity.check_master(a["p"], a["e"], b["p"], b["e"], what, step_size=upd)
            if quantized and dtype == torch.float16:  # unfolded moments: codes and scales are the oracle's
                for key in ("m", "ms", "v", "vs"):
                    assert parity.bits_equal(a[key], b[key]), f"{what}: {key} differs"
            elif quantized:
                for key in ("m", "v"):
                    frac = parity.check_codes(a[key], b[key], f"{what} {key}")
                    assert step > 1 or frac == 0.0, f"{what}: first-step {key} codes differ"
                    parity.check_scales(a[key + "s"], b[key + "s"], f"{what} {key}s")
            else:
                assert parity.bits_equal(a["m"], b["m"]) and parity.bits_equal(a["v"], b["v"]), what


@pytest.mark.parametrize("noise", NOISE)
@pytest.mark.parametrize("dtype,ecc_dtype", [(torch.bfloat16, torch.int8), (torch.bfloat16, torch.int16), (torch.float16, torch.int16)])
def test_operation_by_operation_adam_update_is_bit_exact_for_narrow_parameters_too(noise, dtype, ecc_dtype):
    """The EXACT form of the update (what the kernels use for fp32 parameters) is bit-exact for every dtype: the
    folded form used for bf16 / fp16 parameters is a choice of speed, not something the arithmetic lacks."""
    H.set_noise(noise)
    for step, a, b, _ in _adam_pair((1 << 15) + 5, dtype, ecc_dtype, True, True, steps=4, exact=1):
        assert _all_bits_equal(a, b), f"{dtype} {ecc_dtype} step {step}"


@pytest.mark.parametrize("noise", NOISE)
@pytest.mark.parametrize("dtype,ecc_dtype", [(torch.bfloat16, torch.int8), (torch.float16, torch.int8), (torch.bfloat16, None), (torch.bfloat16, torch.int16)])
def test_groups_that_start_from_zero_get_the_exact_requantiser(noise, dtype, ecc_dtype):
    """After two steps some groups are reset to zero, as if they had seen no gradient yet: every code of such a group
    must equal the oracle's (there the moments are a narrow gradient times a constant and 0.3 % of them sit exactly
    on a rounding boundary, where the quick requantiser forms must give way to the exact one); all other codes may
    differ by one step on fewer than 0.01 % of the elements."""
    H.set_noise(noise)
    n = (1 << 17) + 17
    lr, wd = 1e-3, 1e-5
    a = _adam_state(n, dtype, ecc_dtype, True, seed=5)
    for step in (1, 2):
        g = _rand(n, 1e-3, 50 + step).to(dtype)
        H.adam_step(a["m"], a["ms"], a["v"], a["vs"], a["p"], g, a["e"], lr, 0.9, 0.999, 1e-8, wd, True, step)
    gen = torch.Generator().manual_seed(9)
    n_groups = a["ms"].numel()
    reset = torch.nonzero(torch.rand(n_groups, generator=gen) < 0.02).reshape(-1)
    for grp in reset.tolist():
        a["m"][grp * 32:(grp + 1) * 32] = 0
        a["v"][grp * 32:(grp + 1) * 32] = 0
        a["ms"][grp] = 0
        a["vs"][grp] = 0
    b = _clone(a)
    g = _rand(n, 1e-3, 77).to(dtype)
    T.adam_step_ref(T.MomentState(b["m"], b["ms"]), T.MomentState(b["v"], b["vs"]), b["p"], g, b["e"], lr, 0.9, 0.999, 1e-8, wd, True, 3)
    H.adam_step(a["m"], a["ms"], a["v"], a["vs"], a["p"], g, a["e"], lr, 0.9, 0.999, 1e-8, wd, True, 3)
    in_reset = torch.zeros(n_groups, dtype=torch.bool)
    in_reset[reset] = True
    in_reset = in_reset.repeat_interleave(32)[:n]
    for key in ("m", "v"):
        differs = a[key].to(torch.int32) != b[key].to(torch.int32)
        assert not bool(differs[in_reset].any()), f"{key}: a group that started from zero differs from the oracle"
        parity.check_codes(a[key][~in_reset], b[key][~in_reset], f"{key}, warm groups")


@pytest.mark.parametrize("noise", [0, 7])
def test_a_sudden_jump_of_the_gradient_scale_keeps_the_code_tolerance(noise):
    """When the gradients suddenly grow by orders of magnitude the old second moment is negligible and the new
    values sit as close to rounding boundaries as on a first step, although no scale is zero.  The kernels send
    such values through the exact requantiser form (they fail the quick forms' margin test); the quick forms alone
    miss the oracle's code on up to 0.4 % of the elements here."""
    H.set_noise(noise)
    n = 1 << 17
    for jump in (1.0, 10.0, 30.0, 100.0, 1e3, 1e5):
        a = _adam_state(n, torch.bfloat16, torch.int8, True, seed=3)
        for step in (1, 2, 3):
            g = _rand(n, 1e-4, 10 + step).to(torch.bfloat16)
            H.adam_step(a["m"], a["ms"], a["v"], a["vs"], a["p"], g, a["e"], 1e-3, 0.9, 0.999, 1e-8, 1e-5, True, step)
        b = _clone(a)
        g = _rand(n, 1e-4 * jump, 99).to(torch.bfloat16)
        T.adam_step_ref(T.MomentState(b["m"], b["ms"]), T.MomentState(b["v"], b["vs"]), b["p"], g, b["e"], 1e-3, 0.9, 0.999, 1e-8, 1e-5, True, 4)
        H.adam_step(a["m"], a["ms"], a["v"], a["vs"], a["p"], g, a["e"], 1e-3, 0.9, 0.999, 1e-8, 1e-5, True, 4)
        for key in ("m", "v"):
            parity.check_codes(a[key], b[key], f"jump {jump:g} {key}")


@pytest.mark.parametrize("betas", [(0.0, 0.999), (0.9, 0.0), (0.0, 0.0), (0.01, 0.999), (0.9, 0.1), (0.5, 0.9), (0.99, 0.9999)])
def test_code_tolerance_holds_for_unusual_betas(betas):
    """beta1 = 0 or beta2 = 0 make every step a first step for that moment (the old state has no weight, the new
    values are a narrow gradient times a constant); small betas come close."""
    H.set_noise(7)
    n = 1 << 17
    a = _adam_state(n, torch.bfloat16, torch.int8, True, seed=3)
    for step in range(1, 5):
        g = _rand(n, 1e-3, 10 + step).to(torch.bfloat16)
        b = _clone(a)
        T.adam_step_ref(T.MomentState(b["m"], b["ms"]), T.MomentState(b["v"], b["vs"]), b["p"], g, b["e"], 1e-3, betas[0], betas[1], 1e-8, 1e-5, True, step)
        H.adam_step(a["m"], a["ms"], a["v"], a["vs"], a["p"], g, a["e"], 1e-3, betas[0], betas[1], 1e-8, 1e-5, True, step)
        for key in ("m", "v"):
            parity.check_codes(a[key], b[key], f"betas {betas} step {step} {key}")


def test_master_weight_error_of_the_folded_update_without_allowance():
    """How far the folded Adam update strays from the reference's operation order, with no allowance: the share of
    master weights more than one unit of master precision away from the oracle's (weights ~N(0, 0.02), gradients
    ~N(0, 1e-3), lr 1e-3, bf16 parameters).  The differences sit where the update is as large as the weight
    itself; they do not come from the hardware approximations (same figures with exact stand-ins)."""
    n = 1 << 18
    for ecc_dtype, bound in ((torch.int8, 1e-3), (torch.int16, 6e-2)):
        for noise in (0, 7):
            H.set_noise(noise)
            worst = 0.0
            for step, a, b, upd in _adam_pair(n, torch.bfloat16, ecc_dtype, True, True, steps=3):
                _, beyond = parity.check_master(a["p"], a["e"], b["p"], b["e"], "folded", step_size=upd)
                worst = max(worst, beyond)
            print(f"bf16 + {ecc_dtype}: {worst:.2e} of master weights beyond one unit (noise {noise})")
            assert worst < bound


MOM_MODES = {
    "lion": dict(lr=1e-4, mom_coef=0.99, update_coef=0.9, weight_decay=0.1 * 1e-4, do_lion=True),
    "sgd": dict(lr=1e-2, mom_coef=0.9, update_coef=0.9, weight_decay=1e-4),
    "sgd_nesterov": dict(lr=1e-2, mom_coef=0.9, update_coef=1.0, weight_decay=1e-4, nesterov=True),
    "sgdw": dict(lr=1e-2, mom_coef=0.9, update_coef=1.0, weight_decay=1e-4 * 1e-2, decoupled=True),
}


@pytest.mark.parametrize("noise", NOISE)
@pytest.mark.parametrize("dtype,ecc_dtype", VARIANTS)
@pytest.mark.parametrize("mode", list(MOM_MODES))
def test_momentum_steps_of_the_kernels_are_bit_exact(noise, dtype, ecc_dtype, mode):
    """SGD / SGDW / Nesterov / Lion: free running for five steps, quantised and not, every bit of parameters, ECC,
    codes and scales equals the oracle's."""
    H.set_noise(noise)
    kw = MOM_MODES[mode]
    for quantized in (True, False):
        for n in (1, 33, 4097, (1 << 15) + 17):
            p = _rand(n, 0.02, 3).to(dtype)
            mk = lambda: dict(m=torch.zeros(n, dtype=torch.int8 if quantized else dtype),
                              ms=torch.zeros((n + 31) // 32, dtype=torch.float16) if quantized else None,
                              p=p.clone(), e=None if ecc_dtype is None else torch.zeros(n, dtype=ecc_dtype))
            a, b = mk(), mk()
            for step in range(1, 6):
                g = _rand(n, 1e-3, 50 + step).to(dtype)
                C.momentum_step(b["m"], b["ms"], b["p"], g, b["e"], quantized=quantized, **kw)
                H.momentum_step(a["m"], a["ms"], a["p"], g, a["e"], quantized=quantized, **kw)
                assert _all_bits_equal(a, b), f"{mode} {dtype} {ecc_dtype} q={quantized} n={n} step={step}"


@pytest.mark.parametrize("dtype,ecc_dtype", VARIANTS)
def test_plain_sgd_of_the_kernels_is_bit_exact(dtype, ecc_dtype):
    for decoupled, wd in ((False, 0.0), (False, 1e-2), (True, 1e-4)):
        n = 4099
        pa = _rand(n, 0.02, 4).to(dtype)
        pb = pa.clone()
        ea = None if ecc_dtype is None else torch.zeros(n, dtype=ecc_dtype)
        eb = None if ea is None else ea.clone()
        for step in range(1, 4):
            g = _rand(n, 1e-2, 60 + step).to(dtype)
            C.sgd_plain_step(pb, g, eb, 1e-2, wd, decoupled)
            H.sgd_plain_step(pa, g, ea, 1e-2, wd, decoupled)
            assert parity.bits_equal(pa, pb) and (ea is None or parity.bits_equal(ea, eb))


# ------------------------------------------------------------------------------------------------ ECC


@pytest.mark.parametrize("narrow_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("ecc_dtype", [torch.int8, torch.int16])
def test_ecc_join_and_split_of_the_kernels_are_bit_exact(narrow_dtype, ecc_dtype):
    """Every code value against narrow values of every exponent (zero, subnormal, smallest and largest normal
    included); then random fp32 values split both ways (standalone form and the fused kernels' form)."""
    info = torch.iinfo(ecc_dtype)
    codes = torch.arange(info.min, info.max + 1, dtype=torch.int32).to(ecc_dtype)
    bits = torch.arange(0, 0x7f80 if narrow_dtype == torch.bfloat16 else 0x7c00, 0x80 if narrow_dtype == torch.bfloat16 else 0x400,
                        dtype=torch.int32).to(torch.int16)
    for pattern in (0x0000, 0x0001, 0x0055, 0x007f if narrow_dtype == torch.bfloat16 else 0x03ff):
        for sign in (0, -0x8000):
            narrow_vals = ((bits.to(torch.int32) | pattern) + sign).to(torch.int16).view(narrow_dtype)
            for nv in narrow_vals[:: max(1, len(narrow_vals) // 24)]:
                narrow = nv.repeat(codes.numel()).contiguous()
                assert parity.bits_equal(H.ecc_join(narrow, codes), C.ecc_join(narrow, codes))
    x = torch.cat([_rand(1 << 16, s, 70 + i) for i, s in enumerate((1.0, 1e-3, 1e-6, 300.0))])
    if narrow_dtype == torch.float16:
        x = x.clamp(-6e4, 6e4)
    narrow = x.to(narrow_dtype)
    want = C.ecc_split(x, narrow, ecc_dtype)
    assert torch.equal(H.ecc_split(x, narrow, ecc_dtype, clamp=True), want)
    assert torch.equal(H.ecc_split(x, narrow, ecc_dtype, clamp=False), want)   # narrow is the rounding of x: no clamp needed
    # a narrow value that is NOT the rounding of x: the standalone form clamps like the reference
    other = (x * 1.5).to(narrow_dtype)
    assert torch.equal(H.ecc_split(x, other, ecc_dtype, clamp=True), C.ecc_split(x, other, ecc_dtype))
