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


# ------------------------------------------------------------------------------------------------ wave-level flows


def _centred_wave(seed):
    """512 first-moment and 512 second-moment values (lane l holds values 8l .. 8l+7, four lanes per group) whose quick
    pre-floor values sit in the middle between two integers: none fails the margin test."""
    g = torch.Generator().manual_seed(seed)
    m = torch.empty(16, 32, dtype=torch.float64)
    v = torch.empty(16, 32, dtype=torch.float64)
    for grp in range(16):
        am = 10.0 ** float(torch.empty(1).uniform_(-6, 1, generator=g))
        j = torch.randint(-126, 127, (32,), generator=g).double()
        j[0] = 127.0                                       # the group's largest magnitude
        t = j / 254.0                                      # x = 254 t + 0.5 = j + 0.5
        m[grp] = am * t / (1.0 - t.abs())
        av = 10.0 ** float(torch.empty(1).uniform_(-6, 1, generator=g))
        jv = torch.randint(0, 255, (32,), generator=g).double()
        jv[0] = 255.0
        v[grp] = (av * jv / 255.0) ** 2                    # x = 255 r / av + 0.5 = jv + 0.5
    return m.reshape(-1), v.reshape(-1)


@pytest.mark.parametrize("noise", NOISE)
def test_verified_flows_repair_exactly_the_lane_and_position_that_failed(noise):
    """The control flow of the verified requantisation (fo_math.h: requantize_mom_verified, requantize_var_verified)
    runs here over a simulated wavefront, the same text the kernels compile: a wavefront without a failing value
    asks one question per flow and branches past the repair; one failing value in one lane makes the flow ask once per
    element position, redo exactly that position and replace exactly that one code."""
    H.set_noise(noise)
    m, v = _centred_wave(3)
    H.flow_stats()
    qm, qv, em, ev = H.requantize_wave(m.float(), v.float())
    assert torch.equal(qm, em) and torch.equal(qv, ev)
    assert H.flow_stats() == dict(waves=0, questions=2, yes=0, codes_replaced=0)
    for lane, pos, which in ((0, 1, "m"), (17, 5, "m"), (63, 7, "m"), (5, 3, "v"), (40, 1, "v"), (63, 6, "v")):
        mm, vv = m.clone(), v.clone()
        i, grp = lane * 8 + pos, (lane * 8 + pos) // 32
        if which == "m":                                   # x = 254 t + 0.5 an integer: on the rounding boundary
            am = float(mm[grp * 32:(grp + 1) * 32].abs().max())
            t = (40.0 - 0.5) / 254.0
            mm[i] = am * t / (1.0 - t)
        else:
            av = float(vv[grp * 32:(grp + 1) * 32].max()) ** 0.5
            vv[i] = (av * (90.0 - 0.5) / 255.0) ** 2
        qm, qv, em, ev = H.requantize_wave(mm.float(), vv.float())
        assert torch.equal(qm, em) and torch.equal(qv, ev), (lane, pos, which)
        st = H.flow_stats()
        # the failing flow: one question for the wavefront, eight for the positions, two answered yes; the other: one
        assert st == dict(waves=0, questions=1 + 8 + 1, yes=2, codes_replaced=1), (lane, pos, which, st)
    # the same position failing in two lanes is still one position redone, two codes replaced
    mm = m.clone()
    for lane in (9, 50):
        grp = lane * 8 // 32
        am = float(mm[grp * 32:(grp + 1) * 32].abs().max())
        t = (-30.0 - 0.5) / 254.0
        mm[lane * 8 + 2] = am * t / (1.0 - abs(t))
    qm, qv, em, ev = H.requantize_wave(mm.float(), v.float())
    assert torch.equal(qm, em) and torch.equal(qv, ev)
    assert H.flow_stats() == dict(waves=0, questions=10, yes=2, codes_replaced=2)


@pytest.mark.parametrize("noise", [0, 7])
def test_update_repair_flow_redoes_the_one_flagged_element(noise):
    """adam_redo_flagged over simulated wavefronts: weights a thousand times larger than their updates except one, which
    its update all but cancels.  That element alone is flagged, it comes out with the oracle's bits, and every other
    element of its wavefront keeps its folded result (within one unit)."""
    H.set_noise(noise)
    n = 3 * 512 + 77
    for where in (0, 700, 1535, n - 1):
        a = _adam_state(n, torch.bfloat16, torch.int8, True, seed=8)
        a["p"] = torch.full((n,), 1.5, dtype=torch.bfloat16)
        g = _rand(n, 1e-3, 88).abs().add_(1e-4).to(torch.bfloat16)   # positive gradients: the first update is -lr
        a["p"][where] = 1e-3 * (1.0 + 2.0 ** -7)                     # lands within a few 1e-6 of zero
        b = _clone(a)
        T.adam_step_ref(T.MomentState(b["m"], b["ms"]), T.MomentState(b["v"], b["vs"]), b["p"], g, b["e"], 1e-3, 0.9, 0.999, 1e-8, 0.0, True, 1)
        flagged = H.adam_step(a["m"], a["ms"], a["v"], a["vs"], a["p"], g, a["e"], 1e-3, 0.9, 0.999, 1e-8, 0.0, True, 1)
        assert flagged == 1, (where, flagged)
        assert a["p"][where].view(torch.int16) == b["p"][where].view(torch.int16) and a["e"][where] == b["e"][where]
        parity.check_master(a["p"], a["e"], b["p"], b["e"], f"one flagged element at {where}")
        for key in ("m", "ms", "v", "vs"):
            assert parity.bits_equal(a[key], b[key])


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


def _adam_pair(n, dtype, ecc_dtype, quantized, decoupled, steps, exact=-1, lr=1e-3, seed=1, weight_scale=0.02, grad_scale=1e-3):
    """Yields (step, kernel-math state, oracle state, share of elements the guard of the folded update sent through
    the operation-by-operation form) with both stepped from the kernel-math state of the step before, so that every
    comparison starts from identical inputs."""
    a = _adam_state(n, dtype, ecc_dtype, quantized, seed)
    if weight_scale != 0.02:
        a["p"] = _rand(n, weight_scale, seed).to(dtype)
    wd = 0.01 * lr if decoupled else 0.01
    for step in range(1, steps + 1):
        g = _rand(n, grad_scale, 1000 * seed + step).to(dtype)
        b = _clone(a)
        mom = T.MomentState(b["m"], b["ms"]) if quantized else T.MomentState(plain=b["m"])
        var = T.MomentState(b["v"], b["vs"]) if quantized else T.MomentState(plain=b["v"])
        T.adam_step_ref(mom, var, b["p"], g, b["e"], lr, 0.9, 0.999, 1e-8, wd, decoupled, step)
        flagged = H.adam_step(a["m"], a["ms"], a["v"], a["vs"], a["p"], g, a["e"], lr, 0.9, 0.999, 1e-8, wd, decoupled, step, quantized, exact)
        yield step, a, b, flagged / max(n, 1)


def _folded(dtype, ecc_dtype):
    """The variants whose default update is the guarded folded form (fo_math.h: AdamExact names the others)."""
    return dtype != torch.float32 and (ecc_dtype is None or (dtype == torch.bfloat16 and ecc_dtype == torch.int8))


def _all_bits_equal(a, b):
    return all(a[k] is None or parity.bits_equal(a[k], b[k]) for k in a)


@pytest.mark.parametrize("noise", NOISE)
@pytest.mark.parametrize("dtype,ecc_dtype", VARIANTS)
@pytest.mark.parametrize("quantized", [True, False])
def test_adam_step_of_the_kernels_against_the_oracle(noise, dtype, ecc_dtype, quantized):
    """FlashAdam (decay folded into the gradient) and FlashAdamW, four steps, every step from identical inputs.
    Moments, codes and scales: every bit the oracle's, for every variant.  Parameters and ECC: every bit the oracle's
    where the update runs operation by operation; within one unit of master precision, with no allowance, where
    it is the guarded folded form."""
    H.set_noise(noise)
    for decoupled in (True, False):
        for n in (1, 31, 33, 4099, (1 << 15) + 17):
            for step, a, b, _ in _adam_pair(n, dtype, ecc_dtype, quantized, decoupled, steps=4):
                what = f"adam {dtype} ecc={ecc_dtype} q={quantized} decoupled={decoupled} n={n} step={step}"
                for key in ("m", "ms", "v", "vs"):
                    assert a[key] is None or parity.bits_equal(a[key], b[key]), f"{what}: {key} differs"
                if _folded(dtype, ecc_dtype):
                    parity.check_master(a["p"], a["e"], b["p"], b["e"], what)
                else:
                    assert _all_bits_equal(a, b), what


@pytest.mark.parametrize("noise", NOISE)
@pytest.mark.parametrize("dtype,ecc_dtype", [(torch.bfloat16, torch.int8), (torch.bfloat16, None), (torch.float16, None)])
def test_operation_by_operation_adam_update_is_bit_exact_where_the_folded_one_is_the_default(noise, dtype, ecc_dtype):
    """The `*_exact` entry points run the reference's sequence on every element of the variants whose default is the
    guarded folded update: every bit the oracle's."""
    H.set_noise(noise)
    for step, a, b, flagged in _adam_pair((1 << 15) + 5, dtype, ecc_dtype, True, True, steps=4, exact=1):
        assert _all_bits_equal(a, b), f"{dtype} {ecc_dtype} step {step}"
        assert flagged == 0.0


@pytest.mark.parametrize("noise", [0, 7])
@pytest.mark.parametrize("dtype,ecc_dtype", [(torch.bfloat16, torch.int8), (torch.bfloat16, None), (torch.float16, None)])
def test_guarded_folded_update_keeps_master_weights_within_one_unit(noise, dtype, ecc_dtype):
    """The folded update rounds at other places than the reference's sequence, so the two differ by a few ulps of
    the UPDATE; for a weight that its own update all but cancels that is many units of the weight.  The guard sends
    exactly those elements through the operation-by-operation form.  Held here where it bites: weights as small as
    the updates (every second element is flagged), the usual scales (about 1e-3 of the elements), a learning rate ten
    times smaller, and weights that start at zero (a first update lands on lr exactly; nothing cancels).  With no
    allowance: no master weight is more than one unit away, on any step."""
    H.set_noise(noise)
    n = 1 << 18
    share = {}
    for name, kw in (("usual", {}), ("small lr", dict(lr=1e-4)), ("weights ~ update", dict(weight_scale=1e-3)),
                     ("weights << update", dict(weight_scale=1e-5)), ("zero weights", dict(weight_scale=0.0))):
        worst = flagged_most = 0.0
        for step, a, b, flagged in _adam_pair(n, dtype, ecc_dtype, True, True, steps=4, **kw):
            w, _ = parity.check_master(a["p"], a["e"], b["p"], b["e"], f"{name} step {step}")
            worst, flagged_most = max(worst, w), max(flagged_most, flagged)
        share[name] = flagged_most
        assert worst <= 1.0 + 1e-9
    print(f"{dtype} ecc={ecc_dtype}: largest share of elements redone operation by operation:", {k: f"{v:.1e}" for k, v in share.items()})
    if ecc_dtype is not None:
        assert 1e-4 < share["usual"] < 5e-3 and share["weights ~ update"] > 0.02


def test_folded_update_without_its_guard_would_miss_the_tolerance():
    """The guard is what meets the bar, not luck: among the elements it flags, the unguarded folded result (the guard's
    own first evaluation) lies more than one unit away from the oracle's for a visible share."""
    H.set_noise(0)
    n = 1 << 18
    a = _adam_state(n, torch.bfloat16, torch.int8, True, seed=1)
    g = _rand(n, 1e-3, 1001).to(torch.bfloat16)
    b = _clone(a)
    T.adam_step_ref(T.MomentState(b["m"], b["ms"]), T.MomentState(b["v"], b["vs"]), b["p"], g, b["e"], 1e-3, 0.9, 0.999, 1e-8, 1e-5, True, 1)
    p_folded, redo = H.adam_folded_update(a["p"], a["e"], g, a["m"], a["ms"], a["v"], a["vs"], 1e-3, 0.9, 0.999, 1e-8, 1e-5, True, 1)
    assert 1e-3 < float(redo.float().mean()) < 5e-3
    # split the unguarded fp32 results like the kernels do and compare with the oracle's pair
    narrow = p_folded.to(torch.bfloat16)
    ecc = H.ecc_split(p_folded, narrow, torch.int8, clamp=False)
    units = (parity.master_value(narrow, ecc) - parity.master_value(b["p"], b["e"])).abs() / parity.master_unit(b["p"], b["e"])
    assert float(units[~redo].max()) <= 1.0 + 1e-9   # the elements the guard lets through are fine as they are
    assert float((units[redo] > 1.0).float().mean()) > 0.01 and float(units[redo].max()) > 2.0


def test_code_over_255_is_the_correctly_rounded_quotient():
    q = torch.arange(256, dtype=torch.float32)
    assert torch.equal(H.code_over_255(), q / 255.0)


@pytest.mark.parametrize("noise", NOISE)
@pytest.mark.parametrize("dtype,ecc_dtype", [(torch.bfloat16, torch.int8), (torch.float16, torch.int8), (torch.bfloat16, None), (torch.bfloat16, torch.int16)])
def test_groups_that_start_from_zero_next_to_warm_ones(noise, dtype, ecc_dtype):
    """After two steps some groups are reset to zero, as if they had seen no gradient yet.  There the moments are a
    narrow gradient times a constant and 0.3 % of them sit exactly on a rounding boundary, where the quick requantiser
    forms must give way to the exact one; next to them sit warm groups.  Every code and scale equals the oracle's."""
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
    for key in ("m", "ms", "v", "vs"):
        assert parity.bits_equal(a[key], b[key]), f"{key} differs from the oracle"


@pytest.mark.parametrize("noise", [0, 7])
def test_a_sudden_jump_of_the_gradient_scale_keeps_the_codes_exact(noise):
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
        for key in ("m", "ms", "v", "vs"):
            assert parity.bits_equal(a[key], b[key]), f"jump {jump:g}: {key} differs from the oracle"
        parity.check_master(a["p"], a["e"], b["p"], b["e"], f"jump {jump:g}")


@pytest.mark.parametrize("betas", [(0.0, 0.999), (0.9, 0.0), (0.0, 0.0), (0.01, 0.999), (0.9, 0.1), (0.5, 0.9), (0.99, 0.9999)])
def test_unusual_betas(betas):
    """beta1 = 0 or beta2 = 0 make every step a first step for that moment (the old state has no weight, the new
    values are a narrow gradient times a constant); small betas come close.  Codes and scales stay the oracle's bit for
    bit, master weights within one unit."""
    H.set_noise(7)
    n = 1 << 17
    a = _adam_state(n, torch.bfloat16, torch.int8, True, seed=3)
    for step in range(1, 5):
        g = _rand(n, 1e-3, 10 + step).to(torch.bfloat16)
        b = _clone(a)
        T.adam_step_ref(T.MomentState(b["m"], b["ms"]), T.MomentState(b["v"], b["vs"]), b["p"], g, b["e"], 1e-3, betas[0], betas[1], 1e-8, 1e-5, True, step)
        H.adam_step(a["m"], a["ms"], a["v"], a["vs"], a["p"], g, a["e"], 1e-3, betas[0], betas[1], 1e-8, 1e-5, True, step)
        for key in ("m", "ms", "v", "vs"):
            assert parity.bits_equal(a[key], b[key]), f"betas {betas} step {step}: {key} differs from the oracle"
        parity.check_master(a["p"], a["e"], b["p"], b["e"], f"betas {betas} step {step}")


@pytest.mark.parametrize("lr,eps", [(0.0, 1e-8), (1e-30, 1e-8), (1e20, 1e-8), (1e-3, 0.0), (1e-3, 1e-30), (1e-3, 1.0), (3.0, 1e-8)])
def test_extreme_learning_rates_and_eps(lr, eps):
    """The folded update's constants bc1 / (lr sqrt(bc2)) and eps bc1 / lr leave the range in which its error bound
    holds for absurd learning rates; such launches take the operation-by-operation form (bit-exact).  The others stay
    within one unit."""
    H.set_noise(7)
    n = 1 << 14
    a = _adam_state(n, torch.bfloat16, torch.int8, True, seed=4)
    for step in range(1, 4):
        g = _rand(n, 1e-3, 20 + step).to(torch.bfloat16)
        b = _clone(a)
        T.adam_step_ref(T.MomentState(b["m"], b["ms"]), T.MomentState(b["v"], b["vs"]), b["p"], g, b["e"], lr, 0.9, 0.999, eps, lr * 0.01, True, step)
        H.adam_step(a["m"], a["ms"], a["v"], a["vs"], a["p"], g, a["e"], lr, 0.9, 0.999, eps, lr * 0.01, True, step)
        for key in ("m", "ms", "v", "vs"):
            assert parity.bits_equal(a[key], b[key])
        if lr in (1e-30, 1e20):
            assert _all_bits_equal(a, b), f"lr {lr:g} step {step}"
        else:
            parity.check_master(a["p"], a["e"], b["p"], b["e"], f"lr {lr:g} eps {eps:g} step {step}")


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
