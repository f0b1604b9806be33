"""Pins the ECC split/join of the CPU oracle: hand-derived known answers, exactness properties, the
boundary bit patterns and the per-binade exception counts recorded in the reference's own tests
(/root/reference/test/test_ecc_invariants.py:257-291, /root/reference/test/test_optimizers.py:749-758),
and the two restatements against each other."""

import pytest
import torch

from oracle import c_oracle as C
from oracle import torch_oracle as T

SPLIT = {"torch": T.ecc_split_ref, "c": C.ecc_split}
JOIN = {"torch": T.ecc_join_ref, "c": C.ecc_join}


@pytest.mark.parametrize("backend", SPLIT)
def test_known_answers_bf16(backend):
    split, join = SPLIT[backend], JOIN[backend]
    x = torch.tensor([1.0, 1 + 2.0**-8, 1 + 2.0**-9, -(1 + 2.0**-9), 3.0, -0.0, 1 - 2.0**-9], dtype=torch.float32)
    nar = x.to(torch.bfloat16)
    # bf16 ulp at 1.0 is 2^-7; 1+2^-8 is a tie that rounds to even (1.0), error = +half ulp = full scale
    assert nar.tolist() == [1.0, 1.0, 1.0, -1.0, 3.0, -0.0, 1.0]
    e8 = split(x, nar, torch.int8)
    e16 = split(x, nar, torch.int16)
    # the last one sits below 1.0: the narrow value 1.0 has exponent 0, so the scale is still 2^-8 and the
    # error -2^-9 is minus half of it
    assert e8.tolist() == [0, 127, 64, -64, 0, 0, -64]  # 63.5 rounds half away from zero
    assert e16.tolist() == [0, 32767, 16384, -16384, 0, 0, -16384]
    assert torch.equal(join(nar, e8)[[0, 1, 4]], x[[0, 1, 4]])
    assert torch.equal(join(nar, e16)[[0, 1, 4]], x[[0, 1, 4]])
    # 64/127 * 2^-8 : reconstruction error of the 24-bit master is below one step (2^-8/127)
    assert (join(nar, e8) - x).abs().max() <= 2.0**-8 / 127 / 2 * 1.01
    assert (join(nar, e16) - x).abs().max() <= 2.0**-8 / 32767 / 2 * 1.01


@pytest.mark.parametrize("backend", SPLIT)
def test_known_answers_fp16(backend):
    split, join = SPLIT[backend], JOIN[backend]
    x = torch.tensor([1.0, 1 + 2.0**-11, 1 + 2.0**-12, -(1 + 2.0**-12), 2.0**-24 * 0.5], dtype=torch.float32)
    nar = x.to(torch.float16)
    assert nar.tolist() == [1.0, 1.0, 1.0, -1.0, 0.0]
    e8 = split(x, nar, torch.int8)
    # last: fp16 zero uses the min-normal exponent -14 -> scale 2^-25 -> 2^-25/2^-25 = 1 -> 127
    assert e8.tolist() == [0, 127, 64, -64, 127]
    assert join(nar, e8)[4].item() == 2.0**-25


@pytest.mark.parametrize("narrow", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("ecc_dtype", [torch.int8, torch.int16])
def test_properties_random(narrow, ecc_dtype):
    g = torch.Generator().manual_seed(3)
    mags = torch.exp(torch.empty(200000).uniform_(-20, 10, generator=g))
    x = mags * torch.where(torch.rand(200000, generator=g) < 0.5, -1.0, 1.0)
    if narrow == torch.float16:
        x = x.clamp(-60000, 60000)
    nar = x.to(narrow)
    ecc_t = T.ecc_split_ref(x, nar, ecc_dtype)
    ecc_c = C.ecc_split(x, nar, ecc_dtype)
    assert torch.equal(ecc_t, ecc_c)
    rec_t = T.ecc_join_ref(nar, ecc_t)
    rec_c = C.ecc_join(nar, ecc_c)
    assert torch.equal(rec_t.view(torch.int32), rec_c.view(torch.int32))
    # the master is never further from x than the narrow value alone, and within one master step
    mant = 7 if narrow == torch.bfloat16 else 10
    half_ulp = torch.exp2((T.unbiased_exponent(nar) - mant - 1).float())
    step = half_ulp / (127.0 if ecc_dtype == torch.int8 else 32767.0)
    err = (rec_t.double() - x.double()).abs()
    assert (err <= (nar.double() - x.double()).abs() + 1e-300).all()
    # half a master step, plus the fp32 rounding of the sum (half an fp32 ulp, which is 2^(mant-23) half-ulps)
    assert (err <= step.double() * 0.5 + half_ulp.double() * 2.0 ** (mant - 23) * 1.0001).all()
    # values that are exactly representable in the narrow type need no correction
    exact = nar.float()
    assert T.ecc_split_ref(exact, nar, ecc_dtype).eq(0).all()
    assert C.ecc_split(exact, nar, ecc_dtype).eq(0).all()


def test_boundary_bit_patterns():
    """The fp32 bit patterns the reference feeds its precision test (test_optimizers.py:749-758):
    values just above/below bf16 rounding boundaries must survive split+join to within one step."""
    pats = [0x3F800000, 0x3F808000, 0x3F807FFF, 0x3F808001, 0x3F80FFFF, 0x3F7FFFFF, 0x00800000, 0x7F7FFFFF & 0x7EFFFFFF]
    x = torch.tensor(pats, dtype=torch.int64).to(torch.int32).view(torch.float32)
    nar = x.to(torch.bfloat16)
    for ecc_dtype, mx in ((torch.int8, 127.0), (torch.int16, 32767.0)):
        ecc = T.ecc_split_ref(x, nar, ecc_dtype)
        assert torch.equal(ecc, C.ecc_split(x, nar, ecc_dtype))
        rec = T.ecc_join_ref(nar, ecc)
        half_ulp = torch.exp2((T.unbiased_exponent(nar) - 8).double())
        assert ((rec.double() - x.double()).abs() <= half_ulp / mx * 0.5 + half_ulp * 2.0**-16 * 1.0001).all()


# Exception budgets per (sign, exponent) binade copied as data from the reference's invariants test
# (/root/reference/test/test_ecc_invariants.py:257-262 normals, :282-291 subnormals); unnamed invariants
# allow zero exceptions.  The reference measured them with its Triton kernels over all 2^23 mantissas.
_NORMAL_BUDGET = {
    ("bf16", "16bit_no_worse_zero"): 32,
    ("bf16", "16bit_no_worse_always"): 32,
    ("bf16", "16bit_better_in_middle_range"): 32129,
    ("fp16", "16bit_better_in_middle_range"): 235656,
}
_DENORMAL_BUDGET = {
    ("bf16", "8bit_corrects_representable"): 8192,
    ("bf16", "16bit_corrects_representable"): 25,
    ("bf16", "16bit_better_in_middle_range"): 24319,
    ("fp16", "16bit_no_worse_zero"): 8192,
    ("fp16", "16bit_no_worse_always"): 16383,
    ("fp16", "8bit_corrects_representable"): 7656268,
    ("fp16", "16bit_corrects_representable"): 7602176,
    ("fp16", "16bit_better_in_middle_range"): 123952,
}
_DT = {"bf16": torch.bfloat16, "fp16": torch.float16}


def _sweep(name, exponents, budget):
    worst = {}
    for sign in (1, -1):
        for e in exponents:
            counts = C.ecc_invariants(sign, e, _DT[name])
            for inv, c in counts.items():
                assert c <= budget.get((name, inv), 0), (name, sign, e, inv, c)
                worst[inv] = max(worst.get(inv, 0), c)
    return worst


def test_ecc_invariants_bf16_normal_binades():
    # a spread of the 254 normal binades incl. both ends (the GPU suite sweeps all of them)
    worst = _sweep("bf16", [-126, -125, -120, -113, -64, 0, 1, 126, 127], _NORMAL_BUDGET)
    # the budgets are the reference's own measured maxima: an implementation of the same arithmetic hits them
    assert worst["16bit_no_worse_zero"] == 32 and worst["16bit_better_in_middle_range"] == 32129


def test_ecc_invariants_bf16_subnormal_binade():
    worst = _sweep("bf16", [-127], _DENORMAL_BUDGET)
    assert worst["8bit_corrects_representable"] == 8192
    assert worst["16bit_corrects_representable"] == 25
    assert worst["16bit_better_in_middle_range"] == 24319


def test_ecc_invariants_fp16_normal_binades():
    worst = _sweep("fp16", [-14, -13, 0, 14, 15], _NORMAL_BUDGET)
    assert worst["16bit_better_in_middle_range"] == 235656


def test_ecc_invariants_fp16_subnormal_binades():
    worst = _sweep("fp16", [-30, -25, -24, -20, -16, -15], _DENORMAL_BUDGET)
    assert worst["8bit_corrects_representable"] == 7656268
    assert worst["16bit_corrects_representable"] == 7602176
    assert worst["16bit_better_in_middle_range"] == 123952
