"""Pins the group codec of the CPU oracle (oracle/torch_oracle.py and oracle/fo_oracle.c) without the
reference: hand-derived known answers, the invariants and thresholds of the reference's own codec tests
(/root/reference/test/test_compression.py:59-80, 199-244), brute force over every code, and the two
independent restatements against each other bit for bit."""

import numpy as np
import pytest
import torch

from oracle import c_oracle as C
from oracle import torch_oracle as T

MODES = [(True, False, False), (True, False, True), (False, False, False), (False, True, False)]  # signed, sqrt, softsign
BACKENDS = {"torch": (T.quantize_ref, T.dequantize_ref), "c": (C.quantize, C.dequantize)}


def _bits(t):
    return t.contiguous().view(torch.uint8) if t.dtype != torch.uint8 else t


@pytest.mark.parametrize("backend", BACKENDS)
def test_known_answer_signed_softsign(backend):
    q, dq = BACKENDS[backend]
    x = torch.zeros(32)
    x[:4] = torch.tensor([1.0, 0.5, 0.2, -0.2])
    codes, scales = q(x, True, False, True)
    # softsign(1)=1 ->127 ; softsign(.5)=2/3 -> 84.67 -> 85 ; softsign(.2)=1/3 -> 42.33 -> 42 ; -42.33+.5 -> floor -42
    assert codes[:5].tolist() == [127, 85, 42, -42, 0]
    assert scales.dtype == torch.float16 and scales.tolist() == [1.0]
    back = dq(codes, scales, True, False, True)
    # inverse softsign: y/(2-|y|) with y=q/127
    exp = [1.0, (85 / 127) / (2 - 85 / 127), (42 / 127) / (2 - 42 / 127), -(42 / 127) / (2 - 42 / 127)]
    np.testing.assert_allclose(back[:4].numpy(), exp, rtol=3e-7)


@pytest.mark.parametrize("backend", BACKENDS)
def test_known_answer_unsigned_sqrt(backend):
    q, dq = BACKENDS[backend]
    x = torch.zeros(32)
    x[:3] = torch.tensor([4.0, 1.44, 0.25])
    codes, scales = q(x, False, True, False)
    # sqrt -> [2, 1.2, .5] ; /2 -> [1, .6, .25] ; *255 + .5 -> [255.5, 153.5, 64.25] -> floor
    assert codes[:4].tolist() == [255, 153, 64, 0]
    assert codes.dtype == torch.uint8 and scales.tolist() == [2.0]
    back = dq(codes, scales, False, True, False)
    np.testing.assert_allclose(back[:3].numpy(), [4.0, (153 / 255 * 2) ** 2, (64 / 255 * 2) ** 2], rtol=3e-7)
    assert back[3] == 0


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("signed,sqrt,softsign", MODES)
def test_zeros_and_max(backend, signed, sqrt, softsign):
    q, dq = BACKENDS[backend]
    # all-zero groups: codes 0, scale fp16(1e-12) == 0, dequantised 0   (reference: "zeros stay zeros")
    codes, scales = q(torch.zeros(70), signed, sqrt, softsign)
    assert codes.eq(0).all() and scales.eq(0).all() and scales.numel() == 3
    assert dq(codes, scales, signed, sqrt, softsign).eq(0).all()
    # constant tensor: every element is the group absmax -> every code is the maximum
    top = 127 if signed else 255
    codes, scales = q(torch.full((64,), float(top)), signed, sqrt, softsign)
    assert codes.eq(top).all()
    exp_scale = np.sqrt(np.float32(top)) if sqrt else np.float32(top)
    assert scales.tolist() == [float(np.float16(exp_scale))] * 2


@pytest.mark.parametrize("signed,softsign", [(True, True), (True, False), (False, False)])
def test_bruteforce_all_codes_closed_form(signed, softsign):
    """Every code times a few scales through both dequantisers against the formula in float64."""
    lo, hi = (-127, 127) if signed else (0, 255)
    cmax = 127.0 if signed else 255.0
    for scale in [1.0, 0.5, 3.140625, 6.1035e-05, 5.96e-08, 65504.0]:
        codes = torch.arange(lo, hi + 1, dtype=torch.int32).to(torch.int8 if signed else torch.uint8)
        pad = (-codes.numel()) % 32
        codes = torch.cat([codes, codes.new_zeros(pad)])
        scales = torch.full((codes.numel() // 32,), scale, dtype=torch.float16)
        s = float(scales[0])
        y = codes.double() / cmax
        want = (y / (2 - y.abs()) if softsign else y) * s
        for dq in (T.dequantize_ref, C.dequantize):
            got = dq(codes, scales, signed, False, softsign).double()
            assert torch.allclose(got, want, rtol=4e-7, atol=0)


@pytest.mark.parametrize("signed,sqrt,softsign", MODES)
def test_idempotent_on_codes(signed, sqrt, softsign):
    """quantise(dequantise(q, s)) == q whenever the group holds a full-scale code and the scale is an
    fp16 normal (then the recovered absmax equals the scale exactly)."""
    g = torch.Generator().manual_seed(5)
    n = 32 * 200
    lo, hi = (-127, 128) if signed else (0, 256)
    codes = torch.randint(lo, hi, (n,), generator=g).to(torch.int8 if signed else torch.uint8)
    codes.view(-1, 32)[:, 7] = 127 if signed else 255
    scales = (torch.rand(n // 32, generator=g) * 4 + 0.01).to(torch.float16)
    for q, dq in BACKENDS.values():
        x = dq(codes, scales, signed, sqrt, softsign)
        codes2, scales2 = q(x, signed, sqrt, softsign)
        assert torch.equal(codes2, codes)
        assert torch.equal(_bits(scales2), _bits(scales))


def _make(case, shape, dtype, signed, gen):
    # same five input families as /root/reference/test/test_compression.py:31-56
    if case == "zeros":
        x = torch.zeros(shape, dtype=dtype)
    elif case == "max_vals":
        x = torch.full(shape, 127.0 if signed else 255.0, dtype=dtype)
    elif case == "small_vals":
        x = (torch.rand(shape, generator=gen) * 0.01).to(dtype)
    elif case == "mixed_scales":
        x = torch.randn(shape, generator=gen)
        split = max(1, shape[0] // 2)
        x[:split] *= 0.1
        x[split:] *= 2.0
        x = x.to(dtype)
    else:
        x = torch.randn(shape, generator=gen).to(dtype)
    return x if signed else x.abs()


@pytest.mark.parametrize("case", ["zeros", "max_vals", "random", "small_vals", "mixed_scales"])
@pytest.mark.parametrize("shape", [(1, 5), (1, 12), (1, 16), (1, 17), (1, 32), (17, 32), (1024, 16)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("signed,sqrt,softsign", MODES)
def test_roundtrip_quality_and_c_vs_torch(case, shape, dtype, signed, sqrt, softsign):
    for seed in range(3 if case in ("random", "small_vals", "mixed_scales") else 1):
        gen = torch.Generator().manual_seed(seed)
        x = _make(case, shape, dtype, signed, gen)
        ct, st = T.quantize_ref(x, signed, sqrt, softsign)
        cc, sc = C.quantize(x, signed, sqrt, softsign)
        assert ct.shape == x.shape and ct.dtype == (torch.int8 if signed else torch.uint8)
        assert torch.equal(ct, cc) and torch.equal(_bits(st), _bits(sc))
        rt = T.dequantize_ref(ct, st, signed, sqrt, softsign)
        rc = C.dequantize(cc, sc, signed, sqrt, softsign)
        assert torch.equal(_bits(rt), _bits(rc))
        xr = rt.to(x.dtype).float().ravel()
        xf = x.float().ravel()
        if case == "zeros":
            assert xr.eq(0).all()
            continue
        # thresholds of /root/reference/test/test_compression.py:59-80
        assert torch.cosine_similarity(xf, xr, dim=0).item() > 0.9999
        assert (xr - xf).abs().mean().item() <= (2 * xf.abs().max().item()) / 255.0 / 2 * 1.6


@pytest.mark.parametrize("n", [33, 65, 100, 999, 1000, 1025, 2000, 4097])
@pytest.mark.parametrize("signed", [True, False])
def test_tail_group(n, signed):
    """/root/reference/test/test_compression.py:204-244: a short last group is scaled by its own absmax."""
    x = torch.randn(n, generator=torch.Generator().manual_seed(42)) * 5.0
    if not signed:
        x = x.abs()
    for q, dq in BACKENDS.values():
        codes, scales = q(x, signed)
        back = dq(codes, scales, signed)
        tail = n % 32
        err = (x - back).abs()
        assert err[-tail:].max() <= max(err[:-tail].max() * 2.0, 1e-6)
        want = x[-tail:].abs().max().item()
        assert abs(scales[-1].item() - want) / max(want, 1e-12) < 0.003
        assert scales.numel() == (n + 31) // 32


def test_fp16_scale_conversion_exhaustive_slices():
    """The C restatement's fp32->fp16 (used for every stored scale) against numpy's, including the
    subnormal range that sqrt(v) of 1e-3-sized gradients lands in, ties, and overflow."""
    lib = C.lib()
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.uniform(0, 7e-5, 20000), rng.uniform(0, 1e-7, 5000), rng.uniform(0, 70000, 20000),
        np.array([0.0, 1e-12, 2.0 ** -25, 2.0 ** -24, 3 * 2.0 ** -25, 65504.0, 65519.9, 65520.0, 1e9, np.inf]),
        (np.arange(0, 2048, dtype=np.float64) + 0.5) * 2.0 ** -24,  # every subnormal tie
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([lib.fo_oracle_f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)
    allh = np.arange(0, 0x7C01, dtype=np.uint16)
    back = np.array([lib.fo_oracle_f16_to_f32(int(h)) for h in allh[::7]], dtype=np.float32)
    assert np.array_equal(back, allh[::7].view(np.float16).astype(np.float32))


def test_a_nan_element_does_not_poison_its_groups_scale():
    """The reference's group maximum is `tl.max` followed by `tl.maximum(., 1e-12)` (ref:2657-2658), NaN-ignoring
    reductions: a NaN element leaves the scale of its group to the other 31.  Both restatements agree on that (the
    code stored for the NaN element itself is unspecified and not compared)."""
    x = torch.linspace(-2.0, 3.0, 96)
    x[40] = float("nan")
    _, scales_t = T.quantize_ref(x, True, False, True)
    _, scales_c = C.quantize(x, True, False, True)
    assert torch.equal(scales_t, scales_c) and not bool(torch.isnan(scales_t.float()).any())
    assert scales_t[1] == x[32:64][~torch.isnan(x[32:64])].abs().max().to(torch.float16)
    all_nan = torch.full((32,), float("nan"))
    assert T.quantize_ref(all_nan, True, False, True)[1][0] == torch.tensor(1e-12).to(torch.float16)
