"""GPU parity of the HIP kernels (through the C ABI, via flashoptim_amd.kernels) against the CPU oracle."""

import pytest
import torch

from oracle import c_oracle as C
from oracle import torch_oracle as T
from tests import parity

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
MODES = [(True, False, False), (True, False, True), (False, False, False), (False, True, False)]
SIZES = [1, 5, 31, 32, 33, 1000, 4095, 4096, 4097, 3 * 4096 + 555, 1 << 18]


def _native_lib():
    from flashoptim_amd import _native
    return _native.lib()


def _diag_lib():
    from flashoptim_amd import _native
    return _native.diag_lib()


def _k():
    from flashoptim_amd import kernels
    return kernels


def _rand(n, scale, seed):
    return torch.randn(n, generator=torch.Generator().manual_seed(seed)) * scale


# ------------------------------------------------------------------------------------ standalone codec


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("signed,sqrt,softsign", MODES)
def test_quantize_dequantize_bit_exact(dtype, signed, sqrt, softsign):
    k = _k()
    for i, n in enumerate(SIZES):
        x = (_rand(n, 3.0, i) * (0.01 if i % 3 == 0 else 1.0)).to(dtype)
        if not signed:
            x = x.abs()
        codes, scales = k.quantize(x.to(DEV), signed=signed, sqrt=sqrt, softsign=softsign)
        rc, rs = C.quantize(x, signed, sqrt, softsign)
        assert codes.shape == x.shape and scales.numel() == (n + 31) // 32
        assert torch.equal(codes.cpu(), rc), (n, "codes")
        assert parity.bits_equal(scales, rs), (n, "scales")
        back = k.dequantize(codes, scales, signed=signed, sqrt=sqrt, softsign=softsign)
        assert parity.bits_equal(back, C.dequantize(rc, rs, signed, sqrt, softsign)), (n, "dequantize")


def test_quantize_unaligned_view_and_2d():
    k = _k()
    base = _rand(10001, 1.0, 3).to(torch.bfloat16).to(DEV)
    view = base[1:]  # 2-byte offset: not 16-byte aligned -> guarded path
    codes, scales = k.quantize(view)
    rc, rs = C.quantize(base.cpu()[1:].contiguous())
    assert torch.equal(codes.cpu(), rc) and parity.bits_equal(scales, rs)
    x2 = _rand(64 * 33, 1.0, 4).view(64, 33).to(DEV)
    c2, s2 = k.quantize(x2)
    assert c2.shape == (64, 33)
    rc2, rs2 = C.quantize(x2.cpu())
    assert torch.equal(c2.cpu(), rc2) and parity.bits_equal(s2, rs2)


def test_dequantize_every_code_bit_exact():
    """All 256 code bytes x several scales, signed+softsign and unsigned+sqrt: the table behind the fused
    kernels' dequantisation must equal IEEE evaluation of the reference formula."""
    k = _k()
    for signed, sqrt, softsign in MODES:
        codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
        codes = codes.view(torch.int8) if signed else codes
        scales = torch.tensor([1.0, 0.37, 6.1e-5, 3.2e-5, 5.96e-8, 1234.0, 0.0, 65504.0], dtype=torch.float16)
        got = k.dequantize(codes.to(DEV), scales.to(DEV), signed=signed, sqrt=sqrt, softsign=softsign)
        assert parity.bits_equal(got, C.dequantize(codes, scales, signed, sqrt, softsign))


# ------------------------------------------------------------------------------------- standalone ECC


@pytest.mark.parametrize("narrow", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("ecc_dtype,width", [(torch.int8, 3), (torch.int16, 4)])
def test_ecc_split_join_bit_exact(narrow, ecc_dtype, width):
    k = _k()
    g = torch.Generator().manual_seed(7)
    for n in [1, 17, 4096, 4097, 1 << 18]:
        mags = torch.exp(torch.empty(n).uniform_(-30, 10, generator=g))
        x = mags * torch.where(torch.rand(n, generator=g) < 0.5, -1.0, 1.0)
        x[: min(n, 6)] = torch.tensor([0.0, 1.0, 1 + 2.0**-8, -(1 + 2.0**-9), 2.0**-130, 1e-40])[: min(n, 6)]
        if narrow == torch.float16:
            x = x.clamp(-60000, 60000)
        nar = x.to(narrow)
        ecc = k.compute_ecc_bits(x.to(DEV), nar.to(DEV), master_bytewidth=width)
        ref = C.ecc_split(x, nar, ecc_dtype)
        assert ecc.dtype == ecc_dtype and torch.equal(ecc.cpu(), ref), n
        rec = k.reconstruct_fp32_param(nar.to(DEV), ecc)
        assert parity.bits_equal(rec, C.ecc_join(nar, ref)), n


def test_ecc_join_every_int16_value():
    k = _k()
    ecc = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16)
    for val in [1.0, -3.5, 2.0**-126, 0.0, 1e-3]:
        nar = torch.full((65536,), val).to(torch.bfloat16)
        assert parity.bits_equal(k.reconstruct_fp32_param(nar.to(DEV), ecc.to(DEV)), C.ecc_join(nar, ecc))


def test_wrapper_errors():
    k = _k()
    with pytest.raises(ValueError):
        k.reconstruct_fp32_param(torch.zeros(4, device=DEV), torch.zeros(4, dtype=torch.int8, device=DEV))
    with pytest.raises(ValueError):
        k.reconstruct_fp32_param(torch.zeros(4, device=DEV, dtype=torch.bfloat16), torch.zeros(4, dtype=torch.int32, device=DEV))
    with pytest.raises(ValueError):
        k.compute_ecc_bits(torch.zeros(4, device=DEV, dtype=torch.bfloat16), torch.zeros(4, device=DEV, dtype=torch.bfloat16))
    with pytest.raises(ValueError):
        k.compute_ecc_bits(torch.zeros(4, device=DEV), torch.zeros(4, device=DEV, dtype=torch.bfloat16), master_bytewidth=2)
    with pytest.raises(NotImplementedError):
        k.quantize(torch.zeros(4))


# ---------------------------------------------------------------------------------------- fused steps

VARIANTS = [
    (torch.bfloat16, torch.int8), (torch.bfloat16, torch.int16), (torch.bfloat16, None),
    (torch.float16, torch.int8), (torch.float16, torch.int16), (torch.float16, None), (torch.float32, None),
]


class _Case:
    """State of one tensor on the CPU (oracle side) mirrored on the GPU."""

    def __init__(self, n, dtype, ecc_dtype, quantized, n_states, seed, offset=0):
        self.n, self.dtype, self.quantized = n, dtype, quantized
        self.p = _rand(n, 0.02, seed).to(dtype)
        self.ecc = None if ecc_dtype is None else torch.zeros(n, dtype=ecc_dtype)
        self.states = [T.MomentState.zeros(n, i == 0, quantized, dtype) for i in range(n_states)]
        self.offset = offset
        self.gp = self._dev(self.p)
        self.gecc = None if self.ecc is None else self._dev(self.ecc)
        self.gstates = [
            (self._dev(s.codes), s.scales.to(DEV)) if quantized else (self._dev(s.plain), None) for s in self.states
        ]

    def _dev(self, t):
        # offset > 0 places the tensor at a misaligned address inside a larger buffer (guarded path)
        if self.offset == 0:
            return t.to(DEV)
        buf = torch.zeros(t.numel() + self.offset, dtype=t.dtype, device=DEV)
        buf[self.offset:].copy_(t)
        return buf[self.offset:]

    def resync_oracle(self):
        """Copy the GPU state to the CPU so the next comparison starts from identical inputs."""
        self.p.copy_(self.gp.cpu())
        if self.ecc is not None:
            self.ecc.copy_(self.gecc.cpu())
        for s, (a, b) in zip(self.states, self.gstates):
            if self.quantized:
                s.codes.copy_(a.cpu())
                s.scales.copy_(b.cpu())
            else:
                s.plain.copy_(a.cpu())

    def compare(self, what, exact):
        """exact: every output bit must equal the oracle's (every kernel but Adam with the guarded folded update, see
        tests/parity.py).  Otherwise: moments, codes and scales bit for bit, master weights within one unit of
        master precision and narrow parameters within one ulp, with no allowance.
        Returns (largest master-weight difference in units, fraction of elements whose master weights differ)."""
        for i, (s, (a, b)) in enumerate(zip(self.states, self.gstates)):
            if self.quantized:
                assert parity.bits_equal(a, s.codes), f"{what} state{i}: codes differ"
                assert parity.bits_equal(b, s.scales), f"{what} state{i}: scales differ"
            else:
                assert parity.bits_equal(a, s.plain), f"{what} state{i}: values differ"
        if exact:
            assert parity.bits_equal(self.gp, self.p), f"{what}: parameter bits differ"
            if self.ecc is not None:
                assert parity.bits_equal(self.gecc, self.ecc), f"{what}: ECC bits differ"
            return 0.0, 0.0
        return parity.check_master(self.gp, self.gecc, self.p, self.ecc, what)


def _adam_is_exact(dtype, ecc_dtype, exact_update=False):
    """Whether Adam's update runs operation by operation on every element: asked for, or the variant's default
    (flashoptim_amd/csrc/fo_math.h: AdamExact).  The others take the guarded folded update."""
    folded = dtype != torch.float32 and (ecc_dtype is None or (dtype == torch.bfloat16 and ecc_dtype == torch.int8))
    return exact_update or not folded


def _adam_steps(n, dtype, ecc_dtype, quantized, decoupled, steps, seed, offset=0, grad_scale=1e-3, exact_update=False):
    """Returns per step (largest master-weight difference in units, fraction of elements whose master weights differ)."""
    k = _k()
    c = _Case(n, dtype, ecc_dtype, quantized, 2, seed, offset)
    lr, b1, b2, eps = 1e-3, 0.9, 0.999, 1e-8
    wd = 0.01 * lr if decoupled else 0.01
    exact = _adam_is_exact(dtype, ecc_dtype, exact_update)
    out = []
    for step in range(1, steps + 1):
        g = _rand(n, grad_scale, 1000 * seed + step).to(dtype)
        gg = c._dev(g)
        (m, ms), (v, vs) = c.gstates
        k._fused_adam_step(m, ms, v, vs, c.gp, gg, c.gecc, lr, b1, b2, eps, wd, decoupled, step, quantize_optim_states=quantized,
                           exact_update=exact_update)
        T.adam_step_ref(c.states[0], c.states[1], c.p, g, c.ecc, lr, b1, b2, eps, wd, decoupled, step)
        out.append(c.compare(f"adam n={n} {dtype} ecc={ecc_dtype} q={quantized} step={step}", exact))
        c.resync_oracle()
    return out


@pytest.mark.parametrize("dtype,ecc_dtype", VARIANTS)
@pytest.mark.parametrize("quantized", [True, False])
@pytest.mark.parametrize("decoupled", [True, False])
def test_adam_step_matches_oracle(dtype, ecc_dtype, quantized, decoupled):
    """Every variant, four steps from identical inputs: moments, codes and scales bit for bit; parameters and ECC bit
    for bit where the update runs operation by operation, within one unit of master precision (no allowance) under
    the guarded folded update."""
    for i, n in enumerate([1, 31, 33, 1000, 4096, 4097 + 4096, (1 << 16) + 17]):
        _adam_steps(n, dtype, ecc_dtype, quantized, decoupled, steps=4, seed=i + 1)


@pytest.mark.parametrize("dtype,ecc_dtype", [v for v in VARIANTS if v[0] != torch.float32])
@pytest.mark.parametrize("quantized", [True, False])
@pytest.mark.parametrize("decoupled", [True, False])
def test_adam_exact_update_is_bit_exact_for_narrow_parameters(dtype, ecc_dtype, quantized, decoupled):
    """fo_adam_step_exact: the operation-by-operation update on bf16 / fp16 parameters.  Every output bit of every
    step equals the oracle's (parameters, ECC, codes, scales), as for fp32 parameters."""
    for i, n in enumerate([1, 31, 33, 1000, 4097 + 4096, (1 << 16) + 17]):
        _adam_steps(n, dtype, ecc_dtype, quantized, decoupled, steps=4, seed=i + 1, exact_update=True)
    _adam_steps(5000, dtype, ecc_dtype, quantized, decoupled, steps=3, seed=9, offset=3, exact_update=True)


@pytest.mark.parametrize("ecc_dtype", [torch.int8, torch.int16])
def test_adam_headline_config_parity(ecc_dtype):
    """bf16 + ECC + quantised AdamW on 2^20 and 2^20+17 elements, 10 steps (the sizes of the parity sub-check of
    the throughput runs).  24-bit masters: codes and scales bit for bit, every master weight within one unit; 32-bit
    masters: every output bit."""
    for n in [1 << 20, (1 << 20) + 17]:
        stats = _adam_steps(n, torch.bfloat16, ecc_dtype, True, True, steps=10, seed=5)
        print(f"n={n} ecc={ecc_dtype}: largest master-weight difference per step (units) " + " ".join(f"{a:.2f}" for a, _ in stats)
              + "; share of master weights one unit apart " + " ".join(f"{b:.1e}" for _, b in stats))
        assert max(a for a, _ in stats) <= 1.0 + 1e-9


@pytest.mark.parametrize("dtype,ecc_dtype", [(torch.bfloat16, torch.int8), (torch.bfloat16, None), (torch.float16, None)])
def test_adam_guarded_folded_update_where_weights_are_as_small_as_their_updates(dtype, ecc_dtype):
    """The folded update differs from the reference's sequence by a few ulps of the update, which is many units of a
    weight that the update all but cancels; the kernel flags those elements and redoes them operation by operation.
    Weights drawn as small as the updates (one element in ten is flagged), a hundred times smaller, and zero: no
    master weight may be more than one unit from the oracle's, codes and scales bit for bit."""
    k = _k()
    n = (1 << 18) + 9
    lr, b1, b2, eps = 1e-3, 0.9, 0.999, 1e-8
    for weight_scale in (1e-3, 1e-5, 0.0):
        c = _Case(n, dtype, ecc_dtype, True, 2, seed=21)
        c.p.copy_(_rand(n, weight_scale, 22).to(dtype))
        c.gp.copy_(c.p.to(DEV))
        (m, ms), (v, vs) = c.gstates
        for step in range(1, 5):
            g = _rand(n, 1e-3, 500 + step).to(dtype)
            k._fused_adam_step(m, ms, v, vs, c.gp, g.to(DEV), c.gecc, lr, b1, b2, eps, 1e-5, True, step, quantize_optim_states=True)
            T.adam_step_ref(c.states[0], c.states[1], c.p, g, c.ecc, lr, b1, b2, eps, 1e-5, True, step)
            c.compare(f"adam {dtype} ecc={ecc_dtype} weights x {weight_scale:g} step {step}", exact=False)
            c.resync_oracle()


@pytest.mark.parametrize("dtype,ecc_dtype", [(torch.bfloat16, torch.int8), (torch.float16, torch.int8), (torch.bfloat16, None), (torch.bfloat16, torch.int16)])
def test_adam_groups_that_start_from_zero_get_the_exact_requantiser(dtype, ecc_dtype):
    """Two steps, then 2 % of the groups are reset to a zero state (as if they had seen no gradient yet) and a
    third step is taken: the values of a reset group sit on rounding boundaries in bulk and the quick requantiser
    forms must hand every such value to the exact form.  Every code and scale, of reset and warm groups alike,
    equals the oracle's."""
    k = _k()
    n = (1 << 17) + 17
    c = _Case(n, dtype, ecc_dtype, True, 2, seed=5)
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.999, 1e-8, 1e-5
    for step in (1, 2):
        g = _rand(n, 1e-3, 50 + step).to(dtype)
        (m, ms), (v, vs) = c.gstates
        k._fused_adam_step(m, ms, v, vs, c.gp, g.to(DEV), c.gecc, lr, b1, b2, eps, wd, True, step, quantize_optim_states=True)
    n_groups = (n + 31) // 32
    reset = torch.rand(n_groups, generator=torch.Generator().manual_seed(9)) < 0.02
    in_reset = reset.repeat_interleave(32)[:n]
    for codes, scales in c.gstates:
        codes[in_reset.to(DEV)] = 0
        scales[reset.to(DEV)] = 0
    c.resync_oracle()
    g = _rand(n, 1e-3, 77).to(dtype)
    (m, ms), (v, vs) = c.gstates
    k._fused_adam_step(m, ms, v, vs, c.gp, g.to(DEV), c.gecc, lr, b1, b2, eps, wd, True, 3, quantize_optim_states=True)
    T.adam_step_ref(c.states[0], c.states[1], c.p, g, c.ecc, lr, b1, b2, eps, wd, True, 3)
    c.compare(f"adam {dtype} ecc={ecc_dtype} after a partial reset", exact=_adam_is_exact(dtype, ecc_dtype))


def test_adam_sudden_jump_of_the_gradient_scale_keeps_the_codes_exact():
    """Three steps at gradient scale 1e-4, then one step with gradients 1 to 1e5 times larger: the old second moment
    becomes negligible, the new values sit near rounding boundaries as on a first step, and the margin test of the
    quick requantiser forms must hand them to the exact form (quick forms alone: up to 0.4 % of the codes off)."""
    k = _k()
    n = (1 << 18) + 5
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.999, 1e-8, 1e-5
    for jump in (1.0, 10.0, 30.0, 100.0, 1e3, 1e5):
        c = _Case(n, torch.bfloat16, torch.int8, True, 2, seed=3)
        (m, ms), (v, vs) = c.gstates
        for step in (1, 2, 3):
            g = _rand(n, 1e-4, 10 + step).to(torch.bfloat16)
            k._fused_adam_step(m, ms, v, vs, c.gp, g.to(DEV), c.gecc, lr, b1, b2, eps, wd, True, step, quantize_optim_states=True)
        c.resync_oracle()
        g = _rand(n, 1e-4 * jump, 99).to(torch.bfloat16)
        k._fused_adam_step(m, ms, v, vs, c.gp, g.to(DEV), c.gecc, lr, b1, b2, eps, wd, True, 4, quantize_optim_states=True)
        T.adam_step_ref(c.states[0], c.states[1], c.p, g, c.ecc, lr, b1, b2, eps, wd, True, 4)
        c.compare(f"adam after a {jump:g}-fold gradient jump", exact=False)


@pytest.mark.parametrize("betas", [(0.0, 0.999), (0.9, 0.0), (0.0, 0.0), (0.01, 0.999), (0.9, 0.1), (0.5, 0.9), (0.99, 0.9999)])
def test_adam_with_unusual_betas(betas):
    """beta1 = 0 or beta2 = 0: the old state has no weight and every step is as tie-prone as a first step."""
    k = _k()
    n = (1 << 18) + 5
    c = _Case(n, torch.bfloat16, torch.int8, True, 2, seed=3)
    (m, ms), (v, vs) = c.gstates
    for step in range(1, 5):
        g = _rand(n, 1e-3, 10 + step).to(torch.bfloat16)
        k._fused_adam_step(m, ms, v, vs, c.gp, g.to(DEV), c.gecc, 1e-3, betas[0], betas[1], 1e-8, 1e-5, True, step, quantize_optim_states=True)
        T.adam_step_ref(c.states[0], c.states[1], c.p, g, c.ecc, 1e-3, betas[0], betas[1], 1e-8, 1e-5, True, step)
        c.compare(f"adam betas {betas} step {step}", exact=False)
        c.resync_oracle()


@pytest.mark.parametrize("dtype,exact_update", [(torch.bfloat16, True), (torch.bfloat16, False), (torch.float16, False)])
def test_adam_on_lattice_valued_gradients(dtype, exact_update):
    """Sign gradients of one magnitude and gradients that are small integer multiples of a unit keep the moments on a
    coarse lattice whose ratios (1/2, 1/3, ...) sit exactly on rounding boundaries in bulk.  Codes and scales are
    promised bit for bit on any data and must be so here; parameters and ECC bit for bit where the update runs
    operation by operation (asked for on bf16, the default for fp16 with a 1-byte ECC), within one unit otherwise."""
    k = _k()
    n = (1 << 16) + 9
    lr, b1, b2, eps, wd = 1e-3, 0.5, 0.95, 1e-8, 1e-5
    for kind in ("sign", "integers"):
        c = _Case(n, dtype, torch.int8, True, 2, seed=4)
        (m, ms), (v, vs) = c.gstates
        for step, unit in enumerate((2e-3, 2e-3, 20.0, 20.0, 2e-3), start=1):
            z = _rand(n, 1.0, 300 + step)
            g = (torch.sign(z) * unit if kind == "sign" else torch.round(z) * unit).to(dtype)
            k._fused_adam_step(m, ms, v, vs, c.gp, g.to(DEV), c.gecc, lr, b1, b2, eps, wd, True, step, quantize_optim_states=True,
                               exact_update=exact_update)
            T.adam_step_ref(c.states[0], c.states[1], c.p, g, c.ecc, lr, b1, b2, eps, wd, True, step)
            c.compare(f"adam {dtype} {kind} gradients step {step}", exact=_adam_is_exact(dtype, torch.int8, exact_update))
            c.resync_oracle()


def test_adam_unaligned_pointers():
    _adam_steps(5000, torch.bfloat16, torch.int8, True, True, steps=3, seed=9, offset=3)
    _adam_steps(5000, torch.float32, None, True, True, steps=3, seed=9, offset=1)


def test_adam_large_and_tiny_gradients():
    # 1e-3-sized gradients put sqrt(v) scales into the fp16 subnormal range; 10-sized ones far above it
    _adam_steps(1 << 14, torch.bfloat16, torch.int16, True, True, steps=5, seed=11, grad_scale=10.0)
    _adam_steps(1 << 14, torch.bfloat16, torch.int8, True, True, steps=5, seed=12, grad_scale=1e-7)


MOM_MODES = {
    "lion": dict(lr=1e-4, mom_coef=0.99, update_coef=0.9, weight_decay=0.1 * 1e-4, do_lion=True),
    "sgd": dict(lr=1e-2, mom_coef=0.9, update_coef=0.9, weight_decay=1e-4),
    "sgd_nesterov": dict(lr=1e-2, mom_coef=0.9, update_coef=1.0, weight_decay=1e-4, nesterov=True),
    "sgdw": dict(lr=1e-2, mom_coef=0.9, update_coef=1.0, weight_decay=1e-4 * 1e-2, decoupled=True),
    "sgdw_nesterov": dict(lr=1e-2, mom_coef=0.9, update_coef=1.0, weight_decay=1e-4 * 1e-2, decoupled=True, nesterov=True),
}


@pytest.mark.parametrize("dtype,ecc_dtype", VARIANTS)
@pytest.mark.parametrize("quantized", [True, False])
@pytest.mark.parametrize("mode", list(MOM_MODES))
def test_momentum_step_matches_oracle(dtype, ecc_dtype, quantized, mode):
    k = _k()
    kw = MOM_MODES[mode]
    for i, n in enumerate([1, 33, 1000, 4097, (1 << 16) + 17]):
        c = _Case(n, dtype, ecc_dtype, quantized, 1, seed=20 + i)
        for step in range(1, 5):
            g = _rand(n, 1e-3, 77 * i + step).to(dtype)
            (m, ms), = c.gstates
            k._fused_momentum_step(m, ms, c.gp, g.to(DEV), c.gecc, quantize_optim_states=quantized, **kw)
            info = T.momentum_step_ref(c.states[0], c.p, g, c.ecc, **kw)
            c.compare(f"{mode} n={n} {dtype} ecc={ecc_dtype} q={quantized} step={step}", exact=True)
            c.resync_oracle()


@pytest.mark.parametrize("dtype,ecc_dtype", VARIANTS)
@pytest.mark.parametrize("decoupled,wd", [(False, 0.0), (False, 1e-2), (True, 1e-4)])
def test_plain_sgd_matches_oracle(dtype, ecc_dtype, decoupled, wd):
    k = _k()
    for i, n in enumerate([1, 33, 4097, (1 << 16) + 17]):
        c = _Case(n, dtype, ecc_dtype, False, 0, seed=40 + i)
        for step in range(1, 4):
            g = _rand(n, 1e-2, 99 * i + step).to(dtype)
            k._sgd_plain_step(c.gp, g.to(DEV), c.gecc, 1e-2, wd, decoupled)
            info = T.momentum_step_ref(None, c.p, g, c.ecc, 1e-2, 0.0, 1.0, wd, decoupled=decoupled)
            c.compare(f"plain sgd n={n} step={step}", exact=True)
            c.resync_oracle()


def test_zero_gradients_change_nothing():
    k = _k()
    n = 10000
    c = _Case(n, torch.bfloat16, torch.int8, True, 2, seed=60)
    p0 = c.gp.clone()
    (m, ms), (v, vs) = c.gstates
    for step in range(1, 4):
        k._fused_adam_step(m, ms, v, vs, c.gp, torch.zeros(n, dtype=torch.bfloat16, device=DEV), c.gecc, 1e-3, 0.9, 0.999,
                           1e-8, 0.0, True, step)
    assert torch.equal(c.gp, p0) and m.eq(0).all() and v.eq(0).all() and c.gecc.eq(0).all()
    assert ms.eq(0).all() and vs.eq(0).all()


def test_step_launches_can_be_captured_in_a_graph_and_replayed():
    """The entry points only enqueue kernels on the given stream (no allocation, no memset, no synchronisation),
    so a launch recorded into a HIP graph replays as another step.  Three replays, with eager work and
    synchronisations in between, equal three eager launches bit for bit (Lion: the step needs no step counter)."""
    k = _k()
    from flashoptim_amd.launcher import BucketPlan, StepTensors

    kw = MOM_MODES["lion"]
    lens = [5000, 33, 70001]

    def make(seed):
        ps = [(_rand(n, 0.02, seed + i)).to(torch.bfloat16).to(DEV) for i, n in enumerate(lens)]
        gs = [(_rand(n, 1e-3, seed + 10 + i)).to(torch.bfloat16).to(DEV) for i, n in enumerate(lens)]
        es = [torch.zeros(n, dtype=torch.int8, device=DEV) for n in lens]
        ms = [torch.zeros(n, dtype=torch.int8, device=DEV) for n in lens]
        ss = [torch.zeros((n + 31) // 32, dtype=torch.float16, device=DEV) for n in lens]
        return ps, gs, es, ms, ss

    eager, graphed = make(3), make(3)
    plan = BucketPlan("momentum", torch.bfloat16, 1, True,
                      [StepTensors(p, g, e, m, s) for p, g, e, m, s in zip(*graphed)])
    scalars = dict(lr=kw["lr"], mom_coef=kw["mom_coef"], update_coef=kw["update_coef"], weight_decay=kw["weight_decay"],
                   decoupled=False, nesterov=False, do_lion=True)
    plan.launch(**scalars)          # uploads the tables outside the capture; one eager step on both sides
    for p, g, e, m, s in zip(*eager):
        k._fused_momentum_step(m, s, p, g, e, **kw)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        plan.launch(**scalars)                                                    # multi-tensor launch
        k._fused_momentum_step(graphed[3][0], graphed[4][0], graphed[0][0], graphed[1][0], graphed[2][0], **kw)  # and a single one
    torch.cuda.synchronize()
    for replay in range(3):
        for p, g, e, m, s in zip(*eager):
            k._fused_momentum_step(m, s, p, g, e, **kw)
        k._fused_momentum_step(eager[3][0], eager[4][0], eager[0][0], eager[1][0], eager[2][0], **kw)
        scratch = torch.randn(1 << 16, device=DEV).sum()   # unrelated eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        assert bool(torch.isfinite(scratch))
        for group_e, group_g in zip(eager, graphed):
            for a, b in zip(group_e, group_g):
                assert parity.bits_equal(a, b), f"replay {replay}"


class _Fenced:
    """A tensor carved out of a larger buffer whose bytes before and after it hold a canary pattern."""

    PAD = 512  # bytes on each side (keeps the 16-byte alignment of the payload)

    def __init__(self, n, dtype):
        self.item = torch.empty(0, dtype=dtype).element_size()
        self.raw = torch.full((self.PAD * 2 + n * self.item,), 0x5A, dtype=torch.uint8, device=DEV)
        self.t = self.raw[self.PAD:self.PAD + n * self.item].view(dtype)
        self.t.zero_()

    def intact(self):
        return bool((self.raw[:self.PAD] == 0x5A).all()) and bool((self.raw[self.raw.numel() - self.PAD:] == 0x5A).all())


@pytest.mark.parametrize("n", [1, 31, 32, 33, 255, 256, 257, 511, 512, 513, 4095, 4096, 4097, 8191, 8193, 12288 + 40])
def test_kernels_never_write_outside_their_tensors(n):
    """Every state and parameter tensor sits between canary bytes; single-tensor and multi-tensor launches of every
    kernel family (bf16 with ECC, quantised; fp32 without ECC) leave the canaries untouched."""
    k = _k()
    from flashoptim_amd.launcher import BucketPlan, StepTensors

    groups = (n + 31) // 32
    for dtype, ecc_dtype in ((torch.bfloat16, torch.int8), (torch.bfloat16, torch.int16), (torch.float32, None)):
        def fenced_set():
            f = dict(p=_Fenced(n, dtype), g=_Fenced(n, dtype), m=_Fenced(n, torch.int8), ms=_Fenced(groups, torch.float16),
                     v=_Fenced(n, torch.uint8), vs=_Fenced(groups, torch.float16))
            f["p"].t.copy_(_rand(n, 0.02, 1).to(dtype))
            f["g"].t.copy_(_rand(n, 1e-3, 2).to(dtype))
            f["e"] = None if ecc_dtype is None else _Fenced(n, ecc_dtype)
            return f

        a, b = fenced_set(), fenced_set()
        ecc = lambda f: None if f["e"] is None else f["e"].t
        for step in (1, 2):
            k._fused_adam_step(a["m"].t, a["ms"].t, a["v"].t, a["vs"].t, a["p"].t, a["g"].t, ecc(a), 1e-3, 0.9, 0.999, 1e-8, 1e-5, True, step)
        k._fused_momentum_step(a["m"].t, a["ms"].t, a["p"].t, a["g"].t, ecc(a), **MOM_MODES["lion"])
        k._sgd_plain_step(a["p"].t, a["g"].t, ecc(a), 1e-2, 1e-4, True)
        tensors = [StepTensors(f["p"].t, f["g"].t, ecc(f), f["m"].t, f["ms"].t, f["v"].t, f["vs"].t) for f in (a, b)]
        ecc_bytes = 0 if ecc_dtype is None else torch.empty(0, dtype=ecc_dtype).element_size()
        BucketPlan("adam", dtype, ecc_bytes, True, tensors).launch(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-5, decoupled=True, step=3)
        BucketPlan("momentum", dtype, ecc_bytes, True, tensors).launch(lr=1e-2, mom_coef=0.9, update_coef=1.0, weight_decay=1e-4,
                                                                          decoupled=False, nesterov=True, do_lion=False)
        BucketPlan("plain", dtype, ecc_bytes, False, tensors).launch(lr=1e-2, weight_decay=1e-4, decoupled=False)
        torch.cuda.synchronize()
        for f in (a, b):
            for name, fenced in f.items():
                assert fenced is None or fenced.intact(), f"n={n} {dtype}: bytes next to `{name}` were overwritten"
            assert bool(torch.isfinite(f["p"].t.float()).all())


@pytest.mark.parametrize("n", [1, 33, 511, 4096, 4097, 3 * 4096 + 40, 1 << 20])
def test_access_mix_copy_changes_no_byte(n):
    """The measurement kernels that run the Adam and the momentum step's loads and stores without the arithmetic
    leave parameters, gradients, ECC, codes and scales exactly as they were, and the bytes next to them untouched
    (bf16 with both ECC widths, fp16, fp32; two tensors per launch, one of them after a real step so that no stream
    is all zero)."""
    k = _k()
    from flashoptim_amd.launcher import BucketPlan, StepTensors

    groups = (n + 31) // 32
    for dtype, ecc_dtype in ((torch.bfloat16, torch.int8), (torch.bfloat16, torch.int16), (torch.float16, torch.int8),
                             (torch.float32, None)):
        def fenced_set(seed):
            f = dict(p=_Fenced(n, dtype), g=_Fenced(n, dtype), m=_Fenced(n, torch.int8), ms=_Fenced(groups, torch.float16),
                     v=_Fenced(n, torch.uint8), vs=_Fenced(groups, torch.float16))
            f["p"].t.copy_(_rand(n, 0.02, seed).to(dtype))
            f["g"].t.copy_(_rand(n, 1e-3, seed + 1).to(dtype))
            f["e"] = None if ecc_dtype is None else _Fenced(n, ecc_dtype)
            return f

        a, b = fenced_set(1), fenced_set(3)
        ecc = lambda f: None if f["e"] is None else f["e"].t
        k._fused_adam_step(a["m"].t, a["ms"].t, a["v"].t, a["vs"].t, a["p"].t, a["g"].t, ecc(a), 1e-3, 0.9, 0.999, 1e-8, 1e-5, True, 1)
        before = [{name: fenced.raw.clone() for name, fenced in f.items() if fenced is not None} for f in (a, b)]
        tensors = [StepTensors(f["p"].t, f["g"].t, ecc(f), f["m"].t, f["ms"].t, f["v"].t, f["vs"].t) for f in (a, b)]
        ecc_bytes = 0 if ecc_dtype is None else torch.empty(0, dtype=ecc_dtype).element_size()
        plan = BucketPlan("adam", dtype, ecc_bytes, True, tensors)
        plan.launch_streams_copy()
        plan.launch_streams_copy()
        BucketPlan("momentum", dtype, ecc_bytes, True, tensors).launch_streams_copy()
        torch.cuda.synchronize()
        for f, old in zip((a, b), before):
            for name, raw in old.items():
                assert torch.equal(f[name].raw, raw), f"n={n} {dtype}: `{name}` changed under the access-mix copy"


def test_randomised_configurations_match_oracle():
    """400 seeded random configurations (kernel family, dtype, ECC width, quantisation, length, misalignment,
    hyper-parameters over several decades, gradient and weight scales from 1e-7 to 1e2, sparse gradients), three
    steps each, held to the same parity tolerances.  Degenerate draws (an fp16 second moment that underflows with a
    tiny eps, so the update overflows) must overflow identically on both sides."""
    import random

    k = _k()
    rng = random.Random(20240611)
    for case in range(400):
        dtype, ecc_dtype = rng.choice(VARIANTS)
        quantized = rng.random() < 0.7
        n = rng.choice([1, 7, 31, 32, 33, 500, 511, 512, 513, 4095, 4096, 4097, rng.randint(1, 200000)])
        offset = rng.choice([0, 0, 0, 1, 3, 8]) if dtype != torch.float32 else rng.choice([0, 0, 1, 4])
        lr, b1, b2 = 10 ** rng.uniform(-6, -1), rng.choice([0.0, 0.5, 0.9, 0.99]), rng.choice([0.9, 0.95, 0.999, 0.9999])
        eps, wdv, decoupled = 10 ** rng.uniform(-12, -4), rng.choice([0.0, 1e-4, 1e-2, 0.1]), rng.random() < 0.5
        gscale, pscale = 10 ** rng.uniform(-7, 2), 10 ** rng.uniform(-4, 1)
        kind = rng.choice(["adam", "adam", "lion", "sgd", "plain"])
        what = (f"case {case}: {kind} n={n} {dtype} ecc={ecc_dtype} q={quantized} off={offset} lr={lr:.2e} b1={b1} b2={b2} "
                f"eps={eps:.1e} wd={wdv} dec={decoupled} g={gscale:.1e} p={pscale:.1e}")
        n_states = {"adam": 2, "lion": 1, "sgd": 1, "plain": 0}[kind]
        c = _Case(n, dtype, ecc_dtype, quantized if n_states else False, n_states, seed=case + 1, offset=offset)
        c.p.copy_(_rand(n, pscale, case + 7).to(dtype))
        c.gp.copy_(c.p.to(DEV))
        for step in range(1, 4):
            g = _rand(n, gscale, 1000 * case + step).to(dtype)
            if rng.random() < 0.2:
                g[::3] = 0
            gg = c._dev(g)
            if kind == "adam":
                wd = wdv * lr if decoupled else wdv
                (m, ms), (v, vs) = c.gstates
                k._fused_adam_step(m, ms, v, vs, c.gp, gg, c.gecc, lr, b1, b2, eps, wd, decoupled, step, quantize_optim_states=quantized)
                info = T.adam_step_ref(c.states[0], c.states[1], c.p, g, c.ecc, lr, b1, b2, eps, wd, decoupled, step)
            elif kind == "plain":
                wd = wdv * lr if decoupled else wdv
                k._sgd_plain_step(c.gp, gg, c.gecc, lr, wd, decoupled)
                info = T.momentum_step_ref(None, c.p, g, c.ecc, lr, 0.0, 1.0, wd, decoupled=decoupled)
            else:
                lion = kind == "lion"
                kw = dict(lr=lr, mom_coef=b2 if lion else b1, update_coef=b1 if lion else 1.0,
                          weight_decay=wdv * lr if (decoupled or lion) else wdv, decoupled=decoupled and not lion,
                          nesterov=(not lion) and rng.random() < 0.5, do_lion=lion)
                (m, ms), = c.gstates
                k._fused_momentum_step(m, ms, c.gp, gg, c.gecc, quantize_optim_states=quantized, **kw)
                info = T.momentum_step_ref(c.states[0], c.p, g, c.ecc, **kw)
            c.compare(f"{what} step={step}", exact=kind != "adam" or _adam_is_exact(dtype, ecc_dtype))
            c.resync_oracle()


def test_step_kernels_are_resident_as_planned():
    """Every step kernel bounds the workgroups resident on a compute unit by requesting unused LDS (streaming from
    HBM degrades with too many bytes in flight per compute unit), some also by capping the wavefronts per SIMD.  The
    request is a whole number of the device's LDS allocation units; the plan (LDS units, the runtime's occupancy
    query and the cap per SIMD together) must give the intended residency for every kernel family, in both grid
    shapes, and the second residency the momentum kernels keep for lists of many short tensors."""
    import ctypes

    lib = _diag_lib()  # the same sources and flags as the product library, plus the queries
    want_adam = {(0, 0): 21, (1, 0): 16, (1, 1): 16, (1, 2): 20, (2, 0): 16, (2, 1): 20, (2, 2): 20}
    for (dtype, ecc), want_multi in want_adam.items():
        for quantized in (1, 0):
            for multi in (0, 1, 2):
                want = 18 if (dtype == 0 and multi == 0) else want_multi   # fp32: the single-tensor kernel wants fewer
                t, a, lds = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
                rc = lib.fo_adam_step_residency(dtype, ecc, quantized, 1, multi, ctypes.byref(t), ctypes.byref(a), ctypes.byref(lds))
                assert rc == 0 and t.value == want and a.value == want, (dtype, ecc, quantized, multi, t.value, a.value, lds.value)
    for kind in (0, 1, 2):
        for (dtype, ecc) in want_adam:
            for multi, want in ((0, 21), (1, 21), (2, 25)):
                t, a, lds = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
                rc = lib.fo_momentum_step_residency(dtype, ecc, 1, kind, multi, ctypes.byref(t), ctypes.byref(a), ctypes.byref(lds))
                assert rc == 0 and t.value == want and a.value == want, (kind, dtype, ecc, multi, t.value, a.value, lds.value)


def test_lds_requests_admit_the_workgroups_the_residency_plan_assumes():
    """The residency plan assumes that the device hands out LDS in units of 1280 bytes, 128 per compute unit, so that a
    workgroup asking for k units leaves room for 128 // k workgroups.  Measured here, not assumed: a probe kernel
    whose one-wavefront workgroups count themselves per compute unit is launched with requests of 4 .. 10 units (and
    with one byte more than 4 and 8 units, which must cost a whole further unit), and the largest number resident
    on any compute unit must be what the plan computes.  Then every step kernel's own request (the residency
    queries) is put through the same probe: a workgroup of the probe needs fewer registers than any step kernel, so
    the count it reaches is the bound the request enforces."""
    import ctypes

    lib = _diag_lib()
    counters = torch.zeros(8192, dtype=torch.int32, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream

    def resident(lds_bytes):
        out = ctypes.c_int()
        rc = lib.fo_probe_residency(lds_bytes, counters.data_ptr(), counters.numel() * 4, ctypes.byref(out), stream)
        assert rc == 0, lib.fo_last_error()
        return out.value

    unit = 1280
    for k in (4, 5, 6, 7, 8, 9, 10):
        assert resident(k * unit) == 128 // k, f"{k} units"
    assert resident(4 * unit + 1) == 128 // 5 and resident(8 * unit + 1) == 128 // 9
    assert resident(0) == 32                       # eight wavefronts per SIMD, four SIMDs
    seen = set()
    for dtype, ecc in ((0, 0), (1, 0), (1, 1), (1, 2), (2, 1)):
        for multi in (0, 1, 2):
            for query, extra in ((lib.fo_adam_step_residency, (1,)), (lib.fo_momentum_step_residency, (1,))):
                t, a, lds = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
                assert query(dtype, ecc, 1, *extra, multi, ctypes.byref(t), ctypes.byref(a), ctypes.byref(lds)) == 0
                static = 2048 if ecc == 1 else 1024   # the kernels' own code tables come on top of the dynamic request
                key = (lds.value + static, a.value)
                if key in seen:
                    continue
                seen.add(key)
                # the request enforces the planned residency, unless the kernel's cap per SIMD lowers it further
                got = resident(lds.value + static)
                assert got == a.value or (got > a.value and a.value % 4 == 0), (dtype, ecc, multi, lds.value, a.value, got)


def test_the_binding_shown_in_the_integration_notes_runs():
    """The ctypes stub that the integration notes print (what a maintainer of the reference would add) is executed
    as written, against the built library, and gives the same bits as this package's own binding."""
    import os
    import re

    from flashoptim_amd import _native

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "INTEGRATION.md")).read()
    block = re.search(r"```python\n(.*?)```", text, re.S).group(1)
    block = "\n".join(line[3:] if line.startswith("   ") else line for line in block.splitlines())
    block = block.replace('ctypes.CDLL("libflashoptim_hip.so")', f'ctypes.CDLL({_native.library_path()!r})')
    scope = {}
    exec(compile(block, "INTEGRATION.md", "exec"), scope)
    k = _k()
    n = 10000 + 17

    def tensors():
        p = _rand(n, 0.02, 1).to(torch.bfloat16).to(DEV)
        g = _rand(n, 1e-3, 2).to(torch.bfloat16).to(DEV)
        return (torch.zeros(n, dtype=torch.int8, device=DEV), torch.zeros((n + 31) // 32, dtype=torch.float16, device=DEV),
                torch.zeros(n, dtype=torch.uint8, device=DEV), torch.zeros((n + 31) // 32, dtype=torch.float16, device=DEV),
                p, g, torch.zeros(n, dtype=torch.int8, device=DEV))

    a, b = tensors(), tensors()
    for step in (1, 2):
        scope["_fused_adam_step"](*a, 1e-3, 0.9, 0.999, 1e-8, 1e-5, True, step)
        k._fused_adam_step(*b, 1e-3, 0.9, 0.999, 1e-8, 1e-5, True, step)
    for x, y in zip(a, b):
        assert parity.bits_equal(x, y)
