"""Full-size checks of the step kernels through properties that do not need the oracle at that size.

The update is elementwise and every 32-element group is independent, so the step on any group-aligned window of a
tensor must equal, bit for bit, the same kernel run on a copy of that window alone.  Windows are sampled across a
2^30-element tensor (the flat throughput configuration) and across a tensor longer than 2^31 elements (beyond the
reference's int32 indexing; byte offsets pass 2^32), including the ragged tail, and a few of them are also checked
against the CPU oracle with the usual parity tolerances.  Together with the small-size oracle parity this pins the
full-size runs: an indexing or overflow error at large offsets cannot survive it."""

import pytest
import torch

from oracle import torch_oracle as T
from tests import parity

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
ADAM = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-5, decoupled=True)
LION = dict(lr=1e-4, mom_coef=0.99, update_coef=0.9, weight_decay=1e-5, do_lion=True)


def _k():
    from flashoptim_amd import kernels
    return kernels


def _fill_normal(t, scale, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    chunk = 1 << 27
    for i in range(0, t.numel(), chunk):
        m = min(chunk, t.numel() - i)
        t[i:i + m] = (torch.randn(m, generator=g, device=DEV) * scale).to(t.dtype)


def _windows(n, count, width, seed, extra=()):
    g = torch.Generator().manual_seed(seed)
    starts = [int(x) * 32 for x in torch.randint(0, (n - width) // 32, (count,), generator=g)]
    starts += [0, ((n - width) // 32) * 32] + [s for s in extra if 0 <= s and s + width <= n]
    out = [(s, min(s + width, n)) for s in starts]
    out.append((((n - width // 2) // 32) * 32, n))  # ends at the ragged tail
    return out


class _State:
    def __init__(self, n, n_moments, ecc_dtype=torch.int8):
        self.n = n
        self.p = torch.empty(n, dtype=torch.bfloat16, device=DEV)
        _fill_normal(self.p, 0.02, 1)
        self.g = torch.empty(n, dtype=torch.bfloat16, device=DEV)
        self.ecc = torch.zeros(n, dtype=ecc_dtype, device=DEV)
        self.codes = [torch.zeros(n, dtype=torch.int8 if i == 0 else torch.uint8, device=DEV) for i in range(n_moments)]
        self.scales = [torch.zeros((n + 31) // 32, dtype=torch.float16, device=DEV) for _ in range(n_moments)]

    def tensors(self):
        return [self.p, self.g, self.ecc] + self.codes + self.scales

    def window(self, a, b):
        """Fresh contiguous copies of elements [a, b) (a is a multiple of 32)."""
        w = _State.__new__(_State)
        w.n = b - a
        w.p, w.g, w.ecc = self.p[a:b].clone(), self.g[a:b].clone(), self.ecc[a:b].clone()
        w.codes = [c[a:b].clone() for c in self.codes]
        w.scales = [s[a // 32:(b + 31) // 32].clone() for s in self.scales]
        return w

    def step(self, kind, step):
        k = _k()
        if kind == "adam":
            k._fused_adam_step(self.codes[0], self.scales[0], self.codes[1], self.scales[1], self.p, self.g, self.ecc,
                               ADAM["lr"], ADAM["beta1"], ADAM["beta2"], ADAM["eps"], ADAM["weight_decay"], ADAM["decoupled"], step)
        else:
            k._fused_momentum_step(self.codes[0], self.scales[0], self.p, self.g, self.ecc, **LION)


def _oracle_check(kind, before, after, step, what):
    """`before`: window inputs, `after`: the kernel's outputs for it; both on the GPU."""
    p, g, ecc = before.p.cpu(), before.g.cpu(), before.ecc.cpu()
    states = [T.MomentState(c.cpu(), s.cpu()) for c, s in zip(before.codes, before.scales)]
    if kind == "adam":
        info = T.adam_step_ref(states[0], states[1], p, g, ecc, ADAM["lr"], ADAM["beta1"], ADAM["beta2"], ADAM["eps"],
                               ADAM["weight_decay"], ADAM["decoupled"], step)
    else:
        info = T.momentum_step_ref(states[0], p, g, ecc, **LION)
    if kind != "adam":  # the momentum kernels equal the oracle bit for bit
        assert parity.bits_equal(after.p, p) and parity.bits_equal(after.ecc, ecc), f"{what}: parameter or ECC bits differ"
        assert parity.bits_equal(after.codes[0], states[0].codes) and parity.bits_equal(after.scales[0], states[0].scales), what
        return
    parity.check_master(after.p, after.ecc, p, ecc, what, step_size=info["update_scale"])
    for i in range(2):
        parity.check_codes(after.codes[i], states[i].codes, f"{what} state{i}")
        parity.check_scales(after.scales[i], states[i].scales, f"{what} state{i}")


def _run(kind, n, n_windows, extra=()):
    st = _State(n, 2 if kind == "adam" else 1)
    _fill_normal(st.g, 1e-3, 100)
    st.step(kind, 1)
    _fill_normal(st.g, 1e-3, 101)
    wins = _windows(n, n_windows, 4096 + 64, 7, extra)
    before = [st.window(a, b) for a, b in wins]
    st.step(kind, 2)
    torch.cuda.synchronize()
    for i, ((a, b), w) in enumerate(zip(wins, before)):
        snap = w.window(0, w.n) if i < 4 or i >= len(wins) - 3 else None
        w.step(kind, 2)
        full = st.window(a, b)
        for name, x, y in zip(("param", "grad", "ecc", "codes0", "codes1/scales0", "scales"), w.tensors(), full.tensors()):
            assert parity.bits_equal(x, y), f"{kind} n={n}: window [{a}, {b}) differs in {name}"
        if snap is not None:
            _oracle_check(kind, snap, w, 2, f"{kind} n={n} window [{a}, {b})")
    return st


def test_adam_step_on_2p30_elements_is_window_consistent():
    _run("adam", (1 << 30) + 17, 48)


def test_zero_gradients_leave_2p30_elements_untouched():
    """ref test_optimizers.py:186-236 at full size: with wd = 0 a zero gradient changes neither the weights nor the
    states (codes stay exactly 0)."""
    n = (1 << 30) + 17
    st = _State(n, 2)
    st.g.zero_()
    p0 = st.p.clone()
    k = _k()
    for step in (1, 2):
        k._fused_adam_step(st.codes[0], st.scales[0], st.codes[1], st.scales[1], st.p, st.g, st.ecc,
                           1e-3, 0.9, 0.999, 1e-8, 0.0, True, step)
    assert torch.equal(st.p, p0)
    assert not bool(st.ecc.any()) and not bool(st.codes[0].any()) and not bool(st.codes[1].any())


@pytest.mark.parametrize("kind", ["adam", "lion"])
def test_step_beyond_2p31_elements_is_window_consistent(kind):
    n = (1 << 31) + (1 << 20) + 5
    near = (1 << 31) - 2048  # windows straddling element 2^31 (and byte offset 2^32 of the 2-byte streams)
    _run(kind, n, 24, extra=(near, near + 4096, (1 << 31), (1 << 31) + 32 * 1001))


def test_ragged_4096_tensor_launch_equals_per_tensor_launches():
    """The ragged configuration at full size (4096 bf16 tensors, lengths log-uniform in [1, 2^24], about 1e9
    elements, FlashLion): one multi-tensor launch per step is bit-identical to 4096 single-tensor launches."""
    import warnings

    import flashoptim_amd as fo

    g = torch.Generator().manual_seed(3)
    lens = torch.floor(torch.exp2(24.0 * torch.rand(4096, generator=g, dtype=torch.float64))).clamp(1, 1 << 24)
    lens = torch.floor(lens * (1.0e9 / lens.sum().item())).clamp(1, 1 << 24).to(torch.int64).tolist()
    lens[:3] = [1, 31, 33]
    dg = torch.Generator(device=DEV).manual_seed(5)
    pa = [torch.nn.Parameter((torch.randn(n, generator=dg, device=DEV) * 0.02).to(torch.bfloat16)) for n in lens]
    pb = [torch.nn.Parameter(p.detach().clone()) for p in pa]
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        oa = fo.FlashLion(pa, lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1, master_weight_bits=24)
        ob = fo.FlashLion(pb, lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1, master_weight_bits=24)
    for it in range(2):
        for a, b in zip(pa, pb):
            a.grad = (torch.randn(a.numel(), generator=dg, device=DEV) * 1e-3).to(torch.bfloat16)
            b.grad = a.grad.clone()
        oa.step()
        for p in pb:
            ob.step_param(p)
    for a, b in zip(pa, pb):
        assert torch.equal(a, b)
        sa, sb = oa.state[a], ob.state[b]
        assert torch.equal(sa["error_bits"], sb["error_bits"])
        assert torch.equal(sa["exp_avg"].quantized, sb["exp_avg"].quantized)
        assert parity.bits_equal(sa["exp_avg"].scales, sb["exp_avg"].scales)


def _llama3_8b_lengths():
    h, ffn, kv, vocab = 4096, 14336, 1024, 128256
    lens = [vocab * h]
    for _ in range(32):
        lens += [h * h, kv * h, kv * h, h * h, ffn * h, ffn * h, h * ffn, h, h]
    return lens + [h, vocab * h]


@pytest.mark.parametrize("mwb", [32, 24])
def test_llama8b_multi_tensor_launch_equals_per_tensor_launches(mwb):
    """The 8B configuration at full size (291 bf16 tensors of Llama-3-8B's shapes, 8 030 261 248 elements, FlashAdamW
    with 32-bit and with 24-bit master weights): one multi-tensor launch per step is bit-identical to 291
    single-tensor launches, and every tensor moved."""
    import gc
    import warnings

    import flashoptim_amd as fo

    lens = _llama3_8b_lengths()
    assert len(lens) == 291 and sum(lens) == 8_030_261_248
    dg = torch.Generator(device=DEV).manual_seed(11)
    pa = []
    for n in lens:
        p = torch.empty(n, dtype=torch.bfloat16, device=DEV)
        for i in range(0, n, 1 << 27):
            m = min(1 << 27, n - i)
            p[i:i + m] = (torch.randn(m, generator=dg, device=DEV) * 0.02).to(torch.bfloat16)
        pa.append(torch.nn.Parameter(p))
    pb = [torch.nn.Parameter(p.detach().clone()) for p in pa]
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        oa = fo.FlashAdamW(pa, lr=1e-3, weight_decay=0.01, master_weight_bits=mwb)
        ob = fo.FlashAdamW(pb, lr=1e-3, weight_decay=0.01, master_weight_bits=mwb)
    for it in range(2):
        for a, b in zip(pa, pb):
            if a.grad is None:
                a.grad = torch.empty_like(a)
            for i in range(0, a.numel(), 1 << 27):
                m = min(1 << 27, a.numel() - i)
                a.grad[i:i + m] = (torch.randn(m, generator=dg, device=DEV) * 1e-3).to(torch.bfloat16)
            b.grad = a.grad          # read-only for the kernels: both optimizers may share it
        oa.step()
        for p in pb:
            ob.step_param(p)
    torch.cuda.synchronize()
    for a, b in zip(pa, pb):
        assert torch.equal(a, b)
        sa, sb = oa.state[a], ob.state[b]
        assert sa["error_bits"].dtype == (torch.int16 if mwb == 32 else torch.int8)
        assert torch.equal(sa["error_bits"], sb["error_bits"])
        for name in ("exp_avg", "exp_avg_sq"):
            assert torch.equal(sa[name].quantized, sb[name].quantized)
            assert parity.bits_equal(sa[name].scales, sb[name].scales)
        assert bool(sa["exp_avg"].quantized.any()) and float(sa["step"]) == 2.0
    del oa, ob, pa, pb
    gc.collect()
    torch.cuda.empty_cache()
