"""Pins the update math of the CPU oracle.

* With the codec and ECC bypassed (fp32 parameters, unquantised states) the Adam / AdamW / SGD steps must
  equal ``torch.optim`` -- the same library optimizers the reference's tests use as ground truth
  (/root/reference/test/test_utils.py:108-141) -- to fp32 rounding.
* Lion, SGDW and the decouple_lr variants are checked against the textbook recurrences evaluated in
  float64 (/root/reference/test/reference.py:76-93, 136-154, 215-234 state the same formulas).
* The tensor-at-a-time PyTorch restatement and the element-at-a-time C restatement must agree bit for bit
  on every variant (dtype x ECC width x quantised x optimizer), which catches a dropped term, a swapped
  coefficient or a wrong order of operations in either.
"""

import itertools

import pytest
import torch

from oracle import c_oracle as C
from oracle import torch_oracle as T


def _rand(n, scale, seed):
    return torch.randn(n, generator=torch.Generator().manual_seed(seed)) * scale


# ------------------------------------------------------------------------------ torch.optim pins


@pytest.mark.parametrize("decoupled", [True, False])
@pytest.mark.parametrize("wd", [0.0, 0.01, 0.3])
def test_adam_matches_torch_optim(decoupled, wd):
    n, lr, betas, eps = 4099, 1e-3, (0.9, 0.999), 1e-8
    p0 = _rand(n, 0.02, 0)
    ref_p = torch.nn.Parameter(p0.clone())
    opt_cls = torch.optim.AdamW if decoupled else torch.optim.Adam
    ref = opt_cls([ref_p], lr=lr, betas=betas, eps=eps, weight_decay=wd)
    p = p0.clone()
    mom = T.MomentState.zeros(n, True, False, torch.float32)
    var = T.MomentState.zeros(n, False, False, torch.float32)
    pc, mc, vc = p0.clone(), torch.zeros(n), torch.zeros(n)
    for step in range(1, 31):
        g = _rand(n, 1e-3, 100 + step)
        ref_p.grad = g.clone()
        ref.step()
        wd_arg = wd * lr if decoupled else wd  # the launcher pre-multiplies decoupled decay by lr (ref:1894-1898)
        T.adam_step_ref(mom, var, p, g, None, lr, betas[0], betas[1], eps, wd_arg, decoupled, step)
        C.adam_step(mc, None, vc, None, pc, g, None, lr, betas[0], betas[1], eps, wd_arg, decoupled, step, False)
        assert torch.equal(p, pc)
        torch.testing.assert_close(p, ref_p.data, rtol=1e-5, atol=2e-8)  # a few fp32 ulps at |p| ~ 0.05
    st = ref.state[ref_p]
    torch.testing.assert_close(mom.plain, st["exp_avg"], rtol=1e-5, atol=5e-9)  # a few fp32 ulps at the (decayed) gradient scale
    # the kernels form 1 - beta2 in fp32 from the fp32 beta2 (0.999 -> 0.99900001, so 1 - beta2 is 1.3e-5
    # smaller than 1e-3, ref:2360); torch.optim forms it in double
    torch.testing.assert_close(var.plain, st["exp_avg_sq"], rtol=3e-5, atol=1e-14)


@pytest.mark.parametrize("momentum,nesterov", [(0.9, False), (0.9, True), (0.5, False), (0.0, False)])
@pytest.mark.parametrize("wd", [0.0, 1e-2])
def test_sgd_matches_torch_optim(momentum, nesterov, wd):
    n, lr = 2053, 1e-2
    p0 = _rand(n, 0.5, 1)
    ref_p = torch.nn.Parameter(p0.clone())
    ref = torch.optim.SGD([ref_p], lr=lr, momentum=momentum, nesterov=nesterov, weight_decay=wd)
    p, pc = p0.clone(), p0.clone()
    mom = T.MomentState.zeros(n, True, False, torch.float32) if momentum > 0 else None
    mcb = torch.zeros(n)
    for step in range(1, 21):
        g = _rand(n, 0.1, 200 + step)
        ref_p.grad = g.clone()
        ref.step()
        T.momentum_step_ref(mom, p, g, None, lr, momentum, 1.0, wd, decoupled=False, nesterov=nesterov)
        if momentum > 0:
            C.momentum_step(mcb, None, pc, g, None, lr, momentum, 1.0, wd, False, nesterov, False, False)
        else:
            C.sgd_plain_step(pc, g, None, lr, wd, False)
        assert torch.equal(p, pc)
        # torch seeds its buffer with the first gradient, Flash starts from zero and applies (1 - dampening):
        # identical for dampening == 0 (ref:1496)
        torch.testing.assert_close(p, ref_p.data, rtol=1e-5, atol=1e-8)


# ------------------------------------------------------------------------------ textbook pins (float64)


def test_lion_textbook():
    n, lr, b1, b2, wd = 3001, 1e-4, 0.9, 0.99, 0.1
    p = _rand(n, 0.02, 2)
    p64, m64 = p.double(), torch.zeros(n, dtype=torch.float64)
    mom = T.MomentState.zeros(n, True, False, torch.float32)
    for step in range(1, 26):
        g = _rand(n, 1e-3, 300 + step)
        p64 = p64 * (1 - lr * wd)
        u = torch.sign(m64 * b1 + g.double() * (1 - b1))
        p64 = p64 - lr * u
        m64 = m64 * b2 + g.double() * (1 - b2)
        T.momentum_step_ref(mom, p, g, None, lr, mom_coef=b2, update_coef=b1, weight_decay=wd * lr, do_lion=True)
    torch.testing.assert_close(mom.plain.double(), m64, rtol=1e-5, atol=1e-10)
    # a sign can flip when |m*b1 + g*(1-b1)| is at rounding level; everywhere else the paths coincide
    close = (p.double() - p64).abs() <= 1e-7
    assert close.float().mean() > 0.999


@pytest.mark.parametrize("nesterov", [False, True])
def test_sgdw_textbook(nesterov):
    n, lr, mu, wd = 2000, 1e-2, 0.9, 1e-4
    p = _rand(n, 0.02, 3)
    p64, m64 = p.double(), torch.zeros(n, dtype=torch.float64)
    mom = T.MomentState.zeros(n, True, False, torch.float32)
    for step in range(1, 26):
        g = _rand(n, 1e-3, 400 + step)
        m64 = m64 * mu + g.double()
        p64 = p64 * (1 - lr * wd)
        p64 = p64 - lr * ((g.double() + mu * m64) if nesterov else m64)
        T.momentum_step_ref(mom, p, g, None, lr, mu, 1.0, wd * lr, decoupled=True, nesterov=nesterov)
    torch.testing.assert_close(p.double(), p64, rtol=1e-5, atol=2e-8)  # fp32 rounding at |p| ~ 0.05


def test_adamw_decouple_lr_textbook():
    """decouple_lr: the decay factor is weight_decay * lr / initial_lr (ref:1895-1896)."""
    n, lr0, wd, b1, b2, eps = 1500, 1e-3, 1e-2, 0.9, 0.999, 1e-8
    p = _rand(n, 0.02, 4)
    p64, m64, v64 = p.double(), torch.zeros(n).double(), torch.zeros(n).double()
    mom = T.MomentState.zeros(n, True, False, torch.float32)
    var = T.MomentState.zeros(n, False, False, torch.float32)
    for step in range(1, 16):
        lr = lr0 * (1 - step / 40)
        g = _rand(n, 1e-3, 500 + step)
        m64 = m64 * b1 + g.double() * (1 - b1)
        v64 = v64 * b2 + g.double() ** 2 * (1 - b2)
        p64 = p64 * (1 - wd * lr / lr0)
        p64 = p64 - lr * (m64 / (1 - b1**step)) / ((v64 / (1 - b2**step)).sqrt() + eps)
        T.adam_step_ref(mom, var, p, g, None, lr, b1, b2, eps, wd * (lr / lr0), True, step)
    torch.testing.assert_close(p.double(), p64, rtol=1e-5, atol=2e-8)  # fp32 rounding at |p| ~ 0.05


# ------------------------------------------------------------------------------ torch oracle == C oracle

_VARIANTS = [
    (torch.bfloat16, torch.int8), (torch.bfloat16, torch.int16), (torch.bfloat16, None),
    (torch.float16, torch.int8), (torch.float16, torch.int16), (torch.float16, None), (torch.float32, None),
]


def _bits(t):
    return None if t is None else t.contiguous().view(torch.uint8)


def _same(a, b):
    return (a is None and b is None) or torch.equal(_bits(a), _bits(b))


@pytest.mark.parametrize("dtype,ecc_dtype", _VARIANTS)
@pytest.mark.parametrize("quantized", [True, False])
@pytest.mark.parametrize("decoupled", [True, False])
def test_adam_torch_vs_c(dtype, ecc_dtype, quantized, decoupled):
    n = 32 * 40 + 13
    p = _rand(n, 0.02, 10).to(dtype)
    ecc = None if ecc_dtype is None else torch.zeros(n, dtype=ecc_dtype)
    mom, var = T.MomentState.zeros(n, True, quantized, dtype), T.MomentState.zeros(n, False, quantized, dtype)
    p2, ecc2, mom2, var2 = p.clone(), None if ecc is None else ecc.clone(), mom.clone(), var.clone()
    for step in range(1, 9):
        g = (_rand(n, 1e-3, 600 + step) * (10.0 if step == 4 else 1.0)).to(dtype)
        wd = 0.01 * 1e-3 if decoupled else 0.01
        T.adam_step_ref(mom, var, p, g, ecc, 1e-3, 0.9, 0.999, 1e-8, wd, decoupled, step)
        if quantized:
            C.adam_step(mom2.codes, mom2.scales, var2.codes, var2.scales, p2, g, ecc2, 1e-3, 0.9, 0.999, 1e-8, wd,
                        decoupled, step, True)
        else:
            C.adam_step(mom2.plain, None, var2.plain, None, p2, g, ecc2, 1e-3, 0.9, 0.999, 1e-8, wd, decoupled, step,
                        False)
        assert _same(p, p2) and _same(ecc, ecc2), step
        for a, b in ((mom, mom2), (var, var2)):
            assert _same(a.codes, b.codes) and _same(a.scales, b.scales) and _same(a.plain, b.plain), step


@pytest.mark.parametrize("dtype,ecc_dtype", _VARIANTS)
@pytest.mark.parametrize("quantized", [True, False])
@pytest.mark.parametrize("mode", ["lion", "sgd", "sgd_nesterov", "sgdw", "sgdw_nesterov"])
def test_momentum_torch_vs_c(dtype, ecc_dtype, quantized, mode):
    n = 32 * 33 + 5
    p = _rand(n, 0.02, 11).to(dtype)
    ecc = None if ecc_dtype is None else torch.zeros(n, dtype=ecc_dtype)
    mom = T.MomentState.zeros(n, True, quantized, dtype)
    p2, ecc2, mom2 = p.clone(), None if ecc is None else ecc.clone(), mom.clone()
    if mode == "lion":
        kw = dict(lr=1e-4, mom_coef=0.99, update_coef=0.9, weight_decay=0.1 * 1e-4, do_lion=True)
    else:
        dec = mode.startswith("sgdw")
        kw = dict(lr=1e-2, mom_coef=0.9, update_coef=1.0 - 0.1 * (not mode.endswith("nesterov")),
                  weight_decay=1e-4 * (1e-2 if dec else 1.0), decoupled=dec, nesterov=mode.endswith("nesterov"))
    for step in range(1, 9):
        g = _rand(n, 1e-3, 700 + step).to(dtype)
        T.momentum_step_ref(mom, p, g, ecc, **kw)
        C.momentum_step(mom2.codes if quantized else mom2.plain, mom2.scales, p2, g, ecc2, kw["lr"], kw["mom_coef"],
                        kw["update_coef"], kw["weight_decay"], kw.get("decoupled", False), kw.get("nesterov", False),
                        kw.get("do_lion", False), quantized)
        assert _same(p, p2) and _same(ecc, ecc2), step
        assert _same(mom.codes, mom2.codes) and _same(mom.scales, mom2.scales) and _same(mom.plain, mom2.plain), step


@pytest.mark.parametrize("dtype,ecc_dtype", _VARIANTS)
@pytest.mark.parametrize("decoupled,wd", [(False, 0.0), (False, 1e-2), (True, 1e-4)])
def test_plain_sgd_torch_vs_c(dtype, ecc_dtype, decoupled, wd):
    n = 777
    p = _rand(n, 0.02, 12).to(dtype)
    ecc = None if ecc_dtype is None else torch.zeros(n, dtype=ecc_dtype)
    p2, ecc2 = p.clone(), None if ecc is None else ecc.clone()
    for step in range(1, 6):
        g = _rand(n, 1e-2, 800 + step).to(dtype)
        T.momentum_step_ref(None, p, g, ecc, 1e-2, 0.0, 1.0, wd, decoupled=decoupled)
        C.sgd_plain_step(p2, g, ecc2, 1e-2, wd, decoupled)
        assert _same(p, p2) and _same(ecc, ecc2)


# ------------------------------------------------------------------------------ behavioural properties


@pytest.mark.parametrize("dtype,ecc_dtype", [(torch.bfloat16, torch.int8), (torch.float32, None)])
def test_zero_grad_leaves_everything_unchanged(dtype, ecc_dtype):
    """/root/reference/test/test_optimizers.py:186-236: zero gradients and zero decay change nothing and the
    quantised states stay exactly zero."""
    n = 1000
    p = _rand(n, 0.02, 13).to(dtype)
    p0 = p.clone()
    ecc = None if ecc_dtype is None else torch.zeros(n, dtype=ecc_dtype)
    mom, var = T.MomentState.zeros(n, True, True, dtype), T.MomentState.zeros(n, False, True, dtype)
    for step in range(1, 4):
        T.adam_step_ref(mom, var, p, torch.zeros(n, dtype=dtype), ecc, 1e-3, 0.9, 0.999, 1e-8, 0.0, True, step)
    assert torch.equal(p, p0) and mom.codes.eq(0).all() and var.codes.eq(0).all()
    assert ecc is None or ecc.eq(0).all()


def test_ecc_tracks_fp32_master_better_than_bf16_alone():
    """/root/reference/test/test_optimizers.py:865-876: after many small steps the distance to an fp32-master
    run orders as none > 24-bit > 32-bit."""
    n, steps = 4096, 100
    p_true = _rand(n, 0.02, 14).to(torch.bfloat16).float()
    runs = {}
    for name, ecc_dtype in (("none", None), ("24", torch.int8), ("32", torch.int16)):
        p = p_true.to(torch.bfloat16)
        ecc = None if ecc_dtype is None else torch.zeros(n, dtype=ecc_dtype)
        mom, var = T.MomentState.zeros(n, True, False, torch.bfloat16), T.MomentState.zeros(n, False, False, torch.bfloat16)
        runs[name] = (p, ecc, mom, var)
    pt = p_true.clone()
    mt, vt = T.MomentState.zeros(n, True, False, torch.float32), T.MomentState.zeros(n, False, False, torch.float32)
    for step in range(1, steps + 1):
        g = _rand(n, 1e-3, 900 + step)
        T.adam_step_ref(mt, vt, pt, g, None, 1e-5, 0.9, 0.999, 1e-8, 0.0, True, step)
        for p, ecc, mom, var in runs.values():
            T.adam_step_ref(mom, var, p, g.to(torch.bfloat16), ecc, 1e-5, 0.9, 0.999, 1e-8, 0.0, True, step)
    err = {}
    for name, (p, ecc, _, _) in runs.items():
        master = p.float() if ecc is None else T.ecc_join_ref(p, ecc)
        err[name] = (master - pt).pow(2).mean().item()
    assert err["none"] > err["24"] > err["32"]
