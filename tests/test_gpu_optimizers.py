"""GPU tests of the optimizer layer (host Python over the HIP kernels): the plumbing configuration against an
oracle-driven optimizer, multi-tensor == per-tensor launches, state_dict layouts and round trips, gradient
release, fp32 export/import, and the behavioural thresholds of the reference's own optimizer tests
(/root/reference/test/test_optimizers.py, test_serialization.py, test_training.py; cited per test)."""

import copy
import io
import warnings

import pytest
import torch
import torch.nn as nn

from oracle import torch_oracle as T
from tests import parity

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _fo():
    import flashoptim_amd

    return flashoptim_amd


def _mlp(seed=0):
    torch.manual_seed(seed)
    return nn.Sequential(nn.Linear(128, 256), nn.ReLU(), nn.Linear(256, 10))


class OracleAdamW:
    """Steps GPU parameters with the CPU oracle (test double for FlashAdamW(master_weight_bits=24, quantize=True))."""

    def __init__(self, params, lr, betas, eps, weight_decay, ecc_dtype=torch.int8):
        self.params = list(params)
        self.hp = (lr, betas[0], betas[1], eps, weight_decay * lr)
        self.t = 0
        self.state = []
        for p in self.params:
            n = p.numel()
            self.state.append(dict(
                p=p.detach().cpu().reshape(-1).clone(), ecc=torch.zeros(n, dtype=ecc_dtype),
                m=T.MomentState.zeros(n, True, True, p.dtype), v=T.MomentState.zeros(n, False, True, p.dtype)))

    def step(self):
        self.t += 1
        lr, b1, b2, eps, wd = self.hp
        for p, s in zip(self.params, self.state):
            g = p.grad.detach().cpu().reshape(-1)
            T.adam_step_ref(s["m"], s["v"], s["p"], g, s["ecc"], lr, b1, b2, eps, wd, True, self.t)
            p.data.copy_(s["p"].view(p.shape))


def test_config0_loss_trajectory_matches_oracle():
    """README MLP, FlashAdamW(mwb=24) for 100 steps, x ~ N(0,1) [32,128], loss = sum of outputs.  The fp32 loss
    trajectory of the HIP-stepped model must stay within 1e-3 relative of the oracle-stepped one (free running,
    no resynchronisation)."""
    fo = _fo()
    x = torch.randn(32, 128, generator=torch.Generator().manual_seed(0)).to(DEV, torch.bfloat16)
    model_a, model_b = _mlp().to(DEV), _mlp().to(DEV)
    fo.cast_model(model_a)
    fo.cast_model(model_b)
    hp = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    opt_a = fo.FlashAdamW(model_a.parameters(), master_weight_bits=24, **hp)
    opt_b = OracleAdamW(model_b.parameters(), **hp)
    sizes = sorted(p.numel() for p in model_a.parameters())
    assert sizes == [10, 256, 2560, 32768] and sum(sizes) == 35594
    worst = 0.0
    for step in range(100):
        losses = []
        for model, opt in ((model_a, opt_a), (model_b, opt_b)):
            for p in model.parameters():
                p.grad = None
            loss = model(x).float().sum()
            loss.backward()
            opt.step()
            losses.append(loss.item())
        rel = abs(losses[0] - losses[1]) / max(abs(losses[1]), 1e-6)
        worst = max(worst, rel)
        assert rel <= 1e-3, f"step {step}: loss {losses[0]} vs oracle {losses[1]}"
    assert losses[0] < -1000  # the sum of outputs is driven down steadily
    print(f"config 0: worst relative loss difference over 100 steps {worst:.3e}; final loss {losses[0]:.4f}")
    # end state of two free-running trajectories: the displacement of the master weights over the 100 steps agrees
    # in aggregate (single elements whose gradient is rounding noise wander, Adam normalises them to +-lr)
    init = _mlp()
    fo.cast_model(init)
    for p, s, p0 in zip(model_a.parameters(), opt_b.state, init.parameters()):
        st = opt_a.state[p]
        start = p0.detach().float().reshape(-1)
        d_a = T.ecc_join_ref(p.detach().cpu().reshape(-1), st["error_bits"].cpu().reshape(-1)) - start
        d_b = T.ecc_join_ref(s["p"], s["ecc"]) - start
        assert torch.cosine_similarity(d_a, d_b, dim=0).item() > 0.999
        assert ((d_a - d_b) ** 2).mean().item() / (d_b**2).mean().item() < 5e-4
        assert (st["exp_avg"].quantized.cpu().reshape(-1).int() - s["m"].codes.int()).abs().float().mean() < 1.0


@pytest.mark.parametrize("bits,ecc_dtype", [(24, torch.int8), (32, torch.int16)])
def test_config0_with_exact_update_equals_the_oracle_bit_for_bit(bits, ecc_dtype):
    """FlashAdamW(exact_update=True) on the README MLP (bf16 parameters; one multi-tensor launch per step through
    fo_multi_adam_step_exact), free running for 50 steps next to the oracle-stepped copy: the losses are equal and
    in the end every parameter, ECC code, moment code and scale is the oracle's, bit for bit."""
    fo = _fo()
    x = torch.randn(32, 128, generator=torch.Generator().manual_seed(0)).to(DEV, torch.bfloat16)
    model_a, model_b = _mlp().to(DEV), _mlp().to(DEV)
    fo.cast_model(model_a)
    fo.cast_model(model_b)
    hp = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    opt_a = fo.FlashAdamW(model_a.parameters(), master_weight_bits=bits, exact_update=True, **hp)
    opt_b = OracleAdamW(model_b.parameters(), ecc_dtype=ecc_dtype, **hp)
    for step in range(50):
        losses = []
        for model, opt in ((model_a, opt_a), (model_b, opt_b)):
            for p in model.parameters():
                p.grad = None
            loss = model(x).float().sum()
            loss.backward()
            opt.step()
            losses.append(loss.item())
        assert losses[0] == losses[1], f"step {step}: loss {losses[0]} vs oracle {losses[1]}"
    for p, s in zip(model_a.parameters(), opt_b.state):
        st = opt_a.state[p]
        assert parity.bits_equal(p.detach().reshape(-1), s["p"])
        assert parity.bits_equal(st["error_bits"].reshape(-1), s["ecc"])
        assert parity.bits_equal(st["exp_avg"].quantized.reshape(-1), s["m"].codes)
        assert parity.bits_equal(st["exp_avg"].scales.reshape(-1)[:s["m"].scales.numel()], s["m"].scales)
        assert parity.bits_equal(st["exp_avg_sq"].quantized.reshape(-1), s["v"].codes)
        assert parity.bits_equal(st["exp_avg_sq"].scales.reshape(-1)[:s["v"].scales.numel()], s["v"].scales)


def test_exact_update_defaults_to_the_environment_variable(monkeypatch):
    fo = _fo()
    p = [nn.Parameter(torch.zeros(8, dtype=torch.bfloat16, device=DEV))]
    assert fo.FlashAdamW(p)._exact_update is False
    monkeypatch.setenv("FLASHOPTIM_EXACT_ADAM", "1")
    assert fo.FlashAdamW(p)._exact_update is True
    assert fo.FlashAdam(p, exact_update=False)._exact_update is False


# ------------------------------------------------------------------------------ multi-tensor launcher

_RAGGED = [1, 31, 32, 33, 1000, 4096, 4097, 12289, 70001, 3, 262144 + 7]


def _make_params(shapes, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    out = []
    for n in shapes:
        p = nn.Parameter((torch.randn(n, generator=g) * 0.02).to(dtype).to(DEV))
        out.append(p)
    return out


def _set_grads(params, seed, scale=1e-3):
    g = torch.Generator().manual_seed(seed)
    for p in params:
        p.grad = (torch.randn(p.shape, generator=g) * scale).to(p.dtype).to(DEV)


def _state_tensors(opt, p):
    from flashoptim_amd.optimizers import _MaybeQuantizedTensor

    out = {}
    for k, v in opt.state[p].items():
        if isinstance(v, _MaybeQuantizedTensor):
            if v.is_quantized():
                out[k + "::q"], out[k + "::s"] = v.quantized, v.scales
            else:
                out[k] = v.data
        elif isinstance(v, torch.Tensor):
            out[k] = v
    return out


@pytest.mark.parametrize("factory,kwargs", [
    ("FlashAdamW", dict(lr=1e-3, weight_decay=0.01)),
    ("FlashAdam", dict(lr=1e-3, weight_decay=0.01)),
    ("FlashLion", dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1)),
    ("FlashSGDW", dict(lr=1e-2, momentum=0.9, weight_decay=1e-4)),
    ("FlashSGD", dict(lr=1e-2, momentum=0.9, nesterov=True, weight_decay=1e-4)),
])
@pytest.mark.parametrize("dtype,mwb,quantize", [(torch.bfloat16, 24, True), (torch.bfloat16, 32, True),
                                                (torch.float32, None, True), (torch.float16, 24, False)])
def test_multi_tensor_step_is_bit_identical_to_per_tensor_steps(factory, kwargs, dtype, mwb, quantize):
    fo = _fo()
    pa, pb = _make_params(_RAGGED, dtype, 1), _make_params(_RAGGED, dtype, 1)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        oa = getattr(fo, factory)(pa, master_weight_bits=mwb, quantize=quantize, **kwargs)
        ob = getattr(fo, factory)(pb, master_weight_bits=mwb, quantize=quantize, **kwargs)
    for it in range(3):
        _set_grads(pa, 10 + it)
        _set_grads(pb, 10 + it)
        oa.step()                       # one multi-tensor launch per bucket
        for p in pb:                    # one single-tensor launch per parameter
            ob.step_param(p)
    for a, b in zip(pa, pb):
        assert torch.equal(a, b)
        sa, sb = _state_tensors(oa, a), _state_tensors(ob, b)
        assert sorted(sa) == sorted(sb)
        for k in sa:
            assert parity.bits_equal(sa[k], sb[k]), (factory, k, a.numel())


def test_multi_tensor_handles_mixed_groups_dtypes_and_missing_grads():
    fo = _fo()
    bf = _make_params([5000, 77], torch.bfloat16, 2)
    fp = _make_params([4097, 64], torch.float32, 3)
    frozen = _make_params([100], torch.bfloat16, 4)
    groups = [dict(params=bf, lr=1e-3), dict(params=fp + frozen, lr=5e-4, weight_decay=0.0)]
    opt = fo.FlashAdamW(groups, master_weight_bits=24)
    before = [p.detach().clone() for p in bf + fp + frozen]
    _set_grads(bf + fp, 5)
    opt.step()
    for p, b in zip(bf + fp, before):
        assert not torch.equal(p, b)
    assert torch.equal(frozen[0], before[-1])
    assert "exp_avg" in opt.state[frozen[0]]          # state exists even without a gradient (ref:710-714)
    assert "error_bits" in opt.state[bf[0]] and "error_bits" not in opt.state[fp[0]]
    assert opt.state[bf[0]]["error_bits"].dtype == torch.int8
    assert opt.state[bf[0]]["step"].item() == 1 and opt.state[bf[0]]["step"].device.type == "cpu"


# ------------------------------------------------------------------------- behaviour (reference thresholds)


@pytest.mark.parametrize("factory,kwargs,names", [
    ("FlashAdamW", dict(lr=1e-2), ["exp_avg", "exp_avg_sq"]),
    ("FlashLion", dict(lr=1e-2), ["exp_avg"]),
    ("FlashSGD", dict(lr=1e-2, momentum=0.9), ["momentum_buffer"]),
])
def test_zero_grads_leave_weights_and_states_untouched(factory, kwargs, names):
    """/root/reference/test/test_optimizers.py:186-236."""
    fo = _fo()
    params = _make_params([4096, 333], torch.bfloat16, 6)
    opt = getattr(fo, factory)(params, weight_decay=0.0, **kwargs)
    before = [p.detach().clone() for p in params]
    for _ in range(3):
        for p in params:
            p.grad = torch.zeros_like(p)
        opt.step()
    for p, b in zip(params, before):
        assert torch.equal(p, b)
        for n in names:
            assert opt.state[p][n].quantized.eq(0).all() and opt.state[p][n].materialize().eq(0).all()


@pytest.mark.parametrize("factory,kwargs", [
    ("FlashAdamW", dict(lr=1e-2)), ("FlashAdam", dict(lr=1e-2)), ("FlashLion", dict(lr=1e-3)),
    ("FlashSGD", dict(lr=1e-1, momentum=0.9)), ("FlashSGDW", dict(lr=1e-1, momentum=0.9, nesterov=True)),
    ("FlashSGD", dict(lr=1e-1)),
])
@pytest.mark.parametrize("dtype,mwb", [(torch.bfloat16, 24), (torch.bfloat16, 32), (torch.float32, None)])
def test_descends_on_a_quadratic(factory, kwargs, dtype, mwb):
    """/root/reference/test/test_optimizers.py:250-321: the loss of a toy regression falls monotonically."""
    fo = _fo()
    torch.manual_seed(0)
    w = nn.Parameter((torch.randn(64, 64) * 0.5).to(dtype).to(DEV))
    x = torch.randn(256, 64, device=DEV)
    y = x @ torch.randn(64, 64, device=DEV) * 0.1
    opt = getattr(fo, factory)([w], master_weight_bits=mwb, **kwargs)
    losses = []
    for _ in range(10):
        opt.zero_grad()
        loss = ((x @ w.float() - y) ** 2).mean()
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert all(b < a for a, b in zip(losses, losses[1:])), losses


def test_quantised_run_tracks_an_fp32_run():
    """/root/reference/test/test_optimizers.py:540-578: quantised bf16+ECC vs plain fp32 torch.optim.AdamW after 20
    steps: cosine similarity of the weight change > 0.975 and NMSE < 0.05."""
    fo = _fo()
    torch.manual_seed(1)
    w0 = torch.randn(256, 128) * 0.02
    w_ref = nn.Parameter(w0.clone().to(DEV))
    w_fo = nn.Parameter(w0.clone().to(torch.bfloat16).to(DEV))
    ref = torch.optim.AdamW([w_ref], lr=1e-3, weight_decay=0.01)
    opt = fo.FlashAdamW([w_fo], lr=1e-3, weight_decay=0.01, master_weight_bits=24)
    for it in range(20):
        g = torch.randn(256, 128, generator=torch.Generator().manual_seed(100 + it)).to(DEV) * 1e-2
        w_ref.grad, w_fo.grad = g.clone(), g.to(torch.bfloat16)
        ref.step()
        opt.step()
    d_ref = (w_ref.detach() - w0.to(DEV)).reshape(-1)
    master = fo.reconstruct_fp32_param(w_fo.detach(), opt.state[w_fo]["error_bits"])
    d_fo = (master - w0.to(torch.bfloat16).float().to(DEV)).reshape(-1)
    assert torch.cosine_similarity(d_ref, d_fo, dim=0).item() > 0.975
    assert ((d_ref - d_fo) ** 2).mean().item() / (d_ref**2).mean().item() < 0.05


def test_ecc_orders_precision():
    """/root/reference/test/test_optimizers.py:865-876: distance to an fp32 run orders none > 24-bit > 32-bit."""
    fo = _fo()
    torch.manual_seed(2)
    w0 = (torch.randn(512, 512) * 0.02).to(torch.bfloat16)
    ref_w = nn.Parameter(w0.float().to(DEV))
    ref = torch.optim.AdamW([ref_w], lr=1e-5, weight_decay=0.0)
    runs = {}
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        for mwb in (None, 24, 32):
            w = nn.Parameter(w0.clone().to(DEV))
            runs[mwb] = (w, fo.FlashAdamW([w], lr=1e-5, weight_decay=0.0, master_weight_bits=mwb, quantize=False))
    for it in range(100):
        g = (torch.randn(512, 512, generator=torch.Generator().manual_seed(it)) * 1e-3).to(DEV)
        ref_w.grad = g
        ref.step()
        for w, opt in runs.values():
            w.grad = g.to(torch.bfloat16)
            opt.step()
    err = {}
    for mwb, (w, opt) in runs.items():
        st = opt.state[w]
        master = w.detach().float() if "error_bits" not in st else fo.reconstruct_fp32_param(w.detach(), st["error_bits"])
        err[mwb] = ((master - ref_w.detach()) ** 2).mean().item()
    assert err[None] > err[24] > err[32], err
    assert opt.state[w]["error_bits"].dtype == torch.int16 and runs[24][1].state[runs[24][0]]["error_bits"].dtype == torch.int8


def test_sgd_zero_momentum_matches_torch_sgd():
    """/root/reference/test/test_optimizers.py:1384-1449 (rtol 1e-5, fp32, no state tensor)."""
    fo = _fo()
    w0 = torch.randn(1000, generator=torch.Generator().manual_seed(3))
    a, b = nn.Parameter(w0.clone().to(DEV)), nn.Parameter(w0.clone().to(DEV))
    ours = fo.FlashSGD([a], lr=1e-2, momentum=0.0, weight_decay=1e-2, master_weight_bits=None)
    ref = torch.optim.SGD([b], lr=1e-2, momentum=0.0, weight_decay=1e-2)
    for it in range(5):
        g = torch.randn(1000, generator=torch.Generator().manual_seed(50 + it)).to(DEV)
        a.grad, b.grad = g.clone(), g.clone()
        ours.step()
        ref.step()
    torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-7)
    assert "momentum_buffer" not in ours.state[a]


def test_multi_param_group_uses_each_groups_lr():
    """/root/reference/test/test_optimizers.py:1458-1497."""
    fo = _fo()
    p1, p2 = _make_params([4096], torch.bfloat16, 7)[0], _make_params([4096], torch.bfloat16, 7)[0]
    opt = fo.FlashLion([dict(params=[p1], lr=1e-3), dict(params=[p2], lr=1e-2)], weight_decay=0.0)
    before = p1.detach().float().clone()
    _set_grads([p1, p2], 8)
    opt.step()
    m1 = fo.reconstruct_fp32_param(p1.detach(), opt.state[p1]["error_bits"]) - before
    m2 = fo.reconstruct_fp32_param(p2.detach(), opt.state[p2]["error_bits"]) - before
    torch.testing.assert_close(m1.abs().mean() * 10, m2.abs().mean(), rtol=2e-2, atol=0)


def test_check_numerics_raises_when_lr_cannot_move_the_weights():
    """/root/reference/test/test_optimizers.py:594-632."""
    fo = _fo()
    from flashoptim_amd.optimizers import _BITS_TO_BYTES, _log2_min_expressible_step_size
    import math

    for mwb in (None, 24, 32):
        for maxabs in (1.0, 1e2, 1e-2):
            for lr in (1e-1, 1e-3, 1e-7):
                w = nn.Parameter(((torch.randint(0, 2, (1024,)) * 2 - 1) * maxabs).to(torch.bfloat16).to(DEV))
                with warnings.catch_warnings():
                    warnings.simplefilter("ignore")
                    opt = fo.FlashLion([w], lr=lr, check_numerics=True, master_weight_bits=mwb)
                w.grad = torch.ones_like(w)
                need = _log2_min_expressible_step_size(torch.bfloat16, float(w.detach().abs().max()), _BITS_TO_BYTES[mwb])
                if math.log2(lr) < need:
                    with pytest.raises(fo.NumericsError):
                        opt.step()
                else:
                    opt.step()


def test_error_paths():
    fo = _fo()
    w = nn.Parameter(torch.randn(8, 8, device=DEV, dtype=torch.bfloat16).t())  # non-contiguous
    opt = fo.FlashAdamW([w])
    w.grad = torch.zeros(8, 8, device=DEV, dtype=torch.bfloat16).t()
    with pytest.raises(RuntimeError, match="contiguous parameters"):
        opt.step()
    w2 = nn.Parameter(torch.randn(8, 8, device=DEV, dtype=torch.bfloat16))
    opt2 = fo.FlashAdamW([w2])
    w2.grad = torch.zeros(8, 8, device=DEV, dtype=torch.bfloat16).t()
    with pytest.raises(RuntimeError, match="contiguous gradients"):
        opt2.step()
    with pytest.raises(ValueError, match="no effect when all parameters are fp32"):
        fo.FlashAdamW([nn.Parameter(torch.zeros(4, device=DEV))], master_weight_bits=24)
    with pytest.warns(UserWarning, match="pure low-precision"):
        fo.FlashAdamW([nn.Parameter(torch.zeros(4, device=DEV, dtype=torch.bfloat16))], master_weight_bits=None)
    with pytest.warns(UserWarning, match="fused=False"):
        fo.FlashAdamW([nn.Parameter(torch.zeros(4, device=DEV, dtype=torch.bfloat16))], fused=False)
    with pytest.raises(ValueError, match="not managed"):
        opt2.step_param(nn.Parameter(torch.zeros(2, device=DEV)))
    empty = nn.Parameter(torch.zeros(0, device=DEV, dtype=torch.bfloat16))
    opt3 = fo.FlashAdamW([empty])
    empty.grad = torch.zeros_like(empty)
    opt3.step()
    assert "exp_avg" in opt3.state[empty]
    assert "FlashOptim Config" in repr(opt3) and "master_bytewidth: 3" in repr(opt3)


def test_launch_wrappers_reject_operands_the_kernels_would_overrun():
    """The kernels see raw addresses only; shapes, dtypes and devices that do not fit are refused on the host, before
    anything is launched."""
    from flashoptim_amd import kernels as K

    n = 1000
    groups = (n + 31) // 32
    bf = dict(device=DEV, dtype=torch.bfloat16)
    p, g = torch.zeros(n, **bf), torch.zeros(n, **bf)
    m, v = torch.zeros(n, device=DEV, dtype=torch.int8), torch.zeros(n, device=DEV, dtype=torch.uint8)
    sm, sv = torch.zeros(groups, device=DEV, dtype=torch.float16), torch.zeros(groups, device=DEV, dtype=torch.float16)
    ecc = torch.zeros(n, device=DEV, dtype=torch.int8)
    hp = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0, decoupled=True, step=1)

    def adam(**over):
        a = dict(mom=m, mom_scales_f16=sm, var=v, var_scales_f16=sv, param=p, grad=g, errors=ecc)
        a.update(over)
        K._fused_adam_step(**a, **hp)

    adam()  # the well-formed call goes through
    for over, match in [
        (dict(mom=m[:-1]), "mom must be contiguous with as many elements"),
        (dict(var=v.to(torch.int8)), "quantised var must be uint8"),
        (dict(mom_scales_f16=sm[:-1]), "mom scales hold"),
        (dict(var_scales_f16=sv.float()), "var scales must be a contiguous fp16"),
        (dict(var_scales_f16=sv.cpu()), "var scales is on cpu"),
        (dict(errors=ecc[:-1]), "error_bits and param"),
        (dict(errors=ecc.cpu()), "error_bits is on cpu"),
        (dict(grad=g.float()), "grad dtype"),
        (dict(grad=g[:-1]), "same number of elements"),
    ]:
        with pytest.raises(ValueError, match=match):
            adam(**over)
    with pytest.raises(RuntimeError, match="contiguous"):
        adam(grad=torch.zeros(2 * n, **bf)[::2])
    with pytest.raises(ValueError, match="unquantised momentum must have the parameter's dtype"):
        K._fused_momentum_step(torch.zeros(n, device=DEV), None, p, g, None, 1e-3, 0.9, 1.0, 0.0,
                               quantize_optim_states=False)
    with pytest.raises(ValueError, match="out_scales is on cpu"):
        K.quantize(torch.zeros(n, device=DEV), out_scales=torch.zeros(groups, dtype=torch.float16))
    with pytest.raises(ValueError, match="in_scales is on cpu"):
        K.dequantize(m, sm.cpu())
    with pytest.raises(ValueError, match="error_bits is on cpu"):
        K.reconstruct_fp32_param(p, ecc.cpu())
    with pytest.raises(ValueError, match="dst is on cpu"):
        K.copy_bytes(torch.zeros(n, dtype=torch.int8), m)
    assert torch.count_nonzero(p) == 0 and torch.count_nonzero(m) == 0   # zero gradients: nothing moved


# --------------------------------------------------------------------------------------- state dicts


def _train(opt, params, n, seed):
    for it in range(n):
        _set_grads(params, seed + it)
        opt.step()


@pytest.mark.parametrize("factory,kwargs,names", [
    ("FlashAdamW", dict(lr=1e-3), ["exp_avg", "exp_avg_sq"]),
    ("FlashLion", dict(lr=1e-4), ["exp_avg"]),
    ("FlashSGDW", dict(lr=1e-2, momentum=0.9), ["momentum_buffer"]),
])
@pytest.mark.parametrize("dtype,mwb", [(torch.float32, None), (torch.bfloat16, 24), (torch.bfloat16, 32),
                                       (torch.float16, 24), (torch.float16, 32)])
def test_compressed_state_dict_layout_and_round_trip(factory, kwargs, names, dtype, mwb):
    """Keys `<name>::quantized` / `<name>::scales`, int8/uint8 + fp16; codes survive any parameter dtype, fp16
    scales survive fp32/fp16 parameters bit for bit and pass through bf16 for bf16 parameters; ECC restored with
    its integer dtype (/root/reference/test/test_serialization.py:134-207)."""
    fo = _fo()
    params = _make_params([5000, 33, 4096], dtype, 11)
    opt = getattr(fo, factory)(params, compress_state_dict=True, master_weight_bits=mwb, **kwargs)
    _train(opt, params, 3, 20)
    sd = opt.state_dict()
    entry = sd["state"][0]
    for n in names:
        assert n not in entry
        assert entry[n + "::quantized"].dtype == (torch.uint8 if n == "exp_avg_sq" else torch.int8)
        assert entry[n + "::quantized"].shape == params[0].shape
        assert entry[n + "::scales"].dtype == torch.float16 and entry[n + "::scales"].numel() == (5000 + 31) // 32
    if mwb is not None:
        assert entry["error_bits"].dtype == dtype and entry["error_bits"].shape == params[0].shape
    assert sd["param_groups"][0]["master_bytewidth"] == {None: 0, 24: 3, 32: 4}[mwb]
    assert sd["param_groups"][0]["quantize"] is True and "initial_lr" in sd["param_groups"][0]
    assert "fused" not in sd["param_groups"][0]

    buf = io.BytesIO()
    torch.save(sd, buf)
    buf.seek(0)
    loaded = torch.load(buf, weights_only=True)
    new = getattr(fo, factory)(params, compress_state_dict=True, master_weight_bits=mwb, **kwargs)
    new.load_state_dict(loaded)
    for p in params:
        a, b = opt.state[p], new.state[p]
        assert sorted(a) == sorted(b)
        for n in names:
            assert torch.equal(a[n].quantized, b[n].quantized)
            if dtype == torch.bfloat16:
                torch.testing.assert_close(a[n].scales, b[n].scales, atol=1e-3, rtol=1e-2)
            else:
                assert parity.bits_equal(a[n].scales, b[n].scales)
        if mwb is not None:
            assert b["error_bits"].dtype == (torch.int8 if mwb == 24 else torch.int16)
            assert torch.equal(a["error_bits"], b["error_bits"])
        if "step" in a:
            assert a["step"].item() == b["step"].item() == 3 and b["step"].device.type == "cpu"
    _train(new, params, 1, 30)
    assert all(p.isfinite().all() for p in params)


def test_uncompressed_state_dict_interoperates_with_torch_adamw():
    """/root/reference/test/test_serialization.py:81-132: bf16 tensors under torch's own key names."""
    fo = _fo()
    params = _make_params([3000, 64], torch.float32, 12)
    opt = fo.FlashAdamW(params, lr=0.1, master_weight_bits=None)
    _train(opt, params, 2, 40)
    sd = opt.state_dict()
    assert sd["state"][0]["exp_avg"].dtype == torch.bfloat16 and sd["state"][0]["exp_avg"].shape == params[0].shape
    vanilla = torch.optim.AdamW(params, lr=0.1)
    vanilla.load_state_dict(sd)
    for p in params:
        for k in ("exp_avg", "exp_avg_sq"):
            cs = torch.cosine_similarity(vanilla.state[p][k].reshape(-1).float(),
                                         opt.state[p][k].materialize().reshape(-1), dim=0)
            assert cs > 0.99
    _set_grads(params, 60)
    vanilla.step()
    # and back: a stock checkpoint (no master_bytewidth, maybe no initial_lr) loads into a Flash optimizer
    back = fo.FlashAdamW(params, lr=0.1, master_weight_bits=None)
    back.load_state_dict(vanilla.state_dict())
    assert all("initial_lr" in g for g in back.param_groups)
    for p in params:
        assert back.state[p]["exp_avg"].is_quantized()
        cs = torch.cosine_similarity(vanilla.state[p]["exp_avg"].reshape(-1).float(),
                                     back.state[p]["exp_avg"].materialize().reshape(-1), dim=0)
        assert cs > 0.99
    _train(back, params, 1, 70)
    # a compressed checkpoint is not loadable by the stock optimizer
    comp = fo.FlashAdamW(params, lr=0.1, master_weight_bits=None, compress_state_dict=True)
    _train(comp, params, 1, 80)
    stock = torch.optim.AdamW(params, lr=0.1)
    stock.load_state_dict(comp.state_dict())
    with pytest.raises(KeyError):
        stock.state[params[0]]["exp_avg"]


def test_resume_from_checkpoint_continues_the_same_trajectory():
    """/root/reference/test/test_training.py:353-418: save -> load -> continue equals uninterrupted training
    (relative loss difference < 2e-4)."""
    fo = _fo()
    torch.manual_seed(5)
    x = torch.randn(64, 10, device=DEV)
    y = torch.randn(64, 5, device=DEV)

    def make():
        torch.manual_seed(6)
        return nn.Sequential(nn.Linear(10, 16), nn.ReLU(), nn.Linear(16, 5)).to(DEV)

    def run(model, opt, steps):
        out = []
        for _ in range(steps):
            opt.zero_grad()
            loss = ((model(x) - y) ** 2).mean()
            loss.backward()
            opt.step()
            out.append(loss.item())
        return out

    m1 = make()
    o1 = fo.FlashAdamW(m1.parameters(), lr=1e-2, master_weight_bits=None, compress_state_dict=True)
    full = run(m1, o1, 10)
    m2 = make()
    o2 = fo.FlashAdamW(m2.parameters(), lr=1e-2, master_weight_bits=None, compress_state_dict=True)
    first = run(m2, o2, 5)
    m3 = make()
    m3.load_state_dict(copy.deepcopy(m2.state_dict()))
    o3 = fo.FlashAdamW(m3.parameters(), lr=1e-2, master_weight_bits=None, compress_state_dict=True)
    o3.load_state_dict(copy.deepcopy(o2.state_dict()))
    rest = run(m3, o3, 5)
    for a, b in zip(full, first + rest):
        assert abs(a - b) / abs(a) < 2e-4


# ---------------------------------------------------------------------------------- gradient release


@pytest.mark.parametrize("factory,kwargs", [("FlashAdamW", dict(lr=1e-2)), ("FlashLion", dict(lr=1e-3)),
                                            ("FlashSGD", dict(lr=1e-2, momentum=0.9))])
def test_gradient_release_matches_manual_stepping(factory, kwargs):
    """/root/reference/test/test_optimizers.py:880-945."""
    fo = _fo()
    x = torch.randn(16, 128, device=DEV, dtype=torch.bfloat16)
    ma, mb = _mlp(3).to(DEV), _mlp(3).to(DEV)
    fo.cast_model(ma)
    fo.cast_model(mb)
    oa = getattr(fo, factory)(ma.parameters(), **kwargs)
    ob = getattr(fo, factory)(mb.parameters(), **kwargs)
    handle = fo.enable_gradient_release(mb, ob)
    assert handle.active
    for _ in range(4):
        oa.zero_grad()
        ma(x).float().sum().backward()
        oa.step()
        mb(x).float().sum().backward()
        assert all(p.grad is None for p in mb.parameters())     # freed by the hooks
        with pytest.warns(UserWarning, match="no-op"):
            ob.step()
        with pytest.warns(UserWarning, match="no-op"):
            ob.zero_grad()
    for a, b in zip(ma.parameters(), mb.parameters()):
        assert torch.equal(a, b)
        assert torch.equal(oa.state[a]["error_bits"], ob.state[b]["error_bits"])
    handle.remove()
    assert not handle.active and not ob._gradient_release
    mb(x).float().sum().backward()
    assert all(p.grad is not None for p in mb.parameters())
    ob.step()


def test_gradient_release_steps_tied_parameters_once_and_honours_pre_step():
    """/root/reference/test/test_optimizers.py:948-975."""
    fo = _fo()

    class Tied(nn.Module):
        def __init__(self):
            super().__init__()
            self.embed = nn.Embedding(32, 16)
            self.out = nn.Linear(16, 32, bias=False)
            self.out.weight = self.embed.weight

        def forward(self, idx):
            return self.out(self.embed(idx))

    torch.manual_seed(0)
    m = Tied().to(DEV)
    fo.cast_model(m)
    opt = fo.FlashAdamW(m.parameters(), lr=1e-2)
    seen = []
    handle = fo.enable_gradient_release(m, opt, pre_step=lambda p, g: seen.append(p) or True)
    m(torch.arange(8, device=DEV)).float().sum().backward()
    assert len(seen) == 1 and opt.state[m.embed.weight]["step"].item() == 1
    handle.remove()
    skipped = fo.enable_gradient_release(m, opt, pre_step=lambda p, g: False)
    before = m.embed.weight.detach().clone()
    m(torch.arange(8, device=DEV)).float().sum().backward()
    assert torch.equal(m.embed.weight, before) and m.embed.weight.grad is not None
    skipped.remove()


# ----------------------------------------------------------------------------- fp32 export / import


@pytest.mark.parametrize("dtype,mwb", [(torch.bfloat16, 24), (torch.bfloat16, 32), (torch.float16, 32)])
def test_fp32_state_dict_round_trip(dtype, mwb):
    """/root/reference/test/test_optimizers.py:984-1045: set_fp32 -> get_fp32 is exact to NMSE < 1e-9 (32-bit)."""
    fo = _fo()
    model = _mlp(9).to(DEV)
    fo.cast_model(model, dtype=dtype)
    opt = fo.FlashAdamW(model.parameters(), lr=1e-3, master_weight_bits=mwb)
    model(torch.randn(4, 128, device=DEV, dtype=dtype)).float().sum().backward()
    opt.step()
    exported = opt.get_fp32_model_state_dict(model)
    assert all(v.dtype == torch.float32 for v in exported.values())
    target = {k: v + torch.randn_like(v) * 1e-4 for k, v in exported.items()}
    opt.set_fp32_model_state_dict(model, target)
    back = opt.get_fp32_model_state_dict(model)
    for k in target:
        nmse = ((back[k] - target[k]) ** 2).mean() / (target[k] ** 2).mean()
        assert nmse < (1e-9 if mwb == 32 and dtype == torch.bfloat16 else 1e-7), (k, nmse.item())
    with pytest.raises(ValueError, match="Expected fp32"):
        opt.set_fp32_model_state_dict(model, {k: v.half() for k, v in target.items()})
    opt.zero_grad()
    model(torch.randn(4, 128, device=DEV, dtype=dtype)).float().sum().backward()
    opt.step()  # the replaced error_bits tensors are picked up by the launcher


# ------------------------------------------------------------------------------- container behaviour


def test_maybe_quantized_tensor_container():
    """/root/reference/test/test_compression.py:155-191."""
    from flashoptim_amd.optimizers import _MaybeQuantizedTensor

    x = torch.randn(32, 64, device=DEV, dtype=torch.bfloat16)
    for signed in (True, False):
        q = _MaybeQuantizedTensor(None, try_quantize=True, signed=signed)
        q.set_data(x if signed else x.abs())
        assert q.is_quantized() and q._data is None
        assert q.quantized.dtype == (torch.int8 if signed else torch.uint8) and q.scales.dtype == torch.float16
        assert q.shape == (32, 64) and q.numel() == 2048 and q.is_cuda
        assert q.kernel_tensor is q.quantized and q.kernel_scales_or_self is q.scales
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        plain = _MaybeQuantizedTensor(None, try_quantize=False, storage_dtype=dtype)
        plain.set_data(x.to(dtype))
        assert not plain.is_quantized() and plain.materialize().dtype == dtype
        assert torch.equal(plain.materialize(), x.to(dtype)) and plain.kernel_scales_or_self is plain.data
    with pytest.raises(NotImplementedError):
        _MaybeQuantizedTensor(torch.zeros(4), try_quantize=True)
    with pytest.raises(ValueError, match="must not specify other keys"):
        q.load_state_dict({"m": x, "m::scales": x}, "m")


# ------------------------------------------------------------------------------------ ECC invariants


def test_ecc_invariants_over_every_binade():
    """All 2^23 mantissas of every (sign, exponent) through the HIP split/join kernels: the seven invariants of
    /root/reference/test/test_ecc_invariants.py:39-47 with the exception budgets it records (:257-262, 282-291)."""
    fo = _fo()
    from tests.test_oracle_ecc import _DENORMAL_BUDGET, _NORMAL_BUDGET

    mant = torch.arange(1 << 23, dtype=torch.int32, device=DEV)
    names = ["perfect_downcast_8bit", "perfect_downcast_16bit", "16bit_no_worse_zero", "16bit_no_worse_always",
             "8bit_corrects_representable", "16bit_corrects_representable", "16bit_better_in_middle_range"]

    def counts(sign, exponent, dtype):
        bits = mant if exponent == -127 else (mant | ((exponent + 127) << 23))
        if sign < 0:
            bits = bits | torch.tensor(-(1 << 31), dtype=torch.int32, device=DEV)
        x = bits.view(torch.float32)
        nar = x.to(dtype)
        ok = ~nar.isinf()
        e8 = fo.compute_ecc_bits(x, nar, master_bytewidth=3)
        e16 = fo.compute_ecc_bits(x, nar, master_bytewidth=4)
        xd = x.double()
        err0 = (nar.double() - xd).abs()
        err8 = (fo.reconstruct_fp32_param(nar, e8).double() - xd).abs()
        err16 = (fo.reconstruct_fp32_param(nar, e16).double() - xd).abs()
        den = torch.where(xd.abs() > 0, xd.abs(), torch.ones_like(xd))
        r0, r8, r16 = err0 / den, err8 / den, err16 / den
        t8, t16 = 1.0 / 127.0, 1.0 / 32767.0
        ex = [(err0 == 0) & (err8 > 0), (err0 == 0) & (err16 > 0), (err8 == 0) & (err16 > 0), err16 > err8,
              (r0 >= t8) & (r8 >= t8), (r0 >= t16) & (r16 >= t16), (r0 >= t16) & ~(r0 >= t8) & (err16 >= err8)]
        return [int((e & ok).sum()) for e in ex]

    for name, dtype, exps, budget in (("bf16", torch.bfloat16, range(-126, 128), _NORMAL_BUDGET),
                                      ("bf16", torch.bfloat16, [-127], _DENORMAL_BUDGET),
                                      ("fp16", torch.float16, range(-14, 16), _NORMAL_BUDGET),
                                      ("fp16", torch.float16, range(-30, -14), _DENORMAL_BUDGET)):
        for sign in (1, -1):
            for e in exps:
                for inv, c in zip(names, counts(sign, e, dtype)):
                    assert c <= budget.get((name, inv), 0), (name, sign, e, inv, c)


# ------------------------------------------------------------------------------- cached step() plans


WALKS = ["c++", "python"]


def _use_walk(monkeypatch, walk):
    """The per-step check of a cached plan runs in C++ (flashoptim_amd/lib/_fo_hostscan.so) when that module is built
    and in Python otherwise; both must behave alike."""
    from flashoptim_amd import _hostscan

    if walk == "c++":
        assert _hostscan.scan is not None, "build it with make -C flashoptim_amd/hostscan"
    else:
        monkeypatch.setattr(_hostscan, "scan", None)
        monkeypatch.setattr(_hostscan, "same_objects", None)


@pytest.mark.parametrize("walk", WALKS)
def test_cached_step_plan_follows_moving_missing_and_freed_gradients(walk, monkeypatch):
    """step() caches a group's launch tables after the first call.  The cache must notice gradients that were
    re-allocated at other addresses, fall back when a gradient is missing, never keep a freed gradient alive, and
    stay bit-identical to per-tensor stepping throughout."""
    _use_walk(monkeypatch, walk)
    import gc
    import weakref

    fo = _fo()
    shapes = [5000, 33, 4096, 70001]
    pa, pb = _make_params(shapes, torch.bfloat16, 21), _make_params(shapes, torch.bfloat16, 21)
    oa, ob = fo.FlashAdamW(pa, lr=1e-3), fo.FlashAdamW(pb, lr=1e-3)
    hold = []
    for it in range(6):
        _set_grads(pa, 100 + it)
        _set_grads(pb, 100 + it)
        if it == 2:                       # keep the old gradients alive so the new ones land elsewhere
            hold = [p.grad for p in pa]
            _set_grads(pa, 100 + it)
            assert any(p.grad.data_ptr() != h.data_ptr() for p, h in zip(pa, hold))
        if it == 4:                       # one parameter without a gradient this step
            pa[1].grad = None
            pb[1].grad = None
        if it == 3:
            oa.param_groups[0]["lr"] = ob.param_groups[0]["lr"] = 5e-4   # scheduler-style change
        oa.step()
        for p in pb:
            ob.step_param(p)
    for a, b in zip(pa, pb):
        assert torch.equal(a, b)
        sa, sb = _state_tensors(oa, a), _state_tensors(ob, b)
        for k in sa:
            assert parity.bits_equal(sa[k], sb[k]), k
    assert oa.state[pa[0]]["step"].item() == 6 and oa.state[pa[1]]["step"].item() == 5
    ref = weakref.ref(pa[0].grad)
    oa.zero_grad(set_to_none=True)
    del hold
    gc.collect()
    assert ref() is None, "the optimizer's cached plan kept a gradient alive"


def _count_full_plans(opt):
    """Wrap the optimizer's full planning path with a call counter."""
    calls = []
    full = opt._step_group_slow

    def counted(index, group):
        calls.append(index)
        return full(index, group)

    opt._step_group_slow = counted
    return calls


@pytest.mark.parametrize("walk", WALKS)
def test_cached_step_plan_with_frozen_and_unused_parameters(walk, monkeypatch):
    """A group that holds a frozen parameter and one that never receives a gradient (fine-tuning) still steps from
    the cached plan; the cache is dropped the moment the unused parameter gets a gradient, and the result stays
    bit-identical to per-tensor stepping."""
    _use_walk(monkeypatch, walk)
    fo = _fo()
    shapes = [5000, 33, 4096, 70001, 0]
    pa, pb = _make_params(shapes, torch.bfloat16, 33), _make_params(shapes, torch.bfloat16, 33)
    for params in (pa, pb):
        params[1].requires_grad_(False)
    oa, ob = fo.FlashAdamW(pa, lr=1e-3), fo.FlashAdamW(pb, lr=1e-3)
    full_plans = _count_full_plans(oa)
    frozen_before = pa[1].clone()
    for it in range(6):
        for params in (pa, pb):
            _set_grads(params, 300 + it)
            params[1].grad = None
            if it < 4:
                params[2].grad = None           # unused until the fifth step
        oa.step()
        for p in pb:
            ob.step_param(p)
        if it == 3:
            assert full_plans == [0], "steps 2-4 should have come from the cached plan"
    assert full_plans == [0, 0], "one full plan at the start and one when the unused parameter joined"
    assert torch.equal(pa[1], frozen_before)
    for a, b in zip(pa, pb):
        assert torch.equal(a, b)
        sa, sb = _state_tensors(oa, a), _state_tensors(ob, b)
        for k in sa:
            assert parity.bits_equal(sa[k], sb[k]), k
    assert oa.state[pa[0]]["step"].item() == 6 and oa.state[pa[2]]["step"].item() == 2


@pytest.mark.parametrize("walk", WALKS)
def test_cached_step_plan_notices_replaced_parameter_storage(walk, monkeypatch):
    """`p.data = ...` (what module.to() and friends do) moves a parameter to new memory; the cached launch table
    must not go on updating the old block."""
    _use_walk(monkeypatch, walk)
    fo = _fo()
    shapes = [5000, 4096, 70001]
    pa, pb = _make_params(shapes, torch.bfloat16, 34), _make_params(shapes, torch.bfloat16, 34)
    oa, ob = fo.FlashAdamW(pa, lr=1e-3), fo.FlashAdamW(pb, lr=1e-3)
    old_block = None
    for it in range(4):
        _set_grads(pa, 400 + it)
        _set_grads(pb, 400 + it)
        if it == 2:
            old_block = pa[1].data
            pa[1].data = old_block.clone()
            assert pa[1].data_ptr() != old_block.data_ptr()
            old_copy = old_block.clone()
        oa.step()
        for p in pb:
            ob.step_param(p)
    assert torch.equal(old_block, old_copy), "the step wrote into the parameter's previous storage"
    for a, b in zip(pa, pb):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype,mwb", [(torch.bfloat16, 24), (torch.bfloat16, 32), (torch.float32, None), (torch.float16, None)])
@pytest.mark.parametrize("kwargs", [dict(weight_decay=0.0), dict(weight_decay=1e-2)])
def test_momentum_free_sgd_multi_tensor_is_bit_identical_to_per_tensor_steps(dtype, mwb, kwargs):
    """FlashSGD / FlashSGDW with momentum=0 (eager branch ref:1447-1465) as one multi-tensor launch."""
    fo = _fo()
    for factory in ("FlashSGD", "FlashSGDW"):
        pa, pb = _make_params(_RAGGED, dtype, 2), _make_params(_RAGGED, dtype, 2)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            oa = getattr(fo, factory)(pa, lr=1e-2, momentum=0.0, master_weight_bits=mwb, **kwargs)
            ob = getattr(fo, factory)(pb, lr=1e-2, momentum=0.0, master_weight_bits=mwb, **kwargs)
        for it in range(3):
            _set_grads(pa, 20 + it)
            _set_grads(pb, 20 + it)
            oa.step()
            for p in pb:
                ob.step_param(p)
        for a, b in zip(pa, pb):
            assert torch.equal(a, b)
            assert "momentum_buffer" not in oa.state[a]
            if mwb is not None:
                assert torch.equal(oa.state[a]["error_bits"], ob.state[b]["error_bits"])


def test_absmax_many_matches_torch():
    from flashoptim_amd import kernels

    g = torch.Generator().manual_seed(11)
    tensors = []
    for dtype in (torch.bfloat16, torch.float32, torch.float16):
        for n in (1, 7, 31, 33, 511, 4096, 4097, 65536 + 5, 1_000_003):
            tensors.append((torch.randn(n, generator=g) * 10 ** float(torch.randint(-3, 3, (1,), generator=g))).to(dtype).to(DEV))
    tensors.append(torch.zeros(0, dtype=torch.bfloat16, device=DEV))
    tensors.append(torch.zeros(100, dtype=torch.float32, device=DEV))
    tensors.append(torch.randn(64, 64, generator=g).to(DEV).t())                       # non-contiguous
    big = torch.randn(3_000_000, generator=g).to(torch.bfloat16).to(DEV)
    tensors.append(big[3:])                                                             # 2-byte aligned view
    spike = torch.zeros(70000, dtype=torch.float16, device=DEV); spike[-1] = -60000.0
    tensors.append(spike)
    inf = torch.ones(5000, dtype=torch.float32, device=DEV); inf[123] = float("-inf")
    tensors.append(inf)
    got = kernels.absmax_many(tensors)
    for t, v in zip(tensors, got):
        want = float(t.abs().max().item()) if t.numel() else 0.0
        assert v == want, (t.dtype, t.numel(), v, want)
    nan = torch.ones(5000, dtype=torch.bfloat16, device=DEV); nan[4000] = float("nan")
    import math
    assert math.isnan(kernels.absmax_many([nan])[0])
    with pytest.raises(ValueError):
        kernels.absmax_many([torch.zeros(8, dtype=torch.float64, device=DEV)])
    with pytest.raises(NotImplementedError):
        kernels.absmax_many([torch.zeros(8)])


def test_check_numerics_with_cached_plans_and_one_scan():
    """check_numerics keeps the cached step path: the weights' resolution is cached, a later drop of lr still
    raises, and recompute_param_stats() refreshes the cached magnitudes (ref:656-673, 1149-1181)."""
    fo = _fo()
    params = _make_params([4096, 1000, 33], torch.bfloat16, 5)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = fo.FlashLion(params, lr=1e-2, check_numerics=True, master_weight_bits=None)
    initial = [float(p.detach().abs().max()) for p in params]
    for it in range(3):
        _set_grads(params, 30 + it)
        opt.step()
    assert opt._group_cache, "steps with check_numerics should leave a cached plan behind"
    for p, want in zip(params, initial):  # scanned once, at the first step
        assert opt._transient_state[id(p)]["maxabs"] == want
    opt.param_groups[0]["lr"] = 1e-9
    _set_grads(params, 40)
    with pytest.raises(fo.NumericsError):
        opt.step()
    opt.param_groups[0]["lr"] = 1e-2
    with torch.no_grad():
        params[0].mul_(1e6)          # weights grow: the cached statistic is stale until recomputed
    _set_grads(params, 41)
    opt.step()
    opt.recompute_param_stats()
    assert opt._transient_state[id(params[0])]["maxabs"] == float(params[0].detach().abs().max())
    _set_grads(params, 42)
    with pytest.raises(fo.NumericsError):
        opt.step()


@pytest.mark.parametrize("signed,sqrt,softsign", [(True, False, True), (False, True, False)])
@pytest.mark.parametrize("quantize", [True, False])
def test_zero_state_shortcut_equals_quantising_zeros(signed, sqrt, softsign, quantize):
    """State creation skips the quantise launch for the all-zero start (ref:1006-1013 quantises zeros)."""
    from flashoptim_amd.optimizers import _MaybeQuantizedTensor

    for shape in [(1,), (33,), (4096, 3), (70001,)]:
        ref = torch.empty(shape, dtype=torch.bfloat16, device=DEV)
        kw = dict(try_quantize=quantize, signed=signed, sqrt=sqrt, softsign=softsign, storage_dtype=torch.bfloat16)
        a = _MaybeQuantizedTensor.zeros_like(ref, **kw)
        b = _MaybeQuantizedTensor(torch.zeros_like(ref), **kw)
        assert a.is_quantized() == b.is_quantized() == quantize and a.shape == b.shape
        assert parity.bits_equal(a.kernel_tensor, b.kernel_tensor) and a.kernel_tensor.dtype == b.kernel_tensor.dtype
        if quantize:
            assert parity.bits_equal(a.scales, b.scales) and a.scales.shape == b.scales.shape
        assert sorted(a.state_dict("x")) == sorted(b.state_dict("x"))


def test_pooled_step_counters_behave_like_separate_scalars():
    """Adam's per-parameter CPU `step` scalars are views into one pooled tensor while a cached plan is live; they
    still read, checkpoint and advance like the separate fp32 scalars of the reference (ref:1846-1853)."""
    fo = _fo()
    params = _make_params([4096, 1000, 33, 70001], torch.bfloat16, 6)
    opt = fo.FlashAdamW(params, lr=1e-3)
    for it in range(4):
        _set_grads(params, 60 + it)
        opt.step()
    assert [float(opt.state[p]["step"]) for p in params] == [4.0] * 4
    sd = opt.state_dict()
    for idx in sd["state"]:
        step = sd["state"][idx]["step"]
        assert step.dtype == torch.float32 and step.device.type == "cpu" and step.dim() == 0
        assert step.untyped_storage().nbytes() == 4, "checkpointed counters must not drag the pool along"
    # one parameter stepped on its own moves only its counter, and the next full step keeps them apart
    _set_grads(params, 70)
    opt.step_param(params[1])
    assert [float(opt.state[p]["step"]) for p in params] == [4.0, 5.0, 4.0, 4.0]
    params[1].grad = None
    opt.step()
    opt.step()   # second call runs from the rebuilt cache
    assert [float(opt.state[p]["step"]) for p in params] == [6.0, 5.0, 6.0, 6.0]
    # a reloaded optimizer continues from the saved counters
    fresh_params = [nn.Parameter(p.detach().clone()) for p in params]
    fresh = fo.FlashAdamW(fresh_params, lr=1e-3)
    fresh.load_state_dict(copy.deepcopy(opt.state_dict()))
    for a, b in zip(params, fresh_params):
        a.grad = torch.ones_like(a) * 1e-3
        b.grad = a.grad.clone()
    opt.step()
    fresh.step()
    assert [float(fresh.state[p]["step"]) for p in fresh_params] == [7.0, 6.0, 7.0, 7.0]
    for a, b in zip(params, fresh_params):  # the uncompressed bf16 checkpoint requantises the moments: close, not equal
        torch.testing.assert_close(a.float(), b.float(), rtol=0, atol=2e-3)


def test_deepcopy_of_the_optimizer_is_an_independent_working_optimizer():
    fo = _fo()
    params = _make_params([4096, 33, 70001], torch.bfloat16, 9)
    opt = fo.FlashAdamW(params, lr=1e-3, weight_decay=0.01)
    for it in range(2):
        _set_grads(params, 80 + it)
        opt.step()
    twin = copy.deepcopy(opt)           # copies parameters, gradients and states
    twin_params = twin.param_groups[0]["params"]
    assert all(a is not b and torch.equal(a, b) for a, b in zip(params, twin_params))
    assert twin._quantize == opt._quantize and twin._master_bytewidth == opt._master_bytewidth and not twin._gradient_release
    for it in range(2):
        _set_grads(params, 90 + it)
        for a, b in zip(params, twin_params):
            b.grad = a.grad.clone()
        opt.step()
        twin.step()
    for a, b in zip(params, twin_params):
        assert torch.equal(a, b)
        assert torch.equal(opt.state[a]["exp_avg"].quantized, twin.state[b]["exp_avg"].quantized)
        assert float(twin.state[b]["step"]) == 4.0


@pytest.mark.parametrize("factory,kwargs", [
    ("FlashAdamW", dict(lr=1e-3, weight_decay=0.01)),
    ("FlashSGD", dict(lr=1e-2, momentum=0.9, weight_decay=1e-4)),
])
def test_scheduler_clipping_and_added_group_match_per_tensor_stepping(factory, kwargs):
    """The usual furniture of a training loop around step(): a OneCycleLR schedule (moves lr and beta1 / momentum of
    every group each step), gradient clipping (rewrites the gradients in place) and a parameter group added halfway.
    step() with its cached plans must stay bit-identical to stepping every tensor on its own."""
    fo = _fo()
    shapes = [5000, 33, 4096, 70001]
    late_shapes = [2049, 64]
    runs = []
    for _ in range(2):
        params, late = _make_params(shapes, torch.bfloat16, 50), _make_params(late_shapes, torch.bfloat16, 51)
        opt = getattr(fo, factory)(params, **kwargs)
        sched = torch.optim.lr_scheduler.OneCycleLR(opt, max_lr=kwargs["lr"] * 10, total_steps=12)
        runs.append((params, late, opt, sched))
    seen_lrs = set()
    for it in range(10):
        for which, (params, late, opt, sched) in enumerate(runs):
            live = params + (late if it >= 5 else [])
            if it == 5:  # the schedule keeps its own keys in every group; a late group has to bring them along
                first = opt.param_groups[0]
                cycle_keys = [k for k in first if k.startswith(("max_", "min_", "base_", "initial_"))]
                opt.add_param_group(dict(params=late, **{k: first[k] for k in cycle_keys}))
            _set_grads(live, 500 + it, scale=1e-2)
            torch.nn.utils.clip_grad_norm_(live, 0.05)
            if which == 0:
                opt.step()
            else:
                for p in live:
                    opt.step_param(p)
            with warnings.catch_warnings():
                warnings.simplefilter("ignore")  # the per-tensor run never calls step(), which the scheduler remarks on
                sched.step()
            seen_lrs.add(opt.param_groups[0]["lr"])
    assert len(seen_lrs) == 10, "the schedule should have changed lr every step"
    (pa, la, oa, _), (pb, lb, ob, _) = runs
    for a, b in zip(pa + la, pb + lb):
        assert torch.equal(a, b)
        sa, sb = _state_tensors(oa, a), _state_tensors(ob, b)
        for k in sa:
            assert parity.bits_equal(sa[k], sb[k]), k


@pytest.mark.parametrize("factory,kwargs", [
    ("FlashLion", dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1)),
    ("FlashSGDW", dict(lr=1e-2, momentum=0.9, weight_decay=1e-4)),
])
def test_step_of_the_counter_free_optimizers_can_be_captured_in_a_graph(factory, kwargs):
    """Lion and SGD pass no step counter to their kernels, so once the launch plan is cached step() is nothing but
    kernel launches on the current stream and can be recorded into a HIP graph over static gradient buffers.  Every
    replay is checked against an eagerly stepped twin, with eager work and synchronisations in between."""
    fo = _fo()
    shapes = [5000, 33, 4096, 70001]
    pa, pb = _make_params(shapes, torch.bfloat16, 60), _make_params(shapes, torch.bfloat16, 60)
    oa, ob = getattr(fo, factory)(pa, **kwargs), getattr(fo, factory)(pb, **kwargs)
    _set_grads(pa, 600)
    static_grads = [p.grad for p in pa]

    def feed(seed):
        _set_grads(pb, seed)
        for g, p in zip(static_grads, pb):
            g.copy_(p.grad)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for it in range(2):               # builds the states and the cached plan outside the graph
            feed(600 + it)
            oa.step()
            ob.step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    feed(602)
    with torch.cuda.graph(graph):
        oa.step()
    graph.replay()
    ob.step()
    for it in range(3, 7):
        feed(600 + it)
        torch.cuda.synchronize()
        graph.replay()
        ob.step()
        torch.cuda.synchronize()
        for a, b in zip(pa, pb):
            assert torch.equal(a, b), (it, a.numel())
    for a, b in zip(pa, pb):
        sa, sb = _state_tensors(oa, a), _state_tensors(ob, b)
        for k in sa:
            assert parity.bits_equal(sa[k], sb[k]), k


def test_adam_step_refuses_graph_capture():
    """Adam's bias correction takes the step number by value: a replayed graph would repeat it, so capture raises
    instead of going quietly wrong, and leaves the optimizer usable."""
    fo = _fo()
    params = _make_params([4096, 33], torch.bfloat16, 61)
    opt = fo.FlashAdamW(params, lr=1e-3)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for it in range(2):
            _set_grads(params, 610 + it)
            opt.step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")   # torch remarks that the abandoned graph is empty
        with pytest.raises(RuntimeError, match="while a HIP graph is being recorded"):
            with torch.cuda.graph(graph):
                opt.step()
    torch.cuda.synchronize()
    before = params[0].clone()
    opt.step()
    assert not torch.equal(params[0], before)
    assert all(float(opt.state[p]["step"]) == 3.0 for p in params), "the refused step must not count"


def test_clearing_the_optimizer_state_restarts_the_moments():
    """`optimizer.state.clear()` (a moment reset some training recipes do) must not leave the cached launch plan
    stepping the discarded state tensors: the next step starts from fresh zero moments, like a new optimizer."""
    fo = _fo()
    shapes = [5000, 4096, 70001]
    pa = _make_params(shapes, torch.bfloat16, 70)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")   # pure bf16 training is remarked on
        oa = fo.FlashAdamW(pa, lr=1e-3, master_weight_bits=None, quantize=True)
    for it in range(3):
        _set_grads(pa, 700 + it)
        oa.step()
    oa.state.clear()
    pb = [nn.Parameter(p.detach().clone()) for p in pa]
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        ob = fo.FlashAdamW(pb, lr=1e-3, master_weight_bits=None, quantize=True)
    for it in range(2):
        _set_grads(pa, 710 + it)
        _set_grads(pb, 710 + it)
        oa.step()
        ob.step()
    for a, b in zip(pa, pb):
        assert torch.equal(a, b)
        sa, sb = _state_tensors(oa, a), _state_tensors(ob, b)
        for k in sa:
            assert parity.bits_equal(sa[k], sb[k]), k
        assert float(oa.state[a]["step"]) == 2.0


def test_a_replaced_step_counter_object_is_honoured_by_the_cached_plan():
    """Replacing a counter OBJECT (state[p]["step"] = torch.tensor(0.), as a hand-copied per-parameter state does)
    leaves the pooled counters of the cached plan behind: the next step must notice, take the step number from the
    new tensor, keep incrementing it, and save it in state_dict()."""
    fo = _fo()
    shapes = [5000, 4096, 70001]
    pa, pb = _make_params(shapes, torch.bfloat16, 81), _make_params(shapes, torch.bfloat16, 81)
    oa, ob = fo.FlashAdamW(pa, lr=1e-3), fo.FlashAdamW(pb, lr=1e-3)
    for it in range(6):
        _set_grads(pa, 810 + it)
        _set_grads(pb, 810 + it)
        if it == 3:
            oa.state[pa[2]]["step"] = torch.tensor(0.0)
            ob.state[pb[2]]["step"] = torch.tensor(0.0)
        oa.step()
        for p in pb:
            ob.step_param(p)
    for a, b in zip(pa, pb):
        assert torch.equal(a, b)
        sa, sb = _state_tensors(oa, a), _state_tensors(ob, b)
        for k in sa:
            assert parity.bits_equal(sa[k], sb[k]), k
    assert [float(oa.state[p]["step"]) for p in pa] == [6.0, 6.0, 3.0]
    assert [float(st["step"]) for st in oa.state_dict()["state"].values()] == [6.0, 6.0, 3.0]


def test_a_moved_gradient_during_graph_capture_raises_before_any_launch():
    """A cached multi-tensor plan whose gradient moved to another address needs its pointer table uploaded again.
    Recorded into a HIP graph that copy would replay with whatever the staging buffer holds later, so step() must
    raise on the host instead -- and stay usable afterwards."""
    fo = _fo()
    params = _make_params([5000, 33, 70001], torch.bfloat16, 82)
    opt = fo.FlashLion(params, lr=1e-4)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for it in range(2):
            _set_grads(params, 820 + it)
            opt.step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    keep = [p.grad for p in params]                       # hold the old buffers so the new ones get new addresses
    params[1].grad = torch.zeros_like(params[1])
    assert params[1].grad.data_ptr() != keep[1].data_ptr()
    before = [p.clone() for p in params]
    graph = torch.cuda.CUDAGraph()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")                   # torch remarks that the abandoned graph is empty
        with pytest.raises(RuntimeError, match="cannot be recorded into a HIP graph"):
            with torch.cuda.graph(graph):
                opt.step()
    torch.cuda.synchronize()
    for p, b in zip(params, before):
        assert torch.equal(p, b), "the refused step must not have launched anything"
    _set_grads(params, 825)
    opt.step()                                            # eager stepping still works and uploads the table
    torch.cuda.synchronize()
    assert not torch.equal(params[0], before[0])


def test_rewritten_step_counters_are_honoured_by_the_cached_plan():
    """The per-parameter `step` scalars are ordinary state: zeroing them (a warm restart of the bias correction)
    or setting one of them apart must steer the next cached step exactly as it steers per-tensor stepping."""
    fo = _fo()
    shapes = [5000, 4096, 70001]
    pa, pb = _make_params(shapes, torch.bfloat16, 80), _make_params(shapes, torch.bfloat16, 80)
    oa, ob = fo.FlashAdamW(pa, lr=1e-3), fo.FlashAdamW(pb, lr=1e-3)
    for it in range(8):
        _set_grads(pa, 800 + it)
        _set_grads(pb, 800 + it)
        if it == 3:      # warm restart: every counter back to zero
            for opt in (oa, ob):
                for st in opt.state.values():
                    st["step"].zero_()
        if it == 5:      # one parameter set apart
            oa.state[pa[1]]["step"].fill_(40.0)
            ob.state[pb[1]]["step"].fill_(40.0)
        oa.step()
        for p in pb:
            ob.step_param(p)
    for a, b in zip(pa, pb):
        assert torch.equal(a, b)
        sa, sb = _state_tensors(oa, a), _state_tensors(ob, b)
        for k in sa:
            assert parity.bits_equal(sa[k], sb[k]), k
    assert [float(oa.state[p]["step"]) for p in pa] == [5.0, 43.0, 5.0]


class _ShardStub(nn.Parameter):
    """What a sharding wrapper hands an optimizer: an object whose ``to_local()`` is this rank's shard
    (/root/reference/flashoptim/optimizers.py:598-616).  Here the object's own storage is the shard."""

    @staticmethod
    def __new__(cls, data):
        return torch.Tensor._make_subclass(cls, data, True)

    def to_local(self):
        self.calls = getattr(self, "calls", 0) + 1
        return self.data


@pytest.mark.parametrize("factory,kwargs", [
    ("FlashAdamW", dict(lr=1e-3, weight_decay=0.01)),
    ("FlashLion", dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1)),
])
def test_a_tensor_stepped_as_shards_equals_the_whole_tensor(factory, kwargs):
    """The path shards without any exchange: every 32-element quantisation group is independent and the update is
    elementwise.  One bf16 tensor is stepped whole and as two shards that reach the optimizer through ``to_local()``
    (ref:598-616, 724-730, 999-1001; state is created from the local shard).
    Split at a multiple of 32 elements: parameters, correction codes, moment codes and group scales of the shards,
    laid end to end, equal the whole tensor's bit for bit on every step.
    Split anywhere else: the groups behind the split start at other elements, so their scales and codes are those
    of other groups (which is why a compressed checkpoint is tied to its sharding); the first step, which starts
    from zero states, still gives bit-identical parameters, and later steps stay as close as two quantisations of
    the same moments do."""
    fo = _fo()
    n = 3 * 4096 + 777
    torch.manual_seed(5)
    w0 = (torch.randn(n, device=DEV) * 0.02).to(torch.bfloat16)
    grads = [(torch.randn(n, device=DEV) * 1e-3).to(torch.bfloat16) for _ in range(4)]
    names = [k for k in ("exp_avg", "exp_avg_sq") if factory == "FlashAdamW" or k == "exp_avg"]

    def run(cuts):
        """Steps the tensor cut at `cuts`; returns per step the pieces' outputs laid end to end."""
        bounds = [0] + list(cuts) + [n]
        params = [(_ShardStub if cuts else nn.Parameter)(w0[a:b].clone()) for a, b in zip(bounds, bounds[1:])]
        opt = getattr(fo, factory)(params, master_weight_bits=24, **kwargs)
        out = []
        for g in grads:
            for p, a, b in zip(params, bounds, bounds[1:]):
                p.grad = g[a:b].clone()
            opt.step()
            rec = dict(p=torch.cat([p.detach().reshape(-1) for p in params]).clone(),
                       ecc=torch.cat([opt.state[p]["error_bits"].reshape(-1) for p in params]).clone())
            for k in names:
                rec[k] = torch.cat([opt.state[p][k].quantized.reshape(-1) for p in params]).clone()
                rec[k + "_scales"] = [opt.state[p][k].scales.clone() for p in params]
            out.append(rec)
        if cuts:
            assert all(getattr(p, "calls", 0) > 0 for p in params), "the optimizer never asked for the local shard"
            assert all(opt.state[p][names[0]].quantized.numel() == p.numel() for p in params)
        return out

    whole = run(())
    aligned = run((4096 + 64,))
    for step, (a, b) in enumerate(zip(whole, aligned), start=1):
        for key in ("p", "ecc") + tuple(names):
            assert parity.bits_equal(a[key], b[key]), f"aligned split, step {step}: {key} differs"
        for k in names:
            assert parity.bits_equal(a[k + "_scales"][0], torch.cat(b[k + "_scales"])), f"aligned split, step {step}: {k} scales differ"
    ragged = run((4096 + 50,))
    assert parity.bits_equal(whole[0]["p"], ragged[0]["p"]) and parity.bits_equal(whole[0]["ecc"], ragged[0]["ecc"])
    cut = 4096 + 50
    for step, (a, b) in enumerate(zip(whole, ragged), start=1):
        # in front of the cut nothing changes; behind it only the grouping of the moments does
        for key in ("p", "ecc") + tuple(names):
            assert parity.bits_equal(a[key][:cut - cut % 32], b[key][:cut - cut % 32]), f"ragged split, step {step}: {key} differs before the cut"
        pa, pb = a["p"].float(), b["p"].float()
        # behind the cut the two runs dequantise slightly different moments: their updates (at most lr per step under
        # Adam, exactly lr under Lion, whose sign may flip) drift apart by a fraction of what was applied
        assert float((pa - pb).abs().max()) <= 2.0 * kwargs["lr"] * step, f"ragged split, step {step}"
        assert float((pa - pb).abs().mean()) <= 0.05 * kwargs["lr"] * step, f"ragged split, step {step}"
    assert not parity.bits_equal(whole[-1][names[0]], ragged[-1][names[0]])          # the groups behind the cut are other groups
