"""GPU integration tests on a toy regression model, after /root/reference/test/test_training.py: mixed-precision
training modes against an fp32 run of the same optimizer (thresholds of ref test_training.py:30-33, 255-343) and the
fully lr-decoupled variants against their textbook forms (/root/reference/test/reference.py:76-93, 136-154,
215-234)."""

import copy
import warnings

import numpy as np
import pytest
import torch
import torch.nn as nn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"

AMP_MIN_CORRELATION = 0.9999          # ref test_training.py:30
AMP_MAX_NMSE_GRADSCALER = 5e-4        # ref :31
AMP_MAX_NMSE_BF16_NATIVE = 1e-4       # ref :32
AMP_MAX_NMSE_AUTOCAST = 3e-7          # ref :33


def _fo():
    import flashoptim_amd

    return flashoptim_amd


def _toy_data(n, d_in, d_out, seed):
    """ref test_training.py:50-66: y = sum(x) broadcast + 0.1 noise."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, d_in, generator=g)
    y = x.sum(dim=1, keepdim=True).expand(-1, d_out) + 0.1 * torch.randn(n, d_out, generator=g)
    return x, y


def _model(d_in, d_out, hidden=16):
    return nn.Sequential(nn.Linear(d_in, hidden), nn.ReLU(), nn.Linear(hidden, d_out))


def _factories():
    fo = _fo()
    return {
        "FlashLion": lambda ps, **kw: fo.FlashLion(ps, betas=(0.5, 0.75), **kw),
        "FlashSGDM": lambda ps, **kw: fo.FlashSGD(ps, momentum=0.9, **kw),
        "FlashAdamW": lambda ps, **kw: fo.FlashAdamW(ps, betas=(0.9, 0.999), eps=1e-8, **kw),
    }


def _train(model, opt, x, y, steps, amp_mode, batch=8):
    loss_fn = nn.MSELoss()
    use_autocast = amp_mode in ("fp16_autocast", "bf16_autocast", "fp16_gradscaler")
    ac_dtype = torch.float16 if amp_mode in ("fp16_autocast", "fp16_gradscaler") else torch.bfloat16
    scaler = torch.amp.GradScaler("cuda") if amp_mode == "fp16_gradscaler" else None
    losses = []
    n_batches = x.shape[0] // batch
    for step in range(steps):
        i = step % n_batches
        xb, yb = x[i * batch:(i + 1) * batch].to(DEV), y[i * batch:(i + 1) * batch].to(DEV)
        if amp_mode == "bf16_native":
            xb, yb = xb.to(torch.bfloat16), yb.to(torch.bfloat16)
        opt.zero_grad(set_to_none=True)
        if use_autocast:
            with torch.amp.autocast("cuda", dtype=ac_dtype):
                loss = loss_fn(model(xb), yb)
        else:
            loss = loss_fn(model(xb), yb)
        if scaler is not None:
            scaler.scale(loss).backward()
            scaler.step(opt)
            scaler.update()
        else:
            loss.backward()
            opt.step()
        losses.append(loss.item())
    return losses


@pytest.mark.parametrize("seed", [0, 1])
@pytest.mark.parametrize("amp_mode", ["fp16_autocast", "bf16_autocast", "fp16_gradscaler", "bf16_native"])
@pytest.mark.parametrize("name", ["FlashLion", "FlashSGDM", "FlashAdamW"])
def test_amp_training_tracks_the_fp32_run(name, amp_mode, seed):
    torch.manual_seed(seed)
    d_in, d_out, steps, lr = 10, 5, 20, 1e-3
    x, y = _toy_data(128, d_in, d_out, seed)
    init = copy.deepcopy(_model(d_in, d_out).state_dict())
    factory = _factories()[name]

    base = _model(d_in, d_out).to(DEV)
    base.load_state_dict(init)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt_base = factory(base.parameters(), lr=lr, quantize=False, check_numerics=False, master_weight_bits=None)
    losses_base = _train(base, opt_base, x, y, steps, None)

    test = _model(d_in, d_out).to(DEV)
    test.load_state_dict(init)
    kw = dict(master_weight_bits=None)
    if amp_mode == "bf16_native":
        test = test.to(torch.bfloat16)
        kw = {}  # default 24-bit masters on bf16 parameters, as in the reference's test
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt_test = factory(test.parameters(), lr=lr, quantize=False, check_numerics=False, **kw)
    losses_test = _train(test, opt_test, x, y, steps, amp_mode)

    assert losses_test[-1] < losses_test[0]
    b, t = np.array(losses_base), np.array(losses_test)
    nmse = float(np.mean((t - b) ** 2) / max(np.var(b), 1e-10))
    corr = float(np.corrcoef(b, t)[0, 1])
    assert corr >= AMP_MIN_CORRELATION, (name, amp_mode, corr)
    limit = {"fp16_gradscaler": AMP_MAX_NMSE_GRADSCALER, "bf16_native": AMP_MAX_NMSE_BF16_NATIVE}.get(amp_mode, AMP_MAX_NMSE_AUTOCAST)
    assert nmse < limit, (name, amp_mode, nmse)


def _textbook_step(kind, p, g, state, lr, wd, initial_lr, step):
    """Fully lr-decoupled forms, fp64 on the host (ref reference.py:76-93 AdamW, :136-154 SGDW, :215-234 Lion)."""
    decay = 1.0 - wd * (lr / initial_lr)
    if kind == "adamw":
        b1, b2, eps = 0.9, 0.999, 1e-8
        p *= decay
        state["m"] = state["m"] * b1 + g * (1 - b1)
        state["v"] = state["v"] * b2 + g * g * (1 - b2)
        mh, vh = state["m"] / (1 - b1 ** step), state["v"] / (1 - b2 ** step)
        p -= lr * mh / (np.sqrt(vh) + eps)
    elif kind == "sgdw":
        mu = 0.9
        p *= decay
        state["m"] = state["m"] * mu + g
        p -= lr * state["m"]
    else:
        b1, b2 = 0.5, 0.75
        p *= decay
        u = np.sign(state["m"] * b1 + g * (1 - b1))
        p -= lr * u
        state["m"] = state["m"] * b2 + g * (1 - b2)
    return p


@pytest.mark.parametrize("kind", ["adamw", "sgdw", "lion"])
def test_decouple_lr_variants_match_their_textbook_forms(kind):
    """decouple_lr=True: weight decay scaled by lr/initial_lr, followed through an lr schedule (ref
    optimizers.py:1290-1294, 1438-1442, 1894-1898)."""
    fo = _fo()
    g0 = torch.Generator().manual_seed(4)
    w = torch.randn(3000, generator=g0, dtype=torch.float64) * 0.1
    p = nn.Parameter(w.to(torch.float32).to(DEV))
    lr0, wd = 1e-2, 1e-2
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        if kind == "adamw":
            opt = fo.FlashAdamW([p], lr=lr0, weight_decay=wd, decouple_lr=True, quantize=False, master_weight_bits=None)
        elif kind == "sgdw":
            opt = fo.FlashSGDW([p], lr=lr0, momentum=0.9, weight_decay=wd, decouple_lr=True, quantize=False, master_weight_bits=None)
        else:
            opt = fo.FlashLion([p], lr=lr0, betas=(0.5, 0.75), weight_decay=wd, decouple_lr=True, quantize=False, master_weight_bits=None)
    ref = w.to(torch.float32).to(torch.float64).numpy().copy()
    state = {"m": np.zeros_like(ref), "v": np.zeros_like(ref)}
    for step in range(1, 11):
        lr = lr0 * (1.0 - 0.05 * step)          # a decaying schedule
        opt.param_groups[0]["lr"] = lr
        g = torch.randn(3000, generator=g0, dtype=torch.float64) * 0.01
        g32 = g.to(torch.float32)
        p.grad = g32.to(DEV)
        opt.step()
        ref = _textbook_step(kind, ref, g32.to(torch.float64).numpy(), state, lr, wd, lr0, step)
    got = p.detach().cpu().to(torch.float64).numpy()
    if kind == "lion":  # sign flips of near-zero updates move a weight by 2 lr; bound their share instead
        assert np.mean(np.abs(got - ref) > 1e-6) < 2e-3
    else:
        np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-7)


# ---------------------------------------------------------------------------------- a small language model


class _Block(nn.Module):
    def __init__(self, d, heads):
        super().__init__()
        self.heads = heads
        self.ln1, self.ln2 = nn.LayerNorm(d), nn.LayerNorm(d)
        self.qkv, self.proj = nn.Linear(d, 3 * d), nn.Linear(d, d)
        self.up, self.down = nn.Linear(d, 4 * d), nn.Linear(4 * d, d)

    def forward(self, x, mask):
        b, t, d = x.shape
        q, k, v = self.qkv(self.ln1(x)).view(b, t, 3, self.heads, d // self.heads).permute(2, 0, 3, 1, 4)
        att = (q @ k.transpose(-1, -2)) / (d // self.heads) ** 0.5 + mask
        x = x + self.proj((att.softmax(-1) @ v).transpose(1, 2).reshape(b, t, d))
        return x + self.down(torch.nn.functional.gelu(self.up(self.ln2(x))))


class _TinyLM(nn.Module):
    """Two pre-norm transformer blocks over a tied embedding / output matrix: 1-D norm weights, biases, 2-D and
    tied parameters in one model, i.e. every parameter flavour the optimizers meet in a language model."""

    def __init__(self, vocab=128, d=64, heads=4, seq=32):
        super().__init__()
        self.embed = nn.Embedding(vocab, d)
        self.pos = nn.Parameter(torch.zeros(seq, d))
        self.blocks = nn.ModuleList([_Block(d, heads) for _ in range(2)])
        self.norm = nn.LayerNorm(d)
        self.head = nn.Linear(d, vocab, bias=False)
        self.head.weight = self.embed.weight
        self.register_buffer("mask", torch.full((seq, seq), float("-inf")).triu(1))

    def forward(self, idx):
        x = self.embed(idx) + self.pos
        for blk in self.blocks:
            x = blk(x, self.mask.to(x.dtype))
        return self.head(self.norm(x))


def _lm_batch(step, vocab=128, seq=32, batch=16):
    """Sequences that count upwards modulo the vocabulary in strides of 1..4 from random starts: the next token
    follows from the previous two."""
    g = torch.Generator().manual_seed(1000 + step)
    start = torch.randint(0, vocab, (batch, 1), generator=g)
    stride = torch.randint(1, 5, (batch, 1), generator=g)
    tokens = (start + stride * torch.arange(seq + 1)) % vocab
    return tokens[:, :-1].to(DEV), tokens[:, 1:].to(DEV)


def _lm_loss(model, step):
    x, y = _lm_batch(step)
    return nn.functional.cross_entropy(model(x).float().flatten(0, 1), y.flatten())


def _lm_run(make_opt, steps, bf16, release=False, resume_at=None):
    fo = _fo()
    torch.manual_seed(0)
    model = _TinyLM().to(DEV)
    if bf16:
        fo.cast_model(model)
    opt = make_opt(model.parameters())
    handle = fo.enable_gradient_release(model, opt) if release else None
    losses = []
    for step in range(steps):
        if resume_at is not None and step == resume_at:    # checkpoint, rebuild everything, carry on
            blob = (copy.deepcopy(model.state_dict()), copy.deepcopy(opt.state_dict()))
            torch.manual_seed(1)
            model = _TinyLM().to(DEV)
            if bf16:
                fo.cast_model(model)
            model.load_state_dict(blob[0])
            opt = make_opt(model.parameters())
            opt.load_state_dict(blob[1])
        loss = _lm_loss(model, step)
        loss.backward()
        if not release:
            opt.step()
            opt.zero_grad()
        losses.append(loss.item())
    if handle is not None:
        handle.remove()
    return np.array(losses), model, opt


def test_tiny_language_model_trains_like_fp32_adamw():
    """cast_model + FlashAdamW (bf16 weights, 24-bit masters, 8-bit moments) on a small transformer against an fp32
    model under torch.optim.AdamW: same data, same initialisation, 300 steps.  The loss must fall as far and follow
    the same curve; with gradient release the run is the same computation launched from the hooks; a compressed
    checkpoint taken halfway resumes onto the same curve."""
    fo = _fo()
    hp = dict(lr=3e-3, betas=(0.9, 0.99), weight_decay=0.01)
    steps = 300
    ref, _, _ = _lm_run(lambda ps: torch.optim.AdamW(ps, **hp), steps, bf16=False)
    flash = lambda ps: fo.FlashAdamW(ps, master_weight_bits=24, compress_state_dict=True, **hp)  # noqa: E731
    got, model, opt = _lm_run(flash, steps, bf16=True)
    assert ref[0] > 4.5 and ref[-20:].mean() < 0.5, "the fp32 run should have learned the task"
    assert abs(got[-20:].mean() - ref[-20:].mean()) < 0.15 * ref[-20:].mean(), (got[-20:].mean(), ref[-20:].mean())
    smooth = lambda a: np.convolve(a, np.ones(10) / 10, mode="valid")  # noqa: E731
    assert np.corrcoef(smooth(got), smooth(ref))[0, 1] > 0.999        # measured 0.99997
    # every parameter flavour got its state; the tied matrix has one
    assert len(opt.state) == len(list(model.parameters())) and model.head.weight is model.embed.weight
    assert all(s["error_bits"].dtype == torch.int8 and s["exp_avg"].is_quantized() for s in opt.state.values())

    released, _, _ = _lm_run(flash, steps, bf16=True, release=True)
    assert abs(released[-20:].mean() - got[-20:].mean()) < 0.01 and np.corrcoef(smooth(released), smooth(got))[0, 1] > 0.9999

    resumed, _, _ = _lm_run(flash, steps, bf16=True, resume_at=150)
    assert np.array_equal(resumed[:150], got[:150])
    assert np.allclose(resumed[150:], got[150:], rtol=0.05, atol=0.02), np.abs(resumed[150:] - got[150:]).max()
    print(f"tiny LM, mean loss of the last 20 steps: fp32 AdamW {ref[-20:].mean():.4f}, FlashAdamW {got[-20:].mean():.4f}, "
          f"with gradient release {released[-20:].mean():.4f}, resumed {resumed[-20:].mean():.4f}; "
          f"largest loss difference after the resume {np.abs(resumed[150:] - got[150:]).max():.4f}; "
          f"curve correlation with fp32 {np.corrcoef(smooth(got), smooth(ref))[0, 1]:.5f}")
