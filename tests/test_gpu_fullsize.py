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
        T.adam_step_ref(states[0], states[1], p, g, ecc, ADAM["lr"], ADAM["beta1"], ADAM["beta2"], ADAM["eps"],
                        ADAM["weight_decay"], ADAM["decoupled"], step)
    else:
        T.momentum_step_ref(states[0], p, g, ecc, **LION)
    # codes and scales equal the oracle's bit for bit under every kernel
    for i, st in enumerate(states):
        assert parity.bits_equal(after.codes[i], st.codes) and parity.bits_equal(after.scales[i], st.scales), f"{what} state{i}"
    if kind != "adam":  # the momentum kernels equal the oracle bit for bit
        assert parity.bits_equal(after.p, p) and parity.bits_equal(after.ecc, ecc), f"{what}: parameter or ECC bits differ"
        return
    # Adam on bf16 parameters with a 1-byte ECC: guarded folded update, master weights within one unit
    parity.check_master(after.p, after.ecc, p, ecc, what)


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


def _student_t3(n, gen, scale):
    """Student-t with 3 degrees of freedom, composed from normal draws (z / sqrt((z1^2 + z2^2 + z3^2) / 3)): heavy
    tails without the rejection sampler of torch.distributions."""
    z = torch.randn(4, n, generator=gen, device=DEV)
    return z[0] / ((z[1] * z[1] + z[2] * z[2] + z[3] * z[3]) / 3.0).sqrt() * scale


def _ragged_lengths():
    g = torch.Generator().manual_seed(3)
    lens = torch.floor(torch.exp2(24.0 * torch.rand(4096, generator=g, dtype=torch.float64))).clamp(1, 1 << 24)
    lens = torch.floor(lens * (1.0e9 / lens.sum().item())).clamp(1, 1 << 24).to(torch.int64).tolist()
    lens[:3] = [1, 31, 33]
    return lens


@pytest.mark.parametrize("name", ["FlashLion", "FlashSGDW"])
def test_ragged_4096_tensor_launch_equals_per_tensor_launches_and_the_oracle(name):
    """The ragged configuration at full size (4096 bf16 tensors, lengths log-uniform in [1, 2^24] with many that are
    not multiples of the group size, about 1e9 elements, heavy-tailed Student-t(3) * 1e-3 gradients whose outliers
    pin the group scales; FlashLion and FlashSGDW with 24-bit master weights): one multi-tensor launch per step is
    bit-identical to 4096 single-tensor launches, and on a sample of the tensors (lengths 1, 31, 33, the five
    longest, ten random ones) the last step equals the CPU oracle bit for bit."""
    import warnings

    import flashoptim_amd as fo
    from oracle import c_oracle as C

    lens = _ragged_lengths()
    assert sum(1 for n in lens if n % 32) > 1024
    kwargs = dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1) if name == "FlashLion" else dict(lr=1e-2, momentum=0.9, weight_decay=1e-4)
    dg = torch.Generator(device=DEV).manual_seed(5)
    pa = [torch.nn.Parameter((torch.randn(n, generator=dg, device=DEV) * 0.02).to(torch.bfloat16)) for n in lens]
    pb = [torch.nn.Parameter(p.detach().clone()) for p in pa]
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        oa = getattr(fo, name)(pa, master_weight_bits=24, **kwargs)
        ob = getattr(fo, name)(pb, master_weight_bits=24, **kwargs)
    order = sorted(range(len(lens)), key=lambda i: -lens[i])
    sample = sorted(set([0, 1, 2] + order[:5] + [int(i) for i in torch.randint(0, 4096, (10,), generator=torch.Generator().manual_seed(9))]))
    assert sum(1 for i in sample if lens[i] >= 1 << 20) >= 3
    steps = 3
    for it in range(steps):
        for a, b in zip(pa, pb):
            a.grad = _student_t3(a.numel(), dg, 1e-3).to(torch.bfloat16)
            b.grad = a.grad.clone()
        if it == steps - 1:  # inputs of the last step, for the oracle
            key = "exp_avg" if name == "FlashLion" else "momentum_buffer"
            before = {i: (pa[i].detach().cpu().clone(), pa[i].grad.cpu().clone(), oa.state[pa[i]]["error_bits"].cpu().clone(),
                          oa.state[pa[i]][key].quantized.cpu().clone(), oa.state[pa[i]][key].scales.cpu().clone()) for i in sample}
        oa.step()
        for p in pb:
            ob.step_param(p)
    key = "exp_avg" if name == "FlashLion" else "momentum_buffer"
    for a, b in zip(pa, pb):
        assert torch.equal(a, b)
        sa, sb = oa.state[a], ob.state[b]
        assert torch.equal(sa["error_bits"], sb["error_bits"])
        assert torch.equal(sa[key].quantized, sb[key].quantized)
        assert parity.bits_equal(sa[key].scales, sb[key].scales)
    for i in sample:
        p, g, ecc, codes, scales = before[i]
        if name == "FlashLion":
            C.momentum_step(codes, scales, p, g, ecc, 1e-4, 0.99, 0.9, 0.1 * 1e-4, do_lion=True)
        else:  # FlashSGDW: decoupled decay, weight_decay * lr (ref:1438-1442), update_coef = 1 - dampening
            C.momentum_step(codes, scales, p, g, ecc, 1e-2, 0.9, 1.0, 1e-4 * 1e-2, decoupled=True)
        st = oa.state[pa[i]]
        what = f"{name} tensor {i} ({lens[i]} elements)"
        assert parity.bits_equal(pa[i].detach().reshape(-1), p) and parity.bits_equal(st["error_bits"].reshape(-1), ecc), what
        assert parity.bits_equal(st[key].quantized.reshape(-1), codes) and parity.bits_equal(st[key].scales, scales), what


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
    # gradients ~N(0, 1e-3) scaled per tensor by a log-uniform factor in [0.1, 10]
    tensor_scale = (10.0 ** (torch.rand(len(lens), generator=torch.Generator().manual_seed(2), dtype=torch.float64) * 2.0 - 1.0)).tolist()
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
        for a, b, ts in zip(pa, pb, tensor_scale):
            if a.grad is None:
                a.grad = torch.empty_like(a)
            for i in range(0, a.numel(), 1 << 27):
                m = min(1 << 27, a.numel() - i)
                a.grad[i:i + m] = (torch.randn(m, generator=dg, device=DEV) * (1e-3 * ts)).to(torch.bfloat16)
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


def test_llama8b_fp32_gradient_release_in_reverse_layer_order_and_compressed_checkpoint_round_trip():
    """The fp32 + gradient-release configuration at full size: 291 fp32 tensors of Llama-3-8B's shapes
    (8 030 261 248 elements, quantised moments, no master-weight bits) held by a module whose backward just writes
    the gradients, layer by layer from the last to the first.  enable_gradient_release() steps every tensor from
    its post-accumulate-grad hook, one launch per tensor, and frees the gradient.  Checked: every tensor stepped
    exactly once and in reverse layer order; sampled tensors equal the CPU oracle bit for bit (fp32 Adam follows
    the reference operation by operation); the compressed state_dict survives torch.save -> torch.load(
    weights_only=True) -> load_state_dict into a fresh optimizer with codes, scales and step bit-identical."""
    import gc
    import io
    import warnings

    import flashoptim_amd as fo
    from oracle import c_oracle as C

    lens = _llama3_8b_lengths()
    tensor_scale = (10.0 ** (torch.rand(len(lens), generator=torch.Generator().manual_seed(2), dtype=torch.float64) * 2.0 - 1.0)).tolist()

    def initial(i):
        g = torch.Generator(device=DEV).manual_seed(5000 + i)
        p = torch.empty(lens[i], dtype=torch.float32, device=DEV)
        for o in range(0, lens[i], 1 << 27):
            m = min(1 << 27, lens[i] - o)
            p[o:o + m] = torch.randn(m, generator=g, device=DEV) * 0.02
        return p

    def gradient(i):
        g = torch.Generator(device=DEV).manual_seed(9000 + i)
        out = torch.empty(lens[i], dtype=torch.float32, device=DEV)
        for o in range(0, lens[i], 1 << 27):
            m = min(1 << 27, lens[i] - o)
            out[o:o + m] = torch.randn(m, generator=g, device=DEV) * (1e-3 * tensor_scale[i])
        return out

    class WriteGrads(torch.autograd.Function):
        """Identity on x; its backward hands every parameter of the block its gradient."""

        @staticmethod
        def forward(ctx, x, first_index, *params):
            ctx.first_index, ctx.count = first_index, len(params)
            return x.clone()

        @staticmethod
        def backward(ctx, gx):
            return (gx, None) + tuple(gradient(ctx.first_index + j) for j in range(ctx.count))

    class Model(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.weights = torch.nn.ParameterList([torch.nn.Parameter(initial(i)) for i in range(len(lens))])
            self.blocks = [(0, 1)] + [(1 + 9 * layer, 9) for layer in range(32)] + [(289, 2)]   # embed, 32 layers, norm + lm_head

        def forward(self):
            x = torch.zeros((), device=DEV)
            for first, count in self.blocks:
                x = WriteGrads.apply(x, first, *self.weights[first:first + count])
            return x

    model = Model()
    params = list(model.weights)
    kw = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, master_weight_bits=None, compress_state_dict=True)
    opt = fo.FlashAdamW(params, **kw)
    order = []
    index_of = {id(p): i for i, p in enumerate(params)}
    handle = fo.enable_gradient_release(model, opt, pre_step=lambda p, group: order.append(index_of[id(p)]) is None)
    model().backward()
    torch.cuda.synchronize()
    assert sorted(order) == list(range(291)), "every tensor is stepped exactly once"
    block_of = {}
    for b, (first, count) in enumerate(model.blocks):
        block_of.update({first + j: b for j in range(count)})
    assert [block_of[i] for i in order] == sorted((block_of[i] for i in order), reverse=True), "reverse layer order"
    assert all(p.grad is None for p in params) and all(float(opt.state[p]["step"]) == 1.0 for p in params)

    # sampled tensors against the oracle: a norm vector, a k projection (4 Mi), a q projection (16 Mi)
    for i in (1 + 9 * 31 + 7, 1 + 9 * 17 + 1, 1 + 9 * 3, 289):
        n = lens[i]
        p0, g = initial(i).cpu(), gradient(i).cpu()
        m, ms = torch.zeros(n, dtype=torch.int8), torch.zeros((n + 31) // 32, dtype=torch.float16)
        v, vs = torch.zeros(n, dtype=torch.uint8), torch.zeros((n + 31) // 32, dtype=torch.float16)
        C.adam_step(m, ms, v, vs, p0, g, None, 1e-3, 0.9, 0.999, 1e-8, 0.01 * 1e-3, True, 1)
        st = opt.state[params[i]]
        what = f"tensor {i} ({n} elements)"
        assert parity.bits_equal(params[i].detach().reshape(-1), p0), what
        assert parity.bits_equal(st["exp_avg"].quantized.reshape(-1), m) and parity.bits_equal(st["exp_avg"].scales, ms), what
        assert parity.bits_equal(st["exp_avg_sq"].quantized.reshape(-1), v) and parity.bits_equal(st["exp_avg_sq"].scales, vs), what
    handle.remove()

    # compressed checkpoint: state_dict -> torch.save -> torch.load(weights_only=True) -> fresh optimizer
    sd = opt.state_dict()
    buf = io.BytesIO()
    torch.save(sd, buf)
    size = buf.tell()
    assert size < 2.2 * sum(lens), f"compressed checkpoint takes {size / sum(lens):.2f} bytes per parameter"
    del sd
    buf.seek(0)
    loaded = torch.load(buf, weights_only=True)
    del buf
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        fresh = fo.FlashAdamW(params, **kw)
    fresh.load_state_dict(loaded)
    del loaded
    for p in params:
        a, b = opt.state[p], fresh.state[p]
        assert float(b["step"]) == 1.0
        for name in ("exp_avg", "exp_avg_sq"):
            assert a[name].quantized.data_ptr() != b[name].quantized.data_ptr()
            assert parity.bits_equal(a[name].quantized, b[name].quantized), name
            assert parity.bits_equal(a[name].scales, b[name].scales), name
    del opt, fresh, model, params
    gc.collect()
    torch.cuda.empty_cache()
