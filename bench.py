#!/usr/bin/env python3
"""Throughput of the fused optimizer step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]

A "step" is one pass of the optimizer over a resident synthetic parameter set (``optimizer.step()``: host
planning plus the multi-tensor HIP launch).  W untimed warm-up steps, then exactly K steps between two
``torch.cuda.synchronize()`` calls; one JSON line on stdout.

Workloads (``--workload``):
  llama8b-mwb24   default.  Llama-3-8B-shaped parameter list (291 tensors, 8 030 261 248 bf16 parameters),
                  FlashAdamW, master_weight_bits=24, one multi-tensor launch per step: the configuration the
                  headline metric is quoted on.
  llama8b-mwb32   same shapes, master_weight_bits=32 (int16 correction term).
  llama8b-mwb24-exact / llama8b-mwb32-exact
                  the same with FlashAdamW(exact_update=True): the update evaluated operation by operation
                  (bit-exact with the CPU oracle), to show what that costs.
  llama8b-mwb24-streams / llama8b-mwb32-streams / llama8b-fp32-streams
                  the memory accesses of the bf16 steps and of the fp32 step without the arithmetic (every stream read and written back
                  unchanged by the step kernels' own access code): the rate this access mix can reach on the box,
                  to be read next to the step's (``value`` counts the same parameters and bytes as the step).
  flat-2p30       one flat bf16 tensor of 2^30 elements, FlashAdamW, master_weight_bits=24.
  llama8b-lion / llama8b-sgdw
                  the same parameter list under FlashLion / FlashSGDW (one quantised moment), master_weight_bits=24.
  llama8b-lion-streams / ragged-streams
                  the momentum kernels' loads and stores without their arithmetic, on those two lists.
  ragged-lion / ragged-sgdw
                  4096 bf16 tensors with log-uniform lengths in [1, 2^24] (~1e9 parameters), FlashLion / FlashSGDW.
  llama8b-fp32-release
                  fp32 parameters, quantised moments, one launch per tensor in reverse order as under gradient
                  release; ends with a compressed state_dict save -> load round trip checked bit for bit.
  copy            4 GiB device copy with the library's copy kernel: calibrates the rocprof byte counters and shows
                  the attainable read+write rate (``value`` is meaningless here, read ``roofline``).

Reported: ``value`` = parameters updated per second; ``roofline`` = algorithmic HBM bytes of one step divided
by the average duration of a step (one event pair on the launch stream around the K timed steps, divided by K),
against the 8 TB/s peak (``frac``; ``frac_wall`` divides by the host's wall clock per step instead);
``parity`` (FlashAdamW workloads) = the HIP step against the CPU oracle on 2^20 and 2^20 + 17 elements after the
timed region: raw code mismatch rate per step and the share of master weights beyond one unit;
``cpu_baseline`` = the CPU oracle (oracle/torch_oracle.py, all host cores) on a bounded sample of the same
distribution, a reported baseline only.
"""

from __future__ import annotations

import argparse
import io
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published


def llama3_8b_shapes():
    """(name, shape) of the 291 tensors of a Llama-3-8B: 32 layers, hidden 4096, FFN 14336, 32 query / 8 KV heads of
    128, vocabulary 128256 with untied embedding and lm_head, RMSNorm weights of length 4096."""
    h, ffn, kv, vocab = 4096, 14336, 1024, 128256
    shapes = [("embed", (vocab, h))]
    for i in range(32):
        shapes += [(f"l{i}.q", (h, h)), (f"l{i}.k", (kv, h)), (f"l{i}.v", (kv, h)), (f"l{i}.o", (h, h)),
                   (f"l{i}.gate", (ffn, h)), (f"l{i}.up", (ffn, h)), (f"l{i}.down", (h, ffn)),
                   (f"l{i}.ln1", (h,)), (f"l{i}.ln2", (h,))]
    shapes += [("norm", (h,)), ("lm_head", (vocab, h))]
    return shapes


def ragged_lengths(count=4096, total=1_000_000_000, seed=3):
    """Lengths floor(2^(24 U)) clipped to [1, 2^24], rescaled towards `total`, with the lengths 1, 31, 33 present
    and at least a quarter of them not multiples of the group size."""
    g = torch.Generator().manual_seed(seed)
    lens = torch.floor(torch.exp2(24.0 * torch.rand(count, generator=g, dtype=torch.float64))).clamp(1, 1 << 24)
    lens = torch.floor(lens * (total / lens.sum().item())).clamp(1, 1 << 24).to(torch.int64)
    lens[:3] = torch.tensor([1, 31, 33])
    odd = lens % 32 == 0
    fix = torch.nonzero(odd).flatten()[: max(0, count // 4 - int((~odd).sum()))]
    lens[fix] += 1
    return lens.tolist()


def bytes_per_param(param_bytes: int, ecc_bytes: int, n_states: int) -> float:
    """Algorithmic HBM traffic of one element: read param, grad, ecc, codes, scales; write all but grad."""
    state = n_states * (1.0 + 2.0 / 32.0)
    return (2 * param_bytes + ecc_bytes + state) + (param_bytes + ecc_bytes + state)


def make_params(shapes, dtype, device, grad_scales=None, seed=0):
    torch.manual_seed(seed)
    params = []
    for i, (name, shape) in enumerate(shapes):
        if len(shape) == 1 and ("ln" in name or name == "norm"):
            w = torch.ones(shape, device=device, dtype=dtype)
        else:
            w = (torch.randn(shape, device=device, dtype=torch.float32) * 0.02).to(dtype)
        p = torch.nn.Parameter(w)
        s = 1.0 if grad_scales is None else grad_scales[i]
        p.grad = (torch.randn(shape, device=device, dtype=torch.float32) * (1e-3 * s)).to(dtype)
        params.append(p)
    return params


def rotating_gradients(params, step, device, grad_scales=None, sets=3):
    """Gradients are redrawn for every step, as in training: `sets` gradient lists are drawn once (seeds 1000 + k,
    outside the timed region) and the returned step function installs the next list as ``p.grad`` before each
    ``step()``, so gradient values and addresses change from step to step."""
    rings = []
    for k in range(sets):
        torch.manual_seed(1000 + k)
        ring = []
        for i, p in enumerate(params):
            s = 1.0 if grad_scales is None else grad_scales[i]
            ring.append((torch.randn(p.shape, device=device, dtype=torch.float32) * (1e-3 * s)).to(p.dtype))
        rings.append(ring)
    counter = [0]

    def run():
        ring = rings[counter[0] % sets]
        counter[0] += 1
        for p, g in zip(params, ring):
            p.grad = g
        step()

    return run


def momentum_streams_workload(params, opt, what):
    """The momentum kernels' loads and stores without their arithmetic, on the launch tables of `opt` after one real
    step (so that the states exist and hold values)."""
    from flashoptim_amd.launcher import BucketPlan

    opt.step()
    planned = [opt._plan_param(p, opt.param_groups[0]) for p in params]
    plan = BucketPlan("momentum", torch.bfloat16, 1, True, [t for _, t in planned])
    return dict(params=params, opt=None, step=plan.launch_streams_copy, bpp=bytes_per_param(2, 1, 1),
                desc=f"memory accesses of the FlashLion / FlashSGDW step (master_weight_bits=24) on {what} without the "
                     "arithmetic: every stream read and written back unchanged",
                launch="one multi-tensor launch per step", optimizer=None, mwb=24, keep=(opt, plan))


def build_workload(name: str, device):
    import flashoptim_amd as fo

    hp = dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    if name in ("llama8b-mwb24", "llama8b-mwb32", "llama8b-mwb24-exact", "llama8b-mwb32-exact"):
        shapes = llama3_8b_shapes()
        g = torch.Generator().manual_seed(2)
        scales = (10.0 ** (torch.rand(len(shapes), generator=g) * 2 - 1)).tolist()
        params = make_params(shapes, torch.bfloat16, device, scales)
        mwb = 24 if "mwb24" in name else 32
        exact = name.endswith("-exact")
        opt = fo.FlashAdamW(params, master_weight_bits=mwb, exact_update=exact, **hp)
        return dict(params=params, opt=opt, step=rotating_gradients(params, opt.step, device, scales),
                    bpp=bytes_per_param(2, 1 if mwb == 24 else 2, 2),
                    desc=f"Llama-3-8B-shaped parameter list, bf16, FlashAdamW, master_weight_bits={mwb}, "
                         + ("exact_update=True (operation-by-operation update), " if exact else "")
                         + "gradients redrawn per step (3 rotating sets)",
                    launch="one multi-tensor launch per step", optimizer="FlashAdamW", mwb=mwb)
    if name in ("llama8b-mwb24-streams", "llama8b-mwb32-streams", "llama8b-fp32-streams"):
        from flashoptim_amd.launcher import BucketPlan

        shapes = llama3_8b_shapes()
        g = torch.Generator().manual_seed(2)
        scales = (10.0 ** (torch.rand(len(shapes), generator=g) * 2 - 1)).tolist()
        fp32 = "fp32" in name
        mwb = None if fp32 else (24 if "mwb24" in name else 32)
        ecc_bytes = {None: 0, 24: 1, 32: 2}[mwb]
        dtype = torch.float32 if fp32 else torch.bfloat16
        params = make_params(shapes, dtype, device, scales)
        opt = fo.FlashAdamW(params, master_weight_bits=mwb, **hp)
        rotating_gradients(params, opt.step, device, scales, sets=1)()  # one real step: states exist and hold values
        planned = [opt._plan_param(p, opt.param_groups[0]) for p in params]
        plan = BucketPlan("adam", dtype, ecc_bytes, True, [t for _, t in planned])
        return dict(params=params, opt=None, step=plan.launch_streams_copy, bpp=bytes_per_param(4 if fp32 else 2, ecc_bytes, 2),
                    desc=f"memory accesses of the FlashAdamW step ({'fp32 parameters' if fp32 else f'master_weight_bits={mwb}'}) on the "
                         "Llama-3-8B-shaped list without its arithmetic: every stream read and written back unchanged",
                    launch="one multi-tensor launch per step", optimizer=None, mwb=mwb, keep=(opt, plan))
    if name in ("llama8b-lion", "llama8b-sgdw", "llama8b-lion-streams"):
        shapes = llama3_8b_shapes()
        g = torch.Generator().manual_seed(2)
        scales = (10.0 ** (torch.rand(len(shapes), generator=g) * 2 - 1)).tolist()
        params = make_params(shapes, torch.bfloat16, device, scales)
        if name in ("llama8b-lion", "llama8b-lion-streams"):
            opt = fo.FlashLion(params, lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1, master_weight_bits=24)
        else:
            opt = fo.FlashSGDW(params, momentum=0.9, lr=1e-2, weight_decay=1e-4, master_weight_bits=24)
        if name == "llama8b-lion-streams":
            return momentum_streams_workload(params, opt, "Llama-3-8B-shaped parameter list, bf16")
        return dict(params=params, opt=opt, step=opt.step, bpp=bytes_per_param(2, 1, 1),
                    desc=f"Llama-3-8B-shaped parameter list, bf16, {type(opt).__name__}, master_weight_bits=24",
                    launch="one multi-tensor launch per step", optimizer=type(opt).__name__, mwb=24)
    if name == "flat-2p30":
        params = make_params([("flat", (1 << 30,))], torch.bfloat16, device)
        opt = fo.FlashAdamW(params, master_weight_bits=24, **hp)
        return dict(params=params, opt=opt, step=rotating_gradients(params, opt.step, device), bpp=bytes_per_param(2, 1, 2),
                    desc="one flat bf16 tensor of 2^30 elements, FlashAdamW, master_weight_bits=24, gradients redrawn per "
                         "step (3 rotating sets)",
                    launch="one single-tensor launch per step", optimizer="FlashAdamW", mwb=24)
    if name in ("ragged-lion", "ragged-sgdw", "ragged-streams"):
        lens = ragged_lengths()
        torch.manual_seed(3)
        # parameters and gradients are carved from two flat buffers at 512-byte aligned offsets (what torch's
        # allocator does for tensors allocated one after the other) and drawn with a few large kernels, so that
        # the set-up does not issue tens of thousands of tiny launches (a profiler collecting counters per launch
        # crashed on them)
        offsets, total_padded = [], 0
        for n in lens:
            offsets.append(total_padded)
            total_padded += (n + 255) // 256 * 256
        flat_p = torch.empty(total_padded, dtype=torch.bfloat16, device=device)
        flat_g = torch.empty(total_padded, dtype=torch.bfloat16, device=device)
        for o in range(0, total_padded, 1 << 27):
            m = min(1 << 27, total_padded - o)
            flat_p[o:o + m] = (torch.randn(m, device=device) * 0.02).to(torch.bfloat16)
            # Student-t with 3 degrees of freedom composed from normal draws, z / sqrt((z1^2 + z2^2 + z3^2) / 3)
            z = torch.randn(4, m, device=device)
            flat_g[o:o + m] = (z[0] / ((z[1] * z[1] + z[2] * z[2] + z[3] * z[3]) / 3.0).sqrt() * 1e-3).to(torch.bfloat16)
            del z
        params = []
        for n, o in zip(lens, offsets):
            p = torch.nn.Parameter(flat_p[o:o + n])
            p.grad = flat_g[o:o + n]
            params.append(p)
        if name in ("ragged-lion", "ragged-streams"):
            opt = fo.FlashLion(params, lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1, master_weight_bits=24)
        else:
            opt = fo.FlashSGDW(params, momentum=0.9, lr=1e-2, weight_decay=1e-4, master_weight_bits=24)
        if name == "ragged-streams":
            return momentum_streams_workload(params, opt, "4096 bf16 tensors, lengths log-uniform in [1, 2^24]")
        return dict(params=params, opt=opt, step=opt.step, bpp=bytes_per_param(2, 1, 1),
                    desc="4096 bf16 tensors, lengths log-uniform in [1, 2^24], Student-t(3) gradients, "
                         + type(opt).__name__ + ", master_weight_bits=24",
                    launch="one multi-tensor launch per step", optimizer=type(opt).__name__, mwb=24)
    if name == "llama8b-fp32":
        shapes = llama3_8b_shapes()
        g = torch.Generator().manual_seed(2)
        scales = (10.0 ** (torch.rand(len(shapes), generator=g) * 2 - 1)).tolist()
        params = make_params(shapes, torch.float32, device, scales)
        opt = fo.FlashAdamW(params, master_weight_bits=None, **hp)
        return dict(params=params, opt=opt, step=rotating_gradients(params, opt.step, device, scales, sets=2),
                    bpp=bytes_per_param(4, 0, 2),
                    desc="Llama-3-8B-shaped parameter list, fp32 parameters, FlashAdamW, quantised moments, gradients "
                         "redrawn per step (2 rotating sets)",
                    launch="one multi-tensor launch per step", optimizer="FlashAdamW", mwb=None)
    if name == "llama8b-fp32-release":
        shapes = llama3_8b_shapes()
        g = torch.Generator().manual_seed(2)
        scales = (10.0 ** (torch.rand(len(shapes), generator=g) * 2 - 1)).tolist()
        params = make_params(shapes, torch.float32, device, scales)
        opt = fo.FlashAdamW(params, master_weight_bits=None, compress_state_dict=True, **hp)
        group = opt.param_groups[0]

        def step():  # what the gradient-release hooks do, in the order backward produces gradients
            for p in reversed(params):
                opt.step_param(p, group)

        return dict(params=params, opt=opt, step=step, bpp=bytes_per_param(4, 0, 2),
                    desc="Llama-3-8B-shaped parameter list, fp32 parameters, FlashAdamW, quantised moments, stepped "
                         "per tensor in reverse order as under gradient release",
                    launch="one single-tensor launch per tensor (291 per step)", optimizer="FlashAdamW", mwb=None,
                    checkpoint_roundtrip=True)
    if name == "copy":
        from flashoptim_amd.kernels import copy_bytes

        n = 1 << 32
        src = torch.empty(n, dtype=torch.uint8, device=device).random_(0, 255)
        dst = torch.empty_like(src)
        holder = torch.nn.Parameter(src.view(torch.float32)[:0])  # no parameters: this workload only moves bytes
        return dict(params=[holder], opt=None, step=lambda: copy_bytes(dst, src), bpp=0.0, copy_bytes=2 * n,
                    desc="device copy of 4 GiB with the library's copy kernel (counter calibration, attainable rate)",
                    launch="one copy launch per step", optimizer=None, mwb=None)
    raise SystemExit(f"unknown workload {name!r}")


def checkpoint_roundtrip(work, device) -> bool:
    """Compressed state_dict -> torch.save -> torch.load -> load_state_dict into a fresh optimizer; codes, fp16
    scales and step counters must come back bit for bit (fp32 parameters)."""
    import flashoptim_amd as fo

    opt = work["opt"]
    buf = io.BytesIO()
    torch.save(opt.state_dict(), buf)
    size = buf.tell()
    buf.seek(0)
    loaded = torch.load(buf, weights_only=True)
    fresh = fo.FlashAdamW(work["params"], master_weight_bits=None, compress_state_dict=True, lr=1e-3)
    fresh.load_state_dict(loaded)
    ok = True
    for p in work["params"]:
        a, b = opt.state[p], fresh.state[p]
        for k in ("exp_avg", "exp_avg_sq"):
            ok &= torch.equal(a[k].quantized, b[k].quantized)
            ok &= torch.equal(a[k].scales.view(torch.int16), b[k].scales.view(torch.int16))
        ok &= a["step"].item() == b["step"].item()
    work["checkpoint_bytes"] = size
    return bool(ok)


def cpu_baseline(steps: int = 5, warmup: int = 3, n: int = 1 << 26):
    """The CPU oracle on a bounded sample: one flat bf16 tensor of 2^26 elements drawn like the flat workload
    (params N(0, 0.02) seed 0, gradients N(0, 1e-3) seed 1000 + step), FlashAdamW master_weight_bits=24."""
    from oracle import torch_oracle as T

    torch.set_num_threads(os.cpu_count() or 1)
    p = (torch.randn(n, generator=torch.Generator().manual_seed(0)) * 0.02).to(torch.bfloat16)
    ecc = torch.zeros(n, dtype=torch.int8)
    m, v = T.MomentState.zeros(n, True, True, torch.bfloat16), T.MomentState.zeros(n, False, True, torch.bfloat16)
    elapsed = 0.0
    for step in range(1, warmup + steps + 1):
        g = (torch.randn(n, generator=torch.Generator().manual_seed(1000 + step)) * 1e-3).to(torch.bfloat16)
        t0 = time.perf_counter()
        T.adam_step_ref(m, v, p, g, ecc, 1e-3, 0.9, 0.999, 1e-8, 0.01 * 1e-3, True, step)
        if step > warmup:
            elapsed += time.perf_counter() - t0
    return {
        "value": n * steps / elapsed, "unit": "params/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"FlashAdamW mwb=24 on one flat bf16 tensor of 2^26 elements, {warmup} warm-up + {steps} timed steps "
                  "of the PyTorch CPU restatement (oracle/torch_oracle.py)",
    }


TRAFFIC_FILE = os.path.join("profiles", "hbm_traffic.json")


def measured_traffic(workload: str):
    """HBM bytes per step as recorded earlier with rocprofv3 FETCH_SIZE / WRITE_SIZE (profiles/hbm_traffic.json);
    None when this workload has no entry.  This run does not measure it."""
    try:
        with open(os.path.join(ROOT, TRAFFIC_FILE)) as f:
            return json.load(f).get(workload, {}).get("bytes_per_step")
    except (OSError, ValueError):
        return None


def parity_subcheck(device, ecc_dtype=torch.int8, steps: int = 4, exact_update: bool = False):
    """HIP step against the CPU oracle on 2^20 and 2^20 + 17 bf16 elements (parameters N(0, 0.02), gradients
    N(0, 1e-3) redrawn per step, FlashAdamW hyper-parameters of the throughput run), outside the timed region, every
    step from identical inputs.  Nothing is allowed for: the figures are raw counts.  Per step: the share of moment
    codes and of fp16 group scales that differ at all, the share of master weights (narrow parameter + correction
    code) more than one unit of master precision from the oracle's, the largest such difference in units, and the
    share that is exactly one unit apart (within the bar)."""
    from flashoptim_amd import kernels as k
    from oracle import torch_oracle as T
    from tests import parity

    out = {"sizes": [], "code_mismatch_fraction_per_step": [], "scale_mismatch_fraction_per_step": [],
           "master_beyond_one_unit_per_step": [], "master_max_units_per_step": [], "master_one_unit_apart_per_step": [],
           "narrow_beyond_one_ulp_per_step": []}
    for n in (1 << 20, (1 << 20) + 17):
        p = (torch.randn(n, generator=torch.Generator().manual_seed(0)) * 0.02).to(torch.bfloat16)
        ecc = torch.zeros(n, dtype=ecc_dtype)
        m, v = T.MomentState.zeros(n, True, True, torch.bfloat16), T.MomentState.zeros(n, False, True, torch.bfloat16)
        gp, gecc = p.to(device), ecc.to(device)
        gm, gms, gv, gvs = m.codes.to(device), m.scales.to(device), v.codes.to(device), v.scales.to(device)
        rows = {key: [] for key in out if key != "sizes"}
        for step in range(1, steps + 1):
            g = (torch.randn(n, generator=torch.Generator().manual_seed(1000 + step)) * 1e-3).to(torch.bfloat16)
            k._fused_adam_step(gm, gms, gv, gvs, gp, g.to(device), gecc, 1e-3, 0.9, 0.999, 1e-8, 0.01 * 1e-3, True, step,
                               exact_update=exact_update)
            T.adam_step_ref(m, v, p, g, ecc, 1e-3, 0.9, 0.999, 1e-8, 0.01 * 1e-3, True, step)
            codes = sum(int((a.cpu().view(torch.uint8) != b.view(torch.uint8)).sum()) for a, b in ((gm, m.codes), (gv, v.codes)))
            scales = sum(int((a.cpu().view(torch.int16) != b.view(torch.int16)).sum()) for a, b in ((gms, m.scales), (gvs, v.scales)))
            narrow, master = parity.master_difference(gp, gecc, p, ecc)
            rows["code_mismatch_fraction_per_step"].append(codes / (2 * n))
            rows["scale_mismatch_fraction_per_step"].append(scales / (2 * m.scales.numel()))
            rows["master_beyond_one_unit_per_step"].append(float((master > 1.0 + 1e-9).double().mean()))
            rows["master_max_units_per_step"].append(float(master.max()))
            rows["master_one_unit_apart_per_step"].append(float(((master > 0) & (master <= 1.0 + 1e-9)).double().mean()))
            rows["narrow_beyond_one_ulp_per_step"].append(float((narrow > 1.0 + 1e-9).double().mean()))
            for dst, src in ((p, gp), (ecc, gecc), (m.codes, gm), (m.scales, gms), (v.codes, gv), (v.scales, gvs)):
                dst.copy_(src.cpu())  # the next comparison starts from identical inputs
        out["sizes"].append(n)
        for key, row in rows.items():
            out[key].append(row)
    flat = lambda key: [x for row in out[key] for x in row]
    out["codes_and_scales_bit_exact"] = not any(flat("code_mismatch_fraction_per_step") + flat("scale_mismatch_fraction_per_step"))
    out["within_tolerance"] = out["codes_and_scales_bit_exact"] and not any(flat("master_beyond_one_unit_per_step") + flat("narrow_beyond_one_ulp_per_step"))
    return out


def measure(work, steps: int, warmup: int) -> dict:
    """W warm-up steps, then exactly K steps between two synchronisations.  Returns the timings of one workload."""
    step = work["step"]
    total = sum(p.numel() for p in work["params"])
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # Events on the launch stream (torch's current stream) around the K timed steps, without per-step event overhead
    # (several percent of a 1.6 ms step).  The device idles while the host prepares the first timed step (1 ms for a
    # list of 4096 tensors), so the kernels' average duration is taken from the end of the first step to the end of
    # the last, where the host runs ahead of the device; the wall clock behind `value` includes that lead-in.
    first, second, last = (torch.cuda.Event(enable_timing=True) for _ in range(3))
    t0 = time.perf_counter()
    first.record()
    for i in range(steps):
        step()
        if i == 0:
            second.record()
    last.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / steps
    avg_device_ms = second.elapsed_time(last) / (steps - 1) if steps > 1 else first.elapsed_time(last)
    step_bytes = work.get("copy_bytes", total * work["bpp"])
    achieved = step_bytes / (avg_device_ms * 1e-3) / 1e9
    return dict(total=total, ms_per_step=ms_per_step, avg_device_ms=avg_device_ms, step_bytes=step_bytes, achieved=achieved,
                frac=achieved / HBM_PEAK_GBPS, frac_wall=step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                with_lead_in_ms=first.elapsed_time(last) / steps)


# The other configurations of the baseline, run after the default workload (a few steps each): the flat 2^30 tensor,
# the 8B list with 32-bit masters, the 4096 ragged tensors under Lion and SGDW, fp32 parameters in one launch and in
# gradient-release order.
SECONDARY = ("flat-2p30", "llama8b-mwb32", "ragged-lion", "ragged-sgdw", "llama8b-fp32", "llama8b-fp32-release")


def run_secondary(name: str, device, steps: int, warmup: int, parity: bool) -> dict:
    work = build_workload(name, device)
    t = measure(work, steps, warmup)
    row = {"workload": name, "description": work["desc"], "n_params": t["total"], "steps": steps, "warmup": warmup,
           "algorithmic_bytes_per_param": work["bpp"], "ms_per_step": t["ms_per_step"], "step_device_ms_avg": t["avg_device_ms"],
           "params_per_s": t["total"] / (t["ms_per_step"] * 1e-3), "frac": t["frac"], "frac_wall": t["frac_wall"]}
    if work.get("checkpoint_roundtrip"):
        row["checkpoint_roundtrip_bit_exact"] = checkpoint_roundtrip(work, device)
        row["checkpoint_bytes"] = work["checkpoint_bytes"]
    adam_on_bf16 = work["optimizer"] == "FlashAdamW" and work["mwb"] in (24, 32)
    mwb = work["mwb"]
    work.clear()
    del work
    torch.cuda.empty_cache()
    if adam_on_bf16 and parity:
        sub = parity_subcheck(device, torch.int8 if mwb == 24 else torch.int16, steps=2)
        row["parity"] = {key: sub[key] for key in ("codes_and_scales_bit_exact", "within_tolerance", "master_beyond_one_unit_per_step",
                                                    "master_max_units_per_step")}
    return row


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="llama8b-mwb24")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-parity", action="store_true", help="skip the HIP-vs-oracle sub-check that runs after the timed region")
    ap.add_argument("--no-secondary", action="store_true",
                    help="default workload only: skip the short runs of the other baseline configurations that follow it")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: the optimizer step is shard-local and this build has no "
                         "multi-GPU path (run with --gpus 1).")
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a ROCm GPU")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if not os.path.exists(os.path.join(ROOT, "flashoptim_amd", "lib", "libflashoptim_hip.so")):
        import __graft_entry__

        __graft_entry__.build()  # loads what is built; builds only when nothing is

    work = build_workload(args.workload, device)
    step = work["step"]
    t = measure(work, args.steps, args.warmup)
    total, ms_per_step, avg_device_ms, step_bytes = t["total"], t["ms_per_step"], t["avg_device_ms"], t["step_bytes"]

    # a second pass with an event pair around every step, for the median and the fastest step (the pairs themselves
    # cost a few microseconds per step, which is why the averages above come from the pass without them)
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for begin, end in pairs:
        begin.record()
        step()
        end.record()
    torch.cuda.synchronize()
    per_step = sorted(begin.elapsed_time(end) for begin, end in pairs)
    # ... and, for the default workload, sixty further steps whose last twenty are reported apart: from zero states
    # the step gets faster for dozens of steps (fewer values on rounding boundaries, fewer flagged updates), so the
    # contract's W + K steps measure the early part of that curve and these the later one
    late_ms = None
    if args.workload == "llama8b-mwb24" and not args.no_secondary:
        for _ in range(40):
            step()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        for _ in range(20):
            step()
        end.record()
        torch.cuda.synchronize()
        late_ms = begin.elapsed_time(end) / 20

    out = {
        "metric": "params updated/sec + achieved HBM GB/s (% peak), FlashAdamW step on 8B params",
        "value": total / (ms_per_step * 1e-3),
        "unit": "params/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",  # the arithmetic type of the path; parameters and gradients are config.param_dtype
        "data": "synthetic",
        "config": {
            "workload": args.workload, "description": work["desc"], "optimizer": work["optimizer"],
            "param_dtype": str(work["params"][0].dtype).replace("torch.", "").replace("bfloat16", "bf16").replace("float32", "f32"),
            "master_weight_bits": work["mwb"], "n_tensors": len(work["params"]), "n_params": total,
            "launch": work["launch"], "algorithmic_bytes_per_param": work["bpp"],
        },
        "roofline": {
            "bound": "hbm", "achieved": t["achieved"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": t["frac"],
            # the same algorithmic bytes over the host's wall clock per step (includes the host lead-in of the first step)
            "frac_wall": t["frac_wall"],
            "traffic": measured_traffic(args.workload),
            "traffic_source": TRAFFIC_FILE + " (rocprofv3 FETCH_SIZE + WRITE_SIZE, recorded earlier; not measured by this run)"
                              if measured_traffic(args.workload) is not None else None,
            "step_device_ms_avg": avg_device_ms, "step_device_ms_avg_with_lead_in": t["with_lead_in_ms"],
            "step_device_ms_median": per_step[len(per_step) // 2], "step_device_ms_min": per_step[0],
            "algorithmic_bytes_per_step": step_bytes,
        },
    }
    if late_ms is not None:
        first = args.warmup + 2 * args.steps + 41
        out["roofline"]["later_steps"] = {"steps": [first, first + 19], "step_device_ms_avg": late_ms,
                                          "frac": step_bytes / (late_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
    if work.get("checkpoint_roundtrip"):
        out["config"]["checkpoint_roundtrip_bit_exact"] = checkpoint_roundtrip(work, device)
        out["config"]["checkpoint_bytes"] = work["checkpoint_bytes"]
    adam_on_bf16 = work["optimizer"] == "FlashAdamW" and work["mwb"] in (24, 32)
    exact_update = args.workload.endswith("-exact")
    work.clear()
    del work, step
    torch.cuda.empty_cache()
    if adam_on_bf16 and not args.no_parity:
        out["parity"] = parity_subcheck(device, torch.int8 if out["config"]["master_weight_bits"] == 24 else torch.int16,
                                        exact_update=exact_update)
    if args.workload == "llama8b-mwb24" and not args.no_secondary:
        # the short steps (2 ms and less) get more of them: their first twenty steps from zero states are slower than
        # the steady state (every value of a fresh state sits on a rounding boundary and takes the repair path)
        out["secondary"] = [run_secondary(name, device, steps=20 if name.startswith("llama8b") else 100,
                                          warmup=5 if name.startswith("llama8b") else 20, parity=not args.no_parity)
                            for name in SECONDARY]
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
