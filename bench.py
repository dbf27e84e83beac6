#!/usr/bin/env python3
"""Headline benchmark: fused 4-bit AdamW step on a LLaMA-7B-shaped fp32 parameter set.

One "step" = one `lpmm.optim.AdamW(fused=True).step()` over all 291 tensors (6 738 415 616
parameters) with parameters, gradients and states resident in HBM.  Prints ONE JSON line
with the step throughput (params/s), the HBM roofline of the dominant kernel measured live
with events on the launch stream, and a CPU baseline (the reference's non-fused PyTorch op
sequence on the host cores, bounded sample).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama7b|gpt2xl|tiny]    (defaults: 100 steps, 10 warm-up)

After the timed region the default run also measures, on the same box, what plain streaming
kernels with the fused step's access pattern reach (`roofline.calibration`; `--workload calibrate`
prints the full table alone).

Two further workloads measure the other kernels of the path with the same JSON shape:
`--workload quant64m` (stand-alone quantise/dequantise round trip on 2^26 values) and
`--workload factored` (factored second moment on LLaMA-7B MLP/attention shapes) and
`--workload nonfused_group|nonfused_rank1` (fused=False on the LLaMA-7B-shaped set; with the suffix
`_m32` under the configurations that quantise the second moment only: fp32 first moment;
`nonfused_rank1_mgroup`: first-moment groups of 1024 values; `nonfused_rank1 --bits 5..8`: the
configurations with wider codes; `--shapes gpt2xl|conv`: the GPT-2-XL-shaped set or the convolution
weights of a wide ResNet-152 instead; `--half`: float16 parameters and gradients) and
`--workload sgd` (4-bit SGD momentum on the same set).
"""
import argparse
import contextlib
import gc
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "low-bit-optimizers_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
BYTES_PER_PARAM_4BIT = 14.125  # p r/w 8 + g 4 + m codes 1 + v codes 1 + scales 16/128
BYTES_PER_PARAM_FP32 = 28.0    # p, m, v r/w + g r
MULTI_MAX = 48                 # tensors per launch record (LPMM_MULTI_MAX)
# HBM bytes per launch of the dominant kernel are not measured by this script: they come from
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this same command (each counter scaled by what it
# reads for a plain 1 GiB copy, --copy-probe), whose summary is kept in this file; the line
# "traffic_bytes_per_launch: <number>" in it is what the JSON reports, with the file named as
# "traffic_source".
TRAFFIC_PROFILE = {"llama7b": "profiles/fused_adamw4bit_llama7b_pmc.md"}


def recorded_traffic(workload):
    """(bytes per launch, source) from the committed counter summary, or (None, None)."""
    rel = TRAFFIC_PROFILE.get(workload)
    if rel is None:
        return None, None
    try:
        with open(os.path.join(ROOT, rel)) as fh:
            for line in fh:
                if line.startswith("traffic_bytes_per_launch:"):
                    return float(line.split(":", 1)[1]), (
                        rel + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run of this command; "
                        "not measured in this run)")
    except OSError:
        pass
    return None, None


def llama7b_shapes():
    shapes = [(32000, 4096)]
    for _ in range(32):
        shapes += [(4096, 4096)] * 4 + [(11008, 4096)] * 2 + [(4096, 11008)] + [(4096,)] * 2
    shapes += [(4096,), (32000, 4096)]
    return shapes


def gpt2xl_shapes():
    d = 1600
    shapes = [(50257, d), (1024, d)]
    for _ in range(48):
        shapes += [(d,), (d,), (d, 3 * d), (3 * d,), (d, d), (d,), (d,), (d,), (d, 4 * d), (4 * d,), (4 * d, d), (d,)]
    shapes += [(d,), (d,)]
    return shapes


def conv_shapes():
    """The convolution weights of a ResNet-152 at twice the width (bottleneck blocks: 1x1, 3x3, 1x1), 2.3e8
    parameters in 4-D tensors, plus the stem and the classifier."""
    shapes = [(128, 3, 7, 7)]
    for w, blocks in ((512, 3), (1024, 8), (2048, 36), (4096, 3)):
        for _ in range(blocks):
            shapes += [(w // 4, w, 1, 1), (w // 4, w // 4, 3, 3), (w, w // 4, 1, 1), (w,)]
    shapes += [(1000, 4096), (1000,)]
    return shapes


def tiny_shapes():
    return [(4096, 1024), (1024, 4096), (4096,), (8192,), (1000, 1000)] * 4


WORKLOADS = {
    "llama7b": ("fused 4-bit AdamW, LLaMA-7B-shaped fp32 set (291 tensors, 6.74e9 params), "
                "grads Student-t(3) x 1e-3", llama7b_shapes),
    "gpt2xl": ("fused 4-bit AdamW, GPT-2-XL-shaped fp32 set (580 tensors, 1.56e9 params), grads N(0,1e-3)",
               gpt2xl_shapes),
    "tiny": ("fused 4-bit AdamW, small test set", tiny_shapes),
}


def make_params(torch, shapes, dev, heavy_tailed, interleaved=False):
    """Synthetic parameters and gradients.  All parameters are allocated first and all gradients
    after them, the order in which a model and its first backward pass allocate them;
    `interleaved` puts each gradient right behind its parameter instead (for square tensors the
    two streams are then an exact power of two apart, which costs 1-2 % on this memory system)."""
    gen = torch.Generator(device=dev)

    def grad_for(i, shape):
        gen.manual_seed(20000 + i)
        z = torch.randn(shape, device=dev, generator=gen)
        if heavy_tailed:  # Student-t, 3 degrees of freedom: z / sqrt((a^2+b^2+c^2)/3)
            s = torch.zeros(shape, device=dev)
            for _ in range(3):
                a = torch.randn(shape, device=dev, generator=gen)
                s.addcmul_(a, a)
            z.div_(s.div_(3.0).sqrt_())
            del s, a
        return z.mul_(1e-3)

    params = []
    for i, shape in enumerate(shapes):
        gen.manual_seed(10000 + i)
        p = torch.nn.Parameter(torch.randn(shape, device=dev, generator=gen) * 0.02)
        if interleaved:
            p.grad = grad_for(i, shape)
        params.append(p)
    if not interleaved:
        for i, p in enumerate(params):
            p.grad = grad_for(i, p.shape)
    return params


def cpu_baseline(torch, steps=100):
    """The reference's non-fused PyTorch path (op sequence of _single_tensor_adamw4bit) on the
    host cores: one 4096x4096 fp32 parameter, m group-128 / v rank-1, all threads."""
    from oracle.nonfused_torch import TorchNonFusedAdamW

    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(0)
    p = torch.randn(4096, 4096, generator=g) * 0.02
    opt = TorchNonFusedAdamW([p], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, v_scale_type="rank1")
    times = []
    for s in range(steps + 1):
        gg = torch.Generator().manual_seed(1000 + s)
        grad = torch.randn(4096, 4096, generator=gg) * 1e-3
        t0 = time.perf_counter()
        opt.step([grad])
        times.append(time.perf_counter() - t0)
    times = sorted(times[1:])
    med = times[len(times) // 2]
    # for context: the C restatement of the fused kernel (OpenMP over 128-element groups) on the same tensor size
    import numpy as np

    from oracle import oracle as O

    n = 4096 * 4096
    rng = np.random.default_rng(0)
    pf = (rng.standard_normal(n, dtype=np.float32) * 0.02).astype(np.float32)
    gf = (rng.standard_normal(n, dtype=np.float32) * 1e-3).astype(np.float32)
    mc, vc = np.zeros(n // 2, np.uint8), np.zeros(n // 2, np.uint8)
    ms, vs = np.zeros(n // 128, np.float32), np.zeros(n // 128, np.float32)
    qm, qv = O.qmap_m(), O.qmap_v()
    fused_times = []
    for s in range(4):
        t0 = time.perf_counter()
        O.adamw4bit_step(pf, gf, mc, vc, ms, vs, qm, qv, 0.9, 0.999, 1e-3, 0.01, 1e-8, float(s + 1))
        fused_times.append(time.perf_counter() - t0)
    return {
        "value": p.numel() / med,
        "unit": "params/s",
        "cores": threads,
        "kind": "port",
        "sample": f"non-fused PyTorch-op path on CPU, one 4096x4096 fp32 tensor, m group-128 / v rank-1, "
                  f"median of {steps} steps after 1 warm-up",
        "fused_step_c_restatement_params_per_s": n / sorted(fused_times[1:])[1],
    }


PROBE_KINDS = {"read": (0, 4.0), "write": (1, 4.0), "copy": (2, 8.0), "update_2r1w": (3, 12.0),
               "fused_mix": (4, BYTES_PER_PARAM_4BIT), "fused_mix_dword_codes": (5, BYTES_PER_PARAM_4BIT)}
# workgroup shapes of lpmm_stream_probe (LPMM_PROBE_SHAPE_*) and the flag for the fused step's tile order
PROBE_SHAPES = {"256 threads, 1 tile": 0x000, "512 threads, 2 adjacent tiles": 0x100, "128 threads, half a tile": 0x200,
                "256 threads, 2 tiles loaded up front": 0x300}
PROBE_RUN_ORDER = 0x1000
# dynamic LDS per workgroup -> workgroups resident per CU (160 KB of LDS per CU)
PROBE_RESIDENCY = {16: 10 * 1024, 12: 13 * 1024, 8: 20 * 1024, 6: 26 * 1024, 5: 32 * 1024, 4: 40 * 1024, 3: 53 * 1024,
                   2: 80 * 1024}


def calibrate(torch, lib, n=1 << 29, iters=5, full=False):
    """What the memory system of this box gives to plain streaming kernels with the fused step's
    access pattern (lpmm_stream_probe: same lane layout and nontemporal accesses, no arithmetic):
    read, write, copy, the in-place 2-reads-1-write update, and the seven streams of the fused step,
    for four workgroup shapes at several residencies, with workgroup i on span i ("plain") and with
    the fused step's tile order ("run_order": every XCD streams 128 KB runs).  GB/s over `iters`
    back-to-back launches on 2^29 elements of random data (events on the launch stream), after 2
    warm-up launches."""
    from lpmm import _native

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(7)
    a = torch.randn(n, device=dev, generator=gen) * 0.02
    b = torch.randn(n, device=dev, generator=gen) * 1e-3
    c0 = torch.randint(0, 256, (n // 2,), dtype=torch.uint8, device=dev, generator=gen)
    c1 = torch.randint(0, 256, (n // 2,), dtype=torch.uint8, device=dev, generator=gen)
    s0 = torch.ones(n // 128, device=dev)
    s1 = torch.ones(n // 128, device=dev)
    stream = _native.current_stream(dev)

    def rate(kind, lds, flags=0):
        code, bytes_per_elt = PROBE_KINDS[kind]

        def launch():
            st = lib.lpmm_stream_probe(code | flags, a.data_ptr(), b.data_ptr(), c0.data_ptr(), c1.data_ptr(),
                                       s0.data_ptr(), s1.data_ptr(), n, lds, stream)
            _native.check(st, "stream probe")

        launch()
        launch()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            launch()
        e1.record()
        torch.cuda.synchronize()
        return n * bytes_per_elt * iters / (e0.elapsed_time(e1) * 1e-3) / 1e9

    out = {"elements": n, "unit": "GB/s", "data": "random"}
    # residencies per shape: the same numbers of waves per CU
    shape_res = {"256 threads, 1 tile": (5, 4, 8, 3, 2), "512 threads, 2 adjacent tiles": (3, 2, 4),
                 "128 threads, half a tile": (8, 6, 16, 12), "256 threads, 2 tiles loaded up front": (3, 2, 4)}
    for kind in ("read", "write", "copy", "update_2r1w"):
        for order, flag in (("plain", 0), ("run_order", PROBE_RUN_ORDER)):
            key = kind if order == "plain" else kind + "_run_order"
            if full:
                out[key] = {str(r): round(rate(kind, PROBE_RESIDENCY[r], flag), 1) for r in (8, 5, 4, 3, 2)}
            else:
                out[key] = round(max(rate(kind, PROBE_RESIDENCY[r], flag) for r in (5, 3)), 1)
    best = {}
    for shape, sflag in PROBE_SHAPES.items():
        for order, flag in (("plain", 0), ("run_order", PROBE_RUN_ORDER)):
            res = shape_res[shape] if full else shape_res[shape][:2]
            table = {str(r): round(rate("fused_mix", PROBE_RESIDENCY[r], sflag | flag), 1) for r in res}
            out.setdefault("fused_mix_by_workgroups_per_cu", {})[f"{shape}, {order}"] = table
            best[f"{shape}, {order}"] = max(table.values())
    out["fused_mix_best_by_shape"] = best
    out["fused_mix_best"] = max(best.values())
    if full:  # the same streams with one 4-byte code access per lane and state instead of two 2-byte ones
        out["fused_mix_dword_codes_by_workgroups_per_cu"] = {
            str(r): round(rate("fused_mix_dword_codes", PROBE_RESIDENCY[r], PROBE_RUN_ORDER), 1) for r in (8, 5, 4, 3, 2)}
    del a, b, c0, c1, s0, s1
    return out


def verify_one_more_step(torch, opt, params):
    """Are the timed launches doing the work?  Takes the states the timed steps left for three
    sampled tensors (a quantised one from the middle of a launch group, the last quantised one,
    an fp32-state one), runs ONE more optimizer step over the whole set, and compares what that
    step wrote for them with the CPU oracle's step from the same states: codes and scales bit
    for bit, parameters within 1e-6 relative.  Outside the timed region; the oracle is only the
    checker.  Returns (ok, description)."""
    import numpy as np

    from oracle import oracle as O

    quant = [i for i, p in enumerate(params) if p.numel() > 4096]
    plain = [i for i, p in enumerate(params) if p.numel() <= 4096]
    picks = []
    if quant:
        small = [i for i in quant if params[i].numel() <= (1 << 26)] or quant
        picks.append(small[len(small) // 2])
        if quant[-1] not in picks and params[quant[-1]].numel() <= (1 << 28):
            picks.append(quant[-1])
    if plain:
        picks.append(plain[len(plain) // 2])
    group = opt.param_groups[0]
    hyper = (group["betas"][0], group["betas"][1], group["lr"], group["weight_decay"], group["eps"])
    qm, qv = O.qmap_m(), O.qmap_v()

    def host(t):
        return t.detach().cpu().numpy().reshape(-1).copy()

    before = {}
    for i in picks:
        st = opt.state[params[i]]
        snap = {"p": host(params[i]), "g": host(params[i].grad)}
        if params[i].numel() > 4096:
            snap.update(mc=host(st["exp_avg"]).view(np.uint8), vc=host(st["exp_avg_sq"]).view(np.uint8),
                        ms=host(st["exp_avg_qstate"]["overhead"]["max1"]),
                        vs=host(st["exp_avg_sq_qstate"]["overhead"]["max1"]))
        else:
            snap.update(m=host(st["exp_avg"]), v=host(st["exp_avg_sq"]))
        before[i] = snap
    opt.step()
    torch.cuda.synchronize()
    problems = []
    for i in picks:
        st, b = opt.state[params[i]], before[i]
        step = float(st["step"])
        p_old = b["p"].copy()
        if "mc" in b:
            O.adamw4bit_step(b["p"], b["g"], b["mc"], b["vc"], b["ms"], b["vs"], qm, qv, *hyper, step)
            same = (np.array_equal(host(st["exp_avg"]).view(np.uint8), b["mc"])
                    and np.array_equal(host(st["exp_avg_sq"]).view(np.uint8), b["vc"])
                    and np.array_equal(host(st["exp_avg_qstate"]["overhead"]["max1"]), b["ms"])
                    and np.array_equal(host(st["exp_avg_sq_qstate"]["overhead"]["max1"]), b["vs"]))
        else:
            O.adamw_fp32_step(b["p"], b["g"], b["m"], b["v"], *hyper, step)
            same = np.array_equal(host(st["exp_avg"]), b["m"]) and np.array_equal(host(st["exp_avg_sq"]), b["v"])
        got = host(params[i]).astype(np.float64)
        yard = np.maximum(np.maximum(np.abs(b["p"]), np.abs(p_old)), np.finfo(np.float32).tiny)
        p_ok = bool(np.all(np.abs(got - b["p"]) <= 1e-6 * yard))
        if not (same and p_ok):
            problems.append(f"tensor {i} {tuple(params[i].shape)}: states {'equal' if same else 'DIFFER'}, "
                            f"parameters {'within 1e-6' if p_ok else 'DIFFER'}")
    what = ", ".join(f"#{i} {tuple(params[i].shape)}" for i in picks)
    if problems:
        return False, "; ".join(problems)
    return True, f"step {int(step)} of tensors {what}: codes, scales and fp32 states bit-exact, parameters within 1e-6"


@contextlib.contextmanager
def _gc_paused():
    """A full collection of the interpreter's cyclic garbage collector takes 70-80 ms of host time
    with torch loaded, several optimizer steps: collect first, keep it off inside a timed region.
    The warm-up steps run inside the same block, after the collection: a GPU that sits idle for
    those 80 ms between the warm-up and the timed steps runs the first launches after the pause
    8-15 % slower (the first timed step 15.8 ms against 14.5 ms for the others in a kernel trace)."""
    gc.collect()
    gc.disable()
    try:
        yield
    finally:
        gc.enable()


def _time_events(torch, fn, iters):
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with _gc_paused():
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters  # ms


def run_quant_roundtrip(torch, args):
    """Stand-alone quantise + dequantise round trip on 2^26 fp32 values (--bits wide codes, 4 by
    default: packed two per byte; 3 and 5..8 take a byte each): group-128 with the signed
    dynamic-exponent map (N(0,1) with 0.1 % outliers x50), group-128 with the unsigned linear
    map (|N|^2), rank-1 on the unsigned data viewed 8192 x 8192 and 64 x 1024 x 1024."""
    import lpmm.functional as F

    b = args.bits
    code_bytes = F.storage_bits(b) / 8.0

    dev = torch.device("cuda:0")
    n = 1 << 26
    g = torch.Generator(device=dev)
    g.manual_seed(1)
    signed = torch.randn(n, device=dev, generator=g)
    g.manual_seed(2)
    idx = torch.randperm(n, device=dev, generator=g)[: n // 1000]
    signed[idx] *= 50.0
    g.manual_seed(3)
    unsigned = torch.randn(n, device=dev, generator=g) ** 2
    qm = F.create_general_qmap("nonlinear", b, True).to(dev)
    qv = F.create_general_qmap("power-1", b, False).to(dev)
    md_m = dict(b=b, scale_type="group", quant_type="nonlinear", round_type="real-nearest", gp_sz=128, signed=True)
    md_vg = dict(b=b, scale_type="group", quant_type="power-1", round_type="real-nearest", gp_sz=128, signed=False)
    md_vr = dict(md_vg, scale_type="rank1")
    variants = []
    # bytes per value: 4 read or written as fp32, the code, a scale per 128 values; the rank-1
    # quantiser reads the values twice (statistics, then normalise + search + pack)
    one_pass, two_pass = 4 + code_bytes + 4 / 128, 8 + code_bytes
    for name, x, qmap, md, bytes_q, bytes_dq in (
            ("group-128 signed DE map", signed, qm, md_m, one_pass, one_pass),
            ("group-128 unsigned linear map", unsigned, qv, md_vg, one_pass, one_pass),
            ("rank-1 8192x8192 unsigned linear map", unsigned.view(8192, 8192), qv, md_vr, two_pass, 4 + code_bytes),
            ("rank-1 64x1024x1024 unsigned linear map", unsigned.view(64, 1024, 1024), qv, md_vr, two_pass,
             4 + code_bytes)):
        qx, gen = F.vectorwise_quant(x, qmap=qmap, shape=x.shape, **md)
        kw = {**gen, **md}
        back = F.vectorwise_dequant(qx, qmap=qmap, shape=x.shape, **kw)
        relerr = float((x - back).norm() / x.norm())
        t_q = _time_events(torch, lambda: F.vectorwise_quant(x, qmap=qmap, shape=x.shape, **md), args.steps)
        t_dq = _time_events(torch, lambda: F.vectorwise_dequant(qx, qmap=qmap, shape=x.shape, **kw), args.steps)
        variants.append({"variant": name, "quant_ms": t_q, "dequant_ms": t_dq, "roundtrip_values_per_s": n / ((t_q + t_dq) * 1e-3),
                         "quant_gbs": n * bytes_q / t_q / 1e6, "dequant_gbs": n * bytes_dq / t_dq / 1e6, "relerr": relerr})
    v0 = variants[0]
    print(json.dumps({
        "metric": f"{b}-bit quantize+dequantize round trip (group-128, signed map): values/sec, 1 MI355X",
        "value": v0["roundtrip_values_per_s"], "unit": "values/s", "n_gpus": 1, "steps": args.steps, "warmup": 2,
        "ms_per_step": v0["quant_ms"] + v0["dequant_ms"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"quantize+dequantize round trip on 2^26 fp32 values, {b}-bit codes"},
        "roofline": {"bound": "hbm", "kernel": "lpmm::quant_group_kernel" if b == 4 else "lpmm::quant_group_bits_kernel",
                     "achieved": v0["quant_gbs"],
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": v0["quant_gbs"] / HBM_PEAK_GBS, "traffic": None},
        "variants": variants}))


def run_factored(torch, args):
    """Factored second moment on LLaMA-7B MLP/attention shapes: 32 x {4096x11008, 11008x4096,
    4096x4096} plus 1-D biases (11008: 4-bit m and v; 4096: fp32 states), grads N(0, 1e-3)."""
    import lpmm

    dev = torch.device("cuda:0")
    shapes = []
    for _ in range(32):
        shapes += [(4096, 11008), (11008, 4096), (4096, 4096), (11008,), (4096,)]
    params = make_params(torch, shapes, dev, heavy_tailed=False)
    opt = lpmm.optim.AdamW(params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01,
                           factor_second_moment=True, fused=True)
    n_total = sum(p.numel() for p in params)
    n_2d = sum(p.numel() for p in params if p.dim() == 2)
    with _gc_paused():
        for _ in range(args.warmup):
            opt.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            opt.step()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / args.steps
    achieved = n_2d * 17.0625 / dt / 1e9
    print(json.dumps({
        "metric": "factored-second-moment 4-bit AdamW step: params/sec, 1 MI355X", "value": n_total / dt,
        "unit": "params/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "factor_second_moment=True, 32 x {4096x11008, 11008x4096, 4096x4096} + 1-D biases",
                   "tensors": len(params), "params": n_total},
        "roofline": {"bound": "hbm", "kernel": "factored_partial_kernel + factored_update_kernel (whole step)",
                     "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": None, "bytes_per_param": 17.0625}}))


def run_sgd(torch, args):
    """lpmm.optim.SGD (momentum 0.9, 4-bit momentum buffer) on the LLaMA-7B-shaped set: one pass
    per launch group of 64 tensors, 13.0625 B per quantised parameter (p read and written 8, g 4,
    codes read and written 1, scales 8/128); the 65 norm vectors keep fp32 buffers and take the
    reference's chain of PyTorch ops."""
    import lpmm

    dev = torch.device("cuda:0")
    params = make_params(torch, llama7b_shapes(), dev, heavy_tailed=True)
    opt = lpmm.optim.SGD(params, lr=1e-3, momentum=0.9, weight_decay=1e-4)
    n_total = sum(p.numel() for p in params)
    with _gc_paused():
        for _ in range(args.warmup):
            opt.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            opt.step()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / args.steps
    bytes_per_param = 13.0625
    achieved = n_total * bytes_per_param / dt / 1e9
    print(json.dumps({
        "metric": "4-bit SGD-momentum step: params/sec, 1 MI355X", "value": n_total / dt,
        "unit": "params/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "SGD, momentum 0.9, 4-bit momentum buffer, LLaMA-7B-shaped fp32 set",
                   "tensors": len(params), "params": n_total},
        "roofline": {"bound": "hbm", "kernel": "whole step", "achieved": achieved, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "bytes_per_param": bytes_per_param}}))


def run_nonfused(torch, args, v_scale, m32=False, mgroup=False):
    """fused=False on the LLaMA-7B-shaped set.  v_scale 'group': both moments block-wise over
    128 values, one kernel per launch group of tensors; 'rank1' (the reference's default
    configuration): an update pass and a re-quantise pass per launch group of tensors.
    m32: the configurations that quantise the second moment only (the first moment is an fp32
    state, read and written as floats by the same passes).  mgroup: first-moment groups of 1024
    values with the rank-1 second moment (the first moment's codes are written by the second pass)."""
    import lpmm

    dev = torch.device("cuda:0")
    shapes = {"gpt2xl": gpt2xl_shapes, "conv": conv_shapes, "llama7b": llama7b_shapes}[args.shapes]()
    params = make_params(torch, shapes, dev, heavy_tailed=True)
    half = args.half
    if half:
        if m32 or mgroup or args.bits != 4 or args.shapes != "llama7b":
            sys.exit("bench.py: --half goes with --workload nonfused_group|nonfused_rank1 on the LLaMA-7B-shaped set")
        # float16 parameters and gradients (gradients of 1e-3 scale: most squares underflow in half, as they
        # do in a real float16 run without loss scaling); eps 1e-3, since float16 rounds 1e-8 to zero
        halves = []
        for q in params:
            h = torch.nn.Parameter(q.detach().half())
            h.grad = q.grad.half()
            halves.append(h)
        params = halves
    bits = args.bits if (v_scale == "rank1" and not m32 and not mgroup) else 4
    if bits != 4:
        if bits < 5:
            sys.exit("bench.py: --workload nonfused_rank1 takes --bits 4 (default) to 8")
        name = f"default_{bits}b.yml"
    elif mgroup:
        name = "1st_moment_group_1024.yml"
    elif m32:
        name = "2nd_moment_only_group_128.yml" if v_scale == "group" else "2nd_moment_only_default.yml"
    else:
        name = "2nd_moment_group_128.yml" if v_scale == "group" else "default.yml"
    cfg = os.path.join(os.path.dirname(lpmm.config.__file__), "configs", name)
    opt = lpmm.optim.AdamW(params, lr=1e-3, betas=(0.9, 0.999), eps=1e-3 if half else 1e-8, weight_decay=0.01,
                           fused=False, qconfig=cfg)
    n_total = sum(p.numel() for p in params)
    with _gc_paused():
        for _ in range(args.warmup):
            opt.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            opt.step()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / args.steps
    # one pass: p, g read, p written, two 4-bit codes read and written, scales;
    # rank-1 (two passes): + g and the v codes read a second time, v codes written in the second pass
    bytes_per_param = BYTES_PER_PARAM_4BIT if v_scale == "group" else 18.5625
    if m32:  # m read and written as floats (8) instead of codes and scales (1.0625)
        bytes_per_param += 8.0 - 1.0625
    if mgroup:  # update pass: p 8, g 4, both codes read 1; second pass: g 4, both codes read and written 2
        bytes_per_param = 19.0 + 12.0 / 1024
    if bits != 4:  # one code per byte: p 8, g 4 + 4, m codes 2, v codes 1 + 2, scales 8/128
        bytes_per_param = 21.0625
    if half:  # p 2 + 2, g 2 (+ 2 in the second pass), codes and half scales as above
        bytes_per_param = 8.0625 if v_scale == "group" else 7.53125 + 3.0
    if args.shapes != "llama7b":
        # a mix of paths: per tensor, what its path moves (rank-1: tensors whose shape[0] x rest view has
        # whole 128-column blocks, or half a block left over with an even row count, as above; other
        # multiples of 8 through the kernels for ragged rows 19.0625; what is left takes the staged path
        # (dequantise, update on fp32 temporaries, statistics, quantise: about 50); quantised vectors one
        # pass 14.125; fp32 states 28)
        total = 0.0
        for p in params:
            rows, cols = p.shape[0], p.numel() // p.shape[0]
            if p.numel() <= 4096:
                total += 28.0 * p.numel()
            elif v_scale == "group" or p.dim() == 1:
                total += BYTES_PER_PARAM_4BIT * p.numel()
            elif cols % 128 == 0 or (cols % 128 == 64 and rows % 2 == 0):
                total += 18.5625 * p.numel()
            elif p.dim() == 2 and cols % 8 == 0:
                total += 19.0625 * p.numel()
            else:
                total += 50.0 * p.numel()
        bytes_per_param = total / n_total
    achieved = n_total * bytes_per_param / dt / 1e9
    print(json.dumps({
        "metric": "non-fused 4-bit AdamW step: params/sec, 1 MI355X", "value": n_total / dt,
        "unit": "params/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"fused=False, {'float16 parameters, ' if half else ''}{'fp32 first moment, ' if m32 else ''}{'first-moment groups of 1024, ' if mgroup else ''}second moment '{v_scale}' scaling, "
                               f"{ {'gpt2xl': 'GPT-2-XL-shaped', 'conv': 'wide-ResNet-152 convolution', 'llama7b': 'LLaMA-7B-shaped'}[args.shapes]} {'fp16' if half else 'fp32'} set", "qconfig": name,
                   "tensors": len(params), "params": n_total},
        "roofline": {"bound": "hbm", "kernel": "whole step", "achieved": achieved, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "bytes_per_param": bytes_per_param}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="llama7b", choices=sorted(WORKLOADS) + ["quant64m", "factored", "nonfused_group", "nonfused_rank1", "nonfused_group_m32", "nonfused_rank1_m32", "nonfused_rank1_mgroup", "sgd", "calibrate"])
    ap.add_argument("--half", action="store_true",
                    help="float16 parameters and gradients for --workload nonfused_group|nonfused_rank1")
    ap.add_argument("--bits", type=int, default=4, choices=range(1, 9),
                    help="code width of --workload quant64m (1-8) and nonfused_rank1 (4-8)")
    ap.add_argument("--shapes", default="llama7b", choices=["llama7b", "gpt2xl", "conv"],
                    help="parameter set of the nonfused_* workloads")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--interleaved-grads", action="store_true",
                    help="allocate each gradient right behind its parameter instead of all parameters first")
    ap.add_argument("--no-calibration", action="store_true",
                    help="skip the streaming-rate calibration that follows the timed region")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run three plain 1 GiB device copies first (calibration dispatches for "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported "
                 "(the optimizer step is rank-local: each GPU would run this same kernel on its own shard).")

    import torch

    import lpmm
    from lpmm import _native

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = _native.lib()

    if args.copy_probe:
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)  # 1 GiB read + 1 GiB written per copy
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if args.workload == "calibrate":
        cal = calibrate(torch, lib, iters=max(args.steps, 3), full=True)
        best = cal["fused_mix_best"]
        print(json.dumps({
            "metric": "streaming-rate calibration: the fused step's seven-stream access pattern without arithmetic",
            "value": best, "unit": "GB/s", "n_gpus": 1, "steps": max(args.steps, 3), "warmup": 2,
            "ms_per_step": cal["elements"] * BYTES_PER_PARAM_4BIT / best / 1e6, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "lpmm_stream_probe on 2^29 elements, all kinds and residencies"},
            "roofline": {"bound": "hbm", "kernel": "lpmm::probe_fused_mix_kernel", "achieved": best,
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": best / HBM_PEAK_GBS, "traffic": None},
            "calibration": cal}))
        return
    if args.workload == "quant64m":
        return run_quant_roundtrip(torch, args)
    if args.workload == "factored":
        return run_factored(torch, args)
    if args.workload == "sgd":
        return run_sgd(torch, args)
    if args.workload.startswith("nonfused_"):
        return run_nonfused(torch, args, args.workload.split("_")[1], m32=args.workload.endswith("_m32"),
                            mgroup=args.workload.endswith("_mgroup"))

    desc, shape_fn = WORKLOADS[args.workload]
    shapes = shape_fn()
    params = make_params(torch, shapes, dev, heavy_tailed=(args.workload == "llama7b"),
                         interleaved=args.interleaved_grads)
    opt = lpmm.optim.AdamW(params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01, fused=True)

    n_total = sum(p.numel() for p in params)
    n_quant = sum(p.numel() for p in params if p.numel() > 4096)
    n_quant_tensors = sum(1 for p in params if p.numel() > 4096)
    launches_per_step = math.ceil(n_quant_tensors / MULTI_MAX)

    # events around the dominant kernel's launches (same stream as the launches)
    events = []
    real_call = lib.lpmm_adamw4bit_step_multi
    recording = {"on": False}

    def timed_call(*a):
        if not recording["on"]:
            return real_call(*a)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        st = real_call(*a)
        e1.record()
        events.append((e0, e1))
        return st

    lib.lpmm_adamw4bit_step_multi = timed_call

    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    with _gc_paused():
        for _ in range(args.warmup):
            opt.step()
        torch.cuda.synchronize()
        recording["on"] = True
        t0 = time.perf_counter()
        marks[0].record()
        for i in range(args.steps):
            opt.step()
            marks[i + 1].record()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    recording["on"] = False
    per_step_ms = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))

    verified, verified_on = verify_one_more_step(torch, opt, params)
    traffic, traffic_source = recorded_traffic(args.workload)

    ms_per_step = elapsed * 1e3 / args.steps
    value = n_total / (elapsed / args.steps)
    kernel_ms_per_step = sum(e0.elapsed_time(e1) for e0, e1 in events) / args.steps
    launch_ms = kernel_ms_per_step / launches_per_step
    bytes_per_launch = n_quant * BYTES_PER_PARAM_4BIT / launches_per_step
    achieved = bytes_per_launch / (launch_ms * 1e-3) / 1e9

    out = {
        "metric": "fused 4-bit AdamW step: params/sec and % HBM roofline, 1 MI355X",
        "value": value,
        "unit": "params/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        # the same steps one by one on the GPU's clock (events on the launch stream)
        "step_ms_median": per_step_ms[len(per_step_ms) // 2],
        "step_ms_min": per_step_ms[0],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        # one more step after the timed region, checked against the CPU oracle on sampled tensors
        "verified": verified,
        "verified_on": verified_on,
        "config": {"workload": desc, "tensors": len(params), "params": n_total, "quantized_params": n_quant,
                   # the 4-bit kernel's launches plus the fp32-state kernel's (tensors of <= 4096 elements, 64 per launch)
                   "launches_per_step": launches_per_step + math.ceil((len(params) - n_quant_tensors) / 64)},
        "effective_gbs": (n_quant * BYTES_PER_PARAM_4BIT + (n_total - n_quant) * BYTES_PER_PARAM_FP32)
        / (elapsed / args.steps) / 1e9,
        "roofline": {
            "bound": "hbm",
            # second template argument, chosen per launch: every tensor of the launch is a whole
            # number of 2048-element tiles
            "kernel": "lpmm::adamw4bit_kernel<true, %s, lpmm::FusedArith4>" % (
                "true" if all(p.numel() % 2048 == 0 for p in params if p.numel() > 4096) else "true|false"),
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic,
            "traffic_source": traffic_source,
            "bytes_per_launch": bytes_per_launch,
            "avg_launch_ms": launch_ms,
        },
    }
    if not args.no_calibration:
        # the same box, the same run: what plain streaming kernels with this access pattern reach
        cal = calibrate(torch, lib, iters=20)
        out["roofline"]["calibration"] = cal
        out["roofline"]["frac_of_fused_mix_best"] = achieved / cal["fused_mix_best"]
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch)
    print(json.dumps(out))
    if not verified:
        sys.exit("bench.py: the step after the timed region does not match the CPU oracle: " + verified_on)


if __name__ == "__main__":
    main()
