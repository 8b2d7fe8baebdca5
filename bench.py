#!/usr/bin/env python3
"""Benchmark of the FFT-convolution path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--all-configs] [--no-cpu]

One "step" is one full layer training step of the batch-128 configuration
(updateOutput + updateGradInput + accGradParameters on batch 128, 128 -> 128
planes, 13x13 input, 3x3 kernel, pad 1, FFT size 16) on synthetic inputs that are
resident in HBM before the timed region starts.  `value` is the effective
convolution rate: direct-convolution FLOPs (2*B*F*P*oH*oW*kH*kW per pass, three
passes per step) divided by wall time.  The line also carries ms per pass, the
roofline position of every stage (HIP events recorded by the library on the
stream its kernels run on), the dominant kernel's roofline object, the CPU
oracle timed on this box's host cores and, under "configs", the same per-pass and
per-stage records for the other stated configurations (the 8192-plane FFT round
trip, the batch-128 updateOutput layer and the large-kernel layer).

Every stage is timed three ways.  `ms_in_pass` is the median duration of the stage's
kernel(s) inside an ordinary pass, each launch timed by the start and end of its own
dispatch (what a profiler's kernel trace reports: operands wherever the previous
kernel left them, no launch gap, no event overhead); `frac`, `achieved` and the
`roofline` object use it.  `ms` is the mean of STAGE_REPS back-to-back launches of the
same stage between two events (operands warm in the caches: `frac_warm`), `ms_single`
one launch between two events (about 2 us of event overhead included).  `resident`
says that the stage's whole working set fits the 256 MB memory-side cache, so that
its "HBM" rate is in part cache bandwidth.  For the
contraction, `algorithmic_frac` counts 8 flops per complex multiply-add and
`mfma_issued_frac` the 6 the kernels issue (three real products per complex one):
the second is the utilisation of the fp32 matrix pipe.  Kernel names and grids come
from the library (fbfc_plan_stage_kernel), as a profiler trace shows them.
"""
import argparse
import json
import os
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_FP32_PEAK_TF = 157.3    # MI355X dense fp32 matrix, published

CONFIGS = {
    # name: B, P, F, H(=W), k, pad, passes, weight std, seed
    "config3_fprop_b128_64x64_27x27_k5_p2": (128, 64, 64, 27, 5, 2, ("fprop",), 0.05, 1003),
    "config4_step_b128_128x128_13x13_k3_p1": (128, 128, 128, 13, 3, 1, ("fprop", "bprop", "accgrad"), 0.05, 1004),
    "config5_step_b64_96x256_55x55_k9_p4": (64, 96, 256, 55, 9, 4, ("fprop", "bprop", "accgrad"), 0.02, 1005),
}
MAIN = "config4_step_b128_128x128_13x13_k3_p1"
STAGE_REPS = 10
MALL_BYTES = 256e6           # memory-side cache: a stage whose working set fits is "resident"


def stage_model(cfg, pass_, n, q):
    """Algorithmic bytes / flops of each stage of one pass (intermediates counted
    once written and once read; no scratch traffic)."""
    B, P, F, H, k, pad = cfg[:6]
    o = H + 2 * pad - k + 1
    # the passes leave out the n - 2 frequencies that are conjugates of others (columns kx = 0 and
    # n/2, rows above n/2): they are neither written, contracted nor read
    q = q - (n - 2)
    fft = lambda planes, h: 4 * planes * h * h + 8 * planes * q
    mm_bytes = lambda m, nn_, kk: 8 * q * (m * kk + kk * nn_ + m * nn_)
    mm_flops = lambda m, nn_, kk: 8 * q * m * nn_ * kk
    # "fft": both forward transforms of the pass, which are one launch; in accGradParameters the
    # bias gradient (B*F complex numbers of FFT(gradOutput)'s zero-frequency row) rides on the
    # inverse-FFT launch
    if pass_ == "fprop":
        return {"fft": ("hbm", fft(B * P, H) + fft(F * P, k)),
                "mm": ("mfma", mm_flops(B, F, P), mm_bytes(B, F, P)),
                "ifft": ("hbm", fft(B * F, o))}
    if pass_ == "bprop":
        return {"fft": ("hbm", fft(B * F, o) + fft(F * P, k)),
                "mm": ("mfma", mm_flops(B, P, F), mm_bytes(B, P, F)),
                "ifft": ("hbm", fft(B * P, H))}
    return {"fft": ("hbm", fft(B * F, o) + fft(B * P, H)),
            "mm": ("mfma", mm_flops(F, P, B), mm_bytes(F, P, B)),
            "ifft": ("hbm", fft(F * P, k) + 8 * B * F)}


TRAFFIC_PROFILE = os.path.join("profiles", "hbm_traffic_all_configs.txt")


def csrc_digest():
    """Short SHA-256 over the kernel sources (fbcunn_amd/csrc, sorted by name): the profile summaries
    carry the digest of the sources they were measured on, so that a reader of a bench line can tell
    whether a looked-up counter value belongs to the kernels that ran."""
    import hashlib
    h = hashlib.sha256()
    d = os.path.join(ROOT, "fbcunn_amd", "csrc")
    for name in sorted(os.listdir(d)):
        if name.endswith((".hip", ".h", ".cpp")):
            h.update(name.encode())
            h.update(open(os.path.join(d, name), "rb").read())
    return h.hexdigest()[:12]


def profiled_traffic():
    """HBM bytes per launch, per (kernel, grid), from the committed rocprofv3 --pmc summary
    (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 KiB, the factors a 256 MiB device copy gives for the
    same counters), and the digest of the kernel sources the summary says it was measured on.
    Empty if the file is missing or was measured on other sources than the ones present."""
    import re
    out = {}
    try:
        text = open(os.path.join(ROOT, TRAFFIC_PROFILE)).read()
    except OSError:
        return out, None
    m = re.search(r"csrc_sha256=([0-9a-f]+)", text)
    head = m.group(1) if m else None
    if head != csrc_digest():
        return out, head
    pat = re.compile(r"^(?:fbfc::)?(\S.*?)\s+grid=(\d+)\s+FETCH_SIZE=(\d+) KiB \(x([0-9.]+).*?WRITE_SIZE=(\d+) KiB \(x([0-9.]+)", re.M)
    for m in pat.finditer(text):
        name, grid = m.group(1).strip(), int(m.group(2))
        out[(name, grid)] = (int(m.group(3)) * float(m.group(4)) + int(m.group(5)) * float(m.group(6))) * 1024
    return out, head


TRACE_PROFILE = os.path.join("profiles", "kernel_trace_default_bench_run.txt")


def profiled_durations():
    """Average duration (ms) per (kernel, grid) in the committed rocprofv3 --kernel-trace summary of this
    command, or {} if the summary was measured on other kernel sources than the ones present."""
    import re
    out = {}
    try:
        text = open(os.path.join(ROOT, TRACE_PROFILE)).read()
    except OSError:
        return out
    m = re.search(r"csrc_sha256=([0-9a-f]+)", text)
    if not m or m.group(1) != csrc_digest():
        return out
    for m in re.finditer(r"^(?:fbfc::)?(\S.*?)\s+(\d+)\s+(\d+)\s+(\d+)\s+(\d+)\s+(\d+)\s+(\d+)\s+[0-9.]+\s*$", text, re.M):
        out[(m.group(1).strip(), int(m.group(2)))] = int(m.group(5)) * 1e-6
    return out


def split_launch(desc):
    """'<kernel> grid=<n>; ...' -> [(kernel, grid), ...]"""
    out = []
    for part in desc.split(";"):
        part = part.strip()
        if part:
            name, _, grid = part.rpartition(" grid=")
            out.append((name, int(grid)))
    return out


def make_layer(nn, torch, synth, cfg):
    B, P, F, H, k, pad, _, wstd, seed = cfg
    o = H + 2 * pad - k + 1
    net = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad)
    net.weight.copy_(torch.from_numpy(synth.normal(seed, (F, P, k, k), 0.0, wstd, stream=1)).cuda())
    net.bias.copy_(torch.from_numpy(synth.uniform(seed, (F,), -0.1, 0.1, stream=2)).cuda())
    x = torch.from_numpy(synth.uniform(seed, (B, P, H, H), stream=0)).cuda()
    g = torch.from_numpy(synth.uniform(seed, (B, F, o, o), stream=3)).cuda()
    return net, x, g


def run_pass(net, x, g, pass_):
    if pass_ == "fprop":
        net.updateOutput(x)
    elif pass_ == "bprop":
        net.updateGradInput(x, g)
    else:
        net.accGradParameters(x, g, 1.0)


def time_loop(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def time_each(torch, fn, steps, warmup):
    """Per-call device time of fn (HIP events on the stream the library launches on, which is
    torch's current stream): median and minimum over `steps` calls, in ms."""
    for _ in range(warmup):
        fn()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    ms = sorted(a.elapsed_time(b) for a, b in evs)
    return {"median": ms[len(ms) // 2], "min": ms[0]}


def stage_times(net, x, g, p, reps, runs):
    """Per-stage ms of pass p and what each stage launched.  reps > 1: `reps` back-to-back launches per
    stage between two events, mean over `runs` passes; reps == 1: one launch between two events, median;
    reps == -1: every launch timed by its own dispatch inside an ordinary pass, median."""
    net.timed = reps
    acc, kernels = {}, {}
    run_pass(net, x, g, p)
    for _ in range(runs):
        if reps < 0:
            # the timed pass is queued right behind two untimed ones, so that its kernels find the device
            # busy, as they do in a training loop
            net.timed = False
            run_pass(net, x, g, p)
            run_pass(net, x, g, p)
            net.timed = reps
        run_pass(net, x, g, p)
        one = {}
        for s, v in net.stageTimes(x).items():
            s = "fft" if s in ("fft_a", "fft_b") else s   # the forward transforms of the pass
            one[s] = one.get(s, 0.0) + v
        for s, v in one.items():
            acc.setdefault(s, []).append(v)
    for s, v in net.stageKernels(x).items():
        s = "fft" if s in ("fft_a", "fft_b") else s
        kernels[s] = (kernels[s] + "; " + v) if s in kernels else v
    net.timed = False
    if reps > 1:
        return {s: sum(v) / len(v) for s, v in acc.items()}, kernels
    return {s: sorted(v)[len(v) // 2] for s, v in acc.items()}, kernels


def measure_config(nn, torch, synth, name, steps, warmup, layer=None):
    cfg = CONFIGS[name]
    B, P, F, H, k, pad, passes = cfg[:7]
    o = H + 2 * pad - k + 1
    net, x, g = layer if layer is not None else make_layer(nn, torch, synth, cfg)
    flop_pass = 2.0 * B * F * P * o * o * k * k
    res = {"passes": {}}
    # whole step, untimed stages
    net.timed = False
    ms_step = time_loop(torch, lambda: [run_pass(net, x, g, p) for p in passes], steps, warmup)
    res["ms_per_step"] = ms_step
    res["effective_tflops"] = flop_pass * len(passes) / (ms_step * 1e-3) / 1e12
    plan = net._plan_for(B, H, H)
    n, q = plan.info.fft_size, plan.info.n_freq
    for p in passes:
        net.timed = False
        ms = time_loop(torch, lambda: run_pass(net, x, g, p), steps, warmup)
        entry = {"ms": ms, "effective_tflops": flop_pass / (ms * 1e-3) / 1e12,
                 "ms_single_call": time_each(torch, lambda: run_pass(net, x, g, p), max(10, steps), warmup),
                 "stages": {}}
        warm, kernels = stage_times(net, x, g, p, STAGE_REPS, 3)
        single, _ = stage_times(net, x, g, p, 1, 7)
        in_pass, _ = stage_times(net, x, g, p, -1, 15)
        model = stage_model(cfg, p, n, q)
        for s, spec in model.items():
            ms_w, ms_s = warm.get(s, 0.0), in_pass.get(s, 0.0)
            if ms_w <= 0 or ms_s <= 0:
                continue
            st = {"kernel": kernels.get(s, ""), "ms_in_pass": ms_s, "ms": ms_w, "ms_single": single.get(s),
                  "bound": spec[0]}
            if spec[0] == "hbm":
                ach = spec[1] / (ms_s * 1e-3) / 1e9
                st.update({"bytes": spec[1], "achieved": ach, "unit": "GB/s", "peak": HBM_PEAK_GBS,
                           "frac": ach / HBM_PEAK_GBS, "frac_warm": spec[1] / (ms_w * 1e-3) / 1e9 / HBM_PEAK_GBS,
                           "resident": spec[1] <= MALL_BYTES})
            else:
                ach = spec[1] / (ms_s * 1e-3) / 1e12
                # the kernels form a complex product from three real ones: they issue 6 of the
                # 8 algorithmic flops per complex multiply-add
                issued = spec[1] * 0.75
                st.update({"flops": spec[1], "bytes": spec[2], "achieved": ach, "unit": "TFLOP/s",
                           "peak": MFMA_FP32_PEAK_TF, "frac": ach / MFMA_FP32_PEAK_TF,
                           "frac_warm": spec[1] / (ms_w * 1e-3) / 1e12 / MFMA_FP32_PEAK_TF,
                           "algorithmic_frac": ach / MFMA_FP32_PEAK_TF, "flops_issued": issued,
                           "mfma_issued_frac": issued / (ms_s * 1e-3) / 1e12 / MFMA_FP32_PEAK_TF,
                           "hbm_gbs": spec[2] / (ms_s * 1e-3) / 1e9, "resident": spec[2] <= MALL_BYTES})
            entry["stages"][s] = st
        res["passes"][p] = entry
    res["fft_size"] = n
    net.cleanupBuffers()
    return res


def compact(res):
    """The per-pass / per-stage record of a configuration without the byte and flop counts."""
    keep = ("kernel", "ms_in_pass", "ms", "ms_single", "bound", "frac", "frac_warm", "resident", "algorithmic_frac",
            "mfma_issued_frac")
    return {"ms_per_step": res["ms_per_step"], "effective_tflops": res["effective_tflops"], "fft_size": res["fft_size"],
            "passes": {p: {"ms": e["ms"], "effective_tflops": e["effective_tflops"],
                           "stages": {s: {k: st[k] for k in keep if k in st} for s, st in e["stages"].items()}}
                       for p, e in res["passes"].items()}}


def measure_fft_round_trip(nn, torch, synth, steps, warmup):
    """8192 planes of 32x32: forward then inverse, each timed on its own (`ms`: back-to-back
    launches between two events; `ms_single`: median of single launches, an event pair around each)."""
    n, planes = 32, 8192
    x = torch.from_numpy(synth.uniform(1002, (planes, n, n))).cuda()
    freq = torch.empty((n, n // 2 + 1, planes, 2), device="cuda")
    back = torch.empty_like(x)
    w = nn.FFTWrapper("fbfft")
    out = {}
    for name, fn in (("fft", lambda: w.fft(x, freq)), ("ifft", lambda: w.ffti(back, freq))):
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(warmup):
            fn()
        ev0.record()
        for _ in range(steps):
            fn()
        ev1.record()
        torch.cuda.synchronize()
        ms = ev0.elapsed_time(ev1) / steps
        nbytes = 4 * planes * n * n + 8 * planes * n * (n // 2 + 1)
        ach = nbytes / (ms * 1e-3) / 1e9
        # a stand-alone transform has no pass around it: the figure is the back-to-back one, and its 69 MB
        # working set stays in the memory-side cache between launches
        out[name] = {"kernel": w.lastKernel(), "ms": ms, "ms_single": time_each(torch, fn, 15, 2)["median"],
                     "bound": "hbm", "bytes": nbytes, "achieved": ach, "unit": "GB/s", "peak": HBM_PEAK_GBS,
                     "frac": ach / HBM_PEAK_GBS, "frac_warm": ach / HBM_PEAK_GBS, "resident": nbytes <= MALL_BYTES}
    return out


def measure_fft_1d(nn, torch, steps, warmup):
    """Batched 1-D transforms (fbfft1dHost's job, src/fft/FBFFTHost.cpp:119-131): 256 MiB of real rows
    of each size, forward and unnormalised inverse; bytes = the rows once plus the half spectra once."""
    out = {}
    for n in (8, 32, 64, 128):
        rows = (1 << 26) // n
        x = torch.rand(rows, n, device="cuda")
        freq = torch.empty((rows, n // 2 + 1, 2), device="cuda")
        back = torch.empty_like(x)
        w = nn.FFTWrapper("fbfft")
        rec = {"rows": rows}
        for name, fn in (("fft", lambda: w.fft(x, freq)), ("ifft", lambda: w.ffti(back, freq))):
            ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            for _ in range(warmup):
                fn()
            ev0.record()
            for _ in range(steps):
                fn()
            ev1.record()
            torch.cuda.synchronize()
            ms = ev0.elapsed_time(ev1) / steps
            nbytes = 4 * rows * n + 8 * rows * (n // 2 + 1)
            ach = nbytes / (ms * 1e-3) / 1e9
            rec[name] = {"kernel": w.lastKernel(), "ms": ms, "bound": "hbm", "bytes": nbytes, "achieved": ach,
                         "unit": "GB/s", "peak": HBM_PEAK_GBS, "frac": ach / HBM_PEAK_GBS}
        out["n%d" % n] = rec
        del x, freq, back
    return out


def measure_reuse_step(nn, torch, synth, steps, warmup):
    """The same training step with memoryReuseAll (bprop reuses FFT(weight), accGrad reuses
    FFT(gradOutput) and FFT(input)): 3 forward FFTs per step instead of 6."""
    cfg = CONFIGS[MAIN]
    B, P, F, H, k, pad, passes, wstd, seed = cfg
    o = H + 2 * pad - k + 1
    net = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad, "all")
    net.weight.copy_(torch.from_numpy(synth.normal(seed, (F, P, k, k), 0.0, wstd, stream=1)).cuda())
    net.bias.zero_()
    x = torch.from_numpy(synth.uniform(seed, (B, P, H, H), stream=0)).cuda()
    g = torch.from_numpy(synth.uniform(seed, (B, F, o, o), stream=3)).cuda()
    # auxiliary figure: a long loop, see measure_backward_step
    steps, warmup = max(steps, 200), max(warmup, 50)
    ms = time_loop(torch, lambda: [run_pass(net, x, g, p) for p in passes], steps, warmup)
    net.cleanupBuffers()
    return {"ms_per_step": ms, "steps": steps, "effective_tflops": 3 * 2.0 * B * F * P * o * o * k * k / (ms * 1e-3) / 1e12}


def measure_tiled(nn, torch, synth, steps, warmup):
    """A VGG-like layer (batch 64, 64 -> 128 planes, 112 x 112, 3 x 3, pad 1; the reference's tiled
    benchmark shape, test/test_FFT.lua:466-467) through the tiled modules (tiles 32 and 16) and, for
    comparison, through one FFT of size 128 per plane."""
    B, P, F, H, k, pad, seed = 64, 64, 128, 112, 3, 1, 1006
    o = H + 2 * pad - k + 1
    flop_pass = 2.0 * B * F * P * o * o * k * k
    x = torch.from_numpy(synth.uniform(seed, (B, P, H, H), stream=0)).cuda()
    g = torch.from_numpy(synth.uniform(seed, (B, F, o, o), stream=3)).cuda()
    w = torch.from_numpy(synth.normal(seed, (F, P, k, k), 0.0, 0.05, stream=1)).cuda()
    out = {"workload": "vgg_like_b64_64x128_112x112_k3_p1", "gflop_per_pass": flop_pass / 1e9, "variants": {}}
    passes = ("fprop", "bprop", "accgrad")
    for name, tile in (("tile32", 32), ("tile16", 16), ("untiled_fft128", None)):
        if tile is None:
            net = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad)
        else:
            net = nn.SpatialConvolutionFFTTiled(P, F, k, k, 1, 1, pad, pad, tile, tile)
        net.weight.copy_(w)
        net.bias.zero_()
        n = max(3, steps // 5)
        entry = {"ms_per_step": time_loop(torch, lambda: [run_pass(net, x, g, p) for p in passes], n, 2)}
        entry["effective_tflops"] = 3 * flop_pass / (entry["ms_per_step"] * 1e-3) / 1e12
        entry["ms_per_pass"] = {p: time_loop(torch, lambda: run_pass(net, x, g, p), n, 1) for p in passes}
        net.timed = 3
        entry["stage_ms"] = {}
        for p in passes:
            run_pass(net, x, g, p)
            entry["stage_ms"][p] = {s: v for s, v in net.stageTimes(x).items() if v > 0}
        net.timed = False
        plan = net._plan_for(B, H, H)
        entry["fft_size"] = plan.info.fft_size
        entry["tiles"] = [plan.info.tiles_h, plan.info.tiles_w]
        net.cleanupBuffers()
        out["variants"][name] = entry
    return out


def measure_iterated(nn, torch, synth, steps):
    """First- and last-layer shapes (few planes on one side; batch 64, 112 x 112, 3 x 3, pad 1, tiles of 16)
    through the three-kernel tiled module and through nn.SpatialConvolutionFFTTiledIterated, whose passes are
    single fused kernels that never write a spectrum of a feature map to memory: ms per pass, both ways."""
    out = {}
    passes = ("fprop", "bprop", "accgrad")
    for name, (B, P, F, k, H, pad, tile) in {"first_layer_b64_3to64_112x112_k3_p1_tile16": (64, 3, 64, 3, 112, 1, 16),
                                             "last_layer_b64_64to3_112x112_k3_p1_tile16": (64, 64, 3, 3, 112, 1, 16),
                                             "mid_layer_b64_16to64_112x112_k3_p1_tile16": (64, 16, 64, 3, 112, 1, 16)}.items():
        o = H + 2 * pad - k + 1
        x = torch.from_numpy(synth.uniform(1007, (B, P, H, H), stream=0)).cuda()
        g = torch.from_numpy(synth.uniform(1007, (B, F, o, o), stream=3)).cuda()
        w = torch.from_numpy(synth.normal(1007, (F, P, k, k), 0.0, 0.05, stream=1)).cuda()
        rec = {"gflop_per_pass": 2.0 * B * F * P * o * o * k * k / 1e9}
        for label, cls in (("tiled_three_kernels", "SpatialConvolutionFFTTiled"), ("iterated_fused", "SpatialConvolutionFFTTiledIterated")):
            net = getattr(nn, cls)(P, F, k, k, 1, 1, pad, pad, tile, tile)
            net.weight.copy_(w)
            net.bias.zero_()
            n = max(5, steps // 3)
            per = {p: time_loop(torch, lambda: run_pass(net, x, g, p), n, 2) for p in passes}
            kernels = {}
            for p in passes:
                run_pass(net, x, g, p)
                kernels[p] = net.stageKernels(x).get("mm", "")
            rec[label] = {"ms_per_pass": per, "ms_per_step": sum(per.values()), "contraction_kernel": kernels}
            net.cleanupBuffers()
        rec["speedup_per_pass"] = {p: rec["tiled_three_kernels"]["ms_per_pass"][p] / rec["iterated_fused"]["ms_per_pass"][p]
                                   for p in passes}
        out[name] = rec
    return out


def measure_backward_step(nn, torch, synth, steps, warmup):
    """The training step as a module user runs it: updateOutput, then backward(), whose two gradient
    passes share FFT(gradOutput) (5 forward transforms per step instead of 6)."""
    cfg = CONFIGS[MAIN]
    B, P, F, H, k, pad = cfg[:6]
    o = H + 2 * pad - k + 1
    net, x, g = make_layer(nn, torch, synth, cfg)
    def step():
        net.updateOutput(x)
        net.backward(x, g, 1.0)
    # an auxiliary figure, not the contract's K steps: long loops, so that the idle time spent building the
    # layer does not show (the first hundred steps after an idle period run up to 10 % slower)
    steps, warmup = max(steps, 200), max(warmup, 50)
    ms = time_loop(torch, step, steps, warmup)
    ms_b = time_loop(torch, lambda: net.backward(x, g, 1.0), steps, warmup)
    net.cleanupBuffers()
    # the same with memoryReuseAll: backward() then transforms gradOutput only (3 forward transforms per step)
    wstd, seed = cfg[7], cfg[8]
    keep = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad, "all")
    keep.weight.copy_(torch.from_numpy(synth.normal(seed, (F, P, k, k), 0.0, wstd, stream=1)).cuda())
    keep.bias.zero_()
    def step_keep():
        keep.updateOutput(x)
        keep.backward(x, g, 1.0)
    ms_k = time_loop(torch, step_keep, steps, warmup)
    keep.cleanupBuffers()
    flop = 3 * 2.0 * B * F * P * o * o * k * k
    return {"ms_per_step": ms, "ms_backward": ms_b, "steps": steps, "effective_tflops": flop / (ms * 1e-3) / 1e12,
            "ms_per_step_reuse_all": ms_k, "effective_tflops_reuse_all": flop / (ms_k * 1e-3) / 1e12}


def measure_reference_list(nn, torch, synth, steps):
    """The layers of the reference's own benchmark list for this path (OverFeat-like, test/test_FFT.lua:440-448;
    batch 128, memoryReuseNone): ms per pass and effective TFLOP/s of the three-pass step."""
    layers = [(128, 96, 256, 5, 24, 2), (128, 256, 512, 3, 12, 1), (128, 512, 1024, 3, 12, 1), (128, 1024, 1024, 3, 12, 1)]
    out = {}
    for B, P, F, k, H, pad in layers:
        o = H + 2 * pad - k + 1
        net = nn.SpatialConvolutionFBFFT(P, F, k, k, 1, 1, pad, pad)
        net.bias.zero_()
        x = torch.from_numpy(synth.uniform(7, (B, P, H, H), stream=0)).cuda()
        g = torch.from_numpy(synth.uniform(7, (B, F, o, o), stream=3)).cuda()
        passes = ("fprop", "bprop", "accgrad")
        n = max(3, steps // 5)
        ms = time_loop(torch, lambda: [run_pass(net, x, g, p) for p in passes], n, 2)
        per = {p: time_loop(torch, lambda: run_pass(net, x, g, p), n, 1) for p in passes}
        flop = 2.0 * B * F * P * o * o * k * k
        out["b%d_%dto%d_%dx%d_k%d_p%d" % (B, P, F, H, H, k, pad)] = {
            "ms_per_step": ms, "ms_per_pass": per, "effective_tflops": 3 * flop / (ms * 1e-3) / 1e12,
            "fft_size": net._plan_for(B, H, H).info.fft_size}
        net.cleanupBuffers()
    return out


# Layers measured against the platform library on request (--vendor-layers): the tiled VGG-like layer, the first-,
# last- and mid-layer shapes of the fused module and the reference's benchmark list, each through the module this
# library would run it with.  name: (B, P, F, H, k, pad, passes, weight std, seed, module class, tile)
_STEP = ("fprop", "bprop", "accgrad")
VENDOR_LAYERS = {
    "vgg_like_b64_64x128_112x112_k3_p1": (64, 64, 128, 112, 3, 1, _STEP, 0.05, 1006, "SpatialConvolutionFFTTiled", 32),
    "first_layer_b64_3to64_112x112_k3_p1": (64, 3, 64, 112, 3, 1, _STEP, 0.05, 1007, "SpatialConvolutionFFTTiledIterated", 16),
    "last_layer_b64_64to3_112x112_k3_p1": (64, 64, 3, 112, 3, 1, _STEP, 0.05, 1007, "SpatialConvolutionFFTTiledIterated", 16),
    "mid_layer_b64_16to64_112x112_k3_p1": (64, 16, 64, 112, 3, 1, _STEP, 0.05, 1007, "SpatialConvolutionFFTTiled", 16),
    "b128_96to256_24x24_k5_p2": (128, 96, 256, 24, 5, 2, _STEP, 0.05, 7, "SpatialConvolutionFBFFT", None),
    "b128_256to512_12x12_k3_p1": (128, 256, 512, 12, 3, 1, _STEP, 0.05, 7, "SpatialConvolutionFBFFT", None),
    "b128_512to1024_12x12_k3_p1": (128, 512, 1024, 12, 3, 1, _STEP, 0.05, 7, "SpatialConvolutionFBFFT", None),
    "b128_1024to1024_12x12_k3_p1": (128, 1024, 1024, 12, 3, 1, _STEP, 0.05, 7, "SpatialConvolutionFBFFT", None),
}


def make_vendor_layer(nn, torch, synth, name):
    if name in CONFIGS:
        return make_layer(nn, torch, synth, CONFIGS[name])
    B, P, F, H, k, pad, _, wstd, seed, cls, tile = VENDOR_LAYERS[name]
    o = H + 2 * pad - k + 1
    args = (P, F, k, k, 1, 1, pad, pad) + ((tile, tile) if tile else ())
    net = getattr(nn, cls)(*args)
    net.weight.copy_(torch.from_numpy(synth.normal(seed, (F, P, k, k), 0.0, wstd, stream=1)).cuda())
    net.bias.copy_(torch.from_numpy(synth.uniform(seed, (F,), -0.1, 0.1, stream=2)).cuda())
    x = torch.from_numpy(synth.uniform(seed, (B, P, H, H), stream=0)).cuda()
    g = torch.from_numpy(synth.uniform(seed, (B, F, o, o), stream=3)).cuda()
    return net, x, g


def measure_vendor(nn, torch, synth, names, steps):
    """The same layers through the platform library's convolution (MIOpen behind aten::convolution, fp32, with its
    search for the fastest algorithm switched on) beside this library's time for them: the role cuDNN has in the
    reference's benchmark (test/test_FFT.lua:300-336).  Step = updateOutput + updateGradInput + accGradParameters
    as three calls, as in the headline; fprop_plus_backward = updateOutput + one call that produces both gradients."""
    from fbcunn_amd.vendor import SpatialConvolutionMIOpen
    out = {}
    was = torch.backends.cudnn.benchmark
    torch.backends.cudnn.benchmark = True
    try:
        for name in names:
            cfg = CONFIGS[name] if name in CONFIGS else VENDOR_LAYERS[name]
            B, P, F, H, k, pad = cfg[:6]
            o = H + 2 * pad - k + 1
            passes = cfg[6]
            net, x, g = make_vendor_layer(nn, torch, synth, name)
            print("bench.py: platform library on %s (its search can take minutes)" % name, file=sys.stderr, flush=True)
            ven = SpatialConvolutionMIOpen(P, F, k, k, 1, 1, pad, pad, init=False)
            ven.weight, ven.bias = net.weight, net.bias
            t0 = time.perf_counter()
            # a line a minute while the library searches, for whoever watches the run
            done = threading.Event()
            def heartbeat():
                while not done.wait(60.0):
                    print("bench.py: ... still searching (%d s)" % (time.perf_counter() - t0), file=sys.stderr, flush=True)
            beat = threading.Thread(target=heartbeat, daemon=True)
            beat.start()
            try:
                try:
                    for p in passes:
                        run_pass(ven, x, g, p)      # the library searches and builds its kernels here
                    torch.cuda.synchronize()
                finally:
                    done.set()
                    beat.join()
            except Exception as err:
                out[name] = {"error": "%s: %s" % (type(err).__name__, str(err)[:200])}
                net.cleanupBuffers()
                continue
            first_s = time.perf_counter() - t0
            a, b = net.updateOutput(x), ven.updateOutput(x)
            agree = float((a - b).abs().max()) / float(b.abs().max())
            n = max(steps, 200) if H < 32 else max(steps // 2, 10)
            def step(mod):
                for p in passes:
                    run_pass(mod, x, g, p)
            rec = {"module": type(net).__name__, "first_call_s": first_s, "steps": n, "output_max_diff_over_max": agree,
                   "vendor_ms_per_step": time_loop(torch, lambda: step(ven), n, max(2, n // 10)),
                   "ms_per_step": time_loop(torch, lambda: step(net), n, max(2, n // 10))}
            if len(passes) == 3:
                def fb(mod):
                    mod.updateOutput(x)
                    mod.backward(x, g, 1.0)
                rec["vendor_ms_fprop_plus_backward"] = time_loop(torch, lambda: fb(ven), n, max(2, n // 10))
                rec["ms_fprop_plus_backward"] = time_loop(torch, lambda: fb(net), n, max(2, n // 10))
            flop = len(passes) * 2.0 * B * F * P * o * o * k * k
            rec["vendor_effective_tflops"] = flop / (rec["vendor_ms_per_step"] * 1e-3) / 1e12
            rec["effective_tflops"] = flop / (rec["ms_per_step"] * 1e-3) / 1e12
            rec["speedup"] = rec["vendor_ms_per_step"] / rec["ms_per_step"]
            out[name] = rec
            net.cleanupBuffers()
            ven.cleanupBuffers()
    finally:
        torch.backends.cudnn.benchmark = was
    return out


def measure_spectrum_store_policy(nn, torch, synth, steps, warmup):
    """The forward transforms write their spectra through to the memory side, whose cache keeps them for the
    contraction; non-temporal stores stream them past it.  Measured alone the transform is as fast either way,
    the step is not.  Both ways, same layer, same run: the main workload's step and its fprop FFT stage."""
    from fbcunn_amd import _lib
    cfg = CONFIGS[MAIN]
    passes = cfg[6]
    out = {}
    for name, mode in (("write_through", -1), ("non_temporal", 1)):
        _lib.check(_lib.lib().fbfc_debug_force_spectrum_streaming(mode))
        try:
            net, x, g = make_layer(nn, torch, synth, cfg)
            ms_step = time_loop(torch, lambda: [run_pass(net, x, g, p) for p in passes], max(steps, 100), max(warmup, 10))
            warm, _ = stage_times(net, x, g, "fprop", STAGE_REPS, 3)
            model = stage_model(cfg, "fprop", net._plan_for(cfg[0], cfg[3], cfg[3]).info.fft_size,
                                net._plan_for(cfg[0], cfg[3], cfg[3]).info.n_freq)
            out[name] = {"ms_per_step": ms_step, "fprop_fft_stage_ms_warm": warm["fft"],
                         "fprop_fft_stage_frac_warm": model["fft"][1] / (warm["fft"] * 1e-3) / 1e9 / HBM_PEAK_GBS}
            net.cleanupBuffers()
        finally:
            _lib.check(_lib.lib().fbfc_debug_force_spectrum_streaming(-1))
    return out


def measure_copy_bandwidth(torch, floats=64 * 1024 * 1024, reps=10):
    """A plain device-to-device copy (256 MiB by default): what HBM delivers to a trivial kernel on this box."""
    a = torch.zeros(floats, dtype=torch.float32, device="cuda")
    b = torch.empty_like(a)
    for _ in range(3):
        b.copy_(a)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        b.copy_(a)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    return {"ms": ms, "GBps_read_plus_write": 2 * a.numel() * 4 / (ms * 1e-3) / 1e9}


def measure_small_copies(torch):
    """Plain copies that move as many bytes as the transform launches of the main workload (an inverse
    transform reads 18.9 MB and writes 11.1 MB, a forward pair reads 22 MB and writes 38 MB): launches of
    this size are as much ramp as streaming, and this is what the same box gives a trivial kernel for them."""
    out = {}
    for mb in (30, 60):
        r = measure_copy_bandwidth(torch, floats=mb * 1000 * 1000 // 8, reps=50)
        out["%dMB_moved" % mb] = {"ms": r["ms"], "GBps_read_plus_write": r["GBps_read_plus_write"],
                                  "frac_of_hbm_peak": r["GBps_read_plus_write"] / HBM_PEAK_GBS}
    return out


def measure_mfma_clock(nn, torch):
    """The shader clock the tile contraction kernel runs at (clock counters inside the kernel), for the main
    workload's contraction shape and for a wide one that keeps the matrix pipes busy for milliseconds.
    The published fp32 MFMA peak assumes the 2.4 GHz peak clock."""
    from fbcunn_amd import probe   # the measurement library, not part of the shipped one
    out = {"peak_clock_mhz": 2400.0}
    for name, (Q, m, n, k, launches) in {"config4_contraction": (130, 128, 128, 128, 20),
                                         "wide_contraction_130x128x1024x1024": (130, 128, 1024, 1024, 5)}.items():
        A = torch.rand(Q, m, k, 2, device="cuda") - 0.5
        B = torch.rand(Q, n, k, 2, device="cuda") - 0.5
        C = torch.empty(Q, m, n, 2, device="cuda")
        mhz = probe.contractionClock(0, A, B, C, launches=launches)
        out[name] = {"mhz": mhz, "fp32_mfma_peak_at_this_clock_tflops": MFMA_FP32_PEAK_TF * mhz / 2400.0}
        del A, B, C
    return out


def cpu_baseline(synth):
    """The CPU oracle on the main workload: the whole batch-128 training step
    (three passes, 19.1 GFLOP of direct convolution), all host threads OpenMP
    gives it, one run after a small warm-up."""
    import oracle
    cfg = CONFIGS[MAIN]
    B, P, F, H, k, pad, passes, wstd, seed = cfg
    o = H + 2 * pad - k + 1
    x = synth.uniform(seed, (B, P, H, H), stream=0)
    w = synth.normal(seed, (F, P, k, k), 0.0, wstd, stream=1)
    g = synth.uniform(seed, (B, F, o, o), stream=3)
    p4 = (pad,) * 4
    oracle.cross_correlation_valid(x[:2], w, (1, 1), p4)   # warm-up (loads the library, spins up threads)
    runs, dt = 8, float("inf")
    for _ in range(runs):   # about 6 s of CPU work on 16 threads; the fastest run counts
        t0 = time.perf_counter()
        oracle.cross_correlation_valid(x, w, (1, 1), p4)
        oracle.convolution_full(g, w, (1, 1), p4)
        oracle.cross_correlation_reverse_valid(x, g, (1, 1), 1.0, p4)
        dt = min(dt, time.perf_counter() - t0)
    flops = 3 * 2.0 * B * F * P * o * o * k * k
    threads = oracle.set_threads(0)
    # the reference's own CPU-runnable case (batch 4, 16 -> 16 planes, 32 x 32, 5 x 5, fprop) on one thread
    x1 = synth.uniform(1001, (4, 16, 32, 32), stream=0)
    w1 = synth.uniform(1001, (16, 16, 5, 5), stream=1)
    oracle.set_threads(1)
    t1 = time.perf_counter()
    oracle.cross_correlation_valid(x1, w1, (1, 1), (0, 0, 0, 0))
    dt1 = time.perf_counter() - t1
    oracle.set_threads(threads)
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "ms_per_step": dt * 1e3,
            "config1_fprop_single_thread_ms": dt1 * 1e3,
            "sample": "the whole %s step (fprop+bprop+accGrad, %.1f GFLOP), best of %d runs, OpenMP over independent outputs"
                      % (MAIN, flops / 1e9, runs)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--all-configs", action="store_true",
                    help="also measure the tiled VGG-like layer and the reference's benchmark layers")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU oracle timing")
    ap.add_argument("--no-vendor", action="store_true",
                    help="skip the platform library's convolution (its first call on a layer takes 10 s to 2 min)")
    ap.add_argument("--vendor-layers", action="store_true",
                    help="also time the tiled, first-/last-layer and reference-benchmark layers against the platform "
                         "library (its searches add about 12 minutes)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run a plain 256 MiB device copy 3 times (a kernel of known traffic "
                         "for scaling FETCH_SIZE / WRITE_SIZE counter readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives exist on this path); "
                 "use --gpus 1")

    import torch
    from fbcunn_amd import nn, synth
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    torch.cuda.set_device(0)

    if args.calibrate_copy:
        a = torch.zeros(64 * 1024 * 1024, dtype=torch.float32, device="cuda")
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        del a, b

    # The main workload's tensors and plan are made first and the other stated configurations measured next, so
    # that its W warm-up and K timed steps start on a device that has been busy until that moment, as it is
    # in training: after tens of milliseconds of idling (tensor generation on the host) the first hundred
    # steps run up to 10 % slower than the steady state.
    main_layer = make_layer(nn, torch, synth, CONFIGS[MAIN])
    for p in CONFIGS[MAIN][6]:
        run_pass(main_layer[0], main_layer[1], main_layer[2], p)   # creates the plan and the result tensors
    configs = {}
    configs["config2_fft_round_trip_8192x32x32"] = measure_fft_round_trip(nn, torch, synth, args.steps, args.warmup)
    for name in CONFIGS:   # config 3, then config 5: the heaviest one runs last, right before the main workload
        if name != MAIN:
            # secondary figures: enough steps for 10 ms or more of continuous work per loop
            n_steps = max(args.steps, 200) if CONFIGS[name][3] < 32 else max(args.steps, 30)
            configs[name] = compact(measure_config(nn, torch, synth, name, n_steps, max(args.warmup, n_steps // 10)))
            configs[name]["steps"] = n_steps

    main_res = measure_config(nn, torch, synth, MAIN, args.steps, args.warmup, layer=main_layer)
    # dominant kernel of the step = the stage with the largest in-pass time
    worst, worst_ms = None, -1.0
    for p, e in main_res["passes"].items():
        for s, st in e["stages"].items():
            if st["ms_in_pass"] > worst_ms:
                worst, worst_ms = (p, s, st), st["ms_in_pass"]
    p, s, st = worst
    traffic = None
    launches = split_launch(st["kernel"])
    table, traffic_head = profiled_traffic()
    if len(launches) == 1 and launches[0] in table:
        traffic = table[launches[0]]
    # achieved / frac: the kernel's duration inside an ordinary pass (its own dispatch, as a profiler's
    # kernel trace reports it); frac_warm: 10 launches back to back with the operands warm in the caches
    roofline = {"bound": st["bound"], "achieved": st["achieved"], "peak": st["peak"], "unit": st["unit"],
                "frac": st["frac"], "frac_warm": st["frac_warm"], "resident": st["resident"], "traffic": traffic,
                "traffic_source": (TRAFFIC_PROFILE + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this kernel and grid; "
                                   "not measured in this run)") if traffic is not None else None,
                # digest of the kernel sources the profile was measured on; traffic is null when it is not
                # the digest of the sources that ran (csrc_sha256)
                "traffic_head": traffic_head, "csrc_sha256": csrc_digest(),
                "kernel": st["kernel"], "pass": p, "stage": s, "avg_launch_ms": st["ms_in_pass"],
                "warm_launch_ms": st["ms"], "single_launch_ms": st["ms_single"]}
    # The same kernel's average duration in the committed rocprofv3 kernel trace of this command, and the
    # fraction it gives.  The trace stretches these 5-20 us kernels by a few per cent: its per-kernel averages of
    # one pass add up to more than the pass takes unprofiled, while the per-launch times above add up to it
    # (consistency below).
    prof = profiled_durations()
    if len(launches) == 1 and launches[0] in prof:
        unit_scale = 1e9 if st["bound"] == "hbm" else 1e12
        work = st["bytes"] if st["bound"] == "hbm" else st["flops"]
        roofline["profile_avg_launch_ms"] = prof[launches[0]]
        roofline["frac_from_profile"] = work / (prof[launches[0]] * 1e-3) / unit_scale / st["peak"]
        roofline["profile_source"] = TRACE_PROFILE
    consistency = {}
    for pp, e in main_res["passes"].items():
        consistency[pp] = {"pass_ms": e["ms"], "sum_of_in_pass_kernel_ms": sum(x["ms_in_pass"] for x in e["stages"].values())}
        names = [split_launch(x["kernel"]) for x in e["stages"].values()]
        if all(len(n) == 1 and n[0] in prof for n in names):
            consistency[pp]["sum_of_profile_avg_ms"] = sum(prof[n[0]] for n in names)
    if "mfma_issued_frac" in st:
        # achieved / frac count the algorithmic 8 flops per complex multiply-add; the kernel issues 6 of
        # them: mfma_issued_frac is the utilisation of the fp32 matrix pipe
        roofline["algorithmic_frac"] = st["algorithmic_frac"]
        roofline["mfma_issued_frac"] = st["mfma_issued_frac"]

    line = {
        "metric": "effective conv TFLOP/s (direct-convolution FLOPs / time), full training step at batch 128",
        "value": main_res["effective_tflops"], "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": main_res["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": MAIN, "fft_size": main_res["fft_size"],
                   "step": "updateOutput+updateGradInput+accGradParameters, every pass recomputes its FFTs"},
        "ms_per_pass": {k: v["ms"] for k, v in main_res["passes"].items()},
        "ms_per_pass_single_call": {k: v["ms_single_call"] for k, v in main_res["passes"].items()},
        "tflops_per_pass": {k: v["effective_tflops"] for k, v in main_res["passes"].items()},
        "roofline": roofline,
        "pass_time_consistency": consistency,
        "stages": {k: v["stages"] for k, v in main_res["passes"].items()},
    }
    line["reuse_all_step"] = measure_reuse_step(nn, torch, synth, args.steps, args.warmup)
    line["fprop_plus_backward_step"] = measure_backward_step(nn, torch, synth, args.steps, args.warmup)
    line["copy_256MiB"] = measure_copy_bandwidth(torch)
    line["copy_stage_sized"] = measure_small_copies(torch)
    line["mfma_clock"] = measure_mfma_clock(nn, torch)
    line["spectrum_store_policy"] = measure_spectrum_store_policy(nn, torch, synth, args.steps, args.warmup)
    if "mfma_issued_frac" in roofline:
        # the same utilisation against the matrix peak at the clock the kernel was measured to run at
        c = line["mfma_clock"]["config4_contraction"]["mhz"]
        roofline["mfma_clock_mhz"] = c
        roofline["mfma_issued_frac_at_measured_clock"] = roofline["mfma_issued_frac"] * 2400.0 / c if c > 0 else None
    line["configs"] = configs
    if args.all_configs:
        line["other_workloads"] = {
            "tiled_convolution": measure_tiled(nn, torch, synth, args.steps, args.warmup),
            "iterated_convolution": measure_iterated(nn, torch, synth, args.steps),
            "reference_benchmark_layers": measure_reference_list(nn, torch, synth, args.steps),
            "fft_1d": measure_fft_1d(nn, torch, args.steps, args.warmup)}
    if not args.no_vendor:
        # last of the GPU work: the library's search must not sit between the measurements above.  The default run
        # takes the headline layer only; the others' first calls take minutes
        names = list(CONFIGS) if args.all_configs else [MAIN]
        if args.vendor_layers:
            names += list(VENDOR_LAYERS)
        try:
            line["vendor_convolution"] = measure_vendor(nn, torch, synth, names, args.steps)
        except Exception as err:    # a comparison figure must not cost the line
            line["vendor_convolution"] = {"error": "%s: %s" % (type(err).__name__, str(err)[:200])}
    line["cpu_baseline"] = None if args.no_cpu else cpu_baseline(synth)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
