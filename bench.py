#!/usr/bin/env python3
"""Benchmark of the TAGI Linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload gemm|skinny]

A step is one forward + backward (delta_z, delta_w, delta_b) of a single TAGI
Linear layer on synthetic inputs that are resident in HBM before the timed
region starts. The default workload is the dense one the headline metric is
quoted on (4096 -> 4096, batch 256, fp32); `--workload skinny` times the
HBM-bound one (8192 -> 8192, batch 8) and reports GB/s. The default run also
times the skinny workload (and its 12- and 16-sample variants), the Conv2d
workload, one training step of the MLP configuration and of the CIFAR ResNet-18,
and the CPU baseline, and attaches them to the same JSON line, together with what
the runtime reports for the device and the wall time of the GPU legs.

Prints ONE JSON line. `roofline` is computed for the dominant kernel from its
algorithmic work and its average duration measured with HIP events on the
stream the kernels run on; `cpu_baseline` is the reference's multithreaded CPU path
timed on this host: its own sources compiled in place where that library is present
(kind "reference"), otherwise the bit-identical restatement (kind "port"). Every
secondary workload in `extra` carries its own `cpu_baseline` beside its GPU figure
(a bounded sample of the same workload, stated in `sample`), and its own `roofline`.
`warmup_effective_steps` / `warmup_seconds` say how long the GPU really worked before
the timed region: `--warmup` steps plus as many more as it takes to reach 0.3 s.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix peak (published)
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E peak (published)
FP32_MFMA_FLOP_PER_CLK_PER_CU = 256  # v_mfma_f32_32x32x2_f32: 4096 flop in 64 cycles on each of 4 SIMDs

WORKLOADS = {
    # name: (K, N, B, bound)
    "gemm": (4096, 4096, 256, "mfma"),
    "skinny": (8192, 8192, 8, "hbm"),
    # 12 and 16 samples (their state backward runs on the 16-wide kernel too), in `extra` only
    "skinny12": (8192, 8192, 12, "hbm"),
    "skinny16": (8192, 8192, 16, "hbm"),
    # between the two regimes: the tiled kernels on few rows, reported in `extra.mid`
    "mid32": (4096, 4096, 32, "mfma"),
    "mid64": (4096, 4096, 64, "mfma"),
}
# HBM bytes per launch of the kernel that dominates each phase of a step, keyed by
# the kernel that runs there: FETCH_SIZE and WRITE_SIZE of two `rocprofv3 --pmc`
# runs of this script, each scaled by what the same counter reads for a plain 1 GiB
# copy (`--calibrate` adds that copy to a run). Counters cannot be read from inside
# this process, so the figures of the last profiled build are carried here; the
# summaries, with their commands, are profiles/linear_and_conv2d_hbm_traffic_counters.md,
# written by bench_profile.py; TRAFFIC_MEASURED_AT is the commit whose kernels they
# were measured on and is reported next to every figure taken from the table.
TRAFFIC_MEASURED_AT = "3e86333"
MEASURED_TRAFFIC_BYTES = {
    # (workload, phase): (kernel, bytes)
    ("gemm", "fwd"): ("mfma_tile_kernel<LinearProblem<0,...>, 64, 128, 2, 4>", 237.3e6),      # algorithmic 151.0e6
    ("gemm", "bwd_dw"): ("linear_dw_side_kernel<LinearProblem<2,...>, 64, 128, 2, 4>", 334.7e6),  # algorithmic 213.9e6
    ("gemm", "bwd_dz"): ("mfma_tile_kernel<LinearProblem<1,...>, 64, 128, 2, 4>", 167.9e6),   # algorithmic 88.1e6
    ("skinny", "fwd"): ("gemv16_fwd_kernel<1, 4, 16>", 565.5e6),    # algorithmic 536.9e6
    ("skinny", "bwd_dz"): ("gemv_dz_kernel<2>", 286.5e6),           # algorithmic 268.4e6
    ("skinny", "bwd_dw"): ("gemv_dw_kernel<8, true>", 815.5e6),     # algorithmic 805.3e6
    ("skinny12", "bwd_dw"): ("gemv_dw_kernel<16, true>", 829.1e6),  # algorithmic 805.3e6
    ("skinny16", "bwd_dw"): ("gemv_dw_kernel<16, true>", 829.1e6),
    ("skinny12", "fwd"): ("gemv16_fwd_kernel<1, 3, 16>", 578.2e6),     # algorithmic 536.9e6
    ("skinny16", "fwd"): ("gemv16_fwd_kernel<1, 3, 16>", 578.2e6),
    ("skinny12", "bwd_dz"): ("gemv16_dz_kernel<1>", 291.4e6),          # algorithmic 268.4e6
    ("skinny16", "bwd_dz"): ("gemv16_dz_kernel<1>", 291.4e6),
    ("conv", "fwd"): ("conv_stencil_kernel<false, 32>", 169.2e6),   # algorithmic 134.2e6
}

# Conv2d 3x3, stride 1, pad 1, 64 -> 64 channels on 32x32 maps, batch 128, no bias
CONV = dict(fi=64, fo=64, k=3, stride=1, pad=1, pad_type=1, wi=32, B=128)


def make_inputs(K, N, B, device):
    """Distributions of the benchmark configuration, seed 0."""
    import torch
    g = torch.Generator(device=device)
    g.manual_seed(0)
    randn = lambda *s: torch.randn(*s, device=device, generator=g)
    rand = lambda *s: torch.rand(*s, device=device, generator=g)
    return dict(
        mu_w=randn(N, K) * K ** -0.5,
        var_w=torch.full((N, K), 1.0 / K, device=device),
        mu_b=torch.zeros(N, device=device),
        var_b=torch.full((N,), 1.0 / K, device=device),
        mu_a=randn(B, K),
        var_a=rand(B, K) * 0.09 + 0.01,
        jcb=torch.ones(B, K, device=device),
        delta_mu=randn(B, N) * 0.1,
        delta_var=-rand(B, N) * 1e-3,
    )


def warm_up(step, warmup, min_seconds=0.3):
    """`warmup` untimed steps, and more of them until the GPU has worked for
    `min_seconds`: a handful of sub-millisecond steps right after start-up would
    otherwise be timed on clocks that are still ramping."""
    import torch
    t_start = time.perf_counter()
    done = 0
    for _ in range(warmup):
        step()
    done += warmup
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < min_seconds:
        for _ in range(10):
            step()
        done += 10
        torch.cuda.synchronize()
    return dict(warmup_effective_steps=done,
                warmup_seconds=round(time.perf_counter() - t_start, 3))


def run_workload(name, steps, warmup):
    import torch
    import cutagi_amd.functional as F

    K, N, B, bound = WORKLOADS[name]
    dev = torch.device("cuda:0")
    t = make_inputs(K, N, B, dev)
    out_z = (torch.empty(B, N, device=dev), torch.empty(B, N, device=dev))
    out_dz = (torch.empty(B, K, device=dev), torch.empty(B, K, device=dev))
    out_dw = (torch.empty(N, K, device=dev), torch.empty(N, K, device=dev))
    out_db = (torch.empty(N, device=dev), torch.empty(N, device=dev))

    phases = [
        ("fwd", lambda: F.linear_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"],
                                     t["var_a"], out=out_z)),
        ("bwd_dz", lambda: F.linear_bwd_dz(t["mu_w"], t["jcb"], t["delta_mu"], t["delta_var"],
                                           out=out_dz)),
        ("bwd_dw", lambda: F.linear_bwd_dw(t["var_w"], t["mu_a"], t["delta_mu"], t["delta_var"],
                                           out=out_dw)),
        ("bwd_db", lambda: F.linear_bwd_db(t["var_b"], t["delta_mu"], t["delta_var"],
                                           out=out_db)),
    ]

    out_bwd = list(out_dz + out_dw + out_db)

    def step():
        # what one training step of the layer runs: the forward call, then the one
        # backward call that LinearCuda::backward maps to (delta_z, delta_w, delta_b)
        phases[0][1]()
        F.linear_bwd(t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"], t["delta_mu"],
                     t["delta_var"], out=out_bwd)

    warm = warm_up(step, warmup)

    # timed region: exactly `steps` steps between two synchronisations
    t0 = time.perf_counter()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = e0.elapsed_time(e1) / steps

    # second pass: per-phase durations with HIP events on the same stream
    marks = [[torch.cuda.Event(enable_timing=True) for _ in range(len(phases) + 1)]
             for _ in range(steps)]
    for s in range(steps):
        marks[s][0].record()
        for i, (_, fn) in enumerate(phases):
            fn()
            marks[s][i + 1].record()
    torch.cuda.synchronize()
    phase_ms = {}
    for i, (pname, _) in enumerate(phases):
        phase_ms[pname] = sum(m[i].elapsed_time(m[i + 1]) for m in marks) / steps

    flops = {"fwd": 6.0 * B * N * K, "bwd_dz": 4.0 * B * N * K, "bwd_dw": 4.0 * B * N * K}
    bytes_ = {"fwd": 2.0 * N * K * 4, "bwd_dz": 1.0 * N * K * 4, "bwd_dw": 3.0 * N * K * 4}
    dominant = max(flops, key=lambda p: phase_ms[p])
    if bound == "mfma":
        achieved = flops[dominant] / (phase_ms[dominant] * 1e-3) / 1e12
        roof = dict(bound="mfma", kernel=dominant, achieved=round(achieved, 2),
                    peak=FP32_MFMA_PEAK_TFLOPS, unit="TFLOP/s",
                    frac=round(achieved / FP32_MFMA_PEAK_TFLOPS, 4), traffic=None)
        value = 14.0 * B * N * K / (ms_per_step * 1e-3) / 1e12
        unit = "TFLOP/s"
        peak = FP32_MFMA_PEAK_TFLOPS
    else:
        achieved = bytes_[dominant] / (phase_ms[dominant] * 1e-3) / 1e9
        roof = dict(bound="hbm", kernel=dominant, achieved=round(achieved, 1), peak=HBM_PEAK_GBS,
                    unit="GB/s", frac=round(achieved / HBM_PEAK_GBS, 4), traffic=None)
        value = 6.0 * N * K * 4 / (ms_per_step * 1e-3) / 1e9
        unit = "GB/s"
        peak = HBM_PEAK_GBS
    if name == "gemm":
        # the timed call launches the tile kernel and, after it, the fold of its
        # reduction slices (about 9 of the 211 us); a kernel trace lists them apart
        roof["covers"] = "forward call = tile kernel + fold of its four reduction slices"
    kernel, traffic = MEASURED_TRAFFIC_BYTES.get((name, dominant), (None, None))
    roof["traffic"] = traffic
    roof["traffic_kernel"] = kernel
    roof["traffic_measured_at"] = TRAFFIC_MEASURED_AT if traffic is not None else None
    roof["kernel_ms"] = round(phase_ms[dominant], 5)
    if name.startswith("mid"):
        # both bounds are close at these batches: the step cannot be faster than the
        # slower of "all flops at the matrix peak" and "all weight bytes at the HBM peak"
        t_mfma = 14.0 * B * N * K / (FP32_MFMA_PEAK_TFLOPS * 1e12)
        t_hbm = 6.0 * N * K * 4 / (HBM_PEAK_GBS * 1e9)
        roof = dict(bound="mfma" if t_mfma >= t_hbm else "hbm", covers="whole step",
                    t_mfma_us=round(t_mfma * 1e6, 2), t_hbm_us=round(t_hbm * 1e6, 2),
                    achieved_us=round(ms_per_step * 1e3, 2),
                    frac=round(max(t_mfma, t_hbm) / (ms_per_step * 1e-3), 4), traffic=None)
    return dict(name=name, K=K, N=N, B=B, value=value, unit=unit, frac_of_peak=value / peak,
                ms_per_step=ms_per_step, wall_ms=wall_ms, phase_ms=phase_ms, roofline=roof,
                warm=warm)


def run_conv(steps, warmup):
    """Conv2d forward + backward (delta_w, delta_z) through the index tables."""
    import torch
    import cutagi_amd.functional as F
    from cutagi_amd import capi

    c = CONV
    fi, fo, k, wi, B = c["fi"], c["fo"], c["k"], c["wi"], c["B"]
    idx = capi.conv2d_build_idx(k, c["stride"], wi, wi, c["pad"], c["pad_type"], k * k * fi * fo + 1)
    wihi, woho = wi * wi, idx["wo"] * idx["ho"]
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(0)
    randn = lambda n: torch.randn(n, device=dev, generator=g)
    rand = lambda n: torch.rand(n, device=dev, generator=g)
    R = k * k * fi
    mu_w, var_w = randn(fo * R) * R ** -0.5, torch.full((fo * R,), 1.0 / R, device=dev)
    mu_a, var_a = randn(B * fi * wihi), rand(B * fi * wihi) * 0.09 + 0.01
    jcb = torch.ones(B * fi * wihi, device=dev)
    dmu, dvar = randn(B * fo * woho) * 0.1, -rand(B * fo * woho) * 1e-3
    t = {n: torch.from_numpy(idx[n]).to(dev) for n in ("Fmwa_2", "FCzwa_1", "Szz_ud")}

    def step():
        F.conv2d_fwd(mu_w, var_w, None, None, mu_a, var_a, t["Fmwa_2"], woho, fo, wihi, fi, k, B)
        # the layer's whole backward in one call, as the host class makes it
        F.conv2d_bwd(mu_w, var_w, None, mu_a, jcb, dmu, dvar, t["Fmwa_2"], t["FCzwa_1"], t["Szz_ud"],
                     B, fo, woho, wihi, fi, k, idx["h"])

    warm = warm_up(step, warmup)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    tflops = 14.0 * fo * (B * woho) * R / (ms * 1e-3) / 1e12
    # the forward kernel alone, for the roofline of the dominant kernel
    f0, f1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    f0.record()
    for _ in range(steps):
        F.conv2d_fwd(mu_w, var_w, None, None, mu_a, var_a, t["Fmwa_2"], woho, fo, wihi, fi, k, B)
    f1.record()
    torch.cuda.synchronize()
    fwd_ms = f0.elapsed_time(f1) / steps
    fwd_tflops = 6.0 * fo * (B * woho) * R / (fwd_ms * 1e-3) / 1e12
    return dict(workload="TAGI Conv2d 3x3 s1 p1, 64->64 channels, 32x32 maps, batch 128, no bias, "
                         "forward + backward (tagi_conv2d_fwd, tagi_conv2d_bwd)", value=round(tflops, 3), unit="TFLOP/s",
                frac_of_peak=round(tflops / FP32_MFMA_PEAK_TFLOPS, 4), ms_per_step=round(ms, 5),
                roofline=dict(bound="mfma", kernel="fwd", achieved=round(fwd_tflops, 2),
                              peak=FP32_MFMA_PEAK_TFLOPS, unit="TFLOP/s",
                              frac=round(fwd_tflops / FP32_MFMA_PEAK_TFLOPS, 4),
                              traffic=MEASURED_TRAFFIC_BYTES[("conv", "fwd")][1],
                              traffic_kernel=MEASURED_TRAFFIC_BYTES[("conv", "fwd")][0],
                              traffic_measured_at=TRAFFIC_MEASURED_AT,
                              kernel_ms=round(fwd_ms, 5)), steps=steps, **warm)


MLP_SPEC = "Linear 784 128 1 ReLU Linear 128 128 1 ReLU Linear 128 11 1"


def run_mlp(steps, warmup, B=32):
    """One training step of the MLP configuration (784 -> 128 -> 128 -> 11 with ReLU,
    batch 32: forward, output update on 4 selected units per sample, backward, step)
    through the host classes with host input arrays, outputs fetched: wall time per
    step. Latency-bound (a few dozen small launches), so no throughput is quoted."""
    import numpy as np
    import torch
    from cutagi_amd import cutagi

    cutagi.manual_seed(0)
    net = cutagi.Sequential([cutagi.Linear(784, 128), cutagi.ReLU(), cutagi.Linear(128, 128),
                             cutagi.ReLU(), cutagi.Linear(128, 11)])
    net.to_device("cuda")
    updater = cutagi.OutputUpdater(net.device)
    rng = np.random.default_rng(0)
    x = rng.normal(0, 1, (B, 784)).astype(np.float32)
    sel = np.concatenate([rng.choice(11, 4, replace=False) + 1 for _ in range(B)]).astype(np.int32)
    y = rng.normal(0, 1, B * 4).astype(np.float32)
    var_y = np.ones(B * 4, np.float32)

    def step():
        net.forward(x)
        mu, var = net.get_outputs()
        updater.update_using_indices(net.output_z_buffer, y, var_y, sel, net.input_delta_z_buffer)
        net.backward()
        net.step()
        return mu, var

    warm = warm_up(lambda: step(), warmup)
    n = max(steps, 200)

    def timed():
        t0 = time.perf_counter()
        for _ in range(n):
            out = step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e6 / n, out

    us, (mu, var) = timed()
    # the same step with the forward and backward launches replayed from HIP graphs
    # (Sequential.enable_graphs): reported beside the default, which is the eager path
    net.enable_graphs(True)
    for _ in range(20):
        step()
    torch.cuda.synchronize()
    us_graphs, _ = timed()
    graphs = net.graphs_captured()
    net.enable_graphs(False)
    return dict(workload="TAGI MLP 784->128->128->11 (ReLU), batch %d, one training step through "
                         "the host classes, outputs fetched" % B,
                value=round(us, 1), unit="us/step", higher_is_better=False, steps=n, **warm,
                with_hip_graph_replay=dict(value=round(us_graphs, 1), unit="us/step",
                                           graphs_replayed_per_step=graphs),
                outputs_finite_and_variances_nonnegative=bool(np.all(np.isfinite(mu))
                                                              and var.min() >= 0))


def run_resnet(steps, warmup, B=128):
    """One training step of the CIFAR ResNet-18 (forward, hierarchical-softmax output
    update, backward, parameter step) through the host classes, batch 128. Inputs
    are handed over as host arrays, as the reference's API takes them, so the
    figure includes their copy to the device."""
    import numpy as np
    import torch
    from cutagi_amd import cutagi
    from cutagi_amd.resnet import hrc_softmax, resnet18_cifar10

    cutagi.manual_seed(0)
    net = resnet18_cifar10(cutagi)
    net.to_device("cuda")
    updater = cutagi.OutputUpdater(net.device)
    obs, idx, n_obs, _ = hrc_softmax(10)
    rng = np.random.default_rng(0)
    x = rng.normal(0, 1, (B, 3 * 32 * 32)).astype(np.float32)
    labels = rng.integers(0, 10, B)
    y = np.ascontiguousarray(obs[labels].ravel(), np.float32)
    sel = np.ascontiguousarray(idx[labels].ravel(), np.int32)
    var_y = np.ones(B * n_obs, np.float32)

    def step():
        net.forward(x)
        updater.update_using_indices(net.output_z_buffer, y, var_y, sel, net.input_delta_z_buffer)
        net.backward()
        net.step()

    warm = warm_up(step, warmup)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    mu, var = net.get_outputs()
    ok = bool(np.all(np.isfinite(mu)) and var.min() >= 0)
    # Algorithmic work of the contractions only (Conv2d and Linear layers; BatchNorm,
    # activations, pooling and the update are not counted): per multiply-accumulate of a
    # layer 6 flop forward, 4 for the weight innovations and 4 for the state innovations;
    # the first layer propagates nothing to the input image (10 instead of 14).
    from cutagi_amd.resnet import resnet18_cifar10_macs
    macs = resnet18_cifar10_macs()
    flop = B * sum((14.0 if needs_dz else 10.0) * m for m, needs_dz in macs)
    tflops = flop / (ms * 1e-3) / 1e12
    return dict(workload="TAGI ResNet-18 (CIFAR: 3x32x32 input, BatchNorm, MixtureReLU, 11 "
                         "hierarchical-softmax outputs), batch %d, one training step" % B,
                value=round(B / (ms * 1e-3), 1), unit="images/s", ms_per_step=round(ms, 3),
                steps=steps,
                roofline=dict(bound="mfma", covers="whole training step (wall clock, host "
                              "input arrays): flop of the Conv2d / Linear contractions only",
                              mac_per_image=int(sum(m for m, _ in macs)), flop=flop,
                              achieved=round(tflops, 2), peak=FP32_MFMA_PEAK_TFLOPS,
                              unit="TFLOP/s", frac=round(tflops / FP32_MFMA_PEAK_TFLOPS, 4),
                              traffic=None),
                outputs_finite_and_variances_nonnegative=ok, **warm)


def calibrate_copy():
    """A plain device copy of known size (1 GiB read + 1 GiB written), so that
    hardware byte counters of a profiler run can be scaled."""
    import torch
    a = torch.empty(1 << 28, device="cuda:0")
    b = torch.empty_like(a)
    a.fill_(1.0)
    torch.cuda.synchronize()
    for _ in range(5):
        b.copy_(a)
    torch.cuda.synchronize()


def _cpu_lib():
    """The reference's own CPU kernels where their compiled library travelled with the
    tree (kind "reference"), otherwise this repository's bit-identical restatement of
    them (kind "port")."""
    import oracle
    try:
        lib = oracle.load_ref()
        if lib is not None:
            return lib, "reference"
    except OSError:
        pass
    return oracle.load(), "port"


def _cpu_threads():
    return max(1, min(16, os.cpu_count() or 1))


def cpu_baseline(name, reps=2):
    """Full steps of a Linear workload on the host cores: the reference's thread
    fan-out with 16 std::threads, and one step with its default of 4."""
    import numpy as np

    K, N, B, bound = WORKLOADS[name]
    lib, kind = _cpu_lib()
    threads = _cpu_threads()
    rng = np.random.default_rng(0)
    f = np.float32
    mu_w = (rng.standard_normal((N, K)) * K ** -0.5).astype(f)
    var_w = np.full((N, K), 1.0 / K, f)
    mu_b = np.zeros(N, f)
    var_b = np.full(N, 1.0 / K, f)
    mu_a = rng.standard_normal((B, K)).astype(f)
    var_a = rng.uniform(0.01, 0.1, (B, K)).astype(f)
    jcb = np.ones((B, K), f)
    dmu = (rng.standard_normal((B, N)) * 0.1).astype(f)
    dvar = (-rng.uniform(0, 1e-3, (B, N))).astype(f)

    def steps(n, t):
        t0 = time.perf_counter()
        for _ in range(n):
            lib.linear_fwd(mu_w, var_w, mu_b, var_b, mu_a, var_a, t)
            lib.linear_bwd_dz(mu_w, jcb, dmu, dvar, t)
            lib.linear_bwd_dw(var_w, mu_a, dmu, dvar, t)
            lib.linear_bwd_db(var_b, dmu, dvar, t)
        return (time.perf_counter() - t0) / n

    if bound == "hbm":
        figure, unit = lambda dt: round(6.0 * N * K * 4 / dt / 1e9, 3), "GB/s"
    else:
        figure, unit = lambda dt: round(14.0 * B * N * K / dt / 1e12, 5), "TFLOP/s"
    dt = steps(reps, threads)
    out = dict(value=figure(dt), unit=unit, cores=threads, kind=kind, seconds_per_step=round(dt, 3),
               sample="%d full forward+backward steps of the %s workload (K=%d, N=%d, B=%d), "
                      "reference thread fan-out with %d std::threads"
                      % (reps, name, K, N, B, threads))
    if threads > 4:
        # the reference's default thread count (include/base_layer.h:60), one step
        dt4 = steps(1, 4)
        out["reference_default_threads"] = dict(cores=4, seconds_per_step=round(dt4, 3),
                                                value=figure(dt4))
    return out


def cpu_baseline_conv():
    """One full forward + backward step of the Conv2d workload on the host cores, and
    one step at a quarter of the batch with the reference's default of 4 threads."""
    import numpy as np
    from cutagi_amd import capi

    lib, kind = _cpu_lib()
    threads = _cpu_threads()
    c = CONV
    fi, fo, k, wi = c["fi"], c["fo"], c["k"], c["wi"]
    idx = capi.conv2d_build_idx(k, c["stride"], wi, wi, c["pad"], c["pad_type"], k * k * fi * fo + 1)
    wihi, woho = wi * wi, idx["wo"] * idx["ho"]
    R = k * k * fi
    f = np.float32

    def one_step(B, t):
        rng = np.random.default_rng(0)
        mu_w = (rng.standard_normal(fo * R) * R ** -0.5).astype(f)
        var_w = np.full(fo * R, 1.0 / R, f)
        mu_a = rng.standard_normal(B * fi * wihi).astype(f)
        var_a = rng.uniform(0.01, 0.1, B * fi * wihi).astype(f)
        jcb = np.ones(B * fi * wihi, f)
        dmu = (rng.standard_normal(B * fo * woho) * 0.1).astype(f)
        dvar = (-rng.uniform(0, 1e-3, B * fo * woho)).astype(f)
        t0 = time.perf_counter()
        lib.conv2d_fwd(mu_w, var_w, None, None, mu_a, var_a, idx["Fmwa_2"], woho, fo, wihi, fi, k,
                       B, t)
        lib.conv2d_bwd_dw(var_w, None, mu_a, dmu, dvar, idx["Fmwa_2"], B, fo, woho, wihi, fi, k, t)
        lib.conv2d_bwd_dz(mu_w, jcb, dmu, dvar, idx["FCzwa_1"], idx["Szz_ud"], woho, fo, wihi, fi,
                          k, idx["h"], B, t)
        return time.perf_counter() - t0

    tf = lambda B, dt: round(14.0 * fo * (B * woho) * R / dt / 1e12, 5)
    B = c["B"]
    dt = one_step(B, threads)
    out = dict(value=tf(B, dt), unit="TFLOP/s", cores=threads, kind=kind,
               seconds_per_step=round(dt, 3),
               sample="1 full forward+backward step of the Conv2d workload (batch %d), reference "
                      "thread fan-out with %d std::threads" % (B, threads))
    if threads > 4:
        Bq = B // 4
        dt4 = one_step(Bq, 4)
        out["reference_default_threads"] = dict(
            cores=4, value=tf(Bq, dt4), seconds_per_step_at_full_batch=round(dt4 * B / Bq, 3),
            sample="1 step at batch %d (a quarter of the workload; the work is linear in the "
                   "batch)" % Bq)
    return out


def _ref_model_seconds_per_step(ref, spec, B, n_in, n_obs, n_out, steps_a, steps_b, threads):
    """Seconds per training step of the reference's own Sequential on the CPU
    (oracle/ref_model.cpp): two runs that differ in their number of steps, so that
    building the network and loading its parameters cancel."""
    import numpy as np
    rng = np.random.default_rng(0)
    sizes = ref.model_param_sizes(spec)
    params = [np.abs(rng.standard_normal(n)).astype(np.float32) * 0.05 + 1e-3 for n in sizes]

    def run(steps):
        x = rng.standard_normal((steps, B * n_in)).astype(np.float32)
        y = rng.standard_normal((steps, B * n_obs)).astype(np.float32)
        var_y = np.ones((steps, B * n_obs), np.float32)
        sel = np.stack([np.concatenate([rng.choice(n_out, n_obs, replace=False) + 1
                                        for _ in range(B)]) for _ in range(steps)]).astype(np.int32)
        t0 = time.perf_counter()
        ref.model_run(spec, params, x, None, y, var_y, sel, B, 1, n_enc=n_obs, threads=threads)
        return time.perf_counter() - t0

    ta, tb = run(steps_a), run(steps_b)
    return (tb - ta) / (steps_b - steps_a)


def cpu_baseline_mlp(B=32):
    import oracle
    ref = oracle.load_ref()
    if ref is None:
        return dict(value=None, reason="the compiled reference (oracle/_ref) is not present; "
                                       "its Sequential is what this baseline runs")
    threads = 4  # the reference's default (include/base_layer.h:60)
    dt = _ref_model_seconds_per_step(ref, MLP_SPEC, B, 784, 4, 11, 20, 120, threads)
    return dict(value=round(dt * 1e6, 1), unit="us/step", cores=threads, kind="reference",
                sample="100 training steps of the same network and batch through the reference's "
                       "Sequential / OutputUpdater on the CPU (difference of a 120- and a 20-step "
                       "run), %d std::threads" % threads)


def resnet18_spec():
    """The CIFAR ResNet-18 as the text description oracle/ref_model.cpp builds the
    reference's layers from (same architecture as cutagi_amd/resnet.py)."""
    bn = "BatchNorm2d %d 1e-5 0.9 1"

    def main(i, o, s, pt):
        return ("Conv2d %d %d 3 0 %d 1 %d 0 0 MixtureReLU " % (i, o, s, pt) + bn % o +
                " Conv2d %d %d 3 0 1 1 1 0 0 MixtureReLU " % (o, o) + bn % o)

    same = lambda c: "ResNetBlock [ " + main(c, c, 1, 1) + " ] [ ]"
    down = lambda i, o: ("ResNetBlock [ " + main(i, o, 2, 2) + " ] [ Conv2d %d %d 2 0 2 0 1 0 0 "
                         "MixtureReLU " % (i, o) + bn % o + " ]")
    return " ".join(["Conv2d 3 64 3 0 1 1 1 32 32 MixtureReLU " + bn % 64, same(64), same(64),
                     down(64, 128), same(128), down(128, 256), same(256), down(256, 512),
                     same(512), "AvgPool2d 4 -1 0 0 Linear 512 11 1"])


def cpu_baseline_resnet(B=16, full_batch=128):
    import oracle
    ref = oracle.load_ref()
    if ref is None:
        return dict(value=None, reason="the compiled reference (oracle/_ref) is not present; "
                                       "its Sequential is what this baseline runs")
    threads = _cpu_threads()
    dt = _ref_model_seconds_per_step(ref, resnet18_spec(), B, 3 * 32 * 32, 4, 11, 1, 2, threads)
    return dict(value=round(B / dt, 2), unit="images/s", cores=threads, kind="reference",
                seconds_per_step=round(dt, 3), batch=B,
                sample="1 training step of the same network at batch %d (1/%d of the workload's "
                       "%d: a full-batch step takes minutes on the CPU) through the reference's "
                       "Sequential / OutputUpdater (difference of a 2- and a 1-step run), %d "
                       "std::threads" % (B, full_batch // B, full_batch, threads))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="gemm")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--extra", default="linear,conv,resnet18,mlp",
                    help="comma-separated secondary workloads to run (linear, conv, resnet18, mlp)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run a plain 1 GiB device copy (reference for byte counters)")
    args = ap.parse_args()

    if args.workload not in ("gemm", "skinny"):
        ap.error("--workload is gemm or skinny")
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (torch.cuda.is_available() is False)", file=sys.stderr)
        sys.exit(1)

    gpu_t0 = time.perf_counter()
    from cutagi_amd import capi
    cus, clock_mhz, dev_name = capi.device_info()
    main_res = run_workload(args.workload, args.steps, args.warmup)
    line = {
        "metric": "TAGI Linear fwd+bwd TFLOP/s (% fp32 MFMA peak) 4096^2,B=256; GB/s at B=8",
        "value": round(main_res["value"], 3),
        "unit": main_res["unit"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        # what really ran before the timed region (see warm_up)
        "warmup_effective_steps": main_res["warm"]["warmup_effective_steps"],
        "warmup_seconds": main_res["warm"]["warmup_seconds"],
        "ms_per_step": round(main_res["ms_per_step"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "TAGI Linear %d->%d, batch %d, fp32, forward + backward "
                               "(delta_z, delta_w, delta_b)" % (main_res["K"], main_res["N"],
                                                                main_res["B"]),
                   "name": main_res["name"]},
        "frac_of_peak": round(main_res["frac_of_peak"], 4),
        "phase_ms": {k: round(v, 5) for k, v in main_res["phase_ms"].items()},
        "roofline": main_res["roofline"],
        # what the runtime reports for the part, and the fp32 matrix peak that follows
        # from it (compute units x 256 flop per clock x clock); `roofline.peak` is the
        # published figure
        "device": {"name": dev_name, "cus": cus, "sclk_mhz": clock_mhz,
                   "fp32_mfma_peak_from_device_tflops": round(
                       cus * FP32_MFMA_FLOP_PER_CLK_PER_CU * clock_mhz * 1e6 / 1e12, 1)},
    }
    extras = [] if args.no_extra else [e for e in args.extra.split(",") if e]
    if extras:
        line["extra"] = {}

    def linear_entry(r):
        return {"workload": "TAGI Linear %d->%d, batch %d" % (r["K"], r["N"], r["B"]),
                "value": round(r["value"], 3), "unit": r["unit"],
                "frac_of_peak": round(r["frac_of_peak"], 4),
                "ms_per_step": round(r["ms_per_step"], 5), "steps": args.steps,
                "phase_ms": {k: round(v, 5) for k, v in r["phase_ms"].items()},
                "roofline": r["roofline"], **r["warm"]}

    if "linear" in extras:
        other = "skinny" if args.workload == "gemm" else "gemm"
        line["extra"][other] = linear_entry(run_workload(other, args.steps, args.warmup))
        if args.workload == "gemm":
            for wide in ("skinny12", "skinny16"):
                line["extra"][wide] = linear_entry(run_workload(wide, args.steps, args.warmup))
            # Linear 4096^2 at batch 32 and 64, where the matrix and the memory bound meet
            line["extra"]["mid"] = {name: linear_entry(run_workload(name, args.steps, args.warmup))
                                    for name in ("mid32", "mid64")}
    if "conv" in extras:
        line["extra"]["conv"] = run_conv(max(5, args.steps // 2), args.warmup)
    if "resnet18" in extras:
        line["extra"]["resnet18"] = run_resnet(max(20, args.steps // 2), 5)
    if "mlp" in extras:
        line["extra"]["mlp"] = run_mlp(args.steps, args.warmup)
    if args.calibrate:
        calibrate_copy()
    # wall time of everything that ran on the GPU, so that the short timed regions can
    # be placed inside the whole run (the CPU baselines below take most of it)
    line["gpu_wall_s"] = round(time.perf_counter() - gpu_t0, 2)
    if not args.no_cpu:
        cpu_t0 = time.perf_counter()
        line["cpu_baseline"] = cpu_baseline(args.workload)
        ex = line.get("extra", {})
        other = "skinny" if args.workload == "gemm" else "gemm"
        if other in ex:
            ex[other]["cpu_baseline"] = cpu_baseline(other)
        if "mlp" in ex:
            ex["mlp"]["cpu_baseline"] = cpu_baseline_mlp()
        if "conv" in ex:
            ex["conv"]["cpu_baseline"] = cpu_baseline_conv()
        if "resnet18" in ex:
            ex["resnet18"]["cpu_baseline"] = cpu_baseline_resnet()
        line["cpu_wall_s"] = round(time.perf_counter() - cpu_t0, 2)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
