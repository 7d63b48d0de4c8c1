#!/usr/bin/env python3
"""Writes the rocprofv3 summaries under profiles/ from raw profiler output.

The raw output comes from these commands, run at the repository root on one MI355X
(every summary repeats the command it was made from; counters are collected in runs
of their own, one counter block per run):

    rocprofv3 --kernel-trace --stats --output-format csv -d gpurun_out/prof_bench -o bench -- python3 bench.py --no-cpu --extra linear,conv
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d gpurun_out/pmc_fetch -o f -- python3 bench.py --no-cpu --extra linear,conv --calibrate --steps 10
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d gpurun_out/pmc_write -o w -- python3 bench.py --no-cpu --extra linear,conv --calibrate --steps 10
    rocprofv3 --pmc SQ_INSTS_VALU_MFMA_MOPS_F32 SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CU_CYCLES SQ_WAVES SQ_WAVE_CYCLES SQ_WAIT_INST_ANY SQ_ACTIVE_INST_VMEM GRBM_GUI_ACTIVE --output-format csv -d gpurun_out/pmc_sq -o sq -- python3 bench.py --no-cpu --extra linear,conv --steps 10
    rocprofv3 --kernel-trace --stats --output-format csv -d gpurun_out/prof_resnet -o resnet -- python3 bench.py --no-cpu --extra resnet18
    rocprofv3 --kernel-trace --stats --output-format csv -d gpurun_out/prof_mlp -o mlp -- python3 bench.py --no-cpu --extra mlp

and then, anywhere the raw output and a git checkout are at hand,

    python3 bench_profile.py [--raw gpurun_out] [--out profiles] [--commit ID]

writes one markdown file per run whose output is present. Every file is stamped with
the commit the measured library was built from (`--commit`; default `git rev-parse
--short HEAD`, with "+" appended when the working tree differs from it). After the
traffic summary the script prints the entries of bench.py's MEASURED_TRAFFIC_BYTES
table, to be pasted there together with TRAFFIC_MEASURED_AT = that commit.
"""
import argparse
import collections
import csv
import glob
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.abspath(__file__))
MB = 1e6
PEAK_TFLOPS = 157.3


def short(name):
    name = re.sub(r"\(anonymous namespace\)::", "", name)
    name = re.sub(r"\(.*$", "", name)
    return name.replace("void ", "").replace("tagi::", "")


def find(raw, sub, pattern):
    hits = glob.glob(os.path.join(raw, sub, "**", pattern), recursive=True)
    return hits[0] if hits else None


def commit_stamp(given):
    if given:
        return given
    try:
        head = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], check=True,
                              capture_output=True, text=True).stdout.strip()
        dirty = subprocess.run(["git", "-C", ROOT, "status", "--porcelain", "--", "cutagi_amd",
                                "bench.py"], capture_output=True, text=True).stdout.strip()
        return head + ("+" if dirty else "")
    except Exception:
        return "unknown"


# bench.py runs its main workload (Linear 4096^2, batch 256) first and the batch-32 / 64
# workloads of the same layer later on the same tile kernels: dispatches of a kernel that
# belongs to the main workload count only up to the first skinny-batch kernel.
MAIN_ENDS_AT = ("gemv_fwd_kernel", "gemv16_fwd_kernel")


def main_workload_only(rows, name_key):
    """rows (dicts with Start_Timestamp) -> those that precede the first skinny-batch dispatch."""
    rows = sorted(rows, key=lambda r: int(r["Start_Timestamp"]))
    for i, r in enumerate(rows):
        if short(r[name_key]).startswith(MAIN_ENDS_AT):  # (a tuple of prefixes)
            return rows[:i]
    return rows


def pmc(path, main_kernels=()):
    """Per kernel: average counter values and average duration (us) over its dispatches
    (for the kernels named in main_kernels: over those of the main workload)."""
    values = collections.defaultdict(lambda: collections.defaultdict(list))
    durations = collections.defaultdict(list)
    rows = list(csv.DictReader(open(path)))
    main_ids = set(id(r) for r in main_workload_only(rows, "Kernel_Name"))
    for r in rows:
        k = short(r["Kernel_Name"])
        if k in main_kernels and id(r) not in main_ids:
            continue
        values[k][r["Counter_Name"]].append(float(r["Counter_Value"]))
        durations[k].append(int(r["End_Timestamp"]) - int(r["Start_Timestamp"]))
    avg = {k: {c: sum(v) / len(v) for c, v in cs.items()} for k, cs in values.items()}
    return avg, {k: sum(v) / len(v) / 1e3 for k, v in durations.items()}


# (kernel name as the profiler prints it, workload, algorithmic MB in + out, algorithmic flop)
K2, B2 = 4096, 256
K3, B3 = 8192, 8
CONV_ACT = 128 * 64 * 1024 * 4 / MB   # one [128][64][32x32] fp32 tensor
KERNELS = [
    ("mfma_tile_kernel<LinearProblem<0, true, true, true>, 64, 128, 2, 4>",
     "Linear 4096^2 B=256 forward", (2 * K2 * K2 + 2 * B2 * K2 + 2 * B2 * K2) * 4 / MB, 6.0 * B2 * K2 * K2),
    ("mfma_tile_kernel<LinearProblem<1, true, true, true>, 64, 128, 2, 4>",
     "Linear 4096^2 B=256 delta_z", (K2 * K2 + 2 * B2 * K2 + 3 * B2 * K2) * 4 / MB, 4.0 * B2 * K2 * K2),
    ("mfma_tile_kernel<LinearProblem<2, true, true, true>, 64, 128, 2, 4>",
     "Linear 4096^2 B=256 delta_w (called alone)", (3 * K2 * K2 + B2 * K2 + 2 * B2 * K2) * 4 / MB, 4.0 * B2 * K2 * K2),
    ("linear_dw_side_kernel<LinearProblem<2, true, true, true>, 64, 128, 2, 4>",
     "Linear 4096^2 B=256 delta_w + delta_z fold + delta_b (inside the backward call)",
     (3 * K2 * K2 + B2 * K2 + 2 * B2 * K2) * 4 / MB, 4.0 * B2 * K2 * K2),
    ("gemv16_fwd_kernel<1, 4, 16>", "Linear 8192^2 B=8 forward", 2 * K3 * K3 * 4 / MB, 6.0 * B3 * K3 * K3),
    ("gemv_dz_kernel<2>", "Linear 8192^2 B=8 delta_z", K3 * K3 * 4 / MB, 4.0 * B3 * K3 * K3),
    ("gemv_dw_kernel<8, true>", "Linear 8192^2 B=8 delta_w (+delta_b)", 3 * K3 * K3 * 4 / MB, 4.0 * B3 * K3 * K3),
    ("gemv16_fwd_kernel<1, 3, 16>", "Linear 8192^2 B=12 and B=16 forward", 2 * K3 * K3 * 4 / MB, 6.0 * 14 * K3 * K3),
    ("gemv16_dz_kernel<1>", "Linear 8192^2 B=12 and B=16 delta_z", K3 * K3 * 4 / MB, 4.0 * 14 * K3 * K3),
    ("gemv_dw_kernel<16, true>", "Linear 8192^2 B=12 and B=16 delta_w (+delta_b)", 3 * K3 * K3 * 4 / MB, 4.0 * 14 * K3 * K3),
    ("gemv16_fwd_kernel<2, 2, 8>", "Linear 4096^2 B=32 forward", 2 * K2 * K2 * 4 / MB, 6.0 * 32 * K2 * K2),
    ("conv_stencil_kernel<false, 32>", "Conv2d 3x3 64->64 @32x32 B=128 forward", 4 * CONV_ACT, 6.0 * 64 * 131072 * 576),
    ("conv_stencil_bwd_pair_kernel<32>", "Conv2d delta_z + delta_w (one launch)", 6 * CONV_ACT,
     8.0 * 64 * 131072 * 576),
]
MAIN_KERNELS = tuple(k for k, w, _, _ in KERNELS if "B=256" in w)
# bench.py's table: (workload, phase) -> kernel
_BY_WORKLOAD = {w: k for k, w, _, _ in KERNELS}
TRAFFIC_KEYS = [
    (("gemm", "fwd"), KERNELS[0][0]), (("gemm", "bwd_dw"), KERNELS[3][0]), (("gemm", "bwd_dz"), KERNELS[1][0]),
    (("skinny", "fwd"), _BY_WORKLOAD["Linear 8192^2 B=8 forward"]),
    (("skinny", "bwd_dz"), _BY_WORKLOAD["Linear 8192^2 B=8 delta_z"]),
    (("skinny", "bwd_dw"), _BY_WORKLOAD["Linear 8192^2 B=8 delta_w (+delta_b)"]),
    (("skinny12", "fwd"), _BY_WORKLOAD["Linear 8192^2 B=12 and B=16 forward"]),
    (("skinny12", "bwd_dz"), _BY_WORKLOAD["Linear 8192^2 B=12 and B=16 delta_z"]),
    (("skinny12", "bwd_dw"), _BY_WORKLOAD["Linear 8192^2 B=12 and B=16 delta_w (+delta_b)"]),
    (("conv", "fwd"), _BY_WORKLOAD["Conv2d 3x3 64->64 @32x32 B=128 forward"]),
]


def kernel_stats(raw, out, stamp):
    stats, trace = find(raw, "prof_bench", "*kernel_stats.csv"), find(raw, "prof_bench", "*kernel_trace.csv")
    if not stats or not trace:
        return
    rows = list(csv.DictReader(open(stats)))
    avg = {short(r["Name"]): float(r["AverageNs"]) / 1e3 for r in rows}
    # the kernels of the main workload: their average over that workload's dispatches only
    per_kernel = collections.defaultdict(list)
    for r in main_workload_only(list(csv.DictReader(open(trace))), "Kernel_Name"):
        per_kernel[short(r["Kernel_Name"])].append(int(r["End_Timestamp"]) - int(r["Start_Timestamp"]))
    for k in MAIN_KERNELS:
        if per_kernel.get(k):
            avg[k] = sum(per_kernel[k]) / len(per_kernel[k]) / 1e3
    with open(os.path.join(out, "linear_and_conv2d_bench_kernel_stats.md"), "w") as f:
        f.write("# Kernel durations of the default bench.py run\n\n"
                "Library built from commit `%s`. Workloads: Linear 4096->4096 batch 256, Linear 8192->8192 batch 8 (and 12, 16),\n"
                "Linear 4096->4096 batch 32 and 64, Conv2d 3x3 64->64 on 32x32 maps batch 128; forward + backward each.\n"
                "Command (one MI355X, repository root):\n\n"
                "    rocprofv3 --kernel-trace --stats --output-format csv -d gpurun_out/prof_bench -o bench -- python3 bench.py --no-cpu --extra linear,conv\n\n"
                "Summary written by `python3 bench_profile.py` from `bench_kernel_stats.csv`; this library's kernels only (microseconds):\n\n"
                "| kernel | calls | avg us | min us | max us | %% of GPU time |\n|---|---|---|---|---|---|\n" % stamp)
        for r in rows:
            if "tagi::" not in r["Name"]:
                continue
            f.write("| `%s` | %s | %.1f | %.1f | %.1f | %s |\n" % (
                short(r["Name"]), r["Calls"], float(r["AverageNs"]) / 1e3, float(r["MinNs"]) / 1e3,
                float(r["MaxNs"]) / 1e3, r["Percentage"]))
        f.write("\nWhich kernel belongs to which workload, with the algorithmic work per launch (the tile kernels of the batch-256\n"
                "workload also run the batch-64 one later in the command, which is why their averages above are lower: the rows\n"
                "below take the dispatches of the batch-256 workload only, i.e. those before the first skinny-batch kernel):\n\n"
                "| kernel | workload | GFLOP | TFLOP/s at avg | %% of %.1f | MB (inputs + outputs) | GB/s at avg |\n"
                "|---|---|---|---|---|---|---|\n" % PEAK_TFLOPS)
        for k, w, mb, fl in KERNELS:
            if k in avg:
                tf = fl / avg[k] / 1e6
                f.write("| `%s` | %s | %.2f | %.1f | %.0f %% | %.1f | %.0f |\n" % (
                    k, w, fl / 1e9, tf, tf / PEAK_TFLOPS * 100, mb, mb / avg[k] * 1e3))
        f.write("\nThe small kernels (`reduce_splits_kernel`, `reduce_store_kernel`, `bias_delta_kernel`) fold split-reduction\n"
                "partial sums and bias innovations. The Linear 4096^2 batch 32 / 64 workloads (`extra.mid` of bench.py) run their\n"
                "state and weight backward on the 32x128 / 64x128 tile kernels listed above under their own template arguments.\n")
        fk = KERNELS[0][0]
        tr = main_workload_only(list(csv.DictReader(open(trace))), "Kernel_Name")
        folds = []
        for a, b in zip(tr, tr[1:]):
            if short(a["Kernel_Name"]) == fk and short(b["Kernel_Name"]).startswith("reduce_splits_kernel<0"):
                folds.append((int(b["End_Timestamp"]) - int(b["Start_Timestamp"])) / 1e3)
        if folds and fk in avg:
            mean = sum(folds) / len(folds)
            f.write("\n`bench.py` times the forward *call* of the Linear 4096^2 workload with HIP events (`roofline.kernel_ms`): that is\n"
                    "the tile kernel above plus the fold of its four reduction slices that follows it, %.1f + %.1f = %.1f us here.\n"
                    % (avg[fk], mean, avg[fk] + mean))
    print("wrote linear_and_conv2d_bench_kernel_stats.md")


def traffic(raw, out, stamp):
    ff, wf = find(raw, "pmc_fetch", "*counter_collection.csv"), find(raw, "pmc_write", "*counter_collection.csv")
    if not ff or not wf:
        return
    fa, _ = pmc(ff, MAIN_KERNELS)
    wa, _ = pmc(wf, MAIN_KERNELS)
    ck = [k for k in fa if "copyBuffer" in k][0]
    fs, ws = 1048576.0 / fa[ck]["FETCH_SIZE"], 1048576.0 / wa[ck]["WRITE_SIZE"]
    with open(os.path.join(out, "linear_and_conv2d_hbm_traffic_counters.md"), "w") as f:
        f.write("# HBM traffic per launch (FETCH_SIZE / WRITE_SIZE), all bench.py kernels\n\n"
                "Library built from commit `%s`. Commands (one MI355X, repository root; one counter per run):\n\n"
                "    rocprofv3 --pmc FETCH_SIZE --output-format csv -d gpurun_out/pmc_fetch -o f -- python3 bench.py --no-cpu --extra linear,conv --calibrate --steps 10\n"
                "    rocprofv3 --pmc WRITE_SIZE --output-format csv -d gpurun_out/pmc_write -o w -- python3 bench.py --no-cpu --extra linear,conv --calibrate --steps 10\n\n"
                "Summary written by `python3 bench_profile.py`. Calibration: `bench.py --calibrate` runs a plain 1 GiB device-to-device\n"
                "copy (`%s`, 1048576 KiB read and 1048576 KiB written). For it the counters read FETCH_SIZE = %.1f KiB and\n"
                "WRITE_SIZE = %.1f KiB per dispatch, so the scale factors are **FETCH x %.3f** and **WRITE x %.3f**.\n\n"
                "| kernel | workload | raw FETCH KiB | raw WRITE KiB | scaled traffic MB (read + write) | algorithmic MB (inputs + outputs) | ratio |\n"
                "|---|---|---|---|---|---|---|\n"
                % (stamp, ck.split("<")[0], fa[ck]["FETCH_SIZE"], wa[ck]["WRITE_SIZE"], fs, ws))
        measured = {}
        for k, w, mb, _ in KERNELS:
            if k not in fa or k not in wa:
                continue
            rd = fa[k]["FETCH_SIZE"] * fs * 1024 / MB
            wr = wa[k]["WRITE_SIZE"] * ws * 1024 / MB
            measured[k] = (rd + wr, mb)
            f.write("| `%s` | %s | %.0f | %.0f | %.1f + %.1f = %.1f | %.1f | %.2f |\n" % (
                k, w, fa[k]["FETCH_SIZE"], wa[k]["WRITE_SIZE"], rd, wr, rd + wr, mb, (rd + wr) / mb))
        f.write("\nReading: the skinny-batch kernels move 1.01-1.09x their algorithmic bytes (the excess is the staged\n"
                "activations / innovations and the partial sums). The tiled Linear kernels fetch the weights once (the row tiles\n"
                "that share a weight tile run on one XCD), the small operand (8.4 MB) once per XCD (the eight L2s do not share)\n"
                "and write 33.6 MB of split-reduction partial sums where their reduction is sliced. They are MFMA-bound, so this\n"
                "does not set their time. The Conv2d weight backward reads its innovations once per column tile of the weight\n"
                "matrix (9 tiles): most of that is served by the memory-side cache.\n")
    print("wrote linear_and_conv2d_hbm_traffic_counters.md")
    print("\nbench.py: TRAFFIC_MEASURED_AT = \"%s\"; MEASURED_TRAFFIC_BYTES entries:" % stamp)
    for key, k in TRAFFIC_KEYS:
        if k in measured:
            print("    %r: (%r, %.1fe6),  # algorithmic %.1fe6" % (key, k, measured[k][0], measured[k][1]))


def mfma(raw, out, stamp):
    sf = find(raw, "pmc_sq", "*counter_collection.csv")
    if not sf:
        return
    sa, sd = pmc(sf, MAIN_KERNELS)
    with open(os.path.join(out, "linear_and_conv2d_mfma_utilisation_counters.md"), "w") as f:
        f.write("# MFMA utilisation counters, all bench.py kernels\n\n"
                "Library built from commit `%s`. Command (one MI355X, repository root):\n\n"
                "    rocprofv3 --pmc SQ_INSTS_VALU_MFMA_MOPS_F32 SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CU_CYCLES SQ_WAVES SQ_WAVE_CYCLES SQ_WAIT_INST_ANY SQ_ACTIVE_INST_VMEM GRBM_GUI_ACTIVE --output-format csv -d gpurun_out/pmc_sq -o sq -- python3 bench.py --no-cpu --extra linear,conv --steps 10\n\n"
                "Summary written by `python3 bench_profile.py`; per dispatch averages. `MFMA GFLOP (counter)` =\n"
                "SQ_INSTS_VALU_MFMA_MOPS_F32 x 512, which equals the algorithmic flop count of every kernel (no wasted MFMA work).\n"
                "`MFMA busy` = SQ_VALU_MFMA_BUSY_CYCLES / (GRBM_GUI_ACTIVE x 128); the divisor 128 is empirical: with it the busy\n"
                "fraction agrees with the flop-based utilisation (TFLOP/s over the %.1f peak, where the clock is the 2.4 GHz of the\n"
                "peak figure) within a few points on every MFMA kernel below. `TFLOP/s` = algorithmic flop / duration under the profiler.\n\n"
                "| kernel | workload | us | MFMA GFLOP (counter) | algorithmic GFLOP | TFLOP/s | %% of %.1f | MFMA busy | waves | wait-any / wave-cycles |\n"
                "|---|---|---|---|---|---|---|---|---|---|\n" % (stamp, PEAK_TFLOPS, PEAK_TFLOPS))
        for k, w, _, fl in KERNELS:
            if k not in sa:
                continue
            c = sa[k]
            busy = c["SQ_VALU_MFMA_BUSY_CYCLES"] / (c["GRBM_GUI_ACTIVE"] * 128) if c.get("GRBM_GUI_ACTIVE") else 0
            tf = fl / sd[k] / 1e6
            f.write("| `%s` | %s | %.1f | %.2f | %.2f | %.1f | %.1f %% | %.1f %% | %d | %.2f |\n" % (
                k, w, sd[k], c["SQ_INSTS_VALU_MFMA_MOPS_F32"] * 512 / 1e9, fl / 1e9, tf, tf / PEAK_TFLOPS * 100,
                busy * 100, c["SQ_WAVES"], c["SQ_WAIT_INST_ANY"] / c["SQ_WAVE_CYCLES"]))
        f.write("\nThe skinny-batch forward and delta_z kernels use the MFMA only as a streaming dot-product unit; they are\n"
                "bound by HBM, and their MFMA figures are listed for completeness.\n")
    print("wrote linear_and_conv2d_mfma_utilisation_counters.md")


def resnet(raw, out, stamp):
    tf = find(raw, "prof_resnet", "*kernel_trace.csv")
    if not tf:
        return
    tr = sorted(csv.DictReader(open(tf)), key=lambda r: int(r["Start_Timestamp"]))
    first = next(i for i, r in enumerate(tr) if "conv" in r["Kernel_Name"].lower())
    tr = tr[first:]
    agg = collections.defaultdict(list)
    for r in tr:
        agg[short(r["Kernel_Name"])].append(int(r["End_Timestamp"]) - int(r["Start_Timestamp"]))
    steps = len(agg["avgpool_fwd_kernel"])
    total = sum(sum(v) for v in agg.values())
    groups = collections.OrderedDict([
        ("Conv2d, regular-stencil kernels, 3x3 stride 1", lambda k: k.startswith("conv_stencil") and "_s2_" not in k),
        ("Conv2d, regular-stencil kernels, stride 2 (3x3 and the 2x2 projections)", lambda k: k.startswith("conv_stencil_s2")),
        ("Conv2d, table-driven tile kernels (the 3-channel stem)", lambda k: k.startswith("mfma_tile_kernel<Conv")),
        ("BatchNorm2d passes", lambda k: k.startswith("bn_")),
        ("folds of sliced reductions", lambda k: k.startswith("reduce_")),
    ])
    with open(os.path.join(out, "resnet18_cifar_step_kernel_stats.md"), "w") as f:
        f.write("# Kernel durations of one ResNet-18 (CIFAR, batch 128) training step\n\n"
                "Library built from commit `%s`. Command (one MI355X, repository root):\n\n"
                "    rocprofv3 --kernel-trace --stats --output-format csv -d gpurun_out/prof_resnet -o resnet -- python3 bench.py --no-cpu --extra resnet18\n\n"
                "Summary written by `python3 bench_profile.py` from `resnet_kernel_trace.csv`: the dispatches from the first conv\n"
                "kernel on (the main Linear workload of the same command runs before it), %d training steps (warm-up included).\n"
                "Kernel time %.1f ms = **%.2f ms per step** (the step is GPU-bound: bench.py measures the same per step without\n"
                "the profiler).\n\n| group | ms per step | %% of kernel time |\n|---|---|---|\n"
                % (stamp, steps, total / 1e6, total / 1e6 / steps))
        rest = total
        for name, pred in groups.items():
            t = sum(sum(v) for k, v in agg.items() if pred(k))
            rest -= t
            f.write("| %s | %.3f | %.1f |\n" % (name, t / 1e6 / steps, t / total * 100))
        f.write("| everything else (residual / pooling / Linear head / update / transfers) | %.3f | %.1f |\n\n"
                % (rest / 1e6 / steps, rest / total * 100))
        f.write("| kernel | calls per step | avg us | ms per step | % of kernel time |\n|---|---|---|---|---|\n")
        for k, v in sorted(agg.items(), key=lambda kv: -sum(kv[1]))[:46]:
            f.write("| `%s` | %.1f | %.1f | %.3f | %.1f |\n" % (
                k[:100], len(v) / steps, sum(v) / len(v) / 1e3, sum(v) / 1e6 / steps, sum(v) / total * 100))
    print("wrote resnet18_cifar_step_kernel_stats.md")


def mlp(raw, out, stamp):
    tf = find(raw, "prof_mlp", "*kernel_trace.csv")
    if not tf:
        return
    tr = sorted(csv.DictReader(open(tf)), key=lambda r: int(r["Start_Timestamp"]))
    first = next(i for i, r in enumerate(tr) if "upload_input_kernel" in r["Kernel_Name"])
    tr = tr[first:]
    agg = collections.defaultdict(list)
    order = []
    for r in tr:
        k = short(r["Kernel_Name"]) + " [grid %s]" % r.get("Grid_Size_X", r.get("Grid_Size", "?"))
        if k not in agg:
            order.append(k)
        agg[k].append(int(r["End_Timestamp"]) - int(r["Start_Timestamp"]))
    steps = len(next(v for k, v in agg.items() if k.startswith("out_update_indexed_reset_kernel")))
    per_step = sum(sum(v) for v in agg.values() if len(v) >= steps // 2) / steps / 1e3
    with open(os.path.join(out, "mlp_784_128_128_11_step_kernel_stats.md"), "w") as f:
        f.write("# Kernels of one training step of the 784-128-128-11 perceptron (batch 32)\n\n"
                "Library built from commit `%s`. Command (one MI355X, repository root):\n\n"
                "    rocprofv3 --kernel-trace --stats --output-format csv -d gpurun_out/prof_mlp -o mlp -- python3 bench.py --no-cpu --extra mlp\n\n"
                "Summary written by `python3 bench_profile.py` from `mlp_kernel_trace.csv`: the dispatches from the first input\n"
                "upload on, %d training steps (warm-up and the HIP-graph replay leg of the same command included; both launch the\n"
                "same kernels). One step = forward, outputs to the host, output update on 4 selected units per sample, backward,\n"
                "parameter update: **%d launches, %.1f us of kernel time** (bench.py measures the wall time of the step, which adds\n"
                "the gaps between dependent launches and the host's turn-around after it has read the outputs).\n\n"
                "| kernel, in launch order | launches per step | avg us | min us |\n|---|---|---|---|\n"
                % (stamp, steps, sum(1 for k in order if len(agg[k]) >= steps // 2 for _ in range(round(len(agg[k]) / steps))),
                   per_step))
        for k in order:
            v = agg[k]
            if len(v) < steps // 2:
                continue
            f.write("| `%s` | %.1f | %.1f | %.1f |\n" % (k[:110], len(v) / steps, sum(v) / len(v) / 1e3, min(v) / 1e3))
    print("wrote mlp_784_128_128_11_step_kernel_stats.md")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--raw", default=os.path.join(ROOT, "gpurun_out"))
    ap.add_argument("--out", default=os.path.join(ROOT, "profiles"))
    ap.add_argument("--commit", default=None)
    args = ap.parse_args()
    os.makedirs(args.out, exist_ok=True)
    stamp = commit_stamp(args.commit)
    kernel_stats(args.raw, args.out, stamp)
    traffic(args.raw, args.out, stamp)
    mfma(args.raw, args.out, stamp)
    resnet(args.raw, args.out, stamp)
    mlp(args.raw, args.out, stamp)


if __name__ == "__main__":
    main()
