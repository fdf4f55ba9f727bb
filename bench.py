#!/usr/bin/env python3
"""Benchmark of the TAB hot path on one MI355X.

A step is one pass of Conv2d (quantize + bitwise conv, through the C ABI) over every layer
of the workload, inputs resident in HBM.  The headline workload is the BNN ResNet-18 layer
set at N=16; per-layer latencies, the standalone Quantize HBM rate, the large sweep point and
the CPU oracle's rate are reported in the same JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick]
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

TYPE_NAMES = {0: "TNN", 1: "TBN", 2: "BTN", 3: "BNN"}
# Matrix-core roofline of the default conv kernel: the bit planes are multiplied as FP4 (E2M1)
# operands of v_mfma_f32_32x32x64_f8f6f4; MI355X's published dense FP4 rate is 10.1 PFLOP/s, and
# one effective binary op (half a multiply-accumulate) is one such flop.
MFMA_FP4_PEAK_TOPS = 10100.0
# VALU popcount roofline, for the popcount kernel and as the yardstick the matrix-core kernel has
# to beat.  A SIMD issues one wave64 VALU instruction in `cycles`: measured on MI355X with
# tab_amd/lib/valu_peak (profiles/valu_issue_rates.txt): 2 cycles for v_xor/v_and/v_bitop3
# (128 lanes/clk/CU) and 4 cycles for v_bcnt_u32_b32 (64 lanes/clk/CU).  Per 32-bit word pair
# (= 64 binary ops per lane) the popcount kernels issue
#   BNN xor+bcnt = 6, TBN/BTN bitop3+bcnt = 6, TNN and+bcnt+bitop3+bcnt = 12 cycles.
# peak = 256 CUs x 4 SIMDs x 2.4 GHz x 64 lanes x 64 binary ops / cycles.
SIMD_HZ = 256 * 4 * 2.4e9
ISSUED_CYCLES_PER_PAIR = {0: 12, 1: 6, 2: 6, 3: 6}
# The planning figure: every op at 64 lanes/clk/CU and the reference's un-fused op mix
# (TAB_GEMM.cu:48-51,81-84,113-114,142): TNN 5, TBN 4, BTN 3, BNN 2 lane-ops per pair.
REFERENCE_MIX_OPS = {0: 5, 1: 4, 2: 3, 3: 2}
HBM_PEAK_GBS = 8000.0
STEPS_PER_GRAPH = 10  # steps captured into one HIP graph for the headline figure
HEADLINE_REPS = 7      # repetitions of the timed `steps` loop; the median is reported
# HBM bytes moved by the ten conv launches of one headline step come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE passes
# over `bench.py --profile`, scaled by a 256 MiB copy; the summary of those passes is a tracked file that states the
# figure on a line "conv_step_traffic_bytes = <n>".
TRAFFIC_PROFILE = os.path.join("profiles", "quantize_conv_profile_sequence_traffic.txt")


def profiled_figure(name):
    """(value, source) of a figure the tracked profile summary states on a line "<name> = <integer>"; (None, reason) when
    the file or the line is missing.  conv_step_traffic_bytes: measured HBM traffic of one step's conv-side launches;
    conv_step_trace_ns / step_trace_ns: sum over one step's conv-side / all launches of the average duration in the
    rocprofv3 kernel trace."""
    import re

    path = os.path.join(ROOT, TRAFFIC_PROFILE)
    try:
        for number, line in enumerate(open(path), 1):
            m = re.match(r"\s*" + name + r"\s*=\s*(\d+)", line)
            if m:
                return int(m.group(1)), f"{TRAFFIC_PROFILE}:{number}"
    except OSError:
        return None, f"{TRAFFIC_PROFILE} not found"
    return None, f"{TRAFFIC_PROFILE} has no {name} line"


def valu_peak_tops(type):
    """Roofline of the instruction mix the popcount kernel really issues, at the measured issue rates."""
    return SIMD_HZ * 64 * 64 / ISSUED_CYCLES_PER_PAIR[type] / 1e12


def planning_peak_tops(type):
    """256 CU x 64 lanes x 2.4 GHz lane-ops/s over the reference's op mix."""
    return 256 * 64 * 2.4e9 * 64 / REFERENCE_MIX_OPS[type] / 1e12


def layer_bytes(N, layer, wbits=1):
    """Algorithmic HBM bytes of one Conv2d call: X read (only the pixels a 1x1 strided conv without
    padding touches), QW read, Y written."""
    H, W, C, KN, KH, KW, p1, p2, s1, s2 = layer
    OH, OW = out_extent(H, p1, KH, s1), out_extent(W, p2, KW, s2)
    x_pixels = OH * OW if (KH, KW, p1, p2) == (1, 1, 0, 0) else H * W
    return 4 * N * x_pixels * C + 8 * KN * KH * KW * ((C + 63) // 64) * wbits + 4 * N * OH * OW * KN


def conv_kernel_bytes(N, layer, abits=1, wbits=1):
    """Algorithmic HBM bytes of the conv kernel alone: packed activation and weights read, Y written."""
    H, W, C, KN, KH, KW, p1, p2, s1, s2 = layer
    OH, OW = out_extent(H, p1, KH, s1), out_extent(W, p2, KW, s2)
    PC = (C + 63) // 64
    return 8 * N * H * W * PC * abits + 8 * KN * KH * KW * PC * wbits + 4 * N * OH * OW * KN


# (H, W, C, KN, KH, KW, pad1, pad2, stride1, stride2): ResNet-18 3x3 layers + stride-2 variants
RESNET18_LAYERS = [
    (56, 56, 64, 64, 3, 3, 1, 1, 1, 1), (28, 28, 128, 128, 3, 3, 1, 1, 1, 1),
    (14, 14, 256, 256, 3, 3, 1, 1, 1, 1), (7, 7, 512, 512, 3, 3, 1, 1, 1, 1),
    (56, 56, 64, 128, 3, 3, 1, 1, 2, 2), (28, 28, 128, 256, 3, 3, 1, 1, 2, 2),
    (14, 14, 256, 512, 3, 3, 1, 1, 2, 2), (56, 56, 64, 128, 1, 1, 0, 0, 2, 2),
    (28, 28, 128, 256, 1, 1, 0, 0, 2, 2), (14, 14, 256, 512, 1, 1, 0, 0, 2, 2),
]


# (N, layer): launches of a round or two of the chip (profiled with the counters of bench.py --profile)
MID_SIZE_LAYERS = [
    (256, (7, 7, 512, 512, 3, 3, 1, 1, 1, 1)), (256, (14, 14, 256, 256, 3, 3, 1, 1, 1, 1)),
    (32, (14, 14, 512, 512, 3, 3, 1, 1, 1, 1)),
]


def out_extent(size, pad, k, stride):
    return (size + 2 * pad - k + 1) // stride


def layer_ops(N, layer):
    H, W, C, KN, KH, KW, p1, p2, s1, s2 = layer
    OH, OW = out_extent(H, p1, KH, s1), out_extent(W, p2, KW, s2)
    return 2 * N * OH * OW * KN * KH * KW * C


def layer_name(N, layer):
    H, W, C, KN, KH, KW, p1, p2, s1, s2 = layer
    return f"N{N}_{H}x{W}x{C}->{KN}_k{KH}x{KW}_p{p1}{p2}_s{s1}{s2}"


class Layer:
    """Device-resident inputs of one Conv2d call, built as the benchmark spec says: seeded
    CPU tensors, X ~ N(0,1) NHWC, W ~ N(0,1), ternary thresholds 0.7*mean|.|, binary 0."""

    def __init__(self, tab, torch, type, N, layer, seed=0, relu=False, on_device=False):
        H, W, C, KN, KH, KW, p1, p2, s1, s2 = layer
        self.type, self.N, self.layer = type, N, layer
        abits = 2 if type < 2 else 1
        wbits = 2 if type in (0, 2) else 1
        if on_device:  # shapes too large to generate on the host in reasonable time
            g = torch.Generator("cuda").manual_seed(seed)
            x = torch.randn((N, H, W, C), generator=g, device="cuda")
            w = torch.randn((KN, KH, KW, C), generator=g, device="cuda")
        else:
            x = torch.randn((N, H, W, C), generator=torch.Generator("cpu").manual_seed(seed))
            w = torch.randn((KN, KH, KW, C), generator=torch.Generator("cpu").manual_seed(seed + 1))
        if relu:
            x = torch.relu(x)
        x_ths = 0.7 * x.abs().reshape(N, -1).mean(dim=1) if abits == 2 else torch.zeros(N)
        w_ths = 0.7 * w.abs().reshape(KN, -1).mean(dim=1) if wbits == 2 else torch.zeros(KN)
        self.host = None if on_device else (x, x_ths.float(), w, w_ths.float())
        self.x, self.x_ths = x.cuda().contiguous(), x_ths.float().cuda().contiguous()
        self.QW, self.BTN = tab.Quantize(w.cuda().contiguous(), w_ths.float().cuda().contiguous(), wbits, KN, KH, KW, C)
        self.QX, _ = tab.Quantize(self.x, self.x_ths, abits, N, H, W, C)
        self.abits, self.wbits = abits, wbits
        self.ops = layer_ops(N, layer)
        self.args = (type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW)
        self.tab = tab

    def conv2d(self):
        return self.tab.Conv2d(self.x, self.QW, self.x_ths, self.BTN, *self.args)

    def launches(self):
        """Kernels one conv2d() enqueues: 2 (quantizer, conv) or 1 (small 1x1 layers: quantize + conv in one kernel)."""
        return self.tab.conv2d_launches(self.x, *self.args)

    def conv_side_launch(self):
        """The launch of conv2d() that multiplies: the conv kernel on the packed activation, or the whole call where
        quantizer and conv are one kernel."""
        return self.conv2d() if self.launches() == 1 else self.conv_kernel_only()

    def conv_side_bytes(self):
        """Algorithmic HBM bytes of that launch: packed activation (or, in one launch with the quantizer, the fp32 pixels
        it reads) + weights + fp32 Y."""
        if self.launches() == 1:
            return layer_bytes(self.N, self.layer, self.wbits)
        return conv_kernel_bytes(self.N, self.layer, self.abits, self.wbits)

    def conv_kernel_only(self):
        return self.tab.Conv2dPacked(self.QX, self.QW, self.BTN, *self.args)

    def conv_packed_out(self):
        """Packed in, packed out (1-bit, threshold 0): what a chained binary layer runs."""
        if not hasattr(self, "out_ths"):
            self.out_ths = self.x_ths.new_zeros(self.N)
        return self.tab.Conv2dPackedOut(self.QX, self.QW, self.BTN, *self.args, self.out_ths, 1)

    def quantize_only(self):
        _, p1, p2, s1, s2, N, H, W, C, KN, KH, KW = self.args
        return self.tab.Quantize(self.x, self.x_ths, self.abits, N, H, W, C)


def event_time_ms(torch, fn, reps, warmup=3):
    """Average duration of fn() over `reps` back-to-back launches, HIP events on the current
    stream (the stream the library launches on)."""
    for _ in range(warmup):
        fn()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / reps


def graph_time_ms(torch, fn, launches, replays=5):
    """Average duration of fn() when `launches` calls are captured into one HIP graph and the
    graph is replayed: the launches run back to back on the GPU with no host work between
    them, so this is the kernel's own duration (what rocprofv3 --kernel-trace reports) plus the
    dispatch gap.  Timed with HIP events on the stream the graph is launched on."""
    fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(launches):
            fn()
    # warm up for about 20 ms of replays: the first launches after an idle gap run at a lower clock
    t0 = time.perf_counter()
    while True:
        graph.replay()
        torch.cuda.synchronize()
        if time.perf_counter() - t0 > 0.02:
            break
    samples = []
    for _ in range(3):  # median of three timed batches: single batches of a write-bound kernel scatter by 5-10 %
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(replays):
            graph.replay()
        stop.record()
        torch.cuda.synchronize()
        samples.append(start.elapsed_time(stop) / (replays * launches))
    return sorted(samples)[1]


def median_call_ms(torch, fn, reps, warmup=3):
    """Median duration of single fn() calls, each bracketed by its own pair of events."""
    for _ in range(warmup):
        fn()
    times = []
    for _ in range(reps):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        stop.record()
        stop.synchronize()
        times.append(start.elapsed_time(stop))
    return statistics.median(times)


def cpu_baseline(oracle, layers, check_against=None, budget_s=10.0):
    """The CPU oracle (this repository's C/OpenMP restatement of the reference's CPU path) over
    the same layer set and tensors, on the host cores: whole passes until about `budget_s`
    seconds of CPU work are done, after a small warm-up call."""
    import numpy as np

    l0 = layers[0]
    x, x_ths, w, w_ths = (t.numpy() for t in l0.host)
    _, p1, p2, s1, s2, N, H, W, C, KN, KH, KW = l0.args
    oracle.conv2d(x[:1], l0.QW.cpu().numpy(), x_ths[:1], l0.BTN.cpu().numpy(), l0.type, p1, p2, s1, s2, 1, H, W, C, KN, KH, KW)
    total_ops, total_s, exact, passes = 0, 0.0, True, 0
    host = [[t.numpy() for t in l.host[:2]] + [l.QW.cpu().numpy(), l.BTN.cpu().numpy()] for l in layers]
    while total_s < budget_s:
        for i, l in enumerate(layers):
            x, x_ths, qw, btn = host[i]
            t0 = time.perf_counter()
            y = oracle.conv2d(x, qw, x_ths, btn, l.type, *l.args[1:])
            total_s += time.perf_counter() - t0
            total_ops += l.ops
            if check_against is not None and passes == 0:
                exact = exact and bool(np.array_equal(y, check_against[i]))
        passes += 1
    return total_ops / total_s / 1e12, total_s, exact, passes


def sampled_images(N, rows_per_image, min_rows=4096):
    """Images whose output rows make up the correctness sample: at least `min_rows` rows (all of them when the batch
    has fewer), always the first and the last image, the rest evenly spaced."""
    k = min(N, max(2, -(-min_rows // rows_per_image)))
    if k <= 1:
        return [0]
    return sorted({round(i * (N - 1) / (k - 1)) for i in range(k)})


def gate(oracle, L, y=None):
    """Bit-exact check of a layer's GPU output against the CPU oracle on sampled images (every output row of those
    images, all KN filters, at least 4096 rows) and of the packed activation of the same images."""
    import numpy as np

    type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW = L.args
    if y is None:
        y = L.conv2d()
    OH, OW = out_extent(H, p1, KH, s1), out_extent(W, p2, KW, s2)
    images = sampled_images(N, OH * OW)
    qw, btn = L.QW.cpu().numpy(), L.BTN.cpu().numpy()
    exact = True
    for n in images:
        x, ths = L.x[n:n + 1].cpu().numpy(), L.x_ths[n:n + 1].cpu().numpy()
        want = oracle.conv2d(x, qw, ths, btn, type, p1, p2, s1, s2, 1, H, W, C, KN, KH, KW)
        exact = exact and bool(np.array_equal(y[n:n + 1].cpu().numpy(), want))
        qx, _ = oracle.quantize(x, ths, L.abits, 1, H, W, C)
        exact = exact and bool(np.array_equal(L.QX[n:n + 1].cpu().numpy(), qx))
    return {"bit_exact_vs_cpu": exact, "rows_checked": len(images) * OH * OW, "images_checked": len(images)}


def cpu_reduced_batch(oracle, L, n_small=8):
    """The CPU oracle on the first N' = min(N, 8) images of a layer, timed; the full-batch figure is the per-image time
    times N (images are independent and equally expensive), labelled extrapolated when N' < N."""
    type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW = L.args
    n = min(N, n_small)
    x, ths = L.x[:n].cpu().numpy(), L.x_ths[:n].cpu().numpy()
    qw, btn = L.QW.cpu().numpy(), L.BTN.cpu().numpy()
    oracle.conv2d(x[:1], qw, ths[:1], btn, type, p1, p2, s1, s2, 1, H, W, C, KN, KH, KW)  # warm-up
    best = None
    for _ in range(2):
        t0 = time.perf_counter()
        oracle.conv2d(x, qw, ths, btn, type, p1, p2, s1, s2, n, H, W, C, KN, KH, KW)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    return {"cpu_ms": round(best / n * N * 1e3, 2), "cpu_tops": round(L.ops / N * n / best / 1e12, 3),
            "cpu_images_timed": n, "extrapolated": n < N}


def reference_gemm_baseline(oracle, L, budget_s=3.0):
    """The reference's own BNNGEMM_baseline (TAB_CPU.cpp:312-328, compiled from the reference tree into
    oracle/_ref/libtab_ref.so) on the im2row'd rows of one layer, beside this repository's port of the same GEMM on the
    same rows and threads.  None when that library was not built."""
    import numpy as np

    if not oracle.have_ref():
        return None
    type, p1, p2, s1, s2, N, H, W, C, KN, KH, KW = L.args
    assert type == 3
    x, ths = L.host[0].numpy(), L.host[1].numpy()
    qx, _ = oracle.quantize(x, ths, 1, N, H, W, C)
    PC = (C + 63) // 64
    rows = oracle.img2row(oracle.pad(qx, N, H, W, PC, p1, p2), N, H + 2 * p1, W + 2 * p2, PC, KH, KW, s1, s2)
    M, K = rows.shape
    qw = L.QW.cpu().numpy().reshape(KN, K)
    ops = 2.0 * M * KN * K * 64
    out = {}
    for name, fn in (("reference", oracle.ref_gemm), ("port", oracle.gemm)):
        y = fn(3, rows, qw, M, KN, K, NUM=KH * KW * C)  # warm-up, and the result to compare
        out[name + "_y"] = y
        spent, reps = 0.0, 0
        while spent < budget_s / 2 and reps < 50:
            t0 = time.perf_counter()
            fn(3, rows, qw, M, KN, K, NUM=KH * KW * C)
            spent += time.perf_counter() - t0
            reps += 1
        out[name] = ops * reps / spent / 1e12
    return {"layer": layer_name(N, L.layer), "rows": int(M), "K_words": int(K),
            "reference_BNNGEMM_baseline_tops": round(out["reference"], 4), "port_gemm_tops": round(out["port"], 4),
            "threads": oracle.num_threads(), "results_equal": bool(np.array_equal(out["reference_y"], out["port_y"])),
            "note": "GEMM stage only (rows already im2row'd), the reference's scalar popcount triple loop under its own "
                    "'#pragma omp parallel for' against the port's; the reference's quantize and im2row are not timed "
                    "(TAB_CPU.cpp as a whole does not compile)"}


def profile_sequence(torch, tab):
    """Launch sequence for counter collection: a plain 256 MiB device copy (the yardstick that
    FETCH_SIZE / WRITE_SIZE are scaled with), Quantize at the roofline shape for both bit
    widths, Conv2d on every ResNet-18 N=16 layer (quantizer launch + conv launch, or the one launch that does both on
    the 1x1 layers; bracketed by two threshold launches as markers), the short-K layer
    N=256 56x56x64->64 with fp32 and with packed output, the conv kernel of three mid-size layers
    (N=256 7x7x512->512, N=256 14x14x256->256, N=32 14x14x512->512; BNN and TNN), and the conv kernel of the large
    sweep point for all four types: the default (matrix-core) kernel, then the popcount kernel on
    the same tensors.  Three repetitions each."""
    src = torch.empty(256 * 1024 * 1024 // 4, dtype=torch.float32, device="cuda").normal_()
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    del src, dst
    qN, qH, qW, qC = 256, 56, 56, 256
    xq = torch.randn((qN, qH, qW, qC), generator=torch.Generator("cuda").manual_seed(0), device="cuda")
    ths = (0.7 * xq.abs().reshape(qN, -1).mean(dim=1)).contiguous()
    zeros = torch.zeros(qN, device="cuda")
    for _ in range(3):
        tab.Quantize(xq, zeros, 1, qN, qH, qW, qC)
        tab.Quantize(xq, ths, 2, qN, qH, qW, qC)
    del xq
    layers = [Layer(tab, torch, 3, 16, l, seed=i) for i, l in enumerate(RESNET18_LAYERS)]
    marker = torch.ones(64, device="cuda")
    torch.cuda.synchronize()
    # the launches of the headline step, three times over, between two marker launches (the threshold kernels, which
    # nothing else in this sequence runs) that tell a reader of the trace where they start and end
    tab.Threshold(marker, 1, 1.0)
    for L in layers:
        for _ in range(3):
            L.conv2d()
    tab.Threshold(marker, 1, 1.0)
    del layers
    L = Layer(tab, torch, 3, 256, RESNET18_LAYERS[0], seed=0, on_device=True)
    for _ in range(3):
        L.conv_kernel_only()
    for _ in range(3):
        L.conv_packed_out()
    del L
    # mid-size launches: a grid of a round or two of the chip, where one tile's serial K loop sets the duration
    for n_batch, lay in MID_SIZE_LAYERS:
        for type in (3, 0):
            L = Layer(tab, torch, type, n_batch, lay, seed=11, on_device=True)
            for _ in range(3):
                L.conv_kernel_only()
            del L
    for type in range(4):
        L = Layer(tab, torch, type, 256, (28, 28, 512, 512, 3, 3, 1, 1, 1, 1), seed=7, on_device=True)
        for kernel in (tab.CONV_AUTO, tab.CONV_POPCOUNT):
            tab.set_conv_kernel(kernel, -1)
            for _ in range(3):
                L.conv_kernel_only()
        tab.set_conv_kernel(tab.CONV_AUTO, -1)
        del L
    torch.cuda.synchronize()
    print("profile sequence done")


def timed_steps(torch, run_steps, steps, warmup_steps, reps=HEADLINE_REPS):
    """Wall-clock seconds of `steps` steps, `reps` times over: run_steps(k) enqueues exactly k steps.  Warm-up: the
    requested steps, then at least 20 ms of further steps (the first launches after an idle gap run at a lower
    clock).  Each repetition is bracketed by a device synchronisation on both sides."""
    run_steps(max(1, warmup_steps))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.02:
        run_steps(steps)
        torch.cuda.synchronize()
    times = []
    for _ in range(reps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run_steps(steps)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    return times


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--quick", action="store_true", help="skip the large extra shapes and the CPU baseline")
    ap.add_argument("--profile", action="store_true",
                    help="run a short fixed launch sequence for rocprofv3 (kernel trace or one --pmc pass) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (images are independent; "
              "shard the batch and replicate the weights). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch

    import tab_amd as tab  # raises if the HIP library is not built: there is no fallback

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    if args.profile:
        profile_sequence(torch, tab)
        return
    N = 16
    layers = [Layer(tab, torch, 3, N, l, seed=i) for i, l in enumerate(RESNET18_LAYERS)]
    total_ops = sum(l.ops for l in layers)

    def step():
        for l in layers:
            l.conv2d()

    def median_of(times):
        return statistics.median(times)

    # eager: every call goes Python -> C ABI -> launch; host-bound for layers this small
    eager_times = timed_steps(torch, lambda k: [step() for _ in range(k)], args.steps, args.warmup, reps=3)
    # ... and through the drop-in module a user of the reference imports (pybind11, tab_amd/_C)
    import TAB_CUDA

    def step_extension():
        for l in layers:
            TAB_CUDA.Conv2d(l.x, l.QW, l.x_ths, l.BTN, *l.args)

    ext_times = timed_steps(torch, lambda k: [step_extension() for _ in range(k)], args.steps, args.warmup, reps=3)

    # headline: the same step captured into a HIP graph and replayed (the library only enqueues kernels on the
    # current stream, so a caller can capture it).  One step per graph ...
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    single_times = timed_steps(torch, lambda k: [graph.replay() for _ in range(k)], args.steps, args.warmup)
    # ... and with STEPS_PER_GRAPH steps per graph, so that the graph launch (about 6 us a replay) is paid once per
    # ten steps: a timed repetition is still exactly args.steps steps, every one of them recomputing all ten layers
    per_graph = min(STEPS_PER_GRAPH, args.steps)
    batch = torch.cuda.CUDAGraph()
    with torch.cuda.graph(batch):
        for _ in range(per_graph):
            step()

    def replay_steps(k):
        whole, rest = divmod(k, per_graph)
        for _ in range(whole):
            batch.replay()
        for _ in range(rest):
            graph.replay()

    times = timed_steps(torch, replay_steps, args.steps, args.warmup)
    elapsed = median_of(times)
    ms_per_step = elapsed / args.steps * 1e3
    value = total_ops * args.steps / elapsed / 1e12

    # the same ten layers chained the way a binary network runs them: packed in, packed out, one launch per layer
    packed_graph = torch.cuda.CUDAGraph()
    for l in layers:
        l.conv_packed_out()
    torch.cuda.synchronize()
    with torch.cuda.graph(packed_graph):
        for _ in range(per_graph):
            for l in layers:
                l.conv_packed_out()
    packed_times = timed_steps(torch, lambda k: [packed_graph.replay() for _ in range(max(1, k // per_graph))],
                               args.steps, args.warmup)
    packed_steps = max(1, args.steps // per_graph) * per_graph

    # ---- per layer: latency of the whole call, kernel-only rates -------------------------
    per_layer, conv_ops, conv_ms, step_launches = [], 0, 0.0, 0
    for l in layers:
        call_ms = graph_time_ms(torch, l.conv2d, 20)
        fused = l.launches() == 1
        k_ms = call_ms if fused else graph_time_ms(torch, l.conv_kernel_only, 20)
        q_ms = None if fused else graph_time_ms(torch, l.quantize_only, 20)
        conv_ops += l.ops
        conv_ms += k_ms
        step_launches += l.launches()
        kb = l.conv_side_bytes()
        per_layer.append({"layer": layer_name(N, l.layer), "launches": l.launches(), "latency_us": round(call_ms * 1e3, 2),
                          "conv_kernel_us": round(k_ms * 1e3, 2),
                          "quantize_kernel_us": None if fused else round(q_ms * 1e3, 2),
                          "conv_kernel_tops": round(l.ops / k_ms / 1e9, 2),
                          "frac_mfma_peak": round(l.ops / k_ms / 1e9 / MFMA_FP4_PEAK_TOPS, 4),
                          "over_valu_planning_peak": round(l.ops / k_ms / 1e9 / planning_peak_tops(3), 4),
                          "conv_kernel_hbm_floor_us": round(kb / HBM_PEAK_GBS / 1e3, 2),
                          "conv_kernel_frac_of_hbm_peak": round(kb / HBM_PEAK_GBS / 1e3 / (k_ms * 1e3), 4),
                          "hbm_floor_us": round(layer_bytes(N, l.layer) / HBM_PEAK_GBS / 1e3, 2)})
    achieved = conv_ops / conv_ms / 1e9  # TOP/s over the conv-side launches of one step, HIP events
    # the same launches with the popcount kernel, for the comparison the matrix-core kernel has to win
    tab.set_conv_kernel(tab.CONV_POPCOUNT, -1)
    popcount_ms = sum(graph_time_ms(torch, l.conv_kernel_only, 20) for l in layers)
    tab.set_conv_kernel(tab.CONV_AUTO, -1)
    # Which roof bounds these launches: arithmetic intensity (binary ops per algorithmic HBM byte) against
    # the ridge of the two published peaks.  At N=16 every layer lies below it (the fp32 Y dominates the
    # bytes), so the bound of record is HBM; the matrix-core fraction is kept beside it.
    conv_bytes = sum(l.conv_side_bytes() for l in layers)
    intensity = conv_ops / conv_bytes
    ridge = MFMA_FP4_PEAK_TOPS * 1e12 / (HBM_PEAK_GBS * 1e9)
    hbm_bound = intensity < ridge
    traffic, traffic_source = profiled_figure("conv_step_traffic_bytes")
    # Durations: the sum over the ten launches of their average duration in the rocprofv3 kernel trace of
    # `bench.py --profile` (a tracked summary, like `traffic`): launches timed back to back with HIP events overlap the
    # tail of one with the head of the next and read some 10 % shorter, so the trace is the figure of record and the live
    # HIP-event figure stands beside it.  Without the summary the live figure is all there is.
    trace_ns, trace_source = profiled_figure("conv_step_trace_ns")
    step_trace_ns, step_trace_source = profiled_figure("step_trace_ns")
    record_ms = trace_ns / 1e6 if trace_ns else conv_ms
    record_tops = conv_ops / record_ms / 1e9
    record_gbs = conv_bytes / record_ms / 1e6
    step_bytes = sum(layer_bytes(N, l.layer) for l in layers)
    fused_layers = sum(1 for l in layers if l.launches() == 1)
    roofline = {"kernel": f"the {len(layers)} conv-side launches of one step: {len(layers) - fused_layers}x conv_mfma_direct<BNN> / conv_mfma<BNN> "
                          f"and {fused_layers}x conv1x1_fused<BNN> (v_mfma_f32_32x32x64_f8f6f4, FP4 operands)",
                "bound": "hbm" if hbm_bound else "mfma",
                "achieved": round(record_gbs if hbm_bound else record_tops, 2),
                "peak": HBM_PEAK_GBS if hbm_bound else MFMA_FP4_PEAK_TOPS,
                "unit": "GB/s" if hbm_bound else "TFLOP/s",
                "frac": round(record_gbs / HBM_PEAK_GBS if hbm_bound else record_tops / MFMA_FP4_PEAK_TOPS, 4),
                "durations_from": trace_source if trace_ns else "HIP events of this run (no tracked kernel-trace figure found)",
                "sum_of_launch_durations_us": round(record_ms * 1e3, 2),
                "hip_events": {"sum_of_launch_durations_us": round(conv_ms * 1e3, 2),
                               "achieved": round(conv_bytes / conv_ms / 1e6 if hbm_bound else achieved, 2),
                               "frac": round(conv_bytes / conv_ms / 1e6 / HBM_PEAK_GBS if hbm_bound else achieved / MFMA_FP4_PEAK_TOPS, 4),
                               "note": "the same launches timed in this run: HIP events around graph replays of 20 back-to-back "
                                       "launches per layer"},
                "traffic": traffic, "traffic_source": traffic_source,
                "algorithmic_bytes": conv_bytes,
                "launches": len(layers),
                "ops_per_byte": round(intensity, 1), "ridge_ops_per_byte": round(ridge, 1),
                # the roofline the benchmark specification names for conv: VALU popcount, 256 CU x 64 lanes x 2.4 GHz over
                # the reference's two lane-ops per word pair (BNN); target: at least half of it on these layers
                "valu_popcount_roofline_of_record": {"achieved_tops": round(record_tops, 2), "peak_tops": round(planning_peak_tops(3), 1),
                                                     "frac": round(record_tops / planning_peak_tops(3), 4), "target_frac": 0.5,
                                                     "frac_hip_events": round(achieved / planning_peak_tops(3), 4),
                                                     "popcount_kernel_achieved_tops": round(conv_ops / popcount_ms / 1e9, 2)},
                "mfma": {"achieved_tops": round(record_tops, 2), "peak_tops": MFMA_FP4_PEAK_TOPS,
                         "frac": round(record_tops / MFMA_FP4_PEAK_TOPS, 4)},
                # the whole step against HBM: every launch of the ten calls (quantizers included), the bytes a call has to
                # move (fp32 X, packed weights, fp32 Y)
                "whole_step": {"launches": step_launches, "algorithmic_bytes": step_bytes,
                               "ms_per_step": round(ms_per_step, 4),
                               "achieved_GBps": round(step_bytes / ms_per_step / 1e6, 1),
                               "frac_hbm_peak": round(step_bytes / ms_per_step / 1e6 / HBM_PEAK_GBS, 4),
                               "kernel_trace_sum_us": round(step_trace_ns / 1e3, 2) if step_trace_ns else None,
                               "kernel_trace_source": step_trace_source},
                "note": "the ten conv-side launches of one step (for the three 1x1 layers quantizer and conv are one kernel and "
                        "the launch reads the fp32 pixels): achieved = their algorithmic HBM bytes / the sum of their average "
                        "durations in the rocprofv3 kernel trace named in durations_from (a separate profiler run of "
                        "`bench.py --profile`, as for traffic); hip_events = the same launches timed in this run; bound = hbm "
                        "because their ops per byte lie below the ridge of the published peaks (FP4 MFMA 10.1 PFLOP/s, one "
                        "effective binary op = one FP4 flop; HBM 8 TB/s).  At N=16 every launch is a few microseconds, launch- "
                        "and latency-bound (see resnet18_bnn_N256 and sweep_N256_28x28x512_3x3 for kernels long enough to load "
                        "the matrix cores, quantize for the HBM-bound kernel at its roofline shape); traffic = rocprofv3 "
                        "FETCH_SIZE + WRITE_SIZE of the same launches, scaled by a copy"}

    def rate(times_s, steps):
        return {"tops": round(total_ops * steps / median_of(times_s) / 1e12, 3),
                "ms_per_step": round(median_of(times_s) / steps * 1e3, 4)}

    result = {
        "metric": "tab_conv2d_effective_binary_tops", "value": round(value, 3), "unit": "TOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp4 (e2m1) x fp4 -> f32 accumulate, exact integers",
        "data": "synthetic",
        "config": {"workload": "BNN (type 3) ResNet-18 layer set, N=16: 4x 3x3 s1 + 3x 3x3 s2 + 3x 1x1 s2; "
                               "one step = Conv2d (quantize + conv) on all 10 layers; ten steps per HIP graph replay",
                   "binary_ops_per_step": total_ops, "kernel_launches_per_step": step_launches},
        "timing": {"repetitions": len(times), "value_is": "median repetition of the timed steps loop",
                   "ms_per_step_min": round(min(times) / args.steps * 1e3, 4),
                   "ms_per_step_max": round(max(times) / args.steps * 1e3, 4),
                   "warmup": f"{args.warmup} steps, then >= 20 ms of replays"},
        "eager": {**rate(eager_times, args.steps), "note": "same step launched call by call from Python through the ctypes mirror (host-bound)"},
        "eager_TAB_CUDA": {**rate(ext_times, args.steps),
                           "note": "same step call by call through the drop-in pybind11 module TAB_CUDA.Conv2d (host-bound)"},
        "one_step_per_graph": {**rate(single_times, args.steps),
                               "note": "the same steps with one graph replay per step: the graph launch adds about 6 us a step"},
        "packed_in_packed_out_N16": {**rate(packed_times, packed_steps),
                                     "note": "the same ten layers as Conv2dPackedOut (packed activation in, 1-bit packed output, "
                                             "no quantize launch, no fp32 Y): 10 launches per step, ten steps per graph"},
        "roofline": roofline, "per_layer": per_layer,
    }

    if not args.quick:
        import numpy as np

        import oracle

        # ---- correctness gate + CPU baseline of the headline workload: whole tensors, same tensors --------------
        gpu_out = [l.conv2d().cpu().numpy() for l in layers]
        tops, secs, exact, passes = cpu_baseline(oracle, layers, gpu_out)
        result["cpu_baseline"] = {"value": round(tops, 4), "unit": "TOP/s", "cores": oracle.num_threads(),
                                  "kind": "port",
                                  "sample": f"the full workload (10 layers, N=16, {total_ops:.3e} binary ops per pass), "
                                            f"{passes} passes in {secs:.2f} s: quantize + pad + im2row + popcount GEMM, "
                                            "OpenMP over rows",
                                  "gpu_bit_exact_vs_cpu": exact}
        ref = reference_gemm_baseline(oracle, layers[1])
        result["cpu_baseline"]["reference_gemm"] = ref if ref is not None else "oracle/_ref/libtab_ref.so not built: skipped"

        # ---- the single-image TNN configuration: N=1, 32x32x64 -> 64, 3x3, pad 1 ------------------------------
        L = Layer(tab, torch, 0, 1, (32, 32, 64, 64, 3, 3, 1, 1, 1, 1), seed=0)
        call_ms = graph_time_ms(torch, L.conv2d, 20)
        k_ms = graph_time_ms(torch, L.conv_kernel_only, 20)
        result["tnn_single_image_32x32x64"] = {"latency_us": round(call_ms * 1e3, 2), "conv_kernel_us": round(k_ms * 1e3, 2),
                                               "call_tops": round(L.ops / call_ms / 1e9, 2), **gate(oracle, L),
                                               **cpu_reduced_batch(oracle, L)}

        # ---- TBN and BTN on the ResNet-18 3x3 shapes, N=16, ReLU inputs (zero-heavy ternary planes) ------------
        tern = {}
        for type in (1, 2):
            rows, t_ops, t_ms, t_cpu, ok = [], 0, 0.0, 0.0, True
            for i, l in enumerate(RESNET18_LAYERS[:7]):
                L = Layer(tab, torch, type, N, l, seed=40 + i, relu=True)
                c_ms = graph_time_ms(torch, L.conv2d, 20)
                k_ms = graph_time_ms(torch, L.conv_kernel_only, 20)
                y = L.conv2d()
                want = oracle.conv2d(L.host[0].numpy(), L.QW.cpu().numpy(), L.host[1].numpy(), L.BTN.cpu().numpy(), type, *L.args[1:])
                ok = ok and bool(np.array_equal(y.cpu().numpy(), want))
                cpu = cpu_reduced_batch(oracle, L, n_small=N)
                t_ops += L.ops
                t_ms += c_ms
                t_cpu += cpu["cpu_ms"]
                rows.append({"layer": layer_name(N, l), "latency_us": round(c_ms * 1e3, 2), "conv_kernel_us": round(k_ms * 1e3, 2),
                             "conv_kernel_tops": round(L.ops / k_ms / 1e9, 1), "cpu_ms": cpu["cpu_ms"]})
                del L
            tern[TYPE_NAMES[type]] = {"call_tops": round(t_ops / t_ms / 1e9, 1), "cpu_tops": round(t_ops / t_cpu / 1e9, 3),
                                      "bit_exact_vs_cpu": ok, "checked": "every output of every layer", "layers": rows}
        result["resnet18_tbn_btn_relu_N16"] = tern

        # ---- standalone Quantize at the HBM-roofline shape -------------------------------------
        qN, qH, qW, qC = 256, 56, 56, 256
        xq = torch.randn((qN, qH, qW, qC), generator=torch.Generator("cuda").manual_seed(0), device="cuda")
        quant = {}
        for bitwidth in (1, 2):
            ths = (0.7 * xq.abs().reshape(qN, -1).mean(dim=1)).contiguous() if bitwidth == 2 else torch.zeros(qN, device="cuda")
            ms = event_time_ms(torch, lambda: tab.Quantize(xq, ths, bitwidth, qN, qH, qW, qC), 20)
            nbytes = 4 * qN * qH * qW * qC + 8 * qN * qH * qW * (qC // 64) * bitwidth + 8 * qN
            qx, btn = tab.Quantize(xq, ths, bitwidth, qN, qH, qW, qC)
            ok = True
            for n in (0, qN // 2, qN - 1):  # whole images against the CPU quantizer
                q_o, b_o = oracle.quantize(xq[n:n + 1].cpu().numpy(), ths[n:n + 1].cpu().numpy(), bitwidth, 1, qH, qW, qC)
                ok = ok and bool(np.array_equal(qx[n:n + 1].cpu().numpy(), q_o)) and int(btn[n]) == int(b_o[0])
            quant[f"bitwidth{bitwidth}"] = {"us": round(ms * 1e3, 1), "GBps": round(nbytes / ms / 1e6, 1),
                                            "frac_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                                            "bytes": nbytes, "bit_exact_vs_cpu": ok, "images_checked": 3}
            # the same values read as NCHW (256x256x56x56): the quantizer of PyTorch-layout callers
            xn = xq.view(qN, qC, qH, qW)
            ms = event_time_ms(torch, lambda: tab.QuantizeNCHW(xn, ths, bitwidth, qN, qC, qH, qW), 20)
            qn, btn_n = tab.QuantizeNCHW(xn, ths, bitwidth, qN, qC, qH, qW)
            ok = True
            for n in (0, qN // 2, qN - 1):  # whole images against the CPU quantizer's NCHW reading
                q_o, b_o = oracle.quantize_nchw(xn[n:n + 1].cpu().numpy(), ths[n:n + 1].cpu().numpy(), bitwidth, 1, qC, qH, qW)
                ok = ok and bool(np.array_equal(qn[n:n + 1].cpu().numpy(), q_o)) and int(btn_n[n]) == int(b_o[0])
            quant[f"nchw_bitwidth{bitwidth}"] = {"us": round(ms * 1e3, 1), "GBps": round(nbytes / ms / 1e6, 1),
                                                 "frac_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                                                 "bit_exact_vs_cpu": ok, "images_checked": 3}
            del qx, qn
        ms = event_time_ms(torch, lambda: tab.Threshold(xq, qN, 0.7), 20)
        quant["threshold_abs_mean"] = {"us": round(ms * 1e3, 1), "GBps": round(4 * qN * qH * qW * qC / ms / 1e6, 1),
                                       "frac_hbm_peak": round(4 * qN * qH * qW * qC / ms / 1e6 / HBM_PEAK_GBS, 4)}
        del xq
        result["quantize"] = {"shape": "256x56x56x256 fp32", "bound": "hbm", "peak_GBps": HBM_PEAK_GBS, **quant}

        # ---- the same ResNet-18 layer set at N=256 (kernels long enough not to be launch-bound)
        rn_ops, rn_ms, rn_pop_ms, rn_out_ms, rn_call_ms, rn_layers, rn_ok, rn_cpu_ms = 0, 0.0, 0.0, 0.0, 0.0, [], True, 0.0
        for i, l in enumerate(RESNET18_LAYERS):
            L = Layer(tab, torch, 3, 256, l, seed=i, on_device=True)
            k_ms = graph_time_ms(torch, L.conv_kernel_only, 10, replays=4)
            c_ms = graph_time_ms(torch, L.conv2d, 10, replays=4)
            tab.set_conv_kernel(tab.CONV_POPCOUNT, -1)
            p_ms = graph_time_ms(torch, L.conv_kernel_only, 10, replays=4)
            tab.set_conv_kernel(tab.CONV_AUTO, -1)
            o_ms = graph_time_ms(torch, L.conv_packed_out, 10, replays=4)
            g = gate(oracle, L)
            cpu = cpu_reduced_batch(oracle, L)
            rn_ok = rn_ok and g["bit_exact_vs_cpu"]
            rn_cpu_ms += cpu["cpu_ms"]
            rn_ops += L.ops
            rn_ms += k_ms
            rn_pop_ms += p_ms
            rn_out_ms += o_ms
            rn_call_ms += c_ms
            hbm_us = layer_bytes(256, l) / HBM_PEAK_GBS / 1e3
            k_hbm_us = conv_kernel_bytes(256, l) / HBM_PEAK_GBS / 1e3
            rn_layers.append({"layer": layer_name(256, l), "conv_kernel_us": round(k_ms * 1e3, 1),
                              "call_us": round(c_ms * 1e3, 1), "conv_kernel_tops": round(L.ops / k_ms / 1e9, 1),
                              "popcount_kernel_tops": round(L.ops / p_ms / 1e9, 1),
                              "packed_out_us": round(o_ms * 1e3, 1), "packed_out_tops": round(L.ops / o_ms / 1e9, 1),
                              "frac_mfma_peak": round(L.ops / k_ms / 1e9 / MFMA_FP4_PEAK_TOPS, 4),
                              "conv_kernel_frac_of_hbm_peak": round(k_hbm_us / (k_ms * 1e3), 4),
                              "hbm_floor_us": round(hbm_us, 1), "call_frac_of_hbm_floor": round(hbm_us / (c_ms * 1e3), 4),
                              "rows_checked": g["rows_checked"], "cpu_ms_extrapolated": cpu["cpu_ms"]})
            del L
        result["resnet18_bnn_N256"] = {"conv_kernel_tops": round(rn_ops / rn_ms / 1e9, 1),
                                       "popcount_kernel_tops": round(rn_ops / rn_pop_ms / 1e9, 1),
                                       "call_tops": round(rn_ops / rn_call_ms / 1e9, 1),
                                       "packed_in_packed_out_tops": round(rn_ops / rn_out_ms / 1e9, 1),
                                       "bit_exact_vs_cpu": rn_ok,
                                       "cpu_tops_extrapolated_from_8_images": round(rn_ops / rn_cpu_ms / 1e9, 3),
                                       "note": "conv_kernel = Conv2dPacked (packed in, fp32 out); call = Conv2d (fp32 in, fp32 out: "
                                               "quantize + conv); packed_in_packed_out = Conv2dPackedOut (1-bit output packed in "
                                               "the epilogue, what a chained binary layer runs); gate: every output row of "
                                               "sampled images (>= 4096 rows per layer) and their packed activation against the CPU oracle",
                                       "frac_mfma_peak": round(rn_ops / rn_ms / 1e9 / MFMA_FP4_PEAK_TOPS, 4),
                                       "over_valu_planning_peak": round(rn_ops / rn_ms / 1e9 / planning_peak_tops(3), 4),
                                       "layers": rn_layers}

        # ---- the largest sweep point, all four types (conv kernel only) --------------------
        big = (28, 28, 512, 512, 3, 3, 1, 1, 1, 1)
        sweep = {}
        for type in range(4):
            L = Layer(tab, torch, type, 256, big, seed=7, relu=(type == 1), on_device=True)
            k_ms = graph_time_ms(torch, L.conv_kernel_only, 10, replays=4)
            call_ms = graph_time_ms(torch, L.conv2d, 3, replays=3)
            tab.set_conv_kernel(tab.CONV_POPCOUNT, -1)
            p_ms = graph_time_ms(torch, L.conv_kernel_only, 10, replays=4)
            tab.set_conv_kernel(tab.CONV_AUTO, -1)
            sweep[TYPE_NAMES[type]] = {"conv_kernel_ms": round(k_ms, 3), "call_ms": round(call_ms, 3),
                                       "conv_kernel_tops": round(L.ops / k_ms / 1e9, 1),
                                       "frac_mfma_peak": round(L.ops / k_ms / 1e9 / MFMA_FP4_PEAK_TOPS, 4),
                                       "popcount_kernel_tops": round(L.ops / p_ms / 1e9, 1),
                                       "popcount_frac_valu_peak": round(L.ops / p_ms / 1e9 / valu_peak_tops(type), 4),
                                       "valu_planning_peak_tops": round(planning_peak_tops(type), 1),
                                       "over_valu_planning_peak": round(L.ops / k_ms / 1e9 / planning_peak_tops(type), 4),
                                       **gate(oracle, L), **cpu_reduced_batch(oracle, L)}
            del L
        result["sweep_N256_28x28x512_3x3"] = sweep

        # ---- more points of the large-batch sweep (the N = 64..256 benchmark configuration): conv kernel TOP/s ----
        # (C=KN, kernel, stride, pad1, pad2) at 28x28; asymmetric padding as the config asks
        points = [(256, 3, 1, 1, 0), (512, 3, 2, 1, 0), (512, 1, 1, 0, 0), (256, 1, 2, 1, 0)]
        more, more_ok = {}, True
        for n_batch in (64, 128, 256):
            for C, k, st, p1, p2 in points:
                lay = (28, 28, C, C, k, k, p1, p2, st, st)
                row = {}
                for type in range(4):
                    L = Layer(tab, torch, type, n_batch, lay, seed=3, on_device=True)
                    row[TYPE_NAMES[type]] = round(L.ops / graph_time_ms(torch, L.conv_kernel_only, 10, replays=3) / 1e9, 1)
                    more_ok = more_ok and gate(oracle, L)["bit_exact_vs_cpu"]
                    if type == 3:
                        row["cpu_BNN_tops_extrapolated"] = cpu_reduced_batch(oracle, L)["cpu_tops"]
                    del L
                more[layer_name(n_batch, lay)] = row
        more["bit_exact_vs_cpu"] = more_ok
        result["sweep_more_conv_kernel_tops"] = more

        # ---- TNN VGG-16-style stack at N=32 (the VGG benchmark configuration) ---------------------------
        vgg, vgg_ops, vgg_ms, vgg_call_ms, vgg_ok, vgg_cpu_ms = [], 0, 0.0, 0.0, True, 0.0
        for i, (hw, c) in enumerate([(224, 64), (112, 128), (56, 256), (28, 512), (14, 512)]):
            lay = (hw, hw, c, c, 3, 3, 1, 1, 1, 1)
            L = Layer(tab, torch, 0, 32, lay, seed=20 + i, on_device=True)
            k_ms = graph_time_ms(torch, L.conv_kernel_only, 3, replays=3)
            c_ms = graph_time_ms(torch, L.conv2d, 3, replays=3)
            g = gate(oracle, L)
            cpu = cpu_reduced_batch(oracle, L, n_small=4)
            vgg_ok = vgg_ok and g["bit_exact_vs_cpu"]
            vgg_cpu_ms += cpu["cpu_ms"]
            vgg_ops += L.ops
            vgg_ms += k_ms
            vgg_call_ms += c_ms
            vgg.append({"layer": layer_name(32, lay), "conv_kernel_us": round(k_ms * 1e3, 1), "call_us": round(c_ms * 1e3, 1),
                        "conv_kernel_tops": round(L.ops / k_ms / 1e9, 1),
                        "frac_mfma_peak": round(L.ops / k_ms / 1e9 / MFMA_FP4_PEAK_TOPS, 4), "rows_checked": g["rows_checked"],
                        "cpu_ms_extrapolated": cpu["cpu_ms"]})
            del L
        result["vgg16_tnn_N32"] = {"conv_kernel_tops": round(vgg_ops / vgg_ms / 1e9, 1),
                                   "frac_mfma_peak": round(vgg_ops / vgg_ms / 1e9 / MFMA_FP4_PEAK_TOPS, 4),
                                   "call_tops": round(vgg_ops / vgg_call_ms / 1e9, 1), "bit_exact_vs_cpu": vgg_ok,
                                   "cpu_tops_extrapolated_from_4_images": round(vgg_ops / vgg_cpu_ms / 1e9, 3), "layers": vgg}
        result["all_gates_bit_exact"] = bool(
            result["cpu_baseline"]["gpu_bit_exact_vs_cpu"] and result["tnn_single_image_32x32x64"]["bit_exact_vs_cpu"]
            and all(t["bit_exact_vs_cpu"] for t in tern.values()) and rn_ok and more_ok and vgg_ok
            and all(v["bit_exact_vs_cpu"] for v in sweep.values())
            and all(quant[f"{f}bitwidth{b}"]["bit_exact_vs_cpu"] for b in (1, 2) for f in ("", "nchw_")))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
