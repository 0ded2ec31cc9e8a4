#!/usr/bin/env python3
"""Benchmark of the SOFIE hot path on one MI355X.

Headline workload (the configuration the metric is quoted on): standalone int8 GEMM with QLinearMatMul
semantics, M=N=K=4096, A and B int8 uniform in [-127,127], per-output-channel fp32 scales
uniform in [1e-3,1e-2], int32 accumulate, round-half-to-even requantise to int8. One "step"
is one call of sofie_hip_qgemm_s8 on device-resident operands (one kernel launch). Prints ONE JSON line; next to the
headline value it carries every other configuration of the benchmark:
  fp8_gemm          e4m3 GEMM 8192x8192x4096, bf16 out + bias, TFLOP/s and fraction of the FP8 MFMA peak
  model_inferences  the generated int8 CNN Session at batch 4096, inferences per second
  mlp_f32           the generated fp32 MLP Session (64 -> 128 -> 64 -> 8, batch 256)
  gemm_f32          the reference's Gemm operator at 4096^3 in fp32 (bias row + ReLU), B [K,N] and [N,K]
  conv_f32/conv_s8  the 256 x 64 -> 128 x 56 x 56 3x3 layer in fp32 and int8
  cpu_fp32          the reference's emitted CPU call sequence for the MLP and the convolution layer
                    (oracle/cpu_emitted_bench.c) with sgemm_ from the best BLAS found on the box, at one thread and
                    at the box's core share

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]
"""
import argparse
import glob
import importlib.util
import json
import os
import statistics
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0     # MI355X dense int8 MFMA, 5.0 POP/s
PEAK_FP8_TFLOPS = 5000.0
PEAK_FP32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
# HBM-side bytes of one call of the headline entry point (one GEMM kernel). Not measurable inside this process: the
# figure comes from two rocprofv3 --pmc runs of `bench.py --traffic-probe` (FETCH_SIZE, then WRITE_SIZE), each scaled
# by what the same counter reads for a 64 MiB + 64 MiB copy-like kernel in the same run; the summary is in
# profiles/int8_gemm_4096_k_gemm_dma.md. Algorithmic bytes: 50.3 MB.
TRAFFIC_BYTES_PER_CALL = 112.3 * 1024 * 1024
ALGORITHMIC_BYTES_PER_CALL = 3 * 4096 * 4096 + 4 * 4096


def host_threads():
    """Threads the CPU legs may use: the box's share of cores (OMP_NUM_THREADS is set to it there), at most 16."""
    try:
        n = int(os.environ.get("OMP_NUM_THREADS", "0"))
    except ValueError:
        n = 0
    if n <= 0:
        n = os.cpu_count() or 1
    return max(1, min(n, 16))


def cpu_baseline_int8(A, B, scale, rows, threads):
    """The oracle (a scalar C port of the same arithmetic) on the first `rows` rows of A, cut into one block of rows
    per thread (ctypes releases the interpreter lock during the call)."""
    from oracle import oracle
    rows = min(rows, A.shape[0])
    blocks = [(i * rows // threads, (i + 1) * rows // threads) for i in range(threads)]
    t0 = time.perf_counter()
    with ThreadPoolExecutor(threads) as pool:
        parts = list(pool.map(lambda b: oracle.qgemm_s8(A[b[0]:b[1]], B, scale), blocks))
    dt = time.perf_counter() - t0
    ops = 2.0 * rows * B.shape[0] * B.shape[1]
    return np.concatenate(parts), {
        "value": ops / dt / 1e12, "unit": "TOPS", "cores": threads, "kind": "port",
        "sample": "oracle/sofie_oracle.c or_qgemm_s8 on the first %d of %d rows of A against the full B (%.1f GOP, %.1f s, "
                  "gcc -O2, %d threads, one block of rows each)" % (rows, A.shape[0], ops / 1e9, dt, threads)}


class LaunchTimer:
    """Durations on the stream the kernels are launched on, from HIP events recorded into that stream between blocks
    of back-to-back launches (no host synchronisation inside the timed region)."""

    def __init__(self, torch, stream):
        self.torch, self.stream = torch, stream

    def blocks(self, fn, n_blocks, per_block, warmup):
        torch = self.torch
        for _ in range(warmup):
            fn()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(n_blocks + 1)]
        ev[0].record(self.stream)
        for b in range(n_blocks):
            for _ in range(per_block):
                fn()
            ev[b + 1].record(self.stream)
        self.stream.synchronize()
        return [ev[b].elapsed_time(ev[b + 1]) / per_block for b in range(n_blocks)]

    def median_ms(self, fn, launches, warmup=3, per_block=None):
        per_block = per_block or max(1, min(10, launches // 5))
        n_blocks = max(1, launches // per_block)
        t = self.blocks(fn, n_blocks, per_block, warmup)
        return statistics.median(t), min(t), n_blocks * per_block


def sclk_under_load(torch, launch, stream, seconds=1.5):
    """Shader clock (MHz) that rocm-smi reports while `launch` runs back to back, and the duration of a launch
    measured over the same launches (HIP events on the launch stream around each block of 100): the medians of both
    (None for the clock if the tool is not there). The matrix peaks of the data sheet assume 2400 MHz."""
    import re
    import threading
    samples, stop = [], [False]

    def sampler():
        while not stop[0]:
            try:
                txt = subprocess.run(["rocm-smi", "--showclocks"], stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True,
                                     timeout=10).stdout
                m = re.search(r"sclk clock level:\s*\d+:\s*\((\d+)Mhz\)", txt)
                if m:
                    samples.append(int(m.group(1)))
            except Exception:
                return
    th = threading.Thread(target=sampler)
    th.start()
    t0 = time.perf_counter()
    blocks = []
    while time.perf_counter() - t0 < seconds:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(100):
            launch()
        e1.record(stream)
        torch.cuda.synchronize()
        blocks.append(e0.elapsed_time(e1) / 100)
    stop[0] = True
    th.join()
    ms = statistics.median(blocks[1:]) if len(blocks) > 1 else None
    return (statistics.median(samples[1:]) if len(samples) > 1 else None), ms


def blas_candidates():
    """(path, symbol prefix, name) in the order the baseline prefers them: MKL, OpenBLAS, scipy's OpenBLAS."""
    out = []
    for p in ("/opt/conda/lib/libmkl_rt.so.2", "/opt/conda/lib/libmkl_rt.so.1", "/opt/conda/lib/libmkl_rt.so",
              "/usr/lib/x86_64-linux-gnu/libmkl_rt.so"):
        if os.path.exists(p):
            out.append((p, "", "MKL (%s)" % p))
            break
    for p in ("/usr/lib/x86_64-linux-gnu/libopenblas.so.0", "/opt/conda/lib/libopenblas.so.0", "/opt/conda/lib/libopenblas.so"):
        if os.path.exists(p):
            out.append((p, "", "OpenBLAS (%s)" % p))
            break
    spec = importlib.util.find_spec("scipy")
    if spec is not None and spec.origin:
        hits = sorted(glob.glob(os.path.join(os.path.dirname(os.path.dirname(spec.origin)), "scipy.libs",
                                             "libscipy_openblas-*.so")))
        if hits:
            out.append((hits[0], "scipy_", "scipy's OpenBLAS (%s)" % os.path.basename(hits[0])))
    return out


def cpu_emitted(workload, threads, blas, extra=()):
    """One run of oracle/cpu_emitted_bench as a child process with the thread count in its environment."""
    exe = os.path.join(ROOT, "oracle", "cpu_emitted_bench")
    if not os.path.exists(exe):
        return None
    env = dict(os.environ)
    for k in ("OMP_NUM_THREADS", "MKL_NUM_THREADS", "OPENBLAS_NUM_THREADS"):
        env[k] = str(threads)
    env["MKL_DYNAMIC"] = "FALSE"
    cmd = [exe, "--workload", workload] + list(extra)
    if blas:
        cmd += ["--blas", blas[0], "--prefix", blas[1]]
    try:
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=env, timeout=240)
    except subprocess.TimeoutExpired:
        return None
    if res.returncode != 0:
        return None
    out = json.loads(res.stdout.strip().splitlines()[-1])
    return out if out["selfcheck"] <= 1e-3 else None


def generated_host_session(name, weights, x, threads, blas, iters):
    """The model's Session generated as code for the host cores (Options::kHostCode: the reference's own emission, BLAS
    calls and loops) and compiled ahead of the run (sofie_amd/generated/host/run_host_<name>), timed on `threads`
    threads of the BLAS library: wall time of Session::infer on a host tensor, median over `iters` calls after one."""
    exe = os.path.join(ROOT, "sofie_amd", "generated", "host", "run_host_" + name)
    dat = os.path.join(ROOT, "sofie_amd", "generated", weights + ".dat")
    if not os.path.exists(exe) or not os.path.exists(dat):
        return None
    env = dict(os.environ)
    for k in ("OMP_NUM_THREADS", "MKL_NUM_THREADS", "OPENBLAS_NUM_THREADS"):
        env[k] = str(threads)
    env["MKL_DYNAMIC"] = "FALSE"
    env.pop("SOFIE_BLAS", None)
    env.pop("SOFIE_BLAS_PREFIX", None)
    if blas:
        env["SOFIE_BLAS"], env["SOFIE_BLAS_PREFIX"] = blas[0], blas[1]
    with tempfile.TemporaryDirectory() as tmp:
        fin, fout = os.path.join(tmp, "in.bin"), os.path.join(tmp, "out.bin")
        np.ascontiguousarray(x, np.float32).tofile(fin)
        try:
            res = subprocess.run([exe, dat, fin, fout, str(iters)], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                                 env=env, timeout=240)
        except subprocess.TimeoutExpired:
            return None
        if res.returncode != 0:
            return None
        t = json.loads(res.stdout.strip().splitlines()[-1])
        return {"median_ms": t["host_ms"], "best_ms": t["best_ms"], "calls": iters, "cores": threads,
                "checksum": float(np.fromfile(fout, np.float32).astype(np.float64).sum())}


def cpu_fp32_baselines(threads, conv_images=64):
    """The reference's emitted CPU sequence (bias copy + sgemm_ + ReLU; weight re-layout + Im2col + sgemm_ + saxpy_ +
    Relu) on the host cores: first BLAS that binds and passes the self-check, at 1 thread and at `threads`."""
    chosen = None
    for cand in blas_candidates() + [None]:
        probe = cpu_emitted("mlp", 1, cand, ("--calls", "20"))
        if probe is not None:
            chosen = cand
            break
    name = chosen[2] if chosen else "none found: the bundled loops of oracle/cpu_emitted_bench.c"
    res = {"kind": "reference's emitted call sequence restated in C (oracle/cpu_emitted_bench.c), gcc -O2", "blas": name,
           "host_cpus_visible": os.cpu_count(), "threads_used": sorted({1, threads})}
    flops_conv = 2.0 * conv_images * 128 * 3136 * 576
    for t in sorted({1, threads}):
        m = cpu_emitted("mlp", t, chosen, ("--calls", "200"))
        c = cpu_emitted("conv", t, chosen, ("--images", str(conv_images), "--calls", "3"))
        gemm_rows = 256 if t == 1 else 2048
        gm = cpu_emitted("gemm", t, chosen, ("--images", str(gemm_rows), "--calls", "3"))
        if gm:
            res["gemm_4096_%dthr" % t] = {
                "median_ms": gm["median_ms"], "best_ms": gm["best_ms"], "gflops": 2.0 * gemm_rows * 4096 * 4096 / gm["median_ms"] / 1e6,
                "cores": t, "calls": gm["calls"],
                "sample": "%d of the 4096 rows of the product (rows are independent; %.1f GFLOP per call)"
                          % (gemm_rows, 2.0 * gemm_rows * 4096 * 4096 / 1e9)}
        g8 = cpu_emitted("gemm", t, chosen, ("--images", "8", "--calls", "20"))
        if g8:
            res["gemm_4096_batch8_%dthr" % t] = {
                "median_ms": g8["median_ms"], "best_ms": g8["best_ms"], "gbs": 4.0 * 4096 * 4096 / g8["median_ms"] / 1e6,
                "cores": t, "calls": g8["calls"], "sample": "the whole 8 x 4096 x 4096 product (sgemm_ on 8 rows)"}
        if m:
            res["mlp_b256_%dthr" % t] = {"median_us": m["median_ms"] * 1e3, "best_us": m["best_ms"] * 1e3,
                                         "inferences_per_s": 256 / (m["median_ms"] * 1e-3), "cores": t, "calls": m["calls"]}
        hs = generated_host_session("mlp_c1", "mlp_c1", np.random.default_rng(3).standard_normal((256, 64)).astype(np.float32), t, chosen, 200)
        if hs:
            res["mlp_b256_generated_host_session_%dthr" % t] = {
                "median_us": hs["median_ms"] * 1e3, "best_us": hs["best_ms"] * 1e3, "inferences_per_s": 256 / (hs["median_ms"] * 1e-3),
                "cores": t, "calls": hs["calls"],
                "what": "the MLP's Session generated with Options::kHostCode (this build's emission of the reference's CPU "
                        "path), g++ -O2, Session::infer on a host tensor"}
        if c:
            res["conv_64to128_56x56_%dthr" % t] = {
                "median_ms": c["median_ms"], "best_ms": c["best_ms"], "gflops": flops_conv / c["median_ms"] / 1e6,
                "cores": t, "calls": c["calls"],
                "sample": "%d of the 256 images of the layer (per-image work is independent; %.1f GFLOP per call)"
                          % (conv_images, flops_conv / 1e9)}
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # the device leaves its idle clocks over the first few hundred launches (20 ms): with 20 warm-up steps the timed
    # steps average 68.7 us, with 300 they run at the 61.5 us of the kernel itself
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=300)
    ap.add_argument("--spin-up-ms", type=float, default=60.0,
                    help="run the step back to back for this long before the warm-up steps, whatever their number: a "
                         "device that has been idle (the operands were just uploaded) starts at its idle clocks")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--cpu-rows", type=int, default=0, help="rows of A the int8 CPU baseline evaluates (default: 256 per thread)")
    ap.add_argument("--cpu-images", type=int, default=256, help="images of the CNN batch the CPU baseline leg evaluates")
    ap.add_argument("--extras", action="store_true", help="accepted for compatibility: every configuration is in the default line")
    ap.add_argument("--clock-probe", action="store_true",
                    help="also time the headline launch on all-zero operands and sample the shader clock under it "
                         "(roofline.clock.all_zero_operands)")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="launch a 64 MiB copy-like kernel and the headline call three times and exit (the target of the "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs)")
    ap.add_argument("--kernel-probe", default="",
                    help="launch one named workload a few times and exit (target of rocprofv3 runs): gemm_s8, gemm_s8_nk, "
                         "gemm_fp8, gemm_fp8_nk, gemm_f32, gemm_f32_nk, gemm_f32_batch8, gemm_s8_batch8, conv_s8, conv_f32, conv_f32_batch1, conv_transpose_f32")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus %d is not supported (no collective, no sharding "
                 "code exists). Run with --gpus 1." % args.gpus)

    import torch
    from sofie_amd import lib as L
    from sofie_amd import ops
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible (the HIP library has no CPU fallback)")
    # a stream of torch's (default priority) so that torch's events can be recorded into the stream the library
    # launches on; inputs are made on torch's default stream and the device is synchronised before they are used
    stream = torch.cuda.Stream()
    ctx = ops.Context(0, guard=False, stream=stream)
    # what a generated Session promises in its constructor: the weight tensors of the convolution workloads do not
    # change, so the library lays them out for its kernels once instead of in front of every launch
    ctx.check(ctx.lib.sofie_hip_constant_weights(ctx.h, 1))
    timer = LaunchTimer(torch, stream)
    threads = host_threads()

    n = 4096
    rng = np.random.default_rng(0)
    A = rng.integers(-127, 128, (n, n)).astype(np.int8)
    B = rng.integers(-127, 128, (n, n)).astype(np.int8)
    scale = rng.uniform(1e-3, 1e-2, n).astype(np.float32)
    dA, dB, dS = ctx.dev(A), ctx.dev(B), ctx.dev(scale)
    dY = ctx.empty((n, n), torch.int8)
    torch.cuda.synchronize()

    def step():
        # B as ONNX QLinearMatMul states it: [K, N] row-major; the kernel stages rows of k in LDS and the
        # transposing LDS read builds the matrix operand (no separate transpose, no scratch).
        ctx.check(ctx.lib.sofie_hip_qgemm_s8(ctx.h, 0, n, n, n, ctx.ptr(dA), n, ctx.ptr(dB), n, ctx.ptr(dS), None,
                                             0, L.ACT_NONE, ctx.ptr(dY), n, L.OUT_S8))

    if args.traffic_probe:
        X = torch.randn(16 * 1024 * 1024, device=ctx.device)      # the ReLU kernel reads 64 MiB and writes 64 MiB
        Z = torch.empty_like(X)
        torch.cuda.synchronize()
        for _ in range(3):
            ctx.check(ctx.lib.sofie_hip_relu_f32(ctx.h, ctx.ptr(X), ctx.ptr(Z), X.numel()))
            step()
        torch.cuda.synchronize()
        return
    if args.kernel_probe:
        if args.kernel_probe == "gemm_s8":
            fn = step
        else:
            probes = workloads(ctx, torch, L, rng)
            if args.kernel_probe not in probes:
                sys.exit("bench.py: unknown --kernel-probe %s" % args.kernel_probe)
            fn = probes[args.kernel_probe][0]
        torch.cuda.synchronize()
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        return

    # the device out of its idle clocks first (reported as spin_up_ms), then the warm-up steps, then EXACTLY `steps`
    # timed steps bracketed by device synchronisation
    t_spin = time.perf_counter()
    spin_launches = 0
    while (time.perf_counter() - t_spin) * 1e3 < args.spin_up_ms:
        for _ in range(50):
            step()
        spin_launches += 50
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # (nothing but the launches inside the timed region: two events around the steps cost 25 us of it)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    ops_per_step = 2.0 * n * n * n
    tops = ops_per_step / (ms_per_step * 1e-3) / 1e12

    # duration of one launch: HIP events on the launch stream around blocks of 10 back-to-back launches, 25 blocks
    # (250 launches whatever --steps says), median over the blocks
    kernel_ms, kernel_ms_best, launches = timer.median_ms(step, 250, warmup=10, per_block=10)
    achieved = ops_per_step / (kernel_ms * 1e-3) / 1e12

    out = {
        "metric": "int8/FP8 GEMM TOPS & % MFMA peak; model inferences/sec at batch 4096",
        "value": tops, "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "spin_up_ms": args.spin_up_ms, "untimed_launches_before_the_timed_steps": spin_launches + args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": "int8 GEMM (QLinearMatMul) M=N=K=4096, A [M,K] and B [K,N] int8 U[-127,127], "
                               "zero-point 0, per-column fp32 scale U[1e-3,1e-2], int32 accumulate, RNE requantise "
                               "to int8, operands resident in HBM", "M": n, "N": n, "K": n, "seed": 0},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_INT8_TOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_INT8_TOPS, "traffic": TRAFFIC_BYTES_PER_CALL,
                     "kernel": "k_gemm_dma16<S8,B_KN>",
                     "kernel_ms": kernel_ms, "kernel_ms_best_block": kernel_ms_best, "launches_timed": launches,
                     "kernel_ms_exceeds_ms_per_step": bool(kernel_ms > ms_per_step),
                     "ops_per_launch": ops_per_step, "algorithmic_bytes_per_launch": ALGORITHMIC_BYTES_PER_CALL,
                     "traffic_unit": "HBM bytes per launch, from rocprofv3 --pmc runs (profiles/int8_gemm_4096_k_gemm_dma.md), "
                                     "not measured in this process",
                     "note": "unit counts an int8 multiply-add as 2 ops (TOP/s); one call of the entry point is one launch of "
                             "this kernel; kernel_ms is the median over 25 blocks of 10 back-to-back launches between HIP "
                             "events on the launch stream"},
    }

    # The data sheet's 5.0 POP/s is 256 CUs x 8192 ops per clock at 2400 MHz. With random int8 operands the device
    # holds a lower shader clock under this kernel (it is power-limited: the same launch on all-zero operands runs at
    # the full clock); both are reported next to the headline so that the fraction can be read against either.
    sclk, ms_under_sampling = sclk_under_load(torch, step, stream)
    peak_at_clock = PEAK_INT8_TOPS * sclk / 2400.0 if sclk else None
    out["roofline"]["clock"] = {
        "sclk_mhz_under_this_kernel": sclk, "sclk_mhz_of_the_peak_figure": 2400,
        "peak_at_measured_clock": peak_at_clock,
        # roofline.achieved against the peak at the clock the device holds under this kernel
        "frac_at_measured_clock": achieved / peak_at_clock if sclk else None,
        # the same fraction from the launches that ran while the clock was sampled
        "kernel_ms_while_sampled": ms_under_sampling,
        "frac_at_measured_clock_while_sampled": (ops_per_step / (ms_under_sampling * 1e-3) / 1e12) / peak_at_clock
                                                if sclk and ms_under_sampling else None,
        "source": "rocm-smi --showclocks sampled while the kernel runs back to back (1.5 s of launches, timed in blocks of "
                  "100 between HIP events on the launch stream)"}
    if args.clock_probe:
        # the same launch on all-zero operands: no benchmark figure, it shows what the clock costs. Behind a flag
        # because these launches are launches of the headline kernel and would enter a profiler's average for it.
        dZa, dZb = torch.zeros_like(dA), torch.zeros_like(dB)
        torch.cuda.synchronize()

        def step_zero():
            ctx.check(ctx.lib.sofie_hip_qgemm_s8(ctx.h, 0, n, n, n, ctx.ptr(dZa), n, ctx.ptr(dZb), n, ctx.ptr(dS), None,
                                                 0, L.ACT_NONE, ctx.ptr(dY), n, L.OUT_S8))
        sclk_zero, zero_ms = sclk_under_load(torch, step_zero, stream)
        step()                                   # dY holds the benchmark's result again
        torch.cuda.synchronize()
        out["roofline"]["clock"]["all_zero_operands"] = {
            "kernel_ms": zero_ms, "sclk_mhz": sclk_zero,
            "frac_of_peak": ops_per_step / (zero_ms * 1e-3) / 1e12 / PEAK_INT8_TOPS,
            "note": "same launch, operands all zero: not a benchmark figure"}

    # parity spot check inside the benchmark: the timed output against the oracle on a block of rows, and the same
    # operands once more with scales that spread the outputs over the int8 range (the benchmark's scale range
    # saturates about nine outputs in ten, which exercises the clamp but hardly the rounding)
    if not args.no_cpu:
        rows = args.cpu_rows or 256 * threads
        y_ref, base = cpu_baseline_int8(A, B, scale, rows, threads)
        y_gpu = dY[:rows].cpu().numpy()
        out["cpu_baseline"] = base
        out["parity_rows_checked"] = int(rows)
        out["parity_bit_exact"] = bool(np.array_equal(y_gpu, y_ref))
        from oracle import oracle
        spread = (np.random.default_rng(1).uniform(20, 60, n) / (73.3 * 73.3 * np.sqrt(n))).astype(np.float32)
        dS2 = ctx.dev(spread)
        torch.cuda.synchronize()
        ctx.check(ctx.lib.sofie_hip_qgemm_s8(ctx.h, 0, n, n, n, ctx.ptr(dA), n, ctx.ptr(dB), n, ctx.ptr(dS2), None,
                                             0, L.ACT_NONE, ctx.ptr(dY), n, L.OUT_S8))
        ctx.sync()
        y2 = dY[:128].cpu().numpy()
        r2 = oracle.qgemm_s8(A[:128], B, spread)
        out["parity_spread_scales"] = {"rows": 128, "bit_exact": bool(np.array_equal(y2, r2)),
                                       "saturated_fraction": float(np.mean(np.abs(r2.astype(np.int32)) >= 127))}
    else:
        out["cpu_baseline"] = None

    # second half of the metric: the int8 CNN Session at batch 4096 (its own process, runs in about a second)
    out["model_inferences"] = cnn_session_rate(cpu_images=0 if args.no_cpu else args.cpu_images)
    # every other configuration: each costs milliseconds
    res = {}
    for name, (fn, meta) in workloads(ctx, torch, L, rng).items():
        torch.cuda.synchronize()
        # The same spin-up as in front of the headline steps: the host work between two workloads (operands drawn and
        # uploaded) lets the device fall back to its idle clocks, and it needs tens of milliseconds of launches to
        # leave them. The untimed phase is reported.
        t_spin = time.perf_counter()
        spins = 0
        while (time.perf_counter() - t_spin) * 1e3 < args.spin_up_ms:
            for _ in range(max(1, min(50, meta.get("launches", 50) // 4))):
                fn()
            torch.cuda.synchronize()
            spins += 1
        med, best, count = timer.median_ms(fn, meta.get("launches", 50), warmup=3)
        entry = {"workload": meta["workload"], "ms": med, "ms_best_block": best, "launches_timed": count,
                 "spin_up_ms": args.spin_up_ms}
        rate = meta["ops"] / med / 1e9
        entry[meta["rate_unit"]] = rate
        entry["frac_peak"] = rate / meta["peak"]
        if "bytes" in meta:
            entry["gbs"] = meta["bytes"] / med / 1e6
        if meta.get("bound") == "hbm":
            entry["bound"] = "hbm"
            entry["frac_hbm_peak"] = entry["gbs"] / PEAK_HBM_GBS
        if "check" in meta:
            torch.cuda.synchronize()
            entry["parity"] = meta["check"]()        # outside every timed region
        res[name] = entry
    out["fp8_gemm"] = dict(res["gemm_fp8"], peak_tflops=PEAK_FP8_TFLOPS)
    out["fp8_gemm_b_nk"] = res["gemm_fp8_nk"]
    out["int8_gemm_b_nk"] = res["gemm_s8_nk"]
    out["gemm_f32"] = res["gemm_f32"]
    out["gemm_f32_b_nk"] = res["gemm_f32_nk"]
    out["gemm_f32_batch8"] = res["gemm_f32_batch8"]
    out["int8_gemm_batch8"] = res["gemm_s8_batch8"]
    out["conv_f32"] = res["conv_f32"]
    out["conv_f32_batch1"] = res["conv_f32_batch1"]
    out["conv_s8"] = res["conv_s8"]
    out["conv_transpose_f32"] = res["conv_transpose_f32"]
    out["mlp_f32"] = mlp_session_rate()
    if not args.no_cpu:
        out["cpu_fp32"] = cpu_fp32_baselines(threads)
    print(json.dumps(out))


def fp8_band_check(torch, A8, Bm, transB, sA, sB, bias, Y16, rows=64):
    """The timed FP8 output on a band of rows against the float64 product of the same e4m3 operands (torch's own e4m3
    type and float64 matmul: nothing of this library), with the tolerance the tests state: one bf16 rounding of the
    result plus 7 * 2^-13 of sum|a_k b_k| (what the matrix instruction's sums of eight products may drop)."""
    pick = torch.linspace(0, A8.shape[0] - 1, rows, device=A8.device).long()
    a = A8[pick].view(torch.float8_e4m3fn).to(torch.float64)
    b = Bm.view(torch.float8_e4m3fn).to(torch.float64)
    b = b.t() if transB else b
    truth = (a @ b) * (sA * sB) + bias.to(torch.float64)
    mag = (a.abs() @ b.abs()) * (sA * sB)
    err = (Y16[pick].to(torch.float64) - truth).abs()
    tol = 2.0 ** -8 * truth.abs() + 7 * 2.0 ** -13 * mag + 1e-30
    return {"rows": rows, "within_tolerance": bool((err <= tol).all()), "largest_error_over_tolerance": float((err / tol).max()),
            "tolerance": "2^-8 |ref| + 7 * 2^-13 * sa sb sum|a_k b_k| against the float64 product of the same e4m3 operands"}


def workloads(ctx, torch, L, rng):
    """name -> (launcher, description): the configurations next to the headline one, on resident operands."""
    w = {}
    n = 4096
    A = ctx.dev(rng.integers(-127, 128, (n, n)).astype(np.int8))
    Bt = ctx.dev(rng.integers(-127, 128, (n, n)).astype(np.int8))
    S = ctx.dev(rng.uniform(1e-3, 1e-2, n).astype(np.float32))
    Y = ctx.empty((n, n), torch.int8)
    w["gemm_s8_nk"] = (lambda: ctx.check(ctx.lib.sofie_hip_qgemm_s8(
        ctx.h, 1, n, n, n, ctx.ptr(A), n, ctx.ptr(Bt), n, ctx.ptr(S), None, 0, 0, ctx.ptr(Y), n, L.OUT_S8)),
        {"workload": "int8 GEMM 4096^3 with B pre-transposed to [N,K] (the layout a Session keeps an initializer in)",
         "ops": 2.0 * n ** 3, "rate_unit": "tops", "peak": PEAK_INT8_TOPS, "launches": 200})
    M, N, K = 8192, 8192, 4096
    # operands drawn N(0,1) and cast to e4m3 with per-tensor scales amax / 448 (by the library's own quantiser)
    def e4m3_of(t):
        s_t = float(t.abs().max()) / 448.0
        q = torch.empty(t.shape, dtype=torch.uint8, device=ctx.device)
        ctx.check(ctx.lib.sofie_hip_quantize_f32_e4m3(ctx.h, ctx.ptr(t), ctx.ptr(q), t.numel(), 1.0 / s_t))
        torch.cuda.synchronize()
        return q, s_t
    A8, sA = e4m3_of(torch.randn(M, K, device=ctx.device))
    B8, sB = e4m3_of(torch.randn(K, N, device=ctx.device))
    B8t = B8.t().contiguous()
    bias = torch.randn(N, device=ctx.device)
    Y16 = ctx.empty((M, N), torch.bfloat16)
    for name, tb, Bm in (("gemm_fp8", 0, B8), ("gemm_fp8_nk", 1, B8t)):
        w[name] = ((lambda tb=tb, Bm=Bm: ctx.check(ctx.lib.sofie_hip_gemm_fp8(
            ctx.h, tb, M, N, K, ctx.ptr(A8), K, ctx.ptr(Bm), Bm.shape[1], sA, sB, ctx.ptr(bias), ctx.ptr(Y16), N,
            L.OUT_BF16))),
            {"workload": "FP8 e4m3 GEMM M=N=8192 K=4096, A and B N(0,1) cast to e4m3 with per-tensor scales amax/448, "
                         "B %s, fused bias, bf16 out" % ("[N,K]" if tb else "[K,N]"),
             "ops": 2.0 * M * N * K, "rate_unit": "tflops", "peak": PEAK_FP8_TFLOPS, "launches": 100,
             "check": (lambda tb=tb, Bm=Bm: fp8_band_check(torch, A8, Bm, tb, sA, sB, bias, Y16))})
    # fp32 Gemm as the reference's operator states it (Y = A B + bias, ReLU fused), 4096^3, B as [K,N] and as [N,K]
    Af = torch.randn(n, n, device=ctx.device)
    Bf = torch.randn(n, n, device=ctx.device)
    bf = torch.randn(n, device=ctx.device)
    Yf = ctx.empty((n, n), torch.float32)
    for name, tb in (("gemm_f32", 0), ("gemm_f32_nk", 1)):
        w[name] = ((lambda tb=tb: ctx.check(ctx.lib.sofie_hip_gemm_f32(
            ctx.h, 0, tb, n, n, n, 1.0, ctx.ptr(Af), n, ctx.ptr(Bf), n, 1.0, ctx.ptr(bf), L.BIAS_ROW, ctx.ptr(Yf), n, L.ACT_RELU))),
            {"workload": "fp32 Gemm 4096^3 (ROperator_Gemm: Y = A B + bias row, ReLU fused), A and B N(0,1), B %s"
                         % ("[N,K] (transB = 1)" if tb else "[K,N]"),
             "ops": 2.0 * n ** 3, "rate_unit": "tflops", "peak": PEAK_FP32_TFLOPS, "launches": 20})
    # the same layer on a batch of 8 rows: a pass over the 64 MB of B, bound by memory
    Y8 = ctx.empty((8, n), torch.float32)
    w["gemm_f32_batch8"] = ((lambda: ctx.check(ctx.lib.sofie_hip_gemm_f32(
        ctx.h, 0, 0, 8, n, n, 1.0, ctx.ptr(Af), n, ctx.ptr(Bf), n, 1.0, ctx.ptr(bf), L.BIAS_ROW, ctx.ptr(Y8), n, L.ACT_RELU))),
        {"workload": "fp32 Gemm 8 x 4096 x 4096 (a 4096 -> 4096 layer on a batch of 8: Y = A B + bias row, ReLU fused), B [K,N]; "
                     "memory-bound: gbs = algorithmic bytes (B, A, Y, bias once) per second, frac_hbm_peak against 8 TB/s",
         "ops": 2.0 * 8 * n * n, "rate_unit": "tflops", "peak": PEAK_FP32_TFLOPS, "launches": 200,
         "bytes": 4.0 * (n * n + 8 * n + 8 * n + n), "bound": "hbm"})
    # the int8 layer of the headline on a batch of 8 rows, weights [N,K] as a Session keeps them: a pass over 16 MB of B
    A8r = torch.randint(-127, 128, (8, n), dtype=torch.int8, device=ctx.device)
    B8r = torch.randint(-127, 128, (n, n), dtype=torch.int8, device=ctx.device)
    s8r = torch.full((n,), 2e-4, device=ctx.device)
    Y8r = ctx.empty((8, n), torch.int8)
    w["gemm_s8_batch8"] = ((lambda: ctx.check(ctx.lib.sofie_hip_qgemm_s8(
        ctx.h, 1, 8, n, n, ctx.ptr(A8r), n, ctx.ptr(B8r), n, ctx.ptr(s8r), None, 0, L.ACT_NONE, ctx.ptr(Y8r), n, L.OUT_S8))),
        {"workload": "int8 GEMM 8 x 4096 x 4096 (QLinearMatMul of a 4096 -> 4096 layer on a batch of 8), B [N,K], requantised to "
                     "int8; memory-bound: gbs = algorithmic bytes (B, A, Y, scales once) per second, frac_hbm_peak against 8 TB/s",
         "ops": 2.0 * 8 * n * n, "rate_unit": "tops", "peak": PEAK_INT8_TOPS, "launches": 200,
         "bytes": 1.0 * (n * n + 8 * n + 8 * n) + 4.0 * n, "bound": "hbm"})
    # fp32 conv layer: batch 256, 64 -> 128 channels, 56x56, 3x3, pad 1, bias + ReLU
    x = torch.rand(256, 64, 56, 56, device=ctx.device)
    wt = torch.randn(128, 64, 3, 3, device=ctx.device) * (2.0 / 576) ** 0.5
    b = torch.randn(128, device=ctx.device) * 0.1
    y = ctx.empty((256, 128, 56, 56), torch.float32)
    fl = 2.0 * 256 * 128 * 3136 * 576
    w["conv_f32"] = (lambda: ctx.check(ctx.lib.sofie_hip_conv2d_f32(
        ctx.h, ctx.ptr(x), ctx.ptr(wt), ctx.ptr(b), ctx.ptr(y), 256, 64, 56, 56, 128, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1)),
        {"workload": "fp32 Conv2d NCHW batch 256, 64 -> 128 channels, 56x56, 3x3, stride 1, pad 1, bias + ReLU fused; weights promised constant (laid out once, as in a Session)",
         "ops": fl, "rate_unit": "tflops", "peak": PEAK_FP32_TFLOPS, "launches": 20,
         "bytes": 4.0 * (x.numel() + y.numel() + wt.numel() + 128)})
    # the same layer on one image: 25 tiles of 128 x 128 would leave nine compute units in ten idle
    w["conv_f32_batch1"] = (lambda: ctx.check(ctx.lib.sofie_hip_conv2d_f32(
        ctx.h, ctx.ptr(x), ctx.ptr(wt), ctx.ptr(b), ctx.ptr(y), 1, 64, 56, 56, 128, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1)),
        {"workload": "fp32 Conv2d NCHW, one image, 64 -> 128 channels, 56x56, 3x3, stride 1, pad 1, bias + ReLU fused (64 x 64 "
                     "tiles, channel blocks in slices added by a second pass: two launches); weights promised constant",
         "ops": fl / 256, "rate_unit": "tflops", "peak": PEAK_FP32_TFLOPS, "launches": 200})
    # int8 conv layer of the same shape, channels-last, weights [OC][KH][KW][C], bias + ReLU + requantise fused
    # activations uniform [0,1] quantised with scale 1/255 (zero-point -128); weights Kaiming-normal, symmetric int8 per
    # output channel; the output scale puts the layer's range (about 0..4) on the 8 bits
    xq = (torch.round(torch.rand(256, 56, 56, 64, device=ctx.device) * 255.0) - 128.0).to(torch.int8)
    wf = torch.randn(128, 3, 3, 64, device=ctx.device) * (2.0 / 576) ** 0.5
    sw = wf.abs().amax(dim=(1, 2, 3)) / 127.0
    wq = torch.clamp(torch.round(wf / sw.view(-1, 1, 1, 1)), -127, 127).to(torch.int8)
    sq = (sw * (1.0 / 255.0) / (4.0 / 255.0)).float().contiguous()
    bq = torch.round(torch.randn(128, device=ctx.device) * 0.1 / (sw * (1.0 / 255.0))).to(torch.int32)
    yq = ctx.empty((256, 56, 56, 128), torch.int8)
    w["conv_s8"] = (lambda: ctx.check(ctx.lib.sofie_hip_qconv2d_s8(
        ctx.h, ctx.ptr(xq), L.LAYOUT_NHWC, ctx.ptr(wq), L.LAYOUT_NHWC, ctx.ptr(bq), ctx.ptr(sq), ctx.ptr(yq), L.LAYOUT_NHWC,
        256, 64, 56, 56, 128, 3, 3, 1, 1, 1, 1, 1, 1, 1, -128, -128, L.ACT_RELU, L.OUT_S8)),
        {"workload": "int8 QLinearConv channels-last batch 256, 64 -> 128 channels, 56x56, 3x3, stride 1, pad 1, bias + ReLU "
                     "+ requantise fused; activations U[0,1] at scale 1/255, Kaiming-normal weights symmetric int8 per channel", "ops": fl, "rate_unit": "tops", "peak": PEAK_INT8_TOPS, "launches": 200,
         "bytes": float(xq.numel() + yq.numel() + wq.numel() + 128 * 8)})
    # fp32 transposed conv (an upsampling layer): batch 64, 128 -> 64 channels, 28x28 -> 56x56, 4x4, stride 2, pad 1
    xt = torch.rand(64, 128, 28, 28, device=ctx.device)
    wtt = torch.randn(128, 64, 4, 4, device=ctx.device) * 0.05
    bt = torch.randn(64, device=ctx.device) * 0.1
    yt = ctx.empty((64, 64, 56, 56), torch.float32)
    w["conv_transpose_f32"] = (lambda: ctx.check(ctx.lib.sofie_hip_conv_transpose2d_f32(
        ctx.h, ctx.ptr(xt), ctx.ptr(wtt), ctx.ptr(bt), ctx.ptr(yt), 64, 128, 28, 28, 64, 4, 4, 1, 1, 2, 2, 1, 1, 1, 56, 56, 0)),
        {"workload": "fp32 ConvTranspose batch 64, 128 -> 64 channels, 28x28 -> 56x56, 4x4, stride 2, pad 1; weights promised constant (sub-kernels gathered once, as in a Session)",
         "ops": 2.0 * 64 * 128 * 64 * 16 * 784, "rate_unit": "tflops", "peak": PEAK_FP32_TFLOPS, "launches": 20})
    return w


def run_generated(name, dat, x, iters):
    """Runs sofie_amd/generated/run_<name> (a compiled generated Session) on x; returns (timings, output bytes)."""
    gen = os.path.join(ROOT, "sofie_amd", "generated")
    exe, datf = os.path.join(gen, "run_" + name), os.path.join(gen, dat)
    if not (os.path.exists(exe) and os.path.exists(datf)):
        return {"error": "generated Session %s missing: run build() first" % name}, None
    with tempfile.TemporaryDirectory() as tmp:
        xin, yout = os.path.join(tmp, "x.bin"), os.path.join(tmp, "y.bin")
        x.tofile(xin)
        res = subprocess.run([exe, datf, xin, yout, str(iters)], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                             timeout=300)
        y = np.fromfile(yout, np.float32) if res.returncode == 0 else None
    if res.returncode != 0:
        return {"error": res.stderr.strip()[-300:]}, None
    return json.loads(res.stdout.strip().splitlines()[-1]), y


def mlp_session_rate(iters=2000):
    """The generated Session of the fp32 MLP (64 -> 128 -> 64 -> 8, batch 256): three Gemm launches with fused bias and
    ReLU. Device time of infer_device() on a resident input, replay from a HIP graph, wall time of infer()."""
    x = np.random.default_rng(3).standard_normal((256, 64)).astype(np.float32)
    t, _ = run_generated("mlp_c1", "mlp_c1.dat", x, iters)
    if "error" in t:
        return t
    us = t["device_ms"] * 1e3
    return {"workload": "fp32 MLP 64 -> 128 -> 64 -> 8, batch 256, generated Session (infer_device on a resident input)",
            "us_per_batch": us, "inferences_per_s": 256 / (us * 1e-6), "gbs_algorithmic": 142112 / (us * 1e-6) / 1e9,
            "graph_replay_us": t["graph_ms"] * 1e3, "graph_matches": t["graph_matches"],
            "host_us_with_pcie": t["host_ms"] * 1e3, "bound": "launch latency (8.65 MFLOP, 142,112 algorithmic bytes)"}


def cnn_session_rate(iters=300, cpu_images=0):
    """The generated Session of the int8 CNN at batch 4096 (1x40x40 input; conv 1->32, pool, conv 32->64, pool,
    conv 64->128, fc 12800->256, fc 256->5), run by its prebuilt runner as a child process: device time of
    infer_device() on a resident input, and wall time of infer() including the PCIe copies. With cpu_images > 0 the
    CPU restatement of the same network is timed on that many images of the batch (one thread) and the Session's
    logits of those images are compared with it bit for bit."""
    x = np.random.default_rng(2).uniform(0, 1, (4096, 1, 40, 40)).astype(np.float32)
    t, y = run_generated("qcnn_b4096", "qcnn.dat", x, iters)
    if "error" in t:
        return t
    ops_per_image = 36968960.0
    cpu = None
    if cpu_images > 0:
        # checker and baseline: the oracle's network (tests/models.py builds it from the same seeded parameters)
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        import models
        from oracle import oracle
        models.qcnn_reference(oracle, x[:2])           # parameters and calibration are built on the first call
        t0 = time.perf_counter()
        ref = models.qcnn_reference(oracle, x[:cpu_images])
        sec = time.perf_counter() - t0
        cpu = {"value": cpu_images / sec, "unit": "inferences/s", "cores": 1, "kind": "port",
               "role": "the checker of the Session's logits (a scalar restatement of the int8 arithmetic), not the baseline",
               "sample": "oracle/sofie_oracle.c (quantize, three QLinearConv + ReLU + MaxPool, two QLinearMatMul) on the first "
                         "%d of the 4096 images (%.2f s, gcc -O2, 1 thread)" % (cpu_images, sec),
               "logits_bit_exact": bool(np.array_equal(y.reshape(4096, -1)[:cpu_images], ref.reshape(cpu_images, -1)))}
    # per kernel, from the runner's events behind every launch (the time of a launch runs from the end of the launch
    # before it): operations of the layer(s) the launch computes against the int8 matrix peak
    layer_ops = {"k_qconv_first": 2.0 * 4096 * 1600 * 32 * 9, "k_qconv_ring_pool": 2.0 * 4096 * 400 * 64 * 288,
                 "k_qconv_ring": 2.0 * 4096 * 100 * 128 * 576, "k_gemm_bytes": 2.0 * 4096 * 256 * 12800,
                 "k_qconv_ring_pair": 2.0 * 4096 * 400 * 64 * 288 + 2.0 * 4096 * 100 * 128 * 576,
                 "k_splitk_finish_pair": 2.0 * 4096 * 5 * 256}
    kernels = []
    for k in t.get("kernels", []):
        e = {"kernel": k["kernel"], "us": k["us"]}
        if k["kernel"] in layer_ops and k["us"] > 0:
            e["gop"] = layer_ops[k["kernel"]] / 1e9
            e["frac_peak"] = layer_ops[k["kernel"]] / (k["us"] * 1e-6) / 1e12 / PEAK_INT8_TOPS
        kernels.append(e)
    return {"cpu_baseline": cnn_cpu_reference() if cpu_images > 0 else None, "int8_oracle_checker": cpu,
            "workload": "int8 CNN classifier, batch 4096, 1x40x40 input, generated Session (infer_device on a resident input)",
            "device_ms": t["device_ms"], "inferences_per_s": 4096 / (t["device_ms"] * 1e-3),
            "tops": 4096 * ops_per_image / t["device_ms"] / 1e9,
            "frac_peak": 4096 * ops_per_image / t["device_ms"] / 1e9 / PEAK_INT8_TOPS,
            "kernels": kernels,
            "kernels_note": "one entry per launch of a batch, in launch order; us = time from the end of the launch before it "
                            "to its own end (events on the Session's stream), averaged over up to 200 batches back to back",
            "host_ms_with_pcie": t["host_ms"], "inferences_per_s_with_pcie": 4096 / (t["host_ms"] * 1e-3),
            "host_ms_with_pcie_pinned_input": t.get("host_pinned_ms"),
            "inferences_per_s_with_pcie_pinned_input": 4096 / (t["host_pinned_ms"] * 1e-3) if t.get("host_pinned_ms") else None,
            "pinned_input_same_logits": t.get("pinned_matches"),
            "graph_replay_ms": t.get("graph_ms") or None, "graph_replay_same_logits": t.get("graph_matches"),
            # two Sessions in flight on one device (two contexts and streams, a host thread each): wall time per batch
            "two_sessions_ms_per_batch": t.get("two_sessions_ms_per_batch") or None,
            "two_sessions_inferences_per_s": 4096 / (t["two_sessions_ms_per_batch"] * 1e-3) if t.get("two_sessions_ms_per_batch") else None,
            "two_sessions_same_logits": t.get("two_sessions_match")}


def cnn_cpu_reference(images=256):
    """The CPU baseline of the classifier: the call sequence the reference emits for the float model (Conv as weight
    re-layout + Im2col + sgemm_ + saxpy_ per image, Relu, the MaxPool loop, Gemm as bias copy + sgemm_), restated in
    oracle/cpu_emitted_bench.c, with sgemm_ from the best BLAS on the box, on `images` images at one thread and at the
    box's core share. (The reference has no quantized operators: its path for this network is the fp32 one.)"""
    threads = host_threads()
    chosen = None
    for cand in blas_candidates() + [None]:
        if cpu_emitted("mlp", 1, cand, ("--calls", "20")) is not None:
            chosen = cand
            break
    res = {"kind": "port", "what": "the reference's emitted fp32 call sequence for this network, twice: restated in C "
                                   "(oracle/cpu_emitted_bench.c --workload cnn, gcc -O2: the N_threads entries) and as the "
                                   "Session this build's emitter generates with Options::kHostCode (generated_host_session_*); "
                                   "value is the best of them",
           "blas": chosen[2] if chosen else "none found: the bundled loops", "unit": "inferences/s"}
    for th in sorted({1, threads}):
        c = cpu_emitted("cnn", th, chosen, ("--images", str(images), "--calls", "3"))
        if c:
            res["%d_threads" % th] = {"value": images / (c["median_ms"] * 1e-3), "cores": th, "median_ms": c["median_ms"],
                                      "sample": "%d of the 4096 images, median of %d calls" % (images, c["calls"])}
    x = np.random.default_rng(2).uniform(0, 1, (256, 1, 40, 40)).astype(np.float32)
    for th in sorted({1, threads}):
        hs = generated_host_session("cnn_f32_b256", "cnn_f32", x, th, chosen, 3)
        if hs:
            res["generated_host_session_%d_threads" % th] = {
                "value": 256 / (hs["median_ms"] * 1e-3), "cores": th, "median_ms": hs["median_ms"],
                "sample": "256 of the 4096 images, median of 3 calls of Session::infer",
                "what": "the float model's Session generated with Options::kHostCode (this build's emission of the "
                        "reference's CPU path: Im2col + sgemm_ + saxpy_ per image, Relu and MaxPool loops, Gemm), g++ -O2"}
    # the int8 network itself as generated host code (the quantized operators' host form: scalar loops with int32 sums)
    x8 = np.random.default_rng(2).uniform(0, 1, (4096, 1, 40, 40)).astype(np.float32)[:8]
    hq = generated_host_session("qcnn", "qcnn", x8, 1, None, 3)
    if hq:
        res["generated_host_session_int8"] = {
            "value": 8 / (hq["median_ms"] * 1e-3), "cores": 1, "median_ms": hq["median_ms"],
            "sample": "the first 8 of the 4096 images, median of 3 calls of Session::infer",
            "what": "the int8 model's Session generated with Options::kHostCode (QuantizeLinear, QLinearConv, MaxPool and "
                    "QLinearMatMul as scalar loops), g++ -O2, one thread; its logits are the device Session's bit for bit "
                    "(tests/test_gpu_generated.py)"}
    best = max((v["value"] for k, v in res.items() if k.endswith("_threads")), default=None)
    res["value"] = best
    res["sample"] = "%d of the 4096 images per call" % images
    res["cores"] = max((v["cores"] for k, v in res.items() if k.endswith("_threads") and v["value"] == best), default=None)
    return res


if __name__ == "__main__":
    main()
