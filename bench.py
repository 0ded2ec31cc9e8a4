#!/usr/bin/env python3
"""Benchmark of the SOFIE hot path on one MI355X.

Headline workload (the configuration the metric is quoted on): standalone int8 GEMM with QLinearMatMul
semantics, M=N=K=4096, A and B int8 uniform in [-127,127], per-output-channel fp32 scales
uniform in [1e-3,1e-2], int32 accumulate, round-half-to-even requantise to int8. One "step"
is one call of sofie_hip_qgemm_s8 on device-resident operands. Prints ONE JSON line; next to the headline value it
carries the other two figures the metric names: `fp8_gemm` (e4m3 GEMM 8192x8192x4096, TFLOP/s and fraction of the
FP8 MFMA peak) and `model_inferences` (the generated int8 CNN Session at batch 4096, inferences per second).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--extras]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0     # MI355X dense int8 MFMA, 5.0 POP/s
PEAK_FP8_TFLOPS = 5000.0
PEAK_FP32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
# HBM-side bytes of one call of the headline entry point (one GEMM kernel), from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs scaled by the same counters on a 64 MiB copy-like kernel (FETCH_SIZE x1.999, WRITE_SIZE x1.000):
# 96.3 MiB fetched + 16.0 MiB written. Algorithmic bytes: 50.3 MB.
TRAFFIC_BYTES_PER_CALL = 112.3 * 1024 * 1024


def cpu_baseline_int8(A, B, scale, rows):
    """The oracle (a scalar C port of the same arithmetic) on the first `rows` rows of A."""
    from oracle import oracle
    t0 = time.perf_counter()
    y = oracle.qgemm_s8(A[:rows], B, scale)
    dt = time.perf_counter() - t0
    ops = 2.0 * rows * B.shape[0] * B.shape[1]
    return y, {"value": ops / dt / 1e12, "unit": "TOPS", "cores": 1, "kind": "port",
               "sample": "oracle/sofie_oracle.c or_qgemm_s8 on the first %d of %d rows of A against the full B "
                         "(%.1f GOP, %.1f s, gcc -O2, 1 thread)" % (rows, A.shape[0], ops / 1e9, dt)}


def time_launches(ctx, fn, steps, warmup):
    """HIP events on the stream the kernels run on; returns average ms per launch."""
    for _ in range(warmup):
        fn()
    ctx.sync()
    ctx.timer_start()
    for _ in range(steps):
        fn()
    return ctx.timer_stop() / steps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-rows", type=int, default=1024)
    ap.add_argument("--cpu-images", type=int, default=256, help="images of the CNN batch the CPU baseline leg evaluates")
    ap.add_argument("--extras", action="store_true", help="also time the FP8 GEMM, fp32 GEMM and conv layers")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="launch a 64 MiB copy-like kernel and the headline call three times and exit (the target of the "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus %d is not supported (no collective, no sharding "
                 "code exists). Run with --gpus 1." % args.gpus)

    import torch
    from sofie_amd import lib as L
    from sofie_amd import ops
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible (the HIP library has no CPU fallback)")
    ctx = ops.default_context()

    n = 4096
    rng = np.random.default_rng(0)
    A = rng.integers(-127, 128, (n, n)).astype(np.int8)
    B = rng.integers(-127, 128, (n, n)).astype(np.int8)
    scale = rng.uniform(1e-3, 1e-2, n).astype(np.float32)
    dA, dB, dS = ctx.dev(A), ctx.dev(B), ctx.dev(scale)
    dY = ctx.empty((n, n), torch.int8)

    def step():
        # B as ONNX QLinearMatMul states it: [K, N] row-major; the kernel stages rows of k in LDS and the
        # transposing LDS read builds the matrix operand (no separate transpose, no scratch).
        ctx.check(ctx.lib.sofie_hip_qgemm_s8(ctx.h, 0, n, n, n, ctx.ptr(dA), n, ctx.ptr(dB), n, ctx.ptr(dS), None,
                                             0, L.ACT_NONE, ctx.ptr(dY), n, L.OUT_S8))

    if args.traffic_probe:
        X = torch.randn(16 * 1024 * 1024, device=ctx.device)      # the ReLU kernel reads 64 MiB and writes 64 MiB
        Z = torch.empty_like(X)
        for _ in range(3):
            ctx.check(ctx.lib.sofie_hip_relu_f32(ctx.h, ctx.ptr(X), ctx.ptr(Z), X.numel()))
            step()
        torch.cuda.synchronize()
        return

    # warm-up, then EXACTLY `steps` timed steps bracketed by device synchronisation
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    ops_per_step = 2.0 * n * n * n
    tops = ops_per_step / (ms_per_step * 1e-3) / 1e12

    # kernel duration from HIP events on the launch stream
    kernel_ms = time_launches(ctx, step, args.steps, 2)
    achieved = ops_per_step / (kernel_ms * 1e-3) / 1e12

    out = {
        "metric": "int8/FP8 GEMM TOPS & % MFMA peak; model inferences/sec at batch 4096",
        "value": tops, "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": "int8 GEMM (QLinearMatMul) M=N=K=4096, A [M,K] and B [K,N] int8 U[-127,127], "
                               "zero-point 0, per-column fp32 scale U[1e-3,1e-2], int32 accumulate, RNE requantise "
                               "to int8, operands resident in HBM", "M": n, "N": n, "K": n, "seed": 0},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_INT8_TOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_INT8_TOPS, "traffic": TRAFFIC_BYTES_PER_CALL,
                     "kernel": "k_gemm_dma<MmaI8,128,2,S8,B_KN>",
                     "kernel_ms": kernel_ms, "ops_per_launch": ops_per_step,
                     "traffic_unit": "bytes per launch (profiles/int8_gemm_4096_k_gemm_dma.md)",
                     "note": "unit counts an int8 multiply-add as 2 ops (TOP/s); one call of the entry point is one "
                             "launch of this kernel"},
    }

    # parity spot check inside the benchmark: the timed output against the oracle on a few rows
    if not args.no_cpu:
        y_ref, base = cpu_baseline_int8(A, B, scale, args.cpu_rows)
        y_gpu = dY[:args.cpu_rows].cpu().numpy()
        out["cpu_baseline"] = base
        out["parity_rows_checked"] = int(args.cpu_rows)
        out["parity_bit_exact"] = bool(np.array_equal(y_gpu, y_ref))
    else:
        out["cpu_baseline"] = None

    # second half of the metric: the int8 CNN Session at batch 4096 (its own process, runs in about a second)
    out["model_inferences"] = cnn_session_rate(cpu_images=0 if args.no_cpu else args.cpu_images)
    # the FP8 half of the metric's GEMM figure (e4m3 x e4m3, fp32 accumulate, bf16 out): B as it comes ([K,N])
    fp8 = fp8_gemm_rates(ctx, torch, L)["fp8_gemm_8192x8192x4096_transB0"]
    out["fp8_gemm"] = {"workload": "FP8 e4m3 GEMM M=N=8192 K=4096, B [K,N], bias, bf16 out", "ms": fp8["ms"],
                       "tflops": fp8["tflops"], "frac_peak": fp8["frac_peak"], "peak_tflops": PEAK_FP8_TFLOPS}
    if args.extras:
        out["extras"] = extras(ctx, torch, L, ops, rng)
    print(json.dumps(out))


def fp8_gemm_rates(ctx, torch, L):
    """FP8 e4m3 GEMM 8192 x 8192 x 4096, bf16 out, fused bias, for B given [K,N] and [N,K]."""
    res = {}
    M, N, K = 8192, 8192, 4096
    A8 = torch.randint(0, 120, (M, K), dtype=torch.uint8, device=ctx.device)
    B8 = torch.randint(0, 120, (K, N), dtype=torch.uint8, device=ctx.device)
    bias = torch.randn(N, device=ctx.device)
    Y16 = ctx.empty((M, N), torch.bfloat16)
    for tb, Bm in ((0, B8), (1, B8.t().contiguous())):
        ms = time_launches(ctx, lambda: ctx.check(ctx.lib.sofie_hip_gemm_fp8(
            ctx.h, tb, M, N, K, ctx.ptr(A8), K, ctx.ptr(Bm), Bm.shape[1], 0.01, 0.01, ctx.ptr(bias), ctx.ptr(Y16), N,
            L.OUT_BF16)), 20, 3)
        fl = 2.0 * M * N * K
        res["fp8_gemm_8192x8192x4096_transB%d" % tb] = {"ms": ms, "tflops": fl / ms / 1e9,
                                                        "frac_peak": fl / ms / 1e9 / PEAK_FP8_TFLOPS}
    return res


def extras(ctx, torch, L, ops, rng):
    """Secondary figures of the other benchmark configurations (not the headline value)."""
    ex = {}
    # pre-transposed weights: the layout a Session keeps B in when it is an initializer
    n = 4096
    A = ctx.dev(rng.integers(-127, 128, (n, n)).astype(np.int8))
    Bt = ctx.dev(rng.integers(-127, 128, (n, n)).astype(np.int8))
    S = ctx.dev(rng.uniform(1e-3, 1e-2, n).astype(np.float32))
    Y = ctx.empty((n, n), torch.int8)
    ms = time_launches(ctx, lambda: ctx.check(ctx.lib.sofie_hip_qgemm_s8(
        ctx.h, 1, n, n, n, ctx.ptr(A), n, ctx.ptr(Bt), n, ctx.ptr(S), None, 0, 0, ctx.ptr(Y), n, L.OUT_S8)), 50, 5)
    ex["int8_gemm_4096_transB"] = {"ms": ms, "tops": 2.0 * n ** 3 / ms / 1e9, "frac_peak": 2.0 * n ** 3 / ms / 1e9 / PEAK_INT8_TOPS}
    ex.update(fp8_gemm_rates(ctx, torch, L))
    # fp32 conv layer: batch 256, 64 -> 128 channels, 56x56, 3x3, pad 1, bias + ReLU
    x = torch.rand(256, 64, 56, 56, device=ctx.device)
    w = torch.randn(128, 64, 3, 3, device=ctx.device) * (2.0 / 576) ** 0.5
    b = torch.randn(128, device=ctx.device) * 0.1
    y = ctx.empty((256, 128, 56, 56), torch.float32)
    ms = time_launches(ctx, lambda: ctx.check(ctx.lib.sofie_hip_conv2d_f32(
        ctx.h, ctx.ptr(x), ctx.ptr(w), ctx.ptr(b), ctx.ptr(y), 256, 64, 56, 56, 128, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1)),
        5, 1)
    fl = 2.0 * 256 * 128 * 3136 * 576
    ex["conv2d_f32_b256_64to128_56x56"] = {"ms": ms, "tflops": fl / ms / 1e9, "frac_peak": fl / ms / 1e9 / PEAK_FP32_TFLOPS}
    del x, w, y
    # fp32 transposed conv (an upsampling layer): batch 64, 128 -> 64 channels, 28x28 -> 56x56, 4x4, stride 2, pad 1
    x = torch.rand(64, 128, 28, 28, device=ctx.device)
    w = torch.randn(128, 64, 4, 4, device=ctx.device) * 0.05
    b = torch.randn(64, device=ctx.device) * 0.1
    y = ctx.empty((64, 64, 56, 56), torch.float32)
    ms = time_launches(ctx, lambda: ctx.check(ctx.lib.sofie_hip_conv_transpose2d_f32(
        ctx.h, ctx.ptr(x), ctx.ptr(w), ctx.ptr(b), ctx.ptr(y), 64, 128, 28, 28, 64, 4, 4, 1, 1, 2, 2, 1, 1, 1, 56, 56, 0)),
        5, 1)
    fl = 2.0 * 64 * 128 * 64 * 16 * 784      # every input pixel meets every kernel tap once
    ex["conv_transpose2d_f32_b64_128to64_28to56"] = {"ms": ms, "tflops": fl / ms / 1e9,
                                                      "frac_peak": fl / ms / 1e9 / PEAK_FP32_TFLOPS}
    # fp32 MLP batch 256: 64 -> 128 -> 64 -> 8 (three Gemm launches, ReLU fused)
    X = torch.randn(256, 64, device=ctx.device)
    Ws = [torch.randn(64, 128, device=ctx.device), torch.randn(128, 64, device=ctx.device),
          torch.randn(64, 8, device=ctx.device)]
    Bs = [torch.zeros(128, device=ctx.device), torch.zeros(64, device=ctx.device), torch.zeros(8, device=ctx.device)]
    Hs = [ctx.empty((256, 128), torch.float32), ctx.empty((256, 64), torch.float32), ctx.empty((256, 8), torch.float32)]

    def mlp():
        cur = X
        for i, (Wm, bm, h) in enumerate(zip(Ws, Bs, Hs)):
            ctx.check(ctx.lib.sofie_hip_gemm_f32(ctx.h, 0, 0, 256, Wm.shape[1], Wm.shape[0], 1.0, ctx.ptr(cur),
                                                 Wm.shape[0], ctx.ptr(Wm), Wm.shape[1], 1.0, ctx.ptr(bm), L.BIAS_ROW,
                                                 ctx.ptr(h), Wm.shape[1], 1 if i < 2 else 0))
            cur = h
    ms = time_launches(ctx, mlp, 200, 10)
    ex["mlp_f32_b256"] = {"us": ms * 1e3, "inferences_per_s": 256 / (ms * 1e-3), "gbs": 142112 / (ms * 1e-3) / 1e9}
    del x, w, b, y
    # int8 conv layer of the same shape, channels-last, weights [OC][KH][KW][C], bias + ReLU + requantise fused
    xq = torch.randint(-128, 128, (256, 56, 56, 64), dtype=torch.int8, device=ctx.device)
    wq = torch.randint(-127, 128, (128, 3, 3, 64), dtype=torch.int8, device=ctx.device)
    sq = torch.full((128,), 2.0e-4, device=ctx.device)
    bq = torch.randint(-1000, 1000, (128,), dtype=torch.int32, device=ctx.device)
    yq = ctx.empty((256, 56, 56, 128), torch.int8)
    ms = time_launches(ctx, lambda: ctx.check(ctx.lib.sofie_hip_qconv2d_s8(
        ctx.h, ctx.ptr(xq), L.LAYOUT_NHWC, ctx.ptr(wq), L.LAYOUT_NHWC, ctx.ptr(bq), ctx.ptr(sq), ctx.ptr(yq), L.LAYOUT_NHWC,
        256, 64, 56, 56, 128, 3, 3, 1, 1, 1, 1, 1, -128, -128, L.ACT_RELU, L.OUT_S8)), 20, 3)
    fl = 2.0 * 256 * 128 * 3136 * 576
    ex["conv2d_s8_b256_64to128_56x56"] = {"ms": ms, "tops": fl / ms / 1e9, "frac_peak": fl / ms / 1e9 / PEAK_INT8_TOPS,
                                          "gbs": (xq.numel() + yq.numel() + wq.numel()) / ms / 1e6}
    del xq, yq
    return ex


def cnn_session_rate(iters=50, cpu_images=0):
    """The generated Session of the int8 CNN at batch 4096 (1x40x40 input; conv 1->32, pool, conv 32->64, pool,
    conv 64->128, fc 12800->256, fc 256->5), run by its prebuilt runner as a child process: device time of
    infer_device() on a resident input, and wall time of infer() including the PCIe copies. With cpu_images > 0 the
    CPU restatement of the same network is timed on that many images of the batch (one thread) and the Session's
    logits of those images are compared with it bit for bit."""
    import subprocess
    import tempfile
    gen = os.path.join(ROOT, "sofie_amd", "generated")
    exe, dat = os.path.join(gen, "run_qcnn_b4096"), os.path.join(gen, "qcnn.dat")
    if not (os.path.exists(exe) and os.path.exists(dat)):
        return {"error": "generated Session missing: run build() first"}
    with tempfile.TemporaryDirectory() as tmp:
        xin, yout = os.path.join(tmp, "x.bin"), os.path.join(tmp, "y.bin")
        x = np.random.default_rng(2).uniform(0, 1, (4096, 1, 40, 40)).astype(np.float32)
        x.tofile(xin)
        res = subprocess.run([exe, dat, xin, yout, str(iters)], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                             timeout=300)
        y = np.fromfile(yout, np.float32) if res.returncode == 0 else None
    if res.returncode != 0:
        return {"error": res.stderr.strip()[-300:]}
    t = json.loads(res.stdout.strip().splitlines()[-1])
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
               "sample": "oracle/sofie_oracle.c (quantize, three QLinearConv + ReLU + MaxPool, two QLinearMatMul) on the first "
                         "%d of the 4096 images (%.2f s, gcc -O2, 1 thread)" % (cpu_images, sec),
               "logits_bit_exact": bool(np.array_equal(y.reshape(4096, -1)[:cpu_images], ref.reshape(cpu_images, -1)))}
    return {"cpu_baseline": cpu,"workload": "int8 CNN classifier, batch 4096, 1x40x40 input, generated Session (infer_device on a resident input)",
            "device_ms": t["device_ms"], "inferences_per_s": 4096 / (t["device_ms"] * 1e-3),
            "tops": 4096 * ops_per_image / t["device_ms"] / 1e9,
            "frac_peak": 4096 * ops_per_image / t["device_ms"] / 1e9 / PEAK_INT8_TOPS,
            "host_ms_with_pcie": t["host_ms"], "inferences_per_s_with_pcie": 4096 / (t["host_ms"] * 1e-3)}


if __name__ == "__main__":
    main()
