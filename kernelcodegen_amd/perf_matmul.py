#!/usr/bin/env python3
"""Matmul sweep in the shape of the reference's perf harness.

The reference's driver (test/test.cc:8-61) generates a kernel for 4096x2048x1024
and for 20 square sizes 256..16384 and hands each to a harness that prints, per
size (performance/output.log:1-13):

    Matrix size / M / N / K, Occupancy, My Matmul Latency,
    cublas Latency(NN), cublas Ratio(NN), cublas Latency(TT), cublas Ratio(TT)

This script prints the same fields for the gfx950 kernel, with the ROCm library
GEMM (torch.matmul -> hipBLASLt/rocBLAS) in cuBLAS's place, plus decimal TFLOP/s
and the fraction of the 157.3 TFLOP/s fp32 MFMA peak (the reference's plot.py
divides by 1024^4 instead and therefore reads ~9 % lower).

    python kernelcodegen_amd/perf_matmul.py [--max-dim 16384] [--relu]
"""
import argparse
import ctypes
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

PEAK_FP32_TFLOPS = 157.3
DIMS = [256, 512, 768, 1024, 1536, 2048, 3072, 4096, 5120, 6144, 7168, 8192, 9216, 10240, 11264,
        12288, 13312, 14336, 15360, 16384]


def _time(fn, iters):
    from kernelcodegen_amd.timing import time_launches
    return time_launches(fn, iters)


def occupancy_percent(info):
    """Resident waves per SIMD over the 8 the hardware can hold: workgroups per CU are
    limited by LDS (160 KiB) and by the kernels' register budget (2 waves per SIMD)."""
    by_lds = (160 * 1024) // max(info.lds_bytes, 1)
    by_regs = max(1, 8 // info.waves_per_block)
    waves_per_cu = min(by_lds, by_regs) * info.waves_per_block
    return 100.0 * (waves_per_cu / 4.0) / 8.0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--max-dim", type=int, default=16384)
    ap.add_argument("--relu", action="store_true")
    args = ap.parse_args()

    import torch
    from kernelcodegen_amd import lib, ops

    L = lib.load()
    dev = torch.device("cuda:0")
    shapes = [(4096, 2048, 1024)] + [(d, d, d) for d in DIMS if d <= args.max_dim]
    rows = []
    # The shader clock takes some tens of milliseconds of load to settle: without this the
    # first (small) shapes of the sweep are timed on a ramping clock.
    W = torch.randn(4096, 4096, device=dev)
    for _ in range(200):
        ops.matmul(W, W, relu=args.relu)
    torch.cuda.synchronize()
    del W
    for (M, N, K) in shapes:
        A = torch.randn(M, K, device=dev)
        B = torch.randn(K, N, device=dev)
        C = torch.empty(M, N, device=dev)
        At = A.t().contiguous()
        Bt = B.t().contiguous()
        Ct = torch.empty(N, M, device=dev)
        flops = 2.0 * M * N * K
        iters = max(3, min(50, int(2e12 / flops)))
        info = lib.LaunchInfo()
        lib.check(L.kcg_gemm_f32_query(M, N, K, None, ctypes.byref(info)))
        mine = _time(lambda: ops.matmul(A, B, relu=args.relu, out=C), iters)
        # the result of the timed launches against the library on three bands of rows
        # (first, middle, last: the extremes of every operand's address range)
        err = 0.0
        for r0 in (0, max(0, M // 2 - 128), max(0, M - 256)):
            ref = torch.matmul(A[r0:r0 + 256], B)
            if args.relu:
                ref = torch.relu(ref)
            err = max(err, float((C[r0:r0 + 256] - ref).abs().max() / ref.abs().max()))
        nn = _time(lambda: torch.matmul(A, B, out=C), iters)
        # "TT": both operands transposed in memory, C^T = B^T . A^T
        tt = _time(lambda: torch.matmul(Bt, At, out=Ct), iters)
        tf = flops / mine / 1e9
        print("Matrix size : \n --- M --- : %d\n --- N --- : %d\n --- K --- : %d\n" % (M, N, K))
        print("Occupancy: %.0f%%  (%s, grid %d x %d threads, %d B LDS)" % (
            occupancy_percent(info), info.kernel.decode(), info.grid[0], info.block[0], info.lds_bytes))
        print("My Matmul Latency = %g ms  (%.2f TFLOP/s, %.1f%% of fp32 MFMA peak)\n" % (
            mine, tf, 100 * tf / PEAK_FP32_TFLOPS))
        print("rocm-lib Latency(NN) = %g ms\nrocm-lib Ratio(NN) = %g%%\n" % (nn, 100 * nn / mine))
        print("rocm-lib Latency(TT) = %g ms\nrocm-lib Ratio(TT) = %g%%\n" % (tt, 100 * tt / mine), flush=True)
        print("max |C - library| / max |C| on sampled rows = %.2g\n" % err, flush=True)
        rows.append((M, N, K, mine, tf, 100 * tf / PEAK_FP32_TFLOPS, nn, flops / nn / 1e9, err))
        del A, B, C, At, Bt, Ct
    print("| M x N x K | kernel ms | TFLOP/s | % of 157.3 | library NN ms | library TFLOP/s | max err vs library |")
    print("|---|---|---|---|---|---|---|")
    for r in rows:
        print("| %dx%dx%d | %.5g | %.2f | %.1f | %.5g | %.2f | %.1e |" % r)


if __name__ == "__main__":
    main()
