#!/usr/bin/env python3
"""The un-fused operators timed against their rooflines.

The attention graph of the reference (test/test.cc:71-90) is BatchedMatmul(Q, K^T) ->
Softmax -> BatchedMatmul(P, V); when the fused pattern does not match, every operator
runs as its own kernel (src/Optimizer/Optimizer.cc:597-652).  This script times that
three-kernel chain at the configs[3] shape next to the fused kernel, and the standalone
ReLU at the configs[1] shape:

    BatchedMatmul NT   S = Q.K^T   [B,H,S,D] x [B,H,S,D]^T -> [B,H,S,S]   fp32 MFMA bound
    Softmax            P = softmax(S) in place over the last axis          HBM bound (read + write)
    BatchedMatmul NN   O = P.V     [B,H,S,S] x [B,H,S,D]   -> [B,H,S,D]   fp32 MFMA bound
    Relu               y = max(x, 0)                                        HBM bound (read + write)

    python kernelcodegen_amd/perf_ops.py [--shape B,H,S,D] [--iters N]
"""
import argparse
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

PEAK_FP32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0


def _time(fn, iters):
    from kernelcodegen_amd.timing import time_launches
    return time_launches(fn, iters)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--shape", default="1,32,2048,128")
    ap.add_argument("--iters", type=int, default=30)
    args = ap.parse_args()
    B, H, S, D = (int(x) for x in args.shape.split(","))

    import torch
    from kernelcodegen_amd import lib, ops

    lib.load()
    dev = torch.device("cuda:0")
    W = torch.randn(4096, 4096, device=dev)
    for _ in range(100):     # settle the shader clock
        ops.matmul(W, W)
    torch.cuda.synchronize()

    Q = torch.randn(B, H, S, D, device=dev)
    K = torch.randn_like(Q)
    V = torch.randn_like(Q)
    P = torch.empty(B, H, S, S, device=dev)
    O = torch.empty_like(Q)
    rows = []

    def mfma_row(name, ms, flops):
        tf = flops / ms / 1e9
        rows.append((name, ms, "%.1f TFLOP/s" % tf, "mfma", 100 * tf / PEAK_FP32_TFLOPS))

    def hbm_row(name, ms, nbytes):
        gbs = nbytes / ms / 1e6
        rows.append((name, ms, "%.0f GB/s" % gbs, "hbm", 100 * gbs / PEAK_HBM_GBS))

    t = _time(lambda: ops.batched_matmul(Q, K, trans_b=True, out=P), args.iters)
    mfma_row("BatchedMatmul NT  S = Q.K^T", t, 2.0 * B * H * S * S * D)
    t_qk = t
    # the softmax is timed on scores of realistic spread; it runs in place, so on its own output
    # from the second launch on (timing does not depend on the values)
    P.mul_(D ** -0.5)
    t = _time(lambda: ops.softmax_(P), args.iters)
    hbm_row("Softmax in place   P = softmax(S)", t, 2.0 * 4 * P.numel())
    t_sm = t
    t = _time(lambda: ops.batched_matmul(P, V, out=O), args.iters)
    mfma_row("BatchedMatmul NN  O = P.V", t, 2.0 * B * H * S * S * D)
    t_pv = t
    fused = _time(lambda: ops.fmha(Q, K, V, scale=D ** -0.5, out=O), 4 * args.iters)
    mfma_row("fused FMHA (one kernel)", fused, 4.0 * B * H * S * S * D)
    rows.append(("un-fused chain (three kernels)", t_qk + t_sm + t_pv,
                 "%.1fx the fused kernel" % ((t_qk + t_sm + t_pv) / fused), "-", float("nan")))
    del P

    X = torch.randn(4096, 4096, device=dev)
    Y = torch.empty_like(X)
    t = _time(lambda: ops.relu(X, out=Y), args.iters)
    hbm_row("Relu 4096 x 4096", t, 2.0 * 4 * X.numel())
    X = torch.randn(16384, 16384, device=dev)
    Y = torch.empty_like(X)
    t = _time(lambda: ops.relu(X, out=Y), args.iters)
    hbm_row("Relu 16384 x 16384", t, 2.0 * 4 * X.numel())

    print("shape B,H,S,D = %d,%d,%d,%d" % (B, H, S, D))
    print("| operator | ms | rate | bound | % of peak |")
    print("|---|---|---|---|---|")
    for r in rows:
        print(("| %s | %.4f | %s | %s | %.1f |" % r).replace("| nan |", "| - |"))


if __name__ == "__main__":
    main()
