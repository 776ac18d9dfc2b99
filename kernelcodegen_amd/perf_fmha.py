#!/usr/bin/env python3
"""Fused attention over a grid of shapes, both element types, with the default schedule.

The reference publishes no attention timing (its fused kernel is work in progress,
src/Optimizer/Optimizer.cc:1079-1333); this sweep is the counterpart of perf_matmul.py
for the attention entry points.  FLOPs are 4.B.H.S^2.D, halved for causal launches
(the FlashAttention convention); peaks 157.3 TFLOP/s (fp32 MFMA) and 2500 (bf16 MFMA).

    python kernelcodegen_amd/perf_fmha.py [--iters N]
"""
import argparse
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

PEAK = {"float32": 157.3, "bfloat16": 2500.0}
SHAPES = [(1, 32, 2048, 128), (4, 32, 4096, 128), (2, 16, 8192, 128), (8, 32, 1024, 128),
          (16, 16, 512, 128), (1, 32, 2048, 64), (4, 32, 4096, 64), (8, 32, 1024, 64), (2, 16, 8192, 64)]


def _time(fn, iters):
    from kernelcodegen_amd.timing import time_launches
    return time_launches(fn, iters)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--iters", type=int, default=20)
    args = ap.parse_args()

    import ctypes
    import torch
    from kernelcodegen_amd import lib, ops

    L = lib.load()
    dev = torch.device("cuda:0")
    W = torch.randn(4096, 4096, device=dev)
    for _ in range(100):     # settle the shader clock
        ops.matmul(W, W)
    torch.cuda.synchronize()
    print("| dtype | B,H,S,D | causal | kernel | grid | ms | TFLOP/s | % of peak |")
    print("|---|---|---|---|---|---|---|---|")
    for dt in (torch.float32, torch.bfloat16):
        name = str(dt)[6:]
        for (B, H, S, D) in SHAPES:
            Q = torch.randn(B, H, S, D, device=dev).to(dt)
            K = torch.randn_like(Q)
            V = torch.randn_like(Q)
            O = torch.empty_like(Q)
            for causal in (False, True):
                info = lib.LaunchInfo()
                lib.check(L.kcg_fmha_query(0 if dt == torch.float32 else 1, B, H, S, D, int(causal), None,
                                           ctypes.byref(info)))
                ms = _time(lambda: ops.fmha(Q, K, V, scale=D ** -0.5, causal=causal, out=O), args.iters)
                tf = 4.0 * B * H * S * S * D * (0.5 if causal else 1.0) / ms / 1e9
                print("| %s | %d,%d,%d,%d | %d | %s | %d x %d | %.4f | %.1f | %.1f |" % (
                    name, B, H, S, D, causal, info.kernel.decode(), info.grid[0], info.block[0], ms, tf,
                    100 * tf / PEAK[name]), flush=True)


if __name__ == "__main__":
    main()
