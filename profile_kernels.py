#!/usr/bin/env python3
"""Runs one workload's kernel a few times, preceded by a plain device-to-device
copy of known size, so that a profiler run over this script sees both:

    rocprofv3 --kernel-trace --stats -d OUT -- python3 profile_kernels.py --workload gemm_cfg1
    rocprofv3 --pmc FETCH_SIZE -d OUT -- python3 profile_kernels.py --workload gemm_cfg1
    rocprofv3 --pmc WRITE_SIZE -d OUT -- python3 profile_kernels.py --workload gemm_cfg1

The copy (COPY_MIB MiB read + COPY_MIB MiB written per launch) calibrates the
FETCH_SIZE / WRITE_SIZE counters: the factor is bytes-known / counter-read.

The workload's launches come in two groups: a settle phase (launches of the same call
until --settle-ms of wall-clock time have passed, so that the shader clock has left its
ramp; their number is printed) and then --iters launches.  A kernel trace holds both
groups; the launches after the settle phase are the last --iters of the kernel.
"""
import argparse
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

COPY_MIB = 256


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="gemm_cfg1",
                    choices=["gemm_cfg0", "gemm_cfg1", "gemm_cfg2", "fmha_cfg3", "fmha_cfg4",
                             "bmmnt_cfg3", "bmmnn_cfg3", "softmax_cfg3", "relu_1gib", "gemm_ksplit", "gemm_1536"],
                    help="a BASELINE config of the fused kernels, or an un-fused operator at the "
                         "configs[3] shape (bmmnt: Q.K^T, bmmnn: P.V, softmax: in place on the scores) "
                         "/ ReLU on a 1 GiB tensor / gemm_ksplit: 1536^3 (+ReLU) through the workspace entry "
                         "point, whose plan is two launches (whole tiles and K pieces, then the sum of the pieces) "
                         "/ gemm_1536: 1536^3 (+ReLU) through kcg_gemm_f32 (the 96 x 96 tile by default; --tile applies)")
    ap.add_argument("--tile", default="",
                    help="matmul workloads only: BLOCK_M x BLOCK_N x BLOCK_K of the schedule, e.g. 256x128x32 "
                         "(default: the library's choice)")
    ap.add_argument("--library", default="",
                    help="another build of libkcg_hip.so (an experiment build of `make -C kernelcodegen_amd/csrc "
                         "variants`) instead of the library beside the package")
    ap.add_argument("--iters", type=int, default=200, help="launches of the workload after the settle phase")
    ap.add_argument("--settle-ms", type=float, default=40.0,
                    help="wall-clock time of the launches that precede them (0: none)")
    args = ap.parse_args()

    if args.library:
        os.environ["KCG_LIBRARY"] = os.path.abspath(args.library)
    import numpy as np
    import torch
    from kernelcodegen_amd import inputs, ops

    dev = torch.device("cuda:0")
    src = torch.empty(COPY_MIB * (1 << 20) // 4, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    for _ in range(min(args.iters, 40)):
        dst.copy_(src)
    torch.cuda.synchronize()

    kind, _, cfg = args.workload.partition("_")
    c = inputs.config_inputs(int(cfg[3:])) if cfg.startswith("cfg") else None
    if kind == "relu":
        X = torch.empty(16384, 16384, device=dev).normal_()
        Y = torch.empty_like(X)
        fn = lambda: ops.relu(X, out=Y)
    elif kind in ("bmmnt", "bmmnn", "softmax"):
        Q, K, V = (torch.from_numpy(c[k]).to(dev) for k in "QKV")
        P = ops.batched_matmul(Q, K, trans_b=True)
        O = torch.empty_like(Q)
        if kind == "bmmnt":
            fn = lambda: ops.batched_matmul(Q, K, trans_b=True, out=P)
        elif kind == "bmmnn":
            ops.softmax_(P.mul_(c["scale"]))
            fn = lambda: ops.batched_matmul(P, V, out=O)
        else:
            P.mul_(c["scale"])
            fn = lambda: ops.softmax_(P)
    elif args.workload == "gemm_ksplit":
        d = 1536
        A = torch.empty(d, d, device=dev).normal_()
        B = torch.empty(d, d, device=dev).normal_()
        C = torch.empty(d, d, device=dev)
        ws = torch.empty(ops.matmul_workspace_bytes(d, d, d) // 4, dtype=torch.float32, device=dev)
        assert ws.numel() > 0
        fn = lambda: ops.matmul(A, B, relu=True, out=C, workspace=ws)
    elif args.workload == "gemm_1536":
        d = 1536
        A = torch.empty(d, d, device=dev).normal_()
        B = torch.empty(d, d, device=dev).normal_()
        C = torch.empty(d, d, device=dev)
        sched = None
        if args.tile:
            bm, bn, bk = (int(x) for x in args.tile.split("x"))
            sched = dict(block_m=bm, block_n=bn, block_k=bk)
        fn = lambda: ops.matmul(A, B, relu=True, out=C, sched=sched)
    elif kind == "gemm":
        A = torch.from_numpy(c["A"]).to(dev)
        B = torch.from_numpy(c["B"]).to(dev)
        C = torch.empty((A.shape[0], B.shape[1]), dtype=torch.float32, device=dev)
        sched = None
        if args.tile:
            bm, bn, bk = (int(x) for x in args.tile.split("x"))
            sched = dict(block_m=bm, block_n=bn, block_k=bk)
        fn = lambda: ops.matmul(A, B, relu=c["relu"], out=C, sched=sched)
    else:
        if c["dtype"] == "bf16":
            Q, K, V = (torch.from_numpy(c[k].view(np.int16)).to(dev).view(torch.bfloat16) for k in "QKV")
        else:
            Q, K, V = (torch.from_numpy(c[k]).to(dev) for k in "QKV")
        O = torch.empty_like(Q)
        fn = lambda: ops.fmha(Q, K, V, scale=c["scale"], causal=c["causal"], out=O)
    import time
    settle = 0
    t0 = time.perf_counter()
    while args.settle_ms > 0 and (time.perf_counter() - t0) * 1e3 < args.settle_ms:
        for _ in range(4):
            fn()
        torch.cuda.synchronize()
        settle += 4
    for _ in range(args.iters):
        fn()
    torch.cuda.synchronize()
    print("done", args.workload, "settle launches", settle, "then", args.iters)


if __name__ == "__main__":
    main()
