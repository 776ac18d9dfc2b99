#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

A step is one launch of the fused fp32 matmul + ReLU kernel on BASELINE.json's
configs[1] (M = N = K = 4096, A, B ~ N(0,1) from the seeded generator), inputs
resident in HBM.  Prints ONE JSON line: whole-job TFLOP/s, the roofline of the
kernel (algorithmic FLOPs / HIP-event launch time vs the fp32 MFMA peak), the CPU
oracle timed on the host cores, and the two attention workloads as extras (plus the bf16
one without its causal mask, for comparison).

Every timed region is preceded by an untimed clock-settle phase (SETTLE_MS of back-to-back
launches of the same call) in addition to the --warmup launches, so that the figures do not
depend on how many warm-up steps the caller asks for.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extras]
    python bench.py --sweep matmul [--max-dim D | --dims D1,MxNxK,...] [--relu] [--seeded] [--dump DIR] [--workspace]
                                   [--series FILE]
    python bench.py --sweep fmha | --sweep ops [--shape B,H,S,D]
    python bench.py --sweep fmha-variants      (after `make -C kernelcodegen_amd/csrc variants`)
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_TFLOPS = 157.3    # MI355X dense fp32 MFMA
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA

# HBM bytes per launch (fetch + write).  NOT measured by this script: counters cannot be
# read from inside the timed run, so these are the figures of separate rocprofv3 --pmc
# FETCH_SIZE / --pmc WRITE_SIZE runs of profile_kernels.py, each scaled by
# the same counter's reading for a 256 MiB copy, as recorded in the named profile files.
TRAFFIC = {
    "gemm_cfg1": (743925920, "profiles/gemm_f32_cfg1.md"),
    "fmha_cfg3": (137533632, "profiles/fmha_f32_cfg3.md"),
    "fmha_cfg4": (788052280, "profiles/fmha_bf16_cfg4.md"),
}


def traffic_fields(key):
    nbytes, src = TRAFFIC[key]
    return {"traffic": nbytes,
            "traffic_source": src + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, copy-calibrated; "
                                    "a separate run, not measured here)"}


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


SETTLE_MS = 40.0   # untimed launches before every timed region, whatever --warmup says


def settle(fn, ms=SETTLE_MS):
    """Runs fn back to back, untimed, until at least `ms` milliseconds have passed, and
    returns the milliseconds spent.  The shader clock drops within a millisecond of idle
    time (host work, allocations, the CPU leg) and needs tens of milliseconds of load to
    come back; a handful of warm-up launches of a sub-millisecond kernel is not enough."""
    import torch
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3


def time_launches(fn, steps, warmup):
    """(wall ms per step, HIP-event ms per launch) over `steps` launches of fn, after the
    clock-settle phase and `warmup` further untimed launches."""
    import torch
    stream = torch.cuda.current_stream()
    settle(fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(stream)          # the kernels are launched on this same stream
    for _ in range(steps):
        fn()
    e1.record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, e0.elapsed_time(e1) / steps


def launch_stats(fn, launches=20):
    """(median, min) HIP-event ms of single launches, each bracketed by its own event pair
    on the launch stream (outside the timed region of the headline figure)."""
    import torch
    stream = torch.cuda.current_stream()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(launches)]
    for a, b in pairs:
        a.record(stream)
        fn()
        b.record(stream)
    torch.cuda.synchronize()
    ms = sorted(a.elapsed_time(b) for a, b in pairs)
    return ms[len(ms) // 2], ms[0]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip the attention workloads")
    ap.add_argument("--sweep", choices=["matmul", "fmha", "ops", "fmha-variants"],
                    help="instead of the benchmark line, print a measurement sweep: the reference's "
                         "matmul size sweep in its output.log format, the attention shape grid, or the "
                         "un-fused operators against their rooflines (kernelcodegen_amd/sweeps.py)")
    ap.add_argument("--max-dim", type=int, default=16384, help="--sweep matmul: largest square size")
    ap.add_argument("--relu", action="store_true", help="--sweep matmul: with the fused ReLU epilogue")
    ap.add_argument("--seeded", action="store_true", help="--sweep matmul: operands from the seeded generator")
    ap.add_argument("--dump", help="--sweep matmul: directory that receives sampled rows of every C")
    ap.add_argument("--series", help="--sweep matmul: JSON file that receives the latency / throughput / peak-ratio "
                                     "series of the reference's performance/plot.py")
    ap.add_argument("--dims", default="",
                    help="--sweep matmul: comma-separated sizes instead of the reference's list, each n (square) or MxNxK")
    ap.add_argument("--workspace", action="store_true",
                    help="--sweep matmul: lend the calls a 32 MiB workspace (kcg_gemm_f32_ws)")
    ap.add_argument("--shape", default="1,32,2048,128", help="--sweep ops: B,H,S,D")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the matmul and attention kernels shard over row "
                 "blocks / heads with no exchange step, and this build launches no multi-GPU run "
                 "(use --gpus 1)")

    import numpy as np
    import torch
    import __graft_entry__
    __graft_entry__.ensure_built()      # builds only if no library is there at all
    from kernelcodegen_amd import inputs, lib, ops

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    lib.load()
    dev = torch.device("cuda:0")
    if args.sweep:
        from kernelcodegen_amd import sweeps
        if args.sweep == "matmul":
            sweeps.matmul(args.max_dim, args.relu, args.seeded, args.dump, args.workspace,
                          [int(d) if d.isdigit() else tuple(int(x) for x in d.split("x"))
                           for d in args.dims.split(",")] if args.dims else None, args.series)
        elif args.sweep == "fmha":
            sweeps.fmha()
        elif args.sweep == "fmha-variants":
            sweeps.fmha_variants()
        else:
            sweeps.ops_chain(tuple(int(x) for x in args.shape.split(",")))
        return

    # ---------------- headline: configs[1], fp32 4096^3 matmul + ReLU ----------------
    cfg = inputs.config_inputs(1)
    A_h, B_h = cfg["A"], cfg["B"]
    M, K = A_h.shape
    N = B_h.shape[1]
    A = torch.from_numpy(A_h).to(dev)
    B = torch.from_numpy(B_h).to(dev)
    C = torch.empty((M, N), dtype=torch.float32, device=dev)
    flops = 2.0 * M * N * K
    alg_bytes = 4.0 * (M * K + K * N + M * N)
    wall_ms, ev_ms = time_launches(lambda: ops.matmul(A, B, relu=True, out=C), args.steps, args.warmup)
    value = flops / (wall_ms * 1e-3) / 1e12
    achieved = flops / (ev_ms * 1e-3) / 1e12
    med_ms, min_ms = launch_stats(lambda: ops.matmul(A, B, relu=True, out=C))

    out = {
        "metric": "fp32 GEMM TFLOP/s + % FP32 peak; FMHA TFLOP/s at S=2048,d=128",
        "value": round(value, 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "clock_settle_ms": SETTLE_MS,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "configs[1]: fp32 matmul + fused ReLU, M=N=K=4096, row-major, "
                               "A,B ~ N(0,1) seeded", "M": M, "N": N, "K": K, "epilogue": "relu"},
        "pct_fp32_peak": round(100.0 * value / PEAK_FP32_TFLOPS, 2),
        "roofline": {"bound": "mfma", "achieved": round(achieved, 3), "peak": PEAK_FP32_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / PEAK_FP32_TFLOPS, 4),
                     **traffic_fields("gemm_cfg1"), "kernel": "gemm_f32_dl_kernel",
                     "algorithmic_flops": flops, "algorithmic_bytes": alg_bytes,
                     "launch_ms": round(ev_ms, 5), "launch_ms_median": round(med_ms, 5),
                     "launch_ms_min": round(min_ms, 5)},
    }

    # ---------------- CPU baseline: the oracle on the host cores ----------------
    if not args.no_cpu:
        from oracle import oracle
        oracle.build()
        dt = float("inf")
        for _ in range(3):
            t0 = time.perf_counter()
            ref = oracle.relu(oracle.matmul(A_h, B_h))
            dt = min(dt, time.perf_counter() - t0)
        Ch = C.cpu().numpy()
        d = np.abs(Ch.astype(np.float64) - ref)
        rms = float(np.sqrt((ref.astype(np.float64) ** 2).mean()))
        out["cpu_baseline"] = {
            "value": round(flops / dt / 1e12, 5), "unit": "TFLOP/s", "cores": oracle.num_threads(),
            "cpu_model": _cpu_model(),
            "kind": "port", "sample": "the whole configs[1] workload (4096^3 matmul + ReLU), best of "
                                      "3 runs, %.2f s wall each" % dt,
            "gpu_vs_cpu_max_rel_err": float((d / np.maximum(np.abs(ref), rms)).max()),
        }
        del ref, Ch

    # ---------------- extras: the two attention workloads ----------------
    if not args.no_extras:
        extras = {}
        steps = max(5, args.steps)
        warm = args.warmup
        c3 = inputs.config_inputs(3)
        Q, Kt, V = (torch.from_numpy(c3[k]).to(dev) for k in "QKV")
        O = torch.empty_like(Q)
        Bn, H, S, D = Q.shape
        fl = 4.0 * Bn * H * S * S * D
        w, e = time_launches(lambda: ops.fmha(Q, Kt, V, scale=c3["scale"], causal=False, out=O),
                             steps, warm)
        extras["fmha_f32_cfg3"] = {
            "workload": "configs[3]: fp32 FMHA B=1 H=32 S=2048 D=128 non-causal", "ms_per_step": round(w, 5),
            "value": round(fl / (w * 1e-3) / 1e12, 3), "unit": "TFLOP/s",
            "roofline": {"bound": "mfma", "achieved": round(fl / (e * 1e-3) / 1e12, 3),
                         "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(fl / (e * 1e-3) / 1e12 / PEAK_FP32_TFLOPS, 4),
                         **traffic_fields("fmha_cfg3")}}
        del Q, Kt, V, O
        c4 = inputs.config_inputs(4)
        Q, Kt, V = (torch.from_numpy(c4[k].view(np.int16)).to(dev).view(torch.bfloat16) for k in "QKV")
        O = torch.empty_like(Q)
        Bn, H, S, D = Q.shape
        fl = 0.5 * 4.0 * Bn * H * S * S * D      # causal-counted (half of the full S^2 work)
        w, e = time_launches(lambda: ops.fmha(Q, Kt, V, scale=c4["scale"], causal=True, out=O),
                             steps, warm)
        extras["fmha_bf16_cfg4"] = {
            "workload": "configs[4]: bf16 FMHA B=4 H=32 S=4096 D=128 causal, causal-counted FLOPs",
            "ms_per_step": round(w, 5), "value": round(fl / (w * 1e-3) / 1e12, 3), "unit": "TFLOP/s",
            "roofline": {"bound": "mfma", "achieved": round(fl / (e * 1e-3) / 1e12, 3),
                         "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(fl / (e * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4),
                         **traffic_fields("fmha_cfg4")}}
        # the same tensors without the mask: what the causal structure (diagonal tiles, the
        # restart of the second block of a pair) costs on top of the kernel's own rate
        fl = 4.0 * Bn * H * S * S * D
        w, e = time_launches(lambda: ops.fmha(Q, Kt, V, scale=c4["scale"], causal=False, out=O),
                             steps, warm)
        extras["fmha_bf16_cfg4_shape_noncausal"] = {
            "workload": "the configs[4] tensors (bf16, B=4 H=32 S=4096 D=128) without the causal mask; not a BASELINE config",
            "ms_per_step": round(w, 5), "value": round(fl / (w * 1e-3) / 1e12, 3), "unit": "TFLOP/s",
            "roofline": {"bound": "mfma", "achieved": round(fl / (e * 1e-3) / 1e12, 3),
                         "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(fl / (e * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4), "traffic": None}}
        out["extras"] = extras

    print(json.dumps(out))


if __name__ == "__main__":
    main()
