"""Measurement sweeps behind `bench.py --sweep matmul|fmha|ops`.

matmul: the reference's perf harness.  Its driver (test/test.cc:8-61) generates a kernel
for 4096x2048x1024 and for 20 square sizes 256..16384 and hands each to a harness that
prints, per size (performance/output.log:1-13):

    Matrix size / M / N / K, Occupancy, My Matmul Latency,
    cublas Latency(NN), cublas Ratio(NN), cublas Latency(TT), cublas Ratio(TT)

`matmul()` prints the same fields for the gfx950 kernel, with the ROCm library GEMM
(torch.matmul -> hipBLASLt / rocBLAS) in cuBLAS's place, plus decimal TFLOP/s and the
fraction of the 157.3 TFLOP/s fp32 MFMA peak (the reference's plot.py divides by 1024^4
instead and therefore reads ~9 % lower).  With `seeded` the operands come from the
seeded generator of inputs.py and `dump_dir` receives three bands of rows of every C, so
that a caller can check them against an independent evaluation of the same operands.

fmha: the fused attention entry points over a grid of shapes, both element types (the
reference publishes no attention timing: its fused kernel is work in progress,
src/Optimizer/Optimizer.cc:1079-1333).  FLOPs are 4.B.H.S^2.D, halved for causal launches.

ops: the un-fused operators (BatchedMatmul NT / NN, Softmax, Relu; the fall-through of
src/Optimizer/Optimizer.cc:597-652) against their rooflines, next to the fused kernel.
"""
import ctypes
import os

PEAK_FP32_TFLOPS = 157.3
PEAK_BF16_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0
MATMUL_DIMS = [256, 512, 768, 1024, 1536, 2048, 3072, 4096, 5120, 6144, 7168, 8192, 9216, 10240,
               11264, 12288, 13312, 14336, 15360, 16384]
MATMUL_SEED = 0x5EED
FMHA_SHAPES = [(1, 32, 2048, 128), (4, 32, 4096, 128), (2, 16, 8192, 128), (8, 32, 1024, 128),
               (16, 16, 512, 128), (8, 32, 2048, 64), (1, 32, 2048, 64), (4, 32, 4096, 64),
               (8, 32, 1024, 64), (2, 16, 8192, 64)]


def _time(fn, iters):
    from .timing import time_launches
    return time_launches(fn, iters)


def _settle(dev):
    """Some tens of milliseconds of load before the first (small) shape is timed."""
    import torch
    from . import ops
    W = torch.randn(4096, 4096, device=dev)
    for _ in range(100):
        ops.matmul(W, W)
    torch.cuda.synchronize()


def computed_occupancy_percent(info):
    """Resident waves per SIMD over the 8 the hardware can hold, COMPUTED from the launch
    geometry (workgroups per CU are limited by the 160 KiB of LDS and by the kernels'
    register budget of 2 waves per SIMD) -- not read from a profiler."""
    by_lds = (160 * 1024) // max(info.lds_bytes, 1)
    by_regs = max(1, 8 // info.waves_per_block)
    waves_per_cu = min(by_lds, by_regs) * info.waves_per_block
    return 100.0 * (waves_per_cu / 4.0) / 8.0


def row_bands(M):
    """Three bands of up to 8 rows: first, middle, last (the extremes of the operands' address range)."""
    return [(r0, min(M, r0 + 8)) for r0 in sorted({0, max(0, M // 2 - 4), max(0, M - 8)})]


def matmul_series(rows):
    """The three series the reference's performance/plot.py:43-91 reads out of an output.log
    (latency, throughput, ratio to peak; one line per method), from rows of (M, N, K, kernel ms,
    library NN ms, library TT ms).  Throughput is decimal TFLOP/s (plot.py divides by 1024^4 and
    calls it TFLOPS); the last method is the chip's fp32 matrix peak, as plot.py's is the A100's."""
    methods = ["Generated-Matmul", "rocm-lib-NN", "rocm-lib-TT", "MI355X-fp32-MFMA-Peak"]
    dims, latency, throughput, ratio = [], [[] for _ in methods], [[] for _ in methods], [[] for _ in methods]
    for (M, N, K, mine, nn, tt) in rows:
        flops = 2.0 * M * N * K
        dims.append(M if M == N == K else "%dx%dx%d" % (M, N, K))
        peak_ms = flops / (PEAK_FP32_TFLOPS * 1e9)
        for i, ms in enumerate((mine, nn, tt, peak_ms)):
            latency[i].append(ms)
            throughput[i].append(flops / ms / 1e9)
            ratio[i].append(100.0 * flops / ms / 1e9 / PEAK_FP32_TFLOPS)
    return {"methods": methods, "dims": dims, "latency_ms": latency, "throughput_tflops": throughput,
            "peak_ratio_percent": ratio, "peak_tflops": PEAK_FP32_TFLOPS}


def matmul(max_dim=16384, relu=False, seeded=False, dump_dir=None, workspace=False, dims=None, series_path=None):
    import numpy as np
    import torch
    from . import inputs, lib, ops

    L = lib.load()
    dev = torch.device("cuda:0")
    shapes = [(4096, 2048, 1024)] + [(d, d, d) for d in MATMUL_DIMS if d <= max_dim]
    if dims:   # sizes of the caller's choice instead of the reference's list: n (square) or (M, N, K)
        shapes = [(d, d, d) if isinstance(d, int) else tuple(d) for d in dims]
    rows, series_rows = [], []
    _settle(dev)
    # --workspace: the calls lend 32 MiB (kcg_gemm_f32_ws), which sizes with a K-split plan use
    ws = torch.empty(8 << 20, dtype=torch.float32, device=dev) if workspace else None
    for (M, N, K) in shapes:
        if seeded:
            A = torch.from_numpy(inputs.uniform((M, K), MATMUL_SEED, 0)).to(dev)
            B = torch.from_numpy(inputs.uniform((K, N), MATMUL_SEED, 1)).to(dev)
        else:
            A = torch.randn(M, K, device=dev)
            B = torch.randn(K, N, device=dev)
        C = torch.empty(M, N, device=dev)
        At = A.t().contiguous()
        Bt = B.t().contiguous()
        Ct = torch.empty(N, M, device=dev)
        flops = 2.0 * M * N * K
        iters = max(3, min(50, int(2e12 / flops)))
        info = lib.LaunchInfo()
        # (the geometry of the launches that are timed: with a workspace, the K-split pair)
        if workspace:
            lib.check(L.kcg_gemm_f32_ws_query(M, N, K, None, ws.numel() * 4, ctypes.byref(info)))
        else:
            lib.check(L.kcg_gemm_f32_query(M, N, K, None, ctypes.byref(info)))
        mine = _time(lambda: ops.matmul(A, B, relu=relu, out=C, workspace=ws), iters)
        split_bytes = ops.matmul_workspace_bytes(M, N, K) if workspace else 0
        if dump_dir:
            bands = np.concatenate([C[a:b].cpu().numpy() for a, b in row_bands(M)])
            np.save(os.path.join(dump_dir, "C_%dx%dx%d.npy" % (M, N, K)), bands)
        # the result of the timed launches against the library on three bands of rows
        err = 0.0
        for r0 in (0, max(0, M // 2 - 128), max(0, M - 256)):
            ref = torch.matmul(A[r0:r0 + 256], B)
            if relu:
                ref = torch.relu(ref)
            err = max(err, float((C[r0:r0 + 256] - ref).abs().max() / ref.abs().max()))
        nn = _time(lambda: torch.matmul(A, B, out=C), iters)
        # "TT": both operands transposed in memory, C^T = B^T . A^T
        tt = _time(lambda: torch.matmul(Bt, At, out=Ct), iters)
        tf = flops / mine / 1e9
        kernels = info.kernel.decode()
        geometry = "grid %d x %d threads, %d B LDS" % (info.grid[0], info.block[0], info.lds_bytes)
        if info.launches == 2 and info.tail_rows:
            geometry += "; second launch %s on the last %d rows, grid %d x %d threads, %d B LDS" % (
                info.tail_kernel.decode(), info.tail_rows, info.tail_grid[0], info.tail_block[0], info.tail_lds_bytes)
        elif info.launches == 2:
            geometry += "; K-split plan with %d bytes of partial tiles, second launch %s adds them up, grid %d x %d threads" % (
                split_bytes, info.tail_kernel.decode(), info.tail_grid[0], info.tail_block[0])
        print("Matrix size : \n --- M --- : %d\n --- N --- : %d\n --- K --- : %d\n" % (M, N, K))
        print("Occupancy: %.0f%%  (computed from the launch geometry: %s, %s)" % (
            computed_occupancy_percent(info), kernels, geometry))
        print("My Matmul Latency = %g ms  (%.2f TFLOP/s, %.1f%% of fp32 MFMA peak)\n" % (
            mine, tf, 100 * tf / PEAK_FP32_TFLOPS))
        print("rocm-lib Latency(NN) = %g ms\nrocm-lib Ratio(NN) = %g%%\n" % (nn, 100 * nn / mine))
        print("rocm-lib Latency(TT) = %g ms\nrocm-lib Ratio(TT) = %g%%\n" % (tt, 100 * tt / mine), flush=True)
        print("max |C - library| / max |C| on sampled rows = %.2g\n" % err, flush=True)
        rows.append((M, N, K, mine, tf, 100 * tf / PEAK_FP32_TFLOPS, nn, flops / nn / 1e9, err))
        series_rows.append((M, N, K, mine, nn, tt))
        del A, B, C, At, Bt, Ct
    print("| M x N x K | kernel ms | TFLOP/s | % of 157.3 | library NN ms | library TFLOP/s | max err vs library |")
    print("|---|---|---|---|---|---|---|")
    for r in rows:
        print("| %dx%dx%d | %.5g | %.2f | %.1f | %.5g | %.2f | %.1e |" % r)
    if series_path:
        import json
        with open(series_path, "w") as fp:
            json.dump(matmul_series(series_rows), fp, indent=1)
    return rows


def fmha(iters=20, shapes=None):
    import torch
    from . import lib, ops

    L = lib.load()
    dev = torch.device("cuda:0")
    _settle(dev)
    peak = {"float32": PEAK_FP32_TFLOPS, "bfloat16": PEAK_BF16_TFLOPS}
    print("| dtype | B,H,S,D | causal | kernel | grid | ms | TFLOP/s | % of peak |")
    print("|---|---|---|---|---|---|---|---|")
    out = []
    for dt in (torch.float32, torch.bfloat16):
        name = str(dt)[6:]
        for (B, H, S, D) in (shapes or FMHA_SHAPES):
            Q = torch.randn(B, H, S, D, device=dev).to(dt)
            K = torch.randn_like(Q)
            V = torch.randn_like(Q)
            O = torch.empty_like(Q)
            for causal in (False, True):
                info = lib.LaunchInfo()
                lib.check(L.kcg_fmha_query(0 if dt == torch.float32 else 1, B, H, S, D, int(causal), None,
                                           ctypes.byref(info)))
                ms = _time(lambda: ops.fmha(Q, K, V, scale=D ** -0.5, causal=causal, out=O), iters)
                tf = 4.0 * B * H * S * S * D * (0.5 if causal else 1.0) / ms / 1e9
                print("| %s | %d,%d,%d,%d | %d | %s | %d x %d | %.4f | %.1f | %.1f |" % (
                    name, B, H, S, D, causal, info.kernel.decode(), info.grid[0], info.block[0], ms, tf,
                    100 * tf / peak[name]), flush=True)
                out.append((name, (B, H, S, D), causal, ms, tf))
    return out


def fmha_variants(shape=(4, 32, 4096, 128), iters=20, rounds=4):
    """The experiment builds of the bf16 attention kernel (`make -C kernelcodegen_amd/csrc variants`)
    against the default library on configs[4]'s shape, causal and not: every library is timed in
    every round, one after the other, so that box and clock drift hit all of them alike; the
    output of each build is compared with the default's (the builds change schedules, not
    arithmetic)."""
    import glob
    import torch
    from . import lib

    here = os.path.dirname(os.path.abspath(__file__))
    paths = [lib.LIB_PATH] + sorted(glob.glob(os.path.join(here, "csrc", "variants", "libkcg_hip_*.so")))
    if len(paths) == 1:
        raise RuntimeError("no experiment builds: run `make -C kernelcodegen_amd/csrc variants` first")
    libs = []
    for p in paths:
        L = ctypes.CDLL(p)
        L.kcg_fmha_bf16.restype, L.kcg_fmha_bf16.argtypes = lib.SYMBOLS["kcg_fmha_bf16"]
        libs.append(L)
    B, H, S, D = shape
    dev = torch.device("cuda:0")
    _settle(dev)
    Q = torch.randn(B, H, S, D, device=dev).to(torch.bfloat16)
    K = torch.randn_like(Q)
    V = torch.randn_like(Q)
    O = torch.empty_like(Q)
    sched = lib.FmhaSched(br=256, bc=64)

    def call(L, causal):
        lib.check(L.kcg_fmha_bf16(Q.data_ptr(), K.data_ptr(), V.data_ptr(), O.data_ptr(), 1, B, H, S, D,
                                  D ** -0.5, causal, ctypes.byref(sched), lib.current_stream()))

    ref = {}
    diff = {}
    for i, L in enumerate(libs):
        for causal in (1, 0):
            O.zero_()
            call(L, causal)
            torch.cuda.synchronize()
            if i == 0:
                ref[causal] = O.clone()
            diff[(i, causal)] = float((O.float() - ref[causal].float()).abs().max())
    best = {}
    for _ in range(rounds):
        for i, L in enumerate(libs):
            for causal in (1, 0):
                ms = _time(lambda: call(L, causal), iters)
                best[(i, causal)] = min(ms, best.get((i, causal), ms))
    print("shape B,H,S,D = %d,%d,%d,%d, bf16, 256-row ping-pong kernel; best of %d rounds of %d launches" % (
        B, H, S, D, rounds, iters))
    print("| build | causal ms | causal TFLOP/s | % of 2500 | non-causal ms | non-causal TFLOP/s | % of 2500 | max abs diff vs default |")
    print("|---|---|---|---|---|---|---|---|")
    for i, p in enumerate(paths):
        name = "default" if i == 0 else os.path.basename(p)[len("libkcg_hip_"):-3]
        fc = 2.0 * B * H * S * S * D / best[(i, 1)] / 1e9
        fn = 4.0 * B * H * S * S * D / best[(i, 0)] / 1e9
        print("| %s | %.4f | %.1f | %.1f | %.4f | %.1f | %.1f | %.3g / %.3g |" % (
            name, best[(i, 1)], fc, 100 * fc / PEAK_BF16_TFLOPS, best[(i, 0)], fn, 100 * fn / PEAK_BF16_TFLOPS,
            diff[(i, 1)], diff[(i, 0)]), flush=True)
    return best


def ops_chain(shape=(1, 32, 2048, 128), iters=30):
    import torch
    from . import lib, ops

    lib.load()
    B, H, S, D = shape
    dev = torch.device("cuda:0")
    _settle(dev)
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

    t = _time(lambda: ops.batched_matmul(Q, K, trans_b=True, out=P), iters)
    mfma_row("BatchedMatmul NT  S = Q.K^T", t, 2.0 * B * H * S * S * D)
    t_qk = t
    # the softmax is timed on scores of realistic spread; it runs in place, so on its own output
    # from the second launch on (timing does not depend on the values)
    P.mul_(D ** -0.5)
    t = _time(lambda: ops.softmax_(P), iters)
    hbm_row("Softmax in place   P = softmax(S)", t, 2.0 * 4 * P.numel())
    t_sm = t
    t = _time(lambda: ops.batched_matmul(P, V, out=O), iters)
    mfma_row("BatchedMatmul NN  O = P.V", t, 2.0 * B * H * S * S * D)
    t_pv = t
    fused = _time(lambda: ops.fmha(Q, K, V, scale=D ** -0.5, out=O), 4 * iters)
    mfma_row("fused FMHA (one kernel)", fused, 4.0 * B * H * S * S * D)
    rows.append(("un-fused chain (three kernels)", t_qk + t_sm + t_pv,
                 "%.1fx the fused kernel" % ((t_qk + t_sm + t_pv) / fused), "-", float("nan")))
    del P
    X = torch.randn(4096, 4096, device=dev)
    Y = torch.empty_like(X)
    t = _time(lambda: ops.relu(X, out=Y), iters)
    hbm_row("Relu 4096 x 4096", t, 2.0 * 4 * X.numel())
    X = torch.randn(16384, 16384, device=dev)
    Y = torch.empty_like(X)
    t = _time(lambda: ops.relu(X, out=Y), iters)
    hbm_row("Relu 16384 x 16384", t, 2.0 * 4 * X.numel())

    print("shape B,H,S,D = %d,%d,%d,%d" % (B, H, S, D))
    print("| operator | ms | rate | bound | % of peak |")
    print("|---|---|---|---|---|")
    for r in rows:
        print(("| %s | %.4f | %s | %s | %.1f |" % r).replace("| nan |", "| - |"))
    return rows
