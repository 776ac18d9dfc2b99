"""Seeded random shapes and schedules through the C ABI, against the CPU oracle.

The fixed-shape parity tests pick sizes around the tile edges by hand; this one draws
extents, schedules, scale and mask from a seeded generator so that combinations nobody
thought of (one row, K = 1, a sequence one short of a tile, a ragged causal diagonal
with the 8-wave workgroup, ...) are covered too.  Tolerances as in the other parity
tests: 1e-4 for fp32, 2e-2 for bf16 inputs.
"""
import numpy as np
import pytest

from conftest import rel_err
from kernelcodegen_amd import inputs

pytestmark = pytest.mark.gpu

GEMM_SCHEDS = [
    None,
    dict(block_m=256, block_n=128, block_k=16, wave_m=64, wave_n=64),
    dict(block_m=256, block_n=128, block_k=32, wave_m=64, wave_n=64),
    dict(block_m=128, block_n=128, block_k=8, wave_m=64, wave_n=64),
    dict(block_m=128, block_n=128, block_k=16, wave_m=64, wave_n=64),
    dict(block_m=128, block_n=128, block_k=32, wave_m=64, wave_n=64),
    dict(block_m=128, block_n=64, block_k=32, wave_m=64, wave_n=32),
    dict(block_m=64, block_n=64, block_k=32, wave_m=32, wave_n=32),
]


def _gpu(x, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).to(dev)


def _gpu_bf16(bits, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(dev).view(torch.bfloat16)


def _extent(rng, tile, hi):
    """An extent near a multiple of `tile` (exactly on it, one off, or anywhere)."""
    kind = rng.integers(0, 4)
    if kind == 0:
        return int(rng.integers(1, hi + 1))
    base = int(rng.integers(1, max(2, hi // tile + 1))) * tile
    return max(1, min(hi, base + (0, -1, 1)[kind - 1]))


def test_matmul_random_shapes(oracle, dev):
    from kernelcodegen_amd import ops
    rng = np.random.default_rng(20240531)
    for case in range(48):
        sched = GEMM_SCHEDS[case % len(GEMM_SCHEDS)]
        bm, bn, bk = (sched or {}).get("block_m", 128), (sched or {}).get("block_n", 128), (sched or {}).get("block_k", 16)
        M, N, K = _extent(rng, bm, 520), _extent(rng, bn, 520), _extent(rng, bk, 200)
        relu = bool(rng.integers(0, 2))
        A = inputs.normal((M, K), 9000 + case, 0)
        B = inputs.normal((K, N), 9000 + case, 1)
        ref = oracle.matmul(A, B)
        if relu:
            ref = oracle.relu(ref)
        C = ops.matmul(_gpu(A, dev), _gpu(B, dev), relu=relu, sched=sched).cpu().numpy()
        assert C.shape == (M, N)
        assert max(rel_err(C, ref)) < 1e-4, (case, M, N, K, relu, sched)


def test_attention_random_shapes(oracle, dev):
    import torch
    from kernelcodegen_amd import ops
    rng = np.random.default_rng(20240601)
    f32_tiles = {128: [(128, 32), (128, 64), (256, 32)], 64: [(128, 32), (128, 64), (256, 32), (256, 64)]}
    for case in range(40):
        D = (64, 128)[int(rng.integers(0, 2))]
        bf16 = case % 2 == 1
        br, bc = ((128, 64), (256, 64))[int(rng.integers(0, 2))] if bf16 else \
            f32_tiles[D][int(rng.integers(0, len(f32_tiles[D])))]
        B, H = int(rng.integers(1, 3)), int(rng.integers(1, 4))
        S = _extent(rng, br if rng.integers(0, 2) else bc, 700)
        causal = bool(rng.integers(0, 2))
        scale = float((D ** -0.5, 1.0, 0.3)[int(rng.integers(0, 3))])
        tag = (case, "bf16" if bf16 else "f32", B, H, S, D, br, bc, causal, scale)
        shape = (B, H, S, D)
        if bf16:
            Qb, Kb, Vb = (inputs.to_bf16_bits(inputs.normal(shape, 9500 + case, i)) for i in range(3))
            Q, K, V = (inputs.bf16_bits_to_f32(x) for x in (Qb, Kb, Vb))
            ref = oracle.fmha(Q, K, V, scale=scale, causal=causal, stable=True)
            O = ops.fmha(_gpu_bf16(Qb, dev), _gpu_bf16(Kb, dev), _gpu_bf16(Vb, dev), scale=scale, causal=causal,
                         out_dtype=torch.float32, sched=dict(br=br, bc=bc)).cpu().numpy()
            assert max(rel_err(O, ref)) < 2e-2, tag
        else:
            Q, K, V = (inputs.normal(shape, 9500 + case, i) for i in range(3))
            ref = oracle.fmha(Q, K, V, scale=scale, causal=causal, stable=True)
            O = ops.fmha(_gpu(Q, dev), _gpu(K, dev), _gpu(V, dev), scale=scale, causal=causal,
                         sched=dict(br=br, bc=bc)).cpu().numpy()
            assert max(rel_err(O, ref)) < 1e-4, tag


def test_batched_matmul_random_shapes(oracle, dev):
    """All four layouts; extents around the tile edges, K around the slice depths, with and
    without 16-byte aligned rows (aligned NN / NT run on the tiled kernel, the rest on the
    generic one)."""
    from kernelcodegen_amd import ops
    rng = np.random.default_rng(20240602)
    for case in range(40):
        ta, tb = bool(case & 1) and case % 5 == 0, bool((case >> 1) & 1)
        batch = tuple(int(x) for x in rng.integers(1, 4, size=int(rng.integers(0, 3))))
        M, N = _extent(rng, 64, 300), _extent(rng, 64, 300)
        K = _extent(rng, 16, 160)
        if case % 3:
            K = max(4, K // 4 * 4)          # 16-byte aligned rows of A (and of B^T)
            if not tb:
                N = max(4, N // 4 * 4)
        A = inputs.normal(batch + ((K, M) if ta else (M, K)), 9700 + case, 0)
        B = inputs.normal(batch + ((N, K) if tb else (K, N)), 9700 + case, 1)
        ref = oracle.batched_matmul(A, ta, B, tb)
        C = ops.batched_matmul(_gpu(A, dev), _gpu(B, dev), trans_a=ta, trans_b=tb).cpu().numpy()
        assert C.shape == ref.shape
        assert max(rel_err(C, ref)) < 1e-4, (case, batch, M, N, K, ta, tb)


def test_repeated_launches_give_the_same_bits(dev):
    """Every kernel here sums in a fixed order, and operand registers are refilled from LDS
    behind the MFMAs that read them: a refill that overtook its reader, or any other race,
    would show as a launch whose bits differ.  Forty launches of each of the main kernels
    against the first one."""
    import torch
    from kernelcodegen_amd import ops
    g = torch.Generator(device="cpu").manual_seed(77)
    cases = []
    A = torch.randn(2048, 1024, generator=g).to(dev)
    B = torch.randn(1024, 1536, generator=g).to(dev)
    cases.append(("matmul 256x128 / default", lambda: ops.matmul(A, B, relu=True)))
    A96 = torch.randn(1536, 1536, generator=g).to(dev)
    B96 = torch.randn(1536, 1536, generator=g).to(dev)
    cases.append(("matmul 96x96", lambda: ops.matmul(A96, B96)))
    cases.append(("matmul 96x64", lambda: ops.matmul(A96[:1152, :1024].contiguous(), B96[:1024, :1152].contiguous())))
    As = torch.randn(4096, 768, generator=g).to(dev)
    Bs = torch.randn(768, 4096, generator=g).to(dev)
    cases.append(("matmul streaming", lambda: ops.matmul(As, Bs)))
    Q, K, V = (torch.randn(2, 8, 2048, 128, generator=g).to(dev) for _ in range(3))
    Qb, Kb, Vb = (t.to(torch.bfloat16) for t in (Q, K, V))
    Qs, Ks, Vs = (t[:, :, :1024].contiguous() for t in (Q, K, V))
    for causal in (False, True):
        cases.append(("fmha f32 causal=%d" % causal, lambda c=causal: ops.fmha(Qs, Ks, Vs, scale=0.088, causal=c)))
        cases.append(("fmha bf16 ping-pong causal=%d" % causal,
                      lambda c=causal: ops.fmha(Qb, Kb, Vb, scale=0.088, causal=c, sched=dict(br=256, bc=64))))
        cases.append(("fmha bf16 128-row causal=%d" % causal,
                      lambda c=causal: ops.fmha(Qb, Kb, Vb, scale=0.088, causal=c, sched=dict(br=128, bc=64))))
    for name, fn in cases:
        first = fn()
        assert bool(torch.isfinite(first.float()).all()), name
        for _ in range(40):
            assert torch.equal(fn(), first), name
