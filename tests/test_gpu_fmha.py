"""GPU parity of the fused attention kernels against the CPU oracle.

Tolerances (BASELINE.json north_star): max relative error 1e-4 for fp32 and
2e-2 for bf16 inputs, on both figures of conftest.rel_err.  The oracle is run
with the row-max shift (stable=True), which tests/test_oracle.py shows equal to
the reference's literal exp(x)/sum(exp(x)) form.
"""
import numpy as np
import pytest

from conftest import rel_err
from kernelcodegen_amd import inputs

pytestmark = pytest.mark.gpu
TOL_F32 = 1e-4
TOL_BF16 = 2e-2


def _gpu(x, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).to(dev)


def _gpu_bf16(bits, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(dev).view(torch.bfloat16)


def _p_rounding_bound(Qb, Kb, Vb, scale, causal, out_bf16):
    """Per-element bound on |O_kernel - O_fp32| for bf16 inputs given as bit patterns.

    The kernel rounds the softmax weights to bf16 before P.V (unit roundoff 2^-8) and
    normalises by the sum of the rounded weights: O~ = sum_j p_j (1 + d_j) v_j / sum_j p_j (1 + d_j)
    with |d_j| <= 2^-8, so |O~ - O| <= 2^-8 (sum_j P_ij |v_jd| + |O_id|) to first order, P the
    normalised weights.  Added: 2^-8 |O| when the output is rounded to bf16, and a slack of
    5e-4 (sum_j P_ij |v_jd| + |O_id|) + 1e-6 for fp32 accumulation order, the exponential and
    the second-order terms.  P is evaluated here in float64 from the same inputs."""
    q, k, v = (inputs.bf16_bits_to_f32(t).astype(np.float64) for t in (Qb, Kb, Vb))
    B, H, S, D = q.shape
    bound = np.empty((B, H, S, D))
    tri = np.triu(np.ones((S, S), dtype=bool), 1) if causal else None
    for b in range(B):
        for h in range(H):
            s = (q[b, h] @ k[b, h].T) * scale
            if causal:
                s[tri] = -np.inf
            s -= s.max(axis=1, keepdims=True)
            p = np.exp(s)
            p /= p.sum(axis=1, keepdims=True)
            pv_abs = p @ np.abs(v[b, h])
            o_abs = np.abs(p @ v[b, h])
            bound[b, h] = (2.0 ** -8 + 5e-4) * (pv_abs + o_abs) + (2.0 ** -8 * o_abs if out_bf16 else 0.0) + 1e-6
    return bound


SHAPES = [(1, 2, 128, 128), (1, 2, 256, 64), (2, 3, 200, 128), (1, 1, 77, 64), (1, 1, 1, 128),
          (1, 2, 33, 64), (1, 2, 512, 128), (1, 1, 640, 64)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("tile", [(128, 32), (128, 64), (256, 32)])
def test_f32_parity(oracle, dev, shape, causal, tile):
    from kernelcodegen_amd import ops
    B, H, S, D = shape
    br, bc = tile
    Q, K, V = (inputs.normal(shape, 201, i) for i in range(3))
    for scale in (D ** -0.5, 1.0 / 3):
        ref = oracle.fmha(Q, K, V, scale=scale, causal=causal, stable=True)
        O = ops.fmha(_gpu(Q, dev), _gpu(K, dev), _gpu(V, dev), scale=scale, causal=causal,
                     sched=dict(br=br, bc=bc)).cpu().numpy()
        assert max(rel_err(O, ref)) < TOL_F32


@pytest.mark.parametrize("causal", [False, True])
def test_f32_rising_row_maximum(oracle, dev, causal):
    """Logits that climb along the key axis: by a few units per tile for some rows (the
    reference maximum of the online softmax stays behind the true one) and by far more
    than the rescale threshold for others (it is raised again and again), plus rows whose
    largest logit comes first."""
    from kernelcodegen_amd import ops
    B, H, S, D = 1, 2, 384, 64
    rng = np.random.default_rng(77)
    K = rng.standard_normal((B, H, S, D)).astype(np.float32)
    V = rng.standard_normal((B, H, S, D)).astype(np.float32)
    Q = rng.standard_normal((B, H, S, D)).astype(np.float32) * np.float32(0.1)
    ramp = np.linspace(0.0, 1.0, S, dtype=np.float32)
    K[..., 0] = 60.0 * ramp          # logit contribution q0 * k0 * scale
    Q[:, :, 0::3, 0] = 1.0           # climbs by ~60 over the sweep: repeated rescales
    Q[:, :, 1::3, 0] = 0.05          # climbs by ~3: never exceeds the threshold after tile 0
    Q[:, :, 2::3, 0] = -1.0          # falls: the first tile holds the maximum
    ref = oracle.fmha(Q, K, V, scale=1.0, causal=causal, stable=True)
    for tile in ((128, 32), (128, 64), (256, 32)):
        O = ops.fmha(_gpu(Q, dev), _gpu(K, dev), _gpu(V, dev), scale=1.0, causal=causal,
                     sched=dict(br=tile[0], bc=tile[1])).cpu().numpy()
        assert max(rel_err(O, ref)) < TOL_F32, tile


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("which", [0, 1])
def test_large_logits_in_one_half_of_the_wave(oracle, dev, dtype, which):
    """The two halves of a wave hold different keys of the same query row (keys with
    k % 8 < 4 in the lower half, the others in the upper half) and must agree on the row
    maximum.  Here only one half's keys carry large logits (100 above the rest: 2^144 if
    the reference were not raised), in every tile; a maximum taken from the other half
    alone overflows the exponentials."""
    import torch
    from kernelcodegen_amd import ops
    B, H, S, D = 1, 2, 320, 64
    rng = np.random.default_rng(91)
    Q = (rng.standard_normal((B, H, S, D)) * 0.05).astype(np.float32)
    K = (rng.standard_normal((B, H, S, D)) * 0.05).astype(np.float32)
    V = (rng.standard_normal((B, H, S, D)) + 2.0).astype(np.float32)   # (a mean of many V rows: keep it away from 0)
    keys = np.arange(S)
    big = (keys % 8 >= 4) if which else (keys % 8 < 4)
    Q[..., 0] = 10.0
    K[..., 0] = np.where(big, 10.0, 0.0)
    for causal in (False, True):
        if dtype == "f32":
            ref = oracle.fmha(Q, K, V, scale=1.0, causal=causal, stable=True)
            for tile in ((128, 32), (128, 64), (256, 32)):
                O = ops.fmha(_gpu(Q, dev), _gpu(K, dev), _gpu(V, dev), scale=1.0, causal=causal,
                             sched=dict(br=tile[0], bc=tile[1])).cpu().numpy()
                assert np.isfinite(O).all(), tile
                assert max(rel_err(O, ref)) < TOL_F32, tile
        else:
            qb, kb, vb = (inputs.to_bf16_bits(t) for t in (Q, K, V))
            ref = oracle.fmha(qb, kb, vb, scale=1.0, causal=causal, stable=True)
            for br in (128, 256):
                O = ops.fmha(_gpu_bf16(qb, dev), _gpu_bf16(kb, dev), _gpu_bf16(vb, dev), scale=1.0,
                             causal=causal, out_dtype=torch.float32, sched=dict(br=br, bc=64)).cpu().numpy()
                assert np.isfinite(O).all(), br
                assert max(rel_err(O, ref)) < TOL_BF16, br


@pytest.mark.parametrize("shape", [(1, 2, 128, 128), (2, 3, 200, 128), (1, 1, 1, 128), (1, 2, 512, 128)])
@pytest.mark.parametrize("causal", [False, True])
def test_reference_tile_at_head_dim_128(oracle, dev, shape, causal):
    """Br 64 x Bc 128: the tile the reference's own table gives at Hd = 128 (Br = 8192 / Hd,
    Bc = 8192 / Br; include/KernelCodeGen.h:38-41, src/Optimizer/Optimizer.cc:1136-1144), as a
    named schedule of both entry points (two waves of 32 query rows, 128-key tiles)."""
    import torch
    from kernelcodegen_amd import ops
    B, H, S, D = shape
    Q, K, V = (inputs.normal(shape, 209, i) for i in range(3))
    scale = D ** -0.5
    ref = oracle.fmha(Q, K, V, scale=scale, causal=causal, stable=True)
    O = ops.fmha(_gpu(Q, dev), _gpu(K, dev), _gpu(V, dev), scale=scale, causal=causal,
                 sched=dict(br=64, bc=128)).cpu().numpy()
    assert max(rel_err(O, ref)) < TOL_F32
    qb, kb, vb = (inputs.to_bf16_bits(t) for t in (Q, K, V))
    refb = oracle.fmha(qb, kb, vb, scale=scale, causal=causal, stable=True)
    Ob = ops.fmha(_gpu_bf16(qb, dev), _gpu_bf16(kb, dev), _gpu_bf16(vb, dev), scale=scale, causal=causal,
                  out_dtype=torch.float32, sched=dict(br=64, bc=128)).cpu().numpy()
    assert max(rel_err(Ob, refb)) < TOL_BF16
    # at head dim 64 the reference's table gives 128 x 64, which both entry points build;
    # 64 x 128 is refused there
    from kernelcodegen_amd.lib import KcgError
    q64 = torch.zeros(1, 1, 64, 64, device=dev)
    with pytest.raises(KcgError) as e:
        ops.fmha(q64, q64, q64, sched=dict(br=64, bc=128))
    assert e.value.status == 4


def test_f32_reference_graph_scale_one(oracle, dev):
    """scale = 1, no mask: the reference's own three-operator graph, literal softmax."""
    from kernelcodegen_amd import ops
    shape = (2, 2, 160, 64)
    Q, K, V = (inputs.normal(shape, 202, i) for i in range(3))
    Q = (Q * np.float32(0.25)).astype(np.float32)       # keep exp(x) in range for the literal form
    ref = oracle.fmha(Q, K, V, scale=1.0, causal=False, stable=False)
    graph = oracle.batched_matmul(oracle.softmax(oracle.batched_matmul(Q, 0, K, 1)), 0, V, 0)
    assert np.array_equal(ref, graph)
    O = ops.fmha(_gpu(Q, dev), _gpu(K, dev), _gpu(V, dev), scale=1.0, causal=False).cpu().numpy()
    assert max(rel_err(O, ref)) < TOL_F32


@pytest.mark.parametrize("shape", SHAPES + [(1, 1, 1024, 128)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("br", [128, 256])
def test_bf16_parity(oracle, dev, shape, causal, br):
    import torch
    from kernelcodegen_amd import ops
    B, H, S, D = shape
    Q, K, V = (inputs.to_bf16_bits(inputs.normal(shape, 203, i)) for i in range(3))
    scale = D ** -0.5
    ref = oracle.fmha(Q, K, V, scale=scale, causal=causal, stable=True)
    tq, tk, tv = (_gpu_bf16(t, dev) for t in (Q, K, V))
    for odt in (torch.bfloat16, torch.float32):
        O = ops.fmha(tq, tk, tv, scale=scale, causal=causal, out_dtype=odt,
                     sched=dict(br=br, bc=64))
        assert O.dtype == odt
        assert max(rel_err(O.float().cpu().numpy(), ref)) < TOL_BF16


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(4, 80, 600, 128), (32, 24, 450, 128)])
def test_bf16_streams_of_ragged_work_items(oracle, dev, shape, causal):
    """Default schedule on launches with two to four 256-row work items per CU, whose sequence
    length divides neither the key tile nor the query block: every persistent workgroup chains
    several items (causal: pairs of blocks, the second of a pair partly beyond the sequence),
    each ends on a ragged key tile that is loaded through registers, and waves whose rows lie
    beyond the sequence skip their stores."""
    import ctypes
    import torch
    from kernelcodegen_amd import lib, ops
    B, H, S, D = shape
    info = lib.LaunchInfo()
    assert lib.load().kcg_fmha_query(ops.BF16, B, H, S, D, int(causal), None, ctypes.byref(info)) == 0
    assert b"pingpong" in info.kernel and info.grid[0] == 256
    Q, K, V = (inputs.to_bf16_bits(inputs.normal(shape, 207, i)) for i in range(3))
    scale = D ** -0.5
    ref = oracle.fmha(Q, K, V, scale=scale, causal=causal, stable=True)
    O = ops.fmha(_gpu_bf16(Q, dev), _gpu_bf16(K, dev), _gpu_bf16(V, dev), scale=scale, causal=causal,
                 out_dtype=torch.float32).cpu().numpy()
    assert rel_err(O, ref)[1] < TOL_BF16
    # Every element of every row against the bound that rounding P to bf16 implies (the only
    # stated deviation of the kernel from the fp32 evaluation, see _p_rounding_bound): a wrong
    # mask, a dropped or doubled key or a stale reference maximum breaks it on the early rows.
    bound = _p_rounding_bound(Q, K, V, scale, causal, out_bf16=False)
    excess = np.abs(O.astype(np.float64) - ref) - bound
    assert excess.max() <= 0.0, np.unravel_index(excess.argmax(), excess.shape)
    # The RMS-floored figure holds from query row 16 on in the causal case: a row that sees two
    # or three keys is a weighted sum of as many V rows with bf16-rounded weights, an error of
    # up to 2^-8 |v| that does not average out, while the RMS of the whole output is set by the
    # late rows, which average hundreds of V rows.  Over 320 to 768 heads the largest such
    # element reaches 2.4e-2 of that RMS (inside the bound above), for both kernels alike.
    first = 16 if causal else 0
    assert rel_err(O[:, :, first:], ref[:, :, first:])[0] < TOL_BF16


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_closed_forms(dev, dtype):
    import torch
    from kernelcodegen_amd import ops
    tdt = torch.float32 if dtype == "f32" else torch.bfloat16
    tol = 1e-5 if dtype == "f32" else 1e-2
    B, H, S, D = 1, 2, 300, 128
    g = torch.Generator(device="cpu").manual_seed(5)
    Q = torch.randn(B, H, S, D, generator=g).to(dev).to(tdt)
    K = torch.randn(B, H, S, D, generator=g).to(dev).to(tdt)
    V = torch.randn(B, H, S, D, generator=g).to(dev).to(tdt)
    # V = 1 -> O = 1 (softmax rows sum to one)
    for causal in (False, True):
        O = ops.fmha(Q, K, torch.ones_like(V), scale=0.1, causal=causal, out_dtype=torch.float32)
        assert float((O.float() - 1).abs().max()) < tol
    # K = 0 -> uniform weights: mean of V, or prefix mean when causal
    Z = torch.zeros_like(K)
    O = ops.fmha(Q, Z, V, scale=1.0, causal=False, out_dtype=torch.float32).float()
    mean = V.float().mean(2, keepdim=True).expand_as(O)
    assert float((O - mean).abs().max()) < (1e-5 if dtype == "f32" else 3e-3)
    Oc = ops.fmha(Q, Z, V, scale=1.0, causal=True, out_dtype=torch.float32).float()
    prefix = V.float().cumsum(2) / torch.arange(1, S + 1, device=dev).view(1, 1, S, 1)
    assert float((Oc - prefix).abs().max()) < (1e-5 if dtype == "f32" else 1.5e-2)
    # causal: row 0 sees key 0 only
    assert float((Oc[:, :, 0] - V.float()[:, :, 0]).abs().max()) < (1e-6 if dtype == "f32" else 1e-2)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_causal_future_keys_do_not_leak_and_heads_independent(dev, dtype):
    import torch
    from kernelcodegen_amd import ops
    tdt = torch.float32 if dtype == "f32" else torch.bfloat16
    B, H, S, D = 2, 3, 257, 64
    g = torch.Generator(device="cpu").manual_seed(6)
    Q, K, V = (torch.randn(B, H, S, D, generator=g).to(dev).to(tdt) for _ in range(3))
    O = ops.fmha(Q, K, V, scale=0.2, causal=True)
    K2, V2 = K.clone(), V.clone()
    K2[:, :, 130:] += 4
    V2[:, :, 130:] -= 2
    O2 = ops.fmha(Q, K2, V2, scale=0.2, causal=True)
    assert torch.equal(O2[:, :, :130], O[:, :, :130])
    assert not torch.equal(O2[:, :, 130:], O[:, :, 130:])
    perm = torch.tensor([2, 0, 1], device=dev)
    Op = ops.fmha(Q[:, perm].contiguous(), K[:, perm].contiguous(), V[:, perm].contiguous(),
                  scale=0.2, causal=True)
    assert torch.equal(Op, O[:, perm])


def test_single_tile_vs_repeated_tiles(dev):
    """Keys repeated 4x give the same softmax-weighted mean: exercises the
    running max / sum / rescale across K/V tiles against the single-tile case."""
    import torch
    from kernelcodegen_amd import ops
    g = torch.Generator(device="cpu").manual_seed(7)
    Q = torch.randn(1, 2, 64, 128, generator=g).to(dev)
    K = torch.randn(1, 2, 64, 128, generator=g).to(dev)
    V = torch.randn(1, 2, 64, 128, generator=g).to(dev)
    Qp = torch.cat([Q] * 4, 2).contiguous()
    O1 = ops.fmha(Q, K, V, scale=0.1)
    O4 = ops.fmha(Qp, torch.cat([K] * 4, 2).contiguous(), torch.cat([V] * 4, 2).contiguous(), scale=0.1)
    assert float((O4[:, :, :64] - O1).abs().max()) < 1e-5


def test_cfg3_full_size(oracle, dev):
    """configs[3]: fp32, B=1 H=32 S=2048 D=128, non-causal; sampled query rows."""
    from kernelcodegen_amd import ops
    c = inputs.config_inputs(3)
    O = ops.fmha(_gpu(c["Q"], dev), _gpu(c["K"], dev), _gpu(c["V"], dev), scale=c["scale"],
                 causal=False).cpu().numpy()
    for r0, r1 in [(0, 16), (1000, 1024), (2040, 2048)]:
        ref = oracle.fmha(c["Q"], c["K"], c["V"], scale=c["scale"], causal=False, stable=True,
                          rows=(r0, r1))
        assert max(rel_err(O[:, :, r0:r1], ref)) < TOL_F32


def test_reference_demo_shape_full_size(oracle, dev):
    """The reference's own attention demo (test/test.cc:64-90): [8, 32, 2048, 64] fp32, the
    literal graph BatchedMatmul(Q, K^T) -> Softmax -> BatchedMatmul(P, V) with scale 1 and
    no mask.  Full size on the GPU; sampled rows of four (batch, head) pairs against the
    oracle's literal exp(x) / sum(exp(x)) form (stable=False).  Q is drawn with standard
    deviation 0.25 so that the literal form stays finite at scale 1 (logits ~ N(0, 4))."""
    from kernelcodegen_amd import ops
    B, H, S, D = 8, 32, 2048, 64
    Q = inputs.normal((B, H, S, D), 208, 0, std=0.25)
    K, V = (inputs.normal((B, H, S, D), 208, i) for i in (1, 2))
    O = ops.fmha(_gpu(Q, dev), _gpu(K, dev), _gpu(V, dev), scale=1.0, causal=False).cpu().numpy()
    assert np.isfinite(O).all()
    for b, h in ((0, 0), (3, 17), (7, 31), (5, 8)):
        for r0 in (0, 1021, 2048 - 64):
            ref = oracle.fmha(Q[b:b + 1, h:h + 1], K[b:b + 1, h:h + 1], V[b:b + 1, h:h + 1], scale=1.0, causal=False,
                              stable=False, rows=(r0, r0 + 64))
            assert max(rel_err(O[b:b + 1, h:h + 1, r0:r0 + 64], ref)) < TOL_F32, (b, h, r0)


def test_cfg4_full_size(oracle, dev):
    """configs[4]: bf16, B=4 H=32 S=4096 D=128, causal; sampled query rows and
    the V = 1 property over the whole output."""
    import torch
    from kernelcodegen_amd import ops
    c = inputs.config_inputs(4)
    tq, tk, tv = (_gpu_bf16(c[k], dev) for k in "QKV")
    for br in (128, 256):
        O = ops.fmha(tq, tk, tv, scale=c["scale"], causal=True, sched=dict(br=br, bc=64))
        Oh = O.float().cpu().numpy()
        for r0, r1 in [(0, 8), (2043, 2051), (4088, 4096)]:
            ref = oracle.fmha(c["Q"], c["K"], c["V"], scale=c["scale"], causal=True, stable=True,
                              rows=(r0, r1))
            assert max(rel_err(Oh[:, :, r0:r1], ref)) < TOL_BF16
        ones = ops.fmha(tq, tk, torch.ones_like(tv), scale=c["scale"], causal=True,
                        out_dtype=torch.float32, sched=dict(br=br, bc=64))
        assert float((ones - 1).abs().max()) < 1e-2


def test_errors(dev):
    import torch
    from kernelcodegen_amd import ops
    from kernelcodegen_amd.lib import KcgError
    q = torch.zeros(1, 1, 64, 96, device=dev)
    with pytest.raises(KcgError) as e:
        ops.fmha(q, q, q)
    assert e.value.status == 3
    q = torch.zeros(1, 1, 64, 64, device=dev)
    with pytest.raises(ValueError):
        ops.fmha(q, q[:, :, :32], q)


@pytest.mark.parametrize("scale", [-0.2, 0.0])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_non_positive_scale(oracle, dev, scale, dtype):
    """scale <= 0 takes the kernels' general softmax path (the fast path needs scale > 0)."""
    from kernelcodegen_amd import ops
    shape = (1, 2, 200, 128)
    Q, K, V = (inputs.normal(shape, 205, i) for i in range(3))
    if dtype == "bf16":
        Qb, Kb, Vb = (inputs.to_bf16_bits(t) for t in (Q, K, V))
        ref = oracle.fmha(Qb, Kb, Vb, scale=scale, causal=True, stable=True)
        O = ops.fmha(*(_gpu_bf16(t, dev) for t in (Qb, Kb, Vb)), scale=scale, causal=True)
        assert max(rel_err(O.float().cpu().numpy(), ref)) < TOL_BF16
    else:
        ref = oracle.fmha(Q, K, V, scale=scale, causal=True, stable=True)
        O = ops.fmha(*(_gpu(t, dev) for t in (Q, K, V)), scale=scale, causal=True)
        assert max(rel_err(O.cpu().numpy(), ref)) < TOL_F32


@pytest.mark.parametrize("sched", [None, dict(br=128, bc=64), dict(br=256, bc=64)])
def test_bf16_default_schedule_and_large_logits(oracle, dev, sched):
    """A logit scale large enough that the running maximum keeps growing, which exercises the
    lazy rescale, on the default schedule (18 work items here: the 128-row kernel) and on
    both block sizes by name (256: the ping-pong kernel's mid-pass raise of the reference)."""
    import torch
    from kernelcodegen_amd import ops
    shape = (1, 2, 2048 + 70, 128)
    Q, K, V = (inputs.to_bf16_bits(inputs.normal(shape, 206, i)) for i in range(3))
    tq, tk, tv = (_gpu_bf16(t, dev) for t in (Q, K, V))
    for scale, causal in [(128 ** -0.5, True), (0.75, False), (0.75, True)]:
        ref = oracle.fmha(Q, K, V, scale=scale, causal=causal, stable=True, rows=(1990, 2118))
        O = ops.fmha(tq, tk, tv, scale=scale, causal=causal, out_dtype=torch.float32, sched=sched)
        assert max(rel_err(O[:, :, 1990:2118].cpu().numpy(), ref)) < TOL_BF16


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("br", [128, 256])
def test_bf16_rising_row_maximum(oracle, dev, causal, br, D):
    """bf16 counterpart of test_f32_rising_row_maximum.  Every third query row climbs by ~60
    over the sweep, its neighbours by ~3 or not at all, so that within one wave some rows take
    the path that raises the reference maximum and redoes the tile (sum of the tile's
    exponentials above 2^8) while others stay on the fast path: a divergent redo with the
    half-wave exchange inside it.  Six key tiles for the 256-row kernel's mid-pass raise."""
    import torch
    from kernelcodegen_amd import ops
    B, H, S = 1, 2, 384
    rng = np.random.default_rng(78)
    K = rng.standard_normal((B, H, S, D)).astype(np.float32)
    V = rng.standard_normal((B, H, S, D)).astype(np.float32)
    Q = rng.standard_normal((B, H, S, D)).astype(np.float32) * np.float32(0.1)
    K[..., 0] = 60.0 * np.linspace(0.0, 1.0, S, dtype=np.float32)
    Q[:, :, 0::3, 0] = 1.0
    Q[:, :, 1::3, 0] = 0.05
    Q[:, :, 2::3, 0] = -1.0
    qb, kb, vb = (inputs.to_bf16_bits(t) for t in (Q, K, V))
    ref = oracle.fmha(qb, kb, vb, scale=1.0, causal=causal, stable=True)
    O = ops.fmha(_gpu_bf16(qb, dev), _gpu_bf16(kb, dev), _gpu_bf16(vb, dev), scale=1.0, causal=causal,
                 out_dtype=torch.float32, sched=dict(br=br, bc=64)).cpu().numpy()
    assert np.isfinite(O).all()
    excess = np.abs(O.astype(np.float64) - ref) - _p_rounding_bound(qb, kb, vb, 1.0, causal, out_bf16=False)
    assert excess.max() <= 0.0, np.unravel_index(excess.argmax(), excess.shape)
    assert rel_err(O, ref)[1] < TOL_BF16


@pytest.mark.skip(reason="never run: the matmul test of the same size class ended in a GPU memory fault "
                         "whose cause is not found")
@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_tensors_beyond_two_to_the_31_elements(dev, dtype):
    """Q, K, V, O of 2.15e9 elements each (B=64, H=64, S=4096, D=128): the last heads, whose
    element offsets exceed 2^31, must equal the same heads run on their own."""
    import torch
    from kernelcodegen_amd import ops
    B, H, S, D = 64, 64, 4096, 128
    assert B * H * S * D > 2 ** 31
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    Q = torch.empty(B, H, S, D, device=dev, dtype=td).normal_()
    K = torch.empty_like(Q).normal_()
    V = torch.empty_like(Q).normal_()
    O = ops.fmha(Q, K, V, scale=D ** -0.5, causal=True)
    last = ops.fmha(Q[-1:, -2:].contiguous(), K[-1:, -2:].contiguous(), V[-1:, -2:].contiguous(),
                    scale=D ** -0.5, causal=True)
    tol = 2e-2 if dtype == "bf16" else 1e-4
    assert float((O[-1:, -2:].float() - last.float()).abs().max()) < tol
    assert bool(torch.isfinite(O[-1].float()).all())
