"""GPU parity of the un-fused operators (Relu, BatchedMatmul, Softmax) and of
the three-kernel attention graph against the fused kernel."""
import numpy as np
import pytest

from conftest import rel_err
from kernelcodegen_amd import inputs

pytestmark = pytest.mark.gpu


def _gpu(x, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).to(dev)


@pytest.mark.parametrize("n", [1, 3, 4, 1023, 4096, 1 << 20, (1 << 20) + 3])
def test_relu_bit_exact(oracle, dev, n):
    from kernelcodegen_amd import ops
    x = inputs.normal((n,), 301, 0)
    if n >= 8:
        x[:8] = np.array([-0.0, 0.0, np.nan, np.inf, -np.inf, -1e-40, 1e-40, -5], np.float32)
    ref = oracle.relu(x)
    y = ops.relu(_gpu(x, dev)).cpu().numpy()
    assert np.array_equal(y, ref, equal_nan=True)
    assert np.array_equal(np.signbit(y), np.signbit(ref))
    t = _gpu(x, dev)
    assert ops.relu(t, inplace=True).data_ptr() == t.data_ptr()
    assert np.array_equal(t.cpu().numpy(), ref, equal_nan=True)
    if n > 1:
        # misaligned views take the scalar path
        t = _gpu(np.concatenate([[0], x]).astype(np.float32), dev)[1:]
        assert np.array_equal(ops.relu(t).cpu().numpy(), ref, equal_nan=True)


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("dims", [((2, 3), 10, 5, 7), ((4,), 64, 64, 16), ((1, 2), 130, 77, 33), ((), 200, 96, 64)])
def test_batched_matmul(oracle, dev, ta, tb, dims):
    from kernelcodegen_amd import ops
    batch, M, N, K = dims
    A = inputs.normal(batch + ((K, M) if ta else (M, K)), 302, 0)
    B = inputs.normal(batch + ((N, K) if tb else (K, N)), 302, 1)
    ref = oracle.batched_matmul(A, ta, B, tb)
    C = ops.batched_matmul(_gpu(A, dev), _gpu(B, dev), trans_a=ta, trans_b=tb).cpu().numpy()
    assert C.shape == ref.shape
    assert max(rel_err(C, ref)) < 1e-4


# Shapes that the direct-load matmul kernel takes (rows 16-byte aligned, K at least one
# slice): full tiles, ragged edges, K with 1..7 slices and a partial last one, a B^T whose
# row count is not a multiple of 4, every default tile of the chooser.
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("dims", [
    ((2, 2), 256, 128, 128),      # attention-like, full tiles
    ((3,), 128, 256, 32),         # one slice
    ((2,), 256, 256, 224),        # seven slices of 32
    ((5,), 130, 132, 100),        # ragged everywhere, partial last slice
    ((1, 3), 64, 64, 64),         # smallest tile
    ((2,), 1, 4, 36),             # one row
    ((2,), 300, 72, 40),          # N = 72 (multiple of 4 only)
    ((2,), 96, 77, 64),           # N = 77: only the transposed B is 16-byte aligned per row
    ((40,), 512, 128, 64),        # many matrices: 256 x 128 tiles
])
def test_batched_matmul_direct_load(oracle, dev, tb, dims):
    from kernelcodegen_amd import ops
    batch, M, N, K = dims
    A = inputs.normal(batch + (M, K), 312, 0)
    B = inputs.normal(batch + ((N, K) if tb else (K, N)), 312, 1)
    ref = oracle.batched_matmul(A, False, B, tb)
    C = ops.batched_matmul(_gpu(A, dev), _gpu(B, dev), trans_b=tb).cpu().numpy()
    assert C.shape == ref.shape
    assert max(rel_err(C, ref)) < 1e-4


# Shapes of the streaming kernel (whole 256 x 128 tiles, K a multiple of 64 up to 1024, at least
# two tiles per compute unit): resident workgroups chain their tiles into one stream of K
# slices and write each tile's C during the next tile's first slices.  K = 64 and K = 128 are
# the two store schedules (4 and 8 slices carry stores), 192 and 320 add whole rounds of the
# slice ring behind them, 1024 is the longest K it takes; tile counts that 8 XCDs x 32
# workgroups do not divide leave workgroups with lists of different lengths.
@pytest.mark.parametrize("tb", [True, False])
@pytest.mark.parametrize("dims", [
    ((16,), 1024, 1024, 128),
    ((9,), 1280, 1664, 64),
    ((3, 3), 1280, 1664, 192),
    ((20,), 768, 1152, 320),
    ((5,), 2560, 1408, 1024),
])
def test_batched_matmul_streaming_kernel(oracle, dev, tb, dims):
    import torch
    from kernelcodegen_amd import ops
    batch, M, N, K = dims
    A = inputs.normal(batch + (M, K), 313, 0)
    B = inputs.normal(batch + ((N, K) if tb else (K, N)), 313, 1)
    ref = oracle.batched_matmul(A, False, B, tb)
    count = int(np.prod(batch)) * M * N
    buf = torch.full((count + 1024,), -7.0, device=dev)
    C = buf[:count].view(batch + (M, N))
    ops.batched_matmul(_gpu(A, dev), _gpu(B, dev), trans_b=tb, out=C)
    assert bool((buf[count:] == -7.0).all())
    assert max(rel_err(C.cpu().numpy(), ref)) < 1e-4


def test_streaming_kernel_result_is_the_tiled_kernels(dev):
    """The attention-score product at the configs[3] shape on the streaming kernel, against the
    same product computed one matrix at a time (32 tiles per call: the one-tile-per-workgroup
    kernel).  Same tile, same slice order, same MFMA operand mapping: the results are equal
    bit for bit."""
    import torch
    from kernelcodegen_amd import ops
    H, S, D = 32, 2048, 128
    Q = torch.randn(H, S, D, device=dev)
    K = torch.randn(H, S, D, device=dev)
    P = ops.batched_matmul(Q, K, trans_b=True)
    for h in (0, 13, 31):
        one = ops.batched_matmul(Q[h:h + 1], K[h:h + 1], trans_b=True)
        assert torch.equal(P[h], one[0])


@pytest.mark.parametrize("K", [32, 3])
def test_batched_matmul_more_matrices_than_one_launch_takes(dev, K):
    """70000 small matrices: more than the 65535 a launch holds in its grid (K = 32 on the
    tiled kernel, K = 3 on the generic one)."""
    import torch
    from kernelcodegen_amd import ops
    batch, M, N = 70000, 4, 4
    A = torch.randn(batch, M, K, device=dev)
    B = torch.randn(batch, K, N, device=dev)
    C = ops.batched_matmul(A, B)
    ref = torch.einsum("bmk,bkn->bmn", A.double(), B.double())
    assert float((C.double() - ref).abs().max()) < 1e-4


def test_batched_matmul_output_is_not_touched_outside_c(dev):
    """Ragged tiles of the batched kernel store nothing beyond each matrix of C."""
    import torch
    from kernelcodegen_amd import ops
    batch, M, N, K = 3, 130, 132, 100
    A = torch.randn(batch, M, K, device=dev)
    Bt = torch.randn(batch, N, K, device=dev)
    buf = torch.full((batch * M * N + 512,), -7.0, device=dev)
    C = buf[:batch * M * N].view(batch, M, N)
    ops.batched_matmul(A, Bt, trans_b=True, out=C)
    assert bool((buf[batch * M * N:] == -7.0).all())
    ref = torch.matmul(A.double(), Bt.double().transpose(1, 2))
    assert float((C.double() - ref).abs().max()) < 1e-3


@pytest.mark.parametrize("shape", [(4, 9, 33), (2, 2, 64, 64), (3, 1000), (5, 1), (2, 5000), (7, 4), (9, 256),
                                   (6, 260), (5, 1024), (3, 1028), (5, 2048), (3, 2052), (2, 4096), (3, 8192),
                                   (2, 8196), (1, 3, 100), (3, 1001), (2, 2047), (3, 4099), (2, 8191), (2, 8193),
                                   (2, 16384), (3, 12000), (2, 32768), (2, 32772), (1, 40000)])
def test_softmax(oracle, dev, shape):
    from kernelcodegen_amd import ops
    x = inputs.normal(shape, 303, 0) * np.float32(2)
    ref = oracle.softmax(x)
    t = _gpu(x, dev)
    y = ops.softmax_(t)
    assert y.data_ptr() == t.data_ptr()
    y = y.cpu().numpy()
    assert max(rel_err(y, ref)) < 1e-4
    assert np.allclose(y.sum(-1), 1, atol=1e-5)


def test_softmax_rows_with_large_and_infinite_entries(dev):
    """x = 100 would overflow exp() in the reference's un-shifted form; the shifted form
    stays finite.  A row of -inf except one entry is a one-hot."""
    import torch
    from kernelcodegen_amd import ops
    for n in (8, 512, 2048, 6000):
        x = torch.full((4, n), 100.0, device=dev)
        x[1] = -float("inf")
        x[1, n // 2] = 3.0
        x[2, 0] = 130.0
        y = ops.softmax_(x.clone())
        assert torch.allclose(y[0], torch.full((n,), 1.0 / n, device=dev), rtol=1e-5)
        assert float(y[1, n // 2]) == 1.0 and float(y[1].sum()) == 1.0
        assert abs(float(y[2, 0]) - 1.0) < 1e-6
        assert bool(torch.isfinite(y).all())


def test_unfused_graph_matches_fused_kernel(oracle, dev):
    """BatchedMatmul(Q,K^T) -> Softmax -> BatchedMatmul(P,V) run as three kernels
    equals the fused kernel and the oracle (the reference's test graph,
    test/test.cc:88-90, scale 1 and no mask)."""
    from kernelcodegen_amd import ops
    shape = (2, 4, 256, 64)
    Q, K, V = (inputs.normal(shape, 304, i) for i in range(3))
    Q = (Q * np.float32(0.25)).astype(np.float32)
    dQ, dK, dV = (_gpu(t, dev) for t in (Q, K, V))
    S = ops.batched_matmul(dQ, dK, trans_b=True)
    P = ops.softmax_(S)
    O3 = ops.batched_matmul(P, dV).cpu().numpy()
    ref = oracle.fmha(Q, K, V, scale=1.0, causal=False, stable=False)
    assert max(rel_err(O3, ref)) < 1e-4
    Of = ops.fmha(dQ, dK, dV, scale=1.0, causal=False).cpu().numpy()
    assert max(rel_err(Of, O3)) < 1e-4


def test_unfused_graph_at_full_size_matches_fused_kernel(oracle, dev):
    """configs[3] (B=1, H=32, S=2048, D=128) as three kernels with the 512 MiB score tensor in
    between, against the fused kernel on the whole output and against the oracle on sampled
    query rows.  The scale goes into Q, so the graph itself is the reference's (scale 1)."""
    from kernelcodegen_amd import ops
    c = inputs.config_inputs(3)
    Qs = (c["Q"] * np.float32(c["scale"])).astype(np.float32)
    dQ, dK, dV = (_gpu(t, dev) for t in (Qs, c["K"], c["V"]))
    P = ops.softmax_(ops.batched_matmul(dQ, dK, trans_b=True))
    rows = P.sum(-1)
    assert float((rows - 1).abs().max()) < 1e-4
    O3 = ops.batched_matmul(P, dV)
    Of = ops.fmha(dQ, dK, dV, scale=1.0, causal=False)
    d = (O3 - Of).abs().max() / Of.abs().max()
    assert float(d) < 1e-4
    O3h = O3.cpu().numpy()
    for r0, r1 in [(0, 8), (1023, 1031), (2040, 2048)]:
        ref = oracle.fmha(Qs, c["K"], c["V"], scale=1.0, causal=False, stable=False, rows=(r0, r1))
        assert max(rel_err(O3h[:, :, r0:r1], ref)) < 1e-4


def test_launches_follow_the_callers_stream(oracle, dev):
    """Every entry point is asynchronous on the stream it is given: work queued on a side
    stream (default priority) is ordered after what that stream already holds and is not
    visible to the host before the stream is synchronised; two streams run independently."""
    import torch
    from kernelcodegen_amd import ops
    M = N = K = 512
    A = inputs.normal((M, K), 77, 0)
    B = inputs.normal((K, N), 77, 1)
    ref = oracle.relu(oracle.matmul(A, B))
    tA, tB = _gpu(A, dev), _gpu(B, dev)
    side, other = torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        # the producer of the operand and its consumer are both queued on `side`
        tA2 = tA * 2.0
        C = ops.matmul(tA2, tB, relu=True)
        D = ops.relu(C * -1.0)
    with torch.cuda.stream(other):
        shape = (1, 2, 256, 64)
        Q, Kk, V = (inputs.normal(shape, 78, i) for i in range(3))
        O = ops.fmha(_gpu(Q, dev), _gpu(Kk, dev), _gpu(V, dev), scale=0.125, causal=True)
    side.synchronize()
    other.synchronize()
    assert max(rel_err(C.cpu().numpy(), 2.0 * ref)) < 1e-4
    assert float(D.abs().max()) == 0.0          # relu(-relu(x)) == 0
    assert max(rel_err(O.cpu().numpy(), oracle.fmha(Q, Kk, V, scale=0.125, causal=True, stable=True))) < 1e-4


def test_entry_points_can_be_captured_in_a_graph(dev):
    """The entry points neither allocate nor synchronise, so a caller may record them into a
    HIP graph.  The graph is replayed several times with eager work and synchronisations in
    between and new operand contents each time; every replay must equal the eager result."""
    import torch
    from kernelcodegen_amd import ops
    torch.manual_seed(5)
    A = torch.randn(384, 256, device=dev)
    B = torch.randn(256, 512, device=dev)
    C = torch.empty(384, 512, device=dev)
    Q = torch.randn(1, 2, 320, 128, device=dev)
    K = torch.randn_like(Q)
    V = torch.randn_like(Q)
    O = torch.empty_like(Q)
    Qb, Kb, Vb = Q.bfloat16(), K.bfloat16(), V.bfloat16()
    Ob = torch.empty_like(Qb)
    # a size the default plan cuts into two launches, and a batched product and a softmax
    A2 = torch.randn(5120, 32, device=dev)
    B2 = torch.randn(32, 5120, device=dev)
    C2 = torch.empty(5120, 5120, device=dev)
    P = torch.empty(1, 2, 320, 320, device=dev)

    def launch_all():
        ops.matmul(A, B, relu=True, out=C)
        ops.matmul(A2, B2, out=C2)
        ops.batched_matmul(Q, K, trans_b=True, out=P)
        ops.softmax_(P)
        ops.fmha(Q, K, V, scale=0.09, causal=True, out=O)
        ops.fmha(Qb, Kb, Vb, scale=0.09, causal=True, out=Ob)

    launch_all()                      # first use of each kernel outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch_all()
    for rep in range(3):
        A.normal_()
        A2.normal_()
        Q.normal_()
        Qb.copy_(Q)
        launch_all()
        torch.cuda.synchronize()
        want = (C.clone(), O.clone(), Ob.clone(), C2.clone(), P.clone())
        for t in (C, O, Ob, C2, P):
            t.fill_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = (C, O, Ob, C2, P)
        assert all(torch.equal(g, w) for g, w in zip(got, want)), rep


def test_concurrent_host_threads(oracle, dev):
    """The library keeps no state between calls: four host threads launch different
    problems on their own streams at the same time (ctypes releases the GIL around the
    call) and each gets its own correct result."""
    import threading
    import torch
    from kernelcodegen_amd import ops
    shapes = [(256, 128, 96), (130, 70, 33), (512, 256, 64), (64, 64, 512)]
    hostA = [inputs.normal((m, k), 300 + i, 0) for i, (m, n, k) in enumerate(shapes)]
    hostB = [inputs.normal((k, n), 300 + i, 1) for i, (m, n, k) in enumerate(shapes)]
    devA = [_gpu(a, dev) for a in hostA]
    devB = [_gpu(b, dev) for b in hostB]
    torch.cuda.synchronize()
    results, errors = [None] * len(shapes), []

    def work(i):
        try:
            stream = torch.cuda.Stream(device=dev)
            with torch.cuda.stream(stream):
                out = None
                for _ in range(20):
                    out = ops.matmul(devA[i], devB[i], relu=True)
            stream.synchronize()
            results[i] = out.cpu().numpy()
        except Exception as e:      # surfaced in the main thread below
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(shapes))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(len(shapes)):
        assert max(rel_err(results[i], oracle.relu(oracle.matmul(hostA[i], hostB[i])))) < 1e-4, shapes[i]
