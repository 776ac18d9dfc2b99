"""The C++ host layer end to end on the GPU: graph -> optimize -> bind -> launch
(kernelcodegen_amd/host/tests/demo_rocm.cc, the reference's test_matmul /
test_flash_attention flows), checked against the oracle."""
import os
import subprocess

import numpy as np
import pytest

from conftest import rel_err
from kernelcodegen_amd import inputs

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEMO = os.path.join(ROOT, "kernelcodegen_amd", "host", "demo_rocm")
SEED = 0xD3A0


def _run(args, tmp_path):
    if not os.path.exists(DEMO):
        pytest.fail("kernelcodegen_amd/host/demo_rocm is not built (run __graft_entry__.build())")
    out = str(tmp_path / "out.bin")
    res = subprocess.run([DEMO] + [str(a) for a in args] + [out], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-2000:]
    return np.fromfile(out, dtype=np.float32), res.stdout


@pytest.mark.parametrize("shape,relu", [((512, 384, 256), 1), ((4096, 2048, 1024), 1), ((200, 136, 52), 0)])
def test_matmul_demo(oracle, dev, tmp_path, shape, relu):
    M, N, K = shape
    got, text = _run(["matmul", M, N, K, relu], tmp_path)
    assert "namespace matmul_demo {" in text and "kcg_gemm_f32(arg0, arg1, arg2, %d, %d, %d" % (M, N, K) in text
    A = inputs.uniform((M, K), SEED, 0)
    B = inputs.uniform((K, N), SEED, 1)
    ref = oracle.matmul(A, B)
    if relu:
        ref = oracle.relu(ref)
    assert max(rel_err(got.reshape(M, N), ref)) < 1e-4


@pytest.mark.parametrize("detail,stages,source", [(0, 0, "attributes"), (1, 1, "ir"), (2, 2, "ir"), (3, 3, "ir")])
@pytest.mark.parametrize("shape", [(512, 384, 256), (384, 640, 72), (300, 260, 72)])
def test_schedule_selects_the_kernel(oracle, dev, tmp_path, shape, detail, stages, source):
    """The reference's 128 x 128 x 8 tile with the staged (SCHEDULE_DETAIL 1), pipelined (2) and
    direct-load (3) schedules built on the IR: the binding reads block_k, the LDS buffer count
    and the vector width off the scheduled nest (the shared tiles memref<[2x|3x]8x128xf32, 2>,
    the float4 accesses): one or two copies select the double-buffered register-staged kernel,
    a ring of three the direct-load kernel; the launched result is the oracle's.
    Extents the tile does not divide keep the naive nest at every SCHEDULE_DETAIL (the
    optimizer only stages whole tiles), so their schedule comes from the attributes."""
    M, N, K = shape
    whole_tiles = M % 128 == 0 and N % 128 == 0
    if not whole_tiles:
        stages, source = 0, "attributes"
    got, text = _run(["sched", M, N, K, 1, detail], tmp_path)
    m = [l for l in text.splitlines() if l.startswith("schedule ")]
    assert len(m) == 1
    f = m[0].split()
    assert f[1] == source and int(f[3]) == 8 and int(f[5]) == stages and int(f[7]) == 4
    kernel = f[9]
    assert kernel.startswith("gemm_f32_128x128x8_w2x2")
    assert ("_dl" in kernel) == (stages in (0, 3)) and kernel.endswith("_single") == (stages == 1)
    assert "static const kcg_gemm_sched sched = {128, 128, 8, 8, 64, 64, 4, 64, %d};" % stages in text
    A = inputs.uniform((M, K), SEED, 0)
    B = inputs.uniform((K, N), SEED, 1)
    ref = oracle.relu(oracle.matmul(A, B))
    assert max(rel_err(got.reshape(M, N), ref)) < 1e-4


@pytest.mark.parametrize("shape", [(1024, 768, 512), (512, 256, 48)])
def test_default_tile_scheduled_on_the_ir(oracle, dev, tmp_path, shape):
    """The library's default tile (256 x 128 x 16, eight waves of 64 x 64) staged on the IR as a
    direct-load ring of three (SCHEDULE_DETAIL 3): the binding reads the ring depth and BLOCK_SIZE_K
    off memref<3x16x256xf32, 2> / memref<3x16x128xf32, 2> and launches the default kernel."""
    M, N, K = shape
    got, text = _run(["sched256", M, N, K, 1, 3], tmp_path)
    m = [l for l in text.splitlines() if l.startswith("schedule ")]
    assert len(m) == 1
    f = m[0].split()
    assert f[1] == "ir" and int(f[3]) == 16 and int(f[5]) == 3 and int(f[7]) == 4
    assert f[9].startswith("gemm_f32_256x128x16") and "_dl" in f[9]
    assert "static const kcg_gemm_sched sched = {256, 128, 16, 8, 64, 64, 4, 64, 3};" in text
    A = inputs.uniform((M, K), SEED, 0)
    B = inputs.uniform((K, N), SEED, 1)
    ref = oracle.relu(oracle.matmul(A, B))
    assert max(rel_err(got.reshape(M, N), ref)) < 1e-4


@pytest.mark.parametrize("causal", [0, 1])
def test_flash_attention_demo(oracle, dev, tmp_path, causal):
    B, H, S, D = 2, 4, 384, 64
    scale = 0.125
    got, text = _run(["fmha", B, H, S, D, causal, scale], tmp_path)
    assert "kcg_fmha_f32(arg0, arg1, arg2, arg3, 2, 4, 384, 64, 0.125f, %d" % causal in text
    Q, K, V = (inputs.uniform((B, H, S, D), SEED, i) for i in range(3))
    ref = oracle.fmha(Q, K, V, scale=scale, causal=bool(causal), stable=True)
    assert max(rel_err(got.reshape(B, H, S, D), ref)) < 1e-4


@pytest.mark.parametrize("D,br,bc,threads", [(128, 64, 128, 128), (64, 128, 64, 256)])
@pytest.mark.parametrize("causal", [0, 1])
def test_reference_attention_table(oracle, dev, tmp_path, D, br, bc, threads, causal):
    """The reference's own attention table (include/KernelCodeGen.h:38-41 there: HdxBr = BrxBc =
    8192, src/Optimizer/Optimizer.cc:1136-1144) carried through the facade: Br 64 x Bc 128 at
    head dim 128 (two waves of 32 query rows), Br 128 x Bc 64 at head dim 64."""
    B, H, S = 2, 3, 320
    scale = 0.125
    got, text = _run(["fmharef", B, H, S, D, causal, scale], tmp_path)
    assert "static const kcg_fmha_sched sched = {%d, %d};" % (br, bc) in text
    assert "block dims:(%d, 1, 1)" % threads in text
    Q, K, V = (inputs.uniform((B, H, S, D), SEED, i) for i in range(3))
    ref = oracle.fmha(Q, K, V, scale=scale, causal=bool(causal), stable=True)
    assert max(rel_err(got.reshape(B, H, S, D), ref)) < 1e-4


@pytest.mark.parametrize("shape", [(2, 3, 192, 64), (1, 2, 100, 128)])
def test_unfused_graph(oracle, dev, tmp_path, shape):
    """A graph the attention pattern rejects (the score tensor has a second reader,
    src/Optimizer/Optimizer.cc:597-652 of the reference falls through): S = Q.K^T,
    R = Relu(S) into its own buffer, P = Softmax(S) in place, O = P.V.  The host backend binds
    the four calls to the un-fused kernels, one launcher each in module order, with S shared
    between them; O and R against the oracle's operators chained the same way."""
    B, H, S, D = shape
    got, text = _run(["unfused", "attn", B, H, S, D], tmp_path)
    assert "bindings 4: kcg_batched_matmul_f32 kcg_relu_f32 kcg_softmax_f32 kcg_batched_matmul_f32" in text
    assert "return kcg_batched_matmul_f32(arg0, 0, arg1, 1, arg2, %d, %d, %d, %d, stream);" % (B * H, S, S, D) in text
    assert "return kcg_softmax_f32(arg0, %d, %d, stream);" % (B * H * S, S) in text
    Q, K, V = (inputs.uniform((B, H, S, D), SEED, i) for i in range(3))
    scores = oracle.batched_matmul(Q, 0, K, 1)
    R = oracle.relu(scores)
    O = oracle.batched_matmul(oracle.softmax(scores), 0, V, 0)
    n_o = B * H * S * D
    assert got.size == n_o + B * H * S * S
    assert max(rel_err(got[:n_o].reshape(B, H, S, D), O)) < 1e-4
    assert max(rel_err(got[n_o:].reshape(B, H, S, S), R)) < 1e-4
    assert np.array_equal(got[n_o:] == 0, R.reshape(-1) == 0)


def test_lone_softmax(oracle, dev, tmp_path):
    rows, n = 37, 1000
    got, text = _run(["unfused", "softmax", rows, n], tmp_path)
    assert "bindings 1: kcg_softmax_f32" in text and "namespace softmax_demo {" in text
    x = inputs.uniform((rows, n), SEED, 0) * np.float32(4.0)
    assert max(rel_err(got.reshape(rows, n), oracle.softmax(x))) < 1e-4


def _trials(text):
    trials, best = [], None
    for line in text.splitlines():
        f = line.split()
        if f and f[0] == "trial":
            trials.append((" ".join(f[1:-2]), f[-2], None if f[-1] == "refused" else float(f[-1])))
        elif f and f[0] == "best":
            best = (" ".join(f[1:-1]), float(f[-1]))
    return trials, best


def test_matmul_config_search(oracle, dev, tmp_path):
    """The trial loop with a measured evaluate(): every tile of the search space is timed on
    the device, the fastest one is bound, and its result is still the oracle's."""
    M, N, K = 2048, 2048, 1024
    got, text = _run(["tune", "matmul", M, N, K, 1], tmp_path)
    trials, best = _trials(text)
    assert [t[0] for t in trials] == ["256x128x16", "256x128x32", "128x128x16", "128x128x32", "128x128x8",
                                      "128x64x32", "64x64x32", "96x96x32", "96x64x32"]
    timed = [t for t in trials if t[2] is not None]
    assert len(timed) == 9 and all(0 < t[2] < 50 for t in timed)
    fastest = min(timed, key=lambda t: t[2])
    assert best is not None and best[0] == fastest[0] and abs(best[1] - fastest[2]) < 1e-4
    bm, bn, bk = (int(x) for x in best[0].split("x"))
    assert "static const kcg_gemm_sched sched = {%d, %d, %d," % (bm, bn, bk) in text
    A = inputs.uniform((M, K), SEED, 0)
    B = inputs.uniform((K, N), SEED, 1)
    ref = oracle.relu(oracle.matmul(A, B))
    assert max(rel_err(got.reshape(M, N), ref)) < 1e-4


def test_matmul_config_search_finds_the_96_tile(oracle, dev, tmp_path):
    """1536^3: 256 tiles of 96 x 96 are exactly one round of the CUs, every power-of-two tile
    leaves a partly filled one; the measured search picks it."""
    M = N = K = 1536
    got, text = _run(["tune", "matmul", M, N, K, 1], tmp_path)
    trials, best = _trials(text)
    assert all(t[2] is not None for t in trials) and len(trials) == 9
    assert best is not None and best[0] == "96x96x32"
    assert "static const kcg_gemm_sched sched = {96, 96, 32," in text
    A = inputs.uniform((M, K), SEED, 0)
    B = inputs.uniform((K, N), SEED, 1)
    ref = oracle.relu(oracle.matmul(A, B))
    assert max(rel_err(got.reshape(M, N), ref)) < 1e-4


def test_attention_config_search(oracle, dev, tmp_path):
    """fp32 attention at head dim 128: Br 128 x Bc 32|64 and Br 256 x Bc 32 are timed, Br 256 x
    Bc 64 (built for bf16 and for head dim 64 only) is refused."""
    B, H, S, D = 1, 8, 1024, 128
    scale = D ** -0.5
    got, text = _run(["tune", "fmha", B, H, S, D, 1, scale], tmp_path)
    trials, best = _trials(text)
    assert [t[0] for t in trials] == ["br128 bc32", "br128 bc64", "br256 bc32", "br256 bc64"]
    assert all(t[2] is not None for t in trials[:3]) and trials[3][2] is None
    fastest = min(trials[:3], key=lambda t: t[2])
    assert best is not None and best[0] == fastest[0]
    Q, K, V = (inputs.uniform((B, H, S, D), SEED, i) for i in range(3))
    ref = oracle.fmha(Q, K, V, scale=scale, causal=True, stable=True)
    assert max(rel_err(got.reshape(B, H, S, D), ref)) < 1e-4
