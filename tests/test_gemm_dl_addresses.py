"""Address arithmetic of the direct-load matmul kernels, replayed on the host.

tests/gemm_dl_address_model.cc walks every workgroup, wave and lane of one launch of
gemm_f32_dl_kernel through the kernel's own integer expressions (it shares the tile
geometry header with the kernel) and checks that every global byte a direct load, a tail
re-load or a store of C touches lies inside its tensor, that no 32-bit intermediate
overflows and that the stores cover C exactly.  No GPU is involved.

The cases include the three launches of the one call that ever ended in a GPU memory
fault (A = 66000 x 33000, more than 2^31 elements): 65536 rows on the 256 x 128 x 16 tile,
the remaining 464 rows on 64 x 64 x 32 at A + 65536 * K, and the 488-row call that
followed.  All three are clean, so the kernel's addressing is not the cause of that
fault; kcg_gemm_f32 keeps refusing operands of that size class.
"""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "gemm_dl_address_model.cc")
INC = os.path.join(ROOT, "kernelcodegen_amd", "csrc")


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("gemm_dl") / "gemm_dl_address_model")
    subprocess.run(["g++", "-O2", "-std=c++17", "-I", INC, SRC, "-o", exe], check=True)
    return exe


# (BM, BN, BK, WAVES_M, WAVES_N, M, N, K, GROUP_M)
CASES = [
    # the faulting call, launch by launch
    (256, 128, 16, 4, 2, 65536, 128, 33000, 8),
    (64, 64, 32, 2, 2, 464, 128, 33000, 8),
    (64, 64, 32, 2, 2, 488, 128, 33000, 8),
    # BASELINE configs on their default tiles
    (256, 128, 16, 4, 2, 4096, 4096, 4096, 8),
    (256, 128, 16, 4, 2, 4096, 2048, 1024, 8),
    (256, 128, 16, 4, 2, 32768, 768, 768, 8),
    # ragged in every dimension, every built tile
    (128, 128, 32, 2, 2, 1000, 1000, 1000, 8),
    (128, 128, 16, 2, 2, 4100, 516, 72, 4),
    (128, 128, 8, 2, 2, 130, 132, 44, 8),
    (256, 128, 32, 4, 2, 4100, 4100, 4100, 8),
    (128, 64, 32, 2, 2, 2050, 2052, 36, 1),
    (64, 64, 32, 2, 2, 65, 68, 32, 8),
    # byte offsets beyond 2^32 inside A and inside C
    (256, 128, 16, 4, 2, 40000, 256, 32768, 8),
    (128, 64, 32, 2, 2, 40000, 32768, 64, 8),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(map(str, c)))
def test_every_access_inside_its_tensor(model, case):
    r = subprocess.run([model] + [str(v) for v in case], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert " 0 violations" in r.stdout


# ---- the streaming kernel of BatchedMatmul (gemm_f32_stream_kernel) ----
STREAM_SRC = os.path.join(ROOT, "tests", "gemm_stream_address_model.cc")


@pytest.fixture(scope="module")
def stream_model(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("gemm_stream") / "gemm_stream_address_model")
    subprocess.run(["g++", "-O2", "-std=c++17", "-I", INC, STREAM_SRC, "-o", exe], check=True)
    return exe


# (TRANS_B, BATCH, M, N, K, GRID): the attention-score product of configs[3] in both layouts,
# the shapes of the GPU tests (item counts that 8 XCDs x 32 workgroups do not divide, K of 4,
# 12, 20 and 64 slices), a grid smaller than the CU count, byte offsets beyond 2^32 inside C,
# and the widest N the launcher admits (lane offsets of the stores close to 2^31).
STREAM_CASES = [
    (1, 32, 2048, 2048, 128, 256),
    (0, 32, 2048, 2048, 128, 256),
    (1, 9, 1280, 1664, 64, 256),
    (1, 9, 1280, 1664, 192, 256),
    (0, 20, 768, 1152, 320, 256),
    (1, 5, 2560, 1408, 1024, 256),
    (0, 3, 256, 384, 64, 9),
    (1, 16, 8192, 8192, 128, 256),
    (0, 1, 256, 2097152, 64, 256),
]


@pytest.mark.parametrize("case", STREAM_CASES, ids=lambda c: "x".join(map(str, c)))
def test_streaming_kernel_items_and_addresses(stream_model, case):
    """Every tile is taken by exactly one workgroup, every load (the cursor that runs ahead
    and parks on the last slice included) and every store lies inside its tensor, and the
    stores of the eight waves cover a tile exactly once."""
    r = subprocess.run([stream_model] + [str(v) for v in case], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout + r.stderr
    assert " 0 violations" in r.stdout


# ---- the launch with K-split tail tiles (kcg_gemm_f32_ws) ----
@pytest.mark.parametrize("shape", [(1536, 1536, 1536), (1536, 1536, 1024), (1024, 1088, 1536), (1280, 1088, 2048),
                                   (1536, 1536, 4096), (512, 512, 4096), (256, 256, 8192), (512, 1024, 2048),
                                   (768, 768, 3072), (1280, 1280, 4096), (1344, 1344, 4096), (640, 640, 1280),
                                   (1792, 1792, 1792), (2304, 2304, 1152), (3584, 3584, 1024),
                                   (1500, 1500, 1536), (300, 260, 4096), (1000, 1500, 2048), (1530, 1536, 1536)])
def test_k_split_launch_numbering_and_addresses(model, shape):
    """The plan kcg_gemm_f32_ws_bytes reports (whole tiles of the full rounds, the rest in
    pieces) replayed on the host: every whole tile and every piece is taken once, a piece
    loads only its own K range, the pieces fill the workspace exactly, and whole tiles plus
    reduced tiles write every element of C exactly once.  (1280, 1088, 2048), (768, 768, 3072)
    and the two after it have more pieces than the chip has CUs (672, 432, 1152, 740); the
    last three are sizes whose plan without a workspace uses a larger tile (3, 5 and 12 full
    rounds of 64 x 64 tiles before the pieces); the last four have edge tiles in M, N or both."""
    from kernelcodegen_amd import lib
    M, N, K = shape
    need = int(lib.load().kcg_gemm_f32_ws_bytes(M, N, K, None))
    tiles = ((M + 63) // 64) * ((N + 63) // 64)
    rest = tiles % 256
    assert need > 0 and need % (rest * 64 * 64 * 4) == 0
    parts = need // (rest * 64 * 64 * 4)
    # GROUP_SIZE_M is the one schedule field the plan takes from the caller: the default and two others
    for group_m in (8, 4, 3) if shape in ((1536, 1536, 1536), (1280, 1088, 2048)) else (8,):
        r = subprocess.run([model, "split", str(M), str(N), str(K), str(group_m), str(tiles - rest), str(parts)],
                           capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stdout + r.stderr
        assert " 0 violations" in r.stdout


# ---- the 96 x 96 and 96 x 64 tiles on 16 x 16 x 4 MFMA blocks (gemm_f32_t96_kernel) ----
T96_SRC = os.path.join(ROOT, "tests", "gemm_t96_address_model.cc")


@pytest.fixture(scope="module")
def t96_model(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("gemm_t96") / "gemm_t96_address_model")
    subprocess.run(["g++", "-O2", "-std=c++17", "-I", INC, T96_SRC, "-o", exe], check=True)
    return exe


# (M, N, K, GROUP_M): one tile and one slice, the size the tile exists for, tile counts the
# XCD count and GROUP_M do not divide, lane offsets close to 2^32 / byte offsets beyond it,
# and extents 96 does not divide (a single row, a single column chunk, edges in M, N and both)
@pytest.mark.parametrize("case", [(96, 96, 32, 8), (1536, 1536, 1536, 8), (960, 4128, 64, 3), (672, 1248, 4000 // 32 * 32, 5),
                                  (40032, 384, 32768, 8), (192, 3999936, 32, 8), (1, 4, 32, 8), (97, 100, 96, 3),
                                  (1472, 1500, 64, 8), (40000, 388, 32768, 8)],
                         ids=lambda c: "x".join(map(str, c)))
@pytest.mark.parametrize("block_n", [96, 64])
def test_t96_loads_operands_and_stores(t96_model, case, block_n):
    """The direct loads of a slice fill its A and B stage exactly once from inside the
    tensors; every operand read of every lane fetches the (row, k) / (k, column) its MFMA step
    multiplies, both operands with the same k and every k of the slice once; the stores of
    the four waves cover the part of the C tile inside C exactly once."""
    r = subprocess.run([t96_model, str(block_n)] + [str(v) for v in case], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert " 0 violations" in r.stdout
