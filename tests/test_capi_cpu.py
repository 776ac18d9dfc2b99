"""The C-ABI library without a GPU: it loads, exports every symbol that
include/kcg.h declares, and rejects bad arguments before touching the device.
No kernel is launched here."""
import ctypes
import os
import re

import pytest

from kernelcodegen_amd import lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "kcg.h")).read()
    return sorted(set(re.findall(r"KCG_API[^;(]*?\b(kcg_\w+)\s*\(", text)))


def test_header_declares_what_python_binds():
    assert _declared_symbols() == sorted(lib.SYMBOLS)


def test_library_exports_every_declared_symbol():
    L = ctypes.CDLL(lib.LIB_PATH)
    for name in _declared_symbols():
        assert hasattr(L, name), name


def test_status_strings():
    L = lib.load()
    assert L.kcg_version().decode().count(".") == 2
    seen = set()
    for code in range(0, 8):
        s = lib.status_str(code)
        assert s and s != "unknown status"
        seen.add(s)
    assert len(seen) == 8
    assert lib.status_str(99) == "unknown status"


def test_argument_validation_returns_status_not_abort():
    L = lib.load()
    one = ctypes.c_void_p(16)  # never dereferenced: validation fails first
    assert L.kcg_gemm_f32(None, one, one, 128, 128, 8, 0, None, None) == 1
    assert L.kcg_gemm_f32(one, one, one, 0, 128, 8, 0, None, None) == 2
    assert L.kcg_gemm_f32(one, one, one, 128, 128, 8, 7, None, None) == 5
    bad = lib.GemmSched(block_m=96, block_n=128, block_k=8)
    assert L.kcg_gemm_f32(one, one, one, 128, 128, 8, 0, ctypes.byref(bad), None) == 4
    bad = lib.GemmSched(wave_size=32)
    assert L.kcg_gemm_f32(one, one, one, 128, 128, 8, 0, ctypes.byref(bad), None) == 4
    assert L.kcg_fmha_f32(one, one, None, one, 1, 1, 128, 128, 1.0, 0, None, None) == 1
    assert L.kcg_fmha_f32(one, one, one, one, 1, 1, 0, 128, 1.0, 0, None, None) == 2
    assert L.kcg_fmha_f32(one, one, one, one, 1, 1, 128, 96, 1.0, 0, None, None) == 3
    assert L.kcg_fmha_f32(one, one, one, one, 1, 1, 128, 128, 1.0, 2, None, None) == 5
    assert L.kcg_fmha_f32(one, one, one, one, 1, 1, 128, 128, float("nan"), 0, None, None) == 5
    assert L.kcg_fmha_f32(ctypes.c_void_p(4), one, one, one, 1, 1, 128, 128, 1.0, 0, None, None) == 5
    bad = lib.FmhaSched(br=64, bc=64)
    assert L.kcg_fmha_f32(one, one, one, one, 1, 1, 128, 128, 1.0, 0, ctypes.byref(bad), None) == 4
    assert L.kcg_fmha_bf16(one, one, one, one, 3, 1, 1, 128, 128, 1.0, 0, None, None) == 5
    assert L.kcg_fmha_bf16(one, one, one, None, 1, 1, 1, 128, 128, 1.0, 0, None, None) == 1
    assert L.kcg_relu_f32(None, one, 4, None) == 1
    assert L.kcg_relu_f32(one, one, 0, None) == 2
    assert L.kcg_batched_matmul_f32(one, 2, one, 0, one, 1, 4, 4, 4, None) == 5
    assert L.kcg_batched_matmul_f32(one, 0, one, 0, one, 0, 4, 4, 4, None) == 2
    assert L.kcg_softmax_f32(None, 4, 4, None) == 1
    assert L.kcg_softmax_f32(one, 4, 0, None) == 2


def test_launch_geometry_queries():
    L = lib.load()
    info = lib.LaunchInfo()
    # the reference's demo shape, with its own 128 x 128 x 8 tile: grid (32,16) = 512 tiles
    s = lib.GemmSched(block_m=128, block_n=128, block_k=8, wave_m=64, wave_n=64)
    assert L.kcg_gemm_f32_query(4096, 2048, 1024, ctypes.byref(s), ctypes.byref(info)) == 0
    assert info.grid[0] == 32 * 16 and info.block[0] == 256
    # three LDS stages of the direct-load kernel: A 128 x 8, B as four 1 KiB runs 64 B apart
    assert info.lds_bytes == 3 * (128 * 8 + 4 * 272) * 4 and info.kernel.endswith(b"_dl")
    assert L.kcg_gemm_f32_query(4096, 4096, 4096, None, ctypes.byref(info)) == 0
    assert info.grid[0] * 256 * 128 == 4096 * 4096 and info.lds_bytes <= 160 * 1024
    assert L.kcg_gemm_f32_query(100, 100, 100, None, None) == 1
    # 7168^3: 1568 large tiles would spill 32 into a seventh round; 27 rows of tiles run in
    # whole rounds and the last 256 rows of C as a second launch on the 64 x 64 tile
    assert L.kcg_gemm_f32_query(7168, 7168, 7168, None, ctypes.byref(info)) == 0
    assert info.grid[0] == 27 * 56 and info.block[0] == 512
    assert info.kernel == b"gemm_f32_256x128x16_w4x2_dl+256rows_64x64x32"
    # one copy of the K-slice tiles in LDS: the two tiles the host layer stages, nothing else
    s1 = lib.GemmSched(block_m=128, block_n=128, block_k=8, wave_m=64, wave_n=64, lds_stages=1)
    assert L.kcg_gemm_f32_query(4096, 2048, 1024, ctypes.byref(s1), ctypes.byref(info)) == 0
    assert info.kernel == b"gemm_f32_128x128x8_w2x2_single" and info.lds_bytes == (128 * 12 + 8 * 136) * 4
    s1.block_k = 16
    assert L.kcg_gemm_f32_query(4096, 2048, 1024, ctypes.byref(s1), ctypes.byref(info)) == 4
    s1.block_k, s1.lds_stages = 8, 4
    assert L.kcg_gemm_f32_query(4096, 2048, 1024, ctypes.byref(s1), ctypes.byref(info)) == 4
    s1.lds_stages = -1
    assert L.kcg_gemm_f32_query(4096, 2048, 1024, ctypes.byref(s1), ctypes.byref(info)) == 4
    # an explicit tile is never cut
    s = lib.GemmSched(block_m=256, block_n=128, block_k=16, wave_m=64, wave_n=64)
    assert L.kcg_gemm_f32_query(7168, 7168, 7168, ctypes.byref(s), ctypes.byref(info)) == 0
    assert info.grid[0] == 28 * 56 and b"+" not in info.kernel
    # 1536^3: 576 tiles of 64 x 64 are 2.25 rounds of the 256 CUs, 256 tiles of 96 x 96 exactly one
    assert L.kcg_gemm_f32_query(1536, 1536, 1536, None, ctypes.byref(info)) == 0
    assert info.kernel == b"gemm_f32_96x96x32_w2x2_dl" and info.launches == 1
    assert info.grid[0] == 256 and info.block[0] == 256 and info.waves_per_block == 4
    assert info.lds_bytes == 3 * (96 * 32 + 32 * 96) * 4
    # ... also when only GROUP_SIZE_M is given; with a short K the power-of-two tiles keep the problem
    assert L.kcg_gemm_f32_query(1536, 1536, 1536, ctypes.byref(lib.GemmSched(group_m=4)), ctypes.byref(info)) == 0
    assert info.kernel == b"gemm_f32_96x96x32_w2x2_dl"
    assert L.kcg_gemm_f32_query(1536, 1536, 256, None, ctypes.byref(info)) == 0
    assert b"96x96" not in info.kernel
    # 1472^3: 16 x 16 tiles of 96 x 96 (the last ones partly outside C) are one round as well
    assert L.kcg_gemm_f32_query(1472, 1472, 1472, None, ctypes.byref(info)) == 0
    assert info.kernel == b"gemm_f32_96x96x32_w2x2_dl_ragged" and info.grid[0] == 256
    # 1152^2 x 2048: 216 tiles of 96 x 64 are one round, nothing else comes close
    assert L.kcg_gemm_f32_query(1152, 1152, 2048, None, ctypes.byref(info)) == 0
    assert info.kernel == b"gemm_f32_96x64x32_w2x2_dl" and info.grid[0] == 12 * 18
    assert info.lds_bytes == 3 * (96 * 32 + 32 * 64) * 4
    s64 = lib.GemmSched(block_m=96, block_n=64, block_k=32, wave_m=48, wave_n=32)
    assert L.kcg_gemm_f32_query(100, 100, 64, ctypes.byref(s64), ctypes.byref(info)) == 0
    assert info.kernel == b"gemm_f32_96x64x32_w2x2_dl_ragged" and info.grid[0] == 2 * 2
    s64.wave_n = 48
    assert L.kcg_gemm_f32_query(100, 100, 64, ctypes.byref(s64), ctypes.byref(info)) == 4
    # the tile by name: K in whole slices, N a multiple of 4, direct-load ring only
    s96 = lib.GemmSched(block_m=96, block_n=96, block_k=32, wave_m=48, wave_n=48)
    assert L.kcg_gemm_f32_query(960, 192, 64, ctypes.byref(s96), ctypes.byref(info)) == 0
    assert info.grid[0] == 10 * 2 and info.kernel == b"gemm_f32_96x96x32_w2x2_dl"
    assert L.kcg_gemm_f32_query(950, 200, 64, ctypes.byref(s96), ctypes.byref(info)) == 0
    assert info.grid[0] == 10 * 3 and info.kernel == b"gemm_f32_96x96x32_w2x2_dl_ragged"
    assert L.kcg_gemm_f32_query(960, 198, 64, ctypes.byref(s96), ctypes.byref(info)) == 4
    assert L.kcg_gemm_f32_query(960, 192, 48, ctypes.byref(s96), ctypes.byref(info)) == 4
    s96.lds_stages = 2
    assert L.kcg_gemm_f32_query(960, 192, 64, ctypes.byref(s96), ctypes.byref(info)) == 4
    s96.lds_stages, s96.wave_m = 3, 32
    assert L.kcg_gemm_f32_query(960, 192, 64, ctypes.byref(s96), ctypes.byref(info)) == 4
    # bf16 causal, S = 4096: 256-row query blocks run in pairs (n-1-i, i) -> 8 work items per
    # head, 1024 in all, walked by one persistent 8-wave workgroup per CU
    assert L.kcg_fmha_query(1, 4, 32, 4096, 128, 1, None, ctypes.byref(info)) == 0
    assert info.grid[0] == 256 and info.block[0] == 512 and info.waves_per_block == 8
    assert info.kernel == b"fmha_bf16_d128_br256_bc64_pingpong_causal_paired"
    assert info.lds_bytes == (4 + 5) * 64 * 128 * 2
    # fewer items than CUs: one workgroup each
    assert L.kcg_fmha_query(1, 1, 8, 4096, 128, 1, ctypes.byref(lib.FmhaSched(br=256, bc=64)), ctypes.byref(info)) == 0
    assert info.grid[0] == 8 * 8
    s128 = lib.FmhaSched(br=128, bc=64)
    assert L.kcg_fmha_query(1, 4, 32, 4096, 128, 1, ctypes.byref(s128), ctypes.byref(info)) == 0
    assert info.grid[0] == 4 * 32 * 16 and info.block[0] == 256
    assert L.kcg_fmha_query(1, 4, 32, 4096, 128, 0, ctypes.byref(s128), ctypes.byref(info)) == 0
    assert info.grid[0] == 4 * 32 * 32 and info.lds_bytes == 2 * 2 * 64 * 128 * 2
    assert L.kcg_fmha_query(0, 1, 32, 2048, 128, 0, None, ctypes.byref(info)) == 0
    # fp32, one workgroup per CU fills the chip exactly: the default is the 256-row workgroup ...
    assert info.grid[0] == 32 * 2048 // 256 and info.block[0] == 512
    # ... and the 128-row one where that leaves more (or fewer) workgroups than that
    assert L.kcg_fmha_query(0, 2, 32, 2048, 128, 0, None, ctypes.byref(info)) == 0
    assert info.grid[0] == 2 * 32 * 2048 // 128 and info.block[0] == 256
    assert L.kcg_fmha_query(0, 1, 8, 2048, 128, 0, None, ctypes.byref(info)) == 0
    assert info.grid[0] == 8 * 2048 // 128 and info.block[0] == 256
    # fp32 causal: 128-row query blocks in pairs
    assert L.kcg_fmha_query(0, 1, 32, 2048, 128, 1, None, ctypes.byref(info)) == 0
    assert info.grid[0] == 32 * 8 and b"causal_paired" in info.kernel
    s256 = lib.FmhaSched(br=256, bc=32)
    assert L.kcg_fmha_query(0, 1, 32, 2048, 128, 0, ctypes.byref(s256), ctypes.byref(info)) == 0
    assert info.grid[0] == 32 * 8 and info.block[0] == 512 and info.waves_per_block == 8
    s256.bc = 64
    assert L.kcg_fmha_query(0, 1, 32, 2048, 128, 0, ctypes.byref(s256), ctypes.byref(info)) == 4
    assert L.kcg_fmha_query(7, 1, 1, 128, 128, 0, None, ctypes.byref(info)) == 5
    assert L.kcg_fmha_query(0, 1, 1, 128, 80, 0, None, ctypes.byref(info)) == 3


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(lib, "_lib", None)
    monkeypatch.setattr(lib, "LIB_PATH", "/nonexistent/libkcg_hip.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        lib.load()


def test_tensors_of_two_to_the_31_elements_are_refused():
    """The size check comes before any launch or device query, so it runs without a GPU and
    never touches the (fake) pointers."""
    L = lib.load()
    fake = ctypes.c_void_p(256)
    unsupported = 3
    assert L.kcg_gemm_f32(fake, fake, fake, 66000, 128, 33000, 0, None, None) == unsupported
    assert L.kcg_gemm_f32(fake, fake, fake, 66000, 33000, 64, 0, None, None) == unsupported
    assert L.kcg_gemm_f32(fake, fake, fake, 64, 66000, 33000, 0, None, None) == unsupported
    assert L.kcg_batched_matmul_f32(fake, 0, fake, 1, fake, 64, 8192, 8192, 128, None) == unsupported
    assert L.kcg_fmha_f32(fake, fake, fake, fake, 64, 64, 4096, 128, 1.0, 0, None, None) == unsupported
    assert L.kcg_fmha_bf16(fake, fake, fake, fake, 1, 64, 64, 4096, 128, 1.0, 1, None, None) == unsupported
    assert L.kcg_relu_f32(fake, fake, 1 << 31, None) == unsupported
    assert L.kcg_softmax_f32(fake, 1 << 20, 1 << 11, None) == unsupported


def test_default_matmul_plans_cover_the_problem():
    """Whatever the default chooser decides (one launch, or whole rounds of the large tile
    plus a tail launch on a small tile), the launches it names cover every row of C exactly
    once and the main launch is made of whole tile rows."""
    import re
    import numpy as np
    L = lib.load()
    info = lib.LaunchInfo()
    rng = np.random.default_rng(7)
    shapes = [(d, d) for d in range(1024, 16385, 1024)] + \
             [(int(rng.integers(1, 40000)), int(rng.integers(1, 40000))) for _ in range(300)]
    cut = streamed = 0
    for M, N in shapes:
        K = 768 if M == N and M % 1024 == 0 else 256
        assert L.kcg_gemm_f32_query(M, N, K, None, ctypes.byref(info)) == 0
        name = info.kernel.decode()
        if name.endswith("_stream"):
            assert K == 768
            # a short K (512 to 1024) with whole 256 x 128 tiles, two per CU or more: one persistent
            # workgroup per CU walks the tiles
            assert name == "gemm_f32_256x128x16_w4x2_stream" and M % 256 == 0 and N % 128 == 0
            assert (M // 256) * (N // 128) >= 512 and info.grid[0] == 256 and info.block[0] == 512
            streamed += 1
            continue
        m = re.fullmatch(r"gemm_f32_(\d+)x(\d+)x(\d+)_w\dx\d(?:_dl|_dl_ragged)?(?:\+(\d+)rows_(\d+)x(\d+)x(\d+))?", name)
        assert m, name
        bm, bn = int(m.group(1)), int(m.group(2))
        tiles_n = -(-N // bn)
        assert info.grid[0] % tiles_n == 0
        main_rows = info.grid[0] // tiles_n * bm
        if m.group(4) is None:
            assert main_rows >= M and main_rows - M < bm, (M, N, name)
        else:
            cut += 1
            assert (bm, bn) == (256, 128) and main_rows + int(m.group(4)) == M, (M, N, name)
            assert int(m.group(4)) >= 1
    assert cut > 10 and streamed >= 5


def _meta(shape, dtype, cuda=True, contiguous=True):
    """A tensor stand-in that carries shape / dtype / device / contiguity only (torch's
    'meta' tensors report is_cuda False, so the wrappers' checks are driven through a thin
    subclass instead)."""
    import torch

    class T(torch.Tensor):
        @property
        def is_cuda(self):
            return cuda

        @property
        def device(self):
            return torch.device("cuda:0") if cuda else torch.device("cpu")

        def is_contiguous(self, *a, **k):
            return contiguous

        def data_ptr(self):
            raise AssertionError("validation must fail before a pointer is taken")

    return torch.empty(shape, dtype=dtype).as_subclass(T)


def test_python_wrappers_refuse_mismatched_tensors():
    """Every tensor handed to a kernel is checked for device, dtype, contiguity and exact
    shape first (the kernels only see raw pointers).  None of these calls reaches the GPU."""
    import torch
    from kernelcodegen_amd import ops
    f32, bf16, f16 = torch.float32, torch.bfloat16, torch.float16
    A, B = _meta((64, 32), f32), _meta((32, 48), f32)
    with pytest.raises(ValueError):
        ops.matmul(A, B, out=_meta((64, 40), f32))          # wrong shape
    with pytest.raises(ValueError):
        ops.matmul(A, B, out=_meta((64, 48), f16))          # wrong dtype
    with pytest.raises(ValueError):
        ops.matmul(A, B, out=_meta((64, 48), f32, cuda=False))
    with pytest.raises(ValueError):
        ops.matmul(A, _meta((32, 48), f32, cuda=False))
    with pytest.raises(ValueError):
        ops.matmul(A, _meta((31, 48), f32))                 # K mismatch
    bA, bB = _meta((2, 3, 16, 8), f32), _meta((2, 3, 8, 24), f32)
    with pytest.raises(ValueError):
        ops.batched_matmul(bA, bB, out=_meta((2, 3, 16, 20), f32))
    with pytest.raises(ValueError):
        ops.batched_matmul(bA, bB, out=_meta((2, 3, 16, 24), bf16))
    with pytest.raises(ValueError):
        ops.batched_matmul(bA, bB, out=_meta((2, 3, 16, 24), f32, contiguous=False))
    shape = (1, 2, 64, 64)
    Q = _meta(shape, f32)
    with pytest.raises(ValueError):
        ops.fmha(Q, _meta(shape, bf16), _meta(shape, f32))  # narrower K: would be read past its end
    with pytest.raises(ValueError):
        ops.fmha(Q, _meta(shape, f32, cuda=False), _meta(shape, f32))
    with pytest.raises(ValueError):
        ops.fmha(Q, _meta(shape, f32), _meta((1, 2, 64, 32), f32))
    with pytest.raises(ValueError):
        ops.fmha(Q, _meta(shape, f32), _meta(shape, f32), out=_meta(shape, bf16))
    with pytest.raises(ValueError):
        ops.fmha(Q, _meta(shape, f32), _meta(shape, f32), out_dtype=bf16)
    Qb, Kb, Vb = (_meta(shape, bf16) for _ in range(3))
    with pytest.raises(ValueError):
        ops.fmha(Qb, Kb, Vb, out=_meta(shape, f16))         # 2-byte buffer, would be written as fp32
    with pytest.raises(ValueError):
        ops.fmha(Qb, Kb, Vb, out_dtype=f16)
    with pytest.raises(ValueError):
        ops.fmha(Qb, Kb, Vb, out=_meta(shape, f32), out_dtype=bf16)   # out disagrees with out_dtype
    with pytest.raises(ValueError):
        ops.fmha(Qb, Kb, Vb, out=_meta((1, 2, 64, 32), bf16))
    with pytest.raises(ValueError):
        ops.fmha(_meta(shape, f16), _meta(shape, f16), _meta(shape, f16))


@pytest.mark.parametrize("shape,causal,pingpong", [
    # D = 128: the 256-row ping-pong kernel from two work items per CU on ...
    ((4, 32, 4096, 128), 1, True),      # configs[4]: 1024 paired items
    ((8, 32, 1024, 128), 1, True),      # 2 pairs x 256 heads = 512
    ((32, 32, 512, 128), 1, True),      # 1 pair x 1024 heads
    # ... or exactly filling the CUs on a long or a non-causal sweep
    ((1, 32, 2048, 128), 0, True),      # 8 blocks x 32 heads = 256
    ((1, 32, 4096, 128), 1, True),      # 8 pairs x 32 heads = 256, S >= 2048
    ((4, 32, 1024, 128), 1, False),     # 256 items, short and causal: the 128-row kernel
    ((16, 16, 512, 128), 1, False),
    ((16, 16, 512, 128), 0, True),      # 512 items
    # launches 256-row blocks do not fill
    ((1, 32, 2048, 128), 1, False),
    ((1, 16, 2048, 128), 0, False),
    # D = 64: always the 128-row kernel
    ((2, 16, 8192, 64), 0, False),
    ((4, 32, 4096, 64), 1, False),
])
def test_bf16_attention_default_block_size(shape, causal, pingpong):
    """The block-size rule of kcg_fmha_bf16 with no schedule given, as kcg_fmha_query reports it."""
    L = lib.load()
    info = lib.LaunchInfo()
    B, H, S, D = shape
    assert L.kcg_fmha_query(1, B, H, S, D, causal, None, ctypes.byref(info)) == 0
    assert (b"pingpong" in info.kernel) == pingpong, info.kernel
    assert (b"br256" in info.kernel) == pingpong
    if pingpong:
        blocks = (S + 255) // 256
        items = ((blocks + 1) // 2 if causal else blocks) * B * H
        assert info.grid[0] == min(items, 256) and info.block[0] == 512


def test_workspace_entry_points_check_their_arguments():
    """kcg_gemm_f32_ws / kcg_gemm_f32_noalloc refuse what kcg_gemm_f32 refuses, before any
    device call; kcg_gemm_f32_ws_bytes is pure host arithmetic."""
    L = lib.load()
    fake = ctypes.c_void_p(0x1000)
    assert L.kcg_gemm_f32_ws(None, fake, fake, 64, 64, 64, 0, None, None, 0, None) == 1
    assert L.kcg_gemm_f32_ws(fake, fake, fake, 64, 0, 64, 0, None, None, 0, None) == 2
    assert L.kcg_gemm_f32_ws(fake, fake, fake, 64, 64, 64, 7, None, None, 0, None) == 5
    assert L.kcg_gemm_f32_ws(fake, fake, fake, 64, 64, 64, 0, None, fake, -1, None) == 5
    assert L.kcg_gemm_f32_ws(fake, fake, fake, 66000, 128, 33000, 0, None, None, 0, None) == 3
    assert L.kcg_gemm_f32_noalloc(None, fake, fake, 64, 64, 64, 0, None, None) == 1
    assert L.kcg_gemm_f32_noalloc(fake, fake, fake, -1, 64, 64, 0, None, None) == 2
    assert L.kcg_gemm_f32_noalloc(fake, fake, fake, 64, 64, 64, 9, None, None) == 5
    assert L.kcg_gemm_f32_noalloc(fake, fake, fake, 66000, 128, 33000, 0, None, None) == 3
    # a negative GROUP_SIZE_M on a K-split shape is refused like kcg_gemm_f32 refuses it, before
    # the split launch could number its tiles with it (status only: no device call is reached)
    neg = lib.GemmSched(group_m=-1)
    assert L.kcg_gemm_f32_ws(fake, fake, fake, 1536, 1536, 1536, 0, ctypes.byref(neg), fake, 1 << 26, None) == 4
    assert L.kcg_gemm_f32_noalloc(fake, fake, fake, 1536, 1536, 1536, 0, ctypes.byref(neg), None) == 4
    assert L.kcg_gemm_f32(fake, fake, fake, 1536, 1536, 1536, 0, ctypes.byref(neg), None) == 4
    assert L.kcg_gemm_f32_ws_bytes(1536, 1536, 1536, None) == 64 * 4 * 64 * 64 * 4
    assert L.kcg_gemm_f32_ws_bytes(1536, 1536, 256, None) == 0       # too little K to pay for a second launch
    assert L.kcg_gemm_f32_ws_bytes(4096, 4096, 4096, None) == 0      # the large tile, evenly filled
    assert L.kcg_gemm_f32_ws_bytes(1536, 1536, 1540, None) == 0      # not whole slices
    assert L.kcg_gemm_f32_ws_bytes(0, 1536, 1536, None) == 0
    # the launch pair of that plan, as the query entry point reports it
    info = lib.LaunchInfo()
    assert L.kcg_gemm_f32_ws_query(1536, 1536, 1536, None, 1 << 26, ctypes.byref(info)) == 0
    assert info.launches == 2 and info.grid[0] == 512 + 64 * 4 and info.block[0] == 256
    assert info.lds_bytes == 52224 and b"split" in info.kernel and b"reduce" in info.tail_kernel
    assert info.tail_grid[0] == 64 * 4 and info.main_rows == 1536 and info.tail_rows == 0
    plain = lib.LaunchInfo()
    assert L.kcg_gemm_f32_ws_query(1536, 1536, 1536, None, 0, ctypes.byref(info)) == 0
    assert L.kcg_gemm_f32_query(1536, 1536, 1536, None, ctypes.byref(plain)) == 0
    assert bytes(info) == bytes(plain)           # no room for a plan: the answer of the plain query
    assert L.kcg_gemm_f32_ws_query(1536, 1536, 1536, None, -1, ctypes.byref(info)) == 5
    assert L.kcg_gemm_f32_ws_query(1536, 1536, 1536, ctypes.byref(neg), 1 << 26, ctypes.byref(info)) == 4
    assert L.kcg_gemm_f32_ws_query(1536, 1536, 1536, None, 1 << 26, None) == 1
    fixed = lib.GemmSched(block_m=64, block_n=64, block_k=32, wave_m=32, wave_n=32)
    assert L.kcg_gemm_f32_ws_bytes(1536, 1536, 1536, ctypes.byref(fixed)) == 0
    assert L.kcg_gemm_f32_ws_bytes(1536, 1536, 1536, ctypes.byref(lib.GemmSched(group_m=4))) == 64 * 4 * 64 * 64 * 4
