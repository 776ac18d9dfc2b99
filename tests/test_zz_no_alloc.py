"""kcg_gemm_f32_noalloc: the K-split matmul plan with its partial sums in the library's own
static device array, against kcg_gemm_f32_ws with a workspace lent by the caller.

Lent the 4 MiB the static array has, the workspace entry point picks the same plan and runs
the same two kernels on the same operands, so the results must be equal bit for bit; the
oracle bounds both.  Calls in a row on smaller problems (fewer and other pieces in the same
array): one whose preferred plan would need 10.5 MiB and runs with two pieces per tile
instead of eight, then one without a K-split plan.
"""
import ctypes

import numpy as np
import pytest

from conftest import rel_err
from kernelcodegen_amd import inputs

pytestmark = pytest.mark.gpu


def _gpu(x, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).to(dev)


def test_noalloc_entry_point_matches_the_workspace_entry_point(oracle, dev):
    import torch
    from kernelcodegen_amd import lib
    L = lib.load()
    stream = lib.current_stream()
    vp = ctypes.c_void_p
    array_bytes = 4 << 20
    for seed, (M, N, K), relu in [(451, (1536, 1536, 1536), 1), (452, (1024, 1088, 1536), 0),
                                  (454, (1280, 1088, 2048), 1), (453, (512, 512, 512), 1)]:
        A = inputs.normal((M, K), seed, 0)
        B = inputs.normal((K, N), seed, 1)
        ref = oracle.matmul(A, B)
        if relu:
            ref = oracle.relu(ref)
        tA, tB = _gpu(A, dev), _gpu(B, dev)
        need = int(L.kcg_gemm_f32_ws_bytes(M, N, K, None))
        assert (need > 0) == (K != 512) and (need > array_bytes) == (K == 2048)
        ws = torch.empty(array_bytes // 4, dtype=torch.float32, device=dev)
        C_ws = torch.full((M, N), -3.0, dtype=torch.float32, device=dev)
        C_na = torch.full((M, N), -5.0, dtype=torch.float32, device=dev)
        assert L.kcg_gemm_f32_ws(vp(tA.data_ptr()), vp(tB.data_ptr()), vp(C_ws.data_ptr()), M, N, K, relu, None,
                                 vp(ws.data_ptr()), array_bytes, stream) == 0
        assert L.kcg_gemm_f32_noalloc(vp(tA.data_ptr()), vp(tB.data_ptr()), vp(C_na.data_ptr()), M, N, K, relu, None,
                                      stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(C_na, C_ws), (M, N, K)
        assert max(rel_err(C_na.cpu().numpy(), ref)) < 1e-4
    # argument checks are those of kcg_gemm_f32
    assert L.kcg_gemm_f32_noalloc(None, None, None, 64, 64, 64, 0, None, stream) == 1
    assert L.kcg_gemm_f32_noalloc(vp(tA.data_ptr()), vp(tB.data_ptr()), vp(C_na.data_ptr()), 0, 64, 64, 0, None,
                                  stream) == 2
