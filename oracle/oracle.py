"""ctypes front end of the CPU oracle (oracle/kcg_oracle.c).

Test infrastructure only: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py, never by the product package.  All arguments are
C-contiguous numpy arrays; results are new numpy arrays.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libkcg_oracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_i64 = ctypes.c_int64


def build(force=False):
    """Compile the oracle with the committed Makefile."""
    if force or not os.path.exists(_LIB_PATH):
        args = ["make", "-C", _HERE] + (["-B"] if force else [])
        subprocess.run(args, check=True, capture_output=True)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        L.kcg_oracle_num_threads.restype = ctypes.c_int
        L.kcg_oracle_matmul_f32_literal.argtypes = [_f32p, _f32p, _f32p, _i64, _i64, _i64]
        L.kcg_oracle_matmul_f32.argtypes = [_f32p, _f32p, _f32p, _i64, _i64, _i64]
        L.kcg_oracle_matmul_f32_rows.argtypes = [_f32p, _f32p, _f32p, _i64, _i64, _i64, _i64, _i64]
        L.kcg_oracle_relu_f32.argtypes = [_f32p, _f32p, _i64]
        L.kcg_oracle_batched_matmul_f32.argtypes = [
            _f32p, ctypes.c_int, _f32p, ctypes.c_int, _f32p, _i64, _i64, _i64, _i64]
        L.kcg_oracle_softmax_f32.argtypes = [_f32p, _i64, _i64]
        L.kcg_oracle_fmha_f32.argtypes = [
            _f32p, _f32p, _f32p, _f32p, _i64, _i64, _i64, _i64,
            ctypes.c_float, ctypes.c_int, ctypes.c_int]
        L.kcg_oracle_fmha_f32_rows.argtypes = L.kcg_oracle_fmha_f32.argtypes + [_i64, _i64]
        L.kcg_oracle_fmha_bf16_rows.argtypes = [
            _u16p, _u16p, _u16p, _f32p, _i64, _i64, _i64, _i64,
            ctypes.c_float, ctypes.c_int, ctypes.c_int, _i64, _i64]
        L.kcg_oracle_bf16_to_f32.argtypes = [_u16p, _f32p, _i64]
        L.kcg_oracle_f32_to_bf16.argtypes = [_f32p, _u16p, _i64]
        _lib = L
    return _lib


def num_threads():
    return int(lib().kcg_oracle_num_threads())


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_f32p)


def _u16(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint16, "bf16 tensors are passed as uint16 bit patterns"
    return a, a.ctypes.data_as(_u16p)


def matmul(A, B, literal=False):
    A, pa = _f32(A)
    B, pb = _f32(B)
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    C = np.empty((M, N), dtype=np.float32)
    fn = lib().kcg_oracle_matmul_f32_literal if literal else lib().kcg_oracle_matmul_f32
    fn(pa, pb, C.ctypes.data_as(_f32p), M, N, K)
    return C


def matmul_rows(A, B, row_begin, row_end):
    """Rows [row_begin,row_end) of A.B as a (row_end-row_begin, N) array."""
    A, pa = _f32(A)
    B, pb = _f32(B)
    M, K = A.shape
    N = B.shape[1]
    C = np.empty((M, N), dtype=np.float32) if (row_begin, row_end) == (0, M) else None
    if C is None:
        # Only the sampled rows are materialised: offset the C pointer so that
        # row `row_begin` lands at the start of the small buffer.
        out = np.empty((row_end - row_begin, N), dtype=np.float32)
        base = out.ctypes.data - row_begin * N * 4
        pc = ctypes.cast(ctypes.c_void_p(base), _f32p)
        lib().kcg_oracle_matmul_f32_rows(pa, pb, pc, M, N, K, row_begin, row_end)
        return out
    lib().kcg_oracle_matmul_f32_rows(pa, pb, C.ctypes.data_as(_f32p), M, N, K, 0, M)
    return C


def relu(x):
    x, px = _f32(x)
    y = np.empty_like(x)
    lib().kcg_oracle_relu_f32(px, y.ctypes.data_as(_f32p), x.size)
    return y


def batched_matmul(A, transA, B, transB):
    A, pa = _f32(A)
    B, pb = _f32(B)
    batch_shape = A.shape[:-2]
    batch = int(np.prod(batch_shape)) if batch_shape else 1
    if transA:
        K, M = A.shape[-2:]
    else:
        M, K = A.shape[-2:]
    if transB:
        N, K2 = B.shape[-2:]
    else:
        K2, N = B.shape[-2:]
    assert K == K2 and B.shape[:-2] == batch_shape
    C = np.empty(batch_shape + (M, N), dtype=np.float32)
    lib().kcg_oracle_batched_matmul_f32(pa, int(transA), pb, int(transB),
                                        C.ctypes.data_as(_f32p), batch, M, N, K)
    return C


def softmax(x):
    """Last-axis softmax of a copy of x (the reference operator is in place)."""
    y = np.array(x, dtype=np.float32, order="C", copy=True)
    n = y.shape[-1]
    lib().kcg_oracle_softmax_f32(y.ctypes.data_as(_f32p), y.size // n, n)
    return y


def fmha(Q, K, V, scale=1.0, causal=False, stable=False, rows=None):
    """O = softmax(scale * Q.K^T [+ causal mask]) . V for [B,H,S,D] tensors.

    fp32 inputs, or uint16 arrays holding bf16 bit patterns (widened exactly).
    rows=(r0, r1) computes only query rows r0..r1-1 of every head and returns
    a [B,H,r1-r0,D] array.
    """
    B_, H, S, D = Q.shape
    r0, r1 = rows if rows is not None else (0, S)
    full = np.zeros((B_, H, S, D), dtype=np.float32)
    po = full.ctypes.data_as(_f32p)
    if Q.dtype == np.uint16:
        Q, pq = _u16(Q)
        K, pk = _u16(K)
        V, pv = _u16(V)
        lib().kcg_oracle_fmha_bf16_rows(pq, pk, pv, po, B_, H, S, D, float(scale),
                                        int(causal), int(stable), r0, r1)
    else:
        Q, pq = _f32(Q)
        K, pk = _f32(K)
        V, pv = _f32(V)
        lib().kcg_oracle_fmha_f32_rows(pq, pk, pv, po, B_, H, S, D, float(scale),
                                       int(causal), int(stable), r0, r1)
    if rows is None:
        return full
    return np.ascontiguousarray(full[:, :, r0:r1, :])


def bf16_to_f32(x):
    x, px = _u16(x)
    y = np.empty(x.shape, dtype=np.float32)
    lib().kcg_oracle_bf16_to_f32(px, y.ctypes.data_as(_f32p), x.size)
    return y


def f32_to_bf16(x):
    x, px = _f32(x)
    y = np.empty(x.shape, dtype=np.uint16)
    lib().kcg_oracle_f32_to_bf16(px, y.ctypes.data_as(_u16p), x.size)
    return y
