"""Device operators: torch tensors in, the gfx950 kernels underneath.

Names and argument meaning follow the reference's Frontend operators
(include/Frontend/Operators.h:73-102): Matmul, Relu, BatchedMatmul, Softmax,
and the fused attention the FMHAOptimizer recognises
(src/Optimizer/Optimizer.cc:586-672).  Everything goes through the C-ABI; a
failing status raises lib.KcgError.
"""
import ctypes

import torch

from . import lib

EPILOGUE_NONE = 0
EPILOGUE_RELU = 1
F32 = 0
BF16 = 1


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _dev_f32(t, name):
    if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()):
        raise ValueError("%s must be a contiguous fp32 device tensor" % name)


def _sched(sched, cls):
    if sched is None:
        return None
    if isinstance(sched, cls):
        return ctypes.byref(sched)
    return ctypes.byref(cls(**sched))


def matmul(A, B, relu=False, out=None, sched=None):
    """C = A.B (row-major fp32), optionally with the ReLU epilogue fused."""
    _dev_f32(A, "A")
    _dev_f32(B, "B")
    M, K = A.shape
    K2, N = B.shape
    if K != K2:
        raise ValueError("Can't apply Matmul Operation due to imcompatible K-dim.")
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=A.device)
    _dev_f32(out, "out")
    st = lib.load().kcg_gemm_f32(_ptr(A), _ptr(B), _ptr(out), M, N, K,
                                 EPILOGUE_RELU if relu else EPILOGUE_NONE,
                                 _sched(sched, lib.GemmSched), lib.current_stream())
    lib.check(st)
    return out


def relu(x, inplace=False, out=None):
    _dev_f32(x, "x")
    if out is not None:
        _dev_f32(out, "out")
        if out.numel() != x.numel():
            raise ValueError("relu: out must have as many elements as x")
    y = x if inplace else (out if out is not None else torch.empty_like(x))
    lib.check(lib.load().kcg_relu_f32(_ptr(x), _ptr(y), x.numel(), lib.current_stream()))
    return y


def batched_matmul(A, B, trans_a=False, trans_b=False, out=None):
    """C[b] = op(A[b]).op(B[b]); leading dims are the batch (Layout::colMajor = trans)."""
    _dev_f32(A, "A")
    _dev_f32(B, "B")
    batch_shape = tuple(A.shape[:-2])
    if tuple(B.shape[:-2]) != batch_shape:
        raise ValueError("BatchedMatmul: A, B dim not matched.")
    K, M = (A.shape[-2], A.shape[-1]) if trans_a else (A.shape[-1], A.shape[-2])
    K2, N = (B.shape[-1], B.shape[-2]) if trans_b else (B.shape[-2], B.shape[-1])
    if K != K2:
        raise ValueError("Can't apply BatchedMatmul Operation due to imcompatible K-dim.")
    batch = 1
    for d in batch_shape:
        batch *= d
    if out is None:
        out = torch.empty(batch_shape + (M, N), dtype=torch.float32, device=A.device)
    st = lib.load().kcg_batched_matmul_f32(_ptr(A), int(trans_a), _ptr(B), int(trans_b), _ptr(out),
                                           batch, M, N, K, lib.current_stream())
    lib.check(st)
    return out


def softmax_(x):
    """In-place softmax over the last axis (the reference operator is in place)."""
    _dev_f32(x, "x")
    n = x.shape[-1]
    lib.check(lib.load().kcg_softmax_f32(_ptr(x), x.numel() // n, n, lib.current_stream()))
    return x


def fmha(Q, K, V, scale=1.0, causal=False, out=None, out_dtype=None, sched=None):
    """O = softmax(scale * Q.K^T [+causal]) . V for [B,H,S,D] tensors.

    fp32 tensors run the fp32 kernel; bf16 tensors the bf16 kernel (fp32
    accumulation and softmax), writing `out_dtype` (bf16 by default).
    """
    if not (Q.is_cuda and Q.is_contiguous() and K.is_contiguous() and V.is_contiguous()):
        raise ValueError("Q, K, V must be contiguous device tensors")
    if Q.shape != K.shape or Q.shape != V.shape or Q.dim() != 4:
        raise ValueError("Q, K, V must share one [B,H,S,D] shape")
    B_, H, S, D = Q.shape
    L = lib.load()
    if Q.dtype == torch.float32:
        if out is None:
            out = torch.empty_like(Q)
        st = L.kcg_fmha_f32(_ptr(Q), _ptr(K), _ptr(V), _ptr(out), B_, H, S, D, float(scale),
                            int(causal), _sched(sched, lib.FmhaSched), lib.current_stream())
    elif Q.dtype == torch.bfloat16:
        if out is None:
            out = torch.empty(Q.shape, dtype=out_dtype or torch.bfloat16, device=Q.device)
        o_dtype = BF16 if out.dtype == torch.bfloat16 else F32
        st = L.kcg_fmha_bf16(_ptr(Q), _ptr(K), _ptr(V), _ptr(out), o_dtype, B_, H, S, D,
                             float(scale), int(causal), _sched(sched, lib.FmhaSched),
                             lib.current_stream())
    else:
        raise ValueError("fmha supports float32 and bfloat16")
    lib.check(st)
    return out
