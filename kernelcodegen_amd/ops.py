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


def _check(t, name, dtype, shape, device):
    """The kernels take raw pointers: a tensor of another dtype, shape, device or layout
    would make them read or write out of bounds, so it is refused here."""
    if not isinstance(t, torch.Tensor):
        raise ValueError("%s must be a tensor" % name)
    if not t.is_cuda or t.device != device:
        raise ValueError("%s must be on device %s" % (name, device))
    if t.dtype != dtype:
        raise ValueError("%s must have dtype %s, not %s" % (name, dtype, t.dtype))
    if tuple(t.shape) != tuple(shape):
        raise ValueError("%s must have shape %s, not %s" % (name, tuple(shape), tuple(t.shape)))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)


def _sched(sched, cls):
    if sched is None:
        return None
    if isinstance(sched, cls):
        return ctypes.byref(sched)
    return ctypes.byref(cls(**sched))


def matmul_workspace_bytes(M, N, K, sched=None):
    """Bytes of workspace with which matmul() can run its K-split plan (0: there is none)."""
    return int(lib.load().kcg_gemm_f32_ws_bytes(M, N, K, _sched(sched, lib.GemmSched)))


def matmul(A, B, relu=False, out=None, sched=None, workspace=None):
    """C = A.B (row-major fp32), optionally with the ReLU epilogue fused.

    workspace: a contiguous device tensor the call may use for partial sums
    (kcg_gemm_f32_ws; see matmul_workspace_bytes).  Nothing else may use it until the
    call has completed on the current stream.
    """
    _dev_f32(A, "A")
    _dev_f32(B, "B")
    M, K = A.shape
    K2, N = B.shape
    if K != K2:
        raise ValueError("Can't apply Matmul Operation due to imcompatible K-dim.")
    if B.device != A.device:
        raise ValueError("A and B must be on the same device")
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=A.device)
    _check(out, "out", torch.float32, (M, N), A.device)
    epilogue = EPILOGUE_RELU if relu else EPILOGUE_NONE
    if workspace is not None:
        if not (isinstance(workspace, torch.Tensor) and workspace.is_cuda and workspace.device == A.device
                and workspace.is_contiguous()):
            raise ValueError("workspace must be a contiguous tensor on %s" % A.device)
        st = lib.load().kcg_gemm_f32_ws(_ptr(A), _ptr(B), _ptr(out), M, N, K, epilogue,
                                        _sched(sched, lib.GemmSched), _ptr(workspace),
                                        workspace.numel() * workspace.element_size(), lib.current_stream())
    else:
        st = lib.load().kcg_gemm_f32(_ptr(A), _ptr(B), _ptr(out), M, N, K, epilogue,
                                     _sched(sched, lib.GemmSched), lib.current_stream())
    lib.check(st)
    return out


def relu(x, inplace=False, out=None):
    _dev_f32(x, "x")
    if out is not None:
        _dev_f32(out, "out")
        if out.numel() != x.numel() or out.device != x.device:
            raise ValueError("relu: out must have as many elements as x, on the same device")
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
    if B.device != A.device:
        raise ValueError("A and B must be on the same device")
    if out is None:
        out = torch.empty(batch_shape + (M, N), dtype=torch.float32, device=A.device)
    _check(out, "out", torch.float32, batch_shape + (M, N), A.device)
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
    if not isinstance(Q, torch.Tensor) or Q.dim() != 4:
        raise ValueError("Q, K, V must share one [B,H,S,D] shape")
    if Q.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("fmha supports float32 and bfloat16")
    if not Q.is_cuda:
        raise ValueError("Q, K, V must be contiguous device tensors")
    for t, name in ((Q, "Q"), (K, "K"), (V, "V")):
        _check(t, name, Q.dtype, Q.shape, Q.device)
    B_, H, S, D = Q.shape
    if Q.dtype == torch.float32:
        if out_dtype not in (None, torch.float32):
            raise ValueError("fp32 attention writes fp32: out_dtype must be float32")
        want = torch.float32
    else:
        if out_dtype not in (None, torch.bfloat16, torch.float32):
            raise ValueError("bf16 attention writes bfloat16 or float32, not %s" % out_dtype)
        want = out_dtype or (out.dtype if out is not None else torch.bfloat16)
        if want not in (torch.bfloat16, torch.float32):
            raise ValueError("out must be bfloat16 or float32, not %s" % want)
    if out is not None:
        _check(out, "out", want, Q.shape, Q.device)
    L = lib.load()
    if Q.dtype == torch.float32:
        if out is None:
            out = torch.empty_like(Q)
        st = L.kcg_fmha_f32(_ptr(Q), _ptr(K), _ptr(V), _ptr(out), B_, H, S, D, float(scale),
                            int(causal), _sched(sched, lib.FmhaSched), lib.current_stream())
    else:
        if out is None:
            out = torch.empty(Q.shape, dtype=want, device=Q.device)
        o_dtype = BF16 if out.dtype == torch.bfloat16 else F32
        st = L.kcg_fmha_bf16(_ptr(Q), _ptr(K), _ptr(V), _ptr(out), o_dtype, B_, H, S, D,
                             float(scale), int(causal), _sched(sched, lib.FmhaSched),
                             lib.current_stream())
    lib.check(st)
    return out
