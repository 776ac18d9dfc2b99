"""Loader and thin ctypes bindings of the C-ABI library (include/kcg.h).

The library is hand-written HIP for gfx950.  There is no CPU fallback: if the
shared object is missing, loading raises.  Device tensors are torch tensors;
torch is used for device memory and streams only.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# KCG_LIBRARY names another build of the same library (the experiment builds of
# `make -C kernelcodegen_amd/csrc variants`); unset, the library built beside this file.
LIB_PATH = os.environ.get("KCG_LIBRARY") or os.path.join(_HERE, "libkcg_hip.so")

_lib = None
_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_i32 = ctypes.c_int32


class KcgError(RuntimeError):
    def __init__(self, status, text):
        super().__init__("kcg status %d: %s" % (status, text))
        self.status = status


class GemmSched(ctypes.Structure):
    """kcg_gemm_sched: the reference's matmul tile table (include/KernelCodeGen.h:34-37)."""
    _fields_ = [("block_m", _i32), ("block_n", _i32), ("block_k", _i32), ("group_m", _i32),
                ("wave_m", _i32), ("wave_n", _i32), ("vec_width", _i32), ("wave_size", _i32),
                ("lds_stages", _i32)]


class FmhaSched(ctypes.Structure):
    """kcg_fmha_sched: Br / Bc of the reference's FMHA table (include/KernelCodeGen.h:38-41)."""
    _fields_ = [("br", _i32), ("bc", _i32)]


class LaunchInfo(ctypes.Structure):
    _fields_ = [("grid", _i32 * 3), ("block", _i32 * 3), ("lds_bytes", _i32),
                ("waves_per_block", _i32), ("kernel", ctypes.c_char * 64),
                ("launches", _i32), ("main_rows", _i32), ("tail_rows", _i32),
                ("tail_grid", _i32 * 3), ("tail_block", _i32 * 3), ("tail_lds_bytes", _i32),
                ("tail_kernel", ctypes.c_char * 64)]


# name -> (restype, argtypes); every symbol include/kcg.h declares.
SYMBOLS = {
    "kcg_status_str": (ctypes.c_char_p, [ctypes.c_int]),
    "kcg_version": (ctypes.c_char_p, []),
    "kcg_gemm_f32": (ctypes.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, ctypes.c_int,
                                    ctypes.POINTER(GemmSched), _vp]),
    "kcg_gemm_f32_ws_bytes": (ctypes.c_int64, [_i64, _i64, _i64, ctypes.POINTER(GemmSched)]),
    "kcg_gemm_f32_ws": (ctypes.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, ctypes.c_int,
                                       ctypes.POINTER(GemmSched), _vp, _i64, _vp]),
    "kcg_gemm_f32_ws_query": (ctypes.c_int, [_i64, _i64, _i64, ctypes.POINTER(GemmSched), _i64,
                                             ctypes.POINTER(LaunchInfo)]),
    "kcg_gemm_f32_noalloc": (ctypes.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, ctypes.c_int,
                                            ctypes.POINTER(GemmSched), _vp]),
    "kcg_gemm_f32_query": (ctypes.c_int, [_i64, _i64, _i64, ctypes.POINTER(GemmSched),
                                          ctypes.POINTER(LaunchInfo)]),
    "kcg_fmha_f32": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, ctypes.c_float,
                                    ctypes.c_int, ctypes.POINTER(FmhaSched), _vp]),
    "kcg_fmha_bf16": (ctypes.c_int, [_vp, _vp, _vp, _vp, ctypes.c_int, _i32, _i32, _i32, _i32,
                                     ctypes.c_float, ctypes.c_int, ctypes.POINTER(FmhaSched), _vp]),
    "kcg_fmha_query": (ctypes.c_int, [ctypes.c_int, _i32, _i32, _i32, _i32, ctypes.c_int,
                                      ctypes.POINTER(FmhaSched), ctypes.POINTER(LaunchInfo)]),
    "kcg_relu_f32": (ctypes.c_int, [_vp, _vp, _i64, _vp]),
    "kcg_batched_matmul_f32": (ctypes.c_int, [_vp, ctypes.c_int, _vp, ctypes.c_int, _vp, _i64,
                                              _i64, _i64, _i64, _vp]),
    "kcg_softmax_f32": (ctypes.c_int, [_vp, _i64, _i64, _vp]),
}


def load():
    """dlopen the HIP library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `make -C kernelcodegen_amd/csrc` "
                "(or __graft_entry__.build()); there is no CPU fallback" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            try:
                fn = getattr(L, name)
            except AttributeError:
                raise RuntimeError("%s does not export %s: rebuild it" % (LIB_PATH, name))
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def status_str(status):
    return load().kcg_status_str(int(status)).decode()


def check(status):
    if status != 0:
        raise KcgError(status, status_str(status))


def current_stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
