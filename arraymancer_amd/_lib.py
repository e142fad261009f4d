"""ctypes binding of libam_hip.so — the same C ABI (include/am_hip.h) a Nim `{.importc.}` layer
binds. There is no fallback: if the library is missing or a call fails, an exception is raised."""
from __future__ import annotations

import ctypes
import os

import numpy as np

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
# AM_HIP_LIBRARY overrides the location of the built library (same role as -d:libAmHip=... in Nim).
LIB_PATH = os.environ.get("AM_HIP_LIBRARY") or os.path.join(PKG_DIR, "libam_hip.so")

AM_OK, AM_E_ARG, AM_E_SHAPE, AM_E_DTYPE, AM_E_ALLOC, AM_E_HIP, AM_E_NODEVICE = 0, -1, -2, -3, -4, -5, -6
AM_MAXRANK = 6

OP = dict(add=0, sub=1, mul=2, div=3, mod=4, add_relu=5, add_sigmoid=6, add_tanh=7,
          relu_bwd=8, max=9, min=10, sigmoid_bwd=11, tanh_bwd=12, sqdiff=13, pow=14, floormod=15, copysign=16)
CMP = {"==": 0, "!=": 1, "<": 2, "<=": 3, ">": 4, ">=": 5, "mod_is_zero": 6}
PRED = dict(isnan=0, isnotnan=1, classify=2)
OP3 = dict(muladd=0, gru_candidate=1, gru_blend=2, addmul=3, clamp=4)
UOP = dict(copy=0, neg=1, relu=2, sigmoid=3, tanh=4, exp=5, abs=6, sqrt=7, square=8,
           ln=9, log10=10, log2=11, sin=12, cos=13, tan=14, sinh=15, cosh=16, arcsin=17,
           arccos=18, arctan=19, arcsinh=20, arccosh=21, arctanh=22, cbrt=23, erf=24, erfc=25, gamma=26,
           lgamma=27, floor=28, ceil=29, trunc=30, round=31, reciprocal=32, degtorad=33, radtodeg=34, fac=35)
EPI = dict(none=0, bias=1, relu=2, bias_relu=3)
RED = dict(sum=0, product=1, min=2, max=3)

SFX = {np.dtype(np.float32): "f32", np.dtype(np.float64): "f64",
       np.dtype(np.int32): "i32", np.dtype(np.int64): "i64"}
CTYPE = {"f32": ctypes.c_float, "f64": ctypes.c_double, "i32": ctypes.c_int32, "i64": ctypes.c_int64}


class HipError(RuntimeError):
    """A HIP runtime call failed, no device is usable, or the library is missing."""


class HipAllocError(HipError, MemoryError):
    pass


# Every symbol include/am_hip.h declares, with its ctypes signature.
def _signatures():
    ci, i64, vp, sz = ctypes.c_int, ctypes.c_int64, ctypes.c_void_p, ctypes.c_size_t
    pp = ctypes.POINTER(ctypes.c_void_p)
    sig = {
        "am_hip_last_error": (ctypes.c_char_p, []),
        "am_hip_version": (ctypes.c_char_p, []),
        "am_hip_init": (ci, [ci]),
        "am_hip_device_count": (ci, [ctypes.POINTER(ci)]),
        "am_hip_device_info": (ci, [ctypes.c_char_p, sz, ctypes.POINTER(ci), ctypes.POINTER(ci),
                                    ctypes.POINTER(sz), ctypes.POINTER(ci)]),
        "am_hip_malloc": (ci, [sz, pp]),
        "am_hip_free": (ci, [vp]),
        "am_hip_memcpy_h2d": (ci, [vp, vp, sz]),
        "am_hip_memcpy_d2h": (ci, [vp, vp, sz]),
        "am_hip_memcpy_d2d": (ci, [vp, vp, sz]),
        "am_hip_memset": (ci, [vp, ci, sz]),
        "am_hip_sync": (ci, []),
        "am_hip_stream": (vp, []),
        "am_hip_empty_cache": (ci, []),
        "am_hip_memory_stats": (ci, [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]),
        "am_hip_device_free_bytes": (ci, [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]),
        "am_hip_event_create": (ci, [pp]),
        "am_hip_event_record": (ci, [vp]),
        "am_hip_event_elapsed_ms": (ci, [vp, vp, ctypes.POINTER(ctypes.c_float)]),
        "am_hip_event_destroy": (ci, [vp]),
        "am_hip_graph_begin": (ci, []),
        "am_hip_alloc_hold": (ci, [ci]),
        "am_hip_graph_end": (ci, [pp]),
        "am_hip_graph_launch": (ci, [vp]),
        "am_hip_graph_destroy": (ci, [vp]),
        "am_hip_digits_release": (ci, [vp]),
        "am_hip_diag_peak": (ci, [ci, ci, ci, ctypes.POINTER(ctypes.c_double)]),
        "am_hip_diag_clock_begin": (ci, []),
        "am_hip_diag_clock_end": (ci, [ctypes.POINTER(ctypes.c_double)]),
        "am_hip_diag_phases_begin": (ci, []),
        "am_hip_diag_phases": (ci, [ctypes.POINTER(ctypes.c_double)]),
        "am_hip_diag_hbm": (ci, [ci, sz, ci, ci, ci, ci, ci, ctypes.POINTER(ctypes.c_double)]),
    }
    for sfx, ct in CTYPE.items():
        gemm = [i64, i64, i64, ct, vp, i64, i64, vp, i64, i64, ct, vp, i64, i64]
        sig[f"am_hip_gemm_{sfx}"] = (ci, gemm)
        if sfx == "f32":
            sig["am_hip_gemm_noalloc_f32"] = (ci, gemm)
        if sfx in ("i32", "i64"):
            sig[f"am_hip_digits_prepare_{sfx}"] = (ci, [ci, i64, i64, vp, i64, i64, pp])
            sig[f"am_hip_gemm_prepared_{sfx}"] = (ci, [i64, i64, i64, ct, vp, i64, i64, vp, vp, i64, i64, vp, ct, vp, i64, i64])
        if sfx in ("f32", "f64"):
            sig[f"am_hip_gemm_ex_{sfx}"] = (ci, gemm + [ci, vp, i64, i64])
        sig[f"am_hip_gemm_batched_{sfx}"] = (ci, [i64, i64, i64, i64, ct, vp, i64, i64, i64, vp, i64, i64, i64, ct,
                                                 vp, i64, i64, i64, ci, vp, i64, i64])
        sig[f"am_hip_im2col_{sfx}"] = (ci, [i64, ci, ci, ci, ci, ci, ci, ci, ci, ci, vp, i64, i64, i64, i64, vp])
        sig[f"am_hip_im2col_strided_{sfx}"] = (ci, [i64, ci, ci, ci, ci, ci, ci, ci, ci, ci, vp, i64, i64, i64, i64, vp, i64, i64])
        sig[f"am_hip_col2im_{sfx}"] = (ci, [i64, ci, ci, ci, ci, ci, ci, ci, ci, ci, vp, i64, i64, vp, i64, i64, i64, i64])
        sig[f"am_hip_gemv_{sfx}"] = (ci, [i64, i64, ct, vp, i64, i64, vp, i64, ct, vp, i64])
        sig[f"am_hip_dot_{sfx}"] = (ci, [i64, vp, i64, vp, i64, ctypes.POINTER(ct)])
        sig[f"am_hip_ew_binary_{sfx}"] = (ci, [ci, ci, vp, vp, vp, vp, vp, vp, vp])
        sig[f"am_hip_ew_scalar_{sfx}"] = (ci, [ci, ci, ci, vp, vp, vp, vp, vp, ct])
        sig[f"am_hip_ew_ternary_{sfx}"] = (ci, [ci, ci, vp, vp, vp, vp, vp, vp, vp, vp, vp])
        sig[f"am_hip_ew_unary_{sfx}"] = (ci, [ci, ci, vp, vp, vp, vp, vp])
        sig[f"am_hip_ew_compare_{sfx}"] = (ci, [ci, ci, vp, vp, vp, vp, vp, vp, vp])
        sig[f"am_hip_ew_compare_scalar_{sfx}"] = (ci, [ci, ci, vp, vp, vp, vp, vp, ct])
        sig[f"am_hip_ew_sgn_{sfx}"] = (ci, [ci, vp, vp, vp, vp, vp])
        sig[f"am_hip_ew_clamp_{sfx}"] = (ci, [ci, vp, vp, vp, vp, vp, ct, ct])
        if sfx in ("f32", "f64"):
            sig[f"am_hip_ew_predicate_{sfx}"] = (ci, [ci, ci, vp, vp, vp, vp, vp])
        sig[f"am_hip_reduce_axis_{sfx}"] = (ci, [ci, ci, vp, ci, vp, vp, vp, vp])
        sig[f"am_hip_argreduce_{sfx}"] = (ci, [ci, ci, vp, ci, vp, vp, vp, vp, vp, vp])
        sig[f"am_hip_reduce_all_{sfx}"] = (ci, [ci, ci, vp, vp, vp, ctypes.POINTER(ct)])
        sig[f"am_hip_maxpool2d_backward_{sfx}"] = (ci, [i64, ci, ci, ci, ci, ci, ci, ci, ci, ci, vp, vp, vp])
        sig[f"am_hip_maxpool2d_{sfx}"] = (ci, [i64, ci, ci, ci, ci, ci, ci, ci, ci, ci, vp, vp, vp])
        if sfx in ("f32", "f64"):
            sig[f"am_hip_conv2d_{sfx}"] = (ci, [i64, ci, ci, ci, ci, ci, ci, ci, ci, ci, ci, vp, i64, i64, i64, i64, vp, i64, ci, vp, i64, vp])
            sig[f"am_hip_conv2d_grad_weight_{sfx}"] = (ci, [i64, ci, ci, ci, ci, ci, ci, ci, ci, ci, ci, vp, i64, i64, i64, i64, vp, i64, vp])
            sig[f"am_hip_softmax_rows_{sfx}"] = (ci, [i64, i64, vp, i64, i64, vp, i64, i64])
            sig[f"am_hip_sgd_update_{sfx}"] = (ci, [ci, vp, vp, vp, ct])
            sig[f"am_hip_gru_gates_{sfx}"] = (ci, [i64, i64, vp, i64, vp, i64, vp, i64, vp, vp, vp, vp, i64])
            sig[f"am_hip_gru_gates_backward_{sfx}"] = (ci, [i64, i64, vp, vp, vp, vp, vp, vp, i64, vp, i64, vp, i64])
            sig[f"am_hip_softmax_cross_entropy_{sfx}"] = (ci, [i64, i64, vp, i64, i64, vp, i64, i64, ctypes.POINTER(ct)])
            sig[f"am_hip_sigmoid_cross_entropy_{sfx}"] = (ci, [i64, i64, vp, i64, i64, vp, i64, i64, ctypes.POINTER(ct)])
            sig[f"am_hip_sigmoid_cross_entropy_backward_{sfx}"] = (ci, [i64, i64, ct, vp, i64, i64, vp, i64, i64, vp, i64, i64])
            sig[f"am_hip_sparse_softmax_cross_entropy_{sfx}"] = (ci, [i64, i64, vp, i64, i64, vp, i64, ctypes.POINTER(ct)])
            sig[f"am_hip_softmax_cross_entropy_backward_{sfx}"] = (ci, [i64, i64, ct, vp, i64, i64, vp, i64, i64, vp, i64, i64])
            sig[f"am_hip_sparse_softmax_cross_entropy_backward_{sfx}"] = (ci, [i64, i64, ct, vp, i64, i64, vp, i64, vp, i64, i64])
    return sig


SIGNATURES = _signatures()
_lib = None


def load() -> ctypes.CDLL:
    """Loads the built library (no build is attempted here) and binds every exported symbol."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HipError(f"{LIB_PATH} is missing: build it with `python -m arraymancer_amd.build` "
                       f"(there is no CPU fallback)")
    L = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(L, name)          # AttributeError here = the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def last_error() -> str:
    return (load().am_hip_last_error() or b"").decode("utf-8", "replace")


def check(rc: int) -> None:
    """Maps a status code to the exception the reference raises in the same situation:
    shape problems are ValueError (src/arraymancer/tensor/private/p_checks_cuda.nim:15-19),
    everything the device reports is HipError."""
    if rc == AM_OK:
        return
    msg = last_error()
    if rc in (AM_E_ARG, AM_E_SHAPE):
        raise ValueError(msg)
    if rc == AM_E_DTYPE:
        raise TypeError(msg)
    if rc == AM_E_ALLOC:
        raise HipAllocError(msg)
    raise HipError(f"[{rc}] {msg}")


def i64_array(values):
    values = [int(v) for v in values]
    return (ctypes.c_int64 * max(1, len(values)))(*values)
