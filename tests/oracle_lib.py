"""ctypes view of oracle/liboracle.so for the test-suite (checker only).

The oracle is test infrastructure: nothing under the shipped package imports
this module.  It is built by `make -C oracle` (or __graft_entry__.build()).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_SO = os.path.join(_ROOT, "oracle", "liboracle.so")

_u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
_i8p = np.ctypeslib.ndpointer(np.int8, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")


def _load():
    if not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", os.path.join(_ROOT, "oracle")])
    lib = C.CDLL(_SO)
    I = C.c_int
    sig = {
        "orc_f16_to_f32": (C.c_float, [C.c_uint16]),
        "orc_f32_to_f16": (C.c_uint16, [C.c_float]),
        "orc_f64_to_f16": (C.c_uint16, [C.c_double]),
        "orc_expf_export": (C.c_float, [C.c_float]),
        "orc_quantize_int8": (None, [_u16p, I, I, _i8p, _u16p]),
        "orc_quantize_q4": (I, [_u16p, I, I, _u8p, _u16p]),
        "orc_dequant_int8_to_f16": (None, [_i8p, _u16p, I, I, _u16p]),
        "orc_unpack_q4": (None, [_u8p, I, I, _i8p]),
        "orc_dequant_q4_to_f32": (None, [_u8p, _u16p, I, I, _f32p]),
        "orc_gemv_f16": (None, [_u16p, _u16p, _u16p, I, I, I]),
        "orc_gemv_i8": (None, [_u16p, _i8p, _u16p, _u16p, I, I, I]),
        "orc_gemv_q4": (None, [_u16p, _u8p, _u16p, _u16p, I, I, I]),
        "orc_gemv_i8_f32": (None, [_u16p, _i8p, _u16p, _f32p, I, I]),
        "orc_gemv_f16_add": (None, [_u16p, _u16p, _u16p, I, I]),
        "orc_gemv_i8_add": (None, [_u16p, _i8p, _u16p, _u16p, I, I]),
        "orc_gemv_q4_add": (None, [_u16p, _u8p, _u16p, _u16p, I, I]),
        "orc_gemv_f16_silu_gate": (None, [_u16p, _u16p, _u16p, I, I]),
        "orc_gemv_i8_silu_gate": (None, [_u16p, _i8p, _u16p, _u16p, I, I]),
        "orc_gemv_q4_silu_gate": (None, [_u16p, _u8p, _u16p, _u16p, I, I]),
        "orc_gate_up_silu_i8": (None, [_u16p, _i8p, _i8p, _u16p, _u16p, _u16p, I, I]),
        "orc_gate_up_silu_f16": (None, [_u16p, _u16p, _u16p, _u16p, I, I]),
        "orc_gemm_f16": (None, [_u16p, _u16p, _u16p, I, I, I, I]),
        "orc_gemm_i8": (None, [_u16p, _i8p, _u16p, _u16p, I, I, I, I]),
        "orc_gemm_q4": (None, [_u16p, _u8p, _u16p, _u16p, I, I, I, I]),
        "orc_max_threads": (I, []),
        "orc_build_flags": (C.c_char_p, []),
        "orc_argmax_f16": (I, [_u16p, I, I]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


lib = _load()
THREADS = min(8, lib.orc_max_threads())


def u16(a):
    """fp16 ndarray -> contiguous uint16 bit view."""
    return np.ascontiguousarray(a, dtype=np.float16).view(np.uint16)


def f16(a):
    return np.ascontiguousarray(a, dtype=np.uint16).view(np.float16)


def quantize_int8(w16):
    w = u16(w16)
    N, K = w.shape
    q = np.empty((N, K), np.int8)
    s = np.empty(N, np.uint16)
    lib.orc_quantize_int8(w, N, K, q, s)
    return q, s


def quantize_q4(w16):
    w = u16(w16)
    N, K = w.shape
    if K % 32:
        raise ValueError("Q4 requires K divisible by 32")
    p = np.empty((N, K // 2), np.uint8)
    s = np.empty((N, K // 32), np.uint16)
    rc = lib.orc_quantize_q4(w, N, K, p, s)
    assert rc == 0
    return p, s


def gemv_f16(x, W, threads=THREADS):
    N, K = W.shape
    y = np.empty(N, np.uint16)
    lib.orc_gemv_f16(u16(x), u16(W), y, N, K, threads)
    return y


def gemv_i8(x, q, s, threads=THREADS):
    N, K = q.shape
    y = np.empty(N, np.uint16)
    lib.orc_gemv_i8(u16(x), q, s, y, N, K, threads)
    return y


def gemv_q4(x, p, sc, threads=THREADS):
    N, K = p.shape[0], p.shape[1] * 2
    y = np.empty(N, np.uint16)
    lib.orc_gemv_q4(u16(x), p, np.ascontiguousarray(sc), y, N, K, threads)
    return y


def gemm_f16(X, W, threads=THREADS):
    M, K = X.shape
    N = W.shape[0]
    out = np.empty((M, N), np.uint16)
    lib.orc_gemm_f16(u16(X), u16(W), out, M, N, K, threads)
    return out


def gemm_i8(X, q, s, threads=THREADS):
    M, K = X.shape
    N = q.shape[0]
    out = np.empty((M, N), np.uint16)
    lib.orc_gemm_i8(u16(X), q, s, out, M, N, K, threads)
    return out


def gemm_q4(X, p, sc, threads=THREADS):
    M, K = X.shape
    N = p.shape[0]
    out = np.empty((M, N), np.uint16)
    lib.orc_gemm_q4(u16(X), p, np.ascontiguousarray(sc), out, M, N, K, threads)
    return out


def argmax_f16(x, num_partials=32):
    """x: fp16 values, or their uint16 bit patterns as the gemv_* functions return them."""
    x = np.asarray(x)
    x = (np.ascontiguousarray(x) if x.dtype == np.uint16 else u16(x)).reshape(-1)
    return lib.orc_argmax_f16(x, x.size, num_partials)
