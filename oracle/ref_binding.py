"""ctypes binding of oracle/_ref/libref_cpu.so: the reference's own CPU
translation units behind the C wrappers of ref_shim.cpp.

TEST INFRASTRUCTURE ONLY.  The library exists only where the reference
checkout was present at build time; available() says whether it does.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "_ref", "libref_cpu.so")
_lib = None


def available():
    return os.path.exists(LIB_PATH)


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(LIB_PATH)
        _lib.ref_moe_middle_row.restype = C.c_float
        _lib.ref_moe_middle_row.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_float, C.c_void_p]
    return _lib


def _p(a):
    return C.c_void_p(a.ctypes.data)


def w8_scales(A):
    M, K = A.shape
    s = np.empty(M, np.float32)
    (lib().ref_w8_scales_f16 if A.dtype == np.uint16 else lib().ref_w8_scales_f32)(M, K, _p(A), _p(s))
    return s


def w8_quant(A, scale):
    M, K = A.shape
    q = np.empty((M, K), np.int8)
    scale = np.ascontiguousarray(scale, np.float32)
    (lib().ref_w8_quant_f16 if A.dtype == np.uint16 else lib().ref_w8_quant_f32)(M, K, _p(A), _p(scale), _p(q))
    return q


def w8_dequant(acc, a_scale, w_scale, half):
    acc = np.ascontiguousarray(acc, np.int32)
    M, N = acc.shape
    a_scale = np.ascontiguousarray(a_scale, np.float32)
    w_scale = np.ascontiguousarray(w_scale, np.float32)
    out = np.empty((M, N), np.uint16 if half else np.float32)
    (lib().ref_w8_dequant_f16 if half else lib().ref_w8_dequant_f32)(M, N, _p(acc), _p(a_scale), _p(w_scale), _p(out))
    return out


def w8_reduce_two(acc0, acc1):
    acc0 = np.ascontiguousarray(acc0, np.int32)
    acc1 = np.ascontiguousarray(acc1, np.int32)
    M, N = acc0.shape
    out = np.empty((M, N), np.int32)
    lib().ref_w8_reduce_two_i32(M, N, _p(acc0), _p(acc1), _p(out))
    return out


def w4a8_scales(A):
    M, K = A.shape
    s = np.empty(M, np.float32)
    inv = np.empty(M, np.float32)
    rc = lib().ref_w4a8_scales(_p(A), 1 if A.dtype == np.uint16 else 0, M, K, _p(s), _p(inv))
    return rc, s, inv


def w4a8_quant(A, scales, inverse):
    M, K = A.shape
    q = np.empty((M, K), np.int8)
    rc = lib().ref_w4a8_quant(_p(A), 1 if A.dtype == np.uint16 else 0, M, K, _p(scales), _p(inverse), _p(q))
    return rc, q


def w4a8_dequant(acc, a_scale, w_scale, half):
    acc = np.ascontiguousarray(acc, np.int32)
    M, N = acc.shape
    a_scale = np.ascontiguousarray(a_scale, np.float32)
    w_scale = np.ascontiguousarray(w_scale, np.float32)
    out = np.empty((M, N), np.uint16 if half else np.float32)
    lib().ref_w4a8_dequant(M, N, _p(acc), _p(a_scale), _p(w_scale), 1 if half else 0, _p(out))
    return out


def finish_scales(bits):
    bits = np.ascontiguousarray(bits, np.uint32)
    s = np.empty(bits.size, np.float32)
    inv = np.empty(bits.size, np.float32)
    rc = lib().ref_w4a8_finish_scales(bits.size, _p(bits), _p(s), _p(inv))
    return rc, s, inv


def moe_middle_row(acc, weight_scales, input_scale):
    acc = np.ascontiguousarray(acc, np.int32)
    channels = acc.size // 2
    ws = np.ascontiguousarray(weight_scales, np.float32)
    q = np.empty(channels, np.int8)
    s = lib().ref_moe_middle_row(_p(acc), channels, _p(ws), C.c_float(input_scale), _p(q))
    return float(np.float32(s)), q


def bound_i4(B, requested=0):
    B = np.ascontiguousarray(B, np.int8)
    K, N = B.shape
    return lib().ref_bound_i4(K, N, _p(B), requested)
