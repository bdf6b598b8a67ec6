"""ctypes binding of liboracle.so (the CPU restatement in rk_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke check and the CPU
baseline leg of bench.py -- never by the shipped package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")
EXP_POLY, EXP_LIBM = 0, 1
ERR_PARAM = -3

_lib = None


def build():
    subprocess.check_call(["make", "-C", HERE, "liboracle.so"], stdout=subprocess.DEVNULL)
    return LIB_PATH


class MoeExpert(C.Structure):
    _fields_ = [("gate_up", C.c_void_p), ("gate_up_scales", C.c_void_p),
                ("down", C.c_void_p), ("down_scales", C.c_void_p)]


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = C.CDLL(LIB_PATH)
        _lib.orc_half_to_float.restype = C.c_float
        _lib.orc_half_to_float.argtypes = [C.c_uint16]
        _lib.orc_float_to_half.restype = C.c_uint16
        _lib.orc_float_to_half.argtypes = [C.c_float]
        _lib.orc_silu_mul.restype = C.c_float
        _lib.orc_silu_mul.argtypes = [C.c_float, C.c_float, C.c_int]
        _lib.orc_moe_quant_row.restype = C.c_float
        _lib.orc_num_threads.restype = C.c_int
    return _lib


def _p(a):
    return C.c_void_p(a.ctypes.data) if a is not None else C.c_void_p(0)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def num_threads():
    return lib().orc_num_threads()


def half_to_float(bits):
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, np.float32)
    lib().orc_half_to_float_n(_p(bits), _p(out), C.c_int64(bits.size))
    return out


def float_to_half(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_float_to_half_n(_p(x), _p(out), C.c_int64(x.size))
    return out


def w8_scales(A):
    """A: [M,K] float32 or uint16 (fp16 bits)."""
    M, K = A.shape
    s = np.empty(M, np.float32)
    if A.dtype == np.uint16:
        lib().orc_w8_scales_f16(M, K, _p(A), _p(s))
    else:
        lib().orc_w8_scales_f32(M, K, _p(_c(A, np.float32)), _p(s))
    return s


def w8_quant(A, scale):
    M, K = A.shape
    q = np.empty((M, K), np.int8)
    scale = _c(scale, np.float32)
    if A.dtype == np.uint16:
        lib().orc_w8_quant_f16(M, K, _p(A), _p(scale), _p(q))
    else:
        lib().orc_w8_quant_f32(M, K, _p(_c(A, np.float32)), _p(scale), _p(q))
    return q


def w4a8_scales(A):
    """Returns (rc, scale, inverse)."""
    M, K = A.shape
    s = np.empty(M, np.float32)
    inv = np.empty(M, np.float32)
    if A.dtype == np.uint16:
        rc = lib().orc_w4a8_scales_f16(M, K, _p(A), _p(s), _p(inv))
    else:
        rc = lib().orc_w4a8_scales_f32(M, K, _p(_c(A, np.float32)), _p(s), _p(inv))
    return rc, s, inv


def w4a8_quant(A, inverse):
    M, K = A.shape
    q = np.empty((M, K), np.int8)
    inverse = _c(inverse, np.float32)
    if A.dtype == np.uint16:
        lib().orc_w4a8_quant_f16(M, K, _p(A), _p(inverse), _p(q))
    else:
        lib().orc_w4a8_quant_f32(M, K, _p(_c(A, np.float32)), _p(inverse), _p(q))
    return q


def msd_split(q):
    h, l = C.c_int(0), C.c_int(0)
    lib().orc_w4a8_msd_split(C.c_int8(int(q)), C.byref(h), C.byref(l))
    return h.value, l.value


def moe_quant_row(x, validate=True):
    x = _c(x, np.float32)
    q = np.empty(x.shape, np.int8)
    s = lib().orc_moe_quant_row(_p(x), x.size, 1 if validate else 0, _p(q))
    return float(np.float32(s)), q


def gemm_i8(A, B):
    A = _c(A, np.int8)
    B = _c(B, np.int8)
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    Cm = np.empty((M, N), np.int32)
    lib().orc_gemm_i8(M, N, K, _p(A), _p(B), _p(Cm))
    return Cm


def dequant(acc, a_scale, w_scale, half=False):
    acc = _c(acc, np.int32)
    M, N = acc.shape
    a_scale, w_scale = _c(a_scale, np.float32), _c(w_scale, np.float32)
    if half:
        out = np.empty((M, N), np.uint16)
        lib().orc_dequant_f16(M, N, _p(acc), _p(a_scale), _p(w_scale), _p(out))
    else:
        out = np.empty((M, N), np.float32)
        lib().orc_dequant_f32(M, N, _p(acc), _p(a_scale), _p(w_scale), _p(out))
    return out


def silu_mul(g, u, flavour=EXP_POLY):
    return float(np.float32(lib().orc_silu_mul(C.c_float(g), C.c_float(u), flavour)))


def swiglu(acc, a_scale, w_scale, flavour=EXP_POLY):
    acc = _c(acc, np.int32)
    M, N = acc.shape
    F = N // 2
    mid = np.empty((M, F), np.float32)
    bits = np.empty(M, np.uint32)
    lib().orc_swiglu(M, F, _p(acc), _p(_c(a_scale, np.float32)), _p(_c(w_scale, np.float32)),
                     flavour, _p(mid), _p(bits))
    return mid, bits


def finish_scales(bits):
    bits = _c(bits, np.uint32)
    s = np.empty(bits.size, np.float32)
    inv = np.empty(bits.size, np.float32)
    rc = lib().orc_finish_scales(bits.size, _p(bits), _p(s), _p(inv))
    return rc, s, inv


def w8a8(A, B, w_scale, a_scale_static=None, want_acc=True):
    """A fp16 bits (uint16) or float32 [M,K]; B int8 [K,N].
    Returns dict(C, q, a_scale, acc)."""
    M, K = A.shape
    N = B.shape[1]
    B = _c(B, np.int8)
    w_scale = _c(w_scale, np.float32)
    q = np.empty((M, K), np.int8)
    s = np.empty(M, np.float32)
    acc = np.empty((M, N), np.int32)
    st = _c(a_scale_static, np.float32) if a_scale_static is not None else None
    if A.dtype == np.uint16:
        out = np.empty((M, N), np.uint16)
        lib().orc_w8a8_f16(M, N, K, _p(A), _p(B), _p(w_scale), _p(st), _p(out), _p(q), _p(s), _p(acc))
    else:
        A = _c(A, np.float32)
        out = np.empty((M, N), np.float32)
        lib().orc_w8a8_f32(M, N, K, _p(A), _p(B), _p(w_scale), _p(st), _p(out), _p(q), _p(s), _p(acc))
    return dict(C=out, q=q, a_scale=s, acc=acc)


def w4a8(A, B, w_scale):
    M, K = A.shape
    N = B.shape[1]
    B = _c(B, np.int8)
    w_scale = _c(w_scale, np.float32)
    q = np.empty((M, K), np.int8)
    s = np.empty(M, np.float32)
    acc = np.empty((M, N), np.int32)
    if A.dtype == np.uint16:
        out = np.empty((M, N), np.uint16)
        rc = lib().orc_w4a8_f16(M, N, K, _p(A), _p(B), _p(w_scale), _p(out), _p(q), _p(s), _p(acc))
    else:
        A = _c(A, np.float32)
        out = np.empty((M, N), np.float32)
        rc = lib().orc_w4a8_f32(M, N, K, _p(A), _p(B), _p(w_scale), _p(out), _p(q), _p(s), _p(acc))
    return dict(rc=rc, C=out, q=q, a_scale=s, acc=acc)


def w4a8_swiglu(A, B, w_scale, flavour=EXP_POLY):
    A = _c(A, np.float32)
    M, K = A.shape
    N = B.shape[1]
    mid = np.empty((M, N // 2), np.float32)
    bits = np.empty(M, np.uint32)
    acc = np.empty((M, N), np.int32)
    rc = lib().orc_w4a8_swiglu_f32(M, N, K, _p(A), _p(_c(B, np.int8)), _p(_c(w_scale, np.float32)),
                                   flavour, _p(mid), _p(bits), _p(acc))
    return dict(rc=rc, middle=mid, bits=bits, acc=acc)


def w4a8_ffn(A, B_gu, s_gu, B_down, s_down, flavour=EXP_POLY):
    A = _c(A, np.float32)
    M, H = A.shape
    I = B_gu.shape[1] // 2
    Nout = B_down.shape[1]
    mid = np.empty((M, I), np.float32)
    out = np.empty((M, Nout), np.float32)
    qd = np.empty((M, I), np.int8)
    sd = np.empty(M, np.float32)
    acc = np.empty((M, Nout), np.int32)
    rc = lib().orc_w4a8_ffn_f32(M, H, I, Nout, _p(A), _p(_c(B_gu, np.int8)), _p(_c(s_gu, np.float32)),
                                _p(_c(B_down, np.int8)), _p(_c(s_down, np.float32)), flavour,
                                _p(mid), _p(out), _p(qd), _p(sd), _p(acc))
    return dict(rc=rc, middle=mid, C=out, q_down=qd, down_scale=sd, acc_down=acc)


def moe_w8(experts, H, I, E, shared, top_k, ids, routes, input_f32=None, input_q=None,
           row_scales=None, flavour=EXP_POLY, fused_combine=True):
    """experts: list of (gate_up[H,2I] int8, gate_up_scales[2I], down[I,H] int8, down_scales[H])."""
    keep = []
    arr = (MoeExpert * len(experts))()
    for i, (g, gs, d, ds) in enumerate(experts):
        g, gs, d, ds = _c(g, np.int8), _c(gs, np.float32), _c(d, np.int8), _c(ds, np.float32)
        keep += [g, gs, d, ds]
        arr[i] = MoeExpert(g.ctypes.data, gs.ctypes.data, d.ctypes.data, ds.ctypes.data)
    ids = _c(ids, np.int32)
    routes = _c(routes, np.float32)
    rows = ids.shape[0]
    out = np.zeros((rows, H), np.float32)
    xin = _c(input_f32, np.float32) if input_f32 is not None else None
    xq = _c(input_q, np.int8) if input_q is not None else None
    rs = _c(row_scales, np.float32) if row_scales is not None else None
    rc = lib().orc_moe_w8(rows, H, I, E, shared, top_k, arr, _p(xin), _p(xq), _p(rs), _p(ids),
                          _p(routes), flavour, 1 if fused_combine else 0, _p(out))
    return rc, out
