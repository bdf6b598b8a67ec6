"""Thin numpy-facing wrappers over the rk_npu_* C API.

Each class owns the C handles of one operator instance (context/domain are
shared through Session) and forwards to the C entry points unchanged; return
codes are surfaced, not hidden.  Used by the tests, the smoke check and the
benchmark so that all three exercise the same C ABI a C++ caller would.
"""
import ctypes as C

import numpy as np

from . import capi
from .capi import ptr


class RkError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        lib = capi.load_library()
        super().__init__("%s: %s (%d)" % (what, lib.rk_npu_strerror(code).decode(), code))


def check(code, what):
    if code != capi.RK_NPU_OK:
        raise RkError(code, what)


class Session:
    """One device context plus one domain tag."""

    def __init__(self, dev=None, domain_id=0):
        self.lib = capi.load_library()
        self.ctx = self.lib.rk_npu_open(dev.encode() if dev else None)
        if not self.ctx:
            raise RuntimeError("rk_npu_open failed: no usable HIP device")
        self.domain = self.lib.rk_npu_iommu_domain_create(self.ctx, domain_id)
        if not self.domain:
            raise RuntimeError("rk_npu_iommu_domain_create failed")

    def close(self):
        if self.domain:
            self.lib.rk_npu_iommu_domain_free(self.domain)
            self.domain = None
        if self.ctx:
            self.lib.rk_npu_close(self.ctx)
            self.ctx = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # -- device helpers (MI355X extension) --
    def device_info(self):
        arch = C.create_string_buffer(64)
        cu, khz = C.c_int(0), C.c_int(0)
        check(self.lib.rk_npu_hip_device_info(self.ctx, arch, 64, C.byref(cu), C.byref(khz)), "device_info")
        return arch.value.decode(), cu.value, khz.value

    def to_device(self, array):
        array = np.ascontiguousarray(array)
        d = self.lib.rk_npu_hip_malloc(self.ctx, max(array.nbytes, 16))
        if not d:
            raise MemoryError("rk_npu_hip_malloc")
        check(self.lib.rk_npu_hip_upload(self.ctx, d, ptr(array), array.nbytes), "upload")
        return d

    def empty_device(self, nbytes):
        d = self.lib.rk_npu_hip_malloc(self.ctx, max(nbytes, 16))
        if not d:
            raise MemoryError("rk_npu_hip_malloc")
        return d

    def from_device(self, d, shape, dtype):
        out = np.empty(shape, dtype)
        check(self.lib.rk_npu_hip_download(self.ctx, ptr(out), d, out.nbytes), "download")
        return out

    def free_device(self, d):
        self.lib.rk_npu_hip_free(self.ctx, d)

    def sync(self):
        return self.lib.rk_npu_hip_sync(self.ctx)

    def spin_up(self, fn, seconds=0.05):
        """Keep the device busy with fn() for `seconds` of wall time (untimed):
        after an idle period the first milliseconds of work run at reduced clocks."""
        import time
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(20):
                fn()
            check(self.sync(), "sync")

    def time_us(self, fn, iters, warmup):
        """Average device time of fn() over `iters` calls, HIP events on the
        context's stream (the stream the kernels are launched on)."""
        for _ in range(warmup):
            fn()
        check(self.sync(), "sync")
        e0, e1 = self.lib.rk_npu_hip_event_create(), self.lib.rk_npu_hip_event_create()
        self.lib.rk_npu_hip_event_record(self.ctx, e0)
        for _ in range(iters):
            fn()
        self.lib.rk_npu_hip_event_record(self.ctx, e1)
        us = C.c_double(0)
        check(self.lib.rk_npu_hip_event_elapsed_us(e0, e1, C.byref(us)), "elapsed")
        check(self.sync(), "sync")
        self.lib.rk_npu_hip_event_free(e0)
        self.lib.rk_npu_hip_event_free(e1)
        return us.value / iters


def profile_kernels(sess, fn, iters, warmup=3):
    """Average time per kernel of one fn() call, from stream events between the kernels:
    a list of (kernel name, microseconds) in launch order (kernel plus the launch gap behind it)."""
    for _ in range(warmup):
        fn()
    check(sess.sync(), "sync")
    lib = sess.lib
    check(lib.rk_npu_hip_profile_begin(sess.ctx), "profile_begin")
    for _ in range(iters):
        fn()
    cap = 64 * iters
    us = (C.c_double * cap)()
    names = C.create_string_buffer(64 * cap)
    n = lib.rk_npu_hip_profile_end(sess.ctx, names, len(names), us, cap)
    if n < 0:
        raise RkError(n, "profile_end")
    labels = names.value.decode().split("\n")[:-1]
    per = n // iters
    if per * iters != n or len(labels) != n:
        raise RuntimeError("profile: %d kernels over %d calls" % (n, iters))
    out = []
    for k in range(per):
        out.append((labels[k], sum(us[i * per + k] for i in range(iters)) / iters))
    return out


def default_strategy(kind, M, N, K, k_tile=None, n_tile=None):
    """A strategy any caller of the reference would pass: full-K tile up to
    2048, n_tile <= 3072, one core, one CPU."""
    s = capi.MatmulStrategy()
    s.op_kind = kind
    s.M, s.N, s.K = M, N, K
    s.k_tile = k_tile if k_tile else min(K, 2048)
    s.n_tile = n_tile if n_tile else min(max(N, 32), 3072)
    s.a_layout = 0
    s.wave_count = (K + s.k_tile - 1) // s.k_tile
    s.n_groups = 1
    s.npu_core_mask = 1
    import os
    cpus = sorted(os.sched_getaffinity(0))
    s.cpu_core_mask = 1 << min(c for c in cpus if c < 64)
    s.cpu_threads = 1
    s.c_layout = 0
    return s


class W8A8Linear:
    """rk_npu_{i8i8i32,f16i8f16,f32i8f32}: weights + one workspace of fixed M."""

    _CREATE = {capi.I8I8I32: "rk_npu_i8i8i32", capi.F16I8F16_DYNAMIC: "rk_npu_f16i8f16",
               capi.F16I8F16_STATIC: "rk_npu_f16i8f16", capi.F32I8F32_DYNAMIC: "rk_npu_f32i8f32",
               capi.F32I8F32_STATIC: "rk_npu_f32i8f32"}

    def __init__(self, sess, kind, M, B, w_scale=None, k_tile=None, strategy=None):
        self.s, self.kind, self.M = sess, kind, M
        self.K, self.N = B.shape
        lib = sess.lib
        self.prefix = self._CREATE[kind]
        # `strategy`: a rk_npu_matmul_strategy value, e.g. one returned by the tuning calls
        self.strategy = strategy if strategy is not None else default_strategy(kind, M, self.N, self.K, k_tile)
        wc = capi.MatmulWeightConfig(self.K, self.N, self.strategy.k_tile)
        B = np.ascontiguousarray(B, np.int8)
        create = getattr(lib, self.prefix + "_weights_create")
        if kind == capi.I8I8I32:
            self.w = create(sess.domain, C.byref(wc), ptr(B))
        else:
            ws = np.ascontiguousarray(w_scale, np.float32)
            self.w = create(sess.domain, C.byref(wc), ptr(B), ptr(ws))
        if not self.w:
            raise RuntimeError("weights_create failed")
        self.ws = lib.rk_npu_matmul_workspace_create(sess.domain, C.byref(self.strategy))
        if not self.ws:
            raise RuntimeError("workspace_create failed")

    def out_dtype(self):
        return {capi.I8I8I32: np.int32, capi.F16I8F16_DYNAMIC: np.uint16,
                capi.F16I8F16_STATIC: np.uint16}.get(self.kind, np.float32)

    def run(self, A, a_scale=None):
        lib = self.s.lib
        A = np.ascontiguousarray(A)
        out = np.empty((self.M, self.N), self.out_dtype())
        if self.kind == capi.I8I8I32:
            rc = lib.rk_npu_i8i8i32_run(self.ws, self.w, ptr(A), ptr(out))
        elif self.kind == capi.F16I8F16_DYNAMIC:
            rc = lib.rk_npu_f16i8f16_run_dynamic(self.ws, self.w, ptr(A), ptr(out))
        elif self.kind == capi.F16I8F16_STATIC:
            sc = np.ascontiguousarray(a_scale, np.float32)
            rc = lib.rk_npu_f16i8f16_run_static(self.ws, self.w, ptr(A), ptr(sc), ptr(out))
        elif self.kind == capi.F32I8F32_DYNAMIC:
            rc = lib.rk_npu_f32i8f32_run_dynamic(self.ws, self.w, ptr(A), ptr(out))
        else:
            sc = np.ascontiguousarray(a_scale, np.float32)
            rc = lib.rk_npu_f32i8f32_run_static(self.ws, self.w, ptr(A), ptr(sc), ptr(out))
        return rc, out

    def run_device(self, dA, dC):
        lib = self.s.lib
        fn = {capi.I8I8I32: lib.rk_npu_i8i8i32_run_device,
              capi.F16I8F16_DYNAMIC: lib.rk_npu_f16i8f16_run_dynamic_device,
              capi.F32I8F32_DYNAMIC: lib.rk_npu_f32i8f32_run_dynamic_device}[self.kind]
        return fn(self.ws, self.w, dA, dC)

    def read_quantized(self):
        q = np.empty((self.M, self.K), np.int8)
        s = np.empty(self.M, np.float32)
        check(self.s.lib.rk_npu_matmul_workspace_read_quantized(self.ws, ptr(q), ptr(s)), "read_quantized")
        return q, s

    def close(self):
        lib = self.s.lib
        if self.ws:
            lib.rk_npu_matmul_workspace_free(self.ws)
            self.ws = None
        if self.w:
            getattr(lib, self.prefix + "_weights_free")(self.w)
            self.w = None


class W4A8Weights:
    def __init__(self, sess, B, w_scale, k_tile=480):
        self.s = sess
        self.K, self.N = B.shape
        cfg = capi.I4WeightConfig(self.K, self.N, k_tile)
        B = np.ascontiguousarray(B, np.int8)
        ws = np.ascontiguousarray(w_scale, np.float32)
        self.h = sess.lib.rk_npu_w4a8_weights_create(sess.domain, C.byref(cfg), ptr(B), ptr(ws))
        if not self.h:
            raise RuntimeError("rk_npu_w4a8_weights_create failed")
        info = capi.W4A8WeightInfo()
        check(sess.lib.rk_npu_w4a8_weights_query(self.h, C.byref(info)), "weights_query")
        self.info = info
        self.k_tile = info.config.k_tile

    def close(self):
        if self.h:
            self.s.lib.rk_npu_w4a8_weights_free(self.h)
            self.h = None


class W4A8Workspace:
    def __init__(self, sess, M, N, K, k_tile=480, options=None):
        self.s, self.M, self.N, self.K = sess, M, N, K
        cfg = capi.W4A8Config()
        sess.lib.rk_npu_w4a8_config_init(C.byref(cfg), M, N, K)
        cfg.k_tile = k_tile
        self.cfg = cfg
        if options is None:
            self.h = sess.lib.rk_npu_w4a8_workspace_create(sess.domain, C.byref(cfg))
        else:
            self.h = sess.lib.rk_npu_w4a8_workspace_create_ex(sess.domain, C.byref(cfg), C.byref(options))
        if not self.h:
            raise RuntimeError("rk_npu_w4a8_workspace_create failed")

    def run_f32(self, w, A, timings=None):
        A = np.ascontiguousarray(A, np.float32)
        out = np.empty((self.M, self.N), np.float32)
        t = C.byref(timings) if timings is not None else None
        return self.s.lib.rk_npu_w4a8_run_f32(self.h, w.h, ptr(A), ptr(out), t), out

    def run_f16(self, w, A, timings=None):
        A = np.ascontiguousarray(A, np.uint16)
        out = np.empty((self.M, self.N), np.uint16)
        t = C.byref(timings) if timings is not None else None
        return self.s.lib.rk_npu_w4a8_run_f16(self.h, w.h, ptr(A), ptr(out), t), out

    def run_swiglu_f32(self, w, A, timings=None):
        A = np.ascontiguousarray(A, np.float32)
        out = np.empty((self.M, self.N // 2), np.float32)
        t = C.byref(timings) if timings is not None else None
        return self.s.lib.rk_npu_w4a8_run_swiglu_f32(self.h, w.h, ptr(A), ptr(out), t), out

    def run_i32(self, w, A):
        A = np.ascontiguousarray(A, np.float32)
        out = np.empty((self.M, self.N), np.int32)
        return self.s.lib.rk_npu_w4a8_run_i32(self.h, w.h, ptr(A), ptr(out)), out

    def read_quantized(self):
        q = np.empty((self.M, self.K), np.int8)
        s = np.empty(self.M, np.float32)
        check(self.s.lib.rk_npu_w4a8_workspace_read_quantized(self.h, ptr(q), ptr(s)), "read_quantized")
        return q, s

    def close(self):
        if self.h:
            self.s.lib.rk_npu_w4a8_workspace_free(self.h)
            self.h = None


def w4a8_ffn(sess, gu_ws, gu_w, dn_ws, dn_w, A, timings=None):
    A = np.ascontiguousarray(A, np.float32)
    middle = np.empty((gu_ws.M, gu_ws.N // 2), np.float32)
    out = np.empty((dn_ws.M, dn_ws.N), np.float32)
    t = C.byref(timings) if timings is not None else None
    rc = sess.lib.rk_npu_w4a8_run_ffn_f32(gu_ws.h, gu_w.h, dn_ws.h, dn_w.h, ptr(A), ptr(middle),
                                          ptr(out), t)
    return rc, middle, out


class MoeW8:
    """flavour: "w8" (int8 experts), "quant" (every expert INT4 codes) or "w4" (routed INT4, shared int8)."""
    _CREATE = {"w8": ("rk_npu_moe_w8_weights_create", "rk_npu_moe_w8_workspace_create"),
               "quant": ("rk_npu_moe_quant_weights_create", "rk_npu_moe_quant_workspace_create"),
               "w4": ("rk_npu_moe_w4_weights_create", "rk_npu_moe_w4_workspace_create")}

    def __init__(self, sess, H, I, E, shared, top_k, max_rows, experts, flavour="w8"):
        self.s, self.H, self.I, self.E, self.shared, self.top_k = sess, H, I, E, shared, top_k
        self.flavour = flavour
        lib = sess.lib
        cfg = capi.MoeConfig()
        lib.rk_npu_moe_w8_config_init(C.byref(cfg), H, I, E, shared, top_k, max_rows)
        self.cfg = cfg
        self.w = self.create_weights(experts) if experts is not None else None
        self.ws = getattr(lib, self._CREATE[flavour][1])(sess.domain, C.byref(cfg))
        if not self.ws:
            raise RuntimeError("%s failed" % self._CREATE[flavour][1])

    def create_weights(self, experts, domain=None):
        keep = []
        arr = (capi.MoeExpert * len(experts))()
        for i, (g, gs, d, ds) in enumerate(experts):
            g = np.ascontiguousarray(g, np.int8)
            gs = np.ascontiguousarray(gs, np.float32)
            d = np.ascontiguousarray(d, np.int8)
            ds = np.ascontiguousarray(ds, np.float32)
            keep += [g, gs, d, ds]
            arr[i] = capi.MoeExpert(g.ctypes.data, gs.ctypes.data, d.ctypes.data, ds.ctypes.data)
        name = self._CREATE[self.flavour][0]
        h = getattr(self.s.lib, name)(domain or self.s.domain, C.byref(self.cfg.weights), arr)
        if not h:
            raise RuntimeError("%s failed" % name)
        return h

    def run_f32(self, x, ids, routes, weights=None, timings=None, out=None):
        x = np.ascontiguousarray(x, np.float32)
        ids = np.ascontiguousarray(ids, np.int32)
        routes = np.ascontiguousarray(routes, np.float32)
        rows = x.shape[0]
        if out is None:
            out = np.empty((rows, self.H), np.float32)
        t = C.byref(timings) if timings is not None else None
        rc = self.s.lib.rk_npu_moe_w8_run_f32(self.ws, weights or self.w, rows, ptr(x), ptr(ids),
                                              ptr(routes), ptr(out), t)
        return rc, out

    def run_quantized(self, xq, scales, ids, routes, weights=None, timings=None, out=None):
        xq = np.ascontiguousarray(xq, np.int8)
        scales = np.ascontiguousarray(scales, np.float32)
        ids = np.ascontiguousarray(ids, np.int32)
        routes = np.ascontiguousarray(routes, np.float32)
        rows = xq.shape[0]
        if out is None:
            out = np.empty((rows, self.H), np.float32)
        t = C.byref(timings) if timings is not None else None
        rc = self.s.lib.rk_npu_moe_w8_run_quantized(self.ws, weights or self.w, rows, ptr(xq),
                                                    ptr(scales), ptr(ids), ptr(routes), ptr(out), t)
        return rc, out

    def close(self):
        lib = self.s.lib
        if self.ws:
            lib.rk_npu_moe_w8_workspace_free(self.ws)
            self.ws = None
        if self.w:
            lib.rk_npu_moe_w8_weights_free(self.w)
            self.w = None
