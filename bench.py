#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the hot path over one batch of seeded synthetic input,
with inputs and weights already resident in HBM: per-token quantization +
GEMV / GEMM with the fused dequant epilogue (+ SwiGLU / re-quantize / Down for
the FFN, + route / combine for the MoE layer), enqueued through the
device-pointer entry points of the C ABI and timed with HIP events on the
context's stream (the stream the kernels are launched on).

The headline workload is BASELINE config 1 (w8a8 decode GEMV, M=1, K=4096,
N=14336), reported as weight GB/s.  The same line carries, under "also", every
other BASELINE configuration (0, 2, 3, 4) and the int4 decode GEMV, each with
its own roofline block (bound, dominant kernel, algorithmic bytes / operations,
fraction of the datasheet peak), a per-kernel breakdown from stream events, and
under "practical" what a read-only stream and a pure-MFMA loop reach on the box
at hand -- the ceilings the fractions should be read against.

Prints ONE JSON line.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X published HBM3E bandwidth
INT8_PEAK_TOPS = 5000.0      # MI355X published dense int8 MFMA rate
C1_COPIES = 8                # copies of the decode matrix the timed loop cycles through (8 x 58.7 MB)
FFN_COPIES = 4               # copies of the FFN weights (4 x 88 MB)
MOE_COPIES = 2               # copies of the expert bank (2 x 201 MB)
METRIC = "int8 TOPS @M=2048 and GEMV HBM GB/s @M=1 (w8a8/w4a8), % of roofline"


def log(msg):
    sys.stderr.write("[bench] %s\n" % msg)
    sys.stderr.flush()


def _traffic(kernel_key):
    """HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE + WRITE_SIZE,
    scaled by a copy kernel of known size), if a summary has been committed."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(kernel_key)
    except (OSError, ValueError):
        return None


def _hbm(kernel, algo_bytes, us, traffic_key=None, **extra):
    r = {"bound": "hbm", "kernel": kernel, "achieved": algo_bytes / us / 1e3, "peak": HBM_PEAK_GBS,
         "unit": "GB/s", "frac": algo_bytes / us / 1e3 / HBM_PEAK_GBS, "time_us": us,
         "algorithmic_bytes": algo_bytes, "traffic": _traffic(traffic_key) if traffic_key else None}
    r.update(extra)
    return r


def _mfma(kernel, ops_count, us, traffic_key=None, **extra):
    r = {"bound": "mfma", "kernel": kernel, "achieved": ops_count / us / 1e6, "peak": INT8_PEAK_TOPS,
         "unit": "TOP/s", "frac": ops_count / us / 1e6 / INT8_PEAK_TOPS, "time_us": us,
         "algorithmic_ops": ops_count, "traffic": _traffic(traffic_key) if traffic_key else None}
    r.update(extra)
    return r


def _kernels(sess, ops, step, calls=20):
    """Per-kernel times of one step from stream events between the kernels."""
    return [{"kernel": k, "us": round(us, 3)} for k, us in ops.profile_kernels(sess, step, calls)]


def bench_c1(sess, ops, capi, workloads, steps, warmup, cpu_baseline):
    """w8a8 decode GEMV, M=1, K=4096, N=14336."""
    c = workloads.CONFIGS[1]()
    M, K, N = c["M"], c["K"], c["N"]
    # A decode step streams weights that were not touched since the previous
    # token (a whole model lies between two uses of a layer).  Re-running ONE
    # matrix would instead find part of it in the 256 MB memory-side cache, so
    # the timed loop walks over C1_COPIES identical copies (470 MB): every launch
    # reads its weights from HBM.  The single-copy time is reported beside it.
    copies = [ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, M, c["B"], c["w_scale"]) for _ in range(C1_COPIES)]
    op = copies[0]
    dA = sess.to_device(c["A"])
    dC = sess.empty_device(M * N * 2)
    lib = sess.lib
    turn = [0]

    def step():
        o = copies[turn[0] % C1_COPIES]
        turn[0] += 1
        rc = o.run_device(dA, dC)
        if rc:
            raise RuntimeError("run_device rc=%d" % rc)

    def step_same_matrix():
        rc = op.run_device(dA, dC)
        if rc:
            raise RuntimeError("run_device rc=%d" % rc)

    def gemv_only():
        o = copies[turn[0] % C1_COPIES]
        turn[0] += 1
        rc = lib.rk_npu_matmul_workspace_rerun_gemm_device(o.ws, o.w, dC)
        if rc:
            raise RuntimeError("rerun rc=%d" % rc)

    # For decode-sized M the step is ONE kernel: the GEMV with the per-token
    # quantization fused into its prologue.  The plain GEMV (activations already
    # quantized) is timed as well for reference.
    sess.spin_up(step)
    step_us = sess.time_us(step, steps, warmup)
    for o in copies:  # every copy's workspace holds quantized activations for the plain GEMV
        o.run_device(dA, dC)
    gemv_only_us = sess.time_us(gemv_only, max(steps, 50), warmup)
    same_matrix_us = sess.time_us(step_same_matrix, steps, warmup)
    # the same eight launches recorded once and replayed as a graph: what the step costs when
    # the host's per-launch submission is out of the picture
    graph_us = graph_step_us(sess, step, C1_COPIES, max(steps // C1_COPIES, 5))
    step_same_matrix()
    got = sess.from_device(dC, (M, N), np.uint16)
    weight_bytes = K * N
    # algorithmic bytes of one launch: weights once + fp16 A + fp16 C + weight scales
    algo_bytes = weight_bytes + K * 2 + N * 2 + N * 4
    out = {
        "value": weight_bytes / step_us / 1e3,  # GB/s (bytes / us / 1e3)
        "unit": "GB/s",
        "ms_per_step": step_us / 1e3,
        "dtype": "int8",
        "config": {"workload": "c1: w8a8 decode GEMV M=1 K=4096 N=14336, fp16 in/out, seeds 2/3",
                   "value_is": "int8 weight bytes (58720256) / step time; step = one fused quantize+GEMV kernel; "
                               "the loop cycles through %d copies of the matrix so that every step reads HBM" % C1_COPIES},
        "roofline": _hbm("gemv_kernel<1,false,1,32,burst> (fused per-token quantize + GEMV)", algo_bytes, step_us, "gemv_c1",
                         kernel_us=step_us, gemv_without_quantize_us=gemv_only_us,
                         same_matrix_every_step_us=same_matrix_us, replayed_from_graph_us=graph_us),
    }
    if cpu_baseline:
        from oracle import binding as orc
        want = orc.w8a8(c["A"], c["B"], c["w_scale"])
        out["parity"] = bool(np.array_equal(got, want["C"]))
        out["host_api_us"] = _host_call_us(lambda: op.run(c["A"]))
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < 10.0:
            orc.w8a8(c["A"], c["B"], c["w_scale"])
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        out["cpu_baseline"] = {"value": weight_bytes / dt / 1e9, "unit": "GB/s",
                               "cores": orc.num_threads(), "kind": "port",
                               "sample": "%d full passes of config 1 (quantize + exact int GEMV + dequant), %.1f ms each"
                                         % (reps, dt * 1e3)}
    sess.free_device(dA)
    sess.free_device(dC)
    for o in copies:
        o.close()
    return out


def graph_step_us(sess, step, steps_in_graph, replays):
    """Average time of one step when `steps_in_graph` of them are captured once and replayed."""
    lib = sess.lib
    for _ in range(steps_in_graph):
        step()
    if sess.sync():
        raise RuntimeError("sync")
    if lib.rk_npu_hip_capture_begin(sess.ctx):
        raise RuntimeError("capture_begin")
    for _ in range(steps_in_graph):
        step()
    g = lib.rk_npu_hip_capture_end(sess.ctx)
    if not g:
        raise RuntimeError("capture_end")
    us = sess.time_us(lambda: lib.rk_npu_hip_graph_launch(sess.ctx, g), replays, 3) / steps_in_graph
    lib.rk_npu_hip_graph_free(g)
    return us


def _oracle():
    from oracle import binding as orc
    return orc


def _host_call_us(call, reps=10, warmups=2):
    """Median wall time of a blocking host-pointer call, the reference's own protocol
    (examples/bench_llm_i8.cpp:43-47: 2 warm-ups, median of 10)."""
    for _ in range(warmups):
        call()
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        call()
        times.append((time.perf_counter() - t0) * 1e6)
    return float(np.median(times))


def bench_c2(sess, ops, capi, workloads, steps, warmup, want_mfma_probe=True, check=False):
    """w4a8 prefill GEMM, M=2048, K=4096, N=4096."""
    c = workloads.CONFIGS[2]()
    M, K, N = c["M"], c["K"], c["N"]
    w = ops.W4A8Weights(sess, c["B"], c["w_scale"])
    ws = ops.W4A8Workspace(sess, M, N, K)
    dA = sess.to_device(c["A"])
    dC = sess.empty_device(M * N * 2)
    lib = sess.lib

    def step():
        rc = lib.rk_npu_w4a8_run_f16_device(ws.h, w.h, dA, dC)
        if rc:
            raise RuntimeError("run_device rc=%d" % rc)

    def gemm_only():
        rc = lib.rk_npu_w4a8_workspace_rerun_gemm_device(ws.h, w.h, dC, 1)
        if rc:
            raise RuntimeError("rerun rc=%d" % rc)

    sess.spin_up(step)
    step_us = sess.time_us(step, steps, warmup)
    kernel_us = sess.time_us(gemm_only, steps, warmup)
    ops_count = 2.0 * M * K * N
    out = {"workload": "c2: w4a8 prefill GEMM M=2048 K=4096 N=4096, fp16 in/out, seeds 4/5",
           "tops": ops_count / step_us / 1e6, "ms_per_step": step_us / 1e3,
           "step_frac_of_int8_peak": ops_count / step_us / 1e6 / INT8_PEAK_TOPS,
           "roofline": _mfma("gemm_wk_kernel<int4,f16> (128x256 tile, waves split K)", ops_count, kernel_us,
                             "gemm_c2", kernel_us=kernel_us),
           "kernels": _kernels(sess, ops, step)}
    if check:
        # the timed call (quantize + GEMM through the device-pointer entry) and the GEMM-only call
        # against the CPU oracle: all 2048 x 4096 fp16 outputs
        want = _oracle().w4a8(c["A"], c["B"], c["w_scale"])["C"]
        step()
        ok = np.array_equal(sess.from_device(dC, (M, N), np.uint16), want)
        lib.rk_npu_hip_upload(sess.ctx, dC, capi.ptr(np.zeros((M, N), np.uint16)), M * N * 2)
        gemm_only()
        out["parity_vs_oracle"] = bool(ok and np.array_equal(sess.from_device(dC, (M, N), np.uint16), want))
        out["host_api_us"] = _host_call_us(lambda: ws.run_f16(w, c["A"]))
    if want_mfma_probe:
        # the pure-MFMA loop on operands with this workload's bit patterns: int4 codes carried as
        # 16 * code (weights, first operand) and the int8 codes of the quantized rows (second)
        q, _ = ws.read_quantized()
        wbytes = (c["B"].T.reshape(-1)[:16384].astype(np.int16) * 16).astype(np.int8)
        abytes = q.reshape(-1)[:16384]
        operands = np.concatenate([wbytes[:8192], abytes[:8192], wbytes[8192:], abytes[8192:]])
        out["roofline"]["practical_peak"] = mfma_probe(sess, operands)
        out["roofline"]["frac_of_practical_peak"] = out["roofline"]["achieved"] / out["roofline"]["practical_peak"]
    sess.free_device(dA)
    sess.free_device(dC)
    ws.close()
    w.close()
    return out


def mfma_probe(sess, operands_i8, iterations=2000):
    """TOP/s of the library's pure int8 MFMA loop on the given 32 KiB of operands."""
    lib = sess.lib
    d = sess.to_device(np.ascontiguousarray(operands_i8, np.int8))
    count = C.c_double(0)

    def run():
        if lib.rk_npu_hip_probe_mfma_i8(sess.ctx, d, iterations, C.byref(count)):
            raise RuntimeError("probe_mfma")

    sess.spin_up(run, 0.02)
    us = sess.time_us(run, 20, 3)
    sess.free_device(d)
    return count.value / us / 1e6


def read_probe(sess, bytes_per_launch, span, footprint=C1_COPIES * 58720256, iters=200):
    """GB/s of the library's read-only stream, `bytes_per_launch` per launch, rotating over
    `footprint` bytes so that no launch finds its data in the memory-side cache."""
    lib = sess.lib
    pieces = max(footprint // bytes_per_launch, 1)
    buf = sess.empty_device(pieces * bytes_per_launch)
    base = buf if isinstance(buf, int) else buf.value
    turn = [0]

    def run():
        at = base + (turn[0] % pieces) * bytes_per_launch
        turn[0] += 1
        if lib.rk_npu_hip_probe_stream_read(sess.ctx, C.c_void_p(at), bytes_per_launch, span):
            raise RuntimeError("probe_stream_read")

    us = sess.time_us(run, iters, 20)
    sess.free_device(buf)
    return {"GBps": bytes_per_launch / us / 1e3, "us_per_launch": us, "bytes_per_launch": bytes_per_launch}


def bench_c1w4(sess, ops, capi, workloads, steps, warmup):
    """w4a8 decode GEMV at config 1's shape (M=1, K=4096, N=14336), int4 weights."""
    M, K, N = 1, 4096, 14336
    c = workloads.w4a8_case(M, K, N, seed_w=2, seed_a=3)
    # as in bench_c1: the loop walks over several copies so that every step streams from HBM
    # (16 copies of 29.4 MB = 470 MB)
    copies = [ops.W4A8Weights(sess, c["B"], c["w_scale"]) for _ in range(2 * C1_COPIES)]
    ws = ops.W4A8Workspace(sess, M, N, K)
    dA = sess.to_device(c["A"])
    dC = sess.empty_device(M * N * 2)
    lib = sess.lib
    turn = [0]

    def step():
        w = copies[turn[0] % len(copies)]
        turn[0] += 1
        rc = lib.rk_npu_w4a8_run_f16_device(ws.h, w.h, dA, dC)
        if rc:
            raise RuntimeError("run_device rc=%d" % rc)

    sess.spin_up(step)
    step_us = sess.time_us(step, steps, warmup)
    weight_bytes = K * N // 2
    algo_bytes = weight_bytes + K * 2 + N * 2 + N * 4
    out = {"workload": "w4a8 decode GEMV M=1 K=4096 N=14336 (int4 weights, 29360128 B), fp16 in/out, seeds 2/3",
           "weight_GBps": weight_bytes / step_us / 1e3, "ms_per_step": step_us / 1e3,
           "roofline": _hbm("gemv_kernel<1,true,1,32> (fused per-token quantize + int4 GEMV)", algo_bytes, step_us,
                            "gemv_c1w4", kernel_us=step_us)}
    # the timed call against the CPU oracle: all 14336 fp16 outputs
    step()
    out["parity_vs_oracle"] = bool(np.array_equal(sess.from_device(dC, (M, N), np.uint16),
                                                  _oracle().w4a8(c["A"], c["B"], c["w_scale"])["C"]))
    sess.free_device(dA)
    sess.free_device(dC)
    ws.close()
    for w in copies:
        w.close()
    return out


def bench_c2w8(sess, ops, capi, workloads, steps, warmup):
    """w8a8 prefill GEMM at the same shape as config 2 (M=2048, K=4096, N=4096), int8 weights."""
    M, K, N = 2048, 4096, 4096
    c = workloads.w8a8_case(M, K, N, seed_w=4, seed_a=5)
    op = ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, M, c["B"], c["w_scale"])
    dA = sess.to_device(c["A"])
    dC = sess.empty_device(M * N * 2)
    lib = sess.lib

    def step():
        rc = op.run_device(dA, dC)
        if rc:
            raise RuntimeError("run_device rc=%d" % rc)

    def gemm_only():
        rc = lib.rk_npu_matmul_workspace_rerun_gemm_device(op.ws, op.w, dC)
        if rc:
            raise RuntimeError("rerun rc=%d" % rc)

    sess.spin_up(step)
    step_us = sess.time_us(step, steps, warmup)
    kernel_us = sess.time_us(gemm_only, steps, warmup)
    ops_count = 2.0 * M * K * N
    out = {"workload": "w8a8 prefill GEMM M=2048 K=4096 N=4096, fp16 in/out, seeds 4/5",
           "tops": ops_count / step_us / 1e6, "ms_per_step": step_us / 1e3,
           "roofline": _mfma("gemm_wk_kernel<int8,f16> (128x256 tile, waves split K)", ops_count, kernel_us,
                             kernel_us=kernel_us)}
    sess.free_device(dA)
    sess.free_device(dC)
    op.close()
    return out


def bench_c3(sess, ops, capi, workloads, steps, warmup, check=False):
    """fused w4a8 FFN block, M=128, hidden 4096, intermediate 14336."""
    c = workloads.CONFIGS[3]()
    M, H, I = c["M"], c["H"], c["I"]
    # the loop cycles through FFN_COPIES copies of the weights: see bench_c1
    gws_ = [ops.W4A8Weights(sess, c["B_gu"], c["s_gu"]) for _ in range(FFN_COPIES)]
    dws_ = [ops.W4A8Weights(sess, c["B_down"], c["s_down"]) for _ in range(FFN_COPIES)]
    gws, dws = ops.W4A8Workspace(sess, M, 2 * I, H), ops.W4A8Workspace(sess, M, H, I)
    dA = sess.to_device(c["x"])
    dmid = sess.empty_device(M * I * 4)
    dC = sess.empty_device(M * H * 4)
    turn = [0]

    def step():
        gw, dw = gws_[turn[0] % FFN_COPIES], dws_[turn[0] % FFN_COPIES]
        turn[0] += 1
        rc = sess.lib.rk_npu_w4a8_run_ffn_f32_device(gws.h, gw.h, dws.h, dw.h, dA, dmid, dC)
        if rc:
            raise RuntimeError("ffn rc=%d" % rc)

    sess.spin_up(step)
    step_us = sess.time_us(step, steps, warmup)
    ops_count = 2.0 * M * H * 2 * I + 2.0 * M * I * H
    weight_bytes = (H * 2 * I + I * H) // 2
    # weights once + x in + fp32 middle written and read back (it is an output of the call and
    # the input of the re-quantization) + out + both scale vectors
    algo_bytes = weight_bytes + M * H * 4 + 2 * M * I * 4 + M * H * 4 + (2 * I + H) * 4
    out = {"workload": "c3: fused w4a8 FFN M=128 H=4096 I=14336 (fp32 in / middle / out), seeds 6-9; the loop cycles "
                       "through %d copies of the 88 MB of weights" % FFN_COPIES,
           "tops": ops_count / step_us / 1e6, "weight_GBps": weight_bytes / step_us / 1e3,
           "ms_per_step": step_us / 1e3,
           "roofline": _hbm("whole step; dominant: gemm_wk_kernel<int4,SwiGLU> (gate/up, 58.7 MB of weights)",
                            algo_bytes, step_us, "ffn_c3", frac_of_int8_peak=ops_count / step_us / 1e6 / INT8_PEAK_TOPS,
                            algorithmic_ops=ops_count),
           "kernels": _kernels(sess, ops, step)}
    if check:
        want = _oracle().w4a8_ffn(c["x"], c["B_gu"], c["s_gu"], c["B_down"], c["s_down"], _oracle().EXP_POLY)
        step()
        mid, got = sess.from_device(dmid, (M, I), np.float32), sess.from_device(dC, (M, H), np.float32)
        out["parity_vs_oracle"] = bool(np.array_equal(mid.view(np.uint32), want["middle"].view(np.uint32)) and
                                       np.array_equal(got.view(np.uint32), want["C"].view(np.uint32)))
        out["host_api_us"] = _host_call_us(lambda: ops.w4a8_ffn(sess, gws, gws_[0], dws, dws_[0], c["x"]))
    for d in (dA, dmid, dC):
        sess.free_device(d)
    for o in [gws, dws] + gws_ + dws_:
        o.close()
    return out


def bench_c4(sess, ops, capi, workloads, steps, warmup, check=False):
    """w8a8 MoE layer, 256 tokens, hidden 2048, 32 experts, top-4, intermediate 1024."""
    c = workloads.CONFIGS[4]()
    # the loop alternates between MOE_COPIES banks (403 MB) so that the experts come from HBM
    banks = [ops.MoeW8(sess, c["H"], c["I"], c["E"], 0, c["top_k"], 256, c["experts"]) for _ in range(MOE_COPIES)]
    moe = banks[0]
    dx, dids, drt = sess.to_device(c["x"]), sess.to_device(c["ids"]), sess.to_device(c["routes"])
    dout = sess.empty_device(c["T"] * c["H"] * 4)
    turn = [0]

    def step():
        bank = banks[turn[0] % MOE_COPIES]
        turn[0] += 1
        rc = sess.lib.rk_npu_moe_w8_run_f32_device(moe.ws, bank.w, c["T"], dx, dids, drt, dout)
        if rc:
            raise RuntimeError("moe rc=%d" % rc)

    sess.spin_up(step)
    step_us = sess.time_us(step, steps, warmup)
    assignments = int((c["routes"] != 0).sum())
    ops_count = assignments * (2.0 * c["H"] * 2 * c["I"] + 2.0 * c["I"] * c["H"])
    weight_bytes = c["E"] * 3 * c["H"] * c["I"]
    # every expert's weights once + fp32 tokens in + fp32 result out + routing table + scales
    algo_bytes = (weight_bytes + 2 * c["T"] * c["H"] * 4 + 2 * c["T"] * c["top_k"] * 4 +
                  c["E"] * (2 * c["I"] + c["H"]) * 4)
    out = {"workload": "c4: w8a8 MoE T=256 H=2048 E=32 top-4 I=1024 (fp32 in / out), seeds 10-14; the loop "
                       "alternates between %d copies of the 201 MB expert bank" % MOE_COPIES,
           "tops": ops_count / step_us / 1e6, "weight_GBps": weight_bytes / step_us / 1e3,
           "ms_per_step": step_us / 1e3,
           "roofline": _hbm("whole step; dominant: gemm_stream_kernel<SwiGLU> (grouped gate/up, 134 MB of expert weights)",
                            algo_bytes, step_us, "moe_c4", algorithmic_ops=ops_count),
           "kernels": _kernels(sess, ops, step)}

    # The same layer at decode size: 1, 4 and 8 tokens per call.  Every step takes the next tokens of the
    # 256 (another set of experts) and the other bank, so the expert weights come from HBM here too.
    want = None
    decode = []
    for rows in (1, 4, 8):
        at = [0]

        def small_step():
            first = (at[0] * rows) % (c["T"] - rows + 1)
            bank = banks[at[0] % MOE_COPIES]
            at[0] += 1
            rc = sess.lib.rk_npu_moe_w8_run_f32_device(moe.ws, bank.w, rows, dx + first * c["H"] * 4,
                                                        dids + first * c["top_k"] * 4, drt + first * c["top_k"] * 4, dout)
            if rc:
                raise RuntimeError("moe rc=%d" % rc)

        us = sess.time_us(small_step, steps, warmup)
        # the rows of the last call against the same tokens' rows of the 256-token call (grouped path)
        last = ((at[0] - 1) * rows) % (c["T"] - rows + 1)
        got = sess.from_device(dout, (rows, c["H"]), np.float32)
        if want is None:
            step()
            if sess.sync():
                raise RuntimeError("sync")
            want = sess.from_device(dout, (c["T"], c["H"]), np.float32)
        decode.append({"tokens": rows, "us": us,
                       "equals_rows_of_the_256_token_call": bool(np.array_equal(got.view(np.uint32),
                                                                                want[last:last + rows].view(np.uint32)))})
    if check:
        rc, ref = _oracle().moe_w8(c["experts"], c["H"], c["I"], c["E"], 0, c["top_k"], c["ids"], c["routes"],
                                   input_f32=c["x"])
        step()
        got = sess.from_device(dout, (c["T"], c["H"]), np.float32)
        out["parity_vs_oracle"] = bool(rc == 0 and np.array_equal(got.view(np.uint32), ref.view(np.uint32)))
        out["host_api_us"] = _host_call_us(lambda: moe.run_f32(c["x"], c["ids"], c["routes"]))
    out["decode_sized_calls"] = {"note": "1 / 4 / 8 tokens per call through the same device-pointer call: two launches of "
                                         "dot-product kernels instead of five of the grouped path", "rows": decode}
    for d in (dx, dids, drt, dout):
        sess.free_device(d)
    for b in banks:
        b.close()
    return out


def bench_c0(sess, ops, capi, workloads, steps, warmup, check=False):
    c = workloads.CONFIGS[0]()
    M, K, N = c["M"], c["K"], c["N"]
    op = ops.W8A8Linear(sess, capi.F16I8F16_DYNAMIC, M, c["B"], c["w_scale"])
    dA = sess.to_device(c["A"])
    dC = sess.empty_device(M * N * 2)

    def step():
        rc = op.run_device(dA, dC)
        if rc:
            raise RuntimeError("run_device rc=%d" % rc)

    sess.spin_up(step)
    step_us = sess.time_us(step, steps, warmup)
    ops_count = 2.0 * M * K * N
    algo_bytes = K * N + M * K * 2 + M * N * 2 + N * 4 + M * 4
    out = {"workload": "c0: w8a8 GEMM M=64 K=2048 N=2048, fp16 in/out, seeds 0/1 (4.7 MB and 0.54 GOP: bound by launch "
                       "latency; the weights stay in the memory-side cache)",
           "tops": ops_count / step_us / 1e6, "weight_GBps": K * N / step_us / 1e3, "ms_per_step": step_us / 1e3,
           "roofline": _hbm("whole step; dominant: gemm_stream_kernel<KS=4> (64-column tiles, K split over the waves)",
                            algo_bytes, step_us, algorithmic_ops=ops_count),
           "kernels": _kernels(sess, ops, step)}
    if check:
        want = _oracle().w8a8(c["A"], c["B"], c["w_scale"])["C"]
        step()
        out["parity_vs_oracle"] = bool(np.array_equal(sess.from_device(dC, (M, N), np.uint16), want))
        out["host_api_us"] = _host_call_us(lambda: op.run(c["A"]))
    sess.free_device(dA)
    sess.free_device(dC)
    op.close()
    return out


def bench_llm_i8(sess, ops, capi, steps, warmup):
    """The reference's own quick benchmark (examples/bench_llm_i8.cpp:43-47,288-294): hidden, FFN-up
    and FFN-down projections of a 7B decoder as exact int8 x int8 -> int32 products at M = 1, 4
    and 128, reported its way -- K*N bytes / t as "weight GB/s" below 128 rows, 2*M*K*N / t as
    GOPS at 128 -- and, like it, checked on sampled outputs against the exact integer product.
    Here through the device-pointer call, every step on another copy of the matrix (HBM)."""
    rng = np.random.default_rng(1234)
    lib = sess.lib
    rows = []
    for name, K, N in (("hidden", 4096, 4096), ("ffn_up", 4096, 11008), ("ffn_down", 11008, 4096)):
        B = rng.integers(-128, 128, (K, N)).astype(np.int8)
        copies = max(2, int(400e6 // (K * N)))
        lins = [ops.W8A8Linear(sess, capi.I8I8I32, 1, B) for _ in range(copies)]
        cols = rng.choice(N, 64, replace=False)
        for M in (1, 4, 128):
            A = rng.integers(-128, 128, (M, K)).astype(np.int8)
            dA, dC = sess.to_device(A), sess.empty_device(M * N * 4)
            strategy = ops.default_strategy(capi.I8I8I32, M, N, K)
            ws = lib.rk_npu_matmul_workspace_create(sess.domain, C.byref(strategy))
            if not ws:
                raise RuntimeError("workspace_create")
            turn = [0]

            def step():
                turn[0] += 1
                rc = lib.rk_npu_i8i8i32_run_device(ws, lins[turn[0] % copies].w, dA, dC)
                if rc:
                    raise RuntimeError("i8i8i32_run_device rc=%d" % rc)

            us = sess.time_us(step, steps, warmup)
            got = sess.from_device(dC, (M, N), np.int32)
            exact = A.astype(np.int64) @ B[:, cols].astype(np.int64)
            row = {"projection": name, "M": M, "K": K, "N": N, "us": us,
                   "pass": bool(np.array_equal(got[:, cols], exact.astype(np.int32)))}
            if M < 128:
                row["weight_GBps"] = K * N / us / 1e3
            else:
                row["GOPS"] = 2.0 * M * K * N / us / 1e3
            rows.append(row)
            lib.rk_npu_matmul_workspace_free(ws)
            sess.free_device(dA)
            sess.free_device(dC)
        for l in lins:
            l.close()
    return {"workload": "the reference's bench_llm_i8 grid: rk_npu_i8i8i32 at M = 1 / 4 / 128, its reporting convention "
                        "(weight GB/s = K*N/t below 128 rows, GOPS = 2*M*K*N/t at 128), weights from HBM, no reference "
                        "figures are published for it", "rows": rows}


def bench_copy(sess, steps):
    """Calibration for the rocprofv3 --pmc traffic figures: a plain device-to-device
    copy of a known size (256 MiB read + 256 MiB written per launch)."""
    nbytes = 256 << 20
    src, dst = sess.empty_device(nbytes), sess.empty_device(nbytes)
    us = sess.time_us(lambda: sess.lib.rk_npu_hip_copy(sess.ctx, dst, src, nbytes), steps, 2)
    sess.free_device(src)
    sess.free_device(dst)
    return {"workload": "device-to-device copy, 268435456 B read + 268435456 B written per launch",
            "GBps_read_plus_write": 2 * nbytes / us / 1e3}


def practical_ceilings(sess):
    """What the box at hand gives with no arithmetic in the way (see include/rk_npu_hip.h):
    read-only streams in the decode GEMV's access order at the footprints of the HBM-bound
    configurations, and the pure int8 MFMA loop on random int8 operands."""
    rng = np.random.default_rng(0)
    return {
        "hbm_read_58MB_per_launch": read_probe(sess, 58720256, 131072),
        "hbm_read_29MB_per_launch": read_probe(sess, 29360128, 65536),
        "hbm_read_470MB_per_launch": read_probe(sess, C1_COPIES * 58720256, 131072, iters=20),
        "mfma_int8_random_operands_TOPS": mfma_probe(sess, rng.integers(-127, 128, 32768).astype(np.int8)),
        "mfma_int8_zero_operands_TOPS": mfma_probe(sess, np.zeros(32768, np.int8)),
        "note": "read-only stream (16 B per lane, 8 loads per wave in flight, one workgroup per 128 / 64 KiB span, "
                "rotating over 470 MB) and pure v_mfma_i32_32x32x32_i8 loop (8 waves per CU, operands in registers); "
                "launch gaps included, as in every figure of this line",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="all", choices=["c1", "all"],
                    help="all: the headline line with every BASELINE configuration under \"also\" (default); "
                         "c1: config 1, config 2 and the int4 GEMV only")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--only", default=None, choices=["c0", "c1", "c1w4", "c2", "c2w8", "c3", "c4", "llm_i8", "copy", "probes"],
                    help="profiling aid: run one configuration's loop only")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.stderr.write("bench.py: this path runs on one GPU; --gpus %d is not supported "
                         "(every box of this build has one GPU, no collectives exist)\n" % args.gpus)
        sys.exit(2)

    from rknpu2_matmul_open_amd import capi, ops, workloads
    sess = ops.Session()
    arch, cus, khz = sess.device_info()
    log("device %s, %d CUs, %d MHz" % (arch, cus, khz // 1000))

    if args.only == "copy":
        print(json.dumps(bench_copy(sess, min(args.steps, 10))))
        sess.close()
        return
    if args.only == "probes":
        print(json.dumps(practical_ceilings(sess)))
        sess.close()
        return
    if args.only == "llm_i8":
        print(json.dumps(bench_llm_i8(sess, ops, capi, args.steps, args.warmup)))
        sess.close()
        return
    if args.only:
        fn = {"c0": bench_c0, "c1w4": bench_c1w4, "c2": bench_c2, "c2w8": bench_c2w8, "c3": bench_c3, "c4": bench_c4}.get(args.only)
        res = (bench_c1(sess, ops, capi, workloads, args.steps, args.warmup, False)
               if args.only == "c1" else fn(sess, ops, capi, workloads, args.steps, args.warmup))
        print(json.dumps(res))
        sess.close()
        return

    # GPU measurements first, back to back; the CPU baseline (about 10 s during
    # which the device idles and clocks down) runs last, inside bench_c1.
    log("config 2 (prefill GEMM)")
    check = not args.no_cpu_baseline   # the oracle as checker, outside every timed loop
    also = {"c2": bench_c2(sess, ops, capi, workloads, args.steps, args.warmup, check=check)}
    log("w4a8 decode GEMV")
    also["c1w4"] = bench_c1w4(sess, ops, capi, workloads, args.steps, args.warmup)
    if args.workload == "all":
        for name, fn in (("c0", bench_c0), ("c3", bench_c3), ("c4", bench_c4)):
            log("config %s" % name)
            also[name] = fn(sess, ops, capi, workloads, args.steps, args.warmup, check=check)
        log("the reference's bench_llm_i8 grid")
        also["llm_i8"] = bench_llm_i8(sess, ops, capi, args.steps, args.warmup)
    log("practical ceilings (read-only stream, pure MFMA loop)")
    practical = practical_ceilings(sess)
    log("config 1 (decode GEMV)")
    r1 = bench_c1(sess, ops, capi, workloads, args.steps, args.warmup, not args.no_cpu_baseline)
    r1["roofline"]["practical_peak"] = practical["hbm_read_58MB_per_launch"]["GBps"]
    r1["roofline"]["frac_of_practical_peak"] = r1["roofline"]["achieved"] / r1["roofline"]["practical_peak"]
    w4 = also["c1w4"]["roofline"]
    w4["practical_peak"] = practical["hbm_read_29MB_per_launch"]["GBps"]
    w4["frac_of_practical_peak"] = w4["achieved"] / w4["practical_peak"]
    for name in ("c3", "c4"):
        if name in also:
            r = also[name]["roofline"]
            r["practical_peak"] = practical["hbm_read_470MB_per_launch"]["GBps"]
            r["frac_of_practical_peak"] = r["achieved"] / r["practical_peak"]
    line = {
        "metric": METRIC, "value": r1["value"], "unit": r1["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": r1["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": r1["dtype"],
        "data": "synthetic (seeded numpy PCG64; weights N(0,0.02) quantized per channel, activations fp16 N(0,1))",
        "config": r1["config"], "roofline": r1["roofline"],
        "device": {"arch": arch, "compute_units": cus, "clock_mhz": khz // 1000},
        "practical": practical,
        "also": also,
    }
    if "cpu_baseline" in r1:
        line["cpu_baseline"] = r1["cpu_baseline"]
        line["parity_vs_oracle"] = r1["parity"]
        # The blocking host-pointer calls of the reference API on the same configurations: host
        # buffers in, host buffers out, so PCIe transfers and the stream wait are inside the time.
        # Never `value`; the device-resident step time stands beside each for scale.
        host = {"c1": {"call": "rk_npu_f16i8f16_run_dynamic", "us": r1["host_api_us"],
                       "device_resident_step_us": r1["ms_per_step"] * 1e3}}
        for name, call in (("c0", "rk_npu_f16i8f16_run_dynamic"), ("c2", "rk_npu_w4a8_run_f16"),
                           ("c3", "rk_npu_w4a8_run_ffn_f32"), ("c4", "rk_npu_moe_w8_run_f32")):
            if name in also and "host_api_us" in also[name]:
                host[name] = {"call": call, "us": also[name].pop("host_api_us"),
                              "device_resident_step_us": also[name]["ms_per_step"] * 1e3}
        host["note"] = ("PCIe-inclusive: blocking reference-API calls on host buffers (H2D + kernels + D2H + wait), "
                        "median of 10 after 2 warm-ups as in the reference's examples/bench_llm_i8.cpp:43-47; "
                        "not the headline value")
        also["host_api"] = host
    print(json.dumps(line))
    sess.close()


if __name__ == "__main__":
    main()
