#!/usr/bin/env python3
"""Benchmark of the quantized MUL_MAT hot path on one MI355X.

Headline workload (BASELINE configs[4], the largest single-GPU configuration): every weight matmul of one decode step of a
random-init Llama-3-8B-shaped Q4_K_M model - 32 layers of wq / wk / wv(Q6_K) / wo / ffn_gate / ffn_up / ffn_down(Q6_K) plus
the Q6_K output head, 225 matmuls over 4 875 853 824 weight bytes - at one token.  One "step" = that serial chain, issued
through the C-ABI the way the ggml backend issues it (matmuls that share an activation in one launch), each op doing what
LM_GGML_OP_MUL_MAT does: quantize the fp32 activation on the GPU, then the GEMV.  The weights of a step (4.9 GB) exceed the
256 MB Infinity Cache many times over, so every read is cold.  The step is replayed as a HIP graph (the host cannot issue
225 launches from Python in the time the GPU needs for them); --eager issues the same launches one by one, for runs under a
profiler.

Prints ONE JSON line.  `value` = algorithmic bytes of a step / wall time of a step (HIP events on the launch stream, K steps
between one pair of events).  `roofline` is for the kernel with the largest share of the step, timed with its own HIP event
pair over back-to-back launches on distinct (cold) weights.  `cpu_baseline` times the reference's own ggml-cpu MUL_MAT
(oracle/_ref, when it travelled) or the oracle port on the host cores for a bounded sample of the same workload.  `extra`
carries the other BASELINE configurations (Q4_0 mat-vec, Q8_0 FFN GEMVs, Q4_K GEMV, prefill GEMM TOPS, the trace at 8 tokens
and as a 512-token prefill chunk).
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

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
INT8_PEAK_TOPS = 5000.0        # MI355X published dense int8 MFMA rate
F16_PEAK_TFLOPS = 2500.0       # MI355X published dense fp16 MFMA rate
# HBM bytes per launch of the dominant kernel come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, scaled by what the
# same counters read for a device-to-device copy of known size.  The summary of those runs is a committed text file; its
# line "traffic_bytes_per_launch: <kernel key> <bytes>" is read here, so the figure in the JSON is the profile's.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemv_trace_dominant_kernel_hbm_traffic_pmc.md")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--eager", action="store_true",
                    help="issue every launch of the trace directly instead of replaying a HIP graph, and skip everything that "
                         "replays one (for runs under rocprofv3 --kernel-trace; the host then bounds the step time)")
    ap.add_argument("--no-backend", action="store_true", help="skip the ggml-backend graph timing (a child process)")
    ap.add_argument("--block-order", action="store_true",
                    help="keep the Q6_K weights as block_q6_K rows for the one-token step too (default: rows in planes, as the "
                         "backend keeps them for matmuls of up to 4 tokens)")
    ap.add_argument("--only-trace", type=int, default=0, metavar="N", choices=(0, 1, 8, 512),
                    help="run nothing but the trace step at N tokens, every launch issued directly, --warmup + --steps times, and "
                         "print its time (for a per-kernel table of that step under rocprofv3 --kernel-trace --stats)")
    return ap.parse_args()


class Hip:
    """The few HIP runtime calls the harness needs beyond the C-ABI: events and graph capture."""

    def __init__(self):
        self.lib = L = C.CDLL("libamdhip64.so")
        L.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        L.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        L.hipEventSynchronize.argtypes = [C.c_void_p]
        L.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        L.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
        L.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        L.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
        L.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
        L.hipGraphExecDestroy.argtypes = [C.c_void_p]
        L.hipGraphDestroy.argtypes = [C.c_void_p]
        L.hipStreamWaitEvent.argtypes = [C.c_void_p, C.c_void_p, C.c_uint]
        L.hipDeviceSynchronize.argtypes = []

    def event(self):
        e = C.c_void_p()
        assert self.lib.hipEventCreate(C.byref(e)) == 0
        return e

    def record(self, e, stream):
        assert self.lib.hipEventRecord(e, stream) == 0

    def capture(self, stream, fn):
        """Runs fn() under stream capture and returns a replay function and a destroy function."""
        L = self.lib
        graph, gexec = C.c_void_p(), C.c_void_p()
        assert L.hipStreamBeginCapture(stream, 0) == 0
        fn()
        assert L.hipStreamEndCapture(stream, C.byref(graph)) == 0
        assert L.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0

        def destroy():
            L.hipGraphExecDestroy(gexec)
            L.hipGraphDestroy(graph)
        return (lambda: L.hipGraphLaunch(gexec, stream)), destroy

    def elapsed_ms(self, a, b):
        assert self.lib.hipEventSynchronize(b) == 0
        ms = C.c_float()
        assert self.lib.hipEventElapsedTime(C.byref(ms), a, b) == 0
        return ms.value


def synth_weights(dev, wtype, N, K, rng):
    """Random-init weights directly in block form: random quants, a fixed small fp16 scale per block."""
    L = dev.lib
    be, bb = L.chip_block_elems(wtype), L.chip_block_bytes(wtype)
    w = rng.integers(0, 256, (N, K // be, bb), dtype=np.uint8)
    d = np.array([0.0107], np.float16).view(np.uint8)
    import cactus_amd as ca
    if wtype == ca.F16:
        return rng.standard_normal((N, K)).astype(np.float16).view(np.uint8).reshape(N, -1)
    if wtype == ca.Q6_K:
        w[..., 208:210] = d
    else:
        w[..., 0:2] = d                                   # d first in every other block format
        if wtype in (ca.Q4_K, ca.Q5_K, ca.Q4_1, ca.Q5_1):
            w[..., 2:4] = d                               # dmin / m follow it
    return w.reshape(N, -1)


class RotatingWeights:
    """`copies` distinct copies of one weight matrix in HBM, handed out round robin (cold-cache reads)."""

    def __init__(self, dev, wtype, N, K, rng, min_bytes=640e6, host=None):
        self.dev, self.wtype, self.N, self.K = dev, wtype, N, K
        self.nb01 = dev.row_size(wtype, K)
        self.bytes = N * self.nb01
        self.copies = max(2, int(min_bytes // self.bytes) + 1)
        self.host = synth_weights(dev, wtype, N, K, rng) if host is None else host
        self.buf = dev.alloc(self.copies * self.bytes)
        self.buf.upload(self.host)
        for c in range(1, self.copies):
            dev.check(dev.lib.chip_memcpy_d2d(self.buf.ptr + c * self.bytes, self.buf.ptr, self.bytes, None))
        dev.sync()
        self.i = 0

    def next(self):
        p = self.buf.ptr + (self.i % self.copies) * self.bytes
        self.i += 1
        return p


def algorithmic_bytes(wbytes, K, N, n):
    return wbytes + 4 * n * (K + N)            # weights once + fp32 activations in + fp32 outputs out


def bench_config2(dev, hip, steps=20, warmup=3):
    """BASELINE configs[1]: Q8_0 FFN-shaped GEMVs at 1, 2, 4, 8 tokens, cold weights (rotating copies)."""
    import cactus_amd as ca
    L = dev.lib
    rng = np.random.default_rng(2)
    shapes = [(11008, 4096), (4096, 11008)]
    batches = [1, 2, 4, 8]
    mats = [RotatingWeights(dev, ca.Q8_0, N, K, rng) for (N, K) in shapes]
    xs = {K: dev.to_device(rng.standard_normal((8, K)).astype(np.float32)) for (_, K) in shapes}
    ys = dev.alloc(8 * 11008 * 4)
    wsz = max(L.chip_mul_mat_workspace_size(ca.Q8_0, K, 8) for (_, K) in shapes)
    ws = dev.alloc(wsz)
    st = C.c_void_p()
    dev.check(L.chip_stream_create(C.byref(st)))

    def step():
        for m in mats:
            for n in batches:
                dev.check(L.chip_mul_mat(ca.Q8_0, m.next(), m.nb01, m.K, m.N, xs[m.K].ptr, m.K, n, ys.ptr, m.N, ws.ptr, wsz, st))

    for _ in range(warmup):
        step()
    dev.sync(st)
    e0, e1 = hip.event(), hip.event()
    hip.record(e0, st)
    for _ in range(steps):
        step()
    hip.record(e1, st)
    ms = hip.elapsed_ms(e0, e1)

    step_bytes = sum(algorithmic_bytes(m.bytes, m.K, m.N, n) for m in mats for n in batches)
    ms_per_step = ms / steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # Dominant kernel: the n = 1 GEMV (one launch per op: activation quantization happens in its prologue).
    # Its own timed region: the same two shapes, cold weights, launches back to back on the same stream between
    # one HIP event pair (an event between every launch would cost more than the kernel itself).
    def n1_pass():
        for m in mats:
            dev.check(L.chip_mul_mat(ca.Q8_0, m.next(), m.nb01, m.K, m.N, xs[m.K].ptr, m.K, 1, ys.ptr, m.N, ws.ptr, wsz, st))

    reps = max(20, 2 * steps)
    n1_pass()
    dev.sync(st)
    hip.record(e0, st)
    for _ in range(reps):
        n1_pass()
    hip.record(e1, st)
    k_us = hip.elapsed_ms(e0, e1) * 1e3 / (2 * reps)
    dev.sync(st)
    k_bytes = algorithmic_bytes(mats[0].bytes, 4096, 11008, 1)      # both shapes move the same byte count
    achieved = k_bytes / (k_us * 1e-6) / 1e9
    for m in mats:
        m.buf.free()
    return {"step_8_ops_us": round(ms_per_step * 1e3, 2), "step_GBps": round(value, 1), "bytes_per_step": step_bytes,
            "n1_us_per_launch": round(k_us, 2), "n1_GBps": round(achieved, 1), "n1_hbm_frac": round(achieved / HBM_PEAK_GBS, 4),
            "n1_bytes_per_launch": k_bytes, "copies_per_shape": [m.copies for m in mats]}


def time_runs(dev, hip, st, fn, iters, warm=3):
    for _ in range(warm):
        fn()
    dev.sync(st)
    a, b = hip.event(), hip.event()
    hip.record(a, st)
    for _ in range(iters):
        fn()
    hip.record(b, st)
    return hip.elapsed_ms(a, b) * 1e3 / iters          # microseconds per call


def bench_extra(dev, hip):
    import cactus_amd as ca
    L = dev.lib
    rng = np.random.default_rng(5)
    st = C.c_void_p()
    dev.check(L.chip_stream_create(C.byref(st)))
    out = {}

    def gemv_case(name, wt, N, K, n, iters=200):
        m = RotatingWeights(dev, wt, N, K, rng)
        x = dev.to_device(rng.standard_normal((n, K)).astype(np.float32))
        y = dev.alloc(n * N * 4)
        wsz = L.chip_mul_mat_workspace_size_n(wt, K, N, n)
        ws = dev.alloc(wsz)
        dev.check(L.chip_mul_mat_prepare(wt, K, x.ptr, K, n, ws.ptr, wsz, st))
        us_run = time_runs(dev, hip, st, lambda: L.chip_mul_mat_run_ws(wt, m.next(), m.nb01, K, N, n, ws.ptr, wsz, y.ptr, N, st), iters)
        us_op = time_runs(dev, hip, st, lambda: L.chip_mul_mat(wt, m.next(), m.nb01, K, N, x.ptr, K, n, y.ptr, N, ws.ptr, wsz, st), iters)
        b = algorithmic_bytes(m.bytes, K, N, n)
        out[name] = {"us_gemv": round(us_run, 2), "us_op": round(us_op, 2), "GBps_gemv": round(b / us_run / 1e3, 1),
                     "GBps_op": round(b / us_op / 1e3, 1), "hbm_frac_gemv": round(b / us_run / 1e3 / HBM_PEAK_GBS, 4),
                     "bytes": b, "cold_copies": m.copies}
        m.buf.free()

    gemv_case("config1_q4_0_4096x4096_n1", ca.Q4_0, 4096, 4096, 1)
    gemv_case("config3_q4_K_14336x4096_n1", ca.Q4_K, 14336, 4096, 1)
    # 8 tokens (a small serving batch): the matrix-core GEMV of each weight type that has one, the dot-product GEMV otherwise
    for wt in (ca.Q8_0, ca.Q4_0, ca.Q4_K, ca.Q5_K, ca.Q6_K):
        gemv_case("batch8_%s_14336x4096" % ca.TYPE_NAMES[wt], wt, 14336, 4096, 8, iters=100)

    # config 4: prefill GEMM on int8 MFMA (Q4_0 is the configuration BASELINE names; the other weight types run the
    # same shapes through their own GEMM kernels: block-32 types, K-quants with digit-plane operands, F16 on fp16 MFMA)
    def gemm_case(key, wt, N, M, K=4096):
        w = dev.to_device(synth_weights(dev, wt, N, K, rng))
        x = dev.to_device(rng.standard_normal((M, K)).astype(np.float32))
        y = dev.alloc(M * N * 4)
        wsz = L.chip_mul_mat_workspace_size_n(wt, K, N, M)
        ws = dev.alloc(wsz)
        nb01 = dev.row_size(wt, K)
        dev.check(L.chip_mul_mat_prepare(wt, K, x.ptr, K, M, ws.ptr, wsz, st))
        us_g = time_runs(dev, hip, st, lambda: L.chip_mul_mat_run_ws(wt, w.ptr, nb01, K, N, M, ws.ptr, wsz, y.ptr, N, st), 20)
        us_o = time_runs(dev, hip, st, lambda: L.chip_mul_mat(wt, w.ptr, nb01, K, N, x.ptr, K, M, y.ptr, N, ws.ptr, wsz, st), 20)
        ops = 2.0 * M * N * K
        peak = F16_PEAK_TFLOPS if wt == ca.F16 else INT8_PEAK_TOPS
        out[key] = {"us_gemm": round(us_g, 1), "us_op": round(us_o, 1), "TOPS_gemm": round(ops / us_g / 1e6, 1),
                    "TOPS_op": round(ops / us_o / 1e6, 1), "mfma_frac_gemm": round(ops / us_g / 1e6 / peak, 4)}
        for b in (w, x, y, ws):
            b.free()

    for (N, M) in ((4096, 512), (4096, 2048), (14336, 512), (14336, 2048)):
        gemm_case("config4_q4_0_%dx4096_M%d" % (N, M), ca.Q4_0, N, M)
    for wt in (ca.Q8_0, ca.Q4_K, ca.Q5_K, ca.Q6_K, ca.F16):
        for (N, M) in ((4096, 512), (14336, 2048)):
            gemm_case("prefill_%s_%dx4096_M%d" % (ca.TYPE_NAMES[wt], N, M), wt, N, M)

    # MUL_MAT_ID (mixture-of-experts matmul), decode: one token, every (token, slot) pair a GEMV on its expert
    def moe_case(key, wt, n_as, n_used, N, K, n_tokens=1):
        nb01 = dev.row_size(wt, K)
        one = synth_weights(dev, wt, N, K, rng)
        w = dev.alloc(n_as * N * nb01)
        w.upload(one)
        for e in range(1, n_as):
            dev.check(L.chip_memcpy_d2d(w.ptr + e * N * nb01, w.ptr, N * nb01, None))
        x = dev.to_device(rng.standard_normal((n_tokens, K)).astype(np.float32))
        y = dev.alloc(n_tokens * n_used * N * 4)
        wsz = L.chip_mul_mat_id_workspace_size(wt, K, n_as, n_used, n_tokens, 1)
        ws = dev.alloc(wsz)
        # a different set of experts on every call, so the weights come from HBM like in a real layer stack
        sets = [np.stack([rng.permutation(n_as)[:n_used] for _ in range(n_tokens)]).astype(np.int32) for _ in range(16)]
        ids = [dev.to_device(s_) for s_ in sets]
        state = {"i": 0}

        def call():
            state["i"] += 1
            return L.chip_mul_mat_id(wt, w.ptr, nb01, N * nb01, K, N, n_as, x.ptr, K, 1, ids[state["i"] % 16].ptr, n_used,
                                     n_used, n_tokens, y.ptr, N, ws.ptr, wsz, st)
        us = time_runs(dev, hip, st, call, 100 if n_tokens == 1 else 20)
        if n_tokens == 1:
            b = n_used * N * nb01 + 4 * (K + n_used * N)
            out[key] = {"us_op": round(us, 2), "GBps_op": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 1e3 / HBM_PEAK_GBS, 4),
                        "bytes": b, "experts": n_as, "used": n_used}
        else:                                                       # prefill: pairs grouped by expert, MFMA GEMMs
            ops = 2.0 * n_tokens * n_used * N * K
            out[key] = {"us_op": round(us, 1), "TOPS_op": round(ops / us / 1e6, 1), "tokens": n_tokens, "experts": n_as,
                        "used": n_used}
        for bf in [w, x, y, ws] + ids:
            bf.free()

    moe_case("moe_q4_K_128x8_768x2048_n1", ca.Q4_K, 128, 8, 768, 2048)          # Qwen3-30B-A3B-shaped expert up/gate
    moe_case("moe_q4_K_8x2_14336x4096_n1", ca.Q4_K, 8, 2, 14336, 4096)          # Mixtral-8x7B-shaped expert up/gate
    moe_case("moe_q4_K_128x8_768x2048_n512", ca.Q4_K, 128, 8, 768, 2048, 512)
    moe_case("moe_q4_K_8x2_14336x4096_n512", ca.Q4_K, 8, 2, 14336, 4096, 512)

    # the element-wise ops between the matmuls (F32 rows): HBM-bound streams, bytes = reads + writes
    def ew_case(key, fn, n, ne0, streams):
        a = dev.to_device(rng.standard_normal((n, ne0)).astype(np.float32))
        b = dev.to_device(rng.standard_normal((n, ne0)).astype(np.float32))
        y = dev.alloc(n * ne0 * 4)
        us = time_runs(dev, hip, st, lambda: fn(a, b, y, n, ne0), 50)
        byts = streams * n * ne0 * 4
        out[key] = {"us": round(us, 2), "GBps": round(byts / us / 1e3, 1), "hbm_frac": round(byts / us / 1e3 / HBM_PEAK_GBS, 4)}
        for bf in (a, b, y):
            bf.free()

    for (n, ne0) in ((1, 4096), (512, 4096), (512, 14336)):
        ew_case("rms_norm_%dx%d" % (n, ne0), lambda a, b, y, n_, e: L.chip_rms_norm(a.ptr, e, n_, e, 1e-5, y.ptr, e, st), n, ne0, 2)
        ew_case("silu_%dx%d" % (n, ne0), lambda a, b, y, n_, e: L.chip_silu(a.ptr, e, n_, e, y.ptr, e, st), n, ne0, 2)
        ew_case("mul_%dx%d" % (n, ne0), lambda a, b, y, n_, e: L.chip_mul(a.ptr, e, b.ptr, e, n_, n_, e, y.ptr, e, st), n, ne0, 3)
        ew_case("add_%dx%d" % (n, ne0), lambda a, b, y, n_, e: L.chip_add(a.ptr, e, b.ptr, e, n_, n_, e, y.ptr, e, st), n, ne0, 3)

    # attention-side ops at LLaMA-3-8B shapes (32 heads, 8 KV heads of 128): decode over 4096 cached keys, prefill of 512 tokens
    def attn_side_cases():
        A = C.c_int64 * 4
        hd, n_head, n_head_kv, kv_size = 128, 32, 8, 8192
        n_embd_kv = hd * n_head_kv
        for n_tok, n_kv in ((1, 4096), (512, 512), (512, 4096)):
            rows = n_head * n_tok
            kq = dev.to_device((rng.standard_normal((rows, n_kv)) * 4).astype(np.float32))
            mask = dev.to_device(np.zeros((max(n_tok, 8), n_kv), np.float16))
            us = time_runs(dev, hip, st, lambda: L.chip_soft_max(kq.ptr, n_kv, mask.ptr, ca.F16, n_kv, n_tok, rows, 0.088, 0.0,
                                                                  kq.ptr, n_kv, st), 50)
            byts = rows * n_kv * 8 + n_tok * n_kv * 2
            out["soft_max_%dx%d" % (rows, n_kv)] = {"us": round(us, 2), "GBps": round(byts / us / 1e3, 1)}
            q = dev.to_device(rng.standard_normal((n_tok, n_head, hd)).astype(np.float32))
            pos = dev.to_device(np.arange(n_tok, dtype=np.int32))
            us = time_runs(dev, hip, st, lambda: L.chip_rope(q.ptr, hd, hd * n_head, pos.ptr, None, hd, n_head, n_tok, hd, 2, 8192,
                                                              500000.0, 1.0, 0.0, 1.0, 32.0, 1.0, q.ptr, hd, hd * n_head, st), 50)
            out["rope_%dx%dx%d" % (n_tok, n_head, hd)] = {"us": round(us, 2), "GBps": round(n_tok * n_head * hd * 8 / us / 1e3, 1)}
            k = dev.to_device(rng.standard_normal((n_tok, n_embd_kv)).astype(np.float32))
            cache = dev.alloc(kv_size * n_embd_kv * 2)
            flat, one = A(n_tok * n_embd_kv, 1, 1, 1), n_tok * n_embd_kv
            us = time_runs(dev, hip, st, lambda: L.chip_cpy(k.ptr, ca.F32, flat, A(4, 4 * one, 4 * one, 4 * one), cache.ptr, ca.F16, flat,
                                                             A(2, 2 * one, 2 * one, 2 * one), st), 50)
            out["k_store_%dx%d" % (n_tok, n_embd_kv)] = {"us": round(us, 2), "GBps": round(one * 6 / us / 1e3, 1)}
            shape = A(n_tok, n_embd_kv, 1, 1)
            us = time_runs(dev, hip, st, lambda: L.chip_cpy(k.ptr, ca.F32, shape, A(n_embd_kv * 4, 4, 0, 0), cache.ptr, ca.F16, shape,
                                                             A(2, kv_size * 2, 0, 0), st), 50)
            out["v_store_transposed_%dx%d" % (n_tok, n_embd_kv)] = {"us": round(us, 2), "GBps": round(one * 6 / us / 1e3, 1)}
            # kq = mul_mat(K cache, q) and kqv = mul_mat(transposed V cache, probabilities), F16 caches of kv_size positions
            kcache = dev.to_device((rng.standard_normal((kv_size, n_embd_kv)) * 0.5).astype(np.float16))
            vcache = dev.to_device((rng.standard_normal((n_embd_kv, kv_size)) * 0.5).astype(np.float16))
            kq_out = dev.alloc(n_head * n_tok * n_kv * 4)
            kqv_out = dev.alloc(n_head * n_tok * hd * 4)
            aws_bytes = max(L.chip_mul_mat_f16_batched_workspace_size(hd, n_kv, n_head_kv, n_head, n_tok),
                            L.chip_mul_mat_f16_batched_workspace_size(n_kv, hd, n_head_kv, n_head, n_tok), 256)
            aws = dev.alloc(aws_bytes)
            us = time_runs(dev, hip, st, lambda: L.chip_mul_mat_f16_batched(kcache.ptr, 2 * n_embd_kv, 2 * hd, hd, n_kv, n_head_kv, q.ptr,
                                                                             hd * n_head, hd, n_tok, n_head, kq_out.ptr, n_kv, n_kv * n_tok,
                                                                             aws.ptr, aws_bytes, st), 30)
            cache_bytes = n_kv * n_embd_kv * 2
            flops = 2.0 * n_head * n_tok * n_kv * hd
            out["attn_kq_%dtok_%dkv" % (n_tok, n_kv)] = {"us": round(us, 2), "cache_GBps": round(cache_bytes / us / 1e3, 1),
                                                          "TFLOPs": round(flops / us / 1e6, 2)}
            us = time_runs(dev, hip, st, lambda: L.chip_mul_mat_f16_batched(vcache.ptr, 2 * kv_size, 2 * kv_size * hd, n_kv, hd, n_head_kv,
                                                                             kq.ptr, n_kv, n_kv * n_tok, n_tok, n_head, kqv_out.ptr, hd,
                                                                             hd * n_tok, aws.ptr, aws_bytes, st), 30)
            out["attn_kqv_%dtok_%dkv" % (n_tok, n_kv)] = {"us": round(us, 2), "cache_GBps": round(cache_bytes / us / 1e3, 1),
                                                           "TFLOPs": round(flops / us / 1e6, 2)}
            for bf in (kq, mask, q, pos, k, cache, kcache, vcache, kq_out, kqv_out, aws):
                bf.free()

    attn_side_cases()

    # weight upload, the model loader's two branches (llama-model-loader.cpp:905-1064) with a host memmove standing for the
    # file read: blocking (the tensor read into a pageable buffer, then one synchronous copy) against four pinned 1 MB
    # staging buffers with an event each (chunked set_tensor_async); and the bare synchronous copy for reference
    def upload_case():
        total, chunk, nbuf = 256 << 20, 1 << 20, 4
        src = rng.integers(0, 256, total, dtype=np.uint8)
        tmp = np.empty(total, np.uint8)
        dst = dev.alloc(total)
        t0 = time.perf_counter()
        dev.check(L.chip_memcpy_h2d(dst.ptr, src.ctypes.data, total, None))
        t_copy = time.perf_counter() - t0
        t0 = time.perf_counter()
        C.memmove(tmp.ctypes.data, src.ctypes.data, total)                        # the loader's file read
        dev.check(L.chip_memcpy_h2d(dst.ptr, tmp.ctypes.data, total, None))
        t_sync = time.perf_counter() - t0
        pins, evs = [], []
        for _ in range(nbuf):
            p_, e_ = C.c_void_p(), C.c_void_p()
            dev.check(L.chip_host_malloc(C.byref(p_), chunk))
            dev.check(L.chip_event_create(C.byref(e_)))
            pins.append(p_)
            evs.append(e_)
        t0 = time.perf_counter()
        for i, off in enumerate(range(0, total, chunk)):
            b_ = i % nbuf
            dev.check(L.chip_event_synchronize(evs[b_]))
            C.memmove(pins[b_], src.ctypes.data + off, chunk)                     # the loader's file read
            dev.check(L.chip_memcpy_h2d(dst.ptr + off, pins[b_], chunk, st))
            dev.check(L.chip_event_record(evs[b_], st))
        dev.sync(st)
        t_async = time.perf_counter() - t0
        ok = bool(np.array_equal(dst.download(np.uint8, 1 << 20, total - (1 << 20)), src[-(1 << 20):]))
        for p_, e_ in zip(pins, evs):
            L.chip_host_free(p_)
            L.chip_event_destroy(e_)
        dst.free()
        out["upload_256MB"] = {"blocking_branch_read_then_copy_GBps": round(total / t_sync / 1e9, 2),
                               "async_branch_pinned_chunks_GBps": round(total / t_async / 1e9, 2),
                               "bare_copy_from_pageable_GBps": round(total / t_copy / 1e9, 2), "verified": ok}

    upload_case()

    return out


def measured_mfma_peak():
    """Runs the issue-rate probe (a child process) and returns the best device-wide rate it saw for the MFMA
    form the GEMM uses, so TOPS can be read against the measured matrix peak as well as the datasheet one."""
    import re
    import subprocess
    exe = os.path.join(ROOT, "cactus_amd", "probes", "bin", "issue_rates")
    if not os.path.exists(exe):
        return None
    try:
        txt = subprocess.run([exe], capture_output=True, text=True, timeout=60).stdout
    except Exception:
        return None
    best = 0.0
    for line in txt.splitlines():
        if line.startswith("mfma_i32_32x32x32_i8"):
            m = re.search(r";\s*([\d.]+) Tops/s", line)
            if m:
                best = max(best, float(m.group(1)))
    return {"instruction": "v_mfma_i32_32x32x32_i8", "TOPS": best, "datasheet_TOPS": INT8_PEAK_TOPS} if best else None


def measured_read_floor():
    """Runs the read-only streaming probe (a child process): what a kernel that only reads the bytes of each matrix of the
    decode trace costs on this GPU, cold.  The sum over one step is the floor under a one-kernel-per-op decode step."""
    import re
    import subprocess
    exe = os.path.join(ROOT, "cactus_amd", "probes", "bin", "read_stream")
    if not os.path.exists(exe):
        return None
    try:
        txt = subprocess.run([exe], capture_output=True, text=True, timeout=120).stdout
    except Exception:
        return None
    out = {}
    for line in txt.splitlines():
        m = re.match(r"read\s+([\d.]+) MB \((.*?)\s*\): cold\s+([\d.]+) us", line)
        if m:
            out[m.group(2).strip()] = {"MB": float(m.group(1)), "cold_us": float(m.group(3))}
        m = re.match(r"empty kernel, back to back: ([\d.]+) us", line)
        if m:
            out["empty_launch_us"] = float(m.group(1))
    need = ("wq+wk+wv", "wo Q4_K 4096x4096 / config 1", "ffn_gate+ffn_up", "ffn_down Q6_K / config 2 Q8_0", "output head Q6_K 128256x4096")
    if all(k in out for k in need):
        out["decode_step_floor_us"] = round(32 * sum(out[k]["cold_us"] for k in need[:4]) + out[need[4]]["cold_us"], 1)
    return out or None


class Trace:
    """BASELINE configs[4]: the weight matmuls of a Llama-3-8B-shaped Q4_K_M model (32 layers; attn_v / ffn_down / the
    output head in Q6_K, the rest Q4_K) as random-init weights in one arena, and the launches of one step over them."""
    H, FF, KV, V, NL = 4096, 14336, 1024, 128256, 32

    def __init__(self, dev, hip, rng):
        import cactus_amd as ca
        self.dev, self.hip, self.ca = dev, hip, ca
        L = dev.lib
        H, FF, KV, V, NL = self.H, self.FF, self.KV, self.V, self.NL
        self.layer = [("wq", ca.Q4_K, H, H), ("wk", ca.Q4_K, KV, H), ("wv", ca.Q6_K, KV, H), ("wo", ca.Q4_K, H, H),
                      ("up", ca.Q4_K, FF, H), ("gate", ca.Q4_K, FF, H), ("down", ca.Q6_K, H, FF)]
        sizes = [N * dev.row_size(t, K) for (_, t, N, K) in self.layer]
        self.layer_bytes = sum(sizes)
        self.head_bytes = V * dev.row_size(ca.Q6_K, H)
        self.total = NL * self.layer_bytes + self.head_bytes
        self.arena = dev.alloc(self.total)
        off, self.first = 0, []
        for (name, t, N, K), sz in zip(self.layer, sizes):
            self.arena.upload(synth_weights(dev, t, N, K, rng), offset=off)
            self.first.append(off)
            off += sz
        for l in range(1, NL):
            dev.check(L.chip_memcpy_d2d(self.arena.ptr + l * self.layer_bytes, self.arena.ptr, self.layer_bytes, None))
        self.head_off = NL * self.layer_bytes
        self.arena.upload(synth_weights(dev, ca.Q6_K, V // 8, H, rng), offset=self.head_off)
        for i in range(1, 8):
            dev.check(L.chip_memcpy_d2d(self.arena.ptr + self.head_off + i * (self.head_bytes // 8), self.arena.ptr + self.head_off,
                                        self.head_bytes // 8, None))
        dev.sync()
        self.st = C.c_void_p()
        dev.check(L.chip_stream_create(C.byref(self.st)))
        self.bufs = {}
        self.head_type = ca.Q6_K

    def q6_K_to(self, planes, head=True):
        """Every Q6_K matrix of the arena to planes (what the backend keeps for its decode GEMVs) or back to block order,
        in place; the launches that follow name the layout by its type."""
        ca, dev, L = self.ca, self.dev, self.dev.lib
        want, have = (ca.Q6_K_PLANES, ca.Q6_K) if planes else (ca.Q6_K, ca.Q6_K_PLANES)
        for l in range(self.NL):
            for nm, (t, p, N, K) in self.weights(l).items():
                if t == have:
                    dev.check(L.chip_repack_q6_K(p, dev.row_size(t, K), p, dev.row_size(t, K), K, N, int(planes), None))
        if self.head_type == have and (head or not planes):
            p = self.arena.ptr + self.head_off
            dev.check(L.chip_repack_q6_K(p, dev.row_size(have, self.H), p, dev.row_size(have, self.H), self.H, self.V, int(planes), None))
        dev.sync()
        self.layer = [(nm, want if t == have else t, N, K) for (nm, t, N, K) in self.layer]
        self.head_type = want if self.head_type == have else self.head_type

    def weights(self, l):
        base = self.arena.ptr + l * self.layer_bytes
        return {name: (t, base + o, N, K) for (name, t, N, K), o in zip(self.layer, self.first)}

    def io(self, n):
        """Activations, outputs and workspace for n tokens (kept for the life of the trace)."""
        if n not in self.bufs:
            dev, L, ca = self.dev, self.dev.lib, self.ca
            rng = np.random.default_rng(11 + n)
            wsz = max([L.chip_mul_mat_workspace_size_n(t, K, N, n) for (_, t, N, K) in self.layer] +
                      [L.chip_mul_mat_workspace_size_n(ca.Q6_K, self.H, self.V, n)])
            self.bufs[n] = {"x_h": dev.to_device(rng.standard_normal((n, self.H)).astype(np.float32)),
                            "x_ff": dev.to_device(rng.standard_normal((n, self.FF)).astype(np.float32)),
                            "y": dev.alloc(4 * n * self.V * 4), "ws": dev.alloc(wsz), "wsz": wsz}
        return self.bufs[n]

    def step_bytes(self, n):
        return self.total + 4 * n * (self.NL * sum(K + N for (_, _, N, K) in self.layer) + self.H + self.V)

    # ---- the launches, per class of op (one entry of OPS = what the backend issues as one call)
    def op_calls(self, n):
        """name -> function(layer index) that issues that op of that layer; 'head' ignores the index."""
        dev, L, ca, st = self.dev, self.dev.lib, self.ca, self.st
        b = self.io(n)
        ws, wsz, y = b["ws"].ptr, b["wsz"], b["y"].ptr
        xh, xff = b["x_h"].ptr, b["x_ff"].ptr
        V, H = self.V, self.H
        nV = n * V * 4
        ck = dev.check

        def qkv(l):                      # three matrices on one activation: one call (one launch up to 4 tokens)
            W = self.weights(l)
            arr = (ca.Mat * 3)()
            for i, nm in enumerate(("wq", "wk", "wv")):
                t, p, N, K = W[nm]
                arr[i] = ca.Mat(t, p, dev.row_size(t, K), N, y + i * nV, N, None, 0)
            ck(L.chip_mul_mat_group(arr, 3, H, xh, H, n, ws, wsz, st))

        def single(nm, x):
            def f(l):
                t, p, N, K = self.weights(l)[nm]
                ck(L.chip_mul_mat(t, p, dev.row_size(t, K), K, N, x, K, n, y, N, ws, wsz, st))
            return f

        def gate_up(l):                  # two matrices of one shape on one activation: one call
            W = self.weights(l)
            (t, pg, N, K), (_, pu, _, _) = W["gate"], W["up"]
            ck(L.chip_mul_mat_pair(t, pg, pu, dev.row_size(t, K), K, N, xh, K, n, y, y + nV, N, ws, wsz, st))

        def head(_l):
            ck(L.chip_mul_mat(self.head_type, self.arena.ptr + self.head_off, dev.row_size(ca.Q6_K, H), H, V, xh, H, n, y, V, ws, wsz, st))

        return {"qkv": qkv, "wo": single("wo", xh), "gate_up": gate_up, "down": single("down", xff), "head": head}

    def op_bytes(self, n):
        """Algorithmic bytes of one call of each op class: its weights once, fp32 activations in, fp32 outputs out."""
        sz = {nm: N * self.dev.row_size(t, K) for (nm, t, N, K) in self.layer}
        H, FF, KV, V = self.H, self.FF, self.KV, self.V
        return {"qkv": sz["wq"] + sz["wk"] + sz["wv"] + 4 * n * (H + H + 2 * KV), "wo": sz["wo"] + 4 * n * 2 * H,
                "gate_up": sz["gate"] + sz["up"] + 4 * n * (H + 2 * FF), "down": sz["down"] + 4 * n * (FF + H),
                "head": self.head_bytes + 4 * n * (H + V)}

    ORDER = ("qkv", "wo", "gate_up", "down")

    def step(self, n):
        calls = self.op_calls(n)

        def run():
            for l in range(self.NL):
                for nm in self.ORDER:
                    calls[nm](l)
            calls["head"](0)
        return run

    def free(self):
        for b in self.bufs.values():
            for k in ("x_h", "x_ff", "y", "ws"):
                b[k].free()
        self.arena.free()


def percentiles(xs):
    xs = np.sort(np.asarray(xs, np.float64))
    return {"median": round(float(np.median(xs)), 2), "p10": round(float(np.percentile(xs, 10)), 2),
            "p90": round(float(np.percentile(xs, 90)), 2)}


def time_steps(dev, hip, st, launch, steps, warmup):
    """W untimed steps, a synchronization, exactly K steps between one pair of events (the figure reported), and an event
    after every step for the spread.  Returns (ms per step, per-step microseconds)."""
    for _ in range(warmup):
        launch()
    dev.sync(st)
    marks = [hip.event() for _ in range(steps + 1)]
    hip.record(marks[0], st)
    for i in range(steps):
        launch()
        hip.record(marks[i + 1], st)
    total_ms = hip.elapsed_ms(marks[0], marks[steps])
    dev.sync(st)
    per = [hip.elapsed_ms(marks[i], marks[i + 1]) * 1e3 for i in range(steps)]
    return total_ms / steps, per


def traffic_from_profile(key):
    """HBM bytes per launch of kernel `key` as the committed counter summary states them, or None."""
    try:
        for line in open(TRAFFIC_PROFILE):
            p = line.split()
            if len(p) >= 3 and p[0] == "traffic_bytes_per_launch:" and p[1] == key:
                return int(p[2])
    except OSError:
        pass
    return None


def bench_headline(dev, hip, trace, steps, warmup, eager):
    """One-token decode step over the trace; then each op class alone (32 back-to-back launches on the 32 layers' distinct
    weights between one event pair) to find the kernel with the largest share and its roofline figure."""
    st = trace.st
    run = trace.step(1)
    run()
    dev.sync(st)
    if eager:
        launch, destroy = run, (lambda: None)
    else:
        launch, destroy = hip.capture(st, run)
    ms_per_step, per = time_steps(dev, hip, st, launch, steps, warmup)
    destroy()
    b = trace.step_bytes(1)
    value = b / (ms_per_step * 1e-3) / 1e9

    calls, ob = trace.op_calls(1), trace.op_bytes(1)
    per_op = {}
    for nm in ("qkv", "wo", "gate_up", "down", "head"):
        reps = 4 if nm == "head" else 3

        def sweep(nm=nm):
            for l in range(1 if nm == "head" else trace.NL):
                calls[nm](l)
        launches = reps * (1 if nm == "head" else trace.NL)
        if eager:
            one, kill = sweep, (lambda: None)
        else:
            one, kill = hip.capture(st, sweep)
        one()
        dev.sync(st)
        e0, e1 = hip.event(), hip.event()
        hip.record(e0, st)
        for _ in range(reps):
            one()
        hip.record(e1, st)
        us = hip.elapsed_ms(e0, e1) * 1e3 / launches
        kill()
        count = 1 if nm == "head" else trace.NL
        per_op[nm] = {"us_per_launch": round(us, 2), "bytes_per_launch": ob[nm], "GBps": round(ob[nm] / us / 1e3, 1),
                      "hbm_frac": round(ob[nm] / us / 1e3 / HBM_PEAK_GBS, 4), "launches_per_step": count,
                      "share_of_step": round(count * us / (ms_per_step * 1e3), 3), "launches_timed": launches}
    dom = max(per_op, key=lambda k: per_op[k]["share_of_step"])
    d = per_op[dom]
    q6 = "Q6_K in planes" if trace.head_type == trace.ca.Q6_K_PLANES else "Q6_K"
    kernel_names = {"qkv": "gemv_group_kernel<K-quants, n=1> (wq Q4_K 4096x4096 + wk Q4_K 1024x4096 + wv %s 1024x4096)" % q6,
                    "wo": "gemv_kernel<Q4_K, n=1, fused quantize> (4096x4096)",
                    "gate_up": "gemv_kernel<Q4_K, n=1, fused quantize> over ffn_gate + ffn_up (2 x 14336x4096, one launch)",
                    "down": "gemv_kernel<%s, n=1, fused quantize, image built a step's part at a time> (4096x14336)" % q6,
                    "head": "gemv_kernel<%s, n=1, fused quantize> (128256x4096)" % q6}
    roof = {"bound": "hbm", "achieved": d["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": d["hbm_frac"],
            "traffic": traffic_from_profile(dom), "kernel": kernel_names[dom], "op": dom,
            "bytes_per_launch": d["bytes_per_launch"], "us_per_launch": d["us_per_launch"],
            "launches_timed": d["launches_timed"], "share_of_step": d["share_of_step"]}
    info = {"step_us": percentiles(per), "tokens_per_s": round(1e3 / ms_per_step, 1), "launches_per_step": 4 * trace.NL + 1,
            "matmuls_per_step": 7 * trace.NL + 1, "replay": "eager launches" if eager else "HIP graph",
            "per_op": per_op}
    return value, ms_per_step, b, roof, info


def bench_whole_layers(dev, hip, trace, n, n_kv, fold=True):
    """Every node of the 32 layers as llama.cpp builds them without flash attention (norms, projections, RoPE, cache
    stores, kq, soft-max, kqv, head merge, residuals, SiLU * up), n new tokens against n_kv cached positions, as one
    HIP graph on one stream: what a decode step costs when no activation leaves the device."""
    ca, L, st = trace.ca, dev.lib, trace.st
    H, FF, KV, V, NL = trace.H, trace.FF, trace.KV, trace.V, trace.NL
    hd, n_head, n_head_kv, kv_size = 128, 32, 8, 4096
    rng = np.random.default_rng(17)
    A4 = C.c_int64 * 4
    f32 = lambda *shape: dev.alloc(int(np.prod(shape)) * 4)
    b = trace.io(n)
    ws, wsz, y = b["ws"], b["wsz"], b["y"]
    resid = dev.to_device(rng.standard_normal((n, H)).astype(np.float32))
    wn = dev.to_device((1 + 0.1 * rng.standard_normal(H)).astype(np.float32))
    pos = dev.to_device(np.arange(n_kv - n, n_kv, dtype=np.int32))
    mask = dev.to_device(np.zeros((max(n, 8), n_kv), np.float16))
    cur, q, k, v, merged, att = f32(n, H), f32(n, H), f32(n, KV), f32(n, KV), f32(n, H), f32(n, H)
    kq, kqv = f32(n_head, n, n_kv), f32(n_head, n, hd)
    up, gate = f32(n, FF), f32(n, FF)
    caches = dev.alloc(NL * 2 * kv_size * KV * 2)
    dev.check(L.chip_memset(caches.ptr, 0, caches.nbytes, None))
    aws_bytes = max(L.chip_mul_mat_f16_batched_workspace_size(hd, n_kv, n_head_kv, n_head, n),
                    L.chip_mul_mat_f16_batched_workspace_size(n_kv, hd, n_head_kv, n_head, n), 256)
    aws = dev.alloc(aws_bytes)
    rope_tab = dev.alloc(n * hd * 4)
    ck = dev.check
    # up to 4 tokens the norms run in the prologue of the projections that read them and the residual ADDs in the store of
    # the projections in front of them, where the library has those forms for the model's types
    Wl = trace.weights(0)
    deferred = (fold and n <= 2 and all(L.chip_norm_before_supported(Wl[nm][0], H, n) == 1 for nm in ("wq", "wk", "wv", "gate")) and
                L.chip_mul_mat_pair_silu_mul_supported(Wl["gate"][0], H, FF, n) == 1 and
                L.chip_mul_mat_add_supported(Wl["wo"][0], H, H, n) == 1 and L.chip_mul_mat_add_supported(Wl["down"][0], FF, H, n) == 1)
    nb = ca.NormBefore(wn.ptr, 1e-5, cur.ptr, H)

    def mm(t, wptr, N, K, src, dst, shared=False):
        """shared: src was quantized by the previous matmul (same tensor, same activation type), as the backend reuses it"""
        if n <= 4:                                                    # the GEMV quantizes in its prologue
            ck(L.chip_mul_mat(t, wptr, dev.row_size(t, K), K, N, src.ptr, K, n, dst.ptr, N, ws.ptr, wsz, st))
            return
        if not shared:
            ck(L.chip_mul_mat_prepare(t, K, src.ptr, K, n, ws.ptr, wsz, st))
        ck(L.chip_mul_mat_run_ws(t, wptr, dev.row_size(t, K), K, N, n, ws.ptr, wsz, dst.ptr, N, st))

    def step():
        for l in range(NL):
            W = trace.weights(l)
            kc = caches.ptr + (2 * l) * kv_size * KV * 2
            vc = kc + kv_size * KV * 2
            if l == 0 and not deferred:
                ck(L.chip_rms_norm_mul(resid.ptr, H, n, H, 1e-5, wn.ptr, None, 0, cur.ptr, H, st))  # norm + weight: one kernel, as the backend fuses them
            # q, k, v projections on one activation: one call; V's also stores into the transposed F16 cache
            arr = (ca.Mat * 3)()
            for i, (nm, dst) in enumerate((("wq", q), ("wk", k), ("wv", v))):
                t_, p_, N_, K_ = W[nm]
                arr[i] = ca.Mat(t_, p_, dev.row_size(t_, K_), N_, dst.ptr, N_, None, 0)
            if l == 0:                                                # one cos / sin table per step, as the backend keeps it
                ck(L.chip_rope_table(pos.ptr, None, n, hd, 8192, 500000.0, 1.0, 0.0, 1.0, 32.0, 1.0, rope_tab.ptr, st))
            if n <= 4:
                # up to 4 tokens also the RoPE of Q and of K in the projections' epilogue, K's result going to the F16 cache only
                # (its F32 form has no other reader), as the backend runs the six nodes
                arr[2].y_f16_t = vc + 2 * (n_kv - n)
                arr[2].ld16 = kv_size
                rp = (ca.RopeAfter * 3)()
                rp[0] = ca.RopeAfter(rope_tab.ptr, hd, hd, 2, q.ptr, hd * n_head, None, 0)
                rp[1] = ca.RopeAfter(rope_tab.ptr, hd, hd, 2, None, 0, kc + 2 * KV * (n_kv - n), KV)
                if deferred:                                          # attn_norm and its weight MUL in the same launch's prologue
                    ck(L.chip_mul_mat_group_rope_norm(arr, rp, C.byref(nb), 3, H, resid.ptr, H, n, ws.ptr, wsz, st))
                else:
                    ck(L.chip_mul_mat_group_rope(arr, rp, 3, H, cur.ptr, H, n, ws.ptr, wsz, st))
            else:
                ck(L.chip_mul_mat_group(arr, 3, H, cur.ptr, H, n, ws.ptr, wsz, st))
                # RoPE of Q and of K in one launch; K's also stores into the F16 cache
                ra = ca.RopeOperand(q.ptr, hd, hd * n_head, n_head, q.ptr, hd, hd * n_head, None, 0, 0)
                rb = ca.RopeOperand(k.ptr, hd, KV, n_head_kv, k.ptr, hd, KV, kc + 2 * KV * (n_kv - n), hd, KV)
                ck(L.chip_rope_apply_two(C.byref(ra), C.byref(rb), rope_tab.ptr, hd, n, hd, 2, st))
            if n > 4:
                shp = A4(n, KV, 1, 1)
                ck(L.chip_cpy(v.ptr, ca.F32, shp, A4(KV * 4, 4, 0, 0), vc + 2 * (n_kv - n), ca.F16, shp, A4(2, kv_size * 2, 0, 0), st))
            ck(L.chip_mul_mat_f16_batched(kc, 2 * KV, 2 * hd, hd, n_kv, n_head_kv, q.ptr, hd * n_head, hd, n, n_head, kq.ptr, n_kv,
                                          n_kv * n, aws.ptr, aws_bytes, st))
            ck(L.chip_soft_max(kq.ptr, n_kv, mask.ptr, ca.F16, n_kv, n, n_head * n, 0.0884, 0.0, kq.ptr, n_kv, st))
            if L.chip_mul_mat_f16_batched_second_copy_supported(n_head_kv, n_head, n) == 1:
                # kqv and the head merge that follows it in one launch, as the backend runs the two nodes of a decode step
                ck(L.chip_mul_mat_f16_batched_two_copies(vc, 2 * kv_size, 2 * kv_size * hd, n_kv, hd, n_head_kv, kq.ptr, n_kv, n_kv * n, n,
                                                         n_head, kqv.ptr, hd, hd * n, merged.ptr, H, hd, aws.ptr, aws_bytes, st))
            else:
                ck(L.chip_mul_mat_f16_batched(vc, 2 * kv_size, 2 * kv_size * hd, n_kv, hd, n_head_kv, kq.ptr, n_kv, n_kv * n, n, n_head,
                                              kqv.ptr, hd, hd * n, aws.ptr, aws_bytes, st))
                ck(L.chip_cpy(kqv.ptr, ca.F32, A4(hd, n_head, n, 1), A4(4, 4 * hd * n, 4 * hd, 0), merged.ptr, ca.F32, A4(H, n, 1, 1),
                              A4(4, 4 * H, 4 * H * n, 4 * H * n), st))
            (t_, wg, N_, K_), (_, wu, _, _) = W["gate"], W["up"]
            td, wd, Nd, Kd = W["down"]
            if deferred:
                # wo with the residual ADD in its store; ffn_norm and its weight MUL in the gated pair's prologue; ffn_down with
                # the second residual ADD in its store: four launches for the eleven nodes, as the backend runs them
                to_, wo_, No_, Ko_ = W["wo"]
                ck(L.chip_mul_mat_add(to_, wo_, dev.row_size(to_, Ko_), Ko_, No_, merged.ptr, Ko_, n, resid.ptr, H, resid.ptr, H, ws.ptr, wsz, st))
                ck(L.chip_mul_mat_pair_silu_mul_norm(t_, wg, wu, dev.row_size(t_, K_), K_, N_, resid.ptr, K_, n, C.byref(nb), gate.ptr, N_,
                                                     ws.ptr, wsz, st))
                ck(L.chip_mul_mat_add(td, wd, dev.row_size(td, Kd), Kd, Nd, gate.ptr, Kd, n, resid.ptr, H, resid.ptr, H, ws.ptr, wsz, st))
                continue
            mm(*W["wo"], merged, att)
            # residual + norm + weight: one kernel, as the backend fuses the three nodes
            ck(L.chip_add_rms_norm_mul(att.ptr, H, resid.ptr, H, resid.ptr, H, n, H, 1e-5, wn.ptr, cur.ptr, H, st))
            if n <= 4 and L.chip_mul_mat_pair_silu_mul_supported(t_, K_, N_, n) == 1:
                # gate, SILU, up and their MUL in one launch; ffn_down quantizes its input itself, as the backend runs the five nodes
                ck(L.chip_mul_mat_pair_silu_mul(t_, wg, wu, dev.row_size(t_, K_), K_, N_, cur.ptr, K_, n, gate.ptr, N_, ws.ptr, wsz, st))
                ck(L.chip_mul_mat(td, wd, dev.row_size(td, Kd), Kd, Nd, gate.ptr, Kd, n, att.ptr, Nd, ws.ptr, wsz, st))
            else:
                ck(L.chip_mul_mat_pair(t_, wg, wu, dev.row_size(t_, K_), K_, N_, cur.ptr, K_, n, gate.ptr, up.ptr, N_, ws.ptr, wsz, st))
                # SiLU in its MUL's kernel, which also leaves ffn_down's quantized rows in the workspace, as the backend runs the three nodes
                ck(L.chip_silu_mul_quantized(gate.ptr, FF, up.ptr, FF, n, FF, gate.ptr, FF, td, ws.ptr, wsz, st))
                ck(L.chip_mul_mat_run_ws(td, wd, dev.row_size(td, Kd), Kd, Nd, n, ws.ptr, wsz, att.ptr, Nd, st))
            # the layer's second residual with the next layer's (or the final) norm
            ck(L.chip_add_rms_norm_mul(att.ptr, H, resid.ptr, H, resid.ptr, H, n, H, 1e-5, wn.ptr, cur.ptr, H, st))
        if deferred:                                                  # the final norm has no projection of this kind behind it
            ck(L.chip_rms_norm_mul(resid.ptr, H, n, H, 1e-5, wn.ptr, None, 0, cur.ptr, H, st))
        ck(L.chip_mul_mat(trace.head_type, trace.arena.ptr + trace.head_off, dev.row_size(ca.Q6_K, H), H, V, cur.ptr, H, n, y.ptr, V, ws.ptr, wsz, st))

    step()
    dev.sync(st)
    launch, destroy = hip.capture(st, step)
    ms, per = time_steps(dev, hip, st, launch, 10, 2)
    destroy()
    for bf in (resid, wn, pos, mask, cur, q, k, v, merged, att, kq, kqv, up, gate, caches, aws, rope_tab):
        bf.free()
    cache_bytes = NL * 2 * n_kv * KV * 2
    return {"n_kv": n_kv, "us_per_step": round(ms * 1e3, 1), "step_us": percentiles(per), "tokens_per_s": round(n / (ms * 1e-3), 1),
            "weight_and_cache_GBps": round((trace.total + cache_bytes) / ms / 1e6, 1)}


def bench_trace_more(dev, hip, trace, eager, planes=True):
    """The same trace at 8 tokens (per step: 225 matmuls; shared quantized activations) and as one 512-token prefill chunk,
    both on block-order Q6_K rows (the backend reads its copy in planes up to 4 tokens only)."""
    st = trace.st
    out = {}
    trace.q6_K_to(False)
    for n in (8, 512):
        run = trace.step(n)
        run()
        dev.sync(st)
        if eager:
            launch, destroy = run, (lambda: None)
        else:
            launch, destroy = hip.capture(st, run)
        ms, per = time_steps(dev, hip, st, launch, 10, 2)
        destroy()
        b = trace.step_bytes(n)
        e = {"us_per_step": round(ms * 1e3, 1), "step_us": percentiles(per), "tokens_per_s": round(n / (ms * 1e-3), 1),
             "GBps": round(b / ms / 1e6, 1), "hbm_frac": round(b / ms / 1e6 / HBM_PEAK_GBS, 4)}
        if n > 8:
            ops = 2.0 * n * (trace.NL * sum(N * K for (_, _, N, K) in trace.layer) + trace.V * trace.H)
            e["TOPS"] = round(ops / ms / 1e9, 1)
            e["int8_frac"] = round(ops / ms / 1e9 / INT8_PEAK_TOPS, 4)
        if not eager:
            e["whole_layers"] = bench_whole_layers(dev, hip, trace, n, 512 if n == 512 else 4096)
        out["config5_trace_n%d" % n] = e
    if not eager:
        trace.q6_K_to(planes)
        out["config5_trace_n1_whole_layers"] = bench_whole_layers(dev, hip, trace, 1, 4096)
    return out


def backend_graph_timing():
    """The same model as a ggml graph through the reference's scheduler and libggml-hip.so (every node on the device):
    bench_backend_graph.py in a child process - the host framework there is the reference's own ggml build (oracle/_ref),
    which is there as the host of the backend, not as something measured.  Returns its figures, or the reason there are none."""
    import re
    import subprocess
    script = os.path.join(ROOT, "bench_backend_graph.py")
    ref_so = os.path.join(ROOT, "oracle", "_ref", "libggml_ref.so")
    if not os.path.exists(ref_so):
        return {"skipped": "no host framework on this machine (oracle/_ref/libggml_ref.so)"}
    res = {}
    for n in (1, 8):
        try:
            txt = subprocess.run([sys.executable, "-u", script], env=dict(os.environ, NTOK=str(n)), capture_output=True, text=True,
                                 timeout=240).stdout
        except Exception as exc:                                            # noqa: BLE001
            res["n%d" % n] = {"error": repr(exc)[:200]}
            continue
        m = re.search(r"graph_compute wall us: min (\d+) median (\d+) max (\d+)", txt)
        i = re.search(r"host time to issue one graph us: median (\d+)", txt)
        g = re.search(r"nodes (\d+)", txt)
        if m:
            res["n%d" % n] = {"graph_compute_us_median": int(m.group(2)), "min": int(m.group(1)), "max": int(m.group(3)),
                              "host_issue_us": int(i.group(1)) if i else None, "graph_nodes": int(g.group(1)) if g else None,
                              "tokens_per_s": round(n / (int(m.group(2)) * 1e-6), 1)}
        else:
            res["n%d" % n] = {"error": txt[-300:]}
    res["what"] = ("Llama-3-8B-shaped graph (attention over 4096 cached positions + gated FFN, Q4_K_M type mix) run by the "
                   "reference scheduler on the HIP backend, eager launches, wall time of graph_compute")
    return res


def cpu_model():
    """The first processor entry of /proc/cpuinfo: model string, family / model / stepping, and the SIMD flags that decide
    which ggml-cpu kernels a native build would take (the reference build here is pinned to AVX2)."""
    info = {}
    try:
        for line in open("/proc/cpuinfo"):
            if ":" not in line:
                if info:
                    break
                continue
            k, v = (p.strip() for p in line.split(":", 1))
            if k in ("vendor_id", "cpu family", "model", "model name", "stepping", "cpu cores", "siblings"):
                info[k] = v
            elif k == "flags":
                fl = set(v.split())
                info["simd"] = " ".join(f for f in ("avx2", "fma", "f16c", "avx512f", "avx512bw", "avx512vl", "avx512_vnni", "avx_vnni", "amx_int8") if f in fl)
    except OSError:
        pass
    if not info:
        return "unknown"
    return "%s (%s family %s model %s stepping %s; %s cores / %s threads per package; %s)" % (
        info.get("model name", "?"), info.get("vendor_id", "?"), info.get("cpu family", "?"), info.get("model", "?"),
        info.get("stepping", "?"), info.get("cpu cores", "?"), info.get("siblings", "?"), info.get("simd", ""))


def cpu_topology():
    """Logical CPUs online, those this process may run on, and the distinct physical cores among them."""
    try:
        allowed = sorted(os.sched_getaffinity(0))
    except AttributeError:
        allowed = list(range(os.cpu_count() or 1))
    cores = set()
    for c in allowed:
        try:
            pkg = open("/sys/devices/system/cpu/cpu%d/topology/physical_package_id" % c).read().strip()
            core = open("/sys/devices/system/cpu/cpu%d/topology/core_id" % c).read().strip()
            cores.add((pkg, core))
        except OSError:
            cores.add(("?", c))
    return {"logical_cpus_online": os.cpu_count(), "logical_cpus_allowed": len(allowed), "physical_cores_allowed": len(cores),
            "threads_used_cap": 16}


def physical_cores():
    """Distinct (package, core) pairs of the CPUs this process may run on, capped at the box's CPU share for one GPU."""
    try:
        allowed = sorted(os.sched_getaffinity(0))
    except AttributeError:
        allowed = list(range(os.cpu_count() or 1))
    seen = set()
    for c in allowed:
        try:
            pkg = open("/sys/devices/system/cpu/cpu%d/topology/physical_package_id" % c).read().strip()
            core = open("/sys/devices/system/cpu/cpu%d/topology/core_id" % c).read().strip()
            seen.add((pkg, core))
        except OSError:
            seen.add(("?", c))
    return max(1, min(len(seen), 16))


def cpu_baseline():
    """Reference ggml-cpu MUL_MAT (oracle/_ref) or the oracle port on the host cores, bounded sample of the headline
    workload: the seven weight matmuls of one layer of the trace at one token, each as its own one-node graph with a
    persistent threadpool, at T = 1 and at T = the physical cores this process may use."""
    import oracle as O
    rng = np.random.default_rng(2)
    use_ref = O.Reference.available()
    eng = O.Reference() if use_ref else O.Oracle()
    H, FF, KV = 4096, 14336, 1024
    layer = [(O.Q4_K, H, H), (O.Q4_K, KV, H), (O.Q6_K, KV, H), (O.Q4_K, H, H), (O.Q4_K, FF, H), (O.Q4_K, FF, H), (O.Q6_K, H, FF)]
    d = np.array([0.0107], np.float16).view(np.uint8)
    mats = []
    for (t, N, K) in layer:
        bb = O.BLOCK_BYTES[t]
        w = rng.integers(0, 256, (N, K // 256, bb), dtype=np.uint8)
        if t == O.Q6_K:
            w[..., 208:210] = d
        else:
            w[..., 0:2] = d
            w[..., 2:4] = d
        mats.append((t, w.reshape(N, -1), rng.standard_normal((1, K)).astype(np.float32)))
    nbytes = sum(w.size + 4 * (w.shape[0] + x.shape[1]) for (_, w, x) in mats)
    T = physical_cores()
    legs, t_start = {}, time.perf_counter()
    for threads in (T, 1):
        total = 0.0
        for (t, w, x) in mats:
            if use_ref:
                _, times = eng.mul_mat_graph(t, w, x, nthreads=threads, repeat=8 if threads > 1 else 4)
                total += float(np.median(times[1:]))
            else:
                t0 = time.perf_counter()
                eng.mul_mat(t, w, x, nthreads=threads)
                total += time.perf_counter() - t0
        legs["T%d" % threads] = {"threads": threads, "ms_per_layer": round(total * 1e3, 3), "GBps": round(nbytes / total / 1e9, 2)}
        if time.perf_counter() - t_start > 60:
            break
    main_leg = legs["T%d" % T]
    return {"value": main_leg["GBps"], "unit": "GB/s", "cores": T, "kind": "reference" if use_ref else "port",
            "cpu_model": cpu_model(), "cpu_topology": cpu_topology(), "legs": legs,
            "build": "gcc -O2 -mavx2 -mfma -mf16c -ffp-contract=off (AVX2 kernels of ggml-cpu-quants.c; no -march=native)" if use_ref
                     else "gcc -O2 scalar restatement",
            "sample": "one layer of the headline trace at one token (wq, wk, wv, wo, ffn_up, ffn_gate, ffn_down: 7 matmuls, "
                      "%d bytes), %s, persistent threadpool, median of the calls after the first; random block bytes with a "
                      "constant scale (timing is data independent)" % (nbytes, "reference ggml-cpu MUL_MAT graphs" if use_ref
                                                                        else "oracle restatement")}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (every figure is single-GPU)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    import cactus_amd as ca
    dev = ca.Device(0)
    hip = Hip()
    trace = Trace(dev, hip, np.random.default_rng(5))
    # Q6_K weights as the backend keeps them for matmuls of up to 4 tokens: rows in planes (made once, outside the timed region)
    planes = not args.block_order
    if args.only_trace:
        trace.q6_K_to(planes and args.only_trace <= 4)
        run = trace.step(args.only_trace)
        ms, per = time_steps(dev, hip, trace.st, run, args.steps, args.warmup)
        print(json.dumps({"only_trace": args.only_trace, "launches": "eager", "steps": args.steps, "warmup": args.warmup,
                          "us_per_step": round(ms * 1e3, 1), "step_us": percentiles(per)}))
        trace.free()
        return
    extra = {}
    if planes and not args.no_extra:                                   # the same step on block_q6_K rows as the file stores them
        _, ms_blocks, _, _, info_blocks = bench_headline(dev, hip, trace, min(args.steps, 10), min(args.warmup, 2), args.eager)
        extra["q6_K_in_block_order"] = {"ms_per_step": round(ms_blocks, 4),
                                        "us_per_launch": {k: v["us_per_launch"] for k, v in info_blocks["per_op"].items()}}
    trace.q6_K_to(planes)
    value, ms_per_step, step_bytes, roof, info = bench_headline(dev, hip, trace, args.steps, args.warmup, args.eager)
    info["q6_K_layout"] = ("planes: chip_repack_q6_K at set-up, what the backend keeps for matmuls of up to 4 tokens" if planes
                           else "block_q6_K as stored in the file")
    if not args.no_extra:
        extra.update(bench_trace_more(dev, hip, trace, args.eager, planes))
    trace.free()
    if not args.no_extra:
        extra["config2_q8_0_ffn_gemv"] = bench_config2(dev, hip)
        extra.update(bench_extra(dev, hip))
        extra["mfma_i8_measured_peak"] = measured_mfma_peak()
        extra["read_only_floor"] = measured_read_floor()
        if not args.no_backend and not args.eager:
            extra["backend_graph"] = backend_graph_timing()
    cpu = None if args.no_cpu else cpu_baseline()
    line = {
        "metric": "quant mul_mat GEMV HBM GB/s & prefill int8 TOPS (% of roofline), 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic: random-init weights written directly as GGUF blocks (uniformly random quant and sub-scale bytes, "
                "one constant fp16 block scale), fp32 activations ~N(0,1); kernel timing does not depend on the values",
        "config": {"workload": "BASELINE configs[4]: decode-step MUL_MAT trace of a Llama-3-8B-shaped Q4_K_M model (32 layers, "
                               "hidden 4096, FFN 14336, 32 q / 8 kv heads of 128, Q6_K output head 128256x4096; attn_v and "
                               "ffn_down Q6_K, the rest Q4_K), every weight matmul of one token step at batch 1, serial on one "
                               "stream; step = 225 matmuls in 129 calls (wq+wk+wv one call, ffn_gate+ffn_up one call)",
                   "bytes_per_step": step_bytes, "device": dev.info.arch.decode(), **info},
        "roofline": roof, "cpu_baseline": cpu, "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
