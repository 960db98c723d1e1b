#!/usr/bin/env python3
"""Benchmark of the quantized MUL_MAT hot path on one MI355X.

Headline workload (BASELINE.json configs[1]): Q8_0 x Q8_0 decode GEMV at Llama FFN shapes, W[11008 x 4096]
and W[4096 x 11008], token batch n in {1, 2, 4, 8}.  One "step" = the eight ops (2 shapes x 4 batch sizes),
each op being what LM_GGML_OP_MUL_MAT does: quantize the fp32 activations to Q8_0 on the GPU, then the GEMV.
Inputs are resident in HBM before the timed region; weights rotate through > 512 MB of distinct copies per
shape so that the 256 MB Infinity Cache cannot serve them (cold numbers).

Prints ONE JSON line.  `value` = algorithmic bytes of a step / wall time of a step (HIP events on the launch
stream).  `roofline` is for the dominant kernel, the n = 1 GEMV, timed with its own HIP event pairs inside the
timed region.  `cpu_baseline` times the reference's own ggml-cpu MUL_MAT (oracle/_ref, when it travelled) or the
oracle port on the host cores for a bounded sample of the same workload.  `extra` carries the other BASELINE
configurations (Q4_0 mat-vec, Q4_K GEMV, prefill GEMM TOPS, Llama-3-8B-shaped decode trace).
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
# HBM bytes per launch of the n = 1 Q8_0 GEMV from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by what the same
# counters read for a device-to-device copy of known size (profiles/gemv_q8_0_n1_hbm_traffic_pmc.md): mean of the
# two headline shapes.  Algorithmic bytes per launch: 47 967 232.
N1_GEMV_HBM_TRAFFIC_BYTES = 48350573


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-trace", action="store_true",
                    help="skip the model-shaped HIP-graph trace and the issue-rate probe (for runs under a profiler)")
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
        L.hipDeviceSynchronize.argtypes = []

    def event(self):
        e = C.c_void_p()
        assert self.lib.hipEventCreate(C.byref(e)) == 0
        return e

    def record(self, e, stream):
        assert self.lib.hipEventRecord(e, stream) == 0

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


def bench_headline(dev, hip, steps, warmup):
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
    roof = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": N1_GEMV_HBM_TRAFFIC_BYTES,
            "kernel": "gemv_kernel<Q8_0, n=1, fused activation quantize> (W[11008x4096] and W[4096x11008], cold weights)",
            "bytes_per_launch": k_bytes, "us_per_launch": round(k_us, 2), "launches_timed": 2 * reps}
    return value, ms_per_step, step_bytes, roof, {"copies_per_shape": [m.copies for m in mats]}


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


def bench_extra(dev, hip, trace=True):
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

    # weight upload: one synchronous copy from pageable memory (what set_tensor does) against the loader's protocol of
    # four pinned 1 MB staging buffers with an event each (chunked set_tensor_async)
    def upload_case():
        total, chunk, nbuf = 256 << 20, 1 << 20, 4
        src = rng.integers(0, 256, total, dtype=np.uint8)
        dst = dev.alloc(total)
        t0 = time.perf_counter()
        dev.check(L.chip_memcpy_h2d(dst.ptr, src.ctypes.data, total, None))
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
        out["upload_256MB"] = {"sync_pageable_GBps": round(total / t_sync / 1e9, 2),
                               "async_pinned_chunks_GBps": round(total / t_async / 1e9, 2), "verified": ok}

    upload_case()

    if trace:
        out.update(bench_trace(dev, hip, st, rng))
        out["mfma_i8_measured_peak"] = measured_mfma_peak()
    return out


def measured_mfma_peak():
    """Runs the issue-rate probe (a child process) and returns the best device-wide rate it saw for the MFMA
    form the GEMM uses, so TOPS can be read against the measured matrix peak as well as the datasheet one."""
    import re
    import subprocess
    exe = os.path.join(ROOT, "cactus_amd", "lib", "probe_issue_rates")
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


def bench_trace(dev, hip, st, rng):
    """config 5: every weight matmul of one decode step of a Llama-3-8B-shaped Q4_K_M model (32 layers, 225
    matmuls; attn_v / ffn_down / output head in Q6_K, the rest Q4_K), replayed as a HIP graph, once as a serial
    chain and once with the independent matmuls of a layer as concurrent graph branches; and the same matmuls for
    one 512-token prefill chunk (serial only)."""
    import cactus_amd as ca
    L = dev.lib
    H, FF, KV, V, NL = 4096, 14336, 1024, 128256, 32
    layer = [("wq", ca.Q4_K, H, H, "attn"), ("wk", ca.Q4_K, KV, H, "attn"), ("wv", ca.Q6_K, KV, H, "attn"),
             ("wo", ca.Q4_K, H, H, "wo"), ("up", ca.Q4_K, FF, H, "ffn"), ("gate", ca.Q4_K, FF, H, "ffn"),
             ("down", ca.Q6_K, H, FF, "down")]
    sizes = [N * dev.row_size(t, K) for (_, t, N, K, _) in layer]
    layer_bytes = sum(sizes)
    head_bytes = V * dev.row_size(ca.Q6_K, H)
    total = NL * layer_bytes + head_bytes
    arena = dev.alloc(total)
    off = 0
    first = []
    for (name, t, N, K, _), sz in zip(layer, sizes):
        arena.upload(synth_weights(dev, t, N, K, rng), offset=off)
        first.append(off)
        off += sz
    for l in range(1, NL):
        dev.check(L.chip_memcpy_d2d(arena.ptr + l * layer_bytes, arena.ptr, layer_bytes, None))
    head_off = NL * layer_bytes
    part = V // 8
    arena.upload(synth_weights(dev, ca.Q6_K, part, H, rng), offset=head_off)
    for i in range(1, 8):
        dev.check(L.chip_memcpy_d2d(arena.ptr + head_off + i * (head_bytes // 8), arena.ptr + head_off, head_bytes // 8, None))
    dev.sync()

    hl = hip.lib
    hl.hipStreamWaitEvent.argtypes = [C.c_void_p, C.c_void_p, C.c_uint]
    side = [C.c_void_p(), C.c_void_p()]
    for s_ in side:
        dev.check(L.chip_stream_create(C.byref(s_)))

    def full_layers(n, n_kv, ws, wsz):
        """Every node of the 32 layers as llama.cpp builds them without flash attention (norms, projections, RoPE, cache
        stores, kq, soft-max, kqv, head merge, residuals, SiLU * up), n new tokens against n_kv cached positions, as one
        HIP graph on one stream: what a decode step costs when no activation leaves the device."""
        hd, n_head, n_head_kv, kv_size = 128, 32, 8, 4096
        A4 = C.c_int64 * 4
        f32 = lambda *shape: dev.alloc(int(np.prod(shape)) * 4)
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
                base = arena.ptr + l * layer_bytes
                W = {name: (t, base + o, N, K) for (name, t, N, K, _), o in zip(layer, first)}
                kc = caches.ptr + (2 * l) * kv_size * KV * 2
                vc = kc + kv_size * KV * 2
                if l == 0:
                    ck(L.chip_rms_norm_mul(resid.ptr, H, n, H, 1e-5, wn.ptr, None, 0, cur.ptr, H, st))  # norm + weight: one kernel, as the backend fuses them
                mm(*W["wq"], cur, q); mm(*W["wk"], cur, k, True)
                if n <= 4:                                                # V projection and its transposed store in one launch
                    t_, wv_, N_, K_ = W["wv"]
                    ck(L.chip_mul_mat_store_t(t_, wv_, dev.row_size(t_, K_), K_, N_, cur.ptr, K_, n, v.ptr, N_, vc + 2 * (n_kv - n), kv_size,
                                              ws.ptr, wsz, st))
                else:
                    mm(*W["wv"], cur, v, True)
                if l == 0:                                                # one cos / sin table per step, as the backend keeps it
                    ck(L.chip_rope_table(pos.ptr, None, n, hd, 8192, 500000.0, 1.0, 0.0, 1.0, 32.0, 1.0, rope_tab.ptr, st))
                ck(L.chip_rope_apply(q.ptr, hd, hd * n_head, rope_tab.ptr, hd, n_head, n, hd, 2, q.ptr, hd, hd * n_head, st))
                # K: RoPE and the store into the F16 cache in one launch, as the backend runs the two nodes
                ck(L.chip_rope_apply_store(k.ptr, hd, KV, rope_tab.ptr, hd, n_head_kv, n, hd, 2, k.ptr, hd, KV,
                                           kc + 2 * KV * (n_kv - n), hd, KV, st))
                if n > 4:
                    shp = A4(n, KV, 1, 1)
                    ck(L.chip_cpy(v.ptr, ca.F32, shp, A4(KV * 4, 4, 0, 0), vc + 2 * (n_kv - n), ca.F16, shp, A4(2, kv_size * 2, 0, 0), st))
                ck(L.chip_mul_mat_f16_batched(kc, 2 * KV, 2 * hd, hd, n_kv, n_head_kv, q.ptr, hd * n_head, hd, n, n_head, kq.ptr, n_kv,
                                              n_kv * n, aws.ptr, aws_bytes, st))
                ck(L.chip_soft_max(kq.ptr, n_kv, mask.ptr, ca.F16, n_kv, n, n_head * n, 0.0884, 0.0, kq.ptr, n_kv, st))
                ck(L.chip_mul_mat_f16_batched(vc, 2 * kv_size, 2 * kv_size * hd, n_kv, hd, n_head_kv, kq.ptr, n_kv, n_kv * n, n, n_head,
                                              kqv.ptr, hd, hd * n, aws.ptr, aws_bytes, st))
                ck(L.chip_cpy(kqv.ptr, ca.F32, A4(hd, n_head, n, 1), A4(4, 4 * hd * n, 4 * hd, 0), merged.ptr, ca.F32, A4(H, n, 1, 1),
                              A4(4, 4 * H, 4 * H * n, 4 * H * n), st))
                mm(*W["wo"], merged, att)
                # residual + norm + weight: one kernel, as the backend fuses the three nodes
                ck(L.chip_add_rms_norm_mul(att.ptr, H, resid.ptr, H, resid.ptr, H, n, H, 1e-5, wn.ptr, cur.ptr, H, st))
                if n <= 4:                                                # gate and up in one launch, as the backend pairs them
                    (t_, wg, N_, K_), (_, wu, _, _) = W["gate"], W["up"]
                    ck(L.chip_mul_mat_pair(t_, wg, wu, dev.row_size(t_, K_), K_, N_, cur.ptr, K_, n, gate.ptr, up.ptr, N_, ws.ptr, wsz, st))
                else:
                    mm(*W["up"], cur, up); mm(*W["gate"], cur, gate, True)
                ck(L.chip_silu_mul(gate.ptr, FF, up.ptr, FF, n, FF, gate.ptr, FF, st))                 # SiLU in its MUL's kernel, as the backend runs the pair
                mm(*W["down"], gate, att)
                # the layer's second residual with the next layer's (or the final) norm
                ck(L.chip_add_rms_norm_mul(att.ptr, H, resid.ptr, H, resid.ptr, H, n, H, 1e-5, wn.ptr, cur.ptr, H, st))
            ck(L.chip_mul_mat(ca.Q6_K, arena.ptr + head_off, dev.row_size(ca.Q6_K, H), H, V, cur.ptr, H, n, y.ptr, V, ws.ptr, wsz, st))

        step()
        dev.sync(st)
        graph, gexec = C.c_void_p(), C.c_void_p()
        assert hl.hipStreamBeginCapture(st, 0) == 0
        step()
        assert hl.hipStreamEndCapture(st, C.byref(graph)) == 0
        assert hl.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        us = time_runs(dev, hip, st, lambda: hl.hipGraphLaunch(gexec, st), 10, warm=2)
        for bf in (resid, wn, pos, mask, cur, q, k, v, merged, att, kq, kqv, up, gate, caches, aws, rope_tab):
            bf.free()
        cache_bytes = NL * 2 * n_kv * KV * 2
        return {"n_kv": n_kv, "nodes": 24 * NL + 2, "us_per_step": round(us, 1), "tokens_per_s": round(n / (us * 1e-6), 1),
                "weight_and_cache_GBps": round((total + cache_bytes) / us / 1e3, 1)}

    res = {}
    for n in (1, 8, 512):                                              # decode, small batch, one prefill chunk
        x_h = dev.to_device(rng.standard_normal((n, H)).astype(np.float32))
        x_ff = dev.to_device(rng.standard_normal((n, FF)).astype(np.float32))
        y = dev.alloc(3 * n * V * 4)                                   # one output region per concurrent branch
        wsz = max([L.chip_mul_mat_workspace_size_n(t, K, N, n) for (_, t, N, K, _) in layer] + [L.chip_mul_mat_workspace_size_n(ca.Q6_K, H, V, n)])
        wss = [dev.alloc(wsz) for _ in range(3)]
        fused = n <= 4            # chip_mul_mat quantizes in the GEMV prologue: one launch per matmul

        def matmul(t, wptr, N, K, src, stream, lane, prepared):
            yp = y.ptr + lane * n * V * 4
            if fused:
                dev.check(L.chip_mul_mat(t, wptr, dev.row_size(t, K), K, N, src.ptr, K, n, yp, N, wss[lane].ptr, wsz, stream))
            else:
                if not prepared:
                    dev.check(L.chip_mul_mat_prepare(t, K, src.ptr, K, n, wss[lane].ptr, wsz, stream))
                dev.check(L.chip_mul_mat_run_ws(t, wptr, dev.row_size(t, K), K, N, n, wss[lane].ptr, wsz, yp, N, stream))

        def fork(streams):
            e = hip.event()
            hip.record(e, st)
            for s_ in streams:
                assert hl.hipStreamWaitEvent(s_, e, 0) == 0

        def join(streams):
            for s_ in streams:
                e = hip.event()
                hip.record(e, s_)
                assert hl.hipStreamWaitEvent(st, e, 0) == 0

        def one_step(parallel):
            """serial: the 225 matmuls back to back on one stream (what a one-stream ggml backend issues).
            parallel: matmuls of a layer that share an input and do not depend on each other (wq/wk/wv; up/gate)
            run as concurrent branches of the graph; wo and down wait for them."""
            for l in range(NL):
                base = arena.ptr + l * layer_bytes
                W = {name: (t, base + o, N, K) for (name, t, N, K, _), o in zip(layer, first)}
                if parallel:
                    fork(side)
                    matmul(*W["wq"], x_h, st, 0, False)
                    matmul(*W["wk"], x_h, side[0], 1, False)
                    matmul(*W["wv"], x_h, side[1], 2, False)
                    join(side)
                    matmul(*W["wo"], x_h, st, 0, False)
                    fork(side[:1])
                    matmul(*W["up"], x_h, st, 0, False)
                    matmul(*W["gate"], x_h, side[0], 1, False)
                    join(side[:1])
                    matmul(*W["down"], x_ff, st, 0, False)
                else:
                    matmul(*W["wq"], x_h, st, 0, False)
                    matmul(*W["wk"], x_h, st, 0, True)          # wq/wk share the quantized input (both Q8_K planes)
                    matmul(*W["wv"], x_h, st, 0, True)
                    matmul(*W["wo"], x_h, st, 0, False)
                    matmul(*W["up"], x_h, st, 0, False)
                    matmul(*W["gate"], x_h, st, 0, True)
                    matmul(*W["down"], x_ff, st, 0, False)
            matmul(ca.Q6_K, arena.ptr + head_off, V, H, x_h, st, 0, False)

        b = total + 4 * n * (NL * sum(K + N for (_, _, N, K, _) in layer) + H + V)
        entry = {"weight_bytes": total, "matmuls": 7 * NL + 1}
        for mode in (("serial", "parallel") if n <= 8 else ("serial",)):
            one_step(mode == "parallel")
            dev.sync(st)
            graph, gexec = C.c_void_p(), C.c_void_p()
            assert hl.hipStreamBeginCapture(st, 0) == 0
            one_step(mode == "parallel")
            assert hl.hipStreamEndCapture(st, C.byref(graph)) == 0
            assert hl.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
            us = time_runs(dev, hip, st, lambda: hl.hipGraphLaunch(gexec, st), 20, warm=2)
            entry[mode] = {"us_per_step": round(us, 1), "tokens_per_s": round(n / (us * 1e-6), 1),
                           "GBps": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 1e3 / HBM_PEAK_GBS, 4)}
            if n > 8:                                                   # prefill: the matrix pipe is the yardstick
                ops = 2.0 * n * (NL * sum(N * K for (_, _, N, K, _) in layer) + V * H)
                entry[mode]["TOPS"] = round(ops / us / 1e6, 1)
                entry[mode]["int8_frac"] = round(ops / us / 1e6 / INT8_PEAK_TOPS, 4)
        entry["whole_layers"] = full_layers(n, 512 if n == 512 else 4096, wss[0], wsz)      # decode and the 8-token batch over 4096 cached positions
        res["config5_llama3_8b_q4_K_M_trace_n%d" % n] = entry
        for bf in [x_h, x_ff, y] + wss:
            bf.free()
    arena.free()
    return res


def cpu_baseline(step_bytes_n):
    """Reference ggml-cpu MUL_MAT (oracle/_ref) or the oracle port on the host cores, bounded sample:
    the two headline shapes at n = 1 and n = 8."""
    import oracle as O
    cores = min(16, os.cpu_count() or 1)
    rng = np.random.default_rng(2)
    use_ref = O.Reference.available()
    eng = O.Reference() if use_ref else O.Oracle()
    t_total, b_total, budget = 0.0, 0, 20.0
    t_start = time.perf_counter()
    for (N, K) in ((11008, 4096), (4096, 11008)):
        w = rng.integers(0, 256, (N, K // 32, 34), dtype=np.uint8)
        w[..., 0:2] = np.array([0.0107], np.float16).view(np.uint8)
        w = w.reshape(N, -1)
        for n in (1, 8):
            x = rng.standard_normal((n, K)).astype(np.float32)
            if use_ref:
                _, times = eng.mul_mat_graph(O.Q8_0, w, x, nthreads=cores, repeat=12)
                t = float(np.median(times[2:]))
            else:
                t0 = time.perf_counter()
                eng.mul_mat(O.Q8_0, w, x, nthreads=cores)
                t = time.perf_counter() - t0
            t_total += t
            b_total += w.size + 4 * n * (K + N)
            if time.perf_counter() - t_start > budget:
                break
    return {"value": round(b_total / t_total / 1e9, 2), "unit": "GB/s", "cores": cores,
            "kind": "reference" if use_ref else "port",
            "sample": "Q8_0 W[11008x4096] and W[4096x11008] at n=1 and n=8, median of 10 calls each, "
                      "%s with a persistent %d-thread pool" % ("reference ggml-cpu MUL_MAT graph (AVX2 build)" if use_ref
                                                               else "oracle restatement", cores)}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (every figure is single-GPU)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    import cactus_amd as ca
    dev = ca.Device(0)
    hip = Hip()
    value, ms_per_step, step_bytes, roof, info = bench_headline(dev, hip, args.steps, args.warmup)
    extra = {} if args.no_extra else bench_extra(dev, hip, trace=not args.no_trace)
    cpu = None if args.no_cpu else cpu_baseline(step_bytes)
    line = {
        "metric": "quant mul_mat GEMV HBM GB/s & prefill int8 TOPS (% of roofline), 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": "BASELINE configs[1]: Q8_0 x Q8_0 decode GEMV, W[11008x4096] and W[4096x11008], "
                               "n in {1,2,4,8}; step = 8 ops (GPU Q8_0 activation quantize + GEMV each); cold weights",
                   "bytes_per_step": step_bytes, "device": dev.info.arch.decode(), **info},
        "roofline": roof, "cpu_baseline": cpu, "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
