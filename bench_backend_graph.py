"""Timing of the ggml backend as llama.cpp drives it: a LLaMA-3-8B-shaped graph (NL layers of attention over an F16 KV
cache and a gated FFN, Q4_K / Q6_K weights as in a Q4_K_M file, 4096 cached positions) is built with the reference's own
ggml (oracle/_ref/libggml_ref.so), weights and caches live in HIP buffers, and the reference scheduler runs it on the HIP
backend.  Prints the wall time of lm_ggml_backend_sched_graph_compute for NTOK new tokens (one launch per kernel, no
HIP graph), and the backend's counters.  Not a test (pytest does not collect it):

    NTOK=1 python bench_backend_graph.py          # decode;  NTOK=8 / 32 / 512: small batches, a prefill chunk
"""
import ctypes as C
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))          # ggml_host: the ctypes host over the reference's ggml build
import oracle as O
from ggml_host import Host

NL = int(os.environ.get("NL", "32"))
n = int(os.environ.get("NTOK", "1"))
H, FF, hd, n_head, n_head_kv = 4096, 14336, 128, 32, 8
KV = hd * n_head_kv
kv_size, n_kv = 4352, 4096
head = n_kv - n

host = Host()
host.reg = host.load_hip()
L = host.L
dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
hip = L.lm_ggml_backend_dev_init(dev, None)
cpu = L.lm_ggml_backend_cpu_init()
rng = np.random.default_rng(0)


def blocks(t, N, K):
    bs = {O.Q4_K: 144, O.Q6_K: 210}[t]
    nb = N * K // 256
    a = rng.integers(0, 256, (nb, bs), dtype=np.uint8)
    d = np.frombuffer(np.float16(0.01).tobytes(), np.uint8)
    if t == O.Q4_K:
        a[:, 0:2] = d
        a[:, 2:4] = d
    else:
        a[:, 208:210] = d
    return a


shapes = [("wq", O.Q4_K, H, H), ("wk", O.Q4_K, KV, H), ("wv", O.Q6_K, KV, H), ("wo", O.Q4_K, H, H), ("gate", O.Q4_K, FF, H),
          ("up", O.Q4_K, FF, H), ("down", O.Q6_K, H, FF)]
hostw = {nm: blocks(t, N, K) for nm, t, N, K in shapes}
wctx = host.context(n_tensors=NL * 10 + 8, with_graph=False)
W = []
for l in range(NL):
    W.append({nm: host.tensor_2d(wctx, t, K, N, f"{nm}{l}") for nm, t, N, K in shapes})
tn = L.lm_ggml_new_tensor_1d(wctx, O.F32, H)
wbuf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(wctx, L.lm_ggml_backend_dev_buffer_type(dev))
L.lm_ggml_backend_buffer_set_usage(wbuf, 1)
for l in range(NL):
    for nm, *_ in shapes:
        host.set(W[l][nm], hostw[nm])
host.set(tn, np.ones(H, np.float32))
cctx = host.context(n_tensors=2 * NL + 4, with_graph=False)
caches = [(host.tensor_2d(cctx, O.F16, KV, kv_size), host.tensor_2d(cctx, O.F16, KV, kv_size)) for _ in range(NL)]
cbuf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(cctx, L.lm_ggml_backend_dev_buffer_type(dev))
L.lm_ggml_backend_buffer_clear(cbuf, 0)

ctx = host.context(n_tensors=NL * 64 + 64)
tx = host.tensor_2d(ctx, O.F32, H, n, "x")
tpos = L.lm_ggml_new_tensor_1d(ctx, 26, n)
tmask = host.tensor_2d(ctx, O.F16, n_kv, max(n, 8) if n % 8 else n, "mask")
for t in (tx, tpos, tmask):
    L.lm_ggml_set_input(t)
g = L.lm_ggml_new_graph(ctx)
scale = 1.0 / np.sqrt(hd)
inp = tx
for l in range(NL):
    w = W[l]
    kc, vc = caches[l]
    cur = L.lm_ggml_mul(ctx, L.lm_ggml_rms_norm(ctx, inp, 1e-5), tn)
    rope = lambda t, nh: L.lm_ggml_rope_ext(ctx, L.lm_ggml_reshape_3d(ctx, t, hd, nh, n), tpos, None, hd, 2, 8192, 500000.0, 1.0,
                                         0.0, 1.0, 32.0, 1.0)
    q = rope(L.lm_ggml_mul_mat(ctx, w["wq"], cur), n_head)
    k = rope(L.lm_ggml_mul_mat(ctx, w["wk"], cur), n_head_kv)
    v = L.lm_ggml_mul_mat(ctx, w["wv"], cur)
    k_store = L.lm_ggml_cpy(ctx, k, L.lm_ggml_view_1d(ctx, kc, n * KV, 2 * KV * head))
    v_store = L.lm_ggml_cpy(ctx, L.lm_ggml_transpose(ctx, v), L.lm_ggml_view_2d(ctx, vc, n, KV, kv_size * 2, head * 2))
    for t in (q, k, v, k_store, v_store):                # the reference's order (llama-graph.cpp:1265-1277): q, k, v, then the stores
        L.lm_ggml_build_forward_expand(g, t)
    kview = L.lm_ggml_view_3d(ctx, kc, hd, n_head_kv, n_kv, 2 * hd, 2 * KV, 0)
    vview = L.lm_ggml_view_3d(ctx, vc, n_kv, n_head_kv, hd, 2 * kv_size * hd, 2 * kv_size, 0)
    qp = L.lm_ggml_permute(ctx, q, 0, 2, 1, 3)
    kp = L.lm_ggml_permute(ctx, kview, 0, 2, 1, 3)
    vp = L.lm_ggml_permute(ctx, vview, 0, 2, 1, 3)
    kq = L.lm_ggml_mul_mat(ctx, kp, qp)
    sm = L.lm_ggml_soft_max_ext(ctx, kq, tmask, scale, 0.0)
    kqv = L.lm_ggml_mul_mat(ctx, vp, sm)
    merged = L.lm_ggml_cont_2d(ctx, L.lm_ggml_permute(ctx, kqv, 0, 2, 1, 3), H, n)
    ffn_inp = L.lm_ggml_add(ctx, L.lm_ggml_mul_mat(ctx, w["wo"], merged), inp)
    c2 = L.lm_ggml_mul(ctx, L.lm_ggml_rms_norm(ctx, ffn_inp, 1e-5), tn)
    tmp = L.lm_ggml_mul_mat(ctx, w["up"], c2)
    gt = L.lm_ggml_silu(ctx, L.lm_ggml_mul_mat(ctx, w["gate"], c2))
    act = L.lm_ggml_mul(ctx, gt, tmp)
    inp = L.lm_ggml_add(ctx, L.lm_ggml_mul_mat(ctx, w["down"], act), ffn_inp)
    L.lm_ggml_build_forward_expand(g, inp)
out = L.lm_ggml_mul(ctx, L.lm_ggml_rms_norm(ctx, inp, 1e-5), tn)
L.lm_ggml_set_output(out)
L.lm_ggml_build_forward_expand(g, out)
L.lm_ggml_graph_n_nodes.restype = C.c_int
L.lm_ggml_graph_n_nodes.argtypes = [C.c_void_p]
print("nodes", L.lm_ggml_graph_n_nodes(g), flush=True)
backends = (C.c_void_p * 2)(hip, cpu)
sched = L.lm_ggml_backend_sched_new(backends, None, 2, 4096, False, True)
assert L.lm_ggml_backend_sched_alloc_graph(sched, g)
print("splits", L.lm_ggml_backend_sched_get_n_splits(sched), flush=True)
host.set(tx, rng.standard_normal((n, H)).astype(np.float32))
host.set(tpos, np.arange(head, head + n, dtype=np.int32))
host.set(tmask, np.zeros((max(n, 8) if n % 8 else n, n_kv), np.float16))
import cactus_amd
blib = C.CDLL(cactus_amd.BACKEND_LIB)
blib.lm_ggml_backend_hip_get_fused_pairs.restype = C.c_ulonglong
f0 = blib.lm_ggml_backend_hip_get_fused_pairs()
for it in range(3):
    assert L.lm_ggml_backend_sched_graph_compute(sched, g) == 0
print("fused per graph", (blib.lm_ggml_backend_hip_get_fused_pairs() - f0) / 3, flush=True)
blib.lm_ggml_backend_hip_get_grouped_matmuls.restype = C.c_ulonglong
print("projections run in group launches so far", blib.lm_ggml_backend_hip_get_grouped_matmuls(), "(3 graphs)", flush=True)
blib.lm_ggml_backend_hip_get_quantizers_skipped.restype = C.c_ulonglong
print("quantizers skipped so far", blib.lm_ggml_backend_hip_get_quantizers_skipped(), flush=True)
blib.lm_ggml_backend_hip_get_planes_copies.restype = C.c_ulonglong
blib.lm_ggml_backend_hip_get_planes_bytes.restype = C.c_ulonglong
print("Q6_K weights read from a copy in planes:", blib.lm_ggml_backend_hip_get_planes_copies(), "copies,",
      blib.lm_ggml_backend_hip_get_planes_bytes() >> 20, "MiB", flush=True)
ts = []
for it in range(20):
    t0 = time.perf_counter()
    assert L.lm_ggml_backend_sched_graph_compute(sched, g) == 0
    ts.append(time.perf_counter() - t0)
# the same split in two: how long the host needs to issue the launches, and the wait for the device after that
L.lm_ggml_backend_sched_graph_compute_async.restype = C.c_int
L.lm_ggml_backend_sched_graph_compute_async.argtypes = [C.c_void_p, C.c_void_p]
L.lm_ggml_backend_sched_synchronize.argtypes = [C.c_void_p]
issue = []
for it in range(10):
    t0 = time.perf_counter()
    assert L.lm_ggml_backend_sched_graph_compute_async(sched, g) == 0
    issue.append(time.perf_counter() - t0)
    L.lm_ggml_backend_sched_synchronize(sched)
print(f"NL={NL} n={n}: host time to issue one graph us: median {np.median(issue) * 1e6:.0f}", flush=True)
ts = np.array(ts) * 1e6
print(f"NL={NL} n={n}: graph_compute wall us: min {ts.min():.0f} median {np.median(ts):.0f} max {ts.max():.0f}", flush=True)
y = host.get(out, np.float32, (n, H))
print("finite", np.isfinite(y).all(), float(np.abs(y).mean()))
