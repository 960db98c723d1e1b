"""The ggml backend (libggml-hip.so) driven the way llama.cpp drives a backend, with the reference's own ggml
(oracle/_ref) as the host framework: dynamic load + registration, weight upload into the HIP buffer type,
one-node and multi-node MUL_MAT graphs, the reference scheduler splitting a mixed graph between HIP and CPU,
and lm_ggml_backend_compare_graph_backend node-by-node against the reference CPU backend."""
import ctypes as C

import numpy as np
import pytest

import common
import oracle as O

pytestmark = pytest.mark.gpu

REL_TOL = 1e-5


@pytest.fixture(scope="module")
def host():
    if not O.Reference.available():
        pytest.skip("oracle/_ref/libggml_ref.so not present: no ggml host framework to load the backend into")
    from ggml_host import Host
    h = Host()
    h.reg = h.load_hip()
    return h


def test_registration_and_device(host):
    L = host.L
    assert L.lm_ggml_backend_reg_name(host.reg) == b"HIP"
    assert L.lm_ggml_backend_reg_by_name(b"HIP") == host.reg            # it is in the reference's registry now
    assert L.lm_ggml_backend_reg_dev_count(host.reg) == 1
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    assert L.lm_ggml_backend_dev_name(dev) == b"HIP0"
    assert b"gfx950" in L.lm_ggml_backend_dev_description(dev)
    assert L.lm_ggml_backend_dev_type(dev) == 2                         # ACCEL
    fr, tot = C.c_size_t(), C.c_size_t()
    L.lm_ggml_backend_dev_memory(dev, C.byref(fr), C.byref(tot))
    assert tot.value > 200 << 30 and 0 < fr.value <= tot.value
    buft = L.lm_ggml_backend_dev_buffer_type(dev)
    assert L.lm_ggml_backend_buft_name(buft) == b"HIP"
    assert not L.lm_ggml_backend_buft_is_host(buft)
    assert L.lm_ggml_backend_dev_supports_buft(dev, buft)
    be = L.lm_ggml_backend_dev_init(dev, None)
    assert be and L.lm_ggml_backend_name(be) == b"HIP"
    assert L.lm_ggml_backend_get_default_buffer_type(be) == buft
    L.lm_ggml_backend_free(be)


@pytest.mark.parametrize("wt", O.WEIGHT_TYPES, ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("n", [1, 7, 40])
def test_one_node_graph(host, orc, wt, n):
    """Weights and activations allocated in the HIP buffer type, one MUL_MAT node, direct graph_compute."""
    L = host.L
    K, N = 1024, 200
    wq = orc.quantize_weights(wt, common.weights_f32(wt + n, N, K))
    x = common.activations_f32(wt + n, n, K)
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    be = L.lm_ggml_backend_dev_init(dev, None)
    ctx = host.context()
    a = host.tensor_2d(ctx, wt, K, N, "w")
    b = host.tensor_2d(ctx, O.F32, K, n, "x")
    c = L.lm_ggml_mul_mat(ctx, a, b)
    g = L.lm_ggml_new_graph(ctx)
    L.lm_ggml_build_forward_expand(g, c)
    assert L.lm_ggml_backend_dev_supports_op(dev, c) is False            # weights not in a HIP buffer yet
    buf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(ctx, L.lm_ggml_backend_dev_buffer_type(dev))
    assert buf and L.lm_ggml_backend_buffer_get_size(buf) >= wq.size + x.nbytes + 4 * n * N
    assert L.lm_ggml_backend_dev_supports_op(dev, c) is True
    host.set(a, wq)
    host.set(b, x)
    assert np.array_equal(host.get(a, np.uint8, wq.shape), wq)           # set_tensor / get_tensor round trip
    assert L.lm_ggml_backend_graph_compute(be, g) == 0
    y = host.get(c, np.float32, (n, N))
    ref = orc.mul_mat(wt, wq, x, nthreads=8, want=("sum_abs",))
    assert (np.abs(y.astype(np.float64) - ref["y"]) <= REL_TOL * ref["sum_abs"]).all()
    # memset_tensor / clear
    L.lm_ggml_backend_tensor_memset(c, 0x7f, 0, 4 * n * N)
    assert (host.get(c, np.uint8, (4 * n * N,)) == 0x7f).all()
    L.lm_ggml_backend_buffer_clear(buf, 0)
    assert not host.get(a, np.uint8, wq.shape).any()
    L.lm_ggml_backend_buffer_free(buf)
    L.lm_ggml_backend_free(be)
    L.lm_ggml_free(ctx)


@pytest.mark.parametrize("wt", (O.Q8_0, O.Q4_0, O.Q5_1), ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("K,n", [(576, 1), (960, 9), (896, 40)])
def test_one_node_graph_with_a_hidden_size_that_is_no_multiple_of_256(host, orc, wt, K, n):
    """Small models have hidden sizes such as 576, 896 or 960: rows of the 32-value block types that are multiples of 4
    bytes only.  The backend takes them (GEMV; the GEMM at K = 896 with 40 tokens)."""
    L = host.L
    N = 300
    wq = orc.quantize_weights(wt, common.weights_f32(wt + K, N, K))
    x = common.activations_f32(wt + K + n, n, K)
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    be = L.lm_ggml_backend_dev_init(dev, None)
    ctx = host.context()
    a = host.tensor_2d(ctx, wt, K, N, "w")
    b = host.tensor_2d(ctx, O.F32, K, n, "x")
    c = L.lm_ggml_mul_mat(ctx, a, b)
    g = L.lm_ggml_new_graph(ctx)
    L.lm_ggml_build_forward_expand(g, c)
    buf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(ctx, L.lm_ggml_backend_dev_buffer_type(dev))
    assert L.lm_ggml_backend_dev_supports_op(dev, c) is True
    host.set(a, wq)
    host.set(b, x)
    assert L.lm_ggml_backend_graph_compute(be, g) == 0
    y = host.get(c, np.float32, (n, N))
    ref = orc.mul_mat(wt, wq, x, nthreads=8, want=("sum_abs",))
    assert (np.abs(y.astype(np.float64) - ref["y"]) <= REL_TOL * ref["sum_abs"]).all()
    L.lm_ggml_backend_buffer_free(buf)
    L.lm_ggml_backend_free(be)
    L.lm_ggml_free(ctx)


@pytest.mark.parametrize("wt", (O.Q4_K, O.Q8_0, O.Q6_K, O.Q4_0), ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("n,ne02,ne03,ne12,ne13", [(1, 2, 1, 4, 1), (3, 2, 2, 2, 4), (40, 3, 1, 3, 2)])
def test_batched_and_broadcast_matmul_over_quantized_weights(host, orc, wt, n, ne02, ne03, ne12, ne13):
    """MUL_MAT with batch dimensions over a quantized src0 (reference ggml-cpu/ggml-cpu.c:1188-1189, 1294-1295: slice (i12, i13)
    of src1 meets slice (i12 / r2, i13 / r3) of src0): every slice equals, bit for bit, the one-node graph of that slice's two
    matrices on the same backend, and meets the oracle's tolerance."""
    L = host.L
    K, N = 512, 72
    rng_seed = wt * 100 + n
    wq = np.stack([orc.quantize_weights(wt, common.weights_f32(rng_seed + i, N, K)) for i in range(ne02 * ne03)])
    x = np.stack([common.activations_f32(rng_seed + 50 + i, n, K) for i in range(ne12 * ne13)])
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    be = L.lm_ggml_backend_dev_init(dev, None)
    ctx = host.context()
    a = L.lm_ggml_new_tensor_4d(ctx, wt, K, N, ne02, ne03)
    b = L.lm_ggml_new_tensor_4d(ctx, O.F32, K, n, ne12, ne13)
    c = L.lm_ggml_mul_mat(ctx, a, b)
    wf = L.lm_ggml_new_tensor_4d(ctx, O.F32, K, N, ne02, ne03)
    cf = L.lm_ggml_mul_mat(ctx, wf, b)
    g = L.lm_ggml_new_graph(ctx)
    L.lm_ggml_build_forward_expand(g, c)
    ctx2 = host.context()                                                # the slice's one-node graph, in a context of its own
    a2 = host.tensor_2d(ctx2, wt, K, N, "w")
    b2 = host.tensor_2d(ctx2, O.F32, K, n, "x")
    c2 = L.lm_ggml_mul_mat(ctx2, a2, b2)
    g2 = L.lm_ggml_new_graph(ctx2)
    L.lm_ggml_build_forward_expand(g2, c2)
    buf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(ctx, L.lm_ggml_backend_dev_buffer_type(dev))
    buf2 = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(ctx2, L.lm_ggml_backend_dev_buffer_type(dev))
    assert L.lm_ggml_backend_dev_supports_op(dev, c) is True
    assert L.lm_ggml_backend_dev_supports_op(dev, cf) is False           # F32 weights stay declined
    host.set(a, wq)
    host.set(b, x)
    assert L.lm_ggml_backend_graph_compute(be, g) == 0
    y = host.get(c, np.float32, (ne13, ne12, n, N))
    r2, r3 = ne12 // ne02, ne13 // ne03
    for i13 in range(ne13):
        for i12 in range(ne12):
            wi = (i13 // r3) * ne02 + i12 // r2
            xi = i13 * ne12 + i12
            host.set(a2, wq[wi])
            host.set(b2, x[xi])
            assert L.lm_ggml_backend_graph_compute(be, g2) == 0
            assert y[i13, i12].tobytes() == host.get(c2, np.float32, (n, N)).tobytes(), (i12, i13)
            ref = orc.mul_mat(wt, wq[wi], x[xi], nthreads=8, want=("sum_abs",))
            assert (np.abs(y[i13, i12].astype(np.float64) - ref["y"]) <= REL_TOL * ref["sum_abs"]).all(), (i12, i13)
    L.lm_ggml_backend_buffer_free(buf)
    L.lm_ggml_backend_buffer_free(buf2)
    L.lm_ggml_backend_free(be)
    L.lm_ggml_free(ctx)
    L.lm_ggml_free(ctx2)


def test_unsupported_ops_are_declined(host):
    L = host.L
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    ctx = host.context()
    w = host.tensor_2d(ctx, O.Q4_0, 256, 8)
    wf = host.tensor_2d(ctx, O.F32, 256, 8)
    x = host.tensor_2d(ctx, O.F32, 256, 2)
    k96 = host.tensor_2d(ctx, O.Q8_0, 96, 8)
    x96 = host.tensor_2d(ctx, O.F32, 96, 2)
    mm = L.lm_ggml_mul_mat(ctx, w, x)
    mm_f32 = L.lm_ggml_mul_mat(ctx, wf, x)
    mm_96 = L.lm_ggml_mul_mat(ctx, k96, x96)
    add = L.lm_ggml_add(ctx, x, x)
    x12 = host.tensor_2d(ctx, O.F32, 12, 2)
    silu12 = L.lm_ggml_silu(ctx, x12)
    wide = host.tensor_2d(ctx, O.F32, 256, 4)
    add_bcast = L.lm_ggml_add(ctx, wide, x)                              # src1 [256, 2] repeated over [256, 4]
    sqr = L.lm_ggml_sqr(ctx, x)
    view = L.lm_ggml_reshape_2d(ctx, x, 128, 4)
    buf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(ctx, L.lm_ggml_backend_dev_buffer_type(dev))
    assert L.lm_ggml_backend_dev_supports_op(dev, mm) is True
    assert L.lm_ggml_backend_dev_supports_op(dev, mm_f32) is False       # F32 weights: not this path
    assert L.lm_ggml_backend_dev_supports_op(dev, mm_96) is False        # K not a multiple of 256
    assert L.lm_ggml_backend_dev_supports_op(dev, add) is True           # element-wise F32 ops next to the matmuls
    assert L.lm_ggml_backend_dev_supports_op(dev, L.lm_ggml_mul(ctx, x, x)) is True
    assert L.lm_ggml_backend_dev_supports_op(dev, L.lm_ggml_rms_norm(ctx, x, 1e-5)) is True
    assert L.lm_ggml_backend_dev_supports_op(dev, L.lm_ggml_silu(ctx, x)) is True
    assert L.lm_ggml_backend_dev_supports_op(dev, silu12) is False       # row tail: the reference uses libm's expf there
    assert L.lm_ggml_backend_dev_supports_op(dev, add_bcast) is False    # a broadcast other than one row
    assert L.lm_ggml_backend_dev_supports_op(dev, sqr) is False         # an op outside the path
    assert L.lm_ggml_backend_dev_supports_op(dev, view) is True
    # graph_compute on a node the device declined reports failure, it does not compute on the host
    be = L.lm_ggml_backend_dev_init(dev, None)
    g = L.lm_ggml_new_graph(ctx)
    L.lm_ggml_build_forward_expand(g, sqr)
    assert L.lm_ggml_backend_graph_compute(be, g) == -1                  # LM_GGML_STATUS_FAILED
    L.lm_ggml_backend_free(be)
    L.lm_ggml_backend_buffer_free(buf)
    L.lm_ggml_free(ctx)


def test_scheduler_splits_between_hip_and_cpu(host, orc):
    """llama.cpp's flow: weights in a HIP buffer tagged USAGE_WEIGHTS, activations produced on the CPU; the
    reference scheduler assigns the MUL_MATs and the ADD between them to HIP, the SQR (an op outside the path) to the CPU, and copies
    tensors across."""
    L = host.L
    K, N1, N2, n = 2048, 512, 256, 3
    w1 = orc.quantize_weights(O.Q4_K, common.weights_f32(11, N1, K))
    w2 = orc.quantize_weights(O.Q6_K, common.weights_f32(12, N2, K))
    w3 = orc.quantize_weights(O.Q8_0, common.weights_f32(13, N2, 512))
    x = common.activations_f32(11, n, K)
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    hip = L.lm_ggml_backend_dev_init(dev, None)
    cpu = L.lm_ggml_backend_cpu_init()
    # weights
    wctx = host.context(with_graph=False)
    tw1 = host.tensor_2d(wctx, O.Q4_K, K, N1, "w1")
    tw2 = host.tensor_2d(wctx, O.Q6_K, K, N2, "w2")
    tw3 = host.tensor_2d(wctx, O.Q8_0, 512, N2, "w3")
    wbuf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(wctx, L.lm_ggml_backend_dev_buffer_type(dev))
    L.lm_ggml_backend_buffer_set_usage(wbuf, 1)
    host.set(tw1, w1); host.set(tw2, w2); host.set(tw3, w3)
    # graph: y = w3 @ (w1 @ x)[:512]... keep shapes simple: h = w1 x ; z = w2 x ; s = w3 h + z
    ctx = host.context()
    tx = host.tensor_2d(ctx, O.F32, K, n, "x")
    L.lm_ggml_set_input(tx)
    h = L.lm_ggml_mul_mat(ctx, tw1, tx)          # [N1=512, n]
    z = L.lm_ggml_mul_mat(ctx, tw2, tx)          # [N2, n]
    s = L.lm_ggml_mul_mat(ctx, tw3, h)           # [N2, n]   (K = 512 = N1)
    out_add = L.lm_ggml_add(ctx, s, z)
    L.lm_ggml_set_output(out_add)
    out = L.lm_ggml_sqr(ctx, out_add)
    L.lm_ggml_set_output(out)
    g = L.lm_ggml_new_graph(ctx)
    L.lm_ggml_build_forward_expand(g, out)
    backends = (C.c_void_p * 2)(hip, cpu)
    sched = L.lm_ggml_backend_sched_new(backends, None, 2, 64, False, True)
    assert L.lm_ggml_backend_sched_alloc_graph(sched, g)
    host.set(tx, x)
    before = (C.c_ulonglong(), C.c_ulonglong())
    import cactus_amd
    blib = C.CDLL(cactus_amd.BACKEND_LIB)
    blib.lm_ggml_backend_hip_get_stats(C.byref(before[0]), C.byref(before[1]))
    assert L.lm_ggml_backend_sched_graph_compute(sched, g) == 0
    after = (C.c_ulonglong(), C.c_ulonglong())
    blib.lm_ggml_backend_hip_get_stats(C.byref(after[0]), C.byref(after[1]))
    assert after[0].value - before[0].value == 3                       # the three MUL_MATs ran on the GPU
    assert L.lm_ggml_backend_sched_get_tensor_backend(sched, h) == hip
    assert L.lm_ggml_backend_sched_get_tensor_backend(sched, out_add) == hip
    assert L.lm_ggml_backend_sched_get_tensor_backend(sched, out) == cpu
    assert L.lm_ggml_backend_sched_get_n_splits(sched) >= 2
    y = host.get(out_add, np.float32, (n, N2))
    sq = host.get(out, np.float32, (n, N2))
    assert sq.tobytes() == (y * y).tobytes()
    # reference: same graph entirely on the reference CPU path (through the oracle, bit-identical to it)
    hh = orc.mul_mat(O.Q4_K, w1, x)["y"]
    zz = orc.mul_mat(O.Q6_K, w2, x, want=("sum_abs",))
    ss = orc.mul_mat(O.Q8_0, w3, hh, want=("sum_abs",))
    want = ss["y"] + zz["y"]
    # h itself carries the GPU's rounding (<= 1e-5 relative), which the Q8_0 requantization of h passes on:
    # compare at a tolerance that reflects two chained ops
    scale = ss["sum_abs"] + zz["sum_abs"]
    assert (np.abs(y - want) <= 2e-3 * scale).all()
    L.lm_ggml_backend_sched_free(sched)
    L.lm_ggml_backend_buffer_free(wbuf)
    L.lm_ggml_backend_free(hip)
    L.lm_ggml_backend_free(cpu)
    L.lm_ggml_free(ctx)
    L.lm_ggml_free(wctx)


def test_compare_graph_backend_against_reference_cpu(host, orc):
    """The reference's own node-by-node comparison engine (ggml-backend.cpp:1821-1857): graph built on the CPU
    backend, copied to HIP, each node evaluated on both and handed to a callback."""
    L = host.L
    from ggml_host import EVAL_CB
    K, n = 1024, 5
    specs = [(O.Q4_0, 300), (O.Q8_0, 64), (O.Q4_K, 257), (O.Q6_K, 130), (O.Q5_0, 77), (O.Q5_K, 96), (O.IQ4_NL, 45),
             (O.Q4_1, 51), (O.Q5_1, 38), (O.F16, 29)]
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    hip = L.lm_ggml_backend_dev_init(dev, None)
    cpu = L.lm_ggml_backend_cpu_init()
    ctx = host.context(n_tensors=64)
    tx = host.tensor_2d(ctx, O.F32, K, n, "x")
    tws, outs = [], []
    for i, (wt, N) in enumerate(specs):
        tw = host.tensor_2d(ctx, wt, K, N, "w%d" % i)
        tws.append(tw)
        outs.append(L.lm_ggml_mul_mat(ctx, tw, tx))
    g = L.lm_ggml_new_graph(ctx)
    for o in outs:
        L.lm_ggml_build_forward_expand(g, o)
    buf = L.lm_ggml_backend_alloc_ctx_tensors(ctx, cpu)
    x = common.activations_f32(31, n, K)
    host.set(tx, x)
    weights = []
    for (wt, N), tw in zip(specs, tws):
        wq = orc.quantize_weights(wt, common.weights_f32(31 + wt, N, K))
        weights.append(wq)
        host.set(tw, wq)
    seen = []

    def cb(idx, t1, t2, ud):
        wt, N = specs[idx]
        y1 = host.get(t1, np.float32, (n, N))          # reference CPU backend
        y2 = host.get(t2, np.float32, (n, N))          # HIP backend
        sa = orc.mul_mat(wt, weights[idx], x, nthreads=8, want=("sum_abs",))["sum_abs"]
        seen.append(bool((np.abs(y1.astype(np.float64) - y2) <= REL_TOL * sa).all()))
        return True

    ok = L.lm_ggml_backend_compare_graph_backend(cpu, hip, g, EVAL_CB(cb), None)
    assert ok and seen == [True] * len(specs)
    L.lm_ggml_backend_buffer_free(buf)
    L.lm_ggml_backend_free(hip)
    L.lm_ggml_backend_free(cpu)
    L.lm_ggml_free(ctx)


@pytest.mark.parametrize("wt", (O.Q4_K, O.Q8_0, O.Q6_K, O.F16), ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("n_tokens,ne11", [(1, 1), (6, 4)])
def test_mul_mat_id_node(host, orc, wt, n_tokens, ne11):
    """LM_GGML_OP_MUL_MAT_ID (mixture-of-experts matmul) through the backend: supports_op, direct graph_compute, and
    the reference's node-by-node comparison against its CPU backend."""
    L = host.L
    from ggml_host import EVAL_CB
    K, N, n_as, n_used = 512, 130, 6, 4
    I32 = 26
    rng = np.random.default_rng(5 + wt + n_tokens)
    W = np.stack([orc.quantize_weights(wt, common.weights_f32(60 + wt + e, N, K)) for e in range(n_as)])
    x = common.activations_f32(61 + wt, n_tokens * ne11, K).reshape(n_tokens, ne11, K)
    ids = np.stack([rng.permutation(n_as)[:n_used] for _ in range(n_tokens)]).astype(np.int32)
    ref = orc.mul_mat_id(wt, W, x, ids, nthreads=8, want=("sum_abs",))
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)

    def build(ctx):
        a = host.tensor_3d(ctx, wt, K, N, n_as, "experts")
        b = host.tensor_3d(ctx, O.F32, K, ne11, n_tokens, "x")
        i = host.tensor_2d(ctx, I32, n_used, n_tokens, "ids")
        c = L.lm_ggml_mul_mat_id(ctx, a, b, i)
        g = L.lm_ggml_new_graph(ctx)
        L.lm_ggml_build_forward_expand(g, c)
        return a, b, i, c, g

    # direct: everything in the HIP buffer type
    be = L.lm_ggml_backend_dev_init(dev, None)
    ctx = host.context()
    a, b, i, c, g = build(ctx)
    assert L.lm_ggml_backend_dev_supports_op(dev, c) is False            # experts not in a HIP buffer yet
    buf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(ctx, L.lm_ggml_backend_dev_buffer_type(dev))
    assert L.lm_ggml_backend_dev_supports_op(dev, c) is True
    host.set(a, W); host.set(b, x); host.set(i, ids)
    assert L.lm_ggml_backend_graph_compute(be, g) == 0
    y = host.get(c, np.float32, (n_tokens, n_used, N))
    assert (np.abs(y.astype(np.float64) - ref["y"]) <= REL_TOL * ref["sum_abs"]).all()
    L.lm_ggml_backend_buffer_free(buf)
    L.lm_ggml_free(ctx)

    # node by node against the reference CPU backend
    cpu = L.lm_ggml_backend_cpu_init()
    ctx = host.context()
    a, b, i, c, g = build(ctx)
    buf = L.lm_ggml_backend_alloc_ctx_tensors(ctx, cpu)
    host.set(a, W); host.set(b, x); host.set(i, ids)
    seen = []

    def cb(idx, t1, t2, ud):
        y1 = host.get(t1, np.float32, (n_tokens, n_used, N))
        y2 = host.get(t2, np.float32, (n_tokens, n_used, N))
        seen.append(bool(np.array_equal(y1, ref["y"]) and (np.abs(y1.astype(np.float64) - y2) <= REL_TOL * ref["sum_abs"]).all()))
        return True

    assert L.lm_ggml_backend_compare_graph_backend(cpu, be, g, EVAL_CB(cb), None) and seen == [True]
    L.lm_ggml_backend_buffer_free(buf)
    L.lm_ggml_backend_free(cpu)
    L.lm_ggml_backend_free(be)
    L.lm_ggml_free(ctx)


def test_async_upload_protocol_of_the_model_loader(host, orc):
    """What llama_model_loader::load_all_data does when a device reports async + host_buffer + events
    (reference llama-model-loader.cpp:905-1064): four pinned 1 MB staging buffers with one event each, the tensor
    uploaded chunk by chunk with set_tensor_async, the event of a buffer waited for before the buffer is refilled."""
    from ggml_host import DevProps
    L = host.L
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    props = DevProps()
    L.lm_ggml_backend_dev_get_props(dev, C.byref(props))
    assert props.caps.async_ and props.caps.host_buffer and props.caps.events and not props.caps.buffer_from_host_ptr
    assert props.name == b"HIP0" and props.memory_total > 200 << 30
    host_buft = L.lm_ggml_backend_dev_host_buffer_type(dev)
    assert host_buft and L.lm_ggml_backend_buft_name(host_buft) == b"HIP_Host" and L.lm_ggml_backend_buft_is_host(host_buft)
    assert L.lm_ggml_backend_buft_get_device(host_buft) == dev
    assert not L.lm_ggml_backend_dev_supports_buft(dev, host_buft)      # operands of the kernels live in device memory

    wt, K, N, n = O.Q4_K, 4096, 3000, 3                                  # 6.9 MB of weights: 7 chunks
    wq = orc.quantize_weights(wt, common.weights_f32(77, N, K))
    x = common.activations_f32(78, n, K)
    ctx = host.context()
    a = host.tensor_2d(ctx, wt, K, N, "w")
    b = host.tensor_2d(ctx, O.F32, K, n, "x")
    c = L.lm_ggml_mul_mat(ctx, a, b)
    g = L.lm_ggml_new_graph(ctx)
    L.lm_ggml_build_forward_expand(g, c)
    buf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(ctx, L.lm_ggml_backend_dev_buffer_type(dev))
    assert L.lm_ggml_backend_buffer_get_type(buf) == L.lm_ggml_backend_dev_buffer_type(dev)

    n_buffers, chunk = 4, 1 << 20
    bufs = [L.lm_ggml_backend_buft_alloc_buffer(host_buft, chunk) for _ in range(n_buffers)]
    assert all(bufs) and all(L.lm_ggml_backend_buffer_is_host(hb) for hb in bufs)
    ptrs = [L.lm_ggml_backend_buffer_get_base(hb) for hb in bufs]
    events = [L.lm_ggml_backend_event_new(dev) for _ in range(n_buffers)]
    assert all(events)
    be = L.lm_ggml_backend_dev_init(dev, None)
    raw = wq.reshape(-1)
    done, idx = 0, 0
    while done < raw.size:
        size = min(chunk, raw.size - done)
        L.lm_ggml_backend_event_synchronize(events[idx])                 # the buffer's previous upload has finished
        C.memmove(ptrs[idx], raw[done:done + size].ctypes.data, size)    # "file->read_raw" into pinned memory
        L.lm_ggml_backend_tensor_set_async(be, a, ptrs[idx], done, size)
        L.lm_ggml_backend_event_record(events[idx], be)
        done += size
        idx = (idx + 1) % n_buffers
    for ev in events:
        L.lm_ggml_backend_event_synchronize(ev)
    assert np.array_equal(host.get(a, np.uint8, wq.shape), wq)

    # activations through the async path too, compute on the same stream, result read back asynchronously
    xin = np.ascontiguousarray(x)
    L.lm_ggml_backend_tensor_set_async(be, b, xin.ctypes.data_as(C.c_void_p), 0, xin.nbytes)
    assert L.lm_ggml_backend_graph_compute(be, g) == 0
    y = np.empty((n, N), np.float32)
    L.lm_ggml_backend_tensor_get_async(be, c, y.ctypes.data_as(C.c_void_p), 0, y.nbytes)
    # a second backend (stream) waits for the first one's event before it reads the result
    be2 = L.lm_ggml_backend_dev_init(dev, None)
    L.lm_ggml_backend_event_record(events[0], be)
    L.lm_ggml_backend_event_wait(be2, events[0])
    y2 = np.empty((n, N), np.float32)
    L.lm_ggml_backend_tensor_get_async(be2, c, y2.ctypes.data_as(C.c_void_p), 0, y2.nbytes)
    L.lm_ggml_backend_synchronize(be)
    L.lm_ggml_backend_synchronize(be2)
    ref = orc.mul_mat(wt, wq, x, nthreads=8, want=("sum_abs",))
    assert (np.abs(y.astype(np.float64) - ref["y"]) <= REL_TOL * ref["sum_abs"]).all() and np.array_equal(y, y2)

    for ev in events:
        L.lm_ggml_backend_event_free(ev)
    for hb in bufs:
        L.lm_ggml_backend_buffer_free(hb)
    L.lm_ggml_backend_buffer_free(buf)
    L.lm_ggml_backend_free(be2)
    L.lm_ggml_backend_free(be)
    L.lm_ggml_free(ctx)


@pytest.mark.parametrize("n", [5, 2])
def test_ffn_block_stays_on_the_device(host, orc, n):
    """norm -> up / gate -> SiLU * up -> down -> residual, the FFN half of a transformer layer as llama.cpp builds it
    (reference llama-graph.cpp build_norm / build_ffn): with the element-wise ops on the device the reference scheduler
    puts the whole block into one HIP split."""
    import cactus_amd
    L = host.L
    H, FF = 1024, 2816
    eps = 1e-5
    rng = np.random.default_rng(3)
    wn = (1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    wu = orc.quantize_weights(O.Q4_K, common.weights_f32(21, FF, H))
    wg = orc.quantize_weights(O.Q4_K, common.weights_f32(22, FF, H))
    wd = orc.quantize_weights(O.Q6_K, common.weights_f32(23, H, FF))
    x = common.activations_f32(24, n, H)
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    hip = L.lm_ggml_backend_dev_init(dev, None)
    cpu = L.lm_ggml_backend_cpu_init()
    wctx = host.context(with_graph=False)
    tn = L.lm_ggml_new_tensor_1d(wctx, O.F32, H)
    tu = host.tensor_2d(wctx, O.Q4_K, H, FF, "up")
    tg = host.tensor_2d(wctx, O.Q4_K, H, FF, "gate")
    td = host.tensor_2d(wctx, O.Q6_K, FF, H, "down")
    wbuf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(wctx, L.lm_ggml_backend_dev_buffer_type(dev))
    L.lm_ggml_backend_buffer_set_usage(wbuf, 1)
    host.set(tn, wn); host.set(tu, wu); host.set(tg, wg); host.set(td, wd)
    ctx = host.context()
    tx = host.tensor_2d(ctx, O.F32, H, n, "x")
    L.lm_ggml_set_input(tx)
    cur = L.lm_ggml_mul(ctx, L.lm_ggml_rms_norm(ctx, tx, eps), tn)
    up = L.lm_ggml_mul_mat(ctx, tu, cur)
    gate = L.lm_ggml_mul_mat(ctx, tg, cur)
    act = L.lm_ggml_mul(ctx, L.lm_ggml_silu(ctx, gate), up)
    down = L.lm_ggml_mul_mat(ctx, td, act)
    out = L.lm_ggml_add(ctx, down, tx)
    L.lm_ggml_set_output(out)
    g = L.lm_ggml_new_graph(ctx)
    L.lm_ggml_build_forward_expand(g, out)
    backends = (C.c_void_p * 2)(hip, cpu)
    sched = L.lm_ggml_backend_sched_new(backends, None, 2, 64, False, True)
    assert L.lm_ggml_backend_sched_alloc_graph(sched, g)
    host.set(tx, x)
    blib = C.CDLL(cactus_amd.BACKEND_LIB)
    blib.lm_ggml_backend_hip_get_fused_pairs.restype = C.c_ulonglong
    fused_before = blib.lm_ggml_backend_hip_get_fused_pairs()
    blib.lm_ggml_backend_hip_get_quantizers_skipped.restype = C.c_ulonglong
    skipped_before = blib.lm_ggml_backend_hip_get_quantizers_skipped()
    blib.lm_ggml_backend_hip_get_gated_pairs.restype = C.c_ulonglong
    gated_before = blib.lm_ggml_backend_hip_get_gated_pairs()
    blib.lm_ggml_backend_hip_get_norms_in_prologue.restype = C.c_ulonglong
    norms_before = blib.lm_ggml_backend_hip_get_norms_in_prologue()
    blib.lm_ggml_backend_hip_get_residual_adds.restype = C.c_ulonglong
    adds_before = blib.lm_ggml_backend_hip_get_residual_adds()
    assert L.lm_ggml_backend_sched_graph_compute(sched, g) == 0
    # norm + weight ran as one kernel (the allocator writes the MUL over its only producer); SiLU and its MUL are not
    # neighbours in the node order (the up projection sits between them): the SiLU waits for that matmul and runs in the
    # MUL's kernel
    # 5 tokens: the norm leaves its result quantized in the workspace, so neither gate nor up runs the quantizer, and
    # SiLU * up leaves its result quantized for ffn_down, which runs no quantizer of its own.
    # 2 tokens: gate, SiLU, up and the MUL run as one launch of the GEMV that quantizes in its prologue (three joins), with
    # the norm and its weight MUL (one join) in that prologue too; ffn_down's GEMV quantizes in its own prologue and adds the
    # residual as it stores (one join): two launches for the eight nodes.
    assert blib.lm_ggml_backend_hip_get_fused_pairs() - fused_before == (2 if n > 4 else 5)
    assert blib.lm_ggml_backend_hip_get_quantizers_skipped() - skipped_before == (3 if n > 4 else 0)
    assert blib.lm_ggml_backend_hip_get_gated_pairs() - gated_before == (0 if n > 4 else 1)
    assert blib.lm_ggml_backend_hip_get_norms_in_prologue() - norms_before == (0 if n > 4 else 1)
    assert blib.lm_ggml_backend_hip_get_residual_adds() - adds_before == (0 if n > 4 else 1)
    assert L.lm_ggml_backend_sched_get_n_splits(sched) == 1
    for t in (cur, up, gate, act, down, out):
        assert L.lm_ggml_backend_sched_get_tensor_backend(sched, t) == hip
    y = host.get(out, np.float32, (n, H))
    # the same chain on the oracle (the reference's CPU arithmetic)
    c0 = orc.rms_norm(x, eps) * wn
    u = orc.mul_mat(O.Q4_K, wu, c0)["y"]
    gt = orc.mul_mat(O.Q4_K, wg, c0)["y"]
    a = orc.silu(gt) * u
    d = orc.mul_mat(O.Q6_K, wd, a, want=("sum_abs",))
    want = d["y"] + x
    # up / gate carry the GPU's summation order (<= 1e-5 of their yardstick); the Q8_K requantization of `act` passes
    # that on, so compare at a tolerance for two chained matmuls
    assert (np.abs(y - want) <= 2e-3 * d["sum_abs"] + 1e-6).all()
    L.lm_ggml_backend_sched_free(sched)
    L.lm_ggml_backend_buffer_free(wbuf)
    L.lm_ggml_backend_free(hip)
    L.lm_ggml_backend_free(cpu)
    L.lm_ggml_free(ctx)
    L.lm_ggml_free(wctx)


def test_residual_add_runs_with_the_norm_that_follows(host, orc):
    """ADD -> RMS_NORM -> MUL (a residual and the next block's norm, reference llama-model.cpp build_llama: "ffn_inp" / "l_out"
    followed by build_norm) runs as one kernel, ADD -> RMS_NORM as one kernel, and the sums stay available to the later
    residuals; all element-wise, so the result equals the CPU arithmetic bit for bit."""
    import cactus_amd
    L = host.L
    H, n = 2048, 6
    eps = 1e-5
    rng = np.random.default_rng(8)
    wn = (1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    x, z = common.activations_f32(31, n, H), common.activations_f32(32, n, H)
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    hip = L.lm_ggml_backend_dev_init(dev, None)
    cpu = L.lm_ggml_backend_cpu_init()
    wctx = host.context(with_graph=False)
    tn = L.lm_ggml_new_tensor_1d(wctx, O.F32, H)
    wbuf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(wctx, L.lm_ggml_backend_dev_buffer_type(dev))
    L.lm_ggml_backend_buffer_set_usage(wbuf, 1)
    host.set(tn, wn)
    ctx = host.context()
    tx = host.tensor_2d(ctx, O.F32, H, n, "x")
    tz = host.tensor_2d(ctx, O.F32, H, n, "z")
    L.lm_ggml_set_input(tx); L.lm_ggml_set_input(tz)
    h1 = L.lm_ggml_add(ctx, tx, tz)
    c1 = L.lm_ggml_mul(ctx, L.lm_ggml_rms_norm(ctx, h1, eps), tn)
    h2 = L.lm_ggml_add(ctx, c1, h1)
    o = L.lm_ggml_rms_norm(ctx, h2, eps)
    out = L.lm_ggml_add(ctx, o, h2)
    L.lm_ggml_set_output(out)
    g = L.lm_ggml_new_graph(ctx)
    L.lm_ggml_build_forward_expand(g, out)
    backends = (C.c_void_p * 2)(hip, cpu)
    sched = L.lm_ggml_backend_sched_new(backends, None, 2, 64, False, True)
    for t in (h1, c1, h2, o, out):
        L.lm_ggml_backend_sched_set_tensor_backend(sched, t, hip)
    assert L.lm_ggml_backend_sched_alloc_graph(sched, g)
    host.set(tx, x); host.set(tz, z)
    blib = C.CDLL(cactus_amd.BACKEND_LIB)
    blib.lm_ggml_backend_hip_get_fused_pairs.restype = C.c_ulonglong
    fused_before = blib.lm_ggml_backend_hip_get_fused_pairs()
    assert L.lm_ggml_backend_sched_graph_compute(sched, g) == 0
    assert blib.lm_ggml_backend_hip_get_fused_pairs() - fused_before == 3          # (add, norm, mul) = 2 joins, (add, norm) = 1
    y = host.get(out, np.float32, (n, H))
    s1 = x + z
    s2 = orc.rms_norm(s1, eps) * wn + s1
    want = orc.rms_norm(s2, eps) + s2
    assert y.tobytes() == want.tobytes()
    L.lm_ggml_backend_sched_free(sched)
    L.lm_ggml_backend_buffer_free(wbuf)
    L.lm_ggml_backend_free(hip)
    L.lm_ggml_backend_free(cpu)
    L.lm_ggml_free(ctx)
    L.lm_ggml_free(wctx)


def test_shared_quantized_input_is_dropped_when_the_input_is_overwritten(host, orc):
    """Two matmuls read the same tensor, but an in-place SCALE rewrites it between them: the second matmul must quantize
    again (same data pointer, same shape - only the write in between tells).  A third one after it reuses the new rows."""
    import cactus_amd
    L = host.L
    L.lm_ggml_scale_inplace.restype = C.c_void_p
    L.lm_ggml_scale_inplace.argtypes = [C.c_void_p, C.c_void_p, C.c_float]
    K, N, n = 1024, 300, 6
    w1 = orc.quantize_weights(O.Q4_K, common.weights_f32(91, N, K))
    w2 = orc.quantize_weights(O.Q6_K, common.weights_f32(92, N, K))
    x = common.activations_f32(93, n, K)
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    be = L.lm_ggml_backend_dev_init(dev, None)
    ctx = host.context()
    t1 = host.tensor_2d(ctx, O.Q4_K, K, N, "w1")
    t2 = host.tensor_2d(ctx, O.Q6_K, K, N, "w2")
    tx = host.tensor_2d(ctx, O.F32, K, n, "x")
    y1 = L.lm_ggml_mul_mat(ctx, t1, tx)
    xs = L.lm_ggml_scale_inplace(ctx, tx, 3.0)
    y2 = L.lm_ggml_mul_mat(ctx, t2, xs)
    y3 = L.lm_ggml_mul_mat(ctx, t1, xs)
    g = L.lm_ggml_new_graph(ctx)
    for t in (y1, y2, y3):
        L.lm_ggml_build_forward_expand(g, t)
    buf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(ctx, L.lm_ggml_backend_dev_buffer_type(dev))
    host.set(t1, w1); host.set(t2, w2); host.set(tx, x)
    blib = C.CDLL(cactus_amd.BACKEND_LIB)
    blib.lm_ggml_backend_hip_get_quantizers_skipped.restype = C.c_ulonglong
    before = blib.lm_ggml_backend_hip_get_quantizers_skipped()
    assert L.lm_ggml_backend_graph_compute(be, g) == 0
    assert blib.lm_ggml_backend_hip_get_quantizers_skipped() - before == 1                 # y3 only
    x3 = x * np.float32(3.0)
    for t, wt, w, xin in ((y1, O.Q4_K, w1, x), (y2, O.Q6_K, w2, x3), (y3, O.Q4_K, w1, x3)):
        ref = orc.mul_mat(wt, w, xin, nthreads=8, want=("sum_abs",))
        y = host.get(t, np.float32, (n, N))
        assert (np.abs(y.astype(np.float64) - ref["y"]) <= REL_TOL * ref["sum_abs"]).all()
    L.lm_ggml_backend_buffer_free(buf)
    L.lm_ggml_backend_free(be)
    L.lm_ggml_free(ctx)


def test_cache_store_is_not_run_early_past_a_reader_of_its_destination(host, orc):
    """Between a RoPE and the CPY of its result into the cache lies a node that reads that cache region: the store must
    stay where it is (the reader sees the old contents).  Without the reader the same store runs in the RoPE's kernel."""
    import cactus_amd
    L = host.L
    hd, n_head, n_tok = 64, 4, 3
    E = hd * n_head * n_tok
    rng = np.random.default_rng(4)
    x = rng.standard_normal((n_tok, n_head, hd)).astype(np.float32)
    pos = np.array([3, 4, 5], np.int32)
    old = (rng.standard_normal(E) * 0.5).astype(np.float16)
    blib = C.CDLL(cactus_amd.BACKEND_LIB)
    blib.lm_ggml_backend_hip_get_fused_pairs.restype = C.c_ulonglong
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    for with_reader in (True, False):
        be = L.lm_ggml_backend_dev_init(dev, None)
        ctx = host.context()
        tx = host.tensor_3d(ctx, O.F32, hd, n_head, n_tok, "x")
        tp = L.lm_ggml_new_tensor_1d(ctx, 26, n_tok)
        kc = L.lm_ggml_new_tensor_1d(ctx, O.F16, E)
        seen = L.lm_ggml_new_tensor_1d(ctx, O.F32, E)
        r = L.lm_ggml_rope_ext(ctx, tx, tp, None, hd, 2, 4096, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0)
        reader = L.lm_ggml_cpy(ctx, L.lm_ggml_view_1d(ctx, kc, E, 0), seen)
        store = L.lm_ggml_cpy(ctx, r, L.lm_ggml_view_1d(ctx, kc, E, 0))
        g = L.lm_ggml_new_graph(ctx)
        for t in ((r, reader, store) if with_reader else (r, store)):
            L.lm_ggml_build_forward_expand(g, t)
        buf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(ctx, L.lm_ggml_backend_dev_buffer_type(dev))
        host.set(tx, x); host.set(tp, pos); host.set(kc, old)
        before = blib.lm_ggml_backend_hip_get_fused_pairs()
        assert L.lm_ggml_backend_graph_compute(be, g) == 0
        assert blib.lm_ggml_backend_hip_get_fused_pairs() - before == (0 if with_reader else 1)
        want = orc.rope(x, pos, hd, 2)
        got = host.get(kc, np.float16, (E,)).astype(np.float32)
        assert (np.abs(got - want.reshape(-1)) <= 2 * np.spacing(np.abs(want.reshape(-1)).astype(np.float16)).astype(np.float32) + 1e-3).all()
        if with_reader:
            assert host.get(seen, np.float32, (E,)).tobytes() == old.astype(np.float32).tobytes()
        L.lm_ggml_backend_buffer_free(buf)
        L.lm_ggml_backend_free(be)
        L.lm_ggml_free(ctx)


def test_gelu_and_scale_nodes(host, orc):
    """A GELU-gated FFN entry and a SCALE (Gemma-style graphs: lm_ggml_gelu, lm_ggml_scale): both run on the device, and the
    GELU goes through the host framework's own table, so the result equals the reference CPU backend bit for bit."""
    L = host.L
    L.lm_ggml_gelu.restype = C.c_void_p
    L.lm_ggml_gelu.argtypes = [C.c_void_p, C.c_void_p]
    L.lm_ggml_scale.restype = C.c_void_p
    L.lm_ggml_scale.argtypes = [C.c_void_p, C.c_void_p, C.c_float]
    n, ne0 = 5, 1152
    x = (common.activations_f32(77, n, ne0) * 3).astype(np.float32)
    u = common.activations_f32(78, n, ne0)
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    hip = L.lm_ggml_backend_dev_init(dev, None)
    cpu = L.lm_ggml_backend_cpu_init()
    ctx = host.context()
    tx = host.tensor_2d(ctx, O.F32, ne0, n, "x")
    tu = host.tensor_2d(ctx, O.F32, ne0, n, "u")
    L.lm_ggml_set_input(tx); L.lm_ggml_set_input(tu)
    gl = L.lm_ggml_gelu(ctx, tx)
    act = L.lm_ggml_mul(ctx, gl, tu)
    out = L.lm_ggml_scale(ctx, act, 0.0625)
    L.lm_ggml_set_output(out)
    g = L.lm_ggml_new_graph(ctx)
    L.lm_ggml_build_forward_expand(g, out)
    for t in (gl, act, out):
        assert L.lm_ggml_backend_dev_supports_op(dev, t) is True
    backends = (C.c_void_p * 2)(hip, cpu)
    sched = L.lm_ggml_backend_sched_new(backends, None, 2, 64, False, True)
    for t in (gl, act, out):
        L.lm_ggml_backend_sched_set_tensor_backend(sched, t, hip)
    assert L.lm_ggml_backend_sched_alloc_graph(sched, g)
    host.set(tx, x); host.set(tu, u)
    assert L.lm_ggml_backend_sched_graph_compute(sched, g) == 0
    y = host.get(out, np.float32, (n, ne0))
    want = orc.scale(orc.gelu(x) * u, 0.0625)
    assert y.tobytes() == want.tobytes()
    L.lm_ggml_backend_sched_free(sched)
    L.lm_ggml_backend_free(hip)
    L.lm_ggml_backend_free(cpu)
    L.lm_ggml_free(ctx)


def test_attention_side_nodes_run_on_the_device(host, orc):
    """The nodes llama.cpp puts around the KV cache (reference llama-graph.cpp:1060-1166, llama-kv-cache.cpp:617-656): RoPE of
    Q and K, the K store (F32 -> F16 into a 1-D view of the cache), the transposed V store, the masked soft-max and the
    permuted attention output made dense.  With the caches in a HIP buffer the reference scheduler gives the stores
    (and the RoPE that feeds them) to the HIP backend by itself; results against the oracle."""
    L = host.L
    hd, n_head, n_head_kv, n_tokens, kv_size, head, n_kv = 64, 8, 2, 5, 256, 37, 64
    n_embd_kv = hd * n_head_kv
    rng = np.random.default_rng(12)
    q_in = rng.standard_normal((n_tokens, n_head * hd)).astype(np.float32)
    k_in = rng.standard_normal((n_tokens, n_embd_kv)).astype(np.float32)
    v_in = rng.standard_normal((n_tokens, n_embd_kv)).astype(np.float32)
    kq_in = (rng.standard_normal((n_head, n_tokens, n_kv)) * 4).astype(np.float32)
    kqv_in = rng.standard_normal((n_head, n_tokens, hd)).astype(np.float32)
    pos = np.arange(head, head + n_tokens, dtype=np.int32)
    mask = np.full((8, n_kv), -np.inf, np.float32)                       # token rows padded to 8
    for i in range(n_tokens):
        mask[i, : head + i + 1] = 0.0
    mask16 = mask.astype(np.float16)
    scale = 1.0 / np.sqrt(hd)

    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    hip = L.lm_ggml_backend_dev_init(dev, None)
    cpu = L.lm_ggml_backend_cpu_init()
    cctx = host.context(with_graph=False)
    kc = host.tensor_2d(cctx, O.F16, n_embd_kv, kv_size, "cache_k")
    vc = host.tensor_2d(cctx, O.F16, kv_size, n_embd_kv, "cache_v")       # transposed V cache
    cbuf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(cctx, L.lm_ggml_backend_dev_buffer_type(dev))
    L.lm_ggml_backend_buffer_clear(cbuf, 0)

    ctx = host.context(n_tensors=64)
    tq = host.tensor_2d(ctx, O.F32, n_head * hd, n_tokens, "q_in")
    tk = host.tensor_2d(ctx, O.F32, n_embd_kv, n_tokens, "k_in")
    tv = host.tensor_2d(ctx, O.F32, n_embd_kv, n_tokens, "v_in")
    tkq = host.tensor_3d(ctx, O.F32, n_kv, n_tokens, n_head, "kq_in")
    tkqv = host.tensor_3d(ctx, O.F32, hd, n_tokens, n_head, "kqv_in")
    tpos = L.lm_ggml_new_tensor_1d(ctx, 26, n_tokens)
    tmask = host.tensor_2d(ctx, O.F16, n_kv, 8, "mask")
    for t in (tq, tk, tv, tkq, tkqv, tpos, tmask):
        L.lm_ggml_set_input(t)
    rope = lambda t, nh: L.lm_ggml_rope_ext(ctx, L.lm_ggml_reshape_3d(ctx, t, hd, nh, n_tokens), tpos, None, hd, 2, 4096, 10000.0, 1.0,
                                         0.0, 1.0, 32.0, 1.0)
    q = rope(tq, n_head)
    k = rope(tk, n_head_kv)
    k_store = L.lm_ggml_cpy(ctx, k, L.lm_ggml_view_1d(ctx, kc, n_tokens * n_embd_kv, 2 * n_embd_kv * head))
    v_store = L.lm_ggml_cpy(ctx, L.lm_ggml_transpose(ctx, tv), L.lm_ggml_view_2d(ctx, vc, n_tokens, n_embd_kv, kv_size * 2, head * 2))
    sm = L.lm_ggml_soft_max_ext(ctx, tkq, tmask, scale, 0.0)
    out = L.lm_ggml_cont_2d(ctx, L.lm_ggml_permute(ctx, tkqv, 0, 2, 1, 3), hd * n_head, n_tokens)
    g = L.lm_ggml_new_graph(ctx)
    for t in (q, k_store, v_store, sm, out):
        L.lm_ggml_set_output(t)
        L.lm_ggml_build_forward_expand(g, t)
    backends = (C.c_void_p * 2)(hip, cpu)
    sched = L.lm_ggml_backend_sched_new(backends, None, 2, 128, False, True)
    # in a model these nodes sit between HIP matmuls; here their inputs come from the host, so pin them like the reference
    # pins its attention nodes (llama-graph.cpp:1165-1168)
    for t in (q, sm, out):
        L.lm_ggml_backend_sched_set_tensor_backend(sched, t, hip)
    assert L.lm_ggml_backend_sched_alloc_graph(sched, g)
    for t, a in ((tq, q_in), (tk, k_in), (tv, v_in), (tkq, kq_in), (tkqv, kqv_in), (tpos, pos), (tmask, mask16)):
        host.set(t, a)
    assert L.lm_ggml_backend_sched_graph_compute(sched, g) == 0
    for t in (k_store, v_store):
        assert L.lm_ggml_backend_sched_get_tensor_backend(sched, t) == hip     # stores into a HIP buffer must run there
    y_q = host.get(q, np.float32, (n_tokens, n_head, hd))
    y_sm = host.get(sm, np.float32, (n_head, n_tokens, n_kv))
    y_out = host.get(out, np.float32, (n_tokens, n_head * hd))
    y_kc = host.get(kc, np.float16, (kv_size, n_embd_kv))
    y_vc = host.get(vc, np.float16, (n_embd_kv, kv_size))

    q3 = q_in.reshape(n_tokens, n_head, hd)
    want_q = orc.rope(q3, pos, hd, 2)
    tol = 4e-7 * (np.abs(q3[..., : hd // 2]) + np.abs(q3[..., hd // 2:]))
    assert (np.abs(y_q - want_q) <= np.concatenate([tol, tol], -1)).all()
    want_k = orc.rope(k_in.reshape(n_tokens, n_head_kv, hd), pos, hd, 2).reshape(n_tokens, n_embd_kv)
    want_kc = np.zeros((kv_size, n_embd_kv), np.float16)
    want_kc[head:head + n_tokens] = want_k.astype(np.float16)
    # the stored K went through the device's RoPE: equal to the oracle's within one fp16 step where the fp32 values straddle a tie
    assert (np.abs(y_kc.astype(np.float32) - want_kc.astype(np.float32)) <= np.spacing(np.abs(want_kc)).astype(np.float32)).all()
    assert (y_kc[:head] == 0).all() and (y_kc[head + n_tokens:] == 0).all()
    want_vc = np.zeros((n_embd_kv, kv_size), np.float16)
    want_vc[:, head:head + n_tokens] = v_in.T.astype(np.float16)
    assert y_vc.tobytes() == want_vc.tobytes()
    want_sm = orc.soft_max(kq_in, mask16, scale)
    assert y_sm.tobytes() == want_sm.tobytes()
    assert y_out.tobytes() == np.ascontiguousarray(kqv_in.transpose(1, 0, 2)).tobytes()
    for t in (q, k, sm, out):
        assert L.lm_ggml_backend_sched_get_tensor_backend(sched, t) == hip
    # the next step: the same graph and the same tensors at the same addresses, other positions - the cos / sin table of
    # the previous call must not be used again
    pos2 = pos + 1000
    host.set(tpos, pos2)
    assert L.lm_ggml_backend_sched_graph_compute(sched, g) == 0
    y_q2 = host.get(q, np.float32, (n_tokens, n_head, hd))
    assert (np.abs(y_q2 - orc.rope(q3, pos2, hd, 2)) <= np.concatenate([tol, tol], -1)).all()
    assert not np.array_equal(y_q2, y_q)
    L.lm_ggml_backend_sched_free(sched)
    L.lm_ggml_backend_buffer_free(cbuf)
    L.lm_ggml_backend_free(hip)
    L.lm_ggml_backend_free(cpu)
    L.lm_ggml_free(ctx)
    L.lm_ggml_free(cctx)


def test_attention_side_ops_outside_the_restated_cases_are_declined(host):
    """supports_op says no to what the kernels do not restate: ALiBi slopes, rows that are not a multiple of 8 values,
    multi-section RoPE, copies into quantized tensors."""
    L = host.L
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    ctx = host.context()
    x = host.tensor_3d(ctx, O.F32, 64, 4, 2)
    m = host.tensor_2d(ctx, O.F32, 64, 4)
    assert L.lm_ggml_backend_dev_supports_op(dev, L.lm_ggml_soft_max_ext(ctx, x, m, 1.0, 0.0))
    assert not L.lm_ggml_backend_dev_supports_op(dev, L.lm_ggml_soft_max_ext(ctx, x, m, 1.0, 8.0))
    x2 = host.tensor_3d(ctx, O.F32, 60, 4, 2)
    assert not L.lm_ggml_backend_dev_supports_op(dev, L.lm_ggml_soft_max_ext(ctx, x2, None, 1.0, 0.0))
    pos = L.lm_ggml_new_tensor_1d(ctx, 26, 2)
    assert L.lm_ggml_backend_dev_supports_op(dev, L.lm_ggml_rope_ext(ctx, x, pos, None, 64, 0, 4096, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0))
    assert not L.lm_ggml_backend_dev_supports_op(dev, L.lm_ggml_rope_ext(ctx, x, pos, None, 32, 24, 4096, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0))
    q = host.tensor_2d(ctx, O.Q8_0, 64, 8)
    x3 = host.tensor_2d(ctx, O.F32, 64, 8)
    assert not L.lm_ggml_backend_dev_supports_op(dev, L.lm_ggml_cpy(ctx, x3, q))
    h = host.tensor_2d(ctx, O.F16, 64, 8)
    assert L.lm_ggml_backend_dev_supports_op(dev, L.lm_ggml_cpy(ctx, x3, h))
    L.lm_ggml_free(ctx)


@pytest.mark.parametrize("n_tokens", [5, 2])
def test_attention_block_stays_on_the_device(host, orc, n_tokens):
    """A whole attention block as llama.cpp builds it without flash attention (reference llama-graph.cpp build_norm, build_attn /
    build_attn_mha :1060-1170, llama-kv-cache.cpp get_k / get_v / cpy_k / cpy_v): attn_norm, q/k/v projections, RoPE, the cache stores,
    kq over the F16 K cache, masked soft-max, kqv over the transposed F16 V cache, the merge of the heads, the output
    projection and the residual.  Weights and caches live in HIP buffers: the reference scheduler puts everything into
    one HIP split."""
    L = host.L
    H, hd, n_head, n_head_kv, kv_size, head, n_kv = 1024, 64, 16, 4, 256, 59, 64
    n_embd_kv = hd * n_head_kv
    rng = np.random.default_rng(31)
    wq = orc.quantize_weights(O.Q4_K, common.weights_f32(41, n_head * hd, H))
    wk = orc.quantize_weights(O.Q4_K, common.weights_f32(42, n_embd_kv, H))
    wv = orc.quantize_weights(O.Q6_K, common.weights_f32(43, n_embd_kv, H))
    wo = orc.quantize_weights(O.Q4_K, common.weights_f32(44, H, n_head * hd))
    x = common.activations_f32(45, n_tokens, H)
    wn = (1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    eps = 1e-5
    pos = np.arange(head, head + n_tokens, dtype=np.int32)
    mask = np.full((8, n_kv), -np.inf, np.float32)
    for i in range(n_tokens):
        mask[i, : head + i + 1] = 0.0
    mask16 = mask.astype(np.float16)
    scale = 1.0 / np.sqrt(hd)
    # what the cache holds from earlier tokens
    k_old = (rng.standard_normal((head, n_embd_kv)) * 0.5).astype(np.float16)
    v_old = (rng.standard_normal((head, n_embd_kv)) * 0.5).astype(np.float16)
    kc0 = np.zeros((kv_size, n_embd_kv), np.float16)
    kc0[:head] = k_old
    vc0 = np.zeros((n_embd_kv, kv_size), np.float16)
    vc0[:, :head] = v_old.T

    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    hip = L.lm_ggml_backend_dev_init(dev, None)
    cpu = L.lm_ggml_backend_cpu_init()
    wctx = host.context(with_graph=False)
    tn = L.lm_ggml_new_tensor_1d(wctx, O.F32, H)
    twq = host.tensor_2d(wctx, O.Q4_K, H, n_head * hd, "wq")
    twk = host.tensor_2d(wctx, O.Q4_K, H, n_embd_kv, "wk")
    twv = host.tensor_2d(wctx, O.Q6_K, H, n_embd_kv, "wv")
    two = host.tensor_2d(wctx, O.Q4_K, n_head * hd, H, "wo")
    wbuf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(wctx, L.lm_ggml_backend_dev_buffer_type(dev))
    L.lm_ggml_backend_buffer_set_usage(wbuf, 1)
    for t, a in ((twq, wq), (twk, wk), (twv, wv), (two, wo), (tn, wn)):
        host.set(t, a)
    cctx = host.context(with_graph=False)
    kc = host.tensor_2d(cctx, O.F16, n_embd_kv, kv_size, "cache_k")
    vc = host.tensor_2d(cctx, O.F16, n_embd_kv, kv_size, "cache_v")       # allocated like the reference; used transposed
    cbuf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(cctx, L.lm_ggml_backend_dev_buffer_type(dev))
    host.set(kc, kc0)
    host.set(vc, vc0)

    ctx = host.context(n_tensors=96)
    tx = host.tensor_2d(ctx, O.F32, H, n_tokens, "x")
    tpos = L.lm_ggml_new_tensor_1d(ctx, 26, n_tokens)
    tmask = host.tensor_2d(ctx, O.F16, n_kv, 8, "mask")
    for t in (tx, tpos, tmask):
        L.lm_ggml_set_input(t)
    rope = lambda t, nh: L.lm_ggml_rope_ext(ctx, L.lm_ggml_reshape_3d(ctx, t, hd, nh, n_tokens), tpos, None, hd, 2, 4096, 10000.0, 1.0,
                                         0.0, 1.0, 32.0, 1.0)
    cur = L.lm_ggml_mul(ctx, L.lm_ggml_rms_norm(ctx, tx, eps), tn)
    q = rope(L.lm_ggml_mul_mat(ctx, twq, cur), n_head)
    k = rope(L.lm_ggml_mul_mat(ctx, twk, cur), n_head_kv)
    v = L.lm_ggml_mul_mat(ctx, twv, cur)
    k_store = L.lm_ggml_cpy(ctx, k, L.lm_ggml_view_1d(ctx, kc, n_tokens * n_embd_kv, 2 * n_embd_kv * head))
    v_store = L.lm_ggml_cpy(ctx, L.lm_ggml_transpose(ctx, v), L.lm_ggml_view_2d(ctx, vc, n_tokens, n_embd_kv, kv_size * 2, head * 2))
    kview = L.lm_ggml_view_3d(ctx, kc, hd, n_head_kv, n_kv, 2 * hd, 2 * n_embd_kv, 0)
    vview = L.lm_ggml_view_3d(ctx, vc, n_kv, n_head_kv, hd, 2 * kv_size * hd, 2 * kv_size, 0)
    qp = L.lm_ggml_permute(ctx, q, 0, 2, 1, 3)
    kp = L.lm_ggml_permute(ctx, kview, 0, 2, 1, 3)
    vp = L.lm_ggml_permute(ctx, vview, 0, 2, 1, 3)
    kq = L.lm_ggml_mul_mat(ctx, kp, qp)
    sm = L.lm_ggml_soft_max_ext(ctx, kq, tmask, scale, 0.0)
    kqv = L.lm_ggml_mul_mat(ctx, vp, sm)
    merged = L.lm_ggml_cont_2d(ctx, L.lm_ggml_permute(ctx, kqv, 0, 2, 1, 3), hd * n_head, n_tokens)
    out = L.lm_ggml_add(ctx, L.lm_ggml_mul_mat(ctx, two, merged), tx)
    L.lm_ggml_set_output(out)
    g = L.lm_ggml_new_graph(ctx)
    for t in (q, k, v, k_store, v_store, out):           # q, k, v first, then the two stores, as the reference builds its graph
        L.lm_ggml_build_forward_expand(g, t)              # (llama-graph.cpp:1265-1277)
    backends = (C.c_void_p * 2)(hip, cpu)
    sched = L.lm_ggml_backend_sched_new(backends, None, 2, 128, False, True)
    assert L.lm_ggml_backend_sched_alloc_graph(sched, g)
    host.set(tx, x); host.set(tpos, pos); host.set(tmask, mask16)
    import cactus_amd
    blib = C.CDLL(cactus_amd.BACKEND_LIB)
    blib.lm_ggml_backend_hip_get_rope_tables.restype = C.c_ulonglong
    tables_before = blib.lm_ggml_backend_hip_get_rope_tables()
    blib.lm_ggml_backend_hip_get_fused_pairs.restype = C.c_ulonglong
    fused_before = blib.lm_ggml_backend_hip_get_fused_pairs()
    blib.lm_ggml_backend_hip_get_grouped_matmuls.restype = C.c_ulonglong
    grouped_before = blib.lm_ggml_backend_hip_get_grouped_matmuls()
    blib.lm_ggml_backend_hip_get_rope_pairs.restype = C.c_ulonglong
    pairs_before = blib.lm_ggml_backend_hip_get_rope_pairs()
    blib.lm_ggml_backend_hip_get_rope_epilogues.restype = C.c_ulonglong
    epilogues_before = blib.lm_ggml_backend_hip_get_rope_epilogues()
    blib.lm_ggml_backend_hip_get_residual_adds.restype = C.c_ulonglong
    adds_before = blib.lm_ggml_backend_hip_get_residual_adds()
    blib.lm_ggml_backend_hip_get_norms_in_prologue.restype = C.c_ulonglong
    norms_before = blib.lm_ggml_backend_hip_get_norms_in_prologue()
    assert L.lm_ggml_backend_sched_graph_compute(sched, g) == 0
    assert blib.lm_ggml_backend_hip_get_rope_tables() - tables_before == 1      # Q and K share one cos / sin table
    # The K store ran in the kernel of K's RoPE.  With up to 4 tokens the transposed V store ran in the V projection's
    # launch, and the three projections ran as one launch: one whose own memory the graph allocator placed over a tensor
    # that is still read in between (Kcur over Qcur, which dies at its RoPE, say) wrote into a slot of the backend's instead.
    grouped = blib.lm_ggml_backend_hip_get_grouped_matmuls() - grouped_before
    assert grouped == (0 if n_tokens > 4 else 3), grouped
    fused = blib.lm_ggml_backend_hip_get_fused_pairs() - fused_before
    # Up to 4 tokens the RoPE of Q and of K (with K's store) ran in the epilogue of their projections, so no ROPE kernel at all
    pairs = blib.lm_ggml_backend_hip_get_rope_pairs() - pairs_before
    epilogues = blib.lm_ggml_backend_hip_get_rope_epilogues() - epilogues_before
    assert (epilogues, pairs) == ((0, 0) if n_tokens > 4 else (2, 0)), (epilogues, pairs, grouped)
    adds = blib.lm_ggml_backend_hip_get_residual_adds() - adds_before        # up to 4 tokens wo's GEMV adds the residual as it stores
    assert adds == (0 if n_tokens > 4 else 1), adds
    # attn_norm and its weight MUL are one join at every token count; up to 4 tokens they ran in the prologue of the group launch
    norms = blib.lm_ggml_backend_hip_get_norms_in_prologue() - norms_before
    assert norms == (0 if n_tokens > 4 else 1), norms
    assert fused == 1 + (1 if n_tokens > 4 else 2 + max(grouped - 1, 0) + epilogues + adds), (fused, grouped, epilogues, adds)
    assert L.lm_ggml_backend_sched_get_n_splits(sched) == 1
    for t in (cur, q, k, v, k_store, v_store, kq, sm, kqv, merged, out):
        assert L.lm_ggml_backend_sched_get_tensor_backend(sched, t) == hip
    y = host.get(out, np.float32, (n_tokens, H))
    y_kc = host.get(kc, np.float16, (kv_size, n_embd_kv))
    y_vc = host.get(vc, np.float16, (n_embd_kv, kv_size))

    # the same chain on the oracle
    c_ = orc.rms_norm(x, eps) * wn
    q_ = orc.rope(orc.mul_mat(O.Q4_K, wq, c_)["y"].reshape(n_tokens, n_head, hd), pos, hd, 2)
    k_ = orc.rope(orc.mul_mat(O.Q4_K, wk, c_)["y"].reshape(n_tokens, n_head_kv, hd), pos, hd, 2)
    v_ = orc.mul_mat(O.Q6_K, wv, c_)["y"]
    kc_ = kc0.copy()
    kc_[head:head + n_tokens] = k_.reshape(n_tokens, n_embd_kv).astype(np.float16)
    vc_ = vc0.copy()
    vc_[:, head:head + n_tokens] = v_.T.astype(np.float16)
    # the stored rows went through the device's matmul and RoPE (tolerances of their own): within two fp16 steps
    step = lambda a: 2 * np.spacing(np.abs(a).astype(np.float16)).astype(np.float32) + 1e-3
    assert (np.abs(y_kc.astype(np.float32) - kc_.astype(np.float32)) <= step(kc_)).all()
    assert (np.abs(y_vc.astype(np.float32) - vc_.astype(np.float32)) <= step(vc_)).all()
    assert y_kc[:head].tobytes() == kc0[:head].tobytes() and (y_kc[head + n_tokens:] == 0).all()
    kq_ = orc.mul_mat_f16_batched(kc_[:n_kv].reshape(n_kv, n_head_kv, hd).transpose(1, 0, 2), q_.transpose(1, 0, 2))["y"]
    sm_ = orc.soft_max(kq_, mask16, scale)
    kqv_ = orc.mul_mat_f16_batched(vc_.reshape(n_head_kv, hd, kv_size)[:, :, :n_kv], sm_)["y"]
    merged_ = np.ascontiguousarray(kqv_.transpose(1, 0, 2)).reshape(n_tokens, n_head * hd)
    o = orc.mul_mat(O.Q4_K, wo, merged_, want=("sum_abs",))
    want = o["y"] + x
    assert (np.abs(y - want) <= 5e-3 * o["sum_abs"] + 1e-5).all()
    L.lm_ggml_backend_sched_free(sched)
    L.lm_ggml_backend_buffer_free(cbuf)
    L.lm_ggml_backend_buffer_free(wbuf)
    L.lm_ggml_backend_free(hip)
    L.lm_ggml_backend_free(cpu)
    L.lm_ggml_free(ctx)
    L.lm_ggml_free(cctx)
    L.lm_ggml_free(wctx)


# (hd, n_head, n_head_kv, n_tokens, n_kv, kv_size): LLaMA-3-8B's block, one token; multi-head attention with 1 and 4 tokens; 8 query
# heads per KV head and two tokens of LLaMA-3-8B, where the matmul takes kernels without the second copy and the CONT runs alone
@pytest.mark.parametrize("hd,n_head,n_head_kv,n_tokens,n_kv,kv_size", [(128, 32, 8, 1, 512, 1024), (128, 32, 8, 1, 4096, 4096),
                                                                      (64, 4, 4, 1, 1000, 1024), (64, 4, 4, 4, 136, 256),
                                                                      (128, 16, 2, 1, 512, 512), (128, 32, 8, 2, 520, 1024)])
def test_kqv_writes_the_head_merge_that_follows_it(host, hd, n_head, n_head_kv, n_tokens, n_kv, kv_size):
    """kq -> soft-max -> kqv -> merge (reference llama-graph.cpp:1120-1160) through the scheduler: with up to 4 (query head, token)
    pairs per KV head the CONT runs inside the kqv matmul's launch, and the merged rows have the bits of the four ops called
    one by one through the C-ABI."""
    import cactus_amd
    L = host.L
    n_embd_kv = hd * n_head_kv
    rng = np.random.default_rng(hd + n_kv)
    kc0 = np.zeros((kv_size, n_embd_kv), np.float16)
    kc0[:n_kv] = rng.standard_normal((n_kv, n_embd_kv)).astype(np.float16)
    vc0 = np.zeros((n_embd_kv, kv_size), np.float16)
    vc0[:, :n_kv] = rng.standard_normal((n_embd_kv, n_kv)).astype(np.float16)
    q0 = rng.standard_normal((n_tokens, n_head, hd)).astype(np.float32)
    mask = np.zeros((8, n_kv), np.float32)
    mask[:n_tokens][rng.random((n_tokens, n_kv)) < 0.25] = -np.inf
    mask[:, 0] = 0.0
    mask16 = mask.astype(np.float16)
    scale = float(1.0 / np.sqrt(hd))

    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    hip = L.lm_ggml_backend_dev_init(dev, None)
    cpu = L.lm_ggml_backend_cpu_init()
    cctx = host.context(with_graph=False)
    kc = host.tensor_2d(cctx, O.F16, n_embd_kv, kv_size, "cache_k")
    vc = host.tensor_2d(cctx, O.F16, n_embd_kv, kv_size, "cache_v")
    cbuf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(cctx, L.lm_ggml_backend_dev_buffer_type(dev))
    host.set(kc, kc0)
    host.set(vc, vc0)
    ctx = host.context(n_tensors=64)
    tq = host.tensor_3d(ctx, O.F32, hd, n_head, n_tokens, "q")
    tmask = host.tensor_2d(ctx, O.F16, n_kv, 8, "mask")
    for t in (tq, tmask):
        L.lm_ggml_set_input(t)
    kview = L.lm_ggml_view_3d(ctx, kc, hd, n_head_kv, n_kv, 2 * hd, 2 * n_embd_kv, 0)
    vview = L.lm_ggml_view_3d(ctx, vc, n_kv, n_head_kv, hd, 2 * kv_size * hd, 2 * kv_size, 0)
    qp = L.lm_ggml_permute(ctx, tq, 0, 2, 1, 3)
    kp = L.lm_ggml_permute(ctx, kview, 0, 2, 1, 3)
    vp = L.lm_ggml_permute(ctx, vview, 0, 2, 1, 3)
    kq = L.lm_ggml_mul_mat(ctx, kp, qp)
    sm = L.lm_ggml_soft_max_ext(ctx, kq, tmask, scale, 0.0)
    kqv = L.lm_ggml_mul_mat(ctx, vp, sm)
    merged = L.lm_ggml_cont_2d(ctx, L.lm_ggml_permute(ctx, kqv, 0, 2, 1, 3), hd * n_head, n_tokens)
    # outputs keep their memory to the end: the allocator cannot place the merged rows over the probabilities, which the matmul's
    # workgroups still read while others already store (the backend checks for that and runs the CONT alone then)
    for t in (merged, kqv, sm):
        L.lm_ggml_set_output(t)
    g = L.lm_ggml_new_graph(ctx)
    L.lm_ggml_build_forward_expand(g, merged)
    backends = (C.c_void_p * 2)(hip, cpu)
    sched = L.lm_ggml_backend_sched_new(backends, None, 2, 128, False, True)
    assert L.lm_ggml_backend_sched_alloc_graph(sched, g)
    host.set(tq, q0); host.set(tmask, mask16)
    blib = C.CDLL(cactus_amd.BACKEND_LIB)
    blib.lm_ggml_backend_hip_get_head_merges.restype = C.c_ulonglong
    before = blib.lm_ggml_backend_hip_get_head_merges()
    assert L.lm_ggml_backend_sched_graph_compute(sched, g) == 0
    taken = (n_head // n_head_kv) * n_tokens <= 4
    assert blib.lm_ggml_backend_hip_get_head_merges() - before == (1 if taken else 0)
    assert L.lm_ggml_backend_sched_get_n_splits(sched) == 1
    y = host.get(merged, np.float32, (n_tokens, n_head, hd))
    y_kqv = host.get(kqv, np.float32, (n_head, n_tokens, hd))

    d = cactus_amd.Device(0)
    kv = kc0[:n_kv].reshape(n_kv, n_head_kv, hd).transpose(1, 0, 2)
    vv = vc0.reshape(n_head_kv, hd, kv_size)[:, :, :n_kv]
    kq_ = d.mul_mat_f16_batched(kv, q0.transpose(1, 0, 2))
    sm_ = d.soft_max(kq_, mask16, scale)
    kqv_ = d.mul_mat_f16_batched(vv, sm_)
    assert y_kqv.tobytes() == kqv_.tobytes()
    assert y.tobytes() == np.ascontiguousarray(kqv_.transpose(1, 0, 2)).tobytes()
    L.lm_ggml_backend_sched_free(sched)
    L.lm_ggml_backend_buffer_free(cbuf)
    L.lm_ggml_backend_free(hip)
    L.lm_ggml_backend_free(cpu)
    L.lm_ggml_free(ctx)
    L.lm_ggml_free(cctx)


def test_get_rows_from_a_device_resident_table(host, orc):
    """LM_GGML_OP_GET_ROWS over a quantized table in a HIP buffer (an embedding matrix kept on the device) runs on the HIP
    backend, bit for bit the reference's dequantized rows; a table in host memory is declined."""
    L = host.L
    L.lm_ggml_get_rows.restype = C.c_void_p
    L.lm_ggml_get_rows.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
    nc, ne01, n = 512, 64, 9
    table = orc.quantize_weights(O.Q6_K, common.weights_f32(71, ne01, nc))
    ids = np.array([3, 0, 63, 17, 17, 5, 44, 1, 2], np.int32)
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    hip = L.lm_ggml_backend_dev_init(dev, None)
    cpu = L.lm_ggml_backend_cpu_init()
    wctx = host.context(with_graph=False)
    tt = host.tensor_2d(wctx, O.Q6_K, nc, ne01, "table")
    wbuf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(wctx, L.lm_ggml_backend_dev_buffer_type(dev))
    L.lm_ggml_backend_buffer_set_usage(wbuf, 1)
    host.set(tt, table)
    ctx = host.context()
    ti = L.lm_ggml_new_tensor_1d(ctx, 26, n)
    L.lm_ggml_set_input(ti)
    rows = L.lm_ggml_get_rows(ctx, tt, ti)
    L.lm_ggml_set_output(rows)
    host_table = host.tensor_2d(ctx, O.Q6_K, nc, ne01, "host_table")        # no buffer yet, not F32 / F16: stays with the CPU
    assert L.lm_ggml_backend_dev_supports_op(dev, rows)
    assert not L.lm_ggml_backend_dev_supports_op(dev, L.lm_ggml_get_rows(ctx, host_table, ti))
    g = L.lm_ggml_new_graph(ctx)
    L.lm_ggml_build_forward_expand(g, rows)
    backends = (C.c_void_p * 2)(hip, cpu)
    sched = L.lm_ggml_backend_sched_new(backends, None, 2, 64, False, True)
    assert L.lm_ggml_backend_sched_alloc_graph(sched, g)
    host.set(ti, ids)
    assert L.lm_ggml_backend_sched_graph_compute(sched, g) == 0
    assert L.lm_ggml_backend_sched_get_tensor_backend(sched, rows) == hip
    y = host.get(rows, np.float32, (n, nc))
    assert y.tobytes() == orc.get_rows(O.Q6_K, table, nc, ids).tobytes()
    L.lm_ggml_backend_sched_free(sched)
    L.lm_ggml_backend_buffer_free(wbuf)
    L.lm_ggml_backend_free(hip)
    L.lm_ggml_backend_free(cpu)
    L.lm_ggml_free(ctx)
    L.lm_ggml_free(wctx)


def test_q6_K_weights_are_read_from_a_copy_in_planes_at_decode(host, orc):
    """A 2-D Q6_K weight of K % 2048 == 0: its first matmul of up to 4 tokens makes the copy in planes and reads it (the same
    bits as the C-ABI gives on the block-order rows), the next one reads the same copy, get_tensor still returns the bytes that
    were set, set_tensor and memset_tensor drop the copy (the matmul after them sees the new weights), and a matmul of 8 tokens
    reads the tensor's own bytes."""
    import cactus_amd
    L = host.L
    K, N = 2048, 520
    w1 = orc.quantize_weights(O.Q6_K, common.weights_f32(81, N, K))
    w2 = orc.quantize_weights(O.Q6_K, common.weights_f32(82, N, K))
    cdev = cactus_amd.Device(0)
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    hip = L.lm_ggml_backend_dev_init(dev, None)
    wctx = host.context(with_graph=False)
    tw = host.tensor_2d(wctx, O.Q6_K, K, N, "w")
    wbuf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(wctx, L.lm_ggml_backend_dev_buffer_type(dev))
    L.lm_ggml_backend_buffer_set_usage(wbuf, 1)
    host.set(tw, w1)
    blib = C.CDLL(cactus_amd.BACKEND_LIB)
    counters = {}
    for name in ("copies", "bytes", "dropped", "matmuls"):
        f = getattr(blib, "lm_ggml_backend_hip_get_planes_" + name)
        f.restype = C.c_ulonglong
        counters[name] = f
    def counts():
        return {k: f() for k, f in counters.items()}
    graphs = {}
    for n in (2, 8):
        ctx = host.context()
        tx = host.tensor_2d(ctx, O.F32, K, n, "x")
        ty = L.lm_ggml_mul_mat(ctx, tw, tx)
        g = L.lm_ggml_new_graph(ctx)
        L.lm_ggml_build_forward_expand(g, ty)
        buf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(ctx, L.lm_ggml_backend_dev_buffer_type(dev))
        graphs[n] = (ctx, tx, ty, g, buf)
    x2, x8 = common.activations_f32(83, 2, K), common.activations_f32(84, 8, K)

    def run(n, x):
        ctx, tx, ty, g, buf = graphs[n]
        host.set(tx, x)
        assert L.lm_ggml_backend_graph_compute(hip, g) == 0
        return host.get(ty, np.float32, (n, N))

    c0 = counts()
    y = run(2, x2)
    c1 = counts()
    assert c1["copies"] - c0["copies"] == 1 and c1["bytes"] - c0["bytes"] == w1.size and c1["matmuls"] - c0["matmuls"] == 1
    assert y.tobytes() == cdev.mul_mat(O.Q6_K, w1, x2).tobytes()
    ref = orc.mul_mat(O.Q6_K, w1, x2, nthreads=8, want=("sum_abs",))
    assert (np.abs(y.astype(np.float64) - ref["y"]) <= REL_TOL * ref["sum_abs"]).all()
    assert run(2, x2).tobytes() == y.tobytes()
    c2 = counts()
    assert c2["copies"] == c1["copies"] and c2["matmuls"] - c1["matmuls"] == 1 and c2["dropped"] == c0["dropped"]
    assert np.array_equal(host.get(tw, np.uint8, w1.shape), w1)                    # the tensor's own bytes stay in block order
    y8 = run(8, x8)
    assert counts() == c2                                                          # 8 tokens: no copy read, none made
    assert y8.tobytes() == cdev.mul_mat(O.Q6_K, w1, x8).tobytes()
    host.set(tw, w2)                                                               # new weights: the copy is stale
    c3 = counts()
    assert c3["dropped"] - c2["dropped"] == 1
    y = run(2, x2)
    assert y.tobytes() == cdev.mul_mat(O.Q6_K, w2, x2).tobytes()
    assert counts()["copies"] - c3["copies"] == 1
    L.lm_ggml_backend_tensor_memset(tw, 0, 0, w2.size)                             # d = 0 in every block
    assert counts()["dropped"] - c3["dropped"] == 1
    assert not run(2, x2).any()
    before_free = counts()["dropped"]
    L.lm_ggml_backend_buffer_free(wbuf)                                            # the copy goes with the buffer
    assert counts()["dropped"] - before_free == 1
    for ctx, tx, ty, g, buf in graphs.values():
        L.lm_ggml_backend_buffer_free(buf)
        L.lm_ggml_free(ctx)
    L.lm_ggml_backend_free(hip)
    L.lm_ggml_free(wctx)


def test_planes_copy_of_a_weight_that_is_a_view(host, orc):
    """A Q6_K weight that is a row range of a larger tensor (as a loader slices a fused matrix): the decode matmul reads a copy
    in planes of that range, a set_tensor on the parent drops it, rows of K % 2048 != 0 get no copy."""
    import cactus_amd
    L = host.L
    K, N_all, r0, N = 2048, 96, 32, 40
    w_all = orc.quantize_weights(O.Q6_K, common.weights_f32(91, N_all, K))
    w_new = orc.quantize_weights(O.Q6_K, common.weights_f32(92, N_all, K))
    cdev = cactus_amd.Device(0)
    dev = L.lm_ggml_backend_reg_dev_get(host.reg, 0)
    hip = L.lm_ggml_backend_dev_init(dev, None)
    wctx = host.context(with_graph=False)
    tw = host.tensor_2d(wctx, O.Q6_K, K, N_all, "w_all")
    t768 = host.tensor_2d(wctx, O.Q6_K, 768, 24, "w_768")
    wbuf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(wctx, L.lm_ggml_backend_dev_buffer_type(dev))
    host.set(tw, w_all)
    w768 = orc.quantize_weights(O.Q6_K, common.weights_f32(93, 24, 768))
    host.set(t768, w768)
    row = w_all.shape[1]
    blib = C.CDLL(cactus_amd.BACKEND_LIB)
    for name in ("copies", "dropped", "matmuls"):
        getattr(blib, "lm_ggml_backend_hip_get_planes_" + name).restype = C.c_ulonglong
    ctx = host.context()
    view = L.lm_ggml_view_2d(ctx, tw, K, N, row, r0 * row)
    tx = host.tensor_2d(ctx, O.F32, K, 1, "x")
    ty = L.lm_ggml_mul_mat(ctx, view, tx)
    tx7 = host.tensor_2d(ctx, O.F32, 768, 1, "x7")
    ty7 = L.lm_ggml_mul_mat(ctx, t768, tx7)
    g = L.lm_ggml_new_graph(ctx)
    L.lm_ggml_build_forward_expand(g, ty)
    L.lm_ggml_build_forward_expand(g, ty7)
    buf = L.lm_ggml_backend_alloc_ctx_tensors_from_buft(ctx, L.lm_ggml_backend_dev_buffer_type(dev))
    x, x7 = common.activations_f32(94, 1, K), common.activations_f32(95, 1, 768)
    host.set(tx, x)
    host.set(tx7, x7)
    copies, dropped = blib.lm_ggml_backend_hip_get_planes_copies(), blib.lm_ggml_backend_hip_get_planes_dropped()
    assert L.lm_ggml_backend_graph_compute(hip, g) == 0
    assert blib.lm_ggml_backend_hip_get_planes_copies() - copies == 1                      # the view's rows; none for K = 768
    assert host.get(ty, np.float32, (1, N)).tobytes() == cdev.mul_mat(O.Q6_K, w_all[r0:r0 + N], x).tobytes()
    assert host.get(ty7, np.float32, (1, 24)).tobytes() == cdev.mul_mat(O.Q6_K, w768, x7).tobytes()
    host.set(tw, w_new)                                                                    # through the parent: overlaps the copy
    assert blib.lm_ggml_backend_hip_get_planes_dropped() - dropped == 1
    assert L.lm_ggml_backend_graph_compute(hip, g) == 0
    assert host.get(ty, np.float32, (1, N)).tobytes() == cdev.mul_mat(O.Q6_K, w_new[r0:r0 + N], x).tobytes()
    L.lm_ggml_backend_buffer_free(buf)
    L.lm_ggml_backend_buffer_free(wbuf)
    L.lm_ggml_free(ctx)
    L.lm_ggml_free(wctx)
    L.lm_ggml_backend_free(hip)
