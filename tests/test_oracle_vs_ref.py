"""Differential test: the restatement against the reference's own compiled code on seeded inputs.
Runs only where oracle/_ref/libggml_ref.so exists (it is built from the reference tree, which the GPU box
does not have as source but does receive as a built artefact)."""
import numpy as np
import pytest

import common
import oracle as O


@pytest.mark.parametrize("K", [256, 4096, 11008])
def test_activation_quantizers_bit_exact(orc, ref, K):
    x = common.activations_f32(K, 6, K)
    x[1] *= 1e-3
    x[2] *= 50
    x[3, : K // 2] = 0
    x[4] = 0
    for at in (O.Q8_0, O.Q8_K):
        assert np.array_equal(orc.quantize_activation(at, x), ref.quantize_activation(at, x))


def test_activation_quantizers_many_blocks(orc, ref):
    # 2^20 values at varied scales: the AVX2/ref divergence (127/amax vs 1/(amax/127), ties) shows here if at all
    rng = np.random.default_rng(42)
    x = (rng.standard_normal((64, 16384)) * np.exp(rng.uniform(-6, 6, (64, 1)))).astype(np.float32)
    for at in (O.Q8_0, O.Q8_K):
        assert np.array_equal(orc.quantize_activation(at, x), ref.quantize_activation(at, x))
    a = orc.quantize_activation(O.Q8_0, x)
    b = np.stack([orc.quantize_q8_0_ref(r) for r in x])
    assert not np.array_equal(a, b), "AVX2 and scalar Q8_0 quantizers are expected to differ somewhere"


@pytest.mark.parametrize("wt", O.WEIGHT_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_weight_quantizers_and_dots(orc, ref, wt):
    K, N, n = 2048, 24, 3
    w = common.weights_f32(wt, N, K, outliers=True)
    w[5] = 0
    w[6, :256] = 0
    x = common.activations_f32(wt, n, K)
    b = ref.quantize_weights(wt, w)
    if wt in O.ORACLE_QUANTIZED:
        assert np.array_equal(orc.quantize_weights(wt, w), b)
    assert np.array_equal(orc.dequantize(wt, b, K), ref.dequantize(wt, b, K))
    xq = ref.quantize_activation(O.VEC_DOT_TYPE[wt], x)
    for t in range(n):
        for i in range(N):
            assert orc.vec_dot(wt, K, b[i], xq[t]).tobytes() == ref.vec_dot(wt, K, b[i], xq[t]).tobytes()


@pytest.mark.parametrize("wt", O.LOW_BIT_K_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_low_bit_k_quants_on_random_bytes(orc, ref, wt):
    """Q3_K, Q2_K and IQ4_XS over random block bytes with sane fp16 super-block scales: every code of the packed scales (Q3_K's below
    32, i.e. negative ones, included), every quant and high-bit pattern; dequantizer and dot bit for bit the reference's."""
    K, N, n = 1024, 16, 2
    rng = np.random.default_rng(77 + wt)
    bb, nb = O.BLOCK_BYTES[wt], K // 256
    b = rng.integers(0, 256, (N, nb, bb), dtype=np.uint8)
    d = (0.01 * np.exp(rng.uniform(-1, 1, (N, nb)))).astype(np.float16)
    d[rng.random((N, nb)) < 0.2] *= np.float16(-1)
    off = {O.Q3_K: 108, O.Q2_K: 80, O.IQ4_XS: 0}[wt]
    b[..., off:off + 2] = d.view(np.uint8).reshape(N, nb, 2)
    if wt == O.Q2_K:
        b[..., 82:84] = (d * np.float16(0.5)).view(np.uint8).reshape(N, nb, 2)
    b = b.reshape(N, nb * bb)
    assert np.array_equal(orc.dequantize(wt, b, K), ref.dequantize(wt, b, K))
    xq = ref.quantize_activation(O.Q8_K, common.activations_f32(wt, n, K))
    for t in range(n):
        for i in range(N):
            assert orc.vec_dot(wt, K, b[i], xq[t]).tobytes() == ref.vec_dot(wt, K, b[i], xq[t]).tobytes()
            # the integer sums are those of the dequantized integers (d = 1: the super-block scale taken out)
            v, isum, imin = orc.vec_dot(wt, K, b[i], xq[t], want_sums=True)
            exact, sum_abs = orc.vec_dot_exact(wt, K, b[i], xq[t])
            assert abs(float(v) - exact) <= 1e-5 * sum_abs


@pytest.mark.parametrize("wt", O.WEIGHT_TYPES, ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("n,threads", [(1, 1), (5, 3)])
def test_mul_mat_graph(orc, ref, wt, n, threads):
    K, N = 1024, 70
    wq = orc.quantize_weights(wt, common.weights_f32(9 + wt, N, K))
    x = common.activations_f32(9 + wt, n, K)
    y_ref, _ = ref.mul_mat_graph(wt, wq, x, nthreads=threads)
    y = orc.mul_mat(wt, wq, x, nthreads=threads)["y"]
    assert np.array_equal(y, y_ref)


@pytest.mark.parametrize("wt", (O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K, O.Q5_K, O.Q4_1, O.F16), ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("n_tokens,ne11,threads", [(1, 1, 1), (3, 4, 2), (5, 1, 3)])
def test_mul_mat_id_graph(orc, ref, wt, n_tokens, ne11, threads):
    """MUL_MAT_ID against the reference CPU backend: 6 experts, 4 used per token, activations either shared by the
    slots of a token (ne11 = 1) or one row per slot; bit-exact."""
    K, N, n_as, n_used = 512, 37, 6, 4
    rng = np.random.default_rng(21 + wt + n_tokens)
    W = np.stack([orc.quantize_weights(wt, common.weights_f32(30 + wt + e, N, K)) for e in range(n_as)])
    x = common.activations_f32(31 + wt, n_tokens * ne11, K).reshape(n_tokens, ne11, K)
    ids = np.stack([rng.permutation(n_as)[:n_used] for _ in range(n_tokens)]).astype(np.int32)
    y_ref = ref.mul_mat_id_graph(wt, W, x, ids, nthreads=threads)
    y = orc.mul_mat_id(wt, W, x, ids, nthreads=threads)["y"]
    assert np.array_equal(y, y_ref)
    # the op is MUL_MAT on the selected expert, pair by pair
    t, s = n_tokens - 1, n_used - 1
    one = orc.mul_mat(wt, W[ids[t, s]], x[t, s % ne11][None, :])["y"][0]
    assert np.array_equal(y[t, s], one)


def elementwise_inputs(seed, n, ne0):
    """Activations with the magnitudes that occur next to the matmuls, plus the values that exercise every branch of
    the exponential: large |x| (beyond the two-factor scaling thresholds), zeros, tiny values."""
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((n, ne0)) * rng.choice([0.01, 1.0, 8.0, 40.0], (n, 1))).astype(np.float32)
    special = np.array([0.0, -0.0, 1e-30, -1e-30, 87.0, -87.0, 88.5, -88.5, 89.0, -104.0, 130.0, -130.0, 133.0, -140.0, 1e4, -1e4],
                       np.float32)
    m = min(special.size, ne0)
    x[0, :m] = special[:m]
    return x


@pytest.mark.parametrize("n,ne0,threads", [(1, 256, 1), (7, 4096, 3), (3, 40, 2), (2, 11008, 2)])
def test_rms_norm_and_silu_graph(orc, ref, n, ne0, threads):
    x = elementwise_inputs(n + ne0, n, ne0)
    for eps in (1e-5, 1e-6):
        assert orc.rms_norm(x, eps).tobytes() == ref.op_graph("rms_norm", x, eps=eps, nthreads=threads).tobytes()
    with np.errstate(all="ignore"):
        a, b = orc.silu(x), ref.op_graph("silu", x, nthreads=threads)
    assert a.tobytes() == b.tobytes()


def test_rms_norm_and_silu_rows_with_a_tail(orc, ref):
    # 13 = 8 + 5: the last 5 elements of a row take the reference's scalar expf path
    x = elementwise_inputs(5, 4, 13)
    assert orc.silu(x).tobytes() == ref.op_graph("silu", x).tobytes()
    assert orc.rms_norm(x, 1e-5).tobytes() == ref.op_graph("rms_norm", x, eps=1e-5).tobytes()


def test_add_and_mul_are_single_ieee_operations(ref):
    x = elementwise_inputs(9, 6, 512)
    y = elementwise_inputs(10, 6, 512)
    w = elementwise_inputs(11, 1, 512)
    with np.errstate(all="ignore"):
        assert ref.op_graph("add", x, y).tobytes() == (x + y).tobytes()
        assert ref.op_graph("mul", x, y).tobytes() == (x * y).tobytes()
        assert ref.op_graph("mul", x, w).tobytes() == (x * w).tobytes()        # one row broadcast over all rows
        assert ref.op_graph("add", x, w).tobytes() == (x + w).tobytes()


def causal_mask(ne01, ne00, n_past, dtype, pad_rows=0):
    """The attention mask of a causal decoder: token i (of ne01 new ones after n_past cached) sees keys 0 .. n_past + i."""
    m = np.full((ne01 + pad_rows, ne00), -np.inf, np.float32)
    for i in range(ne01):
        m[i, : min(ne00, n_past + i + 1)] = 0.0
    return m.astype(dtype)


@pytest.mark.parametrize("n_head,ne01,ne00,threads", [(1, 1, 32, 1), (4, 3, 256, 2), (8, 5, 1000, 3), (2, 16, 4096, 2), (3, 2, 13, 1)])
def test_soft_max_graph(orc, ref, n_head, ne01, ne00, threads):
    rng = np.random.default_rng(n_head * 1000 + ne00)
    x = (rng.standard_normal((n_head, ne01, ne00)) * 6).astype(np.float32)
    x[0, 0, : min(8, ne00)] = [30.0, -30.0, 88.0, -104.0, 0.0, 1e-3, -200.0, 50.0][: min(8, ne00)]
    assert orc.soft_max(x).tobytes() == ref.soft_max_graph(x, nthreads=threads).tobytes()
    for dt in (np.float32, np.float16):
        mask = causal_mask(ne01, ne00, max(0, ne00 - ne01 - 3), dt, pad_rows=3)
        for scale in (1.0, 0.08838834764831845):
            a = orc.soft_max(x, mask, scale)
            b = ref.soft_max_graph(x, mask, scale, nthreads=threads)
            assert a.tobytes() == b.tobytes()
            assert np.all(a[:, :, :][np.broadcast_to(np.isinf(mask[:ne01]), a.shape)] == 0.0)
    # a finite additive mask (relative position bias) and ALiBi slopes
    bias = (rng.standard_normal((ne01, ne00)) * 2).astype(np.float32)
    assert orc.soft_max(x, bias, 0.5).tobytes() == ref.soft_max_graph(x, bias, 0.5, nthreads=threads).tobytes()
    assert orc.soft_max(x, bias, 0.5, 8.0).tobytes() == ref.soft_max_graph(x, bias, 0.5, 8.0, nthreads=threads).tobytes()


def test_gelu_graph(orc, ref):
    """Every fp16 value (each entry of the reference's table), values that round to fp16 ties, and the two cut-offs."""
    h = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    h = h[np.isfinite(h)]
    rng = np.random.default_rng(12)
    r = (rng.standard_normal(8192) * 4).astype(np.float32)
    edge = np.array([-10.0, np.nextafter(np.float32(-10), np.float32(0)), 10.0, np.nextafter(np.float32(10), np.float32(0)), 0.0, -0.0,
                     1.0 + 2.0 ** -11, 1.0 + 2.0 ** -11 + 2.0 ** -20, 65519.0, 1e-8, -1e-8, 3e38, -3e38], np.float32)
    x = np.concatenate([h, r, edge])
    x = np.concatenate([x, np.zeros(-x.size % 64, np.float32)]).reshape(-1, 64)
    with np.errstate(all="ignore"):
        assert orc.gelu(x).tobytes() == ref.unary_graph("gelu", x, nthreads=2).tobytes()


def test_gelu_known_values(orc):
    x = np.array([[0.0, 10.0, 25.0, -10.0, -30.0, 1.0, -1.0, 3.0]], np.float32)
    y = orc.gelu(x)[0]
    assert y[0] == 0.0 and y[1] == 10.0 and y[2] == 25.0 and y[3] == 0.0 and y[4] == 0.0
    # the table holds fp16 values of 0.5 x (1 + tanh(...)): 0.8413 / -0.1587 / 2.996 to fp16 precision
    want = [0.5 * v * (1 + np.tanh(np.sqrt(2 / np.pi) * v * (1 + 0.044715 * v * v))) for v in (1.0, -1.0, 3.0)]
    assert np.allclose(y[5:], want, rtol=1e-3)
    assert (orc.gelu(x).view(np.uint32) & 0x1fff == 0).all()             # every output is an fp16 number


def test_scale_graph(orc, ref):
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((7, 96)) * 50).astype(np.float32)
    x[0, :4] = [0.0, -0.0, 3e38, 1e-40]
    for v in (0.125, 0.08838834764831845, -3.7, 1e30):
        with np.errstate(all="ignore"):
            assert orc.scale(x, v).tobytes() == ref.scale_graph(x, v).tobytes()


def test_soft_max_rows_sum_to_one(orc):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((2, 4, 512)) * 4).astype(np.float32)
    y = orc.soft_max(x, None, 0.7)
    assert np.allclose(y.sum(-1, dtype=np.float64), 1.0, atol=1e-6)
    ref64 = np.exp((x * np.float32(0.7)).astype(np.float64) - (x * np.float32(0.7)).max(-1, keepdims=True))
    ref64 /= ref64.sum(-1, keepdims=True)
    assert np.allclose(y, ref64, rtol=3e-6, atol=1e-12)


@pytest.mark.parametrize("mode", [0, 2])
@pytest.mark.parametrize("ne0,n_dims,n_head,n_tokens", [(128, 128, 4, 5), (64, 32, 3, 2), (128, 64, 2, 7)])
def test_rope_graph(orc, ref, mode, ne0, n_dims, n_head, n_tokens):
    rng = np.random.default_rng(ne0 + n_dims + mode)
    x = rng.standard_normal((n_tokens, n_head, ne0)).astype(np.float32)
    pos = np.array([0, 1, 17, 4095, 100000, 31, 2][:n_tokens], np.int32)
    assert orc.rope(x, pos, n_dims, mode).tobytes() == ref.rope_graph(x, pos, n_dims, mode).tobytes()
    kw = dict(freq_base=500000.0, freq_scale=0.25)
    assert orc.rope(x, pos, n_dims, mode, **kw).tobytes() == ref.rope_graph(x, pos, n_dims, mode, **kw).tobytes()
    ff = (1.0 + rng.random(n_dims // 2) * 7).astype(np.float32)
    assert orc.rope(x, pos, n_dims, mode, ff).tobytes() == ref.rope_graph(x, pos, n_dims, mode, ff).tobytes()
    yarn = dict(freq_scale=0.25, ext_factor=1.0, attn_factor=1.2, n_ctx_orig=2048)
    assert orc.rope(x, pos, n_dims, mode, **yarn).tobytes() == ref.rope_graph(x, pos, n_dims, mode, **yarn).tobytes()


def test_rope_is_a_rotation(orc):
    # what the mathematics fixes: position 0 is the identity, pair norms are preserved, the angle of pair i at position
    # p is p * base^(-2i / n_dims)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((3, 2, 64)).astype(np.float32)
    pos = np.array([0, 5, 77], np.int32)
    for mode in (0, 2):
        y = orc.rope(x, pos, 64, mode)
        assert y[0].tobytes() == x[0].tobytes()
        pair = (lambda a: (a[..., 0::2], a[..., 1::2])) if mode == 0 else (lambda a: (a[..., :32], a[..., 32:]))
        x0, x1 = pair(x.astype(np.float64))
        y0, y1 = pair(y.astype(np.float64))
        assert np.allclose(x0 ** 2 + x1 ** 2, y0 ** 2 + y1 ** 2, rtol=1e-5)
        theta = pos[:, None, None].astype(np.float64) * 10000.0 ** (-2.0 * np.arange(32) / 64)
        assert np.allclose(y0, x0 * np.cos(theta) - x1 * np.sin(theta), atol=2e-4)
        assert np.allclose(y1, x0 * np.sin(theta) + x1 * np.cos(theta), atol=2e-4)


@pytest.mark.parametrize("ne1,ne0", [(1, 1024), (7, 96), (33, 130)])
def test_cpy_graphs(orc, ref, ne1, ne0):
    rng = np.random.default_rng(ne1 + ne0)
    x = (rng.standard_normal((ne1, ne0)) * 3).astype(np.float32)
    x.reshape(-1)[:6] = [65504.0, 65520.0, 1e-8, -6.1e-5, 2049.0, 2051.0]     # fp16 max, overflow, underflow, ties
    with np.errstate(all="ignore"):
        assert orc.cpy(x, np.float16).reshape(-1).tobytes() == ref.cpy_graph(x, np.float16, "flat").tobytes()
        assert orc.cpy(x.T, np.float16).tobytes() == ref.cpy_graph(x, np.float16, "transpose").tobytes()
        assert orc.cpy(x.T, np.float32).tobytes() == ref.cpy_graph(x, np.float32, "cont").tobytes()
        h = x.astype(np.float16)
        assert orc.cpy(h.T, np.float16).tobytes() == ref.cpy_graph(h, np.float16, "cont").tobytes()
        assert orc.cpy(h, np.float32).reshape(-1).tobytes() == ref.cpy_graph(h, np.float32, "flat").tobytes()


@pytest.mark.parametrize("hd,n_head,n_head_kv,n_tokens,n_kv,threads", [(128, 8, 2, 3, 96, 2), (64, 4, 4, 1, 40, 1), (96, 6, 2, 5, 33, 3)])
def test_attention_matmuls_over_an_f16_cache(orc, ref, hd, n_head, n_head_kv, n_tokens, n_kv, threads):
    """The batched, broadcast F16 MUL_MAT of the oracle against the reference's graph over permuted cache views."""
    rng = np.random.default_rng(hd + n_kv)
    k_cache = rng.standard_normal((n_kv, n_head_kv, hd)).astype(np.float16)
    vt_cache = rng.standard_normal((hd, n_head_kv, n_kv)).astype(np.float16)
    q = rng.standard_normal((n_tokens, n_head, hd)).astype(np.float32)
    p = rng.random((n_head, n_tokens, n_kv)).astype(np.float32)
    kq_ref, kqv_ref = ref.attention_matmul_graphs(k_cache, vt_cache, q, p, nthreads=threads)
    kq = orc.mul_mat_f16_batched(k_cache.transpose(1, 0, 2), q.transpose(1, 0, 2))["y"]
    kqv = orc.mul_mat_f16_batched(vt_cache.transpose(1, 0, 2), p)["y"]
    assert kq.tobytes() == kq_ref.tobytes()
    assert kqv.tobytes() == kqv_ref.tobytes()


@pytest.mark.parametrize("wt", [O.F32] + list(O.WEIGHT_TYPES))
def test_get_rows_graph(orc, ref, wt):
    nc, ne01 = 512, 37
    rng = np.random.default_rng(wt + 1)
    ids = rng.integers(0, ne01, 11).astype(np.int32)
    ids[:3] = [0, ne01 - 1, 5]
    w = (rng.standard_normal((ne01, nc)) * 0.3).astype(np.float32)
    if wt == O.F32:
        table = w
    elif wt == O.F16:
        table = w.astype(np.float16).view(np.uint8).reshape(ne01, -1)
    else:
        table = orc.quantize_weights(wt, w)
    a = orc.get_rows(wt, table, nc, ids)
    b = ref.get_rows_graph(wt, table, nc, ids, nthreads=2)
    assert a.shape == (11, nc) and a.tobytes() == b.tobytes()
