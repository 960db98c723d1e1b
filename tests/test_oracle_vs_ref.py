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
