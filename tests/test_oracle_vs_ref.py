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
