"""GPU parity: the HIP path, called through the C-ABI, against the CPU oracle on identical seeded inputs and
against the committed golden vectors.

Bars (from the task's contract): activation-quantizer bytes and per-block integer sums bit-exact; each fp32
output within 1e-5 * sum_b |scale_b * isum_b| of the reference value (only the summation order differs)."""
import os

import numpy as np
import pytest

import functools

import common
import oracle as O


@functools.lru_cache(maxsize=12)
def quantized_weights(wt, seed, N, K, outliers=False):
    """Seeded weights quantized by the oracle; kept for the other token counts of the same shape (the quantizer search
    of a 4099 x 11008 matrix costs seconds of CPU)."""
    return O.Oracle().quantize_weights(wt, common.weights_f32(seed, N, K, outliers=outliers))

pytestmark = pytest.mark.gpu

REL_TOL = 1e-5
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def dev():
    import cactus_amd
    d = cactus_amd.Device(0)
    print("device:", d.info.name.decode(), d.info.arch.decode(), "CUs", d.info.compute_units,
          "LDS/block", d.info.max_lds_per_block, flush=True)
    return d


@pytest.fixture
def forced_q6k_matrix_core(dev):
    dev.lib.chip_verify_force_q6k_matrix_core(1)
    yield
    dev.lib.chip_verify_force_q6k_matrix_core(0)


def check_outputs(y_gpu, y_ref, sum_abs, what):
    err = np.abs(y_gpu.astype(np.float64) - y_ref.astype(np.float64))
    bound = REL_TOL * sum_abs
    worst = float((err / np.maximum(bound, 1e-300)).max())
    assert (err <= bound).all(), "%s: worst error is %.3g x the tolerance" % (what, worst)


# ------------------------------------------------------------------------------------------ quantizers
@pytest.mark.parametrize("K", [256, 1024, 4096, 11008, 14336])
def test_quantizers_bit_exact(dev, orc, K):
    x = common.activations_f32(K, 5, K)
    x[1] *= 1e-3
    x[2] *= 300
    x[3, : K // 2] = 0
    x[4] = 0
    for at in (O.Q8_0, O.Q8_K, O.Q8_1, O.F16):
        print("quantize", O.TYPE_NAMES[at], "K", K, flush=True)
        assert np.array_equal(dev.quantize(at, x), orc.quantize_activation(at, x))


def test_quantizers_many_blocks(dev, orc):
    rng = np.random.default_rng(42)
    x = (rng.standard_normal((64, 16384)) * np.exp(rng.uniform(-6, 6, (64, 1)))).astype(np.float32)
    for at in (O.Q8_0, O.Q8_K, O.Q8_1):
        assert np.array_equal(dev.quantize(at, x), orc.quantize_activation(at, x))


def test_quantizer_edge_vectors(dev):
    g = np.load(os.path.join(GOLD, "quantize_q8_0_edges.npz"))
    x = np.zeros((g["x"].shape[0], 256), np.float32)
    x[:, :32] = g["x"]                      # K must be a multiple of 32; pad the edge rows with zero blocks
    got = dev.quantize(O.Q8_0, x)[:, :34]
    assert np.array_equal(got, g["q_avx2"])
    g = np.load(os.path.join(GOLD, "quantize_q8_K_edges.npz"))
    assert np.array_equal(dev.quantize(O.Q8_K, g["x"]), g["q"])
    g = np.load(os.path.join(GOLD, "quantize_q8_1_edges.npz"))
    x = np.zeros((g["x"].shape[0], 256), np.float32)
    x[:, :32] = g["x"]
    assert np.array_equal(dev.quantize(O.Q8_1, x)[:, :36], g["q"])


# ------------------------------------------------------------------------------------------ the op
@pytest.mark.parametrize("wt", O.WEIGHT_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_mul_mat_golden(dev, wt):
    g = np.load(os.path.join(GOLD, "mul_mat_%s.npz" % O.TYPE_NAMES[wt]))
    K = int(g["K"])
    y, blocks = dev.mul_mat(wt, g["wq"], g["x"], want_workspace_blocks=True)
    assert np.array_equal(blocks, g["xq"])          # fused on-the-fly quantization, bit-exact
    import oracle
    o = oracle.Oracle()
    sa = o.mul_mat(wt, g["wq"], g["x"], want=("sum_abs",))["sum_abs"]
    check_outputs(y, g["y_graph"], sa, "golden " + O.TYPE_NAMES[wt])


SHAPES = [(256, 1), (512, 7), (2048, 130), (4096, 257), (11008, 40), (14336, 33)]


@pytest.mark.parametrize("wt", O.WEIGHT_TYPES, ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("K,N", SHAPES)
@pytest.mark.parametrize("n", [1, 2, 3, 5, 8])
def test_mul_mat_vs_oracle(dev, orc, wt, K, N, n):
    print("mul_mat", O.TYPE_NAMES[wt], "K", K, "N", N, "n", n, flush=True)
    wq = orc.quantize_weights(wt, common.weights_f32(K + N + wt, N, K, outliers=(wt in (O.Q4_K, O.Q5_K))))
    x = common.activations_f32(K + n, n, K)
    if n >= 3:
        x[1] = 0                                    # an all-zero token
    ref = orc.mul_mat(wt, wq, x, nthreads=8, want=("wdata", "sum_abs"))
    y, blocks = dev.mul_mat(wt, wq, x, want_workspace_blocks=True)
    assert np.array_equal(blocks, ref["wdata"])
    check_outputs(y, ref["y"], ref["sum_abs"], "mul_mat")


@pytest.mark.parametrize("wt,K,N", [(O.Q4_K, 11008, 5000), (O.Q6_K, 14336, 4500), (O.Q5_K, 12288, 2600), (O.Q6_K, 14336, 4096),
                                    (O.Q4_K, 14336, 300)],
                         ids=["q4_K-5000x11008", "q6_K-4500x14336", "q5_K-2600x12288", "q6_K-4096x14336", "q4_K-300x14336"])
def test_long_rows_quantized_a_part_at_a_time(dev, orc, wt, K, N):
    """One token, K-quant rows of three or four weight steps: the kernel builds its activation image a step's part at a time
    behind the previous step's arithmetic, in workgroups of 4, 8 and 16 waves (by row count), with and without a second
    tile per wave.  Activation bytes bit-exact, outputs within the tolerance and the same bits for every copy of a row; the
    pair form (two matrices as one of twice the rows) returns the same bits."""
    base = orc.quantize_weights(wt, common.weights_f32(K + N + wt, 100, K, outliers=(wt != O.Q6_K)))
    W = np.tile(base, (N // 100 + 1, 1))[:N]
    x = common.activations_f32(K + 3, 1, K)
    ref = orc.mul_mat(wt, base, x, nthreads=8, want=("wdata", "sum_abs"))
    y, blocks = dev.mul_mat(wt, W, x, want_workspace_blocks=True)
    assert np.array_equal(blocks, ref["wdata"])
    idx = np.arange(N) % 100
    check_outputs(y, ref["y"][:, idx], ref["sum_abs"][:, idx], "rows of %d values" % K)
    assert (y[0] == y[0, idx]).all()                                      # row r equals row r % 100
    a, b = dev.mul_mat_pair(wt, W, np.ascontiguousarray(W[::-1]), x)
    assert a.tobytes() == y.tobytes() and b.tobytes() == np.ascontiguousarray(y[:, ::-1]).tobytes()


@pytest.mark.parametrize("wt", O.BLOCK_WEIGHT_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_block_integer_sums_bit_exact(dev, orc, wt):
    K, N, n = 2048, 9, 2
    wq = orc.quantize_weights(wt, common.weights_f32(300 + wt, N, K, outliers=True))
    aq = orc.quantize_activation(O.VEC_DOT_TYPE[wt], common.activations_f32(300 + wt, n, K))
    isum, imin = dev.block_isums(wt, wq, aq, K)
    for t in range(n):
        for i in range(N):
            _, ri, rm = orc.vec_dot(wt, K, wq[i], aq[t], want_sums=True)
            assert np.array_equal(isum[t, i], ri)
            if wt in (O.Q4_K, O.Q5_K):
                assert np.array_equal(imin[t, i], rm)


def test_block_integer_sums_extreme_bytes(dev, orc):
    # saturating patterns: all nibbles 15 / quants +-127 with the largest scales
    K = 256
    for wt in (O.Q4_0, O.Q8_0):
        bb = O.BLOCK_BYTES[wt]
        w = np.zeros((2, K // 32, bb), np.uint8)
        w[..., :2] = np.array([1.0], np.float16).view(np.uint8)
        w[0, :, 2:] = 0xFF if wt == O.Q4_0 else 0x7F
        w[1, :, 2:] = 0x00 if wt == O.Q4_0 else 0x81
        w = w.reshape(2, -1)
        x = np.full((1, K), 5.0, np.float32)
        x[0, ::2] = -5.0 if wt == O.Q8_0 else 5.0
        aq = orc.quantize_activation(O.Q8_0, x)
        isum, _ = dev.block_isums(wt, w, aq, K)
        for i in range(2):
            _, ri, _ = orc.vec_dot(wt, K, w[i], aq[0], want_sums=True)
            assert np.array_equal(isum[0, i], ri)


@pytest.mark.parametrize("wt", O.WEIGHT_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_mul_mat_token_groups(dev, orc, wt):
    # more than 8 tokens: runs as several launches over token groups (or the GEMM), same numbers
    K, N, n = 1024, 48, 19
    wq = orc.quantize_weights(wt, common.weights_f32(500 + wt, N, K))
    x = common.activations_f32(500 + wt, n, K)
    ref = orc.mul_mat(wt, wq, x, nthreads=8, want=("sum_abs",))
    check_outputs(dev.mul_mat(wt, wq, x), ref["y"], ref["sum_abs"], "token groups")


@pytest.mark.parametrize("K,N", [(256, 4100), (1024, 4111), (4096, 4096), (11008, 4099), (14336, 4096)])
@pytest.mark.parametrize("n", [5, 8, 9, 16, 17, 37])
def test_mul_mat_q8_0_matrix_core_gemv(dev, orc, K, N, n):
    # enough 16-row tiles for every CU and 5+ tokens: the integer sums come from v_mfma_i32_16x16x64_i8;
    # ragged N (last tile partly outside), token counts on both sides of the 8- and 16-token images
    print("mmv q8_0 K", K, "N", N, "n", n, flush=True)
    wq = quantized_weights(O.Q8_0, K + N, N, K)
    x = common.activations_f32(K + n, n, K)
    x[2] = 0
    x[3] *= 250
    ref = orc.mul_mat(O.Q8_0, wq, x, nthreads=8, want=("wdata", "sum_abs"))
    y, blocks = dev.mul_mat(O.Q8_0, wq, x, want_workspace_blocks=True)
    assert np.array_equal(blocks, ref["wdata"])
    check_outputs(y, ref["y"], ref["sum_abs"], "matrix-core gemv")


@pytest.mark.parametrize("wt", (O.Q4_K, O.Q5_K), ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("K,N", [(256, 4100), (1024, 4111), (4096, 4096), (11008, 4099), (8192, 4128), (14336, 4096)])
@pytest.mark.parametrize("n", [5, 8, 9, 15, 16])
def test_mul_mat_q4_K_q5_K_matrix_core_gemv(dev, orc, wt, K, N, n):
    # the K-quant form of the matrix-core GEMV: 6-bit sub-block scales and mins applied to exact integer sums (Q5_K: the
    # fifth bit from qh); ragged N, token counts on both sides of the 8-token image, outlier weights (large dmin), a
    # zero row and a large row of activations
    print("mmv", O.TYPE_NAMES[wt], "K", K, "N", N, "n", n, flush=True)
    wq = quantized_weights(wt, K + N + 1, N, K, True)
    x = common.activations_f32(K + n + 1, n, K)
    x[2] = 0
    x[3] *= 250
    ref = orc.mul_mat(wt, wq, x, nthreads=8, want=("wdata", "sum_abs"))
    y, blocks = dev.mul_mat(wt, wq, x, want_workspace_blocks=True)
    assert np.array_equal(blocks, ref["wdata"])
    check_outputs(y, ref["y"], ref["sum_abs"], "matrix-core gemv " + O.TYPE_NAMES[wt])


@pytest.mark.parametrize("K,N", [(256, 4100), (1024, 4111), (4096, 4096), (11008, 4099), (14336, 4096)])
@pytest.mark.parametrize("n", [5, 8, 9, 16, 17, 31])
def test_mul_mat_q4_0_matrix_core_gemv(dev, orc, K, N, n):
    # the Q4_0 form of the matrix-core GEMV: operands 16 * (nibble - 8), scale d / 16
    print("mmv q4_0 K", K, "N", N, "n", n, flush=True)
    wq = quantized_weights(O.Q4_0, K + N + 2, N, K)
    x = common.activations_f32(K + n + 2, n, K)
    x[2] = 0
    x[3] *= 250
    ref = orc.mul_mat(O.Q4_0, wq, x, nthreads=8, want=("wdata", "sum_abs"))
    y, blocks = dev.mul_mat(O.Q4_0, wq, x, want_workspace_blocks=True)
    assert np.array_equal(blocks, ref["wdata"])
    check_outputs(y, ref["y"], ref["sum_abs"], "matrix-core gemv q4_0")


@pytest.mark.parametrize("K,N", [(256, 4100), (1024, 4111), (4096, 4096), (11008, 4099), (14336, 4096)])
@pytest.mark.parametrize("n", [5, 8, 9, 16, 21])
def test_mul_mat_q6_K_matrix_core_gemv(dev, orc, K, N, n, forced_q6k_matrix_core):
    # the Q6_K form: unsigned 6-bit operands, int8 sub-block scales, the -32 taken out through the activation block sums;
    # rows that are only 2-byte aligned (210-byte super-blocks), ragged N, several launches of 8 tokens.  By default the
    # library takes this kernel only on very large matrices (an output head; tests/test_gpu_config5.py runs that shape
    # with the default dispatch); the fixture makes it take these shapes too.
    print("mmv q6_K K", K, "N", N, "n", n, flush=True)
    wq = quantized_weights(O.Q6_K, K + N + 3, N, K)
    x = common.activations_f32(K + n + 3, n, K)
    x[2] = 0
    x[3] *= 250
    ref = orc.mul_mat(O.Q6_K, wq, x, nthreads=8, want=("wdata", "sum_abs"))
    y, blocks = dev.mul_mat(O.Q6_K, wq, x, want_workspace_blocks=True)
    assert np.array_equal(blocks, ref["wdata"])
    check_outputs(y, ref["y"], ref["sum_abs"], "matrix-core gemv q6_K")


def test_matrix_core_gemv_integer_sums_are_exact(dev, orc):
    # all scales 1 and activations that quantize to themselves: the fp32 result is the integer sum itself, so a wrong
    # nibble plane, sign or scale factor in the operand form of the Q4_0 kernel shows as a different integer
    K, N, n = 512, 4096, 8
    rng = np.random.default_rng(77)
    xi = rng.integers(-127, 128, (n, K)).astype(np.float32)
    xi[:, 0::32] = 127.0                                                   # every 32-block's maximum: d = 1 for Q8_0
    w4 = np.zeros((N, K // 32, 18), np.uint8)
    w4[..., 0:2] = np.array([1.0], np.float16).view(np.uint8)
    w4[..., 2:] = rng.integers(0, 256, (N, K // 32, 16), dtype=np.uint8)
    w4 = w4.reshape(N, -1)
    ref = orc.mul_mat(O.Q4_0, w4, xi)
    got = dev.mul_mat(O.Q4_0, w4, xi)
    assert got.tobytes() == ref["y"].tobytes()
    assert np.array_equal(got, np.round(got))


# ------------------------------------------------------------------------------------------ BASELINE sizes
def test_config1_q4_0_4096(dev, orc):
    K = N = 4096
    wq = orc.quantize_weights(O.Q4_0, common.weights_f32(1, N, K))
    x = common.activations_f32(1, 1, K)
    ref = orc.mul_mat(O.Q4_0, wq, x, nthreads=8, want=("sum_abs",))
    check_outputs(dev.mul_mat(O.Q4_0, wq, x), ref["y"], ref["sum_abs"], "config 1")


@pytest.mark.parametrize("N,K", [(11008, 4096), (4096, 11008)])
@pytest.mark.parametrize("n", [1, 2, 4, 8])
def test_config2_q8_0_ffn(dev, orc, N, K, n):
    print("config2", N, K, n, flush=True)
    wq = orc.quantize_weights(O.Q8_0, common.weights_f32(2, N, K))
    x = common.activations_f32(2, n, K)
    ref = orc.mul_mat(O.Q8_0, wq, x, nthreads=8, want=("sum_abs",))
    check_outputs(dev.mul_mat(O.Q8_0, wq, x), ref["y"], ref["sum_abs"], "config 2")


def test_config3_q4_K_outliers(dev, orc):
    N, K = 14336, 4096
    wq = orc.quantize_weights(O.Q4_K, common.weights_f32(3, N, K, outliers=True))
    x = common.activations_f32(3, 1, K)
    ref = orc.mul_mat(O.Q4_K, wq, x, nthreads=8, want=("sum_abs",))
    check_outputs(dev.mul_mat(O.Q4_K, wq, x), ref["y"], ref["sum_abs"], "config 3")


def test_linearity_in_block_scales(dev, orc):
    # size-independent property: doubling every weight scale (exact in fp16) doubles y exactly
    K, N = 4096, 512
    wq = orc.quantize_weights(O.Q8_0, common.weights_f32(77, N, K))
    x = common.activations_f32(77, 2, K)
    y1 = dev.mul_mat(O.Q8_0, wq, x)
    w2 = wq.reshape(N, -1, 34).copy()
    d = w2[..., :2].copy().view(np.float16)
    w2[..., :2] = (d * np.float16(2)).view(np.uint8)
    y2 = dev.mul_mat(O.Q8_0, w2.reshape(N, -1), x)
    assert np.array_equal(y2, 2 * y1)


# ------------------------------------------------------------------------------------------ error behaviour
def test_argument_errors(dev):
    import ctypes as C
    L = dev.lib
    buf = dev.alloc(1 << 16)
    ws = dev.alloc(1 << 16)
    # K not a multiple of 256, unknown type
    assert L.chip_mul_mat(O.Q4_0, buf.ptr, 18, 32, 1, buf.ptr, 32, 1, buf.ptr, 1, ws.ptr, 1 << 16, None) == -2
    assert L.chip_mul_mat(30, buf.ptr, 512, 256, 1, buf.ptr, 256, 1, buf.ptr, 1, ws.ptr, 1 << 16, None) == -2    # BF16
    # workspace too small, null pointers, misaligned weights, row stride below the row size
    assert L.chip_mul_mat(O.Q4_0, buf.ptr, 144, 256, 1, buf.ptr, 256, 1, buf.ptr, 1, ws.ptr, 16, None) == -3
    assert L.chip_mul_mat(O.Q4_0, None, 144, 256, 1, buf.ptr, 256, 1, buf.ptr, 1, ws.ptr, 1 << 16, None) == -1
    assert L.chip_mul_mat(O.Q4_0, buf.ptr + 2, 144, 256, 1, buf.ptr, 256, 1, buf.ptr, 1, ws.ptr, 1 << 16, None) == -1
    assert L.chip_mul_mat(O.Q6_K, buf.ptr + 1, 210, 256, 1, buf.ptr, 256, 1, buf.ptr, 1, ws.ptr, 1 << 16, None) == -1
    assert L.chip_mul_mat(O.Q4_0, buf.ptr, 128, 256, 1, buf.ptr, 256, 1, buf.ptr, 1, ws.ptr, 1 << 16, None) == -1
    # empty problems are fine
    assert L.chip_mul_mat(O.Q4_0, buf.ptr, 144, 256, 0, buf.ptr, 256, 1, buf.ptr, 1, ws.ptr, 1 << 16, None) == 0
    assert L.chip_mul_mat(O.Q4_0, buf.ptr, 144, 256, 1, buf.ptr, 256, 0, buf.ptr, 1, ws.ptr, 1 << 16, None) == 0
    assert L.chip_quantize_q8_0(buf.ptr, 102, 1, 96, buf.ptr, None) == -1     # ldx not a multiple of 4
    assert L.chip_quantize_q8_K(buf.ptr, 128, 1, 128, buf.ptr, None) == -2    # K not a multiple of 256
    dev.sync()


# ------------------------------------------------------------------------------------------ two matrices, one activation
@pytest.mark.parametrize("wt", (O.Q4_K, O.Q8_0, O.Q4_0, O.Q6_K, O.Q5_1, O.F16, O.Q3_K, O.Q2_K, O.IQ4_XS), ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("K,N", [(1024, 333), (4096, 1030)])
def test_mul_mat_pair_equals_two_mul_mats(dev, orc, wt, K, N):
    """chip_mul_mat_pair (ffn_gate and ffn_up in one launch up to 4 tokens; an odd row count puts a two-row tile of Q4_0
    across the two matrices): each output equals the single call's bit for bit, and the oracle within the tolerance."""
    w1 = quantized_weights(wt, K + N, N, K)
    w2 = quantized_weights(wt, K + N + 1, N, K)
    for n in (1, 2, 4, 3, 7):
        x = common.activations_f32(K + n, n, K)
        y1, y2 = dev.mul_mat_pair(wt, w1, w2, x)
        assert y1.tobytes() == dev.mul_mat(wt, w1, x).tobytes(), n
        assert y2.tobytes() == dev.mul_mat(wt, w2, x).tobytes(), n
        ref = orc.mul_mat(wt, w2, x, nthreads=8, want=("sum_abs",))
        check_outputs(y2, ref["y"], ref["sum_abs"], "second matrix of the pair, n = %d" % n)


# (types of wq, wk, wv), K, heads, KV heads, head size, rotated dims, mode: LLaMA-3-8B's attention block in a Q4_K_M file (NORM and
# NEOX pairs); 32-value block types incl. Q4_0 (two rows per step in the plain kernel, one in the pair walk); partial rotation
# (pass-through rows); a head size that is no power of two; more pairs than one pass of the grid takes
GROUP_ROPE_CASES = [((O.Q4_K, O.Q4_K, O.Q6_K), 4096, 32, 8, 128, 128, 0), ((O.Q4_K, O.Q4_K, O.Q6_K), 4096, 32, 8, 128, 128, 2),
                    ((O.Q4_0, O.Q8_0, O.Q5_1), 1024, 8, 2, 64, 32, 2), ((O.Q6_K, O.Q5_K, O.Q4_K), 2048, 6, 2, 96, 64, 0),
                    ((O.Q8_0, O.Q8_0, O.Q8_0), 512, 160, 160, 128, 128, 2), ((O.Q3_K, O.Q2_K, O.Q4_K), 1024, 8, 4, 64, 64, 0),
                    ((O.IQ4_XS, O.IQ4_XS, O.Q6_K), 2048, 16, 4, 128, 64, 2)]


@pytest.mark.parametrize("types,K,n_head,n_head_kv,hd,n_dims,mode", GROUP_ROPE_CASES)
def test_group_with_rope_in_the_epilogue_equals_group_then_rope(dev, types, K, n_head, n_head_kv, hd, n_dims, mode):
    """chip_mul_mat_group_rope: Q and K rotated in their projections' epilogue (K as F32 and as the fp16 cache copy, or the fp16
    copy alone), V untouched - every value bit for bit what chip_mul_mat_group followed by chip_rope_apply_two gives."""
    wq = quantized_weights(types[0], K + 1, n_head * hd, K)
    wk = quantized_weights(types[1], K + 2, n_head_kv * hd, K)
    wv = quantized_weights(types[2], K + 3, n_head_kv * hd, K)
    members = [(types[0], wq), (types[1], wk), (types[2], wv)]
    for n in (1, 2, 4):
        x = common.activations_f32(K + n, n, K)
        pos = np.array([37, 0, 4095, 100000][:n], np.int32)
        q, k, v = dev.mul_mat_group(members, x)
        a, b = dev.rope_two(q.reshape(n, n_head, hd), k.reshape(n, n_head_kv, hd), pos, n_dims, mode, want=(("f32",), ("f32", "f16")),
                            freq_base=500000.0)
        ropes = [(hd, n_dims, mode, ("f32",)), (hd, n_dims, mode, ("f32", "f16")), None]
        rc, got = dev.mul_mat_group_rope(members, x, pos, ropes, freq_base=500000.0)
        assert got[0]["f32"].tobytes() == a["f32"].tobytes(), n
        assert got[1]["f32"].tobytes() == b["f32"].tobytes() and got[1]["f16"].tobytes() == b["f16"].tobytes(), n
        assert got[2]["y"].tobytes() == v.tobytes(), n
        ropes = [(hd, n_dims, mode, ("f32",)), (hd, n_dims, mode, ("f16",)), None]       # K's F32 result has no other reader
        rc, got = dev.mul_mat_group_rope(members, x, pos, ropes, freq_base=500000.0)
        assert got[0]["f32"].tobytes() == a["f32"].tobytes() and got[1]["f16"].tobytes() == b["f16"].tobytes(), n
    import cactus_amd as ca
    x = common.activations_f32(K, 3, K)
    rc, _ = dev.mul_mat_group_rope(members, x, np.arange(3, dtype=np.int32), [(hd, n_dims, mode, ("f32",)), None, None], check=False)
    assert rc == ca.CHIP_EUNSUPPORTED                                            # 3 tokens: no one-launch form
    x = common.activations_f32(K, 1, K)
    rc, _ = dev.mul_mat_group_rope(members, x, np.zeros(1, np.int32), [(hd + 2, n_dims, mode, ("f32",)), None, None], check=False)
    assert rc in (ca.CHIP_EUNSUPPORTED, ca.CHIP_EINVAL)                          # rows are no whole heads of that size
    rc, _ = dev.mul_mat_group_rope(members, x, np.zeros(1, np.int32), [(hd, n_dims, 8, ("f32",)), None, None], check=False)
    assert rc == ca.CHIP_EUNSUPPORTED                                            # multi-section mode


FUSED_FORM_TYPES = (O.Q4_K, O.Q8_0, O.Q4_0, O.Q6_K, O.Q5_1, O.F16, O.Q5_K, O.IQ4_NL, O.Q3_K, O.Q2_K, O.IQ4_XS)


def types_and_shapes(shapes, large, large_types):
    """(type, K, N) for every type and shape; the large shape only for large_types (once per activation family is enough)."""
    return [pytest.param(wt, K, N, id="%s-%dx%d" % (O.TYPE_NAMES[wt], N, K)) for (K, N) in shapes for wt in FUSED_FORM_TYPES
            if (K, N) != large or wt in large_types]


@pytest.mark.parametrize("wt,K,N", types_and_shapes([(1024, 336), (4096, 1032), (4096, 14336), (256, 8), (2048, 4104)], (4096, 14336), (O.Q4_K, O.Q4_0)))
def test_gated_pair_equals_the_pair_and_silu_mul(dev, wt, K, N):
    """chip_mul_mat_pair_silu_mul (ffn_gate, SILU, ffn_up and their MUL in one launch): bit for bit chip_silu_mul of
    chip_mul_mat_pair's two outputs, for a few rows, more rows than a pass of the grid takes, and 1, 2 and 4 tokens; declined
    for other token counts and for row counts that are no multiple of 8 (chip_silu's rule)."""
    import cactus_amd as ca
    w1 = quantized_weights(wt, K + N, N, K)
    w2 = quantized_weights(wt, K + N + 1, N, K)
    for n in (1, 2, 4):
        x = common.activations_f32(K + n, n, K)
        if not dev.lib.chip_mul_mat_pair_silu_mul_supported(wt, K, N, n):
            assert n * K > 16384
            continue
        y1, y2 = dev.mul_mat_pair(wt, w1, w2, x)
        want = dev.silu_mul(y1, y2)
        got = dev.mul_mat_pair_silu_mul(wt, w1, w2, x)
        assert got.tobytes() == want.tobytes(), n
    assert dev.lib.chip_mul_mat_pair_silu_mul_supported(wt, K, N, 3) == 0
    assert dev.lib.chip_mul_mat_pair_silu_mul_supported(wt, K, N, 8) == 0
    assert dev.lib.chip_mul_mat_pair_silu_mul_supported(wt, K, N + 4, 1) == 0
    d = dev.alloc(4096)
    assert dev.lib.chip_mul_mat_pair_silu_mul(wt, d.ptr, d.ptr, 16, K, N, d.ptr, K, 3, d.ptr, N, d.ptr, 4096, None) == ca.CHIP_EUNSUPPORTED


def norm_weight(seed, K):
    return (1.0 + 0.25 * np.random.default_rng(seed).standard_normal(K)).astype(np.float32)


@pytest.mark.parametrize("types,K,n_head,n_head_kv,hd,n_dims,mode", GROUP_ROPE_CASES)
def test_group_with_the_norm_in_its_prologue_equals_norm_then_group(dev, types, K, n_head, n_head_kv, hd, n_dims, mode):
    """chip_mul_mat_group_rope_norm (attn_norm, its weight MUL, wq / wk / wv, both ROPE nodes and the K cache store in one
    launch): every value, the normed rows included, bit for bit what chip_rms_norm_mul followed by chip_mul_mat_group_rope
    gives."""
    members = [(types[0], quantized_weights(types[0], K + 1, n_head * hd, K)), (types[1], quantized_weights(types[1], K + 2, n_head_kv * hd, K)),
               (types[2], quantized_weights(types[2], K + 3, n_head_kv * hd, K))]
    w = norm_weight(K, K)
    ropes = [(hd, n_dims, mode, ("f32",)), (hd, n_dims, mode, ("f32", "f16")), None]
    for n in (1, 2, 4):
        x = common.activations_f32(K + n, n, K) * np.float32(3.0)
        pos = np.array([37, 0, 4095, 100000][:n], np.int32)
        assert dev.lib.chip_norm_before_supported(types[0], K, n) == 1
        normed = dev.rms_norm_mul(x, w, 1e-5)
        rc, want = dev.mul_mat_group_rope(members, normed, pos, ropes, freq_base=500000.0)
        rc, got = dev.mul_mat_group_rope(members, x, pos, ropes, freq_base=500000.0, norm=(w, 1e-5))
        assert got[3]["normed"].tobytes() == normed.tobytes(), n
        assert got[0]["f32"].tobytes() == want[0]["f32"].tobytes(), n
        assert got[1]["f32"].tobytes() == want[1]["f32"].tobytes() and got[1]["f16"].tobytes() == want[1]["f16"].tobytes(), n
        assert got[2]["y"].tobytes() == want[2]["y"].tobytes(), n


@pytest.mark.parametrize("wt,K,N", types_and_shapes([(1024, 336), (4096, 14336), (256, 8), (8192, 1032)], (4096, 14336), (O.Q4_K, O.Q4_0)))
def test_gated_pair_with_the_norm_in_its_prologue(dev, wt, K, N):
    """chip_mul_mat_pair_silu_mul_norm (ffn_norm, its weight MUL and the gated pair in one launch): bit for bit chip_rms_norm_mul
    followed by chip_mul_mat_pair_silu_mul; rows the prologue does not hold whole are declined."""
    import cactus_amd as ca
    w1 = quantized_weights(wt, K + N, N, K)
    w2 = quantized_weights(wt, K + N + 1, N, K)
    w = norm_weight(N, K)
    for n in (1, 2, 4):
        if not dev.lib.chip_mul_mat_pair_silu_mul_supported(wt, K, N, n):
            assert n * K > 16384
            continue
        x = common.activations_f32(K + n, n, K) * np.float32(0.25)
        assert dev.lib.chip_norm_before_supported(wt, K, n) == 1
        normed = dev.rms_norm_mul(x, w, 1e-6)
        want = dev.mul_mat_pair_silu_mul(wt, w1, w2, normed)
        got, got_normed = dev.mul_mat_pair_silu_mul(wt, w1, w2, x, norm=(w, 1e-6))
        assert got_normed.tobytes() == normed.tobytes(), n
        assert got.tobytes() == want.tobytes(), n
    assert dev.lib.chip_norm_before_supported(O.Q4_K, 14336, 1) == 0           # the image of such a row is built a step's part at a time
    assert dev.lib.chip_norm_before_supported(wt, K, 3) == 0
    d = dev.alloc(4096)
    nb = ca.NormBefore(d.ptr, 1e-6, None, 0)
    import ctypes
    assert dev.lib.chip_mul_mat_pair_silu_mul_norm(O.Q4_K, d.ptr, d.ptr, 8064, 14336, 8, d.ptr, 14336, 1, ctypes.byref(nb), d.ptr, 8, d.ptr,
                                                   65536, None) == ca.CHIP_EUNSUPPORTED


@pytest.mark.parametrize("wt,K,N", types_and_shapes([(1024, 333), (4096, 4096), (14336, 4096), (256, 7)], (14336, 4096), (O.Q4_K, O.Q6_K, O.Q8_0)))
def test_matmul_with_the_residual_add_in_its_store(dev, wt, K, N):
    """chip_mul_mat_add (wo / ffn_down and the residual ADD behind them in one launch): bit for bit chip_mul_mat followed by
    chip_add, with the result written apart from the addend and over it."""
    import cactus_amd as ca
    W = quantized_weights(wt, K + N, N, K)
    for n in (1, 2, 4):
        if not dev.lib.chip_mul_mat_add_supported(wt, K, N, n):
            assert n * K > 16384
            continue
        x = common.activations_f32(K + n, n, K)
        b = common.activations_f32(N + n, n, N) * np.float32(5.0)
        want = dev.binary("add", dev.mul_mat(wt, W, x), b)
        assert dev.mul_mat_add(wt, W, x, b).tobytes() == want.tobytes(), n
        assert dev.mul_mat_add(wt, W, x, b, in_place=True).tobytes() == want.tobytes(), n
    assert dev.lib.chip_mul_mat_add_supported(wt, K, N, 3) == 0
    d = dev.alloc(4096)
    assert dev.lib.chip_mul_mat_add(wt, d.ptr, 16, K, N, d.ptr, K, 8, d.ptr, N, d.ptr, N, d.ptr, 4096, None) == ca.CHIP_EUNSUPPORTED


@pytest.mark.parametrize("wt,K,N", [(O.Q4_K, 4096, 8192), (O.Q4_K, 4096, 14336), (O.Q5_K, 2048, 16400), (O.Q4_K, 14336, 4096)],
                         ids=["q4_K-8192x4096", "q4_K-14336x4096", "q5_K-16400x2048", "q4_K-4096x14336"])
def test_mul_mat_pair_on_the_matrix_cores(dev, orc, wt, K, N):
    """ffn_gate and ffn_up at 5..8 tokens: matrices large enough for the matrix-core GEMV run as one launch, through
    chip_mul_mat_pair and through chip_mul_mat_group (fp32 rows and prepared rows); each output equals the single call's bit
    for bit (a row count that is no multiple of 16 puts a partial tile at the end of each matrix), oracle within tolerance."""
    w1 = quantized_weights(wt, K + N, N, K)
    w2 = quantized_weights(wt, K + N + 1, N, K)
    for n in (5, 7, 8):
        x = common.activations_f32(K + n, n, K)
        a, b = dev.mul_mat(wt, w1, x), dev.mul_mat(wt, w2, x)
        y1, y2 = dev.mul_mat_pair(wt, w1, w2, x)
        assert y1.tobytes() == a.tobytes() and y2.tobytes() == b.tobytes(), n
        for prepared in (False, True):
            g1, g2 = dev.mul_mat_group([(wt, w1), (wt, w2)], x, prepared=prepared)[:2]
            assert g1.tobytes() == a.tobytes() and g2.tobytes() == b.tobytes(), (n, prepared)
        if n == 8:
            ref = orc.mul_mat(wt, w2, x, nthreads=8, want=("sum_abs",))
            check_outputs(y2, ref["y"], ref["sum_abs"], "second matrix of the pair, n = 8")


@pytest.mark.parametrize("wt", (O.Q6_K, O.Q4_K, O.Q8_0, O.Q4_0), ids=lambda t: O.TYPE_NAMES[t])
def test_mul_mat_with_transposed_fp16_store(dev, wt):
    """chip_mul_mat_store_t (the V projection and its store into the transposed F16 cache): y equals chip_mul_mat's bit for
    bit, the fp16 matrix holds y transposed and rounded to nearest even in its first n columns and is untouched elsewhere;
    1, 2, 4 tokens in one launch, 3 and 9 through the matmul and the copy."""
    K, N, ld16 = 1024, 515, 24
    w = quantized_weights(wt, K + N + 5, N, K)
    for n in (1, 2, 4, 3, 9):
        x = common.activations_f32(K + n, n, K)
        y, h = dev.mul_mat_store_t(wt, w, x, ld16)
        assert y.tobytes() == dev.mul_mat(wt, w, x).tobytes(), n
        assert h[:, :n].tobytes() == np.ascontiguousarray(y.T.astype(np.float16)).view(np.uint16).tobytes(), n
        assert (h[:, n:] == 0x7bff).all(), n


# ------------------------------------------------------------------------------------------ rows of K % 256 != 0
@pytest.mark.parametrize("wt", (O.Q4_0, O.Q8_0, O.Q5_0, O.IQ4_NL, O.Q4_1, O.Q5_1), ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("K,N", [(576, 1536), (896, 151), (960, 2560), (4160, 300), (64, 5)])
def test_block32_rows_of_k_not_a_multiple_of_256(dev, orc, wt, K, N):
    """Hidden sizes such as 576, 896 and 960 (K % 64 == 0): the rows of the 32-value block types are then multiples of 4
    bytes only.  Every token count class: prologue-quantizing GEMV (1, 2, 4), GEMV over the workspace (3, 5, 8), several
    passes (11, 20), and from 17 tokens the GEMM where K % 128 == 0 (896, 960 is not: passes)."""
    import cactus_amd as ca
    assert dev.lib.chip_mul_mat_supported(wt, K) == 1
    wq = quantized_weights(wt, 7 * K + N, N, K)
    for n in (1, 2, 3, 4, 5, 8, 11, 20, 70):
        x = common.activations_f32(K + n, n, K)
        ref = orc.mul_mat(wt, wq, x, nthreads=8, want=("wdata", "sum_abs"))
        y, blocks = dev.mul_mat(wt, wq, x, want_workspace_blocks=True)
        assert np.array_equal(blocks, ref["wdata"]), n
        check_outputs(y, ref["y"], ref["sum_abs"], "K %% 256 != 0, n = %d" % n)
    for t in (O.Q4_K, O.Q5_K, O.Q6_K):
        assert dev.lib.chip_mul_mat_supported(t, K) == 0                 # super-blocks of 256 values
    assert dev.lib.chip_mul_mat_supported(wt, K + 32) == 0              # an odd number of blocks: rows of 2-byte alignment


# ------------------------------------------------------------------------------------------ prefill GEMM (int8 MFMA)
B32_TYPES = (O.Q4_0, O.Q8_0, O.Q5_0, O.IQ4_NL, O.Q4_1, O.Q5_1)


@pytest.mark.parametrize("wt", B32_TYPES, ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("K,N,n", [(256, 1, 49), (512, 40, 50), (1024, 131, 64), (4096, 300, 130), (2048, 260, 257),
                                   (4096, 12300, 33)])
def test_gemm_block32_vs_oracle(dev, orc, wt, K, N, n):
    print("gemm", O.TYPE_NAMES[wt], "K", K, "N", N, "n", n, flush=True)
    wq = orc.quantize_weights(wt, common.weights_f32(K + N, N, K))
    x = common.activations_f32(K + n, n, K)
    x[3] = 0
    ref = orc.mul_mat(wt, wq, x, nthreads=8, want=("wdata", "sum_abs"))
    y, blocks = dev.mul_mat(wt, wq, x, want_workspace_blocks=True)
    assert np.array_equal(blocks, ref["wdata"])
    check_outputs(y, ref["y"], ref["sum_abs"], "gemm")


@pytest.mark.parametrize("wt", B32_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_gemm_block32_integer_sums_bit_exact(dev, orc, wt):
    """With every scale equal to 1 the fp32 output is the integer sum itself, so the MFMA path's per-block
    integer dot sums can be compared bit for bit: one block at a time (all other weight scales zero), then all.
    The weight bytes are random, so every nibble / fifth bit / code index / int8 value occurs."""
    K, N, n = 256, 70, 56                                 # from 49 tokens on every block-32 type takes the GEMM
    rng = np.random.default_rng(9 + wt)
    bb = O.BLOCK_BYTES[wt]
    x = rng.integers(-127, 128, (n, K)).astype(np.float32)
    x[:, ::32] = 127.0                                   # amax = 127 in every block -> d = 1, q = x
    x[5, 64:96] = 0.0                                    # one all-zero activation block
    aq = orc.quantize_activation(O.Q8_0, x)
    aq1 = orc.quantize_activation(O.Q8_1, x)
    for only in list(range(K // 32)) + [None]:
        w = rng.integers(0, 256, (N, K // 32, bb), dtype=np.uint8)
        w[..., :2] = 0
        if wt in (O.Q4_1, O.Q5_1):
            w[..., 2:4] = 0                              # block minimum 0: the output is the integer sums alone
        sel = slice(None) if only is None else only
        w[:, sel, :2] = np.array([1.0], np.float16).view(np.uint8)
        w = w.reshape(N, -1)
        y = dev.mul_mat(wt, w, x)
        want = np.zeros((n, N), np.int64)
        for t in range(n):
            for i in range(N):
                _, isum, _ = orc.vec_dot(wt, K, w[i], aq1[t] if wt in (O.Q4_1, O.Q5_1) else aq[t], want_sums=True)
                want[t, i] = isum.sum() if only is None else isum[only]
        assert np.array_equal(y.astype(np.int64), want) and np.array_equal(y, want.astype(np.float32))


@pytest.mark.parametrize("N,M", [(4096, 512), (14336, 2048)])
def test_config4_prefill_sampled(dev, orc, N, M):
    """BASELINE prefill shapes: full-size run on the GPU, oracle on a sample of rows and tokens."""
    K = 4096
    print("config4", N, M, flush=True)
    rng = np.random.default_rng(N + M)
    wq = orc.quantize_weights(O.Q4_0, common.weights_f32(4, N, K))
    x = common.activations_f32(4, M, K)
    y = dev.mul_mat(O.Q4_0, wq, x)
    rows = np.sort(rng.choice(N, 96, replace=False))
    rows[:3] = [0, 1, 2]; rows[-1] = N - 1
    toks = np.sort(rng.choice(M, 24, replace=False))
    toks[0] = 0; toks[-1] = M - 1
    ref = orc.mul_mat(O.Q4_0, wq[rows], x[toks], nthreads=8, want=("sum_abs",))
    check_outputs(y[np.ix_(toks, rows)], ref["y"], ref["sum_abs"], "config 4")
    # linearity across tokens is not available (quantization is per row), but row order independence is:
    # the same weights reversed must give the same numbers reversed
    y2 = dev.mul_mat(O.Q4_0, wq[::-1].copy(), x[:64], split_k=False)    # the same walk over K as y: the same bits
    assert np.array_equal(y2[:, ::-1], y[:64])


@pytest.mark.parametrize("K,N,n", [(256, 1, 32), (512, 40, 33), (1024, 131, 64), (4096, 300, 130), (2048, 260, 257)])
def test_gemm_f16_vs_oracle(dev, orc, K, N, n):
    print("gemm f16 K", K, "N", N, "n", n, flush=True)
    wq = orc.quantize_weights(O.F16, common.weights_f32(K + N, N, K, outliers=True))
    x = common.activations_f32(K + n, n, K)
    x[3] = 0
    ref = orc.mul_mat(O.F16, wq, x, nthreads=8, want=("wdata", "sum_abs"))
    y, blocks = dev.mul_mat(O.F16, wq, x, want_workspace_blocks=True)
    assert np.array_equal(blocks, ref["wdata"])
    check_outputs(y, ref["y"], ref["sum_abs"], "f16 gemm")


@pytest.mark.parametrize("K,N,n", [(256, 4096, 2048), (512, 3841, 2305), (768, 8200, 1025)])
def test_gemm_f16_large_shape_kernel_vs_oracle(dev, orc, K, N, n):
    """Shapes with at least one 256 x 256 output tile for every second CU take the large-tile kernel (operands loaded
    straight into LDS): whole and ragged edge tiles in both directions, a K loop shorter and longer than its pipeline."""
    print("gemm f16 large K", K, "N", N, "n", n, flush=True)
    assert -(-N // 256) * -(-n // 256) * 2 >= 256
    wq = orc.quantize_weights(O.F16, common.weights_f32(K + N, N, K, outliers=True))
    x = common.activations_f32(K + n, n, K)
    x[3] = 0
    y = dev.mul_mat(O.F16, wq, x)
    rng = np.random.default_rng(K)
    rows = np.unique(np.concatenate([[0, 1, 255, 256, N - 257, N - 2, N - 1], rng.choice(N, 160, replace=False)]))
    toks = np.unique(np.concatenate([[0, 3, 255, 256, n - 257, n - 2, n - 1], rng.choice(n, 40, replace=False)]))
    ref = orc.mul_mat(O.F16, wq[rows], x[toks], nthreads=8, want=("sum_abs",))
    check_outputs(y[np.ix_(toks, rows)], ref["y"], ref["sum_abs"], "f16 large-shape gemm")
    assert np.isfinite(y).all() and not y[3].any()


def test_gemm_f16_large_shape_kernel_exact_small_integers(dev):
    """Every output of the large-tile kernel, not a sample: integer operands whose dot products fp32 holds exactly."""
    K, N, n = 512, 4100, 2050
    rng = np.random.default_rng(4)
    w = rng.integers(-32, 33, (N, K)).astype(np.float32)
    x = rng.integers(-32, 33, (n, K)).astype(np.float32)
    y = dev.mul_mat(O.F16, w.astype(np.float16).view(np.uint8).reshape(N, -1), x)
    assert np.array_equal(y, x @ w.T)


def test_f16_rows_of_k_not_a_multiple_of_256_are_rejected(dev):
    """F16 weights (like the K-quants) are taken in rows of K % 256 == 0 only: the C-ABI says so instead of computing."""
    K, N, n = 64, 70, 40
    assert dev.lib.chip_mul_mat_supported(O.F16, K) == 0
    assert dev.lib.chip_mul_mat_workspace_size(O.F16, K, n) == 0
    buf = dev.alloc(1 << 16)
    assert dev.lib.chip_mul_mat(O.F16, buf.ptr, 2 * K, K, N, buf.ptr, K, n, buf.ptr, N, buf.ptr, 1 << 16, None) == -2
    assert dev.lib.chip_mul_mat_prepare(O.F16, K, buf.ptr, K, n, buf.ptr, 1 << 16, None) == -2
    dev.sync()


def test_gemm_f16_exact_small_integers(dev, orc):
    """Small integer weights and activations: every product and partial sum is an integer below 2^24, so the fp16 MFMA
    with fp32 accumulation must give the exact dot products whatever its summation order."""
    K, N, n = 512, 100, 64
    rng = np.random.default_rng(3)
    w = rng.integers(-64, 65, (N, K)).astype(np.float32)
    x = rng.integers(-64, 65, (n, K)).astype(np.float32)
    y = dev.mul_mat(O.F16, w.astype(np.float16).view(np.uint8).reshape(N, -1), x)
    assert np.array_equal(y, x @ w.T)


# ------------------------------------------------------------------------------------------ K-quant prefill GEMM
KQ_TYPES = (O.Q4_K, O.Q5_K, O.Q6_K)


@pytest.mark.parametrize("wt", KQ_TYPES, ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("K,N,n", [(256, 1, 49), (512, 40, 50), (1024, 131, 64), (4096, 300, 130), (2048, 260, 257),
                                   (4096, 12300, 33)])
def test_gemm_kquant_vs_oracle(dev, orc, wt, K, N, n):
    print("gemm", O.TYPE_NAMES[wt], "K", K, "N", N, "n", n, flush=True)
    wq = orc.quantize_weights(wt, common.weights_f32(K + N + wt, N, K, outliers=True))
    x = common.activations_f32(K + n + wt, n, K)
    x[3] = 0
    ref = orc.mul_mat(wt, wq, x, nthreads=8, want=("wdata", "sum_abs"))
    y, blocks = dev.mul_mat(wt, wq, x, want_workspace_blocks=True)
    assert np.array_equal(blocks, ref["wdata"])
    check_outputs(y, ref["y"], ref["sum_abs"], "k-quant gemm")


def random_kquant_rows(wt, rng, N, nsb, extreme_rows=0):
    """Raw super-blocks with every super-block scale (d, dmin) equal to 1 and random bytes everywhere else, so all
    6-bit / 8-bit sub-block scales and quants occur; the first `extreme_rows` rows use saturating bytes."""
    one = np.array([1.0], np.float16).view(np.uint8)
    bb = O.BLOCK_BYTES[wt]
    w = rng.integers(0, 256, (N, nsb, bb), dtype=np.uint8)
    fills = (0xFF, 0x00, 0x80, 0x7F)
    for r in range(extreme_rows):
        w[r] = fills[r % 4]
    if wt == O.Q6_K:
        w[..., 208:210] = one
    else:
        w[..., 0:2] = one
        w[..., 2:4] = one
    return w.reshape(N, -1)


def exact_q8_K_inputs(rng, n, K):
    """Integer activations whose first largest-magnitude value per super-block is -127: Q8_K then has
    iscale = -127 / max = 1, so d = 1 and q = x."""
    x = rng.integers(-127, 128, (n, K)).astype(np.float32)
    x[:, ::256] = -127.0
    return x


@pytest.mark.parametrize("wt", KQ_TYPES + B32_TYPES, ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("K,N,n", [(4096, 300, 64), (2304, 131, 70), (14336, 200, 128), (4096, 8000, 50)])
def test_gemm_split_k_vs_oracle(dev, orc, wt, K, N, n):
    """Few tokens on a matrix with few row tiles: K is cut into slices run by separate workgroups and a second kernel adds
    the partial outputs in slice order (uneven slices at K = 2304; N = 131 is no multiple of the adder's four rows).
    Against the oracle, against the unsplit GEMM, and the same bits on a second run."""
    import cactus_amd as ca
    print("split-k gemm", O.TYPE_NAMES[wt], "K", K, "N", N, "n", n, flush=True)
    act = dev.lib.chip_mul_mat_workspace_size(wt, K, n)
    assert dev.lib.chip_mul_mat_workspace_size_n(wt, K, N, n) > act                   # this case does split
    wq = quantized_weights(wt, K + N, N, K)
    x = common.activations_f32(K + n, n, K)
    ref = orc.mul_mat(wt, wq, x, nthreads=8, want=("sum_abs",))
    y = dev.mul_mat(wt, wq, x)
    check_outputs(y, ref["y"], ref["sum_abs"], "split-k gemm")
    check_outputs(dev.mul_mat(wt, wq, x, split_k=False), ref["y"], ref["sum_abs"], "unsplit gemm")
    assert dev.mul_mat(wt, wq, x).tobytes() == y.tobytes()


@pytest.mark.parametrize("wt", KQ_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_gemm_kquant_integer_sums_bit_exact(dev, orc, wt):
    """With d = dmin = 1 and activation scale 1 the fp32 output of a one-super-block product is sumi - summ itself
    (below 2^24), so the digit planes folded into the MFMA operand are compared bit for bit with the reference's
    integer sums, over random scale and quant bytes."""
    K, N, n = 256, 150, 56                                # from 49 tokens on every K-quant takes the GEMM
    rng = np.random.default_rng(77 + wt)
    w = random_kquant_rows(wt, rng, N, 1)
    x = exact_q8_K_inputs(rng, n, K)
    x[7, 1:] = 0.0
    aq = orc.quantize_activation(O.Q8_K, x)
    assert np.array_equal(aq[:, 4:4 + K].view(np.int8).astype(np.float32), x) and (aq[:, :4].view(np.float32) == 1).all()
    y = dev.mul_mat(wt, w, x)
    want = np.zeros((n, N), np.int64)
    for t in range(n):
        for i in range(N):
            _, isum, imin = orc.vec_dot(wt, K, w[i], aq[t], want_sums=True)
            want[t, i] = int(isum.sum()) - int(imin.sum())
    assert np.abs(want).max() < 2 ** 24
    assert np.array_equal(y.astype(np.int64), want)


@pytest.mark.parametrize("wt", KQ_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_gemm_kquant_extreme_bytes(dev, orc, wt):
    # saturating scale / quant bytes in the first rows, activations pinned at +-127: the operand digits at their limits
    K, N, n = 1024, 64, 64
    rng = np.random.default_rng(5 + wt)
    w = random_kquant_rows(wt, rng, N, K // 256, extreme_rows=8)
    x = exact_q8_K_inputs(rng, n, K)
    x[0, :] = 127.0
    x[1, :] = -127.0
    x[0:2, ::256] = -127.0
    ref = orc.mul_mat(wt, w, x, nthreads=8, want=("sum_abs",))
    check_outputs(dev.mul_mat(wt, w, x), ref["y"], ref["sum_abs"], "extreme bytes")


@pytest.mark.parametrize("wt", KQ_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_gemm_kquant_prefill_shape_sampled(dev, orc, wt):
    """A full prefill shape on the GPU, the oracle on a sample of rows and tokens, and row-order independence."""
    K, N, M = 4096, 4096, 512
    rng = np.random.default_rng(wt)
    wq = orc.quantize_weights(wt, common.weights_f32(40 + wt, N, K))
    x = common.activations_f32(40 + wt, M, K)
    y = dev.mul_mat(wt, wq, x)
    rows = np.sort(rng.choice(N, 64, replace=False))
    rows[:2] = [0, 1]; rows[-1] = N - 1
    toks = np.sort(rng.choice(M, 16, replace=False))
    toks[0] = 0; toks[-1] = M - 1
    ref = orc.mul_mat(wt, wq[rows], x[toks], nthreads=8, want=("sum_abs",))
    check_outputs(y[np.ix_(toks, rows)], ref["y"], ref["sum_abs"], "k-quant prefill")
    y2 = dev.mul_mat(wt, wq[::-1].copy(), x[:64], split_k=False)      # the same walk over K: the same bits, whatever the tile
    assert np.array_equal(y2[:, ::-1], y[:64])


@pytest.mark.parametrize("wt", (O.Q4_K, O.Q5_K), ids=lambda t: O.TYPE_NAMES[t])
def test_gemm_kquant_single_plane_kernel(dev, orc, wt):
    """Shapes with many output tiles take the kernel that feeds the quants as one int8 plane and applies the 6-bit
    sub-block scales with integer multiply-adds.  (a) d = dmin = 1, activation scale 1, one super-block: the output is
    sumi - summ itself, compared bit for bit with the reference's integer sums on a sample that covers the first and the
    last (ragged) tiles; (b) real scales over four super-blocks against the oracle within the tolerance; (c) the same bits
    whatever tile a row lands in."""
    N, M = 4090, 1000                                    # 64 x 8 tiles of 64 rows x 128 tokens, both edges ragged
    rng = np.random.default_rng(31 + wt)
    rows = np.unique(np.concatenate([[0, 1, 63, 64, N - 1, N - 2], rng.choice(N, 40, replace=False)]))
    toks = np.unique(np.concatenate([[0, 31, 32, 127, 128, M - 1], rng.choice(M, 18, replace=False)]))
    # (a)
    K = 256
    w = random_kquant_rows(wt, rng, N, 1)
    x = exact_q8_K_inputs(rng, M, K)
    x[7, 1:] = 0.0
    aq = orc.quantize_activation(O.Q8_K, x)
    y = dev.mul_mat(wt, w, x, split_k=False)
    for t in toks:
        for i in rows:
            _, isum, imin = orc.vec_dot(wt, K, w[i], aq[t], want_sums=True)
            want = int(isum.sum()) - int(imin.sum())
            assert abs(want) < 2 ** 24 and int(y[t, i]) == want and float(y[t, i]) == float(want), (t, i)
    # (b), (c)
    K = 1024
    wq = orc.quantize_weights(wt, common.weights_f32(90 + wt, N, K, outliers=True))
    x = common.activations_f32(90 + wt, M, K)
    y = dev.mul_mat(wt, wq, x, split_k=False)
    ref = orc.mul_mat(wt, wq[rows], x[toks], nthreads=8, want=("sum_abs",))
    check_outputs(y[np.ix_(toks, rows)], ref["y"], ref["sum_abs"], "single-plane k-quant gemm")
    y2 = dev.mul_mat(wt, wq[::-1].copy(), x, split_k=False)
    assert np.array_equal(y2[:, ::-1], y)


# ------------------------------------------------------------------------------------------ MUL_MAT_ID (expert matmul)
def moe_case(orc, wt, K, N, n_as, n_used, n_tokens, ne11, seed):
    rng = np.random.default_rng(seed)
    W = np.stack([orc.quantize_weights(wt, common.weights_f32(seed + e, N, K)) for e in range(n_as)])
    x = common.activations_f32(seed + 100, n_tokens * ne11, K).reshape(n_tokens, ne11, K)
    ids = np.stack([rng.permutation(n_as)[:n_used] for _ in range(n_tokens)]).astype(np.int32)
    return W, x, ids


@pytest.mark.parametrize("wt", O.WEIGHT_TYPES, ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("n_tokens,ne11", [(1, 1), (2, 4), (9, 1)])
def test_mul_mat_id_vs_oracle(dev, orc, wt, n_tokens, ne11):
    # decode (one token, fused quantize), per-slot activations, and more pairs than the fused path takes
    K, N, n_as, n_used = 1024, 200, 8, 4
    W, x, ids = moe_case(orc, wt, K, N, n_as, n_used, n_tokens, ne11, 700 + wt)
    ref = orc.mul_mat_id(wt, W, x, ids, nthreads=8, want=("sum_abs",))
    y = dev.mul_mat_id(wt, W, x, ids)
    check_outputs(y, ref["y"], ref["sum_abs"], "mul_mat_id")


@pytest.mark.parametrize("wt", (O.Q4_K, O.Q8_0), ids=lambda t: O.TYPE_NAMES[t])
def test_mul_mat_id_golden(dev, orc, wt):
    g = np.load(os.path.join(GOLD, "mul_mat_id_%s.npz" % O.TYPE_NAMES[wt]))
    sa = orc.mul_mat_id(wt, g["W"], g["x"], g["ids"], want=("sum_abs",))["sum_abs"]
    check_outputs(dev.mul_mat_id(wt, g["W"], g["x"], g["ids"]), g["y_graph"], sa, "mul_mat_id golden")


def test_mul_mat_id_is_mul_mat_on_the_chosen_expert(dev, orc):
    """Same device code as MUL_MAT: each (token, slot) output equals chip_mul_mat on that expert, bit for bit; repeated
    experts and a long K (activation quantized ahead of the GEMV) included."""
    wt, K, N, n_as, n_used, n_tokens = O.Q4_K, 8192, 96, 5, 3, 4
    W, x, ids = moe_case(orc, wt, K, N, n_as, n_used, n_tokens, 1, 41)
    ids[1] = [2, 2, 2]
    y = dev.mul_mat_id(wt, W, x, ids)
    for t in range(n_tokens):
        for s in range(n_used):
            one = dev.mul_mat(wt, W[ids[t, s]], x[t])
            assert np.array_equal(y[t, s], one[0])


@pytest.mark.parametrize("wt", O.WEIGHT_TYPES, ids=lambda t: O.TYPE_NAMES[t])
@pytest.mark.parametrize("n_tokens,ne11,n_as", [(16, 1, 8), (50, 4, 6), (130, 1, 32)])
def test_mul_mat_id_prefill_grouped_by_expert(dev, orc, wt, n_tokens, ne11, n_as):
    """64 (token, slot) pairs and more: grouped by expert on the device and run through the GEMMs.  Uneven loads: one
    expert gets a pair from every token, some get none."""
    K, N, n_used = 512, 150, 4
    rng = np.random.default_rng(900 + wt + n_tokens)
    W = np.stack([orc.quantize_weights(wt, common.weights_f32(900 + wt + e, N, K)) for e in range(n_as)])
    x = common.activations_f32(901 + wt, n_tokens * ne11, K).reshape(n_tokens, ne11, K)
    pool = np.arange(1, n_as - 2)                                    # experts n_as-2 and n_as-1 stay idle
    ids = np.stack([np.concatenate(([0], rng.permutation(pool)[:n_used - 1])) for _ in range(n_tokens)]).astype(np.int32)
    ref = orc.mul_mat_id(wt, W, x, ids, nthreads=8, want=("sum_abs",))
    y = dev.mul_mat_id(wt, W, x, ids)
    check_outputs(y, ref["y"], ref["sum_abs"], "mul_mat_id grouped")


def test_mul_mat_id_grouped_matches_pairwise_and_skips_bad_ids(dev, orc):
    """The grouped GEMM path and the pair-by-pair GEMV path agree within the tolerance on the same inputs (first 15
    tokens alone take the GEMV path), and an id outside [0, n_as) leaves exactly its own output row unwritten."""
    wt, K, N, n_as, n_used, n_tokens = O.Q4_K, 1024, 96, 8, 4, 40
    W, x, ids = moe_case(orc, wt, K, N, n_as, n_used, n_tokens, 1, 77)
    ids[7, 2] = n_as + 5
    ids[9, 0] = -1
    y = dev.mul_mat_id(wt, W, x, ids)
    bad = np.zeros((n_tokens, n_used), bool)
    bad[7, 2] = bad[9, 0] = True
    assert np.isnan(y[bad]).all() and np.isfinite(y[~bad]).all()
    y15 = dev.mul_mat_id(wt, W, x[:15], ids[:15])
    good = ~bad[:15]
    ok_ids = np.where(bad, 0, ids)
    sa = orc.mul_mat_id(wt, W, x, ok_ids, nthreads=8, want=("sum_abs",))["sum_abs"]
    assert (np.abs(y[:15][good].astype(np.float64) - y15[good]) <= 2 * REL_TOL * sa[:15][good]).all()


def test_mul_mat_id_argument_errors(dev, orc):
    import cactus_amd as ca
    L = dev.lib
    wt, K, N = O.Q8_0, 256, 8
    W, x, ids = moe_case(orc, wt, K, N, 2, 2, 1, 1, 5)
    nb01 = dev.row_size(wt, K)
    dW, dx, di, dy = dev.to_device(W), dev.to_device(x), dev.to_device(ids), dev.alloc(2 * N * 4)
    wsz = L.chip_mul_mat_id_workspace_size(wt, K, 2, 2, 1, 1)
    assert wsz > L.chip_mul_mat_workspace_size(wt, K, 1)
    ws = dev.alloc(wsz)
    call = lambda **kw: L.chip_mul_mat_id(*[kw.get(k, v) for k, v in (
        ("type", wt), ("W", dW.ptr), ("nb01", nb01), ("nb02", N * nb01), ("K", K), ("N", N), ("n_as", 2), ("x", dx.ptr),
        ("ldx", K), ("ne11", 1), ("ids", di.ptr), ("ids_stride", 2), ("n_used", 2), ("n_tokens", 1), ("y", dy.ptr),
        ("ldy", N), ("ws", ws.ptr), ("wsz", wsz), ("stream", None))])
    assert call() == 0
    assert call(type=30) != 0 and call(ne11=3) != 0 and call(ids=None) != 0 and call(wsz=16) != 0
    assert call(nb02=nb01) != 0 and call(ldy=N - 1) != 0 and call(n_tokens=0) == 0
    # an id outside [0, n_as) leaves its output row unwritten and does not touch memory outside the experts
    bad = dev.to_device(np.array([[1, 7]], np.int32))
    dev.check(L.chip_memset(dy.ptr, 0xFF, 2 * N * 4, None))
    assert call(ids=bad.ptr) == 0
    dev.sync()
    out = dy.download(np.float32, 2 * N).reshape(2, N)
    assert np.isfinite(out[0]).all() and np.isnan(out[1]).all()


# ------------------------------------------------------------------------------------------ several matrices, one activation
@pytest.mark.parametrize("members", [
    ((O.Q4_K, 300), (O.Q6_K, 77), (O.Q5_K, 1)),                      # K-quants of three types, ragged row counts
    ((O.Q4_0, 129), (O.Q8_0, 64), (O.Q5_1, 33), (O.IQ4_NL, 200)),    # 32-value block types incl. a Q8_1 member, two-row tiles
    ((O.F16, 40), (O.F16, 3)),
    ((O.Q6_K, 2000),),                                               # a group of one
], ids=["kquants", "block32", "f16", "single"])
@pytest.mark.parametrize("K", [1024, 4096, 14336])                   # 14336: a single call builds its LDS image a step's part at a time
def test_mul_mat_group_equals_single_calls(dev, orc, members, K):
    """chip_mul_mat_group: each member's output equals chip_mul_mat on that member alone, bit for bit, for every token
    count class (1, 2, 4: one launch; 3, 7: one quantizer and the GEMVs; 40: the GEMMs), and the oracle within tolerance."""
    ws = [(wt, quantized_weights(wt, K + N + 11, N, K)) for wt, N in members]
    for n in (1, 2, 4, 3, 7, 8, 40):                                 # 8: small members as one launch over prepared rows
        x = common.activations_f32(K + n + 5, n, K)
        ys = dev.mul_mat_group(ws, x)
        for (wt, W), y in zip(ws, ys):
            if n == 8 and len(ws) > 1:          # one launch of the dot-product GEMV; alone, a member may take the matrix-core GEMV
                r = orc.mul_mat(wt, W, x, nthreads=8, want=("sum_abs",))
                check_outputs(y, r["y"], r["sum_abs"], "group member at 8 tokens")
                continue
            assert y.tobytes() == dev.mul_mat(wt, W, x).tobytes(), (O.TYPE_NAMES[wt], n)
        wt, W = ws[0]
        ref = orc.mul_mat(wt, W, x, nthreads=8, want=("sum_abs",))
        check_outputs(ys[0], ref["y"], ref["sum_abs"], "group member 0, n = %d" % n)


@pytest.mark.parametrize("members", [
    ((O.Q4_K, 1100), (O.Q4_K, 256), (O.Q6_K, 260)),
    ((O.Q4_0, 700), (O.Q8_0, 300), (O.Q5_1, 130)),
    ((O.Q6_K, 2000),),
], ids=["kquants", "block32", "single"])
@pytest.mark.parametrize("K", [1024, 14336])
def test_mul_mat_group_run_over_prepared_rows(dev, orc, members, K):
    """chip_mul_mat_group_run: over rows the workspace already holds every member's output equals chip_mul_mat's, bit for
    bit (the quantized rows are the same bytes and the GEMV's arithmetic does not depend on who staged them), also for
    rows longer than the prologue quantizer takes (K = 14336), with the transposed fp16 store on the last member."""
    ws = [(wt, quantized_weights(wt, K + N + 13, N, K)) for wt, N in members]
    for n in (1, 2, 4, 3, 6, 8):
        x = common.activations_f32(K + n + 7, n, K)
        ys = dev.mul_mat_group(ws, x, ld16=8, prepared=True)
        for (wt, W), y in zip(ws, ys):
            if n == 8 and len(ws) > 1:
                r = orc.mul_mat(wt, W, x, nthreads=8, want=("sum_abs",))
                check_outputs(y, r["y"], r["sum_abs"], "group member at 8 tokens")
                continue
            assert y.tobytes() == dev.mul_mat(wt, W, x).tobytes(), (O.TYPE_NAMES[wt], n)
        t16 = ys[-1]
        want = ys[len(ws) - 1].astype(np.float16).view(np.uint16).T
        assert np.array_equal(t16[:, :n], want) and (t16[:, n:] == 0x7bff).all()


def test_mul_mat_group_argument_errors(dev, orc):
    import cactus_amd as ca
    L = dev.lib
    K, N = 1024, 8
    buf, ws = dev.alloc(1 << 16), dev.alloc(1 << 16)
    def mats(*types):
        arr = (ca.Mat * len(types))()
        for i, t in enumerate(types):
            arr[i] = ca.Mat(t, buf.ptr, dev.row_size(t, K), N, buf.ptr, N, None, 0)
        return arr
    call = lambda arr, count, n=1, wsz=1 << 16: L.chip_mul_mat_group(arr, count, K, buf.ptr, K, n, ws.ptr, wsz, None)
    assert call(mats(O.Q4_K, O.Q6_K), 2) == 0
    assert call(mats(O.Q4_K, O.Q8_0), 2) == -2                   # different activation formats
    assert call(mats(O.Q4_K, 30), 2) == -2                       # unknown type
    assert call(mats(O.Q4_K), 5) == -1                           # more members than CHIP_GROUP_MAX
    assert call(mats(O.Q4_K), 1, wsz=16) == -3
    assert call(None, 1) == -1 and call(None, 0) == 0 and call(mats(O.Q4_K), 1, n=0) == 0
    bad = mats(O.Q4_K)
    bad[0].ldy = N - 1
    assert call(bad, 1) == -1
    dev.sync()


# ------------------------------------------------------------------------------------------ Q6_K rows in planes
def q6_K_planes_of(W, K):
    """What chip_repack_q6_K writes, on the host: per row every ql field, then every qh, every scales, every d."""
    N, nsb = W.shape[0], K // 256
    b = W.reshape(N, nsb, 210)
    return np.concatenate([b[:, :, 0:128].reshape(N, -1), b[:, :, 128:192].reshape(N, -1), b[:, :, 192:208].reshape(N, -1),
                           b[:, :, 208:210].reshape(N, -1)], axis=1)


@pytest.mark.parametrize("K,N", [(2048, 64), (4096, 1032), (14336, 304), (6144, 77), (196608, 3)])
def test_q6_K_repack_to_planes_and_back(dev, K, N):
    """chip_repack_q6_K moves every byte of a row to its plane (checked against the same permutation on the host), out of
    place and in place, and the other direction gives the block order back; row lengths that leave a plane misaligned, rows
    longer than the LDS and overlapping matrices are rejected."""
    import cactus_amd as ca
    W = np.random.default_rng(K + N).integers(0, 256, (N, K // 256 * 210), dtype=np.uint8)
    P = dev.repack_q6_K(W, K, True)
    assert np.array_equal(P, q6_K_planes_of(W, K))
    assert np.array_equal(dev.repack_q6_K(W, K, True, in_place=True), P)
    assert np.array_equal(dev.repack_q6_K(P, K, False), W)
    assert np.array_equal(dev.repack_q6_K(P, K, False, in_place=True), W)
    L = dev.lib
    if N <= 304:                                         # rows wider apart than they are long, on both sides
        row, ps, pd = W.shape[1], W.shape[1] + 420, W.shape[1] + 64
        src = np.full((N, ps), 0xa5, np.uint8)
        src[:, :row] = W
        ds, dd = dev.to_device(src), dev.to_device(np.full((N, pd), 0x5a, np.uint8))
        dev.check(L.chip_repack_q6_K(ds.ptr, ps, dd.ptr, pd, K, N, 1, None))
        dev.sync()
        out = dd.download(np.uint8, N * pd).reshape(N, pd)
        assert np.array_equal(out[:, :row], P) and (out[:, row:] == 0x5a).all()
    d = dev.alloc(1 << 20)
    for bad_k in (256, 1024, 2048 + 256, 0):
        assert L.chip_repack_q6_K(d.ptr, 210 * bad_k // 256, d.ptr + (1 << 19), 210 * bad_k // 256, bad_k, 2, 1, None) == ca.CHIP_EUNSUPPORTED
        assert L.chip_mul_mat_supported(ca.Q6_K_PLANES, bad_k) == 0
    assert L.chip_mul_mat_supported(ca.Q6_K_PLANES, 2048) == 1
    assert L.chip_repack_q6_K(d.ptr, 1680, d.ptr + 1680, 1680, 2048, 4, 1, None) == ca.CHIP_EINVAL      # the two overlap
    assert L.chip_repack_q6_K(d.ptr, 1678, d.ptr + (1 << 19), 1680, 2048, 4, 1, None) == ca.CHIP_EINVAL  # stride below a row
    assert L.chip_repack_q6_K(d.ptr, 1680, d.ptr + (1 << 19), 1680, 2048, 0, 1, None) == ca.CHIP_OK
    assert L.chip_repack_q6_K(d.ptr, 210 * 1024, d.ptr, 210 * 1024, 262144, 1, 1, None) == ca.CHIP_EUNSUPPORTED   # 215 040-byte rows


@pytest.mark.parametrize("K,N", [(2048, 72), (4096, 1032), (14336, 4096), (8192, 264)])
def test_q6_K_in_planes_gives_the_bits_of_q6_K(dev, orc, K, N):
    """CHIP_TYPE_Q6_K_PLANES through every matmul entry point that takes it: bit for bit what the same entry point gives on
    the block_q6_K rows the planes were made from (1, 2, 3, 4 tokens; larger batches against single passes of the GEMV), and
    the oracle within tolerance; the entry points that read other layouts reject the type."""
    import cactus_amd as ca
    W = quantized_weights(O.Q6_K, K + N, N, K)
    W2 = quantized_weights(O.Q6_K, K + N + 1, N, K)
    P, P2 = dev.repack_q6_K(W, K), dev.repack_q6_K(W2, K)
    PL = ca.Q6_K_PLANES
    for n in (1, 2, 3, 4):
        x = common.activations_f32(K + n, n, K)
        y = dev.mul_mat(PL, P, x)
        assert y.tobytes() == dev.mul_mat(O.Q6_K, W, x).tobytes(), n
        if n == 1:
            ref = orc.mul_mat(O.Q6_K, W, x, nthreads=8, want=("sum_abs",))
            check_outputs(y, ref["y"], ref["sum_abs"], "Q6_K planes")
        if dev.lib.chip_mul_mat_add_supported(O.Q6_K, K, N, n):
            assert dev.lib.chip_mul_mat_add_supported(PL, K, N, n) == 1
            b = common.activations_f32(N + n, n, N)
            assert dev.mul_mat_add(PL, P, x, b).tobytes() == dev.mul_mat_add(O.Q6_K, W, x, b).tobytes(), n
        y1, y2 = dev.mul_mat_pair(PL, P, P2, x)
        w1, w2 = dev.mul_mat_pair(O.Q6_K, W, W2, x)
        assert y1.tobytes() == w1.tobytes() and y2.tobytes() == w2.tobytes(), n
        yt, ht = dev.mul_mat_store_t(PL, P, x, 8)
        wt_, hw = dev.mul_mat_store_t(O.Q6_K, W, x, 8)
        assert yt.tobytes() == wt_.tobytes() and ht.tobytes() == hw.tobytes(), n
        if n != 3 and dev.lib.chip_mul_mat_pair_silu_mul_supported(O.Q6_K, K, N, n):
            assert dev.lib.chip_mul_mat_pair_silu_mul_supported(PL, K, N, n) == 1
            assert dev.mul_mat_pair_silu_mul(PL, P, P2, x).tobytes() == dev.mul_mat_pair_silu_mul(O.Q6_K, W, W2, x).tobytes(), n
            if dev.lib.chip_norm_before_supported(O.Q6_K, K, n):
                assert dev.lib.chip_norm_before_supported(PL, K, n) == 1
                nw = norm_weight(N, K)
                got, got_normed = dev.mul_mat_pair_silu_mul(PL, P, P2, x, norm=(nw, 1e-6))
                want, want_normed = dev.mul_mat_pair_silu_mul(O.Q6_K, W, W2, x, norm=(nw, 1e-6))
                assert got.tobytes() == want.tobytes() and got_normed.tobytes() == want_normed.tobytes(), n
    if N <= 1032:
        for n in (5, 8, 11):                    # passes of up to 8 tokens of the same kernel
            x = common.activations_f32(K + n, n, K)
            want = np.concatenate([dev.mul_mat(O.Q6_K, W, x[i:i + 1]) for i in range(n)])
            assert dev.mul_mat(PL, P, x).tobytes() == want.tobytes(), n
    d = dev.alloc(1 << 16)
    L = dev.lib
    assert L.chip_get_rows(PL, d.ptr, 1680, 0, 0, 2048, 4, d.ptr, 1, 1, 1, 0, 0, d.ptr, 8192, 0, 0, None) == ca.CHIP_EUNSUPPORTED
    assert L.chip_block_isums(PL, d.ptr, 1680, 2048, 4, d.ptr, 1, d.ptr, d.ptr, None) == ca.CHIP_EUNSUPPORTED
    assert L.chip_mul_mat_id(PL, d.ptr, 1680, 4 * 1680, 2048, 4, 2, d.ptr + 32768, 2048, 1, d.ptr + 49152, 1, 1, 1, d.ptr + 49408, 4,
                             d.ptr + 16384, 16384, None) == ca.CHIP_EUNSUPPORTED
    assert L.chip_mul_mat(PL, d.ptr + 2, 1680, 2048, 4, d.ptr + 32768, 2048, 1, d.ptr + 49152, 4, d.ptr + 16384, 16384, None) == ca.CHIP_EINVAL


@pytest.mark.parametrize("K,members", [(4096, ((O.Q4_K, 4096), (O.Q4_K, 1024), ("planes", 1024))), (2048, (("planes", 520), ("planes", 8), ("planes", 264))),
                                       (2048, ((O.Q6_K, 520), (O.Q5_K, 72), ("planes", 264))), (2048, ((O.Q3_K, 136), ("planes", 264), (O.Q2_K, 64)))],
                         ids=["q4_K_M-qkv", "planes-only", "blocks-and-planes", "with-q3_K"])
def test_group_members_in_planes(dev, K, members):
    """chip_mul_mat_group and chip_mul_mat_group_rope_norm with Q6_K members in planes (beside Q4_K / Q5_K members: the kernel
    family of the Q4_K_M mix; beside block-order Q6_K or low-bit members: the wide family): every output bit for bit the group
    with those members in block order."""
    import cactus_amd as ca
    blocks, planes = [], []
    for i, (wt, N) in enumerate(members):
        real = O.Q6_K if wt == "planes" else wt
        W = quantized_weights(real, K + N + i, N, K)
        blocks.append((real, W))
        planes.append((ca.Q6_K_PLANES, dev.repack_q6_K(W, K)) if wt == "planes" else (real, W))
    for n in (1, 2, 4, 3, 8):
        x = common.activations_f32(K + n + 5, n, K)
        for got, want in zip(dev.mul_mat_group(planes, x), dev.mul_mat_group(blocks, x)):
            assert got.tobytes() == want.tobytes(), n
    if members[0][1] % 128 == 0 and blocks[0][0] in (O.Q4_K, O.Q6_K):
        hd = 128
        ropes = [(hd, hd, 0, ("f32",)), (hd, hd, 0, ("f32", "f16")), None]
        nw = norm_weight(K, K)
        for n in (1, 2, 4):
            x = common.activations_f32(K + n, n, K)
            pos = np.array([37, 0, 4095, 100000][:n], np.int32)
            rc, want = dev.mul_mat_group_rope(blocks, x, pos, ropes, freq_base=500000.0, norm=(nw, 1e-5))
            rc, got = dev.mul_mat_group_rope(planes, x, pos, ropes, freq_base=500000.0, norm=(nw, 1e-5))
            for g, w in zip(got, want):
                for key in w:
                    assert g[key].tobytes() == w[key].tobytes(), (n, key)
