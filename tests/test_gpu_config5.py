"""GPU parity at the shapes of the Llama-3-8B-shaped Q4_K_M decode trace (every distinct weight matmul of one token step,
at 1 and at 8 tokens), through the C-ABI with the library's default dispatch, against the CPU oracle.

Reference behaviour: lm_ggml_compute_forward_mul_mat (ggml-cpu/ggml-cpu.c:1257-1449) with type_traits_cpu[] (:198-367):
Q4_K and Q6_K rows against Q8_K activations quantized inside the op.

Weights: a base block of rows quantized by the oracle's restatement of the reference quantizers, repeated down the matrix
(quantizing 525 M values for the output head on the CPU would take minutes); every output row of every repetition is
compared, so row tiles at every position of the grid are covered, first and last rows included.  A second test gives every
repetition its own scale bytes, so that no two row tiles are alike, and checks a sample of rows of every repetition.  Each case also prints how
far the GPU and the oracle (= the reference's AVX2 summation order) each are from the exact value of sum scale * isum
evaluated in fp64, in units of the tolerance, on a sample of rows."""
import numpy as np
import pytest

import common
import oracle as O

pytestmark = pytest.mark.gpu
REL_TOL = 1e-5

# name, weight type, N, K, base rows (N is a multiple)
TRACE_MATMULS = [
    ("wq_wo", O.Q4_K, 4096, 4096, 1024),
    ("wk", O.Q4_K, 1024, 4096, 1024),
    ("wv", O.Q6_K, 1024, 4096, 512),
    ("ffn_up_gate", O.Q4_K, 14336, 4096, 1024),
    ("ffn_down", O.Q6_K, 4096, 14336, 256),
    ("output_head", O.Q6_K, 128256, 4096, 334),          # 128256 = 384 * 334
]
_cache = {}


def base_rows(orc, wt, seed, rows, K):
    key = (wt, seed, rows, K)
    if key not in _cache:
        _cache[key] = orc.quantize_weights(wt, common.weights_f32(seed, rows, K, outliers=(wt == O.Q4_K)))
    return _cache[key]


@pytest.fixture(scope="module")
def dev():
    import cactus_amd
    return cactus_amd.Device(0)


def attribution(orc, wt, K, base, xq, y_gpu, y_ref, sum_abs, what):
    """|gpu - exact| and |ref - exact| in units of the tolerance, exact = fp64 sum of scale * isum, on 48 rows."""
    rows = np.unique(np.linspace(0, base.shape[0] - 1, 48).astype(int))
    worst_gpu = worst_ref = 0.0
    for t in range(xq.shape[0]):
        for r in rows:
            exact, _ = orc.vec_dot_exact(wt, K, base[r], xq[t])
            tol = REL_TOL * sum_abs[t, r]
            worst_gpu = max(worst_gpu, abs(float(y_gpu[t, r]) - exact) / tol)
            worst_ref = max(worst_ref, abs(float(y_ref[t, r]) - exact) / tol)
    print("%s: |gpu - exact| <= %.3f tol, |ref - exact| <= %.3f tol" % (what, worst_gpu, worst_ref), flush=True)
    return worst_gpu, worst_ref


@pytest.mark.parametrize("name,wt,N,K,nbase", TRACE_MATMULS, ids=[m[0] for m in TRACE_MATMULS])
@pytest.mark.parametrize("n", [1, 8])
def test_trace_matmul_vs_oracle(dev, orc, name, wt, N, K, nbase, n):
    print("config5", name, O.TYPE_NAMES[wt], "N", N, "K", K, "n", n, flush=True)
    base = base_rows(orc, wt, 5000 + N + K, nbase, K)
    reps = N // nbase
    assert reps * nbase == N
    W = np.tile(base, (reps, 1))
    x = common.activations_f32(5 + n + K, n, K)
    ref = orc.mul_mat(wt, base, x, nthreads=8, want=("wdata", "sum_abs"))
    y, blocks = dev.mul_mat(wt, W, x, want_workspace_blocks=True)
    del W
    assert np.array_equal(blocks, ref["wdata"])                       # Q8_K bytes of the activations, bit-exact
    y = y.reshape(n, reps, nbase)
    err = np.abs(y.astype(np.float64) - ref["y"].astype(np.float64)[:, None, :])
    bound = REL_TOL * ref["sum_abs"][:, None, :]
    worst = float((err / bound).max())
    assert (err <= bound).all(), "%s n=%d: worst error %.3g x the tolerance" % (name, n, worst)
    if n == 1:
        # one wave per row and a fixed reduction: the same bits wherever the row sits in the grid (the matrix-core GEMV of
        # the 8-token case splits a tile's K range over its waves by the tile's place in the workgroup: order-only differences)
        assert (y == y[:, :1, :]).all()
    g, r = attribution(orc, wt, K, base, ref["wdata"], y[:, 0, :], ref["y"], ref["sum_abs"], "%s n=%d" % (name, n))
    assert g <= 1.0


def distinct_repetitions(wt, base, reps, K):
    """The base rows repeated `reps` times with one scale byte changed per repetition - the low mantissa byte of the fp16
    super-block scale d of super-block (rep mod super-blocks per row), XORed with a value that differs between neighbouring
    repetitions - so that no two row tiles of the matrix hold the same bytes: a kernel that swaps or aliases whole tiles
    then gives wrong numbers somewhere, which identical repetitions cannot show."""
    nbase, row_bytes = base.shape
    bb = O.BLOCK_BYTES[wt]
    d_off = 208 if wt == O.Q6_K else 0
    W = np.tile(base, (reps, 1)).reshape(reps, nbase, row_bytes)
    nsb = K // 256
    for rep in range(reps):
        W[rep, :, (rep % nsb) * bb + d_off] ^= np.uint8(1 + (rep * 37) % 255)
    return W.reshape(reps * nbase, row_bytes)


@pytest.mark.parametrize("name,wt,N,K,nbase", [m for m in TRACE_MATMULS if m[0] != "wk"], ids=[m[0] for m in TRACE_MATMULS if m[0] != "wk"])
@pytest.mark.parametrize("n", [1, 8])
def test_trace_matmul_no_two_tiles_alike(dev, orc, name, wt, N, K, nbase, n):
    """The same shapes with every repetition of the base rows made distinct; the oracle evaluates a sample of rows of
    every repetition (first and last row of the matrix included, at least 16 per repetition: 6144 rows of the output head)."""
    print("config5 distinct", name, O.TYPE_NAMES[wt], "N", N, "K", K, "n", n, flush=True)
    base = base_rows(orc, wt, 5000 + N + K, nbase, K)
    reps = N // nbase
    W = distinct_repetitions(wt, base, reps, K)
    x = common.activations_f32(5 + n + K, n, K)
    y = dev.mul_mat(wt, W, x)
    rng = np.random.default_rng(N + n)
    per_rep = 16 if reps >= 16 else 256 // reps
    rows = np.concatenate([rep * nbase + np.sort(rng.choice(nbase, per_rep, replace=False)) for rep in range(reps)])
    rows[0], rows[-1] = 0, N - 1
    ref = orc.mul_mat(wt, W[rows], x, nthreads=8, want=("sum_abs",))
    del W
    err = np.abs(y[:, rows].astype(np.float64) - ref["y"].astype(np.float64))
    bound = REL_TOL * ref["sum_abs"]
    assert (err <= bound).all(), "%s n=%d: worst error %.3g x the tolerance" % (name, n, float((err / bound).max()))
    # the changed scale moves a row's result by far more than the tolerance, so a tile read from the wrong repetition fails:
    base_ref = orc.mul_mat(wt, base[rows[per_rep:2 * per_rep] % nbase], x, nthreads=8, want=("sum_abs",))
    moved = np.abs(ref["y"][:, per_rep:2 * per_rep].astype(np.float64) - base_ref["y"].astype(np.float64))
    assert (moved > 4 * bound[:, per_rep:2 * per_rep]).mean() > 0.5


def test_trace_gate_up_pair_and_v_store(dev, orc):
    """The two fused forms the one-token step uses: ffn_gate + ffn_up in one launch (chip_mul_mat_pair) and the V
    projection with its transposed fp16 cache store (chip_mul_mat_store_t), at their real shapes; each equals the single
    chip_mul_mat bit for bit and the oracle within the tolerance."""
    K = 4096
    for n in (1, 4):
        up = np.tile(base_rows(orc, O.Q4_K, 5000 + 14336 + K, 1024, K), (14, 1))
        gate = np.tile(base_rows(orc, O.Q4_K, 77, 1024, K), (14, 1))
        x = common.activations_f32(50 + n, n, K)
        y1, y2 = dev.mul_mat_pair(O.Q4_K, gate, up, x)
        assert y1.tobytes() == dev.mul_mat(O.Q4_K, gate, x).tobytes()
        assert y2.tobytes() == dev.mul_mat(O.Q4_K, up, x).tobytes()
        ref = orc.mul_mat(O.Q4_K, gate[:1024], x, nthreads=8, want=("sum_abs",))
        err = np.abs(y1.reshape(n, 14, 1024).astype(np.float64) - ref["y"].astype(np.float64)[:, None, :])
        assert (err <= REL_TOL * ref["sum_abs"][:, None, :]).all()
        wv = base_rows(orc, O.Q6_K, 5000 + 1024 + K, 512, K)
        wv = np.tile(wv, (2, 1))
        y, h = dev.mul_mat_store_t(O.Q6_K, wv, x, 4096)
        assert y.tobytes() == dev.mul_mat(O.Q6_K, wv, x).tobytes()
        assert h[:, :n].tobytes() == np.ascontiguousarray(y.T.astype(np.float16)).view(np.uint16).tobytes()
        assert (h[:, n:] == 0x7bff).all()
        ref = orc.mul_mat(O.Q6_K, wv[:512], x, nthreads=8, want=("sum_abs",))
        err = np.abs(y.reshape(n, 2, 512).astype(np.float64) - ref["y"].astype(np.float64)[:, None, :])
        assert (err <= REL_TOL * ref["sum_abs"][:, None, :]).all()


@pytest.mark.parametrize("N,M", [(4096, 2048), (14336, 512)])
def test_config4_prefill_remaining_shapes(dev, orc, N, M):
    """The two prefill shapes of the Q4_0 GEMM configuration that the sampled test in test_gpu_parity.py does not run."""
    K = 4096
    rng = np.random.default_rng(N + M)
    wq = np.tile(orc.quantize_weights(O.Q4_0, common.weights_f32(4, 2048, K)), (N // 2048, 1))
    x = common.activations_f32(4, M, K)
    y = dev.mul_mat(O.Q4_0, wq, x)
    rows = np.sort(rng.choice(N, 96, replace=False))
    rows[:3] = [0, 1, 2]; rows[-1] = N - 1
    toks = np.sort(rng.choice(M, 24, replace=False))
    toks[0] = 0; toks[-1] = M - 1
    ref = orc.mul_mat(O.Q4_0, wq[rows], x[toks], nthreads=8, want=("sum_abs",))
    err = np.abs(y[np.ix_(toks, rows)].astype(np.float64) - ref["y"].astype(np.float64))
    assert (err <= REL_TOL * ref["sum_abs"]).all()


def test_trace_qkv_group(dev, orc):
    """wq (Q4_K 4096 rows), wk (Q4_K 1024), wv (Q6_K 1024, with its transposed fp16 cache store) on one activation as one
    call of chip_mul_mat_group, at the trace's shapes: every output equals the member's own chip_mul_mat /
    chip_mul_mat_store_t bit for bit (1, 2, 4 tokens: one launch; 3: one quantizer, then each member).  At 8 tokens the
    three run as one launch of the dot-product GEMV over prepared rows, where wq alone would take the matrix-core GEMV
    (which splits K inside a workgroup): there every member is held to the oracle's tolerance instead, and the fp16 store to
    the rounding of the group's own fp32 result."""
    K = 4096
    wq = np.tile(base_rows(orc, O.Q4_K, 5000 + 4096 + K, 1024, K), (4, 1))
    wk = base_rows(orc, O.Q4_K, 5000 + 1024 + K, 1024, K)
    wv = np.tile(base_rows(orc, O.Q6_K, 5000 + 1024 + K, 512, K), (2, 1))
    for n in (1, 2, 4, 3, 8):
        x = common.activations_f32(60 + n, n, K)
        yq, yk, yv, h = dev.mul_mat_group([(O.Q4_K, wq), (O.Q4_K, wk), (O.Q6_K, wv)], x, ld16=64)
        if n != 8:
            assert yq.tobytes() == dev.mul_mat(O.Q4_K, wq, x).tobytes(), n
            assert yk.tobytes() == dev.mul_mat(O.Q4_K, wk, x).tobytes(), n
            y1, h1 = dev.mul_mat_store_t(O.Q6_K, wv, x, 64)
            assert yv.tobytes() == y1.tobytes() and h.tobytes() == h1.tobytes(), n
        else:
            for wt, W, y in ((O.Q4_K, wq, yq), (O.Q6_K, wv, yv)):
                r = orc.mul_mat(wt, W, x, nthreads=8, want=("sum_abs",))
                assert (np.abs(y.astype(np.float64) - r["y"].astype(np.float64)) <= REL_TOL * r["sum_abs"]).all(), n
            assert np.array_equal(h[:, :n], yv.astype(np.float16).view(np.uint16).T) and (h[:, n:] == 0x7bff).all()
        ref = orc.mul_mat(O.Q4_K, wk, x, nthreads=8, want=("sum_abs",))
        err = np.abs(yk.astype(np.float64) - ref["y"].astype(np.float64))
        assert (err <= REL_TOL * ref["sum_abs"]).all(), n
