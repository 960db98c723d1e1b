"""What the mathematics fixes about the oracle, independent of any reference run."""
import numpy as np
import pytest

import common
import oracle as O


def test_fp16_to_fp32_exhaustive(orc):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([orc.h2f(int(v)) for v in h], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.isnan(got[nan]).all()


def test_fp32_to_fp16_rne(orc):
    rng = np.random.default_rng(0)
    f = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32),          # exact halves
        np.array([65504, 65519.99, 65520, 1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -26, 0.0, -0.0,
                  6.1035e-5, 6.0975e-5, 5.96e-8, 8.94e-8, 2.98e-8, 1e-10], np.float32),
    ])
    # halfway points between consecutive halves: the tie-to-even cases
    hh = np.arange(0, 0x7bff, dtype=np.uint16)
    mid = (hh.view(np.float16).astype(np.float64) + (hh + 1).astype(np.uint16).view(np.float16).astype(np.float64)) / 2
    f = np.concatenate([f, mid.astype(np.float32), -mid.astype(np.float32)])
    f = f[~np.isnan(f)]
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([orc.f2h(v) for v in f], np.uint16)
    assert np.array_equal(got, want)


def test_q8_0_invariants(orc):
    x = common.activations_f32(3, 4, 1024)
    q = orc.quantize_activation(O.Q8_0, x).reshape(4, -1, 34)
    d = q[..., :2].copy().view(np.float16).astype(np.float32)[..., 0]
    qs = q[..., 2:].view(np.int8)
    xb = x.reshape(4, -1, 32)
    amax = np.abs(xb).max(-1)
    # the largest element of each block maps to +-127, the scale is amax/127 rounded to half
    assert (np.abs(qs).max(-1) == 127).all()
    assert np.array_equal(d, (amax / np.float32(127)).astype(np.float16).astype(np.float32))
    idx = np.abs(xb).argmax(-1)
    assert np.array_equal(np.sign(np.take_along_axis(qs, idx[..., None], -1)[..., 0]),
                          np.sign(np.take_along_axis(xb, idx[..., None], -1)[..., 0]))
    # reconstruction error at most half a step, plus up to 127 steps times the fp16 rounding of d (2^-11)
    err = np.abs(qs * d[..., None] - xb)
    assert (err <= d[..., None] * (0.5 + 127 * 2.0 ** -11) + 1e-7).all()
    # exactly representable grid: x = k * amax/127 with amax = 127*2^-3 -> id = 8 -> q == k
    k = np.arange(-16, 16, dtype=np.float32)
    k[0] = 127
    g = k * np.float32(0.125)
    qg = orc.quantize_activation(O.Q8_0, g[None])[0]
    assert np.array_equal(qg[2:].view(np.int8), k.astype(np.int8))


def test_q8_K_invariants(orc):
    x = common.activations_f32(4, 3, 2048)
    q = orc.quantize_activation(O.Q8_K, x).reshape(3, -1, 292)
    d = q[..., :4].copy().view(np.float32)[..., 0]
    qs = q[..., 4:260].view(np.int8)
    bs = q[..., 260:].copy().view(np.int16)
    assert np.array_equal(bs, qs.reshape(3, -1, 16, 16).sum(-1).astype(np.int16))
    xb = x.reshape(3, -1, 256)
    idx = np.abs(xb).argmax(-1)                      # argmax returns the first maximum, as the scan does
    mx = np.take_along_axis(xb, idx[..., None], -1)[..., 0]
    assert np.array_equal(d, np.float32(1) / (np.float32(-127) / mx))
    assert (np.take_along_axis(qs, idx[..., None], -1)[..., 0] == -127).all()   # iscale*max == -127
    assert (np.abs(qs * d[..., None] - xb) <= 0.5 * np.abs(d[..., None]) * 1.0001 + 1e-7).all()


def test_scale_unpack_paths_agree(orc):
    # get_scale_min_k4 (used by the dequantizer) and the kmask shuffle (used by the dot) must agree:
    # dequant-based and dot-based evaluations of the same block only match if they do.
    rng = np.random.default_rng(11)
    K = 256
    for trial in range(64):
        blk = rng.integers(0, 256, 144, dtype=np.uint8)
        if trial < 16:      # one-hot 6-bit patterns
            blk[4:16] = 0
            j = trial % 8
            sc = np.zeros(8, np.uint8); mn = np.zeros(8, np.uint8)
            (sc if trial < 8 else mn)[j] = 63
            s = blk[4:16]
            for jj in range(8):
                if jj < 4:
                    s[jj] |= sc[jj]; s[jj + 4] |= mn[jj]
                else:
                    s[jj + 4] |= (sc[jj] & 0xF) | ((mn[jj] & 0xF) << 4)
                    s[jj - 4] |= (sc[jj] >> 4) << 6
                    s[jj] |= (mn[jj] >> 4) << 6
        blk[0:2] = np.array([1.0], np.float16).view(np.uint8)      # d = 1
        blk[2:4] = np.array([1.0], np.float16).view(np.uint8)      # dmin = 1
        x = rng.integers(-127, 128, K).astype(np.float32)
        x[0] = -127                                                 # iscale = -127/max = +1: q == x, d == 1
        xq = orc.quantize_activation(O.Q8_K, x[None])[0]
        assert np.array_equal(xq[4:260].view(np.int8).astype(np.float32), x)
        w = orc.dequantize(O.Q4_K, blk[None], K)[0]
        want = float(np.dot(w.astype(np.float64), x.astype(np.float64)))
        v, isum, imin = orc.vec_dot(O.Q4_K, K, blk, xq, want_sums=True)
        assert isum[0] - imin[0] == want
        assert float(v) == want


@pytest.mark.parametrize("wt", O.WEIGHT_TYPES, ids=lambda t: O.TYPE_NAMES[t])
def test_vec_dot_is_dot_of_dequantized(orc, wt):
    """Textbook identity: vec_dot(x, y) == sum dequant(x)_i * dequant(y)_i (fp64), and the integer sums
    equal a brute-force evaluation from the dequantised integers."""
    K, N = 1024, 8
    wq = orc.quantize_weights(wt, common.weights_f32(50 + wt, N, K, outliers=True))
    at = O.VEC_DOT_TYPE[wt]
    xq = orc.quantize_activation(at, common.activations_f32(50 + wt, 2, K))
    wd = orc.dequantize(wt, wq, K).astype(np.float64)
    xd = orc.dequantize(at, xq, K).astype(np.float64)
    for t in range(2):
        for i in range(N):
            v, isum, imin = orc.vec_dot(wt, K, wq[i], xq[t], want_sums=True)
            exact, sum_abs = orc.vec_dot_exact(wt, K, wq[i], xq[t])
            want = float(np.dot(wd[i], xd[t]))
            # fp32 products inside the dequantizers; for Q4_1 / Q5_1 the min term uses s = fp16(d * sum q), which
            # differs from m * sum(d * q) by the fp16 rounding of s
            assert abs(exact - want) <= (1e-3 if wt in (O.Q4_1, O.Q5_1) else 1e-6) * sum_abs
            assert abs(float(v) - exact) <= 1e-5 * sum_abs   # the reference's own rounding noise
    # integer sums by brute force, block by block
    if wt in (O.Q4_0, O.Q8_0):
        blocks_w = wq[0].reshape(-1, O.BLOCK_BYTES[wt])
        blocks_x = xq[0].reshape(-1, 34)
        _, isum, _ = orc.vec_dot(wt, K, wq[0], xq[0], want_sums=True)
        for b in range(K // 32):
            qx = blocks_x[b, 2:].view(np.int8).astype(np.int64)
            if wt == O.Q4_0:
                nib = blocks_w[b, 2:]
                qw = np.concatenate([(nib & 0xF).astype(np.int64) - 8, (nib >> 4).astype(np.int64) - 8])
            else:
                qw = blocks_w[b, 2:].view(np.int8).astype(np.int64)
            assert isum[b] == int((qw * qx).sum())


def test_mul_mat_is_independent_dots(orc):
    K, N, n = 512, 33, 3
    for wt in O.WEIGHT_TYPES:
        wq = orc.quantize_weights(wt, common.weights_f32(70 + wt, N, K))
        x = common.activations_f32(70 + wt, n, K)
        out = orc.mul_mat(wt, wq, x, nthreads=3, want=("wdata",))
        xq = orc.quantize_activation(O.VEC_DOT_TYPE[wt], x)
        assert np.array_equal(out["wdata"], xq)
        for t in range(n):
            for i in range(N):
                assert out["y"][t, i].tobytes() == orc.vec_dot(wt, K, wq[i], xq[t]).tobytes()


@pytest.mark.parametrize("wt", (O.Q4_K, O.Q6_K), ids=lambda t: O.TYPE_NAMES[t])
def test_kquant_reconstruction_bound(orc, wt):
    # sanity invariant for the iterative weight quantizers: error stays within a step of the sub-block scale
    K = 2048
    w = common.weights_f32(90 + wt, 4, K, outliers=True)
    wd = orc.dequantize(wt, orc.quantize_weights(wt, w), K)
    step = {O.Q4_K: 0.16 * 2 / 15, O.Q6_K: 0.16 / 31}[wt]
    assert np.abs(wd - w).max() <= step
