"""Seeded input generators shared by the CPU and GPU tests (same arrays feed oracle, reference and GPU)."""
import numpy as np


def weights_f32(seed, n_rows, k, outliers=False, sigma=0.02):
    """~N(0, sigma); with outliers=True, 1 % of entries replaced by +-8 sigma."""
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((n_rows, k)) * sigma).astype(np.float32)
    if outliers:
        m = rng.random(w.shape) < 0.01
        sign = np.where(rng.random(w.shape) < 0.5, -1.0, 1.0).astype(np.float32)
        w = np.where(m, np.float32(8 * sigma) * sign, w).astype(np.float32)
    return w


def activations_f32(seed, n, k):
    rng = np.random.default_rng(seed + 7919)
    return rng.standard_normal((n, k)).astype(np.float32)


def q8_0_edge_rows():
    """Rows of 32 floats that exercise the AVX2 quantize_row_q8_0 corner cases."""
    rows = []
    z = np.zeros(32, np.float32)
    rows.append(z.copy())                                     # all-zero block: d = 0, id = 0
    a = z.copy(); a[0] = 127.0; a[1:11] = [0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, 126.5, -126.5, 63.5]
    rows.append(a)                                            # id == 1: exact .5 ties (to even vs away)
    b = z.copy(); b[5] = -127.0; b[6:12] = [0.5, 1.5, -0.5, -1.5, 2.5, -2.5]
    rows.append(b)                                            # max is negative
    c = np.full(32, 1e-41, np.float32); c[3] = 3e-41
    rows.append(c)                                            # subnormal inputs: 127/amax overflows to inf? no: finite
    d = np.linspace(-1, 1, 32).astype(np.float32) * np.float32(3.0e38)
    rows.append(d)                                            # huge magnitudes (d overflows fp16 -> inf)
    e = np.linspace(-1, 1, 32).astype(np.float32) * np.float32(1e-3)
    rows.append(e)
    f = z.copy(); f[31] = 65504.0 * 127.0
    rows.append(f)                                            # d == fp16 max
    g = (np.arange(32, dtype=np.float32) - 16) / np.float32(127.0) * np.float32(0.3)
    rows.append(g)                                            # grid points k*amax/127-ish
    return np.stack(rows).astype(np.float32)


def q8_K_edge_rows():
    rows = []
    z = np.zeros(256, np.float32)
    rows.append(z.copy())                                     # amax == 0
    a = z.copy(); a[3] = -2.0; a[7] = 2.0; a[9] = 1.0
    rows.append(a)                                            # +-tie: first (negative) max wins -> iscale > 0
    b = z.copy(); b[3] = 2.0; b[7] = -2.0; b[9] = 1.0
    rows.append(b)                                            # first (positive) max wins -> max maps to -127
    c = z.copy(); c[0] = 127.0; c[1:9] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5]
    rows.append(c)                                            # ties under the magic-number rounding
    d = z.copy(); d[0] = -127.0; d[1:9] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5]
    rows.append(d)                                            # iscale = +1: +127.x values hit the min(127, .) clamp
    rng = np.random.default_rng(5)
    rows.append((rng.standard_normal(256) * 1e-3).astype(np.float32))
    rows.append((rng.standard_normal(256) * 1e4).astype(np.float32))
    return np.stack(rows).astype(np.float32)
