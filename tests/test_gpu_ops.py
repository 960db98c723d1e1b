"""GPU parity of the element-wise ops next to the matmuls (RMS_NORM, ADD, MUL, SILU), through the C-ABI, against the
CPU oracle (pinned bit-exact on the reference build).

Bars: ADD, MUL and SILU bit-exact; RMS_NORM within one fp32 ulp per element, and bit-exact in practice (the sum of
squares is a double: only its last bits depend on the order of the additions)."""
import numpy as np
import pytest

import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    import cactus_amd
    return cactus_amd.Device(0)


def inputs(seed, n, ne0):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((n, ne0)) * rng.choice([0.01, 1.0, 8.0, 40.0], (n, 1))).astype(np.float32)
    special = np.array([0.0, -0.0, 1e-30, -1e-30, 87.0, -87.0, 88.5, -88.5, 89.0, -104.0, 130.0, -130.0, 133.0, -140.0, 1e4, -1e4],
                       np.float32)
    m = min(special.size, ne0)
    x[0, :m] = special[:m]
    return x


SHAPES = [(1, 256), (1, 4096), (7, 4096), (3, 40), (2, 11008), (130, 14336), (5, 1000)]


@pytest.mark.parametrize("n,ne0", SHAPES)
def test_rms_norm(dev, orc, n, ne0):
    x = inputs(n + ne0, n, ne0)
    for eps in (1e-5, 1e-6):
        ref = orc.rms_norm(x, eps)
        y = dev.rms_norm(x, eps)
        ulp = np.spacing(np.abs(ref))
        assert (np.abs(y.astype(np.float64) - ref) <= ulp).all()
        assert (y.view(np.uint32) == ref.view(np.uint32)).mean() > 0.999
    z = np.zeros((2, ne0), np.float32)
    assert np.array_equal(dev.rms_norm(z, 1e-5), orc.rms_norm(z, 1e-5))          # all-zero rows: 0 * 1/sqrt(eps)


@pytest.mark.parametrize("n,ne0", [s for s in SHAPES if s[1] % 8 == 0])
def test_silu_bit_exact(dev, orc, n, ne0):
    x = inputs(2 * n + ne0, n, ne0)
    with np.errstate(all="ignore"):
        ref = orc.silu(x)
    assert dev.silu(x).tobytes() == ref.tobytes()


def test_silu_every_exponent_range(dev, orc):
    # a sweep through the whole input range of the exponential, including the thresholds of its scaling branches
    x = np.concatenate([np.linspace(-150, 150, 8192, dtype=np.float32), np.float32([87.3, 88.0, 88.72, 88.73, 103.9, 104.1]),
                        -np.float32([87.3, 88.0, 88.72, 88.73, 103.9, 104.1]), np.float32([np.inf, -np.inf, np.nan, 3e38]),
                        np.zeros(8, np.float32)]).reshape(1, -1)
    assert x.shape[1] % 8 == 0
    with np.errstate(all="ignore"):
        ref = orc.silu(x)
    y = dev.silu(x)
    assert np.array_equal(np.isnan(y), np.isnan(ref))
    assert y[~np.isnan(y)].tobytes() == ref[~np.isnan(ref)].tobytes()


@pytest.mark.parametrize("n,ne0", SHAPES)
def test_add_mul_bit_exact(dev, n, ne0):
    a, b, w = inputs(3 * n + ne0, n, ne0), inputs(4 * n + ne0, n, ne0), inputs(5 + ne0, 1, ne0)
    with np.errstate(all="ignore"):
        assert dev.binary("add", a, b).tobytes() == (a + b).tobytes()
        assert dev.binary("mul", a, b).tobytes() == (a * b).tobytes()
        assert dev.binary("mul", a, w).tobytes() == (a * w).tobytes()             # one row over all rows: norm weight
        assert dev.binary("add", a, w).tobytes() == (a + w).tobytes()             # bias


def test_strided_rows_in_place_and_errors(dev, orc):
    import cactus_amd as ca
    L = dev.lib
    n, ne0, ld = 5, 512, 640
    x = np.zeros((n, ld), np.float32)
    x[:, :ne0] = inputs(1, n, ne0)
    dx = dev.to_device(x)
    dev.check(L.chip_rms_norm(dx.ptr, ld, n, ne0, 1e-5, dx.ptr, ld, None))             # in place, padded rows
    dev.sync()
    out = dx.download(np.float32, n * ld).reshape(n, ld)
    assert np.array_equal(out[:, :ne0], orc.rms_norm(x[:, :ne0].copy(), 1e-5)) and not out[:, ne0:].any()
    dev.check(L.chip_silu(dx.ptr, ld, n, ne0, dx.ptr, ld, None))
    dev.sync()
    assert np.array_equal(dx.download(np.float32, n * ld).reshape(n, ld)[:, :ne0], orc.silu(out[:, :ne0].copy()))
    assert L.chip_silu(dx.ptr, ld, n, 12, dx.ptr, ld, None) == -2                      # row tail: unsupported
    assert L.chip_rms_norm(dx.ptr, 100, n, ne0, 1e-5, dx.ptr, ld, None) != 0           # stride shorter than the row
    assert L.chip_rms_norm(dx.ptr, ld, n, ne0, -1.0, dx.ptr, ld, None) != 0
    assert L.chip_add(dx.ptr, ld, dx.ptr, ld, 2, n, ne0, dx.ptr, ld, None) == -2       # src1 neither 1 nor n rows
    assert L.chip_mul(dx.ptr, ld, None, ld, 1, n, ne0, dx.ptr, ld, None) != 0
    assert L.chip_add(dx.ptr, ld, dx.ptr, ld, n, 0, ne0, dx.ptr, ld, None) == 0
    # unaligned base pointer: the scalar path
    y = dev.alloc(n * ld * 4 + 16)
    dev.check(L.chip_mul(dx.ptr + 4, ld, dx.ptr + 4, ld, n - 1, n - 1, ne0 - 3, y.ptr + 4, ld, None))
    dev.sync()
    cur = dx.download(np.float32, n * ld)
    want = np.stack([cur[1 + r * ld: 1 + r * ld + ne0 - 3] for r in range(n - 1)])
    got = y.download(np.float32, n * ld + 4)
    got = np.stack([got[1 + r * ld: 1 + r * ld + ne0 - 3] for r in range(n - 1)])
    with np.errstate(all="ignore"):
        assert got.tobytes() == (want * want).tobytes()


@pytest.mark.parametrize("n,ne0", [(1, 4096), (7, 4096), (3, 40), (130, 14336), (5, 1000)])
def test_fused_pairs_equal_the_separate_ops(dev, orc, n, ne0):
    """chip_rms_norm_mul and chip_silu_mul against the two separate device calls (bit for bit) and the oracle."""
    x = inputs(3 * n + ne0, n, ne0)
    w = (1.0 + 0.1 * np.random.default_rng(ne0).standard_normal(ne0)).astype(np.float32)
    dx, dw = dev.to_device(x), dev.to_device(w)
    dy, dn = dev.alloc(x.nbytes), dev.alloc(x.nbytes)
    dev.check(dev.lib.chip_rms_norm_mul(dx.ptr, ne0, n, ne0, 1e-5, dw.ptr, dn.ptr, ne0, dy.ptr, ne0, None))
    dev.sync()
    y = dy.download(np.float32, x.size).reshape(n, ne0)
    yn = dn.download(np.float32, x.size).reshape(n, ne0)
    sep = dev.rms_norm(x, 1e-5)
    assert yn.tobytes() == sep.tobytes()
    assert y.tobytes() == dev.binary("mul", sep, w).tobytes() == (sep * w).tobytes()
    dev.check(dev.lib.chip_rms_norm_mul(dx.ptr, ne0, n, ne0, 1e-5, dw.ptr, None, 0, dx.ptr, ne0, None))      # in place, no norm output
    dev.sync()
    assert dx.download(np.float32, x.size).tobytes() == y.tobytes()
    if ne0 % 8 == 0:
        b = inputs(5 * n + ne0, n, ne0)
        da, db = dev.to_device(x), dev.to_device(b)
        dev.check(dev.lib.chip_silu_mul(da.ptr, ne0, db.ptr, ne0, n, ne0, da.ptr, ne0, None))
        dev.sync()
        with np.errstate(all="ignore"):
            want = orc.silu(x) * b
        assert da.download(np.float32, x.size).tobytes() == want.tobytes()
    else:
        import cactus_amd as ca
        assert dev.lib.chip_silu_mul(dx.ptr, ne0, dx.ptr, ne0, n, ne0, dy.ptr, ne0, None) == ca.CHIP_EUNSUPPORTED


@pytest.mark.parametrize("n,ne0", [(1, 4096), (8, 4096), (3, 40), (130, 14336), (5, 1001)])
@pytest.mark.parametrize("with_w", [True, False])
def test_fused_add_norm_equals_the_separate_ops(dev, n, ne0, with_w):
    """chip_add_rms_norm_mul against chip_add, chip_rms_norm and chip_mul run one after the other (bit for bit), with the sum
    written over either operand and the result over the other."""
    a, b = inputs(7 * n + ne0, n, ne0), inputs(11 * n + ne0, n, ne0)
    w = (1.0 + 0.1 * np.random.default_rng(ne0).standard_normal(ne0)).astype(np.float32)
    with np.errstate(all="ignore"):
        s_want = dev.binary("add", a, b)
        y_want = dev.rms_norm(s_want, 1e-6)
        if with_w:
            y_want = dev.binary("mul", y_want, w)
    dw = dev.to_device(w)
    wp = dw.ptr if with_w else None
    for sum_over, y_over in (("new", "new"), ("a", "new"), ("b", "new"), ("b", "a"), ("a", "b"), ("new", "a")):
        da, db = dev.to_device(a), dev.to_device(b)
        ds, dy = dev.alloc(a.nbytes), dev.alloc(a.nbytes)
        sp = {"new": ds, "a": da, "b": db}[sum_over]
        yp = {"new": dy, "a": da, "b": db}[y_over]
        dev.check(dev.lib.chip_add_rms_norm_mul(da.ptr, ne0, db.ptr, ne0, sp.ptr, ne0, n, ne0, 1e-6, wp, yp.ptr, ne0, None))
        dev.sync()
        assert sp.download(np.float32, a.size).tobytes() == s_want.tobytes(), (sum_over, y_over)
        assert yp.download(np.float32, a.size).tobytes() == y_want.tobytes(), (sum_over, y_over)
        for t in (da, db, ds, dy):
            t.free()
    import cactus_amd as ca
    da = dev.to_device(a)
    assert dev.lib.chip_add_rms_norm_mul(da.ptr, ne0, da.ptr, ne0, da.ptr, ne0, n, ne0, 1e-6, wp, da.ptr, ne0, None) == ca.CHIP_EINVAL
    da.free(); dw.free()


def test_scale_and_gelu_equal_the_oracle(dev, orc):
    """chip_scale: one multiply per element.  chip_gelu: the reference's fp16-table form, over every finite fp16 value, random
    values that round to either neighbour, and the two cut-offs; rows with a stride, and a length that is no multiple of 4."""
    import ctypes as C
    rng = np.random.default_rng(21)
    table = np.zeros(65536, np.uint16)
    dev.check(dev.lib.chip_gelu_table(table.ctypes.data_as(C.c_void_p)))
    dt = dev.to_device(table)
    h = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    h = h[np.isfinite(h)]
    edge = np.array([-10.0, np.nextafter(np.float32(-10), np.float32(0)), 10.0, np.nextafter(np.float32(10), np.float32(0)), 0.0, -0.0,
                     1.0 + 2.0 ** -11, 1.0 + 2.0 ** -11 + 2.0 ** -20, 65519.0, 1e-8, -1e-8, 3e38, -3e38], np.float32)
    flat = np.concatenate([h, (rng.standard_normal(20000) * 4).astype(np.float32), edge])
    for ne0 in (64, 1001):
        x = flat[: flat.size // ne0 * ne0].reshape(-1, ne0)
        n = x.shape[0]
        dx, dy = dev.to_device(x), dev.alloc(x.nbytes)
        dev.check(dev.lib.chip_gelu(dx.ptr, ne0, n, ne0, dt.ptr, dy.ptr, ne0, None))
        dev.sync()
        with np.errstate(all="ignore"):
            assert dy.download(np.float32, x.size).tobytes() == orc.gelu(x).tobytes()
        for v in (0.125, 0.08838834764831845, -3.7):
            dev.check(dev.lib.chip_scale(dx.ptr, ne0, n, ne0, v, dy.ptr, ne0, None))
            dev.sync()
            with np.errstate(all="ignore"):
                assert dy.download(np.float32, x.size).tobytes() == orc.scale(x, v).tobytes()
        dev.check(dev.lib.chip_scale(dx.ptr, ne0, n, ne0, 2.0, dx.ptr, ne0, None))                 # in place
        dev.sync()
        with np.errstate(all="ignore"):
            assert dx.download(np.float32, x.size).tobytes() == (x * np.float32(2)).tobytes()
        for t in (dx, dy):
            t.free()
    dt.free()


@pytest.mark.parametrize("wt", ["Q6_K", "Q4_K", "Q8_0", "Q5_1"])
@pytest.mark.parametrize("n,ne0", [(1, 14336), (4, 14336), (9, 4096), (3, 256), (40, 1024)])
def test_silu_mul_that_leaves_quantized_rows(dev, orc, wt, n, ne0):
    """chip_silu_mul_quantized: y equals chip_silu_mul's bit for bit, and the workspace holds what chip_mul_mat_prepare
    writes from y (compared as the reference's activation blocks against the oracle's quantizer); a matmul over those rows
    (chip_mul_mat_run) then equals chip_mul_mat on y."""
    import cactus_amd as ca
    t = getattr(ca, wt)
    a, b = inputs(19 * n + ne0, n, ne0), inputs(23 * n + ne0, n, ne0)
    da, db, dy = dev.to_device(a), dev.to_device(b), dev.alloc(a.nbytes)
    N = 48
    wsz = dev.lib.chip_mul_mat_workspace_size_n(t, ne0, N, n)
    ws = dev.alloc(wsz)
    dev.check(dev.lib.chip_silu_mul_quantized(da.ptr, ne0, db.ptr, ne0, n, ne0, dy.ptr, ne0, t, ws.ptr, wsz, None))
    dev.sync()
    y = dy.download(np.float32, a.size).reshape(n, ne0)
    with np.errstate(all="ignore"):
        want = dev.silu_mul(a, b)
    assert y.tobytes() == want.tobytes()
    at = dev.lib.chip_vec_dot_type(t)
    rs = dev.row_size(at, ne0)
    blk = dev.alloc(n * rs)
    dev.check(dev.lib.chip_workspace_to_blocks(t, ne0, n, ws.ptr, blk.ptr, None))
    dev.sync()
    got = blk.download(np.uint8, n * rs).reshape(n, rs)
    assert np.array_equal(got, orc.quantize_activation(at, y))
    W = orc.quantize_weights(t, (np.random.default_rng(ne0).standard_normal((N, ne0)) * 0.05).astype(np.float32))
    dW, dz = dev.to_device(W), dev.alloc(n * N * 4)
    dev.check(dev.lib.chip_mul_mat_run_ws(t, dW.ptr, dev.row_size(t, ne0), ne0, N, n, ws.ptr, wsz, dz.ptr, N, None))
    dev.sync()
    assert dz.download(np.float32, n * N).reshape(n, N).tobytes() == dev.mul_mat(t, W, y).tobytes()
    for tt in (da, db, dy, ws, blk, dW, dz):
        tt.free()
    # rows that are no multiple of 256 are declined, nothing written
    dx = dev.to_device(inputs(3, 2, 320))
    dyy, ws2 = dev.alloc(2 * 320 * 4), dev.alloc(4096)
    assert dev.lib.chip_silu_mul_quantized(dx.ptr, 320, dx.ptr, 320, 2, 320, dyy.ptr, 320, ca.Q8_0, ws2.ptr, 4096, None) == ca.CHIP_EUNSUPPORTED


def test_silu_mul_quantized_argument_errors(dev):
    import cactus_amd as ca
    L = dev.lib
    ne0 = 512
    a, ws = dev.to_device(inputs(5, 2, ne0)), dev.alloc(1 << 16)
    y = dev.alloc(2 * ne0 * 4)
    call = lambda **k: L.chip_silu_mul_quantized(k.get("x", a.ptr), k.get("ldx", ne0), k.get("b", a.ptr), ne0, k.get("n", 2), k.get("ne0", ne0),
                                                 k.get("y", y.ptr), ne0, k.get("t", ca.Q4_K), k.get("ws", ws.ptr), k.get("wsz", 1 << 16), None)
    assert call() == ca.CHIP_OK
    assert call(n=0) == ca.CHIP_OK and call(ne0=0) == ca.CHIP_OK          # nothing to do
    assert call(n=-1) == ca.CHIP_EINVAL
    assert call(t=ca.F16) == ca.CHIP_EUNSUPPORTED                         # no quantized activation format
    assert call(t=77) == ca.CHIP_EUNSUPPORTED
    assert call(ws=None) == ca.CHIP_EINVAL and call(ws=ws.ptr + 4) == ca.CHIP_EINVAL
    assert call(wsz=64) == ca.CHIP_ENOMEM
    assert call(ldx=ne0 - 4) == ca.CHIP_EINVAL                            # rows overlap
    assert call(x=a.ptr + 4) == ca.CHIP_EUNSUPPORTED                      # not 16-byte aligned: the caller takes chip_silu_mul
    dev.sync()
    for t in (a, ws, y):
        t.free()


@pytest.mark.parametrize("wt", ["Q4_K", "Q6_K", "Q8_0", "Q4_1"])
@pytest.mark.parametrize("n,ne0", [(1, 4096), (9, 4096), (3, 256), (5, 8192), (40, 1024)])
@pytest.mark.parametrize("with_add", [False, True])
def test_norm_that_leaves_quantized_rows(dev, orc, wt, n, ne0, with_add):
    """chip_rms_norm_quantized: y equals the unquantizing entry points bit for bit, and the workspace holds what
    chip_mul_mat_prepare writes from y (compared as the reference's activation blocks, and against the oracle's quantizer)."""
    import cactus_amd as ca
    import oracle as O
    t = getattr(ca, wt)
    a, b = inputs(13 * n + ne0, n, ne0), inputs(17 * n + ne0, n, ne0)
    w = (1.0 + 0.1 * np.random.default_rng(ne0).standard_normal(ne0)).astype(np.float32)
    da, db, dw = dev.to_device(a), dev.to_device(b), dev.to_device(w)
    ds, dy = dev.alloc(a.nbytes), dev.alloc(a.nbytes)
    wsz = dev.lib.chip_mul_mat_workspace_size(t, ne0, n)
    ws = dev.alloc(wsz)
    dev.check(dev.lib.chip_rms_norm_quantized(da.ptr, ne0, db.ptr if with_add else None, ne0, ds.ptr if with_add else None, ne0, n, ne0,
                                              1e-5, dw.ptr, dy.ptr, ne0, t, ws.ptr, wsz, None))
    dev.sync()
    y = dy.download(np.float32, a.size).reshape(n, ne0)
    with np.errstate(all="ignore"):
        x0 = dev.binary("add", a, b) if with_add else a
        want = dev.binary("mul", dev.rms_norm(x0, 1e-5), w)
    assert y.tobytes() == want.tobytes()
    if with_add:
        assert ds.download(np.float32, a.size).tobytes() == x0.tobytes()
    at = dev.lib.chip_vec_dot_type(t)
    rs = dev.row_size(at, ne0)
    blk = dev.alloc(n * rs)
    dev.check(dev.lib.chip_workspace_to_blocks(t, ne0, n, ws.ptr, blk.ptr, None))
    dev.sync()
    got = blk.download(np.uint8, n * rs).reshape(n, rs)
    assert np.array_equal(got, orc.quantize_activation(at, y))
    for tt in (da, db, dw, ds, dy, ws, blk):
        tt.free()
    # rows that are no multiple of 256 are declined, nothing written
    dx = dev.to_device(inputs(3, 2, 320))
    dyy, ws2 = dev.alloc(2 * 320 * 4), dev.alloc(4096)
    assert dev.lib.chip_rms_norm_quantized(dx.ptr, 320, None, 0, None, 0, 2, 320, 1e-5, None, dyy.ptr, 320, ca.Q8_0, ws2.ptr, 4096, None) \
        == ca.CHIP_EUNSUPPORTED
