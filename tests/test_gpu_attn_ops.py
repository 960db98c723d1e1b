"""GPU parity of the attention-side ops (SOFT_MAX, CPY / CONT, ROPE), through the C-ABI, against the CPU oracle (pinned
bit-exact on the reference build).

Bars: CPY / CONT bit-exact; SOFT_MAX within one fp32 ulp per element and bit-exact in practice (the exponentials and the
group sums are the reference's operation by operation; only the double sum over the groups is ordered differently);
ROPE |dy| <= 4e-7 * (|x0| + |x1|) * mscale per rotated pair (cos and sin may differ from the C library's by one unit in
the last place), pass-through channels bit-exact."""
import ctypes as C

import numpy as np
import pytest

import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    import cactus_amd
    return cactus_amd.Device(0)


def causal_mask(ne01, ne00, n_past, dtype, pad_rows=0):
    m = np.full((ne01 + pad_rows, ne00), -np.inf, np.float32)
    for i in range(ne01):
        m[i, : min(ne00, n_past + i + 1)] = 0.0
    return m.astype(dtype)


def assert_soft_max_close(y, ref):
    ulp = np.spacing(np.abs(ref))
    assert (np.abs(y.astype(np.float64) - ref) <= ulp).all()
    assert (y.view(np.uint32) == ref.view(np.uint32)).mean() > 0.999


# (n_head, ne01, ne00): register-resident rows of 1, 2 and 4 groups per thread, and the streaming path beyond 8192 values
SOFT_MAX_SHAPES = [(1, 1, 32), (4, 3, 256), (8, 5, 1000), (32, 1, 2048), (2, 16, 4096), (3, 2, 8192), (2, 3, 8200), (1, 2, 40000)]


@pytest.mark.parametrize("n_head,ne01,ne00", SOFT_MAX_SHAPES)
def test_soft_max(dev, orc, n_head, ne01, ne00):
    rng = np.random.default_rng(n_head * 1000 + ne00)
    x = (rng.standard_normal((n_head, ne01, ne00)) * 6).astype(np.float32)
    x[0, 0, :8] = [30.0, -30.0, 88.0, -104.0, 0.0, 1e-3, -200.0, 50.0]
    assert_soft_max_close(dev.soft_max(x), orc.soft_max(x))
    for dt in (np.float32, np.float16):
        mask = causal_mask(ne01, ne00, max(0, ne00 - ne01 - 3), dt, pad_rows=3)
        for scale in (1.0, 0.08838834764831845):
            ref = orc.soft_max(x, mask, scale)
            y = dev.soft_max(x, mask, scale)
            assert_soft_max_close(y, ref)
            assert np.all(y[np.broadcast_to(np.isinf(mask[:ne01]), y.shape)] == 0.0)
    bias = (rng.standard_normal((ne01, ne00)) * 2).astype(np.float32)
    assert_soft_max_close(dev.soft_max(x, bias, 0.5), orc.soft_max(x, bias, 0.5))


def test_soft_max_in_place_and_strided(dev, orc):
    import cactus_amd as ca
    rng = np.random.default_rng(2)
    n_rows, ne00, ld = 6, 264, 272
    buf = np.zeros((n_rows, ld), np.float32)
    buf[:, :ne00] = rng.standard_normal((n_rows, ne00)) * 3
    d = dev.to_device(buf)
    dev.check(dev.lib.chip_soft_max(d.ptr, ld, None, ca.F32, ne00, n_rows, n_rows, 0.3, 0.0, d.ptr, ld, None))
    dev.sync()
    out = d.download(np.float32, buf.size).reshape(n_rows, ld)
    assert_soft_max_close(np.ascontiguousarray(out[:, :ne00]), orc.soft_max(buf[None, :, :ne00], None, 0.3)[0])
    assert np.array_equal(out[:, ne00:], buf[:, ne00:])                      # the padding between rows is untouched


@pytest.mark.parametrize("ne00", [8192, 16384, 40960, 131072])
def test_soft_max_of_few_long_rows_equals_the_same_rows_in_a_large_batch(dev, orc, ne00):
    """Few rows of 8192 values or more (a decode step over a long context) run with 1024 threads per row: bit for bit what the
    same rows give among more rows than that kernel takes (256 threads per row), with an F16 causal mask and in place; the
    oracle within the soft-max tolerance."""
    import cactus_amd as ca
    rng = np.random.default_rng(ne00)
    few, many = 6, 134
    x = (rng.standard_normal((many, ne00)) * 5).astype(np.float32)
    x[0, :8] = [30.0, -30.0, 88.0, -104.0, 0.0, 1e-3, -200.0, 50.0]
    mask = np.zeros((1, ne00), np.float16)
    mask[0, ne00 - 37:] = -np.inf
    y_many = dev.soft_max(x[:, None, :], mask, 0.0884)[:, 0]
    y_few = dev.soft_max(x[:few, None, :], mask, 0.0884)[:, 0]
    assert y_few.tobytes() == y_many[:few].tobytes()
    assert_soft_max_close(y_few[None], orc.soft_max(x[None, :few], np.repeat(mask, few, 0), 0.0884))
    d, dm = dev.to_device(x[:few]), dev.to_device(mask)
    dev.check(dev.lib.chip_soft_max(d.ptr, ne00, dm.ptr, ca.F16, ne00, 1, few, 0.0884, 0.0, d.ptr, ne00, None))
    dev.sync()
    assert d.download(np.float32, few * ne00).tobytes() == y_few.tobytes()


def test_soft_max_declines_what_it_does_not_restate(dev):
    import cactus_amd as ca
    x = dev.to_device(np.zeros((2, 64), np.float32))
    L = dev.lib
    assert L.chip_soft_max(x.ptr, 64, None, ca.F32, 60, 1, 2, 1.0, 0.0, x.ptr, 64, None) == ca.CHIP_EUNSUPPORTED   # row tail
    assert L.chip_soft_max(x.ptr, 64, x.ptr, ca.F32, 64, 1, 2, 1.0, 8.0, x.ptr, 64, None) == ca.CHIP_EUNSUPPORTED  # ALiBi
    assert L.chip_soft_max(x.ptr, 64, x.ptr, ca.Q8_0, 64, 1, 2, 1.0, 0.0, x.ptr, 64, None) == ca.CHIP_EUNSUPPORTED
    assert L.chip_soft_max(x.ptr, 62, None, ca.F32, 64, 1, 2, 1.0, 0.0, x.ptr, 64, None) == ca.CHIP_EINVAL
    assert L.chip_soft_max(x.ptr, 64, None, ca.F32, 64, 1, 0, 1.0, 0.0, x.ptr, 64, None) == ca.CHIP_OK


def cpy_inputs(shape, seed):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    x.reshape(-1)[:6] = [65504.0, 65520.0, 1e-8, -6.1e-5, 2049.0, 2051.0]         # fp16 max, overflow, underflow, ties
    return x


@pytest.mark.parametrize("ne1,ne0", [(1, 1024), (7, 96), (33, 130), (512, 1024), (5, 3)])
def test_cpy_flat_and_transposed(dev, orc, ne1, ne0):
    x = cpy_inputs((ne1, ne0), ne1 + ne0)
    with np.errstate(all="ignore"):
        h = x.astype(np.float16)
        # the K-cache store: dense F32 -> dense F16
        assert dev.cpy(x, np.float16).tobytes() == orc.cpy(x, np.float16).tobytes()
        # CONT of a transposed view, every type pair
        assert dev.cpy(x.T, np.float16).tobytes() == orc.cpy(x.T, np.float16).tobytes()
        assert dev.cpy(x.T, np.float32).tobytes() == orc.cpy(x.T, np.float32).tobytes()
        assert dev.cpy(h.T, np.float16).tobytes() == orc.cpy(h.T, np.float16).tobytes()
        assert dev.cpy(h.T, np.float32).tobytes() == orc.cpy(h.T, np.float32).tobytes()
        assert dev.cpy(h, np.float32).tobytes() == orc.cpy(h, np.float32).tobytes()


@pytest.mark.parametrize("n_tokens,n_embd,kv_size,head", [(1, 1024, 4096, 77), (33, 256, 512, 100), (512, 1024, 2048, 1024)])
def test_cpy_into_the_transposed_v_cache(dev, orc, n_tokens, n_embd, kv_size, head):
    # reference llama-kv-cache.cpp:631-656: v_cur [n_tokens][n_embd] transposed into the view [n_embd rows of kv_size] at column `head`
    x = cpy_inputs((n_tokens, n_embd), n_tokens)
    with np.errstate(all="ignore"):
        got = dev.cpy(x.T, np.float16, dst_strides=(kv_size * 2, 2), dst_elems=n_embd * kv_size).reshape(n_embd, kv_size)
        want = np.zeros((n_embd, kv_size), np.float16)
        want[:, :n_tokens] = orc.cpy(x.T, np.float16)
    assert got.tobytes() == want.tobytes()
    # placed at column `head` through the destination pointer: same bytes, shifted
    import cactus_amd as ca
    A = C.c_int64 * 4
    dsrc = dev.to_device(x)
    ddst = dev.alloc(n_embd * kv_size * 2)
    ddst.upload(np.zeros(n_embd * kv_size, np.float16))
    if head + n_tokens <= kv_size:
        shape = A(n_tokens, n_embd, 1, 1)
        dev.check(dev.lib.chip_cpy(dsrc.ptr, ca.F32, shape, A(n_embd * 4, 4, 0, 0), ddst.ptr + 2 * head, ca.F16, shape,
                                   A(2, kv_size * 2, 0, 0), None))
        dev.sync()
        got = ddst.download(np.float16, n_embd * kv_size).reshape(n_embd, kv_size)
        want = np.zeros((n_embd, kv_size), np.float16)
        with np.errstate(all="ignore"):
            want[:, head:head + n_tokens] = orc.cpy(x.T, np.float16)
        assert got.tobytes() == want.tobytes()


def test_cont_of_the_permuted_attention_output(dev, orc):
    # reference llama-graph.cpp:1161-1163: kqv [n_head][n_tokens][head_dim] permuted to [n_tokens][n_head][head_dim] and made dense
    rng = np.random.default_rng(4)
    kqv = rng.standard_normal((8, 37, 64)).astype(np.float32)
    view = kqv.transpose(1, 0, 2)
    assert dev.cpy(view, np.float32).tobytes() == orc.cpy(view, np.float32).tobytes()
    assert dev.cpy(view, np.float32, dst_shape=(37, 8 * 64)).tobytes() == orc.cpy(view, np.float32).tobytes()    # lm_ggml_cont_2d
    assert dev.cpy(view, np.float16, dst_shape=(37 * 8, 64)).tobytes() == orc.cpy(view, np.float16).tobytes()
    big = rng.standard_normal((2, 3, 5, 16)).astype(np.float32)
    for perm in ((0, 2, 1, 3), (1, 0, 3, 2), (3, 2, 1, 0), (2, 3, 0, 1)):
        v = big.transpose(perm)
        assert dev.cpy(v, np.float32).tobytes() == orc.cpy(v, np.float32).tobytes()
        assert dev.cpy(v, np.float16).tobytes() == orc.cpy(v, np.float16).tobytes()


def test_cpy_rejects_bad_arguments(dev):
    import cactus_amd as ca
    A = C.c_int64 * 4
    d = dev.alloc(1024)
    L = dev.lib
    ne, nb4, nb2 = A(16, 4, 1, 1), A(4, 64, 256, 256), A(2, 32, 128, 128)
    assert L.chip_cpy(d.ptr, ca.Q8_0, ne, nb4, d.ptr, ca.F16, ne, nb2, None) == ca.CHIP_EUNSUPPORTED
    assert L.chip_cpy(d.ptr, ca.F32, ne, nb4, d.ptr, ca.Q8_0, ne, nb2, None) == ca.CHIP_EUNSUPPORTED
    assert L.chip_cpy(d.ptr, ca.F32, ne, A(3, 64, 256, 256), d.ptr + 512, ca.F16, ne, nb2, None) == ca.CHIP_EINVAL
    assert L.chip_cpy(d.ptr + 2, ca.F32, ne, nb4, d.ptr + 512, ca.F16, ne, nb2, None) == ca.CHIP_EINVAL
    assert L.chip_cpy(None, ca.F32, ne, nb4, d.ptr, ca.F16, ne, nb2, None) == ca.CHIP_EINVAL
    assert L.chip_cpy(d.ptr, ca.F32, ne, nb4, d.ptr + 512, ca.F16, A(16, 5, 1, 1), nb2, None) == ca.CHIP_EINVAL   # element counts differ
    zero = A(0, 4, 1, 1)
    assert L.chip_cpy(None, ca.F32, zero, nb4, None, ca.F16, zero, nb2, None) == ca.CHIP_OK


def rope_tolerance(x, n_dims, mode, mscale):
    half = n_dims // 2
    tol = np.zeros_like(x, dtype=np.float64)
    ax = np.abs(x.astype(np.float64))
    if mode == 0:
        pair = ax[..., 0:n_dims:2] + ax[..., 1:n_dims:2]
        tol[..., 0:n_dims:2] = pair
        tol[..., 1:n_dims:2] = pair
    else:
        pair = ax[..., :half] + ax[..., half:n_dims]
        tol[..., :half] = pair
        tol[..., half:n_dims] = pair
    return 4e-7 * abs(mscale) * tol


@pytest.mark.parametrize("mode", [0, 2])
@pytest.mark.parametrize("ne0,n_dims,n_head,n_tokens", [(128, 128, 32, 1), (128, 128, 8, 7), (64, 32, 3, 2), (128, 64, 2, 7), (256, 256, 4, 3)])
def test_rope(dev, orc, mode, ne0, n_dims, n_head, n_tokens):
    rng = np.random.default_rng(ne0 + n_dims + mode)
    x = rng.standard_normal((n_tokens, n_head, ne0)).astype(np.float32)
    pos = np.array([0, 1, 17, 4095, 100000, 31, 3000000][:n_tokens], np.int32)   # the last one takes the full-range reduction
    ff = (1.0 + rng.random(n_dims // 2) * 7).astype(np.float32)
    cases = [({}, 1.0), (dict(freq_base=500000.0, freq_scale=0.25), 1.0), (dict(freq_factors=ff), 1.0),
             (dict(freq_scale=0.25, ext_factor=1.0, attn_factor=1.2, n_ctx_orig=2048), 1.2 * (1.0 + 0.1 * np.log(4.0)))]
    for kw, mscale in cases:
        ref = orc.rope(x, pos, n_dims, mode, **kw)
        y = dev.rope(x, pos, n_dims, mode, **kw)
        assert (np.abs(y.astype(np.float64) - ref) <= rope_tolerance(x, n_dims, mode, mscale)).all(), kw
        assert y[..., n_dims:].tobytes() == x[..., n_dims:].tobytes()
        assert y[pos == 0].tobytes() == ref[pos == 0].tobytes()               # angle 0: cos 1, sin 0 exactly
        assert (y.view(np.uint32) == ref.view(np.uint32)).mean() > 0.9        # most values agree to the bit
        assert dev.rope(x, pos, n_dims, mode, two_step=True, **kw).tobytes() == y.tobytes()   # table + apply: the same bits


def test_rope_strided_in_place(dev, orc):
    # rope over the Q part of a fused QKV activation: head stride ne0, token stride 3 * n_head * ne0
    import cactus_amd as ca
    rng = np.random.default_rng(9)
    n_tokens, n_head, ne0 = 5, 4, 64
    qkv = rng.standard_normal((n_tokens, 3, n_head, ne0)).astype(np.float32)
    pos = np.arange(10, 10 + n_tokens, dtype=np.int32)
    d, dp = dev.to_device(qkv), dev.to_device(pos)
    tok = 3 * n_head * ne0
    dev.check(dev.lib.chip_rope(d.ptr, ne0, tok, dp.ptr, None, ne0, n_head, n_tokens, ne0, 2, 4096, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0,
                                d.ptr, ne0, tok, None))
    dev.sync()
    out = d.download(np.float32, qkv.size).reshape(qkv.shape)
    ref = orc.rope(qkv[:, 0], pos, ne0, 2)
    assert (np.abs(out[:, 0].astype(np.float64) - ref) <= rope_tolerance(qkv[:, 0], ne0, 2, 1.0)).all()
    assert out[:, 1:].tobytes() == qkv[:, 1:].tobytes()


def test_rope_declines_multi_section_modes(dev):
    import cactus_amd as ca
    d = dev.alloc(4096)
    L = dev.lib
    args = (None, 64, 1, 1, 64)
    for mode in (8, 24):
        assert L.chip_rope(d.ptr, 64, 64, d.ptr, None, 64, 1, 1, 64, mode, 4096, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0, d.ptr, 64, 64,
                           None) == ca.CHIP_EUNSUPPORTED
    assert L.chip_rope(d.ptr, 64, 64, d.ptr, None, 64, 1, 1, 63, 0, 4096, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0, d.ptr, 64, 64,
                       None) == ca.CHIP_EINVAL
    assert L.chip_rope(d.ptr, 64, 64, None, None, 64, 1, 1, 64, 0, 4096, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0, d.ptr, 64, 64,
                       None) == ca.CHIP_EINVAL


def attn_case(seed, hd, n_head, n_head_kv, n_tokens, n_kv, kv_size):
    """An F16 KV cache laid out like the reference's (K: [kv_size][n_head_kv * hd]; V transposed: [n_head_kv * hd][kv_size])
    with n_kv positions in use, new queries and a probability tensor."""
    rng = np.random.default_rng(seed)
    k_cache = np.zeros((kv_size, n_head_kv, hd), np.float16)
    k_cache[:n_kv] = rng.standard_normal((n_kv, n_head_kv, hd)).astype(np.float16)
    vt_cache = np.zeros((n_head_kv, hd, kv_size), np.float16)
    vt_cache[:, :, :n_kv] = rng.standard_normal((n_head_kv, hd, n_kv)).astype(np.float16)
    q = rng.standard_normal((n_tokens, n_head, hd)).astype(np.float32)
    p = rng.random((n_head, n_tokens, n_kv)).astype(np.float32)
    p /= p.sum(-1, keepdims=True)
    return k_cache, vt_cache, q, p


# (hd, n_head, n_head_kv, n_tokens, n_kv, kv_size): LLaMA-3-8B decode and a short prefill, multi-head attention, head sizes
# that use 8 / 16 / 32 lanes per cache row, a GQA ratio that is no power of two, positions that are no multiple of 64
# the last five have 64 or more (head, token) pairs per KV head: with a workspace they take the GEMM route, the last two
# with K (head size 96; 104 and 1056 cache positions) that is no multiple of the GEMM's 64-value stage
@pytest.mark.parametrize("mode", [0, 2])
@pytest.mark.parametrize("ne0,n_dims,n_head,n_tokens", [(128, 128, 8, 1), (128, 128, 8, 7), (64, 32, 3, 2), (256, 256, 40, 3)])
def test_rope_with_the_cache_store_in_one_launch(dev, mode, ne0, n_dims, n_head, n_tokens):
    """chip_rope_apply_store: the fp32 result equals chip_rope's bit for bit, the fp16 copy equals chip_cpy of that result
    (round to nearest even), for rotated and passed-through values, also past the first 2048 items of a token."""
    rng = np.random.default_rng(ne0 + n_head + mode)
    x = (rng.standard_normal((n_tokens, n_head, ne0)) * 3).astype(np.float32)
    pos = np.array([5, 0, 4095, 17, 100000, 31, 2][:n_tokens], np.int32)
    y, h = dev.rope(x, pos, n_dims, mode, freq_base=500000.0, store_f16=True)
    assert y.tobytes() == dev.rope(x, pos, n_dims, mode, freq_base=500000.0).tobytes()
    assert h.tobytes() == dev.cpy(y.reshape(-1, ne0), np.float16).tobytes() == y.astype(np.float16).tobytes()


@pytest.mark.parametrize("mode", [0, 2])
@pytest.mark.parametrize("ne0,n_dims,heads_a,heads_b,n_tokens", [(128, 128, 32, 8, 1), (128, 128, 32, 8, 5), (64, 32, 3, 1, 2), (256, 256, 40, 40, 3)])
def test_rope_of_q_and_k_in_one_launch(dev, mode, ne0, n_dims, heads_a, heads_b, n_tokens):
    """chip_rope_apply_two: every output equals what chip_rope / chip_rope_apply_store give for that tensor alone, bit for
    bit, also when one tensor asks for its fp16 copy only."""
    rng = np.random.default_rng(ne0 + heads_a + mode)
    xa = (rng.standard_normal((n_tokens, heads_a, ne0)) * 3).astype(np.float32)
    xb = (rng.standard_normal((n_tokens, heads_b, ne0)) * 3).astype(np.float32)
    pos = np.array([5, 0, 4095, 17, 100000][:n_tokens], np.int32)
    ya = dev.rope(xa, pos, n_dims, mode, freq_base=500000.0)
    yb, hb = dev.rope(xb, pos, n_dims, mode, freq_base=500000.0, store_f16=True)
    a, b = dev.rope_two(xa, xb, pos, n_dims, mode, freq_base=500000.0)
    assert a["f32"].tobytes() == ya.tobytes() and "f16" not in a
    assert b["f32"].tobytes() == yb.tobytes() and b["f16"].tobytes() == hb.tobytes()
    a, b = dev.rope_two(xa, xb, pos, n_dims, mode, want=(("f32", "f16"), ("f16",)), freq_base=500000.0)
    assert a["f32"].tobytes() == ya.tobytes() and a["f16"].tobytes() == ya.astype(np.float16).tobytes()
    assert b["f16"].tobytes() == hb.tobytes() and "f32" not in b


def test_rope_of_two_tensors_rejects_bad_operands(dev):
    import cactus_amd as ca
    L = dev.lib
    d = dev.alloc(1 << 16)
    good = lambda: ca.RopeOperand(d.ptr, 64, 256, 4, d.ptr + 4096, 64, 256, None, 0, 0)
    a, b = good(), good()
    assert L.chip_rope_apply_two(C.byref(a), C.byref(b), d.ptr + 8192, 64, 1, 64, 2, None) == ca.CHIP_OK
    assert L.chip_rope_apply_two(C.byref(a), None, d.ptr + 8192, 64, 1, 64, 2, None) == ca.CHIP_EINVAL
    assert L.chip_rope_apply_two(C.byref(a), C.byref(b), None, 64, 1, 64, 2, None) == ca.CHIP_EINVAL
    assert L.chip_rope_apply_two(C.byref(a), C.byref(b), d.ptr + 8192, 64, 1, 64, 8, None) == ca.CHIP_EUNSUPPORTED
    b.y = None                                                                    # neither output
    assert L.chip_rope_apply_two(C.byref(a), C.byref(b), d.ptr + 8192, 64, 1, 64, 2, None) == ca.CHIP_EINVAL
    b = good(); b.ldx1 = 32
    assert L.chip_rope_apply_two(C.byref(a), C.byref(b), d.ptr + 8192, 64, 1, 64, 2, None) == ca.CHIP_EINVAL
    b = good(); b.y_f16 = d.ptr + 16384 + 1; b.ld16_1 = 64
    assert L.chip_rope_apply_two(C.byref(a), C.byref(b), d.ptr + 8192, 64, 1, 64, 2, None) == ca.CHIP_EINVAL
    dev.sync()


ATTN_SHAPES = [(128, 32, 8, 1, 4096, 4096), (128, 32, 8, 7, 288, 512), (64, 8, 8, 3, 96, 128), (256, 4, 2, 2, 160, 160),
               (96, 6, 2, 5, 72, 80), (128, 28, 4, 2, 104, 128), (128, 8, 2, 70, 128, 128), (128, 32, 8, 130, 320, 512),
               (64, 4, 4, 100, 192, 256), (96, 6, 2, 40, 104, 128), (128, 32, 8, 512, 1056, 2048),
               # 5 to 63 (head, token) pairs per KV head: the 16 x 16 x 32 matrix-core kernels, one to four column groups
               (128, 32, 8, 8, 1040, 2048), (128, 32, 8, 15, 520, 1024), (256, 8, 2, 4, 296, 512), (256, 8, 2, 8, 296, 512),
               (256, 16, 2, 5, 264, 512), (64, 16, 2, 6, 1032, 2048), (128, 32, 8, 2, 4096, 4096), (80, 8, 1, 3, 24, 32),
               # 65 to 128 pairs: kqv with K split over workgroups (eight column groups), kq through the GEMM
               (128, 32, 8, 32, 1048, 2048), (96, 12, 2, 17, 520, 1024),
               # more than 128 pairs over a long cache (K not a multiple of the GEMM's 64-value stage)
               (128, 8, 2, 40, 2056, 4096), (64, 8, 2, 64, 4104, 4352),
               # a decode step over a long context (kqv rows of more than 8192 values: four cache rows per workgroup)
               (128, 32, 8, 1, 16384, 16384), (128, 8, 2, 1, 9008, 12288)]


@pytest.mark.parametrize("hd,n_head,n_head_kv,n_tokens,n_kv,kv_size", ATTN_SHAPES)
def test_attention_matmuls_over_the_cache(dev, orc, hd, n_head, n_head_kv, n_tokens, n_kv, kv_size):
    k_cache, vt_cache, q, p = attn_case(hd + n_kv, hd, n_head, n_head_kv, n_tokens, n_kv, kv_size)
    # kq = mul_mat(k, q): the K cache as [n_head_kv][n_kv][hd] (rows one position apart), q as [n_head][n_tokens][hd]
    kv = k_cache[:n_kv].transpose(1, 0, 2)
    qv = q.transpose(1, 0, 2)
    want = orc.mul_mat_f16_batched(kv, qv, want=("sum_abs",))
    got = dev.mul_mat_f16_batched(kv, qv)
    assert got.shape == (n_head, n_tokens, n_kv)
    assert (np.abs(got - want["y"]) <= 1e-5 * want["sum_abs"] + 1e-30).all()
    # kqv = mul_mat(v, p): the transposed V cache as [n_head_kv][hd][n_kv] (rows kv_size apart)
    vv = vt_cache[:, :, :n_kv]
    want = orc.mul_mat_f16_batched(vv, p, want=("sum_abs",))
    got = dev.mul_mat_f16_batched(vv, p)
    assert got.shape == (n_head, n_tokens, hd)
    assert (np.abs(got - want["y"]) <= 1e-5 * want["sum_abs"] + 1e-30).all()
    if n_tokens * (n_head // n_head_kv) > 4:                                    # the same without a workspace: the one-launch kernels
        got = dev.mul_mat_f16_batched(vv, p, workspace=False)
        assert (np.abs(got - want["y"]) <= 1e-5 * want["sum_abs"] + 1e-30).all()
        want = orc.mul_mat_f16_batched(kv, qv, want=("sum_abs",))
        got = dev.mul_mat_f16_batched(kv, qv, workspace=False)
        assert (np.abs(got - want["y"]) <= 1e-5 * want["sum_abs"] + 1e-30).all()


# (hd, n_head, n_head_kv, n_tokens, n_kv, kv_size): LLaMA-3-8B's decode step; multi-head attention with 1, 2 and 4 tokens; 3 and 2
# query heads per KV head; a cache short enough for the short-rows kernel; ragged sizes
MERGE_SHAPES = [(128, 32, 8, 1, 4096, 4096), (64, 4, 4, 1, 1000, 1024), (64, 4, 4, 4, 520, 1024), (128, 8, 8, 2, 264, 512),
                (256, 6, 2, 1, 4104, 8192), (96, 4, 2, 2, 72, 128), (128, 2, 1, 1, 5000, 8192), (80, 8, 2, 1, 136, 256),
                (128, 8, 2, 1, 16392, 16640)]


@pytest.mark.parametrize("hd,n_head,n_head_kv,n_tokens,n_kv,kv_size", MERGE_SHAPES)
def test_kqv_with_the_head_merge_in_one_launch(dev, hd, n_head, n_head_kv, n_tokens, n_kv, kv_size):
    """chip_mul_mat_f16_batched_two_copies: both copies hold the bits of chip_mul_mat_f16_batched, the second one laid out
    like chip_cpy's CONT of the permuted result (a token's heads side by side)."""
    _, vt_cache, _, p = attn_case(7 * hd + n_kv, hd, n_head, n_head_kv, n_tokens, n_kv, kv_size)
    vv = vt_cache[:, :, :n_kv]
    assert dev.lib.chip_mul_mat_f16_batched_second_copy_supported(n_head_kv, n_head, n_tokens) == 1
    want = dev.mul_mat_f16_batched(vv, p)
    got, merged = dev.mul_mat_f16_batched(vv, p, merged=True)
    assert got.tobytes() == want.tobytes()
    assert merged.shape == (n_tokens, n_head * hd)
    assert merged.tobytes() == np.ascontiguousarray(want.transpose(1, 0, 2)).tobytes()
    assert merged.tobytes() == dev.cpy(want.transpose(1, 0, 2), np.float32).tobytes()


def test_kqv_with_the_head_merge_declines_the_other_routes(dev):
    import cactus_amd as ca
    L = dev.lib
    for ne02, ne12, n, ok in ((8, 32, 1, 1), (8, 8, 4, 1), (2, 4, 2, 1), (8, 32, 2, 0), (1, 8, 1, 0), (8, 8, 5, 0), (8, 30, 1, 0), (0, 8, 1, 0)):
        assert L.chip_mul_mat_f16_batched_second_copy_supported(ne02, ne12, n) == ok
    d = dev.alloc(1 << 20)
    ok = [d.ptr, 1024, 1024 * 64, 512, 64, 2, d.ptr, 512, 512, 1, 4, d.ptr + (1 << 19), 64, 64, d.ptr + (1 << 18), 256, 64, None, 0, None]
    assert L.chip_mul_mat_f16_batched_two_copies(*ok) == ca.CHIP_OK

    def call(**kw):
        a = list(ok)
        for k, v in kw.items():
            a[int(k[1:])] = v
        return L.chip_mul_mat_f16_batched_two_copies(*a)
    assert call(_14=None) == ca.CHIP_EINVAL                                      # no second destination
    assert call(_10=16) == ca.CHIP_EUNSUPPORTED                                  # 8 query heads per KV head: the matrix-core kernels
    assert call(_9=3) == ca.CHIP_EUNSUPPORTED                                    # 3 tokens x 2 heads
    assert call(_14=d.ptr + (1 << 18) + 2) == ca.CHIP_EINVAL
    assert call(_15=-1) == ca.CHIP_EINVAL
    dev.sync()


def test_attention_matmul_exact_small_integers(dev):
    # halves and activations that are small integers: every product and partial sum is exact in fp32, so any summation
    # order gives the same bits, and a wrong index or a dropped term shows
    rng = np.random.default_rng(8)
    W = rng.integers(-8, 9, (3, 50, 72)).astype(np.float16)
    x = rng.integers(-8, 9, (6, 4, 72)).astype(np.float32)
    want = np.einsum("bnk,btk->btn", W.astype(np.float64)[np.arange(6) // 2], x.astype(np.float64)).astype(np.float32)
    assert dev.mul_mat_f16_batched(W, x).tobytes() == want.tobytes()


def test_attention_matmul_rounds_activations_to_fp16(dev, orc):
    # 1 + 2^-11 is a tie in fp16 (rounds to 1), 1 + 2^-11 + 2^-20 rounds up to 1 + 2^-10; 65520 overflows to inf
    W = np.ones((1, 1, 8), np.float16)
    x = np.zeros((1, 3, 8), np.float32)
    x[0, 0, 0] = 1 + 2.0 ** -11
    x[0, 1, 0] = 1 + 2.0 ** -11 + 2.0 ** -20
    x[0, 2, 0] = 65520.0
    with np.errstate(all="ignore"):
        got = dev.mul_mat_f16_batched(W, x)[0, :, 0]
    assert got[0] == 1.0 and got[1] == np.float32(1 + 2.0 ** -10) and np.isinf(got[2])
    assert got.tobytes() == orc.mul_mat_f16_batched(W, x)["y"][0, :, 0].tobytes()


def test_attention_matmul_rejects_bad_arguments(dev):
    import cactus_amd as ca
    d = dev.alloc(1 << 16)
    L = dev.lib
    ok = (d.ptr, 256, 256 * 16, 128, 16, 2, d.ptr, 128, 512, 1, 4, d.ptr, 16, 16, None, 0, None)
    assert L.chip_mul_mat_f16_batched(*ok) == ca.CHIP_OK
    dev.sync()

    def call(i, v):
        a = list(ok); a[i] = v
        return L.chip_mul_mat_f16_batched(*a)
    assert call(10, 3) == ca.CHIP_EINVAL              # ne12 not a multiple of ne02
    assert call(3, 100) == ca.CHIP_EUNSUPPORTED       # K not a multiple of 8
    assert call(1, 250) == ca.CHIP_EINVAL             # row stride not 16-byte aligned
    assert call(0, d.ptr + 2) == ca.CHIP_EINVAL
    assert call(7, 126) == ca.CHIP_EINVAL             # activation stride not a multiple of 4
    assert call(6, None) == ca.CHIP_EINVAL
    assert call(9, 0) == ca.CHIP_OK                   # no tokens


@pytest.mark.parametrize("wt", [O.F32] + list(O.WEIGHT_TYPES))
def test_get_rows_every_type(dev, orc, wt):
    nc, ne01 = 1024, 53
    rng = np.random.default_rng(wt + 3)
    w = (rng.standard_normal((ne01, nc)) * 0.3).astype(np.float32)
    w[0, :4] = [0.0, -0.0, 3.0, -3.0]
    if wt == O.F32:
        table = w
    elif wt == O.F16:
        table = w.astype(np.float16).view(np.uint8).reshape(ne01, -1)
    else:
        table = orc.quantize_weights(wt, w)
    ids = rng.integers(0, ne01, 40).astype(np.int32)
    ids[:3] = [0, ne01 - 1, 0]
    got = dev.get_rows(wt, table, nc, ids)
    assert got.tobytes() == orc.get_rows(wt, table, nc, ids).tobytes()
    # ids outside the table leave their rows unwritten (the wrapper pre-fills with NaN)
    bad = np.array([1, -1, ne01, 2], np.int32)
    got = dev.get_rows(wt, table, nc, bad)
    assert np.isnan(got[1]).all() and np.isnan(got[2]).all()
    assert got[[0, 3]].tobytes() == orc.get_rows(wt, table, nc, bad[[0, 3]]).tobytes()


def test_get_rows_batched_like_the_expert_weights(dev):
    # reference llama-graph.cpp:746: the router probabilities as [1, n_expert, n_tokens] picked by ids [n_used, n_tokens]
    import cactus_amd as ca
    n_expert, n_tokens, n_used = 8, 5, 2
    rng = np.random.default_rng(6)
    probs = rng.random((n_tokens, n_expert, 1)).astype(np.float32)
    ids = np.stack([rng.permutation(n_expert)[:n_used] for _ in range(n_tokens)]).astype(np.int32)
    dp, di, dy = dev.to_device(probs), dev.to_device(ids), dev.alloc(n_tokens * n_used * 4)
    dev.check(dev.lib.chip_get_rows(ca.F32, dp.ptr, 4, 4 * n_expert, 4 * n_expert * n_tokens, 1, n_expert, di.ptr, n_used, n_tokens, 1,
                                    n_used, n_used * n_tokens, dy.ptr, 1, n_used, n_used * n_tokens, None))
    dev.sync()
    got = dy.download(np.float32, n_tokens * n_used).reshape(n_tokens, n_used)
    assert np.array_equal(got, np.take_along_axis(probs[:, :, 0], ids, axis=1))


def test_get_rows_rejects_bad_arguments(dev):
    import cactus_amd as ca
    d = dev.alloc(1 << 14)
    L = dev.lib
    ok = [ca.Q4_K, d.ptr, 144, 144 * 4, 144 * 4, 256, 4, d.ptr, 2, 1, 1, 2, 2, d.ptr + 8192, 256, 512, 512, None]
    dev.check(L.chip_memset(d.ptr, 0, 1 << 14, None))
    assert L.chip_get_rows(*ok) == ca.CHIP_OK
    dev.sync()

    def call(i, v):
        a = list(ok); a[i] = v
        return L.chip_get_rows(*a)
    assert call(0, ca.Q8_K) == ca.CHIP_EUNSUPPORTED
    assert call(5, 200) == ca.CHIP_EINVAL              # not whole blocks
    assert call(1, d.ptr + 1) == ca.CHIP_EINVAL
    assert call(7, None) == ca.CHIP_EINVAL
    assert call(14, 100) == ca.CHIP_EINVAL             # dst row stride shorter than a row
    assert call(8, 0) == ca.CHIP_OK
