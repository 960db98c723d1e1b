"""ctypes bindings of the CPU oracle (liboracle.so) and, when it has been built, of the reference's own
ggml shared object (oracle/_ref/libggml_ref.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg,
as the checker.  The product package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "liboracle.so")
REF_SO = os.path.join(HERE, "_ref", "libggml_ref.so")

# lm_ggml_type values (reference ggml.h:351-391)
F32, Q4_0, Q8_0, Q4_K, Q6_K, Q8_K = 0, 2, 8, 12, 14, 15
Q5_0, Q5_K, IQ4_NL = 6, 13, 20
Q4_1, Q5_1, Q8_1 = 3, 7, 9
F16 = 1
Q2_K, Q3_K, IQ4_XS = 10, 11, 23
TYPE_NAMES = {Q2_K: "q2_K", Q3_K: "q3_K", IQ4_XS: "iq4_xs", F32: "f32", Q4_0: "q4_0", Q8_0: "q8_0", Q4_K: "q4_K", Q6_K: "q6_K", Q8_K: "q8_K",
              Q5_0: "q5_0", Q5_K: "q5_K", IQ4_NL: "iq4_nl", Q4_1: "q4_1", Q5_1: "q5_1", Q8_1: "q8_1", F16: "f16"}
BLOCK_ELEMS = {Q2_K: 256, Q3_K: 256, IQ4_XS: 256, F32: 1, Q4_0: 32, Q8_0: 32, Q4_K: 256, Q6_K: 256, Q8_K: 256, Q5_0: 32, Q5_K: 256, IQ4_NL: 32,
               Q4_1: 32, Q5_1: 32, Q8_1: 32, F16: 1}
BLOCK_BYTES = {Q2_K: 84, Q3_K: 110, IQ4_XS: 136, F32: 4, Q4_0: 18, Q8_0: 34, Q4_K: 144, Q6_K: 210, Q8_K: 292, Q5_0: 22, Q5_K: 176, IQ4_NL: 18,
               Q4_1: 20, Q5_1: 24, Q8_1: 36, F16: 2}
VEC_DOT_TYPE = {Q2_K: Q8_K, Q3_K: Q8_K, IQ4_XS: Q8_K, Q4_0: Q8_0, Q8_0: Q8_0, Q4_K: Q8_K, Q6_K: Q8_K, Q5_0: Q8_0, Q5_K: Q8_K, IQ4_NL: Q8_0,
                Q4_1: Q8_1, Q5_1: Q8_1, F16: F16}
WEIGHT_TYPES = (Q4_0, Q8_0, Q4_K, Q6_K, Q5_0, Q5_K, IQ4_NL, Q4_1, Q5_1, Q3_K, Q2_K, IQ4_XS, F16)
BLOCK_WEIGHT_TYPES = WEIGHT_TYPES[:-1]        # the types with per-block integer sums
# the 2- and 3-bit K-quants and IQ4_XS: decode and small batches on the GEMV kernels, no matrix-core kernels of their own
LOW_BIT_K_TYPES = (Q3_K, Q2_K, IQ4_XS)
# types whose weight quantizer is restated in the oracle (IQ4_NL, Q3_K and Q2_K weights come from the reference build, from
# the golden fixture, from a plain quantizer here, or are random bytes: any byte string is a valid block)
ORACLE_QUANTIZED = (Q4_0, Q8_0, Q4_K, Q6_K, Q5_0, Q5_K, Q4_1, Q5_1, F16)


IQ4_NL_VALUES = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float32)


def nearest_iq4_nl_rows(w):
    """fp32 [N, K] -> IQ4_NL rows: per 32-block d = max|x| / 127 (sign of the largest element, as fp16), index =
    nearest code point of x / d.  Not the reference's quantizer."""
    w = np.ascontiguousarray(w, np.float32)
    n, k = w.shape
    nb = k // 32
    blk = w.reshape(n, nb, 32)
    imax = np.abs(blk).argmax(-1)
    mx = np.take_along_axis(blk, imax[..., None], -1)[..., 0]
    d = (mx / np.float32(-127)).astype(np.float16)
    df = d.astype(np.float32)
    inv = np.where(df != 0, 1.0 / np.where(df != 0, df, 1), 0).astype(np.float32)
    idx = np.abs((blk * inv[..., None])[..., None] - IQ4_NL_VALUES).argmin(-1).astype(np.uint8)
    out = np.zeros((n, nb, 18), np.uint8)
    out[..., :2] = d.view(np.uint8).reshape(n, nb, 2)
    out[..., 2:] = idx[..., :16] | (idx[..., 16:] << 4)
    return out.reshape(n, nb * 18)


def random_iq4_nl_rows(seed, n, k):
    """Random but plausible IQ4_NL rows: uniform code indices, fp16 scales around 2e-4 (weights ~ N(0, 0.02))."""
    rng = np.random.default_rng(seed)
    nb = k // 32
    blk = np.zeros((n, nb, 18), np.uint8)
    d = (2e-4 * np.exp(rng.uniform(-1.0, 1.0, (n, nb)))).astype(np.float16)
    d[rng.random((n, nb)) < 0.05] *= np.float16(-1)
    blk[..., :2] = d.view(np.uint8).reshape(n, nb, 2)
    blk[..., 2:] = rng.integers(0, 256, (n, nb, 16), dtype=np.uint8)
    return blk.reshape(n, nb * 18)


def _k_sub_blocks(w):
    """fp32 [N, K] -> [N, K/256, 2 halves, 4 shifts, 2 parts, 16]: element 128 h + 32 j + 16 p + l of a super-block, i.e.
    bits 2 j of byte 32 h + 16 p + l of qs in the 2- and 3-bit K-quants; sub-block (scale) index 8 h + 2 j + p."""
    w = np.ascontiguousarray(w, np.float32)
    n, k = w.shape
    return w.reshape(n, k // 256, 2, 4, 2, 16)


def _pack_2bit(q):
    """q uint8 [N, nb, 2, 4, 2, 16] with values 0..3 -> qs uint8 [N, nb, 64]"""
    n, nb = q.shape[:2]
    out = np.zeros((n, nb, 2, 2, 16), np.uint8)
    for j in range(4):
        out |= (q[:, :, :, j] & 3) << (2 * j)
    return out.reshape(n, nb, 64)


def plain_q3_K_rows(w):
    """fp32 [N, K] -> Q3_K rows by a plain round-to-nearest quantizer: sub-block scale = max|x| / 4, super-block d =
    largest scale / 31, codes 0..31 (+32), q = round(x / (d code)) in [-4, 3].  Not the reference's search: it only makes
    meaningful bytes (any byte string is a valid block; the op's parity surface starts at the bytes)."""
    blk = _k_sub_blocks(w)
    n, nb = blk.shape[:2]
    s = np.abs(blk).max(-1) / np.float32(4)                          # [n, nb, 2, 4, 2]
    d = (s.reshape(n, nb, -1).max(-1) / np.float32(31)).astype(np.float16)
    df = d.astype(np.float32)[:, :, None, None, None]
    code = np.where(df > 0, np.rint(s / np.where(df > 0, df, 1)), 0).clip(0, 31).astype(np.int32)
    step = df * code
    q = np.where(step[..., None] > 0, np.rint(blk / np.where(step[..., None] > 0, step[..., None], 1)), 0).clip(-4, 3).astype(np.int32) + 4
    out = np.zeros((n, nb, 110), np.uint8)
    hm = np.zeros((n, nb, 2, 16), np.uint8)                          # hmask[16 p + l], bit 4 h + j
    for h in range(2):
        for j in range(4):
            hm |= ((q[:, :, h, j] >> 2) & 1).astype(np.uint8) << (4 * h + j)
    out[..., :32] = hm.reshape(n, nb, 32)
    out[..., 32:96] = _pack_2bit(q.astype(np.uint8))
    sc = (code + 32).transpose(0, 1, 2, 3, 4).reshape(n, nb, 16)      # index 8 h + 2 j + p
    lo, hi = (sc & 15).astype(np.uint8), (sc >> 4).astype(np.uint8)
    out[..., 96:100] = lo[..., 0:4] | (lo[..., 8:12] << 4)
    out[..., 100:104] = lo[..., 4:8] | (lo[..., 12:16] << 4)
    out[..., 104:108] = hi[..., 0:4] | (hi[..., 4:8] << 2) | (hi[..., 8:12] << 4) | (hi[..., 12:16] << 6)
    out[..., 108:110] = d.view(np.uint8).reshape(n, nb, 2)
    return out.reshape(n, nb * 110)


def plain_q2_K_rows(w):
    """fp32 [N, K] -> Q2_K rows by a plain quantizer: sub-block min m = max(0, -min x), scale = (max x + m) / 3, 4-bit
    codes of both against the super-block's largest, q = round((x + dmin m) / (d sc)) in [0, 3].  Not the reference's."""
    blk = _k_sub_blocks(w)
    n, nb = blk.shape[:2]
    mn = np.maximum(0, -blk.min(-1))
    sc = (blk.max(-1) + mn) / np.float32(3)
    d = (sc.reshape(n, nb, -1).max(-1) / np.float32(15)).astype(np.float16)
    dm = (mn.reshape(n, nb, -1).max(-1) / np.float32(15)).astype(np.float16)
    df, dmf = d.astype(np.float32)[:, :, None, None, None], dm.astype(np.float32)[:, :, None, None, None]
    csc = np.where(df > 0, np.rint(sc / np.where(df > 0, df, 1)), 0).clip(0, 15).astype(np.int32)
    cmn = np.where(dmf > 0, np.rint(mn / np.where(dmf > 0, dmf, 1)), 0).clip(0, 15).astype(np.int32)
    step = (df * csc)[..., None]
    q = np.where(step > 0, np.rint((blk + (dmf * cmn)[..., None]) / np.where(step > 0, step, 1)), 0).clip(0, 3).astype(np.uint8)
    out = np.zeros((n, nb, 84), np.uint8)
    out[..., :16] = (csc | (cmn << 4)).reshape(n, nb, 16).astype(np.uint8)
    out[..., 16:80] = _pack_2bit(q)
    out[..., 80:82] = d.view(np.uint8).reshape(n, nb, 2)
    out[..., 82:84] = dm.view(np.uint8).reshape(n, nb, 2)
    return out.reshape(n, nb * 84)


def plain_iq4_xs_rows(w):
    """fp32 [N, K] -> IQ4_XS rows by a plain quantizer: 32-value sub-block scale = max|x| / 127 (signed like the largest
    element), super-block d = largest |scale| / 31, 6-bit codes ls = round(scale / d) + 32, index = nearest code point of
    x / (d (ls - 32)).  Not the reference's search."""
    w = np.ascontiguousarray(w, np.float32)
    n, k = w.shape
    nb = k // 256
    blk = w.reshape(n, nb, 8, 32)
    imax = np.abs(blk).argmax(-1)
    mx = np.take_along_axis(blk, imax[..., None], -1)[..., 0]
    sc = mx / np.float32(-127)
    d = (np.abs(sc).max(-1) / np.float32(31)).astype(np.float16)
    df = d.astype(np.float32)[..., None]
    ls = np.where(df > 0, np.rint(sc / np.where(df > 0, df, 1)), 0).clip(-32, 31).astype(np.int32)
    step = (df * ls)[..., None]
    idx = np.abs(np.where(step != 0, blk / np.where(step != 0, step, 1), 0)[..., None] - IQ4_NL_VALUES).argmin(-1).astype(np.uint8)
    code = (ls + 32).astype(np.uint16)
    out = np.zeros((n, nb, 136), np.uint8)
    out[..., 0:2] = d.view(np.uint8).reshape(n, nb, 2)
    sh = np.zeros((n, nb), np.uint16)
    for ib in range(8):
        sh |= ((code[..., ib] >> 4) & 3) << (2 * ib)
    out[..., 2:4] = sh.view(np.uint8).reshape(n, nb, 2)
    lo = (code & 15).astype(np.uint8)
    out[..., 4:8] = lo[..., 0::2] | (lo[..., 1::2] << 4)
    out[..., 8:] = (idx[..., :16] | (idx[..., 16:] << 4)).reshape(n, nb, 128)
    return out.reshape(n, nb * 136)


def row_size(t, k):
    return (k // BLOCK_ELEMS[t]) * BLOCK_BYTES[t]


def build(force=False):
    """Compile liboracle.so (and oracle/_ref when the reference tree is mounted)."""
    if force or not os.path.exists(ORACLE_SO):
        subprocess.check_call(["make", "-C", HERE, "oracle"] + (["-B"] if force else []))
    if os.path.isdir("/root/reference/cactus") and (force or not os.path.exists(REF_SO)):
        subprocess.check_call(["make", "-C", HERE, "-j8", "ref"])


_vp, _i64, _i32, _f32p = C.c_void_p, C.c_int64, C.c_int, C.POINTER(C.c_float)


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


class Oracle:
    """The restatement.  Arrays in, arrays out; all quantized data travel as uint8 arrays."""

    def __init__(self, path=ORACLE_SO):
        if not os.path.exists(path):
            build()
        self.lib = L = C.CDLL(path)
        L.orc_fp16_to_fp32.restype = C.c_float
        L.orc_fp16_to_fp32.argtypes = [C.c_uint16]
        L.orc_fp32_to_fp16.restype = C.c_uint16
        L.orc_fp32_to_fp16.argtypes = [C.c_float]
        for n in ("q8_0", "q8_K", "q8_1", "q4_0_ref", "q8_0_ref", "q4_K_ref", "q6_K_ref", "q5_0_ref", "q5_K_ref",
                  "q4_1_ref", "q5_1_ref"):
            f = getattr(L, "orc_quantize_row_" + n)
            f.restype = None
            f.argtypes = [_vp, _vp, _i64]
        L.orc_fp32_to_fp16_row.restype = None
        L.orc_fp32_to_fp16_row.argtypes = [_vp, _vp, _i64]
        L.orc_vec_dot_f16.restype = C.c_float
        L.orc_vec_dot_f16.argtypes = [_i64, _vp, _vp]
        L.orc_quantize_rows.restype = C.c_size_t
        L.orc_quantize_rows.argtypes = [_i32, _vp, _vp, _i64, _i64]
        L.orc_dequantize_row.restype = None
        L.orc_dequantize_row.argtypes = [_i32, _vp, _vp, _i64]
        for n in ("q4_0_q8_0", "q8_0_q8_0", "q6_K_q8_K", "q5_0_q8_0", "iq4_nl_q8_0", "q4_1_q8_1", "q5_1_q8_1", "q3_K_q8_K", "iq4_xs_q8_K"):
            f = getattr(L, "orc_vec_dot_" + n)
            f.restype = C.c_float
            f.argtypes = [_i64, _vp, _vp, _vp]
        for n in ("q4_K_q8_K", "q5_K_q8_K", "q2_K_q8_K"):
            f = getattr(L, "orc_vec_dot_" + n)
            f.restype = C.c_float
            f.argtypes = [_i64, _vp, _vp, _vp, _vp]
        L.orc_vec_dot_exact.restype = C.c_double
        L.orc_vec_dot_exact.argtypes = [_i32, _i64, _vp, _vp, _vp]
        L.orc_mul_mat.restype = None
        L.orc_mul_mat.argtypes = [_i32, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _i32]
        L.orc_rms_norm_f32.restype = None
        L.orc_rms_norm_f32.argtypes = [_vp, _vp, _i64, _i64, C.c_float]
        L.orc_silu_f32.restype = None
        L.orc_silu_f32.argtypes = [_vp, _vp, _i64, _i64]
        L.orc_gelu_f32.restype = None
        L.orc_gelu_f32.argtypes = [_vp, _vp, _i64]
        L.orc_gelu_table.restype = None
        L.orc_gelu_table.argtypes = [_vp]
        L.orc_soft_max_f32.restype = None
        L.orc_soft_max_f32.argtypes = [_vp, _vp, _i32, _i64, _i64, _i64, _i64, C.c_float, C.c_float, _vp]
        L.orc_rope_f32.restype = None
        L.orc_rope_f32.argtypes = [_vp, _vp, _vp, _i64, _i64, _i64, _i32, _i32, _i32] + [C.c_float] * 6 + [_vp]
        L.orc_mul_mat_id.restype = _i32
        L.orc_mul_mat_id.argtypes = [_i32, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _i64, _i64, _vp, _vp, _i32]

    # -- scalars
    def h2f(self, h):
        return self.lib.orc_fp16_to_fp32(int(h))

    def f2h(self, f):
        return self.lib.orc_fp32_to_fp16(float(np.float32(f)))

    # -- quantizers
    def quantize_activation(self, act_type, x):
        """x [..., K] fp32 -> uint8 [..., row_size]; act_type is Q8_0 (AVX2 semantics) or Q8_K."""
        x = _f32(x)
        k = x.shape[-1]
        rows = x.reshape(-1, k)
        out = np.zeros((rows.shape[0], row_size(act_type, k)), np.uint8)
        fn = {Q8_0: self.lib.orc_quantize_row_q8_0, Q8_K: self.lib.orc_quantize_row_q8_K,
              Q8_1: self.lib.orc_quantize_row_q8_1, F16: self.lib.orc_fp32_to_fp16_row}[act_type]
        for r in range(rows.shape[0]):
            fn(_ptr(rows[r]), _ptr(out[r]), k)
        return out.reshape(x.shape[:-1] + (out.shape[1],))

    def quantize_q8_0_ref(self, x):
        x = _f32(x)
        out = np.zeros(row_size(Q8_0, x.size), np.uint8)
        self.lib.orc_quantize_row_q8_0_ref(_ptr(x), _ptr(out), x.size)
        return out

    def quantize_weights(self, wtype, w):
        """w [N, K] fp32 -> uint8 [N, row_size] with the reference's *_ref weight quantizer.
        IQ4_NL: a plain nearest-code-point quantizer (NOT the reference's search; it only makes meaningful bytes,
        the op's parity surface starts at the bytes)."""
        w = _f32(w)
        n, k = w.shape
        if wtype == IQ4_NL:
            return nearest_iq4_nl_rows(w)
        if wtype == Q3_K:
            return plain_q3_K_rows(w)
        if wtype == Q2_K:
            return plain_q2_K_rows(w)
        if wtype == IQ4_XS:
            return plain_iq4_xs_rows(w)
        out = np.zeros((n, row_size(wtype, k)), np.uint8)
        got = self.lib.orc_quantize_rows(wtype, _ptr(w), _ptr(out), n, k)
        assert got == out.size
        return out

    def dequantize(self, t, q, k):
        q = np.ascontiguousarray(q, np.uint8)
        rows = q.reshape(-1, row_size(t, k))
        out = np.zeros((rows.shape[0], k), np.float32)
        for r in range(rows.shape[0]):
            self.lib.orc_dequantize_row(t, _ptr(rows[r]), _ptr(out[r]), k)
        return out.reshape(q.shape[:-1] + (k,))

    # -- dots
    def vec_dot(self, wtype, k, wrow, arow, want_sums=False):
        wrow = np.ascontiguousarray(wrow, np.uint8)
        arow = np.ascontiguousarray(arow, np.uint8)
        nb = k // BLOCK_ELEMS[wtype]
        isum = np.zeros(nb, np.int32)
        imin = np.zeros(nb, np.int32)
        if wtype == Q4_0:
            v = self.lib.orc_vec_dot_q4_0_q8_0(k, _ptr(wrow), _ptr(arow), _ptr(isum))
        elif wtype == Q8_0:
            v = self.lib.orc_vec_dot_q8_0_q8_0(k, _ptr(wrow), _ptr(arow), _ptr(isum))
        elif wtype == Q4_K:
            v = self.lib.orc_vec_dot_q4_K_q8_K(k, _ptr(wrow), _ptr(arow), _ptr(isum), _ptr(imin))
        elif wtype == Q6_K:
            v = self.lib.orc_vec_dot_q6_K_q8_K(k, _ptr(wrow), _ptr(arow), _ptr(isum))
        elif wtype == Q5_0:
            v = self.lib.orc_vec_dot_q5_0_q8_0(k, _ptr(wrow), _ptr(arow), _ptr(isum))
        elif wtype == IQ4_NL:
            v = self.lib.orc_vec_dot_iq4_nl_q8_0(k, _ptr(wrow), _ptr(arow), _ptr(isum))
        elif wtype == Q5_K:
            v = self.lib.orc_vec_dot_q5_K_q8_K(k, _ptr(wrow), _ptr(arow), _ptr(isum), _ptr(imin))
        elif wtype == F16:
            v = self.lib.orc_vec_dot_f16(k, _ptr(wrow), _ptr(arow))
        elif wtype == Q2_K:
            v = self.lib.orc_vec_dot_q2_K_q8_K(k, _ptr(wrow), _ptr(arow), _ptr(isum), _ptr(imin))
        elif wtype == Q3_K:
            v = self.lib.orc_vec_dot_q3_K_q8_K(k, _ptr(wrow), _ptr(arow), _ptr(isum))
        elif wtype == IQ4_XS:
            v = self.lib.orc_vec_dot_iq4_xs_q8_K(k, _ptr(wrow), _ptr(arow), _ptr(isum))
        elif wtype == Q4_1:
            v = self.lib.orc_vec_dot_q4_1_q8_1(k, _ptr(wrow), _ptr(arow), _ptr(isum))
        elif wtype == Q5_1:
            v = self.lib.orc_vec_dot_q5_1_q8_1(k, _ptr(wrow), _ptr(arow), _ptr(isum))
        else:
            raise ValueError(wtype)
        v = np.float32(v)
        return (v, isum, imin) if want_sums else v

    def vec_dot_exact(self, wtype, k, wrow, arow):
        wrow = np.ascontiguousarray(wrow, np.uint8)
        arow = np.ascontiguousarray(arow, np.uint8)
        sa = C.c_double(0)
        v = self.lib.orc_vec_dot_exact(wtype, k, _ptr(wrow), _ptr(arow), C.byref(sa))
        return v, sa.value

    def mul_mat(self, wtype, W, x, nthreads=1, want=()):
        """W uint8 [N, row_size(wtype,K)], x fp32 [n, K] -> y fp32 [n, N].
        want may name 'wdata' (quantized activations) and/or 'sum_abs' (tolerance yardstick)."""
        W = np.ascontiguousarray(W, np.uint8)
        x = _f32(x)
        n, k = x.shape
        N = W.shape[0]
        assert W.shape[1] == row_size(wtype, k)
        y = np.zeros((n, N), np.float32)
        wd = np.zeros((n, row_size(VEC_DOT_TYPE[wtype], k)), np.uint8) if "wdata" in want else None
        sa = np.zeros((n, N), np.float64) if "sum_abs" in want else None
        self.lib.orc_mul_mat(wtype, k, N, n, _ptr(W), _ptr(x), _ptr(y), _ptr(wd), _ptr(sa), nthreads)
        out = {"y": y}
        if wd is not None:
            out["wdata"] = wd
        if sa is not None:
            out["sum_abs"] = sa
        return out

    def mul_mat_f16_batched(self, W, x, want=()):
        """LM_GGML_OP_MUL_MAT with a batched F16 src0 (ggml-cpu/ggml-cpu.c:1177-1456: src0's batch = src1's batch / r2):
        W fp16 [ne02, N, K] (any view), x fp32 [ne12, n, K] (any view) -> y fp32 [ne12, n, N]."""
        ne02, N, K = W.shape
        ne12, n, _ = x.shape
        assert ne12 % ne02 == 0
        r2 = ne12 // ne02
        y = np.zeros((ne12, n, N), np.float32)
        sa = np.zeros((ne12, n, N), np.float64)
        for b in range(ne12):
            wb = np.ascontiguousarray(W[b // r2]).view(np.uint8).reshape(N, 2 * K)
            o = self.mul_mat(F16, wb, np.ascontiguousarray(x[b]), want=("sum_abs",))
            y[b], sa[b] = o["y"], o["sum_abs"]
        return {"y": y, "sum_abs": sa} if "sum_abs" in want else {"y": y}

    def get_rows(self, t, table, nc, ids):
        """LM_GGML_OP_GET_ROWS (ggml-cpu/ops.cpp:4236-4453): the rows ids of a table of type t, dequantized to fp32 with the
        type's dequantize_row (F32: copied).  table: uint8 [ne01, row_size] for block types and F16, fp32 [ne01, nc] for F32."""
        ids = np.asarray(ids, np.int64)
        if t == F32:
            return np.ascontiguousarray(np.asarray(table, np.float32)[ids])
        tb = np.ascontiguousarray(table).view(np.uint8).reshape(len(table), -1)
        return self.dequantize(t, tb[ids], nc)

    def rms_norm(self, x, eps):
        """LM_GGML_OP_RMS_NORM over the rows of x fp32 [n, ne0]."""
        x = _f32(x)
        y = np.empty_like(x)
        self.lib.orc_rms_norm_f32(_ptr(x), _ptr(y), x.shape[0], x.shape[1], eps)
        return y

    def silu(self, x):
        """LM_GGML_UNARY_OP_SILU over the rows of x fp32 [n, ne0] (AVX2 build of the reference)."""
        x = _f32(x)
        y = np.empty_like(x)
        self.lib.orc_silu_f32(_ptr(x), _ptr(y), x.shape[0], x.shape[1])
        return y

    def gelu(self, x):
        """LM_GGML_UNARY_OP_GELU over x fp32 (any shape): the reference's fp16-table form."""
        x = _f32(x)
        y = np.empty_like(x)
        self.lib.orc_gelu_f32(_ptr(x), _ptr(y), x.size)
        return y

    def gelu_table(self):
        """The 65536 fp16 entries lm_ggml_cpu_init computes (as uint16 bit patterns)."""
        t = np.empty(65536, np.uint16)
        self.lib.orc_gelu_table(_ptr(t))
        return t

    @staticmethod
    def scale(x, v):
        """LM_GGML_OP_SCALE (lm_ggml_compute_forward_scale_f32, reference ggml-cpu/ops.cpp:3930-3968): one fp32 multiply
        per element (lm_ggml_vec_scale_f32, ggml-cpu/vec.h:264-293)."""
        return _f32(x) * np.float32(v)

    def soft_max(self, x, mask=None, scale=1.0, max_bias=0.0):
        """LM_GGML_OP_SOFT_MAX (lm_ggml_soft_max_ext): x fp32 [n_head, ne01, ne00]; mask fp32 or fp16 [>= ne01, ne00] or
        None, shared by the heads."""
        x = _f32(x)
        n_head, ne01, ne00 = x.shape
        y = np.empty_like(x)
        if mask is not None:
            mask = np.ascontiguousarray(mask)
            assert mask.dtype in (np.float32, np.float16) and mask.shape[1] == ne00 and mask.shape[0] >= ne01
        self.lib.orc_soft_max_f32(_ptr(x), _ptr(mask) if mask is not None else None,
                                  int(mask is not None and mask.dtype == np.float16), ne00, ne01, n_head,
                                  n_head * ne01, scale, max_bias, _ptr(y))
        return y

    def rope(self, x, pos, n_dims, mode, freq_factors=None, n_ctx_orig=4096, freq_base=10000.0, freq_scale=1.0,
             ext_factor=0.0, attn_factor=1.0, beta_fast=32.0, beta_slow=1.0):
        """LM_GGML_OP_ROPE (lm_ggml_rope_ext), text modes 0 and 2 (NEOX): x fp32 [n_tokens, n_head, ne0], pos int32
        [n_tokens], freq_factors fp32 [n_dims / 2] or None."""
        x = _f32(x)
        pos = np.ascontiguousarray(pos, np.int32)
        ne2, ne1, ne0 = x.shape
        assert pos.shape == (ne2,) and n_dims % 2 == 0 and n_dims <= ne0 and mode in (0, 2)
        ff = _f32(freq_factors) if freq_factors is not None else None
        y = np.empty_like(x)
        self.lib.orc_rope_f32(_ptr(x), _ptr(pos), _ptr(ff) if ff is not None else None, ne0, ne1, ne2, n_dims, mode,
                              n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow, _ptr(y))
        return y

    @staticmethod
    def cpy(x, dst_dtype):
        """LM_GGML_OP_CPY / CONT between F32 and F16 (reference ggml-cpu/ops.cpp lm_ggml_compute_forward_dup): element i of
        the source, in the source's logical order, becomes element i of the destination; F32 -> F16 rounds to nearest
        even (the F16C conversion of LM_GGML_FP32_TO_FP16), F16 -> F32 is exact.  x is a numpy array (or view) in the
        source's logical order; the result is the destination's contents in its logical order."""
        return np.ascontiguousarray(x).astype(dst_dtype)

    def mul_mat_id(self, wtype, W, x, ids, nthreads=1, want=()):
        """LM_GGML_OP_MUL_MAT_ID: W uint8 [n_as, N, row_size], x fp32 [n_tokens, ne11, K] (ne11 = 1 or n_used),
        ids int32 [n_tokens, n_used] -> y fp32 [n_tokens, n_used, N]."""
        W = np.ascontiguousarray(W, np.uint8)
        x = _f32(x)
        ids = np.ascontiguousarray(ids, np.int32)
        n_tokens, ne11, k = x.shape
        n_as, N = W.shape[0], W.shape[1]
        n_used = ids.shape[1]
        assert W.shape[2] == row_size(wtype, k) and ids.shape[0] == n_tokens
        y = np.zeros((n_tokens, n_used, N), np.float32)
        sa = np.zeros((n_tokens, n_used, N), np.float64) if "sum_abs" in want else None
        rc = self.lib.orc_mul_mat_id(wtype, k, N, n_as, _ptr(W), _ptr(x), ne11, _ptr(ids), n_used, n_tokens, _ptr(y),
                                     _ptr(sa), nthreads)
        if rc:
            raise ValueError("orc_mul_mat_id: %d" % rc)
        out = {"y": y}
        if sa is not None:
            out["sum_abs"] = sa
        return out


class _InitParams(C.Structure):
    _fields_ = [("mem_size", C.c_size_t), ("mem_buffer", C.c_void_p), ("no_alloc", C.c_bool)]


class Reference:
    """The reference's own compiled code (oracle/_ref/libggml_ref.so), when present.

    Exposes the hot-path functions directly and the CPU backend's LM_GGML_OP_MUL_MAT through a one-node graph
    with a persistent threadpool (reference ggml-cpu/ggml-cpu.c:3079, ggml-cpu/ggml-cpu.cpp:238-248)."""

    @staticmethod
    def available():
        return os.path.exists(REF_SO)

    def __init__(self, path=REF_SO, mode=C.RTLD_GLOBAL):
        self.lib = L = C.CDLL(path, mode=mode)
        L.lm_ggml_cpu_init.restype = None
        L.lm_ggml_cpu_init()
        # fp16 table is filled by the first lm_ggml_init (reference ggml.c:1418-1431)
        L.lm_ggml_init.restype = _vp
        L.lm_ggml_init.argtypes = [_InitParams]
        L.lm_ggml_free.argtypes = [_vp]
        ctx = L.lm_ggml_init(_InitParams(1 << 20, None, False))
        L.lm_ggml_free(ctx)
        for n in ("quantize_row_q8_0", "quantize_row_q8_K", "quantize_row_q4_0_ref", "quantize_row_q8_0_ref",
                  "quantize_row_q4_K_ref", "quantize_row_q6_K_ref", "quantize_row_q8_K_ref",
                  "quantize_row_q5_0_ref", "quantize_row_q5_K_ref", "quantize_row_iq4_nl_ref",
                  "quantize_row_q4_1_ref", "quantize_row_q5_1_ref", "quantize_row_q8_1",
                  "quantize_row_q2_K_ref", "quantize_row_q3_K_ref", "quantize_row_iq4_xs_ref",
                  "lm_ggml_fp32_to_fp16_row", "lm_ggml_cpu_fp32_to_fp16", "lm_ggml_fp16_to_fp32_row"):
            f = getattr(L, n)
            f.restype = None
            f.argtypes = [_vp, _vp, _i64]
        for n in ("q4_0", "q8_0", "q4_K", "q6_K", "q8_K", "q5_0", "q5_K", "iq4_nl", "q4_1", "q5_1", "q2_K", "q3_K", "iq4_xs"):
            f = getattr(L, "dequantize_row_" + n)
            f.restype = None
            f.argtypes = [_vp, _vp, _i64]
        for n in ("q4_0_q8_0", "q8_0_q8_0", "q4_K_q8_K", "q6_K_q8_K", "q5_0_q8_0", "q5_K_q8_K", "iq4_nl_q8_0",
                  "q4_1_q8_1", "q5_1_q8_1", "f16", "q2_K_q8_K", "q3_K_q8_K", "iq4_xs_q8_K"):
            f = getattr(L, "lm_ggml_vec_dot_" + n)
            f.restype = None
            f.argtypes = [C.c_int, _vp, C.c_size_t, _vp, C.c_size_t, _vp, C.c_size_t, C.c_int]
        L.lm_ggml_quantize_chunk.restype = C.c_size_t
        L.lm_ggml_quantize_chunk.argtypes = [_i32, _vp, _vp, _i64, _i64, _i64, _vp]
        # graph / backend API (opaque pointers)
        L.lm_ggml_new_tensor_2d.restype = _vp
        L.lm_ggml_new_tensor_2d.argtypes = [_vp, _i32, _i64, _i64]
        L.lm_ggml_mul_mat.restype = _vp
        L.lm_ggml_mul_mat.argtypes = [_vp, _vp, _vp]
        L.lm_ggml_new_tensor_3d.restype = _vp
        L.lm_ggml_new_tensor_3d.argtypes = [_vp, _i32, _i64, _i64, _i64]
        for n_ in ("lm_ggml_add", "lm_ggml_mul"):
            getattr(L, n_).restype = _vp
            getattr(L, n_).argtypes = [_vp, _vp, _vp]
        L.lm_ggml_silu.restype = _vp
        L.lm_ggml_silu.argtypes = [_vp, _vp]
        L.lm_ggml_rms_norm.restype = _vp
        L.lm_ggml_rms_norm.argtypes = [_vp, _vp, C.c_float]
        L.lm_ggml_mul_mat_id.restype = _vp
        L.lm_ggml_mul_mat_id.argtypes = [_vp, _vp, _vp, _vp]
        L.lm_ggml_new_tensor_1d.restype = _vp
        L.lm_ggml_new_tensor_1d.argtypes = [_vp, _i32, _i64]
        L.lm_ggml_new_tensor_4d.restype = _vp
        L.lm_ggml_new_tensor_4d.argtypes = [_vp, _i32, _i64, _i64, _i64, _i64]
        L.lm_ggml_soft_max_ext.restype = _vp
        L.lm_ggml_soft_max_ext.argtypes = [_vp, _vp, _vp, C.c_float, C.c_float]
        L.lm_ggml_rope_ext.restype = _vp
        L.lm_ggml_rope_ext.argtypes = [_vp, _vp, _vp, _vp, _i32, _i32, _i32] + [C.c_float] * 6
        for n_ in ("lm_ggml_cpy",):
            getattr(L, n_).restype = _vp
            getattr(L, n_).argtypes = [_vp, _vp, _vp]
        for n_ in ("lm_ggml_cont", "lm_ggml_transpose"):
            getattr(L, n_).restype = _vp
            getattr(L, n_).argtypes = [_vp, _vp]
        L.lm_ggml_permute.restype = _vp
        L.lm_ggml_permute.argtypes = [_vp, _vp, _i32, _i32, _i32, _i32]
        L.lm_ggml_view_2d.restype = _vp
        L.lm_ggml_view_2d.argtypes = [_vp, _vp, _i64, _i64, C.c_size_t, C.c_size_t]
        L.lm_ggml_new_graph.restype = _vp
        L.lm_ggml_new_graph.argtypes = [_vp]
        L.lm_ggml_build_forward_expand.restype = None
        L.lm_ggml_build_forward_expand.argtypes = [_vp, _vp]
        L.lm_ggml_backend_cpu_init.restype = _vp
        L.lm_ggml_backend_cpu_set_n_threads.argtypes = [_vp, _i32]
        L.lm_ggml_backend_cpu_set_threadpool.argtypes = [_vp, _vp]
        L.lm_ggml_backend_alloc_ctx_tensors.restype = _vp
        L.lm_ggml_backend_alloc_ctx_tensors.argtypes = [_vp, _vp]
        L.lm_ggml_backend_tensor_set.argtypes = [_vp, _vp, C.c_size_t, C.c_size_t]
        L.lm_ggml_backend_tensor_get.argtypes = [_vp, _vp, C.c_size_t, C.c_size_t]
        L.lm_ggml_backend_graph_compute.restype = _i32
        L.lm_ggml_backend_graph_compute.argtypes = [_vp, _vp]
        L.lm_ggml_backend_buffer_free.argtypes = [_vp]
        L.lm_ggml_backend_free.argtypes = [_vp]
        L.lm_ggml_tensor_overhead.restype = C.c_size_t
        L.lm_ggml_graph_overhead.restype = C.c_size_t
        L.lm_ggml_threadpool_new.restype = _vp
        L.lm_ggml_threadpool_new.argtypes = [_vp]
        L.lm_ggml_threadpool_free.argtypes = [_vp]
        L.lm_ggml_threadpool_params_init.argtypes = [_vp, _i32]

    _ACT = {Q8_0: "quantize_row_q8_0", Q8_K: "quantize_row_q8_K", Q8_1: "quantize_row_q8_1",
            F16: "lm_ggml_cpu_fp32_to_fp16"}
    _WQ = {Q4_0: "quantize_row_q4_0_ref", Q8_0: "quantize_row_q8_0_ref",
           Q4_K: "quantize_row_q4_K_ref", Q6_K: "quantize_row_q6_K_ref",
           Q5_0: "quantize_row_q5_0_ref", Q5_K: "quantize_row_q5_K_ref", IQ4_NL: "quantize_row_iq4_nl_ref",
           Q4_1: "quantize_row_q4_1_ref", Q5_1: "quantize_row_q5_1_ref", F16: "lm_ggml_fp32_to_fp16_row",
           Q2_K: "quantize_row_q2_K_ref", Q3_K: "quantize_row_q3_K_ref", IQ4_XS: "quantize_row_iq4_xs_ref"}
    _DOT = {Q4_0: "lm_ggml_vec_dot_q4_0_q8_0", Q8_0: "lm_ggml_vec_dot_q8_0_q8_0",
            Q4_K: "lm_ggml_vec_dot_q4_K_q8_K", Q6_K: "lm_ggml_vec_dot_q6_K_q8_K",
            Q5_0: "lm_ggml_vec_dot_q5_0_q8_0", Q5_K: "lm_ggml_vec_dot_q5_K_q8_K", IQ4_NL: "lm_ggml_vec_dot_iq4_nl_q8_0",
            Q4_1: "lm_ggml_vec_dot_q4_1_q8_1", Q5_1: "lm_ggml_vec_dot_q5_1_q8_1", F16: "lm_ggml_vec_dot_f16",
            Q2_K: "lm_ggml_vec_dot_q2_K_q8_K", Q3_K: "lm_ggml_vec_dot_q3_K_q8_K", IQ4_XS: "lm_ggml_vec_dot_iq4_xs_q8_K"}

    def quantize_activation(self, act_type, x):
        x = _f32(x)
        k = x.shape[-1]
        rows = x.reshape(-1, k)
        # bsums of an all-zero Q8_K block are left unwritten by the reference: start from zeros
        out = np.zeros((rows.shape[0], row_size(act_type, k)), np.uint8)
        fn = getattr(self.lib, self._ACT[act_type])
        for r in range(rows.shape[0]):
            fn(_ptr(rows[r]), _ptr(out[r]), k)
        return out.reshape(x.shape[:-1] + (out.shape[1],))

    def quantize_q8_0_ref(self, x):
        x = _f32(x)
        out = np.zeros(row_size(Q8_0, x.size), np.uint8)
        self.lib.quantize_row_q8_0_ref(_ptr(x), _ptr(out), x.size)
        return out

    def quantize_weights(self, wtype, w):
        w = _f32(w)
        n, k = w.shape
        out = np.zeros((n, row_size(wtype, k)), np.uint8)
        fn = getattr(self.lib, self._WQ[wtype])
        for r in range(n):
            fn(_ptr(w[r]), _ptr(out[r]), k)
        return out

    def dequantize(self, t, q, k):
        q = np.ascontiguousarray(q, np.uint8)
        rows = q.reshape(-1, row_size(t, k))
        out = np.zeros((rows.shape[0], k), np.float32)
        fn = getattr(self.lib, "lm_ggml_fp16_to_fp32_row" if t == F16 else "dequantize_row_" + TYPE_NAMES[t])
        for r in range(rows.shape[0]):
            fn(_ptr(rows[r]), _ptr(out[r]), k)
        return out.reshape(q.shape[:-1] + (k,))

    def vec_dot(self, wtype, k, wrow, arow):
        wrow = np.ascontiguousarray(wrow, np.uint8)
        arow = np.ascontiguousarray(arow, np.uint8)
        s = C.c_float(0)
        getattr(self.lib, self._DOT[wtype])(k, C.byref(s), 0, _ptr(wrow), 0, _ptr(arow), 0, 1)
        return np.float32(s.value)

    def mul_mat_graph(self, wtype, W, x, nthreads=1, repeat=1):
        """LM_GGML_OP_MUL_MAT on the reference CPU backend.  Returns (y [n,N], seconds per compute: list)."""
        import time
        L = self.lib
        W = np.ascontiguousarray(W, np.uint8)
        x = _f32(x)
        n, k = x.shape
        N = W.shape[0]
        ctx = L.lm_ggml_init(_InitParams(L.lm_ggml_tensor_overhead() * 8 + L.lm_ggml_graph_overhead() + 4096,
                                         None, True))
        a = L.lm_ggml_new_tensor_2d(ctx, wtype, k, N)
        b = L.lm_ggml_new_tensor_2d(ctx, F32, k, n)
        c = L.lm_ggml_mul_mat(ctx, a, b)
        g = L.lm_ggml_new_graph(ctx)
        L.lm_ggml_build_forward_expand(g, c)
        be = L.lm_ggml_backend_cpu_init()
        L.lm_ggml_backend_cpu_set_n_threads(be, nthreads)
        tpp = (C.c_char * 1024)()          # struct lm_ggml_threadpool_params (opaque, generously sized)
        L.lm_ggml_threadpool_params_init(C.byref(tpp), nthreads)
        tp = L.lm_ggml_threadpool_new(C.byref(tpp))
        L.lm_ggml_backend_cpu_set_threadpool(be, tp)
        buf = L.lm_ggml_backend_alloc_ctx_tensors(ctx, be)
        L.lm_ggml_backend_tensor_set(a, _ptr(W), 0, W.size)
        L.lm_ggml_backend_tensor_set(b, _ptr(x), 0, x.size * 4)
        times = []
        for _ in range(repeat):
            t0 = time.perf_counter()
            st = L.lm_ggml_backend_graph_compute(be, g)
            times.append(time.perf_counter() - t0)
            assert st == 0
        y = np.zeros((n, N), np.float32)
        L.lm_ggml_backend_tensor_get(c, _ptr(y), 0, y.size * 4)
        L.lm_ggml_backend_buffer_free(buf)
        L.lm_ggml_backend_free(be)
        L.lm_ggml_threadpool_free(tp)
        L.lm_ggml_free(ctx)
        return y, times

    def op_graph(self, op, x, b=None, eps=0.0, nthreads=1):
        """One element-wise node on the reference CPU backend: op in {"rms_norm", "silu", "add", "mul"}; x fp32
        [n, ne0]; b fp32 [n, ne0] or [1, ne0] for the binary ops."""
        L = self.lib
        x = _f32(x)
        n, ne0 = x.shape
        ctx = L.lm_ggml_init(_InitParams(L.lm_ggml_tensor_overhead() * 8 + L.lm_ggml_graph_overhead() + 4096,
                                         None, True))
        tx = L.lm_ggml_new_tensor_2d(ctx, F32, ne0, n)
        tb = None
        if op == "rms_norm":
            c = L.lm_ggml_rms_norm(ctx, tx, eps)
        elif op == "silu":
            c = L.lm_ggml_silu(ctx, tx)
        else:
            b = _f32(b)
            tb = L.lm_ggml_new_tensor_2d(ctx, F32, ne0, b.shape[0])
            c = (L.lm_ggml_add if op == "add" else L.lm_ggml_mul)(ctx, tx, tb)
        g = L.lm_ggml_new_graph(ctx)
        L.lm_ggml_build_forward_expand(g, c)
        be = L.lm_ggml_backend_cpu_init()
        L.lm_ggml_backend_cpu_set_n_threads(be, nthreads)
        buf = L.lm_ggml_backend_alloc_ctx_tensors(ctx, be)
        L.lm_ggml_backend_tensor_set(tx, _ptr(x), 0, x.size * 4)
        if tb is not None:
            L.lm_ggml_backend_tensor_set(tb, _ptr(b), 0, b.size * 4)
        assert L.lm_ggml_backend_graph_compute(be, g) == 0
        y = np.zeros((n, ne0), np.float32)
        L.lm_ggml_backend_tensor_get(c, _ptr(y), 0, y.size * 4)
        L.lm_ggml_backend_buffer_free(buf)
        L.lm_ggml_backend_free(be)
        L.lm_ggml_free(ctx)
        return y

    def _run_graph(self, build, inputs, out_shape, out_dtype, nthreads=1, n_tensors=16):
        """Builds a graph with build(ctx) -> (result node, {name: tensor}), uploads inputs[name], computes on the reference
        CPU backend and returns the result node's bytes as an array of out_shape / out_dtype."""
        L = self.lib
        ctx = L.lm_ggml_init(_InitParams(L.lm_ggml_tensor_overhead() * n_tensors + L.lm_ggml_graph_overhead() + 4096,
                                         None, True))
        c, tensors = build(ctx)
        g = L.lm_ggml_new_graph(ctx)
        L.lm_ggml_build_forward_expand(g, c)
        be = L.lm_ggml_backend_cpu_init()
        L.lm_ggml_backend_cpu_set_n_threads(be, nthreads)
        buf = L.lm_ggml_backend_alloc_ctx_tensors(ctx, be)
        for name, t in tensors.items():
            a = np.ascontiguousarray(inputs[name])
            L.lm_ggml_backend_tensor_set(t, _ptr(a), 0, a.nbytes)
        assert L.lm_ggml_backend_graph_compute(be, g) == 0
        y = np.zeros(out_shape, out_dtype)
        L.lm_ggml_backend_tensor_get(c, _ptr(y), 0, y.nbytes)
        L.lm_ggml_backend_buffer_free(buf)
        L.lm_ggml_backend_free(be)
        L.lm_ggml_free(ctx)
        return y

    def unary_graph(self, name, x, nthreads=1):
        """lm_ggml_gelu / lm_ggml_silu (name) on the reference CPU backend: x fp32 [n, ne0]."""
        L = self.lib
        x = _f32(x)
        fn = getattr(L, "lm_ggml_" + name)
        fn.restype = _vp
        fn.argtypes = [_vp, _vp]

        def build(ctx):
            tx = L.lm_ggml_new_tensor_2d(ctx, F32, x.shape[1], x.shape[0])
            return fn(ctx, tx), {"x": tx}
        return self._run_graph(build, {"x": x}, x.shape, np.float32, nthreads)

    def scale_graph(self, x, v, nthreads=1):
        """lm_ggml_scale on the reference CPU backend: x fp32 [n, ne0]."""
        L = self.lib
        x = _f32(x)
        L.lm_ggml_scale.restype = _vp
        L.lm_ggml_scale.argtypes = [_vp, _vp, C.c_float]

        def build(ctx):
            tx = L.lm_ggml_new_tensor_2d(ctx, F32, x.shape[1], x.shape[0])
            return L.lm_ggml_scale(ctx, tx, v), {"x": tx}
        return self._run_graph(build, {"x": x}, x.shape, np.float32, nthreads)

    def soft_max_graph(self, x, mask=None, scale=1.0, max_bias=0.0, nthreads=1):
        """lm_ggml_soft_max_ext on the reference CPU backend: x fp32 [n_head, ne01, ne00], mask fp32 / fp16 [>= ne01, ne00]."""
        L = self.lib
        x = _f32(x)
        n_head, ne01, ne00 = x.shape
        F16 = 1

        def build(ctx):
            tx = L.lm_ggml_new_tensor_3d(ctx, F32, ne00, ne01, n_head)
            ts = {"x": tx}
            tm = None
            if mask is not None:
                tm = L.lm_ggml_new_tensor_2d(ctx, F16 if mask.dtype == np.float16 else F32, ne00, mask.shape[0])
                ts["mask"] = tm
            return L.lm_ggml_soft_max_ext(ctx, tx, tm, scale, max_bias), ts
        return self._run_graph(build, {"x": x, "mask": mask}, x.shape, np.float32, nthreads)

    def rope_graph(self, x, pos, n_dims, mode, freq_factors=None, n_ctx_orig=4096, freq_base=10000.0, freq_scale=1.0,
                   ext_factor=0.0, attn_factor=1.0, beta_fast=32.0, beta_slow=1.0, nthreads=1):
        """lm_ggml_rope_ext on the reference CPU backend: x fp32 [n_tokens, n_head, ne0], pos int32 [n_tokens]."""
        L = self.lib
        x = _f32(x)
        ne2, ne1, ne0 = x.shape
        I32 = 26

        def build(ctx):
            tx = L.lm_ggml_new_tensor_3d(ctx, F32, ne0, ne1, ne2)
            tp = L.lm_ggml_new_tensor_1d(ctx, I32, ne2)
            ts = {"x": tx, "pos": tp}
            tf = None
            if freq_factors is not None:
                tf = L.lm_ggml_new_tensor_1d(ctx, F32, len(freq_factors))
                ts["ff"] = tf
            return L.lm_ggml_rope_ext(ctx, tx, tp, tf, n_dims, mode, n_ctx_orig, freq_base, freq_scale, ext_factor,
                                      attn_factor, beta_fast, beta_slow), ts
        return self._run_graph(build, {"x": x, "pos": np.ascontiguousarray(pos, np.int32),
                                       "ff": _f32(freq_factors) if freq_factors is not None else None},
                               x.shape, np.float32, nthreads)

    def cpy_graph(self, x, dst_dtype, kind, nthreads=1):
        """lm_ggml_cpy / lm_ggml_cont on the reference CPU backend.  x [ne1, ne0] fp32 or fp16.  kind:
          "flat"       contiguous source into a 1-D destination of dst_dtype (the K-cache store);
          "transpose"  the transposed source into a [ne0, ne1] destination (the transposed V-cache store);
          "cont"       lm_ggml_cont of the transposed source (same type).
        Returns the destination in its logical order."""
        L = self.lib
        x = np.ascontiguousarray(x)
        ne1, ne0 = x.shape
        tt = {np.dtype(np.float32): F32, np.dtype(np.float16): 1}
        st, dt = tt[x.dtype], tt[np.dtype(dst_dtype)]

        def build(ctx):
            tx = L.lm_ggml_new_tensor_2d(ctx, st, ne0, ne1)
            if kind == "flat":
                return L.lm_ggml_cpy(ctx, tx, L.lm_ggml_new_tensor_1d(ctx, dt, ne0 * ne1)), {"x": tx}
            if kind == "transpose":
                return L.lm_ggml_cpy(ctx, L.lm_ggml_transpose(ctx, tx), L.lm_ggml_new_tensor_2d(ctx, dt, ne1, ne0)), {"x": tx}
            return L.lm_ggml_cont(ctx, L.lm_ggml_transpose(ctx, tx)), {"x": tx}
        shape = (ne0 * ne1,) if kind == "flat" else (ne0, ne1)
        return self._run_graph(build, {"x": x}, shape, np.dtype(dst_dtype) if kind != "cont" else x.dtype, nthreads)

    def attention_matmul_graphs(self, k_cache, vt_cache, q, p, nthreads=1):
        """The two attention matmuls as the reference builds them (llama-graph.cpp:1069-1071, 1120, 1154):
        k_cache fp16 [n_kv, n_head_kv, hd] and q fp32 [n_tokens, n_head, hd], both permuted (0, 2, 1, 3) -> kq fp32
        [n_head, n_tokens, n_kv]; vt_cache fp16 [hd, n_head_kv, n_kv] (the transposed V cache: positions fastest)
        permuted likewise and p fp32 [n_head, n_tokens, n_kv] -> kqv fp32 [n_head, n_tokens, hd]."""
        L = self.lib
        n_kv, n_head_kv, hd = k_cache.shape
        n_tokens, n_head, _ = q.shape
        F16_ = 1

        def build_kq(ctx):
            tk = L.lm_ggml_new_tensor_3d(ctx, F16_, hd, n_head_kv, n_kv)
            tq = L.lm_ggml_new_tensor_3d(ctx, F32, hd, n_head, n_tokens)
            return L.lm_ggml_mul_mat(ctx, L.lm_ggml_permute(ctx, tk, 0, 2, 1, 3), L.lm_ggml_permute(ctx, tq, 0, 2, 1, 3)), {"k": tk, "q": tq}

        def build_kqv(ctx):
            tv = L.lm_ggml_new_tensor_3d(ctx, F16_, n_kv, n_head_kv, hd)
            tp = L.lm_ggml_new_tensor_3d(ctx, F32, n_kv, n_tokens, n_head)
            return L.lm_ggml_mul_mat(ctx, L.lm_ggml_permute(ctx, tv, 0, 2, 1, 3), tp), {"v": tv, "p": tp}
        kq = self._run_graph(build_kq, {"k": k_cache, "q": _f32(q)}, (n_head, n_tokens, n_kv), np.float32, nthreads)
        kqv = self._run_graph(build_kqv, {"v": vt_cache, "p": _f32(p)}, (n_head, n_tokens, hd), np.float32, nthreads)
        return kq, kqv

    def get_rows_graph(self, t, table, nc, ids, nthreads=1):
        """lm_ggml_get_rows on the reference CPU backend: table as Oracle.get_rows takes it, ids int32 [n] -> fp32 [n, nc]."""
        L = self.lib
        L.lm_ggml_get_rows.restype = _vp
        L.lm_ggml_get_rows.argtypes = [_vp, _vp, _vp]
        table = np.ascontiguousarray(table)
        ids = np.ascontiguousarray(ids, np.int32)
        ne01 = table.shape[0]

        def build(ctx):
            ta = L.lm_ggml_new_tensor_2d(ctx, t, nc, ne01)
            ti = L.lm_ggml_new_tensor_1d(ctx, 26, ids.size)
            return L.lm_ggml_get_rows(ctx, ta, ti), {"a": ta, "i": ti}
        return self._run_graph(build, {"a": table, "i": ids}, (ids.size, nc), np.float32, nthreads)

    def mul_mat_id_graph(self, wtype, W, x, ids, nthreads=1):
        """LM_GGML_OP_MUL_MAT_ID on the reference CPU backend: W uint8 [n_as, N, row_size], x fp32
        [n_tokens, ne11, K], ids int32 [n_tokens, n_used] -> y fp32 [n_tokens, n_used, N]."""
        L = self.lib
        W = np.ascontiguousarray(W, np.uint8)
        x = _f32(x)
        ids = np.ascontiguousarray(ids, np.int32)
        n_tokens, ne11, k = x.shape
        n_as, N = W.shape[0], W.shape[1]
        n_used = ids.shape[1]
        I32 = 26                                                   # LM_GGML_TYPE_I32 (ggml.h)
        ctx = L.lm_ggml_init(_InitParams(L.lm_ggml_tensor_overhead() * 8 + L.lm_ggml_graph_overhead() + 4096,
                                         None, True))
        a = L.lm_ggml_new_tensor_3d(ctx, wtype, k, N, n_as)
        b = L.lm_ggml_new_tensor_3d(ctx, F32, k, ne11, n_tokens)
        i = L.lm_ggml_new_tensor_2d(ctx, I32, n_used, n_tokens)
        c = L.lm_ggml_mul_mat_id(ctx, a, b, i)
        g = L.lm_ggml_new_graph(ctx)
        L.lm_ggml_build_forward_expand(g, c)
        be = L.lm_ggml_backend_cpu_init()
        L.lm_ggml_backend_cpu_set_n_threads(be, nthreads)
        buf = L.lm_ggml_backend_alloc_ctx_tensors(ctx, be)
        L.lm_ggml_backend_tensor_set(a, _ptr(W), 0, W.size)
        L.lm_ggml_backend_tensor_set(b, _ptr(x), 0, x.size * 4)
        L.lm_ggml_backend_tensor_set(i, _ptr(ids), 0, ids.size * 4)
        assert L.lm_ggml_backend_graph_compute(be, g) == 0
        y = np.zeros((n_tokens, n_used, N), np.float32)
        L.lm_ggml_backend_tensor_get(c, _ptr(y), 0, y.size * 4)
        L.lm_ggml_backend_buffer_free(buf)
        L.lm_ggml_backend_free(be)
        L.lm_ggml_free(ctx)
        return y
