// Prefill GEMM for gfx950 over K-quant weights (Q4_K, Q5_K, Q6_K) and Q8_K activations: the batched form of
// lm_ggml_vec_dot_q4_K_q8_K / _q5_K_q8_K / _q6_K_q8_K (reference ggml-cpu/ggml-cpu-quants.c) as driven by
// lm_ggml_compute_forward_mul_mat (ggml-cpu/ggml-cpu.c:1257-1449).
//
// Per 256-value super-block the reference forms two integers per (row, token),
//     sumi = sum_j sc_j * dot(q_j, a_j)        and (Q4_K, Q5_K)        summ = sum_j m_j * bsum_j,
// with 6-bit (Q4_K, Q5_K: 32-value sub-blocks) or 8-bit signed (Q6_K: 16-value sub-blocks) integer sub-block
// scales, and applies the fp16 super-block scales d, dmin and the fp32 activation scale once per super-block.
// Applying an integer scale after each 32-value MFMA would cost vector work per integer sum, which is what bounds
// the Q4_0 GEMM.  Here the integer scales are folded into the int8 MFMA operand instead:
//
//   Q4_K   sc = 8*sh + sl (3-bit digits): planes q*sh and q*sl (both <= 105), sumi = 8*P0 + P1
//   Q5_K   sc = 16*s2 + 4*s1 + s0 (2-bit digits): planes q*s2, q*s1, q*s0 (<= 93), sumi = 16*P0 + 4*P1 + P2
//   Q6_K   (q - 32)*sc + 4064 = 64*hi + lo with hi in 0..127, lo in 0..63: two digit planes of the biased product,
//          sumi = 64*P0 + P1 - 4064 * (sum of the token's 256 quants, i.e. of its 16 bsums)
//   mins   summ = sum_k m_j(k) * a_k: one more MFMA whose weight operand is the sub-block's m_j in all 32 positions
//          (built in registers from one byte, never stored per element)
//
// so every plane accumulates in the MFMA's own int32 accumulator over the 8 k-blocks of a super-block and the
// vector unit only works once per super-block and output (6-7 operations per 256 values instead of 16).  All
// sums are exact integers, equal to the reference's sumi and summ.
//
// Structure: a workgroup of WR x WC waves owns 32*WR rows x 64*WC tokens; each wave owns one 32-row tile by two
// 32-token tiles.  LDS is double buffered over stages of 4 k-blocks (half a super-block), one barrier per stage,
// the next stage's global loads in flight during the current stage's MFMAs.  Operand cells are 16 bytes
// ([plane][k-block][k-half][row]), exactly what one lane feeds v_mfma_i32_32x32x32_i8.
#include "dev_common.h"
#include "act_layout.h"
#include "kernels.h"
#include <cstdlib>
#include <type_traits>

namespace chip {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

constexpr int KQ_KB = 4;                      // 32-value k-blocks per LDS stage
constexpr int KQ_TN = 2;                      // 32-token tiles per wave
constexpr int Q6_BIAS = 4064;                 // 32 * 127: makes (q - 32) * sc + bias >= 0 for every int8 sc

// two independent 16-bit products / multiply-adds per dword (v_pk_mul_lo_u16, v_pk_mad_u16)
__device__ __forceinline__ uint32_t pk_mul16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, (u16x2)(__builtin_bit_cast(u16x2, a) * __builtin_bit_cast(u16x2, b)));
}
__device__ __forceinline__ uint32_t pk_mad16(uint32_t a, uint32_t b, uint32_t c) {
    return __builtin_bit_cast(uint32_t, (u16x2)(__builtin_bit_cast(u16x2, a) * __builtin_bit_cast(u16x2, b) + __builtin_bit_cast(u16x2, c)));
}
__device__ __forceinline__ uint32_t splat16(uint32_t v) { return (v & 0xffffu) | (v << 16); }

// 6-bit scales and mins of sub-blocks 2jp and 2jp+1 (low byte, next byte) from the 12 packed bytes that follow
// d and dmin (reference ggml-quants.c:625-632); uniform branch: jp < 2 for the first half of a super-block
__device__ __forceinline__ void scale_min_pair(const u32x4 &h, int jp, uint32_t &sc, uint32_t &mn) {
    const int sh = 16 * (jp & 1);
    const uint32_t a1 = h.y >> sh, a2 = h.z >> sh, a3 = h.w >> sh;
    if (jp < 2) { sc = a1 & 0x3f3fu; mn = a2 & 0x3f3fu; }
    else        { sc = (a3 & 0x0f0fu) | ((a1 >> 2) & 0x3030u); mn = ((a3 >> 4) & 0x0f0fu) | ((a2 >> 2) & 0x3030u); }
}

// One staging item = (row, x) of a stage h (half of a super-block): 16 bytes of packed quants that expand into
// the 16-value k-half hf = x & 1 of two k-blocks kb0(x), kb1(x) of the stage, for every stored plane.
struct Emit {
    u32x4 cell[3][2];      // [plane][0: k-block kb0, 1: k-block kb1]
    uint32_t mins;         // m of kb0 | m of kb1 << 8
    uint32_t dd;           // d | dmin << 16 (fp16 bits)
};

template <int WT> struct KQ;

template <> struct KQ<T_Q4_K> {
    static constexpr int BYTES = BYTES_Q4_K, NPL = 2, NACC = 3;
    static constexpr bool HAS_MIN = true, HAS_BSUM = false;
    struct Raw { u32x4 hdr, q; };
    __device__ static __forceinline__ void fetch(Raw &r, const uint8_t *blk, int h, int x) {
        r.hdr = *reinterpret_cast<const u32x4 *>(blk);
        r.q = *reinterpret_cast<const u32x4 *>(blk + 16 + 64 * h + 16 * x);       // qs[32*jp + 16*hf], jp = 2h + x/2
    }
    __device__ static __forceinline__ int kb0(int x) { return x & 2; }            // low nibbles: sub-block 2*jp
    __device__ static __forceinline__ int kb1(int x) { return (x & 2) + 1; }      // high nibbles: sub-block 2*jp + 1
    __device__ static __forceinline__ void emit(Emit &e, const Raw &r, int h, int x) {
        uint32_t sc, mn;
        scale_min_pair(r.hdr, 2 * h + (x >> 1), sc, mn);
        const uint32_t sc0 = sc & 0xff, sc1 = sc >> 8;
        const uint32_t sh0 = splat16(sc0 >> 3), sl0 = splat16(sc0 & 7), sh1 = splat16(sc1 >> 3), sl1 = splat16(sc1 & 7);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t lo = r.q[i] & 0x0f0f0f0fu, hi = (r.q[i] >> 4) & 0x0f0f0f0fu;
            e.cell[0][0][i] = pk_mul16(lo, sh0); e.cell[1][0][i] = pk_mul16(lo, sl0);   // byte products < 256: no carries
            e.cell[0][1][i] = pk_mul16(hi, sh1); e.cell[1][1][i] = pk_mul16(hi, sl1);
        }
        e.mins = mn;
        e.dd = r.hdr.x;
    }
    __device__ static __forceinline__ float value(const int (&p)[NACC], uint32_t dd, int) {
        return h2f(dd) * (float)((p[0] << 3) + p[1]) - h2f(dd >> 16) * (float)p[2];
    }
};

template <> struct KQ<T_Q5_K> {
    static constexpr int BYTES = BYTES_Q5_K, NPL = 3, NACC = 4;
    static constexpr bool HAS_MIN = true, HAS_BSUM = false;
    struct Raw { u32x4 hdr, q, qh; };
    __device__ static __forceinline__ void fetch(Raw &r, const uint8_t *blk, int h, int x) {
        r.hdr = *reinterpret_cast<const u32x4 *>(blk);
        r.qh = *reinterpret_cast<const u32x4 *>(blk + 16 + 16 * (x & 1));          // qh[l], l = 16*hf + [0,16)
        r.q = *reinterpret_cast<const u32x4 *>(blk + 48 + 64 * h + 16 * x);
    }
    __device__ static __forceinline__ int kb0(int x) { return x & 2; }
    __device__ static __forceinline__ int kb1(int x) { return (x & 2) + 1; }
    __device__ static __forceinline__ void emit(Emit &e, const Raw &r, int h, int x) {
        const int jp = 2 * h + (x >> 1);
        uint32_t sc, mn;
        scale_min_pair(r.hdr, jp, sc, mn);
        const uint32_t sc0 = sc & 0xff, sc1 = sc >> 8;
        const uint32_t a2 = splat16(sc0 >> 4), a1 = splat16((sc0 >> 2) & 3), a0 = splat16(sc0 & 3);
        const uint32_t b2 = splat16(sc1 >> 4), b1 = splat16((sc1 >> 2) & 3), b0 = splat16(sc1 & 3);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // bit 2*jp of qh[l] is the fifth bit of element 64*jp + l, bit 2*jp + 1 that of 64*jp + 32 + l
            // (reference ggml-quants.c:1460-1478)
            const uint32_t hb = r.qh[i] >> (2 * jp);
            const uint32_t lo = (r.q[i] & 0x0f0f0f0fu) | ((hb << 4) & 0x10101010u);
            const uint32_t hi = ((r.q[i] >> 4) & 0x0f0f0f0fu) | ((hb << 3) & 0x10101010u);
            e.cell[0][0][i] = pk_mul16(lo, a2); e.cell[1][0][i] = pk_mul16(lo, a1); e.cell[2][0][i] = pk_mul16(lo, a0);
            e.cell[0][1][i] = pk_mul16(hi, b2); e.cell[1][1][i] = pk_mul16(hi, b1); e.cell[2][1][i] = pk_mul16(hi, b0);
        }
        e.mins = mn;
        e.dd = r.hdr.x;
    }
    __device__ static __forceinline__ float value(const int (&p)[NACC], uint32_t dd, int) {
        return h2f(dd) * (float)((p[0] << 4) + (p[1] << 2) + p[2]) - h2f(dd >> 16) * (float)p[3];
    }
};

template <> struct KQ<T_Q6_K> {
    static constexpr int BYTES = BYTES_Q6_K, NPL = 2, NACC = 2;
    static constexpr bool HAS_MIN = false, HAS_BSUM = true;
    struct Raw { u32x4 ql, qh; int s0, s1; uint32_t d; };
    // Half h of a super-block holds, for l = 0..31, the elements 128h + 32b + l of k-blocks b = 0..3 as
    //   low / high nibble of ql[64h + l] (b = 0 / 2) and of ql[64h + 32 + l] (b = 1 / 3), two more bits from
    //   qh[32h + l] >> 2b, scale scales[8h + 2b + l/16]                       (reference ggml-quants.c:1695-1711)
    // item x: p = x / 2 picks the ql half (k-blocks p and p + 2), hf = x & 1 the 16 values l = 16*hf + [0,16).
    __device__ static __forceinline__ void fetch(Raw &r, const uint8_t *blk, int h, int x) {
        const int p = x >> 1, hf = x & 1;
        r.ql = *reinterpret_cast<const u32x4_a2 *>(blk + 64 * h + 32 * p + 16 * hf);
        r.qh = *reinterpret_cast<const u32x4_a2 *>(blk + 128 + 32 * h + 16 * hf);
        r.s0 = *reinterpret_cast<const int8_t *>(blk + 192 + 8 * h + 2 * p + hf);
        r.s1 = *reinterpret_cast<const int8_t *>(blk + 192 + 8 * h + 2 * p + 4 + hf);
        r.d = *reinterpret_cast<const unsigned short *>(blk + 208);
    }
    __device__ static __forceinline__ int kb0(int x) { return x >> 1; }
    __device__ static __forceinline__ int kb1(int x) { return (x >> 1) + 2; }
    // q: four 6-bit values 0..63 in bytes -> digits of q*sc + (4064 - 32*sc) = (q - 32)*sc + 4064 in 0..8160
    __device__ static __forceinline__ void digits(uint32_t q, uint32_t sc2, uint32_t bias2, uint32_t &hi, uint32_t &lo) {
        const uint32_t ev = q & 0x00ff00ffu, od = (q >> 8) & 0x00ff00ffu;
        const uint32_t ue = pk_mad16(ev, sc2, bias2), uo = pk_mad16(od, sc2, bias2);
        hi = ((ue >> 6) & 0x007f007fu) | (((uo >> 6) & 0x007f007fu) << 8);
        lo = (ue & 0x003f003fu) | ((uo & 0x003f003fu) << 8);
    }
    __device__ static __forceinline__ void emit(Emit &e, const Raw &r, int, int x) {
        const int p = x >> 1;
        const uint32_t sa = splat16((uint32_t)r.s0), ba = splat16((uint32_t)(Q6_BIAS - 32 * r.s0));
        const uint32_t sb = splat16((uint32_t)r.s1), bb = splat16((uint32_t)(Q6_BIAS - 32 * r.s1));
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t hb = r.qh[i] >> (2 * p);
            const uint32_t q0 = (r.ql[i] & 0x0f0f0f0fu) | ((hb << 4) & 0x30303030u);            // k-block p
            const uint32_t q1 = ((r.ql[i] >> 4) & 0x0f0f0f0fu) | (hb & 0x30303030u);            // k-block p + 2
            uint32_t hi, lo;
            digits(q0, sa, ba, hi, lo);
            e.cell[0][0][i] = hi; e.cell[1][0][i] = lo;
            digits(q1, sb, bb, hi, lo);
            e.cell[0][1][i] = hi; e.cell[1][1][i] = lo;
        }
        e.mins = 0;
        e.dd = r.d;
    }
    __device__ static __forceinline__ float value(const int (&p)[NACC], uint32_t dd, int corr) {
        return h2f(dd) * (float)((p[0] << 6) + p[1] + corr);
    }
};

template <int WT, int WR, int WC>
struct KqCfg {
    using T = KQ<WT>;
    static constexpr int NW = WR * WC, NT = NW * 64;
    static constexpr int BM = 32 * WR;                             // weight rows per workgroup
    static constexpr int BN = 32 * KQ_TN * WC;                     // tokens per workgroup
    // plane stride 2 mod 16 cells: the staging threads of one wave spread over the bank groups
    static constexpr int A_PLANE = BM + 2, B_PLANE = BN + 2;
    static constexpr int A_CELLS = T::NPL * KQ_KB * 2 * A_PLANE;   // 16-byte cells
    static constexpr int B_CELLS = KQ_KB * 2 * B_PLANE;
    static constexpr size_t OFF_A = 0;
    static constexpr size_t OFF_B = OFF_A + (size_t)A_CELLS * 16;
    static constexpr size_t OFF_SD = OFF_B + (size_t)B_CELLS * 16;          // u32 [BM]: d | dmin << 16, permuted per 32 rows
    static constexpr size_t OFF_SM = OFF_SD + (size_t)BM * 4;               // u8  [BM][4]: m of the stage's 4 k-blocks
    static constexpr size_t OFF_SX = OFF_SM + (size_t)BM * 4;               // f32 [BN]: activation scale of the super-block
    static constexpr size_t OFF_SC = OFF_SX + (size_t)BN * 4;               // i32 [BN]: -4064 * sum of the token's quants
    static constexpr size_t STAGE = OFF_SC + (size_t)BN * 4;
    static constexpr int W_ITEMS = BM * 4;
    static constexpr int W_PER_T = (W_ITEMS + NT - 1) / NT;
    static constexpr int X_ITEMS = BN * KQ_KB * 2;
    static constexpr int X_PER_T = (X_ITEMS + NT - 1) / NT;
    static_assert(BN <= NT, "one thread per token stages the activation scale");
    static_assert(STAGE % 16 == 0, "stage buffers keep 16-byte alignment");
};

template <int WT, int WR, int WC, int OCC>
__global__ __launch_bounds__(WR *WC * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void gemm_kq_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N, const uint8_t *__restrict__ ws,
                    size_t ws_stride, int64_t M, float *__restrict__ y, int64_t ldy) {
    using T = KQ<WT>;
    using C = KqCfg<WT, WR, WC>;
    constexpr int TN = KQ_TN;
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave / WC, wc = wave % WC;
    const int half = lane >> 5, l32 = lane & 31;
    const int64_t row_base = (int64_t)blockIdx.x * C::BM;
    const int64_t tok_base = (int64_t)blockIdx.y * C::BN;
    const int nstages = (int)(K / QK_K) * 2;
    const size_t off_d = q8_K_off_d(K), off_bs = q8_K_off_bsums(K);

    // ---- per-thread prefetch registers for one stage ----
    typename T::Raw wraw[C::W_PER_T];
    u32x4 xq[C::X_PER_T];
    float xs = 0.f;
    int xc = 0;

    auto fetch = [&](int stage) {
        const int sb = stage >> 1, h = stage & 1;
#pragma unroll
        for (int i = 0; i < C::W_PER_T; i++) {
            const int item = tid + i * C::NT;
            if (C::W_ITEMS % C::NT == 0 || item < C::W_ITEMS) {
                const int64_t row = min(row_base + (item >> 2), N - 1);
                T::fetch(wraw[i], W + (size_t)row * nb01 + (size_t)sb * T::BYTES, h, item & 3);
            }
        }
#pragma unroll
        for (int i = 0; i < C::X_PER_T; i++) {
            const int item = tid + i * C::NT;
            if (C::X_ITEMS % C::NT == 0 || item < C::X_ITEMS) {
                const int64_t tok = min(tok_base + (item >> 3), M - 1);
                xq[i] = *reinterpret_cast<const u32x4 *>(ws + (size_t)tok * ws_stride + (size_t)stage * (32 * KQ_KB) + 16 * (item & 7));
            }
        }
        if (tid < C::BN) {
            const uint8_t *t = ws + (size_t)min(tok_base + tid, M - 1) * ws_stride;
            xs = reinterpret_cast<const float *>(t + off_d)[sb];
            if constexpr (T::HAS_BSUM) {
                const u32x4 *bp = reinterpret_cast<const u32x4 *>(t + off_bs + (size_t)sb * 32);
                const u32x4 b0 = bp[0], b1 = bp[1];
                const uint32_t w[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
                int sum = 0;
#pragma unroll
                for (int j = 0; j < 8; j++) sum += (int)(int16_t)(w[j] & 0xffffu) + ((int)w[j] >> 16);
                xc = -Q6_BIAS * sum;
            }
        }
    };

    auto commit = [&](int stage, int buf) {
        const int h = stage & 1;
        uint8_t *base = lds + (size_t)buf * C::STAGE;
        u32x4 *A = reinterpret_cast<u32x4 *>(base + C::OFF_A);
        u32x4 *B = reinterpret_cast<u32x4 *>(base + C::OFF_B);
#pragma unroll
        for (int i = 0; i < C::W_PER_T; i++) {
            const int item = tid + i * C::NT;
            if (C::W_ITEMS % C::NT == 0 || item < C::W_ITEMS) {
                const int r = item >> 2, x = item & 3, hf = x & 1;
                Emit e;
                T::emit(e, wraw[i], h, x);
                const int k0 = T::kb0(x), k1 = T::kb1(x);
#pragma unroll
                for (int pl = 0; pl < T::NPL; pl++) {
                    A[((pl * KQ_KB + k0) * 2 + hf) * C::A_PLANE + r] = e.cell[pl][0];
                    A[((pl * KQ_KB + k1) * 2 + hf) * C::A_PLANE + r] = e.cell[pl][1];
                }
                if constexpr (T::HAS_MIN) {
                    // sub-blocks kb0, kb1 = kb0 + 1 of this row: two adjacent bytes, written by the hf = 0 item
                    if (hf == 0) *reinterpret_cast<unsigned short *>(base + C::OFF_SM + r * 4 + k0) = (unsigned short)e.mins;
                }
                if (x == 0) {
                    // the lane that owns MFMA result register v of a 32-row tile holds row 8*(v/4) + 4*half + v%4:
                    // keep the scale of row i at half*16 + (i/8)*4 + i%4 so a lane reads its 16 scales contiguously
                    const int i32 = r & 31;
                    const int pos = ((i32 >> 2) & 1) * 16 + (i32 >> 3) * 4 + (i32 & 3);
                    reinterpret_cast<uint32_t *>(base + C::OFF_SD)[(r & ~31) + pos] = e.dd;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < C::X_PER_T; i++) {
            const int item = tid + i * C::NT;
            if (C::X_ITEMS % C::NT == 0 || item < C::X_ITEMS) B[(item & 7) * C::B_PLANE + (item >> 3)] = xq[i];
        }
        if (tid < C::BN) {
            reinterpret_cast<float *>(base + C::OFF_SX)[tid] = xs;
            if constexpr (T::HAS_BSUM) reinterpret_cast<int *>(base + C::OFF_SC)[tid] = xc;
        }
    };

    i32x16 P[T::NACC][TN];
    float out[TN][16];
#pragma unroll
    for (int c = 0; c < TN; c++)
#pragma unroll
        for (int v = 0; v < 16; v++) out[c][v] = 0.f;

    const int r0 = wr * 32, n0 = wc * TN * 32;

    // 4 k-blocks of one stage; `first` starts the super-block's accumulators from zero
    auto compute = [&](int buf, auto first_tag) {
        constexpr bool first = decltype(first_tag)::value;
        const uint8_t *base = lds + (size_t)buf * C::STAGE;
        const u32x4 *A = reinterpret_cast<const u32x4 *>(base + C::OFF_A);
        const u32x4 *B = reinterpret_cast<const u32x4 *>(base + C::OFF_B);
        uint32_t mw = 0;
        if constexpr (T::HAS_MIN) mw = reinterpret_cast<const uint32_t *>(base + C::OFF_SM)[r0 + l32];
#pragma unroll
        for (int b = 0; b < KQ_KB; b++) {
            i32x4 af[T::NACC], bf[TN];
#pragma unroll
            for (int pl = 0; pl < T::NPL; pl++) {
                const u32x4 t = A[((pl * KQ_KB + b) * 2 + half) * C::A_PLANE + r0 + l32];
                af[pl] = i32x4{(int)t.x, (int)t.y, (int)t.z, (int)t.w};
            }
            if constexpr (T::HAS_MIN) {
                const int m4 = (int)__builtin_amdgcn_perm(mw, mw, 0x01010101u * (uint32_t)b);   // byte b in all four bytes
                af[T::NPL] = i32x4{m4, m4, m4, m4};
            }
#pragma unroll
            for (int c = 0; c < TN; c++) {
                const u32x4 t = B[(b * 2 + half) * C::B_PLANE + n0 + c * 32 + l32];
                bf[c] = i32x4{(int)t.x, (int)t.y, (int)t.z, (int)t.w};
            }
#pragma unroll
            for (int pl = 0; pl < T::NACC; pl++)
#pragma unroll
                for (int c = 0; c < TN; c++) {
                    if constexpr (first) {
                        if (b == 0) {
                            const i32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                            P[pl][c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[pl], bf[c], zero, 0, 0, 0);
                            continue;
                        }
                    }
                    P[pl][c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[pl], bf[c], P[pl][c], 0, 0, 0);
                }
        }
    };

    // once per super-block: fold the planes and apply d, dmin and the activation scale
    auto finish = [&](int buf) {
        const uint8_t *base = lds + (size_t)buf * C::STAGE;
        const u32x4 *sp = reinterpret_cast<const u32x4 *>(base + C::OFF_SD) + (r0 + half * 16) / 4;
        const u32x4 s0 = sp[0], s1 = sp[1], s2 = sp[2], s3 = sp[3];
        const uint32_t sd[16] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w, s2.x, s2.y, s2.z, s2.w, s3.x, s3.y, s3.z, s3.w};
#pragma unroll
        for (int c = 0; c < TN; c++) {
            const float dx = reinterpret_cast<const float *>(base + C::OFF_SX)[n0 + c * 32 + l32];
            int corr = 0;
            if constexpr (T::HAS_BSUM) corr = reinterpret_cast<const int *>(base + C::OFF_SC)[n0 + c * 32 + l32];
#pragma unroll
            for (int v = 0; v < 16; v++) {
                int p[T::NACC];
#pragma unroll
                for (int pl = 0; pl < T::NACC; pl++) p[pl] = P[pl][c][v];
                out[c][v] = __builtin_fmaf(T::value(p, sd[v], corr), dx, out[c][v]);
            }
        }
    };

    fetch(0);
    commit(0, 0);
    __syncthreads();

    for (int s = 0; s < nstages; s += 2) {
        // first half of the super-block (buffer 0), second half (buffer 1)
        fetch(s + 1);
        compute(0, std::true_type{});
        commit(s + 1, 1);
        __syncthreads();

        if (s + 2 < nstages) fetch(s + 2);
        compute(1, std::false_type{});
        finish(1);
        if (s + 2 < nstages) commit(s + 2, 0);
        __syncthreads();
    }

    // ---- epilogue: register v of token tile c is row 8*(v/4) + 4*half + v%4, token l32 ----
#pragma unroll
    for (int c = 0; c < TN; c++) {
        const int64_t tok = tok_base + n0 + c * 32 + l32;
        if (tok >= M) continue;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int64_t row = row_base + r0 + 8 * g + 4 * half;
            float *dst = y + (size_t)tok * ldy + row;
            if (row + 3 < N && (((uintptr_t)dst) & 15) == 0) {
                *reinterpret_cast<float4 *>(dst) = make_float4(out[c][4 * g], out[c][4 * g + 1], out[c][4 * g + 2], out[c][4 * g + 3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (row + e < N) dst[e] = out[c][4 * g + e];
            }
        }
    }
}

bool gemm_kq_supported(int wtype, int64_t K, int64_t N, int64_t n) {
    return (wtype == T_Q4_K || wtype == T_Q5_K || wtype == T_Q6_K) && K >= QK_K && K % QK_K == 0 && N >= 1 && n >= 1;
}

template <int WT, int WR, int WC, int OCC>
static hipError_t launch_kq(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int64_t M,
                            float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st) {
    using C = KqCfg<WT, WR, WC>;
    const size_t lds_bytes = 2 * C::STAGE;
    if ((int64_t)lds_bytes > lim.max_lds_per_block) return hipErrorInvalidValue;
    auto kfn = gemm_kq_kernel<WT, WR, WC, OCC>;
    static LdsGrant grant;                                               // one per kernel instantiation
    if (hipError_t e = grant_dynamic_lds(kfn, lds_bytes, lim, grant); e != hipSuccess) return e;
    dim3 grid((unsigned)ceil_div(N, C::BM), (unsigned)ceil_div(M, C::BN));
    hipLaunchKernelGGL(kfn, grid, dim3(C::NT), lds_bytes, st, (const uint8_t *)W, nb01, K, N, (const uint8_t *)ws, ws_stride,
                       M, y, ldy);
    return hipGetLastError();
}

template <int WT>
static hipError_t launch_kq_type(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                                 int64_t M, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st) {
    const int64_t cus = lim.compute_units > 0 ? lim.compute_units : 256;
    const int64_t g128 = ceil_div(N, 128) * ceil_div(M, 128);
    const char *force = getenv("CHIP_GEMM_KQ_CFG");
    const int cfg = force ? atoi(force) : (g128 >= cus ? 0 : 1);
    switch (cfg) {
        case 0: return launch_kq<WT, 4, 2, 2>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st);      // 128 x 128, 8 waves
        case 1: return launch_kq<WT, 2, 2, 2>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st);      // 64 x 128, 4 waves
        case 2: return launch_kq<WT, 2, 4, 2>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st);      // 64 x 256, 8 waves
        case 3: return launch_kq<WT, 2, 1, 2>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st);      // 64 x 64, 2 waves
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_gemm_kq(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                          int64_t M, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st) {
    if (M <= 0 || N <= 0) return hipSuccess;
    switch (wtype) {
        case T_Q4_K: return launch_kq_type<T_Q4_K>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st);
        case T_Q5_K: return launch_kq_type<T_Q5_K>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st);
        case T_Q6_K: return launch_kq_type<T_Q6_K>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace chip
