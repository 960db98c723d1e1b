// Prefill GEMM for gfx950 over K-quant weights (Q4_K, Q5_K, Q6_K) and Q8_K activations: the batched form of
// lm_ggml_vec_dot_q4_K_q8_K / _q5_K_q8_K / _q6_K_q8_K (reference ggml-cpu/ggml-cpu-quants.c) as driven by
// lm_ggml_compute_forward_mul_mat (ggml-cpu/ggml-cpu.c:1257-1449).
//
// Per 256-value super-block the reference forms two integers per (row, token),
//     sumi = sum_j sc_j * dot(q_j, a_j)        and (Q4_K, Q5_K)        summ = sum_j m_j * bsum_j,
// with 6-bit (Q4_K, Q5_K: 32-value sub-blocks) or 8-bit signed (Q6_K: 16-value sub-blocks) integer sub-block
// scales, and applies the fp16 super-block scales d, dmin and the fp32 activation scale once per super-block.
// Applying an integer scale after each 32-value MFMA would cost vector work per integer sum, which is what bounds
// the Q4_0 GEMM.  Here the integer scales are folded into the int8 MFMA operand instead, as two digit planes:
//
//   Q4_K   sc = 8*sh + sl (3-bit digits): planes q*sh and q*sl (both <= 105), sumi = 8*P0 + P1
//   Q5_K   the same digits on (q - 16) in -16..15 (products in -112..105), sumi = 8*P0 + P1 + 16 * sum_j sc_j * bsum_j
//   Q6_K   (q - 32)*sc + 4064 = 64*hi + lo with hi in 0..127, lo in 0..63: the digits of the biased product,
//          sumi = 64*P0 + P1 - 4064 * (sum of the token's 256 quants, i.e. of its 16 bsums)
//
// so both planes accumulate in the MFMA's own int32 accumulator over the 8 k-blocks of a super-block.  The sums
// against the activation block sums, summ (and Q5_K's sum_j sc_j * bsum_j), are a product with inner dimension 16
// per super-block - the 16 bsums of block_q8_K, each |bsum| <= 2048, against m_j (sc_j) <= 63 taken twice - which
// is exact in fp16 inputs with fp32 accumulation: one v_mfma_f32_32x32x16_f16 per super-block and tile.  The vector
// unit works only once per super-block and output (5-6 operations per 256 values instead of 16).  All sums are
// exact integers, equal to the reference's sumi and summ.
//
// Structure: a workgroup of WR x WC waves owns 32*WR rows x 64*WC tokens; each wave owns one 32-row tile by two
// 32-token tiles.  LDS is double buffered over stages of 4 k-blocks (half a super-block), one barrier per stage.
// Operand cells are 16 bytes ([plane][k-block][k-half][row]), exactly what one lane feeds v_mfma_i32_32x32x32_i8.
#include "dev_common.h"
#include "act_layout.h"
#include "kernels.h"
#include <cstdlib>
#include <type_traits>

namespace chip {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

constexpr int KQ_KB = 4;                      // 32-value k-blocks per LDS stage
constexpr int KQ_TN = 2;                      // 32-token tiles per wave
constexpr int KQ_NPL = 2;                     // int8 digit planes per weight type
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
    else        { sc = (a3 & 0x0f0f0f0fu & 0xffffu) | ((a1 >> 2) & 0x3030u); mn = ((a3 >> 4) & 0x0f0fu) | ((a2 >> 2) & 0x3030u); }
}
// the same for four sub-blocks at once, one per byte: sub-blocks 0..3 (g = 0) or 4..7 (g = 1)
__device__ __forceinline__ void scale_min_quad(const u32x4 &h, int g, uint32_t &sc, uint32_t &mn) {
    if (g == 0) { sc = h.y & 0x3f3f3f3fu; mn = h.z & 0x3f3f3f3fu; }
    else        { sc = (h.w & 0x0f0f0f0fu) | ((h.y >> 2) & 0x30303030u); mn = ((h.w >> 4) & 0x0f0f0f0fu) | ((h.z >> 2) & 0x30303030u); }
}
// four small integers (one per byte) -> the fp16 operand cell {b0, b0, b1, b1, b2, b2, b3, b3}: sub-block j stands
// against the two 16-value bsums 2j and 2j+1
__device__ __forceinline__ u32x4 bytes_to_f16_pairs(uint32_t v) {
    u32x4 c;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t hbits = (uint32_t)__half_as_ushort(__float2half_rn((float)((v >> (8 * i)) & 0xffu)));   // exact
        c[i] = hbits | (hbits << 16);
    }
    return c;
}
// eight int16 -> eight fp16 (exact for |v| <= 2048)
__device__ __forceinline__ u32x4 i16x8_to_f16(const u32x4 &v) {
    u32x4 c;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const _Float16 lo = (_Float16)(int16_t)(v[i] & 0xffffu), hi = (_Float16)(int16_t)(v[i] >> 16);
        c[i] = (uint32_t)__builtin_bit_cast(unsigned short, lo) | ((uint32_t)__builtin_bit_cast(unsigned short, hi) << 16);
    }
    return c;
}

// One staging item = (row, x) of a stage h (half of a super-block): 16 bytes of packed quants that expand into
// the 16-value k-half hf = x & 1 of two k-blocks kb0(x), kb1(x) of the stage, for both digit planes.
struct Emit {
    u32x4 cell[KQ_NPL][2]; // [plane][0: k-block kb0, 1: k-block kb1]
};

template <int WT> struct KQ;

template <> struct KQ<T_Q4_K> {
    static constexpr int BYTES = BYTES_Q4_K, NF16 = 1;             // fp16 products: summ
    static constexpr bool HAS_BSUM = false;
    // what item x of a row needs from one super-block: the 16 header bytes and 16 quant bytes per half
    struct Raw { u32x4 hdr, q[2]; };
    __device__ static __forceinline__ void fetch(Raw &r, const uint8_t *blk, int x) {
        r.hdr = *reinterpret_cast<const u32x4 *>(blk);
        r.q[0] = *reinterpret_cast<const u32x4 *>(blk + 16 + 16 * x);             // qs[32*jp + 16*hf], jp = 2h + x/2
        r.q[1] = *reinterpret_cast<const u32x4 *>(blk + 80 + 16 * x);
    }
    __device__ static __forceinline__ int kb0(int x) { return x & 2; }            // low nibbles: sub-block 2*jp
    __device__ static __forceinline__ int kb1(int x) { return (x & 2) + 1; }      // high nibbles: sub-block 2*jp + 1
    __device__ static __forceinline__ void emit(Emit &e, const Raw &r, int h, int x) {
        uint32_t sc, mn;
        scale_min_pair(r.hdr, 2 * h + (x >> 1), sc, mn);
        const uint32_t sc0 = sc & 0xff, sc1 = sc >> 8;
        const uint32_t sh0 = splat16(sc0 >> 3), sl0 = splat16(sc0 & 7), sh1 = splat16(sc1 >> 3), sl1 = splat16(sc1 & 7);
        const u32x4 q = r.q[h];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t lo = q[i] & 0x0f0f0f0fu, hi = (q[i] >> 4) & 0x0f0f0f0fu;
            e.cell[0][0][i] = pk_mul16(lo, sh0); e.cell[1][0][i] = pk_mul16(lo, sl0);   // byte products < 256: no carries
            e.cell[0][1][i] = pk_mul16(hi, sh1); e.cell[1][1][i] = pk_mul16(hi, sl1);
        }
    }
    __device__ static __forceinline__ uint32_t scales(const Raw &r) { return r.hdr.x; }        // d | dmin << 16
    // fp16 operand cell of item x < 2: mins of sub-blocks 4x .. 4x+3
    __device__ static __forceinline__ u32x4 f16_cell(const Raw &r, int x) {
        uint32_t sc, mn;
        scale_min_quad(r.hdr, x & 1, sc, mn);
        return bytes_to_f16_pairs(mn);
    }
    __device__ static __forceinline__ float value(int p0, int p1, const float (&f)[2], uint32_t dd, int) {
        return __builtin_fmaf(-h2f(dd >> 16), f[0], __builtin_fmaf(h2f(dd), (float)((p0 << 3) + p1), 0.f));
    }
};

template <> struct KQ<T_Q5_K> {
    static constexpr int BYTES = BYTES_Q5_K, NF16 = 2;             // fp16 products: summ, sum_j sc_j * bsum_j
    static constexpr bool HAS_BSUM = false;
    struct Raw { u32x4 hdr, qh, q[2]; };
    __device__ static __forceinline__ void fetch(Raw &r, const uint8_t *blk, int x) {
        r.hdr = *reinterpret_cast<const u32x4 *>(blk);
        r.qh = *reinterpret_cast<const u32x4 *>(blk + 16 + 16 * (x & 1));          // qh[l], l = 16*hf + [0,16)
        r.q[0] = *reinterpret_cast<const u32x4 *>(blk + 48 + 16 * x);
        r.q[1] = *reinterpret_cast<const u32x4 *>(blk + 112 + 16 * x);
    }
    __device__ static __forceinline__ int kb0(int x) { return x & 2; }
    __device__ static __forceinline__ int kb1(int x) { return (x & 2) + 1; }
    __device__ static __forceinline__ void emit(Emit &e, const Raw &r, int h, int x) {
        const int jp = 2 * h + (x >> 1);
        uint32_t sc, mn;
        scale_min_pair(r.hdr, jp, sc, mn);
        const uint32_t sc0 = sc & 0xff, sc1 = sc >> 8;
        // byte = q*s + (128 - 16*s) lies in 16..233 for q in 0..31, s in 0..7: no carries between the bytes of a
        // 16-bit lane, and flipping bit 7 turns it into the signed byte (q - 16)*s
        const uint32_t sh0 = sc0 >> 3, sl0 = sc0 & 7, sh1 = sc1 >> 3, sl1 = sc1 & 7;
        const uint32_t mh0 = splat16(sh0), ml0 = splat16(sl0), mh1 = splat16(sh1), ml1 = splat16(sl1);
        const uint32_t ah0 = splat16((128 - 16 * sh0) * 0x101u), al0 = splat16((128 - 16 * sl0) * 0x101u);
        const uint32_t ah1 = splat16((128 - 16 * sh1) * 0x101u), al1 = splat16((128 - 16 * sl1) * 0x101u);
        const u32x4 q = r.q[h];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // bit 2*jp of qh[l] is the fifth bit of element 64*jp + l, bit 2*jp + 1 that of 64*jp + 32 + l
            // (reference ggml-quants.c:1460-1478)
            const uint32_t hb = r.qh[i] >> (2 * jp);
            const uint32_t lo = (q[i] & 0x0f0f0f0fu) | ((hb << 4) & 0x10101010u);
            const uint32_t hi = ((q[i] >> 4) & 0x0f0f0f0fu) | ((hb << 3) & 0x10101010u);
            e.cell[0][0][i] = pk_mad16(lo, mh0, ah0) ^ 0x80808080u; e.cell[1][0][i] = pk_mad16(lo, ml0, al0) ^ 0x80808080u;
            e.cell[0][1][i] = pk_mad16(hi, mh1, ah1) ^ 0x80808080u; e.cell[1][1][i] = pk_mad16(hi, ml1, al1) ^ 0x80808080u;
        }
    }
    __device__ static __forceinline__ uint32_t scales(const Raw &r) { return r.hdr.x; }
    // item x: x / 2 = 0 mins, 1 scales; x & 1 = sub-blocks 0..3 or 4..7
    __device__ static __forceinline__ u32x4 f16_cell(const Raw &r, int x) {
        uint32_t sc, mn;
        scale_min_quad(r.hdr, x & 1, sc, mn);
        return bytes_to_f16_pairs((x & 2) ? sc : mn);
    }
    __device__ static __forceinline__ float value(int p0, int p1, const float (&f)[2], uint32_t dd, int) {
        const int sumi = (p0 << 3) + p1 + ((int)f[1] << 4);                 // f[1] is an exact integer below 2^24
        return __builtin_fmaf(-h2f(dd >> 16), f[0], __builtin_fmaf(h2f(dd), (float)sumi, 0.f));
    }
};

template <> struct KQ<T_Q6_K> {
    static constexpr int BYTES = BYTES_Q6_K, NF16 = 0;
    static constexpr bool HAS_BSUM = true;
    struct Raw { u32x4 ql[2], qh[2], sc; uint32_t d; };
    // Half h of a super-block holds, for l = 0..31, the elements 128h + 32b + l of k-blocks b = 0..3 as
    //   low / high nibble of ql[64h + l] (b = 0 / 2) and of ql[64h + 32 + l] (b = 1 / 3), two more bits from
    //   qh[32h + l] >> 2b, scale scales[8h + 2b + l/16]                       (reference ggml-quants.c:1695-1711)
    // item x: p = x / 2 picks the ql half (k-blocks p and p + 2), hf = x & 1 the 16 values l = 16*hf + [0,16).
    __device__ static __forceinline__ void fetch(Raw &r, const uint8_t *blk, int x) {
        const int p = x >> 1, hf = x & 1;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            r.ql[h] = *reinterpret_cast<const u32x4_a2 *>(blk + 64 * h + 32 * p + 16 * hf);
            r.qh[h] = *reinterpret_cast<const u32x4_a2 *>(blk + 128 + 32 * h + 16 * hf);
        }
        r.sc = *reinterpret_cast<const u32x4_a2 *>(blk + 192);
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
    __device__ static __forceinline__ void emit(Emit &e, const Raw &r, int h, int x) {
        const int p = x >> 1, hf = x & 1;
        // scales[8h + 2p + hf] and scales[8h + 2p + 4 + hf]: byte 2p + hf of dwords 2h and 2h + 1
        const int s0 = __builtin_amdgcn_sbfe((int)r.sc[2 * h], 8 * (2 * p + hf), 8);
        const int s1 = __builtin_amdgcn_sbfe((int)r.sc[2 * h + 1], 8 * (2 * p + hf), 8);
        const uint32_t sa = splat16((uint32_t)s0), ba = splat16((uint32_t)(Q6_BIAS - 32 * s0));
        const uint32_t sb = splat16((uint32_t)s1), bb = splat16((uint32_t)(Q6_BIAS - 32 * s1));
        const u32x4 ql = r.ql[h], qh = r.qh[h];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t hb = qh[i] >> (2 * p);
            const uint32_t q0 = (ql[i] & 0x0f0f0f0fu) | ((hb << 4) & 0x30303030u);            // k-block p
            const uint32_t q1 = ((ql[i] >> 4) & 0x0f0f0f0fu) | (hb & 0x30303030u);            // k-block p + 2
            uint32_t hi, lo;
            digits(q0, sa, ba, hi, lo);
            e.cell[0][0][i] = hi; e.cell[1][0][i] = lo;
            digits(q1, sb, bb, hi, lo);
            e.cell[0][1][i] = hi; e.cell[1][1][i] = lo;
        }
    }
    __device__ static __forceinline__ uint32_t scales(const Raw &r) { return r.d; }
    __device__ static __forceinline__ u32x4 f16_cell(const Raw &, int) { return u32x4{0u, 0u, 0u, 0u}; }
    __device__ static __forceinline__ float value(int p0, int p1, const float (&)[2], uint32_t dd, int corr) {
        return __builtin_fmaf(h2f(dd), (float)((p0 << 6) + p1 + corr), 0.f);
    }
};

constexpr int KQ_PRODUCERS = 4;               // staging waves per workgroup, one per SIMD

template <int WT, int WR, int WC>
struct KqCfg {
    using T = KQ<WT>;
    static constexpr int NC = WR * WC;                             // MFMA waves
    static constexpr int NW = NC + KQ_PRODUCERS, NT = NW * 64;
    static constexpr int NPT = KQ_PRODUCERS * 64;                  // staging threads
    static constexpr int BM = 32 * WR;                             // weight rows per workgroup
    static constexpr int BN = 32 * KQ_TN * WC;                     // tokens per workgroup
    static constexpr int NF = T::NF16 > 0 ? T::NF16 : 1;
    // plane stride 2 mod 16 cells: the staging threads of one wave spread over the bank groups
    static constexpr int A_PLANE = BM + 2, B_PLANE = BN + 2;
    static constexpr int A_CELLS = KQ_NPL * KQ_KB * 2 * A_PLANE;   // 16-byte cells
    static constexpr int B_CELLS = KQ_KB * 2 * B_PLANE;
    // one stage buffer (two of them, by stage parity)
    static constexpr size_t OFF_A = 0;
    static constexpr size_t OFF_B = OFF_A + (size_t)A_CELLS * 16;
    static constexpr size_t STAGE = OFF_B + (size_t)B_CELLS * 16;
    // one super-block buffer (two of them, by super-block parity)
    static constexpr size_t OFF_FA = 0;                                     // fp16 cells [NF16][k-half][BM]: m_j (sc_j) twice
    static constexpr size_t OFF_FB = OFF_FA + (size_t)NF * 2 * BM * 16;     // fp16 cells [k-half][BN]: the token's 16 bsums
    static constexpr size_t OFF_SD = OFF_FB + (size_t)2 * BN * 16;          // u32 [BM]: d | dmin << 16, permuted per 32 rows
    static constexpr size_t OFF_SX = OFF_SD + (size_t)BM * 4;               // f32 [BN]: activation scale of the super-block
    static constexpr size_t OFF_SC = OFF_SX + (size_t)BN * 4;               // i32 [BN]: -4064 * sum of the token's quants
    static constexpr size_t SBLK = OFF_SC + (size_t)BN * 4;
    static constexpr size_t OFF_STAGES = 0;
    static constexpr size_t OFF_SBLK = 2 * STAGE;
    static constexpr size_t OFF_DUMP = OFF_SBLK + 2 * SBLK;                 // 16 bytes per staging thread: where stores that do not apply go
    static constexpr size_t TOTAL = OFF_DUMP + (size_t)NPT * 16;
    static constexpr int W_ITEMS = BM * 4;
    static constexpr int W_PER_T = W_ITEMS / NPT;
    static constexpr int X_ITEMS = BN * KQ_KB * 2;
    static constexpr int X_PER_T = X_ITEMS / NPT;
    static_assert(2 * BN <= NPT, "two staging threads per token convert its block sums");
    static_assert(W_ITEMS % NPT == 0 && X_ITEMS % NPT == 0, "staging items divide evenly over the staging threads");
    static_assert(STAGE % 16 == 0 && SBLK % 16 == 0, "buffers keep 16-byte alignment");
};

// A workgroup is WR x WC MFMA waves plus four staging waves (one per SIMD).  Per stage (4 k-blocks = half a
// super-block; LDS double buffered; one barrier per stage):
//
//     staging waves : global loads of stage s+3 | expand stage s+1 (loaded two stages ago) into the other buffer
//     MFMA waves    : 4 k-blocks of MFMAs from the current buffer | after a super-block's second half: fold
//
// The two kinds of wave run side by side on every SIMD, so operand expansion (vector pipe, LDS writes, memory
// latency) overlaps the matrix pipe by construction instead of by instruction scheduling.  Nothing in the loops is
// conditional: loads past the last stage repeat it, and stores that do not apply go to a per-thread dump slot.
template <int WT, int WR, int WC, int OCC, bool GATHER>
__global__ __launch_bounds__((WR * WC + KQ_PRODUCERS) * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void gemm_kq_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N, const uint8_t *__restrict__ ws,
                    size_t ws_stride, int64_t M, float *__restrict__ y, int64_t ldy, TileMap map, RowGather rg, int slice_sb) {
    using T = KQ<WT>;
    using C = KqCfg<WT, WR, WC>;
    constexpr int TN = KQ_TN;
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // split K (never with a gather, whose grid rows are the experts): grid row s takes super-blocks sb0 .. of every row
    // and writes its partial tile to slice s of y
    int sb0 = 0, nstages = (int)(K / QK_K) * 2;
    if (!GATHER && slice_sb > 0) {
        sb0 = (int)blockIdx.y * slice_sb;
        nstages = 2 * min(slice_sb, (int)(K / QK_K) - sb0);
        y += (size_t)blockIdx.y * (size_t)M * (size_t)ldy;
    }
    const TileCoord tc = xcd_tile(blockIdx.x, map);
    if (tc.row_tile >= map.row_tiles || tc.tok_tile >= map.tok_tiles) return;        // padding of the tile map
    size_t w_offset;
    const GatherView gv = resolve_gather<GATHER>(rg, w_offset, M);                   // MUL_MAT_ID: this expert's rows
    W += w_offset;
    const int64_t row_base = (int64_t)tc.row_tile * C::BM;
    if (gv.tok_tile < 0) return;
    const int64_t tok_base = (int64_t)(GATHER ? gv.tok_tile : tc.tok_tile) * C::BN;
    if (tok_base >= M) return;

    if (wave >= C::NC) {
        // ------------------------------------------------------------------------------------ staging waves
        const int pt = tid - C::NC * 64;
        const size_t off_d = q8_K_off_d(K), off_bs = q8_K_off_bsums(K);
        uint8_t *const dump = lds + C::OFF_DUMP + pt * 16;
        struct Acts {
            u32x4 x[C::X_PER_T];
            u32x4 bs;          // 8 of the token's bsums (threads 2*token + k-half)
            float xs;
            int xc;
        };
        struct Wts { typename T::Raw w[C::W_PER_T]; };
        Acts E, O;             // activations of an even / odd stage
        Wts W0, W1;            // weights of an even / odd super-block (both halves: every cache line is fetched once)
        // per-thread source addresses of stage 0 (they advance by a constant per stage / super-block)
        const uint8_t *wsrc[C::W_PER_T], *xsrc[C::X_PER_T];
#pragma unroll
        for (int i = 0; i < C::W_PER_T; i++) wsrc[i] = W + (size_t)min(row_base + ((pt + i * C::NPT) >> 2), N - 1) * nb01;
#pragma unroll
        for (int i = 0; i < C::X_PER_T; i++)
            xsrc[i] = ws + (size_t)gv.act_row(min(tok_base + ((pt + i * C::NPT) >> 3), M - 1)) * ws_stride + 16 * ((pt + i * C::NPT) & 7);
        // activation scale: thread t < BN for token t; block sums: thread t < 2*BN for token t/2, half t&1
        const uint8_t *ssrc = ws + (size_t)gv.act_row(min(tok_base + min(pt, C::BN - 1), M - 1)) * ws_stride;
        const uint8_t *bsrc = ws + (size_t)gv.act_row(min(tok_base + min(pt >> 1, C::BN - 1), M - 1)) * ws_stride + off_bs + 16 * (pt & 1);
        const int nsb = nstages >> 1;

        auto fetch_w = [&](Wts &R, int sb_wanted) {
            const int sb = min(sb_wanted, nsb - 1);
#pragma unroll
            for (int i = 0; i < C::W_PER_T; i++) T::fetch(R.w[i], wsrc[i] + (size_t)(sb0 + sb) * T::BYTES, (pt + i * C::NPT) & 3);
        };
        auto fetch_x = [&](Acts &R, int stage_wanted, auto even_tag) {
            constexpr bool even = decltype(even_tag)::value;
            const int stage = min(stage_wanted, nstages - 1);
            const int sb = stage >> 1;
#pragma unroll
            for (int i = 0; i < C::X_PER_T; i++) R.x[i] = *reinterpret_cast<const u32x4 *>(xsrc[i] + (size_t)(2 * sb0 + stage) * (32 * KQ_KB));
            if constexpr (even) {
                R.xs = reinterpret_cast<const float *>(ssrc + off_d)[sb0 + sb];
                if constexpr (T::NF16 > 0) R.bs = *reinterpret_cast<const u32x4 *>(bsrc + (size_t)(sb0 + sb) * 32);
                if constexpr (T::HAS_BSUM) {
                    const u32x4 *bp = reinterpret_cast<const u32x4 *>(ssrc + off_bs + (size_t)(sb0 + sb) * 32);
                    const u32x4 b0 = bp[0], b1 = bp[1];
                    const uint32_t w[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
                    int sum = 0;
#pragma unroll
                    for (int j = 0; j < 8; j++) sum += (int)(int16_t)(w[j] & 0xffffu) + ((int)w[j] >> 16);
                    R.xc = -Q6_BIAS * sum;
                }
            }
        };

        // expand a prefetched stage into LDS buffer `buf`; even stages also carry the super-block's scales
        auto commit = [&](const Wts &RW, const Acts &R, int buf, int sbp, auto even_tag) {
            constexpr bool even = decltype(even_tag)::value;
            constexpr int h = even ? 0 : 1;
            uint8_t *base = lds + C::OFF_STAGES + (size_t)buf * C::STAGE;
            uint8_t *sblk = lds + C::OFF_SBLK + (size_t)sbp * C::SBLK;
            u32x4 *A = reinterpret_cast<u32x4 *>(base + C::OFF_A);
            u32x4 *B = reinterpret_cast<u32x4 *>(base + C::OFF_B);
#pragma unroll
            for (int i = 0; i < C::W_PER_T; i++) {
                const int item = pt + i * C::NPT;
                const int r = item >> 2, x = item & 3, hf = x & 1;
                Emit e;
                T::emit(e, RW.w[i], h, x);
                const int k0 = T::kb0(x), k1 = T::kb1(x);
#pragma unroll
                for (int pl = 0; pl < KQ_NPL; pl++) {
                    A[((pl * KQ_KB + k0) * 2 + hf) * C::A_PLANE + r] = e.cell[pl][0];
                    A[((pl * KQ_KB + k1) * 2 + hf) * C::A_PLANE + r] = e.cell[pl][1];
                }
                if constexpr (even) {
                    // the lane that owns MFMA result register v of a 32-row tile holds row 8*(v/4) + 4*half + v%4:
                    // keep the scale of row i at half*16 + (i/8)*4 + i%4 so a lane reads its 16 scales contiguously
                    const int i32 = r & 31;
                    const int pos = ((i32 >> 2) & 1) * 16 + (i32 >> 3) * 4 + (i32 & 3);
                    uint8_t *dst = (x == 0) ? sblk + C::OFF_SD + ((r & ~31) + pos) * 4 : dump;
                    *reinterpret_cast<uint32_t *>(dst) = T::scales(RW.w[i]);
                    if constexpr (T::NF16 > 0) {
                        // items x < 2*NF16 of a row each build one fp16 operand cell [x/2][x&1][row]
                        uint8_t *fd = (x < 2 * T::NF16) ? sblk + C::OFF_FA + (size_t)(x * C::BM + r) * 16 : dump;
                        *reinterpret_cast<u32x4 *>(fd) = T::f16_cell(RW.w[i], x);
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < C::X_PER_T; i++) {
                const int item = pt + i * C::NPT;
                B[(item & 7) * C::B_PLANE + (item >> 3)] = R.x[i];
            }
            if constexpr (even) {
                uint8_t *dx = (pt < C::BN) ? sblk + C::OFF_SX + pt * 4 : dump;
                *reinterpret_cast<float *>(dx) = R.xs;
                if constexpr (T::HAS_BSUM) {
                    uint8_t *dc = (pt < C::BN) ? sblk + C::OFF_SC + pt * 4 : dump;
                    *reinterpret_cast<int *>(dc) = R.xc;
                }
                if constexpr (T::NF16 > 0) {
                    uint8_t *fb = (pt < 2 * C::BN) ? sblk + C::OFF_FB + (size_t)((pt & 1) * C::BN + (pt >> 1)) * 16 : dump;
                    *reinterpret_cast<u32x4 *>(fb) = i16x8_to_f16(R.bs);
                }
            }
        };

        // the two staging steps that run while the MFMA waves work on super-block j (weights in `cur`); `nxt` holds
        // super-block j + 1, and `cur` is refilled with super-block j + 2 once its second half has been expanded
        auto steps = [&](Wts &cur, Wts &nxt, int j) {
            fetch_x(E, 2 * j + 2, std::true_type{});
            commit(cur, O, 1, j & 1, std::false_type{});                  // stage 2j + 1, during stage 2j
            __syncthreads();
            fetch_x(O, 2 * j + 3, std::false_type{});
            fetch_w(cur, j + 2);
            commit(nxt, E, 0, (j + 1) & 1, std::true_type{});             // stage 2j + 2, during stage 2j + 1 and the fold
            __syncthreads();
        };

        fetch_w(W0, 0);
        fetch_x(E, 0, std::true_type{});
        fetch_x(O, 1, std::false_type{});
        fetch_w(W1, 1);
        commit(W0, E, 0, 0, std::true_type{});
        __syncthreads();
        for (int j = 0; j < nsb; j += 2) {
            steps(W0, W1, j);
            if (j + 1 < nsb) steps(W1, W0, j + 1);
        }
        return;
    }

    // ------------------------------------------------------------------------------------------ MFMA waves
    const int wr = wave / WC, wc = wave % WC;
    const int half = lane >> 5, l32 = lane & 31;
    const int r0 = wr * 32, n0 = wc * TN * 32;

    i32x16 P[KQ_NPL][TN];
    float out[TN][16];
#pragma unroll
    for (int c = 0; c < TN; c++)
#pragma unroll
        for (int v = 0; v < 16; v++) out[c][v] = 0.f;

    // 4 k-blocks of one stage; `first` starts the super-block's accumulators from zero
    auto compute = [&](int buf, auto first_tag) {
        constexpr bool first = decltype(first_tag)::value;
        const uint8_t *base = lds + C::OFF_STAGES + (size_t)buf * C::STAGE;
        const u32x4 *A = reinterpret_cast<const u32x4 *>(base + C::OFF_A);
        const u32x4 *B = reinterpret_cast<const u32x4 *>(base + C::OFF_B);
#pragma unroll
        for (int b = 0; b < KQ_KB; b++) {
            i32x4 af[KQ_NPL], bf[TN];
#pragma unroll
            for (int pl = 0; pl < KQ_NPL; pl++) {
                const u32x4 t = A[((pl * KQ_KB + b) * 2 + half) * C::A_PLANE + r0 + l32];
                af[pl] = i32x4{(int)t.x, (int)t.y, (int)t.z, (int)t.w};
            }
#pragma unroll
            for (int c = 0; c < TN; c++) {
                const u32x4 t = B[(b * 2 + half) * C::B_PLANE + n0 + c * 32 + l32];
                bf[c] = i32x4{(int)t.x, (int)t.y, (int)t.z, (int)t.w};
            }
#pragma unroll
            for (int pl = 0; pl < KQ_NPL; pl++)
#pragma unroll
                for (int c = 0; c < TN; c++) {
                    if (first && b == 0) {
                        const i32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                        P[pl][c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[pl], bf[c], zero, 0, 0, 0);
                    } else {
                        P[pl][c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[pl], bf[c], P[pl][c], 0, 0, 0);
                    }
                }
        }
    };

    // once per super-block: the fp16 products against the block sums, then fold the planes and apply d, dmin and
    // the activation scale
    auto fold = [&](int sbp) {
        const uint8_t *sblk = lds + C::OFF_SBLK + (size_t)sbp * C::SBLK;
        const u32x4 *sp = reinterpret_cast<const u32x4 *>(sblk + C::OFF_SD) + (r0 + half * 16) / 4;
        const u32x4 s0 = sp[0], s1 = sp[1], s2 = sp[2], s3 = sp[3];
        const uint32_t sd[16] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w, s2.x, s2.y, s2.z, s2.w, s3.x, s3.y, s3.z, s3.w};
        f16x8 fa[C::NF];
        if constexpr (T::NF16 > 0) {
#pragma unroll
            for (int f = 0; f < T::NF16; f++)
                fa[f] = *reinterpret_cast<const f16x8 *>(sblk + C::OFF_FA + (size_t)((2 * f + half) * C::BM + r0 + l32) * 16);
        }
#pragma unroll
        for (int c = 0; c < TN; c++) {
            f32x16 F[2];
            if constexpr (T::NF16 > 0) {
                const f16x8 fb = *reinterpret_cast<const f16x8 *>(sblk + C::OFF_FB + (size_t)(half * C::BN + n0 + c * 32 + l32) * 16);
                const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int f = 0; f < T::NF16; f++) F[f] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[f], fb, zero, 0, 0, 0);
            }
            const float dx = reinterpret_cast<const float *>(sblk + C::OFF_SX)[n0 + c * 32 + l32];
            int corr = 0;
            if constexpr (T::HAS_BSUM) corr = reinterpret_cast<const int *>(sblk + C::OFF_SC)[n0 + c * 32 + l32];
#pragma unroll
            for (int v = 0; v < 16; v++) {
                float f[2] = {0.f, 0.f};
#pragma unroll
                for (int j = 0; j < T::NF16; j++) f[j] = F[j][v];
                out[c][v] = __builtin_fmaf(T::value(P[0][c][v], P[1][c][v], f, sd[v], corr), dx, out[c][v]);
            }
        }
    };

    __syncthreads();                                                    // stage 0 is in LDS
    for (int s = 0; s < nstages; s += 2) {
        compute(0, std::true_type{});
        __syncthreads();
        compute(1, std::false_type{});
        fold((s >> 1) & 1);
        __syncthreads();
    }

    // ---- epilogue: register v of token tile c is row 8*(v/4) + 4*half + v%4, token l32 ----
#pragma unroll
    for (int c = 0; c < TN; c++) {
        const int64_t tok = tok_base + n0 + c * 32 + l32;
        if (tok >= M) continue;
        const int64_t orow = gv.out_row(tok);
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int64_t row = row_base + r0 + 8 * g + 4 * half;
            float *dst = y + (size_t)orow * ldy + row;
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

// ---- Q4_K and Q5_K at prefill sizes: one int8 plane, sub-block scales applied by the vector unit ----
// The two digit planes above cost two MFMAs per 32 values.  Measured, an MFMA is worth more time (and power: these kernels
// run clock-limited) than the 16 integer multiply-adds that apply a sub-block scale to its 16 results per lane.  So this
// kernel feeds the quants themselves (Q4_K: 0..15, Q5_K: q - 16) as one plane: every MFMA result is the reference's
// per-sub-block integer dot, and   sumi += isum_j * sc_j   is one v_mad_i32_i24 per result.  The activations are the MFMA's
// first operand and the weights its second, so a lane owns one weight row and its 16 result registers 16 tokens: the
// sub-block scale, d and dmin are one register per lane (no scale vectors from LDS), and a store instruction writes 32
// consecutive rows of a token.  Per super-block the fold is, per output,  out += dx * (d * float(sumi) - dmin * summ)
// with summ (and Q5_K's sum_j sc_j * bsum_j) from one fp16 MFMA as above: the same operations in the same order as
// gemm_kq_kernel, so the outputs are bit-identical to it.
// Skeleton as the block-32 kernel's: activations straight into swizzled LDS rows with global_load_lds_dwordx4, weights
// through registers (a thread fetches its (row, x) item of a whole super-block during the super-block before and every
// stage begins by expanding the next stage's half into the idle buffer), the MFMA of tile i + 1 issued before the 16
// multiply-adds of tile i, two 4-wave workgroups per CU.
template <int WT> struct KS;
template <> struct KS<T_Q4_K> {
    // 16 quant bytes -> the 16-value k-half of sub-blocks 2jp (low nibbles) and 2jp + 1 (high nibbles)
    __device__ static __forceinline__ void emit(const KQ<T_Q4_K>::Raw &r, int h, int, u32x4 &c0, u32x4 &c1) {
        const u32x4 q = r.q[h];
#pragma unroll
        for (int i = 0; i < 4; i++) { c0[i] = q[i] & 0x0f0f0f0fu; c1[i] = (q[i] >> 4) & 0x0f0f0f0fu; }
    }
};
template <> struct KS<T_Q5_K> {
    // q - 16 as a signed byte: (q + 112) ^ 128 (q + 112 <= 143: no carries between bytes)
    __device__ static __forceinline__ void emit(const KQ<T_Q5_K>::Raw &r, int h, int x, u32x4 &c0, u32x4 &c1) {
        const int jp = 2 * h + (x >> 1);
        const u32x4 q = r.q[h];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t hb = r.qh[i] >> (2 * jp);
            const uint32_t lo = (q[i] & 0x0f0f0f0fu) | ((hb << 4) & 0x10101010u);
            const uint32_t hi = ((q[i] >> 4) & 0x0f0f0f0fu) | ((hb << 3) & 0x10101010u);
            c0[i] = (lo + 0x70707070u) ^ 0x80808080u;
            c1[i] = (hi + 0x70707070u) ^ 0x80808080u;
        }
    }
};

template <int WT, int TM, int TN, int WR, int WC>
struct KsCfg {
    using T = KQ<WT>;
    static constexpr int NW = WR * WC, NT = NW * 64;
    static constexpr int BM = 32 * TM * WR, BN = 32 * TN * WC;
    static constexpr int A_PLANE = BM + 2;
    static constexpr size_t OFF_A = 0;                                               // [k-block][half][row] cells
    static constexpr size_t OFF_B = OFF_A + (size_t)KQ_KB * 2 * A_PLANE * 16;        // [token][8 cells], swizzled
    static constexpr size_t STAGE = OFF_B + (size_t)BN * 128;
    // one super-block buffer: written while half 0 is multiplied, read by the scaling of both halves and by the fold
    static constexpr size_t OFF_FA = 0;                                              // fp16 cells [NF16][k-half][BM]
    static constexpr size_t OFF_FB = OFF_FA + (size_t)T::NF16 * 2 * BM * 16;         // fp16 cells [k-half][BN]: the 16 bsums
    static constexpr size_t OFF_SC = OFF_FB + (size_t)2 * BN * 16;                   // i32 [8][BM]: sub-block scales
    static constexpr size_t OFF_SD = OFF_SC + (size_t)8 * BM * 4;                    // u32 [BM]: d | dmin << 16
    static constexpr size_t OFF_SX = OFF_SD + (size_t)BM * 4;                        // f32 [BN]: activation scale
    static constexpr size_t SBLK = OFF_SX + (size_t)BN * 4;
    static constexpr size_t OFF_SBLK = 2 * STAGE;
    static constexpr size_t TOTAL = OFF_SBLK + 2 * SBLK;                             // two: the next super-block's is written during half 1
    static constexpr int W_ITEMS = BM * 4, W_PER_T = W_ITEMS / NT;
    static constexpr int B_INSTR = BN / 8, B_PER_W = B_INSTR / NW;
    static_assert(W_ITEMS % NT == 0 && W_PER_T >= 1, "the weight items divide evenly over the threads");
    static_assert(B_INSTR % NW == 0 && B_PER_W >= 1, "the activation loads divide evenly over the waves");
    static_assert(2 * BN <= NT, "two threads per token convert its block sums");
    static_assert(STAGE % 16 == 0 && SBLK % 16 == 0, "buffers keep 16-byte alignment");
};

__device__ __forceinline__ void kq_load16_into_lds(const uint8_t *src, uint32_t lds_addr) {
    // M0 = LDS byte address of the wave's 1 KB destination; lane i's 16 bytes land at M0 + 16 i.  Inline assembly so that
    // the compiler does not make every later LDS read wait for it; the kernel waits by hand in front of the stage barrier.
    // Nothing else in the kernel may use M0 (no dynamic register indexing).
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_addr) : "memory");
}

template <int WT, int TM, int TN, int WR, int WC, int OCC, bool GATHER>
__global__ __launch_bounds__(WR *WC * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void gemm_ks_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N, const uint8_t *__restrict__ ws,
                    size_t ws_stride, int64_t M, float *__restrict__ y, int64_t ldy, TileMap map, RowGather rg, int slice_sb) {
    using T = KQ<WT>;
    using C = KsCfg<WT, TM, TN, WR, WC>;
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int sb0 = 0, nsb = (int)(K / QK_K);
    if (!GATHER && slice_sb > 0) {
        sb0 = (int)blockIdx.y * slice_sb;
        nsb = min(slice_sb, nsb - sb0);
        y += (size_t)blockIdx.y * (size_t)M * (size_t)ldy;
    }
    const TileCoord tc = xcd_tile(blockIdx.x, map);
    if (tc.row_tile >= map.row_tiles || tc.tok_tile >= map.tok_tiles) return;
    size_t w_offset;
    const GatherView gv = resolve_gather<GATHER>(rg, w_offset, M);
    W += w_offset;
    const int64_t row_base = (int64_t)tc.row_tile * C::BM;
    if (gv.tok_tile < 0) return;
    const int64_t tok_base = (int64_t)(GATHER ? gv.tok_tile : tc.tok_tile) * C::BN;
    if (tok_base >= M) return;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
    const size_t off_d = q8_K_off_d(K), off_bs = q8_K_off_bsums(K);

    // ---- this thread's share of the staging ----
    const uint8_t *wsrc[C::W_PER_T];
#pragma unroll
    for (int i = 0; i < C::W_PER_T; i++) wsrc[i] = W + (size_t)min(row_base + ((tid + i * C::NT) >> 2), N - 1) * nb01 + (size_t)sb0 * T::BYTES;
    const uint8_t *bsrc[C::B_PER_W];
#pragma unroll
    for (int j = 0; j < C::B_PER_W; j++) {
        const int t = (wave * C::B_PER_W + j) * 8 + (lane >> 3);
        const int cell = (lane & 7) ^ ((t >> 1) & 7);
        bsrc[j] = ws + (size_t)gv.act_row(min(tok_base + t, M - 1)) * ws_stride + (size_t)sb0 * QK_K + 16 * cell;
    }
    // activation scale: thread t < BN for token t; block sums: thread t < 2*BN for token t/2, k-half t&1
    const uint8_t *ssrc = ws + (size_t)gv.act_row(min(tok_base + min(tid, C::BN - 1), M - 1)) * ws_stride + off_d + (size_t)sb0 * 4;
    const uint8_t *bssrc = ws + (size_t)gv.act_row(min(tok_base + min(tid >> 1, C::BN - 1), M - 1)) * ws_stride + off_bs + 16 * (tid & 1) + (size_t)sb0 * 32;

    typename T::Raw wq[C::W_PER_T];
    u32x4 bs;
    float xs;
    auto fetch_sb = [&](int sb_wanted) {
        const int sb = min(sb_wanted, nsb - 1);
#pragma unroll
        for (int i = 0; i < C::W_PER_T; i++) T::fetch(wq[i], wsrc[i] + (size_t)sb * T::BYTES, (tid + i * C::NT) & 3);
        xs = reinterpret_cast<const float *>(ssrc)[sb];
        bs = *reinterpret_cast<const u32x4 *>(bssrc + (size_t)sb * 32);
    };
    auto issue_direct = [&](int stage_wanted, uint32_t buf_off) {
        const int stage = min(stage_wanted, 2 * nsb - 1);
#pragma unroll
        for (int j = 0; j < C::B_PER_W; j++)
            kq_load16_into_lds(bsrc[j] + (size_t)stage * (32 * KQ_KB),
                               __builtin_amdgcn_readfirstlane(lds0 + buf_off + (uint32_t)C::OFF_B + (uint32_t)(wave * C::B_PER_W + j) * 1024u));
    };
    // expand half H of the fetched super-block into the stage buffer at buf_off; with H = 0 also write that super-block's
    // scales, fp16 cells and activation sums into super-block buffer sbp
    auto commit = [&](uint32_t buf_off, int sbp, auto half_tag) {
        constexpr int h = decltype(half_tag)::value ? 1 : 0;
        uint8_t *base = lds + buf_off;
        uint8_t *sblk = lds + C::OFF_SBLK + (size_t)sbp * C::SBLK;
        u32x4 *A = reinterpret_cast<u32x4 *>(base + C::OFF_A);
#pragma unroll
        for (int i = 0; i < C::W_PER_T; i++) {
            const int item = tid + i * C::NT;
            const int r = item >> 2, x = item & 3, hf = x & 1;
            u32x4 c0, c1;
            KS<WT>::emit(wq[i], h, x, c0, c1);
            A[(T::kb0(x) * 2 + hf) * C::A_PLANE + r] = c0;
            A[(T::kb1(x) * 2 + hf) * C::A_PLANE + r] = c1;
            if constexpr (h == 0) {
                uint32_t sc, mn;
                scale_min_pair(wq[i].hdr, x, sc, mn);                                      // sub-blocks 2x and 2x + 1
                int *SC = reinterpret_cast<int *>(sblk + C::OFF_SC);
                SC[(2 * x) * C::BM + r] = (int)(sc & 0xffu);
                SC[(2 * x + 1) * C::BM + r] = (int)(sc >> 8);
                if (x == 0) reinterpret_cast<uint32_t *>(sblk + C::OFF_SD)[r] = T::scales(wq[i]);
                // items x < 2*NF16 of a row each build one fp16 operand cell [x/2][x&1][row]
                if (x < 2 * T::NF16) *reinterpret_cast<u32x4 *>(sblk + C::OFF_FA + (size_t)(x * C::BM + r) * 16) = T::f16_cell(wq[i], x);
            }
        }
        if constexpr (h == 0) {
            if (tid < C::BN) reinterpret_cast<float *>(sblk + C::OFF_SX)[tid] = xs;
            if (tid < 2 * C::BN) *reinterpret_cast<u32x4 *>(sblk + C::OFF_FB + (size_t)((tid & 1) * C::BN + (tid >> 1)) * 16) = i16x8_to_f16(bs);
        }
    };

    // ---- this wave's tiles: register v of tile (a, c) is token n0 + 32 c + 8 (v / 4) + 4 half + v % 4, row r0 + 32 a + l32 ----
    const int wr = wave / WC, wc = wave % WC;
    const int half = lane >> 5, l32 = lane & 31;
    const int r0 = wr * TM * 32, n0 = wc * TN * 32;
    const uint32_t a_rd = (uint32_t)C::OFF_A + (uint32_t)(half * C::A_PLANE + r0 + l32) * 16u;
    uint32_t b_rd[KQ_KB];
#pragma unroll
    for (int b = 0; b < KQ_KB; b++) b_rd[b] = (uint32_t)C::OFF_B + (uint32_t)(n0 + l32) * 128u + 16u * (uint32_t)((2 * b + half) ^ ((l32 >> 1) & 7));

    int sumi[TM][TN][16];
    float out[TM][TN][16];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int c = 0; c < TN; c++)
#pragma unroll
            for (int v = 0; v < 16; v++) { out[a][c][v] = 0.f; sumi[a][c][v] = 0; }

    // one stage (half H of a super-block whose scales sit in super-block buffer sbp) from the buffer at byte offset BUF
    auto compute = [&](auto buf_tag, auto half_tag, int sbp) {
        constexpr uint32_t BUF = decltype(buf_tag)::value ? (uint32_t)C::STAGE : 0u;
        constexpr int h = decltype(half_tag)::value ? 1 : 0;
        const uint8_t *base = lds + BUF;
        const int *SC = reinterpret_cast<const int *>(lds + C::OFF_SBLK + (size_t)sbp * C::SBLK + C::OFF_SC);
        i32x4 af[2][TM], bf[2][TN];
        int sc[KQ_KB][TM];
        auto load_operands = [&](int b, int slot) {
#pragma unroll
            for (int a = 0; a < TM; a++) {
                const u32x4 t = *reinterpret_cast<const u32x4 *>(base + a_rd + (b * 2 * C::A_PLANE + a * 32) * 16);
                af[slot][a] = i32x4{(int)t.x, (int)t.y, (int)t.z, (int)t.w};
            }
#pragma unroll
            for (int c = 0; c < TN; c++) {
                const u32x4 t = *reinterpret_cast<const u32x4 *>(base + b_rd[b] + c * 4096);
                bf[slot][c] = i32x4{(int)t.x, (int)t.y, (int)t.z, (int)t.w};
            }
        };
#pragma unroll
        for (int b = 0; b < KQ_KB; b++)
#pragma unroll
            for (int a = 0; a < TM; a++) sc[b][a] = SC[(4 * h + b) * C::BM + r0 + a * 32 + l32];
        constexpr int TILES = TM * TN;
        const i32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        load_operands(0, 0);
        i32x16 d_cur = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[0][0], af[0][0], zero, 0, 0, 0);
#pragma unroll
        for (int b = 0; b < KQ_KB; b++) {
            const int slot = b & 1;
            if (b + 1 < KQ_KB) load_operands(b + 1, slot ^ 1);
#pragma unroll
            for (int i = 0; i < TILES; i++) {
                const int a = i / TN, c = i % TN;
                i32x16 d_next = d_cur;
                if (i + 1 < TILES) d_next = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[slot][(i + 1) % TN], af[slot][(i + 1) / TN], zero, 0, 0, 0);
                else if (b + 1 < KQ_KB) d_next = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[slot ^ 1][0], af[slot ^ 1][0], zero, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);                    // the MFMA goes first: it runs behind the multiply-adds below
                // The first result of a stage is read right behind its MFMA: the compiler does not place the wait states
                // that a vector read of a fresh MFMA result needs in front of inline assembly, so they are written out
                // (later results are a whole group of multiply-adds old when they are read).
                if (b == 0 && i == 0) asm volatile("s_nop 15\n\ts_nop 7");
                // Inline assembly pins the multiply-adds here: as plain arithmetic the compiler gathers the stage's MFMAs in
                // front and moves the multiply-adds behind the stage barrier, with every result register live in between.
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    if (h == 0 && b == 0) asm volatile("v_mul_i32_i24 %0, %1, %2" : "=v"(sumi[a][c][v]) : "v"(d_cur[v]), "v"(sc[b][a]));
                    else asm volatile("v_mad_i32_i24 %0, %1, %2, %0" : "+v"(sumi[a][c][v]) : "v"(d_cur[v]), "v"(sc[b][a]));
                }
                d_cur = d_next;
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    // once per super-block: out += dx * (d * float(sumi) - dmin * summ), the operations of KQ<WT>::value in their order
    auto fold = [&](int sbp) {
        const uint8_t *sblk = lds + C::OFF_SBLK + (size_t)sbp * C::SBLK;
#pragma unroll
        for (int a = 0; a < TM; a++) {
            const uint32_t dd = reinterpret_cast<const uint32_t *>(sblk + C::OFF_SD)[r0 + a * 32 + l32];
            f16x8 fa[T::NF16];
#pragma unroll
            for (int f = 0; f < T::NF16; f++)
                fa[f] = *reinterpret_cast<const f16x8 *>(sblk + C::OFF_FA + (size_t)((2 * f + half) * C::BM + r0 + a * 32 + l32) * 16);
#pragma unroll
            for (int c = 0; c < TN; c++) {
                const f16x8 fb = *reinterpret_cast<const f16x8 *>(sblk + C::OFF_FB + (size_t)(half * C::BN + n0 + c * 32 + l32) * 16);
                const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                f32x16 F[T::NF16];
#pragma unroll
                for (int f = 0; f < T::NF16; f++) F[f] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb, fa[f], zero, 0, 0, 0);
                float dx[16];
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const float4 t = *reinterpret_cast<const float4 *>(sblk + C::OFF_SX + (size_t)(n0 + c * 32 + 8 * g + 4 * half) * 4);
                    dx[4 * g] = t.x; dx[4 * g + 1] = t.y; dx[4 * g + 2] = t.z; dx[4 * g + 3] = t.w;
                }
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    float f[2] = {0.f, 0.f};
#pragma unroll
                    for (int j = 0; j < T::NF16; j++) f[j] = F[j][v];
                    out[a][c][v] = __builtin_fmaf(T::value(0, sumi[a][c][v], f, dd, 0), dx[v], out[a][c][v]);
                }
            }
        }
    };

    // Stage 2j is half 0 of super-block j, stage 2j + 1 its half 1.  Every stage begins by expanding the following stage
    // into the idle buffer (an odd stage's expansion is half 0 of the next super-block and carries that super-block's
    // scales into the other super-block buffer); after an even stage's expansion the registers are free and the next
    // super-block is fetched into them.  Then the following stage's activations are requested, then the stage is
    // multiplied.  In front of the barrier a wave waits for all its loads: they were issued a stage ago.
    constexpr int WAIT0 = 0x0F70;                                          // s_waitcnt vmcnt(0)
    fetch_sb(0);
    issue_direct(0, 0u);
    commit(0u, 0, std::false_type{});
    __builtin_amdgcn_s_waitcnt(WAIT0);
    __syncthreads();
    for (int j = 0; j < nsb; j++) {
        commit((uint32_t)C::STAGE, 0, std::true_type{});                     // half 1 of super-block j
        issue_direct(2 * j + 1, (uint32_t)C::STAGE);
        fetch_sb(j + 1);
        compute(std::false_type{}, std::false_type{}, j & 1);                // stage 2j from buffer 0
        __builtin_amdgcn_s_waitcnt(WAIT0);
        __syncthreads();
        commit(0u, (j + 1) & 1, std::false_type{});                          // half 0 of super-block j + 1 and its scales
        issue_direct(2 * j + 2, 0u);
        compute(std::true_type{}, std::true_type{}, j & 1);                  // stage 2j + 1 from buffer 1
        fold(j & 1);
        __builtin_amdgcn_s_waitcnt(WAIT0);
        __syncthreads();
    }

#pragma unroll
    for (int a = 0; a < TM; a++) {
        const int64_t row = row_base + r0 + a * 32 + l32;
        if (row >= N) continue;
#pragma unroll
        for (int c = 0; c < TN; c++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int64_t tok = tok_base + n0 + c * 32 + 8 * (v >> 2) + 4 * half + (v & 3);
                if (tok < M) y[(size_t)gv.out_row(tok) * ldy + row] = out[a][c][v];
            }
        }
    }
}

// With few tokens the GEMM's time is its walk over K (about 1.5 - 2 us per super-block, whatever the token count:
// 28 - 35 us at K = 4096, 88 - 112 us at K = 14336), while the GEMV forms pass over the weights once per 8 or 16 tokens at
// memory speed.  Up to 128 tokens on a matrix with few row tiles the walk is cut into slices (kq_slices_for below:
// 16 - 19 us at K = 4096, 36 - 41 us at K = 14336).  The token count from which the GEMM is ahead, measured on 4096 x 4096,
// 14336 x 4096 (too many row tiles to split) and 4096 x 14336:
static bool kq_splittable(int64_t N) { return ceil_div(N, (int64_t)64) <= 128; }
static int64_t gemm_kq_min_tokens(int wtype, int64_t K, int64_t N, bool can_split) {
    if (can_split || !kq_splittable(N)) {
        if (wtype == T_Q6_K) return 9;                               // its GEMV passes take 8 tokens
        return kq_splittable(N) ? 17 : 33;                           // Q4_K, Q5_K: passes of 16 tokens
    }
    // the caller's workspace has no room for the partial outputs: the unsplit walk
    const bool long_rows = K > 8192;
    switch (wtype) {
        case T_Q4_K: return long_rows ? 33 : 49;
        case T_Q5_K: return long_rows ? 33 : 49;
        default:     return long_rows ? 41 : 25;
    }
}
bool gemm_kq_supported(int wtype, int64_t K, int64_t N, int64_t n, bool can_split) {
    if (!(wtype == T_Q4_K || wtype == T_Q5_K || wtype == T_Q6_K) || K < QK_K || K % QK_K != 0 || N < 1) return false;
    const int64_t forced = tune("CHIP_GEMM_MIN_TOKENS", 0);
    if (forced > 0) return n >= forced;
    return n >= gemm_kq_min_tokens(wtype, K, N, can_split);
}

// Slices of K for the 64 x 128 shape: up to two workgroups per CU with one token tile, one per CU with more (the partial
// outputs grow with the token count), at least four super-blocks each.
static int kq_slices_for(int64_t K, int64_t N, int64_t M, int64_t cus) {
    const int forced = (int)tune("CHIP_GEMM_SLICES", 0);
    const int64_t units = K / QK_K, tiles = ceil_div(N, (int64_t)64) * ceil_div(M, (int64_t)128);
    if (forced > 0) {
        const int64_t per = ceil_div(units, (int64_t)(forced < units ? forced : units));
        return (int)ceil_div(units, per);
    }
    if (units < 8 || (M <= 128 && !kq_splittable(N))) return 1;
    int64_t s = (M <= 128 ? 2 : 1) * cus / tiles;
    if (s > units / 4) s = units / 4;
    if (s > 16) s = 16;
    if (s < 2) return 1;
    const int64_t per = ceil_div(units, s);
    return (int)ceil_div(units, per);                                   // no empty slice
}
int gemm_kq_slices(int wtype, int64_t K, int64_t N, int64_t n, int compute_units) {
    if (!gemm_kq_supported(wtype, K, N, n, true)) return 1;
    return kq_slices_for(K, N, n, compute_units > 0 ? compute_units : 256);
}

template <int WT, int WR, int WC, int OCC, bool GATHER>
static hipError_t launch_kq(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int64_t M,
                            float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const RowGather &rg, int64_t n_as,
                            int slices = 1, float *part = nullptr) {
    using C = KqCfg<WT, WR, WC>;
    const size_t lds_bytes = C::TOTAL;
    if ((int64_t)lds_bytes > lim.max_lds_per_block) return hipErrorInvalidValue;
    auto kfn = gemm_kq_kernel<WT, WR, WC, OCC, GATHER>;
    static LdsGrant grant;                                               // one per kernel instantiation
    if (hipError_t e = grant_dynamic_lds(kfn, lds_bytes, lim, grant); e != hipSuccess) return e;
    // one workgroup per CU: 32 workgroups run on an XCD at a time
    const TileMap map = make_tile_map(ceil_div(N, C::BM), GATHER ? 1 : ceil_div(M, C::BN), 32);
    if (!GATHER && slices > 1) {
        const int slice_sb = (int)ceil_div(K / QK_K, (int64_t)slices);
        hipLaunchKernelGGL(kfn, dim3(map.grid, (unsigned)slices), dim3(C::NT), lds_bytes, st, (const uint8_t *)W, nb01, K, N,
                           (const uint8_t *)ws, ws_stride, M, part, N, map, rg, slice_sb);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
        return launch_sum_slices(part, slices, M, N, y, ldy, st);
    }
    hipLaunchKernelGGL(kfn, dim3(map.grid, (unsigned)n_as), dim3(C::NT), lds_bytes, st, (const uint8_t *)W, nb01, K, N,
                       (const uint8_t *)ws, ws_stride, M, y, ldy, map, rg, 0);
    return hipGetLastError();
}

template <int WT, int TM, int TN, int WR, int WC, int OCC, bool GATHER>
static hipError_t launch_ks(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int64_t M,
                            float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const RowGather &rg, int64_t n_as,
                            int slices = 1, float *part = nullptr) {
    if constexpr (WT == T_Q6_K) return hipErrorInvalidValue;
    else {
        using C = KsCfg<WT, TM, TN, WR, WC>;
        const size_t lds_bytes = C::TOTAL;
        if ((int64_t)lds_bytes > lim.max_lds_per_block) return hipErrorInvalidValue;
        auto kfn = gemm_ks_kernel<WT, TM, TN, WR, WC, OCC, GATHER>;
        static LdsGrant grant;
        if (hipError_t e = grant_dynamic_lds(kfn, lds_bytes, lim, grant); e != hipSuccess) return e;
        const int per_cu = lds_bytes > 80 * 1024 ? 1 : 2;
        const TileMap map = make_tile_map(ceil_div(N, C::BM), GATHER ? 1 : ceil_div(M, C::BN), 32 * per_cu);
        if (!GATHER && slices > 1) {
            const int slice_sb = (int)ceil_div(K / QK_K, (int64_t)slices);
            hipLaunchKernelGGL(kfn, dim3(map.grid, (unsigned)slices), dim3(C::NT), lds_bytes, st, (const uint8_t *)W, nb01, K, N,
                               (const uint8_t *)ws, ws_stride, M, part, N, map, rg, slice_sb);
            if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
            return launch_sum_slices(part, slices, M, N, y, ldy, st);
        }
        hipLaunchKernelGGL(kfn, dim3(map.grid, (unsigned)n_as), dim3(C::NT), lds_bytes, st, (const uint8_t *)W, nb01, K, N,
                           (const uint8_t *)ws, ws_stride, M, y, ldy, map, rg, 0);
        return hipGetLastError();
    }
}

template <int WT>
static hipError_t launch_kq_type(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                                 int64_t M, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const RowGather &rg,
                                 int64_t n_as, SplitK split) {
    const int64_t cus = lim.compute_units > 0 ? lim.compute_units : 256;
    if (!rg.perm && split.part) {
        const int slices = kq_slices_for(K, N, M, cus);
        if (slices > 1 && split.bytes >= (size_t)slices * (size_t)M * (size_t)N * sizeof(float) && (((uintptr_t)split.part) & 15) == 0)
            return launch_kq<WT, 2, 2, 2, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, slices, split.part);
    }
    // 128 rows x 128 tokens per workgroup when that gives every CU one, else 64 x 128.
    if (rg.perm)                                                                     // expert groups: 64 x 128 tiles
        return launch_kq<WT, 2, 2, 2, true>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);
    // Q4_K and Q5_K with enough 64 x 128 tiles to give every CU its two workgroups more than once: the single-plane kernel.
    // Measured (us, K = 4096, tokens x rows; two-plane kernel -> single plane): Q4_K 2048 x 14336 432 -> 385, 2048 x 4096
    // 118 -> 108, 512 x 4096 36 -> 39 (stays); Q5_K 553 -> 455, 150 -> 125, 43 -> 42; Q4_K 512 x 4096 with K = 14336 107 -> 124 (stays).
    const int64_t g128 = ceil_div(N, 128) * ceil_div(M, 128), g64x128 = ceil_div(N, 64) * ceil_div(M, 128);
    const bool single_plane = WT != T_Q6_K && g64x128 >= (WT == T_Q5_K ? 1 : 2) * cus;
    const int cfg = (int)tune("CHIP_GEMM_KQ_CFG", single_plane ? 11 : g128 >= cus ? 0 : 2);
    switch (cfg) {
        case 0: return launch_kq<WT, 4, 2, 3, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);      // 128 x 128, 8 + 4 waves
        case 1: return launch_kq<WT, 4, 1, 2, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);      // 128 x 64, 4 + 4 waves
        case 2: return launch_kq<WT, 2, 2, 2, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);      // 64 x 128, 4 + 4 waves
        case 11: return launch_ks<WT, 1, 2, 2, 2, 2, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);   // single plane, 64 x 128, 4 waves
        default: return hipErrorInvalidValue;
    }
}

int gemm_kq_moe_tile_tokens() { return KqCfg<T_Q4_K, 2, 2>::BN; }      // the 64 x 128 shape serves the expert groups

hipError_t launch_gemm_kq(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                          int64_t M, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const RowGather *rgp, int64_t n_as,
                          SplitK split) {
    if (M <= 0 || N <= 0 || n_as <= 0) return hipSuccess;
    const RowGather rg = rgp ? *rgp : RowGather{nullptr, nullptr, nullptr, 1, 1, 0};
    switch (wtype) {
        case T_Q4_K: return launch_kq_type<T_Q4_K>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, split);
        case T_Q5_K: return launch_kq_type<T_Q5_K>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, split);
        case T_Q6_K: return launch_kq_type<T_Q6_K>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, split);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace chip
