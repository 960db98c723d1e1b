// Multi-token GEMV on the matrix cores for Q4_K and Q5_K weights, 5..16 tokens: the Q8_0 kernel's structure (gemv_mfma.hip)
// with the K-quant arithmetic of lm_ggml_vec_dot_q4_K_q8_K (reference ggml-cpu/ggml-cpu-quants.c:6772-7085) as driven by
// lm_ggml_compute_forward_mul_mat (ggml-cpu/ggml-cpu.c:1257-1449):
//
//   y[t][r] = sum over super-blocks b of  d[r][b] * dx[t][b] * sum_j sc[r][b][j] * isum[t][r][b][j]
//                                       - dmin[r][b] * dx[t][b] * sum_j m[r][b][j] * bsum[t][b][j]
//
// with j the eight 32-value sub-blocks, isum the integer dot of the 4-bit quants with the Q8_K quants and bsum the sum of
// the 32 activation quants (block_q8_K.bsums, two per sub-block).  Both inner sums are integers and are accumulated as
// integers, so they are exact; the fp32 part is two fused multiply-adds per super-block and (row, token).
//
// One v_mfma_i32_16x16x64_i8 covers 64 values of 16 rows: the 32 bytes qs[32p .. 32p+31] of a super-block hold sub-block
// 2p in their low nibbles and sub-block 2p+1 in their high nibbles.  Lane (x = lane % 16, g = lane / 16) of the weight
// operand holds 16 values of row x: the low (g < 2) or high (g >= 2) nibbles of bytes 32p + 16(g & 1) ... + 15, which puts
// sub-block 2p into k = 0..31 and sub-block 2p+1 into k = 32..63, the order of the activation quants.  The two
// sub-blocks have different scales, so their sums are separated as in the Q8_0 kernel: with 9..16 tokens the activation
// operand is issued twice with the other half of the lane groups zeroed; with 8 tokens or fewer rows 8..15 of the
// operand carry the same tokens again, rows 0..7 real only in the lane groups of sub-block 2p and rows 8..15 only in
// those of sub-block 2p+1, and one MFMA returns both.
//
// A wave fetches a macro tile of 16 rows x 144 bytes (one super-block per row) with row-contiguous 16-byte loads,
// passes it through a private LDS buffer and reads header and operands back from there; the next macro tile's loads
// are in flight meanwhile.  Bound: the weight stream (HBM).
#include "kernels.h"
#include "dev_common.h"
#include "act_layout.h"
#include <cstdlib>
#include <type_traits>

namespace chip {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

// Q4_K: 144-byte super-blocks = 9 chunks of 16 bytes: d | dmin | scales[12] | qs[128].
// Q5_K: 176 bytes = 11 chunks: d | dmin | scales[12] | qh[32] | qs[128]; bit j of qh[l] is the fifth bit of element l of
// sub-block j, so the operand byte is nibble + 16 * bit and everything after the operand is the same as for Q4_K
// (lm_ggml_vec_dot_q5_K_q8_K, reference ggml-cpu/ggml-cpu-quants.c:7699-8150).
template <int WT> struct KqGeom {
    static constexpr int ROW_BYTES = WT == T_Q5_K ? BYTES_Q5_K : BYTES_Q4_K;
    static constexpr int CHUNKS_PER_ROW = ROW_BYTES / 16;
    static constexpr int MACRO_BYTES = 16 * ROW_BYTES;          // per wave; also holds the wave's partial sums
    static constexpr int CHUNKS = MACRO_BYTES / 16;             // 144 or 176: three loads per lane
    static constexpr int QS_OFF = WT == T_Q5_K ? 48 : 16;
    static_assert(ROW_BYTES % 16 == 0 && CHUNKS <= 192 && MACRO_BYTES >= 2048, "macro tile geometry");
};

// LDS: quant image [NT tokens][K + 16] bytes | dx image [K/256][16 tokens] float | bsum image [K/32][16 tokens] int32 |
// 256 zero bytes | [NW waves] macro-tile buffers
template <int WT, int NT, int NW> __host__ __device__ constexpr size_t mmv_q4k_lds_bytes(int64_t K) {
    return (size_t)(K + 16) * NT + (size_t)(K / 256) * 64 + (size_t)(K / 32) * 64 + 256 + NW * (size_t)KqGeom<WT>::MACRO_BYTES;
}

template <int WT, int NT, int NW, int OCC>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void mmv_q4k_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N, const uint8_t *__restrict__ ws,
                    size_t ws_stride, int n, float *__restrict__ y, int64_t ldy, const uint8_t *__restrict__ W2,
                    float *__restrict__ y2) {
    // Two matrices of one shape on the same activation rows (ffn_gate and ffn_up): after its tiles of W / y a workgroup
    // takes the same tile range of W2 / y2, so either result is what a launch of its own returns and the activation
    // image is built once.
    const uint32_t grid = gridDim.x, block = blockIdx.x;
    const int nmat = W2 ? 2 : 1;
    constexpr int WGS = NW * 64;
    constexpr int KQ_ROW_BYTES = KqGeom<WT>::ROW_BYTES, KQ_MACRO_BYTES = KqGeom<WT>::MACRO_BYTES, KQ_CHUNKS = KqGeom<WT>::CHUNKS;
    constexpr int CPR = KqGeom<WT>::CHUNKS_PER_ROW;
    extern __shared__ __align__(16) uint8_t lds[];
    const int np = (int)(K / 256);                                      // macro steps (super-blocks) per row
    const uint32_t q_stride = (uint32_t)K + 16u, q_bytes = q_stride * NT;
    const uint32_t dx_base = q_bytes, bs_base = dx_base + (uint32_t)(K / 256) * 64u;
    const uint32_t zero_off = bs_base + (uint32_t)(K / 32) * 64u, buf_off = zero_off + 256u;
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int x = lane & 15, g = lane >> 4;

    // this lane's three chunks of a macro tile: chunk qi -> row qi / CPR, byte 16 * (qi % CPR)
    int crow[3];
    uint32_t coff[3];
#pragma unroll
    for (int j = 0; j < 3; j++) {
        int qi = 64 * j + lane;
        if (qi > KQ_CHUNKS - 1) qi = KQ_CHUNKS - 1;
        crow[j] = qi / CPR;
        coff[j] = 16u * (uint32_t)(qi % CPR);
    }
    const bool tail_chunk = lane < KQ_CHUNKS - 128;                     // chunk 128 + lane exists (16 or 48 lanes)

    // tiles of 16 rows: a contiguous range per workgroup, in rounds of TC <= 4 tiles whose (tile, macro step) items are
    // split evenly over the waves; a wave's share touches at most two tiles
    const uint32_t tiles = (uint32_t)ceil_div(N, 16);
    const uint32_t t_begin = tiles * block / grid, t_end = tiles * (block + 1) / grid;
    const int T = (int)(t_end - t_begin);
    const int rounds = (T + 3) / 4;
    const int TCmax = rounds ? (T + rounds - 1) / rounds : 0;
    struct Seg { uint32_t tile; int m0, m1; };
    auto segment = [&](int rd, int seg) {
        const uint32_t t0 = t_begin + (uint32_t)(rd * TCmax);
        const int TC = min((int)(t_end - t0), TCmax);
        const int items = TC * np;
        const int i0 = items * wv / NW, i1 = items * (wv + 1) / NW;
        const int k = i0 / np + seg;
        const int lo = seg == 0 ? i0 : (k * np < i1 ? k * np : i1);
        const int hi = (k + 1) * np < i1 ? (k + 1) * np : i1;
        Seg r;
        r.tile = t0 + k;
        r.m0 = lo - k * np;
        r.m1 = (seg == 0 || lo < i1) ? hi - k * np : r.m0;
        return r;
    };
    auto macro_offsets = [&](uint32_t (&co)[3], uint32_t tile) {
        const int last = (int)min((int64_t)15, N - 1 - (int64_t)tile * 16);
#pragma unroll
        for (int j = 0; j < 3; j++) co[j] = (uint32_t)min(crow[j], last) * (uint32_t)nb01 + coff[j];
    };

    // ---- prologue: activation loads, then the first macro tile's weight loads, then the LDS images ----
    // Every load instruction of the prologue costs the same whether one lane or all of them use its result, so the n rows
    // are spread over the threads as flat lists of (token, piece) items - n * K / 16 chunks of quants, n * K / 256 scales,
    // n * K / 32 pairs of block sums - with as many register slots as the workgroup needs for them; a thread past the end
    // of a list loads the last item again and dumps it into the idle macro-tile buffers (all loads unconditional: a load
    // inside a branch makes the compiler wait for everything in flight).  Rows n .. NT-1 of the images are zeros.
    u32x4 v[3];
    {
        const int nchunk = (int)(K / 16), nsb = (int)(K / 256), nsub = (int)(K / 32);
        const int q_items = n * nchunk, d_items = n * nsb, b_items = n * nsub;
        const uint32_t dump = buf_off + 16u * (threadIdx.x % (NW * KQ_CHUNKS));
        // item -> (token, piece): idx / den through the reciprocal, corrected by one (idx < 2^20)
        auto divmod = [](int idx, int den, float rcp, int &q, int &r) {
            q = (int)((float)idx * rcp);
            r = idx - q * den;
            if (r < 0) { q--; r += den; } else if (r >= den) { q++; r -= den; }
        };
        const float rc_chunk = 1.0f / (float)nchunk, rc_sb = 1.0f / (float)nsb, rc_sub = 1.0f / (float)nsub;
        // (token, piece) of item idx, the last item's past the end of the list
        auto q_place = [&](int idx, int t, int c, const u32x4 *&src, uint32_t &dst) {
            const bool in = idx < q_items;
            t = in ? t : n - 1;
            c = in ? c : nchunk - 1;
            src = reinterpret_cast<const u32x4 *>(ws + (size_t)t * ws_stride + 16 * (size_t)c);
            dst = in ? (uint32_t)t * q_stride + 16u * (uint32_t)c : dump;
        };
        auto d_place = [&](int idx, int t, int sb, const float *&src, uint32_t &dst) {
            const bool in = idx < d_items;
            t = in ? t : n - 1;
            sb = in ? sb : nsb - 1;
            src = reinterpret_cast<const float *>(ws + (size_t)t * ws_stride + q8_K_off_d(K)) + sb;
            dst = in ? dx_base + 4u * (uint32_t)(sb * 16 + t) : dump;
        };
        auto b_place = [&](int idx, int t, int sub, const uint32_t *&src, uint32_t &dst) {   // two int16 block sums of a 32-value sub-block
            const bool in = idx < b_items;
            t = in ? t : n - 1;
            sub = in ? sub : nsub - 1;
            src = reinterpret_cast<const uint32_t *>(ws + (size_t)t * ws_stride + q8_K_off_bsums(K)) + sub;
            dst = in ? bs_base + 4u * (uint32_t)(sub * 16 + t) : dump;
        };
        auto q_item = [&](int idx, const u32x4 *&src, uint32_t &dst) {
            int t, c;
            divmod(idx, nchunk, rc_chunk, t, c);
            q_place(idx, t, c, src, dst);
        };
        auto d_item = [&](int idx, const float *&src, uint32_t &dst) {
            int t, sb;
            divmod(idx, nsb, rc_sb, t, sb);
            d_place(idx, t, sb, src, dst);
        };
        auto b_item = [&](int idx, const uint32_t *&src, uint32_t &dst) {
            int t, sub;
            divmod(idx, nsub, rc_sub, t, sub);
            b_place(idx, t, sub, src, dst);
        };
        // a thread's items are WGS apart: one division each for the first, then steps of (WGS / den, WGS % den) with a carry
        auto advance = [](int &t, int &c, int den) {
            t += WGS / den; c += WGS % den;
            if (c >= den) { c -= den; t++; }
        };
        auto pair_sum = [](uint32_t p) { return (int)(int16_t)(p & 0xffffu) + (int)(int16_t)(p >> 16); };
        auto stage = [&](auto slots) {
            constexpr int QL = decltype(slots)::value, BL = QL / 2, DL = 2;
            u32x4 qv[QL];
            uint32_t qdst[QL], bv[BL], bdst[BL], ddst[DL];
            float dv[DL];
            int t, c;
            divmod((int)threadIdx.x, nchunk, rc_chunk, t, c);
#pragma unroll
            for (int j = 0; j < QL; j++) {
                const u32x4 *src;
                q_place(j * WGS + (int)threadIdx.x, t, c, src, qdst[j]);
                qv[j] = *src;
                advance(t, c, nchunk);
            }
            divmod((int)threadIdx.x, nsb, rc_sb, t, c);
#pragma unroll
            for (int j = 0; j < DL; j++) {
                const float *src;
                d_place(j * WGS + (int)threadIdx.x, t, c, src, ddst[j]);
                dv[j] = *src;
                advance(t, c, nsb);
            }
            divmod((int)threadIdx.x, nsub, rc_sub, t, c);
#pragma unroll
            for (int j = 0; j < BL; j++) {
                const uint32_t *src;
                b_place(j * WGS + (int)threadIdx.x, t, c, src, bdst[j]);
                bv[j] = *src;
                advance(t, c, nsub);
            }
            __builtin_amdgcn_sched_barrier(0);                           // activations are requested before weights
            {
                Seg s0 = segment(0, 0);
                s0.tile = min(s0.tile, tiles - 1);
                s0.m0 = max(0, min(s0.m0, np - 1));
                uint32_t co[3];
                macro_offsets(co, s0.tile);
                const uint8_t *tb = W + (size_t)s0.tile * 16 * nb01 + (size_t)s0.m0 * KQ_ROW_BYTES;
#pragma unroll
                for (int j = 0; j < 3; j++) v[j] = *reinterpret_cast<const u32x4 *>(tb + co[j]);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < QL; j++) *reinterpret_cast<u32x4 *>(lds + qdst[j]) = qv[j];
#pragma unroll
            for (int j = 0; j < DL; j++) *reinterpret_cast<float *>(lds + ddst[j]) = dv[j];
#pragma unroll
            for (int j = 0; j < BL; j++) *reinterpret_cast<int *>(lds + bdst[j]) = pair_sum(bv[j]);
            // lists longer than the slots (rows wider than 16384 values at 8 tokens): the rest in plain loops
            for (int idx = QL * WGS + (int)threadIdx.x; idx < q_items; idx += WGS) {
                const u32x4 *src;
                uint32_t dst;
                q_item(idx, src, dst);
                *reinterpret_cast<u32x4 *>(lds + dst) = *src;
            }
            for (int idx = DL * WGS + (int)threadIdx.x; idx < d_items; idx += WGS) {
                const float *src;
                uint32_t dst;
                d_item(idx, src, dst);
                *reinterpret_cast<float *>(lds + dst) = *src;
            }
            for (int idx = BL * WGS + (int)threadIdx.x; idx < b_items; idx += WGS) {
                const uint32_t *src;
                uint32_t dst;
                b_item(idx, src, dst);
                *reinterpret_cast<int *>(lds + dst) = pair_sum(*src);
            }
        };
        const int need = (q_items + WGS - 1) / WGS;
        if (need <= 4) stage(std::integral_constant<int, 4>{});
        else if (need <= 8) stage(std::integral_constant<int, 8>{});
        else if (need <= 12) stage(std::integral_constant<int, 12>{});
        else stage(std::integral_constant<int, 16>{});
        // rows n .. NT-1: zeros
        for (int i = (int)threadIdx.x; i < (NT - n) * nchunk; i += WGS) {
            int t, c;
            divmod(i, nchunk, rc_chunk, t, c);
            *reinterpret_cast<u32x4 *>(lds + (uint32_t)(n + t) * q_stride + 16u * (uint32_t)c) = u32x4{0u, 0u, 0u, 0u};
        }
        for (int i = (int)threadIdx.x; i < nsb * NT; i += WGS)
            if ((i & (NT - 1)) >= n) reinterpret_cast<float *>(lds + dx_base)[(i / NT) * 16 + (i & (NT - 1))] = 0.f;
        for (int i = (int)threadIdx.x; i < nsub * NT; i += WGS)
            if ((i & (NT - 1)) >= n) reinterpret_cast<int *>(lds + bs_base)[(i / NT) * 16 + (i & (NT - 1))] = 0;
        if (threadIdx.x < 64) reinterpret_cast<uint32_t *>(lds + zero_off)[threadIdx.x] = 0u;
    }
    __syncthreads();

    // ---- per-lane LDS addressing ----
    // NT == 16: operand a0 is real in lane groups g < 2 (sub-block 2p), a1 in g >= 2 (sub-block 2p+1).
    // NT == 8 : one operand; row x < 8 is token x, real in g < 2; row x >= 8 is token x - 8, real in g >= 2.
    const int tokx = NT == 16 ? x : (x & 7);
    const bool real0 = NT == 16 ? g < 2 : ((x < 8) == (g < 2));
    const bool real1 = NT == 16 && g >= 2;
    const uint32_t a_real = (uint32_t)tokx * q_stride + 16u * g;
    const uint32_t a0_off = real0 ? a_real : zero_off, a0_step = real0 ? 256u : 0u;
    const uint32_t a1_off = real1 ? a_real : zero_off, a1_step = real1 ? 256u : 0u;
    // result rows 4g..4g+3 of this lane: NT == 16: tokens 4g..4g+3 of both sub-blocks;
    // NT == 8: tokens 4(g&1)..4(g&1)+3 of sub-block 2p + (g >> 1)
    const int par = g >> 1;                                             // NT == 8: the sub-block parity of this lane's results
    const uint32_t tok4 = NT == 16 ? 4u * g : 4u * (g & 1);             // first of the lane's four tokens
    uint8_t *mybuf = lds + buf_off + (uint32_t)wv * KQ_MACRO_BYTES;
    const uint32_t hdr = (uint32_t)x * KQ_ROW_BYTES;                    // row x of the macro tile: d, dmin, scales[12], qs[128]
    const uint32_t b_off = hdr + (uint32_t)KqGeom<WT>::QS_OFF + 16u * (g & 1);     // + 32 * p
    const uint32_t qh_off = hdr + 16u + 16u * (g & 1);                  // Q5_K: the fifth bits of the same 16 elements
    const uint32_t nib_shift = 4u * (g >> 1);

    for (int mat = 0; mat < nmat; mat++) {
    if (mat == 1) { W = W2; y = y2; }
    for (int rd = 0; rd < rounds; rd++) {
        float4 part[2];
#pragma unroll
        for (int seg = 0; seg < 2; seg++) {
            const Seg sg = segment(rd, seg);
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            if (sg.m0 < sg.m1) {                                         // wave-uniform
                uint32_t co[3];
                macro_offsets(co, sg.tile);
                const uint8_t *tb = W + (size_t)sg.tile * 16 * nb01;
                if (rd != 0 || seg != 0 || mat != 0) {
#pragma unroll
                    for (int j = 0; j < 3; j++) v[j] = *reinterpret_cast<const u32x4 *>(tb + (size_t)sg.m0 * KQ_ROW_BYTES + co[j]);
                }
                u32x4 v2[3];
                {
                    const int mn = min(sg.m0 + 1, sg.m1 - 1);
#pragma unroll
                    for (int j = 0; j < 3; j++) v2[j] = *reinterpret_cast<const u32x4 *>(tb + (size_t)mn * KQ_ROW_BYTES + co[j]);
                }
                auto step = [&](u32x4 (&r)[3], int m, int mnext, bool live) {
                    // registers -> LDS (the wave's LDS operations execute in order), then the same registers
                    // receive macro tile mnext
                    reinterpret_cast<u32x4 *>(mybuf)[lane] = r[0];
                    reinterpret_cast<u32x4 *>(mybuf)[64 + lane] = r[1];
                    if (tail_chunk) reinterpret_cast<u32x4 *>(mybuf)[128 + lane] = r[2];
                    const uint8_t *nb = tb + (size_t)min(mnext, sg.m1 - 1) * KQ_ROW_BYTES;
#pragma unroll
                    for (int j = 0; j < 3; j++) r[j] = *reinterpret_cast<const u32x4 *>(nb + co[j]);
                    if (!live) return;                                   // wave-uniform
                    // header of row x: d | dmin, then the 12 scale bytes (get_scale_min_k4, ggml-quants.c)
                    const u32x4 h = *reinterpret_cast<const u32x4 *>(mybuf + hdr);
                    const float d = h2f(h.x), dmin = h2f(h.x >> 16);
                    const uint32_t s0 = h.y, s1 = h.z, s2 = h.w;         // scales[0..3], [4..7], [8..11]
                    // sub-block j < 4: sc = s0.byte[j] & 63, m = s1.byte[j] & 63;
                    // j >= 4: sc = (s2.byte[j-4] & 15) | (s0.byte[j-4] >> 6 << 4), m = (s2.byte[j-4] >> 4) | (s1.byte[j-4] >> 6 << 4)
                    auto sc_of = [&](int j) -> int {
                        return j < 4 ? (int)((s0 >> (8 * j)) & 63u)
                                     : (int)(((s2 >> (8 * (j - 4))) & 15u) | ((((s0 >> (8 * (j - 4))) >> 6) & 3u) << 4));
                    };
                    auto m_of = [&](int j) -> int {
                        return j < 4 ? (int)((s1 >> (8 * j)) & 63u)
                                     : (int)((((s2 >> (8 * (j - 4))) >> 4) & 15u) | ((((s1 >> (8 * (j - 4))) >> 6) & 3u) << 4));
                    };
                    const uint8_t *pa0 = lds + a0_off + (uint32_t)m * a0_step;
                    const uint8_t *pa1 = lds + a1_off + (uint32_t)m * a1_step;
                    const int *pbs = reinterpret_cast<const int *>(lds + bs_base) + ((uint32_t)m * 8u) * 16u + tok4;
                    int isc[4] = {0, 0, 0, 0}, imn[4] = {0, 0, 0, 0};
                    u32x4 qh = {0u, 0u, 0u, 0u};
                    if constexpr (WT == T_Q5_K) qh = *reinterpret_cast<const u32x4 *>(mybuf + qh_off);
#pragma unroll
                    for (int pi = 0; pi < 4; pi++) {
                        const u32x4 wq = *reinterpret_cast<const u32x4 *>(mybuf + b_off + 32u * pi);
                        v4i b = {(int)((wq.x >> nib_shift) & 0x0f0f0f0fu), (int)((wq.y >> nib_shift) & 0x0f0f0f0fu),
                                 (int)((wq.z >> nib_shift) & 0x0f0f0f0fu), (int)((wq.w >> nib_shift) & 0x0f0f0f0fu)};
                        if constexpr (WT == T_Q5_K) {
                            const uint32_t hb = 2u * pi + (g >> 1);                   // the sub-block = the bit of qh
                            b.x |= (int)(((qh.x >> hb) & 0x01010101u) << 4); b.y |= (int)(((qh.y >> hb) & 0x01010101u) << 4);
                            b.z |= (int)(((qh.z >> hb) & 0x01010101u) << 4); b.w |= (int)(((qh.w >> hb) & 0x01010101u) << 4);
                        }
                        const v4i zero = {0, 0, 0, 0};
                        const v4i a0 = *reinterpret_cast<const v4i *>(pa0 + 64 * pi);
                        const v4i r0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, b, zero, 0, 0, 0);
                        if constexpr (NT == 8) {
                            // the lane's results belong to sub-block 2 pi + par
                            const int sc = par ? sc_of(2 * pi + 1) : sc_of(2 * pi);
                            const int mn = par ? m_of(2 * pi + 1) : m_of(2 * pi);
                            const v4i bs = *reinterpret_cast<const v4i *>(pbs + (2 * pi + par) * 16);
                            // 24-bit multiplies (full rate): scales and mins < 2^6, sums < 2^17
                            isc[0] += __mul24(sc, r0.x); isc[1] += __mul24(sc, r0.y); isc[2] += __mul24(sc, r0.z); isc[3] += __mul24(sc, r0.w);
                            imn[0] += __mul24(mn, bs.x); imn[1] += __mul24(mn, bs.y); imn[2] += __mul24(mn, bs.z); imn[3] += __mul24(mn, bs.w);
                        } else {
                            const v4i a1 = *reinterpret_cast<const v4i *>(pa1 + 64 * pi);
                            const v4i r1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, b, zero, 0, 0, 0);
                            const int sc0 = sc_of(2 * pi), sc1 = sc_of(2 * pi + 1), mn0 = m_of(2 * pi), mn1 = m_of(2 * pi + 1);
                            const v4i bs0 = *reinterpret_cast<const v4i *>(pbs + (2 * pi) * 16);
                            const v4i bs1 = *reinterpret_cast<const v4i *>(pbs + (2 * pi + 1) * 16);
                            isc[0] += __mul24(sc0, r0.x) + __mul24(sc1, r1.x); isc[1] += __mul24(sc0, r0.y) + __mul24(sc1, r1.y);
                            isc[2] += __mul24(sc0, r0.z) + __mul24(sc1, r1.z); isc[3] += __mul24(sc0, r0.w) + __mul24(sc1, r1.w);
                            imn[0] += __mul24(mn0, bs0.x) + __mul24(mn1, bs1.x); imn[1] += __mul24(mn0, bs0.y) + __mul24(mn1, bs1.y);
                            imn[2] += __mul24(mn0, bs0.z) + __mul24(mn1, bs1.z); imn[3] += __mul24(mn0, bs0.w) + __mul24(mn1, bs1.w);
                        }
                    }
                    const float4 dx = *reinterpret_cast<const float4 *>(lds + dx_base + ((uint32_t)m * 16u + tok4) * 4u);
                    acc[0] = __builtin_fmaf(d * dx.x, (float)isc[0], acc[0]); acc[0] = __builtin_fmaf(-(dmin * dx.x), (float)imn[0], acc[0]);
                    acc[1] = __builtin_fmaf(d * dx.y, (float)isc[1], acc[1]); acc[1] = __builtin_fmaf(-(dmin * dx.y), (float)imn[1], acc[1]);
                    acc[2] = __builtin_fmaf(d * dx.z, (float)isc[2], acc[2]); acc[2] = __builtin_fmaf(-(dmin * dx.z), (float)imn[2], acc[2]);
                    acc[3] = __builtin_fmaf(d * dx.w, (float)isc[3], acc[3]); acc[3] = __builtin_fmaf(-(dmin * dx.w), (float)imn[3], acc[3]);
                };
                for (int m = sg.m0; m < sg.m1; m += 2) {
                    step(v, m, m + 2, true);
                    step(v2, m + 1, m + 3, m + 1 < sg.m1);
                }
            }
            part[seg] = make_float4(acc[0], acc[1], acc[2], acc[3]);
        }
        // partial sums go to the wave's own (now idle) macro-tile buffer
        reinterpret_cast<float4 *>(mybuf)[lane] = part[0];
        reinterpret_cast<float4 *>(mybuf)[64 + lane] = part[1];
        __syncthreads();

        // wave k adds up tile k's partial sums in wave order and stores 16 rows x n tokens
        const uint32_t t0 = t_begin + (uint32_t)(rd * TCmax);
        const int TC = min((int)(t_end - t0), TCmax);
        const int items = TC * np;
        if (wv < TC) {
            const int k = wv;
            float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
            for (int w = 0; w < NW; w++) {
                const int wi0 = items * w / NW, wi1 = items * (w + 1) / NW;
                if (wi1 <= k * np || wi0 >= (k + 1) * np || wi0 == wi1) continue;
                const int seg = (wi0 / np == k) ? 0 : 1;
                const float4 pv = reinterpret_cast<const float4 *>(lds + buf_off + (uint32_t)w * KQ_MACRO_BYTES)[seg * 64 + lane];
                s.x += pv.x; s.y += pv.y; s.z += pv.z; s.w += pv.w;
            }
            if constexpr (NT == 8) {
                // lanes (x, g) and (x, g + 2) hold the even and odd sub-blocks' halves of the same (row, token) sums
                s.x += __shfl_xor(s.x, 32); s.y += __shfl_xor(s.y, 32);
                s.z += __shfl_xor(s.z, 32); s.w += __shfl_xor(s.w, 32);
            }
            const int64_t row = (int64_t)(t0 + k) * 16 + x;
            if (row < N && (NT == 16 || g < 2)) {
                const int tk = 4 * g;
                if (tk + 0 < n) y[(size_t)(tk + 0) * ldy + row] = s.x;
                if (tk + 1 < n) y[(size_t)(tk + 1) * ldy + row] = s.y;
                if (tk + 2 < n) y[(size_t)(tk + 2) * ldy + row] = s.z;
                if (tk + 3 < n) y[(size_t)(tk + 3) * ldy + row] = s.w;
            }
        }
        __syncthreads();
    }
    }
}

template <int WT, int NT, int NW, int OCC>
hipError_t launch_cfg(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n, float *y,
                      int64_t ldy, const DeviceLimits &lim, hipStream_t st, const void *W2, float *y2) {
    const size_t lds_bytes = mmv_q4k_lds_bytes<WT, NT, NW>(K);
    auto kfn = mmv_q4k_kernel<WT, NT, NW, OCC>;
    static LdsGrant grant;
    if (hipError_t e = grant_dynamic_lds(kfn, lds_bytes, lim, grant); e != hipSuccess) return e;
    const int cus = lim.compute_units > 0 ? lim.compute_units : 256;
    const int64_t tiles = ceil_div(N, 16);
    constexpr int per_cu = OCC * 4 / NW;
    const int64_t groups = tiles < (int64_t)cus * per_cu ? tiles : (int64_t)cus * per_cu;
    hipLaunchKernelGGL(kfn, dim3((unsigned)groups), dim3(NW * 64), lds_bytes, st, (const uint8_t *)W, nb01, K, N,
                       (const uint8_t *)ws, ws_stride, n, y, ldy, (const uint8_t *)W2, y2);
    return hipGetLastError();
}

// Eight waves per workgroup; six when that is what makes the 8-token image of a wide row fit (K = 14336).
template <int WT> int max_tokens_typed(int64_t K, const DeviceLimits &lim) {
    if (mmv_q4k_lds_bytes<WT, 16, 8>(K) <= (size_t)lim.max_lds_per_block) return 16;
    if (mmv_q4k_lds_bytes<WT, 8, 8>(K) <= (size_t)lim.max_lds_per_block) return 8;
    if (mmv_q4k_lds_bytes<WT, 8, 6>(K) <= (size_t)lim.max_lds_per_block) return 8;
    return 0;
}
template <int WT>
hipError_t launch_typed(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n, float *y,
                        int64_t ldy, const DeviceLimits &lim, hipStream_t st, const void *W2, float *y2) {
    if (n <= 8) {
        if (mmv_q4k_lds_bytes<WT, 8, 8>(K) <= (size_t)lim.max_lds_per_block)
            return launch_cfg<WT, 8, 8, 2>(W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st, W2, y2);
        if (mmv_q4k_lds_bytes<WT, 8, 6>(K) <= (size_t)lim.max_lds_per_block)
            return launch_cfg<WT, 8, 6, 2>(W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st, W2, y2);
        return hipErrorInvalidValue;
    }
    if (mmv_q4k_lds_bytes<WT, 16, 8>(K) > (size_t)lim.max_lds_per_block) return hipErrorInvalidValue;
    return launch_cfg<WT, 16, 8, 2>(W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st, W2, y2);
}

}  // namespace

// Tokens one launch takes for this shape and type (Q4_K or Q5_K): 16 if the 16-token image fits in LDS, else 8, else 0
// (use the dot-product GEMV).
int mmv_q4k_max_tokens(int wtype, int64_t K, int64_t N, const DeviceLimits &lim) {
    if (tune("CHIP_MMV_Q4K", 1) == 0 || K % 256 != 0 || (wtype != T_Q4_K && wtype != T_Q5_K)) return 0;
    const int cus = lim.compute_units > 0 ? lim.compute_units : 256;
    if (ceil_div(N, 16) < cus) return 0;                                 // too few 16-row tiles to occupy every CU
    if (N > (1 << 24) || K > (1 << 20)) return 0;                        // 32-bit tile arithmetic
    return wtype == T_Q4_K ? max_tokens_typed<T_Q4_K>(K, lim) : max_tokens_typed<T_Q5_K>(K, lim);
}

// W2 / y2: NULL, or a second matrix of the same type, shape and strides that reads the same rows (one launch for both).
hipError_t launch_mmv_q4k(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n,
                          float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const void *W2, float *y2) {
    if (n < 1 || n > 16 || (wtype != T_Q4_K && wtype != T_Q5_K) || (W2 == nullptr) != (y2 == nullptr)) return hipErrorInvalidValue;
    if (N <= 0) return hipSuccess;
    return wtype == T_Q4_K ? launch_typed<T_Q4_K>(W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st, W2, y2)
                           : launch_typed<T_Q5_K>(W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st, W2, y2);
}

}  // namespace chip
