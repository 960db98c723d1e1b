// Multi-token GEMV on the matrix cores for Q6_K weights, 5..8 tokens per pass: the structure of the Q8_0 / Q4_K kernels
// (gemv_mfma.hip, gemv_mfma_q4k.hip) with the arithmetic of lm_ggml_vec_dot_q6_K_q8_K (reference
// ggml-cpu/ggml-cpu-quants.c:8520-8910) as driven by lm_ggml_compute_forward_mul_mat (ggml-cpu/ggml-cpu.c:1257-1449):
//
//   y[t][r] = sum over super-blocks b of  d[r][b] * dx[t][b] * sum_j sc[r][b][j] * sum_{i in sub-block j} (q[r][i] - 32) * a[t][i]
//
// with j the sixteen 16-value sub-blocks and sc their int8 scales.  The 6-bit quants stay unsigned in the MFMA operand
// (0..63); the -32 comes out as 32 * sc * bsum with bsum the sum of the sub-block's activation quants, which block_q8_K
// carries (bsums).  Everything up to the multiplication by d * dx is integer arithmetic and exact.
//
// One v_mfma_i32_16x16x32_i8 covers 32 values = two sub-blocks of 16 rows.  Lane (x = lane % 16, g = lane / 16) of the
// weight operand holds 8 values of row x; for MFMA q (0..7) of a super-block, half h = q / 4 and quarter c = q % 4, they
// are elements l = 8 g ... 8 g + 7 of that quarter: low (c < 2) or high nibbles of ql[64 h + 32 (c & 1) + l] with bits
// 2 c, 2 c + 1 of qh[32 h + l] on top (the layout dequantize_row_q6_K reads, ggml-quants.c:1684-1713), which is the value
// order of the activations.  Lane groups g < 2 are the first sub-block of the pair, g >= 2 the second; the operand rows
// 8..15 carry the 8 tokens again with the other lane groups live, so one MFMA returns both sub-blocks' sums separately.
//
// A super-block is 210 bytes and rows are only 2-byte aligned: a wave fetches 16 rows x 13 chunks of 16 bytes with
// 2-byte aligned loads (every lane also loads the trailing fp16 d of its row x), lays the rows out at a 224-byte stride
// in its private LDS buffer and reads operands and scales back from there; the next macro tile's loads are in flight
// meanwhile.  Bound: LDS traffic (about 5 bytes of LDS reads and writes per weight byte: two sub-blocks per MFMA mean
// 8-byte operand reads), which is why it is only used for very large matrices.
#include "kernels.h"
#include "dev_common.h"
#include "act_layout.h"
#include <cstdlib>

namespace chip {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int Q6_LDS_ROW = 224;                                 // 13 data chunks, padded to an odd multiple of 32 bytes
constexpr int Q6_MACRO_BYTES = 16 * Q6_LDS_ROW;                 // 3584 per wave; also holds the wave's partial sums
constexpr int Q6_DATA_CHUNKS = 16 * 13;                         // 208 loads of 16 bytes per macro tile

// LDS: quant image [8 tokens][K + 16] bytes | dx image [K/256][8 tokens] float | bsum image [K/16][8 tokens] int16 |
// 256 zero bytes | [NW waves] macro-tile buffers
template <int NW> __host__ __device__ constexpr size_t mmv_q6k_lds_bytes(int64_t K) {
    return (size_t)(K + 16) * 8 + (size_t)(K / 256) * 32 + (size_t)(K / 16) * 16 + 256 + NW * (size_t)Q6_MACRO_BYTES;
}

template <int NW, int OCC>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void mmv_q6k_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N, const uint8_t *__restrict__ ws,
                    size_t ws_stride, int n, float *__restrict__ y, int64_t ldy) {
    constexpr int WGS = NW * 64, NT = 8;
    extern __shared__ __align__(16) uint8_t lds[];
    const int np = (int)(K / 256);                                      // macro steps (super-blocks) per row
    const uint32_t q_stride = (uint32_t)K + 16u, q_bytes = q_stride * NT;
    const uint32_t dx_base = q_bytes, bs_base = dx_base + (uint32_t)(K / 256) * 32u;
    const uint32_t zero_off = bs_base + (uint32_t)(K / 16) * 16u, buf_off = zero_off + 256u;
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int x = lane & 15, g = lane >> 4;

    // this lane's four data chunks of a macro tile: chunk ci -> row ci / 13, byte 16 * (ci % 13); and the d of row lane % 16
    int crow[4];
    uint32_t coff[4], ldst[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        int ci = 64 * j + lane;
        if (ci > Q6_DATA_CHUNKS - 1) ci = Q6_DATA_CHUNKS - 1;
        crow[j] = ci / 13;
        coff[j] = 16u * (uint32_t)(ci % 13);
        ldst[j] = (uint32_t)crow[j] * Q6_LDS_ROW + coff[j];
    }
    const bool tail_chunk = lane < Q6_DATA_CHUNKS - 192;                // chunk 192 + lane exists (16 lanes)

    // tiles of 16 rows: a contiguous range per workgroup, in rounds of TC <= 4 tiles whose (tile, macro step) items are
    // split evenly over the waves; a wave's share touches at most two tiles
    const uint32_t tiles = (uint32_t)ceil_div(N, 16);
    const uint32_t t_begin = tiles * blockIdx.x / gridDim.x, t_end = tiles * (blockIdx.x + 1) / gridDim.x;
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
    struct Offs { uint32_t c[4]; uint32_t d; };
    auto macro_offsets = [&](Offs &o, uint32_t tile) {
        const int last = (int)min((int64_t)15, N - 1 - (int64_t)tile * 16);
#pragma unroll
        for (int j = 0; j < 4; j++) o.c[j] = (uint32_t)min(crow[j], last) * (uint32_t)nb01 + coff[j];
        o.d = (uint32_t)min(x, last) * (uint32_t)nb01 + 208u;
    };
    struct Regs { u32x4 q[4]; uint32_t d; };
    auto fetch = [&](Regs &r, const uint8_t *base, const Offs &o) {
#pragma unroll
        for (int j = 0; j < 4; j++) r.q[j] = *reinterpret_cast<const u32x4_a2 *>(base + o.c[j]);
        r.d = *reinterpret_cast<const uint16_t *>(base + o.d);
    };

    // ---- prologue: the first macro tile's weight loads, then the LDS images ----
    Regs v;
    {
        Seg s0 = segment(0, 0);
        s0.tile = min(s0.tile, tiles - 1);
        s0.m0 = max(0, min(s0.m0, np - 1));
        Offs o;
        macro_offsets(o, s0.tile);
        fetch(v, W + (size_t)s0.tile * 16 * nb01 + (size_t)s0.m0 * BYTES_Q6_K, o);
        const int nchunk = (int)(K / 16), nsb = (int)(K / 256), nsub = (int)(K / 16);
        for (int c = (int)threadIdx.x; c < nchunk; c += WGS)
#pragma unroll
            for (int i = 0; i < NT; i++) {
                u32x4 t = {0u, 0u, 0u, 0u};
                if (i < n) t = *reinterpret_cast<const u32x4 *>(ws + (size_t)i * ws_stride + 16 * (size_t)c);
                *reinterpret_cast<u32x4 *>(lds + (uint32_t)i * q_stride + 16u * c) = t;
            }
        for (int b = (int)threadIdx.x; b < nsb; b += WGS)
#pragma unroll
            for (int i = 0; i < NT; i++)
                reinterpret_cast<float *>(lds + dx_base)[b * NT + i] = i < n ? reinterpret_cast<const float *>(ws + (size_t)i * ws_stride + q8_K_off_d(K))[b] : 0.f;
        for (int b = (int)threadIdx.x; b < nsub; b += WGS)
#pragma unroll
            for (int i = 0; i < NT; i++)
                reinterpret_cast<int16_t *>(lds + bs_base)[b * NT + i] =
                    i < n ? reinterpret_cast<const int16_t *>(ws + (size_t)i * ws_stride + q8_K_off_bsums(K))[b] : (int16_t)0;
        if (threadIdx.x < 64) reinterpret_cast<uint32_t *>(lds + zero_off)[threadIdx.x] = 0u;
    }
    __syncthreads();

    // ---- per-lane LDS addressing ----
    // operand row x < 8 is token x, real in lane groups g < 2; row x >= 8 is token x - 8, real in g >= 2
    const int tokx = x & 7;
    const bool real0 = (x < 8) == (g < 2);
    const uint32_t a_real = (uint32_t)tokx * q_stride + 8u * g;
    const uint32_t a0_off = real0 ? a_real : zero_off, a0_step = real0 ? 256u : 0u, a0_q = real0 ? 32u : 0u;
    // result rows 4g..4g+3 of this lane: tokens 4(g&1)..4(g&1)+3 of the pair's sub-block g >> 1
    const int par = g >> 1;
    const uint32_t tok4 = 4u * (g & 1);
    uint8_t *mybuf = lds + buf_off + (uint32_t)wv * Q6_MACRO_BYTES;
    const uint32_t hdr = (uint32_t)x * Q6_LDS_ROW;                      // row x: ql[128] | qh[64] | scales[16]

    for (int rd = 0; rd < rounds; rd++) {
        float4 part[2];
#pragma unroll
        for (int seg = 0; seg < 2; seg++) {
            const Seg sg = segment(rd, seg);
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            if (sg.m0 < sg.m1) {                                         // wave-uniform
                Offs o;
                macro_offsets(o, sg.tile);
                const uint8_t *tb = W + (size_t)sg.tile * 16 * nb01;
                if (rd != 0 || seg != 0) fetch(v, tb + (size_t)sg.m0 * BYTES_Q6_K, o);
                Regs v2;
                fetch(v2, tb + (size_t)min(sg.m0 + 1, sg.m1 - 1) * BYTES_Q6_K, o);
                auto step = [&](Regs &r, int m, int mnext, bool live) {
                    // registers -> LDS (the wave's LDS operations execute in order), then the same registers
                    // receive macro tile mnext
                    *reinterpret_cast<u32x4 *>(mybuf + ldst[0]) = r.q[0];
                    *reinterpret_cast<u32x4 *>(mybuf + ldst[1]) = r.q[1];
                    *reinterpret_cast<u32x4 *>(mybuf + ldst[2]) = r.q[2];
                    if (tail_chunk) *reinterpret_cast<u32x4 *>(mybuf + ldst[3]) = r.q[3];
                    const float d = h2f(r.d);                            // every lane loaded the d of its own row x
                    fetch(r, tb + (size_t)min(mnext, sg.m1 - 1) * BYTES_Q6_K, o);
                    if (!live) return;                                   // wave-uniform
                    const uint8_t *pa = lds + a0_off + (uint32_t)m * a0_step;
                    const int16_t *pbs = reinterpret_cast<const int16_t *>(lds + bs_base) + ((uint32_t)m * 16u) * NT + tok4;
                    int isc[4] = {0, 0, 0, 0}, ibs[4] = {0, 0, 0, 0};
                    const u32x4 scw = *reinterpret_cast<const u32x4 *>(mybuf + hdr + 192u);     // the 16 int8 scales of row x
                    const uint32_t scws[4] = {scw.x, scw.y, scw.z, scw.w};
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const u32x2 qh = *reinterpret_cast<const u32x2 *>(mybuf + hdr + 128u + 32u * h + 8u * g);
#pragma unroll
                        for (int c = 0; c < 4; c++) {
                            const int q8 = 4 * h + c;
                            const u32x2 ql = *reinterpret_cast<const u32x2 *>(mybuf + hdr + 64u * h + 32u * (c & 1) + 8u * g);
                            const uint32_t sh = (c & 2) ? 4u : 0u;
                            const uint32_t b0 = ((ql.x >> sh) & 0x0f0f0f0fu) | (((qh.x >> (2 * c)) & 0x03030303u) << 4);
                            const uint32_t b1 = ((ql.y >> sh) & 0x0f0f0f0fu) | (((qh.y >> (2 * c)) & 0x03030303u) << 4);
                            const long bop = (long)(((uint64_t)b1 << 32) | b0);
                            const long aop = *reinterpret_cast<const long *>(pa + a0_q * q8);
                            const v4i zero = {0, 0, 0, 0};
                            const v4i r0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(aop, bop, zero, 0, 0, 0);
                            // the lane's results belong to sub-block 2 q8 + par
                            const int sc = (int)(int8_t)((scws[q8 >> 1] >> (16 * (q8 & 1) + 8 * par)) & 0xffu);
                            const u32x2 bsp = *reinterpret_cast<const u32x2 *>(pbs + (2 * q8 + par) * NT);
                            const int bs0 = (int)(int16_t)(bsp.x & 0xffffu), bs1 = (int)bsp.x >> 16;
                            const int bs2 = (int)(int16_t)(bsp.y & 0xffffu), bs3 = (int)bsp.y >> 16;
                            // 24-bit multiplies (full rate): |sc| < 2^7, |sums| < 2^18
                            isc[0] += __mul24(sc, r0.x); isc[1] += __mul24(sc, r0.y); isc[2] += __mul24(sc, r0.z); isc[3] += __mul24(sc, r0.w);
                            ibs[0] += __mul24(sc, bs0); ibs[1] += __mul24(sc, bs1); ibs[2] += __mul24(sc, bs2); ibs[3] += __mul24(sc, bs3);
                        }
                    }
                    const float4 dx = *reinterpret_cast<const float4 *>(lds + dx_base + ((uint32_t)m * NT + tok4) * 4u);
                    acc[0] = __builtin_fmaf(d * dx.x, (float)(isc[0] - 32 * ibs[0]), acc[0]);
                    acc[1] = __builtin_fmaf(d * dx.y, (float)(isc[1] - 32 * ibs[1]), acc[1]);
                    acc[2] = __builtin_fmaf(d * dx.z, (float)(isc[2] - 32 * ibs[2]), acc[2]);
                    acc[3] = __builtin_fmaf(d * dx.w, (float)(isc[3] - 32 * ibs[3]), acc[3]);
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
                const float4 pv = reinterpret_cast<const float4 *>(lds + buf_off + (uint32_t)w * Q6_MACRO_BYTES)[seg * 64 + lane];
                s.x += pv.x; s.y += pv.y; s.z += pv.z; s.w += pv.w;
            }
            {
                // lanes (x, g) and (x, g + 2) hold the even and odd sub-blocks' halves of the same (row, token) sums
                s.x += __shfl_xor(s.x, 32); s.y += __shfl_xor(s.y, 32);
                s.z += __shfl_xor(s.z, 32); s.w += __shfl_xor(s.w, 32);
            }
            const int64_t row = (int64_t)(t0 + k) * 16 + x;
            if (row < N && g < 2) {
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

template <int NW, int OCC>
hipError_t launch_cfg(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n, float *y,
                      int64_t ldy, const DeviceLimits &lim, hipStream_t st) {
    const size_t lds_bytes = mmv_q6k_lds_bytes<NW>(K);
    auto kfn = mmv_q6k_kernel<NW, OCC>;
    static LdsGrant grant;
    if (hipError_t e = grant_dynamic_lds(kfn, lds_bytes, lim, grant); e != hipSuccess) return e;
    const int cus = lim.compute_units > 0 ? lim.compute_units : 256;
    const int64_t tiles = ceil_div(N, 16);
    constexpr int per_cu = OCC * 4 / NW;
    const int64_t groups = tiles < (int64_t)cus * per_cu ? tiles : (int64_t)cus * per_cu;
    hipLaunchKernelGGL(kfn, dim3((unsigned)groups), dim3(NW * 64), lds_bytes, st, (const uint8_t *)W, nb01, K, N,
                       (const uint8_t *)ws, ws_stride, n, y, ldy);
    return hipGetLastError();
}

}  // namespace

// Tokens one launch takes for this shape: 8 if the image fits in LDS, else 0 (use the dot-product GEMV).
int mmv_q6k_max_tokens(int64_t K, int64_t N, const DeviceLimits &lim) {
    if (K % 256 != 0) return 0;
    const int cus = lim.compute_units > 0 ? lim.compute_units : 256;
    if (ceil_div(N, 16) < cus) return 0;                                 // too few 16-row tiles to occupy every CU
    if (N > (1 << 24) || K > (1 << 20)) return 0;                        // 32-bit tile arithmetic
    // Measured against the dot-product GEMV at 8 tokens: 128256 x 4096 131.5 vs 142.5 us, 14336 x 4096 22.0 vs 22.0 us,
    // 4096 x 14336 25.0 vs 21.5 us, 4096 x 4096 12.6 vs 9.4 us.  Two sub-blocks per MFMA mean 8-byte operand reads and
    // twice the LDS traffic per weight of the 16x16x64 kernels: it only pays on very large matrices (an output head).
    if (!g_force_mmv_q6k.load(std::memory_order_relaxed) && N * K < (128LL << 20)) return 0;
    return mmv_q6k_lds_bytes<8>(K) <= (size_t)lim.max_lds_per_block ? 8 : 0;
}

hipError_t launch_mmv_q6k(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n, float *y,
                          int64_t ldy, const DeviceLimits &lim, hipStream_t st) {
    if (n < 1 || n > 8) return hipErrorInvalidValue;
    if (N <= 0) return hipSuccess;
    if (mmv_q6k_lds_bytes<8>(K) > (size_t)lim.max_lds_per_block) return hipErrorInvalidValue;
    return launch_cfg<8, 2>(W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st);
}

}  // namespace chip
