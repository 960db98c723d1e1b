// Multi-token GEMV on the matrix cores for Q4_0 weights, 5..16 tokens: the Q8_0 kernel (gemv_mfma.hip) with a macro tile
// of 16 rows x 144 bytes (8 blocks of 18) and 4-bit operands.
//
//   reference: lm_ggml_vec_dot_q4_0_q8_0 (ggml-cpu/ggml-cpu-quants.c:1906-2420) for every (row, token) pair, as driven by
//   lm_ggml_compute_forward_mul_mat (ggml-cpu/ggml-cpu.c:1257-1449).
//
// One v_mfma_i32_16x16x64_i8 spans two blocks.  A block's 16 quant bytes hold elements 0..15 in their low and 16..31 in
// their high nibbles, so lane (x, g) of the weight operand reads the 16 bytes of block 2p + (g >> 1) of row x and takes
// the low (g even) or high (g odd) nibbles: k = 16 g ... 16 g + 15 is then the element order of the Q8_0 activations.
// The operand byte is 16 * (nibble - 8), made with a shift, a mask and a sign flip; the factor 16 is taken out of the
// fp16 scale (exact).  Separation of the two blocks' sums, macro-tile staging through LDS, work split and the
// deterministic reduction are those of the Q8_0 kernel.  Bound: the weight stream (HBM).
#include "kernels.h"
#include "dev_common.h"
#include "act_layout.h"
#include "mmv_stage.h"
#include <cstdlib>

namespace chip {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));

constexpr int Q40_MACRO_PAIRS = 4;    // block pairs (of 68 bytes) per row in one macro tile
constexpr int Q40_ROW_BYTES = 36 * Q40_MACRO_PAIRS;          // 144 = 9 chunks of 16 bytes (8 blocks of 18)
constexpr int Q40_MACRO_BYTES = 16 * Q40_ROW_BYTES;           // 2304 per wave; also holds the wave's partial sums

// LDS: quant image [NT tokens][K + 16] bytes (the 16 pad bytes put neighbouring tokens 4 banks apart) |
// scale image [K/32 blocks][16 tokens] float | 256 zero bytes | [NW waves] macro-tile buffers
template <int NT, int NW> __host__ __device__ constexpr size_t mmv_q40_lds_bytes(int64_t K) {
    // + 16: the aligned five-dword operand read of the last block of the last row reaches 4 bytes past the tile
    return (size_t)(K + 16) * NT + (size_t)(K / 32) * 64 + 256 + NW * (size_t)Q40_MACRO_BYTES + 16;
}

template <int NT, int NW, int OCC>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void mmv_q4_0_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N,
                                                           const uint8_t *__restrict__ ws, size_t ws_stride, int n,
                                                           float *__restrict__ y, int64_t ldy) {
    constexpr int WGS = NW * 64;
    extern __shared__ __align__(16) uint8_t lds[];
    const int np = (int)(K / 256);                                      // macro steps (4 block pairs) per row
    const uint32_t q_stride = (uint32_t)K + 16u, q_bytes = q_stride * NT, d_bytes = (uint32_t)(K / 32) * 64;
    const uint32_t zero_off = q_bytes + d_bytes, buf_off = zero_off + 256;
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));   // in an SGPR: tile arithmetic stays scalar
    const int x = lane & 15, g = lane >> 4;

    // this lane's three chunks of a macro tile: chunk qi -> row qi / 9, byte 16 * (qi % 9)
    int crow[3];
    uint32_t coff[3];
#pragma unroll
    for (int j = 0; j < 3; j++) {
        int qi = 64 * j + lane;
        if (qi > 143) qi = 143;
        crow[j] = qi / 9;
        coff[j] = 16u * (uint32_t)(qi % 9);
    }
    const bool tail_chunk = lane < 144 - 128;                           // chunk 128 + lane exists

    // tiles of 16 rows: this workgroup owns a contiguous range, processed in rounds of TC <= 4 tiles whose
    // (tile, macro step) items are split evenly over the waves; a wave's share touches at most two tiles
    // (32-bit arithmetic: the launcher rejects shapes whose products below would overflow)
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
    // byte offsets of this lane's chunks from the tile's first row (rows past N re-read row N - 1)
    auto macro_offsets = [&](uint32_t (&co)[3], uint32_t tile) {
        const int last = (int)min((int64_t)15, N - 1 - (int64_t)tile * 16);
#pragma unroll
        for (int j = 0; j < 3; j++) co[j] = (uint32_t)min(crow[j], last) * (uint32_t)nb01 + coff[j];
    };

    // ---- prologue: activation loads, then the first macro tile's weight loads, then the LDS image ----
    u32x4 v[3];
    {
        // the n rows into the LDS image (mmv_stage.h); between their loads and their stores, the wave's first macro tile
        // (clamped into the matrix if the wave has no work: loaded, never used)
        mmv_stage_q8_0_rows<NT, WGS>(lds, ws, ws_stride, n, K, q_stride, q_bytes, buf_off + 32u * threadIdx.x, [&] {
            Seg s0 = segment(0, 0);
            s0.tile = min(s0.tile, tiles - 1);
            s0.m0 = max(0, min(s0.m0, np - 1));
            uint32_t co[3];
            macro_offsets(co, s0.tile);
            const uint8_t *tb = W + (size_t)s0.tile * 16 * nb01 + (size_t)s0.m0 * Q40_ROW_BYTES;
#pragma unroll
            for (int j = 0; j < 3; j++) v[j] = *reinterpret_cast<const u32x4 *>(tb + co[j]);
        });
        if (threadIdx.x < 64) reinterpret_cast<uint32_t *>(lds + zero_off)[threadIdx.x] = 0u;
    }
    __syncthreads();

    // ---- per-lane LDS addressing ----
    // NT == 16: operand a0 is real in lane groups g < 2, a1 in g >= 2; the other reads the zero chunk.
    // NT == 8 : one operand; row x < 8 is token x, real in g < 2; row x >= 8 is token x - 8, real in g >= 2.
    const int tokx = NT == 16 ? x : (x & 7);
    const bool real0 = NT == 16 ? g < 2 : ((x < 8) == (g < 2));
    const bool real1 = NT == 16 && g >= 2;
    // Per macro tile (4 pairs = 256 activation bytes per token) a real lane advances by 256 bytes and reads its
    // pairs at +0, +64, +128, +192; a zero lane stays on the 256-byte zero area with the same offsets.
    const uint32_t a_real = (uint32_t)tokx * q_stride + 16u * g;
    const uint32_t a0_off = real0 ? a_real : zero_off, a0_step = real0 ? 256u : 0u;
    const uint32_t a1_off = real1 ? a_real : zero_off, a1_step = real1 ? 256u : 0u;
    // result rows 4g..4g+3 of this lane: NT == 16: tokens 4g..4g+3 of both blocks;
    // NT == 8: tokens 4(g&1)..4(g&1)+3 of block 2p + (g >> 1)
    const uint32_t dx_off = q_bytes + (NT == 16 ? 16u * g : 16u * (g & 1) + 64u * (g >> 1));
    uint8_t *mybuf = lds + buf_off + (uint32_t)wv * Q40_MACRO_BYTES;
    // operand read position of lane (x, g) inside a macro tile, pair 0
    const uint32_t b_off = (uint32_t)x * Q40_ROW_BYTES + 18u * (g >> 1) + 2u;      // the block's 16 quant bytes
    const bool high_nibbles = (g & 1) != 0;                            // elements 16..31 of the block
    const uint32_t b_al = b_off & ~3u, b_sh = 8u * (b_off & 3u);
    // weight scale: NT == 16 needs d of blocks 2p and 2p+1 (at +34); NT == 8 only that of block 2p + (g >> 1)
    const uint32_t h_off = (uint32_t)x * Q40_ROW_BYTES + (NT == 16 ? 0u : 18u * (g >> 1));

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
                if (rd != 0 || seg != 0) {
#pragma unroll
                    for (int j = 0; j < 3; j++) v[j] = *reinterpret_cast<const u32x4 *>(tb + (size_t)sg.m0 * Q40_ROW_BYTES + co[j]);
                }
                // Two macro tiles in flight in two register sets used alternately (no register rotation: a copy
                // would force a wait for the loads just issued).  Loads are unconditional, indices past the segment
                // are clamped (the last tile is then re-read and not used).
                u32x4 v2[3];
                {
                    const int mn = min(sg.m0 + 1, sg.m1 - 1);
#pragma unroll
                    for (int j = 0; j < 3; j++) v2[j] = *reinterpret_cast<const u32x4 *>(tb + (size_t)mn * Q40_ROW_BYTES + co[j]);
                }
                auto step = [&](u32x4 (&r)[3], int m, int mnext, bool live) {
                    // registers -> LDS (the wave's LDS operations execute in order, so the previous step's operand
                    // reads are done), then the same registers receive macro tile mnext
                    reinterpret_cast<u32x4 *>(mybuf)[lane] = r[0];
                    reinterpret_cast<u32x4 *>(mybuf)[64 + lane] = r[1];
                    if (tail_chunk) reinterpret_cast<u32x4 *>(mybuf)[128 + lane] = r[2];
                    const uint8_t *nb = tb + (size_t)min(mnext, sg.m1 - 1) * Q40_ROW_BYTES;
#pragma unroll
                    for (int j = 0; j < 3; j++) r[j] = *reinterpret_cast<const u32x4 *>(nb + co[j]);
                    if (!live) return;                                   // wave-uniform
                    const uint8_t *pa0 = lds + a0_off + (uint32_t)m * a0_step;
                    const uint8_t *pa1 = lds + a1_off + (uint32_t)m * a1_step;
                    const uint8_t *pdx = lds + dx_off + (uint32_t)m * 512u;
#pragma unroll
                    for (int pi = 0; pi < Q40_MACRO_PAIRS; pi++) {
                        // the 16 quants start 2 bytes past a dword boundary in lane groups g < 2: read five
                        // aligned dwords and funnel-shift by 16 or 0 bits
                        const u32x4 wlo = *reinterpret_cast<const u32x4_a4 *>(mybuf + b_al + 36u * pi);
                        const uint32_t whi = *reinterpret_cast<const uint32_t *>(mybuf + b_al + 36u * pi + 16u);
                        // 16 * (nibble - 8) as int8: the nibble moved to the high half of its byte, sign bit flipped
                        auto plane = [&](uint32_t q) -> int {
                            return (int)(((high_nibbles ? q : (q << 4)) & 0xf0f0f0f0u) ^ 0x80808080u);
                        };
                        const v4i b = {plane(__builtin_amdgcn_alignbit(wlo.y, wlo.x, b_sh)), plane(__builtin_amdgcn_alignbit(wlo.z, wlo.y, b_sh)),
                                       plane(__builtin_amdgcn_alignbit(wlo.w, wlo.z, b_sh)), plane(__builtin_amdgcn_alignbit(whi, wlo.w, b_sh))};
                        const v4i zero = {0, 0, 0, 0};
                        const v4i a0 = *reinterpret_cast<const v4i *>(pa0 + 64 * pi);
                        const float4 dx0 = *reinterpret_cast<const float4 *>(pdx + 128 * pi);
                        const float d0 = 0.0625f * h2f(*reinterpret_cast<const unsigned short *>(mybuf + h_off + 36u * pi));
                        const v4i s0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, b, zero, 0, 0, 0);
                        acc[0] = __builtin_fmaf((float)s0.x, d0 * dx0.x, acc[0]);
                        acc[1] = __builtin_fmaf((float)s0.y, d0 * dx0.y, acc[1]);
                        acc[2] = __builtin_fmaf((float)s0.z, d0 * dx0.z, acc[2]);
                        acc[3] = __builtin_fmaf((float)s0.w, d0 * dx0.w, acc[3]);
                        if constexpr (NT == 16) {
                            const v4i a1 = *reinterpret_cast<const v4i *>(pa1 + 64 * pi);
                            const float4 dx1 = *reinterpret_cast<const float4 *>(pdx + 128 * pi + 64);
                            const float d1 = 0.0625f * h2f(*reinterpret_cast<const unsigned short *>(mybuf + h_off + 36u * pi + 18u));
                            const v4i s1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, b, zero, 0, 0, 0);
                            acc[0] = __builtin_fmaf((float)s1.x, d1 * dx1.x, acc[0]);
                            acc[1] = __builtin_fmaf((float)s1.y, d1 * dx1.y, acc[1]);
                            acc[2] = __builtin_fmaf((float)s1.z, d1 * dx1.z, acc[2]);
                            acc[3] = __builtin_fmaf((float)s1.w, d1 * dx1.w, acc[3]);
                        }
                    }
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
                const float4 pv = reinterpret_cast<const float4 *>(lds + buf_off + (uint32_t)w * Q40_MACRO_BYTES)[seg * 64 + lane];
                s.x += pv.x; s.y += pv.y; s.z += pv.z; s.w += pv.w;
            }
            if constexpr (NT == 8) {
                // lanes (x, g) and (x, g + 2) hold the block-2p and block-2p+1 halves of the same (row, token) sums
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

template <int NT, int NW, int OCC>
hipError_t launch_cfg(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n, float *y,
                      int64_t ldy, const DeviceLimits &lim, hipStream_t st) {
    const size_t lds_bytes = mmv_q40_lds_bytes<NT, NW>(K);
    auto kfn = mmv_q4_0_kernel<NT, NW, OCC>;
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

// Tokens one launch takes for this shape: 16 if the 16-token image fits in LDS, else 8, else 0 (use the dot-product GEMV).
int mmv_q4_0_max_tokens(int64_t K, int64_t N, const DeviceLimits &lim) {
    if (tune("CHIP_MMV_Q4_0", 1) == 0 || K % 256 != 0) return 0;
    const int cus = lim.compute_units > 0 ? lim.compute_units : 256;
    if (ceil_div(N, 16) < cus) return 0;                                 // too few 16-row tiles to occupy every CU
    if (N > (1 << 24) || K > (1 << 20)) return 0;                        // the kernel's 32-bit tile arithmetic
    if (mmv_q40_lds_bytes<16, 8>(K) <= (size_t)lim.max_lds_per_block) return 16;
    if (mmv_q40_lds_bytes<8, 8>(K) <= (size_t)lim.max_lds_per_block) return 8;
    return 0;
}

hipError_t launch_mmv_q4_0(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n, float *y,
                           int64_t ldy, const DeviceLimits &lim, hipStream_t st) {
    if (n < 1 || n > 16) return hipErrorInvalidValue;
    if (N <= 0) return hipSuccess;
    if (n <= 8) {
        if (mmv_q40_lds_bytes<8, 8>(K) > (size_t)lim.max_lds_per_block) return hipErrorInvalidValue;
        return launch_cfg<8, 8, 2>(W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st);
    }
    if (mmv_q40_lds_bytes<16, 8>(K) > (size_t)lim.max_lds_per_block) return hipErrorInvalidValue;
    return launch_cfg<16, 8, 2>(W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st);
}

}  // namespace chip
