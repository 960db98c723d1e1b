// Multi-token GEMV on the matrix cores: y[t][r] = sum_b d_w[r][b] * d_x[t][b] * isum[t][r][b] for 5..16 tokens.
//
// The dot-product GEMV (gemv.hip) spends VALU and LDS bandwidth in proportion to the token count; from about
// five tokens on it is no longer bound by the weight stream.  Here the per-block integer sums come from
// v_mfma_i32_16x16x64_i8 (16 weight rows x 16 tokens per instruction), so the per-token cost is only the
// fp32 scaling of the 16x16 result and the kernel stays on the weight stream up to 16 tokens.
//
//   reference: lm_ggml_vec_dot_q8_0_q8_0 (ggml-cpu/ggml-cpu-quants.c:3591-4009) for every (row, token) pair,
//   as driven by lm_ggml_compute_forward_mul_mat (ggml-cpu/ggml-cpu.c:1257-1449).
//
// One MFMA has K = 64 = two 32-blocks with different scales.  Lane (x = lane % 16, g = lane / 16) of the weight
// operand holds 16 quants of row x: half (g & 1) of block 2p + (g >> 1).  The activation operand is issued
// twice, once with the lane groups g >= 2 zeroed and once with g < 2 zeroed, which yields the two per-block sums
// separately and bit-exactly.
//
// With 8 tokens or fewer the token rows 8..15 of the activation operand would be idle; they carry the same 8
// tokens again, rows 0..7 with only the lane groups of block 2p non-zero and rows 8..15 with only those of block
// 2p+1, so one MFMA returns both blocks' sums (in result rows 0..7 and 8..15) and the scaling work is halved.
//
// Loading the weights directly in that operand layout makes every 16-lane group touch 16 different rows and
// runs at a third of the stream rate (measured), so a wave fetches a "macro tile" of 16 rows x 272 bytes
// (8 blocks per row) with row-contiguous 16-byte loads, passes it through a private 4352-byte LDS buffer and
// reads the operands back from there; the next macro tile's loads are in flight meanwhile.
#include "kernels.h"
#include "dev_common.h"
#include "act_layout.h"
#include "mmv_stage.h"

namespace chip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));

constexpr int MMV_MACRO_PAIRS = 4;    // block pairs (of 68 bytes) per row in one macro tile
constexpr int MMV_ROW_BYTES = 68 * MMV_MACRO_PAIRS;          // 272 = 17 chunks of 16 bytes
constexpr int MMV_MACRO_BYTES = 16 * MMV_ROW_BYTES;           // 4352 per wave; also holds the wave's partial sums

// LDS: quant image [NT tokens][K + 16] bytes (the 16 pad bytes put neighbouring tokens 4 banks apart) |
// scale image [K/32 blocks][16 tokens] float | 256 zero bytes | [NW waves] macro-tile buffers
template <int NT, int NW> __host__ __device__ constexpr size_t mmv_lds_bytes(int64_t K) {
    return (size_t)(K + 16) * NT + (size_t)(K / 32) * 64 + 256 + NW * (size_t)MMV_MACRO_BYTES;
}

template <int NT, int NW, int OCC>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void mmv_q8_0_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N,
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

    // this lane's five chunks of a macro tile: chunk qi -> row qi / 17, byte 16 * (qi % 17)
    int crow[5];
    uint32_t coff[5];
#pragma unroll
    for (int j = 0; j < 5; j++) {
        int qi = 64 * j + lane;
        if (qi > 271) qi = 271;
        crow[j] = qi / 17;
        coff[j] = 16u * (uint32_t)(qi % 17);
    }
    const bool tail_chunk = lane < 272 - 256;                           // chunk 256 + lane exists

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
    auto macro_offsets = [&](uint32_t (&co)[5], uint32_t tile) {
        const int last = (int)min((int64_t)15, N - 1 - (int64_t)tile * 16);
#pragma unroll
        for (int j = 0; j < 5; j++) co[j] = (uint32_t)min(crow[j], last) * (uint32_t)nb01 + coff[j];
    };

    // ---- prologue: activation loads, then the first macro tile's weight loads, then the LDS image ----
    u32x4 v[5];
    {
        // the n rows into the LDS image (mmv_stage.h); between their loads and their stores, the wave's first macro tile
        // (clamped into the matrix if the wave has no work: loaded, never used)
        mmv_stage_q8_0_rows<NT, WGS>(lds, ws, ws_stride, n, K, q_stride, q_bytes, buf_off + 32u * threadIdx.x, [&] {
            Seg s0 = segment(0, 0);
            s0.tile = min(s0.tile, tiles - 1);
            s0.m0 = max(0, min(s0.m0, np - 1));
            uint32_t co[5];
            macro_offsets(co, s0.tile);
            const uint8_t *tb = W + (size_t)s0.tile * 16 * nb01 + (size_t)s0.m0 * MMV_ROW_BYTES;
#pragma unroll
            for (int j = 0; j < 5; j++) v[j] = *reinterpret_cast<const u32x4 *>(tb + co[j]);
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
    uint8_t *mybuf = lds + buf_off + (uint32_t)wv * MMV_MACRO_BYTES;
    // operand read position of lane (x, g) inside a macro tile, pair 0
    const uint32_t b_off = (uint32_t)x * MMV_ROW_BYTES + 34u * (g >> 1) + 2u + 16u * (g & 1);
    const uint32_t b_al = b_off & ~3u, b_sh = 8u * (b_off & 3u);
    // weight scale: NT == 16 needs d of blocks 2p and 2p+1 (at +34); NT == 8 only that of block 2p + (g >> 1)
    const uint32_t h_off = (uint32_t)x * MMV_ROW_BYTES + (NT == 16 ? 0u : 34u * (g >> 1));

    for (int rd = 0; rd < rounds; rd++) {
        float4 part[2];
#pragma unroll
        for (int seg = 0; seg < 2; seg++) {
            const Seg sg = segment(rd, seg);
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            if (sg.m0 < sg.m1) {                                         // wave-uniform
                uint32_t co[5];
                macro_offsets(co, sg.tile);
                const uint8_t *tb = W + (size_t)sg.tile * 16 * nb01;
                if (rd != 0 || seg != 0) {
#pragma unroll
                    for (int j = 0; j < 5; j++) v[j] = *reinterpret_cast<const u32x4 *>(tb + (size_t)sg.m0 * MMV_ROW_BYTES + co[j]);
                }
                // Two macro tiles in flight in two register sets used alternately (no register rotation: a copy
                // would force a wait for the loads just issued).  Loads are unconditional, indices past the segment
                // are clamped (the last tile is then re-read and not used).
                u32x4 v2[5];
                {
                    const int mn = min(sg.m0 + 1, sg.m1 - 1);
#pragma unroll
                    for (int j = 0; j < 5; j++) v2[j] = *reinterpret_cast<const u32x4 *>(tb + (size_t)mn * MMV_ROW_BYTES + co[j]);
                }
                auto step = [&](u32x4 (&r)[5], int m, int mnext, bool live) {
                    // registers -> LDS (the wave's LDS operations execute in order, so the previous step's operand
                    // reads are done), then the same registers receive macro tile mnext
#pragma unroll
                    for (int j = 0; j < 4; j++) reinterpret_cast<u32x4 *>(mybuf)[64 * j + lane] = r[j];
                    if (tail_chunk) reinterpret_cast<u32x4 *>(mybuf)[256 + lane] = r[4];
                    const uint8_t *nb = tb + (size_t)min(mnext, sg.m1 - 1) * MMV_ROW_BYTES;
#pragma unroll
                    for (int j = 0; j < 5; j++) r[j] = *reinterpret_cast<const u32x4 *>(nb + co[j]);
                    if (!live) return;                                   // wave-uniform
                    const uint8_t *pa0 = lds + a0_off + (uint32_t)m * a0_step;
                    const uint8_t *pa1 = lds + a1_off + (uint32_t)m * a1_step;
                    const uint8_t *pdx = lds + dx_off + (uint32_t)m * 512u;
#pragma unroll
                    for (int pi = 0; pi < MMV_MACRO_PAIRS; pi++) {
                        // the 16 quants start 2 bytes past a dword boundary in lane groups g < 2: read five
                        // aligned dwords and funnel-shift by 16 or 0 bits
                        const u32x4 wlo = *reinterpret_cast<const u32x4_a4 *>(mybuf + b_al + 68u * pi);
                        const uint32_t whi = *reinterpret_cast<const uint32_t *>(mybuf + b_al + 68u * pi + 16u);
                        const v4i b = {(int)__builtin_amdgcn_alignbit(wlo.y, wlo.x, b_sh), (int)__builtin_amdgcn_alignbit(wlo.z, wlo.y, b_sh),
                                       (int)__builtin_amdgcn_alignbit(wlo.w, wlo.z, b_sh), (int)__builtin_amdgcn_alignbit(whi, wlo.w, b_sh)};
                        const v4i zero = {0, 0, 0, 0};
                        const v4i a0 = *reinterpret_cast<const v4i *>(pa0 + 64 * pi);
                        const float4 dx0 = *reinterpret_cast<const float4 *>(pdx + 128 * pi);
                        const float d0 = h2f(*reinterpret_cast<const unsigned short *>(mybuf + h_off + 68u * pi));
                        const v4i s0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, b, zero, 0, 0, 0);
                        acc[0] = __builtin_fmaf((float)s0.x, d0 * dx0.x, acc[0]);
                        acc[1] = __builtin_fmaf((float)s0.y, d0 * dx0.y, acc[1]);
                        acc[2] = __builtin_fmaf((float)s0.z, d0 * dx0.z, acc[2]);
                        acc[3] = __builtin_fmaf((float)s0.w, d0 * dx0.w, acc[3]);
                        if constexpr (NT == 16) {
                            const v4i a1 = *reinterpret_cast<const v4i *>(pa1 + 64 * pi);
                            const float4 dx1 = *reinterpret_cast<const float4 *>(pdx + 128 * pi + 64);
                            const float d1 = h2f(*reinterpret_cast<const unsigned short *>(mybuf + h_off + 68u * pi + 34u));
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
                const float4 pv = reinterpret_cast<const float4 *>(lds + buf_off + (uint32_t)w * MMV_MACRO_BYTES)[seg * 64 + lane];
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

// Tokens one launch takes for this shape: 16 if the 16-token image fits in LDS, else 8, else 0 (not supported).
int mmv_max_tokens(int wtype, int64_t K, int64_t N, const DeviceLimits &lim) {
    if (wtype == T_Q4_K || wtype == T_Q5_K) return mmv_q4k_max_tokens(wtype, K, N, lim);
    if (wtype == T_Q4_0) return mmv_q4_0_max_tokens(K, N, lim);
    if (wtype == T_Q6_K) return mmv_q6k_max_tokens(K, N, lim);
    if (wtype != T_Q8_0 || K % 256 != 0) return 0;
    const int cus = lim.compute_units > 0 ? lim.compute_units : 256;
    if (ceil_div(N, 16) < cus) return 0;                                 // too few 16-row tiles to occupy every CU
    if (N > (1 << 24) || K > (1 << 20)) return 0;                        // the kernel's 32-bit tile arithmetic
    if (mmv_lds_bytes<16, 8>(K) <= (size_t)lim.max_lds_per_block) return 16;
    if (mmv_lds_bytes<8, 8>(K) <= (size_t)lim.max_lds_per_block) return 8;
    return 0;
}

template <int NT, int NW, int OCC>
static hipError_t launch_mmv_cfg(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n,
                                 float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st) {
    const size_t lds_bytes = mmv_lds_bytes<NT, NW>(K);
    auto kfn = mmv_q8_0_kernel<NT, NW, OCC>;
    static LdsGrant grant;                                               // one per kernel instantiation
    if (hipError_t e = grant_dynamic_lds(kfn, lds_bytes, lim, grant); e != hipSuccess) return e;
    const int cus = lim.compute_units > 0 ? lim.compute_units : 256;
    const int64_t tiles = ceil_div(N, 16);
    constexpr int per_cu = OCC * 4 / NW;                                 // workgroups resident per CU
    const int64_t groups = tiles < (int64_t)cus * per_cu ? tiles : (int64_t)cus * per_cu;
    hipLaunchKernelGGL(kfn, dim3((unsigned)groups), dim3(NW * 64), lds_bytes, st, (const uint8_t *)W, nb01, K, N,
                       (const uint8_t *)ws, ws_stride, n, y, ldy);
    return hipGetLastError();
}

template <int NT>
static hipError_t launch_mmv_nt(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n,
                                float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st) {
    // one 8-wave group per CU (two groups with half the tiles each measured slower)
    if (mmv_lds_bytes<NT, 8>(K) <= (size_t)lim.max_lds_per_block)
        return launch_mmv_cfg<NT, 8, 2>(W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st);
    return hipErrorInvalidValue;
}

hipError_t launch_mmv(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n,
                      float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st) {
    if (wtype == T_Q4_K || wtype == T_Q5_K) return launch_mmv_q4k(wtype, W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st);
    if (wtype == T_Q4_0) return launch_mmv_q4_0(W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st);
    if (wtype == T_Q6_K) return launch_mmv_q6k(W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st);
    if (wtype != T_Q8_0 || n < 1 || n > 16) return hipErrorInvalidValue;
    if (N <= 0) return hipSuccess;
    if (n <= 8) return launch_mmv_nt<8>(W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st);
    return launch_mmv_nt<16>(W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st);
}

}  // namespace chip
