// Prefill GEMM for gfx950 over F16 weights and activations rounded to fp16: Y[t][r] = sum_k w[r][k] * a[t][k], the
// batched form of lm_ggml_vec_dot_f16 (reference ggml-cpu/ggml-cpu.c type_traits_cpu[LM_GGML_TYPE_F16], vec.cpp) as
// driven by lm_ggml_compute_forward_mul_mat (ggml-cpu/ggml-cpu.c:1257-1449): fp16 products, fp32 accumulation.
//
// v_mfma_f32_32x32x16_f16 multiplies a 32-row x 16-k weight tile by a 16-k x 32-token activation tile; products of
// fp16 numbers are exact in fp32 and the accumulator is fp32, so only the order of the additions differs from the
// reference.  Weights [N][K] and the fp16 workspace [n][K] are both contiguous along k, which is how a lane feeds the
// MFMA (8 consecutive k), so staging is a plain copy: 16-byte cells [k-group][k-half][row] in LDS, double buffered
// over stages of 64 k, the next stage's global loads in flight during the current stage's MFMAs.  There is no vector
// work per MFMA at all; a wave owns TM x TN tiles so that an LDS cell feeds TM (TN) MFMAs.
#include "dev_common.h"
#include "act_layout.h"
#include "kernels.h"
#include <cstdlib>

namespace chip {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int F16_KG = 4;                     // 16-value k-groups per LDS stage

template <int TM, int TN, int WR, int WC>
struct F16Cfg {
    static constexpr int NW = WR * WC, NT = NW * 64;
    static constexpr int BM = 32 * TM * WR;                        // weight rows per workgroup
    static constexpr int BN = 32 * TN * WC;                        // tokens per workgroup
    // plane stride 2 mod 16 cells: the staging threads of one wave spread over the bank groups
    static constexpr int A_PLANE = BM + 2, B_PLANE = BN + 2;
    static constexpr int CELLS = F16_KG * 2;                       // 16-byte cells per row and stage
    static constexpr size_t OFF_A = 0;
    static constexpr size_t OFF_B = OFF_A + (size_t)CELLS * A_PLANE * 16;
    static constexpr size_t STAGE = OFF_B + (size_t)CELLS * B_PLANE * 16;
    static constexpr int W_ITEMS = BM * CELLS, X_ITEMS = BN * CELLS;
    static constexpr int W_PER_T = W_ITEMS / NT, X_PER_T = X_ITEMS / NT;
    static_assert(W_ITEMS % NT == 0 && X_ITEMS % NT == 0, "staging items divide evenly over the threads");
};

// XF32 (row-gather mode only): the activations are read as fp32 from their own tensor - row R of the gather is token
// R % n of batch R / n - and rounded to fp16 (nearest even) on their way into LDS, instead of from an fp16 copy in the
// workspace.  Pays when the output has one or two row tiles (kqv: a head's 64 - 256 rows), so that the fp32 rows are read
// once or twice; with many row tiles the fp16 copy, read back many times, is the cheaper source.
__device__ __forceinline__ u32x4 round8_f16(const float4 a, const float4 b) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const h2 h0 = {(_Float16)a.x, (_Float16)a.y}, h1 = {(_Float16)a.z, (_Float16)a.w};
    const h2 h2v = {(_Float16)b.x, (_Float16)b.y}, h3 = {(_Float16)b.z, (_Float16)b.w};
    u32x4 r;
    r.x = __builtin_bit_cast(uint32_t, h0); r.y = __builtin_bit_cast(uint32_t, h1);
    r.z = __builtin_bit_cast(uint32_t, h2v); r.w = __builtin_bit_cast(uint32_t, h3);
    return r;
}

template <int TM, int TN, int WR, int WC, int OCC, bool GATHER, bool XF32 = false>
__global__ __launch_bounds__(WR *WC * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void gemm_f16_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N, const uint8_t *__restrict__ ws,
                     size_t ws_stride, int64_t M, float *__restrict__ y, int64_t ldy, TileMap map, RowGather rg, F32Rows fs) {
    static_assert(!XF32 || GATHER, "fp32 activation rows come with the row-gather mode");
    using C = F16Cfg<TM, TN, WR, WC>;
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave / WC, wc = wave % WC;
    const int half = lane >> 5, l32 = lane & 31;
    const TileCoord tc = xcd_tile(blockIdx.x, map);
    if (tc.row_tile >= map.row_tiles || tc.tok_tile >= map.tok_tiles) return;
    const int64_t row_base = (int64_t)tc.row_tile * C::BM;
    size_t w_offset;
    const GatherView gv = resolve_gather<GATHER>(rg, w_offset, M);                   // MUL_MAT_ID: this expert's rows
    W += w_offset;
    if (gv.tok_tile < 0) return;
    const int64_t tok_base = (int64_t)(GATHER ? gv.tok_tile : tc.tok_tile) * C::BN;
    if (tok_base >= M) return;
    // The row-gather instantiation also takes K that is not a multiple of the 64-value stage (the attention matmul over
    // n_kv cache positions, a multiple of 8): cells of the last stage that lie past K are zeroed on both sides.
    constexpr bool KTAIL = GATHER;
    const int nstages = (int)(KTAIL ? ceil_div(K, (int64_t)(16 * F16_KG)) : K / (16 * F16_KG));
    constexpr int STAGE_BYTES = 16 * F16_KG * 2;                   // bytes of one row per stage
    static_assert(C::NT % C::CELLS == 0, "a thread's items all have the same cell index");
    const int my_cell = tid % C::CELLS;

    // item = (row, cell): 8 consecutive threads copy 128 contiguous bytes of one row
    const uint8_t *wsrc[C::W_PER_T], *xsrc[C::X_PER_T];
#pragma unroll
    for (int i = 0; i < C::W_PER_T; i++) {
        const int item = tid + i * C::NT;
        wsrc[i] = W + (size_t)min(row_base + item / C::CELLS, N - 1) * nb01 + 16 * (item % C::CELLS);
    }
#pragma unroll
    for (int i = 0; i < C::X_PER_T; i++) {
        const int item = tid + i * C::NT;
        const int64_t arow = gv.act_row(min(tok_base + item / C::CELLS, M - 1));
        if constexpr (XF32) {
            const uint32_t b = (uint32_t)arow / (uint32_t)fs.n, t = (uint32_t)arow - b * (uint32_t)fs.n;
            xsrc[i] = reinterpret_cast<const uint8_t *>(fs.x + (int64_t)b * fs.ldx2 + (int64_t)t * fs.ldx1) + 32 * (item % C::CELLS);
        } else {
            xsrc[i] = ws + (size_t)arow * ws_stride + 16 * (item % C::CELLS);
        }
    }
    u32x4 wq[C::W_PER_T], xq[C::X_PER_T];

    auto fetch = [&](int stage) {
        const bool live = !KTAIL || (int64_t)stage * (16 * F16_KG) + 8 * my_cell < K;
        const size_t off = live ? (size_t)stage * STAGE_BYTES : 0;                   // a dead cell re-reads stage 0 (in bounds) and is zeroed
        const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < C::W_PER_T; i++) {
            wq[i] = *reinterpret_cast<const u32x4 *>(wsrc[i] + off);
            if (KTAIL && !live) wq[i] = z;
        }
#pragma unroll
        for (int i = 0; i < C::X_PER_T; i++) {
            if constexpr (XF32) {
                const float4 *xp = reinterpret_cast<const float4 *>(xsrc[i] + 2 * off);      // a stage is twice the bytes in fp32
                xq[i] = round8_f16(xp[0], xp[1]);
            } else {
                xq[i] = *reinterpret_cast<const u32x4 *>(xsrc[i] + off);
            }
            if (KTAIL && !live) xq[i] = z;
        }
    };
    auto commit = [&](int buf) {
        u32x4 *A = reinterpret_cast<u32x4 *>(lds + (size_t)buf * C::STAGE + C::OFF_A);
        u32x4 *B = reinterpret_cast<u32x4 *>(lds + (size_t)buf * C::STAGE + C::OFF_B);
#pragma unroll
        for (int i = 0; i < C::W_PER_T; i++) {
            const int item = tid + i * C::NT;
            A[(item % C::CELLS) * C::A_PLANE + item / C::CELLS] = wq[i];
        }
#pragma unroll
        for (int i = 0; i < C::X_PER_T; i++) {
            const int item = tid + i * C::NT;
            B[(item % C::CELLS) * C::B_PLANE + item / C::CELLS] = xq[i];
        }
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int c = 0; c < TN; c++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[a][c][v] = 0.f;

    fetch(0);
    commit(0);
    __syncthreads();

    for (int s = 0; s < nstages; s++) {
        const int buf = s & 1;
        fetch(min(s + 1, nstages - 1));                              // unconditional: the last stage is loaded twice
        const f16x8 *A = reinterpret_cast<const f16x8 *>(lds + (size_t)buf * C::STAGE + C::OFF_A);
        const f16x8 *B = reinterpret_cast<const f16x8 *>(lds + (size_t)buf * C::STAGE + C::OFF_B);
#pragma unroll
        for (int g = 0; g < F16_KG; g++) {
            f16x8 af[TM], bf[TN];
#pragma unroll
            for (int a = 0; a < TM; a++) af[a] = A[(g * 2 + half) * C::A_PLANE + (wr * TM + a) * 32 + l32];
#pragma unroll
            for (int c = 0; c < TN; c++) bf[c] = B[(g * 2 + half) * C::B_PLANE + (wc * TN + c) * 32 + l32];
#pragma unroll
            for (int a = 0; a < TM; a++)
#pragma unroll
                for (int c = 0; c < TN; c++) acc[a][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[a], bf[c], acc[a][c], 0, 0, 0);
        }
        commit(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: register v of tile (a, c) is row 8*(v/4) + 4*half + v%4, token l32 ----
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int c = 0; c < TN; c++) {
            const int64_t tok = tok_base + (wc * TN + c) * 32 + l32;
            if (tok >= M) continue;
            const int64_t orow = gv.out_row(tok);
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int64_t row = row_base + (wr * TM + a) * 32 + 8 * g + 4 * half;
                float *dst = y + (size_t)orow * ldy + row;
                if (row + 3 < N && (((uintptr_t)dst) & 15) == 0) {
                    *reinterpret_cast<float4 *>(dst) = make_float4(acc[a][c][4 * g], acc[a][c][4 * g + 1], acc[a][c][4 * g + 2], acc[a][c][4 * g + 3]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (row + e < N) dst[e] = acc[a][c][4 * g + e];
                }
            }
        }
}

// rows must be 16-byte aligned (the weight alignment rule of the C-ABI) and K a multiple of the 64-value stage
bool gemm_f16_supported(int64_t K, int64_t N, int64_t n) { return K >= 64 && K % (16 * F16_KG) == 0 && N >= 1 && n >= 32; }

template <int TM, int TN, int WR, int WC, int OCC, bool GATHER, bool XF32 = false>
static hipError_t launch_f16(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int64_t M,
                             float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const RowGather &rg, int64_t n_as,
                             const F32Rows &fs = F32Rows{nullptr, 0, 0, 1}) {
    using C = F16Cfg<TM, TN, WR, WC>;
    const size_t lds_bytes = 2 * C::STAGE;
    auto kfn = gemm_f16_kernel<TM, TN, WR, WC, OCC, GATHER, XF32>;
    static LdsGrant grant;
    if (hipError_t e = grant_dynamic_lds(kfn, lds_bytes, lim, grant); e != hipSuccess) return e;
    const TileMap map = make_tile_map(ceil_div(N, C::BM), GATHER ? 1 : ceil_div(M, C::BN), 32 * (4 * OCC / C::NW > 0 ? 4 * OCC / C::NW : 1));
    hipLaunchKernelGGL(kfn, dim3(map.grid, (unsigned)n_as), dim3(C::NT), lds_bytes, st, (const uint8_t *)W, nb01, K, N,
                       (const uint8_t *)ws, ws_stride, M, y, ldy, map, rg, fs);
    return hipGetLastError();
}

int gemm_f16_moe_tile_tokens() { return F16Cfg<1, 1, 2, 2>::BN; }      // the 64 x 64 shape serves the expert groups

hipError_t launch_gemm_f16(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int64_t M,
                           float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const RowGather *rgp, int64_t n_as,
                           int gather_tile, const F32Rows *f32_rows) {
    if (M <= 0 || N <= 0 || n_as <= 0) return hipSuccess;
    const RowGather rg = rgp ? *rgp : RowGather{nullptr, nullptr, nullptr, 1, 1, 0};
    const int64_t cus = lim.compute_units > 0 ? lim.compute_units : 256;
    if (rg.perm) {                                                                   // row groups: the tile list was built for 64 or 128 tokens
        if (f32_rows) {
            if (gather_tile == 128) return launch_f16<2, 2, 2, 2, 2, true, true>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, *f32_rows);
            if (gather_tile != 64) return hipErrorInvalidValue;
            return launch_f16<1, 1, 2, 2, 4, true, true>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, *f32_rows);
        }
        if (gather_tile == 128) return launch_f16<2, 2, 2, 2, 2, true>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);
        if (gather_tile != 64) return hipErrorInvalidValue;
        return launch_f16<1, 1, 2, 2, 4, true>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);
    }
    if (f32_rows) return hipErrorInvalidValue;
    const int64_t g128 = ceil_div(N, 128) * ceil_div(M, 128);
    const int cfg = (int)tune("CHIP_GEMM_F16_CFG", g128 >= cus ? 0 : 1);
    switch (cfg) {
        case 0: return launch_f16<2, 2, 2, 2, 2, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);       // 128 x 128, 4 waves
        case 1: return launch_f16<1, 1, 2, 2, 4, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);       // 64 x 64, 4 waves
        case 2: return launch_f16<2, 2, 2, 4, 2, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);       // 128 x 256, 8 waves
        case 3: return launch_f16<2, 4, 2, 2, 2, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);       // 128 x 256, 4 waves
        default: return hipErrorInvalidValue;
    }
}

}  // namespace chip
