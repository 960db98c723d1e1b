// The two matmuls of attention over an F16 KV cache, LM_GGML_OP_MUL_MAT with an F16 src0 that is a strided, batched view
// (reference llama-graph.cpp:1120 kq = mul_mat(k, q) and :1154 kqv = mul_mat(v, kq); CPU path
// lm_ggml_compute_forward_mul_mat, ggml-cpu/ggml-cpu.c:1177-1456, with type_traits_cpu[LM_GGML_TYPE_F16]: src1 rounded to
// fp16 by lm_ggml_cpu_fp32_to_fp16, lm_ggml_vec_dot_f16 accumulating the products of the widened halves in fp32, src0's
// batch index = src1's batch index / r2).
//
//   y[b][t][r] = sum_k  W[b / r2][r][k] * fp16(x[b][t][k])        b < ne12 = ne02 * r2, t < n, r < N
//
// kq:  W = the K cache seen as [head_dim, n_kv, n_head_kv]: rows of head_dim halves, row stride one cache position.
// kqv: W = the transposed V cache seen as [n_kv, head_dim, n_head_kv]: rows of n_kv halves.
//
// A workgroup handles one src0 batch (KV head) and with it the r2 src1 batches (query heads) that share it, so a row of
// the cache is read once for all of them.  The (query head, token) pairs of the KV head are its "columns".
//
// Few columns (decode) - bound: the cache bytes (HBM), in practice launch and memory latency:
//   short rows (K <= 256, kq): LPR = 8, 16 or 32 lanes share a row and a wave reads 64 / LPR rows per load; the lane's
//     slice of every column is rounded to fp16 once and stays in registers while the wave walks the rows.
//   long rows (kqv): a workgroup takes four rows, its four waves a quarter of K each; the activations are read once for
//     the four rows; partial sums meet in LDS.
// Many columns (prefill): the columns of a KV head are the token rows of a GEMM against that head's cache rows, so
//   the work goes to the fp16 MFMA GEMM in its row-gather mode (the mode MUL_MAT_ID uses): activations rounded to fp16
//   into a workspace, one (KV head, 64-column tile) list entry per workgroup column.
// Activations are rounded with v_cvt_f16_f32 (nearest even) and multiplied as halves by v_fma_mix_f32 with an fp32
// accumulator.  The summation order differs from the reference's 4 x 8-lane accumulators, so parity is a tolerance
// (1e-5 of sum |terms|), as for the other fp32-accumulating kernels.
#include "dev_common.h"
#include "kernels.h"
#include "act_layout.h"
#include <cstdlib>

namespace chip {

namespace {

constexpr int AM_THREADS = 256;
constexpr int AM_WAVES = AM_THREADS / 64;
constexpr int AM_COLS = 4;                   // columns per pass: r2 = 4 with one token is one pass

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ u32x4 round8(const float4 a, const float4 b) {
    const half2_t h0 = {(_Float16)a.x, (_Float16)a.y}, h1 = {(_Float16)a.z, (_Float16)a.w};       // round to nearest even
    const half2_t h2 = {(_Float16)b.x, (_Float16)b.y}, h3 = {(_Float16)b.z, (_Float16)b.w};
    u32x4 r;
    r.x = __builtin_bit_cast(uint32_t, h0); r.y = __builtin_bit_cast(uint32_t, h1);
    r.z = __builtin_bit_cast(uint32_t, h2); r.w = __builtin_bit_cast(uint32_t, h3);
    return r;
}
__device__ __forceinline__ float dot8(const u32x4 w, const u32x4 x, float acc) {
    const uint32_t ws[4] = {w.x, w.y, w.z, w.w}, xs[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const half2_t wv = __builtin_bit_cast(half2_t, ws[i]), xv = __builtin_bit_cast(half2_t, xs[i]);
        acc = __builtin_fmaf((float)wv.x, (float)xv.x, acc);
        acc = __builtin_fmaf((float)wv.y, (float)xv.y, acc);
    }
    return acc;
}

// Sum over the LPR lanes that share a row (LPR consecutive lanes, LPR in {8, 16, 32, 64}); every lane of the group gets it.
template <int LPR> __device__ __forceinline__ float group_sum(float v) {
    v += dpp_get<0xB1>(v);                                   // quad_perm [1,0,3,2]
    v += dpp_get<0x4E>(v);                                   // quad_perm [2,3,0,1]
    v += dpp_get<0x141>(v);                                  // row_half_mirror: sums of 8
    if constexpr (LPR >= 16) v += dpp_get<0x140>(v);         // row_mirror: sums of 16
    if constexpr (LPR >= 32) v += __shfl_xor(v, 16);
    if constexpr (LPR >= 64) v += __shfl_xor(v, 32);
    return v;
}

struct BatchedArgs {
    const uint8_t *W; size_t nb01, nb02;
    int64_t K, N;
    const float *x; int64_t ldx1, ldx2;      // token and batch strides of src1, in floats
    int64_t n, r2;
    float *y; int64_t ldy1, ldy2;            // token and batch strides of dst, in floats
};
// Column c of KV head b0: query head c % r2 of its group, token c / r2 (32-bit division: 64-bit is a long software routine).
__device__ __forceinline__ const float *col_x(const BatchedArgs &a, int64_t b0, int64_t c) {
    const uint32_t r2 = (uint32_t)a.r2, t = (uint32_t)c / r2, h = (uint32_t)c - t * r2;
    return a.x + (b0 * a.r2 + h) * a.ldx2 + (int64_t)t * a.ldx1;
}
__device__ __forceinline__ float *col_y(const BatchedArgs &a, int64_t b0, int64_t c) {
    const uint32_t r2 = (uint32_t)a.r2, t = (uint32_t)c / r2, h = (uint32_t)c - t * r2;
    return a.y + (b0 * a.r2 + h) * a.ldy2 + (int64_t)t * a.ldy1;
}

// ---- short rows: K <= 8 * LPR, one 16-byte chunk per lane ----
template <int LPR>
__global__ __launch_bounds__(AM_THREADS) void mm_f16_short_rows_kernel(BatchedArgs a) {
    constexpr int RPS = 64 / LPR;                                    // rows per wave step
    constexpr int UNROLL = 4;                                        // row steps in flight
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane % LPR, grp = lane / LPR;
    const int64_t b0 = blockIdx.y;
    const uint8_t *Wb = a.W + b0 * a.nb02;
    const bool has_chunk = sub < a.K / 8;
    const int64_t cols = a.r2 * a.n;
    const int64_t row_step = (int64_t)gridDim.x * AM_WAVES * RPS;
    const int64_t row0 = ((int64_t)blockIdx.x * AM_WAVES + wave) * RPS + grp;
    for (int64_t c0 = 0; c0 < cols; c0 += AM_COLS) {
        u32x4 xh[AM_COLS];
#pragma unroll
        for (int j = 0; j < AM_COLS; j++) {
            const int64_t c = c0 + j < cols ? c0 + j : cols - 1;                  // clamped: the load stays in bounds, the result is unused
            xh[j] = u32x4{0u, 0u, 0u, 0u};
            if (has_chunk) {
                const float4 *xp = reinterpret_cast<const float4 *>(col_x(a, b0, c) + 8 * sub);
                xh[j] = round8(xp[0], xp[1]);
            }
        }
        for (int64_t rbase = row0; rbase < a.N; rbase += UNROLL * row_step) {
            u32x4 w[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                const int64_t row = rbase + u * row_step;
                w[u] = u32x4{0u, 0u, 0u, 0u};
                if (row < a.N && has_chunk) w[u] = *reinterpret_cast<const u32x4 *>(Wb + row * a.nb01 + 16 * sub);
            }
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                const int64_t row = rbase + u * row_step;
                float acc[AM_COLS];
#pragma unroll
                for (int j = 0; j < AM_COLS; j++) {
                    acc[j] = group_sum<LPR>(dot8(w[u], xh[j], 0.0f));
                }
                if (sub == 0 && row < a.N) {
#pragma unroll
                    for (int j = 0; j < AM_COLS; j++)
                        if (c0 + j < cols) col_y(a, b0, c0 + j)[row] = acc[j];
                }
            }
        }
    }
}

// ---- long rows: a workgroup takes AM_ROWS rows, wave w the chunks w * 64 + lane, + 256, ... of each ----
constexpr int AM_ROWS = 4;
__global__ __launch_bounds__(AM_THREADS) void mm_f16_long_rows_kernel(BatchedArgs a) {
    __shared__ float part[AM_WAVES][AM_ROWS][AM_COLS];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t b0 = blockIdx.y;
    const uint8_t *Wb = a.W + b0 * a.nb02;
    const int64_t chunks = a.K / 8;
    const int64_t cols = a.r2 * a.n;
    for (int64_t r0 = (int64_t)blockIdx.x * AM_ROWS; r0 < a.N; r0 += (int64_t)gridDim.x * AM_ROWS) {
        const uint8_t *wrow[AM_ROWS];
#pragma unroll
        for (int r = 0; r < AM_ROWS; r++) wrow[r] = Wb + (r0 + r < a.N ? r0 + r : a.N - 1) * a.nb01;      // clamped, unused past N
        for (int64_t c0 = 0; c0 < cols; c0 += AM_COLS) {
            const float *xc[AM_COLS];
#pragma unroll
            for (int j = 0; j < AM_COLS; j++) xc[j] = col_x(a, b0, c0 + j < cols ? c0 + j : cols - 1);
            float acc[AM_ROWS][AM_COLS];
#pragma unroll
            for (int r = 0; r < AM_ROWS; r++)
#pragma unroll
                for (int j = 0; j < AM_COLS; j++) acc[r][j] = 0.0f;
            for (int64_t ch = wave * 64 + lane; ch < chunks; ch += AM_THREADS) {
                u32x4 w[AM_ROWS], xh[AM_COLS];
#pragma unroll
                for (int r = 0; r < AM_ROWS; r++) w[r] = *reinterpret_cast<const u32x4 *>(wrow[r] + 16 * ch);
#pragma unroll
                for (int j = 0; j < AM_COLS; j++) {
                    const float4 *xp = reinterpret_cast<const float4 *>(xc[j] + 8 * ch);
                    xh[j] = round8(xp[0], xp[1]);
                }
#pragma unroll
                for (int r = 0; r < AM_ROWS; r++)
#pragma unroll
                    for (int j = 0; j < AM_COLS; j++) acc[r][j] = dot8(w[r], xh[j], acc[r][j]);
            }
#pragma unroll
            for (int r = 0; r < AM_ROWS; r++)
#pragma unroll
                for (int j = 0; j < AM_COLS; j++) {
                    const float v = group_sum<64>(acc[r][j]);
                    if (lane == 0) part[wave][r][j] = v;
                }
            __syncthreads();
            if (threadIdx.x < AM_ROWS * AM_COLS) {
                const int r = threadIdx.x / AM_COLS, j = threadIdx.x % AM_COLS;
                if (r0 + r < a.N && c0 + j < cols)
                    col_y(a, b0, c0 + j)[r0 + r] = (part[0][r][j] + part[1][r][j]) + (part[2][r][j] + part[3][r][j]);
            }
            __syncthreads();
        }
    }
}

// ---- many columns: fp16 rows for the GEMM and its (KV head, tile) list ----
// Row R = b * n + t of the workspace and of y is column (query head b, token t); the pairs of KV head e are the rows
// e * r2 * n ... (e + 1) * r2 * n - 1, in order.
__global__ __launch_bounds__(AM_THREADS) void mm_f16_round_rows_kernel(const float *__restrict__ x, int64_t ldx1, int64_t ldx2,
                                                                       int64_t n, int64_t K, uint8_t *__restrict__ ws, size_t ws_stride) {
    // a workgroup takes as many tokens of one batch as its threads cover with one 8-value chunk each (16 for K = 128)
    const uint32_t chunks = (uint32_t)(K / 8);
    const uint32_t per = chunks >= AM_THREADS ? 1u : AM_THREADS / chunks;
    const int64_t b = blockIdx.y;
    for (uint32_t i = threadIdx.x; i < per * chunks; i += AM_THREADS) {
        const uint32_t r = i / chunks, ch = i - r * chunks;
        const int64_t t = (int64_t)blockIdx.x * per + r;
        if (t >= n) continue;
        const float4 *xp = reinterpret_cast<const float4 *>(x + b * ldx2 + t * ldx1 + 8 * ch);
        reinterpret_cast<u32x4 *>(ws + (size_t)(b * n + t) * ws_stride)[ch] = round8(xp[0], xp[1]);
    }
}
__global__ __launch_bounds__(AM_THREADS) void mm_f16_tile_list_kernel(int64_t ne02, int64_t per_head, int tile_tokens,
                                                                      int32_t *__restrict__ perm, int32_t *__restrict__ offsets,
                                                                      int32_t *__restrict__ tiles) {
    const int64_t i0 = (int64_t)blockIdx.x * AM_THREADS + threadIdx.x, step = (int64_t)gridDim.x * AM_THREADS;
    const int64_t tiles_per_head = ceil_div(per_head, (int64_t)tile_tokens);
    for (int64_t i = i0; i < ne02 * per_head; i += step) perm[i] = (int32_t)i;
    for (int64_t i = i0; i <= ne02; i += step) offsets[i] = (int32_t)(i * per_head);
    for (int64_t i = i0; i < ne02 * tiles_per_head; i += step)
        tiles[1 + i] = (int32_t)(i / tiles_per_head) | (int32_t)((i % tiles_per_head) << MOE_EXPERT_BITS);
    if (i0 == 0) tiles[0] = (int32_t)(ne02 * tiles_per_head);
}

constexpr int64_t GEMM_MIN_COLS = 64;        // columns per KV head from which the GEMM route is taken

struct GemmPlan { bool use; size_t act_stride, off_perm, off_offsets, off_tiles, bytes; int64_t n_tiles; int tile; };
GemmPlan gemm_plan(int64_t K, int64_t N, int64_t ne02, int64_t r2, int64_t n) {
    GemmPlan p{};
    const int64_t per_head = r2 * n;
    p.use = K >= 64 && K % 8 == 0 && N >= 32 && per_head >= GEMM_MIN_COLS && ne02 < (1 << MOE_EXPERT_BITS) && ne02 * per_head < (1LL << 30);
    if (!p.use) return p;
    p.act_stride = f16_stride(K);
    // 128 x 128 tiles once they still give every CU four workgroups, else 64 x 64 (CHIP_ATTN_TILE forces one, for tuning)
    static const int forced = [] { const char *e = getenv("CHIP_ATTN_TILE"); return e ? atoi(e) : 0; }();
    p.tile = (N >= 128 && per_head >= 128 && ne02 * ceil_div(per_head, (int64_t)128) * ceil_div(N, (int64_t)128) >= 1024) ? 128 : 64;
    if (forced == 64 || forced == 128) p.tile = forced;
    p.n_tiles = ne02 * ceil_div(per_head, (int64_t)p.tile);
    if (p.n_tiles > 65535) { p.use = false; return p; }                  // one grid row per list entry
    p.off_perm = align128((size_t)(ne02 * per_head) * p.act_stride);
    p.off_offsets = p.off_perm + align128((size_t)(ne02 * per_head) * 4);
    p.off_tiles = p.off_offsets + align128((size_t)(ne02 + 1) * 4);
    p.bytes = p.off_tiles + align128((size_t)(1 + p.n_tiles) * 4);
    return p;
}

}  // namespace

bool mul_mat_f16_batched_supported(int64_t K) { return K > 0 && K % 8 == 0; }

size_t mul_mat_f16_batched_workspace_size(int64_t K, int64_t N, int64_t ne02, int64_t r2, int64_t n) {
    if (K <= 0 || N <= 0 || ne02 <= 0 || r2 <= 0 || n <= 0) return 0;
    return gemm_plan(K, N, ne02, r2, n).bytes;
}

hipError_t launch_mul_mat_f16_batched(const void *W, size_t nb01, size_t nb02, int64_t K, int64_t N, int64_t ne02, const float *x,
                                      int64_t ldx1, int64_t ldx2, int64_t n, int64_t r2, float *y, int64_t ldy1, int64_t ldy2,
                                      void *workspace, size_t workspace_bytes, const DeviceLimits &lim, hipStream_t st) {
    if (N <= 0 || n <= 0 || ne02 <= 0 || r2 <= 0) return hipSuccess;
    if (!mul_mat_f16_batched_supported(K) || ne02 > 65535 || r2 * n > 0x7fffffff) return hipErrorInvalidValue;
    const GemmPlan plan = gemm_plan(K, N, ne02, r2, n);
    // the GEMM writes row R of y at R * ldy1: the batches of y must follow each other without a gap
    if (plan.use && workspace && workspace_bytes >= plan.bytes && ldy2 == n * ldy1 && n <= 65535 && ne02 * r2 <= 65535) {
        uint8_t *ws = (uint8_t *)workspace;
        int32_t *perm = (int32_t *)(ws + plan.off_perm), *offsets = (int32_t *)(ws + plan.off_offsets), *tiles = (int32_t *)(ws + plan.off_tiles);
        const int64_t chunks = K / 8, per = chunks >= AM_THREADS ? 1 : AM_THREADS / chunks;
        hipLaunchKernelGGL(mm_f16_round_rows_kernel, dim3((unsigned)ceil_div(n, per), (unsigned)(ne02 * r2)), dim3(AM_THREADS), 0, st, x,
                           ldx1, ldx2, n, K, ws, plan.act_stride);
        hipLaunchKernelGGL(mm_f16_tile_list_kernel, dim3(64), dim3(AM_THREADS), 0, st, ne02, r2 * n, plan.tile, perm, offsets, tiles);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
        const RowGather rg{perm, offsets, tiles, 1, 1, nb02};
        return launch_gemm_f16(W, nb01, K, N, ws, plan.act_stride, ne02 * r2 * n, y, ldy1, lim, st, &rg, plan.n_tiles, plan.tile);
    }
    const BatchedArgs a{(const uint8_t *)W, nb01, nb02, K, N, x, ldx1, ldx2, n, r2, y, ldy1, ldy2};
    const int cus = lim.compute_units > 0 ? lim.compute_units : 256;
    if (K <= 256) {
        const int lpr = K <= 64 ? 8 : K <= 128 ? 16 : 32;
        // a wave walks at least four row steps (its loads in flight together); about four workgroups per CU over all KV heads
        const int64_t rows_per_wg = AM_WAVES * (64 / lpr) * 4;
        int64_t gx = ceil_div(N, rows_per_wg);
        const int64_t cap = ceil_div((int64_t)cus * 4, ne02);
        if (gx > cap) gx = cap;
        const dim3 grid((unsigned)gx, (unsigned)ne02);
        switch (lpr) {
            case 8:  hipLaunchKernelGGL(mm_f16_short_rows_kernel<8>, grid, dim3(AM_THREADS), 0, st, a); break;
            case 16: hipLaunchKernelGGL(mm_f16_short_rows_kernel<16>, grid, dim3(AM_THREADS), 0, st, a); break;
            default: hipLaunchKernelGGL(mm_f16_short_rows_kernel<32>, grid, dim3(AM_THREADS), 0, st, a); break;
        }
    } else {
        int64_t gx = ceil_div(N, (int64_t)AM_ROWS);
        const int64_t cap = ceil_div((int64_t)cus * 8, ne02);
        if (gx > cap) gx = cap;
        hipLaunchKernelGGL(mm_f16_long_rows_kernel, dim3((unsigned)gx, (unsigned)ne02), dim3(AM_THREADS), 0, st, a);
    }
    return hipGetLastError();
}

}  // namespace chip
