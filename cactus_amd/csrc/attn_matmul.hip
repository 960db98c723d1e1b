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
    float *y2; int64_t ld2y1, ld2y2;         // optional second copy of dst under strides of its own (the dot-product kernels only)
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
__device__ __forceinline__ float *col_y2(const BatchedArgs &a, int64_t b0, int64_t c) {
    const uint32_t r2 = (uint32_t)a.r2, t = (uint32_t)c / r2, h = (uint32_t)c - t * r2;
    return a.y2 + (b0 * a.r2 + h) * a.ld2y2 + (int64_t)t * a.ld2y1;
}

// ---- short rows: K <= 8 * LPR, one 16-byte chunk per lane ----
template <int LPR>
__global__ __launch_bounds__(AM_THREADS) void mm_f16_short_rows_kernel(BatchedArgs a) {
    constexpr int RPS = 64 / LPR;                                    // rows per wave step
    constexpr int UNROLL = 4;                                        // row steps in flight (2 and 8 measured slower: kq of a decode step 5.7 -> 5.95 / 6.65 us)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane % LPR, grp = lane / LPR;
    const int64_t b0 = blockIdx.y;
    const uint8_t *Wb = a.W + b0 * a.nb02;
    const bool has_chunk = sub < a.K / 8;
    const int subc = has_chunk ? sub : 0;                            // lanes past the row's end load chunk 0 and count zeros
    const int64_t cols = a.r2 * a.n;
    const int64_t row_step = (int64_t)gridDim.x * AM_WAVES * RPS;
    const int64_t row0 = ((int64_t)blockIdx.x * AM_WAVES + wave) * RPS + grp;
    const u32x4 zero = u32x4{0u, 0u, 0u, 0u};
    // Every load is unconditional, from a clamped address, so that the columns' and the first rows' requests leave together:
    // one round trip to memory instead of one per column and then one for the rows.
    auto load_rows = [&](int64_t rbase, u32x4 (&w)[UNROLL]) {
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const int64_t row = rbase + u * row_step;
            w[u] = *reinterpret_cast<const u32x4 *>(Wb + (row < a.N ? row : a.N - 1) * a.nb01 + 16 * subc);
        }
    };
    for (int64_t c0 = 0; c0 < cols; c0 += AM_COLS) {
        float4 xlo[AM_COLS], xhi[AM_COLS];
#pragma unroll
        for (int j = 0; j < AM_COLS; j++) {
            const int64_t c = c0 + j < cols ? c0 + j : cols - 1;                  // clamped: the load stays in bounds, the result is unused
            const float4 *xp = reinterpret_cast<const float4 *>(col_x(a, b0, c) + 8 * subc);
            xlo[j] = xp[0];
            xhi[j] = xp[1];
        }
        u32x4 w[UNROLL];
        if (row0 < a.N) load_rows(row0, w);
        u32x4 xh[AM_COLS];
#pragma unroll
        for (int j = 0; j < AM_COLS; j++) xh[j] = has_chunk ? round8(xlo[j], xhi[j]) : zero;
        for (int64_t rbase = row0; rbase < a.N;) {
            const int64_t next = rbase + UNROLL * row_step;
            u32x4 wn[UNROLL];
            if (next < a.N) load_rows(next, wn);
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                const int64_t row = rbase + u * row_step;
                const u32x4 wu = has_chunk ? w[u] : zero;
                float acc[AM_COLS];
#pragma unroll
                for (int j = 0; j < AM_COLS; j++) {
                    acc[j] = group_sum<LPR>(dot8(wu, xh[j], 0.0f));
                }
                if (sub == 0 && row < a.N) {
#pragma unroll
                    for (int j = 0; j < AM_COLS; j++)
                        if (c0 + j < cols) {
                            col_y(a, b0, c0 + j)[row] = acc[j];
                            if (a.y2) col_y2(a, b0, c0 + j)[row] = acc[j];
                        }
                }
            }
            if (next < a.N) {
#pragma unroll
                for (int u = 0; u < UNROLL; u++) w[u] = wn[u];
            }
            rbase = next;
        }
    }
}

// ---- long rows: a workgroup takes AM_ROWS rows, wave w the chunks w * 64 + lane, + 256, ... of each ----
template <int AM_ROWS>
__global__ __launch_bounds__(AM_THREADS) void mm_f16_long_rows_kernel(BatchedArgs a) {
    __shared__ float part[AM_WAVES][AM_ROWS][AM_COLS];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // Workgroups are handed to the 8 XCDs in turn, in the order of their linear index (x fastest).  The KV head is that index
    // modulo the number of heads, so that with 8 KV heads all workgroups of a head run on one XCD and the head's activation
    // columns (the probabilities: 64 KB per head at 4096 positions) reach one L2 instead of all eight.
    const uint32_t linear = blockIdx.x + gridDim.x * blockIdx.y;
    const int64_t b0 = linear % gridDim.y, bx = linear / gridDim.y;
    const uint8_t *Wb = a.W + b0 * a.nb02;
    const int64_t chunks = a.K / 8;
    const int64_t cols = a.r2 * a.n;
    for (int64_t r0 = bx * AM_ROWS; r0 < a.N; r0 += (int64_t)gridDim.x * AM_ROWS) {
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
                if (r0 + r < a.N && c0 + j < cols) {
                    const float v = (part[0][r][j] + part[1][r][j]) + (part[2][r][j] + part[3][r][j]);
                    col_y(a, b0, c0 + j)[r0 + r] = v;
                    if (a.y2) col_y2(a, b0, c0 + j)[r0 + r] = v;
                }
            }
            __syncthreads();
        }
    }
}

// ---- 5 to 63 columns (a few tokens per step): 16 rows x 16 columns x 32 halves per MFMA ----
// Operand layout of v_mfma_f32_16x16x32_f16: lane (i = lane % 16, g = lane / 16) gives the 8 halves k = 8g .. 8g + 7 of row i
// (A, a cache row) or of column i (B, an activation column), i.e. 16-byte chunk 4 * step + g of that row; it receives
// D[4g .. 4g + 3][i], four consecutive rows of column i, which are four consecutive floats of that column's output.
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f16x8 as_halves(const u32x4 v) { return __builtin_bit_cast(f16x8, v); }
__device__ __forceinline__ void store_rows4(float *yp, int64_t row, int64_t N, const f32x4 d) {
    if (row + 3 < N && (((uintptr_t)(yp + row)) & 15) == 0) {
        *reinterpret_cast<f32x4 *>(yp + row) = d;
    } else {
#pragma unroll
        for (int r = 0; r < 4; r++)
            if (row + r < N) yp[row + r] = d[r];
    }
}

// short rows (kq): K <= 32 * KS; the rounded activation columns stay in registers (KS * CG operands), a wave walks 16-row tiles
template <int KS, int CG>
__global__ __launch_bounds__(AM_THREADS) void mm_f16_mfma_short_kernel(BatchedArgs a) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, g = lane >> 4;
    const int64_t b0 = blockIdx.y;
    const uint8_t *Wb = a.W + b0 * a.nb02;
    const int64_t cols = a.r2 * a.n, chunks = a.K / 8;
    u32x4 bx[CG][KS];
    float *yp[CG];
#pragma unroll
    for (int cg = 0; cg < CG; cg++) {
        const int64_t c = cg * 16 + i;
        const float *xc = col_x(a, b0, c < cols ? c : cols - 1);
        yp[cg] = c < cols ? col_y(a, b0, c) : nullptr;
#pragma unroll
        for (int s = 0; s < KS; s++) {
            const int ch = 4 * s + g;
            bx[cg][s] = u32x4{0u, 0u, 0u, 0u};
            if (c < cols && ch < chunks) {
                const float4 *xp = reinterpret_cast<const float4 *>(xc + 8 * ch);
                bx[cg][s] = round8(xp[0], xp[1]);
            }
        }
    }
    const int64_t tiles = ceil_div(a.N, (int64_t)16);
    for (int64_t t = (int64_t)blockIdx.x * AM_WAVES + wave; t < tiles; t += (int64_t)gridDim.x * AM_WAVES) {
        const int64_t row = t * 16 + i;
        u32x4 aw[KS];
#pragma unroll
        for (int s = 0; s < KS; s++) {
            const int ch = 4 * s + g;
            aw[s] = u32x4{0u, 0u, 0u, 0u};
            if (row < a.N && ch < chunks) aw[s] = *reinterpret_cast<const u32x4 *>(Wb + row * a.nb01 + 16 * ch);
        }
#pragma unroll
        for (int cg = 0; cg < CG; cg++) {
            f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int s = 0; s < KS; s++) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_halves(aw[s]), as_halves(bx[cg][s]), acc, 0, 0, 0);
            if (yp[cg]) store_rows4(yp[cg], t * 16 + 4 * g, a.N, acc);
        }
    }
}

// long rows (kqv): a workgroup of AL_WAVES waves takes 16 rows of one KV head; wave w takes the 32-half steps w, w + AL_WAVES, ...
// of K for all columns; the partial tiles meet in LDS and are added in wave order.
constexpr int AL_WAVES = 16;
template <int CG>
__global__ __launch_bounds__(AL_WAVES * 64) void mm_f16_mfma_long_kernel(BatchedArgs a) {
    __shared__ f32x4 part[AL_WAVES][CG][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, g = lane >> 4;
    const int64_t b0 = blockIdx.y, t = blockIdx.x;
    const uint8_t *Wb = a.W + b0 * a.nb02;
    const int64_t cols = a.r2 * a.n, chunks = a.K / 8, steps = ceil_div(chunks, (int64_t)4);
    const int64_t row = t * 16 + i;
    const uint8_t *wrow = Wb + (row < a.N ? row : a.N - 1) * a.nb01;
    const float *xc[CG];
#pragma unroll
    for (int cg = 0; cg < CG; cg++) {
        const int64_t c = cg * 16 + i;
        xc[cg] = col_x(a, b0, c < cols ? c : cols - 1);
    }
    f32x4 acc[CG];
#pragma unroll
    for (int cg = 0; cg < CG; cg++) acc[cg] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    constexpr int UN = CG == 1 ? 8 : CG == 2 ? 4 : 2;                 // steps whose loads are in flight together (128 registers per lane)
    for (int64_t q0 = wave; q0 < steps; q0 += UN * AL_WAVES) {
        u32x4 aw[UN];
        float4 xr[UN][CG][2];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const int64_t ch = 4 * (q0 + u * AL_WAVES) + g;
            const bool in = ch < chunks;
            aw[u] = u32x4{0u, 0u, 0u, 0u};
            if (in && row < a.N) aw[u] = *reinterpret_cast<const u32x4 *>(wrow + 16 * ch);
#pragma unroll
            for (int cg = 0; cg < CG; cg++) {
                xr[u][cg][0] = xr[u][cg][1] = float4{0.0f, 0.0f, 0.0f, 0.0f};
                if (in && cg * 16 + i < cols) {
                    const float4 *xp = reinterpret_cast<const float4 *>(xc[cg] + 8 * ch);
                    xr[u][cg][0] = xp[0];
                    xr[u][cg][1] = xp[1];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UN; u++)
#pragma unroll
            for (int cg = 0; cg < CG; cg++)
                acc[cg] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_halves(aw[u]), as_halves(round8(xr[u][cg][0], xr[u][cg][1])), acc[cg], 0, 0, 0);
    }
#pragma unroll
    for (int cg = 0; cg < CG; cg++) part[wave][cg][lane] = acc[cg];
    __syncthreads();
    // element e of the tile: column group, lane, row within the lane's four
    for (int e = threadIdx.x; e < CG * 64 * 4; e += AL_WAVES * 64) {
        const int cg = e >> 8, ln = (e >> 2) & 63, r = e & 3;
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < AL_WAVES; w++) v += part[w][cg][ln][r];
        const int64_t c = cg * 16 + (ln & 15), rr = t * 16 + 4 * (ln >> 4) + r;
        if (c < cols && rr < a.N) col_y(a, b0, c)[rr] = v;
    }
}

// long rows, K split over workgroups (kqv with 5 to 128 columns): workgroup (slice, KV head) takes AS_SLICE values of K for
// every row and column of the head.  The slice of the activations is rounded to fp16 once into LDS and shared by the
// waves, each of which owns 16-row tiles; the cache and the activations are each read once overall.  The partial
// sums go to the workspace as [slice][KV head][column][row] and a second kernel adds the slices in order.
constexpr int AS_SLICE = 256, AS_WAVES = 8, AS_STEPS = AS_SLICE / 32;
constexpr int AS_XSTRIDE = AS_SLICE * 2 + 16;                       // bytes per column in LDS
constexpr int64_t AS_MAX_COLS = 128, AS_MAX_ROWS = 256;
template <int CG>
__global__ __launch_bounds__(AS_WAVES * 64) void mm_f16_mfma_slice_kernel(BatchedArgs a, float *__restrict__ part) {
    __shared__ __attribute__((aligned(16))) uint8_t xb[CG * 16 * AS_XSTRIDE];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, g = lane >> 4;
    const int64_t slice = blockIdx.x, b0 = blockIdx.y;
    const int64_t cols = a.r2 * a.n, chunks = a.K / 8, ch0 = slice * (AS_SLICE / 8);
    static_assert(16 * (AS_SLICE / 8) == AS_WAVES * 64, "one column group per staging round");
    float4 raw[CG][2];
#pragma unroll
    for (int it = 0; it < CG; it++) {                                   // all loads first, then the rounding and the LDS writes
        const int e = it * (AS_WAVES * 64) + threadIdx.x;
        const int c = e / (AS_SLICE / 8), ch = e % (AS_SLICE / 8);
        raw[it][0] = raw[it][1] = float4{0.0f, 0.0f, 0.0f, 0.0f};
        if (c < cols && ch0 + ch < chunks) {
            const float4 *xp = reinterpret_cast<const float4 *>(col_x(a, b0, c) + 8 * (ch0 + ch));
            raw[it][0] = xp[0];
            raw[it][1] = xp[1];
        }
    }
#pragma unroll
    for (int it = 0; it < CG; it++) {
        const int e = it * (AS_WAVES * 64) + threadIdx.x;
        const int c = e / (AS_SLICE / 8), ch = e % (AS_SLICE / 8);
        *reinterpret_cast<u32x4 *>(xb + c * AS_XSTRIDE + 16 * ch) = round8(raw[it][0], raw[it][1]);
    }
    __syncthreads();
    const uint8_t *Wb = a.W + b0 * a.nb02;
    float *pbase = part + ((slice * gridDim.y + b0) * cols) * a.N;
    for (int64_t t = wave; t * 16 < a.N; t += AS_WAVES) {
        const int64_t row = t * 16 + i;
        u32x4 aw[AS_STEPS];
#pragma unroll
        for (int s = 0; s < AS_STEPS; s++) {
            const int64_t ch = ch0 + 4 * s + g;
            aw[s] = u32x4{0u, 0u, 0u, 0u};
            if (row < a.N && ch < chunks) aw[s] = *reinterpret_cast<const u32x4 *>(Wb + row * a.nb01 + 16 * ch);
        }
#pragma unroll
        for (int cg = 0; cg < CG; cg++) {
            f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int s = 0; s < AS_STEPS; s++) {
                const u32x4 b = *reinterpret_cast<const u32x4 *>(xb + (cg * 16 + i) * AS_XSTRIDE + 16 * (4 * s + g));
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_halves(aw[s]), as_halves(b), acc, 0, 0, 0);
            }
            const int64_t c = cg * 16 + i;
            if (c < cols) store_rows4(pbase + c * a.N, t * 16 + 4 * g, a.N, acc);
        }
    }
}
__global__ __launch_bounds__(AM_THREADS) void mm_f16_slice_sum_kernel(BatchedArgs a, const float *__restrict__ part, int64_t slices,
                                                                      int64_t ne02) {
    const int64_t cols = a.r2 * a.n, per_slice = ne02 * cols * a.N;
    const int64_t e = (int64_t)blockIdx.x * AM_THREADS + threadIdx.x;
    if (e >= per_slice) return;
    float v = 0.0f;
    for (int64_t sl0 = 0; sl0 < slices; sl0 += 8) {                     // eight loads in flight, added in slice order
        float t[8];
#pragma unroll
        for (int j = 0; j < 8; j++) t[j] = sl0 + j < slices ? part[(sl0 + j) * per_slice + e] : 0.0f;
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (sl0 + j < slices) v += t[j];
    }
    const uint32_t N = (uint32_t)a.N, cr = (uint32_t)(e / N), row = (uint32_t)(e - (int64_t)cr * N);     // e < 2^31 (checked by the launcher)
    const uint32_t b0 = cr / (uint32_t)cols, c = cr - b0 * (uint32_t)cols;
    col_y(a, b0, c)[row] = v;
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
    const int64_t min_cols = tune("CHIP_ATTN_GEMM_MIN", GEMM_MIN_COLS);
    p.use = K >= 64 && K % 8 == 0 && N >= 32 && per_head >= min_cols && ne02 < (1 << MOE_EXPERT_BITS) && ne02 * per_head < (1LL << 30);
    if (!p.use) return p;
    p.act_stride = f16_stride(K);
    // 128 x 128 tiles once they still give every CU four workgroups, else 64 x 64
    const int forced = (int)tune("CHIP_ATTN_TILE", 0);
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
// the second copy of the result: written by the dot-product kernels, which take up to AM_COLS (query head, token) pairs per KV head
bool mul_mat_f16_batched_second_copy_supported(int64_t r2, int64_t n) { return r2 > 0 && n > 0 && r2 * n <= AM_COLS; }

// the split-K pair: 5 to AS_MAX_COLS columns per KV head, long rows, up to AS_MAX_ROWS rows (head sizes)
static size_t slice_plan_bytes(int64_t K, int64_t N, int64_t ne02, int64_t r2, int64_t n) {
    const int64_t cols = r2 * n, slices = ceil_div(K, (int64_t)AS_SLICE);
    if (K <= 256 || K % 8 != 0 || cols <= AM_COLS || cols > AS_MAX_COLS || N > AS_MAX_ROWS || ne02 > 65535 || ne02 * cols * N >= (1LL << 31)) return 0;
    return (size_t)(slices * ne02 * cols * N) * sizeof(float);
}

size_t mul_mat_f16_batched_workspace_size(int64_t K, int64_t N, int64_t ne02, int64_t r2, int64_t n) {
    if (K <= 0 || N <= 0 || ne02 <= 0 || r2 <= 0 || n <= 0) return 0;
    const size_t g = gemm_plan(K, N, ne02, r2, n).bytes, sp = slice_plan_bytes(K, N, ne02, r2, n);
    return g > sp ? g : sp;
}

hipError_t launch_mul_mat_f16_batched(const void *W, size_t nb01, size_t nb02, int64_t K, int64_t N, int64_t ne02, const float *x,
                                      int64_t ldx1, int64_t ldx2, int64_t n, int64_t r2, float *y, int64_t ldy1, int64_t ldy2,
                                      void *workspace, size_t workspace_bytes, const DeviceLimits &lim, hipStream_t st, float *y2,
                                      int64_t ld2y1, int64_t ld2y2) {
    if (N <= 0 || n <= 0 || ne02 <= 0 || r2 <= 0) return hipSuccess;
    if (!mul_mat_f16_batched_supported(K) || ne02 > 65535 || r2 * n > 0x7fffffff) return hipErrorInvalidValue;
    if (y2 && !mul_mat_f16_batched_second_copy_supported(r2, n)) return hipErrorInvalidValue;
    const bool mfma_rows = tune("CHIP_ATTN_MFMA", 1) != 0;
    if (const size_t sp = slice_plan_bytes(K, N, ne02, r2, n); mfma_rows && sp > 0 && workspace && workspace_bytes >= sp &&
                                                              (((uintptr_t)workspace) & 15) == 0) {
        const BatchedArgs a{(const uint8_t *)W, nb01, nb02, K, N, x, ldx1, ldx2, n, r2, y, ldy1, ldy2, nullptr, 0, 0};
        const int64_t cols = r2 * n, slices = ceil_div(K, (int64_t)AS_SLICE);
        const dim3 grid((unsigned)slices, (unsigned)ne02), block(AS_WAVES * 64);
        float *part = (float *)workspace;
        if (cols <= 16)      hipLaunchKernelGGL(mm_f16_mfma_slice_kernel<1>, grid, block, 0, st, a, part);
        else if (cols <= 32) hipLaunchKernelGGL(mm_f16_mfma_slice_kernel<2>, grid, block, 0, st, a, part);
        else if (cols <= 64) hipLaunchKernelGGL(mm_f16_mfma_slice_kernel<4>, grid, block, 0, st, a, part);
        else                 hipLaunchKernelGGL(mm_f16_mfma_slice_kernel<8>, grid, block, 0, st, a, part);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
        hipLaunchKernelGGL(mm_f16_slice_sum_kernel, dim3((unsigned)ceil_div(ne02 * cols * N, (int64_t)AM_THREADS)), dim3(AM_THREADS), 0, st,
                           a, part, slices, ne02);
        return hipGetLastError();
    }
    const GemmPlan plan = gemm_plan(K, N, ne02, r2, n);
    // the GEMM writes row R of y at R * ldy1: the batches of y must follow each other without a gap
    if (plan.use && !y2 && workspace && workspace_bytes >= plan.bytes && ldy2 == n * ldy1 && n <= 65535 && ne02 * r2 <= 65535) {
        uint8_t *ws = (uint8_t *)workspace;
        int32_t *perm = (int32_t *)(ws + plan.off_perm), *offsets = (int32_t *)(ws + plan.off_offsets), *tiles = (int32_t *)(ws + plan.off_tiles);
        // one row tile, or two with at most 1024 columns per KV head (kqv: a head's rows): the GEMM reads the fp32 activations
        // itself and rounds them while staging (measured: 1.3 % of a 128-token step over 4096 positions; with 2048 columns and two
        // row tiles the doubled staging traffic costs more than the rounding pass, and kq, with thousands of cache positions
        // as rows, reads the activations back once per row tile): the others get an fp16 copy first
        const bool f32_direct = tune("CHIP_ATTN_F32_ROWS", 1) != 0;
        const int64_t row_tiles = ceil_div(N, (int64_t)plan.tile);
        const bool direct = f32_direct && (row_tiles == 1 || (row_tiles == 2 && r2 * n <= 1024)) && n <= 0x7fffffff &&
                            ne02 * r2 * n <= 0x7fffffff;
        if (!direct) {
            const int64_t chunks = K / 8, per = chunks >= AM_THREADS ? 1 : AM_THREADS / chunks;
            hipLaunchKernelGGL(mm_f16_round_rows_kernel, dim3((unsigned)ceil_div(n, per), (unsigned)(ne02 * r2)), dim3(AM_THREADS), 0, st, x,
                               ldx1, ldx2, n, K, ws, plan.act_stride);
        }
        hipLaunchKernelGGL(mm_f16_tile_list_kernel, dim3(64), dim3(AM_THREADS), 0, st, ne02, r2 * n, plan.tile, perm, offsets, tiles);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
        const RowGather rg{perm, offsets, tiles, 1, 1, nb02};
        const F32Rows fr{x, ldx1, ldx2, n};
        return launch_gemm_f16(W, nb01, K, N, ws, plan.act_stride, ne02 * r2 * n, y, ldy1, lim, st, &rg, plan.n_tiles, plan.tile,
                               direct ? &fr : nullptr);
    }
    const BatchedArgs a{(const uint8_t *)W, nb01, nb02, K, N, x, ldx1, ldx2, n, r2, y, ldy1, ldy2, y2, ld2y1, ld2y2};
    const int cus = lim.compute_units > 0 ? lim.compute_units : 256;
    const int64_t cols = r2 * n;
    if (mfma_rows && cols > AM_COLS && cols <= 64 && N <= 16LL * 0x7fffffff) {
        const int cg = cols <= 16 ? 1 : cols <= 32 ? 2 : 4;
        const int64_t tiles = ceil_div(N, (int64_t)16);
        if (K <= 256 && (K <= 128 || cg <= 2)) {
            int64_t gx = ceil_div(tiles, (int64_t)AM_WAVES);
            const int64_t cap = ceil_div((int64_t)cus * 4, ne02);
            if (gx > cap) gx = cap;
            const dim3 grid((unsigned)gx, (unsigned)ne02), block(AM_THREADS);
            const int ks = K <= 64 ? 2 : K <= 128 ? 4 : 8;
#define SHORT_CASE(KS, CG) hipLaunchKernelGGL((mm_f16_mfma_short_kernel<KS, CG>), grid, block, 0, st, a)
            if (ks == 2)      { if (cg == 1) SHORT_CASE(2, 1); else if (cg == 2) SHORT_CASE(2, 2); else SHORT_CASE(2, 4); }
            else if (ks == 4) { if (cg == 1) SHORT_CASE(4, 1); else if (cg == 2) SHORT_CASE(4, 2); else SHORT_CASE(4, 4); }
            else              { if (cg == 1) SHORT_CASE(8, 1); else SHORT_CASE(8, 2); }
#undef SHORT_CASE
            return hipGetLastError();
        }
        if (K > 256) {
            const dim3 grid((unsigned)tiles, (unsigned)ne02), block(AL_WAVES * 64);
            if (cg == 1)      hipLaunchKernelGGL(mm_f16_mfma_long_kernel<1>, grid, block, 0, st, a);
            else if (cg == 2) hipLaunchKernelGGL(mm_f16_mfma_long_kernel<2>, grid, block, 0, st, a);
            else              hipLaunchKernelGGL(mm_f16_mfma_long_kernel<4>, grid, block, 0, st, a);
            return hipGetLastError();
        }
    }
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
        // four rows per workgroup; two while that leaves fewer than two workgroups per CU (kqv of a decode step: 128 rows per
        // KV head - twice the workgroups re-read the activation columns from L2 and stream the cache rows with twice the waves:
        // 6.57 -> 6.01 us over a cold 8 MB cache; one row per workgroup 6.54 us)
        // (up to 8192 cached positions: with longer rows the columns' re-reads cost more than the waves gain - 16384 positions
        // 13.7 -> 14.6 us, 32768 22.8 -> 26.8 us; 1024 positions 5.14 -> 4.47 us)
        const int rows = (int)tune("CHIP_KQV_ROWS", (K <= 8192 && ceil_div(N, (int64_t)4) * ne02 < 2 * (int64_t)cus) ? 2 : 4);
        int64_t gx = ceil_div(N, (int64_t)rows);
        const int64_t cap = ceil_div((int64_t)cus * 8, ne02);
        if (gx > cap) gx = cap;
        if (rows == 2) hipLaunchKernelGGL(mm_f16_long_rows_kernel<2>, dim3((unsigned)gx, (unsigned)ne02), dim3(AM_THREADS), 0, st, a);
        else           hipLaunchKernelGGL(mm_f16_long_rows_kernel<4>, dim3((unsigned)gx, (unsigned)ne02), dim3(AM_THREADS), 0, st, a);
    }
    return hipGetLastError();
}

}  // namespace chip
