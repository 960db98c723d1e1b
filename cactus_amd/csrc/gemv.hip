// Decode GEMV for gfx950: y[t][r] = vec_dot(W row r, quantized activation t) for 1..8 tokens, over GGUF
// Q4_0 / Q8_0 / Q4_K / Q6_K rows kept in their on-disk block layout.  Restates the work of
// lm_ggml_vec_dot_{q4_0_q8_0,q8_0_q8_0,q4_K_q8_K,q6_K_q8_K} (reference ggml-cpu/ggml-cpu-quants.c:1906,
// 3591,6772,8520) driven by lm_ggml_compute_forward_mul_mat (ggml-cpu/ggml-cpu.c:1257-1449).
//
// Shape of the kernel (HBM-bound: every weight byte is read exactly once):
//   * a wave owns a tile of R consecutive weight rows and walks along K; lane l handles "unit" u = l + 64*it
//     of every row, a unit being the smallest piece that carries whole scales (two 32-blocks for Q4_0/Q8_0,
//     1/4 of a Q4_K or Q6_K super-block).  Consecutive lanes read consecutive bytes, so a
//     wave's loads cover one contiguous span of each row;
//   * the R rows' loads of an iteration are issued back to back before any use (about 128..144 bytes per lane
//     in flight, the depth at which a plain read kernel with the same access pattern peaks on this GPU), and
//     the first tile's loads are issued before the activation prologue so HBM latency overlaps it;
//   * quantized activations are staged once per workgroup into LDS, transposed so that lane l's 16-byte
//     chunks are adjacent to lane l+1's (conflict-free ds_read_b128), and are re-read per row tile from LDS,
//     never from global memory.  For small token counts the prologue quantizes the fp32 activations itself
//     (same device functions as the stand-alone quantize kernels), which removes a kernel launch per op;
//     workgroup 0 then also writes the quantized activations to the workspace in the split layout;
//   * integer dots use v_dot4_i32_i8; each lane keeps fp32 partial sums per (row, token) and the 64 lanes are
//     combined at the end with a fixed DPP butterfly (no LDS round trip, deterministic order).
#include "gemv_body.h"
#include <algorithm>
#include <cstdlib>

namespace chip {

// NORMED (gated pair only): the RMS norm of the input rows and the MUL with its weight in the prologue (gemv_body.h)
template <int WT, int NTOK, int R, int WGS, bool FUSEQ, int DEPTH, bool PHASED, bool GATED = false, bool NORMED = false>
__global__ __launch_bounds__(WGS) void gemv_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N,
                                                   const float *__restrict__ x, int64_t ldx,
                                                   uint8_t *__restrict__ ws, size_t ws_stride,
                                                   float *__restrict__ y, int64_t ldy, SecondMatrix sec) {
    gemv_body<WT, NTOK, R, WGS, FUSEQ, DEPTH, PHASED, GATED, false, NORMED>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, sec, whole_grid());
}

// LM_GGML_OP_MUL_MAT_ID (reference ggml-cpu/ggml-cpu.c:1460-1710): blockIdx.y is a (token, slot) pair; its expert
// ids[token][slot] picks the weight matrix W + id * nb02, its activation is row token * ne11 + slot % ne11 of x (of
// the workspace), its output row `pair` of y.  Every pair is a one-token GEMV of the kind above.  A pair whose id is
// outside [0, n_as) is skipped (the reference asserts).
struct MoeArgs {
    const int32_t *ids;
    int64_t ids_stride;      // elements between the ids of consecutive tokens
    int64_t n_used, ne11, n_as;
    size_t nb02;
    int64_t pair0;           // first pair of this launch
};
template <int WT, int R, int WGS, bool FUSEQ, int DEPTH>
__global__ __launch_bounds__(WGS) void gemv_id_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N,
                                                      const float *__restrict__ x, int64_t ldx,
                                                      uint8_t *__restrict__ ws, size_t ws_stride,
                                                      float *__restrict__ y, int64_t ldy, MoeArgs m) {
    const int64_t pair = m.pair0 + blockIdx.y;
    const int64_t t = pair / m.n_used, s = pair % m.n_used;
    const int64_t e = m.ids[t * m.ids_stride + s];
    if (e < 0 || e >= m.n_as) return;
    const int64_t xrow = t * m.ne11 + s % m.ne11;
    gemv_body<WT, 1, R, WGS, FUSEQ, DEPTH>(W + (size_t)e * m.nb02, nb01, K, N, FUSEQ ? x + xrow * ldx : x, ldx,
                                          ws + (size_t)xrow * ws_stride, ws_stride, y + pair * ldy, ldy, kNoSecond, whole_grid());
}

// ------------------------------------------------------------------------------------------------ launch
template <int WT, int NTOK, int R, int WGS, bool FUSEQ, int DEPTH>
static hipError_t launch_depth(const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, void *ws,
                               size_t ws_stride, float *y, int64_t ldy, size_t lds_bytes, int64_t max_groups, const DeviceLimits &lim,
                               hipStream_t st, const SecondMatrix &sec) {
    const int64_t tiles = ceil_div(N, R);
    int64_t groups = ceil_div(tiles, WGS / 64);
    if (groups > max_groups) groups = max_groups;
    auto launch = [&](auto kfn, LdsGrant &grant) {
        if (hipError_t e = grant_dynamic_lds(kfn, lds_bytes, lim, grant); e != hipSuccess) return e;
        hipLaunchKernelGGL(kfn, dim3((unsigned)groups), dim3(WGS), lds_bytes, st, (const uint8_t *)W, nb01, K, N, x, ldx,
                           (uint8_t *)ws, ws_stride, y, ldy, sec);
        return hipGetLastError();
    };
    // Rows of more than one step whose activations the prologue quantizes to Q8_K: the kernel that builds the image a
    // step's part at a time (gemv_body.h: PHASED)
    if constexpr (FUSEQ && Traits<WT>::ACT == T_Q8_K && WGS >= 256) {
        // (measured: 4096 x 14336 Q4_K 10.5 -> 9.5 us, 4096 x 11008 8.7 -> 8.0 us, Q6_K 4096 x 14336 15.3-16.1 -> 14.7 us;
        //  two steps - K = 8192 - run 2 % slower that way and keep the plain prologue)
        if (iters_per_row<WT>(K) > 2 && tune("CHIP_GEMV_PHASED", 1) != 0) {
            if (sec.norm_w) return hipErrorInvalidValue;                 // the phased prologue never holds the whole row
            static LdsGrant grant, grant_gated;                          // one per kernel instantiation
            if (sec.gated) return launch(gemv_kernel<WT, NTOK, R, WGS, FUSEQ, DEPTH, true, true>, grant_gated);
            return launch(gemv_kernel<WT, NTOK, R, WGS, FUSEQ, DEPTH, true>, grant);
        }
    }
    static LdsGrant grant;
    if constexpr (FUSEQ) {                                                // the gated pair exists with the quantizing prologue only
        static LdsGrant grant_gated, grant_normed;
        if (sec.gated && sec.norm_w) return launch(gemv_kernel<WT, NTOK, R, WGS, FUSEQ, DEPTH, false, true, true>, grant_normed);
        if (sec.gated) return launch(gemv_kernel<WT, NTOK, R, WGS, FUSEQ, DEPTH, false, true>, grant_gated);
    } else {
        if (sec.gated) return hipErrorInvalidValue;
    }
    if (sec.norm_w) return hipErrorInvalidValue;                         // only the gated pair's kernel is built with the norm
    return launch(gemv_kernel<WT, NTOK, R, WGS, FUSEQ, DEPTH, false>, grant);
}

template <int WT, int NTOK, int R, int WGS, bool FUSEQ>
static hipError_t launch_one(const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, void *ws,
                             size_t ws_stride, float *y, int64_t ldy, size_t lds_bytes, int64_t max_groups, const DeviceLimits &lim,
                             hipStream_t st, const SecondMatrix &sec) {
    return launch_depth<WT, NTOK, R, WGS, FUSEQ, GEMV_DEPTH>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lds_bytes, max_groups, lim, st, sec);
}

template <int WT, int NTOK, bool FUSEQ, int R = RowsPerWave<WT>::R>
static hipError_t launch_typed(const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, void *ws,
                               size_t ws_stride, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st,
                               const SecondMatrix &sec = kNoSecond) {
    size_t lds_bytes = (size_t)NTOK * lds_image_bytes<WT>(K);
    if (sec.norm_w) lds_bytes = ((lds_bytes + 7) & ~(size_t)7) + (size_t)NTOK * NORM_BLOCKS_MAX * sizeof(double);   // the norm's block sums
    if (lds_bytes > (size_t)lim.max_lds_per_block) return hipErrorInvalidValue;
    const int cus = lim.compute_units > 0 ? lim.compute_units : 256;
    if constexpr (R == 2 && NTOK == 1) {
        // Two rows per step halve the tiles: a matrix with no more rows than the device has wave slots (16 per CU) would
        // leave half of them without work, one step each for the others.  One row per step there.
        if (tune("CHIP_GEMV_R1_SMALL", 1) != 0 && N <= 16 * (int64_t)cus)
            return launch_typed<WT, NTOK, FUSEQ, 1>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
    }
    // The activation prologue (staging, or quantizing in the fused variant) is paid once per workgroup, so the
    // grid is persistent: one or two 8-wave groups per CU, each wave striding over the row tiles.  Matrices with
    // too few rows to give every CU an 8-wave group use 4-wave groups instead.
    // The one-token kernel that quantizes in its prologue runs three such groups per CU (24 waves: with one step of loads
    // in flight per wave the bytes in flight per CU grow with the waves; measured on 66 MB and 431 MB: 3 % faster than two).
    // (Q6_K rows in planes: two - the 128256 x 4096 output head 81.5 -> 77.2 us; its aligned loads saturate with 16 waves)
    const int64_t per_cu = tune("CHIP_GEMV_PER_CU", (lds_bytes <= 24 * 1024) ? ((FUSEQ && NTOK == 1 && WT != T_Q6_K_P) ? 3 : 2) : 1);
    const int64_t tiles = ceil_div(N, R);
    if constexpr (FUSEQ) {
        // When the matrix gives each of 16 waves per CU at most one tile, the prologue is a large share of the
        // kernel: one 16-wave group per CU quantizes the row once per CU instead of twice.  Measured faster for
        // every such shape except long Q8_0 rows (K > 8192), where two 8-wave groups win.
        const bool one_tile_per_wave = tiles <= 16 * (int64_t)cus && tiles > 8 * (int64_t)cus;
        const bool long_q8_0_row = Traits<WT>::ACT == T_Q8_0 && NTOK == 1 && K > 8192;
        if (one_tile_per_wave && !long_q8_0_row && tune("CHIP_GEMV_ONE_TILE_WIDE", 1) != 0)
            return launch_one<WT, NTOK, R, 1024, true>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lds_bytes, cus, lim, st, sec);
    }
    if constexpr (FUSEQ && NTOK >= 2) {
        // A narrow matrix (fewer than 8 tiles per CU) is all prologue: every workgroup quantizes NTOK rows before its
        // waves read one tile each.  16-wave groups do that with a quarter of the values per lane and keep the same
        // number of waves reading weights, on fewer CUs.  Measured on a 32-layer decode graph (wk / wv of 1024 rows,
        // K = 4096): 4 tokens 8.5 % faster for the whole step, 2 tokens 3.7 % slower - so from 8192 values up only.
        if (tune("CHIP_GEMV_NARROW_WIDE", 1) != 0 && (int64_t)NTOK * K > 8192 && ceil_div(tiles, 8) < cus)
            return launch_one<WT, NTOK, R, 1024, true>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lds_bytes, cus, lim, st, sec);
    }
    if (ceil_div(tiles, 8) >= cus)
        return launch_one<WT, NTOK, R, 512, FUSEQ>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lds_bytes, cus * per_cu, lim, st, sec);
    return launch_one<WT, NTOK, R, 256, FUSEQ>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lds_bytes, cus * per_cu, lim, st, sec);
}

template <int WT, bool FUSEQ>
static hipError_t launch_ntok(int n, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, void *ws,
                              size_t ws_stride, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st,
                              const SecondMatrix &sec = kNoSecond) {
    switch (n) {
        case 1: return launch_typed<WT, 1, FUSEQ>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case 2: return launch_typed<WT, 2, FUSEQ>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case 3: if constexpr (!FUSEQ) return launch_typed<WT, 3, false>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec); break;
        case 4: return launch_typed<WT, 4, FUSEQ>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case 5: if constexpr (!FUSEQ) return launch_typed<WT, 5, false>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec); break;
        case 6: if constexpr (!FUSEQ) return launch_typed<WT, 6, false>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec); break;
        case 7: if constexpr (!FUSEQ) return launch_typed<WT, 7, false>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec); break;
        case 8: if constexpr (!FUSEQ) return launch_typed<WT, 8, false>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec); break;
        default: break;
    }
    return hipErrorInvalidValue;
}

template <int WT> static int max_tokens_typed(int64_t K, const DeviceLimits &lim) {
    const size_t img = lds_image_bytes<WT>(K);
    const int64_t m = img ? (int64_t)(lim.max_lds_per_block / img) : 0;
    return (int)(m > 8 ? 8 : m);
}

int gemv_max_tokens(int wtype, int64_t K, const DeviceLimits &lim) {
    switch (wtype) {
        case T_Q4_0: return max_tokens_typed<T_Q4_0>(K, lim);
        case T_Q8_0: return max_tokens_typed<T_Q8_0>(K, lim);
        case T_Q4_K: return max_tokens_typed<T_Q4_K>(K, lim);
        case T_Q6_K: return max_tokens_typed<T_Q6_K>(K, lim);
        case T_Q6_K_P: return max_tokens_typed<T_Q6_K_P>(K, lim);
        case T_Q5_0: return max_tokens_typed<T_Q5_0>(K, lim);
        case T_Q5_K: return max_tokens_typed<T_Q5_K>(K, lim);
        case T_Q3_K: return max_tokens_typed<T_Q3_K>(K, lim);
        case T_Q2_K: return max_tokens_typed<T_Q2_K>(K, lim);
        case T_IQ4_XS: return max_tokens_typed<T_IQ4_XS>(K, lim);
        case T_IQ4_NL: return max_tokens_typed<T_IQ4_NL>(K, lim);
        case T_Q4_1: return max_tokens_typed<T_Q4_1>(K, lim);
        case T_Q5_1: return max_tokens_typed<T_Q5_1>(K, lim);
        case T_F16: return max_tokens_typed<T_F16>(K, lim);
        default: return 0;
    }
}

hipError_t launch_gemv(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                       int n, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st) {
    if (N <= 0 || n <= 0) return hipSuccess;
    void *w = const_cast<void *>(ws);
    switch (wtype) {
        case T_Q4_0: return launch_ntok<T_Q4_0, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st);
        case T_Q8_0: return launch_ntok<T_Q8_0, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st);
        case T_Q4_K: return launch_ntok<T_Q4_K, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st);
        case T_Q6_K: return launch_ntok<T_Q6_K, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st);
        case T_Q6_K_P: return launch_ntok<T_Q6_K_P, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st);
        case T_Q5_0: return launch_ntok<T_Q5_0, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st);
        case T_Q5_K: return launch_ntok<T_Q5_K, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st);
        case T_Q3_K: return launch_ntok<T_Q3_K, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st);
        case T_Q2_K: return launch_ntok<T_Q2_K, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st);
        case T_IQ4_XS: return launch_ntok<T_IQ4_XS, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st);
        case T_IQ4_NL: return launch_ntok<T_IQ4_NL, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st);
        case T_Q4_1: return launch_ntok<T_Q4_1, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st);
        case T_Q5_1: return launch_ntok<T_Q5_1, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st);
        case T_F16: return launch_ntok<T_F16, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st);
        default: return hipErrorInvalidValue;
    }
}

// The GEMV over prepared rows with a second matrix behind the first (sec.split rows in) or a transposed fp16 copy of the
// result (sec.t16): what launch_gemv_fused_pair / _store_t do, without the quantizer in the prologue.
hipError_t launch_gemv_sec(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n,
                           float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const SecondMatrix &sec) {
    if (N <= 0 || n <= 0) return hipSuccess;
    void *w = const_cast<void *>(ws);
    switch (wtype) {
        case T_Q4_0: return launch_ntok<T_Q4_0, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st, sec);
        case T_Q8_0: return launch_ntok<T_Q8_0, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st, sec);
        case T_Q4_K: return launch_ntok<T_Q4_K, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st, sec);
        case T_Q6_K: return launch_ntok<T_Q6_K, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st, sec);
        case T_Q6_K_P: return launch_ntok<T_Q6_K_P, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st, sec);
        case T_Q5_0: return launch_ntok<T_Q5_0, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st, sec);
        case T_Q5_K: return launch_ntok<T_Q5_K, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st, sec);
        case T_Q3_K: return launch_ntok<T_Q3_K, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st, sec);
        case T_Q2_K: return launch_ntok<T_Q2_K, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st, sec);
        case T_IQ4_XS: return launch_ntok<T_IQ4_XS, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st, sec);
        case T_IQ4_NL: return launch_ntok<T_IQ4_NL, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st, sec);
        case T_Q4_1: return launch_ntok<T_Q4_1, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st, sec);
        case T_Q5_1: return launch_ntok<T_Q5_1, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st, sec);
        case T_F16: return launch_ntok<T_F16, false>(n, W, nb01, K, N, nullptr, 0, w, ws_stride, y, ldy, lim, st, sec);
        default: return hipErrorInvalidValue;
    }
}
hipError_t launch_gemv_pair(int wtype, const void *W1, const void *W2, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                            int n, float *y1, float *y2, int64_t ldy, const DeviceLimits &lim, hipStream_t st) {
    const SecondMatrix sec{N, (int64_t)((const uint8_t *)W2 - (const uint8_t *)W1) - N * (int64_t)nb01, (int64_t)(y2 - y1) - N, nullptr, 0};
    return launch_gemv_sec(wtype, W1, nb01, K, 2 * N, ws, ws_stride, n, y1, ldy, lim, st, sec);
}
hipError_t launch_gemv_store_t(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n,
                               float *y, int64_t ldy, unsigned short *y16t, int64_t ld16, const DeviceLimits &lim, hipStream_t st) {
    const SecondMatrix sec{INT64_MAX, 0, 0, y16t, ld16};
    return launch_gemv_sec(wtype, W, nb01, K, N, ws, ws_stride, n, y, ldy, lim, st, sec);
}

// One launch for the whole op: quantize in the prologue.  Worth it while a workgroup's share of that work stays
// small: n * K <= 16384 values (64 KB of fp32 per workgroup) and n in {1, 2, 4}.
bool gemv_fused_applicable(int wtype, int64_t K, int n, const DeviceLimits &lim) {
    if (!(n == 1 || n == 2 || n == 4) || (int64_t)n * K > FUSE_MAX_VALUES) return false;
    // Every workgroup repeats the quantizer, and its dependent chains (maximum, two divisions, sums) cost a wave about
    // 0.9 us per 256 values.  With all of it in front of the first weight step, Q6_K rows of more than 8192 values ran
    // faster as a quantizer kernel (1.9 us) and a GEMV over prepared rows (4096 x 14336, one token: 1.97 + 13.0 us against
    // 15.3-16.1 us in one launch); with the image built a step's part at a time behind the previous step's arithmetic
    // (gemv_body.h: PHASED) the single launch is ahead again (14.7 us), as it is for the other types at every length
    // (4096 x 11008 Q8_0 10.7 against 12.3 us in two launches, 4096 x 14336 Q4_K 9.5 against 10.8, Q8_0 13.7 against 14.9).
    size_t img = 0;
    switch (wtype) {
        case T_Q4_0: img = lds_image_bytes<T_Q4_0>(K); break;
        case T_Q8_0: img = lds_image_bytes<T_Q8_0>(K); break;
        case T_Q4_K: img = lds_image_bytes<T_Q4_K>(K); break;
        case T_Q6_K: img = lds_image_bytes<T_Q6_K>(K); break;
        case T_Q6_K_P: img = lds_image_bytes<T_Q6_K_P>(K); break;
        case T_Q5_0: img = lds_image_bytes<T_Q5_0>(K); break;
        case T_Q5_K: img = lds_image_bytes<T_Q5_K>(K); break;
        case T_Q3_K: img = lds_image_bytes<T_Q3_K>(K); break;
        case T_Q2_K: img = lds_image_bytes<T_Q2_K>(K); break;
        case T_IQ4_XS: img = lds_image_bytes<T_IQ4_XS>(K); break;
        case T_IQ4_NL: img = lds_image_bytes<T_IQ4_NL>(K); break;
        case T_Q4_1: img = lds_image_bytes<T_Q4_1>(K); break;
        case T_Q5_1: img = lds_image_bytes<T_Q5_1>(K); break;
        case T_F16: img = lds_image_bytes<T_F16>(K); break;
        default: return false;
    }
    return (size_t)n * img <= (size_t)lim.max_lds_per_block;
}

// The RMS norm of the rows in the prologue (gemv_body.h: NORMED): the prologue that holds whole rows in registers, i.e.
// not the one that builds the image a step's part at a time, and rows of at most NORM_BLOCKS_MAX blocks of 256 values.
bool gemv_norm_prologue_applicable(int wtype, int64_t K, int n, const DeviceLimits &lim) {
    if (!gemv_fused_applicable(wtype, K, n, lim) || K > 256 * NORM_BLOCKS_MAX) return false;
    int iters = 0;
    switch (wtype) {                                                     // the types with Q8_K activations
        case T_Q4_K: iters = iters_per_row<T_Q4_K>(K); break;
        case T_Q5_K: iters = iters_per_row<T_Q5_K>(K); break;
        case T_Q3_K: iters = iters_per_row<T_Q3_K>(K); break;
        case T_Q2_K: iters = iters_per_row<T_Q2_K>(K); break;
        case T_IQ4_XS: iters = iters_per_row<T_IQ4_XS>(K); break;
        case T_Q6_K: iters = iters_per_row<T_Q6_K>(K); break;
        case T_Q6_K_P: iters = iters_per_row<T_Q6_K_P>(K); break;
        default: break;
    }
    return iters <= 2;
}

static hipError_t launch_gemv_fused_sec(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx,
                                        int n, void *ws, size_t ws_stride, float *y, int64_t ldy, const DeviceLimits &lim,
                                        hipStream_t st, const SecondMatrix &sec);
hipError_t launch_gemv_fused(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx,
                             int n, void *ws, size_t ws_stride, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st) {
    return launch_gemv_fused_sec(wtype, W, nb01, K, N, x, ldx, n, ws, ws_stride, y, ldy, lim, st, kNoSecond);
}
// W2 / y2: a second matrix of the same type, shape and row stride on the same activation; both outputs have stride ldy
hipError_t launch_gemv_fused_pair(int wtype, const void *W1, const void *W2, size_t nb01, int64_t K, int64_t N, const float *x,
                                  int64_t ldx, int n, void *ws, size_t ws_stride, float *y1, float *y2, int64_t ldy,
                                  const DeviceLimits &lim, hipStream_t st) {
    const SecondMatrix sec{N, (int64_t)((const uint8_t *)W2 - (const uint8_t *)W1) - N * (int64_t)nb01, (int64_t)(y2 - y1) - N, nullptr, 0};
    return launch_gemv_fused_sec(wtype, W1, nb01, K, 2 * N, x, ldx, n, ws, ws_stride, y1, ldy, lim, st, sec);
}
// silu(W1 x) * (W2 x) -> y, one launch (gemv_body.h: gated)
hipError_t launch_gemv_fused_pair_silu_mul(int wtype, const void *W1, const void *W2, size_t nb01, int64_t K, int64_t N, const float *x,
                                           int64_t ldx, int n, void *ws, size_t ws_stride, float *y, int64_t ldy,
                                           const DeviceLimits &lim, hipStream_t st, const float *norm_w, float norm_eps, float *norm_y,
                                           int64_t norm_ldy) {
    SecondMatrix sec = kNoSecond;
    sec.n_first = N;
    sec.w_off = (int64_t)((const uint8_t *)W2 - (const uint8_t *)W1) - N * (int64_t)nb01;
    sec.gated = 1;
    sec.norm_w = norm_w; sec.norm_eps = norm_eps; sec.norm_y = norm_y; sec.norm_ldy = norm_ldy;
    return launch_gemv_fused_sec(wtype, W1, nb01, K, 2 * N, x, ldx, n, ws, ws_stride, y, ldy, lim, st, sec);
}
// y = W x + addend in one launch (the residual ADD behind wo / ffn_down)
hipError_t launch_gemv_fused_add(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, int n, void *ws,
                                 size_t ws_stride, const float *addend, int64_t ld_add, float *y, int64_t ldy, const DeviceLimits &lim,
                                 hipStream_t st) {
    SecondMatrix sec = kNoSecond;
    sec.addend = addend; sec.ld_add = ld_add;
    return launch_gemv_fused_sec(wtype, W, nb01, K, N, x, ldx, n, ws, ws_stride, y, ldy, lim, st, sec);
}
// y16t: element (token t, row r) of the result also goes to y16t[r * ld16 + t] as fp16
hipError_t launch_gemv_fused_store_t(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, int n,
                                     void *ws, size_t ws_stride, float *y, int64_t ldy, unsigned short *y16t, int64_t ld16,
                                     const DeviceLimits &lim, hipStream_t st) {
    const SecondMatrix sec{INT64_MAX, 0, 0, y16t, ld16};
    return launch_gemv_fused_sec(wtype, W, nb01, K, N, x, ldx, n, ws, ws_stride, y, ldy, lim, st, sec);
}
static hipError_t launch_gemv_fused_sec(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx,
                                        int n, void *ws, size_t ws_stride, float *y, int64_t ldy, const DeviceLimits &lim,
                                        hipStream_t st, const SecondMatrix &sec) {
    if (N <= 0 || n <= 0) return hipSuccess;
    switch (wtype) {
        case T_Q4_0: return launch_ntok<T_Q4_0, true>(n, W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case T_Q8_0: return launch_ntok<T_Q8_0, true>(n, W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case T_Q4_K: return launch_ntok<T_Q4_K, true>(n, W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case T_Q6_K: return launch_ntok<T_Q6_K, true>(n, W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case T_Q6_K_P: return launch_ntok<T_Q6_K_P, true>(n, W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case T_Q5_0: return launch_ntok<T_Q5_0, true>(n, W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case T_Q5_K: return launch_ntok<T_Q5_K, true>(n, W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case T_Q3_K: return launch_ntok<T_Q3_K, true>(n, W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case T_Q2_K: return launch_ntok<T_Q2_K, true>(n, W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case T_IQ4_XS: return launch_ntok<T_IQ4_XS, true>(n, W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case T_IQ4_NL: return launch_ntok<T_IQ4_NL, true>(n, W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case T_Q4_1: return launch_ntok<T_Q4_1, true>(n, W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case T_Q5_1: return launch_ntok<T_Q5_1, true>(n, W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        case T_F16: return launch_ntok<T_F16, true>(n, W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, lim, st, sec);
        default: return hipErrorInvalidValue;
    }
}

// MUL_MAT_ID: one launch of (groups, pairs) workgroups, each pair a one-token GEMV on its expert's rows.  `fused`
// quantizes the pair's activation row in the prologue (x is fp32); otherwise ws holds the quantized rows already.
template <int WT, bool FUSEQ>
static hipError_t launch_id_typed(const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, void *ws,
                                  size_t ws_stride, float *y, int64_t ldy, MoeArgs m, int64_t pairs, const DeviceLimits &lim,
                                  hipStream_t st) {
    const size_t lds_bytes = lds_image_bytes<WT>(K);
    if (lds_bytes > (size_t)lim.max_lds_per_block) return hipErrorInvalidValue;
    const int cus = lim.compute_units > 0 ? lim.compute_units : 256;
    constexpr int R = RowsPerWave<WT>::R, WGS = 256;
    const int64_t tiles = ceil_div(N, R);
    auto kfn = gemv_id_kernel<WT, R, WGS, FUSEQ, GEMV_DEPTH>;
    static LdsGrant grant;
    if (hipError_t e = grant_dynamic_lds(kfn, lds_bytes, lim, grant); e != hipSuccess) return e;
    for (int64_t p0 = 0; p0 < pairs; p0 += 32768) {
        const int64_t np = pairs - p0 < 32768 ? pairs - p0 : 32768;
        // about two 4-wave groups per CU over all pairs of the launch, at least one group per pair
        int64_t groups = ceil_div(tiles, WGS / 64);
        const int64_t cap = ceil_div((int64_t)cus * 4, np);
        if (groups > cap) groups = cap;
        m.pair0 = p0;
        hipLaunchKernelGGL(kfn, dim3((unsigned)groups, (unsigned)np), dim3(WGS), lds_bytes, st, (const uint8_t *)W, nb01, K, N,
                           x, ldx, (uint8_t *)ws, ws_stride, y, ldy, m);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t launch_gemv_id(int wtype, bool fused, const void *W, size_t nb01, size_t nb02, int64_t n_as, int64_t K, int64_t N,
                          const float *x, int64_t ldx, int64_t ne11, const int32_t *ids, int64_t ids_stride, int64_t n_used,
                          int64_t n_tokens, void *ws, size_t ws_stride, float *y, int64_t ldy, const DeviceLimits &lim,
                          hipStream_t st) {
    const int64_t pairs = n_tokens * n_used;
    if (N <= 0 || pairs <= 0) return hipSuccess;
    const MoeArgs m{ids, ids_stride, n_used, ne11, n_as, nb02, 0};
#define ID_CASE(TT) case TT: return fused ? launch_id_typed<TT, true>(W, nb01, K, N, x, ldx, ws, ws_stride, y, ldy, m, pairs, lim, st) \
                                          : launch_id_typed<TT, false>(W, nb01, K, N, nullptr, 0, ws, ws_stride, y, ldy, m, pairs, lim, st);
    switch (wtype) {
        ID_CASE(T_Q4_0) ID_CASE(T_Q8_0) ID_CASE(T_Q4_K) ID_CASE(T_Q6_K) ID_CASE(T_Q5_0) ID_CASE(T_Q5_K) ID_CASE(T_IQ4_NL)
        ID_CASE(T_Q4_1) ID_CASE(T_Q5_1) ID_CASE(T_F16) ID_CASE(T_Q3_K) ID_CASE(T_Q2_K) ID_CASE(T_IQ4_XS)
        default: return hipErrorInvalidValue;
    }
#undef ID_CASE
}

// ------------------------------------------------------------------------------------------------ isum hook
// Reference activation record of a 32-element type: block_q8_0 (34 bytes, quants at +2) unless the traits say
// block_q8_1 (36 bytes, quants at +4).
template <typename T, typename = void> struct ActBlock { static constexpr int BYTES = BYTES_Q8_0, QOFF = 2; };
template <typename T> struct ActBlock<T, decltype((void)T::ABLK_BYTES)> { static constexpr int BYTES = T::ABLK_BYTES, QOFF = T::ABLK_QOFF; };
template <typename T> __host__ __device__ constexpr int act_block_bytes() { return ActBlock<T>::BYTES; }
template <typename T> __host__ __device__ constexpr int act_block_qoff() { return ActBlock<T>::QOFF; }

// Per-block integer sums through the same load_w / isums device code.  One wave per (token, row); activations
// come from reference-layout blocks and are converted to the unit form on the fly (slow path, tests only).
template <int WT>
__global__ __launch_bounds__(64) void block_isums_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N,
                                                        const uint8_t *__restrict__ aq, int32_t *__restrict__ isum,
                                                        int32_t *__restrict__ imin) {
    using T = Traits<WT>;
    const int64_t row = blockIdx.x, t = blockIdx.y;
    const int lane = threadIdx.x;
    const int units = units_per_row<WT>(K);
    const int64_t nblk = K / (T::ACT == T_Q8_0 ? 32 : 256);
    const size_t a_row = (size_t)(T::ACT == T_Q8_0 ? (K / 32) * act_block_bytes<T>() : (K / 256) * BYTES_Q8_K);
    const uint8_t *arow = aq + t * a_row;
    int32_t *out = isum + ((size_t)t * N + row) * nblk;
    int32_t *outm = imin ? imin + ((size_t)t * N + row) * nblk : nullptr;
    for (int u0 = 0; u0 < units; u0 += 64) {
        const int u = u0 + lane;
        int v0 = 0, v1 = 0;
        if (u < units) {
            typename T::Raw raw;
            T::load_raw(raw, W + (size_t)row * nb01, u);
            typename T::W w;
            T::decode(w, raw, u);
            typename T::A a;
            // gather this unit's activation bytes from reference blocks
            if constexpr (T::ACT == T_Q8_0) {
                for (int b = 0; b < 2; b++) {
                    const uint8_t *blk = arow + (size_t)(2 * u + b) * act_block_bytes<T>() + (act_block_qoff<T>() - 2);
                    int s = 0;
                    for (int i = 0; i < 8; i++) {
                        uint32_t d = blk[2 + 4 * i] | (blk[3 + 4 * i] << 8) | (blk[4 + 4 * i] << 16) | ((uint32_t)blk[5 + 4 * i] << 24);
                        a.q[8 * b + i] = d;
                        s = dot4(d, 0x01010101u, s);
                    }
                    if constexpr (T::A_HAS_SUMS) { if (b == 0) a.s0 = s; else a.s1 = s; }
                }
                a.d0 = a.d1 = 1.f;
            } else {
                const int sb = u >> 2;
                const uint8_t *blk = arow + (size_t)sb * BYTES_Q8_K;
                const int16_t *bs = reinterpret_cast<const int16_t *>(blk + 260);
                for (int j = 0; j < T::QCH; j++) {
                    const size_t off = T::src_chunk(K, u, j) - (size_t)sb * 256;
                    for (int i = 0; i < 4; i++) {
                        const uint8_t *p = blk + 4 + off + 4 * i;
                        a.q[4 * j + i] = p[0] | (p[1] << 8) | (p[2] << 16) | ((uint32_t)p[3] << 24);
                    }
                }
                a.d = 1.f;
                if constexpr (T::KQ_STYLE == 0) {
                    const int jp = u & 3;
                    a.s0 = bs[4 * jp] + bs[4 * jp + 1]; a.s1 = bs[4 * jp + 2] + bs[4 * jp + 3];
                } else {
                    const int h = (u >> 1) & 1, ip = u & 1;
                    for (int v = 0; v < 4; v++) a.bs[v] = bs[8 * h + 2 * v + ip];
                }
            }
            T::isums(w, a, v0, v1);
        }
        if constexpr (T::ACT == T_Q8_0) {
            if (u < units) { out[2 * u] = v0; out[2 * u + 1] = v1; }
        } else {
            // sum the four units of each super-block in integer arithmetic
            constexpr int G = 4;
            for (int m = 1; m < G; m <<= 1) { v0 += __shfl_xor(v0, m); v1 += __shfl_xor(v1, m); }
            if (u < units && (lane % G) == 0) {
                out[u / G] = v0;
                if (outm) outm[u / G] = v1;
            }
        }
    }
}

hipError_t launch_block_isums(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *aq, int64_t n,
                              int32_t *isum, int32_t *imin, hipStream_t st) {
    if (N <= 0 || n <= 0) return hipSuccess;
    dim3 grid((unsigned)N, (unsigned)n);
    switch (wtype) {
        case T_Q4_0: hipLaunchKernelGGL(block_isums_kernel<T_Q4_0>, grid, dim3(64), 0, st, (const uint8_t *)W, nb01, K, N, (const uint8_t *)aq, isum, imin); break;
        case T_Q8_0: hipLaunchKernelGGL(block_isums_kernel<T_Q8_0>, grid, dim3(64), 0, st, (const uint8_t *)W, nb01, K, N, (const uint8_t *)aq, isum, imin); break;
        case T_Q4_K: hipLaunchKernelGGL(block_isums_kernel<T_Q4_K>, grid, dim3(64), 0, st, (const uint8_t *)W, nb01, K, N, (const uint8_t *)aq, isum, imin); break;
        case T_Q6_K: hipLaunchKernelGGL(block_isums_kernel<T_Q6_K>, grid, dim3(64), 0, st, (const uint8_t *)W, nb01, K, N, (const uint8_t *)aq, isum, imin); break;
        case T_Q5_0: hipLaunchKernelGGL(block_isums_kernel<T_Q5_0>, grid, dim3(64), 0, st, (const uint8_t *)W, nb01, K, N, (const uint8_t *)aq, isum, imin); break;
        case T_Q5_K: hipLaunchKernelGGL(block_isums_kernel<T_Q5_K>, grid, dim3(64), 0, st, (const uint8_t *)W, nb01, K, N, (const uint8_t *)aq, isum, imin); break;
        case T_Q3_K: hipLaunchKernelGGL(block_isums_kernel<T_Q3_K>, grid, dim3(64), 0, st, (const uint8_t *)W, nb01, K, N, (const uint8_t *)aq, isum, imin); break;
        case T_Q2_K: hipLaunchKernelGGL(block_isums_kernel<T_Q2_K>, grid, dim3(64), 0, st, (const uint8_t *)W, nb01, K, N, (const uint8_t *)aq, isum, imin); break;
        case T_IQ4_XS: hipLaunchKernelGGL(block_isums_kernel<T_IQ4_XS>, grid, dim3(64), 0, st, (const uint8_t *)W, nb01, K, N, (const uint8_t *)aq, isum, imin); break;
        case T_IQ4_NL: hipLaunchKernelGGL(block_isums_kernel<T_IQ4_NL>, grid, dim3(64), 0, st, (const uint8_t *)W, nb01, K, N, (const uint8_t *)aq, isum, imin); break;
        case T_Q4_1: hipLaunchKernelGGL(block_isums_kernel<T_Q4_1>, grid, dim3(64), 0, st, (const uint8_t *)W, nb01, K, N, (const uint8_t *)aq, isum, imin); break;
        case T_Q5_1: hipLaunchKernelGGL(block_isums_kernel<T_Q5_1>, grid, dim3(64), 0, st, (const uint8_t *)W, nb01, K, N, (const uint8_t *)aq, isum, imin); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace chip
