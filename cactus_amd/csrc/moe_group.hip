// Grouping of the (token, slot) pairs of LM_GGML_OP_MUL_MAT_ID by expert, on the device: what the reference builds
// in matrix_row_counts / matrix_rows (ggml-cpu/ggml-cpu.c:1625-1640) as a counting sort, so that each expert's pairs
// can run through a GEMM over that expert's matrix.  The order of the pairs inside an expert's list is not fixed
// (atomic cursors); no output depends on it, since every output row is computed on its own.
#include "dev_common.h"
#include "kernels.h"

namespace chip {

constexpr int MOE_GROUP_THREADS = 1024;
constexpr int MOE_MAX_EXPERTS = 1 << MOE_EXPERT_BITS;   // LDS: three int32 per expert; tile entries keep 12 bits for it

// offsets[e] .. offsets[e+1]: expert e's stretch of perm; perm holds pair numbers token * n_used + slot.  Pairs whose
// id lies outside [0, n_as) are left out (the reference asserts on them).  tiles: the list of (expert, token tile)
// work items for tiles of tile_tokens pairs, its length in front.
__global__ __launch_bounds__(MOE_GROUP_THREADS) void moe_group_kernel(const int32_t *__restrict__ ids, int64_t ids_stride,
                                                                       int n_used, int64_t pairs, int n_as, int tile_tokens,
                                                                       int32_t *__restrict__ offsets, int32_t *__restrict__ perm,
                                                                       int32_t *__restrict__ tiles) {
    __shared__ int32_t count[MOE_MAX_EXPERTS], start[MOE_MAX_EXPERTS + 1], tstart[MOE_MAX_EXPERTS + 1];
    const int tid = threadIdx.x;
    for (int e = tid; e < n_as; e += MOE_GROUP_THREADS) count[e] = 0;
    __syncthreads();
    for (int64_t p = tid; p < pairs; p += MOE_GROUP_THREADS) {
        const int32_t e = ids[(p / n_used) * ids_stride + p % n_used];
        if (e >= 0 && e < n_as) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int32_t run = 0, trun = 0;
        for (int e = 0; e < n_as; e++) {
            start[e] = run;
            tstart[e] = trun;
            run += count[e];
            trun += (count[e] + tile_tokens - 1) / tile_tokens;
        }
        start[n_as] = run;
        tstart[n_as] = trun;
        tiles[0] = trun;
    }
    __syncthreads();
    for (int e = tid; e <= n_as; e += MOE_GROUP_THREADS) {
        offsets[e] = start[e];
        if (e < n_as) {
            for (int t = tstart[e]; t < tstart[e + 1]; t++) tiles[1 + t] = e | ((t - tstart[e]) << MOE_EXPERT_BITS);
            count[e] = 0;                                            // reused as the write cursor
        }
    }
    __syncthreads();
    for (int64_t p = tid; p < pairs; p += MOE_GROUP_THREADS) {
        const int32_t e = ids[(p / n_used) * ids_stride + p % n_used];
        if (e >= 0 && e < n_as) perm[start[e] + atomicAdd(&count[e], 1)] = (int32_t)p;
    }
}

bool moe_group_supported(int64_t n_as, int64_t pairs) {
    return n_as >= 1 && n_as <= MOE_MAX_EXPERTS && pairs / 64 + n_as < ((int64_t)1 << (31 - MOE_EXPERT_BITS)) && pairs / 64 + n_as <= 65535;
}

hipError_t launch_moe_group(const int32_t *ids, int64_t ids_stride, int64_t n_used, int64_t pairs, int64_t n_as,
                            int tile_tokens, int32_t *offsets, int32_t *perm, int32_t *tiles, hipStream_t st) {
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(MOE_GROUP_THREADS), 0, st, ids, ids_stride, (int)n_used, pairs, (int)n_as,
                       tile_tokens, offsets, perm, tiles);
    return hipGetLastError();
}

}  // namespace chip
