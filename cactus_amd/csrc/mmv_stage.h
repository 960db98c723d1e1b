// Prologue of the matrix-core GEMVs over Q8_0 rows (gemv_mfma.hip, gemv_mfma_q4_0.hip): the n quantized activation rows go
// from the workspace planes into the workgroup's LDS image, token-major quants [NT][q_stride] and scales [K / 32][16].
#pragma once
#include "dev_common.h"
#include "act_layout.h"
#include <type_traits>

namespace chip {

// item -> (row, piece): idx / den through the reciprocal, corrected by one (idx < 2^20)
__device__ __forceinline__ void mmv_divmod(int idx, int den, float rcp, int &q, int &r) {
    q = (int)((float)idx * rcp);
    r = idx - q * den;
    if (r < 0) { q--; r += den; } else if (r >= den) { q++; r -= den; }
}

// Every load instruction of the prologue costs the same whether one lane or all of them use its result, so the n rows are
// spread over the threads as flat lists of (token, piece) items - n * K / 16 chunks of quants, n * K / 32 scales - with as
// many register slots as the workgroup needs for them; a thread past the end of a list loads the last item again and dumps
// it at `dump` (LDS that is idle during the prologue: 16-byte aligned, 20 bytes used per thread).  All loads are unconditional: a load inside a
// branch makes the compiler wait for everything in flight.  issue_weights() is called after the activation loads and
// before anything waits for them (loads return in issue order).  Rows n .. NT-1 of the images are zeros.
template <int NT, int WGS, class IssueWeights>
__device__ __forceinline__ void mmv_stage_q8_0_rows(uint8_t *lds, const uint8_t *__restrict__ ws, size_t ws_stride, int n, int64_t K,
                                                    uint32_t q_stride, uint32_t d_base, uint32_t dump, IssueWeights &&issue_weights) {
    const int nchunk = (int)(K / 16), nblk = (int)(K / 32);
    const int q_items = n * nchunk, d_items = n * nblk;
    const float rc_chunk = 1.0f / (float)nchunk, rc_blk = 1.0f / (float)nblk;
    // (token, piece) of item idx, the last item's past the end of the list
    auto q_place = [&](int idx, int t, int c, const u32x4 *&src, uint32_t &dst) {
        const bool in = idx < q_items;
        t = in ? t : n - 1;
        c = in ? c : nchunk - 1;
        src = reinterpret_cast<const u32x4 *>(ws + (size_t)t * ws_stride + 16 * (size_t)c);
        dst = in ? (uint32_t)t * q_stride + 16u * (uint32_t)c : dump;
    };
    auto d_place = [&](int idx, int t, int b, const float *&src, uint32_t &dst) {
        const bool in = idx < d_items;
        t = in ? t : n - 1;
        b = in ? b : nblk - 1;
        src = reinterpret_cast<const float *>(ws + (size_t)t * ws_stride + q8_0_off_d(K)) + b;
        dst = in ? d_base + 4u * (uint32_t)(b * 16 + t) : dump + 16u;
    };
    auto q_item = [&](int idx, const u32x4 *&src, uint32_t &dst) {
        int t, c;
        mmv_divmod(idx, nchunk, rc_chunk, t, c);
        q_place(idx, t, c, src, dst);
    };
    auto d_item = [&](int idx, const float *&src, uint32_t &dst) {
        int t, b;
        mmv_divmod(idx, nblk, rc_blk, t, b);
        d_place(idx, t, b, src, dst);
    };
    // a thread's items are WGS apart: one division each for the first, then steps of (WGS / den, WGS % den) with a carry
    const int q_dt = WGS / nchunk, q_dc = WGS % nchunk, d_dt = WGS / nblk, d_db = WGS % nblk;
    auto stage = [&](auto slots) {
        constexpr int QL = decltype(slots)::value, DL = QL / 2;
        u32x4 qv[QL];
        float dv[DL];
        uint32_t qdst[QL], ddst[DL];
        int t, c;
        mmv_divmod((int)threadIdx.x, nchunk, rc_chunk, t, c);
#pragma unroll
        for (int j = 0; j < QL; j++) {
            const u32x4 *src;
            q_place(j * WGS + (int)threadIdx.x, t, c, src, qdst[j]);
            qv[j] = *src;
            t += q_dt; c += q_dc;
            if (c >= nchunk) { c -= nchunk; t++; }
        }
        mmv_divmod((int)threadIdx.x, nblk, rc_blk, t, c);
#pragma unroll
        for (int j = 0; j < DL; j++) {
            const float *src;
            d_place(j * WGS + (int)threadIdx.x, t, c, src, ddst[j]);
            dv[j] = *src;
            t += d_dt; c += d_db;
            if (c >= nblk) { c -= nblk; t++; }
        }
        __builtin_amdgcn_sched_barrier(0);                               // activations are requested before weights
        issue_weights();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < QL; j++) *reinterpret_cast<u32x4 *>(lds + qdst[j]) = qv[j];
#pragma unroll
        for (int j = 0; j < DL; j++) *reinterpret_cast<float *>(lds + ddst[j]) = dv[j];
        // lists longer than the slots: the rest in plain loops
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
    };
    const int need = (q_items + WGS - 1) / WGS;
    if (need <= 4) stage(std::integral_constant<int, 4>{});
    else if (need <= 8) stage(std::integral_constant<int, 8>{});
    else if (need <= 12) stage(std::integral_constant<int, 12>{});
    else stage(std::integral_constant<int, 16>{});
    for (int i = (int)threadIdx.x; i < (NT - n) * nchunk; i += WGS) {
        int t, c;
        mmv_divmod(i, nchunk, rc_chunk, t, c);
        *reinterpret_cast<u32x4 *>(lds + (uint32_t)(n + t) * q_stride + 16u * (uint32_t)c) = u32x4{0u, 0u, 0u, 0u};
    }
    for (int i = (int)threadIdx.x; i < nblk * NT; i += WGS)
        if ((i & (NT - 1)) >= n) reinterpret_cast<float *>(lds + d_base)[(i / NT) * 16 + (i & (NT - 1))] = 0.f;
}

}  // namespace chip
