// Device functions of the on-the-fly activation quantizers, shared by the stand-alone quantize kernels and by
// the GEMV kernels that quantize in their prologue, so both produce identical bits.
//
// Q8_0: AVX2 branch of quantize_row_q8_0 (reference ggml-cpu/ggml-cpu-quants.c:802-885).
// Q8_K: quantize_row_q8_K_ref (reference ggml-quants.c:2473-2510).
// Compile with -ffp-contract=off: `iscale*x + 12582912.f` must round twice, as the C source says.
#pragma once
#include "dev_common.h"

namespace chip {

// x86 cvtps2dq followed by two saturating packs: NaN or |r| >= 2^31 becomes INT_MIN -> -128.
__device__ __forceinline__ int to_i8_x86(float r) {
    int q = (fabsf(r) < 2147483648.f) ? (int)r : INT32_MIN;
    return max(-128, min(127, q));
}
__device__ __forceinline__ uint32_t pack_i8x4(int q0, int q1, int q2, int q3) {
    return (uint32_t)(q0 & 0xff) | ((uint32_t)(q1 & 0xff) << 8) | ((uint32_t)(q2 & 0xff) << 16) | ((uint32_t)(q3 & 0xff) << 24);
}

struct Q8_0Lane {
    uint32_t packed;        // this lane's four quants
    unsigned short dh;      // block scale as fp16 bits (same in the 8 lanes of the block)
    int sum;                // sum of the block's 32 quants (same in the 8 lanes)
};
// Eight consecutive lanes hold one 32-value block, four consecutive values each.  All 64 lanes must be active.
__device__ __forceinline__ Q8_0Lane quantize_q8_0_lane(float4 v) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, dpp_get<0xB1>(amax));
    amax = fmaxf(amax, dpp_get<0x4E>(amax));
    amax = fmaxf(amax, dpp_get<0x141>(amax));
    const float d = amax / 127.f;
    const float id = (amax != 0.0f) ? 127.f / amax : 0.0f;
    const int q0 = to_i8_x86(__builtin_rintf(v.x * id));
    const int q1 = to_i8_x86(__builtin_rintf(v.y * id));
    const int q2 = to_i8_x86(__builtin_rintf(v.z * id));
    const int q3 = to_i8_x86(__builtin_rintf(v.w * id));
    int s = q0 + q1 + q2 + q3;
    s += __builtin_amdgcn_update_dpp(0, s, 0xB1, 0xf, 0xf, true);
    s += __builtin_amdgcn_update_dpp(0, s, 0x4E, 0xf, 0xf, true);
    s += __builtin_amdgcn_update_dpp(0, s, 0x141, 0xf, 0xf, true);
    Q8_0Lane r;
    r.packed = pack_i8x4(q0, q1, q2, q3);
    r.dh = f2h_rne(d);
    r.sum = s;
    return r;
}

struct Q8_KLane {
    uint32_t packed;        // this lane's four quants
    float d;                // super-block scale (same in all 64 lanes)
    int bsum;               // sum of the 16 quants of this lane's group of 4 lanes
};
// One wave holds one 256-value super-block, four consecutive values per lane.  All 64 lanes must be active.
__device__ __forceinline__ Q8_KLane quantize_q8_K_lane(float4 v) {
    // (amax, max): the first element with the largest magnitude decides, sign kept (strict > in index order)
    float cand = v.x;
    if (fabsf(v.y) > fabsf(cand)) cand = v.y;
    if (fabsf(v.z) > fabsf(cand)) cand = v.z;
    if (fabsf(v.w) > fabsf(cand)) cand = v.w;
    const float amax = wave_max_all(fabsf(cand));
    const unsigned long long holders = __ballot(fabsf(cand) == amax);
    const int first = __builtin_ctzll(holders);
    const float mx = __shfl(cand, first);
    int q0 = 0, q1 = 0, q2 = 0, q3 = 0;
    Q8_KLane r;
    r.d = 0.f;
    if (amax != 0.0f) {
        const float iscale = -127.f / mx;
        auto nearest = [](float f) {
            const float m = f + 12582912.f;
            return (int)(__float_as_uint(m) & 0x007fffffu) - 0x00400000;
        };
        q0 = min(127, nearest(iscale * v.x));
        q1 = min(127, nearest(iscale * v.y));
        q2 = min(127, nearest(iscale * v.z));
        q3 = min(127, nearest(iscale * v.w));
        r.d = 1.0f / iscale;
    }
    r.packed = pack_i8x4(q0, q1, q2, q3);
    int s = q0 + q1 + q2 + q3;
    s += __builtin_amdgcn_update_dpp(0, s, 0xB1, 0xf, 0xf, true);
    s += __builtin_amdgcn_update_dpp(0, s, 0x4E, 0xf, 0xf, true);
    r.bsum = s;
    return r;
}

}  // namespace chip
