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
    unsigned short sh;      // block_q8_1.s as fp16 bits: fp16(d * sum) with the unrounded d and the sum of the int32
                            // conversion results before saturation (reference ggml-cpu/ggml-cpu-quants.c:1094)
    int sum;                // sum of the block's 32 quants (same in the 8 lanes)
};
// Eight consecutive lanes hold one 32-value block, four consecutive values each.  All 64 lanes must be active.
// fp16(a * b) with the product rounded to fp32 first, as the C source of the reference computes it; the empty asm
// keeps the compiler from folding the multiply into a single-rounding mixed-precision instruction
__device__ __forceinline__ unsigned short f2h_of_product(float a, float b) {
    float p = a * b;
    asm volatile("" : "+v"(p));
    return f2h_rne(p);
}
__device__ __forceinline__ int to_i32_x86(float r) { return (fabsf(r) < 2147483648.f) ? (int)r : INT32_MIN; }
__device__ __forceinline__ int clamp_i8(int q) { return max(-128, min(127, q)); }
__device__ __forceinline__ Q8_0Lane quantize_q8_0_lane_general(float4 v) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, dpp_get<0xB1>(amax));
    amax = fmaxf(amax, dpp_get<0x4E>(amax));
    amax = fmaxf(amax, dpp_get<0x141>(amax));
    const float d = amax / 127.f;
    const float id = (amax != 0.0f) ? 127.f / amax : 0.0f;
    const int w0 = to_i32_x86(__builtin_rintf(v.x * id)), w1 = to_i32_x86(__builtin_rintf(v.y * id));
    const int w2 = to_i32_x86(__builtin_rintf(v.z * id)), w3 = to_i32_x86(__builtin_rintf(v.w * id));
    const int q0 = clamp_i8(w0), q1 = clamp_i8(w1), q2 = clamp_i8(w2), q3 = clamp_i8(w3);
    int s = q0 + q1 + q2 + q3;
    s += __builtin_amdgcn_update_dpp(0, s, 0xB1, 0xf, 0xf, true);
    s += __builtin_amdgcn_update_dpp(0, s, 0x4E, 0xf, 0xf, true);
    s += __builtin_amdgcn_update_dpp(0, s, 0x141, 0xf, 0xf, true);
    // the unsaturated sum wraps like the 32-bit vector adds of the reference
    unsigned us = (unsigned)w0 + (unsigned)w1 + (unsigned)w2 + (unsigned)w3;
    us += (unsigned)__builtin_amdgcn_update_dpp(0, (int)us, 0xB1, 0xf, 0xf, true);
    us += (unsigned)__builtin_amdgcn_update_dpp(0, (int)us, 0x4E, 0xf, 0xf, true);
    us += (unsigned)__builtin_amdgcn_update_dpp(0, (int)us, 0x141, 0xf, 0xf, true);
    Q8_0Lane r;
    r.packed = pack_i8x4(q0, q1, q2, q3);
    r.dh = f2h_rne(d);
    r.sh = f2h_of_product(d, (float)(int)us);
    r.sum = s;
    return r;
}

struct Q8_KLane {
    uint32_t packed;        // this lane's four quants
    float d;                // super-block scale (same in all 64 lanes)
    int bsum;               // sum of the 16 quants of this lane's group of 4 lanes
};
// One wave holds one 256-value super-block, four consecutive values per lane.  All 64 lanes must be active.
__device__ __forceinline__ Q8_KLane quantize_q8_K_lane_general(float4 v) {
    // (amax, max): the first element with the largest magnitude decides, sign kept (strict > in index order)
    float cand = v.x;
    if (fabsf(v.y) > fabsf(cand)) cand = v.y;
    if (fabsf(v.z) > fabsf(cand)) cand = v.z;
    if (fabsf(v.w) > fabsf(cand)) cand = v.w;
    const float amax = wave_max_all(fabsf(cand));
    const unsigned long long holders = __ballot(fabsf(cand) == amax);
    const int first = __builtin_ctzll(holders);
    const float mx = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(cand), first));
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

// ---- fast paths -------------------------------------------------------------------------------------------
// When every input of the wave is finite and the scale cannot overflow, |x * iscale| <= 127.00002, so
//   * rounding is one add of 1.5 * 2^23 (ties to even, the same result as rint / the reference's magic add),
//   * the quant is the low byte of that sum's bit pattern, no clamp and no x86 "integer indefinite" case,
//   * |x| orders like its bit pattern, so the max reduction runs on integers (one DPP instruction per step).
// Anything else (NaN, infinity, a sum that overflows, a maximum below 1e-30) takes the general functions above;
// the choice is made per wave, so both paths see full waves.
template <int CTRL, int ROW_MASK = 0xf, bool BOUND = true>
__device__ __forceinline__ uint32_t umax_dpp(uint32_t v) {
    const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, BOUND);
    return v > o ? v : o;
}
__device__ __forceinline__ uint32_t abs_bits(float f) { return __float_as_uint(f) & 0x7fffffffu; }
__device__ __forceinline__ uint32_t umax4(float4 v) {
    const uint32_t a = abs_bits(v.x), b = abs_bits(v.y), c = abs_bits(v.z), d = abs_bits(v.w);
    const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
    return ab > cd ? ab : cd;
}
// low bytes of four magic-add sums -> one dword; the sum of the four quants
__device__ __forceinline__ uint32_t pack_low_bytes(float m0, float m1, float m2, float m3) {
    const uint32_t lo = __builtin_amdgcn_perm(__float_as_uint(m1), __float_as_uint(m0), 0x0c0c0400u);
    const uint32_t hi = __builtin_amdgcn_perm(__float_as_uint(m3), __float_as_uint(m2), 0x04000c0cu);
    return lo | hi;
}
constexpr float QUANT_MAGIC = 12582912.f;
constexpr float QUANT_MIN_AMAX = 1e-30f;

__device__ __forceinline__ Q8_0Lane quantize_q8_0_lane(float4 v) {
    const float s = (v.x + v.y) + (v.z + v.w);
    uint32_t am = umax4(v);
    am = umax_dpp<0xB1>(am);
    am = umax_dpp<0x4E>(am);
    am = umax_dpp<0x141>(am);
    const float amax = __uint_as_float(am);
    const bool odd = !(fabsf(s) < __builtin_inff()) || (am != 0u && amax < QUANT_MIN_AMAX);
    if (__ballot(odd) != 0ull) return quantize_q8_0_lane_general(v);
    const float d = amax / 127.f;
    const float id = (am != 0u) ? 127.f / amax : 0.0f;
    const float m0 = v.x * id + QUANT_MAGIC, m1 = v.y * id + QUANT_MAGIC;
    const float m2 = v.z * id + QUANT_MAGIC, m3 = v.w * id + QUANT_MAGIC;
    Q8_0Lane r;
    r.packed = pack_low_bytes(m0, m1, m2, m3);
    int sum = dot4(r.packed, 0x01010101u, 0);
    sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xf, 0xf, true);
    sum += __builtin_amdgcn_update_dpp(0, sum, 0x4E, 0xf, 0xf, true);
    sum += __builtin_amdgcn_update_dpp(0, sum, 0x141, 0xf, 0xf, true);
    r.dh = f2h_rne(d);
    r.sh = f2h_of_product(d, (float)sum);
    r.sum = sum;
    return r;
}

__device__ __forceinline__ Q8_KLane quantize_q8_K_lane(float4 v) {
    const float s = (v.x + v.y) + (v.z + v.w);
    // first element with the largest magnitude, sign kept (strict > in index order)
    float cand = v.x;
    uint32_t cb = abs_bits(v.x);
    if (abs_bits(v.y) > cb) { cand = v.y; cb = abs_bits(v.y); }
    if (abs_bits(v.z) > cb) { cand = v.z; cb = abs_bits(v.z); }
    if (abs_bits(v.w) > cb) { cand = v.w; cb = abs_bits(v.w); }
    uint32_t am = cb;
    am = umax_dpp<0xB1>(am);
    am = umax_dpp<0x4E>(am);
    am = umax_dpp<0x141>(am);
    am = umax_dpp<0x140>(am);                      // every lane of a 16-lane row holds the row maximum
    am = umax_dpp<0x142, 0xa, false>(am);          // rows 1 and 3 take in rows 0 and 2
    am = umax_dpp<0x143, 0xc, false>(am);          // lane 63 holds the wave maximum
    am = (uint32_t)__builtin_amdgcn_readlane((int)am, 63);
    const bool odd = !(fabsf(s) < __builtin_inff()) || (am != 0u && __uint_as_float(am) < QUANT_MIN_AMAX);
    if (__ballot(odd) != 0ull) return quantize_q8_K_lane_general(v);
    Q8_KLane r;
    if (am == 0u) {                                // wave-uniform
        r.packed = 0u; r.d = 0.f; r.bsum = 0;
        return r;
    }
    const unsigned long long holders = __ballot(cb == am);
    const int first = __builtin_ctzll(holders);
    const float mx = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(cand), first));
    const float iscale = -127.f / mx;
    const float m0 = iscale * v.x + QUANT_MAGIC, m1 = iscale * v.y + QUANT_MAGIC;
    const float m2 = iscale * v.z + QUANT_MAGIC, m3 = iscale * v.w + QUANT_MAGIC;
    r.packed = pack_low_bytes(m0, m1, m2, m3);
    r.d = 1.0f / iscale;
    int sum = dot4(r.packed, 0x01010101u, 0);
    sum += __builtin_amdgcn_update_dpp(0, sum, 0xB1, 0xf, 0xf, true);
    sum += __builtin_amdgcn_update_dpp(0, sum, 0x4E, 0xf, 0xf, true);
    r.bsum = sum;
    return r;
}

}  // namespace chip
