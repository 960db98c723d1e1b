// Device-side helpers shared by the gfx950 kernels: block layout constants, exact fp16 conversion,
// 4-way int8 dot, funnel shift, and a wave64 butterfly sum built from DPP moves (no LDS traffic).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace chip {

// GGUF block sizes in bytes (reference ggml-common.h:172,214,296,326,334).
constexpr int QK_SMALL = 32;     // elements per Q4_0 / Q8_0 block
constexpr int QK_K     = 256;    // elements per K-quant super-block
constexpr int BYTES_Q4_0 = 18, BYTES_Q8_0 = 34, BYTES_Q4_K = 144, BYTES_Q6_K = 210, BYTES_Q8_K = 292;
constexpr int BYTES_Q5_0 = 22, BYTES_Q5_K = 176, BYTES_IQ4_NL = 18, BYTES_Q4_1 = 20, BYTES_Q5_1 = 24, BYTES_Q8_1 = 36;
constexpr int BYTES_Q2_K = 84, BYTES_Q3_K = 110;   // reference ggml-common.h:254-266, 273-278
constexpr int BYTES_IQ4_XS = 136;                  // ggml-common.h:412-417

enum : int { T_F32 = 0, T_Q4_0 = 2, T_Q8_0 = 8, T_Q4_K = 12, T_Q6_K = 14, T_Q8_K = 15, T_Q5_0 = 6, T_Q5_K = 13, T_IQ4_NL = 20,
              T_Q4_1 = 3, T_Q5_1 = 7, T_Q8_1 = 9, T_F16 = 1, T_Q2_K = 10, T_Q3_K = 11, T_IQ4_XS = 23,
              // not a type of the reference: Q6_K rows whose four fields lie in planes (chip_repack_q6_K), read by the GEMV kernels only
              T_Q6_K_P = 114 };

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
// Same vectors with relaxed alignment: gfx950 global loads need no more than the element alignment given
// here, and GGUF blocks (18/34/210 bytes) are only 2-byte aligned inside a 16-byte aligned row.
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));
typedef u32x4 u32x4_a2 __attribute__((aligned(2)));
typedef u32x2 u32x2_a2 __attribute__((aligned(2)));
typedef u32x2 u32x2_a4 __attribute__((aligned(4)));
typedef uint32_t u32_a2 __attribute__((aligned(2)));

__device__ __forceinline__ float h2f(uint32_t h16) {
    return __half2float(__ushort_as_half((unsigned short)(h16 & 0xffffu)));     // exact
}
__device__ __forceinline__ unsigned short f2h_rne(float f) {
    return __half_as_ushort(__float2half_rn(f));                               // IEEE round-to-nearest-even
}
__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);                    // v_dot4_i32_i8, signed x signed
}
// low 32 bits of ((hi:lo) >> 16): re-slices a byte stream that starts 2 bytes into a dword
__device__ __forceinline__ uint32_t shr16(uint32_t hi, uint32_t lo) {
    return __builtin_amdgcn_alignbit(hi, lo, 16);
}

template <int CTRL, int ROW_MASK = 0xf, bool BOUND = true>
__device__ __forceinline__ float dpp_get(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xf, BOUND));
}
// Sum over the 64 lanes of a wave in a fixed butterfly order; the total ends up in lane 63.
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
    v += dpp_get<0xB1>(v);               // quad_perm [1,0,3,2]
    v += dpp_get<0x4E>(v);               // quad_perm [2,3,0,1]
    v += dpp_get<0x141>(v);              // row_half_mirror
    v += dpp_get<0x140>(v);              // row_mirror: every lane of a 16-lane row holds the row sum
    v += dpp_get<0x142, 0xa, false>(v);  // row_bcast15 into rows 1 and 3
    v += dpp_get<0x143, 0xc, false>(v);  // row_bcast31 into rows 2 and 3
    return v;
}
__device__ __forceinline__ float wave_max_all(float v) {
    v = fmaxf(v, dpp_get<0xB1>(v));
    v = fmaxf(v, dpp_get<0x4E>(v));
    v = fmaxf(v, dpp_get<0x141>(v));
    v = fmaxf(v, dpp_get<0x140>(v));
    // rows hold their own maxima; finish through the scalar unit (values are >= 0 here, so 0 is neutral)
    float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// The same butterfly for a double (two 32-bit moves per step); the total ends up in lane 63.
template <int CTRL, int ROW_MASK = 0xf, bool BOUND = true>
__device__ __forceinline__ double dpp_get_f64(double v) {
    const int lo = __builtin_amdgcn_update_dpp(0, __double2loint(v), CTRL, ROW_MASK, 0xf, BOUND);
    const int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(v), CTRL, ROW_MASK, 0xf, BOUND);
    return __hiloint2double(hi, lo);
}
__device__ __forceinline__ double wave_sum_f64_to_lane63(double v) {
    v += dpp_get_f64<0xB1>(v);
    v += dpp_get_f64<0x4E>(v);
    v += dpp_get_f64<0x141>(v);
    v += dpp_get_f64<0x140>(v);
    v += dpp_get_f64<0x142, 0xa, false>(v);
    v += dpp_get_f64<0x143, 0xc, false>(v);
    return v;
}
// The sum of squares of a row for the RMS norm (reference lm_ggml_compute_forward_rms_norm_f32, ggml-cpu/ops.cpp: sum +=
// (lm_ggml_float)(x * x), squares rounded to float, added in double), in an order fixed by where a value lies in the row, so that
// every kernel that forms it gets the same bits whatever its thread layout:
//   a float4 chunk      d = ((x0^2 + x1^2) + x2^2) + x3^2                       (norm_chunk_squares)
//   a 256-value block   B = the butterfly sum of its 64 chunks, lane = chunk % 64  (wave_sum_f64_to_lane63; absent chunks 0.0)
//   S_r = B(r) + B(r + 4) + B(r + 8) + ... for r = 0..3, and the total = ((S_0 + S_1) + S_2) + S_3.
__device__ __forceinline__ double norm_chunk_squares(const float4 v) {
    return (double)(v.x * v.x) + (double)(v.y * v.y) + (double)(v.z * v.z) + (double)(v.w * v.w);
}
constexpr int NORM_BLOCKS_MAX = 32;       // blocks of a row whose B values a kernel may keep side by side (rows up to 8192 values)
// total from the B values of a row (all threads read the same addresses)
__device__ __forceinline__ double norm_total_from_blocks(const double *B, int blocks) {
    double s[4] = {0.0, 0.0, 0.0, 0.0};
    for (int b = 0; b < blocks; b += 4) {
#pragma unroll
        for (int r = 0; r < 4; r++)
            if (b + r < blocks) s[r] += B[b + r];
    }
    double total = 0.0;
#pragma unroll
    for (int r = 0; r < 4; r++) total += s[r];
    return total;
}

// One lane of lm_ggml_v_expf in its AVX2 + FMA form (reference ggml-cpu/vec.h:615-656), operation by operation: the fused
// operations are explicit fmaf calls and the library is built with -ffp-contract=off, so nothing else is contracted.
__device__ __forceinline__ float v_expf_lane(float x) {
    const float r = 0x1.8p23f;
    const float z = __builtin_fmaf(x, 0x1.715476p+0f, r);
    const float n = z - r;
    const float b = __builtin_fmaf(-n, 0x1.7f7d1cp-20f, __builtin_fmaf(-n, 0x1.62e4p-1f, x));
    const uint32_t e = __float_as_uint(z) << 23;
    const float k = __uint_as_float(e + __float_as_uint(1.0f));
    const float u = b * b;
    const float j = __builtin_fmaf(__builtin_fmaf(__builtin_fmaf(0x1.0e4020p-7f, b, 0x1.573e2ep-5f), u,
                                                  __builtin_fmaf(0x1.555e66p-3f, b, 0x1.fffdb6p-2f)),
                                   u, 0x1.ffffecp-1f * b);
    if (!(__builtin_fabsf(n) > 126.0f)) return __builtin_fmaf(j, k, k);
    const uint32_t g = (n <= 0.0f) ? 0x82000000u : 0u;
    const float s1 = __uint_as_float(g + 0x7f000000u), s2 = __uint_as_float(e - g);
    if (__builtin_fabsf(n) > 192.0f) return s1 * s1;
    return __builtin_fmaf(s2, j, s2) * s1;
}
// lm_ggml_vec_silu_f32's lane (reference ggml-cpu/vec.cpp:164-186): x / (1 + exp(-x))
__device__ __forceinline__ float silu1(float x) { return x / (1.0f + v_expf_lane(0.0f - x)); }

__host__ __device__ constexpr int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace chip
