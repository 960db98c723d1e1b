// Kernel-private layout of quantized activations in the MUL_MAT workspace ("split" layout).
//
// The reference keeps quantized activations as arrays of block_q8_0 / block_q8_K (34 / 292-byte records that
// interleave scale and quants).  On the GPU the same numbers are kept per token as three aligned planes so
// that every consumer reads 16-byte aligned vectors:
//
//   Q8_0 activations (for Q4_0 and Q8_0 weights), token stride = q8_0_stride(K):
//       qs  int8  [K]        at +0                 quants, block b at 32*b
//       d   float [K/32]     at +K                 the block scale after rounding to fp16 (exactly as stored
//                                                  in block_q8_0.d), widened back to fp32
//       sum int32 [K/32]     at +K + 4*(K/32)      sum of the 32 quants of the block (Q4_0's -8 offset)
//       s   float [K/32]     at +K + 8*(K/32)      block_q8_1.s (fp16(d * sum), widened): the min term of Q4_1 / Q5_1,
//                                                  whose activation format Q8_1 is Q8_0 plus this number
//
//   Q8_K activations (for Q4_K and Q6_K weights), token stride = q8_K_stride(K):
//       qs    int8  [K]      at +0
//       d     float [K/256]  at +K
//       bsums int16 [K/16]   at +K + 4*(K/256)     block_q8_K.bsums
//
//   F16 activations (for F16 weights), token stride = f16_stride(K): K halves, nothing else.
//
// K is a multiple of 256, so every plane starts 16-byte aligned.  Token strides are multiples of 128 bytes: a token's
// 128-byte stretches of quants then coincide with cache lines, which halves the lines the GEMM kernels touch.
#pragma once
#include <stdint.h>
#include <stddef.h>

namespace chip {

__host__ __device__ constexpr size_t align16(size_t v) { return (v + 15) & ~(size_t)15; }
__host__ __device__ constexpr size_t align128(size_t v) { return (v + 127) & ~(size_t)127; }

__host__ __device__ constexpr size_t q8_0_off_d(int64_t K)   { return (size_t)K; }
__host__ __device__ constexpr size_t q8_0_off_sum(int64_t K) { return (size_t)K + 4 * (size_t)(K / 32); }
__host__ __device__ constexpr size_t q8_0_off_s(int64_t K)   { return (size_t)K + 8 * (size_t)(K / 32); }
__host__ __device__ constexpr size_t q8_0_stride(int64_t K)  { return align128((size_t)K + 12 * (size_t)(K / 32)); }

__host__ __device__ constexpr size_t f16_stride(int64_t K)   { return align128(2 * (size_t)K); }

__host__ __device__ constexpr size_t q8_K_off_d(int64_t K)     { return (size_t)K; }
__host__ __device__ constexpr size_t q8_K_off_bsums(int64_t K) { return (size_t)K + 4 * (size_t)(K / 256); }
__host__ __device__ constexpr size_t q8_K_stride(int64_t K)    { return align128((size_t)K + 4 * (size_t)(K / 256) + 2 * (size_t)(K / 16)); }

}  // namespace chip
