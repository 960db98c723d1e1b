// The element-wise ops that sit between the matmuls of an FFN block, so that a norm -> up/gate -> activation -> down ->
// residual chain can stay on the device: RMS_NORM, ADD, MUL and SILU over F32 rows.  All are HBM-bound streams.
//
//   RMS_NORM  lm_ggml_compute_forward_rms_norm_f32 (reference ggml-cpu/ops.cpp:3270-3316): sum of the float squares in
//             double, mean and scale in float, one float multiply per element.  The reference adds in element order;
//             here the double sum is a tree, which changes the double result in its last bits at most and the float
//             mean only when it falls within ~1e-16 of a rounding boundary.
//   ADD, MUL  binary-ops.cpp: one IEEE operation per element; src1 has the shape of src0 or is one row broadcast over
//             all rows (norm weights, biases).  Bit-exact.
//   SILU      lm_ggml_vec_silu_f32 (ggml-cpu/vec.cpp:164-186) = x / (1 + lm_ggml_v_expf(-x)) with the AVX2 + FMA form of
//             lm_ggml_v_expf (ggml-cpu/vec.h:615-656) restated operation by operation, so that the result is bit-exact
//             for rows whose length is a multiple of 8 (the reference finishes other rows with the C library's expf:
//             those rows are declined).
#include "dev_common.h"
#include "kernels.h"

namespace chip {

constexpr int EW_THREADS = 256;

// one lane of lm_ggml_v_expf (AVX2 + FMA)
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
__device__ __forceinline__ float silu1(float x) { return x / (1.0f + v_expf_lane(0.0f - x)); }

// ---- RMS_NORM: one workgroup per row ----
__global__ __launch_bounds__(EW_THREADS) void rms_norm_kernel(const float *__restrict__ x, int64_t ldx, int64_t ne0, float eps,
                                                              float *__restrict__ y, int64_t ldy) {
    __shared__ double part[EW_THREADS / 64];
    const float *xr = x + (size_t)blockIdx.x * ldx;
    float *yr = y + (size_t)blockIdx.x * ldy;
    const int tid = threadIdx.x;
    const bool vec = ((ne0 | ldx | ldy) & 3) == 0 && ((((uintptr_t)x) | ((uintptr_t)y)) & 15) == 0;
    double sum = 0.0;
    if (vec) {
        for (int64_t i = 4 * tid; i < ne0; i += 4 * EW_THREADS) {
            const float4 v = *reinterpret_cast<const float4 *>(xr + i);
            sum += (double)(v.x * v.x) + (double)(v.y * v.y) + (double)(v.z * v.z) + (double)(v.w * v.w);
        }
    } else {
        for (int64_t i = tid; i < ne0; i += EW_THREADS) sum += (double)(xr[i] * xr[i]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
    if ((tid & 63) == 0) part[tid >> 6] = sum;
    __syncthreads();
    double total = 0.0;
#pragma unroll
    for (int w = 0; w < EW_THREADS / 64; w++) total += part[w];
    const float mean = (float)(total / (double)ne0);
    const float scale = 1.0f / sqrtf(mean + eps);
    if (vec) {
        for (int64_t i = 4 * tid; i < ne0; i += 4 * EW_THREADS) {
            float4 v = *reinterpret_cast<const float4 *>(xr + i);
            v.x *= scale; v.y *= scale; v.z *= scale; v.w *= scale;
            *reinterpret_cast<float4 *>(yr + i) = v;
        }
    } else {
        for (int64_t i = tid; i < ne0; i += EW_THREADS) yr[i] = xr[i] * scale;
    }
}

// ---- element-wise: grid.y walks the rows, grid.x the row in chunks of 4 * EW_THREADS values ----
enum { EW_ADD = 0, EW_MUL = 1, EW_SILU = 2 };
template <int OP> __device__ __forceinline__ float ew_apply(float a, float b) {
    if constexpr (OP == EW_ADD) return a + b;
    else if constexpr (OP == EW_MUL) return a * b;
    else return silu1(a);
}
template <int OP, bool VEC>
__global__ __launch_bounds__(EW_THREADS) void elementwise_kernel(const float *__restrict__ a, int64_t lda,
                                                                 const float *__restrict__ b, int64_t ldb, int64_t ne0,
                                                                 int64_t n, float *__restrict__ y, int64_t ldy) {
    for (int64_t row = blockIdx.y; row < n; row += gridDim.y) {
        const float *ar = a + (size_t)row * lda;
        const float *br = (OP == EW_SILU) ? nullptr : b + (size_t)row * ldb;       // ldb = 0: one row for all
        float *yr = y + (size_t)row * ldy;
        if constexpr (VEC) {
            const int64_t i = 4 * ((int64_t)blockIdx.x * EW_THREADS + threadIdx.x);
            if (i < ne0) {
                const float4 va = *reinterpret_cast<const float4 *>(ar + i);
                float4 vb = {0.f, 0.f, 0.f, 0.f};
                if constexpr (OP != EW_SILU) vb = *reinterpret_cast<const float4 *>(br + i);
                *reinterpret_cast<float4 *>(yr + i) = make_float4(ew_apply<OP>(va.x, vb.x), ew_apply<OP>(va.y, vb.y),
                                                                  ew_apply<OP>(va.z, vb.z), ew_apply<OP>(va.w, vb.w));
            }
        } else {
            for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < ne0; i += (int64_t)gridDim.x * EW_THREADS)
                yr[i] = ew_apply<OP>(ar[i], OP == EW_SILU ? 0.f : br[i]);
        }
    }
}

hipError_t launch_rms_norm(const float *x, int64_t ldx, int64_t n, int64_t ne0, float eps, float *y, int64_t ldy, hipStream_t st) {
    if (n <= 0 || ne0 <= 0) return hipSuccess;
    for (int64_t r0 = 0; r0 < n; r0 += 1 << 30) {
        const int64_t rows = n - r0 < (1 << 30) ? n - r0 : (1 << 30);
        hipLaunchKernelGGL(rms_norm_kernel, dim3((unsigned)rows), dim3(EW_THREADS), 0, st, x + r0 * ldx, ldx, ne0, eps,
                           y + r0 * ldy, ldy);
    }
    return hipGetLastError();
}

template <int OP>
static hipError_t launch_ew(const float *a, int64_t lda, const float *b, int64_t ldb, int64_t ne0, int64_t n, float *y,
                            int64_t ldy, hipStream_t st) {
    if (n <= 0 || ne0 <= 0) return hipSuccess;
    const bool vec = ((ne0 | lda | ldb | ldy) & 3) == 0 && ((((uintptr_t)a) | ((uintptr_t)b) | ((uintptr_t)y)) & 15) == 0;
    const unsigned gy = (unsigned)(n < 32768 ? n : 32768);
    if (vec) {
        const unsigned gx = (unsigned)ceil_div(ne0, 4 * EW_THREADS);
        hipLaunchKernelGGL((elementwise_kernel<OP, true>), dim3(gx, gy), dim3(EW_THREADS), 0, st, a, lda, b, ldb, ne0, n, y, ldy);
    } else {
        const int64_t want = ceil_div(ne0, EW_THREADS);
        const unsigned gx = (unsigned)(want < 64 ? want : 64);
        hipLaunchKernelGGL((elementwise_kernel<OP, false>), dim3(gx, gy), dim3(EW_THREADS), 0, st, a, lda, b, ldb, ne0, n, y, ldy);
    }
    return hipGetLastError();
}

hipError_t launch_add(const float *a, int64_t lda, const float *b, int64_t ldb, int64_t ne0, int64_t n, float *y, int64_t ldy,
                      hipStream_t st) { return launch_ew<EW_ADD>(a, lda, b, ldb, ne0, n, y, ldy, st); }
hipError_t launch_mul(const float *a, int64_t lda, const float *b, int64_t ldb, int64_t ne0, int64_t n, float *y, int64_t ldy,
                      hipStream_t st) { return launch_ew<EW_MUL>(a, lda, b, ldb, ne0, n, y, ldy, st); }
hipError_t launch_silu(const float *x, int64_t ldx, int64_t ne0, int64_t n, float *y, int64_t ldy, hipStream_t st) {
    return launch_ew<EW_SILU>(x, ldx, nullptr, 0, ne0, n, y, ldy, st);
}

}  // namespace chip
