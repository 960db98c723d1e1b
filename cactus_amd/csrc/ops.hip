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
//   SOFT_MAX  lm_ggml_compute_forward_soft_max_f32 (ggml-cpu/ops.cpp:4731-4827) with the AVX2 branch of
//             lm_ggml_vec_soft_max_f32 (ggml-cpu/vec.cpp:198-208): w = x * scale + mask, e = lm_ggml_v_expf(w - max), groups
//             of 8 summed in float in the reference's shuffle order, the groups in double (a tree here, in row order
//             there: same remark as RMS_NORM), y = e * (float)(1 / sum).  Rows of a multiple of 8 values, no ALiBi.
//   CPY, CONT lm_ggml_compute_forward_dup (ggml-cpu/ops.cpp): element i of the source in its logical order becomes element
//             i of the destination; F32 -> F16 rounds to nearest even.  Bit-exact.
//   ROPE      lm_ggml_compute_forward_rope_f32 (ggml-cpu/ops.cpp:5178-5361), modes 0 and NEOX: the angle of pair i at
//             position p follows the reference's float recurrence theta_0 = p, theta_{i+1} = theta_i * theta_scale; cos
//             and sin are computed in double here and rounded once (the reference calls the C library's cosf / sinf,
//             which may differ from that by one unit in the last place), the rotation itself is unfused float
//             arithmetic as in the reference.
//   GET_ROWS  lm_ggml_compute_forward_get_rows (ggml-cpu/ops.cpp:4236-4453): selected rows of a table converted to F32 with
//             the type's dequantize_row_* expression (ggml-quants.c).  Bit-exact.
#include "dev_common.h"
#include "kernels.h"
#include "quant_dev.h"
#include "act_layout.h"

// One rounding per written operation, as in the reference's C code; the fused operations of this file are explicit fmaf calls.
#pragma clang fp contract(off)

namespace chip {

constexpr int EW_THREADS = 256;


// ---- RMS_NORM: one workgroup per row ----
// With w, the row is also multiplied by the weight row w (the MUL node that follows a norm): y = (x * scale) * w, two
// roundings as in the two separate ops; yn (may be NULL) then receives the norm itself.
// With ADD, the row normalised is a + b (the residual ADD node in front of a norm): the sum is stored to xs, which may be a
// or b themselves (every thread reads an element of a and b before it writes that element of xs, and reads back only its
// own elements), and the norm then runs over the stored sum.
template <bool ADD, int QKIND = 0>
__global__ __launch_bounds__(EW_THREADS) void rms_norm_kernel(const float *x, int64_t ldx, int64_t ne0, float eps,
                                                              float *y, int64_t ldy, const float *__restrict__ w,
                                                              float *yn, int64_t ldyn, const float *b, int64_t ldb,
                                                              float *xs, int64_t ldxs, uint8_t *__restrict__ qws, size_t qstride) {
    constexpr int qkind = QKIND;                                 // 0: no quantized copy; 1: Q8_0 / Q8_1 planes; 2: Q8_K planes
    __shared__ double part[EW_THREADS / 64];
    const float *xr = x + (size_t)blockIdx.x * ldx;
    float *yr = y + (size_t)blockIdx.x * ldy;
    const int tid = threadIdx.x;
    bool vec = ((ne0 | ldx | ldy) & 3) == 0 && ((((uintptr_t)x) | ((uintptr_t)y)) & 15) == 0;
    if (ADD) vec = vec && ((ldb | ldxs) & 3) == 0 && ((((uintptr_t)b) | ((uintptr_t)xs)) & 15) == 0;
    float *ynr = yn ? yn + (size_t)blockIdx.x * ldyn : nullptr;
    const bool vecw = vec && (!w || ((uintptr_t)w & 15) == 0) && (!yn || ((ldyn & 3) == 0 && ((uintptr_t)yn & 15) == 0));
    double sum = 0.0;
    // Vector paths: the squares are added in the order dev_common.h fixes for a row (chunk, 256-value block, blocks four
    // apart, four partial sums).  Thread tid's k-th chunk is chunk tid + 256 k, i.e. lane tid % 64 of block tid / 64 + 4 k, so
    // a wave adds the butterfly totals of its blocks as it walks the row; every lane of a wave takes part in each butterfly
    // (lanes past the end with 0.0), hence the wave-uniform bounds.  Lane 63 holds the wave's sum.
    const int64_t wave_first = 4 * (int64_t)(tid & ~63);
    // rows of up to 8192 values stay in registers between the two passes
    constexpr int RC = 8;
    const bool cached = vecw && ne0 <= 4 * EW_THREADS * RC;
    float4 keep[RC], wk[RC];                                     // wk: the weight row, asked for before the reduction
    if (cached) {
        const float *br = ADD ? b + (size_t)blockIdx.x * ldb : nullptr;
        float *sr = ADD ? xs + (size_t)blockIdx.x * ldxs : nullptr;
#pragma unroll
        for (int k = 0; k < RC; k++) {
            const int64_t i = 4 * tid + (int64_t)k * 4 * EW_THREADS;
            double d = 0.0;
            if (i < ne0) {
                float4 v = *reinterpret_cast<const float4 *>(xr + i);
                if (ADD) {
                    const float4 u = *reinterpret_cast<const float4 *>(br + i);
                    v.x += u.x; v.y += u.y; v.z += u.z; v.w += u.w;
                    *reinterpret_cast<float4 *>(sr + i) = v;
                }
                keep[k] = v;
                if (w) wk[k] = *reinterpret_cast<const float4 *>(w + i);
                d = norm_chunk_squares(v);
            }
            if (wave_first + (int64_t)k * 4 * EW_THREADS < ne0) sum += wave_sum_f64_to_lane63(d);
        }
    } else if (vec) {
        const float *br = ADD ? b + (size_t)blockIdx.x * ldb : nullptr;
        float *sr = ADD ? xs + (size_t)blockIdx.x * ldxs : nullptr;
        for (int64_t i0 = wave_first; i0 < ne0; i0 += 4 * EW_THREADS) {
            const int64_t i = i0 + 4 * (tid & 63);
            double d = 0.0;
            if (i < ne0) {
                float4 v = *reinterpret_cast<const float4 *>(xr + i);
                if (ADD) {
                    const float4 u = *reinterpret_cast<const float4 *>(br + i);
                    v.x += u.x; v.y += u.y; v.z += u.z; v.w += u.w;
                    *reinterpret_cast<float4 *>(sr + i) = v;
                }
                d = norm_chunk_squares(v);
            }
            sum += wave_sum_f64_to_lane63(d);
        }
        if (ADD) xr = sr;
    } else {
        if (ADD) {
            const float *br = b + (size_t)blockIdx.x * ldb;
            float *sr = xs + (size_t)blockIdx.x * ldxs;
            for (int64_t i = tid; i < ne0; i += EW_THREADS) {
                const float v = xr[i] + br[i];
                sr[i] = v;
                sum += (double)(v * v);
            }
            xr = sr;
        } else {
            for (int64_t i = tid; i < ne0; i += EW_THREADS) sum += (double)(xr[i] * xr[i]);
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);      // rows that are not 16-byte aligned: element by element
    }
    if ((tid & 63) == 63) part[tid >> 6] = sum;
    __syncthreads();
    double total = 0.0;
#pragma unroll
    for (int w = 0; w < EW_THREADS / 64; w++) total += part[w];
    const float mean = (float)(total / (double)ne0);
    const float scale = 1.0f / sqrtf(mean + eps);
    if (cached) {
#pragma unroll
        for (int k = 0; k < RC; k++) {
            const int64_t i = 4 * tid + (int64_t)k * 4 * EW_THREADS;
            if (i < ne0) {
                float4 v = keep[k];
                v.x *= scale; v.y *= scale; v.z *= scale; v.w *= scale;
                if (w) {
                    if (ynr) *reinterpret_cast<float4 *>(ynr + i) = v;
                    const float4 g = wk[k];
                    v.x *= g.x; v.y *= g.y; v.z *= g.z; v.w *= g.w;
                }
                *reinterpret_cast<float4 *>(yr + i) = v;
                // the row as the next matmuls want it: quantized into the workspace planes of token blockIdx.x (ne0 is a
                // multiple of 256 here, so a wave is inside the row with all its lanes or not at all)
                if constexpr (qkind == 2) {
                    const Q8_KLane q = quantize_q8_K_lane(v);
                    uint8_t *base = qws + (size_t)blockIdx.x * qstride;
                    const int64_t sb = i >> 8;
                    const int lane = tid & 63;
                    *reinterpret_cast<uint32_t *>(base + i) = q.packed;
                    if (lane == 0) reinterpret_cast<float *>(base + q8_K_off_d(ne0))[sb] = q.d;
                    if ((lane & 3) == 0) reinterpret_cast<int16_t *>(base + q8_K_off_bsums(ne0))[sb * 16 + (lane >> 2)] = (int16_t)q.bsum;
                } else if constexpr (qkind == 1) {
                    const Q8_0Lane q = quantize_q8_0_lane(v);
                    uint8_t *base = qws + (size_t)blockIdx.x * qstride;
                    const int64_t blk = i >> 5;
                    *reinterpret_cast<uint32_t *>(base + i) = q.packed;
                    if ((tid & 7) == 0) {
                        reinterpret_cast<float *>(base + q8_0_off_d(ne0))[blk] = h2f(q.dh);
                        reinterpret_cast<int32_t *>(base + q8_0_off_sum(ne0))[blk] = q.sum;
                        reinterpret_cast<float *>(base + q8_0_off_s(ne0))[blk] = h2f(q.sh);
                    }
                }
            }
        }
    } else if (vecw) {
        for (int64_t i = 4 * tid; i < ne0; i += 4 * EW_THREADS) {
            float4 v = *reinterpret_cast<const float4 *>(xr + i);
            v.x *= scale; v.y *= scale; v.z *= scale; v.w *= scale;
            if (w) {
                if (ynr) *reinterpret_cast<float4 *>(ynr + i) = v;
                const float4 g = *reinterpret_cast<const float4 *>(w + i);
                v.x *= g.x; v.y *= g.y; v.z *= g.z; v.w *= g.w;
            }
            *reinterpret_cast<float4 *>(yr + i) = v;
        }
    } else {
        for (int64_t i = tid; i < ne0; i += EW_THREADS) {
            float v = xr[i] * scale;
            if (w) {
                if (ynr) ynr[i] = v;
                v *= w[i];
            }
            yr[i] = v;
        }
    }
}

// ---- element-wise: grid.y walks the rows, grid.x the row in chunks of 4 * EW_THREADS values ----
enum { EW_ADD = 0, EW_MUL = 1, EW_SILU = 2, EW_SILU_MUL = 3 };      // SILU_MUL: silu(a) * b, the two nodes of a gated FFN in one pass
template <int OP> __device__ __forceinline__ float ew_apply(float a, float b) {
    if constexpr (OP == EW_ADD) return a + b;
    else if constexpr (OP == EW_MUL) return a * b;
    else if constexpr (OP == EW_SILU_MUL) return silu1(a) * b;
    else return silu1(a);
}
template <int OP, bool VEC>
__global__ __launch_bounds__(EW_THREADS) void elementwise_kernel(const float *a, int64_t lda,
                                                                 const float *b, int64_t ldb, int64_t ne0,
                                                                 int64_t n, float *y, int64_t ldy) {
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

// silu(x) * b with the result also left as the quantized rows of the matmul that reads it (ffn_down reads
// silu(ffn_gate) * ffn_up): what launch_quantize would write from y afterwards, without its launch.  Quantization is per
// block, so the element-wise grid serves: a lane holds four consecutive values, eight lanes a 32-value block, a wave a
// 256-value super-block, exactly the quantizer kernels' mapping (ne0 % 256 == 0 keeps every wave whole).
// KIND 1: Q8_0 / Q8_1 planes; 2: Q8_K planes.
template <int KIND>
__global__ __launch_bounds__(EW_THREADS) void silu_mul_quantized_kernel(const float *x, int64_t ldx, const float *b, int64_t ldb,
                                                                        int64_t ne0, float *y, int64_t ldy, uint8_t *qws, size_t qstride) {
    const int64_t row = blockIdx.y;
    const int64_t e0 = 4 * ((int64_t)blockIdx.x * EW_THREADS + threadIdx.x);
    if (e0 >= ne0) return;                                                  // whole waves leave together
    const float4 va = *reinterpret_cast<const float4 *>(x + (size_t)row * ldx + e0);
    const float4 vb = *reinterpret_cast<const float4 *>(b + (size_t)row * ldb + e0);
    const float4 v = make_float4(silu1(va.x) * vb.x, silu1(va.y) * vb.y, silu1(va.z) * vb.z, silu1(va.w) * vb.w);
    *reinterpret_cast<float4 *>(y + (size_t)row * ldy + e0) = v;
    uint8_t *base = qws + (size_t)row * qstride;
    if constexpr (KIND == 2) {
        const Q8_KLane q = quantize_q8_K_lane(v);
        const int lane = threadIdx.x & 63;
        const int64_t sb = e0 / QK_K;
        *reinterpret_cast<uint32_t *>(base + e0) = q.packed;
        if (lane == 0) reinterpret_cast<float *>(base + q8_K_off_d(ne0))[sb] = q.d;
        if ((lane & 3) == 0) reinterpret_cast<int16_t *>(base + q8_K_off_bsums(ne0))[sb * 16 + (lane >> 2)] = (int16_t)q.bsum;
    } else {
        const Q8_0Lane q = quantize_q8_0_lane(v);
        const int64_t blk = e0 / 32;
        *reinterpret_cast<uint32_t *>(base + e0) = q.packed;
        if ((threadIdx.x & 7) == 0) {
            reinterpret_cast<float *>(base + q8_0_off_d(ne0))[blk] = h2f(q.dh);
            reinterpret_cast<int32_t *>(base + q8_0_off_sum(ne0))[blk] = q.sum;
            reinterpret_cast<float *>(base + q8_0_off_s(ne0))[blk] = h2f(q.sh);
        }
    }
}
bool silu_mul_quantized_applicable(const float *x, int64_t ldx, const float *b, int64_t ldb, int64_t ne0, const float *y, int64_t ldy) {
    return ne0 > 0 && ne0 % 256 == 0 && ((ldx | ldb | ldy) & 3) == 0 && ((((uintptr_t)x) | ((uintptr_t)b) | ((uintptr_t)y)) & 15) == 0;
}
hipError_t launch_silu_mul_quantized(const float *x, int64_t ldx, const float *b, int64_t ldb, int64_t ne0, int64_t n, float *y,
                                     int64_t ldy, uint8_t *qws, size_t qstride, int act_kind, hipStream_t st) {
    if (n <= 0 || ne0 <= 0) return hipSuccess;
    if (n > 65535 || (act_kind != 1 && act_kind != 2) || !silu_mul_quantized_applicable(x, ldx, b, ldb, ne0, y, ldy)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)ceil_div(ne0, 4 * EW_THREADS), (unsigned)n);
    if (act_kind == 1) hipLaunchKernelGGL(silu_mul_quantized_kernel<1>, grid, dim3(EW_THREADS), 0, st, x, ldx, b, ldb, ne0, y, ldy, qws, qstride);
    else               hipLaunchKernelGGL(silu_mul_quantized_kernel<2>, grid, dim3(EW_THREADS), 0, st, x, ldx, b, ldb, ne0, y, ldy, qws, qstride);
    return hipGetLastError();
}

// ---- SCALE and GELU: one value in, one value out ----
// GELU is the reference's table form (ggml-cpu/vec.h:452-466): 0 at or below -10, x at or above 10, else entry fp16(x) of
// a 65536-entry fp16 table built on the host with the C library's tanhf (the caller uploads it).
enum { UN_SCALE = 0, UN_GELU = 1 };
template <int OP> __device__ __forceinline__ float unary_apply(float x, float s, const unsigned short *__restrict__ table) {
    if constexpr (OP == UN_SCALE) return x * s;
    else {
        if (x <= -10.0f) return 0.0f;
        if (x >= 10.0f) return x;
        return h2f(table[f2h_rne(x)]);
    }
}
template <int OP, bool VEC>
__global__ __launch_bounds__(EW_THREADS) void unary_kernel(const float *x, int64_t ldx, int64_t ne0, int64_t n,
                                                           float *y, int64_t ldy, float s,
                                                           const unsigned short *__restrict__ table) {
    for (int64_t row = blockIdx.y; row < n; row += gridDim.y) {
        const float *xr = x + (size_t)row * ldx;
        float *yr = y + (size_t)row * ldy;
        if constexpr (VEC) {
            const int64_t i = 4 * ((int64_t)blockIdx.x * EW_THREADS + threadIdx.x);
            if (i < ne0) {
                const float4 v = *reinterpret_cast<const float4 *>(xr + i);
                *reinterpret_cast<float4 *>(yr + i) = make_float4(unary_apply<OP>(v.x, s, table), unary_apply<OP>(v.y, s, table),
                                                                  unary_apply<OP>(v.z, s, table), unary_apply<OP>(v.w, s, table));
            }
        } else {
            for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < ne0; i += (int64_t)gridDim.x * EW_THREADS)
                yr[i] = unary_apply<OP>(xr[i], s, table);
        }
    }
}

// ---- SOFT_MAX: one workgroup per row; thread t owns the groups of 8 values t, t + 256, ... ----
// G > 0: the row fits 8 * G * EW_THREADS values and stays in registers.  G == 0: any length, y holds e between passes.
enum { MASK_NONE = 0, MASK_F32 = 1, MASK_F16 = 2 };
template <int MASK>
__device__ __forceinline__ void soft_max_load(const float *xr, const void *mrow, int64_t i, float scale, float (&w)[8]) {
    const float4 a = *reinterpret_cast<const float4 *>(xr + i), b = *reinterpret_cast<const float4 *>(xr + i + 4);
    w[0] = a.x * scale; w[1] = a.y * scale; w[2] = a.z * scale; w[3] = a.w * scale;
    w[4] = b.x * scale; w[5] = b.y * scale; w[6] = b.z * scale; w[7] = b.w * scale;
    if constexpr (MASK == MASK_F32) {
        const float *m = reinterpret_cast<const float *>(mrow) + i;
        const float4 c = *reinterpret_cast<const float4 *>(m), d = *reinterpret_cast<const float4 *>(m + 4);
        w[0] += c.x; w[1] += c.y; w[2] += c.z; w[3] += c.w; w[4] += d.x; w[5] += d.y; w[6] += d.z; w[7] += d.w;
    } else if constexpr (MASK == MASK_F16) {
        const u32x4 h = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const uint16_t *>(mrow) + i);
#pragma unroll
        for (int k = 0; k < 4; k++) { w[2 * k] += h2f(h[k]); w[2 * k + 1] += h2f(h[k] >> 16); }
    }
}
__device__ __forceinline__ float group_sum8(const float (&e)[8]) {
    return ((e[0] + e[4]) + (e[2] + e[6])) + ((e[1] + e[5]) + (e[3] + e[7]));
}
template <int MASK, int G>
__global__ __launch_bounds__(EW_THREADS) void soft_max_kernel(const float *x, int64_t ldx, const void *__restrict__ mask,
                                                              int64_t ne00, int64_t ne01, float scale, float *y,
                                                              int64_t ldy) {
    __shared__ float wmax[EW_THREADS / 64];
    __shared__ double wsum[EW_THREADS / 64];
    const int64_t row = blockIdx.x;
    const float *xr = x + row * ldx;
    float *yr = y + row * ldy;
    const void *mrow = nullptr;
    const int64_t mask_row = (uint32_t)blockIdx.x % (uint32_t)ne01;          // 32-bit: the 64-bit remainder is a long software routine
    if constexpr (MASK == MASK_F32) mrow = reinterpret_cast<const float *>(mask) + mask_row * ne00;
    if constexpr (MASK == MASK_F16) mrow = reinterpret_cast<const uint16_t *>(mask) + mask_row * ne00;
    const int tid = threadIdx.x;
    const int64_t groups = ne00 / 8;
    constexpr int GR = G > 0 ? G : 1;
    float w[GR][8];
    float mx = -INFINITY;
    if constexpr (G > 0) {
#pragma unroll
        for (int j = 0; j < G; j++) {
            const int64_t g = tid + (int64_t)j * EW_THREADS;
            if (g < groups) {
                soft_max_load<MASK>(xr, mrow, 8 * g, scale, w[j]);
#pragma unroll
                for (int k = 0; k < 8; k++) mx = fmaxf(mx, w[j][k]);
            }
        }
    } else {
        for (int64_t g = tid; g < groups; g += EW_THREADS) {
            soft_max_load<MASK>(xr, mrow, 8 * g, scale, w[0]);
#pragma unroll
            for (int k = 0; k < 8; k++) mx = fmaxf(mx, w[0][k]);
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if ((tid & 63) == 0) wmax[tid >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
    static_assert(EW_THREADS == 256, "four waves");

    double sum = 0.0;
    if constexpr (G > 0) {
#pragma unroll
        for (int j = 0; j < G; j++) {
            const int64_t g = tid + (int64_t)j * EW_THREADS;
            if (g < groups) {
#pragma unroll
                for (int k = 0; k < 8; k++) w[j][k] = v_expf_lane(w[j][k] - mx);
                sum += (double)group_sum8(w[j]);
            }
        }
    } else {
        for (int64_t g = tid; g < groups; g += EW_THREADS) {
            soft_max_load<MASK>(xr, mrow, 8 * g, scale, w[0]);
#pragma unroll
            for (int k = 0; k < 8; k++) w[0][k] = v_expf_lane(w[0][k] - mx);
            sum += (double)group_sum8(w[0]);
            *reinterpret_cast<float4 *>(yr + 8 * g) = make_float4(w[0][0], w[0][1], w[0][2], w[0][3]);
            *reinterpret_cast<float4 *>(yr + 8 * g + 4) = make_float4(w[0][4], w[0][5], w[0][6], w[0][7]);
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
    if ((tid & 63) == 0) wsum[tid >> 6] = sum;
    __syncthreads();
    const float inv = (float)(1.0 / ((wsum[0] + wsum[1]) + (wsum[2] + wsum[3])));
    if constexpr (G > 0) {
#pragma unroll
        for (int j = 0; j < G; j++) {
            const int64_t g = tid + (int64_t)j * EW_THREADS;
            if (g < groups) {
                *reinterpret_cast<float4 *>(yr + 8 * g) = make_float4(w[j][0] * inv, w[j][1] * inv, w[j][2] * inv, w[j][3] * inv);
                *reinterpret_cast<float4 *>(yr + 8 * g + 4) = make_float4(w[j][4] * inv, w[j][5] * inv, w[j][6] * inv, w[j][7] * inv);
            }
        }
    } else {
        for (int64_t g = tid; g < groups; g += EW_THREADS) {           // each thread re-reads what it wrote itself
            float4 a = *reinterpret_cast<float4 *>(yr + 8 * g), b = *reinterpret_cast<float4 *>(yr + 8 * g + 4);
            a.x *= inv; a.y *= inv; a.z *= inv; a.w *= inv; b.x *= inv; b.y *= inv; b.z *= inv; b.w *= inv;
            *reinterpret_cast<float4 *>(yr + 8 * g) = a;
            *reinterpret_cast<float4 *>(yr + 8 * g + 4) = b;
        }
    }
}

// Few long rows (a decode step over a long context: one row per query head): the same arithmetic with 1024 threads per row.
// Thread t takes the groups t, t + 1024, ...; its exponentials go to y and each group's sum, as a double, to LDS; the first
// 256 threads then add the group sums in the order the kernel above adds them (thread u: groups u, u + 256, ... one after the
// other, the wave butterfly, the four waves), so a row's result does not depend on which of the two kernels took it.
constexpr int SM_WIDE_THREADS = 1024;
constexpr int64_t SM_WIDE_MAX_ROWS = 128, SM_WIDE_MIN_VALUES = 8192;     // 32 rows: 8192 values 5.8 -> 5.2 us, 32768 22.6 -> 13.1 us; 4096 the same, 1024 slower
template <int MASK>
__global__ __launch_bounds__(SM_WIDE_THREADS) void soft_max_wide_kernel(const float *x, int64_t ldx, const void *__restrict__ mask,
                                                                        int64_t ne00, int64_t ne01, float scale, float *y, int64_t ldy) {
    extern __shared__ __align__(16) double group_sums[];                   // ne00 / 8 doubles
    __shared__ float wmax[SM_WIDE_THREADS / 64];
    __shared__ double wsum[EW_THREADS / 64];
    const int64_t row = blockIdx.x;
    const float *xr = x + row * ldx;
    float *yr = y + row * ldy;
    const void *mrow = nullptr;
    const int64_t mask_row = (uint32_t)blockIdx.x % (uint32_t)ne01;
    if constexpr (MASK == MASK_F32) mrow = reinterpret_cast<const float *>(mask) + mask_row * ne00;
    if constexpr (MASK == MASK_F16) mrow = reinterpret_cast<const uint16_t *>(mask) + mask_row * ne00;
    const int tid = threadIdx.x;
    const int64_t groups = ne00 / 8;
    float w[8];
    float mx = -INFINITY;
    for (int64_t g = tid; g < groups; g += SM_WIDE_THREADS) {
        soft_max_load<MASK>(xr, mrow, 8 * g, scale, w);
#pragma unroll
        for (int k = 0; k < 8; k++) mx = fmaxf(mx, w[k]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if ((tid & 63) == 0) wmax[tid >> 6] = mx;
    __syncthreads();
    mx = wmax[0];
#pragma unroll
    for (int i = 1; i < SM_WIDE_THREADS / 64; i++) mx = fmaxf(mx, wmax[i]);         // a maximum: any order
    for (int64_t g = tid; g < groups; g += SM_WIDE_THREADS) {
        soft_max_load<MASK>(xr, mrow, 8 * g, scale, w);
#pragma unroll
        for (int k = 0; k < 8; k++) w[k] = v_expf_lane(w[k] - mx);
        group_sums[g] = (double)group_sum8(w);
        *reinterpret_cast<float4 *>(yr + 8 * g) = make_float4(w[0], w[1], w[2], w[3]);
        *reinterpret_cast<float4 *>(yr + 8 * g + 4) = make_float4(w[4], w[5], w[6], w[7]);
    }
    __syncthreads();
    if (tid < EW_THREADS) {                                                // whole waves
        double sum = 0.0;
        for (int64_t g = tid; g < groups; g += EW_THREADS) sum += group_sums[g];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
        if ((tid & 63) == 0) wsum[tid >> 6] = sum;
    }
    __syncthreads();
    const float inv = (float)(1.0 / ((wsum[0] + wsum[1]) + (wsum[2] + wsum[3])));
    for (int64_t g = tid; g < groups; g += SM_WIDE_THREADS) {             // each thread re-reads what it wrote itself
        float4 a = *reinterpret_cast<float4 *>(yr + 8 * g), b = *reinterpret_cast<float4 *>(yr + 8 * g + 4);
        a.x *= inv; a.y *= inv; a.z *= inv; a.w *= inv; b.x *= inv; b.y *= inv; b.z *= inv; b.w *= inv;
        *reinterpret_cast<float4 *>(yr + 8 * g) = a;
        *reinterpret_cast<float4 *>(yr + 8 * g + 4) = b;
    }
}

template <int MASK>
static void launch_soft_max_masked(const float *x, int64_t ldx, const void *mask, int64_t ne00, int64_t ne01, int64_t n_rows,
                                   float scale, float *y, int64_t ldy, hipStream_t st) {
    const int64_t per = 8 * EW_THREADS;
    const unsigned rows = (unsigned)n_rows;
    // fewer rows than CUs and rows of more than 8192 values (8 KB of group sums per 8192 values, up to 128 KB of LDS)
    if (n_rows <= SM_WIDE_MAX_ROWS && ne00 >= SM_WIDE_MIN_VALUES && ne00 <= 131072) {
        auto kfn = soft_max_wide_kernel<MASK>;
        const size_t lds = (size_t)ne00;                                   // ne00 / 8 doubles
        static bool granted = false;
        if (lds > 48 * 1024 && !granted) {
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024) == hipSuccess)
                granted = true;
        }
        if (lds <= 48 * 1024 || granted) {
            hipLaunchKernelGGL(kfn, dim3(rows), dim3(SM_WIDE_THREADS), lds, st, x, ldx, mask, ne00, ne01, scale, y, ldy);
            return;
        }
    }
#define SM_GO(G) hipLaunchKernelGGL((soft_max_kernel<MASK, G>), dim3(rows), dim3(EW_THREADS), 0, st, x, ldx, mask, ne00, ne01, scale, y, ldy)
    if (ne00 <= per) SM_GO(1);
    else if (ne00 <= 2 * per) SM_GO(2);
    else if (ne00 <= 4 * per) SM_GO(4);
    else SM_GO(0);
#undef SM_GO
}
hipError_t launch_soft_max(const float *x, int64_t ldx, const void *mask, int mask_f16, int64_t ne00, int64_t ne01, int64_t n_rows,
                           float scale, float *y, int64_t ldy, hipStream_t st) {
    if (n_rows <= 0 || ne00 <= 0) return hipSuccess;
    if (n_rows > 0x7fffffff || ne00 % 8 != 0) return hipErrorInvalidValue;
    if (!mask) launch_soft_max_masked<MASK_NONE>(x, ldx, nullptr, ne00, ne01, n_rows, scale, y, ldy, st);
    else if (mask_f16) launch_soft_max_masked<MASK_F16>(x, ldx, mask, ne00, ne01, n_rows, scale, y, ldy, st);
    else launch_soft_max_masked<MASK_F32>(x, ldx, mask, ne00, ne01, n_rows, scale, y, ldy, st);
    return hipGetLastError();
}

// ---- CPY / CONT: same-shape strided copy with conversion; strides in bytes ----
struct CopyShape { int64_t ne[4]; int64_t nbs[4]; int64_t ned[4]; int64_t nbd[4]; };   // source shape / strides, destination shape / strides
template <typename S, typename D> __device__ __forceinline__ D cpy_conv(S v) {
    if constexpr (sizeof(S) == sizeof(D)) return v;                              // same type: the bits
    else if constexpr (sizeof(D) == 2) return f2h_rne(v);                        // F32 -> F16, nearest even
    else return h2f(v);                                                          // F16 -> F32, exact
}
template <typename S, typename D> __device__ __forceinline__ void cpy_one(const char *s, char *d) {
    *reinterpret_cast<D *>(d) = cpy_conv<S, D>(*reinterpret_cast<const S *>(s));
}
// one thread per element in logical order (i0 fastest); the two sides may have different shapes of one element count.
// IDX is uint32_t whenever the element count allows: 64-bit division is a long software routine.
template <typename IDX>
__device__ __forceinline__ int64_t cpy_offset(IDX i, const int64_t (&ne)[4], const int64_t (&nb)[4]) {
    const IDX n0 = (IDX)ne[0], n1 = (IDX)ne[1], n2 = (IDX)ne[2];
    const IDX r0 = i / n0, i0 = i - r0 * n0;
    const IDX r1 = r0 / n1, i1 = r0 - r1 * n1;
    const IDX i3 = r1 / n2, i2 = r1 - i3 * n2;
    return (int64_t)i0 * nb[0] + (int64_t)i1 * nb[1] + (int64_t)i2 * nb[2] + (int64_t)i3 * nb[3];
}
template <typename S, typename D, typename IDX, bool DENSE_DST>
__global__ __launch_bounds__(EW_THREADS) void cpy_kernel(const char *__restrict__ src, char *__restrict__ dst, CopyShape sh, int64_t total) {
    for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < total; i += (int64_t)gridDim.x * EW_THREADS)
        cpy_one<S, D>(src + cpy_offset<IDX>((IDX)i, sh.ne, sh.nbs),
                      dst + (DENSE_DST ? i * (int64_t)sizeof(D) : cpy_offset<IDX>((IDX)i, sh.ned, sh.nbd)));
}
// both sides dense in the same order: four elements per thread
template <typename S, typename D>
__global__ __launch_bounds__(EW_THREADS) void cpy_flat_kernel(const S *__restrict__ src, D *__restrict__ dst, int64_t total) {
    const int64_t i = 4 * ((int64_t)blockIdx.x * EW_THREADS + threadIdx.x);
    if (i + 3 < total) {
        if constexpr (sizeof(S) == 4 && sizeof(D) == 2) {
            const float4 v = *reinterpret_cast<const float4 *>(src + i);
            u32x2 o;
            o[0] = (uint32_t)f2h_rne(v.x) | ((uint32_t)f2h_rne(v.y) << 16);
            o[1] = (uint32_t)f2h_rne(v.z) | ((uint32_t)f2h_rne(v.w) << 16);
            *reinterpret_cast<u32x2 *>(dst + i) = o;
        } else {
#pragma unroll
            for (int k = 0; k < 4; k++) cpy_one<S, D>(reinterpret_cast<const char *>(src + i + k), reinterpret_cast<char *>(dst + i + k));
        }
    } else {
        for (int64_t k = i; k < total; k++) cpy_one<S, D>(reinterpret_cast<const char *>(src + k), reinterpret_cast<char *>(dst + k));
    }
}
// the source runs fastest along i1, the destination along i0: 32 x 32 tiles through LDS so that both sides see
// consecutive lanes on consecutive addresses
template <typename S, typename D>
__global__ __launch_bounds__(EW_THREADS) void cpy_transpose_kernel(const char *__restrict__ src, char *__restrict__ dst, CopyShape sh) {
    __shared__ S tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int64_t t0 = (int64_t)blockIdx.x * 32, t1 = (int64_t)blockIdx.y * 32;
    const int64_t i3 = (uint32_t)blockIdx.z / (uint32_t)sh.ne[2], i2 = (uint32_t)blockIdx.z - (uint32_t)i3 * (uint32_t)sh.ne[2];
    const char *s = src + i2 * sh.nbs[2] + i3 * sh.nbs[3];
    char *d = dst + i2 * sh.nbd[2] + i3 * sh.nbd[3];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int64_t i0 = t0 + ty + 8 * r, i1 = t1 + tx;
        if (i0 < sh.ne[0] && i1 < sh.ne[1]) tile[ty + 8 * r][tx] = *reinterpret_cast<const S *>(s + i0 * sh.nbs[0] + i1 * sh.nbs[1]);
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int64_t i0 = t0 + tx, i1 = t1 + ty + 8 * r;
        if (i0 < sh.ne[0] && i1 < sh.ne[1])
            *reinterpret_cast<D *>(d + i0 * sh.nbd[0] + i1 * sh.nbd[1]) = cpy_conv<S, D>(tile[tx][ty + 8 * r]);
    }
}
template <typename S, typename D>
static hipError_t launch_cpy_typed(const void *src, void *dst, const CopyShape &sh, hipStream_t st) {
    const int64_t total = sh.ne[0] * sh.ne[1] * sh.ne[2] * sh.ne[3];
    bool dense_s = true, dense_d = true, same = true;
    int64_t es = sizeof(S), ed = sizeof(D);
    for (int k = 0; k < 4; k++) {
        if (sh.ne[k] != 1 && sh.nbs[k] != es) dense_s = false;
        if (sh.ned[k] != 1 && sh.nbd[k] != ed) dense_d = false;
        if (sh.ne[k] != sh.ned[k]) same = false;
        es *= sh.ne[k]; ed *= sh.ned[k];
    }
    if (dense_s && dense_d && (((uintptr_t)src) & 15) == 0 && (((uintptr_t)dst) & 7) == 0) {
        hipLaunchKernelGGL((cpy_flat_kernel<S, D>), dim3((unsigned)ceil_div(total, 4 * EW_THREADS)), dim3(EW_THREADS), 0, st,
                           (const S *)src, (D *)dst, total);
    } else if (same && sh.nbs[1] == (int64_t)sizeof(S) && sh.nbd[0] == (int64_t)sizeof(D) && sh.ne[0] >= 16 && sh.ne[1] >= 16 &&
               sh.ne[2] * sh.ne[3] <= 65535) {
        hipLaunchKernelGGL((cpy_transpose_kernel<S, D>), dim3((unsigned)ceil_div(sh.ne[0], 32), (unsigned)ceil_div(sh.ne[1], 32),
                                                               (unsigned)(sh.ne[2] * sh.ne[3])),
                           dim3(EW_THREADS), 0, st, (const char *)src, (char *)dst, sh);
    } else {
        const int64_t want = ceil_div(total, EW_THREADS);
        const dim3 grid((unsigned)(want < (1 << 20) ? want : (1 << 20)));
        const bool small = total < (1LL << 31);
#define CPY_GO(IDX, DD) hipLaunchKernelGGL((cpy_kernel<S, D, IDX, DD>), grid, dim3(EW_THREADS), 0, st, (const char *)src, (char *)dst, sh, total)
        if (small && dense_d) CPY_GO(uint32_t, true);
        else if (small) CPY_GO(uint32_t, false);
        else if (dense_d) CPY_GO(int64_t, true);
        else CPY_GO(int64_t, false);
#undef CPY_GO
    }
    return hipGetLastError();
}
hipError_t launch_cpy(const void *src, int src_f16, const int64_t *ne_src, const int64_t *nb_src, void *dst, int dst_f16,
                      const int64_t *ne_dst, const int64_t *nb_dst, hipStream_t st) {
    CopyShape sh;
    for (int k = 0; k < 4; k++) {
        sh.ne[k] = ne_src[k]; sh.nbs[k] = nb_src[k]; sh.ned[k] = ne_dst[k]; sh.nbd[k] = nb_dst[k];
        if (ne_src[k] <= 0 || ne_dst[k] <= 0) return hipSuccess;
    }
    if (!src_f16 && !dst_f16) return launch_cpy_typed<float, float>(src, dst, sh, st);
    if (!src_f16 && dst_f16) return launch_cpy_typed<float, uint16_t>(src, dst, sh, st);
    if (src_f16 && dst_f16) return launch_cpy_typed<uint16_t, uint16_t>(src, dst, sh, st);
    return launch_cpy_typed<uint16_t, float>(src, dst, sh, st);
}

// cos and sin of a float angle, evaluated in double and rounded once.  |th| < 1e6: two-term Cody-Waite reduction by pi/2
// (the first term has 33 significant bits, so its product with the quadrant count < 2^20 is exact) and the classic
// degree-13 / degree-14 minimax polynomials on [-pi/4, pi/4]; absolute error near 1e-16, far below half a unit of the
// float result.  Larger angles go through the library's full-range reduction.
__device__ __forceinline__ void sincos_rounded(float th, float &sn, float &cs) {
    const double x = (double)th;
    if (!(fabs(x) < 1.0e6)) {
        double sd, cd;
        sincos(x, &sd, &cd);
        sn = (float)sd; cs = (float)cd;
        return;
    }
    const double fn = rint(x * 6.36619772367581382433e-01);
    const double r = fma(-fn, 1.57079632673412561417e+00, x);
    const double y = fma(-fn, 6.07710050650619224932e-11, r);
    const double z = y * y;
    const double ps = fma(z, fma(z, fma(z, fma(z, fma(z, 1.58969099521155010221e-10, -2.50507602534068634195e-08),
                                               2.75573137070700676789e-06), -1.98412698298579493134e-04),
                                 8.33333333332248946124e-03), -1.66666666666666324348e-01);
    const double s = fma(y * z, ps, y);
    const double pc = fma(z, fma(z, fma(z, fma(z, fma(z, -1.13596475577881948265e-11, 2.08757232129817482790e-09),
                                               -2.75573143513906633035e-07), 2.48015872894767294178e-05),
                                 -1.38888888888741095749e-03), 4.16666666666666019037e-02);
    const double c = fma(z * z, pc, fma(z, -0.5, 1.0));
    const int q = (int)fn & 3;
    const double ss = (q & 1) ? c : s, cc = (q & 1) ? s : c;
    sn = (float)((q & 2) ? -ss : ss);
    cs = (float)(((q + 1) & 2) ? -cc : cc);
}

// ---- GET_ROWS: one thread per output value; element i of a row in the row's block format ----
// The expressions are those of the reference's dequantize_row_* (ggml-quants.c:249-341, 1274-1296, 1476-1501, 1684-1713,
// 2430-2446), one rounding per operation, so the values are bit-identical to the CPU's.
__device__ __forceinline__ void k_scale_min(int j, const uint8_t *q, int &sc, int &m) {        // get_scale_min_k4
    if (j < 4) { sc = q[j] & 63; m = q[j + 4] & 63; }
    else { sc = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4); m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4); }
}
__device__ __constant__ int8_t k_iq4nl_values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
__device__ __forceinline__ uint32_t load_u32_unaligned2(const uint8_t *p) {
    return (uint32_t)reinterpret_cast<const uint16_t *>(p)[0] | ((uint32_t)reinterpret_cast<const uint16_t *>(p)[1] << 16);
}
template <int WT> __device__ __forceinline__ float dequant_at(const uint8_t *row, uint32_t i) {
    if constexpr (WT == T_F32) return reinterpret_cast<const float *>(row)[i];
    else if constexpr (WT == T_F16) return h2f(reinterpret_cast<const uint16_t *>(row)[i]);
    else if constexpr (WT == T_Q4_0 || WT == T_Q4_1 || WT == T_IQ4_NL) {
        constexpr int BYTES = WT == T_Q4_1 ? BYTES_Q4_1 : BYTES_Q4_0, QS = WT == T_Q4_1 ? 4 : 2;
        const uint8_t *b = row + (size_t)(i >> 5) * BYTES;
        const uint32_t j = i & 31;
        const float d = h2f(reinterpret_cast<const uint16_t *>(b)[0]);
        const int q = b[QS + (j & 15)], nib = j < 16 ? (q & 0xF) : (q >> 4);
        if constexpr (WT == T_Q4_0) return (float)(nib - 8) * d;
        else if constexpr (WT == T_Q4_1) return (float)nib * d + h2f(reinterpret_cast<const uint16_t *>(b)[1]);
        else return d * (float)k_iq4nl_values[nib];
    } else if constexpr (WT == T_Q8_0) {
        const uint8_t *b = row + (size_t)(i >> 5) * BYTES_Q8_0;
        return (float)(int8_t)b[2 + (i & 31)] * h2f(reinterpret_cast<const uint16_t *>(b)[0]);
    } else if constexpr (WT == T_Q5_0 || WT == T_Q5_1) {
        constexpr int BYTES = WT == T_Q5_1 ? BYTES_Q5_1 : BYTES_Q5_0, QH = WT == T_Q5_1 ? 4 : 2;
        const uint8_t *b = row + (size_t)(i >> 5) * BYTES;
        const uint32_t j = i & 31;
        const float d = h2f(reinterpret_cast<const uint16_t *>(b)[0]);
        const uint32_t qh = load_u32_unaligned2(b + QH);
        const int q = b[QH + 4 + (j & 15)];
        const int v = j < 16 ? ((q & 0xF) | (int)(((qh >> j) << 4) & 0x10)) : ((q >> 4) | (int)((qh >> (j - 16 + 12)) & 0x10));
        if constexpr (WT == T_Q5_0) return (float)(v - 16) * d;
        else return (float)v * d + h2f(reinterpret_cast<const uint16_t *>(b)[1]);
    } else if constexpr (WT == T_Q4_K || WT == T_Q5_K) {
        constexpr int BYTES = WT == T_Q5_K ? BYTES_Q5_K : BYTES_Q4_K, QS = WT == T_Q5_K ? 48 : 16;
        const uint8_t *b = row + (size_t)(i >> 8) * BYTES;
        const uint32_t r = i & 255, j64 = r >> 6, l = r & 63, hi = l >> 5, ll = l & 31;
        const float d = h2f(reinterpret_cast<const uint16_t *>(b)[0]), mn = h2f(reinterpret_cast<const uint16_t *>(b)[1]);
        int sc, m;
        k_scale_min((int)(2 * j64 + hi), b + 4, sc, m);
        const float d1 = d * (float)sc, m1 = mn * (float)m;
        const int q = b[QS + 32 * j64 + ll];
        int v = hi ? (q >> 4) : (q & 0xF);
        if constexpr (WT == T_Q5_K) v += (b[16 + ll] & (1u << (2 * j64 + hi))) ? 16 : 0;
        return d1 * (float)v - m1;
    } else if constexpr (WT == T_IQ4_XS) {                              // d scales_h scales_l[4] qs[128] (ggml-quants.c dequantize_row_iq4_xs)
        const uint8_t *b = row + (size_t)(i >> 8) * BYTES_IQ4_XS;
        const uint32_t r = i & 255, ib = r >> 5, j = r & 31;
        const uint32_t sh = reinterpret_cast<const uint16_t *>(b)[1];
        const int ls = (int)(((b[4 + (ib >> 1)] >> (4 * (ib & 1))) & 0xFu) | (((sh >> (2 * ib)) & 3u) << 4)) - 32;
        const int q = b[8 + 16 * ib + (j & 15)], nib = j < 16 ? (q & 0xF) : (q >> 4);
        return h2f(reinterpret_cast<const uint16_t *>(b)[0]) * (float)ls * (float)k_iq4nl_values[nib];
    } else if constexpr (WT == T_Q2_K) {                                // scales[16] qs[64] d dmin (reference ggml-quants.c:706-737)
        const uint8_t *b = row + (size_t)(i >> 8) * BYTES_Q2_K;
        const uint32_t r = i & 255, h = r >> 7, j = (r >> 5) & 3, l = r & 31;
        const float d = h2f(reinterpret_cast<const uint16_t *>(b + 80)[0]), mn = h2f(reinterpret_cast<const uint16_t *>(b + 80)[1]);
        const int sc = b[8 * h + 2 * j + (l >> 4)];
        const float dl = d * (float)(sc & 0xF), ml = mn * (float)(sc >> 4);
        return dl * (float)(int8_t)((b[16 + 32 * h + l] >> (2 * j)) & 3) - ml;
    } else if constexpr (WT == T_Q3_K) {                                // hmask[32] qs[64] scales[12] d (ggml-quants.c:1050-1098)
        const uint8_t *b = row + (size_t)(i >> 8) * BYTES_Q3_K;
        const uint32_t r = i & 255, h = r >> 7, j = (r >> 5) & 3, l = r & 31;
        const uint32_t is = 8 * h + 2 * j + (l >> 4);                   // scale index: low nibbles in bytes 0..7, high bit pairs in 8..11
        const uint8_t *s = b + 96;
        const int lo4 = is < 8 ? (s[is] & 0xF) : (s[is - 8] >> 4);
        const int hi2 = (s[8 + (is & 3)] >> (2 * (is >> 2))) & 3;
        const float dl = h2f(reinterpret_cast<const uint16_t *>(b + 108)[0]) * (float)((lo4 | (hi2 << 4)) - 32);
        const int q = (int)(int8_t)((b[32 + 32 * h + l] >> (2 * j)) & 3) - ((b[l] & (1u << (4 * h + j))) ? 0 : 4);
        return dl * (float)q;
    } else {                                                            // T_Q6_K: ql[128] qh[64] scales[16] d
        const uint8_t *b = row + (size_t)(i >> 8) * BYTES_Q6_K;
        const uint32_t r = i & 255, h = r >> 7, rr = r & 127, quarter = rr >> 5, l = rr & 31;
        const uint8_t *ql = b + 64 * h, *qh = b + 128 + 32 * h;
        const int8_t *sc = reinterpret_cast<const int8_t *>(b + 192 + 8 * h);
        const float d = h2f(reinterpret_cast<const uint16_t *>(b + 208)[0]);
        const int lo = (quarter & 1) ? ql[l + 32] : ql[l];
        const int nib = (quarter & 2) ? (lo >> 4) : (lo & 0xF);
        const int q = (int)(int8_t)(nib | (((qh[l] >> (2 * quarter)) & 3) << 4)) - 32;
        return d * (float)sc[(l >> 4) + 2 * quarter] * (float)q;
    }
}
template <int WT>
__global__ __launch_bounds__(EW_THREADS) void get_rows_kernel(GetRowsArgs a) {
    const uint32_t per = (uint32_t)(a.ne11 * a.ne10), rows = per * (uint32_t)a.ne12;
    for (uint32_t r = blockIdx.y; r < rows; r += gridDim.y) {                   // row of dst: (i12, i11, i10), i10 fastest
        const uint32_t i12 = r / per, rem = r - i12 * per, i11 = rem / (uint32_t)a.ne10, i10 = rem - i11 * (uint32_t)a.ne10;
        const int64_t id = a.ids[i10 + i11 * a.ldi1 + i12 * a.ldi2];
        if (id < 0 || id >= a.ne01) continue;                                   // the reference asserts; the row stays unwritten
        const uint8_t *row = a.src + id * a.nb01 + i11 * a.nb02 + i12 * a.nb03;
        float *out = a.dst + i10 * a.ld1 + i11 * a.ld2 + i12 * a.ld3;
        for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < a.nc; i += (int64_t)gridDim.x * EW_THREADS)
            out[i] = dequant_at<WT>(row, (uint32_t)i);
    }
}
hipError_t launch_get_rows(int type, const GetRowsArgs &a, hipStream_t st) {
    const int64_t rows = a.ne10 * a.ne11 * a.ne12;
    if (rows <= 0 || a.nc <= 0) return hipSuccess;
    if (a.nc > 0x7fffffff) return hipErrorInvalidValue;
    const int64_t want = ceil_div(a.nc, EW_THREADS);
    const unsigned gx = (unsigned)(want < 64 ? want : 64);
    if (rows > 0x7fffffff) return hipErrorInvalidValue;
    const dim3 grid(gx, (unsigned)(rows < 65535 ? rows : 65535));
#define GR_CASE(TT) case TT: hipLaunchKernelGGL(get_rows_kernel<TT>, grid, dim3(EW_THREADS), 0, st, a); break;
    switch (type) {
        GR_CASE(T_F32) GR_CASE(T_F16) GR_CASE(T_Q4_0) GR_CASE(T_Q4_1) GR_CASE(T_Q5_0) GR_CASE(T_Q5_1) GR_CASE(T_Q8_0)
        GR_CASE(T_Q4_K) GR_CASE(T_Q5_K) GR_CASE(T_Q6_K) GR_CASE(T_IQ4_NL) GR_CASE(T_Q3_K) GR_CASE(T_Q2_K) GR_CASE(T_IQ4_XS)
        default: return hipErrorInvalidValue;
    }
#undef GR_CASE
    return hipGetLastError();
}

// ---- ROPE: one workgroup per token; the first n_dims / 2 threads build that position's cos / sin table ----
// The table depends on the positions and the op's parameters only, and a graph applies the same one to Q and K of every
// layer: ROPE_BUILD writes it to memory ([token][cos of the n_dims / 2 pairs | sin of the pairs], scaled by mscale) and
// ROPE_APPLY reads it back, which leaves a kernel with no serial part.  ROPE_FULL does both in one launch.  The three give
// the same bits.
enum { ROPE_FULL = 0, ROPE_BUILD = 1, ROPE_APPLY = 2 };
constexpr int ROPE_MAX_PAIRS = 256;
template <int MODE>
__global__ __launch_bounds__(EW_THREADS) void rope_kernel(const float *x, const int32_t *__restrict__ pos,
                                                          const float *__restrict__ freq_factors, RopeArgs a, float *y,
                                                          float *__restrict__ table, const float *xb, RopeArgs ab, float *yb) {
    __shared__ float cs[ROPE_MAX_PAIRS], sn[ROPE_MAX_PAIRS];
    // a second tensor with the same table (Q and K of a layer): the workgroups with blockIdx.y == 1 take it
    if (blockIdx.y == 1) { x = xb; a = ab; y = yb; }
    constexpr int PRE = 8;                                       // items per thread whose loads are issued before the table is built
    const int64_t tok = blockIdx.x;
    const int half = a.n_dims / 2;
    const float *xt = x + tok * a.ldx2;
    float *yt = y ? y + tok * a.ldy2 : nullptr;                  // no fp32 result wanted: only the fp16 copy
    const uint32_t per_head = (uint32_t)(a.ne0 - half);          // one item per rotated pair or per passed-through value
    const uint32_t items = (uint32_t)a.ne1 * per_head;           // 32-bit division: the 64-bit one is a long software routine
    // the operands of the first PRE * EW_THREADS items do not depend on the table: fetch them first
    float x0[PRE], x1[PRE];
    uint32_t ia[PRE], ib[PRE], jj[PRE], ha[PRE], hb[PRE];       // ha / hb: where the two values go in the fp16 copy
    float *tab = table + tok * a.n_dims;                         // this token's cos | sin
    if constexpr (MODE == ROPE_APPLY) {
        for (int p = threadIdx.x; p < half; p += EW_THREADS) { cs[p] = tab[p]; sn[p] = tab[half + p]; }
    }
#pragma unroll
    for (int u = 0; u < PRE; u++) {
        const uint32_t i = threadIdx.x + u * EW_THREADS;
        jj[u] = 0xffffffffu;                                     // no item
        if (MODE != ROPE_BUILD && i < items) {
            const uint32_t h = i / per_head, j = i - h * per_head;
            const uint32_t base = h * (uint32_t)a.ldx1;
            jj[u] = j;
            if (j < (uint32_t)half) { ia[u] = a.neox ? j : 2 * j; ib[u] = a.neox ? j + half : 2 * j + 1; }
            else                    { ia[u] = j + half; ib[u] = j + half; }
            x0[u] = xt[base + ia[u]];
            x1[u] = xt[base + ib[u]];
            ha[u] = ia[u] + h * (uint32_t)a.ld16_1;
            hb[u] = ib[u] + h * (uint32_t)a.ld16_1;
            ia[u] += h * (uint32_t)a.ldy1;
            ib[u] += h * (uint32_t)a.ldy1;
        }
    }
    if (MODE != ROPE_APPLY && ((int)threadIdx.x < half || half > EW_THREADS)) {
        // every lane walks the same chain theta_0 = pos, theta_{k+1} = theta_k * theta_scale and keeps its own step
        float theta = (float)(int64_t)pos[tok];
        for (int p0 = 0; p0 < half; p0 += EW_THREADS) {
            const int p = p0 + threadIdx.x;
            float mine = theta;
            const int steps = half - p0 < EW_THREADS ? half - p0 : EW_THREADS;
            for (int k = 0; k < steps; k++) {
                mine = (k == (int)threadIdx.x) ? theta : mine;
                theta *= a.theta_scale;
            }
            if (p < half) {
                const float ff = freq_factors ? freq_factors[p] : 1.0f;
                const float extrap = mine / ff;
                const float interp = a.freq_scale * extrap;
                float th = interp;
                if (a.ext_factor != 0.0f) {
                    const float d = a.corr1 - a.corr0;
                    const float yv = ((float)p - a.corr0) / fmaxf(0.001f, d);
                    const float ramp_mix = (1.0f - fminf(1.0f, fmaxf(0.0f, yv))) * a.ext_factor;
                    th = interp * (1.0f - ramp_mix) + extrap * ramp_mix;
                }
                float sf, cf;
                sincos_rounded(th, sf, cf);
                cs[p] = cf * a.mscale;
                sn[p] = sf * a.mscale;
                if constexpr (MODE == ROPE_BUILD) { tab[p] = cs[p]; tab[half + p] = sn[p]; }
            }
        }
    }
    if constexpr (MODE == ROPE_BUILD) return;
    __syncthreads();
    unsigned short *ht = a.y16 ? a.y16 + tok * a.ld16_2 : nullptr;
#pragma unroll
    for (int u = 0; u < PRE; u++) {
        if (jj[u] == 0xffffffffu) continue;
        if (jj[u] < (uint32_t)half) {
            const float c = cs[jj[u]], s = sn[jj[u]];
            const float r0 = x0[u] * c - x1[u] * s, r1 = x0[u] * s + x1[u] * c;
            if (yt) { yt[ia[u]] = r0; yt[ib[u]] = r1; }
            if (ht) { ht[ha[u]] = f2h_rne(r0); ht[hb[u]] = f2h_rne(r1); }
        } else {
            if (yt) yt[ia[u]] = x0[u];
            if (ht) ht[ha[u]] = f2h_rne(x0[u]);
        }
    }
    for (uint32_t i = threadIdx.x + PRE * EW_THREADS; i < items; i += EW_THREADS) {
        const uint32_t h = i / per_head, j = i - h * per_head;
        const float *xr = xt + h * a.ldx1;
        float *yr = yt ? yt + h * a.ldy1 : nullptr;
        unsigned short *hr = ht ? ht + h * a.ld16_1 : nullptr;
        if (j < (uint32_t)half) {
            const int64_t ka = a.neox ? j : 2 * j, kb = a.neox ? j + half : 2 * j + 1;
            const float v0 = xr[ka], v1 = xr[kb], c = cs[j], s = sn[j];
            const float r0 = v0 * c - v1 * s, r1 = v0 * s + v1 * c;
            if (yr) { yr[ka] = r0; yr[kb] = r1; }
            if (hr) { hr[ka] = f2h_rne(r0); hr[kb] = f2h_rne(r1); }
        } else {
            if (yr) yr[j + half] = xr[j + half];
            if (hr) hr[j + half] = f2h_rne(xr[j + half]);
        }
    }
}
// table == nullptr: one launch.  Otherwise build (x, y unused) or apply (pos, freq_factors unused) against table.
static bool rope_args_ok(const RopeArgs &a) {
    if (a.n_dims / 2 > ROPE_MAX_PAIRS || a.ne2 > 0x7fffffff || a.ne0 * a.ne1 > 0x7fffffff) return false;
    return !(a.ne1 * a.ldx1 > 0x7fffffff || a.ne1 * a.ldy1 > 0x7fffffff || a.ne1 * a.ld16_1 > 0x7fffffff);   // 32-bit offsets inside a token
}
hipError_t launch_rope(const float *x, const int32_t *pos, const float *freq_factors, const RopeArgs &a, float *y, float *table,
                       bool build, hipStream_t st) {
    if (a.ne2 <= 0 || (!build && (a.ne0 <= 0 || a.ne1 <= 0))) return hipSuccess;
    if (!rope_args_ok(a)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)a.ne2), block(EW_THREADS);
    if (!table) hipLaunchKernelGGL(rope_kernel<ROPE_FULL>, grid, block, 0, st, x, pos, freq_factors, a, y, (float *)nullptr, x, a, y);
    else if (build) hipLaunchKernelGGL(rope_kernel<ROPE_BUILD>, grid, block, 0, st, x, pos, freq_factors, a, y, table, x, a, y);
    else hipLaunchKernelGGL(rope_kernel<ROPE_APPLY>, grid, block, 0, st, x, pos, freq_factors, a, y, table, x, a, y);
    return hipGetLastError();
}
// Two tensors rotated with one table in one launch (same ne0, ne2, n_dims and mode; heads, strides and outputs of their own;
// y may be null where only the fp16 copy is wanted).
hipError_t launch_rope_apply_two(const float *xa, const RopeArgs &a, float *ya, const float *xb, const RopeArgs &b, float *yb,
                                 const float *table, hipStream_t st) {
    if (a.ne2 <= 0 || a.ne0 <= 0 || a.ne1 <= 0 || b.ne1 <= 0) return hipErrorInvalidValue;
    if (a.ne0 != b.ne0 || a.ne2 != b.ne2 || a.n_dims != b.n_dims || a.neox != b.neox || !rope_args_ok(a) || !rope_args_ok(b)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)a.ne2, 2), block(EW_THREADS);
    hipLaunchKernelGGL(rope_kernel<ROPE_APPLY>, grid, block, 0, st, xa, (const int32_t *)nullptr, (const float *)nullptr, a, ya,
                       const_cast<float *>(table), xb, b, yb);
    return hipGetLastError();
}

hipError_t launch_rms_norm(const float *x, int64_t ldx, int64_t n, int64_t ne0, float eps, float *y, int64_t ldy, hipStream_t st) {
    if (n <= 0 || ne0 <= 0) return hipSuccess;
    for (int64_t r0 = 0; r0 < n; r0 += 1 << 30) {
        const int64_t rows = n - r0 < (1 << 30) ? n - r0 : (1 << 30);
        hipLaunchKernelGGL(rms_norm_kernel<false>, dim3((unsigned)rows), dim3(EW_THREADS), 0, st, x + r0 * ldx, ldx, ne0, eps,
                           y + r0 * ldy, ldy, (const float *)nullptr, (float *)nullptr, (int64_t)0, (const float *)nullptr,
                           (int64_t)0, (float *)nullptr, (int64_t)0, (uint8_t *)nullptr, (size_t)0);
    }
    return hipGetLastError();
}
hipError_t launch_rms_norm_mul(const float *x, int64_t ldx, int64_t n, int64_t ne0, float eps, const float *w, float *yn, int64_t ldyn,
                               float *y, int64_t ldy, hipStream_t st) {
    if (n <= 0 || ne0 <= 0) return hipSuccess;
    if (n > 0x7fffffff) return hipErrorInvalidValue;
    hipLaunchKernelGGL(rms_norm_kernel<false>, dim3((unsigned)n), dim3(EW_THREADS), 0, st, x, ldx, ne0, eps, y, ldy, w, yn, ldyn,
                       (const float *)nullptr, (int64_t)0, (float *)nullptr, (int64_t)0, (uint8_t *)nullptr, (size_t)0);
    return hipGetLastError();
}
hipError_t launch_add_rms_norm_mul(const float *a, int64_t lda, const float *b, int64_t ldb, float *xs, int64_t ldxs, int64_t n,
                                   int64_t ne0, float eps, const float *w, float *yn, int64_t ldyn, float *y, int64_t ldy,
                                   hipStream_t st) {
    if (n <= 0 || ne0 <= 0) return hipSuccess;
    if (n > 0x7fffffff) return hipErrorInvalidValue;
    hipLaunchKernelGGL(rms_norm_kernel<true>, dim3((unsigned)n), dim3(EW_THREADS), 0, st, a, lda, ne0, eps, y, ldy, w, yn, ldyn, b,
                       ldb, xs, ldxs, (uint8_t *)nullptr, (size_t)0);
    return hipGetLastError();
}
// The norm (with or without the residual ADD in front: b may be NULL) whose result also goes, quantized as the activation
// type act_kind (1 = Q8_0 / Q8_1 planes, 2 = Q8_K planes), into the matmul workspace.  Rows of up to 8192 values that
// are a multiple of 256 and meet the vector alignment (the register-resident path of the kernel); false otherwise.
bool norm_quantized_applicable(const float *a, int64_t lda, const float *b, int64_t ldb, const float *xs, int64_t ldxs, int64_t ne0,
                               const float *w, const float *y, int64_t ldy) {
    if (ne0 <= 0 || ne0 % 256 != 0 || ne0 > 4 * EW_THREADS * 8) return false;
    bool vec = ((lda | ldy) & 3) == 0 && ((((uintptr_t)a) | ((uintptr_t)y) | ((uintptr_t)w)) & 15) == 0;
    if (b) vec = vec && ((ldb | ldxs) & 3) == 0 && ((((uintptr_t)b) | ((uintptr_t)xs)) & 15) == 0;
    return vec;
}
hipError_t launch_norm_quantized(const float *a, int64_t lda, const float *b, int64_t ldb, float *xs, int64_t ldxs, int64_t n,
                                 int64_t ne0, float eps, const float *w, float *y, int64_t ldy, uint8_t *qws, size_t qstride,
                                 int act_kind, hipStream_t st) {
    if (n <= 0 || ne0 <= 0) return hipSuccess;
    if (n > 0x7fffffff || !norm_quantized_applicable(a, lda, b, ldb, xs, ldxs, ne0, w, y, ldy)) return hipErrorInvalidValue;
    if (act_kind != 1 && act_kind != 2) return hipErrorInvalidValue;
    const dim3 grid((unsigned)n), block(EW_THREADS);
    const float *nob = nullptr;
    float *nos = nullptr, *noyn = nullptr;
    const int64_t z = 0;
    if (b && act_kind == 1)  hipLaunchKernelGGL((rms_norm_kernel<true, 1>), grid, block, 0, st, a, lda, ne0, eps, y, ldy, w, noyn, z, b, ldb, xs, ldxs, qws, qstride);
    else if (b)              hipLaunchKernelGGL((rms_norm_kernel<true, 2>), grid, block, 0, st, a, lda, ne0, eps, y, ldy, w, noyn, z, b, ldb, xs, ldxs, qws, qstride);
    else if (act_kind == 1)  hipLaunchKernelGGL((rms_norm_kernel<false, 1>), grid, block, 0, st, a, lda, ne0, eps, y, ldy, w, noyn, z, nob, z, nos, z, qws, qstride);
    else                     hipLaunchKernelGGL((rms_norm_kernel<false, 2>), grid, block, 0, st, a, lda, ne0, eps, y, ldy, w, noyn, z, nob, z, nos, z, qws, qstride);
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
hipError_t launch_silu_mul(const float *x, int64_t ldx, const float *b, int64_t ldb, int64_t ne0, int64_t n, float *y, int64_t ldy,
                           hipStream_t st) { return launch_ew<EW_SILU_MUL>(x, ldx, b, ldb, ne0, n, y, ldy, st); }
hipError_t launch_silu(const float *x, int64_t ldx, int64_t ne0, int64_t n, float *y, int64_t ldy, hipStream_t st) {
    return launch_ew<EW_SILU>(x, ldx, nullptr, 0, ne0, n, y, ldy, st);
}

template <int OP>
static hipError_t launch_unary(const float *x, int64_t ldx, int64_t ne0, int64_t n, float *y, int64_t ldy, float s,
                               const unsigned short *table, hipStream_t st) {
    if (n <= 0 || ne0 <= 0) return hipSuccess;
    const bool vec = ((ne0 | ldx | ldy) & 3) == 0 && ((((uintptr_t)x) | ((uintptr_t)y)) & 15) == 0;
    const unsigned gy = (unsigned)(n < 32768 ? n : 32768);
    if (vec) {
        hipLaunchKernelGGL((unary_kernel<OP, true>), dim3((unsigned)ceil_div(ne0, 4 * EW_THREADS), gy), dim3(EW_THREADS), 0, st, x, ldx,
                           ne0, n, y, ldy, s, table);
    } else {
        const int64_t want = ceil_div(ne0, EW_THREADS);
        hipLaunchKernelGGL((unary_kernel<OP, false>), dim3((unsigned)(want < 64 ? want : 64), gy), dim3(EW_THREADS), 0, st, x, ldx, ne0,
                           n, y, ldy, s, table);
    }
    return hipGetLastError();
}
// ---- Q6_K rows between block_q6_K order and planes (ql | qh | scales | d per row): one workgroup per row takes the row
// into LDS and writes it in the other order, to the same place or to another matrix; rows of up to 160 KB ----
template <bool TO_PLANES>
__global__ __launch_bounds__(256) void repack_q6_K_kernel(const uint8_t *src, size_t nb01_src, uint8_t *dst, size_t nb01_dst, int nsb) {
    extern __shared__ __align__(16) uint8_t rowbuf[];
    const uint16_t *in = reinterpret_cast<const uint16_t *>(src + (size_t)blockIdx.x * nb01_src);
    uint16_t *row = reinterpret_cast<uint16_t *>(dst + (size_t)blockIdx.x * nb01_dst);
    uint16_t *buf = reinterpret_cast<uint16_t *>(rowbuf);
    const int halves = nsb * (BYTES_Q6_K / 2);                        // the row in 2-byte pieces (its fields are multiples of 2 bytes)
    for (int i = threadIdx.x; i < halves; i += 256) buf[i] = in[i];
    __syncthreads();
    // piece p of super-block sb in block order: ql 0..63 | qh 64..95 | scales 96..103 | d 104; in planes: its field's plane
    for (int i = threadIdx.x; i < halves; i += 256) {
        const int sb = i / 105, p = i - sb * 105;
        const int q = p < 64 ? sb * 64 + p : p < 96 ? nsb * 64 + sb * 32 + (p - 64) : p < 104 ? nsb * 96 + sb * 8 + (p - 96) : nsb * 104 + sb;
        if (TO_PLANES) row[q] = buf[i];
        else row[i] = buf[q];
    }
}
hipError_t launch_repack_q6_K(const void *src, size_t nb01_src, void *dst, size_t nb01_dst, int64_t K, int64_t N, bool to_planes,
                              int max_lds, hipStream_t st) {
    const int64_t nsb = K / 256;
    const size_t bytes = (size_t)nsb * BYTES_Q6_K;
    if (N <= 0 || nsb <= 0) return hipSuccess;
    if (bytes > (size_t)max_lds || N > 0x7fffffff) return hipErrorInvalidValue;
    auto kfn = to_planes ? repack_q6_K_kernel<true> : repack_q6_K_kernel<false>;
    if (bytes > 48 * 1024)
        if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes); e != hipSuccess) return e;
    hipLaunchKernelGGL(kfn, dim3((unsigned)N), dim3(256), bytes, st, (const uint8_t *)src, nb01_src, (uint8_t *)dst, nb01_dst, (int)nsb);
    return hipGetLastError();
}

hipError_t launch_scale(const float *x, int64_t ldx, int64_t ne0, int64_t n, float s, float *y, int64_t ldy, hipStream_t st) {
    return launch_unary<UN_SCALE>(x, ldx, ne0, n, y, ldy, s, nullptr, st);
}
hipError_t launch_gelu(const float *x, int64_t ldx, int64_t ne0, int64_t n, const unsigned short *table, float *y, int64_t ldy,
                       hipStream_t st) {
    return launch_unary<UN_GELU>(x, ldx, ne0, n, y, ldy, 0.0f, table, st);
}

}  // namespace chip
