// The two matmuls of attention over an F16 KV cache, LM_GGML_OP_MUL_MAT with an F16 src0 that is a strided, batched view
// (reference llama-graph.cpp:1120 kq = mul_mat(k, q) and :1154 kqv = mul_mat(v, kq); CPU path
// lm_ggml_compute_forward_mul_mat, ggml-cpu/ggml-cpu.c:1177-1456, with type_traits_cpu[LM_GGML_TYPE_F16]: src1 rounded to
// fp16 by lm_ggml_cpu_fp32_to_fp16, lm_ggml_vec_dot_f16 accumulating the products of the widened halves in fp32, src0's
// batch index = src1's batch index / r2).
//
//   y[b][t][r] = sum_k  W[b / r2][r][k] * fp16(x[b][t][k])        b < ne12 = ne02 * r2, t < n, r < N
//
// kq:  W = the K cache seen as [head_dim, n_kv, n_head_kv]: rows of head_dim halves, row stride one cache position.
//      K = head_dim is small: LPR = K / 8 lanes (8, 16 or 32) share a row, a wave reads 64 / LPR rows per load.
// kqv: W = the transposed V cache seen as [n_kv, head_dim, n_head_kv]: rows of n_kv halves.  K is long: a wave per row.
//
// A workgroup handles one src0 batch (KV head) and with it the r2 src1 batches (query heads) that share it, so a row of
// the cache is read once for all of them.  The (query head, token) pairs of the KV head are "columns"; a pass keeps COLS
// fp32 accumulators per lane and walks the row once.  Activations are rounded to fp16 on the fly (v_cvt_f16_f32, round
// to nearest even) and fed to v_fma_mix_f32 as halves.  Both kernels are bound by the cache bytes (HBM) for few tokens
// and by the vector pipe for many; the summation order differs from the reference's 4 x 8-lane accumulators, so parity
// is a tolerance (1e-5 of sum |terms|), as for the other fp32-accumulating kernels.
#include "dev_common.h"
#include "kernels.h"

namespace chip {

namespace {

constexpr int AM_THREADS = 256;
constexpr int AM_COLS = 8;

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float dot8(const u32x4 w, const float4 a, const float4 b, float acc) {
    const float xs[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const half2_t wv = __builtin_bit_cast(half2_t, ws[i]);
        const _Float16 x0 = (_Float16)xs[2 * i], x1 = (_Float16)xs[2 * i + 1];          // round to nearest even
        acc = __builtin_fmaf((float)wv.x, (float)x0, acc);
        acc = __builtin_fmaf((float)wv.y, (float)x1, acc);
    }
    return acc;
}

struct BatchedArgs {
    const uint8_t *W; size_t nb01, nb02;
    int64_t K, N;
    const float *x; int64_t ldx1, ldx2;      // token and batch strides of src1, in floats
    int64_t n, r2;
    float *y; int64_t ldy1, ldy2;            // token and batch strides of dst, in floats
};

// LPR lanes per row.  Column c of a KV head: query head c % r2 of the group, token c / r2.
template <int LPR>
__global__ __launch_bounds__(AM_THREADS) void mul_mat_f16_batched_kernel(BatchedArgs a) {
    constexpr int RPS = 64 / LPR;                                    // rows per wave step
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane % LPR, grp = lane / LPR;
    const int64_t b0 = blockIdx.y;
    const uint8_t *Wb = a.W + b0 * a.nb02;
    const int64_t chunks = a.K / 8;
    const int64_t cols = a.r2 * a.n;
    const int64_t row_step = (int64_t)gridDim.x * (AM_THREADS / 64) * RPS;
    for (int64_t row = ((int64_t)blockIdx.x * (AM_THREADS / 64) + wave) * RPS + grp; row < a.N; row += row_step) {
        const u32x4 *wrow = reinterpret_cast<const u32x4 *>(Wb + row * a.nb01);
        for (int64_t c0 = 0; c0 < cols; c0 += AM_COLS) {
            float acc[AM_COLS];
            const float *xc[AM_COLS];
#pragma unroll
            for (int j = 0; j < AM_COLS; j++) {
                acc[j] = 0.0f;
                const int64_t c = c0 + j < cols ? c0 + j : cols - 1;               // clamped: loads stay in bounds, result unused
                xc[j] = a.x + (b0 * a.r2 + c % a.r2) * a.ldx2 + (c / a.r2) * a.ldx1;
            }
            for (int64_t ch = sub; ch < chunks; ch += LPR) {
                const u32x4 w = wrow[ch];
#pragma unroll
                for (int j = 0; j < AM_COLS; j++) {
                    const float4 *xp = reinterpret_cast<const float4 *>(xc[j] + 8 * ch);
                    acc[j] = dot8(w, xp[0], xp[1], acc[j]);
                }
            }
#pragma unroll
            for (int j = 0; j < AM_COLS; j++) {
#pragma unroll
                for (int o = LPR / 2; o > 0; o >>= 1) acc[j] += __shfl_xor(acc[j], o);
            }
            if (sub == 0) {
#pragma unroll
                for (int j = 0; j < AM_COLS; j++) {
                    const int64_t c = c0 + j;
                    if (c < cols) a.y[(b0 * a.r2 + c % a.r2) * a.ldy2 + (c / a.r2) * a.ldy1 + row] = acc[j];
                }
            }
        }
    }
}

}  // namespace

bool mul_mat_f16_batched_supported(int64_t K) { return K > 0 && K % 8 == 0; }

hipError_t launch_mul_mat_f16_batched(const void *W, size_t nb01, size_t nb02, int64_t K, int64_t N, int64_t ne02, const float *x,
                                      int64_t ldx1, int64_t ldx2, int64_t n, int64_t r2, float *y, int64_t ldy1, int64_t ldy2,
                                      const DeviceLimits &lim, hipStream_t st) {
    if (N <= 0 || n <= 0 || ne02 <= 0 || r2 <= 0) return hipSuccess;
    if (!mul_mat_f16_batched_supported(K) || ne02 > 65535) return hipErrorInvalidValue;
    const BatchedArgs a{(const uint8_t *)W, nb01, nb02, K, N, x, ldx1, ldx2, n, r2, y, ldy1, ldy2};
    const int cus = lim.compute_units > 0 ? lim.compute_units : 256;
    const int lpr = K <= 64 ? 8 : K <= 128 ? 16 : K <= 256 ? 32 : 64;
    const int64_t rows_per_wg = (AM_THREADS / 64) * (64 / lpr);
    int64_t gx = ceil_div(N, rows_per_wg);
    const int64_t cap = ceil_div((int64_t)cus * 8, ne02);               // about eight workgroups per CU over all KV heads
    if (gx > cap) gx = cap;
    const dim3 grid((unsigned)gx, (unsigned)ne02);
    switch (lpr) {
        case 8:  hipLaunchKernelGGL(mul_mat_f16_batched_kernel<8>, grid, dim3(AM_THREADS), 0, st, a); break;
        case 16: hipLaunchKernelGGL(mul_mat_f16_batched_kernel<16>, grid, dim3(AM_THREADS), 0, st, a); break;
        case 32: hipLaunchKernelGGL(mul_mat_f16_batched_kernel<32>, grid, dim3(AM_THREADS), 0, st, a); break;
        default: hipLaunchKernelGGL(mul_mat_f16_batched_kernel<64>, grid, dim3(AM_THREADS), 0, st, a); break;
    }
    return hipGetLastError();
}

}  // namespace chip
