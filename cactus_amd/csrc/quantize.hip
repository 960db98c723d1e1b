// On-the-fly activation quantizers for gfx950: fp32 rows -> Q8_0 / Q8_K, bit-identical to the reference's
// x86 AVX2 build (reference ggml-cpu/ggml-cpu-quants.c:802-885 for Q8_0; ggml-quants.c:2473-2510 for Q8_K).
//
// Both kernels are pure streaming work: each lane loads one float4 (16-byte coalesced), block maxima are
// combined with DPP moves inside the 8 (Q8_0) or 64 (Q8_K) lanes that share a block, and each lane stores
// one packed dword of four int8 quants.  Output goes either to the reference block layout (SPLIT = false,
// the public quantize entry points) or to the workspace planes of act_layout.h (SPLIT = true).
//
// Exactness notes: fp32 division is the correctly rounded one, denormals are kept, and the file is compiled
// with -ffp-contract=off so `iscale*x + 12582912.f` rounds twice, as the C source of the reference says.
#include "dev_common.h"
#include "act_layout.h"
#include "quant_dev.h"
#include "kernels.h"

namespace chip {

// FMT: 0 = workspace planes, 1 = block_q8_0 records, 2 = block_q8_1 records (reference ggml-common.h:216-227)
template <int FMT>
__global__ __launch_bounds__(256) void quantize_q8_0_kernel(const float *__restrict__ x, int64_t ldx, int64_t K,
                                                           uint8_t *__restrict__ y, size_t y_stride) {
    const int64_t t = blockIdx.y;
    const int64_t e0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;      // first of this lane's 4 elements
    const bool live = e0 < K;                                             // K % 32 == 0: whole 8-lane groups agree
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live) v = *reinterpret_cast<const float4 *>(x + t * ldx + e0);
    const Q8_0Lane q = quantize_q8_0_lane(v);
    const int64_t blk = e0 / 32;
    const int sub = threadIdx.x & 7;
    if (!live) return;
    if (FMT == 0) {
        uint8_t *base = y + t * y_stride;
        *reinterpret_cast<uint32_t *>(base + e0) = q.packed;
        if (sub == 0) {
            reinterpret_cast<float *>(base + q8_0_off_d(K))[blk] = h2f(q.dh);
            reinterpret_cast<int32_t *>(base + q8_0_off_sum(K))[blk] = q.sum;
            reinterpret_cast<float *>(base + q8_0_off_s(K))[blk] = h2f(q.sh);
        }
    } else if (FMT == 1) {
        uint8_t *b = y + t * y_stride + blk * BYTES_Q8_0;
        *reinterpret_cast<u32_a2 *>(b + 2 + 4 * sub) = q.packed;
        if (sub == 0) *reinterpret_cast<unsigned short *>(b) = q.dh;
    } else {
        uint8_t *b = y + t * y_stride + blk * BYTES_Q8_1;
        *reinterpret_cast<uint32_t *>(b + 4 + 4 * sub) = q.packed;
        if (sub == 0) *reinterpret_cast<uint32_t *>(b) = (uint32_t)q.dh | ((uint32_t)q.sh << 16);
    }
}

template <bool SPLIT>
__global__ __launch_bounds__(256) void quantize_q8_K_kernel(const float *__restrict__ x, int64_t ldx, int64_t K,
                                                           uint8_t *__restrict__ y, size_t y_stride) {
    const int64_t t = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const int64_t sb = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);       // one wave per 256-value super-block
    if (sb * QK_K >= K) return;                                           // whole wave leaves together
    const float4 v = *reinterpret_cast<const float4 *>(x + t * ldx + sb * QK_K + lane * 4);
    const Q8_KLane q = quantize_q8_K_lane(v);
    if (SPLIT) {
        uint8_t *base = y + t * y_stride;
        *reinterpret_cast<uint32_t *>(base + sb * QK_K + lane * 4) = q.packed;
        if (lane == 0) reinterpret_cast<float *>(base + q8_K_off_d(K))[sb] = q.d;
        if ((lane & 3) == 0) reinterpret_cast<int16_t *>(base + q8_K_off_bsums(K))[sb * 16 + (lane >> 2)] = (int16_t)q.bsum;
    } else {
        uint8_t *b = y + t * y_stride + sb * BYTES_Q8_K;
        *reinterpret_cast<uint32_t *>(b + 4 + lane * 4) = q.packed;
        if (lane == 0) *reinterpret_cast<float *>(b) = q.d;
        if ((lane & 3) == 0) *reinterpret_cast<int16_t *>(b + 260 + 2 * (lane >> 2)) = (int16_t)q.bsum;
    }
}

// fp32 -> fp16 rows, round to nearest even (reference lm_ggml_cpu_fp32_to_fp16, ggml-cpu/ggml-cpu.c:3161-3190): the
// activation format of F16 weights.  The workspace layout and the reference layout are the same K halves.
__global__ __launch_bounds__(256) void convert_f16_kernel(const float *__restrict__ x, int64_t ldx, int64_t K,
                                                        uint8_t *__restrict__ y, size_t y_stride) {
    const int64_t t = blockIdx.y;
    const int64_t e0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (e0 >= K) return;
    const float4 v = *reinterpret_cast<const float4 *>(x + t * ldx + e0);
    u32x2 h;
    h.x = (uint32_t)f2h_rne(v.x) | ((uint32_t)f2h_rne(v.y) << 16);
    h.y = (uint32_t)f2h_rne(v.z) | ((uint32_t)f2h_rne(v.w) << 16);
    *reinterpret_cast<u32x2 *>(y + t * y_stride + 2 * e0) = h;
}

// Inverse of the split layout: rebuild reference blocks from workspace planes (verification only).
__global__ void split_to_blocks_q8_0_kernel(const uint8_t *__restrict__ ws, size_t ws_stride, int64_t K,
                                            uint8_t *__restrict__ y, size_t y_stride) {
    const int64_t t = blockIdx.y;
    const int64_t blk = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (blk >= K / 32) return;
    const uint8_t *base = ws + t * ws_stride;
    uint8_t *b = y + t * y_stride + blk * BYTES_Q8_0;
    *reinterpret_cast<unsigned short *>(b) = f2h_rne(reinterpret_cast<const float *>(base + q8_0_off_d(K))[blk]);
    for (int i = 0; i < 32; i++) b[2 + i] = base[blk * 32 + i];
}
__global__ void split_to_blocks_q8_1_kernel(const uint8_t *__restrict__ ws, size_t ws_stride, int64_t K,
                                            uint8_t *__restrict__ y, size_t y_stride) {
    const int64_t t = blockIdx.y;
    const int64_t blk = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (blk >= K / 32) return;
    const uint8_t *base = ws + t * ws_stride;
    uint8_t *b = y + t * y_stride + blk * BYTES_Q8_1;
    reinterpret_cast<unsigned short *>(b)[0] = f2h_rne(reinterpret_cast<const float *>(base + q8_0_off_d(K))[blk]);
    reinterpret_cast<unsigned short *>(b)[1] = f2h_rne(reinterpret_cast<const float *>(base + q8_0_off_s(K))[blk]);
    for (int i = 0; i < 32; i++) b[4 + i] = base[blk * 32 + i];
}
__global__ void split_to_blocks_q8_K_kernel(const uint8_t *__restrict__ ws, size_t ws_stride, int64_t K,
                                            uint8_t *__restrict__ y, size_t y_stride) {
    const int64_t t = blockIdx.y;
    const int64_t sb = blockIdx.x;
    const int i = threadIdx.x;                                             // 256 threads
    const uint8_t *base = ws + t * ws_stride;
    uint8_t *b = y + t * y_stride + sb * BYTES_Q8_K;
    b[4 + i] = base[sb * QK_K + i];
    if (i == 0) *reinterpret_cast<float *>(b) = reinterpret_cast<const float *>(base + q8_K_off_d(K))[sb];
    if (i < 16)
        *reinterpret_cast<int16_t *>(b + 260 + 2 * i) = reinterpret_cast<const int16_t *>(base + q8_K_off_bsums(K))[sb * 16 + i];
}

hipError_t launch_quantize(int act_type, bool split, const float *x, int64_t ldx, int64_t n, int64_t K, void *y,
                           size_t y_stride, hipStream_t st) {
    if (n <= 0 || K <= 0) return hipSuccess;
    dim3 grid((unsigned)ceil_div(K, 1024), (unsigned)n);
    if (act_type == T_F16) {
        hipLaunchKernelGGL(convert_f16_kernel, grid, dim3(256), 0, st, x, ldx, K, (uint8_t *)y, y_stride);
    } else if (act_type == T_Q8_0 || act_type == T_Q8_1) {
        // Q8_1 shares the Q8_0 workspace planes (which carry its s); only the block records differ
        if (split)                  hipLaunchKernelGGL(quantize_q8_0_kernel<0>, grid, dim3(256), 0, st, x, ldx, K, (uint8_t *)y, y_stride);
        else if (act_type == T_Q8_0) hipLaunchKernelGGL(quantize_q8_0_kernel<1>, grid, dim3(256), 0, st, x, ldx, K, (uint8_t *)y, y_stride);
        else                        hipLaunchKernelGGL(quantize_q8_0_kernel<2>, grid, dim3(256), 0, st, x, ldx, K, (uint8_t *)y, y_stride);
    } else {
        if (split) hipLaunchKernelGGL(quantize_q8_K_kernel<true>, grid, dim3(256), 0, st, x, ldx, K, (uint8_t *)y, y_stride);
        else       hipLaunchKernelGGL(quantize_q8_K_kernel<false>, grid, dim3(256), 0, st, x, ldx, K, (uint8_t *)y, y_stride);
    }
    return hipGetLastError();
}

hipError_t launch_split_to_blocks(int act_type, const void *ws, size_t ws_stride, int64_t n, int64_t K, void *y,
                                  size_t y_stride, hipStream_t st) {
    if (n <= 0 || K <= 0) return hipSuccess;
    if (act_type == T_F16)
        return hipMemcpy2DAsync(y, y_stride, ws, ws_stride, 2 * (size_t)K, (size_t)n, hipMemcpyDeviceToDevice, st);
    if (act_type == T_Q8_0 || act_type == T_Q8_1) {
        dim3 grid((unsigned)ceil_div(K / 32, 256), (unsigned)n);
        if (act_type == T_Q8_0)
            hipLaunchKernelGGL(split_to_blocks_q8_0_kernel, grid, dim3(256), 0, st, (const uint8_t *)ws, ws_stride, K,
                               (uint8_t *)y, y_stride);
        else
            hipLaunchKernelGGL(split_to_blocks_q8_1_kernel, grid, dim3(256), 0, st, (const uint8_t *)ws, ws_stride, K,
                               (uint8_t *)y, y_stride);
    } else {
        dim3 grid((unsigned)(K / 256), (unsigned)n);
        hipLaunchKernelGGL(split_to_blocks_q8_K_kernel, grid, dim3(256), 0, st, (const uint8_t *)ws, ws_stride, K,
                           (uint8_t *)y, y_stride);
    }
    return hipGetLastError();
}

}  // namespace chip
