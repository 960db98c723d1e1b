// Internal launch interface between the C-ABI layer (capi.hip) and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <atomic>

namespace chip {

struct DeviceLimits {
    int compute_units;
    int max_lds_per_block;   // bytes one workgroup may allocate (static + dynamic)
};

// A kernel that needs more than 48 KB of dynamic LDS must have its limit raised first.  That is a host call per
// launch otherwise, so each launch site raises the limit to the device maximum once per device and remembers it.
struct LdsGrant { std::atomic<unsigned> devices{0}; };
template <typename F> inline hipError_t grant_dynamic_lds(F kfn, size_t need, const DeviceLimits &lim, LdsGrant &g) {
    if (need <= 48 * 1024) return hipSuccess;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const unsigned bit = 1u << (dev & 31);
    if (g.devices.load(std::memory_order_acquire) & bit) return hipSuccess;
    e = hipFuncSetAttribute((const void *)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, lim.max_lds_per_block);
    if (e == hipSuccess) g.devices.fetch_or(bit, std::memory_order_release);
    return e;
}

// quantize.hip
hipError_t launch_quantize(int act_type, bool split, const float *x, int64_t ldx, int64_t n, int64_t K, void *y,
                           size_t y_stride, hipStream_t st);
hipError_t launch_split_to_blocks(int act_type, const void *ws, size_t ws_stride, int64_t n, int64_t K, void *y,
                                  size_t y_stride, hipStream_t st);

// gemv.hip: y[t][r] for t < n (n <= 8 per launch), activations in the split workspace layout.
// Returns hipErrorInvalidValue if the shape does not fit the kernel (caller splits the token range).
int        gemv_max_tokens(int wtype, int64_t K, const DeviceLimits &lim);   // tokens one launch can take (<= 8)
hipError_t launch_gemv(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                       int n, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st);
// One launch for quantize + GEMV (n in {1,2,4}, small n*K): x is fp32; ws receives the split-layout quantized
// activations from workgroup 0.
bool       gemv_fused_applicable(int wtype, int64_t K, int n, const DeviceLimits &lim);
hipError_t launch_gemv_fused(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx,
                             int n, void *ws, size_t ws_stride, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st);
hipError_t launch_block_isums(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *aq, int64_t n,
                              int32_t *isum, int32_t *imin, hipStream_t st);

// gemv_mfma.hip: the same product for up to 16 tokens per launch with the integer sums on the matrix cores.
// mmv_max_tokens returns 16, 8 or 0 (shape or type not covered: use launch_gemv).
int        mmv_max_tokens(int wtype, int64_t K, int64_t N, const DeviceLimits &lim);
hipError_t launch_mmv(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                      int n, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st);

// gemm_q4_0.hip: int8-MFMA prefill GEMM over Q4_0 weights, activations in the split Q8_0 workspace layout.
bool       gemm_q4_0_supported(int64_t K, int64_t N, int64_t n);
hipError_t launch_gemm_q4_0(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                            int64_t n, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st);

// gemm_kquant.hip: int8-MFMA prefill GEMM over Q4_K / Q5_K / Q6_K weights, activations in the split Q8_K workspace
// layout; the integer sub-block scales ride in the MFMA operand.
bool       gemm_kq_supported(int wtype, int64_t K, int64_t N, int64_t n);
hipError_t launch_gemm_kq(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                          int64_t n, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st);

}  // namespace chip
