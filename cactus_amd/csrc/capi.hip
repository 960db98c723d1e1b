// C-ABI of libcactus_hip.so (declared in include/cactus_hip.h): argument checking, device plumbing and the
// dispatch from LM_GGML_OP_MUL_MAT shapes to the gfx950 kernels.  No CPU fallback exists anywhere in this
// library: an unsupported request returns an error code, it is never computed on the host.
#include "../../include/cactus_hip.h"
#include "act_layout.h"
#include "dev_common.h"
#include <math.h>
#include "kernels.h"

#include <atomic>
#include <cstdio>
#include <cstring>
#include <mutex>

using namespace chip;

constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];      // chip_mul_mat_noalloc's workspace

namespace {

// From this many tokens on the matrix-core GEMV beats the dot-product GEMV (measured on Q8_0 4096x11008).
constexpr int MMV_MIN_TOKENS = 5;

}  // namespace
namespace chip { std::atomic<int> g_force_mmv_q6k{0}; }

namespace {

std::mutex g_mu;
bool g_limits_ready[64] = {};
DeviceLimits g_limits[64];

// Device memory of chip_mul_mat_noalloc: quantized activation rows and, behind them, the partial outputs of a GEMM whose
// K is split.  Every GPU holds its own copy of the array for the life of the process; host code never uses the array's
// name as an address, only the per-device pointer hipGetSymbolAddress returned (g_scratch_ptr).
void *g_scratch_ptr[64] = {};

// Address of the current device's scratch array, looked up once per device.
int scratch_address(void **out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= 64) return CHIP_EINVAL;
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return CHIP_EINVAL;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return CHIP_OK;
}

int hip_rc(hipError_t e) { return e == hipSuccess ? CHIP_OK : (int)e; }

// Limits of the current device, read once per device.
int current_limits(DeviceLimits &out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= 64) return CHIP_EINVAL;
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_limits_ready[dev]) {
        hipDeviceProp_t p;
        e = hipGetDeviceProperties(&p, dev);
        if (e != hipSuccess) return (int)e;
        int optin = 0;
        if (hipDeviceGetAttribute(&optin, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) optin = 0;
        size_t lds = p.sharedMemPerBlock;
        if ((size_t)optin > lds) lds = (size_t)optin;
        if (p.maxSharedMemoryPerMultiProcessor > lds) lds = p.maxSharedMemoryPerMultiProcessor;
        if (lds > 160 * 1024) lds = 160 * 1024;
        g_limits[dev].compute_units = p.multiProcessorCount;
        g_limits[dev].max_lds_per_block = (int)lds;
        g_limits_ready[dev] = true;
    }
    out = g_limits[dev];
    return CHIP_OK;
}

bool is_weight_type(int t) {
    return t == T_Q4_0 || t == T_Q8_0 || t == T_Q4_K || t == T_Q6_K || t == T_Q5_0 || t == T_Q5_K || t == T_IQ4_NL ||
           t == T_Q4_1 || t == T_Q5_1 || t == T_F16 || t == T_Q3_K || t == T_Q2_K || t == T_IQ4_XS;
}
bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// Q4_0 / Q8_0 / Q4_K rows of K % 256 == 0 elements are multiples of 16 bytes and the kernels load them with
// 4- and 16-byte aligned vectors.  Q6_K rows are multiples of 210 bytes: only 2-byte alignment can be asked for,
// and that kernel loads with 2-byte aligned vectors throughout.
// The types of 32-value blocks also come with rows of K % 64 == 0 elements (hidden sizes such as 576, 896, 960): such
// rows are multiples of 4 bytes only, and only the kernels that load with 4-byte aligned vectors take them (the
// dot-product GEMV; the GEMM, whose staging reads single blocks, when K % 128 == 0).
bool is_block32_type(int t) { return t == T_Q4_0 || t == T_Q8_0 || t == T_Q5_0 || t == T_IQ4_NL || t == T_Q4_1 || t == T_Q5_1; }
bool weights_aligned(int type, const void *W, size_t nb01, int64_t K = 256) {
    // (Q3_K: 110-byte super-blocks, as Q6_K's 210; Q2_K: 84 bytes; IQ4_XS: 136 bytes, loaded as an 8-byte and 4-byte aligned pieces)
    // (Q6_K rows in planes: 210 * K / 256 bytes with K % 2048 == 0, a multiple of 16)
    const size_t a = (type == T_Q6_K || type == T_Q3_K) ? 2 : type == T_Q2_K ? 4 : type == T_IQ4_XS ? 8 : (is_block32_type(type) && K % 256 != 0) ? 4 : 16;
    return ((uintptr_t)W % a) == 0 && (nb01 % a) == 0;
}

// Q8_1 activations live in the Q8_0 workspace planes (which carry block_q8_1.s as well)
size_t act_stride(int act_type, int64_t K) {
    if (act_type == T_F16) return f16_stride(K);
    return (act_type == T_Q8_0 || act_type == T_Q8_1) ? q8_0_stride(K) : q8_K_stride(K);
}

}  // namespace

extern "C" {

int chip_device_count(void) {
    int n = 0;
    return hipGetDeviceCount(&n) == hipSuccess ? n : 0;
}

int chip_init(int device) {
    int n = chip_device_count();
    if (n <= 0) return CHIP_ENODEVICE;
    if (device < 0 || device >= n) return CHIP_EINVAL;
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return (int)e;
    hipDeviceProp_t p;
    e = hipGetDeviceProperties(&p, device);
    if (e != hipSuccess) return (int)e;
    if (std::strncmp(p.gcnArchName, "gfx950", 6) != 0) return CHIP_ENODEVICE;   // the kernels are built for gfx950 only
    DeviceLimits lim;
    if (int rc = current_limits(lim); rc) return rc;
    void *sp = nullptr;
    return scratch_address(&sp);                                        // chip_mul_mat_noalloc's memory on this device
}

int chip_get_device_info(chip_device_info *out) {
    if (!out) return CHIP_EINVAL;
    std::memset(out, 0, sizeof(*out));
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    constexpr int MAX_DEVICES = 64;
    if (dev < 0 || dev >= MAX_DEVICES) return CHIP_EINVAL;
    // the properties are read once per device (the query takes milliseconds); the memory figures every time
    static chip_device_info fixed[MAX_DEVICES];
    static bool have[MAX_DEVICES];
    static std::mutex mu;
    {
        std::lock_guard<std::mutex> lk(mu);
        if (!have[dev]) {
            hipDeviceProp_t p;
            e = hipGetDeviceProperties(&p, dev);
            if (e != hipSuccess) return (int)e;
            DeviceLimits lim;
            int rc = current_limits(lim);
            if (rc) return rc;
            chip_device_info &f = fixed[dev];
            std::memset(&f, 0, sizeof(f));
            f.device = dev;
            f.compute_units = p.multiProcessorCount;
            f.wavefront_size = p.warpSize;
            f.max_lds_per_block = lim.max_lds_per_block;
            f.clock_khz = p.clockRate;
            f.xcd_count = 0;
            std::snprintf(f.name, sizeof(f.name), "%s", p.name);
            std::snprintf(f.arch, sizeof(f.arch), "%s", p.gcnArchName);
            have[dev] = true;
        }
        *out = fixed[dev];
    }
    size_t fr = 0, tot = 0;
    if (hipMemGetInfo(&fr, &tot) == hipSuccess) { out->hbm_free = fr; out->hbm_total = tot; }
    return CHIP_OK;
}

const char *chip_error_string(int code) {
    switch (code) {
        case CHIP_OK: return "ok";
        case CHIP_EINVAL: return "invalid argument (null, negative, or misaligned)";
        case CHIP_EUNSUPPORTED: return "unsupported type or shape";
        case CHIP_ENOMEM: return "workspace too small";
        case CHIP_ENODEVICE: return "no gfx950 device";
        default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
    }
}

int chip_malloc(void **dptr, size_t bytes) {
    if (!dptr) return CHIP_EINVAL;
    *dptr = nullptr;
    if (bytes == 0) return CHIP_OK;
    const hipError_t e = hipMalloc(dptr, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();                     // or the next kernel launch's own check would report this failure again
        *dptr = nullptr;
    }
    return hip_rc(e);
}
int chip_free(void *dptr) { return dptr ? hip_rc(hipFree(dptr)) : CHIP_OK; }

int chip_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return CHIP_OK;
    if (!dst || !src) return CHIP_EINVAL;
    if (!stream) return hip_rc(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return hip_rc(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
}
int chip_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return CHIP_OK;
    if (!dst || !src) return CHIP_EINVAL;
    if (!stream) return hip_rc(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return hip_rc(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
}
int chip_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return CHIP_OK;
    if (!dst || !src) return CHIP_EINVAL;
    return hip_rc(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
}
int chip_memset(void *dst, int value, size_t bytes, void *stream) {
    if (bytes == 0) return CHIP_OK;
    if (!dst) return CHIP_EINVAL;
    return hip_rc(hipMemsetAsync(dst, value, bytes, (hipStream_t)stream));
}
int chip_stream_create(void **stream) {
    if (!stream) return CHIP_EINVAL;
    hipStream_t s = nullptr;
    hipError_t e = hipStreamCreate(&s);                                  // default priority
    *stream = (void *)s;
    return hip_rc(e);
}
int chip_stream_destroy(void *stream) { return stream ? hip_rc(hipStreamDestroy((hipStream_t)stream)) : CHIP_OK; }
int chip_stream_synchronize(void *stream) { return hip_rc(hipStreamSynchronize((hipStream_t)stream)); }

int chip_host_malloc(void **ptr, size_t bytes) {
    if (!ptr) return CHIP_EINVAL;
    *ptr = nullptr;
    return hip_rc(hipHostMalloc(ptr, bytes ? bytes : 16, hipHostMallocDefault));        // pinned, allocated (never registered)
}
int chip_host_free(void *ptr) { return ptr ? hip_rc(hipHostFree(ptr)) : CHIP_OK; }
int chip_event_create(void **event) {
    if (!event) return CHIP_EINVAL;
    hipEvent_t e = nullptr;
    hipError_t rc = hipEventCreateWithFlags(&e, hipEventDisableTiming);
    *event = (void *)e;
    return hip_rc(rc);
}
int chip_event_destroy(void *event) { return event ? hip_rc(hipEventDestroy((hipEvent_t)event)) : CHIP_OK; }
int chip_event_record(void *event, void *stream) {
    return event ? hip_rc(hipEventRecord((hipEvent_t)event, (hipStream_t)stream)) : CHIP_EINVAL;
}
int chip_event_synchronize(void *event) { return event ? hip_rc(hipEventSynchronize((hipEvent_t)event)) : CHIP_EINVAL; }
int chip_stream_wait_event(void *stream, void *event) {
    return event ? hip_rc(hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)event, 0)) : CHIP_EINVAL;
}

int chip_block_elems(int type) {
    switch (type) {
        case T_F32: case T_F16: return 1;
        case T_Q4_0: case T_Q8_0: case T_Q5_0: case T_IQ4_NL: case T_Q4_1: case T_Q5_1: case T_Q8_1: return 32;
        case T_Q4_K: case T_Q6_K: case T_Q8_K: case T_Q5_K: case T_Q3_K: case T_Q2_K: case T_IQ4_XS: case T_Q6_K_P: return 256;
        default: return 0;
    }
}
size_t chip_block_bytes(int type) {
    switch (type) {
        case T_F32: return 4;
        case T_F16: return 2;
        case T_Q4_0: return BYTES_Q4_0;
        case T_Q8_0: return BYTES_Q8_0;
        case T_Q4_K: return BYTES_Q4_K;
        case T_Q6_K: case T_Q6_K_P: return BYTES_Q6_K;
        case T_Q8_K: return BYTES_Q8_K;
        case T_Q5_0: return BYTES_Q5_0;
        case T_Q5_K: return BYTES_Q5_K;
        case T_IQ4_NL: return BYTES_IQ4_NL;
        case T_Q4_1: return BYTES_Q4_1;
        case T_Q5_1: return BYTES_Q5_1;
        case T_Q8_1: return BYTES_Q8_1;
        case T_Q3_K: return BYTES_Q3_K;
        case T_Q2_K: return BYTES_Q2_K;
        case T_IQ4_XS: return BYTES_IQ4_XS;
        default: return 0;
    }
}
size_t chip_row_size(int type, int64_t k) {
    const int be = chip_block_elems(type);
    return (be && k > 0) ? (size_t)(k / be) * chip_block_bytes(type) : 0;
}
int chip_vec_dot_type(int type) {
    switch (type) {
        case T_Q4_0: case T_Q8_0: case T_Q5_0: case T_IQ4_NL: return T_Q8_0;
        case T_Q4_K: case T_Q6_K: case T_Q5_K: case T_Q3_K: case T_Q2_K: case T_IQ4_XS: case T_Q6_K_P: return T_Q8_K;
        case T_Q4_1: case T_Q5_1: return T_Q8_1;
        case T_F16: return T_F16;
        default: return -1;
    }
}
int chip_mul_mat_supported(int type, int64_t K) {
    // Q6_K rows in planes: every field of a row starts at a multiple of 16 bytes when the row has a multiple of 8 super-blocks
    if (type == T_Q6_K_P) return K > 0 && K % 2048 == 0 && K <= (1 << 20);
    return is_weight_type(type) && K > 0 && K % (is_block32_type(type) ? 64 : 256) == 0 && K <= (1 << 20);
}

int chip_repack_q6_K(const void *src, size_t nb01_src, void *dst, size_t nb01_dst, int64_t K, int64_t N, int to_planes, void *stream) {
    if (N < 0) return CHIP_EINVAL;
    if (!chip_mul_mat_supported(T_Q6_K_P, K)) return CHIP_EUNSUPPORTED;
    if (N == 0) return CHIP_OK;
    const size_t row = chip_row_size(T_Q6_K, K);
    if (!src || !dst || nb01_src < row || nb01_dst < row || (nb01_src % 2) != 0 || (nb01_dst % 2) != 0) return CHIP_EINVAL;
    if (((uintptr_t)src & 1) != 0 || ((uintptr_t)dst & 1) != 0) return CHIP_EINVAL;
    // the same rows (in place), or rows that do not overlap at all
    const uint8_t *s0 = (const uint8_t *)src, *d0 = (const uint8_t *)dst;
    const size_t s_span = (size_t)(N - 1) * nb01_src + row, d_span = (size_t)(N - 1) * nb01_dst + row;
    if (!(s0 == d0 && nb01_src == nb01_dst) && s0 < d0 + d_span && d0 < s0 + s_span) return CHIP_EINVAL;
    DeviceLimits lim;
    if (int rc = current_limits(lim); rc) return rc;
    if (row > (size_t)lim.max_lds_per_block) return CHIP_EUNSUPPORTED;
    return hip_rc(launch_repack_q6_K(src, nb01_src, dst, nb01_dst, K, N, to_planes != 0, lim.max_lds_per_block, (hipStream_t)stream));
}

static int quantize_public(int act_type, const float *x, int64_t ldx, int64_t n, int64_t k, void *y, void *stream) {
    if (n < 0 || k < 0) return CHIP_EINVAL;
    if (n == 0 || k == 0) return CHIP_OK;
    if (!x || !y || ldx < k) return CHIP_EINVAL;
    if (k % chip_block_elems(act_type) != 0) return CHIP_EUNSUPPORTED;
    if (!aligned16(x) || (ldx % 4) != 0) return CHIP_EINVAL;             // float4 loads
    if (((uintptr_t)y & 3) != 0) return CHIP_EINVAL;
    if (n > 65535) return CHIP_EUNSUPPORTED;
    return hip_rc(launch_quantize(act_type, false, x, ldx, n, k, y, chip_row_size(act_type, k), (hipStream_t)stream));
}
int chip_quantize_q8_0(const float *x, int64_t ldx, int64_t n, int64_t k, void *y, void *stream) {
    return quantize_public(T_Q8_0, x, ldx, n, k, y, stream);
}
int chip_quantize_q8_K(const float *x, int64_t ldx, int64_t n, int64_t k, void *y, void *stream) {
    return quantize_public(T_Q8_K, x, ldx, n, k, y, stream);
}
int chip_quantize_q8_1(const float *x, int64_t ldx, int64_t n, int64_t k, void *y, void *stream) {
    return quantize_public(T_Q8_1, x, ldx, n, k, y, stream);
}
int chip_convert_f32_to_f16(const float *x, int64_t ldx, int64_t n, int64_t k, void *y, void *stream) {
    if (k % 4 != 0) return CHIP_EUNSUPPORTED;
    return quantize_public(T_F16, x, ldx, n, k, y, stream);
}

size_t chip_mul_mat_workspace_size(int type, int64_t K, int64_t n) {
    if (!chip_mul_mat_supported(type, K) || n <= 0) return 0;
    return act_stride(chip_vec_dot_type(type), K) * (size_t)n;
}

int chip_mul_mat_prepare(int type, int64_t K, const float *x, int64_t ldx, int64_t n, void *workspace,
                         size_t workspace_bytes, void *stream) {
    if (n < 0) return CHIP_EINVAL;
    if (!chip_mul_mat_supported(type, K)) return CHIP_EUNSUPPORTED;
    if (n == 0) return CHIP_OK;
    if (!x || !workspace || ldx < K) return CHIP_EINVAL;
    if (!aligned16(x) || (ldx % 4) != 0 || !aligned16(workspace)) return CHIP_EINVAL;
    if (workspace_bytes < chip_mul_mat_workspace_size(type, K, n)) return CHIP_ENOMEM;
    const int at = chip_vec_dot_type(type);
    const size_t stride = act_stride(at, K);
    // grid.y carries the token index: split very long prompts
    for (int64_t t0 = 0; t0 < n; t0 += 32768) {
        const int64_t nt = (n - t0 < 32768) ? n - t0 : 32768;
        hipError_t e = launch_quantize(at, true, x + t0 * ldx, ldx, nt, K, (uint8_t *)workspace + t0 * stride, stride,
                                       (hipStream_t)stream);
        if (e != hipSuccess) return (int)e;
    }
    return CHIP_OK;
}

// bytes of the activation rows in the workspace, rounded so that what follows them is 256-byte aligned
static size_t act_rows_bytes(int type, int64_t K, int64_t n) { return (chip_mul_mat_workspace_size(type, K, n) + 255) & ~(size_t)255; }
static int split_slices(int type, int64_t K, int64_t N, int64_t n, int cus) {
    const int a = gemm_blk32_slices(type, K, N, n, cus), b = gemm_kq_slices(type, K, N, n, cus);
    return a > b ? a : b;
}
size_t chip_mul_mat_workspace_size_n(int type, int64_t K, int64_t N, int64_t n) {
    const size_t act = chip_mul_mat_workspace_size(type, K, n);
    if (act == 0 || N <= 0) return act;
    DeviceLimits lim;
    const int cus = current_limits(lim) == CHIP_OK ? lim.compute_units : 256;
    const int slices = split_slices(type, K, N, n, cus);
    return slices > 1 ? act_rows_bytes(type, K, n) + (size_t)slices * (size_t)n * (size_t)N * sizeof(float) : act;
}

// Fewest tokens from which the matrix-core GEMV is taken for this matrix.
// (4-bit weights on a small matrix: the dot-product GEMV is still ahead up to 6 or 7 tokens)
// (and Q4_K rows so wide that the kernel runs with six waves: from 7 tokens)
static int mmv_min_tokens(int type, int64_t K, int64_t N) {
    const int mmv_forced = (int)tune("CHIP_MMV_MIN", 0);
    return mmv_forced > 0 ? mmv_forced
           : ((type == T_Q4_K || type == T_Q5_K || type == T_Q4_0) && N * K < (32LL << 20)) ? (type == T_Q4_0 ? 8 : 7)
           : (type == T_Q4_K && K > 13312) ? 7 : MMV_MIN_TOKENS;
}
// Two Q4_K / Q5_K matrices of one shape on the same rows at 5..8 tokens (ffn_gate and ffn_up): true when each alone would
// take one launch of the matrix-core GEMV whatever the workspace size - they then run as one launch in which every
// workgroup, after its tiles of the first matrix, takes the same tiles of the second (the activation image is built once;
// every tile is computed as in a launch of its own: the same bits).
static bool mmv_pair_applicable(int type, int64_t K, int64_t N, int64_t n, const DeviceLimits &lim) {
    if (n < 5 || n > 8 || !(type == T_Q4_K || type == T_Q5_K) || tune("CHIP_MMV_PAIR", 1) == 0) return false;
    if (gemm_kq_supported(type, K, N, n, false) || gemm_kq_supported(type, K, N, n, true)) return false;
    return n >= mmv_min_tokens(type, K, N) && n <= mmv_q4k_max_tokens(type, K, N, lim);
}
static int mul_mat_run(int type, const void *W, size_t nb01, int64_t K, int64_t N, int64_t n, const void *workspace,
                       size_t workspace_bytes, float *y, int64_t ldy, void *stream);
int chip_mul_mat_run(int type, const void *W, size_t nb01, int64_t K, int64_t N, int64_t n, const void *workspace,
                     float *y, int64_t ldy, void *stream) {
    return mul_mat_run(type, W, nb01, K, N, n, workspace, 0, y, ldy, stream);
}
int chip_mul_mat_run_ws(int type, const void *W, size_t nb01, int64_t K, int64_t N, int64_t n, void *workspace, size_t workspace_bytes,
                        float *y, int64_t ldy, void *stream) {
    if (workspace_bytes < chip_mul_mat_workspace_size(type, K, n)) return CHIP_ENOMEM;
    return mul_mat_run(type, W, nb01, K, N, n, workspace, workspace_bytes, y, ldy, stream);
}
// workspace_bytes: what the caller says lies behind `workspace` (0 = the activation rows only, no room for split-K partials)
static int mul_mat_run(int type, const void *W, size_t nb01, int64_t K, int64_t N, int64_t n, const void *workspace,
                       size_t workspace_bytes, float *y, int64_t ldy, void *stream) {
    if (N < 0 || n < 0) return CHIP_EINVAL;
    if (!chip_mul_mat_supported(type, K)) return CHIP_EUNSUPPORTED;
    if (N == 0 || n == 0) return CHIP_OK;
    if (!W || !workspace || !y || ldy < N) return CHIP_EINVAL;
    if (!weights_aligned(type, W, nb01, K) || nb01 < chip_row_size(type, K) || !aligned16(workspace)) return CHIP_EINVAL;
    if (((uintptr_t)y & 3) != 0) return CHIP_EINVAL;
    DeviceLimits lim;
    int rc = current_limits(lim);
    if (rc) return rc;
    const size_t stride = act_stride(chip_vec_dot_type(type), K);
    hipStream_t st = (hipStream_t)stream;

    SplitK split{nullptr, 0};
    if (const size_t act = act_rows_bytes(type, K, n); workspace_bytes > act)
        split = SplitK{reinterpret_cast<float *>((uint8_t *)const_cast<void *>(workspace) + act), workspace_bytes - act};
    // K is split only with room for every slice's partial output behind the activation rows
    const int want_slices = split.part ? split_slices(type, K, N, n, lim.compute_units) : 1;
    const bool can_split = want_slices > 1 && split.bytes >= (size_t)want_slices * (size_t)n * (size_t)N * sizeof(float);
    if (!can_split) split = SplitK{nullptr, 0};
    if (gemm_blk32_supported(type, K, N, n, can_split))
        return hip_rc(launch_gemm_blk32(type, W, nb01, K, N, workspace, stride, n, y, ldy, lim, st, nullptr, 1, split));
    if (type == T_F16 && gemm_f16_supported(K, N, n))
        return hip_rc(launch_gemm_f16(W, nb01, K, N, workspace, stride, n, y, ldy, lim, st));
    if (gemm_kq_supported(type, K, N, n, can_split))
        return hip_rc(launch_gemm_kq(type, W, nb01, K, N, workspace, stride, n, y, ldy, lim, st, nullptr, 1, split));

    // 5 tokens or more: integer sums on the matrix cores, up to 16 tokens per pass over the weights
    const int mmv_min = mmv_min_tokens(type, K, N);
    const int mgroup = (n >= mmv_min) ? mmv_max_tokens(type, K, N, lim) : 0;
    if (mgroup > 0) {
        for (int64_t t0 = 0; t0 < n; t0 += mgroup) {
            const int nt = (int)((n - t0 < mgroup) ? n - t0 : mgroup);
            hipError_t e = (nt >= mmv_min || nt > gemv_max_tokens(type, K, lim))
                ? launch_mmv(type, W, nb01, K, N, (const uint8_t *)workspace + t0 * stride, stride, nt, y + t0 * ldy, ldy, lim, st)
                : launch_gemv(type, W, nb01, K, N, (const uint8_t *)workspace + t0 * stride, stride, nt, y + t0 * ldy, ldy, lim, st);
            if (e != hipSuccess) return (int)e;
        }
        return CHIP_OK;
    }
    const int group = gemv_max_tokens(type, K, lim);
    if (group < 1) return CHIP_EUNSUPPORTED;
    for (int64_t t0 = 0; t0 < n; t0 += group) {
        const int nt = (int)((n - t0 < group) ? n - t0 : group);
        hipError_t e = launch_gemv(type, W, nb01, K, N, (const uint8_t *)workspace + t0 * stride, stride, nt, y + t0 * ldy,
                                   ldy, lim, st);
        if (e != hipSuccess) return (int)e;
    }
    return CHIP_OK;
}

int chip_mul_mat(int type, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, int64_t n,
                 float *y, int64_t ldy, void *workspace, size_t workspace_bytes, void *stream) {
    const int mmv_forced = (int)tune("CHIP_MMV_MIN", 0);
    if (n >= 1 && n <= 4 && !(mmv_forced > 0 && n >= mmv_forced) && N > 0 && chip_mul_mat_supported(type, K)) {
        // decode: one launch that quantizes in the GEMV prologue (argument checks as in prepare + run)
        DeviceLimits lim;
        int rc0 = current_limits(lim);
        if (rc0) return rc0;
            if (gemv_fused_applicable(type, K, (int)n, lim)) {
            if (!x || !workspace || ldx < K || !W || !y || ldy < N) return CHIP_EINVAL;
            if (!aligned16(x) || (ldx % 4) != 0 || !aligned16(workspace) || (((uintptr_t)y) & 3) != 0) return CHIP_EINVAL;
            if (!weights_aligned(type, W, nb01, K) || nb01 < chip_row_size(type, K)) return CHIP_EINVAL;
            if (workspace_bytes < chip_mul_mat_workspace_size(type, K, n)) return CHIP_ENOMEM;
            return hip_rc(launch_gemv_fused(type, W, nb01, K, N, x, ldx, (int)n, workspace,
                                            act_stride(chip_vec_dot_type(type), K), y, ldy, lim, (hipStream_t)stream));
        }
    }
    int rc = chip_mul_mat_prepare(type, K, x, ldx, n, workspace, workspace_bytes, stream);
    if (rc) return rc;
    return mul_mat_run(type, W, nb01, K, N, n, workspace, workspace_bytes, y, ldy, stream);
}

// chip_mul_mat on the library's own static device array instead of a caller's workspace: no allocation of any kind.
size_t chip_mul_mat_noalloc_max_workspace(void) { return NOALLOC_SCRATCH_BYTES; }
int chip_mul_mat_noalloc(int type, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, int64_t n,
                         float *y, int64_t ldy, void *stream) {
    if (N < 0 || n < 0) return CHIP_EINVAL;
    if (!chip_mul_mat_supported(type, K)) return CHIP_EUNSUPPORTED;
    if (N == 0 || n == 0) return CHIP_OK;
    if (chip_mul_mat_workspace_size(type, K, n) > NOALLOC_SCRATCH_BYTES) return CHIP_ENOMEM;   // the activation rows must fit
    void *sp = nullptr;
    if (int rc = scratch_address(&sp); rc) return rc;
    // With room behind the activation rows a GEMM may split K, exactly as chip_mul_mat does with a workspace of this size.
    return chip_mul_mat(type, W, nb01, K, N, x, ldx, n, y, ldy, sp, NOALLOC_SCRATCH_BYTES, stream);
}

// Two matmuls on one activation (ffn_gate / ffn_up).  Up to 4 tokens: one launch of the prologue-quantizing GEMV over
// both matrices; more tokens: one quantizer, then each matrix on its own path.
int chip_mul_mat_pair(int type, const void *W1, const void *W2, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx,
                      int64_t n, float *y1, float *y2, int64_t ldy, void *workspace, size_t workspace_bytes, void *stream) {
    if (N < 0 || n < 0) return CHIP_EINVAL;
    if (!chip_mul_mat_supported(type, K)) return CHIP_EUNSUPPORTED;
    if (N == 0 || n == 0) return CHIP_OK;
    if (!W1 || !W2 || !x || !y1 || !y2 || !workspace || ldx < K || ldy < N) return CHIP_EINVAL;
    if (!weights_aligned(type, W1, nb01, K) || !weights_aligned(type, W2, nb01, K) || nb01 < chip_row_size(type, K)) return CHIP_EINVAL;
    if (!aligned16(x) || (ldx % 4) != 0 || !aligned16(workspace) || ((((uintptr_t)y1) | ((uintptr_t)y2)) & 3) != 0) return CHIP_EINVAL;
    if (workspace_bytes < chip_mul_mat_workspace_size(type, K, n)) return CHIP_ENOMEM;
    DeviceLimits lim;
    if (int rc = current_limits(lim); rc) return rc;
    if (n <= 4 && 2 * N <= 0x7fffffff && gemv_fused_applicable(type, K, (int)n, lim))
        return hip_rc(launch_gemv_fused_pair(type, W1, W2, nb01, K, N, x, ldx, (int)n, workspace,
                                             act_stride(chip_vec_dot_type(type), K), y1, y2, ldy, lim, (hipStream_t)stream));
    if (int rc = chip_mul_mat_prepare(type, K, x, ldx, n, workspace, workspace_bytes, stream); rc) return rc;
    if (mmv_pair_applicable(type, K, N, n, lim))
        return hip_rc(launch_mmv_q4k(type, W1, nb01, K, N, workspace, act_stride(chip_vec_dot_type(type), K), (int)n, y1, ldy, lim,
                                     (hipStream_t)stream, W2, y2));
    if (int rc = mul_mat_run(type, W1, nb01, K, N, n, workspace, workspace_bytes, y1, ldy, stream); rc) return rc;
    return mul_mat_run(type, W2, nb01, K, N, n, workspace, workspace_bytes, y2, ldy, stream);
}

// MUL(SILU(MUL_MAT(W1, x)), MUL_MAT(W2, x)) in one launch, where chip_mul_mat_pair runs its one-launch GEMV
int chip_mul_mat_pair_silu_mul_supported(int type, int64_t K, int64_t N, int64_t n) {
    if (!chip_mul_mat_supported(type, K) || N <= 0 || n < 1 || n > 4 || 2 * N > 0x7fffffff) return 0;
    if (N % 8 != 0) return 0;                                               // as chip_silu: the reference's row tail uses the C library's expf
    DeviceLimits lim;
    if (current_limits(lim) != CHIP_OK) return 0;
    return gemv_fused_applicable(type, K, (int)n, lim) ? 1 : 0;
}
static int norm_before_checked(const chip_norm_before *norm, int type, int64_t K, int64_t n, const DeviceLimits &lim) {
    if (!norm || !norm->w || !aligned16(norm->w)) return CHIP_EINVAL;
    if (norm->y && (!aligned16(norm->y) || norm->ldy < K || (norm->ldy % 4) != 0)) return CHIP_EINVAL;
    return gemv_norm_prologue_applicable(type, K, (int)n, lim) ? CHIP_OK : CHIP_EUNSUPPORTED;
}
int chip_norm_before_supported(int type, int64_t K, int64_t n) {
    if (!chip_mul_mat_supported(type, K) || n < 1 || n > 4) return 0;
    DeviceLimits lim;
    if (current_limits(lim) != CHIP_OK) return 0;
    return gemv_norm_prologue_applicable(type, K, (int)n, lim) ? 1 : 0;
}
static int pair_silu_mul(int type, const void *W1, const void *W2, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx,
                         int64_t n, const chip_norm_before *norm, float *y, int64_t ldy, void *workspace, size_t workspace_bytes,
                         void *stream);
int chip_mul_mat_pair_silu_mul(int type, const void *W1, const void *W2, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx,
                               int64_t n, float *y, int64_t ldy, void *workspace, size_t workspace_bytes, void *stream) {
    return pair_silu_mul(type, W1, W2, nb01, K, N, x, ldx, n, nullptr, y, ldy, workspace, workspace_bytes, stream);
}
int chip_mul_mat_pair_silu_mul_norm(int type, const void *W1, const void *W2, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx,
                                    int64_t n, const chip_norm_before *norm, float *y, int64_t ldy, void *workspace,
                                    size_t workspace_bytes, void *stream) {
    if (!norm) return CHIP_EINVAL;
    return pair_silu_mul(type, W1, W2, nb01, K, N, x, ldx, n, norm, y, ldy, workspace, workspace_bytes, stream);
}
static int pair_silu_mul(int type, const void *W1, const void *W2, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx,
                         int64_t n, const chip_norm_before *norm, float *y, int64_t ldy, void *workspace, size_t workspace_bytes,
                         void *stream) {
    if (N < 0 || n < 0) return CHIP_EINVAL;
    if (!chip_mul_mat_supported(type, K)) return CHIP_EUNSUPPORTED;
    if (N == 0 || n == 0) return CHIP_OK;
    if (!chip_mul_mat_pair_silu_mul_supported(type, K, N, n)) return CHIP_EUNSUPPORTED;
    if (!W1 || !W2 || !x || !y || !workspace || ldx < K || ldy < N) return CHIP_EINVAL;
    if (!weights_aligned(type, W1, nb01, K) || !weights_aligned(type, W2, nb01, K) || nb01 < chip_row_size(type, K)) return CHIP_EINVAL;
    if (!aligned16(x) || (ldx % 4) != 0 || !aligned16(workspace) || (((uintptr_t)y) & 3) != 0) return CHIP_EINVAL;
    if (workspace_bytes < chip_mul_mat_workspace_size(type, K, n)) return CHIP_ENOMEM;
    DeviceLimits lim;
    if (int rc = current_limits(lim); rc) return rc;
    if (norm)
        if (int rc = norm_before_checked(norm, type, K, n, lim); rc) return rc;
    return hip_rc(launch_gemv_fused_pair_silu_mul(type, W1, W2, nb01, K, N, x, ldx, (int)n, workspace,
                                                  act_stride(chip_vec_dot_type(type), K), y, ldy, lim, (hipStream_t)stream,
                                                  norm ? norm->w : nullptr, norm ? norm->eps : 0.f, norm ? norm->y : nullptr,
                                                  norm ? norm->ldy : 0));
}
int chip_mul_mat_add_supported(int type, int64_t K, int64_t N, int64_t n) {
    if (!chip_mul_mat_supported(type, K) || N <= 0 || n < 1 || n > 4) return 0;
    DeviceLimits lim;
    if (current_limits(lim) != CHIP_OK) return 0;
    return gemv_fused_applicable(type, K, (int)n, lim) ? 1 : 0;
}
int chip_mul_mat_add(int type, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, int64_t n,
                     const float *addend, int64_t ld_add, float *y, int64_t ldy, void *workspace, size_t workspace_bytes, void *stream) {
    if (N < 0 || n < 0) return CHIP_EINVAL;
    if (!chip_mul_mat_supported(type, K)) return CHIP_EUNSUPPORTED;
    if (N == 0 || n == 0) return CHIP_OK;
    if (!chip_mul_mat_add_supported(type, K, N, n)) return CHIP_EUNSUPPORTED;
    if (!x || !workspace || ldx < K || !W || !y || ldy < N || !addend || ld_add < N) return CHIP_EINVAL;
    if (!aligned16(x) || (ldx % 4) != 0 || !aligned16(workspace) || ((((uintptr_t)y) | ((uintptr_t)addend)) & 3) != 0) return CHIP_EINVAL;
    if (!weights_aligned(type, W, nb01, K) || nb01 < chip_row_size(type, K)) return CHIP_EINVAL;
    if (workspace_bytes < chip_mul_mat_workspace_size(type, K, n)) return CHIP_ENOMEM;
    DeviceLimits lim;
    if (int rc = current_limits(lim); rc) return rc;
    return hip_rc(launch_gemv_fused_add(type, W, nb01, K, N, x, ldx, (int)n, workspace, act_stride(chip_vec_dot_type(type), K), addend,
                                        ld_add, y, ldy, lim, (hipStream_t)stream));
}

static int rope_dims_checked(int64_t ne0, int64_t ne1, int64_t ne2, int n_dims, int mode);

// Several matmuls on one activation (wq / wk / wv).  Up to 4 tokens, members of one family: one launch of the
// prologue-quantizing GEMV over all members; otherwise one quantizer and each member on its usual path.
// what chip_mul_mat_group and chip_mul_mat_group_run share: x == nullptr says the workspace already holds the rows
static int mul_mat_group(const chip_mat *mats, int count, int64_t K, const float *x, int64_t ldx, int64_t n, void *workspace,
                         size_t workspace_bytes, void *stream, const chip_rope_after *ropes = nullptr,
                         const chip_norm_before *norm = nullptr) {
    if (count < 0 || n < 0) return CHIP_EINVAL;
    if (count == 0 || n == 0) return CHIP_OK;
    if (!mats || count > CHIP_GROUP_MAX) return CHIP_EINVAL;
    const int at = chip_vec_dot_type(mats[0].type);
    size_t need = 0;
    for (int i = 0; i < count; i++) {
        const chip_mat &m = mats[i];
        if (!chip_mul_mat_supported(m.type, K)) return CHIP_EUNSUPPORTED;
        // one quantized activation serves every member: Q8_1 members read the Q8_0 planes, which carry block_q8_1.s
        const int a = chip_vec_dot_type(m.type);
        if (!(a == at || ((a == T_Q8_0 || a == T_Q8_1) && (at == T_Q8_0 || at == T_Q8_1)))) return CHIP_EUNSUPPORTED;
        if (m.N < 0) return CHIP_EINVAL;
        if (m.N == 0) continue;
        const bool roped = ropes && ropes[i].table;                    // the member's own result is then not stored
        if (!m.W || (!roped && (!m.y || m.ldy < m.N || (((uintptr_t)m.y) & 3) != 0))) return CHIP_EINVAL;
        if (!weights_aligned(m.type, m.W, m.nb01, K) || m.nb01 < chip_row_size(m.type, K)) return CHIP_EINVAL;
        if (m.y_f16_t && (m.ld16 < n || (((uintptr_t)m.y_f16_t) & 1) != 0)) return CHIP_EINVAL;
        if (roped) {
            const chip_rope_after &r = ropes[i];
            if (int rc = rope_dims_checked(r.head_dim, m.N / (r.head_dim > 0 ? r.head_dim : 1), n, r.n_dims, r.mode); rc != CHIP_OK) return rc;
            if (r.head_dim <= 0 || (r.head_dim & 1) || m.N % r.head_dim != 0 || r.head_dim > 0x7fffffff) return CHIP_EUNSUPPORTED;
            if ((!r.y && !r.y_f16) || m.y_f16_t || (((uintptr_t)r.table) & 3) != 0) return CHIP_EINVAL;
            if (r.y && (r.ldy < m.N || (((uintptr_t)r.y) & 3) != 0)) return CHIP_EINVAL;
            if (r.y_f16 && (r.ld16 < m.N || (((uintptr_t)r.y_f16) & 1) != 0)) return CHIP_EINVAL;
        }
        const size_t w = chip_mul_mat_workspace_size(m.type, K, n);
        if (w > need) need = w;
    }
    const bool prepared = x == nullptr;
    if (!workspace || !aligned16(workspace)) return CHIP_EINVAL;
    if (!prepared && (ldx < K || !aligned16(x) || (ldx % 4) != 0)) return CHIP_EINVAL;
    if (workspace_bytes < need) return CHIP_ENOMEM;
    DeviceLimits lim;
    if (int rc = current_limits(lim); rc) return rc;
    GroupMat gm[GROUP_MAX];
    int live = 0;
    bool any_rope = false;
    for (int i = 0; i < count; i++)
        if (mats[i].N > 0) {
            gm[live] = GroupMat{mats[i].type, mats[i].W, mats[i].nb01, mats[i].N, mats[i].y, mats[i].ldy, mats[i].y_f16_t, mats[i].ld16};
            if (ropes && ropes[i].table) {
                const chip_rope_after &r = ropes[i];
                gm[live].y = r.y;
                gm[live].ldy = r.y ? r.ldy : 0;
                gm[live].rope = RopeEpilogue{r.table, (int)r.head_dim, r.n_dims, (r.mode & 2) != 0, r.y != nullptr, r.y_f16, r.y_f16 ? r.ld16 : 0};
                any_rope = true;
            }
            live++;
        }
    if (live == 0) return CHIP_OK;
    if (any_rope) {                                                      // only the one-launch form has the epilogue
        if (prepared || n > 4 || !gemv_group_applicable(gm, live, K, (int)n, lim, false) || gemv_group_family(gm[0].wtype) == 2)
            return CHIP_EUNSUPPORTED;
        GroupNorm gn{nullptr, 0.f, nullptr, 0};
        if (norm) {
            for (int i = 0; i < live; i++)
                if (int rc = norm_before_checked(norm, gm[i].wtype, K, n, lim); rc) return rc;
            gn = GroupNorm{norm->w, norm->eps, norm->y, norm->ldy};
        }
        return hip_rc(launch_gemv_group(gm, live, K, x, ldx, (int)n, workspace, act_stride(at, K), lim, (hipStream_t)stream, false, &gn));
    }
    if (norm) return CHIP_EUNSUPPORTED;
    const size_t stride = act_stride(at, K);
    hipStream_t st = (hipStream_t)stream;
    // Up to 4 tokens.  One member, or two of one type, shape and row stride, take the single-matrix kernel (it keeps more
    // waves per SIMD than the group kernel, whose register count is that of its most demanding member type): a pair runs
    // as one matrix of twice the rows, a member with a transposed fp16 copy as chip_mul_mat_store_t does.
    if (n <= 4 && gemv_group_applicable(gm, live, K, (int)n, lim, prepared)) {
        const GroupMat &a = gm[0], &b = gm[live - 1];
        if (live == 1 && a.t16)
            return hip_rc(prepared ? launch_gemv_store_t(a.wtype, a.W, a.nb01, K, a.N, workspace, stride, (int)n, a.y, a.ldy, a.t16, a.t16_ld, lim, st)
                                   : launch_gemv_fused_store_t(a.wtype, a.W, a.nb01, K, a.N, x, ldx, (int)n, workspace, stride, a.y, a.ldy, a.t16, a.t16_ld, lim, st));
        if (live == 1)
            return hip_rc(prepared ? launch_gemv(a.wtype, a.W, a.nb01, K, a.N, workspace, stride, (int)n, a.y, a.ldy, lim, st)
                                   : launch_gemv_fused(a.wtype, a.W, a.nb01, K, a.N, x, ldx, (int)n, workspace, stride, a.y, a.ldy, lim, st));
        if (live == 2 && a.wtype == b.wtype && a.N == b.N && a.nb01 == b.nb01 && a.ldy == b.ldy && !a.t16 && !b.t16 && 2 * a.N <= 0x7fffffff)
            return hip_rc(prepared ? launch_gemv_pair(a.wtype, a.W, b.W, a.nb01, K, a.N, workspace, stride, (int)n, a.y, b.y, a.ldy, lim, st)
                                   : launch_gemv_fused_pair(a.wtype, a.W, b.W, a.nb01, K, a.N, x, ldx, (int)n, workspace, stride, a.y, b.y, a.ldy, lim, st));
        return hip_rc(launch_gemv_group(gm, live, K, x, ldx, (int)n, workspace, stride, lim, st, prepared));
    }
    // more tokens, or members the one-launch form does not take: quantize once, then every member as chip_mul_mat_run would
    if (!prepared)
        if (int rc = chip_mul_mat_prepare(mats[0].type, K, x, ldx, n, workspace, workspace_bytes, stream); rc) return rc;
    if (n == 8 && live >= 2 && gemv_group_applicable(gm, live, K, 8, lim, true)) {
        // 8 tokens, several small matrices: one launch of the dot-product GEMV over all members when together they stream
        // no more than 24 MB (larger ones are faster through a matrix-core GEMV each)
        double bytes = 0;
        for (int i = 0; i < live; i++) bytes += (double)gm[i].N * (double)gm[i].nb01;
        if (bytes <= tune("CHIP_GROUP8_MAX_MB", 24) * 1048576.0)
            return hip_rc(launch_gemv_group(gm, live, K, nullptr, 0, 8, workspace, stride, lim, st, true));
    }
    if (live == 2) {                                                   // ffn_gate and ffn_up at 5..8 tokens
        const GroupMat &a = gm[0], &b = gm[1];
        const bool twins = a.wtype == b.wtype && a.N == b.N && a.nb01 == b.nb01 && a.ldy == b.ldy && !a.t16 && !b.t16;
        if (twins && mmv_pair_applicable(a.wtype, K, a.N, n, lim))
            return hip_rc(launch_mmv_q4k(a.wtype, a.W, a.nb01, K, a.N, workspace, stride, (int)n, a.y, a.ldy, lim, st, b.W, b.y));
    }
    for (int i = 0; i < live; i++) {
        const GroupMat &m = gm[i];
        if (int rc = mul_mat_run(m.wtype, m.W, m.nb01, K, m.N, n, workspace, workspace_bytes, m.y, m.ldy, stream); rc) return rc;
        if (m.t16) {
            const int64_t ne[4] = {n, m.N, 1, 1};
            const int64_t nbs[4] = {m.ldy * 4, 4, m.N * 4, m.N * 4}, nbd[4] = {2, m.t16_ld * 2, m.N * m.t16_ld * 2, m.N * m.t16_ld * 2};
            if (hipError_t e = launch_cpy(m.y, 0, ne, nbs, m.t16, 1, ne, nbd, (hipStream_t)stream); e != hipSuccess) return (int)e;
        }
    }
    return CHIP_OK;
}
int chip_mul_mat_group(const chip_mat *mats, int count, int64_t K, const float *x, int64_t ldx, int64_t n, void *workspace,
                       size_t workspace_bytes, void *stream) {
    if (count > 0 && n > 0 && !x) return CHIP_EINVAL;
    return mul_mat_group(mats, count, K, x, ldx, n, workspace, workspace_bytes, stream);
}
int chip_mul_mat_group_rope(const chip_mat *mats, const chip_rope_after *ropes, int count, int64_t K, const float *x, int64_t ldx,
                            int64_t n, void *workspace, size_t workspace_bytes, void *stream) {
    if (!ropes || (count > 0 && n > 0 && !x)) return CHIP_EINVAL;
    return mul_mat_group(mats, count, K, x, ldx, n, workspace, workspace_bytes, stream, ropes);
}
int chip_mul_mat_group_rope_norm(const chip_mat *mats, const chip_rope_after *ropes, const chip_norm_before *norm, int count, int64_t K,
                                 const float *x, int64_t ldx, int64_t n, void *workspace, size_t workspace_bytes, void *stream) {
    if (!ropes || !norm || (count > 0 && n > 0 && !x)) return CHIP_EINVAL;
    return mul_mat_group(mats, count, K, x, ldx, n, workspace, workspace_bytes, stream, ropes, norm);
}
int chip_mul_mat_group_run(const chip_mat *mats, int count, int64_t K, int64_t n, void *workspace, size_t workspace_bytes, void *stream) {
    return mul_mat_group(mats, count, K, nullptr, 0, n, workspace, workspace_bytes, stream);
}

// A matmul whose result is also stored transposed as fp16 (the V projection and the store into the transposed F16 V cache).
int chip_mul_mat_store_t(int type, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, int64_t n,
                         float *y, int64_t ldy, uint16_t *y16t, int64_t ld16, void *workspace, size_t workspace_bytes, void *stream) {
    if (!y16t || ld16 < n || (((uintptr_t)y16t) & 1) != 0) return CHIP_EINVAL;
    if (n >= 1 && n <= 4 && N > 0 && chip_mul_mat_supported(type, K)) {
        DeviceLimits lim;
        if (int rc = current_limits(lim); rc) return rc;
            if (gemv_fused_applicable(type, K, (int)n, lim)) {
            if (!x || !workspace || ldx < K || !W || !y || ldy < N) return CHIP_EINVAL;
            if (!aligned16(x) || (ldx % 4) != 0 || !aligned16(workspace) || (((uintptr_t)y) & 3) != 0) return CHIP_EINVAL;
            if (!weights_aligned(type, W, nb01, K) || nb01 < chip_row_size(type, K)) return CHIP_EINVAL;
            if (workspace_bytes < chip_mul_mat_workspace_size(type, K, n)) return CHIP_ENOMEM;
            return hip_rc(launch_gemv_fused_store_t(type, W, nb01, K, N, x, ldx, (int)n, workspace, act_stride(chip_vec_dot_type(type), K),
                                                    y, ldy, y16t, ld16, lim, (hipStream_t)stream));
        }
    }
    if (int rc = chip_mul_mat(type, W, nb01, K, N, x, ldx, n, y, ldy, workspace, workspace_bytes, stream); rc) return rc;
    if (N == 0 || n == 0) return CHIP_OK;
    // y [n tokens][N] read as a matrix of n values per row r (stride 1 token = ldy floats), written as halves with rows ld16 apart
    const int64_t ne[4] = {n, N, 1, 1};
    const int64_t nbs[4] = {ldy * 4, 4, N * 4, N * 4}, nbd[4] = {2, ld16 * 2, N * ld16 * 2, N * ld16 * 2};
    return hip_rc(launch_cpy(y, 0, ne, nbs, y16t, 1, ne, nbd, (hipStream_t)stream));
}

// MUL_MAT_ID workspace: the quantized activation rows, then the expert offsets and the pair list of the grouped path
static size_t moe_rows_bytes(int type, int64_t K, int64_t rows) { return align16(act_stride(chip_vec_dot_type(type), K) * (size_t)rows); }
size_t chip_mul_mat_id_workspace_size(int type, int64_t K, int64_t n_as, int64_t n_used, int64_t n_tokens, int64_t ne11) {
    if (!chip_mul_mat_supported(type, K) || n_as <= 0 || n_used <= 0 || n_tokens <= 0 || ne11 <= 0) return 0;
    const size_t pairs = (size_t)(n_tokens * n_used);
    return moe_rows_bytes(type, K, n_tokens * ne11) + align16(4 * (size_t)(n_as + 1)) + align16(4 * pairs) +
           align16(4 * (pairs / 64 + (size_t)n_as + 2));                // pair list, then the tile list (tiles of >= 64 pairs)
}

// from this many (token, slot) pairs on, the pairs are grouped by expert and run through the GEMM of the weight type
// (one-token GEMVs re-read an expert's matrix for every pair)
constexpr int64_t MOE_GEMM_MIN_PAIRS = 64;

int chip_mul_mat_id(int type, const void *W, size_t nb01, size_t nb02, int64_t K, int64_t N, int64_t n_as, const float *x,
                    int64_t ldx, int64_t ne11, const int32_t *ids, int64_t ids_stride, int64_t n_used, int64_t n_tokens,
                    float *y, int64_t ldy, void *workspace, size_t workspace_bytes, void *stream) {
    if (N < 0 || n_as < 0 || n_used < 0 || n_tokens < 0 || ne11 < 0) return CHIP_EINVAL;
    if (!chip_mul_mat_supported(type, K) || K % 256 != 0 || type == T_Q6_K_P) return CHIP_EUNSUPPORTED;
    if (N == 0 || n_used == 0 || n_tokens == 0) return CHIP_OK;
    if (n_as == 0 || !(ne11 == 1 || ne11 == n_used)) return CHIP_EINVAL;
    if (!W || !x || !ids || !y || !workspace || ldx < K || ldy < N || ids_stride < n_used) return CHIP_EINVAL;
    if (!weights_aligned(type, W, nb01, K) || !weights_aligned(type, W, nb02, K) || nb01 < chip_row_size(type, K) ||
        nb02 < (size_t)N * nb01)
        return CHIP_EINVAL;
    if (!aligned16(x) || (ldx % 4) != 0 || !aligned16(workspace) || (((uintptr_t)y) & 3) != 0 || (((uintptr_t)ids) & 3) != 0)
        return CHIP_EINVAL;
    const int64_t rows = n_tokens * ne11, pairs = n_tokens * n_used;
    if (workspace_bytes < chip_mul_mat_id_workspace_size(type, K, n_as, n_used, n_tokens, ne11)) return CHIP_ENOMEM;
    DeviceLimits lim;
    int rc = current_limits(lim);
    if (rc) return rc;
    const size_t stride = act_stride(chip_vec_dot_type(type), K);
    hipStream_t st = (hipStream_t)stream;

    const bool kq = type == T_Q4_K || type == T_Q5_K || type == T_Q6_K;
    // (the 2- and 3-bit K-quants have no GEMM of their own: every pair takes the GEMV)
    const bool have_gemm = (type == T_Q3_K || type == T_Q2_K || type == T_IQ4_XS) ? false : type == T_F16 ? K % 64 == 0 : (kq ? true : K % 128 == 0);
    if (pairs >= MOE_GEMM_MIN_PAIRS && have_gemm && moe_group_supported(n_as, pairs)) {
        rc = chip_mul_mat_prepare(type, K, x, ldx, rows, workspace, workspace_bytes, stream);
        if (rc) return rc;
        int32_t *offsets = reinterpret_cast<int32_t *>((uint8_t *)workspace + moe_rows_bytes(type, K, rows));
        int32_t *perm = offsets + align16(4 * (size_t)(n_as + 1)) / 4;
        int32_t *tiles = perm + align16(4 * (size_t)pairs) / 4;
        const int bn = type == T_F16 ? gemm_f16_moe_tile_tokens() : (kq ? gemm_kq_moe_tile_tokens() : gemm_blk32_moe_tile_tokens());
        if (hipError_t e = launch_moe_group(ids, ids_stride, n_used, pairs, n_as, bn, offsets, perm, tiles, st); e != hipSuccess)
            return (int)e;
        const RowGather rg{perm, offsets, tiles, (int32_t)n_used, (int32_t)ne11, nb02};
        // the grid provides a slot for every token tile the list can have; slots past its length exit at once
        const int64_t slots = pairs / bn + n_as;
        if (type == T_F16) return hip_rc(launch_gemm_f16(W, nb01, K, N, workspace, stride, pairs, y, ldy, lim, st, &rg, slots));
        if (kq) return hip_rc(launch_gemm_kq(type, W, nb01, K, N, workspace, stride, pairs, y, ldy, lim, st, &rg, slots));
        return hip_rc(launch_gemm_blk32(type, W, nb01, K, N, workspace, stride, pairs, y, ldy, lim, st, &rg, slots));
    }

    // few pairs: one-token GEMVs, quantizing in the prologue (one launch) while that repeats little work
    const bool fused = pairs <= 16 && gemv_fused_applicable(type, K, 1, lim);
    if (!fused) {
        rc = chip_mul_mat_prepare(type, K, x, ldx, rows, workspace, workspace_bytes, stream);
        if (rc) return rc;
    }
    return hip_rc(launch_gemv_id(type, fused, W, nb01, nb02, n_as, K, N, x, ldx, ne11, ids, ids_stride, n_used, n_tokens,
                                 workspace, stride, y, ldy, lim, st));
}

// ---- element-wise ops next to the matmuls ----
static bool rows_ok(const float *p, int64_t ld, int64_t ne0) { return p && ld >= ne0 && (((uintptr_t)p) & 3) == 0; }
int chip_rms_norm(const float *x, int64_t ldx, int64_t n, int64_t ne0, float eps, float *y, int64_t ldy, void *stream) {
    if (n < 0 || ne0 < 0 || !(eps >= 0.0f)) return CHIP_EINVAL;
    if (n == 0 || ne0 == 0) return CHIP_OK;
    if (!rows_ok(x, ldx, ne0) || !rows_ok(y, ldy, ne0)) return CHIP_EINVAL;
    return hip_rc(launch_rms_norm(x, ldx, n, ne0, eps, y, ldy, (hipStream_t)stream));
}
static int binary_checked(bool mul, const float *a, int64_t lda, const float *b, int64_t ldb, int64_t n_b, int64_t n, int64_t ne0,
                          float *y, int64_t ldy, void *stream) {
    if (n < 0 || ne0 < 0) return CHIP_EINVAL;
    if (n == 0 || ne0 == 0) return CHIP_OK;
    if (!(n_b == 1 || n_b == n)) return CHIP_EUNSUPPORTED;               // src1: the shape of src0, or one row for all
    if (!rows_ok(a, lda, ne0) || !rows_ok(y, ldy, ne0) || !b || (((uintptr_t)b) & 3) != 0 || (n_b == n && n > 1 && ldb < ne0))
        return CHIP_EINVAL;
    const int64_t step = (n_b == 1) ? 0 : ldb;
    return hip_rc(mul ? launch_mul(a, lda, b, step, ne0, n, y, ldy, (hipStream_t)stream)
                      : launch_add(a, lda, b, step, ne0, n, y, ldy, (hipStream_t)stream));
}
int chip_add(const float *a, int64_t lda, const float *b, int64_t ldb, int64_t n_b, int64_t n, int64_t ne0, float *y, int64_t ldy,
             void *stream) { return binary_checked(false, a, lda, b, ldb, n_b, n, ne0, y, ldy, stream); }
int chip_mul(const float *a, int64_t lda, const float *b, int64_t ldb, int64_t n_b, int64_t n, int64_t ne0, float *y, int64_t ldy,
             void *stream) { return binary_checked(true, a, lda, b, ldb, n_b, n, ne0, y, ldy, stream); }
int chip_rms_norm_mul(const float *x, int64_t ldx, int64_t n, int64_t ne0, float eps, const float *w, float *y_norm, int64_t ld_norm,
                      float *y, int64_t ldy, void *stream) {
    if (n < 0 || ne0 < 0 || !(eps >= 0.0f)) return CHIP_EINVAL;
    if (n == 0 || ne0 == 0) return CHIP_OK;
    if (!rows_ok(x, ldx, ne0) || !rows_ok(y, ldy, ne0) || !w || (((uintptr_t)w) & 3) != 0 || n > 0x7fffffff) return CHIP_EINVAL;
    if (y_norm && !rows_ok(y_norm, ld_norm, ne0)) return CHIP_EINVAL;
    return hip_rc(launch_rms_norm_mul(x, ldx, n, ne0, eps, w, y_norm, ld_norm, y, ldy, (hipStream_t)stream));
}
int chip_add_rms_norm_mul(const float *a, int64_t lda, const float *b, int64_t ldb, float *sum, int64_t ld_sum, int64_t n, int64_t ne0,
                          float eps, const float *w, float *y, int64_t ldy, void *stream) {
    if (n < 0 || ne0 < 0 || !(eps >= 0.0f)) return CHIP_EINVAL;
    if (n == 0 || ne0 == 0) return CHIP_OK;
    if (!rows_ok(a, lda, ne0) || !rows_ok(b, ldb, ne0) || !rows_ok(sum, ld_sum, ne0) || !rows_ok(y, ldy, ne0) || n > 0x7fffffff ||
        (w && (((uintptr_t)w) & 3) != 0) || (const float *)y == sum)
        return CHIP_EINVAL;
    return hip_rc(launch_add_rms_norm_mul(a, lda, b, ldb, sum, ld_sum, n, ne0, eps, w, nullptr, 0, y, ldy, (hipStream_t)stream));
}
int chip_scale(const float *x, int64_t ldx, int64_t n, int64_t ne0, float scale, float *y, int64_t ldy, void *stream) {
    if (n < 0 || ne0 < 0) return CHIP_EINVAL;
    if (n == 0 || ne0 == 0) return CHIP_OK;
    if (!rows_ok(x, ldx, ne0) || !rows_ok(y, ldy, ne0)) return CHIP_EINVAL;
    return hip_rc(launch_scale(x, ldx, ne0, n, scale, y, ldy, (hipStream_t)stream));
}
// fp16 <-> fp32 on the host, round to nearest even (the conversions lm_ggml_cpu_init uses for its tables)
static float half_bits_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 31u, man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) bits = sign;
        else {                                                           // subnormal half: man * 2^-24
            float f = (float)man * 5.9604644775390625e-8f;
            std::memcpy(&bits, &f, 4);
            bits |= sign;
        }
    } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
    else bits = sign | ((exp + 112u) << 23) | (man << 13);
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}
static uint16_t float_to_half_bits(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u, ax = x & 0x7fffffffu;
    if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((ax & 0x7fffffu) >> 13));   // NaN: quiet, payload kept (as vcvtps2ph does)
    if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);                          // rounds to 65536 or more, or inf
    if (ax < 0x33000001u) return (uint16_t)sign;                                       // at most half the smallest subnormal
    const int e = (int)(ax >> 23) - 127;
    uint32_t man = (ax & 0x7fffffu) | 0x800000u;
    if (e < -14) {                                                                     // subnormal half: units of 2^-24
        const int shift = -e - 1;                                                      // 14 .. 24
        const uint32_t q = man >> shift, rem = man & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
        return (uint16_t)(sign | (q + ((rem > halfway || (rem == halfway && (q & 1u))) ? 1u : 0u)));
    }
    uint32_t h = ((uint32_t)(e + 15) << 10) | ((man >> 13) & 0x3ffu);
    const uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;                            // a carry moves into the exponent as it should
    return (uint16_t)(sign | h);
}
int chip_gelu_table(uint16_t *table) {
    if (!table) return CHIP_EINVAL;
    const float coef_a = 0.044715f, sqrt_2_over_pi = 0.79788456080286535587989211986876f;
    for (uint32_t i = 0; i < 65536u; i++) {
        const float x = half_bits_to_float((uint16_t)i);
        table[i] = float_to_half_bits(0.5f * x * (1.0f + tanhf(sqrt_2_over_pi * x * (1.0f + coef_a * x * x))));
    }
    return CHIP_OK;
}
int chip_gelu(const float *x, int64_t ldx, int64_t n, int64_t ne0, const uint16_t *table, float *y, int64_t ldy, void *stream) {
    if (n < 0 || ne0 < 0) return CHIP_EINVAL;
    if (n == 0 || ne0 == 0) return CHIP_OK;
    if (!rows_ok(x, ldx, ne0) || !rows_ok(y, ldy, ne0) || !table || (((uintptr_t)table) & 1) != 0) return CHIP_EINVAL;
    return hip_rc(launch_gelu(x, ldx, ne0, n, table, y, ldy, (hipStream_t)stream));
}
// The norm in front of a group of matmuls, leaving the quantized rows in their workspace (what chip_mul_mat_prepare would
// write from y afterwards).
int chip_rms_norm_quantized(const float *a, int64_t lda, const float *b, int64_t ldb, float *sum, int64_t ld_sum, int64_t n,
                            int64_t ne0, float eps, const float *w, float *y, int64_t ldy, int wtype, void *workspace,
                            size_t workspace_bytes, void *stream) {
    if (n < 0 || ne0 < 0 || !(eps >= 0.0f)) return CHIP_EINVAL;
    if (!chip_mul_mat_supported(wtype, ne0)) return CHIP_EUNSUPPORTED;
    const int at = chip_vec_dot_type(wtype);
    const int kind = (at == T_Q8_0 || at == T_Q8_1) ? 1 : (at == T_Q8_K ? 2 : 0);
    if (kind == 0) return CHIP_EUNSUPPORTED;                               // F16 weights: plain fp16 rows, not done here
    if (n == 0 || ne0 == 0) return CHIP_OK;
    if (!rows_ok(a, lda, ne0) || !rows_ok(y, ldy, ne0) || (w && (((uintptr_t)w) & 3) != 0) || n > 0x7fffffff) return CHIP_EINVAL;
    if (b && (!rows_ok(b, ldb, ne0) || !rows_ok(sum, ld_sum, ne0) || (const float *)y == sum)) return CHIP_EINVAL;
    if (!workspace || !aligned16(workspace)) return CHIP_EINVAL;
    if (workspace_bytes < chip_mul_mat_workspace_size(wtype, ne0, n)) return CHIP_ENOMEM;
    if (!norm_quantized_applicable(a, lda, b, ldb, sum, ld_sum, ne0, w, y, ldy)) return CHIP_EUNSUPPORTED;
    return hip_rc(launch_norm_quantized(a, lda, b, ldb, sum, ld_sum, n, ne0, eps, w, y, ldy, (uint8_t *)workspace, act_stride(at, ne0),
                                        kind, (hipStream_t)stream));
}
int chip_silu_mul(const float *x, int64_t ldx, const float *b, int64_t ldb, int64_t n, int64_t ne0, float *y, int64_t ldy, void *stream) {
    if (n < 0 || ne0 < 0) return CHIP_EINVAL;
    if (n == 0 || ne0 == 0) return CHIP_OK;
    if (ne0 % 8 != 0) return CHIP_EUNSUPPORTED;                            // as chip_silu
    if (!rows_ok(x, ldx, ne0) || !rows_ok(y, ldy, ne0) || !rows_ok(b, ldb, ne0)) return CHIP_EINVAL;
    return hip_rc(launch_silu_mul(x, ldx, b, ldb, ne0, n, y, ldy, (hipStream_t)stream));
}
// silu(x) * b in front of a matmul, leaving the quantized rows in its workspace (what chip_mul_mat_prepare would write from y).
int chip_silu_mul_quantized(const float *x, int64_t ldx, const float *b, int64_t ldb, int64_t n, int64_t ne0, float *y, int64_t ldy,
                            int wtype, void *workspace, size_t workspace_bytes, void *stream) {
    if (n < 0 || ne0 < 0) return CHIP_EINVAL;
    if (n == 0 || ne0 == 0) return CHIP_OK;
    if (!chip_mul_mat_supported(wtype, ne0)) return CHIP_EUNSUPPORTED;
    const int at = chip_vec_dot_type(wtype);
    const int kind = (at == T_Q8_0 || at == T_Q8_1) ? 1 : (at == T_Q8_K ? 2 : 0);
    if (kind == 0) return CHIP_EUNSUPPORTED;                               // F16 weights: plain fp16 rows, not done here
    if (!rows_ok(x, ldx, ne0) || !rows_ok(y, ldy, ne0) || !rows_ok(b, ldb, ne0) || n > 65535) return CHIP_EINVAL;
    if (!workspace || !aligned16(workspace)) return CHIP_EINVAL;
    if (workspace_bytes < chip_mul_mat_workspace_size(wtype, ne0, n)) return CHIP_ENOMEM;
    if (!silu_mul_quantized_applicable(x, ldx, b, ldb, ne0, y, ldy)) return CHIP_EUNSUPPORTED;
    return hip_rc(launch_silu_mul_quantized(x, ldx, b, ldb, ne0, n, y, ldy, (uint8_t *)workspace, act_stride(at, ne0), kind, (hipStream_t)stream));
}
int chip_silu(const float *x, int64_t ldx, int64_t n, int64_t ne0, float *y, int64_t ldy, void *stream) {
    if (n < 0 || ne0 < 0) return CHIP_EINVAL;
    if (n == 0 || ne0 == 0) return CHIP_OK;
    if (ne0 % 8 != 0) return CHIP_EUNSUPPORTED;                            // the reference's row tail uses the C library's expf
    if (!rows_ok(x, ldx, ne0) || !rows_ok(y, ldy, ne0)) return CHIP_EINVAL;
    return hip_rc(launch_silu(x, ldx, ne0, n, y, ldy, (hipStream_t)stream));
}

// ---- attention matmuls over an F16 cache ----
size_t chip_mul_mat_f16_batched_workspace_size(int64_t K, int64_t N, int64_t ne02, int64_t ne12, int64_t n) {
    if (ne02 <= 0 || ne12 <= 0 || ne12 % ne02 != 0) return 0;
    return mul_mat_f16_batched_workspace_size(K, N, ne02, ne12 / ne02, n);
}
static int mul_mat_f16_batched_checked(const void *W, size_t nb01, size_t nb02, int64_t K, int64_t N, int64_t ne02, const float *x,
                                       int64_t ldx1, int64_t ldx2, int64_t n, int64_t ne12, float *y, int64_t ldy1, int64_t ldy2, float *y2,
                                       int64_t ld2y1, int64_t ld2y2, void *workspace, size_t workspace_bytes, void *stream) {
    if (K < 0 || N < 0 || n < 0 || ne02 < 0 || ne12 < 0) return CHIP_EINVAL;
    if (ne02 > 0 && ne12 % ne02 != 0) return CHIP_EINVAL;                   // src1's batch must be a multiple of src0's
    if (N == 0 || n == 0 || ne12 == 0) return CHIP_OK;
    if (K == 0 || K % 8 != 0 || ne02 > 65535) return CHIP_EUNSUPPORTED;
    if (y2 && !mul_mat_f16_batched_second_copy_supported(ne12 / ne02, n)) return CHIP_EUNSUPPORTED;
    if (!W || !x || !y) return CHIP_EINVAL;
    if (!aligned16(W) || nb01 % 16 != 0 || nb02 % 16 != 0 || nb01 < (size_t)K * 2) return CHIP_EINVAL;
    if (!aligned16(x) || ((ldx1 | ldx2) & 3) != 0 || (((uintptr_t)y) & 3) != 0 || ldy1 < N) return CHIP_EINVAL;
    if (y2 && ((((uintptr_t)y2) & 3) != 0 || ld2y1 < 0 || ld2y2 < 0)) return CHIP_EINVAL;
    if (workspace && !aligned16(workspace)) return CHIP_EINVAL;
    DeviceLimits lim;
    if (int rc = current_limits(lim); rc != CHIP_OK) return rc;
    return hip_rc(launch_mul_mat_f16_batched(W, nb01, nb02, K, N, ne02, x, ldx1, ldx2, n, ne12 / ne02, y, ldy1, ldy2, workspace,
                                             workspace_bytes, lim, (hipStream_t)stream, y2, ld2y1, ld2y2));
}
int chip_mul_mat_f16_batched(const void *W, size_t nb01, size_t nb02, int64_t K, int64_t N, int64_t ne02, const float *x,
                             int64_t ldx1, int64_t ldx2, int64_t n, int64_t ne12, float *y, int64_t ldy1, int64_t ldy2,
                             void *workspace, size_t workspace_bytes, void *stream) {
    return mul_mat_f16_batched_checked(W, nb01, nb02, K, N, ne02, x, ldx1, ldx2, n, ne12, y, ldy1, ldy2, nullptr, 0, 0, workspace,
                                       workspace_bytes, stream);
}
int chip_mul_mat_f16_batched_second_copy_supported(int64_t ne02, int64_t ne12, int64_t n) {
    return ne02 > 0 && ne12 > 0 && ne12 % ne02 == 0 && mul_mat_f16_batched_second_copy_supported(ne12 / ne02, n) ? 1 : 0;
}
int chip_mul_mat_f16_batched_two_copies(const void *W, size_t nb01, size_t nb02, int64_t K, int64_t N, int64_t ne02, const float *x,
                                        int64_t ldx1, int64_t ldx2, int64_t n, int64_t ne12, float *y, int64_t ldy1, int64_t ldy2,
                                        float *y2, int64_t ld2y1, int64_t ld2y2, void *workspace, size_t workspace_bytes, void *stream) {
    if (!y2) return CHIP_EINVAL;
    return mul_mat_f16_batched_checked(W, nb01, nb02, K, N, ne02, x, ldx1, ldx2, n, ne12, y, ldy1, ldy2, y2, ld2y1, ld2y2, workspace,
                                       workspace_bytes, stream);
}

// ---- attention-side ops ----
int chip_soft_max(const float *x, int64_t ldx, const void *mask, int mask_type, int64_t ne00, int64_t ne01, int64_t n_rows,
                  float scale, float max_bias, float *y, int64_t ldy, void *stream) {
    if (ne00 < 0 || ne01 <= 0 || n_rows < 0) return CHIP_EINVAL;
    if (n_rows == 0 || ne00 == 0) return CHIP_OK;
    if (max_bias != 0.0f) return CHIP_EUNSUPPORTED;                          // ALiBi slopes
    if (ne00 % 8 != 0) return CHIP_EUNSUPPORTED;                             // the reference's row tail uses the C library's expf
    if (mask && mask_type != T_F32 && mask_type != T_F16) return CHIP_EUNSUPPORTED;
    if (!x || !y || ldx < ne00 || ldy < ne00 || n_rows > 0x7fffffff || ne01 > 0x7fffffff) return CHIP_EINVAL;
    if (((ldx | ldy) & 3) != 0 || ((((uintptr_t)x) | ((uintptr_t)y) | ((uintptr_t)mask)) & 15) != 0) return CHIP_EINVAL;
    return hip_rc(launch_soft_max(x, ldx, mask, mask_type == T_F16, ne00, ne01, n_rows, scale, y, ldy, (hipStream_t)stream));
}

int chip_cpy(const void *src, int src_type, const int64_t ne_src[4], const int64_t nb_src[4], void *dst, int dst_type,
             const int64_t ne_dst[4], const int64_t nb_dst[4], void *stream) {
    if ((src_type != T_F32 && src_type != T_F16) || (dst_type != T_F32 && dst_type != T_F16)) return CHIP_EUNSUPPORTED;
    if (!ne_src || !nb_src || !ne_dst || !nb_dst) return CHIP_EINVAL;
    const int64_t es = src_type == T_F16 ? 2 : 4, ed = dst_type == T_F16 ? 2 : 4;
    int64_t total_s = 1, total_d = 1;
    for (int k = 0; k < 4; k++) {
        if (ne_src[k] < 0 || ne_dst[k] < 0 || nb_src[k] < 0 || nb_dst[k] < 0) return CHIP_EINVAL;
        if (nb_src[k] % es != 0 || nb_dst[k] % ed != 0) return CHIP_EINVAL;
        total_s *= ne_src[k];
        total_d *= ne_dst[k];
    }
    if (total_s != total_d) return CHIP_EINVAL;
    if (total_s == 0) return CHIP_OK;
    if (!src || !dst || (((uintptr_t)src) % es) != 0 || (((uintptr_t)dst) % ed) != 0) return CHIP_EINVAL;
    return hip_rc(launch_cpy(src, src_type == T_F16, ne_src, nb_src, dst, dst_type == T_F16, ne_dst, nb_dst, (hipStream_t)stream));
}

int chip_get_rows(int type, const void *src, size_t nb01, size_t nb02, size_t nb03, int64_t nc, int64_t ne01, const int32_t *ids,
                  int64_t ne10, int64_t ne11, int64_t ne12, int64_t ldi1, int64_t ldi2, float *dst, int64_t ld1, int64_t ld2, int64_t ld3,
                  void *stream) {
    if (nc < 0 || ne01 < 0 || ne10 < 0 || ne11 < 0 || ne12 < 0) return CHIP_EINVAL;
    if (!(type == T_F32 || is_weight_type(type))) return CHIP_EUNSUPPORTED;
    const int be = (type == T_F32 || type == T_F16) ? 1 : chip_block_elems(type);
    if (nc % be != 0) return CHIP_EINVAL;                                    // whole blocks
    if (nc == 0 || ne10 * ne11 * ne12 == 0) return CHIP_OK;
    if (!src || !ids || !dst || ld1 < nc) return CHIP_EINVAL;
    const size_t al = type == T_F32 ? 4 : 2;                                 // the dequantizers read 2-byte pieces
    if (((uintptr_t)src | nb01 | nb02 | nb03) % al != 0 || ((uintptr_t)ids & 3) != 0 || ((uintptr_t)dst & 3) != 0) return CHIP_EINVAL;
    const GetRowsArgs a{(const uint8_t *)src, nb01, nb02, nb03, nc, ne01, ids, ne10, ne11, ne12, ldi1, ldi2, dst, ld1, ld2, ld3};
    return hip_rc(launch_get_rows(type, a, (hipStream_t)stream));
}

// The constants of a ROPE node, computed like the reference's host code computes them (ggml-cpu/ops.cpp:5229-5232,
// ggml.c:3749-3761).
static void rope_constants(RopeArgs &a, int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale, float ext_factor,
                           float attn_factor, float beta_fast, float beta_slow) {
    a.n_dims = n_dims; a.neox = (mode & 2) != 0;
    a.theta_scale = powf(freq_base, -2.0f / n_dims);
    a.freq_scale = freq_scale;
    a.ext_factor = ext_factor;
    const float lo = n_dims * logf(n_ctx_orig / (beta_fast * 2 * (float)M_PI)) / (2 * logf(freq_base));
    const float hi = n_dims * logf(n_ctx_orig / (beta_slow * 2 * (float)M_PI)) / (2 * logf(freq_base));
    const float start = floorf(lo), end = ceilf(hi);
    a.corr0 = 0 > start ? 0 : start;
    a.corr1 = (n_dims - 1) < end ? (float)(n_dims - 1) : end;
    a.mscale = attn_factor;
    if (ext_factor != 0.0f) a.mscale *= 1.0f + 0.1f * logf(1.0f / freq_scale);
}
static int rope_dims_checked(int64_t ne0, int64_t ne1, int64_t ne2, int n_dims, int mode) {
    if (ne0 < 0 || ne1 < 0 || ne2 < 0 || n_dims <= 0 || n_dims > ne0 || (n_dims & 1)) return CHIP_EINVAL;
    if (mode != 0 && mode != 2) return CHIP_EUNSUPPORTED;                   // multi-section and vision layouts
    if (n_dims / 2 > 256) return CHIP_EUNSUPPORTED;
    return CHIP_OK;
}

int chip_rope(const float *x, int64_t ldx1, int64_t ldx2, const int32_t *pos, const float *freq_factors, int64_t ne0, int64_t ne1,
              int64_t ne2, int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale, float ext_factor,
              float attn_factor, float beta_fast, float beta_slow, float *y, int64_t ldy1, int64_t ldy2, void *stream) {
    if (ne0 == 0 && n_dims == 0) return CHIP_OK;
    if (int rc = rope_dims_checked(ne0, ne1, ne2, n_dims, mode); rc != CHIP_OK) return rc;
    if (ne0 == 0 || ne1 == 0 || ne2 == 0) return CHIP_OK;
    if (!x || !y || !pos || ldx1 < ne0 || ldy1 < ne0 || ne2 > 0x7fffffff) return CHIP_EINVAL;
    if ((((uintptr_t)x) | ((uintptr_t)y) | ((uintptr_t)pos) | ((uintptr_t)freq_factors)) & 3) return CHIP_EINVAL;
    RopeArgs a;
    a.ne0 = ne0; a.ne1 = ne1; a.ne2 = ne2;
    a.ldx1 = ldx1; a.ldx2 = ldx2; a.ldy1 = ldy1; a.ldy2 = ldy2;
    rope_constants(a, n_dims, mode, n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow);
    return hip_rc(launch_rope(x, pos, freq_factors, a, y, nullptr, false, (hipStream_t)stream));
}

int chip_rope_table(const int32_t *pos, const float *freq_factors, int64_t ne2, int n_dims, int n_ctx_orig, float freq_base,
                    float freq_scale, float ext_factor, float attn_factor, float beta_fast, float beta_slow, float *table,
                    void *stream) {
    if (int rc = rope_dims_checked(n_dims, 1, ne2, n_dims, 0); rc != CHIP_OK) return rc;
    if (ne2 == 0) return CHIP_OK;
    if (!pos || !table || ne2 > 0x7fffffff) return CHIP_EINVAL;
    if ((((uintptr_t)table) | ((uintptr_t)pos) | ((uintptr_t)freq_factors)) & 3) return CHIP_EINVAL;
    RopeArgs a;
    a.ne0 = n_dims; a.ne1 = 1; a.ne2 = ne2;
    a.ldx1 = a.ldx2 = a.ldy1 = a.ldy2 = 0;
    rope_constants(a, n_dims, 0, n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow);
    return hip_rc(launch_rope(nullptr, pos, freq_factors, a, nullptr, table, true, (hipStream_t)stream));
}

static int rope_apply_checked(const float *x, int64_t ldx1, int64_t ldx2, const float *table, int64_t ne0, int64_t ne1, int64_t ne2,
                              int n_dims, int mode, float *y, int64_t ldy1, int64_t ldy2, uint16_t *y16, int64_t ld16_1,
                              int64_t ld16_2, void *stream) {
    if (ne0 == 0 && n_dims == 0) return CHIP_OK;
    if (int rc = rope_dims_checked(ne0, ne1, ne2, n_dims, mode); rc != CHIP_OK) return rc;
    if (ne0 == 0 || ne1 == 0 || ne2 == 0) return CHIP_OK;
    if (!x || !y || !table || ldx1 < ne0 || ldy1 < ne0 || ne2 > 0x7fffffff) return CHIP_EINVAL;
    if ((((uintptr_t)x) | ((uintptr_t)y) | ((uintptr_t)table)) & 3) return CHIP_EINVAL;
    if (y16 && (ld16_1 < ne0 || (((uintptr_t)y16) & 1) != 0)) return CHIP_EINVAL;
    RopeArgs a;
    a.ne0 = ne0; a.ne1 = ne1; a.ne2 = ne2;
    a.ldx1 = ldx1; a.ldx2 = ldx2; a.ldy1 = ldy1; a.ldy2 = ldy2;
    a.n_dims = n_dims; a.neox = (mode & 2) != 0;
    a.theta_scale = a.freq_scale = a.ext_factor = a.corr0 = a.corr1 = a.mscale = 0.0f;       // all in the table
    a.y16 = y16; a.ld16_1 = ld16_1; a.ld16_2 = ld16_2;
    return hip_rc(launch_rope(x, nullptr, nullptr, a, y, const_cast<float *>(table), false, (hipStream_t)stream));
}
int chip_rope_apply(const float *x, int64_t ldx1, int64_t ldx2, const float *table, int64_t ne0, int64_t ne1, int64_t ne2,
                    int n_dims, int mode, float *y, int64_t ldy1, int64_t ldy2, void *stream) {
    return rope_apply_checked(x, ldx1, ldx2, table, ne0, ne1, ne2, n_dims, mode, y, ldy1, ldy2, nullptr, 0, 0, stream);
}
int chip_rope_apply_store(const float *x, int64_t ldx1, int64_t ldx2, const float *table, int64_t ne0, int64_t ne1, int64_t ne2,
                          int n_dims, int mode, float *y, int64_t ldy1, int64_t ldy2, uint16_t *y_f16, int64_t ld16_1,
                          int64_t ld16_2, void *stream) {
    if (!y_f16) return CHIP_EINVAL;
    return rope_apply_checked(x, ldx1, ldx2, table, ne0, ne1, ne2, n_dims, mode, y, ldy1, ldy2, y_f16, ld16_1, ld16_2, stream);
}

static int rope_operand_checked(const chip_rope_operand *o, int64_t ne0, int64_t ne2, int n_dims, int mode, RopeArgs &a) {
    if (!o) return CHIP_EINVAL;
    if (int rc = rope_dims_checked(ne0, o->ne1, ne2, n_dims, mode); rc != CHIP_OK) return rc;
    if (ne0 <= 0 || o->ne1 <= 0 || ne2 <= 0 || ne2 > 0x7fffffff) return CHIP_EINVAL;
    if (!o->x || (!o->y && !o->y_f16) || o->ldx1 < ne0 || (o->y && o->ldy1 < ne0)) return CHIP_EINVAL;
    if ((((uintptr_t)o->x) | ((uintptr_t)o->y)) & 3) return CHIP_EINVAL;
    if (o->y_f16 && (o->ld16_1 < ne0 || (((uintptr_t)o->y_f16) & 1) != 0)) return CHIP_EINVAL;
    a.ne0 = ne0; a.ne1 = o->ne1; a.ne2 = ne2;
    a.ldx1 = o->ldx1; a.ldx2 = o->ldx2; a.ldy1 = o->y ? o->ldy1 : 0; a.ldy2 = o->y ? o->ldy2 : 0;
    a.n_dims = n_dims; a.neox = (mode & 2) != 0;
    a.theta_scale = a.freq_scale = a.ext_factor = a.corr0 = a.corr1 = a.mscale = 0.0f;       // all in the table
    a.y16 = o->y_f16; a.ld16_1 = o->y_f16 ? o->ld16_1 : 0; a.ld16_2 = o->y_f16 ? o->ld16_2 : 0;
    return CHIP_OK;
}
int chip_rope_apply_two(const chip_rope_operand *a, const chip_rope_operand *b, const float *table, int64_t ne0, int64_t ne2,
                        int n_dims, int mode, void *stream) {
    RopeArgs ra, rb;
    if (int rc = rope_operand_checked(a, ne0, ne2, n_dims, mode, ra); rc != CHIP_OK) return rc;
    if (int rc = rope_operand_checked(b, ne0, ne2, n_dims, mode, rb); rc != CHIP_OK) return rc;
    if (!table || (((uintptr_t)table) & 3)) return CHIP_EINVAL;
    return hip_rc(launch_rope_apply_two(a->x, ra, a->y, b->x, rb, b->y, table, (hipStream_t)stream));
}

int chip_block_isums(int type, const void *W, size_t nb01, int64_t K, int64_t N, const void *aq, int64_t n,
                     int32_t *isum, int32_t *imin, void *stream) {
    if (N < 0 || n < 0) return CHIP_EINVAL;
    if (!chip_mul_mat_supported(type, K) || type == T_F16 || type == T_Q6_K_P) return CHIP_EUNSUPPORTED;   // F16 has no integer sums
    if (N == 0 || n == 0) return CHIP_OK;
    if (!W || !aq || !isum) return CHIP_EINVAL;
    if (!weights_aligned(type, W, nb01, K) || N > 0x7fffffff || n > 65535) return CHIP_EINVAL;
    return hip_rc(launch_block_isums(type, W, nb01, K, N, aq, n, isum, (type == T_Q4_K || type == T_Q5_K || type == T_Q2_K) ? imin : nullptr, (hipStream_t)stream));
}

int chip_verify_force_q6k_matrix_core(int on) {
    g_force_mmv_q6k.store(on ? 1 : 0, std::memory_order_relaxed);
    return CHIP_OK;
}

int chip_workspace_to_blocks(int type, int64_t K, int64_t n, const void *workspace, void *y, void *stream) {
    if (n < 0) return CHIP_EINVAL;
    if (!chip_mul_mat_supported(type, K)) return CHIP_EUNSUPPORTED;
    if (n == 0) return CHIP_OK;
    if (!workspace || !y || n > 65535) return CHIP_EINVAL;
    const int at = chip_vec_dot_type(type);
    return hip_rc(launch_split_to_blocks(at, workspace, act_stride(at, K), n, K, y, chip_row_size(at, K), (hipStream_t)stream));
}

}  // extern "C"
