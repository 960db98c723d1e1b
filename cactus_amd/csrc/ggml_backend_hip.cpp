// libggml-hip.so: the reference's ggml backend interface (ggml-backend-impl.h:17-207) implemented on top of the
// C-ABI of include/cactus_hip.h.  Host C++ only; every GPU action goes through chip_* calls.
//
//   reg "HIP"  ->  device "HIP0" (ACCEL by default: a weights-only co-processor, like the AMX extra buffer type,
//                  reference ggml-cpu/amx/amx.cpp:141-174; CACTUS_HIP_DEVICE_TYPE=GPU switches)
//              ->  buffer type "HIP": hipMalloc'd buffers, tensors at base + offset, GGUF blocks kept verbatim
//              ->  buffer type "HIP_Host": pinned host memory (the staging buffers of the loader's async upload)
//              ->  backend "HIP": one stream; graph_compute runs MUL_MAT / MUL_MAT_ID (F32 activations x block-quantized
//                  or F16 weights living in a HIP buffer), the ops around them in a transformer layer (RMS_NORM, ADD,
//                  MUL, SILU, ROPE, CPY / CONT / DUP, SOFT_MAX, the batched F16 matmuls over the KV cache) and skips
//                  view ops; set/get_tensor_async and events on that stream.
// No C++ exception crosses the vtables; failures are NULL returns or LM_GGML_STATUS_FAILED.
#include "../../include/cactus_hip.h"
#include "../../include/ggml_abi_mirror.h"
#include "../../include/ggml_backend_hip.h"

#include <algorithm>
#include <atomic>
#include <dlfcn.h>
#include <map>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

namespace {

std::atomic<unsigned long long> g_mul_mat_nodes{0}, g_uploaded{0}, g_elementwise_nodes{0}, g_fused_pairs{0}, g_rope_tables{0},
    g_quantizers_skipped{0}, g_uploaded_async{0}, g_grouped_matmuls{0}, g_head_merges{0}, g_rope_pairs{0}, g_gated_pairs{0}, g_rope_epilogues{0}, g_norms_in_prologue{0}, g_residual_adds{0}, g_planes_copies{0}, g_planes_bytes{0}, g_planes_dropped{0}, g_planes_matmuls{0};

#define HIP_LOG(level, ...) lm_ggml_log_internal(level, __VA_ARGS__)

// A 2-D Q6_K weight's second copy with its rows in planes (chip_repack_q6_K), which the decode GEMVs (up to 4 tokens) read
// instead: block_q6_K's 210-byte pitch leaves every load of those kernels 2-byte aligned, the planes 16-byte aligned, and the
// kernels then run 10 to 15 % faster on the same bits.  The tensor's own bytes stay as they are for every other reader (GEMM,
// MUL_MAT_ID, GET_ROWS, get_tensor); the copy is made at the weight's first decode matmul, kept with the buffer and dropped
// when anything writes over the weight.
struct planes_copy { void *data; size_t src_span; size_t nb01; int64_t K, N; };
struct buffer_ctx {
    void *base; size_t size;
    std::mutex mu;
    std::map<const uint8_t *, planes_copy> planes;     // by the weight's address
    std::atomic<int> n_planes{0};
    size_t max_span = 0;                               // the largest src_span ever entered
    bool planes_failed = false;                        // an allocation failed: no further copies for this buffer
    buffer_ctx(void *b, size_t s) : base(b), size(s) {}
};
// The cos / sin table of the ROPE nodes of one graph_compute call: Q and K of every layer are rotated by the same
// positions, so the first ROPE node of a call builds the table and the others apply it.  The key is only valid inside
// the call (the position tensor keeps its address from call to call while its contents change).
struct rope_table_key {
    const void *pos, *ff;
    int64_t ne2;
    int32_t params[11];        // op_params 1..10 without the mode: n_dims, n_ctx, n_ctx_orig and the six floats
    bool valid;
};
// What the workspace's activation rows were quantized from: wq / wk / wv (and ffn_up / ffn_gate) read the same tensor, so
// the later ones skip the quantizer.  Dropped when anything else uses the workspace or writes over the source.
struct quantized_key {
    bool valid = false;
    const void *src = nullptr; size_t src_bytes = 0;
    int64_t K = 0, n = 0, ldx = 0;
    int vec_dot_type = -1;
};

struct backend_ctx {
    void *stream; void *workspace; size_t workspace_size;
    float *rope_table = nullptr; size_t rope_table_bytes = 0;
    rope_table_key rope_key = {};
    quantized_key quantized = {};
    uint16_t *gelu_table = nullptr;                  // device copy of the 65536-entry fp16 GELU table
    float *group_scratch = nullptr; size_t group_slot_bytes = 0;     // CHIP_GROUP_MAX result slots for projections run early
};

lm_ggml_backend_buffer_type_t hip_buffer_type();
lm_ggml_backend_dev_t hip_device();

bool device_ok() {
    static int ok = -1;
    static std::mutex mu;
    std::lock_guard<std::mutex> lk(mu);
    if (ok < 0) ok = (chip_device_count() > 0 && chip_init(0) == CHIP_OK) ? 1 : 0;
    return ok == 1;
}

bool is_host_buffer(const lm_ggml_backend_buffer *b) {
    return b && b->buft && b->buft->iface.is_host && b->buft->iface.is_host(b->buft);
}
bool is_hip_buffer(const lm_ggml_backend_buffer *b) { return b && b->buft == hip_buffer_type(); }

// ------------------------------------------------------------------------------------------------ buffer
// Drops the planes copies of the weights that [lo, lo + bytes) touches: called by everything that writes into a buffer.
// (chip_free waits for the device, so a GEMV still reading a copy finishes first)
void drop_planes(buffer_ctx *bc, const void *lo, size_t bytes) {
    if (!bc || bc->n_planes.load(std::memory_order_acquire) == 0 || bytes == 0) return;
    std::lock_guard<std::mutex> lk(bc->mu);
    const uint8_t *a = (const uint8_t *)lo, *b = a + bytes;
    // the weights that start below b, from the highest down to the last one a span of the largest size could still reach
    auto it = bc->planes.lower_bound(b);
    while (it != bc->planes.begin()) {
        --it;
        if (it->first + bc->max_span <= a) break;
        if (a < it->first + it->second.src_span) {
            chip_free(it->second.data);
            it = bc->planes.erase(it);
            bc->n_planes--;
            g_planes_dropped++;
        }
    }
}
buffer_ctx *hip_buffer_ctx_of(const lm_ggml_tensor *t) {
    const lm_ggml_backend_buffer *b = t->view_src ? t->view_src->buffer : t->buffer;
    return is_hip_buffer(b) ? (buffer_ctx *)b->context : nullptr;
}
void buf_free(lm_ggml_backend_buffer_t buffer) {
    buffer_ctx *c = (buffer_ctx *)buffer->context;
    drop_planes(c, c->base, c->size);
    chip_free(c->base);
    delete c;
}
void *buf_get_base(lm_ggml_backend_buffer_t buffer) { return ((buffer_ctx *)buffer->context)->base; }
void buf_memset_tensor(lm_ggml_backend_buffer_t buffer, lm_ggml_tensor *t, uint8_t value, size_t offset, size_t size) {
    drop_planes((buffer_ctx *)buffer->context, (char *)t->data + offset, size);
    chip_memset((char *)t->data + offset, value, size, nullptr);
    chip_stream_synchronize(nullptr);
}
void buf_set_tensor(lm_ggml_backend_buffer_t buffer, lm_ggml_tensor *t, const void *data, size_t offset, size_t size) {
    drop_planes((buffer_ctx *)buffer->context, (char *)t->data + offset, size);
    chip_memcpy_h2d((char *)t->data + offset, data, size, nullptr);          // synchronous
    g_uploaded += size;
}
void buf_get_tensor(lm_ggml_backend_buffer_t, const lm_ggml_tensor *t, void *data, size_t offset, size_t size) {
    chip_stream_synchronize(nullptr);
    chip_memcpy_d2h(data, (const char *)t->data + offset, size, nullptr);    // synchronous
}
bool buf_cpy_tensor(lm_ggml_backend_buffer_t buffer, const lm_ggml_tensor *src, lm_ggml_tensor *dst) {
    const size_t n = lm_ggml_nbytes(src);
    drop_planes((buffer_ctx *)buffer->context, dst->data, n);
    if (is_host_buffer(src->buffer)) {
        chip_memcpy_h2d(dst->data, src->data, n, nullptr);
        return true;
    }
    if (is_hip_buffer(src->buffer)) {
        chip_memcpy_d2d(dst->data, src->data, n, nullptr);
        chip_stream_synchronize(nullptr);
        return true;
    }
    return false;
}
void buf_clear(lm_ggml_backend_buffer_t buffer, uint8_t value) {
    buffer_ctx *c = (buffer_ctx *)buffer->context;
    drop_planes(c, c->base, c->size);
    chip_memset(c->base, value, c->size, nullptr);
    chip_stream_synchronize(nullptr);
}
const lm_ggml_backend_buffer_i k_buffer_i = {
    /* free_buffer   */ buf_free,
    /* get_base      */ buf_get_base,
    /* init_tensor   */ nullptr,
    /* memset_tensor */ buf_memset_tensor,
    /* set_tensor    */ buf_set_tensor,
    /* get_tensor    */ buf_get_tensor,
    /* cpy_tensor    */ buf_cpy_tensor,
    /* clear         */ buf_clear,
    /* reset         */ nullptr,
};

// ------------------------------------------------------------------------------------------------ buffer type
const char *buft_name(lm_ggml_backend_buffer_type_t) { return "HIP"; }
lm_ggml_backend_buffer_t buft_alloc(lm_ggml_backend_buffer_type_t buft, size_t size) {
    if (!device_ok()) return nullptr;
    void *p = nullptr;
    if (chip_malloc(&p, size) != CHIP_OK || !p) {
        HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: hipMalloc of %zu bytes failed\n", __func__, size);
        return nullptr;
    }
    buffer_ctx *c = new (std::nothrow) buffer_ctx(p, size);
    if (!c) { chip_free(p); return nullptr; }
    return lm_ggml_backend_buffer_init(buft, k_buffer_i, c, size);
}
size_t buft_alignment(lm_ggml_backend_buffer_type_t) { return 256; }       // rows stay 16-byte aligned for the kernels
bool buft_is_host(lm_ggml_backend_buffer_type_t) { return false; }

// ------------------------------------------------------------------------------------------------ pinned host buffer type
// What lm_ggml_backend_dev_host_buffer_type returns: host memory the GPU can copy from without staging, so that
// set_tensor_async overlaps with the caller (the loader reads the next chunk of the file meanwhile).
lm_ggml_backend_buffer_type_t hip_host_buffer_type();
void hbuf_free(lm_ggml_backend_buffer_t buffer) {
    buffer_ctx *c = (buffer_ctx *)buffer->context;
    chip_host_free(c->base);
    delete c;
}
void hbuf_memset_tensor(lm_ggml_backend_buffer_t, lm_ggml_tensor *t, uint8_t value, size_t offset, size_t size) {
    std::memset((char *)t->data + offset, value, size);
}
void hbuf_set_tensor(lm_ggml_backend_buffer_t, lm_ggml_tensor *t, const void *data, size_t offset, size_t size) {
    std::memcpy((char *)t->data + offset, data, size);
}
void hbuf_get_tensor(lm_ggml_backend_buffer_t, const lm_ggml_tensor *t, void *data, size_t offset, size_t size) {
    std::memcpy(data, (const char *)t->data + offset, size);
}
bool hbuf_cpy_tensor(lm_ggml_backend_buffer_t, const lm_ggml_tensor *src, lm_ggml_tensor *dst) {
    if (!is_host_buffer(src->buffer)) return false;
    std::memcpy(dst->data, src->data, lm_ggml_nbytes(src));
    return true;
}
void hbuf_clear(lm_ggml_backend_buffer_t buffer, uint8_t value) {
    buffer_ctx *c = (buffer_ctx *)buffer->context;
    std::memset(c->base, value, c->size);
}
const lm_ggml_backend_buffer_i k_host_buffer_i = {
    /* free_buffer   */ hbuf_free,
    /* get_base      */ buf_get_base,
    /* init_tensor   */ nullptr,
    /* memset_tensor */ hbuf_memset_tensor,
    /* set_tensor    */ hbuf_set_tensor,
    /* get_tensor    */ hbuf_get_tensor,
    /* cpy_tensor    */ hbuf_cpy_tensor,
    /* clear         */ hbuf_clear,
    /* reset         */ nullptr,
};
const char *hbuft_name(lm_ggml_backend_buffer_type_t) { return "HIP_Host"; }
lm_ggml_backend_buffer_t hbuft_alloc(lm_ggml_backend_buffer_type_t buft, size_t size) {
    if (!device_ok()) return nullptr;
    void *p = nullptr;
    if (chip_host_malloc(&p, size) != CHIP_OK || !p) {
        HIP_LOG(LM_GGML_LOG_LEVEL_WARN, "%s: pinned allocation of %zu bytes failed\n", __func__, size);
        return nullptr;
    }
    buffer_ctx *c = new (std::nothrow) buffer_ctx(p, size);
    if (!c) { chip_host_free(p); return nullptr; }
    return lm_ggml_backend_buffer_init(buft, k_host_buffer_i, c, size);
}
size_t hbuft_alignment(lm_ggml_backend_buffer_type_t) { return 64; }
bool hbuft_is_host(lm_ggml_backend_buffer_type_t) { return true; }

// ------------------------------------------------------------------------------------------------ backend
lm_ggml_guid_t hip_guid() {
    static lm_ggml_guid g = {0x63, 0x61, 0x63, 0x74, 0x75, 0x73, 0x2d, 0x68, 0x69, 0x70, 0x2d, 0x67, 0x66, 0x78, 0x39, 0x35};
    return &g;
}
const char *backend_name(lm_ggml_backend_t) { return "HIP"; }
void backend_free(lm_ggml_backend_t backend) {
    backend_ctx *c = (backend_ctx *)backend->context;
    chip_stream_synchronize(c->stream);
    chip_free(c->workspace);
    chip_free(c->rope_table);
    chip_free(c->gelu_table);
    chip_free(c->group_scratch);
    chip_stream_destroy(c->stream);
    delete c;
    delete backend;
}
void backend_synchronize(lm_ggml_backend_t backend) { chip_stream_synchronize(((backend_ctx *)backend->context)->stream); }
// Asynchronous on the backend's stream, ordered with graph_compute; the host memory must stay untouched until the
// stream (or an event recorded after the call) has been waited for.
void backend_set_tensor_async(lm_ggml_backend_t backend, lm_ggml_tensor *t, const void *data, size_t offset, size_t size) {
    drop_planes(hip_buffer_ctx_of(t), (char *)t->data + offset, size);
    chip_memcpy_h2d((char *)t->data + offset, data, size, ((backend_ctx *)backend->context)->stream);
    g_uploaded += size;
    g_uploaded_async += size;
}
void backend_get_tensor_async(lm_ggml_backend_t backend, const lm_ggml_tensor *t, void *data, size_t offset, size_t size) {
    chip_memcpy_d2h(data, (const char *)t->data + offset, size, ((backend_ctx *)backend->context)->stream);
}
void backend_event_record(lm_ggml_backend_t backend, lm_ggml_backend_event_t event) {
    chip_event_record(event->context, ((backend_ctx *)backend->context)->stream);
}
void backend_event_wait(lm_ggml_backend_t backend, lm_ggml_backend_event_t event) {
    chip_stream_wait_event(((backend_ctx *)backend->context)->stream, event->context);
}

bool is_view_op(int op) {
    return op == LM_GGML_OP_NONE || op == LM_GGML_OP_RESHAPE || op == LM_GGML_OP_VIEW || op == LM_GGML_OP_PERMUTE ||
           op == LM_GGML_OP_TRANSPOSE;
}

// What a weight row's start and stride must be a multiple of: super-blocks of 210 (Q6_K) and 110 bytes (Q3_K) allow 2, of 84
// bytes (Q2_K) and rows of K % 256 != 0 (32-value block types only) 4, everything else 16.
size_t weight_alignment(const lm_ggml_tensor *w) {
    if (w->type == LM_GGML_TYPE_Q6_K || w->type == LM_GGML_TYPE_Q3_K) return 2;
    if (w->type == LM_GGML_TYPE_IQ4_XS) return 8;                     // 136-byte super-blocks
    return (w->type == LM_GGML_TYPE_Q2_K || w->ne[0] % 256 != 0) ? 4 : 16;
}
// The MUL_MAT shapes the kernels take: weights [K, N] of a supported block type with whole-row strides, F32
// activations [K, n] and F32 result [N, n] with element-contiguous rows, no batch dimensions.
bool mul_mat_shape_ok(const lm_ggml_tensor *op) {
    const lm_ggml_tensor *w = op->src[0], *x = op->src[1];
    if (!w || !x) return false;
    if (!chip_mul_mat_supported(w->type, w->ne[0])) return false;
    if (x->type != LM_GGML_TYPE_F32 || op->type != LM_GGML_TYPE_F32) return false;
    if (w->ne[2] != 1 || w->ne[3] != 1 || x->ne[2] != 1 || x->ne[3] != 1) return false;
    if (x->ne[0] != w->ne[0] || op->ne[0] != w->ne[1] || op->ne[1] != x->ne[1]) return false;
    if (w->nb[0] != chip_block_bytes(w->type) || w->nb[1] < chip_row_size(w->type, w->ne[0])) return false;
    if (w->nb[1] % weight_alignment(w) != 0) return false;
    if (x->nb[0] != sizeof(float) || x->nb[1] % 16 != 0 || x->nb[1] < (size_t)x->ne[0] * 4) return false;
    if (op->nb[0] != sizeof(float) || op->nb[1] % 4 != 0 || op->nb[1] < (size_t)op->ne[0] * 4) return false;
    return true;
}

// The attention matmuls: F16 src0 [K, N, ne02] that is a strided view of the KV cache, F32 src1 [K, n, ne12] with ne12 a
// multiple of ne02 (reference llama-graph.cpp:1120, 1154).  Anything the plain 2-D path takes goes there first.
bool elementwise_enabled();
bool mul_mat_f16_batched_shape_ok(const lm_ggml_tensor *op) {
    const lm_ggml_tensor *w = op->src[0], *x = op->src[1];
    if (!w || !x || w->type != LM_GGML_TYPE_F16 || x->type != LM_GGML_TYPE_F32 || op->type != LM_GGML_TYPE_F32) return false;
    if (!elementwise_enabled()) return false;
    const int64_t K = w->ne[0], N = w->ne[1];
    if (K <= 0 || K % 8 != 0 || w->ne[3] != 1 || x->ne[3] != 1 || op->ne[3] != 1) return false;
    if (w->ne[2] < 1 || w->ne[2] > 65535 || x->ne[2] % w->ne[2] != 0) return false;
    if (x->ne[0] != K || op->ne[0] != N || op->ne[1] != x->ne[1] || op->ne[2] != x->ne[2]) return false;
    if (w->nb[0] != 2 || w->nb[1] % 16 != 0 || w->nb[2] % 16 != 0 || w->nb[1] < (size_t)K * 2) return false;
    if (x->nb[0] != 4 || x->nb[1] % 16 != 0 || x->nb[2] % 16 != 0) return false;
    if (op->nb[0] != 4 || op->nb[1] % 4 != 0 || op->nb[2] % 4 != 0 || op->nb[1] < (size_t)N * 4) return false;
    return true;
}

// MUL_MAT with batch dimensions over a weight of a supported block type: src0 [K, N, ne02, ne03], src1 [K, n, ne12, ne13]
// with ne12 / ne13 multiples of ne02 / ne03 (slice (i12, i13) of src1 meets slice (i12 / r2, i13 / r3) of src0: reference
// ggml-cpu/ggml-cpu.c:1188-1189, 1294-1295).  Every slice is a 2-D matmul of the kind above; what the two paths above take goes
// there first.
bool mul_mat_batched_shape_ok(const lm_ggml_tensor *op) {
    const lm_ggml_tensor *w = op->src[0], *x = op->src[1];
    if (!w || !x || !chip_mul_mat_supported(w->type, w->ne[0])) return false;
    if (x->type != LM_GGML_TYPE_F32 || op->type != LM_GGML_TYPE_F32) return false;
    if (w->ne[2] < 1 || w->ne[3] < 1 || x->ne[2] % w->ne[2] != 0 || x->ne[3] % w->ne[3] != 0) return false;
    if (x->ne[2] * x->ne[3] <= 1 || x->ne[2] * x->ne[3] > 65536) return false;
    if (x->ne[0] != w->ne[0] || op->ne[0] != w->ne[1] || op->ne[1] != x->ne[1] || op->ne[2] != x->ne[2] || op->ne[3] != x->ne[3]) return false;
    const size_t a = weight_alignment(w);
    if (w->nb[0] != chip_block_bytes(w->type) || w->nb[1] < chip_row_size(w->type, w->ne[0]) || w->nb[1] % a != 0) return false;
    if (w->nb[2] % a != 0 || w->nb[3] % a != 0) return false;
    if (x->nb[0] != sizeof(float) || x->nb[1] % 16 != 0 || x->nb[1] < (size_t)x->ne[0] * 4 || x->nb[2] % 16 != 0 || x->nb[3] % 16 != 0) return false;
    if (op->nb[0] != sizeof(float) || op->nb[1] % 4 != 0 || op->nb[1] < (size_t)op->ne[0] * 4 || op->nb[2] % 4 != 0 || op->nb[3] % 4 != 0) return false;
    return true;
}

// The MUL_MAT_ID shapes: experts [K, N, n_as] stored one matrix after the other, F32 activations [K, ne11, n_tokens]
// with ne11 = 1 or n_used and the rows of a token adjacent, I32 ids [n_used, n_tokens], F32 result
// [N, n_used, n_tokens] with adjacent rows (reference ggml.c lm_ggml_mul_mat_id, ggml-cpu/ggml-cpu.c:1531-1710).
bool mul_mat_id_shape_ok(const lm_ggml_tensor *op) {
    const lm_ggml_tensor *w = op->src[0], *x = op->src[1], *ids = op->src[2];
    if (!w || !x || !ids) return false;
    if (!chip_mul_mat_supported(w->type, w->ne[0])) return false;
    if (x->type != LM_GGML_TYPE_F32 || op->type != LM_GGML_TYPE_F32 || ids->type != LM_GGML_TYPE_I32) return false;
    const int64_t K = w->ne[0], N = w->ne[1], n_used = ids->ne[0], n_tokens = ids->ne[1];
    if (K % 256 != 0) return false;                                     // the expert kernels assume 16-byte aligned rows
    if (w->ne[3] != 1 || x->ne[3] != 1 || op->ne[3] != 1 || ids->ne[2] != 1 || ids->ne[3] != 1) return false;
    if (x->ne[0] != K || x->ne[2] != n_tokens || !(x->ne[1] == 1 || x->ne[1] == n_used)) return false;
    if (op->ne[0] != N || op->ne[1] != n_used || op->ne[2] != n_tokens) return false;
    const size_t a = weight_alignment(w);
    if (w->nb[0] != chip_block_bytes(w->type) || w->nb[1] < chip_row_size(w->type, K) || w->nb[1] % a != 0) return false;
    if (w->nb[2] < (size_t)N * w->nb[1] || w->nb[2] % a != 0) return false;
    if (x->nb[0] != sizeof(float) || x->nb[1] % 16 != 0 || x->nb[1] < (size_t)K * 4 || x->nb[2] != (size_t)x->ne[1] * x->nb[1]) return false;
    if (ids->nb[0] != sizeof(int32_t) || ids->nb[1] % 4 != 0 || ids->nb[1] < (size_t)n_used * 4) return false;
    if (op->nb[0] != sizeof(float) || op->nb[1] % 4 != 0 || op->nb[1] < (size_t)N * 4 || op->nb[2] != (size_t)n_used * op->nb[1]) return false;
    return true;
}

// ---- the element-wise ops between the matmuls (RMS_NORM, ADD, MUL, UNARY SILU; F32) ----
// A tensor as rows: element-contiguous rows at one uniform stride across the higher dimensions.
bool as_rows(const lm_ggml_tensor *t, int64_t &rows, int64_t &ld) {
    if (t->type != LM_GGML_TYPE_F32 || t->nb[0] != sizeof(float) || t->nb[1] % 4 != 0 || t->nb[1] < (size_t)t->ne[0] * 4) return false;
    if (t->ne[2] > 1 && t->nb[2] != (size_t)t->ne[1] * t->nb[1]) return false;
    if (t->ne[3] > 1 && t->nb[3] != (size_t)t->ne[2] * t->ne[1] * t->nb[1]) return false;
    rows = t->ne[1] * t->ne[2] * t->ne[3];
    ld = (int64_t)(t->nb[1] / 4);
    return true;
}
bool same_shape(const lm_ggml_tensor *a, const lm_ggml_tensor *b) {
    return a->ne[0] == b->ne[0] && a->ne[1] == b->ne[1] && a->ne[2] == b->ne[2] && a->ne[3] == b->ne[3];
}
bool elementwise_enabled() {
    static const bool on = [] { const char *e = std::getenv("CACTUS_HIP_ELEMENTWISE"); return !(e && std::strcmp(e, "0") == 0); }();
    return on;
}
bool fusion_enabled() {
    static const bool on = [] { const char *e = std::getenv("CACTUS_HIP_FUSE"); return !(e && std::strcmp(e, "0") == 0); }();
    return on;
}
bool planes_enabled() {
    static const bool on = [] { const char *e = std::getenv("CACTUS_HIP_Q6K_PLANES"); return !(e && std::strcmp(e, "0") == 0); }();
    return on;
}
// The weight operand of a matmul of n tokens as the kernels take it: the tensor's own bytes, or for a Q6_K weight at up to
// 4 tokens its copy in planes (made here, on the backend's stream, at the first such matmul).
struct weight_arg { int type; const void *data; size_t nb01; };
weight_arg weight_for(backend_ctx *c, const lm_ggml_tensor *w, int64_t n) {
    const weight_arg own{(int)w->type, w->data, w->nb[1]};
    if (w->type != LM_GGML_TYPE_Q6_K || n < 1 || n > 4 || w->ne[2] != 1 || w->ne[3] != 1 || w->ne[1] <= 0 || !planes_enabled()) return own;
    const int64_t K = w->ne[0], N = w->ne[1];
    const size_t row = chip_row_size(CHIP_TYPE_Q6_K, K);
    if (!chip_mul_mat_supported(CHIP_TYPE_Q6_K_PLANES, K) || row > 160 * 1024 || w->nb[1] < row || w->nb[1] % 2 != 0) return own;
    buffer_ctx *bc = hip_buffer_ctx_of(w);
    if (!bc || bc->planes_failed) return own;
    std::lock_guard<std::mutex> lk(bc->mu);
    const uint8_t *key = (const uint8_t *)w->data;
    auto it = bc->planes.find(key);
    if (it != bc->planes.end()) {
        const planes_copy &pc = it->second;
        if (pc.K == K && pc.N == N && pc.nb01 == w->nb[1]) {
            g_planes_matmuls++;
            return weight_arg{CHIP_TYPE_Q6_K_PLANES, pc.data, row};
        }
        chip_free(pc.data);                            // the same address read as another shape
        bc->planes.erase(it);
        bc->n_planes--;
        g_planes_dropped++;
    }
    const size_t bytes = (size_t)N * row;
    chip_device_info info;
    if (chip_get_device_info(&info) != CHIP_OK || info.hbm_free < bytes + ((size_t)1 << 30)) {   // leave the caller a GiB
        bc->planes_failed = true;
        return own;
    }
    void *p = nullptr;
    if (chip_malloc(&p, bytes) != CHIP_OK || !p) {
        bc->planes_failed = true;
        return own;
    }
    // finished before the copy is entered: another backend instance on the same buffer reads it from its own stream
    if (chip_repack_q6_K(w->data, w->nb[1], p, row, K, N, 1, c->stream) != CHIP_OK || chip_stream_synchronize(c->stream) != CHIP_OK) {
        chip_free(p);
        bc->planes_failed = true;
        return own;
    }
    const size_t span = (size_t)(N - 1) * w->nb[1] + row;
    bc->planes.emplace(key, planes_copy{p, span, w->nb[1], K, N});
    bc->max_span = std::max(bc->max_span, span);
    bc->n_planes++;
    g_planes_copies++;
    g_planes_bytes += bytes;
    g_planes_matmuls++;
    return weight_arg{CHIP_TYPE_Q6_K_PLANES, p, row};
}
bool elementwise_shape_ok(const lm_ggml_tensor *op) {
    if (!elementwise_enabled()) return false;
    const lm_ggml_tensor *a = op->src[0], *b = op->src[1];
    int64_t r, ld;
    if (!a || !as_rows(op, r, ld) || !as_rows(a, r, ld) || !same_shape(op, a)) return false;
    switch (op->op) {
        case LM_GGML_OP_RMS_NORM: return true;
        case LM_GGML_OP_SCALE:    return true;
        case LM_GGML_OP_UNARY:    return (op->op_params[0] == LM_GGML_UNARY_OP_SILU && a->ne[0] % 8 == 0) || op->op_params[0] == LM_GGML_UNARY_OP_GELU;
        case LM_GGML_OP_ADD:
        case LM_GGML_OP_MUL:
            // src1: the shape of src0, or one row broadcast over all rows (norm weights, biases)
            if (!b || !as_rows(b, r, ld) || b->ne[0] != a->ne[0]) return false;
            return same_shape(a, b) || (b->ne[1] == 1 && b->ne[2] == 1 && b->ne[3] == 1);
        default: return false;
    }
}
// The table of LM_GGML_UNARY_OP_GELU on the device.  The host framework's own table (lm_ggml_table_gelu_f16, filled by
// lm_ggml_cpu_init, reference ggml-cpu/ggml-cpu.c:3474-3481) is taken when this process exports it and it is filled: the
// device then returns exactly what that framework's CPU backend returns, whatever compiler and C library built it.
// Otherwise the same formula is evaluated here.
bool ensure_gelu_table(backend_ctx *c) {
    if (c->gelu_table) return true;
    static uint16_t host_table[65536];
    const uint16_t *src = (const uint16_t *)dlsym(RTLD_DEFAULT, "lm_ggml_table_gelu_f16");
    if (!src || src[0x3c00] == 0) {                                     // gelu(1.0) is 0.84: a zero entry means "not initialised"
        if (chip_gelu_table(host_table) != CHIP_OK) return false;
        src = host_table;
    }
    void *dev = nullptr;
    if (chip_malloc(&dev, sizeof(host_table)) != CHIP_OK) return false;
    if (chip_memcpy_h2d(dev, src, sizeof(host_table), c->stream) != CHIP_OK || chip_stream_synchronize(c->stream) != CHIP_OK) {
        chip_free(dev);
        return false;
    }
    c->gelu_table = (uint16_t *)dev;
    return true;
}

int run_elementwise(backend_ctx *c, lm_ggml_tensor *op) {
    const lm_ggml_tensor *a = op->src[0], *b = op->src[1];
    int64_t rows, lda, ldy, rb = 0, ldb = 0;
    as_rows(a, rows, lda);
    as_rows(op, rows, ldy);
    const int64_t ne0 = a->ne[0];
    switch (op->op) {
        case LM_GGML_OP_RMS_NORM: {
            float eps;
            std::memcpy(&eps, op->op_params, sizeof(float));
            return chip_rms_norm((const float *)a->data, lda, rows, ne0, eps, (float *)op->data, ldy, c->stream);
        }
        case LM_GGML_OP_SCALE: {
            float v;
            std::memcpy(&v, op->op_params, sizeof(float));
            return chip_scale((const float *)a->data, lda, rows, ne0, v, (float *)op->data, ldy, c->stream);
        }
        case LM_GGML_OP_UNARY:
            if (op->op_params[0] == LM_GGML_UNARY_OP_GELU) {
                if (!ensure_gelu_table(c)) return CHIP_ENOMEM;
                return chip_gelu((const float *)a->data, lda, rows, ne0, c->gelu_table, (float *)op->data, ldy, c->stream);
            }
            return chip_silu((const float *)a->data, lda, rows, ne0, (float *)op->data, ldy, c->stream);
        default:
            as_rows(b, rb, ldb);
            return (op->op == LM_GGML_OP_ADD ? chip_add : chip_mul)((const float *)a->data, lda, (const float *)b->data, ldb, rb, rows,
                                                                 ne0, (float *)op->data, ldy, c->stream);
    }
}

// ---- the attention-side ops around the KV cache (SOFT_MAX, ROPE, CPY / CONT / DUP) ----
bool is_attn_side_op(int op) {
    return op == LM_GGML_OP_SOFT_MAX || op == LM_GGML_OP_ROPE || op == LM_GGML_OP_CPY || op == LM_GGML_OP_CONT || op == LM_GGML_OP_DUP ||
           op == LM_GGML_OP_GET_ROWS;
}
bool dense(const lm_ggml_tensor *t) {                   // lm_ggml_is_contiguous for the unquantized types
    size_t want = (t->type == LM_GGML_TYPE_F16) ? 2 : 4;
    for (int k = 0; k < LM_GGML_MAX_DIMS; k++) {
        if (t->ne[k] != 1 && t->nb[k] != want) return false;
        want *= (size_t)t->ne[k];
    }
    return true;
}
bool f32_or_f16(const lm_ggml_tensor *t) { return t->type == LM_GGML_TYPE_F32 || t->type == LM_GGML_TYPE_F16; }
int64_t n_elements(const lm_ggml_tensor *t) { return t->ne[0] * t->ne[1] * t->ne[2] * t->ne[3]; }

bool soft_max_shape_ok(const lm_ggml_tensor *op) {
    const lm_ggml_tensor *a = op->src[0], *m = op->src[1];
    if (!a || a->type != LM_GGML_TYPE_F32 || op->type != LM_GGML_TYPE_F32 || !dense(a) || !dense(op) || !same_shape(a, op)) return false;
    float max_bias;
    std::memcpy(&max_bias, (const float *)op->op_params + 1, sizeof(float));
    if (max_bias != 0.0f || a->ne[0] % 8 != 0 || a->ne[1] < 1) return false;            // no ALiBi; the AVX2 row tail
    if (m && (!f32_or_f16(m) || !dense(m) || m->ne[0] != a->ne[0] || m->ne[1] < a->ne[1] || m->ne[2] != 1 || m->ne[3] != 1)) return false;
    return true;
}
bool rope_shape_ok(const lm_ggml_tensor *op) {
    const lm_ggml_tensor *a = op->src[0], *pos = op->src[1], *ff = op->src[2];
    if (!a || !pos || a->type != LM_GGML_TYPE_F32 || op->type != LM_GGML_TYPE_F32 || !same_shape(a, op) || a->ne[3] != 1) return false;
    if (pos->type != LM_GGML_TYPE_I32 || pos->nb[0] != 4 || pos->ne[0] != a->ne[2]) return false;   // multi-section modes carry 4 * ne2 positions
    const int n_dims = op->op_params[1], mode = op->op_params[2];
    if ((mode != 0 && mode != 2) || n_dims <= 0 || (n_dims & 1) || n_dims > a->ne[0] || n_dims > 512) return false;
    if (ff && (ff->type != LM_GGML_TYPE_F32 || ff->nb[0] != 4 || ff->ne[0] < n_dims / 2)) return false;
    for (const lm_ggml_tensor *t : {a, (const lm_ggml_tensor *)op})
        if (t->nb[0] != 4 || t->nb[1] % 4 != 0 || t->nb[2] % 4 != 0 || t->nb[1] < (size_t)t->ne[0] * 4) return false;
    return true;
}
// CPY / CONT / DUP: node->data and node->nb are the destination's (for CPY the node is a view of src[1]).
bool cpy_shape_ok(const lm_ggml_tensor *op) {
    const lm_ggml_tensor *a = op->src[0];
    if (!a || !f32_or_f16(a) || !f32_or_f16(op) || n_elements(a) != n_elements(op)) return false;
    return true;                                       // shapes may differ: element i of one logical order to element i of the other
}
// GET_ROWS: a table that lives in a HIP buffer (any type the matmuls take, or F32), or an F32 / F16 activation.
bool get_rows_shape_ok(const lm_ggml_tensor *op) {
    const lm_ggml_tensor *a = op->src[0], *ids = op->src[1];
    if (!a || !ids || ids->type != LM_GGML_TYPE_I32 || op->type != LM_GGML_TYPE_F32) return false;
    const bool plain = a->type == LM_GGML_TYPE_F32 || a->type == LM_GGML_TYPE_F16;
    if (!plain && !chip_mul_mat_supported(a->type, 256)) return false;
    const lm_ggml_backend_buffer_t abuf = a->view_src ? a->view_src->buffer : a->buffer;
    if (abuf ? !is_hip_buffer(abuf) : !plain) return false;                   // a host-resident table stays with the CPU backend
    if (a->nb[0] != (plain ? (a->type == LM_GGML_TYPE_F16 ? 2u : 4u) : chip_block_bytes(a->type))) return false;
    if (!plain && a->ne[0] % chip_block_elems(a->type) != 0) return false;
    if (ids->nb[0] != 4 || ids->nb[1] % 4 != 0 || ids->nb[2] % 4 != 0 || ids->ne[3] != 1) return false;
    if (a->ne[2] != ids->ne[1] || a->ne[3] != ids->ne[2]) return false;       // the reference's batch rule (ne02 == ne11)
    if (op->nb[0] != 4 || op->nb[1] % 4 != 0 || op->nb[2] % 4 != 0 || op->nb[3] % 4 != 0 || op->nb[1] < (size_t)a->ne[0] * 4) return false;
    return op->ne[0] == a->ne[0] && op->ne[1] == ids->ne[0] && op->ne[2] == ids->ne[1] && op->ne[3] == ids->ne[2];
}
bool attn_side_shape_ok(const lm_ggml_tensor *op) {
    if (!elementwise_enabled()) return false;
    switch (op->op) {
        case LM_GGML_OP_SOFT_MAX: return soft_max_shape_ok(op);
        case LM_GGML_OP_ROPE:     return rope_shape_ok(op);
        case LM_GGML_OP_GET_ROWS: return get_rows_shape_ok(op);
        default:               return cpy_shape_ok(op);
    }
}
// store: the F32 -> F16 CPY of the RoPE's result into a dense destination (the K cache store), run in the RoPE's kernel
// The cos / sin table of a ROPE node (positions, frequency factors and parameters; built by the first node of a
// graph_compute call that needs it, kept until a node with another key comes): leaves it in c->rope_table.
int ensure_rope_table(backend_ctx *c, const lm_ggml_tensor *op) {
    const lm_ggml_tensor *a = op->src[0], *pos = op->src[1], *ff = op->src[2];
    float f[6];
    std::memcpy(f, op->op_params + 5, sizeof(f));        // freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow
    rope_table_key k = {pos->data, ff ? ff->data : nullptr, a->ne[2], {}, true};
    k.params[0] = op->op_params[1];
    std::memcpy(k.params + 1, op->op_params + 3, 8 * sizeof(int32_t));
    const size_t need = (size_t)a->ne[2] * (size_t)op->op_params[1] * sizeof(float);
    const bool have = c->rope_key.valid && c->rope_key.pos == k.pos && c->rope_key.ff == k.ff && c->rope_key.ne2 == k.ne2 &&
                      std::memcmp(c->rope_key.params, k.params, sizeof(k.params)) == 0;
    if (have) return CHIP_OK;
    if (need > c->rope_table_bytes) {
        chip_stream_synchronize(c->stream);          // earlier nodes of this call may still read the old table
        chip_free(c->rope_table);
        c->rope_table = nullptr;
        c->rope_table_bytes = 0;
        void *p = nullptr;
        if (chip_malloc(&p, need + need / 2) != CHIP_OK) return CHIP_ENOMEM;
        c->rope_table = (float *)p;
        c->rope_table_bytes = need + need / 2;
    }
    const int rc = chip_rope_table((const int32_t *)pos->data, ff ? (const float *)ff->data : nullptr, a->ne[2], op->op_params[1],
                                   op->op_params[4], f[0], f[1], f[2], f[3], f[4], f[5], c->rope_table, c->stream);
    if (rc != CHIP_OK) return rc;
    c->rope_key = k;
    g_rope_tables++;
    return CHIP_OK;
}

// A second ROPE node run in the first one's launch (K's with Q's): its input, the CPY of its result into the F16 cache that
// runs with it (or null), and whether its own F32 result is written at all.
struct rope_partner {
    const lm_ggml_tensor *op = nullptr;
    const void *src = nullptr;
    const lm_ggml_tensor *store = nullptr;
    int store_index = -1;
    bool write_f32 = true;
};
// src_at: where the ROPE's input really lies (a projection that ran early, into the backend's own memory)
int run_attn_side(backend_ctx *c, lm_ggml_tensor *op, const lm_ggml_tensor *store = nullptr, const void *src_at = nullptr,
                  const rope_partner *partner = nullptr) {
    const lm_ggml_tensor *a = op->src[0];
    switch (op->op) {
        case LM_GGML_OP_SOFT_MAX: {
            const lm_ggml_tensor *m = op->src[1];
            float scale, max_bias;
            std::memcpy(&scale, (const float *)op->op_params + 0, sizeof(float));
            std::memcpy(&max_bias, (const float *)op->op_params + 1, sizeof(float));
            return chip_soft_max((const float *)a->data, a->ne[0], m ? m->data : nullptr, m ? (int)m->type : (int)LM_GGML_TYPE_F32, a->ne[0],
                                 a->ne[1], a->ne[1] * a->ne[2] * a->ne[3], scale, max_bias, (float *)op->data, op->ne[0], c->stream);
        }
        case LM_GGML_OP_ROPE: {
            const lm_ggml_tensor *pos = op->src[1], *ff = op->src[2];
            const float *xa = (const float *)(src_at ? src_at : a->data);
            float f[6];
            std::memcpy(f, op->op_params + 5, sizeof(f));        // freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow
            if (fusion_enabled()) {
                if (const int trc = ensure_rope_table(c, op); trc != CHIP_OK) return trc;
                if (partner) {
                    const lm_ggml_tensor *pb = partner->op, *ab = pb->src[0];
                    chip_rope_operand oa = {xa, (int64_t)(a->nb[1] / 4), (int64_t)(a->nb[2] / 4), a->ne[1], (float *)op->data,
                                            (int64_t)(op->nb[1] / 4), (int64_t)(op->nb[2] / 4), store ? (uint16_t *)store->data : nullptr,
                                            a->ne[0], a->ne[0] * a->ne[1]};
                    chip_rope_operand ob = {(const float *)partner->src, (int64_t)(ab->nb[1] / 4), (int64_t)(ab->nb[2] / 4), ab->ne[1],
                                            partner->write_f32 ? (float *)pb->data : nullptr, (int64_t)(pb->nb[1] / 4),
                                            (int64_t)(pb->nb[2] / 4), partner->store ? (uint16_t *)partner->store->data : nullptr,
                                            ab->ne[0], ab->ne[0] * ab->ne[1]};
                    return chip_rope_apply_two(&oa, &ob, c->rope_table, a->ne[0], a->ne[2], op->op_params[1], op->op_params[2], c->stream);
                }
                if (store)
                    return chip_rope_apply_store(xa, (int64_t)(a->nb[1] / 4), (int64_t)(a->nb[2] / 4), c->rope_table,
                                                 a->ne[0], a->ne[1], a->ne[2], op->op_params[1], op->op_params[2], (float *)op->data,
                                                 (int64_t)(op->nb[1] / 4), (int64_t)(op->nb[2] / 4), (uint16_t *)store->data, a->ne[0],
                                                 a->ne[0] * a->ne[1], c->stream);
                return chip_rope_apply(xa, (int64_t)(a->nb[1] / 4), (int64_t)(a->nb[2] / 4), c->rope_table, a->ne[0],
                                       a->ne[1], a->ne[2], op->op_params[1], op->op_params[2], (float *)op->data,
                                       (int64_t)(op->nb[1] / 4), (int64_t)(op->nb[2] / 4), c->stream);
            }
            return chip_rope(xa, (int64_t)(a->nb[1] / 4), (int64_t)(a->nb[2] / 4), (const int32_t *)pos->data,
                             ff ? (const float *)ff->data : nullptr, a->ne[0], a->ne[1], a->ne[2], op->op_params[1], op->op_params[2],
                             op->op_params[4], f[0], f[1], f[2], f[3], f[4], f[5], (float *)op->data, (int64_t)(op->nb[1] / 4),
                             (int64_t)(op->nb[2] / 4), c->stream);
        }
        case LM_GGML_OP_GET_ROWS: {
            const lm_ggml_tensor *ids = op->src[1];
            return chip_get_rows(a->type, a->data, a->nb[1], a->nb[2], a->nb[3], a->ne[0], a->ne[1], (const int32_t *)ids->data, ids->ne[0],
                                 ids->ne[1], ids->ne[2], (int64_t)(ids->nb[1] / 4), (int64_t)(ids->nb[2] / 4), (float *)op->data,
                                 (int64_t)(op->nb[1] / 4), (int64_t)(op->nb[2] / 4), (int64_t)(op->nb[3] / 4), c->stream);
        }
        default: {
            int64_t nes[4], nbs[4], ned[4], nbd[4];
            for (int k = 0; k < 4; k++) { nes[k] = a->ne[k]; nbs[k] = (int64_t)a->nb[k]; ned[k] = op->ne[k]; nbd[k] = (int64_t)op->nb[k]; }
            return chip_cpy(a->data, a->type, nes, nbs, op->data, op->type, ned, nbd, c->stream);
        }
    }
}

static bool grow_workspace(backend_ctx *c, size_t need) {
    if (need <= c->workspace_size) return true;
    c->quantized.valid = false;
    chip_stream_synchronize(c->stream);
    chip_free(c->workspace);
    c->workspace = nullptr;
    c->workspace_size = 0;
    const size_t want = need + need / 4;
    if (chip_malloc(&c->workspace, want) != CHIP_OK) return false;
    c->workspace_size = want;
    return true;
}

// The first node (views aside) after index `last` when it is a quantized weight matmul of at least min_tokens tokens that
// reads `out`: the kernel in front of it can then leave the quantized rows in the workspace.  NULL otherwise.  A norm asks
// for more than 4 tokens (up to 4 the projections behind it quantize in their own prologue, in one launch for all of
// them); SiLU * up asks for 1: ffn_down's rows are long and its GEMV takes them ready-made at every token count.
const lm_ggml_tensor *quantized_consumer(const lm_ggml_cgraph *g, int last, const lm_ggml_tensor *out, int64_t min_tokens = 5) {
    int j = last + 1;
    while (j < g->n_nodes && is_view_op(g->nodes[j]->op)) j++;
    if (j >= g->n_nodes) return nullptr;
    const lm_ggml_tensor *mm = g->nodes[j];
    if (mm->op != LM_GGML_OP_MUL_MAT || mm->src[1] != out || !mul_mat_shape_ok(mm) || out->ne[1] < min_tokens) return nullptr;
    if (mm->src[0]->type == LM_GGML_TYPE_F16 || out->ne[2] != 1 || out->ne[3] != 1) return nullptr;
    return mm;
}
// Runs the norm (a [+ b -> sum]) [* w] -> out with the quantized rows going to the workspace when the next node is such a
// matmul; sets key to what the workspace then holds.  CHIP_EUNSUPPORTED: not done, the caller runs the plain kernel.
int norm_for_quantized_consumer(backend_ctx *c, const lm_ggml_cgraph *g, int last, const float *a, int64_t lda, const float *b,
                                int64_t ldb, float *sum, int64_t lds, int64_t rows, int64_t ne0, float eps, const float *w,
                                const lm_ggml_tensor *out, int64_t ldy, quantized_key &key) {
    const lm_ggml_tensor *mm = quantized_consumer(g, last, out);
    if (!mm) return CHIP_EUNSUPPORTED;
    const int wtype = mm->src[0]->type;
    if (!grow_workspace(c, chip_mul_mat_workspace_size_n(wtype, ne0, mm->src[0]->ne[1], rows))) return CHIP_EUNSUPPORTED;
    const int rc = chip_rms_norm_quantized(a, lda, b, ldb, sum, lds, rows, ne0, eps, w, (float *)out->data, ldy, wtype, c->workspace,
                                           c->workspace_size, c->stream);
    if (rc == CHIP_OK) {
        key = quantized_key{true, out->data, lm_ggml_nbytes(out), ne0, rows, ldy, chip_vec_dot_type(wtype)};
    }
    return rc;
}

// True when the workspace holds the quantized rows of x in the activation type that w's matmul reads.
bool have_rows(const quantized_key &q, const lm_ggml_tensor *x, const lm_ggml_tensor *w, int64_t n, int64_t ldx) {
    return q.valid && q.src == x->data && q.K == w->ne[0] && q.n == n && q.ldx == ldx && q.vec_dot_type == chip_vec_dot_type(w->type);
}

// silu(a) * b -> out, with the quantized rows going to the workspace when the next node is a quantized weight matmul that
// reads out (ffn_down); sets key to what the workspace then holds.
int silu_mul_for_consumer(backend_ctx *c, const lm_ggml_cgraph *g, int last, const float *a, int64_t lda, const float *b, int64_t ldb,
                          int64_t rows, int64_t ne0, const lm_ggml_tensor *out, int64_t ldy, quantized_key &key) {
    const lm_ggml_tensor *mm = fusion_enabled() ? quantized_consumer(g, last, out, 1) : nullptr;
    if (mm && grow_workspace(c, chip_mul_mat_workspace_size_n(mm->src[0]->type, ne0, mm->src[0]->ne[1], rows))) {
        const int wtype = mm->src[0]->type;
        const int rc = chip_silu_mul_quantized(a, lda, b, ldb, rows, ne0, (float *)out->data, ldy, wtype, c->workspace, c->workspace_size,
                                               c->stream);
        if (rc == CHIP_OK) key = quantized_key{true, out->data, lm_ggml_nbytes(out), ne0, rows, ldy, chip_vec_dot_type(wtype)};
        if (rc != CHIP_EUNSUPPORTED) return rc;
    }
    return chip_silu_mul(a, lda, b, ldb, rows, ne0, (float *)out->data, ldy, c->stream);
}

// RMS_NORM or SILU directly followed by the MUL that consumes it, the MUL written over the first node's output: the
// allocator reuses a node's memory for its consumer only when nothing else reads it (reference ggml-alloc.c in-place
// rule: one child, no views), so the first node's own result is not needed and the pair runs as one kernel.
// Returns CHIP_OK and sets fused, or leaves fused false.
struct held_norm;
bool norm_can_wait(const lm_ggml_cgraph *g, int mul_index, const lm_ggml_tensor *a, const lm_ggml_tensor *mul, const lm_ggml_tensor *wt);
int try_fused_pair(backend_ctx *c, const lm_ggml_cgraph *g, int i, const lm_ggml_tensor *node, const lm_ggml_tensor *next, bool &fused,
                   quantized_key &key, bool &held) {
    fused = false;
    held = false;
    if (!next || next->op != LM_GGML_OP_MUL || next->data != node->data || !elementwise_shape_ok(next)) return CHIP_OK;
    const lm_ggml_tensor *other = next->src[0] == node ? next->src[1] : (next->src[1] == node ? next->src[0] : nullptr);
    if (!other || other == node || !same_shape(next, node)) return CHIP_OK;
    const lm_ggml_tensor *a = node->src[0];
    int64_t rows, lda, ldy, rb, ldb;
    if (!as_rows(a, rows, lda) || !as_rows(next, rows, ldy) || !as_rows(other, rb, ldb)) return CHIP_OK;
    if (node->op == LM_GGML_OP_RMS_NORM) {
        if (rb != 1) return CHIP_OK;                                       // the norm weight: one row
        float eps;
        std::memcpy(&eps, node->op_params, sizeof(float));
        fused = true;
        if (norm_can_wait(g, i + 1, a, next, other)) {                     // the projections behind the MUL run the pair
            held = true;
            return CHIP_OK;
        }
        if (const int rc = norm_for_quantized_consumer(c, g, i + 1, (const float *)a->data, lda, nullptr, 0, nullptr, 0, rows, a->ne[0], eps,
                                                       (const float *)other->data, next, ldy, key);
            rc != CHIP_EUNSUPPORTED)
            return rc;
        return chip_rms_norm_mul((const float *)a->data, lda, rows, a->ne[0], eps, (const float *)other->data, nullptr, 0,
                                 (float *)next->data, ldy, c->stream);
    }
    if (node->op == LM_GGML_OP_UNARY && node->op_params[0] == LM_GGML_UNARY_OP_SILU) {
        if (!same_shape(other, node)) return CHIP_OK;
        fused = true;
        return silu_mul_for_consumer(c, g, i + 1, (const float *)a->data, lda, (const float *)other->data, ldb, rows, a->ne[0], next, ldy, key);
    }
    return CHIP_OK;
}

// Row blocks [p, p + rows * ld) of two tensors: the same block, or no element in common.
bool same_or_disjoint(const void *p, int64_t ldp, const void *q, int64_t ldq, int64_t rows, int64_t ne0) {
    if (p == q) return ldp == ldq;
    const uintptr_t a = (uintptr_t)p, b = (uintptr_t)q;
    const uintptr_t ea = a + (uintptr_t)(((rows - 1) * ldp + ne0) * 4), eb = b + (uintptr_t)(((rows - 1) * ldq + ne0) * 4);
    return ea <= b || eb <= a;
}

// A residual ADD directly followed by the RMS_NORM of its result (and that, as above, by the MUL with the norm weight):
// the sum is still written, since the next residual reads it, but the norm reads it back in the same kernel. The
// allocator may have placed any of the outputs over a dead operand, so every output block is the same block as, or
// apart from, every block read. Sets used to the number of nodes run (0: not this pattern).
int try_fused_add_norm(backend_ctx *c, const lm_ggml_cgraph *g, int i, int &used, quantized_key &key) {
    used = 0;
    const lm_ggml_tensor *add = g->nodes[i];
    const lm_ggml_tensor *norm = i + 1 < g->n_nodes ? g->nodes[i + 1] : nullptr;
    if (!norm || norm->op != LM_GGML_OP_RMS_NORM || norm->src[0] != add || !elementwise_shape_ok(norm)) return CHIP_OK;
    const lm_ggml_tensor *a = add->src[0], *b = add->src[1];
    if (!same_shape(a, b)) return CHIP_OK;
    const lm_ggml_tensor *mul = i + 2 < g->n_nodes ? g->nodes[i + 2] : nullptr, *wt = nullptr;
    if (mul && mul->op == LM_GGML_OP_MUL && mul->data == norm->data && elementwise_shape_ok(mul) && same_shape(mul, norm)) {
        wt = mul->src[0] == norm ? mul->src[1] : (mul->src[1] == norm ? mul->src[0] : nullptr);
        int64_t rw, ldw;
        if (!wt || wt == norm || !as_rows(wt, rw, ldw) || rw != 1) wt = nullptr;
    }
    const lm_ggml_tensor *out = wt ? mul : norm;
    int64_t rows, lda, ldb, lds, ldy;
    if (!as_rows(a, rows, lda) || !as_rows(b, rows, ldb) || !as_rows(add, rows, lds) || !as_rows(out, rows, ldy)) return CHIP_OK;
    const int64_t ne0 = a->ne[0];
    if (rows == 0 || ne0 == 0) return CHIP_OK;
    if (!same_or_disjoint(add->data, lds, a->data, lda, rows, ne0) || !same_or_disjoint(add->data, lds, b->data, ldb, rows, ne0) ||
        !same_or_disjoint(out->data, ldy, a->data, lda, rows, ne0) || !same_or_disjoint(out->data, ldy, b->data, ldb, rows, ne0) ||
        out->data == add->data || !same_or_disjoint(out->data, ldy, add->data, lds, rows, ne0))
        return CHIP_OK;
    if (wt && !same_or_disjoint(out->data, ldy, wt->data, ne0, 1, ne0)) return CHIP_OK;
    if (wt && out->data == wt->data) return CHIP_OK;
    float eps;
    std::memcpy(&eps, norm->op_params, sizeof(float));
    used = wt ? 3 : 2;
    if (const int rc = norm_for_quantized_consumer(c, g, i + used - 1, (const float *)a->data, lda, (const float *)b->data, ldb,
                                                   (float *)add->data, lds, rows, ne0, eps, wt ? (const float *)wt->data : nullptr, out,
                                                   ldy, key);
        rc != CHIP_EUNSUPPORTED)
        return rc;
    return chip_add_rms_norm_mul((const float *)a->data, lda, (const float *)b->data, ldb, (float *)add->data, lds, rows, ne0, eps,
                                 wt ? (const float *)wt->data : nullptr, (float *)out->data, ldy, c->stream);
}

bool disjoint(const lm_ggml_tensor *p, const lm_ggml_tensor *q) {
    const uintptr_t a = (uintptr_t)p->data, b = (uintptr_t)q->data;
    return a + lm_ggml_nbytes(p) <= b || b + lm_ggml_nbytes(q) <= a;
}

// The gated FFN in llama.cpp's node order: gate matmul, SILU, up matmul, MUL(silu, up) (reference llama-graph.cpp:562-690;
// the up projection is the MUL's second operand and is visited after the first). When the matmul between the two
// writes nothing the SILU reads, the SILU can wait for it and run inside the MUL's kernel. True: silu is to be skipped
// now and nodes[i + 2] run as chip_silu_mul.
bool silu_can_wait_for_its_mul(const lm_ggml_cgraph *g, int i) {
    const lm_ggml_tensor *silu = g->nodes[i];
    if (i + 2 >= g->n_nodes) return false;
    const lm_ggml_tensor *mm = g->nodes[i + 1], *mul = g->nodes[i + 2];
    if (mm->op != LM_GGML_OP_MUL_MAT || !mul_mat_shape_ok(mm) || mm->src[0] == silu || mm->src[1] == silu) return false;
    if (mul->op != LM_GGML_OP_MUL || mul->data != silu->data || !elementwise_shape_ok(mul) || !same_shape(mul, silu)) return false;
    const lm_ggml_tensor *other = mul->src[0] == silu ? mul->src[1] : (mul->src[1] == silu ? mul->src[0] : nullptr);
    int64_t r, ld;
    if (!other || other == silu || !same_shape(other, silu) || !as_rows(other, r, ld)) return false;
    return disjoint(mm, silu->src[0]) && disjoint(mm, silu);
}

// A cache store that is run early, inside the kernel that produces what it stores.  The reference builds q, k, v of a layer
// first and the two stores after them (llama-graph.cpp:1265-1277), so between a producer and its CPY lie views, the
// projections of the other tensors and the other store.  Running the CPY at the producer's place is safe when none of
// the nodes in between reads or writes the destination region.  Finds, within the next STORE_LOOKAHEAD nodes after i, the
// CPY node that `wanted` accepts; -1 if there is none or a node in between touches its destination.
constexpr int STORE_LOOKAHEAD = 16;
bool ranges_apart(const lm_ggml_tensor *p, const lm_ggml_tensor *q) {
    if (!p->data || !q->data) return true;            // no memory behind it (an unallocated leaf cannot alias the destination)
    return disjoint(p, q);
}
template <typename F>
int early_store_index(const lm_ggml_cgraph *g, int i, F wanted, int run_at = -1) {
    // run_at: the node at whose place the producer i itself runs (a projection grouped with an earlier one); the
    // destination must stay untouched from there on
    const int first = (run_at >= 0 ? run_at : i) + 1;
    const int end = i + 1 + STORE_LOOKAHEAD < g->n_nodes ? i + 1 + STORE_LOOKAHEAD : g->n_nodes;
    for (int j = i + 1; j < end; j++) {
        const lm_ggml_tensor *cp = g->nodes[j];
        if (cp->op != LM_GGML_OP_CPY || !wanted(cp)) continue;
        for (int m = first; m < j; m++) {
            if (m == i) continue;
            const lm_ggml_tensor *t = g->nodes[m];
            if (is_view_op(t->op)) continue;
            if (!ranges_apart(t, cp)) return -1;
            for (int k = 0; k < LM_GGML_MAX_SRC; k++)
                if (t->src[k] && !ranges_apart(t->src[k], cp)) return -1;
        }
        return j;
    }
    return -1;
}

// The RoPE of K and the CPY of its result into the F16 cache (reference llama-kv-cache.cpp cpy_k: a dense 1-D view of the
// cache): index of that CPY node, or -1.  The RoPE still writes its own F32 result.
int rope_store_index(const lm_ggml_cgraph *g, int i, int run_at = -1) {
    const lm_ggml_tensor *rope = g->nodes[i];
    if (rope->type != LM_GGML_TYPE_F32 || !dense(rope)) return -1;
    return early_store_index(g, i, [rope](const lm_ggml_tensor *cp) {
        return cp->src[0] == rope && cp->type == LM_GGML_TYPE_F16 && attn_side_shape_ok(cp) && dense(cp) &&
               n_elements(cp) == n_elements(rope) && disjoint(cp, rope) && disjoint(cp, rope->src[0]);
    }, run_at);
}

// ffn_gate and ffn_up in llama.cpp's node order: gate matmul, SILU, up matmul, MUL.  With up to 4 tokens the two matmuls
// (same activation tensor, weight type and shape) run as one launch when the SILU between them is one that waits for
// its MUL anyway and the up projection's output overlaps nothing that is read before its own node: the activation, the
// gate's output (which the SILU reads) and the SILU's output.  Index of the up matmul, or -1.
int paired_matmul_index(const lm_ggml_cgraph *g, int i) {
    if (i + 3 >= g->n_nodes) return -1;
    const lm_ggml_tensor *gate = g->nodes[i], *silu = g->nodes[i + 1], *up = g->nodes[i + 2];
    if (silu->op != LM_GGML_OP_UNARY || silu->op_params[0] != LM_GGML_UNARY_OP_SILU || silu->src[0] != gate) return -1;
    if (!elementwise_shape_ok(silu) || !silu_can_wait_for_its_mul(g, i + 1)) return -1;
    if (up->op != LM_GGML_OP_MUL_MAT || !mul_mat_shape_ok(up) || up->src[1] != gate->src[1]) return -1;
    const lm_ggml_tensor *wg = gate->src[0], *wu = up->src[0], *x = gate->src[1];
    if (x->ne[1] > 4 || wg->type != wu->type || wg->ne[0] != wu->ne[0] || wg->ne[1] != wu->ne[1] || wg->nb[1] != wu->nb[1]) return -1;
    if (up->nb[1] != gate->nb[1]) return -1;
    if (!disjoint(up, x) || !disjoint(up, gate) || !disjoint(up, silu)) return -1;
    return i + 2;
}

// The V projection followed (views aside) by the CPY of its transpose into the transposed F16 V cache (reference
// llama-kv-cache.cpp cpy_v without flash attention: dst is a 2-D view [n_tokens, n_embd_v] with rows kv_size apart).
// Index of that CPY node, or -1.  The matmul still writes its own F32 result.
int transposed_store_index(const lm_ggml_cgraph *g, int i, int run_at = -1) {
    const lm_ggml_tensor *mm = g->nodes[i];
    const int64_t N = mm->ne[0], n = mm->ne[1];
    return early_store_index(g, i, [mm, N, n](const lm_ggml_tensor *cp) {
        // the source: a TRANSPOSE of the projection's result (through reshapes: views collapse onto the tensor that owns the memory)
        const lm_ggml_tensor *tr = cp->src[0];
        if (!tr || tr->op != LM_GGML_OP_TRANSPOSE || (tr->view_src != mm && tr->src[0] != mm) || tr->view_offs != 0) return false;
        if (tr->ne[0] != n || tr->ne[1] != N || tr->ne[2] != 1 || tr->ne[3] != 1 || tr->nb[0] != mm->nb[1] || tr->nb[1] != mm->nb[0]) return false;
        if (cp->type != LM_GGML_TYPE_F16 || cp->ne[0] != n || cp->ne[1] != N || cp->ne[2] != 1 || cp->ne[3] != 1 || cp->nb[0] != 2 ||
            cp->nb[1] % 2 != 0 || cp->nb[1] < (size_t)n * 2)
            return false;
        if (!is_hip_buffer(cp->view_src ? cp->view_src->buffer : cp->buffer)) return false;
        return disjoint(cp, mm) && disjoint(cp, mm->src[1]);
    }, run_at);
}

// The projections of one activation tensor (llama.cpp builds Qcur, its RoPE, Kcur, its RoPE, Vcur, ... from the same
// normed input: llama-model.cpp build_llama): MUL_MAT nodes within the next GROUP_LOOKAHEAD nodes after i that read the
// same src[1] as node i and share its activation format.  Such a node may run at node i's place when nothing between the
// two reads or writes the memory of its result (the allocator may have given it the place of a tensor that dies in
// between, Qcur's for instance once its RoPE has read it).  Fills members[] (node i first) and returns their number.
constexpr int GROUP_LOOKAHEAD = 12;
// aliased[k]: member k's own memory is in use between node i and its node (the allocator gave it the place of a tensor that
// dies in between: Kcur over Qcur, once Qcur's RoPE has read it and written elsewhere).  Such a member can still run at
// node i when its result goes to memory of the backend's own; what happens to it then is the caller's business.
int grouped_matmuls(const lm_ggml_cgraph *g, int i, int *members, bool *aliased) {
    const lm_ggml_tensor *first = g->nodes[i], *x = first->src[1];
    const int vt = chip_vec_dot_type(first->src[0]->type);
    int count = 0;
    aliased[count] = false;
    members[count++] = i;
    const int end = i + 1 + GROUP_LOOKAHEAD < g->n_nodes ? i + 1 + GROUP_LOOKAHEAD : g->n_nodes;
    for (int j = i + 1; j < end && count < CHIP_GROUP_MAX; j++) {
        const lm_ggml_tensor *mm = g->nodes[j];
        if (mm->op != LM_GGML_OP_MUL_MAT || mm->src[1] != x || !mul_mat_shape_ok(mm)) continue;
        if (chip_vec_dot_type(mm->src[0]->type) != vt) continue;
        bool safe = disjoint(mm, x);
        for (int m = i; m < j && safe; m++) {
            const lm_ggml_tensor *t = g->nodes[m];
            if (is_view_op(t->op)) continue;
            if (!ranges_apart(t, mm)) safe = false;
            for (int k = 0; k < LM_GGML_MAX_SRC && safe; k++)
                if (t->src[k] && !ranges_apart(t->src[k], mm)) safe = false;
        }
        aliased[count] = !safe;
        members[count++] = j;
    }
    return count;
}

// The tensors the graph's nodes read, views resolved to the tensor that owns the memory: built once per graph_compute,
// when the first question about a tensor's readers comes up.
struct graph_reads {
    std::vector<const lm_ggml_tensor *> owner;       // one entry per (computing node, operand)
    bool built = false;
    void build(const lm_ggml_cgraph *g) {
        owner.clear();
        for (int k = 0; k < g->n_nodes; k++) {
            const lm_ggml_tensor *nd = g->nodes[k];
            if (is_view_op(nd->op)) continue;
            for (int m = 0; m < LM_GGML_MAX_SRC; m++)
                if (const lm_ggml_tensor *sr = nd->src[m]) owner.push_back(sr->view_src ? sr->view_src : sr);
        }
        built = true;
    }
    int readers_of(const lm_ggml_cgraph *g, const lm_ggml_tensor *t) {
        if (!built) build(g);
        int n = 0;
        for (const lm_ggml_tensor *o : owner) n += o == t;
        return n;
    }
};
bool grow_group_scratch(backend_ctx *c, size_t slot_bytes) {
    if (slot_bytes <= c->group_slot_bytes) return true;
    chip_stream_synchronize(c->stream);                  // earlier nodes of this call may still use the old slots
    chip_free(c->group_scratch);
    c->group_scratch = nullptr;
    c->group_slot_bytes = 0;
    void *p = nullptr;
    const size_t want = (slot_bytes + slot_bytes / 2 + 255) & ~(size_t)255;
    if (chip_malloc(&p, want * CHIP_GROUP_MAX) != CHIP_OK) return false;
    c->group_scratch = (float *)p;
    c->group_slot_bytes = want;
    return true;
}

// The kqv matmul and the node that follows it (views aside) in build_attn_mha, CONT(PERMUTE(kqv, 0, 2, 1, 3)) (reference
// llama-graph.cpp:1154-1158): with up to 4 (query head, token) pairs per KV head the matmul's kernel also writes the merged
// layout.  Index of that CONT node, or -1.  The kernel writes both copies while workgroups still read its inputs: the CONT's
// memory must lie apart from them and from the matmul's own result, whatever the allocator reused.
int next_compute_node(const lm_ggml_cgraph *g, int i) {
    for (int j = i + 1; j < g->n_nodes; j++)
        if (!is_view_op(g->nodes[j]->op)) return j;
    return -1;
}
int head_merge_index(const lm_ggml_cgraph *g, int i) {
    const lm_ggml_tensor *kqv = g->nodes[i], *v = kqv->src[0], *p = kqv->src[1];
    const int64_t hd = kqv->ne[0], n = kqv->ne[1], n_head = kqv->ne[2];
    if (!chip_mul_mat_f16_batched_second_copy_supported(v->ne[2], n_head, n)) return -1;
    const int j = next_compute_node(g, i);
    if (j < 0) return -1;
    const lm_ggml_tensor *ct = g->nodes[j], *pm = ct->src[0];
    if (ct->op != LM_GGML_OP_CONT || ct->type != LM_GGML_TYPE_F32 || !pm || pm->op != LM_GGML_OP_PERMUTE || pm->src[0] != kqv ||
        pm->view_src != kqv || pm->view_offs != 0 || !dense(ct) || n_elements(ct) != hd * n_head * n)
        return -1;
    // the permuted view: [hd, n_head, n] with kqv's strides of dimensions 0, 2, 1
    if (pm->ne[0] != hd || pm->ne[1] != n_head || pm->ne[2] != n || pm->ne[3] != 1 || pm->nb[0] != 4 || pm->nb[1] != kqv->nb[2] ||
        pm->nb[2] != kqv->nb[1])
        return -1;
    for (const lm_ggml_tensor *in : {v, p, kqv})
        if (!ranges_apart(in, ct)) return -1;
    return j;
}

// Q's and K's ROPE of a layer (same positions, parameters, head size and token count) in one launch: index of a later ROPE
// node that may run at node i's place, or -1.  Its input must be there already: the result of a projection that ran early
// with node i's own (ran_early says where it lies).  Its F32 result is written early only if nothing in between touches
// that memory; when the cache store that runs with it is its only reader, it is not written at all.
constexpr int ROPE_LOOKAHEAD = 8;
template <typename F>
int rope_partner_index(const lm_ggml_cgraph *g, int i, graph_reads &reads, F ran_early, rope_partner &out) {
    const lm_ggml_tensor *first = g->nodes[i];
    const int end = i + 1 + ROPE_LOOKAHEAD < g->n_nodes ? i + 1 + ROPE_LOOKAHEAD : g->n_nodes;
    for (int j = i + 1; j < end; j++) {
        const lm_ggml_tensor *rp = g->nodes[j];
        if (rp->op != LM_GGML_OP_ROPE) continue;
        const lm_ggml_tensor *in = rp->src[0];
        if (!attn_side_shape_ok(rp) || rp->src[1] != first->src[1] || rp->src[2] != first->src[2] ||
            std::memcmp(rp->op_params, first->op_params, sizeof(rp->op_params)) != 0 || rp->ne[0] != first->ne[0] || rp->ne[2] != first->ne[2])
            return -1;
        const lm_ggml_tensor *owner = in->view_src ? in->view_src : in;
        const void *at = ran_early(owner);
        if (!at) return -1;
        out.op = rp;
        out.src = (const uint8_t *)at + ((const uint8_t *)in->data - (const uint8_t *)owner->data);
        const int st = rope_store_index(g, j, i);
        out.store = st >= 0 ? g->nodes[st] : nullptr;
        out.store_index = st;
        out.write_f32 = !(out.store && !(rp->flags & LM_GGML_TENSOR_FLAG_OUTPUT) && reads.readers_of(g, rp) == 1);
        if (out.write_f32) {
            for (int m = i; m < j; m++) {                // its memory may still belong to someone between the two nodes
                const lm_ggml_tensor *t = g->nodes[m];
                if (is_view_op(t->op)) continue;
                if (!ranges_apart(t, rp)) return -1;
                for (int k = 0; k < LM_GGML_MAX_SRC; k++)
                    if (t->src[k] && !ranges_apart(t->src[k], rp)) return -1;
            }
        }
        return j;
    }
    return -1;
}

// The residual ADD behind a projection (reference cactus/llama-model.cpp build_llama: ffn_inp = lm_ggml_add(cur, inpSA) after wo,
// cur = lm_ggml_add(cur, ffn_inp) after ffn_down), to be run where the projection's GEMV stores its result (chip_mul_mat_add):
// the next computing node, adding a tensor of the projection's shape to it; nothing else reads the projection; the sum's
// rows lie apart from the projection's input and are the other operand's rows or apart from them.  Returns its index or -1.
int residual_add_index(const lm_ggml_cgraph *g, int i, graph_reads &reads) {
    const lm_ggml_tensor *mm = g->nodes[i], *w = mm->src[0], *x = mm->src[1];
    const int j = next_compute_node(g, i);
    if (j < 0 || (mm->flags & LM_GGML_TENSOR_FLAG_OUTPUT)) return -1;
    const lm_ggml_tensor *add = g->nodes[j];
    if (add->op != LM_GGML_OP_ADD || !elementwise_shape_ok(add)) return -1;
    const lm_ggml_tensor *other = add->src[0] == mm ? add->src[1] : (add->src[1] == mm ? add->src[0] : nullptr);
    if (!other || other == mm || !same_shape(other, mm) || !same_shape(add, mm) || reads.readers_of(g, mm) != 1) return -1;
    int64_t rows, ldo, lda;
    if (!as_rows(other, rows, ldo) || !as_rows(add, rows, lda) || rows != x->ne[1] || !other->data) return -1;
    if (!chip_mul_mat_add_supported(w->type, w->ne[0], w->ne[1], rows)) return -1;
    if (!ranges_apart(add, x) || !same_or_disjoint(add->data, lda, other->data, ldo, rows, mm->ne[0])) return -1;
    return j;
}

// An RMS_NORM and the MUL with its weight held back for the projections that read the result: they run the two nodes in
// their prologue (chip_mul_mat_group_rope_norm, chip_mul_mat_pair_silu_mul_norm).  src: the norm's input, out: the MUL node.
struct held_norm {
    const lm_ggml_tensor *src = nullptr, *out = nullptr, *weight = nullptr;
    float eps = 0.f;
    bool held() const { return out != nullptr; }
};
// True when the norm of `a` (RMS_NORM node, then `mul` with the one-row weight `wt`) may wait for the node after the MUL: up
// to 4 tokens, that node a weight matmul of the MUL's result with a prologue that takes the norm, and the norm's input still
// whole when that matmul runs (the MUL's rows lie apart from it).
bool norm_can_wait(const lm_ggml_cgraph *g, int mul_index, const lm_ggml_tensor *a, const lm_ggml_tensor *mul, const lm_ggml_tensor *wt) {
    const int j = next_compute_node(g, mul_index);
    if (j < 0 || (mul->flags & LM_GGML_TENSOR_FLAG_OUTPUT)) return false;
    const lm_ggml_tensor *mm = g->nodes[j];
    if (mm->op != LM_GGML_OP_MUL_MAT || mm->src[1] != mul || !mul_mat_shape_ok(mm)) return false;
    const int64_t n = mul->ne[1];
    // up to 2 tokens: at 4 every workgroup of the projection repeats four rows' norm, which costs more than the norm's own launch
    // (ffn_norm + gated FFN of 2 x 14336 x 4096 Q4_K: 27.9 us in one launch against 26.1 us in two; 2 tokens 18.3 against 19.4,
    // one token 14.4 against 16.9)
    if (mul->ne[2] != 1 || mul->ne[3] != 1 || n > 2 || !chip_norm_before_supported(mm->src[0]->type, mul->ne[0], n)) return false;
    if (((uintptr_t)wt->data & 15) != 0 || ((uintptr_t)mul->data & 15) != 0 || (mul->nb[1] % 16) != 0) return false;
    return ranges_apart(a, mul) && ranges_apart(wt, mul);
}

// The ROPE node behind a projection that runs in a group at node i, to be run in that projection's epilogue
// (chip_mul_mat_group_rope): the projection is read by nothing else, its rows are the ROPE's heads as they lie, and whatever
// the ROPE writes at node i's place is not in use there.  Returns the ROPE's index and fills rope (the table pointer is left
// to the caller), store_index (the cache store that runs with it, or -1); -1: no such node.
int rope_epilogue_index(const lm_ggml_cgraph *g, int i, int member, int64_t n, graph_reads &reads, chip_rope_after &rope, int &store_index) {
    const lm_ggml_tensor *mm = g->nodes[member];
    const int nx = next_compute_node(g, member);
    if (nx < 0 || nx > member + ROPE_LOOKAHEAD) return -1;
    const lm_ggml_tensor *rp = g->nodes[nx], *in = rp->src[0];
    if (rp->op != LM_GGML_OP_ROPE || !in || !attn_side_shape_ok(rp) || (mm->flags & LM_GGML_TENSOR_FLAG_OUTPUT)) return -1;
    if ((in != mm && in->view_src != mm) || in->data != mm->data || reads.readers_of(g, mm) != 1) return -1;
    const int64_t hd = in->ne[0], N = mm->ne[0];
    if (hd <= 0 || (hd & 1) || in->ne[1] * hd != N || in->ne[2] != n || in->ne[3] != 1 || mm->nb[1] != (size_t)N * 4) return -1;
    if (in->nb[1] != (size_t)hd * 4 || in->nb[2] != (size_t)N * 4 || rp->nb[1] != (size_t)hd * 4 || rp->nb[2] != (size_t)N * 4) return -1;
    store_index = rope_store_index(g, nx, i);
    const lm_ggml_tensor *store = store_index >= 0 ? g->nodes[store_index] : nullptr;
    const bool write_f32 = !(store && !(rp->flags & LM_GGML_TENSOR_FLAG_OUTPUT) && reads.readers_of(g, rp) == 1);
    if (write_f32) {
        for (int m = i; m < nx; m++) {                       // the ROPE's own memory, between node i and its node
            const lm_ggml_tensor *t = g->nodes[m];
            if (is_view_op(t->op) || t == mm) continue;      // (over the projection it replaces it may lie: that is not stored)
            if (!ranges_apart(t, rp)) return -1;
            for (int k = 0; k < LM_GGML_MAX_SRC; k++) {
                const lm_ggml_tensor *sr = t->src[k];
                if (sr && sr != mm && sr->view_src != mm && !ranges_apart(sr, rp)) return -1;
            }
        }
    }
    rope = chip_rope_after{nullptr, hd, rp->op_params[1], rp->op_params[2], write_f32 ? (float *)rp->data : nullptr, N,
                           store ? (uint16_t *)store->data : nullptr, N};
    return nx;
}

int backend_graph_compute(lm_ggml_backend_t backend, lm_ggml_cgraph *cgraph) {
    backend_ctx *c = (backend_ctx *)backend->context;
    c->rope_key.valid = false;                        // positions may have changed since the last call
    c->quantized.valid = false;                       // and so may any activation
    const lm_ggml_tensor *waiting_silu = nullptr;     // a SILU held back for the MUL two nodes on
    int stored_early[4] = {-1, -1, -1, -1};           // CPY nodes that already ran inside the RoPE / the projection before them
    auto remember_store = [&stored_early](int j) {
        for (int &slot : stored_early)
            if (slot < 0) { slot = j; return true; }
        return false;
    };
    int paired_matmul = -1;                           // index of an up projection that ran with its gate projection
    int grouped[CHIP_GROUP_MAX] = {-1, -1, -1, -1};   // projections that already ran with an earlier one of the same input
    const float *grouped_copy[CHIP_GROUP_MAX] = {nullptr, nullptr, nullptr, nullptr};   // ... into a scratch slot, still to be copied to their place
    int rope_from_slot = -1, rope_from_slot_owner = -1;   // a ROPE node whose input lies in a scratch slot instead, and the projection's node
    const float *rope_slot_src = nullptr;
    graph_reads reads;
    int rope_done = -1, rope_done_store = -1;         // a ROPE node (and its cache store) that already ran in an earlier ROPE's launch
    int roped_early[CHIP_GROUP_MAX] = {-1, -1, -1, -1};   // ROPE nodes that ran in the epilogue of their projection
    int add_done = -1;                                // a residual ADD that ran in the store of the projection before it
    held_norm held;                                   // a norm and its weight MUL waiting for the projections that read them
    // the held norm as a kernel of its own after all: the matmul that was to run it took a path without that prologue
    auto run_held_norm = [&]() -> int {
        if (!held.held()) return CHIP_OK;
        const lm_ggml_tensor *a = held.src, *out = held.out;
        held.out = nullptr;
        return chip_rms_norm_mul((const float *)a->data, (int64_t)(a->nb[1] / 4), out->ne[1], a->ne[0], held.eps, (const float *)held.weight->data,
                                 nullptr, 0, (float *)out->data, (int64_t)(out->nb[1] / 4), c->stream);
    };
    for (int i = 0; i < cgraph->n_nodes; i++) {
        lm_ggml_tensor *node = cgraph->nodes[i];
        if (is_view_op(node->op)) continue;
        if (held.held() && !(node->op == LM_GGML_OP_MUL_MAT && node->src[1] == held.out)) {
            if (const int rc = run_held_norm(); rc != CHIP_OK) {
                HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: RMS_NORM held for %s failed: %s\n", __func__, node->name, chip_error_string(rc));
                return LM_GGML_STATUS_FAILED;
            }
        }
        if (i == add_done) { add_done = -1; continue; }
        // a node that writes into the tensor the workspace was quantized from, or that uses the workspace itself, ends
        // the reuse of the quantized rows (every node is seen here, also those run inside a neighbour's kernel)
        auto writes = [c](const lm_ggml_tensor *t) {
            drop_planes(hip_buffer_ctx_of(t), t->data, lm_ggml_nbytes(t));
            if (!c->quantized.valid) return;
            const uintptr_t a = (uintptr_t)t->data, b = (uintptr_t)c->quantized.src;
            const bool apart = a + lm_ggml_nbytes(t) <= b || b + c->quantized.src_bytes <= a;
            if (!apart || t->op == LM_GGML_OP_MUL_MAT_ID || (t->op == LM_GGML_OP_MUL_MAT && !mul_mat_shape_ok(t))) c->quantized.valid = false;
        };
        writes(node);
        if (waiting_silu && node->op == LM_GGML_OP_MUL) {
            const lm_ggml_tensor *silu = waiting_silu, *other = node->src[0] == silu ? node->src[1] : node->src[0];
            waiting_silu = nullptr;
            int64_t rows, lda, ldb, ldy;
            as_rows(silu->src[0], rows, lda);
            as_rows(other, rows, ldb);
            as_rows(node, rows, ldy);
            quantized_key key;
            const int rc = silu_mul_for_consumer(c, cgraph, i, (const float *)silu->src[0]->data, lda, (const float *)other->data, ldb, rows,
                                                 silu->ne[0], node, ldy, key);
            if (key.valid) c->quantized = key;
            if (rc != CHIP_OK) {
                HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: %s (SILU run with its MUL) failed: %s\n", __func__, node->name, chip_error_string(rc));
                return LM_GGML_STATUS_FAILED;
            }
            g_elementwise_nodes += 2;
            g_fused_pairs++;
            continue;
        }
        if (node->op == LM_GGML_OP_ADD && elementwise_shape_ok(node) && fusion_enabled()) {
            int used = 0;
            quantized_key key;
            const int rc = try_fused_add_norm(c, cgraph, i, used, key);
            if (rc != CHIP_OK) {
                HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: %s (ADD fused with the norm that follows) failed: %s\n", __func__, node->name,
                        chip_error_string(rc));
                return LM_GGML_STATUS_FAILED;
            }
            if (used) {
                for (int k = 1; k < used; k++) writes(cgraph->nodes[i + k]);
                if (key.valid) c->quantized = key;      // after the group's own writes: the workspace holds the group's result
                g_elementwise_nodes += used;
                g_fused_pairs += used - 1;
                i += used - 1;
                continue;
            }
        }
        if ((node->op == LM_GGML_OP_RMS_NORM || (node->op == LM_GGML_OP_UNARY && node->op_params[0] == LM_GGML_UNARY_OP_SILU)) &&
            elementwise_shape_ok(node) && fusion_enabled()) {
            bool fused = false, waits = false;
            quantized_key key;
            const int rc = try_fused_pair(c, cgraph, i, node, i + 1 < cgraph->n_nodes ? cgraph->nodes[i + 1] : nullptr, fused, key, waits);
            if (rc != CHIP_OK) {
                HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: %s (op %d, fused with the next node) failed: %s\n", __func__, node->name, node->op,
                        chip_error_string(rc));
                return LM_GGML_STATUS_FAILED;
            }
            if (fused) {
                writes(cgraph->nodes[i + 1]);
                if (key.valid) c->quantized = key;
                if (waits) {
                    const lm_ggml_tensor *mul = cgraph->nodes[i + 1];
                    held.src = node->src[0];
                    held.out = mul;
                    held.weight = mul->src[0] == node ? mul->src[1] : mul->src[0];
                    std::memcpy(&held.eps, node->op_params, sizeof(float));
                }
                g_elementwise_nodes += 2;
                g_fused_pairs++;
                i++;
                continue;
            }
            if (node->op == LM_GGML_OP_UNARY && silu_can_wait_for_its_mul(cgraph, i)) {
                waiting_silu = node;                   // nodes[i + 1] is a weight matmul (it runs next), nodes[i + 2] the MUL
                continue;
            }
        }
        if ((node->op == LM_GGML_OP_RMS_NORM || node->op == LM_GGML_OP_ADD || node->op == LM_GGML_OP_MUL || node->op == LM_GGML_OP_UNARY ||
             node->op == LM_GGML_OP_SCALE) && elementwise_shape_ok(node)) {
            const int rc = run_elementwise(c, node);
            if (rc != CHIP_OK) {
                HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: %s (op %d) failed: %s\n", __func__, node->name, node->op, chip_error_string(rc));
                return LM_GGML_STATUS_FAILED;
            }
            g_elementwise_nodes++;
            continue;
        }
        {
            bool done = false;                        // this CPY ran in the kernel of the RoPE / the projection before it
            for (int &slot : stored_early)
                if (slot == i) { slot = -1; done = true; }
            if (done) continue;
        }
        if (i == paired_matmul) {                     // this matmul ran in the launch of the one two nodes before it
            paired_matmul = -1;
            continue;
        }
        if (i == rope_done) { rope_done = -1; continue; }
        {
            bool done = false;
            for (int &slot : roped_early)
                if (slot == i) { slot = -1; done = true; }
            if (done) continue;
        }
        if (i == rope_done_store) { rope_done_store = -1; continue; }
        if (is_attn_side_op(node->op) && attn_side_shape_ok(node)) {
            const lm_ggml_tensor *store = nullptr;
            rope_partner partner;
            bool paired = false;
            if (node->op == LM_GGML_OP_ROPE && fusion_enabled()) {
                const int j = rope_store_index(cgraph, i);
                if (j >= 0 && remember_store(j)) {
                    store = cgraph->nodes[j];
                    writes(store);
                    g_elementwise_nodes++;
                    g_fused_pairs++;
                }
                if (rope_done < 0 && rope_done_store < 0) {
                    // where the result of a projection that already ran with an earlier one lies: its slot or its own memory
                    auto ran_early = [&](const lm_ggml_tensor *t) -> const void * {
                        for (int k = 0; k < CHIP_GROUP_MAX; k++) {
                            if (grouped[k] < 0 || cgraph->nodes[grouped[k]] != t) continue;
                            if (rope_from_slot >= 0 && grouped[k] == rope_from_slot_owner) return rope_slot_src;
                            if (grouped_copy[k]) return t->nb[1] == (size_t)t->ne[0] * sizeof(float) ? grouped_copy[k] : nullptr;
                            return t->data;
                        }
                        return nullptr;
                    };
                    const int pj = rope_partner_index(cgraph, i, reads, ran_early, partner);
                    if (pj >= 0) {
                        paired = true;
                        rope_done = pj;
                        if (pj == rope_from_slot) rope_from_slot = -1;
                        writes(cgraph->nodes[pj]);
                        if (partner.store) {
                            rope_done_store = partner.store_index;
                            writes(partner.store);
                            g_elementwise_nodes++;
                            g_fused_pairs++;
                        }
                        g_elementwise_nodes++;
                        g_fused_pairs++;
                        g_rope_pairs++;
                    }
                }
            }
            const int rc = run_attn_side(c, node, store, i == rope_from_slot ? rope_slot_src : nullptr, paired ? &partner : nullptr);
            if (i == rope_from_slot) rope_from_slot = -1;
            if (rc != CHIP_OK) {
                HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: %s (op %d) failed: %s\n", __func__, node->name, node->op, chip_error_string(rc));
                return LM_GGML_STATUS_FAILED;
            }
            g_elementwise_nodes++;
            continue;
        }
        if (node->op == LM_GGML_OP_MUL_MAT_ID && mul_mat_id_shape_ok(node)) {
            const lm_ggml_tensor *w = node->src[0], *x = node->src[1], *ids = node->src[2];
            const int64_t K = w->ne[0], N = w->ne[1], n_used = ids->ne[0], n_tokens = ids->ne[1];
            if (N == 0 || n_used == 0 || n_tokens == 0) continue;
            if (!grow_workspace(c, chip_mul_mat_id_workspace_size(w->type, K, w->ne[2], n_used, n_tokens, x->ne[1]))) return LM_GGML_STATUS_ALLOC_FAILED;
            const int rc = chip_mul_mat_id(w->type, w->data, w->nb[1], w->nb[2], K, N, w->ne[2], (const float *)x->data,
                                           (int64_t)(x->nb[1] / 4), x->ne[1], (const int32_t *)ids->data, (int64_t)(ids->nb[1] / 4),
                                           n_used, n_tokens, (float *)node->data, (int64_t)(node->nb[1] / 4), c->workspace,
                                           c->workspace_size, c->stream);
            if (rc != CHIP_OK) {
                HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: MUL_MAT_ID %s failed: %s\n", __func__, node->name, chip_error_string(rc));
                return LM_GGML_STATUS_FAILED;
            }
            g_mul_mat_nodes++;
            continue;
        }
        if (node->op == LM_GGML_OP_MUL_MAT && !mul_mat_shape_ok(node) && mul_mat_f16_batched_shape_ok(node)) {
            const lm_ggml_tensor *w = node->src[0], *x = node->src[1];
            if (w->ne[1] == 0 || x->ne[1] == 0 || x->ne[2] == 0) continue;
            if (!grow_workspace(c, chip_mul_mat_f16_batched_workspace_size(w->ne[0], w->ne[1], w->ne[2], x->ne[2], x->ne[1])))
                return LM_GGML_STATUS_ALLOC_FAILED;
            const int merge = fusion_enabled() ? head_merge_index(cgraph, i) : -1;
            int rc;
            if (merge >= 0) {
                lm_ggml_tensor *ct = cgraph->nodes[merge];
                writes(ct);
                // merged[t][h * hd + d] = kqv[h][t][d]
                rc = chip_mul_mat_f16_batched_two_copies(w->data, w->nb[1], w->nb[2], w->ne[0], w->ne[1], w->ne[2], (const float *)x->data,
                                                         (int64_t)(x->nb[1] / 4), (int64_t)(x->nb[2] / 4), x->ne[1], x->ne[2],
                                                         (float *)node->data, (int64_t)(node->nb[1] / 4), (int64_t)(node->nb[2] / 4),
                                                         (float *)ct->data, node->ne[0] * node->ne[2], node->ne[0], c->workspace,
                                                         c->workspace_size, c->stream);
                if (rc == CHIP_OK) {
                    g_elementwise_nodes++;
                    g_fused_pairs++;
                    g_head_merges++;
                    i = merge;                        // only views lie between the two nodes
                }
            } else {
                rc = chip_mul_mat_f16_batched(w->data, w->nb[1], w->nb[2], w->ne[0], w->ne[1], w->ne[2], (const float *)x->data,
                                              (int64_t)(x->nb[1] / 4), (int64_t)(x->nb[2] / 4), x->ne[1], x->ne[2],
                                              (float *)node->data, (int64_t)(node->nb[1] / 4), (int64_t)(node->nb[2] / 4),
                                              c->workspace, c->workspace_size, c->stream);
            }
            if (rc != CHIP_OK) {
                HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: batched F16 MUL_MAT %s failed: %s\n", __func__, node->name, chip_error_string(rc));
                return LM_GGML_STATUS_FAILED;
            }
            g_mul_mat_nodes++;
            continue;
        }
        if (node->op == LM_GGML_OP_MUL_MAT && !mul_mat_shape_ok(node) && mul_mat_batched_shape_ok(node)) {
            // one 2-D matmul per slice of src1, on the slice of src0 that the broadcast assigns to it
            const lm_ggml_tensor *w = node->src[0], *x = node->src[1];
            const int64_t K = w->ne[0], N = w->ne[1], n = x->ne[1];
            if (N == 0 || n == 0) continue;
            if (!grow_workspace(c, chip_mul_mat_workspace_size_n(w->type, K, N, n))) return LM_GGML_STATUS_ALLOC_FAILED;
            const int64_t r2 = x->ne[2] / w->ne[2], r3 = x->ne[3] / w->ne[3];
            c->quantized.valid = false;
            for (int64_t i13 = 0; i13 < x->ne[3]; i13++)
                for (int64_t i12 = 0; i12 < x->ne[2]; i12++) {
                    const uint8_t *ws = (const uint8_t *)w->data + (size_t)(i12 / r2) * w->nb[2] + (size_t)(i13 / r3) * w->nb[3];
                    const float *xs = (const float *)((const uint8_t *)x->data + (size_t)i12 * x->nb[2] + (size_t)i13 * x->nb[3]);
                    float *ys = (float *)((uint8_t *)node->data + (size_t)i12 * node->nb[2] + (size_t)i13 * node->nb[3]);
                    const int rc = chip_mul_mat(w->type, ws, w->nb[1], K, N, xs, (int64_t)(x->nb[1] / 4), n, ys, (int64_t)(node->nb[1] / 4),
                                                c->workspace, c->workspace_size, c->stream);
                    if (rc != CHIP_OK) {
                        HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: batched MUL_MAT %s failed at slice (%lld, %lld): %s\n", __func__, node->name,
                                (long long)i12, (long long)i13, chip_error_string(rc));
                        return LM_GGML_STATUS_FAILED;
                    }
                }
            g_mul_mat_nodes++;
            continue;
        }
        if (node->op != LM_GGML_OP_MUL_MAT || !mul_mat_shape_ok(node)) {
            HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: node %d (%s, op %d) is not supported by the HIP backend\n", __func__, i, node->name, node->op);
            return LM_GGML_STATUS_FAILED;
        }
        {
            bool done = false;
            for (int k = 0; k < CHIP_GROUP_MAX; k++) {
                if (grouped[k] != i) continue;
                grouped[k] = -1;
                done = true;
                if (const float *from = grouped_copy[k]) {          // ran into a scratch slot: its own memory is free to take it now
                    grouped_copy[k] = nullptr;
                    const int64_t N = node->ne[0], n = node->ne[1];
                    const int64_t ne[4] = {N, n, 1, 1}, nbs[4] = {4, N * 4, N * n * 4, N * n * 4};
                    const int64_t nbd[4] = {4, (int64_t)node->nb[1], (int64_t)node->nb[1] * n, (int64_t)node->nb[1] * n};
                    const int rc = chip_cpy(from, LM_GGML_TYPE_F32, ne, nbs, node->data, LM_GGML_TYPE_F32, ne, nbd, c->stream);
                    if (rc != CHIP_OK) {
                        HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: copy of the early result of %s failed: %s\n", __func__, node->name, chip_error_string(rc));
                        return LM_GGML_STATUS_FAILED;
                    }
                }
            }
            if (done) continue;
        }
        const lm_ggml_tensor *w = node->src[0], *x = node->src[1];
        const int64_t K = w->ne[0], N = w->ne[1], n = x->ne[1];
        if (N == 0 || n == 0) continue;
        if (!grow_workspace(c, chip_mul_mat_workspace_size_n(w->type, K, N, n))) return LM_GGML_STATUS_ALLOC_FAILED;   // wdata
        int rc;
        const int64_t ldx = (int64_t)(x->nb[1] / 4);
        int store_t = -1;
        if (n <= 4 && fusion_enabled()) {
            // gate, SILU, up, MUL with nobody else reading the three intermediate results: one launch that stores the MUL's
            // result only.  Its workgroups store while others still read the activation, so the two must lie apart.
            const int up_index = paired_matmul_index(cgraph, i);
            if (up_index >= 0) {
                lm_ggml_tensor *up = cgraph->nodes[up_index], *silu = cgraph->nodes[i + 1], *mul = cgraph->nodes[i + 3];
                const bool kept = ((node->flags | silu->flags | up->flags) & LM_GGML_TENSOR_FLAG_OUTPUT) != 0;
                int64_t mrows, ldm;
                if (!kept && chip_mul_mat_pair_silu_mul_supported(w->type, K, N, n) && as_rows(mul, mrows, ldm) && mrows == n && disjoint(mul, x) &&
                    reads.readers_of(cgraph, node) == 1 && reads.readers_of(cgraph, silu) == 1 && reads.readers_of(cgraph, up) == 1) {
                    c->quantized.valid = false;
                    rc = CHIP_EUNSUPPORTED;
                    weight_arg wg = weight_for(c, w, n), wu = weight_for(c, up->src[0], n);
                    if (wg.type != wu.type) wg = weight_arg{(int)w->type, w->data, w->nb[1]}, wu = weight_arg{(int)w->type, up->src[0]->data, w->nb[1]};
                    if (held.held() && ranges_apart(mul, held.src)) {     // ffn_norm and its weight MUL in the same launch
                        const chip_norm_before nb{(const float *)held.weight->data, held.eps, (float *)x->data, ldx};
                        rc = chip_mul_mat_pair_silu_mul_norm(wg.type, wg.data, wu.data, wg.nb01, K, N, (const float *)held.src->data,
                                                             (int64_t)(held.src->nb[1] / 4), n, &nb, (float *)mul->data, ldm, c->workspace,
                                                             c->workspace_size, c->stream);
                        if (rc == CHIP_OK) { held.out = nullptr; g_norms_in_prologue++; }
                    }
                    if (rc == CHIP_EUNSUPPORTED && (rc = run_held_norm()) == CHIP_OK)
                        rc = chip_mul_mat_pair_silu_mul(wg.type, wg.data, wu.data, wg.nb01, K, N, (const float *)x->data, ldx, n,
                                                        (float *)mul->data, ldm, c->workspace, c->workspace_size, c->stream);
                    if (rc != CHIP_OK) {
                        HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: gated MUL_MAT pair at %s failed: %s\n", __func__, node->name, chip_error_string(rc));
                        return LM_GGML_STATUS_FAILED;
                    }
                    for (int k = 1; k <= 3; k++) writes(cgraph->nodes[i + k]);
                    g_mul_mat_nodes += 2;
                    g_elementwise_nodes += 2;
                    g_fused_pairs += 3;
                    g_gated_pairs++;
                    i += 3;
                    continue;
                }
            }
        }
        int members[CHIP_GROUP_MAX];
        bool aliased[CHIP_GROUP_MAX] = {false, false, false, false};
        int n_members = 1;
        if ((n <= 4 || n == 8) && fusion_enabled()) {      // the token counts chip_mul_mat_group has a one-launch form for
            bool slots_free = true;
            for (int slot : grouped) slots_free = slots_free && slot < 0;
            // A SILU held back for its MUL reads the gate projection's result only when that MUL runs, after this node:
            // a later projection run here could be sitting in memory the allocator freed from under it, so no group then.
            if (slots_free && !waiting_silu && rope_from_slot < 0) n_members = grouped_matmuls(cgraph, i, members, aliased);
        }
        if (n_members >= 2) {
            chip_mat mats[CHIP_GROUP_MAX];
            bool fits = true;
            int stores = 0;
            for (int k = 0; k < n_members; k++) fits = fits && cgraph->nodes[members[k]]->src[0]->ne[1] > 0;
            size_t slot_bytes = 0;
            for (int k = 1; k < n_members; k++)
                if (aliased[k]) slot_bytes = std::max(slot_bytes, (size_t)(cgraph->nodes[members[k]]->ne[0] * n) * sizeof(float));
            if (fits && slot_bytes > 0 && !grow_group_scratch(c, slot_bytes)) return LM_GGML_STATUS_ALLOC_FAILED;
            bool stored[CHIP_GROUP_MAX] = {false, false, false, false};
            for (int k = 0; fits && k < n_members; k++) {
                lm_ggml_tensor *mm = cgraph->nodes[members[k]];
                const lm_ggml_tensor *mw = mm->src[0];
                const weight_arg wa = weight_for(c, mw, n);
                mats[k] = chip_mat{wa.type, wa.data, wa.nb01, mw->ne[1], (float *)mm->data, (int64_t)(mm->nb[1] / 4), nullptr, 0};
                if (aliased[k]) {                      // its own memory is still in use: into the backend's slot k, rows side by side
                    mats[k].y = (float *)((uint8_t *)c->group_scratch + (size_t)k * c->group_slot_bytes);
                    mats[k].ldy = mw->ne[1];
                }
                if (!grow_workspace(c, chip_mul_mat_workspace_size_n(mw->type, K, mw->ne[1], n))) return LM_GGML_STATUS_ALLOC_FAILED;
                const int st = transposed_store_index(cgraph, members[k], i);
                if (st >= 0 && remember_store(st)) {
                    lm_ggml_tensor *cp = cgraph->nodes[st];
                    writes(cp);
                    mats[k].y_f16_t = (uint16_t *)cp->data;
                    mats[k].ld16 = (int64_t)(cp->nb[1] / 2);
                    stores++;
                    stored[k] = true;
                }
            }
            if (fits) {
                // ROPE nodes behind members, run in the members' epilogue (up to 4 tokens, fp32 rows)
                chip_rope_after ropes[CHIP_GROUP_MAX] = {};
                int rope_node[CHIP_GROUP_MAX] = {-1, -1, -1, -1}, rope_store[CHIP_GROUP_MAX] = {-1, -1, -1, -1};
                bool any_rope = false;
                int free_store_slots = 0;
                for (int slot : stored_early) free_store_slots += slot < 0;
                if (n <= 4 && rope_done < 0 && rope_done_store < 0) {
                    for (int k = 0; k < n_members; k++) {
                        if (stored[k]) continue;
                        int st = -1;
                        const int nx = rope_epilogue_index(cgraph, i, members[k], n, reads, ropes[k], st);
                        if (nx < 0) continue;
                        if (st >= 0 && free_store_slots == 0) { ropes[k] = chip_rope_after{}; continue; }
                        if (ensure_rope_table(c, cgraph->nodes[nx]) != CHIP_OK) { ropes[k] = chip_rope_after{}; continue; }
                        // one table serves the launch: a member whose ROPE has another key (positions, parameters) stays as it is
                        bool same_key = true;
                        for (int m = 0; m < k; m++)
                            if (rope_node[m] >= 0 && (cgraph->nodes[rope_node[m]]->src[1] != cgraph->nodes[nx]->src[1] ||
                                                      cgraph->nodes[rope_node[m]]->src[2] != cgraph->nodes[nx]->src[2] ||
                                                      std::memcmp(cgraph->nodes[rope_node[m]]->op_params, cgraph->nodes[nx]->op_params,
                                                                  sizeof(node->op_params)) != 0))
                                same_key = false;
                        if (!same_key) { ropes[k] = chip_rope_after{}; continue; }
                        ropes[k].table = c->rope_table;
                        rope_node[k] = nx;
                        rope_store[k] = st;
                        if (st >= 0) free_store_slots--;
                        any_rope = true;
                    }
                }
                quantized_key &q = c->quantized;
                const int vt = chip_vec_dot_type(w->type);
                rc = CHIP_EUNSUPPORTED;
                if (any_rope) {
                    q.valid = false;
                    bool apart = held.held();                     // everything the launch writes, apart from the held norm's input
                    for (int k = 0; apart && k < n_members; k++) {
                        apart = ranges_apart(cgraph->nodes[members[k]], held.src);
                        if (rope_node[k] >= 0) apart = apart && ranges_apart(cgraph->nodes[rope_node[k]], held.src);
                    }
                    if (apart) {                                  // attn_norm and its weight MUL in the same launch
                        const chip_norm_before nb{(const float *)held.weight->data, held.eps, (float *)x->data, ldx};
                        rc = chip_mul_mat_group_rope_norm(mats, ropes, &nb, n_members, K, (const float *)held.src->data,
                                                          (int64_t)(held.src->nb[1] / 4), n, c->workspace, c->workspace_size, c->stream);
                        if (rc == CHIP_OK) { held.out = nullptr; g_norms_in_prologue++; }
                    }
                    if (rc == CHIP_EUNSUPPORTED && (rc = run_held_norm()) == CHIP_OK)
                        rc = chip_mul_mat_group_rope(mats, ropes, n_members, K, (const float *)x->data, ldx, n, c->workspace, c->workspace_size, c->stream);
                    if (rc == CHIP_EUNSUPPORTED) {               // not a one-launch group: the ROPE nodes run at their own places
                        any_rope = false;
                        for (int k = 0; k < n_members; k++) { ropes[k] = chip_rope_after{}; rope_node[k] = rope_store[k] = -1; }
                    }
                }
                if (!any_rope && (rc = run_held_norm()) != CHIP_OK) {
                    HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: RMS_NORM held for %s failed: %s\n", __func__, node->name, chip_error_string(rc));
                    return LM_GGML_STATUS_FAILED;
                }
                if (!any_rope) {
                    // more than 4 tokens: the workspace holds x's quantized rows afterwards, or already does (the norm in front
                    // left them there, or an earlier matmul of the same input)
                    const bool have_rows = n > 4 && q.valid && q.src == x->data && q.K == K && q.n == n && q.ldx == ldx && q.vec_dot_type == vt;
                    if (have_rows) {
                        rc = chip_mul_mat_group_run(mats, n_members, K, n, c->workspace, c->workspace_size, c->stream);
                        g_quantizers_skipped++;
                    } else {
                        q.valid = false;
                        rc = chip_mul_mat_group(mats, n_members, K, (const float *)x->data, ldx, n, c->workspace, c->workspace_size, c->stream);
                        if (rc == CHIP_OK && n > 4) q = quantized_key{true, x->data, lm_ggml_nbytes(x), K, n, ldx, vt};
                    }
                }
                if (rc != CHIP_OK) {
                    HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: MUL_MAT group of %d at %s failed: %s\n", __func__, n_members, node->name,
                            chip_error_string(rc));
                    return LM_GGML_STATUS_FAILED;
                }
                for (int k = 0; k < n_members; k++) {
                    if (rope_node[k] < 0) continue;               // this member's ROPE (and its cache store) ran with it
                    lm_ggml_tensor *rp = cgraph->nodes[rope_node[k]];
                    writes(rp);
                    roped_early[k] = rope_node[k];
                    if (rope_store[k] >= 0) {
                        remember_store(rope_store[k]);
                        writes(cgraph->nodes[rope_store[k]]);
                        g_elementwise_nodes++;
                        g_fused_pairs++;
                    }
                    g_elementwise_nodes++;
                    g_fused_pairs++;
                    g_rope_epilogues++;
                }
                for (int k = 1; k < n_members; k++) {
                    lm_ggml_tensor *mm = cgraph->nodes[members[k]];
                    writes(mm);
                    grouped[k] = members[k];
                    grouped_copy[k] = nullptr;
                    if (!aliased[k] || rope_node[k] >= 0) continue;
                    // What becomes of a result in a scratch slot.  Its only reader was the cache store that ran with it: nothing.
                    // Its only reader is the ROPE that follows it (views aside) and takes its rows as they lie: that ROPE reads
                    // the slot.  Otherwise it is copied to its own memory when the loop gets to its node.
                    const int readers = reads.readers_of(cgraph, mm);
                    const int nx = next_compute_node(cgraph, members[k]);
                    const lm_ggml_tensor *rp = nx >= 0 ? cgraph->nodes[nx] : nullptr;
                    const bool kept = (mm->flags & LM_GGML_TENSOR_FLAG_OUTPUT) != 0;     // the caller reads it afterwards
                    if (!kept && readers == 1 && stored[k]) continue;
                    if (!kept && readers == 1 && rope_from_slot < 0 && rp && rp->op == LM_GGML_OP_ROPE && rp->src[0] && attn_side_shape_ok(rp) &&
                        (rp->src[0] == mm || rp->src[0]->view_src == mm) && rp->src[0]->data == mm->data && fusion_enabled() &&
                        mm->nb[1] == (size_t)mm->ne[0] * sizeof(float)) {
                        rope_from_slot = nx;
                        rope_from_slot_owner = members[k];
                        rope_slot_src = mats[k].y;
                        continue;
                    }
                    grouped_copy[k] = mats[k].y;
                }
                g_mul_mat_nodes += n_members;
                g_grouped_matmuls += n_members;
                g_elementwise_nodes += stores;
                g_fused_pairs += n_members - 1 + stores;
                continue;
            }
        }
        if (const int hrc = run_held_norm(); hrc != CHIP_OK) {     // none of the paths below has the norm in its prologue
            HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: RMS_NORM held for %s failed: %s\n", __func__, node->name, chip_error_string(hrc));
            return LM_GGML_STATUS_FAILED;
        }
        int add_index = -1;
        if (n <= 4 && fusion_enabled() && (store_t = transposed_store_index(cgraph, i)) >= 0 && remember_store(store_t)) {
            lm_ggml_tensor *cp = cgraph->nodes[store_t];
            writes(cp);
            c->quantized.valid = false;
            const weight_arg wa = weight_for(c, w, n);
            rc = chip_mul_mat_store_t(wa.type, wa.data, wa.nb01, K, N, (const float *)x->data, ldx, n, (float *)node->data,
                                      (int64_t)(node->nb[1] / 4), (uint16_t *)cp->data, (int64_t)(cp->nb[1] / 2), c->workspace,
                                      c->workspace_size, c->stream);
            g_elementwise_nodes++;
            g_fused_pairs++;
        } else if (n <= 4 && fusion_enabled() && (paired_matmul = paired_matmul_index(cgraph, i)) >= 0) {
            lm_ggml_tensor *up = cgraph->nodes[paired_matmul];
            writes(up);
            c->quantized.valid = false;
            weight_arg wg = weight_for(c, w, n), wu = weight_for(c, up->src[0], n);
            if (wg.type != wu.type) wg = weight_arg{(int)w->type, w->data, w->nb[1]}, wu = weight_arg{(int)w->type, up->src[0]->data, w->nb[1]};
            rc = chip_mul_mat_pair(wg.type, wg.data, wu.data, wg.nb01, K, N, (const float *)x->data, ldx, n, (float *)node->data,
                                   (float *)up->data, (int64_t)(node->nb[1] / 4), c->workspace, c->workspace_size, c->stream);
            g_mul_mat_nodes++;
            g_fused_pairs++;
        } else if ((n > 4 || have_rows(c->quantized, x, w, n, ldx)) && fusion_enabled()) {
            // quantize once per source tensor: the matmuls that share an input follow each other closely (up to 4 tokens
            // only a producer's kernel leaves rows here; without them the GEMV below quantizes in its prologue)
            quantized_key &q = c->quantized;
            const int vt = chip_vec_dot_type(w->type);
            if (!have_rows(q, x, w, n, ldx)) {
                q.valid = false;
                rc = chip_mul_mat_prepare(w->type, K, (const float *)x->data, ldx, n, c->workspace, c->workspace_size, c->stream);
                if (rc == CHIP_OK) q = quantized_key{true, x->data, lm_ggml_nbytes(x), K, n, ldx, vt};
            } else {
                rc = CHIP_OK;
                g_quantizers_skipped++;
            }
            if (rc == CHIP_OK)
                {
                const weight_arg wa = weight_for(c, w, n);
                rc = chip_mul_mat_run_ws(wa.type, wa.data, wa.nb01, K, N, n, c->workspace, c->workspace_size, (float *)node->data,
                                         (int64_t)(node->nb[1] / 4), c->stream);
            }
        } else if (n <= 4 && fusion_enabled() && add_done < 0 && (add_index = residual_add_index(cgraph, i, reads)) >= 0) {
            // wo / ffn_down and the residual ADD behind them: the GEMV adds the other operand as it stores, into the ADD's rows
            lm_ggml_tensor *add = cgraph->nodes[add_index];
            const lm_ggml_tensor *other = add->src[0] == node ? add->src[1] : add->src[0];
            c->quantized.valid = false;
            writes(add);
            const weight_arg wa = weight_for(c, w, n);
            rc = chip_mul_mat_add(wa.type, wa.data, wa.nb01, K, N, (const float *)x->data, ldx, n, (const float *)other->data,
                                  (int64_t)(other->nb[1] / 4), (float *)add->data, (int64_t)(add->nb[1] / 4), c->workspace, c->workspace_size,
                                  c->stream);
            add_done = add_index;
            g_elementwise_nodes++;
            g_fused_pairs++;
            g_residual_adds++;
        } else {
            c->quantized.valid = false;               // up to 4 tokens the GEMV quantizes in its own prologue, into the workspace
            const weight_arg wa = weight_for(c, w, n);
            rc = chip_mul_mat(wa.type, wa.data, wa.nb01, K, N, (const float *)x->data, ldx, n, (float *)node->data,
                              (int64_t)(node->nb[1] / 4), c->workspace, c->workspace_size, c->stream);
        }
        if (rc != CHIP_OK) {
            HIP_LOG(LM_GGML_LOG_LEVEL_ERROR, "%s: MUL_MAT %s failed: %s\n", __func__, node->name, chip_error_string(rc));
            return LM_GGML_STATUS_FAILED;
        }
        g_mul_mat_nodes++;
    }
    if (run_held_norm() != CHIP_OK) return LM_GGML_STATUS_FAILED;
    return LM_GGML_STATUS_SUCCESS;
}

const lm_ggml_backend_i k_backend_i = {
    /* get_name           */ backend_name,
    /* free               */ backend_free,
    /* set_tensor_async   */ backend_set_tensor_async,
    /* get_tensor_async   */ backend_get_tensor_async,
    /* cpy_tensor_async   */ nullptr,
    /* synchronize        */ backend_synchronize,
    /* graph_plan_create  */ nullptr,
    /* graph_plan_free    */ nullptr,
    /* graph_plan_update  */ nullptr,
    /* graph_plan_compute */ nullptr,
    /* graph_compute      */ backend_graph_compute,
    /* event_record       */ backend_event_record,
    /* event_wait         */ backend_event_wait,
};

// ------------------------------------------------------------------------------------------------ device
char g_description[160] = "AMD gfx950";

const char *dev_name(lm_ggml_backend_dev_t) { return "HIP0"; }
const char *dev_description(lm_ggml_backend_dev_t) { return g_description; }
void dev_memory(lm_ggml_backend_dev_t, size_t *free_b, size_t *total_b) {
    chip_device_info info;
    *free_b = *total_b = 0;
    if (device_ok() && chip_get_device_info(&info) == CHIP_OK) { *free_b = info.hbm_free; *total_b = info.hbm_total; }
}
int dev_type(lm_ggml_backend_dev_t) {
    // ACCEL: weights of supported matmuls move to the device, every other tensor (KV cache included) stays in
    // host buffers, so a backend that only implements MUL_MAT is safe (reference llama-model.cpp:277-287).
    const char *e = std::getenv("CACTUS_HIP_DEVICE_TYPE");
    return (e && std::strcmp(e, "GPU") == 0) ? LM_GGML_BACKEND_DEVICE_TYPE_GPU : LM_GGML_BACKEND_DEVICE_TYPE_ACCEL;
}
void dev_props(lm_ggml_backend_dev_t dev, lm_ggml_backend_dev_props *props) {
    props->name = dev_name(dev);
    props->description = dev_description(dev);
    props->type = dev_type(dev);
    dev_memory(dev, &props->memory_free, &props->memory_total);
    props->caps = {/* async */ true, /* host_buffer */ true, /* buffer_from_host_ptr */ false, /* events */ true};
}
lm_ggml_backend_t dev_init_backend(lm_ggml_backend_dev_t dev, const char *) {
    if (!device_ok()) return nullptr;
    backend_ctx *c = new (std::nothrow) backend_ctx{};
    if (!c) return nullptr;
    if (chip_stream_create(&c->stream) != CHIP_OK) { delete c; return nullptr; }
    lm_ggml_backend *b = new (std::nothrow) lm_ggml_backend{hip_guid(), k_backend_i, dev, c};
    if (!b) { chip_stream_destroy(c->stream); delete c; return nullptr; }
    return b;
}
lm_ggml_backend_buffer_type_t dev_buffer_type(lm_ggml_backend_dev_t) { return hip_buffer_type(); }
lm_ggml_backend_buffer_type_t dev_host_buffer_type(lm_ggml_backend_dev_t) { return hip_host_buffer_type(); }
lm_ggml_backend_event_t dev_event_new(lm_ggml_backend_dev_t dev) {
    if (!device_ok()) return nullptr;
    void *e = nullptr;
    if (chip_event_create(&e) != CHIP_OK || !e) return nullptr;
    lm_ggml_backend_event *ev = new (std::nothrow) lm_ggml_backend_event{dev, e};
    if (!ev) chip_event_destroy(e);
    return ev;
}
void dev_event_free(lm_ggml_backend_dev_t, lm_ggml_backend_event_t event) {
    if (!event) return;
    chip_event_destroy(event->context);
    delete event;
}
void dev_event_synchronize(lm_ggml_backend_dev_t, lm_ggml_backend_event_t event) { chip_event_synchronize(event->context); }

bool dev_supports_op(lm_ggml_backend_dev_t, const lm_ggml_tensor *op) {
    if (is_view_op(op->op)) return true;
    // element-wise F32 ops run wherever their operands are put: the scheduler keeps them with the matmuls around them
    if (op->op == LM_GGML_OP_RMS_NORM || op->op == LM_GGML_OP_ADD || op->op == LM_GGML_OP_MUL || op->op == LM_GGML_OP_UNARY ||
        op->op == LM_GGML_OP_SCALE)
        return elementwise_shape_ok(op);
    if (is_attn_side_op(op->op)) return attn_side_shape_ok(op);
    if (op->op != LM_GGML_OP_MUL_MAT && op->op != LM_GGML_OP_MUL_MAT_ID) return false;
    // Only weights that already live in a HIP buffer: claiming host-resident weights would make the scheduler
    // copy the whole matrix to the device on every call.  At model load the probe tensor carries a zero-size
    // dummy buffer of the candidate buffer type and NULL data (reference llama-model.cpp:161-165,246-251).
    // A view (the cache views of attention) answers with the buffer of the tensor it views, as the scheduler does.
    const lm_ggml_tensor *w = op->src[0];
    const lm_ggml_backend_buffer_t wbuf = !w ? nullptr : (w->view_src ? w->view_src->buffer : w->buffer);
    if (!wbuf || !is_hip_buffer(wbuf)) return false;
    return op->op == LM_GGML_OP_MUL_MAT ? (mul_mat_shape_ok(op) || mul_mat_f16_batched_shape_ok(op) || mul_mat_batched_shape_ok(op)) : mul_mat_id_shape_ok(op);
}
bool dev_supports_buft(lm_ggml_backend_dev_t, lm_ggml_backend_buffer_type_t buft) { return buft == hip_buffer_type(); }

const lm_ggml_backend_device_i k_device_i = {
    /* get_name             */ dev_name,
    /* get_description      */ dev_description,
    /* get_memory           */ dev_memory,
    /* get_type             */ dev_type,
    /* get_props            */ dev_props,
    /* init_backend         */ dev_init_backend,
    /* get_buffer_type      */ dev_buffer_type,
    /* get_host_buffer_type */ dev_host_buffer_type,
    /* buffer_from_host_ptr */ nullptr,
    /* supports_op          */ dev_supports_op,
    /* supports_buft        */ dev_supports_buft,
    /* offload_op           */ nullptr,
    /* event_new            */ dev_event_new,
    /* event_free           */ dev_event_free,
    /* event_synchronize    */ dev_event_synchronize,
};

// ------------------------------------------------------------------------------------------------ reg
const char *reg_name(lm_ggml_backend_reg_t) { return "HIP"; }
size_t reg_device_count(lm_ggml_backend_reg_t) { return device_ok() ? 1 : 0; }
lm_ggml_backend_dev_t reg_get_device(lm_ggml_backend_reg_t, size_t index) { return (index == 0 && device_ok()) ? hip_device() : nullptr; }
void *reg_get_proc_address(lm_ggml_backend_reg_t, const char *name) {
    if (std::strcmp(name, "lm_ggml_backend_hip_get_stats") == 0) return (void *)lm_ggml_backend_hip_get_stats;
    if (std::strcmp(name, "lm_ggml_backend_hip_get_fused_pairs") == 0) return (void *)lm_ggml_backend_hip_get_fused_pairs;
    if (std::strcmp(name, "lm_ggml_backend_hip_get_quantizers_skipped") == 0) return (void *)lm_ggml_backend_hip_get_quantizers_skipped;
    if (std::strcmp(name, "lm_ggml_backend_hip_get_rope_tables") == 0) return (void *)lm_ggml_backend_hip_get_rope_tables;
    if (std::strcmp(name, "lm_ggml_backend_hip_get_async_uploaded") == 0) return (void *)lm_ggml_backend_hip_get_async_uploaded;
    if (std::strcmp(name, "lm_ggml_backend_hip_get_grouped_matmuls") == 0) return (void *)lm_ggml_backend_hip_get_grouped_matmuls;
    return nullptr;         // no n_threads, no extra buffer types, no split buffer type, no feature list
}
const lm_ggml_backend_reg_i k_reg_i = {reg_name, reg_device_count, reg_get_device, reg_get_proc_address};

lm_ggml_backend_dev_t hip_device() {
    static lm_ggml_backend_device dev = {k_device_i, lm_ggml_backend_hip_reg(), nullptr};
    return &dev;
}
lm_ggml_backend_buffer_type_t hip_host_buffer_type() {
    static lm_ggml_backend_buffer_type buft = {
        {hbuft_name, hbuft_alloc, hbuft_alignment, /* get_max_size */ nullptr, /* get_alloc_size */ nullptr, hbuft_is_host},
        /* device  */ nullptr,
        /* context */ nullptr,
    };
    static std::once_flag once;
    std::call_once(once, [] { buft.device = hip_device(); });
    return &buft;
}
lm_ggml_backend_buffer_type_t hip_buffer_type() {
    static lm_ggml_backend_buffer_type buft = {
        {buft_name, buft_alloc, buft_alignment, /* get_max_size */ nullptr, /* get_alloc_size */ nullptr, buft_is_host},
        /* device  */ nullptr,
        /* context */ nullptr,
    };
    static std::once_flag once;
    std::call_once(once, [] { buft.device = hip_device(); });
    return &buft;
}

}  // namespace

extern "C" {

lm_ggml_backend_reg *lm_ggml_backend_hip_reg(void) {
    static lm_ggml_backend_reg reg = {LM_GGML_BACKEND_API_VERSION, k_reg_i, nullptr};
    static std::once_flag once;
    std::call_once(once, [] {
        chip_device_info info;
        if (device_ok() && chip_get_device_info(&info) == CHIP_OK)
            std::snprintf(g_description, sizeof(g_description), "%.60s (%.40s, %d CUs)", info.name[0] ? info.name : "AMD Instinct", info.arch, info.compute_units);
    });
    return &reg;
}
lm_ggml_backend_reg *lm_ggml_backend_init(void) { return lm_ggml_backend_hip_reg(); }
int lm_ggml_backend_score(void) { return device_ok() ? 100 : 0; }

lm_ggml_backend *lm_ggml_backend_hip_init(void) {
    lm_ggml_backend_hip_reg();
    return dev_init_backend(hip_device(), nullptr);
}
lm_ggml_backend_buffer_type *lm_ggml_backend_hip_buffer_type(void) {
    lm_ggml_backend_hip_reg();
    return hip_buffer_type();
}
int lm_ggml_backend_is_hip(lm_ggml_backend *backend) { return backend && backend->guid == hip_guid(); }
void lm_ggml_backend_hip_get_stats(unsigned long long *mul_mat_nodes, unsigned long long *uploaded_bytes) {
    if (mul_mat_nodes) *mul_mat_nodes = g_mul_mat_nodes.load();
    if (uploaded_bytes) *uploaded_bytes = g_uploaded.load();
}
unsigned long long lm_ggml_backend_hip_get_fused_pairs(void) { return g_fused_pairs.load(); }
unsigned long long lm_ggml_backend_hip_get_quantizers_skipped(void) { return g_quantizers_skipped.load(); }
unsigned long long lm_ggml_backend_hip_get_rope_tables(void) { return g_rope_tables.load(); }
unsigned long long lm_ggml_backend_hip_get_async_uploaded(void) { return g_uploaded_async.load(); }
unsigned long long lm_ggml_backend_hip_get_grouped_matmuls(void) { return g_grouped_matmuls.load(); }
unsigned long long lm_ggml_backend_hip_get_head_merges(void) { return g_head_merges.load(); }
unsigned long long lm_ggml_backend_hip_get_rope_pairs(void) { return g_rope_pairs.load(); }
unsigned long long lm_ggml_backend_hip_get_gated_pairs(void) { return g_gated_pairs.load(); }
unsigned long long lm_ggml_backend_hip_get_rope_epilogues(void) { return g_rope_epilogues.load(); }
unsigned long long lm_ggml_backend_hip_get_norms_in_prologue(void) { return g_norms_in_prologue.load(); }
unsigned long long lm_ggml_backend_hip_get_residual_adds(void) { return g_residual_adds.load(); }
unsigned long long lm_ggml_backend_hip_get_planes_copies(void) { return g_planes_copies.load(); }
unsigned long long lm_ggml_backend_hip_get_planes_bytes(void) { return g_planes_bytes.load(); }
unsigned long long lm_ggml_backend_hip_get_planes_dropped(void) { return g_planes_dropped.load(); }
unsigned long long lm_ggml_backend_hip_get_planes_matmuls(void) { return g_planes_matmuls.load(); }

}  // extern "C"
