/*
 * cactus_hip.h -- C-ABI of libcactus_hip.so: the MI355X (gfx950) kernels for the quantized MUL_MAT path.
 *
 * Plain pointers, sizes and integer return codes only; no ggml, torch or C++ types.  The ggml backend
 * (ggml_backend_hip.h / libggml-hip.so) sits on top of this layer; tests and benchmarks bind it with ctypes.
 *
 * Every entry point names the reference interface it replaces (paths relative to the reference's cactus/
 * directory).  All device pointers are plain HIP device addresses; `stream` is a hipStream_t passed as void*
 * (NULL = the default stream).  Calls are asynchronous with respect to the host unless stated otherwise.
 *
 * Return value: 0 on success, a negative CHIP_E* code on a rejected argument, a positive hipError_t value
 * if the HIP runtime failed.  chip_error_string() renders either.
 */
#ifndef CACTUS_HIP_H
#define CACTUS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CHIP_API __attribute__((visibility("default")))

/* weight / activation type ids: the reference's lm_ggml_type values (ggml.h:351-391) */
enum chip_type {
    CHIP_TYPE_F32  = 0,
    CHIP_TYPE_F16  = 1,      /* weight type and its own activation format (ggml-cpu/ggml-cpu.c:204-209) */
    CHIP_TYPE_Q4_0 = 2,
    CHIP_TYPE_Q8_0 = 8,
    CHIP_TYPE_Q4_K = 12,
    CHIP_TYPE_Q6_K = 14,
    CHIP_TYPE_Q8_K = 15,
    /* further weight types of type_traits_cpu[] (ggml-cpu/ggml-cpu.c:229,278,340) */
    CHIP_TYPE_Q5_0   = 6,
    CHIP_TYPE_Q5_K   = 13,
    CHIP_TYPE_IQ4_NL = 20,
    CHIP_TYPE_Q4_1   = 3,
    CHIP_TYPE_Q5_1   = 7,
    CHIP_TYPE_Q8_1   = 9,    /* activation format of Q4_1 / Q5_1 (ggml-cpu/ggml-cpu.c:221,237) */
    /* the 2- and 3-bit K-quants and IQ4_XS (ggml-cpu/ggml-cpu.c:257-268, 340-345; Q8_K activations): dot-product GEMV at every
     * token count (in passes of up to 8 tokens), GET_ROWS, MUL_MAT_ID per pair; no matrix-core kernels of their own */
    CHIP_TYPE_Q2_K   = 10,
    CHIP_TYPE_Q3_K   = 11,
    CHIP_TYPE_IQ4_XS = 23,
    /* Not a type of the reference: a Q6_K matrix whose rows chip_repack_q6_K has laid out in planes.  Accepted as the weight
     * type of the matmul entry points only (not by chip_get_rows, chip_mul_mat_id, chip_block_isums); every token count runs
     * on the dot-product GEMV, in passes of up to 8 tokens, so this layout is meant for decode (1..4 tokens). */
    CHIP_TYPE_Q6_K_PLANES = 114,
};

enum chip_status {
    CHIP_OK            = 0,
    CHIP_EINVAL        = -1,   /* NULL pointer, negative size, misaligned pointer or stride */
    CHIP_EUNSUPPORTED  = -2,   /* type or shape outside what the kernels implement */
    CHIP_ENOMEM        = -3,   /* workspace too small */
    CHIP_ENODEVICE     = -4,   /* no gfx950 device visible */
};

typedef struct chip_device_info {
    int    device;             /* HIP ordinal */
    int    compute_units;
    int    wavefront_size;
    int    max_lds_per_block;  /* bytes a single workgroup may use */
    int    clock_khz;
    int    xcd_count;          /* 0 if the runtime does not say */
    size_t hbm_total;
    size_t hbm_free;
    char   name[128];
    char   arch[64];
} chip_device_info;

/* ---- device and memory plumbing (what a ggml device/buffer needs; replaces nothing in the CPU path) ---- */
CHIP_API int         chip_init(int device);                    /* selects the device, checks it is gfx950 */
CHIP_API int         chip_device_count(void);
CHIP_API int         chip_get_device_info(chip_device_info *out);
CHIP_API const char *chip_error_string(int code);
CHIP_API int         chip_malloc(void **dptr, size_t bytes);
CHIP_API int         chip_free(void *dptr);
CHIP_API int         chip_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream);   /* synchronous if stream == NULL */
CHIP_API int         chip_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream);
CHIP_API int         chip_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream);
CHIP_API int         chip_memset(void *dst, int value, size_t bytes, void *stream);
CHIP_API int         chip_stream_create(void **stream);
CHIP_API int         chip_stream_destroy(void *stream);
CHIP_API int         chip_stream_synchronize(void *stream);

/* ---- what a ggml device with async uploads needs (reference ggml-backend-impl.h:100-116 set/get_tensor_async,
 * event_record/event_wait; :160 get_host_buffer_type; :176-178 event_new/free/synchronize; used by the model loader's
 * chunked upload, llama-model-loader.cpp:905-1064) ----
 * chip_memcpy_h2d / _d2h with a stream are asynchronous; they overlap with the host only from pinned memory. */
CHIP_API int chip_host_malloc(void **ptr, size_t bytes);          /* pinned host memory (hipHostMalloc) */
CHIP_API int chip_host_free(void *ptr);
CHIP_API int chip_event_create(void **event);
CHIP_API int chip_event_destroy(void *event);
CHIP_API int chip_event_record(void *event, void *stream);        /* the event completes when the stream reaches this point */
CHIP_API int chip_event_synchronize(void *event);                 /* host waits */
CHIP_API int chip_stream_wait_event(void *stream, void *event);   /* later work of the stream waits */

/* ---- layout facts ---- */
/* lm_ggml_blck_size / lm_ggml_type_size / lm_ggml_row_size (ggml.c:1186-1200) for the types above; 0 if unknown */
CHIP_API int    chip_block_elems(int type);
CHIP_API size_t chip_block_bytes(int type);
CHIP_API size_t chip_row_size(int type, int64_t k);
/* type_traits_cpu[type].vec_dot_type (ggml-cpu/ggml-cpu.c:198-367): Q8_0 for Q4_0/Q8_0/Q5_0/IQ4_NL, Q8_K for
 * Q4_K/Q5_K/Q6_K, Q8_1 for Q4_1/Q5_1, F16 for F16 */
CHIP_API int    chip_vec_dot_type(int type);
/* 1 if chip_mul_mat accepts this weight type and K (K must be a multiple of 256) */
CHIP_API int    chip_mul_mat_supported(int type, int64_t K);

/* ---- activation quantizers ----
 * quantize_row_q8_0, AVX2 branch (ggml-cpu/ggml-cpu-quants.c:732-738,802-885) and quantize_row_q8_K
 * (ggml-cpu/ggml-cpu-quants.c:1740,1819-1821 -> ggml-quants.c:2473-2510), for n rows at once.
 *   x       : n rows of k floats, row t at x + t*ldx (ldx in elements, >= k)
 *   y       : n rows of chip_row_size(type, k) bytes, packed, in the reference's block layout
 * Output bytes equal the reference's bit for bit (an all-zero Q8_K block gets zero bsums, which the
 * reference leaves unwritten). */
CHIP_API int chip_quantize_q8_0(const float *x, int64_t ldx, int64_t n, int64_t k, void *y, void *stream);
CHIP_API int chip_quantize_q8_K(const float *x, int64_t ldx, int64_t n, int64_t k, void *y, void *stream);
/* quantize_row_q8_1, AVX2 branch (ggml-cpu/ggml-cpu-quants.c:1047-1140): the activation format of Q4_1 / Q5_1;
 * quants and d as Q8_0, plus s = fp16(d * sum of quants) */
CHIP_API int chip_quantize_q8_1(const float *x, int64_t ldx, int64_t n, int64_t k, void *y, void *stream);
/* lm_ggml_cpu_fp32_to_fp16 (ggml-cpu/ggml-cpu.c:3161-3190): fp32 rows -> fp16 rows, round to nearest even; the
 * activation format of F16 weights (k a multiple of 4) */
CHIP_API int chip_convert_f32_to_f16(const float *x, int64_t ldx, int64_t n, int64_t k, void *y, void *stream);

/* ---- the op: LM_GGML_OP_MUL_MAT over block-quantized weights ----
 * lm_ggml_compute_forward_mul_mat (ggml-cpu/ggml-cpu.c:1257-1449) with src0 = W (type, [K, N], row stride
 * nb01 bytes, GGUF block layout untouched), src1 = x (F32 [K, n], row stride ldx elements), dst = y
 * (F32 [N, n], row stride ldy elements):  y[t][r] = vec_dot(W row r, quantize(x row t)).
 *
 *   workspace : device scratch of at least chip_mul_mat_workspace_size(type, K, n) bytes (params->wdata in the
 *               reference, sized by lm_ggml_graph_plan, ggml-cpu/ggml-cpu.c:2697-2704); holds the quantized
 *               activations in a kernel-private layout
 * n <= 4 runs the dot-product GEMV with the quantizer in its prologue; Q8_0 with n >= 5 the matrix-core GEMV
 * (16 tokens per pass over W); from 16 to 48 tokens on (by type and matrix size) the MFMA GEMM of the weight type;
 * everything else the GEMV in token groups.
 * K must be a multiple of 256; for the types of 32-value blocks (Q4_0, Q8_0, Q5_0, IQ4_NL, Q4_1, Q5_1) a multiple of 64
 * is enough (hidden sizes such as 576, 896, 960: the GEMV, and the GEMM when K % 128 == 0).  W must be 16-byte aligned
 * and nb01 a multiple of 16 (2 and 2 for Q6_K, whose 210-byte blocks allow no more; 4 and 4 for rows of K % 256 != 0);
 * x 16-byte aligned with ldx a multiple of 4; y 4-byte aligned.
 */
CHIP_API size_t chip_mul_mat_workspace_size(int type, int64_t K, int64_t n);
/* The same plus room for the partial outputs of a GEMM whose K is split over workgroups (when the output has fewer
 * tiles than the device holds workgroups: a few hundred tokens at most; the partial tiles are added in a fixed order by
 * a second kernel).  chip_mul_mat splits K only when workspace_bytes is at least this; with the smaller size it runs
 * unsplit, and takes the GEMM from a larger token count on. */
CHIP_API size_t chip_mul_mat_workspace_size_n(int type, int64_t K, int64_t N, int64_t n);
CHIP_API int    chip_mul_mat(int type, const void *W, size_t nb01, int64_t K, int64_t N,
                             const float *x, int64_t ldx, int64_t n,
                             float *y, int64_t ldy, void *workspace, size_t workspace_bytes, void *stream);

/* The two phases of chip_mul_mat separately (Phase A / Phase B of the reference op, ggml-cpu/ggml-cpu.c:1319-1354
 * and :1380-1448), so one quantized activation can feed several matmuls (wq/wk/wv share an input, as do
 * ffn_up/ffn_gate).  chip_mul_mat_prepare fills `workspace` from x; chip_mul_mat_run consumes it.
 * The workspace contents depend on (vec_dot_type of `type`, K, n) only. */
CHIP_API int chip_mul_mat_prepare(int type, int64_t K, const float *x, int64_t ldx, int64_t n,
                                  void *workspace, size_t workspace_bytes, void *stream);
CHIP_API int chip_mul_mat_run(int type, const void *W, size_t nb01, int64_t K, int64_t N, int64_t n,
                              const void *workspace, float *y, int64_t ldy, void *stream);
/* Two matmuls of one type, shape and row stride on the same activation (ffn_gate and ffn_up, llama-graph.cpp:562-690):
 * up to 4 tokens both run in one launch of the GEMV that quantizes in its prologue; with more tokens the activation is
 * quantized once and each matrix takes its usual path (5..8 tokens, Q4_K / Q5_K matrices that would each take the
 * matrix-core GEMV: one launch of it over both).  Results as from two chip_mul_mat calls, bit for bit. */
CHIP_API int chip_mul_mat_pair(int type, const void *W1, const void *W2, size_t nb01, int64_t K, int64_t N, const float *x,
                               int64_t ldx, int64_t n, float *y1, float *y2, int64_t ldy, void *workspace, size_t workspace_bytes,
                               void *stream);
/* The gated FFN up to ffn_down's input in one launch: MUL(SILU(MUL_MAT(W1, x)), MUL_MAT(W2, x)), the four nodes of
 * LLM_FFN_SILU with LLM_FFN_PAR (reference llama-graph.cpp:562-690; lm_ggml_vec_silu_f32, ggml-cpu/vec.cpp:164-186).  Arguments
 * as chip_mul_mat_pair with one output: y[t * ldy + r] = silu(y1[t][r]) * y2[t][r], bit for bit what chip_mul_mat_pair
 * followed by chip_silu_mul gives; the two projections themselves are not stored.  For 1, 2 or 4 tokens and N a multiple
 * of 8 (as chip_silu) where chip_mul_mat_pair runs as one GEMV launch (chip_mul_mat_pair_silu_mul_supported returns 1); CHIP_EUNSUPPORTED
 * otherwise, nothing written.  The workspace holds the quantized rows of x afterwards, as after chip_mul_mat. */
CHIP_API int chip_mul_mat_pair_silu_mul_supported(int type, int64_t K, int64_t N, int64_t n);
CHIP_API int chip_mul_mat_pair_silu_mul(int type, const void *W1, const void *W2, size_t nb01, int64_t K, int64_t N,
                                        const float *x, int64_t ldx, int64_t n, float *y, int64_t ldy, void *workspace,
                                        size_t workspace_bytes, void *stream);
/* Several matmuls that read the same activation rows (wq / wk / wv of an attention block: llama.cpp builds Qcur, Kcur,
 * Vcur from one tensor, llama-model.cpp build_llama; the reference quantizes src1 once per MUL_MAT node,
 * ggml-cpu/ggml-cpu.c:1319-1354) as one call: up to CHIP_GROUP_MAX weight matrices with the same K, each with its own
 * type, row count, row stride and output.  The types must share one activation format (chip_vec_dot_type; Q8_0 and Q8_1
 * count as one).  Up to 4 tokens, members of one family (K-quants / 32-value block types / F16): one launch of the GEMV that
 * quantizes in its prologue, its workgroups divided among the members by the bytes each streams; otherwise one
 * quantizer launch and every member on the path chip_mul_mat_run_ws would take.  A member with y_f16_t != NULL also gets
 * its result rounded to fp16 at y_f16_t[row * ld16 + token], as chip_mul_mat_store_t.  Every output equals, bit for bit,
 * what chip_mul_mat (chip_mul_mat_store_t) returns for that member alone - except at exactly 8 tokens when the members
 * together stream at most 24 MB: they then run as one launch of the dot-product GEMV over the quantized rows, while a
 * member alone may take the matrix-core GEMV, which adds its partial sums in another order (same tolerance against the
 * reference, not the same bits).  The workspace must hold
 * chip_mul_mat_workspace_size(type, K, n) bytes for the members' activation format. */
#define CHIP_GROUP_MAX 4
typedef struct chip_mat {
    int         type;       /* weight type */
    const void *W;          /* N rows of nb01 bytes */
    size_t      nb01;
    int64_t     N;
    float      *y;          /* [n][N], row stride ldy elements */
    int64_t     ldy;
    uint16_t   *y_f16_t;    /* NULL, or the transposed fp16 copy [N][ld16] */
    int64_t     ld16;
} chip_mat;
CHIP_API int chip_mul_mat_group(const chip_mat *mats, int count, int64_t K, const float *x, int64_t ldx, int64_t n,
                                void *workspace, size_t workspace_bytes, void *stream);
/* chip_mul_mat_group with the ROPE node that follows a member run in that member's epilogue (reference
 * cactus/llama-model.cpp build_llama: Qcur / Kcur = lm_ggml_rope_ext(...) right after their projections;
 * lm_ggml_compute_forward_rope_f32, ggml-cpu/ops.cpp:5178-5361, modes 0 and LM_GGML_ROPE_TYPE_NEOX = 2).  ropes[i].table != NULL:
 * member i's rows are heads of head_dim values (N a multiple of head_dim), a wave computes the two rows of a rotated pair one
 * after the other and stores the pair rotated with table (chip_rope_table's output for the n tokens): y receives what
 * chip_rope_apply would write from the member's result, y_f16 its fp16 copy as chip_rope_apply_store (the K cache store);
 * either may be NULL, not both.  mats[i].y is not written for such a member (it may be NULL).  Every value has the bits of
 * chip_mul_mat_group followed by chip_rope_apply / chip_rope_apply_store.  Only where chip_mul_mat_group is one launch (1, 2
 * or 4 tokens, members of one family, K-quants or 32-value block types, fp32 rows x): CHIP_EUNSUPPORTED otherwise, nothing
 * written, and the caller runs the nodes one by one. */
typedef struct chip_rope_after {
    const float *table;      /* NULL: no ROPE behind this member */
    int64_t      head_dim;   /* ne0 of the ROPE */
    int          n_dims, mode;
    float       *y;          /* F32 result [n][N], row stride ldy, or NULL */
    int64_t      ldy;
    uint16_t    *y_f16;      /* fp16 copy [n][N], row stride ld16 halves, or NULL */
    int64_t      ld16;
} chip_rope_after;
CHIP_API int chip_mul_mat_group_rope(const chip_mat *mats, const chip_rope_after *ropes, int count, int64_t K, const float *x,
                                     int64_t ldx, int64_t n, void *workspace, size_t workspace_bytes, void *stream);
/* The RMS norm and the MUL with the norm weight that precede a projection, run in the projection's prologue (reference
 * cactus/llama-graph.cpp build_norm, LLM_NORM_RMS: lm_ggml_rms_norm then lm_ggml_mul with the weight; lm_ggml_compute_forward_rms_norm_f32,
 * ggml-cpu/ops.cpp).  x is then the norm's input; every workgroup norms the rows it has loaded for quantizing, with the
 * additions in chip_rms_norm_mul's order, so every value has the bits of chip_rms_norm_mul followed by the plain call.
 * y (optional) receives the normed rows, as the MUL node's tensor would hold them. */
typedef struct chip_norm_before {
    const float *w;          /* the norm weight, K floats, 16-byte aligned */
    float        eps;
    float       *y;          /* [n][K] at row stride ldy (16-byte aligned, ldy a multiple of 4), or NULL */
    int64_t      ldy;
} chip_norm_before;
/* chip_mul_mat_group_rope on rows normed in the prologue.  CHIP_EUNSUPPORTED where chip_mul_mat_group_rope is, and for rows
 * the prologue does not hold whole (K-quant rows of more than two steps, K > 8192): nothing written then. */
CHIP_API int chip_mul_mat_group_rope_norm(const chip_mat *mats, const chip_rope_after *ropes, const chip_norm_before *norm, int count,
                                          int64_t K, const float *x, int64_t ldx, int64_t n, void *workspace, size_t workspace_bytes,
                                          void *stream);
/* chip_mul_mat_pair_silu_mul on rows normed in the prologue (ffn_norm in front of ffn_gate / ffn_up); same conditions. */
CHIP_API int chip_mul_mat_pair_silu_mul_norm(int type, const void *W1, const void *W2, size_t nb01, int64_t K, int64_t N, const float *x,
                                             int64_t ldx, int64_t n, const chip_norm_before *norm, float *y, int64_t ldy, void *workspace,
                                             size_t workspace_bytes, void *stream);
/* 1 when the two calls above take rows of K values of this weight type at n tokens */
CHIP_API int chip_norm_before_supported(int type, int64_t K, int64_t n);
/* y = W x + addend: the residual ADD that follows wo and ffn_down (reference cactus/llama-model.cpp build_llama: ffn_inp =
 * lm_ggml_add(cur, inpSA), cur = lm_ggml_add(cur, ffn_inp)) done where the GEMV stores its result.  addend [n][N] at row stride
 * ld_add; it may be y itself (same pointer and stride) or lie apart from it.  Bits of chip_mul_mat followed by chip_add
 * (matmul result first operand).  One launch, 1, 2 or 4 tokens where chip_mul_mat quantizes in its prologue
 * (chip_mul_mat_add_supported); CHIP_EUNSUPPORTED otherwise, nothing written. */
CHIP_API int chip_mul_mat_add_supported(int type, int64_t K, int64_t N, int64_t n);
CHIP_API int chip_mul_mat_add(int type, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, int64_t n,
                              const float *addend, int64_t ld_add, float *y, int64_t ldy, void *workspace, size_t workspace_bytes,
                              void *stream);
/* The same over rows the workspace already holds - Phase B of the op alone (ggml-cpu/ggml-cpu.c:1380-1448) for a group, as
 * chip_mul_mat_run is for one matrix: the rows were written by chip_mul_mat_prepare or by the kernel that produced the
 * activations (chip_rms_norm_quantized, chip_silu_mul_quantized).  Up to 4 tokens and members of one family: one launch of
 * the GEMV that stages the rows from the workspace; any row length the activation image of n rows fits in LDS for.  Every
 * output equals, bit for bit, chip_mul_mat_run's for that member (and the fp16 store of chip_mul_mat_store_t). */
CHIP_API int chip_mul_mat_group_run(const chip_mat *mats, int count, int64_t K, int64_t n, void *workspace,
                                    size_t workspace_bytes, void *stream);
/* chip_mul_mat whose result also goes, rounded to fp16 (nearest even), to y_f16_t[row * ld16 + token]: the V projection
 * and its store into the transposed F16 V cache (llama-kv-cache.cpp cpy_v without flash attention) - one launch up to 4
 * tokens, otherwise the matmul followed by the copy.  Results as from chip_mul_mat and chip_cpy. */
CHIP_API int chip_mul_mat_store_t(int type, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, int64_t n,
                                  float *y, int64_t ldy, uint16_t *y_f16_t, int64_t ld16, void *workspace, size_t workspace_bytes,
                                  void *stream);
/* chip_mul_mat_run told how large the workspace is: with chip_mul_mat_workspace_size_n(type, K, N, n) bytes a GEMM may
 * split K (the partial outputs go behind the activation rows, which stay valid for the next matmul). */
CHIP_API int chip_mul_mat_run_ws(int type, const void *W, size_t nb01, int64_t K, int64_t N, int64_t n,
                                 void *workspace, size_t workspace_bytes, float *y, int64_t ldy, void *stream);

/* chip_mul_mat for callers that cannot allocate device memory or hand one over (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The workspace is a static device
 * array inside the library (chip_mul_mat_noalloc_max_workspace() bytes, 16 MiB, held by every GPU the library runs on
 * until the process ends); the call allocates nothing and frees nothing.  Results equal chip_mul_mat's with a workspace
 * of that size, bit for bit.  CHIP_ENOMEM when chip_mul_mat_workspace_size(type, K, n) exceeds the array (e.g. more than
 * 3500 tokens of K = 4096).  All calls on one GPU share the array: calls that may overlap in time (different streams)
 * race; calls on one stream are ordered and safe.  Nothing in the array has to start at zero.
 * Set-up is not part of that promise: chip_init() on the device looks up the array's address, and the first launch of a
 * kernel shape raises that kernel's LDS limit (a host call).  A caller under stream capture therefore calls chip_init()
 * and makes one ordinary call of the same (type, K, N, n) before it captures; captured calls replay correctly. */
CHIP_API size_t chip_mul_mat_noalloc_max_workspace(void);
CHIP_API int    chip_mul_mat_noalloc(int type, const void *W, size_t nb01, int64_t K, int64_t N,
                                     const float *x, int64_t ldx, int64_t n, float *y, int64_t ldy, void *stream);

/* ---- LM_GGML_OP_MUL_MAT_ID: the expert matmul of mixture-of-experts layers ----
 * lm_ggml_compute_forward_mul_mat_id (ggml-cpu/ggml-cpu.c:1460-1710) with src0 = W (type, [K, N, n_as]: n_as expert
 * matrices, row stride nb01 and matrix stride nb02 bytes), src1 = x (F32 [K, ne11, n_tokens], row stride ldx
 * elements, the ne11 rows of a token adjacent: nb12 = ne11 * nb11), ids (I32 [n_used, n_tokens] in device memory,
 * ids_stride elements between tokens), dst = y (F32 [N, n_used, n_tokens], row stride ldy elements, rows adjacent):
 *     y[t][s][r] = vec_dot(row r of expert ids[t][s], quantize(x[t][s % ne11]))
 * ne11 is 1 (all slots of a token share one activation row) or n_used.  Every id must lie in [0, n_as); a pair
 * with an id outside is left unwritten (the reference asserts).  The workspace (at least
 * chip_mul_mat_id_workspace_size bytes) holds the n_tokens * ne11 quantized rows and the pair lists.  Alignment rules
 * as chip_mul_mat; nb02 obeys the rule of nb01.  Below 64 (token, slot) pairs each pair runs as a one-token GEMV on
 * its expert; from 64 on the pairs are grouped by expert on the device (the reference's matrix_rows) and every
 * expert's group runs through the MFMA GEMM of the weight type. */
CHIP_API size_t chip_mul_mat_id_workspace_size(int type, int64_t K, int64_t n_as, int64_t n_used, int64_t n_tokens,
                                               int64_t ne11);
CHIP_API int chip_mul_mat_id(int type, const void *W, size_t nb01, size_t nb02, int64_t K, int64_t N, int64_t n_as,
                             const float *x, int64_t ldx, int64_t ne11, const int32_t *ids, int64_t ids_stride,
                             int64_t n_used, int64_t n_tokens, float *y, int64_t ldy,
                             void *workspace, size_t workspace_bytes, void *stream);

/* ---- the element-wise ops between the matmuls of an FFN block (F32 rows; row strides in elements) ----
 * So that norm -> up/gate -> activation -> down -> residual stays on the device.  In-place use (y == x / a) is allowed.
 *   chip_rms_norm : LM_GGML_OP_RMS_NORM, lm_ggml_compute_forward_rms_norm_f32 (ggml-cpu/ops.cpp:3270-3316):
 *                   y = x / sqrt(mean(x^2) + eps) per row; squares summed in double.
 *   chip_add/_mul : LM_GGML_OP_ADD / LM_GGML_OP_MUL (ggml-cpu/binary-ops.cpp) for src1 of the shape of src0 (n_b == n) or
 *                   one row broadcast over all rows (n_b == 1: norm weights, biases); other broadcasts are declined.
 *   chip_silu     : LM_GGML_UNARY_OP_SILU, lm_ggml_vec_silu_f32 (ggml-cpu/vec.cpp:164-186) in its AVX2 + FMA form
 *                   (lm_ggml_v_expf, ggml-cpu/vec.h:615-656), bit for bit; ne0 must be a multiple of 8 (the reference
 *                   finishes other rows with the C library's expf). */
CHIP_API int chip_rms_norm(const float *x, int64_t ldx, int64_t n, int64_t ne0, float eps, float *y, int64_t ldy, void *stream);
CHIP_API int chip_add(const float *a, int64_t lda, const float *b, int64_t ldb, int64_t n_b, int64_t n, int64_t ne0,
                      float *y, int64_t ldy, void *stream);
CHIP_API int chip_mul(const float *a, int64_t lda, const float *b, int64_t ldb, int64_t n_b, int64_t n, int64_t ne0,
                      float *y, int64_t ldy, void *stream);
CHIP_API int chip_silu(const float *x, int64_t ldx, int64_t n, int64_t ne0, float *y, int64_t ldy, void *stream);
/* Two or three adjacent graph nodes in one launch; every element goes through the same operations in the same order as in the
 * separate calls, so the results are bit-identical to them:
 *   chip_rms_norm_mul : y = chip_rms_norm(x) * w, w one row of ne0 (build_norm's weight, llama-graph.cpp:527-560); y_norm
 *                       (may be NULL) receives the norm itself.
 *   chip_silu_mul     : y = chip_silu(x) * b, b of the shape of x (the gated FFN, llama-graph.cpp:562-690).
 *   chip_add_rms_norm_mul : sum = a + b (the residual, llama-model.cpp build_llama: "ffn_inp", "l_out"), y = chip_rms_norm(sum)
 *                       [* w when w is not NULL]. sum is always written (the next residual reads it) and may be a or b;
 *                       y may be a or b (with their row stride) but not sum; otherwise the blocks must not overlap. */
CHIP_API int chip_rms_norm_mul(const float *x, int64_t ldx, int64_t n, int64_t ne0, float eps, const float *w, float *y_norm,
                               int64_t ld_norm, float *y, int64_t ldy, void *stream);
CHIP_API int chip_silu_mul(const float *x, int64_t ldx, const float *b, int64_t ldb, int64_t n, int64_t ne0, float *y, int64_t ldy,
                           void *stream);
/* LM_GGML_OP_SCALE (lm_ggml_compute_forward_scale_f32, ggml-cpu/ops.cpp:3930-3968): y = x * scale, one fp32 multiply.
 * LM_GGML_UNARY_OP_GELU on F32 (lm_ggml_vec_gelu_f32 with LM_GGML_GELU_FP16, ggml-cpu/vec.h:16,452-466): 0 at or below -10,
 * x at or above 10, else entry fp16(x) of the 65536-entry fp16 table of lm_ggml_cpu_init (ggml-cpu/ggml-cpu.c:3474-3481).
 * `table` is that table in device memory (128 KiB): chip_gelu_table computes it on the host, with this process's tanhf,
 * for the caller to upload - or the caller uploads the host framework's own lm_ggml_table_gelu_f16, as the ggml
 * backend does, and is then bit-identical to that framework's CPU path whatever it was compiled with. */
CHIP_API int chip_scale(const float *x, int64_t ldx, int64_t n, int64_t ne0, float scale, float *y, int64_t ldy, void *stream);
CHIP_API int chip_gelu_table(uint16_t *table_host_65536);
CHIP_API int chip_gelu(const float *x, int64_t ldx, int64_t n, int64_t ne0, const uint16_t *table, float *y, int64_t ldy,
                       void *stream);
/* The norm in front of a group of matmuls: y = chip_rms_norm(a [+ b, the sum stored to `sum` as in chip_add_rms_norm_mul])
 * [* w], and y quantized as the activation type of weight type `wtype` into `workspace`, exactly what chip_mul_mat_prepare
 * (wtype, K = ne0, y, ...) would leave there - the matmuls that read y can go straight to chip_mul_mat_run.  Rows of up to
 * 8192 values, a multiple of 256, 16-byte aligned with strides that are multiples of 4; CHIP_EUNSUPPORTED otherwise (and
 * for F16 weights), in which case nothing has been written. */
CHIP_API int chip_rms_norm_quantized(const float *a, int64_t lda, const float *b, int64_t ldb, float *sum, int64_t ld_sum, int64_t n,
                                     int64_t ne0, float eps, const float *w, float *y, int64_t ldy, int wtype, void *workspace,
                                     size_t workspace_bytes, void *stream);
/* chip_silu_mul in front of a matmul (ffn_down reads silu(ffn_gate) * ffn_up, reference llama-graph.cpp:562-690): y as
 * chip_silu_mul writes it, and y quantized as the activation type of weight type `wtype` into `workspace`, exactly what
 * chip_mul_mat_prepare(wtype, K = ne0, y, ...) would leave there.  Rows of any length that is a multiple of 256, 16-byte
 * aligned with strides that are multiples of 4, at most 65535 rows; CHIP_EUNSUPPORTED otherwise (and for F16 weights), in
 * which case nothing has been written. */
CHIP_API int chip_silu_mul_quantized(const float *x, int64_t ldx, const float *b, int64_t ldb, int64_t n, int64_t ne0, float *y,
                                     int64_t ldy, int wtype, void *workspace, size_t workspace_bytes, void *stream);
CHIP_API int chip_add_rms_norm_mul(const float *a, int64_t lda, const float *b, int64_t ldb, float *sum, int64_t ld_sum, int64_t n,
                                   int64_t ne0, float eps, const float *w, float *y, int64_t ldy, void *stream);

/* ---- the attention matmuls over an F16 KV cache ----
 * LM_GGML_OP_MUL_MAT whose src0 is an F16, batched, strided view and whose src1 is F32 (reference llama-graph.cpp:1120
 * kq = mul_mat(k, q) and :1154 kqv = mul_mat(v, kq); CPU path ggml-cpu/ggml-cpu.c:1177-1456 with
 * type_traits_cpu[LM_GGML_TYPE_F16]: src1 rounded to fp16, lm_ggml_vec_dot_f16, ggml-cpu/vec.cpp:122-162):
 *     y[b][t][r] = sum_k W[b / (ne12 / ne02)][r][k] * fp16(x[b][t][k])       b < ne12, t < n, r < N
 * W: F16, rows of K halves at nb01 bytes, batches (KV heads) at nb02 bytes; x: F32 rows of K at ldx1 floats (tokens) and
 * ldx2 floats (batches: query heads); y likewise, rows of N.  ne12 must be a multiple of ne02 (grouped-query broadcast,
 * the reference's r2); a fourth dimension is not taken.  K a multiple of 8; W, nb01, nb02, x 16-byte aligned, ldx1 and
 * ldx2 multiples of 4.  The workspace is optional (NULL, 0): with chip_mul_mat_f16_batched_workspace_size bytes of it,
 * 64 or more (query head, token) pairs per KV head go through the fp16 MFMA GEMM (K >= 64, y's batches adjacent:
 * ldy2 == n * ldy1); without it, and for fewer pairs, dot-product kernels round the activations on the fly. */
CHIP_API size_t chip_mul_mat_f16_batched_workspace_size(int64_t K, int64_t N, int64_t ne02, int64_t ne12, int64_t n);
CHIP_API int chip_mul_mat_f16_batched(const void *W, size_t nb01, size_t nb02, int64_t K, int64_t N, int64_t ne02,
                                      const float *x, int64_t ldx1, int64_t ldx2, int64_t n, int64_t ne12, float *y,
                                      int64_t ldy1, int64_t ldy2, void *workspace, size_t workspace_bytes, void *stream);

/* The kqv matmul together with the node that follows it in build_attn_mha, cont(permute(kqv, 0, 2, 1, 3)) (reference
 * llama-graph.cpp:1154-1158: the heads of a token put side by side for the output projection): the same matmul, each value
 * also stored at y2[b * ld2y2 + t * ld2y1 + r] (for the merge ld2y2 = N, ld2y1 = ne12 * N), which saves the CONT's launch in a
 * decode step.  Both copies hold the bits of chip_mul_mat_f16_batched.  Taken where that call runs its dot-product kernels
 * (chip_mul_mat_f16_batched_second_copy_supported returns 1): at most 4 (query head, token) pairs per KV head, i.e.
 * (ne12 / ne02) * n <= 4; CHIP_EUNSUPPORTED otherwise, nothing written, and the caller runs the two nodes.  y2 must not
 * overlap W, x or y. */
CHIP_API int chip_mul_mat_f16_batched_second_copy_supported(int64_t ne02, int64_t ne12, int64_t n);
CHIP_API int chip_mul_mat_f16_batched_two_copies(const void *W, size_t nb01, size_t nb02, int64_t K, int64_t N, int64_t ne02,
                                                 const float *x, int64_t ldx1, int64_t ldx2, int64_t n, int64_t ne12, float *y,
                                                 int64_t ldy1, int64_t ldy2, float *y2, int64_t ld2y1, int64_t ld2y2,
                                                 void *workspace, size_t workspace_bytes, void *stream);

/* ---- the attention-side ops around the KV cache ----
 *   chip_soft_max : LM_GGML_OP_SOFT_MAX (lm_ggml_soft_max_ext), lm_ggml_compute_forward_soft_max_f32 (ggml-cpu/ops.cpp:4731-4827):
 *                   y[r] = softmax(x[r] * scale + mask[r % ne01]) over n_rows rows of ne00 values; mask NULL, or a dense
 *                   [>= ne01][ne00] matrix of mask_type LM_GGML_TYPE_F32 / _F16 shared by all heads.  Bit for bit the AVX2
 *                   build (lm_ggml_v_expf, groups of 8 summed in the reference's order); ne00 must be a multiple of 8 (the
 *                   reference finishes other rows with the C library's expf) and max_bias 0 (ALiBi slopes are declined).
 *                   x, y, mask 16-byte aligned, ldx and ldy multiples of 4.  In place (y == x) is allowed.
 *   chip_cpy      : LM_GGML_OP_CPY / LM_GGML_OP_CONT / LM_GGML_OP_DUP, lm_ggml_compute_forward_dup (ggml-cpu/ops.cpp), between
 *                   F32 and F16 tensors of one element count: element i of the source in its logical order (shape
 *                   ne_src[4], byte strides nb_src[4]) becomes element i of the destination (ne_dst[4], nb_dst[4]).  The
 *                   K-cache store (F32 -> F16, both dense), the transposed V-cache store (transposed source, strided
 *                   destination), the permuted attention output made dense under a new shape.
 *                   F32 -> F16 rounds to nearest even like LM_GGML_FP32_TO_FP16's F16C conversion.
 *   chip_rope     : LM_GGML_OP_ROPE (lm_ggml_rope_ext), lm_ggml_compute_forward_rope_f32 (ggml-cpu/ops.cpp:5178-5361), modes 0
 *                   (adjacent pairs) and LM_GGML_ROPE_TYPE_NEOX = 2; x, y F32 [ne2 tokens][ne1 heads][ne0] with head stride
 *                   ld?1 and token stride ld?2 in elements, pos I32 [ne2], freq_factors F32 [n_dims / 2] or NULL; YaRN
 *                   parameters as in the reference.  The angles follow the reference's float recurrence; cos and sin are
 *                   computed in double and rounded once, where the reference calls the C library's cosf / sinf: results
 *                   agree to one unit in the last place of cos / sin (|dy| <= 4e-7 * (|x0| + |x1|) * mscale).  Multi-section
 *                   and vision modes are declined.  In place is allowed. */
CHIP_API int chip_soft_max(const float *x, int64_t ldx, const void *mask, int mask_type, int64_t ne00, int64_t ne01,
                           int64_t n_rows, float scale, float max_bias, float *y, int64_t ldy, void *stream);
CHIP_API int chip_cpy(const void *src, int src_type, const int64_t ne_src[4], const int64_t nb_src[4], void *dst, int dst_type,
                      const int64_t ne_dst[4], const int64_t nb_dst[4], void *stream);
/*   chip_get_rows : LM_GGML_OP_GET_ROWS, lm_ggml_compute_forward_get_rows (ggml-cpu/ops.cpp:4236-4453): dst row (i10, i11, i12) =
 *                   row ids[i10, i11, i12] of matrix (i11, i12) of src, converted to F32 with the type's dequantize_row_*
 *                   (ggml-quants.c) - bit for bit.  src: F32, F16 or any weight type of this library, rows of nc values
 *                   (whole blocks) at nb01 bytes, matrices at nb02 / nb03 bytes; ids I32 with strides ldi1 / ldi2 in
 *                   elements; dst strides in floats.  An id outside [0, ne01) leaves its row unwritten (the reference
 *                   asserts). */
CHIP_API int chip_get_rows(int type, const void *src, size_t nb01, size_t nb02, size_t nb03, int64_t nc, int64_t ne01,
                           const int32_t *ids, int64_t ne10, int64_t ne11, int64_t ne12, int64_t ldi1, int64_t ldi2, float *dst,
                           int64_t ld1, int64_t ld2, int64_t ld3, void *stream);
CHIP_API int chip_rope(const float *x, int64_t ldx1, int64_t ldx2, const int32_t *pos, const float *freq_factors, int64_t ne0,
                       int64_t ne1, int64_t ne2, int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale,
                       float ext_factor, float attn_factor, float beta_fast, float beta_slow, float *y, int64_t ldy1,
                       int64_t ldy2, void *stream);
/* chip_rope in two steps, for graphs that rotate many tensors by the same positions (Q and K of every layer): the
 * reference rebuilds its cos / sin cache per row block (lm_ggml_rope_cache_init, ggml-cpu/ops.cpp:5104-5118); here
 * chip_rope_table writes it once - table[token][cos of the n_dims / 2 pairs | sin of the pairs], n_dims floats per token,
 * already scaled - and chip_rope_apply rotates with it.  Results are bit-identical to chip_rope. */
CHIP_API int chip_rope_table(const int32_t *pos, const float *freq_factors, int64_t ne2, int n_dims, int n_ctx_orig,
                             float freq_base, float freq_scale, float ext_factor, float attn_factor, float beta_fast,
                             float beta_slow, float *table, void *stream);
CHIP_API int chip_rope_apply(const float *x, int64_t ldx1, int64_t ldx2, const float *table, int64_t ne0, int64_t ne1,
                             int64_t ne2, int n_dims, int mode, float *y, int64_t ldy1, int64_t ldy2, void *stream);
/* chip_rope_apply that also stores the result rounded to fp16 (round to nearest even, as lm_ggml_cpu_fp32_to_fp16 does):
 * the RoPE of K and the CPY into the F16 cache that follows it (llama-kv-cache.cpp cpy_k) in one launch.  y_f16 takes
 * the element at (i0, head, token) at i0 + head * ld16_1 + token * ld16_2 halves.  Bit-identical to chip_rope_apply
 * followed by chip_cpy F32 -> F16. */
CHIP_API int chip_rope_apply_store(const float *x, int64_t ldx1, int64_t ldx2, const float *table, int64_t ne0, int64_t ne1,
                                   int64_t ne2, int n_dims, int mode, float *y, int64_t ldy1, int64_t ldy2, uint16_t *y_f16,
                                   int64_t ld16_1, int64_t ld16_2, void *stream);
/* Two tensors rotated with one table in one launch: Q and K of a layer, which the reference rotates in two ROPE nodes with the
 * same positions and parameters (cactus/llama-model.cpp build_llama: lm_ggml_rope_ext on Qcur and on Kcur).  Each operand has
 * its own heads (ne1), strides and outputs: y (F32) and / or y_f16 (the fp16 copy chip_rope_apply_store makes, i.e. the K
 * cache store that follows K's ROPE); one of the two may be NULL - with y NULL only the fp16 copy is written, for a ROPE
 * whose F32 result nobody else reads.  Every value written has the bits chip_rope_apply / chip_rope_apply_store give. */
typedef struct chip_rope_operand {
    const float *x; int64_t ldx1, ldx2;        /* input: head and token strides in floats */
    int64_t ne1;                               /* heads */
    float *y; int64_t ldy1, ldy2;              /* F32 result or NULL */
    uint16_t *y_f16; int64_t ld16_1, ld16_2;   /* fp16 copy or NULL: head and token strides in halves */
} chip_rope_operand;
CHIP_API int chip_rope_apply_two(const chip_rope_operand *a, const chip_rope_operand *b, const float *table, int64_t ne0,
                                 int64_t ne2, int n_dims, int mode, void *stream);


/* ---- Q6_K rows in planes ----
 * No counterpart in the reference, whose CPU kernels read block_q6_K (ggml-common.h:332-338) as stored in the file.
 * A row of K / 256 super-blocks of 210 bytes is laid out as four planes instead - all ql fields (128 bytes each), then all
 * qh (64), then all scales (16), then all d (2) - in the same 210 * K / 256 bytes.  With K % 2048 == 0 every load of the
 * decode GEMV then starts at a multiple of its own size, where block_q6_K's 210-byte pitch leaves them 2-byte aligned;
 * results are the same bits as on the block layout.
 *   to_planes != 0: block order -> planes; 0: planes -> block order (the inverse, byte for byte)
 *   dst == src with nb01_dst == nb01_src repacks in place; otherwise the two matrices must not overlap
 *   K % 2048 == 0, rows of at most the device's LDS per workgroup (160 KB: K <= 196608); src, dst, strides 2-byte aligned
 *   (chip_mul_mat and the other matmul entry points ask 16-byte alignment of a CHIP_TYPE_Q6_K_PLANES matrix and stride) */
CHIP_API int chip_repack_q6_K(const void *src, size_t nb01_src, void *dst, size_t nb01_dst, int64_t K, int64_t N,
                              int to_planes, void *stream);

/* ---- verification hooks ----
 * Per-block integer sums of lm_ggml_vec_dot_{q4_0_q8_0,q8_0_q8_0,q4_K_q8_K,q6_K_q8_K,q5_0_q8_0,q5_K_q8_K,
 * iq4_nl_q8_0} (ggml-cpu/ggml-cpu-quants.c:1906,3591,6772,8520,2924,7699,12751), computed with the same device
 * code the GEMV uses.
 *   aq   : n rows of activations in the reference block layout (chip_quantize_q8_0 / _q8_K output)
 *   isum : [n][N][K/block] int32; for Q4_K/Q5_K/Q6_K one value per 256-block (sum over sub-blocks of scale*dot)
 *   imin : Q4_K and Q5_K only, [n][N][K/256] int32 (sum of min_j * bsum pairs); NULL otherwise */
CHIP_API int chip_block_isums(int type, const void *W, size_t nb01, int64_t K, int64_t N,
                              const void *aq, int64_t n, int32_t *isum, int32_t *imin, void *stream);
/* on != 0: Q6_K matmuls of 5 to 8 tokens take the matrix-core GEMV on every shape it supports, not only on the very
 * large matrices where it is the default, so tests can run that kernel on small inputs; 0 restores the default. */
CHIP_API int chip_verify_force_q6k_matrix_core(int on);
/* Rebuilds the reference block layout from a prepared workspace (inverse of the kernel-private layout), so
 * tests can check that the fused prepare step quantizes bit-identically to chip_quantize_q8_0/_q8_K. */
CHIP_API int chip_workspace_to_blocks(int type, int64_t K, int64_t n, const void *workspace, void *y, void *stream);

#ifdef __cplusplus
}
#endif
#endif
