/*
 * ggml_backend_hip.h -- entry points of libggml-hip.so, the ggml backend that runs LM_GGML_OP_MUL_MAT over
 * block-quantized weights on an MI355X through the C-ABI of cactus_hip.h.
 *
 * It implements the reference's backend interface (ggml-backend-impl.h:17-207): a registry entry with one
 * device, a buffer type that keeps GGUF blocks in their on-disk layout in HBM, and a backend (stream) whose
 * graph_compute handles MUL_MAT and the view ops.  Everything else stays on the CPU backend; the reference's
 * scheduler splits the graph accordingly (ggml-backend.cpp:730-785).
 *
 * Three ways to make it visible to llama.cpp / cactus_context (reference ggml-backend-reg.cpp:162-193,305,401):
 *   - dynamic:  lm_ggml_backend_load("libggml-hip.so")  (or LM_GGML_BACKEND_PATH) -> calls lm_ggml_backend_init()
 *   - explicit: lm_ggml_backend_register(lm_ggml_backend_hip_reg()) before the first model load
 *   - built in: an `#ifdef LM_GGML_USE_HIP  register_backend(lm_ggml_backend_hip_reg());` line in the registry
 * The library resolves lm_ggml_backend_buffer_init, lm_ggml_nbytes and lm_ggml_log_internal from the process
 * that loads it.
 */
#ifndef CACTUS_GGML_BACKEND_HIP_H
#define CACTUS_GGML_BACKEND_HIP_H

#ifdef __cplusplus
extern "C" {
#endif

struct lm_ggml_backend_reg;
struct lm_ggml_backend;
struct lm_ggml_backend_buffer_type;

#define CACTUS_GGML_API __attribute__((visibility("default")))

/* The registry entry ("HIP", one device "HIP0").  Counterpart of lm_ggml_backend_cpu_reg()
 * (ggml-cpu/ggml-cpu.cpp:658-669).  Returns a reg with zero devices if no gfx950 GPU is usable. */
CACTUS_GGML_API struct lm_ggml_backend_reg *lm_ggml_backend_hip_reg(void);

/* Dynamic-loading entry points looked up by lm_ggml_backend_load (ggml-backend-impl.h:215-246,
 * ggml-backend-reg.cpp:227-271): score 0 means "not usable on this machine". */
CACTUS_GGML_API struct lm_ggml_backend_reg *lm_ggml_backend_init(void);
CACTUS_GGML_API int lm_ggml_backend_score(void);

/* Direct construction, like lm_ggml_backend_cpu_init() (ggml-cpu/ggml-cpu.cpp:195-225) and
 * lm_ggml_backend_cpu_buffer_type() (ggml-backend.cpp:1985). */
CACTUS_GGML_API struct lm_ggml_backend *lm_ggml_backend_hip_init(void);
CACTUS_GGML_API struct lm_ggml_backend_buffer_type *lm_ggml_backend_hip_buffer_type(void);
CACTUS_GGML_API int lm_ggml_backend_is_hip(struct lm_ggml_backend *backend);

/* Counters for tests and tracing: MUL_MAT nodes executed on the GPU and bytes uploaded by set_tensor. */
CACTUS_GGML_API void lm_ggml_backend_hip_get_stats(unsigned long long *mul_mat_nodes, unsigned long long *uploaded_bytes);
/* Pairs of adjacent nodes (RMS_NORM + MUL, SILU + MUL) that graph_compute ran as one kernel. */
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_fused_pairs(void);
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_quantizers_skipped(void);   /* matmuls that reused the previous one's quantized input */
/* cos / sin tables built for ROPE nodes (one per graph_compute call and set of parameters; the other ROPE nodes apply it). */
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_rope_tables(void);
/* Bytes that arrived through set_tensor_async (the model loader's pinned-staging upload loop,
 * cactus/llama-model-loader.cpp:1047-1064); a subset of uploaded_bytes above. */
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_async_uploaded(void);
/* MUL_MAT nodes that ran in one launch with other projections of the same activation tensor (Qcur / Kcur / Vcur of an
 * attention block, cactus/llama-model.cpp build_llama), up to 4 tokens. */
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_grouped_matmuls(void);
/* kqv MUL_MAT nodes that also wrote the head merge that follows them, CONT(PERMUTE(kqv)) (cactus/llama-graph.cpp:1154-1158),
 * up to 4 (query head, token) pairs per KV head. */
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_head_merges(void);
/* ROPE nodes that ran in the launch of an earlier ROPE with the same positions and parameters (K's with Q's). */
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_rope_pairs(void);
/* Gated FFNs whose four nodes ffn_gate, SILU, ffn_up, MUL (cactus/llama-graph.cpp:562-690) ran as one launch, up to 4 tokens. */
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_gated_pairs(void);
/* ROPE nodes that ran in the epilogue of the projection in front of them (Q's and K's, in the group launch of wq / wk / wv). */
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_rope_epilogues(void);
/* RMS_NORM + weight MUL pairs (cactus/llama-graph.cpp build_norm) that ran in the prologue of the projections reading them (the
 * group launch of wq / wk / wv, the gated FFN launch), up to 2 tokens (at 4 the norm's own launch is the faster form). */
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_norms_in_prologue(void);
/* Residual ADD nodes that ran where the projection in front of them (wo, ffn_down) stores its result, up to 4 tokens. */
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_residual_adds(void);
/* Q6_K weights in planes.  The decode GEMVs (up to 4 tokens) read a 2-D Q6_K weight of K % 2048 == 0 from a second copy whose
 * rows chip_repack_q6_K laid out in planes; the backend makes the copy at the weight's first such matmul (210 * K / 256 bytes
 * per row of device memory more, skipped when less than that plus 1 GiB is free) and drops it when set_tensor, memset_tensor,
 * cpy_tensor, clear or a graph node writes over the weight.  CACTUS_HIP_Q6K_PLANES=0 in the environment turns this off.
 * Counters: copies made, their bytes, copies dropped, matmul operands read from a copy. */
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_planes_copies(void);
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_planes_bytes(void);
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_planes_dropped(void);
CACTUS_GGML_API unsigned long long lm_ggml_backend_hip_get_planes_matmuls(void);

#ifdef __cplusplus
}
#endif
#endif
