/*
 * oracle.h -- CPU restatement of the reference's quantized MUL_MAT path.
 *
 * TEST INFRASTRUCTURE ONLY.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load
 * this library, and there only as the checker.  The product (libcactus_hip.so, libggml-hip.so) never links,
 * loads or falls back to anything in this directory.
 *
 * Every function restates, in plain scalar C, what the reference computes on an x86-64 AVX2 build, citing the
 * reference file:line it follows (paths relative to the reference's cactus/ directory).  Pinning status:
 *
 *   function                         pinned by
 *   -------------------------------  -------------------------------------------------------------------------
 *   orc_fp16_to_fp32/fp32_to_fp16    exhaustive over all 65536 halves / edge+random floats vs numpy (IEEE RNE)
 *   orc_quantize_row_q8_0            bit-exact vs oracle/_ref on seeded data + committed golden vectors;
 *                                    invariants (max element -> +-127, zero block, ties-to-even cases)
 *   orc_quantize_row_q8_0_ref        bit-exact vs oracle/_ref + golden; half-away-from-zero tie cases
 *   orc_quantize_row_q8_K            bit-exact vs oracle/_ref + golden; bsums == sum of 16, first-max sign rule
 *   orc_quantize_row_q4_0_ref        bit-exact vs oracle/_ref + golden; dequant closed form d*(nib-8)
 *   orc_quantize_row_q4_K_ref        bit-exact vs oracle/_ref + golden (iterative search: only the oracle run
 *   orc_quantize_row_q6_K_ref          pins the bytes); reconstruction-error bound as a sanity invariant
 *   orc_quantize_row_q5_0_ref/_q5_K_ref  bit-exact vs oracle/_ref + golden; dequant closed forms
 *   orc_quantize_row_q4_1_ref/_q5_1_ref  bit-exact vs oracle/_ref + golden; dequant closed form d*u + m
 *   orc_quantize_row_q8_1            bit-exact vs oracle/_ref on seeded data + golden edge rows; quants and d
 *                                    equal orc_quantize_row_q8_0's, s == fp16(d * sum q) on finite rows
 *   (iq4_nl, iq4_xs, q2_K and q3_K have no quantizer here: their weights come from oracle/_ref, committed in the golden
 *    fixtures, or are random quant bits with plausible scales -- any byte string is a valid block of these types)
 *   orc_dequantize_row_*             closed forms; vs oracle/_ref + golden
 *   orc_vec_dot_*                    integer sums: brute force from dequantised integers; float result: bit-exact
 *                                    vs oracle/_ref (the AVX2 lane structure is restated) + golden; fp64 identity
 *                                    sum(dequant(x)*dequant(y))
 *   orc_fp32_to_fp16_row, orc_vec_dot_f16  conversion: the exhaustive fp16 checks above; dot: bit-exact vs oracle/_ref
 *                                    (lane structure restated) + golden; fp64 identity sum w_i * x_i
 *   orc_mul_mat                      == n*N independent vec_dots; vs oracle/_ref's LM_GGML_OP_MUL_MAT graph
 *   orc_mul_mat_id                   == orc_mul_mat per (token, slot) on the expert the id names; vs oracle/_ref's
 *                                       LM_GGML_OP_MUL_MAT_ID graph (bit-exact, tests/test_oracle_vs_ref.py)
 *
 * No function here is "parity unpinned".
 */
#ifndef CACTUS_ORACLE_H
#define CACTUS_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* type ids are the reference's lm_ggml_type values (ggml.h:351-391) */
enum orc_type {
    ORC_TYPE_F32  = 0,
    ORC_TYPE_F16  = 1,      /* as a weight type and as its own activation format */
    ORC_TYPE_Q4_0 = 2,
    ORC_TYPE_Q8_0 = 8,
    ORC_TYPE_Q4_K = 12,
    ORC_TYPE_Q6_K = 14,
    ORC_TYPE_Q8_K = 15,
    /* further weight types (same activation quantizers) */
    ORC_TYPE_Q5_0 = 6,
    ORC_TYPE_Q5_K = 13,
    ORC_TYPE_IQ4_NL = 20,
    ORC_TYPE_Q4_1 = 3,
    ORC_TYPE_Q5_1 = 7,
    ORC_TYPE_Q8_1 = 9,      /* activation format of Q4_1 / Q5_1 */
    ORC_TYPE_Q2_K = 10,
    ORC_TYPE_Q3_K = 11,
    ORC_TYPE_IQ4_XS = 23,
};

/* elements per block / bytes per block / bytes per row of k elements; 0 for an unknown type */
int    orc_block_elems(int type);
size_t orc_block_bytes(int type);
size_t orc_row_size(int type, int64_t k);
/* activation type a weight type is dotted with (type_traits_cpu[].vec_dot_type, ggml-cpu/ggml-cpu.c:198-367) */
int    orc_vec_dot_type(int type);

float    orc_fp16_to_fp32(uint16_t h);
uint16_t orc_fp32_to_fp16(float f);

/* activation quantizers (the two the MUL_MAT op calls on the fly) */
void orc_quantize_row_q8_0(const float *x, void *y, int64_t k);      /* AVX2 semantics */
void orc_quantize_row_q8_K(const float *x, void *y, int64_t k);
void orc_quantize_row_q8_1(const float *x, void *y, int64_t k);      /* AVX2 semantics */
void orc_fp32_to_fp16_row(const float *x, void *y, int64_t k);       /* fp16 round to nearest even */

/* weight quantizers (offline; their output bytes are the op's input) */
void orc_quantize_row_q4_0_ref(const float *x, void *y, int64_t k);
void orc_quantize_row_q8_0_ref(const float *x, void *y, int64_t k);
void orc_quantize_row_q4_K_ref(const float *x, void *y, int64_t k);
void orc_quantize_row_q6_K_ref(const float *x, void *y, int64_t k);
void orc_quantize_row_q5_0_ref(const float *x, void *y, int64_t k);
void orc_quantize_row_q5_K_ref(const float *x, void *y, int64_t k);
void orc_quantize_row_q4_1_ref(const float *x, void *y, int64_t k);
void orc_quantize_row_q5_1_ref(const float *x, void *y, int64_t k);
/* dispatch on weight type, nrows rows of k elements, rows packed back to back; returns bytes written */
size_t orc_quantize_rows(int type, const float *x, void *y, int64_t nrows, int64_t k);

void orc_dequantize_row(int type, const void *x, float *y, int64_t k);

/*
 * Dot products.  Each returns the fp32 value the reference's AVX2 branch produces (same lane structure, same
 * fused multiply-adds, same horizontal-sum order) and optionally the exact integer sums:
 *   q4_0/q8_0 : isum[k/32]   = sum over the block of wq*aq                (wq already offset by -8 for q4_0)
 *   q4_K      : isum[k/256]  = sum_j sc_j * sum_{i<32} q4*q8 ; imin[k/256] = sum_j m_j*(bsums[2j]+bsums[2j+1])
 *   q6_K      : isum[k/256]  = sum_j sc_j * sum_{i<16} (q6-32)*q8
 * Pass NULL to skip an output.
 */
float orc_vec_dot_q4_0_q8_0(int64_t k, const void *vx, const void *vy, int32_t *isum);
float orc_vec_dot_q8_0_q8_0(int64_t k, const void *vx, const void *vy, int32_t *isum);
float orc_vec_dot_q4_K_q8_K(int64_t k, const void *vx, const void *vy, int32_t *isum, int32_t *imin);
float orc_vec_dot_q6_K_q8_K(int64_t k, const void *vx, const void *vy, int32_t *isum);
/* q5_0, iq4_nl: isum[k/32] = sum (q5-16)*aq resp. sum codebook[nib]*aq ; q5_K: as q4_K with 5-bit quants */
float orc_vec_dot_q5_0_q8_0(int64_t k, const void *vx, const void *vy, int32_t *isum);
float orc_vec_dot_iq4_nl_q8_0(int64_t k, const void *vx, const void *vy, int32_t *isum);
float orc_vec_dot_q5_K_q8_K(int64_t k, const void *vx, const void *vy, int32_t *isum, int32_t *imin);
/* q4_1, q5_1: isum[k/32] = sum u*aq with the unsigned weight u; the min term m*s is not part of isum */
float orc_vec_dot_q4_1_q8_1(int64_t k, const void *vx, const void *vy, int32_t *isum);
float orc_vec_dot_q5_1_q8_1(int64_t k, const void *vx, const void *vy, int32_t *isum);
/* q2_K: isum[k/256] = sum_g (sc_g & 15) * sum_{i<16} q2*q8, imin[k/256] = sum_g (sc_g >> 4) * bsums[g];
 * q3_K: isum[k/256] = sum_g (scale_g - 32) * sum_{i<16} (q3 - 4)*q8   (g: the sixteen 16-value sub-blocks) */
float orc_vec_dot_q2_K_q8_K(int64_t k, const void *vx, const void *vy, int32_t *isum, int32_t *imin);
float orc_vec_dot_q3_K_q8_K(int64_t k, const void *vx, const void *vy, int32_t *isum);
/* iq4_xs: isum[k/256] = sum_ib (ls_ib - 32) * sum_{i<32} codebook[nib]*q8   (ib: the eight 32-value sub-blocks) */
float orc_vec_dot_iq4_xs_q8_K(int64_t k, const void *vx, const void *vy, int32_t *isum);
float orc_vec_dot_f16(int64_t k, const void *vx, const void *vy);   /* both operands fp16, fp32 fmadd lanes */
float orc_vec_dot(int type, int64_t k, const void *vx, const void *vy);

/* fp64 evaluation of sum_b scale_b*isum_b (returned) and of sum_b |scale_b*isum_b| (*sum_abs): the tolerance
 * yardstick 1e-5 * sum_abs and an order-free reference value.  A "block" is the smallest group of values that
 * carries its own scale: 32 values for Q4_0/Q8_0, a 32-value sub-block for Q4_K (terms d*sc_j*dot_j and
 * dmin*m_j*bsum_j, both counted), a 16-value sub-block for Q6_K (d*sc_j*dot_j); Q5_0 and
 * IQ4_NL as Q4_0, Q5_K as Q4_K;
 * Q4_1 / Q5_1: d*dy*isum and m*s per 32-block, both counted; F16: every product w_i * x_i.  Coarser terms (whole
 * super-blocks) would cancel internally and make a bound that the reference's own AVX2 result misses. */
double orc_vec_dot_exact(int type, int64_t k, const void *vx, const void *vy, double *sum_abs);

/*
 * MUL_MAT as the CPU backend computes it (ggml-cpu/ggml-cpu.c:1257-1449): quantize each of the n activation
 * rows x[t][0..K) to the weight type's vec_dot_type, then y[t][r] = vec_dot(W row r, quantized row t).
 *   W     : N rows of orc_row_size(type, K) bytes, packed
 *   x     : n rows of K floats;   y : n rows of N floats
 *   wdata : optional out, n rows of orc_row_size(vec_dot_type, K) bytes (the quantized activations)
 *   sum_abs : optional out, n*N doubles (tolerance yardstick per output)
 *   nthreads: rows are split over this many pthreads (>=1)
 */
void orc_mul_mat(int type, int64_t K, int64_t N, int64_t n, const void *W, const float *x, float *y,
                 void *wdata, double *sum_abs, int nthreads);
/* LM_GGML_OP_MUL_MAT_ID: W holds n_as expert matrices [N][row_size] back to back, x is [n_tokens][ne11][K], ids is
 * [n_tokens][n_used], y (and sum_abs, may be NULL) [n_tokens][n_used][N].  Returns 0, or -2 for an id out of range. */
int orc_mul_mat_id(int type, int64_t K, int64_t N, int64_t n_as, const void *W, const float *x, int64_t ne11,
                   const int32_t *ids, int64_t n_used, int64_t n_tokens, float *y, double *sum_abs, int nthreads);

/* Element-wise ops of an FFN block, restated from ggml-cpu/ops.cpp and ggml-cpu/vec.{h,cpp} (AVX2 + FMA build);
 * rows are contiguous.  Pinned bit-exact on oracle/_ref's graphs (tests/test_oracle_vs_ref.py).  ADD and MUL are
 * single IEEE operations per element and need no restatement. */
void orc_rms_norm_f32(const float *x, float *y, int64_t n_rows, int64_t ne0, float eps);
void orc_silu_f32(const float *x, float *y, int64_t n_rows, int64_t ne0);
/* LM_GGML_UNARY_OP_GELU through the reference's fp16 table (ggml-cpu/vec.h:452-466, table of ggml-cpu/ggml-cpu.c:3474-3481);
 * pinned bit-exact on oracle/_ref's lm_ggml_gelu graph, and by gelu(0) = 0, gelu(x) = x from 10 on, 0 down from -10. */
void orc_gelu_table(uint16_t *table);
void orc_gelu_f32(const float *x, float *y, int64_t n);

/* Attention-side ops (ggml-cpu/ops.cpp), contiguous rows.  orc_soft_max_f32: pinned bit-exact on oracle/_ref's
 * lm_ggml_soft_max_ext graphs.  orc_rope_f32: pinned bit-exact on oracle/_ref's lm_ggml_rope_ext graphs on this host (both
 * call the same C library cosf / sinf); a device computes those two functions itself, so its parity with this function
 * is a tolerance, stated in the GPU test. */
void orc_soft_max_f32(const float *x, const void *mask, int mask_is_f16, int64_t ne00, int64_t ne01, int64_t n_head,
                      int64_t n_rows, float scale, float max_bias, float *y);
void orc_rope_f32(const float *x, const int32_t *pos, const float *freq_factors, int64_t ne0, int64_t ne1, int64_t ne2,
                  int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale, float ext_factor,
                  float attn_factor, float beta_fast, float beta_slow, float *y);

#ifdef __cplusplus
}
#endif
#endif
