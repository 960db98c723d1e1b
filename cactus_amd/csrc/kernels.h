// Internal launch interface between the C-ABI layer (capi.hip) and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <atomic>
#include <cstdlib>
#include "dev_common.h"

namespace chip {

// Dispatch thresholds and kernel shapes are constants of the library.  A build with -DCHIP_TUNING (make TUNING=1, never
// the default) lets the environment variable `name` replace one of them for a measurement sweep.
#ifdef CHIP_TUNING
inline int64_t tune(const char *name, int64_t dflt) { const char *e = getenv(name); return e ? (int64_t)atoll(e) : dflt; }
#else
inline constexpr int64_t tune(const char *, int64_t dflt) { return dflt; }
#endif

// Verification hook (chip_verify_force_q6k_matrix_core): the Q6_K matrix-core GEMV on shapes below its size threshold.
extern std::atomic<int> g_force_mmv_q6k;


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

// Output-tile order for the GEMM kernels.  The hardware hands consecutive workgroup ids to the 8 XCDs in turn, and each
// XCD has its own L2.  Tiles are numbered block by block (sr x sc tiles per block, about as many as run on one XCD at a
// time; blocks at the far edges are smaller), the numbering is cut into 8 equal stretches, and XCD x walks stretch x:
// workgroup id L -> XCD L % 8, its (L / 8)-th tile.  The workgroups that share an L2 then read the same few weight
// rows and tokens, every XCD gets the same number of tiles, and no XCD streams the whole weight matrix.
constexpr int XCDS = 8;
struct TileMap {
    int row_tiles, tok_tiles;      // output tiles in each direction
    int sr, sc;                    // tiles per full block
    int blocks_r, blocks_c;
    unsigned tiles, per_xcd;       // tiles in all, tiles per XCD (rounded up)
    unsigned grid;                 // workgroups to launch; those numbered past the last tile exit at once
};
struct TileCoord { int row_tile, tok_tile; };
inline TileMap make_tile_map(int64_t row_tiles, int64_t tok_tiles, int concurrent_per_xcd) {
    TileMap m;
    m.row_tiles = (int)row_tiles;
    m.tok_tiles = (int)tok_tiles;
    m.blocks_c = (int)ceil_div(tok_tiles, 8);
    m.sc = (int)ceil_div(tok_tiles, m.blocks_c);
    int sr = concurrent_per_xcd / m.sc;
    if (sr < 1) sr = 1;
    m.blocks_r = (int)ceil_div(row_tiles, sr);
    m.sr = (int)ceil_div(row_tiles, m.blocks_r);
    m.tiles = (unsigned)(row_tiles * tok_tiles);
    m.per_xcd = (unsigned)ceil_div(m.tiles, XCDS);
    m.grid = m.per_xcd * XCDS;
    return m;
}
__host__ __device__ __forceinline__ TileCoord xcd_tile(unsigned wg, const TileMap &m) {
    unsigned g = (wg % XCDS) * m.per_xcd + wg / XCDS;
    TileCoord t;
    if (wg / XCDS >= m.per_xcd || g >= m.tiles) { t.row_tile = m.row_tiles; t.tok_tile = m.tok_tiles; return t; }
    const unsigned col_block = (unsigned)(m.row_tiles * m.sc);                  // tiles in a full column of blocks
    unsigned cb = g / col_block;
    if (cb > (unsigned)m.blocks_c - 1) cb = m.blocks_c - 1;
    g -= cb * col_block;
    const unsigned wc = (cb < (unsigned)m.blocks_c - 1) ? m.sc : m.tok_tiles - (m.blocks_c - 1) * m.sc;
    unsigned rb = g / (m.sr * wc);
    if (rb > (unsigned)m.blocks_r - 1) rb = m.blocks_r - 1;
    g -= rb * m.sr * wc;
    const unsigned hr = (rb < (unsigned)m.blocks_r - 1) ? m.sr : m.row_tiles - (m.blocks_r - 1) * m.sr;
    t.row_tile = (int)(rb * m.sr + g % hr);
    t.tok_tile = (int)(cb * m.sc + g / hr);
    return t;
}

// Row gather of LM_GGML_OP_MUL_MAT_ID for the GEMM kernels (reference ggml-cpu/ggml-cpu.c:1460-1710 groups the (token,
// slot) pairs by expert the same way: matrix_rows / matrix_row_counts).  With perm set, blockIdx.y walks a list of
// token tiles built on the device: entry i = expert | tile << 12 says "pairs perm[offsets[e] + tile * BN ...] of expert
// e"; entries past tiles[-1] (the count, stored in front of the list) do not exist.  The expert's matrix is
// W + e * nb02; pair p reads activation row (p / n_used) * ne11 + (p % n_used) % ne11 and writes output row p.
// perm == nullptr: plain MUL_MAT.
constexpr int MOE_EXPERT_BITS = 12;
struct RowGather {
    const int32_t *perm, *offsets, *tiles;     // tiles[0] = number of entries, entries from tiles[1]
    int32_t n_used, ne11;
    size_t nb02;
};
struct GatherView {                // resolved once per workgroup
    const int32_t *list;           // this expert's pairs, or nullptr
    int32_t n_used, ne11;
    int32_t tok_tile;              // grouped mode: the token tile of this workgroup, -1 = nothing to do
    __device__ __forceinline__ int64_t act_row(int64_t tok) const {
        if (!list) return tok;
        const int32_t p = list[tok];
        return (int64_t)(p / n_used) * ne11 + (p % n_used) % ne11;
    }
    __device__ __forceinline__ int64_t out_row(int64_t tok) const { return list ? (int64_t)list[tok] : tok; }
};
// Sets the token count M and the byte offset of the weight matrix to the expert's and returns its view.  GATHER is a
// template argument of the kernels so that the plain MUL_MAT instantiations carry none of this.
template <bool GATHER>
__device__ __forceinline__ GatherView resolve_gather(const RowGather &rg, size_t &w_offset, int64_t &M) {
    GatherView v{nullptr, rg.n_used, rg.ne11, 0};
    w_offset = 0;
    if constexpr (GATHER) {
        if ((int)blockIdx.y >= rg.tiles[0]) { v.tok_tile = -1; return v; }
        const int32_t d = rg.tiles[1 + blockIdx.y];
        const int e = d & ((1 << MOE_EXPERT_BITS) - 1);
        const int32_t off = rg.offsets[e];
        M = rg.offsets[e + 1] - off;
        v.list = rg.perm + off;
        v.tok_tile = d >> MOE_EXPERT_BITS;
        w_offset = (size_t)e * rg.nb02;
    }
    return v;
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
hipError_t launch_gemv_fused_store_t(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, int n,
                                     void *ws, size_t ws_stride, float *y, int64_t ldy, unsigned short *y16t, int64_t ld16,
                                     const DeviceLimits &lim, hipStream_t st);
hipError_t launch_gemv_fused_pair(int wtype, const void *W1, const void *W2, size_t nb01, int64_t K, int64_t N, const float *x,
                                  int64_t ldx, int n, void *ws, size_t ws_stride, float *y1, float *y2, int64_t ldy,
                                  const DeviceLimits &lim, hipStream_t st);
// silu(W1 x) * (W2 x) -> y in one launch: the gated FFN's four nodes up to ffn_down's input (shapes as launch_gemv_fused_pair)
bool gemv_norm_prologue_applicable(int wtype, int64_t K, int n, const DeviceLimits &lim);
// norm_w != nullptr: the rows x are RMS-normed (norm_eps) and multiplied by norm_w in the prologue; norm_y may receive them
hipError_t launch_gemv_fused_pair_silu_mul(int wtype, const void *W1, const void *W2, size_t nb01, int64_t K, int64_t N, const float *x,
                                           int64_t ldx, int n, void *ws, size_t ws_stride, float *y, int64_t ldy,
                                           const DeviceLimits &lim, hipStream_t st, const float *norm_w = nullptr, float norm_eps = 0.f,
                                           float *norm_y = nullptr, int64_t norm_ldy = 0);
// y = W x + addend (addend [n][N] at ld_add): the GEMV that quantizes in its prologue with the residual ADD in its store
hipError_t launch_gemv_fused_add(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const float *x, int64_t ldx, int n, void *ws,
                                 size_t ws_stride, const float *addend, int64_t ld_add, float *y, int64_t ldy, const DeviceLimits &lim,
                                 hipStream_t st);
// gemv_group.hip: up to GROUP_MAX matrices that read the same activation rows in one launch of the prologue-quantizing
// GEMV (members of one family: K-quants, 32-value block types, or F16).  t16: optional transposed fp16 copy of a member's
// output, as launch_gemv_fused_store_t.
// The ROPE node that follows a projection (reference llama-model.cpp build_llama: lm_ggml_rope_ext on Qcur and on Kcur;
// lm_ggml_compute_forward_rope_f32, ggml-cpu/ops.cpp:5178-5361, modes 0 and NEOX) run in the projection's kernel (ROPED): the
// rows are heads of head_dim values; a wave takes the two rows of a rotated pair one after the other - (2j, 2j + 1) of a
// head, or (j, j + n_dims / 2) in NEOX mode; rows past n_dims pass through - so both values sit in neighbouring lanes of its
// result registers, and what is stored is the pair rotated by the cos / sin of token t and pair j from table (the layout
// chip_rope_table writes: per token the n_dims / 2 cosines, then the sines), with the ROPE kernel's two expressions.  The
// projection's own result is not stored.  y: the ROPE's F32 result (if write_f32), h16: its fp16 copy [token][row] (the K
// cache store), or nullptr.
struct RopeEpilogue { const float *table; int head_dim, n_dims, neox, write_f32; unsigned short *h16; int64_t h16_ld; };
constexpr RopeEpilogue kNoRope = {nullptr, 0, 0, 0, 0, nullptr, 0};
constexpr int GROUP_MAX = 4;
struct GroupMat { int wtype; const void *W; size_t nb01; int64_t N; float *y; int64_t ldy; unsigned short *t16; int64_t t16_ld;
                  RopeEpilogue rope = kNoRope; };
// the RMS norm (and weight MUL) of the rows x in the prologue of a group launch whose members carry ROPE epilogues
struct GroupNorm { const float *w; float eps; float *y; int64_t ldy; };
int        gemv_group_family(int wtype);
bool       gemv_group_applicable(const GroupMat *mats, int count, int64_t K, int n, const DeviceLimits &lim, bool prepared = false);
// the GEMV over prepared rows for two matrices of one shape in one launch, and with a transposed fp16 copy of the result
hipError_t launch_gemv_pair(int wtype, const void *W1, const void *W2, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                            int n, float *y1, float *y2, int64_t ldy, const DeviceLimits &lim, hipStream_t st);
hipError_t launch_gemv_store_t(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n,
                               float *y, int64_t ldy, unsigned short *y16t, int64_t ld16, const DeviceLimits &lim, hipStream_t st);
hipError_t launch_gemv_group(const GroupMat *mats, int count, int64_t K, const float *x, int64_t ldx, int n, void *ws,
                             size_t ws_stride, const DeviceLimits &lim, hipStream_t st, bool prepared = false,
                             const GroupNorm *norm = nullptr);
// MUL_MAT_ID: every (token, slot) pair is a one-token GEMV on the expert ids[token][slot] names (W + id * nb02), its
// activation row token * ne11 + slot % ne11, its output row token * n_used + slot.  fused: x is fp32 and is quantized in
// the prologue; otherwise ws already holds the quantized rows.
hipError_t launch_gemv_id(int wtype, bool fused, const void *W, size_t nb01, size_t nb02, int64_t n_as, int64_t K, int64_t N,
                          const float *x, int64_t ldx, int64_t ne11, const int32_t *ids, int64_t ids_stride, int64_t n_used,
                          int64_t n_tokens, void *ws, size_t ws_stride, float *y, int64_t ldy, const DeviceLimits &lim,
                          hipStream_t st);
hipError_t launch_block_isums(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *aq, int64_t n,
                              int32_t *isum, int32_t *imin, hipStream_t st);

// gemv_mfma.hip: the same product for up to 16 tokens per launch with the integer sums on the matrix cores.
// mmv_max_tokens returns 16, 8 or 0 (shape or type not covered: use launch_gemv).
int        mmv_max_tokens(int wtype, int64_t K, int64_t N, const DeviceLimits &lim);
// gemv_mfma_q4k.hip: the Q4_K / Q5_K form (activations in the split Q8_K layout); reached through the two functions above.
int        mmv_q4k_max_tokens(int wtype, int64_t K, int64_t N, const DeviceLimits &lim);
hipError_t launch_mmv_q4k(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n,
                          float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const void *W2 = nullptr, float *y2 = nullptr);
// gemv_mfma_q4_0.hip: the Q4_0 form (activations in the split Q8_0 layout).
int        mmv_q4_0_max_tokens(int64_t K, int64_t N, const DeviceLimits &lim);
hipError_t launch_mmv_q4_0(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n, float *y,
                           int64_t ldy, const DeviceLimits &lim, hipStream_t st);
// gemv_mfma_q6k.hip: the Q6_K form (8 tokens per launch; activations in the split Q8_K layout).
int        mmv_q6k_max_tokens(int64_t K, int64_t N, const DeviceLimits &lim);
hipError_t launch_mmv_q6k(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int n, float *y,
                          int64_t ldy, const DeviceLimits &lim, hipStream_t st);
hipError_t launch_mmv(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                      int n, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st);

// gemm_block32.hip: int8-MFMA prefill GEMM over weights in 32-value blocks with one fp16 scale (Q4_0, Q8_0, Q5_0,
// IQ4_NL), activations in the split Q8_0 workspace layout.  _supported includes the token count from which it pays.
// Split K: with fewer output tiles than the machine holds workgroups, K is cut into slices that run as
// separate workgroups; their partial outputs [slice][token][row] go to `part` and launch_sum_slices adds them in slice
// order (same result on every run).  gemm_*_slices: the number of slices the launcher would use (1 = no split), and so
// the size of `part`: slices * n * N floats.
struct SplitK { float *part; size_t bytes; };
int        gemm_blk32_slices(int wtype, int64_t K, int64_t N, int64_t n, int compute_units);
int        gemm_kq_slices(int wtype, int64_t K, int64_t N, int64_t n, int compute_units);
hipError_t launch_sum_slices(const float *part, int slices, int64_t n, int64_t N, float *y, int64_t ldy, hipStream_t st);
bool       gemm_blk32_supported(int wtype, int64_t K, int64_t N, int64_t n, bool can_split = false);
hipError_t launch_gemm_blk32(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                             int64_t n, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st,
                             const RowGather *rg = nullptr, int64_t n_as = 1, SplitK split = SplitK{nullptr, 0});

// gemm_f16.hip: fp16-MFMA prefill GEMM over F16 weights, activations as fp16 in the workspace.
bool       gemm_f16_supported(int64_t K, int64_t N, int64_t n);
// f32_rows (with rg only): the activation rows as fp32, gather row R = token R % n of batch R / n, rounded to fp16 in the
// kernel's staging instead of being read from the fp16 workspace
struct F32Rows { const float *x; int64_t ldx1, ldx2, n; };
hipError_t launch_gemm_f16(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int64_t n,
                           float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const RowGather *rg = nullptr,
                           int64_t n_as = 1, int gather_tile = 64,        // gather_tile: tokens per list entry, 64 or 128
                           const F32Rows *f32_rows = nullptr);

// gemm_kquant.hip: int8-MFMA prefill GEMM over Q4_K / Q5_K / Q6_K weights, activations in the split Q8_K workspace
// layout; the integer sub-block scales ride in the MFMA operand.
bool       gemm_kq_supported(int wtype, int64_t K, int64_t N, int64_t n, bool can_split = false);
hipError_t launch_gemm_kq(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                          int64_t n, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const RowGather *rg = nullptr,
                          int64_t n_as = 1, SplitK split = SplitK{nullptr, 0});
// In the three GEMM launchers: with rg, n_as is the number of token-tile slots the grid provides in y (an upper bound
// of the tile list's length) and n is ignored; gemm_*_moe_tile_tokens gives the tile height the list must be built for.

// ops.hip: RMS_NORM, ADD, MUL, SILU over F32 rows (ldb = 0 broadcasts one row of b over all rows of a).
// LM_GGML_OP_MUL_MAT with a batched, strided F16 src0 (the attention matmuls over the KV cache):
// y[b][t][r] = sum_k W[b / r2][r][k] * fp16(x[b][t][k]); strides of W in bytes, of x and y in floats.
// With a workspace of mul_mat_f16_batched_workspace_size bytes, many columns per KV head go through the fp16 GEMM.
// y2 (optional): a second copy of the result under its own token and batch strides, for up to 4 (query head, token) pairs per
// KV head (mul_mat_f16_batched_second_copy_supported): the head merge that follows kqv in the graph.
bool mul_mat_f16_batched_supported(int64_t K);
bool mul_mat_f16_batched_second_copy_supported(int64_t r2, int64_t n);
size_t mul_mat_f16_batched_workspace_size(int64_t K, int64_t N, int64_t ne02, int64_t r2, int64_t n);
hipError_t launch_mul_mat_f16_batched(const void *W, size_t nb01, size_t nb02, int64_t K, int64_t N, int64_t ne02, const float *x,
                                      int64_t ldx1, int64_t ldx2, int64_t n, int64_t r2, float *y, int64_t ldy1, int64_t ldy2,
                                      void *workspace, size_t workspace_bytes, const DeviceLimits &lim, hipStream_t st,
                                      float *y2 = nullptr, int64_t ld2y1 = 0, int64_t ld2y2 = 0);
hipError_t launch_rms_norm(const float *x, int64_t ldx, int64_t n, int64_t ne0, float eps, float *y, int64_t ldy, hipStream_t st);
hipError_t launch_add(const float *a, int64_t lda, const float *b, int64_t ldb, int64_t ne0, int64_t n, float *y, int64_t ldy, hipStream_t st);
hipError_t launch_mul(const float *a, int64_t lda, const float *b, int64_t ldb, int64_t ne0, int64_t n, float *y, int64_t ldy, hipStream_t st);
hipError_t launch_silu(const float *x, int64_t ldx, int64_t ne0, int64_t n, float *y, int64_t ldy, hipStream_t st);
// Two adjacent graph nodes in one pass: y = (rms_norm(x)) * w with w one row (yn, if given, receives the norm), and
// y = silu(x) * b.  Each element sees the same operations in the same order as in the separate kernels.
hipError_t launch_rms_norm_mul(const float *x, int64_t ldx, int64_t n, int64_t ne0, float eps, const float *w, float *yn, int64_t ldyn,
                               float *y, int64_t ldy, hipStream_t st);
hipError_t launch_add_rms_norm_mul(const float *a, int64_t lda, const float *b, int64_t ldb, float *xs, int64_t ldxs, int64_t n,
                                   int64_t ne0, float eps, const float *w, float *yn, int64_t ldyn, float *y, int64_t ldy,
                                   hipStream_t st);
hipError_t launch_scale(const float *x, int64_t ldx, int64_t ne0, int64_t n, float s, float *y, int64_t ldy, hipStream_t st);
// Q6_K rows between block order and planes (T_Q6_K_P), in place (dst == src) or into another matrix; rows of at most max_lds bytes
hipError_t launch_repack_q6_K(const void *src, size_t nb01_src, void *dst, size_t nb01_dst, int64_t K, int64_t N, bool to_planes,
                              int max_lds, hipStream_t st);
hipError_t launch_gelu(const float *x, int64_t ldx, int64_t ne0, int64_t n, const unsigned short *table, float *y, int64_t ldy,
                       hipStream_t st);
bool norm_quantized_applicable(const float *a, int64_t lda, const float *b, int64_t ldb, const float *xs, int64_t ldxs, int64_t ne0,
                               const float *w, const float *y, int64_t ldy);
hipError_t launch_norm_quantized(const float *a, int64_t lda, const float *b, int64_t ldb, float *xs, int64_t ldxs, int64_t n,
                                 int64_t ne0, float eps, const float *w, float *y, int64_t ldy, uint8_t *qws, size_t qstride,
                                 int act_kind, hipStream_t st);
bool       silu_mul_quantized_applicable(const float *x, int64_t ldx, const float *b, int64_t ldb, int64_t ne0, const float *y, int64_t ldy);
hipError_t launch_silu_mul_quantized(const float *x, int64_t ldx, const float *b, int64_t ldb, int64_t ne0, int64_t n, float *y,
                                     int64_t ldy, uint8_t *qws, size_t qstride, int act_kind, hipStream_t st);
hipError_t launch_silu_mul(const float *x, int64_t ldx, const float *b, int64_t ldb, int64_t ne0, int64_t n, float *y, int64_t ldy,
                           hipStream_t st);
// SOFT_MAX over n_rows rows of ne00 values (a multiple of 8); row r adds row r % ne01 of the mask (fp32 or fp16, dense).
hipError_t launch_soft_max(const float *x, int64_t ldx, const void *mask, int mask_f16, int64_t ne00, int64_t ne01, int64_t n_rows,
                           float scale, float *y, int64_t ldy, hipStream_t st);
// Copy between F32 / F16 tensors of one element count, element i of the source's logical order to element i of the
// destination's; shapes in elements, strides in bytes.
hipError_t launch_cpy(const void *src, int src_f16, const int64_t *ne_src, const int64_t *nb_src, void *dst, int dst_f16,
                      const int64_t *ne_dst, const int64_t *nb_dst, hipStream_t st);
struct RopeArgs {
    int64_t ne0, ne1, ne2;
    int64_t ldx1, ldx2, ldy1, ldy2;        // head and token strides in floats
    int n_dims, neox;
    float theta_scale, freq_scale, ext_factor, corr0, corr1, mscale;
    unsigned short *y16 = nullptr;         // optional second output: y rounded to fp16 (the K cache store that follows a RoPE)
    int64_t ld16_1 = 0, ld16_2 = 0;        // its head and token strides in halves
};
// LM_GGML_OP_GET_ROWS: dst row (i10, i11, i12) = row ids[i10, i11, i12] of matrix (i11, i12) of src, dequantized to F32.
struct GetRowsArgs {
    const uint8_t *src; size_t nb01, nb02, nb03; int64_t nc, ne01;
    const int32_t *ids; int64_t ne10, ne11, ne12, ldi1, ldi2;                 // ids strides in elements
    float *dst; int64_t ld1, ld2, ld3;                                         // dst strides in floats
};
hipError_t launch_get_rows(int type, const GetRowsArgs &a, hipStream_t st);
hipError_t launch_rope_apply_two(const float *xa, const RopeArgs &a, float *ya, const float *xb, const RopeArgs &b, float *yb,
                                 const float *table, hipStream_t st);
hipError_t launch_rope(const float *x, const int32_t *pos, const float *freq_factors, const RopeArgs &a, float *y, float *table,
                       bool build, hipStream_t st);

// moe_group.hip: counting sort of MUL_MAT_ID's (token, slot) pairs by expert into offsets[n_as + 1] / perm[pairs].
// tiles[0] = number of token tiles, tiles[1 + i] = expert | tile << 12 for tiles of `tile_tokens` pairs.
bool       moe_group_supported(int64_t n_as, int64_t pairs);
hipError_t launch_moe_group(const int32_t *ids, int64_t ids_stride, int64_t n_used, int64_t pairs, int64_t n_as,
                            int tile_tokens, int32_t *offsets, int32_t *perm, int32_t *tiles, hipStream_t st);
int        gemm_blk32_moe_tile_tokens();
int        gemm_kq_moe_tile_tokens();
int        gemm_f16_moe_tile_tokens();

}  // namespace chip
