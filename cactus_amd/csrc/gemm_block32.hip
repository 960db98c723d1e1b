// Prefill GEMM for gfx950 over weights in 32-value blocks with one fp16 scale each (Q4_0, Q8_0, Q5_0, IQ4_NL; Q4_1 and
// Q5_1 with a minimum on top) and Q8_0 / Q8_1 activations: Y[t][r] = sum_b dw[r][b] * dx[t][b] * isum[t][r][b], the batched form of lm_ggml_vec_dot_q4_0_q8_0,
// _q8_0_q8_0, _q5_0_q8_0 and _iq4_nl_q8_0 (reference ggml-cpu/ggml-cpu-quants.c) as driven by
// lm_ggml_compute_forward_mul_mat (ggml-cpu/ggml-cpu.c:1257-1449).
//
// Structure
//   * One v_mfma_i32_32x32x32_i8 multiplies a 32-row x 32-k weight tile by a 32-k x 32-token activation tile:
//     its K extent is exactly one 32-value quantization block, so each of the 1024 int32 results is one
//     per-block integer sum isum[t][r][b], bit-exact.
//   * Weight tiles are staged through LDS once per workgroup and k-stage: a block's packed quants are expanded into
//     two 16-byte cells of signed int8 (elements 0..15 and 16..31), possibly times a power of two that is taken
//     back exactly in the epilogue (Q4_0: 16 * (nib - 8), Q5_0: 8 * (q - 16); IQ4_NL: the code point; Q8_0: as is);
//     activations arrive as int8 from the split workspace layout.
//   * Per-block scales are applied in fp32 after the integer accumulate.  The MFMA's C input is a register
//     vector holding the bit pattern of 12582912.0f (1.5 * 2^23): adding |isum| < 2^22 to those bits gives the
//     bits of the float 12582912 + isum, so the accumulator can be used as a float with no conversion.  Then
//         t   = fma(acc_as_float, dx, -12582912 * dx)      exactly round(isum * dx): 12582912*dx is exact
//                                                           because dx comes from fp16 (11-bit significand)
//         out = fma(t, dw, out)                            dw widened to fp32 exactly
//     i.e. two VALU operations per integer sum, 32 per MFMA.  That VALU work, not the matrix pipe, bounds this
//     kernel: an MFMA occupies the matrix unit for 32 cycles; the 32 fp32 operations, which read the MFMA's result
//     registers, take 134 - 144 cycles per SIMD with two to four waves (measured in a register-only loop).
//   * Q4_1 and Q5_1 add m * s per block (the weight block's minimum times the activation block's d * sum, the s of
//     block_q8_1).  Both factors are fp16 numbers, so sum_b m[r][b] * s[t][b] over the 4 blocks of a stage is one
//     v_mfma_f32_32x32x8f16 that adds straight into the fp32 accumulators: no vector work.
//   * A workgroup is WR x WC waves, each wave owns TM x TN MFMA tiles (32*TM rows x 32*TN tokens); LDS is
//     double buffered over stages of KB = 4 blocks with one barrier per stage.
#include "dev_common.h"
#include "act_layout.h"
#include "kernels.h"
#include <cstdlib>
#include <type_traits>

namespace chip {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

constexpr int GEMM_KB = 4;                    // 32-value blocks per LDS stage
constexpr float MAGIC_F = 12582912.f;         // 1.5 * 2^23
constexpr int MAGIC_I = 0x4B400000;

// How a weight type's block becomes two MFMA operand cells.  MULT is the power of two the cells carry on top of the
// quant (taken back through the activation scale, exactly); MULT * |isum| stays below 2^22 for every type.
template <int WT> struct Blk32;

template <> struct Blk32<T_Q4_0> {
    static constexpr int BYTES = BYTES_Q4_0;
    static constexpr bool HAS_MIN = false;
    static constexpr float INV_MULT = 1.f / 16.f;
    struct Raw { u32x4 q; };
    __device__ static __forceinline__ void fetch(Raw &r, const uint8_t *p) { r.q = *reinterpret_cast<const u32x4_a2 *>(p + 2); }
    // a nibble moved to the high half of its byte with its top bit flipped is 16 * (nibble - 8) as a signed byte
    __device__ static __forceinline__ void emit(const Raw &r, u32x4 &lo, u32x4 &hi) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            lo[i] = ((r.q[i] << 4) & 0xf0f0f0f0u) ^ 0x80808080u;
            hi[i] = (r.q[i] & 0xf0f0f0f0u) ^ 0x80808080u;
        }
    }
};

template <> struct Blk32<T_IQ4_NL> {
    static constexpr int BYTES = BYTES_IQ4_NL;
    static constexpr bool HAS_MIN = false;
    static constexpr float INV_MULT = 1.f;
    using Raw = Blk32<T_Q4_0>::Raw;
    __device__ static __forceinline__ void fetch(Raw &r, const uint8_t *p) { Blk32<T_Q4_0>::fetch(r, p); }
    // four code indices (one per byte, 0..15) -> four code points of kvalues_iq4nl (reference ggml-common.h), through
    // two byte permutes of the 16-entry table
    __device__ static __forceinline__ uint32_t lookup4(uint32_t idx) {
        constexpr uint32_t T0 = 0xbfad9881u, T1 = 0xf6eaddcfu, T2 = 0x26190d01u, T3 = 0x71594535u;
        const uint32_t sel = idx & 0x07070707u;
        const uint32_t lo = __builtin_amdgcn_perm(T1, T0, sel), hi = __builtin_amdgcn_perm(T3, T2, sel);
        const uint32_t m = ((idx >> 3) & 0x01010101u) * 0xffu;
        return (lo & ~m) | (hi & m);
    }
    __device__ static __forceinline__ void emit(const Raw &r, u32x4 &lo, u32x4 &hi) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            lo[i] = lookup4(r.q[i] & 0x0f0f0f0fu);
            hi[i] = lookup4((r.q[i] >> 4) & 0x0f0f0f0fu);
        }
    }
};

template <> struct Blk32<T_Q8_0> {
    static constexpr int BYTES = BYTES_Q8_0;
    static constexpr bool HAS_MIN = false;
    static constexpr float INV_MULT = 1.f;
    struct Raw { u32x4 lo, hi; };
    __device__ static __forceinline__ void fetch(Raw &r, const uint8_t *p) {
        r.lo = *reinterpret_cast<const u32x4_a2 *>(p + 2);
        r.hi = *reinterpret_cast<const u32x4_a2 *>(p + 18);
    }
    __device__ static __forceinline__ void emit(const Raw &r, u32x4 &lo, u32x4 &hi) { lo = r.lo; hi = r.hi; }
};

template <> struct Blk32<T_Q5_0> {
    static constexpr int BYTES = BYTES_Q5_0;
    static constexpr bool HAS_MIN = false;
    static constexpr float INV_MULT = 1.f / 8.f;
    struct Raw { u32x4 q; uint32_t qh; };
    __device__ static __forceinline__ void fetch(Raw &r, const uint8_t *p) {
        r.qh = *reinterpret_cast<const u32_a2 *>(p + 2);
        r.q = *reinterpret_cast<const u32x4_a2 *>(p + 6);
    }
    // element j < 16: low nibble of qs[j] with bit j of qh on top, element 16 + j: high nibble with bit 16 + j
    // (reference ggml-quants.c:290-310).  The cell byte is 8 * (q - 16): q << 3 with the top bit flipped.
    __device__ static __forceinline__ void emit(const Raw &r, u32x4 &lo, u32x4 &hi) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // 4 bits -> bit 0 of each byte: bit k lands at 7k + k = 8k
            const uint32_t bl = (((r.qh >> (4 * i)) & 0xfu) * 0x00204081u) & 0x01010101u;
            const uint32_t bh = (((r.qh >> (16 + 4 * i)) & 0xfu) * 0x00204081u) & 0x01010101u;
            lo[i] = (((r.q[i] << 3) & 0x78787878u) | (bl << 7)) ^ 0x80808080u;
            hi[i] = (((r.q[i] >> 1) & 0x78787878u) | (bh << 7)) ^ 0x80808080u;
        }
    }
};

// Q4_1 / Q5_1: unsigned quants, block = d, m (fp16), [qh,] qs; value = d * q + m
template <> struct Blk32<T_Q4_1> {
    static constexpr int BYTES = BYTES_Q4_1;
    static constexpr bool HAS_MIN = true;
    static constexpr float INV_MULT = 1.f / 8.f;
    struct Raw { u32x4 q; };
    __device__ static __forceinline__ void fetch(Raw &r, const uint8_t *p) { r.q = *reinterpret_cast<const u32x4_a4 *>(p + 4); }
    __device__ static __forceinline__ void emit(const Raw &r, u32x4 &lo, u32x4 &hi) {      // 8 * nibble, 0..120
#pragma unroll
        for (int i = 0; i < 4; i++) {
            lo[i] = (r.q[i] << 3) & 0x78787878u;
            hi[i] = (r.q[i] >> 1) & 0x78787878u;
        }
    }
};

template <> struct Blk32<T_Q5_1> {
    static constexpr int BYTES = BYTES_Q5_1;
    static constexpr bool HAS_MIN = true;
    static constexpr float INV_MULT = 1.f / 4.f;
    struct Raw { u32x4 q; uint32_t qh; };
    __device__ static __forceinline__ void fetch(Raw &r, const uint8_t *p) {
        r.qh = *reinterpret_cast<const uint32_t *>(p + 4);
        r.q = *reinterpret_cast<const u32x4_a4 *>(p + 8);
    }
    __device__ static __forceinline__ void emit(const Raw &r, u32x4 &lo, u32x4 &hi) {      // 4 * q, 0..124
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t bl = (((r.qh >> (4 * i)) & 0xfu) * 0x00204081u) & 0x01010101u;
            const uint32_t bh = (((r.qh >> (16 + 4 * i)) & 0xfu) * 0x00204081u) & 0x01010101u;
            lo[i] = ((r.q[i] << 2) & 0x3c3c3c3cu) | (bl << 6);
            hi[i] = ((r.q[i] >> 2) & 0x3c3c3c3cu) | (bh << 6);
        }
    }
};

// ---- how the operands travel and how a wave orders its work ----
//   * Quantized activations and their scales go from the workspace into LDS with global_load_lds_dwordx4: no staging
//     registers, no ds_write, no vector instructions.  A token's 128 bytes of a stage are one LDS row of 8 cells; cell c of
//     token t sits in slot c ^ ((t >> 1) & 7), so the 16 lanes that read one cell index of 16 consecutive tokens hit 16
//     different bank groups (the lane that fills a slot fetches the matching cell).  The four fp32 scales of a token and
//     stage are one more cell.
//   * Weights pass through registers (their 18- to 34-byte blocks must be expanded to int8 cells); they are fetched
//     two stages ahead and expanded one stage ahead, so a load has a whole stage to arrive.  The weight scales are
//     widened to fp32 on the way into LDS: a mixed-precision FMA that reads them as fp16 issues at a lower rate than a
//     plain one (measured: 16 + 16 plain FMAs behind an MFMA 56 - 60 ns per SIMD, with the second 16 mixed 67 - 80 ns).
//   * Inside a stage the MFMA of tile i + 1 is issued before the 32 scaling operations of tile i, across k-blocks too,
//     so one wave keeps the vector unit busy by itself and two waves per SIMD are enough; the stage loop is unrolled by
//     two so that every LDS address is a register plus an immediate.
//   * The power of two that the weight cells carry is taken back once, in the epilogue (exact), not per stage.
// LDS cells: [k-block][half][row] 16-byte cells for the weights (exactly what one lane feeds the MFMA: row = lane % 32,
// half = lane / 32), each plane padded by two cells: the threads that expand one stage walk the planes fastest, and a
// plane stride that is 2 mod 16 cells puts 16 consecutive writers on 16 different bank groups.
template <int TM, int TN, int WR, int WC, bool HAS_MIN>
struct DirectCfg {
    static constexpr int NW = WR * WC, NT = NW * 64;
    static constexpr int BM = 32 * TM * WR, BN = 32 * TN * WC;
    static constexpr int A_PLANE = BM + 2;                                        // cells
    static constexpr size_t OFF_A = 0;
    static constexpr size_t OFF_B = OFF_A + (size_t)GEMM_KB * 2 * A_PLANE * 16;   // [token][8 cells], swizzled
    static constexpr size_t OFF_SX = OFF_B + (size_t)BN * 128;                    // [token][4 floats]
    static constexpr size_t OFF_SW = OFF_SX + (size_t)BN * 16;                    // fp32 [KB][BM], permuted per 32 rows
    // plane b of the weight scales starts 8 * (b & 1) + 32 * (b >> 1) floats late: the 64 lanes that expand 16 rows x 4
    // k-blocks then write to 64 different banks (a row's position inside its 32-row group is 0..7 or 16..23 for the first
    // 16 rows, 8..15 or 24..31 for the others)
    static constexpr int sw_plane(int b) { return b * BM + 8 * (b & 1) + 32 * (b >> 1); }
    static constexpr size_t OFF_MW = OFF_SW + ((size_t)GEMM_KB * BM + 64) * 4;    // fp16 [BM][KB]
    static constexpr size_t OFF_MX = OFF_MW + (HAS_MIN ? (size_t)BM * GEMM_KB * 2 : 0);   // fp16 [BN][KB]
    static constexpr size_t STAGE = OFF_MX + (HAS_MIN ? (size_t)BN * GEMM_KB * 2 : 0);
    static constexpr int W_ITEMS = BM * GEMM_KB, W_PER_T = (W_ITEMS + NT - 1) / NT;
    static constexpr int B_INSTR = BN / 8;                                        // wave instructions that fill B: 8 tokens each
    static constexpr int B_PER_W = B_INSTR / NW;
    static constexpr int SX_INSTR = BN / 64;                                      // 64 tokens' scale cells each
    static constexpr int S_ITEMS = BN * GEMM_KB, S_PER_T = (S_ITEMS + NT - 1) / NT;
    static_assert(B_INSTR % NW == 0 && B_PER_W >= 1, "the activation loads divide evenly over the waves");
    static_assert(SX_INSTR >= 1 && SX_INSTR <= NW, "one scale load instruction per wave at most");
    static_assert(W_ITEMS % NT == 0, "the weight items divide evenly over the threads");
    static_assert(STAGE % 16 == 0 && GEMM_KB == 4, "stage buffers keep 16-byte alignment; four scale planes");
};

constexpr int wait_vm0() { return 0x0F70; }                                      // s_waitcnt vmcnt(0) only

// M0 carries the LDS byte address of the wave's 1 KB destination; lane i's 16 bytes land at M0 + 16 i.  Inline assembly,
// because the compiler would make every later LDS read wait for a load it sees writing LDS; the kernel waits by hand
// (vmcnt(0) in front of the stage barrier).  Nothing else in the kernel may use M0 (no dynamic register indexing).
__device__ __forceinline__ void load16_into_lds(const uint8_t *src, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_addr) : "memory");
}

template <int WT, int TM, int TN, int WR, int WC, int OCC, bool GATHER>
__global__ __launch_bounds__(WR *WC * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void gemm_blk32_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N, const uint8_t *__restrict__ ws,
                              size_t ws_stride, int64_t M, float *__restrict__ y, int64_t ldy, TileMap map, RowGather rg,
                              int slice_stages) {
    using T = Blk32<WT>;
    using C = DirectCfg<TM, TN, WR, WC, T::HAS_MIN>;
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave / WC, wc = wave % WC;
    const int half = lane >> 5, l32 = lane & 31;
    const TileCoord tc = xcd_tile(blockIdx.x, map);
    if (tc.row_tile >= map.row_tiles || tc.tok_tile >= map.tok_tiles) return;
    const int64_t row_base = (int64_t)tc.row_tile * C::BM;
    size_t w_offset;
    const GatherView gv = resolve_gather<GATHER>(rg, w_offset, M);
    W += w_offset;
    if (gv.tok_tile < 0) return;
    const int64_t tok_base = (int64_t)(GATHER ? gv.tok_tile : tc.tok_tile) * C::BN;
    if (tok_base >= M) return;
    int stage0 = 0, nstages = (int)(K / (32 * GEMM_KB));
    if (!GATHER && slice_stages > 0) {
        stage0 = (int)blockIdx.y * slice_stages;
        nstages = min(slice_stages, nstages - stage0);
        y += (size_t)blockIdx.y * (size_t)M * (size_t)ldy;
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;

    // ---- sources of this thread's share of a stage (stage 0 of the slice; they advance by a constant per stage) ----
    const uint8_t *wsrc[C::W_PER_T];
#pragma unroll
    for (int i = 0; i < C::W_PER_T; i++) {
        const int item = tid + i * C::NT, r = item / GEMM_KB, b = item % GEMM_KB;
        wsrc[i] = W + (size_t)min(row_base + r, N - 1) * nb01 + ((size_t)stage0 * GEMM_KB + b) * T::BYTES;
    }
    // activation cells: instruction q = wave * B_PER_W + j fills tokens 8 q .. 8 q + 7, lane -> token lane / 8, slot lane % 8
    const uint8_t *bsrc[C::B_PER_W];
#pragma unroll
    for (int j = 0; j < C::B_PER_W; j++) {
        const int t = (wave * C::B_PER_W + j) * 8 + (lane >> 3);
        const int cell = (lane & 7) ^ ((t >> 1) & 7);
        bsrc[j] = ws + (size_t)gv.act_row(min(tok_base + t, M - 1)) * ws_stride + (size_t)stage0 * (32 * GEMM_KB) + 16 * cell;
    }
    const uint8_t *sxsrc = ws + (size_t)gv.act_row(min(tok_base + (wave < C::SX_INSTR ? wave : 0) * 64 + lane, M - 1)) * ws_stride +
                           q8_0_off_d(K) + (size_t)stage0 * (4 * GEMM_KB);
    const uint8_t *msrc[C::S_PER_T];                                               // block_q8_1.s of the types with a minimum
    if constexpr (T::HAS_MIN) {
#pragma unroll
        for (int i = 0; i < C::S_PER_T; i++) {
            const int item = tid + i * C::NT;
            msrc[i] = ws + (size_t)gv.act_row(min(tok_base + min(item / GEMM_KB, C::BN - 1), M - 1)) * ws_stride + q8_0_off_s(K) +
                      ((size_t)stage0 * GEMM_KB + item % GEMM_KB) * 4;
        }
    }

    typename T::Raw wq[C::W_PER_T];
    uint32_t wd[C::W_PER_T];
    float xm[C::S_PER_T];
    auto fetch_w = [&](int s) {
#pragma unroll
        for (int i = 0; i < C::W_PER_T; i++) {
            const uint8_t *p = wsrc[i] + (size_t)s * (GEMM_KB * T::BYTES);
            if constexpr (T::HAS_MIN) wd[i] = *reinterpret_cast<const uint32_t *>(p);
            else wd[i] = *reinterpret_cast<const unsigned short *>(p);
            T::fetch(wq[i], p);
        }
        if constexpr (T::HAS_MIN) {
#pragma unroll
            for (int i = 0; i < C::S_PER_T; i++) xm[i] = *reinterpret_cast<const float *>(msrc[i] + (size_t)s * (4 * GEMM_KB));
        }
    };
    auto issue_direct = [&](int s, uint32_t buf_off) {
#pragma unroll
        for (int j = 0; j < C::B_PER_W; j++)
            load16_into_lds(bsrc[j] + (size_t)s * (32 * GEMM_KB),
                            __builtin_amdgcn_readfirstlane(lds0 + buf_off + (uint32_t)C::OFF_B + (uint32_t)(wave * C::B_PER_W + j) * 1024u));
        if (wave < C::SX_INSTR)
            load16_into_lds(sxsrc + (size_t)s * (4 * GEMM_KB),
                            __builtin_amdgcn_readfirstlane(lds0 + buf_off + (uint32_t)C::OFF_SX + (uint32_t)wave * 1024u));
    };
    auto commit_w = [&](uint32_t buf_off) {
        uint8_t *base = lds + buf_off;
        u32x4 *A = reinterpret_cast<u32x4 *>(base + C::OFF_A);
        float *SW = reinterpret_cast<float *>(base + C::OFF_SW);
#pragma unroll
        for (int i = 0; i < C::W_PER_T; i++) {
            const int item = tid + i * C::NT, r = item / GEMM_KB, b = item % GEMM_KB;
            u32x4 lo, hi;
            T::emit(wq[i], lo, hi);
            A[(b * 2 + 0) * C::A_PLANE + r] = lo;
            A[(b * 2 + 1) * C::A_PLANE + r] = hi;
            const int i32 = r & 31;
            // the lane that owns MFMA result register v of a 32-row tile holds row 8*(v/4) + 4*half + v%4: the scale of
            // row i goes to half*16 + (i/8)*4 + i%4, so a lane reads its 16 scales as one contiguous run
            const int pos = ((i32 >> 2) & 1) * 16 + (i32 >> 3) * 4 + (i32 & 3);
            SW[C::sw_plane(b) + (r & ~31) + pos] = h2f(wd[i]);
            if constexpr (T::HAS_MIN) reinterpret_cast<unsigned short *>(base + C::OFF_MW)[r * GEMM_KB + b] = (unsigned short)(wd[i] >> 16);
        }
        if constexpr (T::HAS_MIN) {
#pragma unroll
            for (int i = 0; i < C::S_PER_T; i++) {
                const int item = tid + i * C::NT;
                if (C::S_ITEMS % C::NT == 0 || item < C::S_ITEMS)
                    reinterpret_cast<unsigned short *>(base + C::OFF_MX)[item] = f2h_rne(xm[i]);      // [token][KB]; exact
            }
        }
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int c = 0; c < TN; c++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[a][c][v] = 0.f;
    i32x16 magic;
#pragma unroll
    for (int v = 0; v < 16; v++) {
        int m = MAGIC_I;
        asm volatile("" : "+v"(m));
        magic[v] = m;
    }

    // per-lane LDS byte offsets inside a stage buffer; everything else is an immediate
    const int r0 = wr * TM * 32, n0 = wc * TN * 32;
    const uint32_t a_rd = (uint32_t)C::OFF_A + (uint32_t)(half * C::A_PLANE + r0 + l32) * 16u;
    const uint32_t sw_rd = (uint32_t)C::OFF_SW + (uint32_t)(r0 + half * 16) * 4u;
    const uint32_t sx_rd = (uint32_t)C::OFF_SX + (uint32_t)(n0 + l32) * 16u;
    uint32_t b_rd[GEMM_KB];
#pragma unroll
    for (int b = 0; b < GEMM_KB; b++) b_rd[b] = (uint32_t)C::OFF_B + (uint32_t)(n0 + l32) * 128u + 16u * (uint32_t)((2 * b + half) ^ ((l32 >> 1) & 7));

    // one stage from the buffer at byte offset BUF
    auto compute = [&](auto buf_tag) {
        constexpr uint32_t BUF = decltype(buf_tag)::value ? (uint32_t)C::STAGE : 0u;
        const uint8_t *base = lds + BUF;
        if constexpr (T::HAS_MIN) {
            f16x4 ma[TM], sb[TN];
#pragma unroll
            for (int a = 0; a < TM; a++) {
                const u32x2 t = reinterpret_cast<const u32x2 *>(base + C::OFF_MW)[r0 + a * 32 + l32];
                ma[a] = __builtin_bit_cast(f16x4, half ? u32x2{0u, 0u} : t);
            }
#pragma unroll
            for (int c = 0; c < TN; c++) {
                const u32x2 t = reinterpret_cast<const u32x2 *>(base + C::OFF_MX)[n0 + c * 32 + l32];
                sb[c] = __builtin_bit_cast(f16x4, half ? u32x2{0u, 0u} : t);
            }
#pragma unroll
            for (int a = 0; a < TM; a++)
#pragma unroll
                for (int c = 0; c < TN; c++) acc[a][c] = __builtin_amdgcn_mfma_f32_32x32x8f16(ma[a], sb[c], acc[a][c], 0, 0, 0);
        }
        float dxs[TN][GEMM_KB];
#pragma unroll
        for (int c = 0; c < TN; c++) {
            const float4 t = *reinterpret_cast<const float4 *>(base + sx_rd + c * 512);
            dxs[c][0] = t.x; dxs[c][1] = t.y; dxs[c][2] = t.z; dxs[c][3] = t.w;
            if constexpr (T::HAS_MIN) {
#pragma unroll
                for (int b = 0; b < GEMM_KB; b++) dxs[c][b] *= T::INV_MULT;       // the min term has no power of two to take back
            }
        }
        // operand registers of two k-blocks: those of k-block b + 1 are requested while k-block b is worked on, and the
        // first MFMA of k-block b + 1 is issued before the last scaling group of k-block b.  The 16 weight scales of a
        // (k-block, row tile) pair - fp32 in LDS: a mixed-precision FMA that reads them as fp16 issues at a lower rate
        // than a plain one - serve the pair's TN tiles and are requested one pair ahead, in two register sets.
        i32x4 af[2][TM], bf[2][TN];
        float swf[2][16];
        auto load_operands = [&](int b, int slot) {
#pragma unroll
            for (int a = 0; a < TM; a++) {
                const u32x4 t = *reinterpret_cast<const u32x4 *>(base + a_rd + (b * 2 * C::A_PLANE + a * 32) * 16);
                af[slot][a] = i32x4{(int)t.x, (int)t.y, (int)t.z, (int)t.w};
            }
#pragma unroll
            for (int c = 0; c < TN; c++) {
                const u32x4 t = *reinterpret_cast<const u32x4 *>(base + b_rd[b] + c * 4096);
                bf[slot][c] = i32x4{(int)t.x, (int)t.y, (int)t.z, (int)t.w};
            }
        };
        auto load_scales = [&](int g) {                                       // pair g = b * TM + a
            const int b = g / TM, a = g % TM;
            const float4 *sp = reinterpret_cast<const float4 *>(base + sw_rd + (C::sw_plane(b) + a * 32) * 4);
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4 t = sp[q];
                swf[g & 1][4 * q] = t.x; swf[g & 1][4 * q + 1] = t.y; swf[g & 1][4 * q + 2] = t.z; swf[g & 1][4 * q + 3] = t.w;
            }
        };
        load_operands(0, 0);
        load_scales(0);
        i32x16 d_cur = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[0][0], bf[0][0], magic, 0, 0, 0);
#pragma unroll
        for (int b = 0; b < GEMM_KB; b++) {
            const int slot = b & 1;
            if (b + 1 < GEMM_KB) load_operands(b + 1, slot ^ 1);
            float dx[TN], ndx[TN];
#pragma unroll
            for (int c = 0; c < TN; c++) {
                dx[c] = dxs[c][b];
                ndx[c] = -MAGIC_F * dx[c];
            }
#pragma unroll
            for (int a = 0; a < TM; a++) {
                const int g = b * TM + a;
                if (g + 1 < GEMM_KB * TM) load_scales(g + 1);
#pragma unroll
                for (int c = 0; c < TN; c++) {
                    i32x16 d_next = d_cur;
                    if (c + 1 < TN) d_next = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[slot][a], bf[slot][c + 1], magic, 0, 0, 0);
                    else if (a + 1 < TM) d_next = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[slot][a + 1], bf[slot][0], magic, 0, 0, 0);
                    else if (b + 1 < GEMM_KB) d_next = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[slot ^ 1][0], bf[slot ^ 1][0], magic, 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);                // the MFMA goes first: it runs behind the scaling below
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const float t = __builtin_fmaf(__int_as_float(d_cur[v]), dx[c], ndx[c]);
                        acc[a][c][v] = __builtin_fmaf(t, swf[g & 1][v], acc[a][c][v]);
                    }
                    d_cur = d_next;
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };

    // Every load gets a whole stage to arrive.  A stage begins by expanding the weights fetched during the previous stage
    // into the idle buffer (the compiler's own wait for them is exact: nothing younger is outstanding then), then requests
    // the next stage's activations (into that same idle buffer) and the weights of the stage after, and only then starts
    // its arithmetic.  In front of the barrier a wave waits until at most its weight loads - the youngest requests - are
    // outstanding, i.e. for the activations; the barrier publishes them and the expanded weights.
    // Nothing inside a stage is conditional (a branch would end the scheduling region that keeps the MFMAs and their
    // scaling interleaved): stages past the last one are the last one again, loaded and expanded into the idle buffer.
    constexpr int W_LOADS = C::W_PER_T * 2 + (T::HAS_MIN ? C::S_PER_T : 0);          // vector loads of one fetch_w
    constexpr int WAIT_ACTS = 0x0F70 | (W_LOADS & 15) | ((W_LOADS >> 4) << 14);      // s_waitcnt vmcnt(W_LOADS)
    const int last = nstages - 1;
    fetch_w(0);
    issue_direct(0, 0u);
    commit_w(0u);
    fetch_w(min(1, last));
    __builtin_amdgcn_s_waitcnt(WAIT_ACTS);
    __syncthreads();
    for (int s = 0; s < nstages; s += 2) {
        {
            commit_w((uint32_t)C::STAGE);
            issue_direct(min(s + 1, last), (uint32_t)C::STAGE);
            fetch_w(min(s + 2, last));
            compute(std::false_type{});
            __builtin_amdgcn_s_waitcnt(WAIT_ACTS);
            __syncthreads();
        }
        if (s + 1 < nstages) {
            commit_w(0u);
            issue_direct(min(s + 2, last), 0u);
            fetch_w(min(s + 3, last));
            compute(std::true_type{});
            __builtin_amdgcn_s_waitcnt(WAIT_ACTS);
            __syncthreads();
        }
    }
    __builtin_amdgcn_s_waitcnt(wait_vm0());

    // ---- epilogue: register v of tile (a, c) is row 8*(v/4) + 4*half + v%4, token l32 ----
    constexpr float POST = T::HAS_MIN ? 1.f : T::INV_MULT;
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int c = 0; c < TN; c++) {
            const int64_t tok = tok_base + n0 + c * 32 + l32;
            if (tok >= M) continue;
            const int64_t orow = gv.out_row(tok);
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int64_t row = row_base + r0 + a * 32 + 8 * g + 4 * half;
                float *dst = y + (size_t)orow * ldy + row;
                const float o0 = acc[a][c][4 * g] * POST, o1 = acc[a][c][4 * g + 1] * POST, o2 = acc[a][c][4 * g + 2] * POST, o3 = acc[a][c][4 * g + 3] * POST;
                if (row + 3 < N && (((uintptr_t)dst) & 15) == 0) {
                    *reinterpret_cast<float4 *>(dst) = make_float4(o0, o1, o2, o3);
                } else {
                    const float o[4] = {o0, o1, o2, o3};
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (row + e < N) dst[e] = o[e];
                }
            }
        }
}

// With few tokens the GEMM's time is its walk over K, about 0.25 us per 32-value block whatever the token count
// (33 - 37 us at K = 4096, 110 - 120 us at K = 14336), while the GEMV forms pass over the weights once per 8 or 16
// tokens at memory speed.  Up to 128 tokens on a matrix with few row tiles the walk is cut into slices
// (blk32_slices_for below: 17 - 20 us at K = 4096, 28 - 39 us at K = 14336).  The token count from which the GEMM is
// ahead, measured on 4096 x 4096, 14336 x 4096 and 4096 x 14336 (Q8_0 and Q4_0 have the matrix-core GEMV of 16 tokens
// a pass, 8 on very long rows; the other types pass once per 8 tokens or fewer):
static bool blk32_splittable(int64_t N) { return ceil_div(N, (int64_t)64) <= 384; }
static int64_t gemm_blk32_min_tokens(int wtype, int64_t K, int64_t N, bool can_split) {
    const bool long_rows = K > 8192, big = N * K >= ((int64_t)48 << 20);
    if (can_split && blk32_splittable(N)) return (wtype == T_Q8_0 && long_rows) ? 9 : 17;
    // too many row tiles to split, or no room for the partial outputs in the caller's workspace: the unsplit walk
    switch (wtype) {
        case T_Q8_0: return long_rows ? 49 : big ? 17 : 49;
        case T_Q4_0: return long_rows ? 65 : big ? 33 : 49;
        default:     return big ? 32 : 48;
    }
}
bool gemm_blk32_supported(int wtype, int64_t K, int64_t N, int64_t n, bool can_split) {
    if (!(wtype == T_Q4_0 || wtype == T_Q8_0 || wtype == T_Q5_0 || wtype == T_IQ4_NL || wtype == T_Q4_1 || wtype == T_Q5_1)) return false;
    if (K % (32 * GEMM_KB) != 0 || N < 1) return false;
    const int64_t forced = tune("CHIP_GEMM_MIN_TOKENS", 0);
    if (forced > 0) return n >= forced;
    return n >= gemm_blk32_min_tokens(wtype, K, N, can_split);
}

// ---- split K: the partial outputs [slice][token][row] added in slice order ----
__global__ __launch_bounds__(256) void sum_slices_kernel(const float *__restrict__ part, int slices, int64_t per_slice, int64_t n,
                                                         int64_t N, float *__restrict__ y, int64_t ldy) {
    const int64_t e0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;                // four consecutive rows of one token
    if (e0 >= n * N) return;
    const uint32_t t = (uint32_t)(e0 / N);
    const int64_t r = e0 - (int64_t)t * N;
    const bool vec = (N & 3) == 0 && (((uintptr_t)part) & 15) == 0;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < slices; s0 += 8) {
        float4 p[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            p[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (s0 + j < slices) {
                const float *src = part + (size_t)(s0 + j) * per_slice + e0;
                if (vec) p[j] = *reinterpret_cast<const float4 *>(src);
                else {
                    p[j].x = src[0];
                    if (r + 1 < N) p[j].y = src[1];
                    if (r + 2 < N) p[j].z = src[2];
                    if (r + 3 < N) p[j].w = src[3];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (s0 + j < slices) { v[0] += p[j].x; v[1] += p[j].y; v[2] += p[j].z; v[3] += p[j].w; }
    }
    float *dst = y + (size_t)t * ldy + r;
#pragma unroll
    for (int k = 0; k < 4; k++)
        if (r + k < N) dst[k] = v[k];
}
hipError_t launch_sum_slices(const float *part, int slices, int64_t n, int64_t N, float *y, int64_t ldy, hipStream_t st) {
    if (n <= 0 || N <= 0 || slices <= 0) return hipSuccess;
    // a token's rows in fours: with N not a multiple of 4 a group of four would straddle two tokens, so pad per token
    if ((N & 3) != 0) {
        for (int64_t t = 0; t < n; t++) {
            hipLaunchKernelGGL(sum_slices_kernel, dim3((unsigned)ceil_div(N, (int64_t)1024)), dim3(256), 0, st, part + t * N, slices, n * N,
                               (int64_t)1, N, y + t * ldy, ldy);
        }
        return hipGetLastError();
    }
    hipLaunchKernelGGL(sum_slices_kernel, dim3((unsigned)ceil_div(n * N, (int64_t)1024)), dim3(256), 0, st, part, slices, n * N, n, N, y, ldy);
    return hipGetLastError();
}

// Slices of K for the 64 x 64 shape: about three workgroups per CU up to 128 tokens, two with more (the partial outputs
// grow with the token count), at least eight stages each.
static int blk32_slices_for(int64_t K, int64_t N, int64_t M, int64_t cus) {
    const int forced = (int)tune("CHIP_GEMM_SLICES", 0);
    const int64_t units = K / (32 * GEMM_KB), tiles = ceil_div(N, (int64_t)64) * ceil_div(M, (int64_t)64);
    if (forced > 0) {
        const int64_t per = ceil_div(units, (int64_t)(forced < units ? forced : units));
        return (int)ceil_div(units, per);
    }
    if (units < 16 || (M <= 128 && !blk32_splittable(N))) return 1;
    int64_t s = (M <= 128 ? 3 : 2) * cus / tiles;
    if (s > units / 8) s = units / 8;
    if (s > 16) s = 16;
    if (s < 2) return 1;
    const int64_t per = ceil_div(units, s);
    return (int)ceil_div(units, per);                                   // no empty slice
}

template <int WT, int TM, int TN, int WR, int WC, int OCC, bool GATHER>
static hipError_t launch_direct(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int64_t M,
                                float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const RowGather &rg, int64_t n_as,
                                int slices = 1, float *part = nullptr) {
    using C = DirectCfg<TM, TN, WR, WC, Blk32<WT>::HAS_MIN>;
    const size_t lds_bytes = 2 * C::STAGE;
    if ((int64_t)lds_bytes > lim.max_lds_per_block) return hipErrorInvalidValue;
    auto kfn = gemm_blk32_kernel<WT, TM, TN, WR, WC, OCC, GATHER>;
    static LdsGrant grant;
    if (hipError_t e = grant_dynamic_lds(kfn, lds_bytes, lim, grant); e != hipSuccess) return e;
    const int per_cu = (int)(lds_bytes > 80 * 1024 ? 1 : (4 * OCC / C::NW > 0 ? 4 * OCC / C::NW : 1));
    const TileMap map = make_tile_map(ceil_div(N, C::BM), GATHER ? 1 : ceil_div(M, C::BN), 32 * per_cu);
    if (!GATHER && slices > 1) {
        const int slice_stages = (int)ceil_div(K / (32 * GEMM_KB), (int64_t)slices);
        hipLaunchKernelGGL(kfn, dim3(map.grid, (unsigned)slices), dim3(C::NT), lds_bytes, st, (const uint8_t *)W, nb01, K, N,
                           (const uint8_t *)ws, ws_stride, M, part, N, map, rg, slice_stages);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
        return launch_sum_slices(part, slices, M, N, y, ldy, st);
    }
    hipLaunchKernelGGL(kfn, dim3(map.grid, (unsigned)n_as), dim3(C::NT), lds_bytes, st, (const uint8_t *)W, nb01, K, N,
                       (const uint8_t *)ws, ws_stride, M, y, ldy, map, rg, 0);
    return hipGetLastError();
}

template <int WT>
static hipError_t launch_type(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int64_t M,
                              float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const RowGather &rg, int64_t n_as,
                              SplitK split) {
    const int64_t cus = lim.compute_units > 0 ? lim.compute_units : 256;
    if (!rg.perm && split.part) {
        const int slices = blk32_slices_for(K, N, M, cus);
        if (slices > 1 && split.bytes >= (size_t)slices * (size_t)M * (size_t)N * sizeof(float) && (((uintptr_t)split.part) & 15) == 0) {
            return launch_direct<WT, 1, 1, 2, 2, 3, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, slices, split.part);
        }
    }
    if (rg.perm) {                                                                   // expert groups: 64 x 64 tiles
        return launch_direct<WT, 1, 1, 2, 2, 3, true>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);
    }
    // Two 4-wave workgroups of 128 x 128 per CU when that fills the device, else 64 x 128, else 64 x 64 (three workgroups
    // per CU).  Measured on Q4_0 with K = 4096 (us; 128 x 128 / 64 x 128 / 64 x 64 / 128 x 256 with 8 waves): 14336 x 2048
    // tokens 375 / 413 / 468 / 415, 4096 x 2048 106 / 115 / 130 / 106, 14336 x 512 103 / 110 / 114 / 102, 4096 x 512
    // 63 / 38 / 38 / 81.
    const int64_t g128 = ceil_div(N, 128) * ceil_div(M, 128), g64x128 = ceil_div(N, 64) * ceil_div(M, 128);
    const int cfg = (int)tune("CHIP_GEMM_CFG", 2 * g128 >= 3 * cus ? 3 : 2 * g64x128 >= 3 * cus ? 6 : 4);
    switch (cfg) {
        case 3: return launch_direct<WT, 2, 2, 2, 2, 2, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);   // 128 x 128, 4 waves
        case 4: return launch_direct<WT, 1, 1, 2, 2, 3, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);   // 64 x 64, 4 waves
        case 6: return launch_direct<WT, 1, 2, 2, 2, 2, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);   // 64 x 128, 4 waves
        default: return hipErrorInvalidValue;
    }
    return hipErrorInvalidValue;
}

int gemm_blk32_slices(int wtype, int64_t K, int64_t N, int64_t n, int compute_units) {
    if (!gemm_blk32_supported(wtype, K, N, n, true)) return 1;
    return blk32_slices_for(K, N, n, compute_units > 0 ? compute_units : 256);
}

int gemm_blk32_moe_tile_tokens() { return DirectCfg<1, 1, 2, 2, false>::BN; }   // the 64 x 64 shape serves the expert groups

hipError_t launch_gemm_blk32(int wtype, const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride,
                             int64_t M, float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const RowGather *rgp,
                             int64_t n_as, SplitK split) {
    if (M <= 0 || N <= 0 || n_as <= 0) return hipSuccess;
    const RowGather rg = rgp ? *rgp : RowGather{nullptr, nullptr, nullptr, 1, 1, 0};
    switch (wtype) {
        case T_Q4_0:   return launch_type<T_Q4_0>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, split);
        case T_Q8_0:   return launch_type<T_Q8_0>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, split);
        case T_Q5_0:   return launch_type<T_Q5_0>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, split);
        case T_IQ4_NL: return launch_type<T_IQ4_NL>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, split);
        case T_Q4_1:   return launch_type<T_Q4_1>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, split);
        case T_Q5_1:   return launch_type<T_Q5_1>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, split);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace chip
