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
//     two 16-byte cells of signed int8 (elements 0..15 and 16..31), possibly times a power of two that the
//     activation scale takes back (Q4_0: 16 * (nib - 8), Q5_0: 8 * (q - 16); IQ4_NL: the code point; Q8_0: as is);
//     activations arrive as int8 from the split workspace layout.  Both sit in LDS as [k-block][half][row]
//     16-byte cells, which is exactly what one lane feeds the MFMA (row = lane % 32, half = lane / 32).
//   * Per-block scales are applied in fp32 after the integer accumulate.  The MFMA's C input is a register
//     vector holding the bit pattern of 12582912.0f (1.5 * 2^23): adding |isum| < 2^22 to those bits gives the
//     bits of the float 12582912 + isum, so the accumulator can be used as a float with no conversion.  Then
//         t   = fma(acc_as_float, dx, -12582912 * dx)      exactly round(isum * dx): 12582912*dx is exact
//                                                           because dx comes from fp16 (11-bit significand)
//         out = fma(t, dw, out)                            dw read as fp16 by the mixed-precision fma
//     i.e. two VALU operations per integer sum, 32 per MFMA.  That VALU work, not the matrix pipe, bounds this
//     kernel: an MFMA occupies the matrix unit for 32 cycles, 32 wave-wide fp32 operations occupy the vector
//     unit for 128.
//   * Q4_1 and Q5_1 add m * s per block (the weight block's minimum times the activation block's d * sum, the s of
//     block_q8_1).  Both factors are fp16 numbers, so sum_b m[r][b] * s[t][b] over the 4 blocks of a stage is one
//     v_mfma_f32_32x32x8f16 that adds straight into the fp32 accumulators: no vector work.
//   * A workgroup is WR x WC waves, each wave owns TM x TN MFMA tiles (32*TM rows x 32*TN tokens); LDS is
//     double buffered over stages of KB = 4 blocks with one barrier per stage and the next stage's global
//     loads in flight during the current stage's arithmetic.
#include "dev_common.h"
#include "act_layout.h"
#include "kernels.h"
#include <cstdlib>

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

template <int TM, int TN, int WR, int WC>
struct GemmCfg {
    static constexpr int NW = WR * WC, NT = NW * 64;
    static constexpr int BM = 32 * TM * WR;                        // weight rows per workgroup
    static constexpr int BN = 32 * TN * WC;                        // tokens per workgroup
    // Each (k-block, half) plane of 16-byte cells is padded by two cells: the staging threads that write one
    // stage walk the planes fastest, and a plane stride that is 2 mod 16 cells puts 16 consecutive writers on
    // 16 different bank groups (unpadded, all of them hit the same banks).
    static constexpr int A_PLANE = BM + 2, B_PLANE = BN + 2;
    static constexpr int A_CELLS = GEMM_KB * 2 * A_PLANE;          // 16-byte cells
    static constexpr int B_CELLS = GEMM_KB * 2 * B_PLANE;
    static constexpr size_t OFF_A = 0;
    static constexpr size_t OFF_B = OFF_A + (size_t)A_CELLS * 16;
    static constexpr size_t OFF_SW = OFF_B + (size_t)B_CELLS * 16;                 // fp16 [KB][BM], permuted per 32 rows
    static constexpr size_t OFF_SX = OFF_SW + (size_t)GEMM_KB * BM * 2;            // fp32 [KB][BN]
    static constexpr size_t OFF_MW = OFF_SX + (size_t)GEMM_KB * BN * 4;            // fp16 [BM][KB]: block minimum (Q4_1, Q5_1)
    static constexpr size_t OFF_MX = OFF_MW + (size_t)BM * GEMM_KB * 2;            // fp16 [BN][KB]: block_q8_1.s
    static constexpr size_t STAGE = OFF_MX + (size_t)BN * GEMM_KB * 2;
    static constexpr int W_ITEMS = BM * GEMM_KB;                   // (row, block) pairs per stage
    static constexpr int W_PER_T = (W_ITEMS + NT - 1) / NT;
    static constexpr int X_ITEMS = BN * GEMM_KB * 2;               // 16-byte activation cells per stage
    static constexpr int X_PER_T = (X_ITEMS + NT - 1) / NT;
    static constexpr int S_ITEMS = BN * GEMM_KB;                   // activation scales per stage
    static constexpr int S_PER_T = (S_ITEMS + NT - 1) / NT;
};

template <int WT, int TM, int TN, int WR, int WC, int OCC, bool GATHER>
__global__ __launch_bounds__(WR *WC * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void gemm_blk32_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K,
                                                                int64_t N, const uint8_t *__restrict__ ws,
                                                                size_t ws_stride, int64_t M, float *__restrict__ y,
                                                                int64_t ldy, TileMap map, RowGather rg, int slice_stages) {
    using C = GemmCfg<TM, TN, WR, WC>;
    using T = Blk32<WT>;
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wr = wave / WC, wc = wave % WC;
    const int half = lane >> 5, l32 = lane & 31;
    const TileCoord tc = xcd_tile(blockIdx.x, map);
    if (tc.row_tile >= map.row_tiles || tc.tok_tile >= map.tok_tiles) return;        // padding of the tile map
    const int64_t row_base = (int64_t)tc.row_tile * C::BM;
    size_t w_offset;
    const GatherView gv = resolve_gather<GATHER>(rg, w_offset, M);                   // MUL_MAT_ID: this expert's rows
    W += w_offset;
    if (gv.tok_tile < 0) return;
    const int64_t tok_base = (int64_t)(GATHER ? gv.tok_tile : tc.tok_tile) * C::BN;
    if (tok_base >= M) return;
    // split K (never with a gather, whose grid rows are the experts): grid row s takes the stages stage0 .. of every row and
    // writes its partial tile to slice s of y
    int stage0 = 0, nstages = (int)(K / (32 * GEMM_KB));
    if (!GATHER && slice_stages > 0) {
        stage0 = (int)blockIdx.y * slice_stages;
        nstages = min(slice_stages, nstages - stage0);
        y += (size_t)blockIdx.y * (size_t)M * (size_t)ldy;
    }
    const size_t off_d = q8_0_off_d(K);

    // ---- per-thread prefetch registers for one stage ----
    typename T::Raw wq[C::W_PER_T];
    uint32_t wd[C::W_PER_T];
    u32x4 xq[C::X_PER_T];
    float xs[C::S_PER_T];
    float xm[C::S_PER_T];                         // block_q8_1.s, for the types with a minimum
    const size_t off_s = q8_0_off_s(K);
    // activation rows of this thread's staging items (looked up once: with a gather they come from the pair list)
    int64_t xrow[C::X_PER_T], srow[C::S_PER_T];
#pragma unroll
    for (int i = 0; i < C::X_PER_T; i++) xrow[i] = gv.act_row(min(tok_base + (tid + i * C::NT) / (GEMM_KB * 2), M - 1));
#pragma unroll
    for (int i = 0; i < C::S_PER_T; i++) srow[i] = gv.act_row(min(tok_base + (tid + i * C::NT) / GEMM_KB, M - 1));

    auto fetch = [&](int stage) {
        const int64_t kb0 = (int64_t)(stage0 + stage) * GEMM_KB;
#pragma unroll
        for (int i = 0; i < C::W_PER_T; i++) {
            const int item = tid + i * C::NT;
            if (C::W_ITEMS % C::NT == 0 || item < C::W_ITEMS) {
                const int r = item / GEMM_KB, b = item % GEMM_KB;
                const int64_t row = min(row_base + r, N - 1);
                const uint8_t *p = W + (size_t)row * nb01 + (size_t)(kb0 + b) * T::BYTES;
                if constexpr (T::HAS_MIN) wd[i] = *reinterpret_cast<const uint32_t *>(p);          // d | m << 16
                else wd[i] = *reinterpret_cast<const unsigned short *>(p);
                T::fetch(wq[i], p);
            }
        }
#pragma unroll
        for (int i = 0; i < C::X_PER_T; i++) {
            const int item = tid + i * C::NT;
            if (C::X_ITEMS % C::NT == 0 || item < C::X_ITEMS) {
                const int c = item % (GEMM_KB * 2);                                 // c = 2*b + half
                const int64_t tok = xrow[i];
                xq[i] = *reinterpret_cast<const u32x4 *>(ws + (size_t)tok * ws_stride + (size_t)kb0 * 32 + 16 * c);
            }
        }
#pragma unroll
        for (int i = 0; i < C::S_PER_T; i++) {
            const int item = tid + i * C::NT;
            if (C::S_ITEMS % C::NT == 0 || item < C::S_ITEMS) {
                const int b = item % GEMM_KB;
                const int64_t tok = srow[i];
                xs[i] = reinterpret_cast<const float *>(ws + (size_t)tok * ws_stride + off_d)[kb0 + b];
                if constexpr (T::HAS_MIN) xm[i] = reinterpret_cast<const float *>(ws + (size_t)tok * ws_stride + off_s)[kb0 + b];
            }
        }
    };

    auto commit = [&](int buf) {
        uint8_t *base = lds + (size_t)buf * C::STAGE;
        u32x4 *A = reinterpret_cast<u32x4 *>(base + C::OFF_A);
        u32x4 *B = reinterpret_cast<u32x4 *>(base + C::OFF_B);
        unsigned short *SW = reinterpret_cast<unsigned short *>(base + C::OFF_SW);
        float *SX = reinterpret_cast<float *>(base + C::OFF_SX);
#pragma unroll
        for (int i = 0; i < C::W_PER_T; i++) {
            const int item = tid + i * C::NT;
            if (C::W_ITEMS % C::NT == 0 || item < C::W_ITEMS) {
                const int r = item / GEMM_KB, b = item % GEMM_KB;
                u32x4 lo, hi;
                T::emit(wq[i], lo, hi);
                A[(b * 2 + 0) * C::A_PLANE + r] = lo;
                A[(b * 2 + 1) * C::A_PLANE + r] = hi;
                // the lane that owns MFMA result register v of a 32-row tile holds row 8*(v/4) + 4*half + v%4;
                // store the scale of row i at half*16 + (i/8)*4 + i%4 so each lane reads its 16 scales contiguously
                const int i32 = r & 31;
                const int pos = ((i32 >> 2) & 1) * 16 + (i32 >> 3) * 4 + (i32 & 3);
                SW[b * C::BM + (r & ~31) + pos] = (unsigned short)wd[i];
                if constexpr (T::HAS_MIN) reinterpret_cast<unsigned short *>(base + C::OFF_MW)[r * GEMM_KB + b] = (unsigned short)(wd[i] >> 16);
            }
        }
#pragma unroll
        for (int i = 0; i < C::X_PER_T; i++) {
            const int item = tid + i * C::NT;
            if (C::X_ITEMS % C::NT == 0 || item < C::X_ITEMS) {
                const int c = item % (GEMM_KB * 2), n = item / (GEMM_KB * 2);
                B[c * C::B_PLANE + n] = xq[i];
            }
        }
#pragma unroll
        for (int i = 0; i < C::S_PER_T; i++) {
            const int item = tid + i * C::NT;
            if (C::S_ITEMS % C::NT == 0 || item < C::S_ITEMS) {
                const int b = item % GEMM_KB, n = item / GEMM_KB;
                SX[b * C::BN + n] = xs[i] * T::INV_MULT;                   // takes back the power of two in the weight cells
                if constexpr (T::HAS_MIN) reinterpret_cast<unsigned short *>(base + C::OFF_MX)[n * GEMM_KB + b] = f2h_rne(xm[i]);   // exact: s is an fp16 number
            }
        }
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < TN; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[a][b][v] = 0.f;

    // The magic constant lives in 16 registers for the whole kernel; the empty asm keeps the compiler from
    // re-materialising it with 16 moves in front of every MFMA.
    i32x16 magic;
#pragma unroll
    for (int v = 0; v < 16; v++) {
        int m = MAGIC_I;
        asm volatile("" : "+v"(m));
        magic[v] = m;
    }

    fetch(0);
    commit(0);
    __syncthreads();

    for (int s = 0; s < nstages; s++) {
        const int buf = s & 1;
        if (s + 1 < nstages) fetch(s + 1);

        const uint8_t *base = lds + (size_t)buf * C::STAGE;
        const u32x4 *A = reinterpret_cast<const u32x4 *>(base + C::OFF_A);
        const u32x4 *B = reinterpret_cast<const u32x4 *>(base + C::OFF_B);
        const u32x4 *SW = reinterpret_cast<const u32x4 *>(base + C::OFF_SW);
        const float *SX = reinterpret_cast<const float *>(base + C::OFF_SX);

        if constexpr (T::HAS_MIN) {
            // sum over the stage's 4 blocks of m[row][b] * s[token][b]: k = 0..3 live in lanes 0..31, k = 4..7 are zero
            f16x4 ma[TM], sb[TN];
#pragma unroll
            for (int a = 0; a < TM; a++) {
                const u32x2 t = reinterpret_cast<const u32x2 *>(base + C::OFF_MW)[(wr * TM + a) * 32 + l32];
                ma[a] = __builtin_bit_cast(f16x4, half ? u32x2{0u, 0u} : t);
            }
#pragma unroll
            for (int c = 0; c < TN; c++) {
                const u32x2 t = reinterpret_cast<const u32x2 *>(base + C::OFF_MX)[(wc * TN + c) * 32 + l32];
                sb[c] = __builtin_bit_cast(f16x4, half ? u32x2{0u, 0u} : t);
            }
#pragma unroll
            for (int a = 0; a < TM; a++)
#pragma unroll
                for (int c = 0; c < TN; c++) acc[a][c] = __builtin_amdgcn_mfma_f32_32x32x8f16(ma[a], sb[c], acc[a][c], 0, 0, 0);
        }
#pragma unroll 1
        for (int b = 0; b < GEMM_KB; b++) {
            i32x4 af[TM], bf[TN];
            u32x4 sw[TM][2];
            float dx[TN], ndx[TN];
#pragma unroll
            for (int a = 0; a < TM; a++) {
                const int r0 = (wr * TM + a) * 32;
                const u32x4 t = A[(b * 2 + half) * C::A_PLANE + r0 + l32];
                af[a] = i32x4{(int)t.x, (int)t.y, (int)t.z, (int)t.w};
                const u32x4 *sp = SW + ((size_t)b * C::BM + r0 + half * 16) / 8;    // 8 halves per 16-byte cell
                sw[a][0] = sp[0];
                sw[a][1] = sp[1];
            }
#pragma unroll
            for (int c = 0; c < TN; c++) {
                const int n0 = (wc * TN + c) * 32;
                const u32x4 t = B[(b * 2 + half) * C::B_PLANE + n0 + l32];
                bf[c] = i32x4{(int)t.x, (int)t.y, (int)t.z, (int)t.w};
                dx[c] = SX[b * C::BN + n0 + l32];
                ndx[c] = -MAGIC_F * dx[c];
            }
            if constexpr (OCC >= 4) {
                // enough waves per SIMD to cover the MFMA latency: consume each result right away (16 fewer VGPRs)
#pragma unroll
                for (int i = 0; i < TM * TN; i++) {
                    const int a = i / TN, c = i % TN;
                    const i32x16 d = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[a], bf[c], magic, 0, 0, 0);
                    const uint32_t swd[8] = {sw[a][0].x, sw[a][0].y, sw[a][0].z, sw[a][0].w,
                                             sw[a][1].x, sw[a][1].y, sw[a][1].z, sw[a][1].w};
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const float t = __builtin_fmaf(__int_as_float(d[v]), dx[c], ndx[c]);
                        const __half hw = __ushort_as_half((unsigned short)((v & 1) ? (swd[v >> 1] >> 16) : (swd[v >> 1] & 0xffffu)));
                        acc[a][c][v] = __builtin_fmaf(t, __half2float(hw), acc[a][c][v]);
                    }
                }
            } else {
                // Software pipeline over the TM*TN tiles of this k-block: the MFMA of tile i+1 is issued before
                // the 32 scaling operations of tile i.
                i32x16 d_cur = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[0], bf[0], magic, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < TM * TN; i++) {
                    const int a = i / TN, c = i % TN;
                    i32x16 d_next = d_cur;
                    if (i + 1 < TM * TN) d_next = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[(i + 1) / TN], bf[(i + 1) % TN], magic, 0, 0, 0);
                    const uint32_t swd[8] = {sw[a][0].x, sw[a][0].y, sw[a][0].z, sw[a][0].w,
                                             sw[a][1].x, sw[a][1].y, sw[a][1].z, sw[a][1].w};
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const float t = __builtin_fmaf(__int_as_float(d_cur[v]), dx[c], ndx[c]);
                        const __half hw = __ushort_as_half((unsigned short)((v & 1) ? (swd[v >> 1] >> 16) : (swd[v >> 1] & 0xffffu)));
                        acc[a][c][v] = __builtin_fmaf(t, __half2float(hw), acc[a][c][v]);
                    }
                    d_cur = d_next;
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }

        if (s + 1 < nstages) commit(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: register v of tile (a, c) is row 8*(v/4) + 4*half + v%4, token l32 ----
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int c = 0; c < TN; c++) {
            const int64_t tok = tok_base + (wc * TN + c) * 32 + l32;
            if (tok >= M) continue;
            const int64_t orow = gv.out_row(tok);
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int64_t row = row_base + (wr * TM + a) * 32 + 8 * g + 4 * half;
                float *dst = y + (size_t)orow * ldy + row;
                if (row + 3 < N && (((uintptr_t)dst) & 15) == 0) {
                    *reinterpret_cast<float4 *>(dst) = make_float4(acc[a][c][4 * g], acc[a][c][4 * g + 1], acc[a][c][4 * g + 2], acc[a][c][4 * g + 3]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (row + e < N) dst[e] = acc[a][c][4 * g + e];
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
static hipError_t launch_cfg(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int64_t M,
                             float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const RowGather &rg, int64_t n_as,
                             int slices = 1, float *part = nullptr) {
    using C = GemmCfg<TM, TN, WR, WC>;
    const size_t lds_bytes = 2 * C::STAGE;
    auto kfn = gemm_blk32_kernel<WT, TM, TN, WR, WC, OCC, GATHER>;
    static LdsGrant grant;                                               // one per kernel instantiation
    if (hipError_t e = grant_dynamic_lds(kfn, lds_bytes, lim, grant); e != hipSuccess) return e;
    // workgroups that share an XCD (OCC waves per SIMD, 32 CUs) take a compact block of output tiles
    const TileMap map = make_tile_map(ceil_div(N, C::BM), GATHER ? 1 : ceil_div(M, C::BN), 32 * (4 * OCC / C::NW > 0 ? 4 * OCC / C::NW : 1));
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
        if (slices > 1 && split.bytes >= (size_t)slices * (size_t)M * (size_t)N * sizeof(float) && (((uintptr_t)split.part) & 15) == 0)
            return launch_cfg<WT, 1, 1, 2, 2, 4, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, slices, split.part);
    }
    // 128 rows x 128 tokens per 8-wave group, 4 waves per SIMD (two groups per CU); problems too small to give
    // every CU such a group use 64 x 64 groups of 4 waves.  (CHIP_GEMM_CFG selects a shape by hand.)  Larger per-wave tiles
    // with fewer waves per SIMD measured slower on 14336 x 4096 x 2048 (Q4_0): 2 x 2 tiles at two waves 449 us against
    // 447, 4 x 2 and 2 x 4 at one wave 719 and 667 us: the scaling work is vector-bound and wants waves, not tiles.
    if (rg.perm)                                                                     // expert groups: 64 x 64 tiles
        return launch_cfg<WT, 1, 1, 2, 2, 4, true>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);
    const int64_t g128 = ceil_div(N, 128) * ceil_div(M, 128);
    const int cfg = (int)tune("CHIP_GEMM_CFG", g128 >= cus ? 0 : 1);
    switch (cfg) {
        case 0: return launch_cfg<WT, 1, 2, 4, 2, 4, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);
        case 1: return launch_cfg<WT, 1, 1, 2, 2, 4, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);
        default: return hipErrorInvalidValue;
    }
    return hipErrorInvalidValue;
}

int gemm_blk32_slices(int wtype, int64_t K, int64_t N, int64_t n, int compute_units) {
    if (!gemm_blk32_supported(wtype, K, N, n, true)) return 1;
    return blk32_slices_for(K, N, n, compute_units > 0 ? compute_units : 256);
}

int gemm_blk32_moe_tile_tokens() { return GemmCfg<1, 1, 2, 2>::BN; }   // the 64 x 64 shape serves the expert groups

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
