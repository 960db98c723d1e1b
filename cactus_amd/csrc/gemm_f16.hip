// Prefill GEMM for gfx950 over F16 weights and activations rounded to fp16: Y[t][r] = sum_k w[r][k] * a[t][k], the
// batched form of lm_ggml_vec_dot_f16 (reference ggml-cpu/ggml-cpu.c type_traits_cpu[LM_GGML_TYPE_F16], vec.cpp) as
// driven by lm_ggml_compute_forward_mul_mat (ggml-cpu/ggml-cpu.c:1257-1449): fp16 products, fp32 accumulation.
//
// v_mfma_f32_32x32x16_f16 multiplies a 32-row x 16-k weight tile by a 16-k x 32-token activation tile; products of
// fp16 numbers are exact in fp32 and the accumulator is fp32, so only the order of the additions differs from the
// reference.  Weights [N][K] and the fp16 workspace [n][K] are both contiguous along k, which is how a lane feeds the
// MFMA (8 consecutive k), so staging is a plain copy: 16-byte cells [k-group][k-half][row] in LDS, double buffered
// over stages of 64 k, the next stage's global loads in flight during the current stage's MFMAs.  There is no vector
// work per MFMA at all; a wave owns TM x TN tiles so that an LDS cell feeds TM (TN) MFMAs.
#include "dev_common.h"
#include "act_layout.h"
#include "kernels.h"
#include <cstdlib>

namespace chip {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int F16_KG = 4;                     // 16-value k-groups per LDS stage

template <int TM, int TN, int WR, int WC>
struct F16Cfg {
    static constexpr int NW = WR * WC, NT = NW * 64;
    static constexpr int BM = 32 * TM * WR;                        // weight rows per workgroup
    static constexpr int BN = 32 * TN * WC;                        // tokens per workgroup
    // plane stride 2 mod 16 cells: the staging threads of one wave spread over the bank groups
    static constexpr int A_PLANE = BM + 2, B_PLANE = BN + 2;
    static constexpr int CELLS = F16_KG * 2;                       // 16-byte cells per row and stage
    static constexpr size_t OFF_A = 0;
    static constexpr size_t OFF_B = OFF_A + (size_t)CELLS * A_PLANE * 16;
    static constexpr size_t STAGE = OFF_B + (size_t)CELLS * B_PLANE * 16;
    static constexpr int W_ITEMS = BM * CELLS, X_ITEMS = BN * CELLS;
    static constexpr int W_PER_T = W_ITEMS / NT, X_PER_T = X_ITEMS / NT;
    static_assert(W_ITEMS % NT == 0 && X_ITEMS % NT == 0, "staging items divide evenly over the threads");
};

// XF32 (row-gather mode only): the activations are read as fp32 from their own tensor - row R of the gather is token
// R % n of batch R / n - and rounded to fp16 (nearest even) on their way into LDS, instead of from an fp16 copy in the
// workspace.  Pays when the output has one or two row tiles (kqv: a head's 64 - 256 rows), so that the fp32 rows are read
// once or twice; with many row tiles the fp16 copy, read back many times, is the cheaper source.
__device__ __forceinline__ u32x4 round8_f16(const float4 a, const float4 b) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const h2 h0 = {(_Float16)a.x, (_Float16)a.y}, h1 = {(_Float16)a.z, (_Float16)a.w};
    const h2 h2v = {(_Float16)b.x, (_Float16)b.y}, h3 = {(_Float16)b.z, (_Float16)b.w};
    u32x4 r;
    r.x = __builtin_bit_cast(uint32_t, h0); r.y = __builtin_bit_cast(uint32_t, h1);
    r.z = __builtin_bit_cast(uint32_t, h2v); r.w = __builtin_bit_cast(uint32_t, h3);
    return r;
}

template <int TM, int TN, int WR, int WC, int OCC, bool GATHER, bool XF32 = false>
__global__ __launch_bounds__(WR *WC * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void gemm_f16_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N, const uint8_t *__restrict__ ws,
                     size_t ws_stride, int64_t M, float *__restrict__ y, int64_t ldy, TileMap map, RowGather rg, F32Rows fs) {
    static_assert(!XF32 || GATHER, "fp32 activation rows come with the row-gather mode");
    using C = F16Cfg<TM, TN, WR, WC>;
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave / WC, wc = wave % WC;
    const int half = lane >> 5, l32 = lane & 31;
    const TileCoord tc = xcd_tile(blockIdx.x, map);
    if (tc.row_tile >= map.row_tiles || tc.tok_tile >= map.tok_tiles) return;
    const int64_t row_base = (int64_t)tc.row_tile * C::BM;
    size_t w_offset;
    const GatherView gv = resolve_gather<GATHER>(rg, w_offset, M);                   // MUL_MAT_ID: this expert's rows
    W += w_offset;
    if (gv.tok_tile < 0) return;
    const int64_t tok_base = (int64_t)(GATHER ? gv.tok_tile : tc.tok_tile) * C::BN;
    if (tok_base >= M) return;
    // The row-gather instantiation also takes K that is not a multiple of the 64-value stage (the attention matmul over
    // n_kv cache positions, a multiple of 8): cells of the last stage that lie past K are zeroed on both sides.
    constexpr bool KTAIL = GATHER;
    const int nstages = (int)(KTAIL ? ceil_div(K, (int64_t)(16 * F16_KG)) : K / (16 * F16_KG));
    constexpr int STAGE_BYTES = 16 * F16_KG * 2;                   // bytes of one row per stage
    static_assert(C::NT % C::CELLS == 0, "a thread's items all have the same cell index");
    const int my_cell = tid % C::CELLS;

    // item = (row, cell): 8 consecutive threads copy 128 contiguous bytes of one row
    const uint8_t *wsrc[C::W_PER_T], *xsrc[C::X_PER_T];
#pragma unroll
    for (int i = 0; i < C::W_PER_T; i++) {
        const int item = tid + i * C::NT;
        wsrc[i] = W + (size_t)min(row_base + item / C::CELLS, N - 1) * nb01 + 16 * (item % C::CELLS);
    }
#pragma unroll
    for (int i = 0; i < C::X_PER_T; i++) {
        const int item = tid + i * C::NT;
        const int64_t arow = gv.act_row(min(tok_base + item / C::CELLS, M - 1));
        if constexpr (XF32) {
            const uint32_t b = (uint32_t)arow / (uint32_t)fs.n, t = (uint32_t)arow - b * (uint32_t)fs.n;
            xsrc[i] = reinterpret_cast<const uint8_t *>(fs.x + (int64_t)b * fs.ldx2 + (int64_t)t * fs.ldx1) + 32 * (item % C::CELLS);
        } else {
            xsrc[i] = ws + (size_t)arow * ws_stride + 16 * (item % C::CELLS);
        }
    }
    u32x4 wq[C::W_PER_T], xq[C::X_PER_T];

    auto fetch = [&](int stage) {
        const bool live = !KTAIL || (int64_t)stage * (16 * F16_KG) + 8 * my_cell < K;
        const size_t off = live ? (size_t)stage * STAGE_BYTES : 0;                   // a dead cell re-reads stage 0 (in bounds) and is zeroed
        const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < C::W_PER_T; i++) {
            wq[i] = *reinterpret_cast<const u32x4 *>(wsrc[i] + off);
            if (KTAIL && !live) wq[i] = z;
        }
#pragma unroll
        for (int i = 0; i < C::X_PER_T; i++) {
            if constexpr (XF32) {
                const float4 *xp = reinterpret_cast<const float4 *>(xsrc[i] + 2 * off);      // a stage is twice the bytes in fp32
                xq[i] = round8_f16(xp[0], xp[1]);
            } else {
                xq[i] = *reinterpret_cast<const u32x4 *>(xsrc[i] + off);
            }
            if (KTAIL && !live) xq[i] = z;
        }
    };
    auto commit = [&](int buf) {
        u32x4 *A = reinterpret_cast<u32x4 *>(lds + (size_t)buf * C::STAGE + C::OFF_A);
        u32x4 *B = reinterpret_cast<u32x4 *>(lds + (size_t)buf * C::STAGE + C::OFF_B);
#pragma unroll
        for (int i = 0; i < C::W_PER_T; i++) {
            const int item = tid + i * C::NT;
            A[(item % C::CELLS) * C::A_PLANE + item / C::CELLS] = wq[i];
        }
#pragma unroll
        for (int i = 0; i < C::X_PER_T; i++) {
            const int item = tid + i * C::NT;
            B[(item % C::CELLS) * C::B_PLANE + item / C::CELLS] = xq[i];
        }
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int c = 0; c < TN; c++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[a][c][v] = 0.f;

    fetch(0);
    commit(0);
    __syncthreads();

    for (int s = 0; s < nstages; s++) {
        const int buf = s & 1;
        fetch(min(s + 1, nstages - 1));                              // unconditional: the last stage is loaded twice
        const f16x8 *A = reinterpret_cast<const f16x8 *>(lds + (size_t)buf * C::STAGE + C::OFF_A);
        const f16x8 *B = reinterpret_cast<const f16x8 *>(lds + (size_t)buf * C::STAGE + C::OFF_B);
#pragma unroll
        for (int g = 0; g < F16_KG; g++) {
            f16x8 af[TM], bf[TN];
#pragma unroll
            for (int a = 0; a < TM; a++) af[a] = A[(g * 2 + half) * C::A_PLANE + (wr * TM + a) * 32 + l32];
#pragma unroll
            for (int c = 0; c < TN; c++) bf[c] = B[(g * 2 + half) * C::B_PLANE + (wc * TN + c) * 32 + l32];
#pragma unroll
            for (int a = 0; a < TM; a++)
#pragma unroll
                for (int c = 0; c < TN; c++) acc[a][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[a], bf[c], acc[a][c], 0, 0, 0);
        }
        commit(buf ^ 1);
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

// ---- the large-shape kernel: 256 x 256 output tile, 4 waves, each 128 x 128 (4 x 4 MFMA tiles, 256 accumulator registers) ----
// One wave per SIMD, so nothing hides a wait but the wave's own instruction stream: the loop is software pipelined by
// hand, one memory instruction after each MFMA.  Stages of 32 k (two k-groups of 16) in four LDS buffers.  During
// stage s a wave runs the 32 MFMAs of the stage, reads the operand registers of the next k-group (the second group of s,
// then the first group of s + 1) into the other half of a register double buffer, and issues its share of the loads of
// stage s + 3.  One barrier per stage, in the middle: it publishes stage s + 1 and separates the last reads of stage s's
// buffer from the loads the next stage aims at it.
// The operands go straight from global memory into LDS (global_load_lds_dwordx4): no staging registers, no ds_write.
// A wave instruction deposits 64 cells of 16 bytes at consecutive LDS addresses in lane order, and each lane chooses its
// own global address: four neighbouring lanes fetch the four cells of one row's 64 contiguous bytes, 16 rows per
// instruction, so LDS holds [row][4 cells] with a row pitch of 64 bytes.  A 64-byte pitch would put rows r, r + 4, r + 8,
// r + 12 into the same banks when 16 lanes read the same cell of 16 rows; cell c of row r therefore sits in slot
// c ^ ((r >> 2) & 3) (the lane that fills a slot fetches the matching cell).
// Measured on one tile with K = 4096 (32 tiles in flight, 2.39 GHz): 55 us of MFMA issue alone; 63 us with the operand
// reads (a ds_read_b128 between MFMAs costs the wave about 9 clocks); 70 us with the output stores (256 KB leave a CU at
// about 16 bytes per clock); 87 us with the loads.  What the loads cost is not latency (a fifth buffer changes nothing;
// loads that always hit the cache cost the same; half as many loads cost half) but about 37 clocks of the issuing wave
// per 1 KB written to LDS - the same as a ds_write_b128 of register-staged data costs, while plain global loads into
// registers cost nothing.  With all 256 CUs busy a tile takes 1.2 - 1.3 times longer (clock under load).
// Tried and dropped: the same tile with register staging and ds_write_b128 (111 us per tile: the waits for the loads on
// top of the write cost); a fifth stage buffer (no change); the token operands loaded by each wave from global memory
// straight into registers in MFMA layout, only the weights through LDS (154 us per tile: 32 rows x 32 bytes per load
// instruction is far slower through the texture path than it is cheap to issue).
constexpr int BIG_B = 256, BIG_K = 32;
constexpr int D_NBUF = 4, D_AHEAD = D_NBUF - 1;                  // stage s + D_AHEAD is loaded during stage s
constexpr int vmcnt_imm(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }      // s_waitcnt vmcnt(n) only
constexpr int D_OPER = BIG_B * 64;
constexpr int D_STAGE = 2 * D_OPER;
constexpr int D_LDS = D_NBUF * D_STAGE;

// The load itself is inline assembly: the compiler, which cannot tell that a load into one stage buffer does not alias a
// ds_read from another, would otherwise wait for every outstanding load before each LDS read.  The waits are placed by
// hand instead (one vmcnt per stage, below).  M0 carries the LDS byte address of the wave's 1 KB destination.  The
// compiler is not told about that write (it does not take M0 as a clobber of inline assembly), so nothing else in a kernel
// that uses this may need M0: no dynamic indexing of register arrays, no s_sendmsg.
__device__ __forceinline__ void load16_to_lds(const uint8_t *src, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_addr) : "memory");
}

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm_f16_direct_kernel(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N, const uint8_t *__restrict__ ws,
                            size_t ws_stride, int64_t M, float *__restrict__ y, int64_t ldy, TileMap map) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave >> 1, wc = wave & 1;
    const int half = lane >> 5, l32 = lane & 31;
    const TileCoord tc = xcd_tile(blockIdx.x, map);
    if (tc.row_tile >= map.row_tiles || tc.tok_tile >= map.tok_tiles) return;
    const int64_t row_base = (int64_t)tc.row_tile * BIG_B, tok_base = (int64_t)tc.tok_tile * BIG_B;
    const int nst = (int)(K / BIG_K);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;

    // loads: wave w fills rows 64 w .. 64 w + 63 of both operands, instruction j rows 64 w + 16 j + lane / 4
    const int cell = (lane & 3) ^ ((lane >> 4) & 3);
    const uint8_t *wsrc[4], *xsrc[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int r = 64 * wave + 16 * j + (lane >> 2);
        wsrc[j] = W + (size_t)min(row_base + r, N - 1) * nb01 + 16 * cell;
        xsrc[j] = ws + (size_t)min(tok_base + r, M - 1) * ws_stride + 16 * cell;
    }
    const uint32_t ld_dst = lds0 + 64 * wave * 64;                   // + 1024 j, + D_OPER for the activations
    auto load_one = [&](int i, size_t k_off, uint32_t buf_off) {     // i = 0..3 weights, 4..7 activations
        if (i < 4) load16_to_lds(wsrc[i] + k_off, __builtin_amdgcn_readfirstlane(ld_dst + buf_off + 1024 * i));
        else load16_to_lds(xsrc[i - 4] + k_off, __builtin_amdgcn_readfirstlane(ld_dst + buf_off + D_OPER + 1024 * (i - 4)));
    };
    // reads: row wr * 128 + 32 a + l32 (the swizzle term of such a row is (l32 >> 2) & 3), cell 2 g + half
    const int sw = (l32 >> 2) & 3;
    int a_rd[2], b_rd[2];
#pragma unroll
    for (int g = 0; g < 2; g++) {
        a_rd[g] = (wr * 128 + l32) * 64 + (((2 * g + half) ^ sw) << 4);
        b_rd[g] = D_OPER + (wc * 128 + l32) * 64 + (((2 * g + half) ^ sw) << 4);
    }
    auto get_a = [&](int a, int g, int buf_off) { return *reinterpret_cast<const f16x8 *>(lds + buf_off + a_rd[g] + 2048 * a); };
    auto get_b = [&](int c, int g, int buf_off) { return *reinterpret_cast<const f16x8 *>(lds + buf_off + b_rd[g] + 2048 * c); };

    f32x16 acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[a][c][v] = 0.f;

#pragma unroll
    for (int p = 0; p < D_AHEAD; p++)
#pragma unroll
        for (int i = 0; i < 8; i++) load_one(i, (size_t)min(p, nst - 1) * (BIG_K * 2), p * D_STAGE);
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();
    f16x8 af[2][4], bf[2][4];
#pragma unroll
    for (int a = 0; a < 4; a++) { af[0][a] = get_a(a, 0, 0); bf[0][a] = get_b(a, 0, 0); }

    int cur = 0, nxt = D_STAGE, fill = D_AHEAD * D_STAGE;            // buffers of stages s, s + 1, s + D_AHEAD
    for (int s = 0; s < nst; s++) {
        const size_t fill_k = (size_t)min(s + D_AHEAD, nst - 1) * (BIG_K * 2);
        // k-group 0: after each of its first 8 MFMAs one operand read of k-group 1, after each of the other 8 one load of stage s + 2
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int a = i >> 2, c = i & 3;
            acc[a][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[0][c], af[0][a], acc[a][c], 0, 0, 0);
            if (i < 4) af[1][i] = get_a(i, 1, cur);
            else if (i < 8) bf[1][i - 4] = get_b(i - 4, 1, cur);
            else {
                load_one(i - 8, fill_k, fill);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // Stage s + 1 has landed once at most the loads of the D_AHEAD - 1 stages after it are outstanding.  The barrier
        // makes every wave's share of it visible; it also separates the last reads of stage s's buffer, made just
        // above, from the loads the next stage will aim at it.
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(8 * (D_AHEAD - 1)));
        __syncthreads();
        // k-group 1: after each of its first 8 MFMAs one operand read of k-group 0 of stage s + 1
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int a = i >> 2, c = i & 3;
            acc[a][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[1][c], af[1][a], acc[a][c], 0, 0, 0);
            if (i < 4) af[0][i] = get_a(i, 0, nxt);
            else if (i < 8) bf[0][i - 4] = get_b(i - 4, 0, nxt);
            __builtin_amdgcn_sched_barrier(0);
        }
        cur = nxt;
        nxt = nxt + D_STAGE == D_LDS ? 0 : nxt + D_STAGE;
        fill = fill + D_STAGE == D_LDS ? 0 : fill + D_STAGE;
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));                       // the clamped loads of the last stages

    // The tokens are the MFMA's first operand and the weight rows its second, so a lane holds one weight row and its 16
    // registers 16 tokens: register v of tile (a, c) is token 8 (v / 4) + 4 half + v % 4, row l32.  A store instruction
    // then writes 128 contiguous bytes of two token rows.
#pragma unroll
    for (int a = 0; a < 4; a++) {
        const int64_t row = row_base + (wr * 4 + a) * 32 + l32;
        if (row >= N) continue;
#pragma unroll
        for (int c = 0; c < 4; c++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int64_t tok = tok_base + (wc * 4 + c) * 32 + 8 * (v >> 2) + 4 * half + (v & 3);
                if (tok < M) y[(size_t)tok * ldy + row] = acc[a][c][v];
            }
        }
    }
}

static hipError_t launch_f16_direct(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int64_t M,
                                    float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st) {
    static LdsGrant grant;
    if (hipError_t e = grant_dynamic_lds(gemm_f16_direct_kernel, D_LDS, lim, grant); e != hipSuccess) return e;
    const TileMap map = make_tile_map(ceil_div(N, BIG_B), ceil_div(M, BIG_B), 32);
    hipLaunchKernelGGL(gemm_f16_direct_kernel, dim3(map.grid), dim3(256), D_LDS, st, (const uint8_t *)W, nb01, K, N,
                       (const uint8_t *)ws, ws_stride, M, y, ldy, map);
    return hipGetLastError();
}

// rows must be 16-byte aligned (the weight alignment rule of the C-ABI) and K a multiple of the 64-value stage
bool gemm_f16_supported(int64_t K, int64_t N, int64_t n) { return K >= 64 && K % (16 * F16_KG) == 0 && N >= 1 && n >= 32; }

template <int TM, int TN, int WR, int WC, int OCC, bool GATHER, bool XF32 = false>
static hipError_t launch_f16(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int64_t M,
                             float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const RowGather &rg, int64_t n_as,
                             const F32Rows &fs = F32Rows{nullptr, 0, 0, 1}) {
    using C = F16Cfg<TM, TN, WR, WC>;
    const size_t lds_bytes = 2 * C::STAGE;
    auto kfn = gemm_f16_kernel<TM, TN, WR, WC, OCC, GATHER, XF32>;
    static LdsGrant grant;
    if (hipError_t e = grant_dynamic_lds(kfn, lds_bytes, lim, grant); e != hipSuccess) return e;
    const TileMap map = make_tile_map(ceil_div(N, C::BM), GATHER ? 1 : ceil_div(M, C::BN), 32 * (4 * OCC / C::NW > 0 ? 4 * OCC / C::NW : 1));
    hipLaunchKernelGGL(kfn, dim3(map.grid, (unsigned)n_as), dim3(C::NT), lds_bytes, st, (const uint8_t *)W, nb01, K, N,
                       (const uint8_t *)ws, ws_stride, M, y, ldy, map, rg, fs);
    return hipGetLastError();
}

int gemm_f16_moe_tile_tokens() { return F16Cfg<1, 1, 2, 2>::BN; }      // the 64 x 64 shape serves the expert groups

hipError_t launch_gemm_f16(const void *W, size_t nb01, int64_t K, int64_t N, const void *ws, size_t ws_stride, int64_t M,
                           float *y, int64_t ldy, const DeviceLimits &lim, hipStream_t st, const RowGather *rgp, int64_t n_as,
                           int gather_tile, const F32Rows *f32_rows) {
    if (M <= 0 || N <= 0 || n_as <= 0) return hipSuccess;
    const RowGather rg = rgp ? *rgp : RowGather{nullptr, nullptr, nullptr, 1, 1, 0};
    const int64_t cus = lim.compute_units > 0 ? lim.compute_units : 256;
    if (rg.perm) {                                                                   // row groups: the tile list was built for 64 or 128 tokens
        if (f32_rows) {
            if (gather_tile == 128) return launch_f16<2, 2, 2, 2, 2, true, true>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, *f32_rows);
            if (gather_tile != 64) return hipErrorInvalidValue;
            return launch_f16<1, 1, 2, 2, 4, true, true>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as, *f32_rows);
        }
        if (gather_tile == 128) return launch_f16<2, 2, 2, 2, 2, true>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);
        if (gather_tile != 64) return hipErrorInvalidValue;
        return launch_f16<1, 1, 2, 2, 4, true>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);
    }
    if (f32_rows) return hipErrorInvalidValue;
    const int64_t g128 = ceil_div(N, 128) * ceil_div(M, 128), g256 = ceil_div(N, 256) * ceil_div(M, 256);
    const int cfg = (int)tune("CHIP_GEMM_F16_CFG", 2 * g256 >= cus && K >= 4 * BIG_K && n_as == 1 ? 9 : g128 >= cus ? 0 : 1);
    switch (cfg) {
        case 0: return launch_f16<2, 2, 2, 2, 2, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);       // 128 x 128, 4 waves
        case 1: return launch_f16<1, 1, 2, 2, 4, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);       // 64 x 64, 4 waves
        case 2: return launch_f16<2, 2, 2, 4, 2, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);       // 128 x 256, 8 waves
        case 3: return launch_f16<2, 4, 2, 2, 2, false>(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st, rg, n_as);       // 128 x 256, 4 waves
        case 9: return launch_f16_direct(W, nb01, K, N, ws, ws_stride, M, y, ldy, lim, st);                             // 256 x 256, 4 waves, direct to LDS
        default: return hipErrorInvalidValue;
    }
}

}  // namespace chip
