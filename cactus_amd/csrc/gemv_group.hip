// Several matmuls on one activation as one launch of the decode GEMV: wq / wk / wv of an attention block, or any set of
// weight matrices (up to GROUP_MAX, types may differ within a family that shares the activation format) that read the
// same rows x.  Every workgroup belongs to one matrix and runs the ordinary GEMV body of that matrix's type on it, so each
// output equals the single-matrix launch's bit for bit; the prologue (activation quantization, launch latency) is paid
// once for the group instead of once per matrix.
// Reference: the same rows of lm_ggml_compute_forward_mul_mat (ggml-cpu/ggml-cpu.c:1257-1449), which quantizes src1
// once per node; llama.cpp builds Qcur / Kcur / Vcur from one tensor (llama-model.cpp build_llama, llama-graph.cpp).
#include "gemv_body.h"

namespace chip {

namespace {

struct GroupKernelMat {
    const uint8_t *W; size_t nb01; int64_t N; float *y; int64_t ldy; unsigned short *t16; int64_t t16_ld;
    int wtype; int first_block;
    RopeEpilogue rope;                                  // table != nullptr: the member's ROPE node runs in its epilogue
};
struct GroupKernelArgs { GroupKernelMat m[GROUP_MAX]; int count; GroupNorm norm; };

template <int WT, int NTOK, int WGS, bool FUSEQ, int DEPTH, bool ROPE, bool NORMED>
__device__ __forceinline__ void run_member(const GroupKernelMat &m, const GroupNorm &nm, int64_t K, const float *x, int64_t ldx, uint8_t *ws,
                                           size_t ws_stride, const GridPart gp) {
    SecondMatrix sec = kNoSecond;
    sec.t16 = m.t16; sec.t16_ld = m.t16_ld;
    if constexpr (ROPE && FUSEQ) {
        // the kernel for groups with ROPE epilogues, one row per step in the members that have one; NORMED: every body also runs
        // the RMS norm of the rows and the MUL with its weight in its prologue (gemv_body.h)
        if constexpr (NORMED) { sec.norm_w = nm.w; sec.norm_eps = nm.eps; sec.norm_y = nm.y; sec.norm_ldy = nm.ldy; }
        if (m.rope.table)                                               // uniform over the workgroup
            gemv_body<WT, NTOK, 1, WGS, FUSEQ, DEPTH, false, false, true, NORMED>(m.W, m.nb01, K, m.N, x, ldx, ws, ws_stride, m.y, m.ldy, sec, gp,
                                                                                  m.rope);
        else
            gemv_body<WT, NTOK, RowsPerWave<WT>::R, WGS, FUSEQ, DEPTH, false, false, false, NORMED>(m.W, m.nb01, K, m.N, x, ldx, ws, ws_stride, m.y,
                                                                                                    m.ldy, sec, gp);
        return;
    }
    gemv_body<WT, NTOK, RowsPerWave<WT>::R, WGS, FUSEQ, DEPTH>(m.W, m.nb01, K, m.N, x, ldx, ws, ws_stride, m.y, m.ldy, sec, gp);
}

// FAMILY 0: Q4_K / Q5_K / Q6_K (Q8_K activations); 1: 32-value blocks (Q8_0 / Q8_1 planes); 2: F16; 3: family 0 with Q3_K, Q2_K and
// IQ4_XS members as well - a kernel of its own, so that the kernel the common type mixes run (Q4_K_M: 0) stays as small as it was
// (with six member bodies in it the one-token wq + wk + wv launch measured 8.1 instead of 7.6 us); 4: Q4_K / Q5_K with Q6_K rows in
// planes (T_Q6_K_P), again three bodies; any other mix that contains T_Q6_K_P runs in family 3.
// FUSEQ: the workgroups quantize the fp32 rows x themselves; otherwise the workspace already holds the quantized rows
// (written by chip_mul_mat_prepare or by the kernel that produced the activations) and is only read.
// ROPE: a kernel of its own for groups in which a member's ROPE node runs in its epilogue (gemv_body.h: ROPED), so that the
// plain group kernel keeps its registers; NORMED: that kernel with the norm in front (ga.norm), again one of its own.
template <int FAMILY, int NTOK, int WGS, bool FUSEQ, int DEPTH, bool ROPE = false, bool NORMED = false>
__global__ __launch_bounds__(WGS) void gemv_group_kernel(const GroupKernelArgs ga, int64_t K, const float *__restrict__ x,
                                                         int64_t ldx, uint8_t *__restrict__ ws, size_t ws_stride) {
    int i = 0;
#pragma unroll
    for (int j = 1; j < GROUP_MAX; j++)
        if (j < ga.count && (int)blockIdx.x >= ga.m[j].first_block) i = j;
    const GroupKernelMat &m = ga.m[i];
    const int last = (i + 1 < ga.count) ? ga.m[i + 1].first_block : (int)gridDim.x;
    const GridPart gp{(int64_t)((int)blockIdx.x - m.first_block), (int64_t)(last - m.first_block), FUSEQ && blockIdx.x == 0};
    if constexpr (FAMILY == 0) {
        switch (m.wtype) {                                              // uniform over the workgroup
            case T_Q4_K: run_member<T_Q4_K, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            case T_Q5_K: run_member<T_Q5_K, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            default:     run_member<T_Q6_K, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
        }
    } else if constexpr (FAMILY == 4) {                                 // Q4_K / Q5_K with Q6_K rows in planes: the decode mix of a Q4_K_M file
        switch (m.wtype) {
            case T_Q4_K: run_member<T_Q4_K, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            case T_Q5_K: run_member<T_Q5_K, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            default:     run_member<T_Q6_K_P, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
        }
    } else if constexpr (FAMILY == 3) {
        switch (m.wtype) {
            case T_Q4_K: run_member<T_Q4_K, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            case T_Q5_K: run_member<T_Q5_K, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            case T_Q3_K: run_member<T_Q3_K, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            case T_Q2_K: run_member<T_Q2_K, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            case T_IQ4_XS: run_member<T_IQ4_XS, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            case T_Q6_K_P: run_member<T_Q6_K_P, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            default:     run_member<T_Q6_K, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
        }
    } else if constexpr (FAMILY == 1) {
        switch (m.wtype) {
            case T_Q4_0:   run_member<T_Q4_0, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            case T_Q5_0:   run_member<T_Q5_0, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            case T_IQ4_NL: run_member<T_IQ4_NL, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            case T_Q4_1:   run_member<T_Q4_1, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            case T_Q5_1:   run_member<T_Q5_1, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
            default:       run_member<T_Q8_0, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp); break;
        }
    } else {
        run_member<T_F16, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>(m, ga.norm, K, x, ldx, ws, ws_stride, gp);
    }
}

size_t image_bytes(int wtype, int64_t K) {
    switch (wtype) {
        case T_Q4_0: return lds_image_bytes<T_Q4_0>(K);
        case T_Q8_0: return lds_image_bytes<T_Q8_0>(K);
        case T_Q4_K: return lds_image_bytes<T_Q4_K>(K);
        case T_Q6_K: case T_Q6_K_P: return lds_image_bytes<T_Q6_K>(K);
        case T_Q5_0: return lds_image_bytes<T_Q5_0>(K);
        case T_Q5_K: return lds_image_bytes<T_Q5_K>(K);
        case T_Q3_K: return lds_image_bytes<T_Q3_K>(K);
        case T_Q2_K: return lds_image_bytes<T_Q2_K>(K);
        case T_IQ4_XS: return lds_image_bytes<T_IQ4_XS>(K);
        case T_IQ4_NL: return lds_image_bytes<T_IQ4_NL>(K);
        case T_Q4_1: return lds_image_bytes<T_Q4_1>(K);
        case T_Q5_1: return lds_image_bytes<T_Q5_1>(K);
        case T_F16: return lds_image_bytes<T_F16>(K);
        default: return 0;
    }
}
int rows_per_step(int wtype) { return wtype == T_Q4_0 ? RowsPerWave<T_Q4_0>::R : 1; }

template <int FAMILY, int NTOK, int WGS, bool FUSEQ, int DEPTH, bool ROPE = false, bool NORMED = false>
hipError_t launch_depth(const GroupKernelArgs &ga, int grid, int64_t K, const float *x, int64_t ldx, void *ws, size_t ws_stride,
                        size_t lds_bytes, const DeviceLimits &lim, hipStream_t st) {
    auto kfn = gemv_group_kernel<FAMILY, NTOK, WGS, FUSEQ, DEPTH, ROPE, NORMED>;
    static LdsGrant grant;
    if (hipError_t e = grant_dynamic_lds(kfn, lds_bytes, lim, grant); e != hipSuccess) return e;
    hipLaunchKernelGGL(kfn, dim3((unsigned)grid), dim3(WGS), lds_bytes, st, ga, K, x, ldx, (uint8_t *)ws, ws_stride);
    return hipGetLastError();
}
template <int FAMILY, int NTOK, int WGS>
hipError_t launch_cfg(const GroupKernelArgs &ga, int grid, int64_t K, const float *x, int64_t ldx, void *ws, size_t ws_stride,
                      size_t lds_bytes, const DeviceLimits &lim, hipStream_t st, bool prepared, bool rope) {
    if (rope) {
        if constexpr (FAMILY != 2) {
            if (!prepared && ga.norm.w)
                return launch_depth<FAMILY, NTOK, WGS, true, GEMV_DEPTH, true, true>(ga, grid, K, x, ldx, ws, ws_stride, lds_bytes, lim, st);
            if (!prepared) return launch_depth<FAMILY, NTOK, WGS, true, GEMV_DEPTH, true>(ga, grid, K, x, ldx, ws, ws_stride, lds_bytes, lim, st);
        }
        return hipErrorInvalidValue;
    }
    return prepared ? launch_depth<FAMILY, NTOK, WGS, false, GEMV_DEPTH>(ga, grid, K, x, ldx, ws, ws_stride, lds_bytes, lim, st)
                    : launch_depth<FAMILY, NTOK, WGS, true, GEMV_DEPTH>(ga, grid, K, x, ldx, ws, ws_stride, lds_bytes, lim, st);
}
template <int FAMILY, int NTOK>
hipError_t launch_wgs(int wgs, const GroupKernelArgs &ga, int grid, int64_t K, const float *x, int64_t ldx, void *ws,
                      size_t ws_stride, size_t lds_bytes, const DeviceLimits &lim, hipStream_t st, bool prepared, bool rope) {
    return wgs == 1024 ? launch_cfg<FAMILY, NTOK, 1024>(ga, grid, K, x, ldx, ws, ws_stride, lds_bytes, lim, st, prepared, rope)
                       : launch_cfg<FAMILY, NTOK, 512>(ga, grid, K, x, ldx, ws, ws_stride, lds_bytes, lim, st, prepared, rope);
}
template <int FAMILY>
hipError_t launch_ntok(int n, int wgs, const GroupKernelArgs &ga, int grid, int64_t K, const float *x, int64_t ldx, void *ws,
                       size_t ws_stride, size_t lds_bytes, const DeviceLimits &lim, hipStream_t st, bool prepared, bool rope) {
    switch (n) {
        case 1: return launch_wgs<FAMILY, 1>(wgs, ga, grid, K, x, ldx, ws, ws_stride, lds_bytes, lim, st, prepared, rope);
        case 2: return launch_wgs<FAMILY, 2>(wgs, ga, grid, K, x, ldx, ws, ws_stride, lds_bytes, lim, st, prepared, rope);
        case 4: return launch_wgs<FAMILY, 4>(wgs, ga, grid, K, x, ldx, ws, ws_stride, lds_bytes, lim, st, prepared, rope);
        case 8:                                                          // over prepared rows only
            if (!prepared || rope) return hipErrorInvalidValue;
            return wgs == 1024 ? launch_depth<FAMILY, 8, 1024, false, GEMV_DEPTH>(ga, grid, K, x, ldx, ws, ws_stride, lds_bytes, lim, st)
                               : launch_depth<FAMILY, 8, 512, false, GEMV_DEPTH>(ga, grid, K, x, ldx, ws, ws_stride, lds_bytes, lim, st);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

int gemv_group_family(int wtype) {
    switch (wtype) {
        case T_Q4_K: case T_Q5_K: case T_Q6_K: case T_Q3_K: case T_Q2_K: case T_IQ4_XS: case T_Q6_K_P: return 0;
        case T_Q4_0: case T_Q8_0: case T_Q5_0: case T_IQ4_NL: case T_Q4_1: case T_Q5_1: return 1;
        case T_F16: return 2;
        default: return -1;
    }
}

// One launch serves the group when the prologue-quantizing GEMV takes every member (n in {1, 2, 4}, n * K within its
// limit, the largest member's activation image within LDS) and the members are of one family.  Over prepared rows also
// 8 tokens: for matrices that are small enough to be all latency (wq + wk + wv at 8 tokens: one quantizer and three
// launches took 22 us) one launch of the dot-product GEMV beats a matrix-core GEMV launch per member.
bool gemv_group_applicable(const GroupMat *mats, int count, int64_t K, int n, const DeviceLimits &lim, bool prepared) {
    if (count < 1 || count > GROUP_MAX) return false;
    if (n != 1 && n != 2 && n != 4 && !(prepared && n == 8)) return false;
    const int fam = gemv_group_family(mats[0].wtype);
    if (fam < 0) return false;
    int64_t rows = 0;
    for (int i = 0; i < count; i++) {
        if (gemv_group_family(mats[i].wtype) != fam) return false;
        // over prepared rows the only limit is the activation image of n rows in LDS; quantizing in the prologue has its own
        if (prepared ? (size_t)n * image_bytes(mats[i].wtype, K) > (size_t)lim.max_lds_per_block || image_bytes(mats[i].wtype, K) == 0
                     : !gemv_fused_applicable(mats[i].wtype, K, n, lim))
            return false;
        if (mats[i].N <= 0 || mats[i].N > 0x7fffffff) return false;
        rows += mats[i].N;
    }
    // Q8_1 members (Q4_1 / Q5_1) need the same planes as Q8_0 members: one workspace dump serves both
    return rows <= 0x7fffffff;
}

hipError_t launch_gemv_group(const GroupMat *mats, int count, int64_t K, const float *x, int64_t ldx, int n, void *ws,
                             size_t ws_stride, const DeviceLimits &lim, hipStream_t st, bool prepared, const GroupNorm *norm) {
    if (!gemv_group_applicable(mats, count, K, n, lim, prepared)) return hipErrorInvalidValue;
    const int cus = lim.compute_units > 0 ? lim.compute_units : 256;
    const int fam = gemv_group_family(mats[0].wtype);
    size_t img = 0;
    int64_t tiles = 0;
    for (int i = 0; i < count; i++) {
        const size_t b = image_bytes(mats[i].wtype, K);
        if (b > img) img = b;
        tiles += ceil_div(mats[i].N, (int64_t)rows_per_step(mats[i].wtype));
    }
    // members whose ROPE node runs in their epilogue: one row per step (pairs of rows per wave), the cos / sin table behind the image
    bool rope = false;
    int rope_dims = 0;
    for (int i = 0; i < count; i++) {
        const RopeEpilogue &r = mats[i].rope;
        if (!r.table) continue;
        if (prepared || fam == 2 || r.head_dim <= 0 || (r.head_dim & 1) || r.n_dims <= 0 || (r.n_dims & 1) || r.n_dims > r.head_dim ||
            mats[i].N % r.head_dim != 0 || (!r.write_f32 && !r.h16) || mats[i].t16)
            return hipErrorInvalidValue;
        rope = true;
        if (r.n_dims > rope_dims) rope_dims = r.n_dims;
        tiles += mats[i].N - ceil_div(mats[i].N, (int64_t)rows_per_step(mats[i].wtype));
    }
    size_t lds_bytes = (size_t)n * img + (size_t)n * rope_dims * sizeof(float);
    if (norm && norm->w) {                                               // only the kernel with ROPE epilogues is built with it
        if (!rope || K > 256 * NORM_BLOCKS_MAX) return hipErrorInvalidValue;
        lds_bytes = ((lds_bytes + 7) & ~(size_t)7) + (size_t)n * NORM_BLOCKS_MAX * sizeof(double);   // the block sums, behind image and table
    }
    if (lds_bytes > (size_t)lim.max_lds_per_block) return hipErrorInvalidValue;
    // As the single-matrix launcher: a persistent grid; one 16-wave workgroup per CU while every wave gets at most a
    // couple of tiles (the prologue is then most of the kernel and is paid once per CU), else two 8-wave workgroups.
    const int wgs = (int)tune("CHIP_GROUP_WGS", tiles <= 32 * (int64_t)cus ? 1024 : 512);
    // the K-quant and block-32 kernels keep 4 - 5 waves per SIMD (the registers of their most demanding member type): two
    // 8-wave workgroups per CU; the F16 kernel keeps 8 and takes three for one token
    const int per_cu = (int)tune("CHIP_GROUP_PER_CU", (wgs == 1024 || lds_bytes > 24 * 1024) ? 1 : (fam == 2 && n == 1 && !prepared ? 3 : 2));
    int grid = cus * per_cu;
    const int64_t max_useful = ceil_div(tiles, (int64_t)(wgs / 64));
    if (grid > max_useful) grid = (int)max_useful;
    if (grid < count) grid = count;
    // Workgroups per member so that the waves that stream the most bytes stream as few as possible.  A member's waves walk its
    // tiles (a row, R rows, or the two rows of a rotated pair) in turn, so each streams ceil(tiles / waves) tiles: every member
    // starts with one workgroup, each further one goes to the member whose waves stream the most, and at the end a member keeps
    // only as many as that load needs.  (In proportion to the members' bytes, wq + wk + wv of a Q4_K_M layer left wv's waves two
    // 3360-byte rows each while wq's took two 2304-byte rows: 6.6 us against 5.8 us this way.)
    const int waves = wgs / 64;
    int64_t mtiles[GROUP_MAX];
    double tile_bytes[GROUP_MAX];
    for (int i = 0; i < count; i++) {
        const int64_t r = mats[i].rope.table ? 2 : rows_per_step(mats[i].wtype);
        mtiles[i] = ceil_div(mats[i].N, r);
        tile_bytes[i] = (double)r * (double)mats[i].nb01;
    }
    auto wave_load = [&](int i, int b) { return (double)ceil_div(mtiles[i], (int64_t)b * waves) * tile_bytes[i]; };
    int blocks[GROUP_MAX], given = count;
    for (int i = 0; i < count; i++) blocks[i] = 1;
    while (given < grid) {
        int worst = 0;
        for (int i = 1; i < count; i++) if (wave_load(i, blocks[i]) > wave_load(worst, blocks[worst])) worst = i;
        if (ceil_div(mtiles[worst], (int64_t)blocks[worst] * waves) <= 1) break;      // one tile per wave already: nothing left to split
        blocks[worst]++; given++;
    }
    for (int i = 0; i < count; i++) {
        const int64_t per_wave = ceil_div(mtiles[i], (int64_t)blocks[i] * waves);
        blocks[i] = (int)ceil_div(ceil_div(mtiles[i], per_wave), (int64_t)waves);
    }
    GroupKernelArgs ga{};
    ga.count = count;
    ga.norm = (norm && norm->w) ? *norm : GroupNorm{nullptr, 0.f, nullptr, 0};
    int first = 0;
    for (int i = 0; i < count; i++) {
        ga.m[i] = GroupKernelMat{(const uint8_t *)mats[i].W, mats[i].nb01, mats[i].N, mats[i].y, mats[i].ldy, mats[i].t16,
                                 mats[i].t16_ld, mats[i].wtype, first, mats[i].rope};
        first += blocks[i];
    }
    bool low_bit = false, planes = false, raw6 = false;
    for (int i = 0; i < count; i++) {
        low_bit = low_bit || mats[i].wtype == T_Q3_K || mats[i].wtype == T_Q2_K || mats[i].wtype == T_IQ4_XS;
        planes = planes || mats[i].wtype == T_Q6_K_P;
        raw6 = raw6 || mats[i].wtype == T_Q6_K;
    }
    switch (fam != 0 ? fam : (low_bit || (planes && raw6)) ? 3 : planes ? 4 : 0) {
        case 3: return launch_ntok<3>(n, wgs, ga, first, K, x, ldx, ws, ws_stride, lds_bytes, lim, st, prepared, rope);
        case 4: return launch_ntok<4>(n, wgs, ga, first, K, x, ldx, ws, ws_stride, lds_bytes, lim, st, prepared, rope);
        case 0: return launch_ntok<0>(n, wgs, ga, first, K, x, ldx, ws, ws_stride, lds_bytes, lim, st, prepared, rope);
        case 1: return launch_ntok<1>(n, wgs, ga, first, K, x, ldx, ws, ws_stride, lds_bytes, lim, st, prepared, rope);
        default: return launch_ntok<2>(n, wgs, ga, first, K, x, ldx, ws, ws_stride, lds_bytes, lim, st, prepared, rope);
    }
}

}  // namespace chip
