// Device code shared by the decode GEMV kernels (gemv.hip: one matrix, a pair, MUL_MAT_ID; gemv_group.hip: several
// matrices of different types on one activation): per weight type the mapping of a lane's unit to weight bytes and to
// the activation image in LDS, the prologue that builds that image (quantizing fp32 rows, or staging prepared rows),
// and the body every workgroup runs.
#pragma once
#include "dev_common.h"
#include "act_layout.h"
#include "quant_dev.h"
#include "kernels.h"

namespace chip {

// Weight loads are ordinary cached loads.  A lane's unit is 36..68 bytes, so neighbouring load instructions of
// a wave touch the same 128-byte lines; with the non-temporal hint those lines are not kept between instructions
// and the kernel runs ~60 % slower (measured: 18 us instead of 11 us on a 48 MB matrix).
#define WLOAD(ptr) (*(ptr))

// ------------------------------------------------------------------------------------------------ traits
// For each weight type: how a lane's unit maps to weight bytes and to activation planes.
//   UNIT_ELEMS : K elements covered by one lane-unit
//   QCH        : 16-byte activation chunks per unit
//   AUX        : bytes of per-unit activation side data (scales, sums) kept in LDS
template <int WT> struct Traits;

template <> struct Traits<T_Q8_0> {
    static constexpr int ACT = T_Q8_0, UNIT_ELEMS = 64, QCH = 4, AUX = 8;
    static constexpr bool A_HAS_SUMS = false;                   // A carries the per-block activation sums
    struct W { uint32_t q[16]; float d0, d1; };
    struct A { uint32_t q[16]; float d0, d1; };
    struct Raw { u32x4 a, b, c, e; uint32_t f; };

    __device__ static __forceinline__ void load_raw(Raw &r, const uint8_t *row, int u) {
        const uint8_t *p = row + (size_t)u * 68;                       // two 34-byte blocks, 4-byte aligned
        r.a = WLOAD(reinterpret_cast<const u32x4_a4 *>(p));
        r.b = WLOAD(reinterpret_cast<const u32x4_a4 *>(p + 16));
        r.c = WLOAD(reinterpret_cast<const u32x4_a4 *>(p + 32));
        r.e = WLOAD(reinterpret_cast<const u32x4_a4 *>(p + 48));
        r.f = WLOAD(reinterpret_cast<const uint32_t *>(p + 64));
    }
    __device__ static __forceinline__ void decode(W &w, const Raw &r, int) {
        const u32x4 a = r.a, b = r.b, c = r.c, e = r.e;
        const uint32_t f = r.f;
        // block 0: d at byte 0, quants at bytes 2..33 -> re-slice by 16 bits; block 1: d at 34, quants at 36..67
        w.d0 = h2f(a.x);
        w.q[0] = shr16(a.y, a.x); w.q[1] = shr16(a.z, a.y); w.q[2] = shr16(a.w, a.z); w.q[3] = shr16(b.x, a.w);
        w.q[4] = shr16(b.y, b.x); w.q[5] = shr16(b.z, b.y); w.q[6] = shr16(b.w, b.z); w.q[7] = shr16(c.x, b.w);
        w.d1 = h2f(c.x >> 16);
        w.q[8] = c.y; w.q[9] = c.z; w.q[10] = c.w; w.q[11] = e.x;
        w.q[12] = e.y; w.q[13] = e.z; w.q[14] = e.w; w.q[15] = f;
    }
    __device__ static __forceinline__ void load_a(A &a, const uint8_t *tok, int NI, int it, int lane) {
        const u32x4 *q = reinterpret_cast<const u32x4 *>(tok) + (size_t)it * QCH * 64 + lane;
#pragma unroll
        for (int j = 0; j < QCH; j++) {
            const u32x4 v = q[j * 64];
            a.q[4 * j] = v.x; a.q[4 * j + 1] = v.y; a.q[4 * j + 2] = v.z; a.q[4 * j + 3] = v.w;
        }
        const float2 d = reinterpret_cast<const float2 *>(tok + (size_t)NI * QCH * 1024)[it * 64 + lane];
        a.d0 = d.x; a.d1 = d.y;
    }
    __device__ static __forceinline__ void isums(const W &w, const A &a, int &i0, int &i1) {
        i0 = 0; i1 = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) { i0 = dot4(w.q[i], a.q[i], i0); i1 = dot4(w.q[8 + i], a.q[8 + i], i1); }
    }
    __device__ static __forceinline__ float dot(const W &w, const A &a, float acc) {
        int i0, i1;
        isums(w, a, i0, i1);
        acc = __builtin_fmaf(w.d0 * a.d0, (float)i0, acc);
        return __builtin_fmaf(w.d1 * a.d1, (float)i1, acc);
    }
    // staging: where unit u's chunk j and side data live in the split workspace planes of one token
    __device__ static __forceinline__ size_t src_chunk(int64_t, int u, int j) { return (size_t)u * 64 + 16 * j; }
    using AuxT = float2;
    __device__ static __forceinline__ AuxT aux_load(const uint8_t *ws, int64_t K, int u, bool valid) {
        float2 d = make_float2(0.f, 0.f);
        if (valid) d = reinterpret_cast<const float2 *>(ws + q8_0_off_d(K))[u];
        return d;
    }
    // fused prologue: where the dword of elements e..e+3 and the side data of 32-block blk go in the LDS image
    __device__ static __forceinline__ size_t img_qs(int, int e) {
        const int b = e >> 5, u = b >> 1, off = 32 * (b & 1) + (e & 31);
        return ((size_t)((u >> 6) * QCH + (off >> 4)) * 64 + (u & 63)) * 16 + (off & 15);
    }
    __device__ static __forceinline__ void img_block_aux(uint8_t *img, int NI, int blk, float d, int, float) {
        reinterpret_cast<float *>(img + (size_t)NI * QCH * 1024 + (size_t)(blk >> 1) * AUX)[blk & 1] = d;
    }
};

template <> struct Traits<T_Q4_0> {
    static constexpr int ACT = T_Q8_0, UNIT_ELEMS = 64, QCH = 4, AUX = 16;
    static constexpr bool A_HAS_SUMS = true;
    struct W { uint32_t lo[8], hi[8]; float d0, d1; };          // nibbles spread to bytes, 0..15
    struct A { uint32_t q[16]; float d0, d1; int s0, s1; };

    struct Raw { u32x4 a, b; uint32_t c; };
    __device__ static __forceinline__ void load_raw(Raw &r, const uint8_t *row, int u) {
        const uint8_t *p = row + (size_t)u * 36;                       // two 18-byte blocks, 4-byte aligned
        r.a = WLOAD(reinterpret_cast<const u32x4_a4 *>(p));
        r.b = WLOAD(reinterpret_cast<const u32x4_a4 *>(p + 16));
        r.c = WLOAD(reinterpret_cast<const uint32_t *>(p + 32));
    }
    __device__ static __forceinline__ void decode(W &w, const Raw &r, int) {
        const u32x4 a = r.a, b = r.b;
        const uint32_t c = r.c;
        uint32_t q[8];
        w.d0 = h2f(a.x);
        q[0] = shr16(a.y, a.x); q[1] = shr16(a.z, a.y); q[2] = shr16(a.w, a.z); q[3] = shr16(b.x, a.w);
        w.d1 = h2f(b.x >> 16);
        q[4] = b.y; q[5] = b.z; q[6] = b.w; q[7] = c;
#pragma unroll
        for (int i = 0; i < 8; i++) { w.lo[i] = q[i] & 0x0f0f0f0fu; w.hi[i] = (q[i] >> 4) & 0x0f0f0f0fu; }
    }
    __device__ static __forceinline__ void load_a(A &a, const uint8_t *tok, int NI, int it, int lane) {
        const u32x4 *q = reinterpret_cast<const u32x4 *>(tok) + (size_t)it * QCH * 64 + lane;
#pragma unroll
        for (int j = 0; j < QCH; j++) {
            const u32x4 v = q[j * 64];
            a.q[4 * j] = v.x; a.q[4 * j + 1] = v.y; a.q[4 * j + 2] = v.z; a.q[4 * j + 3] = v.w;
        }
        const u32x4 x = reinterpret_cast<const u32x4 *>(tok + (size_t)NI * QCH * 1024)[it * 64 + lane];
        a.d0 = __uint_as_float(x.x); a.d1 = __uint_as_float(x.y); a.s0 = (int)x.z; a.s1 = (int)x.w;
    }
    // byte i of qs holds element i (low nibble) and element i+16 (high nibble); value = nibble - 8
    __device__ static __forceinline__ void isums(const W &w, const A &a, int &i0, int &i1) {
        i0 = -8 * a.s0; i1 = -8 * a.s1;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            i0 = dot4(w.lo[i], a.q[i], i0);         i0 = dot4(w.hi[i], a.q[4 + i], i0);
            i1 = dot4(w.lo[4 + i], a.q[8 + i], i1); i1 = dot4(w.hi[4 + i], a.q[12 + i], i1);
        }
    }
    __device__ static __forceinline__ float dot(const W &w, const A &a, float acc) {
        int i0, i1;
        isums(w, a, i0, i1);
        acc = __builtin_fmaf(w.d0 * a.d0, (float)i0, acc);
        return __builtin_fmaf(w.d1 * a.d1, (float)i1, acc);
    }
    __device__ static __forceinline__ size_t src_chunk(int64_t, int u, int j) { return (size_t)u * 64 + 16 * j; }
    using AuxT = u32x4;
    __device__ static __forceinline__ AuxT aux_load(const uint8_t *ws, int64_t K, int u, bool valid) {
        u32x4 x = {0u, 0u, 0u, 0u};
        if (valid) {
            const u32x2 d = reinterpret_cast<const u32x2 *>(ws + q8_0_off_d(K))[u];
            const u32x2 s = reinterpret_cast<const u32x2 *>(ws + q8_0_off_sum(K))[u];
            x.x = d.x; x.y = d.y; x.z = s.x; x.w = s.y;
        }
        return x;
    }
    __device__ static __forceinline__ size_t img_qs(int, int e) {
        const int b = e >> 5, u = b >> 1, off = 32 * (b & 1) + (e & 31);
        return ((size_t)((u >> 6) * QCH + (off >> 4)) * 64 + (u & 63)) * 16 + (off & 15);
    }
    __device__ static __forceinline__ void img_block_aux(uint8_t *img, int NI, int blk, float d, int sum, float) {
        uint8_t *a = img + (size_t)NI * QCH * 1024 + (size_t)(blk >> 1) * AUX;
        reinterpret_cast<float *>(a)[blk & 1] = d;
        reinterpret_cast<int *>(a)[2 + (blk & 1)] = sum;
    }
};

template <> struct Traits<T_Q4_K> {
    // unit = (super-block sb, 64-value group jp of 4): the 32 qs bytes 32*jp..32*jp+31, whose low nibbles are
    // elements 64*jp + [0,32) (sub-block 2*jp) and whose high nibbles are elements 64*jp + 32 + [0,32)
    // (sub-block 2*jp+1).  The matching activations are the 64 contiguous quants 64*jp..64*jp+63.
    static constexpr int ACT = T_Q8_K, UNIT_ELEMS = 64, QCH = 4, AUX = 8;
    static constexpr int KQ_STYLE = 0;                          // activation side data: two 32-value sub-block sums
    struct W { uint32_t lo[8], hi[8]; float d, dmin; int sc0, sc1, m0, m1; };
    struct A { uint32_t q[16]; float d; int s0, s1; };
    struct Raw { u32x4 h, q0, q1; };

    __device__ static __forceinline__ void load_raw(Raw &r, const uint8_t *row, int u) {
        const int sb = u >> 2, jp = u & 3;
        const uint8_t *p = row + (size_t)sb * BYTES_Q4_K;              // 144-byte super-block, 16-byte aligned
        r.h = WLOAD(reinterpret_cast<const u32x4 *>(p));
        r.q0 = WLOAD(reinterpret_cast<const u32x4 *>(p + 16 + 32 * jp));
        r.q1 = WLOAD(reinterpret_cast<const u32x4 *>(p + 32 + 32 * jp));
    }
    __device__ static __forceinline__ void decode(W &w, const Raw &r, int u) {
        const int jp = u & 3;
        const u32x4 h = r.h;
        w.d = h2f(h.x); w.dmin = h2f(h.x >> 16);
        // 6-bit scale/min of sub-blocks (2jp, 2jp+1) (reference ggml-quants.c:625-632)
        const int sh = 16 * (jp & 1);
        const uint32_t a1 = h.y >> sh, a2 = h.z >> sh, a3 = h.w >> sh;
        uint32_t sc, mn;
        if (jp < 2) { sc = a1 & 0x3f3fu; mn = a2 & 0x3f3fu; }
        else        { sc = (a3 & 0x0f0fu) | ((a1 >> 2) & 0x3030u); mn = ((a3 >> 4) & 0x0f0fu) | ((a2 >> 2) & 0x3030u); }
        w.sc0 = sc & 0xff; w.sc1 = sc >> 8; w.m0 = mn & 0xff; w.m1 = mn >> 8;
        const uint32_t q[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
        for (int i = 0; i < 8; i++) { w.lo[i] = q[i] & 0x0f0f0f0fu; w.hi[i] = (q[i] >> 4) & 0x0f0f0f0fu; }
    }
    __device__ static __forceinline__ void load_a(A &a, const uint8_t *tok, int NI, int it, int lane) {
        const u32x4 *q = reinterpret_cast<const u32x4 *>(tok) + (size_t)it * QCH * 64 + lane;
#pragma unroll
        for (int j = 0; j < QCH; j++) {
            const u32x4 v = q[j * 64];
            a.q[4 * j] = v.x; a.q[4 * j + 1] = v.y; a.q[4 * j + 2] = v.z; a.q[4 * j + 3] = v.w;
        }
        const u32x2 x = reinterpret_cast<const u32x2 *>(tok + (size_t)NI * QCH * 1024)[it * 64 + lane];
        a.d = __uint_as_float(x.x);
        a.s0 = (int)(int16_t)(x.y & 0xffff); a.s1 = (int)(int16_t)(x.y >> 16);
    }
    // this unit's share of the super-block sums: isum = sum_j sc_j * dot_j, imin = sum_j m_j * (sum of sub-block j)
    __device__ static __forceinline__ void isums(const W &w, const A &a, int &is, int &im) {
        int dl = 0, dh = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) { dl = dot4(w.lo[i], a.q[i], dl); dh = dot4(w.hi[i], a.q[8 + i], dh); }
        is = w.sc0 * dl + w.sc1 * dh;
        im = w.m0 * a.s0 + w.m1 * a.s1;
    }
    __device__ static __forceinline__ float dot(const W &w, const A &a, float acc) {
        int is, im;
        isums(w, a, is, im);
        acc = __builtin_fmaf(w.d * a.d, (float)is, acc);
        return __builtin_fmaf(-(w.dmin * a.d), (float)im, acc);
    }
    __device__ static __forceinline__ size_t src_chunk(int64_t, int u, int j) { return (size_t)u * 64 + 16 * j; }
    using AuxT = u32x2;
    __device__ static __forceinline__ AuxT aux_load(const uint8_t *ws, int64_t K, int u, bool valid) {
        u32x2 x = {0u, 0u};
        if (valid) {
            const int sb = u >> 2, jp = u & 3;
            const int16_t *bs = reinterpret_cast<const int16_t *>(ws + q8_K_off_bsums(K)) + sb * 16 + 4 * jp;
            x.x = reinterpret_cast<const uint32_t *>(ws + q8_K_off_d(K))[sb];
            x.y = (uint32_t)(uint16_t)(bs[0] + bs[1]) | ((uint32_t)(uint16_t)(bs[2] + bs[3]) << 16);
        }
        return x;
    }
    // fused prologue (one wave per super-block sb; lane holds elements 4*lane..4*lane+3 of it)
    static constexpr int UNITS_PER_SB = 4;
    __device__ static __forceinline__ size_t img_qs(int, int e) {
        const int u = e >> 6, off = e & 63;
        return ((size_t)((u >> 6) * QCH + (off >> 4)) * 64 + (u & 63)) * 16 + (off & 15);
    }
    __device__ static __forceinline__ uint8_t *img_aux(uint8_t *img, int NI, int u) { return img + (size_t)NI * QCH * 1024 + (size_t)u * AUX; }
    // called by all 64 lanes with the sum of their 16-value group: sub-block sums are two groups (8 lanes)
    __device__ static __forceinline__ void img_bsum(uint8_t *img, int NI, int sb, int lane, int s16) {
        const int s32 = s16 + __builtin_amdgcn_update_dpp(0, s16, 0x141, 0xf, 0xf, true);
        if ((lane & 7) == 0) {
            const int g32 = lane >> 3;                                  // sub-block index 0..7
            reinterpret_cast<int16_t *>(img_aux(img, NI, sb * 4 + (g32 >> 1)) + 4)[g32 & 1] = (int16_t)s32;
        }
    }
};

template <> struct Traits<T_Q6_K> {
    // unit = (super-block sb, half h, ip): 16 consecutive l = 16*ip + [0,16) of half h, i.e. the four
    // 16-element groups {128h + 32v + 16ip + [0,16) : v = 0..3}; scale of group v is scales[8h + 2v + ip]
    static constexpr int ACT = T_Q8_K, UNIT_ELEMS = 64, QCH = 4, AUX = 16;
    static constexpr int KQ_STYLE = 1;                          // four 16-value group sums
    struct W { uint32_t q[16]; float d; int sc[4]; };            // q[4v + k]: 6-bit values 0..63 of group v
    struct A { uint32_t q[16]; float d; int bs[4]; };

    struct Raw { u32x4 l0, l1, qh; u32x2 s; uint32_t d; };
    __device__ static __forceinline__ void load_raw(Raw &r, const uint8_t *row, int u) {
        const int sb = u >> 2, h = (u >> 1) & 1, ip = u & 1;
        const uint8_t *p = row + (size_t)sb * BYTES_Q6_K;              // 210-byte super-block, 2-byte aligned
        r.l0 = WLOAD(reinterpret_cast<const u32x4_a2 *>(p + 64 * h + 16 * ip));
        r.l1 = WLOAD(reinterpret_cast<const u32x4_a2 *>(p + 64 * h + 32 + 16 * ip));
        r.qh = WLOAD(reinterpret_cast<const u32x4_a2 *>(p + 128 + 32 * h + 16 * ip));
        r.s  = WLOAD(reinterpret_cast<const u32x2_a2 *>(p + 192 + 8 * h));
        r.d  = WLOAD(reinterpret_cast<const unsigned short *>(p + 208));
    }
    __device__ static __forceinline__ void decode(W &w, const Raw &r, int u) {
        const int ip = u & 1;
        const u32x4 l0 = r.l0, l1 = r.l1, qh = r.qh;
        const u32x2 s = r.s;
        w.d = h2f(r.d);
        const uint32_t ql0[4] = {l0.x, l0.y, l0.z, l0.w}, ql1[4] = {l1.x, l1.y, l1.z, l1.w}, hh[4] = {qh.x, qh.y, qh.z, qh.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {                                   // reference ggml-quants.c:1695-1711
            w.q[k]      = (ql0[k] & 0x0f0f0f0fu)        | ((hh[k] << 4) & 0x30303030u);
            w.q[4 + k]  = (ql1[k] & 0x0f0f0f0fu)        | ((hh[k] << 2) & 0x30303030u);
            w.q[8 + k]  = ((ql0[k] >> 4) & 0x0f0f0f0fu) | (hh[k] & 0x30303030u);
            w.q[12 + k] = ((ql1[k] >> 4) & 0x0f0f0f0fu) | ((hh[k] >> 2) & 0x30303030u);
        }
        const int b = 8 * ip;                                           // scales[8h + 2v + ip]: byte ip / ip+2 of each dword
        w.sc[0] = (int)(int8_t)(s.x >> b); w.sc[1] = (int)(int8_t)(s.x >> (b + 16));
        w.sc[2] = (int)(int8_t)(s.y >> b); w.sc[3] = (int)(int8_t)(s.y >> (b + 16));
    }
    __device__ static __forceinline__ void load_a(A &a, const uint8_t *tok, int NI, int it, int lane) {
        const u32x4 *q = reinterpret_cast<const u32x4 *>(tok) + (size_t)it * QCH * 64 + lane;
#pragma unroll
        for (int j = 0; j < QCH; j++) {
            const u32x4 v = q[j * 64];
            a.q[4 * j] = v.x; a.q[4 * j + 1] = v.y; a.q[4 * j + 2] = v.z; a.q[4 * j + 3] = v.w;
        }
        const u32x4 x = reinterpret_cast<const u32x4 *>(tok + (size_t)NI * QCH * 1024)[it * 64 + lane];
        a.d = __uint_as_float(x.x);
        a.bs[0] = (int)(int16_t)(x.y & 0xffff); a.bs[1] = (int)(int16_t)(x.y >> 16);
        a.bs[2] = (int)(int16_t)(x.z & 0xffff); a.bs[3] = (int)(int16_t)(x.z >> 16);
    }
    __device__ static __forceinline__ void isums(const W &w, const A &a, int &is, int &unused) {
        is = 0; unused = 0;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            int dv = -32 * a.bs[v];                                     // sum (q-32)*a = sum q*a - 32*sum a
#pragma unroll
            for (int k = 0; k < 4; k++) dv = dot4(w.q[4 * v + k], a.q[4 * v + k], dv);
            is += w.sc[v] * dv;
        }
    }
    __device__ static __forceinline__ float dot(const W &w, const A &a, float acc) {
        int is, unused;
        isums(w, a, is, unused);
        return __builtin_fmaf(w.d * a.d, (float)is, acc);
    }
    __device__ static __forceinline__ size_t src_chunk(int64_t, int u, int j) {
        const int sb = u >> 2, h = (u >> 1) & 1, ip = u & 1;
        return (size_t)sb * 256 + 128 * h + 32 * j + 16 * ip;
    }
    using AuxT = u32x4;
    __device__ static __forceinline__ AuxT aux_load(const uint8_t *ws, int64_t K, int u, bool valid) {
        u32x4 x = {0u, 0u, 0u, 0u};
        if (valid) {
            const int sb = u >> 2, h = (u >> 1) & 1, ip = u & 1;
            const int16_t *bs = reinterpret_cast<const int16_t *>(ws + q8_K_off_bsums(K)) + sb * 16 + 8 * h + ip;
            x.x = reinterpret_cast<const uint32_t *>(ws + q8_K_off_d(K))[sb];
            x.y = (uint32_t)(uint16_t)bs[0] | ((uint32_t)(uint16_t)bs[2] << 16);
            x.z = (uint32_t)(uint16_t)bs[4] | ((uint32_t)(uint16_t)bs[6] << 16);
        }
        return x;
    }
    static constexpr int UNITS_PER_SB = 4;
    __device__ static __forceinline__ size_t img_qs(int, int e) {
        const int sb = e >> 8, o = e & 255;
        const int h = o >> 7, v = (o >> 5) & 3, ip = (o >> 4) & 1, w = o & 15;
        const int u = sb * 4 + 2 * h + ip;
        return ((size_t)((u >> 6) * QCH + v) * 64 + (u & 63)) * 16 + w;
    }
    __device__ static __forceinline__ uint8_t *img_aux(uint8_t *img, int NI, int u) { return img + (size_t)NI * QCH * 1024 + (size_t)u * AUX; }
    // called by all 64 lanes with the sum of their 16-value group g = lane/4 = 8*h + 2*v + ip: unit 2*h + ip, slot v
    __device__ static __forceinline__ void img_bsum(uint8_t *img, int NI, int sb, int lane, int s16) {
        if ((lane & 3) == 0) {
            const int g = lane >> 2;
            const int u = sb * 4 + 2 * (g >> 3) + (g & 1);
            reinterpret_cast<int16_t *>(img_aux(img, NI, u) + 4)[(g >> 1) & 3] = (int16_t)s16;
        }
    }
};

// Q6_K rows re-laid in planes: a row of nsb super-blocks is ql[nsb][128] | qh[nsb][64] | scales[nsb][16] | d[nsb] - the same
// bytes, same total (210 nsb), every field of every super-block at the alignment of its loads (nsb even: the planes start at
// multiples of 16 bytes).  block_q6_K's 210 bytes leave only every eighth super-block 16-byte aligned, and the misaligned
// 16-byte loads cost the one-token GEMV of a 48 MB matrix about 1.5 us of 14.5 (measured with the block bases rounded down to
// 16 bytes: 1.36 -> 1.28 ms for the whole 32-layer trace step).  Everything after the loads - decode, dots, activation side -
// is Q6_K's, so the results have its bits.
template <> struct Traits<T_Q6_K_P> : Traits<T_Q6_K> {
    __device__ static __forceinline__ void load_raw_planes(Raw &r, const uint8_t *row, int u, int nsb) {
        const int sb = u >> 2, h = (u >> 1) & 1, ip = u & 1;
        const uint8_t *ql = row + (size_t)sb * 128 + 64 * h + 16 * ip;
        r.l0 = WLOAD(reinterpret_cast<const u32x4 *>(ql));
        r.l1 = WLOAD(reinterpret_cast<const u32x4 *>(ql + 32));
        r.qh = WLOAD(reinterpret_cast<const u32x4 *>(row + (size_t)nsb * 128 + (size_t)sb * 64 + 32 * h + 16 * ip));
        r.s  = WLOAD(reinterpret_cast<const u32x2 *>(row + (size_t)nsb * 192 + (size_t)sb * 16 + 8 * h));
        r.d  = WLOAD(reinterpret_cast<const unsigned short *>(row + (size_t)nsb * 208 + (size_t)sb * 2));
    }
};

// ---- the 3- and 2-bit K-quants (reference type_traits_cpu[], ggml-cpu/ggml-cpu.c:257-268; lm_ggml_vec_dot_q3_K_q8_K and
// lm_ggml_vec_dot_q2_K_q8_K, ggml-cpu/ggml-cpu-quants.c:5521 ff. / 4506 ff.; dequantize_row_q3_K / _q2_K, ggml-quants.c:1050 / 706).
// Their 64 bytes of qs hold element 128 h + 32 v + l (l < 32) in bits 2 v of byte 32 h + l, and sub-block 8 h + 2 v + (l >= 16)
// carries the scale: the unit (sb, h, ip) of Q6_K - the 16 bytes 32 h + 16 ip ... of qs, four 16-value groups v with scales
// 8 h + 2 v + ip - fits both, so the activation side (image layout, block sums of 16, staging) is Q6_K's unchanged.
template <> struct Traits<T_Q3_K> : Traits<T_Q6_K> {
    // block_q3_K (ggml-common.h:273-278): hmask[32] | qs[64] | scales[12] | fp16 d, 110 bytes, 2-byte aligned.
    // value = d * (scale - 32) * (q - 4), q = the two bits of qs plus 4 where the bit 4 h + v of hmask[l] is set
    struct W { uint32_t q[16]; float d; int sc[4]; };            // q[4v + k]: values 0..7 of group v; the 4 comes off through the block sums
    // The 14 bytes behind qs (12 of packed scales, fp16 d) belong to all four lanes of a super-block: lane j of the quad fetches
    // one dword of them (bytes 96, 100, 104 and, for the fourth, 106: the last two scale bytes and d - no byte past the block)
    // and the quad hands them round by DPP: three load instructions per step instead of six (4096 x 14336 at one token
    // 12.2 -> 11.7 us, the other shapes within 2 %).
    struct Raw { u32x4 qs, hm; uint32_t tail; };
    __device__ static __forceinline__ void load_raw(Raw &r, const uint8_t *row, int u) {
        const int sb = u >> 2, h = (u >> 1) & 1, ip = u & 1, j = u & 3;
        const uint8_t *p = row + (size_t)sb * BYTES_Q3_K;
        r.qs = WLOAD(reinterpret_cast<const u32x4_a2 *>(p + 32 + 32 * h + 16 * ip));
        r.hm = WLOAD(reinterpret_cast<const u32x4_a2 *>(p + 16 * ip));
        r.tail = WLOAD(reinterpret_cast<const u32_a2 *>(p + 96 + (j < 3 ? 4 * j : 10)));
    }
    __device__ static __forceinline__ void decode(W &w, const Raw &rr, int u) {
        struct { u32x4 qs, hm; uint32_t s0, s1, s2, d; } r;
        r.qs = rr.qs; r.hm = rr.hm;
        r.s0 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)rr.tail, 0x00, 0xf, 0xf, false);
        r.s1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)rr.tail, 0x55, 0xf, 0xf, false);
        r.s2 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)rr.tail, 0xAA, 0xf, 0xf, false);
        r.d = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)rr.tail, 0xFF, 0xf, 0xf, false) >> 16;
        const int h = (u >> 1) & 1, ip = u & 1;
        w.d = h2f(r.d);
        const uint32_t lo[4] = {r.qs.x, r.qs.y, r.qs.z, r.qs.w}, hm[4] = {r.hm.x, r.hm.y, r.hm.z, r.hm.w};
#pragma unroll
        for (int v = 0; v < 4; v++)
#pragma unroll
            for (int k = 0; k < 4; k++)
                w.q[4 * v + k] = ((lo[k] >> (2 * v)) & 0x03030303u) | (((hm[k] >> (4 * h + v)) & 0x01010101u) << 2);
        // the sixteen 6-bit scales (ggml-quants.c:1062-1071): scale 4 w + i is byte i of word w below; this unit wants
        // 8 h + 2 v + ip, i.e. bytes ip and 2 + ip of words 2 h and 2 h + 1
        const uint32_t hi2 = r.s2 >> (4 * h);
        const uint32_t wa = ((r.s0 >> (4 * h)) & 0x0f0f0f0fu) | ((hi2 & 0x03030303u) << 4);
        const uint32_t wb = ((r.s1 >> (4 * h)) & 0x0f0f0f0fu) | (((hi2 >> 2) & 0x03030303u) << 4);
        const int b = 8 * ip;
        w.sc[0] = (int)((wa >> b) & 0xffu) - 32; w.sc[1] = (int)((wa >> (b + 16)) & 0xffu) - 32;
        w.sc[2] = (int)((wb >> b) & 0xffu) - 32; w.sc[3] = (int)((wb >> (b + 16)) & 0xffu) - 32;
    }
    __device__ static __forceinline__ void isums(const W &w, const A &a, int &is, int &unused) {
        is = 0; unused = 0;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            int dv = -4 * a.bs[v];                                      // sum (q-4)*a = sum q*a - 4*sum a
#pragma unroll
            for (int k = 0; k < 4; k++) dv = dot4(w.q[4 * v + k], a.q[4 * v + k], dv);
            is += w.sc[v] * dv;
        }
    }
    __device__ static __forceinline__ float dot(const W &w, const A &a, float acc) {
        int is, unused;
        isums(w, a, is, unused);
        return __builtin_fmaf(w.d * a.d, (float)is, acc);
    }
};

template <> struct Traits<T_Q2_K> : Traits<T_Q6_K> {
    // block_q2_K (ggml-common.h:254-266): scales[16] (scale in the low, min in the high nibble) | qs[64] | fp16 d | fp16 dmin,
    // 84 bytes, 4-byte aligned.  value = d * sc * q - dmin * m, q = the two bits of qs
    struct W { uint32_t q[16]; float d, dmin; int sc[4], m[4]; };
    struct Raw { u32x4 qs; uint32_t s0, s1, dd; };
    __device__ static __forceinline__ void load_raw(Raw &r, const uint8_t *row, int u) {
        const int sb = u >> 2, h = (u >> 1) & 1, ip = u & 1;
        const uint8_t *p = row + (size_t)sb * BYTES_Q2_K;
        r.qs = WLOAD(reinterpret_cast<const u32x4_a4 *>(p + 16 + 32 * h + 16 * ip));
        r.s0 = WLOAD(reinterpret_cast<const uint32_t *>(p + 8 * h));
        r.s1 = WLOAD(reinterpret_cast<const uint32_t *>(p + 8 * h + 4));
        r.dd = WLOAD(reinterpret_cast<const uint32_t *>(p + 80));
    }
    __device__ static __forceinline__ void decode(W &w, const Raw &r, int u) {
        const int ip = u & 1;
        w.d = h2f(r.dd); w.dmin = h2f(r.dd >> 16);
        const uint32_t lo[4] = {r.qs.x, r.qs.y, r.qs.z, r.qs.w};
#pragma unroll
        for (int v = 0; v < 4; v++)
#pragma unroll
            for (int k = 0; k < 4; k++) w.q[4 * v + k] = (lo[k] >> (2 * v)) & 0x03030303u;
        const int b = 8 * ip;                                           // scales[8h + 2v + ip]: bytes ip and 2 + ip of the two words
        const uint32_t c0 = r.s0 >> b, c1 = r.s0 >> (b + 16), c2 = r.s1 >> b, c3 = r.s1 >> (b + 16);
        w.sc[0] = (int)(c0 & 15u); w.m[0] = (int)((c0 >> 4) & 15u); w.sc[1] = (int)(c1 & 15u); w.m[1] = (int)((c1 >> 4) & 15u);
        w.sc[2] = (int)(c2 & 15u); w.m[2] = (int)((c2 >> 4) & 15u); w.sc[3] = (int)(c3 & 15u); w.m[3] = (int)((c3 >> 4) & 15u);
    }
    __device__ static __forceinline__ void isums(const W &w, const A &a, int &is, int &im) {
        is = 0; im = 0;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            int dv = 0;
#pragma unroll
            for (int k = 0; k < 4; k++) dv = dot4(w.q[4 * v + k], a.q[4 * v + k], dv);
            is += w.sc[v] * dv;
            im += w.m[v] * a.bs[v];
        }
    }
    __device__ static __forceinline__ float dot(const W &w, const A &a, float acc) {
        int is, im;
        isums(w, a, is, im);
        acc = __builtin_fmaf(w.d * a.d, (float)is, acc);
        return __builtin_fmaf(-(w.dmin * a.d), (float)im, acc);
    }
};

// ---- further weight types (reference type_traits_cpu[], ggml-cpu/ggml-cpu.c:198-367): same activation formats
template <> struct Traits<T_Q5_0> {
    // block_q5_0 (ggml-common.h:187-193): fp16 d, 32 high bits qh, 16 nibble bytes; value = d * (q5 - 16),
    // q5 = nibble | bit << 4, bit j of qh for element j (low nibbles), bit j + 16 for element j + 16 (high nibbles)
    static constexpr int ACT = T_Q8_0, UNIT_ELEMS = 64, QCH = 4, AUX = 16;
    static constexpr bool A_HAS_SUMS = true;
    struct W { uint32_t lo[8], hi[8]; float d0, d1; };          // 5-bit values spread to bytes, 0..31
    struct A { uint32_t q[16]; float d0, d1; int s0, s1; };
    struct Raw { u32x4 a, b; u32x2 c; uint32_t e; };
    __device__ static __forceinline__ void load_raw(Raw &r, const uint8_t *row, int u) {
        const uint8_t *p = row + (size_t)u * 44;                       // two 22-byte blocks, 4-byte aligned
        r.a = WLOAD(reinterpret_cast<const u32x4_a4 *>(p));
        r.b = WLOAD(reinterpret_cast<const u32x4_a4 *>(p + 16));
        r.c = WLOAD(reinterpret_cast<const u32x2_a4 *>(p + 32));
        r.e = WLOAD(reinterpret_cast<const uint32_t *>(p + 40));
    }
    // four high bits -> bit 4 of four bytes
    __device__ static __forceinline__ uint32_t spread4(uint32_t bits) { return (((bits & 0xFu) * 0x00204081u) & 0x01010101u) << 4; }
    __device__ static __forceinline__ void decode(W &w, const Raw &r, int) {
        const uint32_t d[11] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w, r.c.x, r.c.y, r.e};
        // block 0: d at bytes 0..1, qh at 2..5, qs at 6..21; block 1: d at 22..23, qh at 24..27, qs at 28..43
        w.d0 = h2f(d[0]);
        w.d1 = h2f(d[5] >> 16);
        const uint32_t qh0 = shr16(d[1], d[0]), qh1 = d[6];
        const uint32_t q0[4] = {shr16(d[2], d[1]), shr16(d[3], d[2]), shr16(d[4], d[3]), shr16(d[5], d[4])};
        const uint32_t q1[4] = {d[7], d[8], d[9], d[10]};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w.lo[i]     = (q0[i] & 0x0f0f0f0fu)        | spread4(qh0 >> (4 * i));
            w.hi[i]     = ((q0[i] >> 4) & 0x0f0f0f0fu) | spread4(qh0 >> (16 + 4 * i));
            w.lo[4 + i] = (q1[i] & 0x0f0f0f0fu)        | spread4(qh1 >> (4 * i));
            w.hi[4 + i] = ((q1[i] >> 4) & 0x0f0f0f0fu) | spread4(qh1 >> (16 + 4 * i));
        }
    }
    __device__ static __forceinline__ void load_a(A &a, const uint8_t *tok, int NI, int it, int lane) {
        const u32x4 *q = reinterpret_cast<const u32x4 *>(tok) + (size_t)it * QCH * 64 + lane;
#pragma unroll
        for (int j = 0; j < QCH; j++) {
            const u32x4 v = q[j * 64];
            a.q[4 * j] = v.x; a.q[4 * j + 1] = v.y; a.q[4 * j + 2] = v.z; a.q[4 * j + 3] = v.w;
        }
        const u32x4 x = reinterpret_cast<const u32x4 *>(tok + (size_t)NI * QCH * 1024)[it * 64 + lane];
        a.d0 = __uint_as_float(x.x); a.d1 = __uint_as_float(x.y); a.s0 = (int)x.z; a.s1 = (int)x.w;
    }
    __device__ static __forceinline__ void isums(const W &w, const A &a, int &i0, int &i1) {
        i0 = -16 * a.s0; i1 = -16 * a.s1;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            i0 = dot4(w.lo[i], a.q[i], i0);         i0 = dot4(w.hi[i], a.q[4 + i], i0);
            i1 = dot4(w.lo[4 + i], a.q[8 + i], i1); i1 = dot4(w.hi[4 + i], a.q[12 + i], i1);
        }
    }
    __device__ static __forceinline__ float dot(const W &w, const A &a, float acc) {
        int i0, i1;
        isums(w, a, i0, i1);
        acc = __builtin_fmaf(w.d0 * a.d0, (float)i0, acc);
        return __builtin_fmaf(w.d1 * a.d1, (float)i1, acc);
    }
    __device__ static __forceinline__ size_t src_chunk(int64_t, int u, int j) { return (size_t)u * 64 + 16 * j; }
    using AuxT = u32x4;
    __device__ static __forceinline__ AuxT aux_load(const uint8_t *ws, int64_t K, int u, bool valid) { return Traits<T_Q4_0>::aux_load(ws, K, u, valid); }
    __device__ static __forceinline__ size_t img_qs(int NI, int e) { return Traits<T_Q4_0>::img_qs(NI, e); }
    __device__ static __forceinline__ void img_block_aux(uint8_t *img, int NI, int blk, float d, int sum, float s) { Traits<T_Q4_0>::img_block_aux(img, NI, blk, d, sum, s); }
};

template <> struct Traits<T_IQ4_NL> {
    // block_iq4_nl (ggml-common.h:405-410): fp16 d, 16 nibble bytes; value = d * codebook[nibble]
    // (ggml-quants.c:2428), low nibbles are elements 0..15, high nibbles 16..31
    static constexpr int ACT = T_Q8_0, UNIT_ELEMS = 64, QCH = 4, AUX = 8;
    static constexpr bool A_HAS_SUMS = false;
    struct W { uint32_t q[16]; float d0, d1; };                 // signed code points, element order
    using A = Traits<T_Q8_0>::A;
    using Raw = Traits<T_Q4_0>::Raw;
    __device__ static __forceinline__ void load_raw(Raw &r, const uint8_t *row, int u) { Traits<T_Q4_0>::load_raw(r, row, u); }
    // four code indices (one per byte, 0..15) -> four code points, through two byte permutes of the 16-entry table
    __device__ static __forceinline__ uint32_t lookup4(uint32_t idx) {
        constexpr uint32_t T0 = 0xbfad9881u, T1 = 0xf6eaddcfu, T2 = 0x26190d01u, T3 = 0x71594535u;
        const uint32_t sel = idx & 0x07070707u;
        const uint32_t lo = __builtin_amdgcn_perm(T1, T0, sel), hi = __builtin_amdgcn_perm(T3, T2, sel);
        const uint32_t m = ((idx >> 3) & 0x01010101u) * 0xffu;
        return (lo & ~m) | (hi & m);
    }
    __device__ static __forceinline__ void decode(W &w, const Raw &r, int) {
        const u32x4 a = r.a, b = r.b;
        const uint32_t c = r.c;
        uint32_t q[8];
        w.d0 = h2f(a.x);
        q[0] = shr16(a.y, a.x); q[1] = shr16(a.z, a.y); q[2] = shr16(a.w, a.z); q[3] = shr16(b.x, a.w);
        w.d1 = h2f(b.x >> 16);
        q[4] = b.y; q[5] = b.z; q[6] = b.w; q[7] = c;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w.q[i]      = lookup4(q[i] & 0x0f0f0f0fu);        w.q[4 + i]  = lookup4((q[i] >> 4) & 0x0f0f0f0fu);
            w.q[8 + i]  = lookup4(q[4 + i] & 0x0f0f0f0fu);    w.q[12 + i] = lookup4((q[4 + i] >> 4) & 0x0f0f0f0fu);
        }
    }
    __device__ static __forceinline__ void load_a(A &a, const uint8_t *tok, int NI, int it, int lane) { Traits<T_Q8_0>::load_a(a, tok, NI, it, lane); }
    __device__ static __forceinline__ void isums(const W &w, const A &a, int &i0, int &i1) {
        i0 = 0; i1 = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) { i0 = dot4(w.q[i], a.q[i], i0); i1 = dot4(w.q[8 + i], a.q[8 + i], i1); }
    }
    __device__ static __forceinline__ float dot(const W &w, const A &a, float acc) {
        int i0, i1;
        isums(w, a, i0, i1);
        acc = __builtin_fmaf(w.d0 * a.d0, (float)i0, acc);
        return __builtin_fmaf(w.d1 * a.d1, (float)i1, acc);
    }
    __device__ static __forceinline__ size_t src_chunk(int64_t, int u, int j) { return (size_t)u * 64 + 16 * j; }
    using AuxT = float2;
    __device__ static __forceinline__ AuxT aux_load(const uint8_t *ws, int64_t K, int u, bool valid) { return Traits<T_Q8_0>::aux_load(ws, K, u, valid); }
    __device__ static __forceinline__ size_t img_qs(int NI, int e) { return Traits<T_Q8_0>::img_qs(NI, e); }
    __device__ static __forceinline__ void img_block_aux(uint8_t *img, int NI, int blk, float d, int sum, float s) { Traits<T_Q8_0>::img_block_aux(img, NI, blk, d, sum, s); }
};

// F16 weights (type_traits_cpu[LM_GGML_TYPE_F16], ggml-cpu/ggml-cpu.c:204-209): the activations are rounded to fp16
// (lm_ggml_cpu_fp32_to_fp16) and lm_ggml_vec_dot_f16 (ggml-cpu/vec.cpp:122-162) accumulates the products of the
// widened halves in fp32.  A unit is 32 elements = 64 weight bytes and 64 activation bytes; no side data.
template <> struct Traits<T_F16> {
    static constexpr int ACT = T_F16, UNIT_ELEMS = 32, QCH = 4, AUX = 0;
    struct Raw { u32x4 q[4]; };
    using W = Raw;
    struct A { uint32_t q[16]; };
    __device__ static __forceinline__ void load_raw(Raw &r, const uint8_t *row, int u) {
        const u32x4 *p = reinterpret_cast<const u32x4 *>(row + (size_t)u * 64);  // rows are multiples of 512 bytes
#pragma unroll
        for (int j = 0; j < 4; j++) r.q[j] = WLOAD(p + j);
    }
    __device__ static __forceinline__ void decode(W &w, const Raw &r, int) { w = r; }
    __device__ static __forceinline__ void load_a(A &a, const uint8_t *tok, int, int it, int lane) {
        const u32x4 *q = reinterpret_cast<const u32x4 *>(tok) + (size_t)it * QCH * 64 + lane;
#pragma unroll
        for (int j = 0; j < QCH; j++) {
            const u32x4 v = q[j * 64];
            a.q[4 * j] = v.x; a.q[4 * j + 1] = v.y; a.q[4 * j + 2] = v.z; a.q[4 * j + 3] = v.w;
        }
    }
    __device__ static __forceinline__ float dot(const W &w, const A &a, float acc) {
        typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t wq[4] = {w.q[j].x, w.q[j].y, w.q[j].z, w.q[j].w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const half2_t wv = __builtin_bit_cast(half2_t, wq[i]), av = __builtin_bit_cast(half2_t, a.q[4 * j + i]);
                acc = __builtin_fmaf((float)wv.x, (float)av.x, acc);      // v_fma_mix_f32: fp16 operands, fp32 accumulate
                acc = __builtin_fmaf((float)wv.y, (float)av.y, acc);
            }
        }
        return acc;
    }
    __device__ static __forceinline__ size_t src_chunk(int64_t, int u, int j) { return (size_t)u * 64 + 16 * j; }
    using AuxT = uint32_t;                                       // unused (AUX == 0)
    __device__ static __forceinline__ AuxT aux_load(const uint8_t *, int64_t, int, bool) { return 0u; }
    // fused prologue: byte position of element e (an fp16) in the LDS image
    __device__ static __forceinline__ size_t img_h(int, int e) {
        const int u = e >> 5, off = (e & 31) * 2;
        return ((size_t)((u >> 6) * QCH + (off >> 4)) * 64 + (u & 63)) * 16 + (off & 15);
    }
};

// Q4_1 / Q5_1 (ggml-common.h:175-185,196-207): value = d * u + m with an unsigned 4- or 5-bit u.  Their activation
// format Q8_1 is Q8_0 plus s = fp16(d * sum q) per block (kept in the Q8_0 workspace planes), so
// y += (dw * dx) * sum(u * q) + m * s (reference lm_ggml_vec_dot_q4_1_q8_1 / _q5_1_q8_1, AVX2 branches).
template <int WT> struct TraitsMin32 {
    static constexpr bool FIVE = (WT == T_Q5_1);
    static constexpr int ACT = T_Q8_0, UNIT_ELEMS = 64, QCH = 4, AUX = 16;
    static constexpr bool A_HAS_SUMS = false;
    static constexpr int ABLK_BYTES = BYTES_Q8_1, ABLK_QOFF = 4;          // reference activation records (block_isums)
    struct W { uint32_t lo[8], hi[8]; float d0, d1, m0, m1; };
    struct A { uint32_t q[16]; float d0, d1, s0, s1; };
    struct Raw { u32x4 a, b; u32x2 c; uint32_t e[2]; };
    __device__ static __forceinline__ void load_raw(Raw &r, const uint8_t *row, int u) {
        if constexpr (!FIVE) {
            const uint8_t *p = row + (size_t)u * 40;                   // two 20-byte blocks, 4-byte aligned
            r.a = WLOAD(reinterpret_cast<const u32x4_a4 *>(p));
            r.b = WLOAD(reinterpret_cast<const u32x4_a4 *>(p + 16));
            r.c = WLOAD(reinterpret_cast<const u32x2_a4 *>(p + 32));
        } else {
            const uint8_t *p = row + (size_t)u * 48;                   // two 24-byte blocks, 4-byte aligned
            r.a = WLOAD(reinterpret_cast<const u32x4_a4 *>(p));
            r.b = WLOAD(reinterpret_cast<const u32x4_a4 *>(p + 16));
            r.c = WLOAD(reinterpret_cast<const u32x2_a4 *>(p + 32));
            r.e[0] = WLOAD(reinterpret_cast<const uint32_t *>(p + 40));
            r.e[1] = WLOAD(reinterpret_cast<const uint32_t *>(p + 44));
        }
    }
    __device__ static __forceinline__ uint32_t spread4(uint32_t bits) { return (((bits & 0xFu) * 0x00204081u) & 0x01010101u) << 4; }
    __device__ static __forceinline__ void decode(W &w, const Raw &r, int) {
        if constexpr (!FIVE) {
            // block: d, m (one dword), 16 qs bytes
            const uint32_t d[10] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w, r.c.x, r.c.y};
            w.d0 = h2f(d[0]); w.m0 = h2f(d[0] >> 16);
            w.d1 = h2f(d[5]); w.m1 = h2f(d[5] >> 16);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                w.lo[i]     = d[1 + i] & 0x0f0f0f0fu; w.hi[i]     = (d[1 + i] >> 4) & 0x0f0f0f0fu;
                w.lo[4 + i] = d[6 + i] & 0x0f0f0f0fu; w.hi[4 + i] = (d[6 + i] >> 4) & 0x0f0f0f0fu;
            }
        } else {
            // block: d, m (one dword), qh (one dword), 16 qs bytes
            const uint32_t d[12] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w, r.c.x, r.c.y, r.e[0], r.e[1]};
            w.d0 = h2f(d[0]); w.m0 = h2f(d[0] >> 16);
            w.d1 = h2f(d[6]); w.m1 = h2f(d[6] >> 16);
            const uint32_t qh0 = d[1], qh1 = d[7];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                w.lo[i]     = (d[2 + i] & 0x0f0f0f0fu)        | spread4(qh0 >> (4 * i));
                w.hi[i]     = ((d[2 + i] >> 4) & 0x0f0f0f0fu) | spread4(qh0 >> (16 + 4 * i));
                w.lo[4 + i] = (d[8 + i] & 0x0f0f0f0fu)        | spread4(qh1 >> (4 * i));
                w.hi[4 + i] = ((d[8 + i] >> 4) & 0x0f0f0f0fu) | spread4(qh1 >> (16 + 4 * i));
            }
        }
    }
    __device__ static __forceinline__ void load_a(A &a, const uint8_t *tok, int NI, int it, int lane) {
        const u32x4 *q = reinterpret_cast<const u32x4 *>(tok) + (size_t)it * QCH * 64 + lane;
#pragma unroll
        for (int j = 0; j < QCH; j++) {
            const u32x4 v = q[j * 64];
            a.q[4 * j] = v.x; a.q[4 * j + 1] = v.y; a.q[4 * j + 2] = v.z; a.q[4 * j + 3] = v.w;
        }
        const float4 x = reinterpret_cast<const float4 *>(tok + (size_t)NI * QCH * 1024)[it * 64 + lane];
        a.d0 = x.x; a.d1 = x.y; a.s0 = x.z; a.s1 = x.w;
    }
    __device__ static __forceinline__ void isums(const W &w, const A &a, int &i0, int &i1) {
        i0 = 0; i1 = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            i0 = dot4(w.lo[i], a.q[i], i0);         i0 = dot4(w.hi[i], a.q[4 + i], i0);
            i1 = dot4(w.lo[4 + i], a.q[8 + i], i1); i1 = dot4(w.hi[4 + i], a.q[12 + i], i1);
        }
    }
    __device__ static __forceinline__ float dot(const W &w, const A &a, float acc) {
        int i0, i1;
        isums(w, a, i0, i1);
        acc = __builtin_fmaf(w.d0 * a.d0, (float)i0, acc);
        acc = __builtin_fmaf(w.m0, a.s0, acc);
        acc = __builtin_fmaf(w.d1 * a.d1, (float)i1, acc);
        return __builtin_fmaf(w.m1, a.s1, acc);
    }
    __device__ static __forceinline__ size_t src_chunk(int64_t, int u, int j) { return (size_t)u * 64 + 16 * j; }
    using AuxT = float4;
    __device__ static __forceinline__ AuxT aux_load(const uint8_t *ws, int64_t K, int u, bool valid) {
        float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
        if (valid) {
            const float2 d = reinterpret_cast<const float2 *>(ws + q8_0_off_d(K))[u];
            const float2 s = reinterpret_cast<const float2 *>(ws + q8_0_off_s(K))[u];
            x = make_float4(d.x, d.y, s.x, s.y);
        }
        return x;
    }
    __device__ static __forceinline__ size_t img_qs(int NI, int e) { return Traits<T_Q4_0>::img_qs(NI, e); }
    __device__ static __forceinline__ void img_block_aux(uint8_t *img, int NI, int blk, float d, int, float s) {
        float *a = reinterpret_cast<float *>(img + (size_t)NI * QCH * 1024 + (size_t)(blk >> 1) * AUX);
        a[blk & 1] = d;
        a[2 + (blk & 1)] = s;
    }
};
template <> struct Traits<T_Q4_1> : TraitsMin32<T_Q4_1> {};
template <> struct Traits<T_Q5_1> : TraitsMin32<T_Q5_1> {};

template <> struct Traits<T_Q5_K> {
    // block_q5_K (ggml-common.h:303-314): as q4_K plus qh[32]: bit 2jp of qh[l] is the fifth bit of element l of
    // sub-block 2jp (low nibbles of the group's 32 qs bytes), bit 2jp+1 that of sub-block 2jp+1 (high nibbles)
    static constexpr int ACT = T_Q8_K, UNIT_ELEMS = 64, QCH = 4, AUX = 8;
    static constexpr int KQ_STYLE = 0;
    using W = Traits<T_Q4_K>::W;
    using A = Traits<T_Q4_K>::A;
    // The four lanes of a super-block share its header and its 32 qh bytes: lane jp fetches the jp-th 16 bytes of those 48
    // (lane 3 the third again) and the quad hands them round by DPP - three load instructions per step instead of five
    // (14336 x 4096 at one token 10.96 -> 9.85 us; other shapes and 4 tokens within 2 %).  A row has a multiple of four units,
    // so the lanes of a quad are in the row, and decoded, together.
    struct Raw { u32x4 piece, q0, q1; };
    __device__ static __forceinline__ void load_raw(Raw &r, const uint8_t *row, int u) {
        const int sb = u >> 2, jp = u & 3;
        const uint8_t *p = row + (size_t)sb * BYTES_Q5_K;
        r.piece = WLOAD(reinterpret_cast<const u32x4 *>(p + 16 * (jp < 2 ? jp : 2)));
        r.q0 = WLOAD(reinterpret_cast<const u32x4 *>(p + 48 + 32 * jp));
        r.q1 = WLOAD(reinterpret_cast<const u32x4 *>(p + 64 + 32 * jp));
    }
    template <int CTRL> __device__ static __forceinline__ u32x4 quad_from(const u32x4 v) {
        u32x4 o;
        o.x = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.x, CTRL, 0xf, 0xf, false);
        o.y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.y, CTRL, 0xf, 0xf, false);
        o.z = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.z, CTRL, 0xf, 0xf, false);
        o.w = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.w, CTRL, 0xf, 0xf, false);
        return o;
    }
    __device__ static __forceinline__ void decode(W &w, const Raw &rr, int u) {
        struct { u32x4 h, qh0, qh1, q0, q1; } r;
        r.h = quad_from<0x00>(rr.piece);                                // quad_perm [0,0,0,0]
        r.qh0 = quad_from<0x55>(rr.piece);                              // [1,1,1,1]
        r.qh1 = quad_from<0xAA>(rr.piece);                              // [2,2,2,2]
        r.q0 = rr.q0; r.q1 = rr.q1;
        const int jp = u & 3;
        const u32x4 h = r.h;
        w.d = h2f(h.x); w.dmin = h2f(h.x >> 16);
        const int sh = 16 * (jp & 1);
        const uint32_t a1 = h.y >> sh, a2 = h.z >> sh, a3 = h.w >> sh;
        uint32_t sc, mn;
        if (jp < 2) { sc = a1 & 0x3f3fu; mn = a2 & 0x3f3fu; }
        else        { sc = (a3 & 0x0f0fu) | ((a1 >> 2) & 0x3030u); mn = ((a3 >> 4) & 0x0f0fu) | ((a2 >> 2) & 0x3030u); }
        w.sc0 = sc & 0xff; w.sc1 = sc >> 8; w.m0 = mn & 0xff; w.m1 = mn >> 8;
        const uint32_t q[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
        const uint32_t hb[8] = {r.qh0.x, r.qh0.y, r.qh0.z, r.qh0.w, r.qh1.x, r.qh1.y, r.qh1.z, r.qh1.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            w.lo[i] = (q[i] & 0x0f0f0f0fu)        | (((hb[i] >> (2 * jp)) & 0x01010101u) << 4);
            w.hi[i] = ((q[i] >> 4) & 0x0f0f0f0fu) | (((hb[i] >> (2 * jp + 1)) & 0x01010101u) << 4);
        }
    }
    __device__ static __forceinline__ void load_a(A &a, const uint8_t *tok, int NI, int it, int lane) { Traits<T_Q4_K>::load_a(a, tok, NI, it, lane); }
    __device__ static __forceinline__ void isums(const W &w, const A &a, int &is, int &im) { Traits<T_Q4_K>::isums(w, a, is, im); }
    __device__ static __forceinline__ float dot(const W &w, const A &a, float acc) { return Traits<T_Q4_K>::dot(w, a, acc); }
    __device__ static __forceinline__ size_t src_chunk(int64_t K, int u, int j) { return Traits<T_Q4_K>::src_chunk(K, u, j); }
    using AuxT = u32x2;
    __device__ static __forceinline__ AuxT aux_load(const uint8_t *ws, int64_t K, int u, bool valid) { return Traits<T_Q4_K>::aux_load(ws, K, u, valid); }
    static constexpr int UNITS_PER_SB = 4;
    __device__ static __forceinline__ size_t img_qs(int NI, int e) { return Traits<T_Q4_K>::img_qs(NI, e); }
    __device__ static __forceinline__ uint8_t *img_aux(uint8_t *img, int NI, int u) { return Traits<T_Q4_K>::img_aux(img, NI, u); }
    __device__ static __forceinline__ void img_bsum(uint8_t *img, int NI, int sb, int lane, int s16) { Traits<T_Q4_K>::img_bsum(img, NI, sb, lane, s16); }
};

template <int WT> __host__ __device__ constexpr int units_per_row(int64_t K) { return (int)(K / Traits<WT>::UNIT_ELEMS); }
template <int WT> __host__ __device__ constexpr int iters_per_row(int64_t K) { return (int)ceil_div(K / Traits<WT>::UNIT_ELEMS, 64); }
template <int WT> __host__ __device__ constexpr size_t lds_image_bytes(int64_t K) {
    return (size_t)iters_per_row<WT>(K) * (Traits<WT>::QCH * 1024 + 64 * Traits<WT>::AUX);
}

// IQ4_XS (reference type_traits_cpu[], ggml-cpu/ggml-cpu.c:340-345; lm_ggml_vec_dot_iq4_xs_q8_K, ggml-cpu/ggml-cpu-quants.c:12965 ff.;
// dequantize_row_iq4_xs, ggml-quants.c): IQ4_NL's code points in 256-value super-blocks with a 6-bit scale (biased by 32) per
// 32-value sub-block and Q8_K activations.  block_iq4_xs (ggml-common.h:412-417): fp16 d | u16 scales_h | scales_l[4] | qs[128],
// 136 bytes, 8-byte aligned.  Sub-block ib is the 16 bytes qs[16 ib ...]: low nibbles elements 0..15, high nibbles 16..31.
// Q4_K's unit (super-block, 64-value group jp = sub-blocks 2 jp and 2 jp + 1, 64 consecutive activation quants) carries it.
template <> struct Traits<T_IQ4_XS> : Traits<T_Q4_K> {
    struct W { uint32_t q[16]; float d; int ls0, ls1; };          // signed code points in element order
    struct Raw { u32x2 h; u32x4 q0, q1; };
    __device__ static __forceinline__ void load_raw(Raw &r, const uint8_t *row, int u) {
        const int sb = u >> 2, jp = u & 3;
        const uint8_t *p = row + (size_t)sb * BYTES_IQ4_XS;
        r.h = WLOAD(reinterpret_cast<const u32x2 *>(p));
        r.q0 = WLOAD(reinterpret_cast<const u32x4_a4 *>(p + 8 + 32 * jp));
        r.q1 = WLOAD(reinterpret_cast<const u32x4_a4 *>(p + 24 + 32 * jp));
    }
    __device__ static __forceinline__ void decode(W &w, const Raw &r, int u) {
        const int jp = u & 3;
        w.d = h2f(r.h.x);
        const uint32_t sh = (r.h.x >> 16) >> (4 * jp), sl = (r.h.y >> (8 * jp)) & 0xffu;   // scales_h bits of 2jp, 2jp+1; scales_l[jp]
        w.ls0 = (int)((sl & 0xfu) | ((sh & 3u) << 4)) - 32;
        w.ls1 = (int)((sl >> 4) | (((sh >> 2) & 3u) << 4)) - 32;
        const uint32_t a[4] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w}, b[4] = {r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w.q[i]      = Traits<T_IQ4_NL>::lookup4(a[i] & 0x0f0f0f0fu);   w.q[4 + i]  = Traits<T_IQ4_NL>::lookup4((a[i] >> 4) & 0x0f0f0f0fu);
            w.q[8 + i]  = Traits<T_IQ4_NL>::lookup4(b[i] & 0x0f0f0f0fu);   w.q[12 + i] = Traits<T_IQ4_NL>::lookup4((b[i] >> 4) & 0x0f0f0f0fu);
        }
    }
    __device__ static __forceinline__ void isums(const W &w, const A &a, int &is, int &unused) {
        int d0 = 0, d1 = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) { d0 = dot4(w.q[i], a.q[i], d0); d1 = dot4(w.q[8 + i], a.q[8 + i], d1); }
        is = w.ls0 * d0 + w.ls1 * d1;
        unused = 0;
    }
    __device__ static __forceinline__ float dot(const W &w, const A &a, float acc) {
        int is, unused;
        isums(w, a, is, unused);
        return __builtin_fmaf(w.d * a.d, (float)is, acc);
    }
};

// ------------------------------------------------------------------------------------------------ kernel
// Fused prologue: quantize NTOK fp32 rows straight into the LDS image; workgroup 0 also writes the split
// workspace planes so the quantized activations exist in memory as the reference's wdata does.
// The fp32 loads are split from their use (xload_* issues them, quantize_* consumes them) so that the caller
// can put the weight prefetch between the two: all of a thread's loads are then in flight together and the
// quantization waits only for the activations, which were issued first.
constexpr int FUSE_MAX_VALUES = 16384;                     // n * K limit of the fused prologue

// Register slots: token t owns slots [t*PER, (t+1)*PER); slot j of a token covers float4 chunk j*WGS + tid (Q8_0:
// 8 lanes per 32-block) or super-block j*(WGS/64) + wave (Q8_K: one wave per 256 values).  n * K <= FUSE_MAX_VALUES
// guarantees PER slots suffice; the loops stop at the first slot index that is out of range for the whole group.
constexpr int FUSE_ILP = 2;
template <int NTOK, int WGS, int MAXV = FUSE_MAX_VALUES> struct XRegs {      // MAXV: the n * K the registers are sized for
    static constexpr int PER = MAXV / 4 / WGS / NTOK > 0 ? MAXV / 4 / WGS / NTOK : 1;
    float4 v[NTOK][PER];
};

template <int WT, int NTOK, int WGS, int MAXV>
__device__ __forceinline__ void xload(XRegs<NTOK, WGS, MAXV> &xr, const float *__restrict__ x, int64_t ldx, int64_t K) {
    using T = Traits<WT>;
    constexpr int PER = XRegs<NTOK, WGS, MAXV>::PER;
    if constexpr (T::ACT == T_Q8_0 || T::ACT == T_F16) {
        const int nchunk = (int)(K / 4);                                // float4 chunks per token
#pragma unroll
        for (int t = 0; t < NTOK; t++)
#pragma unroll
            for (int j = 0; j < PER; j++) {
                const int c = j * WGS + (int)threadIdx.x;
                xr.v[t][j] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (c < nchunk) xr.v[t][j] = *reinterpret_cast<const float4 *>(x + t * ldx + 4 * (int64_t)c);
            }
    } else {
        const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
        const int nsb = (int)(K / 256);
#pragma unroll
        for (int t = 0; t < NTOK; t++)
#pragma unroll
            for (int j = 0; j < PER; j++) {
                const int sb = j * (WGS / 64) + wv;
                xr.v[t][j] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (sb < nsb) xr.v[t][j] = *reinterpret_cast<const float4 *>(x + t * ldx + (int64_t)sb * 256 + 4 * lane);
            }
    }
}

// slot_lo, slot_hi (Q8_K activations only): the register slots [slot_lo, slot_hi) of every token, i.e. super-blocks
// slot * (WGS / 64) .. - the caller may build the image a weight step's worth at a time.
template <int WT, int NTOK, int WGS, int MAXV>
__device__ __forceinline__ void quantize_into_image(const XRegs<NTOK, WGS, MAXV> &xr, uint8_t *lds, size_t img, int NI, int64_t K,
                                                    uint8_t *__restrict__ ws, size_t ws_stride, bool first_block,
                                                    int slot_lo = 0, int slot_hi = XRegs<NTOK, WGS, MAXV>::PER) {
    using T = Traits<WT>;
    constexpr int PER = XRegs<NTOK, WGS, MAXV>::PER;
    const bool dump = first_block && ws != nullptr;
    if constexpr (T::ACT == T_F16) {
        // plain conversion: four floats -> four halves (round to nearest even), 8 bytes into the image
        const int nchunk = (int)(K / 4);
#pragma unroll
        for (int t = 0; t < NTOK; t++) {
            uint8_t *im = lds + t * img;
#pragma unroll
            for (int j = 0; j < PER; j++) {
                const int c = j * WGS + (int)threadIdx.x;
                if (c < nchunk) {
                    const float4 v = xr.v[t][j];
                    u32x2 h;
                    h.x = (uint32_t)f2h_rne(v.x) | ((uint32_t)f2h_rne(v.y) << 16);
                    h.y = (uint32_t)f2h_rne(v.z) | ((uint32_t)f2h_rne(v.w) << 16);
                    *reinterpret_cast<u32x2 *>(im + T::img_h(NI, 4 * c)) = h;
                    if (dump) *reinterpret_cast<u32x2 *>(ws + t * ws_stride + 8 * (size_t)c) = h;
                }
            }
        }
    } else if constexpr (T::ACT == T_Q8_0) {
        // 8 lanes per 32-block; K % 64 == 0 keeps every group of 8 lanes either fully inside or fully outside the row
        // (every chunk index is tested against nchunk below).
        // Slots are quantized FUSE_ILP at a time so their dependent chains (DPP max, two divisions, DPP sum) overlap.
        const int nchunk = (int)(K / 4);
#pragma unroll
        for (int t = 0; t < NTOK; t++) {
            uint8_t *im = lds + t * img;
#pragma unroll
            for (int j0 = 0; j0 < PER; j0 += FUSE_ILP) {
                if (j0 * WGS >= nchunk) break;                          // uniform over the group
                Q8_0Lane q[FUSE_ILP];
#pragma unroll
                for (int u = 0; u < FUSE_ILP; u++)
                    if (j0 + u < PER) q[u] = quantize_q8_0_lane(xr.v[t][j0 + u]);
#pragma unroll
                for (int u = 0; u < FUSE_ILP; u++) {
                    if (j0 + u >= PER) continue;
                    const int c = (j0 + u) * WGS + (int)threadIdx.x;
                    if (c < nchunk) {
                        const int e = 4 * c, blk = e >> 5;
                        *reinterpret_cast<uint32_t *>(im + T::img_qs(NI, e)) = q[u].packed;
                        const float d = h2f(q[u].dh);
                        if ((threadIdx.x & 7) == 0) T::img_block_aux(im, NI, blk, d, q[u].sum, h2f(q[u].sh));
                        if (dump) {
                            uint8_t *base = ws + t * ws_stride;
                            *reinterpret_cast<uint32_t *>(base + e) = q[u].packed;
                            if ((threadIdx.x & 7) == 0) {
                                reinterpret_cast<float *>(base + q8_0_off_d(K))[blk] = d;
                                reinterpret_cast<int32_t *>(base + q8_0_off_sum(K))[blk] = q[u].sum;
                                reinterpret_cast<float *>(base + q8_0_off_s(K))[blk] = h2f(q[u].sh);
                            }
                        }
                    }
                }
            }
        }
    } else {
        // one wave per 256-value super-block, FUSE_ILP super-blocks in flight per wave
        const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
        const int nsb = (int)(K / 256);
#pragma unroll
        for (int t = 0; t < NTOK; t++) {
            uint8_t *im = lds + t * img;
#pragma unroll
            for (int j0 = 0; j0 < PER; j0 += FUSE_ILP) {
                if (j0 * (WGS / 64) >= nsb) break;                      // uniform over the group
                if (j0 + FUSE_ILP <= slot_lo || j0 >= slot_hi) continue;    // uniform: none of these slots is asked for
                Q8_KLane q[FUSE_ILP];
#pragma unroll
                for (int u = 0; u < FUSE_ILP; u++)
                    if (j0 + u < PER && j0 + u >= slot_lo && j0 + u < slot_hi) q[u] = quantize_q8_K_lane(xr.v[t][j0 + u]);
#pragma unroll
                for (int u = 0; u < FUSE_ILP; u++) {
                    if (j0 + u >= PER || j0 + u < slot_lo || j0 + u >= slot_hi) continue;
                    const int sb = (j0 + u) * (WGS / 64) + wv;
                    if (sb < nsb) {                                     // uniform over the wave
                        *reinterpret_cast<uint32_t *>(im + T::img_qs(NI, sb * 256 + 4 * lane)) = q[u].packed;
                        if (lane < T::UNITS_PER_SB) *reinterpret_cast<float *>(T::img_aux(im, NI, sb * T::UNITS_PER_SB + lane)) = q[u].d;
                        T::img_bsum(im, NI, sb, lane, q[u].bsum);
                        if (dump) {
                            uint8_t *base = ws + t * ws_stride;
                            *reinterpret_cast<uint32_t *>(base + (size_t)sb * 256 + 4 * lane) = q[u].packed;
                            if (lane == 0) reinterpret_cast<float *>(base + q8_K_off_d(K))[sb] = q[u].d;
                            if ((lane & 3) == 0) reinterpret_cast<int16_t *>(base + q8_K_off_bsums(K))[sb * 16 + (lane >> 2)] = (int16_t)q[u].bsum;
                        }
                    }
                }
            }
        }
    }
}

// Staging from an already quantized workspace: transpose the split planes to [it][chunk][lane].  The loads
// are split from their LDS stores (stage_issue / stage_commit) so that the caller can request the first weight
// tiles in between: loads return in issue order, so the staging data must be asked for first or it would wait
// for the much slower weight stream.  Registers cover PQ chunks and one side-data record per token and thread;
// longer rows finish in a plain loop inside stage_commit.
template <int WT, int NTOK> struct StageRegs {
    static constexpr int PQ = NTOK <= 4 ? 2 : 1;
    u32x4 v[NTOK][PQ];
    typename Traits<WT>::AuxT a[NTOK];
};

template <int WT, int NTOK, int WGS>
__device__ __forceinline__ void stage_issue(StageRegs<WT, NTOK> &sr, int NI, int units, int64_t K,
                                            const uint8_t *__restrict__ ws, size_t ws_stride) {
    using T = Traits<WT>;
    constexpr int PQ = StageRegs<WT, NTOK>::PQ;
    const int nq = NI * T::QCH * 64;                                    // 16-byte chunks per token
#pragma unroll
    for (int j = 0; j < PQ; j++) {
        const int r = j * WGS + (int)threadIdx.x;
        const int lane = r & 63, c = (r >> 6) % T::QCH, it = (r >> 6) / T::QCH;
        const int u = it * 64 + lane;
        const bool ok = r < nq && u < units;
        const size_t off = T::src_chunk(K, u, c);
#pragma unroll
        for (int t = 0; t < NTOK; t++) {
            sr.v[t][j] = u32x4{0u, 0u, 0u, 0u};
            if (ok) sr.v[t][j] = *reinterpret_cast<const u32x4 *>(ws + t * ws_stride + off);
        }
    }
    const int u = (int)threadIdx.x;
#pragma unroll
    for (int t = 0; t < NTOK; t++) sr.a[t] = T::aux_load(ws + t * ws_stride, K, u, u < units);   // no-op when AUX == 0
}

template <int WT, int NTOK, int WGS>
__device__ __forceinline__ void stage_commit(const StageRegs<WT, NTOK> &sr, uint8_t *lds, size_t img, int NI, int units,
                                             int64_t K, const uint8_t *__restrict__ ws, size_t ws_stride) {
    using T = Traits<WT>;
    using AuxT = typename T::AuxT;
    constexpr int PQ = StageRegs<WT, NTOK>::PQ;
    const int nq = NI * T::QCH * 64, na = NI * 64;
    const size_t aux0 = (size_t)NI * T::QCH * 1024;
#pragma unroll
    for (int j = 0; j < PQ; j++) {
        const int r = j * WGS + (int)threadIdx.x;
        if (r < nq) {
#pragma unroll
            for (int t = 0; t < NTOK; t++) reinterpret_cast<u32x4 *>(lds + t * img)[r] = sr.v[t][j];
        }
    }
    if constexpr (T::AUX > 0) {
        if ((int)threadIdx.x < na) {
#pragma unroll
            for (int t = 0; t < NTOK; t++) *reinterpret_cast<AuxT *>(lds + t * img + aux0 + (size_t)threadIdx.x * T::AUX) = sr.a[t];
        }
    }
    // rows longer than the register slots
    for (int r = PQ * WGS + (int)threadIdx.x; r < nq; r += WGS) {
        const int lane = r & 63, c = (r >> 6) % T::QCH, it = (r >> 6) / T::QCH;
        const int u = it * 64 + lane;
        const size_t off = T::src_chunk(K, u, c);
#pragma unroll
        for (int t = 0; t < NTOK; t++) {
            u32x4 v = {0u, 0u, 0u, 0u};
            if (u < units) v = *reinterpret_cast<const u32x4 *>(ws + t * ws_stride + off);
            reinterpret_cast<u32x4 *>(lds + t * img)[r] = v;
        }
    }
    if constexpr (T::AUX > 0) {
        for (int u = WGS + (int)threadIdx.x; u < na; u += WGS) {
#pragma unroll
            for (int t = 0; t < NTOK; t++)
                *reinterpret_cast<AuxT *>(lds + t * img + aux0 + (size_t)u * T::AUX) = T::aux_load(ws + t * ws_stride, K, u, u < units);
        }
    }
}


// The float4 chunk of a row that register slot j of this thread holds after xload (-1: none), the first chunk of the
// 256-value block that slot j of this wave covers (wave-uniform), and the RMS norm of the rows in those registers: a slot of a
// wave is one 256-value block with lane = chunk % 64 in both register layouts, which is how dev_common.h orders the sum of
// squares.  Lane 63 of every wave leaves the butterfly totals of its blocks in LDS (B, NORM_BLOCKS_MAX doubles per token, in a
// place the image does not reach), one barrier, every thread adds them up and scales its registers by 1 / sqrt(mean + eps)
// and then by the weight row: the same bits as rms_norm_kernel with a weight (ops.hip).
template <int WT, int WGS> __device__ __forceinline__ int xreg_chunk(int j, int64_t K) {
    using T = Traits<WT>;
    if constexpr (T::ACT == T_Q8_0 || T::ACT == T_F16) {
        const int c = j * WGS + (int)threadIdx.x;
        return c < (int)(K / 4) ? c : -1;
    } else {
        const int sb = j * (WGS / 64) + ((int)threadIdx.x >> 6);
        return sb < (int)(K / 256) ? sb * 64 + ((int)threadIdx.x & 63) : -1;
    }
}
template <int WGS> __device__ __forceinline__ int xreg_block_first_chunk(int j) {
    return j * WGS + ((int)threadIdx.x & ~63);            // both layouts: slot j of wave w starts at chunk j * WGS + 64 w
}
// A kernel with the norm takes rows of at most 256 * NORM_BLOCKS_MAX values and sizes its registers for that.
template <int NTOK> constexpr int norm_max_values() {
    return 256 * NORM_BLOCKS_MAX * NTOK < FUSE_MAX_VALUES ? 256 * NORM_BLOCKS_MAX * NTOK : FUSE_MAX_VALUES;
}
template <int WT, int NTOK, int WGS> struct NormRegs {
    static constexpr int NPER = XRegs<NTOK, WGS, norm_max_values<NTOK>()>::PER;
    float4 w[NPER];
};
template <int WT, int NTOK, int WGS>
__device__ __forceinline__ void norm_issue(NormRegs<WT, NTOK, WGS> &nr, const float *__restrict__ w, int64_t K) {
#pragma unroll
    for (int j = 0; j < NormRegs<WT, NTOK, WGS>::NPER; j++) {
        const int c = xreg_chunk<WT, WGS>(j, K);
        nr.w[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c >= 0) nr.w[j] = *reinterpret_cast<const float4 *>(w + 4 * (int64_t)c);
    }
}
template <int WT, int NTOK, int WGS>
__device__ __forceinline__ void norm_apply(XRegs<NTOK, WGS, norm_max_values<NTOK>()> &xr, const NormRegs<WT, NTOK, WGS> &nr, int64_t K, float eps, float *y,
                                           int64_t ldy, bool store, double *B) {
    constexpr int PER = NormRegs<WT, NTOK, WGS>::NPER;
    const int chunks = (int)(K / 4), blocks = (chunks + 63) >> 6;
#pragma unroll
    for (int t = 0; t < NTOK; t++)
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const int first = xreg_block_first_chunk<WGS>(j);
            if (first < chunks) {                                        // wave-uniform: all 64 lanes take part in the butterfly
                const double d = xreg_chunk<WT, WGS>(j, K) >= 0 ? norm_chunk_squares(xr.v[t][j]) : 0.0;
                const double total = wave_sum_f64_to_lane63(d);
                if ((threadIdx.x & 63) == 63) B[t * NORM_BLOCKS_MAX + (first >> 6)] = total;
            }
        }
    __syncthreads();
    float scale[NTOK];
#pragma unroll
    for (int t = 0; t < NTOK; t++) {
        const double total = norm_total_from_blocks(B + t * NORM_BLOCKS_MAX, blocks);
        const float mean = (float)(total / (double)K);
        scale[t] = 1.0f / sqrtf(mean + eps);
    }
#pragma unroll
    for (int t = 0; t < NTOK; t++)
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const int c = xreg_chunk<WT, WGS>(j, K);
            if (c >= 0) {
                float4 v = xr.v[t][j];
                v.x *= scale[t]; v.y *= scale[t]; v.z *= scale[t]; v.w *= scale[t];
                const float4 g = nr.w[j];
                v.x *= g.x; v.y *= g.y; v.z *= g.z; v.w *= g.w;
                xr.v[t][j] = v;
                if (store) *reinterpret_cast<float4 *>(y + (int64_t)t * ldy + 4 * (int64_t)c) = v;
            }
        }
}

// Two matrices of one shape and type that read the same activation (ffn_gate and ffn_up) as one launch: rows
// [0, n_first) are the first matrix, rows [n_first, N) the second one, whose weights and outputs lie w_off bytes / y_off
// floats away from where the first matrix's row and output of that index would be.  One matrix: n_first = N.
// t16 (one matrix only): the outputs also go, rounded to fp16, to t16[row * t16_ld + token] - the transposed store of V
// into the F16 cache that follows the V projection (reference llama-kv-cache.cpp cpy_v without flash attention).
// The workgroups that share one matrix: this workgroup's index among them, their number, and whether this workgroup
// is the one that also writes the quantized activations to the workspace (prologue-quantizing kernels).
struct GridPart { int64_t block, blocks; bool writes_workspace; };
__device__ __forceinline__ GridPart whole_grid() { return GridPart{(int64_t)blockIdx.x, (int64_t)gridDim.x, blockIdx.x == 0}; }

// gated (two matrices only): a wave takes row r of the first matrix and then row r of the second, and what is stored, at y's
// row r, is silu(first) * second - the SILU and MUL nodes that follow ffn_gate and ffn_up (reference llama-graph.cpp:562-690,
// LLM_FFN_SILU with LLM_FFN_PAR), with lm_ggml_vec_silu_f32's arithmetic; the two projections themselves are not stored.
// addend: a tensor of y's shape added to every output as it is stored (the residual ADD that follows wo and ffn_down, reference
// llama-model.cpp build_llama: ffn_inp = add(cur, inpSA), cur = add(cur, ffn_inp)): y = W x + addend, one IEEE addition as the
// ADD node's.  norm_w (kernels built NORMED, which always have one): the rows x are RMS-normed and multiplied by the weight row norm_w in the
// prologue, before they are quantized - the RMS_NORM and MUL nodes in front of the projections (build_norm, llama-graph.cpp:527-560)
// - with rms_norm_kernel's arithmetic and order of additions; norm_y, if given, receives the normed rows (workgroup 0 stores them).
struct SecondMatrix {
    int64_t n_first, w_off, y_off; unsigned short *t16; int64_t t16_ld; int gated;
    const float *addend; int64_t ld_add;
    const float *norm_w; float norm_eps; float *norm_y; int64_t norm_ldy;
};
constexpr SecondMatrix kNoSecond = {INT64_MAX, 0, 0, nullptr, 0, 0, nullptr, 0, nullptr, 0.f, nullptr, 0};


template <int WT, int NTOK, int R, int WGS, bool FUSEQ, int DEPTH, bool PHASED = false, bool GATED = false, bool ROPED = false,
          bool NORMED = false>
__device__ __forceinline__ void gemv_body(const uint8_t *__restrict__ W, size_t nb01, int64_t K, int64_t N,
                                          const float *__restrict__ x, int64_t ldx,
                                          uint8_t *__restrict__ ws, size_t ws_stride,
                                          float *__restrict__ y, int64_t ldy, const SecondMatrix sec,
                                          const GridPart gp, const RopeEpilogue rope = kNoRope) {
    static_assert(!ROPED || (R == 1 && !GATED && !PHASED && FUSEQ), "the pair walk of the rotated rows takes one row per step");
    static_assert(!NORMED || (FUSEQ && !PHASED), "the norm runs on the whole row in the prologue's registers");
    using T = Traits<WT>;
    extern __shared__ __align__(16) uint8_t lds[];
    static_assert(DEPTH == 1, "one step of weight loads is in flight beyond the one being computed");
    const int NI = iters_per_row<WT>(K);
    const int units = units_per_row<WT>(K);
    const size_t img = lds_image_bytes<WT>(K);
    const int lane = threadIdx.x & 63;
    const int64_t wave = gp.block * (WGS / 64) + (threadIdx.x >> 6);
    const int64_t nwaves = gp.blocks * (WGS / 64);
    // gated: tile T is row tile T / 2 of matrix T % 2; a wave walks 2 * wave, 2 * wave + 1, 2 * (wave + nwaves), ...
    constexpr bool gated = GATED;                      // a kernel of its own: sec.gated picks it in the launcher
    // ROPED: tile T is half T % 2 of rotated pair T / 2; a wave walks 2 * wave, 2 * wave + 1, 2 * (wave + nwaves), ...
    constexpr bool paired = GATED || ROPED;
    const int64_t tiles = gated ? 2 * ceil_div(sec.n_first, (int64_t)R) : ceil_div(N, R);
    const int64_t first_tile = paired ? 2 * wave : wave;
    [[maybe_unused]] auto rope_row = [&](int64_t T) -> int64_t {        // the row of tile T (32-bit division: wave-uniform, once per tile)
        const uint32_t p = (uint32_t)(T >> 1), hp = (uint32_t)rope.head_dim >> 1, rot = (uint32_t)rope.n_dims >> 1;
        const uint32_t h = p / hp, j = p - h * hp;
        const uint32_t ra = j < rot ? (rope.neox ? j : 2 * j) : (uint32_t)rope.n_dims + 2 * (j - rot);
        const uint32_t step = (j < rot && rope.neox) ? rot : 1u;
        return (int64_t)h * rope.head_dim + ra + (uint32_t)(T & 1) * step;
    };

    // A wave walks the steps (tile, it) = (wave, 0), (wave, 1), ..., (wave + nwaves, 0), ...; while it computes one step
    // the loads of the next are in flight.  Measured and dropped: rings of two and three steps (3-8 % slower as a loop; the
    // compiler cannot count the outstanding loads of a second register set across the back-edge and waits for all of
    // them), all steps of a short wave requested up front as straight-line code (exact waits, but 12.6 -> 14.2 us on a
    // 4096 x 14336 Q6_K matrix: four steps per wave at once thrash), tiles drawn from device-scope counters instead of
    // fixed shares (waves on different CUs finish between 53 and 86 us on a 431 MB matrix, yet handing the slow waves' tiles
    // to the fast ones changes nothing: the rate is the memory system's, not the distribution's).  All state is wave-uniform.
    struct Step { int64_t tile; int it; bool have; };
    auto after = [&](const Step &s) {
        Step n = s;
        if (s.it + 1 == NI) {
            n.tile = !paired ? s.tile + nwaves : ((s.tile & 1) ? s.tile + 2 * nwaves - 1 : s.tile + 1);
            n.it = 0;
        } else n.it = s.it + 1;
        n.have = s.have && n.tile < tiles;
        return n;
    };
    // The weights of a step into the raw registers.  Every lane issues the loads (lanes past the end of the row re-read
    // its last unit, the tail tile re-reads the last row; neither is used): a load inside a divergent branch makes the
    // compiler wait for everything in flight, outstanding stores included, before the next use of a load register.
    // In the prologue the loads are issued whether or not the wave has a tile (one without re-reads row 0): behind any
    // branch, the wait for the activations - requested earlier - would turn into a wait for these weights as well.
    typename T::Raw ring[R];
    auto load_step = [&](typename T::Raw (&set)[R], const Step &s, bool always) {
        if (always || s.have) {
            const int u = min(s.it * 64 + lane, units - 1);
#pragma unroll
            for (int r = 0; r < R; r++) {
                int64_t row = s.have ? min(s.tile * R + r, N - 1) : (int64_t)0;
                if (gated) row = s.have ? min((s.tile >> 1) * R + r, sec.n_first - 1) + (s.tile & 1) * sec.n_first : (int64_t)0;
                if constexpr (ROPED) row = s.have ? rope_row(s.tile) : (int64_t)0;
                const uint8_t *wrow = W + (size_t)row * nb01 + (row >= sec.n_first ? sec.w_off : (int64_t)0);
                if constexpr (WT == T_Q6_K_P) T::load_raw_planes(set[r], wrow, u, (int)(K >> 8));
                else T::load_raw(set[r], wrow, u);
            }
        }
    };
    Step s0{first_tile, 0, first_tile < tiles};

    // ---- prologue: activation loads first, then DEPTH steps of weight loads, then the activation image is built in LDS
    //      while the weights are still in flight ----
    // PHASED (rows of several steps with Q8_K activations, chosen by the launcher): a step reads the 16 super-blocks of its
    // own part of the image, which are SPS register slots of every thread.  Only the first step's part is built before the
    // first barrier; the part of step it + 1 is quantized behind the arithmetic of step it of the wave's first tile, while
    // that step's weights are on their way - the quantizer's vector work (a third of a 14336-value row's kernel when it all
    // stood in front) then fills time the waves would spend waiting.  Every wave, with or without a tile, takes part in
    // every part and barrier.  The fp32 registers live until the last part, which is why this is a kernel of its own.
    constexpr int SPS = 16 / (WGS / 64) > 0 ? 16 / (WGS / 64) : 1;      // slots per step
    static_assert(!PHASED || (FUSEQ && T::ACT == T_Q8_K && WGS >= 256 && (SPS % FUSE_ILP == 0 || SPS == 1)),
                  "parts of the image are whole quantizer slots");
    [[maybe_unused]] XRegs<NTOK, (PHASED ? WGS : 64)> xr_parts;
    if constexpr (FUSEQ && PHASED) {
        xload<WT, NTOK, WGS>(xr_parts, x, ldx, K);
        load_step(ring, s0, true);
        quantize_into_image<WT, NTOK, WGS>(xr_parts, lds, img, NI, K, ws, ws_stride, gp.writes_workspace, 0, SPS);
    } else if constexpr (FUSEQ) {
        // NORMED: a kernel of its own (the launcher picks it when there is a norm), with registers for the shorter rows it takes
        XRegs<NTOK, WGS, (NORMED ? norm_max_values<NTOK>() : FUSE_MAX_VALUES)> xr;
        xload<WT, NTOK, WGS>(xr, x, ldx, K);
        [[maybe_unused]] NormRegs<WT, NTOK, WGS> nr;
        if constexpr (NORMED) norm_issue<WT, NTOK, WGS>(nr, sec.norm_w, K);   // requested before the weights, needed before them
        [[maybe_unused]] float rope_cs = 0.f;                           // this thread's entry of the tokens' cos / sin table
        if constexpr (ROPED) {
            if ((int)threadIdx.x < NTOK * rope.n_dims) rope_cs = rope.table[threadIdx.x];
        }
        load_step(ring, s0, true);
        if constexpr (NORMED) {                                         // the block sums go behind the image (and the cos / sin table)
            size_t at = (size_t)NTOK * img;
            if constexpr (ROPED) at += (size_t)NTOK * rope.n_dims * sizeof(float);
            norm_apply<WT, NTOK, WGS>(xr, nr, K, sec.norm_eps, sec.norm_y, sec.norm_ldy, gp.writes_workspace && sec.norm_y,
                                      reinterpret_cast<double *>(lds + ((at + 7) & ~(size_t)7)));
        }
        quantize_into_image<WT, NTOK, WGS>(xr, lds, img, NI, K, ws, ws_stride, gp.writes_workspace);
        if constexpr (ROPED) {                                          // behind the image: [token][cos | sin]
            float *tab = reinterpret_cast<float *>(lds + (size_t)NTOK * img);
            if ((int)threadIdx.x < NTOK * rope.n_dims) tab[threadIdx.x] = rope_cs;
            for (int i = WGS + (int)threadIdx.x; i < NTOK * rope.n_dims; i += WGS) tab[i] = rope.table[i];
        }
    } else {
        StageRegs<WT, NTOK> sr;
        stage_issue<WT, NTOK, WGS>(sr, NI, units, K, ws, ws_stride);
        load_step(ring, s0, true);
        stage_commit<WT, NTOK, WGS>(sr, lds, img, NI, units, K, ws, ws_stride);
    }
    __syncthreads();
    // ---- main loop: decode the raw registers, refill them with the next step, accumulate ----
    // Finished tiles are kept in registers - lane k holds the k-th result of this wave and its row - and go to memory 64 at
    // a time (and at the end): one store instruction per 64 tiles instead of one per tile, and no store is outstanding
    // when the loop waits for its weight loads.
    float acc[R][NTOK], res[R][NTOK];
    int res_row = 0, nres = 0;
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int t = 0; t < NTOK; t++) { acc[r][t] = 0.f; res[r][t] = 0.f; }
    auto flush = [&](int count) {
        if constexpr (ROPED) {                           // lanes 2k and 2k + 1 hold the two values of one rotated pair
            const float *tab = reinterpret_cast<const float *>(lds + (size_t)NTOK * img);
            const int row = res_row, rowb = __shfl_down(res_row, 1);
            const uint32_t off = (uint32_t)row % (uint32_t)rope.head_dim;
            const bool mine = lane < count && !(lane & 1) && row < N;
            const bool rotated = off < (uint32_t)rope.n_dims;
            const uint32_t j = rope.neox ? off : off >> 1;
#pragma unroll
            for (int t = 0; t < NTOK; t++) {
                const float x0 = res[0][t], x1 = __shfl_down(res[0][t], 1);
                if (mine) {
                    float y0 = x0, y1 = x1;
                    if (rotated) {
                        const float c = tab[t * rope.n_dims + j], sn = tab[t * rope.n_dims + (rope.n_dims >> 1) + j];
                        y0 = x0 * c - x1 * sn;
                        y1 = x0 * sn + x1 * c;
                    }
                    if (rope.write_f32) { y[(int64_t)t * ldy + row] = y0; y[(int64_t)t * ldy + rowb] = y1; }
                    if (rope.h16) { rope.h16[(int64_t)t * rope.h16_ld + row] = f2h_rne(y0); rope.h16[(int64_t)t * rope.h16_ld + rowb] = f2h_rne(y1); }
                }
            }
            return;
        }
        if (gated) {                                     // lanes 2j and 2j + 1 hold the two projections of one row tile
#pragma unroll
            for (int r = 0; r < R; r++) {
                const int64_t row = (int64_t)res_row + r;
#pragma unroll
                for (int t = 0; t < NTOK; t++) {
                    const float up = __shfl_down(res[r][t], 1);
                    if (lane < count && !(lane & 1) && row < sec.n_first) y[(int64_t)t * ldy + row] = silu1(res[r][t]) * up;
                }
            }
            return;
        }
        if (lane < count) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                const int64_t row = (int64_t)res_row + r;
                if (row < N) {
#pragma unroll
                    for (int t = 0; t < NTOK; t++) {
                        float v = res[r][t];
                        if (sec.addend) v += sec.addend[(int64_t)t * sec.ld_add + row];
                        y[(int64_t)t * ldy + row + (row >= sec.n_first ? sec.y_off : (int64_t)0)] = v;
                        if (sec.t16) sec.t16[row * sec.t16_ld + t] = f2h_rne(res[r][t]);
                    }
                }
            }
        }
    };
    // one step: decode `set` (holding step s), refill it with step `next`, then the arithmetic of s
    auto consume = [&](typename T::Raw (&set)[R], const Step &s, const Step &next) {
        const int u = s.it * 64 + lane;
        const bool active = s.have && u < units;
        typename T::W w[R];
        if (active) {
#pragma unroll
            for (int r = 0; r < R; r++) T::decode(w[r], set[r], u);
        }
        load_step(set, next, false);
        if (active) {
#pragma unroll
            for (int t = 0; t < NTOK; t++) {
                typename T::A a;
                T::load_a(a, lds + t * img, NI, s.it, lane);
#pragma unroll
                for (int r = 0; r < R; r++) acc[r][t] = T::dot(w[r], a, acc[r][t]);
            }
        }
        if (s.have && s.it + 1 == NI) {
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int t = 0; t < NTOK; t++) {
                    const float sum = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wave_sum_to_lane63(acc[r][t])), 63));
                    res[r][t] = lane == nres ? sum : res[r][t];
                    acc[r][t] = 0.f;
                }
            if constexpr (ROPED) res_row = lane == nres ? (int)rope_row(s.tile) : res_row;
            else res_row = lane == nres ? (int)((gated ? s.tile >> 1 : s.tile) * R) : res_row;
            nres++;
        }
    };

    if constexpr (PHASED) {
        for (int it = 0; it < NI; it++) {                               // uniform over the workgroup
            if (s0.have) {
                const Step cur = s0;
                s0 = after(cur);
                consume(ring, cur, s0);
            }
            if (it + 1 < NI) {
                quantize_into_image<WT, NTOK, WGS>(xr_parts, lds, img, NI, K, ws, ws_stride, gp.writes_workspace, (it + 1) * SPS, (it + 2) * SPS);
                __syncthreads();
            }
        }
    }
    // The stores of a batch of results stay out of the inner loop.
    while (s0.have) {
        while (s0.have && nres < 64) {
            const Step cur = s0;
            s0 = after(cur);
            consume(ring, cur, s0);
        }
        flush(nres);
        nres = 0;
    }
    if constexpr (PHASED) flush(nres);                                  // a wave whose only tile went through the parts above
}

// Rows per wave step.  Two steps are in flight per wave (the next step's loads are issued before the current
// step's arithmetic), so one row of a 48..68-byte unit (Q4_K, Q6_K, Q8_0) or two rows of a 36-byte unit (Q4_0)
// keep about 100..140 bytes per lane outstanding, the depth at which a plain read kernel with the same access
// pattern peaks on this GPU; measured sweeps over rows x group size x groups per CU agree.
template <int WT> struct RowsPerWave { static constexpr int R = (WT == T_Q4_0) ? 2 : 1; };

// Steps of weight loads a wave keeps in flight.  A step is one row of at most 64 units (36..68 bytes per lane).
constexpr int GEMV_DEPTH = 1;                              // ring depths 2 and 3 measured 3-8 % slower
}  // namespace chip
