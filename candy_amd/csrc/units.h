// Per-format "units" of the matvec kernels: what one lane loads from a weight row per step and
// how it contracts it with the quantized activations parked in LDS.
// Arithmetic follows the integer vec-dots of tensor/internal/cuda/kernels/quantized.cu
// (vec_dot_q4_0_q8_1 :1919-1941, vec_dot_q8_0_q8_1 :2058-2073, vec_dot_q4_K_q8_1 :2239-2263,
// vec_dot_q6_K_q8_1 :2367-2389) with Q8_0 activations.
#pragma once

#include "blocks.h"
#include "internal.h"

namespace candy {

// LDS image of the activations: quants with 16 bytes of skew per 256 bytes (keeps 16-byte
// reads of lanes that are 32 or 64 bytes apart on distinct banks), then the scales.
__device__ __forceinline__ int skewed(int byte_off) { return byte_off + ((byte_off >> 8) << 4); }

// Weight loads are plain (cached) loads on purpose: a 128-byte line of a row is touched by up
// to three load instructions of the same wavefront (header, two halves of the nibbles), and a
// non-temporal hint makes the later ones fetch the line again.

// ------------------------------------------------------------------ per-format units

// SPAN: bytes that 64 consecutive units occupy in a row when that is a whole number of 16-byte
// chunks although single blocks are not 16-byte aligned (0: the unit's own loads are aligned).
struct UnitQ4K {
    static constexpr int ELEMS = 64;        // two 32-value sub-blocks sharing 32 bytes of nibbles
    static constexpr int ROW_ALIGN = 16;
    static constexpr int SPAN = 0;
    struct W { u32x4 hdr, q0, q1; };
    __host__ __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)(K >> 8) * 144; }
    __device__ static __forceinline__ void load(const uint8_t *row, int u, W &w) {
        const uint8_t *blk = row + (size_t)(u >> 2) * 144;
        w.hdr = *(const u32x4 *)blk;
        const u32x4 *q = (const u32x4 *)(blk + 16 + (u & 3) * 32);
        w.q0 = q[0];
        w.q1 = q[1];
    }
    // sum over the unit of w*x, with x = d_x * q_x: quantized.cu:2239-2263
    __device__ static __forceinline__ float dot(const W &w, int u, const int8_t *sq, const Q8Scale *ss) {
        return dot_parts(w.hdr, w.q0, w.q1, u, sq, ss);
    }
    // hdr: the block's 16-byte header; q0, q1: the unit's 32 bytes of nibbles
    __device__ static __forceinline__ float dot_parts(const u32x4 &hdr, const u32x4 &q0, const u32x4 &q1, int u,
                                                      const int8_t *sq, const Q8Scale *ss) {
        const uint4 *xa = (const uint4 *)(sq + skewed(u * 64));
        const uint4 x0 = xa[0], x1 = xa[1], x2 = xa[2], x3 = xa[3];
        const Q8Scale s0 = ss[2 * u], s1 = ss[2 * u + 1];
        uint32_t sc2, m2;
        q4k_scale_min_pair(hdr.y, hdr.z, hdr.w, u & 3, sc2, m2);
        const uint32_t M = 0x0F0F0F0Fu;
        int lo = 0, hi = 0;
        lo = dot4_i8(q0.x & M, x0.x, lo); hi = dot4_i8((q0.x >> 4) & M, x2.x, hi);
        lo = dot4_i8(q0.y & M, x0.y, lo); hi = dot4_i8((q0.y >> 4) & M, x2.y, hi);
        lo = dot4_i8(q0.z & M, x0.z, lo); hi = dot4_i8((q0.z >> 4) & M, x2.z, hi);
        lo = dot4_i8(q0.w & M, x0.w, lo); hi = dot4_i8((q0.w >> 4) & M, x2.w, hi);
        lo = dot4_i8(q1.x & M, x1.x, lo); hi = dot4_i8((q1.x >> 4) & M, x3.x, hi);
        lo = dot4_i8(q1.y & M, x1.y, lo); hi = dot4_i8((q1.y >> 4) & M, x3.y, hi);
        lo = dot4_i8(q1.z & M, x1.z, lo); hi = dot4_i8((q1.z >> 4) & M, x3.z, hi);
        lo = dot4_i8(q1.w & M, x1.w, lo); hi = dot4_i8((q1.w >> 4) & M, x3.w, hi);
        const float d = half_bits_to_float((uint16_t)(hdr.x & 0xFFFF));
        const float dmin = half_bits_to_float((uint16_t)(hdr.x >> 16));
        // every factor fits 24 bits (|dot| <= 32*15*127, |bsum| <= 32*127, scales < 64): full-rate v_mul_i32_i24
        const float sd = s0.d * (float)__mul24(lo, (int)(sc2 & 0xFF)) + s1.d * (float)__mul24(hi, (int)(sc2 >> 8));
        const float sm = s0.d * (float)__mul24(s0.bsum, (int)(m2 & 0xFF)) + s1.d * (float)__mul24(s1.bsum, (int)(m2 >> 8));
        return d * sd - dmin * sm;
    }
    // The same dot in two parts for kernels that contract one unit with several activation rows: what depends on
    // the weights only (nibbles spread to bytes, the two 6-bit scale / min pairs, d and dmin) is done once.
    struct P { uint32_t lo[8], hi[8]; int sc_lo, sc_hi, m_lo, m_hi; float d, dmin; };
    __device__ static __forceinline__ void prep(const W &w, int u, P &p) {
        const uint32_t M = 0x0F0F0F0Fu;
        const uint32_t q[8] = {w.q0.x, w.q0.y, w.q0.z, w.q0.w, w.q1.x, w.q1.y, w.q1.z, w.q1.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            p.lo[i] = q[i] & M;
            p.hi[i] = (q[i] >> 4) & M;
        }
        uint32_t sc2, m2;
        q4k_scale_min_pair(w.hdr.y, w.hdr.z, w.hdr.w, u & 3, sc2, m2);
        p.sc_lo = (int)(sc2 & 0xFF); p.sc_hi = (int)(sc2 >> 8);
        p.m_lo = (int)(m2 & 0xFF); p.m_hi = (int)(m2 >> 8);
        p.d = half_bits_to_float((uint16_t)(w.hdr.x & 0xFFFF));
        p.dmin = half_bits_to_float((uint16_t)(w.hdr.x >> 16));
    }
    __device__ static __forceinline__ float dot_p(const P &p, int u, const int8_t *sq, const Q8Scale *ss) {
        const uint4 *xa = (const uint4 *)(sq + skewed(u * 64));
        const uint4 x0 = xa[0], x1 = xa[1], x2 = xa[2], x3 = xa[3];
        const Q8Scale s0 = ss[2 * u], s1 = ss[2 * u + 1];
        const uint32_t xl[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
        const uint32_t xh[8] = {x2.x, x2.y, x2.z, x2.w, x3.x, x3.y, x3.z, x3.w};
        int lo = 0, hi = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            lo = dot4_i8(p.lo[i], xl[i], lo);
            hi = dot4_i8(p.hi[i], xh[i], hi);
        }
        const float sd = s0.d * (float)__mul24(lo, p.sc_lo) + s1.d * (float)__mul24(hi, p.sc_hi);
        const float sm = s0.d * (float)__mul24(s0.bsum, p.m_lo) + s1.d * (float)__mul24(s1.bsum, p.m_hi);
        return p.d * sd - p.dmin * sm;
    }
};

// UnitQ4K for kernels that use a unit once and give lane l unit 64 i + l (whole quads live or clamped together): the
// four units of a block sit in the four lanes of a quad, each lane loads one word of the block's 16-byte header and the
// quad rebuilds it with broadcasts where the dot needs it.  A quarter of the header bytes requested and three
// registers fewer held per unit (batch-1 kernel, 4096 x 11008: 6.53 -> 6.40 us; the fused decode kernels, which hold
// many units per lane, were slower this way: 514 -> 506 tok/s on the Llama-3-8B shape).
struct UnitQ4KQuad {
    static constexpr int ELEMS = UnitQ4K::ELEMS, ROW_ALIGN = UnitQ4K::ROW_ALIGN, SPAN = 0;
    struct W { uint32_t h; u32x4 q0, q1; };
    __host__ __device__ static __forceinline__ size_t row_bytes(int K) { return UnitQ4K::row_bytes(K); }
    __device__ static __forceinline__ void load(const uint8_t *row, int u, W &w) {
        const uint8_t *blk = row + (size_t)(u >> 2) * 144;
        w.h = *(const uint32_t *)(blk + 4 * (u & 3));
        const u32x4 *q = (const u32x4 *)(blk + 16 + (u & 3) * 32);
        w.q0 = q[0];
        w.q1 = q[1];
    }
    __device__ static __forceinline__ float dot(const W &w, int u, const int8_t *sq, const Q8Scale *ss) {
        u32x4 hdr;
        hdr.x = (uint32_t)dpp_move_i<0x00>((int)w.h);  // quad_perm [0,0,0,0] .. [3,3,3,3]
        hdr.y = (uint32_t)dpp_move_i<0x55>((int)w.h);
        hdr.z = (uint32_t)dpp_move_i<0xAA>((int)w.h);
        hdr.w = (uint32_t)dpp_move_i<0xFF>((int)w.h);
        return UnitQ4K::dot_parts(hdr, w.q0, w.q1, u, sq, ss);
    }
};

struct UnitQ8_0 {
    static constexpr int ELEMS = 32;
    static constexpr int ROW_ALIGN = 2;
    static constexpr int SPAN = 64 * 34;
    struct W { u32x4 q0, q1; uint16_t d; };
    __host__ __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)(K >> 5) * 34; }
    __device__ static __forceinline__ void load(const uint8_t *row, int u, W &w) {
        const BlockQ8_0 *blk = (const BlockQ8_0 *)row + u;
        w.d = blk->d;
        w.q0 = *(const u32x4_a2 *)(blk->qs);
        w.q1 = *(const u32x4_a2 *)(blk->qs + 16);
    }
    // quantized.cu:2058-2073
    __device__ static __forceinline__ float dot(const W &w, int u, const int8_t *sq, const Q8Scale *ss) {
        const uint4 *xa = (const uint4 *)(sq + skewed(u * 32));
        const uint4 x0 = xa[0], x1 = xa[1];
        int s = 0;
        s = dot4_i8(w.q0.x, x0.x, s); s = dot4_i8(w.q0.y, x0.y, s); s = dot4_i8(w.q0.z, x0.z, s); s = dot4_i8(w.q0.w, x0.w, s);
        s = dot4_i8(w.q1.x, x1.x, s); s = dot4_i8(w.q1.y, x1.y, s); s = dot4_i8(w.q1.z, x1.z, s); s = dot4_i8(w.q1.w, x1.w, s);
        return (half_bits_to_float(w.d) * ss[u].d) * (float)s;
    }
};

template <bool GGML_ORDER>
struct UnitQ4_0 {
    static constexpr int ELEMS = 32;
    static constexpr int ROW_ALIGN = 2;
    static constexpr int SPAN = 64 * 18;
    struct W { u32x4 q; uint16_t d; };
    __host__ __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)(K >> 5) * 18; }
    __device__ static __forceinline__ void load(const uint8_t *row, int u, W &w) {
        const BlockQ4_0 *blk = (const BlockQ4_0 *)row + u;
        w.d = blk->d;
        w.q = *(const u32x4_a2 *)(blk->qs);
    }
    // Sum (q-8)*x = sum q*x - 8*sum x, all in integers. quantized.cu:1919-1941 gets the
    // second term from the Q8_1 block's float sum; with Q8_0 activations it is the exact integer.
    __device__ static __forceinline__ float dot(const W &w, int u, const int8_t *sq, const Q8Scale *ss) {
        const uint4 *xa = (const uint4 *)(sq + skewed(u * 32));
        const uint4 x0 = xa[0], x1 = xa[1];
        const Q8Scale sx = ss[u];
        const uint32_t M = 0x0F0F0F0Fu;
        int s = 0;
        if (GGML_ORDER) {
            // low nibble of byte j pairs with x[j], high nibble with x[j+16] (quantized.cu:2426-2433)
            s = dot4_i8(w.q.x & M, x0.x, s); s = dot4_i8((w.q.x >> 4) & M, x1.x, s);
            s = dot4_i8(w.q.y & M, x0.y, s); s = dot4_i8((w.q.y >> 4) & M, x1.y, s);
            s = dot4_i8(w.q.z & M, x0.z, s); s = dot4_i8((w.q.z >> 4) & M, x1.z, s);
            s = dot4_i8(w.q.w & M, x0.w, s); s = dot4_i8((w.q.w >> 4) & M, x1.w, s);
        } else {
            // candy CPU order (quantized.go:87-92): byte j holds elements 2j (low) and 2j+1 (high);
            // gather the even and odd activation bytes of each 8-element run
            const uint32_t xs8[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
            const uint32_t qw[4] = {w.q.x, w.q.y, w.q.z, w.q.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t even = __builtin_amdgcn_perm(xs8[2 * j + 1], xs8[2 * j], 0x06040200u);
                const uint32_t odd = __builtin_amdgcn_perm(xs8[2 * j + 1], xs8[2 * j], 0x07050301u);
                s = dot4_i8(qw[j] & M, even, s);
                s = dot4_i8((qw[j] >> 4) & M, odd, s);
            }
        }
        s -= 8 * sx.bsum;
        return (half_bits_to_float(w.d) * sx.d) * (float)s;
    }
};

struct UnitQ6K {
    static constexpr int ELEMS = 32;   // 8 values from each 32-value quarter of one 128-value half
    static constexpr int ROW_ALIGN = 2;
    static constexpr int SPAN = 0;     // picking the unit's scattered bytes out of an LDS slice was measured slower
    struct W { u32x2 ql0, ql1, qh; uint32_t sc; uint16_t d; };
    __host__ __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)(K >> 8) * 210; }
    __device__ static __forceinline__ void load(const uint8_t *row, int u, W &w) {
        const BlockQ6K *blk = (const BlockQ6K *)row + (u >> 3);
        const int ip = (u >> 2) & 1, j = u & 3;
        w.ql0 = *(const u32x2_a2 *)(blk->ql + 64 * ip + 8 * j);
        w.ql1 = *(const u32x2_a2 *)(blk->ql + 64 * ip + 32 + 8 * j);
        w.qh = *(const u32x2_a2 *)(blk->qh + 32 * ip + 8 * j);
        // four single-byte loads: fetching the 16 scale bytes at once and permuting was measured slower, and so was
        // one 8-byte load with one v_perm_b32 picking the four (32000x4096 batch 1: 26.5 against 25.7 us)
        const int8_t *sc = blk->scales + 8 * ip + (j >> 1);
        w.sc = (uint32_t)(uint8_t)sc[0] | ((uint32_t)(uint8_t)sc[2] << 8) | ((uint32_t)(uint8_t)sc[4] << 16) |
               ((uint32_t)(uint8_t)sc[6] << 24);
        w.d = blk->d;
    }
    // quantized.cu:2367-2389: d * sum over 16-value groups of d8 * (dot * scale); the -32 offset is
    // applied as dot(q,x) - 32*sum(x) in integers.
    __device__ static __forceinline__ float dot(const W &w, int u, const int8_t *sq, const Q8Scale *ss) {
        return dot_parts(w.ql0, w.ql1, w.qh, w.sc, w.d, u, sq, ss);
    }
    // sc: the unit's four scales, one per byte; d: the block's fp16 scale
    __device__ static __forceinline__ float dot_parts(const u32x2 &wql0, const u32x2 &wql1, const u32x2 &wqh, uint32_t wsc,
                                                      uint16_t wd, int u, const int8_t *sq, const Q8Scale *ss) {
        const int sb = u >> 3, ip = (u >> 2) & 1, j = u & 3;
        const int blk0 = sb * 8 + ip * 4;  // first of the four 32-value activation blocks
        float sumf = 0.0f;
        const uint32_t M = 0x0F0F0F0Fu, H = 0x30303030u, ones = 0x01010101u;
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
            const uint2 x = *(const uint2 *)(sq + skewed((blk0 + qd) * 32 + 8 * j));
            const u32x2 ql = (qd & 1) ? wql1 : wql0;
            const uint32_t lx = (qd < 2) ? (ql.x & M) : ((ql.x >> 4) & M);
            const uint32_t ly = (qd < 2) ? (ql.y & M) : ((ql.y >> 4) & M);
            const uint32_t vx = lx | (((wqh.x >> (2 * qd)) << 4) & H);
            const uint32_t vy = ly | (((wqh.y >> (2 * qd)) << 4) & H);
            int dq = dot4_i8(vy, x.y, dot4_i8(vx, x.x, 0));
            const int sx = dot4_i8(ones, x.y, dot4_i8(ones, x.x, 0));
            dq -= 32 * sx;
            const int scale = (int)(int8_t)((wsc >> (8 * qd)) & 0xFF);
            sumf += ss[blk0 + qd].d * (float)__mul24(dq, scale);  // |dq| < 2^15, |scale| < 2^7
        }
        return half_bits_to_float(wd) * sumf;
    }
};

// UnitQ6K for kernels that use a unit once and give lane l unit 64 i + l (whole quads live or clamped together).  The
// four lanes of a quad hold the units j = 0 .. 3 of one half ip of a block; between them they need the eight scale
// bytes 8 ip .. 8 ip + 7 and d.  Lanes 0 and 1 load one word of scales each, lanes 2 and 3 the block's last word
// (scales 14, 15 and d), and the quad hands them round with broadcasts in the dot: one 4-byte request per lane where
// four single bytes and a half were five.
struct UnitQ6KQuad {
    static constexpr int ELEMS = UnitQ6K::ELEMS, ROW_ALIGN = UnitQ6K::ROW_ALIGN, SPAN = 0;
    struct W { u32x2 ql0, ql1, qh; uint32_t h; };
    __host__ __device__ static __forceinline__ size_t row_bytes(int K) { return UnitQ6K::row_bytes(K); }
    __device__ static __forceinline__ void load(const uint8_t *row, int u, W &w) {
        const BlockQ6K *blk = (const BlockQ6K *)row + (u >> 3);
        const int ip = (u >> 2) & 1, j = u & 3;
        w.ql0 = *(const u32x2_a2 *)(blk->ql + 64 * ip + 8 * j);
        w.ql1 = *(const u32x2_a2 *)(blk->ql + 64 * ip + 32 + 8 * j);
        w.qh = *(const u32x2_a2 *)(blk->qh + 32 * ip + 8 * j);
        w.h = *(const u32_a2 *)((const uint8_t *)blk + (j < 2 ? 192 + 8 * ip + 4 * j : 206));
    }
    __device__ static __forceinline__ float dot(const W &w, int u, const int8_t *sq, const Q8Scale *ss) {
        const uint32_t lo = (uint32_t)dpp_move_i<0x00>((int)w.h), hi = (uint32_t)dpp_move_i<0x55>((int)w.h);
        const uint32_t last = (uint32_t)dpp_move_i<0xAA>((int)w.h);
        // scales 8 ip + (j >> 1) + {0, 2, 4, 6}: the even or the odd bytes of the two words
        const uint32_t sc = (u & 2) ? __builtin_amdgcn_perm(hi, lo, 0x07050301u) : __builtin_amdgcn_perm(hi, lo, 0x06040200u);
        return UnitQ6K::dot_parts(w.ql0, w.ql1, w.qh, sc, (uint16_t)(last >> 16), u, sq, ss);
    }
};

}  // namespace candy
