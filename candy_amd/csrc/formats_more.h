// The reference's other block formats (Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K, Q8_K): for each, four consecutive
// dequantized values (the dequantize kernel writes one float4 per lane) and the matvec "unit" (what one lane
// loads from a weight row per step and how it contracts it with the Q8_0 activations in LDS).
// Dequantize: quantized.go:107-116 (Q4_1, candy's CPU order); quantized.cu:728-795 through dequantize_block
// :815-836 (Q4_1 ggml order :870-899, Q5_0, Q5_1), :902-920 (Q2_K), :936-966 (Q3_K), :1054-1087 (Q5_K),
// :1178-1199 (Q8_K).  Every product in those formulas is exact in f32 (an fp16 scale times a small integer),
// so each value is rounded at most once and does not depend on whether multiply and add are fused.
// Vec-dots: quantized.cu:1947-2053 (Q4_1, Q5_0, Q5_1), :2108-2135 (Q2_K), :2177-2209 (Q3_K), :2300-2331 (Q5_K),
// with the Q8_1 `sum` half replaced by the exact integer sum of the activation block.
#pragma once

#include "blocks.h"
#include "internal.h"
#include "units.h"

namespace candy {

__device__ __forceinline__ uint32_t load_u32_a2(const uint8_t *p) { return *(const u32_a2 *)p; }

// The 5th bits of four consecutive elements e0..e0+3 of a Q5_0 / Q5_1 block, moved to bit 4 of each byte.
__device__ __forceinline__ uint32_t q5_high4(uint32_t qh, int e0) {
    // one 24-bit multiply copies the nibble to offsets 0, 7, 14 and 21 (no two copies of different bits meet, so
    // nothing carries); bit i is then picked from the copy that puts it at 8i
    const uint32_t n = (qh >> e0) & 0xFu;
    return (__umul24(n, 0x00204081u) << 4) & 0x10101010u;
}
__device__ __forceinline__ int sum4_i8(uint32_t x, int acc) { return dot4_i8(0x01010101u, x, acc); }

// ------------------------------------------------------------------ Q4_1
template <bool GGML_ORDER>
struct FmtQ4_1 {
    static constexpr int ELEMS = 32, BYTES = 20;
    // values 4j .. 4j+3
    __device__ static __forceinline__ float4 quad(const uint8_t *blk, int j) {
        const BlockQ4_1 *b = (const BlockQ4_1 *)blk;
        const float d = half_bits_to_float(b->d), m = half_bits_to_float(b->m);
        int q[4];
        if (GGML_ORDER) {
            const uint32_t w = load_u32_a2(b->qs + 4 * (j & 3));
#pragma unroll
            for (int i = 0; i < 4; ++i) q[i] = (int)((w >> (8 * i + (j >= 4 ? 4 : 0))) & 0xF);
        } else {
            const uint32_t b0 = b->qs[2 * j], b1 = b->qs[2 * j + 1];
            q[0] = (int)(b0 & 0xF); q[1] = (int)(b0 >> 4); q[2] = (int)(b1 & 0xF); q[3] = (int)(b1 >> 4);
        }
        return make_float4(d * (float)q[0] + m, d * (float)q[1] + m, d * (float)q[2] + m, d * (float)q[3] + m);
    }
};

template <bool GGML_ORDER>
struct UnitQ4_1 {
    static constexpr int ELEMS = 32, ROW_ALIGN = 4, SPAN = 0;
    struct W { u32x4 q; uint32_t dm; };
    __host__ __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)(K >> 5) * 20; }
    __device__ static __forceinline__ void load(const uint8_t *row, int u, W &w) {
        const uint8_t *blk = row + (size_t)u * 20;
        w.dm = load_u32_a2(blk);
        w.q = *(const u32x4_a2 *)(blk + 4);
    }
    // sum q*x * (d*d8) + m * (d8 * sum x)
    __device__ static __forceinline__ float dot(const W &w, int u, const int8_t *sq, const Q8Scale *ss) {
        const uint4 *xa = (const uint4 *)(sq + skewed(u * 32));
        const uint4 x0 = xa[0], x1 = xa[1];
        const Q8Scale sx = ss[u];
        const uint32_t M = 0x0F0F0F0Fu;
        int s = 0;
        if (GGML_ORDER) {
            s = dot4_i8(w.q.x & M, x0.x, s); s = dot4_i8((w.q.x >> 4) & M, x1.x, s);
            s = dot4_i8(w.q.y & M, x0.y, s); s = dot4_i8((w.q.y >> 4) & M, x1.y, s);
            s = dot4_i8(w.q.z & M, x0.z, s); s = dot4_i8((w.q.z >> 4) & M, x1.z, s);
            s = dot4_i8(w.q.w & M, x0.w, s); s = dot4_i8((w.q.w >> 4) & M, x1.w, s);
        } else {
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
        const float d = half_bits_to_float((uint16_t)(w.dm & 0xFFFF)), m = half_bits_to_float((uint16_t)(w.dm >> 16));
        return (d * sx.d) * (float)s + (m * sx.d) * (float)sx.bsum;
    }
};

// ------------------------------------------------------------------ Q5_0 / Q5_1 (level = nibble | 5th bit << 4)
template <bool HAS_MIN>
struct FmtQ5 {
    static constexpr int ELEMS = 32, BYTES = HAS_MIN ? 24 : 22;
    __device__ static __forceinline__ float4 quad(const uint8_t *blk, int j) {
        const int off = HAS_MIN ? 4 : 2;
        const float d = half_bits_to_float(*(const uint16_t *)blk);
        const uint32_t qh = load_u32_a2(blk + off);
        const uint32_t w = load_u32_a2(blk + off + 4 + 4 * (j & 3));
        const uint32_t lev = ((w >> (j >= 4 ? 4 : 0)) & 0x0F0F0F0Fu) | q5_high4(qh, 4 * j);
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float l = (float)((lev >> (8 * i)) & 0xFF);
            if (HAS_MIN) v[i] = l * d + half_bits_to_float(*(const uint16_t *)(blk + 2));
            else v[i] = (l - 16.0f) * d;
        }
        return make_float4(v[0], v[1], v[2], v[3]);
    }
};

template <bool HAS_MIN>
struct UnitQ5 {
    static constexpr int ELEMS = 32, ROW_ALIGN = 2, SPAN = 0;
    static constexpr int BYTES = HAS_MIN ? 24 : 22;
    struct W { u32x4 q; uint32_t qh, dm; };
    __host__ __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)(K >> 5) * BYTES; }
    __device__ static __forceinline__ void load(const uint8_t *row, int u, W &w) {
        const uint8_t *blk = row + (size_t)u * BYTES;
        if (HAS_MIN) {
            w.dm = load_u32_a2(blk);
            w.qh = load_u32_a2(blk + 4);
            w.q = *(const u32x4_a2 *)(blk + 8);
        } else {
            w.dm = *(const uint16_t *)blk;
            w.qh = load_u32_a2(blk + 2);
            w.q = *(const u32x4_a2 *)(blk + 6);
        }
    }
    __device__ static __forceinline__ float dot(const W &w, int u, const int8_t *sq, const Q8Scale *ss) {
        const uint4 *xa = (const uint4 *)(sq + skewed(u * 32));
        const uint4 x0 = xa[0], x1 = xa[1];
        const Q8Scale sx = ss[u];
        const uint32_t M = 0x0F0F0F0Fu;
        const uint32_t qw[4] = {w.q.x, w.q.y, w.q.z, w.q.w};
        const uint32_t xl[4] = {x0.x, x0.y, x0.z, x0.w}, xh[4] = {x1.x, x1.y, x1.z, x1.w};
        int s = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {  // bytes 4i..4i+3: low nibbles are elements 4i.., high nibbles 16+4i..
            s = dot4_i8((qw[i] & M) | q5_high4(w.qh, 4 * i), xl[i], s);
            s = dot4_i8(((qw[i] >> 4) & M) | q5_high4(w.qh, 16 + 4 * i), xh[i], s);
        }
        const float d = half_bits_to_float((uint16_t)(w.dm & 0xFFFF));
        if (HAS_MIN) return (d * sx.d) * (float)s + (half_bits_to_float((uint16_t)(w.dm >> 16)) * sx.d) * (float)sx.bsum;
        return (d * sx.d) * (float)(s - 16 * sx.bsum);
    }
};

// ------------------------------------------------------------------ Q2_K
// element 128n + 32k + l = bits 2k.. of qs[32n + l]; 16-value group e/16: scale = low nibble, min = high nibble
struct FmtQ2K {
    static constexpr int ELEMS = 256, BYTES = 84;
    __device__ static __forceinline__ float4 quad(const uint8_t *blk, int j) {
        const BlockQ2K *b = (const BlockQ2K *)blk;
        const int e = 4 * j, n = e >> 7, k = (e & 127) >> 5, l = e & 31;
        const float dall = half_bits_to_float(b->d), dmin = half_bits_to_float(b->dmin);
        const uint32_t sc = b->scales[e >> 4];
        const float ds = dall * (float)(sc & 0xF), ms = dmin * (float)(sc >> 4);
        const uint32_t q = load_u32_a2(b->qs + 32 * n + l) >> (2 * k);
        return make_float4(ds * (float)(q & 3) - ms, ds * (float)((q >> 8) & 3) - ms, ds * (float)((q >> 16) & 3) - ms,
                           ds * (float)((q >> 24) & 3) - ms);
    }
};

// unit = the 8 bytes qs[32n + 8j ..]: elements 128n + 32k + 8j + i (k = 0..3, i = 0..7)
struct UnitQ2K {
    static constexpr int ELEMS = 32, ROW_ALIGN = 4, SPAN = 0;
    struct W { u32x2 q; uint32_t sc, dm; };
    __host__ __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)(K >> 8) * 84; }
    __device__ static __forceinline__ void load(const uint8_t *row, int u, W &w) {
        const BlockQ2K *b = (const BlockQ2K *)(row + (size_t)(u >> 3) * 84);
        const int n = (u >> 2) & 1, j = u & 3;
        w.q = *(const u32x2_a2 *)(b->qs + 32 * n + 8 * j);
        const uint8_t *sc = b->scales + 8 * n + (j >> 1);  // group (128n + 32k + 8j) / 16 = 8n + 2k + j/2
        w.sc = (uint32_t)sc[0] | ((uint32_t)sc[2] << 8) | ((uint32_t)sc[4] << 16) | ((uint32_t)sc[6] << 24);
        w.dm = load_u32_a2((const uint8_t *)b + 80);  // d, dmin
    }
    __device__ static __forceinline__ float dot(const W &w, int u, const int8_t *sq, const Q8Scale *ss) {
        const int sb = u >> 3, n = (u >> 2) & 1, j = u & 3;
        const int blk0 = sb * 8 + n * 4;
        float sumf_d = 0.0f, sumf_m = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint2 x = *(const uint2 *)(sq + skewed((blk0 + k) * 32 + 8 * j));
            const int dq = dot4_i8((w.q.y >> (2 * k)) & 0x03030303u, x.y, dot4_i8((w.q.x >> (2 * k)) & 0x03030303u, x.x, 0));
            const int sx = sum4_i8(x.y, sum4_i8(x.x, 0));
            const int sc = (int)((w.sc >> (8 * k)) & 0xFF);
            const float d8 = ss[blk0 + k].d;
            sumf_d += d8 * (float)(dq * (sc & 0xF));
            sumf_m += d8 * (float)(sx * (sc >> 4));
        }
        return half_bits_to_float((uint16_t)(w.dm & 0xFFFF)) * sumf_d - half_bits_to_float((uint16_t)(w.dm >> 16)) * sumf_m;
    }
};

// ------------------------------------------------------------------ Q3_K
// 6-bit scale of 16-value group `is`: low 4 bits in the nibbles of bytes 0..7, high 2 bits in bit pairs of bytes 8..11
__device__ __forceinline__ int q3k_scale6(const uint8_t *sc, int is) {
    const int lo = (sc[is & 7] >> (4 * (is >> 3))) & 0xF;
    const int hi = (sc[8 + (is & 3)] >> (2 * (is >> 2))) & 3;
    return lo | (hi << 4);
}

struct FmtQ3K {
    static constexpr int ELEMS = 256, BYTES = 110;
    __device__ static __forceinline__ float4 quad(const uint8_t *blk, int j4) {
        const BlockQ3K *b = (const BlockQ3K *)blk;
        const int e = 4 * j4, n = e >> 7, j = (e & 127) >> 5, l = e & 31;
        const float dl = half_bits_to_float(b->d) * (float)(q3k_scale6(b->scales, e >> 4) - 32);
        const uint32_t q = load_u32_a2(b->qs + 32 * n + l) >> (2 * j);
        const uint32_t h = load_u32_a2(b->hmask + l) >> (4 * n + j);
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int lev = (int)((q >> (8 * i)) & 3) - (((h >> (8 * i)) & 1) ? 0 : 4);
            v[i] = dl * (float)lev;
        }
        return make_float4(v[0], v[1], v[2], v[3]);
    }
};

// unit as for Q2_K, plus the 8 mask bytes hmask[8j ..] (bit 4n + k) and the 6-bit scales of its four groups
struct UnitQ3K {
    static constexpr int ELEMS = 32, ROW_ALIGN = 2, SPAN = 0;
    struct W { u32x2 q, h; uint32_t sc; uint16_t d; };
    __host__ __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)(K >> 8) * 110; }
    __device__ static __forceinline__ void load(const uint8_t *row, int u, W &w) {
        const BlockQ3K *b = (const BlockQ3K *)(row + (size_t)(u >> 3) * 110);
        const int n = (u >> 2) & 1, j = u & 3;
        w.q = *(const u32x2_a2 *)(b->qs + 32 * n + 8 * j);
        w.h = *(const u32x2_a2 *)(b->hmask + 8 * j);
        // eight single-byte loads: fetching the 12 scale bytes as two 8-byte loads and picking the fields with
        // byte permutes was measured slower (4096x11008 batch 1: 14.1 against 11.6 us)
        uint32_t sc = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) sc |= (uint32_t)q3k_scale6(b->scales, 8 * n + 2 * k + (j >> 1)) << (8 * k);
        w.sc = sc;
        w.d = b->d;
    }
    // level = two bits + 4 * mask bit - 4: sum level*x = sum (q | h << 2) x - 4 sum x
    __device__ static __forceinline__ float dot(const W &w, int u, const int8_t *sq, const Q8Scale *ss) {
        return dot_parts(w.q, w.h, w.sc, w.d, u, sq, ss);
    }
    // sc: the unit's four 6-bit scales, one per byte; d: the block's fp16 scale
    __device__ static __forceinline__ float dot_parts(const u32x2 &wq, const u32x2 &wh, uint32_t wsc, uint16_t wd, int u,
                                                      const int8_t *sq, const Q8Scale *ss) {
        const int sb = u >> 3, n = (u >> 2) & 1, j = u & 3;
        const int blk0 = sb * 8 + n * 4;
        float sumf = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint2 x = *(const uint2 *)(sq + skewed((blk0 + k) * 32 + 8 * j));
            const uint32_t vx = ((wq.x >> (2 * k)) & 0x03030303u) | (((wh.x >> (4 * n + k)) & 0x01010101u) << 2);
            const uint32_t vy = ((wq.y >> (2 * k)) & 0x03030303u) | (((wh.y >> (4 * n + k)) & 0x01010101u) << 2);
            const int dq = dot4_i8(vy, x.y, dot4_i8(vx, x.x, 0)) - 4 * sum4_i8(x.y, sum4_i8(x.x, 0));
            const int sc = (int)((wsc >> (8 * k)) & 0xFF) - 32;
            sumf += ss[blk0 + k].d * (float)(dq * sc);
        }
        return half_bits_to_float(wd) * sumf;
    }
};

// UnitQ3K for kernels that give lane l unit 64 i + l: the quad that holds the units j = 0 .. 3 of one half n of a block
// shares the twelve scale bytes and d.  Lanes 0, 1 and 2 load one word of scales each, lane 3 the block's last word
// (scales 10, 11 and d); the dot takes them by quad broadcast and picks the unit's four 6-bit scales, groups
// is = 8 n + 2 k + (j >> 1): low nibbles from the even or odd bytes of words 0 and 1 shifted by 4 n, high bit pairs from
// bytes (is & 3) of word 2 shifted by 2 (is >> 2).  Three requests per unit where there were eleven.
struct UnitQ3KQuad {
    static constexpr int ELEMS = UnitQ3K::ELEMS, ROW_ALIGN = UnitQ3K::ROW_ALIGN, SPAN = 0;
    struct W { u32x2 q, h; uint32_t s; };
    __host__ __device__ static __forceinline__ size_t row_bytes(int K) { return UnitQ3K::row_bytes(K); }
    __device__ static __forceinline__ void load(const uint8_t *row, int u, W &w) {
        const BlockQ3K *b = (const BlockQ3K *)(row + (size_t)(u >> 3) * 110);
        const int n = (u >> 2) & 1, j = u & 3;
        w.q = *(const u32x2_a2 *)(b->qs + 32 * n + 8 * j);
        w.h = *(const u32x2_a2 *)(b->hmask + 8 * j);
        w.s = load_u32_a2((const uint8_t *)b + (j < 3 ? 96 + 4 * j : 106));
    }
    __device__ static __forceinline__ float dot(const W &w, int u, const int8_t *sq, const Q8Scale *ss) {
        const uint32_t w0 = (uint32_t)dpp_move_i<0x00>((int)w.s), w1 = (uint32_t)dpp_move_i<0x55>((int)w.s);
        const uint32_t w2 = (uint32_t)dpp_move_i<0xAA>((int)w.s), last = (uint32_t)dpp_move_i<0xFF>((int)w.s);
        const int n = (u >> 2) & 1;
        const bool odd = (u & 2) != 0;
        const uint32_t lo4 = ((odd ? __builtin_amdgcn_perm(w1, w0, 0x07050301u) : __builtin_amdgcn_perm(w1, w0, 0x06040200u)) >> (4 * n)) & 0x0F0F0F0Fu;
        const uint32_t t = odd ? __builtin_amdgcn_perm(w2, w2, 0x03010301u) : __builtin_amdgcn_perm(w2, w2, 0x02000200u);
        const uint32_t hi4 = ((t >> (4 * n)) & 0x00000303u) | ((t >> (4 * n + 2)) & 0x03030000u);
        return UnitQ3K::dot_parts(w.q, w.h, lo4 | (hi4 << 4), (uint16_t)(last >> 16), u, sq, ss);
    }
};

// ------------------------------------------------------------------ Q5_K
// sub-block t: low (t even) or high nibble of qs[32 (t/2) + l] plus 16 * bit t of qh[l]
struct FmtQ5K {
    static constexpr int ELEMS = 256, BYTES = 176;
    __device__ static __forceinline__ float4 quad(const uint8_t *blk, int j) {
        const uint32_t *w = (const uint32_t *)blk;  // 176-byte blocks keep 16-byte alignment
        const int e = 4 * j, t = e >> 5, l = e & 31;
        const float dall = half_bits_to_float((uint16_t)(w[0] & 0xFFFF)), dmin = half_bits_to_float((uint16_t)(w[0] >> 16));
        uint32_t sc2, m2;
        q4k_scale_min_pair(w[1], w[2], w[3], t >> 1, sc2, m2);
        const float d1 = dall * (float)((sc2 >> (8 * (t & 1))) & 0xFF), m1 = dmin * (float)((m2 >> (8 * (t & 1))) & 0xFF);
        const uint32_t q = (w[12 + 8 * (t >> 1) + (l >> 2)] >> (4 * (t & 1))) & 0x0F0F0F0Fu;
        const uint32_t h = (w[4 + (l >> 2)] >> t) & 0x01010101u;
        const uint32_t lev = q | (h << 4);
        return make_float4(d1 * (float)(lev & 0xFF) - m1, d1 * (float)((lev >> 8) & 0xFF) - m1,
                           d1 * (float)((lev >> 16) & 0xFF) - m1, d1 * (float)(lev >> 24) - m1);
    }
};

// unit = two sub-blocks sharing 32 nibble bytes (as UnitQ4K) plus the 32 bytes of 5th bits
struct UnitQ5K {
    static constexpr int ELEMS = 64, ROW_ALIGN = 16, SPAN = 0;
    struct W { u32x4 hdr, h0, h1, q0, q1; };
    __host__ __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)(K >> 8) * 176; }
    __device__ static __forceinline__ void load(const uint8_t *row, int u, W &w) {
        const uint8_t *blk = row + (size_t)(u >> 2) * 176;
        w.hdr = *(const u32x4 *)blk;
        w.h0 = *(const u32x4 *)(blk + 16);
        w.h1 = *(const u32x4 *)(blk + 32);
        const u32x4 *q = (const u32x4 *)(blk + 48 + (u & 3) * 32);
        w.q0 = q[0];
        w.q1 = q[1];
    }
    __device__ static __forceinline__ float dot(const W &w, int u, const int8_t *sq, const Q8Scale *ss) {
        const uint32_t h[8] = {w.h0.x, w.h0.y, w.h0.z, w.h0.w, w.h1.x, w.h1.y, w.h1.z, w.h1.w};
        return dot_parts(w.hdr, h, w.q0, w.q1, u, sq, ss);
    }
    // hdr: the block's 16-byte header; h: its 32 bytes of fifth bits; q0, q1: the unit's 32 bytes of nibbles
    __device__ static __forceinline__ float dot_parts(const u32x4 &hdr, const uint32_t (&h)[8], const u32x4 &q0,
                                                      const u32x4 &q1, int u, const int8_t *sq, const Q8Scale *ss) {
        const uint4 *xa = (const uint4 *)(sq + skewed(u * 64));
        const uint4 x0 = xa[0], x1 = xa[1], x2 = xa[2], x3 = xa[3];
        const Q8Scale s0 = ss[2 * u], s1 = ss[2 * u + 1];
        const int p = u & 3;
        uint32_t sc2, m2;
        q4k_scale_min_pair(hdr.y, hdr.z, hdr.w, p, sc2, m2);
        const uint32_t M = 0x0F0F0F0Fu, B = 0x01010101u;
        const uint32_t q[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        const uint32_t xl[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
        const uint32_t xh[8] = {x2.x, x2.y, x2.z, x2.w, x3.x, x3.y, x3.z, x3.w};
        int lo = 0, hi = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            lo = dot4_i8((q[i] & M) | (((h[i] >> (2 * p)) & B) << 4), xl[i], lo);
            hi = dot4_i8(((q[i] >> 4) & M) | (((h[i] >> (2 * p + 1)) & B) << 4), xh[i], hi);
        }
        const float d = half_bits_to_float((uint16_t)(hdr.x & 0xFFFF));
        const float dmin = half_bits_to_float((uint16_t)(hdr.x >> 16));
        const float sd = s0.d * (float)(lo * (int)(sc2 & 0xFF)) + s1.d * (float)(hi * (int)(sc2 >> 8));
        const float sm = s0.d * (float)(s0.bsum * (int)(m2 & 0xFF)) + s1.d * (float)(s1.bsum * (int)(m2 >> 8));
        return d * sd - dmin * sm;
    }
};

// UnitQ5K for kernels that give lane l unit 64 i + l.  The four units of a block sit in the four lanes of a quad and all
// need the block's first 48 bytes (header and fifth bits): lane j loads words 3 j .. 3 j + 2 of them and the dot takes
// the twelve words by quad broadcast.  Two 16-byte and one 12-byte request per unit where there were five of 16 bytes.
template <int LANE>
__device__ __forceinline__ uint32_t quad_from(uint32_t v) {
    return (uint32_t)dpp_move_i<LANE * 0x55>((int)v);  // quad_perm [LANE, LANE, LANE, LANE]
}
struct UnitQ5KQuad {
    static constexpr int ELEMS = UnitQ5K::ELEMS, ROW_ALIGN = UnitQ5K::ROW_ALIGN, SPAN = 0;
    struct W { uint32_t s0, s1, s2; u32x4 q0, q1; };
    __host__ __device__ static __forceinline__ size_t row_bytes(int K) { return UnitQ5K::row_bytes(K); }
    __device__ static __forceinline__ void load(const uint8_t *row, int u, W &w) {
        const uint8_t *blk = row + (size_t)(u >> 2) * 176;
        const uint32_t *s = (const uint32_t *)(blk + 12 * (u & 3));
        w.s0 = s[0];
        w.s1 = s[1];
        w.s2 = s[2];
        const u32x4 *q = (const u32x4 *)(blk + 48 + (u & 3) * 32);
        w.q0 = q[0];
        w.q1 = q[1];
    }
    __device__ static __forceinline__ float dot(const W &w, int u, const int8_t *sq, const Q8Scale *ss) {
        u32x4 hdr;
        hdr.x = quad_from<0>(w.s0); hdr.y = quad_from<0>(w.s1); hdr.z = quad_from<0>(w.s2); hdr.w = quad_from<1>(w.s0);
        const uint32_t h[8] = {quad_from<1>(w.s1), quad_from<1>(w.s2), quad_from<2>(w.s0), quad_from<2>(w.s1),
                               quad_from<2>(w.s2), quad_from<3>(w.s0), quad_from<3>(w.s1), quad_from<3>(w.s2)};
        return UnitQ5K::dot_parts(hdr, h, w.q0, w.q1, u, sq, ss);
    }
};

// ------------------------------------------------------------------ Q8_K (dequantize only)
struct FmtQ8K {
    static constexpr int ELEMS = 256, BYTES = 292;
    __device__ static __forceinline__ float4 quad(const uint8_t *blk, int j) {
        const BlockQ8K *b = (const BlockQ8K *)blk;
        const float d = b->d;
        const uint32_t q = *(const uint32_t *)(b->qs + 4 * j);
        return make_float4((float)(int8_t)(q & 0xFF) * d, (float)(int8_t)((q >> 8) & 0xFF) * d,
                           (float)(int8_t)((q >> 16) & 0xFF) * d, (float)(int8_t)(q >> 24) * d);
    }
};

}  // namespace candy
