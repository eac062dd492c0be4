// Batched (m >= 16) Q4_K and Q6_K matmul on the integer matrix cores, exact like the matvec:
// y[m, N] = x[m, K] . W^T with x quantized to Q8_0.
//
// mul_mat_q + vec_dot_q4_K_q8_1_impl_mmq / vec_dot_q6_K_q8_1_impl_mmq
// (tensor/internal/cuda/kernels/quantized.cu:455-578, :2266-2294, :2392-2417) tile the contraction
// for dp4a; here a 32-value sub-block is one v_mfma_i32_16x16x32_i8 (16 weight rows x 16
// activation rows) and the scales are applied to the int32 tile as the batch-1 vec-dots do
// (quantized.cu:2239-2263, :2367-2389):
//   Q4_K  sumf_d += d8 * float(dot * sc);  sumf_m += d8 * float(bsum * m);  y += d * sumf_d - dmin * sumf_m
//         (d and dmin folded into the per-sub-block factors)
//   Q6_K  y += d * sum over 16-value groups of d8 * float(sc * dot): the two groups of a sub-block are two
//         MFMAs whose A operand is zeroed in the other half (lanes 0-31 hold k 0-15, lanes 32-63 k 16-31),
//         combined as integers (sc_lo * dot_lo + sc_hi * dot_hi < 2^24, exact in f32).
// The result differs from the CPU contraction only by f32 summation order (no fp16 operand
// rounding). Running the Q4_K min term as a small f32 MFMA product instead was measured slower:
// the kernel is bound by the sum of matrix and vector issue.
//
// Work split: a wavefront owns 16 weight rows and all BM = 16*TM activation rows of the
// workgroup; the four wavefronts of a workgroup share the activation tile in LDS.
//   * weights are fetched a stage (up to four super-blocks, 1024 values) ahead as 16-byte chunks
//     that run along the rows, so every wavefront load covers whole cache lines (fetching them
//     directly in the A-operand layout, 8 bytes per lane from 16 rows, was 1.3x slower); the stage
//     is parked in the wavefront's own LDS slice, every super-block at a 16-byte aligned slot
//     (Q6_K blocks are 210 bytes and only 2-byte aligned in memory), from where each lane picks
//     its A-operand bytes (row = lane%16, 8 consecutive k per lane);
//   * Q4_K's 6-bit scales are unpacked once per (row, pair) by the lane that owns that row in the
//     A layout and handed through LDS to the lanes that own the row in the C layout
//     (4 consecutive weight rows per lane); Q6_K's int8 scales are read from the slice directly;
//   * activations: 256 int8 per row per super-block plus {d, d*bsum} per block, loaded one
//     super-block ahead into registers and parked in LDS between two barriers.
// The rescale costs 16 VALU instructions per 16x16x32 tile (convert, multiply and two fused
// multiply-adds per result register), which is what bounds the large-m rate.
#include <algorithm>
#include <cstdlib>

#include "blocks.h"
#include "internal.h"
#include "formats_more.h"

namespace candy {

typedef int int4v __attribute__((ext_vector_type(4)));

constexpr int XROW = 272;  // LDS pitch of an activation row: 256 quants + 16 (bank spread)

__device__ __forceinline__ void wave_lds_fence() {
    // orders LDS traffic of one wavefront (its LDS operations complete in order): no barrier needed
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---------------------------------------------------------------------------------------------
// Per-format part: what one super-block of the wavefront's 16 rows does to the accumulators.
//   slice   the wavefront's LDS slice, row r's super-block b at slice + r * pitch + b * SLOT
//   s_xq    activation tile [16*TM][XROW] int8, s_xs {d, d*bsum} [16*TM][8]
//   acc     lane (j = lane%16, c = lane/16) holds activation row 16a+j, weight rows 4c+i
// Q4_K and Q5_K share everything but the fifth bit: a Q5_K block is a Q4_K block with 32 bytes of high bits
// between the header and the nibbles (bit t of byte l belongs to value l of sub-block t, quantized.cu:1044-1080).
struct ExchangeK {
    float dsc[8][16];  // d * scale    [sub-block][row]
    float dmf[8][16];  // dmin * min
};
template <int TM, bool FIVE>
__device__ __forceinline__ void superblock_q45k(const uint8_t *wl, int j, int c, ExchangeK &ex, const int8_t *s_xq,
                                                const float2 *s_xs, float (&acc)[TM][4]) {
    constexpr int QS = FIVE ? 48 : 16;  // where the nibbles start
    {   // lane (row j, pair c) unpacks one pair of 6-bit scales / mins, folds the row's d / dmin in and parks
        // the four factors for the lanes that own the row in the C layout
        const u32x4 h = *(const u32x4 *)wl;
        uint32_t sc2, m2;
        q4k_scale_min_pair(h.y, h.z, h.w, c, sc2, m2);
        const float d = half_bits_to_float((uint16_t)(h.x & 0xFFFF)), dmin = half_bits_to_float((uint16_t)(h.x >> 16));
        ex.dsc[2 * c][j] = d * (float)(sc2 & 0xFF);
        ex.dsc[2 * c + 1][j] = d * (float)(sc2 >> 8);
        ex.dmf[2 * c][j] = dmin * (float)(m2 & 0xFF);
        ex.dmf[2 * c + 1][j] = dmin * (float)(m2 >> 8);
    }
    wave_lds_fence();
    float4 dsq[8], dmq[8];  // my four C rows 4c .. 4c+3, per sub-block
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        dsq[t] = *(const float4 *)&ex.dsc[t][4 * c];
        dmq[t] = *(const float4 *)&ex.dmf[t][4 * c];
    }
    wave_lds_fence();  // the slots are rewritten by the next super-block
    u32x2 qh = {0u, 0u};
    if (FIVE) qh = *(const u32x2 *)(wl + 16 + 8 * c);  // fifth bits of values 8c .. 8c+7 of every sub-block
    auto afrag_of = [&](int t) __attribute__((always_inline)) {
        const u32x2 qa = *(const u32x2 *)(wl + QS + 32 * (t >> 1) + 8 * c);
        const int sh = (t & 1) * 4;
        uint32_t lo = (qa.x >> sh) & 0x0F0F0F0Fu, hi = (qa.y >> sh) & 0x0F0F0F0Fu;
        if (FIVE) {
            lo |= ((qh.x >> t) & 0x01010101u) << 4;
            hi |= ((qh.y >> t) & 0x01010101u) << 4;
        }
        return (long)(((uint64_t)hi << 32) | lo);
    };
    if constexpr (TM == 1) {
        // one tile per sub-block: nothing else in the wavefront covers an MFMA's latency, so all eight products
        // of the super-block are issued first and rescaled afterwards
        int4v d8[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const long bfrag = *(const long *)&s_xq[j * XROW + 32 * t + 8 * c];
            d8[t] = __builtin_amdgcn_mfma_i32_16x16x32_i8(afrag_of(t), bfrag, int4v{0, 0, 0, 0}, 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const float dsc[4] = {dsq[t].x, dsq[t].y, dsq[t].z, dsq[t].w};
            const float dmf[4] = {dmq[t].x, dmq[t].y, dmq[t].z, dmq[t].w};
            const float2 sx = s_xs[j * 8 + t];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[0][i] += sx.x * ((float)d8[t][i] * dsc[i]);
                acc[0][i] -= dmf[i] * sx.y;
            }
        }
        return;
    }
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const long afrag = afrag_of(t);
        const float dsc[4] = {dsq[t].x, dsq[t].y, dsq[t].z, dsq[t].w};  // d * sc and dmin * m of my four weight rows
        const float dmf[4] = {dmq[t].x, dmq[t].y, dmq[t].z, dmq[t].w};
        int4v d[TM];  // all tiles of the sub-block first, so the matrix pipe runs under the rescale
#pragma unroll
        for (int a = 0; a < TM; ++a) {
            const long bfrag = *(const long *)&s_xq[(16 * a + j) * XROW + 32 * t + 8 * c];
            d[a] = __builtin_amdgcn_mfma_i32_16x16x32_i8(afrag, bfrag, int4v{0, 0, 0, 0}, 0, 0, 0);
        }
#pragma unroll
        for (int a = 0; a < TM; ++a) {
            const float2 sx = s_xs[(16 * a + j) * 8 + t];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[a][i] += sx.x * ((float)d[a][i] * dsc[i]);  // d8 * d * sc * dot
                acc[a][i] -= dmf[i] * sx.y;                     // d8 * bsum * dmin * m
            }
        }
    }
}

struct TileQ4K {
    static constexpr int BLOCK = 144, SLOT = 144;
    typedef u32x4 GlobalChunk;  // rows are 16-byte aligned
    typedef ExchangeK Exchange;
    template <int TM>
    static __device__ __forceinline__ void superblock(const uint8_t *slice, int pitch, int b, int j, int c, Exchange &ex,
                                                      const int8_t *s_xq, const float2 *s_xs, float (&acc)[TM][4]) {
        superblock_q45k<TM, false>(slice + j * pitch + SLOT * b, j, c, ex, s_xq, s_xs, acc);
    }
};

struct TileQ5K {
    static constexpr int BLOCK = 176, SLOT = 176;
    typedef u32x4 GlobalChunk;
    typedef ExchangeK Exchange;
    template <int TM>
    static __device__ __forceinline__ void superblock(const uint8_t *slice, int pitch, int b, int j, int c, Exchange &ex,
                                                      const int8_t *s_xq, const float2 *s_xs, float (&acc)[TM][4]) {
        superblock_q45k<TM, true>(slice + j * pitch + SLOT * b, j, c, ex, s_xq, s_xs, acc);
    }
};

struct TileQ6K {
    static constexpr int BLOCK = 210, SLOT = 224;  // 14 chunks: the last one runs 14 bytes into the next block
    typedef u32x4_a2 GlobalChunk;                  // blocks sit on 2-byte boundaries
    struct Exchange {};
    template <int TM>
    static __device__ __forceinline__ void superblock(const uint8_t *slice, int pitch, int b, int j, int c, Exchange &,
                                                      const int8_t *s_xq, const float2 *s_xs, float (&acc)[TM][4]) {
        const uint8_t *wl = slice + j * pitch + SLOT * b;
        // scales[16] (int8) and d of my four C rows, straight from the slice
        u32x4 scq[4];
        float dw[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint8_t *row = slice + (4 * c + i) * pitch + SLOT * b;
            scq[i] = *(const u32x4 *)(row + 192);
            dw[i] = half_bits_to_float(*(const uint16_t *)(row + 208));
        }
        float part[TM][4];  // sum over the super-block of d8 * (sc . dot), before the row's d
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int i = 0; i < 4; ++i) part[a][i] = 0.0f;
        const bool low_half = c < 2;  // my 8 values belong to the sub-block's first 16-value group
#pragma unroll
        for (int ip = 0; ip < 2; ++ip) {
            // element 128*ip + 32*quarter + il: ql[64*ip + 32*(quarter&1) + il] low/high nibble, qh[32*ip + il] bit pair
            const u32x2 qla = *(const u32x2 *)(wl + 64 * ip + 8 * c), qlb = *(const u32x2 *)(wl + 64 * ip + 32 + 8 * c);
            const u32x2 qh = *(const u32x2 *)(wl + 128 + 32 * ip + 8 * c);
#pragma unroll
            for (int quarter = 0; quarter < 4; ++quarter) {
                const int t = 4 * ip + quarter;
                const u32x2 ql = (quarter & 1) ? qlb : qla;
                uint32_t w2[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const uint32_t nib = (quarter & 2) ? (ql[e] >> 4) & 0x0F0F0F0Fu : ql[e] & 0x0F0F0F0Fu;
                    const uint32_t top = quarter == 0 ? (qh[e] << 4) : quarter == 1 ? (qh[e] << 2)
                                       : quarter == 2 ? qh[e] : (qh[e] >> 2);
                    const uint32_t q6 = nib | (top & 0x30303030u);
                    // bytewise q6 - 32 (0..63 -> -32..31): bias by 128 so no byte borrows, then flip the bias off
                    w2[e] = ((q6 | 0x80808080u) - 0x20202020u) ^ 0x80808080u;
                }
                const long full = (long)(((uint64_t)w2[1] << 32) | w2[0]);
                const long a_lo = low_half ? full : 0, a_hi = low_half ? 0 : full;
                int sc_lo[4], sc_hi[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {  // scales[2t], scales[2t+1], sign-extended
                    const uint32_t word = scq[i][t >> 1];
                    sc_lo[i] = (int)(word << (24 - 16 * (t & 1))) >> 24;
                    sc_hi[i] = (int)(word << (16 - 16 * (t & 1))) >> 24;
                }
                int4v dl[TM], dh[TM];
#pragma unroll
                for (int a = 0; a < TM; ++a) {
                    const long bfrag = *(const long *)&s_xq[(16 * a + j) * XROW + 32 * t + 8 * c];
                    dl[a] = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_lo, bfrag, int4v{0, 0, 0, 0}, 0, 0, 0);
                    dh[a] = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_hi, bfrag, int4v{0, 0, 0, 0}, 0, 0, 0);
                }
#pragma unroll
                for (int a = 0; a < TM; ++a) {
                    const float dx = s_xs[(16 * a + j) * 8 + t].x;
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        part[a][i] += dx * (float)(__mul24(dh[a][i], sc_hi[i]) + __mul24(dl[a][i], sc_lo[i]));  // |dot| < 2^17
                }
            }
        }
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[a][i] += dw[i] * part[a][i];
    }
};

// Q8_0: the weights are int8 already.  A super-block is eight 34-byte blocks (272 bytes = 17 chunks, no overrun);
// the A operand of sub-block t is 8 of the block's 32 quants as they lie (2-byte aligned in the slice), and the
// rescale is acc += (d_w * d_x) * dot as vec_dot_q8_0_q8_1 does (quantized.cu:2058-2073).  The fp16 scales of a row
// are widened once per super-block by the lane that feeds the row into the A operand (row j, blocks 2c and 2c + 1)
// and handed through LDS to the lanes that own the row in the C layout, like Q4_K's factors.
struct TileQ8_0 {
    static constexpr int BLOCK = 272, SLOT = 272;
    typedef u32x4_a2 GlobalChunk;  // rows sit on 2-byte boundaries
    struct Exchange {
        float dw[8][16];  // block scale [sub-block][row]
    };
    template <int TM>
    static __device__ __forceinline__ void superblock(const uint8_t *slice, int pitch, int b, int j, int c, Exchange &ex,
                                                      const int8_t *s_xq, const float2 *s_xs, float (&acc)[TM][4]) {
        const uint8_t *wl = slice + j * pitch + SLOT * b;
        ex.dw[2 * c][j] = half_bits_to_float(*(const uint16_t *)(wl + 34 * (2 * c)));
        ex.dw[2 * c + 1][j] = half_bits_to_float(*(const uint16_t *)(wl + 34 * (2 * c + 1)));
        wave_lds_fence();
        float4 dq[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) dq[t] = *(const float4 *)&ex.dw[t][4 * c];
        wave_lds_fence();  // the slots are rewritten by the next super-block
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const u32x2 qa = *(const u32x2_a2 *)(wl + 34 * t + 2 + 8 * c);
            const long afrag = (long)(((uint64_t)qa.y << 32) | qa.x);
            const float dw[4] = {dq[t].x, dq[t].y, dq[t].z, dq[t].w};
            int4v d[TM];
#pragma unroll
            for (int a = 0; a < TM; ++a) {
                const long bfrag = *(const long *)&s_xq[(16 * a + j) * XROW + 32 * t + 8 * c];
                d[a] = __builtin_amdgcn_mfma_i32_16x16x32_i8(afrag, bfrag, int4v{0, 0, 0, 0}, 0, 0, 0);
            }
#pragma unroll
            for (int a = 0; a < TM; ++a) {
                const float dx = s_xs[(16 * a + j) * 8 + t].x;
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[a][i] += (dw[i] * dx) * (float)d[a][i];
            }
        }
    }
};

// The 32-value formats with 4- or 5-bit levels: Q4_0 (18 bytes: d, 16 bytes of nibbles), Q4_1 (20: d, m, nibbles),
// Q5_0 (22: d, 32 fifth bits, nibbles) and Q5_1 (24: d, m, fifth bits, nibbles).  Eight blocks make a super-block
// (144 / 160 / 176 / 192 bytes: whole 16-byte chunks, no overrun).  A lane's 8 values of a sub-block are the two
// nibbles of 4 consecutive bytes in candy's element order (quantized.go:85-93, 107-116: y[2j] low, y[2j+1] high) or
// one nibble of 8 consecutive bytes in ggml's (low nibbles are values 0-15, high 16-31; the only order of Q5_0 and
// Q5_1).  The level offset (-8, -16) or the block minimum goes through the activation block sum:
//   acc += d_w * (d_x * dot - OFF * d_x * bsum)        Q4_0, Q5_0   (quantized.cu:1919-1941, 2001-2025)
//   acc += d_w * (d_x * dot) + m_w * (d_x * bsum)      Q4_1, Q5_1   (quantized.cu:1947-1975, 2027-2053)
// with the exact integer sum in place of Q8_1's rounded one, like the vector kernels.
template <int BYTES, bool HAS_MIN, bool HAS_HIGH, bool GGML>
struct TileQ32 {
    static constexpr int BLOCK = 8 * BYTES, SLOT = 8 * BYTES;
    static constexpr int QH = 2 + 2 * HAS_MIN, QS = QH + 4 * HAS_HIGH;
    typedef u32x4_a2 GlobalChunk;
    struct Exchange {
        float dw[8][16];
        float mw[HAS_MIN ? 8 : 1][16];
    };
    template <int TM>
    static __device__ __forceinline__ void superblock(const uint8_t *slice, int pitch, int b, int j, int c, Exchange &ex,
                                                      const int8_t *s_xq, const float2 *s_xs, float (&acc)[TM][4]) {
        static_assert(!HAS_HIGH || GGML, "Q5_0 / Q5_1 exist in ggml's element order only");
        const uint8_t *wl = slice + j * pitch + SLOT * b;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            ex.dw[2 * c + h][j] = half_bits_to_float(*(const uint16_t *)(wl + BYTES * (2 * c + h)));
            if (HAS_MIN) ex.mw[2 * c + h][j] = half_bits_to_float(*(const uint16_t *)(wl + BYTES * (2 * c + h) + 2));
        }
        wave_lds_fence();
        float4 dq[8], mq[HAS_MIN ? 8 : 1];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            dq[t] = *(const float4 *)&ex.dw[t][4 * c];
            if (HAS_MIN) mq[t] = *(const float4 *)&ex.mw[t][4 * c];
        }
        wave_lds_fence();  // the slots are rewritten by the next super-block
        const uint32_t M = 0x0F0F0F0Fu;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const uint8_t *blk = wl + BYTES * t;
            uint32_t lo, hi;  // values 8c .. 8c+3 and 8c+4 .. 8c+7 of the sub-block, one per byte
            if (GGML) {
                const u32x2 q = *(const u32x2_a2 *)(blk + QS + 8 * (c & 1));
                const int sh = (c >> 1) * 4;
                lo = (q.x >> sh) & M;
                hi = (q.y >> sh) & M;
                if (HAS_HIGH) {
                    uint32_t qh;
                    __builtin_memcpy(&qh, blk + QH, 4);
                    lo |= q5_high4(qh, 8 * c);
                    hi |= q5_high4(qh, 8 * c + 4);
                }
            } else {
                uint32_t q;
                __builtin_memcpy(&q, blk + QS + 4 * c, 4);
                const uint32_t l = q & M, h = (q >> 4) & M;
                lo = __builtin_amdgcn_perm(h, l, 0x05010400u);  // l0 h0 l1 h1
                hi = __builtin_amdgcn_perm(h, l, 0x07030602u);  // l2 h2 l3 h3
            }
            const long afrag = (long)(((uint64_t)hi << 32) | lo);
            const float dw[4] = {dq[t].x, dq[t].y, dq[t].z, dq[t].w};
            const float4 mt = HAS_MIN ? mq[t] : make_float4(0.f, 0.f, 0.f, 0.f);
            const float mw[4] = {mt.x, mt.y, mt.z, mt.w};
            int4v d[TM];
#pragma unroll
            for (int a = 0; a < TM; ++a) {
                const long bfrag = *(const long *)&s_xq[(16 * a + j) * XROW + 32 * t + 8 * c];
                d[a] = __builtin_amdgcn_mfma_i32_16x16x32_i8(afrag, bfrag, int4v{0, 0, 0, 0}, 0, 0, 0);
            }
#pragma unroll
            for (int a = 0; a < TM; ++a) {
                const float2 sx = s_xs[(16 * a + j) * 8 + t];
                const float off = (HAS_HIGH ? -16.0f : -8.0f) * sx.y;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (HAS_MIN) acc[a][i] += dw[i] * (sx.x * (float)d[a][i]) + mw[i] * sx.y;
                    else acc[a][i] += dw[i] * (sx.x * (float)d[a][i] + off);
                }
            }
        }
    }
};
template <bool GGML> using TileQ4_0 = TileQ32<18, false, false, GGML>;
template <bool GGML> using TileQ4_1 = TileQ32<20, true, false, GGML>;
using TileQ5_0 = TileQ32<22, false, true, true>;
using TileQ5_1 = TileQ32<24, true, true, true>;

// Q2_K (84 bytes: 16 bytes of {4-bit scale, 4-bit min} per 16-value group, 64 bytes of 2-bit levels, d, dmin;
// quantized.cu:902-935).  A 32-value sub-block spans two groups with their own scale and min, but a level times
// its scale is at most 3 * 15 and fits the int8 operand: one MFMA contracts scale * level with the activations,
// a second one contracts the group's min (every value of the group carries it) with them, and the rescale is
//   acc += d * (d_x * dot) - dmin * (d_x * dot_min)
// which is vec_dot_q2_K_q8_1 (quantized.cu:2108-2135) with the sums over the group taken by the matrix core.
// Blocks are not a whole number of 16-byte chunks: the slot is 96 bytes and the last chunk runs 12 bytes into
// the next block (past the tensor's end on the last row: library-owned, padded buffers only).
struct TileQ2K {
    static constexpr int BLOCK = 84, SLOT = 96;
    typedef u32x4_a2 GlobalChunk;
    struct Exchange {};
    template <int TM>
    static __device__ __forceinline__ void superblock(const uint8_t *slice, int pitch, int b, int j, int c, Exchange &,
                                                      const int8_t *s_xq, const float2 *s_xs, float (&acc)[TM][4]) {
        const uint8_t *wl = slice + j * pitch + SLOT * b;
        float dw[4], mw[4];  // d and dmin of my four C rows
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t dm = *(const uint32_t *)(slice + (4 * c + i) * pitch + SLOT * b + 80);
            dw[i] = half_bits_to_float((uint16_t)(dm & 0xFFFF));
            mw[i] = half_bits_to_float((uint16_t)(dm >> 16));
        }
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            const u32x2 q = *(const u32x2 *)(wl + 16 + 32 * n + 8 * c);  // levels of values 8c .. 8c+7 of four sub-blocks
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int t = 4 * n + k;
                const uint32_t sm = wl[2 * t + (c >> 1)];  // my group's {scale, min}
                const uint32_t sc = sm & 0xF, mn = (sm >> 4) * 0x01010101u;
                const uint32_t lo = ((q.x >> (2 * k)) & 0x03030303u) * sc, hi = ((q.y >> (2 * k)) & 0x03030303u) * sc;
                const long afrag = (long)(((uint64_t)hi << 32) | lo), mfrag = (long)(((uint64_t)mn << 32) | mn);
                int4v d[TM], dm[TM];
#pragma unroll
                for (int a = 0; a < TM; ++a) {
                    const long bfrag = *(const long *)&s_xq[(16 * a + j) * XROW + 32 * t + 8 * c];
                    d[a] = __builtin_amdgcn_mfma_i32_16x16x32_i8(afrag, bfrag, int4v{0, 0, 0, 0}, 0, 0, 0);
                    dm[a] = __builtin_amdgcn_mfma_i32_16x16x32_i8(mfrag, bfrag, int4v{0, 0, 0, 0}, 0, 0, 0);
                }
#pragma unroll
                for (int a = 0; a < TM; ++a) {
                    const float dx = s_xs[(16 * a + j) * 8 + t].x;
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[a][i] += dw[i] * (dx * (float)d[a][i]) - mw[i] * (dx * (float)dm[a][i]);
                }
            }
        }
    }
};

// Q3_K (110 bytes: 32 mask bytes, 64 bytes of 2-bit levels, 12 bytes of 6-bit scales, d; quantized.cu:938-990).
// A value is d * (scale - 32) * (level - 4) with level = two bits | mask bit << 2.  (32 - scale) * (level - 4) lies
// in [-128, 124] and fits the int8 operand ((scale - 32) * (level - 4) would reach +128), so one MFMA per sub-block
// contracts it with the activations and the rescale is acc -= d * (d_x * dot): vec_dot_q3_K_q8_1
// (quantized.cu:2177-2209) with the scale folded into the operand.  The four signed bytes of a word are multiplied
// by the group's factor as two pairs of 16-bit lanes.  Slot of 112 bytes: the last chunk runs 2 bytes into the next
// block (library-owned, padded buffers only).
typedef short short2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t mul_s8x4(uint32_t w, int f) {  // four signed bytes times f, products within int8
    short2v ws;
    __builtin_memcpy(&ws, &w, 4);
    const short2v sh8 = {8, 8}, ff = {(short)f, (short)f};
    const short2v pe = ((ws << sh8) >> sh8) * ff, po = (ws >> sh8) * ff;  // bytes 0 and 2, bytes 1 and 3
    uint32_t e, o;
    __builtin_memcpy(&e, &pe, 4);
    __builtin_memcpy(&o, &po, 4);
    return __builtin_amdgcn_perm(o, e, 0x06020400u);
}
struct TileQ3K {
    static constexpr int BLOCK = 110, SLOT = 112;
    typedef u32x4_a2 GlobalChunk;
    struct Exchange {};
    template <int TM>
    static __device__ __forceinline__ void superblock(const uint8_t *slice, int pitch, int b, int j, int c, Exchange &,
                                                      const int8_t *s_xq, const float2 *s_xs, float (&acc)[TM][4]) {
        const uint8_t *wl = slice + j * pitch + SLOT * b;
        float dw[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) dw[i] = half_bits_to_float(*(const uint16_t *)(slice + (4 * c + i) * pitch + SLOT * b + 108));
        const u32x2 hm = *(const u32x2 *)(wl + 8 * c);  // mask bytes of values 8c .. 8c+7: bit t belongs to sub-block t
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            const u32x2 q = *(const u32x2 *)(wl + 32 + 32 * n + 8 * c);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int t = 4 * n + k;
                const int f = 32 - q3k_scale6(wl + 96, 2 * t + (c >> 1));
                uint32_t lev[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const uint32_t raw = ((q[e] >> (2 * k)) & 0x03030303u) | (((hm[e] >> t) & 0x01010101u) << 2);  // 0 .. 7
                    lev[e] = ((raw | 0x80808080u) - 0x04040404u) ^ 0x80808080u;                                 // - 4, bytewise
                }
                const uint32_t lo = mul_s8x4(lev[0], f), hi = mul_s8x4(lev[1], f);
                const long afrag = (long)(((uint64_t)hi << 32) | lo);
                int4v d[TM];
#pragma unroll
                for (int a = 0; a < TM; ++a) {
                    const long bfrag = *(const long *)&s_xq[(16 * a + j) * XROW + 32 * t + 8 * c];
                    d[a] = __builtin_amdgcn_mfma_i32_16x16x32_i8(afrag, bfrag, int4v{0, 0, 0, 0}, 0, 0, 0);
                }
#pragma unroll
                for (int a = 0; a < TM; ++a) {
                    const float dx = s_xs[(16 * a + j) * 8 + t].x;
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[a][i] -= dw[i] * (dx * (float)d[a][i]);
                }
            }
        }
    }
};

// ---------------------------------------------------------------------------------------------
// LDS carve-up of k_mmq_i8 (dynamic: the K-split variant needs more than the 64 KB a static layout may take)
template <class F, int TM, int STG, int KS>
struct MmqI8Lds {
    static constexpr int BM = 16 * TM;
    static constexpr int WPITCH = STG * F::SLOT + (((STG * F::SLOT / 16) & 1) ? 32 : 16);
    static constexpr int XS = TM <= 2 ? STG : 1;
    static constexpr int XQ = XS * BM * XROW;                         // activation quants of one K group
    static constexpr int XSS = XS * BM * 8 * (int)sizeof(float2);     // their {d, d * bsum}
    static constexpr int SW = 16 * WPITCH;                            // one wavefront's weight slice
    static constexpr int EX = ((int)sizeof(typename F::Exchange) + 15) & ~15;
    static constexpr int PART = KS > 1 ? 4 * 64 * TM * 4 * (int)sizeof(float) : 0;
    static constexpr int BYTES = KS * (XQ + XSS) + 4 * KS * (SW + EX) + PART;
};

// KS = 2: eight wavefronts, the second four walk the second half of K for the same 64 weight rows (a grid of
// few workgroups leaves one wavefront per SIMD, which waits out every latency of its own instruction stream);
// the halves are added through LDS, first half + second half.
template <class F, int TM, int STG, int KS>
__global__ __launch_bounds__(256 * KS) void k_mmq_i8(const uint8_t *__restrict__ W, const int8_t *__restrict__ xq,
                                                     const Q8Scale *__restrict__ xs, float *__restrict__ y, int N, int M,
                                                     int K, int sb_split) {
    typedef MmqI8Lds<F, TM, STG, KS> L;
    constexpr int BM = 16 * TM;
    constexpr int XSC = (BM * 8 + 255) / 256;  // activation scales per thread per super-block
    // slice pitch: an odd multiple of 16 bytes, so the 16 rows of an 8-byte pick fall in distinct banks
    constexpr int WPITCH = STG * F::SLOT + (((STG * F::SLOT / 16) & 1) ? 32 : 16);
    static_assert((WPITCH / 16) % 2 == 1, "pitch must be an odd number of 16-byte units");
    // few activation rows (TM <= 2): a super-block's work is too short to cover the latency of the next one's
    // activation loads, so the tile holds a whole stage and is refilled once per stage, a stage ahead
    constexpr int XS = TM <= 2 ? STG : 1;                       // super-blocks of activations in the tile
    static_assert(KS == 1 || XS > 1, "the K split goes with the stage-wide activation tile");
    static_assert(WPITCH == L::WPITCH && XS == L::XS, "layout");
    extern __shared__ __align__(16) uint8_t smem_i8[];
    const int kg = threadIdx.x >> 8;                     // K group of this thread
    const int tid = threadIdx.x & 255, lane = tid & 63, wave = tid >> 6, gw = threadIdx.x >> 6;
    int8_t *s_xq = (int8_t *)smem_i8 + kg * L::XQ;                                  // [XS][BM][XROW]
    float2 *s_xs = (float2 *)(smem_i8 + KS * L::XQ + kg * L::XSS);                  // {d, d * bsum} [XS][BM][8]
    uint8_t *s_wm = smem_i8 + KS * (L::XQ + L::XSS) + gw * L::SW;                   // this wavefront's weight rows
    typename F::Exchange &s_exm = *(typename F::Exchange *)(smem_i8 + KS * (L::XQ + L::XSS) + 4 * KS * L::SW + gw * L::EX);
    float *s_part = (float *)(smem_i8 + KS * (L::XQ + L::XSS) + 4 * KS * (L::SW + L::EX));

    const int j = lane & 15, c = lane >> 4;
    const int n0 = blockIdx.x * 64 + wave * 16, m0 = blockIdx.y * BM;
    const int nsb = K >> 8;
    const size_t rb = (size_t)nsb * F::BLOCK;
    // the super-blocks of this K group: [sb_lo, sb_hi), `per` (whole stages) for every group
    // blockIdx.z walks super-blocks [z * sb_split, ...) and writes its own copy of the output (summed afterwards)
    const int sb_first = blockIdx.z * sb_split, sb_end = min(nsb, sb_first + sb_split);
    const int per = ((sb_end - sb_first + KS - 1) / KS + STG - 1) / STG * STG;
    const int sb_lo = sb_first + kg * per, sb_hi = min(sb_end, sb_lo + per);
    y += (size_t)blockIdx.z * M * N;

    // weights of one stage: 16 rows x STG blocks as 16-byte chunks along the rows, in registers
    // while in flight, then parked in the wavefront's LDS slice
    constexpr int CPB = F::SLOT / 16;           // chunks per block
    constexpr int CPR = CPB * STG;              // chunks per row per stage
    constexpr int WCH = (16 * CPR + 63) / 64;   // chunks per lane
    u32x4 wr[WCH];
    auto load_stage = [&](int s0) {
#pragma unroll
        for (int i = 0; i < WCH; ++i) {
            const int q = min(lane + 64 * i, 16 * CPR - 1), row = q / CPR, col = q % CPR;
            const int sb = min(s0 + col / CPB, nsb - 1);
            wr[i] = *(const typename F::GlobalChunk *)(W + (size_t)min(n0 + row, N - 1) * rb + (size_t)sb * F::BLOCK +
                                                       (col % CPB) * 16);
        }
    };
    auto park_stage = [&]() {
#pragma unroll
        for (int i = 0; i < WCH; ++i) {
            const int q = lane + 64 * i, row = q / CPR, col = q % CPR;
            if ((16 * CPR) % 64 == 0 || q < 16 * CPR) *(u32x4 *)&s_wm[row * WPITCH + col * 16] = wr[i];
        }
    };
    // activations of one super-block: registers first (loaded a super-block ahead), then LDS
    u32x4 xr[XS][TM];
    float xsd[XS][XSC];
    int xsb[XS][XSC];
    auto load_x = [&](int s, int slot) __attribute__((always_inline)) {
        const int sb = min(s, nsb - 1);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int q = tid + i * 256, row = q >> 4, col = q & 15;
            xr[slot][i] = *(const u32x4 *)(xq + (size_t)min(m0 + row, M - 1) * K + (size_t)sb * 256 + col * 16);
        }
#pragma unroll
        for (int i = 0; i < XSC; ++i) {
            const int e = min(tid + i * 256, BM * 8 - 1), row = e >> 3, t = e & 7;
            const Q8Scale v = xs[(size_t)min(m0 + row, M - 1) * (K >> 5) + sb * 8 + t];
            xsd[slot][i] = v.d;
            xsb[slot][i] = v.bsum;
        }
    };
    auto park_x = [&](int slot) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int q = tid + i * 256, row = q >> 4, col = q & 15;
            *(u32x4 *)&s_xq[slot * BM * XROW + row * XROW + col * 16] = xr[slot][i];
        }
#pragma unroll
        for (int i = 0; i < XSC; ++i) {
            const int e = tid + i * 256;
            if (BM * 8 % 256 == 0 || e < BM * 8) s_xs[slot * BM * 8 + e] = make_float2(xsd[slot][i], xsd[slot][i] * (float)xsb[slot][i]);
        }
    };

#pragma unroll
    for (int b = 0; b < XS; ++b) load_x(sb_lo + b, b);
    load_stage(sb_lo);

    float acc[TM][4];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[a][i] = 0.0f;

    for (int it = 0; it < per; it += STG) {  // the same trip count in every K group: the barriers are workgroup-wide
        const int s0 = sb_lo + it;
        wave_lds_fence();  // this wavefront is done reading the previous stage
        park_stage();
        load_stage(s0 + STG);
        wave_lds_fence();
        if constexpr (XS > 1) {
#pragma unroll
            for (int b = 0; b < STG; ++b) park_x(b);
            __syncthreads();
#pragma unroll
            for (int b = 0; b < STG; ++b) load_x(s0 + STG + b, b);  // the next stage's activations fly under this stage
#pragma unroll
            for (int b = 0; b < STG; ++b)
                if (s0 + b < sb_hi)  // uniform over the wavefront
                    F::template superblock<TM>(s_wm, WPITCH, b, j, c, s_exm, s_xq + b * BM * XROW, s_xs + b * BM * 8, acc);
            __syncthreads();  // the activation tile is rewritten next
        } else {
#pragma unroll
            for (int b = 0; b < STG; ++b) {
                const int s = s0 + b;
                if (s < sb_hi) {  // uniform
                    park_x(0);
                    __syncthreads();
                    load_x(s + 1, 0);  // the next super-block's activations fly under this one's MFMAs
                    F::template superblock<TM>(s_wm, WPITCH, b, j, c, s_exm, s_xq, s_xs, acc);
                    __syncthreads();  // the activation tile is rewritten next
                }
            }
        }
    }

    if constexpr (KS > 1) {  // second half of K handed to the first through LDS
        float4 *slot = (float4 *)s_part + (wave * 64 + lane) * TM;
        if (kg == 1) {
#pragma unroll
            for (int a = 0; a < TM; ++a) slot[a] = make_float4(acc[a][0], acc[a][1], acc[a][2], acc[a][3]);
        }
        __syncthreads();
        if (kg == 1) return;
#pragma unroll
        for (int a = 0; a < TM; ++a) {
            const float4 o = slot[a];
            acc[a][0] += o.x; acc[a][1] += o.y; acc[a][2] += o.z; acc[a][3] += o.w;
        }
    }
    // C layout: lane holds activation row j of each m-tile and weight rows 4c .. 4c+3
#pragma unroll
    for (int a = 0; a < TM; ++a) {
        const int m = m0 + 16 * a + j, n = n0 + 4 * c;
        if (m >= M) continue;
        float *dst = y + (size_t)m * N + n;
        if (n + 3 < N && (N & 3) == 0) {
            *(float4 *)dst = make_float4(acc[a][0], acc[a][1], acc[a][2], acc[a][3]);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (n + i < N) dst[i] = acc[a][i];
        }
    }
}

template <class F>
static int launch_i8(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales,
                     int64_t m, float *y) {
    const int N = (int)w->rows, K = (int)w->cols, M = (int)m;
    const unsigned gx = (unsigned)((N + 63) / 64);
#define CANDY_MMQ_I8(TMV, STGV, KSV)                                                                            \
    do {                                                                                                        \
        constexpr int lds = MmqI8Lds<F, TMV, STGV, KSV>::BYTES;                                                 \
        auto kern = k_mmq_i8<F, TMV, STGV, KSV>;                                                                \
        CANDY_HIP_TRY(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds)); \
        const unsigned gy = (unsigned)((M + 16 * TMV - 1) / (16 * TMV));                                          \
        /* a wavefront walks its share of K alone, about 1.3 us per super-block, and LDS lets two of them share a */ \
        /* SIMD: a grid of at most one per SIMD splits K over workgroups up to two per SIMD, at least one stage   */ \
        /* per K group each; the copies are added in a fixed order by k_splitk_sum                                 */ \
        const int64_t waves = (int64_t)gx * gy * 4 * KSV, simds = 4 * (int64_t)dev->num_cus;                       \
        if (!no_gs && waves <= simds) n_split = (int)std::min<int64_t>(2 * simds / waves, nsb / (STGV * KSV));     \
        if (n_split < 1) n_split = 1;                                                                             \
        sb_split = (nsb + n_split - 1) / n_split;                                                                 \
        n_split = (nsb + sb_split - 1) / sb_split;                                                                \
        if (n_split > 1) {                                                                                        \
            void *p = nullptr;                                                                                    \
            if (int rc = splitk_workspace(dev, (size_t)n_split * (size_t)M * N * sizeof(float), &p)) return rc;   \
            out = (float *)p;                                                                                     \
        }                                                                                                         \
        hipLaunchKernelGGL(kern, dim3(gx, gy, (unsigned)n_split), dim3(256 * KSV), lds, dev->stream,              \
                           (const uint8_t *)w->data, qs, scales, out, N, M, K, sb_split);                         \
    } while (0)
    // Tile height: 64 activation rows per workgroup from 33 rows on (a weight fragment serves four MFMAs), 16 below
    // that; one super-block per stage and four wavefronts per workgroup throughout.  Where the grid is at most one
    // wavefront per SIMD the launch macro splits K over workgroups.  Measured on 4096x11008, 11008x4096, 4096x4096
    // and 14336x4096 at 8 .. 255 rows for Q4_K, Q6_K and Q8_0: deeper stages (2 or 4 super-blocks in flight per
    // wavefront) and a K split inside an eight-wavefront workgroup, both of which helped before the split over
    // workgroups existed, now cost 1-10 % (Q6_K at 64-row tiles: 25 %); 32-row tiles won nowhere.
    const bool no_gs = dev->opt.i8_grid_split == 0;  // comparison runs and tests
    const int nsb = K >> 8;
    int n_split = 1, sb_split = nsb;
    float *out = y;
    if (M > 32) CANDY_MMQ_I8(4, 1, 1);
    else CANDY_MMQ_I8(1, 1, 1);
#undef CANDY_MMQ_I8
    CANDY_LAUNCH_CHECK();
    if (n_split > 1) return launch_splitk_sum(dev, out, y, nullptr, (size_t)M * N, n_split);
    return CANDY_HIP_OK;
}

bool mmq_i8_covers(const candy_hip_qtensor *w, const int8_t *qs) {
    if (((uintptr_t)qs & 15) != 0 || w->cols % 256 != 0) return false;
    if (w->fmt == CANDY_HIP_Q4_K || w->fmt == CANDY_HIP_Q5_K) return ((uintptr_t)w->data & 15) == 0;
    // the last chunk of a Q6_K row runs 14 bytes past the block: only buffers known to have that room after the
    // last row (allocated by the library, which pads them, or wrapped with a size that says so)
    if (w->fmt == CANDY_HIP_Q6_K || w->fmt == CANDY_HIP_Q2_K || w->fmt == CANDY_HIP_Q3_K) return w->padded && ((uintptr_t)w->data & 1) == 0;
    switch (w->fmt) {
    case CANDY_HIP_Q8_0: case CANDY_HIP_Q4_0: case CANDY_HIP_Q4_0_GGML: case CANDY_HIP_Q4_1: case CANDY_HIP_Q4_1_GGML:
    case CANDY_HIP_Q5_0: case CANDY_HIP_Q5_1:
        return ((uintptr_t)w->data & 1) == 0;
    default:
        break;
    }
    return false;
}

int launch_mmq_i8(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales,
                  int64_t m, float *y) {
    if (w->fmt == CANDY_HIP_Q8_0) return launch_i8<TileQ8_0>(dev, w, qs, scales, m, y);
    if (w->fmt == CANDY_HIP_Q5_K) return launch_i8<TileQ5K>(dev, w, qs, scales, m, y);
    if (w->fmt == CANDY_HIP_Q2_K) return launch_i8<TileQ2K>(dev, w, qs, scales, m, y);
    if (w->fmt == CANDY_HIP_Q3_K) return launch_i8<TileQ3K>(dev, w, qs, scales, m, y);
    if (w->fmt == CANDY_HIP_Q4_0) return launch_i8<TileQ4_0<false>>(dev, w, qs, scales, m, y);
    if (w->fmt == CANDY_HIP_Q4_0_GGML) return launch_i8<TileQ4_0<true>>(dev, w, qs, scales, m, y);
    if (w->fmt == CANDY_HIP_Q4_1) return launch_i8<TileQ4_1<false>>(dev, w, qs, scales, m, y);
    if (w->fmt == CANDY_HIP_Q4_1_GGML) return launch_i8<TileQ4_1<true>>(dev, w, qs, scales, m, y);
    if (w->fmt == CANDY_HIP_Q5_0) return launch_i8<TileQ5_0>(dev, w, qs, scales, m, y);
    if (w->fmt == CANDY_HIP_Q5_1) return launch_i8<TileQ5_1>(dev, w, qs, scales, m, y);
    return w->fmt == CANDY_HIP_Q4_K ? launch_i8<TileQ4K>(dev, w, qs, scales, m, y)
                                    : launch_i8<TileQ6K>(dev, w, qs, scales, m, y);
}

}  // namespace candy
