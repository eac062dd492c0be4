// Prompt-sized batches of Q4_K, Q5_K, Q6_K, Q8_0 and Q4_0 on the fp16 matrix cores: y[m, N] = x[m, K] . W^T.
//
// Replaces mul_mat_q / load_tiles_q4_K / load_tiles_q6_K (tensor/internal/cuda/kernels/quantized.cu
// :455-578, :4116-4205) for prompt-sized batches.  With hundreds of activation rows the contraction
// is a dense GEMM, and the per-sub-block rescale that keeps the integer kernel exact costs several
// times the matrix-core time; here the scales are folded into the operands instead:
//   * weights are dequantized exactly as dequantize_block_q4_K / dequantize_block_q6_K do
//     (quantized.cu:1008-1041: (d*sc)*q - dmin*m; :1103-1128: d*sc*(q-32); evaluated in f32) and
//     rounded once to fp16;
//   * activations are the Q8_0 values d_x * q_x (exact in f32) rounded once to fp16;
//   * products accumulate in f32 (v_mfma_f32_16x16x32_f16).
// Both roundings are 2^-12 relative per element; the result stays a few 1e-4 (max-norm) from the
// CPU contraction, inside the 1e-3 bar.
//
// Tiling: a workgroup owns 128 weight rows x 256 (or 128) activation rows and walks K in steps of 64.
//   k_mmq_f16_pc (what runs): four producer wavefronts dequantize 16 weights per thread and step into an LDS tile
//     (two or three buffers, one barrier per step); four consumer wavefronts read the weight fragments from LDS,
//     load their activation fragments straight from memory into operand registers (the fp16 image is stored
//     fragment by fragment, xh_index4) and issue the matrix instructions.
//   k_mmq_f16 (comparison: option mmq.f16_shape 3): every wavefront dequantizes, copies activations into a second LDS
//     tile and multiplies a 64 x 64 sub-tile.
// Global requests run ahead in registers: a thread's share of a whole super-block of weights four steps ahead
// (HBM), the activations one or two steps ahead (L2).  Workgroups are numbered so that those sharing an XCD (and its
// L2) work on neighbouring weight tiles of the same activation tile.  When the output has too few tiles to fill the
// chip (N = 4096 or 1024 projections), K is split over several workgroups per tile; their partial sums go to a
// scratch buffer and a second kernel adds them in a fixed order (bitwise reproducible).  One launch can serve up to
// three weight tensors that share their activations (q / k / v, gate / up).
#include <algorithm>
#include <cstdlib>
#include <type_traits>

#include "blocks.h"
#include "internal.h"

namespace candy {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ half2v bits_h2(uint32_t u) { return __builtin_bit_cast(half2v, u); }

constexpr int BIG_BK = 64;
// LDS tiles are stored as the matrix instruction reads them: a fragment of 16 rows x 32 values of K is 1 KB, its
// 16-byte pieces (8 values of K of one row) in the order lane = 16 * (piece of K) + row, so that a wavefront's
// operand read is 64 consecutive pieces.  (With rows laid end to end, padded or not, the 8 lanes of a group
// straddle both halves of the 64 banks and every 128-bit read takes close to twice the cycles; measured with a
// read-only probe: 2.8 against 4.7 ticks per instruction at 16 wavefronts.)  Offset in halves of piece (row, k):
__device__ __forceinline__ int frag_off(int row, int k) {
    const int piece = (k >> 3) & 3;
    return (((row >> 4) * 2 + (k >> 5)) << 9) + (((piece << 4) + ((row & 15) ^ piece)) << 3);
}
// ... and of the piece lane `lane` of a wavefront reads from a fragment
__device__ __forceinline__ int frag_lane_off(int lane) { return (((lane >> 4) << 4) + ((lane & 15) ^ (lane >> 4))) << 3; }

// ------------------------------------------------------------------ per-format policies
// A task is (row, quarter c in 0..3) of one 64-wide step g in 0..3 of a super-block: 16 weights.
//   load():    the task's bytes of a whole super-block -> registers (requested four steps ahead)
//   dequant(): step g's 16 weights as two 8-value chunks and their positions (in halves) in the
//              64-wide LDS row

struct BigQ4K {
    static constexpr int BLOCK = 144;
    struct Raw { u32x4 hdr; u32x2 q[4]; };  // header + bytes 8c..8c+7 of each 32-byte nibble group
    __device__ static __forceinline__ void load(const uint8_t *blk, int c, Raw &r) {
        r.hdr = *(const u32x4 *)blk;
#pragma unroll
        for (int g = 0; g < 4; ++g) r.q[g] = *(const u32x2 *)(blk + 16 + g * 32 + c * 8);
    }
    // group g holds sub-blocks 2g (low nibbles, k = 0..31 of the step) and 2g+1 (high nibbles, k = 32..63).
    // A nibble n is placed in the mantissa of the half 1024 (bits 0x6400 | n = 1024 + n, exact), two nibbles per
    // instruction, and each value is one mixed-precision multiply-add (f16 operand, f32 scale and offset, f32
    // arithmetic, rounded once to fp16): (1024 + n) * (d*sc) + (-(dmin*m) - 1024 * (d*sc)) = (d*sc)*n - dmin*m.
    // High nibbles stay where they are, four bits up (0x6400 | 16 n = 1024 + 16 n, exact as well), and take the
    // scale d*sc / 16 and the offset -(dmin*m) - 64 * (d*sc): one shift per word instead of three.
    // The offset's own f32 rounding (2^-24 of 1024 d*sc) is a thirtieth of the fp16 rounding that follows.
    __device__ static __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t bits) {
        uint32_t r;  // (x & mask) | bits in one instruction; the mask rides on the constant bus, the bits in a register
        asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(mask), "v"(bits));
        return r;
    }
    __device__ static __forceinline__ void dequant(const Raw &r, int g, int c, half8 &o0, half8 &o1, int &k0, int &k1) {
        uint32_t sc2, m2;
        q4k_scale_min_pair(r.hdr.y, r.hdr.z, r.hdr.w, g, sc2, m2);
        const float d = half_bits_to_float((uint16_t)(r.hdr.x & 0xFFFF));
        const float dmin = half_bits_to_float((uint16_t)(r.hdr.x >> 16));
        const float d_lo = d * (float)(sc2 & 0xFF), d_hi = d * (float)((sc2 >> 8) & 0xFF);
        const float c_lo = fmaf(-1024.0f, d_lo, -(dmin * (float)(m2 & 0xFF)));
        const float c_hi = fmaf(-64.0f, d_hi, -(dmin * (float)((m2 >> 8) & 0xFF)));
        const float d_hi16 = d_hi * 0.0625f;
        const u32x2 q = r.q[g];
        const uint32_t MAGIC = 0x64006400u, LO = 0x000F000Fu, HI = 0x00F000F0u;
#pragma unroll
        for (int wi = 0; wi < 2; ++wi) {
            const uint32_t w = wi ? q.y : q.x, w8 = w >> 8;
            const half2v l02 = bits_h2(and_or(w, LO, MAGIC)), l13 = bits_h2(and_or(w8, LO, MAGIC));
            const half2v h02 = bits_h2(and_or(w, HI, MAGIC)), h13 = bits_h2(and_or(w8, HI, MAGIC));
            o0[4 * wi + 0] = (_Float16)fmaf((float)l02[0], d_lo, c_lo);
            o0[4 * wi + 1] = (_Float16)fmaf((float)l13[0], d_lo, c_lo);
            o0[4 * wi + 2] = (_Float16)fmaf((float)l02[1], d_lo, c_lo);
            o0[4 * wi + 3] = (_Float16)fmaf((float)l13[1], d_lo, c_lo);
            o1[4 * wi + 0] = (_Float16)fmaf((float)h02[0], d_hi16, c_hi);
            o1[4 * wi + 1] = (_Float16)fmaf((float)h13[0], d_hi16, c_hi);
            o1[4 * wi + 2] = (_Float16)fmaf((float)h02[1], d_hi16, c_hi);
            o1[4 * wi + 3] = (_Float16)fmaf((float)h13[1], d_hi16, c_hi);
        }
        k0 = c * 8;
        k1 = 32 + c * 8;
    }
    // The same in two parts for the kernel whose four neighbouring lanes hold the four quarters of one row: the scale
    // and offset of group g are the same for all four, so lane c works out those of group c once per super-block
    // (prepare) and each step fetches its group's from the lane that has them (four cross-lane moves instead of the
    // unpacking and six multiplies).  The same operations on the same values as dequant(): the same bits.
    struct Pre { float d_lo, d_hi16, c_lo, c_hi; };
    __device__ static __forceinline__ void prepare(const Raw &r, int c, Pre &p) {
        uint32_t sc2, m2;
        q4k_scale_min_pair(r.hdr.y, r.hdr.z, r.hdr.w, c, sc2, m2);
        const float d = half_bits_to_float((uint16_t)(r.hdr.x & 0xFFFF));
        const float dmin = half_bits_to_float((uint16_t)(r.hdr.x >> 16));
        const float d_lo = d * (float)(sc2 & 0xFF), d_hi = d * (float)((sc2 >> 8) & 0xFF);
        p.c_lo = fmaf(-1024.0f, d_lo, -(dmin * (float)(m2 & 0xFF)));
        p.c_hi = fmaf(-64.0f, d_hi, -(dmin * (float)((m2 >> 8) & 0xFF)));
        p.d_lo = d_lo;
        p.d_hi16 = d_hi * 0.0625f;
    }
    __device__ static __forceinline__ float quad_lane(float v, int g) {  // the value lane g of this lane's quad holds
        switch (g) {
        case 0: return dpp_move<0x00>(v);
        case 1: return dpp_move<0x55>(v);
        case 2: return dpp_move<0xAA>(v);
        default: return dpp_move<0xFF>(v);
        }
    }
    __device__ static __forceinline__ void dequant_pre(const Raw &r, const Pre &p, int g, int c, half8 &o0, half8 &o1,
                                                       int &k0, int &k1) {
        const float d_lo = quad_lane(p.d_lo, g), d_hi16 = quad_lane(p.d_hi16, g);
        const float c_lo = quad_lane(p.c_lo, g), c_hi = quad_lane(p.c_hi, g);
        const u32x2 q = r.q[g];
        const uint32_t MAGIC = 0x64006400u, LO = 0x000F000Fu, HI = 0x00F000F0u;
#pragma unroll
        for (int wi = 0; wi < 2; ++wi) {
            const uint32_t w = wi ? q.y : q.x, w8 = w >> 8;
            const half2v l02 = bits_h2(and_or(w, LO, MAGIC)), l13 = bits_h2(and_or(w8, LO, MAGIC));
            const half2v h02 = bits_h2(and_or(w, HI, MAGIC)), h13 = bits_h2(and_or(w8, HI, MAGIC));
            o0[4 * wi + 0] = (_Float16)fmaf((float)l02[0], d_lo, c_lo);
            o0[4 * wi + 1] = (_Float16)fmaf((float)l13[0], d_lo, c_lo);
            o0[4 * wi + 2] = (_Float16)fmaf((float)l02[1], d_lo, c_lo);
            o0[4 * wi + 3] = (_Float16)fmaf((float)l13[1], d_lo, c_lo);
            o1[4 * wi + 0] = (_Float16)fmaf((float)h02[0], d_hi16, c_hi);
            o1[4 * wi + 1] = (_Float16)fmaf((float)h13[0], d_hi16, c_hi);
            o1[4 * wi + 2] = (_Float16)fmaf((float)h02[1], d_hi16, c_hi);
            o1[4 * wi + 3] = (_Float16)fmaf((float)h13[1], d_hi16, c_hi);
        }
        k0 = c * 8;
        k1 = 32 + c * 8;
    }
};

// Q5_K: Q4_K's layout with 32 bytes of fifth bits between the header and the nibbles (quantized.cu:1044-1080):
// bit t of byte l is the fifth bit of value l of sub-block t.
struct BigQ5K {
    static constexpr int BLOCK = 176;
    struct Raw { u32x4 hdr; u32x2 qh; u32x2 q[4]; };
    __device__ static __forceinline__ void load(const uint8_t *blk, int c, Raw &r) {
        r.hdr = *(const u32x4 *)blk;
        r.qh = *(const u32x2 *)(blk + 16 + c * 8);
#pragma unroll
        for (int g = 0; g < 4; ++g) r.q[g] = *(const u32x2 *)(blk + 48 + g * 32 + c * 8);
    }
    __device__ static __forceinline__ void dequant(const Raw &r, int g, int c, half8 &o0, half8 &o1, int &k0, int &k1) {
        uint32_t sc2, m2;
        q4k_scale_min_pair(r.hdr.y, r.hdr.z, r.hdr.w, g, sc2, m2);
        const float d = half_bits_to_float((uint16_t)(r.hdr.x & 0xFFFF));
        const float dmin = half_bits_to_float((uint16_t)(r.hdr.x >> 16));
        const float d_lo = d * (float)(sc2 & 0xFF), d_hi = d * (float)((sc2 >> 8) & 0xFF);
        const float m_lo = dmin * (float)(m2 & 0xFF), m_hi = dmin * (float)((m2 >> 8) & 0xFF);
        const u32x2 q = r.q[g];
#pragma unroll
        for (int l = 0; l < 8; ++l) {
            const uint32_t byte = ((l < 4 ? q.x : q.y) >> (8 * (l & 3))) & 0xFF;
            const uint32_t hb = ((l < 4 ? r.qh.x : r.qh.y) >> (8 * (l & 3))) & 0xFF;
            o0[l] = (_Float16)(d_lo * (float)((byte & 0xF) | (((hb >> (2 * g)) & 1) << 4)) - m_lo);
            o1[l] = (_Float16)(d_hi * (float)((byte >> 4) | (((hb >> (2 * g + 1)) & 1) << 4)) - m_hi);
        }
        k0 = c * 8;
        k1 = 32 + c * 8;
    }
};

// Q8_0: a "super-block" is eight 34-byte blocks (272 bytes); step g holds blocks 2g and 2g + 1, the task's quarter c
// the 16 quants of half a block and that block's scale.  d * q is exact in f32 (DequantizeBlockQ8_0F32,
// quantized.go:131-136), one rounding to fp16.
struct BigQ8_0 {
    static constexpr int BLOCK = 272;
    struct Raw { u32x4 q[4]; uint32_t d01, d23; };
    __device__ static __forceinline__ void load(const uint8_t *blk, int c, Raw &r) {
        uint32_t d[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const uint8_t *b = blk + 34 * (2 * g + (c >> 1));
            d[g] = *(const uint16_t *)b;
            r.q[g] = *(const u32x4_a2 *)(b + 2 + 16 * (c & 1));
        }
        r.d01 = d[0] | (d[1] << 16);
        r.d23 = d[2] | (d[3] << 16);
    }
    __device__ static __forceinline__ void dequant(const Raw &r, int g, int c, half8 &o0, half8 &o1, int &k0, int &k1) {
        const uint32_t dd = g < 2 ? r.d01 : r.d23;
        const float d = half_bits_to_float((uint16_t)((dd >> (16 * (g & 1))) & 0xFFFF));
        const uint32_t w[4] = {r.q[g].x, r.q[g].y, r.q[g].z, r.q[g].w};
#pragma unroll
        for (int l = 0; l < 8; ++l) {
            o0[l] = (_Float16)(d * (float)(int)(int8_t)((w[l >> 2] >> (8 * (l & 3))) & 0xFF));
            o1[l] = (_Float16)(d * (float)(int)(int8_t)((w[2 + (l >> 2)] >> (8 * (l & 3))) & 0xFF));
        }
        k0 = 32 * (c >> 1) + 16 * (c & 1);
        k1 = k0 + 8;
    }
};

// Q4_0: eight 18-byte blocks per "super-block" (144 bytes).  The task's 16 values of block 2g + c/2 are the two
// nibbles of 8 consecutive bytes in candy's element order (quantized.go:85-93) or one nibble of all 16 bytes in
// ggml's.  d * (q - 8) is exact in f32, one rounding to fp16.
template <bool GGML>
struct BigQ4_0 {
    static constexpr int BLOCK = 144;
    struct Raw { u32x4 q[4]; uint32_t d01, d23; };
    __device__ static __forceinline__ void load(const uint8_t *blk, int c, Raw &r) {
        uint32_t d[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const uint8_t *b = blk + 18 * (2 * g + (c >> 1));
            d[g] = *(const uint16_t *)b;
            if (GGML) {
                r.q[g] = *(const u32x4_a2 *)(b + 2);
            } else {
                const u32x2 h = *(const u32x2_a2 *)(b + 2 + 8 * (c & 1));
                r.q[g] = u32x4{h.x, h.y, 0u, 0u};
            }
        }
        r.d01 = d[0] | (d[1] << 16);
        r.d23 = d[2] | (d[3] << 16);
    }
    __device__ static __forceinline__ void dequant(const Raw &r, int g, int c, half8 &o0, half8 &o1, int &k0, int &k1) {
        const uint32_t dd = g < 2 ? r.d01 : r.d23;
        const float d = half_bits_to_float((uint16_t)((dd >> (16 * (g & 1))) & 0xFFFF));
        const uint32_t w[4] = {r.q[g].x, r.q[g].y, r.q[g].z, r.q[g].w};
#pragma unroll
        for (int l = 0; l < 8; ++l) {
            int q0, q1;  // values l and 8 + l of the task's sixteen
            if (GGML) {
                const int sh = 4 * (c & 1);
                q0 = (int)((w[l >> 2] >> (8 * (l & 3) + sh)) & 0xF);
                q1 = (int)((w[2 + (l >> 2)] >> (8 * (l & 3) + sh)) & 0xF);
            } else {
                q0 = (int)((w[0] >> (8 * (l >> 1) + 4 * (l & 1))) & 0xF);
                q1 = (int)((w[1] >> (8 * (l >> 1) + 4 * (l & 1))) & 0xF);
            }
            o0[l] = (_Float16)(d * (float)(q0 - 8));
            o1[l] = (_Float16)(d * (float)(q1 - 8));
        }
        k0 = 32 * (c >> 1) + 16 * (c & 1);
        k1 = k0 + 8;
    }
};

struct BigQ6K {
    static constexpr int BLOCK = 210;
    // per half ip: ql bytes 64ip+16c..+15 (low nibbles: quarters 0/1, high nibbles: quarters 2/3) and qh bytes
    // 32ip+16(c&1)..+15; the four scales of this quarter-column (8ip + 4p + c) packed in one word; d
    struct Raw { u32x4 ql[2], qh[2]; uint32_t sc4; uint32_t d; };
    __device__ static __forceinline__ void load(const uint8_t *blk, int c, Raw &r) {
#pragma unroll
        for (int ip = 0; ip < 2; ++ip) {
            r.ql[ip] = *(const u32x4_a2 *)(blk + 64 * ip + 16 * c);
            r.qh[ip] = *(const u32x4_a2 *)(blk + 128 + 32 * ip + 16 * (c & 1));
        }
        const uint8_t *sc = blk + 192 + c;
        r.sc4 = (uint32_t)sc[0] | ((uint32_t)sc[4] << 8) | ((uint32_t)sc[8] << 16) | ((uint32_t)sc[12] << 24);
        r.d = *(const uint16_t *)(blk + 208);
    }
    // step g = 2*ip + p covers k = 128ip + 64p .. +63: quarters 2p and 2p+1 of half ip; this task owns
    // values 16c..16c+15 of the step, i.e. quarter 2p + (c>>1), il = 16(c&1)..+15, one scale
    __device__ static __forceinline__ void dequant(const Raw &r, int g, int c, half8 &o0, half8 &o1, int &k0, int &k1) {
        const int ip = g >> 1, p = g & 1;
        const int shift = 2 * (2 * p + (c >> 1));
        const float dsc = half_bits_to_float((uint16_t)r.d) * (float)(int)(int8_t)((r.sc4 >> (8 * g)) & 0xFF);
        const float off = -32.0f * dsc;
        const uint32_t qlw[4] = {r.ql[ip].x, r.ql[ip].y, r.ql[ip].z, r.ql[ip].w};
        const uint32_t qhw[4] = {r.qh[ip].x, r.qh[ip].y, r.qh[ip].z, r.qh[ip].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t lo4 = (qlw[j] >> (4 * p)) & 0x0F0F0F0Fu;
            const uint32_t hi2 = ((qhw[j] >> shift) & 0x03030303u) << 4;
            const uint32_t q = lo4 | hi2;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const _Float16 v = (_Float16)(dsc * (float)((q >> (8 * b)) & 0xFF) + off);  // = d*sc*(q-32), exact in f32
                if (j < 2) o0[4 * j + b] = v;
                else o1[4 * (j - 2) + b] = v;
            }
        }
        k0 = 16 * c;
        k1 = 16 * c + 8;
    }
};

// ------------------------------------------------------------------ tile kernel
// One launch may serve up to three weight tensors that share the activations (q / k / v of a prompt pass): weight
// tiles [tile0, next tile0) belong to segment s, which has its own weights, row count, output and residual.
// Whether a policy offers the two-part dequantization (Pre, prepare, dequant_pre)
template <class F, class = void>
struct F16Pre {
    struct type {};
    static constexpr bool value = false;
};
template <class F>
struct F16Pre<F, std::void_t<typename F::Pre>> {
    typedef typename F::Pre type;
    static constexpr bool value = true;
};

struct F16Seg {
    const uint8_t *W;
    float *out;
    const float *res;
    int N, tile0;
};
struct F16Group {
    F16Seg seg[3];
    int count;
    __device__ __forceinline__ F16Seg pick(int nt) const {
        F16Seg s = seg[0];
        if (count > 1 && nt >= seg[1].tile0) s = seg[1];
        if (count > 2 && nt >= seg[2].tile0) s = seg[2];
        return s;
    }
};

// grid = tiles * n_split; workgroup (tile, split) contracts super-blocks [split*sb_per, ...) and writes
// its tile to out + split * split_stride (out = y when n_split == 1).
template <class F, int BN, int BM, int WN, int WM, bool RES>
__global__ __launch_bounds__(WN * WM * 64) void k_mmq_f16(const F16Group grp, const _Float16 *__restrict__ xh, int M, int K,
                                                          int n_tiles, int m_tiles, int sb_per, size_t split_stride) {
    constexpr int T = WN * WM * 64;
    constexpr int TN = BN / WN / 16, TM = BM / WM / 16;
    constexpr int ATK = BN * 4 / T;   // dequantization tasks per thread per step
    constexpr int BCH = BM * 8 / T;   // 16-byte activation chunks per thread per step
    static_assert(BN * 4 % T == 0 && BM * 8 % T == 0 && TN >= 1 && TM >= 1, "tile shape");
    extern __shared__ __align__(16) uint8_t smem_raw[];
    _Float16 *sA = (_Float16 *)smem_raw;               // [2][BN / 16][2] fragments
    _Float16 *sB = sA + 2 * BN * BIG_BK;               // [2][BM / 16][2] fragments

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave % WN, wm = wave / WN;
    // Weight staging lane map: neighbouring lanes take neighbouring quarters of a row (global loads of whole 64-byte
    // runs); the 32 lanes of a half-wavefront take rows {x, x+4, x+8, x+12}, which the row ^ piece term of the
    // layout spreads over all 16 bank windows.  The activations lie in memory fragment by fragment (xh_index4): the
    // tile's share of a step is 2 KB per 16 rows, copied piece by piece into the LDS order.
    const int a_c = lane & 3, a_r = 4 * ((lane >> 2) & 3) + (lane >> 4);

    // tile numbering: the hardware deals workgroups round-robin to the 8 XCDs; give each XCD a
    // contiguous run of weight tiles inside one activation tile
    const int total = n_tiles * m_tiles;
    const int split = blockIdx.x / total;
    int v = blockIdx.x - split * total;
    if ((total & 7) == 0) v = (v & 7) * (total >> 3) + (v >> 3);
    const int mt = v / n_tiles, nt = v - mt * n_tiles;
    const F16Seg seg = grp.pick(nt);
    const int N = seg.N;
    const int n0 = (nt - seg.tile0) * BN, m0 = mt * BM;

    const size_t rb = (size_t)(K >> 8) * F::BLOCK;
    const int sb0 = split * sb_per;
    const int n_sb = min(K >> 8, sb0 + sb_per) - sb0;  // >= 1 by construction of the grid
    const int steps = n_sb * 4;
    const uint8_t *__restrict__ W = seg.W + (size_t)sb0 * F::BLOCK;
    xh += (size_t)sb0 * 8 * 512;  // 8 fragments of 32 values further along K, in every row block
    float *out = seg.out + (size_t)split * split_stride;
    const float *res = seg.res;
    const _Float16 *xtile = xh + (size_t)(m0 >> 4) * (K >> 5) * 512;

    typename F::Raw raw[2][ATK];
    u32x4 xr[2][BCH];
    auto gload_a = [&](int sb, int slot) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < ATK; ++i) {
            const int row = ((tid + i * T) >> 6) * 16 + a_r;
            F::load(W + (size_t)min(n0 + row, N - 1) * rb + (size_t)sb * F::BLOCK, a_c, raw[slot][i]);
        }
    };
    auto gload_b = [&](int ks, int slot) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < BCH; ++i) {
            // LDS piece q of the tile: 16-row block q >> 7, half of the step (q >> 6) & 1, piece p = (q >> 4) & 3 of row
            // (q & 15) ^ p; in memory a fragment is 16 rows of 64 bytes
            const int q = tid + i * T, pc = (q >> 4) & 3, row = (q & 15) ^ pc;
            xr[slot][i] = *(const u32x4 *)(xtile + ((size_t)(q >> 7) * (K >> 5) + (size_t)ks * 2 + ((q >> 6) & 1)) * 512 +
                                           row * 32 + pc * 8);
        }
    };
    auto stage = [&](int g, int aslot, int bslot, int buf) __attribute__((always_inline)) {
        _Float16 *a = sA + buf * BN * BIG_BK;
        _Float16 *b = sB + buf * BM * BIG_BK;
#pragma unroll
        for (int i = 0; i < ATK; ++i) {
            const int row = ((tid + i * T) >> 6) * 16 + a_r;
            half8 o0, o1;
            int k0, k1;
            F::dequant(raw[aslot][i], g, a_c, o0, o1, k0, k1);
            *(half8 *)&a[frag_off(row, k0)] = o0;
            *(half8 *)&a[frag_off(row, k1)] = o1;
        }
#pragma unroll
        for (int i = 0; i < BCH; ++i) *(u32x4 *)&b[(tid + i * T) * 8] = xr[bslot][i];
    };

    float4v acc[TN][TM];
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b) acc[a][b] = float4v{0.f, 0.f, 0.f, 0.f};

    auto compute = [&](int buf) __attribute__((always_inline)) {
        const _Float16 *a = sA + buf * BN * BIG_BK + wn * (BN / WN) * BIG_BK + frag_lane_off(lane);
        const _Float16 *b = sB + buf * BM * BIG_BK + wm * (BM / WM) * BIG_BK + frag_lane_off(lane);
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            half8 af[TN], bf[TM];
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) af[tn] = *(const half8 *)&a[(tn * 2 + kk) * 512];
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) bf[tm] = *(const half8 *)&b[(tm * 2 + kk) * 512];
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int tm = 0; tm < TM; ++tm)
                    acc[tn][tm] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[tn], bf[tm], acc[tn][tm], 0, 0, 0);
        }
    };

    // Step ks = 4*sb + g computes from LDS buffer (ks & 1) and, meanwhile, stages step ks+1 into the
    // other buffer.  Staging step 4*sb+4 (g == 3) is the first use of super-block sb+1, which was
    // requested when super-block sb was first used.  Super-blocks alternate between the two register
    // slots, so the loop body covers two of them.
    gload_a(0, 0);
    gload_b(0, 0);
    gload_b(1, 1);
    gload_a(min(1, n_sb - 1), 1);
    stage(0, 0, 0, 0);
    gload_b(2, 0);
    __syncthreads();
    for (int sb2 = 0; sb2 < n_sb; sb2 += 2) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int sb = sb2 + half;
            if (sb >= n_sb) break;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                // One straight-line block per step (loads past the end are clamped to valid addresses and
                // the last step stages a buffer nobody reads).
                const int ks = sb * 4 + g;
                compute(g & 1);
                // (g + 1) & 1 is both the activation slot and the LDS buffer of step ks + 1
                if (g < 3) stage(g + 1, half, (g + 1) & 1, (g + 1) & 1);
                else stage(0, half ^ 1, 0, 0);
                gload_b(min(ks + 3, steps - 1), (g + 1) & 1);
                if (g == 3) gload_a(min(sb + 2, n_sb - 1), half);
                __syncthreads();
            }
        }
    }

    // C layout of a 16x16 tile: lane holds activation row (lane & 15) and weight rows 4*(lane>>4)..+3
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            const int m = m0 + wm * (BM / WM) + tm * 16 + (lane & 15);
            const int n = n0 + wn * (BN / WN) + tn * 16 + 4 * (lane >> 4);
            if (m >= M) continue;
            float *dst = out + (size_t)m * N + n;
            const float *r = RES && res ? res + (size_t)m * N + n : nullptr;  // may alias dst: read before the store
            if (n + 3 < N && (N & 3) == 0) {
                float4 o = make_float4(acc[tn][tm][0], acc[tn][tm][1], acc[tn][tm][2], acc[tn][tm][3]);
                if (r) {
                    const float4 rv = *(const float4 *)r;
                    o = make_float4(rv.x + o.x, rv.y + o.y, rv.z + o.z, rv.w + o.w);
                }
                *(float4 *)dst = o;
            } else {
#pragma unroll
                for (int l = 0; l < 4; ++l)
                    if (n + l < N) dst[l] = r ? r[l] + acc[tn][tm][l] : acc[tn][tm][l];
            }
        }
}

// ------------------------------------------------------------------ the same tile with the work split by role
// 128 weight rows x BM (256 or 128) activation rows, 8 wavefronts: wavefronts 0-3 (one per SIMD) are producers, 4-7
// consumers.
// Producers request weights, dequantize them and fill the LDS weight buffer of step s + 1 (two buffers) while the
// consumers contract step s; one workgroup barrier per step hands a buffer over.  The activations never touch LDS:
// their fp16 image lies in memory fragment by fragment, 1 KB per B operand of a matrix instruction (xh_index4), so a
// consumer loads each fragment it needs with one 128-bit load per lane, 1 KB of consecutive memory per wavefront,
// straight into operand registers, one step ahead.  Each consumer owns all 128 weight rows and a quarter of the tile's
// activation rows, so every activation fragment is loaded by exactly one wavefront of the workgroup.
//   Why: with the activations staged through LDS by the producers (8 loads and 8 LDS writes per thread and step for
//   BM = 256), disabling parts of the kernel showed the producers alone taking 72 of the kernel's 81 us at
//   14336 x 4096 x 512 - 23 us of that the activation copy, 12 us the dequantization - against 55 us for the consumers
//   alone: moving a step's 32 KB of activations into the CU costs 700 to 950 cycles whichever wavefronts do it, and
//   LDS carried 144 KB per step (now 80 KB: 16 KB of weight tile written, 4 x 16 KB read).
// A consumer walks a step in four phases (two halves of K x two halves of the weight rows) of 16 or 8 matrix
// instructions, reading the next phase's four weight fragments from LDS and requesting a quarter of the next step's
// activation fragments while the current phase's instructions run; it runs at raised priority, so that its matrix
// instruction goes ahead of a producer's vector instruction when both are ready.
// The two roles are separate loops with the same number of barriers, so that their registers (accumulators and
// operand fragments here, raw blocks there) share one allocation.
// BN = 112 (seven 16-row fragments: the second half of the weight rows is three fragments instead of four) is for
// row counts that are a multiple of 7 * 16 and not of 256 * 128: 14336 = 128 * 112 rows are 128 tiles, one or two per
// CU, where 112 tiles of 128 rows leave an eighth of the chip idle or wait for a short last round.  The LDS buffers
// keep room for 128 rows; the producer wavefront whose second task would fall on rows 112 .. 127 repeats its first.
template <class F, int BN, int BM, bool RES>
__global__ __launch_bounds__(512) void k_mmq_f16_pc(const F16Group grp, const _Float16 *__restrict__ xh, int M, int K,
                                                    int n_tiles, int m_tiles, int sb_per, size_t split_stride) {
    constexpr int PT = 256, BNB = 128;  // BNB: weight rows an LDS buffer has room for
    constexpr int ATK = BNB * 4 / PT;   // dequantization tasks per producer thread per step
    constexpr int TNF = BN / 16;        // 16-row weight fragments of the tile
    static_assert(BN == 128 || BN == 112, "weight rows per tile");
    constexpr int TM = BM / 64;       // 16-row activation fragments of a consumer's sub-tile (its rows: BM / 4)
    static_assert(BM == 256 || BM == 128, "activation rows per tile");
    // BM = 256: the producers work two steps ahead into the third of three weight buffers, and a consumer reads the
    // first weight fragments of step s + 1 during the last matrix instructions of step s (16 per phase cover the
    // read).  BM = 128 (8 matrix instructions per phase) is faster one step ahead with two buffers: 33.8 against
    // 35.2 us at 14336 x 4096 x 128.
    constexpr int LEAD = BM == 256 ? 2 : 1, NB = LEAD + 1;
    extern __shared__ __align__(16) uint8_t smem_raw[];
    _Float16 *sA = (_Float16 *)smem_raw;               // [NB][BNB / 16][2] fragments

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    const int total = n_tiles * m_tiles;
    const int split = blockIdx.x / total;
    int v = blockIdx.x - split * total;
    if ((total & 7) == 0) v = (v & 7) * (total >> 3) + (v >> 3);
    const int mt = v / n_tiles, nt = v - mt * n_tiles;
    const F16Seg seg = grp.pick(nt);
    const int N = seg.N;
    const int n0 = (nt - seg.tile0) * BN, m0 = mt * BM;

    const size_t rb = (size_t)(K >> 8) * F::BLOCK;
    const int sb0 = split * sb_per;
    const int n_sb = min(K >> 8, sb0 + sb_per) - sb0;  // >= 1 by construction of the grid
    const int steps = n_sb * 4;
    const uint8_t *__restrict__ W = seg.W + (size_t)sb0 * F::BLOCK;
    xh += (size_t)sb0 * 8 * 512;  // 8 fragments of 32 values further along K, in every row block
    float *out = seg.out + (size_t)split * split_stride;
    const float *res = seg.res;

    if (wave < 4) {
        // ---------------- producers: the weight tile of step t + LEAD (buffer (t + LEAD) % NB) while step t is contracted
        typename F::Raw raw[2][ATK];
        typename F16Pre<F>::type pre[2][ATK];
        // neighbouring lanes take neighbouring quarters of a row; a half-wavefront takes rows {x, x+4, x+8, x+12}
        const int a_c = lane & 3, a_row = 16 * wave + 4 * ((lane >> 2) & 3) + (lane >> 4);   // + a_step i
        const int a_step = BN == 112 && wave == 3 ? 0 : 64;
        auto gload_a = [&](int sb, int slot) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < ATK; ++i)
                F::load(W + (size_t)min(n0 + a_row + a_step * i, N - 1) * rb + (size_t)sb * F::BLOCK, a_c, raw[slot][i]);
        };
        auto stage = [&](int g, int aslot, int buf) __attribute__((always_inline)) {
            _Float16 *a = sA + buf * BNB * BIG_BK;
#pragma unroll
            for (int i = 0; i < ATK; ++i) {
                half8 o0, o1;
                int k0, k1;
                if constexpr (F16Pre<F>::value) {
                    if (g == 0) F::prepare(raw[aslot][i], a_c, pre[aslot][i]);  // a super-block's first step
                    F::dequant_pre(raw[aslot][i], pre[aslot][i], g, a_c, o0, o1, k0, k1);
                } else {
                    F::dequant(raw[aslot][i], g, a_c, o0, o1, k0, k1);
                }
                *(half8 *)&a[frag_off(a_row + a_step * i, k0)] = o0;
                *(half8 *)&a[frag_off(a_row + a_step * i, k1)] = o1;
            }
        };
        gload_a(0, 0);
        gload_a(min(1, n_sb - 1), 1);
        stage(0, 0, 0);
        if (LEAD == 2) stage(1, 0, 1);
        __syncthreads();
        // Iteration t = 8 j + u stages step t + LEAD (past the end: a clamped super-block, into a buffer nobody
        // reads): super-blocks alternate between the two raw slots, so u fixes group and slot of the staged step.
        int buf = LEAD % NB;
        for (int t8 = 0; t8 < steps; t8 += 8) {
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int t = t8 + u;
                if ((u & 3) == 0 && t >= steps) break;  // steps is a multiple of 4
                const int g = (u + LEAD) & 3, slot = ((u + LEAD) >> 2) & 1;
                stage(g, slot, NB == 2 ? ((u + LEAD) & 1) : buf);  // two buffers: a constant of the unrolled body
                buf = buf == NB - 1 ? 0 : buf + 1;
                if (g == 3) gload_a(min(((t + LEAD) >> 2) + 2, n_sb - 1), slot);
                __syncthreads();
            }
        }
        return;
    }

    // ---------------- consumers: wavefront cw owns the BN weight rows x activation rows [cw * BM / 4, + BM / 4)
    const int cw = wave - 4;
    __builtin_amdgcn_s_setprio(3);
    float4v acc[TNF][TM];
#pragma unroll
    for (int a = 0; a < TNF; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b) acc[a][b] = float4v{0.f, 0.f, 0.f, 0.f};
    // activation fragment (16-row block rbk of the tile, 32-value block kb of K): 1 KB at ((m0 / 16 + rbk) * (K / 32) + kb)
    // * 1 KB; lane l takes row l & 15, values 8 (l >> 4) .. + 7: the wavefront's 64 loads cover the fragment once
    const _Float16 *xfrag = xh + ((size_t)((m0 >> 4) + cw * TM) * (K >> 5)) * 512 + (lane & 15) * 32 + (lane >> 4) * 8;
    // steps the activation loads run ahead, and register slots for them: two steps for the 128-row tiles, whose steps
    // are shorter than a load from L2 under this traffic takes (14336 x 4096 x 128: 31.5 us; one step 32.2, three 32.6)
    constexpr int BD = BM == 128 ? 2 : 1, NS = 2 * BD;
    half8 bf[NS][2][TM];  // [step % NS][half of the step][fragment]
    auto load_b = [&](int ks, int slot) __attribute__((always_inline)) {
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
                bf[slot][kk][tm] = *(const half8 *)(xfrag + ((size_t)tm * (K >> 5) + (size_t)ks * 2 + kk) * 512);
    };
    // A step is four phases, phase p = 2 * kk + h: weight rows 64 h .. min(64 h + 63, BN - 1), values 32 kk .. 32 kk + 31
    // (two phases of all the weight rows for the 128-row tiles, whose phases have 8 matrix instructions: 34.4 against
    // 33.8 us at 14336 x 4096 x 128; eight producer wavefronts for them: 33.6 against 33.0)
    constexpr int PH = 4, HN = 4;  // phases per step, weight fragments per phase
    half8 af[2][HN];
    auto fetch = [&](int abuf, int p) __attribute__((always_inline)) {
        const _Float16 *a = sA + abuf * BNB * BIG_BK + frag_lane_off(lane);
        const int kk = PH == 4 ? p >> 1 : p, t0 = PH == 4 ? (p & 1) * 4 : 0;
#pragma unroll
        for (int tn = 0; tn < HN; ++tn)
            if (t0 + tn < TNF) af[p & 1][tn] = *(const half8 *)&a[((t0 + tn) * 2 + kk) * 512];
    };
    auto mma = [&](int bslot, int p) __attribute__((always_inline)) {
        const int kk = PH == 4 ? p >> 1 : p, t0 = PH == 4 ? (p & 1) * 4 : 0;
#pragma unroll
        for (int tn = 0; tn < HN; ++tn)
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
                if (t0 + tn < TNF)
                    acc[t0 + tn][tm] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[p & 1][tn], bf[bslot][kk][tm],
                                                                            acc[t0 + tn][tm], 0, 0, 0);
    };
    load_b(0, 0);
    if (BD == 2) load_b(min(1, steps - 1), 1);
    __syncthreads();  // the weight tiles of the first LEAD steps are in LDS
    constexpr bool AHEAD = LEAD == 2;
    if (AHEAD) fetch(0, 0);
    int abuf = 0;
    for (int sb = 0; sb < n_sb; ++sb) {  // four steps per iteration: no exit inside the unrolled body
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int ks = sb * 4 + g;
            const int anext = abuf == NB - 1 ? 0 : abuf + 1;
            const int acur = NB == 2 ? (g & 1) : abuf;  // two buffers: a constant of the unrolled body
            const int ksn = min(ks + BD, steps - 1);  // a later step's activations, in flight during this one:
            if (!AHEAD) fetch(acur, 0);               // a quarter of them requested in front of each phase
#pragma unroll
            for (int p = 0; p < PH; ++p) {
#pragma unroll
                for (int t = 0; t < 2 * TM / PH; ++t) {
                    const int l = p * (2 * TM / PH) + t, kk = l / TM, tm = l % TM;
                    bf[(g + BD) & (NS - 1)][kk][tm] = *(const half8 *)(xfrag + ((size_t)tm * (K >> 5) + (size_t)ksn * 2 + kk) * 512);
                }
                // the next phase's weight fragments - after the last phase: the next step's first, whose buffer has
                // been complete since the barrier before this step - are read while this phase multiplies
                if (p < PH - 1) fetch(acur, p + 1);
                else if (AHEAD) fetch(anext, 0);
                __builtin_amdgcn_sched_barrier(0);
                mma(g & (NS - 1), p);
                __builtin_amdgcn_sched_barrier(0);
            }
            abuf = anext;
            __syncthreads();
        }
    }

    // C layout of a 16x16 tile: lane holds activation row (lane & 15) and weight rows 4*(lane>>4)..+3
#pragma unroll
    for (int tn = 0; tn < TNF; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            const int m = m0 + cw * (BM / 4) + tm * 16 + (lane & 15);
            const int n = n0 + tn * 16 + 4 * (lane >> 4);
            if (m >= M) continue;
            float *dst = out + (size_t)m * N + n;
            const float *r = RES && res ? res + (size_t)m * N + n : nullptr;  // may alias dst: read before the store
            if (n + 3 < N && (N & 3) == 0) {
                float4 o = make_float4(acc[tn][tm][0], acc[tn][tm][1], acc[tn][tm][2], acc[tn][tm][3]);
                if (r) {
                    const float4 rv = *(const float4 *)r;
                    o = make_float4(rv.x + o.x, rv.y + o.y, rv.z + o.z, rv.w + o.w);
                }
                *(float4 *)dst = o;
            } else {
#pragma unroll
                for (int l = 0; l < 4; ++l)
                    if (n + l < N) dst[l] = r ? r[l] + acc[tn][tm][l] : acc[tn][tm][l];
            }
        }
}

// y[i] = (res[i] +) part[0][i] + part[1][i] + ... in that order (copies `stride` floats apart); res may alias y
__global__ __launch_bounds__(256) void k_splitk_sum(const float *__restrict__ part, float *y, const float *res, size_t count,
                                                    int n_split, size_t stride) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= count) return;
    if (i + 4 <= count && (((uintptr_t)y | (uintptr_t)part | (uintptr_t)res) & 15) == 0 && ((count | stride) & 3) == 0) {
        float4 s = *(const float4 *)(part + i);
        for (int k = 1; k < n_split; ++k) {
            const float4 v = *(const float4 *)(part + (size_t)k * stride + i);
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
        if (res) {
            const float4 r = *(const float4 *)(res + i);
            s = make_float4(r.x + s.x, r.y + s.y, r.z + s.z, r.w + s.w);
        }
        *(float4 *)(y + i) = s;
    } else {
        for (size_t j = i; j < i + 4 && j < count; ++j) {
            float s = part[j];
            for (int k = 1; k < n_split; ++k) s += part[(size_t)k * stride + j];
            y[j] = res ? res[j] + s : s;
        }
    }
}

int launch_splitk_sum(candy_hip_device *dev, const float *part, float *y, const float *res, size_t count, int n_split,
                      size_t stride) {
    hipLaunchKernelGGL(k_splitk_sum, dim3((unsigned)((count / 4 + 256) / 256)), dim3(256), 0, dev->stream, part, y, res,
                       count, n_split, stride ? stride : count);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

// Up to three contractions that share the activations, in one launch (a single one: count = 1).  Every tensor but the
// last has a multiple of BN rows (a tile belongs to one tensor).
struct F16Job {
    const candy_hip_qtensor *w;
    float *y;
    const float *res;
};

// Workgroups per tile along K: split K until the grid covers the chip, keeping at least two super-blocks (8 steps)
// per workgroup: as many workgroups per tile as leave every workgroup a CU of its own (measured against rounding up:
// 14336 x 4096 at 128 rows 44.8 us with 2 against 47.6 with 3; 11008 x 4096 at 256 rows 57.4 with 2 against 66.6 with
// 3, at 512 rows 88.8 with 1 against 105.7 with 2)
static int plan_split(const candy_hip_device *dev, int tiles, int n_sb) {
    int n_split = 1;
    if (tiles < (3 * dev->num_cus) / 4) {
        n_split = dev->num_cus / tiles;
        if (n_split > n_sb / 2) n_split = n_sb / 2;
        if (n_split > 16) n_split = 16;
        if (n_split < 1) n_split = 1;
    }
    if (dev->opt.f16_split > 0) n_split = std::min(dev->opt.f16_split, n_sb);  // comparison runs
    return n_split;
}

template <class F, int BN, int BM, int WN, int WM, bool PC = false>
static int launch_big(candy_hip_device *dev, const F16Job *jobs, int count, const _Float16 *xh, int64_t m) {
    static_assert(!PC || ((BN == 128 || BN == 112) && (BM == 256 || BM == 128) && WN * WM == 8), "the role-split kernel's tiles");
    const int K = (int)jobs[0].w->cols;
    F16Group grp{};
    grp.count = count;
    int n_tiles = 0;
    int64_t n_total = 0;
    bool any_res = false;
    for (int s = 0; s < count; ++s) {
        grp.seg[s] = F16Seg{(const uint8_t *)jobs[s].w->data, jobs[s].y, jobs[s].res, (int)jobs[s].w->rows, n_tiles};
        n_tiles += (int)((jobs[s].w->rows + BN - 1) / BN);
        n_total += jobs[s].w->rows;
        any_res = any_res || jobs[s].res;
    }
    const int m_tiles = (int)((m + BM - 1) / BM);
    const int tiles = n_tiles * m_tiles, n_sb = K >> 8;
    int n_split = plan_split(dev, tiles, n_sb);
    const int sb_per = (n_sb + n_split - 1) / n_split;
    n_split = (n_sb + sb_per - 1) / sb_per;  // no empty splits
    const size_t split_stride = (size_t)m * (size_t)n_total;
    float *part = nullptr;
    if (n_split > 1) {
        // each workgroup writes its partial tile to copy `split` of a workspace laid out [split][tensor][m][rows]
        void *p = nullptr;
        if (int rc = splitk_workspace(dev, (size_t)n_split * split_stride * sizeof(float), &p)) return rc;
        part = (float *)p;
        size_t off = 0;
        for (int s = 0; s < count; ++s) {
            grp.seg[s].out = part + off;
            grp.seg[s].res = nullptr;  // the split sum adds it
            off += (size_t)m * (size_t)jobs[s].w->rows;
        }
    }
    constexpr size_t smem = (size_t)(PC ? 3 * 128 : 2 * (BN + BM)) * BIG_BK * sizeof(_Float16);  // role-split: weight tiles only
    const bool epi_res = any_res && n_split == 1;
    void (*kern)(const F16Group, const _Float16 *, int, int, int, int, int, size_t);
    if constexpr (PC) kern = epi_res ? k_mmq_f16_pc<F, BN, BM, true> : k_mmq_f16_pc<F, BN, BM, false>;
    else kern = epi_res ? k_mmq_f16<F, BN, BM, WN, WM, true> : k_mmq_f16<F, BN, BM, WN, WM, false>;
    CANDY_HIP_TRY(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(kern, dim3((unsigned)(tiles * n_split)), dim3(WN * WM * 64), smem, dev->stream, grp, xh, (int)m, K,
                       n_tiles, m_tiles, sb_per, split_stride);
    CANDY_LAUNCH_CHECK();
    bool one_run = true;  // outputs end to end, no residual but a single job's
    for (int s = 1; s < count; ++s)
        one_run = one_run && !jobs[0].res && !jobs[s].res && jobs[s].y == jobs[s - 1].y + (size_t)m * (size_t)jobs[s - 1].w->rows;
    if (n_split > 1 && one_run && dev->defer_split) {
        SplitPending &sp = *dev->defer_split;  // the caller sums the copies
        sp.part = part; sp.y = jobs[0].y; sp.res = jobs[0].res;
        sp.count = split_stride; sp.stride = split_stride; sp.n_split = n_split;
    } else if (n_split > 1) {
        // one sum per run of outputs that lie end to end (the prompt pass allocates q, k and v that way)
        size_t off = 0;
        for (int s = 0; s < count;) {
            size_t run = (size_t)m * (size_t)jobs[s].w->rows;
            int e = s + 1;
            while (e < count && !jobs[s].res && !jobs[e].res && jobs[e].y == jobs[s].y + run) {
                run += (size_t)m * (size_t)jobs[e].w->rows;
                ++e;
            }
            hipLaunchKernelGGL(k_splitk_sum, dim3((unsigned)((run / 4 + 256) / 256)), dim3(256), 0, dev->stream, part + off,
                               jobs[s].y, jobs[s].res, run, n_split, split_stride);
            CANDY_LAUNCH_CHECK();
            off += run;
            s = e;
        }
    }
    return CANDY_HIP_OK;
}

template <class F, int BN, int BM, int WN, int WM, bool PC = false>
static int launch_big(candy_hip_device *dev, const candy_hip_qtensor *w, const _Float16 *xh, int64_t m, float *y,
                      const float *res) {
    const F16Job job{w, y, res};
    return launch_big<F, BN, BM, WN, WM, PC>(dev, &job, 1, xh, m);
}

bool mmq_f16_big_covers(const candy_hip_qtensor *w, int64_t m, int min_m) {
    // A lower threshold than the decoder's holds for single contractions through the API: Q4_K and Q6_K from `min_m`
    // rows, the other formats from 65: up to 64 rows are one tile of the int8 kernel, which is level with the fp16 tiles
    // there for Q8_0, Q4_0 and Q5_K (and exact).  Measured, us per call, int8 / fp16 tiles: Q6_K 14336 x 4096 at 33 rows
    // 43.8 / 36.6, 4096 x 14336 at 96 rows 71.5 / 39.2, at 255 rows 133 / 57; Q8_0 14336 x 4096 at 48 rows 46.2 / 41.9
    // (4096 x 4096 22.4 / 22.6), at 96 rows 77.8 / 44.7, at 255 rows 121 / 61; Q4_0 at 48 rows 38.9 / 38.0 (4096 x 4096
    // 19.9 / 22.4), at 96 rows 64.3 / 48.7; Q5_K 36.9 / 35.1 (19.9 / 19.9) and 58.6 / 47.2.
    if (min_m <= 0) min_m = w->dev->opt.f16_big_min_m;
    else if (w->fmt != CANDY_HIP_Q4_K && w->fmt != CANDY_HIP_Q6_K) min_m = std::max(min_m, 65);
    if (m < min_m || w->cols % 256 != 0) return false;
    if (w->fmt == CANDY_HIP_Q4_K || w->fmt == CANDY_HIP_Q5_K) return ((uintptr_t)w->data & 15) == 0;
    if (w->fmt == CANDY_HIP_Q6_K || w->fmt == CANDY_HIP_Q8_0 || w->fmt == CANDY_HIP_Q4_0 || w->fmt == CANDY_HIP_Q4_0_GGML)
        return ((uintptr_t)w->data & 1) == 0;
    return false;
}

// Tile shape by batch and grid.  Every format: 128 x 128 tiles up to 128 activation rows, 128 x 256 above.  Q4_K, whose
// dequantization is the cheapest, also takes the narrower tiles on some grids above 128 rows (with the heavier formats
// the producers then set the pace: Q6_K 14336 x 4096 at 192 rows 58.3 us on 128 x 128 tiles against 53.8, Q8_0 68.5
// against 58.6), and tiles of 112 weight rows.
template <class F>
static int launch_shapes(candy_hip_device *dev, const F16Job *jobs, int count, const _Float16 *xh, int64_t m) {
    const int shape = dev->opt.f16_shape;  // comparison runs
    const bool single = shape == 3;        // every wavefront in both roles
    // Tiles of 112 weight rows where every tensor's rows divide by 112 and the grid then takes fewer row-steps of its
    // busiest CU: rounds of workgroups x rows per tile x super-blocks per workgroup (14336 rows: 128 tiles instead of
    // 112, so 256 instead of 224 workgroups at 512 activation rows, 512 instead of 448 for a gate / up pair).
    auto narrow = [&](int bm) {
        if (!std::is_same<F, BigQ4K>::value || single || shape == 4) return false;
        const int n_sb = (int)(jobs[0].w->cols >> 8), m_tiles = (int)((m + bm - 1) / bm);
        int64_t t112 = 0, t128 = 0;
        for (int s = 0; s < count; ++s) {
            if (jobs[s].w->rows % 112 != 0) return false;
            t112 += jobs[s].w->rows / 112;
            t128 += (jobs[s].w->rows + 127) / 128;
        }
        auto cost = [&](int64_t tiles, int bn) {
            const int ns = plan_split(dev, (int)(tiles * m_tiles), n_sb), sb_per = (n_sb + ns - 1) / ns;
            const int64_t wgs = tiles * m_tiles * ((n_sb + sb_per - 1) / sb_per);
            return ((wgs + dev->num_cus - 1) / dev->num_cus) * bn * sb_per;
        };
        return cost(t112, 112) < cost(t128, 128);
    };
    auto small_tiles = [&]() {
        if (single) return launch_big<F, 128, 128, 2, 4>(dev, jobs, count, xh, m);
        if constexpr (std::is_same<F, BigQ4K>::value)
            if (narrow(128)) return launch_big<F, 112, 128, 2, 4, true>(dev, jobs, count, xh, m);
        return launch_big<F, 128, 128, 2, 4, true>(dev, jobs, count, xh, m);
    };
    // up to 128 activation rows: 128 x 128 tiles, K split over workgroups to fill the chip
    if (shape == 2 || m <= 128) return small_tiles();
    constexpr bool q4k = std::is_same<F, BigQ4K>::value;
    // up to 256 rows where the 128 x 128 tiles fill the chip and the 128 x 256 tiles would have to split K
    // (Q4_K 14336 x 4096 at 256 rows: 70.7 us against 80.3)
    int64_t n128 = 0;
    for (int s = 0; s < count; ++s) n128 += (jobs[s].w->rows + 127) / 128;
    const int64_t fill = (3 * (int64_t)dev->num_cus) / 4;
    if (q4k && m <= 256 && n128 * ((m + 127) / 128) >= fill && n128 * ((m + 255) / 256) < fill) return small_tiles();
    // short K (at most 16 super-blocks) on a grid that 128 x 256 tiles would have to split: 128 x 128 tiles halve the
    // split as long as they still fit one round (Q4_K 4096 x 4096 at 512 rows 35.5 against 36.8 us, at 1024 rows 50.9
    // against 54.2; 6144 x 4096 at 512 rows 44.8 against 47.1; with K = 14336 the split is cheap and the wider tile wins)
    if (q4k && shape == 0 && jobs[0].w->cols <= 4096 && n128 * ((m + 255) / 256) < fill && n128 * ((m + 127) / 128) <= dev->num_cus)
        return small_tiles();
    if (single) return launch_big<F, 128, 256, 2, 4>(dev, jobs, count, xh, m);
    if constexpr (std::is_same<F, BigQ4K>::value)
        if (narrow(256)) return launch_big<F, 112, 256, 2, 4, true>(dev, jobs, count, xh, m);
    return launch_big<F, 128, 256, 2, 4, true>(dev, jobs, count, xh, m);
}

static int launch_jobs(candy_hip_device *dev, const F16Job *jobs, int count, const _Float16 *xh, int64_t m) {
    switch (jobs[0].w->fmt) {
    case CANDY_HIP_Q6_K: return launch_shapes<BigQ6K>(dev, jobs, count, xh, m);
    case CANDY_HIP_Q5_K: return launch_shapes<BigQ5K>(dev, jobs, count, xh, m);
    case CANDY_HIP_Q8_0: return launch_shapes<BigQ8_0>(dev, jobs, count, xh, m);
    case CANDY_HIP_Q4_0: return launch_shapes<BigQ4_0<false>>(dev, jobs, count, xh, m);
    case CANDY_HIP_Q4_0_GGML: return launch_shapes<BigQ4_0<true>>(dev, jobs, count, xh, m);
    default: return launch_shapes<BigQ4K>(dev, jobs, count, xh, m);
    }
}

// xh: fp16 activations [mmq_m_pad(m)][K], rows past m zero.
int launch_mmq_f16_big(candy_hip_device *dev, const candy_hip_qtensor *w, const _Float16 *xh, int64_t m, float *y,
                       const float *res) {
    const F16Job job{w, y, res};
    return launch_jobs(dev, &job, 1, xh, m);
}

// Two or three projections of the same activations (q / k / v) as one grid: their tiles fill the chip together where
// each alone would split K many ways (Llama-3-8B shape, 512 rows: 1024 x 4096 alone is 16 tiles).
bool mmq_f16_group_covers(const candy_hip_qtensor *const *ws, int count, int64_t m) {
    if (count < 2 || count > 3 || !ws[0]->dev->opt.prefill_qkv_group || ws[0]->dev->opt.mmq_fp16_only) return false;
    for (int s = 0; s < count; ++s) {
        if (!mmq_f16_big_covers(ws[s], m) || ws[s]->fmt != ws[0]->fmt || ws[s]->cols != ws[0]->cols) return false;
        if (s + 1 < count && ws[s]->rows % 128 != 0) return false;  // a tile belongs to one tensor
    }
    return true;
}

int launch_mmq_f16_group(candy_hip_device *dev, const candy_hip_qtensor *const *ws, float *const *ys, int count,
                         const _Float16 *xh, int64_t m) {
    CANDY_REQUIRE(mmq_f16_group_covers(ws, count, m), "internal: projections cannot share a grid");
    F16Job jobs[3];
    for (int s = 0; s < count; ++s) jobs[s] = F16Job{ws[s], ys[s], nullptr};
    return launch_jobs(dev, jobs, count, xh, m);
}

}  // namespace candy
