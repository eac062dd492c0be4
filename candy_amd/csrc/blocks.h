// Device-side view of candy's block formats
// (tensor/internal/cpu/kernels/quantized.go:8-11, 34-37, 55-59, 70-75; little-endian, packed).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

// Kernel attributes: threads per workgroup, and the fewest / most wavefronts per SIMD the kernel is meant to run with.
// The fewest caps the registers (512 / MINW per lane).  The most matters as much: without it the instruction
// scheduler works towards the highest occupancy the hardware has, and to save registers it sinks the last loads of a
// wavefront below the first wait for memory, where they start a whole memory round trip late.  With the intended
// occupancy stated, every load of a wavefront is issued before its first wait.
#define CANDY_KERNEL(T, MINW, MAXW) \
    __global__ __attribute__((amdgpu_flat_work_group_size(1, T), amdgpu_waves_per_eu(MINW, MAXW)))

namespace candy {

struct __attribute__((packed)) BlockQ4_0 {
    uint16_t d;
    uint8_t qs[16];
};
struct __attribute__((packed)) BlockQ8_0 {
    uint16_t d;
    int8_t qs[32];
};
struct __attribute__((packed)) BlockQ4K {
    uint16_t d, dmin;
    uint8_t scales[12];
    uint8_t qs[128];
};
struct __attribute__((packed)) BlockQ6K {
    uint8_t ql[128];
    uint8_t qh[64];
    int8_t scales[16];
    uint16_t d;
};
// quantized.go:13-31, 39-52, 62-67, 78-82
struct __attribute__((packed)) BlockQ4_1 {
    uint16_t d, m;
    uint8_t qs[16];
};
struct __attribute__((packed)) BlockQ5_0 {
    uint16_t d;
    uint8_t qh[4];
    uint8_t qs[16];
};
struct __attribute__((packed)) BlockQ5_1 {
    uint16_t d, m;
    uint8_t qh[4];
    uint8_t qs[16];
};
struct __attribute__((packed)) BlockQ2K {
    uint8_t scales[16];
    uint8_t qs[64];
    uint16_t d, dmin;
};
struct __attribute__((packed)) BlockQ3K {
    uint8_t hmask[32];
    uint8_t qs[64];
    uint8_t scales[12];
    uint16_t d;
};
struct __attribute__((packed)) BlockQ5K {
    uint16_t d, dmin;
    uint8_t scales[12];
    uint8_t qh[32];
    uint8_t qs[128];
};
struct __attribute__((packed)) BlockQ8K {
    float d;
    int8_t qs[256];
    int16_t bsums[16];
};
static_assert(sizeof(BlockQ4_1) == 20 && sizeof(BlockQ5_0) == 22 && sizeof(BlockQ5_1) == 24, "block size");
static_assert(sizeof(BlockQ2K) == 84 && sizeof(BlockQ3K) == 110 && sizeof(BlockQ5K) == 176 && sizeof(BlockQ8K) == 292, "block size");
static_assert(sizeof(BlockQ4_0) == 18 && sizeof(BlockQ8_0) == 34, "block size");
static_assert(sizeof(BlockQ4K) == 144 && sizeof(BlockQ6K) == 210, "block size");

// Vector types whose loads may sit on 2-byte boundaries (Q8_0 / Q4_0 / Q6_K blocks are only
// 2-byte aligned); gfx950 global loads accept unaligned addresses.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
typedef uint32_t u32x2_a2 __attribute__((ext_vector_type(2), aligned(2)));
typedef uint32_t u32_a2 __attribute__((aligned(2)));

// IEEE half -> single; exact for every input including subnormals
// (same mapping as fp16ToFloat32, quantized.go:149-173).
__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
    return __half2float(__ushort_as_half(h));
}

// The 6-bit (scale, min) pairs of sub-blocks 2*pair and 2*pair+1 of a Q4_K super-block,
// unpacked on 16-bit lanes (get_scale_min_k4, quantized.cu:993-1005).
// s0, s1, s2 are scales[0..3], scales[4..7], scales[8..11] as little-endian words.
// Returns sc in bytes 0,1 of `sc2` and m in bytes 0,1 of `m2`.
__device__ __forceinline__ void q4k_scale_min_pair(uint32_t s0, uint32_t s1, uint32_t s2, int pair,
                                                   uint32_t &sc2, uint32_t &m2) {
    const int sh = (pair & 1) * 16;
    const uint32_t a = (s0 >> sh) & 0xFFFFu, b = (s1 >> sh) & 0xFFFFu, c = (s2 >> sh) & 0xFFFFu;
    const uint32_t sc_lo = a & 0x3F3Fu, m_lo = b & 0x3F3Fu;
    const uint32_t sc_hi = (c & 0x0F0Fu) | ((a & 0xC0C0u) >> 2);
    const uint32_t m_hi = ((c >> 4) & 0x0F0Fu) | ((b & 0xC0C0u) >> 2);
    sc2 = pair < 2 ? sc_lo : sc_hi;
    m2 = pair < 2 ? m_lo : m_hi;
}

__device__ __forceinline__ int dot4_i8(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

// Cross-lane moves on the DPP path (no LDS traffic, no waits).
template <int CTRL, int ROW_MASK = 0xF, int BANK_MASK = 0xF>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, BANK_MASK, true));
}

template <int CTRL, int ROW_MASK = 0xF, int BANK_MASK = 0xF>
__device__ __forceinline__ int dpp_move_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, BANK_MASK, true);
}

// Sum over the 64 lanes of a wavefront; every lane gets the total.
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move<0xB1>(v);        // quad_perm [1,0,3,2]
    v += dpp_move<0x4E>(v);        // quad_perm [2,3,0,1]
    v += dpp_move<0x141>(v);       // row_half_mirror
    v += dpp_move<0x140>(v);       // row_mirror: every lane of a 16-lane row holds the row sum
    v += dpp_move<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3
    v += dpp_move<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3: lane 63 holds the total
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}


// 1 / sqrt(v) as reduce.go:3083-3085 evaluates it for RMSNorm: 1 / float32(math.Sqrt(float64(v))).  The square root
// of an f32 taken in f64 and rounded back is the correctly rounded f32 square root (53 bits >= 2 * 24 + 2), which is
// what sqrtf is here (hipcc rounds f32 sqrt and division correctly by default), so no f64 instruction is needed.
__device__ __forceinline__ float rms_inv_sqrt(float v) { return 1.0f / sqrtf(v); }

// (int)roundf(x / d) with the IEEE division of quantize_q8_1 (quantized.cu:3546-3547), without dividing in the
// common case: x * (1 / d) with the hardware reciprocal is within 2 ulp of the quotient, and the two can only round
// to different integers when a half-integer lies between them, i.e. when the product is within a few ulp of one.
// Only then (and for products outside the range of levels: d subnormal, x not finite) is the division carried out.
__device__ __forceinline__ int q8_level(float x, float d) {
    const float t = x * __builtin_amdgcn_rcpf(d);
    const float a = fabsf(t);
    const float frac = a - truncf(a);           // exact
    const bool near_half = fabsf(frac - 0.5f) <= 6.1e-5f;  // 8 ulp of 127.5: the quotient never exceeds that here
    if (__builtin_expect(near_half || !(a < 128.0f), 0)) return (int)roundf(x / d);
    return (int)roundf(t);
}

// Q8_0 quantization of 4 consecutive values held by one lane; the 8 lanes that share a 32-value
// block must be consecutive lanes of one wavefront (lane % 8 == position in the block) and all
// active.  quantize_q8_1 (quantized.cu:3521-3558) without its `sum`: amax over the block,
// d = amax / 127 (IEEE division), q = amax == 0 ? 0 : roundf(x / d).
// Returns the 4 quants packed little-endian; d_half / bsum are valid in every lane of the block.
__device__ __forceinline__ uint32_t quantize_q8_lane4(float4 v, __half &d_half, int &bsum) {
    // 8-lane reductions on the DPP path: two quad permutes, then the mirror within each 8 lanes
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, dpp_move<0xB1>(amax));
    amax = fmaxf(amax, dpp_move<0x4E>(amax));
    amax = fmaxf(amax, dpp_move<0x141>(amax));
    const float d = amax / 127.0f;
    int q0 = 0, q1 = 0, q2 = 0, q3 = 0;
    if (amax != 0.0f) {
        q0 = q8_level(v.x, d);
        q1 = q8_level(v.y, d);
        q2 = q8_level(v.z, d);
        q3 = q8_level(v.w, d);
    }
    int s = q0 + q1 + q2 + q3;
    s += dpp_move_i<0xB1>(s);
    s += dpp_move_i<0x4E>(s);
    s += dpp_move_i<0x141>(s);
    bsum = s;
    d_half = __float2half_rn(d);
    return (uint32_t)(q0 & 0xFF) | ((uint32_t)(q1 & 0xFF) << 8) | ((uint32_t)(q2 & 0xFF) << 16) |
           ((uint32_t)(q3 & 0xFF) << 24);
}

// The 4 quantized values of a lane as fp16(d * q): what the fp16 tile kernels contract with
// (d = the fp16-rounded block scale widened to f32; the product is exact in f32, one rounding).
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ half4v q8_lane4_to_half(uint32_t packed, __half d_half) {
    const float d = __half2float(d_half);
    half4v r;
#pragma unroll
    for (int l = 0; l < 4; ++l) r[l] = (_Float16)(d * (float)(int8_t)((packed >> (8 * l)) & 0xFF));
    return r;
}

// Where those 4 values go.  The fp16 image of an activation matrix [rows][K] lies in memory as the B operands of
// 16x16x32 matrix instructions: fragments of 16 rows x 32 values (1 KB), [row block][32-value block of K], 64
// bytes per row inside a fragment.  The 64 lanes of a wavefront (lane l: row l & 15, values 8 (l >> 4) .. + 7) load
// a fragment with one 128-bit load each, 1 KB of consecutive memory, straight into the operand registers; a
// quantizer writes a row's 32-value block as 64 consecutive bytes.  Index in units of 4 halves of values
// 4 c4 .. 4 c4 + 3 of `row`; rows are padded to a multiple of 16 by the caller's allocation, K is a multiple of 32.
__host__ __device__ __forceinline__ int64_t xh_index4(int64_t row, int64_t c4, int64_t K) {
    return ((row >> 4) * (K >> 5) + (c4 >> 3)) * 128 + (row & 15) * 8 + (c4 & 7);
}

// Same quantization with one value per lane: the 32 lanes of a block are consecutive lanes
// (lane % 32 == position in the block), all active.
__device__ __forceinline__ int quantize_q8_lane1(float v, __half &d_half, int &bsum) {
    // 32-lane reductions: quad permutes, half mirror, mirror (16-lane row), then the neighbouring row
    float amax = fabsf(v);
    amax = fmaxf(amax, dpp_move<0xB1>(amax));
    amax = fmaxf(amax, dpp_move<0x4E>(amax));
    amax = fmaxf(amax, dpp_move<0x141>(amax));
    amax = fmaxf(amax, dpp_move<0x140>(amax));
    amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
    const float d = amax / 127.0f;
    const int q = amax != 0.0f ? q8_level(v, d) : 0;
    int s = q;
    s += dpp_move_i<0xB1>(s);
    s += dpp_move_i<0x4E>(s);
    s += dpp_move_i<0x141>(s);
    s += dpp_move_i<0x140>(s);
    s += __shfl_xor(s, 16, 64);
    bsum = s;
    d_half = __float2half_rn(d);
    return q;
}

}  // namespace candy
