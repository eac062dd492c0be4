// Weight quantizers from f32: Q4_0 (both element orders), Q4_K, Q6_K.
//
// candy names these kernels (tensor/internal/metal/kernels/kernels.go:563-592: quantize_q4_0,
// quantize_q4_k, quantize_q6_k ...) but holds no implementation; the arithmetic is that of ggml's
// published reference quantizers (quantize_row_q4_0_ref; quantize_row_q4_K_ref with make_qkx2_quants;
// quantize_row_q6_K_ref with make_qx_quants), every f32 operation rounding once, in their order, so the
// blocks come out bit for bit as a CPU evaluation of the same steps gives them.  This file is compiled
// with -ffp-contract=off for that reason (a fused multiply-add rounds once where the steps round twice).
//
// A load-time operation: one thread per block of 32 values (Q4_0, and the sub-blocks of Q4_K, whose eight
// lanes settle the super-block's header with shuffles) or of 16 (Q6_K's groups), the candidate search running
// serially in that thread.  Inputs must be finite.
#include "blocks.h"
#include "internal.h"

namespace candy {

// Round to nearest, ties to even (|f| <= 4194303): adding 1.5 * 2^23 leaves the integer in the mantissa.
__device__ __forceinline__ int rne_int(float f) {
    const float v = f + 12582912.0f;
    return (int)(__float_as_uint(v) & 0x007FFFFFu) - 0x00400000;
}
__device__ __forceinline__ int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }
// The f32 value is rounded to fp16 as it stands: left to the compiler, a product feeding the conversion
// is folded into one mixed-precision multiply-add with a +0 addend, which turns a -0 product into +0.
__device__ __forceinline__ uint16_t f32_to_half_bits(float f) {
    asm volatile("" : "+v"(f));
    return __half_as_ushort(__float2half_rn(f));
}

// ------------------------------------------------------------------ Q4_0
// The value of largest magnitude maps to level -8 (d = max / -8 keeps its sign), the others to
// (int)(x / d + 8.5) capped at 15.  ggml_order: byte j = elements j (low nibble) and j + 16 (high);
// otherwise candy's CPU order, byte j = elements 2j and 2j + 1 (quantized.go:85-93).
__global__ __launch_bounds__(256) void k_wquant_q4_0(const float *__restrict__ x, int64_t nb, BlockQ4_0 *__restrict__ out,
                                                     int ggml_order) {
    const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= nb) return;
    const float4 *src = (const float4 *)(x + 32 * b);
    float v[32];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float4 t = src[i];
        v[4 * i] = t.x; v[4 * i + 1] = t.y; v[4 * i + 2] = t.z; v[4 * i + 3] = t.w;
    }
    float amax = 0.0f, vmax = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const float a = fabsf(v[i]);
        if (amax < a) { amax = a; vmax = v[i]; }
    }
    const float d = vmax / -8.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint32_t q[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const int l = (int)(v[i] * id + 8.5f);
        q[i] = (uint32_t)(l < 15 ? l : 15);
    }
    BlockQ4_0 *y = out + b;
    y->d = f32_to_half_bits(d);
#pragma unroll
    for (int j = 0; j < 16; ++j)
        y->qs[j] = ggml_order ? (uint8_t)(q[j] | (q[j + 16] << 4)) : (uint8_t)(q[2 * j] | (q[2 * j + 1] << 4));
}

// ------------------------------------------------------------------ Q4_K
// Levels 0..15 with scale and non-positive minimum for 32 values (make_qkx2_quants with rmin -1,
// rdelta 0.1, 20 steps, squared error): min/max rounding first, then 21 nearby scales, each followed by
// the weighted least-squares fit of (scale, min) to the levels it yields; the best weighted error wins.
// Returns the scale; neg_min receives -min.
__device__ __forceinline__ float search_affine32(const float (&x)[32], const float (&w)[32], int (&L)[32], float &neg_min) {
    float lo = x[0], hi = x[0];
    float sum_w = w[0], sum_x = sum_w * x[0];
#pragma unroll
    for (int i = 1; i < 32; ++i) {
        if (x[i] < lo) lo = x[i];
        if (x[i] > hi) hi = x[i];
        sum_w += w[i];
        sum_x += w[i] * x[i];
    }
    if (lo > 0.0f) lo = 0.0f;
    if (hi == lo) {
#pragma unroll
        for (int i = 0; i < 32; ++i) L[i] = 0;
        neg_min = -lo;
        return 0.0f;
    }
    float iscale = 15.0f / (hi - lo);
    float scale = 1.0f / iscale;
    float best = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const int l = clampi(rne_int(iscale * (x[i] - lo)), 0, 15);
        L[i] = l;
        float diff = scale * (float)l + lo - x[i];
        diff = diff * diff;
        best += w[i] * diff;
    }
    int cand[32];
#pragma unroll 1
    for (int is = 0; is <= 20; ++is) {
        iscale = (-1.0f + 0.1f * (float)is + 15.0f) / (hi - lo);  // lo: the best minimum so far
        float sum_l = 0.0f, sum_l2 = 0.0f, sum_xl = 0.0f;
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const int l = clampi(rne_int(iscale * (x[i] - lo)), 0, 15);
            cand[i] = l;
            sum_l += w[i] * (float)l;
            sum_l2 += w[i] * (float)l * (float)l;
            sum_xl += w[i] * (float)l * x[i];
        }
        const float det = sum_w * sum_l2 - sum_l * sum_l;
        if (det > 0.0f) {
            float s = (sum_w * sum_xl - sum_x * sum_l) / det;
            float m = (sum_l2 * sum_x - sum_l * sum_xl) / det;
            if (m > 0.0f) {
                m = 0.0f;
                s = sum_xl / sum_l2;
            }
            float err = 0.0f;
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                float diff = s * (float)cand[i] + m - x[i];
                diff = diff * diff;
                err += w[i] * diff;
            }
            if (err < best) {
#pragma unroll
                for (int i = 0; i < 32; ++i) L[i] = cand[i];
                best = err;
                scale = s;
                lo = m;
            }
        }
    }
    neg_min = -lo;
    return scale;
}

// One super-block per eight neighbouring lanes, one 32-value sub-block per lane (values, weights and levels
// in registers): per-sub-block (scale, min) with weights rms + |x|, both stored in 6 bits relative to their
// maxima over the eight lanes (d, dmin in fp16, packed as get_scale_min_k4 of quantized.cu:993-1005 unpacks
// them), then the levels assigned again with the STORED scales (a sub-block whose stored scale is 0 keeps the
// search's).  Lanes past the last super-block work on zeros and store nothing, so every shuffle is full.
__global__ __launch_bounds__(256) void k_wquant_q4_k(const float *__restrict__ x, int64_t nb, BlockQ4K *__restrict__ out) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t b = t >> 3;
    const int j = (int)(t & 7);
    const bool live = b < nb;
    float xs[32], w[32];
    {
        const float4 *src = (const float4 *)(x + 256 * b + 32 * j);
#pragma unroll
        for (int l = 0; l < 8; ++l) {
            const float4 v = live ? src[l] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            xs[4 * l] = v.x, xs[4 * l + 1] = v.y, xs[4 * l + 2] = v.z, xs[4 * l + 3] = v.w;
        }
    }
    float sum_x2 = 0.0f;
#pragma unroll
    for (int l = 0; l < 32; ++l) sum_x2 += xs[l] * xs[l];
    const float av = sqrtf(sum_x2 / 32.0f);
#pragma unroll
    for (int l = 0; l < 32; ++l) w[l] = av + fabsf(xs[l]);
    int L[32];
    float neg_min;
    const float scale = search_affine32(xs, w, L, neg_min);
    float max_scale = scale, max_min = neg_min;
#pragma unroll
    for (int o = 1; o < 8; o <<= 1) {
        max_scale = fmaxf(max_scale, __shfl_xor(max_scale, o));
        max_min = fmaxf(max_min, __shfl_xor(max_min, o));
    }
    if (!(max_scale > 0.0f)) max_scale = 0.0f;  // the serial maximum starts from +0
    if (!(max_min > 0.0f)) max_min = 0.0f;
    const float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    const float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    const int ls = rne_int(inv_scale * scale), lm = rne_int(inv_min * neg_min);
    const int sc6 = ls < 63 ? ls : 63, mn6 = lm < 63 ? lm : 63;
    const int sc6_hi = __shfl_down(sc6, 4), mn6_hi = __shfl_down(mn6, 4);  // lanes 0-3: sub-block j + 4
    const uint16_t dh = f32_to_half_bits(max_scale / 63.0f), mh = f32_to_half_bits(max_min / 63.0f);
    BlockQ4K *y = out + b;
    if (live && j < 4) {
        y->scales[j] = (uint8_t)(sc6 | ((sc6_hi >> 4) << 6));
        y->scales[j + 4] = (uint8_t)(mn6 | ((mn6_hi >> 4) << 6));
        y->scales[j + 8] = (uint8_t)((sc6_hi & 0xF) | ((mn6_hi & 0xF) << 4));
    }
    if (live && j == 0) {
        y->d = dh;
        y->dmin = mh;
    }
    const float d = half_bits_to_float(dh) * (float)sc6;
    if (d != 0.0f) {
        const float dm = half_bits_to_float(mh) * (float)mn6;
#pragma unroll
        for (int i = 0; i < 32; ++i) L[i] = clampi(rne_int((xs[i] + dm) / d), 0, 15);
    }
    // Byte l of a 64-value group = level l of its even sub-block | level l of the odd one << 4: the two lanes
    // exchange their levels, four to a word, and each stores 16 of the 32 bytes.
    uint32_t mine[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) mine[i] = (uint32_t)(L[4 * i] | (L[4 * i + 1] << 8) | (L[4 * i + 2] << 16) | (L[4 * i + 3] << 24));
    const int odd = j & 1;
    uint16_t *dst = (uint16_t *)(y->qs + 32 * (j >> 1) + 16 * odd);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t give = odd ? mine[i] : mine[4 + i];       // the half the other lane stores
        const uint32_t keep = odd ? mine[4 + i] : mine[i];
        const uint32_t got = (uint32_t)__shfl_xor((int)give, 1);
        const uint32_t word = odd ? (got | (keep << 4)) : (keep | (got << 4));
        if (live) {
            dst[2 * i] = (uint16_t)word;
            dst[2 * i + 1] = (uint16_t)(word >> 16);
        }
    }
}

// ------------------------------------------------------------------ Q6_K
// Symmetric levels -32..31 for 16 values (make_qx_quants, weights x^2): the value of largest magnitude
// maps to -32, then 18 nearby scales are tried and the largest (sum w x l)^2 / (sum w l^2) wins.
// L receives level + 32.
__device__ __forceinline__ float search_symmetric16(const float (&x)[16], int (&L)[16]) {
    float vmax = 0.0f, amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const float a = fabsf(x[i]);
        if (a > amax) { amax = a; vmax = x[i]; }
    }
    if (amax < 1e-15f) {
#pragma unroll
        for (int i = 0; i < 16; ++i) L[i] = 0;
        return 0.0f;
    }
    float iscale = -32.0f / vmax;
    float sumlx = 0.0f, suml2 = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int l = clampi(rne_int(iscale * x[i]), -32, 31);
        L[i] = l + 32;
        const float w = x[i] * x[i];
        sumlx += w * x[i] * (float)l;
        suml2 += w * (float)l * (float)l;
    }
    float scale = suml2 != 0.0f ? sumlx / suml2 : 0.0f;
    float best = scale * sumlx;
#pragma unroll 1
    for (int is = -9; is <= 9; ++is) {
        if (is == 0) continue;
        iscale = -(32.0f + 0.1f * (float)is) / vmax;
        sumlx = 0.0f;
        suml2 = 0.0f;
        int cand[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int l = clampi(rne_int(iscale * x[i]), -32, 31);
            cand[i] = l + 32;
            const float w = x[i] * x[i];
            sumlx += w * x[i] * (float)l;
            suml2 += w * (float)l * (float)l;
        }
        if (suml2 > 0.0f && sumlx * sumlx > best * suml2) {
#pragma unroll
            for (int i = 0; i < 16; ++i) L[i] = cand[i];
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

// One super-block per sixteen neighbouring lanes, one 16-value group per lane: sixteen group scales, the
// first of largest magnitude mapping to -128 in int8 (d in fp16 keeps its sign), levels assigned again with
// the STORED scales, handed over through LDS and packed as quantized.cu:1103-1128 reads them (ql: low
// nibbles of two quarters per byte, qh: the two high bits of four quarters), each lane storing 8 bytes of
// ql, 4 of qh and its scale.  Lanes past the last super-block work on zeros and store nothing.
__global__ __launch_bounds__(256) void k_wquant_q6_k(const float *__restrict__ x, int64_t nb, BlockQ6K *__restrict__ out) {
    __shared__ __align__(16) uint8_t s_levels[16][256];
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t b = t >> 4;
    const int g = (int)(t & 15);
    const bool live = b < nb;
    float xs[16];
    {
        const float4 *src = (const float4 *)(x + 256 * b + 16 * g);
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            const float4 v = live ? src[l] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            xs[4 * l] = v.x, xs[4 * l + 1] = v.y, xs[4 * l + 2] = v.z, xs[4 * l + 3] = v.w;
        }
    }
    int L[16];
    const float scale = search_symmetric16(xs, L);
    float max_abs = fabsf(scale), max_scale = scale;
    int max_at = g;
#pragma unroll
    for (int o = 1; o < 16; o <<= 1) {
        const float oa = __shfl_xor(max_abs, o), os = __shfl_xor(max_scale, o);
        const int oi = __shfl_xor(max_at, o);
        if (oa > max_abs || (oa == max_abs && oi < max_at)) max_abs = oa, max_scale = os, max_at = oi;
    }
    const bool zero = max_abs < 1e-15f;  // the whole super-block is stored as zero bytes
    const float iscale = -128.0f / max_scale;
    const uint16_t dh = zero ? (uint16_t)0 : f32_to_half_bits(1.0f / iscale);
    const int v = rne_int(iscale * scale);
    const int sc8 = zero ? 0 : (int)(int8_t)(v < 127 ? v : 127);
    const float d = half_bits_to_float(dh) * (float)sc8;
    if (d != 0.0f) {
#pragma unroll
        for (int i = 0; i < 16; ++i) L[i] = clampi(rne_int(xs[i] / d), -32, 31) + 32;
    }
    uint8_t *mine = s_levels[threadIdx.x >> 4];
    {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            w[i] = (uint32_t)(L[4 * i] | (L[4 * i + 1] << 8) | (L[4 * i + 2] << 16) | (L[4 * i + 3] << 24));
            if (zero) w[i] = 0;
        }
        *(uint4 *)(mine + 16 * g) = make_uint4(w[0], w[1], w[2], w[3]);
    }
    __syncthreads();
    if (!live) return;
    BlockQ6K *y = out + b;
    if (g == 0) y->d = dh;
    y->scales[g] = (int8_t)sc8;
    {  // ql bytes 8g .. 8g + 7: byte 64h + r = level (128h + r) low nibble | level (128h + 64 + r) low nibble << 4
        const int h = g >> 3, r = (8 * g) & 63;
        const uint2 lo = *(const uint2 *)(mine + 128 * h + r), hi = *(const uint2 *)(mine + 128 * h + 64 + r);
        const uint32_t q0 = (lo.x & 0x0F0F0F0Fu) | ((hi.x & 0x0F0F0F0Fu) << 4);
        const uint32_t q1 = (lo.y & 0x0F0F0F0Fu) | ((hi.y & 0x0F0F0F0Fu) << 4);
        uint16_t *dst = (uint16_t *)(y->ql + 8 * g);
        dst[0] = (uint16_t)q0, dst[1] = (uint16_t)(q0 >> 16), dst[2] = (uint16_t)q1, dst[3] = (uint16_t)(q1 >> 16);
    }
    {  // qh bytes 4g .. 4g + 3: byte 32h + l = bits 4-5 of levels 128h + 32q + l, q = 0..3, two bits each
        const int h = g >> 3, l = (4 * g) & 31;
        uint32_t q = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t a = *(const uint32_t *)(mine + 128 * h + 32 * k + l);
            q |= ((a >> 4) & 0x03030303u) << (2 * k);
        }
        uint16_t *dst = (uint16_t *)(y->qh + 4 * g);
        dst[0] = (uint16_t)q, dst[1] = (uint16_t)(q >> 16);
    }
}

}  // namespace candy

using namespace candy;

int candy_hip_quantize(candy_hip_device *dev, int fmt, const float *dev_x, int64_t rows, int64_t cols, void *dev_out_blocks) {
    CANDY_REQUIRE(dev, "device is nil");
    const int qk = candy_hip_block_elems(fmt);
    CANDY_REQUIRE(qk != 0, "unknown block format %d", fmt);
    CANDY_REQUIRE(rows >= 0 && cols >= 0, "invalid matrix dimensions");
    CANDY_REQUIRE(cols % qk == 0, "cols %lld is not a multiple of the block size %d", (long long)cols, qk);
    if (fmt == CANDY_HIP_Q8_0) return candy_hip_quantize_q8_0(dev, dev_x, rows, cols, dev_out_blocks);
    if (rows * cols == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(dev_x && dev_out_blocks, "nil pointer");
    CANDY_REQUIRE(((uintptr_t)dev_x & 15) == 0, "input must be 16-byte aligned");
    CANDY_REQUIRE(((uintptr_t)dev_out_blocks & 1) == 0, "output blocks must be 2-byte aligned");
    if (int rc = use_device(dev)) return rc;
    const int64_t nb = rows * cols / qk;
    const int per = qk == 32 ? 256 : (fmt == CANDY_HIP_Q4_K ? 32 : 16);
    const int64_t grid = (nb + per - 1) / per;
    CANDY_REQUIRE(grid <= 0x7FFFFFFF, "matrix too large");
    switch (fmt) {
    case CANDY_HIP_Q4_0:
    case CANDY_HIP_Q4_0_GGML:
        hipLaunchKernelGGL(k_wquant_q4_0, dim3((unsigned)grid), dim3(256), 0, dev->stream, dev_x, nb,
                           (BlockQ4_0 *)dev_out_blocks, fmt == CANDY_HIP_Q4_0_GGML ? 1 : 0);
        break;
    case CANDY_HIP_Q4_K:
        hipLaunchKernelGGL(k_wquant_q4_k, dim3((unsigned)grid), dim3(256), 0, dev->stream, dev_x, nb, (BlockQ4K *)dev_out_blocks);
        break;
    case CANDY_HIP_Q6_K:
        hipLaunchKernelGGL(k_wquant_q6_k, dim3((unsigned)grid), dim3(256), 0, dev->stream, dev_x, nb, (BlockQ6K *)dev_out_blocks);
        break;
    default: CANDY_REQUIRE(false, "no quantizer for format %d", fmt);
    }
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}
