// The reference's other dequantize outputs and its second matvec:
//   * dequantize_block_*_f16 (tensor/internal/cuda/kernels/kernels.go:486-505; template quantized.cu:1229-1249 and
//     the per-format K-quant kernels with dst_t = half): every value is computed in f32 exactly as for the f32
//     output and converted to fp16 on the store (round to nearest even);
//   * DequantizeBlockQ4_0F64 / Q4_1F64 / Q8_0F64 (tensor/internal/cpu/kernels/quantized.go:96-104, 119-128, 139-144):
//     the f32-widened scale times the level in float64;
//   * dequantize_mul_mat_vec (quantized.cu:1251-1345 for the 32-value formats, :1550-1693 q4_K, :1810-1911 q6_K):
//     y[row] = sum_k dequant(W)[row, k] * x[k] with f32 activations, no activation quantizer.
#include "blocks.h"
#include "formats_more.h"
#include "internal.h"

namespace candy {

// ------------------------------------------------------------------ four consecutive values of the main formats
// (the f32 dequantize kernels of these formats have their own lane maps; these give the same values)
template <bool GGML_ORDER>
struct FmtQ4_0 {
    static constexpr int ELEMS = 32, BYTES = 18;
    __device__ static __forceinline__ float4 quad(const uint8_t *blk, int j) {
        const BlockQ4_0 *b = (const BlockQ4_0 *)blk;
        const float d = half_bits_to_float(b->d);
        if (GGML_ORDER) {  // quantized.cu:862-866
            const uint32_t q = load_u32_a2(b->qs + 4 * (j & 3)) >> (j >= 4 ? 4 : 0);
            const float dm = -8.0f * d;
            return make_float4(d * (float)(q & 0xF) + dm, d * (float)((q >> 8) & 0xF) + dm, d * (float)((q >> 16) & 0xF) + dm,
                               d * (float)((q >> 24) & 0xF) + dm);
        }
        const uint32_t q = *(const uint16_t *)(b->qs + 2 * j);  // quantized.go:85-93
        return make_float4(d * ((float)(q & 0xF) - 8.0f), d * ((float)((q >> 4) & 0xF) - 8.0f),
                           d * ((float)((q >> 8) & 0xF) - 8.0f), d * ((float)(q >> 12) - 8.0f));
    }
};
struct FmtQ8_0 {
    static constexpr int ELEMS = 32, BYTES = 34;
    __device__ static __forceinline__ float4 quad(const uint8_t *blk, int j) {  // quantized.go:131-136
        const BlockQ8_0 *b = (const BlockQ8_0 *)blk;
        const float d = half_bits_to_float(b->d);
        const uint32_t q = load_u32_a2((const uint8_t *)b->qs + 4 * j);
        return make_float4(d * (float)(int8_t)(q & 0xFF), d * (float)(int8_t)((q >> 8) & 0xFF),
                           d * (float)(int8_t)((q >> 16) & 0xFF), d * (float)(int8_t)(q >> 24));
    }
};
struct FmtQ4K {
    static constexpr int ELEMS = 256, BYTES = 144;
    __device__ static __forceinline__ float4 quad(const uint8_t *blk, int j) {  // quantized.cu:1008-1041
        const uint32_t *w = (const uint32_t *)blk;
        const int il = j >> 4, hi = (j >> 3) & 1, ir = j & 7;  // 64-value group, nibble half, dword of the group
        uint32_t sc2, m2;
        q4k_scale_min_pair(w[1], w[2], w[3], il, sc2, m2);
        const float dall = half_bits_to_float((uint16_t)(w[0] & 0xFFFF)), dmin = half_bits_to_float((uint16_t)(w[0] >> 16));
        const float d = dall * (float)(hi ? sc2 >> 8 : sc2 & 0xFF), m = dmin * (float)(hi ? m2 >> 8 : m2 & 0xFF);
        const uint32_t q = w[4 + il * 8 + ir] >> (4 * hi);
        return make_float4(d * (float)(q & 0xF) - m, d * (float)((q >> 8) & 0xF) - m, d * (float)((q >> 16) & 0xF) - m,
                           d * (float)((q >> 24) & 0xF) - m);
    }
};
struct FmtQ6K {
    static constexpr int ELEMS = 256, BYTES = 210;
    __device__ static __forceinline__ float4 quad(const uint8_t *blk, int j) {  // quantized.cu:1103-1128
        const BlockQ6K *b = (const BlockQ6K *)blk;
        const int ip = j >> 5, qd = (j >> 3) & 3, l0 = (j & 7) * 4;  // half, 32-value quarter, first of four lanes
        const uint32_t ql = load_u32_a2(b->ql + 64 * ip + 32 * (qd & 1) + l0) >> (qd >= 2 ? 4 : 0);
        const uint32_t qh = load_u32_a2(b->qh + 32 * ip + l0) >> (2 * qd);
        const float s = half_bits_to_float(b->d) * (float)b->scales[8 * ip + (l0 >> 4) + 2 * qd];
        float v[4];
#pragma unroll
        for (int l = 0; l < 4; ++l)
            v[l] = s * (float)((int)(((ql >> (8 * l)) & 0xF) | (((qh >> (8 * l)) & 3) << 4)) - 32);
        return make_float4(v[0], v[1], v[2], v[3]);
    }
};

// ------------------------------------------------------------------ fp16 output
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
template <class F>
__global__ __launch_bounds__(256) void k_dequant_f16(const uint8_t *__restrict__ blocks, int64_t nb, half4v *__restrict__ y) {
    constexpr int LPB = F::ELEMS / 4;
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t b = t / LPB;
    if (b >= nb) return;
    float4 v = F::quad(blocks + b * F::BYTES, (int)(t - b * LPB));
    // the f32 values first, then the conversion: left alone, the compiler folds multiply and conversion into a
    // mixed-precision fma with a +0 addend, which turns the -0 of a zero scale into +0
    asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w));
    y[t] = half4v{(_Float16)v.x, (_Float16)v.y, (_Float16)v.z, (_Float16)v.w};
}
template <class F>
static int launch_dequant_f16(candy_hip_device *dev, const void *blocks, int64_t nb, void *out) {
    const int64_t grid = (nb * (F::ELEMS / 4) + 255) / 256;
    CANDY_REQUIRE(grid <= 0x7FFFFFFF, "too many blocks");
    hipLaunchKernelGGL(k_dequant_f16<F>, dim3((unsigned)grid), dim3(256), 0, dev->stream, (const uint8_t *)blocks, nb,
                       (half4v *)out);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

// ------------------------------------------------------------------ float64 output (Q4_0, Q4_1, Q8_0: the formats the
// CPU kernels have float64 twins of); 8 lanes per block, four doubles each.  d * level is exact in float64
// (an fp16 mantissa times at most 8 bits), so the Q4_1 sum is rounded once, fused or not.
template <int FMT>
__global__ __launch_bounds__(256) void k_dequant_f64(const uint8_t *__restrict__ blocks, int64_t nb, double *__restrict__ y) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t b = t >> 3;
    if (b >= nb) return;
    const int j = (int)(t & 7);
    double v[4];
    if (FMT == CANDY_HIP_Q4_0) {
        const BlockQ4_0 *blk = (const BlockQ4_0 *)blocks + b;
        const double d = (double)half_bits_to_float(blk->d);
        const uint32_t q = *(const uint16_t *)(blk->qs + 2 * j);
        v[0] = d * ((double)(q & 0xF) - 8.0); v[1] = d * ((double)((q >> 4) & 0xF) - 8.0);
        v[2] = d * ((double)((q >> 8) & 0xF) - 8.0); v[3] = d * ((double)(q >> 12) - 8.0);
    } else if (FMT == CANDY_HIP_Q4_1) {
        const BlockQ4_1 *blk = (const BlockQ4_1 *)blocks + b;
        const double d = (double)half_bits_to_float(blk->d), m = (double)half_bits_to_float(blk->m);
        const uint32_t q = (uint32_t)blk->qs[2 * j] | ((uint32_t)blk->qs[2 * j + 1] << 8);
        v[0] = d * (double)(q & 0xF) + m; v[1] = d * (double)((q >> 4) & 0xF) + m;
        v[2] = d * (double)((q >> 8) & 0xF) + m; v[3] = d * (double)(q >> 12) + m;
    } else {
        const BlockQ8_0 *blk = (const BlockQ8_0 *)blocks + b;
        const double d = (double)half_bits_to_float(blk->d);
#pragma unroll
        for (int l = 0; l < 4; ++l) v[l] = d * (double)blk->qs[4 * j + l];
    }
    double2 *out = (double2 *)(y + t * 4);
    out[0] = make_double2(v[0], v[1]);
    out[1] = make_double2(v[2], v[3]);
}

// ------------------------------------------------------------------ f32-activation matvec
// A wavefront takes R weight rows at a time (their loads are in flight together), four wavefronts per workgroup; a
// lane takes every 64th group of four values, so a wavefront's loads of x and of a row are consecutive.  Partial
// sums meet in a DPP tree (f32 order differs from the reference's own 32-thread tree; the per-value products are
// the reference's).
template <class F, int R>
__global__ __launch_bounds__(256) void k_dmmv(const uint8_t *__restrict__ W, const float4 *__restrict__ x, float *__restrict__ y,
                                               int rows, int cols) {
    constexpr int LPB = F::ELEMS / 4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nq = cols >> 2;
    const size_t rb = (size_t)(cols / F::ELEMS) * F::BYTES;
    for (int row0 = (blockIdx.x * 4 + wave) * R; row0 < rows; row0 += gridDim.x * 4 * R) {
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r] = 0.0f;
        for (int t = lane; t < nq; t += 64) {
            const int b = t / LPB;
            const float4 xv = x[t];
            float4 w[R];
#pragma unroll
            for (int r = 0; r < R; ++r)  // rows past the end repeat the last one and are not stored
                w[r] = F::quad(W + (size_t)min(row0 + r, rows - 1) * rb + (size_t)b * F::BYTES, t - b * LPB);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                acc[r] = fmaf(w[r].x, xv.x, acc[r]); acc[r] = fmaf(w[r].y, xv.y, acc[r]);
                acc[r] = fmaf(w[r].z, xv.z, acc[r]); acc[r] = fmaf(w[r].w, xv.w, acc[r]);
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float sum = wave_sum(acc[r]);
            if (lane == 0 && row0 + r < rows) y[row0 + r] = sum;
        }
    }
}

// Q4_K: a lane takes 16 bytes of a super-block's nibbles (16 values of each of two sub-blocks), eight lanes a
// super-block; the scales are unpacked once per 32 values instead of once per 4.
template <int R>
__global__ __launch_bounds__(256) void k_dmmv_q4k(const uint8_t *__restrict__ W, const float4 *__restrict__ x,
                                                   float *__restrict__ y, int rows, int cols) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nsb = cols >> 8;
    const size_t rb = (size_t)nsb * 144;
    const int il = (lane >> 1) & 3, half16 = lane & 1;  // 64-value group of the super-block, which 16 bytes of its 32
    for (int row0 = (blockIdx.x * 4 + wave) * R; row0 < rows; row0 += gridDim.x * 4 * R) {
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r] = 0.0f;
        for (int sb = lane >> 3; sb < nsb; sb += 8) {
            u32x4 h[R], q[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t *w = (const uint32_t *)(W + (size_t)min(row0 + r, rows - 1) * rb + (size_t)sb * 144);
                h[r] = *(const u32x4 *)w;
                q[r] = *(const u32x4 *)(w + 4 + il * 8 + half16 * 4);
            }
            const float4 *xl = x + sb * 64 + il * 16 + half16 * 4, *xh = xl + 8;
            float av[16], bv[16];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float4 a = xl[i], b = xh[i];
                av[4 * i] = a.x; av[4 * i + 1] = a.y; av[4 * i + 2] = a.z; av[4 * i + 3] = a.w;
                bv[4 * i] = b.x; bv[4 * i + 1] = b.y; bv[4 * i + 2] = b.z; bv[4 * i + 3] = b.w;
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                uint32_t sc2, m2;
                q4k_scale_min_pair(h[r].y, h[r].z, h[r].w, il, sc2, m2);
                const float dall = half_bits_to_float((uint16_t)(h[r].x & 0xFFFF)), dmin = half_bits_to_float((uint16_t)(h[r].x >> 16));
                const float d1 = dall * (float)(sc2 & 0xFF), m1 = dmin * (float)(m2 & 0xFF);
                const float d2 = dall * (float)(sc2 >> 8), m2f = dmin * (float)(m2 >> 8);
                const uint32_t qq[4] = {q[r].x, q[r].y, q[r].z, q[r].w};
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int l = 0; l < 4; ++l) {
                        acc[r] = fmaf(d1 * (float)((qq[i] >> (8 * l)) & 0xF) - m1, av[4 * i + l], acc[r]);
                        acc[r] = fmaf(d2 * (float)((qq[i] >> (8 * l + 4)) & 0xF) - m2f, bv[4 * i + l], acc[r]);
                    }
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float sum = wave_sum(acc[r]);
            if (lane == 0 && row0 + r < rows) y[row0 + r] = sum;
        }
    }
}

static unsigned dmmv_grid(const candy_hip_device *dev, int64_t rows, int R) {
    return (unsigned)std::min<int64_t>((rows + 4 * R - 1) / (4 * R), 16 * (int64_t)dev->num_cus);
}

// rows a wavefront takes at a time: more share each load of x, fewer leave more wavefronts (at least two per SIMD)
template <class F>
static int launch_dmmv(candy_hip_device *dev, const candy_hip_qtensor *w, const float *x, float *y) {
    const int rows = (int)w->rows, cols = (int)w->cols;
    const int64_t per_two = 2 * 4 * (int64_t)dev->num_cus;
    if (rows >= 2 * per_two)
        hipLaunchKernelGGL((k_dmmv<F, 2>), dim3(dmmv_grid(dev, rows, 2)), dim3(256), 0, dev->stream, (const uint8_t *)w->data,
                           (const float4 *)x, y, rows, cols);
    else
        hipLaunchKernelGGL((k_dmmv<F, 1>), dim3(dmmv_grid(dev, rows, 1)), dim3(256), 0, dev->stream, (const uint8_t *)w->data,
                           (const float4 *)x, y, rows, cols);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

static int launch_dmmv_q4k(candy_hip_device *dev, const candy_hip_qtensor *w, const float *x, float *y) {
    const int rows = (int)w->rows, cols = (int)w->cols;
    const int64_t per_two = 2 * 4 * (int64_t)dev->num_cus;
    const uint8_t *W = (const uint8_t *)w->data;
    if (rows >= 4 * per_two)
        hipLaunchKernelGGL(k_dmmv_q4k<4>, dim3(dmmv_grid(dev, rows, 4)), dim3(256), 0, dev->stream, W, (const float4 *)x, y, rows, cols);
    else if (rows >= 2 * per_two)
        hipLaunchKernelGGL(k_dmmv_q4k<2>, dim3(dmmv_grid(dev, rows, 2)), dim3(256), 0, dev->stream, W, (const float4 *)x, y, rows, cols);
    else
        hipLaunchKernelGGL(k_dmmv_q4k<1>, dim3(dmmv_grid(dev, rows, 1)), dim3(256), 0, dev->stream, W, (const float4 *)x, y, rows, cols);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

}  // namespace candy

using namespace candy;

extern "C" {

int candy_hip_dequantize_blocks_f16(candy_hip_device *dev, int fmt, const void *dev_blocks, int64_t n_blocks, void *dev_out) {
    FormatInfo fi = format_info(fmt);
    CANDY_REQUIRE(dev, "device handle is nil");
    CANDY_REQUIRE(fi.elems != 0, "unknown quantized format %d", fmt);
    CANDY_REQUIRE(n_blocks >= 0, "negative block count");
    if (n_blocks == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(dev_blocks && dev_out, "nil pointer");
    CANDY_REQUIRE(((uintptr_t)dev_out & 7) == 0, "output must be 8-byte aligned");
    CANDY_REQUIRE(((uintptr_t)dev_blocks & (uintptr_t)(block_alignment(fmt) - 1)) == 0, "blocks are misaligned");
    if (int rc = use_device(dev)) return rc;
    switch (fmt) {
    case CANDY_HIP_Q4_0: return launch_dequant_f16<FmtQ4_0<false>>(dev, dev_blocks, n_blocks, dev_out);
    case CANDY_HIP_Q4_0_GGML: return launch_dequant_f16<FmtQ4_0<true>>(dev, dev_blocks, n_blocks, dev_out);
    case CANDY_HIP_Q8_0: return launch_dequant_f16<FmtQ8_0>(dev, dev_blocks, n_blocks, dev_out);
    case CANDY_HIP_Q4_K: return launch_dequant_f16<FmtQ4K>(dev, dev_blocks, n_blocks, dev_out);
    case CANDY_HIP_Q6_K: return launch_dequant_f16<FmtQ6K>(dev, dev_blocks, n_blocks, dev_out);
    case CANDY_HIP_Q4_1: return launch_dequant_f16<FmtQ4_1<false>>(dev, dev_blocks, n_blocks, dev_out);
    case CANDY_HIP_Q4_1_GGML: return launch_dequant_f16<FmtQ4_1<true>>(dev, dev_blocks, n_blocks, dev_out);
    case CANDY_HIP_Q5_0: return launch_dequant_f16<FmtQ5<false>>(dev, dev_blocks, n_blocks, dev_out);
    case CANDY_HIP_Q5_1: return launch_dequant_f16<FmtQ5<true>>(dev, dev_blocks, n_blocks, dev_out);
    case CANDY_HIP_Q2_K: return launch_dequant_f16<FmtQ2K>(dev, dev_blocks, n_blocks, dev_out);
    case CANDY_HIP_Q3_K: return launch_dequant_f16<FmtQ3K>(dev, dev_blocks, n_blocks, dev_out);
    case CANDY_HIP_Q5_K: return launch_dequant_f16<FmtQ5K>(dev, dev_blocks, n_blocks, dev_out);
    case CANDY_HIP_Q8_K: return launch_dequant_f16<FmtQ8K>(dev, dev_blocks, n_blocks, dev_out);
    default: break;
    }
    return fail(CANDY_HIP_ERR_UNSUPPORTED, "no fp16 dequantize for format %d", fmt);
}

int candy_hip_dequantize_f16(candy_hip_device *dev, const candy_hip_qtensor *q, void *dev_out) {
    CANDY_REQUIRE(q, "qtensor is nil");
    CANDY_REQUIRE(dev && q->dev == dev, "qtensor lives on another device handle");
    return candy_hip_dequantize_blocks_f16(dev, q->fmt, q->data, q->rows * (q->cols / format_info(q->fmt).elems), dev_out);
}

int candy_hip_dequantize_blocks_f64(candy_hip_device *dev, int fmt, const void *dev_blocks, int64_t n_blocks, double *dev_out) {
    CANDY_REQUIRE(dev, "device handle is nil");
    CANDY_REQUIRE(format_info(fmt).elems != 0, "unknown quantized format %d", fmt);
    if (fmt != CANDY_HIP_Q4_0 && fmt != CANDY_HIP_Q4_1 && fmt != CANDY_HIP_Q8_0)
        return fail(CANDY_HIP_ERR_UNSUPPORTED, "float64 dequantize exists for Q4_0, Q4_1 and Q8_0 only, got format %d", fmt);
    CANDY_REQUIRE(n_blocks >= 0, "negative block count");
    if (n_blocks == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(dev_blocks && dev_out, "nil pointer");
    CANDY_REQUIRE(((uintptr_t)dev_out & 15) == 0, "output must be 16-byte aligned");
    CANDY_REQUIRE(((uintptr_t)dev_blocks & (uintptr_t)(block_alignment(fmt) - 1)) == 0, "blocks are misaligned");
    if (int rc = use_device(dev)) return rc;
    const int64_t grid = (n_blocks * 8 + 255) / 256;
    CANDY_REQUIRE(grid <= 0x7FFFFFFF, "too many blocks");
    const dim3 g((unsigned)grid), b(256);
    if (fmt == CANDY_HIP_Q4_0)
        hipLaunchKernelGGL(k_dequant_f64<CANDY_HIP_Q4_0>, g, b, 0, dev->stream, (const uint8_t *)dev_blocks, n_blocks, dev_out);
    else if (fmt == CANDY_HIP_Q4_1)
        hipLaunchKernelGGL(k_dequant_f64<CANDY_HIP_Q4_1>, g, b, 0, dev->stream, (const uint8_t *)dev_blocks, n_blocks, dev_out);
    else
        hipLaunchKernelGGL(k_dequant_f64<CANDY_HIP_Q8_0>, g, b, 0, dev->stream, (const uint8_t *)dev_blocks, n_blocks, dev_out);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int candy_hip_dmmv(candy_hip_device *dev, const candy_hip_qtensor *w, const float *dev_x, float *dev_y) {
    CANDY_REQUIRE(w, "rhs qtensor is nil");
    CANDY_REQUIRE(dev && w->dev == dev, "rhs storage must live on the same HIP device");
    CANDY_REQUIRE(dev_x && dev_y, "nil pointer");
    CANDY_REQUIRE(((uintptr_t)dev_x & 15) == 0, "lhs must be 16-byte aligned");
    CANDY_REQUIRE(w->rows <= 0x7FFFFFFF && w->cols <= 0x7FFFFFFF, "matrix too large");
    if (w->rows == 0) return CANDY_HIP_OK;
    if (int rc = use_device(dev)) return rc;
    switch (w->fmt) {
    case CANDY_HIP_Q4_K: return launch_dmmv_q4k(dev, w, dev_x, dev_y);
    case CANDY_HIP_Q4_0: return launch_dmmv<FmtQ4_0<false>>(dev, w, dev_x, dev_y);
    case CANDY_HIP_Q4_0_GGML: return launch_dmmv<FmtQ4_0<true>>(dev, w, dev_x, dev_y);
    case CANDY_HIP_Q8_0: return launch_dmmv<FmtQ8_0>(dev, w, dev_x, dev_y);
    case CANDY_HIP_Q6_K: return launch_dmmv<FmtQ6K>(dev, w, dev_x, dev_y);
    case CANDY_HIP_Q4_1: return launch_dmmv<FmtQ4_1<false>>(dev, w, dev_x, dev_y);
    case CANDY_HIP_Q4_1_GGML: return launch_dmmv<FmtQ4_1<true>>(dev, w, dev_x, dev_y);
    case CANDY_HIP_Q5_0: return launch_dmmv<FmtQ5<false>>(dev, w, dev_x, dev_y);
    case CANDY_HIP_Q5_1: return launch_dmmv<FmtQ5<true>>(dev, w, dev_x, dev_y);
    case CANDY_HIP_Q2_K: return launch_dmmv<FmtQ2K>(dev, w, dev_x, dev_y);
    case CANDY_HIP_Q3_K: return launch_dmmv<FmtQ3K>(dev, w, dev_x, dev_y);
    case CANDY_HIP_Q5_K: return launch_dmmv<FmtQ5K>(dev, w, dev_x, dev_y);
    default: break;
    }
    return fail(CANDY_HIP_ERR_UNSUPPORTED, "no f32-activation matvec for format %d", w->fmt);
}

}  // extern "C"
