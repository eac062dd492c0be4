// f32 ops of the decode step, one per BackendStorage method a Llama block calls (backend.go).
// Semantics follow candy's CPU kernels (tensor/internal/cpu/kernels/reduce.go, unary.go,
// binary.go, indexing.go, conv.go); reductions run in parallel, so sums differ from the
// sequential CPU loops by f32 rounding only.
#include "blocks.h"
#include "internal.h"

namespace candy {

// Sum / max across a workgroup of up to 1024 threads; every thread gets the result.
template <bool IS_MAX>
__device__ __forceinline__ float block_reduce(float v, float *red) {
    v = IS_MAX ? wave_max(v) : wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();  // red may still be read from a previous reduction
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = IS_MAX ? -3.402823466e+38f : 0.0f;
    for (int i = 0; i < nw; ++i) t = IS_MAX ? fmaxf(t, red[i]) : t + red[i];
    return t;
}

// reduce.go:3071-3092: mean of squares, eps inside the square root (taken in f64), scale*x*alpha.
__global__ __launch_bounds__(256) void k_rms_norm(const float *__restrict__ x, const float *__restrict__ alpha,
                                                  float eps, int cols, float *__restrict__ out) {
    __shared__ float red[16];
    const float *xr = x + (size_t)blockIdx.x * cols;
    float *orow = out + (size_t)blockIdx.x * cols;
    float s = 0.0f;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) s += xr[c] * xr[c];
    s = block_reduce<false>(s, red);
    const float mean = s / (float)cols;
    const float scale = rms_inv_sqrt(mean + eps);
    for (int c = threadIdx.x; c < cols; c += blockDim.x)
        orow[c] = alpha ? scale * xr[c] * alpha[c] : scale * xr[c];
}

// reduce.go:3987-4006
__global__ __launch_bounds__(256) void k_rope(const float *__restrict__ src, const float *__restrict__ cos_t,
                                              const float *__restrict__ sin_t, int64_t num_pairs, int64_t td,
                                              int64_t d, int64_t stride_b, float *__restrict__ dst) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= num_pairs) return;
    const int64_t half_td = td / 2, half_d = d / 2;
    const int64_t i_bh = idx / half_td;
    const int64_t i_td = idx - half_td * i_bh;
    const int64_t i_t = i_td / half_d;
    const int64_t i_d = i_td - half_d * i_t;
    const int64_t i1 = i_bh * td + i_t * d + i_d;
    const int64_t i2 = i1 + half_d;
    int64_t i_cs = i_t * half_d + i_d;
    if (stride_b > 0) i_cs += ((2 * idx) / stride_b) * half_td;
    const float c = cos_t[i_cs], s = sin_t[i_cs];
    const float a = src[i1], b = src[i2];
    dst[i1] = a * c - b * s;
    dst[i2] = a * s + b * c;
}

// reduce.go:3825-3838 (rope_i): adjacent pairs (2i, 2i + 1)
__global__ __launch_bounds__(256) void k_rope_i(const float2 *__restrict__ src, const float *__restrict__ cos_t,
                                                const float *__restrict__ sin_t, int64_t num_pairs, int64_t half_td,
                                                int64_t stride_b, float2 *__restrict__ dst) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= num_pairs) return;
    int64_t rope_idx = idx % half_td;
    if (stride_b > 0) rope_idx += ((2 * idx) / stride_b) * half_td;
    const float c = cos_t[rope_idx], s = sin_t[rope_idx];
    const float2 v = src[idx];
    dst[idx] = make_float2(v.x * c - v.y * s, v.x * s + v.y * c);
}

// reduce.go:4178-4196 (rope_thd): [b, t, h, d], pairs (i, i + d/2), cos / sin rows by the token index
__global__ __launch_bounds__(256) void k_rope_thd(const float *__restrict__ src, const float *__restrict__ cos_t,
                                                  const float *__restrict__ sin_t, int64_t num_pairs, int64_t t, int64_t h,
                                                  int64_t d, int64_t stride_b, float *__restrict__ dst) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= num_pairs) return;
    const int64_t half_d = d / 2;
    const int64_t i_bth = idx / half_d;
    const int64_t i_d = idx - half_d * i_bth;
    const int64_t i_t = (i_bth / h) % t;
    const int64_t i1 = i_bth * d + i_d, i2 = i1 + half_d;
    int64_t i_cs = i_t * half_d + i_d;
    if (stride_b > 0) i_cs += ((2 * idx) / stride_b) * ((t * d) / 2);
    const float c = cos_t[i_cs], s = sin_t[i_cs];
    const float a = src[i1], b = src[i2];
    dst[i1] = a * c - b * s;
    dst[i2] = a * s + b * c;
}

// reduce.go:2855-2879: max, exp(x - max), multiply by 1/sum.
__global__ __launch_bounds__(256) void k_softmax(const float *__restrict__ src, int cols, float *__restrict__ dst) {
    __shared__ float red[16];
    const float *xr = src + (size_t)blockIdx.x * cols;
    float *orow = dst + (size_t)blockIdx.x * cols;
    float m = -3.402823466e+38f;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) m = fmaxf(m, xr[c]);
    m = block_reduce<true>(m, red);
    float s = 0.0f;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) {
        const float e = expf(xr[c] - m);
        orow[c] = e;
        s += e;
    }
    s = block_reduce<false>(s, red);
    const float inv = 1.0f / s;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) orow[c] *= inv;
}

// unary.go:3353-3366: x / (1 + exp(-x))
__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }

enum { EW_SILU = 0, EW_ADD = 1, EW_MUL = 2, EW_SILU_MUL = 3 };
template <int OP>
__global__ __launch_bounds__(256) void k_elementwise(const float *__restrict__ a, const float *__restrict__ b,
                                                     int64_t n, float *__restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float r;
    if (OP == EW_SILU) r = silu_f(a[i]);
    else if (OP == EW_ADD) r = a[i] + b[i];
    else if (OP == EW_MUL) r = a[i] * b[i];
    else r = silu_f(a[i]) * b[i];
    out[i] = r;
}

// reduce.go:846-862: index of the first maximum (strict > against -MaxFloat32, so a row of
// -inf or NaN yields 0).
__global__ __launch_bounds__(1024) void k_argmax(const float *__restrict__ src, int cols, uint32_t *__restrict__ out) {
    __shared__ float sv[16];
    __shared__ uint32_t si[16];
    const float *xr = src + (size_t)blockIdx.x * cols;
    float best = -3.402823466e+38f;
    uint32_t bi = 0xFFFFFFFFu;
    if ((cols & 3) == 0 && ((uintptr_t)xr & 15) == 0) {
        // sixteen independent 16-byte loads in flight per thread: one block has to cover a whole vocabulary row, and
        // every round of loads is a memory latency (128256 logits: two rounds; with four loads per round 13 us)
        constexpr int U = 16;
        const float4 *x4 = (const float4 *)xr;
        const int n4 = cols >> 2, step = (int)blockDim.x;
        for (int c0 = threadIdx.x; c0 < n4; c0 += U * step) {
            float4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = x4[min(c0 + u * step, n4 - 1)];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int c = c0 + u * step;
                const bool in = c < n4;  // past the row: the clamped load is a value already seen at a lower index
                // ascending index within the thread, strict >: the first maximum wins
                if (in && v[u].x > best) { best = v[u].x; bi = (uint32_t)(4 * c); }
                if (in && v[u].y > best) { best = v[u].y; bi = (uint32_t)(4 * c + 1); }
                if (in && v[u].z > best) { best = v[u].z; bi = (uint32_t)(4 * c + 2); }
                if (in && v[u].w > best) { best = v[u].w; bi = (uint32_t)(4 * c + 3); }
            }
        }
    } else {
        for (int c = threadIdx.x; c < cols; c += blockDim.x) {
            const float v = xr[c];
            if (v > best) { best = v; bi = (uint32_t)c; }
        }
    }
    // lexicographic (value desc, index asc) reduction
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off, 64);
        const uint32_t oi = __shfl_xor(bi, off, 64);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if (lane == 0) { sv[wave] = best; si[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < nw; ++i)
            if (sv[i] > best || (sv[i] == best && si[i] < bi)) { best = sv[i]; bi = si[i]; }
        out[blockIdx.x] = bi == 0xFFFFFFFFu ? 0u : bi;
    }
}

// The same choice over many workgroups, for one long row (the decode step's vocabulary): every workgroup reduces
// its part to (value, index) and folds it into one 64-bit word with an atomic maximum - the value's bits made
// monotonic in the upper half, 0xFFFFFFFF - index in the lower, so that the larger value wins and among equal values
// the smaller index, whatever order the workgroups arrive in.  Values that the CPU loop's strict > against
// -MaxFloat32 never selects (NaN, -inf, -MaxFloat32) fold in nothing; a word still zero means index 0
// (argmax_key_index).  The word must be zero before the launch.  One workgroup pulls 128 KB of logits in 6.8 us; this
// takes about 3.
__global__ __launch_bounds__(256) void k_argmax_key(const float *__restrict__ src, int cols, unsigned long long *key) {
    constexpr int U = 2;
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    const int n4 = cols >> 2;  // a 16-byte aligned row (launcher); the last cols % 4 values go to workgroup 0
    const float4 *x4 = (const float4 *)src;
    const int c0 = blockIdx.x * (256 * U) + threadIdx.x;
    float4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = x4[max(min(c0 + 256 * u, n4 - 1), 0)];  // a row shorter than 4: one piece past it (allocated)
    float best = -3.402823466e+38f;
    uint32_t bi = 0xFFFFFFFFu;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int c = c0 + 256 * u;
        const bool in = c < n4;
        if (in && v[u].x > best) { best = v[u].x; bi = (uint32_t)(4 * c); }
        if (in && v[u].y > best) { best = v[u].y; bi = (uint32_t)(4 * c + 1); }
        if (in && v[u].z > best) { best = v[u].z; bi = (uint32_t)(4 * c + 2); }
        if (in && v[u].w > best) { best = v[u].w; bi = (uint32_t)(4 * c + 3); }
    }
    if (blockIdx.x == 0 && (int)threadIdx.x < (cols & 3)) {  // indices past every float4 of this thread
        const float t = src[4 * n4 + threadIdx.x];
        if (t > best) { best = t; bi = (uint32_t)(4 * n4 + threadIdx.x); }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off, 64);
        const uint32_t oi = __shfl_xor(bi, off, 64);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { sv[wave] = best; si[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < 4; ++i)
            if (sv[i] > best || (sv[i] == best && si[i] < bi)) { best = sv[i]; bi = si[i]; }
        if (bi != 0xFFFFFFFFu) {
            const uint32_t b = __float_as_uint(best);
            const uint32_t ordered = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
            atomicMax(key, ((unsigned long long)ordered << 32) | (unsigned long long)(0xFFFFFFFFu - bi));
        }
    }
}

// indexing.go:8-26 along dim 0 of a [n_src, width] table; id == MaxInt64 selects zeros.
// indexing.go:8-26: the MaxInt64 id selects a row of zeros.  Any other id outside [0, n_src) makes the CPU loop
// panic on its bounds check; a kernel cannot, so the row is written as zeros, nothing is read, and the device
// handle's fault word is raised for the next synchronising call to report.
__global__ __launch_bounds__(256) void k_index_select(const float *__restrict__ table, int64_t n_src, int64_t width,
                                                      const int64_t *__restrict__ ids, float *__restrict__ out,
                                                      int *fault) {
    const int64_t id = ids[blockIdx.x];
    const bool in_range = id >= 0 && id < n_src;
    if (!in_range && id != 0x7FFFFFFFFFFFFFFFll && threadIdx.x == 0) *fault = 1;
    float *orow = out + (size_t)blockIdx.x * width;
    for (int64_t c = threadIdx.x; c < width; c += blockDim.x)
        orow[c] = in_range ? table[id * width + c] : 0.0f;
}

// conv.go:251-267 / :373-389: c[b,i,j] = sum_l a[b,i,l] * B[b,l,j]; one output per thread,
// l ascending, single f32 accumulator (the CPU loop's order), the product rounded before it is added (no fused
// multiply-add: the Go compiler does not fuse on amd64), so the result is the CPU loop's bit for bit.
__global__ __launch_bounds__(256) void k_matmul_f32(const float *__restrict__ a, const float *__restrict__ b,
                                                    float *__restrict__ c, int64_t m, int64_t n, int64_t k,
                                                    int rhs_transposed) {
#pragma clang fp contract(off)
    const int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t i = blockIdx.y, bb = blockIdx.z;
    if (j >= n) return;
    const float *ar = a + (bb * m + i) * k;
    const float *bm = b + bb * k * n;
    float sum = 0.0f;
    if (rhs_transposed) {
        const float *br = bm + j * k;
        for (int64_t l = 0; l < k; ++l) sum += ar[l] * br[l];
    } else {
        for (int64_t l = 0; l < k; ++l) sum += ar[l] * bm[l * n + j];
    }
    c[(bb * m + i) * n + j] = sum;
}


// conv.go:373-389 with the strides CpuStorage.MatMul hands it for one batch (cpu/storage.go:893-910: the last two
// strides of each layout): c[i,j] = sum_l a[i*ars + l*acs] * b[l*brs + j*bcs], l ascending, one f32 accumulator.
__global__ __launch_bounds__(256) void k_matmul_f32_strided(const float *__restrict__ a, const float *__restrict__ b,
                                                            float *__restrict__ c, int64_t n, int64_t k, int64_t ars,
                                                            int64_t acs, int64_t brs, int64_t bcs) {
#pragma clang fp contract(off)
    const int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t i = blockIdx.y;
    if (j >= n) return;
    float sum = 0.0f;
    for (int64_t l = 0; l < k; ++l) sum += a[i * ars + l * acs] * b[l * brs + j * bcs];
    c[i * n + j] = sum;
}


// ------------------------------------------------------------------ fused decode-step kernels
// Each produces the planar Q8_0 activations the next quantized Linear consumes, so the f32
// intermediate never makes a round trip through a separate quantize launch.  The arithmetic of
// each stage is the unfused one (RMSNorm: reduce.go:3071-3092; SiLU: unary.go:3353-3366; Mul;
// activation quantization: quantized.cu:3521-3558).

// RMSNorm of one row followed by Q8_0 quantization. cols % 32 == 0. One workgroup per row.
__global__ __launch_bounds__(256) void k_rms_norm_quant(const float *__restrict__ x, const float *__restrict__ alpha,
                                                        float eps, int cols, float *__restrict__ xn_out,
                                                        uint32_t *__restrict__ qs, Q8Scale *__restrict__ scales,
                                                        half4v *__restrict__ xh) {
    __shared__ float red[16];
    const float4 *xr = (const float4 *)(x + (size_t)blockIdx.x * cols);
    const int n4 = cols >> 2;
    float s = 0.0f;
    for (int c = threadIdx.x; c < n4; c += 256) {
        const float4 v = xr[c];
        s += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
    s = block_reduce<false>(s, red);
    const float mean = s / (float)cols;
    const float scale = rms_inv_sqrt(mean + eps);
    const int n4_pad = (n4 + 255) & ~255;  // whole wavefronts take part in the cross-lane steps
    for (int c = threadIdx.x; c < n4_pad; c += 256) {
        const bool live = c < n4;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live) {
            v = xr[c];
            if (alpha) {
                const float4 a = ((const float4 *)alpha)[c];
                v = make_float4(scale * v.x * a.x, scale * v.y * a.y, scale * v.z * a.z, scale * v.w * a.w);
            } else {
                v = make_float4(scale * v.x, scale * v.y, scale * v.z, scale * v.w);
            }
        }
        __half h;
        int bsum;
        const uint32_t packed = quantize_q8_lane4(v, h, bsum);
        if (!live) continue;
        const size_t i = (size_t)blockIdx.x * n4 + c;
        if (xn_out) ((float4 *)xn_out)[i] = v;
        qs[i] = packed;
        if (xh) xh[xh_index4(blockIdx.x, c, cols)] = q8_lane4_to_half(packed, h);
        if ((c & 7) == 0) {
            Q8Scale sc;
            sc.d = __half2float(h);
            sc.bsum = bsum;
            scales[i >> 3] = sc;
        }
    }
}

// The same for rows of up to 1024 * ITER values: row and norm weight requested together and held in registers, one
// memory round trip where the kernel above makes two (the decode step's final norm, one row of 4096: 6.9 -> about 4 us).
// Same additions in the same order, same bits.
template <int ITER>
__global__ __launch_bounds__(256) void k_rms_norm_quant_row(const float *__restrict__ x, const float *__restrict__ alpha,
                                                            float eps, int cols, float *__restrict__ xn_out,
                                                            uint32_t *__restrict__ qs, Q8Scale *__restrict__ scales,
                                                            half4v *__restrict__ xh) {
    __shared__ float red[16];
    const float4 *xr = (const float4 *)(x + (size_t)blockIdx.x * cols);
    const int n4 = cols >> 2;
    float4 v[ITER], al[ITER];
#pragma unroll
    for (int i = 0; i < ITER; ++i) {
        const int c = min((int)threadIdx.x + 256 * i, n4 - 1);
        v[i] = xr[c];
        if (alpha) al[i] = ((const float4 *)alpha)[c];
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < ITER; ++i)
        if ((int)threadIdx.x + 256 * i < n4) s += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
    s = block_reduce<false>(s, red);
    const float mean = s / (float)cols;
    const float scale = rms_inv_sqrt(mean + eps);
#pragma unroll
    for (int i = 0; i < ITER; ++i) {
        const int c = (int)threadIdx.x + 256 * i;
        if (c >= ((n4 + 255) & ~255)) break;  // whole wavefronts take part in the cross-lane steps
        const bool live = c < n4;
        float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live) {
            if (alpha) o = make_float4(scale * v[i].x * al[i].x, scale * v[i].y * al[i].y, scale * v[i].z * al[i].z, scale * v[i].w * al[i].w);
            else o = make_float4(scale * v[i].x, scale * v[i].y, scale * v[i].z, scale * v[i].w);
        }
        __half h;
        int bsum;
        const uint32_t packed = quantize_q8_lane4(o, h, bsum);
        if (!live) continue;
        const size_t at = (size_t)blockIdx.x * n4 + c;
        if (xn_out) ((float4 *)xn_out)[at] = o;
        qs[at] = packed;
        if (xh) xh[xh_index4(blockIdx.x, c, cols)] = q8_lane4_to_half(packed, h);
        if ((c & 7) == 0) {
            Q8Scale sc;
            sc.d = __half2float(h);
            sc.bsum = bsum;
            scales[at >> 3] = sc;
        }
    }
}

// The same for rows of up to 1024 * ITER values, the row held in registers between the two passes, and with the row
// optionally assembled first from the partial copies a contraction split along K has left: x = res + (part[0] +
// part[1] + ...), the additions in the order of the separate split sum, written back to x_out (res may alias x_out:
// a thread reads what it overwrites).  With n_split == 0 the row is read from res.
// NS: the number of partial copies when it is 2 or 4 (what the prompt pass's o and down projections leave) - every
// load of the thread, norm weight included, is then requested before the first is used; 0: any number, read one after
// the other.
template <int ITER, int NS = 0>
__global__ __launch_bounds__(256) void k_rms_norm_quant_regs(const float *res, const float *__restrict__ part, int n_split,
                                                             size_t stride, float *x_out,
                                                             const float *__restrict__ alpha, float eps, int cols,
                                                             uint32_t *__restrict__ qs, Q8Scale *__restrict__ scales,
                                                             half4v *__restrict__ xh) {
    __shared__ float red[16];
    const int n4 = cols >> 2;
    const size_t row4 = (size_t)blockIdx.x * n4;
    float4 v[ITER], al[ITER];
    if constexpr (NS > 0) {
        // rows of n4 = 256 * ITER float4 or fewer: chunks past the row re-read its last one and are dropped below
        float4 pv[ITER][NS], rv[ITER];
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            const int c = min((int)threadIdx.x + 256 * it, n4 - 1);
#pragma unroll
            for (int k = 0; k < NS; ++k) pv[it][k] = ((const float4 *)(part + (size_t)k * stride))[row4 + c];
            if (res) rv[it] = ((const float4 *)res)[row4 + c];
            if (alpha) al[it] = ((const float4 *)alpha)[c];
        }
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            const int c = threadIdx.x + 256 * it;
            float4 t = pv[it][0];
#pragma unroll
            for (int k = 1; k < NS; ++k) { t.x += pv[it][k].x; t.y += pv[it][k].y; t.z += pv[it][k].z; t.w += pv[it][k].w; }
            if (res) t = make_float4(rv[it].x + t.x, rv[it].y + t.y, rv[it].z + t.z, rv[it].w + t.w);
            v[it] = c < n4 ? t : make_float4(0.f, 0.f, 0.f, 0.f);
            if (c < n4) ((float4 *)x_out)[row4 + c] = t;
        }
    } else
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        const int c = threadIdx.x + 256 * it;
        v[it] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c < n4) {
            if (n_split > 0) {
                float4 t = ((const float4 *)part)[row4 + c];
                for (int k = 1; k < n_split; ++k) {
                    const float4 u = ((const float4 *)(part + (size_t)k * stride))[row4 + c];
                    t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w;
                }
                if (res) {
                    const float4 r = ((const float4 *)res)[row4 + c];
                    t = make_float4(r.x + t.x, r.y + t.y, r.z + t.z, r.w + t.w);
                }
                v[it] = t;
                ((float4 *)x_out)[row4 + c] = t;
            } else {
                v[it] = ((const float4 *)res)[row4 + c];
            }
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int it = 0; it < ITER; ++it) s += v[it].x * v[it].x + v[it].y * v[it].y + v[it].z * v[it].z + v[it].w * v[it].w;
    s = block_reduce<false>(s, red);
    const float mean = s / (float)cols;
    const float scale = rms_inv_sqrt(mean + eps);
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        const int c = threadIdx.x + 256 * it;
        if (256 * it >= n4) break;  // whole wavefronts take part in the cross-lane steps (n4 % 8 == 0)
        const bool live = c < n4;
        float4 w = v[it];
        if (live) {
            if (alpha) {
                const float4 a = NS > 0 ? al[it] : ((const float4 *)alpha)[c];
                w = make_float4(scale * w.x * a.x, scale * w.y * a.y, scale * w.z * a.z, scale * w.w * a.w);
            } else {
                w = make_float4(scale * w.x, scale * w.y, scale * w.z, scale * w.w);
            }
        }
        __half h;
        int bsum;
        const uint32_t packed = quantize_q8_lane4(w, h, bsum);
        if (!live) continue;
        const size_t i = row4 + c;
        qs[i] = packed;
        if (xh) xh[xh_index4(blockIdx.x, c, cols)] = q8_lane4_to_half(packed, h);
        if ((c & 7) == 0) {
            Q8Scale sc;
            sc.d = __half2float(h);
            sc.bsum = bsum;
            scales[i >> 3] = sc;
        }
    }
}

// silu(gate) * up, then Q8_0 quantization. n % 32 == 0.
__global__ __launch_bounds__(256) void k_silu_mul_quant(const float4 *__restrict__ gate, const float4 *__restrict__ up,
                                                        int64_t n4, int64_t row_n4, float4 *__restrict__ act_out,
                                                        uint32_t *__restrict__ qs, Q8Scale *__restrict__ scales,
                                                        half4v *__restrict__ xh) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool live = i < n4;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live) {
        const float4 g = gate[i], u = up[i];
        v = make_float4(silu_f(g.x) * u.x, silu_f(g.y) * u.y, silu_f(g.z) * u.z, silu_f(g.w) * u.w);
    }
    __half h;
    int bsum;
    const uint32_t packed = quantize_q8_lane4(v, h, bsum);
    if (!live) return;
    if (act_out) act_out[i] = v;
    qs[i] = packed;
    if (xh) xh[xh_index4(i / row_n4, i % row_n4, 4 * row_n4)] = q8_lane4_to_half(packed, h);
    if ((i & 7) == 0) {
        Q8Scale sc;
        sc.d = __half2float(h);
        sc.bsum = bsum;
        scales[i >> 3] = sc;
    }
}

// ------------------------------------------------------------------ launchers shared with llama.hip
int launch_argmax_key(candy_hip_device *dev, const float *logits, int64_t cols, unsigned long long *key) {
    CANDY_REQUIRE(cols > 0 && cols <= 0x7FFFFFFF && ((uintptr_t)logits & 15) == 0, "argmax over a row of another shape");
    const int64_t n4 = cols >> 2;
    hipLaunchKernelGGL(k_argmax_key, dim3((unsigned)std::max<int64_t>(1, (n4 + 511) / 512)), dim3(256), 0, dev->stream, logits,
                       (int)cols, key);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int launch_rms_norm_quant(candy_hip_device *dev, const float *x, const float *alpha, float eps, int64_t rows,
                          int64_t cols, float *xn_out, int8_t *qs, Q8Scale *scales, _Float16 *xh) {
    CANDY_REQUIRE(cols % 32 == 0 && cols > 0 && rows > 0 && cols <= 0x7FFFFFFF, "rms_norm_quant needs cols %% 32 == 0");
    auto kern = cols <= 4096 ? k_rms_norm_quant_row<4> : cols <= 8192 ? k_rms_norm_quant_row<8> : k_rms_norm_quant;
    hipLaunchKernelGGL(kern, dim3((unsigned)rows), dim3(256), 0, dev->stream, x, alpha, eps, (int)cols, xn_out, (uint32_t *)qs,
                       scales, (half4v *)xh);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

// RMSNorm + quantization of rows that a split contraction has left as partial copies (SplitPending, filled by the
// fp16 tile launcher while dev->defer_split points at it): the sum, the residual add and the norm in one launch for
// rows of up to 8192 values, the separate split sum first for longer ones.
int launch_split_rms_norm_quant(candy_hip_device *dev, const SplitPending &sp, const float *alpha, float eps, int64_t rows,
                                int64_t cols, int8_t *qs, Q8Scale *scales, _Float16 *xh) {
    CANDY_REQUIRE(cols % 32 == 0 && cols > 0 && rows > 0 && cols <= 0x7FFFFFFF, "rms_norm_quant needs cols %% 32 == 0");
    CANDY_REQUIRE(sp.count == (size_t)rows * (size_t)cols && sp.n_split > 0, "internal: pending split sum of another shape");
    if (cols > 8192 || !dev->opt.prefill_fold_split_sums) {
        if (int rc = launch_splitk_sum(dev, sp.part, sp.y, sp.res, sp.count, sp.n_split, sp.stride)) return rc;
        return launch_rms_norm_quant(dev, sp.y, alpha, eps, rows, cols, nullptr, qs, scales, xh);
    }
    auto kern = cols <= 4096 ? (sp.n_split == 2 ? k_rms_norm_quant_regs<4, 2> : sp.n_split == 4 ? k_rms_norm_quant_regs<4, 4>
                                                                                                 : k_rms_norm_quant_regs<4>)
                             : k_rms_norm_quant_regs<8>;
    hipLaunchKernelGGL(kern, dim3((unsigned)rows), dim3(256), 0, dev->stream, sp.res, sp.part, sp.n_split, sp.stride, sp.y,
                       alpha, eps, (int)cols, (uint32_t *)qs, scales, (half4v *)xh);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int launch_silu_mul_quant(candy_hip_device *dev, const float *gate, const float *up, int64_t rows, int64_t cols,
                          float *act_out, int8_t *qs, Q8Scale *scales, _Float16 *xh) {
    CANDY_REQUIRE(cols % 32 == 0 && cols > 0 && rows > 0, "silu_mul_quant needs cols %% 32 == 0");
    const int64_t n4 = rows * cols >> 2;
    hipLaunchKernelGGL(k_silu_mul_quant, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, dev->stream,
                       (const float4 *)gate, (const float4 *)up, n4, cols >> 2, (float4 *)act_out, (uint32_t *)qs, scales,
                       (half4v *)xh);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

}  // namespace candy

using namespace candy;

static inline unsigned blocks_for(int64_t n) { return (unsigned)((n + 255) / 256); }

template <int OP>
static int elementwise(candy_hip_device *dev, const float *a, const float *b, int64_t n, float *out) {
    CANDY_REQUIRE(n >= 0, "invalid length");
    if (n == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(a && out && (OP == EW_SILU || b), "nil pointer");
    if (int rc = use_device(dev)) return rc;
    hipLaunchKernelGGL((k_elementwise<OP>), dim3(blocks_for(n)), dim3(256), 0, dev->stream, a, b, n, out);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}


extern "C" {

int candy_hip_matmul_f32(candy_hip_device *dev, const float *a, const float *b, float *c, int64_t batch, int64_t m,
                         int64_t n, int64_t k, int rhs_transposed) {
    CANDY_REQUIRE(m > 0 && n > 0 && k > 0 && batch > 0, "invalid matrix dimensions");  // cpu/storage.go:877-879
    CANDY_REQUIRE(a && b && c, "layouts cannot be nil");
    CANDY_REQUIRE(m <= 65535 && batch <= 65535, "matrix too large");
    if (int rc = use_device(dev)) return rc;
    hipLaunchKernelGGL(k_matmul_f32, dim3(blocks_for(n), (unsigned)m, (unsigned)batch), dim3(256), 0, dev->stream, a, b,
                       c, m, n, k, rhs_transposed);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int candy_hip_matmul_f32_strided(candy_hip_device *dev, const float *a, const float *b, float *c, int64_t m, int64_t n,
                                 int64_t k, int64_t a_row_stride, int64_t a_col_stride, int64_t b_row_stride,
                                 int64_t b_col_stride) {
    CANDY_REQUIRE(m > 0 && n > 0 && k > 0, "invalid matrix dimensions");  // cpu/storage.go:877-879
    CANDY_REQUIRE(a && b && c, "layouts cannot be nil");
    CANDY_REQUIRE(m <= 65535, "matrix too large");
    CANDY_REQUIRE(a_row_stride >= 0 && a_col_stride >= 0 && b_row_stride >= 0 && b_col_stride >= 0,
                  "negative strides are not supported");
    if (int rc = use_device(dev)) return rc;
    hipLaunchKernelGGL(k_matmul_f32_strided, dim3(blocks_for(n), (unsigned)m), dim3(256), 0, dev->stream, a, b, c, n, k,
                       a_row_stride, a_col_stride, b_row_stride, b_col_stride);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int candy_hip_rms_norm(candy_hip_device *dev, const float *x, const float *alpha, float eps, int64_t rows, int64_t cols,
                       float *out) {
    CANDY_REQUIRE(rows >= 0 && cols >= 0 && cols <= 0x7FFFFFFF && rows <= 0x7FFFFFFF, "invalid dimensions");
    if (rows * cols == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(x && out, "nil pointer");
    if (int rc = use_device(dev)) return rc;
    hipLaunchKernelGGL(k_rms_norm, dim3((unsigned)rows), dim3(256), 0, dev->stream, x, alpha, eps, (int)cols, out);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int candy_hip_rope(candy_hip_device *dev, const float *src, const float *cos_t, const float *sin_t, int64_t bh,
                   int64_t td, int64_t d, int64_t stride_b, float *dst) {
    CANDY_REQUIRE(bh >= 0 && td >= 0 && d >= 0 && stride_b >= 0, "invalid dimensions");
    const int64_t pairs = bh * td / 2;
    if (pairs == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(d >= 2 && d % 2 == 0 && td % d == 0, "rope needs an even head dim that divides t*d");
    CANDY_REQUIRE(src && cos_t && sin_t && dst, "nil pointer");
    if (int rc = use_device(dev)) return rc;
    hipLaunchKernelGGL(k_rope, dim3(blocks_for(pairs)), dim3(256), 0, dev->stream, src, cos_t, sin_t, pairs, td, d,
                       stride_b, dst);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int candy_hip_rope_i(candy_hip_device *dev, const float *src, const float *cos_t, const float *sin_t, int64_t bh,
                     int64_t td, int64_t stride_b, float *dst) {
    CANDY_REQUIRE(bh >= 0 && td >= 0 && stride_b >= 0, "invalid dimensions");
    const int64_t pairs = bh * td / 2;
    if (pairs == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(td % 2 == 0, "rope_i needs an even t*d");
    CANDY_REQUIRE(src && cos_t && sin_t && dst, "nil pointer");
    CANDY_REQUIRE((((uintptr_t)src | (uintptr_t)dst) & 7) == 0, "rope_i operands must be 8-byte aligned");
    if (int rc = use_device(dev)) return rc;
    hipLaunchKernelGGL(k_rope_i, dim3(blocks_for(pairs)), dim3(256), 0, dev->stream, (const float2 *)src, cos_t, sin_t,
                       pairs, td / 2, stride_b, (float2 *)dst);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int candy_hip_rope_thd(candy_hip_device *dev, const float *src, const float *cos_t, const float *sin_t, int64_t b,
                       int64_t t, int64_t h, int64_t d, int64_t stride_b, float *dst) {
    CANDY_REQUIRE(b >= 0 && t >= 0 && h >= 0 && d >= 0 && stride_b >= 0, "invalid dimensions");
    const int64_t pairs = b * t * h * d / 2;
    if (pairs == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(d >= 2 && d % 2 == 0, "rope_thd needs an even head dim");
    CANDY_REQUIRE(src && cos_t && sin_t && dst, "nil pointer");
    if (int rc = use_device(dev)) return rc;
    hipLaunchKernelGGL(k_rope_thd, dim3(blocks_for(pairs)), dim3(256), 0, dev->stream, src, cos_t, sin_t, pairs, t, h, d,
                       stride_b, dst);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int candy_hip_softmax(candy_hip_device *dev, const float *src, int64_t rows, int64_t cols, float *dst) {
    CANDY_REQUIRE(rows >= 0 && cols >= 0 && cols <= 0x7FFFFFFF && rows <= 0x7FFFFFFF, "invalid dimensions");
    if (rows * cols == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(src && dst, "nil pointer");
    if (int rc = use_device(dev)) return rc;
    hipLaunchKernelGGL(k_softmax, dim3((unsigned)rows), dim3(256), 0, dev->stream, src, (int)cols, dst);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int candy_hip_silu(candy_hip_device *dev, const float *x, int64_t n, float *out) {
    return elementwise<EW_SILU>(dev, x, nullptr, n, out);
}
int candy_hip_add(candy_hip_device *dev, const float *a, const float *b, int64_t n, float *out) {
    return elementwise<EW_ADD>(dev, a, b, n, out);
}
int candy_hip_mul(candy_hip_device *dev, const float *a, const float *b, int64_t n, float *out) {
    return elementwise<EW_MUL>(dev, a, b, n, out);
}
int candy_hip_silu_mul(candy_hip_device *dev, const float *gate, const float *up, int64_t n, float *out) {
    return elementwise<EW_SILU_MUL>(dev, gate, up, n, out);
}

int candy_hip_argmax(candy_hip_device *dev, const float *src, int64_t rows, int64_t cols, uint32_t *out) {
    CANDY_REQUIRE(rows >= 0 && cols >= 0 && cols <= 0x7FFFFFFF && rows <= 0x7FFFFFFF, "invalid dimensions");
    if (rows * cols == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(src && out, "nil pointer");
    if (int rc = use_device(dev)) return rc;
    hipLaunchKernelGGL(k_argmax, dim3((unsigned)rows), dim3(1024), 0, dev->stream, src, (int)cols, out);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int candy_hip_index_select(candy_hip_device *dev, const float *table, int64_t n_src, int64_t width,
                           const int64_t *dev_ids, int64_t n_ids, float *out) {
    CANDY_REQUIRE(n_src >= 0 && width >= 0 && n_ids >= 0 && n_ids <= 0x7FFFFFFF, "invalid dimensions");
    if (n_ids * width == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(table && dev_ids && out, "nil pointer");
    if (int rc = use_device(dev)) return rc;
    hipLaunchKernelGGL(k_index_select, dim3((unsigned)n_ids), dim3(256), 0, dev->stream, table, n_src, width, dev_ids, out,
                       dev->fault);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

}  // extern "C"
