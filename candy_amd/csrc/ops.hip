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
    const float scale = 1.0f / (float)sqrt((double)(mean + eps));
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
    for (int c = threadIdx.x; c < cols; c += blockDim.x) {
        const float v = xr[c];
        if (v > best) { best = v; bi = (uint32_t)c; }
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

// indexing.go:8-26 along dim 0 of a [n_src, width] table; id == MaxInt64 selects zeros.
__global__ __launch_bounds__(256) void k_index_select(const float *__restrict__ table, int64_t width,
                                                      const int64_t *__restrict__ ids, float *__restrict__ out) {
    const int64_t id = ids[blockIdx.x];
    float *orow = out + (size_t)blockIdx.x * width;
    for (int64_t c = threadIdx.x; c < width; c += blockDim.x)
        orow[c] = id == 0x7FFFFFFFFFFFFFFFll ? 0.0f : table[id * width + c];
}

// conv.go:251-267 / :373-389: c[b,i,j] = sum_l a[b,i,l] * B[b,l,j]; one output per thread,
// l ascending, single f32 accumulator (the CPU loop's order).
__global__ __launch_bounds__(256) void k_matmul_f32(const float *__restrict__ a, const float *__restrict__ b,
                                                    float *__restrict__ c, int64_t m, int64_t n, int64_t k,
                                                    int rhs_transposed) {
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

// ------------------------------------------------------------------ attention over the f32 KV cache
// Split over positions (grid = kv heads x splits): each workgroup streams its slice of K and V
// once for all query heads that share the kv head, keeps a running (max, sum, weighted V) per
// query head, and a second kernel merges the splits.  head_dim is 128 here: a wavefront holds
// one cache row as 64 lanes x float2.

template <int GROUP>
__global__ __launch_bounds__(256) void k_attn_partial(const float *__restrict__ q, const float *__restrict__ kc,
                                                      const float *__restrict__ vc, int head_dim, int n_pos,
                                                      int64_t cache_stride, float scale, int n_splits,
                                                      float *__restrict__ part_o, float *__restrict__ part_ml) {
    // part_o: [n_heads][n_splits][head_dim]; part_ml: [n_heads][n_splits][2] (max, sum)
    const int kvh = blockIdx.x, split = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int per = (n_pos + n_splits - 1) / n_splits;
    const int p0 = split * per, p1 = min(n_pos, p0 + per);
    const float *kh = kc + (size_t)kvh * cache_stride;
    const float *vh = vc + (size_t)kvh * cache_stride;
    const int hd2 = head_dim >> 1;  // float2 per row
    const int loops = (hd2 + 63) >> 6;  // 1 for head_dim 128

    // each wave: positions p0+wave, p0+wave+4, ...
    float m_run[GROUP], l_run[GROUP];
    float2 o_run[GROUP][2];
    float2 qv[GROUP][2];
#pragma unroll
    for (int g = 0; g < GROUP; ++g) {
        m_run[g] = -3.402823466e+38f;
        l_run[g] = 0.0f;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            o_run[g][t] = make_float2(0.f, 0.f);
            const int c = lane + 64 * t;
            qv[g][t] = (t < loops && c < hd2) ? ((const float2 *)(q + (size_t)(kvh * GROUP + g) * head_dim))[c]
                                              : make_float2(0.f, 0.f);
        }
    }
    for (int p = p0 + wave; p < p1; p += 4) {
        float2 kv[2], vv[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int c = lane + 64 * t;
            const bool ok = t < loops && c < hd2;
            kv[t] = ok ? ((const float2 *)(kh + (size_t)p * head_dim))[c] : make_float2(0.f, 0.f);
            vv[t] = ok ? ((const float2 *)(vh + (size_t)p * head_dim))[c] : make_float2(0.f, 0.f);
        }
#pragma unroll
        for (int g = 0; g < GROUP; ++g) {
            float s = qv[g][0].x * kv[0].x + qv[g][0].y * kv[0].y + qv[g][1].x * kv[1].x + qv[g][1].y * kv[1].y;
            s = wave_sum(s) * scale;
            const float m_new = fmaxf(m_run[g], s);
            const float corr = expf(m_run[g] - m_new), pw = expf(s - m_new);
            l_run[g] = l_run[g] * corr + pw;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                o_run[g][t].x = o_run[g][t].x * corr + pw * vv[t].x;
                o_run[g][t].y = o_run[g][t].y * corr + pw * vv[t].y;
            }
            m_run[g] = m_new;
        }
    }
    // merge the 4 waves through LDS
    __shared__ float sm[4][GROUP], sl[4][GROUP];
    __shared__ float2 so[4][GROUP][128];
#pragma unroll
    for (int g = 0; g < GROUP; ++g) {
        if (lane == 0) { sm[wave][g] = m_run[g]; sl[wave][g] = l_run[g]; }
#pragma unroll
        for (int t = 0; t < 2; ++t) so[wave][g][lane + 64 * t] = o_run[g][t];
    }
    __syncthreads();
    // thread -> (g, column c of float2)
    for (int idx = threadIdx.x; idx < GROUP * hd2; idx += 256) {
        const int g = idx / hd2, c = idx - g * hd2;
        float m = sm[0][g];
        for (int w = 1; w < 4; ++w) m = fmaxf(m, sm[w][g]);
        float l = 0.0f;
        float2 o = make_float2(0.f, 0.f);
        for (int w = 0; w < 4; ++w) {
            const float f = expf(sm[w][g] - m);
            l += sl[w][g] * f;
            o.x += so[w][g][c].x * f;
            o.y += so[w][g][c].y * f;
        }
        const int h = kvh * GROUP + g;
        ((float2 *)(part_o + ((size_t)h * n_splits + split) * head_dim))[c] = o;
        if (c == 0) {
            part_ml[((size_t)h * n_splits + split) * 2 + 0] = m;
            part_ml[((size_t)h * n_splits + split) * 2 + 1] = l;
        }
    }
}

__global__ __launch_bounds__(128) void k_attn_merge(const float *__restrict__ part_o, const float *__restrict__ part_ml,
                                                    int head_dim, int n_splits, float *__restrict__ out) {
    const int h = blockIdx.x;
    float m = -3.402823466e+38f;
    for (int s = 0; s < n_splits; ++s) m = fmaxf(m, part_ml[((size_t)h * n_splits + s) * 2]);
    float l = 0.0f;
    for (int s = 0; s < n_splits; ++s) {
        const float ls = part_ml[((size_t)h * n_splits + s) * 2 + 1];
        l += ls * expf(part_ml[((size_t)h * n_splits + s) * 2] - m);
    }
    const float inv = 1.0f / l;
    for (int c = threadIdx.x; c < head_dim; c += blockDim.x) {
        float o = 0.0f;
        for (int s = 0; s < n_splits; ++s) {
            const float f = expf(part_ml[((size_t)h * n_splits + s) * 2] - m);
            o += part_o[((size_t)h * n_splits + s) * head_dim + c] * f;
        }
        out[(size_t)h * head_dim + c] = o * inv;
    }
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
    hipLaunchKernelGGL(k_index_select, dim3((unsigned)n_ids), dim3(256), 0, dev->stream, table, width, dev_ids, out);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int candy_hip_attention_decode(candy_hip_device *dev, const float *q, const float *k_cache, const float *v_cache,
                               int64_t n_heads, int64_t n_kv_heads, int64_t head_dim, int64_t n_pos,
                               int64_t cache_stride, float scale, float *out) {
    CANDY_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0, "invalid head counts %lld / %lld",
                  (long long)n_heads, (long long)n_kv_heads);
    CANDY_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && head_dim <= 256, "head_dim %lld unsupported (even, <= 256)",
                  (long long)head_dim);
    CANDY_REQUIRE(n_pos > 0 && cache_stride >= n_pos * head_dim, "invalid cache shape");
    CANDY_REQUIRE(q && k_cache && v_cache && out, "nil pointer");
    const int group = (int)(n_heads / n_kv_heads);
    CANDY_REQUIRE(group == 1 || group == 2 || group == 4 || group == 8, "query heads per kv head must be 1, 2, 4 or 8");
    if (int rc = use_device(dev)) return rc;
    // enough workgroups to fill the chip, at least 64 positions per split
    int n_splits = (int)((2 * (int64_t)dev->num_cus + n_kv_heads - 1) / n_kv_heads);
    const int max_splits = (int)((n_pos + 63) / 64);
    if (n_splits > max_splits) n_splits = max_splits;
    if (n_splits < 1) n_splits = 1;
    const size_t po_bytes = (size_t)n_heads * n_splits * head_dim * sizeof(float);
    const size_t ml_bytes = (size_t)n_heads * n_splits * 2 * sizeof(float);
    void *ws = nullptr;
    if (int rc = workspace(dev, po_bytes + ml_bytes, &ws)) return rc;
    float *part_o = (float *)ws, *part_ml = (float *)((uint8_t *)ws + po_bytes);
    dim3 grid((unsigned)n_kv_heads, (unsigned)n_splits);
#define CANDY_ATTN(G)                                                                                          \
    hipLaunchKernelGGL((k_attn_partial<G>), grid, dim3(256), 0, dev->stream, q, k_cache, v_cache, (int)head_dim, \
                       (int)n_pos, cache_stride, scale, n_splits, part_o, part_ml)
    switch (group) {
    case 1: CANDY_ATTN(1); break;
    case 2: CANDY_ATTN(2); break;
    case 4: CANDY_ATTN(4); break;
    default: CANDY_ATTN(8); break;
    }
#undef CANDY_ATTN
    CANDY_LAUNCH_CHECK();
    hipLaunchKernelGGL(k_attn_merge, dim3((unsigned)n_heads), dim3(128), 0, dev->stream, part_o, part_ml, (int)head_dim,
                       n_splits, out);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

}  // extern "C"
