// Prompt (prefill) stages of the Llama-style decoder: n tokens at once.
//
// candy has no attention on the CPU; a candy model composes it from MatMul / FastSoftmax / MatMul
// (backend.go:78,147) per token. For a prompt of n tokens at positions pos0 .. pos0+n-1 that is,
// per head, softmax over the cached positions 0 .. pos0+i of q_i . K^T * scale, times V:
// the same arithmetic as n successive decode steps, evaluated tile by tile here.
//   k_prefill_rope_kv   Rope (reduce.go:3987-4006: pairs (j, j + d/2)) on q in place and on k, and the
//                       new k / v rows written into the f32 cache [kv_head][position][head_dim]
//   k_attn_prefill      causal attention of 32 queries of one head against the cache, f32 on the
//                       vector ALU with K / V / probabilities tiled through LDS, online softmax
#include "blocks.h"
#include "internal.h"

namespace candy {

__global__ __launch_bounds__(256) void k_prefill_rope_kv(float *__restrict__ q, const float *__restrict__ k,
                                                         const float *__restrict__ v,
                                                         const float *__restrict__ cos_t,
                                                         const float *__restrict__ sin_t, float *__restrict__ k_cache,
                                                         float *__restrict__ v_cache, int n, int pos0, int n_heads,
                                                         int n_kv_heads, int head_dim, int64_t cache_stride) {
    const int half = head_dim >> 1;
    const int slots = n_heads + 2 * n_kv_heads;  // q heads, then k heads, then v heads
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t total = (int64_t)n * slots * half;
    if (idx >= total) return;
    const int j = (int)(idx % half);
    const int slot = (int)((idx / half) % slots);
    const int i = (int)(idx / ((int64_t)half * slots));
    const int pos = pos0 + i;
    const float c = cos_t[(size_t)pos * half + j], s = sin_t[(size_t)pos * half + j];
    if (slot < n_heads) {
        float *p = q + ((size_t)i * n_heads + slot) * head_dim + j;
        const float a = p[0], b = p[half];
        p[0] = a * c - b * s;
        p[half] = a * s + b * c;
    } else if (slot < n_heads + n_kv_heads) {
        const int h = slot - n_heads;
        const float *p = k + ((size_t)i * n_kv_heads + h) * head_dim + j;
        float *dst = k_cache + (size_t)h * cache_stride + (size_t)pos * head_dim + j;
        const float a = p[0], b = p[half];
        dst[0] = a * c - b * s;
        dst[half] = a * s + b * c;
    } else {
        const int h = slot - n_heads - n_kv_heads;
        const float *p = v + ((size_t)i * n_kv_heads + h) * head_dim + j;
        float *dst = v_cache + (size_t)h * cache_stride + (size_t)pos * head_dim + j;
        dst[0] = p[0];
        dst[half] = p[half];
    }
}

// grid (n_heads, ceil(n / 32)), 256 threads. Thread t serves query row t/8 throughout: in the score
// phase it owns keys {t%8 + 8r}, in the output phase columns {4*(t%8) + 32r .. +3}; the 8 threads of
// a row sit in adjacent lanes, so the row maximum and sum are three xor-shuffles.
template <int HD>
__global__ __launch_bounds__(256) void k_attn_prefill(const float *__restrict__ q, const float *__restrict__ k_cache,
                                                      const float *__restrict__ v_cache, float *__restrict__ out,
                                                      int n, int pos0, int n_heads, int n_kv_heads,
                                                      int64_t cache_stride, float scale) {
    constexpr int QT = 32, KT = 32, PITCH = HD + 4;  // pitch = 4 mod 64 banks: the 8 rows of a read never collide
    __shared__ __align__(16) float s_q[QT * PITCH];
    __shared__ __align__(16) float s_k[KT * PITCH];
    __shared__ __align__(16) float s_v[KT * HD];
    __shared__ __align__(16) float s_p[QT * KT];
    const int tid = threadIdx.x, qi = tid >> 3, sub = tid & 7;
    const int head = blockIdx.x, i0 = blockIdx.y * QT;
    const int kvh = head / (n_heads / n_kv_heads);
    const float *kh = k_cache + (size_t)kvh * cache_stride, *vh = v_cache + (size_t)kvh * cache_stride;
    const int rows = min(QT, n - i0);
    const int n_keys = pos0 + i0 + rows;    // the tile's last query sees this many positions
    const int my_last = pos0 + i0 + qi;     // last position query row qi may attend
    constexpr int F4 = HD / 4;

    for (int e = tid; e < QT * F4; e += 256) {
        const int r = e / F4, c4 = e % F4;
        const int i = min(i0 + r, n - 1);
        *(float4 *)&s_q[r * PITCH + 4 * c4] = *(const float4 *)(q + ((size_t)i * n_heads + head) * HD + 4 * c4);
    }
    float m_run = -INFINITY, l_run = 0.0f;
    float4 o[HD / 32];
#pragma unroll
    for (int r = 0; r < HD / 32; ++r) o[r] = make_float4(0.f, 0.f, 0.f, 0.f);

    for (int p0 = 0; p0 < n_keys; p0 += KT) {
        __syncthreads();  // previous tile fully consumed (and s_q written, first time round)
        for (int e = tid; e < KT * F4; e += 256) {
            const int r = e / F4, c4 = e % F4;
            const size_t p = (size_t)min(p0 + r, n_keys - 1);
            *(float4 *)&s_k[r * PITCH + 4 * c4] = *(const float4 *)(kh + p * HD + 4 * c4);
            *(float4 *)&s_v[r * HD + 4 * c4] = *(const float4 *)(vh + p * HD + 4 * c4);
        }
        __syncthreads();
        // scores of (row qi, keys sub + 8r)
        float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
        for (int d = 0; d < HD; d += 4) {
            const float4 qv = *(const float4 *)&s_q[qi * PITCH + d];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float4 kv = *(const float4 *)&s_k[(sub + 8 * r) * PITCH + d];
                s[r] += qv.x * kv.x + qv.y * kv.y + qv.z * kv.z + qv.w * kv.w;
            }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const bool ok = p0 + sub + 8 * r <= my_last;
            s[r] = ok ? s[r] * scale : -INFINITY;
            mx = fmaxf(mx, s[r]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 1));
        mx = fmaxf(mx, __shfl_xor(mx, 2));
        mx = fmaxf(mx, __shfl_xor(mx, 4));
        const float m_new = fmaxf(m_run, mx);  // position 0 is visible to every row, so m_new is finite
        const float corr = expf(m_run - m_new);
        float ps = 0.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float pw = expf(s[r] - m_new);  // exp(-inf) = 0 for masked keys
            s_p[qi * KT + sub + 8 * r] = pw;
            ps += pw;
        }
        ps += __shfl_xor(ps, 1);
        ps += __shfl_xor(ps, 2);
        ps += __shfl_xor(ps, 4);
        l_run = l_run * corr + ps;
        m_run = m_new;
#pragma unroll
        for (int r = 0; r < HD / 32; ++r) {
            o[r].x *= corr; o[r].y *= corr; o[r].z *= corr; o[r].w *= corr;
        }
        __syncthreads();  // probabilities of the whole tile are in LDS
#pragma unroll 4
        for (int kk = 0; kk < KT; ++kk) {
            const float pw = s_p[qi * KT + kk];
#pragma unroll
            for (int r = 0; r < HD / 32; ++r) {
                const float4 vv = *(const float4 *)&s_v[kk * HD + 4 * sub + 32 * r];
                o[r].x += pw * vv.x; o[r].y += pw * vv.y; o[r].z += pw * vv.z; o[r].w += pw * vv.w;
            }
        }
    }
    if (qi < rows) {
        const float inv = 1.0f / l_run;
        float *dst = out + ((size_t)(i0 + qi) * n_heads + head) * HD;
#pragma unroll
        for (int r = 0; r < HD / 32; ++r)
            *(float4 *)(dst + 4 * sub + 32 * r) = make_float4(o[r].x * inv, o[r].y * inv, o[r].z * inv, o[r].w * inv);
    }
}

int launch_prefill_rope_kv(candy_hip_device *dev, float *q, const float *k, const float *v, const float *cos_t,
                           const float *sin_t, float *k_cache, float *v_cache, int n, int pos0, int n_heads,
                           int n_kv_heads, int head_dim, int64_t cache_stride) {
    const int64_t total = (int64_t)n * (n_heads + 2 * n_kv_heads) * (head_dim / 2);
    hipLaunchKernelGGL(k_prefill_rope_kv, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, dev->stream, q, k, v,
                       cos_t, sin_t, k_cache, v_cache, n, pos0, n_heads, n_kv_heads, head_dim, cache_stride);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int launch_attn_prefill(candy_hip_device *dev, const float *q, const float *k_cache, const float *v_cache, float *out,
                        int n, int pos0, int n_heads, int n_kv_heads, int head_dim, int64_t cache_stride, float scale) {
    CANDY_REQUIRE(head_dim == 64 || head_dim == 128, "head_dim must be 64 or 128");
    CANDY_REQUIRE(n > 0 && pos0 >= 0 && n_heads % n_kv_heads == 0, "invalid attention shape");
    const dim3 grid((unsigned)n_heads, (unsigned)((n + 31) / 32));
    if (head_dim == 128)
        hipLaunchKernelGGL(k_attn_prefill<128>, grid, dim3(256), 0, dev->stream, q, k_cache, v_cache, out, n, pos0,
                           n_heads, n_kv_heads, cache_stride, scale);
    else
        hipLaunchKernelGGL(k_attn_prefill<64>, grid, dim3(256), 0, dev->stream, q, k_cache, v_cache, out, n, pos0,
                           n_heads, n_kv_heads, cache_stride, scale);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

}  // namespace candy
