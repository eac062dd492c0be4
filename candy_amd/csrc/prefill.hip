// Prompt (prefill) stages of the Llama-style decoder: n tokens at once.
//
// candy has no attention on the CPU; a candy model composes it from MatMul / FastSoftmax / MatMul
// (backend.go:78,147) per token. For a prompt of n tokens at positions pos0 .. pos0+n-1 that is,
// per head, softmax over the cached positions 0 .. pos0+i of q_i . K^T * scale, times V:
// the same arithmetic as n successive decode steps, evaluated tile by tile here.
//   k_prefill_rope_kv   Rope (reduce.go:3987-4006: pairs (j, j + d/2)) on q in place and on k, and the
//                       new k / v rows written into the f32 cache [kv_head][position][head_dim]
//   k_attn_prefill      causal attention of 32 queries of one head against the cache, f32 on the
//                       vector ALU with K / V / probabilities tiled through LDS, online softmax (head_dim 64)
//   k_attn_prefill_mfma the same for head_dim 128 on the matrix cores, 64 queries per workgroup
#include <cstdlib>

#include "blocks.h"
#include "internal.h"

namespace candy {

// Four consecutive cache values as f32; KV is float (candy's cache) or _Float16 (the optional half-size cache).
template <class KV>
__device__ __forceinline__ float4 kv_load4(const KV *p);
template <>
__device__ __forceinline__ float4 kv_load4<float>(const float *p) { return *(const float4 *)p; }
template <>
__device__ __forceinline__ float4 kv_load4<_Float16>(const _Float16 *p) {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    const h4 v = *(const h4 *)p;
    return make_float4((float)v[0], (float)v[1], (float)v[2], (float)v[3]);
}

template <class KV>
__global__ __launch_bounds__(256) void k_prefill_rope_kv(float *__restrict__ q, const float *__restrict__ k,
                                                         const float *__restrict__ v,
                                                         const float *__restrict__ cos_t,
                                                         const float *__restrict__ sin_t, KV *__restrict__ k_cache,
                                                         KV *__restrict__ v_cache, int n, int pos0, int n_heads,
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
        KV *dst = k_cache + (size_t)h * cache_stride + (size_t)pos * head_dim + j;
        const float a = p[0], b = p[half];
        dst[0] = (KV)(a * c - b * s);
        dst[half] = (KV)(a * s + b * c);
    } else {
        const int h = slot - n_heads - n_kv_heads;
        const float *p = v + ((size_t)i * n_kv_heads + h) * head_dim + j;
        KV *dst = v_cache + (size_t)h * cache_stride + (size_t)pos * head_dim + j;
        dst[0] = (KV)p[0];
        dst[half] = (KV)p[half];
    }
}

// The same four pairs per thread, for q, k and v rows that lie end to end in `src` ([n][q heads], [n][kv heads] twice),
// optionally still as the n_split partial copies of a contraction split along K, `stride` floats apart, summed here in
// the order of the separate split sum.  q is written to `q` (which may be `src`), k and v go to the cache only.
template <class KV>
__global__ __launch_bounds__(256) void k_prefill_rope_kv4(float *q, const float *src, int n_split, size_t stride,
                                                          const float *__restrict__ cos_t,
                                                          const float *__restrict__ sin_t, KV *__restrict__ k_cache,
                                                          KV *__restrict__ v_cache, int n, int pos0, int n_heads,
                                                          int n_kv_heads, int head_dim, int64_t cache_stride) {
    const int half = head_dim >> 1, hq = half >> 2;
    const int slots = n_heads + 2 * n_kv_heads;  // q heads, then k heads, then v heads
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t total = (int64_t)n * slots * hq;
    if (idx >= total) return;
    const int j = (int)(idx % hq) * 4;
    const int slot = (int)((idx / hq) % slots);
    const int i = (int)(idx / ((int64_t)hq * slots));
    const int pos = pos0 + i;
    auto load = [&](size_t off) {
        float4 t = *(const float4 *)(src + off);
        for (int k = 1; k < n_split; ++k) {
            const float4 u = *(const float4 *)(src + (size_t)k * stride + off);
            t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w;
        }
        return t;
    };
    auto store = [&](KV *dst, float4 t) {  // 4-element aligned: head_dim % 8 == 0
        typedef KV kv4 __attribute__((ext_vector_type(4)));
        kv4 o;
        o[0] = (KV)t.x; o[1] = (KV)t.y; o[2] = (KV)t.z; o[3] = (KV)t.w;
        *(kv4 *)dst = o;
    };
    const size_t k_base = (size_t)n * n_heads * head_dim, v_base = k_base + (size_t)n * n_kv_heads * head_dim;
    if (slot >= n_heads + n_kv_heads) {
        const int h = slot - n_heads - n_kv_heads;
        const size_t off = v_base + ((size_t)i * n_kv_heads + h) * head_dim + j;
        KV *dst = v_cache + (size_t)h * cache_stride + (size_t)pos * head_dim + j;
        store(dst, load(off));
        store(dst + half, load(off + half));
        return;
    }
    const float4 c = *(const float4 *)(cos_t + (size_t)pos * half + j), s = *(const float4 *)(sin_t + (size_t)pos * half + j);
    const bool is_q = slot < n_heads;
    const int h = is_q ? slot : slot - n_heads;
    const size_t off = is_q ? ((size_t)i * n_heads + h) * head_dim + j : k_base + ((size_t)i * n_kv_heads + h) * head_dim + j;
    const float4 a = load(off), b = load(off + half);
    const float4 lo = make_float4(a.x * c.x - b.x * s.x, a.y * c.y - b.y * s.y, a.z * c.z - b.z * s.z, a.w * c.w - b.w * s.w);
    const float4 hi = make_float4(a.x * s.x + b.x * c.x, a.y * s.y + b.y * c.y, a.z * s.z + b.z * c.z, a.w * s.w + b.w * c.w);
    if (is_q) {
        *(float4 *)(q + off) = lo;
        *(float4 *)(q + off + half) = hi;
    } else {
        KV *dst = k_cache + (size_t)h * cache_stride + (size_t)pos * head_dim + j;
        store(dst, lo);
        store(dst + half, hi);
    }
}

// grid (n_heads, ceil(n / 32)), 256 threads. Thread t serves query row t/8 throughout: in the score
// phase it owns keys {t%8 + 8r}, in the output phase columns {4*(t%8) + 32r .. +3}; the 8 threads of
// a row sit in adjacent lanes, so the row maximum and sum are three xor-shuffles.
template <int HD, class KV>
__global__ __launch_bounds__(256) void k_attn_prefill(const float *__restrict__ q, const KV *__restrict__ k_cache,
                                                      const KV *__restrict__ v_cache, float *__restrict__ out,
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
    const KV *kh = k_cache + (size_t)kvh * cache_stride, *vh = v_cache + (size_t)kvh * cache_stride;
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
            *(float4 *)&s_k[r * PITCH + 4 * c4] = kv_load4(kh + p * HD + 4 * c4);
            *(float4 *)&s_v[r * HD + 4 * c4] = kv_load4(vh + p * HD + 4 * c4);
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

// ------------------------------------------------------------------ causal attention on the matrix cores
// head_dim 128.  grid (n_heads, ceil(n / 64)), 4 wavefronts, wavefront w owns query rows 16w .. 16w+15 of
// the tile.  Keys and values are walked in tiles of 32 positions through LDS.  Scores S = Q.K^T and
// outputs O += P.V run on v_mfma_f32_16x16x32_f16 with every f32 operand split into an fp16 head and an
// fp16 tail (x = hi + lo, |lo| <= 2^-11 |x|): hi.hi + hi.lo + lo.hi carries 22 bits of each operand into
// the f32 accumulators, so the result stays at f32-like distance from the CPU composition while the
// vector ALU only does the softmax.  (The arithmetic being replaced is MatMul / FastSoftmax / MatMul,
// backend.go:78,147; online softmax as in the vector-ALU kernel above.)
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4h __attribute__((ext_vector_type(4)));
typedef _Float16 half2h __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));

struct HiLo { _Float16 hi, lo; };
__device__ __forceinline__ HiLo split_half(float x) {
    HiLo r;
    r.hi = (_Float16)x;
    r.lo = (_Float16)(x - (float)r.hi);
    return r;
}

// 16-lane row reductions on the DPP path (C-layout columns live in the 16 lanes of a row)
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));
    v = fmaxf(v, dpp_move<0x4E>(v));
    v = fmaxf(v, dpp_move<0x141>(v));
    v = fmaxf(v, dpp_move<0x140>(v));
    return v;
}
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    v += dpp_move<0x140>(v);
    return v;
}

// GROUPS = 2: two groups of four wavefronts share the workgroup's 64 queries and take alternate key tiles, each with
// tile buffers of its own, and merge their (max, sum, output) per row at the end: a short prompt has about one
// workgroup per CU and the launch lasts as long as the last query tile's walk over all the keys, which this halves.
template <class KV, int GROUPS>
__global__ __launch_bounds__(256 * GROUPS) void k_attn_prefill_mfma(const float *__restrict__ q, const KV *__restrict__ k_cache,
                                                                    const KV *__restrict__ v_cache, float *__restrict__ out,
                                                                    int n, int pos0, int n_heads, int n_kv_heads,
                                                                    int64_t cache_stride, float scale,
                                                                    _Float16 *__restrict__ xh_out) {
    constexpr int HD = 128, QT = 64, KT = 32;
    constexpr bool HALF_KV = std::is_same<KV, _Float16>::value;  // cache values are their own fp16 head: no tail tiles
    constexpr int KP = HD + 8;   // K tile pitch in halves (272 bytes: the 16 rows of an operand read hit distinct banks)
    constexpr int VP = KT + 8;   // V^T tile pitch in halves (80 bytes, same property)
    constexpr int PP = KT + 8;   // P tile pitch
    constexpr int K_HALVES = 2 * KT * KP, VT_HALVES = 2 * HD * VP, P_HALVES = 4 * 2 * 16 * PP;
    constexpr int GROUP_HALVES = K_HALVES + VT_HALVES + P_HALVES;
    static_assert(GROUP_HALVES * 2 >= 40 * 256 * 4, "a group's buffers hold the other group's state at the merge");
    __shared__ __align__(16) _Float16 s_all[GROUPS * GROUP_HALVES];
    const int grp = GROUPS == 1 ? 0 : (int)(threadIdx.x >> 8);
    const int tid = threadIdx.x & 255, lane = tid & 63, wave = tid >> 6;
    _Float16 *const s_kb = s_all + grp * GROUP_HALVES;   // [hi/lo][key][d]
    _Float16 *const s_vtb = s_kb + K_HALVES;              // [hi/lo][d][key]
    _Float16 *const s_pb = s_vtb + VT_HALVES;             // per wavefront [hi/lo][row][key]
    _Float16 *const s_k[2] = {s_kb, s_kb + KT * KP};
    _Float16 *const s_vt[2] = {s_vtb, s_vtb + HD * VP};
    const int r16 = lane & 15, c4 = lane >> 4;
    const int head = blockIdx.x, i0 = blockIdx.y * QT;
    const int kvh = head / (n_heads / n_kv_heads);
    const KV *kh = k_cache + (size_t)kvh * cache_stride, *vh = v_cache + (size_t)kvh * cache_stride;
    const int n_keys = pos0 + min(i0 + QT, n);   // positions the tile's last query may see
    const int wave_last = pos0 + i0 + 16 * wave + 15;  // last position any row of this wavefront may see

    // Q as the A operand (row = query r16, 8 consecutive d per k-step), pre-scaled by scale * log2(e) (the softmax
    // runs on powers of two: one v_exp_f32 per value), split hi / lo
    half8 qh[4], ql[4];
    {
        const int i = min(i0 + 16 * wave + r16, n - 1);
        const float *qr = q + ((size_t)i * n_heads + head) * HD;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const float4 a = *(const float4 *)(qr + ks * 32 + c4 * 8), b = *(const float4 *)(qr + ks * 32 + c4 * 8 + 4);
            const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const HiLo t = split_half(v[e] * (scale * 1.44269504088896341f));
                qh[ks][e] = t.hi;
                ql[ks][e] = t.lo;
            }
        }
    }
    // C layout: lane holds rows 4*c4 + j (j = 0..3) of the wavefront's 16 queries, column r16
    float m_run[4], l_run[4];
    float4v o[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) { m_run[j] = -INFINITY; l_run[j] = 0.0f; }
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) o[dt] = float4v{0.f, 0.f, 0.f, 0.f};

    // global -> register requests of a tile: K: thread -> (key, 4 consecutive d), 4 passes; V: thread -> (key pair,
    // 4 consecutive d), 2 passes.  The next tile is requested before the current one is consumed.
    float4 kreg[4], vreg[2][2];
    auto request = [&](int p0) __attribute__((always_inline)) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int e = tid + it * 256, key = e >> 5, d4 = e & 31;
            kreg[it] = kv_load4(kh + (size_t)min(p0 + key, n_keys - 1) * HD + 4 * d4);
        }
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            // a wavefront's lanes: 16 key pairs x 4 neighbouring d4.  With the 32 d4 of one key pair per half wavefront
            // the transposed stores below put 32 lanes on two LDS banks (a row of V^T is 80 bytes: 4 rows are 320,
            // a multiple of 64) - 16-way conflicts on every one of them: 512 prompt tokens 48 -> 42.5 us per launch
            const int e = tid + it * 256, kp = e & 15, d4 = e >> 4;
            vreg[it][0] = kv_load4(vh + (size_t)min(p0 + 2 * kp, n_keys - 1) * HD + 4 * d4);
            vreg[it][1] = kv_load4(vh + (size_t)min(p0 + 2 * kp + 1, n_keys - 1) * HD + 4 * d4);
        }
    };
    // every group runs the same number of rounds (the barriers are the workgroup's); a group without a tile in the
    // last round sits it out
    const int n_rounds = ((n_keys + KT - 1) / KT + GROUPS - 1) / GROUPS;
    if (grp * KT < n_keys) request(grp * KT);
    for (int round = 0; round < n_rounds; ++round) {
        const int p0 = (round * GROUPS + grp) * KT;
        __syncthreads();  // previous tile fully consumed
        if (GROUPS > 1 && p0 >= n_keys) {
            __syncthreads();
            continue;
        }
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int e = tid + it * 256, key = e >> 5, d4 = e & 31;
            const float4 kv = kreg[it];
            half4h hi, lo;
            const float kvv[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const HiLo t = split_half(kvv[c]);
                hi[c] = t.hi;
                lo[c] = t.lo;
            }
            *(half4h *)&s_k[0][key * KP + 4 * d4] = hi;
            if (!HALF_KV) *(half4h *)&s_k[1][key * KP + 4 * d4] = lo;
        }
        // V transposed: two keys of one d share a 32-bit store
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int e = tid + it * 256, kp = e & 15, d4 = e >> 4;
            const float4 v0 = vreg[it][0], v1 = vreg[it][1];
            const float a[4] = {v0.x, v0.y, v0.z, v0.w}, b[4] = {v1.x, v1.y, v1.z, v1.w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                half2h hi, lo;
                const HiLo ta = split_half(a[c]), tb = split_half(b[c]);
                hi[0] = ta.hi; lo[0] = ta.lo;
                hi[1] = tb.hi; lo[1] = tb.lo;
                *(half2h *)&s_vt[0][(4 * d4 + c) * VP + 2 * kp] = hi;
                if (!HALF_KV) *(half2h *)&s_vt[1][(4 * d4 + c) * VP + 2 * kp] = lo;
            }
        }
        if (p0 + GROUPS * KT < n_keys) request(p0 + GROUPS * KT);
        __syncthreads();
        if (p0 > wave_last) continue;  // every key of the tile is in the future of all 16 rows (the barriers above stay uniform)

        // ---- S = Q.K^T for 32 keys: two 16-key column tiles
        float4v s_acc[2];
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
            float4v acc = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const int off = (nt * 16 + r16) * KP + ks * 32 + c4 * 8;
                const half8 kh8 = *(const half8 *)&s_k[0][off];
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ql[ks], kh8, acc, 0, 0, 0);
                if (!HALF_KV) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(qh[ks], *(const half8 *)&s_k[1][off], acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(qh[ks], kh8, acc, 0, 0, 0);
            }
            s_acc[nt] = acc;
        }
        // ---- online softmax per row
        float corr[4];
        _Float16 *ph = s_pb + wave * 2 * 16 * PP, *pl = ph + 16 * PP;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int qpos = pos0 + i0 + 16 * wave + 4 * c4 + j;
            float sv[2];
            float mx = -INFINITY;
#pragma unroll
            for (int nt = 0; nt < 2; ++nt) {
                const bool ok = p0 + nt * 16 + r16 <= qpos;
                sv[nt] = ok ? s_acc[nt][j] : -INFINITY;
                mx = fmaxf(mx, sv[nt]);
            }
            mx = row16_max(mx);
            // position 0 is visible to every row: with one group finite from the first tile on; a second group's first
            // tile may lie in a row's future altogether
            const float m_new = fmaxf(m_run[j], mx);
            const bool seen = GROUPS == 1 || m_new != -INFINITY;
            corr[j] = seen ? __builtin_amdgcn_exp2f(m_run[j] - m_new) : 1.0f;
            float ps = 0.0f;
#pragma unroll
            for (int nt = 0; nt < 2; ++nt) {
                const float pw = seen ? __builtin_amdgcn_exp2f(sv[nt] - m_new) : 0.0f;  // 2^-inf = 0 for masked keys
                ps += pw;
                const HiLo t = split_half(pw);
                ph[(4 * c4 + j) * PP + nt * 16 + r16] = t.hi;
                pl[(4 * c4 + j) * PP + nt * 16 + r16] = t.lo;
            }
            ps = row16_sum(ps);
            l_run[j] = l_run[j] * corr[j] + ps;
            m_run[j] = m_new;
        }
        // the running maxima settle after the first tiles: most rounds have nothing to rescale
        if (__any(corr[0] != 1.0f || corr[1] != 1.0f || corr[2] != 1.0f || corr[3] != 1.0f)) {
#pragma unroll
            for (int dt = 0; dt < 8; ++dt)
#pragma unroll
                for (int j = 0; j < 4; ++j) o[dt][j] *= corr[j];
        }
        // the wavefront's own P tile: its LDS operations complete in order, no workgroup barrier needed
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // ---- O += P.V: P as the A operand (row r16, keys 8*c4 .. +7), V^T rows as the B operand
        const half8 pa_h = *(const half8 *)&ph[r16 * PP + c4 * 8], pa_l = *(const half8 *)&pl[r16 * PP + c4 * 8];
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) {
            const int off = (dt * 16 + r16) * VP + c4 * 8;
            const half8 vh8 = *(const half8 *)&s_vt[0][off];
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa_l, vh8, o[dt], 0, 0, 0);
            if (!HALF_KV) o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa_h, *(const half8 *)&s_vt[1][off], o[dt], 0, 0, 0);
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa_h, vh8, o[dt], 0, 0, 0);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    if constexpr (GROUPS == 2) {
        // the second group's state goes through its own tile buffers (value k of thread t at k * 256 + t); the first
        // group, whose tiles hold position 0, always has a finite maximum
        float *st = (float *)(s_all + GROUP_HALVES);
        __syncthreads();
        if (grp == 1) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                st[j * 256 + tid] = m_run[j];
                st[(4 + j) * 256 + tid] = l_run[j];
            }
#pragma unroll
            for (int dt = 0; dt < 8; ++dt)
#pragma unroll
                for (int j = 0; j < 4; ++j) st[(8 + 4 * dt + j) * 256 + tid] = o[dt][j];
        }
        __syncthreads();
        if (grp == 1) return;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float m1 = st[j * 256 + tid], l1 = st[(4 + j) * 256 + tid];
            const float m = fmaxf(m_run[j], m1);
            const float f0 = __builtin_amdgcn_exp2f(m_run[j] - m), f1 = __builtin_amdgcn_exp2f(m1 - m);
            l_run[j] = l_run[j] * f0 + l1 * f1;
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) o[dt][j] = o[dt][j] * f0 + st[(8 + 4 * dt + j) * 256 + tid] * f1;
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int i = i0 + 16 * wave + 4 * c4 + j;
        if (i >= n) continue;
        const float inv = 1.0f / l_run[j];
        if (xh_out) {
            // The output row leaves as the fp16 image of its Q8_0 quantization (what the o projection's fp16 tiles
            // contract with), the arithmetic of quantize_q8_lane4 + q8_lane4_to_half value by value: a 32-value block
            // is columns 32 b .. 32 b + 31 = this 16-lane row's o[2 b] and o[2 b + 1].
            const int K = n_heads * HD;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const float v0 = o[2 * b][j] * inv, v1 = o[2 * b + 1][j] * inv;
                const float amax = row16_max(fmaxf(fabsf(v0), fabsf(v1)));
                const float d = amax / 127.0f;
                const int q0 = amax != 0.0f ? q8_level(v0, d) : 0, q1 = amax != 0.0f ? q8_level(v1, d) : 0;
                const float df = __half2float(__float2half_rn(d));
                const int col = head * HD + 32 * b + r16;
                xh_out[xh_index4(i, col >> 2, K) * 4 + (col & 3)] = (_Float16)(df * (float)q0);
                xh_out[xh_index4(i, (col + 16) >> 2, K) * 4 + (col & 3)] = (_Float16)(df * (float)q1);
            }
            continue;
        }
        float *dst = out + ((size_t)i * n_heads + head) * HD + r16;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) dst[dt * 16] = o[dt][j] * inv;
    }
}

int launch_prefill_rope_kv(candy_hip_device *dev, float *q, const float *k, const float *v, const float *cos_t,
                           const float *sin_t, void *k_cache, void *v_cache, bool kv_f16, int n, int pos0, int n_heads,
                           int n_kv_heads, int head_dim, int64_t cache_stride, const SplitPending *sp) {
    const size_t q_count = (size_t)n * n_heads * head_dim, kv_count = (size_t)n * n_kv_heads * head_dim;
    const bool pending = sp && sp->n_split > 0;
    if (pending) CANDY_REQUIRE(sp->y == q && !sp->res && sp->count == q_count + 2 * kv_count, "internal: pending split sum of another shape");
    if (head_dim % 8 == 0 && k == q + q_count && v == k + kv_count && dev->opt.prefill_fold_split_sums) {
        // q, k and v end to end: four pairs per thread, and the partial copies of a split contraction summed on the way
        const int64_t total4 = (int64_t)n * (n_heads + 2 * n_kv_heads) * (head_dim / 8);
        const dim3 grid4((unsigned)((total4 + 255) / 256));
        const float *src = pending ? sp->part : q;
        const int n_split = pending ? sp->n_split : 1;
        const size_t stride = pending ? sp->stride : 0;
        if (kv_f16)
            hipLaunchKernelGGL(k_prefill_rope_kv4<_Float16>, grid4, dim3(256), 0, dev->stream, q, src, n_split, stride, cos_t,
                               sin_t, (_Float16 *)k_cache, (_Float16 *)v_cache, n, pos0, n_heads, n_kv_heads, head_dim,
                               cache_stride);
        else
            hipLaunchKernelGGL(k_prefill_rope_kv4<float>, grid4, dim3(256), 0, dev->stream, q, src, n_split, stride, cos_t,
                               sin_t, (float *)k_cache, (float *)v_cache, n, pos0, n_heads, n_kv_heads, head_dim,
                               cache_stride);
        CANDY_LAUNCH_CHECK();
        return CANDY_HIP_OK;
    }
    if (pending)
        if (int rc = launch_splitk_sum(dev, sp->part, sp->y, nullptr, sp->count, sp->n_split, sp->stride)) return rc;
    const int64_t total = (int64_t)n * (n_heads + 2 * n_kv_heads) * (head_dim / 2);
    const dim3 grid((unsigned)((total + 255) / 256));
    if (kv_f16)
        hipLaunchKernelGGL(k_prefill_rope_kv<_Float16>, grid, dim3(256), 0, dev->stream, q, k, v, cos_t, sin_t,
                           (_Float16 *)k_cache, (_Float16 *)v_cache, n, pos0, n_heads, n_kv_heads, head_dim, cache_stride);
    else
        hipLaunchKernelGGL(k_prefill_rope_kv<float>, grid, dim3(256), 0, dev->stream, q, k, v, cos_t, sin_t,
                           (float *)k_cache, (float *)v_cache, n, pos0, n_heads, n_kv_heads, head_dim, cache_stride);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

template <class KV>
static void launch_attn_prefill_kv(candy_hip_device *dev, const float *q, const KV *k_cache, const KV *v_cache, float *out,
                                   int n, int pos0, int n_heads, int n_kv_heads, int head_dim, int64_t cache_stride,
                                   float scale, _Float16 *xh_out) {
    const dim3 grid((unsigned)n_heads, (unsigned)((n + 31) / 32));
    const bool valu_only = dev->opt.prefill_attention_valu != 0;  // comparison runs
    if (head_dim == 128 && !valu_only) {
        // Two key-tile groups per workgroup where the launch lasts as long as its longest workgroup: a grid of about one
        // workgroup per CU and a walk of more than four key tiles.  A larger grid fills the CUs with several of the
        // smaller workgroups, a shorter walk does not pay for the merge.
        const dim3 tiles((unsigned)n_heads, (unsigned)((n + 63) / 64));
        const int64_t wgs = (int64_t)tiles.x * tiles.y;
        const int groups = dev->opt.prefill_attention_groups ? dev->opt.prefill_attention_groups
                                                             : (n > 128 && 2 * wgs <= 3 * (int64_t)dev->num_cus ? 2 : 1);
        if (groups == 2)
            hipLaunchKernelGGL((k_attn_prefill_mfma<KV, 2>), tiles, dim3(512), 0, dev->stream, q, k_cache, v_cache, out, n,
                               pos0, n_heads, n_kv_heads, cache_stride, scale, xh_out);
        else
            hipLaunchKernelGGL((k_attn_prefill_mfma<KV, 1>), tiles, dim3(256), 0, dev->stream, q, k_cache, v_cache, out, n,
                               pos0, n_heads, n_kv_heads, cache_stride, scale, xh_out);
    } else if (head_dim == 128)
        hipLaunchKernelGGL((k_attn_prefill<128, KV>), grid, dim3(256), 0, dev->stream, q, k_cache, v_cache, out, n, pos0,
                           n_heads, n_kv_heads, cache_stride, scale);
    else
        hipLaunchKernelGGL((k_attn_prefill<64, KV>), grid, dim3(256), 0, dev->stream, q, k_cache, v_cache, out, n, pos0,
                           n_heads, n_kv_heads, cache_stride, scale);
}

// The matrix-core kernel can leave its output as the fp16 image of the quantized rows instead of f32 (no separate
// quantize launch in front of an o projection that runs on the fp16 tiles).
bool attn_prefill_writes_half(const candy_hip_device *dev, int head_dim) {
    return head_dim == 128 && !dev->opt.prefill_attention_valu && dev->opt.prefill_fold_split_sums;
}

int launch_attn_prefill(candy_hip_device *dev, const float *q, const void *k_cache, const void *v_cache, bool kv_f16,
                        float *out, int n, int pos0, int n_heads, int n_kv_heads, int head_dim, int64_t cache_stride,
                        float scale, _Float16 *xh_out) {
    CANDY_REQUIRE(head_dim == 64 || head_dim == 128, "head_dim must be 64 or 128");
    CANDY_REQUIRE(n > 0 && pos0 >= 0 && n_heads % n_kv_heads == 0, "invalid attention shape");
    CANDY_REQUIRE(!xh_out || attn_prefill_writes_half(dev, head_dim), "internal: this attention kernel writes f32 only");
    if (kv_f16)
        launch_attn_prefill_kv(dev, q, (const _Float16 *)k_cache, (const _Float16 *)v_cache, out, n, pos0, n_heads,
                               n_kv_heads, head_dim, cache_stride, scale, xh_out);
    else
        launch_attn_prefill_kv(dev, q, (const float *)k_cache, (const float *)v_cache, out, n, pos0, n_heads, n_kv_heads,
                               head_dim, cache_stride, scale, xh_out);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

}  // namespace candy
