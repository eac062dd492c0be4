// Batch-1 attention of one new token over the f32 KV cache: softmax(q.K^T * scale).V per head,
// the MatMul / FastSoftmax / MatMul sequence (backend.go:78, :147) a candy Llama block issues,
// with Rope (backend.go:159, reduce.go:3987-4006) on the new q / k rows folded in.
//
// HBM-bound: every step reads 2 * n_pos * head_dim * 4 bytes per kv head. The cache is split over
// positions (grid = kv heads x splits); all query heads that share a kv head ride on one pass
// over K and V. Half a wavefront (32 lanes x VEC floats) holds one cache row, so a load
// instruction brings two positions, UNR of them are issued back to back (2*UNR positions = up to
// 8 KB of K and of V in flight per wavefront), the dot products are reduced on the DPP path, and
// each half-wavefront keeps a running (max, sum, weighted V) per query head. The workgroup's
// eight partial states meet in LDS and leave as one partial per (head, split); a second, tiny
// kernel merges the splits and, if asked, quantizes the head outputs to planar Q8_0 for the
// output projection.  (Merging in the last workgroup to finish was measured and dropped: the
// device-scope release fence it needs writes back the whole L2 of the XCD, once per workgroup.)
#include "blocks.h"
#include "internal.h"

namespace candy {

constexpr float NEG_BIG = -3.402823466e+38f;

// Sum over each 32-lane half of the wavefront; every lane gets its half's total.
__device__ __forceinline__ float half_wave_sum(float v) {
    v += dpp_move<0xB1>(v);        // quad_perm [1,0,3,2]
    v += dpp_move<0x4E>(v);        // quad_perm [2,3,0,1]
    v += dpp_move<0x141>(v);       // row_half_mirror
    v += dpp_move<0x140>(v);       // row_mirror: row sums
    v += dpp_move<0x142, 0xA>(v);  // row_bcast:15: rows 1 and 3 now hold their half's sum in every lane
    const float lo = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 31));
    const float hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
    return (threadIdx.x & 32) ? hi : lo;
}

// What the first cache loads need are the kernel's plain leading arguments (14 dwords: they arrive in registers with
// the wavefront, so the position can be fetched at once); the rest comes through the argument block.
struct AttnHead {
    const int *pos_ptr;    // optional: position of the new token in device memory
    void *k_cache;         // [n_kv_heads, *, hd] of f32 or fp16 (the kernel's KV type), cache_stride elements between heads
    void *v_cache;
    const float *q;        // [n_heads, hd]; pre-Rope when k_new is set
    int64_t cache_stride;
    int n_pos;             // used when pos_ptr is null: positions 0..n_pos-1 are in the cache
    int n_splits;
    float scale;
    int fresh;             // the new token's k / v rows arrive in k_new / v_new (pre-Rope) and are appended here
};
struct AttnRest {
    const float *k_new;    // optional [n_kv_heads, hd] pre-Rope key of the new token
    const float *v_new;    // optional [n_kv_heads, hd]
    const float *cos_t;    // [max_pos, hd/2] (only with k_new)
    const float *sin_t;
    float *part_o;         // [n_heads, n_splits, hd]
    float *part_ml;        // [n_heads, n_splits, 2]
    float *out;            // optional [n_heads, hd]
    int8_t *oq;            // optional planar Q8_0 of the output
    Q8Scale *os;
};
struct AttnArgs {
    AttnHead h;
    AttnRest r;
};

// KV: float (candy's cache) or _Float16 (optional: half the bytes of the step's largest stream; the rows are
// rounded once, when they enter the cache, and every product and sum stays f32).
template <int GROUP, int VEC, class KV>
__global__ __launch_bounds__(256) void k_attn_decode(const int *__restrict__ pos_ptr, void *k_cache, void *v_cache,
                                                     const float *__restrict__ q, int64_t cache_stride, int n_pos,
                                                     int n_splits, float scale, int fresh_arg, const AttnRest a) {
    constexpr int HD = 32 * VEC;
    constexpr int UNR = 4;
    typedef float vecf __attribute__((ext_vector_type(VEC)));
    typedef KV veckv __attribute__((ext_vector_type(VEC)));
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int hw = lane >> 5, hl = lane & 31;
    const int kvh = blockIdx.x, split = blockIdx.y;
    const bool fresh = fresh_arg != 0;                        // new token's k/v arrive in registers
    KV *kh = (KV *)k_cache + (size_t)kvh * cache_stride;
    KV *vh = (KV *)v_cache + (size_t)kvh * cache_stride;
    // Groups of 32 cached positions (one batch of rows per wavefront of the workgroup) are dealt to the splits round
    // robin: split s takes groups s, s + n_splits, ...  Which rows a split reads first therefore does not depend on
    // the position, and its first batch is requested before the position (a scalar load from device memory, a
    // memory round trip of its own) is known; rows at or past the position are masked afterwards.  With the position
    // in device memory the cache is the decoder's own and every row below cache_stride / HD is memory of this head;
    // with the position as an argument only the rows up to it are known to exist.
    constexpr int GROUP_POS = 4 * 2 * UNR;
    const int max_row = pos_ptr ? (int)(cache_stride / HD) - 1 : n_pos - 1;
    vecf kv0[UNR], vv0[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        const int p = split * GROUP_POS + wave * 2 * UNR + 2 * u + hw;
        const size_t off = (size_t)min(p, max_row) * HD + hl * VEC;
        kv0[u] = __builtin_convertvector(__builtin_nontemporal_load((const veckv *)(kh + off)), vecf);
        vv0[u] = __builtin_convertvector(__builtin_nontemporal_load((const veckv *)(vh + off)), vecf);
    }
    const int pos = pos_ptr ? *pos_ptr : n_pos - 1;           // position of the new token
    const int n_cached = fresh ? pos : pos + 1;               // rows to read from the cache
    const int n_groups = (n_cached + GROUP_POS - 1) / GROUP_POS;
    const int p1 = n_cached;

    // Rope pairs (i, i + HD/2) sit 16 lanes apart inside the half-wavefront
    vecf cs, sn;
    if (fresh) {
        const int i0 = (hl & 15) * VEC;
        cs = *(const vecf *)(a.cos_t + (size_t)pos * (HD / 2) + i0);
        sn = *(const vecf *)(a.sin_t + (size_t)pos * (HD / 2) + i0);
    }
    auto rope = [&](vecf v) -> vecf {
        vecf other, r;
#pragma unroll
        for (int j = 0; j < VEC; ++j) other[j] = __shfl_xor(v[j], 16, 64);
#pragma unroll
        for (int j = 0; j < VEC; ++j)  // low half: a*c - b*s ; high half: a*s + b*c with (a, b) = (low, high)
            r[j] = hl < 16 ? v[j] * cs[j] - other[j] * sn[j] : other[j] * sn[j] + v[j] * cs[j];
        return r;
    };

    vecf qv[GROUP];
#pragma unroll
    for (int g = 0; g < GROUP; ++g) {
        qv[g] = *(const vecf *)(q + (size_t)(kvh * GROUP + g) * HD + hl * VEC);
        if (fresh) qv[g] = rope(qv[g]);
    }

    float m_run[GROUP], l_run[GROUP];
    vecf o_run[GROUP];
#pragma unroll
    for (int g = 0; g < GROUP; ++g) {
        m_run[g] = NEG_BIG;
        l_run[g] = 0.0f;
#pragma unroll
        for (int j = 0; j < VEC; ++j) o_run[g][j] = 0.0f;
    }

    auto absorb = [&](const vecf (&kv)[UNR], const vecf (&vv)[UNR], const bool (&valid)[UNR]) {
#pragma unroll
        for (int g = 0; g < GROUP; ++g) {
            float s[UNR];
            float m_new = m_run[g];
#pragma unroll
            for (int u = 0; u < UNR; ++u) {
                float d = 0.0f;
#pragma unroll
                for (int j = 0; j < VEC; ++j) d += qv[g][j] * kv[u][j];
                d = half_wave_sum(d) * scale;
                s[u] = valid[u] ? d : NEG_BIG;
                m_new = fmaxf(m_new, s[u]);
            }
            const float corr = expf(m_run[g] - m_new);
            float l = l_run[g] * corr;
            vecf o = o_run[g] * corr;
#pragma unroll
            for (int u = 0; u < UNR; ++u) {
                const float pw = valid[u] ? expf(s[u] - m_new) : 0.0f;
                l += pw;
                o += pw * vv[u];
            }
            m_run[g] = m_new;
            l_run[g] = l;
            o_run[g] = o;
        }
    };

    // cached positions: in group g wavefront w, half hw, slot u takes position 32 g + 8 w + 2u + hw.  The next
    // group's rows are requested before the current ones are absorbed, so two batches (up to 16 KB) are in flight
    // per wavefront.
    auto fetch = [&](int base, vecf (&kv)[UNR], vecf (&vv)[UNR], bool (&valid)[UNR]) {
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const int p = base + 2 * u + hw;
            valid[u] = p < p1;
            const size_t off = (size_t)max(min(p, p1 - 1), 0) * HD + hl * VEC;
            // every cache byte is read once, by one instruction: stream it past the caches
            kv[u] = __builtin_convertvector(__builtin_nontemporal_load((const veckv *)(kh + off)), vecf);
            vv[u] = __builtin_convertvector(__builtin_nontemporal_load((const veckv *)(vh + off)), vecf);
        }
    };
    {
        int g = split;
        vecf kv[UNR], vv[UNR], kn[UNR], vn[UNR];
        bool valid[UNR], vnext[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {  // the first group: requested above
            kv[u] = kv0[u];
            vv[u] = vv0[u];
            valid[u] = split * GROUP_POS + wave * 2 * UNR + 2 * u + hw < p1;
        }
        while (g < n_groups) {
            const int gn = g + n_splits;
            if (gn < n_groups) fetch(gn * GROUP_POS + wave * 2 * UNR, kn, vn, vnext);
            absorb(kv, vv, valid);
            if (gn >= n_groups) break;
#pragma unroll
            for (int u = 0; u < UNR; ++u) {
                kv[u] = kn[u];
                vv[u] = vn[u];
                valid[u] = vnext[u];
            }
            g = gn;
        }
    }

    // the new token: Rope its key, append both rows to the cache, attend to them from registers
    if (fresh && split == n_splits - 1 && wave == 0) {
        vecf kn = rope(*(const vecf *)(a.k_new + (size_t)kvh * HD + hl * VEC));
        vecf vn = *(const vecf *)(a.v_new + (size_t)kvh * HD + hl * VEC);
        const veckv kc = __builtin_convertvector(kn, veckv), vc = __builtin_convertvector(vn, veckv);
        if (hw == 0) {
            *(veckv *)(kh + (size_t)pos * HD + hl * VEC) = kc;
            *(veckv *)(vh + (size_t)pos * HD + hl * VEC) = vc;
        }
        kn = __builtin_convertvector(kc, vecf);  // attend to the rows as the cache holds them
        vn = __builtin_convertvector(vc, vecf);
        vecf kv[UNR], vv[UNR];
        bool valid[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            kv[u] = kn;
            vv[u] = vn;
            valid[u] = (u == 0) && (hw == 0);
        }
        absorb(kv, vv, valid);
    }

    // merge the workgroup's 8 half-wavefront states
    __shared__ float sm[8][GROUP], sl[8][GROUP];
    __shared__ float so[8][GROUP][HD];
    const int slot = wave * 2 + hw;
#pragma unroll
    for (int g = 0; g < GROUP; ++g) {
        if (hl == 0) {
            sm[slot][g] = m_run[g];
            sl[slot][g] = l_run[g];
        }
        *(vecf *)&so[slot][g][hl * VEC] = o_run[g];
    }
    __syncthreads();
    for (int idx = tid; idx < GROUP * HD; idx += 256) {
        const int g = idx / HD, c = idx - g * HD;
        float m = sm[0][g];
#pragma unroll
        for (int w = 1; w < 8; ++w) m = fmaxf(m, sm[w][g]);
        float l = 0.0f, o = 0.0f;
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            const float f = expf(sm[w][g] - m);
            l += sl[w][g] * f;
            o += so[w][g][c] * f;
        }
        const size_t ps = (size_t)(kvh * GROUP + g) * n_splits + split;
        a.part_o[ps * HD + c] = o;
        if (c == 0) {
            a.part_ml[ps * 2 + 0] = m;
            a.part_ml[ps * 2 + 1] = l;
        }
    }

}

// Merges the splits of one head (one workgroup per head) and, if asked, quantizes the head output to planar Q8_0 for
// the output projection.  Everything it needs is requested up front: lane s of every wavefront reads split s's
// (max, sum); the 256 threads share the head's partial outputs as 16-byte loads, thread (sg, c4) taking columns
// 4 c4 .. 4 c4 + 3 of splits sg, sg + SG, ...; the SG partial sums per column meet in LDS.
template <int HD>
__global__ __launch_bounds__(256) void k_attn_merge(const float *__restrict__ part_o, const float *__restrict__ part_ml,
                                                    int n_splits, float *__restrict__ out, int8_t *__restrict__ oq,
                                                    Q8Scale *__restrict__ os) {
    constexpr int MAX_SPLITS = 64, C4 = HD / 4, SG = 256 / C4, PER = MAX_SPLITS / SG;
    const int h = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
    const int c4 = tid % C4, sg = tid / C4;
    const float2 *ml = (const float2 *)(part_ml + (size_t)h * n_splits * 2);
    const float4 *po = (const float4 *)(part_o + (size_t)h * n_splits * HD) + c4;
    const float2 mine = lane < n_splits ? ml[lane] : make_float2(NEG_BIG, 0.0f);
    float4 acc[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        // splits at and past n_splits re-read the last one (finite values) and get weight zero below: no branch
        // around a load, every load in flight before the first wait
        acc[j] = po[(size_t)min(sg + SG * j, n_splits - 1) * C4];
    }
    __builtin_amdgcn_sched_barrier(0);  // keep the reductions below from being scheduled between the loads
    const float m = wave_max(mine.x);
    const float f = lane < n_splits ? expf(mine.x - m) : 0.0f;
    const float l = wave_sum(mine.y * f);
    float4 o4 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const float fs = __shfl(f, sg + SG * j, 64);  // zero for lanes at and past n_splits
        o4.x += acc[j].x * fs;
        o4.y += acc[j].y * fs;
        o4.z += acc[j].z * fs;
        o4.w += acc[j].w * fs;
    }
    __shared__ float4 red[SG][C4];
    red[sg][c4] = o4;
    __syncthreads();
    if (tid >= HD) return;
    const int c = tid;
    float o = 0.0f;
#pragma unroll
    for (int g = 0; g < SG; ++g) o += ((const float *)&red[g][0])[c];
    o *= 1.0f / l;
    if (out) out[(size_t)h * HD + c] = o;
    if (oq) {
        __half dh;
        int bsum;
        const int q8 = quantize_q8_lane1(o, dh, bsum);
        const size_t i = (size_t)h * HD + c;
        oq[i] = (int8_t)q8;
        if ((c & 31) == 0) {
            Q8Scale sc;
            sc.d = __half2float(dh);
            sc.bsum = bsum;
            os[i >> 5] = sc;
        }
    }
}

int attention_splits(const candy_hip_device *dev, int64_t n_kv_heads, int64_t max_pos) {
    // enough workgroups to fill the chip a few times over (twice as many measured slower: 7B shape at 2048 positions
    // 531 against 539 tokens/s), at least 32 positions per split - one batch of rows per wavefront (Llama-3-8B shape at
    // 512-640 positions: 503 tokens/s against 489 with 64 and 491 with 16) -, at most 64 splits (the merge kernel
    // gives each split a lane)
    int n_splits = (int)((4 * (int64_t)dev->num_cus + n_kv_heads - 1) / n_kv_heads);
    const int max_splits = (int)((max_pos + 31) / 32);
    if (dev->opt.attn_splits > 0) n_splits = dev->opt.attn_splits;  // comparison runs
    if (n_splits > max_splits) n_splits = max_splits;
    if (n_splits > 64) n_splits = 64;
    return n_splits < 1 ? 1 : n_splits;
}

size_t attention_scratch_bytes(int n_heads, int n_kv_heads, int head_dim, int n_splits) {
    (void)n_kv_heads;
    return ((size_t)n_heads * n_splits * (head_dim + 2) + 64) * sizeof(float);
}

template <int GROUP, class KV>
static int launch_group(candy_hip_device *dev, const AttnArgs &a, int n_kv_heads, int head_dim) {
    dim3 grid((unsigned)n_kv_heads, (unsigned)a.h.n_splits);
    const AttnHead &h = a.h;
    const unsigned n_heads = (unsigned)(n_kv_heads * GROUP);
    switch (head_dim) {
    case 64:
        hipLaunchKernelGGL((k_attn_decode<GROUP, 2, KV>), grid, dim3(256), 0, dev->stream, h.pos_ptr, h.k_cache, h.v_cache,
                           h.q, h.cache_stride, h.n_pos, h.n_splits, h.scale, h.fresh, a.r);
        CANDY_LAUNCH_CHECK();
        hipLaunchKernelGGL((k_attn_merge<64>), dim3(n_heads), dim3(256), 0, dev->stream, a.r.part_o, a.r.part_ml, h.n_splits,
                           a.r.out, a.r.oq, a.r.os);
        break;
    case 128:
        hipLaunchKernelGGL((k_attn_decode<GROUP, 4, KV>), grid, dim3(256), 0, dev->stream, h.pos_ptr, h.k_cache, h.v_cache,
                           h.q, h.cache_stride, h.n_pos, h.n_splits, h.scale, h.fresh, a.r);
        CANDY_LAUNCH_CHECK();
        hipLaunchKernelGGL((k_attn_merge<128>), dim3(n_heads), dim3(256), 0, dev->stream, a.r.part_o, a.r.part_ml,
                           h.n_splits, a.r.out, a.r.oq, a.r.os);
        break;
    default: return fail(CANDY_HIP_ERR_UNSUPPORTED, "head_dim %d unsupported (64 or 128)", head_dim);
    }
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int launch_attention(candy_hip_device *dev, const AttnLaunch &L) {
    AttnArgs a{};
    a.h.q = L.q; a.r.k_new = L.k_new; a.r.v_new = L.v_new; a.r.cos_t = L.cos_t; a.r.sin_t = L.sin_t;
    a.h.fresh = L.k_new != nullptr;
    a.h.k_cache = L.k_cache; a.h.v_cache = L.v_cache; a.h.pos_ptr = L.pos_ptr; a.h.n_pos = L.n_pos;
    a.h.cache_stride = L.cache_stride; a.h.scale = L.scale; a.h.n_splits = L.n_splits;
    a.r.part_o = (float *)L.scratch;
    a.r.part_ml = a.r.part_o + (size_t)L.n_heads * L.n_splits * L.head_dim;
    a.r.out = L.out; a.r.oq = L.oq; a.r.os = L.os;
    const int group = L.n_heads / L.n_kv_heads;
    if (L.kv_f16) switch (group) {
        case 1: return launch_group<1, _Float16>(dev, a, L.n_kv_heads, L.head_dim);
        case 2: return launch_group<2, _Float16>(dev, a, L.n_kv_heads, L.head_dim);
        case 4: return launch_group<4, _Float16>(dev, a, L.n_kv_heads, L.head_dim);
        case 8: return launch_group<8, _Float16>(dev, a, L.n_kv_heads, L.head_dim);
        default: return fail(CANDY_HIP_ERR_UNSUPPORTED, "query heads per kv head must be 1, 2, 4 or 8");
        }
    switch (group) {
    case 1: return launch_group<1, float>(dev, a, L.n_kv_heads, L.head_dim);
    case 2: return launch_group<2, float>(dev, a, L.n_kv_heads, L.head_dim);
    case 4: return launch_group<4, float>(dev, a, L.n_kv_heads, L.head_dim);
    case 8: return launch_group<8, float>(dev, a, L.n_kv_heads, L.head_dim);
    default: return fail(CANDY_HIP_ERR_UNSUPPORTED, "query heads per kv head must be 1, 2, 4 or 8");
    }
}

}  // namespace candy

using namespace candy;

extern "C" int candy_hip_attention_decode(candy_hip_device *dev, const float *q, const float *k_cache,
                                          const float *v_cache, int64_t n_heads, int64_t n_kv_heads, int64_t head_dim,
                                          int64_t n_pos, int64_t cache_stride, float scale, float *out) {
    CANDY_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0, "invalid head counts %lld / %lld",
                  (long long)n_heads, (long long)n_kv_heads);
    CANDY_REQUIRE(head_dim == 64 || head_dim == 128, "head_dim %lld unsupported (64 or 128)", (long long)head_dim);
    CANDY_REQUIRE(n_pos > 0 && cache_stride >= n_pos * head_dim, "invalid cache shape");
    CANDY_REQUIRE(n_pos <= 0x7FFFFFFF && n_heads <= 65535, "attention shape too large");
    CANDY_REQUIRE(q && k_cache && v_cache && out, "nil pointer");
    CANDY_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)k_cache & 15) == 0 && ((uintptr_t)v_cache & 15) == 0,
                  "attention operands must be 16-byte aligned");
    const int64_t group = n_heads / n_kv_heads;
    CANDY_REQUIRE(group == 1 || group == 2 || group == 4 || group == 8, "query heads per kv head must be 1, 2, 4 or 8");
    if (int rc = use_device(dev)) return rc;
    AttnLaunch L{};
    L.n_heads = (int)n_heads; L.n_kv_heads = (int)n_kv_heads; L.head_dim = (int)head_dim;
    L.n_splits = attention_splits(dev, n_kv_heads, n_pos);
    const size_t bytes = attention_scratch_bytes(L.n_heads, L.n_kv_heads, L.head_dim, L.n_splits);
    void *ws = nullptr;
    if (int rc = workspace(dev, bytes, &ws)) return rc;
    L.scratch = ws;
    L.q = q; L.k_cache = (float *)k_cache; L.v_cache = (float *)v_cache;
    L.n_pos = (int)n_pos; L.cache_stride = cache_stride; L.scale = scale; L.out = out;
    return launch_attention(dev, L);
}
