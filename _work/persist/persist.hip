// The whole batch-1 decode step of the Llama-style decoder as ONE persistent kernel (experimental, opt-in).
//
// The step issued kernel by kernel (llama.hip) is six launches per layer, and each launch costs about
// 3.4 us that no byte moves in (an empty kernel lasts 1.8 us, then the first load's latency), on top of
// kernels that stream their weights near the HBM rate.  Here one workgroup per compute unit stays
// resident for the whole token and the stages of the step become phases of that kernel.  What a phase
// hands to the next (hidden state, q/k/v, attention partials, activations) travels through device memory
// as 8-byte words that carry their own phase tag next to the value, written with agent-scope stores and
// polled with agent-scope loads (the L2 of one XCD does not snoop another's, and these bypass it).  There
// is no separate barrier: a consumer spins on exactly the words it needs, and requests its first round of
// weights before it starts to wait.  Every spin is bounded: on a time-out the workgroup raises a flag in
// device memory and leaves, the others follow at their own time-outs, and the host falls back to the
// kernel-by-kernel step.
//
// Where it stands (7B shape, 2048 cached positions, 256 CUs): about 75 us per layer against 59.5 us for the
// six launches.  Each phase lasts its weight stream (polls return behind the weight loads issued before
// them) plus quantizing the activations, the dots and one hop through memory, so nothing of one phase yet
// runs under another; and every workgroup reads every exchanged vector whole at 8 bytes per value (88 KB
// for the d_ffn-long one, as much as the workgroup's share of the down projection's weights).  Getting ahead
// needs the next phase's weights requested under the current phase's dots, and the d_ffn-long hand-over
// quantized at the producer.
//
// Arithmetic is that of the kernel-by-kernel step: RMSNorm (reduce.go:3071-3092) and Q8_0 quantization
// (quantized.cu:3521-3558) in the prologues, the integer vec-dots of units.h, Rope (reduce.go:3987-4006),
// online-softmax attention over the f32 cache split over positions, SiLU * Mul (unary.go:3353-3366),
// residual adds, first-maximum argmax (reduce.go:846-862).
//
// Covers: head_dim 128, one kv head per query head, Q4_K layer weights, Q4_K or Q6_K head.
#include <cstdlib>

#include "blocks.h"
#include "internal.h"
#include "persist.h"
#include "units.h"

namespace candy {

constexpr int PT = 512;        // threads per workgroup: 2 wavefronts per SIMD, 256 vector registers each
constexpr int PW = PT / 64;    // wavefronts per workgroup
constexpr int HD = 128;
constexpr int XD = 4096 / 4 / PT;    // float4 chunks per thread of a d_model-long vector (host: d_model <= 4096)
constexpr int XF = 16384 / 4 / PT;   // ... of a d_ffn-long vector (host: d_ffn <= 16384)
constexpr float P_NEG_BIG = -3.402823466e+38f;

__device__ __forceinline__ u64 tagged(float v, unsigned tag) { return ((u64)tag << 32) | __float_as_uint(v); }

__device__ __forceinline__ void publish(u64 *dst, float v, unsigned tag) {
    __hip_atomic_store(dst, tagged(v, tag), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Between two looks at a word that has not arrived.  Longer naps were measured slower (the waiting
// workgroups' polls do not hold up the ones still streaming), shorter ones no faster.
__device__ __forceinline__ void nap() { __builtin_amdgcn_s_sleep(8); }

// Spins until the word carries `tag`; ok is cleared on a time-out (the value is then meaningless).
__device__ __forceinline__ float poll(const u64 *src, unsigned tag, int spin_limit, bool &ok) {
    u64 u = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    int n = 0;
    while ((unsigned)(u >> 32) != tag) {
        if (++n > spin_limit) { ok = false; break; }
        nap();
        u = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return __uint_as_float((unsigned)u);
}

// N words requested together; while any of them lacks the tag, all are requested again (one spin loop
// whatever N is: the kernel's code has to stay within the instruction cache's reach).
template <int N>
__device__ __forceinline__ void poll_n(const u64 *const (&src)[N], unsigned tag, int spin_limit, bool &ok, float (&out)[N]) {
    u64 u[N];
    int n = 0;
    for (;;) {
#pragma unroll
        for (int i = 0; i < N; ++i) u[i] = __hip_atomic_load(src[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        bool all = true;
#pragma unroll
        for (int i = 0; i < N; ++i) all = all && (unsigned)(u[i] >> 32) == tag;
        if (all) break;
        if (++n > spin_limit) { ok = false; break; }
        nap();
    }
#pragma unroll
    for (int i = 0; i < N; ++i) out[i] = __uint_as_float((unsigned)u[i]);
}

// Four consecutive words (one float4 of the exchanged vector).
__device__ __forceinline__ float4 poll4(const u64 *src, unsigned tag, int spin_limit, bool &ok) {
    const u64 *const p[4] = {src, src + 1, src + 2, src + 3};
    float v[4];
    poll_n<4>(p, tag, spin_limit, ok, v);
    return make_float4(v[0], v[1], v[2], v[3]);
}

// The thread's NX float4 chunks (c = tid + i * PT, those below n4) of an exchanged vector, in one spin loop.
template <int NX>
__device__ __forceinline__ void poll_chunks(const u64 *src, int tid, int n4, unsigned tag, int spin_limit, bool &ok,
                                            float4 (&xv)[NX]) {
    u64 u[NX][4];
    int n = 0;
    for (;;) {
        bool all = true;
#pragma unroll
        for (int i = 0; i < NX; ++i) {
            const int c = tid + i * PT;
            if (c < n4) {
#pragma unroll
                for (int j = 0; j < 4; ++j) u[i][j] = __hip_atomic_load(src + 4 * c + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
#pragma unroll
        for (int i = 0; i < NX; ++i) {
            const int c = tid + i * PT;
            if (c < n4) {
#pragma unroll
                for (int j = 0; j < 4; ++j) all = all && (unsigned)(u[i][j] >> 32) == tag;
            }
        }
        if (all) break;
        if (++n > spin_limit) { ok = false; break; }
        nap();
    }
#pragma unroll
    for (int i = 0; i < NX; ++i) {
        const int c = tid + i * PT;
        xv[i] = c < n4 ? make_float4(__uint_as_float((unsigned)u[i][0]), __uint_as_float((unsigned)u[i][1]),
                                     __uint_as_float((unsigned)u[i][2]), __uint_as_float((unsigned)u[i][3]))
                       : make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

// The value again, as far as the compiler knows a new one: what is computed from it inside a phase is not
// hoisted out of the layer loop (hoisted, such per-thread offsets of all six phases stay live together and
// end in scratch memory).
__device__ __forceinline__ int opaque(int x) {
    asm volatile("" : "+v"(x));
    return x;
}
#define PHASE_IDS                                                    \
    const int tid = opaque(tid0);                                    \
    const int lane = tid & 63;                                       \
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);       \
    (void)lane; (void)wave;

// The layer table holds addresses as integers: a pointer read from device memory is "generic" to the compiler
// and its loads become flat loads, which count against the LDS counter as well; made from an integer as a
// pointer to global memory, the loads are global loads.
template <class T>
__device__ __forceinline__ const T *global_ptr(u64 addr) {
    return (const T *)(const __attribute__((address_space(1))) T *)addr;
}
struct LayerPtrs {
    const uint8_t *wq, *wk, *wv, *wo, *gate, *up, *down;
    const float *attn_norm, *ffn_norm;
};

__device__ __forceinline__ float p_silu(float x) { return x / (1.0f + expf(-x)); }

// ---- activations -> LDS image (quants with the 16-byte skew of units.h, then scales)
// Each thread holds NX float4 chunks c = tid + i * PT of the K-long vector (chunks past K/4 are dead).
// RMS: the RMSNorm of fused.hip's prologue (mean of squares over K, eps inside the square root taken in f64).
template <int NX, bool RMS>
__device__ __forceinline__ void stage_activations(int tid, const float4 (&xv)[NX], const float *alpha, float eps, int K,
                                                  int8_t *sq, Q8Scale *ss, float *s_red) {
    const int lane = tid & 63, wave = tid >> 6, n4 = K >> 2;
    float scale = 1.0f;
    if (RMS) {
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < NX; ++i) {
            const float4 v = xv[i];
            const float t = v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
            s += (tid + i * PT < n4) ? t : 0.0f;
        }
        s = wave_sum(s);
        if (lane == 0) s_red[wave] = s;
        __syncthreads();
        float tot = 0.0f;
#pragma unroll
        for (int i = 0; i < PW; ++i) tot += s_red[i];
        scale = 1.0f / (float)sqrt((double)(tot / (float)K + eps));
    }
#pragma unroll
    for (int i = 0; i < NX; ++i) {
        const int c = tid + i * PT;
        float4 v = xv[i];
        if (RMS) {
            const float4 al = c < n4 ? ((const float4 *)alpha)[c] : make_float4(0.f, 0.f, 0.f, 0.f);
            v = make_float4(scale * v.x * al.x, scale * v.y * al.y, scale * v.z * al.z, scale * v.w * al.w);
        }
        if (c >= n4) v = make_float4(0.f, 0.f, 0.f, 0.f);
        __half h;
        int bsum;
        const uint32_t packed = quantize_q8_lane4(v, h, bsum);  // whole wavefronts take part (8 lanes per block)
        if (c < n4) {
            *(uint32_t *)(sq + skewed(4 * c)) = packed;
            if ((c & 7) == 0) {
                Q8Scale sc;
                sc.d = __half2float(h);
                sc.bsum = bsum;
                ss[c >> 3] = sc;
            }
        }
    }
    __syncthreads();
}

// ---- one matvec phase of a wavefront: rounds of R rows each, IT units per lane and row.
// The first round's weights are requested BEFORE the activations are waited for (stage: polls the
// exchanged words, leaves on a time-out, quantizes into the LDS image), so that the exchange's latency
// passes under the weight stream; later rounds load, then contract.
//   rows_fn(r0, rows): the R row pointers of the round that starts at row index r0 (may request more, e.g. residuals)
//   stage_fn() -> bool: false when the workgroup has to leave
//   epi_fn(r0, y): consumes the R sums (every lane holds them)
template <class U, int IT, int R, class RowsFn, class StageFn, class EpiFn, class StampFn>
__device__ __forceinline__ bool phase_rows(int lane, int first, int step, int r_end, int units, const int8_t *sq,
                                           const Q8Scale *ss, RowsFn rows_fn, StageFn stage_fn, EpiFn epi_fn, StampFn stamp_fn) {
    typename U::W w[R][IT];
    const uint8_t *rows[R];
    const int its = (units + 63) >> 6;  // steps in use (<= IT), the same for every wavefront
    auto request = [&](int r0) __attribute__((always_inline)) {
        rows_fn(r0, rows);
#pragma unroll
        for (int it = 0; it < IT; ++it)
            if (it < its) {
#pragma unroll
                for (int r = 0; r < R; ++r) U::load(rows[r], min(it * 64 + lane, units - 1), w[r][it]);
            }
    };
    int r0 = first;
    if (r0 < r_end) request(r0);
    if (!stage_fn()) return false;
    stamp_fn(2);
    while (r0 < r_end) {
        float y[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float acc = 0.0f;
#pragma unroll
            for (int it = 0; it < IT; ++it)
                if (it < its) {
                    const int u = it * 64 + lane;
                    const bool live = u < units;
                    const float v = U::dot(w[r][it], live ? u : units - 1, sq, ss);
                    acc += live ? v : 0.0f;
                }
            y[r] = wave_sum(acc);
        }
        epi_fn(r0, y);
        r0 += step;
        if (r0 < r_end) request(r0);
    }
    stamp_fn(3);
    return true;
}

// Sum over each 32-lane half of the wavefront; every lane gets its half's total.
__device__ __forceinline__ float p_half_sum(float v) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    v += dpp_move<0x140>(v);
    v += dpp_move<0x142, 0xA>(v);
    const float lo = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 31));
    const float hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
    return (threadIdx.x & 32) ? hi : lo;
}

__global__ __launch_bounds__(PT) void k_decode_step(const PersistArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    // LDS: activation image | reduction scratch | attention states
    const int kmax = max(a.d_model, a.d_ffn);
    int8_t *sq = (int8_t *)smem;
    Q8Scale *ss = (Q8Scale *)(smem + ((skewed(kmax) + 255) & ~255));
    float *s_red = (float *)((uint8_t *)ss + (size_t)(kmax >> 5) * sizeof(Q8Scale));   // [PW * 2]
    float *s_att = s_red + 64;                                                           // [2 * PW][HD + 2] states, then the new token's k and v
    __shared__ int s_abort;

    const int tid0 = threadIdx.x;
    const int G = gridDim.x, g = blockIdx.x;
    const int D = a.d_model, F = a.d_ffn, NH = a.n_heads;
    const int S = G / NH;  // position splits per head in the attention phase (host: G % NH == 0, S divides HD)
    const int pos = *a.pos_ptr;
    const unsigned tbase = (*a.epoch_ptr & 0xFFFFFu) << 12;  // tag = epoch * 4096 + phase number (1 ..)
    const int spin = a.spin_limit;
    if (spin < 0) {  // the host asks for the time-out path (tests of its fallback): every workgroup leaves at once
        if (tid0 == 0 && g == 0) atomicOr(a.fail, 1u);
        return;
    }
    if (tid0 == 0) s_abort = 0;
    __syncthreads();

    bool ok = true;
    // returns true when the workgroup has to leave (some thread timed out)
    auto bail = [&]() -> bool {
        if (!ok) s_abort = 1;
        __syncthreads();
        if (s_abort) {
            if (tid0 == 0) atomicOr(a.fail, 1u);
            return true;
        }
        return false;
    };
    auto stamp = [&](int l, int ph) {
        if (a.prof && tid0 == 0) a.prof[((size_t)g * (a.n_layers + 1) + l) * PROF_SLOTS + ph] = wall_clock64();
    };
    const int d_units = D / UnitQ4K::ELEMS, f_units = F / UnitQ4K::ELEMS;
    const size_t d_rb = UnitQ4K::row_bytes(D), f_rb = UnitQ4K::row_bytes(F);
    const size_t layer_kv = (size_t)NH * a.max_pos * HD;

    for (int l = 0; l < a.n_layers; ++l) {
        const PersistLayer T = a.layers[l];
        LayerPtrs L;
        L.wq = global_ptr<uint8_t>(T.wq); L.wk = global_ptr<uint8_t>(T.wk); L.wv = global_ptr<uint8_t>(T.wv);
        L.wo = global_ptr<uint8_t>(T.wo); L.gate = global_ptr<uint8_t>(T.gate); L.up = global_ptr<uint8_t>(T.up);
        L.down = global_ptr<uint8_t>(T.down);
        L.attn_norm = global_ptr<float>(T.attn_norm); L.ffn_norm = global_ptr<float>(T.ffn_norm);
        const int par = l & 1;
        const unsigned t_in = tbase + (unsigned)(l * 6);  // tag of this layer's input (phase 6 of the previous layer)
        u64 *ha = a.x_ha + (size_t)par * D, *hb = a.x_hb + (size_t)par * D;
        u64 *ha_next = a.x_ha + (size_t)(par ^ 1) * D;
        u64 *xqkv = a.x_qkv + (size_t)par * 3 * D;
        u64 *xpart = a.x_part + (size_t)par * NH * S * (HD + 2);
        u64 *xatt = a.x_att + (size_t)par * D, *xact = a.x_act + (size_t)par * F;

        // ================= phase 1: RMSNorm + q/k/v
        stamp(l, 0);
        {
            PHASE_IDS
            auto st = [&](int k) __attribute__((always_inline)) { stamp(l, 0 + k); };
            constexpr int R = 6;  // rows per wavefront and round: 48 rows per workgroup at d_model 4096 on 256 CUs
            const int total = 3 * D, per_wg = (total + G - 1) / G;
            const int r_end = min(total, (g + 1) * per_wg);
            auto rows_fn = [&](int r0, const uint8_t *(&rows)[R]) __attribute__((always_inline)) {
#pragma unroll
                for (int j = 0; j < R; ++j) {
                    const int r = min(r0 + j, total - 1);
                    const u64 w = r < D ? T.wq : (r < 2 * D ? T.wk : T.wv);  // chosen as integers: the choice keeps the address space
                    rows[j] = global_ptr<uint8_t>(w + (u64)(r % D) * d_rb);
                }
            };
            auto stage_fn = [&]() __attribute__((always_inline)) -> bool {
                float4 xv[XD];
                if (l == 0) {
#pragma unroll
                    for (int i = 0; i < XD; ++i) {
                        const int c = tid + i * PT;
                        xv[i] = c < (D >> 2) ? ((const float4 *)a.h_in)[c] : make_float4(0.f, 0.f, 0.f, 0.f);
                    }
                } else poll_chunks<XD>(ha, tid, D >> 2, t_in, spin, ok, xv);
                if (bail()) return false;
                st(1);
                stage_activations<XD, true>(tid, xv, L.attn_norm, a.eps, D, sq, ss, s_red);
                return true;
            };
            auto epi_fn = [&](int r0, const float (&y)[R]) __attribute__((always_inline)) {
#pragma unroll
                for (int j = 0; j < R; ++j)
                    if (lane == 0 && r0 + j < r_end) publish(xqkv + r0 + j, y[j], t_in + 1);
            };
            if (!phase_rows<UnitQ4K, 1, R>(lane, g * per_wg + wave * R, PW * R, r_end, d_units, sq, ss, rows_fn, stage_fn, epi_fn, st))
                return;
        }
        // ================= phase 2: Rope, cache append, attention over this workgroup's share of the positions
        stamp(l, 4);
        if (g < NH * S) {
            PHASE_IDS
            const int head = g / S, split = g - head * S;
            const int hw = lane >> 5, hl = lane & 31;
            float *kh = a.k_cache + (size_t)l * layer_kv + (size_t)head * a.max_pos * HD;
            float *vh = a.v_cache + (size_t)l * layer_kv + (size_t)head * a.max_pos * HD;
            const int per = (pos + S - 1) / S;
            const int p0 = split * per, p1 = min(pos, p0 + per);
            // the cache rows of this wavefront are requested before anything is polled: half-wave slot = position
            constexpr int UNR = 4;
            typedef float vecf __attribute__((ext_vector_type(4)));
            vecf kv[UNR], vv[UNR];
            bool valid[UNR];
            auto fetch = [&](int base, vecf (&k4)[UNR], vecf (&v4)[UNR], bool (&vd)[UNR]) {
#pragma unroll
                for (int u = 0; u < UNR; ++u) {
                    const int p = base + 2 * u + hw;
                    vd[u] = p < p1;
                    const size_t off = (size_t)max(min(p, p1 - 1), 0) * HD + hl * 4;
                    k4[u] = __builtin_nontemporal_load((const vecf *)(kh + off));
                    v4[u] = __builtin_nontemporal_load((const vecf *)(vh + off));
                }
            };
            constexpr int STEP = PW * 2 * UNR;
            int base = p0 + wave * 2 * UNR;
            if (base < p1) fetch(base, kv, vv, valid);
            // q of this head (and the new k / v for the split that owns the new token), then Rope
            const int i0 = (hl & 15) * 4;
            const vecf cs = *(const vecf *)(a.cos_t + (size_t)pos * (HD / 2) + i0);
            const vecf sn = *(const vecf *)(a.sin_t + (size_t)pos * (HD / 2) + i0);
            auto rope = [&](vecf v) -> vecf {
                vecf other, r;
#pragma unroll
                for (int j = 0; j < 4; ++j) other[j] = __shfl_xor(v[j], 16, 64);
#pragma unroll
                for (int j = 0; j < 4; ++j) r[j] = hl < 16 ? v[j] * cs[j] - other[j] * sn[j] : other[j] * sn[j] + v[j] * cs[j];
                return r;
            };
            const bool owner = split == S - 1 && wave == 0;
            float *stash = s_att + 2 * PW * (HD + 2);  // the new token's k (after Rope) and v wait here for the walk to end
            vecf qv;
            {
                const u64 *qp = xqkv + head * HD + hl * 4;
                if (owner) {
                    const u64 *const p[12] = {qp, qp + 1, qp + 2, qp + 3, qp + D, qp + D + 1, qp + D + 2, qp + D + 3,
                                              qp + 2 * D, qp + 2 * D + 1, qp + 2 * D + 2, qp + 2 * D + 3};
                    float v[12];
                    poll_n<12>(p, t_in + 1, spin, ok, v);
                    qv = rope(vecf{v[0], v[1], v[2], v[3]});
                    const vecf kn = rope(vecf{v[4], v[5], v[6], v[7]});
                    if (hw == 0) {
                        *(vecf *)(stash + hl * 4) = kn;
                        *(vecf *)(stash + HD + hl * 4) = vecf{v[8], v[9], v[10], v[11]};
                    }
                } else {
                    const float4 q4 = poll4(qp, t_in + 1, spin, ok);
                    qv = rope(vecf{q4.x, q4.y, q4.z, q4.w});
                }
            }
            if (bail()) return;
            stamp(l, 5);
            float m_run = P_NEG_BIG, l_run = 0.0f;
            vecf o_run = vecf{0.f, 0.f, 0.f, 0.f};
            auto absorb = [&](const vecf (&k4)[UNR], const vecf (&v4)[UNR], const bool (&vd)[UNR]) {
                float s[UNR];
                float m_new = m_run;
#pragma unroll
                for (int u = 0; u < UNR; ++u) {
                    float d = qv[0] * k4[u][0] + qv[1] * k4[u][1] + qv[2] * k4[u][2] + qv[3] * k4[u][3];
                    d = p_half_sum(d) * a.scale;
                    s[u] = vd[u] ? d : P_NEG_BIG;
                    m_new = fmaxf(m_new, s[u]);
                }
                const float corr = expf(m_run - m_new);
                float lsum = l_run * corr;
                vecf o = o_run * corr;
#pragma unroll
                for (int u = 0; u < UNR; ++u) {
                    const float pw = vd[u] ? expf(s[u] - m_new) : 0.0f;
                    lsum += pw;
                    o += pw * v4[u];
                }
                m_run = m_new;
                l_run = lsum;
                o_run = o;
            };
            while (base < p1) {
                const int nb = base + STEP;
                vecf kn2[UNR], vn2[UNR];
                bool vd2[UNR];
                if (nb < p1) fetch(nb, kn2, vn2, vd2);
                absorb(kv, vv, valid);
                if (nb >= p1) break;
#pragma unroll
                for (int u = 0; u < UNR; ++u) { kv[u] = kn2[u]; vv[u] = vn2[u]; valid[u] = vd2[u]; }
                base = nb;
            }
            stamp(l, 6);
            if (owner) {  // the new token: append to the cache, attend to it from registers
                const vecf kn = *(const vecf *)(stash + hl * 4), vn = *(const vecf *)(stash + HD + hl * 4);
                if (hw == 0) {
                    *(vecf *)(kh + (size_t)pos * HD + hl * 4) = kn;
                    *(vecf *)(vh + (size_t)pos * HD + hl * 4) = vn;
                }
                vecf k4[UNR], v4[UNR];
                bool vd[UNR];
#pragma unroll
                for (int u = 0; u < UNR; ++u) { k4[u] = kn; v4[u] = vn; vd[u] = (u == 0) && (hw == 0); }
                absorb(k4, v4, vd);
            }
            stamp(l, 7);
            // merge the 2 * PW half-wave states
            const int slot = wave * 2 + hw;
            float *st = s_att + slot * (HD + 2);
            if (hl == 0) { st[HD] = m_run; st[HD + 1] = l_run; }
            *(vecf *)(st + hl * 4) = o_run;
            __syncthreads();
            if (tid < HD) {
                float m = P_NEG_BIG;
                for (int w = 0; w < 2 * PW; ++w) m = fmaxf(m, s_att[w * (HD + 2) + HD]);
                float lsum = 0.0f, o = 0.0f;
                for (int w = 0; w < 2 * PW; ++w) {
                    const float f = expf(s_att[w * (HD + 2) + HD] - m);
                    lsum += s_att[w * (HD + 2) + HD + 1] * f;
                    o += s_att[w * (HD + 2) + tid] * f;
                }
                u64 *dst = xpart + (size_t)(head * S + split) * (HD + 2);
                publish(dst + tid, o, t_in + 2);
                if (tid == 0) { publish(dst + HD, m, t_in + 2); publish(dst + HD + 1, lsum, t_in + 2); }
            }
        }
        // ================= phase 3: merge the splits; workgroup (head, part) owns HD / S dims of its head
        stamp(l, 8);
        if (g < NH * S) {
            PHASE_IDS
            const int head = g / S, part = g - head * S, dims = HD / S;
            // thread (s, j): split s, word j of {this workgroup's dims, m, l}; lands in LDS as [s][dims + 2]
            const int per_split = dims + 2;
            __syncthreads();  // phase 2's merge has read the states this overwrites
            if (tid < S * per_split) {
                const int sp = tid / per_split, j = tid - sp * per_split;
                const u64 *src = xpart + (size_t)(head * S + sp) * (HD + 2) + (j < dims ? part * dims + j : HD + (j - dims));
                s_att[tid] = poll(src, t_in + 2, spin, ok);
            }
            if (bail()) return;
            stamp(l, 9);
            if (tid < dims) {
                float m = P_NEG_BIG;
                for (int sp = 0; sp < S; ++sp) m = fmaxf(m, s_att[sp * per_split + dims]);
                float lsum = 0.0f, o = 0.0f;
                for (int sp = 0; sp < S; ++sp) {
                    const float f = expf(s_att[sp * per_split + dims] - m);
                    lsum += s_att[sp * per_split + dims + 1] * f;
                    o += s_att[sp * per_split + tid] * f;
                }
                publish(xatt + head * HD + part * dims + tid, o * (1.0f / lsum), t_in + 3);
            }
        }
        // ================= phase 4: o projection + residual
        stamp(l, 10);
        {
            PHASE_IDS
            auto st = [&](int k) __attribute__((always_inline)) { stamp(l, 10 + k); };
            constexpr int R = 2;
            const int per_wg = (D + G - 1) / G, r_end = min(D, (g + 1) * per_wg);
            u64 ru[R];  // the residual (published a whole layer ago) is requested with the weights, consumed after the dot
            auto rows_fn = [&](int r0, const uint8_t *(&rows)[R]) __attribute__((always_inline)) {
#pragma unroll
                for (int j = 0; j < R; ++j) {
                    const int r = min(r0 + j, D - 1);
                    ru[j] = l == 0 ? tagged(a.h_in[r], t_in) : __hip_atomic_load(ha + r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    rows[j] = L.wo + (size_t)r * d_rb;
                }
            };
            auto stage_fn = [&]() __attribute__((always_inline)) -> bool {
                float4 xv[XD];
                poll_chunks<XD>(xatt, tid, D >> 2, t_in + 3, spin, ok, xv);
                if (bail()) return false;
                st(1);
                stage_activations<XD, false>(tid, xv, nullptr, 0.0f, D, sq, ss, s_red);
                return true;
            };
            auto epi_fn = [&](int r0, const float (&y)[R]) __attribute__((always_inline)) {
#pragma unroll
                for (int j = 0; j < R; ++j)
                    if (lane == 0 && r0 + j < r_end) {
                        const float res = (unsigned)(ru[j] >> 32) == t_in ? __uint_as_float((unsigned)ru[j])
                                                                           : poll(ha + r0 + j, t_in, spin, ok);
                        publish(hb + r0 + j, res + y[j], t_in + 4);
                    }
            };
            if (!phase_rows<UnitQ4K, 1, R>(lane, g * per_wg + wave * R, PW * R, r_end, d_units, sq, ss, rows_fn, stage_fn, epi_fn, st))
                return;
        }
        // ================= phase 5: RMSNorm + gate / up + SiLU * Mul
        stamp(l, 14);
        {
            PHASE_IDS
            auto st = [&](int k) __attribute__((always_inline)) { stamp(l, 14 + k); };
            constexpr int NP = 6;  // (gate, up) row pairs per wavefront and round: 43 pairs per workgroup at d_ffn 11008
            const int per_wg = (F + G - 1) / G, r_end = min(F, (g + 1) * per_wg);
            auto rows_fn = [&](int r0, const uint8_t *(&rows)[2 * NP]) __attribute__((always_inline)) {
#pragma unroll
                for (int j = 0; j < NP; ++j) {
                    const int r = min(r0 + j * PW, F - 1);
                    rows[2 * j] = L.gate + (size_t)r * d_rb;
                    rows[2 * j + 1] = L.up + (size_t)r * d_rb;
                }
            };
            auto stage_fn = [&]() __attribute__((always_inline)) -> bool {
                float4 xv[XD];
                poll_chunks<XD>(hb, tid, D >> 2, t_in + 4, spin, ok, xv);
                if (bail()) return false;
                st(1);
                stage_activations<XD, true>(tid, xv, L.ffn_norm, a.eps, D, sq, ss, s_red);
                return true;
            };
            auto epi_fn = [&](int r0, const float (&y)[2 * NP]) __attribute__((always_inline)) {
#pragma unroll
                for (int j = 0; j < NP; ++j)
                    if (lane == 0 && r0 + j * PW < r_end) publish(xact + r0 + j * PW, p_silu(y[2 * j]) * y[2 * j + 1], t_in + 5);
            };
            if (!phase_rows<UnitQ4K, 1, 2 * NP>(lane, g * per_wg + wave, PW * NP, r_end, d_units, sq, ss, rows_fn, stage_fn, epi_fn, st))
                return;
        }
        // ================= phase 6: down projection + residual
        stamp(l, 18);
        {
            PHASE_IDS
            auto st = [&](int k) __attribute__((always_inline)) { stamp(l, 18 + k); };
            constexpr int R = 2;
            const int per_wg = (D + G - 1) / G, r_end = min(D, (g + 1) * per_wg);
            u64 ru[R];
            auto rows_fn = [&](int r0, const uint8_t *(&rows)[R]) __attribute__((always_inline)) {
#pragma unroll
                for (int j = 0; j < R; ++j) {
                    const int r = min(r0 + j, D - 1);
                    ru[j] = __hip_atomic_load(hb + r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    rows[j] = L.down + (size_t)r * f_rb;
                }
            };
            auto stage_fn = [&]() __attribute__((always_inline)) -> bool {
                float4 xv[XF];
                poll_chunks<XF>(xact, tid, F >> 2, t_in + 5, spin, ok, xv);
                if (bail()) return false;
                st(1);
                stage_activations<XF, false>(tid, xv, nullptr, 0.0f, F, sq, ss, s_red);
                return true;
            };
            auto epi_fn = [&](int r0, const float (&y)[R]) __attribute__((always_inline)) {
#pragma unroll
                for (int j = 0; j < R; ++j)
                    if (lane == 0 && r0 + j < r_end) {
                        const float res = (unsigned)(ru[j] >> 32) == t_in + 4 ? __uint_as_float((unsigned)ru[j])
                                                                               : poll(hb + r0 + j, t_in + 4, spin, ok);
                        publish(ha_next + r0 + j, res + y[j], t_in + 6);
                    }
            };
            // up to four steps per row (d_ffn <= 16384)
            if (!phase_rows<UnitQ4K, 4, R>(lane, g * per_wg + wave * R, PW * R, r_end, f_units, sq, ss, rows_fn, stage_fn, epi_fn, st))
                return;
        }
    }

    // ================= final norm, head, argmax
    {
        const unsigned t_in = tbase + (unsigned)(a.n_layers * 6);
        const u64 *ha = a.x_ha + (size_t)(a.n_layers & 1) * D;
        stamp(a.n_layers, 0);
        PHASE_IDS
        auto st = [&](int k) __attribute__((always_inline)) { stamp(a.n_layers, k); };
        constexpr int R = 4;
        const int V = a.vocab, per_wg = (V + G - 1) / G, r_end = min(V, (g + 1) * per_wg);
        const size_t h_rb = a.head_is_q6k ? UnitQ6K::row_bytes(D) : d_rb;
        float best = P_NEG_BIG;
        unsigned bi = 0xFFFFFFFFu;
        auto rows_fn = [&](int r0, const uint8_t *(&rows)[R]) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < R; ++j) rows[j] = a.head + (size_t)min(r0 + j, V - 1) * h_rb;
        };
        auto stage_fn = [&]() __attribute__((always_inline)) -> bool {
            float4 xv[XD];
            poll_chunks<XD>(ha, tid, D >> 2, t_in, spin, ok, xv);
            if (bail()) return false;
            st(1);
            stage_activations<XD, true>(tid, xv, a.out_norm, a.eps, D, sq, ss, s_red);
            return true;
        };
        auto epi_fn = [&](int r0, const float (&y)[R]) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < R; ++j)
                if (r0 + j < r_end) {
                    if (lane == 0) a.logits[r0 + j] = y[j];
                    if (y[j] > best) { best = y[j]; bi = (unsigned)(r0 + j); }  // ascending rows, strict >: first maximum
                }
        };
        const int first = g * per_wg + wave * R, step = PW * R;
        bool stay;
        if (!a.head_is_q6k) stay = phase_rows<UnitQ4K, 1, R>(lane, first, step, r_end, d_units, sq, ss, rows_fn, stage_fn, epi_fn, st);
        else stay = phase_rows<UnitQ6K, 2, R>(lane, first, step, r_end, D / UnitQ6K::ELEMS, sq, ss, rows_fn, stage_fn, epi_fn, st);
        if (!stay) return;
        stamp(a.n_layers, 4);
        // the workgroup's first maximum, then the grid's (workgroup 0)
        float *sv = s_red;
        unsigned *si = (unsigned *)(s_red + 32);
        __syncthreads();
        if (lane == 0) { sv[wave] = best; si[wave] = bi; }
        __syncthreads();
        if (tid == 0) {
            for (int i = 1; i < PW; ++i)
                if (sv[i] > best || (sv[i] == best && si[i] < bi)) { best = sv[i]; bi = si[i]; }
            publish(a.x_best + 2 * g, best, t_in + 1);
            publish(a.x_best + 2 * g + 1, __uint_as_float(bi), t_in + 1);
        }
        if (g == 0) {
            float v = P_NEG_BIG;
            unsigned idx = 0xFFFFFFFFu;
            for (int w = tid; w < G; w += PT) {
                const float bv = poll(a.x_best + 2 * w, t_in + 1, spin, ok);
                const unsigned bx = __float_as_uint(poll(a.x_best + 2 * w + 1, t_in + 1, spin, ok));
                if (bv > v || (bv == v && bx < idx)) { v = bv; idx = bx; }
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const float ov = __shfl_xor(v, off, 64);
                const unsigned oi = __shfl_xor(idx, off, 64);
                if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
            }
            __syncthreads();
            if (lane == 0) { sv[wave] = v; si[wave] = idx; }
            if (bail()) return;
            if (tid == 0) {
                for (int i = 1; i < PW; ++i)
                    if (sv[i] > v || (sv[i] == v && si[i] < idx)) { v = sv[i]; idx = si[i]; }
                *a.next_tok = idx == 0xFFFFFFFFu ? 0u : idx;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------- host side

size_t persist_lds_bytes(int d_model, int d_ffn) {
    const int kmax = d_model > d_ffn ? d_model : d_ffn;
    size_t b = ((size_t)(kmax + ((kmax >> 8) << 4)) + 255) & ~(size_t)255;
    b += (size_t)(kmax >> 5) * sizeof(Q8Scale);
    b += 64 * sizeof(float);
    b += (size_t)(2 * PW + 2) * (HD + 2) * sizeof(float);
    // more than half of the CU's LDS, so that no two workgroups share a compute unit
    return b > 96 * 1024 ? b : 96 * 1024;
}

int launch_decode_step(candy_hip_device *dev, const PersistArgs &a) {
    const size_t lds = persist_lds_bytes(a.d_model, a.d_ffn);
    CANDY_HIP_TRY(hipFuncSetAttribute((const void *)k_decode_step, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(k_decode_step, dim3((unsigned)dev->num_cus), dim3(PT), lds, dev->stream, a);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

}  // namespace candy
