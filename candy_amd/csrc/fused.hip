// Decode-step matvecs with the neighbouring f32 stages folded in, so a Llama block is five
// launches instead of ten and no activation makes a round trip through HBM between them:
//   prologue RMS:   RMSNorm (reduce.go:3071-3092) of the f32 input + Q8_0 quantization
//                   (quantized.cu:3521-3558), recomputed by every workgroup under the shadow of
//                   its own weight loads (the weights dominate the time; the input is 16 KB);
//   epilogue PAIR:  the workgroup owns 32 consecutive rows of BOTH gate and up, so it can apply
//                   SiLU (unary.go:3353-3366) * Mul and quantize the 32 results to one Q8_0 block
//                   for the down projection;
//   epilogue RES:   residual Add (backend.go:21) on the output.
// The contraction itself is the batch-1 kernel of matvec.hip (same units, same exact load
// counting: inputs first, then every weight load, nothing branches around a memory operation).
#include <cstdlib>
#include <type_traits>

#include "blocks.h"
#include "internal.h"
#include "units.h"
#include "formats_more.h"

namespace candy {

enum { PRO_Q8 = 0, PRO_RMS = 1 };
enum { EPI_PLAIN = 0, EPI_PAIR = 1 };

// What a wavefront's first loads need - the input and the weights' addresses - are the kernel's plain leading
// arguments (14 dwords: they arrive in registers with the wavefront); the rest comes through the argument block
// while those loads are in flight.
struct FusedHead {
    const void *in0, *in1;  // PRO_Q8: planar Q8_0 activations (int8 quants, Q8Scale); PRO_RMS: f32 input row, RMSNorm weight
    const uint8_t *W[3];    // PLAIN: up to 3 weights as one run of rows; PAIR: W[0] = gate, W[1] = up (same shape)
    int K;
    int e[3];               // PLAIN: each weight's END ROW in the run; PAIR: e[0] = rows of gate (and of up)
};
struct FusedRest {
    float *y[3];
    const float *res[3];
    float eps;
    // PAIR epilogue output: planar Q8_0 of silu(gate.x) * (up.x)
    int8_t *oq;
    Q8Scale *os;
    // PAIR workgroups that own less than a 32-value block: their f32 results and one counter per block
    float *pair_act;
    unsigned *pair_tickets;
};
struct FusedArgs {
    FusedHead h;
    FusedRest r;
    int n;      // host side only: weights in the launch
    int N[3];   // host side only: rows of each weight
};

__device__ __forceinline__ float silu_exact(float x) { return x / (1.0f + expf(-x)); }

template <class U, int ITER, int R, int WAVES, int PRO, int EPI>
CANDY_KERNEL(WAVES * 64, ((EPI == EPI_PAIR && ITER == 1) ? 4 : 1), 4) void k_matvec_fused(
    const void *__restrict__ in0, const void *__restrict__ in1, const uint8_t *__restrict__ W0, const uint8_t *__restrict__ W1,
    const uint8_t *__restrict__ W2, int K, int e0, int e1, int e2, const FusedRest a) {
    constexpr int T = WAVES * 64;
    constexpr int CAP = ITER * 64 * U::ELEMS;       // activation values the LDS image is sized for
    constexpr int AQ = (CAP / 16 + T - 1) / T;      // PRO_Q8: 16-byte chunks of quants per thread
    constexpr int AS = (CAP / 32 + T - 1) / T;      // PRO_Q8: 8-byte scales per thread
    constexpr int XF = (CAP / 4 + T - 1) / T;       // PRO_RMS: float4 of input per thread
    constexpr int NW = EPI == EPI_PAIR ? 2 : 1;     // weights contracted per wavefront
    extern __shared__ __align__(16) uint8_t smem[];
    int8_t *sq = (int8_t *)smem;
    constexpr int QBYTES = (PRO == PRO_Q8 ? AQ * T * 16 : XF * T * 4);
    Q8Scale *ss = (Q8Scale *)(smem + QBYTES + ((QBYTES >> 8) << 4));
    __shared__ float s_red[WAVES];
    __shared__ float s_act[32];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int units = K / U::ELEMS;
    const size_t rb = U::row_bytes(K);

    // PLAIN: the (up to three) weights form one run of rows, wg_end holding each weight's END ROW in that run, and
    // a workgroup takes R * WAVES consecutive rows of the run wherever they fall, so that the run divides over the
    // CUs evenly whatever the single row counts are (6144 rows of an 8B q/k/v = 256 workgroups of 24).  A wavefront
    // resolves each of its rows to a weight and a row of that weight (wavefront-uniform).  PAIR: blockIdx is the
    // group of S row pairs.
    const int wg = blockIdx.x;
    const int N = e0;  // PAIR: both weights have N rows

    // ---- inputs first (oldest entries of the in-order return queue)
    uint4 aq[AQ];
    uint2 as[AS];
    float4 xv[XF], av[XF];
    if (PRO == PRO_Q8) {
        const int qchunks = K >> 4, sblocks = K >> 5;
#pragma unroll
        for (int i = 0; i < AQ; ++i) aq[i] = ((const uint4 *)in0)[min(tid + i * T, qchunks - 1)];
#pragma unroll
        for (int i = 0; i < AS; ++i) as[i] = ((const uint2 *)in1)[min(tid + i * T, sblocks - 1)];
    } else {
        const int n4 = K >> 2;
#pragma unroll
        for (int i = 0; i < XF; ++i) {
            const int c = min(tid + i * T, n4 - 1);
            xv[i] = ((const float4 *)in0)[c];
            av[i] = ((const float4 *)in1)[c];
        }
    }

    // ---- every weight load of the wavefront
    const int row0 = (wg * WAVES + wave) * R;
    typename U::W w[NW][R][ITER];
    int job[R], jrow[R];  // PLAIN: weight and row within it, -1 past the end of the run
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int g = row0 + r;
        const int ji = (int)(g >= e0) + (int)(g >= e1);
        job[r] = g < e2 ? ji : -1;
        jrow[r] = g < e2 ? g - (ji == 0 ? 0 : ji == 1 ? e0 : e1) : 0;
    }
#pragma unroll
    for (int m = 0; m < NW; ++m) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint8_t *row = EPI == EPI_PAIR ? (m == 0 ? W0 : W1) + (size_t)min(row0 + r, N - 1) * rb
                                                 : (job[r] <= 0 ? W0 : job[r] == 1 ? W1 : W2) + (size_t)jrow[r] * rb;
#pragma unroll
            for (int it = 0; it < ITER; ++it) U::load(row, min(it * 64 + lane, units - 1), w[m][r][it]);
        }
    }

    // PLAIN: where each row goes, and the residual it is added to, requested now: asked for after the reduction it
    // would be a memory round trip (two, with the output pointer picked out of the argument block by a vector
    // index) at the very end of every wavefront.  Rows without a residual read their own output slot (valid
    // memory, value unused), so that nothing branches around a load.
    float *yp[R];
    float rv[R];
    bool has_res[R];
    if (EPI == EPI_PLAIN) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int j = job[r];
            yp[r] = (j <= 0 ? a.y[0] : j == 1 ? a.y[1] : a.y[2]) + jrow[r];  // may alias the residual (h += W.x)
            const float *rp = j <= 0 ? a.res[0] : j == 1 ? a.res[1] : a.res[2];
            has_res[r] = rp != nullptr;
            rv[r] = *(has_res[r] ? rp + jrow[r] : yp[r]);
        }
    }

    // ---- park the quantized activations in LDS
    if (PRO == PRO_Q8) {
#pragma unroll
        for (int i = 0; i < AQ; ++i) {
            const int c = tid + i * T;
            ((uint4 *)sq)[c + (c >> 4)] = aq[i];
        }
#pragma unroll
        for (int i = 0; i < AS; ++i) ((uint2 *)ss)[tid + i * T] = as[i];
    } else {
        const int n4 = K >> 2;
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < XF; ++i) {
            const float4 v = xv[i];
            const float t = v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
            s += (tid + i * T < n4) ? t : 0.0f;
        }
        s = wave_sum(s);
        if (lane == 0) s_red[wave] = s;
        __syncthreads();
        float tot = 0.0f;
#pragma unroll
        for (int i = 0; i < WAVES; ++i) tot += s_red[i];
        const float mean = tot / (float)K;
        const float scale = rms_inv_sqrt(mean + a.eps);
#pragma unroll
        for (int i = 0; i < XF; ++i) {
            const int c = tid + i * T;
            const float4 v = xv[i], al = av[i];
            const float4 xn = make_float4(scale * v.x * al.x, scale * v.y * al.y, scale * v.z * al.z, scale * v.w * al.w);
            __half h;
            int bsum;
            const uint32_t packed = quantize_q8_lane4(xn, h, bsum);
            *(uint32_t *)(sq + skewed(4 * c)) = packed;  // c past the row lands in the padding
            if ((c & 7) == 0) {
                Q8Scale sc;
                sc.d = __half2float(h);
                sc.bsum = bsum;
                ss[c >> 3] = sc;
            }
        }
    }
    __syncthreads();

    // ---- contraction
    float acc[NW][R];
#pragma unroll
    for (int m = 0; m < NW; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[m][r] = 0.0f;
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        const int u = it * 64 + lane;
        const bool live = u < units;
        const int uc = live ? u : units - 1;
#pragma unroll
        for (int m = 0; m < NW; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const float v = U::dot(w[m][r][it], uc, sq, ss);
                acc[m][r] += live ? v : 0.0f;
            }
    }

    if (EPI == EPI_PLAIN) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float v = wave_sum(acc[0][r]);
            if (lane == 0 && job[r] >= 0) *yp[r] = has_res[r] ? rv[r] + v : v;
        }
    } else {
        // A PAIR workgroup owns S = 32, 16 or 8 consecutive outputs: a whole Q8_0 block, or a part of one.  Parts
        // exist so that the grid divides evenly over the CUs (344 whole blocks of a 11008-wide layer leave 88 CUs
        // with twice the bytes of the others).  A part leaves its f32 values in pair_act and takes a ticket of its
        // block; whoever draws the last ticket quantizes the block from pair_act (the same 32 values whichever
        // workgroup that is, so the result does not depend on the order) and puts the counter back to zero.
        constexpr int S = R * WAVES;
        static_assert(EPI != EPI_PAIR || S == 32 || S == 16 || S == 8 || S == 4, "a PAIR workgroup owns a 32-value block or a part");
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float g = wave_sum(acc[0][r]), u = wave_sum(acc[1][r]);
            if (lane == 0) s_act[wave * R + r] = silu_exact(g) * u;
        }
        __syncthreads();
        if (wave == 0) {
            const int blk = (wg * S) >> 5;  // N % 32 == 0
            float mine;
            if constexpr (S == 32) {
                mine = s_act[lane & 31];
            } else {
                if (lane < S) __hip_atomic_store(a.pair_act + wg * S + lane, s_act[lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                // The values are out before the ticket is drawn: agent-scope atomic stores write through to where
                // every XCD sees them, and the store counter reaches zero when they have arrived.  (A release fence
                // would also write the whole L2 back and an acquire fence invalidate it: 17 us per launch, measured.)
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                unsigned old = 0;
                if (lane == 0) old = __hip_atomic_fetch_add(a.pair_tickets + blk, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                old = (unsigned)__builtin_amdgcn_readfirstlane((int)old);
                if (old != 32 / S - 1) return;  // a later workgroup finishes the block
                asm volatile("" ::: "memory");  // agent-scope atomic loads below: they do not hit a stale cache line
                mine = __hip_atomic_load(a.pair_act + blk * 32 + (lane & 31), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (lane == 0) __hip_atomic_store(a.pair_tickets + blk, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            __half h;
            int bsum;
            const int q = quantize_q8_lane1(mine, h, bsum);
            if (lane < 32) a.oq[(size_t)blk * 32 + lane] = (int8_t)q;
            if (lane == 0) {
                Q8Scale sc;
                sc.d = __half2float(h);
                sc.bsum = bsum;
                a.os[blk] = sc;
            }
        }
    }
}

template <class U, int ITER, int R, int WAVES, int PRO, int EPI>
static int launch_fused_cfg(candy_hip_device *dev, FusedArgs a) {
    constexpr int T = WAVES * 64, CAP = ITER * 64 * U::ELEMS;
    constexpr int AQ = (CAP / 16 + T - 1) / T, AS = (CAP / 32 + T - 1) / T, XF = (CAP / 4 + T - 1) / T;
    constexpr size_t QBYTES = PRO == PRO_Q8 ? (size_t)AQ * T * 16 : (size_t)XF * T * 4;
    constexpr size_t SBYTES = PRO == PRO_Q8 ? (size_t)AS * T * 8 : ((size_t)XF * T / 8 + 1) * 8;
    constexpr size_t smem = QBYTES + ((QBYTES >> 8) << 4) + SBYTES;
    static_assert(smem <= 60 * 1024, "LDS image too large");
    const int rows_per_wg = R * WAVES;
    int total = 0;
    if (EPI == EPI_PAIR) {
        total = a.N[0] / rows_per_wg;
        a.h.e[0] = a.h.e[1] = a.h.e[2] = a.N[0];
    } else {
        int rows = 0;
        for (int i = 0; i < 3; ++i) {
            if (i < a.n) rows += a.N[i];
            a.h.e[i] = rows;  // end row in the run; unused slots end where the last real one does
        }
        total = (rows + rows_per_wg - 1) / rows_per_wg;
    }
    hipLaunchKernelGGL((k_matvec_fused<U, ITER, R, WAVES, PRO, EPI>), dim3((unsigned)total), dim3(T), smem, dev->stream,
                       a.h.in0, a.h.in1, a.h.W[0], a.h.W[1], a.h.W[2], a.h.K, a.h.e[0], a.h.e[1], a.h.e[2], a.r);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

// Rows per PAIR workgroup, out of hi, hi/2, ... lo: the largest that leaves the fullest CU the fewest rows.  A
// kernel whose workgroups all start at once lasts as long as its fullest CU streams (about 26 bytes per nanosecond
// each), so 1.34 workgroups per CU cost as much as 2.  Measured on the 7B decode step (d_ffn 11008): 32 rows 1.914,
// 16 rows (16 wavefronts x 1) 1.859, 8 rows (8 x 1) 1.855 ms per token; 4 rows 1.960; with four rows per wavefront
// the 16-row shape is slower than whole blocks (2.036).  d_ffn 14336: 32 rows 1.983, 8 rows 1.957.  The same choice
// for the plain RMSNorm-prologue kernel (16 or 8 rows) did not pay: 8 rows lose more to the repeated prologue than
// the even split wins (24-row workgroups over the weights' rows as one run do).  `forced` (the fused.pair_rows
// option) overrides the choice for comparison runs.
static int balanced_rows(int rows, int cus, int hi, int lo, int forced) {
    for (int s = hi; s >= lo; s >>= 1)
        if (forced == s) return s;
    int best = hi;
    long best_cost = -1;
    for (int s = hi; s >= lo; s >>= 1) {
        const long wgs = (rows + s - 1) / s, cost = (wgs + cus - 1) / cus * s;
        if (best_cost < 0 || cost < best_cost) { best = s; best_cost = cost; }
    }
    return best;
}

// Tile shapes: PLAIN keeps the batch-1 kernel's one row per wavefront when the input is already
// quantized; with the RMSNorm prologue a workgroup takes 16 rows so that the (redundant) prologue
// is amortised; PAIR is 8 wavefronts x 4 rows of each of the two weights (a whole 32-value block), or
// 16 x 1 / 8 x 1 (half a block, a quarter) where that divides the rows more evenly over the CUs and the caller
// has given the scratch the parts need.
template <class U, int ITER>
static int launch_fused_iter(candy_hip_device *dev, const FusedArgs &a, int pro, int epi) {
    // Q5_K holds 80 bytes of registers per unit: one row (pair) per wavefront, or two with the RMSNorm prologue
    if constexpr (sizeof(typename U::W) > 48) {
        if (epi == EPI_PAIR) {
            if constexpr (ITER <= 2) {
                if (pro != PRO_RMS || !a.r.pair_act || !a.r.pair_tickets) return CANDY_HIP_ERR_UNSUPPORTED;
                if (balanced_rows(a.N[0], dev->num_cus, 16, 8, dev->opt.pair_rows) == 8)
                    return launch_fused_cfg<U, ITER, 1, 8, PRO_RMS, EPI_PAIR>(dev, a);
                return launch_fused_cfg<U, ITER, 1, 16, PRO_RMS, EPI_PAIR>(dev, a);
            } else {
                return CANDY_HIP_ERR_UNSUPPORTED;
            }
        }
        if (pro == PRO_RMS) {
            if constexpr (ITER <= 2) return launch_fused_cfg<U, ITER, 2, 8, PRO_RMS, EPI_PLAIN>(dev, a);
            else return CANDY_HIP_ERR_UNSUPPORTED;
        }
        return launch_fused_cfg<U, ITER, 1, 4, PRO_Q8, EPI_PLAIN>(dev, a);
    } else {
        if (epi == EPI_PAIR) {
            if constexpr (ITER <= 2) {  // two weights x 4 rows x ITER units must stay in registers
                if (pro != PRO_RMS) return launch_fused_cfg<U, ITER, 4, 8, PRO_Q8, EPI_PAIR>(dev, a);
                const int s = a.r.pair_act && a.r.pair_tickets ? balanced_rows(a.N[0], dev->num_cus, 32, 8, dev->opt.pair_rows) : 32;
                if (s == 16) return launch_fused_cfg<U, ITER, 1, 16, PRO_RMS, EPI_PAIR>(dev, a);
                if (s == 8) return launch_fused_cfg<U, ITER, 1, 8, PRO_RMS, EPI_PAIR>(dev, a);
                return launch_fused_cfg<U, ITER, 4, 8, PRO_RMS, EPI_PAIR>(dev, a);
            } else {
                return CANDY_HIP_ERR_UNSUPPORTED;
            }
        }
        if (pro == PRO_RMS) {
            if constexpr (ITER <= 2) {
                // 16 rows per workgroup (4 x 4), or 24 (8 wavefronts x 3) where that leaves the fullest CU fewer rows
                int rows = 0;
                for (int i = 0; i < a.n; ++i) rows += a.N[i];
                const int cus = dev->num_cus;
                const long c16 = (long)((rows + 15) / 16 + cus - 1) / cus * 16, c24 = (long)((rows + 23) / 24 + cus - 1) / cus * 24;
                const int forced = dev->opt.rms_rows;  // comparison runs
                if (forced ? forced == 24 : c24 < c16) return launch_fused_cfg<U, ITER, 3, 8, PRO_RMS, EPI_PLAIN>(dev, a);
                return launch_fused_cfg<U, ITER, 4, 4, PRO_RMS, EPI_PLAIN>(dev, a);
            } else {
                return launch_fused_cfg<U, ITER, 2, 4, PRO_RMS, EPI_PLAIN>(dev, a);
            }
        }
        return launch_fused_cfg<U, ITER, 1, 4, PRO_Q8, EPI_PLAIN>(dev, a);
    }
}

template <class U>
static int launch_fused_fmt(candy_hip_device *dev, const FusedArgs &a, int pro, int epi) {
    const int iter = (a.h.K / U::ELEMS + 63) / 64;
    switch (iter) {
    case 1: return launch_fused_iter<U, 1>(dev, a, pro, epi);
    case 2: return launch_fused_iter<U, 2>(dev, a, pro, epi);
    case 3: return launch_fused_iter<U, 3>(dev, a, pro, epi);
    case 4: return launch_fused_iter<U, 4>(dev, a, pro, epi);
    default: return CANDY_HIP_ERR_UNSUPPORTED;
    }
}

// Returns CANDY_HIP_ERR_UNSUPPORTED (without setting the error text) when no instantiation covers
// the request; the caller then runs the unfused sequence.
int launch_matvec_fused(candy_hip_device *dev, const FusedLaunch &L) {
    const int n = L.n;
    if (n < 1 || n > 3) return CANDY_HIP_ERR_UNSUPPORTED;
    const candy_hip_qtensor *w0 = L.w[0];
    for (int i = 1; i < n; ++i)
        if (L.w[i]->fmt != w0->fmt || L.w[i]->cols != w0->cols) return CANDY_HIP_ERR_UNSUPPORTED;
    const int pro = L.x ? PRO_RMS : PRO_Q8, epi = L.pair ? EPI_PAIR : EPI_PLAIN;
    if (L.pair && (n != 2 || L.w[0]->rows != L.w[1]->rows || w0->rows % 32 != 0)) return CANDY_HIP_ERR_UNSUPPORTED;
    if (w0->cols > 0x7FFFFFFF) return CANDY_HIP_ERR_UNSUPPORTED;
    FusedArgs a{};
    a.n = n;
    for (int i = 0; i < 3; ++i) {
        const int j = i < n ? i : n - 1;  // unused slots repeat the last weight: no row resolves to them
        if (L.w[j]->rows > 0x7FFFFFFF) return CANDY_HIP_ERR_UNSUPPORTED;
        a.h.W[i] = (const uint8_t *)L.w[j]->data;
        a.r.y[i] = L.y[j];
        a.r.res[i] = L.res[j];
        a.N[i] = i < n ? (int)L.w[i]->rows : 0;
    }
    if (L.x) { a.h.in0 = L.x; a.h.in1 = L.alpha; }
    else { a.h.in0 = L.xq; a.h.in1 = L.xs; }
    a.r.eps = L.eps; a.r.oq = L.oq; a.r.os = L.os;
    a.r.pair_act = L.pair_act; a.r.pair_tickets = L.pair_tickets;
    a.h.K = (int)w0->cols;
    switch (w0->fmt) {
    case CANDY_HIP_Q4_K: return launch_fused_fmt<UnitQ4K>(dev, a, pro, epi);
    case CANDY_HIP_Q8_0: return launch_fused_fmt<UnitQ8_0>(dev, a, pro, epi);
    case CANDY_HIP_Q4_0: return launch_fused_fmt<UnitQ4_0<false>>(dev, a, pro, epi);
    case CANDY_HIP_Q4_0_GGML: return launch_fused_fmt<UnitQ4_0<true>>(dev, a, pro, epi);
    case CANDY_HIP_Q6_K: return launch_fused_fmt<UnitQ6K>(dev, a, pro, epi);
    case CANDY_HIP_Q5_K: return launch_fused_fmt<UnitQ5K>(dev, a, pro, epi);
    default: return CANDY_HIP_ERR_UNSUPPORTED;
    }
}

}  // namespace candy
