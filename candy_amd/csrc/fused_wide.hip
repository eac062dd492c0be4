// Decode-step matvecs of the big Q4_K shapes as ONE workgroup per compute unit.
//
// The fused kernels of fused.hip give every workgroup 16 or 32 rows and let each of them repeat the prologue
// (RMSNorm + Q8_0 quantization of the hidden state: 32 KB from L2, a reduction, a barrier).  On a 7B layer that is
// 688 prologues for gate/up and 768 for q/k/v, 2 us of each launch, and row counts that do not divide by the CUs
// leave some CUs a third more bytes than others.  Here the grid is a multiple of the CU count, every workgroup
// takes an equal share of the rows (to within one row) wherever they fall, its 16 (or 8) wavefronts walk that
// share round-robin with every weight load in flight before the first dot, and the prologue runs once per CU.
//   prologue RMS:    RMSNorm (reduce.go:3071-3092) + Q8_0 quantization (quantized.cu:3521-3558) of the f32 input
//   prologue QUANT:  Q8_0 quantization of the f32 input as it is (the whole f32-in -> f32-out QMatMul of one row
//                    as one launch: the same quants and scales as the quantize kernel, hence the same result)
//   epilogue PLAIN:  y = W.x (+ residual), up to three weights as one run of rows
//   epilogue PAIR:   silu(gate.x) * (up.x) quantized to planar Q8_0 for the down projection; a 32-value block
//                    whose rows belong to two workgroups is quantized by whichever of them finishes last
// Contraction and units are those of the batch-1 kernel (matvec.hip, units.h): same integer dots, same order of
// additions per row, so the results are the bits the narrower kernels give.
#include <algorithm>

#include "blocks.h"
#include "internal.h"
#include "units.h"

namespace candy {

enum { WPRO_RMS = 0, WPRO_QUANT = 1 };
enum { WEPI_PLAIN = 0, WEPI_PAIR = 1 };

// What the first loads of a wavefront need - the prologue's input and the weights' addresses - are the kernel's plain
// leading arguments (14 dwords: they arrive in registers with the wavefront); the rest comes through the argument
// block while those loads are in flight.
struct WideHead {
    const float *x, *alpha;  // prologue input and (RMS) the norm weight
    const uint8_t *W[3];     // PLAIN: up to 3 weights as one run of rows; PAIR: W[0] gate, W[1] up
    int per_rem;             // rows of the run (PLAIN) or row pairs (PAIR) per workgroup | (the remainder << 16)
    int K;
    int e0, e1;              // PLAIN: END ROW of the first and second weight in the run
};
struct WideRest {
    float *y[3];
    const float *res[3];
    float eps;
    // PAIR epilogue
    int8_t *oq;
    Q8Scale *os;
    float *pair_act;         // total floats of scratch
    unsigned *pair_tickets;  // total / 32 counters, zero before and after every launch
};
struct WideArgs {
    WideHead h;
    WideRest r;
};

__device__ __forceinline__ float wide_silu(float x) { return x / (1.0f + expf(-x)); }

// `total` items dealt to G workgroups as evenly as they go: the first `rem` = total % G workgroups take `per` + 1 =
// total / G + 1 items, the others `per`.  The host passes per and rem (packed: per | rem << 16), so that a workgroup
// finds its share with a multiply and an add - a 64-bit division here was 350 scalar instructions in front of the
// first load of every wavefront.
__device__ __forceinline__ int wide_start(int g, int per, int rem) { return g * per + min(g, rem); }
// How many workgroups hold a part of the 32-item block that starts at `first`, seen from workgroup g, which holds
// one (shares are at least 8 items, so at most four boundaries between workgroups fall inside the block, none
// further than three workgroups from g).
__device__ __forceinline__ int wide_sharers(int first, int g, int G, int per, int rem) {
    int n = 1;
#pragma unroll
    for (int d = -3; d <= 4; ++d) {
        const int b = g + d;  // the boundary between workgroups b - 1 and b
        const int at = wide_start(b, per, rem);
        n += (b >= 1 && b <= G - 1 && at > first && at < first + 32) ? 1 : 0;
    }
    return n;
}

// Two workgroups of 8 wavefronts (or one of 16) per CU are four wavefronts per SIMD: 128 registers each.  The shapes
// that hold up to eight rows of weights per lane are held to that (gate / up with four pairs per wavefront came to
// 130 registers without it, one workgroup per CU at a time and two rounds: 22.5 us per launch on a 2 x 14336 x 4096
// pair); the one-workgroup-per-CU shape with sixteen rows per lane keeps its 226.
template <class U, int ITER, int R, int WAVES, int PRO, int EPI, int SLOTS = R>
CANDY_KERNEL(WAVES * 64, ((EPI == WEPI_PAIR ? 2 : 1) * SLOTS * ITER <= 8 ? 4 : 2), 4)
void k_matvec_wide(const float *__restrict__ x, const float *__restrict__ alpha, const uint8_t *__restrict__ W0,
                   const uint8_t *__restrict__ W1, const uint8_t *__restrict__ W2, int per_rem, int K, int e0, int e1,
                   const WideRest a) {
    constexpr int T = WAVES * 64;
    constexpr int CAP = ITER * 64 * U::ELEMS;   // activation values the LDS image is sized for
    constexpr int XF = (CAP / 4 + T - 1) / T;   // float4 of prologue input per thread
    constexpr int NW = EPI == WEPI_PAIR ? 2 : 1;
    extern __shared__ __align__(16) uint8_t smem[];
    int8_t *sq = (int8_t *)smem;
    constexpr int QBYTES = XF * T * 4;
    Q8Scale *ss = (Q8Scale *)(smem + QBYTES + ((QBYTES >> 8) << 4));
    __shared__ float s_red[WAVES];
    __shared__ float s_act[R * WAVES];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int units = K / U::ELEMS;
    const size_t rb = U::row_bytes(K);
    const int G = gridDim.x;
    const int per = per_rem & 0xFFFF, rem = per_rem >> 16;
    const int start = wide_start(blockIdx.x, per, rem), end = wide_start(blockIdx.x + 1, per, rem);
    const int n4 = K >> 2;

    // ---- prologue inputs first (they return first)
    float4 xv[XF], av[XF];
#pragma unroll
    for (int i = 0; i < XF; ++i) {
        const int c = min(tid + i * T, n4 - 1);
        xv[i] = ((const float4 *)x)[c];
        if (PRO == WPRO_RMS) av[i] = ((const float4 *)alpha)[c];
    }

    // ---- every weight load of the wavefront: items start + wave + WAVES * r
    typename U::W w[NW][SLOTS][ITER];  // item r sits in slot r % SLOTS
    int job[R], jrow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        // slots past the workgroup's share repeat its own last row (dropped at the store): a row this CU fetches
        // anyway, where one row for all workgroups would have every CU queue at the same few cache lines
        const int g = min(start + wave + WAVES * r, end - 1);
        if (EPI == WEPI_PAIR) {
            job[r] = 0;
            jrow[r] = g;
        } else {
            const int ji = (int)(g >= e0) + (int)(g >= e1);
            job[r] = ji;
            jrow[r] = g - (ji == 0 ? 0 : ji == 1 ? e0 : e1);
        }
    }
    // Only ONE row's loads (the gate row of the wavefront's first pair) go out in front of the prologue, the rest
    // behind it.  With every row requested up front (as the batch-1 kernel does, which has no barrier) the step of the
    // 7B shape measured 614 tokens/s; with the first pair (or two plain rows) in front 637 (630); with one row 645; with
    // none 628.  What fits that: a CU accepts a bounded number of bytes in flight, so wavefronts that request all their
    // rows sit in their load instructions for most of the stream, the prologue's barrier - behind those instructions in
    // program order - is reached when the stream is nearly over, and normalising and quantizing the activation row
    // then runs after the weights have arrived instead of under them.  One row per wavefront (18 KB per workgroup at
    // 4096 columns) is taken at once and keeps the memory busy while the prologue runs.
    // Items beyond the SLOTS whose weights fit the registers are requested as items in front of them are contracted.
    auto load_row = [&](int r, int m) __attribute__((always_inline)) {
        const uint8_t *Wj = EPI == WEPI_PAIR ? (m == 0 ? W0 : W1) : (job[r] == 0 ? W0 : job[r] == 1 ? W1 : W2);
        const uint8_t *row = Wj + (size_t)jrow[r] * rb;
#pragma unroll
        for (int it = 0; it < ITER; ++it) U::load(row, min(it * 64 + lane, units - 1), w[m][r % SLOTS][it]);
    };
    auto load_item = [&](int r) __attribute__((always_inline)) {
#pragma unroll
        for (int m = 0; m < NW; ++m) load_row(r, m);
    };
    static_assert(SLOTS >= 1 && SLOTS <= R, "register slots for the items' weights");
    if (PRO == WPRO_RMS) {
        // every wavefront's prologue inputs are in the CU's memory pipeline before any weight request of this
        // workgroup (the pipeline returns data in the order it took the requests, whichever wavefront they belong
        // to).  The bare barrier instruction: __syncthreads() would wait for the loads themselves first.
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
    load_row(0, 0);
    __builtin_amdgcn_sched_barrier(0);

    // ---- the activation row: normalised (or merged) and quantized into LDS, once per workgroup
    float4 val[XF];
    if (PRO == WPRO_QUANT) {
#pragma unroll
        for (int i = 0; i < XF; ++i) val[i] = xv[i];
    } else if (PRO == WPRO_RMS) {
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
            const float4 v = xv[i], al = av[i];
            val[i] = make_float4(scale * v.x * al.x, scale * v.y * al.y, scale * v.z * al.z, scale * v.w * al.w);
        }
    }
#pragma unroll
    for (int i = 0; i < XF; ++i) {
        const int c = tid + i * T;
        __half hd;
        int bsum;
        const uint32_t packed = quantize_q8_lane4(val[i], hd, bsum);
        *(uint32_t *)(sq + skewed(4 * c)) = packed;  // c past the row lands in the padding
        if ((c & 7) == 0) {
            Q8Scale sc;
            sc.d = __half2float(hd);
            sc.bsum = bsum;
            ss[c >> 3] = sc;
        }
    }
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);

    // ---- the other items' loads
    if (NW == 2) load_row(0, 1);
#pragma unroll
    for (int r = 1; r < SLOTS; ++r) load_item(r);
    // PLAIN: where each row goes, and the residual it is added to, requested now rather than as a memory round
    // trip after the reduction (rows without one read their own output slot: valid memory, value unused).
    float *yp[R];
    float rv[R];
    bool has_res[R];
    if (EPI == WEPI_PLAIN) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int j = job[r];
            yp[r] = (j == 0 ? a.y[0] : j == 1 ? a.y[1] : a.y[2]) + jrow[r];  // may alias the residual (h += W.x)
            const float *rp = j == 0 ? a.res[0] : j == 1 ? a.res[1] : a.res[2];
            has_res[r] = rp != nullptr;
            rv[r] = *(has_res[r] ? rp + jrow[r] : yp[r]);
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- contraction
    float acc[NW][R];
#pragma unroll
    for (int m = 0; m < NW; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[m][r] = 0.0f;
    if constexpr (SLOTS == R) {
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
    } else {
        // more items than register slots: an item is contracted (units in the same order as above) and the item
        // SLOTS further on is requested into the registers it leaves
#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma unroll
            for (int it = 0; it < ITER; ++it) {
                const int u = it * 64 + lane;
                const bool live = u < units;
                const int uc = live ? u : units - 1;
#pragma unroll
                for (int m = 0; m < NW; ++m) {
                    const float v = U::dot(w[m][r % SLOTS][it], uc, sq, ss);
                    acc[m][r] += live ? v : 0.0f;
                }
            }
            if (r + SLOTS < R) {
                __builtin_amdgcn_sched_barrier(0);
                load_item(r + SLOTS);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    if (EPI == WEPI_PLAIN) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float v = wave_sum(acc[0][r]);
            if (lane == 0 && start + wave + WAVES * r < end) *yp[r] = has_res[r] ? rv[r] + v : v;
        }
        return;
    }

    // ---- PAIR: silu(gate) * up of this workgroup's pairs, then the 32-value blocks they belong to
    // Without a quantized output (oq null) the f32 values go to pair_act as they are and the consumer quantizes them in
    // its own prologue (the down projection, QUANT prologue): no block is shared between workgroups then, no tickets.
    const bool f32_out = a.oq == nullptr;  // uniform
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float g = wave_sum(acc[0][r]), u = wave_sum(acc[1][r]);
        const float act = wide_silu(g) * u;
        if (lane == 0) {
            if (f32_out) {
                if (start + wave + WAVES * r < end) a.pair_act[jrow[r]] = act;
            } else {
                s_act[wave + WAVES * r] = act;  // slots past `end` hold a clamped row: never read
            }
        }
    }
    if (f32_out) return;
    __syncthreads();
    const int b0 = start >> 5, b1 = (end - 1) >> 5;
    for (int blk = b0 + wave; blk <= b1; blk += WAVES) {  // wavefront-uniform: one block per wavefront
        const int first = blk << 5;
        const int lo = max(start, first), hi = min(end, first + 32);
        const int l32 = lane & 31;
        float mine;
        if (hi - lo == 32) {
            mine = s_act[first + l32 - start];
        } else {
            // Part of the block lies with a neighbouring workgroup.  This part goes to pair_act with agent-scope
            // atomic stores, which on gfx950 write through to the memory side where every XCD sees them; the store
            // counter reaching zero means they have arrived (no release fence: that would write the whole L2 back).
            // Then a ticket of the block is drawn; whoever draws the last one reads all 32 values back with
            // agent-scope atomic loads (which do not hit a stale cache line), quantizes them, and puts the counter
            // back to zero.  This rests on those two hardware properties, not on the HIP memory model.
            if (lane < 32 && first + lane >= lo && first + lane < hi)
                __hip_atomic_store(a.pair_act + first + lane, s_act[first + lane - start], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            const unsigned expected = (unsigned)wide_sharers(first, blockIdx.x, G, per, rem);
            unsigned old = 0;
            if (lane == 0) old = __hip_atomic_fetch_add(a.pair_tickets + blk, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            old = (unsigned)__builtin_amdgcn_readfirstlane((int)old);
            if (old != expected - 1) continue;  // a later workgroup finishes the block
            asm volatile("" ::: "memory");
            mine = __hip_atomic_load(a.pair_act + first + l32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (lane == 0) __hip_atomic_store(a.pair_tickets + blk, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __half hd;
        int bsum;
        const int q = quantize_q8_lane1(mine, hd, bsum);
        if (lane < 32) a.oq[(size_t)first + lane] = (int8_t)q;
        if (lane == 0) {
            Q8Scale sc;
            sc.d = __half2float(hd);
            sc.bsum = bsum;
            a.os[blk] = sc;
        }
    }
}

template <class U, int ITER, int R, int WAVES, int PRO, int EPI, int SLOTS = R>
static int launch_wide_cfg(candy_hip_device *dev, WideArgs a, int total, int grid) {
    if ((EPI == WEPI_PAIR && total / grid < 8) || total / grid > 0xFFFF || grid > 0x7FFF)
        return CANDY_HIP_ERR_UNSUPPORTED;  // what wide_sharers and the packing assume
    a.h.per_rem = (total / grid) | ((total % grid) << 16);
    constexpr int T = WAVES * 64, CAP = ITER * 64 * U::ELEMS;
    constexpr int XF = (CAP / 4 + T - 1) / T;
    constexpr size_t QBYTES = (size_t)XF * T * 4;
    constexpr size_t smem = QBYTES + ((QBYTES >> 8) << 4) + ((size_t)XF * T / 8 + 1) * 8;
    static_assert(smem <= 48 * 1024, "LDS image too large");
    hipLaunchKernelGGL((k_matvec_wide<U, ITER, R, WAVES, PRO, EPI, SLOTS>), dim3((unsigned)grid), dim3(T), smem, dev->stream, a.h.x,
                       a.h.alpha, a.h.W[0], a.h.W[1], a.h.W[2], a.h.per_rem, a.h.K, a.h.e0, a.h.e1, a.r);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

// The shapes these kernels exist for: Q4_K weights, rows up to 8192 values (two rounds of units), at least a
// few rows per wavefront.  Anything else: CANDY_HIP_ERR_UNSUPPORTED without error text (the caller takes the
// narrower kernels).
// One Q4_K weight with rows of 4097 .. 16384 values and at most eight rows per workgroup at two workgroups per CU, f32
// input quantized in the prologue: what the decode step's down projection asks for.
bool wide_quant_long_covers(const candy_hip_device *dev, const WideLaunch &L) {
    if (!dev->opt.fused_wide || !dev->opt.down_quant || L.n != 1 || L.alpha || L.pair || !L.x || ((uintptr_t)L.x & 15) != 0) return false;
    const candy_hip_qtensor *w = L.w[0];
    if (w->fmt != CANDY_HIP_Q4_K || ((uintptr_t)w->data & 15) != 0 || w->cols % 256 != 0) return false;
    const int iter = (int)((w->cols / 64 + 63) / 64);
    return iter >= 2 && iter <= 4 && w->rows >= 4 * (int64_t)dev->num_cus && w->rows <= 16 * (int64_t)dev->num_cus;
}

int launch_matvec_wide(candy_hip_device *dev, const WideLaunch &L) {
    const int n = L.n;
    if (n < 1 || n > 3 || !dev->opt.fused_wide) return CANDY_HIP_ERR_UNSUPPORTED;
    const candy_hip_qtensor *w0 = L.w[0];
    for (int i = 0; i < n; ++i) {
        if (L.w[i]->fmt != CANDY_HIP_Q4_K || L.w[i]->cols != w0->cols || ((uintptr_t)L.w[i]->data & 15) != 0) return CANDY_HIP_ERR_UNSUPPORTED;
        if (L.w[i]->rows > 0x3FFFFFFF) return CANDY_HIP_ERR_UNSUPPORTED;
    }
    const int64_t K = w0->cols;
    const bool quant = L.alpha == nullptr;
    if (K % 256 != 0 || K > (quant ? 16384 : 8192)) return CANDY_HIP_ERR_UNSUPPORTED;
    const int iter = (int)((K / 64 + 63) / 64);
    if (!L.x || ((uintptr_t)L.x & 15) != 0) return CANDY_HIP_ERR_UNSUPPORTED;
    if (quant && L.pair) return CANDY_HIP_ERR_UNSUPPORTED;
    WideArgs a{};
    int rows = 0, ends[3];
    for (int i = 0; i < 3; ++i) {
        // unused slots repeat the last weight and end where it does: no row resolves to them
        a.h.W[i] = (const uint8_t *)L.w[i < n ? i : n - 1]->data;
        a.r.y[i] = L.y[i < n ? i : n - 1];
        a.r.res[i] = L.res[i < n ? i : n - 1];
        if (i < n) rows += (int)L.w[i]->rows;
        ends[i] = rows;
    }
    a.h.e0 = ends[0]; a.h.e1 = ends[1];
    a.h.K = (int)K;
    a.h.x = L.x; a.h.alpha = L.alpha; a.r.eps = L.eps;
    a.r.oq = L.oq; a.r.os = L.os; a.r.pair_act = L.pair_act; a.r.pair_tickets = L.pair_tickets;
    const int cus = dev->num_cus;
    if (L.pair) {
        if (n != 2 || L.w[0]->rows != L.w[1]->rows || w0->rows % 32 != 0 || !L.pair_act || !L.pair_tickets) return CANDY_HIP_ERR_UNSUPPORTED;
        if (iter != 1) return CANDY_HIP_ERR_UNSUPPORTED;
        const int total = (int)w0->rows;
        a.h.e0 = a.h.e1 = total;
        if (total < 16 * cus) return CANDY_HIP_ERR_UNSUPPORTED;
        // one workgroup per CU; 16 wavefronts x 3 pairs while a CU's share fits, else 8 wavefronts x up to 8 pairs
        // (the weights of a wavefront's pairs stay in registers: 24 per pair and round of units)
        const int per = (total + cus - 1) / cus;
        if (iter == 1 && dev->opt.wide_waves == 8) {  // two workgroups of eight wavefronts per CU
            const int per2 = (total + 2 * cus - 1) / (2 * cus);
            if (per2 <= 16) return launch_wide_cfg<UnitQ4K, 1, 2, 8, WPRO_RMS, WEPI_PAIR>(dev, a, total, 2 * cus);
            if (per2 <= 24) return launch_wide_cfg<UnitQ4K, 1, 3, 8, WPRO_RMS, WEPI_PAIR>(dev, a, total, 2 * cus);
            // More pairs per wavefront than three: their weights would need more than the 128 registers that let two
            // workgroups share a CU, so the fourth .. sixth pair is requested into the registers of the first .. third
            // once that is contracted (2 x 14336 x 4096, four pairs: 605 tokens/s on the Llama-3-8B shape against 585
            // for three workgroups of three pairs per CU, the third starting when the first is done).
            if (per2 <= 32) return launch_wide_cfg<UnitQ4K, 1, 4, 8, WPRO_RMS, WEPI_PAIR, 3>(dev, a, total, 2 * cus);
            if (per2 <= 40) return launch_wide_cfg<UnitQ4K, 1, 5, 8, WPRO_RMS, WEPI_PAIR, 3>(dev, a, total, 2 * cus);
            if (per2 <= 48) return launch_wide_cfg<UnitQ4K, 1, 6, 8, WPRO_RMS, WEPI_PAIR, 3>(dev, a, total, 2 * cus);
        }
        if (iter == 1) {
            if (per <= 32) return launch_wide_cfg<UnitQ4K, 1, 2, 16, WPRO_RMS, WEPI_PAIR>(dev, a, total, cus);
            if (per <= 48) return launch_wide_cfg<UnitQ4K, 1, 3, 16, WPRO_RMS, WEPI_PAIR>(dev, a, total, cus);
            if (per <= 64) return launch_wide_cfg<UnitQ4K, 1, 8, 8, WPRO_RMS, WEPI_PAIR>(dev, a, total, cus);
            if (per <= 96) return launch_wide_cfg<UnitQ4K, 1, 3, 16, WPRO_RMS, WEPI_PAIR>(dev, a, total, 2 * cus);
        }
        return CANDY_HIP_ERR_UNSUPPORTED;
    }
    const int total = rows;
    if (rows < 16 * cus) return CANDY_HIP_ERR_UNSUPPORTED;
    const int per = (rows + cus - 1) / cus;
    if (quant) {
        // the whole f32-in -> f32-out contraction of one row as one launch: measured ahead of quantize + matvec only
        // for short rows and one row per wavefront (4096 x 4096: 5.0 against 5.8 us; 11008 x 4096: 9.5 against 8.2;
        // 4096 x 11008: 9.0 against 8.9), where the prologue's 16 KB do not hold the weight stream up
        if (iter == 1 && per <= 16 && !L.res[0]) return launch_wide_cfg<UnitQ4K, 1, 1, 16, WPRO_QUANT, WEPI_PLAIN>(dev, a, total, cus);
        // long rows, one row per wavefront, two workgroups of eight per CU: the down projection of a decode step taking
        // the f32 SiLU*Mul values as they come (the gate / up launch then has no 32-value blocks to hand between
        // workgroups)
        if (wide_quant_long_covers(dev, L)) switch (iter) {
            case 2: return launch_wide_cfg<UnitQ4K, 2, 1, 8, WPRO_QUANT, WEPI_PLAIN>(dev, a, total, 2 * cus);
            case 3: return launch_wide_cfg<UnitQ4K, 3, 1, 8, WPRO_QUANT, WEPI_PLAIN>(dev, a, total, 2 * cus);
            case 4: return launch_wide_cfg<UnitQ4K, 4, 1, 8, WPRO_QUANT, WEPI_PLAIN>(dev, a, total, 2 * cus);
            default: break;
            }
        return CANDY_HIP_ERR_UNSUPPORTED;
    }
    if (iter == 1) {
        if (dev->opt.wide_waves == 8) {
            const int per2 = (rows + 2 * cus - 1) / (2 * cus);
            if (per2 <= 16) return launch_wide_cfg<UnitQ4K, 1, 2, 8, WPRO_RMS, WEPI_PLAIN>(dev, a, total, 2 * cus);
            if (per2 <= 24) return launch_wide_cfg<UnitQ4K, 1, 3, 8, WPRO_RMS, WEPI_PLAIN>(dev, a, total, 2 * cus);
            if (per2 <= 32) return launch_wide_cfg<UnitQ4K, 1, 4, 8, WPRO_RMS, WEPI_PLAIN>(dev, a, total, 2 * cus);
        }
        if (per <= 16) return launch_wide_cfg<UnitQ4K, 1, 1, 16, WPRO_RMS, WEPI_PLAIN>(dev, a, total, cus);
        if (per <= 32) return launch_wide_cfg<UnitQ4K, 1, 2, 16, WPRO_RMS, WEPI_PLAIN>(dev, a, total, cus);
        if (per <= 48) return launch_wide_cfg<UnitQ4K, 1, 3, 16, WPRO_RMS, WEPI_PLAIN>(dev, a, total, cus);
        if (per <= 64) return launch_wide_cfg<UnitQ4K, 1, 4, 16, WPRO_RMS, WEPI_PLAIN>(dev, a, total, cus);
        if (per <= 128) return launch_wide_cfg<UnitQ4K, 1, 4, 16, WPRO_RMS, WEPI_PLAIN>(dev, a, total, 2 * cus);
    }
    return CANDY_HIP_ERR_UNSUPPORTED;
}

}  // namespace candy
