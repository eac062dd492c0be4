// Batch-1 (and small-batch, m < 16) quantized matvec: y[m, N] = x[m, K] . W^T with W in candy's
// block formats and x pre-quantized to planar Q8_0.  Bandwidth-bound: the weights are read
// exactly once, 16 bytes per load, straight from the original block layout.
//
// Arithmetic follows the integer vec-dots of tensor/internal/cuda/kernels/quantized.cu
// (vec_dot_q4_0_q8_1 :1919-1941, vec_dot_q8_0_q8_1 :2058-2073, vec_dot_q4_K_q8_1 :2239-2263,
// vec_dot_q6_K_q8_1 :2367-2389) with Q8_0 activations; the launch shape replaces
// mul_mat_vec_q (:2787-2871), which is laid out for 32-wide warps.
//
// Work split: a workgroup of WAVES wavefronts stages the quantized activations in LDS once,
// then every wavefront owns R consecutive weight rows.  A lane owns one "unit" of the row
// (64 weights of a Q4_K super-block, 32 weights otherwise) per step, so consecutive lanes read
// consecutive bytes of the row; the R rows' loads are issued together to keep many bytes in
// flight per wavefront.  Per-row partial sums are reduced across the 64 lanes at the end.
#include <algorithm>
#include <type_traits>

#include "blocks.h"
#include "internal.h"
#include "units.h"
#include "formats_more.h"

namespace candy {

// m <= NB rows exist; the images past them are copies of row m - 1 (their results are not stored)
template <int NB, int THREADS>
__device__ __forceinline__ void stage_activations(const int8_t *__restrict__ xq, const Q8Scale *__restrict__ xs,
                                                  int K, int m, uint8_t *smem, int8_t *&sq, Q8Scale *&ss) {
    const int q_bytes = skewed(K);  // per activation row, a multiple of 16
    sq = (int8_t *)smem;
    ss = (Q8Scale *)(smem + NB * q_bytes);
    const int chunks = K >> 4;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int row = min(nb, m - 1);
        const uint4 *src = (const uint4 *)(xq + (size_t)row * K);
        uint4 *dst = (uint4 *)(sq + nb * q_bytes);
        for (int c = threadIdx.x; c < chunks; c += THREADS) dst[c + (c >> 4)] = src[c];
        const uint2 *s2 = (const uint2 *)xs + (size_t)row * (K >> 5);
        uint2 *d2 = (uint2 *)ss + (size_t)nb * (K >> 5);
        for (int i = threadIdx.x; i < (K >> 5); i += THREADS) d2[i] = s2[i];
    }
    __syncthreads();
}

// ------------------------------------------------------------------ kernels
// Nothing in these kernels branches around a memory operation: out-of-range lanes load a
// clamped (valid) address and their contribution is dropped afterwards.  That keeps the
// hardware load counter exact, so waiting for the activations (issued first, returned first)
// leaves the weight loads in flight.

// Batch-1 kernel.  ITER = ceil(units / 64) is a compile-time bound: every weight load of the
// wavefront's R rows is in flight before anything waits.  The grid covers all rows at once.
// The unit type this kernel loads and contracts with: Q4_K blocks with the header shared over a quad of lanes.
template <class U> struct OnceUnit { typedef U type; };
template <> struct OnceUnit<UnitQ4K> { typedef UnitQ4KQuad type; };
template <> struct OnceUnit<UnitQ6K> { typedef UnitQ6KQuad type; };
template <> struct OnceUnit<UnitQ3K> { typedef UnitQ3KQuad type; };
template <> struct OnceUnit<UnitQ5K> { typedef UnitQ5KQuad type; };

// The body: workgroup `wg` of weight W (N rows), output y (+ residual res, which may alias y: h += W.x).
template <class UT, int ITER, int R, int WAVES>
__device__ __forceinline__ void matvec1_body(const uint8_t *__restrict__ W, float *y, const float *res, int N, int wg,
                                             const int8_t *__restrict__ xq, const Q8Scale *__restrict__ xs, int K) {
    typedef typename OnceUnit<UT>::type U;
    constexpr int T = WAVES * 64;
    constexpr int CAP = ITER * 64 * U::ELEMS;       // activation bytes the LDS image is sized for
    constexpr int AQ = (CAP / 16 + T - 1) / T;      // 16-byte chunks of quants per thread
    constexpr int AS = (CAP / 32 + T - 1) / T;      // 8-byte scales per thread
    extern __shared__ __align__(16) uint8_t smem[];  // sized for AQ*T chunks + AS*T scales: no bounds checks
    int8_t *sq = (int8_t *)smem;
    Q8Scale *ss = (Q8Scale *)(smem + skewed(AQ * T * 16));
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int units = K / U::ELEMS;
    const size_t rb = U::row_bytes(K);
    const int qchunks = K >> 4, sblocks = K >> 5;

    uint4 aq[AQ];
    uint2 as[AS];
#pragma unroll
    for (int i = 0; i < AQ; ++i) aq[i] = ((const uint4 *)xq)[min(tid + i * T, qchunks - 1)];
#pragma unroll
    for (int i = 0; i < AS; ++i) as[i] = ((const uint2 *)xs)[min(tid + i * T, sblocks - 1)];

    const int row0 = (wg * WAVES + wave) * R;
    typename U::W w[R][ITER];
    // Long rows (more than three rounds of units): the first three rounds' loads go out in front of the barrier
    // below, the rest right behind it (held there by a scheduling barrier: the compiler would spread them between the
    // dots of the rounds already in).  With every round in front of the barrier the compiler put the wait for the
    // activations and the barrier itself in front of most weight loads - a memory round trip before the stream
    // starts (Q6_K rows of 14336 values, the Llama-3-8B down projection: 603.5 tokens/s against 611 this way; two,
    // four or five rounds in front measure the same).
    constexpr int FIRST = ITER > 3 ? 3 : ITER;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint8_t *row = W + (size_t)min(row0 + r, N - 1) * rb;
#pragma unroll
        for (int it = 0; it < FIRST; ++it) U::load(row, min(it * 64 + lane, units - 1), w[r][it]);
    }

    // chunks past the row's end land in the padding of the LDS image
#pragma unroll
    for (int i = 0; i < AQ; ++i) {
        const int c = tid + i * T;
        ((uint4 *)sq)[c + (c >> 4)] = aq[i];
    }
#pragma unroll
    for (int i = 0; i < AS; ++i) ((uint2 *)ss)[tid + i * T] = as[i];
    __syncthreads();
    if constexpr (ITER > FIRST) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint8_t *row = W + (size_t)min(row0 + r, N - 1) * rb;
#pragma unroll
            for (int it = FIRST; it < ITER; ++it) U::load(row, min(it * 64 + lane, units - 1), w[r][it]);
        }
        __builtin_amdgcn_sched_barrier(0);  // requested here, not between the dots of the rounds already in
    }

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.0f;
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        const int u = it * 64 + lane;
        const bool live = u < units;
        const int uc = live ? u : units - 1;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float v = U::dot(w[r][it], uc, sq, ss);
            acc[r] += live ? v : 0.0f;
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float v = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < N) y[row0 + r] = res ? res[row0 + r] + v : v;  // Add (backend.go:21) folded in
    }
}

// One weight: everything the first loads need is a plain leading argument (12 dwords, preloaded into registers
// when the wavefront starts), so the activation and weight requests go out without waiting for a scalar load
// of the argument block.
template <class UT, int ITER, int R, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void k_matvec1(const int8_t *__restrict__ xq, const Q8Scale *__restrict__ xs,
                                                        const uint8_t *__restrict__ W, float *y, const float *res, int K,
                                                        int N) {
    matvec1_body<UT, ITER, R, WAVES>(W, y, res, N, (int)blockIdx.x, xq, xs, K);
}

// Up to three weights that share the activation (q / k / v): the workgroup finds its weight in the job table.
template <class UT, int ITER, int R, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void k_matvec1_jobs(const int8_t *__restrict__ xq, const Q8Scale *__restrict__ xs,
                                                             int K, const MatvecJobs jobs) {
    const int ji = (int)(blockIdx.x >= (unsigned)jobs.j[0].wg_end) + (int)(blockIdx.x >= (unsigned)jobs.j[1].wg_end);
    const int wg = blockIdx.x - (ji > 0 ? jobs.j[ji - 1].wg_end : 0);
    matvec1_body<UT, ITER, R, WAVES>(jobs.j[ji].W, jobs.j[ji].y, jobs.j[ji].res, jobs.j[ji].N, wg, xq, xs, K);
}

// Batch-1 kernel for the formats whose blocks are not 16-byte aligned (34, 18, 210 bytes).  Loading
// block by block makes every wavefront load straddle twice the cache lines it uses and touch each
// line from three instructions (measured on the Q8_0 pattern alone: 3.8 TB/s against 5.6 TB/s for
// the same bytes as aligned chunks).  Here the 64 units of a step are fetched as the aligned
// 16-byte chunks of their span, one touch per line (non-temporal), parked in a slice of LDS private
// to the wavefront, and each lane then picks its own block from the slice.  Needs rows that start
// and end on 16-byte boundaries.
template <class U, int ITER, int WAVES>
__device__ __forceinline__ void matvec1_span_body(const uint8_t *__restrict__ W, float *y, const float *res, int N, int wg,
                                                  const int8_t *__restrict__ xq, const Q8Scale *__restrict__ xs, int K) {
    constexpr int T = WAVES * 64;
    constexpr int CAP = ITER * 64 * U::ELEMS;
    constexpr int AQ = (CAP / 16 + T - 1) / T;
    constexpr int AS = (CAP / 32 + T - 1) / T;
    constexpr int CHUNKS = U::SPAN / 16, CPL = (CHUNKS + 63) / 64;
    extern __shared__ __align__(16) uint8_t smem[];
    int8_t *sq = (int8_t *)smem;
    Q8Scale *ss = (Q8Scale *)(smem + skewed(AQ * T * 16));
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    uint8_t *slice = smem + skewed(AQ * T * 16) + AS * T * (int)sizeof(Q8Scale) + wave * (CPL * 64 * 16);
    const int units = K / U::ELEMS;
    const size_t rb = U::row_bytes(K);
    const int qchunks = K >> 4, sblocks = K >> 5, row_chunks = (int)(rb >> 4);

    uint4 aq[AQ];
    uint2 as[AS];
#pragma unroll
    for (int i = 0; i < AQ; ++i) aq[i] = ((const uint4 *)xq)[min(tid + i * T, qchunks - 1)];
#pragma unroll
    for (int i = 0; i < AS; ++i) as[i] = ((const uint2 *)xs)[min(tid + i * T, sblocks - 1)];

    const int row = wg * WAVES + wave;
    const u32x4 *rowp = (const u32x4 *)(W + (size_t)min(row, N - 1) * rb);
    u32x4 ch[ITER][CPL];
#pragma unroll
    for (int it = 0; it < ITER; ++it)
#pragma unroll
        for (int k = 0; k < CPL; ++k) {
            const int ci = k * 64 + lane;  // chunks past the span reload its first one, chunks past the row its last
            ch[it][k] = __builtin_nontemporal_load(rowp + min(it * CHUNKS + (ci < CHUNKS ? ci : 0), row_chunks - 1));
        }

#pragma unroll
    for (int i = 0; i < AQ; ++i) {
        const int c = tid + i * T;
        ((uint4 *)sq)[c + (c >> 4)] = aq[i];
    }
#pragma unroll
    for (int i = 0; i < AS; ++i) ((uint2 *)ss)[tid + i * T] = as[i];
    __syncthreads();

    float acc = 0.0f;
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        // the slice is private to the wavefront, whose LDS operations complete in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int k = 0; k < CPL; ++k) *(u32x4 *)(slice + 16 * (k * 64 + lane)) = ch[it][k];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int u = it * 64 + lane;
        const bool live = u < units;
        typename U::W w;
        U::load(slice, lane, w);
        const float v = U::dot(w, live ? u : units - 1, sq, ss);
        acc += live ? v : 0.0f;
    }
    const float v = wave_sum(acc);
    if (lane == 0 && row < N) y[row] = res ? res[row] + v : v;
}

template <class U, int ITER, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void k_matvec1_span(const int8_t *__restrict__ xq, const Q8Scale *__restrict__ xs,
                                                             const uint8_t *__restrict__ W, float *y, const float *res,
                                                             int K, int N) {
    matvec1_span_body<U, ITER, WAVES>(W, y, res, N, (int)blockIdx.x, xq, xs, K);
}

template <class U, int ITER, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void k_matvec1_span_jobs(const int8_t *__restrict__ xq,
                                                                  const Q8Scale *__restrict__ xs, int K,
                                                                  const MatvecJobs jobs) {
    const int ji = (int)(blockIdx.x >= (unsigned)jobs.j[0].wg_end) + (int)(blockIdx.x >= (unsigned)jobs.j[1].wg_end);
    const int wg = blockIdx.x - (ji > 0 ? jobs.j[ji - 1].wg_end : 0);
    matvec1_span_body<U, ITER, WAVES>(jobs.j[ji].W, jobs.j[ji].y, jobs.j[ji].res, jobs.j[ji].N, wg, xq, xs, K);
}

// General kernel: NB activation rows (small batch) and any contraction length; each wavefront
// owns R weight rows and walks the row 64 units at a time.
template <class U> struct LoopUnit { typedef U type; };
template <> struct LoopUnit<UnitQ6K> { typedef UnitQ6KQuad type; };
template <> struct LoopUnit<UnitQ3K> { typedef UnitQ3KQuad type; };
template <> struct LoopUnit<UnitQ5K> { typedef UnitQ5KQuad type; };
template <> struct LoopUnit<UnitQ4K> { typedef UnitQ4KQuad type; };  // 2 rows: 4096 x 32768 41.1 -> 39.0 us, 32000 x 4096 23.1 -> 22.7

template <class UT, int NB, int R, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void k_matvec(const uint8_t *__restrict__ W, const int8_t *__restrict__ xq,
                                                       const Q8Scale *__restrict__ xs, float *__restrict__ y,
                                                       int N, int K, int m) {
    typedef typename LoopUnit<UT>::type U;
    extern __shared__ __align__(16) uint8_t smem[];
    int8_t *sq;
    Q8Scale *ss;
    stage_activations<NB, WAVES * 64>(xq, xs, K, m, smem, sq, ss);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row0 = (blockIdx.x * WAVES + wave) * R;
    if (row0 >= N) return;
    const int units = K / U::ELEMS;
    const size_t rb = U::row_bytes(K);
    const int q_bytes = skewed(K);
    const int blocks_per_row = K >> 5;

    float acc[R][NB];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[r][nb] = 0.0f;

    for (int u0 = 0; u0 < units; u0 += 64) {
        const int u = u0 + lane;
        const bool live = u < units;
        const int uc = live ? u : units - 1;
        typename U::W w[R];
#pragma unroll
        for (int r = 0; r < R; ++r) U::load(W + (size_t)min(row0 + r, N - 1) * rb, uc, w[r]);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const float v = U::dot(w[r], uc, sq + nb * q_bytes, ss + nb * blocks_per_row);
                acc[r][nb] += live ? v : 0.0f;
            }
    }

#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const float v = wave_sum(acc[r][nb]);
            if (lane == 0 && row0 + r < N && nb < m) y[(size_t)nb * N + row0 + r] = v;
        }
}

template <class U, int ITER, int R, int WAVES>
static int launch1(candy_hip_device *dev, MatvecJobs jobs, int K, const int8_t *qs, const Q8Scale *scales) {
    constexpr int T = WAVES * 64, CAP = ITER * 64 * U::ELEMS;
    constexpr int AQ = (CAP / 16 + T - 1) / T, AS = (CAP / 32 + T - 1) / T;
    constexpr size_t smem = (size_t)AQ * T * 16 + (((size_t)AQ * T * 16 >> 8) << 4) + (size_t)AS * T * sizeof(Q8Scale);
    static_assert(smem <= 64 * 1024, "LDS image too large");
    const int rows_per_wg = R * WAVES;
    int total = 0;
    for (int i = 0; i < 3; ++i) {
        if (i < jobs.n) total += (jobs.j[i].N + rows_per_wg - 1) / rows_per_wg;
        jobs.j[i].wg_end = total;  // unused slots end where the last real one does
    }
    if (jobs.n == 1)
        hipLaunchKernelGGL((k_matvec1<U, ITER, R, WAVES>), dim3((unsigned)total), dim3(WAVES * 64), smem, dev->stream, qs,
                           scales, jobs.j[0].W, jobs.j[0].y, jobs.j[0].res, K, jobs.j[0].N);
    else
        hipLaunchKernelGGL((k_matvec1_jobs<U, ITER, R, WAVES>), dim3((unsigned)total), dim3(WAVES * 64), smem, dev->stream,
                           qs, scales, K, jobs);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

template <class U, int ITER, int WAVES>
static int launch1_span(candy_hip_device *dev, MatvecJobs jobs, int K, const int8_t *qs, const Q8Scale *scales) {
    constexpr int T = WAVES * 64, CAP = ITER * 64 * U::ELEMS;
    constexpr int AQ = (CAP / 16 + T - 1) / T, AS = (CAP / 32 + T - 1) / T;
    constexpr int CPL = (U::SPAN / 16 + 63) / 64;
    constexpr size_t smem = (size_t)AQ * T * 16 + (((size_t)AQ * T * 16 >> 8) << 4) + (size_t)AS * T * sizeof(Q8Scale) +
                            (size_t)WAVES * CPL * 64 * 16;
    static_assert(smem <= 64 * 1024, "LDS image too large");
    int total = 0;
    for (int i = 0; i < 3; ++i) {
        if (i < jobs.n) total += (jobs.j[i].N + WAVES - 1) / WAVES;
        jobs.j[i].wg_end = total;
    }
    if (jobs.n == 1)
        hipLaunchKernelGGL((k_matvec1_span<U, ITER, WAVES>), dim3((unsigned)total), dim3(WAVES * 64), smem, dev->stream, qs,
                           scales, jobs.j[0].W, jobs.j[0].y, jobs.j[0].res, K, jobs.j[0].N);
    else
        hipLaunchKernelGGL((k_matvec1_span_jobs<U, ITER, WAVES>), dim3((unsigned)total), dim3(WAVES * 64), smem,
                           dev->stream, qs, scales, K, jobs);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

template <class U>
static int launch_jobs_fmt(candy_hip_device *dev, const MatvecJobs &jobs, int64_t K, const int8_t *qs,
                           const Q8Scale *scales) {
    const int iter = (int)((K / U::ELEMS + 63) / 64);
    if constexpr (U::SPAN > 0) {
        bool aligned = U::row_bytes((int)K) % 16 == 0 && dev->opt.matvec_span != 0;
        for (int i = 0; i < jobs.n; ++i) aligned = aligned && ((uintptr_t)jobs.j[i].W & 15) == 0;
        if (aligned) switch (iter) {
            case 1: return launch1_span<U, 1, 4>(dev, jobs, (int)K, qs, scales);
            case 2: return launch1_span<U, 2, 4>(dev, jobs, (int)K, qs, scales);
            case 3: return launch1_span<U, 3, 4>(dev, jobs, (int)K, qs, scales);
            case 4: return launch1_span<U, 4, 4>(dev, jobs, (int)K, qs, scales);
            case 5: return launch1_span<U, 5, 4>(dev, jobs, (int)K, qs, scales);
            case 6: return launch1_span<U, 6, 4>(dev, jobs, (int)K, qs, scales);
            case 7: return launch1_span<U, 7, 4>(dev, jobs, (int)K, qs, scales);
            default: break;
            }
    }
    switch (iter) {
    case 1: return launch1<U, 1, 1, 4>(dev, jobs, (int)K, qs, scales);
    case 2: return launch1<U, 2, 1, 4>(dev, jobs, (int)K, qs, scales);
    case 3: return launch1<U, 3, 1, 4>(dev, jobs, (int)K, qs, scales);
    case 4: return launch1<U, 4, 1, 4>(dev, jobs, (int)K, qs, scales);
    case 5: return launch1<U, 5, 1, 4>(dev, jobs, (int)K, qs, scales);
    case 6: return launch1<U, 6, 1, 4>(dev, jobs, (int)K, qs, scales);
    case 7: return launch1<U, 7, 1, 4>(dev, jobs, (int)K, qs, scales);
    case 8: return launch1<U, 8, 1, 4>(dev, jobs, (int)K, qs, scales);
    default: return CANDY_HIP_ERR_UNSUPPORTED;  // longer rows take the looping kernel
    }
}

static int launch_jobs(candy_hip_device *dev, int fmt, const MatvecJobs &jobs, int64_t K, const int8_t *qs,
                       const Q8Scale *scales) {
    switch (fmt) {
    case CANDY_HIP_Q4_K: return launch_jobs_fmt<UnitQ4K>(dev, jobs, K, qs, scales);
    case CANDY_HIP_Q8_0: return launch_jobs_fmt<UnitQ8_0>(dev, jobs, K, qs, scales);
    case CANDY_HIP_Q4_0: return launch_jobs_fmt<UnitQ4_0<false>>(dev, jobs, K, qs, scales);
    case CANDY_HIP_Q4_0_GGML: return launch_jobs_fmt<UnitQ4_0<true>>(dev, jobs, K, qs, scales);
    case CANDY_HIP_Q6_K: return launch_jobs_fmt<UnitQ6K>(dev, jobs, K, qs, scales);
    case CANDY_HIP_Q4_1: return launch_jobs_fmt<UnitQ4_1<false>>(dev, jobs, K, qs, scales);
    case CANDY_HIP_Q4_1_GGML: return launch_jobs_fmt<UnitQ4_1<true>>(dev, jobs, K, qs, scales);
    case CANDY_HIP_Q5_0: return launch_jobs_fmt<UnitQ5<false>>(dev, jobs, K, qs, scales);
    case CANDY_HIP_Q5_1: return launch_jobs_fmt<UnitQ5<true>>(dev, jobs, K, qs, scales);
    case CANDY_HIP_Q2_K: return launch_jobs_fmt<UnitQ2K>(dev, jobs, K, qs, scales);
    case CANDY_HIP_Q3_K: return launch_jobs_fmt<UnitQ3K>(dev, jobs, K, qs, scales);
    case CANDY_HIP_Q5_K: return launch_jobs_fmt<UnitQ5K>(dev, jobs, K, qs, scales);
    default:
        if (format_info(fmt).elems != 0) return CANDY_HIP_ERR_UNSUPPORTED;  // Q8_K: no vec-dot
        return fail(CANDY_HIP_ERR_INVALID, "unknown quantized format %d", fmt);
    }
}

// A unit's dot product in two parts where the unit offers them (U::P, U::prep, U::dot_p), in one otherwise.
template <class U, class = void>
struct Prepped {
    typedef typename U::W P;
    __device__ static __forceinline__ void prep(const typename U::W &w, int, P &p) { p = w; }
    __device__ static __forceinline__ float dot(const P &p, int u, const int8_t *sq, const Q8Scale *ss) { return U::dot(p, u, sq, ss); }
};
template <class U>
struct Prepped<U, std::void_t<typename U::P>> {
    typedef typename U::P P;
    __device__ static __forceinline__ void prep(const typename U::W &w, int u, P &p) { U::prep(w, u, p); }
    __device__ static __forceinline__ float dot(const P &p, int u, const int8_t *sq, const Q8Scale *ss) { return U::dot_p(p, u, sq, ss); }
};

// Small batches (2 <= m <= 8 rows of activations per pass).  One workgroup of 16 wavefronts per CU holds all NB
// quantized activation rows in LDS (up to 150 KB: staged once per CU, not once per 8 weight rows) and walks its
// share of the weight rows, one row per wavefront at a time, every load of the row in flight before the first
// dot, as in the batch-1 kernel; a lane dots its unit against each activation row in turn.  The weights are read
// once whatever the batch; past m = 2 the kernel is bound by the dots (NB times the batch-1 arithmetic) and by the
// LDS reads of the activation images, not by HBM.  Rows of the batch beyond m are a copy of row m - 1 and are not
// stored.  No barrier after the staging: the wavefronts drift apart and cover each other's load latency.
template <class U, int ITER, int NB>
__global__ __launch_bounds__(1024) void k_matvec_mb(const uint8_t *__restrict__ W, const int8_t *__restrict__ xq,
                                                    const Q8Scale *__restrict__ xs, float *__restrict__ y, int N, int K,
                                                    int m) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int units = K / U::ELEMS;
    const size_t rb = U::row_bytes(K);
    const int q_bytes = skewed(K), blocks_per_row = K >> 5;
    int8_t *sq = (int8_t *)smem;
    Q8Scale *ss = (Q8Scale *)(smem + NB * q_bytes);

    const int step = gridDim.x * 16;
    int row = blockIdx.x * 16 + wave;
    typename U::W w[ITER];
    {   // the first row's weights are requested before the activations are staged
        const uint8_t *rp = W + (size_t)min(row, N - 1) * rb;
#pragma unroll
        for (int it = 0; it < ITER; ++it) U::load(rp, min(it * 64 + lane, units - 1), w[it]);
    }
    {
        const int chunks = K >> 4;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int src_row = min(nb, m - 1);
            const uint4 *src = (const uint4 *)(xq + (size_t)src_row * K);
            uint4 *dst = (uint4 *)(sq + nb * q_bytes);
            for (int c = tid; c < chunks; c += 1024) dst[c + (c >> 4)] = src[c];
            const uint2 *s2 = (const uint2 *)(xs + (size_t)src_row * blocks_per_row);
            uint2 *d2 = (uint2 *)(ss + nb * blocks_per_row);
            for (int i = tid; i < blocks_per_row; i += 1024) d2[i] = s2[i];
        }
    }
    __syncthreads();

    while (row < N) {
        typename Prepped<U>::P pw[ITER];  // the weight-only part of the dots, once per weight row
#pragma unroll
        for (int it = 0; it < ITER; ++it) Prepped<U>::prep(w[it], min(it * 64 + lane, units - 1), pw[it]);
        // one activation row at a time (not unrolled: a lane's share of NB rows at once does not fit the registers)
#pragma unroll 1
        for (int nb = 0; nb < NB; ++nb) {
            const int8_t *q = sq + nb * q_bytes;
            const Q8Scale *sc = ss + nb * blocks_per_row;
            float acc = 0.0f;
#pragma unroll
            for (int it = 0; it < ITER; ++it) {
                const int u = it * 64 + lane;
                const bool live = u < units;
                const float v = Prepped<U>::dot(pw[it], live ? u : units - 1, q, sc);
                acc += live ? v : 0.0f;
            }
            acc = wave_sum(acc);
            if (lane == 0 && nb < m) y[(size_t)nb * N + row] = acc;
        }
        row += step;
        if (row < N) {  // wavefront-uniform
            const uint8_t *rp = W + (size_t)row * rb;
#pragma unroll
            for (int it = 0; it < ITER; ++it) U::load(rp, min(it * 64 + lane, units - 1), w[it]);
        }
    }
}

// LDS the small-batch kernel needs for NB activation rows of length K
static size_t mb_lds_bytes(int nb, int64_t K) {
    return (size_t)nb * ((size_t)K + (((size_t)K >> 8) << 4) + (size_t)(K >> 5) * sizeof(Q8Scale));
}
constexpr size_t MB_LDS_MAX = 160 * 1024;

template <class U, int ITER, int NB>
static int launch_mb_cfg(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales, int m,
                         float *y) {
    const int N = (int)w->rows, K = (int)w->cols;
    const size_t smem = mb_lds_bytes(NB, K);
    auto kern = k_matvec_mb<U, ITER, NB>;
    CANDY_HIP_TRY(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    const int groups = (N + 15) / 16;
    hipLaunchKernelGGL(kern, dim3((unsigned)std::min(groups, dev->num_cus)), dim3(1024), smem, dev->stream,
                       (const uint8_t *)w->data, qs, scales, y, N, K, m);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

// One pass of up to 8 activation rows; CANDY_HIP_ERR_UNSUPPORTED (no error text) when the row is too long for it.
template <class U>
static int launch_mb(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales, int m,
                     float *y) {
    const int64_t K = w->cols;
    const int iter = (int)((K / U::ELEMS + 63) / 64);
    const bool wide = m > 4 && mb_lds_bytes(8, K) <= MB_LDS_MAX;
    // rounds of 64 units the kernel holds in registers without spilling, per format (Q6_K: none so far)
    constexpr int max_iter = std::is_same<U, UnitQ4K>::value ? 4 : (std::is_same<U, UnitQ8_0>::value || std::is_same<U, UnitQ4_0<false>>::value || std::is_same<U, UnitQ4_0<true>>::value) ? 8 : 0;
    if (iter > max_iter || (!wide && (m > 4 || mb_lds_bytes(4, K) > MB_LDS_MAX))) return CANDY_HIP_ERR_UNSUPPORTED;
#define CANDY_MB(IT)                                                                  \
    return wide ? launch_mb_cfg<U, IT, 8>(dev, w, qs, scales, m, y) : launch_mb_cfg<U, IT, 4>(dev, w, qs, scales, m, y)
    switch (iter) {
    case 1: CANDY_MB(1);
    case 2: CANDY_MB(2);
    case 3: CANDY_MB(3);
    case 4: CANDY_MB(4);
    case 5: case 6: CANDY_MB(6);
    default: CANDY_MB(8);
    }
#undef CANDY_MB
}

// Two activation rows, even split: the weight rows dealt evenly (to within one row) to two workgroups of 8 wavefronts
// per CU; a wavefront requests all of its R rows before the NB = 2 quantized activation rows are staged in LDS, so the
// whole share of a CU is in flight at once, as in the batch-1 kernel, and the dots of a row (its weight-only part
// prepared once, then one dot per activation row) start as its bytes arrive.  Per row and activation row the
// additions are those of the other vector kernels: a lane's units in ascending order, then the wavefront sum - the
// same bits.  The role of mul_mat_vec_q<2> (quantized.cu:2787-2871).  Measured with more images (us per call with the
// quantizer, 4096 x 11008): 2 rows 12.2 against 14.5 on the looping kernel; 3 and 4 rows 15.6 and 16.3 against 14.0 on
// the one-pass matrix-core kernel - every further image costs a CU 1.7 us of dot4 arithmetic that starts only when
// the rows have arrived - so only the two-image form is built.
template <class U, int ITER, int R, int NB>
__global__ __launch_bounds__(512, 4) void k_matvec_even(const uint8_t *__restrict__ W, const int8_t *__restrict__ xq,
                                                     const Q8Scale *__restrict__ xs, float *__restrict__ y, int N, int K,
                                                     int m, int per, int rem) {
    constexpr int WAVES = 8;
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int units = K / U::ELEMS;
    const size_t rb = U::row_bytes(K);
    const int q_bytes = skewed(K), blocks_per_row = K >> 5;
    int8_t *sq = (int8_t *)smem;
    Q8Scale *ss = (Q8Scale *)(smem + NB * q_bytes);
    // the first `rem` = N % grid workgroups take per + 1 = N / grid + 1 rows, the others per (both from the host: a
    // 64-bit division here is some 350 scalar instructions in front of the first load)
    const int g = blockIdx.x;
    const int start = g * per + min(g, rem), end = (g + 1) * per + min(g + 1, rem);

    typename U::W w[R][ITER];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        // slots past the share repeat its last row (not stored): a row this workgroup fetches anyway
        const uint8_t *rp = W + (size_t)min(start + wave + WAVES * r, end - 1) * rb;
#pragma unroll
        for (int it = 0; it < ITER; ++it) U::load(rp, min(it * 64 + lane, units - 1), w[r][it]);
    }
    {
        const int chunks = K >> 4;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int src_row = min(nb, m - 1);  // images past m: a copy of the last row, not stored
            const uint4 *src = (const uint4 *)(xq + (size_t)src_row * K);
            uint4 *dst = (uint4 *)(sq + nb * q_bytes);
            for (int c = tid; c < chunks; c += WAVES * 64) dst[c + (c >> 4)] = src[c];
            const uint2 *s2 = (const uint2 *)(xs + (size_t)src_row * blocks_per_row);
            uint2 *d2 = (uint2 *)(ss + nb * blocks_per_row);
            for (int i = tid; i < blocks_per_row; i += WAVES * 64) d2[i] = s2[i];
        }
    }
    __syncthreads();

#pragma unroll
    for (int r = 0; r < R; ++r) {
        float acc[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[nb] = 0.0f;
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            const int u = it * 64 + lane;
            const bool live = u < units;
            const int uc = live ? u : units - 1;
            typename Prepped<U>::P pw;
            Prepped<U>::prep(w[r][it], uc, pw);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const float v = Prepped<U>::dot(pw, uc, sq + nb * q_bytes, ss + nb * blocks_per_row);
                acc[nb] += live ? v : 0.0f;
                // one dot's activations in registers at a time: the sum is pinned here and no LDS read crosses (the
                // reads of every image and round hoisted cost registers; the SIMD's other wavefronts cover the latency)
                asm volatile("" : "+v"(acc[nb]) : : "memory");
            }
        }
        const int row = start + wave + WAVES * r;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const float sum = wave_sum(acc[nb]);
            if (lane == 0 && nb < m && row < end) y[(size_t)nb * N + row] = sum;
        }
    }
}

template <class U, int ITER, int R, int NB>
static int launch_even_cfg(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales, int m,
                           float *y, int grid) {
    const int N = (int)w->rows, K = (int)w->cols;
    const size_t smem = mb_lds_bytes(NB, K);
    auto kern = k_matvec_even<U, ITER, R, NB>;
    if (smem > 48 * 1024)
        CANDY_HIP_TRY(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), smem, dev->stream, (const uint8_t *)w->data, qs, scales, y, N,
                       K, m, N / grid, N % grid);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

// Rows of a weight per wavefront (R) in the even-split kernel, or 0 where it does not apply: two activation rows,
// Q4_K with rows of up to four rounds of units, at least 16 weight rows per CU and at most R * rounds = 3 or 4 units
// per lane (measured, us per call with the quantizer, against the looping kernel: 4096 x 14336 14.3 / 17.4, 4096 x
// 11008 12.2 / 14.5, 4096 x 4096 7.3 / 7.9, 11008 x 4096 11.8 / 12.2; with four rows per wavefront 14336 x 4096 13.9 /
// 13.2), and the images of two workgroups fitting a CU's LDS.
static int even_rows_per_wave(const candy_hip_qtensor *w, int64_t m) {
    const candy_hip_device *dev = w->dev;
    if (w->fmt != CANDY_HIP_Q4_K || m != 2 || !dev->opt.even_two_rows || ((uintptr_t)w->data & 15) != 0) return 0;
    const int64_t K = w->cols;
    if (K % 256 != 0 || K > 16384 || w->rows < 16 * (int64_t)dev->num_cus || w->rows > 0x3FFFFFFF) return 0;
    if (2 * mb_lds_bytes(2, K) > MB_LDS_MAX) return 0;
    const int iter = (int)((K / UnitQ4K::ELEMS + 63) / 64);
    const int64_t per2 = (w->rows + 2 * dev->num_cus - 1) / (2 * dev->num_cus);
    const int r = (int)((per2 + 7) / 8);
    return r <= (iter == 1 ? 3 : 1) ? r : 0;
}
bool matvec_even_covers(const candy_hip_qtensor *w, int64_t m) { return even_rows_per_wave(w, m) != 0; }

static int launch_even(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales, int m,
                       float *y) {
    typedef UnitQ4K U;
    const int r = even_rows_per_wave(w, m);
    if (!r) return CANDY_HIP_ERR_UNSUPPORTED;
    const int iter = (int)((w->cols / U::ELEMS + 63) / 64), grid = 2 * dev->num_cus;
    if (iter == 1) {
        if (r == 1) return launch_even_cfg<U, 1, 1, 2>(dev, w, qs, scales, m, y, grid);
        if (r == 2) return launch_even_cfg<U, 1, 2, 2>(dev, w, qs, scales, m, y, grid);
        return launch_even_cfg<U, 1, 3, 2>(dev, w, qs, scales, m, y, grid);
    }
    if (iter == 2) return launch_even_cfg<U, 2, 1, 2>(dev, w, qs, scales, m, y, grid);
    if (iter == 3) return launch_even_cfg<U, 3, 1, 2>(dev, w, qs, scales, m, y, grid);
    return launch_even_cfg<U, 4, 1, 2>(dev, w, qs, scales, m, y, grid);
}

template <class U, int NB, int R, int WAVES>
static int launch_one(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales,
                      float *y, int m = NB) {
    const int N = (int)w->rows, K = (int)w->cols;
    const size_t q_bytes = (size_t)K + (((size_t)K >> 8) << 4);
    const size_t smem = NB * (q_bytes + (size_t)(K >> 5) * sizeof(Q8Scale));
    CANDY_REQUIRE(smem <= 64 * 1024, "contraction dim %d too large for the matvec kernel (%zu bytes of LDS)", K, smem);
    const int rows_per_wg = R * WAVES;
    const unsigned grid = (unsigned)((N + rows_per_wg - 1) / rows_per_wg);
    hipLaunchKernelGGL((k_matvec<U, NB, R, WAVES>), dim3(grid), dim3(WAVES * 64), smem, dev->stream,
                       (const uint8_t *)w->data, qs, scales, y, N, K, m);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

// Activation images per launch of the looping kernel: the smallest of 1, 2, 4, 8 that covers what is left (three rows
// ride in a four-image launch, the fourth image a copy nobody stores), capped so that the images stay under 64 KB
// of LDS.
static int looping_rows(int64_t left, int64_t K) {
    const int cap = K <= 5632 ? 8 : K <= 11264 ? 4 : K <= 16384 ? 2 : 1;
    int nb = 1;
    while (nb < left && nb < cap) nb <<= 1;
    return nb;
}

template <class U>
static int launch_fmt(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales,
                      int64_t m, float *y) {
    const int64_t K = w->cols, N = w->rows;
    const int64_t sstride = K >> 5;
    if (m == 1) {
        MatvecJobs jobs{};
        jobs.n = 1;
        jobs.j[0].W = (const uint8_t *)w->data;
        jobs.j[0].y = y;
        jobs.j[0].N = (int)N;
        const int rc = launch_jobs_fmt<U>(dev, jobs, K, qs, scales);
        if (rc != CANDY_HIP_ERR_UNSUPPORTED) return rc;
    }
    int64_t done = 0;
    const bool old_small = dev->opt.small_batch_kernel == 0;  // comparison runs and tests
    while (done < m) {
        const int64_t left = m - done;
        const int8_t *q = qs + done * K;
        const Q8Scale *s = scales + done * sstride;
        float *yo = y + done * N;
        int rc;
        if (!old_small && matvec_even_covers(w, left)) {  // what is left in one pass of the even-split kernel
            rc = launch_even(dev, w, q, s, (int)left, yo);
            if (rc == CANDY_HIP_OK) { done += left; continue; }
            if (rc != CANDY_HIP_ERR_UNSUPPORTED) return rc;
        }
        {
            // The looping kernel below takes up to 8, 4, 2 or 1 rows per launch (fewer the longer the row is); where that
            // covers what is left in as few launches as this kernel's 8 per pass, it is as fast or a little faster
            // (short rows, up to about 16K of them), and two rows cost less there than as half of a 4-row pass.
            int old_launches = 0;
            for (int64_t l = left; l > 0; ++old_launches) l -= std::min<int64_t>(l, looping_rows(l, K));
            const bool old_is_fine = left == 2 || (K <= 5632 && N <= 16384 && old_launches == (left + 7) / 8);
            if (left >= 2 && !old_small && !old_is_fine) {  // up to 8 rows per pass, or 4 where 8 do not fit LDS
                const int take = (int)std::min<int64_t>(left, mb_lds_bytes(8, K) <= MB_LDS_MAX ? 8 : 4);
                rc = launch_mb<U>(dev, w, q, s, take, yo);
                if (rc == CANDY_HIP_OK) { done += take; continue; }
                if (rc != CANDY_HIP_ERR_UNSUPPORTED) return rc;
            }
        }
        const int nb = looping_rows(left, K), take = (int)std::min<int64_t>(left, nb);
        switch (nb) {
        case 8: rc = launch_one<U, 8, 2, 4>(dev, w, q, s, yo, take); break;
        case 4: rc = launch_one<U, 4, 2, 4>(dev, w, q, s, yo, take); break;
        case 2: rc = launch_one<U, 2, 2, 4>(dev, w, q, s, yo, take); break;
        default: rc = launch_one<U, 1, 2, 4>(dev, w, q, s, yo, take); break;
        }
        if (rc) return rc;
        done += take;
    }
    return CANDY_HIP_OK;
}

// Batch-1 contraction of one quantized activation row against up to three weights in ONE launch
// (q/k/v, gate/up), each with an optional residual added to its output.  Weights must share
// format and contraction length; otherwise, or for very long rows, one launch per weight.
int launch_matvec_multi(candy_hip_device *dev, const candy_hip_qtensor *const *ws, float *const *ys,
                        const float *const *res, int n, const int8_t *qs, const Q8Scale *scales) {
    CANDY_REQUIRE(n >= 1 && n <= 3, "internal: 1..3 weights per launch");
    bool same = true;
    for (int i = 1; i < n; ++i) same = same && ws[i]->fmt == ws[0]->fmt && ws[i]->cols == ws[0]->cols;
    if (same) {
        MatvecJobs jobs{};
        jobs.n = n;
        for (int i = 0; i < n; ++i) {
            CANDY_REQUIRE(ws[i]->rows <= 0x7FFFFFFF && ws[i]->cols <= 0x7FFFFFFF, "matrix too large");
            jobs.j[i].W = (const uint8_t *)ws[i]->data;
            jobs.j[i].y = ys[i];
            jobs.j[i].res = res ? res[i] : nullptr;
            jobs.j[i].N = (int)ws[i]->rows;
        }
        const int rc = launch_jobs(dev, ws[0]->fmt, jobs, ws[0]->cols, qs, scales);
        if (rc != CANDY_HIP_ERR_UNSUPPORTED) return rc;
    }
    for (int i = 0; i < n; ++i) {
        if (res && res[i]) return CANDY_HIP_ERR_UNSUPPORTED;  // rows too long for the batch-1 kernel: the caller adds the residual itself
        if (int rc = launch_matvec(dev, ws[i], qs, scales, 1, ys[i])) return rc;
    }
    return CANDY_HIP_OK;
}

int act_workspace(candy_hip_device *dev, int64_t m, int64_t cols, bool need_quants, ActWorkspace *out) {
    const size_t q_bytes = need_quants ? (((size_t)(m * cols) + 255) & ~(size_t)255) : 0;
    const size_t s_bytes = need_quants ? (((size_t)(m * (cols >> 5)) * sizeof(Q8Scale) + 255) & ~(size_t)255) : 0;
    const size_t h_bytes = m >= 16 ? (size_t)(mmq_m_pad(m) * cols) * 2 : 0;
    const size_t v_bytes = need_quants && m >= 2 && m <= 32 && cols % 256 == 0 ? mmv_workspace_bytes(cols) : 0;
    void *ws = nullptr;
    if (int rc = workspace(dev, q_bytes + s_bytes + h_bytes + v_bytes + 256, &ws)) return rc;
    out->qs = (int8_t *)ws;
    out->scales = (Q8Scale *)((uint8_t *)ws + q_bytes);
    out->half_ws = h_bytes ? (uint8_t *)ws + q_bytes + s_bytes : nullptr;
    out->mmv_ws = v_bytes ? (uint8_t *)ws + q_bytes + s_bytes + h_bytes : nullptr;
    return CANDY_HIP_OK;
}

int launch_matvec(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales,
                  int64_t m, float *y, bool vector_only) {
    CANDY_REQUIRE(w->rows <= 0x7FFFFFFF && w->cols <= 0x7FFFFFFF, "matrix too large");
    // the 32-value formats: the vector kernels match the tile kernel up to 8 rows (one pass) on small weights; from 9
    // rows on they need two passes, and on weights of 40 M values and more the tile kernel is level or ahead from 5 rows
    // (us per call, 5-8 rows on the vector kernels / 9 rows on the tiles: Q8_0 32000 x 4096 50.5-51.4 / 46.3, 4096 x 11008
    // 26 / 25.3; Q4_0 32000 x 4096 49.2-50.3 / 40.2, 4096 x 11008 24.8-25.9 / 23.1; but 4096 x 4096 13.4-15.0 / 15.1)
    const bool big_weight = (double)w->rows * (double)w->cols >= 4.0e7;
    if (!vector_only && (m >= 9 || (m >= 5 && big_weight)) && w->fmt != CANDY_HIP_Q4_K && w->fmt != CANDY_HIP_Q6_K &&
        w->fmt != CANDY_HIP_Q5_K && dev->opt.i8_min_m == 0 && mmq_i8_covers(w, qs))
        return launch_mmq_i8(dev, w, qs, scales, m, y);
    if (!vector_only && m >= 3 && (w->fmt == CANDY_HIP_Q4_K || w->fmt == CANDY_HIP_Q6_K || w->fmt == CANDY_HIP_Q5_K) && mmq_i8_covers(w, qs)) {
        // 3 .. 15 rows: the vector kernels below or one pass of the int8 tile kernel with a 16-row tile, whichever a
        // fit to measurements on this chip says is shorter, in us.  The tile kernel's time hardly depends on m: Q4_K
        // 4096x4096 12.7, 11008x4096 19.6, 4096x11008 19.3, 32000x4096 31.5; Q6_K 10.9, 20.8, 19.0, 38.3, 4096x14336
        // 22.0, 128256x4096 132 (short rows: a few us per super-block).  Q6_K and Q5_K have only the looping vector
        // kernel, which takes 8, 4, 2 or 1 activation rows per launch the longer the weight rows are and costs their
        // padded count: 0.07 us per M values and image with rows of up to 5632 values, 0.105 beyond (Q6_K at 3 / 5 rows:
        // 4096x4096 9.2 / 15.1, 11008x4096 16.8 / 31.5, 4096x11008 22.6 / 33.8, 32000x4096 39.7 / 77.5, 4096x14336
        // 33.8 / 51.2, 128256x4096 151 / 273).
        const bool q6 = w->fmt != CANDY_HIP_Q4_K;
        const double nsb = (double)(w->cols >> 8), mnk = (double)w->rows * (double)w->cols * 1e-6;
        double t_tiles, t_vector;
        if (q6) {
            t_tiles = std::min(3.5 + 2.5 * nsb * (1.0 + mnk / 40.0), 7.0 + 0.24 * mnk);
            const double per_image = (w->cols > 5632 ? 0.105 : 0.07) * mnk;
            t_vector = 0.0;
            for (int64_t left = m; left > 0;) {
                const int nb = looping_rows(left, w->cols);
                t_vector += 4.0 + per_image * nb;
                left -= std::min<int64_t>(left, nb);
            }
        } else {
            const int m_pad = (int)((m + 3) / 4 * 4);
            t_tiles = std::min(3.5 + 2.0 * nsb * (1.0 + mnk / 40.0), 11.0 + 0.16 * mnk);
            t_vector = m < 5 ? 0.0 : 4.0 + (m > 8 ? 2.0 : 0.0) + 0.052 * mnk * m_pad;  // Q4_K, 3 and 4 rows: vector
        }
        const int from = dev->opt.i8_min_m;  // comparison runs: tiles from this batch size on
        if (from ? m >= std::max(from, 3) : t_tiles < t_vector) return launch_mmq_i8(dev, w, qs, scales, m, y);
    }
    switch (w->fmt) {
    case CANDY_HIP_Q4_K: return launch_fmt<UnitQ4K>(dev, w, qs, scales, m, y);
    case CANDY_HIP_Q8_0: return launch_fmt<UnitQ8_0>(dev, w, qs, scales, m, y);
    case CANDY_HIP_Q4_0: return launch_fmt<UnitQ4_0<false>>(dev, w, qs, scales, m, y);
    case CANDY_HIP_Q4_0_GGML: return launch_fmt<UnitQ4_0<true>>(dev, w, qs, scales, m, y);
    case CANDY_HIP_Q6_K: return launch_fmt<UnitQ6K>(dev, w, qs, scales, m, y);
    case CANDY_HIP_Q4_1: return launch_fmt<UnitQ4_1<false>>(dev, w, qs, scales, m, y);
    case CANDY_HIP_Q4_1_GGML: return launch_fmt<UnitQ4_1<true>>(dev, w, qs, scales, m, y);
    case CANDY_HIP_Q5_0: return launch_fmt<UnitQ5<false>>(dev, w, qs, scales, m, y);
    case CANDY_HIP_Q5_1: return launch_fmt<UnitQ5<true>>(dev, w, qs, scales, m, y);
    case CANDY_HIP_Q2_K: return launch_fmt<UnitQ2K>(dev, w, qs, scales, m, y);
    case CANDY_HIP_Q3_K: return launch_fmt<UnitQ3K>(dev, w, qs, scales, m, y);
    case CANDY_HIP_Q5_K: return launch_fmt<UnitQ5K>(dev, w, qs, scales, m, y);
    case CANDY_HIP_Q8_K: return fail(CANDY_HIP_ERR_UNSUPPORTED, "Q8_K weights only dequantize (the reference has no vec-dot for them)");
    default: return fail(CANDY_HIP_ERR_INVALID, "unknown quantized format %d", w->fmt);
    }
}

// Scratch of the allocation-free entry point: the quantized activations of one call (planar quants, then scales).
// One copy per GPU for the life of the process; every call on a GPU shares it.
constexpr size_t NOALLOC_SCRATCH_BYTES = size_t(1) << 20;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];

int noalloc_scratch_init(candy_hip_device *dev) {
    // The array's name is only a handle on the host: the address kernels may use is this GPU's, asked for here.
    void *p = nullptr;
    CANDY_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    CANDY_REQUIRE(p && ((uintptr_t)p & 255) == 0, "scratch array is not where it was declared to be");
    dev->noalloc_scratch = p;
    return CANDY_HIP_OK;
}

int mmq_min_m(const candy_hip_device *dev) { return dev->opt.mmq_min_m < 16 ? 16 : dev->opt.mmq_min_m; }

int launch_contract(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales,
                    int64_t m, float *y, const _Float16 *xh_ready, const float *res) {
    if (m < mmq_min_m(dev)) {
        CANDY_REQUIRE(res != y, "internal: in-place residual needs the fused epilogue");
        if (int rc = launch_matvec(dev, w, qs, scales, m, y)) return rc;
        return res ? candy_hip_add(dev, res, y, m * w->rows, y) : CANDY_HIP_OK;
    }
    ActWorkspace extra;
    if (int rc = act_workspace(dev, m, w->cols, false, &extra)) return rc;
    return launch_mmq(dev, w, qs, scales, m, y, extra.half_ws, xh_ready, res);
}

}  // namespace candy

using namespace candy;

extern "C" {

static int qmatmul_check(candy_hip_device *dev, const candy_hip_qtensor *w, int64_t m, float *dev_y) {
    CANDY_REQUIRE(w, "rhs qtensor is nil");
    CANDY_REQUIRE(dev && w->dev == dev, "rhs storage must live on the same HIP device");
    CANDY_REQUIRE(m >= 0, "invalid matrix dimensions");
    CANDY_REQUIRE(m == 0 || dev_y, "output is nil");
    return CANDY_HIP_OK;
}

static int contract(candy_hip_device *dev, const candy_hip_qtensor *w, const ActWorkspace &a, int64_t m, float *y) {
    return m < mmq_min_m(dev) ? launch_matvec(dev, w, a.qs, a.scales, m, y)
                               : launch_mmq(dev, w, a.qs, a.scales, m, y, a.half_ws, nullptr, nullptr, dev->opt.f16_api_min_m);
}

// f32 in -> f32 out.  One row against a big Q4_K weight is ONE launch (the row is quantized in the contraction's
// prologue, once per compute unit); everything else quantizes into the workspace first.  Same quants either way.
static int qmatmul_f32(candy_hip_device *dev, const candy_hip_qtensor *w, const float *dev_x, int64_t m, float *dev_y,
                       const ActWorkspace &a) {
    if (m == 1) {
        WideLaunch Wd;
        Wd.n = 1; Wd.w[0] = w; Wd.y[0] = dev_y; Wd.x = dev_x;
        const int rc = launch_matvec_wide(dev, Wd);
        if (rc != CANDY_HIP_ERR_UNSUPPORTED) return rc;
    }
    if (a.mmv_ws && mmv_covers(w, m) && !matvec_even_covers(w, m)) return launch_mmv(dev, w, dev_x, nullptr, m, dev_y, a.mmv_ws);
    if (a.half_ws && m >= mmq_min_m(dev) && !dev->opt.mmq_fp16_only && mmq_f16_big_covers(w, m, dev->opt.f16_api_min_m)) {
        // the fp16 tiles read d * q as fp16: the quantizer writes that image directly (one launch, no int8 copy)
        if (int rc = launch_quantize_q8(dev, dev_x, m, w->cols, nullptr, nullptr, nullptr, (_Float16 *)a.half_ws)) return rc;
        return launch_mmq(dev, w, nullptr, nullptr, m, dev_y, a.half_ws, (const _Float16 *)a.half_ws, nullptr,
                          dev->opt.f16_api_min_m);
    }
    if (int rc = launch_quantize_q8(dev, dev_x, m, w->cols, a.qs, a.scales, nullptr)) return rc;
    return contract(dev, w, a, m, dev_y);
}

int candy_hip_qmatmul(candy_hip_device *dev, const candy_hip_qtensor *w, const float *dev_x, int64_t m, float *dev_y) {
    if (int rc = qmatmul_check(dev, w, m, dev_y)) return rc;
    if (m == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(dev_x, "lhs is nil");
    CANDY_REQUIRE(((uintptr_t)dev_x & 15) == 0, "lhs must be 16-byte aligned");
    if (int rc = use_device(dev)) return rc;
    ActWorkspace a;
    if (int rc = act_workspace(dev, m, w->cols, true, &a)) return rc;
    return qmatmul_f32(dev, w, dev_x, m, dev_y, a);
}

int candy_hip_qmatmul_noalloc(candy_hip_device *dev, const candy_hip_qtensor *w, const float *dev_x, int64_t m,
                              float *dev_y) {
    if (int rc = qmatmul_check(dev, w, m, dev_y)) return rc;
    if (m == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(dev_x, "lhs is nil");
    CANDY_REQUIRE(((uintptr_t)dev_x & 15) == 0, "lhs must be 16-byte aligned");
    CANDY_REQUIRE(m <= 15, "the allocation-free contraction takes 1 .. 15 activation rows, got %lld", (long long)m);
    const size_t q_bytes = ((size_t)(m * w->cols) + 255) & ~(size_t)255;
    const size_t s_bytes = ((size_t)(m * (w->cols >> 5)) * sizeof(Q8Scale) + 255) & ~(size_t)255;
    CANDY_REQUIRE(q_bytes + s_bytes <= NOALLOC_SCRATCH_BYTES,
                  "%lld x %lld activations need %zu bytes of scratch, the allocation-free contraction has %zu",
                  (long long)m, (long long)w->cols, q_bytes + s_bytes, NOALLOC_SCRATCH_BYTES);
    CANDY_REQUIRE(dev->noalloc_scratch, "device handle has no scratch address");
    if (int rc = use_device(dev)) return rc;
    int8_t *qs = (int8_t *)dev->noalloc_scratch;  // the address hipGetSymbolAddress gave for this GPU, never the array's name
    Q8Scale *scales = (Q8Scale *)((uint8_t *)dev->noalloc_scratch + q_bytes);
    if (int rc = launch_quantize_q8(dev, dev_x, m, w->cols, qs, scales, nullptr)) return rc;
    return launch_matvec(dev, w, qs, scales, m, dev_y, /*vector_only=*/true);
}

int candy_hip_qmatmul_q8(candy_hip_device *dev, const candy_hip_qtensor *w, const void *dev_x_q8_0, int64_t m,
                         float *dev_y) {
    if (int rc = qmatmul_check(dev, w, m, dev_y)) return rc;
    if (m == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(dev_x_q8_0, "lhs is nil");
    CANDY_REQUIRE(((uintptr_t)dev_x_q8_0 & 1) == 0, "lhs blocks must be 2-byte aligned");
    if (int rc = use_device(dev)) return rc;
    ActWorkspace a;
    if (int rc = act_workspace(dev, m, w->cols, true, &a)) return rc;
    if (a.mmv_ws && mmv_covers(w, m) && !matvec_even_covers(w, m)) return launch_mmv(dev, w, nullptr, dev_x_q8_0, m, dev_y, a.mmv_ws);
    if (int rc = launch_q8_blocks_to_planar(dev, dev_x_q8_0, m * (w->cols >> 5), a.qs, a.scales)) return rc;
    return contract(dev, w, a, m, dev_y);
}

int candy_hip_qact_create(candy_hip_device *dev, int64_t max_m, int64_t max_cols, candy_hip_qact **out) {
    CANDY_REQUIRE(out, "out is nil");
    *out = nullptr;
    CANDY_REQUIRE(max_m > 0 && max_cols > 0 && max_cols % 32 == 0, "invalid capacity %lld x %lld", (long long)max_m,
                  (long long)max_cols);
    if (int rc = use_device(dev)) return rc;
    candy_hip_qact *a = new candy_hip_qact();
    a->dev = dev;
    a->max_m = max_m;
    a->max_cols = max_cols;
    void *q = nullptr, *s = nullptr;
    int rc = candy_hip_alloc(dev, (size_t)(max_m * max_cols), &q);
    if (!rc) rc = candy_hip_alloc(dev, (size_t)(max_m * (max_cols >> 5)) * sizeof(Q8Scale), &s);
    if (rc) {
        if (q) (void)candy_hip_free(dev, q);
        delete a;
        return rc;
    }
    a->qs = (int8_t *)q;
    a->scales = (Q8Scale *)s;
    *out = a;
    return CANDY_HIP_OK;
}

int candy_hip_qact_free(candy_hip_qact *a) {
    if (!a) return CANDY_HIP_OK;
    int rc = candy_hip_free(a->dev, a->qs);
    int rc2 = candy_hip_free(a->dev, a->scales);
    delete a;
    return rc ? rc : rc2;
}

int candy_hip_qact_quantize(candy_hip_qact *a, const float *dev_x, int64_t m, int64_t cols) {
    CANDY_REQUIRE(a, "qact is nil");
    CANDY_REQUIRE(m > 0 && cols > 0, "invalid matrix dimensions");
    CANDY_REQUIRE(cols % 32 == 0, "cols %lld is not a multiple of the block size 32", (long long)cols);
    CANDY_REQUIRE(m * cols <= a->max_m * a->max_cols, "%lld x %lld exceeds the capacity %lld x %lld", (long long)m,
                  (long long)cols, (long long)a->max_m, (long long)a->max_cols);
    CANDY_REQUIRE(dev_x && ((uintptr_t)dev_x & 15) == 0, "input must be non-nil and 16-byte aligned");
    if (int rc = use_device(a->dev)) return rc;
    a->m = m;
    a->cols = cols;
    return launch_quantize_q8(a->dev, dev_x, m, cols, a->qs, a->scales, nullptr);
}

int candy_hip_qmatmul_qact(candy_hip_device *dev, const candy_hip_qtensor *w, const candy_hip_qact *a, float *dev_y) {
    CANDY_REQUIRE(w && a, "nil argument");
    CANDY_REQUIRE(dev && w->dev == dev && a->dev == dev, "operands must live on the same HIP device");
    CANDY_REQUIRE(a->m > 0, "activations have not been quantized yet");
    CANDY_REQUIRE(a->cols == w->cols, "activation width %lld does not match the weight's contraction dim %lld",
                  (long long)a->cols, (long long)w->cols);
    CANDY_REQUIRE(dev_y, "output is nil");
    if (int rc = use_device(dev)) return rc;
    return launch_contract(dev, w, a->qs, a->scales, a->m, dev_y);
}

int candy_hip_qmatmul_sweep(candy_hip_device *dev, const candy_hip_qtensor *const *ws, int n_ws, const float *dev_x,
                            int64_t m, float *dev_y, int iters, int quantize_each, float *elapsed_ms) {
    CANDY_REQUIRE(dev && ws && n_ws > 0 && dev_x && dev_y && elapsed_ms, "nil argument");
    CANDY_REQUIRE(m > 0 && iters > 0, "invalid iteration count or batch");
    for (int i = 0; i < n_ws; ++i) {
        CANDY_REQUIRE(ws[i] && ws[i]->dev == dev, "weight %d is nil or on another device", i);
        CANDY_REQUIRE(ws[i]->cols == ws[0]->cols && ws[i]->rows == ws[0]->rows, "weights must share one shape");
    }
    CANDY_REQUIRE(((uintptr_t)dev_x & 15) == 0, "lhs must be 16-byte aligned");
    if (int rc = use_device(dev)) return rc;
    const int64_t K = ws[0]->cols;
    ActWorkspace a;
    if (int rc = act_workspace(dev, m, K, true, &a)) return rc;
    if (int rc = launch_quantize_q8(dev, dev_x, m, K, a.qs, a.scales, nullptr)) return rc;
    CANDY_HIP_TRY(hipEventRecord(dev->ev_start, dev->stream));
    for (int i = 0; i < iters; ++i) {
        if (quantize_each) {
            if (int rc = qmatmul_f32(dev, ws[i % n_ws], dev_x, m, dev_y, a)) return rc;
        } else if (int rc = contract(dev, ws[i % n_ws], a, m, dev_y)) return rc;
    }
    CANDY_HIP_TRY(hipEventRecord(dev->ev_stop, dev->stream));
    CANDY_HIP_TRY(hipEventSynchronize(dev->ev_stop));
    CANDY_HIP_TRY(hipEventElapsedTime(elapsed_ms, dev->ev_start, dev->ev_stop));
    return CANDY_HIP_OK;
}


// Batch-1 contractions with the fixed part of a launch amortised or hidden: `group` weights of the rotation that share
// the quantized activation row go out as ONE launch (the q / k / v mechanism), and with n_streams = 2 the launches
// alternate between the handle's stream and a second one, so that one launch's start overlaps the other's tail.
// A figure for independent contractions; the serialized single launch is what candy_hip_qmatmul_sweep times.
int candy_hip_qmatmul_sustained_sweep(candy_hip_device *dev, const candy_hip_qtensor *const *ws, int n_ws, int group,
                                      int n_streams, const float *dev_x, float *dev_y, int iters, float *elapsed_ms) {
    CANDY_REQUIRE(dev && ws && n_ws > 0 && dev_x && dev_y && elapsed_ms, "nil argument");
    CANDY_REQUIRE(group >= 1 && group <= 3 && n_ws >= group, "1 .. 3 weights per launch, no more than the rotation holds");
    CANDY_REQUIRE(n_streams == 1 || n_streams == 2, "one or two streams");
    CANDY_REQUIRE(iters > 0, "invalid iteration count");
    for (int i = 0; i < n_ws; ++i) {
        CANDY_REQUIRE(ws[i] && ws[i]->dev == dev, "weight %d is nil or on another device", i);
        CANDY_REQUIRE(ws[i]->cols == ws[0]->cols && ws[i]->rows == ws[0]->rows && ws[i]->fmt == ws[0]->fmt,
                      "weights must share one shape and format");
    }
    CANDY_REQUIRE(format_has_batch1_kernel(ws[0]->fmt), "format has no batch-1 kernel");
    CANDY_REQUIRE(((uintptr_t)dev_x & 15) == 0, "lhs must be 16-byte aligned");
    if (int rc = use_device(dev)) return rc;
    const int64_t K = ws[0]->cols, N = ws[0]->rows;
    ActWorkspace a;
    if (int rc = act_workspace(dev, 1, K, true, &a)) return rc;
    if (int rc = launch_quantize_q8(dev, dev_x, 1, K, a.qs, a.scales, nullptr)) return rc;
    hipStream_t main_stream = dev->stream, second = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
    int rc = CANDY_HIP_OK;
    hipError_t e = hipSuccess;
    if (n_streams == 2) {
        e = hipStreamCreateWithFlags(&second, hipStreamNonBlocking);  // default priority
        if (e == hipSuccess) e = hipEventCreateWithFlags(&fork, hipEventDisableTiming);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&join, hipEventDisableTiming);
    }
    const int groups = n_ws / group;  // whole groups of the rotation
    if (e == hipSuccess) e = hipEventRecord(dev->ev_start, main_stream);
    if (e == hipSuccess && second) {
        e = hipEventRecord(fork, main_stream);
        if (e == hipSuccess) e = hipStreamWaitEvent(second, fork, 0);
    }
    for (int i = 0; i < iters && e == hipSuccess && rc == CANDY_HIP_OK; ++i) {
        const int lane = second ? (i & 1) : 0;
        const candy_hip_qtensor *const *w = ws + (size_t)(i % groups) * group;
        float *ys[3];
        for (int j = 0; j < group; ++j) ys[j] = dev_y + ((size_t)lane * group + j) * N;  // each stream its own outputs
        dev->stream = lane ? second : main_stream;
        rc = launch_matvec_multi(dev, w, ys, nullptr, group, a.qs, a.scales);
    }
    dev->stream = main_stream;
    if (e == hipSuccess && second) {
        e = hipEventRecord(join, second);
        if (e == hipSuccess) e = hipStreamWaitEvent(main_stream, join, 0);
    }
    if (e == hipSuccess) e = hipEventRecord(dev->ev_stop, main_stream);
    if (e == hipSuccess) e = hipEventSynchronize(dev->ev_stop);
    if (second) (void)hipStreamSynchronize(second);
    if (e == hipSuccess) e = hipEventElapsedTime(elapsed_ms, dev->ev_start, dev->ev_stop);
    if (fork) (void)hipEventDestroy(fork);
    if (join) (void)hipEventDestroy(join);
    if (second) (void)hipStreamDestroy(second);
    if (rc) return rc;
    if (e != hipSuccess) return fail(CANDY_HIP_ERR_HIP, "sustained sweep failed: %s", hipGetErrorString(e));
    return CANDY_HIP_OK;
}

}  // extern "C"
