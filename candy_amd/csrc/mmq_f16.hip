// Large-batch (m >= 256) Q4_K matmul on the fp16 matrix cores: y[m, N] = x[m, K] . W^T.
//
// Replaces mul_mat_q / load_tiles_q4_K (tensor/internal/cuda/kernels/quantized.cu:455-578,
// :4116-4205) for prompt-sized batches.  With hundreds of activation rows the contraction is a dense
// GEMM, and the per-sub-block rescale that keeps the integer kernel exact costs several times the
// matrix-core time; here the scales are folded into the operands instead:
//   * weights are dequantized exactly as dequantize_block_q4_K does (quantized.cu:1008-1041:
//     (d*sc)*q - dmin*m, evaluated in f32) and rounded once to fp16;
//   * activations are the Q8_0 values d_x * q_x (exact in f32) rounded once to fp16;
//   * products accumulate in f32 (v_mfma_f32_16x16x32_f16).
// Both roundings are 2^-12 relative per element; the result stays a few 1e-4 (max-norm) from the
// CPU contraction, inside the 1e-3 bar.
//
// Tiling: a workgroup owns BN weight rows x BM activation rows and walks K in steps of 64 (one
// 32-byte nibble group of a super-block = two sub-blocks).  Every thread dequantizes 16 weights per
// step (8 bytes of nibbles: 8 low + 8 high) into an LDS tile, the fp16 activations go into a second
// LDS tile, both double-buffered so one barrier per step suffices, and the next step's global
// loads are issued before the current step's MFMAs.  Each wavefront owns a (BN/WN) x (BM/WM)
// sub-tile; LDS rows are padded to 144 bytes so that the 16-byte operand reads of a wavefront
// spread over all banks.  Workgroups are numbered so that those sharing an XCD (and its L2) work
// on neighbouring weight tiles of the same activation tile.
#include <cstdlib>

#include "blocks.h"
#include "internal.h"

namespace candy {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int BIG_BK = 64;
constexpr int BIG_PITCH = BIG_BK + 8;  // halves per LDS row (144 bytes)

template <int BN, int BM, int WN, int WM>
__global__ __launch_bounds__(WN * WM * 64) void k_mmq_q4k_f16(const uint8_t *__restrict__ W,
                                                              const _Float16 *__restrict__ xh,
                                                              float *__restrict__ y, int N, int M, int K, int n_tiles,
                                                              int m_tiles) {
    constexpr int T = WN * WM * 64;
    constexpr int TN = BN / WN / 16, TM = BM / WM / 16;
    constexpr int ATK = BN * 4 / T;   // quarter-row dequantization tasks per thread per step
    constexpr int BCH = BM * 8 / T;   // 16-byte activation chunks per thread per step
    static_assert(BN * 4 % T == 0 && BM * 8 % T == 0 && TN >= 1 && TM >= 1, "tile shape");
    extern __shared__ __align__(16) uint8_t smem_raw[];
    _Float16 *sA = (_Float16 *)smem_raw;               // [2][BN][PITCH]
    _Float16 *sB = sA + 2 * BN * BIG_PITCH;            // [2][BM][PITCH]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave % WN, wm = wave / WN;

    // tile numbering: the hardware deals workgroups round-robin to the 8 XCDs; give each XCD a
    // contiguous run of weight tiles inside one activation tile
    int v = blockIdx.x;
    const int total = n_tiles * m_tiles;
    if ((total & 7) == 0) v = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
    const int mt = v / n_tiles, nt = v - mt * n_tiles;
    const int n0 = nt * BN, m0 = mt * BM;

    const size_t rb = (size_t)(K >> 8) * 144;
    const int steps = K / BIG_BK;

    // Register pipeline.  Weights: the 16-byte header and this thread's four 8-byte nibble runs (one per
    // 64-value group) of a whole super-block are requested one super-block (four steps) ahead, far
    // enough for HBM.  Activations (L2-resident): requested two steps ahead.
    // Task (row, quarter c) of step g dequantizes bytes 8c..8c+7 of group g: 8 low + 8 high nibbles.
    u32x4 hdr[2][ATK];
    u32x2 qs[2][ATK][4];
    u32x4 xr[2][BCH];
    auto gload_a = [&](int sb, int slot) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < ATK; ++i) {
            const int task = tid + i * T, row = task >> 2, c = task & 3;
            const uint8_t *blk = W + (size_t)min(n0 + row, N - 1) * rb + (size_t)sb * 144;
            hdr[slot][i] = *(const u32x4 *)blk;
#pragma unroll
            for (int g = 0; g < 4; ++g) qs[slot][i][g] = *(const u32x2 *)(blk + 16 + g * 32 + c * 8);
        }
    };
    auto gload_b = [&](int ks, int slot) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < BCH; ++i) {
            const int ch = tid + i * T, r = ch >> 3, kc = ch & 7;
            xr[slot][i] = *(const u32x4 *)(xh + (size_t)(m0 + r) * K + (size_t)ks * BIG_BK + kc * 8);
        }
    };
    auto stage = [&](int g, int aslot, int bslot, int buf) __attribute__((always_inline)) {
        _Float16 *a = sA + buf * BN * BIG_PITCH;
        _Float16 *b = sB + buf * BM * BIG_PITCH;
#pragma unroll
        for (int i = 0; i < ATK; ++i) {
            const int task = tid + i * T, row = task >> 2, c = task & 3;
            const u32x4 h = hdr[aslot][i];
            const u32x2 q = qs[aslot][i][g];
            uint32_t sc2, m2;
            q4k_scale_min_pair(h.y, h.z, h.w, g, sc2, m2);
            const float d = half_bits_to_float((uint16_t)(h.x & 0xFFFF));
            const float dmin = half_bits_to_float((uint16_t)(h.x >> 16));
            const float d_lo = d * (float)(sc2 & 0xFF), d_hi = d * (float)((sc2 >> 8) & 0xFF);
            const float m_lo = dmin * (float)(m2 & 0xFF), m_hi = dmin * (float)((m2 >> 8) & 0xFF);
            half8 lo, hi;
#pragma unroll
            for (int l = 0; l < 8; ++l) {
                const uint32_t byte = ((l < 4 ? q.x : q.y) >> (8 * (l & 3))) & 0xFF;
                lo[l] = (_Float16)(d_lo * (float)(byte & 0xF) - m_lo);
                hi[l] = (_Float16)(d_hi * (float)(byte >> 4) - m_hi);
            }
            *(half8 *)&a[row * BIG_PITCH + c * 8] = lo;
            *(half8 *)&a[row * BIG_PITCH + 32 + c * 8] = hi;
        }
#pragma unroll
        for (int i = 0; i < BCH; ++i) {
            const int ch = tid + i * T, r = ch >> 3, kc = ch & 7;
            *(u32x4 *)&b[r * BIG_PITCH + kc * 8] = xr[bslot][i];
        }
    };

    float4v acc[TN][TM];
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b) acc[a][b] = float4v{0.f, 0.f, 0.f, 0.f};

    auto compute = [&](int buf) __attribute__((always_inline)) {
        const _Float16 *a = sA + buf * BN * BIG_PITCH + (wn * (BN / WN) + (lane & 15)) * BIG_PITCH + (lane >> 4) * 8;
        const _Float16 *b = sB + buf * BM * BIG_PITCH + (wm * (BM / WM) + (lane & 15)) * BIG_PITCH + (lane >> 4) * 8;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            half8 af[TN], bf[TM];
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) af[tn] = *(const half8 *)&a[tn * 16 * BIG_PITCH + kk * 32];
#pragma unroll
            for (int tm = 0; tm < TM; ++tm) bf[tm] = *(const half8 *)&b[tm * 16 * BIG_PITCH + kk * 32];
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int tm = 0; tm < TM; ++tm)
                    acc[tn][tm] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[tn], bf[tm], acc[tn][tm], 0, 0, 0);
        }
    };

    // Step ks = 4*sb + g computes from LDS buffer (ks & 1) and, meanwhile, stages step ks+1 into the
    // other buffer.  Staging step 4*sb+4 (g == 3) is the first use of super-block sb+1, which was
    // requested when super-block sb was first used.  Super-blocks alternate between the two register
    // slots, so the loop body covers two of them.
    const int n_sb = K >> 8;
    gload_a(0, 0);
    gload_b(0, 0);
    gload_b(1, 1);
    if (n_sb > 1) gload_a(1, 1);
    stage(0, 0, 0, 0);
    gload_b(2, 0);
    __syncthreads();
    for (int sb2 = 0; sb2 < n_sb; sb2 += 2) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int sb = sb2 + half;
            if (sb >= n_sb) break;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                // One straight-line block per step (loads past the end are clamped to valid addresses and
                // the last step stages a buffer nobody reads).
                const int ks = sb * 4 + g;
                compute(g & 1);
                // (g + 1) & 1 is both the activation slot and the LDS buffer of step ks + 1
                if (g < 3) stage(g + 1, half, (g + 1) & 1, (g + 1) & 1);
                else stage(0, half ^ 1, 0, 0);
                gload_b(min(ks + 3, steps - 1), (g + 1) & 1);
                if (g == 3) gload_a(min(sb + 2, n_sb - 1), half);
                __syncthreads();
            }
        }
    }

    // C layout of a 16x16 tile: lane holds activation row (lane & 15) and weight rows 4*(lane>>4)..+3
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            const int m = m0 + wm * (BM / WM) + tm * 16 + (lane & 15);
            const int n = n0 + wn * (BN / WN) + tn * 16 + 4 * (lane >> 4);
            if (m >= M) continue;
            float *dst = y + (size_t)m * N + n;
            if (n + 3 < N && (N & 3) == 0) {
                *(float4 *)dst = make_float4(acc[tn][tm][0], acc[tn][tm][1], acc[tn][tm][2], acc[tn][tm][3]);
            } else {
#pragma unroll
                for (int l = 0; l < 4; ++l)
                    if (n + l < N) dst[l] = acc[tn][tm][l];
            }
        }
}

template <int BN, int BM, int WN, int WM>
static int launch_big(candy_hip_device *dev, const candy_hip_qtensor *w, const _Float16 *xh, int64_t m, float *y) {
    const int N = (int)w->rows, K = (int)w->cols;
    const int n_tiles = (N + BN - 1) / BN, m_tiles = (int)((m + BM - 1) / BM);
    constexpr size_t smem = (size_t)2 * (BN + BM) * BIG_PITCH * sizeof(_Float16);
    CANDY_HIP_TRY(hipFuncSetAttribute((const void *)k_mmq_q4k_f16<BN, BM, WN, WM>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL((k_mmq_q4k_f16<BN, BM, WN, WM>), dim3((unsigned)(n_tiles * m_tiles)), dim3(WN * WM * 64), smem,
                       dev->stream, (const uint8_t *)w->data, xh, y, N, (int)m, K, n_tiles, m_tiles);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

bool mmq_f16_big_covers(const candy_hip_qtensor *w, int64_t m) {
    static const int min_m = getenv("CANDY_HIP_MMQ_BIG_MIN_M") ? atoi(getenv("CANDY_HIP_MMQ_BIG_MIN_M")) : 256;
    return w->fmt == CANDY_HIP_Q4_K && m >= min_m && w->cols % 256 == 0 && ((uintptr_t)w->data & 15) == 0;
}

// xh: fp16 activations [mmq_m_pad(m)][K], rows past m zero.
int launch_mmq_f16_big(candy_hip_device *dev, const candy_hip_qtensor *w, const _Float16 *xh, int64_t m, float *y) {
    return launch_big<128, 256, 2, 4>(dev, w, xh, m, y);
}

}  // namespace candy
