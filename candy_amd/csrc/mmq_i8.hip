// Batched (m >= 16) Q4_K matmul on the integer matrix cores, exact like the matvec:
// y[m, N] = x[m, K] . W^T with x quantized to Q8_0.
//
// mul_mat_q + vec_dot_q4_K_q8_1_impl_mmq (tensor/internal/cuda/kernels/quantized.cu:455-578,
// :2266-2294) tile the contraction for dp4a; here every 32-value sub-block is one
// v_mfma_i32_16x16x32_i8 (16 weight rows x 16 activation rows), and the per-sub-block scales are
// applied to the int32 tile exactly as the batch-1 vec-dot does (quantized.cu:2239-2263):
//   sumf_d += d8 * float(dot * sc);  sumf_m += d8 * float(bsum * m);  y += d * sumf_d - dmin * sumf_m
// with d and dmin folded into the per-sub-block factors, so the result matches the CPU contraction
// to f32 rounding (no fp16 operand rounding). (Running the min term as a small f32 MFMA product
// instead was measured slower: the kernel is bound by the sum of matrix and vector issue.)
//
// Work split: a wavefront owns 16 weight rows and all BM = 16*TM activation rows of the
// workgroup; the four wavefronts of a workgroup share the activation tile in LDS.
//   * weights are fetched a stage (up to four super-blocks, 1024 values) ahead as 16-byte chunks
//     that run along the rows, so every wavefront load covers whole cache lines; the stage is then
//     parked in the wavefront's own LDS slice, from where each lane picks 8 bytes of nibbles per
//     64-value group in the A-operand layout (row = lane%16, 8 consecutive k per lane);
//   * the 6-bit scales are unpacked once per (row, pair) by the lane that owns that row in the
//     A layout and handed through LDS to the lanes that own the row in the C layout
//     (4 consecutive weight rows per lane);
//   * activations: 256 int8 per row per super-block plus {d, d*bsum} per block, loaded one
//     super-block ahead into registers and parked in LDS between two barriers.
// The rescale costs 16 VALU instructions per 16x16x32 tile (convert, multiply and two fused
// multiply-adds per result register), which is what bounds the large-m rate.
#include "blocks.h"
#include "internal.h"

namespace candy {

typedef int int4v __attribute__((ext_vector_type(4)));

template <int TM>
__global__ __launch_bounds__(256) void k_mmq_q4k_i8(const uint8_t *__restrict__ W, const int8_t *__restrict__ xq,
                                                    const Q8Scale *__restrict__ xs, float *__restrict__ y, int N,
                                                    int M, int K) {
    constexpr int BM = 16 * TM;
    constexpr int XROW = 272;                              // LDS pitch of an activation row: 256 quants + 16 (bank spread)
    constexpr int STG = TM <= 2 ? 4 : (TM == 4 ? 2 : 1);   // super-blocks per stage: deep prefetch where m is small
    constexpr int XSC = (BM * 8 + 255) / 256;              // activation scales per thread per super-block
    __shared__ __align__(16) int8_t s_xq[BM * XROW];
    __shared__ __align__(16) float2 s_xs[BM * 8];     // {d, d * bsum} per (row, block)
    constexpr int WPITCH = STG * 144 + (STG == 1 ? 32 : 16);  // odd multiple of 16 bytes: conflict-free 8-byte picks
    __shared__ __align__(16) uint8_t s_w[4][16 * WPITCH];   // per wavefront: the current stage's weight rows
    __shared__ __align__(16) uint8_t s_sc[4][16 * 8];      // per wavefront: scale / min bytes [row][sub-block]
    __shared__ __align__(16) uint8_t s_mn[4][16 * 8];
    __shared__ __align__(16) float2 s_dd[4][16];           // {d, dmin} per row

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int j = lane & 15, c = lane >> 4;
    const int n0 = blockIdx.x * 64 + wave * 16, m0 = blockIdx.y * BM;
    const int nsb = K >> 8;
    const size_t rb = (size_t)nsb * 144;

    // weights of one stage: 16 rows x STG blocks, fetched as whole 16-byte chunks that run along the
    // rows (full cache lines per wavefront load), kept in registers while in flight, then parked in
    // the wavefront's own LDS slice from where the lanes pick their A-operand bytes
    constexpr int CPR = 9 * STG;                       // 16-byte chunks per row per stage
    constexpr int WCH = (16 * CPR + 63) / 64;          // chunks per lane
    u32x4 wr[WCH];
    auto load_stage = [&](int s0) {
#pragma unroll
        for (int i = 0; i < WCH; ++i) {
            const int q = min(lane + 64 * i, 16 * CPR - 1), row = q / CPR, col = q % CPR;
            const int sb = min(s0 + col / 9, nsb - 1);
            wr[i] = *(const u32x4 *)(W + (size_t)min(n0 + row, N - 1) * rb + (size_t)sb * 144 + (col % 9) * 16);
        }
    };
    auto park_stage = [&]() {
#pragma unroll
        for (int i = 0; i < WCH; ++i) {
            const int q = lane + 64 * i, row = q / CPR, col = q % CPR;
            if ((16 * CPR) % 64 == 0 || q < 16 * CPR) *(u32x4 *)&s_w[wave][row * WPITCH + col * 16] = wr[i];
        }
    };
    // activations of one super-block: registers first (loaded a super-block ahead), then LDS
    u32x4 xr[TM];
    float xsd[XSC];
    int xsb[XSC];
    auto load_x = [&](int s) {
        const int sb = min(s, nsb - 1);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int q = tid + i * 256, row = q >> 4, col = q & 15;
            xr[i] = *(const u32x4 *)(xq + (size_t)min(m0 + row, M - 1) * K + (size_t)sb * 256 + col * 16);
        }
#pragma unroll
        for (int i = 0; i < XSC; ++i) {
            const int e = min(tid + i * 256, BM * 8 - 1), row = e >> 3, t = e & 7;
            const Q8Scale v = xs[(size_t)min(m0 + row, M - 1) * (K >> 5) + sb * 8 + t];
            xsd[i] = v.d;
            xsb[i] = v.bsum;
        }
    };

    load_x(0);
    load_stage(0);

    float acc[TM][4];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[a][i] = 0.0f;

    for (int s0 = 0; s0 < nsb; s0 += STG) {
        // the slice is private to the wavefront, whose LDS operations complete in order: no barrier
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        park_stage();
        load_stage(s0 + STG);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const uint8_t *wl = &s_w[wave][j * WPITCH];  // the row this lane feeds into the A operand
#pragma unroll
        for (int b = 0; b < STG; ++b) {
            const int s = s0 + b;
            if (s < nsb) {  // uniform
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    const int q = tid + i * 256, row = q >> 4, col = q & 15;
                    *(u32x4 *)&s_xq[row * XROW + col * 16] = xr[i];
                }
#pragma unroll
                for (int i = 0; i < XSC; ++i) {
                    const int e = tid + i * 256;
                    if (BM * 8 % 256 == 0 || e < BM * 8) s_xs[e] = make_float2(xsd[i], xsd[i] * (float)xsb[i]);
                }
                // scales: lane (row j, pair c) unpacks one pair and parks it for the C-layout owners
                {
                    const u32x4 h = *(const u32x4 *)(wl + 144 * b);
                    uint32_t sc2, m2;
                    q4k_scale_min_pair(h.y, h.z, h.w, c, sc2, m2);
                    *(uint16_t *)&s_sc[wave][j * 8 + 2 * c] = (uint16_t)sc2;
                    *(uint16_t *)&s_mn[wave][j * 8 + 2 * c] = (uint16_t)m2;
                    if (c == 0)
                        s_dd[wave][j] = make_float2(half_bits_to_float((uint16_t)(h.x & 0xFFFF)),
                                                    half_bits_to_float((uint16_t)(h.x >> 16)));
                }
                __syncthreads();
                load_x(s + 1);  // the next super-block's activations fly under this one's MFMAs
                // my four C rows are 4c .. 4c+3: 8 scale bytes, 8 min bytes, {d, dmin} each
                const u32x4 scA = *(const u32x4 *)&s_sc[wave][32 * c], scB = *(const u32x4 *)&s_sc[wave][32 * c + 16];
                const u32x4 mnA = *(const u32x4 *)&s_mn[wave][32 * c], mnB = *(const u32x4 *)&s_mn[wave][32 * c + 16];
                const float4 dd0 = *(const float4 *)&s_dd[wave][4 * c], dd1 = *(const float4 *)&s_dd[wave][4 * c + 2];
                const uint32_t scw[8] = {scA.x, scA.y, scA.z, scA.w, scB.x, scB.y, scB.z, scB.w};
                const uint32_t mnw[8] = {mnA.x, mnA.y, mnA.z, mnA.w, mnB.x, mnB.y, mnB.z, mnB.w};
                const float dw[4] = {dd0.x, dd0.z, dd1.x, dd1.z}, dmn[4] = {dd0.y, dd0.w, dd1.y, dd1.w};
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const u32x2 qa = *(const u32x2 *)(wl + 144 * b + 16 + 32 * (t >> 1) + 8 * c);
                    const int sh = (t & 1) * 4;
                    const uint32_t lo = (qa.x >> sh) & 0x0F0F0F0Fu, hi = (qa.y >> sh) & 0x0F0F0F0Fu;
                    const long afrag = (long)(((uint64_t)hi << 32) | lo);
                    float dsc[4], dmf[4];  // d * sc and dmin * m of my four weight rows for this sub-block
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        dsc[i] = dw[i] * (float)((scw[2 * i + (t >> 2)] >> (8 * (t & 3))) & 0xFF);
                        dmf[i] = dmn[i] * (float)((mnw[2 * i + (t >> 2)] >> (8 * (t & 3))) & 0xFF);
                    }
                    int4v d[TM];  // all tiles of the sub-block first, so the matrix pipe runs under the rescale
#pragma unroll
                    for (int a = 0; a < TM; ++a) {
                        const long bfrag = *(const long *)&s_xq[(16 * a + j) * XROW + 32 * t + 8 * c];
                        d[a] = __builtin_amdgcn_mfma_i32_16x16x32_i8(afrag, bfrag, int4v{0, 0, 0, 0}, 0, 0, 0);
                    }
#pragma unroll
                    for (int a = 0; a < TM; ++a) {
                        const float2 sx = s_xs[(16 * a + j) * 8 + t];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            acc[a][i] += sx.x * ((float)d[a][i] * dsc[i]);  // d8 * d * sc * dot
                            acc[a][i] -= dmf[i] * sx.y;                     // d8 * bsum * dmin * m
                        }
                    }
                }
                __syncthreads();  // the tile and the scale slots are rewritten next
            }
        }
    }

    // C layout: lane holds activation row j of each m-tile and weight rows 4c .. 4c+3
#pragma unroll
    for (int a = 0; a < TM; ++a) {
        const int m = m0 + 16 * a + j, n = n0 + 4 * c;
        if (m >= M) continue;
        float *dst = y + (size_t)m * N + n;
        if (n + 3 < N && (N & 3) == 0) {
            *(float4 *)dst = make_float4(acc[a][0], acc[a][1], acc[a][2], acc[a][3]);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (n + i < N) dst[i] = acc[a][i];
        }
    }
}

int launch_mmq_q4k_i8(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales,
                      int64_t m, float *y) {
    const int N = (int)w->rows, K = (int)w->cols, M = (int)m;
    const unsigned gx = (unsigned)((N + 63) / 64);
#define CANDY_MMQ_I8(TMV)                                                                                         \
    hipLaunchKernelGGL((k_mmq_q4k_i8<TMV>), dim3(gx, (unsigned)((M + 16 * TMV - 1) / (16 * TMV))), dim3(256), 0, \
                       dev->stream, (const uint8_t *)w->data, qs, scales, y, N, M, K)
    // the largest tile height that still leaves about 1.5 wavefronts per SIMD: a wavefront walks the
    // whole contraction on its own, so a grid below that leaves load latency exposed
    const int64_t strips = (N + 15) / 16, want = 1536;
    if (M > 32 && strips * ((M + 63) / 64) >= want) CANDY_MMQ_I8(4);
    else if (M > 16 && strips * ((M + 31) / 32) >= want) CANDY_MMQ_I8(2);
    else CANDY_MMQ_I8(1);
#undef CANDY_MMQ_I8
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

}  // namespace candy
