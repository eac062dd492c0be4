// Batched (m >= 16) quantized matmul on the matrix cores: y[m, N] = x[m, K] . W^T.
//
// Replaces the tiled dp4a kernel mul_mat_q (tensor/internal/cuda/kernels/quantized.cu:455-578,
// tile loaders / vec-dots :4116-4205, :2266-2294) with a design for gfx950:
//   * the activations, already quantized to Q8_0 (the contraction candy defines), are expanded
//     once per call to fp16 (d_x * q_x, exact in f32, one rounding to fp16);
//   * each workgroup owns a BN x BM output tile and walks K in steps of BK: 256 threads pull the
//     raw weight blocks of the step into registers (original block layout, no repacking),
//     dequantize them to fp16 exactly as the dequantize kernels do ((d*sc)*q - dmin*m in f32, one
//     rounding to fp16) into an LDS tile, the fp16 activations go into a second LDS tile, and four
//     wavefronts run v_mfma_f32_16x16x32_f16 over the two tiles with f32 accumulators;
//   * the next step's global loads are issued right after the barrier, so they fly under the
//     MFMAs of the current step.
// Per-32 scale products are folded into the fp16 operands, so the inner loop has no per-block
// rescale (with integer MFMA every K=32 step would need a rank-1 f32 rescale of the whole
// accumulator tile on the VALU, several times the MFMA time).
// Rounding: fp16 operands carry 2^-12 relative rounding each; the f32 result stays within a few
// 1e-4 (max-norm) of the CPU contraction, inside the 1e-3 bar (tests/test_gpu_mmq.py).
// Bound: HBM (weights read once) for m = 16..32, MFMA for m >= 128.
#include "blocks.h"
#include "formats_more.h"
#include "internal.h"

namespace candy {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half8 to_half8(const float (&v)[8]) {
    half8 h;
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = (_Float16)v[i];  // v_cvt_f16_f32: round to nearest even
    return h;
}

// ------------------------------------------------------------------ per-format 32-weight tasks
// load(): raw bytes of the 32 consecutive weights kb*32 .. kb*32+31 of one row -> registers.
// dequant(): those registers -> 32 fp16 values (4 x half8), same arithmetic as quant.hip.

struct MmqQ4K {
    struct Raw { u32x4 hdr, q0, q1; };
    __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)(K >> 8) * 144; }
    __device__ static __forceinline__ void load(const uint8_t *row, int kb, Raw &r) {
        const uint8_t *blk = row + (size_t)(kb >> 3) * 144;
        r.hdr = *(const u32x4 *)blk;
        const u32x4 *q = (const u32x4 *)(blk + 16 + ((kb & 7) >> 1) * 32);
        r.q0 = q[0];
        r.q1 = q[1];
    }
    __device__ static __forceinline__ void dequant(const Raw &r, int kb, half8 (&out)[4]) {
        const int t = kb & 7;
        uint32_t sc2, m2;
        q4k_scale_min_pair(r.hdr.y, r.hdr.z, r.hdr.w, t >> 1, sc2, m2);
        const int bsh = (t & 1) * 8;
        const float d1 = half_bits_to_float((uint16_t)(r.hdr.x & 0xFFFF)) * (float)((sc2 >> bsh) & 0xFF);
        const float m1 = half_bits_to_float((uint16_t)(r.hdr.x >> 16)) * (float)((m2 >> bsh) & 0xFF);
        const int nsh = (t & 1) * 4;
        const uint32_t qw[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float v[8];
#pragma unroll
            for (int l = 0; l < 8; ++l) {
                const uint32_t q = (qw[2 * g + (l >> 2)] >> (8 * (l & 3) + nsh)) & 0xF;
                v[l] = d1 * (float)q - m1;
            }
            out[g] = to_half8(v);
        }
    }
};

struct MmqQ8_0 {
    struct Raw { u32x4 q0, q1; uint16_t d; };
    __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)(K >> 5) * 34; }
    __device__ static __forceinline__ void load(const uint8_t *row, int kb, Raw &r) {
        const BlockQ8_0 *blk = (const BlockQ8_0 *)row + kb;
        r.d = blk->d;
        r.q0 = *(const u32x4_a2 *)(blk->qs);
        r.q1 = *(const u32x4_a2 *)(blk->qs + 16);
    }
    __device__ static __forceinline__ void dequant(const Raw &r, int, half8 (&out)[4]) {
        const float d = half_bits_to_float(r.d);
        const uint32_t qw[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float v[8];
#pragma unroll
            for (int l = 0; l < 8; ++l) v[l] = d * (float)(int8_t)((qw[2 * g + (l >> 2)] >> (8 * (l & 3))) & 0xFF);
            out[g] = to_half8(v);
        }
    }
};

template <bool GGML_ORDER>
struct MmqQ4_0 {
    struct Raw { u32x4 q; uint16_t d; };
    __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)(K >> 5) * 18; }
    __device__ static __forceinline__ void load(const uint8_t *row, int kb, Raw &r) {
        const BlockQ4_0 *blk = (const BlockQ4_0 *)row + kb;
        r.d = blk->d;
        r.q = *(const u32x4_a2 *)(blk->qs);
    }
    __device__ static __forceinline__ void dequant(const Raw &r, int, half8 (&out)[4]) {
        const float d = half_bits_to_float(r.d);
        const uint32_t qw[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float v[8];
#pragma unroll
            for (int l = 0; l < 8; ++l) {
                const int e = 8 * g + l;  // element of the block
                // candy CPU order: e = 2j (low nibble of byte j), 2j+1 (high); ggml: e = j, j+16
                const int byte = GGML_ORDER ? (e & 15) : (e >> 1);
                const int high = GGML_ORDER ? (e >> 4) : (e & 1);
                const uint32_t q = (qw[byte >> 2] >> (8 * (byte & 3) + 4 * high)) & 0xF;
                v[l] = d * ((float)q - 8.0f);
            }
            out[g] = to_half8(v);
        }
    }
};

struct MmqQ6K {
    struct Raw { u32x4 ql0, ql1, qh0, qh1; uint16_t sc, d; };
    __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)(K >> 8) * 210; }
    __device__ static __forceinline__ void load(const uint8_t *row, int kb, Raw &r) {
        const BlockQ6K *blk = (const BlockQ6K *)row + (kb >> 3);
        const int ip = (kb >> 2) & 1, qd = kb & 3;
        const uint8_t *ql = blk->ql + 64 * ip + 32 * (qd & 1);
        r.ql0 = *(const u32x4_a2 *)ql;
        r.ql1 = *(const u32x4_a2 *)(ql + 16);
        r.qh0 = *(const u32x4_a2 *)(blk->qh + 32 * ip);
        r.qh1 = *(const u32x4_a2 *)(blk->qh + 32 * ip + 16);
        r.sc = *(const uint16_t *)(blk->scales + 8 * ip + 2 * qd);
        r.d = blk->d;
    }
    __device__ static __forceinline__ void dequant(const Raw &r, int kb, half8 (&out)[4]) {
        const int qd = kb & 3;
        const float d = half_bits_to_float(r.d);
        const float s0 = d * (float)(int8_t)(r.sc & 0xFF), s1 = d * (float)(int8_t)(r.sc >> 8);
        const uint32_t ql[8] = {r.ql0.x, r.ql0.y, r.ql0.z, r.ql0.w, r.ql1.x, r.ql1.y, r.ql1.z, r.ql1.w};
        const uint32_t qh[8] = {r.qh0.x, r.qh0.y, r.qh0.z, r.qh0.w, r.qh1.x, r.qh1.y, r.qh1.z, r.qh1.w};
        const int nsh = qd >= 2 ? 4 : 0;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float v[8];
#pragma unroll
            for (int l = 0; l < 8; ++l) {
                const int il = 8 * g + l;
                const uint32_t lo4 = (ql[il >> 2] >> (8 * (il & 3) + nsh)) & 0xF;
                const uint32_t hi2 = (qh[il >> 2] >> (8 * (il & 3) + 2 * qd)) & 3;
                v[l] = (g < 2 ? s0 : s1) * (float)((int)(lo4 | (hi2 << 4)) - 32);
            }
            out[g] = to_half8(v);
        }
    }
};

// The other formats (formats_more.h): the 32 weights are dequantized with the format's own quad() straight from
// memory when the tile is built (no raw-byte stage ahead of it: these formats are not on the headline path).
template <class F>
struct MmqMore {
    struct Raw { const uint8_t *blk; int j0; };
    __device__ static __forceinline__ size_t row_bytes(int K) { return (size_t)(K / F::ELEMS) * F::BYTES; }
    __device__ static __forceinline__ void load(const uint8_t *row, int kb, Raw &r) {
        const int e = kb * 32;
        r.blk = row + (size_t)(e / F::ELEMS) * F::BYTES;
        r.j0 = (e % F::ELEMS) >> 2;
    }
    __device__ static __forceinline__ void dequant(const Raw &r, int, half8 (&out)[4]) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float4 a = F::quad(r.blk, r.j0 + 2 * g), b = F::quad(r.blk, r.j0 + 2 * g + 1);
            const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
            out[g] = to_half8(v);
        }
    }
};

// ------------------------------------------------------------------ activation expansion
// planar Q8_0 -> fp16 [m_pad, K]; rows m..m_pad-1 are zero so the tile kernel needs no row guard.  FRAG: in the
// fragment order of xh_index4 (what the big fp16 tiles read) instead of row by row (k_mmq below).
template <bool FRAG>
__global__ __launch_bounds__(256) void k_q8_to_half(const int8_t *__restrict__ qs, const Q8Scale *__restrict__ sc,
                                                    int64_t m, int64_t m_pad, int64_t K, half8 *__restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one 8-value run
    const int64_t per_row = K >> 3;
    if (i >= m_pad * per_row) return;
    const int64_t row = i / per_row, c = i - row * per_row;
    half8 h = {0, 0, 0, 0, 0, 0, 0, 0};
    if (row < m) {
        const uint2 q = *(const uint2 *)(qs + row * K + c * 8);
        const float d = sc[row * (K >> 5) + (c >> 2)].d;
        float v[8];
#pragma unroll
        for (int l = 0; l < 8; ++l) v[l] = d * (float)(int8_t)(((l < 4 ? q.x : q.y) >> (8 * (l & 3))) & 0xFF);
        h = to_half8(v);
    }
    out[FRAG ? xh_index4(row, 2 * c, K) >> 1 : i] = h;
}

// ------------------------------------------------------------------ tile kernel
template <class F, int BN, int BM, int BK>
__global__ __launch_bounds__(256) void k_mmq(const uint8_t *__restrict__ W, const _Float16 *__restrict__ xh,
                                             float *__restrict__ y, int N, int M, int K) {
    constexpr int LD = BK + 8;                 // LDS row pitch in halves (16 bytes of padding)
    constexpr int KB = BK / 32;                // 32-weight tasks per row per step
    constexpr int TPT = BN * KB / 256;         // weight tasks per thread
    constexpr int XCH = BM * BK / 8;           // 16-byte activation chunks per step
    constexpr int XPT = (XCH + 255) / 256;
    constexpr int TN = BN / 64, TM = BM / 16;  // 16x16 tiles per wavefront
    static_assert(BN * KB % 256 == 0 && TN >= 1 && TM >= 1, "tile shape");
    __shared__ __align__(16) _Float16 sA[BN * LD];
    __shared__ __align__(16) _Float16 sB[BM * LD];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM;
    const size_t rb = F::row_bytes(K);
    const int steps = K / BK;

    typename F::Raw raw[TPT];
    u32x4 xr[XPT];
    auto gload = [&](int ks) {
#pragma unroll
        for (int i = 0; i < TPT; ++i) {
            const int task = tid + i * 256, row = task / KB, kb = task % KB;
            F::load(W + (size_t)min(n0 + row, N - 1) * rb, ks * KB + kb, raw[i]);
        }
#pragma unroll
        for (int i = 0; i < XPT; ++i) {
            const int c = min(tid + i * 256, XCH - 1), r = c / (BK / 8), kc = c % (BK / 8);
            xr[i] = *(const u32x4 *)(xh + (size_t)(m0 + r) * K + (size_t)ks * BK + kc * 8);
        }
    };
    gload(0);

    float4v acc[TN][TM];
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b) acc[a][b] = float4v{0.f, 0.f, 0.f, 0.f};

    for (int ks = 0; ks < steps; ++ks) {
#pragma unroll
        for (int i = 0; i < TPT; ++i) {
            const int task = tid + i * 256, row = task / KB, kb = task % KB;
            half8 h[4];
            F::dequant(raw[i], ks * KB + kb, h);
            half8 *dst = (half8 *)&sA[row * LD + kb * 32];
#pragma unroll
            for (int g = 0; g < 4; ++g) dst[g] = h[g];
        }
#pragma unroll
        for (int i = 0; i < XPT; ++i) {
            const int c = tid + i * 256;
            if (XCH % 256 == 0 || c < XCH) *(u32x4 *)&sB[(c / (BK / 8)) * LD + (c % (BK / 8)) * 8] = xr[i];
        }
        __syncthreads();
        if (ks + 1 < steps) gload(ks + 1);
#pragma unroll
        for (int kk = 0; kk < KB; ++kk) {
            half8 a[TN], b[TM];
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
                a[tn] = *(const half8 *)&sA[(wave * (BN / 4) + tn * 16 + (lane & 15)) * LD + kk * 32 + (lane >> 4) * 8];
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
                b[tm] = *(const half8 *)&sB[(tm * 16 + (lane & 15)) * LD + kk * 32 + (lane >> 4) * 8];
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int tm = 0; tm < TM; ++tm)
                    acc[tn][tm] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[tn], b[tm], acc[tn][tm], 0, 0, 0);
        }
        __syncthreads();
    }

    // C layout of the 16x16 tile: lane holds column (lane & 15) = activation row, rows 4*(lane>>4)..+3 =
    // four consecutive weight rows -> one 16-byte store into y[m, n..n+3]
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
            const int m = m0 + tm * 16 + (lane & 15);
            const int n = n0 + wave * (BN / 4) + tn * 16 + 4 * (lane >> 4);
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

template <class F, int BN, int BM, int BK>
static int launch_tile(candy_hip_device *dev, const candy_hip_qtensor *w, const _Float16 *xh, int64_t m, float *y) {
    const int N = (int)w->rows, K = (int)w->cols;
    dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((m + BM - 1) / BM));
    hipLaunchKernelGGL((k_mmq<F, BN, BM, BK>), grid, dim3(256), 0, dev->stream, (const uint8_t *)w->data, xh, y, N,
                       (int)m, K);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

template <class F>
static int launch_fmt(candy_hip_device *dev, const candy_hip_qtensor *w, const _Float16 *xh, int64_t m, float *y) {
    if (m <= 16 && w->cols % 128 == 0) return launch_tile<F, 64, 16, 128>(dev, w, xh, m, y);
    if (m <= 32 && w->cols % 128 == 0) return launch_tile<F, 64, 32, 128>(dev, w, xh, m, y);
    if (m <= 64) return launch_tile<F, 128, 64, 64>(dev, w, xh, m, y);
    return launch_tile<F, 128, 128, 64>(dev, w, xh, m, y);
}

int64_t mmq_m_pad(int64_t m) { return (m + 255) / 256 * 256; }  // a multiple of every tile height

static int mmq_dispatch(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales,
                        int64_t m, float *y, void *half_ws, const _Float16 *xh_ready, const float *res, bool *res_done,
                        int f16_min_m);

static bool force_old_fp16(const candy_hip_device *dev) { return dev->opt.mmq_fp16_only != 0; }

bool mmq_fuses_residual(const candy_hip_qtensor *w, int64_t m) {
    return m >= mmq_min_m(w->dev) && w->cols % 64 == 0 && !force_old_fp16(w->dev) && mmq_f16_big_covers(w, m);
}

int launch_mmq(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales, int64_t m,
               float *y, void *half_ws, const _Float16 *xh_ready, const float *res, int f16_min_m) {
    CANDY_REQUIRE(res != y || mmq_fuses_residual(w, m), "internal: in-place residual needs the fused epilogue");
    bool res_done = false;
    if (int rc = mmq_dispatch(dev, w, qs, scales, m, y, half_ws, xh_ready, res, &res_done, f16_min_m)) return rc;
    if (res && !res_done) return candy_hip_add(dev, res, y, m * w->rows, y);  // kernels without a residual epilogue
    return CANDY_HIP_OK;
}

static int mmq_dispatch(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales,
                        int64_t m, float *y, void *half_ws, const _Float16 *xh_ready, const float *res, bool *res_done,
                        int f16_min_m) {
    const int64_t K = w->cols;
    CANDY_REQUIRE(w->rows <= 0x7FFFFFFF && K <= 0x7FFFFFFF && m <= 0x7FFFFFFF, "matrix too large");
    if (K % 64 != 0) return launch_matvec(dev, w, qs, scales, m, y);  // odd block counts: small-batch kernel in slices
    if (w->fmt == CANDY_HIP_Q8_K) return launch_matvec(dev, w, qs, scales, m, y);  // reports that Q8_K does not contract
    // prompt-sized batches of Q4_K: big fp16 tiles (the integer kernel is bound by its per-sub-block rescale there);
    // smaller batches of Q4_K and Q6_K: int8 matrix cores (exact); the fp16 tile kernel below serves the rest
    const bool force_fp16 = force_old_fp16(dev);
    const bool big = !force_fp16 && mmq_f16_big_covers(w, m, f16_min_m);
    // the 32-value formats (Q8_0, Q4_0, Q4_1, Q5_0, Q5_1) on the int8 tiles as well, except where the 128 x 128 fp16 tiles below fill the chip (many weight rows and
    // a prompt-sized batch; measured: 11008x4096 m = 256 127 against 123 us, m = 512 228 against 134; 32000x4096
    // m = 128 165 against 129; but 4096x11008 m = 128 68 against 313, 4096x4096 m = 512 88 against 121)
    const bool is_q32 = w->fmt == CANDY_HIP_Q8_0 || w->fmt == CANDY_HIP_Q4_0 || w->fmt == CANDY_HIP_Q4_0_GGML ||
                        w->fmt == CANDY_HIP_Q4_1 || w->fmt == CANDY_HIP_Q4_1_GGML || w->fmt == CANDY_HIP_Q5_0 || w->fmt == CANDY_HIP_Q5_1;
    const bool q8_wide = is_q32 && w->rows >= 8192 && (double)m * (double)w->rows >= 2.8e6;
    if (!force_fp16 && !big && !q8_wide && mmq_i8_covers(w, qs)) return launch_mmq_i8(dev, w, qs, scales, m, y);
    if (big && xh_ready) {
        *res_done = res != nullptr;
        return launch_mmq_f16_big(dev, w, xh_ready, m, y, res);
    }
    CANDY_REQUIRE(half_ws, "internal: no workspace for the fp16 activations");
    const int64_t m_pad = mmq_m_pad(m);
    const int64_t runs = m_pad * (K >> 3);
    hipLaunchKernelGGL(big ? k_q8_to_half<true> : k_q8_to_half<false>, dim3((unsigned)((runs + 255) / 256)), dim3(256), 0,
                       dev->stream, qs, scales, m, m_pad, K, (half8 *)half_ws);
    CANDY_LAUNCH_CHECK();
    const _Float16 *xh = (const _Float16 *)half_ws;
    if (big) {
        *res_done = res != nullptr;
        return launch_mmq_f16_big(dev, w, xh, m, y, res);
    }
    switch (w->fmt) {
    case CANDY_HIP_Q4_K: return launch_fmt<MmqQ4K>(dev, w, xh, m, y);
    case CANDY_HIP_Q8_0: return launch_fmt<MmqQ8_0>(dev, w, xh, m, y);
    case CANDY_HIP_Q4_0: return launch_fmt<MmqQ4_0<false>>(dev, w, xh, m, y);
    case CANDY_HIP_Q4_0_GGML: return launch_fmt<MmqQ4_0<true>>(dev, w, xh, m, y);
    case CANDY_HIP_Q6_K: return launch_fmt<MmqQ6K>(dev, w, xh, m, y);
    case CANDY_HIP_Q4_1: return launch_fmt<MmqMore<FmtQ4_1<false>>>(dev, w, xh, m, y);
    case CANDY_HIP_Q4_1_GGML: return launch_fmt<MmqMore<FmtQ4_1<true>>>(dev, w, xh, m, y);
    case CANDY_HIP_Q5_0: return launch_fmt<MmqMore<FmtQ5<false>>>(dev, w, xh, m, y);
    case CANDY_HIP_Q5_1: return launch_fmt<MmqMore<FmtQ5<true>>>(dev, w, xh, m, y);
    case CANDY_HIP_Q2_K: return launch_fmt<MmqMore<FmtQ2K>>(dev, w, xh, m, y);
    case CANDY_HIP_Q3_K: return launch_fmt<MmqMore<FmtQ3K>>(dev, w, xh, m, y);
    case CANDY_HIP_Q5_K: return launch_fmt<MmqMore<FmtQ5K>>(dev, w, xh, m, y);
    default: return fail(CANDY_HIP_ERR_INVALID, "unknown quantized format %d", w->fmt);
    }
}

}  // namespace candy
