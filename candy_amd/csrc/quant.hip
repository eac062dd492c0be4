// Activation quantization to Q8_0 and block dequantization. Both are bit-exact with candy's
// definitions: every product in the dequantizers is exact in f32 (fp16 scale times small
// integers), so instruction selection cannot change a result.
#include "blocks.h"
#include "formats_more.h"
#include "internal.h"

namespace candy {

// ------------------------------------------------------------------ quantize_q8_0
// quantize_q8_1 (quantized.cu:3521-3558) without its `sum` half: per 32 values
//   amax = max|x|, d = amax / 127 (IEEE f32 division), q = amax == 0 ? 0 : roundf(x / d),
// the stored scale is fp16(d) while q uses the unrounded d.
// One lane owns 4 consecutive values; the 8 lanes of a block reduce with cross-lane xor.
__global__ __launch_bounds__(256) void k_quantize_q8_0(const float4 *__restrict__ x, int64_t n4, int64_t row_n4,
                                                       uint32_t *__restrict__ qs, Q8Scale *__restrict__ scales,
                                                       uint8_t *__restrict__ blocks, half4v *__restrict__ xh) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool active = i < n4;  // n4 is a multiple of 8, so a block's 8 lanes agree
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (active) v = x[i];
    __half h;
    int s;
    const uint32_t packed = quantize_q8_lane4(v, h, s);
    if (!active) return;
    const int64_t b = i >> 3;
    const int part = (int)(i & 7);
    if (qs) qs[i] = packed;
    if (xh) xh[xh_index4(i / row_n4, i % row_n4, 4 * row_n4)] = q8_lane4_to_half(packed, h);
    if (scales && part == 0) {
        Q8Scale sc;
        sc.d = __half2float(h);
        sc.bsum = s;
        scales[b] = sc;
    }
    if (blocks) {
        uint8_t *blk = blocks + b * 34;  // 2-byte aligned only
        if (part == 0) *(uint16_t *)blk = __half_as_ushort(h);
        uint16_t *p = (uint16_t *)(blk + 2 + part * 4);
        p[0] = (uint16_t)(packed & 0xFFFFu);
        p[1] = (uint16_t)(packed >> 16);
    }
}

// Q8_0 blocks (34 B) -> planar quants + scales, one lane per block.
__global__ __launch_bounds__(256) void k_q8_blocks_to_planar(const BlockQ8_0 *__restrict__ blocks, int64_t nb,
                                                             uint32_t *__restrict__ qs, Q8Scale *__restrict__ scales) {
    const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= nb) return;
    const BlockQ8_0 *blk = blocks + b;
    const u32x4 a = *(const u32x4_a2 *)(blk->qs);
    const u32x4 c = *(const u32x4_a2 *)(blk->qs + 16);
    int s = 0;
    const uint32_t ones = 0x01010101u;
    s = dot4_i8(a.x, ones, s); s = dot4_i8(a.y, ones, s); s = dot4_i8(a.z, ones, s); s = dot4_i8(a.w, ones, s);
    s = dot4_i8(c.x, ones, s); s = dot4_i8(c.y, ones, s); s = dot4_i8(c.z, ones, s); s = dot4_i8(c.w, ones, s);
    u32x4 *out = (u32x4 *)(qs + b * 8);
    out[0] = a;
    out[1] = c;
    Q8Scale sc;
    sc.d = half_bits_to_float(blk->d);
    sc.bsum = s;
    scales[b] = sc;
}

int launch_quantize_q8(candy_hip_device *dev, const float *x, int64_t rows, int64_t cols, int8_t *qs, Q8Scale *scales,
                       void *blocks, _Float16 *xh) {
    const int64_t n4 = rows * cols / 4;
    if (n4 == 0) return CANDY_HIP_OK;
    const int64_t grid = (n4 + 255) / 256;
    CANDY_REQUIRE(grid <= 0x7FFFFFFF, "activation too large");
    hipLaunchKernelGGL(k_quantize_q8_0, dim3((unsigned)grid), dim3(256), 0, dev->stream, (const float4 *)x, n4, cols / 4,
                       (uint32_t *)qs, scales, (uint8_t *)blocks, (half4v *)xh);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int launch_q8_blocks_to_planar(candy_hip_device *dev, const void *blocks, int64_t nb, int8_t *qs, Q8Scale *scales) {
    if (nb == 0) return CANDY_HIP_OK;
    const int64_t grid = (nb + 255) / 256;
    CANDY_REQUIRE(grid <= 0x7FFFFFFF, "activation too large");
    hipLaunchKernelGGL(k_q8_blocks_to_planar, dim3((unsigned)grid), dim3(256), 0, dev->stream,
                       (const BlockQ8_0 *)blocks, nb, (uint32_t *)qs, scales);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

// ------------------------------------------------------------------ dequantize
// Each lane writes whole float4 vectors so the (dominant) output stream is coalesced.
// With `ids` set the kernels gather rows: output block b comes from row ids[b / bpr] of a
// table with bpr blocks per row (embedding lookup, indexing.go:8-26 on a quantized table).
// An id outside [0, n_rows) cannot stop the kernel the way the CPU loop's bounds check stops the program: the
// block is read from row 0 instead (a valid address) and the device handle's fault word is raised, which the
// next synchronising call reports.
struct Gather {
    const int64_t *ids;  // null: no gather
    int64_t bpr;         // blocks per table row
    int64_t n_rows;      // rows of the table
    int *fault;          // host-visible word of the device handle
};
__device__ __forceinline__ int64_t src_block(int64_t b, const Gather &g) {
    if (!g.ids) return b;
    int64_t row = g.ids[b / g.bpr];
    if (row < 0 || row >= g.n_rows) {
        *g.fault = 1;
        row = 0;
    }
    return row * g.bpr + b % g.bpr;
}

// Q4_0 and Q8_0: 8 lanes per 32-value block, one float4 each, and DQ_ROUNDS such rounds per lane 1 KB of output
// apart, so that every store instruction of a wavefront fills whole lines (a lane that wrote two float4 32 bytes
// apart left every store half-filling its lines: 2.9 TB/s) and the index arithmetic is paid once per four stores
// (one round per lane: Q4_0 48.3, Q8_0 42.3 us for 4096 x 11008).
constexpr int DQ_ROUNDS = 4;
__device__ __forceinline__ int64_t dq_first_chunk() {
    return ((int64_t)blockIdx.x * 256 + (threadIdx.x & ~63)) * DQ_ROUNDS + (threadIdx.x & 63);
}

// quantized.go:85-93: y[2j] = d*(lo(qs[j])-8), y[2j+1] = d*(hi(qs[j])-8).
__global__ __launch_bounds__(256) void k_dequant_q4_0(const BlockQ4_0 *__restrict__ blocks, int64_t nb,
        const Gather gather,
                                                      float4 *__restrict__ y, int ggml_order) {
    const int64_t t0 = dq_first_chunk();
    const int j = (int)(t0 & 7);  // values 4j..4j+3 (the rounds are 64 chunks apart: the same j in each)
    uint32_t word[DQ_ROUNDS], qg[DQ_ROUNDS];
#pragma unroll
    for (int u = 0; u < DQ_ROUNDS; ++u) {
        const int64_t b = min((t0 + 64 * u) >> 3, nb - 1);
        const BlockQ4_0 *blk = blocks + src_block(b, gather);
        // one 4-byte request per lane: bytes 2j .. 2j+3 of the 18-byte block are lane j's two quant bytes in the
        // upper half, and lane 0's lower half is d, which it hands to the other seven lanes of the block (a 2-byte
        // load of d and a 2-byte load of the quants per lane: 52 against 48 us for 4096 x 11008)
        word[u] = *(const u32_a2 *)((const uint8_t *)blk + 2 * j);
        if (ggml_order) qg[u] = *(const u32_a2 *)(blk->qs + 4 * (j & 3)) >> (j >= 4 ? 4 : 0);
    }
#pragma unroll
    for (int u = 0; u < DQ_ROUNDS; ++u) {
        const int64_t t = t0 + 64 * u;
        const float d = half_bits_to_float((uint16_t)(__shfl((int)word[u], (int)(threadIdx.x & 63 & ~7), 64) & 0xFFFF));
        float v[4];
        if (ggml_order) {  // quantized.cu:862-866: low nibbles fill y[0..15], high nibbles y[16..31]; d*q + (-8 d)
            const float dm = -8.0f * d;
#pragma unroll
            for (int l = 0; l < 4; ++l) v[l] = d * (float)((qg[u] >> (8 * l)) & 0xF) + dm;
        } else {  // the two reference forms agree everywhere except the sign of a zero result
            const uint32_t q = word[u] >> 16;
            v[0] = d * ((float)(q & 0xF) - 8.0f);
            v[1] = d * ((float)((q >> 4) & 0xF) - 8.0f);
            v[2] = d * ((float)((q >> 8) & 0xF) - 8.0f);
            v[3] = d * ((float)(q >> 12) - 8.0f);
        }
        if ((t >> 3) < nb) y[t] = make_float4(v[0], v[1], v[2], v[3]);
    }
}

// quantized.go:131-136: y[i] = d*qs[i].
__global__ __launch_bounds__(256) void k_dequant_q8_0(const BlockQ8_0 *__restrict__ blocks, int64_t nb,
        const Gather gather,
                                                      float4 *__restrict__ y) {
    const int64_t t0 = dq_first_chunk();
    const int j = (int)(t0 & 7);
    uint32_t q[DQ_ROUNDS];
    uint16_t dh[DQ_ROUNDS];
#pragma unroll
    for (int u = 0; u < DQ_ROUNDS; ++u) {
        const int64_t b = min((t0 + 64 * u) >> 3, nb - 1);
        const BlockQ8_0 *blk = blocks + src_block(b, gather);
        q[u] = *(const u32_a2 *)(blk->qs + 4 * j);
        dh[u] = blk->d;
    }
#pragma unroll
    for (int u = 0; u < DQ_ROUNDS; ++u) {
        const int64_t t = t0 + 64 * u;
        const float d = half_bits_to_float(dh[u]);
        if ((t >> 3) < nb)
            y[t] = make_float4(d * (float)(int8_t)(q[u] & 0xFF), d * (float)(int8_t)((q[u] >> 8) & 0xFF),
                               d * (float)(int8_t)((q[u] >> 16) & 0xFF), d * (float)(int8_t)(q[u] >> 24));
    }
}

// quantized.cu:1008-1041: group il of 64 values, low nibbles with (sc, m) of sub-block 2il,
// high nibbles with those of 2il+1; y = (d*sc)*q - (dmin*m). 32 lanes per super-block.
__global__ __launch_bounds__(256) void k_dequant_q4_k(const BlockQ4K *__restrict__ blocks, int64_t nb,
        const Gather gather,
                                                      float4 *__restrict__ y) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t b = t >> 5;
    if (b >= nb) return;
    const int il = (int)(t & 31) >> 3;  // 64-value group
    const int ir = (int)(t & 7);        // 4 bytes within the group's 32
    const uint32_t *w = (const uint32_t *)(blocks + src_block(b, gather));  // 144-byte blocks keep 16-byte alignment
    const uint32_t dm = w[0];
    const float dall = half_bits_to_float((uint16_t)(dm & 0xFFFF));
    const float dmin = half_bits_to_float((uint16_t)(dm >> 16));
    uint32_t sc2, m2;
    q4k_scale_min_pair(w[1], w[2], w[3], il, sc2, m2);
    const float d1 = dall * (float)(sc2 & 0xFF), m1 = dmin * (float)(m2 & 0xFF);
    const float d2 = dall * (float)(sc2 >> 8), m2f = dmin * (float)(m2 >> 8);
    const uint32_t q = w[4 + il * 8 + ir];
    float lo[4], hi[4];
#pragma unroll
    for (int l = 0; l < 4; ++l) {
        lo[l] = d1 * (float)((q >> (8 * l)) & 0xF) - m1;
        hi[l] = d2 * (float)((q >> (8 * l + 4)) & 0xF) - m2f;
    }
    float4 *out = y + b * 64 + il * 16 + ir;
    out[0] = make_float4(lo[0], lo[1], lo[2], lo[3]);
    out[8] = make_float4(hi[0], hi[1], hi[2], hi[3]);
}

// quantized.cu:1103-1128. 16 lanes per super-block, each 4 consecutive `il` of one half.
__global__ __launch_bounds__(256) void k_dequant_q6_k(const BlockQ6K *__restrict__ blocks, int64_t nb,
        const Gather gather,
                                                      float4 *__restrict__ y) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t b = t >> 4;
    if (b >= nb) return;
    const int ip = (int)(t & 15) >> 3;
    const int il0 = ((int)(t & 7)) * 4;
    const BlockQ6K *blk = blocks + src_block(b, gather);
    const float d = half_bits_to_float(blk->d);
    const uint32_t ql0 = *(const u32_a2 *)(blk->ql + 64 * ip + il0);
    const uint32_t ql1 = *(const u32_a2 *)(blk->ql + 64 * ip + 32 + il0);
    const uint32_t qh = *(const u32_a2 *)(blk->qh + 32 * ip + il0);
    const int is = 8 * ip + il0 / 16;
    const float s0 = d * (float)blk->scales[is], s1 = d * (float)blk->scales[is + 2];
    const float s2 = d * (float)blk->scales[is + 4], s3 = d * (float)blk->scales[is + 6];
    float o[4][4];
#pragma unroll
    for (int l = 0; l < 4; ++l) {
        const uint32_t a = (ql0 >> (8 * l)) & 0xFF, c = (ql1 >> (8 * l)) & 0xFF, h = (qh >> (8 * l)) & 0xFF;
        o[0][l] = s0 * (float)((int)((a & 0xF) | (((h >> 0) & 3) << 4)) - 32);
        o[1][l] = s1 * (float)((int)((c & 0xF) | (((h >> 2) & 3) << 4)) - 32);
        o[2][l] = s2 * (float)((int)((a >> 4) | (((h >> 4) & 3) << 4)) - 32);
        o[3][l] = s3 * (float)((int)((c >> 4) | (((h >> 6) & 3) << 4)) - 32);
    }
    float4 *out = y + b * 64 + ip * 32 + il0 / 4;
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) out[8 * qd] = make_float4(o[qd][0], o[qd][1], o[qd][2], o[qd][3]);
}

// The other formats: one lane per float4 of output, F::quad gives values 4j .. 4j+3 of a block.
template <class F>
__global__ __launch_bounds__(256) void k_dequant_more(const uint8_t *__restrict__ blocks, int64_t nb,
                                                      const Gather gather, float4 *__restrict__ y) {
    constexpr int LPB = F::ELEMS / 4;
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t b = t / LPB;
    if (b >= nb) return;
    y[t] = F::quad(blocks + src_block(b, gather) * F::BYTES, (int)(t - b * LPB));
}

template <class F>
static int launch_dequant_more(candy_hip_device *dev, const void *blocks, int64_t nb, const Gather &gather, float *out) {
    const int64_t grid = (nb * (F::ELEMS / 4) + 255) / 256;
    CANDY_REQUIRE(grid <= 0x7FFFFFFF, "too many blocks");
    hipLaunchKernelGGL(k_dequant_more<F>, dim3((unsigned)grid), dim3(256), 0, dev->stream, (const uint8_t *)blocks, nb, gather,
                       (float4 *)out);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

// Alignment the block array of a format needs (its widest aligned load).
int block_alignment(int fmt) {
    switch (fmt) {
    case CANDY_HIP_Q4_K:
    case CANDY_HIP_Q5_K: return 16;
    case CANDY_HIP_Q4_1:
    case CANDY_HIP_Q4_1_GGML:
    case CANDY_HIP_Q5_1:
    case CANDY_HIP_Q2_K:
    case CANDY_HIP_Q8_K: return 4;
    default: return 2;
    }
}

}  // namespace candy

using namespace candy;

extern "C" {

static int dequantize_impl(candy_hip_device *dev, int fmt, const void *dev_blocks, int64_t n_blocks,
                           const int64_t *ids, int64_t bpr, int64_t n_rows, float *dev_out) {
    FormatInfo fi = format_info(fmt);
    CANDY_REQUIRE(fi.elems != 0, "unknown quantized format %d", fmt);
    CANDY_REQUIRE(n_blocks >= 0, "negative block count");
    if (n_blocks == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(dev_blocks && dev_out, "nil pointer");
    CANDY_REQUIRE(((uintptr_t)dev_out & 15) == 0, "output must be 16-byte aligned");
    CANDY_REQUIRE(((uintptr_t)dev_blocks & (uintptr_t)(block_alignment(fmt) - 1)) == 0, "blocks are misaligned");
    if (int rc = use_device(dev)) return rc;
    const Gather gather{ids, bpr, n_rows, dev->fault};
    switch (fmt) {
    case CANDY_HIP_Q4_1: return launch_dequant_more<FmtQ4_1<false>>(dev, dev_blocks, n_blocks, gather, dev_out);
    case CANDY_HIP_Q4_1_GGML: return launch_dequant_more<FmtQ4_1<true>>(dev, dev_blocks, n_blocks, gather, dev_out);
    case CANDY_HIP_Q5_0: return launch_dequant_more<FmtQ5<false>>(dev, dev_blocks, n_blocks, gather, dev_out);
    case CANDY_HIP_Q5_1: return launch_dequant_more<FmtQ5<true>>(dev, dev_blocks, n_blocks, gather, dev_out);
    case CANDY_HIP_Q2_K: return launch_dequant_more<FmtQ2K>(dev, dev_blocks, n_blocks, gather, dev_out);
    case CANDY_HIP_Q3_K: return launch_dequant_more<FmtQ3K>(dev, dev_blocks, n_blocks, gather, dev_out);
    case CANDY_HIP_Q5_K: return launch_dequant_more<FmtQ5K>(dev, dev_blocks, n_blocks, gather, dev_out);
    case CANDY_HIP_Q8_K: return launch_dequant_more<FmtQ8K>(dev, dev_blocks, n_blocks, gather, dev_out);
    default: break;
    }
    const int lanes_per_block = fmt == CANDY_HIP_Q4_K ? 32 : fmt == CANDY_HIP_Q6_K ? 16 : 8;
    const int64_t per_wg = lanes_per_block == 8 ? 256 * DQ_ROUNDS : 256;  // chunks (lanes of work) per workgroup
    const int64_t grid = (n_blocks * lanes_per_block + per_wg - 1) / per_wg;
    CANDY_REQUIRE(grid <= 0x7FFFFFFF, "too many blocks");
    dim3 g((unsigned)grid), blk(256);
    switch (fmt) {
    case CANDY_HIP_Q4_0:
    case CANDY_HIP_Q4_0_GGML:
        hipLaunchKernelGGL(k_dequant_q4_0, g, blk, 0, dev->stream, (const BlockQ4_0 *)dev_blocks, n_blocks, gather,
                           (float4 *)dev_out, fmt == CANDY_HIP_Q4_0_GGML ? 1 : 0);
        break;
    case CANDY_HIP_Q8_0:
        hipLaunchKernelGGL(k_dequant_q8_0, g, blk, 0, dev->stream, (const BlockQ8_0 *)dev_blocks, n_blocks, gather,
                           (float4 *)dev_out);
        break;
    case CANDY_HIP_Q4_K:
        hipLaunchKernelGGL(k_dequant_q4_k, g, blk, 0, dev->stream, (const BlockQ4K *)dev_blocks, n_blocks, gather,
                           (float4 *)dev_out);
        break;
    case CANDY_HIP_Q6_K:
        hipLaunchKernelGGL(k_dequant_q6_k, g, blk, 0, dev->stream, (const BlockQ6K *)dev_blocks, n_blocks, gather,
                           (float4 *)dev_out);
        break;
    }
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

int candy_hip_dequantize_blocks(candy_hip_device *dev, int fmt, const void *dev_blocks, int64_t n_blocks,
                                float *dev_out) {
    return dequantize_impl(dev, fmt, dev_blocks, n_blocks, nullptr, 1, 0, dev_out);
}

int candy_hip_qindex_select(candy_hip_device *dev, const candy_hip_qtensor *q, const int64_t *dev_ids, int64_t n_ids,
                            float *out) {
    CANDY_REQUIRE(q, "qtensor is nil");
    CANDY_REQUIRE(q->dev == dev, "qtensor lives on another device");
    CANDY_REQUIRE(n_ids >= 0, "negative id count");
    if (n_ids == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(dev_ids, "ids is nil");
    const int64_t bpr = q->cols / format_info(q->fmt).elems;
    return dequantize_impl(dev, q->fmt, q->data, n_ids * bpr, dev_ids, bpr, q->rows, out);
}

int candy_hip_dequantize(candy_hip_device *dev, const candy_hip_qtensor *q, float *dev_out) {
    CANDY_REQUIRE(q, "qtensor is nil");
    CANDY_REQUIRE(q->dev == dev, "qtensor lives on another device");
    return candy_hip_dequantize_blocks(dev, q->fmt, q->data, q->rows * (q->cols / format_info(q->fmt).elems), dev_out);
}

int candy_hip_quantize_q8_0(candy_hip_device *dev, const float *dev_x, int64_t rows, int64_t cols,
                            void *dev_out_blocks) {
    CANDY_REQUIRE(rows >= 0 && cols >= 0, "invalid matrix dimensions");
    CANDY_REQUIRE(cols % 32 == 0, "cols %lld is not a multiple of the block size 32", (long long)cols);
    if (rows * cols == 0) return CANDY_HIP_OK;
    CANDY_REQUIRE(dev_x && dev_out_blocks, "nil pointer");
    CANDY_REQUIRE(((uintptr_t)dev_x & 15) == 0, "input must be 16-byte aligned");
    CANDY_REQUIRE(((uintptr_t)dev_out_blocks & 1) == 0, "output blocks must be 2-byte aligned");
    if (int rc = use_device(dev)) return rc;
    return launch_quantize_q8(dev, dev_x, rows, cols, nullptr, nullptr, dev_out_blocks);
}

int candy_hip_dequantize_sweep(candy_hip_device *dev, const candy_hip_qtensor *const *ws, int n_ws, float *dev_out,
                               int n_out, int iters, float *elapsed_ms) {
    CANDY_REQUIRE(dev && ws && n_ws > 0 && n_out > 0 && dev_out && elapsed_ms && iters > 0, "nil argument");
    if (int rc = use_device(dev)) return rc;
    CANDY_HIP_TRY(hipEventRecord(dev->ev_start, dev->stream));
    for (int i = 0; i < iters; ++i) {
        const candy_hip_qtensor *w = ws[i % n_ws];
        CANDY_REQUIRE(w, "weight %d is nil", i % n_ws);
        if (int rc = candy_hip_dequantize(dev, w, dev_out + (size_t)(i % n_out) * (size_t)(w->rows * w->cols))) return rc;
    }
    CANDY_HIP_TRY(hipEventRecord(dev->ev_stop, dev->stream));
    CANDY_HIP_TRY(hipEventSynchronize(dev->ev_stop));
    CANDY_HIP_TRY(hipEventElapsedTime(elapsed_ms, dev->ev_start, dev->ev_stop));
    return CANDY_HIP_OK;
}

int candy_hip_quantize_sweep(candy_hip_device *dev, const float *dev_x, int64_t x_stride, int n_x, int64_t rows,
                             int64_t cols, void *dev_out_blocks, int n_out, int iters, float *elapsed_ms) {
    CANDY_REQUIRE(dev && dev_x && dev_out_blocks && elapsed_ms && iters > 0 && n_x > 0 && n_out > 0, "nil argument");
    if (int rc = use_device(dev)) return rc;
    const size_t out_bytes = (size_t)(rows * (cols >> 5)) * sizeof(BlockQ8_0);
    CANDY_HIP_TRY(hipEventRecord(dev->ev_start, dev->stream));
    for (int i = 0; i < iters; ++i)
        if (int rc = candy_hip_quantize_q8_0(dev, dev_x + (int64_t)(i % n_x) * x_stride, rows, cols,
                                             (uint8_t *)dev_out_blocks + (size_t)(i % n_out) * out_bytes))
            return rc;
    CANDY_HIP_TRY(hipEventRecord(dev->ev_stop, dev->stream));
    CANDY_HIP_TRY(hipEventSynchronize(dev->ev_stop));
    CANDY_HIP_TRY(hipEventElapsedTime(elapsed_ms, dev->ev_start, dev->ev_stop));
    return CANDY_HIP_OK;
}

}  // extern "C"
