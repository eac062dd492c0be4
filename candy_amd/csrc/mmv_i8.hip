// Small batches (2 .. 32 activation rows) of Q4_K on the int8 matrix cores, shaped like the batch-1 matvec:
// y[m, N] = x[m, K] . W^T, weights read once, every load of a wavefront in flight before its first dot, no loop.
//
// mul_mat_vec_q<ncols_y> (tensor/internal/cuda/kernels/quantized.cu:2787-2871) serves 1 .. 8 activation rows from
// one pass over the weights with dp4a; here the batch is the 16-wide N side of v_mfma_i32_16x16x32_i8, a 32-value
// sub-block is one instruction, and the scales are applied to the int32 tile exactly as vec_dot_q4_K_q8_1 does
// (quantized.cu:2239-2263): the result differs from the CPU contraction by f32 summation order only.
//
// Work split: a workgroup owns 16 weight rows; its WAVES wavefronts each take SBW consecutive super-blocks of
// those rows (a slice of K), and the slices' partial sums meet in LDS in a fixed order.
//   * the A operand wants lane (row j, k-chunk c), i.e. neighbouring lanes on different rows: loading it that way
//     costs one memory request per lane (measured on this chip: 11.1 us for a 14336 x 4096 matrix against 7.4 us
//     for the same bytes fetched row-contiguously).  So the wavefront fetches its 16 x SBW blocks as consecutive
//     16-byte pieces of each row, parks them in its own LDS slot and reads the operands back in A layout;
//   * the quantized activations are read from a copy the quantizer writes in B-operand order (pack kernel below):
//     one coalesced 16-byte load per lane brings the B operands of two sub-blocks;
//   * d * scale is unpacked by the lane that feeds the row into the A operand and handed through LDS to the lanes
//     that own the row in the C layout; dmin * min meets d8 * sum(q8) in an f32 matrix instruction whose A and B
//     operands are exactly what lane (row j, pair c) and lane (activation row j, pair c) already hold.
#include "blocks.h"
#include "internal.h"

namespace candy {

typedef int int4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void mmv_wave_lds_fence() {
    // orders LDS traffic of one wavefront (its LDS operations complete in order): no barrier needed
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ------------------------------------------------------------------ activations in operand order
// Activation rows come in tiles of 16 (one or two tiles).  Per tile:
// xfrag: [K/256][4][64 lanes][16 bytes]: lane (row r = lane & 15, chunk c = lane >> 4) of pair tp holds values
//        8c .. 8c+7 of sub-blocks 2tp and 2tp+1 of row r.  Rows from m on are zero.
// xd:    [K/256 + 1][16 rows][8 sub-blocks] d;  xm: the same shape, d * sum(q8).  The last block of both is zero.
struct MmvOperands {
    uint8_t *xfrag;
    float *xd, *xm;
    size_t frag_stride, scale_stride;  // bytes / floats from one tile to the next
};
__device__ __forceinline__ size_t mmv_frag_offset(int r, int k) {
    const int sb = k >> 8, t = (k >> 5) & 7, c = (k >> 3) & 3;
    return ((size_t)((sb * 4 + (t >> 1)) * 64 + c * 16 + r)) * 16 + (t & 1) * 8 + (k & 7);
}

// f32 [m, K] -> Q8_0 (quantize_q8_1 without its sum, quantized.cu:3521-3558; the same lane code as the quantize
// kernel, hence the same quants and scales) written in operand order for 16 rows.
// (plain leading arguments: they arrive in registers with the wavefront, no scalar load of the argument block first)
__global__ __launch_bounds__(256) void k_mmv_quantize_pack(const float4 *__restrict__ x, int m, int K, uint8_t *xfrag_,
                                                          float *xd_, float *xm_, size_t frag_stride_,
                                                          size_t scale_stride_) {
    const MmvOperands o = {xfrag_, xd_, xm_, frag_stride_, scale_stride_};
    const int per_row = K >> 2;
    const int i = blockIdx.x * 256 + threadIdx.x;  // 16 * tiles * per_row lanes in all (a multiple of 256)
    const int row = i / per_row, k = (i - row * per_row) * 4;
    const int tile = row >> 4, r = row & 15;
    const float4 v = row < m ? x[(size_t)row * per_row + (k >> 2)] : make_float4(0.f, 0.f, 0.f, 0.f);
    __half h;
    int bsum;
    const uint32_t packed = quantize_q8_lane4(v, h, bsum);
    *(uint32_t *)(o.xfrag + tile * o.frag_stride + mmv_frag_offset(r, k)) = packed;
    if ((k & 31) == 0) {
        const float d = __half2float(h);
        const size_t at = tile * o.scale_stride + ((size_t)(k >> 8) * 16 + r) * 8 + ((k >> 5) & 7);
        o.xd[at] = d;
        o.xm[at] = d * (float)bsum;
        if (k < 256) o.xd[at + (size_t)(K >> 8) * 128] = o.xm[at + (size_t)(K >> 8) * 128] = 0.0f;
    }
}

// Q8_0 blocks [m, K / 32] (34 bytes each) -> the same operand order; one lane per block of each of the 16 rows.
__global__ __launch_bounds__(256) void k_mmv_pack_blocks(const BlockQ8_0 *__restrict__ blocks, int m, int tiles, int K,
                                                        MmvOperands o) {
    const int bpr = K >> 5;
    const int i = blockIdx.x * 256 + threadIdx.x;  // 16 * tiles * bpr lanes in all (a multiple of 128)
    if (i >= 16 * tiles * bpr) return;
    const int row = i / bpr, blk = i - row * bpr, k = blk * 32;
    const int tile = row >> 4, r = row & 15;
    uint8_t *xfrag = o.xfrag + tile * o.frag_stride;
    float *xd = o.xd + tile * o.scale_stride, *xm = o.xm + tile * o.scale_stride;
    u32x4 a = {0u, 0u, 0u, 0u}, c = {0u, 0u, 0u, 0u};
    float d = 0.0f;
    if (row < m) {
        const BlockQ8_0 *src = blocks + (size_t)row * bpr + blk;
        a = *(const u32x4_a2 *)(src->qs);
        c = *(const u32x4_a2 *)(src->qs + 16);
        d = half_bits_to_float(src->d);
    }
    int s = 0;
    const uint32_t ones = 0x01010101u;
    s = dot4_i8(a.x, ones, s); s = dot4_i8(a.y, ones, s); s = dot4_i8(a.z, ones, s); s = dot4_i8(a.w, ones, s);
    s = dot4_i8(c.x, ones, s); s = dot4_i8(c.y, ones, s); s = dot4_i8(c.z, ones, s); s = dot4_i8(c.w, ones, s);
    // values 8 chunk .. 8 chunk + 7 of the block go to lane (r, chunk) of its pair
    *(u32x2 *)(xfrag + mmv_frag_offset(r, k)) = u32x2{a.x, a.y};
    *(u32x2 *)(xfrag + mmv_frag_offset(r, k + 8)) = u32x2{a.z, a.w};
    *(u32x2 *)(xfrag + mmv_frag_offset(r, k + 16)) = u32x2{c.x, c.y};
    *(u32x2 *)(xfrag + mmv_frag_offset(r, k + 24)) = u32x2{c.z, c.w};
    const size_t at = ((size_t)(k >> 8) * 16 + r) * 8 + ((k >> 5) & 7);
    xd[at] = d;
    xm[at] = d * (float)s;
    if (k < 256) xd[at + (size_t)(K >> 8) * 128] = xm[at + (size_t)(K >> 8) * 128] = 0.0f;
}

// ------------------------------------------------------------------ contraction
template <int MT, int STRIPS, int SBW, int WAVES>
struct MmvShape {
    static constexpr int CHUNKS_ROW = 9 * SBW;                 // 16-byte pieces of one row's slice
    static constexpr int ROWS_LD = 64 / CHUNKS_ROW;            // whole rows one load instruction covers
    static constexpr int NLD = (16 + ROWS_LD - 1) / ROWS_LD;   // load instructions per 16-row strip
    static constexpr int PITCH = SBW * 144 + 16;               // LDS pitch of a row's slice (bank spread, 16-byte aligned)
    static constexpr int STAGE_BYTES = 16 * PITCH;
    static constexpr int EX_BYTES = SBW * 8 * 16 * 4;          // d * scale [super-block of the slice][sub-block][row]
    static constexpr int WAVE_LDS = STAGE_BYTES + EX_BYTES;
    static constexpr int OUT = MT * STRIPS * 4;                // output registers of a lane
    static constexpr size_t SMEM = (size_t)WAVES * WAVE_LDS + (size_t)WAVES * OUT * 64 * sizeof(float);
};

// A workgroup owns 16 * STRIPS weight rows.  Each wavefront issues the loads of its K slice for every strip at once,
// then takes the strips in the order their bytes return (loads complete in order): strip s is parked in LDS and
// contracted while strip s+1 is still arriving, and the B operands and activation scales, which depend on the slice
// only, stay in registers for all strips.  MT tiles of 16 activation rows share every A operand.
template <int MT, int STRIPS, int SBW, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void k_mmv_q4k(const uint8_t *__restrict__ W, const uint8_t *xfrag_,
                                                        const float *xd_, const float *xm_, float *__restrict__ y, int N,
                                                        int M, int K, size_t frag_stride_, size_t scale_stride_) {
    // plain leading arguments (13 dwords up to K arrive in registers with the wavefront; the two strides matter to
    // the second activation tile only)
    const MmvOperands o = {(uint8_t *)xfrag_, (float *)xd_, (float *)xm_, frag_stride_, scale_stride_};
    using S = MmvShape<MT, STRIPS, SBW, WAVES>;
    static_assert(S::ROWS_LD >= 1, "a row's slice must fit one load instruction");
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, c = lane >> 4;
    uint8_t *stage = smem + wave * S::WAVE_LDS;                 // [16 rows][PITCH]
    float *s_dsc = (float *)(stage + S::STAGE_BYTES);           // [SBW][8][16]
    float *s_red = (float *)(smem + WAVES * S::WAVE_LDS);       // [WAVES][OUT][64]

    const int nsb = K >> 8;
    const uint32_t rb = (uint32_t)nsb * 144u;
    const int n0 = blockIdx.x * (16 * STRIPS);                  // N is a multiple of 16 * STRIPS (launcher)
    const int sb0 = wave * SBW;
    const int sbc = min(sb0, nsb - 1);                          // slices past the end of K read the last block and add nothing
    const int nvalid = max(min(nsb - sb0, SBW), 0);

    // ---- activation scales and operands of this K slice first (they come from L2 and return first).
    // Wavefront-uniform bases, 32-bit lane offsets: the address arithmetic stays on the scalar unit.
    float4 d8[MT][SBW][2];
    float2 xmv[MT][SBW];
    u32x4 bf[MT][SBW][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const uint8_t *xfrag = o.xfrag + mt * o.frag_stride;
        const float *xd = o.xd + mt * o.scale_stride, *xm = o.xm + mt * o.scale_stride;
        const uint32_t at_d = (uint32_t)j * 32u, at_m = (uint32_t)j * 32u + (uint32_t)c * 8u, at_f = (uint32_t)lane * 16u;
#pragma unroll
        for (int b = 0; b < SBW; ++b) {
            // a slice past the end of K takes its scales from the all-zero block the quantizer appends: it runs the
            // same instructions on the last block's bytes and adds zeros (a branch here would let the compiler sink
            // these loads behind the wait for the weights)
            const int sb = min(sb0 + b, nsb - 1), sbz = min(sb0 + b, nsb);
            const uint8_t *pd = (const uint8_t *)xd + (size_t)sbz * 512, *pm = (const uint8_t *)xm + (size_t)sbz * 512;
            const uint8_t *pf = xfrag + (size_t)sb * 4096;
            d8[mt][b][0] = *(const float4 *)(pd + at_d);
            d8[mt][b][1] = *(const float4 *)(pd + at_d + 16);
            xmv[mt][b] = *(const float2 *)(pm + at_m);
#pragma unroll
            for (int tp = 0; tp < 4; ++tp) bf[mt][b][tp] = *(const u32x4 *)(pf + tp * 1024 + at_f);
        }
    }

    // ---- every weight load of the wavefront: each instruction fetches the slice of ROWS_LD whole rows as
    // consecutive 16-byte pieces (lanes past the last piece repeat it)
    u32x4 wq[STRIPS][S::NLD];
    uint32_t park_at, park_last;
    {
        const int rl = min(lane / S::CHUNKS_ROW, S::ROWS_LD - 1);
        const int ch = min(lane - (lane / S::CHUNKS_ROW) * S::CHUNKS_ROW, S::CHUNKS_ROW - 1);
        const int ch_c = min(ch, max(9 * nvalid, 1) - 1);
        constexpr int LAST0 = (S::NLD - 1) * S::ROWS_LD;        // first row of a strip's last instruction
        const int rl_last = min(rl, 15 - LAST0);
        const uint32_t at = (uint32_t)rl * rb + (uint32_t)ch_c * 16u, at_last = (uint32_t)rl_last * rb + (uint32_t)ch_c * 16u;
        park_at = (uint32_t)(rl * S::PITCH + ch * 16);
        park_last = (uint32_t)(rl_last * S::PITCH + ch * 16);
        const uint8_t *base = W + (size_t)n0 * rb + (size_t)sbc * 144;
#pragma unroll
        for (int s = 0; s < STRIPS; ++s)
#pragma unroll
            for (int n = 0; n < S::NLD; ++n)
                wq[s][n] = *(const u32x4 *)(base + (size_t)(16 * s + n * S::ROWS_LD) * rb + (n == S::NLD - 1 ? at_last : at));
    }
    __builtin_amdgcn_sched_barrier(0);  // every load above is issued before anything below waits

    float acc[MT][STRIPS][4];
    float4v accm[MT][STRIPS];
    const uint8_t *mine = stage + j * S::PITCH;

#pragma unroll
    for (int s = 0; s < STRIPS; ++s) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[mt][s][i] = 0.0f;
            accm[mt][s] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
        }
        // park strip s (the previous strip's operand reads are done: fence at the end of its last super-block)
#pragma unroll
        for (int n = 0; n < S::NLD; ++n)
            *(u32x4 *)(stage + n * S::ROWS_LD * S::PITCH + (n == S::NLD - 1 ? park_last : park_at)) = wq[s][n];
        mmv_wave_lds_fence();
        // (a) every super-block's scales: lane (row j, pair c) unpacks the pair's two scales and mins, folds the row's
        // d and dmin in, parks d * scale for the lanes that own the row in the C layout and feeds dmin * min to the
        // f32 matrix instruction; (b) one fence; (c) the sub-block dots.  Two fences per strip, not per super-block.
#pragma unroll
        for (int b = 0; b < SBW; ++b) {
            // a slice past the end of K contracts the last block it has again (finite numbers) against zero scales
            const uint8_t *blk = mine + min(b, max(nvalid, 1) - 1) * 144;
            const u32x4 h = *(const u32x4 *)blk;
            uint32_t sc2, m2;
            q4k_scale_min_pair(h.y, h.z, h.w, c, sc2, m2);
            const float d = half_bits_to_float((uint16_t)(h.x & 0xFFFF)), dmin = half_bits_to_float((uint16_t)(h.x >> 16));
            s_dsc[b * 128 + (2 * c) * 16 + j] = d * (float)(sc2 & 0xFF);
            s_dsc[b * 128 + (2 * c + 1) * 16 + j] = d * (float)(sc2 >> 8);
            // sum over the 8 sub-blocks of (dmin * m)[weight row] * (d8 * bsum)[activation row]: k = pair c, two halves
            const float m_lo = dmin * (float)(m2 & 0xFF), m_hi = dmin * (float)(m2 >> 8);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                accm[mt][s] = __builtin_amdgcn_mfma_f32_16x16x4f32(m_lo, xmv[mt][b].x, accm[mt][s], 0, 0, 0);
                accm[mt][s] = __builtin_amdgcn_mfma_f32_16x16x4f32(m_hi, xmv[mt][b].y, accm[mt][s], 0, 0, 0);
            }
        }
        mmv_wave_lds_fence();
#pragma unroll
        for (int b = 0; b < SBW; ++b) {
            const uint8_t *blk = mine + min(b, max(nvalid, 1) - 1) * 144;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const u32x2 qa = *(const u32x2 *)(blk + 16 + 32 * p + 8 * c);
                const long a_lo = (long)(((uint64_t)(qa.y & 0x0F0F0F0Fu) << 32) | (qa.x & 0x0F0F0F0Fu));
                const long a_hi = (long)(((uint64_t)((qa.y >> 4) & 0x0F0F0F0Fu) << 32) | ((qa.x >> 4) & 0x0F0F0F0Fu));
                // C layout: lane (activation row j, weight rows 4c .. 4c+3)
                const float4 sc_lo = *(const float4 *)&s_dsc[b * 128 + (2 * p) * 16 + 4 * c];
                const float4 sc_hi = *(const float4 *)&s_dsc[b * 128 + (2 * p + 1) * 16 + 4 * c];
                const float dl[4] = {sc_lo.x, sc_lo.y, sc_lo.z, sc_lo.w}, dh[4] = {sc_hi.x, sc_hi.y, sc_hi.z, sc_hi.w};
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const u32x4 bb = bf[mt][b][p];
                    const long b_lo = (long)(((uint64_t)bb.y << 32) | bb.x), b_hi = (long)(((uint64_t)bb.w << 32) | bb.z);
                    const int4v d_lo = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_lo, b_lo, int4v{0, 0, 0, 0}, 0, 0, 0);
                    const int4v d_hi = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_hi, b_hi, int4v{0, 0, 0, 0}, 0, 0, 0);
                    const float4 dq = d8[mt][b][p >> 1];
                    const float d8_lo = (p & 1) ? dq.z : dq.x, d8_hi = (p & 1) ? dq.w : dq.y;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        acc[mt][s][i] += d8_lo * ((float)d_lo[i] * dl[i]);  // d8 * (d * sc) * dot
                        acc[mt][s][i] += d8_hi * ((float)d_hi[i] * dh[i]);
                    }
                }
            }
        }
        mmv_wave_lds_fence();  // the stage and the scale slots are rewritten by the next strip
    }

    // ---- the K slices meet: each output register is summed by one wavefront, slices in order
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int s = 0; s < STRIPS; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                s_red[(wave * S::OUT + (mt * STRIPS + s) * 4 + i) * 64 + lane] = acc[mt][s][i] - accm[mt][s][i];
    __syncthreads();
    for (int r = wave; r < S::OUT; r += WAVES) {
        float sum = 0.0f;
#pragma unroll
        for (int w2 = 0; w2 < WAVES; ++w2) sum += s_red[(w2 * S::OUT + r) * 64 + lane];
        const int mt = r / (STRIPS * 4), s = (r >> 2) % STRIPS;
        const int n = n0 + 16 * s + 4 * c + (r & 3), row = 16 * mt + j;
        if (row < M) y[(size_t)row * N + n] = sum;
    }
}

template <int MT, int STRIPS, int SBW, int WAVES>
static int launch_mmv_cfg(candy_hip_device *dev, const candy_hip_qtensor *w, const MmvOperands &o, int M, float *y) {
    using S = MmvShape<MT, STRIPS, SBW, WAVES>;
    static_assert(S::SMEM <= 160 * 1024, "LDS");
    auto kern = k_mmv_q4k<MT, STRIPS, SBW, WAVES>;
    if (S::SMEM > 48 * 1024)
        CANDY_HIP_TRY(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::SMEM));
    const int N = (int)w->rows, K = (int)w->cols;
    hipLaunchKernelGGL(kern, dim3((unsigned)(N / (16 * STRIPS))), dim3(WAVES * 64), S::SMEM, dev->stream,
                       (const uint8_t *)w->data, (const uint8_t *)o.xfrag, (const float *)o.xd, (const float *)o.xm, y, N, M, K,
                       o.frag_stride, o.scale_stride);
    CANDY_LAUNCH_CHECK();
    return CANDY_HIP_OK;
}

static size_t mmv_scales_bytes(int64_t K) { return (((size_t)((K >> 8) + 1) * 16 * 8 * sizeof(float)) + 255) & ~(size_t)255; }
static size_t mmv_frag_bytes(int64_t K) { return ((size_t)16 * (size_t)K + 255) & ~(size_t)255; }
size_t mmv_workspace_bytes(int64_t K) { return 2 * (mmv_frag_bytes(K) + 2 * mmv_scales_bytes(K)) + 256; }

bool mmv_covers(const candy_hip_qtensor *w, int64_t m) {
    if (w->fmt != CANDY_HIP_Q4_K || m < 2 || m > 32 || ((uintptr_t)w->data & 15) != 0) return false;
    if (m < w->dev->opt.mmv_min_m || m > w->dev->opt.mmv_max_m) return false;
    const int64_t nsb = w->cols >> 8;
    // two tiles of activation rows keep twice the operands in registers: rows of up to 16 super-blocks only
    return w->cols % 256 == 0 && nsb >= 1 && nsb <= (m > 16 ? 16 : 48) && w->rows >= 16 && w->rows % 16 == 0 &&
           w->rows <= 0x7FFFFFFF;
}

// Activations [m, K] (2 <= m <= 32), f32 (x) or Q8_0 blocks (x null), against a Q4_K weight: into operand order
// (quantizing the f32), then one pass over the weights.  ws: mmv_workspace_bytes(K) of device memory.
int launch_mmv(candy_hip_device *dev, const candy_hip_qtensor *w, const float *x, const void *q8_blocks, int64_t m,
               float *y, void *ws) {
    const int K = (int)w->cols, nsb = K >> 8, tiles = m > 16 ? 2 : 1;
    MmvOperands o;
    o.frag_stride = mmv_frag_bytes(K);
    o.scale_stride = mmv_scales_bytes(K) / sizeof(float);
    o.xfrag = (uint8_t *)ws;
    o.xd = (float *)((uint8_t *)ws + 2 * o.frag_stride);
    o.xm = o.xd + 2 * o.scale_stride;
    if (x)
        hipLaunchKernelGGL(k_mmv_quantize_pack, dim3((unsigned)(16 * tiles * (K >> 2) / 256)), dim3(256), 0, dev->stream,
                           (const float4 *)x, (int)m, K, o.xfrag, o.xd, o.xm, o.frag_stride, o.scale_stride);
    else
        hipLaunchKernelGGL(k_mmv_pack_blocks, dim3((unsigned)((16 * tiles * (K >> 5) + 255) / 256)), dim3(256), 0,
                           dev->stream, (const BlockQ8_0 *)q8_blocks, (int)m, tiles, K, o);
    CANDY_LAUNCH_CHECK();
    const int M = (int)m;
    const int variant = dev->opt.mmv_variant;  // comparison runs: 1 one strip per wavefront, 2 two
    // Measured on this chip (us per call with the quantizer, 16 rows): two strips per wavefront pay once every resident
    // wavefront has work anyway, 14336 x 4096 14.5 against 15.9, 32000 x 4096 25.5 against 28.1; below that the
    // extra wavefronts of the one-strip shape win, 11008 x 4096 13.1 against 13.8, 4096 x 4096 7.7 against 9.6.
    const bool two = w->rows % 32 == 0 && (variant ? variant == 2 : w->rows >= 48 * (int64_t)dev->num_cus);
    if (tiles == 2) {
        if (nsb <= 8) return launch_mmv_cfg<2, 1, 1, 8>(dev, w, o, M, y);
        if (two) return launch_mmv_cfg<2, 2, 1, 16>(dev, w, o, M, y);
        return launch_mmv_cfg<2, 1, 1, 16>(dev, w, o, M, y);
    }
    if (nsb <= 8) return launch_mmv_cfg<1, 1, 1, 8>(dev, w, o, M, y);
    if (nsb <= 16) {
        if (two) return launch_mmv_cfg<1, 2, 2, 8>(dev, w, o, M, y);
        return launch_mmv_cfg<1, 1, 1, 16>(dev, w, o, M, y);
    }
    if (nsb <= 24) return launch_mmv_cfg<1, 1, 3, 8>(dev, w, o, M, y);
    if (nsb <= 32) {
        if (two) return launch_mmv_cfg<1, 2, 2, 16>(dev, w, o, M, y);
        return launch_mmv_cfg<1, 1, 2, 16>(dev, w, o, M, y);
    }
    return launch_mmv_cfg<1, 1, 3, 16>(dev, w, o, M, y);
}

}  // namespace candy
