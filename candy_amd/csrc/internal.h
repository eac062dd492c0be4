// Host-side internals shared by the translation units of libcandy_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../include/candy_hip.h"

namespace candy {

// Thread-local failure text behind candy_hip_last_error().
void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define CANDY_HIP_TRY(expr)                                                              \
    do {                                                                                 \
        hipError_t _e = (expr);                                                          \
        if (_e != hipSuccess)                                                            \
            return ::candy::fail(_e == hipErrorOutOfMemory ? CANDY_HIP_ERR_OOM : CANDY_HIP_ERR_HIP, \
                                 "%s failed: %s", #expr, hipGetErrorString(_e));         \
    } while (0)

#define CANDY_REQUIRE(cond, ...)                                                          \
    do {                                                                                 \
        if (!(cond)) return ::candy::fail(CANDY_HIP_ERR_INVALID, __VA_ARGS__);           \
    } while (0)

// Check the launch that was just enqueued.
#define CANDY_LAUNCH_CHECK() CANDY_HIP_TRY(hipGetLastError())

struct FormatInfo {
    int elems;
    int bytes;
};
FormatInfo format_info(int fmt);  // {0,0} if unknown
int block_alignment(int fmt);      // alignment the block array of a format needs (its widest aligned load)

// Planar Q8_0 activations: the matvec / MFMA kernels read the int8 quants and the
// per-32 scale separately so every load is naturally aligned.
struct Q8Scale {
    float d;       // fp16-rounded scale, widened back to f32 (what a Q8_0 block stores)
    int32_t bsum;  // sum of the block's 32 quants (for the `min` term of Q4_K)
};

// Switches of one device handle, set with candy_hip_set_option (the keys are listed in runtime.hip and in
// include/candy_hip.h).  The defaults are what the library is measured and shipped with; the others select a
// kernel that the default dispatch would not pick, for comparison runs and for tests that want a given kernel.
struct Options {
    int matvec_span = 1;         // batch-1 kernel of the 2-byte aligned formats: aligned 16-byte spans through LDS
    int small_batch_kernel = 1;  // 2..8 rows: the one-workgroup-per-CU kernel (0: the looping kernel only)
    int even_two_rows = 1;       // Q4_K, 2 rows: the even-split vector kernel (0: the looping kernel)
    int i8_min_m = 0;            // 5..15 rows: int8 tiles from this batch on (0: whichever the fitted times say)
    int mmq_min_m = 16;          // batch from which the tile kernels take over from the matvec family (>= 16)
    int f16_big_min_m = 256;     // decoder prompt pass: batch from which the fp16 big tiles take over from the int8 tiles
    int f16_api_min_m = 33;      // candy_hip_qmatmul*: the same for a single contraction (Q4_K, Q6_K; the others from 65)
    int mmq_fp16_only = 0;       // 1: every tile contraction on the single-buffered fp16 tiles
    int i8_grid_split = 1;       // int8 tiles: split K over workgroups on small grids
    int f16_shape = 0;           // comparison runs: Q4_K fp16 tiles 128 x 128 (2); single-role 128 x 256 kernel (3); never 112-row tiles (4)
    int f16_split = 0;           // comparison runs: workgroups that share one fp16 tile's K (0: by grid size)
    int mmv_min_m = 3;           // f32 x Q4_K with this many .. mmv_max_m rows: the one-pass int8 kernel
    int mmv_max_m = 32;          //   (0: never; more than 16 rows only for rows of up to 4096 values)
    int mmv_variant = 0;         // comparison runs: 1 = one 16-row strip per wavefront, 2 = two
    int pair_rows = 0;           // fused gate/up: row pairs per workgroup, 32 / 16 / 8 (0: the most even split)
    int rms_rows = 0;            // fused RMSNorm prologue: rows per workgroup, 16 / 24 (0: the most even split)
    int prefill_fold_split_sums = 1; // prompt pass: split-K copies summed inside the launch that follows (norm, rope)
    int prefill_qkv_group = 1;       // prompt pass: q / k / v (and gate / up) on one grid each where they run on the fp16 tiles
    int prefill_attention_valu = 0;  // prompt attention for head_dim 128 on the vector ALU instead of the matrix cores
    int llama_graph = 1;         // decoders created afterwards replay a captured HIP graph (0: eager launches)
    int fused_wide = 1;          // decode step: one-workgroup-per-CU kernels for the big Q4_K shapes (0: the narrower ones)
    int wide_waves = 8;          // wavefronts per workgroup of those kernels: 8 (two workgroups per CU) or 16 (one)
    int prefill_attention_groups = 0;  // comparison runs: key-tile groups per workgroup in matrix-core prompt attention, 1 or 2 (0: by shape)
    int attn_splits = 0;         // comparison runs: splits of the cached positions in decode attention, 1..64 (0: by shape)
    int down_quant = 0;          // decode step: 1 = gate / up leaves f32 SiLU*Mul values and the down projection quantizes them in its prologue (measured slower: 561 against 583 tok/s on the 7B shape); 0 = gate / up quantizes, blocks shared between workgroups through tickets
};

}  // namespace candy

namespace candy {
// y = res + (part[0] + part[1] + ...), `count` floats, copies `stride` floats apart: a split sum not yet launched
struct SplitPending {
    const float *part = nullptr;
    float *y = nullptr;
    const float *res = nullptr;
    size_t count = 0, stride = 0;
    int n_split = 0;  // 0: nothing pending
};
}  // namespace candy

struct candy_hip_device {
    int ordinal = 0;
    candy::Options opt;
    unsigned opt_epoch = 0;  // counts candy_hip_set_option calls: a decoder's captured graph is stale when it moved
    hipStream_t stream = nullptr;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    int num_cus = 0;
    char name[256] = {0};
    // Workspace for quantized activations (grown on demand, never shrunk).
    void *ws = nullptr;
    size_t ws_bytes = 0;
    // Partial sums of the split-K tile kernel (same policy).
    void *ws_split = nullptr;
    size_t ws_split_bytes = 0;
    // One word of pinned host memory that kernels raise when they meet an index outside its table (the condition
    // the CPU path panics on); check_fault() reports and clears it after a synchronisation.
    int *fault = nullptr;
    // While this points at a record, a single fp16-tile contraction that splits K leaves its partial copies unsummed
    // and describes them there; the caller's next launch adds them up (the prompt pass: inside its norm kernel).
    candy::SplitPending *defer_split = nullptr;
    // This GPU's copy of the library's file-scope scratch array (matvec.hip), resolved when the handle is opened.
    void *noalloc_scratch = nullptr;
};

struct candy_hip_qtensor {
    candy_hip_device *dev = nullptr;
    int fmt = 0;
    int64_t rows = 0, cols = 0;
    size_t nbytes = 0;
    void *data = nullptr;
    bool owned = false;
    bool padded = false;  // at least 16 readable bytes follow the last block
};

namespace candy {
// Kernel argument of the batch-1 matvec: up to three weights that share one activation row.
struct MatvecJob {
    const uint8_t *W;
    float *y;
    const float *res;  // optional residual added to the output (may alias y)
    int N;
    int wg_end;        // cumulative workgroup count, filled by the launcher
};
struct MatvecJobs {
    MatvecJob j[3];
    int n;
};
}  // namespace candy

struct candy_hip_qact {
    candy_hip_device *dev = nullptr;
    int64_t max_m = 0, max_cols = 0;  // capacity
    int64_t m = 0, cols = 0;          // shape of what it currently holds
    int8_t *qs = nullptr;             // [m, cols] int8
    candy::Q8Scale *scales = nullptr; // [m, cols/32]
};

namespace candy {

// Makes dev's GPU current for the calling thread (cgo may move goroutines between threads).
int use_device(const candy_hip_device *dev);
// After the stream has been synchronised: CANDY_HIP_ERR_INVALID if a kernel since the last check met an
// out-of-range index (the word is cleared), CANDY_HIP_OK otherwise.
int check_fault(candy_hip_device *dev);
// Returns a workspace of at least `bytes` bytes (256-byte aligned).
int workspace(candy_hip_device *dev, size_t bytes, void **out);
// Second buffer, for the split-K partial sums (lives beside the activation workspace).
int splitk_workspace(candy_hip_device *dev, size_t bytes, void **out);
// mmq_f16.hip: y[i] = (res[i] +) part[0][i] + part[1][i] + ... in that order (count floats per part)
int launch_splitk_sum(candy_hip_device *dev, const float *part, float *y, const float *res, size_t count, int n_split,
                      size_t stride = 0);  // copies `stride` floats apart (0: count)
// ops.hip: the pending sum, the residual add, RMSNorm and Q8_0 quantization of the rows in one launch
int launch_split_rms_norm_quant(candy_hip_device *dev, const SplitPending &sp, const float *alpha, float eps, int64_t rows,
                                int64_t cols, int8_t *qs, Q8Scale *scales, _Float16 *xh);
// Formats the batch-1 kernel contracts (residual epilogue, several weights per launch): all that have a vec-dot.
// The fused decode kernels exist for Q4_K, Q6_K, Q8_0 and the two Q4_0 orders only.
inline bool format_has_batch1_kernel(int fmt) {
    switch (fmt) {
    case CANDY_HIP_Q4_K: case CANDY_HIP_Q6_K: case CANDY_HIP_Q8_0: case CANDY_HIP_Q4_0: case CANDY_HIP_Q4_0_GGML:
    case CANDY_HIP_Q4_1: case CANDY_HIP_Q4_1_GGML: case CANDY_HIP_Q5_0: case CANDY_HIP_Q5_1: case CANDY_HIP_Q2_K:
    case CANDY_HIP_Q3_K: case CANDY_HIP_Q5_K:
        return true;
    default:
        return false;
    }
}

// quant.hip: x[rows, cols] -> planar int8 quants + scales; optionally also 34-byte blocks.
// xh (optional): also the fp16 values d * q, row-major like x (what the fp16 tile kernels contract with).
int launch_quantize_q8(candy_hip_device *dev, const float *x, int64_t rows, int64_t cols,
                       int8_t *qs, Q8Scale *scales, void *blocks, _Float16 *xh = nullptr);
// quant.hip: Q8_0 blocks -> planar form.
int launch_q8_blocks_to_planar(candy_hip_device *dev, const void *blocks, int64_t n_blocks,
                               int8_t *qs, Q8Scale *scales);
// matvec.hip: y[m, rows] for m in 1..15 from planar activations.
// vector_only: never the int8 tile kernel (whose K split takes a workspace), whatever the batch.
int launch_matvec(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs,
                  const Q8Scale *scales, int64_t m, float *y, bool vector_only = false);
// matvec.hip: resolves this GPU's address of the file-scope scratch array (dev's GPU must be current).
int noalloc_scratch_init(candy_hip_device *dev);
// matvec.hip: one activation row against up to three weights in one launch, optional residuals.
int launch_matvec_multi(candy_hip_device *dev, const candy_hip_qtensor *const *ws, float *const *ys,
                        const float *const *res, int n, const int8_t *qs, const Q8Scale *scales);
// mmq.hip: MFMA tile kernel for m >= 16. half_ws: mmq_m_pad(m) * cols fp16 values of scratch.
int64_t mmq_m_pad(int64_t m);
// Whether launch_mmq / launch_contract add `res` in the contraction's own epilogue (then res may alias y).
bool mmq_fuses_residual(const candy_hip_qtensor *w, int64_t m);
// xh_ready (optional): the activations already expanded to fp16, >= mmq_m_pad(m) rows of `cols` values in the
// fragment order of xh_index4 (rows past m may hold anything); res (optional, may alias y): y = res + x . W^T.
// f16_min_m: batch from which the fp16 big tiles may answer (0: the decoder's threshold, opt.f16_big_min_m)
int launch_mmq(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs,
               const Q8Scale *scales, int64_t m, float *y, void *half_ws, const _Float16 *xh_ready = nullptr,
               const float *res = nullptr, int f16_min_m = 0);
// mmq_i8.hip: Q4_K / Q6_K on v_mfma_i32_16x16x32_i8 with the batch-1 kernels' integer arithmetic.
bool mmq_i8_covers(const candy_hip_qtensor *w, const int8_t *qs);
// mmv_i8.hip: 2 .. 32 activation rows against a Q4_K weight, one pass over the weights on the int8 matrix cores
size_t mmv_workspace_bytes(int64_t K);
bool mmv_covers(const candy_hip_qtensor *w, int64_t m);
bool matvec_even_covers(const candy_hip_qtensor *w, int64_t m);  // the even-split vector kernel takes this batch
int launch_mmv(candy_hip_device *dev, const candy_hip_qtensor *w, const float *x, const void *q8_blocks, int64_t m,
               float *y, void *ws);
int launch_mmq_i8(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs,
                  const Q8Scale *scales, int64_t m, float *y);
// mmq_f16.hip: prompt-sized batches on big fp16 tiles. xh: fp16 activations, mmq_m_pad(m) rows in the fragment order
// of xh_index4.
bool mmq_f16_big_covers(const candy_hip_qtensor *w, int64_t m, int min_m = 0);
int launch_mmq_f16_big(candy_hip_device *dev, const candy_hip_qtensor *w, const _Float16 *xh, int64_t m, float *y,
                       const float *res = nullptr);
// Two or three projections of the same activations on one grid (every tensor but the last: a multiple of 128 rows).
bool mmq_f16_group_covers(const candy_hip_qtensor *const *ws, int count, int64_t m);
int launch_mmq_f16_group(candy_hip_device *dev, const candy_hip_qtensor *const *ws, float *const *ys, int count,
                         const _Float16 *xh, int64_t m);
// ops.hip: fused decode-step stages (all enqueue on dev->stream, no allocation, no sync).
int launch_rms_norm_quant(candy_hip_device *dev, const float *x, const float *alpha, float eps, int64_t rows,
                          int64_t cols, float *xn_out, int8_t *qs, Q8Scale *scales, _Float16 *xh = nullptr);
int launch_silu_mul_quant(candy_hip_device *dev, const float *gate, const float *up, int64_t rows, int64_t cols,
                          float *act_out, int8_t *qs, Q8Scale *scales, _Float16 *xh = nullptr);
// fused.hip: batch-1 contraction of one activation row with up to three weights, with optional
// RMSNorm+quantize prologue (x != nullptr, else planar Q8_0 in xq/xs), residuals, or the
// gate/up SiLU*Mul+quantize epilogue (pair). Returns CANDY_HIP_ERR_UNSUPPORTED when the shape
// has no fused instantiation (caller falls back to the unfused sequence).
struct FusedLaunch {
    int n = 0;
    const candy_hip_qtensor *w[3] = {nullptr, nullptr, nullptr};
    float *y[3] = {nullptr, nullptr, nullptr};
    const float *res[3] = {nullptr, nullptr, nullptr};
    const int8_t *xq = nullptr;
    const Q8Scale *xs = nullptr;
    const float *x = nullptr, *alpha = nullptr;
    float eps = 0.0f;
    bool pair = false;
    int8_t *oq = nullptr;
    Q8Scale *os = nullptr;
    // pair only, optional: rows floats and rows / 32 counters (zero before the first launch; every launch leaves
    // them zero) that let a workgroup own part of a 32-value output block where that spreads the rows evenly
    float *pair_act = nullptr;
    unsigned *pair_tickets = nullptr;
};
int launch_matvec_fused(candy_hip_device *dev, const FusedLaunch &launch);
// fused_wide.hip: the same contractions for the big Q4_K shapes as one workgroup per compute unit (an even share of
// the rows each, the prologue once or twice per CU).  Prologue: RMSNorm + quantize of x (x, alpha, eps), or the
// plain quantization of x (alpha null).  Returns CANDY_HIP_ERR_UNSUPPORTED (no error text) for shapes it does not cover.
struct WideLaunch {
    int n = 0;
    const candy_hip_qtensor *w[3] = {nullptr, nullptr, nullptr};
    float *y[3] = {nullptr, nullptr, nullptr};
    const float *res[3] = {nullptr, nullptr, nullptr};
    const float *x = nullptr, *alpha = nullptr;
    float eps = 0.0f;
    bool pair = false;
    int8_t *oq = nullptr;
    Q8Scale *os = nullptr;
    float *pair_act = nullptr;
    unsigned *pair_tickets = nullptr;
};
int launch_matvec_wide(candy_hip_device *dev, const WideLaunch &launch);
// whether launch_matvec_wide takes this launch on its long-row QUANT shape (the decode step's down projection)
bool wide_quant_long_covers(const candy_hip_device *dev, const WideLaunch &launch);
// attention.hip
struct AttnLaunch {
    const float *q = nullptr;      // [n_heads, head_dim]; pre-Rope when k_new is set
    const float *k_new = nullptr;  // optional pre-Rope key / value rows of the new token, [n_kv_heads, head_dim]
    const float *v_new = nullptr;
    const float *cos_t = nullptr;  // Rope tables [max_pos, head_dim/2] (with k_new)
    const float *sin_t = nullptr;
    void *k_cache = nullptr;       // this layer's cache (f32, or fp16 with kv_f16), cache_stride elements between kv heads
    void *v_cache = nullptr;
    bool kv_f16 = false;
    const int *pos_ptr = nullptr;  // position of the new token in device memory, or
    int n_pos = 0;                 // number of cached positions to attend when pos_ptr is null
    int64_t cache_stride = 0;
    float scale = 1.0f;
    int n_heads = 0, n_kv_heads = 0, head_dim = 0, n_splits = 1;
    void *scratch = nullptr;       // attention_scratch_bytes() of device memory
    float *out = nullptr;          // optional f32 output [n_heads, head_dim]
    int8_t *oq = nullptr;          // optional planar Q8_0 output
    Q8Scale *os = nullptr;
};
// ops.hip: FastArgmax of one long row over many workgroups into a 64-bit word (zero before the launch), and the index
// the word stands for
int launch_argmax_key(candy_hip_device *dev, const float *logits, int64_t cols, unsigned long long *key);
__host__ __device__ inline uint32_t argmax_key_index(unsigned long long key) {
    return key ? 0xFFFFFFFFu - (uint32_t)(key & 0xFFFFFFFFull) : 0u;
}
int attention_splits(const candy_hip_device *dev, int64_t n_kv_heads, int64_t max_pos);
size_t attention_scratch_bytes(int n_heads, int n_kv_heads, int head_dim, int n_splits);
int launch_attention(candy_hip_device *dev, const AttnLaunch &launch);
// runtime.hip: zero-fill with a kernel (safe to capture into a HIP graph, unlike a memset node)
int launch_zero(candy_hip_device *dev, void *dptr, size_t bytes);
// Workspace carved for one contraction: planar quants, scales and (m >= 16) fp16 activations.
struct ActWorkspace {
    int8_t *qs;
    Q8Scale *scales;
    void *half_ws;
    void *mmv_ws = nullptr;  // operand-order activations for the small-batch int8 kernel (2 .. 32 rows)
};
int act_workspace(candy_hip_device *dev, int64_t m, int64_t cols, bool need_quants, ActWorkspace *out);
// matvec.hip: y[m, rows] = x . W^T for any m from planar activations that live OUTSIDE the device
// workspace (the tile kernel may carve its fp16 scratch from it).
int mmq_min_m(const candy_hip_device *dev);
int launch_contract(candy_hip_device *dev, const candy_hip_qtensor *w, const int8_t *qs, const Q8Scale *scales,
                    int64_t m, float *y, const _Float16 *xh_ready = nullptr, const float *res = nullptr);
// prefill.hip: prompt stages of the decoder (n tokens at positions pos0 ..).
int launch_prefill_rope_kv(candy_hip_device *dev, float *q, const float *k, const float *v, const float *cos_t,
                           const float *sin_t, void *k_cache, void *v_cache, bool kv_f16, int n, int pos0, int n_heads,
                           int n_kv_heads, int head_dim, int64_t cache_stride, const SplitPending *sp = nullptr);
int launch_attn_prefill(candy_hip_device *dev, const float *q, const void *k_cache, const void *v_cache, bool kv_f16,
                        float *out, int n, int pos0, int n_heads, int n_kv_heads, int head_dim, int64_t cache_stride,
                        float scale, _Float16 *xh_out = nullptr);  // xh_out: the fp16 image of the quantized rows, not `out`
bool attn_prefill_writes_half(const candy_hip_device *dev, int head_dim);

}  // namespace candy
