/*
 * candy_hip.h -- C ABI of libcandy_hip.so: candy's quantized-matmul path on one MI355X.
 *
 * This is the boundary a cgo shim binds (the way llm/internal/flashattn/flashattn.go:3-13
 * binds flash_api.h:71-117): plain C, opaque handles, raw device pointers, sizes by value.
 * Unlike that precedent every call returns a status and the failure text is retrievable
 * (candy's Go convention is `(value, error)` on every fallible call, tensor/ops.go:88-90).
 *
 * Each declaration names the reference interface it stands behind.  "QCU" is
 * tensor/internal/cuda/kernels/quantized.cu, "QGO" is tensor/internal/cpu/kernels/quantized.go.
 *
 * Threading: handles may be used from any OS thread (cgo migrates goroutines between
 * threads); every call selects its device itself.  Calls on one device handle are
 * enqueued on that handle's stream in call order; two threads using the same handle at
 * the same time must serialise themselves, as candy's tensors do (no locks anywhere in
 * the reference).  No host pointer passed in is retained after the call returns.
 */
#ifndef CANDY_HIP_H
#define CANDY_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct candy_hip_device candy_hip_device;     /* one GPU + its stream + its workspace   */
typedef struct candy_hip_qtensor candy_hip_qtensor;   /* device-resident quantized weight matrix */
typedef struct candy_hip_qact candy_hip_qact;         /* activations quantized once, reusable     */
typedef struct candy_hip_llama candy_hip_llama;       /* Llama-style decoder built on the ops    */

enum candy_hip_status {
    CANDY_HIP_OK = 0,
    CANDY_HIP_ERR_INVALID = 1,     /* bad argument: nil pointer, shape, unknown format        */
    CANDY_HIP_ERR_HIP = 2,         /* a HIP runtime call failed; text has hipGetErrorString   */
    CANDY_HIP_ERR_OOM = 3,         /* device allocation failed                                 */
    CANDY_HIP_ERR_UNSUPPORTED = 4  /* valid request this build has no kernel for               */
};

/* Block formats; values are the GGML type ids (what a GGUF file stores).
 * Layouts: QGO:8-11 (Q4_0, 18 B / 32), QGO:34-37 (Q8_0, 34 B / 32),
 * QGO:55-59 (Q4_K, 144 B / 256), QGO:70-75 (Q6_K, 210 B / 256). */
enum candy_hip_qformat {
    CANDY_HIP_Q4_0 = 2,        /* element order of candy's CPU dequantize, QGO:85-93 (interleaved) */
    CANDY_HIP_Q8_0 = 8,
    CANDY_HIP_Q4_K = 12,
    CANDY_HIP_Q6_K = 14,
    CANDY_HIP_Q4_0_GGML = 102, /* element order of QCU:862-866 / GGUF files (low half, high half)   */
    /* The reference's other block formats: dequantize, row gather and QMatMul at any batch through the
     * general matvec kernel (no matrix-core tiles, no fused decode kernels).  Layouts QGO:13-31, 39-52,
     * 62-67, 78-82; dequantize QGO:107-116 and QCU:728-795, 870-990, 1054-1102, 1178-1206; vec-dots
     * QCU:1947-2053, 2108-2135, 2177-2209, 2300-2331. */
    CANDY_HIP_Q4_1 = 3,        /* 20 B / 32; element order of candy's CPU dequantize, QGO:107-116 */
    CANDY_HIP_Q4_1_GGML = 103, /* element order of QCU:870-899 / GGUF files */
    CANDY_HIP_Q5_0 = 6,        /* 22 B / 32 */
    CANDY_HIP_Q5_1 = 7,        /* 24 B / 32 */
    CANDY_HIP_Q2_K = 10,       /* 84 B / 256 */
    CANDY_HIP_Q3_K = 11,       /* 110 B / 256 */
    CANDY_HIP_Q5_K = 13,       /* 176 B / 256 */
    CANDY_HIP_Q8_K = 15        /* 292 B / 256; dequantize and row gather only (the reference has no weight vec-dot) */
};

/* ------------------------------------------------------------------ library / device
 * Stands behind candy.BackendDevice (device.go:49-82): Location/IsSame -> ordinal,
 * Synchronize -> candy_hip_synchronize, StorageFromSlice -> alloc + h2d, Alloc/Zeros -> alloc + zero. */
const char *candy_hip_last_error(void);                 /* thread-local text of the last failure   */
const char *candy_hip_version(void);
int candy_hip_device_count(int *count);
int candy_hip_open(int ordinal, candy_hip_device **out);
int candy_hip_close(candy_hip_device *dev);
int candy_hip_device_ordinal(const candy_hip_device *dev, int *ordinal);
int candy_hip_device_name(const candy_hip_device *dev, char *buf, size_t buf_len);
int candy_hip_synchronize(candy_hip_device *dev);       /* device.go:81 Synchronize                */

/* Switches of one device handle.  No environment variable is ever read: what selects a kernel is an argument
 * or one of these, set from the thread that uses the handle.  The defaults are the measured, shipped choice;
 * everything else exists so that comparison runs and tests can ask for a kernel the dispatch would not pick
 * (results stay within the documented tolerance whichever is chosen).  Unknown keys and values out of range
 * are CANDY_HIP_ERR_INVALID.  No counterpart in the reference.
 *   key                          default  meaning
 *   "llama.graph"                1        decoders created afterwards replay a captured HIP graph (0: eager)
 *   "mmq.min_m"                  16       batch from which tile kernels replace the matvec family (>= 16)
 *   "mmq.f16_big_min_m"          256      decoder prompt pass: batch from which fp16 big tiles (3e-4 per matmul) replace the
 *                                         exact int8 tiles (below it the pass holds the decode step's 1e-3 end to end)
 *   "mmq.f16_api_min_m"          33       the same for one contraction through candy_hip_qmatmul / candy_hip_qmatmul_q8 (one
 *                                         matmul: 3e-4 < 1e-3): Q4_K and Q6_K from this many rows, the other formats from 65
 *                                         or this if larger
 *   -- comparison / test only --
 *   "matvec.span"                1        batch-1 kernel of 2-byte aligned formats fetches aligned 16-byte spans
 *   "matvec.small_batch_kernel"  1        2..8 rows on the one-workgroup-per-CU kernel (0: looping kernel)
 *   "matvec.even_two_rows"       1        Q4_K, 2 rows: the vector kernel that deals the weight rows evenly to two
 *                                         workgroups per CU (0: looping kernel)
 *   "mmq.i8_min_m"               0        5..15 rows: int8 tiles from this batch on (0: by measured cost model)
 *   "mmq.fp16_only"              0        every tile contraction on the single-buffered fp16 tiles
 *   "mmq.i8_grid_split"          1        int8 tiles split K over workgroups on small grids
 *   "mmq.f16_shape"              0        comparison runs: Q4_K fp16 tiles of 128 x 128 at every batch (2); fp16 tiles
 *                                         computed by the kernel whose wavefronts each dequantize and multiply (3)
 *                                         instead of the one that splits the two roles over wavefronts; 128 weight
 *                                         rows per tile also where 112 divide the rows and fill the chip better (4)
 *                                         (0: by shape)
 *   "mmq.f16_split"              0        comparison runs: K split of the fp16 tile kernels over this many workgroups per
 *                                         tile, 1..16 (0: as many as fill the chip)
 *   "mmv.min_m"                  3        candy_hip_qmatmul on Q4_K: batches of this many .. "mmv.max_m" rows take the
 *   "mmv.max_m"                  32         one-pass int8 matrix-core kernel (max 0: never)
 *   "mmv.variant"                0        that kernel with one (1) or two (2) 16-row strips per wavefront (0: by shape)
 *   "fused.pair_rows"            0        fused gate/up: row pairs per workgroup 32 / 16 / 8 (0: most even split)
 *   "fused.rms_rows"             0        fused RMSNorm prologue: rows per workgroup 16 / 24 (0: most even split)
 *   "fused.wide"                 1        decode step: kernels that deal the rows of the big Q4_K shapes evenly over the CUs
 *   "fused.wide_waves"           8        wavefronts per workgroup of those kernels: 8 (two workgroups per CU) or 16 (one)
 *   "fused.down_quant"           0        decode step, comparison runs and tests: 1 = the gate / up launch leaves its f32
 *                                         SiLU*Mul values and the down projection quantizes them in its own prologue (0: gate /
 *                                         up quantizes them, handing 32-value blocks that two workgroups share through
 *                                         per-block tickets); same bits, measured slower
 *   "attention.splits"           0        comparison runs: decode attention deals the cached positions to this many
 *                                         workgroups per kv head, 1..64 (0: by shape); read when a decoder is created
 *   "prefill.qkv_group"          1        prompt pass: projections that share their input (q / k / v; gate / up) as one
 *                                         grid each where all of them run on the fp16 tiles (0: one launch each)
 *   "prefill.fold_split_sums"    1        prompt pass: the partial copies a projection split along K leaves are summed by the
 *                                         launch that follows (RMSNorm + quantize behind o / down, rope behind q / k / v;
 *                                         0: a launch of its own sums them)
 *   "prefill.attention_valu"     0        prompt attention for head_dim 128 on the vector ALU
 *   "prefill.attention_groups"   0        comparison runs: matrix-core prompt attention with one (1) or two (2) groups of
 *                                         wavefronts per query tile that take alternate key tiles (0: two for prompts of
 *                                         more than 128 tokens whose grid is at most 1.5 workgroups per CU)
 * A decoder whose step has been captured into a graph notices a later candy_hip_set_option on its device and captures
 * the step again at its next decode call.
 * Read-only keys (candy_hip_get_option): "runtime.workspace_bytes", "runtime.split_workspace_bytes" - what the
 * handle's two grow-only workspaces hold at the moment (0 until a call needs them). */
int candy_hip_set_option(candy_hip_device *dev, const char *key, int64_t value);
int candy_hip_get_option(const candy_hip_device *dev, const char *key, int64_t *value);

/* ------------------------------------------------------------------ raw device memory
 * Backs BackendStorage[T] (backend.go:4-16): Data() is a d2h copy, Clone() a d2d copy. */
int candy_hip_alloc(candy_hip_device *dev, size_t bytes, void **dptr);
int candy_hip_free(candy_hip_device *dev, void *dptr);
int candy_hip_zero(candy_hip_device *dev, void *dptr, size_t bytes);
int candy_hip_h2d(candy_hip_device *dev, void *dst_dev, const void *src_host, size_t bytes);
int candy_hip_d2h(candy_hip_device *dev, void *dst_host, const void *src_dev, size_t bytes); /* synchronises */
int candy_hip_d2d(candy_hip_device *dev, void *dst_dev, const void *src_dev, size_t bytes);

/* ------------------------------------------------------------------ block formats */
int candy_hip_block_elems(int fmt);   /* 32 / 256, 0 if unknown                                   */
int candy_hip_block_bytes(int fmt);   /* 18 / 34 / 144 / 210 / 20 / 22 / 24 / 84 / 110 / 176 / 292, 0 if unknown */
/* bytes of a [rows, cols] weight, 0 if fmt is unknown or cols is not a multiple of the block */
size_t candy_hip_qweight_bytes(int fmt, int64_t rows, int64_t cols);

/* Quantized weight [rows, cols] (cols = contraction dim) kept on the device in the ORIGINAL
 * block layout, row-major blocks, as QCU:2827 indexes them (`x[kbx + row*blocks_per_row]`).
 * upload copies host blocks; wrap adopts device memory the caller keeps owning: nbytes is the size of
 * that buffer, at least candy_hip_qweight_bytes(); a buffer with 16 or more spare bytes after the blocks
 * lets Q6_K / Q2_K / Q3_K weights take the int8 tile kernel (its last load of a row starts inside the
 * last block and runs past it), otherwise they take the fp16 tiles. */
int candy_hip_qtensor_upload(candy_hip_device *dev, int fmt, int64_t rows, int64_t cols,
                             const void *host_blocks, size_t nbytes, candy_hip_qtensor **out);
int candy_hip_qtensor_wrap(candy_hip_device *dev, int fmt, int64_t rows, int64_t cols,
                           void *dev_blocks, size_t nbytes, candy_hip_qtensor **out);
int candy_hip_qtensor_free(candy_hip_qtensor *q);
int candy_hip_qtensor_info(const candy_hip_qtensor *q, int *fmt, int64_t *rows, int64_t *cols,
                           size_t *nbytes, void **dev_blocks);

/* Dequantize n_blocks blocks to f32 (device -> device).
 * QGO:85-93 DequantizeBlockQ4_0F32, QGO:131-136 DequantizeBlockQ8_0F32,
 * QCU:1008-1041 dequantize_block_q4_K, QCU:1103-1128 dequantize_block_q6_K.  Bit-exact. */
int candy_hip_dequantize_blocks(candy_hip_device *dev, int fmt, const void *dev_blocks,
                                int64_t n_blocks, float *dev_out);
int candy_hip_dequantize(candy_hip_device *dev, const candy_hip_qtensor *q, float *dev_out);

/* The same values as fp16: dequantize_block_*_f16 (tensor/internal/cuda/kernels/kernels.go:486-505; template
 * QCU:1229-1249 and the K-quant kernels with dst_t = half).  Each value is computed in f32 as above and rounded to
 * nearest even on the store: bit-exact against the f32 output rounded to fp16.  dev_out: 8-byte aligned. */
int candy_hip_dequantize_blocks_f16(candy_hip_device *dev, int fmt, const void *dev_blocks,
                                    int64_t n_blocks, void *dev_out_f16);
int candy_hip_dequantize_f16(candy_hip_device *dev, const candy_hip_qtensor *q, void *dev_out_f16);

/* float64 output for the formats whose CPU kernels have float64 twins: QGO:96-104 DequantizeBlockQ4_0F64,
 * QGO:119-128 DequantizeBlockQ4_1F64, QGO:139-144 DequantizeBlockQ8_0F64 (the f32-widened scale times the level,
 * in float64).  Other formats: CANDY_HIP_ERR_UNSUPPORTED.  Bit-exact. */
int candy_hip_dequantize_blocks_f64(candy_hip_device *dev, int fmt, const void *dev_blocks,
                                    int64_t n_blocks, double *dev_out);

/* f32 [rows, cols] -> Q8_0 blocks (34 B each, rows*cols/32 of them), cols % 32 == 0.
 * QCU:3521-3558 quantize_q8_1 without its `sum` half.  Bit-exact. */
int candy_hip_quantize_q8_0(candy_hip_device *dev, const float *dev_x, int64_t rows, int64_t cols,
                            void *dev_out_blocks);

/* Weight quantizer: f32 [rows, cols] (device) -> blocks of fmt (device, rows*cols/qk of them), cols a
 * multiple of the block.  candy only names these kernels (tensor/internal/metal/kernels/kernels.go:563-592,
 * quantize_q4_0 ... quantize_q6_k) and has no implementation; the arithmetic is ggml's reference
 * quantizers (quantize_row_q4_0_ref, quantize_row_q4_K_ref, quantize_row_q6_K_ref), step for step in f32;
 * Q8_0 is candy_hip_quantize_q8_0.  Wrap the result with candy_hip_qtensor_wrap.  Inputs must be finite. */
int candy_hip_quantize(candy_hip_device *dev, int fmt, const float *dev_x, int64_t rows, int64_t cols,
                       void *dev_out_blocks);

/* y[m, rows] = x[m, cols] . W^T, activations quantized to Q8_0 on the device first.
 * m < 16 runs the bandwidth-bound matvec family (QCU:2787-2871 mul_mat_vec_q and its entry
 * points :2874, :2906, :2930, :2946); m >= 16 the MFMA tile kernel (QCU:455-578 mul_mat_q).
 * Q4_K with 3 <= m <= 16, rows % 16 == 0 and cols <= 12288 (m <= 32 for cols <= 4096): one pass over
 * the weights with the batch on the 16-wide side of the int8 matrix instruction (same integer dots,
 * same scales).
 * y is row-major [m, rows] (candy's result layout, tensor/ops.go:1264). */
int candy_hip_qmatmul(candy_hip_device *dev, const candy_hip_qtensor *w, const float *dev_x,
                      int64_t m, float *dev_y);

/* y[rows] = dequantize(W)[rows, cols] . x[cols] with f32 activations and no activation quantizer: the reference's
 * other matvec, dequantize_mul_mat_vec (QCU:1251-1345 for the 32-value formats, :1550-1693 q4_K, :1810-1911 q6_K
 * and the other K-quants beside them).  It equals what candy's CPU backend computes (Dequantize, then the naive f32
 * MatMul) up to f32 summation order, and does not carry the Q8_0 rounding of the activations that
 * candy_hip_qmatmul does.  Batch 1.  dev_x: 16-byte aligned. */
int candy_hip_dmmv(candy_hip_device *dev, const candy_hip_qtensor *w, const float *dev_x, float *dev_y);

/* candy_hip_qmatmul for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): no counterpart in the reference.  Same result as candy_hip_qmatmul,
 * 1 <= m <= 15 activation rows (the matvec family; the vector kernels answer every batch, so from 5 rows on the
 * bits may differ from candy_hip_qmatmul's tile kernel by f32 summation order).  The quantized activations live
 * in a 1 MiB array inside the library that every call on a GPU shares: a call whose m * cols * 1.25 bytes (plus
 * rounding to 256) exceed it fails with CANDY_HIP_ERR_INVALID, and calls that overlap on one GPU (two handles,
 * two threads) race on it.  Calls no hipMalloc / hipFree. */
int candy_hip_qmatmul_noalloc(candy_hip_device *dev, const candy_hip_qtensor *w, const float *dev_x, int64_t m,
                              float *dev_y);

/* Same contraction, activations already in Q8_0 blocks on the device ([m, cols/32] blocks). */
int candy_hip_qmatmul_q8(candy_hip_device *dev, const candy_hip_qtensor *w, const void *dev_x_q8_0,
                         int64_t m, float *dev_y);

/* Activations quantized once and contracted against several weights (q/k/v share one input,
 * gate/up another): QCU's host flow quantizes with quantize_q8_1 (:3521) and then launches
 * mul_mat_vec_q (:2787) per weight.  The handle owns its device memory; quantize may be called
 * again on the same handle with any shape up to the capacity it was created with. */
int candy_hip_qact_create(candy_hip_device *dev, int64_t max_m, int64_t max_cols, candy_hip_qact **out);
int candy_hip_qact_free(candy_hip_qact *a);
int candy_hip_qact_quantize(candy_hip_qact *a, const float *dev_x, int64_t m, int64_t cols);
int candy_hip_qmatmul_qact(candy_hip_device *dev, const candy_hip_qtensor *w, const candy_hip_qact *a,
                           float *dev_y);

/* ------------------------------------------------------------------ f32 ops of the decode step
 * One-to-one with the BackendStorage methods a Llama block calls (backend.go). */
/* backend.go:78 MatMul on contiguous f32: c[b,m,n] = a[b,m,k] . b[b,k,n]; if rhs_transposed the
 * rhs is [b,n,k] (the strided W^T view nn/linear.go:65 creates).  CONV:251-267 / :373-389. */
int candy_hip_matmul_f32(candy_hip_device *dev, const float *a, const float *b, float *c,
                         int64_t batch, int64_t m, int64_t n, int64_t k, int rhs_transposed);
/* The same MatMul for one batch with operands viewed through strides, in elements: a[i, l] sits at
 * a[i * a_row_stride + l * a_col_stride], b[l, j] at b[l * b_row_stride + j * b_col_stride] -- what
 * cpu/storage.go:889-910 passes to CONV:373-389 (the last two strides of each Layout).  The caller adds each
 * Layout's StartOffset() to the pointer it passes (cpu/storage.go:889-927 forgets it; this boundary does not).
 * c is contiguous [m, n].  Layouts with a batch dimension must be contiguous (candy_hip_matmul_f32). */
int candy_hip_matmul_f32_strided(candy_hip_device *dev, const float *a, const float *b, float *c, int64_t m, int64_t n,
                                 int64_t k, int64_t a_row_stride, int64_t a_col_stride, int64_t b_row_stride,
                                 int64_t b_col_stride);
/* backend.go:150 FastRmsNorm; reduce.go:3071-3092.  alpha may be NULL. */
int candy_hip_rms_norm(candy_hip_device *dev, const float *x, const float *alpha, float eps,
                       int64_t rows, int64_t cols, float *out);
/* backend.go:159 Rope; reduce.go:3987-4006 (pairs (i, i+d/2)). */
int candy_hip_rope(candy_hip_device *dev, const float *src, const float *cos_t, const float *sin_t,
                   int64_t bh, int64_t td, int64_t d, int64_t stride_b, float *dst);
/* backend.go:156 RopeI; reduce.go:3825-3838: adjacent pairs (2i, 2i + 1) of rows of td = t*d values, cos / sin
 * [t*d/2] per row of the tables (stride_b > 0: one table row per stride_b source elements, as in Rope). */
int candy_hip_rope_i(candy_hip_device *dev, const float *src, const float *cos_t, const float *sin_t,
                     int64_t bh, int64_t td, int64_t stride_b, float *dst);
/* backend.go:162 RopeThd; reduce.go:4178-4196: src [b, t, h, d], pairs (i, i + d/2), cos / sin [t, d/2] picked by
 * the token index. */
int candy_hip_rope_thd(candy_hip_device *dev, const float *src, const float *cos_t, const float *sin_t,
                       int64_t b, int64_t t, int64_t h, int64_t d, int64_t stride_b, float *dst);
/* backend.go:147 FastSoftmax; reduce.go:2855-2879. */
int candy_hip_softmax(candy_hip_device *dev, const float *src, int64_t rows, int64_t cols, float *dst);
/* backend.go:228 Silu; unary.go:3353-3366. */
int candy_hip_silu(candy_hip_device *dev, const float *x, int64_t n, float *out);
/* backend.go:21 Add, :27 Mul on contiguous same-shape operands. */
int candy_hip_add(candy_hip_device *dev, const float *a, const float *b, int64_t n, float *out);
int candy_hip_mul(candy_hip_device *dev, const float *a, const float *b, int64_t n, float *out);
/* silu(gate) * up in one pass (Silu then Mul). */
int candy_hip_silu_mul(candy_hip_device *dev, const float *gate, const float *up, int64_t n, float *out);
/* backend.go:129 FastArgmax; reduce.go:846-862 (first maximum wins). */
int candy_hip_argmax(candy_hip_device *dev, const float *src, int64_t rows, int64_t cols, uint32_t *out);
/* IndexSelect along dim 0 of a [n_src, width] f32 table; indexing.go:8-26. ids are int64 on the device; the
 * MaxInt64 id selects zeros, as there.  Any other id outside [0, n_src) -- where the CPU loop panics on its bounds
 * check -- reads nothing (f32 table: the row is zeros; quantized table: row 0 is read) and makes the next
 * candy_hip_synchronize or candy_hip_d2h on the handle fail with CANDY_HIP_ERR_INVALID. */
int candy_hip_index_select(candy_hip_device *dev, const float *table, int64_t n_src, int64_t width,
                           const int64_t *dev_ids, int64_t n_ids, float *out);
/* Row gather from a quantized table (embedding lookup): dequantizes rows ids[i] of q. */
int candy_hip_qindex_select(candy_hip_device *dev, const candy_hip_qtensor *q, const int64_t *dev_ids,
                            int64_t n_ids, float *out);
/* Batch-1 attention of one new token over an f32 KV cache: softmax(q.K^T * scale).V per head,
 * the MatMul / FastSoftmax / MatMul sequence a candy Llama block would issue.
 * q, out: [n_heads, head_dim]; k_cache, v_cache: [n_kv_heads, *, head_dim] with cache_stride
 * elements between kv heads; positions 0..n_pos-1 are attended. */
int candy_hip_attention_decode(candy_hip_device *dev, const float *q, const float *k_cache,
                               const float *v_cache, int64_t n_heads, int64_t n_kv_heads,
                               int64_t head_dim, int64_t n_pos, int64_t cache_stride, float scale,
                               float *out);

/* ------------------------------------------------------------------ Llama-style decoder
 * A decoder assembled from the ops above (candy has no model code; the layer order is the
 * standard Llama block: RMSNorm, q/k/v, RoPE, attention over the cache, o, residual,
 * RMSNorm, SwiGLU, residual; final RMSNorm, head, argmax). */
typedef struct candy_hip_llama_config {
    int32_t n_layers, d_model, n_heads, n_kv_heads, head_dim, d_ffn, vocab, max_pos;
    float rms_eps, rope_base;
} candy_hip_llama_config;

enum candy_hip_llama_weight {
    CANDY_HIP_W_ATTN_NORM = 0,  /* f32 [d_model]                 */
    CANDY_HIP_W_Q = 1,          /* q  [n_heads*head_dim, d_model]    */
    CANDY_HIP_W_K = 2,          /* q  [n_kv_heads*head_dim, d_model] */
    CANDY_HIP_W_V = 3,
    CANDY_HIP_W_O = 4,          /* q  [d_model, n_heads*head_dim]    */
    CANDY_HIP_W_FFN_NORM = 5,   /* f32 [d_model]                 */
    CANDY_HIP_W_GATE = 6,       /* q  [d_ffn, d_model]           */
    CANDY_HIP_W_UP = 7,
    CANDY_HIP_W_DOWN = 8,       /* q  [d_model, d_ffn]           */
    CANDY_HIP_W_OUT_NORM = 9,   /* f32 [d_model], layer = -1     */
    CANDY_HIP_W_HEAD = 10,      /* q  [vocab, d_model], layer = -1 */
    CANDY_HIP_W_EMBED = 11      /* q  [vocab, d_model], layer = -1 (row gather) */
};

int candy_hip_llama_create(candy_hip_device *dev, const candy_hip_llama_config *cfg, candy_hip_llama **out);
int candy_hip_llama_free(candy_hip_llama *m);
/* The model borrows the tensors; they must outlive it. */
int candy_hip_llama_set_qweight(candy_hip_llama *m, int which, int layer, const candy_hip_qtensor *w);
int candy_hip_llama_set_norm(candy_hip_llama *m, int which, int layer, const float *dev_alpha);
/* The decode step is captured into a HIP graph on first use and replayed afterwards (the
 * position and token travel through device memory); enable = 0 launches the kernels one by
 * one instead.  Results are identical either way. */
int candy_hip_llama_set_graph(candy_hip_llama *m, int enable);
/* Optional fp16 KV cache (off by default: candy's tensors are f32).  The new token's k (after Rope) and v are
 * rounded to fp16 once, as they enter the cache; attention reads them back as f32 and every product and sum
 * stays f32.  Halves the largest stream of a long-context decode step.  Changing the setting clears the cache.
 * No counterpart in the reference. */
int candy_hip_llama_set_kv_f16(candy_hip_llama *m, int enable);
/* KV cache, [n_layers][n_kv_heads][max_pos][head_dim] for K and the same for V: f32, or fp16 after
 * candy_hip_llama_set_kv_f16(m, 1) (bytes_each tells which). */
int candy_hip_llama_kv_cache(candy_hip_llama *m, float **dev_k, float **dev_v, size_t *bytes_each);
/* The residual stream [d_model] as the last decode step left it behind its last layer (before the final norm): a
 * device pointer owned by the model, valid until the next step.  What a candy model holds in its hidden-state tensor
 * between blocks; lets a caller run a model one block at a time (a one-layer model per block, its input through
 * candy_hip_llama_decode_hidden). */
int candy_hip_llama_hidden(candy_hip_llama *m, const float **dev_hidden);
/* One decode step: token id at position pos -> logits [vocab] (device pointer owned by the
 * model, valid until the next step) and the greedy next token.  Either output may be NULL. */
int candy_hip_llama_decode(candy_hip_llama *m, int32_t token, int32_t pos, const float **dev_logits,
                           int32_t *next_token);
/* n_steps greedy decode steps in a row, the host out of the loop: step 0 takes `token` at position pos, step i the
 * token step i-1 chose (handed over in device memory), at position pos + i; tokens[i] receives what step i chose.
 * The steps are enqueued back to back and the list is copied out once at the end, where n_steps calls of
 * candy_hip_llama_decode wait for the device and copy one token after every step (the same kernels and the same
 * tokens; 21 us less per token on the 7B shape).  No counterpart in the reference, which has no generation loop
 * (llm/ holds a FlashAttention binding only). */
int candy_hip_llama_generate(candy_hip_llama *m, int32_t token, int32_t pos, int32_t n_steps, int32_t *tokens);
/* Same step with the hidden state of the token given directly instead of an embedding row. */
int candy_hip_llama_decode_hidden(candy_hip_llama *m, const float *dev_hidden, int32_t pos,
                                  const float **dev_logits, int32_t *next_token);
/* Prompt pass: n_tokens token ids (host memory) enter the cache at positions pos0 .. pos0+n_tokens-1
 * in one batched pass -- every Linear is one [n_tokens, K] x W^T contraction (the MatMul call shape
 * of nn/linear.go:58-112 with m = n_tokens; MFMA tiles from 16 rows up), attention is causal over
 * the cache -- and the logits / greedy next token of the LAST prompt token come back.  Equivalent
 * to n_tokens successive candy_hip_llama_decode calls up to f32 summation order. */
int candy_hip_llama_prefill(candy_hip_llama *m, const int32_t *tokens, int32_t n_tokens, int32_t pos0,
                            const float **dev_logits, int32_t *next_token);

/* ------------------------------------------------------------------ timing (HIP events on the handle's stream) */
/* Runs `iters` contractions back to back, iteration i using weight ws[i % n_ws] (all the same
 * shape), and returns the elapsed time between HIP events recorded on the handle's stream
 * around the loop.  Rotating over more distinct weights than the last-level cache holds makes
 * every iteration stream from HBM.  quantize_each != 0: each iteration is the whole f32-in ->
 * f32-out path (activation quantization + contraction); 0: the activations are quantized once
 * before the timed region and each iteration is the contraction kernel alone. */
int candy_hip_qmatmul_sweep(candy_hip_device *dev, const candy_hip_qtensor *const *ws, int n_ws,
                            const float *dev_x, int64_t m, float *dev_y, int iters, int quantize_each,
                            float *elapsed_ms);
/* The two conversions timed the same way: `iters` dequantizations rotating over n_ws weights and over n_out
 * outputs laid end to end in dev_out (n_out * rows*cols f32), and `iters` Q8_0 quantizations of x[rows, cols] rotating
 * over n_x inputs spaced x_stride elements apart and n_out outputs end to end (each rows*cols/32 blocks).  Rotating
 * inputs AND outputs over more bytes than the last-level cache holds makes both sides HBM traffic. */
int candy_hip_dequantize_sweep(candy_hip_device *dev, const candy_hip_qtensor *const *ws, int n_ws,
                               float *dev_out, int n_out, int iters, float *elapsed_ms);
int candy_hip_quantize_sweep(candy_hip_device *dev, const float *dev_x, int64_t x_stride, int n_x, int64_t rows,
                             int64_t cols, void *dev_out_blocks, int n_out, int iters, float *elapsed_ms);
/* The same batch-1 contraction with the fixed part of a launch amortised or hidden (timing only; no counterpart in
 * the reference): every launch contracts `group` (1 .. 3) weights of the rotation that share the one quantized
 * activation row - the mechanism q / k / v use, after mul_mat_vec_q's one weight per launch (quantized.cu:2787-2871)
 * - and with n_streams = 2 the launches alternate between the handle's stream and a second stream the call creates,
 * so that one launch starts while the other drains.  dev_y holds n_streams * group * rows floats.  A figure for
 * independent contractions: a caller whose next contraction needs this one's result gets candy_hip_qmatmul_sweep's. */
int candy_hip_qmatmul_sustained_sweep(candy_hip_device *dev, const candy_hip_qtensor *const *ws, int n_ws, int group,
                                      int n_streams, const float *dev_x, float *dev_y, int iters, float *elapsed_ms);
/* What the device delivers to a kernel that only reads (no counterpart in the reference; the matvec's bytes per
 * second are quoted against it beside the published peak).  `iters` launches back to back, launch i reading
 * bytes_per_launch bytes (a multiple of 16) with 16-byte loads from region i of a scratch buffer of span_bytes
 * that the call allocates, zero-fills and frees; a span larger than the last-level cache makes every launch read
 * HBM.  bytes_per_launch = 0 times launches of an empty kernel.  Returns the time between HIP events recorded
 * on the handle's stream around the loop. */
int candy_hip_stream_probe(candy_hip_device *dev, size_t bytes_per_launch, size_t span_bytes, int iters,
                           float *elapsed_ms);
/* Where the fixed part of a launch goes (no counterpart in the reference; bench.py reports it beside the headline
 * kernel).  `iters` launches back to back of: kind 0 an empty kernel of one wavefront; 1 an empty kernel of 1024
 * workgroups x 256 threads (the grid of a 4096-row batch-1 contraction); 2 that grid with every wavefront issuing
 * one 16-byte load per lane, rows 6192 bytes apart, the same lines every launch (cache-warm); 3 the same with every
 * launch in a region of its own out of 640 MiB (cold).  Returns the time between HIP events around the loop. */
int candy_hip_launch_probe(candy_hip_device *dev, int kind, int iters, float *elapsed_ms);
int candy_hip_timer_start(candy_hip_device *dev);
int candy_hip_timer_stop(candy_hip_device *dev, float *elapsed_ms);   /* synchronises */

#ifdef __cplusplus
}
#endif
#endif
