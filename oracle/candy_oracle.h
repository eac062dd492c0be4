/*
 * candy_oracle.h -- CPU restatement of candy's quantized-matmul path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships (the HIP library, its host
 * wrappers) may include, link or call this.  It exists so that the GPU
 * results can be compared against the arithmetic candy defines:
 *   - tensor/internal/cpu/kernels/quantized.go  (block structs, fp16ToFloat32,
 *     Q4_0 / Q8_0 dequantize)
 *   - tensor/internal/cuda/kernels/quantized.cu (the only place candy holds
 *     Q4_K / Q6_K dequantize, activation quantization and the integer vec-dots)
 *   - tensor/internal/cpu/kernels/conv.go       (f32 matmul accumulation order)
 *   - tensor/internal/cpu/kernels/reduce.go, unary.go (decode-step glue ops)
 *
 * Pinning status of each function is listed in the header of candy_oracle.c.
 */
#ifndef CANDY_ORACLE_H
#define CANDY_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Format ids are the GGML type ids (the ids a GGUF file would carry). */
enum {
    CO_Q4_0 = 2,  /* candy CPU element order: y[2j]=lo(qs[j]), y[2j+1]=hi(qs[j]) */
    CO_Q8_0 = 8,
    CO_Q4_K = 12,
    CO_Q6_K = 14,
    CO_Q4_0_GGML = 102, /* ggml/CUDA element order: y[j]=lo(qs[j]), y[j+16]=hi(qs[j]) */
    /* the reference's other block formats (numbers are ggml's type ids) */
    CO_Q4_1 = 3,        /* candy CPU element order (QGO:107-116) */
    CO_Q4_1_GGML = 103, /* ggml/CUDA element order (QCU:728-746) */
    CO_Q5_0 = 6,
    CO_Q5_1 = 7,
    CO_Q2_K = 10,
    CO_Q3_K = 11,
    CO_Q5_K = 13,
    CO_Q8_K = 15        /* dequantize only: the reference has no weight vec-dot for it */
};

int co_block_elems(int fmt);  /* 32 or 256; 0 for an unknown format */
int co_block_bytes(int fmt);  /* 18, 34, 144, 210, 20, 22, 24, 84, 110, 176, 292; 0 for an unknown format */

float    co_fp16_to_f32(uint16_t h);
uint16_t co_f32_to_fp16(float f);

void co_get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m);

/* y receives n_blocks * co_block_elems(fmt) floats. Returns 0, or -1 for a bad format. */
int co_dequantize(int fmt, const void *blocks, int64_t n_blocks, float *y);

/* x: rows*cols f32, cols % 32 == 0. out: rows*cols/32 Q8_0 blocks (34 B each). */
int co_quantize_q8_0(const float *x, int64_t rows, int64_t cols, void *out_blocks);

/* Weight quantizer from f32 for any of the formats (ggml's reference quantizers; Q8_0 is the one
 * above): x is rows*cols f32, cols a multiple of the block; out receives rows*cols/qk blocks. */
int co_quantize(int fmt, const float *x, int64_t rows, int64_t cols, void *out_blocks);

/* Test hooks on the scale searches inside co_quantize (Q4_K sub-blocks: n = 32, nmax = 15, rmin = -1,
 * rdelta = 0.1, nstep = 20, weights rms + |x|; Q6_K groups: n = 16, nmax = 32). */
float co_make_qkx2_quants(int n, int nmax, const float *x, const float *weights, uint8_t *L, float *the_min,
                          float rmin, float rdelta, int nstep);
float co_make_qx_quants(int n, int nmax, const float *x, int8_t *L);

/* One weight row (k/qk blocks) against one activation row (k/32 Q8_0 blocks). */
float co_vec_dot_q8_0(int fmt, const void *w_row, const void *x_q8_0, int64_t k);

/* Test aid: the order in which co_vec_dot_q8_0 (and everything built on it) adds a row's blocks: 0 ascending
 * (the default), 1 descending, 2 even-numbered then odd-numbered, 3 second half then first.  Process-wide. */
void co_set_block_order(int order);

/* y[m, rows] = x[m, cols] . W^T with activations quantized to Q8_0 first. */
int co_qmatmul(int fmt, const void *w_blocks, int64_t rows, int64_t cols,
               const float *x, int64_t m, float *y);

/* candy's literal CPU composition: dequantize W, then the naive f32 loops. */
int co_matmul_dequant_f32(int fmt, const void *w_blocks, int64_t rows, int64_t cols,
                          const float *x, int64_t m, float *y);

void co_naive_batched_matmul_f32(int64_t b, int64_t m, int64_t n, int64_t k,
                                 const float *a, const float *bm, float *c);
void co_naive_batched_matmul_strided_f32(int64_t b, int64_t m, int64_t n, int64_t k,
                                         const float *a, const float *bm, float *c,
                                         const int64_t a_strides[3], const int64_t b_strides[3],
                                         const int64_t c_strides[3]);

/* decode-step glue */
void co_fast_rms_norm_f32(int64_t numel, int64_t ncols, float eps, const float *alpha,
                          const float *x, float *dst);
void co_rope_f32(int64_t bh, int64_t td, int64_t d, int64_t stride_b, const float *src,
                 const float *cos_t, const float *sin_t, float *dst);
void co_rope_i_f32(int64_t bh, int64_t td, int64_t stride_b, const float *src, const float *cos_t,
                   const float *sin_t, float *dst);
void co_rope_thd_f32(int64_t b, int64_t t, int64_t h, int64_t d, int64_t stride_b, const float *src,
                     const float *cos_t, const float *sin_t, float *dst);
void co_fast_softmax_f32(int64_t numel, int64_t ncols, const float *src, float *dst);
void co_silu_f32(int64_t numel, const float *inp, float *out);
void co_fast_argmax_f32(int64_t numel, int64_t ncols, const float *src, uint32_t *dst);
void co_index_select_f32(int64_t numel, const int64_t *ids, const float *inp, float *out,
                         int64_t left, int64_t src_dim, int64_t ids_dim, int64_t right);
void co_add_f32(int64_t n, const float *a, const float *b, float *out);
void co_mul_f32(int64_t n, const float *a, const float *b, float *out);

/* Batch-1 attention for one new token over an f32 KV cache, composed from the ops
 * above: scores = q.K^T * scale (naive f32 loop), FastSoftmax, out = p.V (naive loop).
 * k_cache, v_cache: [n_kv_heads, n_pos, head_dim]; q, out: [n_heads, head_dim].
 * cache_stride = elements between consecutive kv heads (>= n_pos*head_dim). */
void co_attention_decode_f32(const float *q, const float *k_cache, const float *v_cache,
                             int64_t n_heads, int64_t n_kv_heads, int64_t head_dim,
                             int64_t n_pos, int64_t cache_stride, float scale, float *out);

#ifdef __cplusplus
}
#endif
#endif
