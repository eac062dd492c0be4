/*
 * candy_oracle.c -- CPU restatement of candy's quantized-matmul path.
 *
 * TEST INFRASTRUCTURE ONLY: used by tests/, the smoke check and the CPU-baseline
 * leg of the benchmark as the checker.  The shipped HIP library never links it.
 *
 * Build with -ffp-contract=off: every f32 expression below is meant to round
 * once per operation, exactly as written.
 *
 * Reference files are cited relative to the candy checkout:
 *   QGO  = tensor/internal/cpu/kernels/quantized.go
 *   QCU  = tensor/internal/cuda/kernels/quantized.cu
 *   CONV = tensor/internal/cpu/kernels/conv.go
 *   RED  = tensor/internal/cpu/kernels/reduce.go
 *   UNA  = tensor/internal/cpu/kernels/unary.go
 *   IDX  = tensor/internal/cpu/kernels/indexing.go
 *
 * Pinning status (what fixes each function besides this restatement itself;
 * the checks live in tests/test_oracle_*.py):
 *   co_fp16_to_f32        QGO:149-173. Pinned: all 65536 inputs against numpy's IEEE
 *                         float16->float32 (bit patterns, NaN payloads included).
 *   co_f32_to_fp16        no reference implementation (candy never narrows to fp16 on
 *                         the CPU; QCU:3556 relies on the hardware conversion). Pinned:
 *                         round-to-nearest-even against numpy's float32->float16 on all
 *                         fp16 values, all midpoints and a random sweep.
 *   co_dequantize Q4_0    QGO:85-93 (interleaved order). Pinned: exact rational values
 *                         with Python Fractions; order relation to the ggml order QCU:862-866.
 *   co_dequantize Q8_0    QGO:131-136. Pinned: exact rational values.
 *   co_get_scale_min_k4   QCU:993-1005. Pinned: against an independent reading of the
 *                         16-bit masked unpack QCU:2600-2612 over random and exhaustive
 *                         byte-pair patterns.
 *   co_dequantize Q4_K    QCU:1008-1041. Pinned: exact value (one rounding) in Fractions.
 *   co_dequantize Q6_K    QCU:1103-1128. Pinned: exact value in Fractions.
 *   co_dequantize Q4_1    QGO:107-116 (candy CPU order) and QCU:728-746 (ggml order). Pinned: exact
 *                         rational values; the two orders are a permutation of each other.
 *   co_dequantize Q5_0/Q5_1  QCU:749-795 through dequantize_block (QCU:1208-1216). Pinned: exact values.
 *   co_dequantize Q2_K    QCU:902-935.   Pinned: exact value rounded once (Fractions).
 *   co_dequantize Q3_K    QCU:936-990.   Pinned: exact value (no rounding happens: 17-bit scale x 3-bit level).
 *   co_dequantize Q5_K    QCU:1054-1102. Pinned: exact value rounded once.
 *   co_dequantize Q8_K    QCU:1178-1206. Pinned: exact value rounded once.
 *   vec-dots of these     QCU:1947-2053 (Q4_1, Q5_0, Q5_1), 2108-2135 (Q2_K), 2177-2209 (Q3_K),
 *                         2300-2331 (Q5_K): integer dot products per scale group, combined in f32 as the
 *                         kernels do, the Q8_1 `sum` half replaced by the exact integer block sum.
 *                         Pinned: against the exact-arithmetic sum of dequantized products.
 *   co_quantize_q8_0      QCU:3521-3558 without the `sum` half. Pinned: float64 evaluation
 *                         of round-half-away(x/d) with numpy float32 division; invariants.
 *   co_quantize (Q4_0 / Q4_0_GGML / Q4_K / Q6_K)
 *                         PARITY UNPINNED against the original.  candy has no quantizer from f32
 *                         (only kernel names, tensor/internal/metal/kernels/kernels.go:563-592);
 *                         the algorithm is ggml's published reference quantizer, which is not in
 *                         the checkout: quantize_row_q4_0_ref, quantize_row_q4_K_ref with
 *                         make_qkx2_quants, quantize_row_q6_K_ref with make_qx_quants
 *                         (ggml/src/ggml-quants.c of llama.cpp, 2024 releases; candle's
 *                         k_quants.rs `from_float` is a port of the same).  Restated here from
 *                         the published algorithm.  What the tests do pin: Q4_0 against an
 *                         independent numpy evaluation of its closed form; for the K formats the
 *                         level-assignment pass against the stored scales (recomputed from the
 *                         block in Fractions), the error bound of the result, that the searched
 *                         scale is never worse in the weighted objective than plain rounding,
 *                         special blocks (zeros, constants, a single spike), and determinism.
 *   co_vec_dot_q8_0       QCU:2058-2073, 2239-2263, 2367-2389 (shape of the float
 *                         combination); integer parts pinned with Python ints, the float
 *                         result against exact-arithmetic sum of dequantized products.
 *   co_set_block_order    test aid, no reference counterpart: the same terms of a row added in another order
 *                         (descending, even then odd, second half first).  Pinned: equals the ascending sum to
 *                         1e-6 per Linear; the terms themselves are the pinned ones.
 *   co_qmatmul            authored here (candy has no CPU QMatMul); pinned as above.
 *   co_matmul_dequant_f32 CONV:373-389 applied to dequantized weights.
 *   co_naive_batched_*    CONV:251-267, 373-389. Pinned: reference fixtures of
 *                         conv_test.go:11-65.
 *   co_fast_rms_norm_f32  RED:3071-3092. Pinned: reduce_test.go:1909-1971 fixtures.
 *   co_rope_f32           RED:3987-4006. Pinned: reduce_test.go:2775-2832 fixtures.
 *   co_rope_i_f32         RED:3825-3838. Pinned: reduce_test.go:2507-2560 fixtures; a rotation of adjacent pairs (float64).
 *   co_rope_thd_f32       RED:4178-4196. Pinned: reduce_test.go:3033-3094 fixtures; equals co_rope_f32 on the transposed layout.
 *   co_fast_softmax_f32   RED:2855-2879. Pinned: reduce_test.go:1665-1717 fixtures.
 *   co_silu_f32           UNA:3353-3366. Pinned: unary_test.go:4199-4241 closed form.
 *   co_fast_argmax_f32    RED:846-862. Pinned: reduce_test.go:1063-1113 fixtures.
 *   co_index_select_f32   IDX:8-26. Pinned: gather identity against numpy take.
 *   co_attention_decode_f32  authored here as a composition of the ops above (candy has
 *                         no attention on the CPU); pinned against a float64 numpy evaluation.
 */
#include "candy_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ---- block layouts: QGO:8-11, 34-37, 55-59, 70-75; sizes asserted at QCU:305,347,410,444 ---- */
#pragma pack(push, 1)
typedef struct { uint16_t d; uint8_t qs[16]; } co_block_q4_0;
typedef struct { uint16_t d; int8_t qs[32]; } co_block_q8_0;
typedef struct { uint16_t dm[2]; uint8_t scales[12]; uint8_t qs[128]; } co_block_q4_k;
typedef struct { uint8_t ql[128]; uint8_t qh[64]; int8_t scales[16]; uint16_t d; } co_block_q6_k;
/* QGO:13-31, 39-52, 62-67, 78-82; QCU:310-336, 370-390, 416-431, 447-452 */
typedef struct { uint16_t dm[2]; uint8_t qs[16]; } co_block_q4_1;
typedef struct { uint16_t d; uint8_t qh[4]; uint8_t qs[16]; } co_block_q5_0;
typedef struct { uint16_t dm[2]; uint8_t qh[4]; uint8_t qs[16]; } co_block_q5_1;
typedef struct { uint8_t scales[16]; uint8_t qs[64]; uint16_t dm[2]; } co_block_q2_k;
typedef struct { uint8_t hmask[32]; uint8_t qs[64]; uint8_t scales[12]; uint16_t d; } co_block_q3_k;
typedef struct { uint16_t dm[2]; uint8_t scales[12]; uint8_t qh[32]; uint8_t qs[128]; } co_block_q5_k;
typedef struct { float d; int8_t qs[256]; int16_t bsums[16]; } co_block_q8_k;
#pragma pack(pop)
_Static_assert(sizeof(co_block_q4_1) == 20 && sizeof(co_block_q5_0) == 22 && sizeof(co_block_q5_1) == 24, "32-value blocks");
_Static_assert(sizeof(co_block_q2_k) == 84 && sizeof(co_block_q3_k) == 110, "q2_K / q3_K");
_Static_assert(sizeof(co_block_q5_k) == 176 && sizeof(co_block_q8_k) == 292, "q5_K / q8_K");

_Static_assert(sizeof(co_block_q4_0) == 18, "q4_0");
_Static_assert(sizeof(co_block_q8_0) == 34, "q8_0");
_Static_assert(sizeof(co_block_q4_k) == 144, "q4_K");
_Static_assert(sizeof(co_block_q6_k) == 210, "q6_K");

int co_block_elems(int fmt) {
    switch (fmt) {
    case CO_Q4_0: case CO_Q4_0_GGML: case CO_Q8_0: return 32;
    case CO_Q4_1: case CO_Q4_1_GGML: case CO_Q5_0: case CO_Q5_1: return 32;
    case CO_Q4_K: case CO_Q6_K: return 256;
    case CO_Q2_K: case CO_Q3_K: case CO_Q5_K: case CO_Q8_K: return 256;
    default: return 0;
    }
}

int co_block_bytes(int fmt) {
    switch (fmt) {
    case CO_Q4_0: case CO_Q4_0_GGML: return 18;
    case CO_Q8_0: return 34;
    case CO_Q4_K: return 144;
    case CO_Q6_K: return 210;
    case CO_Q4_1: case CO_Q4_1_GGML: return 20;
    case CO_Q5_0: return 22;
    case CO_Q5_1: return 24;
    case CO_Q2_K: return 84;
    case CO_Q3_K: return 110;
    case CO_Q5_K: return 176;
    case CO_Q8_K: return 292;
    default: return 0;
    }
}

static float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* QGO:149-173 */
float co_fp16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (uint32_t)(h & 0x7C00u);
    uint32_t mant = (uint32_t)(h & 0x03FFu);
    if (exp == 0x7C00u) /* inf / NaN keeps the payload shifted up: QGO:156 */
        return bits_to_f32(sign | 0x7F800000u | (mant << 13));
    if (exp == 0) {
        if (mant == 0) return bits_to_f32(sign);
        exp = (127u - 14u) << 23; /* QGO:162-168: normalise the subnormal */
        while ((mant & 0x400u) == 0) { mant <<= 1; exp -= 1u << 23; }
        mant &= 0x3FFu;
        return bits_to_f32(sign | exp | (mant << 13));
    }
    return bits_to_f32(sign | ((((exp >> 10) - 15u + 127u) << 23)) | (mant << 13));
}

/* IEEE-754 binary32 -> binary16, round to nearest even (what QCU:3556 gets from the
 * hardware conversion when it stores `d` into a half). */
uint16_t co_f32_to_fp16(float f) {
    uint32_t x = f32_to_bits(f);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) { /* inf / NaN */
        if (ax == 0x7F800000u) return (uint16_t)(sign | 0x7C00u);
        uint16_t payload = (uint16_t)((ax >> 13) & 0x3FFu);
        return (uint16_t)(sign | 0x7C00u | 0x200u | payload); /* quiet NaN, keep top payload bits */
    }
    if (ax >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* >= 65520 rounds to inf */
    if (ax < 0x33000001u) return sign;                          /* <= 2^-25 rounds to zero */
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t m = (ax & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
    uint32_t shift, half_e;
    if (e < -14) { shift = (uint32_t)(13 + (-14 - e)); half_e = 0; }
    else { shift = 13; half_e = (uint32_t)(e + 15); }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) q++;
    /* for normals q carries the implicit bit (0x400); adding the exponent field on top
     * lets a mantissa overflow carry into the exponent naturally */
    uint32_t out = (half_e == 0) ? q : ((half_e - 1u) << 10) + q;
    return (uint16_t)(sign | out);
}

/* QCU:993-1005 */
void co_get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* QGO:85-93: interleaved element order */
static void dequant_q4_0(const co_block_q4_0 *b, float *y) {
    float d = co_fp16_to_f32(b->d);
    for (int i = 0; i < 32; i += 2) {
        int q1 = b->qs[i / 2] & 0xF;
        int q2 = b->qs[i / 2] >> 4;
        y[i] = d * ((float)q1 - 8.0f);
        y[i + 1] = d * ((float)q2 - 8.0f);
    }
}

/* QCU:862-866: low nibbles first, then high nibbles; d*q + (-8d) */
static void dequant_q4_0_ggml(const co_block_q4_0 *b, float *y) {
    float d = co_fp16_to_f32(b->d);
    float dm = -8.0f * d;
    for (int l = 0; l < 16; ++l) {
        y[l] = d * (float)(b->qs[l] & 0xF) + dm;
        y[l + 16] = d * (float)(b->qs[l] >> 4) + dm;
    }
}

/* QGO:131-136 */
static void dequant_q8_0(const co_block_q8_0 *b, float *y) {
    float d = co_fp16_to_f32(b->d);
    for (int i = 0; i < 32; ++i) y[i] = d * (float)b->qs[i];
}

/* QCU:1008-1041: group il of 64 values; low nibbles use scale 2il, high use 2il+1 */
static void dequant_q4_k(const co_block_q4_k *b, float *y) {
    float dall = co_fp16_to_f32(b->dm[0]);
    float dmin = co_fp16_to_f32(b->dm[1]);
    for (int il = 0; il < 4; ++il) {
        uint8_t sc, m;
        co_get_scale_min_k4(2 * il, b->scales, &sc, &m);
        float d1 = dall * (float)sc, m1 = dmin * (float)m;
        co_get_scale_min_k4(2 * il + 1, b->scales, &sc, &m);
        float d2 = dall * (float)sc, m2 = dmin * (float)m;
        const uint8_t *q = b->qs + 32 * il;
        for (int l = 0; l < 32; ++l) {
            y[64 * il + l] = d1 * (float)(q[l] & 0xF) - m1;
            y[64 * il + 32 + l] = d2 * (float)(q[l] >> 4) - m2;
        }
    }
}

/* QCU:1103-1128 */
static void dequant_q6_k(const co_block_q6_k *b, float *y) {
    float d = co_fp16_to_f32(b->d);
    for (int ip = 0; ip < 2; ++ip) {
        for (int il = 0; il < 32; ++il) {
            int is = 8 * ip + il / 16;
            const uint8_t *ql = b->ql + 64 * ip + il;
            uint8_t qh = b->qh[32 * ip + il];
            const int8_t *sc = b->scales + is;
            float *yy = y + 128 * ip + il;
            yy[0] = d * (float)sc[0] * (float)((int8_t)((ql[0] & 0xF) | (((qh >> 0) & 3) << 4)) - 32);
            yy[32] = d * (float)sc[2] * (float)((int8_t)((ql[32] & 0xF) | (((qh >> 2) & 3) << 4)) - 32);
            yy[64] = d * (float)sc[4] * (float)((int8_t)((ql[0] >> 4) | (((qh >> 4) & 3) << 4)) - 32);
            yy[96] = d * (float)sc[6] * (float)((int8_t)((ql[32] >> 4) | (((qh >> 6) & 3) << 4)) - 32);
        }
    }
}

/* QGO:107-116: y[2j] = d*lo(qs[j]) + m, y[2j+1] = d*hi(qs[j]) + m */
static void dequant_q4_1(const co_block_q4_1 *b, float *y) {
    const float d = co_fp16_to_f32(b->dm[0]), m = co_fp16_to_f32(b->dm[1]);
    for (int i = 0; i < 32; i += 2) {
        y[i] = d * (float)(b->qs[i / 2] & 0xF) + m;
        y[i + 1] = d * (float)(b->qs[i / 2] >> 4) + m;
    }
}

/* QCU:728-746 placed by dequantize_block (QCU:870-899): y[j] = d*lo(qs[j]) + m, y[j+16] = d*hi(qs[j]) + m */
static void dequant_q4_1_ggml(const co_block_q4_1 *b, float *y) {
    const float d = co_fp16_to_f32(b->dm[0]), m = co_fp16_to_f32(b->dm[1]);
    for (int j = 0; j < 16; ++j) {
        y[j] = d * (float)(b->qs[j] & 0xF) + m;
        y[j + 16] = d * (float)(b->qs[j] >> 4) + m;
    }
}

/* the 5-bit level of element e (0..31): nibble of qs[e % 16] (low for e < 16), bit e of qh on top: QCU:756-763 */
static int q5_level(const uint8_t *qs, const uint8_t *qh4, int e) {
    uint32_t qh;
    memcpy(&qh, qh4, 4);
    const int nib = e < 16 ? (qs[e] & 0xF) : (qs[e - 16] >> 4);
    return nib | (int)(((qh >> e) & 1u) << 4);
}

/* QCU:749-770: (level - 16) * d */
static void dequant_q5_0(const co_block_q5_0 *b, float *y) {
    const float d = co_fp16_to_f32(b->d);
    for (int e = 0; e < 32; ++e) y[e] = ((float)q5_level(b->qs, b->qh, e) - 16.0f) * d;
}

/* QCU:773-795: level * d + m */
static void dequant_q5_1(const co_block_q5_1 *b, float *y) {
    const float d = co_fp16_to_f32(b->dm[0]), m = co_fp16_to_f32(b->dm[1]);
    for (int e = 0; e < 32; ++e) y[e] = (float)q5_level(b->qs, b->qh, e) * d + m;
}

/* QCU:902-920: element 128n + 32k + l is bits 2k.. of qs[32n + l]; its 16-value group e/16 has a 4-bit
 * scale (low nibble) and a 4-bit min (high nibble): y = dall*scale*q - dmin*min */
static void dequant_q2_k(const co_block_q2_k *b, float *y) {
    const float dall = co_fp16_to_f32(b->dm[0]), dmin = co_fp16_to_f32(b->dm[1]);
    for (int e = 0; e < 256; ++e) {
        const int n = e / 128, k = (e % 128) / 32, l = e % 32;
        const uint8_t sc = b->scales[e / 16];
        const int q = (b->qs[32 * n + l] >> (2 * k)) & 3;
        y[e] = dall * (float)(sc & 0xF) * (float)q - dmin * (float)(sc >> 4);
    }
}

/* the 6-bit scale of 16-value group is (0..15) of a Q3_K block: QCU:953-956 */
static int q3k_scale(const uint8_t *sc, int is) {
    if (is < 4) return (sc[is] & 0xF) | (((sc[is + 8] >> 0) & 3) << 4);
    if (is < 8) return (sc[is] & 0xF) | (((sc[is + 4] >> 2) & 3) << 4);
    if (is < 12) return (sc[is - 8] >> 4) | (((sc[is] >> 4) & 3) << 4);
    return (sc[is - 8] >> 4) | (((sc[is - 4] >> 6) & 3) << 4);
}

/* the level -4..3 of element e = 128n + 32j + l: two bits of qs[32n + l], minus 4 unless bit 4n + j of hmask[l] is set */
static int q3k_level(const co_block_q3_k *b, int e) {
    const int n = e / 128, j = (e % 128) / 32, l = e % 32;
    const int q = (b->qs[32 * n + l] >> (2 * j)) & 3;
    return q - ((b->hmask[l] >> (4 * n + j)) & 1 ? 0 : 4);
}

/* QCU:936-966: y = d*(scale - 32) * level */
static void dequant_q3_k(const co_block_q3_k *b, float *y) {
    const float d_all = co_fp16_to_f32(b->d);
    for (int e = 0; e < 256; ++e) {
        const float dl = d_all * (float)(q3k_scale(b->scales, e / 16) - 32);
        y[e] = dl * (float)q3k_level(b, e);
    }
}

/* the 5-bit level of element e of a Q5_K block: sub-block t = e/32 takes the low (t even) or high nibble of
 * qs[32*(t/2) + l] and bit t of qh[l]: QCU:1068-1087 */
static int q5k_level(const co_block_q5_k *b, int e) {
    const int t = e / 32, l = e % 32;
    const uint8_t q = b->qs[32 * (t / 2) + l];
    return ((t & 1) ? (q >> 4) : (q & 0xF)) + (((b->qh[l] >> t) & 1) ? 16 : 0);
}

/* QCU:1054-1087: y = (dall*sc)*level - dmin*m with the (sc, m) of the sub-block (get_scale_min_k4) */
static void dequant_q5_k(const co_block_q5_k *b, float *y) {
    const float dall = co_fp16_to_f32(b->dm[0]), dmin = co_fp16_to_f32(b->dm[1]);
    for (int t = 0; t < 8; ++t) {
        uint8_t sc, m;
        co_get_scale_min_k4(t, b->scales, &sc, &m);
        const float d1 = dall * (float)sc, m1 = dmin * (float)m;
        for (int l = 0; l < 32; ++l) y[32 * t + l] = d1 * (float)q5k_level(b, 32 * t + l) - m1;
    }
}

/* QCU:1178-1199: y = q * d, d in f32 */
static void dequant_q8_k(const co_block_q8_k *b, float *y) {
    for (int e = 0; e < 256; ++e) y[e] = (float)b->qs[e] * b->d;
}

int co_dequantize(int fmt, const void *blocks, int64_t n_blocks, float *y) {
    switch (fmt) {
    case CO_Q4_1:
        for (int64_t i = 0; i < n_blocks; ++i) dequant_q4_1((const co_block_q4_1 *)blocks + i, y + 32 * i);
        return 0;
    case CO_Q4_1_GGML:
        for (int64_t i = 0; i < n_blocks; ++i) dequant_q4_1_ggml((const co_block_q4_1 *)blocks + i, y + 32 * i);
        return 0;
    case CO_Q5_0:
        for (int64_t i = 0; i < n_blocks; ++i) dequant_q5_0((const co_block_q5_0 *)blocks + i, y + 32 * i);
        return 0;
    case CO_Q5_1:
        for (int64_t i = 0; i < n_blocks; ++i) dequant_q5_1((const co_block_q5_1 *)blocks + i, y + 32 * i);
        return 0;
    case CO_Q2_K:
        for (int64_t i = 0; i < n_blocks; ++i) dequant_q2_k((const co_block_q2_k *)blocks + i, y + 256 * i);
        return 0;
    case CO_Q3_K:
        for (int64_t i = 0; i < n_blocks; ++i) dequant_q3_k((const co_block_q3_k *)blocks + i, y + 256 * i);
        return 0;
    case CO_Q5_K:
        for (int64_t i = 0; i < n_blocks; ++i) dequant_q5_k((const co_block_q5_k *)blocks + i, y + 256 * i);
        return 0;
    case CO_Q8_K:
        for (int64_t i = 0; i < n_blocks; ++i) dequant_q8_k((const co_block_q8_k *)blocks + i, y + 256 * i);
        return 0;
    case CO_Q4_0:
        for (int64_t i = 0; i < n_blocks; ++i) dequant_q4_0((const co_block_q4_0 *)blocks + i, y + 32 * i);
        return 0;
    case CO_Q4_0_GGML:
        for (int64_t i = 0; i < n_blocks; ++i) dequant_q4_0_ggml((const co_block_q4_0 *)blocks + i, y + 32 * i);
        return 0;
    case CO_Q8_0:
        for (int64_t i = 0; i < n_blocks; ++i) dequant_q8_0((const co_block_q8_0 *)blocks + i, y + 32 * i);
        return 0;
    case CO_Q4_K:
        for (int64_t i = 0; i < n_blocks; ++i) dequant_q4_k((const co_block_q4_k *)blocks + i, y + 256 * i);
        return 0;
    case CO_Q6_K:
        for (int64_t i = 0; i < n_blocks; ++i) dequant_q6_k((const co_block_q6_k *)blocks + i, y + 256 * i);
        return 0;
    default:
        return -1;
    }
}

/* QCU:3521-3558 with the `sum` half dropped (Q8_0 instead of Q8_1).
 * amax is a NaN-ignoring maximum (fmaxf, as warp_reduce_max uses); d = amax/127 in f32;
 * q = amax == 0 ? 0 : roundf(x/d) with the UNROUNDED d; the stored scale is fp16(d). */
int co_quantize_q8_0(const float *x, int64_t rows, int64_t cols, void *out_blocks) {
    if (cols % 32 != 0 || rows < 0 || cols < 0) return -1;
    co_block_q8_0 *out = (co_block_q8_0 *)out_blocks;
    int64_t nb = rows * cols / 32;
    for (int64_t b = 0; b < nb; ++b) {
        const float *xb = x + 32 * b;
        float amax = 0.0f;
        for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(xb[i]));
        const float d = amax / 127.0f;
        for (int i = 0; i < 32; ++i)
            out[b].qs[i] = (amax == 0.0f) ? 0 : (int8_t)roundf(xb[i] / d);
        out[b].d = co_f32_to_fp16(d);
    }
    return 0;
}

/* ---- weight quantizers from f32 (ggml's reference quantizers, see the header: parity unpinned) ---- */

/* Round to nearest, ties to even, by the 1.5 * 2^23 trick; |f| <= 4194303. */
static int nearest_int(float f) {
    const float v = f + 12582912.0f;
    return (int)(f32_to_bits(v) & 0x007FFFFFu) - 0x00400000;
}

/* quantize_row_q4_0_ref: the element of largest magnitude maps to level -8 (so d carries its sign);
 * levels are (int8)(x / d + 8.5) capped at 15.  ggml_order: low nibbles hold elements 0..15 and high
 * nibbles 16..31 (QCU:862-866); otherwise candy's CPU order, byte i = elements 2i, 2i+1 (QGO:85-93). */
static void quantize_block_q4_0(const float *x, co_block_q4_0 *y, int ggml_order) {
    float amax = 0.0f, max = 0.0f;
    for (int j = 0; j < 32; ++j) {
        const float v = x[j];
        if (amax < fabsf(v)) { amax = fabsf(v); max = v; }
    }
    const float d = max / -8.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    y->d = co_f32_to_fp16(d);
    uint8_t q[32];
    for (int j = 0; j < 32; ++j) {
        const int v = (int)(int8_t)(x[j] * id + 8.5f);
        q[j] = (uint8_t)(v < 15 ? v : 15);
    }
    for (int j = 0; j < 16; ++j)
        y->qs[j] = ggml_order ? (uint8_t)(q[j] | (q[j + 16] << 4)) : (uint8_t)(q[2 * j] | (q[2 * j + 1] << 4));
}

/* make_qkx2_quants: levels 0..nmax with scale and (non-positive) minimum for n values; starts from
 * min/max rounding and tries nstep+1 nearby scales, each followed by the weighted least-squares fit
 * of (scale, min) to the levels it yields; keeps the best weighted squared error.  Returns the scale,
 * *the_min receives -min (>= 0). */
static float make_qkx2_quants(int n, int nmax, const float *x, const float *weights, uint8_t *L, float *the_min,
                              uint8_t *Laux, float rmin, float rdelta, int nstep) {
    float min = x[0], max = x[0];
    float sum_w = weights[0], sum_x = sum_w * x[0];
    for (int i = 1; i < n; ++i) {
        if (x[i] < min) min = x[i];
        if (x[i] > max) max = x[i];
        const float w = weights[i];
        sum_w += w;
        sum_x += w * x[i];
    }
    if (min > 0.0f) min = 0.0f;
    if (max == min) {
        for (int i = 0; i < n; ++i) L[i] = 0;
        *the_min = -min;
        return 0.0f;
    }
    float iscale = (float)nmax / (max - min);
    float scale = 1.0f / iscale;
    float best = 0.0f;
    for (int i = 0; i < n; ++i) {
        int l = nearest_int(iscale * (x[i] - min));
        l = l < 0 ? 0 : (l > nmax ? nmax : l);
        L[i] = (uint8_t)l;
        float diff = scale * (float)L[i] + min - x[i];
        diff = diff * diff;
        best += weights[i] * diff;
    }
    if (nstep < 1) {
        *the_min = -min;
        return scale;
    }
    for (int is = 0; is <= nstep; ++is) {
        iscale = (rmin + rdelta * (float)is + (float)nmax) / (max - min);
        float sum_l = 0.0f, sum_l2 = 0.0f, sum_xl = 0.0f;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int(iscale * (x[i] - min));
            l = l < 0 ? 0 : (l > nmax ? nmax : l);
            Laux[i] = (uint8_t)l;
            const float w = weights[i];
            sum_l += w * (float)l;
            sum_l2 += w * (float)l * (float)l;
            sum_xl += w * (float)l * x[i];
        }
        const float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0.0f) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0.0f) {
                this_min = 0.0f;
                this_scale = sum_xl / sum_l2;
            }
            float mad = 0.0f;
            for (int i = 0; i < n; ++i) {
                float diff = this_scale * (float)Laux[i] + this_min - x[i];
                diff = diff * diff;
                mad += weights[i] * diff;
            }
            if (mad < best) {
                for (int i = 0; i < n; ++i) L[i] = Laux[i];
                best = mad;
                scale = this_scale;
                min = this_min;
            }
        }
    }
    *the_min = -min;
    return scale;
}

/* Test hooks: the two searches on their own, so that a test can hold their answer against a brute-force
 * evaluation of every candidate the published algorithms name. */
float co_make_qkx2_quants(int n, int nmax, const float *x, const float *weights, uint8_t *L, float *the_min,
                          float rmin, float rdelta, int nstep) {
    uint8_t Laux[256];
    if (n < 1 || n > 256) return NAN;
    return make_qkx2_quants(n, nmax, x, weights, L, the_min, Laux, rmin, rdelta, nstep);
}

/* quantize_row_q4_K_ref for one super-block: eight 32-value sub-blocks get (scale, min) from
 * make_qkx2_quants with weights rms + |x|; scales and mins are stored in 6 bits relative to their
 * maxima (d, dmin in fp16), then the levels are assigned again with the STORED scales. */
static void quantize_block_q4_k(const float *x, co_block_q4_k *y) {
    uint8_t L[256], Laux[32];
    float weights[32], mins[8], scales[8];
    float max_scale = 0.0f, max_min = 0.0f;
    for (int j = 0; j < 8; ++j) {
        float sum_x2 = 0.0f;
        for (int l = 0; l < 32; ++l) sum_x2 += x[32 * j + l] * x[32 * j + l];
        const float av_x = sqrtf(sum_x2 / 32.0f);
        for (int l = 0; l < 32; ++l) weights[l] = av_x + fabsf(x[32 * j + l]);
        scales[j] = make_qkx2_quants(32, 15, x + 32 * j, weights, L + 32 * j, &mins[j], Laux, -1.0f, 0.1f, 20);
        if (scales[j] > max_scale) max_scale = scales[j];
        if (mins[j] > max_min) max_min = mins[j];
    }
    const float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    const float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    memset(y->scales, 0, sizeof(y->scales));
    for (int j = 0; j < 8; ++j) {
        int ls = nearest_int(inv_scale * scales[j]);
        int lm = nearest_int(inv_min * mins[j]);
        ls = ls < 63 ? ls : 63;
        lm = lm < 63 ? lm : 63;
        if (j < 4) {
            y->scales[j] = (uint8_t)ls;
            y->scales[j + 4] = (uint8_t)lm;
        } else {
            y->scales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
            y->scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
            y->scales[j] |= (uint8_t)((lm >> 4) << 6);
        }
    }
    y->dm[0] = co_f32_to_fp16(max_scale / 63.0f);
    y->dm[1] = co_f32_to_fp16(max_min / 63.0f);
    for (int j = 0; j < 8; ++j) {
        uint8_t sc, m;
        co_get_scale_min_k4(j, y->scales, &sc, &m);
        const float d = co_fp16_to_f32(y->dm[0]) * (float)sc;
        if (d == 0.0f) continue;  /* keeps the levels of the search */
        const float dm = co_fp16_to_f32(y->dm[1]) * (float)m;
        for (int ii = 0; ii < 32; ++ii) {
            int l = nearest_int((x[32 * j + ii] + dm) / d);
            l = l < 0 ? 0 : (l > 15 ? 15 : l);
            L[32 * j + ii] = (uint8_t)l;
        }
    }
    uint8_t *q = y->qs;
    for (int j = 0; j < 256; j += 64) {
        for (int l = 0; l < 32; ++l) q[l] = (uint8_t)(L[j + l] | (L[j + l + 32] << 4));
        q += 32;
    }
}

/* make_qx_quants with rmse_type 1 (weights x^2) and no external weights: symmetric levels
 * -nmax..nmax-1 stored as L = level + nmax; the value of largest magnitude maps to -nmax; 18 nearby
 * scales are tried and the one with the largest (sum w x l)^2 / (sum w l^2) kept. */
static float make_qx_quants(int n, int nmax, const float *x, int8_t *L) {
    float max = 0.0f, amax = 0.0f;
    for (int i = 0; i < n; ++i) {
        const float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; max = x[i]; }
    }
    if (amax < 1e-15f) {
        for (int i = 0; i < n; ++i) L[i] = 0;
        return 0.0f;
    }
    float iscale = -(float)nmax / max;
    float sumlx = 0.0f, suml2 = 0.0f;
    for (int i = 0; i < n; ++i) {
        int l = nearest_int(iscale * x[i]);
        l = l < -nmax ? -nmax : (l > nmax - 1 ? nmax - 1 : l);
        L[i] = (int8_t)(l + nmax);
        const float w = x[i] * x[i];
        sumlx += w * x[i] * (float)l;
        suml2 += w * (float)l * (float)l;
    }
    float scale = suml2 != 0.0f ? sumlx / suml2 : 0.0f;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; ++is) {
        if (is == 0) continue;
        iscale = -((float)nmax + 0.1f * (float)is) / max;
        sumlx = suml2 = 0.0f;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int(iscale * x[i]);
            l = l < -nmax ? -nmax : (l > nmax - 1 ? nmax - 1 : l);
            const float w = x[i] * x[i];
            sumlx += w * x[i] * (float)l;
            suml2 += w * (float)l * (float)l;
        }
        if (suml2 > 0.0f && sumlx * sumlx > best * suml2) {
            for (int i = 0; i < n; ++i) {
                int l = nearest_int(iscale * x[i]);
                l = l < -nmax ? -nmax : (l > nmax - 1 ? nmax - 1 : l);
                L[i] = (int8_t)(nmax + l);
            }
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

float co_make_qx_quants(int n, int nmax, const float *x, int8_t *L) { return make_qx_quants(n, nmax, x, L); }

/* quantize_row_q6_K_ref for one super-block: sixteen 16-value groups, each with a make_qx_quants
 * scale; the scale of largest magnitude maps to -128 in int8 (d in fp16 carries its sign), then
 * the levels -32..31 are assigned again with the STORED scales and packed as QCU:1103-1128 reads them. */
static void quantize_block_q6_k(const float *x, co_block_q6_k *y) {
    int8_t L[256];
    float scales[16];
    float max_scale = 0.0f, max_abs_scale = 0.0f;
    for (int ib = 0; ib < 16; ++ib) {
        const float scale = make_qx_quants(16, 32, x + 16 * ib, L + 16 * ib);
        scales[ib] = scale;
        const float abs_scale = fabsf(scale);
        if (abs_scale > max_abs_scale) { max_abs_scale = abs_scale; max_scale = scale; }
    }
    if (max_abs_scale < 1e-15f) {
        memset(y, 0, sizeof(*y));
        return;
    }
    const float iscale = -128.0f / max_scale;
    y->d = co_f32_to_fp16(1.0f / iscale);
    for (int ib = 0; ib < 16; ++ib) {
        const int v = nearest_int(iscale * scales[ib]);
        y->scales[ib] = (int8_t)(v < 127 ? v : 127);
    }
    for (int j = 0; j < 16; ++j) {
        const float d = co_fp16_to_f32(y->d) * (float)y->scales[j];
        if (d == 0.0f) continue;
        for (int ii = 0; ii < 16; ++ii) {
            int l = nearest_int(x[16 * j + ii] / d);
            l = l < -32 ? -32 : (l > 31 ? 31 : l);
            L[16 * j + ii] = (int8_t)(l + 32);
        }
    }
    uint8_t *ql = y->ql, *qh = y->qh;
    for (int j = 0; j < 256; j += 128) {
        for (int l = 0; l < 32; ++l) {
            const uint8_t q1 = (uint8_t)L[j + l] & 0xF, q2 = (uint8_t)L[j + l + 32] & 0xF;
            const uint8_t q3 = (uint8_t)L[j + l + 64] & 0xF, q4 = (uint8_t)L[j + l + 96] & 0xF;
            ql[l] = (uint8_t)(q1 | (q3 << 4));
            ql[l + 32] = (uint8_t)(q2 | (q4 << 4));
            qh[l] = (uint8_t)(((uint8_t)L[j + l] >> 4) | (((uint8_t)L[j + l + 32] >> 4) << 2) |
                              (((uint8_t)L[j + l + 64] >> 4) << 4) | (((uint8_t)L[j + l + 96] >> 4) << 6));
        }
        ql += 64;
        qh += 32;
    }
}

int co_quantize(int fmt, const float *x, int64_t rows, int64_t cols, void *out_blocks) {
    const int qk = co_block_elems(fmt);
    if (qk == 0 || rows < 0 || cols < 0 || cols % qk != 0) return -1;
    const int64_t nb = rows * cols / qk;
    switch (fmt) {
    case CO_Q8_0: return co_quantize_q8_0(x, rows, cols, out_blocks);
    case CO_Q4_0:
    case CO_Q4_0_GGML:
        for (int64_t b = 0; b < nb; ++b) quantize_block_q4_0(x + 32 * b, (co_block_q4_0 *)out_blocks + b, fmt == CO_Q4_0_GGML);
        return 0;
    case CO_Q4_K:
        for (int64_t b = 0; b < nb; ++b) quantize_block_q4_k(x + 256 * b, (co_block_q4_k *)out_blocks + b);
        return 0;
    case CO_Q6_K:
        for (int64_t b = 0; b < nb; ++b) quantize_block_q6_k(x + 256 * b, (co_block_q6_k *)out_blocks + b);
        return 0;
    default: return -1;
    }
}

/* ---- integer vec-dots against Q8_0 activation blocks ---- */

/* QGO:85-93 element order: even elements pair with low nibbles, odd with high. */
static float vec_dot_q4_0(const co_block_q4_0 *w, const co_block_q8_0 *x, int64_t nb) {
    float acc = 0.0f;
    for (int64_t b = 0; b < nb; ++b) {
        int32_t sumi = 0;
        for (int j = 0; j < 16; ++j) {
            sumi += ((int)(w[b].qs[j] & 0xF) - 8) * (int)x[b].qs[2 * j];
            sumi += ((int)(w[b].qs[j] >> 4) - 8) * (int)x[b].qs[2 * j + 1];
        }
        acc += (co_fp16_to_f32(w[b].d) * co_fp16_to_f32(x[b].d)) * (float)sumi;
    }
    return acc;
}

/* ggml order (QCU:2426-2433 pairs low nibbles with q8[0..15], high with q8[16..31]) */
static float vec_dot_q4_0_ggml(const co_block_q4_0 *w, const co_block_q8_0 *x, int64_t nb) {
    float acc = 0.0f;
    for (int64_t b = 0; b < nb; ++b) {
        int32_t sumi = 0;
        for (int j = 0; j < 16; ++j) {
            sumi += ((int)(w[b].qs[j] & 0xF) - 8) * (int)x[b].qs[j];
            sumi += ((int)(w[b].qs[j] >> 4) - 8) * (int)x[b].qs[j + 16];
        }
        acc += (co_fp16_to_f32(w[b].d) * co_fp16_to_f32(x[b].d)) * (float)sumi;
    }
    return acc;
}

/* QCU:2058-2073: d8_0 * d8_1 * sumi */
static float vec_dot_q8_0(const co_block_q8_0 *w, const co_block_q8_0 *x, int64_t nb) {
    float acc = 0.0f;
    for (int64_t b = 0; b < nb; ++b) {
        int32_t sumi = 0;
        for (int i = 0; i < 32; ++i) sumi += (int)w[b].qs[i] * (int)x[b].qs[i];
        acc += (co_fp16_to_f32(w[b].d) * co_fp16_to_f32(x[b].d)) * (float)sumi;
    }
    return acc;
}

/* QCU:2239-2263: sumf_d += d8*(dot1*sc); sumf_m += d8*(dot2*m); dm.x*sumf_d - dm.y*sumf_m,
 * taken over the eight 32-value sub-blocks of one super-block in ascending order. */
static float vec_dot_q4_k(const co_block_q4_k *w, const co_block_q8_0 *x, int64_t nsb) {
    float acc = 0.0f;
    for (int64_t s = 0; s < nsb; ++s) {
        float sumf_d = 0.0f, sumf_m = 0.0f;
        for (int t = 0; t < 8; ++t) {
            const co_block_q8_0 *xb = x + 8 * s + t;
            const uint8_t *q = w[s].qs + 32 * (t / 2);
            int32_t dot1 = 0, dot2 = 0;
            for (int l = 0; l < 32; ++l) {
                int q4 = (t & 1) ? (q[l] >> 4) : (q[l] & 0xF);
                dot1 += q4 * (int)xb->qs[l];
                dot2 += (int)xb->qs[l];
            }
            uint8_t sc, m;
            co_get_scale_min_k4(t, w[s].scales, &sc, &m);
            float d8 = co_fp16_to_f32(xb->d);
            sumf_d += d8 * (float)(dot1 * (int)sc);
            sumf_m += d8 * (float)(dot2 * (int)m);
        }
        acc += co_fp16_to_f32(w[s].dm[0]) * sumf_d - co_fp16_to_f32(w[s].dm[1]) * sumf_m;
    }
    return acc;
}

/* QCU:2367-2389: sumf += d8 * (dot * sc) per 16-value group; d * sumf per super-block. */
static float vec_dot_q6_k(const co_block_q6_k *w, const co_block_q8_0 *x, int64_t nsb) {
    float acc = 0.0f;
    for (int64_t s = 0; s < nsb; ++s) {
        float sumf = 0.0f;
        for (int g = 0; g < 16; ++g) {
            const co_block_q8_0 *xb = x + 8 * s + g / 2;
            int32_t dot = 0;
            for (int l = 0; l < 16; ++l) {
                int e = 16 * g + l;
                int ip = e / 128, quarter = (e % 128) / 32, il = e % 32;
                uint8_t qlb = w[s].ql[64 * ip + il + 32 * (quarter & 1)];
                int lo4 = (quarter < 2) ? (qlb & 0xF) : (qlb >> 4);
                int hi2 = (w[s].qh[32 * ip + il] >> (2 * quarter)) & 3;
                int q6 = (lo4 | (hi2 << 4)) - 32;
                dot += q6 * (int)xb->qs[(e % 32)];
            }
            sumf += co_fp16_to_f32(xb->d) * (float)(dot * (int)w[s].scales[g]);
        }
        acc += co_fp16_to_f32(w[s].d) * sumf;
    }
    return acc;
}

static int32_t q8_block_sum(const co_block_q8_0 *x) {
    int32_t s = 0;
    for (int i = 0; i < 32; ++i) s += (int)x->qs[i];
    return s;
}

/* QCU:1947-1975: sumi * (d4*d8) + m4 * s8, s8 = d8 * (sum of the block's quants), here with the exact integer sum.
 * elem(j, hi) says which activation the low / high nibble of byte j pairs with (the two element orders). */
static float vec_dot_q4_1(const co_block_q4_1 *w, const co_block_q8_0 *x, int64_t nb, int ggml_order) {
    float acc = 0.0f;
    for (int64_t b = 0; b < nb; ++b) {
        int32_t sumi = 0;
        for (int j = 0; j < 16; ++j) {
            sumi += (int)(w[b].qs[j] & 0xF) * (int)x[b].qs[ggml_order ? j : 2 * j];
            sumi += (int)(w[b].qs[j] >> 4) * (int)x[b].qs[ggml_order ? j + 16 : 2 * j + 1];
        }
        const float d8 = co_fp16_to_f32(x[b].d);
        acc += (co_fp16_to_f32(w[b].dm[0]) * d8) * (float)sumi + (co_fp16_to_f32(w[b].dm[1]) * d8) * (float)q8_block_sum(x + b);
    }
    return acc;
}

/* QCU:1982-2009: d5 * (sumi*d8 - 16*s8) = (d5*d8) * (sumi - 16*sum) with the exact integer sum */
static float vec_dot_q5_0(const co_block_q5_0 *w, const co_block_q8_0 *x, int64_t nb) {
    float acc = 0.0f;
    for (int64_t b = 0; b < nb; ++b) {
        int32_t sumi = 0;
        for (int e = 0; e < 32; ++e) sumi += q5_level(w[b].qs, w[b].qh, e) * (int)x[b].qs[e];
        sumi -= 16 * q8_block_sum(x + b);
        acc += (co_fp16_to_f32(w[b].d) * co_fp16_to_f32(x[b].d)) * (float)sumi;
    }
    return acc;
}

/* QCU:2016-2053: sumi * (d5*d8) + m5 * s8 */
static float vec_dot_q5_1(const co_block_q5_1 *w, const co_block_q8_0 *x, int64_t nb) {
    float acc = 0.0f;
    for (int64_t b = 0; b < nb; ++b) {
        int32_t sumi = 0;
        for (int e = 0; e < 32; ++e) sumi += q5_level(w[b].qs, w[b].qh, e) * (int)x[b].qs[e];
        const float d8 = co_fp16_to_f32(x[b].d);
        acc += (co_fp16_to_f32(w[b].dm[0]) * d8) * (float)sumi + (co_fp16_to_f32(w[b].dm[1]) * d8) * (float)q8_block_sum(x + b);
    }
    return acc;
}

/* QCU:2108-2135: per 16-value group sumf_d += d8*(dot*scale), sumf_m += d8*(sum*min); dall*sumf_d - dmin*sumf_m
 * per super-block, groups in ascending order. */
static float vec_dot_q2_k(const co_block_q2_k *w, const co_block_q8_0 *x, int64_t nsb) {
    float acc = 0.0f;
    for (int64_t s = 0; s < nsb; ++s) {
        float sumf_d = 0.0f, sumf_m = 0.0f;
        for (int g = 0; g < 16; ++g) {
            const co_block_q8_0 *xb = x + 8 * s + g / 2;
            int32_t dot = 0, sum = 0;
            for (int i = 0; i < 16; ++i) {
                const int e = 16 * g + i, n = e / 128, k = (e % 128) / 32, l = e % 32;
                const int q = (w[s].qs[32 * n + l] >> (2 * k)) & 3;
                dot += q * (int)xb->qs[e % 32];
                sum += (int)xb->qs[e % 32];
            }
            const float d8 = co_fp16_to_f32(xb->d);
            sumf_d += d8 * (float)(dot * (int)(w[s].scales[g] & 0xF));
            sumf_m += d8 * (float)(sum * (int)(w[s].scales[g] >> 4));
        }
        acc += co_fp16_to_f32(w[s].dm[0]) * sumf_d - co_fp16_to_f32(w[s].dm[1]) * sumf_m;
    }
    return acc;
}

/* QCU:2177-2209: sumf += d8 * (dot * (scale - 32)) per 16-value group; d * sumf per super-block */
static float vec_dot_q3_k(const co_block_q3_k *w, const co_block_q8_0 *x, int64_t nsb) {
    float acc = 0.0f;
    for (int64_t s = 0; s < nsb; ++s) {
        float sumf = 0.0f;
        for (int g = 0; g < 16; ++g) {
            const co_block_q8_0 *xb = x + 8 * s + g / 2;
            int32_t dot = 0;
            for (int i = 0; i < 16; ++i) dot += q3k_level(w + s, 16 * g + i) * (int)xb->qs[(16 * g + i) % 32];
            sumf += co_fp16_to_f32(xb->d) * (float)(dot * (q3k_scale(w[s].scales, g) - 32));
        }
        acc += co_fp16_to_f32(w[s].d) * sumf;
    }
    return acc;
}

/* QCU:2300-2331: as Q4_K with 5-bit levels */
static float vec_dot_q5_k(const co_block_q5_k *w, const co_block_q8_0 *x, int64_t nsb) {
    float acc = 0.0f;
    for (int64_t s = 0; s < nsb; ++s) {
        float sumf_d = 0.0f, sumf_m = 0.0f;
        for (int t = 0; t < 8; ++t) {
            const co_block_q8_0 *xb = x + 8 * s + t;
            int32_t dot1 = 0;
            for (int l = 0; l < 32; ++l) dot1 += q5k_level(w + s, 32 * t + l) * (int)xb->qs[l];
            uint8_t sc, m;
            co_get_scale_min_k4(t, w[s].scales, &sc, &m);
            const float d8 = co_fp16_to_f32(xb->d);
            sumf_d += d8 * (float)(dot1 * (int)sc);
            sumf_m += d8 * (float)(q8_block_sum(xb) * (int)m);
        }
        acc += co_fp16_to_f32(w[s].dm[0]) * sumf_d - co_fp16_to_f32(w[s].dm[1]) * sumf_m;
    }
    return acc;
}

/* Other, equally valid orders of the same f32 additions: 0 the blocks (super-blocks) of a row ascending, as
 * everywhere else in this file; 1 descending; 2 the even-numbered blocks ascending, then the odd-numbered ones;
 * 3 the second half of the row, then the first.  Nothing in the reference prescribes the order (QCU:2787-2871
 * spreads the blocks of a row over the lanes of a warp and adds the lanes' partial sums in a tree); the others
 * exist so that tests can measure, on the CPU alone, how far correct evaluations of one model drift apart. */
static int g_block_order = 0;
void co_set_block_order(int order) { g_block_order = (order >= 0 && order <= 3) ? order : 0; }

static float vec_dot_ascending(int fmt, const void *w_row, const void *x_q8_0, int64_t k);

float co_vec_dot_q8_0(int fmt, const void *w_row, const void *x_q8_0, int64_t k) {
    if (g_block_order == 0) return vec_dot_ascending(fmt, w_row, x_q8_0, k);
    const int qk = co_block_elems(fmt), bs = co_block_bytes(fmt);
    if (qk == 0 || k % qk != 0) return NAN;
    const int64_t nu = k / qk;
    float acc = 0.0f;
    for (int64_t i = 0; i < nu; ++i) {
        int64_t u = i;
        if (g_block_order == 1) u = nu - 1 - i;
        else if (g_block_order == 2) u = i < (nu + 1) / 2 ? 2 * i : 2 * (i - (nu + 1) / 2) + 1;
        else if (g_block_order == 3) u = (i + nu / 2) % nu;
        /* one block at a time: 0.0f + its term is the term itself */
        acc += vec_dot_ascending(fmt, (const uint8_t *)w_row + (size_t)u * (size_t)bs,
                                 (const uint8_t *)x_q8_0 + (size_t)u * (size_t)(qk / 32) * 34, qk);
    }
    return acc;
}

static float vec_dot_ascending(int fmt, const void *w_row, const void *x_q8_0, int64_t k) {
    const co_block_q8_0 *x = (const co_block_q8_0 *)x_q8_0;
    switch (fmt) {
    case CO_Q4_1: return vec_dot_q4_1((const co_block_q4_1 *)w_row, x, k / 32, 0);
    case CO_Q4_1_GGML: return vec_dot_q4_1((const co_block_q4_1 *)w_row, x, k / 32, 1);
    case CO_Q5_0: return vec_dot_q5_0((const co_block_q5_0 *)w_row, x, k / 32);
    case CO_Q5_1: return vec_dot_q5_1((const co_block_q5_1 *)w_row, x, k / 32);
    case CO_Q2_K: return vec_dot_q2_k((const co_block_q2_k *)w_row, x, k / 256);
    case CO_Q3_K: return vec_dot_q3_k((const co_block_q3_k *)w_row, x, k / 256);
    case CO_Q5_K: return vec_dot_q5_k((const co_block_q5_k *)w_row, x, k / 256);
    case CO_Q4_0: return vec_dot_q4_0((const co_block_q4_0 *)w_row, x, k / 32);
    case CO_Q4_0_GGML: return vec_dot_q4_0_ggml((const co_block_q4_0 *)w_row, x, k / 32);
    case CO_Q8_0: return vec_dot_q8_0((const co_block_q8_0 *)w_row, x, k / 32);
    case CO_Q4_K: return vec_dot_q4_k((const co_block_q4_k *)w_row, x, k / 256);
    case CO_Q6_K: return vec_dot_q6_k((const co_block_q6_k *)w_row, x, k / 256);
    default: return NAN;
    }
}

int co_qmatmul(int fmt, const void *w_blocks, int64_t rows, int64_t cols,
               const float *x, int64_t m, float *y) {
    int qk = co_block_elems(fmt), bs = co_block_bytes(fmt);
    if (qk == 0 || cols % qk != 0 || rows < 0 || m < 0) return -1;
    size_t xq_bytes = (size_t)(m * cols / 32) * 34;
    void *xq = malloc(xq_bytes ? xq_bytes : 1);
    if (!xq) return -2;
    co_quantize_q8_0(x, m, cols, xq);
    size_t row_bytes = (size_t)(cols / qk) * (size_t)bs;
    size_t xrow_bytes = (size_t)(cols / 32) * 34;
    /* every output is its own chain of operations: spreading the outputs over threads changes no bit
     * (the candy CPU path itself is single-threaded; the timed baseline, co_matmul_dequant_f32, stays so) */
    #pragma omp parallel for collapse(2) schedule(static)
    for (int64_t i = 0; i < m; ++i)
        for (int64_t n = 0; n < rows; ++n)
            y[i * rows + n] = co_vec_dot_q8_0(fmt, (const uint8_t *)w_blocks + (size_t)n * row_bytes,
                                              (const uint8_t *)xq + (size_t)i * xrow_bytes, cols);
    free(xq);
    return 0;
}

/* CONV:251-267 */
void co_naive_batched_matmul_f32(int64_t bsz, int64_t m, int64_t n, int64_t k,
                                 const float *a, const float *b, float *c) {
    for (int64_t bb = 0; bb < bsz; ++bb) {
        int64_t a_base = bb * m * k, b_base = bb * k * n, c_base = bb * m * n;
        for (int64_t i = 0; i < m; ++i)
            for (int64_t j = 0; j < n; ++j) {
                float sum = 0.0f;
                for (int64_t l = 0; l < k; ++l) sum += a[a_base + i * k + l] * b[b_base + l * n + j];
                c[c_base + i * n + j] = sum;
            }
    }
}

/* CONV:373-389 */
void co_naive_batched_matmul_strided_f32(int64_t bsz, int64_t m, int64_t n, int64_t k,
                                         const float *a, const float *b, float *c,
                                         const int64_t as[3], const int64_t bs[3], const int64_t cs[3]) {
    for (int64_t bb = 0; bb < bsz; ++bb)
        for (int64_t i = 0; i < m; ++i)
            for (int64_t j = 0; j < n; ++j) {
                float sum = 0.0f;
                for (int64_t l = 0; l < k; ++l)
                    sum += a[bb * as[0] + i * as[1] + l * as[2]] * b[bb * bs[0] + l * bs[1] + j * bs[2]];
                c[bb * cs[0] + i * cs[1] + j * cs[2]] = sum;
            }
}

/* What nn.Linear does on candy's CPU backend (nn/linear.go:58-112 -> cpu/storage.go:889-909):
 * the weight is a [rows, cols] tensor viewed transposed with strides {1, cols}. */
int co_matmul_dequant_f32(int fmt, const void *w_blocks, int64_t rows, int64_t cols,
                          const float *x, int64_t m, float *y) {
    int qk = co_block_elems(fmt);
    if (qk == 0 || cols % qk != 0) return -1;
    int64_t nel = rows * cols;
    float *wf = (float *)malloc((size_t)(nel > 0 ? nel : 1) * sizeof(float));
    if (!wf) return -2;
    co_dequantize(fmt, w_blocks, rows * cols / qk, wf);
    const int64_t as[3] = {0, cols, 1}, bs[3] = {0, 1, cols}, cs[3] = {0, rows, 1};
    co_naive_batched_matmul_strided_f32(1, m, rows, cols, x, wf, y, as, bs, cs);
    free(wf);
    return 0;
}

/* RED:3071-3092 */
void co_fast_rms_norm_f32(int64_t numel, int64_t ncols, float eps, const float *alpha,
                          const float *x, float *dst) {
    if (ncols <= 0) return;
    int64_t rows = numel / ncols;
    for (int64_t r = 0; r < rows; ++r) {
        float sum = 0.0f;
        for (int64_t c = 0; c < ncols; ++c) { float xi = x[r * ncols + c]; sum += xi * xi; }
        float mean = sum / (float)ncols;
        float scale = 1.0f / (float)sqrt((double)(mean + eps));
        for (int64_t c = 0; c < ncols; ++c) {
            int64_t i = r * ncols + c;
            dst[i] = alpha ? scale * x[i] * alpha[c] : scale * x[i];
        }
    }
}

/* RED:3987-4006 */
void co_rope_f32(int64_t bh, int64_t td, int64_t d, int64_t stride_b, const float *src,
                 const float *cos_t, const float *sin_t, float *dst) {
    int64_t num_pairs = bh * td / 2;
    for (int64_t idx = 0; idx < num_pairs; ++idx) {
        int64_t i_bh = idx / (td / 2);
        int64_t i_td = idx - (td / 2) * i_bh;
        int64_t i_t = i_td / (d / 2);
        int64_t i_d = i_td - (d / 2) * i_t;
        int64_t i1 = i_bh * td + i_t * d + i_d;
        int64_t i2 = i1 + d / 2;
        int64_t i_cs = i_t * (d / 2) + i_d;
        if (stride_b > 0) i_cs += ((2 * idx) / stride_b) * (td / 2);
        float c = cos_t[i_cs], s = sin_t[i_cs];
        float a = src[i1], b = src[i2];
        dst[i1] = a * c - b * s;
        dst[i2] = a * s + b * c;
    }
}

/* RED:3825-3838: adjacent pairs (2i, 2i + 1), cos / sin indexed by the pair within the row of td values */
void co_rope_i_f32(int64_t bh, int64_t td, int64_t stride_b, const float *src, const float *cos_t,
                   const float *sin_t, float *dst) {
    int64_t num_pairs = bh * td / 2;
    for (int64_t idx = 0; idx < num_pairs; ++idx) {
        int64_t rope_idx = idx % (td / 2);
        if (stride_b > 0) rope_idx += ((2 * idx) / stride_b) * (td / 2);
        float c = cos_t[rope_idx], s = sin_t[rope_idx];
        float a = src[2 * idx], b = src[2 * idx + 1];
        dst[2 * idx] = a * c - b * s;
        dst[2 * idx + 1] = a * s + b * c;
    }
}

/* RED:4178-4196: [b, t, h, d] layout, pairs (i, i + d/2), cos / sin rows picked by the token index t */
void co_rope_thd_f32(int64_t b, int64_t t, int64_t h, int64_t d, int64_t stride_b, const float *src,
                     const float *cos_t, const float *sin_t, float *dst) {
    int64_t num_pairs = b * t * h * d / 2;
    for (int64_t idx = 0; idx < num_pairs; ++idx) {
        int64_t i_bth = idx / (d / 2);
        int64_t i_d = idx - (d / 2) * i_bth;
        int64_t i_t = (i_bth / h) % t;
        int64_t i1 = i_bth * d + i_d;
        int64_t i2 = i1 + d / 2;
        int64_t i_cs = i_t * (d / 2) + i_d;
        if (stride_b > 0) i_cs += ((2 * idx) / stride_b) * ((t * d) / 2);
        float c = cos_t[i_cs], s = sin_t[i_cs];
        float a = src[i1], bb = src[i2];
        dst[i1] = a * c - bb * s;
        dst[i2] = a * s + bb * c;
    }
}

/* RED:2855-2879 */
void co_fast_softmax_f32(int64_t numel, int64_t ncols, const float *src, float *dst) {
    if (ncols <= 0) return;
    int64_t rows = numel / ncols;
    for (int64_t r = 0; r < rows; ++r) {
        float max_val = -3.40282346638528859811704183484516925440e+38f;
        for (int64_t c = 0; c < ncols; ++c) if (src[r * ncols + c] > max_val) max_val = src[r * ncols + c];
        float sum = 0.0f;
        for (int64_t c = 0; c < ncols; ++c) {
            float v = (float)exp((double)(src[r * ncols + c] - max_val));
            dst[r * ncols + c] = v;
            sum += v;
        }
        float inv = 1.0f / sum;
        for (int64_t c = 0; c < ncols; ++c) dst[r * ncols + c] *= inv;
    }
}

/* UNA:3353-3366 */
void co_silu_f32(int64_t numel, const float *inp, float *out) {
    const float *s = inp ? inp : out;
    for (int64_t i = 0; i < numel; ++i) { double x = (double)s[i]; out[i] = (float)(x / (1.0 + exp(-x))); }
}

/* RED:846-862 */
void co_fast_argmax_f32(int64_t numel, int64_t ncols, const float *src, uint32_t *dst) {
    if (ncols <= 0) return;
    int64_t n = numel / ncols;
    for (int64_t i = 0; i < n; ++i) {
        float max_val = -3.40282346638528859811704183484516925440e+38f;
        uint32_t max_idx = 0;
        for (int64_t j = 0; j < ncols; ++j)
            if (src[i * ncols + j] > max_val) { max_val = src[i * ncols + j]; max_idx = (uint32_t)j; }
        dst[i] = max_idx;
    }
}

/* IDX:8-26 (ids equal to MaxInt64 select zero) */
void co_index_select_f32(int64_t numel, const int64_t *ids, const float *inp, float *out,
                         int64_t left, int64_t src_dim, int64_t ids_dim, int64_t right) {
    (void)left;
    for (int64_t i = 0; i < numel; ++i) {
        int64_t left_i = i / (ids_dim * right);
        int64_t id_i = (i / right) % ids_dim;
        int64_t right_i = i % right;
        int64_t idx = ids[id_i];
        if (idx == INT64_MAX) { out[i] = 0.0f; continue; }
        out[i] = inp[left_i * src_dim * right + idx * right + right_i];
    }
}

/* binary.go BAddF32 / BMulF32: plain elementwise loops */
void co_add_f32(int64_t n, const float *a, const float *b, float *out) { for (int64_t i = 0; i < n; ++i) out[i] = a[i] + b[i]; }
void co_mul_f32(int64_t n, const float *a, const float *b, float *out) { for (int64_t i = 0; i < n; ++i) out[i] = a[i] * b[i]; }

void co_attention_decode_f32(const float *q, const float *k_cache, const float *v_cache,
                             int64_t n_heads, int64_t n_kv_heads, int64_t head_dim,
                             int64_t n_pos, int64_t cache_stride, float scale, float *out) {
    float *s = (float *)malloc((size_t)(n_pos ? n_pos : 1) * sizeof(float));
    int64_t group = n_heads / n_kv_heads;
    for (int64_t h = 0; h < n_heads; ++h) {
        const float *kh = k_cache + (h / group) * cache_stride;
        const float *vh = v_cache + (h / group) * cache_stride;
        const float *qh = q + h * head_dim;
        for (int64_t p = 0; p < n_pos; ++p) { /* q . K^T: CONV:251-267 with m=1 */
            float sum = 0.0f;
            for (int64_t d = 0; d < head_dim; ++d) sum += qh[d] * kh[p * head_dim + d];
            s[p] = sum * scale;
        }
        co_fast_softmax_f32(n_pos, n_pos, s, s);
        for (int64_t d = 0; d < head_dim; ++d) { /* p . V */
            float sum = 0.0f;
            for (int64_t p = 0; p < n_pos; ++p) sum += s[p] * vh[p * head_dim + d];
            out[h * head_dim + d] = sum;
        }
    }
    free(s);
}
