// Llama-style batch-1 decoder assembled from the library's ops.  candy has no model code; the
// block is the standard one (RMSNorm, q/k/v, RoPE, attention over the f32 KV cache, o, residual,
// RMSNorm, SwiGLU, residual; final RMSNorm, head, argmax) written as the sequence of
// BackendStorage calls (backend.go) a candy model would issue, with the quantized Linear in
// place of MatMul.
#include <cmath>
#include <vector>

#include "blocks.h"
#include "internal.h"

struct candy_hip_llama {
    candy_hip_device *dev = nullptr;
    candy_hip_llama_config cfg{};
    struct Layer {
        const float *attn_norm = nullptr, *ffn_norm = nullptr;
        const candy_hip_qtensor *wq = nullptr, *wk = nullptr, *wv = nullptr, *wo = nullptr;
        const candy_hip_qtensor *gate = nullptr, *up = nullptr, *down = nullptr;
    };
    std::vector<Layer> layers;
    const float *out_norm = nullptr;
    const candy_hip_qtensor *head = nullptr, *embed = nullptr;
    // device buffers
    float *k_cache = nullptr, *v_cache = nullptr;  // [n_layers][n_kv_heads][max_pos][head_dim]
    float *cos_t = nullptr, *sin_t = nullptr;      // [max_pos][head_dim/2]
    float *h = nullptr, *xn = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *att = nullptr;
    float *gate_o = nullptr, *up_o = nullptr, *act = nullptr, *tmp = nullptr, *logits = nullptr;
    int8_t *xq = nullptr;           // planar Q8_0 quants of the current activation
    candy::Q8Scale *xs = nullptr;
    uint32_t *next_tok = nullptr;
    int64_t *tok_id = nullptr;
    std::vector<void *> owned;
};

namespace candy {

// RoPE on the new q and k rows (reduce.go:3987-4006 with t = 1: pairs (i, i + d/2), cos/sin row
// of this position), then k and v go to row `pos` of their kv head's cache.
__global__ __launch_bounds__(256) void k_rope_store(float *__restrict__ q, const float *__restrict__ k,
                                                    const float *__restrict__ v, const float *__restrict__ cos_row,
                                                    const float *__restrict__ sin_row, int n_heads, int n_kv_heads,
                                                    int head_dim, int pos, int max_pos, float *__restrict__ k_cache,
                                                    float *__restrict__ v_cache) {
    const int half = head_dim >> 1;
    const int idx = blockIdx.x * 256 + threadIdx.x;
    const int nq = n_heads * half, nk = n_kv_heads * half;
    if (idx < nq) {
        const int hh = idx / half, i = idx - hh * half;
        float *p = q + hh * head_dim;
        const float a = p[i], b = p[i + half], c = cos_row[i], s = sin_row[i];
        p[i] = a * c - b * s;
        p[i + half] = a * s + b * c;
    } else if (idx < nq + nk) {
        const int j = idx - nq;
        const int hh = j / half, i = j - hh * half;
        const float *p = k + hh * head_dim;
        const float a = p[i], b = p[i + half], c = cos_row[i], s = sin_row[i];
        float *kd = k_cache + ((size_t)hh * max_pos + pos) * head_dim;
        kd[i] = a * c - b * s;
        kd[i + half] = a * s + b * c;
        const float *pv = v + hh * head_dim;
        float *vd = v_cache + ((size_t)hh * max_pos + pos) * head_dim;
        vd[i] = pv[i];
        vd[i + half] = pv[i + half];
    }
}

}  // namespace candy

using namespace candy;

template <class T>
static int dev_alloc(candy_hip_llama *m, T **p, size_t count) {
    void *d = nullptr;
    if (int rc = candy_hip_alloc(m->dev, count * sizeof(T), &d)) return rc;
    m->owned.push_back(d);
    *p = (T *)d;
    return CANDY_HIP_OK;
}

static int linear(candy_hip_llama *m, const candy_hip_qtensor *w, float *y) {
    return launch_matvec(m->dev, w, m->xq, m->xs, 1, y);
}

static int quantize(candy_hip_llama *m, const float *x, int64_t n) {
    return launch_quantize_q8(m->dev, x, 1, n, m->xq, m->xs, nullptr);
}

extern "C" {

int candy_hip_qindex_select(candy_hip_device *dev, const candy_hip_qtensor *q, const int64_t *dev_ids, int64_t n_ids,
                            float *out);

int candy_hip_llama_create(candy_hip_device *dev, const candy_hip_llama_config *cfg, candy_hip_llama **out) {
    CANDY_REQUIRE(out, "out is nil");
    *out = nullptr;
    CANDY_REQUIRE(dev && cfg, "nil argument");
    CANDY_REQUIRE(cfg->n_layers > 0 && cfg->d_model > 0 && cfg->n_heads > 0 && cfg->n_kv_heads > 0 &&
                      cfg->head_dim > 0 && cfg->d_ffn > 0 && cfg->vocab > 0 && cfg->max_pos > 0,
                  "every size in the config must be positive");
    CANDY_REQUIRE(cfg->n_heads % cfg->n_kv_heads == 0, "n_heads must be a multiple of n_kv_heads");
    CANDY_REQUIRE(cfg->head_dim % 2 == 0 && cfg->head_dim <= 256, "head_dim must be even and <= 256");
    CANDY_REQUIRE(cfg->d_model % 256 == 0 && cfg->d_ffn % 256 == 0 && (cfg->n_heads * cfg->head_dim) % 256 == 0,
                  "d_model, d_ffn and n_heads*head_dim must be multiples of 256");
    if (int rc = use_device(dev)) return rc;
    candy_hip_llama *m = new candy_hip_llama();
    m->dev = dev;
    m->cfg = *cfg;
    m->layers.resize(cfg->n_layers);
    const size_t kv = (size_t)cfg->n_layers * cfg->n_kv_heads * cfg->max_pos * cfg->head_dim;
    const int half = cfg->head_dim / 2;
    const size_t widest = (size_t)std::max(std::max(cfg->d_model, cfg->d_ffn), cfg->n_heads * cfg->head_dim);
    int rc = CANDY_HIP_OK;
    if (!rc) rc = dev_alloc(m, &m->k_cache, kv);
    if (!rc) rc = dev_alloc(m, &m->v_cache, kv);
    if (!rc) rc = dev_alloc(m, &m->cos_t, (size_t)cfg->max_pos * half);
    if (!rc) rc = dev_alloc(m, &m->sin_t, (size_t)cfg->max_pos * half);
    if (!rc) rc = dev_alloc(m, &m->h, (size_t)cfg->d_model);
    if (!rc) rc = dev_alloc(m, &m->xn, widest);
    if (!rc) rc = dev_alloc(m, &m->q, (size_t)cfg->n_heads * cfg->head_dim);
    if (!rc) rc = dev_alloc(m, &m->k, (size_t)cfg->n_kv_heads * cfg->head_dim);
    if (!rc) rc = dev_alloc(m, &m->v, (size_t)cfg->n_kv_heads * cfg->head_dim);
    if (!rc) rc = dev_alloc(m, &m->att, (size_t)cfg->n_heads * cfg->head_dim);
    if (!rc) rc = dev_alloc(m, &m->gate_o, (size_t)cfg->d_ffn);
    if (!rc) rc = dev_alloc(m, &m->up_o, (size_t)cfg->d_ffn);
    if (!rc) rc = dev_alloc(m, &m->act, (size_t)cfg->d_ffn);
    if (!rc) rc = dev_alloc(m, &m->tmp, (size_t)cfg->d_model);
    if (!rc) rc = dev_alloc(m, &m->logits, (size_t)cfg->vocab);
    if (!rc) rc = dev_alloc(m, &m->xq, widest);
    if (!rc) rc = dev_alloc(m, &m->xs, widest / 32);
    if (!rc) rc = dev_alloc(m, &m->next_tok, 1);
    if (!rc) rc = dev_alloc(m, &m->tok_id, 1);
    if (!rc) rc = candy_hip_zero(dev, m->k_cache, kv * sizeof(float));
    if (!rc) rc = candy_hip_zero(dev, m->v_cache, kv * sizeof(float));
    if (!rc) {
        // angle(p, i) = p * base^(-2i/d), evaluated in double, stored as f32
        std::vector<float> c((size_t)cfg->max_pos * half), s((size_t)cfg->max_pos * half);
        for (int p = 0; p < cfg->max_pos; ++p)
            for (int i = 0; i < half; ++i) {
                const double ang = (double)p * std::pow((double)cfg->rope_base, -2.0 * i / (double)cfg->head_dim);
                c[(size_t)p * half + i] = (float)std::cos(ang);
                s[(size_t)p * half + i] = (float)std::sin(ang);
            }
        rc = candy_hip_h2d(dev, m->cos_t, c.data(), c.size() * sizeof(float));
        if (!rc) rc = candy_hip_h2d(dev, m->sin_t, s.data(), s.size() * sizeof(float));
    }
    if (rc) {
        candy_hip_llama_free(m);
        return rc;
    }
    *out = m;
    return CANDY_HIP_OK;
}

int candy_hip_llama_free(candy_hip_llama *m) {
    if (!m) return CANDY_HIP_OK;
    for (void *p : m->owned) (void)candy_hip_free(m->dev, p);
    delete m;
    return CANDY_HIP_OK;
}

int candy_hip_llama_set_qweight(candy_hip_llama *m, int which, int layer, const candy_hip_qtensor *w) {
    CANDY_REQUIRE(m && w, "nil argument");
    CANDY_REQUIRE(w->dev == m->dev, "weight lives on another device");
    const candy_hip_llama_config &c = m->cfg;
    const int64_t qd = (int64_t)c.n_heads * c.head_dim, kvd = (int64_t)c.n_kv_heads * c.head_dim;
    int64_t rows = 0, cols = 0;
    switch (which) {
    case CANDY_HIP_W_Q: rows = qd; cols = c.d_model; break;
    case CANDY_HIP_W_K:
    case CANDY_HIP_W_V: rows = kvd; cols = c.d_model; break;
    case CANDY_HIP_W_O: rows = c.d_model; cols = qd; break;
    case CANDY_HIP_W_GATE:
    case CANDY_HIP_W_UP: rows = c.d_ffn; cols = c.d_model; break;
    case CANDY_HIP_W_DOWN: rows = c.d_model; cols = c.d_ffn; break;
    case CANDY_HIP_W_HEAD:
    case CANDY_HIP_W_EMBED: rows = c.vocab; cols = c.d_model; break;
    default: return fail(CANDY_HIP_ERR_INVALID, "weight kind %d is not a quantized matrix", which);
    }
    CANDY_REQUIRE(w->rows == rows && w->cols == cols, "weight kind %d must be %lld x %lld, got %lld x %lld", which,
                  (long long)rows, (long long)cols, (long long)w->rows, (long long)w->cols);
    if (which == CANDY_HIP_W_HEAD) { m->head = w; return CANDY_HIP_OK; }
    if (which == CANDY_HIP_W_EMBED) { m->embed = w; return CANDY_HIP_OK; }
    CANDY_REQUIRE(layer >= 0 && layer < c.n_layers, "layer %d out of range", layer);
    candy_hip_llama::Layer &L = m->layers[layer];
    switch (which) {
    case CANDY_HIP_W_Q: L.wq = w; break;
    case CANDY_HIP_W_K: L.wk = w; break;
    case CANDY_HIP_W_V: L.wv = w; break;
    case CANDY_HIP_W_O: L.wo = w; break;
    case CANDY_HIP_W_GATE: L.gate = w; break;
    case CANDY_HIP_W_UP: L.up = w; break;
    default: L.down = w; break;
    }
    return CANDY_HIP_OK;
}

int candy_hip_llama_set_norm(candy_hip_llama *m, int which, int layer, const float *dev_alpha) {
    CANDY_REQUIRE(m && dev_alpha, "nil argument");
    if (which == CANDY_HIP_W_OUT_NORM) { m->out_norm = dev_alpha; return CANDY_HIP_OK; }
    CANDY_REQUIRE(which == CANDY_HIP_W_ATTN_NORM || which == CANDY_HIP_W_FFN_NORM, "weight kind %d is not a norm", which);
    CANDY_REQUIRE(layer >= 0 && layer < m->cfg.n_layers, "layer %d out of range", layer);
    if (which == CANDY_HIP_W_ATTN_NORM) m->layers[layer].attn_norm = dev_alpha;
    else m->layers[layer].ffn_norm = dev_alpha;
    return CANDY_HIP_OK;
}

int candy_hip_llama_kv_cache(candy_hip_llama *m, float **dev_k, float **dev_v, size_t *bytes_each) {
    CANDY_REQUIRE(m, "model is nil");
    if (dev_k) *dev_k = m->k_cache;
    if (dev_v) *dev_v = m->v_cache;
    if (bytes_each)
        *bytes_each = (size_t)m->cfg.n_layers * m->cfg.n_kv_heads * m->cfg.max_pos * m->cfg.head_dim * sizeof(float);
    return CANDY_HIP_OK;
}

static int llama_check_complete(const candy_hip_llama *m) {
    CANDY_REQUIRE(m->out_norm && m->head, "final norm / head not set");
    for (size_t l = 0; l < m->layers.size(); ++l) {
        const candy_hip_llama::Layer &L = m->layers[l];
        CANDY_REQUIRE(L.attn_norm && L.ffn_norm && L.wq && L.wk && L.wv && L.wo && L.gate && L.up && L.down,
                      "layer %zu is missing weights", l);
    }
    return CANDY_HIP_OK;
}

static int llama_step(candy_hip_llama *m, int32_t pos, const float **dev_logits, int32_t *next_token) {
    const candy_hip_llama_config &c = m->cfg;
    candy_hip_device *dev = m->dev;
    const int64_t qd = (int64_t)c.n_heads * c.head_dim;
    const size_t layer_kv = (size_t)c.n_kv_heads * c.max_pos * c.head_dim;
    const int half = c.head_dim / 2;
    const float scale = 1.0f / std::sqrt((float)c.head_dim);
    int rc;
    for (int l = 0; l < c.n_layers; ++l) {
        const candy_hip_llama::Layer &L = m->layers[l];
        float *kc = m->k_cache + (size_t)l * layer_kv, *vc = m->v_cache + (size_t)l * layer_kv;
        if ((rc = candy_hip_rms_norm(dev, m->h, L.attn_norm, c.rms_eps, 1, c.d_model, m->xn))) return rc;
        if ((rc = quantize(m, m->xn, c.d_model))) return rc;
        if ((rc = linear(m, L.wq, m->q))) return rc;
        if ((rc = linear(m, L.wk, m->k))) return rc;
        if ((rc = linear(m, L.wv, m->v))) return rc;
        const int threads = (c.n_heads + c.n_kv_heads) * half;
        hipLaunchKernelGGL(k_rope_store, dim3((threads + 255) / 256), dim3(256), 0, dev->stream, m->q, m->k, m->v,
                           m->cos_t + (size_t)pos * half, m->sin_t + (size_t)pos * half, c.n_heads, c.n_kv_heads,
                           c.head_dim, pos, c.max_pos, kc, vc);
        CANDY_LAUNCH_CHECK();
        if ((rc = candy_hip_attention_decode(dev, m->q, kc, vc, c.n_heads, c.n_kv_heads, c.head_dim, pos + 1,
                                             (int64_t)c.max_pos * c.head_dim, scale, m->att)))
            return rc;
        if ((rc = quantize(m, m->att, qd))) return rc;
        if ((rc = linear(m, L.wo, m->tmp))) return rc;
        if ((rc = candy_hip_add(dev, m->h, m->tmp, c.d_model, m->h))) return rc;
        if ((rc = candy_hip_rms_norm(dev, m->h, L.ffn_norm, c.rms_eps, 1, c.d_model, m->xn))) return rc;
        if ((rc = quantize(m, m->xn, c.d_model))) return rc;
        if ((rc = linear(m, L.gate, m->gate_o))) return rc;
        if ((rc = linear(m, L.up, m->up_o))) return rc;
        if ((rc = candy_hip_silu_mul(dev, m->gate_o, m->up_o, c.d_ffn, m->act))) return rc;
        if ((rc = quantize(m, m->act, c.d_ffn))) return rc;
        if ((rc = linear(m, L.down, m->tmp))) return rc;
        if ((rc = candy_hip_add(dev, m->h, m->tmp, c.d_model, m->h))) return rc;
    }
    if ((rc = candy_hip_rms_norm(dev, m->h, m->out_norm, c.rms_eps, 1, c.d_model, m->xn))) return rc;
    if ((rc = quantize(m, m->xn, c.d_model))) return rc;
    if ((rc = linear(m, m->head, m->logits))) return rc;
    if (dev_logits) *dev_logits = m->logits;
    if (next_token) {
        if ((rc = candy_hip_argmax(dev, m->logits, 1, c.vocab, m->next_tok))) return rc;
        uint32_t t = 0;
        if ((rc = candy_hip_d2h(dev, &t, m->next_tok, sizeof(t)))) return rc;
        *next_token = (int32_t)t;
    }
    return CANDY_HIP_OK;
}

int candy_hip_llama_decode_hidden(candy_hip_llama *m, const float *dev_hidden, int32_t pos, const float **dev_logits,
                                  int32_t *next_token) {
    CANDY_REQUIRE(m && dev_hidden, "nil argument");
    CANDY_REQUIRE(pos >= 0 && pos < m->cfg.max_pos, "position %d outside the cache (max_pos %d)", pos, m->cfg.max_pos);
    if (int rc = llama_check_complete(m)) return rc;
    if (int rc = use_device(m->dev)) return rc;
    if (int rc = candy_hip_d2d(m->dev, m->h, dev_hidden, (size_t)m->cfg.d_model * sizeof(float))) return rc;
    return llama_step(m, pos, dev_logits, next_token);
}

int candy_hip_llama_decode(candy_hip_llama *m, int32_t token, int32_t pos, const float **dev_logits,
                           int32_t *next_token) {
    CANDY_REQUIRE(m, "model is nil");
    CANDY_REQUIRE(m->embed, "embedding table not set");
    CANDY_REQUIRE(token >= 0 && token < m->cfg.vocab, "token %d outside the vocabulary", token);
    CANDY_REQUIRE(pos >= 0 && pos < m->cfg.max_pos, "position %d outside the cache (max_pos %d)", pos, m->cfg.max_pos);
    if (int rc = llama_check_complete(m)) return rc;
    if (int rc = use_device(m->dev)) return rc;
    const int64_t id = token;
    if (int rc = candy_hip_h2d(m->dev, m->tok_id, &id, sizeof(id))) return rc;
    if (int rc = candy_hip_qindex_select(m->dev, m->embed, m->tok_id, 1, m->h)) return rc;
    return llama_step(m, pos, dev_logits, next_token);
}

}  // extern "C"
