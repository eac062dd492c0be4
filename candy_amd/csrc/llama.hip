// Llama-style batch-1 decoder assembled from the library's ops.  candy has no model code; the
// block is the standard one (RMSNorm, q/k/v, RoPE, attention over the f32 KV cache, o, residual,
// RMSNorm, SwiGLU, residual; final RMSNorm, head, argmax) written as the sequence of
// BackendStorage calls (backend.go) a candy model would issue, with the quantized Linear in
// place of MatMul.
#include <cmath>
#include <cstdlib>
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
    float *k_cache = nullptr, *v_cache = nullptr;  // [n_layers][n_kv_heads][max_pos][head_dim], f32 or (kv_f16) fp16 in the same memory
    bool kv_f16 = false;
    float *cos_t = nullptr, *sin_t = nullptr;      // [max_pos][head_dim/2]
    float *h = nullptr, *q = nullptr, *k = nullptr, *v = nullptr;
    float *gate_o = nullptr, *up_o = nullptr, *logits = nullptr;
    unsigned *pair_tickets = nullptr;  // one counter per 32 FFN rows (fused gate/up kernel), zero between launches
    float *proj = nullptr;  // [d_model]: a projection's output before the residual add, for formats without that epilogue
    int8_t *xq = nullptr;           // planar Q8_0 quants of the current activation
    candy::Q8Scale *xs = nullptr;
    unsigned long long *next_key = nullptr;  // greedy token of the last step as k_argmax_key leaves it; zero before a step
    int64_t *tok_id = nullptr;
    int *d_pos = nullptr;                         // position of the token being decoded (device copy)
    void *attn_scratch = nullptr;                 // attention split partials
    int n_splits = 1;
    hipGraph_t graph = nullptr;                   // the captured step (layers + head + argmax)
    hipGraphExec_t graph_exec = nullptr;
    bool graph_dirty = true;
    bool use_graph = true;
    unsigned graph_epoch = 0;                     // the device's option epoch the graph was captured under
    std::vector<void *> owned;
    // prompt buffers, grown on demand to the longest prompt seen: [n][width] activations
    struct Prompt {
        int cap = 0;
        int64_t *ids = nullptr;
        float *h = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *att = nullptr, *tmp = nullptr;
        float *gate = nullptr, *up = nullptr;
        int8_t *xq = nullptr;
        candy::Q8Scale *xs = nullptr;
        _Float16 *xh = nullptr;  // the quantized activations as fp16 (d * q), for the fp16 tile kernels
        std::vector<void *> owned;
    } pf;
};

namespace candy {

// Parks the step's position and token id in device memory (read by the captured kernels).
__global__ void k_set_step(int *pos_dst, int pos, int64_t *tok_dst, int64_t tok, unsigned long long *key) {
    *pos_dst = pos;
    if (tok >= 0) *tok_dst = tok;
    *key = 0;  // the step's argmax folds into it
}

// Greedy generation without the host in the loop: the token the last step chose becomes the next step's input and
// is written to the list the caller gets at the end.
__global__ void k_chain_step(int *pos_dst, int pos, int64_t *tok_dst, unsigned long long *key, int32_t *list) {
    *pos_dst = pos;
    const uint32_t t = argmax_key_index(*key);
    *key = 0;
    *tok_dst = (int64_t)t;
    *list = (int32_t)t;
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

template <class T>
static int prompt_alloc(candy_hip_llama *m, T **p, size_t count) {
    void *d = nullptr;
    if (int rc = candy_hip_alloc(m->dev, count * sizeof(T), &d)) return rc;
    m->pf.owned.push_back(d);
    *p = (T *)d;
    return CANDY_HIP_OK;
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
    CANDY_REQUIRE(cfg->head_dim == 64 || cfg->head_dim == 128, "head_dim must be 64 or 128");
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
    if (!rc) rc = dev_alloc(m, &m->q, (size_t)cfg->n_heads * cfg->head_dim);
    if (!rc) rc = dev_alloc(m, &m->k, (size_t)cfg->n_kv_heads * cfg->head_dim);
    if (!rc) rc = dev_alloc(m, &m->v, (size_t)cfg->n_kv_heads * cfg->head_dim);
    if (!rc) rc = dev_alloc(m, &m->gate_o, (size_t)cfg->d_ffn);
    if (!rc) rc = dev_alloc(m, &m->pair_tickets, (size_t)cfg->d_ffn / 32 + 1);
    if (!rc) rc = candy_hip_zero(dev, m->pair_tickets, ((size_t)cfg->d_ffn / 32 + 1) * sizeof(unsigned));
    if (!rc) rc = dev_alloc(m, &m->proj, (size_t)cfg->d_model);
    if (!rc) rc = dev_alloc(m, &m->up_o, (size_t)cfg->d_ffn);
    if (!rc) rc = dev_alloc(m, &m->logits, (size_t)cfg->vocab + 4);  // the argmax kernel reads whole 16-byte pieces
    if (!rc) rc = dev_alloc(m, &m->xq, widest);
    if (!rc) rc = dev_alloc(m, &m->xs, widest / 32);
    if (!rc) rc = dev_alloc(m, &m->next_key, 1);
    if (!rc) rc = candy_hip_zero(dev, m->next_key, sizeof(unsigned long long));
    if (!rc) rc = dev_alloc(m, &m->tok_id, 1);
    if (!rc) rc = dev_alloc(m, &m->d_pos, 1);
    m->n_splits = attention_splits(dev, cfg->n_kv_heads, cfg->max_pos);
    if (!rc) {
        uint8_t *p = nullptr;
        rc = dev_alloc(m, &p, attention_scratch_bytes(cfg->n_heads, cfg->n_kv_heads, cfg->head_dim, m->n_splits));
        m->attn_scratch = p;
    }
    m->use_graph = dev->opt.llama_graph != 0;
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
    (void)hipSetDevice(m->dev->ordinal);
    (void)hipStreamSynchronize(m->dev->stream);
    if (m->graph_exec) (void)hipGraphExecDestroy(m->graph_exec);
    if (m->graph) (void)hipGraphDestroy(m->graph);
    for (void *p : m->owned) (void)candy_hip_free(m->dev, p);
    for (void *p : m->pf.owned) (void)candy_hip_free(m->dev, p);
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
    m->graph_dirty = true;
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
    m->graph_dirty = true;
    if (which == CANDY_HIP_W_OUT_NORM) { m->out_norm = dev_alpha; return CANDY_HIP_OK; }
    CANDY_REQUIRE(which == CANDY_HIP_W_ATTN_NORM || which == CANDY_HIP_W_FFN_NORM, "weight kind %d is not a norm", which);
    CANDY_REQUIRE(layer >= 0 && layer < m->cfg.n_layers, "layer %d out of range", layer);
    if (which == CANDY_HIP_W_ATTN_NORM) m->layers[layer].attn_norm = dev_alpha;
    else m->layers[layer].ffn_norm = dev_alpha;
    return CANDY_HIP_OK;
}

int candy_hip_llama_set_graph(candy_hip_llama *m, int enable) {
    CANDY_REQUIRE(m, "model is nil");
    m->use_graph = enable != 0;
    m->graph_dirty = true;  // also the way to have a changed device option picked up: the step is captured again
    return CANDY_HIP_OK;
}

int candy_hip_llama_kv_cache(candy_hip_llama *m, float **dev_k, float **dev_v, size_t *bytes_each) {
    CANDY_REQUIRE(m, "model is nil");
    if (dev_k) *dev_k = m->k_cache;
    if (dev_v) *dev_v = m->v_cache;
    if (bytes_each)
        *bytes_each = (size_t)m->cfg.n_layers * m->cfg.n_kv_heads * m->cfg.max_pos * m->cfg.head_dim * (m->kv_f16 ? 2 : 4);
    return CANDY_HIP_OK;
}

int candy_hip_llama_hidden(candy_hip_llama *m, const float **dev_hidden) {
    CANDY_REQUIRE(m && dev_hidden, "nil argument");
    *dev_hidden = m->h;
    return CANDY_HIP_OK;
}

int candy_hip_llama_set_kv_f16(candy_hip_llama *m, int enable) {
    CANDY_REQUIRE(m, "model is nil");
    if (int rc = use_device(m->dev)) return rc;
    m->kv_f16 = enable != 0;
    m->graph_dirty = true;
    // the cache's contents do not survive a change of element type
    const size_t kv = (size_t)m->cfg.n_layers * m->cfg.n_kv_heads * m->cfg.max_pos * m->cfg.head_dim;
    if (int rc = candy_hip_zero(m->dev, m->k_cache, kv * sizeof(float))) return rc;
    return candy_hip_zero(m->dev, m->v_cache, kv * sizeof(float));
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

// Enqueues one decode step (hidden state in m->h, position in *m->d_pos) on the stream:
// 10 launches per layer. Everything it touches is owned by the model, nothing allocates or
// synchronises, so the sequence can be captured once and replayed for every token.
// y_i = W_i . q8(rmsnorm(h) * alpha) for up to three weights: one fused launch, or
// RMSNorm+quantize then the batch-1 kernel when no fused instantiation covers the shape.
// Layer l's part of a cache array (elements are 4 bytes, or 2 with the fp16 cache).
static void *layer_cache(const candy_hip_llama *m, float *base, int l) {
    const size_t layer_kv = (size_t)m->cfg.n_kv_heads * m->cfg.max_pos * m->cfg.head_dim;
    return (uint8_t *)base + (size_t)l * layer_kv * (m->kv_f16 ? 2 : 4);
}

static int norm_linear(candy_hip_llama *m, const float *alpha, const candy_hip_qtensor *const *ws, float *const *ys,
                       int n) {
    const candy_hip_llama_config &c = m->cfg;
    int rc;
    WideLaunch Wd;
    Wd.n = n;
    for (int i = 0; i < n; ++i) { Wd.w[i] = ws[i]; Wd.y[i] = ys[i]; }
    Wd.x = m->h; Wd.alpha = alpha; Wd.eps = c.rms_eps;
    rc = launch_matvec_wide(m->dev, Wd);
    if (rc != CANDY_HIP_ERR_UNSUPPORTED) return rc;
    // a vocabulary-sized Q6_K head: the norm as a launch of its own and the batch-1 kernel stream the rows faster than
    // the fused kernel, whose thousands of workgroups each repeat the prologue
    const bool plain_head = n == 1 && ws[0]->fmt == CANDY_HIP_Q6_K && ws[0]->rows >= 16384;
    FusedLaunch F;
    F.n = n;
    for (int i = 0; i < n; ++i) { F.w[i] = ws[i]; F.y[i] = ys[i]; }
    F.x = m->h; F.alpha = alpha; F.eps = c.rms_eps;
    rc = plain_head ? CANDY_HIP_ERR_UNSUPPORTED : launch_matvec_fused(m->dev, F);
    if (rc != CANDY_HIP_ERR_UNSUPPORTED) return rc;
    if ((rc = launch_rms_norm_quant(m->dev, m->h, alpha, c.rms_eps, 1, c.d_model, nullptr, m->xq, m->xs))) return rc;
    return launch_matvec_multi(m->dev, ws, ys, nullptr, n, m->xq, m->xs);
}

// h += W . (quantized activations in xq/xs)
static int linear_residual(candy_hip_llama *m, const candy_hip_qtensor *w) {
    FusedLaunch F;
    F.n = 1; F.w[0] = w; F.y[0] = m->h; F.res[0] = m->h; F.xq = m->xq; F.xs = m->xs;
    int rc = launch_matvec_fused(m->dev, F);
    if (rc != CANDY_HIP_ERR_UNSUPPORTED) return rc;
    const candy_hip_qtensor *ws[1] = {w};
    float *ys[1] = {m->h};
    const float *res[1] = {m->h};
    if (format_has_batch1_kernel(w->fmt)) {
        rc = launch_matvec_multi(m->dev, ws, ys, res, 1, m->xq, m->xs);
        if (rc != CANDY_HIP_ERR_UNSUPPORTED) return rc;
    }
    // rows too long for the batch-1 kernel: looping kernel into a buffer of its own, then the add
    if ((rc = launch_matvec(m->dev, w, m->xq, m->xs, 1, m->proj))) return rc;
    return candy_hip_add(m->dev, m->h, m->proj, w->rows, m->h);
}

// Enqueues one decode step (hidden state in m->h, position in *m->d_pos) on the stream: six
// launches per layer. Everything it touches is owned by the model, nothing allocates or
// synchronises, so the sequence can be captured once and replayed for every token.
static int llama_enqueue_step(candy_hip_llama *m) {
    const candy_hip_llama_config &c = m->cfg;
    candy_hip_device *dev = m->dev;
    const float scale = 1.0f / std::sqrt((float)c.head_dim);
    int rc;
    for (int l = 0; l < c.n_layers; ++l) {
        const candy_hip_llama::Layer &L = m->layers[l];
        void *kc = layer_cache(m, m->k_cache, l), *vc = layer_cache(m, m->v_cache, l);
        {   // RMSNorm + quantize + q/k/v
            const candy_hip_qtensor *ws[3] = {L.wq, L.wk, L.wv};
            float *ys[3] = {m->q, m->k, m->v};
            if ((rc = norm_linear(m, L.attn_norm, ws, ys, 3))) return rc;
        }
        {   // Rope on q and the new k, append k/v to the cache, attention; the merge quantizes for Wo
            AttnLaunch A;
            A.q = m->q; A.k_new = m->k; A.v_new = m->v; A.cos_t = m->cos_t; A.sin_t = m->sin_t;
            A.k_cache = kc; A.v_cache = vc; A.kv_f16 = m->kv_f16; A.pos_ptr = m->d_pos;
            A.cache_stride = (int64_t)c.max_pos * c.head_dim; A.scale = scale;
            A.n_heads = c.n_heads; A.n_kv_heads = c.n_kv_heads; A.head_dim = c.head_dim; A.n_splits = m->n_splits;
            A.scratch = m->attn_scratch;
            A.oq = m->xq; A.os = m->xs;
            if ((rc = launch_attention(dev, A))) return rc;
        }
        if ((rc = linear_residual(m, L.wo))) return rc;  // h += Wo . att
        {   // RMSNorm + quantize + gate/up + SiLU*Mul + quantize
            WideLaunch Wd;
            Wd.n = 2; Wd.w[0] = L.gate; Wd.w[1] = L.up; Wd.pair = true;
            Wd.x = m->h; Wd.alpha = L.ffn_norm; Wd.eps = c.rms_eps; Wd.oq = m->xq; Wd.os = m->xs;
            Wd.pair_act = m->gate_o; Wd.pair_tickets = m->pair_tickets;
            // Where the down projection can quantize its input itself, gate / up leaves the f32 values: the same 32
            // values per block quantized by the same code, so the same bits, without blocks shared between workgroups.
            WideLaunch Dn;
            Dn.n = 1; Dn.w[0] = L.down; Dn.y[0] = m->h; Dn.res[0] = m->h; Dn.x = m->gate_o;
            const bool down_quant = wide_quant_long_covers(dev, Dn);
            if (down_quant) { Wd.oq = nullptr; Wd.os = nullptr; }
            rc = launch_matvec_wide(dev, Wd);
            if (rc == CANDY_HIP_OK) {
                if (down_quant) {
                    if ((rc = launch_matvec_wide(dev, Dn))) return rc;  // h += Wdown . q8(act)
                    continue;
                }
                if ((rc = linear_residual(m, L.down))) return rc;  // h += Wdown . act
                continue;
            }
            if (down_quant && rc == CANDY_HIP_ERR_UNSUPPORTED) return fail(CANDY_HIP_ERR_HIP, "internal: gate / up launch refused");
            if (rc != CANDY_HIP_ERR_UNSUPPORTED) return rc;
            FusedLaunch F;
            F.n = 2; F.w[0] = L.gate; F.w[1] = L.up; F.pair = true;
            F.x = m->h; F.alpha = L.ffn_norm; F.eps = c.rms_eps; F.oq = m->xq; F.os = m->xs;
            F.pair_act = m->gate_o; F.pair_tickets = m->pair_tickets;
            rc = launch_matvec_fused(dev, F);
            if (rc == CANDY_HIP_ERR_UNSUPPORTED) {
                const candy_hip_qtensor *ws[2] = {L.gate, L.up};
                float *ys[2] = {m->gate_o, m->up_o};
                if ((rc = norm_linear(m, L.ffn_norm, ws, ys, 2))) return rc;
                rc = launch_silu_mul_quant(dev, m->gate_o, m->up_o, 1, c.d_ffn, nullptr, m->xq, m->xs);
            }
            if (rc) return rc;
        }
        if ((rc = linear_residual(m, L.down))) return rc;  // h += Wdown . act
    }
    {
        const candy_hip_qtensor *ws[1] = {m->head};
        float *ys[1] = {m->logits};
        if ((rc = norm_linear(m, m->out_norm, ws, ys, 1))) return rc;
    }
    return launch_argmax_key(dev, m->logits, c.vocab, m->next_key);
}

// chain_to: null, or where the token chosen by the previous step is recorded while it becomes this step's input
static int llama_step(candy_hip_llama *m, int32_t pos, int64_t token, const float *dev_hidden,
                      const float **dev_logits, int32_t *next_token, int32_t *chain_to = nullptr) {
    candy_hip_device *dev = m->dev;
    int rc;
    if (chain_to)
        hipLaunchKernelGGL(k_chain_step, dim3(1), dim3(1), 0, dev->stream, m->d_pos, (int)pos, m->tok_id, m->next_key, chain_to);
    else
        hipLaunchKernelGGL(k_set_step, dim3(1), dim3(1), 0, dev->stream, m->d_pos, (int)pos, m->tok_id, token, m->next_key);
    CANDY_LAUNCH_CHECK();
    if (dev_hidden) {
        if ((rc = candy_hip_d2d(dev, m->h, dev_hidden, (size_t)m->cfg.d_model * sizeof(float)))) return rc;
    } else {
        if ((rc = candy_hip_qindex_select(dev, m->embed, m->tok_id, 1, m->h))) return rc;
    }
    if (m->use_graph) {
        if (m->graph_epoch != dev->opt_epoch) m->graph_dirty = true;  // an option changed: other kernels may be due
        if (m->graph_dirty) {
            // a replay of the old graph may still be in flight (a caller that did not ask for the token): drain first
            if (m->graph_exec) CANDY_HIP_TRY(hipStreamSynchronize(dev->stream));
            if (m->graph_exec) CANDY_HIP_TRY(hipGraphExecDestroy(m->graph_exec));
            if (m->graph) CANDY_HIP_TRY(hipGraphDestroy(m->graph));
            m->graph_exec = nullptr;
            m->graph = nullptr;
            // the gate/up kernels count on their per-block tickets being zero at launch and leave them so; a step
            // that was cut short (an error, a device reset) may not have: start every new graph from zero
            if ((rc = launch_zero(dev, m->pair_tickets, ((size_t)m->cfg.d_ffn / 32 + 1) * sizeof(unsigned)))) return rc;
            CANDY_HIP_TRY(hipStreamBeginCapture(dev->stream, hipStreamCaptureModeThreadLocal));
            rc = llama_enqueue_step(m);
            hipError_t e = hipStreamEndCapture(dev->stream, &m->graph);
            if (rc) return rc;
            CANDY_HIP_TRY(e);
            CANDY_HIP_TRY(hipGraphInstantiate(&m->graph_exec, m->graph, nullptr, nullptr, 0));
            m->graph_dirty = false;
            m->graph_epoch = dev->opt_epoch;
        }
        CANDY_HIP_TRY(hipGraphLaunch(m->graph_exec, dev->stream));
    } else if ((rc = llama_enqueue_step(m))) {
        (void)launch_zero(dev, m->pair_tickets, ((size_t)m->cfg.d_ffn / 32 + 1) * sizeof(unsigned));  // see above
        return rc;
    }
    if (dev_logits) *dev_logits = m->logits;
    if (next_token) {
        unsigned long long key = 0;
        if ((rc = candy_hip_d2h(dev, &key, m->next_key, sizeof(key)))) return rc;
        *next_token = (int32_t)argmax_key_index(key);
    }
    return CANDY_HIP_OK;
}

static int prompt_reserve(candy_hip_llama *m, int n) {
    candy_hip_llama::Prompt &P = m->pf;
    if (n <= P.cap) return CANDY_HIP_OK;
    const candy_hip_llama_config &c = m->cfg;
    CANDY_HIP_TRY(hipStreamSynchronize(m->dev->stream));
    for (void *p : P.owned) (void)candy_hip_free(m->dev, p);
    P.owned.clear();
    P.cap = 0;
    const size_t N = (size_t)n, qd = (size_t)c.n_heads * c.head_dim, kvd = (size_t)c.n_kv_heads * c.head_dim;
    const size_t widest = std::max(std::max((size_t)c.d_model, (size_t)c.d_ffn), qd);
    int rc = CANDY_HIP_OK;
    if (!rc) rc = prompt_alloc(m, &P.ids, N);
    if (!rc) rc = prompt_alloc(m, &P.h, N * c.d_model);
    if (!rc) rc = prompt_alloc(m, &P.q, N * (qd + 2 * kvd));  // q, k, v end to end: one split-K sum serves the three
    if (!rc) {
        P.k = P.q + N * qd;
        P.v = P.k + N * kvd;
    }
    if (!rc) rc = prompt_alloc(m, &P.att, N * qd);
    if (!rc) rc = prompt_alloc(m, &P.tmp, N * c.d_model);
    if (!rc) rc = prompt_alloc(m, &P.gate, N * c.d_ffn);
    if (!rc) rc = prompt_alloc(m, &P.up, N * c.d_ffn);
    if (!rc) rc = prompt_alloc(m, &P.xq, N * widest);
    if (!rc) rc = prompt_alloc(m, &P.xs, N * (widest / 32));
    if (!rc) rc = prompt_alloc(m, &P.xh, (size_t)mmq_m_pad(n) * widest);  // the tile kernel reads whole tiles of rows
    if (rc) return rc;
    P.cap = n;
    return CANDY_HIP_OK;
}

// The prompt pass: the decode step's sequence with n rows per activation. Linears go through the
// batched contraction (MFMA tiles from 16 rows up), attention is causal over the cache, and only
// the last row goes through the final norm and the head.
static int llama_enqueue_prompt(candy_hip_llama *m, int n, int pos0) {
    const candy_hip_llama_config &c = m->cfg;
    candy_hip_device *dev = m->dev;
    candy_hip_llama::Prompt &P = m->pf;
    const int64_t cache_stride = (int64_t)c.max_pos * c.head_dim;
    const int64_t qd = (int64_t)c.n_heads * c.head_dim;
    const float scale = 1.0f / std::sqrt((float)c.head_dim);
    int rc;
    P.k = P.q + (size_t)n * qd;  // q, k and v of this pass end to end, whatever the buffer's capacity
    P.v = P.k + (size_t)n * c.n_kv_heads * c.head_dim;
    if ((rc = candy_hip_qindex_select(dev, m->embed, P.ids, n, P.h))) return rc;
    // A projection that splits K leaves its partial copies for the launch that follows: the norm launch behind o / down
    // sums them, adds the residual and writes P.h before it normalizes, the rope launch behind q / k / v sums them on
    // its way to the cache (one launch and one pass over the outputs less each time).
    SplitPending pend;
    auto norm_quant = [&](const float *alpha, _Float16 *xh_out) -> int {
        const int e = pend.n_split > 0
                          ? launch_split_rms_norm_quant(dev, pend, alpha, c.rms_eps, n, c.d_model, P.xq, P.xs, xh_out)
                          : launch_rms_norm_quant(dev, P.h, alpha, c.rms_eps, n, c.d_model, nullptr, P.xq, P.xs, xh_out);
        pend.n_split = 0;
        return e;
    };
    for (int l = 0; l < c.n_layers; ++l) {
        const candy_hip_llama::Layer &L = m->layers[l];
        void *kc = layer_cache(m, m->k_cache, l), *vc = layer_cache(m, m->v_cache, l);
        // Where a projection runs on the fp16 tiles, the kernel that quantizes its input also writes the
        // fp16 expansion (one conversion for q/k/v, one for gate/up), and the residual add rides in the
        // projection's epilogue.
        auto xh_for = [&](const candy_hip_qtensor *w) { return mmq_f16_big_covers(w, n) ? P.xh : nullptr; };
        auto add_linear = [&](const candy_hip_qtensor *w) -> int {  // P.h += (quantized activations) . w^T
            if (mmq_fuses_residual(w, n)) {
                dev->defer_split = &pend;
                const int e = launch_contract(dev, w, P.xq, P.xs, n, P.h, xh_for(w), P.h);
                dev->defer_split = nullptr;
                return e;
            }
            if (int e = launch_contract(dev, w, P.xq, P.xs, n, P.tmp)) return e;
            return candy_hip_add(dev, P.h, P.tmp, (int64_t)n * c.d_model, P.h);
        };
        _Float16 *xh = (xh_for(L.wq) || xh_for(L.wk) || xh_for(L.wv)) ? P.xh : nullptr;
        if ((rc = norm_quant(L.attn_norm, xh))) return rc;
        const candy_hip_qtensor *qkv_w[3] = {L.wq, L.wk, L.wv};
        float *qkv_y[3] = {P.q, P.k, P.v};
        if (xh && mmq_f16_group_covers(qkv_w, 3, n)) {  // one grid for the three projections
            dev->defer_split = &pend;  // q, k and v lie end to end: the rope launch sums their partial copies
            rc = launch_mmq_f16_group(dev, qkv_w, qkv_y, 3, xh, n);
            dev->defer_split = nullptr;
            if (rc) return rc;
        } else {
            if ((rc = launch_contract(dev, L.wq, P.xq, P.xs, n, P.q, xh_for(L.wq)))) return rc;
            if ((rc = launch_contract(dev, L.wk, P.xq, P.xs, n, P.k, xh_for(L.wk)))) return rc;
            if ((rc = launch_contract(dev, L.wv, P.xq, P.xs, n, P.v, xh_for(L.wv)))) return rc;
        }
        rc = launch_prefill_rope_kv(dev, P.q, P.k, P.v, m->cos_t, m->sin_t, kc, vc, m->kv_f16, n, pos0, c.n_heads,
                                    c.n_kv_heads, c.head_dim, cache_stride, &pend);
        pend.n_split = 0;
        if (rc) return rc;
        _Float16 *att_xh = xh_for(L.wo) && mmq_fuses_residual(L.wo, n) && attn_prefill_writes_half(dev, c.head_dim) ? P.xh : nullptr;
        if ((rc = launch_attn_prefill(dev, P.q, kc, vc, m->kv_f16, P.att, n, pos0, c.n_heads, c.n_kv_heads, c.head_dim,
                                      cache_stride, scale, att_xh)))
            return rc;
        if (!att_xh && (rc = launch_quantize_q8(dev, P.att, n, qd, P.xq, P.xs, nullptr, xh_for(L.wo)))) return rc;
        if ((rc = add_linear(L.wo))) return rc;  // h += Wo . att
        xh = (xh_for(L.gate) || xh_for(L.up)) ? P.xh : nullptr;
        if ((rc = norm_quant(L.ffn_norm, xh))) return rc;
        const candy_hip_qtensor *gu_w[2] = {L.gate, L.up};
        float *gu_y[2] = {P.gate, P.up};
        if (xh && mmq_f16_group_covers(gu_w, 2, n)) {  // the second projection's tiles fill the first one's last round
            if ((rc = launch_mmq_f16_group(dev, gu_w, gu_y, 2, xh, n))) return rc;
        } else {
            if ((rc = launch_contract(dev, L.gate, P.xq, P.xs, n, P.gate, xh_for(L.gate)))) return rc;
            if ((rc = launch_contract(dev, L.up, P.xq, P.xs, n, P.up, xh_for(L.up)))) return rc;
        }
        if ((rc = launch_silu_mul_quant(dev, P.gate, P.up, n, c.d_ffn, nullptr, P.xq, P.xs, xh_for(L.down))))
            return rc;
        if ((rc = add_linear(L.down))) return rc;  // h += Wdown . act
    }
    if (pend.n_split > 0 &&
        (rc = launch_splitk_sum(dev, pend.part, pend.y, pend.res, pend.count, pend.n_split, pend.stride)))
        return rc;
    if ((rc = candy_hip_d2d(dev, m->h, P.h + (size_t)(n - 1) * c.d_model, (size_t)c.d_model * sizeof(float)))) return rc;
    const candy_hip_qtensor *ws[1] = {m->head};
    float *ys[1] = {m->logits};
    if ((rc = norm_linear(m, m->out_norm, ws, ys, 1))) return rc;
    if ((rc = launch_zero(dev, m->next_key, sizeof(unsigned long long)))) return rc;  // no step kernel in front here
    return launch_argmax_key(dev, m->logits, c.vocab, m->next_key);
}

int candy_hip_llama_prefill(candy_hip_llama *m, const int32_t *tokens, int32_t n_tokens, int32_t pos0,
                            const float **dev_logits, int32_t *next_token) {
    CANDY_REQUIRE(m, "model is nil");
    CANDY_REQUIRE(m->embed, "embedding table not set");
    CANDY_REQUIRE(tokens && n_tokens > 0, "prompt is empty");
    CANDY_REQUIRE(pos0 >= 0 && (int64_t)pos0 + n_tokens <= m->cfg.max_pos,
                  "positions %d..%lld outside the cache (max_pos %d)", pos0, (long long)pos0 + n_tokens - 1,
                  m->cfg.max_pos);
    std::vector<int64_t> ids((size_t)n_tokens);
    for (int32_t i = 0; i < n_tokens; ++i) {
        CANDY_REQUIRE(tokens[i] >= 0 && tokens[i] < m->cfg.vocab, "token %d outside the vocabulary", tokens[i]);
        ids[(size_t)i] = tokens[i];
    }
    if (int rc = llama_check_complete(m)) return rc;
    if (int rc = use_device(m->dev)) return rc;
    if (int rc = prompt_reserve(m, n_tokens)) return rc;
    if (int rc = candy_hip_h2d(m->dev, m->pf.ids, ids.data(), ids.size() * sizeof(int64_t))) return rc;
    if (int rc = llama_enqueue_prompt(m, n_tokens, pos0)) return rc;
    if (dev_logits) *dev_logits = m->logits;
    if (next_token) {
        unsigned long long key = 0;
        if (int rc = candy_hip_d2h(m->dev, &key, m->next_key, sizeof(key))) return rc;
        *next_token = (int32_t)argmax_key_index(key);
    }
    return CANDY_HIP_OK;
}

int candy_hip_llama_decode_hidden(candy_hip_llama *m, const float *dev_hidden, int32_t pos, const float **dev_logits,
                                  int32_t *next_token) {
    CANDY_REQUIRE(m && dev_hidden, "nil argument");
    CANDY_REQUIRE(pos >= 0 && pos < m->cfg.max_pos, "position %d outside the cache (max_pos %d)", pos, m->cfg.max_pos);
    if (int rc = llama_check_complete(m)) return rc;
    if (int rc = use_device(m->dev)) return rc;
    return llama_step(m, pos, -1, dev_hidden, dev_logits, next_token);
}

int candy_hip_llama_decode(candy_hip_llama *m, int32_t token, int32_t pos, const float **dev_logits,
                           int32_t *next_token) {
    CANDY_REQUIRE(m, "model is nil");
    CANDY_REQUIRE(m->embed, "embedding table not set");
    CANDY_REQUIRE(token >= 0 && token < m->cfg.vocab, "token %d outside the vocabulary", token);
    CANDY_REQUIRE(pos >= 0 && pos < m->cfg.max_pos, "position %d outside the cache (max_pos %d)", pos, m->cfg.max_pos);
    if (int rc = llama_check_complete(m)) return rc;
    if (int rc = use_device(m->dev)) return rc;
    return llama_step(m, pos, token, nullptr, dev_logits, next_token);
}

int candy_hip_llama_generate(candy_hip_llama *m, int32_t token, int32_t pos, int32_t n_steps, int32_t *tokens) {
    CANDY_REQUIRE(m && tokens, "nil argument");
    CANDY_REQUIRE(m->embed, "embedding table not set");
    CANDY_REQUIRE(token >= 0 && token < m->cfg.vocab, "token %d outside the vocabulary", token);
    CANDY_REQUIRE(n_steps >= 1, "invalid number of steps %d", n_steps);
    CANDY_REQUIRE(pos >= 0 && (int64_t)pos + n_steps <= m->cfg.max_pos, "positions %d .. %lld outside the cache (max_pos %d)",
                  pos, (long long)pos + n_steps - 1, m->cfg.max_pos);
    if (int rc = llama_check_complete(m)) return rc;
    if (int rc = use_device(m->dev)) return rc;
    int32_t *list = nullptr;  // one slot per step; slot i takes the token step i chose
    if (int rc = candy_hip_alloc(m->dev, (size_t)(n_steps + 1) * sizeof(int32_t), (void **)&list)) return rc;
    int rc = llama_step(m, pos, token, nullptr, nullptr, nullptr);
    for (int i = 1; i < n_steps && !rc; ++i) rc = llama_step(m, pos + i, -1, nullptr, nullptr, nullptr, list + i - 1);
    if (!rc) {
        // the last step's choice: recorded by the same kernel, into a step that is not run (position and token
        // registers are rewritten by whatever step comes next)
        hipLaunchKernelGGL(k_chain_step, dim3(1), dim3(1), 0, m->dev->stream, m->d_pos, (int)(pos + n_steps - 1), m->tok_id,
                           m->next_key, list + n_steps - 1);
        if (hipGetLastError() != hipSuccess) rc = fail(CANDY_HIP_ERR_HIP, "launch failed");
    }
    if (!rc) rc = candy_hip_d2h(m->dev, tokens, list, (size_t)n_steps * sizeof(int32_t));
    const int rc2 = candy_hip_free(m->dev, list);
    return rc ? rc : rc2;
}

}  // extern "C"
