// Arguments of the persistent decode-step kernel (persist.hip), filled by the decoder (llama.hip).
#pragma once

#include <stdint.h>

#include "internal.h"

namespace candy {

typedef unsigned long long u64;

// Device addresses of one layer's tensors (as integers: see global_ptr in persist.hip).
struct PersistLayer {
    u64 wq, wk, wv, wo, gate, up, down;
    u64 attn_norm, ffn_norm;
};

constexpr int PROF_SLOTS = 24;

struct PersistArgs {
    const PersistLayer *layers;
    int n_layers, d_model, n_heads, d_ffn, vocab, max_pos;
    float eps, scale;
    const float *out_norm;
    const uint8_t *head;
    int head_is_q6k;
    const float *cos_t, *sin_t;
    float *k_cache, *v_cache;     // [layer][head][max_pos][HD]
    const float *h_in;            // hidden state of the token (plain f32)
    const int *pos_ptr;
    const unsigned *epoch_ptr;    // bumped once per step by the host's set-step kernel, never 0
    // tagged exchange buffers, two of each (layer parity)
    u64 *x_ha, *x_hb;             // [2][d_model]: layer input / after attention
    u64 *x_qkv;                   // [2][3 * d_model]
    u64 *x_part;                  // [2][n_heads * n_splits * (HD + 2)]
    u64 *x_att;                   // [2][d_model]
    u64 *x_act;                   // [2][d_ffn]
    u64 *x_best;                  // [2 * G]: per workgroup (max logit, its index)
    float *logits;
    uint32_t *next_tok;
    unsigned *fail;
    int spin_limit;
    u64 *prof;                    // optional [G][n_layers + 1][PROF_SLOTS] wall-clock stamps inside the phases (nullptr: none)
};

// Dynamic LDS the kernel is launched with, and the launch itself (on dev->stream, one workgroup per CU).
size_t persist_lds_bytes(int d_model, int d_ffn);
int launch_decode_step(candy_hip_device *dev, const PersistArgs &a);

}  // namespace candy
