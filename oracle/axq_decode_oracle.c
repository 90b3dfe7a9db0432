/*
 * CPU oracle for the Llama/Mistral-style decode step.  TEST INFRASTRUCTURE ONLY
 * (loaded by tests, the smoke entry and the benchmark's CPU leg; never by the
 * product library).
 *
 * Formulas follow the reference model code, with its known defects left out
 * (whole-tensor softmax, flat `cat`; the cache here is f16, as the decode
 * workload specifies, where the reference's is f32):
 *
 *   RMSNorm            crates/axonml-llm/src/llama.rs:158-187
 *                      rms = sqrt(mean(x^2) + eps); y = (x / rms) * w
 *   RoPE (half-split)  crates/axonml-llm/src/llama.rs:223-252, 281-321
 *                      inv_freq_i = 1 / theta^(2i/d); angle = pos * inv_freq_i
 *                      o[i] = x[i] c - x[i+d/2] s; o[i+d/2] = x[i] s + x[i+d/2] c
 *   KV cache append    crates/axonml-llm/src/attention.rs:19-126
 *   GQA attention      crates/axonml-llm/src/llama.rs:378-495
 *                      kv head = q head / (heads / kv_heads); causal softmax of
 *                      q.k / sqrt(d) over positions 0..pos; weighted sum of v
 *   SwiGLU MLP         crates/axonml-llm/src/llama.rs:562-567,
 *                      silu(x) = x * sigmoid(x) (crates/axonml-tensor/src/ops/mod.rs:214-217)
 *   greedy argmax      crates/axonml-llm/src/llama.rs:980-1036 (Iterator::max_by:
 *                      of equal maxima the LAST index wins)
 *   linears            y = x W^T with W dequantised per oracle/axq_oracle.c
 *                      (crates/axonml-nn/src/layers/linear.rs:104-140); the
 *                      reference builds its LLaMA linears with a bias that is
 *                      never loaded (zeros), so no bias is added here.
 *
 * Parity status: the reference decode cannot be compiled or run here and its
 * own tests check shapes only (llama.rs:1123-1211), so this restatement is
 * pinned by closed-form cases in the tests (RMSNorm of a constant vector, RoPE
 * at position 0 and against numpy, single-position softmax, a numpy float64
 * forward on a tiny model), not by reference outputs: "parity unpinned" with
 * respect to the reference's bits.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define AXO_API __attribute__((visibility("default")))

uint16_t axo_f32_to_f16(float f);
float axo_f16_to_f32(uint16_t h);
int axo_dequantize(int type, const uint8_t *packed, size_t numel, float *out);

typedef struct {
    int32_t vocab_size, hidden_size, intermediate_size, num_layers;
    int32_t num_heads, num_kv_heads, head_dim, max_seq_len;
    float rms_norm_eps, rope_theta;
    int32_t sliding_window; /* 0 = attend to the whole cache; else the last sliding_window positions (mistral.rs:204-238) */
} axo_model_config;

enum { AXO_LIN_Q = 0, AXO_LIN_K, AXO_LIN_V, AXO_LIN_O, AXO_LIN_GATE, AXO_LIN_UP, AXO_LIN_DOWN, AXO_LIN_COUNT };

typedef struct {
    float *lin[AXO_LIN_COUNT]; /* dequantised f32, [out, in] */
    float *norm[2];            /* attention norm, ffn norm */
    uint16_t *kc, *vc;         /* f16 [kv_heads][max_seq][head_dim] */
} axo_layer;

typedef struct axo_model {
    axo_model_config cfg;
    uint16_t *emb; /* f16 [vocab, hidden], or */
    float *emb32;  /* f32 [vocab, hidden] (embedding.rs:103-146 keeps f32): one of the two is set */
    float *final_norm;
    float *head; /* f32 [vocab, hidden] */
    axo_layer *layers;
    float *h, *xn, *q, *k, *v, *att, *o, *g, *u, *scores;
} axo_model;

static void lin_dims(const axo_model_config *c, int which, size_t *out, size_t *in) {
    size_t H = (size_t)c->hidden_size, I = (size_t)c->intermediate_size;
    size_t qd = (size_t)c->num_heads * c->head_dim, kd = (size_t)c->num_kv_heads * c->head_dim;
    switch (which) {
    case AXO_LIN_Q: *out = qd; *in = H; break;
    case AXO_LIN_K: case AXO_LIN_V: *out = kd; *in = H; break;
    case AXO_LIN_O: *out = H; *in = qd; break;
    case AXO_LIN_GATE: case AXO_LIN_UP: *out = I; *in = H; break;
    default: *out = H; *in = I; break;
    }
}

AXO_API axo_model *axo_model_create(const axo_model_config *cfg) {
    axo_model *m = (axo_model *)calloc(1, sizeof *m);
    if (!m) return NULL;
    m->cfg = *cfg;
    size_t H = (size_t)cfg->hidden_size, I = (size_t)cfg->intermediate_size;
    size_t qd = (size_t)cfg->num_heads * cfg->head_dim, kd = (size_t)cfg->num_kv_heads * cfg->head_dim;
    m->layers = (axo_layer *)calloc((size_t)cfg->num_layers, sizeof(axo_layer));
    for (int l = 0; l < cfg->num_layers; l++) {
        for (int n = 0; n < 2; n++) {
            m->layers[l].norm[n] = (float *)malloc(H * sizeof(float));
            for (size_t i = 0; i < H; i++) m->layers[l].norm[n][i] = 1.0f;
        }
        m->layers[l].kc = (uint16_t *)calloc(kd * (size_t)cfg->max_seq_len, 2);
        m->layers[l].vc = (uint16_t *)calloc(kd * (size_t)cfg->max_seq_len, 2);
    }
    m->final_norm = (float *)malloc(H * sizeof(float));
    for (size_t i = 0; i < H; i++) m->final_norm[i] = 1.0f;
    m->h = (float *)calloc(H, 4); m->xn = (float *)calloc(H, 4);
    m->q = (float *)calloc(qd, 4); m->k = (float *)calloc(kd, 4); m->v = (float *)calloc(kd, 4);
    m->att = (float *)calloc(qd, 4); m->o = (float *)calloc(H > I ? H : I, 4);
    m->g = (float *)calloc(I, 4); m->u = (float *)calloc(I, 4);
    m->scores = (float *)calloc((size_t)cfg->max_seq_len, 4);
    return m;
}

AXO_API void axo_model_free(axo_model *m) {
    if (!m) return;
    for (int l = 0; l < m->cfg.num_layers; l++) {
        for (int i = 0; i < AXO_LIN_COUNT; i++) free(m->layers[l].lin[i]);
        free(m->layers[l].norm[0]); free(m->layers[l].norm[1]);
        free(m->layers[l].kc); free(m->layers[l].vc);
    }
    free(m->layers); free(m->emb); free(m->emb32); free(m->final_norm); free(m->head);
    free(m->h); free(m->xn); free(m->q); free(m->k); free(m->v); free(m->att); free(m->o);
    free(m->g); free(m->u); free(m->scores);
    free(m);
}

AXO_API int axo_model_set_embedding_f16(axo_model *m, const uint16_t *table) {
    size_t n = (size_t)m->cfg.vocab_size * m->cfg.hidden_size;
    free(m->emb);
    free(m->emb32);
    m->emb32 = NULL;
    m->emb = (uint16_t *)malloc(n * 2);
    if (!m->emb) return -1;
    memcpy(m->emb, table, n * 2);
    return 0;
}

/* Embedding::lookup on the f32 weight (nn/src/layers/embedding.rs:103-146): the row is copied as it is. */
AXO_API int axo_model_set_embedding_f32(axo_model *m, const float *table) {
    size_t n = (size_t)m->cfg.vocab_size * m->cfg.hidden_size;
    free(m->emb);
    free(m->emb32);
    m->emb = NULL;
    m->emb32 = (float *)malloc(n * 4);
    if (!m->emb32) return -1;
    memcpy(m->emb32, table, n * 4);
    return 0;
}

/* layer = -1 selects the final norm; which = 0 attention norm, 1 ffn norm. */
AXO_API int axo_model_set_norm(axo_model *m, int layer, int which, const float *w) {
    size_t H = (size_t)m->cfg.hidden_size;
    float *dst = layer < 0 ? m->final_norm : m->layers[layer].norm[which];
    memcpy(dst, w, H * sizeof(float));
    return 0;
}

/* layer = -1 selects lm_head (which ignored). */
AXO_API int axo_model_set_linear(axo_model *m, int layer, int which, int type, const uint8_t *packed) {
    size_t out, in;
    float **slot;
    if (layer < 0) {
        out = (size_t)m->cfg.vocab_size; in = (size_t)m->cfg.hidden_size;
        slot = &m->head;
    } else {
        lin_dims(&m->cfg, which, &out, &in);
        slot = &m->layers[layer].lin[which];
    }
    free(*slot);
    *slot = (float *)malloc(out * in * sizeof(float));
    if (!*slot) return -1;
    return axo_dequantize(type, packed, out * in, *slot);
}

static void matvec(const float *w, const float *x, size_t out, size_t in, float *y) {
#pragma omp parallel for schedule(static)
    for (long long j = 0; j < (long long)out; j++) {
        const float *wr = w + (size_t)j * in;
        float acc = 0.0f;
        for (size_t p = 0; p < in; p++) acc += x[p] * wr[p];
        y[j] = acc;
    }
}

static void rmsnorm(const float *x, const float *w, size_t n, float eps, float *y) {
    float sum_sq = 0.0f;
    for (size_t i = 0; i < n; i++) sum_sq += x[i] * x[i];
    float rms = sqrtf(sum_sq / (float)n + eps);
    for (size_t i = 0; i < n; i++) y[i] = (x[i] / rms) * w[i];
}

static void rope(float *x, int heads, int d, int pos, float theta) {
    int half = d / 2;
    for (int h = 0; h < heads; h++) {
        float *xh = x + (size_t)h * d;
        for (int i = 0; i < half; i++) {
            float inv_freq = 1.0f / powf(theta, 2.0f * (float)i / (float)d);
            float angle = (float)pos * inv_freq;
            float c = cosf(angle), s = sinf(angle);
            float x1 = xh[i], x2 = xh[i + half];
            xh[i] = x1 * c - x2 * s;
            xh[i + half] = x1 * s + x2 * c;
        }
    }
}

/* One token at position `pos` (0-based; the cache must hold positions < pos).
 * Writes vocab logits to `logits` when non-NULL and returns the greedy token. */
AXO_API int axo_model_forward(axo_model *m, int token, int pos, float *logits) {
    const axo_model_config *c = &m->cfg;
    size_t H = (size_t)c->hidden_size, I = (size_t)c->intermediate_size;
    int d = c->head_dim, nh = c->num_heads, nkv = c->num_kv_heads;
    size_t qd = (size_t)nh * d, kd = (size_t)nkv * d;
    int group = nh / nkv;
    if (token < 0 || token >= c->vocab_size || pos < 0 || pos >= c->max_seq_len) return -1;
    if (m->emb32) memcpy(m->h, m->emb32 + (size_t)token * H, H * sizeof(float));
    else for (size_t i = 0; i < H; i++) m->h[i] = axo_f16_to_f32(m->emb[(size_t)token * H + i]);
    float scale = 1.0f / sqrtf((float)d);
    for (int l = 0; l < c->num_layers; l++) {
        axo_layer *L = &m->layers[l];
        rmsnorm(m->h, L->norm[0], H, c->rms_norm_eps, m->xn);
        matvec(L->lin[AXO_LIN_Q], m->xn, qd, H, m->q);
        matvec(L->lin[AXO_LIN_K], m->xn, kd, H, m->k);
        matvec(L->lin[AXO_LIN_V], m->xn, kd, H, m->v);
        rope(m->q, nh, d, pos, c->rope_theta);
        rope(m->k, nkv, d, pos, c->rope_theta);
        for (int kh = 0; kh < nkv; kh++)
            for (int i = 0; i < d; i++) {
                size_t idx = ((size_t)kh * c->max_seq_len + (size_t)pos) * d + i;
                L->kc[idx] = axo_f32_to_f16(m->k[(size_t)kh * d + i]);
                L->vc[idx] = axo_f32_to_f16(m->v[(size_t)kh * d + i]);
            }
        for (int h = 0; h < nh; h++) {
            int kh = h / group;
            const float *qh = m->q + (size_t)h * d;
            float mx = -INFINITY;
            const int j0 = (c->sliding_window > 0 && pos + 1 > c->sliding_window) ? pos + 1 - c->sliding_window : 0;
            for (int j = j0; j <= pos; j++) {
                const uint16_t *kr = L->kc + ((size_t)kh * c->max_seq_len + (size_t)j) * d;
                float s = 0.0f;
                for (int i = 0; i < d; i++) s += qh[i] * axo_f16_to_f32(kr[i]);
                s *= scale;
                m->scores[j] = s;
                if (s > mx) mx = s;
            }
            float sum = 0.0f;
            for (int j = j0; j <= pos; j++) {
                m->scores[j] = expf(m->scores[j] - mx);
                sum += m->scores[j];
            }
            float *oh = m->att + (size_t)h * d;
            for (int i = 0; i < d; i++) oh[i] = 0.0f;
            for (int j = j0; j <= pos; j++) {
                const uint16_t *vr = L->vc + ((size_t)kh * c->max_seq_len + (size_t)j) * d;
                float p = m->scores[j] / sum;
                for (int i = 0; i < d; i++) oh[i] += p * axo_f16_to_f32(vr[i]);
            }
        }
        matvec(L->lin[AXO_LIN_O], m->att, H, qd, m->o);
        for (size_t i = 0; i < H; i++) m->h[i] += m->o[i];
        rmsnorm(m->h, L->norm[1], H, c->rms_norm_eps, m->xn);
        matvec(L->lin[AXO_LIN_GATE], m->xn, I, H, m->g);
        matvec(L->lin[AXO_LIN_UP], m->xn, I, H, m->u);
        for (size_t i = 0; i < I; i++) {
            float gx = m->g[i];
            float silu = gx * (1.0f / (1.0f + expf(-gx)));
            m->g[i] = silu * m->u[i];
        }
        matvec(L->lin[AXO_LIN_DOWN], m->g, H, I, m->o);
        for (size_t i = 0; i < H; i++) m->h[i] += m->o[i];
    }
    rmsnorm(m->h, m->final_norm, H, c->rms_norm_eps, m->xn);
    float *lg = logits ? logits : (float *)malloc((size_t)c->vocab_size * sizeof(float));
    matvec(m->head, m->xn, (size_t)c->vocab_size, H, lg);
    int best = 0;
    float bv = -INFINITY;
    for (int i = 0; i < c->vocab_size; i++)
        if (lg[i] >= bv) { /* >= : the last of equal maxima wins */
            bv = lg[i];
            best = i;
        }
    if (!logits) free(lg);
    return best;
}

/* f16 cache of a layer, [kv_heads][max_seq][head_dim]; which = 0 keys (after RoPE), 1 values. */
AXO_API const uint16_t *axo_model_kv(const axo_model *m, int layer, int which) {
    return which ? m->layers[layer].vc : m->layers[layer].kc;
}

/* Hidden state after the last forward (for intermediate checks). */
AXO_API const float *axo_model_hidden(const axo_model *m) { return m->h; }
