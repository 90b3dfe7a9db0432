/* Sanitizer run of the CPU oracle (TEST INFRASTRUCTURE, like everything under oracle/).
 *
 * `make -C oracle asan` compiles the oracle's sources together with this driver under
 * -fsanitize=address,undefined and runs it: every codec on whole, tail and odd-length inputs (the cases where
 * the reference pads or truncates, quantize.rs:84-111, 163-205, dequantize.rs:44-50), the matmul composition,
 * a small decode model over its whole cache, the sampler and the GGUF block conversion.  A finding aborts
 * the run (-fno-sanitize-recover); the exit status is 0 and the last line "asan driver: ok" otherwise. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

typedef struct axo_model axo_model;
typedef struct {
    int32_t vocab_size, hidden_size, intermediate_size, num_layers;
    int32_t num_heads, num_kv_heads, head_dim, max_seq_len;
    float rms_norm_eps, rope_theta;
    int32_t sliding_window;
} axo_model_config;
typedef struct {
    float temperature;
    int32_t top_k;
    float top_p;
    float repetition_penalty;
    int32_t do_sample;
} axo_sampling_config;

size_t axo_packed_bytes(int type, size_t numel);
size_t axo_bytes_per_block(int type);
int axo_quantize(int type, const float *x, size_t numel, uint8_t *out);
int axo_dequantize(int type, const uint8_t *packed, size_t numel, float *out);
int axo_matmul_ref(int type, const uint8_t *wq, const float *x, const float *bias, size_t M, size_t N, size_t K, float *y, float *scratch);
void axo_matmul_f64(const float *w, const float *x, const float *bias, size_t M, size_t N, size_t K, double *y);
axo_model *axo_model_create(const axo_model_config *cfg);
void axo_model_free(axo_model *m);
int axo_model_set_embedding_f16(axo_model *m, const uint16_t *table);
int axo_model_set_norm(axo_model *m, int layer, int which, const float *w);
int axo_model_set_linear(axo_model *m, int layer, int which, int type, const uint8_t *packed);
int axo_model_forward(axo_model *m, int token, int pos, float *logits);
uint16_t axo_f32_to_f16(float f);
int axo_gguf_convert(int type, const uint8_t *src, uint8_t *dst, size_t nblocks, size_t block_bytes, int to_gguf);
int axo_ggml_dequantize(int type, const uint8_t *blocks, size_t nblocks, float *dst);
int axo_get_next_token(float *logits, int n, const int32_t *generated, int n_generated, const axo_sampling_config *c, float u);

enum { Q8_0, Q4_0, Q4_1, Q5_0, Q5_1, F16, F32, Q4_K, Q6_K, Q5_K };

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static float rnd(void) { /* uniform in (-1, 1) */
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 7;
    rng_state ^= rng_state << 17;
    return (float)((double)(rng_state >> 11) / 9007199254740992.0 * 2.0 - 1.0);
}

/* exactly-sized heap buffers, so that one byte past either end is a finding */
static void *exact(size_t bytes) {
    void *p = malloc(bytes ? bytes : 1);
    if (!p) { fprintf(stderr, "asan driver: out of memory\n"); exit(2); }
    return p;
}

static void codecs(void) {
    static const size_t sizes[] = {1, 2, 31, 32, 33, 35, 40, 63, 255, 256, 257, 300, 1000, 4096};
    for (int t = Q8_0; t <= Q5_K; t++) {
        for (size_t si = 0; si < sizeof sizes / sizeof sizes[0]; si++) {
            const size_t n = sizes[si], nb = axo_packed_bytes(t, n);
            float *x = exact(n * sizeof(float)), *y = exact(n * sizeof(float));
            uint8_t *p = exact(nb);
            for (size_t i = 0; i < n; i++) x[i] = rnd() * (i % 97 == 0 ? 0.5f : 0.02f);
            if (axo_quantize(t, x, n, p) || axo_dequantize(t, p, n, y)) { fprintf(stderr, "codec %d n=%zu failed\n", t, n); exit(1); }
            for (size_t i = 0; i < n; i++)
                if (!isfinite(y[i])) { fprintf(stderr, "codec %d n=%zu: element %zu not finite\n", t, n, i); exit(1); }
            free(x); free(y); free(p);
        }
    }
    printf("asan driver: codecs ok\n");
}

static void matmul(void) {
    for (int t = Q8_0; t <= Q5_K; t++) {
        const size_t M = 3, N = 37, K = 512;
        float *w = exact(N * K * sizeof(float)), *x = exact(M * K * sizeof(float)), *b = exact(N * sizeof(float));
        float *y = exact(M * N * sizeof(float)), *scratch = exact(2 * N * K * sizeof(float)), *deq = exact(N * K * sizeof(float));
        double *y64 = exact(M * N * sizeof(double));
        uint8_t *p = exact(axo_packed_bytes(t, N * K));
        for (size_t i = 0; i < N * K; i++) w[i] = rnd() * 0.05f;
        for (size_t i = 0; i < M * K; i++) x[i] = rnd();
        for (size_t i = 0; i < N; i++) b[i] = rnd();
        if (axo_quantize(t, w, N * K, p) || axo_matmul_ref(t, p, x, b, M, N, K, y, scratch) || axo_dequantize(t, p, N * K, deq)) {
            fprintf(stderr, "matmul %d failed\n", t);
            exit(1);
        }
        axo_matmul_f64(deq, x, b, M, N, K, y64);
        double worst = 0, top = 0;
        for (size_t i = 0; i < M * N; i++) top = fmax(top, fabs(y64[i]));
        for (size_t i = 0; i < M * N; i++) worst = fmax(worst, fabs((double)y[i] - y64[i]) / fmax(fabs(y64[i]), 1e-2 * top));
        if (worst > 1e-3) { fprintf(stderr, "matmul %d: f32 result %g away from the float64 product\n", t, worst); exit(1); }
        free(w); free(x); free(b); free(y); free(scratch); free(deq); free(y64); free(p);
    }
    printf("asan driver: matmul ok\n");
}

static void decode(void) {
    axo_model_config c = {96, 256, 512, 2, 4, 2, 64, 12, 1e-5f, 10000.0f, 5};
    axo_model *m = axo_model_create(&c);
    if (!m) { fprintf(stderr, "model\n"); exit(1); }
    uint16_t *emb = exact((size_t)c.vocab_size * c.hidden_size * 2);
    for (size_t i = 0; i < (size_t)c.vocab_size * c.hidden_size; i++) emb[i] = axo_f32_to_f16(rnd() * 0.7f);
    axo_model_set_embedding_f16(m, emb);
    const size_t qd = (size_t)c.num_heads * c.head_dim, kd = (size_t)c.num_kv_heads * c.head_dim, H = c.hidden_size, I = c.intermediate_size;
    const size_t dims[7][2] = {{qd, H}, {kd, H}, {kd, H}, {H, qd}, {I, H}, {I, H}, {H, I}};
    for (int l = -1; l < c.num_layers; l++) {
        for (int which = 0; which < (l < 0 ? 1 : 7); which++) {
            const size_t n = l < 0 ? (size_t)c.vocab_size : dims[which][0], k = l < 0 ? H : dims[which][1];
            float *w = exact(n * k * sizeof(float));
            uint8_t *p = exact(axo_packed_bytes(Q4_K, n * k));
            for (size_t i = 0; i < n * k; i++) w[i] = rnd() * 0.06f;
            if (axo_quantize(Q4_K, w, n * k, p) || axo_model_set_linear(m, l, which, Q4_K, p)) { fprintf(stderr, "linear %d %d\n", l, which); exit(1); }
            free(w); free(p);
        }
    }
    float *logits = exact((size_t)c.vocab_size * sizeof(float));
    int tok = 3;
    for (int pos = 0; pos < c.max_seq_len; pos++) { /* the whole cache, the sliding window included */
        tok = axo_model_forward(m, tok, pos, logits);
        if (tok < 0 || tok >= c.vocab_size) { fprintf(stderr, "forward at %d: %d\n", pos, tok); exit(1); }
    }
    if (axo_model_forward(m, tok, c.max_seq_len, logits) >= 0) { fprintf(stderr, "a position past the cache was accepted\n"); exit(1); }
    free(logits); free(emb);
    axo_model_free(m);
    printf("asan driver: decode ok\n");
}

static void sampler(void) {
    const int n = 1000;
    float *logits = exact(n * sizeof(float));
    int32_t gen[5] = {1, 7, 7, 999, 0};
    const axo_sampling_config cfgs[] = {{1.0f, 0, -1.0f, 1.0f, 0}, {0.8f, 40, 0.9f, 1.1f, 1}, {0.5f, 1, -1.0f, 1.3f, 1}, {1.5f, 0, 0.5f, 1.0f, 1},
                                        {1.0f, 5000, 1.0f, 1.0f, 1}};
    for (size_t ci = 0; ci < sizeof cfgs / sizeof cfgs[0]; ci++) {
        for (int rep = 0; rep < 4; rep++) {
            for (int i = 0; i < n; i++) logits[i] = rnd() * 4.0f;
            const int tok = axo_get_next_token(logits, n, gen, 5, &cfgs[ci], 0.25f * (float)rep + 0.1f);
            if (tok < 0 || tok >= n) { fprintf(stderr, "sampler config %zu: token %d\n", ci, tok); exit(1); }
        }
    }
    free(logits);
    printf("asan driver: sampler ok\n");
}

static void gguf(void) {
    for (int t = Q8_0; t <= Q5_K; t++) {
        if (t == F16 || t == F32) continue;
        const size_t nb = 9, bb = axo_bytes_per_block(t), total = nb * bb;
        uint8_t *a = exact(total), *b = exact(total), *c = exact(total);
        for (size_t i = 0; i < total; i++) a[i] = (uint8_t)(rng_state >> (8 * (i % 7))), rnd();
        if (axo_gguf_convert(t, a, b, nb, bb, 1) || axo_gguf_convert(t, b, c, nb, bb, 0) || memcmp(a, c, total)) {
            fprintf(stderr, "gguf conversion of type %d is not its own inverse\n", t);
            exit(1);
        }
        if (t == Q4_0 || t == Q4_1) {
            float *d = exact(nb * 32 * sizeof(float));
            for (size_t i = 0; i < nb; i++) { b[i * bb] = 0x00; b[i * bb + 1] = 0x38; if (t == Q4_1) { b[i * bb + 2] = 0x00; b[i * bb + 3] = 0x3C; } }
            if (axo_ggml_dequantize(t, b, nb, d)) { fprintf(stderr, "ggml dequantize %d\n", t); exit(1); }
            free(d);
        }
        free(a); free(b); free(c);
    }
    printf("asan driver: gguf ok\n");
}

int main(void) {
    codecs();
    matmul();
    decode();
    sampler();
    gguf();
    printf("asan driver: ok\n");
    return 0;
}
