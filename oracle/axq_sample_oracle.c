/*
 * CPU oracle for next-token selection.  TEST INFRASTRUCTURE ONLY (see axq_oracle.c).
 *
 * Restates TextGenerator of crates/axonml-llm/src/generation.rs, statement by statement, in f32:
 *   apply_repetition_penalty :145-158   (once per occurrence in `generated`)
 *   apply_temperature        :136-142
 *   apply_top_k              :161-180   (stable descending sort: among equal logits the lower index ranks first)
 *   apply_top_p              :183-214   (softmax with sequential f32 sums, stable descending sort, cumsum > p)
 *   sample                   :217-245   (softmax, sequential cumsum, first i with u < cumsum; last token otherwise)
 *   argmax                   :248-255   (Iterator::max_by: the last of equal maxima)
 *   get_next_token           :258-269
 * The reference draws `u` from rand::thread_rng (third party, not reproducible); here it is an argument.
 * f32::exp is libm's expf.
 *
 * Pin status: pinned by the reference's own test vectors (generation.rs:421-467: top-k keeps two of
 * [1,5,3,4,2]; temperature 2 turns [2,4,6] into [1,2,3]; argmax of [1,5,3,4,2] is 1; penalty 2 lowers
 * logits 1 and 3 of [1,2,3,4]) and by hand-computed cases in tests/test_sampling.py (ties, the element
 * that crosses p is kept, draw boundaries, repeated ids compounding the penalty).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define AXO_API __attribute__((visibility("default")))

typedef struct {
    float temperature;
    int32_t top_k;  /* 0 = None */
    float top_p;    /* negative = None */
    float repetition_penalty;
    int32_t do_sample;
} axo_sampling_config;

static const float *g_sort_vals;
/* descending by value; equal values keep their index order (what a stable sort leaves) */
static int cmp_desc(const void *pa, const void *pb) {
    const int a = *(const int *)pa, b = *(const int *)pb;
    if (g_sort_vals[b] < g_sort_vals[a]) return -1;
    if (g_sort_vals[b] > g_sort_vals[a]) return 1;
    return a < b ? -1 : (a > b);
}

static void softmax_seq(const float *logits, int n, float *probs) {
    float mx = -INFINITY;
    for (int i = 0; i < n; i++) mx = fmaxf(mx, logits[i]); /* fold(NEG_INFINITY, f32::max) */
    float sum = 0.0f;
    for (int i = 0; i < n; i++) { probs[i] = expf(logits[i] - mx); sum += probs[i]; }
    for (int i = 0; i < n; i++) probs[i] = probs[i] / sum;
}

/* logits: n values, modified in place into the filtered logits; returns the token. */
AXO_API int axo_get_next_token(float *logits, int n, const int32_t *generated, int n_generated, const axo_sampling_config *c,
                               float u) {
    int *idx = (int *)malloc(sizeof(int) * (size_t)n);
    float *probs = (float *)malloc(sizeof(float) * (size_t)n);
    char *keep = (char *)malloc((size_t)n);
    if (c->repetition_penalty != 1.0f)
        for (int g = 0; g < n_generated; g++) {
            const int t = generated[g];
            if (t >= 0 && t < n) {
                if (logits[t] > 0.0f) logits[t] /= c->repetition_penalty;
                else logits[t] *= c->repetition_penalty;
            }
        }
    if (c->temperature != 1.0f)
        for (int i = 0; i < n; i++) logits[i] /= c->temperature;
    if (c->top_k > 0 && c->top_k < n) {
        for (int i = 0; i < n; i++) idx[i] = i;
        g_sort_vals = logits;
        qsort(idx, (size_t)n, sizeof(int), cmp_desc);
        memset(keep, 0, (size_t)n);
        for (int i = 0; i < c->top_k; i++) keep[idx[i]] = 1;
        for (int i = 0; i < n; i++) if (!keep[i]) logits[i] = -INFINITY;
    }
    if (c->top_p >= 0.0f) {
        softmax_seq(logits, n, probs);
        for (int i = 0; i < n; i++) idx[i] = i;
        g_sort_vals = probs;
        qsort(idx, (size_t)n, sizeof(int), cmp_desc);
        float cumsum = 0.0f;
        int cutoff = n;
        for (int i = 0; i < n; i++) {
            cumsum += probs[idx[i]];
            if (cumsum > c->top_p) { cutoff = i + 1; break; }
        }
        memset(keep, 0, (size_t)n);
        for (int i = 0; i < cutoff; i++) keep[idx[i]] = 1;
        for (int i = 0; i < n; i++) if (!keep[i]) logits[i] = -INFINITY;
    }
    int token;
    if (!c->do_sample) {
        token = 0;
        for (int i = 1; i < n; i++) if (!(logits[i] < logits[token])) token = i; /* max_by keeps the last maximum */
    } else {
        softmax_seq(logits, n, probs);
        float cumsum = 0.0f;
        token = n - 1;
        for (int i = 0; i < n; i++) {
            cumsum += probs[i];
            if (u < cumsum) { token = i; break; }
        }
    }
    free(idx); free(probs); free(keep);
    return token;
}
