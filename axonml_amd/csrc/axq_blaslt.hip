// Plain f16 GEMMs of the large prefill shapes on the vendor's GEMM library (hipBLASLt).
//
// A quantised weight that meets many activation rows is expanded once per call into two f16 planes
// (axq_gemm.hip), laid side by side, and multiplied with the row-scaled f16 activations (each row twice) by one
// library GEMM that accumulates in f32.  The library is opened at first use (dlopen) and is not needed to load this one: where it
// cannot be opened, or has no kernel for a shape, the caller stays on its own fused kernel.
#include <dlfcn.h>

#include <mutex>
#include <hipblaslt/hipblaslt.h>

#include "axq_internal.h"

namespace {

struct LtApi {
    void *lib = nullptr;
    bool tried = false, ok = false;
    decltype(&hipblasLtCreate) create = nullptr;
    decltype(&hipblasLtDestroy) destroy = nullptr;
    decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
    decltype(&hipblasLtMatrixLayoutDestroy) layout_destroy = nullptr;
    decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
    decltype(&hipblasLtMatmulDescDestroy) desc_destroy = nullptr;
    decltype(&hipblasLtMatmulDescSetAttribute) desc_set = nullptr;
    decltype(&hipblasLtMatmulPreferenceCreate) pref_create = nullptr;
    decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy = nullptr;
    decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set = nullptr;
    decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
    decltype(&hipblasLtMatmul) matmul = nullptr;
};

LtApi g_api;

template <class F>
bool sym(F &f, const char *name) {
    f = reinterpret_cast<F>(dlsym(g_api.lib, name));
    return f != nullptr;
}

// Contexts are independent of each other and may meet here from different threads: the library is opened once.
std::once_flag g_api_once;

void open_api_once() {
    g_api.tried = true;
    g_api.lib = dlopen("libhipblaslt.so.1", RTLD_NOW | RTLD_LOCAL);
    if (!g_api.lib) g_api.lib = dlopen("libhipblaslt.so", RTLD_NOW | RTLD_LOCAL);
    if (!g_api.lib) return;
    g_api.ok = sym(g_api.create, "hipblasLtCreate") && sym(g_api.destroy, "hipblasLtDestroy") &&
               sym(g_api.layout_create, "hipblasLtMatrixLayoutCreate") && sym(g_api.layout_destroy, "hipblasLtMatrixLayoutDestroy") &&
               sym(g_api.desc_create, "hipblasLtMatmulDescCreate") && sym(g_api.desc_destroy, "hipblasLtMatmulDescDestroy") &&
               sym(g_api.desc_set, "hipblasLtMatmulDescSetAttribute") && sym(g_api.pref_create, "hipblasLtMatmulPreferenceCreate") &&
               sym(g_api.pref_destroy, "hipblasLtMatmulPreferenceDestroy") && sym(g_api.pref_set, "hipblasLtMatmulPreferenceSetAttribute") &&
               sym(g_api.heuristic, "hipblasLtMatmulAlgoGetHeuristic") && sym(g_api.matmul, "hipblasLtMatmul");
}

bool open_api() {
    std::call_once(g_api_once, open_api_once);
    return g_api.ok;
}

constexpr size_t WORKSPACE_BYTES = 64u << 20;
constexpr int PLAN_SLOTS = 64;
constexpr int CHOICE_SLOTS = 256;
constexpr int ROW_BUCKET = 128; // row counts that round up to the same multiple share a tuned choice

// One (rows, n, k) shape: layouts and the algorithm the library's heuristic picked.
constexpr int CANDIDATES = 8;

struct LtPlan {
    int m = 0, n = 0, k = 0, ldw = 0, ldx = 0;
    bool usable = false, tuned = false;
    hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr;
    hipblasLtMatmulHeuristicResult_t heur[CANDIDATES]; // the library's candidates, best guess first
    int n_heur = 0, best = 0;
};

// Which of the library's candidates won for a shape; kept per bucket of row counts, so that prompts of every length do
// not each pay for a tuning run (the candidate lists of neighbouring row counts are the same in practice).
struct LtChoice {
    int bucket = 0, n = 0, k = 0, ldw = 0, ldx = 0, best = 0;
};

struct LtState {
    LtChoice choices[CHOICE_SLOTS];
    int n_choices = 0;
    hipblasLtHandle_t handle = nullptr;
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatmulPreference_t pref = nullptr;
    void *workspace = nullptr;
    hipEvent_t t0 = nullptr, t1 = nullptr; // for timing candidates (the context's own pair may be in use by the caller)
    LtPlan plans[PLAN_SLOTS];
    int n_plans = 0;
    bool failed = false;
};

void drop_plan(LtPlan &p) {
    if (p.la) (void)g_api.layout_destroy(p.la);
    if (p.lb) (void)g_api.layout_destroy(p.lb);
    if (p.lc) (void)g_api.layout_destroy(p.lc);
    p = LtPlan();
}

LtState *state_of(axq_ctx *ctx) {
    if (ctx->blaslt) return reinterpret_cast<LtState *>(ctx->blaslt);
    if (!open_api()) return nullptr;
    LtState *s = new LtState();
    ctx->blaslt = s;
    const hipblasOperation_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
    const uint64_t ws = WORKSPACE_BYTES;
    if (g_api.create(&s->handle) != HIPBLAS_STATUS_SUCCESS || g_api.desc_create(&s->desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS ||
        g_api.desc_set(s->desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof op_t) != HIPBLAS_STATUS_SUCCESS ||
        g_api.desc_set(s->desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof op_n) != HIPBLAS_STATUS_SUCCESS ||
        g_api.pref_create(&s->pref) != HIPBLAS_STATUS_SUCCESS ||
        g_api.pref_set(s->pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof ws) != HIPBLAS_STATUS_SUCCESS ||
        hipMalloc(&s->workspace, WORKSPACE_BYTES) != hipSuccess || hipEventCreate(&s->t0) != hipSuccess ||
        hipEventCreate(&s->t1) != hipSuccess) {
        (void)hipGetLastError();
        s->failed = true;
    }
    return s;
}

// In the library's column-major terms: D[n, m] = W[k, n]^T X[k, m], leading dimensions ldw, ldx and n, which is
// y[m, n] = x[m, k] W[n, k]^T on row-major arrays whose rows are ldx and ldw elements apart.
LtPlan *plan_for(LtState *s, int m, int n, int k, int ldw, int ldx) {
    for (int i = 0; i < s->n_plans; i++)
        if (s->plans[i].m == m && s->plans[i].n == n && s->plans[i].k == k && s->plans[i].ldw == ldw && s->plans[i].ldx == ldx)
            return &s->plans[i];
    if (s->n_plans == PLAN_SLOTS) { // forget the oldest
        drop_plan(s->plans[0]);
        for (int i = 1; i < PLAN_SLOTS; i++) s->plans[i - 1] = s->plans[i];
        s->plans[PLAN_SLOTS - 1] = LtPlan();
        s->n_plans--;
    }
    LtPlan &p = s->plans[s->n_plans++];
    p.m = m; p.n = n; p.k = k; p.ldw = ldw; p.ldx = ldx;
    int found = 0;
    if (g_api.layout_create(&p.la, HIP_R_16F, (uint64_t)k, (uint64_t)n, ldw) == HIPBLAS_STATUS_SUCCESS &&
        g_api.layout_create(&p.lb, HIP_R_16F, (uint64_t)k, (uint64_t)m, ldx) == HIPBLAS_STATUS_SUCCESS &&
        g_api.layout_create(&p.lc, HIP_R_32F, (uint64_t)n, (uint64_t)m, n) == HIPBLAS_STATUS_SUCCESS &&
        g_api.heuristic(s->handle, s->desc, p.la, p.lb, p.lc, p.lc, s->pref, CANDIDATES, p.heur, &found) == HIPBLAS_STATUS_SUCCESS) {
        for (int i = 0; i < found; i++) // keep the ones that fit the workspace, in the library's order
            if (p.heur[i].workspaceSize <= WORKSPACE_BYTES) p.heur[p.n_heur++] = p.heur[i];
        p.usable = p.n_heur > 0;
    }
    const int bucket = (m + ROW_BUCKET - 1) / ROW_BUCKET;
    for (int i = 0; i < s->n_choices && p.usable; i++) {
        const LtChoice &c = s->choices[i];
        if (c.bucket == bucket && c.n == n && c.k == k && c.ldw == ldw && c.ldx == ldx) {
            p.best = c.best < p.n_heur ? c.best : 0;
            p.tuned = true;
            break;
        }
    }
    return &p;
}

} // namespace

namespace {

// First use of a shape: the library's first guess is not always its fastest kernel (at 2048 x 4096 x 8192 by a
// quarter), so every candidate runs four times on the real operands, overwriting y, and the one with the quickest run
// stays.  Returns whether a candidate ran (the product is then in y).
bool tune(axq_ctx *ctx, LtState *s, LtPlan *p, const _Float16 *w, const _Float16 *x, float *y) {
    const float one = 1.0f, zero = 0.0f;
    auto run = [&](int i) {
        return g_api.matmul(s->handle, s->desc, &one, w, p->la, x, p->lb, &zero, y, p->lc, y, p->lc, &p->heur[i].algo, s->workspace,
                            WORKSPACE_BYTES, ctx->stream);
    };
    p->tuned = true;
    float best_ms = 0.f;
    bool have = false;
    for (int i = 0; i < p->n_heur; i++) {
        if (run(i) != HIPBLAS_STATUS_SUCCESS) continue; // warm-up
        float fastest = 0.f;
        bool timed = false;
        for (int rep = 0; rep < 3; rep++) {
            float ms = 0.f;
            if (hipEventRecord(s->t0, ctx->stream) != hipSuccess || run(i) != HIPBLAS_STATUS_SUCCESS ||
                hipEventRecord(s->t1, ctx->stream) != hipSuccess || hipEventSynchronize(s->t1) != hipSuccess ||
                hipEventElapsedTime(&ms, s->t0, s->t1) != hipSuccess) {
                (void)hipGetLastError();
                timed = false;
                break;
            }
            if (!timed || ms < fastest) fastest = ms;
            timed = true;
        }
        if (timed && (!have || fastest < best_ms)) { have = true; best_ms = fastest; p->best = i; }
    }
    if (!have) p->usable = false;
    if (have && s->n_choices < CHOICE_SLOTS) {
        LtChoice &c = s->choices[s->n_choices++];
        c.bucket = (p->m + ROW_BUCKET - 1) / ROW_BUCKET; c.n = p->n; c.k = p->k; c.ldw = p->ldw; c.ldx = p->ldx; c.best = p->best;
    }
    return have;
}

} // namespace

// y[m, n] (f32, row-major, rows n apart) = x[m, k] w[n, k]^T (+ y when `accumulate`), both operands f16 in device memory
// with rows ldx and ldw elements apart.  Returns 1 when the GEMM was enqueued on the context's stream, 0 when the library
// is not there or has no kernel for the shape (nothing that matters was enqueued), a negative status when the launch
// failed.  A shape met for the first time is tuned on the way (not when accumulating, which must run exactly once:
// axq_blaslt_tune_f16 in front of such a call does it).
int axq_blaslt_gemm_f16(axq_ctx *ctx, const _Float16 *w, int ldw, const _Float16 *x, int ldx, int m, int n, int k, bool accumulate, float *y) {
    LtState *s = state_of(ctx);
    if (!s || s->failed) return 0;
    LtPlan *p = plan_for(s, m, n, k, ldw, ldx);
    if (!p->usable) return 0;
    if (!p->tuned && !accumulate) return tune(ctx, s, p, w, x, y) ? 1 : 0;
    const float one = 1.0f, zero = 0.0f;
    const hipblasStatus_t st = g_api.matmul(s->handle, s->desc, &one, w, p->la, x, p->lb, accumulate ? &one : &zero, y, p->lc, y, p->lc,
                                            &p->heur[p->tuned ? p->best : 0].algo, s->workspace, WORKSPACE_BYTES, ctx->stream);
    if (st != HIPBLAS_STATUS_SUCCESS) return axq_fail(ctx, AXQ_ERR_BLAS, "hipblasLtMatmul: status %d", (int)st);
    return 1;
}

// Tunes the shape if it has not been met yet (y is overwritten then); 1 = the shape can run, 0 = it cannot.
int axq_blaslt_tune_f16(axq_ctx *ctx, const _Float16 *w, int ldw, const _Float16 *x, int ldx, int m, int n, int k, float *y) {
    LtState *s = state_of(ctx);
    if (!s || s->failed) return 0;
    LtPlan *p = plan_for(s, m, n, k, ldw, ldx);
    if (!p->usable) return 0;
    if (!p->tuned) return tune(ctx, s, p, w, x, y) ? 1 : 0;
    return 1;
}

void axq_blaslt_release(axq_ctx *ctx) {
    if (!ctx->blaslt) return;
    LtState *s = reinterpret_cast<LtState *>(ctx->blaslt);
    for (int i = 0; i < s->n_plans; i++) drop_plan(s->plans[i]);
    if (s->pref) (void)g_api.pref_destroy(s->pref);
    if (s->desc) (void)g_api.desc_destroy(s->desc);
    if (s->handle) (void)g_api.destroy(s->handle);
    if (s->workspace) (void)hipFree(s->workspace);
    if (s->t0) (void)hipEventDestroy(s->t0);
    if (s->t1) (void)hipEventDestroy(s->t1);
    delete s;
    ctx->blaslt = nullptr;
}
