// Next-token selection on the device: TextGenerator::get_next_token
// (crates/axonml-llm/src/generation.rs:258-269) = repetition penalty (:145-158), temperature (:136-142),
// top-k (:161-180), top-p (:183-214), then sample (:217-245) or argmax (:248-255).
//
// One workgroup of 1024 threads works on a copy of the logits in device memory.  The reference sorts the
// vocabulary twice; here "the k largest" and "the smallest head of the sorted probabilities whose sum exceeds
// p" are found by a three-pass radix selection over the bit patterns (11 + 11 + 10 bits), with counts for
// top-k and with probability mass in 2^-40 fixed point for top-p, so that every sum is exact and independent
// of the order in which the threads add.  Ties are resolved as the reference's stable sort does: lower
// indices first.  Penalty, temperature and top-k reproduce the reference bit for bit.  The softmax sums of
// top-p and of the final draw are exact here where the reference adds 32-bit floats one after the other, so
// a decision can differ from the reference's when the cumulative probability comes within about 1e-5 of the
// threshold (p, or the uniform variate).
#include "axq_internal.h"

namespace {

typedef unsigned long long u64;
constexpr int ST = 1024;          // threads
constexpr int BINS = 2048;
constexpr float FX = 1099511627776.0f; // 2^40

struct SampleArgs {
    const float *logits;
    float *work;          // scratch in device memory: two padded copies of the vocabulary (see axq_sample_scratch_bytes)
    int vocab;
    const int32_t *hist;  // tokens the repetition penalty looks at
    const int32_t *hist_len_dev; // their number, on the device (NULL: hist_len)
    int hist_len;
    float temperature, top_p, penalty;
    int top_k, do_sample;
    float u;                    // uniform variate in [0, 1) ...
    const int32_t *counter_dev; // ... or, when not NULL, drawn from (seed, *counter_dev)
    u64 seed;
    int32_t *out;
    float *filtered_out;        // optional: the logits after all filters
    // one workgroup per row: row r reads logits + r * logits_stride, hist + r * hist_stride, hist_len_dev[r],
    // counter_dev[r], works in work + r * work_stride, draws with seed + r * seed_stride and writes out[r]
    size_t logits_stride, hist_stride, work_stride;
    u64 seed_stride;
};

constexpr int FAST_K = 128;   // top-k up to here takes the short path below ...
constexpr int MAX_CAND = 256; // ... as long as its first cut leaves at most this many candidates

struct Shared {
    u64 hist[BINS];        // radix histogram; the short path keeps its candidate list here afterwards
    uint32_t tk[ST];       // one key per thread (the short path's thread maxima)
    u64 part[17];
    float fpart[16];
    int ipart[16];
    u64 bc_u64[4];
    int bc_i32[4];
    float bc_f32[2];
};

// ascending unsigned order == ascending float order (-inf lowest)
__device__ inline uint32_t order_key(float x) {
    const uint32_t b = __builtin_bit_cast(uint32_t, x);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

__device__ inline u64 wave_incl_scan(u64 v, int lane) {
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const u64 o = __shfl_up(v, d);
        if (lane >= d) v += o;
    }
    return v;
}

// exclusive prefix sums over the threads in thread order; *total = sum over all threads
__device__ inline u64 block_excl_scan(u64 v, Shared &sh, u64 *total) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const u64 inc = wave_incl_scan(v, lane);
    __syncthreads(); // sh.part may still be read from an earlier call
    if (lane == 63) sh.part[wave] = inc;
    __syncthreads();
    if (tid == 0) {
        u64 run = 0;
        for (int w = 0; w < ST / 64; w++) { const u64 t = sh.part[w]; sh.part[w] = run; run += t; }
        sh.part[16] = run;
    }
    __syncthreads();
    *total = sh.part[16];
    return sh.part[wave] + inc - v;
}

__device__ inline float block_max(float v, Shared &sh) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m));
    __syncthreads();
    if (lane == 0) sh.fpart[wave] = v;
    __syncthreads();
    float r = sh.fpart[0];
    for (int w = 1; w < ST / 64; w++) r = fmaxf(r, sh.fpart[w]);
    return r;
}

__device__ inline u64 fx_of(float p) { return (u64)(p * FX); }

// Walks the first nb bins of sh.hist from the top: the bin at which the running weight crosses `remaining`
// (MASS: exceeds it; otherwise: reaches it), and the weight above that bin.  Returns -1 when nothing crosses.
template <bool MASS>
__device__ int find_crossing(int nb, u64 remaining, Shared &sh, u64 *above) {
    const int tid = threadIdx.x;
    // thread t looks at bins nb-1-2t and nb-2-2t (descending); threads past the bins hold nothing
    const int b0 = nb - 1 - 2 * tid, b1 = b0 - 1;
    const u64 w0 = b0 >= 0 ? sh.hist[b0] : 0, w1 = b1 >= 0 ? sh.hist[b1] : 0;
    u64 total;
    const u64 before = block_excl_scan(w0 + w1, sh, &total);
    auto crosses = [&](u64 v) { return MASS ? v > remaining : v >= remaining; };
    if (tid == 0) sh.bc_i32[0] = -1;
    __syncthreads();
    if (!crosses(before) && crosses(before + w0 + w1)) { // exactly one thread
        const bool first = crosses(before + w0);
        sh.bc_i32[0] = first ? b0 : b1;
        sh.bc_u64[0] = first ? before : before + w0;
    }
    __syncthreads();
    const int d = sh.bc_i32[0];
    *above = sh.bc_u64[0];
    __syncthreads();
    return d;
}

// Radix selection over key(i), i < n, walking from the largest key down.
//   MASS = false: weight 1 per element, crossing when the running count reaches `target` (the target-th largest)
//   MASS = true : weight(i), crossing when the running mass exceeds `target`
// Returns false when the whole array does not cross (keep everything).  Otherwise *thr = the key at which the
// crossing happens and *rest = target minus the weight of all keys above it.
template <bool MASS, class KeyFn, class WeightFn>
__device__ bool radix_select(int n, u64 target, KeyFn key, WeightFn weight, Shared &sh, uint32_t *thr, u64 *rest) {
    const int tid = threadIdx.x;
    uint32_t prefix = 0, mask = 0;
    u64 remaining = target;
    const int shifts[3] = {21, 10, 0}, widths[3] = {11, 11, 10};
    for (int pass = 0; pass < 3; pass++) {
        const int shift = shifts[pass], nb = 1 << widths[pass];
        for (int b = tid; b < BINS; b += ST) sh.hist[b] = 0;
        __syncthreads();
#pragma unroll 8
        for (int i = tid; i < n; i += ST) {
            const u64 wt = weight(i); // weightless elements (dropped logits) would all pile onto one bin
            if (wt != 0) {
                const uint32_t k = key(i);
                if ((k & mask) == prefix) atomicAdd(&sh.hist[(k >> shift) & (uint32_t)(nb - 1)], wt);
            }
        }
        __syncthreads();
        u64 above;
        const int d = find_crossing<MASS>(nb, remaining, sh, &above);
        if (d < 0) return false; // the first pass did not cross: less than `target` in total
        remaining -= above;
        prefix |= (uint32_t)d << shift;
        mask |= (uint32_t)(nb - 1) << shift;
    }
    *thr = prefix;
    *rest = remaining;
    return true;
}

// Among the elements with key(i) == thr, in index order, marks all but the first `quota` as dropped; elements
// with a smaller key are dropped, with a larger key kept.  drop(i) does the dropping.
template <class KeyFn, class DropFn>
__device__ void keep_head_of_ties(int n, uint32_t thr, u64 quota, KeyFn key, DropFn drop, Shared &sh) {
    const int tid = threadIdx.x;
    const int chunk = (n + ST - 1) / ST, lo = tid * chunk, hi = lo + chunk < n ? lo + chunk : n;
    u64 mine = 0;
#pragma unroll 8
    for (int i = lo; i < hi; i++) mine += key(i) == thr;
    u64 total;
    u64 rank = block_excl_scan(mine, sh, &total);
    for (int i = lo; i < hi; i++) {
        const uint32_t k = key(i);
        if (k < thr) drop(i);
        else if (k == thr) { if (rank >= quota) drop(i); rank++; }
    }
    __syncthreads();
}

__device__ inline float uniform_from(u64 seed, u64 counter) { // splitmix64 of (seed, counter) -> [0, 1) with 24 bits
    u64 z = seed + 0x9E3779B97F4A7C15ull * (counter + 1);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (float)(z >> 40) * (1.0f / 16777216.0f);
}

// The working copy of the logits lives in LDS when the vocabulary fits (LDS_W), else in device memory.
constexpr int LDS_VOCAB = 32768;
// element i sits at i + i / 32: a thread that walks 32 consecutive elements then strides 33 words across the
// lanes (no LDS bank is hit twice), and consecutive elements stay consecutive for the strided loops
__device__ inline int ix(int i) { return i + (i >> 5); }
__host__ __device__ inline size_t padded_words(int n) { return (size_t)n + (size_t)(n >> 5) + 1; }

template <bool IN_LDS>
__global__ void __launch_bounds__(ST) sample_kernel(SampleArgs a) {
    __shared__ Shared sh;
    extern __shared__ float lds_w[];
    const int tid = threadIdx.x, n = a.vocab;
    if (blockIdx.x) {
        const size_t r = blockIdx.x;
        a.logits += r * a.logits_stride;
        a.work += r * a.work_stride;
        if (a.hist) a.hist += r * a.hist_stride;
        if (a.hist_len_dev) a.hist_len_dev += r;
        if (a.counter_dev) a.counter_dev += r;
        a.seed += r * a.seed_stride;
        a.out += r;
        if (a.filtered_out) a.filtered_out += r * (size_t)n;
    }
    constexpr bool in_lds = IN_LDS;
    float *const w = IN_LDS ? lds_w : a.work; // the working copy of the logits (address space known at compile time)
#pragma unroll 8
    for (int i = tid; i < n; i += ST) w[ix(i)] = a.logits[i];
    __syncthreads();
    // repetition penalty: once per occurrence (a division of a positive logit, a product otherwise).  Repeats
    // of one id apply the same step again, so the order among them does not matter: each occurrence swaps
    // its step in atomically.
    if (a.penalty != 1.0f) {
        const int nh = a.hist_len_dev ? *a.hist_len_dev : a.hist_len;
        for (int h = tid; h < nh; h += ST) {
            const int t = a.hist[h];
            if (t >= 0 && t < n) {
                int *p = reinterpret_cast<int *>(w + ix(t));
                int old = *p, seen;
                do {
                    seen = old;
                    const float v = __builtin_bit_cast(float, seen);
                    const float r = v > 0.0f ? v / a.penalty : v * a.penalty;
                    old = atomicCAS(p, seen, __builtin_bit_cast(int, r));
                } while (old != seen);
            }
        }
        __syncthreads();
    }
    if (a.temperature != 1.0f)
#pragma unroll 8
        for (int i = tid; i < n; i += ST) w[ix(i)] = w[ix(i)] / a.temperature;
    __syncthreads();
    auto wkey = [&](int i) { return order_key(w[ix(i)]); };
    float tmax = -INFINITY; // this thread's maximum over its strided share
#pragma unroll 8
    for (int i = tid; i < n; i += ST) tmax = fmaxf(tmax, w[ix(i)]);
    const float mx = block_max(tmax, sh);
    // Short path for a small top-k (the usual 20 ... 100): the k largest logits lie among the elements that
    // reach the k-th largest of the 1024 thread maxima (each thread's maximum over its strided share), usually
    // little more than k of them.  Those candidates go into a list, one per thread, and everything after that
    // -- exact top-k with ties by index, softmax, top-p, the draw -- works on the list with the same rules and
    // the same exact sums as the long path, in a few loops over at most MAX_CAND entries.
    if (a.top_k > 0 && a.top_k <= FAST_K && a.top_k < n) {
        sh.tk[tid] = order_key(tmax);
        if (tid == 0) sh.bc_i32[2] = 0;
        __syncthreads();
        uint32_t cut;
        u64 unused;
        (void)radix_select<false>(ST, (u64)a.top_k, [&](int i) { return sh.tk[i]; }, [](int) { return (u64)1; }, sh, &cut, &unused);
        uint32_t *ckey = reinterpret_cast<uint32_t *>(sh.hist);
        int *cidx = reinterpret_cast<int *>(ckey + MAX_CAND);
        u64 *cfx = reinterpret_cast<u64 *>(cidx + MAX_CAND);
#pragma unroll 8
        for (int i = tid; i < n; i += ST) {
            const uint32_t k = wkey(i);
            if (k >= cut) {
                const int slot = atomicAdd(&sh.bc_i32[2], 1);
                if (slot < MAX_CAND) { ckey[slot] = k; cidx[slot] = i; }
            }
        }
        __syncthreads();
        const int m = sh.bc_i32[2];
        if (m <= MAX_CAND) { // else: too many ties at the cut; the long path below handles it
            const bool mine = tid < m;
            const uint32_t key = mine ? ckey[tid] : 0;
            const int idx = mine ? cidx[tid] : 0;
            // exact top-k: rank in the reference's stable descending order
            int rank = 0;
            if (mine)
                for (int j = 0; j < m; j++) rank += (ckey[j] > key) || (ckey[j] == key && cidx[j] < idx);
            bool keep = mine && rank < a.top_k;
            const float val = mine ? w[ix(idx)] : -INFINITY;
            float ev = keep ? expf(val - mx) : 0.0f;
            u64 total;
            if (a.top_p >= 0.0f) {
                (void)block_excl_scan(fx_of(ev), sh, &total);
                const float sum = (float)((double)total * (1.0 / 1099511627776.0));
                if (keep) ev = ev / sum; // now a probability; the draw below uses what is left of these
                __syncthreads();
                if (tid < MAX_CAND) ckey[tid] = keep ? __builtin_bit_cast(uint32_t, ev) : 0u;
                __syncthreads();
                // mass of everything that precedes this entry in descending order of probability (ties by index)
                u64 before = 0;
                if (keep)
                    for (int j = 0; j < m; j++) {
                        const uint32_t pj = ckey[j];
                        const uint32_t pt = __builtin_bit_cast(uint32_t, ev);
                        if (pj > pt || (pj == pt && pj != 0 && cidx[j] < idx)) before += fx_of(__builtin_bit_cast(float, pj));
                    }
                const u64 target = (u64)((double)a.top_p * 1099511627776.0);
                if (keep && before > target) { keep = false; ev = 0.0f; } // the entry that crosses p itself stays
                __syncthreads();
            }
            if (a.filtered_out) {
#pragma unroll 8
                for (int i = tid; i < n; i += ST) a.filtered_out[i] = -INFINITY;
                __syncthreads();
                if (keep) a.filtered_out[idx] = val;
            }
            if (!a.do_sample) { // the last of the equal maxima; the maximum is always kept
                int best = (keep && val == mx) ? idx : -1;
#pragma unroll
                for (int s2 = 32; s2 >= 1; s2 >>= 1) { const int o = __shfl_xor(best, s2); best = o > best ? o : best; }
                __syncthreads();
                if ((tid & 63) == 0) sh.ipart[tid >> 6] = best;
                __syncthreads();
                if (tid == 0) {
                    for (int wv = 1; wv < ST / 64; wv++) best = sh.ipart[wv] > best ? sh.ipart[wv] : best;
                    a.out[0] = best < 0 ? 0 : best;
                }
                return;
            }
            // the draw: first entry in index order whose cumulative weight exceeds u times the total
            (void)block_excl_scan(fx_of(ev), sh, &total);
            __syncthreads();
            if (tid < MAX_CAND) cfx[tid] = fx_of(ev);
            __syncthreads();
            const float u = a.counter_dev ? uniform_from(a.seed, (u64)*a.counter_dev) : a.u;
            const u64 target = (u64)((double)u * (double)total);
            u64 before = 0;
            if (keep)
                for (int j = 0; j < m; j++) before += cidx[j] < idx ? cfx[j] : 0;
            if (tid == 0) sh.bc_i32[1] = n - 1; // the reference's fallback: the last token
            __syncthreads();
            if (keep && before <= target && target < before + fx_of(ev)) sh.bc_i32[1] = idx;
            __syncthreads();
            if (tid == 0) a.out[0] = sh.bc_i32[1];
            return;
        }
    }
    // top-k: the k largest stay (ties: lower index first), the rest become -inf
    if (a.top_k > 0 && a.top_k < n) {
        uint32_t thr;
        u64 rest;
        if (radix_select<false>(n, (u64)a.top_k, wkey, [](int) { return (u64)1; }, sh, &thr, &rest))
            keep_head_of_ties(n, thr, rest, wkey, [&](int i) { w[ix(i)] = -INFINITY; }, sh);
    }
    const int chunk = (n + ST - 1) / ST, lo = tid * chunk, hi = lo + chunk < n ? lo + chunk : n;

    // From here on the fast memory holds e_i = exp(w_i - max), computed once (0 for a dropped logit); the
    // logits themselves move to (or stay in) device memory, where only drops and the final read touch them.
    const bool need_e = a.top_p >= 0.0f || a.do_sample;
    float *const e = !need_e ? w : (IN_LDS ? lds_w : a.work + padded_words(n));
    float *const wg = need_e ? a.work : w;
    if (need_e) {
#pragma unroll 8
        for (int i = tid; i < n; i += ST) {
            const float v = w[ix(i)];
            if (in_lds) wg[ix(i)] = v;
            e[ix(i)] = v == -INFINITY ? 0.0f : expf(v - mx);
        }
        __syncthreads();
    }
    // top-p: softmax, then the head of the descending order whose cumulative probability first exceeds p.
    // e_i becomes p_i = e_i / sum in place; the draw below works on the p_i that are left, which is the
    // softmax of the filtered logits up to one common factor.
    if (a.top_p >= 0.0f) {
        u64 mine = 0;
#pragma unroll 8
        for (int i = tid; i < n; i += ST) mine += fx_of(e[ix(i)]);
        u64 total;
        (void)block_excl_scan(mine, sh, &total);
        const float sum = (float)((double)total * (1.0 / 1099511627776.0));
#pragma unroll 8
        for (int i = tid; i < n; i += ST) { const float v = e[ix(i)]; if (v != 0.0f) e[ix(i)] = v / sum; }
        __syncthreads();
        auto pkey = [&](int i) { return __builtin_bit_cast(uint32_t, e[ix(i)]); }; // probabilities are >= 0
        uint32_t thr;
        u64 rest;
        const u64 target = (u64)((double)a.top_p * 1099511627776.0);
        if (radix_select<true>(n, target, pkey, [&](int i) { return fx_of(e[ix(i)]); }, sh, &thr, &rest)) {
            // every tie has the same probability q: the first m of them, m the least with m q > what is missing
            const u64 q = fx_of(__builtin_bit_cast(float, thr));
            const u64 m = q ? rest / q + 1 : 1;
            keep_head_of_ties(n, thr, m, pkey, [&](int i) { e[ix(i)] = 0.0f; wg[ix(i)] = -INFINITY; }, sh);
        }
    }
    if (a.filtered_out) {
#pragma unroll 8
        for (int i = tid; i < n; i += ST) a.filtered_out[i] = wg[ix(i)];
    }
    if (!a.do_sample) {
        // argmax as Iterator::max_by leaves it: the last of equal maxima (the maximum itself is never dropped)
        int best = -1;
#pragma unroll 8
        for (int i = tid; i < n; i += ST) if (wg[ix(i)] == mx) best = i > best ? i : best;
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) { const int o = __shfl_xor(best, m); best = o > best ? o : best; }
        __syncthreads();
        if ((tid & 63) == 0) sh.ipart[tid >> 6] = best;
        __syncthreads();
        if (tid == 0) {
            for (int wv = 1; wv < ST / 64; wv++) best = sh.ipart[wv] > best ? sh.ipart[wv] : best;
            a.out[0] = best < 0 ? 0 : best;
        }
        return;
    }
    // inverse CDF in index order: the first i whose cumulative probability exceeds u.  The softmax of the
    // filtered logits has the same maximum, so its terms are the e_i (or p_i) that are left.
    const float u = a.counter_dev ? uniform_from(a.seed, (u64)*a.counter_dev) : a.u;
    u64 mine = 0;
#pragma unroll 8
    for (int i = lo; i < hi; i++) mine += fx_of(e[ix(i)]);
    u64 total;
    const u64 before = block_excl_scan(mine, sh, &total);
    const u64 target = (u64)((double)u * (double)total);
    if (tid == 0) sh.bc_i32[1] = n - 1; // the reference's fallback: the last token
    __syncthreads();
    if (before <= target && target < before + mine) { // exactly one thread
        u64 run = before;
        for (int i = lo; i < hi; i++) {
            run += fx_of(e[ix(i)]);
            if (run > target) { sh.bc_i32[1] = i; break; }
        }
    }
    __syncthreads();
    if (tid == 0) a.out[0] = sh.bc_i32[1];
}

struct Temp {
    void *p = nullptr;
    ~Temp() { if (p) (void)hipFree(p); }
};

} // namespace

// Enqueues the selection on the context's stream; every pointer is a device pointer.  scratch: axq_sample_scratch_bytes(vocab).
int axq_dev_sample(axq_ctx *ctx, const float *logits, int vocab, const int32_t *hist, const int32_t *hist_len_dev, int hist_len,
                   const axq_sampling_config *cfg, float u, const int32_t *counter_dev, uint64_t seed, void *scratch,
                   int32_t *out, float *filtered_out) {
    return axq_dev_sample_rows(ctx, 1, logits, 0, vocab, hist, 0, hist_len_dev, hist_len, cfg, u, counter_dev, seed, 0, scratch, out,
                               filtered_out);
}

// `rows` independent draws in one launch, one workgroup each: row r takes logits + r * logits_stride,
// hist + r * hist_stride, hist_len_dev[r], counter_dev[r], the seed seed + r * seed_stride and
// axq_sample_scratch_bytes(vocab) bytes of scratch of its own, and writes out[r].
int axq_dev_sample_rows(axq_ctx *ctx, int rows, const float *logits, size_t logits_stride, int vocab, const int32_t *hist,
                        size_t hist_stride, const int32_t *hist_len_dev, int hist_len, const axq_sampling_config *cfg, float u,
                        const int32_t *counter_dev, uint64_t seed, uint64_t seed_stride, void *scratch, int32_t *out,
                        float *filtered_out) {
    SampleArgs a;
    a.logits = logits;
    a.work = reinterpret_cast<float *>(scratch);
    a.vocab = vocab;
    a.hist = hist; a.hist_len_dev = hist_len_dev; a.hist_len = hist ? hist_len : 0;
    if (!hist) a.hist_len_dev = nullptr;
    a.temperature = cfg->temperature; a.top_p = cfg->top_p; a.penalty = cfg->repetition_penalty;
    a.top_k = cfg->top_k; a.do_sample = cfg->do_sample;
    a.u = u; a.counter_dev = counter_dev; a.seed = seed;
    a.out = out; a.filtered_out = filtered_out;
    a.logits_stride = logits_stride; a.hist_stride = hist_stride; a.work_stride = 2 * padded_words(vocab); a.seed_stride = seed_stride;
    static std::atomic<uint64_t> lds_allowed{0};
    {
        int rc;
        if ((rc = axq_allow_lds(ctx, reinterpret_cast<const void *>(&sample_kernel<true>), lds_allowed, padded_words(LDS_VOCAB) * 4))) return rc;
    }
    if (vocab <= LDS_VOCAB) sample_kernel<true><<<rows, ST, padded_words(vocab) * 4, ctx->stream>>>(a);
    else sample_kernel<false><<<rows, ST, 0, ctx->stream>>>(a);
    AXQ_LAUNCH_CHECK(ctx, "sample_kernel");
    return AXQ_OK;
}

size_t axq_sample_scratch_bytes(int vocab) { return 2 * padded_words(vocab) * 4; }

int axq_check_sampling_config(axq_ctx *ctx, const axq_sampling_config *cfg) {
    if (!cfg) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "sampling: NULL configuration");
    if (!(cfg->temperature > 0.0f)) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "sampling: temperature must be positive");
    if (!(cfg->repetition_penalty > 0.0f)) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "sampling: repetition penalty must be positive");
    if (cfg->top_k < 0) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "sampling: top_k must not be negative");
    return AXQ_OK;
}

extern "C" {

int axq_sample_token(axq_ctx *ctx, const float *logits, int vocab, const int32_t *generated, int n_generated,
                     const axq_sampling_config *cfg, float u, int32_t *token, float *filtered_logits, int mem) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_sample_token: NULL context");
    int rc;
    if ((rc = axq_check_sampling_config(ctx, cfg))) return rc;
    if (!logits || !token || vocab <= 0 || n_generated < 0 || (n_generated > 0 && !generated))
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_sample_token: bad argument");
    if (mem != AXQ_MEM_HOST && mem != AXQ_MEM_DEVICE) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "bad memory space %d", mem);
    if (!(u >= 0.0f && u < 1.0f)) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_sample_token: u must lie in [0, 1)");
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    const size_t vb = (size_t)vocab * 4, hb = (size_t)n_generated * 4;
    Temp scratch, dl, dh, dt, df;
    AXQ_HIP(ctx, hipMalloc(&scratch.p, axq_sample_scratch_bytes(vocab)), AXQ_ERR_ALLOCATION_FAILED);
    if (mem == AXQ_MEM_DEVICE) {
        if ((rc = axq_dev_sample(ctx, logits, vocab, generated, nullptr, n_generated, cfg, u, nullptr, 0, scratch.p, token,
                                 filtered_logits)))
            return rc;
        AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER); // the scratch is released on return
        return AXQ_OK;
    }
    AXQ_HIP(ctx, hipMalloc(&dl.p, vb), AXQ_ERR_ALLOCATION_FAILED);
    AXQ_HIP(ctx, hipMalloc(&dt.p, 4), AXQ_ERR_ALLOCATION_FAILED);
    AXQ_HIP(ctx, hipMemcpyAsync(dl.p, logits, vb, hipMemcpyHostToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    if (n_generated) {
        AXQ_HIP(ctx, hipMalloc(&dh.p, hb), AXQ_ERR_ALLOCATION_FAILED);
        AXQ_HIP(ctx, hipMemcpyAsync(dh.p, generated, hb, hipMemcpyHostToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    }
    if (filtered_logits) AXQ_HIP(ctx, hipMalloc(&df.p, vb), AXQ_ERR_ALLOCATION_FAILED);
    if ((rc = axq_dev_sample(ctx, (const float *)dl.p, vocab, (const int32_t *)dh.p, nullptr, n_generated, cfg, u, nullptr, 0,
                             scratch.p, (int32_t *)dt.p, (float *)df.p)))
        return rc;
    AXQ_HIP(ctx, hipMemcpyAsync(token, dt.p, 4, hipMemcpyDeviceToHost, ctx->stream), AXQ_ERR_COPY_FAILED);
    if (filtered_logits) AXQ_HIP(ctx, hipMemcpyAsync(filtered_logits, df.p, vb, hipMemcpyDeviceToHost, ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

} // extern "C"
