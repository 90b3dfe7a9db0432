// Causal attention for many prompt rows of one sequence on the matrix pipe.
//
// What it computes is the attention core of LLaMAAttention::forward (crates/axonml-llm/src/llama.rs:420-447)
// with GQA head sharing (llama.rs:450-480) for `T` new positions at once: row b holds the query heads of position
// pos0 + b, the keys and values of positions 0 .. pos0 + T - 1 are in the f16 cache already, and query (b, head)
// attends to positions lo .. pos0 + b (lo > 0 under a sliding window, mistral.rs:204-238).
//
// A workgroup takes one KV head and a tile of 32 / rep consecutive rows, i.e. 32 "virtual queries" (row, head of
// the group).  Each of its four waves walks every fourth tile of 32 key positions with an online softmax of its
// own (running maximum m, sum l and output O per virtual query), and the four are merged at the end:
//   S = Q K^T      v_mfma_f32_32x32x16_f16, A = the RoPE-rotated, 1/sqrt(d)-scaled queries as f16 pairs q = qh + ql
//                  (two MFMAs per step, so that 22 bits of every query survive), B = keys straight from the cache
//                  (a lane's operand is 16 contiguous bytes of one key row);
//   P = exp(S - m) in the accumulator layout (lane = key position, register = virtual query): row maxima and sums
//                  are reductions over 32 lanes; P goes through a small LDS tile to become an A operand, again as
//                  an f16 pair;
//   O += P V       B = values, which need the key position as the contiguous index of a lane's operand: the value
//                  tile is staged in LDS and read column-wise.
// Rows beyond T, positions outside a query's range and an empty range are masked, never read as data.
#include <hip/hip_fp16.h>
#include <math.h>

#include "axq_internal.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4))); // a 16-byte register quad (arrays of HIP's uint4 struct end up in scratch)

constexpr int VQ = 32;  // virtual queries per workgroup (one MFMA tile of rows)
constexpr int TK = 32;  // key positions per step of a wave
constexpr int PADH = 8; // halfs of padding per LDS row

struct FlashArgs {
    const float *qkv;
    int qkv_rows;
    const float *rope_cos, *rope_sin;
    const uint16_t *kcache, *vcache; // of this layer and sequence: [kv_head][max_pos][D]
    int pos0, T, n_heads, n_kv, max_pos, window;
    float *att; // [T][n_heads * D]
};

// maximum / sum over the 32 lanes of a half-wave, result in every lane (quad permutes and row mirrors inside a
// 16-lane row, one exchange across rows)
__device__ inline float half_wave_max(float v) {
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, true)));
    return fmaxf(v, __shfl_xor(v, 16));
}
__device__ inline float half_wave_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, true));
    return v + __shfl_xor(v, 16);
}

// accumulator layout of the 32x32 MFMA: lane -> column lane % 32; register r -> row 8 (r / 4) + 4 (lane / 32) + r % 4
__device__ inline int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

template <int D, int REP>
__global__ void __launch_bounds__(256) attn_flash_kernel(FlashArgs a) {
    constexpr int HALF = D / 2, TQ = VQ / REP, KS = D / 16, DB = D / 32;
    constexpr int QLD = D + PADH;  // halfs per row of the query planes and of a value tile
    constexpr int PLD = TK + PADH; // halfs per row of a probability plane
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    _Float16 *qh = reinterpret_cast<_Float16 *>(lds_raw);         // [VQ][QLD]
    _Float16 *ql = qh + VQ * QLD;                                  // [VQ][QLD]
    _Float16 *wave_base = ql + VQ * QLD;                           // per wave: value tile [TK][QLD], P planes 2 x [VQ][PLD]
    constexpr int WAVE_HALFS = TK * QLD + 2 * VQ * PLD;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, lk = (lane >> 5) * 8;
    _Float16 *vs = wave_base + wave * WAVE_HALFS;
    _Float16 *ph = vs + TK * QLD, *pl = ph + VQ * PLD;
    float *mrg = reinterpret_cast<float *>(wave_base); // after the key loop: [VQ][D + 2] floats of one wave's (O, m, l)

    const int kvh = blockIdx.x, b0 = blockIdx.y * TQ;
    const int q_dim = a.n_heads * D;
    const int nrows = a.T - b0 < TQ ? a.T - b0 : TQ; // valid query rows of this tile
    const uint16_t *kc = a.kcache + (size_t)kvh * a.max_pos * D;
    const uint16_t *vc = a.vcache + (size_t)kvh * a.max_pos * D;

    // ---- queries: RoPE (RotaryEmbedding::rotate_tensor, llama.rs:281-321, half-split pairs), scale, split into f16 pairs
    const float scale = 1.0f / sqrtf((float)D);
    for (int t = tid; t < VQ * HALF; t += 256) {
        const int vq = t / HALF, e = t % HALF, qi = vq / REP, h = vq % REP;
        float r1 = 0.f, r2 = 0.f;
        if (qi < nrows) {
            const int p = a.pos0 + b0 + qi;
            const float *qrow = a.qkv + (size_t)(b0 + qi) * a.qkv_rows + (size_t)(kvh * REP + h) * D;
            const float c = a.rope_cos[(size_t)p * HALF + e], s = a.rope_sin[(size_t)p * HALF + e];
            const float q1 = qrow[e], q2 = qrow[e + HALF];
            r1 = (q1 * c - q2 * s) * scale;
            r2 = (q1 * s + q2 * c) * scale;
        }
        const _Float16 h1 = (_Float16)r1, h2 = (_Float16)r2;
        qh[vq * QLD + e] = h1; ql[vq * QLD + e] = (_Float16)(r1 - (float)h1);
        qh[vq * QLD + e + HALF] = h2; ql[vq * QLD + e + HALF] = (_Float16)(r2 - (float)h2);
    }
    __syncthreads();
    // this lane's A operands for every step over d: row li, halfs 16 ks + lk .. + 8
    half8 qa_h[KS], qa_l[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        qa_h[ks] = *reinterpret_cast<const half8 *>(qh + li * QLD + ks * 16 + lk);
        qa_l[ks] = *reinterpret_cast<const half8 *>(ql + li * QLD + ks * 16 + lk);
    }

    // ---- the range of key positions any query of the tile looks at, from a multiple of 8 (operand alignment)
    const int p_first = a.pos0 + b0, p_last = a.pos0 + b0 + nrows - 1;
    int k_lo = (a.window > 0 && p_first + 1 > a.window) ? p_first + 1 - a.window : 0;
    k_lo &= ~7;
    const int ntiles = (p_last - k_lo) / TK + 1;

    // register r of the accumulator belongs to query row acc_row(r, lane) / REP of the tile; that query looks at positions
    // lo .. hi (hi = -1 for a row beyond T: no position qualifies)
    auto key_range = [&](int r, int &lo, int &hi) {
        const int qi = acc_row(r, lane) / REP;
        const int p = p_first + qi;
        hi = qi < nrows ? p : -1;
        lo = (a.window > 0 && p + 1 > a.window) ? p + 1 - a.window : 0;
    };

    float m[16], l[16];
    float16v O[DB];
#pragma unroll
    for (int r = 0; r < 16; r++) { m[r] = -INFINITY; l[r] = 0.f; }
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) O[db][r] = 0.f;

    // keys (this lane's B operands: column = position j0 + li) and values (16 bytes per lane and pass) of a tile, clamped
    // into the cache; what lies beyond a query's range is masked below.  The next tile's are requested while the
    // current one is worked on.
    constexpr int NV = TK * D / 8 / 64;
    half8 kb_next[KS];
    u32x4 vraw_next[NV];
    auto fetch = [&](int kt) {
        const int j0 = k_lo + kt * TK;
        const int jk = j0 + li <= p_last ? j0 + li : p_last;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) kb_next[ks] = *reinterpret_cast<const half8 *>(kc + (size_t)jk * D + ks * 16 + lk);
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int idx = i * 64 + lane, row = idx / (D / 8), c8 = idx % (D / 8);
            const int jv = j0 + row <= p_last ? j0 + row : p_last;
            vraw_next[i] = *reinterpret_cast<const u32x4 *>(vc + (size_t)jv * D + c8 * 8);
        }
    };
    if (wave < ntiles) fetch(wave);
    for (int kt = wave; kt < ntiles; kt += 4) {
        const int j0 = k_lo + kt * TK;
        half8 kb[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) kb[ks] = kb_next[ks];
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int idx = i * 64 + lane, row = idx / (D / 8), c8 = idx % (D / 8);
            *reinterpret_cast<u32x4 *>(vs + row * QLD + c8 * 8) = vraw_next[i];
        }
        if (kt + 4 < ntiles) fetch(kt + 4);
        float16v S;
#pragma unroll
        for (int r = 0; r < 16; r++) S[r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            S = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa_l[ks], kb[ks], S, 0, 0, 0);
            S = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa_h[ks], kb[ks], S, 0, 0, 0);
        }
        // online softmax, row by row (a row = a register across the 32 lanes of a half-wave).  A tile that every
        // query of the workgroup sees whole (most of them) needs no masks.  exp(x) = 2^(x log2 e), one instruction.
        const int pos = j0 + li;
        const int lo_last = (a.window > 0 && p_last + 1 > a.window) ? p_last + 1 - a.window : 0;
        const bool whole = nrows == TQ && j0 + TK - 1 <= p_first && j0 >= lo_last;
        constexpr float LOG2E = 1.4426950408889634f;
        float alpha[16];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            float s = S[r];
            if (!whole) {
                int k_from, k_to;
                key_range(r, k_from, k_to);
                s = (pos <= k_to && pos >= k_from) ? s : -INFINITY;
            }
            const float mx = fmaxf(m[r], half_wave_max(s));
            const float p = mx == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((s - mx) * LOG2E); // a row with nothing to look at yet stays empty
            alpha[r] = mx == -INFINITY ? 1.f : __builtin_amdgcn_exp2f((m[r] - mx) * LOG2E);   // 2^(-inf) = 0 on the first tile with keys
            l[r] = l[r] * alpha[r] + half_wave_sum(p);
            m[r] = mx;
            // P as an f16 pair into this wave's planes, transposed: row = virtual query, column = position in the tile
            const _Float16 hi = (_Float16)p;
            const int row = acc_row(r, lane);
            ph[row * PLD + li] = hi;
            pl[row * PLD + li] = (_Float16)(p - (float)hi);
        }
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) O[db][r] *= alpha[r];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): this wave's LDS writes (values, P) have landed
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // O += P V: contraction over the tile's positions, 16 per step
#pragma unroll
        for (int ks = 0; ks < TK / 16; ks++) {
            const half8 pa_h = *reinterpret_cast<const half8 *>(ph + li * PLD + ks * 16 + lk);
            const half8 pa_l = *reinterpret_cast<const half8 *>(pl + li * PLD + ks * 16 + lk);
#pragma unroll
            for (int db = 0; db < DB; db++) {
                half8 vb; // column = dim 32 db + li, rows = positions 16 ks + lk .. + 8 of the tile
#pragma unroll
                for (int i = 0; i < 8; i++) vb[i] = vs[(ks * 16 + lk + i) * QLD + db * 32 + li];
                O[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(pa_l, vb, O[db], 0, 0, 0);
                O[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(pa_h, vb, O[db], 0, 0, 0);
            }
        }
        __builtin_amdgcn_wave_barrier(); // the next tile overwrites vs / ph / pl only after every lane has read them
    }

    // ---- merge the four waves (in wave order, so that the result does not depend on timing): waves 1..3 hand their
    //      state to wave 0 through LDS, one at a time
    for (int w = 1; w < 4; w++) {
        __syncthreads();
        if (wave == w) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = acc_row(r, lane);
#pragma unroll
                for (int db = 0; db < DB; db++) mrg[row * (D + 2) + db * 32 + li] = O[db][r];
                if (li == 0) { mrg[row * (D + 2) + D] = m[r]; mrg[row * (D + 2) + D + 1] = l[r]; }
            }
        }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = acc_row(r, lane);
                const float mo = mrg[row * (D + 2) + D], lo = mrg[row * (D + 2) + D + 1];
                const float mx = fmaxf(m[r], mo);
                const float wa = mx == -INFINITY ? 1.f : expf(m[r] - mx), wb = mx == -INFINITY ? 0.f : expf(mo - mx);
                l[r] = l[r] * wa + lo * wb;
                m[r] = mx;
#pragma unroll
                for (int db = 0; db < DB; db++) O[db][r] = O[db][r] * wa + mrg[row * (D + 2) + db * 32 + li] * wb;
            }
        }
    }
    if (wave == 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int row = acc_row(r, lane), qi = row / REP, h = row % REP;
            if (qi < nrows) {
                float *o = a.att + (size_t)(b0 + qi) * q_dim + (size_t)(kvh * REP + h) * D;
                const float inv = 1.0f / l[r]; // every valid query sees at least its own position
#pragma unroll
                for (int db = 0; db < DB; db++) o[db * 32 + li] = O[db][r] * inv;
            }
        }
    }
}

template <int D, int REP>
size_t flash_lds_bytes() {
    const size_t planes = (size_t)2 * VQ * (D + PADH) * 2;
    const size_t per_wave = ((size_t)TK * (D + PADH) + 2 * VQ * (TK + PADH)) * 2;
    const size_t merge = (size_t)VQ * (D + 2) * 4;
    return planes + (4 * per_wave > merge ? 4 * per_wave : merge);
}

template <int D, int REP>
int launch_flash(axq_ctx *ctx, const FlashArgs &a) {
    const size_t lds = flash_lds_bytes<D, REP>();
    static bool big_lds_allowed = false; // dynamic LDS beyond 64 KB has to be asked for once per kernel
    if (lds > 48 * 1024 && !big_lds_allowed) {
        AXQ_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_flash_kernel<D, REP>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)lds), AXQ_ERR_DRIVER);
        big_lds_allowed = true;
    }
    const int tq = VQ / REP;
    attn_flash_kernel<D, REP><<<dim3(a.n_kv, (a.T + tq - 1) / tq), 256, lds, ctx->stream>>>(a);
    AXQ_LAUNCH_CHECK(ctx, "attn_flash_kernel");
    return 1;
}

template <int D>
int launch_flash_d(axq_ctx *ctx, const FlashArgs &a, int rep) {
    switch (rep) {
    case 1: return launch_flash<D, 1>(ctx, a);
    case 2: return launch_flash<D, 2>(ctx, a);
    case 4: return launch_flash<D, 4>(ctx, a);
    case 8: return launch_flash<D, 8>(ctx, a);
    default: return 0;
    }
}

} // namespace

// 1 = launched, 0 = shape not covered (head size other than 32, 64, 128; query heads per KV head not 1, 2, 4 or 8),
// < 0 = error.  The rows' keys and values must be in the cache already.
int axq_dev_attn_rows_mfma(axq_ctx *ctx, const float *qkv, int qkv_rows, const float *rope_cos, const float *rope_sin,
                           const uint16_t *kcache, const uint16_t *vcache, int pos0, int T, int n_heads, int n_kv, int head_dim,
                           int max_pos, int window, float *att) {
    FlashArgs a;
    a.qkv = qkv; a.qkv_rows = qkv_rows; a.rope_cos = rope_cos; a.rope_sin = rope_sin;
    a.kcache = kcache; a.vcache = vcache;
    a.pos0 = pos0; a.T = T; a.n_heads = n_heads; a.n_kv = n_kv; a.max_pos = max_pos; a.window = window;
    a.att = att;
    if (T < 1 || n_heads % n_kv != 0) return 0;
    const int rep = n_heads / n_kv;
    switch (head_dim) {
    case 32: return launch_flash_d<32>(ctx, a, rep);
    case 64: return launch_flash_d<64>(ctx, a, rep);
    case 128: return launch_flash_d<128>(ctx, a, rep);
    default: return 0;
    }
}
