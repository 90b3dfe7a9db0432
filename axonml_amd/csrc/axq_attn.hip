// Causal attention for many prompt rows of one sequence on the matrix pipe.
//
// What it computes is the attention core of LLaMAAttention::forward (crates/axonml-llm/src/llama.rs:420-447)
// with GQA head sharing (llama.rs:450-480) for `T` new positions at once: row b holds the query heads of position
// pos0 + b, the keys and values of positions 0 .. pos0 + T - 1 are in the f16 cache already, and query (b, head)
// attends to positions lo .. pos0 + b (lo > 0 under a sliding window, mistral.rs:204-238).
//
// A workgroup takes one KV head and a tile of 32 / rep consecutive rows, i.e. 32 "virtual queries" (row, head of
// the group).  Each of its four waves walks every fourth tile of 32 key positions with an online softmax of its
// own (running maximum m, sum l and output O per virtual query), and the four are merged at the end.  Both
// products are taken transposed, so that a virtual query is a LANE (column lane % 32) all the way through:
//   S^T = K Q^T    v_mfma_f32_32x32x16_f16, A = keys straight from the cache (a lane's operand is 16 contiguous bytes
//                  of one key row), B = the RoPE-rotated, 1/sqrt(d)-scaled queries as f16 pairs q = qh + ql (two
//                  MFMAs per step, so that 22 bits of every query survive).  A lane then holds 16 of its query's 32
//                  scores, the lane 32 further on the other 16: maximum and sum cost one exchange each, and m, l and
//                  the rescaling factor are one number per lane;
//   P^T = exp(S^T - m) as an f16 pair is already where the B operand of the second product wants it, but for runs of
//                  four positions that sit in the partner lane: one v_permlane32_swap per register pair;
//   O^T += V^T P^T A = values with the key position as the contiguous index, which it is not in the cache: the value
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

// accumulator layout of the 32x32 MFMA: lane -> column lane % 32; register r -> row 8 (r / 4) + 4 (lane / 32) + r % 4
__device__ inline int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

template <int D, int REP>
__global__ void __launch_bounds__(256, 2) attn_flash_kernel(FlashArgs a) {
    constexpr int HALF = D / 2, TQ = VQ / REP, KS = D / 16, DB = D / 32;
    constexpr int QLD = D + PADH;  // halfs per row of the query planes and of a value tile
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    _Float16 *qh = reinterpret_cast<_Float16 *>(lds_raw);         // [VQ][QLD]
    _Float16 *ql = qh + VQ * QLD;                                  // [VQ][QLD]
    _Float16 *wave_base = ql + VQ * QLD;                           // per wave: value tile [TK][QLD]
    constexpr int WAVE_HALFS = TK * QLD;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, lk = (lane >> 5) * 8;
    _Float16 *vs = wave_base + wave * WAVE_HALFS;
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
    // (the query operands of a lane, row li, halfs 16 ks + lk .. + 8 of both planes, are read from LDS tile by tile:
    //  kept in registers they would cost 64 of them and with that the second workgroup per compute unit)

    // ---- the range of key positions any query of the tile looks at, from a multiple of 8 (operand alignment)
    const int p_first = a.pos0 + b0, p_last = a.pos0 + b0 + nrows - 1;
    int k_lo = (a.window > 0 && p_first + 1 > a.window) ? p_first + 1 - a.window : 0;
    k_lo &= ~7;
    const int ntiles = (p_last - k_lo) / TK + 1;

    // this lane's virtual query, and the positions it looks at (none for a row beyond T)
    const int hf = lane >> 5;
    const int my_qi = li / REP;
    const int k_to = my_qi < nrows ? p_first + my_qi : -1;
    const int k_from = (a.window > 0 && p_first + my_qi + 1 > a.window) ? p_first + my_qi + 1 - a.window : 0;
    const int lo_last = (a.window > 0 && p_last + 1 > a.window) ? p_last + 1 - a.window : 0;

    float m = -INFINITY, l = 0.f;
    float16v O[DB]; // O^T: register r of block db = dim 32 db + acc_row(r, lane)
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) O[db][r] = 0.f;

    // keys (this lane's A operands: row = position j0 + li) and values (16 bytes per lane and pass) of a tile, clamped
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
    constexpr float LOG2E = 1.4426950408889634f; // exp(x) = 2^(x log2 e), one instruction
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
        int qoff = li * QLD + lk;
        asm volatile("" : "+v"(qoff)); // opaque: keeps the compiler from hoisting these loads out of the loop into registers
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const half8 qa_l = *reinterpret_cast<const half8 *>(ql + qoff + ks * 16);
            const half8 qa_h = *reinterpret_cast<const half8 *>(qh + qoff + ks * 16);
            S = __builtin_amdgcn_mfma_f32_32x32x16_f16(kb[ks], qa_l, S, 0, 0, 0);
            S = __builtin_amdgcn_mfma_f32_32x32x16_f16(kb[ks], qa_h, S, 0, 0, 0);
        }
        // online softmax of this lane's query over its 16 positions and the partner lane's 16.  A tile that every query
        // of the workgroup sees whole (most of them) needs no masks.
        const bool whole = nrows == TQ && j0 + TK - 1 <= p_first && j0 >= lo_last;
        float mloc = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            if (!whole) {
                const int pos = j0 + acc_row(r, lane);
                S[r] = (pos <= k_to && pos >= k_from) ? S[r] : -INFINITY;
            }
            mloc = fmaxf(mloc, S[r]);
        }
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
        const float mx = fmaxf(m, mloc);
        const bool empty = mx == -INFINITY; // nothing to look at yet: the state stays as it is
        const float alpha = empty ? 1.f : __builtin_amdgcn_exp2f((m - mx) * LOG2E); // 2^(-inf) = 0 on the first tile with keys
        float psum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            S[r] = empty ? 0.f : __builtin_amdgcn_exp2f((S[r] - mx) * LOG2E);
            psum += S[r];
        }
        psum += __shfl_xor(psum, 32);
        l = l * alpha + psum;
        m = mx;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) O[db][r] *= alpha;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): this wave's LDS writes (the value tile) have landed
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // O^T += V^T P^T: contraction over the tile's positions, 16 per step.  Registers 8 ks .. 8 ks + 3 (X) and
        // 8 ks + 4 .. 8 ks + 7 (Y) hold positions 16 ks + {0..3, 8..11} in the lower half-wave and {4..7, 12..15} in the
        // upper one; the operand wants 16 ks + 0..7 below and 16 ks + 8..15 above: swapping X's upper half with Y's lower
        // half leaves, in both, the operand's first four positions in X and its last four in Y.
#pragma unroll
        for (int ks = 0; ks < TK / 16; ks++) {
            uint32_t xh[2], yh[2], xl[2], yl[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const float x0 = S[8 * ks + 2 * i], x1 = S[8 * ks + 2 * i + 1], y0 = S[8 * ks + 4 + 2 * i], y1 = S[8 * ks + 5 + 2 * i];
                // the f16 part is the value with its mantissa cut to eleven bits (exact in f16), the rest its own leading bits
                const float x0h = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, x0) & 0xFFFFE000u);
                const float x1h = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, x1) & 0xFFFFE000u);
                const float y0h = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, y0) & 0xFFFFE000u);
                const float y1h = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, y1) & 0xFFFFE000u);
                xh[i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x0h, x1h));
                yh[i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(y0h, y1h));
                xl[i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x0 - x0h, x1 - x1h));
                yl[i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(y0 - y0h, y1 - y1h));
                auto sh = __builtin_amdgcn_permlane32_swap(xh[i], yh[i], false, false);
                xh[i] = sh[0]; yh[i] = sh[1];
                auto sl = __builtin_amdgcn_permlane32_swap(xl[i], yl[i], false, false);
                xl[i] = sl[0]; yl[i] = sl[1];
            }
            const u32x4 bh = {xh[0], xh[1], yh[0], yh[1]}, bl = {xl[0], xl[1], yl[0], yl[1]};
            const half8 pb_h = __builtin_bit_cast(half8, bh), pb_l = __builtin_bit_cast(half8, bl);
#pragma unroll
            for (int db = 0; db < DB; db++) {
                half8 va; // row = dim 32 db + li, columns = positions 16 ks + lk .. + 8 of the tile
#pragma unroll
                for (int i = 0; i < 8; i++) va[i] = vs[(ks * 16 + lk + i) * QLD + db * 32 + li];
                O[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va, pb_l, O[db], 0, 0, 0);
                O[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va, pb_h, O[db], 0, 0, 0);
            }
        }
        __builtin_amdgcn_wave_barrier(); // the next tile overwrites the value tile only after every lane has read it
    }

    // ---- merge the four waves (in wave order, so that the result does not depend on timing): waves 1..3 hand their
    //      state to wave 0 through LDS, one at a time; row = virtual query, D outputs, then m and l
    for (int w = 1; w < 4; w++) {
        __syncthreads();
        if (wave == w) {
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) mrg[li * (D + 2) + db * 32 + acc_row(r, lane)] = O[db][r];
            if (hf == 0) { mrg[li * (D + 2) + D] = m; mrg[li * (D + 2) + D + 1] = l; }
        }
        __syncthreads();
        if (wave == 0) {
            const float mo = mrg[li * (D + 2) + D], lo = mrg[li * (D + 2) + D + 1];
            const float mx = fmaxf(m, mo);
            const float wa = mx == -INFINITY ? 1.f : expf(m - mx), wb = mx == -INFINITY ? 0.f : expf(mo - mx);
            l = l * wa + lo * wb;
            m = mx;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) O[db][r] = O[db][r] * wa + mrg[li * (D + 2) + db * 32 + acc_row(r, lane)] * wb;
        }
    }
    __syncthreads();
    if (wave == 0) {
        const float inv = k_to >= 0 ? 1.0f / l : 0.f; // every valid query sees at least its own position
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) mrg[li * (D + 2) + db * 32 + acc_row(r, lane)] = O[db][r] * inv;
    }
    __syncthreads();
    // rows of the output, 16 bytes per thread
    for (int idx = tid; idx < VQ * (D / 4); idx += 256) {
        const int vq = idx / (D / 4), c4 = idx % (D / 4), qi = vq / REP, h = vq % REP;
        if (qi < nrows) {
            const float *src = mrg + vq * (D + 2) + c4 * 4;
            *reinterpret_cast<float4 *>(a.att + (size_t)(b0 + qi) * q_dim + (size_t)(kvh * REP + h) * D + c4 * 4) =
                make_float4(src[0], src[1], src[2], src[3]);
        }
    }
}

template <int D, int REP>
size_t flash_lds_bytes() {
    const size_t planes = (size_t)2 * VQ * (D + PADH) * 2;
    const size_t per_wave = (size_t)TK * (D + PADH) * 2;
    const size_t merge = (size_t)VQ * (D + 2) * 4;
    return planes + (4 * per_wave > merge ? 4 * per_wave : merge);
}

template <int D, int REP>
int launch_flash(axq_ctx *ctx, const FlashArgs &a) {
    const size_t lds = flash_lds_bytes<D, REP>();
    static std::atomic<uint64_t> lds_allowed{0};
    int rc;
    if (lds > 48 * 1024 && (rc = axq_allow_lds(ctx, reinterpret_cast<const void *>(&attn_flash_kernel<D, REP>), lds_allowed, lds))) return rc;
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
