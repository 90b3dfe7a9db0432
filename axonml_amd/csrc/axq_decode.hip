// Decode step of a LLaMA/Mistral-shape model with every linear block-quantized.
//
// Follows LLaMA::forward_with_cache (crates/axonml-llm/src/llama.rs:731-762) and
// LLaMAForCausalLM::generate (llama.rs:900-977) for one sequence (batch 1):
//   embedding lookup            crates/axonml-nn/src/layers/embedding.rs:103-146
//   RMSNorm                     llama.rs:158-187
//   q/k/v, o, gate/up/down      Linear::forward on quantized weights (the GEMV kernels)
//   RoPE, half-split            llama.rs:223-252, 281-321 (tables built on the host as the reference does)
//   KV cache append             crates/axonml-llm/src/attention.rs:46-70 (f16 here, grown in place)
//   GQA causal attention        llama.rs:420-447 without the repeat_kv copy (llama.rs:450-480)
//   SwiGLU                      llama.rs:562-567
//   greedy argmax               llama.rs:1025-1030 (of equal maxima the last index wins)
//
// Device-side structure: q,k,v are one fused weight, gate and up another; every kernel that
// produces a GEMV input also writes it in split (int8 limb) form, so the GEMV kernels never
// re-split x; position and current token live in device memory so that the whole step is one
// HIP graph replayed per token with no host round trip.
#include <hip/hip_fp16.h>
#include <math.h>
#include <stdlib.h>

#include <vector>

#include "axq_internal.h"
#include "axq_split.h"

struct axq_model {
    axq_ctx *ctx;
    axq_model_config cfg;
    int qkv_rows, q_dim, kv_dim;
    // weights
    uint16_t *emb;                  // f16 [vocab, hidden], or
    float *emb32 = nullptr;         // f32 [vocab, hidden] as the reference keeps it (one of the two is set)
    float *norm_attn, *norm_ffn;    // [layers, hidden]
    float *norm_final;              // [hidden]
    std::vector<axq_weight *> w_qkv, w_o, w_gu, w_down;
    // q, k or v of a layer whose block type differs from the fused weight's (GGUF files that keep attn_v at six bits
    // beside four-bit attn_q and attn_k): a weight of its own, multiplied after the fused one into its rows of qkv
    std::vector<axq_weight *> w_sep[3];
    axq_weight *w_head;
    std::vector<uint32_t> set_mask; // per layer: bit per axq_linear_id that has been set
    bool head_set;
    float *rope_cos, *rope_sin;     // [max_pos, head_dim / 2]
    uint16_t *kcache, *vcache;      // f16 [layers, kv_heads, max_pos, head_dim]
    // activations
    float *h, *xn, *qkv, *att, *gu, *act, *logits;
    float *att_part;                // [kv_heads][max_splits][rep][head_dim + 2] partial attention results
    float *pb_h, *pb_xn, *pb_qkv, *pb_att, *pb_gu, *pb_act; // the same activations for pb_cap prompt tokens at a time
    int pb_cap;
    int n_seq;                      // sequences the caches and the per-sequence state hold (axq_model_set_batch)
    size_t seq_stride;              // cache elements of one sequence: layers * kv_heads * max_pos * head_dim
    size_t part_stride;             // floats of att_part per sequence
    std::vector<int> seq_pos;       // host mirror of pos[s] for the batched calls (sequence 0: host_pos)
    int32_t *bprompt, *boffsets, *bout; // prompts, their offsets and the generated ids of a batched generate
    hipGraphExec_t graph_b, graph_bf; // batched step: split attention / one attention workgroup per head (short contexts)
    bool graph_b_ok, graph_bf_ok;
    int max_splits;
    // device-side state
    int32_t *pos, *tok, *next, *gen, *prompt, *out;
    int32_t *hist;                  // every token fed so far, by position (what a repetition penalty looks at)
    void *sample_scratch;           // scratch of the sampler, allocated when one is set
    bool sampling;                  // next token by axq_sampling_config instead of the plain argmax
    axq_sampling_config sampler;
    uint64_t sample_seed;
    int prompt_cap, out_cap;
    int host_pos;
    hipGraphExec_t graph;           // the one-token step with the attention split over the positions
    bool graph_ok;
    hipGraphExec_t graph_f;         // the same with one attention workgroup per head (short contexts)
    bool graph_f_ok;
    int fused_max;                  // contexts up to this many positions take graph_f
    int prompt_chunk;               // most prompt rows per pass through the layers
    bool attn_mfma;                 // prompt attention of many rows on the matrix pipe (development knob AXQ_ATTN_MFMA=0: off)
};

namespace {

__device__ inline float block_sum(float v, float *scratch) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m);
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; i++) t += scratch[i];
    return t;
}

// h = embedding[tok] widened to f32 (Embedding::lookup, nn/src/layers/embedding.rs:103-146); grid.y = tokens.
__global__ void __launch_bounds__(256) embed_kernel(const uint16_t *emb, const float *emb32, const int32_t *tok, float *h, int hidden) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= (hidden >> 3)) return;
    h += (size_t)blockIdx.y * hidden;
    if (emb32) { // an f32 table: the row as it is
        const float4 *src = reinterpret_cast<const float4 *>(emb32 + (size_t)tok[blockIdx.y] * hidden + (size_t)t * 8);
        float4 *dst = reinterpret_cast<float4 *>(h + (size_t)t * 8);
        dst[0] = src[0];
        dst[1] = src[1];
        return;
    }
    const uint4 raw = *reinterpret_cast<const uint4 *>(emb + (size_t)tok[blockIdx.y] * hidden + (size_t)t * 8);
    const uint32_t r[4] = {raw.x, raw.y, raw.z, raw.w};
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        v[2 * i] = __half2float(__ushort_as_half((unsigned short)(r[i] & 0xFFFF)));
        v[2 * i + 1] = __half2float(__ushort_as_half((unsigned short)(r[i] >> 16)));
    }
    float4 *o = reinterpret_cast<float4 *>(h + (size_t)t * 8);
    o[0] = make_float4(v[0], v[1], v[2], v[3]);
    o[1] = make_float4(v[4], v[5], v[6], v[7]);
}

// xn = rmsnorm(h) * w (RMSNorm::forward, llm/src/llama.rs:158-187).  One workgroup per vector.  Used in front of
// linears that the matrix-pipe GEMV does not cover (otherwise the GEMV normalises its input itself) and for
// prompt tokens that go through the layers several at a time.
__global__ void __launch_bounds__(1024) norm_kernel(const float *h, const float *w, int hidden, float eps, float *xn) {
    __shared__ float scratch[16];
    const int ntask = hidden >> 3;
    h += (size_t)blockIdx.x * hidden;
    xn += (size_t)blockIdx.x * hidden;
    float ss = 0.f;
    for (int t = threadIdx.x; t < ntask; t += blockDim.x) {
        const float4 *p = reinterpret_cast<const float4 *>(h + (size_t)t * 8);
        float4 a = p[0], b = p[1];
        const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int i = 0; i < 8; i++) ss = fmaf(v[i], v[i], ss);
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
    for (int t = threadIdx.x; t < ntask; t += blockDim.x) {
        const float4 *p = reinterpret_cast<const float4 *>(h + (size_t)t * 8);
        const float4 *pw = reinterpret_cast<const float4 *>(w + (size_t)t * 8);
        float4 a = p[0], b = p[1], wa = pw[0], wb = pw[1];
        float4 *o = reinterpret_cast<float4 *>(xn + (size_t)t * 8);
        o[0] = make_float4((a.x * inv) * wa.x, (a.y * inv) * wa.y, (a.z * inv) * wa.z, (a.w * inv) * wa.w);
        o[1] = make_float4((b.x * inv) * wb.x, (b.y * inv) * wb.y, (b.z * inv) * wb.z, (b.w * inv) * wb.w);
    }
}

// Attention for one new token, split over the cached positions ("flash decoding"):
//
// attn_partial_kernel, grid (kv_heads, max_splits): workgroup (g, s) covers positions [s*CHUNK, (s+1)*CHUNK)
// of KV head g for all the query heads that share it (GQA without the repeat_kv copy, llama.rs:450-480).
// It applies RoPE to those query heads, computes q.k / sqrt(d) against the cached f16 keys with 16-byte
// loads (d/8 lanes per position), keeps the chunk's running maximum m, exponentials and their sum l, and
// accumulates sum_p exp(s_p - m) v_p.  The workgroup whose chunk holds the newest position also applies
// RoPE to the new key, rounds k and v to f16, appends them to the cache and uses them from registers.
// Workgroups whose chunk starts beyond the newest position leave at once (the grid is sized for the
// longest context so that the launch can sit in a graph).
//
// attn_combine_kernel, grid (heads): merges the partial (m, l, o) triples of a head in a fixed order,
// normalises, and writes the head's output as f32 and in split form.
constexpr int ATT_CHUNK = 32;
constexpr int ATT_MAX_REP = 8;  // query heads per KV head

__device__ inline void halves_to_floats(const uint4 &raw, float (&f)[8]) {
    const uint32_t rr[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int e = 0; e < 4; e++) {
        f[2 * e] = __half2float(__ushort_as_half((unsigned short)(rr[e] & 0xFFFF)));
        f[2 * e + 1] = __half2float(__ushort_as_half((unsigned short)(rr[e] >> 16)));
    }
}

// Sum over aligned groups of LP lanes (4, 8, 16 or 32), every lane of the group gets the total: DPP quad
// permutes and row mirrors inside a 16-lane row, one lane exchange beyond it.
template <int LP>
__device__ inline float group_sum(float s) {
    s += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, s), 0xB1, 0xf, 0xf, true));
    s += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, s), 0x4E, 0xf, 0xf, true));
    if (LP >= 8) s += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, s), 0x141, 0xf, 0xf, true));
    if (LP >= 16) s += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, s), 0x140, 0xf, 0xf, true));
    if (LP >= 32) s += __shfl_xor(s, 16);
    return s;
}

// D = head size (32, 64, 128, 256), REP = query heads per KV head rounded up to a power of two (the real
// count `rep` may be smaller).  Specialised so that the code is short and straight: a kernel that runs once
// per layer is fetched cold, and its instruction fetch is part of its run time.
template <int D, int REP>
__global__ void __launch_bounds__(256) attn_partial_kernel(const float *qkv, const float *rope_cos, const float *rope_sin,
                                                           uint16_t *kcache, uint16_t *vcache, const int32_t *pos_p,
                                                           int n_heads, int n_kv, int max_pos, int max_splits, int window,
                                                           float *part, int qkv_stride, size_t seq_stride, size_t part_stride) {
    constexpr int HALF = D / 2;
    constexpr int LP = D / 8, PPW = 64 / LP;                 // lanes per position, positions per wave pass
    constexpr int NPASS = (ATT_CHUNK + 4 * PPW - 1) / (4 * PPW); // passes of the four waves over the chunk
    constexpr int NQ = (REP * HALF + 255) / 256;             // rotation pairs of the query heads per thread
    constexpr int NHG = 256 / D > 0 ? 256 / D : 1;           // head groups in the value sum (threads = NHG * D)
    constexpr int HPT = (REP + NHG - 1) / NHG;               // heads per thread in the value sum
    static_assert(D <= 256 && ATT_CHUNK <= 64 && REP <= ATT_MAX_REP, "shape limits");
    __shared__ float qs[REP * D];            // rotated query heads
    __shared__ float knew[D], vnew[D];       // the new key and value, f16-rounded
    __shared__ __attribute__((aligned(16))) float sc[ATT_CHUNK * REP]; // scores, then exp(score - max), head-minor
    __shared__ float stat[2 * REP];          // per head: m, l
    __shared__ __attribute__((aligned(16))) float vs[ATT_CHUNK * D];   // the chunk's values
    const int rep = n_heads / n_kv;
    const int kvh = blockIdx.x, split = blockIdx.y;
    // blockIdx.z: the sequence (batched steps: its own row of qkv, position counter, cache and partial results)
    qkv += (size_t)blockIdx.z * qkv_stride;
    kcache += (size_t)blockIdx.z * seq_stride;
    vcache += (size_t)blockIdx.z * seq_stride;
    part += (size_t)blockIdx.z * part_stride;
    const int pos = pos_p[blockIdx.z];
    const int p0 = split * ATT_CHUNK;
    // sliding window (MistralAttention, mistral.rs:204-238): positions before p_lo are not attended to
    const int p_lo = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
    if (p0 > pos || p0 + ATT_CHUNK <= p_lo) return;
    const int p1 = (p0 + ATT_CHUNK < pos + 1) ? p0 + ATT_CHUNK : pos + 1;
    const int np = p1 - p0;
    const bool has_new = pos < p1;
    const int q_dim = n_heads * D, kv_dim = n_kv * D;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    uint16_t *kc = kcache + (size_t)kvh * max_pos * D;
    uint16_t *vc = vcache + (size_t)kvh * max_pos * D;

    // Everything this workgroup reads from memory is requested here, so that the kernel pays one memory
    // latency and not one per stage.  Positions outside the chunk and the newest one (still in registers)
    // re-read the chunk's first row and are not used.
    const int c8 = lane % LP, r = lane / LP;
    uint4 kraw[NPASS], vraw[NPASS];
#pragma unroll
    for (int it = 0; it < NPASS; it++) {
        const int pi = (it * 4 + wave) * PPW + r;
        const int p = (pi < np && p0 + pi != pos) ? p0 + pi : p0;
        kraw[it] = *reinterpret_cast<const uint4 *>(kc + (size_t)p * D + c8 * 8);
        vraw[it] = *reinterpret_cast<const uint4 *>(vc + (size_t)p * D + c8 * 8);
    }
    const float *cs = rope_cos + (size_t)pos * HALF, *sn = rope_sin + (size_t)pos * HALF;
    float qx1[NQ], qx2[NQ], qc[NQ], qn[NQ];
#pragma unroll
    for (int u = 0; u < NQ; u++) {
        int i = tid + u * 256;
        i = i < rep * HALF ? i : 0;
        const int h = i / HALF, e = i % HALF;
        const float *qh = qkv + (size_t)(kvh * rep + h) * D;
        qc[u] = cs[e]; qn[u] = sn[e]; qx1[u] = qh[e]; qx2[u] = qh[e + HALF];
    }
    const int en = tid < HALF ? tid : 0;
    const float *kh = qkv + q_dim + (size_t)kvh * D;
    const float *vh = qkv + q_dim + kv_dim + (size_t)kvh * D;
    const float nc = cs[en], ns = sn[en], k1 = kh[en], k2 = kh[en + HALF], v1 = vh[en], v2 = vh[en + HALF];

    // RoPE (RotaryEmbedding::rotate_tensor, llm/src/llama.rs:281-321: half-split pairs) on the query heads ...
#pragma unroll
    for (int u = 0; u < NQ; u++) {
        const int i = tid + u * 256;
        if (i < rep * HALF) {
            const int h = i / HALF, e = i % HALF;
            qs[h * D + e] = qx1[u] * qc[u] - qx2[u] * qn[u];
            qs[h * D + e + HALF] = qx1[u] * qn[u] + qx2[u] * qc[u];
        }
    }
    // ... and on the new key, which goes to the cache with the new value, rounded to f16
    if (has_new && tid < HALF) {
        const int e = tid;
        __half ka = __float2half_rn(k1 * nc - k2 * ns), kb = __float2half_rn(k1 * ns + k2 * nc);
        __half va = __float2half_rn(v1), vb = __float2half_rn(v2);
        knew[e] = __half2float(ka); knew[e + HALF] = __half2float(kb);
        vnew[e] = __half2float(va); vnew[e + HALF] = __half2float(vb);
        kc[(size_t)pos * D + e] = __half_as_ushort(ka); kc[(size_t)pos * D + e + HALF] = __half_as_ushort(kb);
        vc[(size_t)pos * D + e] = __half_as_ushort(va); vc[(size_t)pos * D + e + HALF] = __half_as_ushort(vb);
    }
    __syncthreads();
    // scores, and the chunk's values into LDS as f32
    const float scale = 1.0f / sqrtf((float)D);
#pragma unroll
    for (int it = 0; it < NPASS; it++) {
        const int pi = (it * 4 + wave) * PPW + r; // position within the chunk
        if (pi < ATT_CHUNK) {
            float kf[8], vf[8];
            halves_to_floats(kraw[it], kf);
            halves_to_floats(vraw[it], vf);
            const bool cached = pi < np && p0 + pi != pos;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                kf[e] = cached ? kf[e] : (pi < np ? knew[c8 * 8 + e] : 0.f);
                vf[e] = cached ? vf[e] : (pi < np ? vnew[c8 * 8 + e] : 0.f);
            }
            float4 *dst = reinterpret_cast<float4 *>(vs + pi * D + c8 * 8);
            dst[0] = make_float4(vf[0], vf[1], vf[2], vf[3]);
            dst[1] = make_float4(vf[4], vf[5], vf[6], vf[7]);
            float sh[REP];
#pragma unroll
            for (int h = 0; h < REP; h++) {
                const float4 *qh = reinterpret_cast<const float4 *>(qs + h * D + c8 * 8);
                const float4 qa = qh[0], qb = qh[1];
                float s = qa.x * kf[0];
                s = fmaf(qa.y, kf[1], s); s = fmaf(qa.z, kf[2], s); s = fmaf(qa.w, kf[3], s);
                s = fmaf(qb.x, kf[4], s); s = fmaf(qb.y, kf[5], s); s = fmaf(qb.z, kf[6], s); s = fmaf(qb.w, kf[7], s);
                sh[h] = s;
            }
#pragma unroll
            for (int h = 0; h < REP; h++) sh[h] = group_sum<LP>(sh[h]);
            if (c8 == 0) {
#pragma unroll
                for (int h = 0; h < REP; h++) sc[pi * REP + h] = (pi < np && p0 + pi >= p_lo && h < rep) ? sh[h] * scale : -INFINITY;
            }
        }
    }
    __syncthreads();
    // per head: chunk maximum, exponentials, their sum (one wave per head, heads strided over the 4 waves)
    for (int h = wave; h < rep; h += 4) {
        float v = lane < ATT_CHUNK ? sc[lane * REP + h] : -INFINITY;
        float mx = v;
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m));
        float e = (lane < np && p0 + lane >= p_lo) ? expf(v - mx) : 0.f;
        float sum = e;
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) sum += __shfl_xor(sum, m);
        if (lane < ATT_CHUNK) sc[lane * REP + h] = e; // zero beyond the chunk's last position
        if (lane == 0) { stat[2 * h] = mx; stat[2 * h + 1] = sum; }
    }
    __syncthreads();
    // sum_p e_p v_p: thread = (head group, dim), heads hg, hg + NHG, ...; positions in order, rows beyond
    // np carry weight zero
    const int dim = tid % D, hg = tid / D;
    float acc[HPT];
#pragma unroll
    for (int i = 0; i < HPT; i++) acc[i] = 0.f;
#pragma unroll 8
    for (int pi = 0; pi < ATT_CHUNK; pi++) {
        const float vv = vs[pi * D + dim];
#pragma unroll
        for (int i = 0; i < HPT; i++) {
            const int h = hg + i * NHG;
            acc[i] = fmaf(sc[pi * REP + (h < REP ? h : 0)], vv, acc[i]);
        }
    }
#pragma unroll
    for (int i = 0; i < HPT; i++) {
        const int h = hg + i * NHG;
        if (h < rep && tid < NHG * D) {
            float *o = part + ((size_t)(kvh * max_splits + split) * rep + h) * (D + 2);
            o[2 + dim] = acc[i];
            if (dim == 0) { o[0] = stat[2 * h]; o[1] = stat[2 * h + 1]; }
        }
    }
}

// Where an attention kernel leaves its output rows a second time, as the operands of the small-batch GEMV with the
// output projection (which then skips its own packing pass): xa = nullptr for nothing.
struct PackOut {
    uint8_t *xa = nullptr;
    float *xsg = nullptr;
    int even_odd = 0;
};

// o[0 .. d) of head `head` of row b (LDS) -> operands; the first d / 8 threads of the workgroup, whole lane quads.
// The workgroups of the last row also write the zeros of the rows that the batch does not have.
__device__ inline void pack_head_out(const float *o, int d, int head, int n_heads, int b, int rows, const PackOut &pk) {
    const int tid = threadIdx.x;
    if (tid >= (d >> 3)) return;
    const int t = head * (d >> 3) + tid, nblk = (n_heads * d) >> 5;
    float v[8];
    const float4 a0 = *reinterpret_cast<const float4 *>(o + tid * 8), a1 = *reinterpret_cast<const float4 *>(o + tid * 8 + 4);
    v[0] = a0.x; v[1] = a0.y; v[2] = a0.z; v[3] = a0.w; v[4] = a1.x; v[5] = a1.y; v[6] = a1.z; v[7] = a1.w;
    const int b_end = b == rows - 1 ? 8 : b + 1;
    for (int bb = b; bb < b_end; bb++) {
        if (pk.even_odd) axq_store_packed<true>(v, t, bb, rows, nblk, pk.xa, pk.xsg);
        else axq_store_packed<false>(v, t, bb, rows, nblk, pk.xa, pk.xsg);
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = 0.f;
    }
}

// grid (heads), 256 threads.  The (m, l) pairs of the head's splits go through LDS so that every thread
// knows the weights exp(m_s - max) before it walks the splits.  Everything the first COMB_PRE splits need is
// requested before the first barrier (a context of up to COMB_PRE * ATT_CHUNK positions pays one memory latency, not
// three); the walk over further splits has no dependent loads either.
constexpr int COMB_PRE = 16;

__global__ void __launch_bounds__(256) attn_combine_kernel(const float *part, const int32_t *pos_p, int n_heads, int n_kv,
                                                           int d, int max_splits, int window, float *att, size_t part_stride,
                                                           PackOut pk) {
    extern __shared__ float cm[];
    __shared__ __attribute__((aligned(16))) float ov[256];
    float *wgt = cm;                 // [max_splits] exp(m_s - max)
    float *lv = wgt + max_splits;    // [max_splits] l_s
    float *red = lv + max_splits;    // [4] wave maxima
    const int head = blockIdx.x, rep = n_heads / n_kv, kvh = head / rep, h = head - kvh * rep;
    part += (size_t)blockIdx.y * part_stride; // blockIdx.y: the sequence
    att += (size_t)blockIdx.y * n_heads * d;
    const int pos = pos_p[blockIdx.y];
    const int s_lo = (window > 0 && pos + 1 > window) ? (pos + 1 - window) / ATT_CHUNK : 0; // first split inside the window
    const int nsplit = pos / ATT_CHUNK + 1 - s_lo;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *base = part + ((size_t)(kvh * max_splits + s_lo) * rep + h) * (d + 2);
    const size_t stride = (size_t)rep * (d + 2);
    const int dim = tid < d ? tid : 0;
    // requests: (m, l) of split tid, the first splits' outputs of this thread's dim
    const bool mine = tid < nsplit;
    const float m0 = mine ? base[tid * stride] : -INFINITY, l0 = mine ? base[tid * stride + 1] : 0.f;
    float opre[COMB_PRE];
#pragma unroll
    for (int u = 0; u < COMB_PRE; u++) opre[u] = base[(u < nsplit ? u : 0) * stride + 2 + dim];
    // maxima
    float mx = m0;
    for (int s = tid + 256; s < nsplit; s += 256) mx = fmaxf(mx, base[s * stride]);
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m));
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    // weights; the normaliser is summed below in split order by every thread so that the result does not depend on timing
    if (mine) { wgt[tid] = expf(m0 - mx); lv[tid] = l0; }
    for (int s = tid + 256; s < nsplit; s += 256) { wgt[s] = expf(base[s * stride] - mx); lv[s] = base[s * stride + 1]; }
    __syncthreads();
    {
        float l = 0.f, o = 0.f;
#pragma unroll
        for (int u = 0; u < COMB_PRE; u++) {
            if (u < nsplit) {
                l = fmaf(lv[u], wgt[u], l);
                o = fmaf(opre[u], wgt[u], o);
            }
        }
        int s = COMB_PRE;
        for (; s + 4 <= nsplit; s += 4) {
            float o4[4];
#pragma unroll
            for (int u = 0; u < 4; u++) o4[u] = base[(s + u) * stride + 2 + dim];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                l = fmaf(lv[s + u], wgt[s + u], l);
                o = fmaf(o4[u], wgt[s + u], o);
            }
        }
        for (; s < nsplit; s++) {
            l = fmaf(lv[s], wgt[s], l);
            o = fmaf(base[s * stride + 2 + dim], wgt[s], o);
        }
        if (tid < d) {
            const float v = o / l;
            att[(size_t)head * d + tid] = v;
            ov[tid] = v;
        }
    }
    if (pk.xa) {
        __syncthreads();
        pack_head_out(ov, d, head, n_heads, blockIdx.y, gridDim.y, pk);
    }
}

// Prompt tokens go through the layers up to eight at a time (one pass over the weights serves all of them).
// rope_append_kernel, grid (kv_heads, tokens), head_dim / 2 threads: RoPE on the new keys, keys and values
// rounded to f16 into the cache at positions pos0 + b, exactly as the one-token kernel above writes them.
constexpr int PROMPT_BATCH = 8;
constexpr int MAX_SEQUENCES = 64;    // sequences side by side
constexpr int GEMV_GROUPS_MAX = 24;  // up to here a batched step goes in groups of PROMPT_BATCH rows, beyond its linears are GEMMs

__global__ void __launch_bounds__(128) rope_append_kernel(const float *qkv, int qkv_rows, int q_dim, int kv_dim,
                                                          const float *rope_cos, const float *rope_sin, uint16_t *kcache,
                                                          uint16_t *vcache, int pos0, const int32_t *pos_arr,
                                                          size_t seq_stride, int max_pos, int d) {
    const int half = d >> 1, e = threadIdx.x, kvh = blockIdx.x, b = blockIdx.y;
    // rows of one sequence at consecutive positions, or (pos_arr given) one row per sequence at that sequence's position
    const int p = pos_arr ? pos_arr[b] : pos0 + b;
    if (pos_arr) { kcache += (size_t)b * seq_stride; vcache += (size_t)b * seq_stride; }
    const float *row = qkv + (size_t)b * qkv_rows;
    const float *kh = row + q_dim + (size_t)kvh * d, *vh = row + q_dim + kv_dim + (size_t)kvh * d;
    const float nc = rope_cos[(size_t)p * half + e], ns = rope_sin[(size_t)p * half + e];
    const float k1 = kh[e], k2 = kh[e + half];
    uint16_t *kc = kcache + ((size_t)kvh * max_pos + p) * d, *vc = vcache + ((size_t)kvh * max_pos + p) * d;
    kc[e] = __half_as_ushort(__float2half_rn(k1 * nc - k2 * ns));
    kc[e + half] = __half_as_ushort(__float2half_rn(k1 * ns + k2 * nc));
    vc[e] = __half_as_ushort(__float2half_rn(vh[e]));
    vc[e + half] = __half_as_ushort(__float2half_rn(vh[e + half]));
}

// attn_prompt_kernel, grid (heads, tokens), 1024 threads: the query of head `head` at position p = pos0 + b
// against the cached keys lo..p (causal, llama.rs:420-447; lo > 0 under a sliding window): scores into LDS, their
// maximum, exponentials and sum, then sum_j e_j v_j / sum.  Keys and values are read 16 bytes per lane,
// head_dim / 8 lanes per position.  APPEND (rows of different sequences only, pos_arr given): the row's own key and
// value are not in the cache yet; every workgroup rotates the key itself, uses both from LDS (rounded to f16 as the
// cache holds them), and the first query head of each KV head writes them to the cache.
template <int D, bool APPEND>
__global__ void __launch_bounds__(1024) attn_prompt_kernel(const float *qkv, int qkv_rows, const float *rope_cos,
                                                           const float *rope_sin, uint16_t *kcache, uint16_t *vcache, int pos0,
                                                           const int32_t *pos_arr, size_t seq_stride, int n_heads, int n_kv,
                                                           int max_pos, int window, float *att, PackOut pk) {
    constexpr int HALF = D / 2, LP = D / 8, PPB = 1024 / LP; // lanes per position, positions per pass of the workgroup
    extern __shared__ float sc[];                            // scores, then exp(score - max)
    __shared__ __attribute__((aligned(16))) float qs[D];
    __shared__ __attribute__((aligned(16))) float knew[APPEND ? D : 4], vnew[APPEND ? D : 4];
    __shared__ float red[16];
    __shared__ __attribute__((aligned(16))) float osum[16 * D];
    const int head = blockIdx.x, b = blockIdx.y;
    const int p = pos_arr ? pos_arr[b] : pos0 + b; // as in rope_append_kernel
    if (pos_arr) { kcache += (size_t)b * seq_stride; vcache += (size_t)b * seq_stride; }
    const int rep = n_heads / n_kv, kvh = head / rep;
    const int p_lo = (window > 0 && p + 1 > window) ? p + 1 - window : 0;
    const int span = p + 1 - p_lo;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint16_t *kc = kcache + ((size_t)kvh * max_pos + p_lo) * D;
    const uint16_t *vc = vcache + ((size_t)kvh * max_pos + p_lo) * D;
    if (tid < HALF) {
        const float *qh = qkv + (size_t)b * qkv_rows + (size_t)head * D;
        const float c = rope_cos[(size_t)p * HALF + tid], s = rope_sin[(size_t)p * HALF + tid];
        const float q1 = qh[tid], q2 = qh[tid + HALF];
        qs[tid] = q1 * c - q2 * s;
        qs[tid + HALF] = q1 * s + q2 * c;
    } else if (APPEND && tid >= 512 && tid < 512 + HALF) { // other waves: the new key and value (arithmetic of rope_append_kernel)
        const int e = tid - 512, q_dim = n_heads * D, kv_dim = n_kv * D;
        const float *row = qkv + (size_t)b * qkv_rows;
        const float *kh = row + q_dim + (size_t)kvh * D, *vh = row + q_dim + kv_dim + (size_t)kvh * D;
        const float nc = rope_cos[(size_t)p * HALF + e], ns = rope_sin[(size_t)p * HALF + e];
        const float k1 = kh[e], k2 = kh[e + HALF];
        const __half ka = __float2half_rn(k1 * nc - k2 * ns), kb = __float2half_rn(k1 * ns + k2 * nc);
        const __half va = __float2half_rn(vh[e]), vb = __float2half_rn(vh[e + HALF]);
        knew[e] = __half2float(ka); knew[e + HALF] = __half2float(kb);
        vnew[e] = __half2float(va); vnew[e + HALF] = __half2float(vb);
        if (head == kvh * rep) {
            uint16_t *kw = kcache + ((size_t)kvh * max_pos + p) * D, *vw = vcache + ((size_t)kvh * max_pos + p) * D;
            kw[e] = __half_as_ushort(ka); kw[e + HALF] = __half_as_ushort(kb);
            vw[e] = __half_as_ushort(va); vw[e + HALF] = __half_as_ushort(vb);
        }
    }
    __syncthreads();
    const int c8 = tid % LP, r = tid / LP;
    float qf[8];
    {
        const float4 *qp = reinterpret_cast<const float4 *>(qs + c8 * 8);
        const float4 qa = qp[0], qb = qp[1];
        qf[0] = qa.x; qf[1] = qa.y; qf[2] = qa.z; qf[3] = qa.w; qf[4] = qb.x; qf[5] = qb.y; qf[6] = qb.z; qf[7] = qb.w;
    }
    const float scale = 1.0f / sqrtf((float)D);
    constexpr int UN = 4; // 16-byte loads in flight per lane (8 was slower at every context, 16 spills)
    for (int j0 = 0; j0 < span; j0 += UN * PPB) {
        uint4 raw[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const int j = j0 + u * PPB + r;
            raw[u] = *reinterpret_cast<const uint4 *>(kc + (size_t)(j < span - (APPEND ? 1 : 0) ? j : 0) * D + c8 * 8);
        }
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const int j = j0 + u * PPB + r;
            float kf[8];
            halves_to_floats(raw[u], kf);
            if (APPEND && j == span - 1) {
#pragma unroll
                for (int e = 0; e < 8; e++) kf[e] = knew[c8 * 8 + e];
            }
            float s = qf[0] * kf[0];
#pragma unroll
            for (int e = 1; e < 8; e++) s = fmaf(qf[e], kf[e], s);
            s = group_sum<LP>(s);
            if (j < span && c8 == 0) sc[j] = s * scale;
        }
    }
    __syncthreads();
    float mx = -INFINITY;
    for (int j = tid; j < span; j += 1024) mx = fmaxf(mx, sc[j]);
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m));
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = red[0];
#pragma unroll
    for (int w = 1; w < 16; w++) mx = fmaxf(mx, red[w]);
    float sum = 0.f;
    for (int j = tid; j < span; j += 1024) {
        const float e = expf(sc[j] - mx);
        sc[j] = e;
        sum += e;
    }
    sum = block_sum(sum, red); // its barriers also publish the exponentials
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j0 = 0; j0 < span; j0 += UN * PPB) {
        uint4 raw[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const int j = j0 + u * PPB + r;
            raw[u] = *reinterpret_cast<const uint4 *>(vc + (size_t)(j < span - (APPEND ? 1 : 0) ? j : 0) * D + c8 * 8);
        }
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const int j = j0 + u * PPB + r;
            const float e = j < span ? sc[j] : 0.f;
            float vf[8];
            halves_to_floats(raw[u], vf);
            if (APPEND && j == span - 1) {
#pragma unroll
                for (int i = 0; i < 8; i++) vf[i] = vnew[c8 * 8 + i];
            }
#pragma unroll
            for (int i = 0; i < 8; i++) acc[i] = fmaf(e, vf[i], acc[i]);
        }
    }
    // lanes of a wave that hold the same dims, then the sixteen waves in order
#pragma unroll
    for (int m = LP; m < 64; m <<= 1) {
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] += __shfl_xor(acc[i], m);
    }
    if (lane < LP) {
        float4 *dst = reinterpret_cast<float4 *>(osum + wave * D + c8 * 8);
        dst[0] = make_float4(acc[0], acc[1], acc[2], acc[3]);
        dst[1] = make_float4(acc[4], acc[5], acc[6], acc[7]);
    }
    __syncthreads();
    if (tid < D) {
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < 16; w++) o += osum[w * D + tid];
        o /= sum;
        att[(size_t)b * n_heads * D + (size_t)head * D + tid] = o;
        qs[tid] = o; // the query is in registers by now
    }
    if (pk.xa) {
        __syncthreads();
        pack_head_out(qs, D, head, n_heads, b, gridDim.y, pk);
    }
}

// act = silu(gate) * up over [inter]; gu alternates four gate values with the four up values of the same indices
// (the row order of the fused gate/up weight); grid.y = vectors.
__global__ void __launch_bounds__(256) swiglu_kernel(const float *gu, int inter, float *act) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x; // four consecutive outputs
    if (t >= (inter >> 2)) return;
    gu += (size_t)blockIdx.y * 2 * inter;
    act += (size_t)blockIdx.y * inter;
    const float4 g = *reinterpret_cast<const float4 *>(gu + (size_t)t * 8);
    const float4 u = *reinterpret_cast<const float4 *>(gu + (size_t)t * 8 + 4);
    float4 o;
    o.x = (g.x * (1.0f / (1.0f + expf(-g.x)))) * u.x;
    o.y = (g.y * (1.0f / (1.0f + expf(-g.y)))) * u.y;
    o.z = (g.z * (1.0f / (1.0f + expf(-g.z)))) * u.z;
    o.w = (g.w * (1.0f / (1.0f + expf(-g.w)))) * u.w;
    *reinterpret_cast<float4 *>(act + (size_t)t * 4) = o;
}

// argmax over the logits, last index among equal maxima (Iterator::max_by); then pos += 1.
__global__ void __launch_bounds__(1024) argmax_kernel(const float *logits, int vocab, int32_t *next, int32_t *pos) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    logits += (size_t)blockIdx.x * vocab; // one workgroup per sequence
    next += blockIdx.x;
    pos += blockIdx.x;
    float best = -INFINITY;
    int idx = 0;
    // eight 16-byte loads per thread in flight at a time; a thread's indices rise, and `>=` keeps the last maximum
    const int n4 = vocab >> 2;
    const float4 *l4 = reinterpret_cast<const float4 *>(logits);
    for (int base = threadIdx.x; base < n4; base += 8 * 1024) {
        float4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int f = base + u * 1024;
            v[u] = l4[f < n4 ? f : n4 - 1];
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int f = base + u * 1024;
            if (f < n4) {
                const float e[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
                for (int c = 0; c < 4; c++)
                    if (e[c] >= best) { best = e[c]; idx = 4 * f + c; }
            }
        }
    }
    for (int i = 4 * n4 + threadIdx.x; i < vocab; i += 1024) {
        float v = logits[i];
        if (v >= best) { best = v; idx = i; }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        float ov = __shfl_xor(best, m);
        int oi = __shfl_xor(idx, m);
        if (ov > best || (ov == best && oi > idx)) { best = ov; idx = oi; }
    }
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) { bv[wave] = best; bi[wave] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); w++)
            if (bv[w] > best || (bv[w] == best && bi[w] > idx)) { best = bv[w]; idx = bi[w]; }
        next[0] = idx;
        pos[0] = pos[0] + 1;
    }
}

__global__ void pick_prompt_kernel(const int32_t *prompt, const int32_t *pos, int base, int32_t *tok) {
    tok[0] = prompt[pos[0] - base];
}
__global__ void commit_next_kernel(const int32_t *next, int32_t *tok, int32_t *gen, int32_t *out, int out_cap) {
    int g = gen[0];
    tok[0] = next[0];
    if (g < out_cap) out[g] = next[0];
    gen[0] = g + 1;
}
__global__ void set_i32_kernel(int32_t *p, int32_t v) { p[0] = v; }
__global__ void add_i32_kernel(int32_t *p, int32_t v) { p[0] += v; }
__global__ void record_tokens_kernel(int32_t *hist, int pos0, const int32_t *toks) { hist[pos0 + threadIdx.x] = toks[threadIdx.x]; }
__global__ void record_token_kernel(int32_t *hist, const int32_t *pos, const int32_t *tok) { hist[pos[0]] = tok[0]; }
// one thread per sequence
__global__ void record_rows_kernel(int32_t *hist, int max_pos, const int32_t *pos, const int32_t *tok) {
    hist[(size_t)threadIdx.x * max_pos + pos[threadIdx.x]] = tok[threadIdx.x];
}
__global__ void last_tokens_kernel(const int32_t *prompts, const int32_t *offsets, int32_t *tok) {
    tok[threadIdx.x] = prompts[offsets[threadIdx.x + 1] - 1];
}
__global__ void commit_rows_kernel(const int32_t *next, int32_t *tok, int32_t *out, int step, int out_cap) {
    tok[threadIdx.x] = next[threadIdx.x];
    out[(size_t)threadIdx.x * out_cap + step] = next[threadIdx.x];
}
__global__ void fill_f32_kernel(float *p, size_t n, float v) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}
__global__ void f32_to_f16_kernel(const float *src, size_t n, uint16_t *dst) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = __half_as_ushort(__float2half_rn(src[i]));
}

int lin_dims(const axq_model *m, int layer, int which, int64_t *rows, int64_t *k) {
    const axq_model_config &c = m->cfg;
    if (layer < 0) { *rows = c.vocab_size; *k = c.hidden_size; return 0; }
    switch (which) {
    case AXQ_LIN_Q: *rows = m->q_dim; *k = c.hidden_size; break;
    case AXQ_LIN_K: case AXQ_LIN_V: *rows = m->kv_dim; *k = c.hidden_size; break;
    case AXQ_LIN_O: *rows = c.hidden_size; *k = m->q_dim; break;
    case AXQ_LIN_GATE: case AXQ_LIN_UP: *rows = c.intermediate_size; *k = c.hidden_size; break;
    case AXQ_LIN_DOWN: *rows = c.hidden_size; *k = c.intermediate_size; break;
    default: return -1;
    }
    return 0;
}

// Copies all rows of src into dst starting at dst row `row_off` (same type and k): plane by plane.
int copy_rows(axq_ctx *ctx, axq_weight *dst, const axq_weight *src, int64_t row_off) {
    struct { uint8_t *d; const uint8_t *s; size_t pitch; } planes[3] = {
        {dst->codes, src->codes, src->codes_pitch}, {dst->meta, src->meta, src->meta_pitch}, {dst->qh, src->qh, src->qh_pitch}};
    for (auto &p : planes) {
        if (p.pitch == 0) continue;
        AXQ_HIP(ctx, hipMemcpyAsync(p.d + (size_t)row_off * p.pitch, p.s, p.pitch * (size_t)src->n_rows,
                                    hipMemcpyDeviceToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    }
    return AXQ_OK;
}

// Rows of `src` into every other group of four rows of `dst`, starting at group `first` (0 or 1): the fused
// gate/up weight alternates four gate rows with the four up rows of the same indices, so that a GEMV
// workgroup holds both halves of every pair it needs for silu(gate) * up.
int copy_rows_interleaved(axq_ctx *ctx, axq_weight *dst, const axq_weight *src, int first) {
    struct { uint8_t *d; const uint8_t *s; size_t pitch; } planes[3] = {
        {dst->codes, src->codes, src->codes_pitch}, {dst->meta, src->meta, src->meta_pitch}, {dst->qh, src->qh, src->qh_pitch}};
    for (auto &p : planes) {
        if (p.pitch == 0) continue;
        AXQ_HIP(ctx, hipMemcpy2DAsync(p.d + (size_t)first * 4 * p.pitch, 8 * p.pitch, p.s, 4 * p.pitch, 4 * p.pitch,
                                      (size_t)src->n_rows / 4, hipMemcpyDeviceToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    }
    return AXQ_OK;
}

// Attention of the newest token of the `nseq` sequences from s0 on (rows of qkv, qkv_rows apart), split over the positions,
// and the merge of the splits; results to att (rows n_heads * d apart).
template <int D, int REP>
void launch_attn_partial_t(axq_model *m, int l, const float *qkv, int nseq, int s0, hipStream_t st) {
    const axq_model_config &c = m->cfg;
    const size_t kv_layer = (size_t)c.num_key_value_heads * c.max_position_embeddings * D;
    attn_partial_kernel<D, REP><<<dim3(c.num_key_value_heads, m->max_splits, nseq), 256, 0, st>>>(
        qkv, m->rope_cos, m->rope_sin, m->kcache + (size_t)l * kv_layer + (size_t)s0 * m->seq_stride,
        m->vcache + (size_t)l * kv_layer + (size_t)s0 * m->seq_stride, m->pos + s0, c.num_attention_heads, c.num_key_value_heads,
        c.max_position_embeddings, m->max_splits, c.sliding_window, m->att_part + (size_t)s0 * m->part_stride, m->qkv_rows, m->seq_stride,
        m->part_stride);
}

template <int D>
void launch_attn_partial_d(axq_model *m, int l, const float *qkv, int nseq, int s0, hipStream_t st) {
    const int rep = m->cfg.num_attention_heads / m->cfg.num_key_value_heads;
    if (rep == 1) launch_attn_partial_t<D, 1>(m, l, qkv, nseq, s0, st);
    else if (rep == 2) launch_attn_partial_t<D, 2>(m, l, qkv, nseq, s0, st);
    else if (rep <= 4) launch_attn_partial_t<D, 4>(m, l, qkv, nseq, s0, st);
    else launch_attn_partial_t<D, 8>(m, l, qkv, nseq, s0, st);
}

void launch_attn_split(axq_model *m, int l, const float *qkv, int nseq, float *att, hipStream_t st, PackOut pk = PackOut(), int s0 = 0) {
    const axq_model_config &c = m->cfg;
    switch (c.head_dim) { // axq_model_create admits these four sizes only
    case 32: launch_attn_partial_d<32>(m, l, qkv, nseq, s0, st); break;
    case 64: launch_attn_partial_d<64>(m, l, qkv, nseq, s0, st); break;
    case 128: launch_attn_partial_d<128>(m, l, qkv, nseq, s0, st); break;
    default: launch_attn_partial_d<256>(m, l, qkv, nseq, s0, st); break;
    }
    const size_t comb_lds = (size_t)(2 * m->max_splits + 8) * sizeof(float);
    attn_combine_kernel<<<dim3(c.num_attention_heads, nseq), 256, comb_lds, st>>>(m->att_part + (size_t)s0 * m->part_stride, m->pos + s0, c.num_attention_heads,
                                                                                c.num_key_value_heads, c.head_dim, m->max_splits,
                                                                                c.sliding_window, att, m->part_stride, pk);
}

// y = g(W f(x) (+ bias)): f = identity or RMSNorm with weights `aux`; g = identity, or, for the fused gate/up
// weight, silu(gate) * up over its row pairs (y then has half as many entries as W has rows).  The matrix-pipe
// GEMV applies f while it stages x and g while it writes y; for a linear it does not cover (other weight types,
// K not a multiple of 64 or beyond 16384) f and g run as kernels of their own around the f32 GEMV, through `tmp`.
// First row of q (0), k (1) or v (2) in a row of qkv.
inline int64_t qkv_part_offset(const axq_model *m, int part) { return part == 0 ? 0 : (part == 1 ? m->q_dim : m->q_dim + m->kv_dim); }

int linear(axq_model *m, const axq_weight *w, const float *x, int xmode, const float *aux, int ymode, float *tmp,
           const float *bias, float *y) {
    axq_ctx *ctx = m->ctx;
    if (axq_dev_gemv_dp_covers(w)) {
        int rc = axq_dev_gemv_dp_ex(ctx, w, x, nullptr, xmode, aux, m->cfg.rms_norm_eps, ymode, bias, y);
        return rc < 0 ? rc : AXQ_OK;
    }
    const int k = (int)w->k, n = (int)w->n_rows;
    if (xmode == AXQ_X_RMSNORM) {
        norm_kernel<<<1, 1024, 0, ctx->stream>>>(x, aux, k, m->cfg.rms_norm_eps, tmp);
        x = tmp;
    }
    if (ymode == AXQ_Y_SWIGLU) {
        int rc = axq_dev_gemv(ctx, w, x, 1, bias, m->gu);
        if (rc) return rc;
        swiglu_kernel<<<(n / 8 + 255) / 256, 256, 0, ctx->stream>>>(m->gu, n / 2, y);
        return AXQ_OK;
    }
    return axq_dev_gemv(ctx, w, x, 1, bias, y);
}

// The kernels of one token, enqueued on the context's stream: six per layer when every linear is covered
// by the matrix-pipe GEMV (norms and SwiGLU ride in the GEMVs, residual adds in their bias slot).
void launch_attn_rows(axq_model *m, int l, const float *qkv, int nb, int pos0, const int32_t *pos_arr, size_t cache_off, size_t lds,
                      float *att, hipStream_t st, PackOut pk = PackOut());
size_t prompt_attn_lds(const axq_model *m, int last);

// short: the context is at most m->fused_max positions: one attention workgroup per head does everything (the new key
// and value included); otherwise the positions are split over workgroups and a second kernel merges them.
int enqueue_step(axq_model *m, bool short_ctx) {
    axq_ctx *ctx = m->ctx;
    const axq_model_config &c = m->cfg;
    hipStream_t st = ctx->stream;
    const int H = c.hidden_size;
    int rc;
    embed_kernel<<<(H / 8 + 255) / 256, 256, 0, st>>>(m->emb, m->emb32, m->tok, m->h, H);
    for (int l = 0; l < c.num_hidden_layers; l++) {
        if ((rc = linear(m, m->w_qkv[l], m->h, AXQ_X_RMSNORM, m->norm_attn + (size_t)l * H, AXQ_Y_PLAIN, m->xn, nullptr, m->qkv)))
            return rc;
        for (int part = 0; part < 3; part++)
            if (const axq_weight *w = m->w_sep[part][l])
                if ((rc = linear(m, w, m->h, AXQ_X_RMSNORM, m->norm_attn + (size_t)l * H, AXQ_Y_PLAIN, m->xn, nullptr,
                                 m->qkv + qkv_part_offset(m, part))))
                    return rc;
        if (short_ctx) {
            launch_attn_rows(m, l, m->qkv, 1, 0, m->pos, 0, prompt_attn_lds(m, m->fused_max), m->att, st);
        } else {
            launch_attn_split(m, l, m->qkv, 1, m->att, st);
        }
        // residual adds go through the bias slot, in place
        if ((rc = linear(m, m->w_o[l], m->att, AXQ_X_PLAIN, nullptr, AXQ_Y_PLAIN, nullptr, m->h, m->h))) return rc;
        if ((rc = linear(m, m->w_gu[l], m->h, AXQ_X_RMSNORM, m->norm_ffn + (size_t)l * H, AXQ_Y_SWIGLU, m->xn, nullptr, m->act)))
            return rc;
        if ((rc = linear(m, m->w_down[l], m->act, AXQ_X_PLAIN, nullptr, AXQ_Y_PLAIN, nullptr, m->h, m->h))) return rc;
    }
    if ((rc = linear(m, m->w_head, m->h, AXQ_X_RMSNORM, m->norm_final, AXQ_Y_PLAIN, m->xn, nullptr, m->logits))) return rc;
    argmax_kernel<<<1, 1024, 0, st>>>(m->logits, c.vocab_size, m->next, m->pos);
    AXQ_LAUNCH_CHECK(ctx, "decode step");
    return AXQ_OK;
}

int check_ready(axq_model *m) {
    if ((!m->emb && !m->emb32) || !m->head_set) return axq_fail(m->ctx, AXQ_ERR_INVALID_DATA, "Invalid quantized data: embedding or lm_head not set");
    for (int l = 0; l < m->cfg.num_hidden_layers; l++)
        if (m->set_mask[l] != (1u << AXQ_LIN_COUNT) - 1)
            return axq_fail(m->ctx, AXQ_ERR_INVALID_DATA, "Invalid quantized data: layer %d has unset linears (mask %#x)", l,
                            m->set_mask[l]);
    return AXQ_OK;
}

// Captures the step into a graph on first use; later calls replay it.  pos: the position of the token being fed.
int run_step_graph(axq_model *m, int pos) {
    axq_ctx *ctx = m->ctx;
    const bool short_ctx = pos < m->fused_max;
    static const bool no_graph = getenv("AXQ_DECODE_GRAPH") && getenv("AXQ_DECODE_GRAPH")[0] == '0';
    if (no_graph) return enqueue_step(m, short_ctx); // development knob: plain launches instead of a graph replay
    hipGraphExec_t &exec = short_ctx ? m->graph_f : m->graph;
    bool &ok = short_ctx ? m->graph_f_ok : m->graph_ok;
    if (!ok) {
        hipGraph_t g = nullptr;
        AXQ_HIP(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal), AXQ_ERR_DRIVER);
        int rc = enqueue_step(m, short_ctx);
        hipError_t e = hipStreamEndCapture(ctx->stream, &g);
        if (rc) {
            if (g) (void)hipGraphDestroy(g);
            return rc;
        }
        if (e != hipSuccess) return axq_fail(ctx, AXQ_ERR_DRIVER, "hipStreamEndCapture: %s", hipGetErrorString(e));
        e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
        (void)hipGraphDestroy(g);
        if (e != hipSuccess) return axq_fail(ctx, AXQ_ERR_DRIVER, "hipGraphInstantiate: %s", hipGetErrorString(e));
        ok = true;
    }
    AXQ_HIP(ctx, hipGraphLaunch(exec, ctx->stream), AXQ_ERR_KERNEL_LAUNCH_FAILED);
    return AXQ_OK;
}

// One token: note it in the history, run the step, and when a sampler is set let it replace the step's argmax.
// The uniform variate of a draw comes from (seed, position), so a run is repeatable.
int run_token(axq_model *m, int pos) {
    axq_ctx *ctx = m->ctx;
    record_token_kernel<<<1, 1, 0, ctx->stream>>>(m->hist, m->pos, m->tok);
    int rc = run_step_graph(m, pos);
    if (rc || !m->sampling) return rc;
    return axq_dev_sample(ctx, m->logits, m->cfg.vocab_size, m->hist, m->pos, 0, &m->sampler, 0.f, m->pos, m->sample_seed,
                          m->sample_scratch, m->next, nullptr);
}

// Rows go through the layers several at a time: prompt tokens of one sequence at consecutive positions, or one token
// of each of several sequences (a batched step).  Up to PROMPT_BATCH rows use the small-batch GEMV (one pass over the
// weights for eight vectors), up to PROMPT_CHUNK the matrix-pipe GEMM on f32 activations once there are enough of
// them to fill its tiles.
constexpr int PROMPT_CHUNK = 2048;
constexpr int PROMPT_GEMM_MIN = 32;

// LDS of attn_prompt_kernel for queries up to position `last` (exclusive)
size_t prompt_attn_lds(const axq_model *m, int last) {
    int span = last;
    if (m->cfg.sliding_window > 0 && span > m->cfg.sliding_window) span = m->cfg.sliding_window;
    return (size_t)((span + 255) / 256 * 256) * sizeof(float);
}

// dst[b, 0 .. n) = src[b, 0 .. n) for rows of different lengths (n a multiple of 4; both sides 16-byte aligned).
__global__ void place_columns_kernel(const float *__restrict__ src, int n, float *__restrict__ dst, int dst_row) {
    const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 4, b = blockIdx.y;
    if (i < n) *reinterpret_cast<float4 *>(dst + (size_t)b * dst_row + i) = *reinterpret_cast<const float4 *>(src + (size_t)b * n + i);
}

enum RowsMode { ROWS_NONE = 0, ROWS_GEMV = 1, ROWS_GEMM = 2 };

// Whether `nb` rows ending before position `last` can go through the layers together in that mode: the scores of the
// longest query within LDS; for the GEMM every linear of the layers within its reach.  (The GEMV mode takes any
// weight: what the small-batch kernel does not cover goes row by row.)
bool rows_mode_covers(const axq_model *m, int mode, int last, int nb) {
    if (nb < 1 || prompt_attn_lds(m, last) > 128 * 1024) return false;
    if (mode == ROWS_GEMV) return nb <= PROMPT_BATCH;
    for (int l = 0; l < m->cfg.num_hidden_layers; l++)
        for (const axq_weight *w : {m->w_qkv[l], m->w_o[l], m->w_gu[l], m->w_down[l], m->w_sep[0][l], m->w_sep[1][l], m->w_sep[2][l]})
            if (w && !axq_dev_gemm_f32_covers(w, nb)) return false;
    return true;
}

bool all_layers_in_small_batch_reach(const axq_model *m, int nb) {
    if (nb < 2) return false;
    for (int l = 0; l < m->cfg.num_hidden_layers; l++)
        for (const axq_weight *w : {m->w_qkv[l], m->w_o[l], m->w_gu[l], m->w_down[l], m->w_sep[0][l], m->w_sep[1][l], m->w_sep[2][l]})
            if (w && !axq_dev_gemv_batch_covers(w, nb < PROMPT_BATCH ? nb : PROMPT_BATCH)) return false;
    return true;
}

template <class T>
hipError_t dev_alloc(T **p, size_t count);

// Activation rows for `cap` tokens (the model starts with PROMPT_BATCH of them).
int reserve_prompt_rows(axq_model *m, int cap) {
    if (cap <= m->pb_cap) return AXQ_OK;
    axq_ctx *ctx = m->ctx;
    const int H = m->cfg.hidden_size, I = m->cfg.intermediate_size;
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    // the batched step's graphs hold the old addresses
    if (m->graph_b_ok) (void)hipGraphExecDestroy(m->graph_b);
    if (m->graph_bf_ok) (void)hipGraphExecDestroy(m->graph_bf);
    m->graph_b_ok = m->graph_bf_ok = false;
    for (float **p : {&m->pb_h, &m->pb_qkv, &m->pb_att, &m->pb_gu, &m->pb_act}) {
        if (*p) (void)hipFree(*p);
        *p = nullptr;
    }
    m->pb_cap = 0;
    hipError_t e = dev_alloc(&m->pb_h, (size_t)cap * H);
    if (e == hipSuccess) e = dev_alloc(&m->pb_qkv, (size_t)cap * m->qkv_rows);
    if (e == hipSuccess) e = dev_alloc(&m->pb_att, (size_t)cap * m->q_dim);
    if (e == hipSuccess) e = dev_alloc(&m->pb_gu, (size_t)cap * 2 * I);
    if (e == hipSuccess) e = dev_alloc(&m->pb_act, (size_t)cap * I);
    if (e != hipSuccess) return axq_fail(ctx, AXQ_ERR_ALLOCATION_FAILED, "activations for %d rows: %s", cap, hipGetErrorString(e));
    m->pb_cap = cap;
    return AXQ_OK;
}

// What a call of enqueue_rows works on.
struct Rows {
    int mode;            // ROWS_GEMV or ROWS_GEMM
    const int32_t *toks; // [nb] device
    int nb;
    bool per_seq;        // false: rows pos0.. of sequence `seq`; true: row b is the next token of sequence seq + b
    int seq, pos0;
    size_t lds;          // of the attention kernel
    bool split_attn;     // per_seq: the positions split over workgroups and merged (long contexts) instead of one workgroup per head
};

template <int D, bool APPEND>
void launch_attn_rows_t(axq_model *m, int l, const float *qkv, int nb, int pos0, const int32_t *pos_arr, size_t cache_off, size_t lds,
                        float *att, hipStream_t st, PackOut pk) {
    const axq_model_config &c = m->cfg;
    static std::atomic<uint64_t> lds_allowed{0};
    if (lds > 48 * 1024) (void)axq_allow_lds(m->ctx, reinterpret_cast<const void *>(&attn_prompt_kernel<D, APPEND>), lds_allowed, 128 * 1024); // a
    // refusal is the context's error now, and the launch below fails with it
    const size_t off = (size_t)l * c.num_key_value_heads * c.max_position_embeddings * D + cache_off;
    attn_prompt_kernel<D, APPEND><<<dim3(c.num_attention_heads, nb), 1024, lds, st>>>(
        qkv, m->qkv_rows, m->rope_cos, m->rope_sin, m->kcache + off, m->vcache + off, pos0, pos_arr, m->seq_stride, c.num_attention_heads,
        c.num_key_value_heads, c.max_position_embeddings, c.sliding_window, att, pk);
}

// Attention of `nb` rows of layer l.  pos_arr == NULL: rows of one sequence (cache at cache_off) at positions pos0.., whose
// keys and values rope_append_kernel has put into the cache.  Otherwise row b belongs to sequence b at position
// pos_arr[b], and the kernel appends that row's key and value itself.
void launch_attn_rows(axq_model *m, int l, const float *qkv, int nb, int pos0, const int32_t *pos_arr, size_t cache_off, size_t lds,
                      float *att, hipStream_t st, PackOut pk) {
    const bool ap = pos_arr != nullptr;
    switch (m->cfg.head_dim) {
    case 32: ap ? launch_attn_rows_t<32, true>(m, l, qkv, nb, pos0, pos_arr, cache_off, lds, att, st, pk)
                : launch_attn_rows_t<32, false>(m, l, qkv, nb, pos0, pos_arr, cache_off, lds, att, st, pk); break;
    case 64: ap ? launch_attn_rows_t<64, true>(m, l, qkv, nb, pos0, pos_arr, cache_off, lds, att, st, pk)
                : launch_attn_rows_t<64, false>(m, l, qkv, nb, pos0, pos_arr, cache_off, lds, att, st, pk); break;
    case 128: ap ? launch_attn_rows_t<128, true>(m, l, qkv, nb, pos0, pos_arr, cache_off, lds, att, st, pk)
                 : launch_attn_rows_t<128, false>(m, l, qkv, nb, pos0, pos_arr, cache_off, lds, att, st, pk); break;
    default: ap ? launch_attn_rows_t<256, true>(m, l, qkv, nb, pos0, pos_arr, cache_off, lds, att, st, pk)
                : launch_attn_rows_t<256, false>(m, l, qkv, nb, pos0, pos_arr, cache_off, lds, att, st, pk); break;
    }
}

// The layers for `nb` rows (LLaMA::forward_with_cache on [batch, seq] input ids, llama.rs:731-762, for seq > 1 with
// batch 1, or batch > 1 with seq 1).  Prompt rows of one sequence leave what nb steps would leave in that sequence's KV
// cache, history and position counter, without the final norm and lm_head (generate never looks at the logits of
// prompt positions before the last, llama.rs:900-977).  A batched step goes on to the logits and the argmax of
// every sequence, as the one-token step does for one.
int enqueue_rows(axq_model *m, const Rows &r) {
    axq_ctx *ctx = m->ctx;
    const axq_model_config &c = m->cfg;
    hipStream_t st = ctx->stream;
    const int H = c.hidden_size, I = c.intermediate_size, d = c.head_dim, nb = r.nb;
    int rc;
    // y = f(x) W^T (+ resid): f = RMSNorm with weights aux, or SwiGLU over the gate/up rows in x, or nothing.  The
    // small-batch GEMV applies f while it packs x; elsewhere f runs as a kernel of its own (the GEMM normalises itself).
    // `next` (with RMSNorm weights next_aux): the linear that takes y next; where both are small-batch GEMVs, the first
    // one's reduction prepares the second one's operands, which then skips its own packing.
    const axq_weight *packed_for = nullptr; // the weight whose operands the GEMV scratch holds, if any
    auto lin = [&](const axq_weight *w, const float *x, int xmode, const float *aux, const float *resid, float *y, const axq_weight *next,
                   const float *next_aux) -> int {
        const bool batch_kernel = r.mode == ROWS_GEMV && axq_dev_gemv_batch_covers(w, nb);
        if (batch_kernel) {
            const bool ready = packed_for == w;
            const bool chain = next && axq_dev_gemv_batch_covers(next, nb);
            packed_for = chain ? next : nullptr;
            return axq_dev_gemv_batch_chain(ctx, w, x, ready ? AXQ_X_PACKED : xmode, aux, c.rms_norm_eps, nb, nullptr, resid, y,
                                            chain ? next : nullptr, chain ? next_aux : nullptr);
        }
        packed_for = nullptr;
        if (r.mode == ROWS_GEMM && xmode == AXQ_X_SWIGLU && axq_dev_gemm_f32_takes_swiglu(w)) // the GEMM's row pass applies SwiGLU itself
            return axq_dev_gemm_f32_ex(ctx, w, x, true, nb, nullptr, c.rms_norm_eps, nullptr, resid, y);
        if (xmode == AXQ_X_SWIGLU) {
            swiglu_kernel<<<dim3((I / 4 + 255) / 256, nb), 256, 0, st>>>(x, I, m->pb_act);
            x = m->pb_act;
        }
        if (r.mode == ROWS_GEMM)
            return axq_dev_gemm_f32(ctx, w, x, nb, xmode == AXQ_X_RMSNORM ? aux : nullptr, c.rms_norm_eps, nullptr, resid, y);
        if (xmode == AXQ_X_RMSNORM) {
            norm_kernel<<<nb, 1024, 0, st>>>(x, aux, (int)w->k, c.rms_norm_eps, m->pb_xn);
            x = m->pb_xn;
        }
        for (int b = 0; b < nb; b++) { // row by row, the residual row in the bias slot
            int e = axq_dev_gemv(ctx, w, x + (size_t)b * w->k, 1, resid ? resid + (size_t)b * w->n_rows : nullptr, y + (size_t)b * w->n_rows);
            if (e) return e;
        }
        return AXQ_OK;
    };
    const size_t seq_off = (size_t)r.seq * m->seq_stride;
    const int s0 = r.per_seq ? r.seq : 0; // per_seq: row b is sequence s0 + b
    if (r.per_seq) {
        record_rows_kernel<<<1, nb, 0, st>>>(m->hist + (size_t)s0 * c.max_position_embeddings, c.max_position_embeddings, m->pos + s0, r.toks);
    } else {
        int32_t *hist = m->hist + (size_t)r.seq * c.max_position_embeddings;
        for (int t0 = 0; t0 < nb; t0 += 1024) record_tokens_kernel<<<1, nb - t0 < 1024 ? nb - t0 : 1024, 0, st>>>(hist, r.pos0 + t0, r.toks + t0);
    }
    embed_kernel<<<dim3((H / 8 + 255) / 256, nb), 256, 0, st>>>(m->emb, m->emb32, r.toks, m->pb_h, H);
    for (int l = 0; l < c.num_hidden_layers; l++) {
        const size_t off = (size_t)l * c.num_key_value_heads * c.max_position_embeddings * d + seq_off;
        if ((rc = lin(m->w_qkv[l], m->pb_h, AXQ_X_RMSNORM, m->norm_attn + (size_t)l * H, nullptr, m->pb_qkv, nullptr, nullptr))) return rc;
        for (int part = 0; part < 3; part++)
            if (const axq_weight *w = m->w_sep[part][l]) { // through the gate/up rows (free until the feed-forward) into its columns of qkv
                if ((rc = lin(w, m->pb_h, AXQ_X_RMSNORM, m->norm_attn + (size_t)l * H, nullptr, m->pb_gu, nullptr, nullptr))) return rc;
                const int rows = (int)w->n_rows;
                place_columns_kernel<<<dim3((rows / 4 + 255) / 256, nb), 256, 0, st>>>(m->pb_gu, rows, m->pb_qkv + qkv_part_offset(m, part),
                                                                                       m->qkv_rows);
            }
        if (!r.per_seq)
            rope_append_kernel<<<dim3(c.num_key_value_heads, nb), d / 2, 0, st>>>(
                m->pb_qkv, m->qkv_rows, m->q_dim, m->kv_dim, m->rope_cos, m->rope_sin, m->kcache + off, m->vcache + off, r.pos0, nullptr,
                m->seq_stride, c.max_position_embeddings, d);
        // many rows of one sequence: attention on the matrix pipe, a tile of rows against every key once
        int on_mfma = 0;
        if (!r.per_seq && nb >= PROMPT_GEMM_MIN && m->attn_mfma) {
            on_mfma = axq_dev_attn_rows_mfma(ctx, m->pb_qkv, m->qkv_rows, m->rope_cos, m->rope_sin, m->kcache + off, m->vcache + off, r.pos0,
                                             nb, c.num_attention_heads, c.num_key_value_heads, d, c.max_position_embeddings,
                                             c.sliding_window, m->pb_att);
            if (on_mfma < 0) return on_mfma;
        }
        // where the output projection is a small-batch GEMV, the attention kernels leave its operands as well
        PackOut pk;
        if (!on_mfma && r.mode == ROWS_GEMV && axq_dev_gemv_batch_covers(m->w_o[l], nb)) {
            pk.even_odd = axq_dev_gemv_batch_operands(ctx, m->w_o[l], &pk.xa, &pk.xsg) ? 1 : 0;
            packed_for = m->w_o[l];
        }
        if (r.per_seq && r.split_attn) launch_attn_split(m, l, m->pb_qkv, nb, m->pb_att, st, pk, s0);
        else if (!on_mfma) launch_attn_rows(m, l, m->pb_qkv, nb, r.pos0, r.per_seq ? m->pos + s0 : nullptr, seq_off, r.lds, m->pb_att, st, pk);
        if ((rc = lin(m->w_o[l], m->pb_att, AXQ_X_PLAIN, nullptr, m->pb_h, m->pb_h, m->w_gu[l], m->norm_ffn + (size_t)l * H))) return rc;
        if ((rc = lin(m->w_gu[l], m->pb_h, AXQ_X_RMSNORM, m->norm_ffn + (size_t)l * H, nullptr, m->pb_gu, nullptr, nullptr))) return rc;
        if ((rc = lin(m->w_down[l], m->pb_gu, AXQ_X_SWIGLU, nullptr, m->pb_h, m->pb_h, l + 1 < c.num_hidden_layers ? m->w_qkv[l + 1] : nullptr,
                      m->norm_attn + (size_t)(l + 1 < c.num_hidden_layers ? l + 1 : l) * H))) return rc;
    }
    if (r.per_seq) {
        norm_kernel<<<nb, 1024, 0, st>>>(m->pb_h, m->norm_final, H, c.rms_norm_eps, m->pb_xn);
        float *logits = m->logits + (size_t)s0 * c.vocab_size;
        if ((rc = axq_dev_gemv(ctx, m->w_head, m->pb_xn, nb, nullptr, logits))) return rc;
        argmax_kernel<<<nb, 1024, 0, st>>>(logits, c.vocab_size, m->next + s0, m->pos + s0);
    } else {
        add_i32_kernel<<<1, 1, 0, st>>>(m->pos + r.seq, nb);
    }
    AXQ_LAUNCH_CHECK(ctx, "rows through the layers");
    return AXQ_OK;
}

// Feeds toks[0..n) (device memory) to sequence `seq` from position pos0 on as rows, several at a time; returns how many
// went in (all, unless the attention scores of so long a context do not fit LDS: then none from there on).
int feed_rows(axq_model *m, int seq, const int32_t *toks, int n, int pos0, int *fed) {
    static const char *knob = getenv("AXQ_PROMPT_BATCH"); // development knob: 0 = no rows at all, 1 = no GEMM
    const int allow = knob ? atoi(knob) : 2;
    int i = 0, rc;
    *fed = 0;
    while (allow >= 1 && i < n) {
        const int left = n - i;
        Rows r;
        r.mode = ROWS_NONE; r.toks = toks + i; r.per_seq = false; r.seq = seq; r.pos0 = pos0 + i; r.split_attn = false;
        // enough rows to fill GEMM tiles (fewer where the small-batch GEMV does not apply and single rows are the alternative)
        r.nb = left < m->prompt_chunk ? left : m->prompt_chunk;
        if (allow >= 2 && r.nb >= (all_layers_in_small_batch_reach(m, left) ? PROMPT_GEMM_MIN : PROMPT_BATCH) &&
            rows_mode_covers(m, ROWS_GEMM, r.pos0 + r.nb, r.nb))
            r.mode = ROWS_GEMM;
        if (r.mode == ROWS_NONE) {
            r.nb = left < PROMPT_BATCH ? left : PROMPT_BATCH;
            if (rows_mode_covers(m, ROWS_GEMV, r.pos0 + r.nb, r.nb)) r.mode = ROWS_GEMV;
        }
        if (r.mode == ROWS_NONE) break;
        r.lds = prompt_attn_lds(m, r.pos0 + r.nb);
        if ((rc = reserve_prompt_rows(m, r.nb))) return rc;
        if ((rc = enqueue_rows(m, r))) return rc;
        i += r.nb;
        *fed = i;
    }
    return AXQ_OK;
}

// Feeds prompt[0..n) (already in m->prompt) to sequence 0 from position base on: all but the last token as rows,
// the last (and whatever the rows could not take) by the one-token step, which also yields the logits.
int feed_prompt(axq_model *m, int base, int n_prompt) {
    axq_ctx *ctx = m->ctx;
    int i = 0, rc;
    if ((rc = feed_rows(m, 0, m->prompt, n_prompt - 1, base, &i))) return rc;
    for (; i < n_prompt && !rc; i++) {
        pick_prompt_kernel<<<1, 1, 0, ctx->stream>>>(m->prompt, m->pos, base, m->tok);
        rc = run_token(m, base + i);
    }
    return rc;
}

// One token of every sequence: graphs of their own, captured on first use.  max_pos_now: the largest position any
// sequence feeds a token at in this step (contexts beyond m->fused_max take the split form of the attention).
int run_batch_step(axq_model *m, int max_pos_now) {
    axq_ctx *ctx = m->ctx;
    Rows r;
    r.mode = ROWS_GEMV; r.toks = m->tok; r.nb = m->n_seq; r.per_seq = true; r.seq = 0; r.pos0 = 0;
    r.split_attn = max_pos_now >= m->fused_max;
    // sized for the longest context this form serves, so that the launch can sit in a graph
    r.lds = prompt_attn_lds(m, r.split_attn ? 1 : m->fused_max);
    static const bool no_graph = getenv("AXQ_DECODE_GRAPH") && getenv("AXQ_DECODE_GRAPH")[0] == '0';
    int rc;
    if (m->n_seq > PROMPT_BATCH && m->n_seq <= GEMV_GROUPS_MAX && all_layers_in_small_batch_reach(m, PROMPT_BATCH)) {
        // a few more rows than the small-batch GEMV takes: groups of eight sequences, one after the other (three passes
        // over the weights at 2.4 ms each still beat the GEMM's 8.5-10 ms at the 7B shape); plain launches
        rc = AXQ_OK;
        for (int s = 0; s < m->n_seq && !rc; s += PROMPT_BATCH) {
            Rows g = r;
            g.seq = s; g.toks = m->tok + s;
            g.nb = m->n_seq - s < PROMPT_BATCH ? m->n_seq - s : PROMPT_BATCH;
            rc = enqueue_rows(m, g);
        }
    } else if (m->n_seq > PROMPT_BATCH) {
        // many more: the linears are GEMMs on f32 rows (which size their scratch as they go, so no graph: a step of so
        // many rows is long against its launches anyway)
        r.mode = ROWS_GEMM;
        if (!rows_mode_covers(m, ROWS_GEMM, 1, r.nb))
            return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: more than %d sequences need linears the GEMM covers (K a multiple of 64)",
                            PROMPT_BATCH);
        if ((rc = reserve_prompt_rows(m, r.nb))) return rc;
        rc = enqueue_rows(m, r);
    } else if (no_graph) {
        rc = enqueue_rows(m, r);
    } else {
        hipGraphExec_t &exec = r.split_attn ? m->graph_b : m->graph_bf;
        bool &ok = r.split_attn ? m->graph_b_ok : m->graph_bf_ok;
        if (!ok) {
            hipGraph_t g = nullptr;
            AXQ_HIP(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal), AXQ_ERR_DRIVER);
            rc = enqueue_rows(m, r);
            hipError_t e = hipStreamEndCapture(ctx->stream, &g);
            if (rc) {
                if (g) (void)hipGraphDestroy(g);
                return rc;
            }
            if (e != hipSuccess) return axq_fail(ctx, AXQ_ERR_DRIVER, "hipStreamEndCapture: %s", hipGetErrorString(e));
            e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
            (void)hipGraphDestroy(g);
            if (e != hipSuccess) return axq_fail(ctx, AXQ_ERR_DRIVER, "hipGraphInstantiate: %s", hipGetErrorString(e));
            ok = true;
        }
        AXQ_HIP(ctx, hipGraphLaunch(exec, ctx->stream), AXQ_ERR_KERNEL_LAUNCH_FAILED);
        rc = AXQ_OK;
    }
    if (rc || !m->sampling) return rc;
    // one workgroup per sequence; the draw of sequence s comes from (seed + s * odd constant, position)
    return axq_dev_sample_rows(ctx, m->n_seq, m->logits, (size_t)m->cfg.vocab_size, m->cfg.vocab_size, m->hist,
                               (size_t)m->cfg.max_position_embeddings, m->pos, 0, &m->sampler, 0.f, m->pos, m->sample_seed,
                               0x9E3779B97F4A7C15ull, m->sample_scratch, m->next, nullptr);
}

template <class T>
hipError_t dev_alloc(T **p, size_t count) { return hipMalloc((void **)p, (count ? count : 1) * sizeof(T)); }

// The captured steps hold device addresses: whoever replaces a buffer they read drops them; the next step captures anew.
void invalidate_graphs(axq_model *m) {
    if (m->graph_ok) (void)hipGraphExecDestroy(m->graph);
    if (m->graph_f_ok) (void)hipGraphExecDestroy(m->graph_f);
    if (m->graph_b_ok) (void)hipGraphExecDestroy(m->graph_b);
    if (m->graph_bf_ok) (void)hipGraphExecDestroy(m->graph_bf);
    m->graph_ok = m->graph_f_ok = m->graph_b_ok = m->graph_bf_ok = false;
}

} // namespace

extern "C" {

int axq_model_create(axq_ctx *ctx, const axq_model_config *cfg, axq_model **out) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_model_create: NULL context");
    if (!cfg || !out) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_model_create: NULL pointer");
    *out = NULL;
    const axq_model_config &c = *cfg;
    if (c.vocab_size <= 0 || c.hidden_size <= 0 || c.intermediate_size <= 0 || c.num_hidden_layers < 0 ||
        c.num_attention_heads <= 0 || c.num_key_value_heads <= 0 || c.head_dim <= 0 || c.max_position_embeddings <= 0 ||
        c.sliding_window < 0)
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: model dimensions must be positive");
    if (c.num_attention_heads % c.num_key_value_heads != 0)
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: %d query heads are not a multiple of %d kv heads",
                        c.num_attention_heads, c.num_key_value_heads);
    if (c.hidden_size % 32 || c.intermediate_size % 32 ||
        (c.head_dim != 32 && c.head_dim != 64 && c.head_dim != 128 && c.head_dim != 256))
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH,
                        "Shape mismatch: hidden and intermediate sizes must be multiples of 32 and head_dim one of 32, 64, "
                        "128, 256");
    if (c.num_attention_heads / c.num_key_value_heads > ATT_MAX_REP)
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: at most %d query heads per KV head, got %d", ATT_MAX_REP,
                        c.num_attention_heads / c.num_key_value_heads);
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    axq_model *m = new (std::nothrow) axq_model();
    if (!m) return axq_fail(ctx, AXQ_ERR_ALLOCATION_FAILED, "out of host memory");
    m->ctx = ctx;
    m->cfg = c;
    m->q_dim = c.num_attention_heads * c.head_dim;
    m->kv_dim = c.num_key_value_heads * c.head_dim;
    m->qkv_rows = m->q_dim + 2 * m->kv_dim;
    m->max_splits = (c.max_position_embeddings + ATT_CHUNK - 1) / ATT_CHUNK;
    {
        const char *knob = getenv("AXQ_ATTN_FUSED_MAX"); // development knob: 0 = always split the positions
        // measured at the 7B shape: one sequence 660-680 against 642-660 tokens/s up to 224 positions, behind from 256 on;
        // batched steps (which share the threshold and the fused kernel's LDS sizing) still gain at 150, are even around 400
        m->fused_max = knob ? atoi(knob) : 240;
        if (m->fused_max > 32768) m->fused_max = 32768;
        m->attn_mfma = !(getenv("AXQ_ATTN_MFMA") && getenv("AXQ_ATTN_MFMA")[0] == '0');
        const char *chunk = getenv("AXQ_PROMPT_CHUNK"); // development knob: fewer prompt rows per pass (tests cross chunk borders with it)
        m->prompt_chunk = chunk ? atoi(chunk) : PROMPT_CHUNK;
        if (m->prompt_chunk < PROMPT_GEMM_MIN) m->prompt_chunk = PROMPT_GEMM_MIN;
        if (m->prompt_chunk > PROMPT_CHUNK) m->prompt_chunk = PROMPT_CHUNK;
    }
    m->n_seq = 1;
    m->seq_stride = (size_t)c.num_hidden_layers * c.num_key_value_heads * c.max_position_embeddings * c.head_dim;
    m->seq_pos.assign(1, 0);
    const int L = c.num_hidden_layers, H = c.hidden_size, I = c.intermediate_size;
    m->w_qkv.assign(L, nullptr); m->w_o.assign(L, nullptr); m->w_gu.assign(L, nullptr); m->w_down.assign(L, nullptr);
    for (auto &v : m->w_sep) v.assign(L, nullptr);
    m->set_mask.assign(L, 0);
    m->prompt_cap = c.max_position_embeddings;
    m->out_cap = c.max_position_embeddings;
    const size_t kv = (size_t)L * c.num_key_value_heads * c.max_position_embeddings * c.head_dim;
    hipError_t e = hipSuccess;
#define TRY(x) if (e == hipSuccess) e = (x)
    TRY(dev_alloc(&m->norm_attn, (size_t)L * H)); TRY(dev_alloc(&m->norm_ffn, (size_t)L * H)); TRY(dev_alloc(&m->norm_final, H));
    TRY(dev_alloc(&m->rope_cos, (size_t)c.max_position_embeddings * c.head_dim / 2));
    TRY(dev_alloc(&m->rope_sin, (size_t)c.max_position_embeddings * c.head_dim / 2));
    TRY(dev_alloc(&m->kcache, kv)); TRY(dev_alloc(&m->vcache, kv));
    TRY(dev_alloc(&m->h, H)); TRY(dev_alloc(&m->xn, H)); TRY(dev_alloc(&m->qkv, m->qkv_rows)); TRY(dev_alloc(&m->att, m->q_dim));
    m->part_stride = (size_t)c.num_key_value_heads * m->max_splits * (c.num_attention_heads / c.num_key_value_heads) * (c.head_dim + 2);
    TRY(dev_alloc(&m->att_part, m->part_stride));
    TRY(dev_alloc(&m->gu, (size_t)2 * I)); TRY(dev_alloc(&m->act, I)); TRY(dev_alloc(&m->logits, c.vocab_size));
    m->pb_cap = PROMPT_BATCH;
    TRY(dev_alloc(&m->pb_h, (size_t)PROMPT_BATCH * H)); TRY(dev_alloc(&m->pb_xn, (size_t)MAX_SEQUENCES * (H > I ? H : I))); // normalised rows in front of the lm_head and of linears outside the GEMV's reach
    TRY(dev_alloc(&m->pb_qkv, (size_t)PROMPT_BATCH * m->qkv_rows)); TRY(dev_alloc(&m->pb_att, (size_t)PROMPT_BATCH * m->q_dim));
    TRY(dev_alloc(&m->pb_gu, (size_t)PROMPT_BATCH * 2 * I)); TRY(dev_alloc(&m->pb_act, (size_t)PROMPT_BATCH * I));
    TRY(dev_alloc(&m->pos, 1)); TRY(dev_alloc(&m->tok, 1)); TRY(dev_alloc(&m->next, 1)); TRY(dev_alloc(&m->gen, 1));
    TRY(dev_alloc(&m->prompt, m->prompt_cap)); TRY(dev_alloc(&m->out, m->out_cap));
    TRY(dev_alloc(&m->hist, c.max_position_embeddings));
#undef TRY
    if (e != hipSuccess) {
        int rc = axq_fail(ctx, AXQ_ERR_ALLOCATION_FAILED, "model buffers: %s", hipGetErrorString(e));
        axq_model_free(m);
        return rc;
    }
    // unit norms by default (RMSNorm::new, llama.rs:150-156); zeroed cache and state
    size_t nn = (size_t)L * H;
    if (nn) fill_f32_kernel<<<(unsigned)((nn + 255) / 256), 256, 0, ctx->stream>>>(m->norm_attn, nn, 1.0f);
    if (nn) fill_f32_kernel<<<(unsigned)((nn + 255) / 256), 256, 0, ctx->stream>>>(m->norm_ffn, nn, 1.0f);
    fill_f32_kernel<<<(H + 255) / 256, 256, 0, ctx->stream>>>(m->norm_final, H, 1.0f);
    {
        hipError_t e = hipMemsetAsync(m->kcache, 0, kv * 2, ctx->stream);
        if (e == hipSuccess) e = hipMemsetAsync(m->vcache, 0, kv * 2, ctx->stream);
        if (e == hipSuccess) e = hipMemsetAsync(m->pos, 0, 4, ctx->stream);
        if (e == hipSuccess) e = hipMemsetAsync(m->gen, 0, 4, ctx->stream);
        if (e == hipSuccess) e = hipMemsetAsync(m->tok, 0, 4, ctx->stream);
        if (e != hipSuccess) {
            const int st = axq_fail(ctx, AXQ_ERR_DRIVER, "axq_model_create: clearing the cache and the counters: %s", hipGetErrorString(e));
            axq_model_free(m);
            return st;
        }
    }
    // RotaryEmbedding::new (llama.rs:223-252): inv_freq_i = 1 / theta^(2i/d), tables of cos/sin(pos * inv_freq_i)
    {
        const int half = c.head_dim / 2;
        std::vector<float> hc((size_t)c.max_position_embeddings * half), hs(hc.size());
        for (int i = 0; i < half; i++) {
            float inv_freq = 1.0f / powf(c.rope_theta, 2.0f * (float)i / (float)c.head_dim);
            for (int p = 0; p < c.max_position_embeddings; p++) {
                float angle = (float)p * inv_freq;
                hc[(size_t)p * half + i] = cosf(angle);
                hs[(size_t)p * half + i] = sinf(angle);
            }
        }
        e = hipMemcpyAsync(m->rope_cos, hc.data(), hc.size() * 4, hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess) e = hipMemcpyAsync(m->rope_sin, hs.data(), hs.size() * 4, hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) {
            int rc = axq_fail(ctx, AXQ_ERR_COPY_FAILED, "rope tables: %s", hipGetErrorString(e));
            axq_model_free(m);
            return rc;
        }
    }
    *out = m;
    return AXQ_OK;
}

void axq_model_free(axq_model *m) {
    if (!m) return;
    axq_ctx *ctx = m->ctx;
    (void)hipStreamSynchronize(ctx->stream);
    if (m->graph_ok) (void)hipGraphExecDestroy(m->graph);
    if (m->graph_f_ok) (void)hipGraphExecDestroy(m->graph_f);
    if (m->graph_b_ok) (void)hipGraphExecDestroy(m->graph_b);
    if (m->graph_bf_ok) (void)hipGraphExecDestroy(m->graph_bf);
    for (void *p : {(void *)m->bprompt, (void *)m->boffsets, (void *)m->bout})
        if (p) (void)hipFree(p);
    for (auto *w : m->w_qkv) axq_weight_free(ctx, w);
    for (auto &v : m->w_sep)
        for (auto *w : v) axq_weight_free(ctx, w);
    for (auto *w : m->w_o) axq_weight_free(ctx, w);
    for (auto *w : m->w_gu) axq_weight_free(ctx, w);
    for (auto *w : m->w_down) axq_weight_free(ctx, w);
    axq_weight_free(ctx, m->w_head);
    void *bufs[] = {m->emb, m->emb32, m->norm_attn, m->norm_ffn, m->norm_final, m->rope_cos, m->rope_sin, m->kcache, m->vcache, m->h,
                    m->xn, m->qkv, m->att, m->att_part, m->gu, m->act, m->logits, m->pos, m->tok,
                    m->next, m->gen, m->prompt, m->out, m->hist, m->sample_scratch, m->pb_h, m->pb_xn, m->pb_qkv, m->pb_att,
                    m->pb_gu, m->pb_act};
    for (void *p : bufs)
        if (p) (void)hipFree(p);
    delete m;
}

int axq_model_set_embedding_f16(axq_model *m, const uint16_t *table, int mem) {
    if (!m || !table) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    size_t n = (size_t)m->cfg.vocab_size * m->cfg.hidden_size;
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    if (m->emb32) { (void)hipFree(m->emb32); m->emb32 = nullptr; invalidate_graphs(m); } // the graphs hold the table's address
    if (!m->emb) { AXQ_HIP(ctx, dev_alloc(&m->emb, n), AXQ_ERR_ALLOCATION_FAILED); invalidate_graphs(m); }
    AXQ_HIP(ctx, hipMemcpyAsync(m->emb, table, n * 2, mem == AXQ_MEM_DEVICE ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice,
                                ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_model_set_embedding_f32(axq_model *m, const float *table, int mem) {
    if (!m || !table) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    size_t n = (size_t)m->cfg.vocab_size * m->cfg.hidden_size;
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    if (m->emb) { (void)hipFree(m->emb); m->emb = nullptr; invalidate_graphs(m); }
    if (!m->emb32) { AXQ_HIP(ctx, dev_alloc(&m->emb32, n), AXQ_ERR_ALLOCATION_FAILED); invalidate_graphs(m); }
    AXQ_HIP(ctx, hipMemcpyAsync(m->emb32, table, n * 4, mem == AXQ_MEM_DEVICE ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice,
                                ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_model_set_norm(axq_model *m, int layer, int which, const float *w, int mem) {
    if (!m || !w) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    const int H = m->cfg.hidden_size;
    if (layer >= m->cfg.num_hidden_layers || (layer >= 0 && (which < 0 || which > 1)))
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_model_set_norm: layer %d / which %d out of range", layer, which);
    float *dst = layer < 0 ? m->norm_final : (which == 0 ? m->norm_attn : m->norm_ffn) + (size_t)layer * H;
    AXQ_HIP(ctx, hipMemcpyAsync(dst, w, (size_t)H * 4, mem == AXQ_MEM_DEVICE ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice,
                                ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_model_set_linear(axq_model *m, int layer, int which, const axq_weight *w) {
    if (!m || !w) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    if (layer >= m->cfg.num_hidden_layers)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_model_set_linear: layer %d out of range", layer);
    int64_t rows, k;
    if (lin_dims(m, layer, which, &rows, &k))
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_model_set_linear: unknown linear %d", which);
    if (w->n_rows != rows || w->k != k)
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: expected [%lld, %lld], got [%lld, %lld]", (long long)rows,
                        (long long)k, (long long)w->n_rows, (long long)w->k);
    axq_weight **slot;
    int64_t slot_rows = rows, row_off = 0;
    if (layer < 0) {
        slot = &m->w_head;
    } else if (which <= AXQ_LIN_V) {
        slot = &m->w_qkv[layer];
        slot_rows = m->qkv_rows;
        row_off = which == AXQ_LIN_Q ? 0 : (which == AXQ_LIN_K ? m->q_dim : m->q_dim + m->kv_dim);
    } else if (which == AXQ_LIN_O) {
        slot = &m->w_o[layer];
    } else if (which == AXQ_LIN_DOWN) {
        slot = &m->w_down[layer];
    } else {
        slot = &m->w_gu[layer];
        slot_rows = 2 * (int64_t)m->cfg.intermediate_size;
        row_off = which == AXQ_LIN_GATE ? 0 : m->cfg.intermediate_size;
    }
    int rc;
    // a linear that has its slot to itself (o, down, lm_head) may come back in another block type: the slot is made anew
    if (*slot && (*slot)->type != w->type && slot_rows == rows) {
        AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
        axq_weight *fresh = nullptr;
        if ((rc = axq_weight_alloc(ctx, w->type, slot_rows, k, &fresh))) return rc;
        axq_weight_free(ctx, *slot);
        *slot = fresh;
        invalidate_graphs(m);
    }
    if (!*slot && (rc = axq_weight_alloc(ctx, w->type, slot_rows, k, slot))) return rc;
    const bool qkv_part = layer >= 0 && which <= AXQ_LIN_V;
    if (qkv_part && (m->w_sep[which][layer] || (*slot)->type != w->type)) {
        // the part's place in the fused weight is given up (a part of the fused weight's own type goes back into it)
        AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
        axq_weight_free(ctx, m->w_sep[which][layer]);
        m->w_sep[which][layer] = nullptr;
        invalidate_graphs(m);
    }
    if (qkv_part && (*slot)->type != w->type) {
        // q, k or v of another block type than the fused weight: kept apart (the fused weight's rows for it stay as they
        // are and are multiplied for nothing; whoever sets q first gives the fused weight q's type)
        if (rows % 4 != 0 || m->qkv_rows % 4 != 0)
            return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: q, k and v of different block types need row counts that are multiples of 4");
        axq_weight *sep = nullptr;
        if ((rc = axq_weight_alloc(ctx, w->type, rows, k, &sep))) return rc;
        if ((rc = copy_rows(ctx, sep, w, 0))) { axq_weight_free(ctx, sep); return rc; }
        if (hipStreamSynchronize(ctx->stream) != hipSuccess) {
            axq_weight_free(ctx, sep);
            return axq_fail(ctx, AXQ_ERR_DRIVER, "axq_model_set_linear: the copy of the weight did not complete");
        }
        m->w_sep[which][layer] = sep;
        m->set_mask[layer] |= 1u << which;
        return AXQ_OK;
    }
    if ((*slot)->type != w->type)
        return axq_fail(ctx, AXQ_ERR_INVALID_QUANT_TYPE, "Invalid quantization type: fused weight holds %s, got %s",
                        axq_type_name((*slot)->type), axq_type_name(w->type));
    const bool pair = layer >= 0 && (which == AXQ_LIN_GATE || which == AXQ_LIN_UP);
    if ((rc = pair ? copy_rows_interleaved(ctx, *slot, w, which == AXQ_LIN_UP) : copy_rows(ctx, *slot, w, row_off))) return rc;
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    if (layer < 0) m->head_set = true; else m->set_mask[layer] |= 1u << which;
    return AXQ_OK;
}

int axq_model_random_init(axq_model *m, int type, float std, uint64_t seed) {
    if (!m) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    const axq_model_config &c = m->cfg;
    size_t max_elems = (size_t)c.vocab_size * c.hidden_size;
    for (int which = 0; which < AXQ_LIN_COUNT; which++) {
        int64_t r, k;
        lin_dims(m, 0, which, &r, &k);
        if ((size_t)(r * k) > max_elems) max_elems = (size_t)(r * k);
    }
    float *tmp = nullptr;
    AXQ_HIP(ctx, dev_alloc(&tmp, max_elems), AXQ_ERR_ALLOCATION_FAILED);
    int rc = AXQ_OK;
    uint64_t s = seed;
    auto one = [&](int layer, int which) {
        int64_t r, k;
        lin_dims(m, layer, which, &r, &k);
        rc = axq_fill_normal_f32(ctx, tmp, (size_t)(r * k), 0.0f, std, 0.0f, 0.0f, ++s);
        axq_weight *w = nullptr;
        if (!rc) rc = axq_weight_quantize(ctx, type, r, k, tmp, AXQ_MEM_DEVICE, &w);
        if (!rc) rc = axq_model_set_linear(m, layer, which, w);
        axq_weight_free(ctx, w);
    };
    for (int l = 0; l < c.num_hidden_layers && !rc; l++)
        for (int which = 0; which < AXQ_LIN_COUNT && !rc; which++) one(l, which);
    if (!rc) one(-1, 0);
    if (!rc) {
        size_t n = (size_t)c.vocab_size * c.hidden_size;
        rc = axq_fill_normal_f32(ctx, tmp, n, 0.0f, std, 0.0f, 0.0f, ++s);
        if (!rc && m->emb32) { (void)hipFree(m->emb32); m->emb32 = nullptr; invalidate_graphs(m); }
        if (!rc && !m->emb) {
            if (dev_alloc(&m->emb, n) != hipSuccess) rc = axq_fail(ctx, AXQ_ERR_ALLOCATION_FAILED, "embedding");
            invalidate_graphs(m);
        }
        if (!rc) f32_to_f16_kernel<<<(unsigned)((n + 255) / 256), 256, 0, ctx->stream>>>(tmp, n, m->emb);
    }
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(tmp);
    return rc;
}

int axq_model_reset(axq_model *m) {
    if (!m) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    for (int s = 0; s < m->n_seq; s++) set_i32_kernel<<<1, 1, 0, ctx->stream>>>(m->pos + s, 0);
    set_i32_kernel<<<1, 1, 0, ctx->stream>>>(m->gen, 0);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    m->host_pos = 0;
    m->seq_pos.assign(m->n_seq, 0);
    return AXQ_OK;
}

int axq_model_truncate(axq_model *m, int n_positions) {
    if (!m) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    if (n_positions < 0 || n_positions > m->host_pos)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_model_truncate: %d positions asked, the cache holds %d", n_positions,
                        m->host_pos);
    set_i32_kernel<<<1, 1, 0, ctx->stream>>>(m->pos, n_positions);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    m->host_pos = n_positions;
    return AXQ_OK;
}

int axq_model_set_batch(axq_model *m, int n_seq) {
    if (!m) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    const axq_model_config &c = m->cfg;
    if (n_seq < 1 || n_seq > MAX_SEQUENCES)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_model_set_batch: 1 to %d sequences, got %d", MAX_SEQUENCES, n_seq);

    if (n_seq > 1 && (c.vocab_size % 4 != 0 || prompt_attn_lds(m, c.max_position_embeddings) > 128 * 1024))
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH,
                        "Shape mismatch: batched steps need a vocabulary that is a multiple of 4 and at most 32768 positions "
                        "(or a sliding window) per sequence");
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    // the graphs hold the old addresses
    if (m->graph_ok) (void)hipGraphExecDestroy(m->graph);
    if (m->graph_f_ok) (void)hipGraphExecDestroy(m->graph_f);
    if (m->graph_b_ok) (void)hipGraphExecDestroy(m->graph_b);
    if (m->graph_bf_ok) (void)hipGraphExecDestroy(m->graph_bf);
    m->graph_ok = m->graph_f_ok = m->graph_b_ok = m->graph_bf_ok = false;
    const size_t P = c.max_position_embeddings, S = (size_t)n_seq;
    for (void **p : {(void **)&m->kcache, (void **)&m->vcache, (void **)&m->pos, (void **)&m->tok, (void **)&m->next, (void **)&m->hist,
                     (void **)&m->logits, (void **)&m->bprompt, (void **)&m->boffsets, (void **)&m->bout, (void **)&m->att_part}) {
        if (*p) (void)hipFree(*p);
        *p = nullptr;
    }
    m->n_seq = 1; // what the pointers can back until everything below has worked
    hipError_t e = dev_alloc(&m->kcache, S * m->seq_stride);
    if (e == hipSuccess) e = dev_alloc(&m->vcache, S * m->seq_stride);
    if (e == hipSuccess) e = dev_alloc(&m->pos, S);
    if (e == hipSuccess) e = dev_alloc(&m->tok, S);
    if (e == hipSuccess) e = dev_alloc(&m->next, S);
    if (e == hipSuccess) e = dev_alloc(&m->hist, S * P);
    if (e == hipSuccess) e = dev_alloc(&m->logits, S * c.vocab_size);
    if (e == hipSuccess) e = dev_alloc(&m->bprompt, S * P);
    if (e == hipSuccess) e = dev_alloc(&m->boffsets, S + 1);
    if (e == hipSuccess) e = dev_alloc(&m->bout, S * m->out_cap);
    if (e == hipSuccess) e = dev_alloc(&m->att_part, S * m->part_stride);
    if (e == hipSuccess) e = hipMemsetAsync(m->kcache, 0, S * m->seq_stride * 2, ctx->stream);
    if (e == hipSuccess) e = hipMemsetAsync(m->vcache, 0, S * m->seq_stride * 2, ctx->stream);
    if (e == hipSuccess) e = hipMemsetAsync(m->pos, 0, S * 4, ctx->stream);
    if (e == hipSuccess) e = hipMemsetAsync(m->tok, 0, S * 4, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess)
        return axq_fail(ctx, AXQ_ERR_ALLOCATION_FAILED, "caches and state for %d sequences: %s (the model is unusable until a call of "
                        "axq_model_set_batch succeeds)", n_seq, hipGetErrorString(e));
    m->n_seq = n_seq;
    m->host_pos = 0;
    m->seq_pos.assign(n_seq, 0);
    if (m->sample_scratch) { // the sampler's scratch goes by sequences too
        (void)hipFree(m->sample_scratch);
        m->sample_scratch = nullptr;
        AXQ_HIP(ctx, hipMalloc(&m->sample_scratch, (size_t)n_seq * axq_sample_scratch_bytes(c.vocab_size)), AXQ_ERR_ALLOCATION_FAILED);
    }
    return AXQ_OK;
}

int axq_model_batch(const axq_model *m) { return m ? m->n_seq : -1; }

int axq_model_seq_len_of(const axq_model *m, int seq) {
    if (!m || seq < 0 || seq >= m->n_seq) return -1;
    return seq == 0 ? m->host_pos : m->seq_pos[seq];
}

int axq_model_copy_sequence(axq_model *m, int src, int dst) {
    if (!m) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    const axq_model_config &c = m->cfg;
    if (src < 0 || src >= m->n_seq || dst < 0 || dst >= m->n_seq)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_model_copy_sequence: sequences %d -> %d of %d", src, dst, m->n_seq);
    if (src == dst) return AXQ_OK;
    m->seq_pos[0] = m->host_pos;
    const int n = m->seq_pos[src];
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    if (n > 0) {
        // per (layer, kv head): the first n rows of max_pos
        const size_t pitch = (size_t)c.max_position_embeddings * c.head_dim * 2, width = (size_t)n * c.head_dim * 2;
        const size_t rows = (size_t)c.num_hidden_layers * c.num_key_value_heads;
        AXQ_HIP(ctx, hipMemcpy2DAsync(m->kcache + (size_t)dst * m->seq_stride, pitch, m->kcache + (size_t)src * m->seq_stride, pitch, width,
                                      rows, hipMemcpyDeviceToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
        AXQ_HIP(ctx, hipMemcpy2DAsync(m->vcache + (size_t)dst * m->seq_stride, pitch, m->vcache + (size_t)src * m->seq_stride, pitch, width,
                                      rows, hipMemcpyDeviceToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
        AXQ_HIP(ctx, hipMemcpyAsync(m->hist + (size_t)dst * c.max_position_embeddings, m->hist + (size_t)src * c.max_position_embeddings,
                                    (size_t)n * 4, hipMemcpyDeviceToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    }
    set_i32_kernel<<<1, 1, 0, ctx->stream>>>(m->pos + dst, n);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    m->seq_pos[dst] = n;
    m->host_pos = m->seq_pos[0];
    return AXQ_OK;
}

int axq_model_forward_batch(axq_model *m, const int32_t *tokens, float *logits, int32_t *next_tokens) {
    if (!m || !tokens) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    int rc;
    if ((rc = check_ready(m))) return rc;
    const int S = m->n_seq, V = m->cfg.vocab_size;
    m->seq_pos[0] = m->host_pos;
    for (int s = 0; s < S; s++) {
        if (tokens[s] < 0 || tokens[s] >= V)
            return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "token %d outside the vocabulary of %d", tokens[s], V);
        if (m->seq_pos[s] >= m->cfg.max_position_embeddings)
            return axq_fail(ctx, AXQ_ERR_OVERFLOW, "Numerical overflow during quantization: KV cache of sequence %d is full (%d positions)", s,
                            m->cfg.max_position_embeddings);
    }
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    AXQ_HIP(ctx, hipMemcpyAsync(m->tok, tokens, (size_t)S * 4, hipMemcpyHostToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    int max_pos_now = 0;
    for (int s = 0; s < S; s++) max_pos_now = m->seq_pos[s] > max_pos_now ? m->seq_pos[s] : max_pos_now;
    if ((rc = run_batch_step(m, max_pos_now))) return rc;
    for (int s = 0; s < S; s++) m->seq_pos[s]++;
    m->host_pos = m->seq_pos[0];
    if (logits)
        AXQ_HIP(ctx, hipMemcpyAsync(logits, m->logits, (size_t)S * V * 4, hipMemcpyDeviceToHost, ctx->stream), AXQ_ERR_COPY_FAILED);
    if (next_tokens)
        AXQ_HIP(ctx, hipMemcpyAsync(next_tokens, m->next, (size_t)S * 4, hipMemcpyDeviceToHost, ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_model_generate_batch(axq_model *m, const int32_t *prompts, const int32_t *offsets, int max_new_tokens, int32_t *out_tokens,
                             float *prefill_ms, float *decode_ms) {
    if (!m || !prompts || !offsets || !out_tokens) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    int rc;
    if ((rc = check_ready(m))) return rc;
    const int S = m->n_seq, P = m->cfg.max_position_embeddings;
    if (max_new_tokens < 1 || max_new_tokens > m->out_cap || offsets[0] != 0)
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: 1 to %d new tokens, offsets starting at 0", m->out_cap);
    for (int s = 0; s < S; s++) {
        const int n = offsets[s + 1] - offsets[s];
        if (n < 1) return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: prompt %d must hold at least one token", s);
        if (n + max_new_tokens - 1 > P)
            return axq_fail(ctx, AXQ_ERR_OVERFLOW, "Numerical overflow during quantization: %d + %d positions of sequence %d exceed the cache of %d",
                            n, max_new_tokens, s, P);
        for (int i = offsets[s]; i < offsets[s + 1]; i++)
            if (prompts[i] < 0 || prompts[i] >= m->cfg.vocab_size)
                return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "prompt token %d outside the vocabulary", prompts[i]);
    }
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    if ((rc = axq_model_reset(m))) return rc;
    if (!m->bprompt) { // a model that never saw axq_model_set_batch: one sequence
        hipError_t e = dev_alloc(&m->bprompt, (size_t)P);
        if (e == hipSuccess) e = dev_alloc(&m->boffsets, 2);
        if (e == hipSuccess) e = dev_alloc(&m->bout, (size_t)m->out_cap);
        if (e != hipSuccess) return axq_fail(ctx, AXQ_ERR_ALLOCATION_FAILED, "prompt buffers: %s", hipGetErrorString(e));
    }
    AXQ_HIP(ctx, hipMemcpyAsync(m->bprompt, prompts, (size_t)offsets[S] * 4, hipMemcpyHostToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipMemcpyAsync(m->boffsets, offsets, (size_t)(S + 1) * 4, hipMemcpyHostToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    hipEvent_t e0, e1, e2;
    AXQ_HIP(ctx, hipEventCreate(&e0), AXQ_ERR_DRIVER);
    AXQ_HIP(ctx, hipEventCreate(&e1), AXQ_ERR_DRIVER);
    AXQ_HIP(ctx, hipEventCreate(&e2), AXQ_ERR_DRIVER);
    (void)hipEventRecord(e0, ctx->stream);
    // every prompt but its last token, sequence by sequence; the last tokens are the input of the first batched step
    for (int s = 0; s < S && !rc; s++) {
        const int n = offsets[s + 1] - offsets[s] - 1;
        int fed = 0;
        rc = feed_rows(m, s, m->bprompt + offsets[s], n, 0, &fed);
        if (!rc && fed != n) rc = axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: prompt %d cannot go through the layers as rows", s);
    }
    if (!rc) last_tokens_kernel<<<1, S, 0, ctx->stream>>>(m->bprompt, m->boffsets, m->tok);
    (void)hipEventRecord(e1, ctx->stream);
    int longest = 0;
    for (int s = 0; s < S; s++) longest = offsets[s + 1] - offsets[s] > longest ? offsets[s + 1] - offsets[s] : longest;
    for (int i = 0; i < max_new_tokens && !rc; i++) {
        rc = run_batch_step(m, longest - 1 + i); // step i feeds sequence s its token at position n_s - 1 + i
        if (!rc) commit_rows_kernel<<<1, S, 0, ctx->stream>>>(m->next, m->tok, m->bout, i, m->out_cap);
    }
    (void)hipEventRecord(e2, ctx->stream);
    hipError_t e = hipStreamSynchronize(ctx->stream);
    float ms = 0.f;
    if (!rc && e == hipSuccess) {
        if (prefill_ms && hipEventElapsedTime(&ms, e0, e1) == hipSuccess) *prefill_ms = ms;
        if (decode_ms && hipEventElapsedTime(&ms, e1, e2) == hipSuccess) *decode_ms = ms;
    }
    (void)hipEventDestroy(e0); (void)hipEventDestroy(e1); (void)hipEventDestroy(e2);
    if (rc || e != hipSuccess) { // positions on the device may have moved: start over
        (void)axq_model_reset(m);
        return rc ? rc : axq_fail(ctx, AXQ_ERR_DRIVER, "generate: %s", hipGetErrorString(e));
    }
    for (int s = 0; s < S; s++) {
        m->seq_pos[s] = offsets[s + 1] - offsets[s] + max_new_tokens - 1;
        AXQ_HIP(ctx, hipMemcpy(out_tokens + (size_t)s * max_new_tokens, m->bout + (size_t)s * m->out_cap, (size_t)max_new_tokens * 4,
                               hipMemcpyDeviceToHost), AXQ_ERR_COPY_FAILED);
    }
    m->host_pos = m->seq_pos[0];
    return AXQ_OK;
}

int axq_model_set_sampling(axq_model *m, const axq_sampling_config *cfg, uint64_t seed) {
    if (!m) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    if (!cfg) { // back to the greedy argmax of the step itself
        m->sampling = false;
        return AXQ_OK;
    }
    int rc;
    if ((rc = axq_check_sampling_config(ctx, cfg))) return rc;
    if (!m->sample_scratch) // a row of scratch per sequence
        AXQ_HIP(ctx, hipMalloc(&m->sample_scratch, (size_t)m->n_seq * axq_sample_scratch_bytes(m->cfg.vocab_size)), AXQ_ERR_ALLOCATION_FAILED);
    m->sampler = *cfg;
    m->sample_seed = seed;
    m->sampling = true;
    return AXQ_OK;
}

int axq_model_seq_len(const axq_model *m) { return m ? m->host_pos : -1; }

int axq_model_read_kv(axq_model *m, int layer, int which, uint16_t *out) {
    if (!m || !out || layer < 0 || layer >= m->cfg.num_hidden_layers) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    size_t per_layer = (size_t)m->cfg.num_key_value_heads * m->cfg.max_position_embeddings * m->cfg.head_dim;
    const uint16_t *src = (which ? m->vcache : m->kcache) + (size_t)layer * per_layer;
    AXQ_HIP(ctx, hipMemcpyAsync(out, src, per_layer * 2, hipMemcpyDeviceToHost, ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_model_read_hidden(axq_model *m, float *hidden_out) {
    if (!m || !hidden_out) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    AXQ_HIP(ctx, hipMemcpyAsync(hidden_out, m->h, (size_t)m->cfg.hidden_size * 4, hipMemcpyDeviceToHost, ctx->stream),
            AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_model_forward(axq_model *m, int32_t token, float *logits, int32_t *next_token) {
    if (!m) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    int rc;
    if ((rc = check_ready(m))) return rc;
    if (token < 0 || token >= m->cfg.vocab_size)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "token %d outside the vocabulary of %d", token, m->cfg.vocab_size);
    if (m->host_pos >= m->cfg.max_position_embeddings)
        return axq_fail(ctx, AXQ_ERR_OVERFLOW, "Numerical overflow during quantization: KV cache is full (%d positions)",
                        m->cfg.max_position_embeddings);
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    set_i32_kernel<<<1, 1, 0, ctx->stream>>>(m->tok, token);
    if ((rc = run_token(m, m->host_pos))) return rc;
    m->host_pos++;
    if (logits)
        AXQ_HIP(ctx, hipMemcpyAsync(logits, m->logits, (size_t)m->cfg.vocab_size * 4, hipMemcpyDeviceToHost, ctx->stream),
                AXQ_ERR_COPY_FAILED);
    if (next_token)
        AXQ_HIP(ctx, hipMemcpyAsync(next_token, m->next, 4, hipMemcpyDeviceToHost, ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_model_forward_tokens(axq_model *m, const int32_t *tokens, int n, float *logits, int32_t *next_token) {
    if (!m || !tokens) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    int rc;
    if ((rc = check_ready(m))) return rc;
    if (n <= 0) return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: at least one token is needed");
    if (m->host_pos + n > m->cfg.max_position_embeddings || n > m->prompt_cap)
        return axq_fail(ctx, AXQ_ERR_OVERFLOW, "Numerical overflow during quantization: %d + %d positions exceed the cache of %d",
                        m->host_pos, n, m->cfg.max_position_embeddings);
    for (int i = 0; i < n; i++)
        if (tokens[i] < 0 || tokens[i] >= m->cfg.vocab_size)
            return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "token %d outside the vocabulary of %d", tokens[i], m->cfg.vocab_size);
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    AXQ_HIP(ctx, hipMemcpyAsync(m->prompt, tokens, (size_t)n * 4, hipMemcpyHostToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    rc = feed_prompt(m, m->host_pos, n);
    if (rc) { // the device-side position may have moved: bring both sides back to where the call started
        set_i32_kernel<<<1, 1, 0, ctx->stream>>>(m->pos, m->host_pos);
        (void)hipStreamSynchronize(ctx->stream);
        return rc;
    }
    m->host_pos += n;
    if (logits)
        AXQ_HIP(ctx, hipMemcpyAsync(logits, m->logits, (size_t)m->cfg.vocab_size * 4, hipMemcpyDeviceToHost, ctx->stream),
                AXQ_ERR_COPY_FAILED);
    if (next_token)
        AXQ_HIP(ctx, hipMemcpyAsync(next_token, m->next, 4, hipMemcpyDeviceToHost, ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_model_generate(axq_model *m, const int32_t *prompt, int n_prompt, int max_new_tokens, int32_t *out_tokens,
                       float *prefill_ms, float *decode_ms) {
    if (!m || !prompt || (max_new_tokens > 0 && !out_tokens)) return AXQ_ERR_INVALID_ARGUMENT;
    axq_ctx *ctx = m->ctx;
    int rc;
    if ((rc = check_ready(m))) return rc;
    if (n_prompt <= 0 || max_new_tokens < 0)
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: prompt must hold at least one token");
    if (m->host_pos + n_prompt + max_new_tokens - 1 > m->cfg.max_position_embeddings || n_prompt > m->prompt_cap ||
        max_new_tokens > m->out_cap)
        return axq_fail(ctx, AXQ_ERR_OVERFLOW, "Numerical overflow during quantization: %d + %d + %d positions exceed the cache of %d",
                        m->host_pos, n_prompt, max_new_tokens, m->cfg.max_position_embeddings);
    for (int i = 0; i < n_prompt; i++)
        if (prompt[i] < 0 || prompt[i] >= m->cfg.vocab_size)
            return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "prompt token %d outside the vocabulary", prompt[i]);
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    AXQ_HIP(ctx, hipMemcpyAsync(m->prompt, prompt, (size_t)n_prompt * 4, hipMemcpyHostToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    set_i32_kernel<<<1, 1, 0, ctx->stream>>>(m->gen, 0);
    const int base = m->host_pos;
    hipEvent_t e0, e1, e2;
    AXQ_HIP(ctx, hipEventCreate(&e0), AXQ_ERR_DRIVER);
    AXQ_HIP(ctx, hipEventCreate(&e1), AXQ_ERR_DRIVER);
    AXQ_HIP(ctx, hipEventCreate(&e2), AXQ_ERR_DRIVER);
    (void)hipEventRecord(e0, ctx->stream);
    // prompt: up to eight tokens per pass over the weights, the last one by the step that also yields logits
    rc = feed_prompt(m, base, n_prompt);
    (void)hipEventRecord(e1, ctx->stream);
    // generation: the argmax of step i is the input of step i+1, on the device
    for (int i = 0; i < max_new_tokens && !rc; i++) {
        commit_next_kernel<<<1, 1, 0, ctx->stream>>>(m->next, m->tok, m->gen, m->out, m->out_cap);
        if (i + 1 < max_new_tokens) rc = run_token(m, base + n_prompt + i);
    }
    (void)hipEventRecord(e2, ctx->stream);
    hipError_t e = hipStreamSynchronize(ctx->stream);
    float ms = 0.f;
    if (!rc && e == hipSuccess) {
        if (prefill_ms && hipEventElapsedTime(&ms, e0, e1) == hipSuccess) *prefill_ms = ms;
        if (decode_ms && hipEventElapsedTime(&ms, e1, e2) == hipSuccess) *decode_ms = ms;
    }
    (void)hipEventDestroy(e0); (void)hipEventDestroy(e1); (void)hipEventDestroy(e2);
    if (rc || e != hipSuccess) { // the device-side position may have moved: bring both sides back to where the call started
        set_i32_kernel<<<1, 1, 0, ctx->stream>>>(m->pos, base);
        (void)hipStreamSynchronize(ctx->stream);
        return rc ? rc : axq_fail(ctx, AXQ_ERR_DRIVER, "generate: %s", hipGetErrorString(e));
    }
    m->host_pos = base + n_prompt + (max_new_tokens > 0 ? max_new_tokens - 1 : 0);
    if (max_new_tokens > 0)
        AXQ_HIP(ctx, hipMemcpy(out_tokens, m->out, (size_t)max_new_tokens * 4, hipMemcpyDeviceToHost), AXQ_ERR_COPY_FAILED);
    return AXQ_OK;
}

} // extern "C"
