// Decode-path quantized matmul: y[b, n] = sum_k x[b, k] * W[n, k] (+ bias[n]).
//
// This fuses the reference composition dequantize_tensor -> transpose ->
// sgemm (crates/axonml-quant/src/dequantize.rs:34-54,
// crates/axonml-tensor/src/tensor.rs:1020-1045,
// crates/axonml-core/src/backends/cpu.rs:566-598) into one pass over the packed
// weight bytes.  The kernel is HBM-bound: every weight byte is read once.
//
// Work decomposition (wave64):
//   - A lane owns a fixed K-range ("chunk": one 16-byte vector of codes, two for
//     Q4_K) for the whole kernel, so its slice of x is loaded once into VGPRs
//     and reused for every row the wave visits.
//   - 64 consecutive chunks form a wave "slice"; S = ceil(chunks_per_row / 64)
//     waves of a workgroup cover one row together (split-K), G groups of S
//     waves share a workgroup, each group walks R rows.
//   - Per row a lane issues 128-bit loads of codes (fully coalesced: lane
//     stride 16 B) plus its block's scale data, unpacks in registers and
//     accumulates; the 64 partial sums are folded with DPP row shifts and row
//     broadcasts; the S slice totals are added in a fixed order through LDS
//     (no atomics: results are run-to-run identical).
//   - U rows are in flight per lane at a time to keep enough HBM requests
//     outstanding.
#include <hip/hip_fp16.h>

#include <stdlib.h>

#include "axq_internal.h"

namespace {

struct GemvArgs {
    const uint8_t *codes, *meta, *qh;
    size_t codes_pitch, meta_pitch, qh_pitch;
    const float *x, *bias;
    float *y;
    int n_rows;
    int cpr;     // chunks per row
    int S, G, R; // slices per row, row groups per workgroup, rows per group
    int npass;   // > 1 when a lane must visit several chunks per row
    float fp8_unit_inv;
};

typedef float float2v __attribute__((ext_vector_type(2)));

__device__ inline float f16_bits_to_f32(uint32_t h) { return __half2float(__ushort_as_half((unsigned short)h)); }

__device__ inline float ubyte0(uint32_t v) { float r; asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(r) : "v"(v)); return r; }
__device__ inline float ubyte1(uint32_t v) { float r; asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(r) : "v"(v)); return r; }
__device__ inline float ubyte2(uint32_t v) { float r; asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(r) : "v"(v)); return r; }
__device__ inline float ubyte3(uint32_t v) { float r; asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(r) : "v"(v)); return r; }

// Sum over the 64 lanes of a wave; the total is valid in lane 63.
template <int CTRL, int ROW_MASK, bool BOUND>
__device__ inline float dpp_add(float v) {
    int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, BOUND);
    return v + __builtin_bit_cast(float, t);
}
__device__ inline float wave_sum_lane63(float v) {
    v = dpp_add<0x111, 0xf, true>(v); // row_shr:1
    v = dpp_add<0x112, 0xf, true>(v); // row_shr:2
    v = dpp_add<0x114, 0xf, true>(v); // row_shr:4
    v = dpp_add<0x118, 0xf, true>(v); // row_shr:8  -> lane 15 of each row holds the row total
    v = dpp_add<0x142, 0xa, false>(v); // row_bcast:15 into rows 1 and 3
    v = dpp_add<0x143, 0xc, false>(v); // row_bcast:31 into rows 2 and 3
    return v;
}

// The four bytes of `v` must each hold a value 0..15.  v_cvt_pk_f32_fp8 turns
// such a byte n into n * unit (the 8-bit float with a 3-bit mantissa is linear
// over 0..15), two bytes per instruction; x has been pre-multiplied by 1/unit.
// `c` = 8 * unit: the codes are centred (n - 8) before the multiply so that no large sums cancel later.
__device__ inline void fma_nibbles4(uint32_t v, const float *xs, float c, float &acc) {
    float2v a = __builtin_amdgcn_cvt_pk_f32_fp8((int)v, false);
    float2v b = __builtin_amdgcn_cvt_pk_f32_fp8((int)v, true);
    acc = fmaf(a[0] - c, xs[0], acc);
    acc = fmaf(a[1] - c, xs[1], acc);
    acc = fmaf(b[0] - c, xs[2], acc);
    acc = fmaf(b[1] - c, xs[3], acc);
}

// ---------------------------------------------------------------------------
// Per-type traits.  W = weights per chunk; X holds what a lane keeps of x;
// Raw what it loads per row; load() issues the loads; dot() folds them.
// ---------------------------------------------------------------------------
struct Q4K {
    static constexpr int W = 64;
    struct X { float xs[64]; float sum_lo, sum_hi; };
    struct Raw { uint4 q0, q1, h; };
    template <class F>
    __device__ static void set_x(const GemvArgs &a, F fetch, X &o) {
        float lo = 0.f, hi = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            float4 v = fetch(i);
            float s = (v.x + v.y) + (v.z + v.w);
            if (i < 8) lo += s; else hi += s;
            o.xs[4 * i] = v.x * a.fp8_unit_inv; o.xs[4 * i + 1] = v.y * a.fp8_unit_inv;
            o.xs[4 * i + 2] = v.z * a.fp8_unit_inv; o.xs[4 * i + 3] = v.w * a.fp8_unit_inv;
        }
        o.sum_lo = lo; o.sum_hi = hi;
    }
    __device__ static void load(const GemvArgs &a, int row, int chunk, Raw &r) {
        // chunk = pair index in the row; slice = chunk / 64; P = pairs in this slice
        int slice = chunk >> 6, lane_pair = chunk & 63;
        int P = a.cpr - (slice << 6);
        P = P < 64 ? P : 64;
        const uint8_t *base = a.codes + (size_t)row * a.codes_pitch + (size_t)slice * 2048 + (size_t)lane_pair * 16;
        r.q0 = *reinterpret_cast<const uint4 *>(base);
        r.q1 = *reinterpret_cast<const uint4 *>(base + (size_t)P * 16);
        r.h = *reinterpret_cast<const uint4 *>(a.meta + (size_t)row * a.meta_pitch + (size_t)(chunk >> 2) * 16);
    }
    __device__ static float dot(const GemvArgs &a, const Raw &r, const X &x, int chunk) {
        const float c8 = 8.0f / a.fp8_unit_inv;
        int p = chunk & 3;
        // 6-bit scale/min of sub-blocks 2p and 2p+1 (ggml get_scale_min_k4 order)
        int sh = (p & 1) * 16;
        uint32_t ya = r.h.y >> sh, za = r.h.z >> sh, wa = r.h.w >> sh;
        uint32_t scp, mp;
        if (p < 2) {
            scp = ya & 0x3F3F;
            mp = za & 0x3F3F;
        } else {
            scp = (wa & 0x0F0F) | ((ya >> 2) & 0x3030);
            mp = ((wa >> 4) & 0x0F0F) | ((za >> 2) & 0x3030);
        }
        float d = f16_bits_to_f32(r.h.x & 0xFFFF), dmin = f16_bits_to_f32(r.h.x >> 16);
        float alo0 = 0.f, alo1 = 0.f, ahi0 = 0.f, ahi1 = 0.f;
        const uint32_t q0[4] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w};
        const uint32_t q1[4] = {r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
        for (int w = 0; w < 4; w++) {
            // first half of the pair: bytes 4w..4w+3 -> elements 4w.. (low), 32+4w.. (high)
            fma_nibbles4(q0[w] & 0x0F0F0F0Fu, &x.xs[4 * w], c8, alo0);
            fma_nibbles4((q0[w] >> 4) & 0x0F0F0F0Fu, &x.xs[32 + 4 * w], c8, ahi0);
            // second half: bytes 16+4w.. -> elements 16+4w.. (low), 48+4w.. (high)
            fma_nibbles4(q1[w] & 0x0F0F0F0Fu, &x.xs[16 + 4 * w], c8, alo1);
            fma_nibbles4((q1[w] >> 4) & 0x0F0F0F0Fu, &x.xs[48 + 4 * w], c8, ahi1);
        }
        float s0 = d * ubyte0(scp), s1 = d * ubyte1(scp);
        float y = fmaf(s0, alo0 + alo1, s1 * (ahi0 + ahi1)); // sum d*sc*(q - 8)*x
        y = fmaf(fmaf(8.0f, s0, -(dmin * ubyte0(mp))), x.sum_lo, y);
        y = fmaf(fmaf(8.0f, s1, -(dmin * ubyte1(mp))), x.sum_hi, y);
        return y;
    }
};

template <bool WITH_MIN>
struct Q4x { // Q4_0 / Q4_1: adjacent-pair nibble order (types.rs:179-198)
    static constexpr int W = 32;
    struct X { float xs[32]; float sum; };
    struct Raw { uint4 q; uint32_t m; };
    template <class F>
    __device__ static void set_x(const GemvArgs &a, F fetch, X &o) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float4 v = fetch(i);
            s += (v.x + v.y) + (v.z + v.w);
            o.xs[4 * i] = v.x * a.fp8_unit_inv; o.xs[4 * i + 1] = v.y * a.fp8_unit_inv;
            o.xs[4 * i + 2] = v.z * a.fp8_unit_inv; o.xs[4 * i + 3] = v.w * a.fp8_unit_inv;
        }
        o.sum = s;
    }
    __device__ static void load(const GemvArgs &a, int row, int chunk, Raw &r) {
        r.q = *reinterpret_cast<const uint4 *>(a.codes + (size_t)row * a.codes_pitch + (size_t)chunk * 16);
        const uint8_t *m = a.meta + (size_t)row * a.meta_pitch;
        if (WITH_MIN) r.m = *reinterpret_cast<const uint32_t *>(m + (size_t)chunk * 4);
        else r.m = *reinterpret_cast<const uint16_t *>(m + (size_t)chunk * 2);
    }
    __device__ static float dot(const GemvArgs &a, const Raw &r, const X &x, int) {
        const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
        const float c8 = 8.0f / a.fp8_unit_inv;
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            // dword w: nibble j = element 8w + j; even elements sit in the low nibbles
            uint32_t lo = q[w] & 0x0F0F0F0Fu, hi = (q[w] >> 4) & 0x0F0F0F0Fu;
            float2v la = __builtin_amdgcn_cvt_pk_f32_fp8((int)lo, false), lb = __builtin_amdgcn_cvt_pk_f32_fp8((int)lo, true);
            float2v ha = __builtin_amdgcn_cvt_pk_f32_fp8((int)hi, false), hb = __builtin_amdgcn_cvt_pk_f32_fp8((int)hi, true);
            const float *xs = &x.xs[8 * w];
            a0 = fmaf(la[0] - c8, xs[0], a0); a1 = fmaf(ha[0] - c8, xs[1], a1);
            a0 = fmaf(la[1] - c8, xs[2], a0); a1 = fmaf(ha[1] - c8, xs[3], a1);
            a0 = fmaf(lb[0] - c8, xs[4], a0); a1 = fmaf(hb[0] - c8, xs[5], a1);
            a0 = fmaf(lb[1] - c8, xs[6], a0); a1 = fmaf(hb[1] - c8, xs[7], a1);
        }
        float scale = f16_bits_to_f32(r.m & 0xFFFF);
        float acc = a0 + a1; // sum (n - 8) x
        if (WITH_MIN) return fmaf(scale, acc, fmaf(8.0f, scale, f16_bits_to_f32(r.m >> 16)) * x.sum);
        return scale * acc;
    }
};

template <bool WITH_MIN>
struct Q5x { // Q5_0 / Q5_1: byte j = elements j (low nibble) and j+16 (high); qh bit e = bit 4 of element e
    static constexpr int W = 32;
    struct X { float xs[32]; float sum; };
    struct Raw { uint4 q; uint32_t qh; uint32_t m; };
    template <class F>
    __device__ static void set_x(const GemvArgs &, F fetch, X &o) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float4 v = fetch(i);
            s += (v.x + v.y) + (v.z + v.w);
            o.xs[4 * i] = v.x; o.xs[4 * i + 1] = v.y; o.xs[4 * i + 2] = v.z; o.xs[4 * i + 3] = v.w;
        }
        o.sum = s;
    }
    __device__ static void load(const GemvArgs &a, int row, int chunk, Raw &r) {
        r.q = *reinterpret_cast<const uint4 *>(a.codes + (size_t)row * a.codes_pitch + (size_t)chunk * 16);
        r.qh = *reinterpret_cast<const uint32_t *>(a.qh + (size_t)row * a.qh_pitch + (size_t)chunk * 4);
        const uint8_t *m = a.meta + (size_t)row * a.meta_pitch;
        if (WITH_MIN) r.m = *reinterpret_cast<const uint32_t *>(m + (size_t)chunk * 4);
        else r.m = *reinterpret_cast<const uint16_t *>(m + (size_t)chunk * 2);
    }
    __device__ static float dot(const GemvArgs &, const Raw &r, const X &x, int) {
        const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            // spread 4 bits of qh to bit 4 of each byte: t * 0x00204081 puts bit i at bit 8i
            uint32_t bl = (((r.qh >> (4 * w)) & 0xFu) * 0x00204081u) & 0x01010101u;
            uint32_t bh = (((r.qh >> (16 + 4 * w)) & 0xFu) * 0x00204081u) & 0x01010101u;
            uint32_t lo = (q[w] & 0x0F0F0F0Fu) | (bl << 4);
            uint32_t hi = ((q[w] >> 4) & 0x0F0F0F0Fu) | (bh << 4);
            const float *xl = &x.xs[4 * w], *xh = &x.xs[16 + 4 * w];
            a0 = fmaf(ubyte0(lo) - 16.0f, xl[0], a0); a1 = fmaf(ubyte0(hi) - 16.0f, xh[0], a1);
            a0 = fmaf(ubyte1(lo) - 16.0f, xl[1], a0); a1 = fmaf(ubyte1(hi) - 16.0f, xh[1], a1);
            a0 = fmaf(ubyte2(lo) - 16.0f, xl[2], a0); a1 = fmaf(ubyte2(hi) - 16.0f, xh[2], a1);
            a0 = fmaf(ubyte3(lo) - 16.0f, xl[3], a0); a1 = fmaf(ubyte3(hi) - 16.0f, xh[3], a1);
        }
        float d = f16_bits_to_f32(r.m & 0xFFFF);
        float acc = a0 + a1; // sum (u - 16) x
        if (WITH_MIN) return fmaf(d, acc, fmaf(16.0f, d, f16_bits_to_f32(r.m >> 16)) * x.sum);
        return d * acc;
    }
};

struct Q80 { // chunk = 16 int8 = half a block
    static constexpr int W = 16;
    struct X { float xs[16]; };
    struct Raw { uint4 q; uint32_t m; };
    template <class F>
    __device__ static void set_x(const GemvArgs &, F fetch, X &o) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float4 v = fetch(i);
            o.xs[4 * i] = v.x; o.xs[4 * i + 1] = v.y; o.xs[4 * i + 2] = v.z; o.xs[4 * i + 3] = v.w;
        }
    }
    __device__ static void load(const GemvArgs &a, int row, int chunk, Raw &r) {
        r.q = *reinterpret_cast<const uint4 *>(a.codes + (size_t)row * a.codes_pitch + (size_t)chunk * 16);
        r.m = *reinterpret_cast<const uint16_t *>(a.meta + (size_t)row * a.meta_pitch + (size_t)(chunk >> 1) * 2);
    }
    __device__ static float dot(const GemvArgs &, const Raw &r, const X &x, int) {
        const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            int v = (int)q[w];
            a0 = fmaf((float)(signed char)(v), x.xs[4 * w], a0);
            a1 = fmaf((float)(signed char)(v >> 8), x.xs[4 * w + 1], a1);
            a0 = fmaf((float)(signed char)(v >> 16), x.xs[4 * w + 2], a0);
            a1 = fmaf((float)(v >> 24), x.xs[4 * w + 3], a1);
        }
        return f16_bits_to_f32(r.m) * (a0 + a1);
    }
};

struct Q5K { // GGUF Q5_K; chunk = one pair of sub-blocks (64 elements): Q4_K's codes and header, the fifth bits from the qh plane
    static constexpr int W = 64;
    struct X { float xs[64]; };
    struct Raw { uint4 q0, q1, h, b0, b1; };
    template <class F>
    __device__ static void set_x(const GemvArgs &, F fetch, X &o) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            float4 v = fetch(i);
            o.xs[4 * i] = v.x; o.xs[4 * i + 1] = v.y; o.xs[4 * i + 2] = v.z; o.xs[4 * i + 3] = v.w;
        }
    }
    __device__ static void load(const GemvArgs &a, int row, int chunk, Raw &r) {
        int slice = chunk >> 6, lane_pair = chunk & 63;
        int P = a.cpr - (slice << 6);
        P = P < 64 ? P : 64;
        const uint8_t *base = a.codes + (size_t)row * a.codes_pitch + (size_t)slice * 2048 + (size_t)lane_pair * 16;
        r.q0 = *reinterpret_cast<const uint4 *>(base);
        r.q1 = *reinterpret_cast<const uint4 *>(base + (size_t)P * 16);
        r.h = *reinterpret_cast<const uint4 *>(a.meta + (size_t)row * a.meta_pitch + (size_t)(chunk >> 2) * 16);
        const uint4 *qh = reinterpret_cast<const uint4 *>(a.qh + (size_t)row * a.qh_pitch + (size_t)(chunk >> 2) * 32);
        r.b0 = qh[0]; // byte l: bit 2 p + h = fifth bit of element l of sub-block 2 p + h
        r.b1 = qh[1];
    }
    __device__ static float dot(const GemvArgs &, const Raw &r, const X &x, int chunk) {
        const int p = chunk & 3;
        const int sh = (p & 1) * 16;
        const uint32_t ya = r.h.y >> sh, za = r.h.z >> sh, wa = r.h.w >> sh;
        uint32_t scp, mp;
        if (p < 2) {
            scp = ya & 0x3F3F;
            mp = za & 0x3F3F;
        } else {
            scp = (wa & 0x0F0F) | ((ya >> 2) & 0x3030);
            mp = ((wa >> 4) & 0x0F0F) | ((za >> 2) & 0x3030);
        }
        const float d = f16_bits_to_f32(r.h.x & 0xFFFF), dmin = f16_bits_to_f32(r.h.x >> 16);
        const uint32_t q[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
        const uint32_t b[8] = {r.b0.x, r.b0.y, r.b0.z, r.b0.w, r.b1.x, r.b1.y, r.b1.z, r.b1.w};
        float lo = 0.f, hi = 0.f, slo = 0.f, shi = 0.f;
#pragma unroll
        for (int w = 0; w < 8; w++) { // bytes 4 w ..: elements 4 w .. of the low sub-block, 32 + 4 w .. of the high one
            const uint32_t ul = (q[w] & 0x0F0F0F0Fu) | (((b[w] >> (2 * p)) & 0x01010101u) << 4);
            const uint32_t uh = ((q[w] >> 4) & 0x0F0F0F0Fu) | (((b[w] >> (2 * p + 1)) & 0x01010101u) << 4);
            // codes centred (u - 16) before the multiply: no large sums cancel for an x with a mean
            lo = fmaf(ubyte0(ul) - 16.0f, x.xs[4 * w], lo);      hi = fmaf(ubyte0(uh) - 16.0f, x.xs[32 + 4 * w], hi);
            lo = fmaf(ubyte1(ul) - 16.0f, x.xs[4 * w + 1], lo);  hi = fmaf(ubyte1(uh) - 16.0f, x.xs[32 + 4 * w + 1], hi);
            lo = fmaf(ubyte2(ul) - 16.0f, x.xs[4 * w + 2], lo);  hi = fmaf(ubyte2(uh) - 16.0f, x.xs[32 + 4 * w + 2], hi);
            lo = fmaf(ubyte3(ul) - 16.0f, x.xs[4 * w + 3], lo);  hi = fmaf(ubyte3(uh) - 16.0f, x.xs[32 + 4 * w + 3], hi);
            slo += (x.xs[4 * w] + x.xs[4 * w + 1]) + (x.xs[4 * w + 2] + x.xs[4 * w + 3]);
            shi += (x.xs[32 + 4 * w] + x.xs[32 + 4 * w + 1]) + (x.xs[32 + 4 * w + 2] + x.xs[32 + 4 * w + 3]);
        }
        const float s0 = d * ubyte0(scp), s1 = d * ubyte1(scp);
        float y = fmaf(s0, lo, s1 * hi); // sum d * sc * (u - 16) * x
        y = fmaf(fmaf(16.0f, s0, -(dmin * ubyte0(mp))), slo, y);
        y = fmaf(fmaf(16.0f, s1, -(dmin * ubyte1(mp))), shi, y);
        return y;
    }
};

struct Q6K { // GGUF Q6_K; chunk = one sub-block of 16 elements: 16 bytes of low nibbles, 16 of bit pairs, an int8 scale
    static constexpr int W = 16;
    struct X { float xs[16]; };
    struct Raw { uint4 ql, qh; int sc; uint32_t d; };
    template <class F>
    __device__ static void set_x(const GemvArgs &, F fetch, X &o) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float4 v = fetch(i);
            o.xs[4 * i] = v.x; o.xs[4 * i + 1] = v.y; o.xs[4 * i + 2] = v.z; o.xs[4 * i + 3] = v.w;
        }
    }
    __device__ static void load(const GemvArgs &a, int row, int chunk, Raw &r) {
        // sub-block s = 8 n + 2 c + lh of superblock sb: elements 128 n + 32 c + 16 lh ..
        const int sb = chunk >> 4, s = chunk & 15, n = s >> 3, c = (s >> 1) & 3, lh = s & 1;
        r.ql = *reinterpret_cast<const uint4 *>(a.codes + (size_t)row * a.codes_pitch + (size_t)sb * 128 + 64 * n + 32 * (c & 1) + 16 * lh);
        r.qh = *reinterpret_cast<const uint4 *>(a.qh + (size_t)row * a.qh_pitch + (size_t)sb * 64 + 32 * n + 16 * lh);
        const uint8_t *m = a.meta + (size_t)row * a.meta_pitch;
        r.sc = (int)(int8_t)m[(size_t)sb * 16 + s];
        r.d = *reinterpret_cast<const uint16_t *>(m + (size_t)(a.cpr >> 4) * 16 + (size_t)sb * 2);
    }
    __device__ static float dot(const GemvArgs &, const Raw &r, const X &x, int chunk) {
        const int c = (chunk >> 1) & 3;
        const uint32_t ql[4] = {r.ql.x, r.ql.y, r.ql.z, r.ql.w}, qh[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) { // codes centred before the multiply: no large sums cancel for an x with a mean
            const uint32_t u = ((ql[w] >> (4 * (c >> 1))) & 0x0F0F0F0Fu) | (((qh[w] >> (2 * c)) & 0x03030303u) << 4);
            a0 = fmaf(ubyte0(u) - 32.0f, x.xs[4 * w], a0);
            a1 = fmaf(ubyte1(u) - 32.0f, x.xs[4 * w + 1], a1);
            a0 = fmaf(ubyte2(u) - 32.0f, x.xs[4 * w + 2], a0);
            a1 = fmaf(ubyte3(u) - 32.0f, x.xs[4 * w + 3], a1);
        }
        return (f16_bits_to_f32(r.d) * (float)r.sc) * (a0 + a1);
    }
};

struct F16W { // chunk = 8 halfs
    static constexpr int W = 8;
    struct X { float xs[8]; };
    struct Raw { uint4 q; };
    template <class F>
    __device__ static void set_x(const GemvArgs &, F fetch, X &o) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            float4 v = fetch(i);
            o.xs[4 * i] = v.x; o.xs[4 * i + 1] = v.y; o.xs[4 * i + 2] = v.z; o.xs[4 * i + 3] = v.w;
        }
    }
    __device__ static void load(const GemvArgs &a, int row, int chunk, Raw &r) {
        r.q = *reinterpret_cast<const uint4 *>(a.codes + (size_t)row * a.codes_pitch + (size_t)chunk * 16);
    }
    __device__ static float dot(const GemvArgs &, const Raw &r, const X &x, int) {
        const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            a0 = fmaf(f16_bits_to_f32(q[w] & 0xFFFF), x.xs[2 * w], a0);
            a1 = fmaf(f16_bits_to_f32(q[w] >> 16), x.xs[2 * w + 1], a1);
        }
        return a0 + a1;
    }
};

struct F32W { // chunk = 4 floats
    static constexpr int W = 4;
    struct X { float xs[4]; };
    struct Raw { float4 q; };
    template <class F>
    __device__ static void set_x(const GemvArgs &, F fetch, X &o) {
        float4 v = fetch(0);
        o.xs[0] = v.x; o.xs[1] = v.y; o.xs[2] = v.z; o.xs[3] = v.w;
    }
    __device__ static void load(const GemvArgs &a, int row, int chunk, Raw &r) {
        r.q = *reinterpret_cast<const float4 *>(a.codes + (size_t)row * a.codes_pitch + (size_t)chunk * 16);
    }
    __device__ static float dot(const GemvArgs &, const Raw &r, const X &x, int) {
        return fmaf(r.q.x, x.xs[0], r.q.y * x.xs[1]) + fmaf(r.q.z, x.xs[2], r.q.w * x.xs[3]);
    }
};

// x straight from global memory (fallback kernel)
template <class T>
__device__ inline void load_x_global(const GemvArgs &a, int chunk, bool active, typename T::X &o) {
    const float4 *p = reinterpret_cast<const float4 *>(a.x + (size_t)chunk * T::W);
    T::set_x(a, [&](int i) { return active ? p[i] : make_float4(0, 0, 0, 0); }, o);
}

// ---------------------------------------------------------------------------
// Fallback kernel (any K): x is read from global memory per wave, U rows in
// flight per lane, several passes over K when one lane cannot cover its share.
// ---------------------------------------------------------------------------
template <class T, int U>
__global__ void __launch_bounds__(512) gemv_kernel(GemvArgs a) {
    extern __shared__ float red[]; // [G][R][S] slice totals
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int grp = wave / a.S, slice = wave - grp * a.S;
    const int row0 = (blockIdx.x * a.G + grp) * a.R;
    int row_end = row0 + a.R;
    row_end = row_end < a.n_rows ? row_end : a.n_rows;

    typename T::X xr;
    int chunk = slice * 64 + lane;
    bool active = chunk < a.cpr;
    int cchunk = active ? chunk : a.cpr - 1; // inactive lanes re-read a valid chunk against x = 0
    if (a.npass == 1) load_x_global<T>(a, cchunk, active, xr);

    for (int r = row0; r < row_end; r += U) {
        float part[U];
#pragma unroll
        for (int u = 0; u < U; u++) part[u] = 0.f;
        for (int pass = 0; pass < a.npass; pass++) {
            if (a.npass > 1) {
                chunk = (pass * a.S + slice) * 64 + lane;
                active = chunk < a.cpr;
                cchunk = active ? chunk : a.cpr - 1;
                load_x_global<T>(a, cchunk, active, xr);
            }
            typename T::Raw raw[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                int row = r + u;
                row = row < a.n_rows ? row : a.n_rows - 1; // rows past the end are loaded and dropped
                T::load(a, row, cchunk, raw[u]);
            }
#pragma unroll
            for (int u = 0; u < U; u++) part[u] += T::dot(a, raw[u], xr, cchunk);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            float tot = wave_sum_lane63(part[u]);
            int row = r + u;
            if (lane == 63 && row < row_end) {
                if (a.S == 1) a.y[row] = a.bias ? tot + a.bias[row] : tot;
                else red[(grp * a.R + (row - row0)) * a.S + slice] = tot;
            }
        }
    }
    if (a.S > 1) {
        __syncthreads();
        int t = threadIdx.x;
        if (t < a.G * a.R) {
            int g = t / a.R, rr = t - g * a.R;
            int row = (blockIdx.x * a.G + g) * a.R + rr;
            if (row < a.n_rows) {
                float tot = 0.f;
                for (int s = 0; s < a.S; s++) tot += red[(g * a.R + rr) * a.S + s];
                a.y[row] = a.bias ? tot + a.bias[row] : tot;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Staged kernel (K*4 bytes of x fit in LDS): the main path.
//   - up to 8 waves per workgroup; x is fetched once per workgroup (coalesced),
//     parked in LDS in a [slice][vector][lane] order so that every lane then
//     pulls its own K-range into registers without bank conflicts (a short
//     last slice is packed with its own lane count as the stride);
//   - the weight loads of a wave's first U rows are issued before anything else,
//     the next U rows while the workgroup meets at the x barrier; every load is
//     unconditional (row indices are clamped) so that the compiler can count
//     outstanding loads and wait per row rather than for everything: unpacking
//     row i overlaps the arrival of row i+1...;
//   - later row batches cycle through a ring of NB register buffers (batch
//     i+NB is requested as soon as batch i has been folded);
//   - row totals go to LDS; the last phase adds the S slice totals in a fixed
//     order, adds the bias and writes y coalesced.
// ---------------------------------------------------------------------------
template <class T, int U>
__device__ inline void load_batch(const GemvArgs &a, int r, int row_last, int cchunk, typename T::Raw (&raw)[U]) {
#pragma unroll
    for (int u = 0; u < U; u++) {
        int row = r + u;
        row = row < row_last ? row : row_last; // rows past the end re-read the last row (cache hit, result dropped)
        T::load(a, row, cchunk, raw[u]);
    }
}

template <class T, int U>
__device__ inline void fold_batch(const GemvArgs &a, const typename T::Raw (&raw)[U], const typename T::X &xr, int cchunk,
                                  int r, int row0, int row_end, int grp, int slice, int lane, float *red) {
#pragma unroll
    for (int u = 0; u < U; u++) {
        float tot = wave_sum_lane63(T::dot(a, raw[u], xr, cchunk));
        int row = r + u;
        if (lane == 63 && row < row_end) red[(grp * a.R + (row - row0)) * a.S + slice] = tot;
    }
}

template <class T, int U, int NB, int XTN>
__global__ void __launch_bounds__(512) gemv_staged_kernel(GemvArgs a) {
    extern __shared__ float4 lds4[];
    constexpr int F4 = T::W / 4; // float4 per chunk
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave / a.S, slice = wave - grp * a.S;
    const int nf4 = a.cpr * F4;
    float *red = reinterpret_cast<float *>(lds4 + nf4);

    // 1. weights of the first row batch: gets HBM going at once
    const int chunk = slice * 64 + lane;
    const bool active = chunk < a.cpr;
    const int cchunk = active ? chunk : a.cpr - 1;
    const int row0 = (blockIdx.x * a.G + grp) * a.R;
    int row_end = row0 + a.R;
    row_end = row_end < a.n_rows ? row_end : a.n_rows;
    const int row_last = (row_end > row0 ? row_end : a.n_rows) - 1;
    typename T::Raw buf[NB][U];
    load_batch<T, U>(a, row0 < a.n_rows ? row0 : a.n_rows - 1, row_last, cchunk, buf[0]);

    // 2. x: global -> registers (an L2 hit; younger than the first batch, so waiting for it is enough)
    float4 xt[XTN];
    const float4 *xg = reinterpret_cast<const float4 *>(a.x);
#pragma unroll
    for (int j = 0; j < XTN; j++) {
        int f = tid + (int)blockDim.x * j;
        xt[j] = xg[f < nf4 ? f : nf4 - 1];
    }

    // 3. x: registers -> LDS (swizzled) -> this lane's K-range
#pragma unroll
    for (int j = 0; j < XTN; j++) {
        int f = tid + (int)blockDim.x * j;
        if (f < nf4) {
            int c = f / F4, i = f - c * F4;
            int sl = c >> 6;
            int P = a.cpr - (sl << 6); // chunks in this slice (the last one may be short)
            P = P < 64 ? P : 64;
            lds4[sl * (64 * F4) + i * P + (c & 63)] = xt[j];
        }
    }
    // the next batches go out while the workgroup meets at the barrier
#pragma unroll
    for (int b = 1; b < NB; b++) load_batch<T, U>(a, row0 + b * U, row_last, cchunk, buf[b]);
    __syncthreads();
    typename T::X xr;
    {
        const float4 *mine = lds4 + slice * (64 * F4) + lane;
        int P = a.cpr - (slice << 6);
        P = P < 64 ? P : 64;
        T::set_x(a, [&](int i) { return active ? mine[i * P] : make_float4(0, 0, 0, 0); }, xr);
    }

    // 4. fold the batches: a ring of NB register buffers, refilled as soon as they are consumed
    for (int r = row0; r < row_end; r += NB * U) {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            if (r + b * U < row_end) {
                fold_batch<T, U>(a, buf[b], xr, cchunk, r + b * U, row0, row_end, grp, slice, lane, red);
                if (r + (NB + b) * U < row_end) load_batch<T, U>(a, r + (NB + b) * U, row_last, cchunk, buf[b]);
            }
        }
    }

    // 5. slice totals -> y
    __syncthreads();
    for (int t = tid; t < a.G * a.R; t += (int)blockDim.x) {
        int g = t / a.R, rr = t - g * a.R;
        int row = (blockIdx.x * a.G + g) * a.R + rr;
        if (row < a.n_rows) {
            float tot = red[(g * a.R + rr) * a.S];
            for (int sidx = 1; sidx < a.S; sidx++) tot += red[(g * a.R + rr) * a.S + sidx];
            a.y[row] = a.bias ? tot + a.bias[row] : tot;
        }
    }
}

template <class T, int U, int NB>
void launch_staged(const GemvArgs &a, unsigned grid, unsigned block, size_t lds, int xt_need, hipStream_t st) {
    if (xt_need <= 1) gemv_staged_kernel<T, U, NB, 1><<<grid, block, lds, st>>>(a);
    else if (xt_need <= 2) gemv_staged_kernel<T, U, NB, 2><<<grid, block, lds, st>>>(a);
    else if (xt_need <= 4) gemv_staged_kernel<T, U, NB, 4><<<grid, block, lds, st>>>(a);
    else gemv_staged_kernel<T, U, NB, 8><<<grid, block, lds, st>>>(a);
}

template <class T>
int launch(axq_ctx *ctx, const axq_weight *w, const float *x, const float *bias, float *y) {
    GemvArgs a;
    a.codes = w->codes; a.meta = w->meta; a.qh = w->qh;
    a.codes_pitch = w->codes_pitch; a.meta_pitch = w->meta_pitch; a.qh_pitch = w->qh_pitch;
    a.x = x; a.bias = bias; a.y = y;
    a.n_rows = (int)w->n_rows;
    a.cpr = (int)(w->k / T::W);
    a.fp8_unit_inv = ctx->fp8_unit_inv;
    int cus = ctx->prop.multiProcessorCount;
    constexpr int U = 4;
    int s_need = (a.cpr + 63) / 64;
    constexpr int F4 = T::W / 4;
    if (s_need <= 8) {
        // staged path: up to 8 waves per workgroup, one workgroup per CU
        a.S = s_need;
        a.G = 8 / a.S;
        a.npass = 1;
        unsigned block = (unsigned)(64 * a.S * a.G);
        int nf4 = a.cpr * F4;
        int xt_need = (nf4 + (int)block - 1) / (int)block;
        if (xt_need <= 8) {
            int groups = cus * a.G;
            a.R = (a.n_rows + groups - 1) / groups;
            if (a.R < 1) a.R = 1;
            int rows_per_wg = a.G * a.R;
            unsigned grid = (unsigned)((a.n_rows + rows_per_wg - 1) / rows_per_wg);
            size_t lds = (size_t)nf4 * 16 + (size_t)a.G * a.R * a.S * sizeof(float);
            if (lds <= 64 * 1024) {
                if (a.R <= 2) launch_staged<T, 2, 1>(a, grid, block, lds, xt_need, ctx->stream);
                else if (a.R <= 4) launch_staged<T, 2, 2>(a, grid, block, lds, xt_need, ctx->stream);
                else launch_staged<T, 2, 4>(a, grid, block, lds, xt_need, ctx->stream);
                AXQ_LAUNCH_CHECK(ctx, "gemv_staged_kernel");
                return AXQ_OK;
            }
        }
    }
    const int SMAX = 8;
    a.S = s_need < SMAX ? s_need : SMAX;
    a.npass = (s_need + a.S - 1) / a.S;
    a.G = a.S >= 4 ? 1 : 4 / a.S;
    int target_wgs = cus * 2;
    int R = (a.n_rows + a.G * target_wgs - 1) / (a.G * target_wgs);
    R = (R + U - 1) / U * U;
    if (R < U) R = U;
    if (R > 64) R = 64;
    a.R = R;
    int rows_per_wg = a.G * a.R;
    unsigned grid = (unsigned)((a.n_rows + rows_per_wg - 1) / rows_per_wg);
    unsigned block = (unsigned)(64 * a.S * a.G);
    size_t lds = a.S > 1 ? (size_t)a.G * a.R * a.S * sizeof(float) : 0;
    gemv_kernel<T, U><<<grid, block, lds, ctx->stream>>>(a);
    AXQ_LAUNCH_CHECK(ctx, "gemv_kernel");
    return AXQ_OK;
}

} // namespace

int axq_dev_gemv(axq_ctx *ctx, const axq_weight *w, const float *x, int batch, const float *bias, float *y) {
    if (w->n_rows > INT32_MAX || w->k > INT32_MAX)
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: weight dimensions exceed 2^31");
    // many vectors: through the matrix-pipe GEMM, each f32 row as two f16 rows; worth it from about 40 rows where the
    // small-batch kernel below is the alternative, from 8 where single-vector passes are
    static const bool no_gemm = getenv("AXQ_GEMV_GEMM") && getenv("AXQ_GEMV_GEMM")[0] == '0'; // development knob
    while (!no_gemm && batch >= (axq_dev_gemv_batch_covers(w, 8) ? 40 : 8) && axq_dev_gemm_f32_covers(w, 1)) {
        const int nb = batch < AXQ_GEMM_F32_MAX_ROWS ? batch : AXQ_GEMM_F32_MAX_ROWS;
        int rc = axq_dev_gemm_f32(ctx, w, x, nb, nullptr, 0.f, bias, nullptr, y);
        if (rc) return rc;
        x += (size_t)nb * (size_t)w->k;
        y += (size_t)nb * (size_t)w->n_rows;
        batch -= nb;
    }
    // small batches: eight vectors at a time against one pass over the weights, where that kernel applies
    while (batch >= 2 && axq_dev_gemv_batch_covers(w, batch < 8 ? batch : 8)) {
        const int nb = batch < 8 ? batch : 8;
        int rc = axq_dev_gemv_batch(ctx, w, x, nb, bias, nullptr, y);
        if (rc) return rc;
        x += (size_t)nb * (size_t)w->k;
        y += (size_t)nb * (size_t)w->n_rows;
        batch -= nb;
    }
    for (int b = 0; b < batch; b++) {
        const float *xb = x + (size_t)b * (size_t)w->k;
        float *yb = y + (size_t)b * (size_t)w->n_rows;
        const uint8_t *xq = nullptr;
        if (ctx->gemv_prep && axq_type_is_block_quantized(w->type) && w->k % 64 == 0 && w->k <= AXQ_XQ_MAX_K) {
            int prc = axq_dev_prep_x(ctx, xb, w->k, ctx->xq);
            if (prc) return prc;
            xq = ctx->xq;
        }
        int rc = axq_dev_gemv_dp(ctx, w, xb, xq, bias, yb);
        if (rc < 0) return rc;
        if (rc == 1) continue;
        switch (w->type) {
        case AXQ_Q4_K: rc = launch<Q4K>(ctx, w, xb, bias, yb); break;
        case AXQ_Q6_K: rc = launch<Q6K>(ctx, w, xb, bias, yb); break;
        case AXQ_Q5_K: rc = launch<Q5K>(ctx, w, xb, bias, yb); break;
        case AXQ_Q4_0: rc = launch<Q4x<false>>(ctx, w, xb, bias, yb); break;
        case AXQ_Q4_1: rc = launch<Q4x<true>>(ctx, w, xb, bias, yb); break;
        case AXQ_Q5_0: rc = launch<Q5x<false>>(ctx, w, xb, bias, yb); break;
        case AXQ_Q5_1: rc = launch<Q5x<true>>(ctx, w, xb, bias, yb); break;
        case AXQ_Q8_0: rc = launch<Q80>(ctx, w, xb, bias, yb); break;
        case AXQ_F16: rc = launch<F16W>(ctx, w, xb, bias, yb); break;
        case AXQ_F32: rc = launch<F32W>(ctx, w, xb, bias, yb); break;
        default: return axq_fail(ctx, AXQ_ERR_INVALID_QUANT_TYPE, "Invalid quantization type: %d", w->type);
        }
        if (rc) return rc;
    }
    return AXQ_OK;
}
