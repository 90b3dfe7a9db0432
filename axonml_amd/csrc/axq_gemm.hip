// Prefill-path quantized matmul: y[M, N] = x[M, K] (bf16) * W[N, K]^T, f32 accumulate and output.
//
// The reference composition is dequantize_tensor -> f32 sgemm (crates/axonml-quant/src/dequantize.rs:34-54,
// crates/axonml-core/src/backends/cpu.rs:566-598).  Here the packed weights are read once per M tile,
// dequantised in registers into LDS tiles and multiplied on the matrix pipe (v_mfma_f32_32x32x16_f16).
//
// Numerics: results must agree with the f32 reference to 1e-3 per element even where the output is
// small, which plain f16 weights (11 bits) do not give.  So
//   - a dequantised weight w (f32, rounded exactly as the reference rounds it) is split into two f16
//     values w = wh + wl (22 bits), and both halves are multiplied: two MFMAs per tile and K step;
//   - x comes in bf16 (8 significant bits) and is converted to f16 exactly: a small pre-pass scales
//     every row by a power of two so that its largest magnitude sits below 2^15, which keeps every
//     element that matters inside f16's normal range; the row scale is undone on the output.
// Accumulation is f32 inside the MFMA, in K order.
//
// Tiling: a workgroup computes BM x 128 outputs (BM = 128 or 256); K advances 64 at a time through two LDS
// stages, each holding the x tile and the two weight tiles.  Half of the waves multiply, the other half
// feed (see gemm_kernel).
#include <hip/hip_fp16.h>

#include <stdlib.h>

#include <type_traits>

#include "axq_internal.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4))); // a 16-byte register quad (arrays of HIP's uint4 struct end up in scratch)

constexpr int BN = 128;  // output columns (weight rows) per workgroup
constexpr int BK = 64;   // K per stage
constexpr int LDK = 72;  // LDS row length in halfs (64 + 8 padding against bank conflicts)

struct GemmArgs {
    const uint8_t *codes, *meta, *qh;
    size_t codes_pitch, meta_pitch, qh_pitch;
    const _Float16 *xh;    // [M, K] row-scaled f16
    const float *rowscale; // [M]
    float *y;              // [M, N]
    float *ypart;          // split K: [splits, M, N] unscaled partial sums (NULL when one workgroup covers all of K)
    int m, n, k;
    int steps_per_split;   // K steps per workgroup (grid.y of them cover K)
    // pair mode (f32 activations): rows 2t and 2t + 1 of xh are the two f16 parts of activation row t, and their results
    // are added into output row t (+ bias[n] + resid[t, n]); y, ypart and resid then have m / 2 rows
    int pair;
    const float *bias, *resid;
    int wm;                // 1: 128-row tiles, 2: 256-row tiles
    // Q4_K kernel only: the rows' sub-block sums as f16 pairs, per split of K [hi | hi | lo | zeros] (see gemm_q4k_kernel)
    const _Float16 *xs3;
    int xs3_pitch;         // halfs per xs3 row
};

__device__ inline float h2f(uint32_t bits) { return __half2float(__ushort_as_half((unsigned short)bits)); }
template <int B>
__device__ inline float ubyte(uint32_t v) { // byte B of v as a float, one instruction
    float r;
    if (B == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(r) : "v"(v));
    else if (B == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(r) : "v"(v));
    else if (B == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(r) : "v"(v));
    else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(r) : "v"(v));
    return r;
}

// Weights go through the matrix pipe as WSCALE * w = wh + wl with wh, wl in f16: the power-of-two factor
// keeps the low part of ordinary weights (|w| > 5e-4) out of f16's subnormal range; the epilogue divides
// it out again.  A trait names its factor WS, and says PRESCALED when its convert step applies it already.
constexpr float WSCALE = 256.0f;

// ---------------------------------------------------------------------------
// Dequantisation units.  A unit is 16 weights of one weight row inside the current 64-wide K step:
// two runs of 8 consecutive k (k0.., k1..).  unit index u4 = 0..3 per row.  Each trait reproduces the
// element formula of crates/axonml-quant/src/dequantize.rs (Q8_0 :89-92, Q4_0 :116-121, Q4_1 :145-151)
// or of the GGUF spec (Q5_0, Q5_1, Q4_K), rounding as the f32 reference does (multiply, then add).
// ---------------------------------------------------------------------------
struct GQ4K {
    static constexpr bool PRESCALED = true;
    static constexpr float WS = WSCALE;
    struct Raw { uint2 q; uint4 h; };
    __device__ static void load16(const GemmArgs &a, size_t row, int kstep, int u4, Raw &r) {
        const int cpr = a.k >> 6;          // pairs per row
        const int pair = kstep;            // one pair of sub-blocks per K step
        const int slice = pair >> 6, pr = pair & 63;
        int P = cpr - (slice << 6);
        P = P < 64 ? P : 64;
        const int half = u4 >> 1, part = u4 & 1;
        const uint8_t *base = a.codes + row * a.codes_pitch + (size_t)slice * 2048 + (size_t)half * 16 * P + (size_t)pr * 16 + part * 8;
        r.q = *reinterpret_cast<const uint2 *>(base);
        r.h = *reinterpret_cast<const uint4 *>(a.meta + row * a.meta_pitch + (size_t)(pair >> 2) * 16);
    }
    __device__ static void cvt16(const Raw &r, int kstep, int u4, float (&w)[16], int &k0, int &k1) {
        const uint2 q = r.q;
        const uint4 h = r.h;
        const int pair = kstep, half = u4 >> 1, part = u4 & 1;
        const int p = pair & 3, sh = (p & 1) * 16;
        const uint32_t ya = h.y >> sh, za = h.z >> sh, wa = h.w >> sh;
        uint32_t scp, mp;
        if (p < 2) {
            scp = ya & 0x3F3F;
            mp = za & 0x3F3F;
        } else {
            scp = (wa & 0x0F0F) | ((ya >> 2) & 0x3030);
            mp = ((wa >> 4) & 0x0F0F) | ((za >> 2) & 0x3030);
        }
        const float d = WSCALE * h2f(h.x & 0xFFFF), dmin = WSCALE * h2f(h.x >> 16);
        const float sd0 = d * ubyte<0>(scp), sd1 = d * ubyte<1>(scp);
        const float sm0 = dmin * ubyte<0>(mp), sm1 = dmin * ubyte<1>(mp);
        // one rounding per weight (fma) where the f32 reference has two: far below what f16 pairs resolve
        const uint32_t ml[2] = {q.x & 0x0F0F0F0Fu, q.y & 0x0F0F0F0Fu};
        const uint32_t mh[2] = {(q.x >> 4) & 0x0F0F0F0Fu, (q.y >> 4) & 0x0F0F0F0Fu};
#pragma unroll
        for (int j = 0; j < 2; j++) {
            w[4 * j + 0] = fmaf(sd0, ubyte<0>(ml[j]), -sm0); w[4 * j + 1] = fmaf(sd0, ubyte<1>(ml[j]), -sm0);
            w[4 * j + 2] = fmaf(sd0, ubyte<2>(ml[j]), -sm0); w[4 * j + 3] = fmaf(sd0, ubyte<3>(ml[j]), -sm0);
            w[8 + 4 * j + 0] = fmaf(sd1, ubyte<0>(mh[j]), -sm1); w[8 + 4 * j + 1] = fmaf(sd1, ubyte<1>(mh[j]), -sm1);
            w[8 + 4 * j + 2] = fmaf(sd1, ubyte<2>(mh[j]), -sm1); w[8 + 4 * j + 3] = fmaf(sd1, ubyte<3>(mh[j]), -sm1);
        }
        k0 = half * 16 + part * 8;
        k1 = 32 + k0;
    }
};

template <bool WITH_MIN>
struct GQ4x { // reference nibble order: byte i = elements 2i (low), 2i+1 (high)
    static constexpr bool PRESCALED = true;
    static constexpr float WS = WSCALE;
    struct Raw { uint2 q; uint32_t m; };
    __device__ static void load16(const GemmArgs &a, size_t row, int kstep, int u4, Raw &r) {
        const int blk = kstep * 2 + (u4 >> 1), part = u4 & 1;
        r.q = *reinterpret_cast<const uint2 *>(a.codes + row * a.codes_pitch + (size_t)blk * 16 + part * 8);
        const uint8_t *mp = a.meta + row * a.meta_pitch;
        r.m = WITH_MIN ? *reinterpret_cast<const uint32_t *>(mp + (size_t)blk * 4)
                       : (uint32_t) * reinterpret_cast<const uint16_t *>(mp + (size_t)blk * 2);
    }
    __device__ static void cvt16(const Raw &r, int, int u4, float (&w)[16], int &k0, int &k1) {
        const int part = u4 & 1;
        // (nib - 8) * d = nib * d - 8 d exactly; with a minimum one rounding (fma) where the f32 reference has two: far
        // below what f16 pairs resolve.  Four codes per mask, one conversion per code straight from its byte.
        const float scale = WSCALE * h2f(r.m & 0xFFFF), mn = WITH_MIN ? WSCALE * h2f(r.m >> 16) : -8.0f * scale;
        const uint32_t qq[2] = {r.q.x, r.q.y};
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint32_t lo = qq[j] & 0x0F0F0F0Fu, hi = (qq[j] >> 4) & 0x0F0F0F0Fu;
            w[8 * j + 0] = fmaf(ubyte<0>(lo), scale, mn); w[8 * j + 1] = fmaf(ubyte<0>(hi), scale, mn);
            w[8 * j + 2] = fmaf(ubyte<1>(lo), scale, mn); w[8 * j + 3] = fmaf(ubyte<1>(hi), scale, mn);
            w[8 * j + 4] = fmaf(ubyte<2>(lo), scale, mn); w[8 * j + 5] = fmaf(ubyte<2>(hi), scale, mn);
            w[8 * j + 6] = fmaf(ubyte<3>(lo), scale, mn); w[8 * j + 7] = fmaf(ubyte<3>(hi), scale, mn);
        }
        k0 = (u4 >> 1) * 32 + part * 16;
        k1 = k0 + 8;
    }
};

template <bool WITH_MIN>
struct GQ5x { // byte j = elements j (low nibble) and j + 16 (high); qh bit e = bit 4 of element e
    static constexpr bool PRESCALED = true;
    static constexpr float WS = WSCALE;
    struct Raw { uint2 q; uint32_t qh, m; };
    __device__ static void load16(const GemmArgs &a, size_t row, int kstep, int u4, Raw &r) {
        const int blk = kstep * 2 + (u4 >> 1), part = u4 & 1;
        r.q = *reinterpret_cast<const uint2 *>(a.codes + row * a.codes_pitch + (size_t)blk * 16 + part * 8);
        r.qh = *reinterpret_cast<const uint32_t *>(a.qh + row * a.qh_pitch + (size_t)blk * 4);
        const uint8_t *mp = a.meta + row * a.meta_pitch;
        r.m = WITH_MIN ? *reinterpret_cast<const uint32_t *>(mp + (size_t)blk * 4)
                       : (uint32_t) * reinterpret_cast<const uint16_t *>(mp + (size_t)blk * 2);
    }
    __device__ static void cvt16(const Raw &r, int, int u4, float (&w)[16], int &k0, int &k1) {
        const int part = u4 & 1;
        const uint32_t qh = r.qh;
        // (u - 16) * d = u * d - 16 d exactly; with a minimum one rounding (fma) where the f32 reference has two.
        const float d = WSCALE * h2f(r.m & 0xFFFF), mn = WITH_MIN ? WSCALE * h2f(r.m >> 16) : -16.0f * d;
        const uint32_t qq[2] = {r.q.x, r.q.y};
        // four bits of qh -> bit 4 of four bytes: the copies of the multiplication lie 7 bits apart and do not meet
        auto fifth = [](uint32_t four) { return ((four * 0x00204081u) & 0x01010101u) << 4; };
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int e = part * 8 + 4 * j;
            const uint32_t lo = (qq[j] & 0x0F0F0F0Fu) | fifth((qh >> e) & 0xFu);
            const uint32_t hi = ((qq[j] >> 4) & 0x0F0F0F0Fu) | fifth((qh >> (e + 16)) & 0xFu);
            w[4 * j + 0] = fmaf(ubyte<0>(lo), d, mn); w[4 * j + 1] = fmaf(ubyte<1>(lo), d, mn);
            w[4 * j + 2] = fmaf(ubyte<2>(lo), d, mn); w[4 * j + 3] = fmaf(ubyte<3>(lo), d, mn);
            w[8 + 4 * j + 0] = fmaf(ubyte<0>(hi), d, mn); w[8 + 4 * j + 1] = fmaf(ubyte<1>(hi), d, mn);
            w[8 + 4 * j + 2] = fmaf(ubyte<2>(hi), d, mn); w[8 + 4 * j + 3] = fmaf(ubyte<3>(hi), d, mn);
        }
        k0 = (u4 >> 1) * 32 + part * 8;
        k1 = k0 + 16;
    }
};

struct GQ80 {
    static constexpr bool PRESCALED = true;
    static constexpr float WS = WSCALE;
    struct Raw { uint4 q; uint32_t m; };
    __device__ static void load16(const GemmArgs &a, size_t row, int kstep, int u4, Raw &r) {
        const int blk = kstep * 2 + (u4 >> 1), part = u4 & 1;
        r.q = *reinterpret_cast<const uint4 *>(a.codes + row * a.codes_pitch + (size_t)blk * 32 + part * 16);
        r.m = *reinterpret_cast<const uint16_t *>(a.meta + row * a.meta_pitch + (size_t)blk * 2);
    }
    __device__ static void cvt16(const Raw &r, int, int u4, float (&w)[16], int &k0, int &k1) {
        const int part = u4 & 1;
        // q * d = (q + 128) * d - 128 d exactly: the codes as unsigned bytes, one conversion each
        const float scale = WSCALE * h2f(r.m), off = -128.0f * scale;
        const uint32_t qq[4] = {r.q.x ^ 0x80808080u, r.q.y ^ 0x80808080u, r.q.z ^ 0x80808080u, r.q.w ^ 0x80808080u};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            w[4 * j + 0] = fmaf(ubyte<0>(qq[j]), scale, off); w[4 * j + 1] = fmaf(ubyte<1>(qq[j]), scale, off);
            w[4 * j + 2] = fmaf(ubyte<2>(qq[j]), scale, off); w[4 * j + 3] = fmaf(ubyte<3>(qq[j]), scale, off);
        }
        k0 = (u4 >> 1) * 32 + part * 16;
        k1 = k0 + 8;
    }
};

struct GQ5K { // GGUF Q5_K on Q4_K's planes: the codes' low four bits as GQ4K reads them, the fifth bits from the qh plane
    static constexpr bool PRESCALED = true;
    static constexpr float WS = WSCALE;
    struct Raw { uint2 q, b; uint4 h; };
    __device__ static void load16(const GemmArgs &a, size_t row, int kstep, int u4, Raw &r) {
        const int cpr = a.k >> 6;
        const int pair = kstep;
        const int slice = pair >> 6, pr = pair & 63;
        int P = cpr - (slice << 6);
        P = P < 64 ? P : 64;
        const int half = u4 >> 1, part = u4 & 1;
        r.q = *reinterpret_cast<const uint2 *>(a.codes + row * a.codes_pitch + (size_t)slice * 2048 + (size_t)half * 16 * P + (size_t)pr * 16 + part * 8);
        r.h = *reinterpret_cast<const uint4 *>(a.meta + row * a.meta_pitch + (size_t)(pair >> 2) * 16);
        // bytes l = 16 half + 8 part .. + 7 of the superblock's 32: bit 2 p (+ 1) = fifth bit of element l of the pair's low (high) sub-block
        r.b = *reinterpret_cast<const uint2 *>(a.qh + row * a.qh_pitch + (size_t)(pair >> 2) * 32 + half * 16 + part * 8);
    }
    __device__ static void cvt16(const Raw &r, int kstep, int u4, float (&w)[16], int &k0, int &k1) {
        const int pair = kstep, half = u4 >> 1, part = u4 & 1;
        const int p = pair & 3, sh = (p & 1) * 16;
        const uint32_t ya = r.h.y >> sh, za = r.h.z >> sh, wa = r.h.w >> sh;
        uint32_t scp, mp;
        if (p < 2) {
            scp = ya & 0x3F3F;
            mp = za & 0x3F3F;
        } else {
            scp = (wa & 0x0F0F) | ((ya >> 2) & 0x3030);
            mp = ((wa >> 4) & 0x0F0F) | ((za >> 2) & 0x3030);
        }
        const float d = WSCALE * h2f(r.h.x & 0xFFFF), dmin = WSCALE * h2f(r.h.x >> 16);
        const float sd0 = d * ubyte<0>(scp), sd1 = d * ubyte<1>(scp);
        const float sm0 = dmin * ubyte<0>(mp), sm1 = dmin * ubyte<1>(mp);
        const uint32_t q[2] = {r.q.x, r.q.y}, b[2] = {r.b.x, r.b.y};
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint32_t ul = (q[j] & 0x0F0F0F0Fu) | (((b[j] >> (2 * p)) & 0x01010101u) << 4);
            const uint32_t uh = ((q[j] >> 4) & 0x0F0F0F0Fu) | (((b[j] >> (2 * p + 1)) & 0x01010101u) << 4);
            w[4 * j + 0] = fmaf(sd0, ubyte<0>(ul), -sm0); w[4 * j + 1] = fmaf(sd0, ubyte<1>(ul), -sm0);
            w[4 * j + 2] = fmaf(sd0, ubyte<2>(ul), -sm0); w[4 * j + 3] = fmaf(sd0, ubyte<3>(ul), -sm0);
            w[8 + 4 * j + 0] = fmaf(sd1, ubyte<0>(uh), -sm1); w[8 + 4 * j + 1] = fmaf(sd1, ubyte<1>(uh), -sm1);
            w[8 + 4 * j + 2] = fmaf(sd1, ubyte<2>(uh), -sm1); w[8 + 4 * j + 3] = fmaf(sd1, ubyte<3>(uh), -sm1);
        }
        k0 = half * 16 + part * 8;
        k1 = 32 + k0;
    }
};

struct GQ6K { // GGUF Q6_K: a unit is one sub-block of 16 consecutive elements with its own int8 scale
    static constexpr bool PRESCALED = true;
    // d * scale * q reaches 127 * 32 times d: a smaller factor than WSCALE leaves weights up to 4000 finite in f16 and
    // still keeps the low parts of weights above 8e-3 normal
    static constexpr float WS = 16.0f;
    struct Raw { uint4 ql, qh; int sc; uint32_t d; };
    __device__ static void load16(const GemmArgs &a, size_t row, int kstep, int u4, Raw &r) {
        // K step = 64 elements = sub-blocks 4 (kstep % 4) .. of superblock kstep / 4; s = 8 n + 2 c + lh
        const int sb = kstep >> 2, s = (kstep & 3) * 4 + u4, n = s >> 3, c = (s >> 1) & 3, lh = s & 1;
        r.ql = *reinterpret_cast<const uint4 *>(a.codes + row * a.codes_pitch + (size_t)sb * 128 + 64 * n + 32 * (c & 1) + 16 * lh);
        r.qh = *reinterpret_cast<const uint4 *>(a.qh + row * a.qh_pitch + (size_t)sb * 64 + 32 * n + 16 * lh);
        const uint8_t *m = a.meta + row * a.meta_pitch;
        r.sc = (int)(int8_t)m[(size_t)sb * 16 + s];
        r.d = *reinterpret_cast<const uint16_t *>(m + (size_t)(a.k >> 8) * 16 + (size_t)sb * 2);
    }
    __device__ static void cvt16(const Raw &r, int kstep, int u4, float (&w)[16], int &k0, int &k1) {
        const int c = ((((kstep & 3) * 4 + u4) >> 1) & 3);
        // (d * scale) * (u - 32) = u * ds - 32 ds: one rounding (fma) where the f32 reference has one as well
        const float ds = WS * (h2f(r.d) * (float)r.sc), off = -32.0f * ds;
        const uint32_t ql[4] = {r.ql.x, r.ql.y, r.ql.z, r.ql.w}, qh[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t u = ((ql[j] >> (4 * (c >> 1))) & 0x0F0F0F0Fu) | (((qh[j] >> (2 * c)) & 0x03030303u) << 4);
            w[4 * j + 0] = fmaf(ubyte<0>(u), ds, off); w[4 * j + 1] = fmaf(ubyte<1>(u), ds, off);
            w[4 * j + 2] = fmaf(ubyte<2>(u), ds, off); w[4 * j + 3] = fmaf(ubyte<3>(u), ds, off);
        }
        k0 = u4 * 16;
        k1 = k0 + 8;
    }
};

struct GF16 {
    static constexpr bool PRESCALED = false;
    static constexpr float WS = 1.0f; // plain weights may be large: no headroom to give away
    struct Raw { uint4 v0, v1; };
    __device__ static void load16(const GemmArgs &a, size_t row, int kstep, int u4, Raw &r) {
        const uint4 *p = reinterpret_cast<const uint4 *>(a.codes + row * a.codes_pitch + ((size_t)kstep * 64 + u4 * 16) * 2);
        r.v0 = p[0];
        r.v1 = p[1];
    }
    __device__ static void cvt16(const Raw &r, int, int u4, float (&w)[16], int &k0, int &k1) {
        const uint4 v0 = r.v0, v1 = r.v1;
        const uint32_t qq[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            w[2 * i] = h2f(qq[i] & 0xFFFF);
            w[2 * i + 1] = h2f(qq[i] >> 16);
        }
        k0 = u4 * 16;
        k1 = k0 + 8;
    }
};

struct GF32 {
    static constexpr bool PRESCALED = false;
    static constexpr float WS = 1.0f; // plain weights may be large: no headroom to give away
    struct Raw { float4 v[4]; };
    __device__ static void load16(const GemmArgs &a, size_t row, int kstep, int u4, Raw &r) {
        const float4 *p = reinterpret_cast<const float4 *>(a.codes + row * a.codes_pitch + ((size_t)kstep * 64 + u4 * 16) * 4);
#pragma unroll
        for (int i = 0; i < 4; i++) r.v[i] = p[i];
    }
    __device__ static void cvt16(const Raw &r, int, int u4, float (&w)[16], int &k0, int &k1) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float4 v = r.v[i];
            w[4 * i] = v.x; w[4 * i + 1] = v.y; w[4 * i + 2] = v.z; w[4 * i + 3] = v.w;
        }
        k0 = u4 * 16;
        k1 = k0 + 8;
    }
};

// Eight values times `scale` -> eight f16 high parts and eight f16 remainders, as
// two 16-byte vectors.  The high part is the value with its mantissa cut to f16's eleven bits, a mask, exact in
// f16; the remainder is exact in f32 and keeps its own top eleven bits.
__device__ inline void split8_f16(const float *w, float scale, uint4 &hi, uint4 &lo) {
    uint32_t h[4], l[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float a = w[2 * i] * scale, b = w[2 * i + 1] * scale; // scale 1 folds away
        const float ah = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, a) & 0xFFFFE000u);
        const float bh = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, b) & 0xFFFFE000u);
        h[i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(ah, bh));
        l[i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a - ah, b - bh));
    }
    hi = make_uint4(h[0], h[1], h[2], h[3]);
    lo = make_uint4(l[0], l[1], l[2], l[3]);
}

// A workgroup barrier that orders LDS traffic only: __syncthreads() also waits for every global load in flight, which
// would pull the prefetched operands of later steps in front of every barrier.
__device__ inline void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0); // nothing moves across: what follows may count on the waits in front of the barrier
}

// WM = 1 or 2: the workgroup computes (128 * WM) x 128 outputs with eight waves of two kinds.
//   - four "multiplier" waves each own a (64 * WM) x 64 block (2 WM x 2 MFMA tiles) and do nothing but read the
//     current LDS stage and issue MFMAs;
//   - four "feeder" waves fetch the x tile and the packed weights of the step after next, convert the
//     next step's weights (dequantise, split into two f16) and write the other LDS stage.
// Waves are dealt to the four SIMDs in turn, so every SIMD holds one wave of each kind and its vector ALU converts
// while its matrix pipe multiplies; one barrier per K step hands the stages over.
template <class T, int WM>
__global__ void __launch_bounds__(512) gemm_kernel(GemmArgs a) {
    constexpr int BM = 128 * WM, NTF = 256;      // rows of x per tile; feeder threads
    constexpr int MI = 2 * WM;                   // MFMA tiles of a multiplier wave along M
    constexpr int XV = BM * 8 / NTF;             // 16-byte x vectors per feeder thread and K step (4 or 8)
    constexpr int UNITS = BN * 4 / NTF;          // 16-weight units per feeder thread and K step (= 2)
    constexpr int STAGE = (BM + 2 * BN) * LDK;   // halfs per LDS stage
    extern __shared__ _Float16 lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool feeder = tid >= NTF;
    // Workgroups of one XCD (those with equal id modulo 8) take consecutive tiles, N fastest: the x tile is
    // the big operand of a step (BM x 64 halfs against 128 x 64 packed weights), so the workgroups that share
    // an x tile should share an L2.
    const int nt = (a.n + BN - 1) / BN, total = (int)gridDim.x;
    int tile = blockIdx.x;
    if (total % 8 == 0) tile = (tile & 7) * (total >> 3) + (tile >> 3);
    const int m0 = (tile / nt) * BM, n0 = (tile % nt) * BN;
    // split K: workgroup (x, y) covers K steps [kbeg, kbeg + ksteps)
    const int kbeg = (int)blockIdx.y * a.steps_per_split;
    const int ksteps = a.k / BK - kbeg < a.steps_per_split ? a.k / BK - kbeg : a.steps_per_split;

    if (feeder) {
        const int ft = tid - NTF;
        u32x4 xa[XV];
        typename T::Raw raw[UNITS];
        // row addresses do not change from step to step
        const _Float16 *xrow[XV];
        size_t wrow[UNITS];
#pragma unroll
        for (int i = 0; i < XV; i++) {
            int v = ft + i * NTF;
            int gm = m0 + (v >> 3);
            gm = gm < a.m ? gm : a.m - 1;
            xrow[i] = a.xh + (size_t)gm * a.k + (v & 7) * 8;
        }
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            int gn = n0 + ((ft + u * NTF) >> 2);
            wrow[u] = (size_t)(gn < a.n ? gn : a.n - 1);
        }
        auto fetch = [&](int ks) { // clamped: past the last step the feeders re-read it and nobody looks
            ks = ks < ksteps ? ks : ksteps - 1;
#pragma unroll
            for (int i = 0; i < XV; i++) xa[i] = *reinterpret_cast<const u32x4 *>(xrow[i] + (size_t)(kbeg + ks) * BK);
#pragma unroll
            for (int u = 0; u < UNITS; u++) T::load16(a, wrow[u], kbeg + ks, (ft + u * NTF) & 3, raw[u]);
        };
        fetch(0);
        for (int ks = 0; ks <= ksteps; ks++) {
            // registers hold step ks: convert it into stage ks & 1, with step ks + 1 already requested
            _Float16 *As = lds + (ks & 1) * STAGE, *Bh = As + BM * LDK, *Bl = Bh + BN * LDK;
            const int kcur = ks < ksteps ? ks : ksteps - 1;
            u32x4 xs[XV];
            float w[UNITS][16];
            int k0[UNITS], k1[UNITS];
#pragma unroll
            for (int i = 0; i < XV; i++) xs[i] = xa[i];
#pragma unroll
            for (int u = 0; u < UNITS; u++) T::cvt16(raw[u], kbeg + kcur, (ft + u * NTF) & 3, w[u], k0[u], k1[u]);
            fetch(ks + 1);
            if (ks < ksteps) {
#pragma unroll
                for (int i = 0; i < XV; i++) {
                    int v = ft + i * NTF;
                    int row = v >> 3, c = v & 7;
                    *reinterpret_cast<u32x4 *>(As + row * LDK + c * 8) = xs[i];
                }
#pragma unroll
                for (int u = 0; u < UNITS; u++) {
                    int row = (ft + u * NTF) >> 2;
                    uint4 h0, l0, h1, l1;
                    split8_f16(w[u], T::PRESCALED ? 1.0f : T::WS, h0, l0);
                    split8_f16(w[u] + 8, T::PRESCALED ? 1.0f : T::WS, h1, l1);
                    *reinterpret_cast<uint4 *>(Bh + row * LDK + k0[u]) = h0;
                    *reinterpret_cast<uint4 *>(Bh + row * LDK + k1[u]) = h1;
                    *reinterpret_cast<uint4 *>(Bl + row * LDK + k0[u]) = l0;
                    *reinterpret_cast<uint4 *>(Bl + row * LDK + k1[u]) = l1;
                }
            }
            lds_barrier(); // barrier ks: stage ks & 1 is complete, stage (ks + 1) & 1 has been read; the loads of step
                           // ks + 1 stay in flight across it
        }
        return;
    }

    const int wm = (wave >> 1) * (32 * MI), wn = (wave & 1) * 64; // this wave's block inside the tile
    const int li = lane & 31, lk = (lane >> 5) * 8;
    float16v acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
    __syncthreads(); // barrier 0
    for (int ks = 0; ks < ksteps; ks++) {
        const _Float16 *As = lds + (ks & 1) * STAGE, *Bh = As + BM * LDK, *Bl = Bh + BN * LDK;
        // fragments of sub-step kk + 1 are read from LDS while the sixteen MFMAs of sub-step kk run
        half8 af[2][MI], bh[2][2], bl[2][2];
        auto read_frags = [&](int kk, int slot) {
#pragma unroll
            for (int i = 0; i < MI; i++) af[slot][i] = *reinterpret_cast<const half8 *>(As + (wm + i * 32 + li) * LDK + kk + lk);
#pragma unroll
            for (int j = 0; j < 2; j++) {
                bh[slot][j] = *reinterpret_cast<const half8 *>(Bh + (wn + j * 32 + li) * LDK + kk + lk);
                bl[slot][j] = *reinterpret_cast<const half8 *>(Bl + (wn + j * 32 + li) * LDK + kk + lk);
            }
        };
        read_frags(0, 0);
#pragma unroll
        for (int t = 0; t < BK / 16; t++) {
            if (t + 1 < BK / 16) read_frags((t + 1) * 16, (t + 1) & 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[t & 1][i], bl[t & 1][j], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[t & 1][i], bh[t & 1][j], acc[i][j], 0, 0, 0);
                }
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads(); // barrier ks + 1
    }
    // D layout: lane -> column li; register r -> row 8 * (r / 4) + 4 * (lane / 32) + r % 4
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int gn = n0 + wn + j * 32 + li;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int gm = m0 + wm + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (gm < a.m && gn < a.n) {
                    if (!a.pair) {
                        if (a.ypart) a.ypart[((size_t)blockIdx.y * a.m + gm) * a.n + gn] = acc[i][j][r];
                        else a.y[(size_t)gm * a.n + gn] = acc[i][j][r] * (a.rowscale[gm] * (1.0f / T::WS));
                    } else if ((r & 1) == 0) { // gm is even: this register and the next hold the two parts of row gm / 2
                        const size_t t = (size_t)(gm >> 1);
                        const float v = acc[i][j][r] + acc[i][j][r + 1];
                        if (a.ypart) {
                            a.ypart[((size_t)blockIdx.y * (a.m >> 1) + t) * a.n + gn] = v;
                        } else {
                            float out = v * (a.rowscale[gm] * (1.0f / T::WS));
                            if (a.bias) out += a.bias[gn];
                            if (a.resid) out += a.resid[t * a.n + gn];
                            a.y[t * a.n + gn] = out;
                        }
                    }
                }
            }
        }
}

// ---------------------------------------------------------------------------
// Q4_K and Q5_K: one MFMA per product.
//
// A Q4_K weight is w = d * (sc * q) - dmin * m with a 4-bit code q, 6-bit sub-block scale sc and minimum m, and
// f16 d, dmin per 256-element superblock (GGUF layout); Q5_K is the same with a 5-bit code.  It goes through the matrix
// pipe as w = d * sc * (q - C) + (C d sc - dmin m) with C = 8 (16) in the middle of the codes:
//   - sc * (q - C) is an integer of magnitude <= 504 (1008), so it is EXACT in f16, and cheap to make: 0x6400 | n is the
//     f16 number 1024 + n for n < 1024, so q * sc + 0x6400 (one multiply-add on a pair of codes) less 1024 + 8 sc is
//     sc * (q - 8) (Q5_K: 1024 + q less 1040, times sc).  That is the B operand of the main loop; products x * sc * (q - C)
//     are exact in the f32 accumulator, and the superblock's d is applied to the accumulator, not to the weights:
//     the accumulator of an output column n holds the running sum in units of u_n, the d of the superblock being
//     added; at a superblock boundary it is multiplied by u_n / d_next (one multiply per accumulator register per
//     256 k; a lane of the 32x32 MFMA output owns one column, so the factor is one number per lane).  A superblock
//     with d = 0 contributes zeros and leaves the unit alone.
//   - the offset term, sum_g c[n, g] * (sum of x over sub-block g) with c = C d sc - dmin m, is a second, short GEMM
//     over K / 32 "columns" that runs through the same pipeline after the main loop: c goes in as two f16 (c S = ch + cl
//     under a power-of-two S chosen per column from the largest d and dmin it meets), the sub-block sums of x as two
//     f16 (hi + lo, written by the x pre-pass), three products hi ch + hi cl + lo ch laid side by side along the
//     extended K axis.
//   Why centred: with the codes as they are (0 .. 15) and - dmin m as the second term, both sums are a sub-block's
//   range times sum x, and for activation rows with a mean (all positive, say) each is a hundred times their difference:
//   their f32 rounding then shows in the result (4e-5 of a row's largest output at K = 4096, past the 1e-3 bound for its
//   small outputs).  Centred, the first sum is as well conditioned as the weights themselves and c is a sub-block's
//   middle, small for weights around zero: 2e-6.
// Against two MFMAs per product over all of K (the other block types below) this is 1 + 3/32.
//
// Tiling: a workgroup computes BM x 256 outputs with eight waves, each a block of 128 x 64 (BM = 256: 4 x 2 MFMA
// tiles) or 64 x 64 (BM = 128), and every thread also feeds: per K step of 64 it copies 64 bytes of the x tile and turns 32 codes of
// one weight row into operands for the step after the next one's... (two LDS stages, one barrier per step;
// the global loads of step s + 2 are in flight while step s + 1 is converted and step s multiplied).
// x is stored by the pre-pass with elements 1 and 2 of every group of four exchanged: the codes of a dword
// unpack to the pairs (0, 2) and (1, 3) with one mask each, and the order of k inside an MFMA is free as long
// as both operands agree.
// ---------------------------------------------------------------------------
constexpr int QBN = 256; // output columns (weight rows) per workgroup

// 6-bit scales and minimums of sub-blocks 2p, 2p + 1 (ggml get_scale_min_k4 order) as two bytes each
__device__ inline void q4k_scale_min(const u32x4 &h, int p, uint32_t &scp, uint32_t &mp) {
    const int sh = (p & 1) * 16;
    const uint32_t ya = h[1] >> sh, za = h[2] >> sh, wa = h[3] >> sh;
    if (p < 2) {
        scp = ya & 0x3F3F;
        mp = za & 0x3F3F;
    } else {
        scp = (wa & 0x0F0F) | ((ya >> 2) & 0x3030);
        mp = ((wa >> 4) & 0x0F0F) | ((za >> 2) & 0x3030);
    }
}


typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void gbl_void;

// s_waitcnt vmcnt(N) lgkmcnt(0) (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4 left at 7, lgkmcnt 11:8)
template <int N>
__device__ inline void wait_vm_and_lds() {
    __builtin_amdgcn_s_waitcnt(((N >> 4) << 14) | (7 << 4) | (N & 15));
}

template <int BM, int NT, bool Q5 = false>
__global__ void __launch_bounds__(NT) gemm_q4k_kernel(GemmArgs a) {
    constexpr int NW = NT / 64;          // waves: NW / 4 rows of four, each wave a block of WROWS x 64
    constexpr int WROWS = BM / (NW / 4); // 128 or 64
    constexpr int MI = WROWS / 32;       // MFMA tiles of a wave along M
    constexpr int BT = QBN * 2 / NT;     // (weight row, half) tasks per thread and step (1 or 2)
    constexpr int AROWS = BM / NW;       // x rows a wave brings in per step: XL loads of eight rows
    constexpr int XL = AROWS / 8;
    static_assert(AROWS % 16 == 0 && MI % 2 == 0 && BT >= 1, "tile shape");
    // LDS (halfs): three stages of the x tile, then two of the weight tile.  A tile row is 64 halfs, unpadded, its eight
    // 16-byte chunks stored at chunk ^ ((row / 2) & 7): x tiles are written by loads that go straight to LDS, 1 KB per
    // wave and instruction in lane order, so padding is not to be had; the exchange keeps the fragment reads of sixteen
    // consecutive rows, which LDS serves together, on distinct banks (64 banks of four bytes, even rows in the lower half).
    constexpr int ASTAGE = BM * 64, BSTAGE = QBN * 64, BOFF = 3 * ASTAGE;
    extern __shared__ _Float16 lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nt = (a.n + QBN - 1) / QBN, total = (int)gridDim.x;
    int tile = blockIdx.x;
    if (total % 8 == 0) tile = (tile & 7) * (total >> 3) + (tile >> 3); // workgroups of one XCD share x tiles
    const int m0 = (tile / nt) * BM, n0 = (tile % nt) * QBN;
    const int kbeg = (int)blockIdx.y * a.steps_per_split; // in steps of 64 k; a multiple of 4 (whole superblocks)
    const int t_main = a.k / BK - kbeg < a.steps_per_split ? a.k / BK - kbeg : a.steps_per_split;
    const int nsb = t_main >> 2;         // superblocks of this workgroup's part of K
    const int t_min = (nsb + 1) >> 1;
    const int last_sb = (a.k >> 8) - 1;

    // ---- feeder side.  Addresses are (uniform 64-bit base of the workgroup) + (32-bit offset of the thread).  The x
    // rows of the scratch buffer are allocated up to a multiple of BM, so they need no clamp; weight rows past the end
    // are clamped.
    // What a thread holds of a group of four steps: main loop = one superblock: the 16 code bytes of its (row, half) for
    // each of the four pairs (64 consecutive bytes in memory) and the superblock's header; minimum term: the headers of
    // the four steps' superblocks (in q) -- five, or four, loads per task and group.
    // Q5_K: also the 16 bytes of fifth bits that go with the thread's code bytes (one set per superblock: bit 2 p and
    // 2 p + 1 of a byte belong to the two sub-blocks of pair p).
    struct Raw { u32x4 q[BT][4]; u32x4 h[BT]; u32x4 b[BT]; };
    const uint8_t *xbase = reinterpret_cast<const uint8_t *>(a.xh + (size_t)m0 * a.k + (size_t)kbeg * BK);
    const uint8_t *x3base = reinterpret_cast<const uint8_t *>(a.xs3 + (size_t)m0 * a.xs3_pitch + (size_t)(kbeg >> 2) * 32);
    // a lane's part of a wave's x load: row lane / 8 of the eight, and the chunk that belongs at slot lane % 8 of that row:
    // slot ^ ((row / 2) & 7) -- for the rows of load i that is (lane % 8) ^ (lane / 16) ^ 4 (i & 1)
    const uint32_t xrow_l = (uint32_t)(wave * AROWS + (lane >> 3)), xchunk_l = (uint32_t)((lane & 7) ^ (lane >> 4));
    const uint32_t xoff = (xrow_l * (uint32_t)a.k + xchunk_l * 8) * 2, x3off = (xrow_l * (uint32_t)a.xs3_pitch + xchunk_l * 8) * 2;
    const size_t x8rows = (size_t)8 * a.k * 2, x38rows = (size_t)8 * a.xs3_pitch * 2;
    const uint8_t *cbase = a.codes + (size_t)n0 * a.codes_pitch, *mbase = a.meta + (size_t)n0 * a.meta_pitch;
    const uint8_t *qbase = Q5 ? a.qh + (size_t)n0 * a.qh_pitch : nullptr;
    uint32_t coff[BT], moff[BT], qoff[BT];
    const int cpr = a.k >> 6; // pairs of sub-blocks (K steps) per row
    const int bh = tid & 1;   // which 16 bytes of a pair's 32 (NT is even: the same for every task of the thread)
    int b_wr[BT];             // where the thread's operands go in a weight stage (halfs): row, and the chunk exchange
#pragma unroll
    for (int u = 0; u < BT; u++) {
        const int row = (tid + u * NT) >> 1;
        const int crow = n0 + row < a.n ? row : a.n - 1 - n0;
        coff[u] = (uint32_t)crow * (uint32_t)a.codes_pitch;
        moff[u] = (uint32_t)crow * (uint32_t)a.meta_pitch;
        qoff[u] = Q5 ? (uint32_t)crow * (uint32_t)a.qh_pitch + (uint32_t)(bh * 16) : 0u;
        b_wr[u] = row * 64 + ((((row >> 1) & 7) ^ (bh * 2)) * 8);
    }
    // x tile of main step `step` (or, MIN, of step s2 of the minimum term, clamped to the last) -> x stage `stage`
    auto load_x = [&](auto is_min, int step, int stage) {
        constexpr bool MIN = decltype(is_min)::value;
        if (MIN) step = step < t_min ? step : t_min - 1;
        const uint8_t *g = (MIN ? x3base : xbase) + (size_t)step * (BK * 2);
        const uint32_t off = MIN ? x3off : xoff;
        const size_t rows8 = MIN ? x38rows : x8rows;
        _Float16 *dst = lds + stage * ASTAGE + wave * AROWS * 64;
#pragma unroll
        for (int i = 0; i < AROWS / 8; i++)
            __builtin_amdgcn_global_load_lds((gbl_void *)(g + i * rows8 + ((i & 1) ? off ^ 64u : off)), (lds_void *)(dst + i * 8 * 64), 16, 0, 0);
        asm volatile("" ::: "memory"); // what is requested after this stays after it: the waits in front of the barriers count on the order
    };
    // Main loop: the packed weights of superblock `sb` (0 .. nsb - 1, clamped) of this workgroup's part of K.
    auto fetch_main = [&](int sb, Raw &r) {
        sb = sb < nsb ? sb : nsb - 1;
        const int pair = kbeg + 4 * sb, slice = pair >> 6, pr = pair & 63; // the four pairs of a superblock share a slice
        int P = cpr - (slice << 6);
        P = P < 64 ? P : 64;
        const uint8_t *cb = cbase + (size_t)slice * 2048 + (size_t)pr * 16, *mb = mbase + (size_t)(pair >> 2) * 16;
        const uint32_t hoff = (uint32_t)(bh * 16 * P);
#pragma unroll
        for (int u = 0; u < BT; u++) {
#pragma unroll
            for (int j = 0; j < 4; j++) r.q[u][j] = *reinterpret_cast<const u32x4 *>(cb + j * 16 + (coff[u] + hoff));
            r.h[u] = *reinterpret_cast<const u32x4 *>(mb + moff[u]);
            if constexpr (Q5) r.b[u] = *reinterpret_cast<const u32x4 *>(qbase + (size_t)(pair >> 2) * 32 + qoff[u]);
        }
    };
    // The minimum term: steps 4 grp .. 4 grp + 3 (clamped to the last step); a step = 64 columns = two superblocks of
    // [hi | hi | lo | 0] x [ch | cl | ch | 0], of which the thread makes one
    auto fetch_min = [&](int grp, Raw &r) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int s2 = 4 * grp + j;
            s2 = s2 < t_min ? s2 : t_min - 1;
            int sb = (kbeg >> 2) + 2 * s2 + bh;
            sb = sb < last_sb ? sb : last_sb;
#pragma unroll
            for (int u = 0; u < BT; u++) r.q[u][j] = *reinterpret_cast<const u32x4 *>(mbase + (size_t)sb * 16 + moff[u]);
        }
    };
    // While the offset term is added the accumulators of a column hold the result times S, a power of two chosen from the
    // largest |d| or |dmin| (f16 bits) the column's weight row has in this part of K: both < 2^(e + 1) -> |c| < 63 * 17 *
    // 2^(e + 1) < 2^(e + 12), the operands are c * 2^(3 - e) < 2^15; they meet sub-block sums stored times 1 / 64, so
    // S = 2^(-3 - e).  All zero, or inf / nan: e = 8.  The feeder of a row and the lanes that own its column both work it
    // out from the row's headers.
    auto s_of = [](uint32_t mx) {
        const int e = (mx == 0 || mx >= 0x7C00u) ? 8 : (mx >= 0x400u ? (int)(mx >> 10) - 15 : -15);
        return __builtin_bit_cast(float, (uint32_t)(127 - 3 - e) << 23);
    };
    uint32_t dmax_r[BT];
#pragma unroll
    for (int u = 0; u < BT; u++) dmax_r[u] = 0;
    // half c1 (0, 1) of the conversion of main-loop step j (0..3) of the superblock in `r` into weight stage `stage`: bytes
    // 8 c1 .. 8 c1 + 7 of the thread's 16, i.e. elements 16 bh + 8 c1 .. of both sub-blocks = chunk 2 bh + c1 of the row
    // (low nibbles) and the chunk four further (high nibbles)
    auto convert_main = [&](const Raw &r, int j, int stage, int c1) {
        _Float16 *bs = lds + BOFF + stage * BSTAGE;
        const int p = j; // kbeg is a multiple of 4: step j of a superblock is its pair j
#pragma unroll
        for (int u = 0; u < BT; u++) {
            uint32_t scp, mp;
            q4k_scale_min(r.h[u], p, scp, mp);
            const uint32_t dd = r.h[u][0];
            scp = (dd & 0x7FFFu) == 0 ? 0u : scp; // d = 0: the superblock adds nothing and leaves the unit alone
            const uint32_t dm = (dd >> 16) & 0x7FFFu, da = dd & 0x7FFFu;
            dmax_r[u] = dm > dmax_r[u] ? dm : dmax_r[u];
            dmax_r[u] = da > dmax_r[u] ? da : dmax_r[u];
            const uint32_t s0 = scp & 0xFF, s1 = scp >> 8;
            uint32_t lo[4], hi[4];
            auto bits = [](half2v v) { return __builtin_bit_cast(uint32_t, v); };
            auto halfs = [](uint32_t v) { return __builtin_bit_cast(half2v, v); };
            auto pk2 = [](float v) { return __builtin_bit_cast(half2v, __builtin_amdgcn_cvt_pkrtz(v, v)); }; // v twice; exact for these
            constexpr uint32_t K1024 = 0x64006400u; // 0x6400 | n is the f16 number 1024 + n for n < 1024
            if constexpr (Q5) {
                // (q - 16) * sc: 1024 + q less 1040, times sc, every step exact in f16 (|.| <= 16 * 63)
                const half2v m0 = pk2((float)s0), m1 = pk2((float)s1);
                const half2v off = {(_Float16)-1040.0f, (_Float16)-1040.0f};
#pragma unroll
                for (int d = 0; d < 2; d++) {
                    const uint32_t w = r.q[u][j][2 * c1 + d], f = r.b[u][2 * c1 + d];
                    const uint32_t fl = p < 2 ? f << (4 - 2 * p) : (p == 2 ? f : f >> 2); // bit 2 p of every byte at bit 4
                    const uint32_t fh = p < 2 ? f << (3 - 2 * p) : f >> (2 * p - 3);      // bit 2 p + 1
                    const uint32_t ql = (w & 0x0F0F0F0Fu) | (fl & 0x10101010u), qh = ((w >> 4) & 0x0F0F0F0Fu) | (fh & 0x10101010u);
                    lo[2 * d] = bits((halfs((ql & 0x001F001Fu) | K1024) + off) * m0);
                    lo[2 * d + 1] = bits((halfs(((ql >> 8) & 0x001F001Fu) | K1024) + off) * m0);
                    hi[2 * d] = bits((halfs((qh & 0x001F001Fu) | K1024) + off) * m1);
                    hi[2 * d + 1] = bits((halfs(((qh >> 8) & 0x001F001Fu) | K1024) + off) * m1);
                }
            } else {
                // (q - 8) * sc: q * sc <= 945 as an integer, 1024 + that as f16, less 1024 + 8 sc (exact: below 2048)
                const float f0 = -1024.0f - (float)(8 * s0), f1 = -1024.0f - (float)(8 * s1);
                const half2v o0 = pk2(f0), o1 = pk2(f1);
#pragma unroll
                for (int d = 0; d < 2; d++) {
                    const uint32_t w = r.q[u][j][2 * c1 + d];
                    lo[2 * d] = bits(halfs((w & 0x000F000Fu) * s0 + K1024) + o0);
                    lo[2 * d + 1] = bits(halfs(((w >> 8) & 0x000F000Fu) * s0 + K1024) + o0);
                    hi[2 * d] = bits(halfs(((w >> 4) & 0x000F000Fu) * s1 + K1024) + o1);
                    hi[2 * d + 1] = bits(halfs(((w >> 12) & 0x000F000Fu) * s1 + K1024) + o1);
                }
            }
            const int at = b_wr[u] ^ (c1 * 8);
            *reinterpret_cast<u32x4 *>(bs + at) = u32x4{lo[0], lo[1], lo[2], lo[3]};
            *reinterpret_cast<u32x4 *>(bs + (at ^ 32)) = u32x4{hi[0], hi[1], hi[2], hi[3]};
        }
    };
    // part t (0..3) of step s2 of the minimum term, whose headers are q[.][j] of `r` (an odd count of superblocks: the
    // second half of the last step gets zeros, which meet the sums of the next superblock, or the zeros that end an x row)
    float S_r[BT];
    auto convert_min = [&](int s2, const Raw &r, int j, int stage, int t) {
        _Float16 *bs = lds + BOFF + stage * BSTAGE;
        const bool live = 2 * s2 + bh < nsb;
#pragma unroll
        for (int u = 0; u < BT; u++) {
            const u32x4 h = r.q[u][j];
            const float s64 = live ? 64.0f * S_r[u] : 0.f;
            const float dmin = h2f(h[0] >> 16), dc = (Q5 ? 16.0f : 8.0f) * h2f(h[0] & 0xFFFFu);
            uint32_t o[4];
#pragma unroll
            for (int p = 0; p < 4; p++) {
                uint32_t scp, mp;
                q4k_scale_min(h, p, scp, mp);
                // what the centred codes leave: (8 or 16) d sc - dmin m per sub-block, both products exact (11 x 6 bits)
                const float c0 = s64 * (dc * ubyte<0>(scp) - dmin * ubyte<0>(mp)), c1 = s64 * (dc * ubyte<1>(scp) - dmin * ubyte<1>(mp));
                const float h0 = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, c0) & 0xFFFFE000u);
                const float h1 = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, c1) & 0xFFFFE000u);
                const float v0 = t == 1 ? c0 - h0 : h0, v1 = t == 1 ? c1 - h1 : h1; // t: 0 ch, 1 cl, 2 ch, 3 nothing
                o[p] = t == 3 ? 0u : __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(v0, v1));
            }
            // chunk 4 bh + t of the row; b_wr holds chunk 2 bh (and the exchange)
            *reinterpret_cast<u32x4 *>(bs + (b_wr[u] ^ (((bh * 6) ^ t) * 8))) = u32x4{o[0], o[1], o[2], o[3]};
        }
    };

    // ---- multiplier side
    const int wm = (wave >> 2) * WROWS, wn = (wave & 3) * 64;
    const int li = lane & 31, hh = lane >> 5;
    // fragment of sub-step t: tile row r = w + 32 i + li, chunk 2 t + hh, stored at chunk ^ ((r / 2) & 7): the address is
    // (r * 64 + ((hh ^ (li / 2)) & 7) * 8) ^ (16 t) in halfs
    const int sw = ((hh ^ (li >> 1)) & 7) * 8;
    const int a_rd = (wm + li) * 64 + sw, b_rd = BOFF + (wn + li) * 64 + sw;
    float16v acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
    uint32_t doff[2]; // this lane's two output columns: their superblock headers
    float unit[2] = {1.0f, 1.0f};
    uint32_t dnext[2], dmax_c[2] = {0, 0};
#pragma unroll
    for (int j = 0; j < 2; j++) {
        int col = wn + j * 32 + li;
        col = n0 + col < a.n ? col : a.n - 1 - n0;
        doff[j] = (uint32_t)col * (uint32_t)a.meta_pitch;
        dnext[j] = *reinterpret_cast<const uint32_t *>(mbase + (size_t)(kbeg >> 2) * 16 + doff[j]);
    }
    // a new superblock (index sb of the row): the accumulators change their unit to its d (no branches: the loads at the end
    // must be the same on every path, see load_x)
    auto new_unit = [&](int sb) {
        const int sbn = sb + 1 < last_sb ? sb + 1 : last_sb;
        float r[2];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const float dn = h2f(dnext[j] & 0xFFFFu);
            const uint32_t dm = (dnext[j] >> 16) & 0x7FFFu, da = dnext[j] & 0x7FFFu;
            dmax_c[j] = dm > dmax_c[j] ? dm : dmax_c[j];
            dmax_c[j] = da > dmax_c[j] ? da : dmax_c[j];
            const bool some = dn != 0.f;
            const float q = unit[j] / (some ? dn : 1.0f);
            r[j] = some ? q : 1.0f;
            unit[j] = some ? dn : unit[j];
            dnext[j] = *reinterpret_cast<const uint32_t *>(mbase + (size_t)sbn * 16 + doff[j]);
        }
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int q = 0; q < 16; q++) acc[i][j][q] *= r[j];
    };
    // the eight MFMAs of sub-step t (x stage at halfs `as`, weight stage PAR); the x fragments two at a time: registers
    // are short, and while this wave waits for fragments the other wave of its SIMD multiplies
    auto multiply = [&](int as, int par, int t) {
        half8 bf[2];
#pragma unroll
        for (int j = 0; j < 2; j++) bf[j] = *reinterpret_cast<const half8 *>(lds + par * BSTAGE + (b_rd ^ (t * 16)) + j * 32 * 64);
#pragma unroll
        for (int ih = 0; ih < MI / 2; ih++) {
            half8 af[2];
#pragma unroll
            for (int i = 0; i < 2; i++) af[i] = *reinterpret_cast<const half8 *>(lds + as + (a_rd ^ (t * 16)) + (2 * ih + i) * 32 * 64);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[2 * ih + i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[2 * ih + i][j], 0, 0, 0);
        }
    };
    // The steps of the main loop and of the minimum term are numbered through, g = 0 .. t_main + t_min - 1, and taken in
    // groups of four (a superblock of the main loop; four steps of the minimum term).  Step g multiplies x stage g % 3 with
    // weight stage g & 1, brings the x tile of step g + 2 into its stage and converts the packed weights of step g + 1
    // into the other weight stage; the first step of a group also requests the packed weights of the next group.  Every
    // path through a step issues the same loads in the same order, so that the wait in front of its barrier (for the
    // x tile of step g + 1, requested a step ago) can leave the younger requests in flight.
    Raw cur, nxt; // this group's packed weights, the next group's
    const int sb0 = kbeg >> 2;
    int g3 = 0;   // g % 3
    // One group.  KG, KN, KF: kind (0 main, 1 minimum term) of this group, the next one, and the one after (whose x tiles
    // this one does not touch); grp: index of the group among those of its kind.
    auto group = [&](auto kg, auto kn, int grp) {
        constexpr bool KG = decltype(kg)::value, KN = decltype(kn)::value;
        constexpr int F = KN ? 4 * BT : (Q5 ? 6 : 5) * BT; // loads of the weight request
        if (!KG) new_unit(sb0 + grp);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if (KG && 4 * grp + i >= t_min) break; // the minimum term's last group may be short (the same for every wave)
            const int as = g3 * ASTAGE, xs = (g3 == 0 ? 2 : g3 - 1); // x stages g % 3 and (g + 2) % 3
            // x tile of step g + 2: of this group (i < 2) or the next
            if (i < 2) load_x(kg, 4 * grp + i + 2, xs);
            else load_x(kn, (KG == KN ? 4 * grp + 4 : 0) + i - 2, xs);
            if (i == 0) {
                if (KN) fetch_min(KG ? grp + 1 : 0, nxt);
                else fetch_main(grp + 1, nxt);
            }
#pragma unroll
            for (int t = 0; t < BK / 16; t++) {
                multiply(as, i & 1, t);
                // step g + 1: of this group (i < 3) or the first of the next
                if (i < 3) {
                    if (KG) {
                        if (4 * grp + i + 1 < t_min) convert_min(4 * grp + i + 1, cur, i + 1, (i + 1) & 1, t);
                    } else if (t & 1) {
                        convert_main(cur, i + 1, (i + 1) & 1, t >> 1);
                    }
                } else {
                    if (KN) {
                        const int s2 = KG ? 4 * grp + 4 : 0;
                        if (s2 < t_min) convert_min(s2, nxt, 0, 0, t);
                    } else if (t & 1) {
                        convert_main(nxt, 0, 0, t >> 1);
                    }
                }
            }
            // younger than the x tile of step g + 1: see the order of the loads above
            if (i == 0) wait_vm_and_lds<(KG ? 0 : 2) + XL + F>();
            else if (i == 1) wait_vm_and_lds<F + XL>();
            else wait_vm_and_lds<XL>();
            lds_barrier();
            g3 = g3 == 2 ? 0 : g3 + 1;
            if (i == 2 && !KG && KN) {
#pragma unroll
                for (int u = 0; u < BT; u++) S_r[u] = s_of(dmax_r[u]); // every header of the thread's rows has been looked at
            }
        }
        cur = nxt;
    };
    using MAIN = std::false_type;
    using MIN = std::true_type;

    load_x(MAIN{}, 0, 0);
    load_x(MAIN{}, 1, 1);
    fetch_main(0, cur);
    convert_main(cur, 0, 0, 0);
    convert_main(cur, 0, 0, 1);
    wait_vm_and_lds<0>();
    lds_barrier();
    for (int sb = 0; sb < nsb - 1; sb++) group(MAIN{}, MAIN{}, sb); // every superblock but the last
    group(MAIN{}, MIN{}, nsb - 1); // the last: what it requests and prepares beyond itself belongs to the minimum term
    // the main sum in true units, times S: the minimum term joins it
    float S_c[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        S_c[j] = s_of(dmax_c[j]);
        const float f = unit[j] * S_c[j];
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int q = 0; q < 16; q++) acc[i][j][q] *= f;
    }
    for (int grp = 0; 4 * grp < t_min; grp++) group(MIN{}, MIN{}, grp);
    wait_vm_and_lds<0>(); // nothing of this workgroup may still be on its way into LDS when it ends
    // D layout: lane -> column li; register r -> row 8 * (r / 4) + 4 * (lane / 32) + r % 4
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int gn = n0 + wn + j * 32 + li;
            const float inv_s = 1.0f / S_c[j];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int gm = m0 + wm + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (gm < a.m && gn < a.n) {
                    if (!a.pair) {
                        if (a.ypart) a.ypart[((size_t)blockIdx.y * a.m + gm) * a.n + gn] = acc[i][j][r] * inv_s;
                        else a.y[(size_t)gm * a.n + gn] = acc[i][j][r] * (a.rowscale[gm] * inv_s);
                    } else if ((r & 1) == 0) { // gm is even: this register and the next hold the two parts of row gm / 2
                        const size_t t = (size_t)(gm >> 1);
                        const float v = (acc[i][j][r] + acc[i][j][r + 1]) * inv_s;
                        if (a.ypart) {
                            a.ypart[((size_t)blockIdx.y * (a.m >> 1) + t) * a.n + gn] = v;
                        } else {
                            float out = v * a.rowscale[gm];
                            if (a.bias) out += a.bias[gn];
                            if (a.resid) out += a.resid[t * a.n + gn];
                            a.y[t * a.n + gn] = out;
                        }
                    }
                }
            }
        }
}

// ---------------------------------------------------------------------------
// Q4_0 / Q4_1 / Q5_0 / Q5_1 / Q8_0 (blocks of 32): one MFMA per product, the block's scale applied by the vector ALU.
//
// w = d * (q - c) (Q4_0: c = 8, Q5_0: 16, Q8_0: the code is a signed byte) or d * q + m (Q4_1, Q5_1) with f16 d (and
// m) per block of 32.  The B operand is the centred code q - c itself, an integer that f16 holds exactly: the two
// MFMAs of a block (32 k) start from zero, so their result is the block's sum of (q - c) * x, exact in f32 to within
// the accumulation, and every lane then adds it, times the d of its column and block, into its accumulators (a lane of
// the 32 x 32 MFMA output owns one column): sixteen v_fma per tile and block where gemm_kernel pays a second MFMA per
// product and about ten vector-ALU instructions per weight for the dequantisation and the high/low split.  Converting
// costs two instructions per pair of weights: the code pairs come out of the packed nibbles two at a time with one mask
// each (Q4: after one byte permutation, its neighbours share a byte; Q8_0: bytes 0, 2 and 1, 3 of a dword), Q5's fifth
// bits out of qh four at a time with one multiplication, 0x6400 | q is the f16 number 1024 + q, and one packed
// subtraction of 1024 + c centres it.  x is stored with elements 1 and 2 of every four exchanged, as for the Q4_K
// kernel, which is the order the masks produce.
// The types with a minimum go in as d * (q - c) + (m + c d): the first sum is then as well conditioned as the weights
// themselves (with q as it is, two sums three times the size of the result would cancel in f32).  The second,
// sum_b (m + c d)[n, b] * (sum of x over block b), goes through the matrix pipe too, two MFMAs per tile and
// superblock of 256 k: A = the eight block sums of the row as f16 pairs (hi for k 0..7, lo for k 8..15, written by the
// x pre-pass for the Q4_K kernel's offset term, times 1 / 64), B = the column's eight offsets m + c d as f16 pairs
// (the leading halves twice, then the remainders against the sums' leading halves); the sum is added times 256 and
// the main term's scales are d * 256 / 64 to match.
//
// The pipeline is the Q4_K kernel's: BM x 128 outputs per workgroup of eight waves (BM = 256: 64 x 64 each; 128: 32 x 64),
// x tiles straight from memory into three LDS stages, two weight stages, one barrier per K step that waits for LDS only,
// explicit counts of the loads issued since.  A thread converts half a block (16 weights of one row) per step.  The
// scale records of the tile's columns lie in LDS too, a superblock of them at a time.
// ---------------------------------------------------------------------------
constexpr int PBN = 128; // output columns (weight rows) per workgroup
constexpr float XSUM_SCALE = 1.0f / 64.0f; // the x pre-pass stores the block sums times this

template <int BITS, bool WITH_MIN, int BM>
__global__ void __launch_bounds__(512) gemm_blk32_kernel(GemmArgs a) {
    constexpr int NW = 8, AROWS = BM / NW, XL = AROWS / 8; // BM = 256 or 128 rows of x per workgroup
    constexpr int MI = BM / 128;                           // MFMA tiles of a wave along M: the waves lie 4 x 2, (32 MI) x 64 each
    constexpr int ASTAGE = BM * 64, BSTAGE = PBN * 64, BOFF = 3 * ASTAGE; // halfs
    constexpr int F = BITS == 5 ? 2 : 1;   // loads of a weight request: codes (and fifth bits)
    constexpr int CENTER = BITS == 5 ? 16 : BITS == 4 ? 8 : 128; // the codes go in centred (Q5_0's, Q4_0's and Q8_0's own form)
    constexpr int ML = 1;                  // per superblock: this wave's kilobyte of scale records
    constexpr float OFF = 1024.0f + CENTER; // 0x6400 | q is 1024 + q
    constexpr float ASCALE = WSCALE * XSUM_SCALE; // the accumulators hold the result times this
    extern __shared__ _Float16 lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nt = (a.n + PBN - 1) / PBN, total = (int)gridDim.x;
    int tile = blockIdx.x;
    if (total % 8 == 0) tile = (tile & 7) * (total >> 3) + (tile >> 3); // workgroups of one XCD share x tiles
    const int m0 = (tile / nt) * BM, n0 = (tile % nt) * PBN;
    const int kbeg = (int)blockIdx.y * a.steps_per_split; // in steps of 64 k; a multiple of 4 (whole superblocks)
    const int T = a.k / BK - kbeg < a.steps_per_split ? a.k / BK - kbeg : a.steps_per_split; // a multiple of 4

    // ---- x tiles (rows of the scratch buffer are allocated up to a multiple of BM: no clamp)
    const uint8_t *xbase = reinterpret_cast<const uint8_t *>(a.xh + (size_t)m0 * a.k + (size_t)kbeg * BK);
    const uint32_t xrow_l = (uint32_t)(wave * AROWS + (lane >> 3)), xchunk_l = (uint32_t)((lane & 7) ^ (lane >> 4));
    const uint32_t xoff = (xrow_l * (uint32_t)a.k + xchunk_l * 8) * 2;
    const size_t x8rows = (size_t)8 * a.k * 2;
    auto load_x = [&](int step, int stage) {
        step = step < T ? step : T - 1;
        const uint8_t *g = xbase + (size_t)step * (BK * 2);
        _Float16 *dst = lds + stage * ASTAGE + wave * AROWS * 64;
#pragma unroll
        for (int i = 0; i < XL; i++)
            __builtin_amdgcn_global_load_lds((gbl_void *)(g + i * x8rows + ((i & 1) ? xoff ^ 64u : xoff)), (lds_void *)(dst + i * 8 * 64), 16, 0, 0);
        asm volatile("" ::: "memory"); // what is requested after this stays after it: the waits in front of the barriers count on the order
    };

    // ---- weights: this thread's half block (16 weights) of every step
    const int wrow = tid & 127, bis = tid >> 8, half = (tid >> 7) & 1; // row of the tile; which of the step's two blocks; which half of it
    const int crow = n0 + wrow < a.n ? n0 + wrow : a.n - 1;
    const uint8_t *cp = a.codes + (size_t)crow * a.codes_pitch, *qp = BITS == 5 ? a.qh + (size_t)crow * a.qh_pitch : nullptr;
    struct Raw { u32x4 q; uint32_t qh; };
    // the thread's block of a step: 16 bytes of nibbles (Q5: both halves fetch all of them, they interleave), or its own
    // 16 of the block's 32 bytes (Q8_0)
    auto fetch = [&](int step, Raw &r) {
        step = step < T ? step : T - 1;
        const size_t blk = (size_t)(kbeg + step) * 2 + bis;
        r.q = *reinterpret_cast<const u32x4 *>(BITS == 8 ? cp + blk * 32 + half * 16 : cp + blk * 16);
        if (BITS == 5) r.qh = *reinterpret_cast<const uint32_t *>(qp + blk * 4);
        asm volatile("" ::: "memory");
    };
    const int b_wr = wrow * 64; // the thread's row in a weight plane; chunk ch of it lies at (ch ^ ((wrow / 2) & 7)) * 8
    const int b_sw = (wrow >> 1) & 7;
    // chunk c = 2 half + cc (cc = 0, 1: elements 8 c .. 8 c + 7) of the block in `r` -> weight stage `stage`, as pairs of
    // codes in the two halves of a dword, in the order [e0, e2, e1, e3, e4, e6, e5, e7]
    auto convert = [&](const Raw &r, int cc, int stage) {
        const int c = 2 * half + cc;
        uint32_t pr[4];
        if (BITS == 5) { // GGUF: byte j = elements j (low nibble) and j + 16 (high); qh bit e = bit 4 of element e
            const uint32_t d0 = cc ? r.q[2] : r.q[0], d1 = cc ? r.q[3] : r.q[1];
            const int sh = half * 4;
            pr[0] = (d0 >> sh) & 0x000F000Fu; pr[1] = (d0 >> (sh + 8)) & 0x000F000Fu;
            pr[2] = (d1 >> sh) & 0x000F000Fu; pr[3] = (d1 >> (sh + 8)) & 0x000F000Fu;
            // bits b0..b3 of `four` times (2^4 + 2^18): b0 lands on bit 4 and b2 on bit 20 (of the pair e, e + 2), nothing else does
            const uint32_t eight = (r.qh >> (8 * c)) & 0xFFu;
            pr[0] |= ((eight & 0xFu) * 0x40010u) & 0x00100010u;
            pr[1] |= (((eight >> 1) & 0x7u) * 0x40010u) & 0x00100010u;
            pr[2] |= ((eight >> 4) * 0x40010u) & 0x00100010u;
            pr[3] |= ((eight >> 5) * 0x40010u) & 0x00100010u;
        } else if (BITS == 4) { // reference nibble order: byte i = elements 2 i (low), 2 i + 1 (high): dword c is the chunk
            const uint32_t w = half ? (cc ? r.q[3] : r.q[2]) : (cc ? r.q[1] : r.q[0]);
            const uint32_t p4 = __builtin_amdgcn_perm(w, w, 0x03010200u); // bytes 0, 2, 1, 3: a half dword = two neighbours
            pr[0] = p4 & 0x000F000Fu; pr[1] = (p4 >> 4) & 0x000F000Fu;
            pr[2] = (p4 >> 8) & 0x000F000Fu; pr[3] = (p4 >> 12) & 0x000F000Fu;
        } else { // signed bytes in element order, as unsigned ones (+ 128)
            const uint32_t x0 = (cc ? r.q[2] : r.q[0]) ^ 0x80808080u, x1 = (cc ? r.q[3] : r.q[1]) ^ 0x80808080u;
            pr[0] = x0 & 0x00FF00FFu; pr[1] = (x0 >> 8) & 0x00FF00FFu;
            pr[2] = x1 & 0x00FF00FFu; pr[3] = (x1 >> 8) & 0x00FF00FFu;
        }
        const half2v off2 = {(_Float16)OFF, (_Float16)OFF};
        uint32_t oh[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t bits = pr[i] | 0x64006400u;
            const half2v qf = __builtin_bit_cast(half2v, bits) - off2; // exact: integers below 2048
            oh[i] = __builtin_bit_cast(uint32_t, qf);
        }
        _Float16 *bs = lds + BOFF + stage * BSTAGE + b_wr + (((4 * bis + c) ^ b_sw) * 8);
        *reinterpret_cast<u32x4 *>(bs) = u32x4{oh[0], oh[1], oh[2], oh[3]};
    };

    // ---- multiplier side
    const int wm = (wave >> 1) * (32 * MI), wn = (wave & 1) * 64;
    const int li = lane & 31, hh = lane >> 5;
    const int sw = ((hh ^ (li >> 1)) & 7) * 8;
    const int a_rd = (wm + li) * 64 + sw, b_rd = BOFF + (wn + li) * 64 + sw;
    float16v acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
    // The scale records of the tile's 128 columns, eight blocks of a superblock each ((d, m) pairs for Q5_1: 32 bytes;
    // d alone for Q5_0: 16 bytes), lie in LDS behind the weight stages, two superblocks of them: every wave brings in a
    // kilobyte of the next superblock's at the first step of a superblock (the same kilobyte twice or four times over:
    // one request per wave keeps the waves' counts of loads equal).
    constexpr int RV = WITH_MIN ? 2 : 1;      // 16-byte vectors per column and superblock
    constexpr int RECB = PBN * 16 * RV;       // bytes of one superblock's records
    uint8_t *rec_lds = reinterpret_cast<uint8_t *>(lds + BOFF + 2 * BSTAGE);
    const int nsb = T >> 2;
    const int rc0 = WITH_MIN ? (wave & 3) * 32 : (wave & 1) * 64; // first column of this wave's kilobyte
    int rcol = n0 + rc0 + (WITH_MIN ? lane >> 1 : lane);
    rcol = rcol < a.n ? rcol : a.n - 1;
    const uint8_t *rsrc = a.meta + (size_t)rcol * a.meta_pitch + (size_t)(kbeg >> 2) * (16 * RV) + (WITH_MIN ? (lane & 1) * 16 : 0);
    auto fetch_records = [&](int sb) {
        sb = sb < nsb ? sb : nsb - 1;
        __builtin_amdgcn_global_load_lds((gbl_void *)(rsrc + (size_t)sb * (16 * RV)), (lds_void *)(rec_lds + (sb & 1) * RECB + rc0 * 16 * RV), 16, 0, 0);
        asm volatile("" ::: "memory");
    };
    u32x4 mx[MI];
    const uint8_t *x3p = reinterpret_cast<const uint8_t *>(a.xs3 + (size_t)(m0 + wm + li) * a.xs3_pitch + (size_t)(kbeg >> 2) * 32 + hh * 16);
    auto fetch_sums = [&](int sb) {
#pragma unroll
        for (int i = 0; i < MI; i++) mx[i] = *reinterpret_cast<const u32x4 *>(x3p + ((size_t)i * 32 * a.xs3_pitch + (size_t)sb * 32) * 2);
    };
    // d of block bq (0..7) of superblock sb, column j of this lane, times WSCALE
    const uint8_t *rlane = rec_lds + (wn + li) * 16 * RV;
    auto scale_of = [&](int sb, int j, int bq) {
        const uint16_t w = *reinterpret_cast<const uint16_t *>(rlane + (sb & 1) * RECB + j * 32 * 16 * RV + bq * (WITH_MIN ? 4 : 2));
        return ASCALE * h2f(w);
    };
    // One block of 32 k = two sub-steps t0 = 2 hb, t0 + 1 of the step: its sum over k, then times the block's d into the
    // accumulators.  bq: the block's number in the superblock.
    auto multiply_block = [&](int as, int par, int hb, int sb, int bq) {
        const float16v zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        const int t0 = 2 * hb, t1 = 2 * hb + 1;
        const float df[2] = {scale_of(sb, 0, bq), scale_of(sb, 1, bq)};
        half8 b0[2], b1[2]; // the block's weight fragments serve both row tiles
#pragma unroll
        for (int j = 0; j < 2; j++) {
            b0[j] = *reinterpret_cast<const half8 *>(lds + par * BSTAGE + (b_rd ^ (t0 * 16)) + j * 32 * 64);
            b1[j] = *reinterpret_cast<const half8 *>(lds + par * BSTAGE + (b_rd ^ (t1 * 16)) + j * 32 * 64);
        }
#pragma unroll
        for (int i = 0; i < MI; i++) { // one row tile's two sums at a time: registers
            const half8 a0 = *reinterpret_cast<const half8 *>(lds + as + (a_rd ^ (t0 * 16)) + i * 32 * 64);
            const half8 a1 = *reinterpret_cast<const half8 *>(lds + as + (a_rd ^ (t1 * 16)) + i * 32 * 64);
            float16v S[2];
#pragma unroll
            for (int j = 0; j < 2; j++) S[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, b0[j], zero, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 2; j++) S[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, b1[j], S[j], 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = fmaf(S[j][r], df[j], acc[i][j][r]);
        }
    };
    auto multiply_min = [&](int sb) {
        // B = the blocks' offsets m + CENTER d (the weight of the middle code), each worked out in f32 (exact to its last
        // bit) and cut into two f16, vh + vl: the first product takes [vh | vh] against the sums' [hi | lo], the second
        // [vl | 0].  Kept apart (m against the sums, then CENTER d against the sums, added afterwards) the two halves of the
        // offset are each as large as a block's range times sum x and cancel in f32: 1.1e-3 at the strict floor of the
        // parity test for rows with a mean; together they are the block's middle, small for weights around zero.  An
        // offset beyond f16's range (weights past 65504) saturates.
        half8 bh[2], bl[2];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            uint32_t oh[4], ol[4];
#pragma unroll
            for (int q = 0; q < 4; q++) { // blocks 2 q, 2 q + 1: (d, m) records
                // (read as a plain vector: a read through HIP's uint2 made the compiler wait for every load in flight)
                typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
                const u32x2 r2 = *reinterpret_cast<const u32x2 *>(rlane + (sb & 1) * RECB + j * 32 * 16 * RV + q * 8);
                const float v0 = fmaf((float)CENTER, h2f(r2[0] & 0xFFFFu), h2f(r2[0] >> 16));
                const float v1 = fmaf((float)CENTER, h2f(r2[1] & 0xFFFFu), h2f(r2[1] >> 16));
                const auto vh = __builtin_amdgcn_cvt_pkrtz(v0, v1);
                oh[q] = __builtin_bit_cast(uint32_t, vh);
                const uint32_t low = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(v0 - (float)vh[0], v1 - (float)vh[1]));
                ol[q] = hh ? 0u : low; // the sums' low halves meet vh only
            }
            bh[j] = __builtin_bit_cast(half8, u32x4{oh[0], oh[1], oh[2], oh[3]});
            bl[j] = __builtin_bit_cast(half8, u32x4{ol[0], ol[1], ol[2], ol[3]});
        }
        // the block sums are stored times XSUM_SCALE: with the factor below the accumulators receive the term times
        // WSCALE * XSUM_SCALE, which is what the main term scales its sums to (scale_of)
        // (added by the vector ALU like the main term: accumulators that the matrix pipe also wrote would be kept twice)
        const float16v zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < MI; i++) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                float16v S = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, mx[i]), bh[j], zero, 0, 0, 0);
                S = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, mx[i]), bl[j], S, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = fmaf(S[r], WSCALE, acc[i][j][r]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    // Steps g = 0 .. T - 1 in groups of four (a superblock).  Step g multiplies x stage g % 3 with weight stage g & 1,
    // brings the x tile of step g + 2 into its stage, converts the weights of step g + 1 into the other weight stage
    // and requests those of step g + 3; the first step of a group also requests the scale records of the next
    // superblock, the third this one's block sums.  Every wave issues the same loads in the same order, so that the
    // wait in front of a barrier (for the x tile of step g + 1, requested a step ago) can leave the younger requests in
    // flight.
    Raw buf[4]; // the blocks of steps g .. g + 3, at g % 4 ..
    load_x(0, 0);
    load_x(1, 1);
    fetch(0, buf[0]);
    fetch(1, buf[1]);
    fetch(2, buf[2]);
    fetch_records(0);
    convert(buf[0], 0, 0);
    convert(buf[0], 1, 0);
    wait_vm_and_lds<0>();
    lds_barrier();
    int g3 = 0;
    for (int sb = 0; sb < nsb; sb++) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int g = 4 * sb + i;
            const int as = g3 * ASTAGE, xs = (g3 == 0 ? 2 : g3 - 1);
            // the order of the requests: the weight blocks first, so that the wait at the end of the next step, which
            // lets that step's x tile and what follows it stay out, covers them
            if (WITH_MIN && i == 2) { // this superblock's block sums, for the end of the next step: ahead of the step's other
                fetch_sums(sb);       // requests, so that the wait at its end covers them
                asm volatile("" ::: "memory");
            }
            fetch(g + 3, buf[(i + 3) & 3]);
            load_x(g + 2, xs);
            if (i == 0) fetch_records(sb + 1);
            // (past the last step the conversion writes a stage that nobody reads)
#pragma unroll
            for (int hb = 0; hb < 2; hb++) {
                multiply_block(as, i & 1, hb, sb, 2 * i + hb);
                convert(buf[(i + 1) & 3], hb, (i + 1) & 1);
            }
            if (WITH_MIN && i == 3) multiply_min(sb);
            // younger than the x tile of step g + 1 (requested a step ago): what followed it in that step, and this step's
            if (i == 0) wait_vm_and_lds<F + XL + ML>();
            else if (i == 1) wait_vm_and_lds<ML + F + XL>();
            else wait_vm_and_lds<F + XL>();
            lds_barrier();
            g3 = g3 == 2 ? 0 : g3 + 1;
        }
    }
    wait_vm_and_lds<0>(); // nothing of this workgroup may still be on its way into LDS when it ends
    // D layout: lane -> column li; register r -> row 8 * (r / 4) + 4 * (lane / 32) + r % 4
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int gn = n0 + wn + j * 32 + li;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int gm = m0 + wm + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (gm < a.m && gn < a.n) {
                    if (!a.pair) {
                        if (a.ypart) a.ypart[((size_t)blockIdx.y * a.m + gm) * a.n + gn] = acc[i][j][r];
                        else a.y[(size_t)gm * a.n + gn] = acc[i][j][r] * (a.rowscale[gm] * (1.0f / ASCALE));
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < 16; r += 2) { // pair mode: an even row and the next hold the two parts of activation row gm / 2
                const int gm = m0 + wm + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (a.pair && gm < a.m && gn < a.n) {
                    const size_t t = (size_t)(gm >> 1);
                    const float v = acc[i][j][r] + acc[i][j][r + 1];
                    if (a.ypart) {
                        a.ypart[((size_t)blockIdx.y * (a.m >> 1) + t) * a.n + gn] = v;
                    } else {
                        float out = v * (a.rowscale[gm] * (1.0f / ASCALE));
                        if (a.bias) out += a.bias[gn];
                        if (a.resid) out += a.resid[t * a.n + gn];
                        a.y[t * a.n + gn] = out;
                    }
                }
            }
        }
}

// What the Q4_K kernel wants from the x pre-pass besides the scaled f16 rows: elements 1 and 2 of every group of four
// exchanged, and the sums of every 32 consecutive (scaled, f16) elements as f16 pairs hi + lo: 32 halfs per superblock,
// [hi of its 8 sub-blocks | the same | lo | zeros] (NULL xs3: plain rows for the other kernels).
struct XSums {
    _Float16 *xs3;
    int pitch; // halfs per row: 32 per superblock and 32 or 64 zeros, see xs3_pitch
};
// one or two superblocks of zeros end a row: the last step of the minimum term may look one superblock past the end
__host__ __device__ inline int xs3_pitch(int64_t k) { return (int)(((k >> 8) + 2) & ~(int64_t)1) * 32; }

// The sum `s` of the caller's four elements, added over the eight threads of a 32-element group; the first of them
// stores the pair.  g = index of the group along the row.
__device__ inline void store_group_sum(float s, int g, int n_groups, _Float16 *row3, const XSums &xs) {
    s += __shfl_xor(s, 1);
    s += __shfl_xor(s, 2);
    s += __shfl_xor(s, 4);
    if ((threadIdx.x & 7) == 0 && g < n_groups) {
        s *= XSUM_SCALE; // 32 elements below 2^15 each: the sum must not leave f16's range
        const _Float16 hi = (_Float16)s, lo = (_Float16)(s - (float)hi);
        _Float16 *base = row3 + (size_t)(g >> 3) * 32 + (g & 7);
        base[0] = hi;
        base[8] = hi;
        base[16] = lo;
        base[24] = (_Float16)0.f;
    }
}

// bf16 rows -> f16 rows scaled by a power of two (largest magnitude below 2^15), and the scale to undo it.
__global__ void __launch_bounds__(256) gemm_prep_x_kernel(const uint16_t *x, int m, int k, _Float16 *xh, float *rowscale, XSums xs) {
    __shared__ float red[4];
    const int row = blockIdx.x;
    const uint16_t *xr = x + (size_t)row * k;
    uint32_t amax_bits = 0;
    for (int i = threadIdx.x; i < k; i += blockDim.x) {
        uint32_t b = (uint32_t)(xr[i] & 0x7FFF);
        amax_bits = b > amax_bits ? b : amax_bits;
    }
    float amax = __builtin_bit_cast(float, amax_bits << 16);
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) amax = fmaxf(amax, __shfl_xor(amax, s));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
    _Float16 *row3 = xs.xs3 ? xs.xs3 + (size_t)row * xs.pitch : nullptr;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    // amax in [2^e, 2^(e+1)) -> multiply by 2^(14 - e); inf/nan rows are passed through unscaled
    int eb = (int)((__builtin_bit_cast(uint32_t, amax) >> 23) & 0xFF);
    if (eb == 0 || eb == 0xFF) eb = 127 + 14;
    int sb = 127 + 14 - (eb - 127);
    sb = sb < 1 ? 1 : (sb > 254 ? 254 : sb);
    const float f = __builtin_bit_cast(float, (uint32_t)sb << 23);
    typedef _Float16 half4 __attribute__((ext_vector_type(4)));
    for (int i4 = threadIdx.x; i4 < (k >> 2); i4 += blockDim.x) { // k is a multiple of 64: whole groups of eight threads
        const uint2 raw = reinterpret_cast<const uint2 *>(xr)[i4];
        const _Float16 h0 = (_Float16)(__builtin_bit_cast(float, raw.x << 16) * f), h1 = (_Float16)(__builtin_bit_cast(float, raw.x & 0xFFFF0000u) * f);
        const _Float16 h2 = (_Float16)(__builtin_bit_cast(float, raw.y << 16) * f), h3 = (_Float16)(__builtin_bit_cast(float, raw.y & 0xFFFF0000u) * f);
        if (row3) {
            reinterpret_cast<half4 *>(xh + (size_t)row * k)[i4] = half4{h0, h2, h1, h3};
            store_group_sum(((float)h0 + (float)h1) + ((float)h2 + (float)h3), i4 >> 3, k >> 5, row3, xs);
        } else {
            reinterpret_cast<half4 *>(xh + (size_t)row * k)[i4] = half4{h0, h1, h2, h3};
        }
    }
    if (row3 && (int)threadIdx.x < xs.pitch - (k >> 8) * 32) row3[(size_t)(k >> 8) * 32 + threadIdx.x] = (_Float16)0.f; // the zeros that end a row
    if (threadIdx.x == 0) rowscale[row] = 1.0f / f;
}

// y = (sum over the splits, in order) * rowscale / ws (+ bias + resid): four outputs per thread.  `rows` output rows;
// row_mul = 2 in pair mode (output row t was scaled as activation rows 2t, 2t + 1).
__global__ void __launch_bounds__(256) gemm_reduce_kernel(const float *ypart, const float *rowscale, int rows, int n, int splits,
                                                          float inv_ws, int row_mul, const float *bias, const float *resid, float *y) {
    const size_t i4 = (size_t)blockIdx.x * blockDim.x + threadIdx.x, total4 = (size_t)rows * n / 4;
    if (i4 >= total4) return;
    float4 acc = reinterpret_cast<const float4 *>(ypart)[i4];
    for (int s = 1; s < splits; s++) {
        const float4 v = reinterpret_cast<const float4 *>(ypart + (size_t)s * rows * n)[i4];
        acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
    }
    const size_t row = (i4 * 4) / (size_t)n, col = (i4 * 4) % (size_t)n; // n is a multiple of 4: the four share a row
    const float f = rowscale[row * row_mul] * inv_ws;
    float4 out = make_float4(acc.x * f, acc.y * f, acc.z * f, acc.w * f);
    if (bias) {
        out.x += bias[col]; out.y += bias[col + 1]; out.z += bias[col + 2]; out.w += bias[col + 3];
    }
    if (resid) {
        const float4 r = reinterpret_cast<const float4 *>(resid)[i4];
        out.x += r.x; out.y += r.y; out.z += r.z; out.w += r.w;
    }
    reinterpret_cast<float4 *>(y)[i4] = out;
}

template <class T>
int launch_gemm(axq_ctx *ctx, GemmArgs a, int splits) {
    static std::atomic<uint64_t> lds_allowed[2]; // per kernel: a bit per device
    const int wm = a.wm, bm = 128 * wm;
    const unsigned tiles = (unsigned)(((a.n + BN - 1) / BN) * ((a.m + bm - 1) / bm));
    const dim3 grid(tiles, (unsigned)splits);
    const size_t lds = (size_t)2 * (bm + 2 * BN) * LDK * sizeof(_Float16); // two stages
    {
        int rc;
        if ((rc = axq_allow_lds(ctx, reinterpret_cast<const void *>(gemm_kernel<T, 2>), lds_allowed[1], 2 * (256 + 2 * BN) * LDK * 2))) return rc;
        if ((rc = axq_allow_lds(ctx, reinterpret_cast<const void *>(gemm_kernel<T, 1>), lds_allowed[0], 2 * (128 + 2 * BN) * LDK * 2))) return rc;
    }
    if (wm == 2) gemm_kernel<T, 2><<<grid, 512, lds, ctx->stream>>>(a);
    else gemm_kernel<T, 1><<<grid, 512, lds, ctx->stream>>>(a);
    AXQ_LAUNCH_CHECK(ctx, "gemm_kernel");
    if (splits > 1) {
        const int rows = a.pair ? a.m / 2 : a.m;
        const size_t total4 = (size_t)rows * a.n / 4;
        gemm_reduce_kernel<<<(unsigned)((total4 + 255) / 256), 256, 0, ctx->stream>>>(a.ypart, a.rowscale, rows, a.n, splits, 1.0f / T::WS,
                                                                                    a.pair ? 2 : 1, a.bias, a.resid, a.y);
        AXQ_LAUNCH_CHECK(ctx, "gemm_reduce_kernel");
    }
    return AXQ_OK;
}

// f32 rows, optionally RMS-normalised on the way ((x * inv_rms) * norm_w, RMSNorm::forward, llm/src/llama.rs:158-187),
// -> two f16 rows each under one power-of-two scale: row 2t holds the leading 11 bits of every element, row 2t + 1
// what those leave, so that their GEMM results add up to the f32 product (the GEMM's epilogue adds them: pair mode).
// SWIGLU: x holds rows of 2 k gate/up values, four gate values followed by the four up values of the same indices (the row
// order of the fused gate/up weight), and the row that is split is silu(gate) * up (k a multiple of 4, at most 16384).
template <bool SWIGLU>
__global__ void __launch_bounds__(256) gemm_prep_x_f32_kernel(const float *x, const float *norm_w, float eps, int m, int k,
                                                              _Float16 *xh, float *rowscale, XSums xs) {
    // the row stays in registers between the passes: 16 bytes per thread and step, up to 16 steps (k <= 16384);
    // longer rows (or k not a multiple of 4) take the plain loops below
    constexpr int STEPS = 16;
    __shared__ float red[4];
    const int row = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float *xr = x + (size_t)row * (SWIGLU ? 2 * k : k);
    const bool in_regs = SWIGLU || ((k & 3) == 0 && k <= STEPS * 256 * 4);
    float4 v[STEPS];
    if (in_regs) {
#pragma unroll
        for (int c = 0; c < STEPS; c++) {
            const int i4 = c * 256 + threadIdx.x;
            if (SWIGLU) {
                v[c] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (i4 * 4 < k) {
                    const float4 g = reinterpret_cast<const float4 *>(xr)[2 * i4], u = reinterpret_cast<const float4 *>(xr)[2 * i4 + 1];
                    v[c].x = (g.x * (1.0f / (1.0f + expf(-g.x)))) * u.x;
                    v[c].y = (g.y * (1.0f / (1.0f + expf(-g.y)))) * u.y;
                    v[c].z = (g.z * (1.0f / (1.0f + expf(-g.z)))) * u.z;
                    v[c].w = (g.w * (1.0f / (1.0f + expf(-g.w)))) * u.w;
                }
            } else {
                v[c] = i4 * 4 < k ? reinterpret_cast<const float4 *>(xr)[i4] : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    }
    float inv = 1.0f;
    if (norm_w) {
        float ss = 0.f;
        if (in_regs) {
#pragma unroll
            for (int c = 0; c < STEPS; c++) {
                ss = fmaf(v[c].x, v[c].x, ss); ss = fmaf(v[c].y, v[c].y, ss); ss = fmaf(v[c].z, v[c].z, ss); ss = fmaf(v[c].w, v[c].w, ss);
            }
        } else {
            for (int i = threadIdx.x; i < k; i += blockDim.x) ss = fmaf(xr[i], xr[i], ss);
        }
#pragma unroll
        for (int s = 32; s >= 1; s >>= 1) ss += __shfl_xor(ss, s);
        if (lane == 0) red[wave] = ss;
        __syncthreads();
        ss = (red[0] + red[1]) + (red[2] + red[3]);
        __syncthreads();
        inv = 1.0f / sqrtf(ss / (float)k + eps);
        if (in_regs) {
#pragma unroll
            for (int c = 0; c < STEPS; c++) {
                const int i4 = c * 256 + threadIdx.x;
                if (i4 * 4 < k) {
                    const float4 w = reinterpret_cast<const float4 *>(norm_w)[i4];
                    v[c] = make_float4((v[c].x * inv) * w.x, (v[c].y * inv) * w.y, (v[c].z * inv) * w.z, (v[c].w * inv) * w.w);
                }
            }
        }
    }
    uint32_t amax_bits = 0; // of |v| as integers: a NaN ranks above everything and is not dropped
    auto note = [&](float f) {
        const uint32_t b = __builtin_bit_cast(uint32_t, f) & 0x7FFFFFFFu;
        amax_bits = b > amax_bits ? b : amax_bits;
    };
    if (in_regs) {
#pragma unroll
        for (int c = 0; c < STEPS; c++) { note(v[c].x); note(v[c].y); note(v[c].z); note(v[c].w); }
    } else {
        for (int i = threadIdx.x; i < k; i += blockDim.x) note(norm_w ? (xr[i] * inv) * norm_w[i] : xr[i]);
    }
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) {
        const uint32_t o = (uint32_t)__shfl_xor((int)amax_bits, s);
        amax_bits = o > amax_bits ? o : amax_bits;
    }
    if (lane == 0) red[wave] = __builtin_bit_cast(float, amax_bits);
    __syncthreads();
    uint32_t ab = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t o = __builtin_bit_cast(uint32_t, red[i]);
        ab = o > ab ? o : ab;
    }
    // amax in [2^e, 2^(e+1)) -> multiply by 2^(14 - e); inf/nan rows are passed through unscaled
    int eb = (int)((ab >> 23) & 0xFF);
    if (eb == 0 || eb == 0xFF) eb = 127 + 14;
    int sb = 127 + 14 - (eb - 127);
    sb = sb < 1 ? 1 : (sb > 254 ? 254 : sb);
    const float f = __builtin_bit_cast(float, (uint32_t)sb << 23);
    _Float16 *hi_row = xh + (size_t)(2 * row) * k, *lo_row = hi_row + k;
    // the Q4_K kernel's extras (callers ask for them only when the row fits the registers and k is a multiple of 64)
    _Float16 *hi3 = xs.xs3 ? xs.xs3 + (size_t)(2 * row) * xs.pitch : nullptr, *lo3 = hi3 ? hi3 + xs.pitch : nullptr;
    if (in_regs) {
#pragma unroll
        for (int c = 0; c < STEPS; c++) {
            const int i4 = c * 256 + threadIdx.x;
            if (c * 256 * 4 < k) { // uniform per step; with the extras k is a multiple of 32 and whole groups of eight threads are in
                const bool live = i4 * 4 < k;
                const float e[4] = {v[c].x * f, v[c].y * f, v[c].z * f, v[c].w * f};
                _Float16 h[4], l[4];
#pragma unroll
                for (int j = 0; j < 4; j++) { h[j] = (_Float16)e[j]; l[j] = (_Float16)(e[j] - (float)h[j]); }
                typedef _Float16 half4 __attribute__((ext_vector_type(4)));
                if (hi3) {
                    if (live) {
                        reinterpret_cast<half4 *>(hi_row)[i4] = half4{h[0], h[2], h[1], h[3]};
                        reinterpret_cast<half4 *>(lo_row)[i4] = half4{l[0], l[2], l[1], l[3]};
                    }
                    store_group_sum(((float)h[0] + (float)h[1]) + ((float)h[2] + (float)h[3]), live ? i4 >> 3 : k, k >> 5, hi3, xs);
                    store_group_sum(((float)l[0] + (float)l[1]) + ((float)l[2] + (float)l[3]), live ? i4 >> 3 : k, k >> 5, lo3, xs);
                } else if (live) {
                    reinterpret_cast<half4 *>(hi_row)[i4] = half4{h[0], h[1], h[2], h[3]};
                    reinterpret_cast<half4 *>(lo_row)[i4] = half4{l[0], l[1], l[2], l[3]};
                }
            }
        }
    } else {
        for (int i = threadIdx.x; i < k; i += blockDim.x) {
            const float e = (norm_w ? (xr[i] * inv) * norm_w[i] : xr[i]) * f;
            const _Float16 hi = (_Float16)e;
            hi_row[i] = hi;
            lo_row[i] = (_Float16)(e - (float)hi);
        }
    }
    if (hi3 && (int)threadIdx.x < xs.pitch - (k >> 8) * 32) { // the zeros that end a row
        hi3[(size_t)(k >> 8) * 32 + threadIdx.x] = (_Float16)0.f;
        lo3[(size_t)(k >> 8) * 32 + threadIdx.x] = (_Float16)0.f;
    }
    if (threadIdx.x == 0) {
        rowscale[2 * row] = 1.0f / f;
        rowscale[2 * row + 1] = 1.0f / f;
    }
}

// The context's GEMM scratch, grown to `need` bytes (work that still uses the old one is waited for first).
int reserve_scratch(axq_ctx *ctx, size_t need) {
    if (ctx->gemm_scratch_bytes >= need) return AXQ_OK;
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    if (ctx->gemm_scratch) (void)hipFree(ctx->gemm_scratch);
    ctx->gemm_scratch = nullptr;
    ctx->gemm_scratch_bytes = 0;
    AXQ_HIP(ctx, hipMalloc(&ctx->gemm_scratch, need), AXQ_ERR_ALLOCATION_FAILED);
    ctx->gemm_scratch_bytes = need;
    return AXQ_OK;
}

struct GemmPlan {
    int splits, steps_per_split, wm;
    bool q4k;     // the one-MFMA Q4_K kernel (gemm_q4k_kernel) instead of the two-plane kernel
    bool q5;      // the one-MFMA kernel of the types with blocks of 32 (gemm_blk32_kernel)
    size_t xh_bytes, rs_bytes, part_bytes, xs3_bytes;
};

// Whether the one-MFMA kernel takes this weight; in_regs_only: the caller's x pre-pass produces the extras only for rows
// that fit its registers (f32 rows).
bool q4k_route(const axq_weight *w, bool in_regs_only) {
    static const bool off = getenv("AXQ_GEMM_Q4K") && getenv("AXQ_GEMM_Q4K")[0] == '0'; // development knob
    const bool type_ok = w->type == AXQ_Q4_K || (w->type == AXQ_Q5_K && w->qh_pitch % 16 == 0);
    return !off && type_ok && w->k % 256 == 0 && (!in_regs_only || w->k <= 16 * 256 * 4);
}

// Whether gemm_blk32_kernel takes this call.
bool q5_route(const axq_weight *w, int m, bool in_regs_only) {
    static const bool off = getenv("AXQ_GEMM_BLK32") && getenv("AXQ_GEMM_BLK32")[0] == '0'; // development knob
    const bool type_ok = w->type == AXQ_Q4_0 || w->type == AXQ_Q4_1 || w->type == AXQ_Q5_0 || w->type == AXQ_Q5_1 || w->type == AXQ_Q8_0;
    static const int min_rows = getenv("AXQ_GEMM_BLK32_MIN_ROWS") ? atoi(getenv("AXQ_GEMM_BLK32_MIN_ROWS")) : 1; // development knob
    return !off && type_ok && w->k % 256 == 0 && m >= min_rows && w->meta_pitch % 16 == 0 && (!in_regs_only || w->k <= 16 * 256 * 4);
}

// Split K when the output tiles alone leave most compute units idle (short prompts): the splits' partial sums go
// through scratch and are added in order by a second kernel.  Scratch (kept in the context, grown on demand):
// f16 activations [m, k] | row scales [m] | partial sums of a split K | sub-block sums (Q4_K) | `extra` bytes for the caller.
int plan_gemm(axq_ctx *ctx, const axq_weight *w, int m, bool f32_rows, size_t extra, GemmPlan *p) {
    if (w->k % BK != 0)
        return axq_fail(ctx, AXQ_ERR_INVALID_BLOCK_SIZE, "Invalid block size: the prefill GEMM needs k %% 64 == 0, got %lld",
                        (long long)w->k);
    if (w->n_rows > INT32_MAX || w->k > INT32_MAX)
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: weight dimensions exceed 2^31");
    // rows of a workgroup's tile: the Q4_K kernel's 128-row tile keeps eight waves (64 x 64 each), so it also serves
    // 129..256 rows, where the 256-row tile would leave half the compute units idle
    const bool route_q4k = q4k_route(w, f32_rows);
    static const int bm_knob = getenv("AXQ_GEMM_BM") ? atoi(getenv("AXQ_GEMM_BM")) : 0; // development knob: 128 or 256 for every shape
    const int bm = bm_knob ? bm_knob : (m > (route_q4k ? 256 : 128) ? 256 : 128);
    p->wm = bm / 128;
    p->q4k = route_q4k;
    p->q5 = q5_route(w, m, f32_rows);
    const int bn = p->q4k ? QBN : BN;
    const long tiles = (long)((w->n_rows + bn - 1) / bn) * ((m + bm - 1) / bm);
    const int ksteps = (int)(w->k / BK), cus = ctx->prop.multiProcessorCount;
    int splits = (int)(cus / tiles);
    splits = splits > 8 ? 8 : splits;
    if (splits > ksteps / 4) splits = ksteps / 4;
    if (splits < 2 || w->n_rows % 4 != 0) splits = 1;
    p->steps_per_split = (ksteps + splits - 1) / splits;
    if (p->q4k || p->q5) p->steps_per_split = (p->steps_per_split + 3) & ~3; // whole superblocks per split
    p->splits = (ksteps + p->steps_per_split - 1) / p->steps_per_split;
    // the Q4_K kernel reads whole row tiles without a clamp: its x buffers have rows up to a multiple of the tile
    const size_t mpad = (p->q4k || p->q5) ? (size_t)(m + bm - 1) / bm * bm : (size_t)m;
    p->xh_bytes = axq_align_up(mpad * (size_t)w->k * 2, 256);
    p->rs_bytes = axq_align_up((size_t)m * 4, 256);
    p->part_bytes = axq_align_up(p->splits > 1 ? (size_t)p->splits * m * (size_t)w->n_rows * 4 : 0, 256);
    p->xs3_bytes = axq_align_up((p->q4k || p->q5) ? mpad * (size_t)xs3_pitch(w->k) * 2 : 0, 256);
    return reserve_scratch(ctx, p->xh_bytes + p->rs_bytes + p->part_bytes + p->xs3_bytes + extra);
}

// What the x pre-pass has to write besides the rows (nothing for the two-plane kernel).
XSums plan_sums(axq_ctx *ctx, const axq_weight *w, const GemmPlan &p) {
    XSums xs = {nullptr, 0};
    if (p.q4k || p.q5) {
        xs.xs3 = reinterpret_cast<_Float16 *>(reinterpret_cast<uint8_t *>(ctx->gemm_scratch) + p.xh_bytes + p.rs_bytes + p.part_bytes);
        xs.pitch = xs3_pitch(w->k);
    }
    return xs;
}

template <bool Q5>
int launch_q4k_tiles(axq_ctx *ctx, const GemmArgs &a, dim3 grid, size_t lds) {
    static std::atomic<uint64_t> lds_allowed[2]; // per kernel: a bit per device
    int rc;
    if ((rc = axq_allow_lds(ctx, reinterpret_cast<const void *>(gemm_q4k_kernel<256, 512, Q5>), lds_allowed[1], (3 * 256 * 64 + 2 * QBN * 64) * 2))) return rc;
    if ((rc = axq_allow_lds(ctx, reinterpret_cast<const void *>(gemm_q4k_kernel<128, 512, Q5>), lds_allowed[0], (3 * 128 * 64 + 2 * QBN * 64) * 2))) return rc;
    if (a.wm == 2) gemm_q4k_kernel<256, 512, Q5><<<grid, 512, lds, ctx->stream>>>(a);
    else gemm_q4k_kernel<128, 512, Q5><<<grid, 512, lds, ctx->stream>>>(a);
    return AXQ_OK;
}

int launch_gemm_q4k(axq_ctx *ctx, GemmArgs a, int splits, bool q5k) {
    const int bm = 128 * a.wm;
    const unsigned tiles = (unsigned)(((a.n + QBN - 1) / QBN) * ((a.m + bm - 1) / bm));
    const dim3 grid(tiles, (unsigned)splits);
    const size_t lds = (size_t)(3 * bm * 64 + 2 * QBN * 64) * sizeof(_Float16); // three x stages, two weight stages
    if (int rc = q5k ? launch_q4k_tiles<true>(ctx, a, grid, lds) : launch_q4k_tiles<false>(ctx, a, grid, lds)) return rc;
    AXQ_LAUNCH_CHECK(ctx, "gemm_q4k_kernel");
    if (splits > 1) {
        const int rows = a.pair ? a.m / 2 : a.m;
        const size_t total4 = (size_t)rows * a.n / 4;
        gemm_reduce_kernel<<<(unsigned)((total4 + 255) / 256), 256, 0, ctx->stream>>>(a.ypart, a.rowscale, rows, a.n, splits, 1.0f,
                                                                                    a.pair ? 2 : 1, a.bias, a.resid, a.y);
        AXQ_LAUNCH_CHECK(ctx, "gemm_reduce_kernel");
    }
    return AXQ_OK;
}

template <int BITS, bool WITH_MIN>
int launch_blk32(axq_ctx *ctx, const GemmArgs &a, dim3 grid, size_t lds) {
    static std::atomic<uint64_t> lds_allowed[2]; // per kernel: a bit per device
    int rc;
    if (a.wm == 2) {
        if ((rc = axq_allow_lds(ctx, reinterpret_cast<const void *>(gemm_blk32_kernel<BITS, WITH_MIN, 256>), lds_allowed[1], lds))) return rc;
        gemm_blk32_kernel<BITS, WITH_MIN, 256><<<grid, 512, lds, ctx->stream>>>(a);
    } else {
        if ((rc = axq_allow_lds(ctx, reinterpret_cast<const void *>(gemm_blk32_kernel<BITS, WITH_MIN, 128>), lds_allowed[0], lds))) return rc;
        gemm_blk32_kernel<BITS, WITH_MIN, 128><<<grid, 512, lds, ctx->stream>>>(a);
    }
    return AXQ_OK;
}

int launch_gemm_q5(axq_ctx *ctx, GemmArgs a, int splits, int type) {
    const int bm = 128 * a.wm;
    const unsigned tiles = (unsigned)(((a.n + PBN - 1) / PBN) * ((a.m + bm - 1) / bm));
    const dim3 grid(tiles, (unsigned)splits);
    const size_t lds = (size_t)(3 * bm * 64 + 2 * PBN * 64) * sizeof(_Float16) + 2 * PBN * 32; // three x stages, two weight stages, scale records
    int rc;
    switch (type) {
    case AXQ_Q4_0: rc = launch_blk32<4, false>(ctx, a, grid, lds); break;
    case AXQ_Q4_1: rc = launch_blk32<4, true>(ctx, a, grid, lds); break;
    case AXQ_Q5_0: rc = launch_blk32<5, false>(ctx, a, grid, lds); break;
    case AXQ_Q5_1: rc = launch_blk32<5, true>(ctx, a, grid, lds); break;
    default: rc = launch_blk32<8, false>(ctx, a, grid, lds); break;
    }
    if (rc) return rc;
    AXQ_LAUNCH_CHECK(ctx, "gemm_blk32_kernel");
    if (splits > 1) {
        const int rows = a.pair ? a.m / 2 : a.m;
        const size_t total4 = (size_t)rows * a.n / 4;
        gemm_reduce_kernel<<<(unsigned)((total4 + 255) / 256), 256, 0, ctx->stream>>>(a.ypart, a.rowscale, rows, a.n, splits,
                                                                                    1.0f / (WSCALE * XSUM_SCALE), a.pair ? 2 : 1, a.bias, a.resid, a.y);
        AXQ_LAUNCH_CHECK(ctx, "gemm_reduce_kernel");
    }
    return AXQ_OK;
}

// The GEMM proper over activations that already sit in scratch as scaled f16 rows.
int run_gemm(axq_ctx *ctx, const axq_weight *w, int m, const GemmPlan &p, float *y, bool pair = false, const float *bias = nullptr,
             const float *resid = nullptr) {
    uint8_t *base = reinterpret_cast<uint8_t *>(ctx->gemm_scratch);
    GemmArgs a;
    a.codes = w->codes; a.meta = w->meta; a.qh = w->qh;
    a.codes_pitch = w->codes_pitch; a.meta_pitch = w->meta_pitch; a.qh_pitch = w->qh_pitch;
    a.xh = reinterpret_cast<_Float16 *>(base); a.rowscale = reinterpret_cast<float *>(base + p.xh_bytes); a.y = y;
    a.ypart = p.splits > 1 ? reinterpret_cast<float *>(base + p.xh_bytes + p.rs_bytes) : nullptr;
    a.m = m; a.n = (int)w->n_rows; a.k = (int)w->k;
    a.steps_per_split = p.steps_per_split;
    a.pair = pair ? 1 : 0; a.bias = bias; a.resid = resid; a.wm = p.wm;
    const XSums xs = plan_sums(ctx, w, p);
    a.xs3 = xs.xs3; a.xs3_pitch = xs.pitch;
    if (p.q4k) return launch_gemm_q4k(ctx, a, p.splits, w->type == AXQ_Q5_K);
    if (p.q5) return launch_gemm_q5(ctx, a, p.splits, w->type);
    switch (w->type) {
    case AXQ_Q4_K: return launch_gemm<GQ4K>(ctx, a, p.splits);
    case AXQ_Q6_K: return launch_gemm<GQ6K>(ctx, a, p.splits);
    case AXQ_Q5_K: return launch_gemm<GQ5K>(ctx, a, p.splits);
    case AXQ_Q4_0: return launch_gemm<GQ4x<false>>(ctx, a, p.splits);
    case AXQ_Q4_1: return launch_gemm<GQ4x<true>>(ctx, a, p.splits);
    case AXQ_Q5_0: return launch_gemm<GQ5x<false>>(ctx, a, p.splits);
    case AXQ_Q5_1: return launch_gemm<GQ5x<true>>(ctx, a, p.splits);
    case AXQ_Q8_0: return launch_gemm<GQ80>(ctx, a, p.splits);
    case AXQ_F16: return launch_gemm<GF16>(ctx, a, p.splits);
    case AXQ_F32: return launch_gemm<GF32>(ctx, a, p.splits);
    default: return axq_fail(ctx, AXQ_ERR_INVALID_QUANT_TYPE, "Invalid quantization type: %d", w->type);
    }
}

} // namespace

int axq_dev_gemm_bf16(axq_ctx *ctx, const axq_weight *w, const uint16_t *x, int m, float *y) {
    GemmPlan p;
    int rc;
    if ((rc = plan_gemm(ctx, w, m, false, 0, &p))) return rc;
    uint8_t *base = reinterpret_cast<uint8_t *>(ctx->gemm_scratch);
    gemm_prep_x_kernel<<<m, 256, 0, ctx->stream>>>(x, m, (int)w->k, reinterpret_cast<_Float16 *>(base),
                                                   reinterpret_cast<float *>(base + p.xh_bytes), plan_sums(ctx, w, p));
    return run_gemm(ctx, w, m, p, y);
}

bool axq_dev_gemm_f32_covers(const axq_weight *w, int m) {
    return w->k % BK == 0 && m >= 1 && m <= AXQ_GEMM_F32_MAX_ROWS && w->n_rows <= INT32_MAX && w->k <= INT32_MAX;
}

// y[m, n] = f(x)[m, k] W^T (+ bias[n]) (+ resid[m, n], which may be y) with f32 activations: each row goes through the
// matrix pipe as two adjacent f16 rows (2m rows in all), and the GEMM's epilogue adds the two results.  f = RMSNorm with weight norm_w
// when that is given.
int axq_dev_gemm_f32(axq_ctx *ctx, const axq_weight *w, const float *x, int m, const float *norm_w, float eps, const float *bias,
                     const float *resid, float *y) {
    return axq_dev_gemm_f32_ex(ctx, w, x, false, m, norm_w, eps, bias, resid, y);
}

// The same with f = SwiGLU when `swiglu`: x holds m rows of 2 k interleaved gate/up values (see the pre-pass).
bool axq_dev_gemm_f32_takes_swiglu(const axq_weight *w) { return w->k % 4 == 0 && w->k <= 16 * 256 * 4; }

int axq_dev_gemm_f32_ex(axq_ctx *ctx, const axq_weight *w, const float *x, bool swiglu, int m, const float *norm_w, float eps,
                        const float *bias, const float *resid, float *y) {
    GemmPlan p;
    int rc;
    if (swiglu && (norm_w || !axq_dev_gemm_f32_takes_swiglu(w)))
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_dev_gemm_f32_ex: SwiGLU rows need k %% 4 == 0, k <= 16384 and no norm");
    if ((rc = plan_gemm(ctx, w, 2 * m, true, 0, &p))) return rc;
    uint8_t *base = reinterpret_cast<uint8_t *>(ctx->gemm_scratch);
    _Float16 *xh = reinterpret_cast<_Float16 *>(base);
    float *rowscale = reinterpret_cast<float *>(base + p.xh_bytes);
    if (swiglu) gemm_prep_x_f32_kernel<true><<<m, 256, 0, ctx->stream>>>(x, nullptr, eps, m, (int)w->k, xh, rowscale, plan_sums(ctx, w, p));
    else gemm_prep_x_f32_kernel<false><<<m, 256, 0, ctx->stream>>>(x, norm_w, eps, m, (int)w->k, xh, rowscale, plan_sums(ctx, w, p));
    return run_gemm(ctx, w, 2 * m, p, y, true, bias, resid);
}
