// Device codecs: quantize_tensor / dequantize_tensor on the GPU, bit-exact with
// the CPU algorithm of crates/axonml-quant/src/quantize.rs and dequantize.rs,
// plus the permutation between the packed (`to_bytes`) image and the planar
// device layout.
//
// This file must be compiled with -ffp-contract=off: the reference rounds each
// multiply, divide, add and subtract separately (f32), and so do these kernels.
#include <hip/hip_fp16.h>

#include <stdint.h>

#include "axq_internal.h"

namespace {

__device__ inline uint16_t f32_to_f16_bits(float f) { return __half_as_ushort(__float2half_rn(f)); }
__device__ inline float f16_bits_to_f32(uint16_t h) { return __half2float(__ushort_as_half(h)); }

// Rust: v.round().clamp(lo, hi) as iN -- roundf is half away from zero, NaN -> 0.
__device__ inline int round_clamp(float v, float lo, float hi) {
    float r = roundf(v);
    if (isnan(r)) return 0;
    r = r < lo ? lo : r;
    r = r > hi ? hi : r;
    return (int)r;
}

// Loads the (up to) 32 floats of block `b`; elements past numel are +0.0 and
// `len` says how many are real.
__device__ inline void load_block32(const float *src, size_t numel, size_t b, float (&x)[32], int &len) {
    size_t start = b * 32;
    size_t rem = numel - start;
    len = rem < 32 ? (int)rem : 32;
    if (len == 32) {
        const float4 *p = reinterpret_cast<const float4 *>(src + start);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float4 v = p[i];
            x[4 * i] = v.x; x[4 * i + 1] = v.y; x[4 * i + 2] = v.z; x[4 * i + 3] = v.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 32; i++) x[i] = i < len ? src[start + i] : 0.0f;
    }
}

__device__ inline void store_u16(uint8_t *p, uint16_t v) { *reinterpret_cast<uint16_t *>(p) = v; }
__device__ inline uint16_t load_u16(const uint8_t *p) { return *reinterpret_cast<const uint16_t *>(p); }

// ---- Q8_0: quantize.rs:82-114, image types.rs:142-147 ---------------------
// The images of a workgroup's 128 blocks are put together in LDS and leave as one run of 16-byte stores (a thread
// writing its own image would store 2 bytes at a time, IMG bytes from its neighbour's).  Called by every thread of
// the workgroup; 128 * IMG is a multiple of 16, so the run is as aligned as `out`.
template <int IMG>
__device__ inline void flush_images(const uint8_t *img, uint8_t *out, size_t b0, size_t nblk) {
    __syncthreads();
    const int nb = nblk - b0 < 128 ? (int)(nblk - b0) : 128, nbytes = nb * IMG;
    uint8_t *g = out + b0 * IMG;
    if ((reinterpret_cast<uintptr_t>(out) & 15) == 0) {
        for (int o = threadIdx.x * 16; o + 16 <= nbytes; o += 128 * 16) *reinterpret_cast<uint4 *>(g + o) = *reinterpret_cast<const uint4 *>(img + o);
        for (int o = (nbytes & ~15) + threadIdx.x * 2; o < nbytes; o += 256) store_u16(g + o, load_u16(img + o));
    } else {
        for (int o = threadIdx.x * 2; o < nbytes; o += 256) store_u16(g + o, load_u16(img + o));
    }
}

__global__ void __launch_bounds__(128) quant_q8_0_kernel(const float *src, size_t numel, size_t nblk, uint8_t *out) {
    __shared__ __attribute__((aligned(16))) uint8_t img[128 * 34];
    const size_t b0 = (size_t)blockIdx.x * 128, b = b0 + threadIdx.x;
    if (b < nblk) {
        float x[32];
        int len;
        load_block32(src, numel, b, x, len);
        float max_abs = 0.0f;
#pragma unroll
        for (int i = 0; i < 32; i++)
            if (i < len) max_abs = fmaxf(max_abs, fabsf(x[i]));
        float scale = max_abs > 0.0f ? max_abs / 127.0f : 1.0f;
        uint8_t *o = img + threadIdx.x * 34;
        store_u16(o, f32_to_f16_bits(scale));
#pragma unroll
        for (int i = 0; i < 16; i++) {
            int q0 = (2 * i) < len ? round_clamp(x[2 * i] / scale, -127.0f, 127.0f) : 0;
            int q1 = (2 * i + 1) < len ? round_clamp(x[2 * i + 1] / scale, -127.0f, 127.0f) : 0;
            store_u16(o + 2 + 2 * i, (uint16_t)((q0 & 0xFF) | ((q1 & 0xFF) << 8)));
        }
    }
    flush_images<34>(img, out, b0, nblk);
}

// ---- Q4_0: quantize.rs:121-156, pack types.rs:190-198 ---------------------
__global__ void __launch_bounds__(128) quant_q4_0_kernel(const float *src, size_t numel, size_t nblk, uint8_t *out) {
    __shared__ __attribute__((aligned(16))) uint8_t img[128 * 18];
    const size_t b0 = (size_t)blockIdx.x * 128, b = b0 + threadIdx.x;
    if (b < nblk) {
        float x[32];
        int len;
        load_block32(src, numel, b, x, len);
        float max_abs = 0.0f;
#pragma unroll
        for (int i = 0; i < 32; i++)
            if (i < len) max_abs = fmaxf(max_abs, fabsf(x[i]));
        float scale = max_abs > 0.0f ? max_abs / 7.0f : 1.0f;
        uint8_t *o = img + threadIdx.x * 18;
        store_u16(o, f32_to_f16_bits(scale));
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t w = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                int e = 4 * i + j;
                int q = e < len ? round_clamp(x[e] / scale, -8.0f, 7.0f) : 0;
                w |= (uint32_t)((q + 8) & 0x0F) << (4 * j);
            }
            store_u16(o + 2 + 2 * i, (uint16_t)w);
        }
    }
    flush_images<18>(img, out, b0, nblk);
}

// ---- Q4_1: quantize.rs:163-205, image types.rs:249-255 --------------------
__global__ void __launch_bounds__(128) quant_q4_1_kernel(const float *src, size_t numel, size_t nblk, uint8_t *out) {
    __shared__ __attribute__((aligned(16))) uint8_t img[128 * 20];
    const size_t b0 = (size_t)blockIdx.x * 128, b = b0 + threadIdx.x;
    if (b < nblk) {
        float x[32];
        int len;
        load_block32(src, numel, b, x, len);
        float mn = INFINITY, mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 32; i++)
            if (i < len) {
                mn = fminf(mn, x[i]);
                mx = fmaxf(mx, x[i]);
            }
        float scale = mx > mn ? (mx - mn) / 15.0f : 1.0f;
        uint8_t *o = img + threadIdx.x * 20;
        store_u16(o, f32_to_f16_bits(scale));
        store_u16(o + 2, f32_to_f16_bits(mn));
        int nbytes = len / 2 < 16 ? len / 2 : 16; // the reference's pack loop bound
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t w = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                int e = 4 * i + j;
                int q = e < len ? round_clamp((x[e] - mn) / scale, 0.0f, 15.0f) : 0;
                if ((e >> 1) >= nbytes) q = 0;
                w |= (uint32_t)(q & 0x0F) << (4 * j);
            }
            store_u16(o + 4 + 2 * i, (uint16_t)w);
        }
    }
    flush_images<20>(img, out, b0, nblk);
}

// ---- Q5_0 / Q5_1: GGUF layouts; scale rules max_abs/15 and (max-min)/31 ---
template <bool WITH_MIN>
__global__ void __launch_bounds__(128) quant_q5_kernel(const float *src, size_t numel, size_t nblk, uint8_t *out) {
    __shared__ __attribute__((aligned(16))) uint8_t img[128 * 24];
    const size_t b0 = (size_t)blockIdx.x * 128, b = b0 + threadIdx.x;
    if (b < nblk) {
        float x[32];
        int len;
        load_block32(src, numel, b, x, len);
        float scale, mn = 0.0f;
        if (WITH_MIN) {
            float lo = INFINITY, hi = -INFINITY;
#pragma unroll
            for (int i = 0; i < 32; i++)
                if (i < len) {
                    lo = fminf(lo, x[i]);
                    hi = fmaxf(hi, x[i]);
                }
            scale = hi > lo ? (hi - lo) / 31.0f : 1.0f;
            mn = lo;
        } else {
            float max_abs = 0.0f;
#pragma unroll
            for (int i = 0; i < 32; i++)
                if (i < len) max_abs = fmaxf(max_abs, fabsf(x[i]));
            scale = max_abs > 0.0f ? max_abs / 15.0f : 1.0f;
        }
        uint32_t u[32];
#pragma unroll
        for (int i = 0; i < 32; i++) {
            if (WITH_MIN)
                u[i] = i < len ? (uint32_t)round_clamp((x[i] - mn) / scale, 0.0f, 31.0f) : 0u;
            else
                u[i] = i < len ? (uint32_t)(round_clamp(x[i] / scale, -16.0f, 15.0f) + 16) : 16u;
        }
        uint8_t *o = img + threadIdx.x * (WITH_MIN ? 24 : 22);
        store_u16(o, f32_to_f16_bits(scale));
        int off = 2;
        if (WITH_MIN) {
            store_u16(o + 2, f32_to_f16_bits(mn));
            off = 4;
        }
        uint32_t qh = 0;
#pragma unroll
        for (int j = 0; j < 16; j++) {
            qh |= ((u[j] >> 4) & 1u) << j;
            qh |= ((u[j + 16] >> 4) & 1u) << (j + 16);
        }
        store_u16(o + off, (uint16_t)qh);
        store_u16(o + off + 2, (uint16_t)(qh >> 16));
#pragma unroll
        for (int j = 0; j < 8; j++) {
            uint32_t b0 = (u[2 * j] & 0x0F) | ((u[2 * j + 16] & 0x0F) << 4);
            uint32_t b1 = (u[2 * j + 1] & 0x0F) | ((u[2 * j + 17] & 0x0F) << 4);
            store_u16(o + off + 4 + 2 * j, (uint16_t)(b0 | (b1 << 8)));
        }
    }
    flush_images<(WITH_MIN ? 24 : 22)>(img, out, b0, nblk);
}

// ---- Q4_K: one lane per 32-element sub-block, 8 lanes per superblock -------
// Rule: per sub-block mn = min(0, min x), mx = max x, scale = (mx-mn)/15,
// min = -mn; the superblock's d = max scale / 63, dmin = max min / 63 (stored
// as f16); 6-bit ls = round(63/max_scale * scale), lm likewise; codes
// q = clamp(round((x + dmin*lm) / (d*ls)), 0, 15) with the f16-rounded d, dmin.
// BITS = 5 is Q5_K: the same rule with 31 steps; image [header 16][qh 32][qs 128], the low four bits of a code where
// Q4_K has the code, the fifth bit of sub-block s, element l at bit s of qh[l].
template <int BITS>
__global__ void quant_qk_kernel(const float *src, size_t numel, size_t nsb, uint8_t *out) {
    constexpr float TOP = BITS == 5 ? 31.0f : 15.0f;
    constexpr int IMG = BITS == 5 ? 176 : 144, QS = BITS == 5 ? 48 : 16;
    size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t sb = t >> 3;
    int s = (int)(t & 7);
    bool live = sb < nsb;
    float x[32];
#pragma unroll
    for (int i = 0; i < 32; i++) x[i] = 0.0f;
    if (live) {
        size_t start = sb * 256 + (size_t)s * 32;
        if (start + 32 <= numel) {
            const float4 *p = reinterpret_cast<const float4 *>(src + start);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float4 v = p[i];
                x[4 * i] = v.x; x[4 * i + 1] = v.y; x[4 * i + 2] = v.z; x[4 * i + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 32; i++)
                if (start + i < numel) x[i] = src[start + i];
        }
    }
    float mn = INFINITY, mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 32; i++) {
        mn = fminf(mn, x[i]);
        mx = fmaxf(mx, x[i]);
    }
    if (mn > 0.0f) mn = 0.0f;
    float scale, smin;
    if (!(mx > mn)) {
        scale = 0.0f;
        smin = isfinite(mn) ? -mn : 0.0f;
    } else {
        scale = (mx - mn) / TOP;
        smin = -mn;
    }
    float max_scale = scale, max_min = smin;
#pragma unroll
    for (int m = 1; m < 8; m <<= 1) {
        max_scale = fmaxf(max_scale, __shfl_xor(max_scale, m));
        max_min = fmaxf(max_min, __shfl_xor(max_min, m));
    }
    float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    int ls = round_clamp(inv_scale * scale, 0.0f, 63.0f);
    int lm = round_clamp(inv_min * smin, 0.0f, 63.0f);
    uint16_t dh = f32_to_f16_bits(max_scale / 63.0f);
    uint16_t dminh = f32_to_f16_bits(max_min / 63.0f);
    float d = f16_bits_to_f32(dh), dmin = f16_bits_to_f32(dminh);
    float sd = d * (float)ls;
    float sm = dmin * (float)lm;
    // codes as 8 dwords of one code per byte (their low four bits), the fifth bits as one bit per element
    uint32_t cb[8], hb = 0;
#pragma unroll
    for (int w = 0; w < 8; w++) {
        uint32_t v = 0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int q = sd == 0.0f ? 0 : round_clamp((x[4 * w + j] + sm) / sd, 0.0f, TOP);
            v |= (uint32_t)(q & 15) << (8 * j);
            hb |= (uint32_t)(q >> 4) << (4 * w + j);
        }
        cb[w] = v;
    }
    // pair partner exchange: even lane (sub-block 2p) holds the low nibbles
    uint32_t other[8];
#pragma unroll
    for (int w = 0; w < 8; w++) other[w] = (uint32_t)__shfl_xor((int)cb[w], 1);
    // header values of all 8 sub-blocks
    int base_lane = (int)(threadIdx.x & 63) & ~7;
    uint32_t lsv[8], lmv[8], hbv[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        lsv[j] = (uint32_t)__shfl(ls, base_lane + j);
        lmv[j] = (uint32_t)__shfl(lm, base_lane + j);
        if (BITS == 5) hbv[j] = (uint32_t)__shfl((int)hb, base_lane + j);
    }
    if (!live) return;
    uint8_t *o = out + sb * IMG;
    if (BITS == 5) { // this lane's four bytes of qh: elements 4 s .. 4 s + 3, bit j from sub-block j
        uint32_t v = 0;
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int i = 0; i < 4; i++) v |= ((hbv[j] >> (4 * s + i)) & 1u) << (8 * i + j);
        *reinterpret_cast<uint32_t *>(o + 16 + 4 * s) = v;
    }
    if (s == 0) {
        uint32_t h[4];
        h[0] = (uint32_t)dh | ((uint32_t)dminh << 16);
        uint8_t sc[12];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            sc[j] = (uint8_t)(lsv[j] | ((lsv[j + 4] >> 4) << 6));
            sc[j + 4] = (uint8_t)(lmv[j] | ((lmv[j + 4] >> 4) << 6));
            sc[j + 8] = (uint8_t)((lsv[j + 4] & 0x0F) | ((lmv[j + 4] & 0x0F) << 4));
        }
#pragma unroll
        for (int w = 0; w < 3; w++)
            h[1 + w] = (uint32_t)sc[4 * w] | ((uint32_t)sc[4 * w + 1] << 8) | ((uint32_t)sc[4 * w + 2] << 16) |
                       ((uint32_t)sc[4 * w + 3] << 24);
        *reinterpret_cast<uint4 *>(o) = make_uint4(h[0], h[1], h[2], h[3]);
    }
    if ((s & 1) == 0) {
        int p = s >> 1;
        uint32_t pk[8];
#pragma unroll
        for (int w = 0; w < 8; w++) pk[w] = cb[w] | (other[w] << 4);
        uint4 *q = reinterpret_cast<uint4 *>(o + QS + 32 * p);
        q[0] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
        q[1] = make_uint4(pk[4], pk[5], pk[6], pk[7]);
    }
}

// Q6_K (GGUF superblock of 16 sub-blocks of 16 elements, 210 bytes: ql[128], qh[64], int8 scales[16], f16 d).
// One thread per sub-block, sixteen neighbouring lanes per superblock.  The quantiser rule is this build's own:
// per sub-block a = max |x|, scale = a / 31; the superblock's d = max scale / 127 (stored as f16);
// ls = round(127 / max_scale * scale) in 0..127; q = clamp(round(x / (d * ls)), -32, 31) with the f16-rounded d.
// Element e = 128 n + 32 c + l keeps the low four bits of u = q + 32 in ql[64 n + 32 (c & 1) + l] (low nibble for
// c < 2) and the upper two in qh[32 n + l] at bit 2 c.
__global__ void quant_q6_k_kernel(const float *src, size_t numel, size_t nsb, uint8_t *out) {
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t sb = t >> 4;
    const int s = (int)(t & 15);
    const bool live = sb < nsb;
    float x[16];
#pragma unroll
    for (int i = 0; i < 16; i++) x[i] = 0.0f;
    if (live) {
        const size_t start = sb * 256 + (size_t)s * 16;
#pragma unroll
        for (int i = 0; i < 16; i++)
            if (start + i < numel) x[i] = src[start + i];
    }
    float a = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) a = fmaxf(a, fabsf(x[i]));
    const float scale = a / 31.0f;
    float max_scale = scale;
#pragma unroll
    for (int m = 1; m < 16; m <<= 1) max_scale = fmaxf(max_scale, __shfl_xor(max_scale, m));
    const float inv = max_scale > 0.0f ? 127.0f / max_scale : 0.0f;
    const int ls = round_clamp(inv * scale, 0.0f, 127.0f);
    const uint16_t dh = f32_to_f16_bits(max_scale / 127.0f);
    const float sd = f16_bits_to_f32(dh) * (float)ls;
    // the sixteen codes u = q + 32, one per byte; low nibbles and upper bit pairs apart
    uint32_t lo[4], hi[4];
#pragma unroll
    for (int w = 0; w < 4; w++) {
        lo[w] = hi[w] = 0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int q = sd == 0.0f ? 0 : round_clamp(x[4 * w + j] / sd, -32.0f, 31.0f);
            const uint32_t u = (uint32_t)(q + 32);
            lo[w] |= (u & 0x0Fu) << (8 * j);
            hi[w] |= (u >> 4) << (8 * j);
        }
    }
    // s = 8 n + 2 c + lh: the partner with c + 2 (lane s ^ 4) supplies the high nibbles of the same ql bytes; the
    // lanes s + 2, s + 4, s + 6 supply the other bit pairs of the same qh bytes
    const int c = (s >> 1) & 3, n = s >> 3, lh = s & 1;
    uint32_t plo[4], h2[4], h4[4], h6[4];
#pragma unroll
    for (int w = 0; w < 4; w++) {
        plo[w] = (uint32_t)__shfl_xor((int)lo[w], 4);
        h2[w] = (uint32_t)__shfl_xor((int)hi[w], 2);
        h4[w] = (uint32_t)__shfl_xor((int)hi[w], 4);
        h6[w] = (uint32_t)__shfl_xor((int)hi[w], 6);
    }
    if (!live) return;
    uint8_t *o = out + sb * 210;
    if (c < 2) {
        uint8_t *ql = o + 64 * n + 32 * c + 16 * lh;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const uint32_t v = lo[w] | (plo[w] << 4);
            store_u16(ql + 4 * w, (uint16_t)v);
            store_u16(ql + 4 * w + 2, (uint16_t)(v >> 16));
        }
    }
    if (c == 0) {
        uint8_t *qh = o + 128 + 32 * n + 16 * lh;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const uint32_t v = hi[w] | (h2[w] << 2) | (h4[w] << 4) | (h6[w] << 6);
            store_u16(qh + 4 * w, (uint16_t)v);
            store_u16(qh + 4 * w + 2, (uint16_t)(v >> 16));
        }
    }
    o[192 + s] = (uint8_t)ls;
    if (s == 0) store_u16(o + 208, dh);
}

// ---- F16: quantize.rs:212-218 --------------------------------------------
// eight elements per thread where both sides are 16-byte aligned, one by one otherwise and for the last few
__global__ void quant_f16_kernel(const float *src, size_t numel, uint16_t *out) {
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x, i = t * 8;
    if (i >= numel) return;
    if (i + 8 <= numel && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
        const float4 a = reinterpret_cast<const float4 *>(src + i)[0], b = reinterpret_cast<const float4 *>(src + i)[1];
        const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        uint32_t w[4];
#pragma unroll
        for (int j = 0; j < 4; j++) w[j] = (uint32_t)f32_to_f16_bits(v[2 * j]) | ((uint32_t)f32_to_f16_bits(v[2 * j + 1]) << 16);
        *reinterpret_cast<uint4 *>(out + i) = make_uint4(w[0], w[1], w[2], w[3]);
    } else {
        for (size_t j = i; j < numel && j < i + 8; j++) out[j] = f32_to_f16_bits(src[j]);
    }
}
__global__ void dequant_f16_kernel(const uint16_t *src, size_t numel, float *out) {
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x, i = t * 8;
    if (i >= numel) return;
    if (i + 8 <= numel && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
        const uint4 q = *reinterpret_cast<const uint4 *>(src + i);
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        float v[8];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v[2 * j] = f16_bits_to_f32((uint16_t)w[j]);
            v[2 * j + 1] = f16_bits_to_f32((uint16_t)(w[j] >> 16));
        }
        reinterpret_cast<float4 *>(out + i)[0] = make_float4(v[0], v[1], v[2], v[3]);
        reinterpret_cast<float4 *>(out + i)[1] = make_float4(v[4], v[5], v[6], v[7]);
    } else {
        for (size_t j = i; j < numel && j < i + 8; j++) out[j] = f16_bits_to_f32(src[j]);
    }
}

// ---- dequantisers: dequantize.rs:89-92, 116-121, 145-151 -------------------
// One thread per 32 elements; for Q4_K a thread handles one sub-block.
// The 32 values of a thread go through an LDS tile (rows padded to 33 floats), so that the workgroup's 16 KB of
// output leave as consecutive 16-byte stores instead of 128-byte strides between neighbouring threads.
__global__ void __launch_bounds__(128) dequant_kernel(int type, const uint8_t *packed, size_t numel, size_t n32, float *out) {
    __shared__ float tile[128 * 33];
    const size_t t0 = (size_t)blockIdx.x * 128;
    size_t t = t0 + threadIdx.x;
    const bool live = t < n32;
    if (!live) t = n32 - 1; // computes a block again, stores nothing: every thread has to reach the barrier
    float y[32];
    switch (type) {
    case AXQ_Q8_0: {
        const uint8_t *b = packed + t * 34;
        float scale = f16_bits_to_f32(load_u16(b));
#pragma unroll
        for (int i = 0; i < 16; i++) {
            uint16_t w = load_u16(b + 2 + 2 * i);
            y[2 * i] = (float)(int8_t)(w & 0xFF) * scale;
            y[2 * i + 1] = (float)(int8_t)(w >> 8) * scale;
        }
        break;
    }
    case AXQ_Q4_0: {
        const uint8_t *b = packed + t * 18;
        float scale = f16_bits_to_f32(load_u16(b));
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t w = load_u16(b + 2 + 2 * i);
#pragma unroll
            for (int j = 0; j < 4; j++) y[4 * i + j] = (float)((int)((w >> (4 * j)) & 0x0F) - 8) * scale;
        }
        break;
    }
    case AXQ_Q4_1: {
        const uint8_t *b = packed + t * 20;
        float scale = f16_bits_to_f32(load_u16(b));
        float mn = f16_bits_to_f32(load_u16(b + 2));
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t w = load_u16(b + 4 + 2 * i);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float a = (float)((w >> (4 * j)) & 0x0F) * scale;
                y[4 * i + j] = a + mn;
            }
        }
        break;
    }
    case AXQ_Q5_0:
    case AXQ_Q5_1: {
        bool with_min = type == AXQ_Q5_1;
        const uint8_t *b = packed + t * (with_min ? 24 : 22);
        float d = f16_bits_to_f32(load_u16(b));
        float m = with_min ? f16_bits_to_f32(load_u16(b + 2)) : 0.0f;
        int off = with_min ? 4 : 2;
        uint32_t qh = (uint32_t)load_u16(b + off) | ((uint32_t)load_u16(b + off + 2) << 16);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            uint32_t w = load_u16(b + off + 4 + 2 * j);
#pragma unroll
            for (int h = 0; h < 2; h++) {
                int e = 2 * j + h;
                uint32_t byte = (w >> (8 * h)) & 0xFF;
                int u0 = (int)((byte & 0x0F) | (((qh >> e) & 1u) << 4));
                int u1 = (int)((byte >> 4) | (((qh >> (e + 16)) & 1u) << 4));
                if (with_min) {
                    float a = (float)u0 * d;
                    float c = (float)u1 * d;
                    y[e] = a + m;
                    y[e + 16] = c + m;
                } else {
                    y[e] = (float)(u0 - 16) * d;
                    y[e + 16] = (float)(u1 - 16) * d;
                }
            }
        }
        break;
    }
    case AXQ_Q4_K:
    case AXQ_Q5_K: {
        size_t sb = t >> 3;
        int s = (int)(t & 7);
        const bool five = type == AXQ_Q5_K;
        const uint8_t *b = packed + sb * (five ? 176 : 144);
        float d = f16_bits_to_f32(load_u16(b));
        float dmin = f16_bits_to_f32(load_u16(b + 2));
        const uint8_t *sc = b + 4;
        uint32_t l, m;
        if (s < 4) {
            l = sc[s] & 63;
            m = sc[s + 4] & 63;
        } else {
            l = (uint32_t)((sc[s + 4] & 0x0F) | ((sc[s - 4] >> 6) << 4));
            m = (uint32_t)((sc[s + 4] >> 4) | ((sc[s] >> 6) << 4));
        }
        float sd = d * (float)l;
        float sm = dmin * (float)m;
        const uint32_t *qs = reinterpret_cast<const uint32_t *>(b + (five ? 48 : 16) + 32 * (s >> 1));
        const uint32_t *qh = reinterpret_cast<const uint32_t *>(b + 16); // Q5_K: bit s of byte l = fifth bit of the sub-block's element l
        int shift = (s & 1) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t w = (qs[i] >> shift) & 0x0F0F0F0Fu;
            if (five) w |= ((qh[i] >> s) & 0x01010101u) << 4;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float a = sd * (float)((w >> (8 * j)) & 0x1F);
                y[4 * i + j] = a - sm;
            }
        }
        break;
    }
    case AXQ_Q6_K: { // elements 32 (t % 8) .. of superblock t / 8: two sub-blocks; y = (d * scale) * q
        const size_t sb = t >> 3;
        const int g = (int)(t & 7), n = g >> 2, c = g & 3;
        const uint8_t *b = packed + sb * 210;
        const float d = f16_bits_to_f32(load_u16(b + 208));
        const float ds0 = d * (float)(int8_t)b[192 + 2 * g], ds1 = d * (float)(int8_t)b[192 + 2 * g + 1];
        const uint8_t *ql = b + 64 * n + 32 * (c & 1), *qh = b + 128 + 32 * n;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const uint32_t wl = load_u16(ql + 2 * i), wh = load_u16(qh + 2 * i);
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int lo = (int)((wl >> (8 * j + 4 * (c >> 1))) & 0x0F), hi = (int)((wh >> (8 * j + 2 * c)) & 3);
                const int q = (lo | (hi << 4)) - 32;
                y[2 * i + j] = (i < 8 ? ds0 : ds1) * (float)q;
            }
        }
        break;
    }
    default:
        return;
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < 32; i++) tile[threadIdx.x * 33 + i] = y[i];
    }
    __syncthreads();
    const size_t start = t0 * 32; // of the workgroup
    const bool vec = (reinterpret_cast<uintptr_t>(out) & 15) == 0;
#pragma unroll
    for (int r = 0; r < 8; r++) {
        const int e4 = r * 128 + threadIdx.x, row = e4 >> 3, col = (e4 & 7) * 4;
        const size_t g = start + (size_t)e4 * 4;
        const float *src = tile + row * 33 + col;
        if (vec && g + 4 <= numel) {
            *reinterpret_cast<float4 *>(out + g) = make_float4(src[0], src[1], src[2], src[3]);
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (g + i < numel) out[g + i] = src[i];
        }
    }
}

// ---- packed image <-> planar device layout ---------------------------------
// One thread per block (per superblock for Q4_K).  to_planar selects the copy
// direction; the two directions are exact inverses.
struct PlanarDesc {
    uint8_t *codes, *meta, *qh;
    size_t codes_pitch, meta_pitch, qh_pitch;
    int64_t n_rows, blocks_per_row;
    int type;
};

__device__ inline void copy_u16s(uint8_t *dst, const uint8_t *src, int nbytes) {
    for (int i = 0; i < nbytes; i += 2) store_u16(dst + i, load_u16(src + i));
}

__global__ void repack_kernel(PlanarDesc d, uint8_t *packed, bool to_planar) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t total = d.n_rows * d.blocks_per_row;
    if (t >= total) return;
    int64_t row = t / d.blocks_per_row, blk = t % d.blocks_per_row;
    int code_bytes, meta_bytes, qh_bytes = 0;
    switch (d.type) {
    case AXQ_Q8_0: code_bytes = 32; meta_bytes = 2; break;
    case AXQ_Q4_0: code_bytes = 16; meta_bytes = 2; break;
    case AXQ_Q4_1: code_bytes = 16; meta_bytes = 4; break;
    case AXQ_Q5_0: code_bytes = 16; meta_bytes = 2; qh_bytes = 4; break;
    case AXQ_Q5_1: code_bytes = 16; meta_bytes = 4; qh_bytes = 4; break;
    case AXQ_Q4_K: code_bytes = 128; meta_bytes = 16; break;
    default: return;
    }
    uint8_t *img = packed + (size_t)t * (size_t)(code_bytes + meta_bytes + qh_bytes);
    uint8_t *meta = d.meta + (size_t)row * d.meta_pitch + (size_t)blk * meta_bytes;
    if (to_planar) copy_u16s(meta, img, meta_bytes); else copy_u16s(img, meta, meta_bytes);
    if (qh_bytes) {
        uint8_t *qh = d.qh + (size_t)row * d.qh_pitch + (size_t)blk * 4;
        if (to_planar) copy_u16s(qh, img + meta_bytes, 4); else copy_u16s(img + meta_bytes, qh, 4);
    }
    uint8_t *img_codes = img + meta_bytes + qh_bytes;
    uint8_t *row_codes = d.codes + (size_t)row * d.codes_pitch;
    if (d.type == AXQ_Q4_K) {
        for (int c = 0; c < 8; c++) { // 16-byte runs keep their order inside the run
            uint8_t *pl = row_codes + q4k_code_offset(d.blocks_per_row, blk, 16 * c);
            if (to_planar) copy_u16s(pl, img_codes + 16 * c, 16); else copy_u16s(img_codes + 16 * c, pl, 16);
        }
    } else {
        uint8_t *pl = row_codes + (size_t)blk * code_bytes;
        if (to_planar) copy_u16s(pl, img_codes, code_bytes); else copy_u16s(img_codes, pl, code_bytes);
    }
}

// The same copy for images whose base is 16-byte aligned: a workgroup takes 128 consecutive blocks, whose images
// form one contiguous, 16-byte aligned run (128 times any image size is a multiple of 16), moves that run between
// memory and LDS with 16-byte accesses, and serves the planes from LDS: one thread per block for the scales (and
// the high bits), one thread per 16 bytes of codes.  Every access to memory is as wide as its alignment allows
// and consecutive threads touch consecutive addresses.
template <int IMG, int META, int QH, int CODE>
__global__ void __launch_bounds__(256) repack_lds_kernel(PlanarDesc d, uint8_t *packed, bool to_planar, int64_t total) {
    constexpr int NB = 128, CU = CODE / 16;
    __shared__ __attribute__((aligned(16))) uint8_t img[NB * IMG];
    const int tid = threadIdx.x;
    const int64_t t0 = (int64_t)blockIdx.x * NB;
    const int nb = total - t0 < NB ? (int)(total - t0) : NB;
    const int nbytes = nb * IMG;
    uint8_t *g = packed + (size_t)t0 * IMG;
    if (to_planar) {
        for (int o = tid * 16; o + 16 <= nbytes; o += 256 * 16) *reinterpret_cast<uint4 *>(img + o) = *reinterpret_cast<const uint4 *>(g + o);
        for (int o = (nbytes & ~15) + tid * 2; o < nbytes; o += 512) store_u16(img + o, load_u16(g + o)); // a last run's tail
        __syncthreads();
    }
    for (int u = tid; u < nb; u += 256) {
        const int64_t t = t0 + u, row = t / d.blocks_per_row, blk = t - row * d.blocks_per_row;
        uint8_t *li = img + u * IMG;
        uint8_t *pm = d.meta + (size_t)row * d.meta_pitch + (size_t)blk * META;
        if (META == 2) {
            if (to_planar) store_u16(pm, load_u16(li)); else store_u16(li, load_u16(pm));
        } else if (META == 4) {
            if (to_planar) {
                *reinterpret_cast<uint32_t *>(pm) = (uint32_t)load_u16(li) | ((uint32_t)load_u16(li + 2) << 16);
            } else {
                const uint32_t v = *reinterpret_cast<const uint32_t *>(pm);
                store_u16(li, (uint16_t)v); store_u16(li + 2, (uint16_t)(v >> 16));
            }
        } else { // 16: IMG is a multiple of 16 too, so the LDS side is aligned as well
            if (to_planar) *reinterpret_cast<uint4 *>(pm) = *reinterpret_cast<const uint4 *>(li);
            else *reinterpret_cast<uint4 *>(li) = *reinterpret_cast<const uint4 *>(pm);
        }
        if (QH) {
            uint8_t *ph = d.qh + (size_t)row * d.qh_pitch + (size_t)blk * 4;
            if (to_planar) {
                *reinterpret_cast<uint32_t *>(ph) = (uint32_t)load_u16(li + META) | ((uint32_t)load_u16(li + META + 2) << 16);
            } else {
                const uint32_t v = *reinterpret_cast<const uint32_t *>(ph);
                store_u16(li + META, (uint16_t)v); store_u16(li + META + 2, (uint16_t)(v >> 16));
            }
        }
    }
    for (int v = tid; v < nb * CU; v += 256) {
        const int u = v / CU, c = v - u * CU;
        const int64_t t = t0 + u, row = t / d.blocks_per_row, blk = t - row * d.blocks_per_row;
        uint8_t *li = img + u * IMG + META + QH + 16 * c; // 2-byte aligned
        uint8_t *pc = d.codes + (size_t)row * d.codes_pitch +
                      (d.type == AXQ_Q4_K ? q4k_code_offset(d.blocks_per_row, blk, 16 * c) : (size_t)blk * CODE + 16 * c);
        if (to_planar) {
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; i++) w[i] = (uint32_t)load_u16(li + 4 * i) | ((uint32_t)load_u16(li + 4 * i + 2) << 16);
            *reinterpret_cast<uint4 *>(pc) = make_uint4(w[0], w[1], w[2], w[3]);
        } else {
            const uint4 q = *reinterpret_cast<const uint4 *>(pc);
            const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int i = 0; i < 4; i++) { store_u16(li + 4 * i, (uint16_t)w[i]); store_u16(li + 4 * i + 2, (uint16_t)(w[i] >> 16)); }
        }
    }
    if (!to_planar) {
        __syncthreads();
        for (int o = tid * 16; o + 16 <= nbytes; o += 256 * 16) *reinterpret_cast<uint4 *>(g + o) = *reinterpret_cast<const uint4 *>(img + o);
        for (int o = (nbytes & ~15) + tid * 2; o < nbytes; o += 512) store_u16(g + o, load_u16(img + o));
    }
}

// Q6_K: image [ql 128][qh 64][scales 16][d 2] <-> planes: codes = the rows' ql runs (128 bytes per superblock), qh = their
// qh runs (64), meta = per row the superblocks' scales (16 bytes each) followed by their d values (2 bytes each).
// One thread per 16-byte piece (13 per superblock, the last one scales and d); two bytes at a time on the image side.
__global__ void __launch_bounds__(256) repack_q6k_kernel(PlanarDesc d, uint8_t *packed, bool to_planar, int64_t total) {
    const int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (v >= total * 13) return;
    const int64_t t = v / 13;
    const int piece = (int)(v - t * 13);
    const int64_t row = t / d.blocks_per_row, sb = t - row * d.blocks_per_row;
    uint8_t *img = packed + (size_t)t * 210;
    uint8_t *pl, *im;
    if (piece < 8) { pl = d.codes + (size_t)row * d.codes_pitch + (size_t)sb * 128 + 16 * piece; im = img + 16 * piece; }
    else if (piece < 12) { pl = d.qh + (size_t)row * d.qh_pitch + (size_t)sb * 64 + 16 * (piece - 8); im = img + 128 + 16 * (piece - 8); }
    else { pl = d.meta + (size_t)row * d.meta_pitch + (size_t)sb * 16; im = img + 192; }
    if (to_planar) copy_u16s(pl, im, 16); else copy_u16s(im, pl, 16);
    if (piece == 12) {
        uint8_t *dp = d.meta + (size_t)row * d.meta_pitch + (size_t)d.blocks_per_row * 16 + (size_t)sb * 2;
        if (to_planar) store_u16(dp, load_u16(img + 208)); else store_u16(img + 208, load_u16(dp));
    }
}

// Q5_K: image [header 16][qh 32][qs 128] <-> planes: meta = the headers, qh = the fifth bits as they are, codes = the qs
// runs laid out as Q4_K's (q4k_code_offset).  One thread per 16-byte piece, eleven per superblock.
__global__ void __launch_bounds__(256) repack_q5k_kernel(PlanarDesc d, uint8_t *packed, bool to_planar, int64_t total) {
    const int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (v >= total * 11) return;
    const int64_t t = v / 11;
    const int piece = (int)(v - t * 11);
    const int64_t row = t / d.blocks_per_row, sb = t - row * d.blocks_per_row;
    uint8_t *im = packed + (size_t)t * 176 + 16 * piece, *pl;
    if (piece == 0) pl = d.meta + (size_t)row * d.meta_pitch + (size_t)sb * 16;
    else if (piece < 3) pl = d.qh + (size_t)row * d.qh_pitch + (size_t)sb * 32 + 16 * (piece - 1);
    else pl = d.codes + (size_t)row * d.codes_pitch + q4k_code_offset(d.blocks_per_row, sb, 16 * (piece - 3));
    if (to_planar) copy_u16s(pl, im, 16); else copy_u16s(im, pl, 16);
}

inline unsigned grid_for(size_t n, unsigned block) { return (unsigned)((n + block - 1) / block); }

} // namespace

int axq_dev_quantize(axq_ctx *ctx, int type, const float *src, size_t numel, uint8_t *packed) {
    if (numel == 0) return AXQ_OK;
    size_t nblk = axq_num_blocks(type, numel);
    const unsigned B = 128;
    switch (type) {
    case AXQ_Q8_0: quant_q8_0_kernel<<<grid_for(nblk, B), B, 0, ctx->stream>>>(src, numel, nblk, packed); break;
    case AXQ_Q4_0: quant_q4_0_kernel<<<grid_for(nblk, B), B, 0, ctx->stream>>>(src, numel, nblk, packed); break;
    case AXQ_Q4_1: quant_q4_1_kernel<<<grid_for(nblk, B), B, 0, ctx->stream>>>(src, numel, nblk, packed); break;
    case AXQ_Q5_0: quant_q5_kernel<false><<<grid_for(nblk, B), B, 0, ctx->stream>>>(src, numel, nblk, packed); break;
    case AXQ_Q5_1: quant_q5_kernel<true><<<grid_for(nblk, B), B, 0, ctx->stream>>>(src, numel, nblk, packed); break;
    case AXQ_Q4_K: quant_qk_kernel<4><<<grid_for(nblk * 8, B), B, 0, ctx->stream>>>(src, numel, nblk, packed); break;
    case AXQ_Q5_K: quant_qk_kernel<5><<<grid_for(nblk * 8, B), B, 0, ctx->stream>>>(src, numel, nblk, packed); break;
    case AXQ_Q6_K: quant_q6_k_kernel<<<grid_for(nblk * 16, B), B, 0, ctx->stream>>>(src, numel, nblk, packed); break;
    case AXQ_F16: quant_f16_kernel<<<grid_for((numel + 7) / 8, 256), 256, 0, ctx->stream>>>(src, numel, (uint16_t *)packed); break;
    case AXQ_F32:
        AXQ_HIP(ctx, hipMemcpyAsync(packed, src, numel * 4, hipMemcpyDeviceToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
        return AXQ_OK;
    default: return axq_fail(ctx, AXQ_ERR_INVALID_QUANT_TYPE, "Invalid quantization type: %d", type);
    }
    AXQ_LAUNCH_CHECK(ctx, "quantize kernel");
    return AXQ_OK;
}

int axq_dev_dequantize(axq_ctx *ctx, int type, const uint8_t *packed, size_t numel, float *dst) {
    if (numel == 0) return AXQ_OK;
    switch (type) {
    case AXQ_Q8_0: case AXQ_Q4_0: case AXQ_Q4_1: case AXQ_Q5_0: case AXQ_Q5_1: case AXQ_Q4_K: case AXQ_Q6_K: case AXQ_Q5_K: {
        size_t n32 = (numel + 31) / 32;
        dequant_kernel<<<grid_for(n32, 128), 128, 0, ctx->stream>>>(type, packed, numel, n32, dst);
        break;
    }
    case AXQ_F16:
        dequant_f16_kernel<<<grid_for((numel + 7) / 8, 256), 256, 0, ctx->stream>>>((const uint16_t *)packed, numel, dst);
        break;
    case AXQ_F32:
        AXQ_HIP(ctx, hipMemcpyAsync(dst, packed, numel * 4, hipMemcpyDeviceToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
        return AXQ_OK;
    default: return axq_fail(ctx, AXQ_ERR_INVALID_QUANT_TYPE, "Invalid quantization type: %d", type);
    }
    AXQ_LAUNCH_CHECK(ctx, "dequantize kernel");
    return AXQ_OK;
}

int axq_dev_repack(axq_ctx *ctx, const axq_weight *w, uint8_t *packed, bool to_planar) {
    if (w->type == AXQ_F16 || w->type == AXQ_F32) {
        void *dst = to_planar ? (void *)w->codes : (void *)packed;
        const void *src = to_planar ? (const void *)packed : (const void *)w->codes;
        AXQ_HIP(ctx, hipMemcpyAsync(dst, src, w->packed_bytes, hipMemcpyDeviceToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
        return AXQ_OK;
    }
    PlanarDesc d;
    d.codes = w->codes; d.meta = w->meta; d.qh = w->qh;
    d.codes_pitch = w->codes_pitch; d.meta_pitch = w->meta_pitch; d.qh_pitch = w->qh_pitch;
    d.n_rows = w->n_rows;
    d.blocks_per_row = w->k / (int64_t)axq_type_block_size(w->type);
    d.type = w->type;
    size_t total = (size_t)(d.n_rows * d.blocks_per_row);
    if (total == 0) return AXQ_OK;
    if (w->type == AXQ_Q5_K) {
        repack_q5k_kernel<<<grid_for(total * 11, 256), 256, 0, ctx->stream>>>(d, packed, to_planar, (int64_t)total);
        AXQ_LAUNCH_CHECK(ctx, "repack kernel");
        return AXQ_OK;
    }
    if (w->type == AXQ_Q6_K) {
        repack_q6k_kernel<<<grid_for(total * 13, 256), 256, 0, ctx->stream>>>(d, packed, to_planar, (int64_t)total);
        AXQ_LAUNCH_CHECK(ctx, "repack kernel");
        return AXQ_OK;
    }
    if ((reinterpret_cast<uintptr_t>(packed) & 15) == 0) { // the usual case: allocations are aligned far beyond that
        const unsigned grid = grid_for(total, 128);
        const int64_t n = (int64_t)total;
        switch (w->type) {
        case AXQ_Q8_0: repack_lds_kernel<34, 2, 0, 32><<<grid, 256, 0, ctx->stream>>>(d, packed, to_planar, n); break;
        case AXQ_Q4_0: repack_lds_kernel<18, 2, 0, 16><<<grid, 256, 0, ctx->stream>>>(d, packed, to_planar, n); break;
        case AXQ_Q4_1: repack_lds_kernel<20, 4, 0, 16><<<grid, 256, 0, ctx->stream>>>(d, packed, to_planar, n); break;
        case AXQ_Q5_0: repack_lds_kernel<22, 2, 4, 16><<<grid, 256, 0, ctx->stream>>>(d, packed, to_planar, n); break;
        case AXQ_Q5_1: repack_lds_kernel<24, 4, 4, 16><<<grid, 256, 0, ctx->stream>>>(d, packed, to_planar, n); break;
        default: repack_lds_kernel<144, 16, 0, 128><<<grid, 256, 0, ctx->stream>>>(d, packed, to_planar, n); break;
        }
    } else {
        repack_kernel<<<grid_for(total, 128), 128, 0, ctx->stream>>>(d, packed, to_planar);
    }
    AXQ_LAUNCH_CHECK(ctx, "repack kernel");
    return AXQ_OK;
}
