/*
 * CPU oracle for the block-quantized matmul path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker that the GPU library is compared against.  It is
 * loaded by the tests, by the smoke entry and by the benchmark's cpu_baseline
 * leg; the product library never links, loads or calls it.
 *
 * It restates, function by function, the CPU algorithm of the reference crate
 * `axonml-quant` (Rust, cannot be compiled here: no cargo/rustc in the image):
 *
 *   quantize_q8_0   <- crates/axonml-quant/src/quantize.rs:82-114
 *   quantize_q4_0   <- crates/axonml-quant/src/quantize.rs:121-156
 *   quantize_q4_1   <- crates/axonml-quant/src/quantize.rs:163-205
 *   quantize_f16    <- crates/axonml-quant/src/quantize.rs:212-218
 *   quantize_f32    <- crates/axonml-quant/src/quantize.rs:225-228
 *   byte images     <- crates/axonml-quant/src/types.rs:142-147 (Q8),
 *                      :190-206 (Q4_0 pack + to_bytes), :249-255 (Q4_1)
 *   dequantize      <- crates/axonml-quant/src/dequantize.rs:34-54 (truncate to
 *                      numel), :89-92 (Q8), :116-121 (Q4_0), :145-151 (Q4_1)
 *   matmul          <- the composition dequantize_tensor -> Tensor::matmul
 *                      (crates/axonml-tensor/src/tensor.rs:1020-1045) ->
 *                      CpuBackend::sgemm (crates/axonml-core/src/backends/
 *                      cpu.rs:566-598) with Linear's y = x * W^T convention
 *                      (crates/axonml-nn/src/layers/linear.rs:104-140).
 *
 * Third-party arithmetic on that path, absent from the reference tree:
 *   half 2.7.1 (f16::from_f32 / to_f32): IEEE 754 binary16, round to nearest
 *     even, restated in axo_f32_to_f16 / axo_f16_to_f32 and pinned in the tests
 *     against numpy's float16 over every binary16 boundary.
 *   matrixmultiply 0.3.10 (sgemm): f32 multiply-accumulate in a blocked order
 *     that is not restated; outputs are pinned to the reference only within the
 *     1e-3 relative tolerance the path is specified to, and against an f64
 *     accumulation of the same dequantised weights.
 *
 * Pin status of each function:
 *   Q8_0 / Q4_0 / Q4_1 / F16 / F32 codecs: pinned by hand-computed known-answer
 *     blocks derived from the reference source (zero block, ramp, half-way
 *     rounding cases, tail block, Q4_1 odd tail) and by the reference's own
 *     test inputs (types.rs:366-389, dequantize.rs:204-272).
 *   Q5_K: Q4_K's rule with 31 steps and a fifth bit per code; layout and dequantiser from the published GGUF block
 *     (hand-built superblocks, an independent numpy statement of ggml's row dequantiser); quantiser "parity unpinned".
 *   Q6_K: as Q4_K below -- no reference code, no fixture; the layout and the dequantiser follow the published GGUF
 *     block (pinned by hand-built superblocks, one-hot codes and an independent numpy statement of ggml's row
 *     dequantiser), the QUANTISER rule is this build's own ("parity unpinned").
 *   Q5_0 / Q5_1 / Q4_K: the reference defines no codec for them (Q5_x silently
 *     aliases Q4_0, quantize.rs:47-50; Q4_K does not exist).  Byte layouts
 *     follow the public GGUF block spec and are pinned by hand-built blocks;
 *     the QUANTISER rules are this build's own ("parity unpinned": nothing in
 *     the reference can confirm them).  What the rules say is pinned by
 *     known-answer blocks worked by hand (half-way values, a whole Q4_K
 *     superblock with power-of-two spans, the 6-bit rounding of scale and
 *     minimum) and by the error bound the rule implies from the stored fields.
 *
 * Build: see oracle/Makefile (gcc, -O2 -ffp-contract=off, no fast-math).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define AXO_API __attribute__((visibility("default")))

/* Type ids: the reference enum order (types.rs:17-41) with Q4_K appended. */
enum {
    AXO_Q8_0 = 0,
    AXO_Q4_0 = 1,
    AXO_Q4_1 = 2,
    AXO_Q5_0 = 3,
    AXO_Q5_1 = 4,
    AXO_F16 = 5,
    AXO_F32 = 6,
    AXO_Q4_K = 7,
    AXO_Q6_K = 8,
    AXO_Q5_K = 9
};

/* ------------------------------------------------------------------------- */
/* binary16 <-> binary32, IEEE round-to-nearest-even (half 2.7.1 semantics)   */
/* ------------------------------------------------------------------------- */

AXO_API uint16_t axo_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x7FFFFFu;
    if (exp == 0xFF) { /* inf / nan */
        if (man == 0) return (uint16_t)(sign | 0x7C00u);
        /* quiet the nan, keep top payload bits */
        return (uint16_t)(sign | 0x7C00u | 0x0200u | (man >> 13));
    }
    int32_t e = (int32_t)exp - 127 + 15;
    if (e >= 0x1F) return (uint16_t)(sign | 0x7C00u); /* overflow -> inf */
    if (e <= 0) {
        /* subnormal half or zero */
        if (e < -10) return (uint16_t)sign; /* too small: rounds to zero */
        man |= 0x800000u;                   /* implicit one */
        uint32_t shift = (uint32_t)(14 - e); /* 14..24 */
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1u))) half_man++;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half = sign | ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++; /* may carry into exp/inf: correct */
    return (uint16_t)half;
}

AXO_API float axo_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t x;
    if (exp == 0) {
        if (man == 0) {
            x = sign;
        } else {
            /* normalise the subnormal */
            int e = -1;
            do {
                e++;
                man <<= 1;
            } while ((man & 0x400u) == 0);
            man &= 0x3FFu;
            x = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 0x1F) {
        x = sign | 0x7F800000u | (man << 13);
    } else {
        x = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

/* ------------------------------------------------------------------------- */
/* Type registry  (types.rs:45-78, with Q4_K = 256-element / 144-byte)        */
/* ------------------------------------------------------------------------- */

AXO_API size_t axo_block_size(int type) {
    switch (type) {
    case AXO_Q8_0: case AXO_Q4_0: case AXO_Q4_1: case AXO_Q5_0: case AXO_Q5_1: return 32;
    case AXO_Q4_K: case AXO_Q6_K: case AXO_Q5_K: return 256;
    case AXO_F16: case AXO_F32: return 1;
    default: return 0;
    }
}

AXO_API size_t axo_bytes_per_block(int type) {
    switch (type) {
    case AXO_Q8_0: return 34;
    case AXO_Q4_0: return 18;
    case AXO_Q4_1: return 20;
    case AXO_Q5_0: return 22;
    case AXO_Q5_1: return 24;
    case AXO_Q4_K: return 144;
    case AXO_Q6_K: return 210;
    case AXO_Q5_K: return 176;
    case AXO_F16: return 2;
    case AXO_F32: return 4;
    default: return 0;
    }
}

AXO_API size_t axo_num_blocks(int type, size_t numel) {
    size_t bs = axo_block_size(type);
    if (bs == 0) return 0;
    return (numel + bs - 1) / bs;
}

AXO_API size_t axo_packed_bytes(int type, size_t numel) {
    return axo_num_blocks(type, numel) * axo_bytes_per_block(type);
}

/* Rust `f32::max`/`min` ignore a NaN operand; fmaxf/fminf do the same. */
static inline float rs_max(float a, float b) { return fmaxf(a, b); }
static inline float rs_min(float a, float b) { return fminf(a, b); }

/* Rust: v.round().clamp(lo, hi) as iN.  round() is half away from zero
 * (roundf); clamp keeps NaN; the `as` cast maps NaN to 0 and saturates. */
static inline int rs_round_clamp(float v, float lo, float hi) {
    float r = roundf(v);
    if (isnan(r)) return 0;
    if (r < lo) r = lo;
    if (r > hi) r = hi;
    return (int)r;
}

static inline void put_u16(uint8_t *p, uint16_t v) {
    p[0] = (uint8_t)(v & 0xFF);
    p[1] = (uint8_t)(v >> 8);
}
static inline uint16_t get_u16(const uint8_t *p) { return (uint16_t)(p[0] | ((uint16_t)p[1] << 8)); }

/* ------------------------------------------------------------------------- */
/* Quantisers.  `x` points at the block's first element, `len` <= block size  */
/* is the number of real elements (the tail block is shorter).                */
/* ------------------------------------------------------------------------- */

/* quantize.rs:82-114 + types.rs:142-147 */
static void quant_block_q8_0(const float *x, size_t len, uint8_t *out) {
    float max_abs = 0.0f;
    for (size_t i = 0; i < len; i++) max_abs = rs_max(max_abs, fabsf(x[i]));
    float scale = max_abs > 0.0f ? max_abs / 127.0f : 1.0f;
    int8_t q[32];
    memset(q, 0, sizeof q);
    for (size_t i = 0; i < len; i++) q[i] = (int8_t)rs_round_clamp(x[i] / scale, -127.0f, 127.0f);
    put_u16(out, axo_f32_to_f16(scale));
    for (int i = 0; i < 32; i++) out[2 + i] = (uint8_t)q[i];
}

/* quantize.rs:121-156 + types.rs:190-206 (adjacent-pair nibble order) */
static void quant_block_q4_0(const float *x, size_t len, uint8_t *out) {
    float max_abs = 0.0f;
    for (size_t i = 0; i < len; i++) max_abs = rs_max(max_abs, fabsf(x[i]));
    float scale = max_abs > 0.0f ? max_abs / 7.0f : 1.0f;
    int8_t q[32];
    memset(q, 0, sizeof q);
    for (size_t i = 0; i < len; i++) q[i] = (int8_t)rs_round_clamp(x[i] / scale, -8.0f, 7.0f);
    put_u16(out, axo_f32_to_f16(scale));
    for (int i = 0; i < 16; i++) {
        uint8_t low = (uint8_t)(q[2 * i] + 8) & 0x0F;
        uint8_t high = (uint8_t)(q[2 * i + 1] + 8) & 0x0F;
        out[2 + i] = (uint8_t)(low | (high << 4));
    }
}

/* quantize.rs:163-205 + types.rs:249-255.  The pack loop runs over
 * min(16, len/2) bytes, so a tail block of odd length drops its last code. */
static void quant_block_q4_1(const float *x, size_t len, uint8_t *out) {
    float mn = INFINITY, mx = -INFINITY;
    for (size_t i = 0; i < len; i++) mn = rs_min(mn, x[i]);
    for (size_t i = 0; i < len; i++) mx = rs_max(mx, x[i]);
    float scale = mx > mn ? (mx - mn) / 15.0f : 1.0f;
    uint8_t q[32];
    memset(q, 0, sizeof q);
    for (size_t i = 0; i < len; i++) q[i] = (uint8_t)rs_round_clamp((x[i] - mn) / scale, 0.0f, 15.0f);
    put_u16(out, axo_f32_to_f16(scale));
    put_u16(out + 2, axo_f32_to_f16(mn));
    memset(out + 4, 0, 16);
    size_t nb = len / 2 < 16 ? len / 2 : 16;
    for (size_t i = 0; i < nb; i++) out[4 + i] = (uint8_t)((q[2 * i] & 0x0F) | ((q[2 * i + 1] & 0x0F) << 4));
}

/* Q5_0, GGUF layout [f16 d][u8 qh[4]][u8 qs[16]]: element j (<16) has its low
 * nibble in qs[j]&0xF and bit 4 in qh bit j; element j+16 has qs[j]>>4 and qh
 * bit j+16.  Quantiser rule (this build's, in the style of quantize.rs:139):
 * scale = max_abs/15 (1.0 for a zero block), q = round(x/scale) in [-16,15],
 * stored code = q + 16. */
static void quant_block_q5_0(const float *x, size_t len, uint8_t *out) {
    float max_abs = 0.0f;
    for (size_t i = 0; i < len; i++) max_abs = rs_max(max_abs, fabsf(x[i]));
    float scale = max_abs > 0.0f ? max_abs / 15.0f : 1.0f;
    uint8_t u[32];
    for (int i = 0; i < 32; i++) u[i] = 16; /* q = 0 */
    for (size_t i = 0; i < len; i++) u[i] = (uint8_t)(rs_round_clamp(x[i] / scale, -16.0f, 15.0f) + 16);
    uint32_t qh = 0;
    put_u16(out, axo_f32_to_f16(scale));
    for (int j = 0; j < 16; j++) {
        out[6 + j] = (uint8_t)((u[j] & 0x0F) | ((u[j + 16] & 0x0F) << 4));
        qh |= (uint32_t)((u[j] >> 4) & 1) << j;
        qh |= (uint32_t)((u[j + 16] >> 4) & 1) << (j + 16);
    }
    out[2] = (uint8_t)qh; out[3] = (uint8_t)(qh >> 8); out[4] = (uint8_t)(qh >> 16); out[5] = (uint8_t)(qh >> 24);
}

/* Q5_1, GGUF layout [f16 d][f16 m][u8 qh[4]][u8 qs[16]].  Quantiser rule (this
 * build's, in the style of quantize.rs:175-184): scale = (max-min)/31 (1.0 if
 * max<=min), code = round((x-min)/scale) in [0,31]. */
static void quant_block_q5_1(const float *x, size_t len, uint8_t *out) {
    float mn = INFINITY, mx = -INFINITY;
    for (size_t i = 0; i < len; i++) mn = rs_min(mn, x[i]);
    for (size_t i = 0; i < len; i++) mx = rs_max(mx, x[i]);
    float scale = mx > mn ? (mx - mn) / 31.0f : 1.0f;
    uint8_t u[32];
    memset(u, 0, sizeof u);
    for (size_t i = 0; i < len; i++) u[i] = (uint8_t)rs_round_clamp((x[i] - mn) / scale, 0.0f, 31.0f);
    uint32_t qh = 0;
    put_u16(out, axo_f32_to_f16(scale));
    put_u16(out + 2, axo_f32_to_f16(mn));
    for (int j = 0; j < 16; j++) {
        out[8 + j] = (uint8_t)((u[j] & 0x0F) | ((u[j + 16] & 0x0F) << 4));
        qh |= (uint32_t)((u[j] >> 4) & 1) << j;
        qh |= (uint32_t)((u[j + 16] >> 4) & 1) << (j + 16);
    }
    out[4] = (uint8_t)qh; out[5] = (uint8_t)(qh >> 8); out[6] = (uint8_t)(qh >> 16); out[7] = (uint8_t)(qh >> 24);
}

/* Q4_K, GGUF layout [f16 d][f16 dmin][u8 scales[12]][u8 qs[128]] over 256
 * elements = 8 sub-blocks of 32.  scales[] packs eight 6-bit scales and eight
 * 6-bit mins (ggml's get_scale_min_k4 order).  qs: for pair p in 0..3, bytes
 * qs[32p..32p+31] hold sub-block 2p in the low nibbles and 2p+1 in the high.
 * Dequant: w = (d*sc_s)*q - (dmin*m_s).
 *
 * Quantiser rule (this build's; ggml's iterative search is not restated):
 *   per sub-block: mn = min(0, min x), mx = max x; scale_s = (mx-mn)/15,
 *   min_s = -mn;  max_scale = max scale_s, max_min = max min_s;
 *   ls_s = min(63, round(63/max_scale * scale_s)), lm_s likewise (0 if the
 *   maximum is 0);  d = f16(max_scale/63), dmin = f16(max_min/63);
 *   with the f16-rounded d,dmin:  sd = d*ls_s, sm = dmin*lm_s,
 *   q = clamp(round((x + sm)/sd), 0, 15)  (0 when sd == 0).
 * A short tail superblock is zero-padded before quantisation. */
static void quant_block_qk(const float *xin, size_t len, uint8_t *out, int bits);
static void quant_block_q4_k(const float *xin, size_t len, uint8_t *out) { quant_block_qk(xin, len, out, 4); }

/* Q5_K, GGUF layout [f16 d][f16 dmin][u8 scales[12]][u8 qh[32]][u8 qs[128]] (176 bytes): header and qs as Q4_K's, with
 * the low four bits of the 5-bit codes in qs; the fifth bit of element 64 p + 32 h + l (pair p, half h) is bit 2 p + h of
 * qh[l].  Dequant: w = (d*sc_s)*q - (dmin*m_s), q in 0..31.  Quantiser rule: Q4_K's with 31 steps instead of 15. */
static void quant_block_q5_k(const float *xin, size_t len, uint8_t *out) { quant_block_qk(xin, len, out, 5); }

static void quant_block_qk(const float *xin, size_t len, uint8_t *out, int bits) {
    const float top = bits == 5 ? 31.0f : 15.0f;
    float x[256];
    memset(x, 0, sizeof x);
    memcpy(x, xin, len * sizeof(float));
    float scales[8], mins[8];
    float max_scale = 0.0f, max_min = 0.0f;
    for (int s = 0; s < 8; s++) {
        float mn = INFINITY, mx = -INFINITY;
        for (int i = 0; i < 32; i++) mn = rs_min(mn, x[32 * s + i]);
        for (int i = 0; i < 32; i++) mx = rs_max(mx, x[32 * s + i]);
        if (mn > 0.0f) mn = 0.0f;
        if (!(mx > mn)) { /* constant (or all-NaN) sub-block */
            scales[s] = 0.0f;
            mins[s] = isfinite(mn) ? -mn : 0.0f;
        } else {
            scales[s] = (mx - mn) / top;
            mins[s] = -mn;
        }
        max_scale = rs_max(max_scale, scales[s]);
        max_min = rs_max(max_min, mins[s]);
    }
    float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    uint8_t ls[8], lm[8];
    for (int s = 0; s < 8; s++) {
        ls[s] = (uint8_t)rs_round_clamp(inv_scale * scales[s], 0.0f, 63.0f);
        lm[s] = (uint8_t)rs_round_clamp(inv_min * mins[s], 0.0f, 63.0f);
    }
    uint16_t dh = axo_f32_to_f16(max_scale / 63.0f);
    uint16_t dminh = axo_f32_to_f16(max_min / 63.0f);
    put_u16(out, dh);
    put_u16(out + 2, dminh);
    uint8_t *sc = out + 4;
    for (int j = 0; j < 4; j++) {
        sc[j] = (uint8_t)(ls[j] | ((ls[j + 4] >> 4) << 6));
        sc[j + 4] = (uint8_t)(lm[j] | ((lm[j + 4] >> 4) << 6));
        sc[j + 8] = (uint8_t)((ls[j + 4] & 0x0F) | ((lm[j + 4] & 0x0F) << 4));
    }
    float d = axo_f16_to_f32(dh), dmin = axo_f16_to_f32(dminh);
    uint8_t q[256];
    for (int s = 0; s < 8; s++) {
        float sd = d * (float)ls[s];
        float sm = dmin * (float)lm[s];
        for (int i = 0; i < 32; i++) {
            if (sd == 0.0f) {
                q[32 * s + i] = 0;
            } else {
                q[32 * s + i] = (uint8_t)rs_round_clamp((x[32 * s + i] + sm) / sd, 0.0f, top);
            }
        }
    }
    uint8_t *qs = out + 16;
    if (bits == 5) {
        uint8_t *qh = out + 16;
        qs = out + 48;
        memset(qh, 0, 32);
        for (int p = 0; p < 4; p++)
            for (int h = 0; h < 2; h++)
                for (int l = 0; l < 32; l++) qh[l] |= (uint8_t)((q[64 * p + 32 * h + l] >> 4) << (2 * p + h));
    }
    for (int p = 0; p < 4; p++)
        for (int l = 0; l < 32; l++) qs[32 * p + l] = (uint8_t)((q[64 * p + l] & 0x0F) | ((q[64 * p + 32 + l] & 0x0F) << 4));
}

/* Q6_K, GGUF layout [u8 ql[128]][u8 qh[64]][i8 scales[16]][f16 d] over 256 elements = 16 sub-blocks of 16, each
 * with a signed 8-bit scale.  Element e = 128 n + 32 c + l (n = 0, 1; c = 0..3; l = 0..31) has the 6-bit code
 * u = q + 32 with its low four bits in ql[64 n + 32 (c & 1) + l] (low nibble for c < 2, high for c >= 2) and its
 * upper two bits in qh[32 n + l] at bit 2 c; its scale is scales[e / 16].  Dequant: w = (d * scale) * q.
 *
 * Quantiser rule (this build's; ggml's make_qx_quants search is not restated): per sub-block a_s = max |x|,
 * scale_s = a_s / 31; max_scale = max scale_s; ls_s = round(127 / max_scale * scale_s) in 0..127 (0 if the
 * maximum is 0); d = f16(max_scale / 127); with the f16-rounded d: sd = d * ls_s,
 * q = clamp(round(x / sd), -32, 31)  (0 when sd == 0).  A short tail superblock is zero-padded. */
static void quant_block_q6_k(const float *xin, size_t len, uint8_t *out) {
    float x[256];
    memset(x, 0, sizeof x);
    memcpy(x, xin, len * sizeof(float));
    float scales[16], max_scale = 0.0f;
    for (int s = 0; s < 16; s++) {
        float a = 0.0f;
        for (int i = 0; i < 16; i++) a = rs_max(a, fabsf(x[16 * s + i]));
        scales[s] = a / 31.0f;
        max_scale = rs_max(max_scale, scales[s]);
    }
    float inv = max_scale > 0.0f ? 127.0f / max_scale : 0.0f;
    uint16_t dh = axo_f32_to_f16(max_scale / 127.0f);
    float d = axo_f16_to_f32(dh);
    uint8_t *ql = out, *qh = out + 128;
    int8_t *sc = (int8_t *)(out + 192);
    memset(out, 0, 192);
    for (int s = 0; s < 16; s++) {
        int ls = rs_round_clamp(inv * scales[s], 0.0f, 127.0f);
        sc[s] = (int8_t)ls;
        float sd = d * (float)ls;
        for (int i = 0; i < 16; i++) {
            int e = 16 * s + i;
            int q = sd == 0.0f ? 0 : rs_round_clamp(x[e] / sd, -32.0f, 31.0f);
            unsigned u = (unsigned)(q + 32);
            int n = e >> 7, c = (e >> 5) & 3, l = e & 31;
            ql[64 * n + 32 * (c & 1) + l] |= (uint8_t)((u & 0x0F) << (4 * (c >> 1)));
            qh[32 * n + l] |= (uint8_t)((u >> 4) << (2 * c));
        }
    }
    put_u16(out + 208, dh);
}

/* quantize_tensor (quantize.rs:36-54): flat row-major f32 -> concatenated
 * `to_bytes` images in block order.  Unlike the reference, Q5_0/Q5_1 get
 * real codecs instead of aliasing Q4_0.  Returns 0, or -2 for an unknown type. */
AXO_API int axo_quantize(int type, const float *x, size_t numel, uint8_t *out) {
    size_t bs = axo_block_size(type), bb = axo_bytes_per_block(type);
    if (bs == 0) return -2;
    if (type == AXO_F32) { /* quantize.rs:225-228 */
        memcpy(out, x, numel * 4);
        return 0;
    }
    if (type == AXO_F16) { /* quantize.rs:212-218 */
#pragma omp parallel for schedule(static)
        for (long long i = 0; i < (long long)numel; i++) put_u16(out + 2 * i, axo_f32_to_f16(x[i]));
        return 0;
    }
    long long nb = (long long)((numel + bs - 1) / bs);
#pragma omp parallel for schedule(static)
    for (long long b = 0; b < nb; b++) {
        size_t start = (size_t)b * bs;
        size_t len = numel - start < bs ? numel - start : bs;
        uint8_t *o = out + (size_t)b * bb;
        switch (type) {
        case AXO_Q8_0: quant_block_q8_0(x + start, len, o); break;
        case AXO_Q4_0: quant_block_q4_0(x + start, len, o); break;
        case AXO_Q4_1: quant_block_q4_1(x + start, len, o); break;
        case AXO_Q5_0: quant_block_q5_0(x + start, len, o); break;
        case AXO_Q5_1: quant_block_q5_1(x + start, len, o); break;
        case AXO_Q4_K: quant_block_q4_k(x + start, len, o); break;
        case AXO_Q5_K: quant_block_q5_k(x + start, len, o); break;
        case AXO_Q6_K: quant_block_q6_k(x + start, len, o); break;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* Dequantisers (one block -> bs floats)                                      */
/* ------------------------------------------------------------------------- */

static void dequant_block(int type, const uint8_t *b, float *y) {
    switch (type) {
    case AXO_Q8_0: { /* dequantize.rs:89-92 */
        float scale = axo_f16_to_f32(get_u16(b));
        for (int i = 0; i < 32; i++) y[i] = (float)(int8_t)b[2 + i] * scale;
        break;
    }
    case AXO_Q4_0: { /* dequantize.rs:116-121 + types.rs:179-187 */
        float scale = axo_f16_to_f32(get_u16(b));
        for (int i = 0; i < 16; i++) {
            uint8_t byte = b[2 + i];
            y[2 * i] = (float)((int)(byte & 0x0F) - 8) * scale;
            y[2 * i + 1] = (float)((int)(byte >> 4) - 8) * scale;
        }
        break;
    }
    case AXO_Q4_1: { /* dequantize.rs:145-151: multiply, then add (two roundings) */
        float scale = axo_f16_to_f32(get_u16(b));
        float mn = axo_f16_to_f32(get_u16(b + 2));
        for (int i = 0; i < 16; i++) {
            uint8_t byte = b[4 + i];
            float a = (float)(byte & 0x0F) * scale;
            float c = (float)(byte >> 4) * scale;
            y[2 * i] = a + mn;
            y[2 * i + 1] = c + mn;
        }
        break;
    }
    case AXO_Q5_0: {
        float d = axo_f16_to_f32(get_u16(b));
        uint32_t qh = (uint32_t)b[2] | ((uint32_t)b[3] << 8) | ((uint32_t)b[4] << 16) | ((uint32_t)b[5] << 24);
        for (int j = 0; j < 16; j++) {
            int u0 = (b[6 + j] & 0x0F) | (int)(((qh >> j) & 1u) << 4);
            int u1 = (b[6 + j] >> 4) | (int)(((qh >> (j + 16)) & 1u) << 4);
            y[j] = (float)(u0 - 16) * d;
            y[j + 16] = (float)(u1 - 16) * d;
        }
        break;
    }
    case AXO_Q5_1: {
        float d = axo_f16_to_f32(get_u16(b));
        float m = axo_f16_to_f32(get_u16(b + 2));
        uint32_t qh = (uint32_t)b[4] | ((uint32_t)b[5] << 8) | ((uint32_t)b[6] << 16) | ((uint32_t)b[7] << 24);
        for (int j = 0; j < 16; j++) {
            int u0 = (b[8 + j] & 0x0F) | (int)(((qh >> j) & 1u) << 4);
            int u1 = (b[8 + j] >> 4) | (int)(((qh >> (j + 16)) & 1u) << 4);
            float a = (float)u0 * d;
            float c = (float)u1 * d;
            y[j] = a + m;
            y[j + 16] = c + m;
        }
        break;
    }
    case AXO_Q4_K:
    case AXO_Q5_K: { /* ggml's dequantize_row_q4_K / _q5_K: y = (d * sc) * q - dmin * m */
        float d = axo_f16_to_f32(get_u16(b));
        float dmin = axo_f16_to_f32(get_u16(b + 2));
        const uint8_t *sc = b + 4;
        const uint8_t *qh = b + 16; /* Q5_K only */
        const uint8_t *qs = type == AXO_Q5_K ? b + 48 : b + 16;
        for (int s = 0; s < 8; s++) {
            uint8_t l, m;
            if (s < 4) {
                l = sc[s] & 63;
                m = sc[s + 4] & 63;
            } else {
                l = (uint8_t)((sc[s + 4] & 0x0F) | ((sc[s - 4] >> 6) << 4));
                m = (uint8_t)((sc[s + 4] >> 4) | ((sc[s] >> 6) << 4));
            }
            float sd = d * (float)l;
            float sm = dmin * (float)m;
            int p = s >> 1;
            for (int i = 0; i < 32; i++) {
                uint8_t byte = qs[32 * p + i];
                int q = (s & 1) ? (byte >> 4) : (byte & 0x0F);
                if (type == AXO_Q5_K) q |= ((qh[i] >> s) & 1) << 4;
                float a = sd * (float)q;
                y[32 * s + i] = a - sm;
            }
        }
        break;
    }
    case AXO_Q6_K: { /* ggml's dequantize_row_q6_K: y = d * scale * q, the product d * scale taken first */
        const uint8_t *ql = b, *qh = b + 128;
        const int8_t *sc = (const int8_t *)(b + 192);
        float d = axo_f16_to_f32(get_u16(b + 208));
        for (int e = 0; e < 256; e++) {
            int n = e >> 7, c = (e >> 5) & 3, l = e & 31;
            int lo = (ql[64 * n + 32 * (c & 1) + l] >> (4 * (c >> 1))) & 0x0F;
            int hi = (qh[32 * n + l] >> (2 * c)) & 3;
            int q = (lo | (hi << 4)) - 32;
            float ds = d * (float)sc[e >> 4];
            y[e] = ds * (float)q;
        }
        break;
    }
    }
}

/* dequantize_tensor (dequantize.rs:34-54): all blocks, truncated to numel. */
AXO_API int axo_dequantize(int type, const uint8_t *packed, size_t numel, float *out) {
    size_t bs = axo_block_size(type), bb = axo_bytes_per_block(type);
    if (bs == 0) return -2;
    if (type == AXO_F32) {
        memcpy(out, packed, numel * 4);
        return 0;
    }
    if (type == AXO_F16) {
#pragma omp parallel for schedule(static)
        for (long long i = 0; i < (long long)numel; i++) out[i] = axo_f16_to_f32(get_u16(packed + 2 * i));
        return 0;
    }
    long long nb = (long long)((numel + bs - 1) / bs);
#pragma omp parallel for schedule(static)
    for (long long b = 0; b < nb; b++) {
        size_t start = (size_t)b * bs;
        size_t len = numel - start < bs ? numel - start : bs;
        float tmp[256];
        if (len == bs) {
            dequant_block(type, packed + (size_t)b * bb, out + start);
        } else {
            dequant_block(type, packed + (size_t)b * bb, tmp);
            memcpy(out + start, tmp, len * sizeof(float));
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* Matmul: y[M,N] = x[M,K] * W[N,K]^T (+ bias[N])                             */
/* ------------------------------------------------------------------------- */

/* Single-threaded row-major sgemm C[m,n] = A[m,k] * B[k,n], f32 accumulate, in
 * the role of matrixmultiply::sgemm (cpu.rs:580-597; built without its
 * `threading` feature, so one thread).  k is blocked so that a strip of B stays
 * in cache; within a block the i-k-j order lets gcc vectorise over j. */
static void sgemm_rowmajor(float *c, const float *a, const float *b, size_t m, size_t n, size_t k) {
    memset(c, 0, m * n * sizeof(float));
    const size_t KB = 256, JB = 2048;
    for (size_t j0 = 0; j0 < n; j0 += JB) {
        size_t j1 = j0 + JB < n ? j0 + JB : n;
        for (size_t p0 = 0; p0 < k; p0 += KB) {
            size_t p1 = p0 + KB < k ? p0 + KB : k;
            for (size_t i = 0; i < m; i++) {
                float *ci = c + i * n;
                for (size_t p = p0; p < p1; p++) {
                    float av = a[i * k + p];
                    const float *bp = b + p * n;
                    for (size_t j = j0; j < j1; j++) ci[j] += av * bp[j];
                }
            }
        }
    }
}

/* The reference composition, timed as a whole by the benchmark's cpu_baseline:
 *   w  = dequantize_tensor(wq)            (block-parallel, dequantize.rs:34-54)
 *   wt = w.t().contiguous()               (tensor.rs:1041, a strided gather)
 *   y  = sgemm(x, wt)                     (cpu.rs:566-598, one thread)
 *   y += bias                             (linear.rs:126-129)
 * `scratch` must hold 2*N*K floats.  Returns 0 on success. */
AXO_API int axo_matmul_ref(int type, const uint8_t *wq, const float *x, const float *bias, size_t M, size_t N, size_t K,
                           float *y, float *scratch) {
    float *w = scratch, *wt = scratch + N * K;
    int rc = axo_dequantize(type, wq, N * K, w);
    if (rc) return rc;
#pragma omp parallel for schedule(static)
    for (long long kk = 0; kk < (long long)K; kk++)
        for (size_t nn = 0; nn < N; nn++) wt[(size_t)kk * N + nn] = w[nn * K + (size_t)kk];
    sgemm_rowmajor(y, x, wt, M, N, K);
    if (bias)
        for (size_t i = 0; i < M; i++)
            for (size_t j = 0; j < N; j++) y[i * N + j] = y[i * N + j] + bias[j];
    return 0;
}

/* Same product from already-dequantised weights W[N,K] (f32), accumulating in
 * f64: the error-budget reference for the tolerance tests. */
AXO_API void axo_matmul_f64(const float *w, const float *x, const float *bias, size_t M, size_t N, size_t K, double *y) {
#pragma omp parallel for schedule(static)
    for (long long j = 0; j < (long long)N; j++) {
        const float *wr = w + (size_t)j * K;
        for (size_t i = 0; i < M; i++) {
            const float *xr = x + i * K;
            double acc = 0.0;
            for (size_t p = 0; p < K; p++) acc += (double)xr[p] * (double)wr[p];
            if (bias) acc += (double)bias[j];
            y[i * N + (size_t)j] = acc;
        }
    }
}

/* Steady-state variant for the benchmark: weights already dequantised and
 * transposed once (wt[K,N]); one sgemm per call, single thread. */
AXO_API void axo_sgemm_wt(const float *x, const float *wt, size_t M, size_t N, size_t K, float *y) {
    sgemm_rowmajor(y, x, wt, M, N, K);
}

/* bf16 helpers for the prefill inputs (activations are bf16, widened exactly). */
AXO_API uint16_t axo_f32_to_bf16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x0040u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7FFFu + lsb;
    return (uint16_t)(x >> 16);
}
AXO_API float axo_bf16_to_f32(uint16_t h) {
    uint32_t x = (uint32_t)h << 16;
    float f;
    memcpy(&f, &x, 4);
    return f;
}

AXO_API int axo_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
