/*
 * CPU oracle for GGUF interop.  TEST INFRASTRUCTURE ONLY (see axq_oracle.c).
 *
 * The reference has no GGUF code: `.gguf` appears only as an accepted file
 * extension (crates/axonml-cli/src/commands/quant.rs:218).  The algorithm here
 * is the GGUF / ggml specification (ggml `block_q4_0`, `block_q4_1`,
 * `dequantize_row_q4_0`, `dequantize_row_q4_1`; third party, not in the
 * reference tree), restated, next to the reference's own nibble order:
 *
 *   ggml      : qs[j] = element j | element (j + 16) << 4
 *   reference : data[i] = element 2i | element (2i + 1) << 4
 *               (Q4Block::pack / unpack, crates/axonml-quant/src/types.rs:179-198)
 *
 * Pin status: axo_gguf_convert is pinned by hand-written blocks and, through
 * two independently stated element formulas, by
 *   axo_dequantize(reference order, dequantize.rs:116-121,145-151) o convert
 *     == axo_ggml_dequantize(ggml order)
 * on random blocks, and by convert o convert^-1 == identity (tests/test_gguf.py).
 */
#include <stdint.h>
#include <string.h>

#define AXO_API __attribute__((visibility("default")))

float axo_f16_to_f32(uint16_t h);

enum { T_Q4_0 = 1, T_Q4_1 = 2 };

/* nblocks block images; to_gguf = 0: ggml order -> reference order, 1: back.  Other types: plain copy. */
AXO_API int axo_gguf_convert(int type, const uint8_t *src, uint8_t *dst, size_t nblocks, size_t block_bytes, int to_gguf) {
    if (type != T_Q4_0 && type != T_Q4_1) {
        memmove(dst, src, nblocks * block_bytes);
        return 0;
    }
    const size_t hdr = type == T_Q4_0 ? 2 : 4;
    if (block_bytes != hdr + 16) return -1;
    for (size_t b = 0; b < nblocks; b++) {
        const uint8_t *s = src + b * block_bytes;
        uint8_t *d = dst + b * block_bytes;
        uint8_t e[32], out[16];
        if (!to_gguf) {
            for (int j = 0; j < 16; j++) { e[j] = s[hdr + j] & 0x0F; e[j + 16] = s[hdr + j] >> 4; }
            for (int i = 0; i < 16; i++) out[i] = (uint8_t)(e[2 * i] | (e[2 * i + 1] << 4));
        } else {
            for (int i = 0; i < 16; i++) { e[2 * i] = s[hdr + i] & 0x0F; e[2 * i + 1] = s[hdr + i] >> 4; }
            for (int j = 0; j < 16; j++) out[j] = (uint8_t)(e[j] | (e[j + 16] << 4));
        }
        memmove(d, s, hdr);
        memcpy(d + hdr, out, 16);
    }
    return 0;
}

/* ggml's dequantize_row_q4_0 / dequantize_row_q4_1 on blocks in ggml order. */
AXO_API int axo_ggml_dequantize(int type, const uint8_t *blocks, size_t nblocks, float *dst) {
    if (type != T_Q4_0 && type != T_Q4_1) return -1;
    const size_t hdr = type == T_Q4_0 ? 2 : 4, bb = hdr + 16;
    for (size_t b = 0; b < nblocks; b++) {
        const uint8_t *s = blocks + b * bb;
        uint16_t dh, mh = 0;
        memcpy(&dh, s, 2);
        if (type == T_Q4_1) memcpy(&mh, s + 2, 2);
        const float d = axo_f16_to_f32(dh), m = axo_f16_to_f32(mh);
        for (int j = 0; j < 16; j++) {
            const int x0 = s[hdr + j] & 0x0F, x1 = s[hdr + j] >> 4;
            if (type == T_Q4_0) {
                dst[b * 32 + j] = (float)(x0 - 8) * d;
                dst[b * 32 + j + 16] = (float)(x1 - 8) * d;
            } else {
                dst[b * 32 + j] = (float)x0 * d + m;
                dst[b * 32 + j + 16] = (float)x1 * d + m;
            }
        }
    }
    return 0;
}
