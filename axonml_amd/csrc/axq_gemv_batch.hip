// Decode-path quantized matmul for a small batch (2..8 activation vectors): y[b, n] = sum_k x[b, k] W[n, k].
//
// The weights are read once for the whole batch.  The dot products run on v_mfma_i32_32x32x32_i8 with
//   A (32 x 32): row 4 b + l = limb l of activation vector b (the split form of axq_split.h), 32 k of one block,
//   B (32 x 32): column n = one of 32 weight rows, the block's 32 codes as signed bytes, centred (a 4-bit code q goes in
//                as 16 (q - 8): its nibble moved to the top of the byte with the top bit flipped; a 5-bit one as 8 (q - 16)),
// so one instruction multiplies a 32-element block of 32 weight rows with all vectors and limbs.  Lane
// (n, h) = (lane % 32, lane / 32) supplies 16 of the block's codes of row n and receives D[4 b + l][n] for
// b = h, h + 2, h + 4, h + 6: all four limbs of four vectors, which it recombines and scales by itself.
//
// A workgroup owns 32 weight rows; its up to 8 waves take the row's chunks of 16 blocks (512 weights) in turn,
// the A operands of a chunk in registers; the partial sums of the waves meet in LDS and are added in a fixed
// order.  K is a multiple of 256, so a row's last chunk holds 16 or 8 blocks.  The split form of
// the batch is made once, by a small kernel in front (a workgroup could not afford to split eight vectors
// for its 32 rows).
#include <hip/hip_fp16.h>

#include <stdlib.h>

#include <mutex>

#include "axq_internal.h"
#include "axq_split.h"

namespace {

typedef int int4v __attribute__((ext_vector_type(4)));
typedef int int16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int UNITS = 8;       // 32-element blocks per wave and chunk
constexpr int WAVE_K = 32 * UNITS;
constexpr int MAX_BATCH = 8;

struct MbArgs {
    const uint8_t *codes, *meta, *qh;
    size_t codes_pitch, meta_pitch, qh_pitch;
    const uint8_t *xa;  // the batch's limbs as MFMA A operands: [block][h][row 4 b + l] x 16 bytes (pack_x_kernel)
    const float *xsg;   // [block][h][4]: group scales of vectors h, h + 2, h + 4, h + 6; then the plain sums, same layout
    const float *bias;
    const float *resid; // [batch, n_rows] added to y (may be y itself), or null
    float *y;
    float *ypart; // K split over several workgroups: [split][batch][n_rows] partial sums, added by mb_reduce_kernel
    int n_rows, k, batch;
    int chunks_per_split; // chunks of a row that one workgroup (blockIdx.y) takes
};

__device__ inline float f16lo(uint32_t v) { return __half2float(__ushort_as_half((unsigned short)(v & 0xFFFF))); }
__device__ inline float f16hi(uint32_t v) { return __half2float(__ushort_as_half((unsigned short)(v >> 16))); }
__device__ inline u32x4 ldg16(const uint8_t *p) { return *reinterpret_cast<const u32x4 *>(p); }

// sum_k n_k x_k over one 32-element block of one vector from its four limb sums (limb 0 most significant)
__device__ inline float recombine4(int d0, int d1, int d2, int d3) {
    // |d_i| <= 32 * 127 * 64 < 2^18: two limbs combine exactly in an integer (< 2^25 ... the f32 of it rounds like the fma chain would)
    return fmaf((float)(d0 * 128 + d1), 16384.0f, (float)(d2 * 128 + d3));
}

// ---------------------------------------------------------------------------
// Per-type traits.  `u` counts the wave's blocks 0..15, `blk0` is the wave's first block in the row,
// h = lane / 32 says which 16 of a block's 32 codes the lane supplies.
//   EVEN_ODD : h = 0 supplies the even elements, h = 1 the odd ones (reference nibble order); otherwise
//              h = 0 supplies elements 0..15, h = 1 elements 16..31
//   coef()   : w = d * operand + mo with the operand the centred code times 16 (or 8), so d is the block's scale over
//              16 (8) and mo the weight of the middle code (nothing for Q4_0, Q5_0).  Centred because the integer sums
//              are exact but their f32 images are not: with codes 0..15 the sum over the codes and the offset term
//              are each a block's range times sum x, and for an activation with a mean their roundings, 2^-24 of that,
//              showed in the small outputs (4-8e-4 at the strict floor of the parity test; centred 1e-4)
// ---------------------------------------------------------------------------
template <bool WITH_MIN>
struct MQ4x {
    static constexpr int NP2 = 0; // no second plane
    static constexpr bool RUNS16 = false;
    static constexpr bool EVEN_ODD = true;
    static constexpr bool OFFSET = WITH_MIN; // w = d (q - 8) + mo with mo = min + 8 d (Q4_1) or nothing (Q4_0)
    static constexpr int NV = UNITS * (WITH_MIN ? 4 : 2) / 16 > 0 ? UNITS * (WITH_MIN ? 4 : 2) / 16 : 1; // 16-byte vectors of scales per chunk
    struct Raw { u32x4 q[UNITS]; u32x4 m[NV]; };
    // the chunk's codes of one row: NP 16-byte pieces, piece p = block blk0 + p; a lane wants piece u for block u
    static constexpr int NP = UNITS, NQ = UNITS;
    __device__ static size_t piece_off(const MbArgs &, int blk0, int p) { return (size_t)(blk0 + p) * 16; }
    __device__ static int want(int j, int) { return j; }
    __device__ static void load_meta(const MbArgs &a, size_t row, int blk0, int nblk, Raw &r) {
        const uint8_t *meta = a.meta + row * a.meta_pitch;
        constexpr int PER = WITH_MIN ? 4 : 8; // blocks per 16-byte vector of scales
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int v = blk0 / PER + i < nblk / PER ? blk0 / PER + i : nblk / PER - 1;
            r.m[i] = ldg16(meta + (size_t)v * 16);
        }
    }
    __device__ static int4v operand(const Raw &r, int u, int h) {
        const int sh = 4 - 4 * h;
        int4v b;
#pragma unroll
        for (int i = 0; i < 4; i++) b[i] = (int)(((r.q[u][i] << sh) & 0xF0F0F0F0u) ^ 0x80808080u); // 16 (q - 8)
        return b;
    }
    __device__ static void coef(const Raw &r, int u, float &d, float &mo) {
        if (WITH_MIN) {
            const uint32_t v = r.m[u >> 2][u & 3];
            const float dd = f16lo(v);
            d = dd * 0.0625f;
            mo = fmaf(8.0f, dd, f16hi(v));
        } else {
            const uint32_t v = r.m[u >> 3][(u >> 1) & 3];
            d = ((u & 1) ? f16hi(v) : f16lo(v)) * 0.0625f;
            mo = 0.f;
        }
    }
};

struct MQ80 {
    static constexpr int NP2 = 0; // no second plane
    static constexpr bool RUNS16 = false;
    static constexpr bool EVEN_ODD = false;
    static constexpr bool OFFSET = false;
    static constexpr int NV = UNITS / 8 > 0 ? UNITS / 8 : 1;
    struct Raw { u32x4 q[UNITS]; u32x4 m[NV]; };
    // 32 code bytes per block: piece 2u + h = the h-th half of block blk0 + u
    static constexpr int NP = 2 * UNITS, NQ = UNITS;
    __device__ static size_t piece_off(const MbArgs &, int blk0, int p) { return (size_t)blk0 * 32 + (size_t)p * 16; }
    __device__ static int want(int j, int h) { return 2 * j + h; }
    __device__ static void load_meta(const MbArgs &a, size_t row, int blk0, int nblk, Raw &r) {
        const uint8_t *meta = a.meta + row * a.meta_pitch;
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int v = blk0 / 8 + i < nblk / 8 ? blk0 / 8 + i : nblk / 8 - 1;
            r.m[i] = ldg16(meta + (size_t)v * 16);
        }
    }
    __device__ static int4v operand(const Raw &r, int u, int) {
        int4v b = {(int)r.q[u][0], (int)r.q[u][1], (int)r.q[u][2], (int)r.q[u][3]};
        return b;
    }
    __device__ static void coef(const Raw &r, int u, float &d, float &mo) {
        const uint32_t v = r.m[u >> 3][(u >> 1) & 3];
        d = (u & 1) ? f16hi(v) : f16lo(v);
        mo = 0.f;
    }
};

// Q4_K: a block is a sub-block; the lane's 16-byte piece of pair p (first half for h = 0, second for h = 1)
// holds its codes of sub-block 2p in the low nibbles and of sub-block 2p + 1 in the high ones.
struct MQ4K {
    static constexpr int NP2 = 0; // no second plane
    static constexpr bool RUNS16 = false;
    static constexpr bool EVEN_ODD = false;
    static constexpr bool OFFSET = true;
    struct Raw { u32x4 q[UNITS / 2]; u32x4 h[UNITS / 8]; };
    // a chunk is one superblock = 4 pairs: pieces 0..3 = the first 16 bytes of its pairs, 4..7 = their second 16 bytes
    static_assert(UNITS == 8, "one superblock per chunk");
    static constexpr int NP = 8, NQ = 4;
    __device__ static size_t piece_off(const MbArgs &a, int blk0, int p) {
        const int cpr = a.k >> 6;          // pairs per row
        const int pair0 = blk0 >> 1;       // the chunk's first pair; its 4 pairs lie inside one 64-pair slice
        const int slice = pair0 >> 6, pr = pair0 & 63;
        int P = cpr - (slice << 6);
        P = P < 64 ? P : 64;
        return (size_t)slice * 2048 + (size_t)(p >> 2) * 16 * P + (size_t)(pr + (p & 3)) * 16;
    }
    __device__ static int want(int j, int h) { return 4 * h + j; }
    __device__ static void load_meta(const MbArgs &a, size_t row, int blk0, int, Raw &r) {
        r.h[0] = ldg16(a.meta + row * a.meta_pitch + (size_t)(blk0 >> 3) * 16);
    }
    __device__ static int4v operand(const Raw &r, int u, int) {
        int4v b;
#pragma unroll
        for (int i = 0; i < 4; i++) { // 16 (q - 8)
            const uint32_t w = r.q[u >> 1][i];
            b[i] = (int)((((u & 1) ? w : w << 4) & 0xF0F0F0F0u) ^ 0x80808080u);
        }
        return b;
    }
    __device__ static void coef(const Raw &r, int u, float &d, float &mo) {
        float dsc, dm;
        scale_min(r.h[u >> 3], u & 7, dsc, dm);
        coef_of(dsc, dm, 8.0f, d, mo);
    }
    // operand = (16 or 8) (q - C): the scale over that factor, and the weight of the middle code (both products exact)
    __device__ static void coef_of(float dsc, float dm, float C, float &d, float &mo) {
        d = dsc * (C == 8.0f ? 0.0625f : 0.125f);
        mo = C * dsc - dm;
    }
    // the 6-bit scale and minimum of sub-block j of the superblock with header h (ggml get_scale_min_k4 order), times d and dmin
    __device__ static void scale_min(const u32x4 &h, int j, float &dsc, float &dm) {
        const uint32_t sc_lo = (j & 4) ? h[3] : h[1], mn_lo = (j & 4) ? h[3] : h[2];
        const int sh = 8 * (j & 3);
        uint32_t sc, mn;
        if (j < 4) {
            sc = (h[1] >> sh) & 63;
            mn = (h[2] >> sh) & 63;
        } else {
            sc = ((sc_lo >> sh) & 0xF) | (((h[1] >> sh) >> 6 & 3) << 4);
            mn = ((mn_lo >> sh) >> 4 & 0xF) | (((h[2] >> sh) >> 6 & 3) << 4);
        }
        dsc = f16lo(h[0]) * (float)sc;
        dm = f16hi(h[0]) * (float)mn;
    }
};

// Q5_K: Q4_K's pieces and headers; the fifth bits from the qh plane (32 bytes per superblock, byte l bit s = element l of
// sub-block s): its two 16-byte pieces go through a second patch, lane half h wants piece h.
struct MQ5K {
    static constexpr int NP2 = 2, NQ2 = 1;
    static constexpr bool RUNS16 = false;
    static constexpr bool EVEN_ODD = false;
    static constexpr bool OFFSET = true;
    struct Raw { u32x4 q[UNITS / 2]; u32x4 h[UNITS / 8]; u32x4 q2[1]; };
    static constexpr int NP = 8, NQ = 4;
    __device__ static size_t piece_off(const MbArgs &a, int blk0, int p) { return MQ4K::piece_off(a, blk0, p); }
    __device__ static int want(int j, int h) { return 4 * h + j; }
    __device__ static size_t piece2_off(const MbArgs &, int blk0, int p) { return (size_t)(blk0 >> 3) * 32 + (size_t)p * 16; }
    __device__ static int want2(int, int h) { return h; }
    __device__ static void load_meta(const MbArgs &a, size_t row, int blk0, int, Raw &r) {
        r.h[0] = ldg16(a.meta + row * a.meta_pitch + (size_t)(blk0 >> 3) * 16);
    }
    __device__ static int4v operand(const Raw &r, int u, int) {
        int4v b;
#pragma unroll
        for (int i = 0; i < 4; i++) { // 8 (q - 16): the nibble at bits 3..6, the fifth bit, flipped, at bit 7
            const uint32_t w = r.q[u >> 1][i];
            const uint32_t nib = ((u & 1) ? w >> 1 : w << 3) & 0x78787878u, fifth = (r.q2[0][i] << (7 - u)) & 0x80808080u;
            b[i] = (int)(nib ^ fifth ^ 0x80808080u);
        }
        return b;
    }
    __device__ static void coef(const Raw &r, int u, float &d, float &mo) {
        float dsc, dm;
        MQ4K::scale_min(r.h[u >> 3], u & 7, dsc, dm);
        MQ4K::coef_of(dsc, dm, 16.0f, d, mo);
    }
};

// Q6_K (planes in ggml's order): a chunk is one superblock, its blocks u = 4 n + c the 32 elements 128 n + 32 c ..; the two
// halves of a block are sub-blocks with a scale each, so a block is two products, each with the other half's codes
// as zeros.  ql piece 4 n + 2 (c % 2) + h holds the lane's 16 codes of blocks (n, c) and (n, c + 2) in its low and
// high nibbles, qh piece 2 n + h their bit pairs c; the codes go in as signed bytes q - 32.
struct MQ6K {
    static constexpr int NP2 = 4, NQ2 = 2;
    static constexpr bool RUNS16 = true;
    static constexpr bool EVEN_ODD = false;
    [[maybe_unused]] static constexpr bool OFFSET = false;
    struct Raw { u32x4 q[4]; u32x4 m[1]; float d; u32x4 q2[2]; };
    static_assert(UNITS == 8, "one superblock per chunk");
    static constexpr int NP = 8, NQ = 4;
    __device__ static size_t piece_off(const MbArgs &, int blk0, int p) { return (size_t)(blk0 >> 3) * 128 + (size_t)p * 16; }
    __device__ static int want(int j, int h) { return 2 * j + h; }
    __device__ static size_t piece2_off(const MbArgs &, int blk0, int p) { return (size_t)(blk0 >> 3) * 64 + (size_t)p * 16; }
    __device__ static int want2(int j, int h) { return 2 * j + h; }
    __device__ static void load_meta(const MbArgs &a, size_t row, int blk0, int nblk, Raw &r) {
        const uint8_t *m = a.meta + row * a.meta_pitch;
        r.m[0] = ldg16(m + (size_t)(blk0 >> 3) * 16);
        r.d = __half2float(__ushort_as_half(*reinterpret_cast<const unsigned short *>(m + (size_t)(nblk >> 3) * 16 + (size_t)(blk0 >> 3) * 2)));
    }
    __device__ static int4v operand(const Raw &r, int u, int) {
        const int n = u >> 2, c = u & 3, sh = 4 * (c >> 1);
        int4v b;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t v = ((r.q[2 * n + (c & 1)][i] >> sh) & 0x0F0F0F0Fu) | (((r.q2[n][i] >> (2 * c)) & 0x03030303u) << 4);
            b[i] = (int)((v + 0x60606060u) ^ 0x80808080u); // q - 32 as a signed byte, no carry between bytes
        }
        return b;
    }
    // d * scale of half `hh` of block u (sub-block 2 u + hh)
    __device__ static float coef16(const Raw &r, int u, int hh) {
        const int sb = 2 * u + hh;
        return r.d * (float)(int8_t)((r.m[0][sb >> 2] >> (8 * (sb & 3))) & 0xFF);
    }
    __device__ static void coef(const Raw &, int, float &d, float &mo) { d = 0.f; mo = 0.f; } // not used (RUNS16)
};

// Q5_0 / Q5_1 (GGUF): byte j of a block's 16 = elements j (low nibble) and j + 16 (high); the qh plane holds the fifth bits,
// 4 bytes per block: the chunk's 32 bytes are two pieces, every lane wants both.
template <bool WITH_MIN>
struct MQ5x {
    static constexpr int NP2 = 2, NQ2 = 2;
    static constexpr bool RUNS16 = false;
    static constexpr bool EVEN_ODD = false;
    static constexpr bool OFFSET = WITH_MIN;
    static constexpr int NV = MQ4x<WITH_MIN>::NV;
    struct Raw { u32x4 q[UNITS]; u32x4 m[NV]; u32x4 q2[2]; };
    static constexpr int NP = UNITS, NQ = UNITS;
    __device__ static size_t piece_off(const MbArgs &, int blk0, int p) { return (size_t)(blk0 + p) * 16; }
    __device__ static int want(int j, int) { return j; }
    __device__ static size_t piece2_off(const MbArgs &, int blk0, int p) { return (size_t)blk0 * 4 + (size_t)p * 16; }
    __device__ static int want2(int j, int) { return j; }
    __device__ static void load_meta(const MbArgs &a, size_t row, int blk0, int nblk, Raw &r) {
        typename MQ4x<WITH_MIN>::Raw t;
        MQ4x<WITH_MIN>::load_meta(a, row, blk0, nblk, t);
#pragma unroll
        for (int i = 0; i < NV; i++) r.m[i] = t.m[i];
    }
    __device__ static int4v operand(const Raw &r, int u, int h) {
        const uint32_t bits = ~(r.q2[u >> 2][u & 3] >> (16 * h)); // flipped: 8 (q - 16) has the fifth bit's complement on top
        int4v b;
#pragma unroll
        for (int i = 0; i < 4; i++) // four bits to bit 7 of four bytes: t * 0x00204081 puts bit i at bit 8 i
            b[i] = (int)((((r.q[u][i] >> (4 * h)) & 0x0F0F0F0Fu) << 3) | (((((bits >> (4 * i)) & 0xFu) * 0x00204081u) & 0x01010101u) << 7));
        return b;
    }
    __device__ static void coef(const Raw &r, int u, float &d, float &mo) {
        if (WITH_MIN) {
            const uint32_t v = r.m[u >> 2][u & 3];
            const float dd = f16lo(v);
            d = dd * 0.125f;
            mo = fmaf(16.0f, dd, f16hi(v));
        } else {
            const uint32_t v = r.m[u >> 3][(u >> 1) & 3];
            d = ((u & 1) ? f16hi(v) : f16lo(v)) * 0.125f;
            mo = 0.f;
        }
    }
};

template <class T>
__global__ void __launch_bounds__(512, 4) gemv_mb_kernel(MbArgs a) {
    extern __shared__ float lds_f[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int S = (int)blockDim.x >> 6;
    const int n = lane & 31, h = lane >> 5;
    const int nblk = a.k >> 5;
    float *sgs = lds_f;                    // [block of the row][h][4]: group scales of vectors h, h+2, h+4, h+6
    float *xss = sgs + (size_t)nblk * 8;   // same layout: plain sums of x over the group (contiguous with sgs)
    float *red = xss + (size_t)nblk * 8;   // [wave][vector][row]
    u32x4 *patch = reinterpret_cast<u32x4 *>(red + (size_t)S * MAX_BATCH * 32) + (size_t)wave * 32 * (T::NP + T::NP2); // this wave's 32 x NP pieces
    u32x4 *patch2 = patch + 32 * T::NP;                                                                              // and 32 x NP2 of the qh plane

    // scales and sums of all vectors -> LDS (already in the order the lanes read them).  Requesting the waves' first
    // chunks before this barrier instead of after it was slower (2.70 against 2.54 ms per batched 7B step): nobody
    // multiplies until the slowest wave's chunk has arrived.
    for (int t = tid; t < nblk * 4; t += (int)blockDim.x)
        reinterpret_cast<float4 *>(lds_f)[t] = reinterpret_cast<const float4 *>(a.xsg)[t];
    const int row0 = blockIdx.x * 32;
    int row = row0 + n;
    row = row < a.n_rows ? row : a.n_rows - 1;
    __syncthreads();

    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    const int nchunks = (nblk + UNITS - 1) / UNITS;
    const int c_lo = (int)blockIdx.y * a.chunks_per_split, c_hi = c_lo + a.chunks_per_split < nchunks ? c_lo + a.chunks_per_split : nchunks;
    for (int c = c_lo + wave; c < c_hi; c += S) {
        const int blk0 = c * UNITS;
        const int nu = nblk - blk0 < UNITS ? nblk - blk0 : UNITS;
        // 1. this lane's A operands for the chunk's blocks: one contiguous kilobyte per wave and block
        int4v A[UNITS];
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            const int b = u < nu ? blk0 + u : blk0;
            const u32x4 v = ldg16(a.xa + ((size_t)(b * 2 + h) * 32 + n) * 16);
            A[u] = int4v{(int)v[0], (int)v[1], (int)v[2], (int)v[3]};
        }
        // 2. the weights of the chunk.  Codes: the wave fetches its 32 rows' pieces with whole runs per row (eight
        //    or sixteen lanes side by side on one row) and turns them into "lane = row" through its LDS patch;
        //    a lane reading 16 bytes of its own row per load would touch 32 cache lines per instruction.
        constexpr int NP = T::NP, NI = NP / 2;
        u32x4 stage[NI];
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const int idx = i * 64 + lane, r = idx / NP, pc = idx % NP;
            const int gr = row0 + r < a.n_rows ? row0 + r : a.n_rows - 1;
            stage[i] = ldg16(a.codes + (size_t)gr * a.codes_pitch + T::piece_off(a, blk0, pc));
        }
        constexpr int NP2 = T::NP2, NI2 = (32 * NP2 + 63) / 64;
        u32x4 stage2[NI2 > 0 ? NI2 : 1];
        if constexpr (NP2 > 0) {
#pragma unroll
            for (int i = 0; i < NI2; i++) {
                const int idx = i * 64 + lane, r = idx / NP2, pc = idx % NP2;
                const int gr = row0 + r < a.n_rows ? row0 + r : a.n_rows - 1;
                stage2[i] = ldg16(a.qh + (size_t)gr * a.qh_pitch + T::piece2_off(a, blk0, pc));
            }
        }
        typename T::Raw raw;
        T::load_meta(a, (size_t)row, blk0, nblk, raw);
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const int idx = i * 64 + lane, r = idx / NP, pc = idx % NP;
            patch[r * NP + (pc ^ (r & (NP - 1)))] = stage[i]; // rotated per row: the reads below spread over the banks
        }
        if constexpr (NP2 > 0) {
#pragma unroll
            for (int i = 0; i < NI2; i++) {
                const int idx = i * 64 + lane, r = idx / NP2, pc = idx % NP2;
                patch2[r * NP2 + (pc ^ (r & (NP2 - 1)))] = stage2[i];
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): the wave's LDS writes have landed
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int j = 0; j < T::NQ; j++) raw.q[j] = patch[n * NP + (T::want(j, h) ^ (n & (NP - 1)))];
        if constexpr (NP2 > 0) {
#pragma unroll
            for (int j = 0; j < T::NQ2; j++) raw.q2[j] = patch2[n * NP2 + (T::want2(j, h) ^ (n & (NP2 - 1)))];
        }
        // 3. one MFMA per block; the lane scales and adds its four vectors
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            if constexpr (T::RUNS16) {
                if (u < nu) { // a scale per half block: two products, each with the other half's codes as zeros
                    const int16v zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    const int4v codes = T::operand(raw, u, h), none = {0, 0, 0, 0};
                    const int g = blk0 + u;
                    const float4 sg4 = *reinterpret_cast<const float4 *>(sgs + (size_t)(g * 2 + h) * 4);
                    const float sgv[4] = {sg4.x, sg4.y, sg4.z, sg4.w};
#pragma unroll
                    for (int hh = 0; hh < 2; hh++) {
                        const int16v D = __builtin_amdgcn_mfma_i32_32x32x32_i8(A[u], h == hh ? codes : none, zero, 0, 0, 0);
                        const float d = T::coef16(raw, u, hh);
#pragma unroll
                        for (int bi = 0; bi < 4; bi++)
                            acc[bi] = fmaf(d * sgv[bi], recombine4(D[4 * bi], D[4 * bi + 1], D[4 * bi + 2], D[4 * bi + 3]), acc[bi]);
                    }
                }
            } else if (u < nu) {
                const int16v zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                const int16v D = __builtin_amdgcn_mfma_i32_32x32x32_i8(A[u], T::operand(raw, u, h), zero, 0, 0, 0);
                float d, mo;
                T::coef(raw, u, d, mo);
                const int g = blk0 + u;
                const float4 sg4 = *reinterpret_cast<const float4 *>(sgs + (size_t)(g * 2 + h) * 4);
                const float sgv[4] = {sg4.x, sg4.y, sg4.z, sg4.w};
#pragma unroll
                for (int bi = 0; bi < 4; bi++)
                    acc[bi] = fmaf(d * sgv[bi], recombine4(D[4 * bi], D[4 * bi + 1], D[4 * bi + 2], D[4 * bi + 3]), acc[bi]);
                if (T::OFFSET) {
                    const float4 xs4 = *reinterpret_cast<const float4 *>(xss + (size_t)(g * 2 + h) * 4);
                    acc[0] = fmaf(mo, xs4.x, acc[0]); acc[1] = fmaf(mo, xs4.y, acc[1]);
                    acc[2] = fmaf(mo, xs4.z, acc[2]); acc[3] = fmaf(mo, xs4.w, acc[3]);
                }
            }
        }
    }
    // 4. partial sums of the waves -> y, in wave order
#pragma unroll
    for (int bi = 0; bi < 4; bi++) red[((size_t)wave * MAX_BATCH + (2 * bi + h)) * 32 + n] = acc[bi];
    __syncthreads();
    for (int t = tid; t < a.batch * 32; t += (int)blockDim.x) {
        const int b = t >> 5, r = t & 31;
        if (row0 + r < a.n_rows) {
            float tot = 0.f;
            for (int w = 0; w < S; w++) tot += red[((size_t)w * MAX_BATCH + b) * 32 + r];
            if (a.ypart) {
                a.ypart[((size_t)blockIdx.y * a.batch + b) * a.n_rows + row0 + r] = tot;
            } else {
                if (a.bias) tot += a.bias[row0 + r];
                if (a.resid) tot += a.resid[(size_t)b * a.n_rows + row0 + r];
                a.y[(size_t)b * a.n_rows + row0 + r] = tot;
            }
        }
    }
}

// f(x)[batch, k] -> A operands and group records.  Thread = (8-element task, vector b); vectors beyond the batch
// are written as zeros.  EVEN_ODD: the h = 0 half of a block's operand holds its even elements, h = 1 the odd.
// XMODE: AXQ_X_PLAIN; AXQ_X_RMSNORM: f = x / sqrt(mean(x^2) + eps) * aux (every workgroup sums its vector's squares
// itself); AXQ_X_SWIGLU: x holds [batch, 2k] gate/up values, four gate values followed by the four up values of the
// same indices, and f = silu(gate) * up.
template <bool EVEN_ODD, int XMODE>
__global__ void __launch_bounds__(256) pack_x_kernel(const float *x, const float *aux, float eps, int k, int batch, uint8_t *xa,
                                                     float *xsg) {
    __shared__ float red[4];
    const int t = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
    const int ntask = k >> 3, nblk = k >> 5;
    float inv = 1.0f;
    if (XMODE == AXQ_X_RMSNORM && b < batch) { // before any thread leaves: the sum needs the whole workgroup
        const float4 *row = reinterpret_cast<const float4 *>(x + (size_t)b * k);
        float ss = 0.f;
        for (int i = threadIdx.x; i < (k >> 2); i += 256) {
            const float4 v = row[i];
            ss = fmaf(v.x, v.x, ss); ss = fmaf(v.y, v.y, ss); ss = fmaf(v.z, v.z, ss); ss = fmaf(v.w, v.w, ss);
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
        __syncthreads();
        ss = (red[0] + red[1]) + (red[2] + red[3]);
        inv = 1.0f / sqrtf(ss / (float)k + eps);
    }
    if (t >= ntask) return; // k is a multiple of 256: whole quads of tasks
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (b < batch) {
        if (XMODE == AXQ_X_SWIGLU) {
            const float4 *p = reinterpret_cast<const float4 *>(x + (size_t)b * 2 * k + (size_t)t * 16);
#pragma unroll
            for (int g = 0; g < 2; g++) {
                const float4 gt = p[2 * g], up = p[2 * g + 1];
                v[4 * g + 0] = (gt.x * (1.0f / (1.0f + expf(-gt.x)))) * up.x;
                v[4 * g + 1] = (gt.y * (1.0f / (1.0f + expf(-gt.y)))) * up.y;
                v[4 * g + 2] = (gt.z * (1.0f / (1.0f + expf(-gt.z)))) * up.z;
                v[4 * g + 3] = (gt.w * (1.0f / (1.0f + expf(-gt.w)))) * up.w;
            }
        } else {
            const float4 *p = reinterpret_cast<const float4 *>(x + (size_t)b * k + (size_t)t * 8);
            const float4 v0 = p[0], v1 = p[1];
            v[0] = v0.x; v[1] = v0.y; v[2] = v0.z; v[3] = v0.w; v[4] = v1.x; v[5] = v1.y; v[6] = v1.z; v[7] = v1.w;
            if (XMODE == AXQ_X_RMSNORM) {
                const float4 *pw = reinterpret_cast<const float4 *>(aux + (size_t)t * 8);
                const float4 w0 = pw[0], w1 = pw[1];
                const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
                for (int i = 0; i < 8; i++) v[i] = (v[i] * inv) * wv[i];
            }
        }
    }
    axq_store_packed<EVEN_ODD>(v, t, b, batch, nblk, xa, xsg);
}

// y = sum over the splits, in order (+ bias, + resid)
__global__ void __launch_bounds__(256) mb_reduce_kernel(const float *ypart, const float *bias, const float *resid, int n_rows, int batch,
                                                        int splits, float *y) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x, total = n_rows * batch;
    if (i >= total) return;
    float tot = ypart[i];
    for (int z = 1; z < splits; z++) tot += ypart[(size_t)z * total + i];
    if (bias) tot += bias[i % n_rows];
    if (resid) tot += resid[i];
    y[i] = tot;
}

// The same reduction for a result that is the input of the next small-batch GEMV (its n_rows are that GEMV's k):
// one workgroup per vector adds the splits (+ bias, + resid), writes y, and goes on to what pack_x_kernel would do
// with y next (RMSNorm with the weights next_aux when those are given, then the split into limbs), with the row in
// registers in between.  splits = 0: `src` is the finished y already.  n <= 16384, a multiple of 256.
template <bool EVEN_ODD>
__global__ void __launch_bounds__(512) mb_reduce_pack_kernel(const float *src, int splits, const float *bias, const float *resid, int n,
                                                             int batch, float *y, const float *next_aux, float eps, uint8_t *xa,
                                                             float *xsg) {
    constexpr int TPT = 4; // tasks of eight elements per thread
    __shared__ float red[8];
    const int b = blockIdx.x, ntask = n >> 3, nblk = n >> 5;
    const size_t total = (size_t)n * batch;
    float v[TPT][8];
    float ss = 0.f;
#pragma unroll
    for (int q = 0; q < TPT; q++) {
        const int t = q * 512 + (int)threadIdx.x;
#pragma unroll
        for (int i = 0; i < 8; i++) v[q][i] = 0.f;
        if (t < ntask && b < batch) {
            const size_t at = (size_t)b * n + (size_t)t * 8;
            const float4 *p = reinterpret_cast<const float4 *>(src + at);
            float4 a0 = p[0], a1 = p[1];
            for (int z = 1; z < splits; z++) {
                const float4 *pz = reinterpret_cast<const float4 *>(src + (size_t)z * total + at);
                const float4 c0 = pz[0], c1 = pz[1];
                a0.x += c0.x; a0.y += c0.y; a0.z += c0.z; a0.w += c0.w;
                a1.x += c1.x; a1.y += c1.y; a1.z += c1.z; a1.w += c1.w;
            }
            if (splits > 0) {
                if (bias) {
                    const float *pb = bias + (size_t)t * 8;
                    a0.x += pb[0]; a0.y += pb[1]; a0.z += pb[2]; a0.w += pb[3];
                    a1.x += pb[4]; a1.y += pb[5]; a1.z += pb[6]; a1.w += pb[7];
                }
                if (resid) {
                    const float4 *pr = reinterpret_cast<const float4 *>(resid + at);
                    const float4 r0 = pr[0], r1 = pr[1];
                    a0.x += r0.x; a0.y += r0.y; a0.z += r0.z; a0.w += r0.w;
                    a1.x += r1.x; a1.y += r1.y; a1.z += r1.z; a1.w += r1.w;
                }
                reinterpret_cast<float4 *>(y + at)[0] = a0;
                reinterpret_cast<float4 *>(y + at)[1] = a1;
            }
            v[q][0] = a0.x; v[q][1] = a0.y; v[q][2] = a0.z; v[q][3] = a0.w;
            v[q][4] = a1.x; v[q][5] = a1.y; v[q][6] = a1.z; v[q][7] = a1.w;
#pragma unroll
            for (int i = 0; i < 8; i++) ss = fmaf(v[q][i], v[q][i], ss);
        }
    }
    if (next_aux) { // RMSNorm of the whole row (RMSNorm::forward, llm/src/llama.rs:158-187)
        // the norm weights are requested before the workgroup meets over the sum of squares
        float4 w0[TPT], w1[TPT];
#pragma unroll
        for (int q = 0; q < TPT; q++) {
            const int t = q * 512 + (int)threadIdx.x;
            const float4 *pw = reinterpret_cast<const float4 *>(next_aux + (size_t)(t < ntask ? t : 0) * 8);
            w0[q] = pw[0];
            w1[q] = pw[1];
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
        __syncthreads();
        ss = ((red[0] + red[1]) + (red[2] + red[3])) + ((red[4] + red[5]) + (red[6] + red[7]));
        const float inv = 1.0f / sqrtf(ss / (float)n + eps);
#pragma unroll
        for (int q = 0; q < TPT; q++) {
            const int t = q * 512 + (int)threadIdx.x;
            if (t < ntask && b < batch) {
                const float wv[8] = {w0[q].x, w0[q].y, w0[q].z, w0[q].w, w1[q].x, w1[q].y, w1[q].z, w1[q].w};
#pragma unroll
                for (int i = 0; i < 8; i++) v[q][i] = (v[q][i] * inv) * wv[i];
            }
        }
    }
#pragma unroll
    for (int q = 0; q < TPT; q++) {
        const int t = q * 512 + (int)threadIdx.x;
        if (t < ntask) axq_store_packed<EVEN_ODD>(v[q], t, b, batch, nblk, xa, xsg); // ntask is a multiple of 4: whole quads
    }
}

// next_even_odd < 0: nothing follows.  Otherwise y is the input of another small-batch GEMV whose operands
// (EVEN_ODD as given, RMSNorm with next_aux when that is not null) are prepared here, in the same scratch.
// Dynamic LDS beyond 64 KB is asked for once per kernel and device; bit d = device d has been asked (axq_allow_lds).
template <class T>
std::atomic<uint64_t> &mb_lds_mask() {
    static std::atomic<uint64_t> mask{0};
    return mask;
}
unsigned mb_max_waves() {
    static const unsigned smax = getenv("AXQ_BATCH_WAVES") ? (unsigned)atoi(getenv("AXQ_BATCH_WAVES")) : 8; // development knob (1..8)
    return smax < 1 ? 1 : (smax > 8 ? 8 : smax);
}

template <class T>
int launch_mb(axq_ctx *ctx, MbArgs a, uint8_t *sc, const float *x, int xmode, const float *aux, float eps, int next_even_odd, const float *next_aux) {
    const dim3 pgrid((unsigned)((a.k / 8 + 255) / 256), MAX_BATCH);
    uint8_t *xa = const_cast<uint8_t *>(a.xa);
    float *xsg = const_cast<float *>(a.xsg);
    if (xmode == AXQ_X_PACKED) {
        // the operands are in place already (the previous call prepared them)
    } else if (xmode == AXQ_X_RMSNORM) pack_x_kernel<T::EVEN_ODD, AXQ_X_RMSNORM><<<pgrid, 256, 0, ctx->stream>>>(x, aux, eps, a.k, a.batch, xa, xsg);
    else if (xmode == AXQ_X_SWIGLU) pack_x_kernel<T::EVEN_ODD, AXQ_X_SWIGLU><<<pgrid, 256, 0, ctx->stream>>>(x, aux, eps, a.k, a.batch, xa, xsg);
    else pack_x_kernel<T::EVEN_ODD, AXQ_X_PLAIN><<<pgrid, 256, 0, ctx->stream>>>(x, aux, eps, a.k, a.batch, xa, xsg);
    const unsigned chunks = (unsigned)((a.k + WAVE_K - 1) / WAVE_K);
    const unsigned tiles = (unsigned)((a.n_rows + 31) / 32);
    // few row tiles (a narrow output): split K over up to four workgroups per tile so that the chip is full
    // (twice as many, for two workgroups per compute unit, was slower: 2.36 against 2.32 ms per batched 7B step; so were
    // 64-row workgroups that fetch the A operands once for two row tiles: 1 % faster on the gate/up shape, slower elsewhere)
    unsigned splits = (unsigned)ctx->prop.multiProcessorCount / tiles;
    splits = splits > 4 ? 4 : splits;
    if (splits > chunks / 8) splits = chunks / 8;
    if (splits < 2 || !a.ypart) splits = 1;
    a.chunks_per_split = (int)((chunks + splits - 1) / splits);
    splits = (chunks + a.chunks_per_split - 1) / a.chunks_per_split;
    if (splits < 2) a.ypart = nullptr;
    const unsigned smax = mb_max_waves();
    const unsigned S = (unsigned)a.chunks_per_split < smax ? (unsigned)a.chunks_per_split : smax;
    const size_t lds = ((size_t)(a.k / 32) * 16 + (size_t)S * MAX_BATCH * 32) * sizeof(float) + (size_t)S * 32 * (T::NP + T::NP2) * 16;
    if (lds > 64 * 1024) {
        const int st = axq_allow_lds(ctx, reinterpret_cast<const void *>(&gemv_mb_kernel<T>), mb_lds_mask<T>(), 160 * 1024);
        if (st != AXQ_OK) return st; // the refusal is the call's error: nothing is launched into it
    }
    gemv_mb_kernel<T><<<dim3(tiles, splits), 64 * S, lds, ctx->stream>>>(a);
    if (next_even_odd >= 0) {
        // y's operands for the next GEMV (k' = n_rows): the scratch layout of that call
        uint8_t *nxa = sc;
        float *nxsg = reinterpret_cast<float *>(sc + (size_t)32 * a.n_rows);
        const float *src = splits > 1 ? a.ypart : a.y;
        const int nsp = splits > 1 ? (int)splits : 0;
        if (next_even_odd)
            mb_reduce_pack_kernel<true><<<MAX_BATCH, 512, 0, ctx->stream>>>(src, nsp, a.bias, a.resid, a.n_rows, a.batch, a.y, next_aux, eps, nxa, nxsg);
        else
            mb_reduce_pack_kernel<false><<<MAX_BATCH, 512, 0, ctx->stream>>>(src, nsp, a.bias, a.resid, a.n_rows, a.batch, a.y, next_aux, eps, nxa, nxsg);
    } else if (splits > 1) {
        const int total = a.n_rows * a.batch;
        mb_reduce_kernel<<<(total + 255) / 256, 256, 0, ctx->stream>>>(a.ypart, a.bias, a.resid, a.n_rows, a.batch, (int)splits, a.y);
    }
    return AXQ_OK;
}

// One call of the small-batch GEMV with its scratch at `sc` (AXQ_BATCH_SCRATCH_BYTES bytes): 32 k bytes of A operands,
// then 2 * (k / 32) * 8 floats of scales and sums; behind AXQ_BATCH_MAX_K's worth of those the partial sums of a split
// K (splits only happen below AXQ_BATCH_SPLIT_ROWS rows).  Every byte that a kernel reads there is written earlier in
// the same call, so the buffer needs no clearing between calls.
int gemv_batch_in(axq_ctx *ctx, uint8_t *sc, const axq_weight *w, const float *x, int xmode, const float *aux, float eps, int batch,
                  const float *bias, const float *resid, float *y, int next_even_odd, const float *next_aux) {
    const int k = (int)w->k;
    MbArgs a;
    a.codes = w->codes; a.meta = w->meta; a.qh = w->qh;
    a.codes_pitch = w->codes_pitch; a.meta_pitch = w->meta_pitch; a.qh_pitch = w->qh_pitch;
    a.xa = sc; a.xsg = reinterpret_cast<float *>(sc + (size_t)32 * k);
    a.bias = bias; a.resid = resid; a.y = y;
    a.ypart = w->n_rows <= AXQ_BATCH_SPLIT_ROWS ? reinterpret_cast<float *>(sc + (size_t)34 * AXQ_BATCH_MAX_K) : nullptr;
    a.n_rows = (int)w->n_rows; a.k = k; a.batch = batch;
    int st;
    switch (w->type) {
    case AXQ_Q4_0: st = launch_mb<MQ4x<false>>(ctx, a, sc, x, xmode, aux, eps, next_even_odd, next_aux); break;
    case AXQ_Q4_1: st = launch_mb<MQ4x<true>>(ctx, a, sc, x, xmode, aux, eps, next_even_odd, next_aux); break;
    case AXQ_Q8_0: st = launch_mb<MQ80>(ctx, a, sc, x, xmode, aux, eps, next_even_odd, next_aux); break;
    case AXQ_Q4_K: st = launch_mb<MQ4K>(ctx, a, sc, x, xmode, aux, eps, next_even_odd, next_aux); break;
    case AXQ_Q5_K: st = launch_mb<MQ5K>(ctx, a, sc, x, xmode, aux, eps, next_even_odd, next_aux); break;
    case AXQ_Q6_K: st = launch_mb<MQ6K>(ctx, a, sc, x, xmode, aux, eps, next_even_odd, next_aux); break;
    case AXQ_Q5_0: st = launch_mb<MQ5x<false>>(ctx, a, sc, x, xmode, aux, eps, next_even_odd, next_aux); break;
    case AXQ_Q5_1: st = launch_mb<MQ5x<true>>(ctx, a, sc, x, xmode, aux, eps, next_even_odd, next_aux); break;
    default: return axq_fail(ctx, AXQ_ERR_INVALID_QUANT_TYPE, "Invalid quantization type: %d", w->type);
    }
    if (st != AXQ_OK) return st;
    AXQ_LAUNCH_CHECK(ctx, "gemv_mb_kernel");
    return AXQ_OK;
}

} // namespace

// Whether the batched kernel covers this call.
bool axq_dev_gemv_batch_covers(const axq_weight *w, int batch) {
    if (batch < 2 || batch > MAX_BATCH) return false;
    if (w->k % 256 != 0 || w->k > AXQ_BATCH_MAX_K) return false; // 34 k bytes of scratch: the context's x buffer holds that much
    switch (w->type) {
    case AXQ_Q4_0: case AXQ_Q4_1: case AXQ_Q5_0: case AXQ_Q5_1: case AXQ_Q8_0: case AXQ_Q4_K: case AXQ_Q5_K: case AXQ_Q6_K: return true;
    default: return false;
    }
}

// Where a caller that prepares the operands of the call with w itself (axq_store_packed, then xmode = AXQ_X_PACKED) has
// to put them; returns whether w takes the even and the odd elements of a block in separate halves.
bool axq_dev_gemv_batch_operands(axq_ctx *ctx, const axq_weight *w, uint8_t **xa, float **xsg) {
    *xa = ctx->xq;
    *xsg = reinterpret_cast<float *>(ctx->xq + (size_t)32 * w->k);
    return w->type == AXQ_Q4_0 || w->type == AXQ_Q4_1;
}

int axq_dev_gemv_batch(axq_ctx *ctx, const axq_weight *w, const float *x, int batch, const float *bias, const float *resid, float *y) {
    return axq_dev_gemv_batch_ex(ctx, w, x, AXQ_X_PLAIN, nullptr, 0.f, batch, bias, resid, y);
}

// y[batch, n_rows] = f(x)[batch, k] W^T (+ bias per row of W) (+ resid[batch, n_rows], which may be y) for
// 2 <= batch <= 8: split the batch (f = xmode, see pack_x_kernel), then one pass over W.
int axq_dev_gemv_batch_ex(axq_ctx *ctx, const axq_weight *w, const float *x, int xmode, const float *aux, float eps, int batch,
                          const float *bias, const float *resid, float *y) {
    return axq_dev_gemv_batch_chain(ctx, w, x, xmode, aux, eps, batch, bias, resid, y, nullptr, nullptr);
}

// The same, and when `next` is given (a weight with k = w's n_rows that the small-batch kernel covers), y's operands for
// the GEMV with `next` are prepared on the way (RMSNorm with next_aux when that is not null): that call then takes
// xmode = AXQ_X_PACKED and no x.  The eps of a following RMSNorm is this call's eps.
int axq_dev_gemv_batch_chain(axq_ctx *ctx, const axq_weight *w, const float *x, int xmode, const float *aux, float eps, int batch,
                             const float *bias, const float *resid, float *y, const axq_weight *next, const float *next_aux) {
    int next_even_odd = -1;
    if (next) {
        if (next->k != w->n_rows || !axq_dev_gemv_batch_covers(next, batch))
            return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: the next weight does not take this one's output");
        next_even_odd = (next->type == AXQ_Q4_0 || next->type == AXQ_Q4_1) ? 1 : 0;
    }
    return gemv_batch_in(ctx, ctx->xq, w, x, xmode, aux, eps, batch, bias, resid, y, next_even_odd, next_aux);
}

// ---------------------------------------------------------------------------
// The entry point that allocates nothing.  Its kernels are the ones above; the scratch they need (the batch's
// operands, the partial sums of a split K) lives in a device array of this file instead of an allocation, one
// copy per GPU, held until the process ends.  Host code never uses the array's name as an address: the set-up
// below asks the runtime once per device where that device's copy lies and keeps the pointer.
// ---------------------------------------------------------------------------
static __device__ __align__(256) uint8_t scratch[AXQ_BATCH_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
uint8_t *g_scratch_ptr[MAX_DEVICES]; // per device: where `scratch` lies there (NULL: not looked up yet)
std::mutex g_scratch_mutex;
} // namespace

// Called by axq_init with the context's device current.
int axq_gemv_static_setup(axq_ctx *ctx) {
    if (ctx->device < 0 || ctx->device >= MAX_DEVICES)
        return axq_fail(ctx, AXQ_ERR_DEVICE_NOT_FOUND, "device %d: the static GEMV scratch is kept for devices 0..%d", ctx->device,
                        MAX_DEVICES - 1);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[ctx->device]) return AXQ_OK;
    uint8_t *ptr = nullptr;
    AXQ_HIP(ctx, hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)), AXQ_ERR_DRIVER);
    if (!ptr) return axq_fail(ctx, AXQ_ERR_DRIVER, "hipGetSymbolAddress gave no address for the static GEMV scratch");
    // Dynamic LDS beyond 64 KB has to be asked for once per kernel and device, and the development knob is read once: both
    // here, through the very masks the launch code consults, so that the entry point itself only launches.
    int st = axq_allow_lds(ctx, reinterpret_cast<const void *>(&gemv_mb_kernel<MQ4x<false>>), mb_lds_mask<MQ4x<false>>(), 160 * 1024);
    if (st == AXQ_OK) st = axq_allow_lds(ctx, reinterpret_cast<const void *>(&gemv_mb_kernel<MQ4x<true>>), mb_lds_mask<MQ4x<true>>(), 160 * 1024);
    if (st == AXQ_OK) st = axq_allow_lds(ctx, reinterpret_cast<const void *>(&gemv_mb_kernel<MQ80>), mb_lds_mask<MQ80>(), 160 * 1024);
    if (st == AXQ_OK) st = axq_allow_lds(ctx, reinterpret_cast<const void *>(&gemv_mb_kernel<MQ4K>), mb_lds_mask<MQ4K>(), 160 * 1024);
    if (st != AXQ_OK) return st;
    (void)mb_max_waves();
    g_scratch_ptr[ctx->device] = ptr;
    return AXQ_OK;
}

int axq_gemv_f32_static(axq_ctx *ctx, const axq_weight *w, const float *x, int batch, const float *bias, float *y) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_gemv_f32_static: NULL context");
    if (!w || !x || !y) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_gemv_f32_static: NULL pointer");
    if (batch < 2 || batch > MAX_BATCH)
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: axq_gemv_f32_static takes 2..%d vectors per call, got %d", MAX_BATCH,
                        batch);
    if (w->k > AXQ_BATCH_MAX_K)
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: k = %lld is beyond the static scratch (k <= %d)", (long long)w->k,
                        AXQ_BATCH_MAX_K);
    if (w->n_rows > INT32_MAX)
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: weight dimensions exceed 2^31");
    if (w->k % 256 != 0)
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: axq_gemv_f32_static takes k a multiple of 256, got %lld", (long long)w->k);
    if (!axq_dev_gemv_batch_covers(w, batch))
        return axq_fail(ctx, AXQ_ERR_INVALID_QUANT_TYPE, "axq_gemv_f32_static covers the block types (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q4_K, Q5_K, Q6_K), not type %d", w->type);
    uint8_t *ptr = (ctx->device >= 0 && ctx->device < MAX_DEVICES) ? g_scratch_ptr[ctx->device] : nullptr;
    if (!ptr) return axq_fail(ctx, AXQ_ERR_DRIVER, "the static GEMV scratch of device %d was not set up (devices 0..%d have one)", ctx->device, MAX_DEVICES - 1);
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    return gemv_batch_in(ctx, ptr, w, x, AXQ_X_PLAIN, nullptr, 0.f, batch, bias, nullptr, y, -1, nullptr);
}
