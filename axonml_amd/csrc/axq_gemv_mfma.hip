// Decode-path quantized matmul, main kernel: integer dot products on the matrix
// pipe.  y[n] = sum_k x[k] * W[n, k] (+ bias[n]) for the block-quantized types.
//
// Why: the kernel is HBM-bound on paper, but unpacking 4-bit codes to f32 and
// issuing one FMA per weight costs about 200 VALU instructions per 4096-wide
// row and makes the vector ALU the real limit.  Here the multiply-accumulate
// runs as v_mfma_i32_4x4x4_16B_i8 ("16 independent 4x4x4 int8 products"), used
// as a wide dot-product unit, not as a GEMM:
//
//   - x is split, once per workgroup, into four signed 7-bit limbs per element
//     against a power-of-two scale per 32-element group:
//         x = s_g * (l0*128^3 + l1*128^2 + l2*128 + l3),   |l_i| <= 64
//     (28 bits below the group's largest magnitude: finer than f32's 24).
//     The limbs are the MFMA's A operand, one limb per matrix row.
//   - a lane's weight codes are the B operand: the four bytes of
//     (q & 0x0F0F0F0F) are four int8 weights of the lane's own row, so a dword
//     of eight 4-bit codes costs three VALU instructions (and, shift, and) and
//     two MFMAs.  Lane (blk, j) = (lane / 4, lane % 4) supplies column j of
//     block blk: row j of the current 4-row step, k-chunk blk of the wave's
//     1024-wide K slice.  Its four accumulators are its own row's dot products
//     with the four limbs: no cross-lane traffic until the final sum.
//   - integer accumulation is exact; per 32-element group the four sums are
//     recombined in f32, scaled by s_g and the block's f16 scale/min; the 16
//     k-chunks of a row are added with two DPP row shifts, then across the four
//     DPP rows and the K slices in a fixed order through LDS: no atomics,
//     results are run-to-run identical.
//
// Memory side: every weight byte is read exactly once with 128-bit loads, 256
// contiguous bytes per row per instruction; a ring of NB row steps per wave is
// kept in flight and refilled as soon as a step has been consumed.
#include <hip/hip_fp16.h>

#include <stdlib.h>

#include "axq_internal.h"
#include "axq_split.h"

namespace {

typedef int int4v __attribute__((ext_vector_type(4)));

struct DpArgs {
    const uint8_t *codes, *meta, *qh;
    size_t codes_pitch, meta_pitch, qh_pitch;
    const float *x, *bias;
    const uint8_t *xq; // x already split into limbs (see stage_x), or NULL: the kernel splits it itself
    float *y;
    int n_rows, k;
    int S, G, P;   // K slices per pass, row groups per workgroup, passes over K per lane
    int steps;     // 4-row steps per group
    int mode;      // what x is: AXQ_X_PLAIN, or a vector still to be normalised (see axq_internal.h)
    const float *aux; // AXQ_X_RMSNORM: the norm weights
    float eps;
    int ymode;     // AXQ_Y_PLAIN or AXQ_Y_SWIGLU
};
// The kernels take these fields as scalar arguments, the ones the first loads need in front: the first fourteen dwords
// are preloaded into scalar registers when a wave starts (-amdgpu-kernarg-preload-count), a struct passed by value is not.
// shape = S | G << 8 | steps << 16, flags = mode | ymode << 8.
#define DP_KERNEL_PARAMS const float *p_x, const uint8_t *p_codes, const uint8_t *p_meta, uint32_t p_cp, uint32_t p_mp, int p_n_rows, int p_k, \
                         int p_shape, int p_flags, float p_eps, float *p_y, const float *p_bias, const float *p_aux, const uint8_t *p_qh, uint32_t p_qp, \
                         const uint8_t *p_xq
#define DP_KERNEL_ARGS DpArgs{p_codes, p_meta, p_qh, p_cp, p_mp, p_qp, p_x, p_bias, p_xq, p_y, p_n_rows, p_k, p_shape & 0xFF, (p_shape >> 8) & 0xFF, 1, \
                              p_shape >> 16, p_flags & 0xFF, p_aux, p_eps, (p_flags >> 8) & 0xFF}
#define DP_LAUNCH_ARGS(a) (a).x, (a).codes, (a).meta, (uint32_t)(a).codes_pitch, (uint32_t)(a).meta_pitch, (a).n_rows, (a).k, \
                          ((a).S | ((a).G << 8) | ((a).steps << 16)), ((a).mode | ((a).ymode << 8)), (a).eps, (a).y, (a).bias, (a).aux, (a).qh, \
                          (uint32_t)(a).qh_pitch, (a).xq

__device__ inline float f16lo(uint32_t v) { return __half2float(__ushort_as_half((unsigned short)(v & 0xFFFF))); }
__device__ inline float f16hi(uint32_t v) { return __half2float(__ushort_as_half((unsigned short)(v >> 16))); }
__device__ inline float ub0(uint32_t v) { float r; asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(r) : "v"(v)); return r; }
__device__ inline float ub1(uint32_t v) { float r; asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(r) : "v"(v)); return r; }

__device__ inline int4v mfma(int a, uint32_t b, int4v c) { return __builtin_amdgcn_mfma_i32_4x4x4i8(a, (int)b, c, 0, 0, 0); }

// sum_k n_k x_k over one 32-element group from its four limb sums
__device__ inline float recombine(int4v d, float sg) {
    float f = fmaf((float)d[0], 128.0f, (float)d[1]);
    f = fmaf(f, 128.0f, (float)d[2]);
    f = fmaf(f, 128.0f, (float)d[3]);
    return f * sg;
}

// What a lane keeps of x for one pass: limb (lane % 4) of its 64 k-values as 16
// MFMA A operands, and scale / plain sum of its two 32-element groups.
struct XOp {
    int a[16];
    float sg[4], xs[2]; // sg[2], sg[3]: types whose lane covers four runs of 16 (RUNS16)
    int4v init[2]; // -(code centre) * (limb sums of the group): the accumulators start here, so that the
                   // MFMAs sum (n - centre) * limb exactly and no large terms cancel in f32 afterwards
};

// Addressing.  A workgroup's rows lie within a few megabytes, so a lane addresses its bytes as
// (uniform 64-bit plane base of the workgroup's first row) + (32-bit offset): one integer add per load.
struct Bases { const uint8_t *codes, *meta, *qh; };  // planes at the workgroup's first row
struct RowOff { uint32_t c, m, h; };                 // (row - first row) * pitch, per plane
struct LaneOff { uint32_t c[2], m[2], h[2], d[2]; }; // the lane's byte offsets inside a row, per plane (d: a second kind of record in the meta plane)
// Weights are read once per call: non-temporal loads keep them from displacing x and the other kernels' operands in
// the caches, and stream measurably faster (a pure read of 33 MB: 6.2 against 6.75 us per launch).
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ inline uint4 ld16(const uint8_t *base, uint32_t off) {
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(base + off));
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ inline uint32_t ld4(const uint8_t *base, uint32_t off) { return __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(base + off)); }
__device__ inline uint32_t ld2(const uint8_t *base, uint32_t off) { return __builtin_nontemporal_load(reinterpret_cast<const uint16_t *>(base + off)); }

// ---------------------------------------------------------------------------
// Per-type traits.  A lane covers 64 weights of one row per pass = two
// 32-element groups.  group_k() gives the K offset of group g for chunk index
// c (c counts 64-weight lane chunks along the row); load() fetches the lane's
// bytes of one row; dot() returns its share of the row's dot product.
// ---------------------------------------------------------------------------
struct DQ4K {
    struct Raw { uint4 q0, q1, h; };
    static constexpr bool X_REQUESTS_FIRST = true; // gemv_dpw_kernel: a barrier between the waves' x requests and their weight requests
    static constexpr bool TWO_SLICE_WAVES = false;
    static constexpr bool RUNS16 = false, OWN_META_PIECES = false;
    static constexpr bool PERM_A = false;
    static constexpr int CENTRE = 8; // w = d*sc*(q - 8) + (8*d*sc - dmin*m)
    static constexpr int BIG_NB = 4; // row steps a lane can hold within 128 registers
    // The kernel that stages x per wave fetches the scale records once per round of up to four row steps (see
    // gemv_dp_kernel's RND): META_SLICE_BYTES of the meta plane per row and 1024-wide K slice, parked in LDS; set_meta picks
    // the lane's own out of its row's.
    static constexpr bool ROUND_META = true;
    static constexpr int META_SLICE_BYTES = 64; // four superblock headers
    __host__ __device__ static int meta_row_bytes(int k) { return (k >> 8) * 16; }
    __device__ static void load_codes(const Bases &b, const RowOff &ro, const LaneOff &o, Raw &r) {
        r.q0 = ld16(b.codes, ro.c + o.c[0]);
        r.q1 = ld16(b.codes, ro.c + o.c[1]);
    }
    __device__ static void set_meta(Raw &r, const uint8_t *row, int blk, int) { r.h = *reinterpret_cast<const uint4 *>(row + (blk >> 2) * 16); }
    __device__ static int group_k(int c, int g) { return c * 64 + g * 32; }
    __device__ static void lane_offsets(int k, int c, LaneOff &o) {
        // the code plane interleaves, per 64-pair slice, the first 16 bytes of every pair, then the second 16
        const int cpr = k >> 6;
        c = c < cpr ? c : cpr - 1; // lanes past the end of the row re-read its last chunk against x = 0
        int slice = c >> 6, pr = c & 63;
        int P = cpr - (slice << 6);
        P = P < 64 ? P : 64;
        o.c[0] = (uint32_t)(slice * 2048 + pr * 16);
        o.c[1] = o.c[0] + (uint32_t)P * 16;
        o.m[0] = (uint32_t)(c >> 2) * 16;
    }
    __device__ static void load(const Bases &b, const RowOff &ro, const LaneOff &o, Raw &r) {
        r.q0 = ld16(b.codes, ro.c + o.c[0]);
        r.q1 = ld16(b.codes, ro.c + o.c[1]);
        r.h = ld16(b.meta, ro.m + o.m[0]);
    }
    __device__ static float dot(const Raw &r, const XOp &x, int c) {
        const uint32_t q0[4] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w};
        const uint32_t q1[4] = {r.q1.x, r.q1.y, r.q1.z, r.q1.w};
        int4v lo = x.init[0], hi = x.init[1];
        // all sixteen B operands first, then the products: the matrix pipe must not read a register the
        // vector ALU has just written
        uint32_t ml[8], mh[8];
#pragma unroll
        for (int w = 0; w < 4; w++) {
            ml[w] = q0[w] & 0x0F0F0F0Fu;            // first half: elements 4w.. of the low-nibble sub-block
            mh[w] = (q0[w] >> 4) & 0x0F0F0F0Fu;     //             ... and of the high-nibble sub-block
            ml[4 + w] = q1[w] & 0x0F0F0F0Fu;        // second half: elements 16+4w..
            mh[4 + w] = (q1[w] >> 4) & 0x0F0F0F0Fu;
        }
#pragma unroll
        for (int w = 0; w < 8; w++) {
            lo = mfma(x.a[w], ml[w], lo);
            hi = mfma(x.a[8 + w], mh[w], hi);
        }
        // 6-bit scale/min of sub-blocks 2p, 2p+1 (ggml get_scale_min_k4 order); p is fixed per lane
        int p = c & 3;
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
        const float d = f16lo(r.h.x), dmin = f16hi(r.h.x);
        const float s0 = d * ub0(scp), s1 = d * ub1(scp);
        float y = fmaf(s0, recombine(lo, x.sg[0]), s1 * recombine(hi, x.sg[1]));
        // what is left of the offsets after centring: small, since dmin*m ~ 8*d*sc for weights centred on zero
        y = fmaf(fmaf(8.0f, s0, -(dmin * ub0(mp))), x.xs[0], y);
        y = fmaf(fmaf(8.0f, s1, -(dmin * ub1(mp))), x.xs[1], y);
        return y;
    }
};

// Q5_K (GGUF): Q4_K's code plane and headers; the fifth bits lie in a plane of their own, 32 bytes per superblock, byte l
// bit s = fifth bit of element l of sub-block s.  A lane (pair p of its superblock) takes bits 2p and 2p + 1 of all 32
// bytes.  Four lanes share those bytes, so they are not loaded per lane and step (a load of 1 KB of lane addresses for
// 256 bytes) but fetched once per round with the headers, as part of the record that goes through LDS.
struct DQ5K {
    struct Raw { uint4 q0, q1, b0, b1, h; };
    static constexpr bool X_REQUESTS_FIRST = false; // gemv_dpw_kernel: a barrier between the waves' x requests and their weight requests
    static constexpr bool TWO_SLICE_WAVES = false;
    static constexpr bool RUNS16 = false, OWN_META_PIECES = true;
    static constexpr bool PERM_A = false;
    static constexpr int CENTRE = 16; // w = d*sc*(q - 16) + (16*d*sc - dmin*m)
    static constexpr int BIG_NB = 4;
    static constexpr bool ROUND_META = true;
    static constexpr int META_SLICE_BYTES = 192; // per row and slice in LDS: four superblock headers, then their 4 x 32 bytes of fifth bits
    __host__ __device__ static int meta_row_bytes(int k) { return (k >> 8) * 16; }
    __device__ static int meta_piece(int k, int slice, int piece, bool &from_qh) {
        const int nsb = k >> 8;
        from_qh = piece >= 4;
        if (!from_qh) {
            const int off = slice * 64 + piece * 16;
            return off + 16 <= nsb * 16 ? off : nsb * 16 - 16;
        }
        const int off = slice * 128 + (piece - 4) * 16;
        return off + 16 <= nsb * 32 ? off : nsb * 32 - 16;
    }
    // with per-round records the fifth bits come with the headers, through LDS
    __device__ static void load_codes(const Bases &b, const RowOff &ro, const LaneOff &o, Raw &r) {
        r.q0 = ld16(b.codes, ro.c + o.c[0]);
        r.q1 = ld16(b.codes, ro.c + o.c[1]);
    }
    __device__ static void set_meta(Raw &r, const uint8_t *row, int blk, int) {
        r.h = *reinterpret_cast<const uint4 *>(row + (blk >> 2) * 16);
        r.b0 = *reinterpret_cast<const uint4 *>(row + 64 + (blk >> 2) * 32);
        r.b1 = *reinterpret_cast<const uint4 *>(row + 64 + (blk >> 2) * 32 + 16);
    }
    __device__ static int group_k(int c, int g) { return c * 64 + g * 32; }
    __device__ static void lane_offsets(int k, int c, LaneOff &o) {
        DQ4K::lane_offsets(k, c, o);
        const int cpr = k >> 6;
        c = c < cpr ? c : cpr - 1;
        o.h[0] = (uint32_t)(c >> 2) * 32;
    }
    __device__ static void load(const Bases &b, const RowOff &ro, const LaneOff &o, Raw &r) {
        load_codes(b, ro, o, r);
        r.b0 = ld16(b.qh, ro.h + o.h[0]); // the four lanes of a superblock read the same 32 bytes
        r.b1 = ld16(b.qh, ro.h + o.h[0] + 16);
        r.h = ld16(b.meta, ro.m + o.m[0]);
    }
    __device__ static float dot(const Raw &r, const XOp &x, int c) {
        const uint32_t q0[4] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w};
        const uint32_t q1[4] = {r.q1.x, r.q1.y, r.q1.z, r.q1.w};
        const uint32_t b0[4] = {r.b0.x, r.b0.y, r.b0.z, r.b0.w};
        const uint32_t b1[4] = {r.b1.x, r.b1.y, r.b1.z, r.b1.w};
        const int p = c & 3;
        int4v lo = x.init[0], hi = x.init[1];
        uint32_t ml[8], mh[8];
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const uint32_t f0 = b0[w] >> (2 * p), f1 = b1[w] >> (2 * p); // bit 0 of a byte: sub-block 2p, bit 1: 2p + 1
            ml[w] = (q0[w] & 0x0F0F0F0Fu) | ((f0 & 0x01010101u) << 4);
            mh[w] = ((q0[w] >> 4) & 0x0F0F0F0Fu) | ((f0 & 0x02020202u) << 3);
            ml[4 + w] = (q1[w] & 0x0F0F0F0Fu) | ((f1 & 0x01010101u) << 4);
            mh[4 + w] = ((q1[w] >> 4) & 0x0F0F0F0Fu) | ((f1 & 0x02020202u) << 3);
        }
#pragma unroll
        for (int w = 0; w < 8; w++) {
            lo = mfma(x.a[w], ml[w], lo);
            hi = mfma(x.a[8 + w], mh[w], hi);
        }
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
        const float d = f16lo(r.h.x), dmin = f16hi(r.h.x);
        const float s0 = d * ub0(scp), s1 = d * ub1(scp);
        float y = fmaf(s0, recombine(lo, x.sg[0]), s1 * recombine(hi, x.sg[1]));
        y = fmaf(fmaf(16.0f, s0, -(dmin * ub0(mp))), x.xs[0], y);
        y = fmaf(fmaf(16.0f, s1, -(dmin * ub1(mp))), x.xs[1], y);
        return y;
    }
};

// Q4_0 / Q4_1 (reference nibble order, types.rs:179-198: byte i = elements 2i, 2i+1).  The lane's
// two groups are the 32-element blocks c*2 and c*2+1... taken 16 blocks apart so that one load
// instruction reads 256 contiguous bytes per row.
template <bool WITH_MIN>
struct DQ4x {
    struct Raw { uint4 q[2]; uint32_t m[2]; };
    static constexpr bool X_REQUESTS_FIRST = true; // gemv_dpw_kernel: a barrier between the waves' x requests and their weight requests
    static constexpr bool TWO_SLICE_WAVES = false;
    static constexpr bool RUNS16 = false, OWN_META_PIECES = false;
    static constexpr bool PERM_A = true; // dword w of a block: low nibbles = elements 8w+{0,2,4,6}, high = 8w+{1,3,5,7}
    static constexpr int CENTRE = 8;
    static constexpr int BIG_NB = 4;
    static constexpr bool ROUND_META = true;
    static constexpr int META_SLICE_BYTES = WITH_MIN ? 128 : 64; // 32 blocks' scales (and minimums)
    __host__ __device__ static int meta_row_bytes(int k) { return (k >> 5) * (WITH_MIN ? 4 : 2); }
    __device__ static void load_codes(const Bases &b, const RowOff &ro, const LaneOff &o, Raw &r) {
        r.q[0] = ld16(b.codes, ro.c + o.c[0]);
        r.q[1] = ld16(b.codes, ro.c + o.c[1]);
    }
    __device__ static void set_meta(Raw &r, const uint8_t *row, int, int c) {
#pragma unroll
        for (int g = 0; g < 2; g++) {
            const int b = g * 16 + (c & 15); // the block inside the slice
            r.m[g] = WITH_MIN ? *reinterpret_cast<const uint32_t *>(row + b * 4) : *reinterpret_cast<const uint16_t *>(row + b * 2);
        }
    }
    __device__ static int blk_index(int c, int g) { return ((c >> 4) << 5) + g * 16 + (c & 15); }
    __device__ static int group_k(int c, int g) { return blk_index(c, g) * 32; }
    __device__ static void lane_offsets(int k, int c, LaneOff &o) {
        const int nblk = k >> 5;
#pragma unroll
        for (int g = 0; g < 2; g++) {
            int b = blk_index(c, g);
            b = b < nblk ? b : nblk - 1;
            o.c[g] = (uint32_t)b * 16;
            o.m[g] = (uint32_t)b * (WITH_MIN ? 4 : 2);
        }
    }
    __device__ static void load(const Bases &b, const RowOff &ro, const LaneOff &o, Raw &r) {
#pragma unroll
        for (int g = 0; g < 2; g++) {
            r.q[g] = ld16(b.codes, ro.c + o.c[g]);
            r.m[g] = WITH_MIN ? ld4(b.meta, ro.m + o.m[g]) : ld2(b.meta, ro.m + o.m[g]);
        }
    }
    __device__ static float dot(const Raw &r, const XOp &x, int) {
        float tot = 0.f;
#pragma unroll
        for (int g = 0; g < 2; g++) {
            const uint32_t q[4] = {r.q[g].x, r.q[g].y, r.q[g].z, r.q[g].w};
            int4v e = x.init[g], o = {0, 0, 0, 0};
#pragma unroll
            for (int w = 0; w < 4; w++) {
                e = mfma(x.a[8 * g + 2 * w], q[w] & 0x0F0F0F0Fu, e);
                o = mfma(x.a[8 * g + 2 * w + 1], (q[w] >> 4) & 0x0F0F0F0Fu, o);
            }
            float acc = recombine(e + o, x.sg[g]); // sum (n - 8) x
            float scale = f16lo(r.m[g]);
            if (WITH_MIN) tot += fmaf(scale, acc, fmaf(8.0f, scale, f16hi(r.m[g])) * x.xs[g]);
            else tot += scale * acc;
        }
        return tot;
    }
};

// Q5_0 / Q5_1 (GGUF): byte j = elements j (low nibble) and j+16 (high); qh bit e = bit 4 of element e.
template <bool WITH_MIN>
struct DQ5x {
    struct Raw { uint4 q[2]; uint32_t qh[2]; uint32_t m[2]; };
    static constexpr bool X_REQUESTS_FIRST = false; // gemv_dpw_kernel: a barrier between the waves' x requests and their weight requests
    static constexpr bool TWO_SLICE_WAVES = false;
    static constexpr bool RUNS16 = false, OWN_META_PIECES = false;
    static constexpr bool PERM_A = false;
    static constexpr int CENTRE = 16;
    static constexpr int BIG_NB = 4;
    static constexpr bool ROUND_META = true;
    static constexpr int META_SLICE_BYTES = WITH_MIN ? 128 : 64;
    __host__ __device__ static int meta_row_bytes(int k) { return (k >> 5) * (WITH_MIN ? 4 : 2); }
    __device__ static void load_codes(const Bases &b, const RowOff &ro, const LaneOff &o, Raw &r) {
#pragma unroll
        for (int g = 0; g < 2; g++) {
            r.q[g] = ld16(b.codes, ro.c + o.c[g]);
            r.qh[g] = ld4(b.qh, ro.h + o.h[g]);
        }
    }
    __device__ static void set_meta(Raw &r, const uint8_t *row, int, int c) {
#pragma unroll
        for (int g = 0; g < 2; g++) {
            const int b = g * 16 + (c & 15);
            r.m[g] = WITH_MIN ? *reinterpret_cast<const uint32_t *>(row + b * 4) : *reinterpret_cast<const uint16_t *>(row + b * 2);
        }
    }
    __device__ static int blk_index(int c, int g) { return ((c >> 4) << 5) + g * 16 + (c & 15); }
    __device__ static int group_k(int c, int g) { return blk_index(c, g) * 32; }
    __device__ static void lane_offsets(int k, int c, LaneOff &o) {
        const int nblk = k >> 5;
#pragma unroll
        for (int g = 0; g < 2; g++) {
            int b = blk_index(c, g);
            b = b < nblk ? b : nblk - 1;
            o.c[g] = (uint32_t)b * 16;
            o.h[g] = (uint32_t)b * 4;
            o.m[g] = (uint32_t)b * (WITH_MIN ? 4 : 2);
        }
    }
    __device__ static void load(const Bases &b, const RowOff &ro, const LaneOff &o, Raw &r) {
#pragma unroll
        for (int g = 0; g < 2; g++) {
            r.q[g] = ld16(b.codes, ro.c + o.c[g]);
            r.qh[g] = ld4(b.qh, ro.h + o.h[g]);
            r.m[g] = WITH_MIN ? ld4(b.meta, ro.m + o.m[g]) : ld2(b.meta, ro.m + o.m[g]);
        }
    }
    __device__ static float dot(const Raw &r, const XOp &x, int) {
        float tot = 0.f;
#pragma unroll
        for (int g = 0; g < 2; g++) {
            const uint32_t q[4] = {r.q[g].x, r.q[g].y, r.q[g].z, r.q[g].w};
            int4v lo = x.init[g], hi = {0, 0, 0, 0};
#pragma unroll
            for (int w = 0; w < 4; w++) {
                // spread 4 bits of qh to bit 4 of each byte: t * 0x00204081 puts bit i at bit 8i
                uint32_t bl = (((r.qh[g] >> (4 * w)) & 0xFu) * 0x00204081u) & 0x01010101u;
                uint32_t bh = (((r.qh[g] >> (16 + 4 * w)) & 0xFu) * 0x00204081u) & 0x01010101u;
                lo = mfma(x.a[8 * g + w], (q[w] & 0x0F0F0F0Fu) | (bl << 4), lo);
                hi = mfma(x.a[8 * g + 4 + w], ((q[w] >> 4) & 0x0F0F0F0Fu) | (bh << 4), hi);
            }
            float acc = recombine(lo + hi, x.sg[g]); // sum (u - 16) x
            float d = f16lo(r.m[g]);
            if (WITH_MIN) tot += fmaf(d, acc, fmaf(16.0f, d, f16hi(r.m[g])) * x.xs[g]);
            else tot += d * acc;
        }
        return tot;
    }
};

// Q8_0: four 16-byte vectors of int8 codes per lane per pass = two blocks; the codes are the B operand as they are.
struct DQ80 {
    struct Raw { uint4 q[4]; uint32_t m[2]; };
    static constexpr bool X_REQUESTS_FIRST = false; // gemv_dpw_kernel: a barrier between the waves' x requests and their weight requests
    // K beyond eight slices: the split-wave kernel with two slices per weight wave (4096 x 14336: 14.0 against 19.0 us on the
    // kernel with per-wave staging, whose ring holds three of these steps; every other type is ahead there, 8.9 against 9.7 us for Q4_K)
    static constexpr bool TWO_SLICE_WAVES = true;
    static constexpr bool RUNS16 = false, OWN_META_PIECES = false;
    static constexpr bool PERM_A = false;
    static constexpr int CENTRE = 0;
    static constexpr int BIG_NB = 3;
    static constexpr bool ROUND_META = true;
    static constexpr int META_SLICE_BYTES = 64;
    __host__ __device__ static int meta_row_bytes(int k) { return (k >> 5) * 2; }
    __device__ static void load_codes(const Bases &b, const RowOff &ro, const LaneOff &o, Raw &r) {
#pragma unroll
        for (int g = 0; g < 2; g++) {
            r.q[2 * g] = ld16(b.codes, ro.c + o.c[g]);
            r.q[2 * g + 1] = ld16(b.codes, ro.c + o.c[g] + 16);
        }
    }
    __device__ static void set_meta(Raw &r, const uint8_t *row, int, int c) {
#pragma unroll
        for (int g = 0; g < 2; g++) r.m[g] = *reinterpret_cast<const uint16_t *>(row + (g * 16 + (c & 15)) * 2);
    }
    // 16-byte vector v (0..3) of chunk c: vector index along the row; block = vector / 2
    __device__ static int vec_index(int c, int v) { return ((c >> 4) << 6) + (v >> 1) * 32 + (c & 15) * 2 + (v & 1); }
    __device__ static int group_k(int c, int g) { return vec_index(c, 2 * g) * 16; }
    __device__ static void lane_offsets(int k, int c, LaneOff &o) {
        const int nvec = k >> 4;
#pragma unroll
        for (int g = 0; g < 2; g++) {
            int v0 = vec_index(c, 2 * g);
            v0 = v0 < nvec ? v0 : nvec - 2;
            o.c[g] = (uint32_t)v0 * 16;
            o.m[g] = (uint32_t)(v0 >> 1) * 2;
        }
    }
    __device__ static void load(const Bases &b, const RowOff &ro, const LaneOff &o, Raw &r) {
#pragma unroll
        for (int g = 0; g < 2; g++) {
            r.q[2 * g] = ld16(b.codes, ro.c + o.c[g]);
            r.q[2 * g + 1] = ld16(b.codes, ro.c + o.c[g] + 16);
            r.m[g] = ld2(b.meta, ro.m + o.m[g]);
        }
    }
    __device__ static float dot(const Raw &r, const XOp &x, int) {
        float tot = 0.f;
#pragma unroll
        for (int g = 0; g < 2; g++) {
            const uint32_t q[8] = {r.q[2 * g].x, r.q[2 * g].y, r.q[2 * g].z, r.q[2 * g].w,
                                   r.q[2 * g + 1].x, r.q[2 * g + 1].y, r.q[2 * g + 1].z, r.q[2 * g + 1].w};
            int4v e = {0, 0, 0, 0}, o = {0, 0, 0, 0};
#pragma unroll
            for (int w = 0; w < 4; w++) {
                e = mfma(x.a[8 * g + 2 * w], q[2 * w], e);
                o = mfma(x.a[8 * g + 2 * w + 1], q[2 * w + 1], o);
            }
            tot += f16lo(r.m[g]) * recombine(e + o, x.sg[g]);
        }
        return tot;
    }
};

// Q6_K (GGUF, planes in ggml's order: ql 128 bytes, qh 64 bytes per superblock; meta row = int8 scales 16 bytes per
// superblock, then the f16 d of every superblock).  A 16-byte piece of ql holds two runs of 16 weights 64 apart (low and
// high nibbles) with one scale each; their bit pairs lie in one 16-byte piece of qh.  A lane takes piece `blk` and piece
// `blk + 16` of its wave's 1024-wide K slice (32 pieces), so that either load instruction reads 256 contiguous bytes of
// each row: four runs of 16, four accumulators, four scales.  The slice has 16 pieces of bit pairs, each wanted by two
// lanes: lane blk loads piece blk (one instruction, 256 contiguous bytes per row, nothing twice) and the lanes of a row
// hand each other the two pieces they need when the step is folded.  The codes go in as signed bytes q - 32.
struct DQ6K {
    struct Raw { uint4 l0, l1, hq; uint32_t sc; uint32_t d; };
    static constexpr bool X_REQUESTS_FIRST = false; // gemv_dpw_kernel: a barrier between the waves' x requests and their weight requests
    static constexpr bool TWO_SLICE_WAVES = false;
    static constexpr bool RUNS16 = true, OWN_META_PIECES = true;
    static constexpr bool PERM_A = false;
    static constexpr int CENTRE = 0;
    static constexpr int BIG_NB = 4;
    static constexpr bool ROUND_META = true;
    static constexpr int META_SLICE_BYTES = 128; // per row and slice in LDS: 64 bytes of scales, the 16-byte piece with its four d (four times)
    __host__ __device__ static int meta_row_bytes(int k) { return (k >> 8) * 16 + ((((k >> 8) * 2) + 15) & ~15); }
    __device__ static int meta_piece(int k, int slice, int piece, bool &from_qh) {
        const int nsb = k >> 8;
        from_qh = false;
        if (piece < 4) {
            const int off = slice * 64 + piece * 16;
            return off + 16 <= nsb * 16 ? off : nsb * 16 - 16;
        }
        return nsb * 16 + ((slice * 8) & ~15);
    }
    // piece P (0..31) of a slice: superblock P / 8 of the slice, half n = (P / 4) % 2, h = P % 4; its runs are sub-blocks
    // 8n + h (low nibbles, elements 128n + 16h ..) and 8n + 4 + h (high nibbles, 64 elements on)
    __device__ static int run_k(int c, int r) {
        const int P = (c & 15) + (r >> 1) * 16;
        return (c >> 4) * 1024 + (P >> 3) * 256 + ((P >> 2) & 1) * 128 + (P & 3) * 16 + (r & 1) * 64;
    }
    __device__ static int group_k(int c, int g) { return run_k(c, 2 * g); } // not used by RUNS16 types
    __device__ static void lane_offsets(int k, int c, LaneOff &o) {
        const int ql_bytes = k >> 1, qh_bytes = k >> 2;
        const int blk = c & 15, slice = c >> 4;
        const int l0 = slice * 512 + blk * 16, l1 = l0 + 256, h0 = slice * 256 + blk * 16;
        o.c[0] = (uint32_t)(l0 + 16 <= ql_bytes ? l0 : ql_bytes - 16); // pieces past the row's end meet x = 0
        o.c[1] = (uint32_t)(l1 + 16 <= ql_bytes ? l1 : ql_bytes - 16);
        o.h[0] = (uint32_t)(h0 + 16 <= qh_bytes ? h0 : qh_bytes - 16);
        // without per-round records: the first scale byte and the d of either piece
        const int nsb = k >> 8, in_sb = ((blk >> 2) & 1) * 8 + (blk & 3);
        int sb0 = slice * 4 + (blk >> 3), sb1 = sb0 + 2;
        sb0 = sb0 < nsb ? sb0 : nsb - 1;
        sb1 = sb1 < nsb ? sb1 : nsb - 1;
        o.m[0] = (uint32_t)(sb0 * 16 + in_sb);
        o.m[1] = (uint32_t)(sb1 * 16 + in_sb);
        o.d[0] = (uint32_t)(nsb * 16 + sb0 * 2);
        o.d[1] = (uint32_t)(nsb * 16 + sb1 * 2);
    }
    __device__ static void load_codes(const Bases &b, const RowOff &ro, const LaneOff &o, Raw &r) {
        r.l0 = ld16(b.codes, ro.c + o.c[0]);
        r.l1 = ld16(b.codes, ro.c + o.c[1]);
        r.hq = ld16(b.qh, ro.h + o.h[0]);
    }
    // row: this row's 128 bytes of the wave's patch (scales of the slice's four superblocks, then the piece with the d's)
    __device__ static void set_meta(Raw &r, const uint8_t *row, int, int c) {
        const int blk = c & 15, slice = c >> 4;
        const int sbl = blk >> 3, n8 = ((blk >> 2) & 1) * 8, h = blk & 3;
        const uint8_t *s0 = row + sbl * 16 + n8 + h, *s1 = s0 + 32;
        r.sc = (uint32_t)s0[0] | ((uint32_t)s0[4] << 8) | ((uint32_t)s1[0] << 16) | ((uint32_t)s1[4] << 24);
        const uint16_t *d = reinterpret_cast<const uint16_t *>(row + 64 + (slice & 1) * 8) + sbl;
        r.d = (uint32_t)d[0] | ((uint32_t)d[2] << 16);
    }
    __device__ static void load(const Bases &b, const RowOff &ro, const LaneOff &o, Raw &r) {
        load_codes(b, ro, o, r);
        const uint8_t *m = b.meta + ro.m;
        r.sc = (uint32_t)m[o.m[0]] | ((uint32_t)m[o.m[0] + 4] << 8) | ((uint32_t)m[o.m[1]] << 16) | ((uint32_t)m[o.m[1] + 4] << 24);
        r.d = (uint32_t)*reinterpret_cast<const uint16_t *>(m + o.d[0]) | ((uint32_t)*reinterpret_cast<const uint16_t *>(m + o.d[1]) << 16);
    }
    __device__ static float dot(const Raw &r, const XOp &x, int c) {
        const uint32_t ql[2][4] = {{r.l0.x, r.l0.y, r.l0.z, r.l0.w}, {r.l1.x, r.l1.y, r.l1.z, r.l1.w}};
        // the bit pairs of piece P lie in piece (P / 8) * 4 + ((P / 4) % 2) * 2 + P % 2 of the slice's sixteen, those of piece
        // P + 16 eight pieces on: held by the lanes of this row (lane % 4) whose blk is that number
        const int lane = (int)(threadIdx.x & 63), blk = c & 15;
        const int src0 = ((((blk >> 3) * 4 + ((blk >> 2) & 1) * 2 + (blk & 1)) << 2) | (lane & 3)) << 2, src1 = src0 + (8 << 4); // byte addresses of lanes
        const int hq[4] = {(int)r.hq.x, (int)r.hq.y, (int)r.hq.z, (int)r.hq.w};
        uint32_t qh[2][4];
#pragma unroll
        for (int w = 0; w < 4; w++) {
            qh[0][w] = (uint32_t)__builtin_amdgcn_ds_bpermute(src0, hq[w]);
            qh[1][w] = (uint32_t)__builtin_amdgcn_ds_bpermute(src1, hq[w]);
        }
        const int sh = ((c >> 1) & 1) * 2; // bit pair h / 2 for the low-nibble run, two pairs on for the high-nibble run
        int4v acc[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
#pragma unroll
        for (int t = 0; t < 2; t++) {
            uint32_t bl[4], bh[4]; // the piece's eight B operands first, then its products
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const uint32_t f = qh[t][w] >> sh;
                const uint32_t ul = (ql[t][w] & 0x0F0F0F0Fu) | ((f & 0x03030303u) << 4);
                const uint32_t uh = ((ql[t][w] >> 4) & 0x0F0F0F0Fu) | (f & 0x30303030u);
                bl[w] = (ul + 0x60606060u) ^ 0x80808080u; // q - 32 as a signed byte, no carry between bytes
                bh[w] = (uh + 0x60606060u) ^ 0x80808080u;
            }
#pragma unroll
            for (int w = 0; w < 4; w++) {
                acc[2 * t] = mfma(x.a[8 * t + w], bl[w], acc[2 * t]);
                acc[2 * t + 1] = mfma(x.a[8 * t + 4 + w], bh[w], acc[2 * t + 1]);
            }
        }
        const float d0 = f16lo(r.d), d1 = f16hi(r.d);
        float y0 = (float)(int8_t)(r.sc & 0xFF) * recombine(acc[0], x.sg[0]);
        y0 = fmaf((float)(int8_t)((r.sc >> 8) & 0xFF), recombine(acc[1], x.sg[1]), y0);
        float y1 = (float)(int8_t)((r.sc >> 16) & 0xFF) * recombine(acc[2], x.sg[2]);
        y1 = fmaf((float)(int8_t)(r.sc >> 24), recombine(acc[3], x.sg[3]), y1);
        return fmaf(d0, y0, d1 * y1);
    }
};

// The 16-byte piece `piece` of the record that a round fetches per row and K slice: its byte offset in the row of the meta
// plane, or (from_qh) of the qh plane, for types that keep their high bits in the record as well.  Pieces past the end
// of a row that does not fill its last slice are moved back inside it (they serve lanes whose x is zero).
template <class T>
__device__ inline int record_piece(int k, int slice, int piece, bool &from_qh) {
    from_qh = false;
    if constexpr (T::OWN_META_PIECES) {
        return T::meta_piece(k, slice, piece, from_qh);
    } else {
        const int off = slice * T::META_SLICE_BYTES + piece * 16, row_bytes = T::meta_row_bytes(k);
        return off + 16 <= row_bytes ? off : row_bytes - 16;
    }
}

// Gather bytes {0,2} of lo and {0,2} of hi (sel = 0) or {1,3} of each (sel = 1)
__device__ inline int pick_alt(uint32_t lo, uint32_t hi, int sel) {
    return (int)__builtin_amdgcn_perm(hi, lo, sel ? 0x07050301u : 0x06040200u);
}

template <class T>
__device__ inline void fetch_xop(const uint8_t *planes, const uint4 *grp, int kpad, int k, int limb, int c, XOp &o) {
    if constexpr (T::RUNS16) { // four runs of 16: one 16-byte piece of the limb plane and the scale of its 32-element group each
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int kb = T::run_k(c, r);
            uint4 u = {0, 0, 0, 0};
            o.sg[r] = 0.f;
            if (kb < k) {
                u = *reinterpret_cast<const uint4 *>(planes + (size_t)limb * kpad + kb);
                o.sg[r] = __builtin_bit_cast(float, grp[kb >> 5].x);
            }
            o.a[4 * r] = (int)u.x; o.a[4 * r + 1] = (int)u.y; o.a[4 * r + 2] = (int)u.z; o.a[4 * r + 3] = (int)u.w;
        }
        o.xs[0] = o.xs[1] = 0.f;
        o.init[0] = o.init[1] = int4v{0, 0, 0, 0};
        return;
    }
#pragma unroll
    for (int g = 0; g < 2; g++) {
        int kb = T::group_k(c, g);
        uint32_t nat[8];
        if (kb < k) { // groups past the end of the row contribute nothing
            const uint4 *p = reinterpret_cast<const uint4 *>(planes + (size_t)limb * kpad + kb);
            uint4 u = p[0], v = p[1];
            nat[0] = u.x; nat[1] = u.y; nat[2] = u.z; nat[3] = u.w; nat[4] = v.x; nat[5] = v.y; nat[6] = v.z; nat[7] = v.w;
            uint4 sv = grp[kb >> 5];
            o.sg[g] = __builtin_bit_cast(float, sv.x);
            o.xs[g] = __builtin_bit_cast(float, sv.y);
            o.init[g][0] = -T::CENTRE * ((int)(sv.z << 16) >> 16);
            o.init[g][1] = -T::CENTRE * ((int)sv.z >> 16);
            o.init[g][2] = -T::CENTRE * ((int)(sv.w << 16) >> 16);
            o.init[g][3] = -T::CENTRE * ((int)sv.w >> 16);
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) nat[i] = 0;
            o.sg[g] = 0.f;
            o.xs[g] = 0.f;
            o.init[g] = int4v{0, 0, 0, 0};
        }
        if (T::PERM_A) {
#pragma unroll
            for (int w = 0; w < 4; w++) {
                o.a[8 * g + 2 * w] = pick_alt(nat[2 * w], nat[2 * w + 1], 0);
                o.a[8 * g + 2 * w + 1] = pick_alt(nat[2 * w], nat[2 * w + 1], 1);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) o.a[8 * g + i] = (int)nat[i];
        }
    }
}

// Sum over the four k-chunks of each 16-lane DPP row (lanes with equal lane % 4): lanes 12..15 of every
// row end with that row's four totals.  The four DPP rows are added later, from LDS.
__device__ inline float sum_within_row(float v) {
    int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x114, 0xf, 0xf, true); // row_shr:4
    v += __builtin_bit_cast(float, t);
    t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x118, 0xf, 0xf, true); // row_shr:8
    v += __builtin_bit_cast(float, t);
    return v;
}

// ---------------------------------------------------------------------------
// The kernel.  A workgroup is G row groups of S waves; wave `slice` of a group covers k-chunks
// [16*slice, 16*slice+16) of the row (1024 weights), so S = ceil(K / 1024) waves span K once.  A group
// owns `steps` consecutive 4-row steps; each wave keeps a ring of NB of them in flight and refills a slot
// as soon as it has been folded.
//
// Waves issue in order, a load that finds the memory pipeline full blocks its wave, and the pipeline is one
// queue per compute unit.  So the order of the first instructions decides the ramp: every wave requests x
// (or its split form) first, a barrier keeps all weight requests behind all x requests, and the split of x
// runs while the first weights are on their way.
// ---------------------------------------------------------------------------
__device__ inline void lds_only_barrier() {
    // __syncthreads() would also wait for the weight loads in flight
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ---------------------------------------------------------------------------
// RND: the scale records fetched once per round of up to four row steps (Q4_K from a raw x takes this route).
//
// A compute unit keeps about 64 vector memory instructions in flight, whatever they fetch (a wave that finds them
// taken waits at its next load and does nothing else), and the stream runs at (bytes in flight) / latency.  A Q4_K
// header load has four lanes on each 16 bytes and so fetches 256 bytes where a code load fetches 1024: one in three
// places in flight was spent on one ninth of the bytes.  With RND one load per round fetches the headers of all its
// 16 rows (lane = row and superblock), the wave parks them in an LDS patch of its own, and every fold reads its
// header from there: nine loads of 1 KB per round instead of twelve.  The ring is then four steps deep: 8 waves x 4
// steps x 2 loads fill the compute unit's 64 places, and no refill waits.
// ---------------------------------------------------------------------------
template <class T, int NB, bool PRE, bool RND>
__global__ void __launch_bounds__(NB > T::BIG_NB ? 512 : 1024) gemv_dp_kernel(DP_KERNEL_PARAMS) {
    const DpArgs a = DP_KERNEL_ARGS;
    static_assert(!RND || (!PRE && T::ROUND_META && NB <= 4), "per-round scale records: a raw x, a type that has them, at most four steps per round");
    constexpr int MSB = T::META_SLICE_BYTES, NM = MSB / 64, CPR = MSB / 16; // scale loads per round, 16-byte chunks per row
    extern __shared__ uint4 lds_raw[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g_idx = wave / a.S, slice = wave - g_idx * a.S;
    const int blk = lane >> 2, j = lane & 3;
    const int c = (slice << 4) + blk; // this lane's 64-weight chunk of the row

    // LDS: the split form of x (limb planes, then group records), then the reduction buffer
    uint8_t *wplanes = reinterpret_cast<uint8_t *>(lds_raw);
    const int kpad = (a.k + 15) & ~15;
    uint4 *wgrp = reinterpret_cast<uint4 *>(wplanes + (size_t)4 * kpad);
    const int n16 = (int)(axq_split_bytes(a.k) >> 4);
    // one spare 16-byte slot takes the surplus stores of step 3, 64 bytes hold per-wave sums of a fused RMSNorm
    float *red = reinterpret_cast<float *>(lds_raw + n16 + 1 + 4);
    const int rows_per_group = a.steps * 4;
    const int last = a.n_rows - 1;
    const int red_stride = 4 * a.S; // partial sums per output row in the LDS reduction buffer
    float *red_lane = red + (g_idx * rows_per_group + j) * red_stride + slice * 4 + (lane >> 4);
    const int nthreads = (int)blockDim.x;
    // this wave's patch of scale records: 64 * NM x 16 bytes behind the reduction buffer
    uint4 *wmeta = lds_raw + n16 + 1 + 4 + (a.G * rows_per_group * red_stride) / 4 + wave * 64 * NM;

    // 1. x first.  The compute unit's memory pipeline is one queue for all its waves, so the barrier makes
    //    sure that no wave's x request stands behind another wave's weight requests.  A thread fetches one
    //    8-element split task of raw x, and a second one where K exceeds eight elements per thread (K <= 16 per thread by
    //    construction of the launch): a load nobody needs would still take a place in the pipeline.  Of an x that arrives
    //    already split it fetches at most five 16-byte pieces.
    const uint4 zero4 = {0, 0, 0, 0};
    uint4 x0, x1, x2 = zero4, x3 = zero4, x4 = zero4;
    uint4 e0 = zero4, e1 = zero4, e2 = zero4, e3 = zero4; // second operand of a fused prologue
    const int ntask = a.k >> 3; // K is a multiple of 64 here: whole quads of tasks
    const bool second = nthreads < ntask;
    if (PRE) {
        const uint4 *src = reinterpret_cast<const uint4 *>(a.xq);
        auto piece = [&](int u) { int i = tid + u * nthreads; return src[i < n16 ? i : 0]; };
        x0 = piece(0); x1 = piece(1); x2 = piece(2); x3 = piece(3); x4 = piece(4);
    } else {
        auto half = [&](const float *src, int u, int h) {
            int t = tid + u * nthreads;
            t = t < ntask ? t : (t & 3);
            return reinterpret_cast<const uint4 *>(src + (size_t)t * 8)[h];
        };
        x0 = half(a.x, 0, 0); x1 = half(a.x, 0, 1);
        if (second) { x2 = half(a.x, 1, 0); x3 = half(a.x, 1, 1); }
        if (a.mode != AXQ_X_PLAIN) {
            e0 = half(a.aux, 0, 0); e1 = half(a.aux, 0, 1);
            if (second) { e2 = half(a.aux, 1, 0); e3 = half(a.aux, 1, 1); }
        }
    }
    __builtin_amdgcn_s_barrier();
    // 2. the ring: rows past the group's end re-read its first step (cache hits, no HBM traffic)
    typename T::Raw buf[NB];
    uint4 hm[NM];
    LaneOff lo;
    T::lane_offsets(a.k, c, lo);
    const int wg_row0 = blockIdx.x * a.G * rows_per_group;
    const Bases bases = {a.codes + (size_t)wg_row0 * a.codes_pitch, a.meta + (size_t)wg_row0 * a.meta_pitch,
                         a.qh + (size_t)wg_row0 * a.qh_pitch};
    const uint32_t cp = (uint32_t)a.codes_pitch, mp = (uint32_t)a.meta_pitch, qp = (uint32_t)a.qh_pitch;
    const int rl0 = g_idx * rows_per_group + j, rl_last = last - wg_row0; // rows relative to the workgroup's first
    // scale loads of a round (RND): 64 * NM lanes = (row of the round's 16, 16-byte chunk of the slice's MSB bytes); chunks past
    // the row's end (a last slice that is not whole) are moved back inside it: they serve lanes whose x is zero
    uint32_t moff[NM], mpitch[NM];
    const uint8_t *mbase[NM];
    int mrl0[NM];
    {
#pragma unroll
        for (int i = 0; i < NM; i++) {
            const int flat = i * 64 + lane;
            bool from_qh;
            moff[i] = (uint32_t)record_piece<T>(a.k, slice, flat % CPR, from_qh);
            mbase[i] = from_qh ? bases.qh : bases.meta;
            mpitch[i] = from_qh ? qp : mp;
            mrl0[i] = g_idx * rows_per_group + flat / CPR;
        }
    }
    auto request = [&](int step, int b) {
        const int s = step < a.steps ? step : 0;
        int rl = rl0 + 4 * s;
        rl = rl < rl_last ? rl : rl_last;
        const RowOff ro = {(uint32_t)rl * cp, (uint32_t)rl * mp, (uint32_t)rl * qp};
        if constexpr (RND) {
            if (b == 0) { // rows past the group's steps belong to the next group or repeat the matrix's last row: read, not used
#pragma unroll
                for (int i = 0; i < NM; i++) {
                    int rlm = mrl0[i] + 4 * s;
                    rlm = rlm < rl_last ? rlm : rl_last;
                    hm[i] = ld16(mbase[i], (uint32_t)rlm * mpitch[i] + moff[i]);
                }
            }
            T::load_codes(bases, ro, lo, buf[b]);
        } else {
            T::load(bases, ro, lo, buf[b]);
        }
    };
    // steps requested before x is staged: enough to start the stream, few enough that no wave is still held up issuing them
    // when the others want to pass the barrier.  With per-round records three: x (two loads) and the record load make nine
    // places per wave, a few more than the compute unit holds -- x comes back first and makes room.
    constexpr int NB0 = NB < (RND ? 3 : 2) ? NB : (RND ? 3 : 2);
#pragma unroll
    for (int b = 0; b < NB0; b++) request(b, b);
    // 3. x -> LDS in split form -> this lane's A operands, while the weights are on their way
    if (PRE) {
        auto put = [&](int u, const uint4 &v) { int i = tid + u * nthreads; lds_raw[i < n16 ? i : n16] = v; };
        put(0, x0); put(1, x1); put(2, x2); put(3, x3); put(4, x4);
    } else {
        auto unpack = [](const uint4 &lo, const uint4 &hi, float (&v)[8]) {
            v[0] = __builtin_bit_cast(float, lo.x); v[1] = __builtin_bit_cast(float, lo.y);
            v[2] = __builtin_bit_cast(float, lo.z); v[3] = __builtin_bit_cast(float, lo.w);
            v[4] = __builtin_bit_cast(float, hi.x); v[5] = __builtin_bit_cast(float, hi.y);
            v[6] = __builtin_bit_cast(float, hi.z); v[7] = __builtin_bit_cast(float, hi.w);
        };
        float xv[2][8], ev[2][8];
        unpack(x0, x1, xv[0]);
        unpack(x2, x3, xv[1]);
        const bool live0 = tid < ntask, live1 = tid + nthreads < ntask; // whole quads of lanes: K is a multiple of 64
        if (a.mode == AXQ_X_RMSNORM) {
            // RMSNorm::forward (llm/src/llama.rs:158-187) of the whole vector, by every workgroup for itself
            unpack(e0, e1, ev[0]);
            unpack(e2, e3, ev[1]);
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                if (live0) ss = fmaf(xv[0][i], xv[0][i], ss);
                if (live1) ss = fmaf(xv[1][i], xv[1][i], ss);
            }
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m);
            float *wsum = reinterpret_cast<float *>(lds_raw + n16 + 1); // 16 floats kept for this between x and `red`
            if (lane == 0) wsum[wave] = ss; // read after the final barrier: 1 / rms is a factor on the result
#pragma unroll
            for (int i = 0; i < 8; i++) {
                xv[0][i] *= ev[0][i];
                xv[1][i] *= ev[1][i];
            }
        }
        if (live0) axq_split8(xv[0], tid, true, wplanes, wgrp, kpad);
        if (live1) axq_split8(xv[1], tid + nthreads, true, wplanes, wgrp, kpad);
    }
    lds_only_barrier(); // not __syncthreads(): that would also wait for the weights in flight
    XOp xo;
    fetch_xop<T>(wplanes, wgrp, kpad, a.k, j, c, xo);
#pragma unroll
    for (int b = NB0; b < NB; b++) request(b, b);

    // 4. fold the steps through the ring
    const bool writer = (blk & 3) == 3;
    const int red_step = 4 * red_stride;
    auto fold = [&](int b, int step) {
        if constexpr (RND) {
            if (b == 0) { // the wave's own patch: LDS serves a wave's stores and loads in order
#pragma unroll
                for (int i = 0; i < NM; i++) wmeta[i * 64 + lane] = hm[i];
            }
            T::set_meta(buf[b], reinterpret_cast<const uint8_t *>(wmeta) + (b * 4 + j) * MSB, blk, c);
        }
        float tot = sum_within_row(T::dot(buf[b], xo, c));
        if (writer) red_lane[step * red_step] = tot;
    };
    const int rounds = (a.steps + NB - 1) / NB;
    int step = 0;
    for (int round = 0; round < rounds - 1; round++, step += NB) {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            fold(b, step + b);
            request(step + NB + b, b);
        }
    }
#pragma unroll
    for (int b = 0; b < NB; b++)
        if (step + b < a.steps) fold(b, step + b); // the last round may be short: its spare slots hold re-reads

    // partial sums -> y, in a fixed order
    __syncthreads();
    const int wg_rows = a.G * rows_per_group;
    float inv = 1.0f;
    if (!PRE && a.mode == AXQ_X_RMSNORM) {
        const float *wsum = reinterpret_cast<const float *>(lds_raw + n16 + 1);
        float tot = 0.f;
        for (int i = 0; i < (nthreads >> 6); i++) tot += wsum[i];
        inv = 1.0f / sqrtf(tot / (float)a.k + a.eps);
    }
    auto row_total = [&](int t) { // slice by slice, the four DPP rows of each in order
        const float4 *pr = reinterpret_cast<const float4 *>(red + (size_t)t * red_stride);
        float tot = 0.f;
        for (int s = 0; s < a.S; s++) {
            float4 v = pr[s];
            tot += (v.x + v.y) + (v.z + v.w);
        }
        return tot * inv;
    };
    if (a.ymode == AXQ_Y_SWIGLU) {
        // rows 8b..8b+3 are gate rows, 8b+4..8b+7 the up rows of the same outputs (wg_rows is a multiple of 8)
        for (int t = tid; t < (wg_rows >> 1); t += nthreads) {
            const int lg = ((t >> 2) << 3) + (t & 3);
            const int row = blockIdx.x * wg_rows + lg;
            if (row + 4 < a.n_rows) {
                const float g = row_total(lg), u = row_total(lg + 4);
                a.y[(blockIdx.x * wg_rows >> 1) + t] = (g * (1.0f / (1.0f + expf(-g)))) * u;
            }
        }
        return;
    }
    for (int t = tid; t < wg_rows; t += nthreads) {
        int row = blockIdx.x * wg_rows + t;
        if (row < a.n_rows) {
            const float tot = row_total(t);
            a.y[row] = a.bias ? tot + a.bias[row] : tot;
        }
    }
}

#ifdef AXQ_STAMPS
// Development builds only (-DAXQ_STAMPS): every wave keeps wall-clock stamps (100 MHz) of its progress in LDS (the last
// 4 KB of the 160) and copies them out when it ends, into a buffer the host has set with axq_debug_set_stamps:
// [launch % 4][workgroup][wave (16)][slot (16)].
__device__ unsigned long long *axq_stamps;
__device__ unsigned int axq_stamp_launch;
#define STAMP_INIT() unsigned long long *st_lds_ = reinterpret_cast<unsigned long long *>(reinterpret_cast<uint8_t *>(lds_raw) + 156 * 1024) + wave * 16; \
                     if (lane < 16) st_lds_[lane] = 0
#define STAMP(slot) do { if (lane == 0) st_lds_[slot] = wall_clock64(); } while (0)
#define STAMP_END() do { unsigned long long *g_ = axq_stamps; if (g_ && lane < 16) { \
                         g_[((((size_t)(*(volatile unsigned int *)&axq_stamp_launch & 3) * gridDim.x + blockIdx.x) * 16 + wave) * 16) + lane] = st_lds_[lane]; } \
                         __syncthreads(); if (g_ && blockIdx.x == 0 && threadIdx.x == 0) atomicAdd(&axq_stamp_launch, 1u); } while (0)
#else
#define STAMP_INIT() do {} while (0)
#define STAMP(slot) do {} while (0)
#define STAMP_END() do {} while (0)
#endif

// ---------------------------------------------------------------------------
// The same kernel with x staged per wave.  Timestamps of the kernel above showed its critical path: x requested
// 0.4 us after entry, split by all waves together, two workgroup barriers (every wave waits for the one that was held
// up longest issuing its first weight requests) -- first fold 3.5 us after entry, then seven folds at the vector
// ALU's pace, 0.5 us each: latency and ALU in series, with the memory stream idling beside them.  Here a wave needs
// nobody: it fetches and splits the 1024 elements of x of its own K slice (the G row groups of a workgroup repeat
// that work, which costs less than the barriers did), keeps the split form in an LDS region of its own, and starts
// folding as soon as its own x and its first weights have arrived.  A fused RMSNorm needs the whole vector's sum
// of squares, but only as one factor on the result: y = inv_rms * sum_k W[n, k] (x[k] w[k]), so the waves split
// x[k] w[k] and leave their slices' sums of squares in LDS for the final reduction.
// ---------------------------------------------------------------------------
template <class T, int NB>
__global__ void __launch_bounds__(NB > T::BIG_NB ? 512 : 1024) gemv_dpw_kernel(DP_KERNEL_PARAMS) {
    const DpArgs a = DP_KERNEL_ARGS;
    extern __shared__ uint4 lds_raw[];
    constexpr int SLICE_K = 1024, REGION16 = (4 * SLICE_K + (SLICE_K / 32) * 16) / 16; // a wave's split x, in 16-byte units
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g_idx = wave / a.S, slice = wave - g_idx * a.S;
    const int blk = lane >> 2, j = lane & 3;
    const int c = (slice << 4) + blk; // this lane's 64-weight chunk of the row
    const int nwaves = a.G * a.S;
    const int k0 = slice * SLICE_K;
    const int klen = a.k - k0 < SLICE_K ? a.k - k0 : SLICE_K; // a multiple of 64
    STAMP_INIT();
    STAMP(0);

    // 1. x first: this wave's slice, two 8-element tasks per lane (and the norm weights of a fused RMSNorm)
    const bool live0 = lane * 8 < klen, live1 = (lane + 64) * 8 < klen; // whole quads of lanes
    const float *xs = a.x + k0 + (live0 ? lane * 8 : (lane & 3) * 8);
    const float *xs1 = a.x + k0 + (live1 ? (lane + 64) * 8 : (lane & 3) * 8);
    const uint4 x0 = reinterpret_cast<const uint4 *>(xs)[0], x1 = reinterpret_cast<const uint4 *>(xs)[1];
    const uint4 x2 = reinterpret_cast<const uint4 *>(xs1)[0], x3 = reinterpret_cast<const uint4 *>(xs1)[1];
    uint4 e0 = {0, 0, 0, 0}, e1 = e0, e2 = e0, e3 = e0;
    if (a.mode == AXQ_X_RMSNORM) {
        const float *es = a.aux + (xs - a.x), *es1 = a.aux + (xs1 - a.x);
        e0 = reinterpret_cast<const uint4 *>(es)[0]; e1 = reinterpret_cast<const uint4 *>(es)[1];
        e2 = reinterpret_cast<const uint4 *>(es1)[0]; e3 = reinterpret_cast<const uint4 *>(es1)[1];
    }
    // 2. the ring: rows past the group's end re-read its first step (cache hits, no HBM traffic)
    uint8_t *wplanes = reinterpret_cast<uint8_t *>(lds_raw + wave * REGION16);
    uint4 *wgrp = reinterpret_cast<uint4 *>(wplanes + 4 * SLICE_K);
    float *wsum = reinterpret_cast<float *>(lds_raw + nwaves * REGION16); // one float per wave (64 bytes kept)
    float *red = wsum + 16;
    const int rows_per_group = a.steps * 4;
    const int last = a.n_rows - 1;
    const int red_stride = 4 * a.S; // partial sums per output row in the LDS reduction buffer
    float *red_lane = red + (g_idx * rows_per_group + j) * red_stride + slice * 4 + (lane >> 4);
    typename T::Raw buf[NB];
    // T::ROUND_META (see gemv_dp_kernel's RND): one load of scale records per round of NB <= 4 steps, parked in an LDS patch of the wave
    constexpr bool ROUNDS = T::ROUND_META && NB <= 4;
    constexpr int MSB = T::META_SLICE_BYTES, NM = MSB / 64, CPR = MSB / 16; // loads per round, 16-byte chunks per row
    uint4 hm[NM];
    uint4 *wmeta = reinterpret_cast<uint4 *>(red + a.G * rows_per_group * red_stride) + wave * 64 * NM;
    LaneOff lo;
    T::lane_offsets(a.k, c, lo);
    const int wg_row0 = blockIdx.x * a.G * rows_per_group;
    const Bases bases = {a.codes + (size_t)wg_row0 * a.codes_pitch, a.meta + (size_t)wg_row0 * a.meta_pitch,
                         a.qh + (size_t)wg_row0 * a.qh_pitch};
    const uint32_t cp = (uint32_t)a.codes_pitch, mp = (uint32_t)a.meta_pitch, qp = (uint32_t)a.qh_pitch;
    const int rl0 = g_idx * rows_per_group + j, rl_last = last - wg_row0; // rows relative to the workgroup's first
    // header loads of a round: 64 * NM lanes = (row of the round's 16, 16-byte chunk of the slice's MSB bytes); chunks past the
    // row's end (a last slice that is not whole) are moved back inside it: they serve lanes whose x is zero
    uint32_t moff[NM], mpitch[NM];
    const uint8_t *mbase[NM];
    int mrl0[NM];
    {
#pragma unroll
        for (int i = 0; i < NM; i++) {
            const int flat = i * 64 + lane;
            bool from_qh;
            moff[i] = (uint32_t)record_piece<T>(a.k, slice, flat % CPR, from_qh);
            mbase[i] = from_qh ? bases.qh : bases.meta;
            mpitch[i] = from_qh ? qp : mp;
            mrl0[i] = g_idx * rows_per_group + flat / CPR;
        }
    }
    auto request = [&](int step, int b) {
        const int s = step < a.steps ? step : 0;
        int rl = rl0 + 4 * s;
        rl = rl < rl_last ? rl : rl_last;
        const RowOff ro = {(uint32_t)rl * cp, (uint32_t)rl * mp, (uint32_t)rl * qp};
        if constexpr (ROUNDS) {
            if (b == 0) { // rows past the group's steps: read, not used
#pragma unroll
                for (int i = 0; i < NM; i++) {
                    int rlm = mrl0[i] + 4 * s;
                    rlm = rlm < rl_last ? rlm : rl_last;
                    hm[i] = ld16(mbase[i], (uint32_t)rlm * mpitch[i] + moff[i]);
                }
            }
            T::load_codes(bases, ro, lo, buf[b]);
        } else {
            T::load(bases, ro, lo, buf[b]);
        }
    };
    // One step requested before x is split (two: 9.3 against 9.1 us at Q4_K 4096 x 14336; the stamps showed the workgroup's
    // last six waves standing 2.5-3.5 us at their first loads, behind the first eight waves' x and weight requests).  Types
    // with two loads per step gain again when every wave's x requests are out before any weight request (8.6-8.7 us).
    constexpr int NB0 = 1;
    if constexpr (T::X_REQUESTS_FIRST) __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int b = 0; b < NB0; b++) request(b, b);
    STAMP(1);
    // 3. x -> split form in the wave's own LDS region -> this lane's A operands
    {
        auto unpack = [](const uint4 &lo4, const uint4 &hi4, float (&v)[8]) {
            v[0] = __builtin_bit_cast(float, lo4.x); v[1] = __builtin_bit_cast(float, lo4.y);
            v[2] = __builtin_bit_cast(float, lo4.z); v[3] = __builtin_bit_cast(float, lo4.w);
            v[4] = __builtin_bit_cast(float, hi4.x); v[5] = __builtin_bit_cast(float, hi4.y);
            v[6] = __builtin_bit_cast(float, hi4.z); v[7] = __builtin_bit_cast(float, hi4.w);
        };
        float xv[2][8], ev[2][8];
        unpack(x0, x1, xv[0]);
        unpack(x2, x3, xv[1]);
        if (a.mode == AXQ_X_RMSNORM) {
            // RMSNorm::forward (llm/src/llama.rs:158-187): (x / rms) * w; the 1 / rms is applied to the result
            unpack(e0, e1, ev[0]);
            unpack(e2, e3, ev[1]);
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                if (live0) ss = fmaf(xv[0][i], xv[0][i], ss);
                if (live1) ss = fmaf(xv[1][i], xv[1][i], ss);
            }
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m);
            if (lane == 0) wsum[wave] = ss; // read after the final barrier (group 0's waves cover K once)
#pragma unroll
            for (int i = 0; i < 8; i++) {
                xv[0][i] *= ev[0][i];
                xv[1][i] *= ev[1][i];
            }
        }
        if (!live0) {
#pragma unroll
            for (int i = 0; i < 8; i++) xv[0][i] = 0.f;
        }
        if (!live1) {
#pragma unroll
            for (int i = 0; i < 8; i++) xv[1][i] = 0.f;
        }
        axq_split8(xv[0], lane, live0, wplanes, wgrp, SLICE_K);
        axq_split8(xv[1], lane + 64, live1, wplanes, wgrp, SLICE_K);
    }
    STAMP(2);
    XOp xo;
    fetch_xop<T>(wplanes, wgrp, SLICE_K, klen, j, blk, xo); // same wave: LDS serves its stores and loads in order
#pragma unroll
    for (int b = NB0; b < NB; b++) request(b, b);
    STAMP(4);

    // 4. fold the steps through the ring
    const bool writer = (blk & 3) == 3;
    const int red_step = 4 * red_stride;
    auto fold = [&](int b, int step) {
        if constexpr (ROUNDS) {
            if (b == 0) { // the wave's own patch: LDS serves a wave's stores and loads in order
#pragma unroll
                for (int i = 0; i < NM; i++) wmeta[i * 64 + lane] = hm[i];
            }
            T::set_meta(buf[b], reinterpret_cast<const uint8_t *>(wmeta) + (b * 4 + j) * MSB, blk, c);
        }
        float tot = sum_within_row(T::dot(buf[b], xo, c));
        if (writer) red_lane[step * red_step] = tot;
        STAMP(5 + (step < 8 ? step : 8));
    };
    const int rounds = (a.steps + NB - 1) / NB;
    int step = 0;
    for (int round = 0; round < rounds - 1; round++, step += NB) {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            fold(b, step + b);
            request(step + NB + b, b);
        }
    }
#pragma unroll
    for (int b = 0; b < NB; b++)
        if (step + b < a.steps) fold(b, step + b); // the last round may be short: its spare slots hold re-reads

    // partial sums -> y, in a fixed order
    __syncthreads();
    STAMP(14);
    const int nthreads = 64 * nwaves;
    const int wg_rows = a.G * rows_per_group;
    float inv = 1.0f;
    if (a.mode == AXQ_X_RMSNORM) {
        float tot = 0.f;
        for (int s = 0; s < a.S; s++) tot += wsum[s];
        inv = 1.0f / sqrtf(tot / (float)a.k + a.eps);
    }
    auto row_total = [&](int t) { // slice by slice, the four DPP rows of each in order
        const float4 *pr = reinterpret_cast<const float4 *>(red + (size_t)t * red_stride);
        float tot = 0.f;
        for (int s = 0; s < a.S; s++) {
            float4 v = pr[s];
            tot += (v.x + v.y) + (v.z + v.w);
        }
        return tot * inv;
    };
    if (a.ymode == AXQ_Y_SWIGLU) {
        // rows 8b..8b+3 are gate rows, 8b+4..8b+7 the up rows of the same outputs (wg_rows is a multiple of 8)
        for (int t = tid; t < (wg_rows >> 1); t += nthreads) {
            const int lg = ((t >> 2) << 3) + (t & 3);
            const int row = blockIdx.x * wg_rows + lg;
            if (row + 4 < a.n_rows) {
                const float g = row_total(lg), u = row_total(lg + 4);
                a.y[(blockIdx.x * wg_rows >> 1) + t] = (g * (1.0f / (1.0f + expf(-g)))) * u;
            }
        }
        STAMP(15);
        STAMP_END();
        return;
    }
    for (int t = tid; t < wg_rows; t += nthreads) {
        int row = blockIdx.x * wg_rows + t;
        if (row < a.n_rows) {
            const float tot = row_total(t);
            a.y[row] = a.bias ? tot + a.bias[row] : tot;
        }
    }
    STAMP(15);
    STAMP_END();
}


// ---------------------------------------------------------------------------
// The kernel with waves of two kinds.  Whoever splits x cannot request weights meanwhile, and whoever stands at a
// weight request (the compute unit's places for loads in flight taken) cannot split: in the kernels above x is split by
// the waves that also own the weights, and the memory pipeline drains while they do it.  Here a workgroup is NS
// "split" waves, which own no weights (they fetch x, split it -- two tasks per lane at K = 4096 -- and stage it in LDS),
// beside the G x S weight waves, which start requesting at once, three row steps and the round's scale records, and
// meet the split waves at one LDS-only barrier; from there on the ring runs as in gemv_dp_kernel with per-round
// records.  The split waves are the workgroup's first, so their requests for x stand in front of the weights'.  The
// workgroup's row steps are dealt to its G row groups in turn (group g takes steps g, g + G, ...).
//
// Scalar arguments instead of a struct passed by value: the first fourteen dwords are preloaded into scalar
// registers when the wave starts (the file is compiled with -amdgpu-kernarg-preload-count), so the pointers the first
// loads need are there without a trip to memory.
// ---------------------------------------------------------------------------
template <class T, int NB, int NB0, int NS, int KS = 1>
__global__ void __launch_bounds__(1024) gemv_sw_kernel(const float *__restrict__ x, const uint8_t *__restrict__ codes,
                                                               const uint8_t *__restrict__ meta, uint32_t cp, uint32_t mp, int n_rows, int k,
                                                               int steps, int flags, float eps, float *__restrict__ y,
                                                               const float *__restrict__ bias, const float *__restrict__ aux,
                                                               const uint8_t *__restrict__ qhp, uint32_t qp) {
    static_assert(T::ROUND_META && NB <= 8 && NB0 <= NB && NB0 >= 1, "per-round scale records; a ring of at most eight steps");
    // scale records of a round of NB steps: 4 NB rows x CPR 16-byte chunks of this wave's K slice, in NM loads of 64 lanes
    constexpr int MSB = T::META_SLICE_BYTES, CPR = MSB / 16, NM = (4 * NB * CPR + 63) / 64;
    constexpr int NST = 64 * NS, MAXT = 4;                                   // split threads; tasks of eight elements each of them takes at most
    extern __shared__ uint4 lds_raw[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int mode = flags & 0xFF, ymode = (flags >> 8) & 0xFF, G = (flags >> 16) & 0xFF;
    STAMP_INIT();
    STAMP(0);
    const int S = (k + 1023) >> 10;
    // LDS: the split form of x (limb planes, then group records), a spare slot, per-wave sums of a fused RMSNorm, the
    // reduction buffer, the weight waves' patches of scale records
    uint8_t *wplanes = reinterpret_cast<uint8_t *>(lds_raw);
    const int kpad = (k + 15) & ~15;
    uint4 *wgrp = reinterpret_cast<uint4 *>(wplanes + (size_t)4 * kpad);
    const int n16 = (int)(axq_split_bytes(k) >> 4);
    float *wsum = reinterpret_cast<float *>(lds_raw + n16 + 1);
    float *red = reinterpret_cast<float *>(lds_raw + n16 + 1 + 4);
    // `steps` 4-row steps per workgroup, dealt to its G row groups in turn: group g takes steps g, g + G, g + 2 G, ...
    const int wg_rows = steps * 4;
    const int red_stride = 4 * S; // partial sums per output row in the LDS reduction buffer

    if (wave < NS) {
        // ---- split waves: x (times the norm weights of a fused RMSNorm) -> split form in LDS
        const int ntask = k >> 3; // K is a multiple of 64: whole quads of tasks
        uint4 xa[MAXT], xb[MAXT], ea[MAXT], eb[MAXT];
#pragma unroll
        for (int u = 0; u < MAXT; u++) {
            if (u * NST < ntask) {
                int t = tid + u * NST;
                t = t < ntask ? t : (t & 3);
                const uint4 *px = reinterpret_cast<const uint4 *>(x + (size_t)t * 8);
                xa[u] = px[0]; xb[u] = px[1];
                if (mode == AXQ_X_RMSNORM) {
                    const uint4 *pe = reinterpret_cast<const uint4 *>(aux + (size_t)t * 8);
                    ea[u] = pe[0]; eb[u] = pe[1];
                }
            }
        }
        STAMP(1);
        auto unpack = [](const uint4 &lo, const uint4 &hi, float (&v)[8]) {
            v[0] = __builtin_bit_cast(float, lo.x); v[1] = __builtin_bit_cast(float, lo.y);
            v[2] = __builtin_bit_cast(float, lo.z); v[3] = __builtin_bit_cast(float, lo.w);
            v[4] = __builtin_bit_cast(float, hi.x); v[5] = __builtin_bit_cast(float, hi.y);
            v[6] = __builtin_bit_cast(float, hi.z); v[7] = __builtin_bit_cast(float, hi.w);
        };
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < MAXT; u++) {
            if (u * NST < ntask) {
                const int t = tid + u * NST;
                const bool live = t < ntask;
                float xv[8];
                unpack(xa[u], xb[u], xv);
                if (mode == AXQ_X_RMSNORM) {
                    // RMSNorm::forward (llm/src/llama.rs:158-187); the 1 / rms is one factor on the result
                    float ev[8];
                    unpack(ea[u], eb[u], ev);
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        if (live) ss = fmaf(xv[i], xv[i], ss);
                        xv[i] *= ev[i];
                    }
                }
                if (live) axq_split8(xv, t, true, wplanes, wgrp, kpad);
            }
        }
        if (mode == AXQ_X_RMSNORM) {
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m);
            if (lane == 0) wsum[wave] = ss;
        }
        STAMP(2);
        lds_only_barrier(); // x is staged
        STAMP(3);
    } else if constexpr (KS == 2) {
        // ---- weight waves that cover two K slices each (K beyond eight slices, one row group): wave ww has slices ww
        // and ww + W, its steps go through them in turn -- ring slot b holds a step of slice b % 2, a round of four steps is
        // two row steps -- and the x operands of a step are fetched from LDS when it is folded (two sets do not fit the
        // registers beside the ring).
        static_assert(NB == 4 && NB0 <= 4, "ring slot parity = slice");
        const int ww = wave - NS, W = (S + 1) >> 1;
        const int blk = lane >> 2, j = lane & 3;
        const bool live1 = ww + W < S; // an odd count of slices: the last wave has one, its other steps meet x = 0
        const int sl[2] = {ww, live1 ? ww + W : ww};
        const int cq[2] = {(sl[0] << 4) + blk, ((ww + W) << 4) + blk};
        const int my_t = 2 * steps; // the wave's steps: row step t / 2 of slice t % 2
        float *red_q[2] = {red + j * red_stride + sl[0] * 4 + (lane >> 4), red + j * red_stride + sl[1] * 4 + (lane >> 4)};
        uint4 *wmeta = lds_raw + n16 + 1 + 4 + (wg_rows * red_stride) / 4 + ww * 64 * NM;
        typename T::Raw buf[NB];
        uint4 hm[NM];
        LaneOff lo[2];
        T::lane_offsets(k, cq[0], lo[0]);
        T::lane_offsets(k, cq[1], lo[1]);
        const int wg_row0 = blockIdx.x * wg_rows;
        const Bases bases = {codes + (size_t)wg_row0 * cp, meta + (size_t)wg_row0 * mp, qhp + (size_t)wg_row0 * qp};
        const int rl_last = n_rows - 1 - wg_row0; // rows relative to the workgroup's first
        // the round's records: record 4 b + j = row j of ring slot b's row step, the slot's slice
        uint32_t moff[NM], mpitch[NM];
        const uint8_t *mbase[NM];
        int mrow[NM];
        {
#pragma unroll
            for (int i = 0; i < NM; i++) {
                const int flat = i * 64 + lane;
                const int rec = flat / CPR < 4 * NB ? flat / CPR : 4 * NB - 1; // lanes beyond the round's records repeat its last
                const int slot = rec >> 2;
                bool from_qh;
                moff[i] = (uint32_t)record_piece<T>(k, sl[slot & 1], flat % CPR, from_qh);
                mbase[i] = from_qh ? bases.qh : bases.meta;
                mpitch[i] = from_qh ? qp : mp;
                mrow[i] = (slot >> 1) * 4 + (rec & 3);
            }
        }
        auto request = [&](int t, int b) { // b = t % NB
            const int tt = t < my_t ? t : b; // steps past the end re-read the first round's
            int rl = 4 * (tt >> 1) + j;
            rl = rl < rl_last ? rl : rl_last;
            const RowOff ro = {(uint32_t)rl * cp, (uint32_t)rl * mp, (uint32_t)rl * qp};
            if (b == 0) {
#pragma unroll
                for (int i = 0; i < NM; i++) {
                    int rlm = 4 * (tt >> 1) + mrow[i]; // rows past the workgroup's steps are the next workgroup's: read, not used
                    rlm = rlm < rl_last ? rlm : rl_last;
                    hm[i] = ld16(mbase[i], (uint32_t)rlm * mpitch[i] + moff[i]);
                }
            }
            T::load_codes(bases, ro, lo[b & 1], buf[b]);
        };
#pragma unroll
        for (int b = 0; b < NB0; b++) request(b, b);
        lds_only_barrier(); // x is staged
#pragma unroll
        for (int b = NB0; b < NB; b++) request(b, b);
        const bool writer = (blk & 3) == 3;
        auto fold = [&](int b, int t) {
            if (b == 0) {
#pragma unroll
                for (int i = 0; i < NM; i++) wmeta[i * 64 + lane] = hm[i];
            }
            XOp xo;
            fetch_xop<T>(wplanes, wgrp, kpad, k, j, cq[b & 1], xo);
            T::set_meta(buf[b], reinterpret_cast<const uint8_t *>(wmeta) + (b * 4 + j) * MSB, blk, cq[b & 1]);
            const float tot = sum_within_row(T::dot(buf[b], xo, cq[b & 1]));
            if (writer && ((b & 1) == 0 || live1)) red_q[b & 1][(t >> 1) * 4 * red_stride] = tot;
        };
        const int rounds = (my_t + NB - 1) / NB;
        int step = 0;
        for (int round = 0; round < rounds - 1; round++, step += NB) {
#pragma unroll
            for (int b = 0; b < NB; b++) {
                fold(b, step + b);
                request(step + NB + b, b);
            }
        }
#pragma unroll
        for (int b = 0; b < NB; b++)
            if (step + b < my_t) fold(b, step + b);
    } else {
        // ---- weight waves
        const int ww = wave - NS;
        const int g_idx = ww / S, slice = ww - g_idx * S;
        const int blk = lane >> 2, j = lane & 3;
        const int c = (slice << 4) + blk; // this lane's 64-weight chunk of the row
        // This group's steps: base, base + stride, ... (my_steps of them).  Dealt in turn, or, with two groups and a count n0
        // in the flags, the first n0 steps to group 0 and the rest to group 1: the waves of group 1 issue their first
        // requests behind group 0's and get every step later, so they are given fewer.
        const int n0 = (flags >> 24) & 0xFF;
        const bool uneven = n0 != 0 && G == 2;
        const int base_step = uneven ? (g_idx ? n0 : 0) : g_idx, step_stride = uneven ? 1 : G;
        const int my_steps = uneven ? (g_idx ? steps - n0 : n0) : (steps - g_idx + G - 1) / G;
        float *red_lane = red + (4 * base_step + j) * red_stride + slice * 4 + (lane >> 4);
        uint4 *wmeta = lds_raw + n16 + 1 + 4 + (wg_rows * red_stride) / 4 + ww * 64 * NM;
        typename T::Raw buf[NB];
        uint4 hm[NM];
        LaneOff lo;
        T::lane_offsets(k, c, lo);
        const int wg_row0 = blockIdx.x * wg_rows;
        const Bases bases = {codes + (size_t)wg_row0 * cp, meta + (size_t)wg_row0 * mp, qhp + (size_t)wg_row0 * qp};
        const int rl0 = 4 * base_step + j, rl_last = n_rows - 1 - wg_row0; // rows relative to the workgroup's first
        const int gstride = 4 * step_stride;                                  // rows from one of the group's steps to its next
        uint32_t moff[NM], mpitch[NM];
        const uint8_t *mbase[NM];
        int mrl0[NM], mst[NM];
        {
#pragma unroll
            for (int i = 0; i < NM; i++) {
                const int flat = i * 64 + lane;
                const int r = flat / CPR < 4 * NB ? flat / CPR : 4 * NB - 1; // lanes beyond the round's rows repeat its last
                bool from_qh;
                moff[i] = (uint32_t)record_piece<T>(k, slice, flat % CPR, from_qh);
                mbase[i] = from_qh ? bases.qh : bases.meta;
                mpitch[i] = from_qh ? qp : mp;
                mrl0[i] = 4 * base_step + (r & 3); // row r of the round: row r % 4 of its step r / 4
                mst[i] = r >> 2;
            }
        }
        auto request = [&](int step, int b) {
            const int s = step < my_steps ? step : 0;
            int rl = rl0 + gstride * s;
            rl = rl < rl_last ? rl : rl_last;
            const RowOff ro = {(uint32_t)rl * cp, (uint32_t)rl * mp, (uint32_t)rl * qp};
            if (b == 0) { // rows past the group's steps belong to the next group or repeat the matrix's last row: read, not used
#pragma unroll
                for (int i = 0; i < NM; i++) {
                    int sm = s + mst[i];
                    sm = sm < my_steps ? sm : 0;
                    int rlm = mrl0[i] + gstride * sm;
                    rlm = rlm < rl_last ? rlm : rl_last;
                    hm[i] = ld16(mbase[i], (uint32_t)rlm * mpitch[i] + moff[i]);
                }
            }
            T::load_codes(bases, ro, lo, buf[b]);
        };
        // three steps before x is staged (with the round's records and the split waves' x a few more loads than the compute
        // unit holds in flight: x returns first and makes room), the ring's last after the barrier
#pragma unroll
        for (int b = 0; b < NB0; b++) request(b, b);
        STAMP(1);
        lds_only_barrier(); // x is staged
        STAMP(3);
        XOp xo;
        fetch_xop<T>(wplanes, wgrp, kpad, k, j, c, xo);
#pragma unroll
        for (int b = NB0; b < NB; b++) request(b, b);
        STAMP(4);
        const bool writer = (blk & 3) == 3;
        const int red_step = gstride * red_stride;
        auto fold = [&](int b, int step) {
            if (b == 0) { // the wave's own patch: LDS serves a wave's stores and loads in order
#pragma unroll
                for (int i = 0; i < NM; i++) wmeta[i * 64 + lane] = hm[i];
            }
            T::set_meta(buf[b], reinterpret_cast<const uint8_t *>(wmeta) + (b * 4 + j) * MSB, blk, c);
#ifdef AXQ_TIMING_NOFOLD // timing builds only (results not valid): the loads are waited for and nothing is computed
            float tot = __builtin_bit_cast(float, reinterpret_cast<const uint32_t *>(&buf[b])[0] ^ reinterpret_cast<const uint32_t *>(&buf[b])[7]) + xo.sg[0];
#else
            float tot = sum_within_row(T::dot(buf[b], xo, c));
#endif
            if (writer) red_lane[step * red_step] = tot;
            STAMP(5 + (step < 8 ? step : 8));
        };
        const int rounds = (my_steps + NB - 1) / NB;
        int step = 0;
        for (int round = 0; round < rounds - 1; round++, step += NB) {
#pragma unroll
            for (int b = 0; b < NB; b++) {
                fold(b, step + b);
                // steps past the end re-read the first (cache hits): every wave's count of loads stays the same (leaving
                // them out, with the last two rounds written out per count of steps, measured the same)
                request(step + NB + b, b);
            }
        }
#pragma unroll
        for (int b = 0; b < NB; b++)
            if (step + b < my_steps) fold(b, step + b);
    }

    // partial sums -> y, in a fixed order, by every thread of the workgroup
    __syncthreads();
    STAMP(14);
    const int nthreads = (int)blockDim.x;
    float inv = 1.0f;
    if (mode == AXQ_X_RMSNORM) {
        float tot = 0.f;
#pragma unroll
        for (int i = 0; i < NS; i++) tot += wsum[i];
        inv = 1.0f / sqrtf(tot / (float)k + eps);
    }
    auto row_total = [&](int t) { // slice by slice, the four DPP rows of each in order
        const float4 *pr = reinterpret_cast<const float4 *>(red + (size_t)t * red_stride);
        float tot = 0.f;
        for (int s2 = 0; s2 < S; s2++) {
            float4 v = pr[s2];
            tot += (v.x + v.y) + (v.z + v.w);
        }
        return tot * inv;
    };
    if (ymode == AXQ_Y_SWIGLU) {
        // rows 8b..8b+3 are gate rows, 8b+4..8b+7 the up rows of the same outputs (wg_rows is a multiple of 8)
        for (int t = tid; t < (wg_rows >> 1); t += nthreads) {
            const int lg = ((t >> 2) << 3) + (t & 3);
            const int row = blockIdx.x * wg_rows + lg;
            if (row + 4 < n_rows) {
                const float g = row_total(lg), u = row_total(lg + 4);
                y[(blockIdx.x * wg_rows >> 1) + t] = (g * (1.0f / (1.0f + expf(-g)))) * u;
            }
        }
        STAMP(15);
        STAMP_END();
        return;
    }
    for (int t = tid; t < wg_rows; t += nthreads) {
        int row = blockIdx.x * wg_rows + t;
        if (row < n_rows) {
            const float tot = row_total(t);
            y[row] = bias ? tot + bias[row] : tot;
        }
    }
    STAMP(15);
    STAMP_END();
}

__global__ void __launch_bounds__(256) prep_x_kernel(const float *x, int k, uint8_t *xq) {
    const int kpad = (k + 15) & ~15;
    stage_x(x, k, xq, reinterpret_cast<uint4 *>(xq + (size_t)4 * kpad), (int)(blockIdx.x * blockDim.x + threadIdx.x),
            (int)(gridDim.x * blockDim.x));
}

// The launchers return AXQ_OK or the status of a refused request for dynamic LDS (nothing is launched then).
template <class T, int NB, bool PRE>
int launch_one(axq_ctx *ctx, const DpArgs &a, unsigned grid, unsigned block, size_t lds) {
    static std::atomic<uint64_t> lds_allowed{0}, lds_allowed_w{0}; // dynamic LDS beyond 64 KB is asked for per kernel and device
    int st;
    static const bool shared_x = getenv("AXQ_GEMV_SHARED_X") && getenv("AXQ_GEMV_SHARED_X")[0] == '1'; // development knob: the kernel that splits x once per workgroup
    // the per-round scale loads are 16 bytes wide: the rows of the meta plane have to be whole 16-byte pieces
    const bool rounds_ok = !T::ROUND_META || NB > 4 || (T::meta_row_bytes(a.k) % 16 == 0 && a.meta_pitch % 16 == 0 && T::meta_row_bytes(a.k) >= 16);
    if (!PRE && !shared_x && rounds_ok) {
        // x arrives raw: every wave stages its own slice
        const size_t lds_w = (size_t)(block / 64) * (4 * 1024 + 32 * 16 + (T::ROUND_META ? 16 * T::META_SLICE_BYTES : 0)) + 64 +
                             (size_t)a.G * a.steps * 4 * a.S * 4 * sizeof(float);
#ifdef AXQ_STAMPS
        if (lds_w <= 160 * 1024 &&
#else
        if (lds_w > 64 * 1024 && lds_w <= 160 * 1024 &&
#endif
            (st = axq_allow_lds(ctx, reinterpret_cast<const void *>(&gemv_dpw_kernel<T, NB>), lds_allowed_w, 160 * 1024)) != AXQ_OK)
            return st;
        if (lds_w <= 160 * 1024) {
#ifdef AXQ_STAMPS
            gemv_dpw_kernel<T, NB><<<grid, block, 160 * 1024, ctx->stream>>>(DP_LAUNCH_ARGS(a)); // the stamps live in the last 4 KB
#else
            gemv_dpw_kernel<T, NB><<<grid, block, lds_w, ctx->stream>>>(DP_LAUNCH_ARGS(a));
#endif
            return AXQ_OK;
        }
    }
    if (lds > 64 * 1024 && (st = axq_allow_lds(ctx, reinterpret_cast<const void *>(&gemv_dp_kernel<T, NB, PRE, false>), lds_allowed, 160 * 1024)) != AXQ_OK)
        return st;
    gemv_dp_kernel<T, NB, PRE, false><<<grid, block, lds, ctx->stream>>>(DP_LAUNCH_ARGS(a));
    return AXQ_OK;
}

template <class T, bool PRE>
int launch_nb(axq_ctx *ctx, const DpArgs &a, int nb, unsigned grid, unsigned block, size_t lds) {
    switch (nb) {
    case 1: return launch_one<T, 1, PRE>(ctx, a, grid, block, lds);
    case 2: return launch_one<T, 2, PRE>(ctx, a, grid, block, lds);
    case 3: return launch_one<T, 3, PRE>(ctx, a, grid, block, lds);
    case 4: return launch_one<T, 4, PRE>(ctx, a, grid, block, lds);
    case 5: return launch_one<T, 5, PRE>(ctx, a, grid, block, lds);
    case 6: return launch_one<T, 6, PRE>(ctx, a, grid, block, lds);
    case 7: return launch_one<T, 7, PRE>(ctx, a, grid, block, lds);
    default: return launch_one<T, 8, PRE>(ctx, a, grid, block, lds);
    }
}

// Q4_K with a raw x: the kernel with one header load per round.  1 = launched, 0 = not this kernel's case, < 0 = status.
template <class T>
int launch_q4k_rounds(axq_ctx *, const DpArgs &, unsigned, unsigned, size_t) { return 0; }
template <>
int launch_q4k_rounds<DQ4K>(axq_ctx *ctx, const DpArgs &a, unsigned grid, unsigned block, size_t lds) {
    static const bool off = getenv("AXQ_GEMV_Q4K_ROUNDS") && getenv("AXQ_GEMV_Q4K_ROUNDS")[0] == '0'; // development knob
    static std::atomic<uint64_t> lds_allowed[2];
    if (off) return 0;
    // measured inside the 7B-shape decode: a gain from three steps per group on (qkv 6.6 -> 6.0 us, gate/up 15.4 -> 14.8 us);
    // with two steps (o projection) or one group of 14 waves over a long K (down projection, two split tasks per thread)
    // the kernel with per-wave staging and no barrier is ahead
    if (a.G < 2 || a.steps < 3) return 0;
    lds += (size_t)(block / 64) * 16 * DQ4K::META_SLICE_BYTES; // the waves' patches of scale records
    if (lds > 160 * 1024) return 0;
    if (lds > 64 * 1024) {
        int st = axq_allow_lds(ctx, reinterpret_cast<const void *>(&gemv_dp_kernel<DQ4K, 3, false, true>), lds_allowed[0], 160 * 1024);
        if (st == AXQ_OK) st = axq_allow_lds(ctx, reinterpret_cast<const void *>(&gemv_dp_kernel<DQ4K, 4, false, true>), lds_allowed[1], 160 * 1024);
        if (st != AXQ_OK) return st;
    }
    if (a.steps == 3) gemv_dp_kernel<DQ4K, 3, false, true><<<grid, block, lds, ctx->stream>>>(DP_LAUNCH_ARGS(a));
    else gemv_dp_kernel<DQ4K, 4, false, true><<<grid, block, lds, ctx->stream>>>(DP_LAUNCH_ARGS(a));
    return 1;
}

// The kernel with split waves: a raw x, K within eight 1024-wide slices and four tasks per split thread.  The row steps
// are dealt to workgroups (one per compute unit) and, inside a workgroup, to G row groups in turn.
template <class T>
int launch_sw(axq_ctx *ctx, const DpArgs &a) {
    constexpr int NS = 4; // split waves: two tasks per lane at K = 4096 (8 measured slower, 2 much slower)
    static std::atomic<uint64_t> lds_allowed[8];
    const int S = a.S;
    if (S > 8 || (a.k >> 3) > 4 * 64 * NS) return 0;
    // the per-round scale loads are 16 bytes wide: the rows of the meta plane have to be whole 16-byte pieces
    if (T::meta_row_bytes(a.k) % 16 != 0 || a.meta_pitch % 16 != 0 || T::meta_row_bytes(a.k) < 16) return 0;
    int G = 8 / S; // eight weight waves (twelve, three per SIMD, measured slower: 8.7 against 8.1 us at 14336 x 4096)
    const int rowsteps = (a.n_rows + 3) / 4;
    const int cus = ctx->prop.multiProcessorCount * ctx->gemv_wgs_per_cu;
    int steps = (rowsteps + cus - 1) / cus;
    if (a.ymode == AXQ_Y_SWIGLU && (steps & 1)) steps++; // a workgroup must hold whole gate/up groups of 8 rows
    if (steps < G) G = steps;
    const unsigned grid = (unsigned)((rowsteps + steps - 1) / steps);
    // Two groups: each takes a run of consecutive steps, group 0 three of every five.  Its waves issue their first requests
    // ahead of group 1's and get every step sooner; measured against steps dealt in turn, launches of one kernel in a row:
    // 8.2 -> 7.6 us at 14336 x 4096 (14 steps), 12.7 -> 12.2 us at 28672 x 4096, 14.1 -> 13.4 us at 32000 x 4096.  Not
    // at six steps: 6144 x 4096 gains alone (5.6 -> 5.05 us) and loses inside the decode step (4 + 2 steps leave a ring of two).
    static const int split0 = getenv("AXQ_GEMV_SPLIT0") ? atoi(getenv("AXQ_GEMV_SPLIT0")) : 60; // development knob, percent; 0 = dealt in turn
    int n0 = 0;
    if (G == 2 && steps >= 7 && steps < 256 && split0 > 0) {
        n0 = (steps * split0 + 50) / 100;
        n0 = n0 < 2 ? 2 : (n0 > steps - 2 ? steps - 2 : n0);
    }
    const int per_group = n0 ? (steps - n0 < n0 ? steps - n0 : n0) : (steps + G - 1) / G;
    const int nb = per_group < 4 ? per_group : 4; // ring depth: deeper rings measured slower (a wave that stands at its requests folds nothing)
    const int cpr = T::META_SLICE_BYTES / 16, nm = (4 * nb * cpr + 63) / 64;
    size_t lds = axq_split_bytes(a.k) + 16 + 64 + (size_t)steps * 4 * 4 * S * sizeof(float) + (size_t)(S * G) * nm * 1024;
    if (lds > 160 * 1024) return 0;
    const unsigned block = (unsigned)(64 * (S * G + NS));
    const int flags = a.mode | (a.ymode << 8) | (G << 16) | (n0 << 24);
    auto go = [&](auto kern, std::atomic<uint64_t> &mask) -> int {
#ifdef AXQ_STAMPS
        lds = 160 * 1024; // the stamps live in the last 4 KB
#endif
        if (lds > 64 * 1024) {
            const int st = axq_allow_lds(ctx, reinterpret_cast<const void *>(kern), mask, 160 * 1024);
            if (st != AXQ_OK) return st;
        }
        kern<<<grid, block, lds, ctx->stream>>>(a.x, a.codes, a.meta, (uint32_t)a.codes_pitch, (uint32_t)a.meta_pitch, a.n_rows, a.k, steps, flags,
                                                a.eps, a.y, a.bias, a.aux, a.qh, (uint32_t)a.qh_pitch);
        return 1;
    };
    switch (nb) {
    case 1: return go(&gemv_sw_kernel<T, 1, 1, NS>, lds_allowed[1]);
    case 2: return go(&gemv_sw_kernel<T, 2, 2, NS>, lds_allowed[2]);
    case 3: return go(&gemv_sw_kernel<T, 3, 3, NS>, lds_allowed[3]);
    default: return go(&gemv_sw_kernel<T, 4, 3, NS>, lds_allowed[4]);
    }
}

// The same kernel for K beyond eight slices (up to sixteen): eight split waves, and weight waves of two slices each.  Taken
// by the types that say so (TWO_SLICE_WAVES).
template <class T>
int launch_sw2(axq_ctx *ctx, const DpArgs &a) {
    if constexpr (!T::TWO_SLICE_WAVES) {
        return 0;
    } else {
    constexpr int NS = 8;
    static std::atomic<uint64_t> lds_allowed{0};
    static const bool off = getenv("AXQ_GEMV_SW2") && getenv("AXQ_GEMV_SW2")[0] == '0'; // development knob: such K on the kernel with per-wave staging
    const int S = a.S;
    if (off || S <= 8 || S > 16 || (a.k >> 3) > 4 * 64 * NS) return 0;
    if (T::meta_row_bytes(a.k) % 16 != 0 || a.meta_pitch % 16 != 0 || T::meta_row_bytes(a.k) < 16) return 0;
    const int rowsteps = (a.n_rows + 3) / 4;
    const int cus = ctx->prop.multiProcessorCount * ctx->gemv_wgs_per_cu;
    int steps = (rowsteps + cus - 1) / cus;
    if (a.ymode == AXQ_Y_SWIGLU && (steps & 1)) steps++; // a workgroup must hold whole gate/up groups of 8 rows
    if (steps < 2 || steps > 64) return 0;               // a ring of four steps = two row steps at least
    const unsigned grid = (unsigned)((rowsteps + steps - 1) / steps);
    const int W = (S + 1) / 2;
    const int cpr = T::META_SLICE_BYTES / 16, nm = (4 * 4 * cpr + 63) / 64;
    const size_t lds = axq_split_bytes(a.k) + 16 + 64 + (size_t)steps * 4 * 4 * S * sizeof(float) + (size_t)W * nm * 1024;
    if (lds > 160 * 1024) return 0;
    const unsigned block = (unsigned)(64 * (W + NS));
    const int flags = a.mode | (a.ymode << 8) | (1 << 16);
    auto kern = &gemv_sw_kernel<T, 4, 3, NS, 2>;
    if (lds > 64 * 1024) {
        const int st = axq_allow_lds(ctx, reinterpret_cast<const void *>(kern), lds_allowed, 160 * 1024);
        if (st != AXQ_OK) return st;
    }
    kern<<<grid, block, lds, ctx->stream>>>(a.x, a.codes, a.meta, (uint32_t)a.codes_pitch, (uint32_t)a.meta_pitch, a.n_rows, a.k, steps, flags,
                                            a.eps, a.y, a.bias, a.aux, a.qh, (uint32_t)a.qh_pitch);
    return 1;
    }
}

// 1 = launched, 0 = the shape is not this kernel's, < 0 = status
template <class T>
int launch_dp(axq_ctx *ctx, const axq_weight *w, const float *x, const uint8_t *xq, int mode, const float *aux, float eps,
              int ymode, const float *bias, float *y) {
    if (w->k % 64 != 0 || w->k > 16384) return 0;
    DpArgs a;
    a.codes = w->codes; a.meta = w->meta; a.qh = w->qh;
    a.codes_pitch = w->codes_pitch; a.meta_pitch = w->meta_pitch; a.qh_pitch = w->qh_pitch;
    a.x = x; a.xq = xq; a.bias = bias; a.y = y;
    a.mode = mode; a.aux = aux; a.eps = eps; a.ymode = ymode;
    a.n_rows = (int)w->n_rows;
    a.k = (int)w->k;
    a.S = (a.k + 1023) / 1024;            // waves that span K once (<= 16)
    a.G = a.S <= 8 ? 8 / a.S : 1;         // row groups per workgroup
    a.P = 1;
    const unsigned block = (unsigned)(64 * a.S * a.G);
    // 4-row steps per group: one workgroup per compute unit unless that makes a group's share of the
    // reduction buffer too large; the ring depth is what a lane can hold in registers
    const int rowsteps = (a.n_rows + 3) / 4;
    const int cus = ctx->prop.multiProcessorCount;
    int wgs = cus * ctx->gemv_wgs_per_cu;
    int steps = (rowsteps + wgs * a.G - 1) / (wgs * a.G);
    if (steps > 64) steps = 64;
    if (ymode == AXQ_Y_SWIGLU && ((a.G * steps) & 1)) steps++; // a workgroup must hold whole gate/up groups of 8 rows
    a.steps = steps;
    int nb = block > 512 ? T::BIG_NB : 8;
    if (nb > ctx->gemv_max_nb) nb = ctx->gemv_max_nb;
    if (nb > steps) nb = steps;
    if (T::ROUND_META && !xq && nb > 4) nb = 4; // a round of the per-wave staging kernel is at most four steps
    const unsigned grid = (unsigned)((rowsteps + steps * a.G - 1) / (steps * a.G));
    size_t lds = (size_t)a.G * steps * 4 * a.S * 4 * sizeof(float);
    lds += axq_split_bytes(a.k) + 16 + 64;
    if (lds > 160 * 1024) return 0;
    static const bool sw_off = getenv("AXQ_GEMV_SW") && getenv("AXQ_GEMV_SW")[0] == '0'; // development knob: no split waves
    if (!xq && !sw_off) {
        int r = launch_sw<T>(ctx, a);
        if (r != 0) return r;
        r = launch_sw2<T>(ctx, a);
        if (r != 0) return r;
    }
    if (!xq) {
        const int r = launch_q4k_rounds<T>(ctx, a, grid, block, lds);
        if (r != 0) return r;
    }
    const int st = xq ? launch_nb<T, true>(ctx, a, nb, grid, block, lds) : launch_nb<T, false>(ctx, a, nb, grid, block, lds);
    return st == AXQ_OK ? 1 : st;
}

} // namespace

// Bytes of the split form of a K-vector: four limb planes and one (scale, sum) pair per 32 elements.
size_t axq_xq_bytes(int64_t k) { return axq_split_bytes(k); }

// x[k] (f32, device) -> split form at xq (device, axq_xq_bytes(k) bytes).
int axq_dev_prep_x(axq_ctx *ctx, const float *x, int64_t k, uint8_t *xq) {
    int tasks = (int)((k + 7) / 8);
    int grid = (tasks + 255) / 256;
    prep_x_kernel<<<grid, 256, 0, ctx->stream>>>(x, (int)k, xq);
    AXQ_LAUNCH_CHECK(ctx, "prep_x_kernel");
    return AXQ_OK;
}

// Returns 1 when the launch was made, 0 when this kernel does not cover the shape (the caller falls
// back to the vector-ALU kernels), or a negative status.  xq = NULL: the kernel splits x itself, after
// applying the prologue `mode` (axq_internal.h) with its second operand `aux`.
int axq_dev_gemv_dp_ex(axq_ctx *ctx, const axq_weight *w, const float *x, const uint8_t *xq, int mode, const float *aux,
                       float eps, int ymode, const float *bias, float *y) {
    int ok;
    if (xq && mode != AXQ_X_PLAIN) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "a fused prologue needs the raw x");
    if (ymode == AXQ_Y_SWIGLU && (w->n_rows % 8 != 0 || bias))
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "the SwiGLU epilogue needs whole groups of 8 rows and no bias");
    switch (w->type) {
    case AXQ_Q4_K: ok = launch_dp<DQ4K>(ctx, w, x, xq, mode, aux, eps, ymode, bias, y); break;
    case AXQ_Q5_K: ok = launch_dp<DQ5K>(ctx, w, x, xq, mode, aux, eps, ymode, bias, y); break;
    case AXQ_Q6_K: ok = launch_dp<DQ6K>(ctx, w, x, xq, mode, aux, eps, ymode, bias, y); break;
    case AXQ_Q4_0: ok = launch_dp<DQ4x<false>>(ctx, w, x, xq, mode, aux, eps, ymode, bias, y); break;
    case AXQ_Q4_1: ok = launch_dp<DQ4x<true>>(ctx, w, x, xq, mode, aux, eps, ymode, bias, y); break;
    case AXQ_Q5_0: ok = launch_dp<DQ5x<false>>(ctx, w, x, xq, mode, aux, eps, ymode, bias, y); break;
    case AXQ_Q5_1: ok = launch_dp<DQ5x<true>>(ctx, w, x, xq, mode, aux, eps, ymode, bias, y); break;
    case AXQ_Q8_0: ok = launch_dp<DQ80>(ctx, w, x, xq, mode, aux, eps, ymode, bias, y); break;
    default: return 0;
    }
    if (ok <= 0) return ok;
    AXQ_LAUNCH_CHECK(ctx, "gemv_dp_kernel");
    return 1;
}

int axq_dev_gemv_dp(axq_ctx *ctx, const axq_weight *w, const float *x, const uint8_t *xq, const float *bias, float *y) {
    return axq_dev_gemv_dp_ex(ctx, w, x, xq, AXQ_X_PLAIN, nullptr, 0.f, AXQ_Y_PLAIN, bias, y);
}

// Whether axq_dev_gemv_dp_ex covers a weight of this type and width.
bool axq_dev_gemv_dp_covers(const axq_weight *w) {
    switch (w->type) {
    case AXQ_Q4_K: case AXQ_Q5_K: case AXQ_Q6_K: case AXQ_Q4_0: case AXQ_Q4_1: case AXQ_Q5_0: case AXQ_Q5_1: case AXQ_Q8_0:
        return w->k % 64 == 0 && w->k <= 16384;
    default: return false;
    }
}

#ifdef AXQ_STAMPS
extern "C" __attribute__((visibility("default"))) int axq_debug_set_stamps(void *buf) {
    unsigned int zero = 0;
    if (hipMemcpyToSymbol(HIP_SYMBOL(axq_stamps), &buf, sizeof buf) != hipSuccess) return -1;
    if (hipMemcpyToSymbol(HIP_SYMBOL(axq_stamp_launch), &zero, sizeof zero) != hipSuccess) return -1;
    return 0;
}
#endif
