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
// Tiling: a workgroup computes BM x 128 outputs (BM = 128 or 256) with BM/32 waves, one 64 x 64 block
// (2 x 2 MFMA tiles) per wave; K advances 64 at a time through one LDS stage holding the x tile and
// the two weight tiles; two workgroups share a compute unit and fill each other's load/dequant gaps.
#include <hip/hip_fp16.h>

#include "axq_internal.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int BN = 128;  // output columns (weight rows) per workgroup
constexpr int BK = 64;   // K per stage
constexpr int LDK = 72;  // LDS row length in halfs (64 + 8 padding against bank conflicts)

struct GemmArgs {
    const uint8_t *codes, *meta, *qh;
    size_t codes_pitch, meta_pitch, qh_pitch;
    const _Float16 *xh;    // [M, K] row-scaled f16
    const float *rowscale; // [M]
    float *y;              // [M, N]
    int m, n, k;
};

__device__ inline float h2f(uint32_t bits) { return __half2float(__ushort_as_half((unsigned short)bits)); }

// ---------------------------------------------------------------------------
// Dequantisation units.  A unit is 16 weights of one weight row inside the current 64-wide K step:
// two runs of 8 consecutive k (k0.., k1..).  unit index u4 = 0..3 per row.  Each trait reproduces the
// element formula of crates/axonml-quant/src/dequantize.rs (Q8_0 :89-92, Q4_0 :116-121, Q4_1 :145-151)
// or of the GGUF spec (Q5_0, Q5_1, Q4_K), rounding as the f32 reference does (multiply, then add).
// ---------------------------------------------------------------------------
struct GQ4K {
    __device__ static void deq16(const GemmArgs &a, size_t row, int kstep, int u4, float (&w)[16], int &k0, int &k1) {
        const int cpr = a.k >> 6;          // pairs per row
        const int pair = kstep;            // one pair of sub-blocks per K step
        const int slice = pair >> 6, pr = pair & 63;
        int P = cpr - (slice << 6);
        P = P < 64 ? P : 64;
        const int half = u4 >> 1, part = u4 & 1;
        const uint8_t *base = a.codes + row * a.codes_pitch + (size_t)slice * 2048 + (size_t)half * 16 * P + (size_t)pr * 16 + part * 8;
        const uint2 q = *reinterpret_cast<const uint2 *>(base);
        const uint4 h = *reinterpret_cast<const uint4 *>(a.meta + row * a.meta_pitch + (size_t)(pair >> 2) * 16);
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
        const float d = h2f(h.x & 0xFFFF), dmin = h2f(h.x >> 16);
        const float sd0 = d * (float)(scp & 0xFF), sd1 = d * (float)(scp >> 8);
        const float sm0 = dmin * (float)(mp & 0xFF), sm1 = dmin * (float)(mp >> 8);
        const uint32_t qq[2] = {q.x, q.y};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t byte = (qq[i >> 2] >> (8 * (i & 3))) & 0xFF;
            float lo = sd0 * (float)(byte & 0xF), hi = sd1 * (float)(byte >> 4);
            w[i] = lo - sm0;
            w[8 + i] = hi - sm1;
        }
        k0 = half * 16 + part * 8;
        k1 = 32 + k0;
    }
};

template <bool WITH_MIN>
struct GQ4x { // reference nibble order: byte i = elements 2i (low), 2i+1 (high)
    __device__ static void deq16(const GemmArgs &a, size_t row, int kstep, int u4, float (&w)[16], int &k0, int &k1) {
        const int blk = kstep * 2 + (u4 >> 1), part = u4 & 1;
        const uint2 q = *reinterpret_cast<const uint2 *>(a.codes + row * a.codes_pitch + (size_t)blk * 16 + part * 8);
        const uint8_t *mp = a.meta + row * a.meta_pitch;
        float scale, mn = 0.f;
        if (WITH_MIN) {
            uint32_t m = *reinterpret_cast<const uint32_t *>(mp + (size_t)blk * 4);
            scale = h2f(m & 0xFFFF);
            mn = h2f(m >> 16);
        } else {
            scale = h2f(*reinterpret_cast<const uint16_t *>(mp + (size_t)blk * 2));
        }
        const uint32_t qq[2] = {q.x, q.y};
#pragma unroll
        for (int i = 0; i < 16; i++) {
            uint32_t nib = (qq[i >> 3] >> (4 * (i & 7))) & 0xF;
            if (WITH_MIN) {
                float t = (float)nib * scale;
                w[i] = t + mn;
            } else {
                w[i] = (float)((int)nib - 8) * scale;
            }
        }
        k0 = (u4 >> 1) * 32 + part * 16;
        k1 = k0 + 8;
    }
};

template <bool WITH_MIN>
struct GQ5x { // byte j = elements j (low nibble) and j + 16 (high); qh bit e = bit 4 of element e
    __device__ static void deq16(const GemmArgs &a, size_t row, int kstep, int u4, float (&w)[16], int &k0, int &k1) {
        const int blk = kstep * 2 + (u4 >> 1), part = u4 & 1;
        const uint2 q = *reinterpret_cast<const uint2 *>(a.codes + row * a.codes_pitch + (size_t)blk * 16 + part * 8);
        const uint32_t qh = *reinterpret_cast<const uint32_t *>(a.qh + row * a.qh_pitch + (size_t)blk * 4);
        const uint8_t *mp = a.meta + row * a.meta_pitch;
        float d, mn = 0.f;
        if (WITH_MIN) {
            uint32_t m = *reinterpret_cast<const uint32_t *>(mp + (size_t)blk * 4);
            d = h2f(m & 0xFFFF);
            mn = h2f(m >> 16);
        } else {
            d = h2f(*reinterpret_cast<const uint16_t *>(mp + (size_t)blk * 2));
        }
        const uint32_t qq[2] = {q.x, q.y};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int e = part * 8 + i;
            uint32_t byte = (qq[i >> 2] >> (8 * (i & 3))) & 0xFF;
            int u0 = (int)((byte & 0xF) | (((qh >> e) & 1u) << 4));
            int u1 = (int)((byte >> 4) | (((qh >> (e + 16)) & 1u) << 4));
            if (WITH_MIN) {
                float t0 = (float)u0 * d, t1 = (float)u1 * d;
                w[i] = t0 + mn;
                w[8 + i] = t1 + mn;
            } else {
                w[i] = (float)(u0 - 16) * d;
                w[8 + i] = (float)(u1 - 16) * d;
            }
        }
        k0 = (u4 >> 1) * 32 + part * 8;
        k1 = k0 + 16;
    }
};

struct GQ80 {
    __device__ static void deq16(const GemmArgs &a, size_t row, int kstep, int u4, float (&w)[16], int &k0, int &k1) {
        const int blk = kstep * 2 + (u4 >> 1), part = u4 & 1;
        const uint4 q = *reinterpret_cast<const uint4 *>(a.codes + row * a.codes_pitch + (size_t)blk * 32 + part * 16);
        const float scale = h2f(*reinterpret_cast<const uint16_t *>(a.meta + row * a.meta_pitch + (size_t)blk * 2));
        const uint32_t qq[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 16; i++) w[i] = (float)(signed char)((qq[i >> 2] >> (8 * (i & 3))) & 0xFF) * scale;
        k0 = (u4 >> 1) * 32 + part * 16;
        k1 = k0 + 8;
    }
};

struct GF16 {
    __device__ static void deq16(const GemmArgs &a, size_t row, int kstep, int u4, float (&w)[16], int &k0, int &k1) {
        const uint4 *p = reinterpret_cast<const uint4 *>(a.codes + row * a.codes_pitch + ((size_t)kstep * 64 + u4 * 16) * 2);
        const uint4 v0 = p[0], v1 = p[1];
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
    __device__ static void deq16(const GemmArgs &a, size_t row, int kstep, int u4, float (&w)[16], int &k0, int &k1) {
        const float4 *p = reinterpret_cast<const float4 *>(a.codes + row * a.codes_pitch + ((size_t)kstep * 64 + u4 * 16) * 4);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float4 v = p[i];
            w[4 * i] = v.x; w[4 * i + 1] = v.y; w[4 * i + 2] = v.z; w[4 * i + 3] = v.w;
        }
        k0 = u4 * 16;
        k1 = k0 + 8;
    }
};

__device__ inline uint32_t pack_h2(_Float16 a, _Float16 b) {
    return (uint32_t)__builtin_bit_cast(unsigned short, a) | ((uint32_t)__builtin_bit_cast(unsigned short, b) << 16);
}

// w[0..7] -> eight f16 "high" parts and eight f16 remainders, as two 16-byte vectors
__device__ inline void split8_f16(const float *w, uint4 &hi, uint4 &lo) {
    uint32_t h[4], l[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        _Float16 h0 = (_Float16)w[2 * i], h1 = (_Float16)w[2 * i + 1];
        _Float16 l0 = (_Float16)(w[2 * i] - (float)h0), l1 = (_Float16)(w[2 * i + 1] - (float)h1);
        h[i] = pack_h2(h0, h1);
        l[i] = pack_h2(l0, l1);
    }
    hi = make_uint4(h[0], h[1], h[2], h[3]);
    lo = make_uint4(l[0], l[1], l[2], l[3]);
}

template <class T, int BM>
__global__ void __launch_bounds__(2 * BM) gemm_kernel(GemmArgs a) {
    extern __shared__ _Float16 lds[];
    _Float16 *As = lds;               // [BM][LDK]
    _Float16 *Bh = As + BM * LDK;     // [BN][LDK]
    _Float16 *Bl = Bh + BN * LDK;     // [BN][LDK]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nthreads = 2 * BM;
    const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64; // this wave's 64 x 64 block inside the tile
    const int li = lane & 31, lk = (lane >> 5) * 8;

    float16v acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    const int ksteps = a.k / BK;
    for (int ks = 0; ks < ksteps; ks++) {
        // x tile: BM rows of 64 halfs = 8 vectors of 16 bytes per row
        uint4 xa[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int v = tid + i * nthreads; // BM * 8 vectors in all = 4 per thread
            int row = v >> 3, c = v & 7;
            int gm = m0 + row;
            gm = gm < a.m ? gm : a.m - 1;
            xa[i] = *reinterpret_cast<const uint4 *>(a.xh + (size_t)gm * a.k + (size_t)ks * BK + c * 8);
        }
        // weight tile: 128 rows x 4 units of 16 weights
        constexpr int UNITS = BN * 4 / (2 * BM); // per thread: 2 (BM = 128) or 1 (BM = 256)
        uint4 wh[UNITS][2], wl[UNITS][2];
        int wk0[UNITS], wk1[UNITS];
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            int unit = tid + u * nthreads;
            int row = unit >> 2, u4 = unit & 3;
            int gn = n0 + row;
            gn = gn < a.n ? gn : a.n - 1;
            float w[16];
            T::deq16(a, (size_t)gn, ks, u4, w, wk0[u], wk1[u]);
            split8_f16(w, wh[u][0], wl[u][0]);
            split8_f16(w + 8, wh[u][1], wl[u][1]);
        }
        __syncthreads(); // the previous step's MFMAs have read the stage
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int v = tid + i * nthreads;
            int row = v >> 3, c = v & 7;
            *reinterpret_cast<uint4 *>(As + row * LDK + c * 8) = xa[i];
        }
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            int unit = tid + u * nthreads;
            int row = unit >> 2;
            *reinterpret_cast<uint4 *>(Bh + row * LDK + wk0[u]) = wh[u][0];
            *reinterpret_cast<uint4 *>(Bh + row * LDK + wk1[u]) = wh[u][1];
            *reinterpret_cast<uint4 *>(Bl + row * LDK + wk0[u]) = wl[u][0];
            *reinterpret_cast<uint4 *>(Bl + row * LDK + wk1[u]) = wl[u][1];
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; kk += 16) {
            half8 af[2], bh[2], bl[2];
#pragma unroll
            for (int i = 0; i < 2; i++) af[i] = *reinterpret_cast<const half8 *>(As + (wm + i * 32 + li) * LDK + kk + lk);
#pragma unroll
            for (int j = 0; j < 2; j++) {
                bh[j] = *reinterpret_cast<const half8 *>(Bh + (wn + j * 32 + li) * LDK + kk + lk);
                bl[j] = *reinterpret_cast<const half8 *>(Bl + (wn + j * 32 + li) * LDK + kk + lk);
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bl[j], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bh[j], acc[i][j], 0, 0, 0);
                }
        }
    }
    // D layout: lane -> column li; register r -> row 8 * (r / 4) + 4 * (lane / 32) + r % 4
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int gn = n0 + wn + j * 32 + li;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int gm = m0 + wm + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (gm < a.m && gn < a.n) a.y[(size_t)gm * a.n + gn] = acc[i][j][r] * a.rowscale[gm];
            }
        }
}

// bf16 rows -> f16 rows scaled by a power of two (largest magnitude below 2^15), and the scale to undo it.
__global__ void __launch_bounds__(256) gemm_prep_x_kernel(const uint16_t *x, int m, int k, _Float16 *xh, float *rowscale) {
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
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    // amax in [2^e, 2^(e+1)) -> multiply by 2^(14 - e); inf/nan rows are passed through unscaled
    int eb = (int)((__builtin_bit_cast(uint32_t, amax) >> 23) & 0xFF);
    if (eb == 0 || eb == 0xFF) eb = 127 + 14;
    int sb = 127 + 14 - (eb - 127);
    sb = sb < 1 ? 1 : (sb > 254 ? 254 : sb);
    const float f = __builtin_bit_cast(float, (uint32_t)sb << 23);
    for (int i = threadIdx.x; i < k; i += blockDim.x) {
        float v = __builtin_bit_cast(float, (uint32_t)xr[i] << 16);
        xh[(size_t)row * k + i] = (_Float16)(v * f);
    }
    if (threadIdx.x == 0) rowscale[row] = 1.0f / f;
}

template <class T>
int launch_gemm(axq_ctx *ctx, const GemmArgs &a) {
    static bool attr_set = false;
    const int bm = a.m > 128 ? 256 : 128;
    dim3 grid((a.n + BN - 1) / BN, (a.m + bm - 1) / bm);
    size_t lds = (size_t)(bm + 2 * BN) * LDK * sizeof(_Float16);
    if (!attr_set) {
        AXQ_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_kernel<T, 256>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)((256 + 2 * BN) * LDK * 2)), AXQ_ERR_DRIVER);
        attr_set = true;
    }
    if (bm == 256) gemm_kernel<T, 256><<<grid, 512, lds, ctx->stream>>>(a);
    else gemm_kernel<T, 128><<<grid, 256, lds, ctx->stream>>>(a);
    AXQ_LAUNCH_CHECK(ctx, "gemm_kernel");
    return AXQ_OK;
}

} // namespace

int axq_dev_gemm_bf16(axq_ctx *ctx, const axq_weight *w, const uint16_t *x, int m, float *y) {
    if (w->k % BK != 0)
        return axq_fail(ctx, AXQ_ERR_INVALID_BLOCK_SIZE, "Invalid block size: the prefill GEMM needs k %% 64 == 0, got %lld",
                        (long long)w->k);
    if (w->n_rows > INT32_MAX || w->k > INT32_MAX)
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: weight dimensions exceed 2^31");
    // scratch: f16 activations [m, k] then the row scales [m]; kept in the context and grown on demand
    const size_t xh_bytes = axq_align_up((size_t)m * (size_t)w->k * 2, 256), need = xh_bytes + (size_t)m * 4;
    if (ctx->gemm_scratch_bytes < need) {
        AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
        if (ctx->gemm_scratch) (void)hipFree(ctx->gemm_scratch);
        ctx->gemm_scratch = nullptr;
        ctx->gemm_scratch_bytes = 0;
        AXQ_HIP(ctx, hipMalloc(&ctx->gemm_scratch, need), AXQ_ERR_ALLOCATION_FAILED);
        ctx->gemm_scratch_bytes = need;
    }
    _Float16 *xh = reinterpret_cast<_Float16 *>(ctx->gemm_scratch);
    float *rowscale = reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(ctx->gemm_scratch) + xh_bytes);
    gemm_prep_x_kernel<<<m, 256, 0, ctx->stream>>>(x, m, (int)w->k, xh, rowscale);
    GemmArgs a;
    a.codes = w->codes; a.meta = w->meta; a.qh = w->qh;
    a.codes_pitch = w->codes_pitch; a.meta_pitch = w->meta_pitch; a.qh_pitch = w->qh_pitch;
    a.xh = xh; a.rowscale = rowscale; a.y = y;
    a.m = m; a.n = (int)w->n_rows; a.k = (int)w->k;
    int rc;
    switch (w->type) {
    case AXQ_Q4_K: rc = launch_gemm<GQ4K>(ctx, a); break;
    case AXQ_Q4_0: rc = launch_gemm<GQ4x<false>>(ctx, a); break;
    case AXQ_Q4_1: rc = launch_gemm<GQ4x<true>>(ctx, a); break;
    case AXQ_Q5_0: rc = launch_gemm<GQ5x<false>>(ctx, a); break;
    case AXQ_Q5_1: rc = launch_gemm<GQ5x<true>>(ctx, a); break;
    case AXQ_Q8_0: rc = launch_gemm<GQ80>(ctx, a); break;
    case AXQ_F16: rc = launch_gemm<GF16>(ctx, a); break;
    case AXQ_F32: rc = launch_gemm<GF32>(ctx, a); break;
    default: rc = axq_fail(ctx, AXQ_ERR_INVALID_QUANT_TYPE, "Invalid quantization type: %d", w->type);
    }
    return rc;
}
