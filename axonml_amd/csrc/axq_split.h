// Splitting an activation vector into int8 limbs for the matrix-pipe GEMV (device code, header only).
//
// Split form of x[K] ("xq"): four int8 planes of kpad = round_up(K, 16) bytes, then one 16-byte record
// per 32-element group g:
//     x[k] ~= sg * (l0[k]*128^3 + l1[k]*128^2 + l2[k]*128 + l3[k]),   |l_i| <= 64,  g = k / 32
//     record = { f32 sg; f32 xs = sum of x over the group; i16 L[4] = sum of each limb over the group }
// sg is a power of two chosen from the group's largest magnitude so that the limbs hold 28 bits below
// it; a group holding inf or nan gets a nan scale, so that the dot product comes out nan.  The limb
// sums let a kernel centre unsigned weight codes exactly, in integers: sum (n - c) l_i = D_i - c L_i.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

__host__ __device__ static inline size_t axq_split_bytes(int64_t k) {
    return (size_t)4 * (size_t)((k + 15) & ~15) + (size_t)((k + 31) / 32) * 16;
}

// lane ^ 1 and lane ^ 2 within a quad, as one DPP move each
__device__ inline float axq_quad_xor1(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));
}
__device__ inline float axq_quad_xor2(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true));
}
__device__ inline int axq_quad_xor1(int v) { return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, true); }
__device__ inline int axq_quad_xor2(int v) { return __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, true); }

// One task = 8 consecutive elements v[0..7] = x[8*task .. 8*task+7].  The four lanes of an aligned
// lane quad must call this together with four consecutive tasks (task % 4 == lane % 4): they share a
// 32-element group and exchange its maximum and sum through DPP quad moves.  `live` = false lanes take
// part in the shuffles (with zeros) and store nothing.
// The arithmetic of a task: limb bytes pk[limb][dword] (limb 0 most significant; dword 0 = elements 0..3),
// the group's scale, plain sum and limb sums (the latter three equal in the four lanes of the quad).
__device__ inline void axq_split8_compute(const float (&v)[8], uint32_t (&pk)[4][2], float &sg, float &sum, int (&ls)[4]) {
    // largest magnitude as an integer maximum of the sign-less bit patterns: a nan ranks above everything
    // (a float maximum would drop it, and the nan would then count as zero)
    uint32_t amax = 0;
    sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t m = __builtin_bit_cast(uint32_t, v[i]) & 0x7FFFFFFFu;
        amax = amax > m ? amax : m;
        sum += v[i];
    }
    {
        const uint32_t o1 = (uint32_t)axq_quad_xor1((int)amax);
        amax = amax > o1 ? amax : o1;
        const uint32_t o2 = (uint32_t)axq_quad_xor2((int)amax);
        amax = amax > o2 ? amax : o2;
    }
    sum += axq_quad_xor1(sum);
    sum += axq_quad_xor2(sum);
    // amax in [2^e, 2^(e+1)): scale so that |x| * f < 2^27, f = 2^(26-e); limb sums times 2^(e-26) give back x
    uint32_t eb = amax >> 23;
    const bool bad = eb == 0xFF;
    eb = eb < 30 ? 30 : eb;
    eb = eb > 254 ? 254 : eb;
    float f = __builtin_bit_cast(float, (280u - eb) << 23);
    sg = __builtin_bit_cast(float, (eb - 26u) << 23);
    if (bad) sg = __builtin_nanf("");
    // t = rint(x f) = sum_i l_i 128^i with balanced digits; adding 64 (1 + 128 + 128^2 + 128^3) makes every
    // digit non-negative, d_i = l_i + 64 in 0..127 (the top one up to 128), so that plain bit fields extract
    // them; bytes go back to l_i = d_i - 64 four at a time: (d + 64) ^ 0x80 is d - 64 modulo 256.
#pragma unroll
    for (int i = 0; i < 4; i++) pk[i][0] = pk[i][1] = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t u = (uint32_t)((bad ? 0 : (int)rintf(v[i] * f)) + 135274560);
        const int sh = 8 * (i & 3);
        pk[3][i >> 2] |= (u & 127u) << sh;
        pk[2][i >> 2] |= ((u >> 7) & 127u) << sh;
        pk[1][i >> 2] |= ((u >> 14) & 127u) << sh;
        pk[0][i >> 2] |= (u >> 21) << sh;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        ls[i] = (int)__builtin_amdgcn_sad_u8(pk[i][0], 0u, __builtin_amdgcn_sad_u8(pk[i][1], 0u, 0u)) - 512;
        ls[i] += axq_quad_xor1(ls[i]);
        ls[i] += axq_quad_xor2(ls[i]);
        pk[i][0] = (pk[i][0] + 0x40404040u) ^ 0x80808080u;
        pk[i][1] = (pk[i][1] + 0x40404040u) ^ 0x80808080u;
    }
}

__device__ inline void axq_split8(const float (&v)[8], int task, bool live, uint8_t *planes, uint4 *grp, int kpad) {
    uint32_t pk[4][2];
    float sg, sum;
    int ls[4];
    axq_split8_compute(v, pk, sg, sum, ls);
    if (live) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            *reinterpret_cast<uint2 *>(planes + (size_t)i * kpad + (size_t)task * 8) = make_uint2(pk[i][0], pk[i][1]);
        if ((task & 3) == 0)
            grp[task >> 2] = make_uint4(__builtin_bit_cast(uint32_t, sg), __builtin_bit_cast(uint32_t, sum),
                                        (uint32_t)(ls[0] & 0xFFFF) | ((uint32_t)ls[1] << 16),
                                        (uint32_t)(ls[2] & 0xFFFF) | ((uint32_t)ls[3] << 16));
    }
}

// x[k] (any address space) -> split form, by `nthreads` threads of which this is number `tid`
// (nthreads a multiple of 4, k a multiple of 32).
__device__ inline void stage_x(const float *x, int k, uint8_t *planes, uint4 *grp, int tid, int nthreads) {
    const int kpad = (k + 15) & ~15;
    const int ntask = (k + 7) >> 3;
    const int ntask_pad = (ntask + 3) & ~3;
    for (int t = tid; t < ntask_pad; t += nthreads) {
        float v[8];
        const bool live = t < ntask;
        if (live) {
            const float4 *p = reinterpret_cast<const float4 *>(x + (size_t)t * 8);
            float4 a = p[0], b = p[1];
            v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = 0.f;
        }
        axq_split8(v, t, live, planes, grp, kpad);
    }
}

// ---- operands of the small-batch GEMV (2..8 vectors on the 32x32x32 int8 product) -------------------------
// Scratch of a K-wide call: 32 K bytes of A operands (per 32-element block two halves of 32 rows x 16 bytes,
// row 4 b + l = limb l of vector b), then 2 * (K / 32) * 8 floats: the blocks' scales, then their sums.

// bytes {0, 2} of lo and of hi (sel = 0) or bytes {1, 3} of each (sel = 1)
__device__ inline int axq_pick_alt(uint32_t lo, uint32_t hi, int sel) {
    return (int)__builtin_amdgcn_perm(hi, lo, sel ? 0x07050301u : 0x06040200u);
}

// Eight consecutive elements (task t) of vector b -> their limbs in the A operands and, from the first task of a
// 32-element block, the block's scale and sum.  The four tasks of a block sit in four consecutive lanes, which
// all have to call this together.
template <bool EVEN_ODD>
__device__ inline void axq_store_packed(const float (&v)[8], int t, int b, int batch, int nblk, uint8_t *xa, float *xsg) {
    uint32_t pk[4][2];
    float sg, sum;
    int ls[4];
    axq_split8_compute(v, pk, sg, sum, ls);
    if (b >= batch) { sg = 0.f; sum = 0.f; }
    const int blk = t >> 2, e0 = (t & 3) * 8; // first element of the task inside its block
#pragma unroll
    for (int l = 0; l < 4; l++) {
        const int row = 4 * b + l;
        if (EVEN_ODD) {
            uint8_t *d0 = xa + ((size_t)(blk * 2 + 0) * 32 + row) * 16 + (e0 >> 1);
            uint8_t *d1 = xa + ((size_t)(blk * 2 + 1) * 32 + row) * 16 + (e0 >> 1);
            *reinterpret_cast<uint32_t *>(d0) = (uint32_t)axq_pick_alt(pk[l][0], pk[l][1], 0);
            *reinterpret_cast<uint32_t *>(d1) = (uint32_t)axq_pick_alt(pk[l][0], pk[l][1], 1);
        } else {
            uint8_t *d = xa + ((size_t)(blk * 2 + (e0 >> 4)) * 32 + row) * 16 + (e0 & 15);
            *reinterpret_cast<uint2 *>(d) = make_uint2(pk[l][0], pk[l][1]);
        }
    }
    if ((t & 3) == 0) {
        const int slot = (blk * 2 + (b & 1)) * 4 + (b >> 1);
        xsg[slot] = sg;
        xsg[(size_t)nblk * 8 + slot] = sum;
    }
}
