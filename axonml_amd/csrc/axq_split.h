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

// One task = 8 consecutive elements v[0..7] = x[8*task .. 8*task+7].  The four lanes of an aligned
// lane quad must call this together with four consecutive tasks (task % 4 == lane % 4): they share a
// 32-element group and exchange its maximum and sum through lane shuffles.  `live` = false lanes take
// part in the shuffles (with zeros) and store nothing.
__device__ inline void axq_split8(const float (&v)[8], int task, bool live, uint8_t *planes, uint4 *grp, int kpad) {
    float amax = 0.f, sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        amax = fmaxf(amax, fabsf(v[i]));
        sum += v[i];
    }
    amax = fmaxf(amax, __shfl_xor(amax, 1));
    amax = fmaxf(amax, __shfl_xor(amax, 2));
    sum += __shfl_xor(sum, 1);
    sum += __shfl_xor(sum, 2);
    // amax in [2^e, 2^(e+1)): scale so that |x| * f < 2^27, f = 2^(26-e); limb sums times 2^(e-26) give back x
    uint32_t eb = (__builtin_bit_cast(uint32_t, amax) >> 23) & 0xFF;
    const bool bad = eb == 0xFF;
    eb = eb < 30 ? 30 : eb;
    eb = eb > 254 ? 254 : eb;
    float f = __builtin_bit_cast(float, (280u - eb) << 23);
    float sg = __builtin_bit_cast(float, (eb - 26u) << 23);
    if (bad) sg = __builtin_nanf("");
    uint32_t l[4][2] = {{0, 0}, {0, 0}, {0, 0}, {0, 0}};
    int ls[4] = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 8; i++) {
        int tq = bad ? 0 : (int)rintf(v[i] * f);
        int l3 = ((tq + 64) & 127) - 64;
        tq = (tq - l3) >> 7;
        int l2 = ((tq + 64) & 127) - 64;
        tq = (tq - l2) >> 7;
        int l1 = ((tq + 64) & 127) - 64;
        int l0 = (tq - l1) >> 7;
        int sh = 8 * (i & 3);
        l[0][i >> 2] |= (uint32_t)(l0 & 0xFF) << sh;
        l[1][i >> 2] |= (uint32_t)(l1 & 0xFF) << sh;
        l[2][i >> 2] |= (uint32_t)(l2 & 0xFF) << sh;
        l[3][i >> 2] |= (uint32_t)(l3 & 0xFF) << sh;
        ls[0] += l0; ls[1] += l1; ls[2] += l2; ls[3] += l3;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        ls[i] += __shfl_xor(ls[i], 1);
        ls[i] += __shfl_xor(ls[i], 2);
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < 4; i++)
            *reinterpret_cast<uint2 *>(planes + (size_t)i * kpad + (size_t)task * 8) = make_uint2(l[i][0], l[i][1]);
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
