// GGUF interop: block images in ggml's order <-> the order of the reference's `to_bytes` images.
//
// The reference knows GGUF only as a file extension (crates/axonml-cli/src/commands/quant.rs:218); the
// block layouts below are those of the GGUF / ggml specification.  Q8_0, Q5_0, Q5_1 and Q4_K images are
// byte-identical on both sides.  Q4_0 and Q4_1 differ in where a block's 32 nibbles sit:
//     ggml      : byte j of qs = element j (low nibble) and element j + 16 (high nibble)
//     reference : byte i of data = element 2i (low) and element 2i + 1 (high)   (types.rs:179-198)
// so a block converts by a fixed nibble permutation, scales untouched.  The element formulas agree
// (d * (q - 8), resp. d * q + m), hence a converted tensor dequantises to exactly ggml's values.
#include "axq_internal.h"

namespace {

constexpr int CV_BLOCKS = 256; // blocks per workgroup

// 16 code bytes, ggml order -> reference order
__device__ inline void to_native(const uint32_t (&g)[4], uint32_t (&n)[4]) {
    uint32_t tl[4], th[4];
#pragma unroll
    for (int m = 0; m < 4; m++) {
        const uint32_t lo = g[m] & 0x0F0F0F0Fu, hi = (g[m] >> 4) & 0x0F0F0F0Fu;
        tl[m] = lo | (lo >> 4); // bytes 0 and 2: elements (4m, 4m+1) and (4m+2, 4m+3) as reference bytes
        th[m] = hi | (hi >> 4); // the same for elements 16 + ...
    }
    n[0] = __builtin_amdgcn_perm(tl[1], tl[0], 0x06040200u);
    n[1] = __builtin_amdgcn_perm(tl[3], tl[2], 0x06040200u);
    n[2] = __builtin_amdgcn_perm(th[1], th[0], 0x06040200u);
    n[3] = __builtin_amdgcn_perm(th[3], th[2], 0x06040200u);
}

// 16 code bytes, reference order -> ggml order
__device__ inline void to_ggml(const uint32_t (&n)[4], uint32_t (&g)[4]) {
#pragma unroll
    for (int m = 0; m < 2; m++) {
        // reference bytes 4m..4m+3 hold elements 8m..8m+7, bytes 8+4m.. hold elements 16+8m..
        const uint32_t ae = n[m] & 0x0F0F0F0Fu, ao = (n[m] >> 4) & 0x0F0F0F0Fu;
        const uint32_t be = n[2 + m] & 0x0F0F0F0Fu, bo = (n[2 + m] >> 4) & 0x0F0F0F0Fu;
        const uint32_t lo0 = __builtin_amdgcn_perm(ao, ae, 0x05010400u), lo1 = __builtin_amdgcn_perm(ao, ae, 0x07030602u);
        const uint32_t hi0 = __builtin_amdgcn_perm(bo, be, 0x05010400u), hi1 = __builtin_amdgcn_perm(bo, be, 0x07030602u);
        g[2 * m] = lo0 | (hi0 << 4);
        g[2 * m + 1] = lo1 | (hi1 << 4);
    }
}

// One workgroup converts CV_BLOCKS consecutive blocks of BS bytes (codes at byte HDR of each): coalesced
// 16-byte loads into LDS, one thread per block on the LDS copy, coalesced stores.  src and dst are 16-byte
// aligned; the last workgroup moves its tail byte by byte.
template <int BS, int HDR>
__global__ void __launch_bounds__(CV_BLOCKS) gguf_convert_kernel(const uint8_t *src, uint8_t *dst, // may be the same buffer
                                                                 size_t nblocks, int to_gguf) {
    __shared__ __attribute__((aligned(16))) uint8_t buf[CV_BLOCKS * BS];
    const size_t b0 = (size_t)blockIdx.x * CV_BLOCKS;
    const int nb = (int)((nblocks - b0) < (size_t)CV_BLOCKS ? (nblocks - b0) : (size_t)CV_BLOCKS);
    const int bytes = nb * BS, n16 = bytes >> 4;
    const uint8_t *s = src + b0 * BS;
    uint8_t *d = dst + b0 * BS;
    for (int i = threadIdx.x; i < n16; i += CV_BLOCKS) reinterpret_cast<uint4 *>(buf)[i] = reinterpret_cast<const uint4 *>(s)[i];
    for (int i = (n16 << 4) + threadIdx.x; i < bytes; i += CV_BLOCKS) buf[i] = s[i];
    __syncthreads();
    if ((int)threadIdx.x < nb) {
        uint16_t *q = reinterpret_cast<uint16_t *>(buf + threadIdx.x * BS + HDR); // block sizes and headers are even
        uint32_t in[4], out[4];
#pragma unroll
        for (int m = 0; m < 4; m++) in[m] = (uint32_t)q[2 * m] | ((uint32_t)q[2 * m + 1] << 16);
        if (to_gguf) to_ggml(in, out); else to_native(in, out);
#pragma unroll
        for (int m = 0; m < 4; m++) {
            q[2 * m] = (uint16_t)(out[m] & 0xFFFF);
            q[2 * m + 1] = (uint16_t)(out[m] >> 16);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n16; i += CV_BLOCKS) reinterpret_cast<uint4 *>(d)[i] = reinterpret_cast<const uint4 *>(buf)[i];
    for (int i = (n16 << 4) + threadIdx.x; i < bytes; i += CV_BLOCKS) d[i] = buf[i];
}

int dev_convert(axq_ctx *ctx, int type, const uint8_t *src, uint8_t *dst, size_t nblocks, int to_gguf) {
    const size_t bytes = nblocks * axq_type_bytes_per_block(type);
    if (type != AXQ_Q4_0 && type != AXQ_Q4_1) { // identical images
        if (src != dst) AXQ_HIP(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
        return AXQ_OK;
    }
    if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_gguf_convert_blocks: device pointers must be 16-byte aligned");
    const unsigned grid = (unsigned)((nblocks + CV_BLOCKS - 1) / CV_BLOCKS);
    if (type == AXQ_Q4_0) gguf_convert_kernel<18, 2><<<grid, CV_BLOCKS, 0, ctx->stream>>>(src, dst, nblocks, to_gguf);
    else gguf_convert_kernel<20, 4><<<grid, CV_BLOCKS, 0, ctx->stream>>>(src, dst, nblocks, to_gguf);
    AXQ_LAUNCH_CHECK(ctx, "gguf_convert_kernel");
    return AXQ_OK;
}

struct Temp { // a device buffer that is released when the call returns
    void *p = nullptr;
    ~Temp() { if (p) (void)hipFree(p); }
};

} // namespace

extern "C" {

// ggml_type numbers of the GGUF tensor table -> quantization type of this library, or -1.
int axq_type_from_ggml(int ggml_type) {
    switch (ggml_type) {
    case 0: return AXQ_F32;
    case 1: return AXQ_F16;
    case 2: return AXQ_Q4_0;
    case 3: return AXQ_Q4_1;
    case 6: return AXQ_Q5_0;
    case 7: return AXQ_Q5_1;
    case 8: return AXQ_Q8_0;
    case 12: return AXQ_Q4_K;
    case 13: return AXQ_Q5_K;
    case 14: return AXQ_Q6_K;
    default: return -1;
    }
}

int axq_type_to_ggml(int type) {
    switch (type) {
    case AXQ_F32: return 0;
    case AXQ_F16: return 1;
    case AXQ_Q4_0: return 2;
    case AXQ_Q4_1: return 3;
    case AXQ_Q5_0: return 6;
    case AXQ_Q5_1: return 7;
    case AXQ_Q8_0: return 8;
    case AXQ_Q4_K: return 12;
    case AXQ_Q5_K: return 13;
    case AXQ_Q6_K: return 14;
    default: return -1;
    }
}

int axq_gguf_convert_blocks(axq_ctx *ctx, int type, const void *src, void *dst, size_t nblocks, int direction, int mem) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_gguf_convert_blocks: NULL context");
    if (axq_type_to_ggml(type) < 0) return axq_fail(ctx, AXQ_ERR_INVALID_QUANT_TYPE, "Invalid quantization type: %d", type);
    if (mem != AXQ_MEM_HOST && mem != AXQ_MEM_DEVICE) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "bad memory space %d", mem);
    if (direction != AXQ_GGUF_TO_NATIVE && direction != AXQ_NATIVE_TO_GGUF)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_gguf_convert_blocks: bad direction %d", direction);
    if (nblocks == 0) return AXQ_OK;
    if (!src || !dst) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_gguf_convert_blocks: NULL pointer");
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    const size_t bytes = nblocks * axq_type_bytes_per_block(type);
    if (mem == AXQ_MEM_DEVICE) return dev_convert(ctx, type, (const uint8_t *)src, (uint8_t *)dst, nblocks, direction);
    if (type != AXQ_Q4_0 && type != AXQ_Q4_1) { // identical images: nothing for the device to do
        if (src != dst) memmove(dst, src, bytes);
        return AXQ_OK;
    }
    Temp t;
    AXQ_HIP(ctx, hipMalloc(&t.p, bytes), AXQ_ERR_ALLOCATION_FAILED);
    AXQ_HIP(ctx, hipMemcpyAsync(t.p, src, bytes, hipMemcpyHostToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    int rc = dev_convert(ctx, type, (const uint8_t *)t.p, (uint8_t *)t.p, nblocks, direction);
    if (rc) return rc;
    AXQ_HIP(ctx, hipMemcpyAsync(dst, t.p, bytes, hipMemcpyDeviceToHost, ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

} // extern "C"
