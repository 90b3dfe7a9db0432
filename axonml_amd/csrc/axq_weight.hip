// Codec and weight entry points of the C ABI (host-side staging around the
// device kernels of axq_codec.hip).
#include <stdlib.h>

#include <stdio.h>
#include <stdlib.h>
#include <new>

#include <algorithm>
#include <vector>

#include "axq_internal.h"

namespace {

// RAII for a temporary device buffer on the context's stream.
struct DevTemp {
    axq_ctx *ctx;
    void *p = nullptr;
    explicit DevTemp(axq_ctx *c) : ctx(c) {}
    hipError_t alloc(size_t bytes) { return hipMalloc(&p, bytes ? bytes : 1); }
    ~DevTemp() {
        if (p) {
            (void)hipStreamSynchronize(ctx->stream);
            (void)hipFree(p);
        }
    }
};

int check_type(axq_ctx *ctx, int type) {
    if (axq_type_block_size(type) == 0)
        return axq_fail(ctx, AXQ_ERR_INVALID_QUANT_TYPE, "Invalid quantization type: %d", type);
    return AXQ_OK;
}

int check_mem(axq_ctx *ctx, int mem) {
    if (mem != AXQ_MEM_HOST && mem != AXQ_MEM_DEVICE)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "mem must be AXQ_MEM_HOST or AXQ_MEM_DEVICE, got %d", mem);
    return AXQ_OK;
}

} // namespace

int axq_weight_alloc(axq_ctx *ctx, int type, int64_t n_rows, int64_t k, axq_weight **out) {
    size_t bs = axq_type_block_size(type);
    if (n_rows <= 0 || k <= 0)
        return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: weight must be [n_rows>0, k>0], got [%lld, %lld]",
                        (long long)n_rows, (long long)k);
    if ((size_t)k % bs != 0)
        return axq_fail(ctx, AXQ_ERR_INVALID_BLOCK_SIZE,
                        "Invalid block size: k=%lld is not a multiple of the %zu-element block of %s", (long long)k, bs,
                        axq_type_name(type));
    axq_weight *w = (axq_weight *)calloc(1, sizeof(axq_weight));
    if (!w) return axq_fail(ctx, AXQ_ERR_ALLOCATION_FAILED, "out of host memory");
    w->type = type;
    w->n_rows = n_rows;
    w->k = k;
    w->packed_bytes = axq_packed_bytes(type, (size_t)n_rows * (size_t)k);
    size_t nblk = (size_t)k / bs;
    size_t meta_per_block = 0, qh_per_block = 0;
    switch (type) {
    case AXQ_Q8_0: w->codes_pitch = (size_t)k; meta_per_block = 2; break;
    case AXQ_Q4_0: w->codes_pitch = (size_t)k / 2; meta_per_block = 2; break;
    case AXQ_Q4_1: w->codes_pitch = (size_t)k / 2; meta_per_block = 4; break;
    case AXQ_Q5_0: w->codes_pitch = (size_t)k / 2; meta_per_block = 2; qh_per_block = 4; break;
    case AXQ_Q5_1: w->codes_pitch = (size_t)k / 2; meta_per_block = 4; qh_per_block = 4; break;
    case AXQ_Q4_K: w->codes_pitch = (size_t)k / 2; meta_per_block = 16; break;
    case AXQ_Q6_K: w->codes_pitch = (size_t)k / 2; meta_per_block = 18; qh_per_block = 64; break; // scales, then the row's d values
    case AXQ_Q5_K: w->codes_pitch = (size_t)k / 2; meta_per_block = 16; qh_per_block = 32; break; // Q4_K's planes and the fifth bits as they are
    case AXQ_F16: w->codes_pitch = (size_t)k * 2; break;
    case AXQ_F32: w->codes_pitch = (size_t)k * 4; break;
    }
    w->meta_pitch = type == AXQ_Q6_K ? axq_align_up(nblk * meta_per_block, 16) : nblk * meta_per_block;
    w->qh_pitch = nblk * qh_per_block;
    size_t codes_bytes = axq_align_up(w->codes_pitch * (size_t)n_rows, 256);
    size_t meta_bytes = axq_align_up(w->meta_pitch * (size_t)n_rows, 256);
    size_t qh_bytes = axq_align_up(w->qh_pitch * (size_t)n_rows, 256);
    // 64 bytes of slack: the GEMV kernels may read (and discard) up to one
    // 16-byte vector past the last real byte of a plane.
    w->alloc_bytes = codes_bytes + meta_bytes + qh_bytes + 256;
    hipError_t e = hipMalloc((void **)&w->base, w->alloc_bytes);
    if (e != hipSuccess) {
        free(w);
        return axq_fail(ctx, AXQ_ERR_ALLOCATION_FAILED, "hipMalloc(%zu): %s", w->alloc_bytes, hipGetErrorString(e));
    }
    w->codes = w->base;
    w->meta = w->base + codes_bytes;
    w->qh = w->meta + meta_bytes;
    w->owns = true;
    // zero the padding so that stray vector reads are deterministic
    e = hipMemsetAsync(w->base, 0, w->alloc_bytes, ctx->stream);
    if (e != hipSuccess) {
        (void)hipFree(w->base);
        free(w);
        return axq_fail(ctx, AXQ_ERR_DRIVER, "hipMemsetAsync: %s", hipGetErrorString(e));
    }
    *out = w;
    return AXQ_OK;
}

// Plain 16-byte-per-lane copy: reads `n16*16` bytes and writes as many.  Used to calibrate the memory
// counters of a profiler run against a kernel whose traffic is known.
__global__ void axq_copy16_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

// A barrier over every workgroup of one launch, through device-scope atomics, timed: what a kernel that stays resident
// across the steps of a decode layer would pay where separate kernels pay a launch boundary.  Each of `rounds` rounds:
// every thread publishes `publish_bytes` / threads of data with device-scope stores and waits for their acknowledgement,
// the workgroup counts itself in and polls (bounded: a round nobody completes sets `fail` and the kernel ends all the
// same).  levels = 1: one counter; 2: 16 groups of workgroups count in separately, the last of a group counts the group
// in, the last group writes a release word that everybody polls.
constexpr int BARRIER_WORDS = 18 * 32;
__global__ void __launch_bounds__(256) grid_barrier_kernel(int *words, int *fail, float *data, long long *stamps, int rounds, int levels,
                                                          int floats_per_thread) {
    const int tid = threadIdx.x, wg = blockIdx.x, nwg = gridDim.x;
    for (int r = 0; r < rounds; r++) {
        const long long t0 = wall_clock64();
        for (int i = 0; i < floats_per_thread; i++)
            __hip_atomic_store(data + ((size_t)wg * floats_per_thread + i) * 256 + tid, (float)(r + wg), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        const long long t1 = wall_clock64();
        if (tid == 0) {
            // a round's words lie 128 bytes apart (polls and counts on one line queue behind each other): the one counter or
            // the groups' counter, the release word, sixteen group counters
            int *base = words + (size_t)r * BARRIER_WORDS;
            int spins = 0, v = 0;
            if (levels == 1) {
                __hip_atomic_fetch_add(base, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                while ((v = __hip_atomic_load(base, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) < nwg && ++spins < (1 << 18)) __builtin_amdgcn_s_sleep(2);
                if (v < nwg) atomicExch(fail, 1);
            } else {
                const int g = wg & 15, in_group = (nwg - g + 15) / 16;
                if (__hip_atomic_fetch_add(base + (2 + g) * 32, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == in_group - 1)
                    if (__hip_atomic_fetch_add(base, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (nwg < 16 ? nwg : 16) - 1)
                        __hip_atomic_store(base + 32, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                while ((v = __hip_atomic_load(base + 32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) == 0 && ++spins < (1 << 18)) __builtin_amdgcn_s_sleep(2);
                if (v == 0) atomicExch(fail, 1);
            }
        }
        __syncthreads();
        const long long t2 = wall_clock64();
        if (tid == 0) {
            long long *st = stamps + ((size_t)r * nwg + wg) * 3;
            st[0] = t0; st[1] = t1; st[2] = t2;
        }
    }
}


// Reads `n16*16` bytes and keeps nothing: what the memory system gives a launch that only streams a weight.  Each
// workgroup takes one contiguous share and keeps U 16-byte loads per lane in flight (non-temporal when NT); a lane whose
// index lies past the workgroup's share re-reads the share's last element (a cache hit), so that the bytes fetched
// from memory are the image's own and no more.
typedef uint32_t axq_u32x4 __attribute__((ext_vector_type(4)));
template <int U, bool NT, int TPB>
__global__ void __launch_bounds__(TPB) axq_read_kernel(const axq_u32x4 *__restrict__ src, size_t n16, uint32_t *sink) {
    const size_t share = (n16 + gridDim.x - 1) / gridDim.x;
    const size_t lo = (size_t)blockIdx.x * share, hi = lo + share < n16 ? lo + share : n16;
    uint32_t acc = 0;
    for (size_t i = lo + threadIdx.x; i < hi; i += (size_t)U * TPB) {
        axq_u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            size_t j = i + (size_t)u * TPB;
            j = j < hi ? j : hi - 1;
            v[u] = NT ? __builtin_nontemporal_load(src + j) : src[j];
        }
#pragma unroll
        for (int u = 0; u < U; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x9E3779B9u) sink[0] = acc; // keeps the loads alive; a match writes four bytes of no consequence
}

// The same bytes in the order the one-vector GEMV asks for them: a workgroup of eight waves owns `rows` consecutive rows of
// the code plane (pitch bytes each, 2048 of them used), wave (g, s) walks the 4-row steps of half g and reads, per step,
// two pieces of 256 bytes of each of the step's four rows (lane = (16-byte chunk, row)), NB steps in flight.
template <int NB, int LIN = 0>
__global__ void __launch_bounds__(512) axq_read_rows_kernel(const uint8_t *__restrict__ codes, size_t pitch, int n_rows, int rows_per_wg, uint32_t *sink) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = wave >> 2, s = wave & 3;
    const int blk = lane >> 2, j = lane & 3;
    const int half_rows = rows_per_wg / 2, steps = half_rows / 4;
    const int row0 = blockIdx.x * rows_per_wg + g * half_rows + j;
    uint32_t acc = 0;
    for (int st = 0; st < steps; st += NB) {
        axq_u32x4 v[NB][2];
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const int sb = st + b < steps ? st + b : 0;
            int row = row0 + 4 * sb;
            row = row < n_rows ? row : n_rows - 1;
            const uint8_t *p = codes + (size_t)row * pitch + s * 256 + blk * 16;
            size_t second = 1024;
            if (LIN == 1) { // the same bytes per wave and step (2 KB), each wave walking a contiguous run of its own
                size_t off = (((size_t)blockIdx.x * 8 + wave) * steps + sb) * 2048;
                const size_t total = (size_t)n_rows * pitch;
                off = off + 2048 <= total ? off : 0;
                p = codes + off + lane * 16;
            } else if (LIN == 2) { // ... the workgroup's eight waves side by side, the workgroup walking one contiguous run
                size_t off = (((size_t)blockIdx.x * steps + sb) * 8 + wave) * 2048;
                const size_t total = (size_t)n_rows * pitch;
                off = off + 2048 <= total ? off : 0;
                p = codes + off + lane * 16;
            }
            v[b][0] = __builtin_nontemporal_load(reinterpret_cast<const axq_u32x4 *>(p));
            v[b][1] = __builtin_nontemporal_load(reinterpret_cast<const axq_u32x4 *>(p + second));
        }
#pragma unroll
        for (int b = 0; b < NB; b++) acc ^= v[b][0].x ^ v[b][0].w ^ v[b][1].y ^ v[b][1].z;
    }
    if (acc == 0x9E3779B9u) sink[0] = acc;
}

template <int U, bool NT>
static void launch_read(int threads, unsigned grid, hipStream_t st, const axq_u32x4 *src, size_t n16, uint32_t *sink) {
    if (threads == 256) axq_read_kernel<U, NT, 256><<<grid, 256, 0, st>>>(src, n16, sink);
    else if (threads == 512) axq_read_kernel<U, NT, 512><<<grid, 512, 0, st>>>(src, n16, sink);
    else axq_read_kernel<(U > 16 ? 16 : U), NT, 1024><<<grid, 1024, 0, st>>>(src, n16, sink); // 1024 threads: 128 registers each
}
template <bool NT>
static void launch_read_u(int in_flight, int threads, unsigned grid, hipStream_t st, const axq_u32x4 *src, size_t n16, uint32_t *sink) {
    if (in_flight <= 4) launch_read<4, NT>(threads, grid, st, src, n16, sink);
    else if (in_flight <= 8) launch_read<8, NT>(threads, grid, st, src, n16, sink);
    else if (in_flight <= 16) launch_read<16, NT>(threads, grid, st, src, n16, sink);
    else launch_read<32, NT>(threads, grid, st, src, n16, sink);
}

// Streams beside the context's own, for launches that may overlap (benchmarks only; default priority).  The first use
// creates them; axq_destroy releases them.
int axq_aux_streams(axq_ctx *ctx, int n) {
    if (n > AXQ_AUX_STREAMS) n = AXQ_AUX_STREAMS;
    for (int i = 0; i < n; i++) {
        if (!ctx->aux_stream[i]) AXQ_HIP(ctx, hipStreamCreateWithFlags(&ctx->aux_stream[i], hipStreamNonBlocking), AXQ_ERR_DRIVER);
        if (!ctx->aux_event[i]) AXQ_HIP(ctx, hipEventCreateWithFlags(&ctx->aux_event[i], hipEventDisableTiming), AXQ_ERR_DRIVER);
    }
    if (!ctx->aux_fork) AXQ_HIP(ctx, hipEventCreateWithFlags(&ctx->aux_fork, hipEventDisableTiming), AXQ_ERR_DRIVER);
    return AXQ_OK;
}
// Everything enqueued on the context's stream so far happens before what the first n side streams get next ...
int axq_aux_fork(axq_ctx *ctx, int n) {
    AXQ_HIP(ctx, hipEventRecord(ctx->aux_fork, ctx->stream), AXQ_ERR_DRIVER);
    for (int i = 0; i < n; i++) AXQ_HIP(ctx, hipStreamWaitEvent(ctx->aux_stream[i], ctx->aux_fork, 0), AXQ_ERR_DRIVER);
    return AXQ_OK;
}
// ... and what they have been given happens before whatever the context's stream gets next.
int axq_aux_join(axq_ctx *ctx, int n) {
    for (int i = 0; i < n; i++) {
        AXQ_HIP(ctx, hipEventRecord(ctx->aux_event[i], ctx->aux_stream[i]), AXQ_ERR_DRIVER);
        AXQ_HIP(ctx, hipStreamWaitEvent(ctx->stream, ctx->aux_event[i], 0), AXQ_ERR_DRIVER);
    }
    return AXQ_OK;
}

extern "C" {

int axq_quantize(axq_ctx *ctx, int type, const float *src, size_t numel, void *packed, int mem) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_quantize: NULL context");
    int rc;
    if ((rc = check_type(ctx, type)) || (rc = check_mem(ctx, mem))) return rc;
    if (numel == 0) return AXQ_OK;
    if (!src || !packed) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_quantize: NULL pointer");
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    size_t bytes = axq_packed_bytes(type, numel);
    if (mem == AXQ_MEM_DEVICE) return axq_dev_quantize(ctx, type, src, numel, (uint8_t *)packed);
    DevTemp dsrc(ctx), dout(ctx);
    AXQ_HIP(ctx, dsrc.alloc(numel * 4), AXQ_ERR_ALLOCATION_FAILED);
    AXQ_HIP(ctx, dout.alloc(bytes), AXQ_ERR_ALLOCATION_FAILED);
    AXQ_HIP(ctx, hipMemcpyAsync(dsrc.p, src, numel * 4, hipMemcpyHostToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    if ((rc = axq_dev_quantize(ctx, type, (const float *)dsrc.p, numel, (uint8_t *)dout.p))) return rc;
    AXQ_HIP(ctx, hipMemcpyAsync(packed, dout.p, bytes, hipMemcpyDeviceToHost, ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_dequantize(axq_ctx *ctx, int type, const void *packed, size_t numel, float *dst, int mem) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_dequantize: NULL context");
    int rc;
    if ((rc = check_type(ctx, type)) || (rc = check_mem(ctx, mem))) return rc;
    if (numel == 0) return AXQ_OK;
    if (!dst || !packed) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_dequantize: NULL pointer");
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    size_t bytes = axq_packed_bytes(type, numel);
    if (mem == AXQ_MEM_DEVICE) return axq_dev_dequantize(ctx, type, (const uint8_t *)packed, numel, dst);
    DevTemp dsrc(ctx), dout(ctx);
    AXQ_HIP(ctx, dsrc.alloc(bytes), AXQ_ERR_ALLOCATION_FAILED);
    AXQ_HIP(ctx, dout.alloc(numel * 4), AXQ_ERR_ALLOCATION_FAILED);
    AXQ_HIP(ctx, hipMemcpyAsync(dsrc.p, packed, bytes, hipMemcpyHostToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    if ((rc = axq_dev_dequantize(ctx, type, (const uint8_t *)dsrc.p, numel, (float *)dout.p))) return rc;
    AXQ_HIP(ctx, hipMemcpyAsync(dst, dout.p, numel * 4, hipMemcpyDeviceToHost, ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_weight_upload(axq_ctx *ctx, int type, int64_t n_rows, int64_t k, const void *packed, size_t bytes, int mem,
                      axq_weight **out) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_weight_upload: NULL context");
    if (!out || !packed) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_weight_upload: NULL pointer");
    *out = NULL;
    int rc;
    if ((rc = check_type(ctx, type)) || (rc = check_mem(ctx, mem))) return rc;
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    axq_weight *w = NULL;
    if ((rc = axq_weight_alloc(ctx, type, n_rows, k, &w))) return rc;
    if (bytes != w->packed_bytes) {
        rc = axq_fail(ctx, AXQ_ERR_DATA_LENGTH_MISMATCH, "Data length mismatch: expected %zu, got %zu", w->packed_bytes,
                      bytes);
        axq_weight_free(ctx, w);
        return rc;
    }
    if (mem == AXQ_MEM_DEVICE) {
        rc = axq_dev_repack(ctx, w, (uint8_t *)packed, true);
    } else {
        DevTemp tmp(ctx);
        hipError_t e = tmp.alloc(bytes);
        if (e == hipSuccess) e = hipMemcpyAsync(tmp.p, packed, bytes, hipMemcpyHostToDevice, ctx->stream);
        if (e != hipSuccess)
            rc = axq_fail(ctx, AXQ_ERR_COPY_FAILED, "staging upload: %s", hipGetErrorString(e));
        else
            rc = axq_dev_repack(ctx, w, (uint8_t *)tmp.p, true);
    }
    if (rc) {
        axq_weight_free(ctx, w);
        return rc;
    }
    *out = w;
    return AXQ_OK;
}

int axq_weight_quantize(axq_ctx *ctx, int type, int64_t n_rows, int64_t k, const float *wsrc, int mem, axq_weight **out) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_weight_quantize: NULL context");
    if (!out || !wsrc) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_weight_quantize: NULL pointer");
    *out = NULL;
    int rc;
    if ((rc = check_type(ctx, type)) || (rc = check_mem(ctx, mem))) return rc;
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    axq_weight *w = NULL;
    if ((rc = axq_weight_alloc(ctx, type, n_rows, k, &w))) return rc;
    size_t numel = (size_t)n_rows * (size_t)k;
    {
        DevTemp fsrc(ctx), img(ctx);
        const float *src_dev = wsrc;
        hipError_t e = hipSuccess;
        if (mem == AXQ_MEM_HOST) {
            e = fsrc.alloc(numel * 4);
            if (e == hipSuccess) e = hipMemcpyAsync(fsrc.p, wsrc, numel * 4, hipMemcpyHostToDevice, ctx->stream);
            src_dev = (const float *)fsrc.p;
        }
        if (e == hipSuccess) e = img.alloc(w->packed_bytes);
        if (e != hipSuccess)
            rc = axq_fail(ctx, AXQ_ERR_ALLOCATION_FAILED, "staging quantize: %s", hipGetErrorString(e));
        if (!rc) rc = axq_dev_quantize(ctx, type, src_dev, numel, (uint8_t *)img.p);
        if (!rc) rc = axq_dev_repack(ctx, w, (uint8_t *)img.p, true);
    }
    if (rc) {
        axq_weight_free(ctx, w);
        return rc;
    }
    *out = w;
    return AXQ_OK;
}

int axq_weight_download(axq_ctx *ctx, const axq_weight *w, void *packed, size_t bytes, int mem) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_weight_download: NULL context");
    if (!w || !packed) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_weight_download: NULL pointer");
    int rc;
    if ((rc = check_mem(ctx, mem))) return rc;
    if (bytes != w->packed_bytes)
        return axq_fail(ctx, AXQ_ERR_DATA_LENGTH_MISMATCH, "Data length mismatch: expected %zu, got %zu", w->packed_bytes,
                        bytes);
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    if (mem == AXQ_MEM_DEVICE) return axq_dev_repack(ctx, w, (uint8_t *)packed, false);
    DevTemp tmp(ctx);
    AXQ_HIP(ctx, tmp.alloc(bytes), AXQ_ERR_ALLOCATION_FAILED);
    if ((rc = axq_dev_repack(ctx, w, (uint8_t *)tmp.p, false))) return rc;
    AXQ_HIP(ctx, hipMemcpyAsync(packed, tmp.p, bytes, hipMemcpyDeviceToHost, ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_weight_info(const axq_weight *w, int *type, int64_t *n_rows, int64_t *k, size_t *bytes) {
    if (!w) return AXQ_ERR_INVALID_ARGUMENT;
    if (type) *type = w->type;
    if (n_rows) *n_rows = w->n_rows;
    if (k) *k = w->k;
    if (bytes) *bytes = w->packed_bytes;
    return AXQ_OK;
}

void axq_weight_free(axq_ctx *ctx, axq_weight *w) {
    if (!w) return;
    if (w->owns && w->base) {
        if (ctx) (void)hipStreamSynchronize(ctx->stream);
        (void)hipFree(w->base);
    }
    free(w);
}

int axq_gemv_f32(axq_ctx *ctx, const axq_weight *w, const float *x, int batch, const float *bias, float *y, int mem) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_gemv_f32: NULL context");
    if (!w || !x || !y) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_gemv_f32: NULL pointer");
    int rc;
    if ((rc = check_mem(ctx, mem))) return rc;
    if (batch <= 0) return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: batch must be positive, got %d", batch);
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    if (mem == AXQ_MEM_DEVICE) return axq_dev_gemv(ctx, w, x, batch, bias, y);
    size_t xb = (size_t)batch * (size_t)w->k * 4, yb = (size_t)batch * (size_t)w->n_rows * 4;
    DevTemp dx(ctx), dy(ctx), db(ctx);
    AXQ_HIP(ctx, dx.alloc(xb), AXQ_ERR_ALLOCATION_FAILED);
    AXQ_HIP(ctx, dy.alloc(yb), AXQ_ERR_ALLOCATION_FAILED);
    AXQ_HIP(ctx, hipMemcpyAsync(dx.p, x, xb, hipMemcpyHostToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    if (bias) {
        AXQ_HIP(ctx, db.alloc((size_t)w->n_rows * 4), AXQ_ERR_ALLOCATION_FAILED);
        AXQ_HIP(ctx, hipMemcpyAsync(db.p, bias, (size_t)w->n_rows * 4, hipMemcpyHostToDevice, ctx->stream),
                AXQ_ERR_COPY_FAILED);
    }
    if ((rc = axq_dev_gemv(ctx, w, (const float *)dx.p, batch, (const float *)db.p, (float *)dy.p))) return rc;
    AXQ_HIP(ctx, hipMemcpyAsync(y, dy.p, yb, hipMemcpyDeviceToHost, ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_gemm_bf16(axq_ctx *ctx, const axq_weight *w, const uint16_t *x, int m, float *y, int mem) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_gemm_bf16: NULL context");
    if (!w || !x || !y) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_gemm_bf16: NULL pointer");
    int rc;
    if ((rc = check_mem(ctx, mem))) return rc;
    if (m <= 0) return axq_fail(ctx, AXQ_ERR_SHAPE_MISMATCH, "Shape mismatch: m must be positive, got %d", m);
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    if (mem == AXQ_MEM_DEVICE) return axq_dev_gemm_bf16(ctx, w, x, m, y);
    size_t xb = (size_t)m * (size_t)w->k * 2, yb = (size_t)m * (size_t)w->n_rows * 4;
    DevTemp dx(ctx), dy(ctx);
    AXQ_HIP(ctx, dx.alloc(xb), AXQ_ERR_ALLOCATION_FAILED);
    AXQ_HIP(ctx, dy.alloc(yb), AXQ_ERR_ALLOCATION_FAILED);
    AXQ_HIP(ctx, hipMemcpyAsync(dx.p, x, xb, hipMemcpyHostToDevice, ctx->stream), AXQ_ERR_COPY_FAILED);
    if ((rc = axq_dev_gemm_bf16(ctx, w, (const uint16_t *)dx.p, m, (float *)dy.p))) return rc;
    AXQ_HIP(ctx, hipMemcpyAsync(y, dy.p, yb, hipMemcpyDeviceToHost, ctx->stream), AXQ_ERR_COPY_FAILED);
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_bench_gemv_ring(axq_ctx *ctx, const axq_weight *const *weights, int n_weights, int first, const float *x_dev,
                        int batch, float *y_dev, int iters) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_gemv_ring: NULL context");
    if (!weights || n_weights <= 0 || first < 0 || !x_dev || !y_dev || batch <= 0)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_gemv_ring: bad argument");
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    for (int i = 0; i < iters; i++) {
        const axq_weight *w = weights[(first + i) % n_weights];
        if (!w) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_gemv_ring: NULL weight");
        int rc = axq_dev_gemv(ctx, w, x_dev, batch, NULL, y_dev);
        if (rc) return rc;
    }
    return AXQ_OK;
}

// A recorded ring: `iters` GEMV launches captured once into a graph and replayed as one submission (what a decode loop
// does with its step).  The capture runs on the context's stream; nothing executes until the replay.
struct axq_bench_graph {
    hipGraph_t graph;
    hipGraphExec_t exec;
    int launches;
};

int axq_bench_graph_create(axq_ctx *ctx, const axq_weight *const *weights, int n_weights, int first, const float *x_dev, int batch,
                           float *y_dev, int iters, axq_bench_graph **out) {
    if (!ctx || !out) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_graph_create: NULL argument");
    *out = nullptr;
    if (!weights || n_weights <= 0 || first < 0 || !x_dev || !y_dev || batch <= 0 || iters <= 0)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_graph_create: bad argument");
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    // every kernel the ring uses has run once before the capture (attributes are set on first use, outside any capture)
    int rc = axq_dev_gemv(ctx, weights[first % n_weights], x_dev, batch, NULL, y_dev);
    if (rc) return rc;
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    axq_bench_graph *g = new (std::nothrow) axq_bench_graph{nullptr, nullptr, iters};
    if (!g) return axq_fail(ctx, AXQ_ERR_ALLOCATION_FAILED, "out of host memory");
    hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) {
        delete g;
        return axq_fail(ctx, AXQ_ERR_DRIVER, "hipStreamBeginCapture: %s", hipGetErrorString(e));
    }
    for (int i = 0; i < iters && rc == AXQ_OK; i++) {
        const axq_weight *w = weights[(first + i) % n_weights];
        rc = w ? axq_dev_gemv(ctx, w, x_dev, batch, NULL, y_dev) : axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_graph_create: NULL weight");
    }
    e = hipStreamEndCapture(ctx->stream, &g->graph);
    if (rc == AXQ_OK && e != hipSuccess) rc = axq_fail(ctx, AXQ_ERR_DRIVER, "hipStreamEndCapture: %s", hipGetErrorString(e));
    if (rc == AXQ_OK) {
        e = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
        if (e != hipSuccess) rc = axq_fail(ctx, AXQ_ERR_DRIVER, "hipGraphInstantiate: %s", hipGetErrorString(e));
    }
    if (rc != AXQ_OK) {
        if (g->graph) (void)hipGraphDestroy(g->graph);
        delete g;
        return rc;
    }
    *out = g;
    return AXQ_OK;
}

// The read-only kernel's ring (axq_bench_read_ring) recorded the same way.
int axq_bench_graph_create_read(axq_ctx *ctx, const axq_weight *const *weights, int n_weights, int first, uint32_t *sink_dev, int iters,
                                axq_bench_graph **out) {
    if (!ctx || !out) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_graph_create_read: NULL argument");
    *out = nullptr;
    if (!weights || n_weights <= 0 || first < 0 || !sink_dev || iters <= 0)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_graph_create_read: bad argument");
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    int rc = axq_bench_read_ring(ctx, weights, n_weights, first, sink_dev, 1);
    if (rc) return rc;
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    axq_bench_graph *g = new (std::nothrow) axq_bench_graph{nullptr, nullptr, iters};
    if (!g) return axq_fail(ctx, AXQ_ERR_ALLOCATION_FAILED, "out of host memory");
    hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) {
        delete g;
        return axq_fail(ctx, AXQ_ERR_DRIVER, "hipStreamBeginCapture: %s", hipGetErrorString(e));
    }
    rc = axq_bench_read_ring(ctx, weights, n_weights, first, sink_dev, iters);
    e = hipStreamEndCapture(ctx->stream, &g->graph);
    if (rc == AXQ_OK && e != hipSuccess) rc = axq_fail(ctx, AXQ_ERR_DRIVER, "hipStreamEndCapture: %s", hipGetErrorString(e));
    if (rc == AXQ_OK) {
        e = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
        if (e != hipSuccess) rc = axq_fail(ctx, AXQ_ERR_DRIVER, "hipGraphInstantiate: %s", hipGetErrorString(e));
    }
    if (rc != AXQ_OK) {
        if (g->graph) (void)hipGraphDestroy(g->graph);
        delete g;
        return rc;
    }
    *out = g;
    return AXQ_OK;
}

int axq_bench_graph_launch(axq_ctx *ctx, axq_bench_graph *g, int times) {
    if (!ctx || !g) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_graph_launch: NULL argument");
    for (int i = 0; i < times; i++) AXQ_HIP(ctx, hipGraphLaunch(g->exec, ctx->stream), AXQ_ERR_KERNEL_LAUNCH_FAILED);
    return AXQ_OK;
}

void axq_bench_graph_destroy(axq_ctx *ctx, axq_bench_graph *g) {
    if (!g) return;
    if (ctx) (void)hipStreamSynchronize(ctx->stream);
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    delete g;
}

int axq_bench_gemv_ring_streams(axq_ctx *ctx, const axq_weight *const *weights, int n_weights, int first, const float *x_dev,
                                int batch, float *y_dev, int iters, int streams) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_gemv_ring_streams: NULL context");
    if (!weights || n_weights <= 0 || first < 0 || !x_dev || !y_dev || batch != 1 || streams < 1 || streams > AXQ_AUX_STREAMS)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_gemv_ring_streams: bad argument (one vector per launch, 1..%d streams)", AXQ_AUX_STREAMS);
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    int rc;
    if ((rc = axq_aux_streams(ctx, streams)) || (rc = axq_aux_fork(ctx, streams))) return rc;
    hipStream_t own = ctx->stream;
    for (int i = 0; i < iters && rc == AXQ_OK; i++) {
        const axq_weight *w = weights[(first + i) % n_weights];
        if (!w) { rc = axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_gemv_ring_streams: NULL weight"); break; }
        ctx->stream = ctx->aux_stream[i % streams]; // the one-vector GEMV keeps no scratch outside its own launch
        rc = axq_dev_gemv(ctx, w, x_dev, 1, NULL, y_dev);
    }
    ctx->stream = own;
    if (rc) return rc;
    return axq_aux_join(ctx, streams);
}

int axq_bench_read_ring(axq_ctx *ctx, const axq_weight *const *weights, int n_weights, int first, uint32_t *sink_dev,
                        int iters) {
    return axq_bench_read_ring_ex(ctx, weights, n_weights, first, sink_dev, iters, 1, 512, 16, 1, 0, 1);
}

int axq_bench_read_ring_ex(axq_ctx *ctx, const axq_weight *const *weights, int n_weights, int first, uint32_t *sink_dev,
                           int iters, int wgs_per_cu, int threads, int in_flight, int nontemporal, int pattern, int streams) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_read_ring: NULL context");
    if (!weights || n_weights <= 0 || first < 0 || !sink_dev)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_read_ring: bad argument");
    if (wgs_per_cu < 1 || wgs_per_cu > 8 || (threads != 256 && threads != 512 && threads != 1024) || in_flight < 1 || in_flight > 32 ||
        streams < 1 || streams > AXQ_AUX_STREAMS || pattern < 0 || pattern > 3)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_read_ring_ex: 1..8 workgroups per compute unit, 256/512/1024 threads, 1..32 "
                                                       "loads in flight, 1..%d streams, pattern 0 or 1", AXQ_AUX_STREAMS);
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    int rc;
    if (streams > 1) {
        if ((rc = axq_aux_streams(ctx, streams))) return rc;
        if ((rc = axq_aux_fork(ctx, streams))) return rc;
    }
    const unsigned grid = (unsigned)(ctx->prop.multiProcessorCount * wgs_per_cu);
    for (int i = 0; i < iters; i++) {
        const axq_weight *w = weights[(first + i) % n_weights];
        if (!w) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_read_ring: NULL weight");
        hipStream_t st = streams > 1 ? ctx->aux_stream[i % streams] : ctx->stream;
        if (pattern >= 1) {
            // the code plane of a Q4_K weight with k = 4096, rows in the one-vector GEMV's order
            if (w->type != AXQ_Q4_K || w->k != 4096)
                return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_read_ring_ex: the row pattern reads Q4_K weights with k = 4096");
            int rows_per_wg = (int)((w->n_rows + grid - 1) / grid);
            rows_per_wg = (rows_per_wg + 7) / 8 * 8;
            const unsigned g2 = (unsigned)((w->n_rows + rows_per_wg - 1) / rows_per_wg);
#define AXQ_ROWS(L) \
            if (in_flight <= 4) axq_read_rows_kernel<2, L><<<g2, 512, 0, st>>>(w->codes, w->codes_pitch, (int)w->n_rows, rows_per_wg, sink_dev); \
            else if (in_flight <= 8) axq_read_rows_kernel<4, L><<<g2, 512, 0, st>>>(w->codes, w->codes_pitch, (int)w->n_rows, rows_per_wg, sink_dev); \
            else axq_read_rows_kernel<7, L><<<g2, 512, 0, st>>>(w->codes, w->codes_pitch, (int)w->n_rows, rows_per_wg, sink_dev);
            if (pattern == 1) { AXQ_ROWS(0) } else if (pattern == 2) { AXQ_ROWS(1) } else { AXQ_ROWS(2) }
#undef AXQ_ROWS
        } else {
            const size_t n16 = w->alloc_bytes / 16;
            if (n16 == 0) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_read_ring: empty weight");
            if (nontemporal) launch_read_u<true>(in_flight, threads, grid, st, (const axq_u32x4 *)w->base, n16, sink_dev);
            else launch_read_u<false>(in_flight, threads, grid, st, (const axq_u32x4 *)w->base, n16, sink_dev);
        }
        AXQ_LAUNCH_CHECK(ctx, "axq_bench_read_ring");
    }
    if (streams > 1 && (rc = axq_aux_join(ctx, streams))) return rc;
    return AXQ_OK;
}

int axq_bench_grid_barrier(axq_ctx *ctx, int levels, int publish_bytes, int rounds, float *out_us) {
    if (!ctx || !out_us) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_grid_barrier: NULL argument");
    if (levels < 1 || levels > 2 || rounds < 2 || rounds > 4096 || publish_bytes < 0 || publish_bytes % 1024 || publish_bytes > (1 << 20))
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_grid_barrier: levels 1 or 2, 2..4096 rounds, publish_bytes a multiple of 1024 up to 1 MiB");
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    const int nwg = ctx->prop.multiProcessorCount; // one workgroup per compute unit: all of them resident together
    const int fpt = publish_bytes / 1024;
    int *words = nullptr, *fail = nullptr;
    float *data = nullptr;
    long long *stamps = nullptr;
    const size_t wbytes = (size_t)rounds * BARRIER_WORDS * sizeof(int), sbytes = (size_t)rounds * nwg * 3 * sizeof(long long);
    int rc = AXQ_OK, failed = 0;
    std::vector<long long> h((size_t)rounds * nwg * 3);
    if (hipMalloc(&words, wbytes) != hipSuccess || hipMalloc(&fail, sizeof(int)) != hipSuccess ||
        hipMalloc(&data, (size_t)nwg * (fpt ? fpt : 1) * 1024) != hipSuccess || hipMalloc(&stamps, sbytes) != hipSuccess) {
        rc = axq_fail(ctx, AXQ_ERR_ALLOCATION_FAILED, "axq_bench_grid_barrier: device allocation failed");
    } else {
        for (int rep = 0; rep < 2 && rc == AXQ_OK; rep++) { // the second run is the one read
            if (hipMemsetAsync(words, 0, wbytes, ctx->stream) != hipSuccess || hipMemsetAsync(fail, 0, sizeof(int), ctx->stream) != hipSuccess) {
                rc = axq_fail(ctx, AXQ_ERR_DRIVER, "axq_bench_grid_barrier: memset failed");
                break;
            }
            grid_barrier_kernel<<<nwg, 256, 0, ctx->stream>>>(words, fail, data, stamps, rounds, levels, fpt);
            if (hipGetLastError() != hipSuccess || hipStreamSynchronize(ctx->stream) != hipSuccess)
                rc = axq_fail(ctx, AXQ_ERR_DRIVER, "axq_bench_grid_barrier: launch failed");
        }
        if (rc == AXQ_OK && (hipMemcpy(&failed, fail, sizeof(int), hipMemcpyDeviceToHost) != hipSuccess ||
                             hipMemcpy(h.data(), stamps, sbytes, hipMemcpyDeviceToHost) != hipSuccess))
            rc = axq_fail(ctx, AXQ_ERR_DRIVER, "axq_bench_grid_barrier: copy failed");
        if (rc == AXQ_OK && failed) rc = axq_fail(ctx, AXQ_ERR_DRIVER, "axq_bench_grid_barrier: a round was not completed within its bounded wait");
    }
    (void)hipFree(words); (void)hipFree(fail); (void)hipFree(data); (void)hipFree(stamps);
    if (rc != AXQ_OK) return rc;
    // per round (the first quarter left out): from the last workgroup's arrival to the release as each workgroup sees it;
    // wall_clock64 counts 100 MHz
    std::vector<double> med, worst, pub;
    for (int r = rounds / 4; r < rounds; r++) {
        long long last = 0;
        double p = 0;
        for (int w = 0; w < nwg; w++) {
            const long long *st = &h[((size_t)r * nwg + w) * 3];
            last = st[1] > last ? st[1] : last;
            p += (double)(st[1] - st[0]) * 0.01 / nwg;
        }
        std::vector<double> d(nwg);
        for (int w = 0; w < nwg; w++) d[w] = (double)(h[((size_t)r * nwg + w) * 3 + 2] - last) * 0.01;
        std::sort(d.begin(), d.end());
        med.push_back(d[nwg / 2]); worst.push_back(d[nwg - 1]); pub.push_back(p);
    }
    auto median = [](std::vector<double> &v) { std::sort(v.begin(), v.end()); return (float)v[v.size() / 2]; };
    out_us[0] = median(med); out_us[1] = median(worst); out_us[2] = median(pub);
    return AXQ_OK;
}

int axq_bench_copy(axq_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes, int iters) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_copy: NULL context");
    if (!dst_dev || !src_dev || bytes == 0 || bytes % 16 || ((uintptr_t)dst_dev | (uintptr_t)src_dev) % 16)
        return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_bench_copy: pointers and size must be multiples of 16");
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    size_t n16 = bytes / 16;
    int grid = (int)((n16 + 255) / 256 < 16384 ? (n16 + 255) / 256 : 16384);
    for (int i = 0; i < iters; i++) {
        axq_copy16_kernel<<<grid, 256, 0, ctx->stream>>>((uint4 *)dst_dev, (const uint4 *)src_dev, n16);
        AXQ_LAUNCH_CHECK(ctx, "axq_bench_copy");
    }
    return AXQ_OK;
}

} // extern "C"
