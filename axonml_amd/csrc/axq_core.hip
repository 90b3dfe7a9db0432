// Context, memory, type registry and error plumbing of the axq C ABI.
#include <stdarg.h>
#include <stdlib.h>
#include <strings.h>

#include "axq_internal.h"

static thread_local char g_init_err[512] = "";

int axq_fail(axq_ctx *ctx, int code, const char *fmt, ...) {
    char *dst = ctx ? ctx->err : g_init_err;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(dst, 512, fmt, ap);
    va_end(ap);
    return code;
}

// ---------------------------------------------------------------------------
// Type registry (QuantType, crates/axonml-quant/src/types.rs:45-120)
// ---------------------------------------------------------------------------
extern "C" {

size_t axq_type_block_size(int type) {
    switch (type) {
    case AXQ_Q8_0: case AXQ_Q4_0: case AXQ_Q4_1: case AXQ_Q5_0: case AXQ_Q5_1: return 32;
    case AXQ_Q4_K: case AXQ_Q6_K: case AXQ_Q5_K: return 256;
    case AXQ_F16: case AXQ_F32: return 1;
    default: return 0;
    }
}

size_t axq_type_bytes_per_block(int type) {
    switch (type) {
    case AXQ_Q8_0: return 2 + 32;
    case AXQ_Q4_0: return 2 + 16;
    case AXQ_Q4_1: return 4 + 16;
    case AXQ_Q5_0: return 2 + 20;
    case AXQ_Q5_1: return 4 + 20;
    case AXQ_Q4_K: return 4 + 12 + 128;
    case AXQ_Q6_K: return 128 + 64 + 16 + 2;
    case AXQ_Q5_K: return 4 + 12 + 32 + 128;
    case AXQ_F16: return 2;
    case AXQ_F32: return 4;
    default: return 0;
    }
}

size_t axq_type_bits_per_value(int type) {
    switch (type) {
    case AXQ_Q8_0: return 8;
    case AXQ_Q4_0: case AXQ_Q4_1: case AXQ_Q4_K: return 4;
    case AXQ_Q5_0: case AXQ_Q5_1: case AXQ_Q5_K: return 5;
    case AXQ_Q6_K: return 6;
    case AXQ_F16: return 16;
    case AXQ_F32: return 32;
    default: return 0;
    }
}

int axq_type_is_block_quantized(int type) {
    switch (type) {
    case AXQ_Q8_0: case AXQ_Q4_0: case AXQ_Q4_1: case AXQ_Q5_0: case AXQ_Q5_1: case AXQ_Q4_K: case AXQ_Q6_K: case AXQ_Q5_K: return 1;
    default: return 0;
    }
}

const char *axq_type_name(int type) {
    switch (type) {
    case AXQ_Q8_0: return "Q8_0";
    case AXQ_Q4_0: return "Q4_0";
    case AXQ_Q4_1: return "Q4_1";
    case AXQ_Q5_0: return "Q5_0";
    case AXQ_Q5_1: return "Q5_1";
    case AXQ_F16: return "F16";
    case AXQ_F32: return "F32";
    case AXQ_Q4_K: return "Q4_K";
    case AXQ_Q6_K: return "Q6_K";
    case AXQ_Q5_K: return "Q5_K";
    default: return NULL;
    }
}

// from_str upper-cases its argument and accepts the aliases of types.rs:94-105.
int axq_type_from_str(const char *s) {
    if (!s) return -1;
    static const struct { const char *name; int type; } table[] = {
        {"Q8_0", AXQ_Q8_0}, {"Q8", AXQ_Q8_0}, {"INT8", AXQ_Q8_0},
        {"Q4_0", AXQ_Q4_0}, {"Q4", AXQ_Q4_0}, {"INT4", AXQ_Q4_0},
        {"Q4_1", AXQ_Q4_1},
        {"Q5_0", AXQ_Q5_0}, {"Q5", AXQ_Q5_0},
        {"Q5_1", AXQ_Q5_1},
        {"F16", AXQ_F16}, {"FLOAT16", AXQ_F16}, {"HALF", AXQ_F16},
        {"F32", AXQ_F32}, {"FLOAT32", AXQ_F32}, {"FLOAT", AXQ_F32},
        {"Q4_K", AXQ_Q4_K}, {"Q4K", AXQ_Q4_K},
        {"Q6_K", AXQ_Q6_K}, {"Q6K", AXQ_Q6_K},
        {"Q5_K", AXQ_Q5_K}, {"Q5K", AXQ_Q5_K},
    };
    for (size_t i = 0; i < sizeof table / sizeof table[0]; i++)
        if (strcasecmp(s, table[i].name) == 0) return table[i].type;
    return -1;
}

size_t axq_num_blocks(int type, size_t numel) {
    size_t bs = axq_type_block_size(type);
    return bs ? (numel + bs - 1) / bs : 0;
}

size_t axq_packed_bytes(int type, size_t numel) { return axq_num_blocks(type, numel) * axq_type_bytes_per_block(type); }

const char *axq_status_str(int status) {
    switch (status) {
    case AXQ_OK: return "ok";
    case AXQ_ERR_INVALID_BLOCK_SIZE: return "Invalid block size";
    case AXQ_ERR_INVALID_QUANT_TYPE: return "Invalid quantization type";
    case AXQ_ERR_SHAPE_MISMATCH: return "Shape mismatch";
    case AXQ_ERR_DATA_LENGTH_MISMATCH: return "Data length mismatch";
    case AXQ_ERR_CALIBRATION: return "Calibration error";
    case AXQ_ERR_OVERFLOW: return "Numerical overflow during quantization";
    case AXQ_ERR_INVALID_DATA: return "Invalid quantized data";
    case AXQ_ERR_TENSOR_CONVERSION: return "Tensor conversion error";
    case AXQ_ERR_DEVICE_NOT_FOUND: return "Device not found";
    case AXQ_ERR_ALLOCATION_FAILED: return "Memory allocation failed";
    case AXQ_ERR_COPY_FAILED: return "Memory copy failed";
    case AXQ_ERR_KERNEL_LAUNCH_FAILED: return "Kernel launch failed";
    case AXQ_ERR_DRIVER: return "Driver error";
    case AXQ_ERR_BLAS: return "BLAS error";
    case AXQ_ERR_INVALID_ARGUMENT: return "Invalid argument";
    default: return "unknown status";
    }
}

} // extern "C"

// ---------------------------------------------------------------------------
// Context
// ---------------------------------------------------------------------------
// Reports what v_cvt_pk_f32_fp8 makes of the byte 0x01, so the nibble->float
// conversion in the GEMV kernels does not depend on which 8-bit float format
// (OCP e4m3, bias 7, or the older bias-8 variant) the device implements.
__global__ void axq_probe_fp8_kernel(float *out) {
    auto f = __builtin_amdgcn_cvt_pk_f32_fp8(0x0F01, false);
    out[0] = f[0];
    out[1] = f[1];
}

extern "C" {

int axq_init(int device, axq_ctx **out) {
    if (!out) return axq_fail(NULL, AXQ_ERR_INVALID_ARGUMENT, "axq_init: out is NULL");
    *out = NULL;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return axq_fail(NULL, AXQ_ERR_DEVICE_NOT_FOUND, "no HIP device (%s)",
                        e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    if (device < 0 || device >= count)
        return axq_fail(NULL, AXQ_ERR_DEVICE_NOT_FOUND, "device %d out of range (have %d)", device, count);
    axq_ctx *ctx = (axq_ctx *)calloc(1, sizeof(axq_ctx));
    if (!ctx) return axq_fail(NULL, AXQ_ERR_ALLOCATION_FAILED, "out of host memory");
    ctx->device = device;
    // one way out of a failed set-up: whatever exists by then is released, with the device still current
    auto undo = [&]() {
        if (ctx->xq) (void)hipFree(ctx->xq);
        if (ctx->ev_start) (void)hipEventDestroy(ctx->ev_start);
        if (ctx->ev_stop) (void)hipEventDestroy(ctx->ev_stop);
        if (ctx->own_stream) (void)hipStreamDestroy(ctx->own_stream);
        free(ctx);
    };
#define INIT_HIP(call)                                                                         \
    do {                                                                                       \
        hipError_t e_ = (call);                                                                \
        if (e_ != hipSuccess) {                                                                \
            axq_fail(NULL, AXQ_ERR_DRIVER, "%s: %s", #call, hipGetErrorString(e_));            \
            undo();                                                                            \
            return AXQ_ERR_DRIVER;                                                             \
        }                                                                                      \
    } while (0)
    INIT_HIP(hipSetDevice(device));
    INIT_HIP(hipGetDeviceProperties(&ctx->prop, device));
    if (strncmp(ctx->prop.gcnArchName, "gfx950", 6) != 0) {
        axq_fail(NULL, AXQ_ERR_DEVICE_NOT_FOUND, "device %d is %s; this library is built for gfx950 only", device,
                 ctx->prop.gcnArchName);
        undo();
        return AXQ_ERR_DEVICE_NOT_FOUND;
    }
    INIT_HIP(hipStreamCreateWithFlags(&ctx->own_stream, hipStreamNonBlocking));
    ctx->stream = ctx->own_stream;
    INIT_HIP(hipEventCreate(&ctx->ev_start));
    INIT_HIP(hipEventCreate(&ctx->ev_stop));
    float *probe = NULL;
    INIT_HIP(hipMalloc((void **)&probe, 2 * sizeof(float)));
    axq_probe_fp8_kernel<<<1, 1, 0, ctx->stream>>>(probe);
    float h[2] = {0, 0};
    hipError_t pe = hipMemcpyAsync(h, probe, sizeof h, hipMemcpyDeviceToHost, ctx->stream);
    if (pe == hipSuccess) pe = hipStreamSynchronize(ctx->stream);
    (void)hipFree(probe);
    INIT_HIP(pe);
    if (!(h[0] > 0.0f) || h[1] != 15.0f * h[0]) {
        axq_fail(NULL, AXQ_ERR_DRIVER, "fp8 probe: byte 0x01 -> %g, 0x0F -> %g (not linear)", h[0], h[1]);
        undo();
        return AXQ_ERR_DRIVER;
    }
    ctx->fp8_unit_inv = 1.0f / h[0];
    {
        // one vector split, or a small batch packed plus the partial sums of its split K
        size_t xq_bytes = axq_xq_bytes(AXQ_XQ_MAX_K), mb_bytes = AXQ_BATCH_SCRATCH_BYTES;
        INIT_HIP(hipMalloc((void **)&ctx->xq, xq_bytes > mb_bytes ? xq_bytes : mb_bytes));
    }
    // this device's copy of the scratch of axq_gemv_f32_static; a device the table has no place for (or a failed
    // look-up) leaves that one entry point refusing its calls, the rest of the library works
    (void)axq_gemv_static_setup(ctx);
    ctx->err[0] = 0;
    // A lone GEMV call splits x inside the kernel (one launch); callers that produce x on the device
    // hand over the split form instead.  AXQ_GEMV_PREP=separate forces the two-kernel form (development).
    const char *prep = getenv("AXQ_GEMV_PREP");
    ctx->gemv_prep = (prep && strcmp(prep, "separate") == 0) ? 1 : 0;
    const char *mnb = getenv("AXQ_GEMV_MAX_NB");
    ctx->gemv_max_nb = mnb ? atoi(mnb) : 4;
    if (ctx->gemv_max_nb < 1 || ctx->gemv_max_nb > 8) ctx->gemv_max_nb = 4;
    const char *wpc = getenv("AXQ_GEMV_WGS_PER_CU");
    ctx->gemv_wgs_per_cu = wpc ? atoi(wpc) : 1;
    if (ctx->gemv_wgs_per_cu < 1 || ctx->gemv_wgs_per_cu > 16) ctx->gemv_wgs_per_cu = 1;
#undef INIT_HIP
    *out = ctx;
    return AXQ_OK;
}

void axq_destroy(axq_ctx *ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipEventDestroy(ctx->ev_start);
    (void)hipEventDestroy(ctx->ev_stop);
    (void)hipStreamDestroy(ctx->own_stream);
    for (int i = 0; i < AXQ_AUX_STREAMS; i++) {
        if (ctx->aux_stream[i]) (void)hipStreamDestroy(ctx->aux_stream[i]);
        if (ctx->aux_event[i]) (void)hipEventDestroy(ctx->aux_event[i]);
    }
    if (ctx->aux_fork) (void)hipEventDestroy(ctx->aux_fork);
    (void)hipFree(ctx->xq);
    if (ctx->gemm_scratch) (void)hipFree(ctx->gemm_scratch);
    free(ctx);
}

const char *axq_last_error(axq_ctx *ctx) { return ctx ? ctx->err : g_init_err; }

int axq_device_info(axq_ctx *ctx, axq_device_info_t *out) {
    if (!ctx || !out) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_device_info: NULL argument");
    memset(out, 0, sizeof *out);
    strncpy(out->name, ctx->prop.name, sizeof out->name - 1);
    strncpy(out->arch, ctx->prop.gcnArchName, sizeof out->arch - 1);
    out->compute_units = ctx->prop.multiProcessorCount;
    out->wavefront_size = ctx->prop.warpSize;
    out->lds_bytes_per_cu = (int32_t)ctx->prop.maxSharedMemoryPerMultiProcessor;
    out->clock_mhz = ctx->prop.clockRate / 1000;
    out->hbm_bytes = ctx->prop.totalGlobalMem;
    return AXQ_OK;
}

int axq_malloc(axq_ctx *ctx, size_t bytes, void **dptr) {
    if (!ctx || !dptr) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_malloc: NULL argument");
    *dptr = NULL;
    AXQ_HIP(ctx, hipSetDevice(ctx->device), AXQ_ERR_DRIVER);
    AXQ_HIP(ctx, hipMalloc(dptr, bytes ? bytes : 1), AXQ_ERR_ALLOCATION_FAILED);
    return AXQ_OK;
}

int axq_free(axq_ctx *ctx, void *dptr) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_free: NULL context");
    if (!dptr) return AXQ_OK;
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    AXQ_HIP(ctx, hipFree(dptr), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

static int copy_sync(axq_ctx *ctx, void *dst, const void *src, size_t bytes, hipMemcpyKind kind, const char *what) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "%s: NULL context", what);
    if (bytes == 0) return AXQ_OK;
    if (!dst || !src) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "%s: NULL pointer", what);
    AXQ_HIP(ctx, hipMemcpyAsync(dst, src, bytes, kind, ctx->stream), AXQ_ERR_COPY_FAILED);
    if (kind != hipMemcpyDeviceToDevice) AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_COPY_FAILED);
    return AXQ_OK;
}

int axq_copy_to_device(axq_ctx *ctx, void *dst, const void *src, size_t bytes) {
    return copy_sync(ctx, dst, src, bytes, hipMemcpyHostToDevice, "axq_copy_to_device");
}
int axq_copy_to_host(axq_ctx *ctx, void *dst, const void *src, size_t bytes) {
    return copy_sync(ctx, dst, src, bytes, hipMemcpyDeviceToHost, "axq_copy_to_host");
}
int axq_copy_device_to_device(axq_ctx *ctx, void *dst, const void *src, size_t bytes) {
    return copy_sync(ctx, dst, src, bytes, hipMemcpyDeviceToDevice, "axq_copy_device_to_device");
}

int axq_synchronize(axq_ctx *ctx) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_synchronize: NULL context");
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_set_stream(axq_ctx *ctx, void *hip_stream) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_set_stream: NULL context");
    AXQ_HIP(ctx, hipStreamSynchronize(ctx->stream), AXQ_ERR_DRIVER);
    ctx->stream = hip_stream ? (hipStream_t)hip_stream : ctx->own_stream;
    return AXQ_OK;
}

int axq_timer_start(axq_ctx *ctx) {
    if (!ctx) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_timer_start: NULL context");
    AXQ_HIP(ctx, hipEventRecord(ctx->ev_start, ctx->stream), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

int axq_timer_stop(axq_ctx *ctx, float *elapsed_ms) {
    if (!ctx || !elapsed_ms) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_timer_stop: NULL argument");
    AXQ_HIP(ctx, hipEventRecord(ctx->ev_stop, ctx->stream), AXQ_ERR_DRIVER);
    AXQ_HIP(ctx, hipEventSynchronize(ctx->ev_stop), AXQ_ERR_DRIVER);
    AXQ_HIP(ctx, hipEventElapsedTime(elapsed_ms, ctx->ev_start, ctx->ev_stop), AXQ_ERR_DRIVER);
    return AXQ_OK;
}

} // extern "C"

// ---------------------------------------------------------------------------
// Seeded normal fill (benchmark inputs generated on the device)
// ---------------------------------------------------------------------------
__device__ static inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__global__ void axq_fill_normal_kernel(float *dst, size_t n, float mean, float std, float outlier_p, float outlier_mag,
                                       uint64_t seed) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        uint64_t r = splitmix64(seed ^ splitmix64(i));
        uint64_t r2 = splitmix64(r);
        float u1 = ((float)(uint32_t)(r >> 40) + 1.0f) * (1.0f / 16777217.0f); // (0,1)
        float u2 = (float)(uint32_t)((r >> 8) & 0xFFFFFF) * (1.0f / 16777216.0f);
        float z = sqrtf(-2.0f * logf(u1)) * cosf(6.28318530718f * u2);
        float v = mean + std * z;
        if (outlier_p > 0.0f) {
            float u3 = (float)(uint32_t)(r2 >> 40) * (1.0f / 16777216.0f);
            if (u3 < outlier_p) v = (r2 & 1) ? outlier_mag : -outlier_mag;
        }
        dst[i] = v;
    }
}

extern "C" int axq_fill_normal_f32(axq_ctx *ctx, float *dst_dev, size_t n, float mean, float std, float outlier_p,
                                   float outlier_mag, uint64_t seed) {
    if (!ctx || (!dst_dev && n)) return axq_fail(ctx, AXQ_ERR_INVALID_ARGUMENT, "axq_fill_normal_f32: NULL argument");
    if (n == 0) return AXQ_OK;
    size_t blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    axq_fill_normal_kernel<<<(unsigned)blocks, 256, 0, ctx->stream>>>(dst_dev, n, mean, std, outlier_p, outlier_mag, seed);
    AXQ_LAUNCH_CHECK(ctx, "axq_fill_normal_kernel");
    return AXQ_OK;
}
