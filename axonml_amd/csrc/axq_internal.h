// Internal declarations shared by the axq translation units (not installed).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <atomic>

#include "../../include/axq.h"

// ---------------------------------------------------------------------------
// Context: one device, one stream, an error string, a timer pair.
// ---------------------------------------------------------------------------
struct axq_ctx {
    int device;
    hipStream_t own_stream;
    hipStream_t stream; // own_stream or an adopted one
    hipEvent_t ev_start, ev_stop;
    hipDeviceProp_t prop;
    float fp8_unit_inv; // 1 / value(fp8 byte 0x01) as converted by v_cvt_pk_f32_fp8
    uint8_t *xq;        // device scratch: the split form of one activation vector (AXQ_XQ_MAX_K elements)
    int gemv_prep;      // 0: split x inside the GEMV kernel, 1: in a kernel of its own
    int gemv_max_nb;    // most 4-row steps a GEMV lane holds in flight (1..8)
    int gemv_wgs_per_cu; // GEMV workgroups per compute unit that the rows are spread over
    void *gemm_scratch; // device scratch of the prefill GEMM (scaled f16 activations + row scales), grown on demand
    size_t gemm_scratch_bytes;
    hipStream_t aux_stream[4]; // benchmarks only: launches that may overlap (created on first use, default priority)
    hipEvent_t aux_event[4], aux_fork;
    char err[512];
};
#define AXQ_AUX_STREAMS 4
int axq_aux_streams(axq_ctx *ctx, int n);
int axq_aux_fork(axq_ctx *ctx, int n);
int axq_aux_join(axq_ctx *ctx, int n);

// ---------------------------------------------------------------------------
// Device-resident weight: "planar" layout, one allocation.
//
//   plane 0 (codes)   : the 4/5/8-bit code bytes of every block, row-major,
//                       row pitch = codes_pitch bytes (16-byte aligned rows)
//   plane 1 (meta)    : per-block scale data, row-major, meta_pitch bytes/row
//                         Q8_0, Q4_0, Q5_0 : f16 scale             (2 B/block)
//                         Q4_1, Q5_1       : f16 scale | f16 min   (4 B/block)
//                         Q4_K             : d, dmin, scales[12]   (16 B/superblock)
//   plane 2 (qh)      : Q5_0/Q5_1 only, the 32 high bits of each block (4 B/block)
//
// The bytes are exactly those of the packed (`to_bytes`) image, permuted, so
// upload -> download is the identity and HBM traffic per matmul equals the
// packed size.  For Q4_K the 128 code bytes of a superblock are further
// interleaved inside 16-superblock "slices" so that one wavefront reads two
// fully contiguous 1 KiB runs per row (see q4k_code_offset).
// ---------------------------------------------------------------------------
struct axq_weight {
    int type;
    int64_t n_rows, k;
    size_t packed_bytes; // size of the to_bytes image
    uint8_t *base;       // device allocation
    size_t alloc_bytes;
    uint8_t *codes, *meta, *qh;
    size_t codes_pitch, meta_pitch, qh_pitch;
    bool owns;
};

#define AXQ_XQ_MAX_K 65536
#define AXQ_BATCH_MAX_K 16384 // widest weight of the small-batch GEMV: its x operands take 34 bytes per element of K
#define AXQ_BATCH_SPLIT_ROWS 8192 // it splits K only for weights of at most this many rows: 4 splits x 8 vectors of partial sums
// its scratch: the batch's operands (34 bytes per element of K), then the partial sums of a split K
#define AXQ_BATCH_SCRATCH_BYTES ((size_t)34 * AXQ_BATCH_MAX_K + (size_t)4 * 8 * AXQ_BATCH_SPLIT_ROWS * 4)

static inline size_t axq_align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Byte offset, inside one row of the Q4_K code plane, of byte `b` (0..127) of
// superblock `sb`.  A slice is 16 superblocks = 64 "pairs" of 32 bytes (pair p
// of a superblock = bytes 32p..32p+31 = sub-blocks 2p (low nibbles) and 2p+1
// (high nibbles)).  Inside a slice holding P pairs, the first 16 bytes of every
// pair come first (16 B x P, pair-major), then the second 16 bytes of every pair.
__host__ __device__ static inline size_t q4k_code_offset(int64_t nsb_row, int64_t sb, int b) {
    int64_t slice = sb >> 4;
    int64_t sb_in = sb & 15;
    int64_t nsb_slice = (nsb_row - (slice << 4)) < 16 ? (nsb_row - (slice << 4)) : 16;
    int64_t P = nsb_slice * 4;
    int64_t pair = sb_in * 4 + (b >> 5);
    int half = (b >> 4) & 1;
    return (size_t)(slice * 2048 + (int64_t)half * 16 * P + pair * 16 + (b & 15));
}

// Error helpers -------------------------------------------------------------
int axq_fail(axq_ctx *ctx, int code, const char *fmt, ...);
#define AXQ_HIP(ctx, call, code)                                                              \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess) return axq_fail((ctx), (code), "%s: %s", #call, hipGetErrorString(e_)); \
    } while (0)
#define AXQ_LAUNCH_CHECK(ctx, what)                                                           \
    do {                                                                                      \
        hipError_t e_ = hipGetLastError();                                                    \
        if (e_ != hipSuccess)                                                                 \
            return axq_fail((ctx), AXQ_ERR_KERNEL_LAUNCH_FAILED, "%s: %s", (what), hipGetErrorString(e_)); \
    } while (0)

// Dynamic LDS beyond the default limit has to be asked for once per kernel AND device.  `done` holds a bit per device (a
// static of the call site, so one per kernel instantiation); asking twice is harmless, hence so is the race of two first
// callers.  A refusal is recorded as the context's error and returned; the launch that follows would fail too.
static inline int axq_allow_lds(axq_ctx *ctx, const void *kernel, std::atomic<uint64_t> &done, size_t bytes) {
    const uint64_t bit = 1ull << (ctx->device & 63);
    if (done.load(std::memory_order_acquire) & bit) return AXQ_OK;
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return axq_fail(ctx, AXQ_ERR_DRIVER, "hipFuncSetAttribute(max dynamic LDS %zu): %s", bytes, hipGetErrorString(e));
    done.fetch_or(bit, std::memory_order_release);
    return AXQ_OK;
}

// Cross-TU entry points -----------------------------------------------------
// codec.hip
int axq_dev_quantize(axq_ctx *ctx, int type, const float *src_dev, size_t numel, uint8_t *packed_dev);
int axq_dev_dequantize(axq_ctx *ctx, int type, const uint8_t *packed_dev, size_t numel, float *dst_dev);
int axq_dev_repack(axq_ctx *ctx, const axq_weight *w, uint8_t *packed_dev, bool to_planar);
// weight.hip
int axq_weight_alloc(axq_ctx *ctx, int type, int64_t n_rows, int64_t k, axq_weight **out);
// gemv.hip
int axq_dev_gemv(axq_ctx *ctx, const axq_weight *w, const float *x_dev, int batch, const float *bias_dev, float *y_dev);
// gemv_mfma.hip: 1 = launched, 0 = shape not covered, <0 = error
int axq_dev_gemv_dp(axq_ctx *ctx, const axq_weight *w, const float *x, const uint8_t *xq, const float *bias, float *y);
// What the GEMV does to x before it uses it (xq must be NULL for the fused forms):
enum { AXQ_X_PLAIN = 0,    // nothing
       AXQ_X_RMSNORM = 1,  // x <- x / sqrt(mean(x^2) + eps) * aux   (aux = norm weights, K floats)
       AXQ_X_SWIGLU = 2,   // small-batch GEMV only: x holds 2K gate/up values (groups of four and four), x <- silu(gate) * up
       AXQ_X_PACKED = 3 }; // small-batch GEMV only: the previous call of a chain has prepared this call's operands
// ... and to its result before it writes it:
enum { AXQ_Y_PLAIN = 0,    // y[row] = dot (+ bias[row])
       AXQ_Y_SWIGLU = 1 }; // rows come in groups of four "gate" rows followed by their four "up" rows:
                           // y[i] = silu(gate_i) * up_i, half as many outputs as rows (no bias)
int axq_dev_gemv_dp_ex(axq_ctx *ctx, const axq_weight *w, const float *x, const uint8_t *xq, int mode, const float *aux,
                       float eps, int ymode, const float *bias, float *y);
bool axq_dev_gemv_dp_covers(const axq_weight *w);
size_t axq_xq_bytes(int64_t k);
int axq_dev_prep_x(axq_ctx *ctx, const float *x, int64_t k, uint8_t *xq);
// gemv_batch.hip: batches of 2..8 vectors against one pass over the weights
bool axq_dev_gemv_batch_covers(const axq_weight *w, int batch);
int axq_dev_gemv_batch(axq_ctx *ctx, const axq_weight *w, const float *x, int batch, const float *bias, const float *resid, float *y);
int axq_dev_gemv_batch_ex(axq_ctx *ctx, const axq_weight *w, const float *x, int xmode, const float *aux, float eps, int batch,
                          const float *bias, const float *resid, float *y);
int axq_dev_gemv_batch_chain(axq_ctx *ctx, const axq_weight *w, const float *x, int xmode, const float *aux, float eps, int batch,
                             const float *bias, const float *resid, float *y, const axq_weight *next, const float *next_aux);
bool axq_dev_gemv_batch_operands(axq_ctx *ctx, const axq_weight *w, uint8_t **xa, float **xsg);
// looks up, once per device, where this device's copy of the static scratch of axq_gemv_f32_static lies (axq_init calls it)
int axq_gemv_static_setup(axq_ctx *ctx);
// sample.hip: every pointer a device pointer; scratch = axq_sample_scratch_bytes(vocab)
size_t axq_sample_scratch_bytes(int vocab);
int axq_check_sampling_config(axq_ctx *ctx, const axq_sampling_config *cfg);
int axq_dev_sample(axq_ctx *ctx, const float *logits, int vocab, const int32_t *hist, const int32_t *hist_len_dev, int hist_len,
                   const axq_sampling_config *cfg, float u, const int32_t *counter_dev, uint64_t seed, void *scratch,
                   int32_t *out, float *filtered_out);
int axq_dev_sample_rows(axq_ctx *ctx, int rows, const float *logits, size_t logits_stride, int vocab, const int32_t *hist,
                        size_t hist_stride, const int32_t *hist_len_dev, int hist_len, const axq_sampling_config *cfg, float u,
                        const int32_t *counter_dev, uint64_t seed, uint64_t seed_stride, void *scratch, int32_t *out,
                        float *filtered_out);
// attn.hip: causal attention of T prompt rows of one sequence on the matrix pipe; 1 = launched, 0 = shape not covered
int axq_dev_attn_rows_mfma(axq_ctx *ctx, const float *qkv, int qkv_rows, const float *rope_cos, const float *rope_sin,
                           const uint16_t *kcache, const uint16_t *vcache, int pos0, int T, int n_heads, int n_kv, int head_dim,
                           int max_pos, int window, float *att);
// gemm.hip
int axq_dev_gemm_bf16(axq_ctx *ctx, const axq_weight *w, const uint16_t *x_dev, int m, float *y_dev);
#define AXQ_GEMM_F32_MAX_ROWS 2048 // rows per call of the f32-activation GEMM (its scratch grows with them)
bool axq_dev_gemm_f32_covers(const axq_weight *w, int m);
bool axq_dev_gemm_f32_takes_swiglu(const axq_weight *w);
int axq_dev_gemm_f32_ex(axq_ctx *ctx, const axq_weight *w, const float *x_dev, bool swiglu, int m, const float *norm_w, float eps,
                        const float *bias, const float *resid, float *y_dev);
int axq_dev_gemm_f32(axq_ctx *ctx, const axq_weight *w, const float *x_dev, int m, const float *norm_w, float eps,
                     const float *bias, const float *resid, float *y_dev);
