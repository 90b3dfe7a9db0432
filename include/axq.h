/*
 * axq -- MI355X (gfx950) block-quantized matmul path, C ABI.
 *
 * This is the drop-in boundary for the `axonml-quant` crate's path
 * (quantize -> QuantizedTensor -> dequantize / quantized matmul) as an
 * `axonml-llm` decode or prefill loop would use it.  Every entry point is
 * plain C: opaque handles, pointers and sizes.  All compute runs in HIP
 * kernels on the device; there is no CPU fallback -- without a usable GPU
 * axq_init() fails with AXQ_ERR_DEVICE_NOT_FOUND and nothing else can be
 * called.
 *
 * Conventions
 *   - Every function returns AXQ_OK (0) or a negative axq_status; none aborts
 *     and no C++ exception crosses the boundary.  axq_last_error() gives the
 *     text of the last failure on a context (or of the last failed axq_init
 *     when called with NULL).
 *   - "packed" buffers are the concatenation, in block order, of the
 *     reference's per-block byte images (`to_bytes`,
 *     crates/axonml-quant/src/types.rs:142-147, 201-206, 249-255); Q5_0, Q5_1
 *     and Q4_K use the GGUF block layouts.  Blocks run along the flat
 *     row-major buffer (crates/axonml-quant/src/quantize.rs:84-91).
 *   - `mem` says where the caller's data pointers live: AXQ_MEM_HOST (the
 *     library stages them through the device) or AXQ_MEM_DEVICE (used in
 *     place, on the context's stream, no synchronisation).
 *   - A context owns one HIP stream (or adopts the caller's through
 *     axq_set_stream).  Calls on one context must not overlap; distinct
 *     contexts are independent.  This mirrors the reference CUDA backend's
 *     "one device, default stream, Send but not re-entrant" convention
 *     (crates/axonml-core/src/backends/cuda.rs:34-35, 52-55, 224-226).
 */
#ifndef AXQ_H
#define AXQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AXQ_API __attribute__((visibility("default")))

typedef struct axq_ctx axq_ctx;
typedef struct axq_weight axq_weight;
typedef struct axq_model axq_model;

/* QuantType, crates/axonml-quant/src/types.rs:17-41, in the same order, with
 * the 256-element GGUF superblock types appended: Q4_K (144 bytes) and Q6_K (210 bytes: 128 bytes of low nibbles,
 * 64 of high bit pairs, sixteen int8 scales of 16 elements each, f16 d; w = d * scale * (q - 32)), the type llama.cpp
 * keeps output.weight and part of the value and down projections in when it writes "Q4_0" and "Q4_K_M" files; and
 * Q5_K (176 bytes: Q4_K's header, 32 bytes of fifth bits, 128 of low nibbles; w = d * sc * q - dmin * m, q in 0..31). */
typedef enum {
    AXQ_Q8_0 = 0,
    AXQ_Q4_0 = 1,
    AXQ_Q4_1 = 2,
    AXQ_Q5_0 = 3,
    AXQ_Q5_1 = 4,
    AXQ_F16 = 5,
    AXQ_F32 = 6,
    AXQ_Q4_K = 7,
    AXQ_Q6_K = 8,
    AXQ_Q5_K = 9,
    AXQ_TYPE_COUNT = 10
} axq_type;

typedef enum {
    AXQ_OK = 0,
    /* QuantError, crates/axonml-quant/src/error.rs:14-57 */
    AXQ_ERR_INVALID_BLOCK_SIZE = -1,
    AXQ_ERR_INVALID_QUANT_TYPE = -2,
    AXQ_ERR_SHAPE_MISMATCH = -3,
    AXQ_ERR_DATA_LENGTH_MISMATCH = -4,
    AXQ_ERR_CALIBRATION = -5,
    AXQ_ERR_OVERFLOW = -6,
    AXQ_ERR_INVALID_DATA = -7,
    AXQ_ERR_TENSOR_CONVERSION = -8,
    /* CudaError, crates/axonml-core/src/backends/cuda.rs:272-289 */
    AXQ_ERR_DEVICE_NOT_FOUND = -20,
    AXQ_ERR_ALLOCATION_FAILED = -21,
    AXQ_ERR_COPY_FAILED = -22,
    AXQ_ERR_KERNEL_LAUNCH_FAILED = -23,
    AXQ_ERR_DRIVER = -24,
    AXQ_ERR_BLAS = -25, /* BlasError (kept for the mirror; this library calls no BLAS) */
    /* boundary misuse (NULL handle or pointer, bad flag) */
    AXQ_ERR_INVALID_ARGUMENT = -30
} axq_status;

typedef enum { AXQ_MEM_HOST = 0, AXQ_MEM_DEVICE = 1 } axq_mem;

/* ---- type registry: QuantType methods, types.rs:45-120 ------------------- */
AXQ_API size_t axq_type_block_size(int type);      /* block_size(), :45-54; 0 if unknown */
AXQ_API size_t axq_type_bytes_per_block(int type); /* bytes_per_block(), :57-67 */
AXQ_API size_t axq_type_bits_per_value(int type);  /* bits_per_value(), :70-78 */
AXQ_API int axq_type_is_block_quantized(int type); /* is_block_quantized(), :86-91 */
AXQ_API const char *axq_type_name(int type);       /* Display, :108-120; NULL if unknown */
AXQ_API int axq_type_from_str(const char *s);      /* from_str() with its aliases, :94-105; -1 if unknown */
AXQ_API size_t axq_num_blocks(int type, size_t numel);   /* ceil(numel / block), quantize.rs:84 */
AXQ_API size_t axq_packed_bytes(int type, size_t numel); /* QuantizedTensor::size_bytes, types.rs:320-322 */
AXQ_API const char *axq_status_str(int status);

/* ---- device context: Backend trait, backends/mod.rs:73-100, and
 *      CudaBackend::new -> Option, backends/cuda.rs:69-81 ------------------ */
typedef struct {
    char name[128];
    char arch[32];
    int32_t compute_units;
    int32_t wavefront_size;
    int32_t lds_bytes_per_cu;
    int32_t clock_mhz;
    uint64_t hbm_bytes;
} axq_device_info_t;

AXQ_API int axq_init(int device, axq_ctx **out);
AXQ_API void axq_destroy(axq_ctx *ctx);
AXQ_API const char *axq_last_error(axq_ctx *ctx);
AXQ_API int axq_device_info(axq_ctx *ctx, axq_device_info_t *out);   /* capabilities() */
AXQ_API int axq_malloc(axq_ctx *ctx, size_t bytes, void **dptr);     /* allocate() */
AXQ_API int axq_free(axq_ctx *ctx, void *dptr);                      /* deallocate() */
AXQ_API int axq_copy_to_device(axq_ctx *ctx, void *dst, const void *src, size_t bytes);
AXQ_API int axq_copy_to_host(axq_ctx *ctx, void *dst, const void *src, size_t bytes);
AXQ_API int axq_copy_device_to_device(axq_ctx *ctx, void *dst, const void *src, size_t bytes);
AXQ_API int axq_synchronize(axq_ctx *ctx);                           /* synchronize() */
/* Adopt a caller-owned hipStream_t (NULL = back to the context's own). */
AXQ_API int axq_set_stream(axq_ctx *ctx, void *hip_stream);
/* HIP-event stopwatch on the context's stream (for the benchmark). */
AXQ_API int axq_timer_start(axq_ctx *ctx);
AXQ_API int axq_timer_stop(axq_ctx *ctx, float *elapsed_ms); /* synchronises on the stop event */

/* ---- codecs: quantize_tensor (quantize.rs:36-54) and dequantize_tensor
 *      (dequantize.rs:34-54), run on the device ---------------------------- */
/* src: numel f32; packed: axq_packed_bytes(type, numel) bytes. */
AXQ_API int axq_quantize(axq_ctx *ctx, int type, const float *src, size_t numel, void *packed, int mem);
/* dst: numel f32 (the tail block is truncated, dequantize.rs:44-50). */
AXQ_API int axq_dequantize(axq_ctx *ctx, int type, const void *packed, size_t numel, float *dst, int mem);

/* ---- GGUF interop.  The reference names GGUF only as a file extension
 *      (crates/axonml-cli/src/commands/quant.rs:218) and has no reader; the
 *      block layouts are those of the GGUF / ggml specification.  Q8_0, Q5_0,
 *      Q5_1, Q4_K, F16 and F32 images are the same on both sides; Q4_0 and
 *      Q4_1 keep their scales and permute the 32 nibbles of a block (ggml: byte
 *      j = elements j, j+16; reference pack(), types.rs:190-198: byte i =
 *      elements 2i, 2i+1).  Element formulas agree, so a converted tensor
 *      dequantises (dequantize.rs:116-121, 145-151) to ggml's values. ------- */
enum { AXQ_GGUF_TO_NATIVE = 0, AXQ_NATIVE_TO_GGUF = 1 };
/* ggml_type number of a GGUF tensor table entry -> axq_quant_type, -1 if this library has no such type. */
AXQ_API int axq_type_from_ggml(int ggml_type);
AXQ_API int axq_type_to_ggml(int type);
/* Converts nblocks block images between the two orders; src == dst is allowed.
 * Device pointers must be 16-byte aligned. */
AXQ_API int axq_gguf_convert_blocks(axq_ctx *ctx, int type, const void *src, void *dst, size_t nblocks, int direction,
                                    int mem);

/* ---- device-resident weights: QuantizedTensor (types.rs:296-334) of shape
 *      [n_rows, k] as a Linear weight (nn/src/layers/linear.rs:41-42) -------- */
/* Copies `packed` (bytes must equal axq_packed_bytes(type, n_rows*k)); the
 * caller keeps ownership of its buffer.  k must be a multiple of the block. */
AXQ_API int axq_weight_upload(axq_ctx *ctx, int type, int64_t n_rows, int64_t k, const void *packed, size_t bytes,
                              int mem, axq_weight **out);
/* quantize_tensor straight into a device-resident weight. */
AXQ_API int axq_weight_quantize(axq_ctx *ctx, int type, int64_t n_rows, int64_t k, const float *w, int mem,
                                axq_weight **out);
/* Returns the exact bytes that were uploaded / produced by the quantiser. */
AXQ_API int axq_weight_download(axq_ctx *ctx, const axq_weight *w, void *packed, size_t bytes, int mem);
AXQ_API int axq_weight_info(const axq_weight *w, int *type, int64_t *n_rows, int64_t *k, size_t *bytes);
AXQ_API void axq_weight_free(axq_ctx *ctx, axq_weight *w);

/* ---- quantized matmul: the composition dequantize_tensor -> Tensor::matmul
 *      (tensor/src/tensor.rs:1020-1045) behind Linear::forward
 *      (nn/src/layers/linear.rs:104-140), fused ------------------------------ */
/* y[batch, n_rows] = x[batch, k] * W^T (+ bias[n_rows] if non-NULL), f32.
 * Any batch: one vector and 2..8 vectors per pass over the weights (decode), from 40 rows on (k a
 * multiple of 64) the matrix-pipe GEMM with every f32 row carried as two f16 rows, so that the result
 * keeps f32 accuracy.  bias lives where x and y live. */
AXQ_API int axq_gemv_f32(axq_ctx *ctx, const axq_weight *w, const float *x, int batch, const float *bias, float *y,
                         int mem);
/* axq_gemv_f32 for 2..8 vectors on device pointers, for callers that cannot allocate.  No counterpart in the
 * reference: it exists for code under HIP graph capture, tight serving loops and harnesses that forbid
 * hipMalloc.  It allocates nothing: the scratch of its kernels (the batch's matrix-pipe operands and the
 * partial sums of a split K, 1,605,632 bytes) is a device array inside the library, one copy per GPU, held
 * until the process ends.  Limits: weights of a block type (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q4_K, Q5_K, Q6_K), k a multiple of 256 up to 16384, any
 * n_rows, batch 2..8; anything else is refused with AXQ_ERR_SHAPE_MISMATCH / AXQ_ERR_INVALID_QUANT_TYPE.
 * x, bias (may be NULL) and y are device pointers; the launches go to the context's stream and nothing is
 * synchronised.  Every call on a GPU shares that GPU's array (it needs no clearing: each call writes what it
 * reads), so calls that overlap on one GPU -- from two contexts or two streams -- race; serialise them. */
AXQ_API int axq_gemv_f32_static(axq_ctx *ctx, const axq_weight *w, const float *x, int batch, const float *bias, float *y);
/* y[m, n_rows] = x[m, k] * W^T, x in bf16 (raw uint16), y f32.  Prefill path. */
AXQ_API int axq_gemm_bf16(axq_ctx *ctx, const axq_weight *w, const uint16_t *x_bf16, int m, float *y, int mem);

/* ---- decode: LLaMA/Mistral-shape model, llm/src/llama.rs:731-762, 900-977 - */
/* Field names follow LLaMAConfig / MistralConfig (llama.rs:56-121, mistral.rs:56-70). */
typedef struct {
    int32_t vocab_size, hidden_size, intermediate_size, num_hidden_layers;
    int32_t num_attention_heads, num_key_value_heads, head_dim, max_position_embeddings;
    float rms_norm_eps, rope_theta;
    /* MistralConfig::sliding_window (mistral.rs:56-70): a token attends to the last `sliding_window`
     * cache positions only (MistralAttention::forward_with_cache slices the cache, mistral.rs:204-238);
     * 0 = the whole cache (LLaMA). */
    int32_t sliding_window;
} axq_model_config;

typedef enum {
    AXQ_LIN_Q = 0, AXQ_LIN_K, AXQ_LIN_V, AXQ_LIN_O, AXQ_LIN_GATE, AXQ_LIN_UP, AXQ_LIN_DOWN, AXQ_LIN_COUNT
} axq_linear_id;

AXQ_API int axq_model_create(axq_ctx *ctx, const axq_model_config *cfg, axq_model **out);
AXQ_API void axq_model_free(axq_model *m);
/* f16 table [vocab, hidden] (Embedding::lookup, nn/src/layers/embedding.rs:103-146). */
AXQ_API int axq_model_set_embedding_f16(axq_model *m, const uint16_t *table, int mem);
/* The same table in f32, as the reference keeps it (embedding.rs:103-146: lookup copies f32 rows); replaces an f16 table
 * and the other way round. */
AXQ_API int axq_model_set_embedding_f32(axq_model *m, const float *table, int mem);
/* layer -1 = final norm; which 0 = attention norm, 1 = ffn norm.  f32[hidden]. */
AXQ_API int axq_model_set_norm(axq_model *m, int layer, int which, const float *w, int mem);
/* layer -1 = lm_head.  The model copies the weight's blocks; the caller may free `w`.  q, k and v of a layer share one
 * fused weight of the block type of whichever is set first; a q, k or v of another type is kept as a weight of its own
 * (row counts must be multiples of 4 then).  gate and up share one weight and one type (AXQ_ERR_INVALID_QUANT_TYPE).
 * o, down and the lm_head may be set again in another block type. */
AXQ_API int axq_model_set_linear(axq_model *m, int layer, int which, const axq_weight *w);
/* Fill every linear (Q4_K by default), the embedding and unit norms from a
 * seeded device generator: N(0, std) weights.  For benchmarks of random-init
 * models too large to stage through the host. */
AXQ_API int axq_model_random_init(axq_model *m, int type, float std, uint64_t seed);
/* KVCache::clear (attention.rs:80-83). */
AXQ_API int axq_model_reset(axq_model *m);
/* Rewind the cache to its first n_positions (KVCache.seq_len is a public field, attention.rs:18-26: a caller
 * that tries several continuations of one prefix, beam search for one, sets it back); the rows beyond are
 * overwritten by the next tokens.  n_positions <= axq_model_seq_len. */
AXQ_API int axq_model_truncate(axq_model *m, int n_positions);
/* forward_with_cache for one token at the cache's current length; appends to
 * the cache.  logits (f32[vocab], host) may be NULL.  next_token (host) may be NULL. */
AXQ_API int axq_model_forward(axq_model *m, int32_t token, float *logits, int32_t *next_token);
/* forward_with_cache (llama.rs:731-762) for n >= 1 tokens at once (a prompt): appends n positions to the
 * cache; logits / next_token are those of the last position.  Tokens before the last go through the
 * layers together: from 32 on through the GEMM (f32 activations, K a multiple of 64), fewer up to eight
 * per pass over the weights when every linear of the layers is of a block type (Q4_0 ... Q6_K) with K a
 * multiple of 256 up to 16384, else one by one; results agree with n calls of axq_model_forward to
 * rounding (sums are taken in another order). */
AXQ_API int axq_model_forward_tokens(axq_model *m, const int32_t *tokens, int n, float *logits, int32_t *next_token);
/* Several sequences side by side (the batch dimension of forward_with_cache's input ids and of KVCache,
 * llama.rs:731-762, attention.rs:28-35): n_seq = 1..64 caches and position counters; a batched step feeds
 * one token of every sequence and reads the weights once for all of them (up to eight sequences through the
 * small-batch GEMV as a replayed graph, more through the GEMM on f32 rows, which needs K a multiple of 64).  Calling it discards every
 * cache and starts all sequences at position 0.  The one-sequence calls above keep working on sequence 0. */
AXQ_API int axq_model_set_batch(axq_model *m, int n_seq);
AXQ_API int axq_model_batch(const axq_model *m);
AXQ_API int axq_model_seq_len_of(const axq_model *m, int seq);
/* Sequence dst becomes a copy of sequence src (cache rows, token history, position): two continuations of one
 * prefix, as beam search forks them. */
AXQ_API int axq_model_copy_sequence(axq_model *m, int src, int dst);
/* tokens: int32[n_seq]; logits (host, may be NULL): f32[n_seq, vocab]; next_tokens (host, may be NULL): int32[n_seq].
 * Sequences may stand at different positions. */
AXQ_API int axq_model_forward_batch(axq_model *m, const int32_t *tokens, float *logits, int32_t *next_tokens);
/* generate for n_seq prompts of any lengths at once: prompts holds them back to back, prompt s is
 * prompts[offsets[s] .. offsets[s+1]) (offsets: int32[n_seq + 1], offsets[0] = 0).  Starts every sequence
 * afresh.  out_tokens: int32[n_seq, max_new_tokens].  Each sequence gets what axq_model_generate gives for
 * its prompt alone, to rounding (sums are taken in another order). */
AXQ_API int axq_model_generate_batch(axq_model *m, const int32_t *prompts, const int32_t *offsets, int max_new_tokens,
                                     int32_t *out_tokens, float *prefill_ms, float *decode_ms);
/* generate (llama.rs:900-977), greedy: feeds the prompt (as axq_model_forward_tokens does), then max_new_tokens
 * steps, each consuming the previous argmax on the device.  out_tokens gets
 * max_new_tokens ids (host).  Timings (ms, may be NULL) cover prompt and
 * generation separately. */
AXQ_API int axq_model_generate(axq_model *m, const int32_t *prompt, int n_prompt, int max_new_tokens,
                               int32_t *out_tokens, float *prefill_ms, float *decode_ms);
AXQ_API int axq_model_seq_len(const axq_model *m);
/* The residual stream after the last step (f32[hidden], host): for intermediate checks in tests. */
AXQ_API int axq_model_read_hidden(axq_model *m, float *hidden_out);
/* One layer's f16 cache, [kv_heads][max_position_embeddings][head_dim] (host); which 0 = keys, 1 = values. */
AXQ_API int axq_model_read_kv(axq_model *m, int layer, int which, uint16_t *out);

/* ---- next-token selection: TextGenerator::get_next_token (llm/src/generation.rs:258-269) =
 *      apply_repetition_penalty (:145-158, once per occurrence), apply_temperature (:136-142),
 *      apply_top_k (:161-180), apply_top_p (:183-214), then sample (:217-245) or argmax (:248-255),
 *      on the device.  Penalty, temperature and top-k are bit-exact; the softmax sums of top-p
 *      and of the draw are exact where the reference adds f32 sequentially, so a decision may
 *      differ when a cumulative probability comes within ~1e-5 of its threshold. ---------- */
/* The GenerationConfig fields that get_next_token reads (generation.rs:11-35). */
typedef struct {
    float temperature;        /* > 0; 1.0 leaves the logits alone */
    int32_t top_k;            /* 0 = None */
    float top_p;              /* negative = None */
    float repetition_penalty; /* > 0; 1.0 = none */
    int32_t do_sample;        /* 0: argmax of the filtered logits (ties: the last, as Iterator::max_by) */
} axq_sampling_config;
/* logits: f32[vocab]; generated: the ids the penalty looks at (may be NULL when n_generated = 0);
 * u in [0, 1) stands for the reference's rand::thread_rng draw; token: one id; filtered_logits
 * (optional, f32[vocab]): the logits after all filters, dropped entries -inf. */
AXQ_API int axq_sample_token(axq_ctx *ctx, const float *logits, int vocab, const int32_t *generated, int n_generated,
                             const axq_sampling_config *cfg, float u, int32_t *token, float *filtered_logits, int mem);
/* Makes axq_model_forward / axq_model_generate choose the next token this way instead of by the plain
 * argmax; the penalty sees every token fed so far, the draw of a step comes from (seed, position).
 * cfg = NULL: back to greedy.  In batched steps sequence s draws from (seed + s * 0x9E3779B97F4A7C15, position). */
AXQ_API int axq_model_set_sampling(axq_model *m, const axq_sampling_config *cfg, uint64_t seed);

/* ---- benchmark utilities ------------------------------------------------- */
/* dst[i] ~ N(mean, std) from a counter-based generator (seed, i); with
 * outlier_p > 0 each element is instead +/-outlier_mag with that probability. */
AXQ_API int axq_fill_normal_f32(axq_ctx *ctx, float *dst_dev, size_t n, float mean, float std, float outlier_p,
                                float outlier_mag, uint64_t seed);

/* Enqueues `iters` GEMV launches back to back from C, launch i using weights[(first + i) % n_weights] (a ring
 * of copies larger than the last-level cache keeps every launch streaming from HBM).  Device pointers. */
AXQ_API int axq_bench_gemv_ring(axq_ctx *ctx, const axq_weight *const *weights, int n_weights, int first,
                                const float *x_dev, int batch, float *y_dev, int iters);

/* The ring as a recorded graph: `iters` launches, launch i on weights[(first + i) % n_weights], captured once and replayed
 * with one submission per axq_bench_graph_launch (`times` replays back to back).  Device pointers; the graph keeps
 * them, so they must stay valid until axq_bench_graph_destroy. */
typedef struct axq_bench_graph axq_bench_graph;
AXQ_API int axq_bench_graph_create(axq_ctx *ctx, const axq_weight *const *weights, int n_weights, int first,
                                   const float *x_dev, int batch, float *y_dev, int iters, axq_bench_graph **out);
AXQ_API int axq_bench_graph_create_read(axq_ctx *ctx, const axq_weight *const *weights, int n_weights, int first,
                                        uint32_t *sink_dev, int iters, axq_bench_graph **out); /* axq_bench_read_ring's launches */
AXQ_API int axq_bench_graph_launch(axq_ctx *ctx, axq_bench_graph *g, int times);
AXQ_API void axq_bench_graph_destroy(axq_ctx *ctx, axq_bench_graph *g);

/* The same ring walked by a kernel that only reads each weight's device image (one 512-thread workgroup per
 * compute unit, non-temporal 16-byte loads): the rate the memory system gives a launch of that size, to set
 * beside the GEMV's.  sink_dev: four writable device bytes. */
AXQ_API int axq_bench_read_ring(axq_ctx *ctx, const axq_weight *const *weights, int n_weights, int first,
                                uint32_t *sink_dev, int iters);

/* The read-only kernel with its parameters open, for the table of what the memory system gives a launch of this size:
 * wgs_per_cu workgroups per compute unit (1..8) of `threads` (256, 512, 1024), each lane keeping `in_flight` 16-byte loads
 * in flight (4, 8, 16, 32; 16 at most with 1024 threads), non-temporal or plain loads; pattern 0 reads each weight's
 * device image as contiguous shares, pattern 1 reads the code plane of a Q4_K weight with k = 4096 row step by row step,
 * as the one-vector GEMV does (in_flight = 4, 8 or 14: two loads per step), patterns 2 and 3 read as many bytes of that
 * plane per wave and step from one contiguous run per wave / per workgroup; streams > 1 spreads the launches over that
 * many streams so that consecutive launches may overlap (the context's stream waits for all of them at the end).
 * axq_bench_read_ring is (1, 512, 16, 1, 0, 1). */
AXQ_API int axq_bench_read_ring_ex(axq_ctx *ctx, const axq_weight *const *weights, int n_weights, int first,
                                   uint32_t *sink_dev, int iters, int wgs_per_cu, int threads, int in_flight,
                                   int nontemporal, int pattern, int streams);

/* axq_bench_gemv_ring with the launches spread over `streams` streams (1..4): GEMVs that do not depend on each other
 * (every launch of the ring reads the same x and overwrites the same y) may then overlap.  A figure beside the
 * single-stream one, which is the one reported. */
AXQ_API int axq_bench_gemv_ring_streams(axq_ctx *ctx, const axq_weight *const *weights, int n_weights, int first,
                                        const float *x_dev, int batch, float *y_dev, int iters, int streams);

/* Enqueues `iters` launches of a plain copy kernel (reads `bytes`, writes `bytes`; both pointers and the
 * size multiples of 16).  A kernel of known traffic against which profiler memory counters are scaled. */
AXQ_API int axq_bench_copy(axq_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes, int iters);

/* Measures a barrier over all workgroups of one resident launch (one workgroup per compute unit) through device-scope
 * atomics: what a kernel that stays on the chip across dependent steps would pay where separate kernels pay a launch
 * boundary.  levels = 1: one counter; 2: sixteen group counters, then a release word.  Before counting in, every
 * workgroup publishes publish_bytes (a multiple of 1024, may be 0) with device-scope stores.  Waits are bounded: a round
 * that does not complete returns AXQ_ERR_DRIVER.  out_us[0]: from the last workgroup's arrival to the release as the
 * median workgroup sees it, [1]: as the slowest sees it, [2]: the publishing, all medians over the rounds.  Synchronous.
 * No counterpart in the reference. */
AXQ_API int axq_bench_grid_barrier(axq_ctx *ctx, int levels, int publish_bytes, int rounds, float *out_us);

#ifdef __cplusplus
}
#endif
#endif /* AXQ_H */
