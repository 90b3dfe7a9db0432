//! Raw bindings to `libaxq.so` (`include/axq.h`): the block-quantized matmul path on MI355X.
//!
//! NOT COMPILED in this repository's build or tests: the image this library is built in has no Rust toolchain.
//! The declarations restate `include/axq.h` by hand; `tests/test_abi.py` checks that the shared library exports every
//! symbol the header declares.  A safe layer (context, device weight, quantized_matmul) belongs in `axonml-quant` itself.
#![allow(non_camel_case_types)]
use std::os::raw::{c_char, c_int, c_void};

#[repr(C)] pub struct axq_ctx { _p: [u8; 0] }
#[repr(C)] pub struct axq_weight { _p: [u8; 0] }
#[repr(C)] pub struct axq_model { _p: [u8; 0] }

pub const AXQ_MEM_HOST: c_int = 0;
pub const AXQ_MEM_DEVICE: c_int = 1;

#[repr(C)]
pub struct axq_model_config {
    pub vocab_size: i32, pub hidden_size: i32, pub intermediate_size: i32, pub num_hidden_layers: i32,
    pub num_attention_heads: i32, pub num_key_value_heads: i32, pub head_dim: i32,
    pub max_position_embeddings: i32, pub rms_norm_eps: f32, pub rope_theta: f32, pub sliding_window: i32,
}

#[link(name = "axq")]
extern "C" {
    pub fn axq_init(device: c_int, out: *mut *mut axq_ctx) -> c_int;
    pub fn axq_destroy(ctx: *mut axq_ctx);
    pub fn axq_last_error(ctx: *mut axq_ctx) -> *const c_char;
    pub fn axq_synchronize(ctx: *mut axq_ctx) -> c_int;
    pub fn axq_packed_bytes(ty: c_int, numel: usize) -> usize;

    pub fn axq_quantize(ctx: *mut axq_ctx, ty: c_int, src: *const f32, numel: usize,
                        packed: *mut c_void, mem: c_int) -> c_int;
    pub fn axq_dequantize(ctx: *mut axq_ctx, ty: c_int, packed: *const c_void, numel: usize,
                          dst: *mut f32, mem: c_int) -> c_int;

    pub fn axq_weight_upload(ctx: *mut axq_ctx, ty: c_int, n_rows: i64, k: i64, packed: *const c_void,
                             bytes: usize, mem: c_int, out: *mut *mut axq_weight) -> c_int;
    pub fn axq_weight_quantize(ctx: *mut axq_ctx, ty: c_int, n_rows: i64, k: i64, w: *const f32,
                               mem: c_int, out: *mut *mut axq_weight) -> c_int;
    pub fn axq_weight_download(ctx: *mut axq_ctx, w: *const axq_weight, packed: *mut c_void,
                               bytes: usize, mem: c_int) -> c_int;
    pub fn axq_weight_free(ctx: *mut axq_ctx, w: *mut axq_weight);

    pub fn axq_gemv_f32(ctx: *mut axq_ctx, w: *const axq_weight, x: *const f32, batch: c_int,
                        bias: *const f32, y: *mut f32, mem: c_int) -> c_int;
    /// `axq_gemv_f32` for 2..=8 vectors on device pointers that allocates nothing (callers under graph capture).
    pub fn axq_gemv_f32_static(ctx: *mut axq_ctx, w: *const axq_weight, x: *const f32, batch: c_int,
                               bias: *const f32, y: *mut f32) -> c_int;
    pub fn axq_gemm_bf16(ctx: *mut axq_ctx, w: *const axq_weight, x_bf16: *const u16, m: c_int,
                         y: *mut f32, mem: c_int) -> c_int;

    pub fn axq_model_create(ctx: *mut axq_ctx, cfg: *const axq_model_config, out: *mut *mut axq_model) -> c_int;
    pub fn axq_model_free(m: *mut axq_model);
    pub fn axq_model_set_embedding_f16(m: *mut axq_model, table: *const u16, mem: c_int) -> c_int;
    pub fn axq_model_set_embedding_f32(m: *mut axq_model, table: *const f32, mem: c_int) -> c_int;
    pub fn axq_model_set_norm(m: *mut axq_model, layer: c_int, which: c_int, w: *const f32, mem: c_int) -> c_int;
    pub fn axq_model_set_linear(m: *mut axq_model, layer: c_int, which: c_int, w: *const axq_weight) -> c_int;
    pub fn axq_model_reset(m: *mut axq_model) -> c_int;
    pub fn axq_model_truncate(m: *mut axq_model, n_positions: c_int) -> c_int;
    pub fn axq_model_forward(m: *mut axq_model, token: i32, logits: *mut f32, next: *mut i32) -> c_int;
    pub fn axq_model_forward_tokens(m: *mut axq_model, tokens: *const i32, n: c_int, logits: *mut f32,
                                    next: *mut i32) -> c_int;
    pub fn axq_model_set_batch(m: *mut axq_model, n_seq: c_int) -> c_int;
    pub fn axq_model_copy_sequence(m: *mut axq_model, src: c_int, dst: c_int) -> c_int;
    pub fn axq_model_forward_batch(m: *mut axq_model, tokens: *const i32, logits: *mut f32, next: *mut i32) -> c_int;
    pub fn axq_model_generate_batch(m: *mut axq_model, prompts: *const i32, offsets: *const i32, max_new: c_int,
                                    out: *mut i32, prefill_ms: *mut f32, decode_ms: *mut f32) -> c_int;
    pub fn axq_model_generate(m: *mut axq_model, prompt: *const i32, n_prompt: c_int, max_new: c_int,
                              out: *mut i32, prefill_ms: *mut f32, decode_ms: *mut f32) -> c_int;
}
