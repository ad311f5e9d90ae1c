//! Raw declarations of `include/hipcompute.h`, one to one and in the header's order.
//! Nothing here is safe to call without the header's comments at hand; `lib.rs` is the safe surface.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};

macro_rules! opaque {
    ($($name:ident),*) => { $(#[repr(C)] pub struct $name { _private: [u8; 0] })* };
}
opaque!(hipc_ctx, hipc_graph, hipc_nbits_weight, hipc_int8_weight, hipc_conv_weight, hipc_decoder);

pub const HIPC_OK: c_int = 0;
pub const HIPC_ERR_INVALID: c_int = 1;
pub const HIPC_ERR_UNSUPPORTED: c_int = 2;
pub const HIPC_ERR_BACKEND: c_int = 3;

/// element types, numbered as ONNX `TensorProto.DataType`
pub const HIPC_F32: c_int = 1;
pub const HIPC_U8: c_int = 2;
pub const HIPC_I8: c_int = 3;
pub const HIPC_I32: c_int = 6;
pub const HIPC_F16: c_int = 10;

pub const HIPC_DQL_STATIC_MAX_N: i64 = 1 << 30;

/// `ConvGeom` (interp.rs:3361-3536): NCHW, 1-D given as H = 1
#[repr(C)]
#[derive(Clone, Copy, Debug, Default, PartialEq, Eq)]
pub struct hipc_conv_geom {
    pub n: i64,
    pub c_in: i64,
    pub h: i64,
    pub w: i64,
    pub c_out: i64,
    pub kh: i64,
    pub kw: i64,
    pub stride_h: i64,
    pub stride_w: i64,
    pub dil_h: i64,
    pub dil_w: i64,
    pub pad_top: i64,
    pub pad_left: i64,
    pub pad_bottom: i64,
    pub pad_right: i64,
    pub group: i64,
}

#[repr(C)]
#[derive(Clone, Copy, Debug, Default, PartialEq)]
pub struct hipc_decoder_config {
    pub n_layers: i32,
    pub hidden: i32,
    pub ffn: i32,
    pub n_q_heads: i32,
    pub n_kv_heads: i32,
    pub head_dim: i32,
    pub vocab: i32,
    pub max_seq: i32,
    pub block_size: i32,
    pub rms_eps: f32,
    pub rope_theta: f32,
    /// 0 => 1 / sqrt(head_dim)
    pub attn_scale: f32,
    /// the embedding row is multiplied by this (gemma: sqrt(hidden))
    pub embed_scale: f32,
}

pub const HIPC_INITIALIZER_MAX_DIMS: usize = 8;

/// what `hipc_initializer_read` reports about a TensorProto
#[repr(C)]
#[derive(Clone, Copy)]
pub struct hipc_initializer_info {
    /// `TensorProto.DataType` (the `HIPC_*` element types use the same numbers)
    pub data_type: i32,
    pub n_dims: i32,
    pub dims: [i64; HIPC_INITIALIZER_MAX_DIMS],
    /// length of the little-endian payload
    pub bytes: usize,
    /// NUL-terminated
    pub name: [c_char; 256],
}

pub const HIPC_DEC_QKV: c_int = 0;
pub const HIPC_DEC_O: c_int = 1;
pub const HIPC_DEC_GATE_UP: c_int = 2;
pub const HIPC_DEC_DOWN: c_int = 3;
pub const HIPC_DEC_LM_HEAD: c_int = 4;
pub const HIPC_DEC_NORM_INPUT: c_int = 0;
pub const HIPC_DEC_NORM_POST_ATTN: c_int = 1;
pub const HIPC_DEC_NORM_PRE_FFN: c_int = 2;
pub const HIPC_DEC_NORM_POST_FFN: c_int = 3;
pub const HIPC_DEC_NORM_Q: c_int = 4;
pub const HIPC_DEC_NORM_K: c_int = 5;
pub const HIPC_DEC_NORM_FINAL: c_int = 6;

unsafe extern "C" {
    // ---- context
    pub fn hipc_ctx_create(device: c_int, out: *mut *mut hipc_ctx) -> c_int;
    pub fn hipc_ctx_create_on_stream(device: c_int, stream: *mut c_void, out: *mut *mut hipc_ctx) -> c_int;
    pub fn hipc_ctx_destroy(ctx: *mut hipc_ctx);
    pub fn hipc_last_error(ctx: *mut hipc_ctx) -> *const c_char;
    pub fn hipc_version() -> *const c_char;
    pub fn hipc_stream(ctx: *mut hipc_ctx) -> *mut c_void;
    pub fn hipc_set_option(ctx: *mut hipc_ctx, name: *const c_char, value: c_int) -> c_int;

    // ---- buffers
    pub fn hipc_alloc(ctx: *mut hipc_ctx, bytes: usize, dptr: *mut *mut c_void) -> c_int;
    pub fn hipc_free_deferred(ctx: *mut hipc_ctx, dptr: *mut c_void) -> c_int;
    pub fn hipc_pool_stats(ctx: *mut hipc_ctx, hits: *mut usize, misses: *mut usize, bytes_waiting: *mut usize) -> c_int;
    pub fn hipc_upload(ctx: *mut hipc_ctx, dst: *mut c_void, dst_offset: usize, host: *const c_void, bytes: usize) -> c_int;
    pub fn hipc_download(ctx: *mut hipc_ctx, host: *mut c_void, src: *const c_void, src_offset: usize, bytes: usize) -> c_int;
    pub fn hipc_copy(ctx: *mut hipc_ctx, dst: *mut c_void, dst_offset: usize, src: *const c_void, src_offset: usize, bytes: usize) -> c_int;
    pub fn hipc_fill(ctx: *mut hipc_ctx, dst: *mut c_void, dst_offset: usize, bytes: usize, word: u32) -> c_int;
    pub fn hipc_flush(ctx: *mut hipc_ctx) -> c_int;

    // ---- capture and replay
    pub fn hipc_capture_begin(ctx: *mut hipc_ctx) -> c_int;
    pub fn hipc_capture_end(ctx: *mut hipc_ctx, out: *mut *mut hipc_graph) -> c_int;
    pub fn hipc_graph_launch(ctx: *mut hipc_ctx, graph: *mut hipc_graph) -> c_int;
    pub fn hipc_graph_destroy(ctx: *mut hipc_ctx, graph: *mut hipc_graph);
    pub fn hipc_graph_op_count(ctx: *mut hipc_ctx, graph: *mut hipc_graph, count: *mut c_int) -> c_int;
    pub fn hipc_graph_set_scalar(ctx: *mut hipc_ctx, graph: *mut hipc_graph, op: c_int, which: c_int, value: i32) -> c_int;
    pub fn hipc_measure_graph(ctx: *mut hipc_ctx, graph: *mut hipc_graph, samples: c_int, launches_per_sample: c_int, ns_out: *mut f64) -> c_int;
    pub fn hipc_probe_int8_mfma(ctx: *mut hipc_ctx, random_operands: c_int, waves_per_simd: c_int, iterations: c_int, tops: *mut f64) -> c_int;

    // ---- MatMulNBits
    pub fn hipc_matmul_nbits(
        ctx: *mut hipc_ctx, a: *const c_void, a_dtype: c_int, b: *const c_void, b_len: usize, scales: *const c_void,
        scale_dtype: c_int, scales_len: usize, zp: *const c_void, zp_len: usize, y: *mut c_void, m: i64, k: i64, n: i64,
        block_size: i64, accuracy_level: c_int,
    ) -> c_int;
    pub fn hipc_prepack_matmul_nbits(
        ctx: *mut hipc_ctx, b: *const c_void, b_len: usize, scales: *const c_void, scale_dtype: c_int, scales_len: usize,
        zp: *const c_void, zp_len: usize, k: i64, n: i64, block_size: i64, out: *mut *mut hipc_nbits_weight,
    ) -> c_int;
    pub fn hipc_nbits_weight_destroy(ctx: *mut hipc_ctx, w: *mut hipc_nbits_weight);
    pub fn hipc_nbits_weight_bytes(w: *const hipc_nbits_weight) -> usize;
    pub fn hipc_matmul_nbits_packed(
        ctx: *mut hipc_ctx, a: *const c_void, a_dtype: c_int, w: *const hipc_nbits_weight, y: *mut c_void, m: i64,
        accuracy_level: c_int,
    ) -> c_int;

    // ---- DynamicQuantizeLinear, DecomposedGelu
    pub fn hipc_dynamic_quantize_linear(
        ctx: *mut hipc_ctx, x: *const c_void, n: i64, y: *mut c_void, scale_out: *mut c_void, zp_out: *mut c_void,
        range: *mut c_void, range_ready: c_int,
    ) -> c_int;
    pub fn hipc_decomposed_gelu(
        ctx: *mut hipc_ctx, x: *const c_void, n: i64, divisor: f32, offset: f32, factor: f32, factor_first: c_int, y: *mut c_void,
    ) -> c_int;
    pub fn hipc_dynamic_quantize_linear_gelu(
        ctx: *mut hipc_ctx, x: *const c_void, n: i64, divisor: f32, offset: f32, factor: f32, factor_first: c_int,
        y: *mut c_void, scale_out: *mut c_void, zp_out: *mut c_void, range: *mut c_void,
    ) -> c_int;
    pub fn hipc_dynamic_quantize_linear_static(
        ctx: *mut hipc_ctx, x: *const c_void, n: i64, y: *mut c_void, scale_out: *mut c_void, zp_out: *mut c_void,
    ) -> c_int;

    // ---- MatMulInteger
    pub fn hipc_prepack_int8_b(ctx: *mut hipc_ctx, b: *const c_void, b_dtype: c_int, k: i64, n: i64, out: *mut *mut hipc_int8_weight) -> c_int;
    pub fn hipc_int8_weight_destroy(ctx: *mut hipc_ctx, w: *mut hipc_int8_weight);
    pub fn hipc_matmul_integer(
        ctx: *mut hipc_ctx, a: *const c_void, a_dtype: c_int, b: *const hipc_int8_weight, a_zp: *const c_void,
        b_zp: *const c_void, y: *mut c_void, m: i64,
    ) -> c_int;
    pub fn hipc_matmul_integer_raw(
        ctx: *mut hipc_ctx, a: *const c_void, a_dtype: c_int, b: *const c_void, b_dtype: c_int, a_zp: *const c_void,
        b_zp: *const c_void, y: *mut c_void, m: i64, k: i64, n: i64,
    ) -> c_int;
    pub fn hipc_matmul_integer_scale_bias(
        ctx: *mut hipc_ctx, a: *const c_void, a_dtype: c_int, b: *const hipc_int8_weight, a_zp: *const c_void,
        b_zp: *const c_void, scale: *const c_void, scale_step: c_int, product: *const c_void, product_step: c_int,
        bias: *const c_void, bias_step: c_int, relu: c_int, range: *mut c_void, y: *mut c_void, m: i64,
    ) -> c_int;

    // ---- Requantize / QLinearMatMul
    pub fn hipc_requantize(
        ctx: *mut hipc_ctx, acc: *const c_void, bias: *const c_void, ratio: *const c_void, n: i64, inner: i64,
        axis_len: i64, y_zp: i32, out_dtype: c_int, out: *mut c_void,
    ) -> c_int;
    pub fn hipc_qlinear_matmul(
        ctx: *mut hipc_ctx, a: *const c_void, a_dtype: c_int, a_scale: f32, a_zp: i32, b: *const hipc_int8_weight,
        b_scale: *const f32, n_b_scale: i64, b_zp: i32, y_scale: f32, y_zp: i32, y_dtype: c_int, y: *mut c_void, m: i64,
    ) -> c_int;

    // ---- ConvInteger / QLinearConv
    pub fn hipc_conv_out_shape(g: *const hipc_conv_geom, h_out: *mut i64, w_out: *mut i64) -> c_int;
    pub fn hipc_same_pads(input: i64, kernel: i64, stride: i64, dilation: i64, upper: c_int, pad_begin: *mut i64, pad_end: *mut i64);
    pub fn hipc_prepack_conv_w(ctx: *mut hipc_ctx, w: *const c_void, w_dtype: c_int, g: *const hipc_conv_geom, out: *mut *mut hipc_conv_weight) -> c_int;
    pub fn hipc_conv_weight_destroy(ctx: *mut hipc_ctx, w: *mut hipc_conv_weight);
    pub fn hipc_conv_integer(
        ctx: *mut hipc_ctx, x: *const c_void, x_dtype: c_int, w: *const hipc_conv_weight, x_zp: *const c_void,
        w_zp: *const c_void, g: *const hipc_conv_geom, y: *mut c_void,
    ) -> c_int;
    pub fn hipc_qlinear_conv(
        ctx: *mut hipc_ctx, x: *const c_void, x_dtype: c_int, x_scale: f32, x_zp: i32, w: *const hipc_conv_weight,
        w_scale: *const f32, n_w_scale: i64, w_zp: i32, y_scale: f32, y_zp: i32, y_dtype: c_int, bias: *const c_void,
        g: *const hipc_conv_geom, y: *mut c_void,
    ) -> c_int;

    // ---- ONNX initializers (host code only)
    pub fn hipc_initializer_read(
        tensor: *const c_void, len: usize, base_dir: *const c_char, info: *mut hipc_initializer_info, data: *mut c_void,
        data_cap: usize,
    ) -> c_int;
    pub fn hipc_model_initializers(
        model: *const c_void, len: usize, offsets: *mut usize, sizes: *mut usize, cap: i64, count: *mut i64,
    ) -> c_int;
    pub fn hipc_host_error() -> *const c_char;

    // ---- decode step
    pub fn hipc_decoder_create(ctx: *mut hipc_ctx, cfg: *const hipc_decoder_config, out: *mut *mut hipc_decoder) -> c_int;
    pub fn hipc_decoder_destroy(ctx: *mut hipc_ctx, dec: *mut hipc_decoder);
    pub fn hipc_decoder_set_linear(
        ctx: *mut hipc_ctx, dec: *mut hipc_decoder, layer: c_int, which: c_int, b: *const c_void, b_len: usize,
        scales: *const c_void, scales_len: usize, zp: *const c_void, zp_len: usize,
    ) -> c_int;
    pub fn hipc_decoder_set_norm(ctx: *mut hipc_ctx, dec: *mut hipc_decoder, layer: c_int, which: c_int, w: *const c_void) -> c_int;
    pub fn hipc_decoder_set_embedding(
        ctx: *mut hipc_ctx, dec: *mut hipc_decoder, b: *const c_void, b_len: usize, scales: *const c_void,
        scales_len: usize, zp: *const c_void, zp_len: usize,
    ) -> c_int;
    pub fn hipc_decoder_set_layer_attention(ctx: *mut hipc_ctx, dec: *mut hipc_decoder, layer: c_int, window: i32, rope_theta: f32) -> c_int;
    pub fn hipc_decoder_reset(ctx: *mut hipc_ctx, dec: *mut hipc_decoder, token: i32, pos: i32) -> c_int;
    pub fn hipc_decoder_kv_cache(ctx: *mut hipc_ctx, dec: *mut hipc_decoder, layer: c_int, k_cache: *mut *mut c_void, v_cache: *mut *mut c_void) -> c_int;
    pub fn hipc_decoder_step(ctx: *mut hipc_ctx, dec: *mut hipc_decoder) -> c_int;
    pub fn hipc_decoder_read(
        ctx: *mut hipc_ctx, dec: *mut hipc_decoder, token: *mut i32, pos: *mut i32, logits: *mut f32, history: *mut i32,
        n_history: i32,
    ) -> c_int;
}
