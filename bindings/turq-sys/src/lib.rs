//! Raw FFI declarations of `libturq` (include/turq.h): GGUF block-quantized linear layers on MI355X (gfx950).
//!
//! One `extern "C"` item per entry point of the header, same order, same names.  The safe layer is the `tur-hip` crate.
//! UNCOMPILED in the tree this file ships in (its image has no Rust toolchain); `tests/test_rust_bindings.py` checks every
//! declaration here against the header mechanically: name, number of arguments, pointer depth and constness, integer widths.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};

#[repr(C)]
pub struct turq_ctx {
    _private: [u8; 0],
}
#[repr(C)]
pub struct turq_weight {
    _private: [u8; 0],
}
#[repr(C)]
pub struct turq_gguf {
    _private: [u8; 0],
}
#[repr(C)]
pub struct turq_graph {
    _private: [u8; 0],
}

// status codes
pub const TURQ_OK: c_int = 0;
pub const TURQ_ERR_INVALID: c_int = 1;
pub const TURQ_ERR_SHAPE: c_int = 2;
pub const TURQ_ERR_DTYPE: c_int = 3;
pub const TURQ_ERR_HIP: c_int = 4;
pub const TURQ_ERR_OOM: c_int = 5;
pub const TURQ_ERR_IO: c_int = 6;
pub const TURQ_ERR_NOT_FOUND: c_int = 7;

// ggml dtype ids as stored in GGUF tensor infos (candle GgmlDType)
pub const TURQ_F32: c_int = 0;
pub const TURQ_F16: c_int = 1;
pub const TURQ_Q8_0: c_int = 8;
pub const TURQ_Q4_K: c_int = 12;
pub const TURQ_Q5_K: c_int = 13;
pub const TURQ_Q6_K: c_int = 14;
pub const TURQ_BF16: c_int = 30;

// element type of activation / output buffers
pub const TURQ_ACT_F32: c_int = 0;
pub const TURQ_ACT_BF16: c_int = 1;
pub const TURQ_ACT_F16: c_int = 2;
/// OR-ed into the y_dtype of turq_qmatmul / turq_qmatmul_noalloc / turq_mlp / turq_norm_mlp: results are added to y
pub const TURQ_OUT_ACCUMULATE: c_int = 0x100;

// weight layouts in HBM
pub const TURQ_LAYOUT_NATIVE: c_int = 0;
pub const TURQ_LAYOUT_TILED: c_int = 1;

// where the pointers of a call live
pub const TURQ_MEM_HOST: c_int = 0;
pub const TURQ_MEM_DEVICE: c_int = 1;

// matmul algorithm selection
pub const TURQ_ALGO_AUTO: c_int = 0;
pub const TURQ_ALGO_SIMPLE: c_int = 1;
pub const TURQ_ALGO_GEMV: c_int = 2;
pub const TURQ_ALGO_GEMM: c_int = 3;

pub const TURQ_ACTFN_SILU: c_int = 0;

/// bytes of the static scratch array of `turq_qmatmul_noalloc`
pub const TURQ_NOALLOC_SCRATCH_BYTES: usize = 16 << 20;

#[link(name = "turq")]
extern "C" {
    pub fn turq_version() -> *const c_char;
    pub fn turq_block_elems(ggml_dtype: c_int) -> c_int;
    pub fn turq_block_bytes(ggml_dtype: c_int) -> c_int;
    pub fn turq_weight_nbytes(ggml_dtype: c_int, n: i64, k: i64) -> usize;
    pub fn turq_ctx_create(device_ordinal: c_int, out: *mut *mut turq_ctx) -> c_int;
    pub fn turq_ctx_destroy(ctx: *mut turq_ctx);
    pub fn turq_last_error(ctx: *const turq_ctx) -> *const c_char;
    pub fn turq_sync(ctx: *mut turq_ctx) -> c_int;
    pub fn turq_ctx_stream(ctx: *mut turq_ctx) -> *mut c_void;
    pub fn turq_ctx_set_wide_activations(ctx: *mut turq_ctx, on: c_int) -> c_int;
    pub fn turq_ctx_nonfinite_count(ctx: *mut turq_ctx, count: *mut u64, reset: c_int) -> c_int;
    pub fn turq_ctx_device_info(ctx: *mut turq_ctx, name: *mut c_char, name_cap: usize, compute_units: *mut c_int) -> c_int;
    pub fn turq_dev_alloc(ctx: *mut turq_ctx, nbytes: usize, out: *mut *mut c_void) -> c_int;
    pub fn turq_dev_free(ctx: *mut turq_ctx, ptr: *mut c_void) -> c_int;
    pub fn turq_memcpy_h2d(ctx: *mut turq_ctx, dst_dev: *mut c_void, src_host: *const c_void, nbytes: usize) -> c_int;
    pub fn turq_memcpy_d2h(ctx: *mut turq_ctx, dst_host: *mut c_void, src_dev: *const c_void, nbytes: usize) -> c_int;
    pub fn turq_weight_upload(ctx: *mut turq_ctx, ggml_dtype: c_int, n: i64, k: i64, host_bytes: *const c_void, nbytes: usize, layout: c_int, out: *mut *mut turq_weight) -> c_int;
    pub fn turq_weight_retain(w: *mut turq_weight) -> c_int;
    pub fn turq_weight_release(w: *mut turq_weight) -> c_int;
    pub fn turq_weight_info(w: *const turq_weight, ggml_dtype: *mut c_int, n: *mut i64, k: *mut i64, layout: *mut c_int, device_bytes: *mut usize) -> c_int;
    pub fn turq_weight_export(ctx: *mut turq_ctx, w: *const turq_weight, host_bytes: *mut c_void, nbytes: usize) -> c_int;
    pub fn turq_tiled_nbytes(ggml_dtype: c_int, n: i64, k: i64) -> usize;
    pub fn turq_tile_host(ggml_dtype: c_int, n: i64, k: i64, native: *const c_void, tiled: *mut c_void) -> c_int;
    pub fn turq_untile_host(ggml_dtype: c_int, n: i64, k: i64, tiled: *const c_void, native: *mut c_void) -> c_int;
    pub fn turq_dequantize(ctx: *mut turq_ctx, w: *const turq_weight, out: *mut f32, out_mem: c_int) -> c_int;
    pub fn turq_embedding_lookup(ctx: *mut turq_ctx, w: *const turq_weight, ids: *const u32, count: i64, out: *mut c_void, out_dtype: c_int, ldo: i64, mem: c_int) -> c_int;
    pub fn turq_rms_norm(ctx: *mut turq_ctx, x: *const c_void, x_dtype: c_int, m: i64, k: i64, ldx: i64, weight: *const f32, eps: f32, y: *mut c_void, y_dtype: c_int, ldy: i64, mem: c_int) -> c_int;
    pub fn turq_qmatmul(ctx: *mut turq_ctx, w: *const turq_weight, x: *const c_void, x_dtype: c_int, m: i64, ldx: i64, y: *mut c_void, y_dtype: c_int, ldy: i64, bias: *const f32, mem: c_int, algo: c_int) -> c_int;
    pub fn turq_qmatmul_noalloc(ctx: *mut turq_ctx, w: *const turq_weight, x: *const c_void, x_dtype: c_int, m: i64, ldx: i64, y: *mut c_void, y_dtype: c_int, ldy: i64, bias: *const f32) -> c_int;
    pub fn turq_qmatmul_multi(ctx: *mut turq_ctx, count: c_int, weights: *const *const turq_weight, x: *const c_void, x_dtype: c_int, m: i64, ldx: i64, ys: *const *mut c_void, y_dtype: c_int, ldys: *const i64, biases: *const *const f32, mem: c_int, algo: c_int) -> c_int;
    pub fn turq_qmatmul_gate_up(ctx: *mut turq_ctx, gate: *const turq_weight, up: *const turq_weight, x: *const c_void, x_dtype: c_int, m: i64, ldx: i64, y: *mut c_void, y_dtype: c_int, ldy: i64, bias_gate: *const f32, bias_up: *const f32, act: c_int, mem: c_int) -> c_int;
    pub fn turq_mlp(ctx: *mut turq_ctx, gate: *const turq_weight, up: *const turq_weight, down: *const turq_weight, x: *const c_void, x_dtype: c_int, m: i64, ldx: i64, y: *mut c_void, y_dtype: c_int, ldy: i64, bias_gate: *const f32, bias_up: *const f32, bias_down: *const f32, act: c_int, mem: c_int) -> c_int;
    pub fn turq_norm_qmatmul_multi(ctx: *mut turq_ctx, count: c_int, weights: *const *const turq_weight, x: *const c_void, x_dtype: c_int, m: i64, ldx: i64, norm_weight: *const f32, eps: f32, ys: *const *mut c_void, y_dtype: c_int, ldys: *const i64, biases: *const *const f32, mem: c_int) -> c_int;
    pub fn turq_norm_mlp(ctx: *mut turq_ctx, gate: *const turq_weight, up: *const turq_weight, down: *const turq_weight, x: *const c_void, x_dtype: c_int, m: i64, ldx: i64, norm_weight: *const f32, eps: f32, y: *mut c_void, y_dtype: c_int, ldy: i64, bias_gate: *const f32, bias_up: *const f32, bias_down: *const f32, act: c_int, mem: c_int) -> c_int;
    pub fn turq_weight_prefetch(ctx: *mut turq_ctx, w: *const turq_weight) -> c_int;
    pub fn turq_quantize_q8_0(ctx: *mut turq_ctx, x: *const f32, m: i64, k: i64, out: *mut c_void, mem: c_int) -> c_int;
    pub fn turq_quantize_q8_k(ctx: *mut turq_ctx, x: *const f32, m: i64, k: i64, out: *mut c_void, mem: c_int) -> c_int;
    pub fn turq_graph_begin(ctx: *mut turq_ctx) -> c_int;
    pub fn turq_graph_end(ctx: *mut turq_ctx, out: *mut *mut turq_graph) -> c_int;
    pub fn turq_graph_launch(ctx: *mut turq_ctx, g: *mut turq_graph) -> c_int;
    pub fn turq_graph_destroy(g: *mut turq_graph);
    pub fn turq_ctx_scratch_info(ctx: *const turq_ctx, live_graphs: *mut c_int, retired_buffers: *mut c_int, act_prep_bytes: *mut usize) -> c_int;
    pub fn turq_profile_begin(ctx: *mut turq_ctx) -> c_int;
    pub fn turq_profile_end(ctx: *mut turq_ctx, launches: *mut i64, total_ms: *mut f64) -> c_int;
    pub fn turq_read_yardstick(ctx: *mut turq_ctx, dev_ptr: *const c_void, nbytes: usize) -> c_int;
    pub fn turq_prefill_plan(
        dtype: c_int,
        n: i64,
        k: i64,
        m: i64,
        compute_units: c_int,
        tile: *mut c_int,
        split: *mut c_int,
        wave_groups: *mut c_int,
    ) -> c_int;
    pub fn turq_prefill_plan_multi(dtype: c_int, n: i64, k: i64, m: i64, count: c_int, compute_units: c_int, merged: *mut c_int) -> c_int;
    pub fn turq_tuning_describe(buf: *mut c_char, cap: usize, needed: *mut usize) -> c_int;
    pub fn turq_gguf_open(path: *const c_char, out: *mut *mut turq_gguf) -> c_int;
    pub fn turq_gguf_close(g: *mut turq_gguf);
    pub fn turq_gguf_last_error(g: *const turq_gguf) -> *const c_char;
    pub fn turq_gguf_tensor_count(g: *const turq_gguf) -> i64;
    pub fn turq_gguf_tensor_name(g: *const turq_gguf, index: i64) -> *const c_char;
    pub fn turq_gguf_tensor_info(g: *const turq_gguf, name: *const c_char, ggml_dtype: *mut c_int, n_dims: *mut c_int, dims: *mut i64, file_offset: *mut u64, nbytes: *mut usize) -> c_int;
    pub fn turq_gguf_meta_u64(g: *const turq_gguf, key: *const c_char, out: *mut u64) -> c_int;
    pub fn turq_gguf_meta_f64(g: *const turq_gguf, key: *const c_char, out: *mut f64) -> c_int;
    pub fn turq_gguf_meta_str(g: *const turq_gguf, key: *const c_char, out: *mut c_char, cap: usize) -> c_int;
    pub fn turq_gguf_read_tensor(g: *mut turq_gguf, name: *const c_char, host_bytes: *mut c_void, nbytes: usize) -> c_int;
    pub fn turq_gguf_load_weight(ctx: *mut turq_ctx, g: *mut turq_gguf, name: *const c_char, expect_n: i64, expect_k: i64, layout: c_int, out: *mut *mut turq_weight) -> c_int;
}
