//! Raw FFI bindings to `libronn_bitnet_hip.so`, the MI355X (gfx950) implementation of RONN's
//! BitNet ternary hot path.
//!
//! One `extern "C"` declaration per entry point of `include/ronn_bitnet_hip.h` (kernel level,
//! `rbn_*`) and `include/ronn_bitnet_provider.h` (provider level, `rbp_*`), in header order,
//! with the same parameter names.  A test of the library's repository parses both headers and
//! this file and fails on a missing symbol or a different number of parameters.
//!
//! The functions these stand in for are cited in the headers; in short:
//! `BitNetQuantizer::quantize_ternary` / `pack_ternary_bits` / `dequantize_ternary`
//! (`crates/ronn-providers/src/bitnet/quantization.rs:67-207`), `TernaryTensor::get_value`
//! (`:275-291`), `BitNetKernel::execute_ternary_matmul` and `CompiledKernel::execute`
//! (`bitnet/kernels.rs:134-178`, `:254-319`), `BitNetMemoryAllocator` (`bitnet/allocator.rs:39-149`).
//!
//! Conventions of the C side: every call returns 0 or a negative status and never unwinds;
//! `rbn_last_error()` / `rbp_last_error()` give the calling thread's last message; `d_*`
//! pointers are device memory, `h_*` host memory; a context serialises its callers, so the
//! safe wrappers may be `Send + Sync`.
#![allow(non_camel_case_types, non_snake_case, clippy::too_many_arguments)]

use std::ffi::CStr;
use std::os::raw::{c_char, c_int, c_void};

/// Opaque context: one GPU, one HIP stream, an internal lock.
#[repr(C)]
pub struct rbn_ctx {
    _private: [u8; 0],
}
/// Opaque captured HIP graph.
#[repr(C)]
pub struct rbn_graph {
    _private: [u8; 0],
}
/// Opaque provider-level objects of `ronn_bitnet_provider.h`.
#[repr(C)]
pub struct rbp_provider {
    _private: [u8; 0],
}
#[repr(C)]
pub struct rbp_kernel {
    _private: [u8; 0],
}
#[repr(C)]
pub struct rbp_ternary {
    _private: [u8; 0],
}

// rbn_status
pub const RBN_OK: c_int = 0;
pub const RBN_ERR_INVALID: c_int = -1;
pub const RBN_ERR_HIP: c_int = -2;
pub const RBN_ERR_OOM: c_int = -3;
pub const RBN_ERR_UNSUPPORTED: c_int = -4;
pub const RBN_ERR_NO_DEVICE: c_int = -5;
pub const RBP_OK: c_int = 0;
pub const RBP_ERR: c_int = -1;

// rbn_sum_mode
/// Bit-exact emulation of the reference's `iter().sum::<f32>()` (quantization.rs:79, :96).
pub const RBN_SUM_STRICT_SEQ: c_int = 0;
/// f64 tree reduction: faster, NOT reference-exact on large tensors.
pub const RBN_SUM_TREE: c_int = 1;

pub const RBN_GEMV_MAX_M: u64 = 16;
pub const RBN_SKINNY_MAX_M: u64 = 64;
pub const RBN_GEMV_GROUP_MAX: usize = 32;
pub const RBN_KERNEL_GEMV: c_int = 0;
pub const RBN_KERNEL_SKINNY: c_int = 1;
pub const RBN_KERNEL_MFMA: c_int = 2;
pub const RBN_FLAG_HISTORY_OVERFLOW: u32 = 1;
pub const RBN_STATIC_SCRATCH_TILES: usize = 1024;
pub const RBN_STATIC_SCRATCH_BYTES: usize = RBN_STATIC_SCRATCH_TILES * 4096 + 128 * 4;

// DataType codes of rbn_tensor_bytes / rbp_* (declaration order of ronn_core::DataType,
// crates/ronn-core/src/types.rs:39-60)
pub const RBN_DT_F32: c_int = 0;
pub const RBN_DT_F16: c_int = 1;
pub const RBN_DT_BF16: c_int = 2;
pub const RBN_DT_I8: c_int = 3;
pub const RBN_DT_I32: c_int = 4;
pub const RBN_DT_I64: c_int = 5;
pub const RBN_DT_U8: c_int = 6;
pub const RBN_DT_U32: c_int = 7;
pub const RBN_DT_BOOL: c_int = 8;
pub const RBN_DT_F64: c_int = 9;

#[repr(C)]
#[derive(Clone, Copy)]
pub struct rbn_device_info {
    pub name: [c_char; 128],
    pub arch: [c_char; 64],
    pub compute_units: c_int,
    pub clock_khz: c_int,
    pub mem_clock_khz: c_int,
    pub mem_bus_bits: c_int,
    pub hbm_bytes: u64,
    pub l2_bytes: u64,
}

/// One GEMV of a grouped launch (`rbn_gemv_t2_i8_grouped`); the pointers are device pointers.
#[repr(C)]
#[derive(Clone, Copy)]
pub struct rbn_gemv_problem {
    pub d_q: *const i8,
    pub d_act_scale: *const f32,
    pub d_rowsum: *const i32,
    pub d_tiled: *const u32,
    pub d_out: *mut f32,
    pub d_acc: *mut i32,
    pub w_scale: f32,
    pub reserved: u32,
}

/// `BitNetProviderConfig` (bitnet/provider.rs:41-55) plus `activation`,
/// `strict_reference_sum` and `device`.
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct rbp_config {
    pub quantization_method: c_int,
    pub enable_kernel_caching: c_int,
    pub max_cache_size: u64,
    pub enable_mixed_precision: c_int,
    pub memory_optimization_level: c_int,
    pub enable_simd: c_int,
    pub activation: c_int,
    pub strict_reference_sum: c_int,
    pub device: c_int,
}

#[link(name = "ronn_bitnet_hip")]
extern "C" {
// ---- include/ronn_bitnet_hip.h ----
    pub fn rbn_version() -> *const c_char;
    pub fn rbn_last_error() -> *const c_char;
    pub fn rbn_device_count() -> c_int;
    pub fn rbn_ctx_create(device: c_int, out: *mut *mut rbn_ctx) -> c_int;
    pub fn rbn_ctx_destroy(ctx: *mut rbn_ctx) -> c_int;
    pub fn rbn_get_device_info(ctx: *mut rbn_ctx, out: *mut rbn_device_info) -> c_int;
    pub fn rbn_malloc(ctx: *mut rbn_ctx, bytes: usize, d_out: *mut *mut c_void) -> c_int;
    pub fn rbn_free(ctx: *mut rbn_ctx, d_ptr: *mut c_void) -> c_int;
    pub fn rbn_h2d(ctx: *mut rbn_ctx, d_dst: *mut c_void, h_src: *const c_void, bytes: usize) -> c_int;
    pub fn rbn_d2h(ctx: *mut rbn_ctx, h_dst: *mut c_void, d_src: *const c_void, bytes: usize) -> c_int;
    pub fn rbn_d2d(ctx: *mut rbn_ctx, d_dst: *mut c_void, d_src: *const c_void, bytes: usize) -> c_int;
    pub fn rbn_fill_u8(ctx: *mut rbn_ctx, d_dst: *mut c_void, value: c_int, bytes: usize) -> c_int;
    pub fn rbn_sync(ctx: *mut rbn_ctx) -> c_int;
    pub fn rbn_device_flags(ctx: *mut rbn_ctx, h_flags: *mut u32) -> c_int;
    pub fn rbn_memory_info(ctx: *mut rbn_ctx, allocated: *mut u64, peak: *mut u64) -> c_int;
    pub fn rbn_tensor_bytes(element_count: u64, dtype: c_int) -> i64;
    pub fn rbn_tensor_alignment(dtype: c_int) -> usize;
    pub fn rbn_packed_capacity(n: u64) -> usize;
    pub fn rbn_tiled_bytes(K: u64, N: u64) -> usize;
    pub fn rbn_act_pitch(K: u64) -> usize;
    pub fn rbn_timer_start(ctx: *mut rbn_ctx) -> c_int;
    pub fn rbn_timer_stop(ctx: *mut rbn_ctx, h_ms: *mut f32) -> c_int;
    pub fn rbn_graph_begin_capture(ctx: *mut rbn_ctx) -> c_int;
    pub fn rbn_graph_end_capture(ctx: *mut rbn_ctx, out: *mut *mut rbn_graph) -> c_int;
    pub fn rbn_graph_launch(ctx: *mut rbn_ctx, graph: *mut rbn_graph) -> c_int;
    pub fn rbn_graph_destroy(ctx: *mut rbn_ctx, graph: *mut rbn_graph) -> c_int;
    pub fn rbn_abs_sum_f32(
        ctx: *mut rbn_ctx,
        d_x: *const f32,
        n: u64,
        mode: c_int,
        use_mask: c_int,
        mask_threshold: f32,
        h_sum: *mut f32,
        h_count: *mut u64,
    ) -> c_int;
    pub fn rbn_pack_ternary(
        ctx: *mut rbn_ctx,
        d_x: *const f32,
        n: u64,
        threshold: f32,
        d_packed: *mut u8,
    ) -> c_int;
    pub fn rbn_quantize_ternary(
        ctx: *mut rbn_ctx,
        d_x: *const f32,
        n: u64,
        mode: c_int,
        d_packed: *mut u8,
        h_scale: *mut f32,
        h_threshold: *mut f32,
        h_survivors: *mut u64,
    ) -> c_int;
    pub fn rbn_dequantize_ternary(
        ctx: *mut rbn_ctx,
        d_packed: *const u8,
        n: u64,
        scale: f32,
        d_out: *mut f32,
    ) -> c_int;
    pub fn rbn_unpack_ternary_i8(
        ctx: *mut rbn_ctx,
        d_packed: *const u8,
        rows: u64,
        cols: u64,
        pitch: u64,
        d_q: *mut i8,
        d_rowsum: *mut i32,
    ) -> c_int;
    pub fn rbn_tile_weights(
        ctx: *mut rbn_ctx,
        d_packed: *const u8,
        K: u64,
        N: u64,
        d_tiled: *mut u32,
    ) -> c_int;
    pub fn rbn_act_quant_i8(
        ctx: *mut rbn_ctx,
        d_x: *const f32,
        M: u64,
        K: u64,
        d_q: *mut i8,
        d_act_scale: *mut f32,
        d_rowsum: *mut i32,
    ) -> c_int;
    pub fn rbn_act_quant_ternary(
        ctx: *mut rbn_ctx,
        d_x: *const f32,
        M: u64,
        K: u64,
        mode: c_int,
        d_q: *mut i8,
        d_act_scale: *mut f32,
        d_rowsum: *mut i32,
        h_scale: *mut f32,
        h_threshold: *mut f32,
    ) -> c_int;
    pub fn rbn_gemv_t2_i8(
        ctx: *mut rbn_ctx,
        d_q: *const i8,
        d_act_scale: *const f32,
        d_rowsum: *const i32,
        d_tiled: *const u32,
        w_scale: f32,
        M: u64,
        K: u64,
        N: u64,
        d_acc: *mut i32,
        d_out: *mut f32,
    ) -> c_int;
    pub fn rbn_gemv_t2_i8_kernel_time(
        ctx: *mut rbn_ctx,
        d_q: *const i8,
        d_act_scale: *const f32,
        d_rowsum: *const i32,
        d_tiled: *const u32,
        w_scale: f32,
        M: u64,
        K: u64,
        N: u64,
        d_acc: *mut i32,
        d_out: *mut f32,
        h_kernel_us: *mut f32,
    ) -> c_int;
    pub fn rbn_gemv_t2_i8_grouped(
        ctx: *mut rbn_ctx,
        h_problems: *const rbn_gemv_problem,
        count: u64,
        M: u64,
        K: u64,
        N: u64,
    ) -> c_int;
    pub fn rbn_gemm_t2_i8_skinny(
        ctx: *mut rbn_ctx,
        d_q: *const i8,
        d_act_scale: *const f32,
        d_rowsum: *const i32,
        d_tiled: *const u32,
        w_scale: f32,
        M: u64,
        K: u64,
        N: u64,
        d_acc: *mut i32,
        d_out: *mut f32,
    ) -> c_int;
    pub fn rbn_gemm_t2_i8_mfma(
        ctx: *mut rbn_ctx,
        d_q: *const i8,
        d_act_scale: *const f32,
        d_rowsum: *const i32,
        d_tiled: *const u32,
        w_scale: f32,
        M: u64,
        K: u64,
        N: u64,
        d_acc: *mut i32,
        d_out: *mut f32,
    ) -> c_int;
    pub fn rbn_skinny_launch_shape(M: u64, K: u64, N: u64, shape: *mut i32) -> c_int;
    pub fn rbn_gemm_t2_i8_skinny_static(
        ctx: *mut rbn_ctx,
        d_q: *const i8,
        d_act_scale: *const f32,
        d_rowsum: *const i32,
        d_tiled: *const u32,
        w_scale: f32,
        M: u64,
        K: u64,
        N: u64,
        d_acc: *mut i32,
        d_out: *mut f32,
    ) -> c_int;
    pub fn rbn_matmul_t2_i8(
        ctx: *mut rbn_ctx,
        d_q: *const i8,
        d_act_scale: *const f32,
        d_rowsum: *const i32,
        d_tiled: *const u32,
        w_scale: f32,
        M: u64,
        K: u64,
        N: u64,
        d_acc: *mut i32,
        d_out: *mut f32,
    ) -> c_int;
    pub fn rbn_matmul_kernel_choice(M: u64, K: u64, N: u64) -> c_int;
    pub fn rbn_execute_ternary_matmul(
        ctx: *mut rbn_ctx,
        h_a: *const f32,
        h_b: *const f32,
        M: u64,
        N: u64,
        K: u64,
        mode: c_int,
        h_out: *mut f32,
        h_acc: *mut i32,
    ) -> c_int;
    pub fn rbn_bitlinear_gemv_f32(
        ctx: *mut rbn_ctx,
        d_x: *const f32,
        d_gate_up: *const f32,
        d_gamma: *const f32,
        eps: f32,
        d_tiled: *const u32,
        w_scale: f32,
        K: u64,
        N: u64,
        d_residual: *const f32,
        d_out: *mut f32,
    ) -> c_int;
    pub fn rbn_embed_f32(
        ctx: *mut rbn_ctx,
        d_table: *const f32,
        d_tokens: *const i32,
        M: u64,
        H: u64,
        vocab: u64,
        d_x: *mut f32,
    ) -> c_int;
    pub fn rbn_rmsnorm_quant_i8(
        ctx: *mut rbn_ctx,
        d_x: *mut f32,
        d_delta: *const f32,
        d_gate_up: *const f32,
        d_gamma: *const f32,
        eps: f32,
        M: u64,
        H: u64,
        d_q: *mut i8,
        d_act_scale: *mut f32,
        d_rowsum: *mut i32,
    ) -> c_int;
    pub fn rbn_rope_kv_store_f16(
        ctx: *mut rbn_ctx,
        d_qkv: *mut f32,
        d_pos0: *const i32,
        M: u64,
        heads: u64,
        head_dim: u64,
        theta: f32,
        d_kcache: *mut c_void,
        d_vcache: *mut c_void,
        max_seq: u64,
    ) -> c_int;
    pub fn rbn_attention_f16kv(
        ctx: *mut rbn_ctx,
        d_qkv: *const f32,
        d_pos0: *const i32,
        M: u64,
        heads: u64,
        head_dim: u64,
        d_kcache: *const c_void,
        d_vcache: *const c_void,
        max_seq: u64,
        d_out: *mut f32,
    ) -> c_int;
    pub fn rbn_attention_decode_f16kv(
        ctx: *mut rbn_ctx,
        d_qkv: *const f32,
        d_pos: *const i32,
        heads: u64,
        head_dim: u64,
        theta: f32,
        d_kcache: *mut c_void,
        d_vcache: *mut c_void,
        max_seq: u64,
        d_out: *mut f32,
    ) -> c_int;
    pub fn rbn_swiglu_f32(ctx: *mut rbn_ctx, d_gate_up: *const f32, M: u64, F: u64, d_h: *mut f32) -> c_int;
    pub fn rbn_argmax_f32(
        ctx: *mut rbn_ctx,
        d_values: *const f32,
        n: u64,
        d_index: *mut i32,
        d_history: *mut i32,
        d_history_pos: *const i32,
        history_capacity: u64,
    ) -> c_int;
    pub fn rbn_greedy_next_f32(
        ctx: *mut rbn_ctx,
        d_logits: *const f32,
        vocab: u64,
        d_token: *mut i32,
        d_history: *mut i32,
        d_pos: *mut i32,
        history_capacity: u64,
        d_table: *const f32,
        H: u64,
        d_x: *mut f32,
    ) -> c_int;
    pub fn rbn_add_i32(ctx: *mut rbn_ctx, d_value: *mut i32, delta: i32) -> c_int;
    pub fn rbn_synth_normal_device_f32(
        ctx: *mut rbn_ctx,
        seed: u64,
        sigma: f32,
        d_out: *mut f32,
        n: u64,
    ) -> c_int;
    pub fn rbn_synth_normal_f32(seed: u64, sigma: f64, first: u64, count: u64, h_out: *mut f32);
// ---- include/ronn_bitnet_provider.h ----
    pub fn rbp_last_error() -> *const c_char;
    pub fn rbp_default_config(cfg: *mut rbp_config);
    pub fn rbp_provider_create(cfg: *const rbp_config, out: *mut *mut rbp_provider) -> c_int;
    pub fn rbp_provider_destroy(p: *mut rbp_provider) -> c_int;
    pub fn rbp_provider_id(p: *mut rbp_provider) -> c_int;
    pub fn rbp_provider_get_config(p: *mut rbp_provider, out: *mut rbp_config) -> c_int;
    pub fn rbp_provider_supports(p: *mut rbp_provider, op_type: *const c_char) -> c_int;
    pub fn rbp_provider_estimate_speedup(p: *mut rbp_provider, op_type: *const c_char) -> f32;
    pub fn rbp_provider_capability(
        p: *mut rbp_provider,
        n_ops: *mut c_int,
        performance_profile: *mut c_int,
    ) -> c_int;
    pub fn rbp_provider_has_data_type(p: *mut rbp_provider, dtype: c_int) -> c_int;
    pub fn rbp_provider_configure(
        p: *mut rbp_provider,
        memory_limit: u64,
        optimization_level: c_int,
        keys: *const *const c_char,
        values: *const *const c_char,
        n: c_int,
    ) -> c_int;
    pub fn rbp_provider_shutdown(p: *mut rbp_provider) -> c_int;
    pub fn rbp_provider_compile_subgraph(
        p: *mut rbp_provider,
        op_types: *const *const c_char,
        n_nodes: c_int,
        out: *mut *mut rbp_kernel,
    ) -> c_int;
    pub fn rbp_allocate(
        p: *mut rbp_provider,
        shape: *const u64,
        ndim: c_int,
        dtype: c_int,
        d_ptr: *mut *mut c_void,
        size: *mut u64,
        alignment: *mut u64,
    ) -> c_int;
    pub fn rbp_deallocate(p: *mut rbp_provider, d_ptr: *mut c_void, size: u64, alignment: u64) -> c_int;
    pub fn rbp_memory_info(
        p: *mut rbp_provider,
        total: *mut u64,
        allocated: *mut u64,
        peak: *mut u64,
    ) -> c_int;
    pub fn rbp_provider_memory_stats(
        p: *mut rbp_provider,
        binary_tensor_count: *mut u64,
        ternary_tensor_count: *mut u64,
        memory_saved_bytes: *mut u64,
        average_compression_ratio: *mut f32,
    ) -> c_int;
    pub fn rbp_create_ternary_matmul_kernel(
        p: *mut rbp_provider,
        m: u64,
        n: u64,
        k: u64,
        out: *mut *mut rbp_kernel,
    ) -> c_int;
    pub fn rbp_kernel_destroy(k: *mut rbp_kernel) -> c_int;
    pub fn rbp_kernel_execute(
        k: *mut rbp_kernel,
        n_inputs: c_int,
        h_data: *const *const f32,
        shapes: *const *const u64,
        ndims: *const c_int,
        dtypes: *const c_int,
        h_out: *mut f32,
        out_capacity: u64,
        out_shape: *mut u64,
    ) -> c_int;
    pub fn rbp_kernel_stats(
        k: *mut rbp_kernel,
        execution_count: *mut u64,
        average_us: *mut f64,
        min_us: *mut f64,
        max_us: *mut f64,
    ) -> c_int;
    pub fn rbp_kernel_memory_usage(
        k: *mut rbp_kernel,
        peak: *mut u64,
        current: *mut u64,
        allocations: *mut u64,
    ) -> c_int;
    pub fn rbp_quantize_ternary(
        p: *mut rbp_provider,
        h_data: *const f32,
        shape: *const u64,
        ndim: c_int,
        dtype: c_int,
        out: *mut *mut rbp_ternary,
    ) -> c_int;
    pub fn rbp_ternary_destroy(t: *mut rbp_ternary) -> c_int;
    pub fn rbp_ternary_info(
        t: *mut rbp_ternary,
        scale: *mut f32,
        threshold: *mut f32,
        element_count: *mut u64,
        memory_size: *mut u64,
        compression_ratio: *mut f32,
    ) -> c_int;
    pub fn rbp_ternary_packed(t: *mut rbp_ternary, h_out: *mut u8, capacity: u64) -> c_int;
    pub fn rbp_ternary_get_value(t: *mut rbp_ternary, index: u64) -> c_int;
    pub fn rbp_dequantize_ternary(
        p: *mut rbp_provider,
        t: *mut rbp_ternary,
        h_out: *mut f32,
        capacity: u64,
    ) -> c_int;
    pub fn rbp_ternary_from_parts(
        h_packed: *const u8,
        packed_bytes: u64,
        shape: *const u64,
        ndim: c_int,
        scale: f32,
        threshold: f32,
        out: *mut *mut rbp_ternary,
    ) -> c_int;
    pub fn rbp_ternary_shape(t: *mut rbp_ternary, shape: *mut u64, ndim: *mut c_int) -> c_int;
    pub fn rbp_ternary_save(t: *mut rbp_ternary, path: *const c_char) -> c_int;
    pub fn rbp_ternary_load(path: *const c_char, out: *mut *mut rbp_ternary) -> c_int;
    pub fn rbp_kernel_execute_prepacked(
        k: *mut rbp_kernel,
        h_a: *const f32,
        shape_a: *const u64,
        ndim_a: c_int,
        w: *mut rbp_ternary,
        h_out: *mut f32,
        out_capacity: u64,
        out_shape: *mut u64,
    ) -> c_int;
    pub fn rbp_kernel_execute_group(
        k: *mut rbp_kernel,
        n_pairs: c_int,
        h_a: *const *const f32,
        h_b: *const *const f32,
        shape_a: *const u64,
        shape_b: *const u64,
        h_out: *const *mut f32,
        out_capacity_each: u64,
        launches: *mut c_int,
    ) -> c_int;

}

/// Turns a status into `Result`, with the library's message for the calling thread.
pub fn check(rc: c_int) -> Result<(), String> {
    if rc == RBN_OK {
        return Ok(());
    }
    // SAFETY: rbn_last_error returns a NUL-terminated string owned by the library (thread-local).
    let msg = unsafe { CStr::from_ptr(rbn_last_error()) }.to_string_lossy().into_owned();
    Err(format!("{msg} (rbn status {rc})"))
}

/// The same for the provider-level calls.
pub fn check_provider(rc: c_int) -> Result<(), String> {
    if rc == RBP_OK {
        return Ok(());
    }
    // SAFETY: as above.
    let msg = unsafe { CStr::from_ptr(rbp_last_error()) }.to_string_lossy().into_owned();
    Err(msg)
}
