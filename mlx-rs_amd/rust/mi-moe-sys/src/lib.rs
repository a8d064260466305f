//! Raw declarations of `include/mi_moe.h`, one to one.  Status convention as in mlx-c: `0` is
//! success, anything else a failure whose text `mi_moe_last_error` returns (thread-local).
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};

#[repr(C)]
pub struct mi_moe_s {
    _private: [u8; 0],
}
pub type mi_moe_handle = *mut mi_moe_s;

pub const MI_MOE_SCORE_SOFTMAX_THEN_TOPK_RENORM: i32 = 0;
pub const MI_MOE_SCORE_SOFTMAX_THEN_TOPK: i32 = 1;
pub const MI_MOE_SCORE_TOPK_THEN_SOFTMAX: i32 = 2;
pub const MI_MOE_DTYPE_BF16: i32 = 0;
pub const MI_MOE_DTYPE_F16: i32 = 1;
pub const MI_MOE_DTYPE_F32: i32 = 2;
pub const MI_MOE_N_STAGES: usize = 6;
pub const MI_MOE_N_KERNEL_TIMES: usize = 8;
pub const MI_MOE_STATIC_SCRATCH_BYTES: usize = 8388608;

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct mi_moe_config {
    pub hidden: i32,
    pub n_experts: i32,
    pub top_k: i32,
    pub intermediate: i32,
    pub bits: i32,
    pub group_size: i32,
    pub score_mode: i32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct mi_moe_qmat {
    pub w: *const u32,
    pub scales: *const u16,
    pub biases: *const u16,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct mi_moe_weights {
    pub router_w: *const u16,
    pub router_bias: *const f32,
    pub gate: mi_moe_qmat,
    pub up: mi_moe_qmat,
    pub down: mi_moe_qmat,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct mi_moe_debug_out {
    pub topk_idx: *mut u32,
    pub topk_w: *mut u16,
    pub counts: *mut u32,
    pub offsets: *mut u32,
    pub perm: *mut u32,
    pub inv_perm: *mut u32,
}

pub type mi_moe_error_handler = Option<unsafe extern "C" fn(msg: *const c_char, data: *mut c_void)>;
pub type mi_moe_data_dtor = Option<unsafe extern "C" fn(data: *mut c_void)>;

extern "C" {
    pub fn mi_moe_last_error() -> *const c_char;
    pub fn mi_moe_set_error_handler(handler: mi_moe_error_handler, data: *mut c_void, dtor: mi_moe_data_dtor);

    pub fn mi_moe_create(cfg: *const mi_moe_config, weights: *const mi_moe_weights, out: *mut mi_moe_handle) -> c_int;
    pub fn mi_moe_destroy(h: mi_moe_handle) -> c_int;
    pub fn mi_moe_workspace_size(cfg: *const mi_moe_config, max_tokens: i64, bytes: *mut usize) -> c_int;
    pub fn mi_moe_forward(h: mi_moe_handle, x: *const u16, T: i64, out: *mut u16, workspace: *mut c_void, workspace_bytes: usize, dbg: *const mi_moe_debug_out, stream: *mut c_void) -> c_int;
    pub fn mi_moe_forward_static(h: mi_moe_handle, x: *const u16, T: i64, out: *mut u16, dbg: *const mi_moe_debug_out, stream: *mut c_void) -> c_int;
    pub fn mi_moe_forward_residual(h: mi_moe_handle, x: *const u16, norm_weight: *const u16, eps: f32, T: i64, out: *mut u16, workspace: *mut c_void, workspace_bytes: usize, dbg: *const mi_moe_debug_out, stream: *mut c_void) -> c_int;
    pub fn mi_moe_rms_norm(x: *const u16, weight: *const u16, eps: f32, T: i64, hidden: i32, out: *mut u16, stream: *mut c_void) -> c_int;
    pub fn mi_moe_forward_timed(h: mi_moe_handle, x: *const u16, T: i64, out: *mut u16, workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void, stage_ms: *mut f32, kernel_ms: *mut f32) -> c_int;

    pub fn mi_moe_route_workspace_size(n_experts: i32, T: i64, bytes: *mut usize) -> c_int;
    pub fn mi_moe_route(x: *const u16, router_w: *const u16, router_bias: *const f32, T: i64, hidden: i32, n_experts: i32, top_k: i32, score_mode: i32, topk_idx: *mut u32, topk_w: *mut u16, logits_out: *mut u16, workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void) -> c_int;

    pub fn mi_moe_router_logits_workspace_size(T: i64, hidden: i32, n_experts: i32, bytes: *mut usize) -> c_int;
    pub fn mi_moe_router_logits(x: *const u16, router_w: *const u16, router_bias: *const f32, T: i64, hidden: i32, n_experts: i32, logits: *mut u16, workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void) -> c_int;

    pub fn mi_moe_dispatch_workspace_size(n_experts: i32, P: i64, bytes: *mut usize) -> c_int;
    pub fn mi_moe_dispatch(expert_of_pair: *const u32, P: i64, n_experts: i32, counts: *mut u32, offsets: *mut u32, perm: *mut u32, inv_perm: *mut u32, workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void) -> c_int;

    pub fn mi_moe_gather_qmm_workspace_size(n_experts: i32, n_idx: i64, M: i32, bytes: *mut usize) -> c_int;
    pub fn mi_moe_gather_qmm(x: *const u16, w: *const u32, scales: *const u16, biases: *const u16, lhs_indices: *const u32, rhs_indices: *const u32, n_idx: i64, x_batch: i64, M: i32, N: i32, K: i32, n_experts: i32, transpose: i32, group_size: i32, bits: i32, sorted_indices: i32, y: *mut u16, workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void) -> c_int;

    pub fn mi_moe_gather_qmm_typed(x: *const c_void, w: *const u32, scales: *const c_void, biases: *const c_void, lhs_indices: *const u32, rhs_indices: *const u32, n_idx: i64, x_batch: i64, M: i32, N: i32, K: i32, n_experts: i32, transpose: i32, group_size: i32, bits: i32, sorted_indices: i32, dtype: i32, y: *mut c_void, workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void) -> c_int;

    pub fn mi_moe_quantized_matmul_workspace_size(M: i64, K: i32, bits: i32, bytes: *mut usize) -> c_int;
    pub fn mi_moe_quantized_matmul(x: *const u16, w: *const u32, scales: *const u16, biases: *const u16, M: i64, N: i32, K: i32, transpose: i32, group_size: i32, bits: i32, y: *mut u16, workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void) -> c_int;

    pub fn mi_moe_quantized_matmul_typed(x: *const c_void, w: *const u32, scales: *const c_void, biases: *const c_void, M: i64, N: i32, K: i32, transpose: i32, group_size: i32, bits: i32, dtype: i32, y: *mut c_void, workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void) -> c_int;

    pub fn mi_moe_swiglu(gate: *const u16, up: *const u16, n: i64, out: *mut u16, stream: *mut c_void) -> c_int;
    pub fn mi_moe_combine(y: *const u16, scores: *const u16, inv_perm: *const u32, T: i64, top_k: i32, hidden: i32, out: *mut u16, stream: *mut c_void) -> c_int;

    pub fn mi_moe_quantize(w: *const f32, rows: i64, cols: i64, group_size: i32, bits: i32, q: *mut u32, scales: *mut u16, biases: *mut u16, stream: *mut c_void) -> c_int;
    pub fn mi_moe_dequantize(q: *const u32, scales: *const u16, biases: *const u16, rows: i64, cols: i64, group_size: i32, bits: i32, w_hat: *mut f32, stream: *mut c_void) -> c_int;

    pub fn mi_moe_quantize_typed(w: *const f32, rows: i64, cols: i64, group_size: i32, bits: i32, dtype: i32, q: *mut u32, scales: *mut c_void, biases: *mut c_void, stream: *mut c_void) -> c_int;
    pub fn mi_moe_dequantize_typed(q: *const u32, scales: *const c_void, biases: *const c_void, rows: i64, cols: i64, group_size: i32, bits: i32, dtype: i32, w_hat: *mut f32, stream: *mut c_void) -> c_int;

    pub fn mi_moe_quantized_linear_typed(x: *const c_void, w: *const u32, scales: *const c_void, biases: *const c_void, linear_bias: *const c_void, M: i64, N: i32, K: i32, group_size: i32, bits: i32, dtype: i32, y: *mut c_void, workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void) -> c_int;
    pub fn mi_moe_dequantize_native(q: *const u32, scales: *const c_void, biases: *const c_void, rows: i64, cols: i64, group_size: i32, bits: i32, dtype: i32, w_hat: *mut c_void, stream: *mut c_void) -> c_int;

    pub fn mi_moe_debug_kernel_count() -> i32;
    pub fn mi_moe_debug_kernel_name(index: i32) -> *const c_char;
    pub fn mi_moe_debug_kernel_launches(index: i32) -> i64;
    pub fn mi_moe_debug_plan_forward(cfg: *const mi_moe_config, T: i64, out: *mut c_char, cap: usize) -> c_int;
    pub fn mi_moe_debug_plan_grouped(N: i32, K: i32, bits: i32, glu: i32, total_rows: i64, max_active: i32, max_rows_per_expert: i64, max_streamed_rows: i64, tile_lists: i32, paired_out: i32, out: *mut c_char, cap: usize) -> c_int;
    pub fn mi_moe_debug_tile_rule(cfg: *const mi_moe_config, T: i64, tiled: *mut i32, tile_min_rows: *mut i32) -> c_int;
    pub fn mi_moe_debug_side_streams_created() -> i32;

    pub fn mi_moe_stream_probe(buf: *const c_void, bytes: usize, sink: *mut u32, stream: *mut c_void) -> c_int;

    pub fn mi_moe_version() -> *const c_char;
}
