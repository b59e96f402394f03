//! `extern "C"` declarations of include/larql_hip.h — only what the trait impls call.
//! Return codes: 0 = Some, 1 (unsupported) / 2 (refused shape) = None, negative = device error (None; the text is
//! in `larql_hip_last_error`).
#![allow(non_camel_case_types, dead_code)]

use std::os::raw::{c_char, c_int};

#[repr(C)]
pub struct Ctx {
    _private: [u8; 0],
}

#[repr(C)]
#[derive(Clone, Copy, Default)]
pub struct Clock {
    pub submissions: u64,
    pub commit_to_done_nanos: u64,
    pub gpu_nanos: u64,
}

#[repr(C)]
pub struct MoeLayer {
    _private: [u8; 0],
}

/// `larql_hip_moe_layer_weights`: `larql_compute::MoeLayerWeights` as plain pointers.
#[repr(C)]
pub struct MoeLayerWeights {
    pub num_experts: usize,
    pub top_k: usize,
    pub hidden: usize,
    pub intermediate_size: usize,
    pub expert_data_format: c_int,
    pub fused_row_layout: c_int,
    pub expert_scales: c_int,
    pub experts_gate_up: *const *const u8,
    pub experts_gate_up_len: *const usize,
    pub experts_down: *const *const u8,
    pub experts_down_len: *const usize,
    pub scales_gate_up: *const *const u8,
    pub scales_gate_up_len: *const usize,
    pub scales_down: *const *const u8,
    pub scales_down_len: *const usize,
    pub router_proj: *const f32,
    pub router_bias: *const f32,
    pub experts_gate_up_bias: *const f32,
    pub experts_down_bias: *const f32,
    pub router_per_expert_scale: *const f32,
    pub renormalized_softmax: c_int,
    pub per_expert_scale: c_int,
    pub glu_limit: f32,
    pub glu_alpha: f32,
    pub gate_rule: c_int,
}

pub const MOE_SCALES_INLINE: c_int = 0;
pub const MOE_SCALES_PAIRED: c_int = 1;
pub const MOE_ROWS_CONTIGUOUS_HALVES: c_int = 0;
pub const MOE_ROWS_INTERLEAVED: c_int = 1;
pub const MOE_GATE_CLAMPED_GLU: c_int = 0;
pub const MOE_GATE_GELU_TANH: c_int = 1;
pub const MOE_GATE_SILU: c_int = 2;
pub const MOE_GATE_SITU_GLU: c_int = 3;
pub const MOE_GATE_CLAMPED_GELU_TANH: c_int = 4;
pub const MOE_GATE_CLAMPED_SILU: c_int = 5;

pub const OK: c_int = 0;

// QuantFormat discriminants as the library numbers them (the order of larql_compute::QuantFormat)
pub const FMT_Q4_0: c_int = 0;
pub const FMT_Q4_K: c_int = 1;
pub const FMT_Q4_KF: c_int = 2;
pub const FMT_Q5_K: c_int = 3;
pub const FMT_Q6_K: c_int = 4;
pub const FMT_Q8_0: c_int = 5;
pub const FMT_BF16: c_int = 6;
pub const FMT_F16: c_int = 7;
pub const FMT_F32: c_int = 8;
pub const FMT_I2S: c_int = 9;
pub const FMT_MXFP4: c_int = 10;

pub const CAP_F32_GEMV: c_int = 0;
pub const CAP_F16_GEMV: c_int = 1;
pub const CAP_QUANT_MATVEC: c_int = 2;

extern "C" {
    pub fn larql_hip_create(out: *mut *mut Ctx, device: c_int) -> c_int;
    pub fn larql_hip_destroy(ctx: *mut Ctx);
    pub fn larql_hip_name(ctx: *const Ctx) -> *const c_char;
    pub fn larql_hip_device_info(ctx: *const Ctx) -> *const c_char;
    pub fn larql_hip_last_error(ctx: *const Ctx) -> *const c_char;
    pub fn larql_hip_supports_quant(ctx: *const Ctx, format: c_int) -> c_int;
    pub fn larql_hip_supports(ctx: *const Ctx, capability: c_int) -> c_int;
    pub fn larql_hip_register_weight_region(ctx: *mut Ctx, region: *const u8, len: usize) -> c_int;
    pub fn larql_hip_seal_weight_regions(ctx: *mut Ctx) -> c_int;
    pub fn larql_hip_clear_weight_regions(ctx: *mut Ctx) -> c_int;
    pub fn larql_hip_get_submission_clock(ctx: *mut Ctx, out: *mut Clock) -> c_int;

    pub fn larql_hip_q4k_matvec(ctx: *mut Ctx, w: *const u8, w_len: usize, x: *const f32, x_len: usize, rows: usize,
                                hidden: usize, out: *mut f32, out_len: usize) -> c_int;
    pub fn larql_hip_q6k_matvec(ctx: *mut Ctx, w: *const u8, w_len: usize, x: *const f32, x_len: usize, rows: usize,
                                hidden: usize, out: *mut f32) -> c_int;
    pub fn larql_hip_q4k_dual_matvec(ctx: *mut Ctx, a: *const u8, a_len: usize, b: *const u8, b_len: usize, x: *const f32,
                                     x_len: usize, rows: usize, hidden: usize, out_a: *mut f32, out_b: *mut f32,
                                     out_len: usize) -> c_int;
    pub fn larql_hip_q4k_matmul(ctx: *mut Ctx, w: *const u8, w_len: usize, x: *const f32, x_len: usize, rows: usize,
                                hidden: usize, seq: usize, out: *mut f32, out_len: usize) -> c_int;
    pub fn larql_hip_q4k_matvec_topk(ctx: *mut Ctx, w: *const u8, w_len: usize, x: *const f32, x_len: usize, rows: usize,
                                     hidden: usize, top_k: usize, idx: *mut u32, score: *mut f32, n_out: *mut usize) -> c_int;
    pub fn larql_hip_q4_matvec(ctx: *mut Ctx, w: *const u8, w_len: usize, q8: *const i8, q8_len: usize, scales: *const f32,
                               n_scales: usize, rows: usize, hidden: usize, out: *mut f32) -> c_int;
    pub fn larql_hip_quant_matvec(ctx: *mut Ctx, format: c_int, w: *const u8, w_len: usize, x: *const f32, x_len: usize,
                                  rows: usize, hidden: usize, out: *mut f32) -> c_int;
    pub fn larql_hip_quant_matvec_q8_input(ctx: *mut Ctx, format: c_int, w: *const u8, w_len: usize, q8: *const i8,
                                           q8_len: usize, scales: *const f32, n_scales: usize, rows: usize, hidden: usize,
                                           out: *mut f32) -> c_int;
    pub fn larql_hip_q8_0_gemv(ctx: *mut Ctx, blocks: *const u8, blocks_len: usize, x: *const f32, x_len: usize, n: usize,
                               k: usize, out: *mut f32) -> c_int;
    pub fn larql_hip_q8_0_gemv_topk(ctx: *mut Ctx, blocks: *const u8, blocks_len: usize, x: *const f32, x_len: usize,
                                    n: usize, k: usize, top_k: usize, idx: *mut u32, score: *mut f32, n_out: *mut usize) -> c_int;

    pub fn larql_hip_f32_gemv(ctx: *mut Ctx, w: *const f32, w_len: usize, x: *const f32, x_len: usize, n: usize, k: usize,
                              out: *mut f32, force: c_int) -> c_int;
    pub fn larql_hip_f16_gemv(ctx: *mut Ctx, w: *const u8, w_len: usize, x: *const f32, x_len: usize, n: usize, k: usize,
                              out: *mut f32, force: c_int) -> c_int;
    pub fn larql_hip_bf16_gemv(ctx: *mut Ctx, w: *const u8, w_len: usize, x: *const f32, x_len: usize, n: usize, k: usize,
                               out: *mut f32, force: c_int) -> c_int;
    pub fn larql_hip_f16_gemv_multi(ctx: *mut Ctx, n_mats: usize, w: *const *const u8, w_len: *const usize, n: *const usize,
                                    k: *const usize, x: *const f32, x_len: usize, out: *const *mut f32) -> c_int;
    pub fn larql_hip_bf16_gemv_multi(ctx: *mut Ctx, n_mats: usize, w: *const *const u8, w_len: *const usize, n: *const usize,
                                     k: *const usize, x: *const f32, x_len: usize, out: *const *mut f32) -> c_int;
    pub fn larql_hip_mxfp4_gemv(ctx: *mut Ctx, packed: *const u8, packed_len: usize, scales: *const u8, scales_len: usize,
                                x: *const f32, x_len: usize, n: usize, k: usize, out: *mut f32) -> c_int;
    pub fn larql_hip_mxfp4_gemv_multi(ctx: *mut Ctx, n_mats: usize, packed: *const *const u8, packed_len: *const usize,
                                      scales: *const *const u8, scales_len: *const usize, n: *const usize, k: *const usize,
                                      x: *const f32, x_len: usize, out: *const *mut f32) -> c_int;

    pub fn larql_hip_gate_knn(ctx: *mut Ctx, format: c_int, gate: *const u8, gate_len: usize, x: *const f32, batch: usize,
                              n_features: usize, hidden: usize, top_k: usize, idx: *mut u32, score: *mut f32,
                              n_out: *mut usize) -> c_int;
    pub fn larql_hip_moe_layer_create(ctx: *mut Ctx, weights: *const MoeLayerWeights, out: *mut *mut MoeLayer) -> c_int;
    pub fn larql_hip_moe_layer_destroy(ctx: *mut Ctx, layer: *mut MoeLayer);
    pub fn larql_hip_moe_layer_forward(ctx: *mut Ctx, layer: *mut MoeLayer, router_in: *const f32, x: *const f32, tokens: usize,
                                       out: *mut f32, experts_out: *mut u32, weights_out: *mut f32) -> c_int;

    pub fn larql_hip_gate_scores(ctx: *mut Ctx, format: c_int, gate: *const u8, gate_len: usize, x: *const f32, batch: usize,
                                 n_features: usize, hidden: usize, scores: *mut f32) -> c_int;
}
