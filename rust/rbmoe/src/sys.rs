//! Raw declarations of `include/rbmoe.h`, one to one.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};

pub const RBMOE_OK: c_int = 0;
pub const RBMOE_INVALID_INPUT: c_int = 1;
pub const RBMOE_INVALID_CONFIG: c_int = 2;
pub const RBMOE_DEVICE_ERROR: c_int = 3;
pub const RBMOE_BACKEND_UNAVAILABLE: c_int = 4;
pub const RBMOE_MEMORY_BUDGET: c_int = 5;
pub const RBMOE_OUT_OF_MEMORY: c_int = 6;
pub const RBMOE_UNSUPPORTED: c_int = 7;
pub const RBMOE_NULL_POINTER: c_int = 8;

pub const RBMOE_F32: i32 = 0;
pub const RBMOE_BF16: i32 = 1;
pub const RBMOE_I8: i32 = 2;

pub const RBMOE_W_ROUTER: i32 = 0;
pub const RBMOE_W_GATE: i32 = 1;
pub const RBMOE_W_UP: i32 = 2;
pub const RBMOE_W_DOWN: i32 = 3;
pub const RBMOE_W_SHARED_GATE: i32 = 4;
pub const RBMOE_W_SHARED_UP: i32 = 5;
pub const RBMOE_W_SHARED_DOWN: i32 = 6;
pub const RBMOE_W_NORM: i32 = 7;

pub const RBMOE_OPT_FORCE_GENERIC: i32 = 0;
pub const RBMOE_OPT_EXPLICIT_GATHER: i32 = 1;
pub const RBMOE_OPT_GROUP_M: i32 = 2;
pub const RBMOE_OPT_DECODE_PATH: i32 = 3;
pub const RBMOE_OPT_DECODE_FRONT: i32 = 4;
pub const RBMOE_OPT_FUSED_ROUTER: i32 = 5;
pub const RBMOE_OPT_SIDE_STREAM: i32 = 6;
pub const RBMOE_OPT_WGRAD_MODE: i32 = 7;
pub const RBMOE_OPT_WGRAD_GENERIC: i32 = 8;
pub const RBMOE_OPT_DECODE_COMBINE_FOLD: i32 = 9;
pub const RBMOE_OPT_QUANT_RULE: i32 = 10;
pub const RBMOE_OPT_QUANTIZE_ROUTER: i32 = 11;
pub const RBMOE_OPT_DECODE_DOWN_BY_EXPERT: i32 = 12;

pub const RBMOE_NUM_STAGES: usize = 8;

#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct rbmoe_config {
    pub d_model: i32,
    pub num_experts: i32,
    pub experts_per_token: i32,
    pub d_ff: i32,
    pub shared_expert: i32,
    pub shared_d_ff: i32,
    pub aux_loss_weight: f32,
    pub router_z_loss_weight: f32,
    pub weight_dtype: i32,
    pub act_dtype: i32,
    pub max_tokens: i32,
}

#[repr(C)]
pub struct rbmoe_routing {
    pub expert_of: *mut i32,
    pub gate_of: *mut f32,
    pub counts: *mut i32,
    pub offsets: *mut i32,
    pub perm_slot: *mut i32,
    pub perm_token: *mut i32,
    pub probabilities: *mut f32,
    pub log_sum_exp: *mut f32,
}

#[repr(C)]
pub struct rbmoe_ctx {
    _private: [u8; 0],
}
#[repr(C)]
pub struct rbmoe_layer {
    _private: [u8; 0],
}

extern "C" {
    pub fn rbmoe_config_init(cfg: *mut rbmoe_config, d_model: i32, num_experts: i32, experts_per_token: i32,
                             d_ff: i32) -> c_int;
    pub fn rbmoe_validate(cfg: *const rbmoe_config, msg: *mut c_char, msg_cap: usize) -> c_int;
    pub fn rbmoe_parameter_counts(cfg: *const rbmoe_config, total: *mut u64, active: *mut u64) -> c_int;
    pub fn rbmoe_ctx_create(device: i32, budget_mib: usize, out: *mut *mut rbmoe_ctx) -> c_int;
    pub fn rbmoe_ctx_destroy(ctx: *mut rbmoe_ctx);
    pub fn rbmoe_ctx_set_stream(ctx: *mut rbmoe_ctx, hip_stream: *mut c_void) -> c_int;
    pub fn rbmoe_synchronize(ctx: *mut rbmoe_ctx) -> c_int;
    pub fn rbmoe_last_error(ctx: *const rbmoe_ctx) -> *const c_char;
    pub fn rbmoe_last_global_error() -> *const c_char;
    pub fn rbmoe_layer_create(ctx: *mut rbmoe_ctx, cfg: *const rbmoe_config, out: *mut *mut rbmoe_layer) -> c_int;
    pub fn rbmoe_layer_destroy(layer: *mut rbmoe_layer);
    pub fn rbmoe_layer_set_option(layer: *mut rbmoe_layer, option: i32, value: i32) -> c_int;
    pub fn rbmoe_set_weight(layer: *mut rbmoe_layer, which: i32, expert: i32, data: *const c_void, dtype: i32,
                            scales: *const f32, rows: i32, cols: i32) -> c_int;
    pub fn rbmoe_forward(layer: *mut rbmoe_layer, x: *const c_void, tokens: i32, cols: i32, valid: *const u8,
                         router_bias: *const f32, residual: *const c_void, out: *mut c_void) -> c_int;
    // rbmoe_forward with every intermediate buffer in the library's static device array (no allocation)
    pub fn rbmoe_forward_static(layer: *mut rbmoe_layer, x: *const c_void, tokens: i32, cols: i32, valid: *const u8,
                                router_bias: *const f32, residual: *const c_void, out: *mut c_void) -> c_int;
    pub fn rbmoe_forward_host(layer: *mut rbmoe_layer, x: *const c_void, tokens: i32, cols: i32, valid: *const u8,
                              router_bias: *const f32, residual: *const c_void, out: *mut c_void) -> c_int;
    pub fn rbmoe_forward_timed(layer: *mut rbmoe_layer, x: *const c_void, tokens: i32, cols: i32, valid: *const u8,
                               router_bias: *const f32, residual: *const c_void, out: *mut c_void,
                               ms: *mut f32) -> c_int;
    pub fn rbmoe_forward_kernel_times(layer: *mut rbmoe_layer, x: *const c_void, tokens: i32, cols: i32, valid: *const u8,
                               router_bias: *const f32, residual: *const c_void, out: *mut c_void,
                               ms: *mut f32) -> c_int;
    pub fn rbmoe_get_losses(layer: *mut rbmoe_layer, aux_loss: *mut f32, z_loss: *mut f32) -> c_int;
    pub fn rbmoe_get_routing(layer: *mut rbmoe_layer, routing: *mut rbmoe_routing) -> c_int;
    pub fn rbmoe_get_expert_rows(layer: *mut rbmoe_layer, hidden: *mut f32, expert_out: *mut f32) -> c_int;
    // the block's steps either side of the layer (src/transformer_block.rs:216-222)
    pub fn rbmoe_set_feed_forward_norm(layer: *mut rbmoe_layer, weight: *const f32, cols: i32, eps: f32) -> c_int;
    pub fn rbmoe_forward_block(layer: *mut rbmoe_layer, x: *const c_void, tokens: i32, cols: i32, valid: *const u8,
                               router_bias: *const f32, out: *mut c_void) -> c_int;
    pub fn rbmoe_forward_block_host(layer: *mut rbmoe_layer, x: *const c_void, tokens: i32, cols: i32,
                                    valid: *const u8, router_bias: *const f32, out: *mut c_void) -> c_int;
    // backward pass (MoeLayer::backward, src/moe.rs:348-489)
    pub fn rbmoe_layer_enable_training(layer: *mut rbmoe_layer) -> c_int;
    pub fn rbmoe_backward(layer: *mut rbmoe_layer, grad_output: *const c_void, tokens: i32, cols: i32,
                          grad_input: *mut c_void) -> c_int;
    pub fn rbmoe_backward_host(layer: *mut rbmoe_layer, grad_output: *const c_void, tokens: i32, cols: i32,
                               grad_input: *mut c_void) -> c_int;
    pub fn rbmoe_backward_block(layer: *mut rbmoe_layer, grad_output: *const c_void, tokens: i32, cols: i32,
                                grad_input: *mut c_void) -> c_int;
    pub fn rbmoe_backward_block_host(layer: *mut rbmoe_layer, grad_output: *const c_void, tokens: i32, cols: i32,
                                     grad_input: *mut c_void) -> c_int;
    pub fn rbmoe_zero_grads(layer: *mut rbmoe_layer) -> c_int;
    pub fn rbmoe_get_weight_grad(layer: *mut rbmoe_layer, which: i32, expert: i32, host: *mut f32, rows: i32,
                                 cols: i32) -> c_int;
    pub fn rbmoe_expert_kernel_name(layer: *const rbmoe_layer) -> *const c_char;
    pub fn rbmoe_device_alloc(ctx: *mut rbmoe_ctx, bytes: usize, out: *mut *mut c_void) -> c_int;
    pub fn rbmoe_device_free(ctx: *mut rbmoe_ctx, ptr: *mut c_void) -> c_int;
    pub fn rbmoe_copy_to_device(ctx: *mut rbmoe_ctx, dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn rbmoe_copy_to_host(ctx: *mut rbmoe_ctx, dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn rbmoe_copy_device(ctx: *mut rbmoe_ctx, dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    // calibration: a multiply-only kernel and a plain read, for roofline figures to be read against
    pub fn rbmoe_replay_stage(layer: *mut rbmoe_layer, stage: i32, launches: i32, ms_per_launch: *mut f32) -> c_int;
    pub fn rbmoe_version() -> *const c_char;
}
