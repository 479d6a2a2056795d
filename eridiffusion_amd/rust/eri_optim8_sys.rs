//! Raw `extern "C"` declarations of include/eri_optim8.h and include/eri_adam8bit.h.
//! This is the whole FFI surface: plain pointers, sizes and ints; no cudarc, no CUDA types.
//! It takes the place of the reference's only in-tree Rust<->C seam
//! (crates/core/src/tensor_narrow.rs:7-40, crates/core/src/cuda/utils_pinned.rs).
#![allow(non_camel_case_types)]
use core::ffi::{c_char, c_int, c_void};

pub const ERI_DTYPE_F32: i32 = 0; // crates/core/src/cuda/dtype_tag.rs:3-19
pub const ERI_DTYPE_F16: i32 = 1;
pub const ERI_DTYPE_BF16: i32 = 2;
pub const ERI_DTYPE_I32: i32 = 3;
pub const ERI_ADAM8_MODE_ERI: i32 = 0;
pub const ERI_ADAM8_MODE_L2: i32 = 1;
pub const ERI_ADAM8_MODE_BNB: i32 = 2;
pub const ERI_ADAM8_FLAG_GRAD_SCALE: u32 = 1;
pub const ERI_ADAM8_FLAG_EXACT_PARAM: u32 = 2;
pub const ERI_ADAM8_FLAG_BSEARCH: u32 = 4;
pub const ERI_ADAM8_FLAG_NO_PIPELINE: u32 = 8;
pub const ERI_ADAM8_FLAG_CLIP_FROM_TABLE: u32 = 16;
pub const ERI_ADAM8_FLAG_ONE_WAVE: u32 = 32;
pub const ERI_ADAM8_FLAG_EMA: u32 = 64;

#[repr(C)]
#[derive(Clone, Copy, Default)]
pub struct EriAdam8Hyper {
    pub beta1: f32, pub beta2: f32, pub omb1: f32, pub omb2: f32, pub eps: f32, pub weight_decay: f32,
    pub step_size: f32, pub bc1: f32, pub bc2: f32, pub grad_scale: f32, pub mode: i32, pub flags: u32,
    pub ema_decay: f32, pub reserved: u32,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct EriAdam8Tensor {
    pub p: *mut c_void, pub g: *const c_void, pub m: *mut u8, pub v: *mut u8,
    pub absmax_m: *mut f32, pub absmax_v: *mut f32,
    pub numel: u64, pub block_start: u64, pub dtype_tag: i32, pub grad_scale: f32,
    pub p_src: *const c_void, pub grad_f32: i32, pub reserved: i32, pub ema_shadow: *mut c_void,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct EriAdam8bitConfig {
    pub lr: f64, pub beta1: f64, pub beta2: f64, pub eps: f64, pub weight_decay: f64,
    pub amsgrad: i32, pub block_wise: i32, pub percentile_clipping: u64,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct EriAdamW32Tensor { pub p: *mut c_void, pub g: *const c_void, pub m: *mut f32, pub v: *mut f32, pub master: *mut f32, pub numel: u64, pub dtype_tag: i32, pub grad_scale: f32 }
#[repr(C)]
#[derive(Clone, Copy)]
pub struct EriAdamW32Hyper { pub lr: f32, pub beta1: f32, pub beta2: f32, pub eps: f32, pub weight_decay: f32 }
#[repr(C)]
#[derive(Clone, Copy)]
pub struct EriEmaTensor { pub shadow: *mut c_void, pub p: *const c_void, pub numel: u64, pub dtype_tag: i32, pub reserved: i32 }

#[repr(C)]
#[derive(Clone, Copy)]
pub struct EriOptimizerMemoryReport { pub num_params: u64, pub param_memory_gb: f64, pub state_memory_gb: f64, pub total_memory_gb: f64,
    pub memory_reduction_percent: f64, pub has_reduction: i32, pub description: [c_char; 44] }

pub enum EriEmaModel {}
pub enum EriAdam8Table {}
pub enum EriHipPool {}
pub enum EriParameter {}
pub enum EriAdam8bit {}
pub enum EriAdam8bitFn {}

extern "C" {
    pub fn eri_last_error() -> *const c_char;
    pub fn eri_set_last_error(message: *const c_char);
    // device storage
    pub fn eri_hip_device_count(count: *mut c_int) -> c_int;
    pub fn eri_hip_set_device(device: c_int) -> c_int;
    pub fn eri_hip_get_device(device: *mut c_int) -> c_int;
    pub fn eri_hip_malloc_zeroed(device: c_int, bytes: usize, out: *mut *mut c_void) -> c_int;
    pub fn eri_hip_free(ptr: *mut c_void) -> c_int;
    pub fn eri_hip_host_alloc(bytes: usize) -> *mut c_void;
    pub fn eri_hip_host_free(ptr: *mut c_void) -> c_int;
    pub fn eri_hip_memcpy_async(dst: *mut c_void, src: *const c_void, bytes: usize, kind: c_int, stream: *mut c_void) -> c_int;
    pub fn eri_hip_memset_async(dst: *mut c_void, value: c_int, bytes: usize, stream: *mut c_void) -> c_int;
    pub fn eri_hip_stream_create(stream: *mut *mut c_void) -> c_int;
    pub fn eri_hip_stream_sync(stream: *mut c_void) -> c_int;
    pub fn eri_hip_stream_destroy(stream: *mut c_void) -> c_int;
    pub fn eri_hip_mem_info(free_bytes: *mut usize, total_bytes: *mut usize) -> c_int;
    /// 0 = memory the runtime never allocated, 1 = pinned host, 2 = device, 3 = managed
    pub fn eri_hip_pointer_kind(p: *const c_void, kind: *mut c_int) -> c_int;
    pub fn eri_hip_pool_create(device: c_int, bytes: usize, lanes: u32, out: *mut *mut EriHipPool) -> c_int;
    pub fn eri_hip_pool_alloc_zeroed(pool: *mut EriHipPool, lane: u32, bytes: usize, out: *mut *mut c_void) -> c_int;
    pub fn eri_hip_pool_alloc_zeroed_async(pool: *mut EriHipPool, lane: u32, bytes: usize, stream: *mut c_void, out: *mut *mut c_void) -> c_int;
    pub fn eri_hip_pool_retain(pool: *mut EriHipPool) -> c_int;
    pub fn eri_hip_pool_unretain(pool: *mut EriHipPool) -> c_int;
    pub fn eri_hip_pool_release(pool: *mut EriHipPool, ptr: *mut c_void, bytes: usize) -> c_int;
    pub fn eri_hip_pool_info(pool: *const EriHipPool, lanes: *mut u32, lane_bytes: *mut usize) -> c_int;
    pub fn eri_hip_pool_lane_used(pool: *const EriHipPool, lane: u32, used_bytes: *mut usize) -> c_int;
    pub fn eri_hip_pool_reset(pool: *mut EriHipPool) -> c_int;
    pub fn eri_hip_pool_destroy(pool: *mut EriHipPool) -> c_int;
    // the step
    pub fn eri_adam8_init() -> c_int;
    pub fn eri_adam8_get_maps(signed256: *mut f32, unsigned256: *mut f32) -> c_int;
    pub fn eri_adam8_table_image(out: *mut c_void, cap: usize, bytes: *mut usize, offsets: *mut u32) -> c_int;
    pub fn eri_adam8_hyper_pack(lr: f64, beta1: f64, beta2: f64, eps: f64, weight_decay: f64, step: u64, mode: c_int, flags: u32, out: *mut EriAdam8Hyper) -> c_int;
    pub fn eri_adam8_state_init(m: *mut u8, v: *mut u8, absmax_m: *mut f32, absmax_v: *mut f32, numel: u64, stream: *mut c_void) -> c_int;
    pub fn eri_adam8_table_create(rows: *const EriAdam8Tensor, n: u32, stream: *mut c_void, out: *mut *mut EriAdam8Table) -> c_int;
    pub fn eri_adam8_table_update(table: *mut EriAdam8Table, rows: *const EriAdam8Tensor, n: u32, stream: *mut c_void) -> c_int;
    pub fn eri_adam8_table_destroy(table: *mut EriAdam8Table) -> c_int;
    pub fn eri_adam8_table_info(table: *const EriAdam8Table, total_numel: *mut u64, total_blocks: *mut u64) -> c_int;
    pub fn eri_adam8_step_table(table: *mut EriAdam8Table, hyper: *const EriAdam8Hyper, stream: *mut c_void) -> c_int;
    pub fn eri_adam8_grad_norm(table: *mut EriAdam8Table, max_norm: f32, denom_eps: f32, stream: *mut c_void) -> c_int;
    pub fn eri_adam8_grad_table_create(rows: *const EriAdam8Tensor, n: u32, stream: *mut c_void, out: *mut *mut EriAdam8Table) -> c_int;
    pub fn eri_adam8_grad_norm_joint(table: *mut EriAdam8Table, also: *mut EriAdam8Table, max_norm: f32, denom_eps: f32, stream: *mut c_void) -> c_int;
    pub fn eri_adam8_grad_norm_scale_ptr(table: *const EriAdam8Table, dev_scale: *mut *const f32) -> c_int;
    pub fn eri_adam8_grad_norm_static(table: *mut EriAdam8Table, max_norm: f32, denom_eps: f32, result: *mut c_void, stream: *mut c_void) -> c_int;
    pub fn eri_adam8_grad_norm_read(table: *mut EriAdam8Table, norm: *mut f32, scale: *mut f32, stream: *mut c_void) -> c_int;
    pub fn eri_adam8_grad_nonfinite_read(table: *mut EriAdam8Table, count: *mut u64, stream: *mut c_void) -> c_int;
    pub fn eri_adam8_traffic_probe(table: *mut EriAdam8Table, stream: *mut c_void) -> c_int;
    pub fn eri_adam8_quant_error(table: *mut EriAdam8Table, hyper: *const EriAdam8Hyper, stream: *mut c_void) -> c_int;
    pub fn eri_adam8_quant_error_read(table: *mut EriAdam8Table, m_error: *mut f32, v_error: *mut f32, stream: *mut c_void) -> c_int;
    pub fn eri_adam8_step_multi(rows: *const EriAdam8Tensor, n: u32, hyper: *const EriAdam8Hyper, stream: *mut c_void) -> c_int;
    pub fn eri_adam8_dequantize(codes: *const u8, absmax: *const f32, signed_map: c_int, numel: u64, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn eri_adam8_quantize(x: *const f32, signed_map: c_int, numel: u64, codes: *mut u8, absmax: *mut f32, stream: *mut c_void) -> c_int;
    // 32-bit sibling and EMA sweep
    pub fn eri_adamw32_step_multi(rows: *const EriAdamW32Tensor, n: u32, hyper: *const EriAdamW32Hyper, stream: *mut c_void) -> c_int;
    pub fn eri_adamw32_step_multi_scaled(rows: *const EriAdamW32Tensor, n: u32, hyper: *const EriAdamW32Hyper, grad_scale: f32, dev_scale: *const f32, stream: *mut c_void) -> c_int;
    pub fn eri_ema_update_multi(rows: *const EriEmaTensor, n: u32, decay: f32, stream: *mut c_void) -> c_int;
    // optimizer objects
    pub fn eri_param_create(data: *mut c_void, numel: u64, dtype_tag: c_int, out: *mut *mut EriParameter) -> c_int;
    pub fn eri_param_set_grad(param: *mut EriParameter, grad: *const c_void) -> c_int;
    pub fn eri_param_set_grad_typed(param: *mut EriParameter, grad: *const c_void, grad_dtype_tag: c_int) -> c_int;
    pub fn eri_param_set_data(param: *mut EriParameter, data: *mut c_void) -> c_int;
    pub fn eri_param_retain(param: *mut EriParameter) -> c_int;
    pub fn eri_param_release(param: *mut EriParameter) -> c_int;
    pub fn eri_adam8bit_config_default(cfg: *mut EriAdam8bitConfig);
    pub fn eri_adam8bit_new(params: *const *mut EriParameter, n: u32, cfg: *const EriAdam8bitConfig, stream: *mut c_void, out: *mut *mut EriAdam8bit) -> c_int;
    pub fn eri_adam8bit_destroy(opt: *mut EriAdam8bit) -> c_int;
    pub fn eri_adam8bit_step(opt: *mut EriAdam8bit, skipped: *mut u32) -> c_int;
    pub fn eri_adam8bit_zero_grad(opt: *mut EriAdam8bit) -> c_int;
    pub fn eri_adam8bit_current_lr(opt: *const EriAdam8bit) -> f64;
    pub fn eri_adam8bit_set_learning_rate(opt: *mut EriAdam8bit, lr: f64) -> c_int;
    pub fn eri_adam8bit_quantized_memory_usage(opt: *const EriAdam8bit) -> u64;
    pub fn eri_adam8bit_get_step(opt: *const EriAdam8bit) -> u64;
    pub fn eri_adam8bit_set_grad_scale(opt: *mut EriAdam8bit, scale: f32) -> c_int;
    pub fn eri_adam8bit_set_param_grad_scale(opt: *mut EriAdam8bit, index: u32, scale: f32) -> c_int;
    pub fn eri_adam8bit_attach_ema(opt: *mut EriAdam8bit, ema: *mut EriEmaModel, names: *const *const c_char, n: u32) -> c_int;
    pub fn eri_adam8bit_set_min_8bit_size(opt: *mut EriAdam8bit, numel: u64) -> c_int;
    pub fn eri_adam8bit_set_state_pool(opt: *mut EriAdam8bit, pool: *mut EriHipPool, lane: u32) -> c_int;
    pub fn eri_adam8bit_state32_ptrs(opt: *const EriAdam8bit, index: u32, m: *mut *mut f32, v: *mut *mut f32) -> c_int;
    pub fn eri_adam8bit_set_max_grad_norm(opt: *mut EriAdam8bit, max_norm: f32, denom_eps: f32) -> c_int;
    pub fn eri_ema_new(decay: f32, use_bias_correction: c_int, power: f32, stream: *mut c_void, out: *mut *mut EriEmaModel) -> c_int;
    pub fn eri_ema_destroy(ema: *mut EriEmaModel) -> c_int;
    pub fn eri_ema_init_from_params(ema: *mut EriEmaModel, names: *const *const c_char, params: *const *mut EriParameter, n: u32) -> c_int;
    pub fn eri_ema_update(ema: *mut EriEmaModel, names: *const *const c_char, params: *const *mut EriParameter, n: u32) -> c_int;
    pub fn eri_ema_copy_to(ema: *mut EriEmaModel, names: *const *const c_char, params: *const *mut EriParameter, n: u32) -> c_int;
    pub fn eri_ema_step(ema: *const EriEmaModel) -> u64;
    pub fn eri_ema_set_step(ema: *mut EriEmaModel, step: u64) -> c_int;
    pub fn eri_ema_current_decay(ema: *const EriEmaModel) -> f32;
    pub fn eri_ema_num_shadows(ema: *const EriEmaModel) -> u32;
    pub fn eri_ema_shadow(ema: *const EriEmaModel, name: *const c_char, data: *mut *mut c_void, numel: *mut u64, dtype_tag: *mut c_int) -> c_int;
    pub fn eri_analyze_optimizer_memory(num_params: u64, precision: *const c_char, out: *mut EriOptimizerMemoryReport) -> c_int;
    pub fn eri_ema_decay_from_half_life(half_life_steps: u64) -> f32;
    pub fn eri_ema_decay_from_window(window_size: u64) -> f32;
    pub fn eri_ema_effective_decay(decay: f32, step: u64, power: f32, use_bias_correction: c_int) -> f32;
    pub fn eri_adam8bit_set_mode(opt: *mut EriAdam8bit, mode: c_int) -> c_int;
    pub fn eri_adam8bit_last_grad_norm(opt: *mut EriAdam8bit, norm: *mut f32, scale: *mut f32) -> c_int;
    pub fn eri_adam8bit_last_nonfinite_grads(opt: *mut EriAdam8bit, count: *mut u64) -> c_int;
    pub fn eri_adam8bit_track_quantization_error(opt: *mut EriAdam8bit, enabled: c_int) -> c_int;
    pub fn eri_adam8bit_quantization_stats(opt: *mut EriAdam8bit, m_error: *mut f32, v_error: *mut f32) -> c_int;
    pub fn eri_adam8bit_set_flags(opt: *mut EriAdam8bit, flags: u32) -> c_int;
    pub fn eri_adam8bit_save_state(opt: *mut EriAdam8bit, path: *const c_char) -> c_int;
    pub fn eri_adam8bit_load_state(opt: *mut EriAdam8bit, path: *const c_char) -> c_int;
    pub fn eri_adam8bit_load_legacy_state(opt: *mut EriAdam8bit, path: *const c_char) -> c_int;
    pub fn eri_adam8bit_state_ptrs(opt: *const EriAdam8bit, index: u32, m: *mut *mut u8, v: *mut *mut u8, absmax_m: *mut *mut f32, absmax_v: *mut *mut f32) -> c_int;
    pub fn eri_adam8bit_fn_with_params(lr: f64, beta1: f64, beta2: f64, eps: f64, weight_decay: f64, stream: *mut c_void, out: *mut *mut EriAdam8bitFn) -> c_int;
    pub fn eri_adam8bit_fn_destroy(opt: *mut EriAdam8bitFn) -> c_int;
    pub fn eri_adam8bit_fn_update(opt: *mut EriAdam8bitFn, name: *const c_char, param: *const c_void, grad: *const c_void, numel: u64, dtype_tag: c_int, grad_dtype_tag: c_int, out: *mut c_void) -> c_int;
    pub fn eri_adam8bit_fn_set_batching(opt: *mut EriAdam8bitFn, enabled: c_int) -> c_int;
    pub fn eri_adam8bit_fn_set_state_pool(opt: *mut EriAdam8bitFn, pool: *mut EriHipPool, lane: u32) -> c_int;
    pub fn eri_adam8bit_fn_flush(opt: *mut EriAdam8bitFn) -> c_int;
    pub fn eri_adam8bit_fn_update_many(opt: *mut EriAdam8bitFn, names: *const *const c_char, params: *const *const c_void, grads: *const *const c_void, numels: *const u64, dtype_tags: *const i32, grad_dtype_tags: *const i32, outs: *const *mut c_void, n: u32) -> c_int;
    pub fn eri_adam8bit_fn_step(opt: *mut EriAdam8bitFn) -> c_int;
    pub fn eri_adam8bit_fn_set_lr(opt: *mut EriAdam8bitFn, lr: f32) -> c_int;
    pub fn eri_adam8bit_fn_get_step(opt: *const EriAdam8bitFn) -> u64;
    pub fn eri_adam8bit_fn_table_stats(opt: *const EriAdam8bitFn, flushes: *mut u64, uploads: *mut u64) -> c_int;
    pub fn eri_adam8bit_fn_memory_stats(opt: *const EriAdam8bitFn, num_params: *mut u64, bytes: *mut u64) -> c_int;
    pub fn eri_adam8bit_fn_state_numel(opt: *const EriAdam8bitFn, name: *const c_char, numel: *mut u64) -> c_int;
    pub fn eri_adam8bit_fn_get_state_fp32(opt: *mut EriAdam8bitFn, name: *const c_char, m_out: *mut f32, v_out: *mut f32) -> c_int;
    pub fn eri_adam8bit_fn_load_state_fp32(opt: *mut EriAdam8bitFn, name: *const c_char, m: *const f32, v: *const f32, numel: u64) -> c_int;
}
