//! Drop-in for `src/trainers/adam8bit_enhanced.rs` and `src/trainers/adam8bit.rs`: the same public
//! items and signatures, every method forwarding to the C ABI in `eri_optim8_sys`.
//!
//! Source text only (no Rust toolchain where this repository is built).  It assumes what the
//! reference already uses from flame-core: `Parameter::{tensor, grad}`, `Tensor::{dtype, shape,
//! device, cuda_ptr, cuda_ptr_mut}` and `device().cuda_stream_raw_ptr()`
//! (crates/core/src/tensor_narrow.rs:197-201).
use std::collections::HashMap;
use std::ffi::{CStr, CString};
use std::os::raw::c_void;
use std::path::Path;

use flame_core::device::CudaStreamRawPtrExt;
use flame_core::{DType, Error, Parameter, Result, Tensor};

use crate::eri_optim8_sys as sys;

fn check(code: i32, what: &str) -> Result<()> {
    if code == 0 {
        return Ok(());
    }
    let msg = unsafe { CStr::from_ptr(sys::eri_last_error()) }.to_string_lossy().into_owned();
    // same shape as tensor_narrow.rs:221-227: "... failed with code N"
    Err(Error::InvalidOperation(format!("{what} failed with code {code}: {msg}")))
}

/// The gradient as the step reads it, with its dtype tag.  An F32 gradient of a BF16 parameter goes in as it
/// is: the reference casts every gradient to F32 and never rounds it (adam8bit_enhanced.rs:231-235,
/// adam8bit.rs:110).  Any other mismatch is cast to the parameter's dtype (BF16 -> F32 is exact).
fn usable_grad(grad: &Tensor, param_dtype: DType) -> Result<(Tensor, i32)> {
    if grad.dtype() == param_dtype || (param_dtype == DType::BF16 && grad.dtype() == DType::F32) {
        Ok((grad.clone(), dtype_tag(grad.dtype())?))
    } else {
        Ok((grad.to_dtype(param_dtype)?, dtype_tag(param_dtype)?))
    }
}

/// One device allocation cut into equal lanes, the backing store for `MemoryPool::allocate_raw_memory`
/// (crates/core/src/memory.rs:289-311): a lane per kind of tensor keeps the kinds far apart in device memory.
pub struct DevicePool {
    pub(crate) pool: *mut sys::EriHipPool,
}

impl DevicePool {
    /// `bytes` = 0 takes nine tenths of the free device memory, `lanes` = 0 makes the lanes 48 GiB.
    pub fn new(device: i32, bytes: usize, lanes: u32) -> Result<Self> {
        let mut pool = std::ptr::null_mut();
        check(unsafe { sys::eri_hip_pool_create(device, bytes, lanes, &mut pool) }, "eri_hip_pool_create")?;
        Ok(Self { pool })
    }
    /// 256-byte aligned, zero-filled; the lane counts modulo the pool's lanes (e.g. the dtype tag).
    pub fn alloc_zeroed(&self, lane: u32, bytes: usize) -> Result<*mut u8> {
        let mut p: *mut c_void = std::ptr::null_mut();
        check(unsafe { sys::eri_hip_pool_alloc_zeroed(self.pool, lane, bytes, &mut p) }, "eri_hip_pool_alloc_zeroed")?;
        Ok(p as *mut u8)
    }
    /// The same, cleared by a kernel on `stream` (no host wait; usable under stream capture).
    pub fn alloc_zeroed_on(&self, lane: u32, bytes: usize, stream: *mut c_void) -> Result<*mut u8> {
        let mut p: *mut c_void = std::ptr::null_mut();
        check(unsafe { sys::eri_hip_pool_alloc_zeroed_async(self.pool, lane, bytes, stream, &mut p) }, "eri_hip_pool_alloc_zeroed_async")?;
        Ok(p as *mut u8)
    }
    /// Gives one piece back (`bytes` as requested); the next request of that size in its lane takes it.
    pub fn release(&self, ptr: *mut u8, bytes: usize) -> Result<()> {
        check(unsafe { sys::eri_hip_pool_release(self.pool, ptr as *mut c_void, bytes) }, "eri_hip_pool_release")
    }
    pub fn reset(&self) -> Result<()> {
        check(unsafe { sys::eri_hip_pool_reset(self.pool) }, "eri_hip_pool_reset")
    }
}

impl Drop for DevicePool {
    fn drop(&mut self) {
        unsafe { sys::eri_hip_pool_destroy(self.pool) };
    }
}

unsafe impl Send for DevicePool {}
unsafe impl Sync for DevicePool {}

fn dtype_tag(dt: DType) -> Result<i32> {
    match dt {
        DType::F32 => Ok(sys::ERI_DTYPE_F32),
        DType::BF16 => Ok(sys::ERI_DTYPE_BF16),
        other => Err(Error::Unsupported(format!("8-bit Adam takes F32 or BF16 parameters, got {other:?}"))),
    }
}

/// adam8bit_enhanced.rs:372-395
#[derive(Debug, Clone)]
pub struct Adam8bitConfig {
    pub lr: f64,
    pub betas: (f64, f64),
    pub eps: f64,
    pub weight_decay: f64,
    pub amsgrad: bool,
    pub block_wise: bool,
    pub percentile_clipping: usize,
    /// Not in the reference's struct, but written by its trainers (pipeline_flux_lora_1024.rs:451,
    /// `min_8bit_size: 4096`): tensors with fewer elements keep fp32 moments.  0 = all tensors 8-bit.
    pub min_8bit_size: usize,
}

impl Default for Adam8bitConfig {
    fn default() -> Self {
        Self { lr: 1e-3, betas: (0.9, 0.999), eps: 1e-8, weight_decay: 0.01, amsgrad: false, block_wise: true, percentile_clipping: 99, min_8bit_size: 0 }
    }
}

/// adam8bit_enhanced.rs:10-27.  The quantised states live on the device, owned by the C side.
pub struct Adam8bit {
    pub params: Vec<Parameter>,
    handles: Vec<*mut sys::EriParameter>,
    opt: *mut sys::EriAdam8bit,
    // Gradient tensors of the step in flight.  The launch is asynchronous, so they are released only when
    // the next step begins, which on the same stream is after the kernel that read them.
    live_grads: Vec<Tensor>,
    flushed: bool, // flush() has launched the step that reads live_grads
}

unsafe impl Send for Adam8bit {}
unsafe impl Sync for Adam8bit {}

impl Adam8bit {
    /// adam8bit_enhanced.rs:161.  The object starts in the arithmetic that reproduces the reference's bf16
    /// parameters bit for bit (ERI_ADAM8_FLAG_EXACT_PARAM); `eri_adam8bit_set_flags(opt, 0)` trades that for
    /// under one per cent of step time.
    pub fn new(params: Vec<Parameter>, config: Adam8bitConfig) -> Result<Self> {
        let mut handles = Vec::with_capacity(params.len());
        let mut stream: *mut c_void = std::ptr::null_mut();
        for p in &params {
            let t = p.tensor()?;
            stream = t.device().cuda_stream_raw_ptr();
            let mut h = std::ptr::null_mut();
            let numel: usize = t.shape().dims().iter().product();
            check(unsafe { sys::eri_param_create(t.cuda_ptr_mut() as *mut c_void, numel as u64, dtype_tag(t.dtype())?, &mut h) }, "eri_param_create")?;
            handles.push(h);
        }
        let cfg = sys::EriAdam8bitConfig {
            lr: config.lr, beta1: config.betas.0, beta2: config.betas.1, eps: config.eps,
            weight_decay: config.weight_decay, amsgrad: config.amsgrad as i32,
            block_wise: config.block_wise as i32, percentile_clipping: config.percentile_clipping as u64,
        };
        let mut opt = std::ptr::null_mut();
        check(unsafe { sys::eri_adam8bit_new(handles.as_ptr(), handles.len() as u32, &cfg, stream, &mut opt) }, "eri_adam8bit_new")?;
        if config.min_8bit_size > 0 {
            check(unsafe { sys::eri_adam8bit_set_min_8bit_size(opt, config.min_8bit_size as u64) }, "eri_adam8bit_set_min_8bit_size")?;
        }
        Ok(Self { params, handles, opt, live_grads: Vec::new(), flushed: false })
    }

    /// adam8bit_enhanced.rs:202-291.  One kernel launch for all parameters; parameters without a
    /// gradient are skipped with the reference's warning.
    pub fn step(&mut self) -> Result<()> {
        self.live_grads.clear();
        for (p, &h) in self.params.iter().zip(&self.handles) {
            let t = p.tensor()?;
            check(unsafe { sys::eri_param_set_data(h, t.cuda_ptr_mut() as *mut c_void) }, "eri_param_set_data")?;
            match p.grad() {
                Some(g) => {
                    let (g, tag) = usable_grad(&g, t.dtype())?;
                    check(unsafe { sys::eri_param_set_grad_typed(h, g.cuda_ptr() as *const c_void, tag) }, "eri_param_set_grad_typed")?;
                    self.live_grads.push(g);
                }
                None => check(unsafe { sys::eri_param_set_grad(h, std::ptr::null()) }, "eri_param_set_grad")?,
            }
        }
        check(unsafe { sys::eri_adam8bit_step(self.opt, std::ptr::null_mut()) }, "eri_adam8bit_step")
    }

    /// adam8bit_enhanced.rs:294
    pub fn zero_grad(&mut self) -> Result<()> {
        check(unsafe { sys::eri_adam8bit_zero_grad(self.opt) }, "eri_adam8bit_zero_grad")
    }
    /// :302
    pub fn current_lr(&self) -> f64 {
        unsafe { sys::eri_adam8bit_current_lr(self.opt) }
    }
    /// :307
    pub fn set_learning_rate(&mut self, lr: f64) {
        unsafe { sys::eri_adam8bit_set_learning_rate(self.opt, lr) };
    }
    /// :312
    pub fn quantized_memory_usage(&self) -> usize {
        unsafe { sys::eri_adam8bit_quantized_memory_usage(self.opt) as usize }
    }
    /// :318.  Tracking is opt-in here (`track_quantization_error(true)`): it costs one read pass per step.
    pub fn quantization_stats(&self) -> (f32, f32) {
        let (mut m, mut v) = (0f32, 0f32);
        unsafe { sys::eri_adam8bit_quantization_stats(self.opt, &mut m, &mut v) };
        (m, v)
    }
    pub fn track_quantization_error(&mut self, enabled: bool) {
        unsafe { sys::eri_adam8bit_track_quantization_error(self.opt, enabled as i32) };
    }
    /// Fold the global-norm clip factor into the next steps instead of rewriting every gradient
    /// (pipeline_flux_lora_sequential.rs:1198-1213).
    pub fn set_grad_scale(&mut self, scale: f32) -> Result<()> {
        check(unsafe { sys::eri_adam8bit_set_grad_scale(self.opt, scale) }, "eri_adam8bit_set_grad_scale")
    }
    /// States that do not exist yet (they are created at the first step) come out of `lane` of the pool: a lane
    /// 32 GiB or more away from the parameters' makes every later step 10-17 % faster on LoRA- and SDXL-sized sets.
    /// The pool must outlive the optimizer.
    pub fn set_state_pool(&mut self, pool: &DevicePool, lane: u32) -> Result<()> {
        check(unsafe { sys::eri_adam8bit_set_state_pool(self.opt, pool.pool, lane) }, "eri_adam8bit_set_state_pool")
    }
    /// From now on every step() also performs `ema.update(params)` (ema_enhanced.rs:79-104) over this optimizer's
    /// parameters, `names[i]` being the model's name for parameter i; the trainer drops its own ema.update() call.
    /// The model must outlive the optimizer or be detached with `detach_ema()`.
    pub fn attach_ema(&mut self, ema: &mut EMAModel, names: &[&str]) -> Result<()> {
        let c: Vec<CString> = names.iter().map(|n| CString::new(*n).unwrap()).collect();
        let ptrs: Vec<*const std::os::raw::c_char> = c.iter().map(|n| n.as_ptr()).collect();
        check(unsafe { sys::eri_adam8bit_attach_ema(self.opt, ema.ema, ptrs.as_ptr(), ptrs.len() as u32) }, "eri_adam8bit_attach_ema")
    }
    pub fn detach_ema(&mut self) {
        unsafe { sys::eri_adam8bit_attach_ema(self.opt, std::ptr::null_mut(), std::ptr::null(), 0) };
    }
    /// Global-norm clipping inside step(): norm on the device, factor applied by the step kernel.
    pub fn set_max_grad_norm(&mut self, max_norm: f32, denom_eps: f32) -> Result<()> {
        check(unsafe { sys::eri_adam8bit_set_max_grad_norm(self.opt, max_norm, denom_eps) }, "eri_adam8bit_set_max_grad_norm")
    }
    /// (norm, clip factor, NaN/inf gradient elements) of the last step that clipped.
    pub fn last_grad_norm(&mut self) -> Result<(f32, f32, u64)> {
        let (mut n, mut s, mut bad) = (0f32, 1f32, 0u64);
        check(unsafe { sys::eri_adam8bit_last_grad_norm(self.opt, &mut n, &mut s) }, "eri_adam8bit_last_grad_norm")?;
        check(unsafe { sys::eri_adam8bit_last_nonfinite_grads(self.opt, &mut bad) }, "eri_adam8bit_last_nonfinite_grads")?;
        Ok((n, s, bad))
    }
    /// Imports a file written by the reference's own save_state (bincode of OptimizerState, :330-347).
    pub fn load_legacy_state(&mut self, path: &Path) -> Result<()> {
        let c = CString::new(path.to_string_lossy().as_bytes()).map_err(|e| Error::InvalidOperation(e.to_string()))?;
        check(unsafe { sys::eri_adam8bit_load_legacy_state(self.opt, c.as_ptr()) }, "eri_adam8bit_load_legacy_state")
    }
    /// :330
    pub fn save_state(&self, path: &Path) -> Result<()> {
        let c = CString::new(path.to_string_lossy().as_bytes()).map_err(|e| Error::InvalidOperation(e.to_string()))?;
        check(unsafe { sys::eri_adam8bit_save_state(self.opt, c.as_ptr()) }, "eri_adam8bit_save_state")
    }
    /// :350
    pub fn load_state(&mut self, path: &Path) -> Result<()> {
        let c = CString::new(path.to_string_lossy().as_bytes()).map_err(|e| Error::InvalidOperation(e.to_string()))?;
        check(unsafe { sys::eri_adam8bit_load_state(self.opt, c.as_ptr()) }, "eri_adam8bit_load_state")
    }
}

impl Drop for Adam8bit {
    fn drop(&mut self) {
        unsafe {
            sys::eri_adam8bit_destroy(self.opt);
            for &h in &self.handles {
                sys::eri_param_release(h);
            }
        }
    }
}

/// Functional flavour, `src/trainers/adam8bit.rs:15-28`: states keyed by the name given to update().
pub struct Adam8bitFunctional {
    opt: *mut sys::EriAdam8bitFn,
    names: Vec<String>,
    batched: bool,
    // With batching, the tensors a queued update reads and writes, kept until the step after the launch.
    live: Vec<Tensor>,
    launched: bool,
}

unsafe impl Send for Adam8bitFunctional {}
unsafe impl Sync for Adam8bitFunctional {}

impl Adam8bitFunctional {
    /// adam8bit.rs:69-86
    pub fn with_params(learning_rate: f64, beta1: f64, beta2: f64, eps: f64, weight_decay: f64) -> Self {
        let mut opt = std::ptr::null_mut();
        unsafe { sys::eri_adam8bit_fn_with_params(learning_rate, beta1, beta2, eps, weight_decay, std::ptr::null_mut(), &mut opt) };
        Self { opt, names: Vec::new(), batched: false, live: Vec::new(), launched: false }
    }
    /// Queue update() calls and run them as ONE launch at step(): for trainers that only store the tensor
    /// update() returns (`layer.lora_down.set_data(updated)`, pipeline_flux_lora_sequential.rs:767-792).
    /// A trainer that reads the returned tensor before step() (pipeline_sdxl_lora.rs:710) keeps the
    /// default, or moves to update_many().
    pub fn batched(mut self, enabled: bool) -> Self {
        unsafe { sys::eri_adam8bit_fn_set_batching(self.opt, enabled as i32) };
        self.batched = enabled;
        self
    }
    /// States of names not seen yet come out of `lane` of the pool (see `Adam8bit::set_state_pool`).
    pub fn state_pool(self, pool: &DevicePool, lane: u32) -> Self {
        unsafe { sys::eri_adam8bit_fn_set_state_pool(self.opt, pool.pool, lane) };
        self
    }
    /// :89-92
    pub fn step(&mut self) -> Result<()> {
        let rc = check(unsafe { sys::eri_adam8bit_fn_step(self.opt) }, "eri_adam8bit_fn_step");
        self.launched = true; // `live` is released when the next update arrives, after this launch in stream order
        rc
    }
    /// :95-98
    pub fn set_lr(&mut self, lr: f32) -> Result<()> {
        check(unsafe { sys::eri_adam8bit_fn_set_lr(self.opt, lr) }, "eri_adam8bit_fn_set_lr")
    }
    /// :311-313
    pub fn get_step(&self) -> usize {
        unsafe { sys::eri_adam8bit_fn_get_step(self.opt) as usize }
    }
    /// :101-208: returns the updated tensor, the input is left alone
    pub fn update(&mut self, name: &str, param: &Tensor, grad: &Tensor) -> Result<Tensor> {
        if self.launched {
            self.live.clear();
            self.launched = false;
        }
        let out = Tensor::zeros_dtype(param.shape().clone(), param.dtype(), param.device().clone())?;
        let (g, g_tag) = usable_grad(grad, param.dtype())?;
        let numel: usize = param.shape().dims().iter().product();
        let c = CString::new(name).map_err(|e| Error::InvalidOperation(e.to_string()))?;
        check(unsafe {
            sys::eri_adam8bit_fn_update(self.opt, c.as_ptr(), param.cuda_ptr() as *const c_void, g.cuda_ptr() as *const c_void,
                                        numel as u64, dtype_tag(param.dtype())?, g_tag, out.cuda_ptr_mut() as *mut c_void)
        }, "eri_adam8bit_fn_update")?;
        // the launch is asynchronous (and, batched, still to come): what it reads and writes must not be freed
        // under it; released when the first update after the launch arrives
        self.live.push(g);
        self.live.push(param.clone());
        self.live.push(out.clone());
        if !self.batched {
            self.launched = true;
        }
        if !self.names.iter().any(|n| n == name) {
            self.names.push(name.to_string());
        }
        Ok(out)
    }
    /// :253-266
    pub fn memory_stats(&self) -> (usize, usize) {
        let (mut n, mut b) = (0u64, 0u64);
        unsafe { sys::eri_adam8bit_fn_memory_stats(self.opt, &mut n, &mut b) };
        (n as usize, b as usize)
    }
    /// :296-308: fp32 moments per name, the layout the trainers write as `optimizer.{name}.m|.v`
    /// (pipeline_flux_lora_sequential.rs:1481-1487)
    pub fn get_state_as_tensors(&self, device: &flame_core::device::Device) -> Result<HashMap<String, (Tensor, Tensor)>> {
        let mut out = HashMap::new();
        for name in &self.names {
            let c = CString::new(name.as_str()).unwrap();
            let mut numel = 0u64;
            check(unsafe { sys::eri_adam8bit_fn_state_numel(self.opt, c.as_ptr(), &mut numel) }, "eri_adam8bit_fn_state_numel")?;
            let shape = flame_core::Shape::from_dims(&[numel as usize]);
            let m = Tensor::zeros(shape.clone(), device.cuda_device_arc())?;
            let v = Tensor::zeros(shape, device.cuda_device_arc())?;
            check(unsafe { sys::eri_adam8bit_fn_get_state_fp32(self.opt, c.as_ptr(), m.cuda_ptr_mut() as *mut f32, v.cuda_ptr_mut() as *mut f32) },
                  "eri_adam8bit_fn_get_state_fp32")?;
            out.insert(name.clone(), (m, v));
        }
        Ok(out)
    }
    /// :316-329
    pub fn load_state_from_tensors(&mut self, state: HashMap<String, (Tensor, Tensor)>) -> Result<()> {
        for (name, (m, v)) in state {
            let m = m.to_dtype(DType::F32)?;
            let v = v.to_dtype(DType::F32)?;
            let numel: usize = m.shape().dims().iter().product();
            let c = CString::new(name.as_str()).map_err(|e| Error::InvalidOperation(e.to_string()))?;
            check(unsafe { sys::eri_adam8bit_fn_load_state_fp32(self.opt, c.as_ptr(), m.cuda_ptr() as *const f32, v.cuda_ptr() as *const f32, numel as u64) },
                  "eri_adam8bit_fn_load_state_fp32")?;
            if !self.names.contains(&name) {
                self.names.push(name);
            }
        }
        Ok(())
    }
}

impl Drop for Adam8bitFunctional {
    fn drop(&mut self) {
        unsafe { sys::eri_adam8bit_fn_destroy(self.opt) };
    }
}

impl Adam8bitFunctional {
    /// Every (name, param, grad) in one launch; returns the new tensors in the same order.
    pub fn update_many(&mut self, items: &[(&str, &Tensor, &Tensor)]) -> Result<Vec<Tensor>> {
        if self.launched {
            self.live.clear();
            self.launched = false;
        }
        let n = items.len();
        let (mut names, mut name_ptrs, mut ps, mut gs, mut outs_ptr) = (Vec::with_capacity(n), Vec::with_capacity(n), Vec::with_capacity(n), Vec::with_capacity(n), Vec::with_capacity(n));
        let (mut numels, mut tags, mut g_tags, mut outs) = (Vec::with_capacity(n), Vec::with_capacity(n), Vec::with_capacity(n), Vec::with_capacity(n));
        for (name, param, grad) in items {
            let (g, g_tag) = usable_grad(grad, param.dtype())?;
            let out = Tensor::zeros_dtype(param.shape().clone(), param.dtype(), param.device().clone())?;
            names.push(CString::new(*name).map_err(|e| Error::InvalidOperation(e.to_string()))?);
            ps.push(param.cuda_ptr() as *const c_void);
            gs.push(g.cuda_ptr() as *const c_void);
            outs_ptr.push(out.cuda_ptr_mut() as *mut c_void);
            numels.push(param.shape().dims().iter().product::<usize>() as u64);
            tags.push(dtype_tag(param.dtype())?);
            g_tags.push(g_tag);
            self.live.push(g);
            self.live.push((*param).clone()); // the kernel reads the old parameter in place, without a copy
            self.live.push(out.clone());
            outs.push(out);
            if !self.names.iter().any(|k| k == name) {
                self.names.push(name.to_string());
            }
        }
        for c in &names {
            name_ptrs.push(c.as_ptr());
        }
        check(unsafe {
            sys::eri_adam8bit_fn_update_many(self.opt, name_ptrs.as_ptr(), ps.as_ptr(), gs.as_ptr(), numels.as_ptr(), tags.as_ptr(),
                                             g_tags.as_ptr(), outs_ptr.as_ptr(), n as u32)
        }, "eri_adam8bit_fn_update_many")?;
        self.launched = true;
        Ok(outs)
    }
}

/// adam8bit.rs:333-345, as one launch instead of a loop of update() calls
pub fn update_params_8bit(optimizer: &mut Adam8bitFunctional, params: &mut HashMap<String, Tensor>, grads: &HashMap<String, Tensor>) -> Result<()> {
    let names: Vec<String> = params.keys().filter(|k| grads.contains_key(*k)).cloned().collect();
    let items: Vec<(&str, &Tensor, &Tensor)> = names.iter().map(|k| (k.as_str(), &params[k], &grads[k])).collect();
    let outs = optimizer.update_many(&items)?;
    for (k, t) in names.iter().zip(outs) {
        params.insert(k.clone(), t);
    }
    Ok(())
}

// ---- the reference's optimizer traits ---------------------------------------------------------
// Paths as in the reference tree; each impl only forwards to the methods above.

/// `OptimizerWrapper { step, zero_grad, vars }`, crates/training/src/optimizers/wrapper.rs:40-44.
impl crate::optimizers::wrapper::OptimizerWrapper for Adam8bit {
    fn step(&mut self) -> Result<()> {
        Adam8bit::step(self)
    }
    fn zero_grad(&mut self) {
        let _ = Adam8bit::zero_grad(self);
    }
    fn vars(&mut self) -> &mut [Parameter] {
        self.params.as_mut_slice()
    }
}

/// `training::OptimizerTrait`, src/trainers/training/optimization.rs:61-73.  The reference's impl for
/// Adam8bit is a set of placeholders (:75-103: step does nothing, get_lr returns 1e-4); here the
/// per-parameter step() hands the gradient to the matching handle and the launch happens in
/// `flush()`, which the trainer calls once per accumulation boundary where it called nothing before.
impl crate::trainers::training::optimization::OptimizerTrait for Adam8bit {
    fn step(&mut self, param: &Parameter, grad: &Tensor) -> Result<()> {
        let t = param.tensor()?;
        let at = self.params.iter().position(|p| p.tensor().map(|q| q.cuda_ptr() == t.cuda_ptr()).unwrap_or(false))
            .ok_or_else(|| Error::InvalidOperation("parameter is not owned by this optimizer".into()))?;
        if self.flushed {
            self.live_grads.clear(); // the step that read them was launched before this call, on the same stream
            self.flushed = false;
        }
        let (g, tag) = usable_grad(grad, t.dtype())?;
        check(unsafe { sys::eri_param_set_grad_typed(self.handles[at], g.cuda_ptr() as *const c_void, tag) }, "eri_param_set_grad_typed")?;
        self.live_grads.push(g);
        Ok(())
    }
    fn zero_grad(&mut self) -> Result<()> {
        Adam8bit::zero_grad(self)
    }
    fn get_lr(&self) -> f32 {
        self.current_lr() as f32
    }
    fn set_lr(&mut self, lr: f32) {
        self.set_learning_rate(lr as f64)
    }
    fn state_dict(&self) -> Result<HashMap<String, Tensor>> {
        Err(Error::Unsupported("the 8-bit state is saved with save_state(path), not as tensors".into()))
    }
    fn load_state_dict(&mut self, _state: HashMap<String, Tensor>) -> Result<()> {
        Err(Error::Unsupported("the 8-bit state is loaded with load_state(path)".into()))
    }
}

impl Adam8bit {
    /// Launches the step for the gradients handed over through `OptimizerTrait::step`.
    pub fn flush(&mut self) -> Result<()> {
        let rc = check(unsafe { sys::eri_adam8bit_step(self.opt, std::ptr::null_mut()) }, "eri_adam8bit_step");
        self.flushed = true; // live_grads stay until the next gradient arrives: the launch above still reads them
        rc
    }
}

/// crates/training/src/optimizers/adam8bit.rs:4-28.  The quantile fields steer the reference's per-tensor
/// clipping (adam8bit_enhanced.rs:53-69); the blockwise format has no such step, so they are carried only.
#[derive(Debug, Clone)]
pub struct AdamW8bitConfig {
    pub lr: f64,
    pub beta1: f64,
    pub beta2: f64,
    pub epsilon: f64,
    pub weight_decay: f64,
    pub quantile_alpha: f32,
    pub adaptive_quantization: bool,
    pub quantization_warmup_steps: usize,
}

impl Default for AdamW8bitConfig {
    fn default() -> Self {
        Self { lr: 1e-3, beta1: 0.9, beta2: 0.999, epsilon: 1e-8, weight_decay: 0.01, quantile_alpha: 0.99,
               adaptive_quantization: true, quantization_warmup_steps: 100 }
    }
}

impl From<AdamW8bitConfig> for Adam8bitConfig {
    fn from(c: AdamW8bitConfig) -> Self {
        Self { lr: c.lr, betas: (c.beta1, c.beta2), eps: c.epsilon, weight_decay: c.weight_decay, ..Self::default() }
    }
}

/// src/trainers/training/optimization.rs:9-27
#[derive(Debug, Clone, serde::Serialize, serde::Deserialize)]
pub struct OptimizerConfig {
    pub optimizer_type: String,
    pub learning_rate: f32,
    pub weight_decay: Option<f32>,
    pub betas: Option<(f32, f32)>,
    pub eps: Option<f32>,
}

impl Default for OptimizerConfig {
    fn default() -> Self {
        Self { optimizer_type: "adamw8bit".to_string(), learning_rate: 1e-4, weight_decay: Some(0.01),
               betas: Some((0.9, 0.999)), eps: Some(1e-8) }
    }
}

/// optimization.rs:30-58 with its own argument list (f32 fields widened as the reference does, :38-41)
pub fn create_optimizer_from_config(config: &OptimizerConfig, parameters: Vec<Parameter>) -> Result<Adam8bit> {
    create_optimizer(&config.optimizer_type, parameters, config.learning_rate as f64,
                     config.betas.map(|(a, b)| (a as f64, b as f64)), config.eps.map(|e| e as f64),
                     config.weight_decay.map(|w| w as f64))
}

/// String-keyed factory, src/trainers/training/optimization.rs:30-58 and
/// src/optimizers/memory_efficient_optimizers.rs:285-308.
pub fn create_optimizer(optimizer_type: &str, parameters: Vec<Parameter>, learning_rate: f64, betas: Option<(f64, f64)>,
                        eps: Option<f64>, weight_decay: Option<f64>) -> Result<Adam8bit> {
    match optimizer_type {
        "adam8bit" | "adamw8bit" | "adamw_8bit" => Adam8bit::new(parameters, Adam8bitConfig {
            lr: learning_rate, betas: betas.unwrap_or((0.9, 0.999)), eps: eps.unwrap_or(1e-8),
            weight_decay: weight_decay.unwrap_or(0.0), ..Adam8bitConfig::default()
        }),
        other => Err(Error::InvalidOperation(format!("Unknown optimizer: {other}"))),
    }
}

// ---- EMAModel, src/trainers/ema_enhanced.rs:12-204 ---------------------------------------------

pub struct EMAModel {
    ema: *mut sys::EriEmaModel,
}

unsafe impl Send for EMAModel {}

impl EMAModel {
    /// :35-52 (bias correction on, power 1)
    pub fn new(decay: f32, stream: *mut c_void) -> Result<Self> {
        Self::with_config(decay, stream, true, 1.0)
    }
    /// :55-64
    pub fn with_config(decay: f32, stream: *mut c_void, use_bias_correction: bool, power: f32) -> Result<Self> {
        let mut ema = std::ptr::null_mut();
        check(unsafe { sys::eri_ema_new(decay, use_bias_correction as i32, power, stream, &mut ema) }, "eri_ema_new")?;
        Ok(Self { ema })
    }
    fn with_handles<R>(params: &HashMap<String, &Parameter>, f: impl FnOnce(*const *const std::os::raw::c_char, *const *mut sys::EriParameter, u32) -> i32, what: &str) -> Result<()> {
        let names: Vec<CString> = params.keys().map(|k| CString::new(k.as_str()).unwrap()).collect();
        let name_ptrs: Vec<*const std::os::raw::c_char> = names.iter().map(|c| c.as_ptr()).collect();
        let mut handles = Vec::with_capacity(params.len());
        for p in params.values() {
            let t = p.tensor()?;
            let numel: usize = t.shape().dims().iter().product();
            let mut h = std::ptr::null_mut();
            check(unsafe { sys::eri_param_create(t.cuda_ptr_mut() as *mut c_void, numel as u64, dtype_tag(t.dtype())?, &mut h) }, "eri_param_create")?;
            handles.push(h);
        }
        let rc = f(name_ptrs.as_ptr(), handles.as_ptr(), handles.len() as u32);
        for h in handles {
            unsafe { sys::eri_param_release(h) };
        }
        check(rc, what)
    }
    /// :67-76
    pub fn init_from_params(&mut self, params: &HashMap<String, &Parameter>) -> Result<()> {
        let ema = self.ema;
        Self::with_handles::<()>(params, |n, h, k| unsafe { sys::eri_ema_init_from_params(ema, n, h, k) }, "eri_ema_init_from_params")
    }
    /// :79-104, one launch over every known parameter
    pub fn update(&mut self, params: &HashMap<String, &Parameter>) -> Result<()> {
        let ema = self.ema;
        Self::with_handles::<()>(params, |n, h, k| unsafe { sys::eri_ema_update(ema, n, h, k) }, "eri_ema_update")
    }
    /// :130-142 (the shadow's values are copied into the parameter's memory)
    pub fn copy_to(&self, params: &HashMap<String, &Parameter>) -> Result<()> {
        let ema = self.ema;
        Self::with_handles::<()>(params, |n, h, k| unsafe { sys::eri_ema_copy_to(ema, n, h, k) }, "eri_ema_copy_to")
    }
    pub fn step(&self) -> usize {
        unsafe { sys::eri_ema_step(self.ema) as usize }
    }
    pub fn set_step(&mut self, step: usize) {
        unsafe { sys::eri_ema_set_step(self.ema, step as u64) };
    }
    pub fn current_decay(&self) -> f32 {
        unsafe { sys::eri_ema_current_decay(self.ema) }
    }
}

impl Drop for EMAModel {
    fn drop(&mut self) {
        unsafe { sys::eri_ema_destroy(self.ema) };
    }
}

/// :268-279
pub fn decay_from_half_life(half_life_steps: usize) -> f32 {
    unsafe { sys::eri_ema_decay_from_half_life(half_life_steps as u64) }
}
pub fn decay_from_window(window_size: usize) -> f32 {
    unsafe { sys::eri_ema_decay_from_window(window_size as u64) }
}
