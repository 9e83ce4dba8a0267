//! Host side of the MI355X mixture-of-experts layer in the reference's own shapes:
//! `MoeConfig` (src/moe.rs:25-87), `MoeLayer::{new, forward, forward_train}` (src/moe.rs:215-341),
//! `MoeCache` (src/moe.rs:131-188), `Layout` (src/batch.rs:224-269) and the error variants of
//! `NetworkError` (src/network.rs:19-83) that this path can produce.
//!
//! UNVERIFIED: written without a Rust toolchain; it has never been compiled.  The same surface is
//! tested through the C++ header `rusting_brain_moe.hpp` and the Python package `rustingbrain_amd`.
//!
//! Matrices are plain row-major `Vec<f32>` with a row and column count, as the reference's `Matrix`
//! (src/matrix.rs:13-18).  This wrapper talks f32 to the library's host entry point; the layer keeps
//! its weights in the dtype chosen at construction.

pub mod sys;

use std::ffi::CStr;
use std::os::raw::{c_int, c_void};
use std::ptr;
use std::sync::Arc;

/// The reference's marker for "this slot was not routed" (src/moe.rs:190-191).
pub const UNROUTED: usize = usize::MAX;

#[derive(Debug, Clone, PartialEq)]
pub enum NetworkError {
    InvalidInput { expected: usize, actual: usize },
    InvalidConfig(String),
    /// `NetworkError::Cuda` in the reference: a device call failed.
    Device(String),
    /// `NetworkError::CudaFeatureDisabled`: no usable GPU; there is no CPU fallback.
    BackendUnavailable,
    MemoryBudget(String),
    OutOfMemory(String),
    Unsupported(String),
}

fn message(ctx: *const sys::rbmoe_ctx) -> String {
    let p = unsafe { if ctx.is_null() { sys::rbmoe_last_global_error() } else { sys::rbmoe_last_error(ctx) } };
    if p.is_null() {
        String::new()
    } else {
        unsafe { CStr::from_ptr(p) }.to_string_lossy().into_owned()
    }
}

fn check(code: c_int, ctx: *const sys::rbmoe_ctx, expected: usize, actual: usize) -> Result<(), NetworkError> {
    match code {
        sys::RBMOE_OK => Ok(()),
        sys::RBMOE_INVALID_INPUT => Err(NetworkError::InvalidInput { expected, actual }),
        sys::RBMOE_INVALID_CONFIG => Err(NetworkError::InvalidConfig(message(ctx))),
        sys::RBMOE_BACKEND_UNAVAILABLE => Err(NetworkError::BackendUnavailable),
        sys::RBMOE_MEMORY_BUDGET => Err(NetworkError::MemoryBudget(message(ctx))),
        sys::RBMOE_OUT_OF_MEMORY => Err(NetworkError::OutOfMemory(message(ctx))),
        sys::RBMOE_UNSUPPORTED => Err(NetworkError::Unsupported(message(ctx))),
        _ => Err(NetworkError::Device(message(ctx))),
    }
}

/// Storage type of the expert weights on the device.
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum WeightDtype {
    F32,
    Bf16,
    Int8,
}

/// `MoeConfig` (src/moe.rs:25-39) with the reference's defaults (src/moe.rs:20-23, :41-51).
#[derive(Clone, Debug, PartialEq)]
pub struct MoeConfig {
    pub num_experts: usize,
    pub experts_per_token: usize,
    pub d_ff: usize,
    pub shared_expert: bool,
    pub aux_loss_weight: f32,
    pub router_z_loss_weight: f32,
}

impl MoeConfig {
    pub fn new(num_experts: usize, experts_per_token: usize, d_ff: usize) -> Self {
        Self { num_experts, experts_per_token, d_ff, shared_expert: false, aux_loss_weight: 0.01,
               router_z_loss_weight: 1e-3 }
    }
    pub fn with_shared_expert(mut self, enabled: bool) -> Self {
        self.shared_expert = enabled;
        self
    }
    pub fn with_aux_loss_weight(mut self, weight: f32) -> Self {
        self.aux_loss_weight = weight;
        self
    }
    pub fn with_router_z_loss_weight(mut self, weight: f32) -> Self {
        self.router_z_loss_weight = weight;
        self
    }
}

/// `Layout` (src/batch.rs:224-269): which rows are real tokens.
#[derive(Clone, Debug, Default)]
pub struct Layout<'a> {
    pub valid: Option<&'a [bool]>,
}

struct ContextHandle(*mut sys::rbmoe_ctx);
unsafe impl Send for ContextHandle {}
unsafe impl Sync for ContextHandle {}
impl Drop for ContextHandle {
    fn drop(&mut self) {
        unsafe { sys::rbmoe_ctx_destroy(self.0) }
    }
}

/// One GPU, one stream, one memory budget: the role of `CudaDevice::open` (src/param.rs:86-190).
#[derive(Clone)]
pub struct Device(Arc<ContextHandle>);

impl Device {
    pub fn open(ordinal: usize, budget_mib: usize) -> Result<Self, NetworkError> {
        let mut ctx = ptr::null_mut();
        check(unsafe { sys::rbmoe_ctx_create(ordinal as i32, budget_mib, &mut ctx) }, ptr::null(), 0, 0)?;
        Ok(Self(Arc::new(ContextHandle(ctx))))
    }
    pub fn synchronize(&self) -> Result<(), NetworkError> {
        check(unsafe { sys::rbmoe_synchronize(self.raw()) }, self.raw(), 0, 0)
    }
    fn raw(&self) -> *mut sys::rbmoe_ctx {
        (self.0).0
    }
}

/// What `forward_train` hands back (src/moe.rs:131-188), routing tables included.
#[derive(Clone, Debug)]
pub struct MoeCache {
    pub probabilities: Vec<f32>,
    pub log_sum_exp: Vec<f32>,
    /// `(expert, gate)` per slot, slot = token * k + rank; `UNROUTED` for padding rows.
    pub assignments: Vec<(usize, f32)>,
    pub valid_tokens: usize,
    pub expert_tokens: Vec<Vec<usize>>,
    pub expert_slots: Vec<Vec<usize>>,
    aux_loss: f32,
    z_loss: f32,
}

impl MoeCache {
    pub fn aux_loss(&self) -> f32 {
        self.aux_loss
    }
    pub fn z_loss(&self) -> f32 {
        self.z_loss
    }
    pub fn auxiliary_loss(&self) -> f32 {
        self.aux_loss + self.z_loss
    }
    /// Share of the routed slots each expert received (src/moe.rs:176-182).
    pub fn load_fractions(&self) -> Vec<f32> {
        let total: usize = self.expert_tokens.iter().map(Vec::len).sum();
        if total == 0 {
            return vec![0.0; self.expert_tokens.len()];
        }
        self.expert_tokens.iter().map(|t| t.len() as f32 / total as f32).collect()
    }
}

/// The device layer behind `MoeLayer`'s surface.
pub struct MoeLayer {
    device: Device,
    layer: *mut sys::rbmoe_layer,
    d_model: usize,
    config: MoeConfig,
    max_tokens: usize,
}

unsafe impl Send for MoeLayer {}

impl Drop for MoeLayer {
    fn drop(&mut self) {
        unsafe { sys::rbmoe_layer_destroy(self.layer) }
    }
}

impl MoeLayer {
    /// `MoeLayer::new` (src/moe.rs:215-231) on a device: validates, checks the budget before
    /// allocating, allocates weights (zeroed) and a workspace for `max_tokens` rows.
    pub fn new(d_model: usize, config: MoeConfig, device: &Device, weights: WeightDtype,
               max_tokens: usize) -> Result<Self, NetworkError> {
        let mut c = sys::rbmoe_config::default();
        check(unsafe {
            sys::rbmoe_config_init(&mut c, d_model as i32, config.num_experts as i32,
                                   config.experts_per_token as i32, config.d_ff as i32)
        }, device.raw(), 0, 0)?;
        c.shared_expert = config.shared_expert as i32;
        c.aux_loss_weight = config.aux_loss_weight;
        c.router_z_loss_weight = config.router_z_loss_weight;
        c.weight_dtype = match weights {
            WeightDtype::F32 => sys::RBMOE_F32,
            WeightDtype::Bf16 => sys::RBMOE_BF16,
            WeightDtype::Int8 => sys::RBMOE_I8,
        };
        // f32 on the boundary, as the reference's `Matrix`.  With bf16 or int8 weights the library routes on
        // the f32 rows and runs the expert products on the bf16 matrix cores over a bf16 copy of them.
        c.act_dtype = sys::RBMOE_F32;
        c.max_tokens = max_tokens as i32;
        let mut layer = ptr::null_mut();
        check(unsafe { sys::rbmoe_layer_create(device.raw(), &c, &mut layer) }, device.raw(), 0, 0)?;
        Ok(Self { device: device.clone(), layer, d_model, config, max_tokens })
    }

    fn set(&mut self, which: i32, expert: usize, data: &[f32], rows: usize, cols: usize) -> Result<(), NetworkError> {
        if data.len() != rows * cols {
            return Err(NetworkError::InvalidInput { expected: rows * cols, actual: data.len() });
        }
        check(unsafe {
            sys::rbmoe_set_weight(self.layer, which, expert as i32, data.as_ptr() as *const c_void, sys::RBMOE_F32,
                                  ptr::null(), rows as i32, cols as i32)
        }, self.device.raw(), rows * cols, data.len())
    }

    /// Router weight `[num_experts, d_model]` (src/moe.rs:91-100).
    pub fn set_router(&mut self, weight: &[f32]) -> Result<(), NetworkError> {
        let (e, d) = (self.config.num_experts, self.d_model);
        self.set(sys::RBMOE_W_ROUTER, 0, weight, e, d)
    }

    /// One expert's `gate [d_ff, d]`, `up [d_ff, d]`, `down [d, d_ff]` (src/ffn.rs:19-23).
    pub fn set_expert(&mut self, expert: usize, gate: &[f32], up: &[f32], down: &[f32]) -> Result<(), NetworkError> {
        let (f, d) = (self.config.d_ff, self.d_model);
        self.set(sys::RBMOE_W_GATE, expert, gate, f, d)?;
        self.set(sys::RBMOE_W_UP, expert, up, f, d)?;
        self.set(sys::RBMOE_W_DOWN, expert, down, d, f)
    }

    pub fn set_shared(&mut self, gate: &[f32], up: &[f32], down: &[f32]) -> Result<(), NetworkError> {
        let (f, d) = (self.config.d_ff, self.d_model);
        self.set(sys::RBMOE_W_SHARED_GATE, 0, gate, f, d)?;
        self.set(sys::RBMOE_W_SHARED_UP, 0, up, f, d)?;
        self.set(sys::RBMOE_W_SHARED_DOWN, 0, down, d, f)
    }

    /// Makes the forward pass keep what `backward` needs and allocates the f32 gradient accumulators (the
    /// role of `Param.grad`).  Call before the weights are set.  Every f32 and bf16 layer has a backward pass
    /// (matrix-core kernels where the widths fit them, plain ones otherwise); int8 layers report `UnsupportedCuda`.
    /// A behaviour switch of the layer (`sys::RBMOE_OPT_*`); every default is the fast path.
    pub fn set_option(&mut self, option: i32, value: i32) -> Result<(), NetworkError> {
        check(unsafe { sys::rbmoe_layer_set_option(self.layer, option, value) }, self.device.raw(), 0, 0)
    }

    pub fn enable_training(&mut self) -> Result<(), NetworkError> {
        check(unsafe { sys::rbmoe_layer_enable_training(self.layer) }, self.device.raw(), 0, 0)
    }

    /// `MoeLayer::backward` (src/moe.rs:348-489) for the last `forward_train`: `grad_output` and the
    /// returned gradient of the input are `[rows, d_model]` in the layer's activation type (raw bytes of
    /// f32 or bf16 values); weight gradients accumulate until `zero_grads`.  `rows` must be the last
    /// forward's row count: the library refuses anything else before it touches either buffer, and a slice
    /// whose length is not `rows * d_model` elements is refused here.
    pub fn backward_raw(&mut self, grad_output: &[u8], rows: usize) -> Result<Vec<u8>, NetworkError> {
        let elem = 4; // the layer is created with f32 rows on the boundary (see `new`)
        let expected = rows * self.d_model * elem;
        if grad_output.len() != expected {
            return Err(NetworkError::InvalidInput { expected, actual: grad_output.len() });
        }
        let mut grad_input = vec![0u8; expected];
        check(unsafe {
            sys::rbmoe_backward_host(self.layer, grad_output.as_ptr() as *const c_void, rows as i32,
                                     self.d_model as i32, grad_input.as_mut_ptr() as *mut c_void)
        }, self.device.raw(), 0, 0)?;
        Ok(grad_input)
    }

    /// `Param::zero_grad` over every weight of the layer.
    pub fn zero_grads(&mut self) -> Result<(), NetworkError> {
        check(unsafe { sys::rbmoe_zero_grads(self.layer) }, self.device.raw(), 0, 0)
    }

    /// The accumulated gradient of one weight matrix (`which`: `sys::RBMOE_W_*`), `[rows, cols]` as the weight.
    pub fn weight_grad(&self, which: i32, expert: usize, rows: usize, cols: usize) -> Result<Vec<f32>, NetworkError> {
        let mut g = vec![0f32; rows * cols];
        check(unsafe {
            sys::rbmoe_get_weight_grad(self.layer, which, expert as i32, g.as_mut_ptr(), rows as i32, cols as i32)
        }, self.device.raw(), 0, 0)?;
        Ok(g)
    }

    /// `MoeLayer::forward` (src/moe.rs:237-241).
    pub fn forward(&self, input: &[f32], rows: usize, cols: usize) -> Result<Vec<f32>, NetworkError> {
        self.forward_train(input, rows, cols, Layout::default()).map(|(out, _)| out)
    }

    /// `MoeLayer::forward_train` (src/moe.rs:243-341): output `[rows, d_model]` and the cache.
    pub fn forward_train(&self, input: &[f32], rows: usize, cols: usize, layout: Layout<'_>)
                         -> Result<(Vec<f32>, MoeCache), NetworkError> {
        if cols != self.d_model {
            return Err(NetworkError::InvalidInput { expected: self.d_model, actual: cols });
        }
        if input.len() != rows * cols {
            return Err(NetworkError::InvalidInput { expected: rows * cols, actual: input.len() });
        }
        if rows > self.max_tokens {
            return Err(NetworkError::InvalidInput { expected: self.max_tokens, actual: rows });
        }
        let valid_bytes: Option<Vec<u8>> = match layout.valid {
            Some(v) if v.len() != rows => return Err(NetworkError::InvalidInput { expected: rows, actual: v.len() }),
            Some(v) => Some(v.iter().map(|&b| b as u8).collect()),
            None => None,
        };
        let valid_ptr = valid_bytes.as_ref().map_or(ptr::null(), |v| v.as_ptr());
        let ctx = self.device.raw();
        let mut out = vec![0.0f32; rows * self.d_model];
        check(unsafe {
            sys::rbmoe_forward_host(self.layer, input.as_ptr() as *const c_void, rows as i32, cols as i32, valid_ptr,
                                    ptr::null(), ptr::null(), out.as_mut_ptr() as *mut c_void)
        }, ctx, self.d_model, cols)?;

        let (e, k) = (self.config.num_experts, self.config.experts_per_token);
        let slots = rows * k;
        let mut expert_of = vec![0i32; slots];
        let mut gate_of = vec![0f32; slots];
        let mut counts = vec![0i32; e];
        let mut offsets = vec![0i32; e + 1];
        let mut perm_slot = vec![0i32; slots];
        let mut perm_token = vec![0i32; slots];
        let mut probabilities = vec![0f32; rows * e];
        let mut log_sum_exp = vec![0f32; rows];
        let mut routing = sys::rbmoe_routing {
            expert_of: expert_of.as_mut_ptr(),
            gate_of: gate_of.as_mut_ptr(),
            counts: counts.as_mut_ptr(),
            offsets: offsets.as_mut_ptr(),
            perm_slot: perm_slot.as_mut_ptr(),
            perm_token: perm_token.as_mut_ptr(),
            probabilities: probabilities.as_mut_ptr(),
            log_sum_exp: log_sum_exp.as_mut_ptr(),
        };
        check(unsafe { sys::rbmoe_get_routing(self.layer, &mut routing) }, ctx, 0, 0)?;
        let (mut aux_loss, mut z_loss) = (0f32, 0f32);
        check(unsafe { sys::rbmoe_get_losses(self.layer, &mut aux_loss, &mut z_loss) }, ctx, 0, 0)?;

        let assignments = expert_of.iter().zip(&gate_of)
            .map(|(&x, &g)| (if x < 0 { UNROUTED } else { x as usize }, g))
            .collect();
        let group = |table: &[i32]| -> Vec<Vec<usize>> {
            (0..e).map(|x| table[offsets[x] as usize..offsets[x + 1] as usize].iter().map(|&v| v as usize).collect())
                .collect()
        };
        let valid_tokens = layout.valid.map_or(rows, |v| v.iter().filter(|&&b| b).count());
        let cache = MoeCache {
            probabilities,
            log_sum_exp,
            assignments,
            valid_tokens,
            expert_tokens: group(&perm_token),
            expert_slots: group(&perm_slot),
            aux_loss,
            z_loss,
        };
        Ok((out, cache))
    }
}
