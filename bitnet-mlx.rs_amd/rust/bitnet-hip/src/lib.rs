//! bitnet-hip: safe wrappers over the C ABI, shaped like the types they stand in for.
//!
//! * `HipBitLinear` keeps the surface of `bitnet_quant::bitlinear::{BitLinear, BitLinearForward}`
//!   (bitnet-quant/src/bitlinear/layer.rs:113-179,299-352; forward.rs:14-51): `new(config, name)`,
//!   `forward`, `forward_batch`, `update_weights`, `update_bias`.
//! * `HipBackend::w2a8_gemv` keeps the signature of `CudaBackend::w2a8_gemv`
//!   (bitnet-cuda/src/backend.rs:129-157).
//! * `HipError` carries the same variants call sites already match on (`ShapeMismatch{expected, actual}`, ...).
//!
//! Tensors cross this boundary as `DeviceTensor`: a device pointer plus dims, which is what a candle
//! tensor on a HIP device, or any allocator the host runtime uses, can hand out.
pub mod ffi;

use std::ffi::CStr;
use std::os::raw::{c_int, c_void};
use std::ptr;

#[derive(thiserror::Error, Debug)]
pub enum HipError {
    #[error("HIP feature not enabled - compile with --features hip")]
    HipNotEnabled,
    #[error("Shape mismatch: expected {expected:?}, got {actual:?}")]
    ShapeMismatch { expected: Vec<usize>, actual: Vec<usize> },
    #[error("Configuration error: {0}")]
    ConfigError(String),
    #[error("Device operation error: {0}")]
    DeviceError(String),
    #[error("Memory management error: {0}")]
    MemoryError(String),
    #[error("Quantization failed: {0}")]
    QuantizationError(String),
    #[error("Layer not initialized: {0}")]
    NotInitialized(String),
    #[error("HIP kernel execution failed: {0}")]
    KernelExecution(String),
    #[error("Unsupported HIP operation: {0}")]
    UnsupportedOperation(String),
}
pub type HipResult<T> = Result<T, HipError>;

fn check(status: c_int) -> HipResult<()> {
    if status == ffi::BITNET_HIP_OK {
        return Ok(());
    }
    let msg = unsafe { CStr::from_ptr(ffi::bitnet_hip_last_error()) }.to_string_lossy().into_owned();
    Err(match status {
        ffi::BITNET_HIP_SHAPE_MISMATCH => {
            let (mut e, mut a, mut ar) = ([0usize; 4], [0usize; 4], 0 as c_int);
            let er = unsafe { ffi::bitnet_hip_last_shape_mismatch(e.as_mut_ptr(), a.as_mut_ptr(), &mut ar) };
            HipError::ShapeMismatch { expected: e[..er as usize].to_vec(), actual: a[..ar as usize].to_vec() }
        }
        ffi::BITNET_HIP_INVALID_CONFIG | ffi::BITNET_HIP_NULL_POINTER => HipError::ConfigError(msg),
        ffi::BITNET_HIP_MEMORY_ERROR => HipError::MemoryError(msg),
        ffi::BITNET_HIP_QUANTIZATION_ERROR => HipError::QuantizationError(msg),
        ffi::BITNET_HIP_NOT_INITIALIZED => HipError::NotInitialized(msg),
        ffi::BITNET_HIP_KERNEL_ERROR => HipError::KernelExecution(msg),
        ffi::BITNET_HIP_UNSUPPORTED => HipError::UnsupportedOperation(msg),
        _ => HipError::DeviceError(msg),
    })
}

/// A dense row-major f32 tensor living in device memory that the caller owns.
pub struct DeviceTensor {
    pub ptr: *mut f32,
    pub dims: Vec<usize>,
}

/// The arithmetic-relevant part of `BitLinearConfig` (layer.rs:20-75).
#[derive(Debug, Clone)]
pub struct BitLinearConfig {
    pub in_features: usize,
    pub out_features: usize,
    pub use_bias: bool,
    pub ternary_method: c_int,
    pub threshold_factor: f32,
    pub rms_norm_eps: f32,
}
impl Default for BitLinearConfig {
    fn default() -> Self {
        Self { in_features: 512, out_features: 512, use_bias: false,
               ternary_method: ffi::BITNET_HIP_TERNARY_ABSMEAN_ROUNDCLIP, threshold_factor: 0.5, rms_norm_eps: 1e-5 }
    }
}

pub struct HipBitLinear {
    config: BitLinearConfig,
    layer_name: String,
    handle: *mut ffi::bitnet_hip_bitlinear,
    stream: *mut c_void,
}
// The C side guards weights with a reader/writer lock, as the reference's Arc<RwLock<Tensor>> does.
unsafe impl Send for HipBitLinear {}
unsafe impl Sync for HipBitLinear {}

impl HipBitLinear {
    pub fn new(config: BitLinearConfig, layer_name: String) -> HipResult<Self> {
        if cfg!(not(feature = "hip")) {
            return Err(HipError::HipNotEnabled);
        }
        let mut handle = ptr::null_mut();
        check(unsafe {
            ffi::bitnet_hip_bitlinear_create(config.in_features, config.out_features, config.use_bias as c_int, &mut handle)
        })?;
        Ok(Self { config, layer_name, handle, stream: ptr::null_mut() })
    }
    pub fn config(&self) -> &BitLinearConfig { &self.config }
    pub fn layer_name(&self) -> &str { &self.layer_name }

    /// `BitLinear::update_weights`: latent f32 weights [out, in] in host memory.
    pub fn update_weights(&self, weights: &[f32], rows: usize, cols: usize) -> HipResult<()> {
        check(unsafe {
            ffi::bitnet_hip_bitlinear_set_weights_f32(self.handle, weights.as_ptr(), rows, cols,
                ffi::BITNET_HIP_LAYOUT_OUT_IN, 0, self.config.ternary_method, self.config.threshold_factor, self.stream)
        })
    }
    pub fn update_bias(&self, bias: &[f32]) -> HipResult<()> {
        check(unsafe { ffi::bitnet_hip_bitlinear_set_bias(self.handle, bias.as_ptr(), bias.len(), 0, self.stream) })
    }
    /// `BitLinearForward::forward`: input [.., in_features] -> output [.., out_features] (caller-allocated).
    pub fn forward(&self, input: &DeviceTensor, output: &mut DeviceTensor) -> HipResult<()> {
        check(unsafe {
            ffi::bitnet_hip_bitlinear_forward(self.handle, input.ptr, input.dims.as_ptr(), input.dims.len() as c_int,
                ptr::null(), self.config.rms_norm_eps, ffi::BITNET_HIP_SUM_BLOCK256, ptr::null(), output.ptr,
                ptr::null_mut(), 0, ptr::null_mut(), ptr::null_mut(), ptr::null_mut(), self.stream)
        })
    }
    pub fn forward_batch(&self, inputs: &DeviceTensor, output: &mut DeviceTensor) -> HipResult<()> {
        if inputs.dims.len() < 2 {
            return Err(HipError::ShapeMismatch { expected: vec![1, 1, self.config.in_features], actual: inputs.dims.clone() });
        }
        self.forward(inputs, output)
    }
}
impl Drop for HipBitLinear {
    fn drop(&mut self) {
        unsafe { ffi::bitnet_hip_bitlinear_destroy(self.handle) }
    }
}

/// Stand-in for `CudaBackend` (bitnet-cuda/src/backend.rs).
pub struct HipBackend {
    stream: *mut c_void,
}
impl HipBackend {
    pub fn new(device: i32) -> HipResult<Self> {
        if cfg!(not(feature = "hip")) {
            return Err(HipError::HipNotEnabled);
        }
        check(unsafe { ffi::bitnet_hip_init(device) })?;
        Ok(Self { stream: ptr::null_mut() })
    }
    /// Same arguments as `CudaBackend::w2a8_gemv`; the three buffers are device slices (pointer, length).
    pub fn w2a8_gemv(&self, weights: (*const u8, usize), activations: (*const i8, usize), output: (*mut i32, usize),
                     m: usize, k: usize) -> HipResult<()> {
        check(unsafe {
            ffi::bitnet_hip_gemv_w2a8_checked(weights.0, weights.1, activations.0, activations.1, output.0, output.1,
                                              m, k, self.stream)
        })
    }
}

/// Device-side stand-in for the kernels `KernelSelector` hands out (bitnet-core/src/cpu/mod.rs:107-127): the
/// arithmetic of `TernaryLookupKernel::compute` / `I2SLookupKernel::compute` (bitnet-core/src/cpu/mod.rs:132-169,
/// kernels/generic.rs:54-75,118-139) on device slices (pointer, length).  A crate that owns the trait definitions
/// implements them for this type by staging its host slices through device buffers.
pub struct HipLookupKernel {
    kind: c_int,
    stream: *mut c_void,
}
impl HipLookupKernel {
    pub fn ternary() -> Self { Self { kind: ffi::BITNET_HIP_LOOKUP_TERNARY, stream: ptr::null_mut() } }
    pub fn i2s() -> Self { Self { kind: ffi::BITNET_HIP_LOOKUP_I2S, stream: ptr::null_mut() } }
    /// `output[i] = inputs[i] * lut[weights[i]]` over the shortest of the three; an empty slice is an error.
    pub fn compute(&self, weights: (*const i8, usize), inputs: (*const f32, usize), output: (*mut f32, usize)) -> HipResult<()> {
        check(unsafe {
            ffi::bitnet_hip_lookup_compute(self.kind, weights.0, weights.1, inputs.0, inputs.1, output.0, output.1, self.stream)
        })
    }
    pub fn name(&self) -> &'static str {
        if self.kind == ffi::BITNET_HIP_LOOKUP_TERNARY { "HIP-gfx950-Ternary" } else { "HIP-gfx950-I2S" }
    }
    pub fn optimal_batch_size(&self) -> usize { 1 << 20 }
}
