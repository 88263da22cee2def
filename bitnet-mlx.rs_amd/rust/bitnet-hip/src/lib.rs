//! bitnet-hip: safe wrappers over the C ABI of the MI355X (gfx950) BitLinear path, shaped like the types they
//! stand in for, and the implementations of the reference's traits for them.
//!
//! * `HipBitLinear` keeps the surface of `bitnet_quant::bitlinear::{BitLinear, BitLinearForward}`
//!   (bitnet-quant/src/bitlinear/layer.rs:113-179,299-352; forward.rs:14-51): `new(config, name)`, `forward`,
//!   `forward_with_quantized_weights`, `forward_batch`, `update_weights`, `update_bias`.
//! * `HipBackend::w2a8_gemv` keeps the signature of `CudaBackend::w2a8_gemv` (bitnet-cuda/src/backend.rs:129-157).
//! * `HipLookupKernel` implements `TernaryLookupKernel` / `I2SLookupKernel` (bitnet-core/src/cpu/mod.rs:132-169).
//! * `HipInferenceBackend` implements `InferenceBackend` (bitnet-inference/src/engine/mod.rs:126-138).
//! * `HipError` carries the variants call sites already match on (`ShapeMismatch{expected, actual}`, ...).
//!
//! Features: `hip` links the library and enables every call; without it the constructors return
//! `HipError::HipNotEnabled` and no symbol of the library is referenced (the analogue of bitnet-cuda's `cuda`
//! feature).  `reference-traits` (needs `hip`) pulls in bitnet-quant / bitnet-core / bitnet-inference / candle-core
//! and adds the trait implementations; candle tensors live in host memory on this path (candle has no HIP device),
//! so they are staged through device buffers owned by the wrapper objects.
pub mod ffi;

use std::os::raw::{c_int, c_void};
use std::sync::Mutex;

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

/// Order of the f32 sum of squares inside RMSNorm (`BITNET_HIP_SUM_*`).
#[derive(Debug, Clone, Copy, PartialEq, Eq)]
pub enum SumOrder {
    /// one running sum, the literal order of inference_integration.rs:476
    Sequential,
    /// 256 strided partials and butterflies (default)
    Block256,
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
    pub sum_order: SumOrder,
}
impl Default for BitLinearConfig {
    fn default() -> Self {
        Self { in_features: 512, out_features: 512, use_bias: false,
               ternary_method: ffi::BITNET_HIP_TERNARY_ABSMEAN_ROUNDCLIP, threshold_factor: 0.5, rms_norm_eps: 1e-5,
               sum_order: SumOrder::Block256 }
    }
}

#[cfg(feature = "hip")]
mod imp {
    use super::*;
    use std::ffi::CStr;
    use std::marker::PhantomData;
    use std::ptr;

    // the three HIP runtime calls the staging buffers need (libamdhip64 is linked by build.rs)
    extern "C" {
        fn hipMalloc(ptr: *mut *mut c_void, size: usize) -> c_int;
        fn hipFree(ptr: *mut c_void) -> c_int;
        fn hipMemcpy(dst: *mut c_void, src: *const c_void, size: usize, kind: c_int) -> c_int;
    }
    const HIP_MEMCPY_HOST_TO_DEVICE: c_int = 1;
    const HIP_MEMCPY_DEVICE_TO_HOST: c_int = 2;

    pub(crate) fn check(status: c_int) -> HipResult<()> {
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

    /// Device memory owned by this crate: allocated, grown and freed here; never handed out as a raw pointer by
    /// safe code.
    pub struct DeviceBuffer<T> {
        ptr: *mut c_void,
        len: usize,
        _t: PhantomData<T>,
    }
    unsafe impl<T> Send for DeviceBuffer<T> {}
    impl<T: Copy> DeviceBuffer<T> {
        pub fn new(len: usize) -> HipResult<Self> {
            let mut ptr = ptr::null_mut();
            let bytes = len.max(1) * std::mem::size_of::<T>();
            if unsafe { hipMalloc(&mut ptr, bytes) } != 0 {
                return Err(HipError::MemoryError(format!("hipMalloc({bytes}) failed")));
            }
            Ok(Self { ptr, len, _t: PhantomData })
        }
        pub fn len(&self) -> usize { self.len }
        pub fn is_empty(&self) -> bool { self.len == 0 }
        /// Grows to at least `len` elements (contents are not kept).
        pub fn reserve(&mut self, len: usize) -> HipResult<()> {
            if len > self.len {
                *self = Self::new(len)?;
            }
            Ok(())
        }
        pub fn upload(&mut self, host: &[T]) -> HipResult<()> {
            self.reserve(host.len())?;
            let bytes = std::mem::size_of_val(host);
            if bytes != 0 && unsafe { hipMemcpy(self.ptr, host.as_ptr() as *const c_void, bytes, HIP_MEMCPY_HOST_TO_DEVICE) } != 0 {
                return Err(HipError::DeviceError("hipMemcpy (host to device) failed".into()));
            }
            Ok(())
        }
        pub fn download(&self, host: &mut [T]) -> HipResult<()> {
            if host.len() > self.len {
                return Err(HipError::ShapeMismatch { expected: vec![self.len], actual: vec![host.len()] });
            }
            let bytes = std::mem::size_of_val(host);
            if bytes != 0 && unsafe { hipMemcpy(host.as_mut_ptr() as *mut c_void, self.ptr, bytes, HIP_MEMCPY_DEVICE_TO_HOST) } != 0 {
                return Err(HipError::DeviceError("hipMemcpy (device to host) failed".into()));
            }
            Ok(())
        }
        pub(crate) fn as_ptr(&self) -> *mut T { self.ptr as *mut T }
    }
    impl<T> Drop for DeviceBuffer<T> {
        fn drop(&mut self) {
            unsafe { hipFree(self.ptr); }
        }
    }

    /// A dense row-major f32 tensor in device memory that the CALLER owns (a candle tensor on a future HIP device,
    /// an allocation of the host runtime).  Constructing one from a raw pointer is the caller's promise that the
    /// memory holds `dims.iter().product()` floats and outlives the calls it is passed to.
    pub struct DeviceTensor {
        ptr: *mut f32,
        dims: Vec<usize>,
    }
    impl DeviceTensor {
        /// # Safety
        /// `ptr` must be a device pointer to at least `dims.iter().product()` f32 values, valid for as long as this
        /// value is used.
        pub unsafe fn from_raw(ptr: *mut f32, dims: Vec<usize>) -> Self { Self { ptr, dims } }
        pub fn from_buffer(buf: &mut DeviceBuffer<f32>, dims: Vec<usize>) -> HipResult<Self> {
            let need: usize = dims.iter().product();
            if need > buf.len() {
                return Err(HipError::ShapeMismatch { expected: vec![buf.len()], actual: vec![need] });
            }
            Ok(Self { ptr: buf.as_ptr(), dims })
        }
        pub fn dims(&self) -> &[usize] { &self.dims }
        pub fn elem_count(&self) -> usize { self.dims.iter().product() }
    }

    fn sum_order_code(o: SumOrder) -> c_int {
        match o { SumOrder::Sequential => ffi::BITNET_HIP_SUM_SEQUENTIAL, SumOrder::Block256 => ffi::BITNET_HIP_SUM_BLOCK256 }
    }

    pub struct HipBitLinear {
        config: BitLinearConfig,
        layer_name: String,
        handle: *mut ffi::bitnet_hip_bitlinear,
        stream: *mut c_void,
        device: i32,  // the library drives one GPU per process: the ordinal given to `HipBackend::new`, 0 by default
        // scratch for the quantised activations and the staging buffers of the host-tensor entry points: grown on
        // demand, never allocated per call once warm
        scratch: Mutex<Scratch>,
    }
    struct Scratch {
        workspace: DeviceBuffer<u8>,
        input: DeviceBuffer<f32>,
        output: DeviceBuffer<f32>,
    }
    // The C side guards weights with a reader/writer lock, as the reference's Arc<RwLock<Tensor>> does
    // (layer.rs:82-109; `unsafe impl Send + Sync for BitLinear`, layer.rs:427-428).
    unsafe impl Send for HipBitLinear {}
    unsafe impl Sync for HipBitLinear {}

    impl HipBitLinear {
        pub fn new(config: BitLinearConfig, layer_name: String) -> HipResult<Self> {
            let mut handle = ptr::null_mut();
            check(unsafe {
                ffi::bitnet_hip_bitlinear_create(config.in_features, config.out_features, config.use_bias as c_int, &mut handle)
            })?;
            let scratch = Scratch { workspace: DeviceBuffer::new(0)?, input: DeviceBuffer::new(0)?, output: DeviceBuffer::new(0)? };
            Ok(Self { config, layer_name, handle, stream: ptr::null_mut(), device: 0, scratch: Mutex::new(scratch) })
        }
        pub fn config(&self) -> &BitLinearConfig { &self.config }
        pub fn layer_name(&self) -> &str { &self.layer_name }

        /// `BitLinear::update_weights`: latent f32 weights [out, in] in host memory.
        pub fn update_weights(&self, weights: &[f32], rows: usize, cols: usize) -> HipResult<()> {
            if weights.len() != rows * cols {
                return Err(HipError::ShapeMismatch { expected: vec![rows, cols], actual: vec![weights.len()] });
            }
            check(unsafe {
                ffi::bitnet_hip_bitlinear_set_weights_f32(self.handle, weights.as_ptr(), rows, cols,
                    ffi::BITNET_HIP_LAYOUT_OUT_IN, 0, self.config.ternary_method, self.config.threshold_factor, self.stream)
            })
        }
        /// Pre-quantised weights in the reference's 2-bit byte format ([out, in] flat) plus their scale.
        pub fn set_quantized_weights(&self, packed: &[u8], w_scale: f32) -> HipResult<()> {
            check(unsafe {
                ffi::bitnet_hip_bitlinear_set_weights_packed(self.handle, packed.as_ptr(), packed.len(), w_scale, 0, self.stream)
            })
        }
        pub fn update_bias(&self, bias: &[f32]) -> HipResult<()> {
            check(unsafe { ffi::bitnet_hip_bitlinear_set_bias(self.handle, bias.as_ptr(), bias.len(), 0, self.stream) })
        }
        /// `BitLinear::clear_cache` (layer.rs:353-361).  The reference caches the quantised form of its latent f32
        /// weights; this layer holds only the quantised weights (`update_weights` quantises at once), so there is
        /// nothing to clear.
        pub fn clear_cache(&self) -> HipResult<()> {
            Ok(())
        }
        /// `BitLinear::to_device` (layer.rs:376-411): the layer lives on the GPU the library was initialised on; that
        /// device is the reference's same-device no-op, any other ordinal is refused.
        pub fn to_device(&mut self, device: i32) -> HipResult<()> {
            if device == self.device {
                Ok(())
            } else {
                Err(HipError::DeviceError(format!("Failed to move weights to device: {device} (the layer lives on {})", self.device)))
            }
        }
        /// `BitLinear::device` (layer.rs:223): the ordinal of the GPU the layer was created on.
        pub fn device(&self) -> i32 { self.device }

        /// The forward on device tensors: input [.., in_features] -> output [.., out_features]; `gamma` is the RMSNorm
        /// weight [in_features] applied before quantisation, if any.  The output's dims are checked here, so safe code
        /// cannot make the kernels write past it.
        pub fn forward_device(&self, input: &DeviceTensor, gamma: Option<&DeviceTensor>, output: &mut DeviceTensor) -> HipResult<()> {
            let rank = input.dims.len();
            if rank >= 1 && input.dims[rank - 1] == self.config.in_features {
                let mut want = input.dims[..rank - 1].to_vec();
                want.push(self.config.out_features);
                if output.dims != want {
                    return Err(HipError::ShapeMismatch { expected: want, actual: output.dims.clone() });
                }
            }
            if let Some(g) = gamma {
                if g.elem_count() != self.config.in_features {
                    return Err(HipError::ShapeMismatch { expected: vec![self.config.in_features], actual: g.dims.clone() });
                }
            }
            let rows: usize = if rank >= 1 { input.dims[..rank - 1].iter().product() } else { 0 };
            let mut scratch = self.scratch.lock().map_err(|_| HipError::DeviceError("scratch lock poisoned".into()))?;
            let need = unsafe { ffi::bitnet_hip_bitlinear_workspace_size(self.handle, rows) };
            scratch.workspace.reserve(need)?;
            check(unsafe {
                ffi::bitnet_hip_bitlinear_forward(self.handle, input.ptr, input.dims.as_ptr(), rank as c_int,
                    gamma.map_or(ptr::null(), |g| g.ptr as *const f32), self.config.rms_norm_eps,
                    sum_order_code(self.config.sum_order), ptr::null(), output.ptr,
                    scratch.workspace.as_ptr() as *mut c_void, scratch.workspace.len(), ptr::null_mut(), ptr::null_mut(),
                    ptr::null_mut(), self.stream)
            })
        }
        pub fn forward_batch_device(&self, inputs: &DeviceTensor, output: &mut DeviceTensor) -> HipResult<()> {
            if inputs.dims.len() < 2 {
                return Err(HipError::ShapeMismatch { expected: vec![1, 1, self.config.in_features], actual: inputs.dims.clone() });
            }
            self.forward_device(inputs, None, output)
        }

        /// The forward on a host slice shaped `dims`: staged through this layer's device buffers.
        pub fn forward_host(&self, input: &[f32], dims: &[usize]) -> HipResult<(Vec<f32>, Vec<usize>)> {
            let count: usize = dims.iter().product();
            if input.len() != count {
                return Err(HipError::ShapeMismatch { expected: dims.to_vec(), actual: vec![input.len()] });
            }
            let rank = dims.len();
            if rank == 0 || dims[rank - 1] != self.config.in_features {
                return Err(HipError::ShapeMismatch { expected: vec![dims.first().copied().unwrap_or(1), self.config.in_features],
                                                     actual: dims.to_vec() });
            }
            let mut out_dims = dims[..rank - 1].to_vec();
            out_dims.push(self.config.out_features);
            let out_count: usize = out_dims.iter().product();
            let (inp, mut out) = {
                let mut scratch = self.scratch.lock().map_err(|_| HipError::DeviceError("scratch lock poisoned".into()))?;
                scratch.input.upload(input)?;
                scratch.output.reserve(out_count)?;
                (unsafe { DeviceTensor::from_raw(scratch.input.as_ptr(), dims.to_vec()) },
                 unsafe { DeviceTensor::from_raw(scratch.output.as_ptr(), out_dims.clone()) })
            };
            self.forward_device(&inp, None, &mut out)?;
            let mut host = vec![0f32; out_count];
            let scratch = self.scratch.lock().map_err(|_| HipError::DeviceError("scratch lock poisoned".into()))?;
            scratch.output.download(&mut host)?;  // hipMemcpy orders itself behind the null stream's work
            Ok((host, out_dims))
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
            check(unsafe { ffi::bitnet_hip_init(device) })?;
            Ok(Self { stream: ptr::null_mut() })
        }
        /// Same arguments as `CudaBackend::w2a8_gemv`; the three buffers are device slices (pointer, length).
        /// # Safety
        /// The pointers must be device pointers to buffers of the given lengths.
        pub unsafe fn w2a8_gemv(&self, weights: (*const u8, usize), activations: (*const i8, usize), output: (*mut i32, usize),
                                m: usize, k: usize) -> HipResult<()> {
            check(ffi::bitnet_hip_gemv_w2a8_checked(weights.0, weights.1, activations.0, activations.1, output.0, output.1,
                                                    m, k, self.stream))
        }
    }

    /// The kernels `KernelSelector` hands out (bitnet-core/src/cpu/mod.rs:107-127) on the GPU: the arithmetic of
    /// `TernaryLookupKernel::compute` / `I2SLookupKernel::compute` (bitnet-core/src/cpu/mod.rs:132-169,
    /// kernels/generic.rs:54-75,118-139).  `compute` takes host slices and stages them through its own device buffers.
    pub struct HipLookupKernel {
        kind: c_int,
        stream: *mut c_void,
        staging: Mutex<(DeviceBuffer<i8>, DeviceBuffer<f32>, DeviceBuffer<f32>)>,
    }
    unsafe impl Send for HipLookupKernel {}
    unsafe impl Sync for HipLookupKernel {}
    impl HipLookupKernel {
        fn with_kind(kind: c_int) -> HipResult<Self> {
            Ok(Self { kind, stream: ptr::null_mut(),
                      staging: Mutex::new((DeviceBuffer::new(0)?, DeviceBuffer::new(0)?, DeviceBuffer::new(0)?)) })
        }
        pub fn ternary() -> HipResult<Self> { Self::with_kind(ffi::BITNET_HIP_LOOKUP_TERNARY) }
        pub fn i2s() -> HipResult<Self> { Self::with_kind(ffi::BITNET_HIP_LOOKUP_I2S) }
        /// `output[i] = inputs[i] * lut[weights[i]]` over the shortest of the three; an empty slice is an error.
        pub fn compute(&self, weights: &[i8], inputs: &[f32], output: &mut [f32]) -> HipResult<()> {
            let mut st = self.staging.lock().map_err(|_| HipError::DeviceError("staging lock poisoned".into()))?;
            st.0.upload(weights)?;
            st.1.upload(inputs)?;
            st.2.reserve(output.len())?;
            check(unsafe {
                ffi::bitnet_hip_lookup_compute(self.kind, st.0.as_ptr(), weights.len(), st.1.as_ptr(), inputs.len(),
                                               st.2.as_ptr(), output.len(), self.stream)
            })?;
            let n = weights.len().min(inputs.len()).min(output.len());
            st.2.download(&mut output[..n])
        }
        /// The same on device slices (pointer, length).
        /// # Safety
        /// The pointers must be device pointers to buffers of the given lengths.
        pub unsafe fn compute_device(&self, weights: (*const i8, usize), inputs: (*const f32, usize), output: (*mut f32, usize)) -> HipResult<()> {
            check(ffi::bitnet_hip_lookup_compute(self.kind, weights.0, weights.1, inputs.0, inputs.1, output.0, output.1, self.stream))
        }
        pub fn name(&self) -> &'static str {
            if self.kind == ffi::BITNET_HIP_LOOKUP_TERNARY { "HIP-gfx950-Ternary" } else { "HIP-gfx950-I2S" }
        }
        pub fn optimal_batch_size(&self) -> usize { 1 << 20 }
    }

    /// `QuantizationPrecision` values of the per-tensor activation quantisers (`BITNET_HIP_PRECISION_*`).
    #[derive(Debug, Clone, Copy, PartialEq, Eq)]
    pub enum HipPrecision {
        OneFiveFiveBit,
        EightBit,
    }
    impl HipPrecision {
        fn code(self) -> c_int {
            match self {
                HipPrecision::OneFiveFiveBit => ffi::BITNET_HIP_PRECISION_ONE_FIVE_FIVE_BIT,
                HipPrecision::EightBit => ffi::BITNET_HIP_PRECISION_EIGHT_BIT,
            }
        }
        pub fn effective_bit_width(self) -> f32 {
            match self {
                HipPrecision::OneFiveFiveBit => 1.58,
                HipPrecision::EightBit => 8.0,
            }
        }
    }

    /// What `absmax_quantize_activations` / `DynamicActivationQuantizer::quantize` return, in host memory: the signed
    /// values, the one scale of the tensor and the statistics of `QuantizationStats` that the call fills.
    #[derive(Debug, Clone)]
    pub struct HipQuantizedActivation {
        pub values: Vec<i8>,
        pub scale: f32,
        pub original_shape: Vec<usize>,
        pub precision: HipPrecision,
        pub quantization_error: f32,
        pub min_value: f32,
        pub max_value: f32,
        pub sequence_length: Option<usize>,
    }

    /// `absmax_quantize_activations(&Tensor, &Device, Option<QuantizationPrecision>)`
    /// (bitnet-quant/src/quantization/activations.rs:530-641) on the GPU: one scale per tensor.
    pub fn absmax_quantize_activations(activations: &[f32], shape: &[usize], precision: Option<HipPrecision>) -> HipResult<HipQuantizedActivation> {
        let precision = precision.unwrap_or(HipPrecision::OneFiveFiveBit);
        if shape.iter().product::<usize>() != activations.len() {
            return Err(HipError::ShapeMismatch { expected: shape.to_vec(), actual: vec![activations.len()] });
        }
        let mut x = DeviceBuffer::<f32>::new(activations.len())?;
        x.upload(activations)?;
        let q = DeviceBuffer::<i8>::new(activations.len().max(1))?;
        let st = DeviceBuffer::<f32>::new(4)?;
        check(unsafe {
            ffi::bitnet_hip_absmax_quantize_activations(x.as_ptr(), activations.len(), precision.code(), q.as_ptr(), st.as_ptr(), ptr::null_mut())
        })?;
        let mut values = vec![0i8; activations.len()];
        let mut stats = [0f32; 4];
        q.download(&mut values)?;
        st.download(&mut stats)?;
        Ok(HipQuantizedActivation { values, scale: stats[0], original_shape: shape.to_vec(), precision, quantization_error: stats[1],
                                    min_value: stats[2], max_value: stats[3], sequence_length: None })
    }

    /// `ActivationQuantizationConfig` (activations.rs:14-45) with its defaults.
    #[derive(Debug, Clone)]
    pub struct HipActivationQuantizationConfig {
        pub precision: HipPrecision,
        pub moving_average_window: usize,
        pub outlier_percentile: f32,
        pub per_token: bool,
        pub calibration_warmup: usize,
        pub ema_decay: f32,
        pub quantize_attention: bool,
    }
    impl Default for HipActivationQuantizationConfig {
        fn default() -> Self {
            Self { precision: HipPrecision::OneFiveFiveBit, moving_average_window: 100, outlier_percentile: 99.9, per_token: false,
                   calibration_warmup: 50, ema_decay: 0.99, quantize_attention: true }
        }
    }
    impl HipActivationQuantizationConfig {
        /// activations.rs:71-91
        pub fn validate(&self) -> HipResult<()> {
            if self.moving_average_window == 0 {
                return Err(HipError::ConfigError("Moving average window cannot be zero".into()));
            }
            if self.outlier_percentile <= 0.0 || self.outlier_percentile > 100.0 {
                return Err(HipError::ConfigError("Outlier percentile must be in range (0, 100]".into()));
            }
            if self.ema_decay < 0.0 || self.ema_decay > 1.0 {
                return Err(HipError::ConfigError("EMA decay must be in range [0, 1]".into()));
            }
            Ok(())
        }
    }

    /// `DynamicActivationQuantizer` (activations.rs:203-454): the state (moving average of the scale, window of recent
    /// scales, warm-up counter, calibration flag) on the host in `f32`, as the reference keeps it; abs-max and the
    /// quantisation with the current scale on the GPU (`bitnet_hip_abs_max`, `bitnet_hip_quantize_activations_scaled`).
    #[derive(Debug)]
    pub struct HipDynamicActivationQuantizer {
        config: HipActivationQuantizationConfig,
        scale_history: std::collections::VecDeque<f32>,
        ema_scale: Option<f32>,
        calibration_samples: usize,
        calibrated: bool,
        step_count: usize,
    }
    impl HipDynamicActivationQuantizer {
        pub fn new(config: HipActivationQuantizationConfig) -> Self {
            let window = config.moving_average_window;
            Self { config, scale_history: std::collections::VecDeque::with_capacity(window), ema_scale: None, calibration_samples: 0,
                   calibrated: false, step_count: 0 }
        }
        pub fn config(&self) -> &HipActivationQuantizationConfig { &self.config }
        fn device_abs_max(x: &DeviceBuffer<f32>, len: usize) -> HipResult<f32> {
            let mut m = 0f32;
            check(unsafe { ffi::bitnet_hip_abs_max(x.as_ptr(), len, &mut m, ptr::null_mut()) })?;
            Ok(m)
        }
        /// compute_dynamic_scale (:241-267)
        fn compute_dynamic_scale(&mut self, abs_max: f32) -> f32 {
            let current_scale = match self.config.precision {
                HipPrecision::OneFiveFiveBit => abs_max / 1.0,
                HipPrecision::EightBit => abs_max / 127.0,
            };
            self.ema_scale = Some(match self.ema_scale {
                Some(prev) => self.config.ema_decay * prev + (1.0 - self.config.ema_decay) * current_scale,
                None => current_scale,
            });
            if self.scale_history.len() >= self.config.moving_average_window {
                self.scale_history.pop_front();
            }
            self.scale_history.push_back(current_scale);
            self.ema_scale.unwrap()
        }
        fn quantize_buffer(&self, x: &DeviceBuffer<f32>, host: &[f32], shape: &[usize]) -> HipResult<HipQuantizedActivation> {
            if shape.is_empty() {
                return Err(HipError::QuantizationError("Activation tensor must have at least 1 dimension".into()));
            }
            let scale = match self.ema_scale {
                Some(s) => s,
                None => Self::device_abs_max(x, host.len())?,
            };
            let q = DeviceBuffer::<i8>::new(host.len().max(1))?;
            check(unsafe {
                ffi::bitnet_hip_quantize_activations_scaled(x.as_ptr(), host.len(), self.config.precision.code(), scale, 0, q.as_ptr(), ptr::null_mut())
            })?;
            let mut values = vec![0i8; host.len()];
            q.download(&mut values)?;
            Ok(HipQuantizedActivation { values, scale, original_shape: shape.to_vec(), precision: self.config.precision,
                                        quantization_error: 0.0, min_value: 0.0, max_value: 0.0, sequence_length: None })
        }
        fn upload(host: &[f32], shape: &[usize]) -> HipResult<DeviceBuffer<f32>> {
            if shape.iter().product::<usize>() != host.len() {
                return Err(HipError::ShapeMismatch { expected: shape.to_vec(), actual: vec![host.len()] });
            }
            let mut x = DeviceBuffer::<f32>::new(host.len())?;
            x.upload(host)?;
            Ok(x)
        }
        /// quantize (:315-360): the moving-average scale if there is one, else the tensor's own abs-max.
        pub fn quantize(&self, activations: &[f32], shape: &[usize]) -> HipResult<HipQuantizedActivation> {
            let x = Self::upload(activations, shape)?;
            self.quantize_buffer(&x, activations, shape)
        }
        /// quantize_dynamic (:372-383)
        pub fn quantize_dynamic(&mut self, activations: &[f32], shape: &[usize]) -> HipResult<HipQuantizedActivation> {
            self.step_count += 1;
            let x = Self::upload(activations, shape)?;
            let abs_max = Self::device_abs_max(&x, activations.len())?;
            self.update_with_abs_max(abs_max);
            self.quantize_buffer(&x, activations, shape)
        }
        /// quantize_attention (:385-404)
        pub fn quantize_attention(&self, attention_scores: &[f32], shape: &[usize], sequence_length: usize) -> HipResult<HipQuantizedActivation> {
            if !self.config.quantize_attention {
                return Err(HipError::QuantizationError("Attention quantization is disabled".into()));
            }
            let mut result = self.quantize(attention_scores, shape)?;
            result.sequence_length = Some(sequence_length);
            Ok(result)
        }
        /// update_dynamic_params (:406-433) for a tensor whose max |x| is `abs_max`.
        fn update_with_abs_max(&mut self, abs_max: f32) {
            let _scale = self.compute_dynamic_scale(abs_max);
            if self.step_count <= self.config.calibration_warmup {
                if self.calibration_samples < self.config.calibration_warmup {
                    self.calibration_samples += 1;
                }
            } else if !self.calibrated {
                self.calibrated = true;
            }
        }
        pub fn update_dynamic_params(&mut self, activations: &[f32], shape: &[usize]) -> HipResult<()> {
            let x = Self::upload(activations, shape)?;
            let abs_max = Self::device_abs_max(&x, activations.len())?;
            self.update_with_abs_max(abs_max);
            Ok(())
        }
        pub fn get_dynamic_scales(&self) -> f32 { self.ema_scale.unwrap_or(1.0) }
        pub fn reset_dynamic_state(&mut self) {
            self.scale_history.clear();
            self.ema_scale = None;
            self.calibration_samples = 0;
            self.calibrated = false;
            self.step_count = 0;
        }
        /// calibrate (:459-483): the abs-max at index floor(len * outlier_percentile / 100) of the sorted list.
        pub fn calibrate(&mut self, data: &[(&[f32], &[usize])]) -> HipResult<()> {
            if data.is_empty() {
                return Err(HipError::QuantizationError("Calibration data cannot be empty".into()));
            }
            let mut all_scales = Vec::with_capacity(data.len());
            for (host, shape) in data {
                let x = Self::upload(host, shape)?;
                all_scales.push(Self::device_abs_max(&x, host.len())?);
            }
            all_scales.sort_by(|a, b| a.partial_cmp(b).unwrap());
            let percentile_idx = (all_scales.len() as f32 * self.config.outlier_percentile / 100.0) as usize;
            self.ema_scale = Some(all_scales[percentile_idx.min(all_scales.len() - 1)]);
            self.calibrated = true;
            Ok(())
        }
        pub fn needs_calibration(&self) -> bool { !self.calibrated || self.step_count <= self.config.calibration_warmup }
    }

    /// `WeightQuantizationConfig`'s arithmetic-relevant fields (weights.rs:58-95) with their defaults.
    #[derive(Debug, Clone)]
    pub struct HipWeightQuantizationConfig {
        /// TernaryMethod as 0 MeanThreshold, 1 MedianThreshold, 2 AdaptiveThreshold, 3 OptimalThreshold, 4 DetSTE
        pub ternary_method: c_int,
        pub normalize_weights: bool,
        pub outlier_threshold: f32,
        pub custom_threshold_factor: Option<f32>,
    }
    impl Default for HipWeightQuantizationConfig {
        fn default() -> Self {
            Self { ternary_method: 0, normalize_weights: true, outlier_threshold: 3.0, custom_threshold_factor: None }
        }
    }
    /// What `BitNetWeightQuantizer::quantize` returns, in host memory: ternary values, the reference's 2-bit bytes, the
    /// least-squares scale and the twelve statistics of the pipeline (see `bitnet_hip_quantize_weights_reference`).
    #[derive(Debug, Clone)]
    pub struct HipQuantizedWeight {
        pub values: Vec<i8>,
        pub packed: Vec<u8>,
        pub scale: f32,
        pub original_shape: [usize; 2],
        pub stats: [f32; 12],
    }
    /// `BitNetWeightQuantizer` (weights.rs:341-611) on the GPU: normalise, clip, ternarise by the configured method,
    /// least-squares scale.
    #[derive(Debug, Clone, Default)]
    pub struct HipWeightQuantizer {
        config: HipWeightQuantizationConfig,
    }
    impl HipWeightQuantizer {
        pub fn new(config: HipWeightQuantizationConfig) -> Self { Self { config } }
        pub fn config(&self) -> &HipWeightQuantizationConfig { &self.config }
        pub fn quantize(&self, weights: &[f32], rows: usize, cols: usize) -> HipResult<HipQuantizedWeight> {
            if rows * cols != weights.len() {
                return Err(HipError::ShapeMismatch { expected: vec![rows, cols], actual: vec![weights.len()] });
            }
            let mut w = DeviceBuffer::<f32>::new(weights.len())?;
            w.upload(weights)?;
            let n_packed = (weights.len() + 3) / 4;
            let packed = DeviceBuffer::<u8>::new(n_packed.max(1))?;
            let q = DeviceBuffer::<i8>::new(weights.len().max(1))?;
            let scale = DeviceBuffer::<f32>::new(1)?;
            let stats = DeviceBuffer::<f32>::new(12)?;
            check(unsafe {
                ffi::bitnet_hip_quantize_weights_reference(w.as_ptr(), rows, cols, self.config.ternary_method,
                    self.config.normalize_weights as c_int, self.config.outlier_threshold,
                    self.config.custom_threshold_factor.unwrap_or(0.0), packed.as_ptr(), scale.as_ptr(), q.as_ptr(), stats.as_ptr(),
                    ptr::null_mut())
            })?;
            let mut out = HipQuantizedWeight { values: vec![0i8; weights.len()], packed: vec![0u8; n_packed], scale: 0.0,
                                               original_shape: [rows, cols], stats: [0f32; 12] };
            q.download(&mut out.values)?;
            packed.download(&mut out.packed)?;
            let mut s = [0f32; 1];
            scale.download(&mut s)?;
            out.scale = s[0];
            stats.download(&mut out.stats)?;
            Ok(out)
        }
        /// dequantize (weights.rs:613-626): values * scale.
        pub fn dequantize(&self, quantized: &HipQuantizedWeight) -> Vec<f32> {
            quantized.values.iter().map(|v| *v as f32 * quantized.scale).collect()
        }
    }

    /// The seven BitLinear projections of a stack of decoder blocks (bitnet_hip_decoder_*).
    pub struct HipDecoder {
        pub(crate) handle: *mut ffi::bitnet_hip_decoder,
        pub hidden: usize,
        pub max_tokens: usize,
    }
    unsafe impl Send for HipDecoder {}
    unsafe impl Sync for HipDecoder {}
    impl HipDecoder {
        #[allow(clippy::too_many_arguments)]
        pub fn new(layers: usize, hidden: usize, ffn: usize, q_heads: usize, kv_heads: usize, head_dim: usize, eps: f32,
                   sum_order: SumOrder, max_tokens: usize) -> HipResult<Self> {
            let mut handle = ptr::null_mut();
            check(unsafe {
                ffi::bitnet_hip_decoder_create(layers, hidden, ffn, q_heads, kv_heads, head_dim, eps, sum_order_code(sum_order),
                                               max_tokens, &mut handle)
            })?;
            Ok(Self { handle, hidden, max_tokens })
        }
        /// Pre-quantised weights of projection `proj` (BITNET_HIP_PROJ_*) of block `layer`.
        pub fn set_projection_packed(&self, layer: usize, proj: c_int, packed: &[u8], w_scale: f32) -> HipResult<()> {
            let mut bl = ptr::null_mut();
            check(unsafe { ffi::bitnet_hip_decoder_projection(self.handle, layer, proj, &mut bl) })?;
            check(unsafe { ffi::bitnet_hip_bitlinear_set_weights_packed(bl, packed.as_ptr(), packed.len(), w_scale, 0, ptr::null_mut()) })
        }
        /// A whole GGUF tensor of type BitnetB158 (8-byte scale / offset header + 2-bit codes; gguf.rs:1089-1165) as the
        /// weights of projection `proj` of block `layer`; `transposed`: the tensor is [in, out] (inference_integration.rs:431).
        pub fn set_projection_gguf(&self, layer: usize, proj: c_int, data: &[u8], rows: usize, cols: usize, transposed: bool) -> HipResult<()> {
            let mut bl = ptr::null_mut();
            check(unsafe { ffi::bitnet_hip_decoder_projection(self.handle, layer, proj, &mut bl) })?;
            let layout = if transposed { ffi::BITNET_HIP_LAYOUT_IN_OUT } else { ffi::BITNET_HIP_LAYOUT_OUT_IN };
            check(unsafe {
                ffi::bitnet_hip_bitlinear_set_weights_gguf(bl, data.as_ptr(), data.len(), rows, cols, layout, 0, ptr::null_mut(), ptr::null_mut(),
                                                           ptr::null_mut())
            })
        }
        /// Row groups a step of several token rows is split into, each a chain of launches on its own stream
        /// (0 and 1 = one chain, the default).
        pub fn set_chains(&self, chains: usize) -> HipResult<()> {
            check(unsafe { ffi::bitnet_hip_decoder_set_chains(self.handle, chains) })
        }
        pub fn set_norm(&self, layer: usize, which: c_int, gamma: &[f32]) -> HipResult<()> {
            if gamma.len() != self.hidden {
                return Err(HipError::ShapeMismatch { expected: vec![self.hidden], actual: vec![gamma.len()] });
            }
            check(unsafe { ffi::bitnet_hip_decoder_set_norm(self.handle, layer, which, gamma.as_ptr(), 0, ptr::null_mut()) })
        }
    }
    impl Drop for HipDecoder {
        fn drop(&mut self) {
            unsafe { ffi::bitnet_hip_decoder_destroy(self.handle) }
        }
    }

    /// A decode step of a `HipDecoder` recorded as a HIP graph (bitnet_hip_decoder_graph_*): `replay` enqueues the
    /// whole step with one call.  It borrows the decoder, so it cannot outlive it.
    pub struct HipDecoderGraph<'a> {
        handle: *mut ffi::bitnet_hip_decoder_graph,
        _decoder: std::marker::PhantomData<&'a HipDecoder>,
    }
    impl HipDecoder {
        /// Records the step `x_in [m, hidden] -> x_out [m, hidden]` through blocks `layers.start .. layers.end`.
        /// # Safety
        /// `x_in` and `x_out` are device pointers to `m * hidden` floats that stay valid for the life of the graph.
        pub unsafe fn record(&self, layers: std::ops::Range<usize>, x_in: *const f32, m: usize, x_out: *mut f32)
                             -> HipResult<HipDecoderGraph<'_>> {
            if m > self.max_tokens {
                return Err(HipError::ShapeMismatch { expected: vec![self.max_tokens, self.hidden], actual: vec![m, self.hidden] });
            }
            let mut handle = ptr::null_mut();
            check(ffi::bitnet_hip_decoder_graph_create(self.handle, layers.start, layers.end, x_in, m, x_out, ptr::null_mut(),
                                                       ptr::null_mut(), &mut handle))?;
            Ok(HipDecoderGraph { handle, _decoder: std::marker::PhantomData })
        }
    }
    impl HipDecoderGraph<'_> {
        pub fn replay(&self) -> HipResult<()> {
            check(unsafe { ffi::bitnet_hip_decoder_graph_launch(self.handle, ptr::null_mut()) })
        }
    }
    impl Drop for HipDecoderGraph<'_> {
        fn drop(&mut self) {
            unsafe { ffi::bitnet_hip_decoder_graph_destroy(self.handle) }
        }
    }

    /// `InferenceBackend` for this path (bitnet-inference/src/engine/mod.rs:126-138), selected where
    /// `InferenceEngine::create_backend` selects the CPU / Metal backends (api/mod.rs:426-460).
    pub struct HipInferenceBackend {
        handle: *mut ffi::bitnet_hip_backend,
        model: Option<std::sync::Arc<HipDecoder>>,
        staging: Mutex<(DeviceBuffer<f32>, DeviceBuffer<f32>)>,
    }
    unsafe impl Send for HipInferenceBackend {}
    unsafe impl Sync for HipInferenceBackend {}
    /// `BackendCapabilities` (engine/mod.rs:141-148) with the device as an ordinal.
    #[derive(Debug, Clone)]
    pub struct HipBackendCapabilities {
        pub supports_batching: bool,
        pub supports_streaming: bool,
        pub max_batch_size: usize,
        pub memory_limit: Option<usize>,
        pub device: i32,
    }
    impl HipInferenceBackend {
        pub fn new(device: i32) -> HipResult<Self> {
            let mut handle = ptr::null_mut();
            check(unsafe { ffi::bitnet_hip_backend_create(device, &mut handle) })?;
            Ok(Self { handle, model: None, staging: Mutex::new((DeviceBuffer::new(0)?, DeviceBuffer::new(0)?)) })
        }
        /// The decoder bound by `bind_decoder` / `optimize_model`, if any.
        pub fn bound_decoder(&self) -> Option<&std::sync::Arc<HipDecoder>> { self.model.as_ref() }
        /// Binds the decoder stack `execute_batch` runs (what `optimize_model` does for the stack it builds from a `Model`).
        pub fn bind_decoder(&mut self, model: std::sync::Arc<HipDecoder>) -> HipResult<()> {
            check(unsafe { ffi::bitnet_hip_backend_optimize_model(self.handle, model.handle) })?;
            self.model = Some(model);
            Ok(())
        }
        /// Each input is a host matrix [rows, hidden] (row-major); returns the hidden states after the stack.
        pub fn execute_batch_host(&self, inputs: &[(&[f32], usize)]) -> HipResult<Vec<Vec<f32>>> {
            let model = self.model.as_ref().ok_or_else(|| HipError::NotInitialized("no model bound".into()))?;
            let hidden = model.hidden;
            let total: usize = inputs.iter().map(|(d, _)| d.len()).sum();
            let mut st = self.staging.lock().map_err(|_| HipError::DeviceError("staging lock poisoned".into()))?;
            let mut flat = Vec::with_capacity(total);
            for (data, rows) in inputs {
                if data.len() != rows * hidden {
                    return Err(HipError::ShapeMismatch { expected: vec![*rows, hidden], actual: vec![data.len()] });
                }
                flat.extend_from_slice(data);
            }
            st.0.upload(&flat)?;
            st.1.reserve(total)?;
            let (mut ins, mut outs, mut rows_v, mut at) = (Vec::new(), Vec::new(), Vec::new(), 0usize);
            for (data, rows) in inputs {
                ins.push(unsafe { st.0.as_ptr().add(at) } as *const f32);
                outs.push(unsafe { st.1.as_ptr().add(at) });
                rows_v.push(*rows);
                at += data.len();
            }
            check(unsafe {
                ffi::bitnet_hip_backend_execute_batch(self.handle, ins.as_ptr(), rows_v.as_ptr(), inputs.len(), outs.as_ptr(), ptr::null_mut())
            })?;
            let mut host = vec![0f32; total];
            st.1.download(&mut host)?;
            let mut result = Vec::with_capacity(inputs.len());
            let mut at = 0usize;
            for (data, _) in inputs {
                result.push(host[at..at + data.len()].to_vec());
                at += data.len();
            }
            Ok(result)
        }
        pub fn get_memory_usage(&self) -> usize { unsafe { ffi::bitnet_hip_backend_get_memory_usage(self.handle) } }
        pub fn capabilities(&self) -> HipResult<HipBackendCapabilities> {
            let (mut sb, mut ss, mut dev) = (0 as c_int, 0 as c_int, 0 as c_int);
            let (mut mb, mut ml) = (0usize, 0usize);
            check(unsafe { ffi::bitnet_hip_backend_capabilities(self.handle, &mut sb, &mut ss, &mut mb, &mut ml, &mut dev) })?;
            Ok(HipBackendCapabilities { supports_batching: sb != 0, supports_streaming: ss != 0, max_batch_size: mb,
                                        memory_limit: if ml == 0 { None } else { Some(ml) }, device: dev })
        }
    }
    impl Drop for HipInferenceBackend {
        fn drop(&mut self) {
            unsafe { ffi::bitnet_hip_backend_destroy(self.handle) }
        }
    }
}
#[cfg(feature = "hip")]
pub use imp::*;

/// Without the `hip` feature nothing of the library is linked: constructing any of the types fails the way
/// bitnet-cuda fails without its `cuda` feature (`CudaError::CudaNotEnabled`).
#[cfg(not(feature = "hip"))]
mod disabled {
    use super::*;
    pub struct HipBitLinear { _never: std::convert::Infallible }
    impl HipBitLinear {
        pub fn new(_config: BitLinearConfig, _layer_name: String) -> HipResult<Self> { Err(HipError::HipNotEnabled) }
    }
    pub struct HipBackend { _never: std::convert::Infallible }
    impl HipBackend {
        pub fn new(_device: i32) -> HipResult<Self> { Err(HipError::HipNotEnabled) }
    }
    pub struct HipLookupKernel { _never: std::convert::Infallible }
    impl HipLookupKernel {
        pub fn ternary() -> HipResult<Self> { Err(HipError::HipNotEnabled) }
        pub fn i2s() -> HipResult<Self> { Err(HipError::HipNotEnabled) }
    }
    pub struct HipInferenceBackend { _never: std::convert::Infallible }
    impl HipInferenceBackend {
        pub fn new(_device: i32) -> HipResult<Self> { Err(HipError::HipNotEnabled) }
    }
}
#[cfg(not(feature = "hip"))]
pub use disabled::*;

// Silences "unused" in builds without the feature.
#[allow(dead_code)]
fn _uses(_: Option<Mutex<()>>, _: *mut c_void) {}

/// The reference's traits implemented for the wrappers above.  Candle tensors of the reference live in host memory,
/// so every call stages its operands through the wrapper's device buffers.
#[cfg(all(feature = "hip", feature = "reference-traits"))]
mod reference_traits {
    use super::*;
    use bitnet_core::cpu::{I2SLookupKernel, TernaryLookupKernel};
    use bitnet_inference::engine::{BackendCapabilities, InferenceBackend, Model};
    use bitnet_quant::bitlinear::error::{BitLinearError, BitLinearResult};
    use bitnet_quant::bitlinear::forward::BitLinearForward;
    use bitnet_quant::quantization::activations::{ActivationQuantizationConfig, QuantizedActivation};
    use bitnet_quant::quantization::utils::QuantizationError;
    use bitnet_quant::quantization::weights::{QuantizedWeight, TernaryMethod, WeightQuantizationConfig};
    use bitnet_quant::quantization::{QuantizationPrecision, QuantizationStats, Quantizer};
    use candle_core::{Device, Tensor};

    fn to_bitlinear_error(e: HipError) -> BitLinearError {
        match e {
            HipError::ShapeMismatch { expected, actual } => BitLinearError::ShapeMismatch { expected, actual },
            HipError::MemoryError(m) => BitLinearError::MemoryError(m),
            HipError::QuantizationError(m) => BitLinearError::QuantizationError(m),
            other => BitLinearError::DeviceError(other.to_string()),
        }
    }

    fn host_f32(t: &Tensor) -> BitLinearResult<(Vec<f32>, Vec<usize>)> {
        let dims = t.dims().to_vec();
        let flat = t.flatten_all().and_then(|f| f.to_vec1::<f32>()).map_err(|e| BitLinearError::DeviceError(e.to_string()))?;
        Ok((flat, dims))
    }

    /// 2-bit bytes in the reference's format from ternary values (code = w + 1, element i at bits 2*(i mod 4)).
    fn pack_2bit(values: &[f32]) -> Vec<u8> {
        let mut out = vec![0u8; (values.len() + 3) / 4];
        for (i, v) in values.iter().enumerate() {
            let code = if *v > 0.5 { 2u8 } else if *v < -0.5 { 0u8 } else { 1u8 };
            out[i / 4] |= code << (2 * (i % 4));
        }
        out
    }

    impl BitLinearForward for HipBitLinear {
        fn forward(&self, input: &Tensor) -> BitLinearResult<Tensor> {
            let (flat, dims) = host_f32(input)?;
            let (out, out_dims) = self.forward_host(&flat, &dims).map_err(to_bitlinear_error)?;
            Tensor::from_vec(out, out_dims, &Device::Cpu).map_err(|e| BitLinearError::DeviceError(e.to_string()))
        }

        fn forward_with_quantized_weights(&self, input: &Tensor, quantized_weights: &QuantizedWeight) -> BitLinearResult<Tensor> {
            // the ternary values and the scalar scale of the QuantizedWeight replace the layer's own weights for this call
            let values = quantized_weights.values.to_dtype(candle_core::DType::F32).map_err(|e| BitLinearError::DeviceError(e.to_string()))?;
            let (w, w_dims) = host_f32(&values)?;
            let cfg = self.config();
            if w_dims != [cfg.out_features, cfg.in_features] {
                return Err(BitLinearError::ShapeMismatch { expected: vec![cfg.out_features, cfg.in_features], actual: w_dims });
            }
            let scale = quantized_weights.scales.flatten_all().and_then(|s| s.to_vec1::<f32>())
                .map_err(|e| BitLinearError::DeviceError(e.to_string()))?;
            let scale = *scale.first().ok_or_else(|| BitLinearError::QuantizationError("empty scales".into()))?;
            let temp = HipBitLinear::new(cfg.clone(), format!("{}:quantized", self.layer_name())).map_err(to_bitlinear_error)?;
            temp.set_quantized_weights(&pack_2bit(&w), scale).map_err(to_bitlinear_error)?;
            temp.forward(input)
        }
    }

    impl TernaryLookupKernel for HipLookupKernel {
        fn compute(&self, weights: &[i8], inputs: &[f32], output: &mut [f32]) -> anyhow::Result<()> {
            HipLookupKernel::compute(self, weights, inputs, output).map_err(|e| anyhow::anyhow!(e.to_string()))
        }
        fn name(&self) -> &'static str { HipLookupKernel::name(self) }
        fn optimal_batch_size(&self) -> usize { HipLookupKernel::optimal_batch_size(self) }
    }
    impl I2SLookupKernel for HipLookupKernel {
        fn compute(&self, weights: &[i8], inputs: &[f32], output: &mut [f32]) -> anyhow::Result<()> {
            HipLookupKernel::compute(self, weights, inputs, output).map_err(|e| anyhow::anyhow!(e.to_string()))
        }
        fn name(&self) -> &'static str { HipLookupKernel::name(self) }
        fn optimal_batch_size(&self) -> usize { HipLookupKernel::optimal_batch_size(self) }
    }

    /// The decoder stack a `Model` describes: the BitLinear layers of `ModelArchitecture::BitLinear` in groups of seven
    /// (q, k, v, o, gate, up, down), all hidden -> hidden except k / v (hidden -> kv_heads * head_dim), gate / up
    /// (hidden -> ffn) and down (ffn -> hidden); the RMSNorm layers give eps.
    struct DecoderShape {
        blocks: usize, hidden: usize, ffn: usize, heads: usize, kv_heads: usize, head_dim: usize, eps: f32, max_tokens: usize,
    }
    fn decoder_shape_of(model: &Model) -> HipResult<DecoderShape> {
        use bitnet_inference::engine::{LayerParameters, LayerType, ModelArchitecture};
        let (layers, heads, hidden) = match &model.architecture {
            ModelArchitecture::BitLinear { layers, attention_heads, hidden_dim } => (layers, *attention_heads, *hidden_dim),
            other => return Err(HipError::UnsupportedOperation(format!(
                "optimize_model: only ModelArchitecture::BitLinear maps onto the decoder stack (got {other:?}); bind a decoder with bind_decoder"))),
        };
        let bitlinear: Vec<_> = layers.iter().filter(|l| matches!(l.layer_type, LayerType::BitLinear)).collect();
        if bitlinear.is_empty() || bitlinear.len() % 7 != 0 {
            return Err(HipError::UnsupportedOperation(format!(
                "optimize_model: {} BitLinear layers are not whole blocks of seven projections; bind a decoder with bind_decoder", bitlinear.len())));
        }
        let last = |shape: &Vec<usize>| shape.last().copied().unwrap_or(0);
        let (kv_dim, ffn) = (last(&bitlinear[1].output_shape), last(&bitlinear[4].output_shape));
        let heads = heads.ok_or_else(|| HipError::ConfigError("optimize_model: the architecture names no attention heads".into()))?;
        if heads == 0 || hidden % heads != 0 || kv_dim == 0 || ffn == 0 {
            return Err(HipError::ConfigError(format!("optimize_model: hidden {hidden}, heads {heads}, kv width {kv_dim}, ffn {ffn}")));
        }
        let head_dim = hidden / heads;
        for (i, l) in bitlinear.iter().enumerate() {
            let want = match i % 7 { 1 | 2 => (hidden, kv_dim), 4 | 5 => (hidden, ffn), 6 => (ffn, hidden), _ => (hidden, hidden) };
            if (last(&l.input_shape), last(&l.output_shape)) != want {
                return Err(HipError::ShapeMismatch { expected: vec![want.0, want.1], actual: vec![last(&l.input_shape), last(&l.output_shape)] });
            }
        }
        let eps = layers.iter().find_map(|l| match l.parameters { LayerParameters::RMSNorm { eps } => Some(eps), _ => None }).unwrap_or(1e-5);
        Ok(DecoderShape { blocks: bitlinear.len() / 7, hidden, ffn, heads, kv_heads: kv_dim / head_dim, head_dim, eps, max_tokens: 16 })
    }

    impl HipInferenceBackend {
        /// One projection's weights as the GGUF file holds them (type BitnetB158: scale, offset, 2-bit codes;
        /// `decode_ternary_weights`, gguf.rs:1089-1165), into the decoder `optimize_model` built.  `transposed`: the
        /// tensor is [in, out] (inference_integration.rs:431).
        pub fn load_projection_gguf(&self, block: usize, proj: c_int, data: &[u8], rows: usize, cols: usize, transposed: bool) -> HipResult<()> {
            let model = self.bound_decoder().ok_or_else(|| HipError::NotInitialized("no model bound: call optimize_model first".into()))?;
            model.set_projection_gguf(block, proj, data, rows, cols, transposed)
        }
    }

    fn to_quantization_error(e: HipError) -> QuantizationError {
        match e {
            HipError::ShapeMismatch { expected, actual } => QuantizationError::InvalidInput(format!("expected {expected:?}, got {actual:?}")),
            HipError::ConfigError(m) => QuantizationError::ConfigurationError(m),
            HipError::MemoryError(m) => QuantizationError::MemoryError(m),
            HipError::QuantizationError(m) => QuantizationError::InvalidInput(m),
            HipError::UnsupportedOperation(m) => QuantizationError::UnsupportedPrecision(m),
            other => QuantizationError::DeviceError(other.to_string()),
        }
    }

    /// `BitNetWeightQuantizer` behind the reference's `Quantizer` trait (quantization/mod.rs:96-116): the pipeline runs on
    /// the GPU (`bitnet_hip_quantize_weights_reference`), tensors cross as host memory.
    #[derive(Debug)]
    pub struct HipBitNetWeightQuantizer {
        config: WeightQuantizationConfig,
        inner: HipWeightQuantizer,
        stats: std::sync::Mutex<QuantizationStats>,
    }
    impl HipBitNetWeightQuantizer {
        pub fn new(config: WeightQuantizationConfig) -> Self {
            let method = match config.ternary_method {
                TernaryMethod::MeanThreshold => 0,
                TernaryMethod::MedianThreshold => 1,
                TernaryMethod::AdaptiveThreshold => 2,
                TernaryMethod::OptimalThreshold => 3,
                TernaryMethod::DetSTE => 4,
            };
            let inner = HipWeightQuantizer::new(HipWeightQuantizationConfig { ternary_method: method, normalize_weights: config.normalize_weights,
                outlier_threshold: config.outlier_threshold, custom_threshold_factor: config.custom_threshold_factor });
            Self { config, inner, stats: std::sync::Mutex::new(QuantizationStats::default()) }
        }
    }
    impl Quantizer for HipBitNetWeightQuantizer {
        type Input = Tensor;
        type Output = QuantizedWeight;
        type Config = WeightQuantizationConfig;
        type Error = QuantizationError;

        fn quantize(&self, weights: &Tensor) -> Result<QuantizedWeight, QuantizationError> {
            self.validate_input(weights)?;
            let dims = weights.dims().to_vec();
            let cols = *dims.last().unwrap();
            let rows = dims[..dims.len() - 1].iter().product();
            let flat = weights.to_dtype(candle_core::DType::F32)?.flatten_all()?.to_vec1::<f32>()?;
            let q = self.inner.quantize(&flat, rows, cols).map_err(to_quantization_error)?;
            let values: Vec<f32> = q.values.iter().map(|v| *v as f32).collect();
            let stats = QuantizationStats { elements_count: flat.len(), scale_factor: q.scale, compression_ratio: 32.0 / 1.58,
                                            min_value: q.stats[4], max_value: q.stats[5], ..Default::default() };
            *self.stats.lock().unwrap() = stats.clone();
            Ok(QuantizedWeight::new(Tensor::from_vec(values, dims.clone(), &Device::Cpu)?, Tensor::new(q.scale, &Device::Cpu)?, None,
                                    weights.shape().clone(), candle_core::DType::U8, self.config.clone(), stats))
        }
        fn dequantize(&self, quantized: &QuantizedWeight) -> Result<Tensor, QuantizationError> {
            Ok(quantized.values.broadcast_mul(&quantized.scales)?)
        }
        fn config(&self) -> &WeightQuantizationConfig { &self.config }
        fn validate_input(&self, weights: &Tensor) -> Result<(), QuantizationError> {
            if weights.rank() < 2 {
                return Err(QuantizationError::InvalidInput("Weight tensor must have at least 2 dimensions".to_string()));
            }
            if weights.dtype() != candle_core::DType::F32 && weights.dtype() != candle_core::DType::F16 {
                return Err(QuantizationError::InvalidInput("Weight tensor must be float type".to_string()));
            }
            Ok(())
        }
        fn get_stats(&self) -> QuantizationStats { self.stats.lock().unwrap().clone() }
    }

    /// `DynamicActivationQuantizer` behind the `Quantizer` trait (activations.rs:303-370): `quantize` uses the moving-average
    /// scale held by the wrapped `HipDynamicActivationQuantizer` (or the tensor's own abs-max), on the GPU.
    #[derive(Debug)]
    pub struct HipActivationQuantizerAdapter {
        config: ActivationQuantizationConfig,
        pub inner: HipDynamicActivationQuantizer,
    }
    impl HipActivationQuantizerAdapter {
        pub fn new(config: ActivationQuantizationConfig) -> Result<Self, QuantizationError> {
            let precision = match config.base.precision {
                QuantizationPrecision::OneFiveFiveBit => HipPrecision::OneFiveFiveBit,
                QuantizationPrecision::EightBit => HipPrecision::EightBit,
                other => return Err(QuantizationError::UnsupportedPrecision(format!("{other:?}"))),
            };
            let inner = HipDynamicActivationQuantizer::new(HipActivationQuantizationConfig { precision,
                moving_average_window: config.moving_average_window, outlier_percentile: config.outlier_percentile,
                per_token: config.per_token, calibration_warmup: config.calibration_warmup, ema_decay: config.ema_decay,
                quantize_attention: config.quantize_attention });
            Ok(Self { config, inner })
        }
        /// quantize_dynamic of the ActivationQuantizer trait (activations.rs:372-383)
        pub fn quantize_dynamic(&mut self, activations: &Tensor) -> Result<QuantizedActivation, QuantizationError> {
            self.validate_input(activations)?;
            let dims = activations.dims().to_vec();
            let flat = activations.to_dtype(candle_core::DType::F32)?.flatten_all()?.to_vec1::<f32>()?;
            let q = self.inner.quantize_dynamic(&flat, &dims).map_err(to_quantization_error)?;
            self.wrap(q, activations)
        }
        fn wrap(&self, q: HipQuantizedActivation, activations: &Tensor) -> Result<QuantizedActivation, QuantizationError> {
            let values: Vec<f32> = q.values.iter().map(|v| *v as f32).collect();
            let stats = QuantizationStats { elements_count: values.len(), scale_factor: q.scale,
                                            compression_ratio: 32.0 / q.precision.effective_bit_width(), ..Default::default() };
            Ok(QuantizedActivation::new(Tensor::from_vec(values, q.original_shape.clone(), &Device::Cpu)?, Tensor::new(q.scale, &Device::Cpu)?,
                                        None, activations.shape().clone(), candle_core::DType::U8, self.config.clone(), stats, q.sequence_length))
        }
    }
    impl Quantizer for HipActivationQuantizerAdapter {
        type Input = Tensor;
        type Output = QuantizedActivation;
        type Config = ActivationQuantizationConfig;
        type Error = QuantizationError;

        fn quantize(&self, activations: &Tensor) -> Result<QuantizedActivation, QuantizationError> {
            self.validate_input(activations)?;
            let dims = activations.dims().to_vec();
            let flat = activations.to_dtype(candle_core::DType::F32)?.flatten_all()?.to_vec1::<f32>()?;
            let q = self.inner.quantize(&flat, &dims).map_err(to_quantization_error)?;
            self.wrap(q, activations)
        }
        fn dequantize(&self, quantized: &QuantizedActivation) -> Result<Tensor, QuantizationError> {
            Ok(quantized.values.to_dtype(candle_core::DType::F32)?.broadcast_mul(&quantized.scales)?)
        }
        fn config(&self) -> &ActivationQuantizationConfig { &self.config }
        fn validate_input(&self, activations: &Tensor) -> Result<(), QuantizationError> {
            if activations.rank() < 1 {
                return Err(QuantizationError::InvalidInput("Activation tensor must have at least 1 dimension".to_string()));
            }
            if activations.dtype() != candle_core::DType::F32 && activations.dtype() != candle_core::DType::F16 {
                return Err(QuantizationError::InvalidInput("Activation tensor must be float type".to_string()));
            }
            Ok(())
        }
        fn get_stats(&self) -> QuantizationStats { QuantizationStats::default() }
    }

    impl InferenceBackend for HipInferenceBackend {
        fn execute_batch(&self, inputs: &[Tensor]) -> bitnet_inference::Result<Vec<Tensor>> {
            let mut host = Vec::with_capacity(inputs.len());
            for t in inputs {
                let (flat, dims) = host_f32(t).map_err(|e| bitnet_inference::InferenceError::backend(e.to_string()))?;
                let rows = if dims.len() <= 1 { 1 } else { dims[..dims.len() - 1].iter().product() };
                host.push((flat, rows, dims));
            }
            let views: Vec<(&[f32], usize)> = host.iter().map(|(f, r, _)| (f.as_slice(), *r)).collect();
            let outs = self.execute_batch_host(&views).map_err(|e| bitnet_inference::InferenceError::backend(e.to_string()))?;
            outs.into_iter().zip(host.iter())
                .map(|(o, (_, _, dims))| Tensor::from_vec(o, dims.clone(), &Device::Cpu)
                    .map_err(|e| bitnet_inference::InferenceError::backend(e.to_string())))
                .collect()
        }
        /// Builds the decoder stack the model's architecture describes and binds it, as the CPU backend builds its
        /// computation graph from the same description (cpu_backend.rs:116-160, 253-260).  A `Model` carries no
        /// tensors (engine/mod.rs:191-206): the weights follow through `load_projection_gguf`, one BitnetB158 tensor
        /// per projection, straight from the bytes `GgufLoader` holds (gguf.rs:1089-1165).  A decoder bound earlier
        /// with `bind_decoder` is replaced.
        fn optimize_model(&mut self, model: &Model) -> bitnet_inference::Result<()> {
            let shape = decoder_shape_of(model).map_err(|e| bitnet_inference::InferenceError::backend(e.to_string()))?;
            let decoder = HipDecoder::new(shape.blocks, shape.hidden, shape.ffn, shape.heads, shape.kv_heads, shape.head_dim, shape.eps,
                                          SumOrder::Block256, shape.max_tokens)
                .map_err(|e| bitnet_inference::InferenceError::backend(e.to_string()))?;
            self.bind_decoder(std::sync::Arc::new(decoder)).map_err(|e| bitnet_inference::InferenceError::backend(e.to_string()))
        }
        fn get_memory_usage(&self) -> usize { HipInferenceBackend::get_memory_usage(self) }
        fn capabilities(&self) -> BackendCapabilities {
            let c = HipInferenceBackend::capabilities(self).ok();
            BackendCapabilities {
                supports_batching: true,
                supports_streaming: false,
                max_batch_size: c.as_ref().map_or(0, |c| c.max_batch_size),
                memory_limit: c.as_ref().and_then(|c| c.memory_limit),
                // `Device` here is candle's enum (Cpu, Cuda, Metal; bitnet-core re-exports it): it has no variant for this
                // device and its GPU variants cannot be built without that runtime, so the field names where the trait's
                // tensors live (host memory).  The GPU is `HipInferenceBackend::capabilities()?.device` (an ordinal).
                device_type: bitnet_inference::Device::Cpu,
            }
        }
    }
}
