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
        /// Binds the decoder stack `execute_batch` runs (what `optimize_model` does once a model's weights are in it).
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
    use bitnet_quant::quantization::weights::QuantizedWeight;
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
        fn optimize_model(&mut self, model: &Model) -> bitnet_inference::Result<()> {
            let _ = model;
            // the weights reach the device through bind_decoder (the loader that fills a HipDecoder from a Model is the
            // GGUF path's job); the trait call only confirms that a model is bound
            if self.capabilities().map(|c| c.max_batch_size).unwrap_or(0) == 0 {
                return Err(bitnet_inference::InferenceError::backend("no decoder bound: call bind_decoder first"));
            }
            Ok(())
        }
        fn get_memory_usage(&self) -> usize { HipInferenceBackend::get_memory_usage(self) }
        fn capabilities(&self) -> BackendCapabilities {
            let c = HipInferenceBackend::capabilities(self).ok();
            BackendCapabilities {
                supports_batching: true,
                supports_streaming: false,
                max_batch_size: c.as_ref().map_or(0, |c| c.max_batch_size),
                memory_limit: c.as_ref().and_then(|c| c.memory_limit),
                device_type: bitnet_inference::Device::Cpu,  // the reference's Device enum has no HIP variant; tensors cross as host memory
            }
        }
    }
}
