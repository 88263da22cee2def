/*
 * bitnet_hip.h — C ABI of the MI355X (gfx950) BitLinear W1.58A8 forward path.
 *
 * This is the boundary a Rust `extern "C"` block (or any FFI) binds.  Plain pointers and sizes only.
 * Unless a parameter is marked HOST, every data pointer is a DEVICE pointer owned by the caller, the
 * call is asynchronous on `stream` (a hipStream_t passed as void*, NULL = the null stream), and the
 * caller keeps the buffers alive until the stream has passed the call.
 *
 * Every function returns a bitnet_hip_status.  On failure nothing is launched and a message is kept
 * per thread (bitnet_hip_last_error).  Nothing here aborts or throws.
 *
 * Each entry point cites the reference interface it replaces (paths relative to the root of
 * leizerowicz/bitnet-mlx.rs).
 */
#ifndef BITNET_HIP_H
#define BITNET_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes.  One per error variant of the reference that can occur on this path:
 * BitLinearError (bitnet-quant/src/bitlinear/error.rs:10-84) and CudaError
 * (bitnet-cuda/src/error.rs:7-60). */
typedef enum bitnet_hip_status {
    BITNET_HIP_OK = 0,
    BITNET_HIP_SHAPE_MISMATCH = 1,  /* BitLinearError::ShapeMismatch / CudaError::IncompatibleShapes */
    BITNET_HIP_INVALID_CONFIG = 2,  /* BitLinearError::ConfigError, InvalidConfig / CudaError::InvalidConfig */
    BITNET_HIP_DEVICE_ERROR = 3,    /* BitLinearError::DeviceError / CudaError::DeviceError */
    BITNET_HIP_MEMORY_ERROR = 4,    /* BitLinearError::MemoryError / CudaError::MemoryAllocation */
    BITNET_HIP_QUANTIZATION_ERROR = 5, /* BitLinearError::QuantizationError */
    BITNET_HIP_NOT_INITIALIZED = 6, /* BitLinearError::NotInitialized (weights never set) */
    BITNET_HIP_KERNEL_ERROR = 7,    /* CudaError::KernelExecution */
    BITNET_HIP_NULL_POINTER = 8,    /* a required pointer argument was NULL */
    BITNET_HIP_UNSUPPORTED = 9      /* CudaError::UnsupportedOperation */
} bitnet_hip_status;

/* Order of the f32 sum of squares inside RMSNorm. */
#define BITNET_HIP_SUM_SEQUENTIAL 0 /* one running sum, k ascending: the literal order of
                                       bitnet-inference/src/engine/inference_integration.rs:476 (slow) */
#define BITNET_HIP_SUM_BLOCK256 1   /* 256 lane-strided partials, four 64-lane xor butterflies, then
                                       ((s0+s1)+s2)+s3 (default; one wavefront or one workgroup pass) */

/* Weight matrix orientation handed to set_weights. */
#define BITNET_HIP_LAYOUT_OUT_IN 0 /* [out_features, in_features], bitnet-quant/src/bitlinear/layer.rs:86,122 */
#define BITNET_HIP_LAYOUT_IN_OUT 1 /* [in_features, out_features], bitnet-inference/src/engine/inference_integration.rs:431 */

/* Weight ternarisation recipes (TernaryMethod, bitnet-quant/src/quantization/weights.rs:17-30). */
#define BITNET_HIP_TERNARY_ABSMEAN_ROUNDCLIP 0 /* w_scale = mean|W|, q = RoundClip(W / w_scale, -1, 1):
                                                  BitNet b1.58; RoundClip = quantization/utils.rs:391-393 */
#define BITNET_HIP_TERNARY_MEAN_THRESHOLD 1    /* q = sign(w) * [|w| > factor * mean|w|], scale = mean|W|
                                                  (bitnet-quant/src/simd/ternary.rs:27-41,87-101) */

/* BitNetWeightQuantizer::quantize (weights.rs:568-611) with WeightQuantizationConfig's defaults (normalise, clip
 * at 3.0 mean|w|, :81-95) and one of the five TernaryMethods (:17-30); threshold_factor is then
 * custom_threshold_factor (<= 0: none, the method's own factor).  bitnet_hip_quantize_weights_reference takes the
 * whole configuration. */
#define BITNET_HIP_TERNARY_REF_MEAN_THRESHOLD 2     /* TernaryMethod::MeanThreshold: BitLinear's default (layer.rs:53-63) */
#define BITNET_HIP_TERNARY_REF_MEDIAN_THRESHOLD 3   /* TernaryMethod::MedianThreshold */
#define BITNET_HIP_TERNARY_REF_ADAPTIVE_THRESHOLD 4 /* TernaryMethod::AdaptiveThreshold */
#define BITNET_HIP_TERNARY_REF_OPTIMAL_THRESHOLD 5  /* TernaryMethod::OptimalThreshold */
#define BITNET_HIP_TERNARY_REF_DETSTE 6             /* TernaryMethod::DetSTE */

/* Input transform fused in front of the activation quantiser. */
#define BITNET_HIP_INPUT_PLAIN 0     /* row = x[m, :] */
#define BITNET_HIP_INPUT_RELU2_MUL 1 /* row = x2[m, :] * relu(x[m, :])^2   (x = gate, x2 = up):
                                        bitnet-inference/src/engine/transformer_layers.rs:307-316,605-618 */
#define BITNET_HIP_INPUT_GQA_BROADCAST 2 /* row[h*hd + d] = x[m, (h / group)*hd + d]: one-token attention,
                                            every query head reads its KV group's value head */

/* ---- library ---------------------------------------------------------------------------------- */

/* Message of the last failing call on this thread ("" if none).  Never NULL. */
const char *bitnet_hip_last_error(void);

/* Expected / actual dimensions recorded by the last BITNET_HIP_SHAPE_MISMATCH on this thread
 * (BitLinearError::ShapeMismatch{expected, actual}).  Each array receives up to 4 entries; the
 * return value is the number of valid entries in `expected` (actual_rank likewise). */
int bitnet_hip_last_shape_mismatch(size_t expected[4], size_t actual[4], int *actual_rank);

/* Selects `device`, checks that it is a gfx950 part and prepares per-device state.  Replaces
 * CudaBackend::new + check_device_capabilities (bitnet-cuda/src/backend.rs:42-93,192-213). */
int bitnet_hip_init(int device);

/* Name (gcnArchName), compute-unit count and memory clock of the current device.  HOST outputs. */
int bitnet_hip_device_info(char *arch_name, size_t arch_name_len, int *compute_units, int *clock_mhz,
                           size_t *total_mem_bytes);

/* Diagnostic: the int8 rate, in 10^12 operations per second, that a loop of nothing but v_mfma_i32_16x16x64_i8
 * (operands in registers, two wavefronts per SIMD on every compute unit, about 2.5 ms) sustains on the current
 * device: the practical ceiling of bitnet_hip_gemm_w2a8 there, clock under a matrix load included.
 * random_operands != 0: every lane holds different int8 activations and 2-bit codes 0..2 as weights, as the GEMM's
 * operands are; 0: every byte of both operands is 1.  Allocates a small buffer and waits for the result
 * (tera_ops_per_second is a HOST pointer).  No counterpart in the reference; bench.py reports it beside the
 * prefill rates. */
int bitnet_hip_measure_mfma_i8_rate(int random_operands, double *tera_ops_per_second, void *stream);
/* Diagnostic: microseconds one replay of a recorded chain of `launches` dependent kernel launches takes on the current
 * device (each launch starts when the one before it has finished, as the 120 launches of a batch-1 token step do), the
 * floor a decode step of that many launches cannot go below.  buf == NULL: kernels that do nothing.  Otherwise launch i
 * only reads bytes_per_launch[i % pattern_len] bytes (multiples of 16) of buf, each launch the bytes behind those of
 * the launch before it (buf, 16-byte aligned DEVICE memory, holds at least the sum over all launches), with the
 * non-temporal loads the decode GEMV uses for its weight tiles.  The chain is replayed twice untimed, then `replays`
 * times between two events on `stream`; us_per_replay is a HOST pointer; allocates a few hundred bytes and waits for
 * the result.  No counterpart in the reference; bench.py reports both floors beside the measured token step. */
int bitnet_hip_measure_launch_chain(const void *buf, const size_t *bytes_per_launch, size_t pattern_len,
                                    size_t launches, size_t replays, double *us_per_replay, void *stream);
/* Diagnostic: microseconds one hand-over of a vector costs INSIDE a single launch whose workgroups stay resident (one per
 * compute unit) and pass `values` 32-bit values from step to step through memory: every workgroup produces its share with
 * device-scope stores and must have seen all values of a step before it produces the next (what a persistent decoder
 * would do in place of a kernel boundary).  two_level == 0: every workgroup polls all values; != 0: one workgroup per
 * XCD polls them and republishes them in its XCD's L2, the others poll that copy.  Runs `hops` steps twice (the second run
 * is timed, launch included), checks the final values, and reports whether every wait was met within spin_limit looks
 * (<= 0 or above 100000: 20000; every wait is bounded, and a thread whose wait ran out looks only once from then on, so
 * the kernel ends in any case): *intact = 1 if so, 0 if a wait ran out or a value is wrong (spin_limit = 1 forces that).
 * us_per_hop and intact are HOST pointers; allocates a few hundred KB and waits for the result.  No counterpart in the
 * reference. */
int bitnet_hip_measure_hop(int two_level, size_t values, size_t hops, int spin_limit, double *us_per_hop, int *intact,
                           void *stream);

/* ---- activation side -------------------------------------------------------------------------- */

/* Fused RMSNorm + per-token absmax int8 quantiser (one wavefront per token row).
 *   replaces LayerOperation::rms_normalize (bitnet-inference/src/engine/inference_integration.rs:449-493)
 *   followed by TernaryProcessor::quantize_activations (bitnet-inference/src/engine/ternary_operations.rs:117-172).
 *   x        [m, k] f32, row stride ldx elements
 *   x2       second input for BITNET_HIP_INPUT_RELU2_MUL (same shape/stride), else NULL
 *   gamma    [k] f32 RMSNorm weight, or NULL for no normalisation (plain quantize_activations)
 *   q        [m, k] int8 out;  a_scale [m] f32 out (127/absmax, 1.0 for an all-zero row)
 *   a_sum    [m] int32 out or NULL: sum over k of q[m, k]
 *   y_f32    [m, k] f32 out or NULL: the normalised row before quantisation
 *   gqa_group / head_dim: only for BITNET_HIP_INPUT_GQA_BROADCAST (x is then [m, k / gqa_group]). */
int bitnet_hip_quantize_activations_i8(const float *x, const float *x2, size_t ldx, size_t m, size_t k,
                                       int input_mode, size_t gqa_group, size_t head_dim,
                                       const float *gamma, float eps, int sum_order, int8_t *q,
                                       float *a_scale, int32_t *a_sum, float *y_f32, void *stream);

/* QuantizationPrecision values absmax_quantize_activations supports (bitnet-quant/src/quantization/mod.rs). */
#define BITNET_HIP_PRECISION_ONE_FIVE_FIVE_BIT 0 /* ternary: q = [x/scale > 0.5] - [x/scale < -0.5], scale = abs_max */
#define BITNET_HIP_PRECISION_EIGHT_BIT 1         /* q = round(clamp(x/scale, -127, 127)), scale = abs_max / 127 */

/* One scale for the whole tensor:
 *   replaces absmax_quantize_activations (bitnet-quant/src/quantization/activations.rs:530-641), the body behind
 *   QuantizedActivation / DynamicActivationQuantizer (:95-112,203-454).
 *   x [count] f32 (any shape, flattened);  values [count] int8 out;  stats 4 f32 out (device): scale (abs_max below
 *   f32::EPSILON gives 1.0), quantization_error = mean((x - q*scale)^2), min_value, max_value (QuantizationStats,
 *   :609-626).  Anything but the two precisions above is BITNET_HIP_UNSUPPORTED (UnsupportedPrecision, :603-607).
 *   The reference casts its 8-bit result to U8 (:599), which zeroes every negative value; values stay signed here.
 *   The per-token int8 quantiser of the BitLinear path is bitnet_hip_quantize_activations_i8, not this function. */
int bitnet_hip_absmax_quantize_activations(const float *x, size_t count, int precision, int8_t *values, float *stats,
                                           void *stream);
/* The two device steps of DynamicActivationQuantizer (bitnet-quant/src/quantization/activations.rs:203-454), whose
 * state (exponential moving average of the scale, history window, warm-up counter) lives on the host, where the
 * reference keeps it:
 *   bitnet_hip_abs_max: max |x| over the tensor into *abs_max, a HOST float; waits for the stream, as
 *     activations.abs().max_all().to_scalar() does (compute_dynamic_scale, :241-267; calibrate, :472-475).
 *   bitnet_hip_quantize_activations_scaled: DynamicActivationQuantizer::quantize with the scale given
 *     (quantize_int8 :269-275, quantize_ternary_activation :277-294): y = x * (float)(1.0 / (double)scale);
 *     ternary +1 / -1 beyond +-0.5; 8-bit round(clamp(y, -127, 127)) as int8, or with reference_u8 != 0 the reference's
 *     literal clamp(0, 255).round() stored as the byte of a u8 (it zeroes every negative activation).  NaN gives 0. */
int bitnet_hip_abs_max(const float *x, size_t count, float *abs_max, void *stream);
int bitnet_hip_quantize_activations_scaled(const float *x, size_t count, int precision, float scale, int reference_u8,
                                           int8_t *values, void *stream);

/* ---- lookup-table kernels --------------------------------------------------------------------- */

#define BITNET_HIP_LOOKUP_TERNARY 0 /* weights {-1,0,+1}, anything else counts as 0 */
#define BITNET_HIP_LOOKUP_I2S 1     /* weights {-2,-1,0,+1}, anything else counts as 0 */

/* output[i] = inputs[i] * lut[weights[i]] over min(n_weights, n_inputs, n_output) elements, device buffers.
 * INVALID_CONFIG ("Empty input arrays") when one of the three lengths is 0.
 *   replaces TernaryLookupKernel::compute and I2SLookupKernel::compute (bitnet-core/src/cpu/mod.rs:132-169) as
 *   GenericTernaryKernel / GenericI2SKernel implement them (bitnet-core/src/cpu/kernels/generic.rs:54-75,118-139),
 *   the kernels KernelSelector hands out (bitnet-core/src/cpu/mod.rs:107-127).  Element-wise and memory-bound
 *   (9 bytes per element); it is not on the BitLinear path, which never expands weights to f32. */
int bitnet_hip_lookup_compute(int kind, const int8_t *weights, size_t n_weights, const float *inputs, size_t n_inputs,
                              float *output, size_t n_output, void *stream);

/* ---- weight side ------------------------------------------------------------------------------ */

/* Bytes of `count` ternary values in the reference's 2-bit format: (count + 3) / 4
 * (bitnet-quant/src/quantization/packing.rs:353-376, bitnet-cuda/src/backend.rs:226). */
size_t bitnet_hip_packed_size(size_t count);

/* 2-bit pack / unpack in the reference's byte format: code = w + 1, element i of a byte at bits
 * 2*(i mod 4); decode 0,1,2,3 -> -1,0,+1,0.
 *   replaces BitPacked2BitPacker::{pack,unpack} (bitnet-quant/src/quantization/packing.rs:353-394),
 *   BitUtils::{pack_bits,unpack_bits} (bitnet-quant/src/quantization/utils.rs:434-475) and
 *   WeightConverter::convert_ternary_weights (bitnet-inference/src/engine/weight_conversion.rs:143-191). */
int bitnet_hip_pack_ternary_2bit(const int8_t *q, size_t count, uint8_t *packed, void *stream);
int bitnet_hip_unpack_ternary_2bit(const uint8_t *packed, size_t count, int8_t *q, void *stream);

/* Base-3 pack / unpack, 5 ternary values per byte: byte = sum_{j<5} (w[5b+j] + 1) * 3^j; value j of a byte is
 * (byte / 3^j) % 3 - 1 (bytes above 242 decode by the same divisions).  bitnet_hip_base3_packed_size(count) =
 * (count + 4) / 5 bytes.
 *   replaces Base3PackedPacker::{pack,unpack} (bitnet-quant/src/quantization/packing.rs:424-501). */
size_t bitnet_hip_base3_packed_size(size_t count);
int bitnet_hip_pack_ternary_base3(const int8_t *q, size_t count, uint8_t *packed, void *stream);
int bitnet_hip_unpack_ternary_base3(const uint8_t *packed, size_t count, int8_t *q, void *stream);
/* The decode GEMV on base-3 bytes themselves (1.6 bits per weight, 20 % fewer bytes than the 2-bit codes): one token,
 * acc[n] = sum_k a[k] * w[n, k] in int32, out[n] = (float(acc) * w_scale) / a_scale.
 *   bitnet_hip_retile_base3 re-orders the bytes Base3PackedPacker::pack emits for the flat row-major [n, k] tensor
 *   (packing.rs:421-501; base3 holds (n*k + 4) / 5 bytes) into a streaming layout of bitnet_hip_base3_tiled_size(n, k)
 *   bytes: tiles of 16 rows x 320 columns, a byte = five consecutive columns of one row, weight 0 past the matrix.
 *   bitnet_hip_gemv_base3 contracts that layout with int8 activations a[k]; acc or out may be NULL (out needs w_scale;
 *   a_scale NULL = 1).  All pointers are DEVICE memory.  Semantics as bitnet_hip_gemv_w2a8
 *   (bitnet-quant/src/simd/matrix.rs:471-490).  The kernel is bound by the table look-ups that take a base-3 byte
 *   apart, not by memory: it is slower than the 2-bit GEMV at every size measured and no BitLinear object uses it. */
size_t bitnet_hip_base3_tiled_size(size_t n, size_t k);
int bitnet_hip_retile_base3(const uint8_t *base3, size_t n, size_t k, uint8_t *tiled, void *stream);
int bitnet_hip_gemv_base3(const uint8_t *tiled, const int8_t *a, size_t n, size_t k, const float *w_scale,
                          const float *a_scale, int32_t *acc, float *out, void *stream);

/* Ternarise an f32 weight matrix [n, k] (row-major) and pack it in the reference's byte format.
 *   replaces SimdTernaryOps::{compute_absmean, quantize_batch} (bitnet-quant/src/simd/ternary.rs:27-66)
 *   / BitNetWeightQuantizer::quantize (bitnet-quant/src/quantization/weights.rs:568-611) + the packer.
 *   method   BITNET_HIP_TERNARY_*;  threshold_factor: MEAN_THRESHOLD's factor (reference: 0.5 / 0.7), the custom
 *            factor of the REF_* methods (<= 0: none), unused for ABSMEAN_ROUNDCLIP
 *   packed   [(n*k+3)/4] u8 out;  w_scale  1 f32 out (device);  q_i8 [n*k] int8 out or NULL. */
int bitnet_hip_quantize_weights(const float *w, size_t n, size_t k, int method, float threshold_factor,
                                uint8_t *packed, float *w_scale, int8_t *q_i8, void *stream);

/* The reference's weight pipeline with its whole configuration, on the GPU:
 *   replaces BitNetWeightQuantizer::quantize (bitnet-quant/src/quantization/weights.rs:568-611):
 *   normalize_before_quantize (:671-686, if normalize_weights), handle_outliers (:688-699, if outlier_threshold > 0),
 *   quantize_ternary_with_method (:370-480; ternary_method 0 MeanThreshold, 1 MedianThreshold, 2 AdaptiveThreshold,
 *   3 OptimalThreshold, 4 DetSTE; custom_threshold_factor <= 0 means None), apply_ternary_quantization (:482-496),
 *   compute_ternary_scale (:546-559).  INVALID_CONFIG where WeightQuantizationConfig::validate errs (:120-150).
 *   w [n, k] f32;  packed [(n*k+3)/4] u8 out (codes q + 1);  w_scale 1 f32 out: sum(w''q)/sum(q q);  q_i8 [n*k] or NULL;
 *   stats 12 f32 out or NULL: mean, sd, clip centre, clip mean|.|, lo, hi, mean|w''|, max|w''|, threshold, numerator,
 *   denominator, scale.  Tensor-wide sums are carried in f64 in a fixed order (per row 64 strided partials and a
 *   butterfly, then the rows likewise); the reference sums in f32 in candle-core's order. */
int bitnet_hip_quantize_weights_reference(const float *w, size_t n, size_t k, int ternary_method, int normalize_weights,
                                          float outlier_threshold, float custom_threshold_factor, uint8_t *packed,
                                          float *w_scale, int8_t *q_i8, float *stats, void *stream);

/* Device layout both contraction kernels stream: tiles of 16 rows x 256 columns, 1 KiB each, stored
 * [row_block][k_tile]; inside a tile the 16 bytes at offset 16*(16*kq + r) hold row r's columns
 * 64*t + 16*kq .. +15 in dword t (t = 0..3), bit-interleaved so that (dword >> 2j) & 0x03030303 is the code
 * bytes of columns 4j..4j+3; rows/columns past n/k are zero weights; code 3 is rewritten to
 * code 1 (both decode to 0).  bitnet_hip_tiled_size gives the byte size for an [n, k] matrix.
 * retile/untile are inverse bijections on the n*k valid positions (up to the code 3 -> 1 rewrite). */
size_t bitnet_hip_tiled_size(size_t n, size_t k);
int bitnet_hip_retile_weights(const uint8_t *packed, size_t n, size_t k, int layout, uint8_t *tiled,
                              void *stream);
int bitnet_hip_untile_weights(const uint8_t *tiled, size_t n, size_t k, uint8_t *packed, void *stream);

/* ---- contraction ------------------------------------------------------------------------------ */

/* W2A8 GEMV on the reference's flat row-major packing: out[n] = sum_k w[n,k] * a[k] in int32.
 *   replaces launch_w2a8_gemv_optimized (bitnet-cuda/src/kernels/w2a8_gemv.cu:188-214) and
 *   CudaBackend::w2a8_gemv + validate_w2a8_dimensions (bitnet-cuda/src/backend.rs:129-157,217-257).
 *   weights [(m*k+3)/4] u8, activations [k] i8, output [m] i32; m = output features, k = input features
 *   (the reference's naming).  The *_checked form also takes the element counts of the three buffers
 *   and returns BITNET_HIP_SHAPE_MISMATCH exactly where validate_w2a8_dimensions errs.
 *   Code 3 (which no packer of the reference emits) counts as weight 0, as every Rust decoder of the reference
 *   decodes it (weight_conversion.rs:175-181, gguf.rs:1130-1141); the CUDA kernel this call replaces clamps
 *   code 3 - 1 = 2 to +1 instead (w2a8_gemv.cu:32-41).  The two differ only on bytes holding code 3. */
int bitnet_hip_gemv_w2a8(const uint8_t *weights, const int8_t *activations, int32_t *output, size_t m,
                         size_t k, void *stream);
int bitnet_hip_gemv_w2a8_checked(const uint8_t *weights, size_t weights_len, const int8_t *activations,
                                 size_t activations_len, int32_t *output, size_t output_len, size_t m,
                                 size_t k, void *stream);

/* BitLinear contraction + epilogue on re-tiled weights, any token count m:
 *   acc[t, n] = sum_k a[t, k] * w[n, k]                          (int32, exact)
 *   out[t, n] = (float(acc) * *w_scale) / a_scale[t] (+ bias[n]) (+ residual[t, n])
 *   replaces SimdMatrixOps::{ternary_gemv_scalar, ternary_gemm_scalar}
 *   (bitnet-quant/src/simd/matrix.rs:471-490, :256-282), BitLinear::quantized_matmul
 *   (bitnet-quant/src/bitlinear/forward.rs:153-223) and TernaryProcessor::ternary_matmul
 *   (bitnet-inference/src/engine/ternary_operations.rs:87-113,283-338).
 *   Small m runs the HBM-bound decode GEMV, large m the int8 MFMA GEMM.
 *   a_sum [m] int32 = sum over k of a[t, k], as bitnet_hip_quantize_activations_i8 returns it; may be NULL
 *   (the kernels then compute it; the fastest GEMM kernel needs it supplied).
 *   acc / out may each be NULL (at least one must be given); out needs w_scale and a_scale. */
int bitnet_hip_matmul_w2a8(const uint8_t *tiled, const int8_t *a, const int32_t *a_sum, size_t m, size_t n,
                           size_t k, int32_t *acc, const float *w_scale, const float *a_scale,
                           const float *bias, const float *residual, float *out, void *stream);

/* ---- BitLinear layer object ------------------------------------------------------------------- */

typedef struct bitnet_hip_bitlinear bitnet_hip_bitlinear; /* opaque; mirrors BitLinear, layer.rs:82-109 */

/* BitLinear::new(BitLinearConfig{in_features,out_features,use_bias,..}) (layer.rs:113-179).  The layer
 * holds no weights until one of the set_weights calls (forward then returns NOT_INITIALIZED). */
int bitnet_hip_bitlinear_create(size_t in_features, size_t out_features, int use_bias,
                                bitnet_hip_bitlinear **layer);
void bitnet_hip_bitlinear_destroy(bitnet_hip_bitlinear *layer);

/* BitLinear::update_weights (layer.rs:299-326) + get_quantized_weights (layer.rs:236-294): takes the
 * latent f32 matrix (`layout` orientation; HOST pointer if on_device == 0), ternarises it with `method`
 * on the GPU, packs and re-tiles it.  `rows`/`cols` are checked against the layer's shape. */
int bitnet_hip_bitlinear_set_weights_f32(bitnet_hip_bitlinear *layer, const float *w, size_t rows,
                                         size_t cols, int layout, int on_device, int method,
                                         float threshold_factor, void *stream);
/* Pre-quantised weights in the reference's 2-bit byte format ([out,in] flat), plus their scale:
 * BitLinearForward::forward_with_quantized_weights (forward.rs:46-50) / GGUF-decoded tensors. */
int bitnet_hip_bitlinear_set_weights_packed(bitnet_hip_bitlinear *layer, const uint8_t *packed,
                                            size_t packed_len, float w_scale, int on_device, void *stream);
/* A GGUF tensor of type BitnetB158 as GgufLoader::decode_ternary_weights reads it (bitnet-inference/src/gguf.rs:
 * 1089-1165): 4 bytes scale (f32, little endian), 4 bytes offset (f32, little endian), then the 2-bit codes, 4 per
 * byte, flat over a rows x cols matrix in `layout` orientation (BITNET_HIP_LAYOUT_IN_OUT for the transposed
 * tensors of inference_integration.rs:431).  `data` is a HOST pointer (if on_device == 0) to the whole tensor,
 * header included.  The header's scale becomes the layer's w_scale; scale and offset are also returned through
 * scale_out / offset_out (either may be NULL).  Unlike the reference, which accepts any buffer of at least
 * ceil(rows*cols/4) bytes and then silently decodes fewer elements, a buffer shorter than 8 + ceil(rows*cols/4)
 * bytes is a SHAPE_MISMATCH ("Insufficient packed data", gguf.rs:1098-1102). */
int bitnet_hip_bitlinear_set_weights_gguf(bitnet_hip_bitlinear *layer, const uint8_t *data, size_t len, size_t rows,
                                          size_t cols, int layout, int on_device, float *scale_out,
                                          float *offset_out, void *stream);
/* Pre-quantised weights in the reference's base-3 byte format (TernaryPackingStrategy::Base3Packed,
 * packing.rs:424-501: 1.6 bits per weight on disk), [out,in] flat, plus their scale.  The bytes are re-coded once into
 * the 2-bit tiles the kernels stream; a buffer shorter than ceil(out*in/5) bytes is a SHAPE_MISMATCH. */
int bitnet_hip_bitlinear_set_weights_base3(bitnet_hip_bitlinear *layer, const uint8_t *packed, size_t packed_len,
                                           float w_scale, int on_device, void *stream);
/* BitLinear::update_bias (layer.rs:329-352): INVALID_CONFIG if the layer was created without bias. */
int bitnet_hip_bitlinear_set_bias(bitnet_hip_bitlinear *layer, const float *bias, size_t len, int on_device,
                                  void *stream);

/* HOST outputs: the scale and the packed bytes the layer holds (the reference's QuantizedWeight,
 * bitnet-quant/src/quantization/weights.rs:158-175).  Synchronises the device. */
int bitnet_hip_bitlinear_get_quantized(bitnet_hip_bitlinear *layer, float *w_scale, uint8_t *packed,
                                       size_t packed_len);

/* Bytes of device workspace forward needs for m tokens: the quantised activations (int8 rows, a_scale, a_sum) and,
 * for 97 to about 256 tokens on rows of 4096 and more columns, the int32 partial tiles and tile counters of a GEMM
 * that splits k across workgroups.  forward accepts a workspace that holds only the first part (m * in_features
 * rounded up to 256, plus two arrays of 4 * m bytes rounded up to 256, plus 256) and then runs without the split:
 * same results, 10 to 20 % slower in that range. */
size_t bitnet_hip_bitlinear_workspace_size(const bitnet_hip_bitlinear *layer, size_t m);

/* BitLinearForward::forward (forward.rs:55-92) / BitLinearLayer::forward (transformer_layers.rs:119-201):
 * x has `rank` dimensions `dims` (HOST array); rank 2 [m, in] or rank 3 [b, s, in] (flattened to
 * [b*s, in]); anything else, or a last dimension != in_features, is BITNET_HIP_SHAPE_MISMATCH.
 *   gamma      NULL, or the RMSNorm weight [in] applied before quantisation (eps, sum_order as above)
 *   residual   NULL or [m, out] f32 added after the bias
 *   workspace  device buffer of at least workspace_size(m) bytes, or NULL to let the call allocate
 *              stream-ordered scratch itself
 *   debug outputs (each may be NULL): q [m,in] int8, a_scale [m] f32, acc [m,out] int32. */
int bitnet_hip_bitlinear_forward(bitnet_hip_bitlinear *layer, const float *x, const size_t *dims, int rank,
                                 const float *gamma, float eps, int sum_order, const float *residual,
                                 float *out, void *workspace, size_t workspace_bytes, int8_t *dbg_q,
                                 float *dbg_a_scale, int32_t *dbg_acc, void *stream);

/* bitnet_hip_bitlinear_forward for callers that cannot allocate device memory and have no workspace to pass:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in
 * the reference (BitLinearForward::forward returns a fresh tensor, forward.rs:55-92).  The quantised
 * activations (int8 [m, in], a_scale [m], a_sum [m]) live in a file-scope device array of the library,
 * 1,081,856 bytes per GPU, held until the process ends; the call performs no hipMalloc / hipFree of any kind.
 * Limits: m <= 4096 rows and m * in_features <= 1,048,576 per call, otherwise BITNET_HIP_MEMORY_ERROR and
 * nothing is launched (use bitnet_hip_bitlinear_forward with a workspace).  Same arguments, shape rules and
 * results (bit for bit) as bitnet_hip_bitlinear_forward without the debug outputs.  All calls on one GPU share
 * the array: calls that overlap in time on the same GPU (two streams, two threads) race; issue them on one
 * stream, or order them with events. */
int bitnet_hip_bitlinear_forward_noalloc(bitnet_hip_bitlinear *layer, const float *x, const size_t *dims, int rank,
                                         const float *gamma, float eps, int sum_order, const float *residual,
                                         float *out, void *stream);

/* Several layers applied to the same input x [m, in] (q, k, v of an attention block; gate, up of an FFN):
 * MultiHeadAttention::forward runs q_proj/k_proj/v_proj on one input
 * (bitnet-inference/src/engine/transformer_layers.rs:470-475), FeedForwardNetwork::forward up_proj/gate_proj
 * (:605-611).  The input is quantised once; at decode token counts up to three layers share one kernel
 * launch.  outs[j] is [m, out_features of layers[j]].  All layers must have the same in_features
 * (else SHAPE_MISMATCH).  workspace as for bitnet_hip_bitlinear_forward (sized for layers[0]). */
int bitnet_hip_bitlinear_forward_multi(bitnet_hip_bitlinear *const *layers, size_t count, const float *x, size_t m,
                                       const float *gamma, float eps, int sum_order, float *const *outs,
                                       void *workspace, size_t workspace_bytes, void *stream);

/* The contraction + epilogue of a layer on activations that are already quantised:
 * TernaryProcessor::ternary_matmul (bitnet-inference/src/engine/ternary_operations.rs:87-113) /
 * BitLinearForward::forward_with_quantized_weights (forward.rs:95-136) without the activation quantiser.
 *   a [m, in] int8, a_scale [m] f32, a_sum [m] int32 or NULL (see bitnet_hip_matmul_w2a8);
 *   acc [m, out] int32 and out [m, out] f32 may each be NULL (not both). */
int bitnet_hip_bitlinear_matmul(bitnet_hip_bitlinear *layer, const int8_t *a, const int32_t *a_sum, size_t m,
                                const float *a_scale, const float *residual, int32_t *acc, float *out,
                                void *stream);

/* ---- decoder projections (seven BitLinear layers per block) ------------------------------------ */

typedef struct bitnet_hip_decoder bitnet_hip_decoder; /* opaque */

#define BITNET_HIP_PROJ_Q 0
#define BITNET_HIP_PROJ_K 1
#define BITNET_HIP_PROJ_V 2
#define BITNET_HIP_PROJ_O 3
#define BITNET_HIP_PROJ_GATE 4
#define BITNET_HIP_PROJ_UP 5
#define BITNET_HIP_PROJ_DOWN 6

/* A stack of `layers` decoder blocks' BitLinear projections (TransformerBlock,
 * bitnet-inference/src/engine/transformer_layers.rs:626-710; MultiHeadAttention q/k/v/o :470-475,545;
 * FeedForwardNetwork :603-623) at decode time with no KV history: per block
 *   a = quant(rmsnorm(x, g_attn)); q,k,v = Wq a, Wk a, Wv a; x1 = x + Wo quant(gqa_broadcast(v));
 *   b = quant(rmsnorm(x1, g_ffn)); x2 = x1 + Wd quant(Wu b * relu(Wg b)^2).
 * max_tokens bounds m of decode() and sizes the internal activation buffers. */
int bitnet_hip_decoder_create(size_t layers, size_t hidden, size_t ffn, size_t q_heads, size_t kv_heads,
                              size_t head_dim, float eps, int sum_order, size_t max_tokens,
                              bitnet_hip_decoder **dec);
void bitnet_hip_decoder_destroy(bitnet_hip_decoder *dec);
/* The BitLinear object of projection `proj` of block `layer` (owned by the decoder). */
int bitnet_hip_decoder_projection(bitnet_hip_decoder *dec, size_t layer, int proj, bitnet_hip_bitlinear **out);
/* RMSNorm weights of a block: which = 0 (before attention) or 1 (before the FFN); [hidden] f32. */
int bitnet_hip_decoder_set_norm(bitnet_hip_decoder *dec, size_t layer, int which, const float *gamma,
                                int on_device, void *stream);
/* Row groups of a decode step.  Token rows never interact on this path (the reference fans independent inputs out
 * over threads, bitnet-inference/src/engine/cpu_backend.rs:206-238), so a step of m > 1 rows is run as `chains` groups
 * of consecutive rows, each a dependent chain of launches through all blocks on a stream of the decoder's own, forked
 * from and joined to the caller's stream by events (also inside a recorded step): the chains' launches overlap, the
 * results are those of the single chain bit for bit.  chains = 0 (the default) and 1 keep every row in one chain on
 * the caller's stream, which is the faster form on the device measured (kernels this short are started one at a time
 * whatever the number of queues); at most 8. */
int bitnet_hip_decoder_set_chains(bitnet_hip_decoder *dec, size_t chains);
/* Packed-weight bytes one decode step streams (sum of n*k/4 over all projections). */
size_t bitnet_hip_decoder_weight_bytes(const bitnet_hip_decoder *dec);
/* One decode step: x_in [m, hidden] -> x_out [m, hidden] through all blocks.  A decoder owns one set of activation
 * buffers: its decode calls are serialised (a call on another stream waits, on the GPU, for the one before it); use one
 * decoder per concurrent sequence group.  q_last / k_last (may be
 * NULL) receive the last block's q [m, hidden] and k [m, kv_heads*head_dim] projections. */
int bitnet_hip_decoder_decode(bitnet_hip_decoder *dec, const float *x_in, size_t m, float *x_out,
                              float *q_last, float *k_last, void *stream);
/* The same for blocks layer_begin .. layer_end-1 only (x_in may equal x_out). */
int bitnet_hip_decoder_decode_layers(bitnet_hip_decoder *dec, size_t layer_begin, size_t layer_end,
                                     const float *x_in, size_t m, float *x_out, float *q_last, float *k_last,
                                     void *stream);
/* A decode step recorded once and replayed: the launches of bitnet_hip_decoder_decode_layers(dec, layer_begin, layer_end,
 * x_in, m, x_out, q_last, k_last) as a HIP graph.  create waits for the device to be idle, runs the step once on a
 * stream of its own (x_out is written), records it and returns when both are done; launch replays it on `stream`, reading x_in and writing x_out (and q_last,
 * k_last) at the addresses given to create, with the locking and ordering of a decode call.  Weight, bias and norm
 * updates of the decoder's layers keep their device buffers, so a graph stays valid across them and reads the new
 * values; it must be destroyed before the decoder.
 *   No counterpart in the reference (its CPU path has no launches to batch).  For serving loops: enqueuing the 120
 *   launches of a batch-1 token step one by one costs the host as much time as the GPU needs to run them. */
typedef struct bitnet_hip_decoder_graph bitnet_hip_decoder_graph; /* opaque */
int bitnet_hip_decoder_graph_create(bitnet_hip_decoder *dec, size_t layer_begin, size_t layer_end, const float *x_in,
                                    size_t m, float *x_out, float *q_last, float *k_last,
                                    bitnet_hip_decoder_graph **graph);
int bitnet_hip_decoder_graph_launch(bitnet_hip_decoder_graph *graph, void *stream);
void bitnet_hip_decoder_graph_destroy(bitnet_hip_decoder_graph *graph);

/* ---- inference backend -------------------------------------------------------------------------------- */

typedef struct bitnet_hip_backend bitnet_hip_backend; /* opaque; the InferenceBackend of this path */

/* The plug-in point InferenceEngine::create_backend selects a backend at (bitnet-inference/src/api/mod.rs:426-460):
 *   replaces CpuInferenceBackend::new / MetalInferenceBackend::new behind the trait InferenceBackend
 *   (bitnet-inference/src/engine/mod.rs:126-138; CPU implementation engine/cpu_backend.rs:203-260).
 * Selects `device` (as bitnet_hip_init) and prepares an empty backend. */
int bitnet_hip_backend_create(int device, bitnet_hip_backend **backend);
void bitnet_hip_backend_destroy(bitnet_hip_backend *backend);
/* InferenceBackend::optimize_model (engine/mod.rs:131): binds the model this backend executes, a decoder stack whose
 * projections hold their weights (the decoder stays owned by the caller and must outlive the backend's use of it), and
 * allocates the staging buffers of execute_batch for up to the decoder's max_tokens rows. */
int bitnet_hip_backend_optimize_model(bitnet_hip_backend *backend, bitnet_hip_decoder *model);
/* InferenceBackend::execute_batch(&[Tensor]) -> Vec<Tensor> (engine/mod.rs:128): `count` inputs, input i a [rows[i], hidden]
 * f32 DEVICE matrix, output i a [rows[i], hidden] f32 DEVICE matrix owned by the caller: the hidden states after the
 * bound decoder stack.  inputs / rows / outputs are HOST arrays.  Inputs whose rows together fit the decoder's
 * max_tokens share one pass over the weights (the reference fans the inputs out over host threads,
 * cpu_backend.rs:206-238); every row's result is independent of what it is batched with.  NOT_INITIALIZED before
 * optimize_model; SHAPE_MISMATCH if one input alone exceeds max_tokens. */
int bitnet_hip_backend_execute_batch(bitnet_hip_backend *backend, const float *const *inputs, const size_t *rows,
                                     size_t count, float *const *outputs, void *stream);
/* InferenceBackend::get_memory_usage (engine/mod.rs:134): device bytes held by the bound model (packed and re-tiled
 * weights, scales, norms, activation buffers) and by the backend's staging buffers; 0 before optimize_model. */
size_t bitnet_hip_backend_get_memory_usage(const bitnet_hip_backend *backend);
/* InferenceBackend::capabilities (engine/mod.rs:137; BackendCapabilities :141-148).  HOST outputs, each may be NULL:
 * supports_batching (1), supports_streaming (0), max_batch_size (rows per pass: the bound decoder's max_tokens, 0 before
 * optimize_model), memory_limit (the device's total memory), device (the HIP device ordinal). */
int bitnet_hip_backend_capabilities(const bitnet_hip_backend *backend, int *supports_batching, int *supports_streaming,
                                    size_t *max_batch_size, size_t *memory_limit, int *device);

#ifdef __cplusplus
}
#endif
#endif /* BITNET_HIP_H */
