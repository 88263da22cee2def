//! Raw `extern "C"` declarations of include/bitnet_hip.h, one per exported symbol, same order.
//! Device pointers are plain raw pointers owned by the caller; `stream` is a `hipStream_t`.
#![allow(non_camel_case_types)]
use std::os::raw::{c_char, c_int, c_void};

#[repr(C)]
pub struct bitnet_hip_bitlinear {
    _private: [u8; 0],
}
#[repr(C)]
pub struct bitnet_hip_decoder {
    _private: [u8; 0],
}
#[repr(C)]
pub struct bitnet_hip_decoder_graph {
    _private: [u8; 0],
}
#[repr(C)]
pub struct bitnet_hip_backend {
    _private: [u8; 0],
}

pub const BITNET_HIP_OK: c_int = 0;
pub const BITNET_HIP_SHAPE_MISMATCH: c_int = 1;
pub const BITNET_HIP_INVALID_CONFIG: c_int = 2;
pub const BITNET_HIP_DEVICE_ERROR: c_int = 3;
pub const BITNET_HIP_MEMORY_ERROR: c_int = 4;
pub const BITNET_HIP_QUANTIZATION_ERROR: c_int = 5;
pub const BITNET_HIP_NOT_INITIALIZED: c_int = 6;
pub const BITNET_HIP_KERNEL_ERROR: c_int = 7;
pub const BITNET_HIP_NULL_POINTER: c_int = 8;
pub const BITNET_HIP_UNSUPPORTED: c_int = 9;

pub const BITNET_HIP_SUM_SEQUENTIAL: c_int = 0;
pub const BITNET_HIP_SUM_BLOCK256: c_int = 1;
pub const BITNET_HIP_LAYOUT_OUT_IN: c_int = 0;
pub const BITNET_HIP_LAYOUT_IN_OUT: c_int = 1;
pub const BITNET_HIP_TERNARY_ABSMEAN_ROUNDCLIP: c_int = 0;
pub const BITNET_HIP_TERNARY_MEAN_THRESHOLD: c_int = 1;
pub const BITNET_HIP_TERNARY_REF_MEAN_THRESHOLD: c_int = 2;
pub const BITNET_HIP_TERNARY_REF_MEDIAN_THRESHOLD: c_int = 3;
pub const BITNET_HIP_TERNARY_REF_ADAPTIVE_THRESHOLD: c_int = 4;
pub const BITNET_HIP_TERNARY_REF_OPTIMAL_THRESHOLD: c_int = 5;
pub const BITNET_HIP_TERNARY_REF_DETSTE: c_int = 6;
pub const BITNET_HIP_INPUT_PLAIN: c_int = 0;
pub const BITNET_HIP_INPUT_RELU2_MUL: c_int = 1;
pub const BITNET_HIP_INPUT_GQA_BROADCAST: c_int = 2;
pub const BITNET_HIP_PRECISION_ONE_FIVE_FIVE_BIT: c_int = 0;
pub const BITNET_HIP_PRECISION_EIGHT_BIT: c_int = 1;
pub const BITNET_HIP_LOOKUP_TERNARY: c_int = 0;
pub const BITNET_HIP_LOOKUP_I2S: c_int = 1;

// Only with the `hip` feature: without it nothing of the library is referenced, so the crate links without it.
#[cfg(feature = "hip")]
extern "C" {
    pub fn bitnet_hip_last_error() -> *const c_char;
    pub fn bitnet_hip_last_shape_mismatch(expected: *mut usize, actual: *mut usize, actual_rank: *mut c_int) -> c_int;
    pub fn bitnet_hip_init(device: c_int) -> c_int;
    pub fn bitnet_hip_device_info(arch_name: *mut c_char, arch_name_len: usize, compute_units: *mut c_int,
                                  clock_mhz: *mut c_int, total_mem_bytes: *mut usize) -> c_int;
    pub fn bitnet_hip_measure_mfma_i8_rate(random_operands: c_int, tera_ops_per_second: *mut f64, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_measure_launch_chain(buf: *const c_void, bytes_per_launch: *const usize, pattern_len: usize,
                                           launches: usize, replays: usize, us_per_replay: *mut f64,
                                           stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_measure_hop(two_level: c_int, values: usize, hops: usize, spin_limit: c_int, us_per_hop: *mut f64, intact: *mut c_int,
                                  stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_quantize_activations_i8(x: *const f32, x2: *const f32, ldx: usize, m: usize, k: usize,
                                              input_mode: c_int, gqa_group: usize, head_dim: usize, gamma: *const f32,
                                              eps: f32, sum_order: c_int, q: *mut i8, a_scale: *mut f32,
                                              a_sum: *mut i32, y_f32: *mut f32, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_absmax_quantize_activations(x: *const f32, count: usize, precision: c_int, values: *mut i8,
                                                  stats: *mut f32, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_abs_max(x: *const f32, count: usize, abs_max: *mut f32, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_quantize_activations_scaled(x: *const f32, count: usize, precision: c_int, scale: f32,
                                                  reference_u8: c_int, values: *mut i8, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_lookup_compute(kind: c_int, weights: *const i8, n_weights: usize, inputs: *const f32,
                                     n_inputs: usize, output: *mut f32, n_output: usize, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_packed_size(count: usize) -> usize;
    pub fn bitnet_hip_pack_ternary_2bit(q: *const i8, count: usize, packed: *mut u8, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_unpack_ternary_2bit(packed: *const u8, count: usize, q: *mut i8, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_base3_packed_size(count: usize) -> usize;
    pub fn bitnet_hip_pack_ternary_base3(q: *const i8, count: usize, packed: *mut u8, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_unpack_ternary_base3(packed: *const u8, count: usize, q: *mut i8, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_base3_tiled_size(n: usize, k: usize) -> usize;
    pub fn bitnet_hip_retile_base3(base3: *const u8, n: usize, k: usize, tiled: *mut u8, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_gemv_base3(tiled: *const u8, a: *const i8, n: usize, k: usize, w_scale: *const f32,
                                 a_scale: *const f32, acc: *mut i32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_quantize_weights(w: *const f32, n: usize, k: usize, method: c_int, threshold_factor: f32,
                                       packed: *mut u8, w_scale: *mut f32, q_i8: *mut i8, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_quantize_weights_reference(w: *const f32, n: usize, k: usize, ternary_method: c_int,
                                                 normalize_weights: c_int, outlier_threshold: f32,
                                                 custom_threshold_factor: f32, packed: *mut u8, w_scale: *mut f32,
                                                 q_i8: *mut i8, stats: *mut f32, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_tiled_size(n: usize, k: usize) -> usize;
    pub fn bitnet_hip_retile_weights(packed: *const u8, n: usize, k: usize, layout: c_int, tiled: *mut u8,
                                     stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_untile_weights(tiled: *const u8, n: usize, k: usize, packed: *mut u8, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_gemv_w2a8(weights: *const u8, activations: *const i8, output: *mut i32, m: usize, k: usize,
                                stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_gemv_w2a8_checked(weights: *const u8, weights_len: usize, activations: *const i8,
                                        activations_len: usize, output: *mut i32, output_len: usize, m: usize,
                                        k: usize, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_matmul_w2a8(tiled: *const u8, a: *const i8, a_sum: *const i32, m: usize, n: usize, k: usize,
                                  acc: *mut i32, w_scale: *const f32, a_scale: *const f32, bias: *const f32,
                                  residual: *const f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_bitlinear_create(in_features: usize, out_features: usize, use_bias: c_int,
                                       layer: *mut *mut bitnet_hip_bitlinear) -> c_int;
    pub fn bitnet_hip_bitlinear_destroy(layer: *mut bitnet_hip_bitlinear);
    pub fn bitnet_hip_bitlinear_set_weights_f32(layer: *mut bitnet_hip_bitlinear, w: *const f32, rows: usize,
                                                cols: usize, layout: c_int, on_device: c_int, method: c_int,
                                                threshold_factor: f32, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_bitlinear_set_weights_packed(layer: *mut bitnet_hip_bitlinear, packed: *const u8,
                                                   packed_len: usize, w_scale: f32, on_device: c_int,
                                                   stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_bitlinear_set_weights_base3(layer: *mut bitnet_hip_bitlinear, packed: *const u8,
                                                  packed_len: usize, w_scale: f32, on_device: c_int,
                                                  stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_bitlinear_set_weights_gguf(layer: *mut bitnet_hip_bitlinear, data: *const u8, len: usize,
                                                 rows: usize, cols: usize, layout: c_int, on_device: c_int,
                                                 scale_out: *mut f32, offset_out: *mut f32,
                                                 stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_bitlinear_set_bias(layer: *mut bitnet_hip_bitlinear, bias: *const f32, len: usize,
                                         on_device: c_int, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_bitlinear_get_quantized(layer: *mut bitnet_hip_bitlinear, w_scale: *mut f32, packed: *mut u8,
                                              packed_len: usize) -> c_int;
    pub fn bitnet_hip_bitlinear_workspace_size(layer: *const bitnet_hip_bitlinear, m: usize) -> usize;
    pub fn bitnet_hip_bitlinear_forward(layer: *mut bitnet_hip_bitlinear, x: *const f32, dims: *const usize,
                                        rank: c_int, gamma: *const f32, eps: f32, sum_order: c_int,
                                        residual: *const f32, out: *mut f32, workspace: *mut c_void,
                                        workspace_bytes: usize, dbg_q: *mut i8, dbg_a_scale: *mut f32,
                                        dbg_acc: *mut i32, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_bitlinear_forward_noalloc(layer: *mut bitnet_hip_bitlinear, x: *const f32, dims: *const usize,
                                                rank: c_int, gamma: *const f32, eps: f32, sum_order: c_int,
                                                residual: *const f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_bitlinear_forward_multi(layers: *const *mut bitnet_hip_bitlinear, count: usize, x: *const f32,
                                              m: usize, gamma: *const f32, eps: f32, sum_order: c_int,
                                              outs: *const *mut f32, workspace: *mut c_void, workspace_bytes: usize,
                                              stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_bitlinear_matmul(layer: *mut bitnet_hip_bitlinear, a: *const i8, a_sum: *const i32, m: usize,
                                       a_scale: *const f32, residual: *const f32, acc: *mut i32, out: *mut f32,
                                       stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_decoder_create(layers: usize, hidden: usize, ffn: usize, q_heads: usize, kv_heads: usize,
                                     head_dim: usize, eps: f32, sum_order: c_int, max_tokens: usize,
                                     dec: *mut *mut bitnet_hip_decoder) -> c_int;
    pub fn bitnet_hip_decoder_destroy(dec: *mut bitnet_hip_decoder);
    pub fn bitnet_hip_decoder_projection(dec: *mut bitnet_hip_decoder, layer: usize, proj: c_int,
                                         out: *mut *mut bitnet_hip_bitlinear) -> c_int;
    pub fn bitnet_hip_decoder_set_norm(dec: *mut bitnet_hip_decoder, layer: usize, which: c_int, gamma: *const f32,
                                       on_device: c_int, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_decoder_set_chains(dec: *mut bitnet_hip_decoder, chains: usize) -> c_int;
    pub fn bitnet_hip_decoder_weight_bytes(dec: *const bitnet_hip_decoder) -> usize;
    pub fn bitnet_hip_decoder_decode(dec: *mut bitnet_hip_decoder, x_in: *const f32, m: usize, x_out: *mut f32,
                                     q_last: *mut f32, k_last: *mut f32, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_decoder_decode_layers(dec: *mut bitnet_hip_decoder, layer_begin: usize, layer_end: usize,
                                            x_in: *const f32, m: usize, x_out: *mut f32, q_last: *mut f32,
                                            k_last: *mut f32, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_decoder_graph_create(dec: *mut bitnet_hip_decoder, layer_begin: usize, layer_end: usize,
                                           x_in: *const f32, m: usize, x_out: *mut f32, q_last: *mut f32,
                                           k_last: *mut f32, graph: *mut *mut bitnet_hip_decoder_graph) -> c_int;
    pub fn bitnet_hip_decoder_graph_launch(graph: *mut bitnet_hip_decoder_graph, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_decoder_graph_destroy(graph: *mut bitnet_hip_decoder_graph);
    pub fn bitnet_hip_backend_create(device: c_int, backend: *mut *mut bitnet_hip_backend) -> c_int;
    pub fn bitnet_hip_backend_destroy(backend: *mut bitnet_hip_backend);
    pub fn bitnet_hip_backend_optimize_model(backend: *mut bitnet_hip_backend, model: *mut bitnet_hip_decoder) -> c_int;
    pub fn bitnet_hip_backend_execute_batch(backend: *mut bitnet_hip_backend, inputs: *const *const f32, rows: *const usize,
                                            count: usize, outputs: *const *mut f32, stream: *mut c_void) -> c_int;
    pub fn bitnet_hip_backend_get_memory_usage(backend: *const bitnet_hip_backend) -> usize;
    pub fn bitnet_hip_backend_capabilities(backend: *const bitnet_hip_backend, supports_batching: *mut c_int,
                                           supports_streaming: *mut c_int, max_batch_size: *mut usize,
                                           memory_limit: *mut usize, device: *mut c_int) -> c_int;
}
