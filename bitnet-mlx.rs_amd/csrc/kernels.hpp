// Internal launchers, one per kernel family.  Arguments are validated by the C-ABI layer (api.hip);
// these only pick a kernel variant and launch it.  All return a bitnet_hip_status.
#pragma once
#include "common.hpp"
#include "ieee.hpp"

namespace bitnet {

// ---- geometry of the re-tiled weight layout (see weight_prep.hip) ----
constexpr int TILE_ROWS = 16;    // output rows per tile
constexpr int TILE_K = 256;      // input columns per tile
constexpr int TILE_BYTES = 1024; // TILE_ROWS * TILE_K / 4
inline size_t row_blocks(size_t n) { return (n + TILE_ROWS - 1) / TILE_ROWS; }
inline size_t k_tiles(size_t k) { return (k + TILE_K - 1) / TILE_K; }
inline size_t tiled_bytes(size_t n, size_t k) { return row_blocks(n) * k_tiles(k) * (size_t)TILE_BYTES; }

// act_quant.hip
int launch_act_quant(const float *x, const float *x2, size_t ldx, size_t m, size_t k, int input_mode,
                     size_t gqa_group, size_t head_dim, const float *gamma, float eps, int sum_order,
                     int8_t *q, float *a_scale, int32_t *a_sum, float *y, hipStream_t stream, unsigned *zero = nullptr,
                     size_t zero_n = 0);  // zero[0 .. zero_n): cleared by the launch (tile counters of the GEMM behind it)

// absmax_quantize_activations (activations.rs:530-641): one scale per tensor; scratch of absmax_quantize_scratch_bytes(n)
// bytes; stats: 4 floats (scale, mse, min, max)
size_t absmax_quantize_scratch_bytes(size_t n);
int launch_absmax_quantize(const float *x, size_t n, int precision, void *scratch, int8_t *q, float *stats, hipStream_t stream);
// max |x| of a tensor into the first float of `scratch` (absmax_quantize_scratch_bytes(n) bytes), and the quantiser of
// DynamicActivationQuantizer with the scale given from outside (activations.rs:269-294, 315-360)
int launch_abs_max(const float *x, size_t n, void *scratch, hipStream_t stream);
int launch_scaled_quantize(const float *x, size_t n, int precision, float scale, int reference_u8, int8_t *q, hipStream_t stream);

// weight_prep.hip
int launch_pack_2bit(const int8_t *q, size_t count, uint8_t *packed, hipStream_t stream);
int launch_unpack_2bit(const uint8_t *packed, size_t count, int8_t *q, hipStream_t stream);
int launch_lookup_compute(int kind, const int8_t *w, const float *x, float *out, size_t n, hipStream_t stream);
// base-3 bytes (5 values each): pack, unpack, and re-code into the 2-bit bytes (4 values each)
int launch_pack_base3(const int8_t *q, size_t count, uint8_t *packed, hipStream_t stream);
int launch_unpack_base3(const uint8_t *packed, size_t count, int8_t *q, hipStream_t stream);
int launch_base3_to_2bit(const uint8_t *base3, size_t count, uint8_t *packed, hipStream_t stream);
// row_sums: device scratch of n doubles
int launch_quantize_weights(const float *w, size_t n, size_t k, int method, float threshold_factor,
                            double *row_sums, uint8_t *packed, float *w_scale, int8_t *q_i8,
                            hipStream_t stream);
// BitNetWeightQuantizer::quantize (weights.rs:568-611): method = TernaryMethod 0..4, custom_factor <= 0 = none;
// scratch: quantize_weights_reference_scratch_bytes(n) bytes of device memory; stats: 12 floats or null
size_t quantize_weights_reference_scratch_bytes(size_t n);
int launch_quantize_weights_reference(const float *w, size_t n, size_t k, int method, int normalize, float outlier_threshold,
                                      float custom_factor, void *scratch, uint8_t *packed, float *w_scale, int8_t *q_i8,
                                      float *stats, hipStream_t stream);
int launch_retile(const uint8_t *packed, size_t n, size_t k, int layout, uint8_t *tiled, hipStream_t stream);
int launch_untile(const uint8_t *tiled, size_t n, size_t k, uint8_t *packed, hipStream_t stream);

// gemv_base3.hip: the decode GEMV on base-3 bytes (five values per byte) in their own streaming layout
size_t base3_tiled_bytes(size_t n, size_t k);
int launch_retile_base3(const uint8_t *flat, size_t n, size_t k, uint8_t *tiled, hipStream_t stream);
int launch_gemv_base3(const uint8_t *tiled, const int8_t *a, int32_t *acc, float *out, const float *w_scale, const float *a_scale,
                      size_t n, size_t k, hipStream_t stream);

// gemv_w2a8.hip
int launch_gemv_rowmajor(const uint8_t *packed, const int8_t *a, int32_t *out, size_t n, size_t k,
                         hipStream_t stream);
constexpr int GEMV_MAX_M = 95;      // token rows the decode-GEMV path always takes
// More rows go to the prefill GEMM, except where the token-group GEMV (gemv_mfma_tg_kernel: k a multiple of 256 up to
// 8192, 16-byte aligned rows) runs as a single round of workgroups: it then beats a GEMM that is too small to fill the
// chip (6912 -> 2560 at 96 tokens: 13.6 us against 18.9 us; 2560 -> 2560 up to 192 tokens: 8.4 .. 9.8 us against
// 10.7 .. 11.0 us), and loses as soon as its workgroups need a second round (6912 -> 2560 at 112 tokens: 21.6 us
// against 19.1 us).  n_blocks: 16-row blocks of all projections of the launch.  The row blocks per workgroup and
// the workgroup slots follow launch_gemv_tiled.
constexpr int GEMV_WIDE_MAX_M = 512;
inline bool gemv_takes(size_t m, size_t k, size_t n_blocks, const void *a)
{
    if (m <= (size_t)GEMV_MAX_M) return true;
    if (m > (size_t)GEMV_WIDE_MAX_M || k % 256 != 0 || k > 8192 || (reinterpret_cast<uintptr_t>(a) & 15) != 0) return false;
    const size_t tgroups = (m + 15) / 16, slots = k <= 3072 ? 768 : 256;
    const size_t rb = n_blocks * tgroups > 2 * slots ? 4 : (n_blocks * tgroups > slots ? 2 : 1);
    return (n_blocks + rb - 1) / rb * tgroups <= slots;
}
constexpr int GEMV_MFMA_MAX_M = 64; // rows per launch of the MFMA variant of the decode GEMV (2 and more rows)
constexpr int GEMV_MAX_PROJ = 3;  // projections sharing one input row per launch (q,k,v / gate,up)
// One projection of a decode-GEMV launch: re-tiled weights [n, k], its scale, optional bias [n] and
// residual [m, n]; out [m, n] f32 and acc [m, n] int32 are each optional.
struct GemvProj {
    const uint8_t *tiled;
    const float *w_scale;
    const float *bias;
    const float *residual;
    float *out;
    int32_t *acc;
    size_t n;
};
// activations already int8 ([m, k], a_scale [m]); any m (launched in groups of up to GEMV_MAX_M rows)
int launch_gemv_tiled(const GemvProj *projs, int nproj, const int8_t *a, const float *a_scale, size_t m, size_t k,
                      hipStream_t stream);
// f32 input quantised inside the GEMV launch; only where gemv_fused_supported() says so.  q_out / a_scale_out /
// a_sum_out (each optional) receive the quantiser's results.
bool gemv_fused_supported(const float *x, const float *x2, size_t ldx, size_t m, size_t k, int input_mode,
                          size_t head_dim, const float *gamma, int sum_order, size_t blocks);
// blocks: 16-row blocks of all projections of the launch (of its largest launch group)
int launch_gemv_fused(const GemvProj *projs, int nproj, const float *x, const float *x2, size_t ldx, size_t m,
                      size_t k, int input_mode, size_t gqa_group, size_t head_dim, const float *gamma, float eps,
                      int sum_order, int8_t *q_out, float *a_scale_out, int32_t *a_sum_out, hipStream_t stream);

// gemm_w2a8.hip
constexpr int GEMM_MAX_PROJ = 3;  // projections sharing one activation matrix per launch of the LDS-direct kernels
// several projections in one launch; BITNET_HIP_UNSUPPORTED (no message) if the LDS-direct kernels do not apply
// Scratch of a GEMM launch that splits k across workgroups (gemm_split_plan): int32 partial tiles, and one counter per
// output tile that MUST be zero when the launch starts (the activation quantiser in front of the GEMM zeroes them:
// launch_act_quant's zero / zero_n) and is zero again when it ends.  Both belong to the caller's workspace.
struct GemmSplitScratch {
    int32_t *partials = nullptr;
    unsigned *counters = nullptr;
    size_t partial_bytes = 0, counter_count = 0;
};
// What launch_gemm_multi needs to split k for this launch: bytes of partials (a multiple of 256) and the number of
// counters; both 0 when it would not split.  n: output widths of the projections that share the launch.
void gemm_split_plan(size_t m, size_t k, const size_t *n, int nproj, size_t *partial_bytes, size_t *counters);
int launch_gemm_multi(const GemvProj *projs, int nproj, const int8_t *a, const int32_t *a_sum, const float *a_scale,
                      size_t m, size_t k, hipStream_t stream, const GemmSplitScratch *split = nullptr);
// a_sum (sum_k a[t, k] per row, from the activation quantiser) may be NULL: the slower kernel then computes it
int launch_gemm_tiled(const uint8_t *tiled, const int8_t *a, const int32_t *a_sum, size_t m, size_t n, size_t k,
                      int32_t *acc, const float *w_scale, const float *a_scale, const float *bias,
                      const float *residual, float *out, hipStream_t stream);

// Diagnostic: `iters` rounds of eight v_mfma_i32_16x16x64_i8 per wavefront, MFMA_RATE_THREADS / 64 wavefronts on each of
// `compute_units` workgroups, operands in registers; sink receives compute_units * MFMA_RATE_THREADS ints.
constexpr int MFMA_RATE_THREADS = 512;
constexpr int MFMA_RATE_PER_ITER = 8;
int launch_mfma_rate(bool random_operands, int iters, int compute_units, int *sink, hipStream_t stream);

}  // namespace bitnet
