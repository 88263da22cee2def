// Weight-side kernels: ternarisation, 2-bit packing in the reference's byte format, and the re-tiling
// into the layout the contraction kernels stream.  All of them run once per weight update.
//
// Reference byte format (bitnet-quant/src/quantization/packing.rs:353-394 over
// bitnet-quant/src/quantization/utils.rs:434-451): code = w + 1 in {0,1,2}; flat element i lives in
// byte i/4 at bits 2*(i mod 4); missing tail elements leave 0 bits.  Decoding maps 0,1,2,3 to
// -1,0,+1,0 (bitnet-inference/src/engine/weight_conversion.rs:169-184).
//
// Re-tiled layout: the [n, k] matrix is cut into tiles of TILE_ROWS(16) rows x TILE_K(256) columns.  A
// tile is 1 KiB = 64 slots of 16 bytes.  Slot s = kq*16 + r (kq = 0..3, r = 0..15) belongs to row r of the
// tile; its dword t (t = 0..3) holds the 16 columns 64*t + 16*kq .. +15.  Inside a dword the weight with
// column offset 4j + b sits at bits 2j + 8b, so that (dword >> 2j) & 0x03030303 yields the four code
// bytes of columns 4j..4j+3 in activation byte order.  Tiles are stored row-block major: tile (rb, kt)
// starts at byte ((rb * k_tiles) + kt) * 1024.
// Why this order: a wavefront whose lane l loads slot l reads one tile as a single contiguous 1 KiB
// burst, and dword t of every lane is then exactly the B operand of the t-th 16x16x64 int8 MFMA over
// the tile's columns 64t..64t+63 (operand row/column = lane mod 16, 16-column k block = lane / 16).
// Lanes l, l+16, l+32, l+48 share a row, so the decode GEMV combines them with two shuffles.
// Positions outside the matrix hold code 1 (weight 0) and code 3 is rewritten to code 1, so the
// contraction kernels never see code 3.
#include "kernels.hpp"

namespace bitnet {

namespace {

__global__ __launch_bounds__(256) void pack_2bit_kernel(const int8_t *q, size_t count, uint8_t *packed,
                                                        size_t nbytes)
{
    size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nbytes) return;
    unsigned byte = 0;
    for (int j = 0; j < 4; ++j) {
        size_t i = 4 * b + j;
        if (i < count) byte |= ((unsigned)(q[i] + 1) & 3u) << (2 * j);
    }
    packed[b] = (uint8_t)byte;
}

__global__ __launch_bounds__(256) void unpack_2bit_kernel(const uint8_t *packed, size_t count, int8_t *q)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    unsigned code = (packed[i >> 2] >> (2 * (i & 3))) & 3u;
    q[i] = code == 0 ? -1 : (code == 2 ? 1 : 0);
}

// Base-3 bytes: value j of byte b is digit j of b in base 3 (bitnet-quant/src/quantization/packing.rs:424-501).
__device__ __forceinline__ unsigned base3_digit(unsigned byte, unsigned j)
{
    const unsigned div = j == 0 ? 1u : (j == 1 ? 3u : (j == 2 ? 9u : (j == 3 ? 27u : 81u)));
    return (byte / div) % 3u;
}

__global__ __launch_bounds__(256) void pack_base3_kernel(const int8_t *q, size_t count, uint8_t *packed, size_t nbytes)
{
    size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nbytes) return;
    unsigned byte = 0, mult = 1;
    for (int j = 0; j < 5; ++j) {
        size_t i = 5 * b + j;
        if (i < count) byte += (unsigned)(uint8_t)(q[i] + 1) * mult;
        mult *= 3;
    }
    packed[b] = (uint8_t)byte;
}

__global__ __launch_bounds__(256) void unpack_base3_kernel(const uint8_t *packed, size_t count, int8_t *q)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    q[i] = (int8_t)base3_digit(packed[i / 5], (unsigned)(i % 5)) - 1;
}

// One 2-bit byte (elements 4b .. 4b+3) per thread: both formats use the code w + 1.
__global__ __launch_bounds__(256) void base3_to_2bit_kernel(const uint8_t *base3, size_t count, uint8_t *packed, size_t nbytes)
{
    size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nbytes) return;
    unsigned byte = 0;
    for (int j = 0; j < 4; ++j) {
        size_t i = 4 * b + j;
        if (i < count) byte |= base3_digit(base3[i / 5], (unsigned)(i % 5)) << (2 * j);
    }
    packed[b] = (uint8_t)byte;
}

// TernaryLookupKernel / I2SLookupKernel::compute (bitnet-core/src/cpu/kernels/generic.rs:54-75,118-139).
__global__ __launch_bounds__(256) void lookup_compute_kernel(int kind, const int8_t *w, const float *x, float *out, size_t n)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int v = w[i];
    float l;
    if (kind == BITNET_HIP_LOOKUP_TERNARY) l = v == -1 ? -1.0f : (v == 1 ? 1.0f : 0.0f);
    else l = v == -2 ? -2.0f : (v == -1 ? -1.0f : (v == 1 ? 1.0f : 0.0f));
    out[i] = f32_mul(x[i], l);
}

__device__ __forceinline__ double wave_sum_f64(double p)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) p = p + __shfl_xor(p, off, 64);
    return p;
}

// Sum of |w| of one row in f64: lane l adds columns l, l+64, ... in ascending order, then the
// butterfly.  One wavefront per row.
__global__ __launch_bounds__(256) void absmean_rows_kernel(const float *w, size_t n, size_t k, double *row_sums)
{
    const int lane = threadIdx.x;
    const size_t row = (size_t)blockIdx.x * blockDim.y + threadIdx.y;
    if (row >= n) return;
    const float *wr = w + row * k;
    double s = 0.0;
    for (size_t c = lane; c < k; c += 64) s = s + (double)fabsf(wr[c]);
    s = wave_sum_f64(s);
    if (lane == 0) row_sums[row] = s;
}

// Combines the row sums the same way (lane l takes rows l, l+64, ...) and writes mean|W| as f32.
__global__ __launch_bounds__(64) void absmean_final_kernel(const double *row_sums, size_t n, size_t k, float *w_scale)
{
    const int lane = threadIdx.x;
    double s = 0.0;
    for (size_t r = lane; r < n; r += 64) s = s + row_sums[r];
    s = wave_sum_f64(s);
    if (lane == 0) *w_scale = (n == 0 || k == 0) ? 0.0f : (float)(s / ((double)n * (double)k));
}

__device__ __forceinline__ int ternarize_one(float w, int method, float s, float thr)
{
    if (method == BITNET_HIP_TERNARY_ABSMEAN_ROUNDCLIP) {
        // RoundClip(w / s, -1, 1); s == 0 gives 0
        if (s == 0.0f) return 0;
        float r = roundf(f32_div(w, s));
        if (r != r) return 0;
        r = fminf(fmaxf(r, -1.0f), 1.0f);
        return (int)r;
    }
    return w > thr ? 1 : (w < -thr ? -1 : 0);  // strict comparisons, bitnet-quant/src/simd/ternary.rs:75-83
}

__global__ __launch_bounds__(256) void ternarize_pack_kernel(const float *w, size_t count, int method,
                                                             float factor, const float *w_scale,
                                                             uint8_t *packed, int8_t *q_i8, size_t nbytes)
{
    size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nbytes) return;
    const float s = *w_scale;
    const float thr = f32_mul(factor, s);
    unsigned byte = 0;
    for (int j = 0; j < 4; ++j) {
        size_t i = 4 * b + j;
        if (i < count) {
            int t = ternarize_one(w[i], method, s, thr);
            if (q_i8) q_i8[i] = (int8_t)t;
            byte |= ((unsigned)(t + 1) & 3u) << (2 * j);
        }
    }
    packed[b] = (uint8_t)byte;
}

// ---- BitNetWeightQuantizer::quantize, the reference's weight pipeline (bitnet-quant/src/quantization/weights.rs:568-611)
//
//   w' = (w - mean) / sqrt(var + 1e-8)                   normalize_before_quantize, :671-686
//   w'' = clamp(w', mean' - t*mad, mean' + t*mad)        handle_outliers, :688-699 (mad = mean|w'|)
//   thr by TernaryMethod from mean|w''| (and max|w''|)   :370-480
//   q = sign(w'') * [|w''| > thr]                        apply_ternary_quantization, :482-496
//   scale = sum(w''*q) / sum(q*q)                        compute_ternary_scale, :546-559
//
// Nothing but the packed codes and the scale is written: w'' is recomputed from w wherever it is needed (two
// f32 operations and a clamp).  Every tensor-wide sum is carried in f64 in the order of the absmean kernels above
// (per row: lane l adds columns l, l+64, ..., then the butterfly; the row sums the same way), so the f32 scalars
// have the bits the CPU restatement of the same order has.  The scalars stay on the device in WqState; one
// wavefront finishes each reduction and derives the next stage's scalars.
struct WqState {
    float mean, sd;            // normalisation (0, 1 when switched off)
    float clip_mean, clip_mad; // centre and mean |.| of the normalised tensor
    float lo, hi;              // clip bounds (-inf, +inf when switched off)
    float mean_abs, max_abs;   // of the processed tensor
    float thr;
    float num, den, scale;
};
static_assert(sizeof(WqState) == 12 * sizeof(float), "stats are returned as 12 floats");

enum WqPass { WQ_SUM = 0, WQ_SQDIFF, WQ_CLIP_STATS, WQ_ABS_STATS, WQ_OPTIMAL, WQ_SCALE };
constexpr int WQ_MAX_ACC = 10;

__device__ __forceinline__ float wq_normalised(float w, const WqState &st, bool normalize)
{
    return normalize ? f32_div(w - st.mean, st.sd) : w;
}
__device__ __forceinline__ float wq_processed(float w, const WqState &st, bool normalize, bool clip)
{
    float x = wq_normalised(w, st, normalize);
    if (clip) {
        x = x > st.hi ? st.hi : x;
        x = x < st.lo ? st.lo : x;
    }
    return x;
}
__device__ __forceinline__ float wq_code(float x, float thr) { return x > thr ? 1.0f : (x < -thr ? -1.0f : 0.0f); }

__constant__ float wq_factors[10] = {0.3f, 0.4f, 0.5f, 0.6f, 0.7f, 0.8f, 0.9f, 1.0f, 1.1f, 1.2f};

// One wavefront per row; accumulator a of row r goes to row_sums[a * n + r] (and the row's max |.| to row_max[r]).
template <int PASS>
__global__ __launch_bounds__(256) void wq_rows_kernel(const float *w, size_t n, size_t k, const WqState *state, int normalize,
                                                      int clip, double *row_sums, float *row_max)
{
    constexpr int NACC = PASS == WQ_OPTIMAL ? 10 : ((PASS == WQ_CLIP_STATS || PASS == WQ_SCALE) ? 2 : 1);
    const int lane = threadIdx.x;
    const size_t row = (size_t)blockIdx.x * blockDim.y + threadIdx.y;
    if (row >= n) return;
    const WqState st = *state;
    const float *wr = w + row * k;
    double acc[NACC];
#pragma unroll
    for (int a = 0; a < NACC; ++a) acc[a] = 0.0;
    float mx = 0.0f;
    float cand[PASS == WQ_OPTIMAL ? 10 : 1];
    if constexpr (PASS == WQ_OPTIMAL) {
#pragma unroll
        for (int f = 0; f < 10; ++f) cand[f] = f32_mul(st.mean_abs, wq_factors[f]);
    }
    for (size_t c = lane; c < k; c += 64) {
        const float v = wr[c];
        if constexpr (PASS == WQ_SUM) {
            acc[0] = acc[0] + (double)v;
        } else if constexpr (PASS == WQ_SQDIFF) {
            const float d = v - st.mean;
            acc[0] = acc[0] + (double)f32_mul(d, d);
        } else if constexpr (PASS == WQ_CLIP_STATS) {
            const float x = wq_normalised(v, st, normalize != 0);
            acc[0] = acc[0] + (double)x;
            acc[1] = acc[1] + (double)fabsf(x);
        } else if constexpr (PASS == WQ_ABS_STATS) {
            const float ax = fabsf(wq_processed(v, st, normalize != 0, clip != 0));
            acc[0] = acc[0] + (double)ax;
            mx = fmaxf(mx, ax);
        } else if constexpr (PASS == WQ_OPTIMAL) {
            const float x = wq_processed(v, st, normalize != 0, clip != 0);
#pragma unroll
            for (int f = 0; f < 10; ++f) {
                const float d = x - wq_code(x, cand[f]);
                acc[f] = acc[f] + (double)f32_mul(d, d);
            }
        } else {
            const float x = wq_processed(v, st, normalize != 0, clip != 0);
            const float q = wq_code(x, st.thr);
            acc[0] = acc[0] + (double)f32_mul(x, q);
            acc[1] = acc[1] + (double)f32_mul(q, q);
        }
    }
#pragma unroll
    for (int a = 0; a < NACC; ++a) {
        const double s = wave_sum_f64(acc[a]);
        if (lane == 0) row_sums[(size_t)a * n + row] = s;
    }
    if constexpr (PASS == WQ_ABS_STATS) {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        if (lane == 0) row_max[row] = mx;
    }
}

// One wavefront: combines the row sums of every accumulator (lane l takes rows l, l+64, ...; butterfly) and derives
// the scalars of the next stage.  method: TernaryMethod 0..4; custom <= 0: the method's own factor.
template <int PASS>
__global__ __launch_bounds__(64) void wq_final_kernel(const double *row_sums, const float *row_max, size_t n, size_t k,
                                                      WqState *state, int method, float outlier_threshold, float custom)
{
    constexpr int NACC = PASS == WQ_OPTIMAL ? 10 : ((PASS == WQ_CLIP_STATS || PASS == WQ_SCALE) ? 2 : 1);
    const int lane = threadIdx.x;
    double tot[NACC];
#pragma unroll
    for (int a = 0; a < NACC; ++a) {
        double s = 0.0;
        for (size_t r = lane; r < n; r += 64) s = s + row_sums[(size_t)a * n + r];
        tot[a] = wave_sum_f64(s);
    }
    float mx = 0.0f;
    if constexpr (PASS == WQ_ABS_STATS) {
        for (size_t r = lane; r < n; r += 64) mx = fmaxf(mx, row_max[r]);
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    }
    if (lane != 0) return;
    const double count = (double)n * (double)k;
    WqState st = *state;
    if constexpr (PASS == WQ_SUM) {
        st.mean = (float)(tot[0] / count);
    } else if constexpr (PASS == WQ_SQDIFF) {
        const float var = (float)(tot[0] / count);
        st.sd = f32_sqrt(var + 1e-8f);
    } else if constexpr (PASS == WQ_CLIP_STATS) {
        st.clip_mean = (float)(tot[0] / count);
        st.clip_mad = (float)(tot[1] / count);
        const float spread = f32_mul(outlier_threshold, st.clip_mad);
        st.lo = st.clip_mean - spread;
        st.hi = st.clip_mean + spread;
    } else if constexpr (PASS == WQ_ABS_STATS) {
        st.mean_abs = (float)(tot[0] / count);
        st.max_abs = mx;
        const bool has_custom = custom > 0.0f;
        float thr;
        if (method == 1) thr = f32_mul(st.mean_abs, has_custom ? custom : 0.8f);
        else if (method == 2)
            thr = has_custom ? f32_mul(st.mean_abs, custom)
                             : (st.max_abs > f32_mul(3.0f, st.mean_abs) ? f32_mul(st.mean_abs, 0.5f) : f32_mul(st.mean_abs, 0.7f));
        else thr = f32_mul(st.mean_abs, has_custom ? custom : 0.7f);  // mean, DetSTE; optimal without its search
        st.thr = thr;
    } else if constexpr (PASS == WQ_OPTIMAL) {
        float best = __builtin_inff(), thr = f32_mul(st.mean_abs, 0.7f);
#pragma unroll
        for (int f = 0; f < 10; ++f) {
            const float mse = (float)(tot[f] / count);
            if (mse < best) { best = mse; thr = f32_mul(st.mean_abs, wq_factors[f]); }
        }
        st.thr = thr;
    } else {
        st.num = (float)tot[0];
        st.den = (float)tot[1];
        st.scale = fabsf(st.den) < 1.1920929e-07f ? 1.0f : f32_div(st.num, st.den);
    }
    *state = st;
}

__global__ void wq_init_kernel(WqState *state)
{
    WqState st;
    st.mean = 0.0f; st.sd = 1.0f; st.clip_mean = 0.0f; st.clip_mad = 0.0f; st.lo = -__builtin_inff(); st.hi = __builtin_inff();
    st.mean_abs = 0.0f; st.max_abs = 0.0f; st.thr = 0.0f; st.num = 0.0f; st.den = 0.0f; st.scale = 1.0f;
    *state = st;
}

// Ternarise the processed tensor with the threshold found, pack; thread b builds byte b.  Also publishes the scale and
// (optionally) the twelve scalars.
__global__ __launch_bounds__(256) void wq_ternarize_pack_kernel(const float *w, size_t count, const WqState *state, int normalize,
                                                                int clip, uint8_t *packed, int8_t *q_i8, size_t nbytes)
{
    size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nbytes) return;
    const WqState st = *state;
    unsigned byte = 0;
    for (int j = 0; j < 4; ++j) {
        size_t i = 4 * b + j;
        if (i < count) {
            const int t = (int)wq_code(wq_processed(w[i], st, normalize != 0, clip != 0), st.thr);
            if (q_i8) q_i8[i] = (int8_t)t;
            byte |= ((unsigned)(t + 1) & 3u) << (2 * j);
        }
    }
    packed[b] = (uint8_t)byte;
}

__global__ void wq_publish_kernel(const WqState *state, int clip, float *w_scale, float *stats)
{
    const WqState st = *state;
    *w_scale = st.scale;
    if (stats) {
        const float v[12] = {st.mean, st.sd, st.clip_mean, st.clip_mad, clip ? st.lo : 0.0f, clip ? st.hi : 0.0f,
                             st.mean_abs, st.max_abs, st.thr, st.num, st.den, st.scale};
        for (int i = 0; i < 12; ++i) stats[i] = v[i];
    }
}

__device__ __forceinline__ unsigned code_at(const uint8_t *packed, size_t e)
{
    return (packed[e >> 2] >> (2 * (e & 3))) & 3u;
}

// One thread builds one dword (16 weights of one row) of the tiled layout.
__global__ __launch_bounds__(256) void retile_kernel(const uint8_t *packed, size_t n, size_t k, int layout,
                                                     uint32_t *tiled, size_t kt_count, size_t total_dwords)
{
    size_t d = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (d >= total_dwords) return;
    size_t tile = d >> 8;
    unsigned wd = (unsigned)(d & 255);
    unsigned slot = wd >> 2, t = wd & 3;
    unsigned r = slot & 15, g = 4 * t + (slot >> 4);
    size_t rb = tile / kt_count, kt = tile % kt_count;
    size_t row = rb * TILE_ROWS + r;
    size_t kbase = kt * TILE_K + (size_t)g * 16;
    uint32_t word = 0;
    for (int j = 0; j < 16; ++j) {
        size_t kk = kbase + j;
        unsigned code = 1;
        if (row < n && kk < k) {
            size_t e = layout == BITNET_HIP_LAYOUT_OUT_IN ? row * k + kk : kk * n + row;
            code = code_at(packed, e);
            if (code == 3) code = 1;
        }
        word |= code << (2 * (j >> 2) + 8 * (j & 3));
    }
    tiled[d] = word;
}

// Inverse: one thread rebuilds one byte of the flat [n, k] packing.
__global__ __launch_bounds__(256) void untile_kernel(const uint32_t *tiled, size_t n, size_t k, uint8_t *packed,
                                                     size_t kt_count, size_t nbytes)
{
    size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nbytes) return;
    const size_t count = n * k;
    unsigned byte = 0;
    for (int j = 0; j < 4; ++j) {
        size_t e = 4 * b + j;
        if (e >= count) break;
        size_t row = e / k, kk = e % k;
        size_t tile = (row / TILE_ROWS) * kt_count + kk / TILE_K;
        unsigned g = (unsigned)((kk % TILE_K) / 16), c = (unsigned)(kk % 16);
        unsigned wd = (((g & 3) * 16 + (unsigned)(row % TILE_ROWS)) << 2) + (g >> 2);
        uint32_t word = tiled[tile * 256 + wd];
        byte |= ((word >> (2 * (c >> 2) + 8 * (c & 3))) & 3u) << (2 * j);
    }
    packed[b] = (uint8_t)byte;
}

inline unsigned blocks_for(size_t items, unsigned per_block) { return (unsigned)((items + per_block - 1) / per_block); }

}  // namespace

int launch_pack_2bit(const int8_t *q, size_t count, uint8_t *packed, hipStream_t stream)
{
    size_t nbytes = (count + 3) / 4;
    if (nbytes == 0) return BITNET_HIP_OK;
    hipLaunchKernelGGL(pack_2bit_kernel, dim3(blocks_for(nbytes, 256)), dim3(256), 0, stream, q, count, packed, nbytes);
    BITNET_HIP_CHECK_LAUNCH("pack_2bit_kernel");
    return BITNET_HIP_OK;
}

int launch_unpack_2bit(const uint8_t *packed, size_t count, int8_t *q, hipStream_t stream)
{
    if (count == 0) return BITNET_HIP_OK;
    hipLaunchKernelGGL(unpack_2bit_kernel, dim3(blocks_for(count, 256)), dim3(256), 0, stream, packed, count, q);
    BITNET_HIP_CHECK_LAUNCH("unpack_2bit_kernel");
    return BITNET_HIP_OK;
}

int launch_lookup_compute(int kind, const int8_t *w, const float *x, float *out, size_t n, hipStream_t stream)
{
    if (n == 0) return BITNET_HIP_OK;
    hipLaunchKernelGGL(lookup_compute_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, stream, kind, w, x, out, n);
    BITNET_HIP_CHECK_LAUNCH("lookup_compute_kernel");
    return BITNET_HIP_OK;
}

int launch_pack_base3(const int8_t *q, size_t count, uint8_t *packed, hipStream_t stream)
{
    size_t nbytes = (count + 4) / 5;
    if (nbytes == 0) return BITNET_HIP_OK;
    hipLaunchKernelGGL(pack_base3_kernel, dim3(blocks_for(nbytes, 256)), dim3(256), 0, stream, q, count, packed, nbytes);
    BITNET_HIP_CHECK_LAUNCH("pack_base3_kernel");
    return BITNET_HIP_OK;
}

int launch_unpack_base3(const uint8_t *packed, size_t count, int8_t *q, hipStream_t stream)
{
    if (count == 0) return BITNET_HIP_OK;
    hipLaunchKernelGGL(unpack_base3_kernel, dim3(blocks_for(count, 256)), dim3(256), 0, stream, packed, count, q);
    BITNET_HIP_CHECK_LAUNCH("unpack_base3_kernel");
    return BITNET_HIP_OK;
}

int launch_base3_to_2bit(const uint8_t *base3, size_t count, uint8_t *packed, hipStream_t stream)
{
    size_t nbytes = (count + 3) / 4;
    if (nbytes == 0) return BITNET_HIP_OK;
    hipLaunchKernelGGL(base3_to_2bit_kernel, dim3(blocks_for(nbytes, 256)), dim3(256), 0, stream, base3, count, packed, nbytes);
    BITNET_HIP_CHECK_LAUNCH("base3_to_2bit_kernel");
    return BITNET_HIP_OK;
}

int launch_quantize_weights(const float *w, size_t n, size_t k, int method, float threshold_factor,
                            double *row_sums, uint8_t *packed, float *w_scale, int8_t *q_i8, hipStream_t stream)
{
    if (n > 0 && k > 0) {
        hipLaunchKernelGGL(absmean_rows_kernel, dim3(blocks_for(n, 4)), dim3(64, 4), 0, stream, w, n, k, row_sums);
        BITNET_HIP_CHECK_LAUNCH("absmean_rows_kernel");
    }
    hipLaunchKernelGGL(absmean_final_kernel, dim3(1), dim3(64), 0, stream, row_sums, n, k, w_scale);
    BITNET_HIP_CHECK_LAUNCH("absmean_final_kernel");
    size_t count = n * k, nbytes = (count + 3) / 4;
    if (nbytes == 0) return BITNET_HIP_OK;
    hipLaunchKernelGGL(ternarize_pack_kernel, dim3(blocks_for(nbytes, 256)), dim3(256), 0, stream, w, count,
                       method, threshold_factor, w_scale, packed, q_i8, nbytes);
    BITNET_HIP_CHECK_LAUNCH("ternarize_pack_kernel");
    return BITNET_HIP_OK;
}

size_t quantize_weights_reference_scratch_bytes(size_t n)
{
    return sizeof(double) * WQ_MAX_ACC * (n ? n : 1) + sizeof(float) * (n ? n : 1) + 256;
}

int launch_quantize_weights_reference(const float *w, size_t n, size_t k, int method, int normalize, float outlier_threshold,
                                      float custom_factor, void *scratch, uint8_t *packed, float *w_scale, int8_t *q_i8,
                                      float *stats, hipStream_t stream)
{
    // scratch: WqState (256 bytes reserved), then WQ_MAX_ACC * n doubles, then n floats
    WqState *state = static_cast<WqState *>(scratch);
    double *row_sums = reinterpret_cast<double *>(static_cast<uint8_t *>(scratch) + 256);
    float *row_max = reinterpret_cast<float *>(row_sums + WQ_MAX_ACC * (n ? n : 1));
    const int clip = outlier_threshold > 0.0f ? 1 : 0;
    hipLaunchKernelGGL(wq_init_kernel, dim3(1), dim3(1), 0, stream, state);
    BITNET_HIP_CHECK_LAUNCH("wq_init_kernel");
    const size_t count = n * k, nbytes = (count + 3) / 4;
    if (count != 0) {
        const dim3 rgrid(blocks_for(n, 4)), rblock(64, 4);
#define BITNET_WQ_PASS(PASS)                                                                                              \
    do {                                                                                                                  \
        hipLaunchKernelGGL((wq_rows_kernel<PASS>), rgrid, rblock, 0, stream, w, n, k, state, normalize, clip, row_sums,  \
                           row_max);                                                                                      \
        BITNET_HIP_CHECK_LAUNCH("wq_rows_kernel");                                                                        \
        hipLaunchKernelGGL((wq_final_kernel<PASS>), dim3(1), dim3(64), 0, stream, row_sums, row_max, n, k, state, method, \
                           outlier_threshold, custom_factor);                                                             \
        BITNET_HIP_CHECK_LAUNCH("wq_final_kernel");                                                                       \
    } while (0)
        if (normalize) {
            BITNET_WQ_PASS(WQ_SUM);
            BITNET_WQ_PASS(WQ_SQDIFF);
        }
        if (clip) BITNET_WQ_PASS(WQ_CLIP_STATS);
        BITNET_WQ_PASS(WQ_ABS_STATS);
        if (method == 3 && !(custom_factor > 0.0f)) BITNET_WQ_PASS(WQ_OPTIMAL);
        BITNET_WQ_PASS(WQ_SCALE);
#undef BITNET_WQ_PASS
        hipLaunchKernelGGL(wq_ternarize_pack_kernel, dim3(blocks_for(nbytes, 256)), dim3(256), 0, stream, w, count, state,
                           normalize, clip, packed, q_i8, nbytes);
        BITNET_HIP_CHECK_LAUNCH("wq_ternarize_pack_kernel");
    }
    hipLaunchKernelGGL(wq_publish_kernel, dim3(1), dim3(1), 0, stream, state, clip, w_scale, stats);
    BITNET_HIP_CHECK_LAUNCH("wq_publish_kernel");
    return BITNET_HIP_OK;
}

int launch_retile(const uint8_t *packed, size_t n, size_t k, int layout, uint8_t *tiled, hipStream_t stream)
{
    size_t total_dwords = tiled_bytes(n, k) / 4;
    if (total_dwords == 0) return BITNET_HIP_OK;
    hipLaunchKernelGGL(retile_kernel, dim3(blocks_for(total_dwords, 256)), dim3(256), 0, stream, packed, n, k,
                       layout, reinterpret_cast<uint32_t *>(tiled), k_tiles(k), total_dwords);
    BITNET_HIP_CHECK_LAUNCH("retile_kernel");
    return BITNET_HIP_OK;
}

int launch_untile(const uint8_t *tiled, size_t n, size_t k, uint8_t *packed, hipStream_t stream)
{
    size_t nbytes = (n * k + 3) / 4;
    if (nbytes == 0) return BITNET_HIP_OK;
    hipLaunchKernelGGL(untile_kernel, dim3(blocks_for(nbytes, 256)), dim3(256), 0, stream,
                       reinterpret_cast<const uint32_t *>(tiled), n, k, packed, k_tiles(k), nbytes);
    BITNET_HIP_CHECK_LAUNCH("untile_kernel");
    return BITNET_HIP_OK;
}

}  // namespace bitnet
