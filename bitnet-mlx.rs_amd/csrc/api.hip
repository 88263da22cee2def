// extern "C" entry points: argument validation, error records, and the BitLinear / decoder objects.
// No arithmetic lives here; every result comes from the kernels behind the launch_* functions.
#include <cstring>
#include <memory>
#include <mutex>
#include <new>
#include <shared_mutex>
#include <vector>

#include "kernels.hpp"

namespace bitnet {

ErrorRecord &error_record()
{
    static thread_local ErrorRecord rec;
    return rec;
}

int fail(int code, const char *fmt, ...)
{
    ErrorRecord &r = error_record();
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(r.msg, sizeof r.msg, fmt, ap);
    va_end(ap);
    return code;
}

int fail_shape(const size_t *expected, int erank, const size_t *actual, int arank, const char *what)
{
    ErrorRecord &r = error_record();
    r.expected_rank = erank > 4 ? 4 : erank;
    r.actual_rank = arank > 4 ? 4 : arank;
    for (int i = 0; i < r.expected_rank; ++i) r.expected[i] = expected[i];
    for (int i = 0; i < r.actual_rank; ++i) r.actual[i] = actual[i];
    char e[96] = {0}, a[96] = {0};
    size_t eo = 0, ao = 0;
    for (int i = 0; i < r.expected_rank; ++i)
        eo += snprintf(e + eo, sizeof e - eo, i ? ", %zu" : "%zu", expected[i]);
    for (int i = 0; i < r.actual_rank; ++i)
        ao += snprintf(a + ao, sizeof a - ao, i ? ", %zu" : "%zu", actual[i]);
    snprintf(r.msg, sizeof r.msg, "Shape mismatch (%s): expected [%s], got [%s]", what, e, a);
    return BITNET_HIP_SHAPE_MISMATCH;
}

namespace {

// Device buffer freed when it goes out of scope (after the stream it was used on has been drained).
struct DeviceTemp {
    void *ptr = nullptr;
    ~DeviceTemp() { if (ptr) (void)hipFree(ptr); }
    int alloc(size_t bytes)
    {
        hipError_t e = hipMalloc(&ptr, bytes ? bytes : 1);
        if (e != hipSuccess) {
            ptr = nullptr;
            return fail(BITNET_HIP_MEMORY_ERROR, "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
        }
        return BITNET_HIP_OK;
    }
};

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace

}  // namespace bitnet

using namespace bitnet;

// ---------------------------------------------------------------------------------------------------
// Static scratch of bitnet_hip_bitlinear_forward_noalloc: the quantised activations of one call
// (int8 [m, in], a_scale [m], a_sum [m]) live in this file-scope device array instead of a workspace the
// caller passes or the call allocates.  Every GPU the library runs on holds its own copy until the process
// ends.  In host code the array's name is only a handle for hipGetSymbolAddress: the address each device
// gave it is looked up once per device and kept in noalloc_scratch_ptr; kernels only ever get that pointer.
// ---------------------------------------------------------------------------------------------------
namespace {
constexpr size_t NOALLOC_MAX_ELEMS = (size_t)1 << 20;  // m * in_features of one call
constexpr size_t NOALLOC_MAX_ROWS = 4096;              // m of one call
constexpr size_t NOALLOC_SCRATCH_BYTES = NOALLOC_MAX_ELEMS + 2 * NOALLOC_MAX_ROWS * sizeof(float) + 512;
constexpr int NOALLOC_MAX_DEVICES = 64;
}  // namespace

static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];

namespace {
std::mutex noalloc_lock;
void *noalloc_scratch_ptr[NOALLOC_MAX_DEVICES] = {};

// Device address of `scratch` on the current device (looked up on first use, per device).
int noalloc_scratch(void **out)
{
    int device = 0;
    BITNET_HIP_TRY(hipGetDevice(&device));
    if (device < 0 || device >= NOALLOC_MAX_DEVICES)
        return fail(BITNET_HIP_UNSUPPORTED, "device ordinal %d is beyond the %d this library keeps scratch for", device,
                    NOALLOC_MAX_DEVICES);
    std::lock_guard<std::mutex> guard(noalloc_lock);
    if (!noalloc_scratch_ptr[device]) {
        void *ptr = nullptr;
        BITNET_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return fail(BITNET_HIP_DEVICE_ERROR, "hipGetSymbolAddress returned no address for the static scratch");
        noalloc_scratch_ptr[device] = ptr;
    }
    *out = noalloc_scratch_ptr[device];
    return BITNET_HIP_OK;
}
}  // namespace

// ---------------------------------------------------------------------------------------------------
// BitLinear object
// ---------------------------------------------------------------------------------------------------
struct bitnet_hip_bitlinear {
    size_t in_features = 0;
    size_t out_features = 0;
    bool use_bias = false;
    bool has_weights = false;
    uint8_t *packed = nullptr;  // reference byte format, [out, in] flat
    uint8_t *tiled = nullptr;   // streaming layout
    float *w_scale = nullptr;   // one float, device
    float *bias = nullptr;      // [out], device (zeros until set, like the reference's Tensor::zeros)
    // readers: forward; writer: set_weights / set_bias (the reference guards weights with a RwLock)
    mutable std::shared_mutex lock;

    ~bitnet_hip_bitlinear()
    {
        if (packed) (void)hipFree(packed);
        if (tiled) (void)hipFree(tiled);
        if (w_scale) (void)hipFree(w_scale);
        if (bias) (void)hipFree(bias);
    }
};

namespace {

// Row blocks of the largest launch group (up to GEMV_MAX_PROJ projections share a decode launch).
size_t launch_group_blocks(bitnet_hip_bitlinear *const *layers, size_t count)
{
    size_t most = 0;
    for (size_t j0 = 0; j0 < count; j0 += GEMV_MAX_PROJ) {
        size_t sum = 0;
        for (size_t j = j0; j < count && j < j0 + GEMV_MAX_PROJ; ++j) sum += row_blocks(layers[j]->out_features);
        most = sum > most ? sum : most;
    }
    return most;
}

// Runs `count` projections that share one input row block [m, k].  At decode token counts the quantiser runs
// inside the GEMV launch (up to GEMV_MAX_PROJ projections per launch); otherwise the stand-alone quantiser
// fills q / a_scale / a_sum (scratch the caller provides) and the GEMV or GEMM kernels consume them.
// residual / out / acc are per-projection arrays (entries of residual and acc may be null, and so may the arrays).
int run_projections(bitnet_hip_bitlinear *const *layers, int count, const float *x, const float *x2, size_t ldx,
                    size_t m, int input_mode, size_t gqa_group, size_t head_dim, const float *gamma, float eps,
                    int sum_order, const float *const *residual, float *const *out, int32_t *const *acc, int8_t *q,
                    float *a_scale, int32_t *a_sum, bool want_quant_outputs, hipStream_t s,
                    const GemmSplitScratch *split = nullptr)
{
    const size_t k = layers[0]->in_features;
    auto proj_of = [&](int j) {
        bitnet_hip_bitlinear *bl = layers[j];
        GemvProj pj = {bl->tiled, bl->w_scale, bl->use_bias ? bl->bias : nullptr, residual ? residual[j] : nullptr,
                       out[j], acc ? acc[j] : nullptr, bl->out_features};
        return pj;
    };
    if (gemv_fused_supported(x, x2, ldx, m, k, input_mode, head_dim, gamma, sum_order, launch_group_blocks(layers, count))) {
        for (int j0 = 0; j0 < count; j0 += GEMV_MAX_PROJ) {
            GemvProj pjs[GEMV_MAX_PROJ];
            const int nj = count - j0 < GEMV_MAX_PROJ ? count - j0 : GEMV_MAX_PROJ;
            for (int j = 0; j < nj; ++j) pjs[j] = proj_of(j0 + j);
            const bool first = j0 == 0 && want_quant_outputs;
            int rc = launch_gemv_fused(pjs, nj, x, x2, ldx, m, k, input_mode, gqa_group, head_dim, gamma, eps, sum_order,
                                       first ? q : nullptr, first ? a_scale : nullptr, first ? a_sum : nullptr, s);
            if (rc != BITNET_HIP_OK) return rc;
        }
        return BITNET_HIP_OK;
    }
    if (!q || !a_scale || !a_sum) return fail(BITNET_HIP_MEMORY_ERROR, "projection: no scratch for the quantised activations");
    size_t n_blocks = 0;
    for (int j = 0; j < count; ++j) n_blocks += row_blocks(layers[j]->out_features);
    // A GEMM that splits k across workgroups finds its tile counters zeroed by the quantiser launched in front of it.  One
    // scratch serves one launch: more projections than one launch takes run without the split.
    const bool use_split = split && split->counters && count <= GEMM_MAX_PROJ && !gemv_takes(m, k, n_blocks, q);
    int rc = launch_act_quant(x, x2, ldx, m, k, input_mode, gqa_group, head_dim, gamma, eps, sum_order, q, a_scale, a_sum,
                              nullptr, s, use_split ? split->counters : nullptr, use_split ? split->counter_count : 0);
    if (rc != BITNET_HIP_OK) return rc;
    if (gemv_takes(m, k, n_blocks, q)) {
        for (int j0 = 0; j0 < count; j0 += GEMV_MAX_PROJ) {
            GemvProj pjs[GEMV_MAX_PROJ];
            const int nj = count - j0 < GEMV_MAX_PROJ ? count - j0 : GEMV_MAX_PROJ;
            for (int j = 0; j < nj; ++j) pjs[j] = proj_of(j0 + j);
            rc = launch_gemv_tiled(pjs, nj, q, a_scale, m, k, s);
            if (rc != BITNET_HIP_OK) return rc;
        }
        return BITNET_HIP_OK;
    }
    for (int j0 = 0; j0 < count; j0 += GEMM_MAX_PROJ) {
        GemvProj pjs[GEMM_MAX_PROJ];
        const int nj = count - j0 < GEMM_MAX_PROJ ? count - j0 : GEMM_MAX_PROJ;
        for (int j = 0; j < nj; ++j) pjs[j] = proj_of(j0 + j);
        rc = launch_gemm_multi(pjs, nj, q, a_sum, a_scale, m, k, s, use_split ? split : nullptr);  // all of them in one launch where that applies
        if (rc == BITNET_HIP_UNSUPPORTED) {
            for (int j = 0; j < nj; ++j) {
                const GemvProj &pj = pjs[j];
                rc = launch_gemm_tiled(pj.tiled, q, a_sum, m, pj.n, k, pj.acc, pj.w_scale, a_scale, pj.bias, pj.residual,
                                       pj.out, s);
                if (rc != BITNET_HIP_OK) return rc;
            }
        } else if (rc != BITNET_HIP_OK) {
            return rc;
        }
    }
    return BITNET_HIP_OK;
}

// Scratch for the quantised activations of m rows of width k: q [m*k] int8, a_scale [m] f32, a_sum [m] int32.
struct QuantScratch {
    int8_t *q;
    float *a_scale;
    int32_t *a_sum;
};
size_t quant_scratch_bytes(size_t m, size_t k) { return align_up(m * k, 256) + 2 * align_up(m * sizeof(float), 256) + 256; }
QuantScratch carve_scratch(void *ws, size_t m, size_t k)
{
    uintptr_t base = align_up(reinterpret_cast<uintptr_t>(ws), 256);
    QuantScratch sc;
    sc.q = reinterpret_cast<int8_t *>(base);
    sc.a_scale = reinterpret_cast<float *>(base + align_up(m * k, 256));
    sc.a_sum = reinterpret_cast<int32_t *>(base + align_up(m * k, 256) + align_up(m * sizeof(float), 256));
    return sc;
}

// Scratch of a GEMM that splits k across workgroups, behind the quantised activations in the same workspace.
size_t split_scratch_bytes(size_t m, size_t k, size_t n)
{
    size_t partial_bytes = 0, counters = 0;
    gemm_split_plan(m, k, &n, 1, &partial_bytes, &counters);
    return partial_bytes ? partial_bytes + align_up(counters * sizeof(unsigned), 256) : 0;
}
GemmSplitScratch carve_split(void *ws, size_t m, size_t k, size_t n)
{
    GemmSplitScratch sp;
    gemm_split_plan(m, k, &n, 1, &sp.partial_bytes, &sp.counter_count);
    if (sp.partial_bytes == 0) return sp;
    const uintptr_t base = align_up(reinterpret_cast<uintptr_t>(ws), 256) + quant_scratch_bytes(m, k) - 256;  // behind a_sum: quant_scratch_bytes counts 256 bytes of alignment slack
    sp.partials = reinterpret_cast<int32_t *>(base);
    sp.counters = reinterpret_cast<unsigned *>(base + sp.partial_bytes);
    return sp;
}

}  // namespace

extern "C" {

const char *bitnet_hip_last_error(void) { return error_record().msg; }

int bitnet_hip_last_shape_mismatch(size_t expected[4], size_t actual[4], int *actual_rank)
{
    ErrorRecord &r = error_record();
    for (int i = 0; i < r.expected_rank; ++i) expected[i] = r.expected[i];
    for (int i = 0; i < r.actual_rank; ++i) actual[i] = r.actual[i];
    if (actual_rank) *actual_rank = r.actual_rank;
    return r.expected_rank;
}

int bitnet_hip_init(int device)
{
    int count = 0;
    BITNET_HIP_TRY(hipGetDeviceCount(&count));
    if (device < 0 || device >= count)
        return fail(BITNET_HIP_INVALID_CONFIG, "device %d out of range (%d visible)", device, count);
    BITNET_HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    BITNET_HIP_TRY(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(BITNET_HIP_UNSUPPORTED, "device %d is %s; this library carries gfx950 code only", device,
                    prop.gcnArchName);
    void *ptr = nullptr;
    return noalloc_scratch(&ptr);  // this device's address of the static scratch, kept for forward_noalloc
}

int bitnet_hip_device_info(char *arch_name, size_t arch_name_len, int *compute_units, int *clock_mhz,
                           size_t *total_mem_bytes)
{
    int device = 0;
    BITNET_HIP_TRY(hipGetDevice(&device));
    hipDeviceProp_t prop;
    BITNET_HIP_TRY(hipGetDeviceProperties(&prop, device));
    if (arch_name && arch_name_len) {
        strncpy(arch_name, prop.gcnArchName, arch_name_len - 1);
        arch_name[arch_name_len - 1] = 0;
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (clock_mhz) *clock_mhz = prop.clockRate / 1000;
    if (total_mem_bytes) *total_mem_bytes = prop.totalGlobalMem;
    return BITNET_HIP_OK;
}

int bitnet_hip_measure_mfma_i8_rate(int random_operands, double *tera_ops_per_second, void *stream)
{
    if (!tera_ops_per_second) return fail(BITNET_HIP_NULL_POINTER, "measure_mfma_i8_rate: the result pointer is required");
    int device = 0, units = 0;
    BITNET_HIP_TRY(hipGetDevice(&device));
    BITNET_HIP_TRY(hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device));
    DeviceTemp sink;
    int rc = sink.alloc((size_t)units * MFMA_RATE_THREADS * sizeof(int));
    if (rc != BITNET_HIP_OK) return rc;
    struct Events {
        hipEvent_t e[2] = {nullptr, nullptr};
        ~Events() { for (hipEvent_t v : e) if (v) (void)hipEventDestroy(v); }
    } ev;
    BITNET_HIP_TRY(hipEventCreate(&ev.e[0]));
    BITNET_HIP_TRY(hipEventCreate(&ev.e[1]));
    hipStream_t s = as_stream(stream);
    const int iters = 20000;  // about 2.5 ms
    rc = launch_mfma_rate(random_operands != 0, 200, units, static_cast<int *>(sink.ptr), s);  // warm-up
    if (rc != BITNET_HIP_OK) return rc;
    BITNET_HIP_TRY(hipEventRecord(ev.e[0], s));
    rc = launch_mfma_rate(random_operands != 0, iters, units, static_cast<int *>(sink.ptr), s);
    if (rc != BITNET_HIP_OK) return rc;
    BITNET_HIP_TRY(hipEventRecord(ev.e[1], s));
    BITNET_HIP_TRY(hipEventSynchronize(ev.e[1]));  // the sink is freed on return: nothing of the launch is left running
    float ms = 0.0f;
    BITNET_HIP_TRY(hipEventElapsedTime(&ms, ev.e[0], ev.e[1]));
    // 2 * 16 * 16 * 64 operations per instruction
    const double ops = 32768.0 * MFMA_RATE_PER_ITER * (double)iters * (MFMA_RATE_THREADS / 64) * (double)units;
    *tera_ops_per_second = ops / ((double)ms * 1e-3) / 1e12;
    return BITNET_HIP_OK;
}

// ---- activation side ------------------------------------------------------------------------------

int bitnet_hip_quantize_activations_i8(const float *x, const float *x2, size_t ldx, size_t m, size_t k,
                                       int input_mode, size_t gqa_group, size_t head_dim, const float *gamma,
                                       float eps, int sum_order, int8_t *q, float *a_scale, int32_t *a_sum,
                                       float *y_f32, void *stream)
{
    if (m == 0 || k == 0) return BITNET_HIP_OK;
    if (!x || !q || !a_scale) return fail(BITNET_HIP_NULL_POINTER, "quantize_activations_i8: x, q and a_scale are required");
    if (k > 0x7fffffffu) return fail(BITNET_HIP_UNSUPPORTED, "quantize_activations_i8: k=%zu too large", k);
    if (sum_order != BITNET_HIP_SUM_SEQUENTIAL && sum_order != BITNET_HIP_SUM_BLOCK256)
        return fail(BITNET_HIP_INVALID_CONFIG, "quantize_activations_i8: unknown sum_order %d", sum_order);
    size_t src_cols = k;
    switch (input_mode) {
        case BITNET_HIP_INPUT_PLAIN: break;
        case BITNET_HIP_INPUT_RELU2_MUL:
            if (!x2) return fail(BITNET_HIP_NULL_POINTER, "quantize_activations_i8: RELU2_MUL needs x2");
            break;
        case BITNET_HIP_INPUT_GQA_BROADCAST:
            if (gqa_group == 0 || head_dim == 0 || k % (gqa_group * head_dim) != 0)
                return fail(BITNET_HIP_INVALID_CONFIG,
                            "quantize_activations_i8: k=%zu is not a multiple of gqa_group*head_dim=%zu*%zu", k,
                            gqa_group, head_dim);
            src_cols = k / gqa_group;
            break;
        default: return fail(BITNET_HIP_INVALID_CONFIG, "quantize_activations_i8: unknown input_mode %d", input_mode);
    }
    if (ldx < src_cols) {
        size_t e[2] = {m, src_cols}, a[2] = {m, ldx};
        return fail_shape(e, 2, a, 2, "row stride smaller than the row");
    }
    return launch_act_quant(x, x2, ldx, m, k, input_mode, gqa_group, head_dim, gamma, eps, sum_order, q, a_scale,
                            a_sum, y_f32, as_stream(stream));
}

int bitnet_hip_absmax_quantize_activations(const float *x, size_t count, int precision, int8_t *values, float *stats,
                                           void *stream)
{
    if (precision != BITNET_HIP_PRECISION_ONE_FIVE_FIVE_BIT && precision != BITNET_HIP_PRECISION_EIGHT_BIT)
        return fail(BITNET_HIP_UNSUPPORTED, "absmax_quantize_activations: unsupported precision %d", precision);
    if (!stats) return fail(BITNET_HIP_NULL_POINTER, "absmax_quantize_activations: stats is required");
    if (count != 0 && (!x || !values)) return fail(BITNET_HIP_NULL_POINTER, "absmax_quantize_activations: null buffer");
    DeviceTemp scratch;
    int rc = scratch.alloc(absmax_quantize_scratch_bytes(count));
    if (rc != BITNET_HIP_OK) return rc;
    rc = launch_absmax_quantize(x, count, precision, scratch.ptr, values, stats, as_stream(stream));
    if (rc != BITNET_HIP_OK) return rc;
    BITNET_HIP_TRY(hipStreamSynchronize(as_stream(stream)));  // the scratch is released on return
    return BITNET_HIP_OK;
}

int bitnet_hip_abs_max(const float *x, size_t count, float *abs_max, void *stream)
{
    if (!abs_max) return fail(BITNET_HIP_NULL_POINTER, "abs_max: the result pointer is required");
    *abs_max = 0.0f;
    if (count == 0) return BITNET_HIP_OK;
    if (!x) return fail(BITNET_HIP_NULL_POINTER, "abs_max: null buffer");
    DeviceTemp scratch;
    int rc = scratch.alloc(absmax_quantize_scratch_bytes(count));
    if (rc != BITNET_HIP_OK) return rc;
    rc = launch_abs_max(x, count, scratch.ptr, as_stream(stream));
    if (rc != BITNET_HIP_OK) return rc;
    BITNET_HIP_TRY(hipMemcpyAsync(abs_max, scratch.ptr, sizeof(float), hipMemcpyDeviceToHost, as_stream(stream)));
    BITNET_HIP_TRY(hipStreamSynchronize(as_stream(stream)));  // the value is the caller's on return, as to_scalar() is
    return BITNET_HIP_OK;
}

int bitnet_hip_quantize_activations_scaled(const float *x, size_t count, int precision, float scale, int reference_u8,
                                           int8_t *values, void *stream)
{
    if (precision != BITNET_HIP_PRECISION_ONE_FIVE_FIVE_BIT && precision != BITNET_HIP_PRECISION_EIGHT_BIT)
        return fail(BITNET_HIP_UNSUPPORTED, "quantize_activations_scaled: unsupported precision %d", precision);
    if (count != 0 && (!x || !values)) return fail(BITNET_HIP_NULL_POINTER, "quantize_activations_scaled: null buffer");
    return launch_scaled_quantize(x, count, precision, scale, reference_u8 != 0, values, as_stream(stream));
}

// ---- lookup-table kernels ----------------------------------------------------------------------------

int bitnet_hip_lookup_compute(int kind, const int8_t *weights, size_t n_weights, const float *inputs, size_t n_inputs,
                              float *output, size_t n_output, void *stream)
{
    if (kind != BITNET_HIP_LOOKUP_TERNARY && kind != BITNET_HIP_LOOKUP_I2S)
        return fail(BITNET_HIP_INVALID_CONFIG, "lookup_compute: unknown kind %d", kind);
    if (n_weights == 0 || n_inputs == 0 || n_output == 0) return fail(BITNET_HIP_INVALID_CONFIG, "Empty input arrays");
    if (!weights || !inputs || !output) return fail(BITNET_HIP_NULL_POINTER, "lookup_compute: null buffer");
    size_t n = n_weights < n_inputs ? n_weights : n_inputs;
    if (n_output < n) n = n_output;
    return launch_lookup_compute(kind, weights, inputs, output, n, as_stream(stream));
}

// ---- weight side -----------------------------------------------------------------------------------

size_t bitnet_hip_packed_size(size_t count) { return (count + 3) / 4; }

int bitnet_hip_pack_ternary_2bit(const int8_t *q, size_t count, uint8_t *packed, void *stream)
{
    if (count == 0) return BITNET_HIP_OK;
    if (!q || !packed) return fail(BITNET_HIP_NULL_POINTER, "pack_ternary_2bit: null buffer");
    return launch_pack_2bit(q, count, packed, as_stream(stream));
}

int bitnet_hip_unpack_ternary_2bit(const uint8_t *packed, size_t count, int8_t *q, void *stream)
{
    if (count == 0) return BITNET_HIP_OK;
    if (!q || !packed) return fail(BITNET_HIP_NULL_POINTER, "unpack_ternary_2bit: null buffer");
    return launch_unpack_2bit(packed, count, q, as_stream(stream));
}

size_t bitnet_hip_base3_packed_size(size_t count) { return (count + 4) / 5; }

int bitnet_hip_pack_ternary_base3(const int8_t *q, size_t count, uint8_t *packed, void *stream)
{
    if (count == 0) return BITNET_HIP_OK;
    if (!q || !packed) return fail(BITNET_HIP_NULL_POINTER, "pack_ternary_base3: null buffer");
    return launch_pack_base3(q, count, packed, as_stream(stream));
}

int bitnet_hip_unpack_ternary_base3(const uint8_t *packed, size_t count, int8_t *q, void *stream)
{
    if (count == 0) return BITNET_HIP_OK;
    if (!q || !packed) return fail(BITNET_HIP_NULL_POINTER, "unpack_ternary_base3: null buffer");
    return launch_unpack_base3(packed, count, q, as_stream(stream));
}

size_t bitnet_hip_base3_tiled_size(size_t n, size_t k) { return base3_tiled_bytes(n, k); }

int bitnet_hip_retile_base3(const uint8_t *base3, size_t n, size_t k, uint8_t *tiled, void *stream)
{
    if (n == 0 || k == 0) return BITNET_HIP_OK;
    if (!base3 || !tiled) return fail(BITNET_HIP_NULL_POINTER, "retile_base3: null argument");
    return launch_retile_base3(base3, n, k, tiled, as_stream(stream));
}

int bitnet_hip_gemv_base3(const uint8_t *tiled, const int8_t *a, size_t n, size_t k, const float *w_scale,
                          const float *a_scale, int32_t *acc, float *out, void *stream)
{
    if (n == 0) return BITNET_HIP_OK;
    if (k == 0) return fail(BITNET_HIP_INVALID_CONFIG, "gemv_base3: k must be positive");
    if (!tiled || !a) return fail(BITNET_HIP_NULL_POINTER, "gemv_base3: null weights or activations");
    if (!acc && !out) return fail(BITNET_HIP_NULL_POINTER, "gemv_base3: neither acc nor out given");
    if (out && !w_scale) return fail(BITNET_HIP_NULL_POINTER, "gemv_base3: out needs w_scale");
    if ((reinterpret_cast<uintptr_t>(tiled) & 15) != 0)
        return fail(BITNET_HIP_INVALID_CONFIG, "gemv_base3: the tiled weights must be 16-byte aligned");
    return launch_gemv_base3(tiled, a, acc, out, w_scale, a_scale, n, k, as_stream(stream));
}

int bitnet_hip_quantize_weights(const float *w, size_t n, size_t k, int method, float threshold_factor,
                                uint8_t *packed, float *w_scale, int8_t *q_i8, void *stream)
{
    if (!w_scale) return fail(BITNET_HIP_NULL_POINTER, "quantize_weights: w_scale is required");
    if (n * k != 0 && (!w || !packed)) return fail(BITNET_HIP_NULL_POINTER, "quantize_weights: null buffer");
    if (method >= BITNET_HIP_TERNARY_REF_MEAN_THRESHOLD && method <= BITNET_HIP_TERNARY_REF_DETSTE)
        // the reference's own pipeline with WeightQuantizationConfig's defaults (weights.rs:81-95): normalise, clip at 3.0
        return bitnet_hip_quantize_weights_reference(w, n, k, method - BITNET_HIP_TERNARY_REF_MEAN_THRESHOLD, 1, 3.0f,
                                                     threshold_factor, packed, w_scale, q_i8, nullptr, stream);
    if (method != BITNET_HIP_TERNARY_ABSMEAN_ROUNDCLIP && method != BITNET_HIP_TERNARY_MEAN_THRESHOLD)
        return fail(BITNET_HIP_INVALID_CONFIG, "quantize_weights: unknown method %d", method);
    DeviceTemp row_sums;
    int rc = row_sums.alloc(sizeof(double) * (n ? n : 1));
    if (rc != BITNET_HIP_OK) return rc;
    rc = launch_quantize_weights(w, n, k, method, threshold_factor, static_cast<double *>(row_sums.ptr), packed,
                                 w_scale, q_i8, as_stream(stream));
    if (rc != BITNET_HIP_OK) return rc;
    BITNET_HIP_TRY(hipStreamSynchronize(as_stream(stream)));  // row_sums is released on return
    return BITNET_HIP_OK;
}

int bitnet_hip_quantize_weights_reference(const float *w, size_t n, size_t k, int ternary_method, int normalize_weights,
                                          float outlier_threshold, float custom_threshold_factor, uint8_t *packed,
                                          float *w_scale, int8_t *q_i8, float *stats, void *stream)
{
    if (!w_scale) return fail(BITNET_HIP_NULL_POINTER, "quantize_weights_reference: w_scale is required");
    if (n * k != 0 && (!w || !packed)) return fail(BITNET_HIP_NULL_POINTER, "quantize_weights_reference: null buffer");
    if (ternary_method < 0 || ternary_method > 4)
        return fail(BITNET_HIP_INVALID_CONFIG, "quantize_weights_reference: unknown TernaryMethod %d", ternary_method);
    // WeightQuantizationConfig::validate (weights.rs:120-150)
    if (outlier_threshold < 0.0f) return fail(BITNET_HIP_INVALID_CONFIG, "Outlier threshold cannot be negative");
    if (custom_threshold_factor > 2.0f) return fail(BITNET_HIP_INVALID_CONFIG, "Custom threshold factor must be in range (0, 2]");
    DeviceTemp scratch;
    int rc = scratch.alloc(quantize_weights_reference_scratch_bytes(n));
    if (rc != BITNET_HIP_OK) return rc;
    rc = launch_quantize_weights_reference(w, n, k, ternary_method, normalize_weights != 0, outlier_threshold,
                                           custom_threshold_factor, scratch.ptr, packed, w_scale, q_i8, stats, as_stream(stream));
    if (rc != BITNET_HIP_OK) return rc;
    BITNET_HIP_TRY(hipStreamSynchronize(as_stream(stream)));  // the scratch is released on return
    return BITNET_HIP_OK;
}

size_t bitnet_hip_tiled_size(size_t n, size_t k) { return tiled_bytes(n, k); }

int bitnet_hip_retile_weights(const uint8_t *packed, size_t n, size_t k, int layout, uint8_t *tiled, void *stream)
{
    if (n * k == 0) return BITNET_HIP_OK;
    if (!packed || !tiled) return fail(BITNET_HIP_NULL_POINTER, "retile_weights: null buffer");
    if (layout != BITNET_HIP_LAYOUT_OUT_IN && layout != BITNET_HIP_LAYOUT_IN_OUT)
        return fail(BITNET_HIP_INVALID_CONFIG, "retile_weights: unknown layout %d", layout);
    if (reinterpret_cast<uintptr_t>(tiled) % 16)
        return fail(BITNET_HIP_INVALID_CONFIG, "retile_weights: tiled buffer must be 16-byte aligned");
    return launch_retile(packed, n, k, layout, tiled, as_stream(stream));
}

int bitnet_hip_untile_weights(const uint8_t *tiled, size_t n, size_t k, uint8_t *packed, void *stream)
{
    if (n * k == 0) return BITNET_HIP_OK;
    if (!packed || !tiled) return fail(BITNET_HIP_NULL_POINTER, "untile_weights: null buffer");
    return launch_untile(tiled, n, k, packed, as_stream(stream));
}

// ---- contraction -----------------------------------------------------------------------------------

int bitnet_hip_gemv_w2a8(const uint8_t *weights, const int8_t *activations, int32_t *output, size_t m, size_t k,
                         void *stream)
{
    if (m == 0) return BITNET_HIP_OK;
    if (!output) return fail(BITNET_HIP_NULL_POINTER, "gemv_w2a8: output is NULL");
    if (k != 0 && (!weights || !activations)) return fail(BITNET_HIP_NULL_POINTER, "gemv_w2a8: null input buffer");
    return launch_gemv_rowmajor(weights, activations, output, m, k, as_stream(stream));
}

int bitnet_hip_gemv_w2a8_checked(const uint8_t *weights, size_t weights_len, const int8_t *activations,
                                 size_t activations_len, int32_t *output, size_t output_len, size_t m, size_t k,
                                 void *stream)
{
    // same three checks, same order, as validate_w2a8_dimensions (bitnet-cuda/src/backend.rs:217-257)
    size_t expected_w = (m * k + 3) / 4;
    if (weights_len != expected_w) {
        size_t e[1] = {expected_w}, a[1] = {weights_len};
        return fail_shape(e, 1, a, 1, "weight bytes for an m x k matrix");
    }
    if (activations_len != k) {
        size_t e[1] = {k}, a[1] = {activations_len};
        return fail_shape(e, 1, a, 1, "activation elements");
    }
    if (output_len != m) {
        size_t e[1] = {m}, a[1] = {output_len};
        return fail_shape(e, 1, a, 1, "output elements");
    }
    return bitnet_hip_gemv_w2a8(weights, activations, output, m, k, stream);
}

int bitnet_hip_matmul_w2a8(const uint8_t *tiled, const int8_t *a, const int32_t *a_sum, size_t m, size_t n, size_t k,
                           int32_t *acc, const float *w_scale, const float *a_scale, const float *bias,
                           const float *residual, float *out, void *stream)
{
    if (m == 0 || n == 0) return BITNET_HIP_OK;
    if (!tiled || !a) return fail(BITNET_HIP_NULL_POINTER, "matmul_w2a8: null input buffer");
    if (!acc && !out) return fail(BITNET_HIP_NULL_POINTER, "matmul_w2a8: give acc, out or both");
    if (out && (!w_scale || !a_scale)) return fail(BITNET_HIP_NULL_POINTER, "matmul_w2a8: out needs w_scale and a_scale");
    if (reinterpret_cast<uintptr_t>(tiled) % 16)
        return fail(BITNET_HIP_INVALID_CONFIG, "matmul_w2a8: tiled weights must be 16-byte aligned");
    if (n > 0x7fffffffu || k > 0x7fffffffu) return fail(BITNET_HIP_UNSUPPORTED, "matmul_w2a8: dimension too large");
    if (gemv_takes(m, k, row_blocks(n), a)) {
        GemvProj pj = {tiled, w_scale, bias, residual, out, acc, n};
        return launch_gemv_tiled(&pj, 1, a, a_scale, m, k, as_stream(stream));
    }
    return launch_gemm_tiled(tiled, a, a_sum, m, n, k, acc, w_scale, a_scale, bias, residual, out, as_stream(stream));
}

// ---- BitLinear layer object -------------------------------------------------------------------------

int bitnet_hip_bitlinear_create(size_t in_features, size_t out_features, int use_bias, bitnet_hip_bitlinear **layer)
{
    if (!layer) return fail(BITNET_HIP_NULL_POINTER, "bitlinear_create: layer is NULL");
    *layer = nullptr;
    if (in_features == 0 || out_features == 0)
        return fail(BITNET_HIP_INVALID_CONFIG, "bitlinear_create: in_features=%zu out_features=%zu must be positive",
                    in_features, out_features);
    bitnet_hip_bitlinear *l = new (std::nothrow) bitnet_hip_bitlinear;
    if (!l) return fail(BITNET_HIP_MEMORY_ERROR, "bitlinear_create: out of host memory");
    l->in_features = in_features;
    l->out_features = out_features;
    l->use_bias = use_bias != 0;
    hipError_t e = hipMalloc(&l->packed, (in_features * out_features + 3) / 4);
    if (e == hipSuccess) e = hipMalloc(&l->tiled, tiled_bytes(out_features, in_features));
    if (e == hipSuccess) e = hipMalloc(&l->w_scale, sizeof(float));
    if (e == hipSuccess && l->use_bias) {
        e = hipMalloc(&l->bias, sizeof(float) * out_features);
        if (e == hipSuccess) e = hipMemset(l->bias, 0, sizeof(float) * out_features);
    }
    if (e != hipSuccess) {
        delete l;
        return fail(BITNET_HIP_MEMORY_ERROR, "bitlinear_create: device allocation failed: %s", hipGetErrorString(e));
    }
    *layer = l;
    return BITNET_HIP_OK;
}

void bitnet_hip_bitlinear_destroy(bitnet_hip_bitlinear *layer) { delete layer; }

int bitnet_hip_bitlinear_set_weights_f32(bitnet_hip_bitlinear *layer, const float *w, size_t rows, size_t cols,
                                         int layout, int on_device, int method, float threshold_factor, void *stream)
{
    if (!layer || !w) return fail(BITNET_HIP_NULL_POINTER, "set_weights_f32: null argument");
    if (layout != BITNET_HIP_LAYOUT_OUT_IN && layout != BITNET_HIP_LAYOUT_IN_OUT)
        return fail(BITNET_HIP_INVALID_CONFIG, "set_weights_f32: unknown layout %d", layout);
    const size_t n = layer->out_features, k = layer->in_features;
    const size_t er = layout == BITNET_HIP_LAYOUT_OUT_IN ? n : k, ec = layout == BITNET_HIP_LAYOUT_OUT_IN ? k : n;
    if (rows != er || cols != ec) {
        size_t e[2] = {er, ec}, a[2] = {rows, cols};
        return fail_shape(e, 2, a, 2, "weight matrix");  // BitLinear::update_weights, layer.rs:301-307
    }
    hipStream_t s = as_stream(stream);
    DeviceTemp w_dev, flat;
    const float *src = w;
    if (!on_device) {
        int rc = w_dev.alloc(sizeof(float) * n * k);
        if (rc != BITNET_HIP_OK) return rc;
        BITNET_HIP_TRY(hipMemcpyAsync(w_dev.ptr, w, sizeof(float) * n * k, hipMemcpyHostToDevice, s));
        src = static_cast<const float *>(w_dev.ptr);
    }
    int rc = flat.alloc((n * k + 3) / 4);
    if (rc != BITNET_HIP_OK) return rc;
    std::unique_lock<std::shared_mutex> guard(layer->lock);
    BITNET_HIP_TRY(hipDeviceSynchronize());  // forwards already queued on any stream still read the old weights
    rc = bitnet_hip_quantize_weights(src, rows, cols, method, threshold_factor, static_cast<uint8_t *>(flat.ptr),
                                     layer->w_scale, nullptr, stream);
    if (rc != BITNET_HIP_OK) return rc;
    rc = launch_retile(static_cast<const uint8_t *>(flat.ptr), n, k, layout, layer->tiled, s);
    if (rc != BITNET_HIP_OK) return rc;
    rc = launch_untile(layer->tiled, n, k, layer->packed, s);  // canonical [out, in] bytes
    if (rc != BITNET_HIP_OK) return rc;
    BITNET_HIP_TRY(hipStreamSynchronize(s));
    layer->has_weights = true;
    return BITNET_HIP_OK;
}

int bitnet_hip_bitlinear_set_weights_packed(bitnet_hip_bitlinear *layer, const uint8_t *packed, size_t packed_len,
                                            float w_scale, int on_device, void *stream)
{
    if (!layer || !packed) return fail(BITNET_HIP_NULL_POINTER, "set_weights_packed: null argument");
    const size_t n = layer->out_features, k = layer->in_features, need = (n * k + 3) / 4;
    if (packed_len < need) {
        // WeightConverter::convert_ternary_weights rejects short buffers (weight_conversion.rs:153-158)
        size_t e[1] = {need}, a[1] = {packed_len};
        return fail_shape(e, 1, a, 1, "packed weight bytes");
    }
    hipStream_t s = as_stream(stream);
    std::unique_lock<std::shared_mutex> guard(layer->lock);
    BITNET_HIP_TRY(hipDeviceSynchronize());  // forwards already queued on any stream still read the old weights
    BITNET_HIP_TRY(hipMemcpyAsync(layer->packed, packed, need, on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice, s));
    BITNET_HIP_TRY(hipMemcpyAsync(layer->w_scale, &w_scale, sizeof(float), hipMemcpyHostToDevice, s));
    int rc = launch_retile(layer->packed, n, k, BITNET_HIP_LAYOUT_OUT_IN, layer->tiled, s);
    if (rc != BITNET_HIP_OK) return rc;
    BITNET_HIP_TRY(hipStreamSynchronize(s));  // w_scale is read from the caller's stack
    layer->has_weights = true;
    return BITNET_HIP_OK;
}

int bitnet_hip_bitlinear_set_weights_base3(bitnet_hip_bitlinear *layer, const uint8_t *packed, size_t packed_len,
                                           float w_scale, int on_device, void *stream)
{
    if (!layer || !packed) return fail(BITNET_HIP_NULL_POINTER, "set_weights_base3: null argument");
    const size_t n = layer->out_features, k = layer->in_features, need = (n * k + 4) / 5;
    if (packed_len < need) {
        size_t e[1] = {need}, a[1] = {packed_len};
        return fail_shape(e, 1, a, 1, "base-3 packed weight bytes");
    }
    hipStream_t s = as_stream(stream);
    DeviceTemp staged;  // the base-3 bytes on the device
    const uint8_t *src = packed;
    if (!on_device) {
        int rc = staged.alloc(need);
        if (rc != BITNET_HIP_OK) return rc;
        BITNET_HIP_TRY(hipMemcpyAsync(staged.ptr, packed, need, hipMemcpyHostToDevice, s));
        src = static_cast<const uint8_t *>(staged.ptr);
    }
    std::unique_lock<std::shared_mutex> guard(layer->lock);
    BITNET_HIP_TRY(hipDeviceSynchronize());  // forwards already queued on any stream still read the old weights
    int rc = launch_base3_to_2bit(src, n * k, layer->packed, s);
    if (rc != BITNET_HIP_OK) return rc;
    BITNET_HIP_TRY(hipMemcpyAsync(layer->w_scale, &w_scale, sizeof(float), hipMemcpyHostToDevice, s));
    rc = launch_retile(layer->packed, n, k, BITNET_HIP_LAYOUT_OUT_IN, layer->tiled, s);
    if (rc != BITNET_HIP_OK) return rc;
    BITNET_HIP_TRY(hipStreamSynchronize(s));  // w_scale is read from the caller's stack; `staged` is freed on return
    layer->has_weights = true;
    return BITNET_HIP_OK;
}

int bitnet_hip_bitlinear_set_weights_gguf(bitnet_hip_bitlinear *layer, const uint8_t *data, size_t len, size_t rows,
                                          size_t cols, int layout, int on_device, float *scale_out, float *offset_out,
                                          void *stream)
{
    if (!layer || !data) return fail(BITNET_HIP_NULL_POINTER, "set_weights_gguf: null argument");
    if (layout != BITNET_HIP_LAYOUT_OUT_IN && layout != BITNET_HIP_LAYOUT_IN_OUT)
        return fail(BITNET_HIP_INVALID_CONFIG, "set_weights_gguf: unknown layout %d", layout);
    const size_t n = layer->out_features, k = layer->in_features;
    const size_t er = layout == BITNET_HIP_LAYOUT_OUT_IN ? n : k, ec = layout == BITNET_HIP_LAYOUT_OUT_IN ? k : n;
    if (rows != er || cols != ec) {
        size_t e[2] = {er, ec}, a[2] = {rows, cols};
        return fail_shape(e, 2, a, 2, "GGUF tensor dimensions");
    }
    const size_t codes = (n * k + 3) / 4, need = 8 + codes;
    if (len < need) {
        size_t e[1] = {need}, a[1] = {len};
        return fail_shape(e, 1, a, 1, "Insufficient packed data (8-byte scale/offset header + 2-bit codes)");
    }
    hipStream_t s = as_stream(stream);
    float header[2];  // little-endian host, as f32::from_le_bytes on the reference's targets
    if (on_device) BITNET_HIP_TRY(hipMemcpy(header, data, 8, hipMemcpyDeviceToHost));
    else memcpy(header, data, 8);
    if (scale_out) *scale_out = header[0];
    if (offset_out) *offset_out = header[1];
    // the codes start 8 bytes into the tensor: stage them at an aligned device address, in their own orientation
    DeviceTemp flat;
    int rc = flat.alloc(codes);
    if (rc != BITNET_HIP_OK) return rc;
    std::unique_lock<std::shared_mutex> guard(layer->lock);
    BITNET_HIP_TRY(hipDeviceSynchronize());  // forwards already queued on any stream still read the old weights
    BITNET_HIP_TRY(hipMemcpyAsync(flat.ptr, data + 8, codes, on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice, s));
    BITNET_HIP_TRY(hipMemcpyAsync(layer->w_scale, &header[0], sizeof(float), hipMemcpyHostToDevice, s));
    rc = launch_retile(static_cast<const uint8_t *>(flat.ptr), n, k, layout, layer->tiled, s);
    if (rc != BITNET_HIP_OK) return rc;
    rc = launch_untile(layer->tiled, n, k, layer->packed, s);  // canonical [out, in] bytes, code 3 stored as code 1
    if (rc != BITNET_HIP_OK) return rc;
    BITNET_HIP_TRY(hipStreamSynchronize(s));
    layer->has_weights = true;
    return BITNET_HIP_OK;
}

int bitnet_hip_bitlinear_set_bias(bitnet_hip_bitlinear *layer, const float *bias, size_t len, int on_device, void *stream)
{
    if (!layer || !bias) return fail(BITNET_HIP_NULL_POINTER, "set_bias: null argument");
    if (!layer->use_bias) return fail(BITNET_HIP_INVALID_CONFIG, "Bias is not enabled for this layer");
    if (len != layer->out_features) {
        size_t e[1] = {layer->out_features}, a[1] = {len};
        return fail_shape(e, 1, a, 1, "bias");
    }
    std::unique_lock<std::shared_mutex> guard(layer->lock);
    BITNET_HIP_TRY(hipDeviceSynchronize());  // forwards already queued on any stream still read the old bias
    BITNET_HIP_TRY(hipMemcpyAsync(layer->bias, bias, sizeof(float) * len,
                                  on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice, as_stream(stream)));
    BITNET_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return BITNET_HIP_OK;
}

int bitnet_hip_bitlinear_get_quantized(bitnet_hip_bitlinear *layer, float *w_scale, uint8_t *packed, size_t packed_len)
{
    if (!layer) return fail(BITNET_HIP_NULL_POINTER, "get_quantized: layer is NULL");
    std::shared_lock<std::shared_mutex> guard(layer->lock);
    if (!layer->has_weights) return fail(BITNET_HIP_NOT_INITIALIZED, "get_quantized: the layer has no weights yet");
    BITNET_HIP_TRY(hipDeviceSynchronize());
    if (w_scale) BITNET_HIP_TRY(hipMemcpy(w_scale, layer->w_scale, sizeof(float), hipMemcpyDeviceToHost));
    if (packed) {
        size_t need = (layer->in_features * layer->out_features + 3) / 4;
        if (packed_len < need) {
            size_t e[1] = {need}, a[1] = {packed_len};
            return fail_shape(e, 1, a, 1, "packed weight bytes");
        }
        BITNET_HIP_TRY(hipMemcpy(packed, layer->packed, need, hipMemcpyDeviceToHost));
    }
    return BITNET_HIP_OK;
}

size_t bitnet_hip_bitlinear_workspace_size(const bitnet_hip_bitlinear *layer, size_t m)
{
    if (!layer) return 0;
    // the quantised activations, and the partial tiles of a GEMM that splits k across workgroups where one would run
    return quant_scratch_bytes(m, layer->in_features) + split_scratch_bytes(m, layer->in_features, layer->out_features);
}

int bitnet_hip_bitlinear_forward(bitnet_hip_bitlinear *layer, const float *x, const size_t *dims, int rank,
                                 const float *gamma, float eps, int sum_order, const float *residual, float *out,
                                 void *workspace, size_t workspace_bytes, int8_t *dbg_q, float *dbg_a_scale,
                                 int32_t *dbg_acc, void *stream)
{
    if (!layer) return fail(BITNET_HIP_NULL_POINTER, "forward: layer is NULL");
    const size_t in = layer->in_features;
    // shape rules of BitLinearForward::forward (forward.rs:60-76) and quantized_matmul (:179-214)
    if (rank <= 0 || !dims) {
        size_t e[2] = {1, in};
        return fail_shape(e, 2, dims, 0, "input");
    }
    if (dims[rank - 1] != in) {
        size_t e[2] = {dims[0], in};
        return fail_shape(e, 2, dims, rank, "last input dimension");
    }
    if (rank != 2 && rank != 3) {
        size_t e[2] = {1, in};
        return fail_shape(e, 2, dims, rank, "input rank");
    }
    const size_t m = rank == 2 ? dims[0] : dims[0] * dims[1];
    if (m == 0) return BITNET_HIP_OK;
    if (!x || !out) return fail(BITNET_HIP_NULL_POINTER, "forward: x and out are required");

    std::shared_lock<std::shared_mutex> guard(layer->lock);
    if (!layer->has_weights) return fail(BITNET_HIP_NOT_INITIALIZED, "forward: the layer has no weights yet");

    hipStream_t s = as_stream(stream);
    const bool debug = dbg_q || dbg_a_scale || dbg_acc;
    const bool fused = gemv_fused_supported(x, nullptr, in, m, in, BITNET_HIP_INPUT_PLAIN, 1, gamma, sum_order, row_blocks(layer->out_features));
    void *ws = workspace;
    bool own_ws = false;
    QuantScratch sc = {dbg_q, dbg_a_scale, nullptr};
    GemmSplitScratch split;
    if (!fused || debug) {  // the fused decode launch needs no scratch unless the caller wants q / a_scale back
        const size_t need = quant_scratch_bytes(m, in), extra = split_scratch_bytes(m, in, layer->out_features);
        bool with_split = extra != 0;
        if (!ws) {
            hipError_t e = hipMallocAsync(&ws, need + extra, s);
            if (e != hipSuccess) return fail(BITNET_HIP_MEMORY_ERROR, "forward: hipMallocAsync(%zu) failed: %s", need + extra, hipGetErrorString(e));
            own_ws = true;
        } else if (workspace_bytes < need) {
            return fail(BITNET_HIP_MEMORY_ERROR, "forward: workspace of %zu bytes given, %zu needed", workspace_bytes, need);
        } else if (workspace_bytes < need + extra) {
            with_split = false;  // room for the quantised activations only: the GEMM walks k without the split
        }
        sc = carve_scratch(ws, m, in);
        if (with_split) split = carve_split(ws, m, in, layer->out_features);
        if (dbg_q) sc.q = dbg_q;
        if (dbg_a_scale) sc.a_scale = dbg_a_scale;
    }
    bitnet_hip_bitlinear *layers[1] = {layer};
    const float *res[1] = {residual};
    float *outs[1] = {out};
    int32_t *accs[1] = {dbg_acc};
    int rc = run_projections(layers, 1, x, nullptr, in, m, BITNET_HIP_INPUT_PLAIN, 1, 1, gamma, eps, sum_order, res, outs,
                             accs, sc.q, sc.a_scale, sc.a_sum, debug, s, split.partials ? &split : nullptr);
    if (own_ws) {
        hipError_t e = hipFreeAsync(ws, s);
        if (rc == BITNET_HIP_OK && e != hipSuccess)
            rc = fail(BITNET_HIP_MEMORY_ERROR, "forward: hipFreeAsync failed: %s", hipGetErrorString(e));
    }
    return rc;
}

int bitnet_hip_bitlinear_forward_noalloc(bitnet_hip_bitlinear *layer, const float *x, const size_t *dims, int rank,
                                         const float *gamma, float eps, int sum_order, const float *residual,
                                         float *out, void *stream)
{
    if (!layer) return fail(BITNET_HIP_NULL_POINTER, "forward_noalloc: layer is NULL");
    const size_t in = layer->in_features;
    if (rank <= 0 || !dims) {
        size_t e[2] = {1, in};
        return fail_shape(e, 2, dims, 0, "input");
    }
    if (dims[rank - 1] != in) {
        size_t e[2] = {dims[0], in};
        return fail_shape(e, 2, dims, rank, "last input dimension");
    }
    if (rank != 2 && rank != 3) {
        size_t e[2] = {1, in};
        return fail_shape(e, 2, dims, rank, "input rank");
    }
    const size_t m = rank == 2 ? dims[0] : dims[0] * dims[1];
    if (m == 0) return BITNET_HIP_OK;
    if (!x || !out) return fail(BITNET_HIP_NULL_POINTER, "forward_noalloc: x and out are required");
    if (m > NOALLOC_MAX_ROWS || m * in > NOALLOC_MAX_ELEMS)
        return fail(BITNET_HIP_MEMORY_ERROR,
                    "forward_noalloc: %zu rows x %zu features exceed the static scratch (at most %zu rows and %zu "
                    "rows*features per call); use bitnet_hip_bitlinear_forward with a workspace",
                    m, in, NOALLOC_MAX_ROWS, NOALLOC_MAX_ELEMS);
    static_assert(NOALLOC_MAX_ELEMS % 256 == 0 && (NOALLOC_MAX_ROWS * sizeof(float)) % 256 == 0 &&
                      NOALLOC_SCRATCH_BYTES >= NOALLOC_MAX_ELEMS + 2 * NOALLOC_MAX_ROWS * sizeof(float) + 256,
                  "the scratch holds q, a_scale and a_sum of the largest call");
    void *ws = nullptr;
    int rc = noalloc_scratch(&ws);
    if (rc != BITNET_HIP_OK) return rc;
    if (quant_scratch_bytes(m, in) > NOALLOC_SCRATCH_BYTES)
        return fail(BITNET_HIP_MEMORY_ERROR, "forward_noalloc: %zu bytes of scratch needed, %zu held", quant_scratch_bytes(m, in),
                    NOALLOC_SCRATCH_BYTES);

    std::shared_lock<std::shared_mutex> guard(layer->lock);
    if (!layer->has_weights) return fail(BITNET_HIP_NOT_INITIALIZED, "forward_noalloc: the layer has no weights yet");
    const QuantScratch sc = carve_scratch(ws, m, in);
    bitnet_hip_bitlinear *layers[1] = {layer};
    const float *res[1] = {residual};
    float *outs[1] = {out};
    return run_projections(layers, 1, x, nullptr, in, m, BITNET_HIP_INPUT_PLAIN, 1, 1, gamma, eps, sum_order, res, outs,
                           nullptr, sc.q, sc.a_scale, sc.a_sum, false, as_stream(stream));
}

int bitnet_hip_bitlinear_forward_multi(bitnet_hip_bitlinear *const *layers, size_t count, const float *x, size_t m,
                                       const float *gamma, float eps, int sum_order, float *const *outs, void *workspace,
                                       size_t workspace_bytes, void *stream)
{
    if (!layers || !outs) return fail(BITNET_HIP_NULL_POINTER, "forward_multi: null argument");
    if (count == 0 || m == 0) return BITNET_HIP_OK;
    if (count > 16) return fail(BITNET_HIP_INVALID_CONFIG, "forward_multi: at most 16 layers per call, got %zu", count);
    if (!x) return fail(BITNET_HIP_NULL_POINTER, "forward_multi: x is NULL");
    std::vector<std::shared_lock<std::shared_mutex>> guards;
    for (size_t j = 0; j < count; ++j) {
        if (!layers[j] || !outs[j]) return fail(BITNET_HIP_NULL_POINTER, "forward_multi: layer or output %zu is NULL", j);
        if (layers[j]->in_features != layers[0]->in_features) {
            size_t e[2] = {m, layers[0]->in_features}, a[2] = {m, layers[j]->in_features};
            return fail_shape(e, 2, a, 2, "layers of one forward_multi call must share in_features");
        }
        guards.emplace_back(layers[j]->lock);
        if (!layers[j]->has_weights) return fail(BITNET_HIP_NOT_INITIALIZED, "forward_multi: layer %zu has no weights yet", j);
    }
    const size_t in = layers[0]->in_features;
    hipStream_t s = as_stream(stream);
    const bool fused = gemv_fused_supported(x, nullptr, in, m, in, BITNET_HIP_INPUT_PLAIN, 1, gamma, sum_order, launch_group_blocks(layers, count));
    void *ws = workspace;
    bool own_ws = false;
    QuantScratch sc = {nullptr, nullptr, nullptr};
    if (!fused) {
        const size_t need = quant_scratch_bytes(m, in);
        if (!ws) {
            hipError_t e = hipMallocAsync(&ws, need, s);
            if (e != hipSuccess) return fail(BITNET_HIP_MEMORY_ERROR, "forward_multi: hipMallocAsync(%zu) failed: %s", need, hipGetErrorString(e));
            own_ws = true;
        } else if (workspace_bytes < need) {
            return fail(BITNET_HIP_MEMORY_ERROR, "forward_multi: workspace of %zu bytes given, %zu needed", workspace_bytes, need);
        }
        sc = carve_scratch(ws, m, in);
    }
    int rc = run_projections(layers, (int)count, x, nullptr, in, m, BITNET_HIP_INPUT_PLAIN, 1, 1, gamma, eps, sum_order,
                             nullptr, outs, nullptr, sc.q, sc.a_scale, sc.a_sum, false, s);
    if (own_ws) {
        hipError_t e = hipFreeAsync(ws, s);
        if (rc == BITNET_HIP_OK && e != hipSuccess)
            rc = fail(BITNET_HIP_MEMORY_ERROR, "forward_multi: hipFreeAsync failed: %s", hipGetErrorString(e));
    }
    return rc;
}

int bitnet_hip_bitlinear_matmul(bitnet_hip_bitlinear *layer, const int8_t *a, const int32_t *a_sum, size_t m,
                                const float *a_scale, const float *residual, int32_t *acc, float *out, void *stream)
{
    if (!layer) return fail(BITNET_HIP_NULL_POINTER, "bitlinear_matmul: layer is NULL");
    std::shared_lock<std::shared_mutex> guard(layer->lock);
    if (!layer->has_weights) return fail(BITNET_HIP_NOT_INITIALIZED, "bitlinear_matmul: the layer has no weights yet");
    return bitnet_hip_matmul_w2a8(layer->tiled, a, a_sum, m, layer->out_features, layer->in_features, acc, layer->w_scale,
                                  a_scale, layer->use_bias ? layer->bias : nullptr, residual, out, stream);
}

}  // extern "C"

// ---------------------------------------------------------------------------------------------------
// Decoder projections
// ---------------------------------------------------------------------------------------------------
constexpr size_t DECODER_MAX_CHAINS = 8;

struct bitnet_hip_decoder {
    size_t layers = 0, hidden = 0, ffn = 0, q_heads = 0, kv_heads = 0, head_dim = 0, max_tokens = 0;
    float eps = 1e-5f;
    int sum_order = BITNET_HIP_SUM_BLOCK256;
    std::vector<bitnet_hip_bitlinear *> proj;  // layers * 7
    float *gamma = nullptr;                    // [layers][2][hidden]
    // activation buffers, sized for max_tokens
    int8_t *a8 = nullptr;
    float *a_scale = nullptr;
    int32_t *a_sum = nullptr;
    float *qb = nullptr, *kb = nullptr, *vb = nullptr, *x1 = nullptr, *gate = nullptr, *up = nullptr;
    float *ping = nullptr;
    // One decode at a time: the activation buffers above are shared by every call on this decoder.  The mutex
    // serialises the enqueue; `done` (recorded behind every decode) makes a decode on another stream wait for it.
    std::mutex decode_lock;
    hipEvent_t done = nullptr;
    hipStream_t done_stream = nullptr;
    bool done_recorded = false;
    // Token rows never interact on this path (CpuInferenceBackend::execute_batch fans independent inputs out over
    // threads, bitnet-inference/src/engine/cpu_backend.rs:206-238).  A step of several rows is therefore split into up
    // to DECODER_MAX_CHAINS groups of rows can be run as chains of launches side by side, each through all blocks on a
    // stream of its own (its rows of the activation buffers are its own), forked from and joined to the caller's stream
    // by events.  Off unless asked for (chains <= 1 = one chain): on the part measured the command processor starts one
    // kernel per 2.2 us whatever the number of queues, so chains of these short kernels take turns instead of
    // overlapping (8 tokens, 30 blocks: 957 us as one chain, 918 as two, 1355 as four, 2155 as eight).
    size_t chains = 0;
    hipStream_t side[DECODER_MAX_CHAINS - 1] = {};
    hipEvent_t fork = nullptr, join[DECODER_MAX_CHAINS - 1] = {};

    ~bitnet_hip_decoder()
    {
        for (auto *p : proj) delete p;
        void *bufs[] = {gamma, a8, a_scale, a_sum, qb, kb, vb, x1, gate, up, ping};
        for (void *b : bufs)
            if (b) (void)hipFree(b);
        if (done) (void)hipEventDestroy(done);
        if (fork) (void)hipEventDestroy(fork);
        for (hipEvent_t e : join)
            if (e) (void)hipEventDestroy(e);
        for (hipStream_t st : side)
            if (st) (void)hipStreamDestroy(st);
    }
};

extern "C" {

int bitnet_hip_decoder_create(size_t layers, size_t hidden, size_t ffn, size_t q_heads, size_t kv_heads,
                              size_t head_dim, float eps, int sum_order, size_t max_tokens, bitnet_hip_decoder **dec)
{
    if (!dec) return fail(BITNET_HIP_NULL_POINTER, "decoder_create: dec is NULL");
    *dec = nullptr;
    if (!layers || !hidden || !ffn || !q_heads || !kv_heads || !head_dim || !max_tokens)
        return fail(BITNET_HIP_INVALID_CONFIG, "decoder_create: every size must be positive");
    if (q_heads * head_dim != hidden || q_heads % kv_heads != 0)
        return fail(BITNET_HIP_INVALID_CONFIG,
                    "decoder_create: q_heads*head_dim=%zu must equal hidden=%zu and q_heads %% kv_heads must be 0",
                    q_heads * head_dim, hidden);
    bitnet_hip_decoder *d = new (std::nothrow) bitnet_hip_decoder;
    if (!d) return fail(BITNET_HIP_MEMORY_ERROR, "decoder_create: out of host memory");
    d->layers = layers; d->hidden = hidden; d->ffn = ffn; d->q_heads = q_heads; d->kv_heads = kv_heads;
    d->head_dim = head_dim; d->eps = eps; d->sum_order = sum_order; d->max_tokens = max_tokens;
    const size_t kv_dim = kv_heads * head_dim;
    const size_t outs[7] = {hidden, kv_dim, kv_dim, hidden, ffn, ffn, hidden};
    const size_t ins[7] = {hidden, hidden, hidden, hidden, hidden, hidden, ffn};
    int rc = BITNET_HIP_OK;
    for (size_t l = 0; l < layers && rc == BITNET_HIP_OK; ++l)
        for (int p = 0; p < 7 && rc == BITNET_HIP_OK; ++p) {
            bitnet_hip_bitlinear *bl = nullptr;
            rc = bitnet_hip_bitlinear_create(ins[p], outs[p], 0, &bl);
            if (rc == BITNET_HIP_OK) d->proj.push_back(bl);
        }
    const size_t widest = hidden > ffn ? hidden : ffn;
    auto dev_alloc = [&](auto **ptr, size_t bytes) {
        if (rc != BITNET_HIP_OK) return;
        hipError_t e = hipMalloc(reinterpret_cast<void **>(ptr), bytes);
        if (e != hipSuccess) rc = fail(BITNET_HIP_MEMORY_ERROR, "decoder_create: hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    };
    dev_alloc(&d->gamma, sizeof(float) * layers * 2 * hidden);
    dev_alloc(&d->a8, max_tokens * widest);
    dev_alloc(&d->a_scale, sizeof(float) * max_tokens);
    dev_alloc(&d->a_sum, sizeof(int32_t) * max_tokens);
    dev_alloc(&d->qb, sizeof(float) * max_tokens * hidden);
    dev_alloc(&d->kb, sizeof(float) * max_tokens * kv_dim);
    dev_alloc(&d->vb, sizeof(float) * max_tokens * kv_dim);
    dev_alloc(&d->x1, sizeof(float) * max_tokens * hidden);
    dev_alloc(&d->gate, sizeof(float) * max_tokens * ffn);
    dev_alloc(&d->up, sizeof(float) * max_tokens * ffn);
    dev_alloc(&d->ping, sizeof(float) * max_tokens * hidden);
    if (rc == BITNET_HIP_OK) {
        // RMSNorm weights start at one
        std::vector<float> ones(layers * 2 * hidden, 1.0f);
        hipError_t e = hipMemcpy(d->gamma, ones.data(), sizeof(float) * ones.size(), hipMemcpyHostToDevice);
        if (e != hipSuccess) rc = fail(BITNET_HIP_DEVICE_ERROR, "decoder_create: hipMemcpy failed: %s", hipGetErrorString(e));
    }
    if (rc == BITNET_HIP_OK) {
        hipError_t e = hipEventCreateWithFlags(&d->done, hipEventDisableTiming);
        if (e != hipSuccess) rc = fail(BITNET_HIP_DEVICE_ERROR, "decoder_create: hipEventCreate failed: %s", hipGetErrorString(e));
    }
    // streams (default priority) and events of the row-group chains, made here so that no decode call creates any
    const size_t side_streams = (max_tokens < DECODER_MAX_CHAINS ? max_tokens : DECODER_MAX_CHAINS) - 1;
    if (rc == BITNET_HIP_OK && side_streams > 0) {
        hipError_t e = hipEventCreateWithFlags(&d->fork, hipEventDisableTiming);
        for (size_t i = 0; i < side_streams && e == hipSuccess; ++i) {
            e = hipStreamCreateWithFlags(&d->side[i], hipStreamNonBlocking);
            if (e == hipSuccess) e = hipEventCreateWithFlags(&d->join[i], hipEventDisableTiming);
        }
        if (e != hipSuccess) rc = fail(BITNET_HIP_DEVICE_ERROR, "decoder_create: chain streams: %s", hipGetErrorString(e));
    }
    if (rc != BITNET_HIP_OK) {
        delete d;
        return rc;
    }
    *dec = d;
    return BITNET_HIP_OK;
}

int bitnet_hip_decoder_set_chains(bitnet_hip_decoder *dec, size_t chains)
{
    if (!dec) return fail(BITNET_HIP_NULL_POINTER, "decoder_set_chains: dec is NULL");
    if (chains > DECODER_MAX_CHAINS)
        return fail(BITNET_HIP_INVALID_CONFIG, "decoder_set_chains: %zu chains, at most %zu", chains, DECODER_MAX_CHAINS);
    std::lock_guard<std::mutex> one_decode(dec->decode_lock);
    dec->chains = chains;
    return BITNET_HIP_OK;
}

void bitnet_hip_decoder_destroy(bitnet_hip_decoder *dec) { delete dec; }

int bitnet_hip_decoder_projection(bitnet_hip_decoder *dec, size_t layer, int proj, bitnet_hip_bitlinear **out)
{
    if (!dec || !out) return fail(BITNET_HIP_NULL_POINTER, "decoder_projection: null argument");
    if (layer >= dec->layers || proj < 0 || proj > 6)
        return fail(BITNET_HIP_INVALID_CONFIG, "decoder_projection: layer %zu / projection %d out of range", layer, proj);
    *out = dec->proj[layer * 7 + (size_t)proj];
    return BITNET_HIP_OK;
}

int bitnet_hip_decoder_set_norm(bitnet_hip_decoder *dec, size_t layer, int which, const float *gamma, int on_device,
                                void *stream)
{
    if (!dec || !gamma) return fail(BITNET_HIP_NULL_POINTER, "decoder_set_norm: null argument");
    if (layer >= dec->layers || which < 0 || which > 1)
        return fail(BITNET_HIP_INVALID_CONFIG, "decoder_set_norm: layer %zu / which %d out of range", layer, which);
    float *dst = dec->gamma + (layer * 2 + (size_t)which) * dec->hidden;
    // as a weight update: no decode is being enqueued, and those already queued (on any stream) have finished
    std::lock_guard<std::mutex> one_decode(dec->decode_lock);
    BITNET_HIP_TRY(hipDeviceSynchronize());
    BITNET_HIP_TRY(hipMemcpyAsync(dst, gamma, sizeof(float) * dec->hidden,
                                  on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice, as_stream(stream)));
    BITNET_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return BITNET_HIP_OK;
}

size_t bitnet_hip_decoder_weight_bytes(const bitnet_hip_decoder *dec)
{
    if (!dec) return 0;
    size_t total = 0;
    for (auto *p : dec->proj) total += p->in_features * p->out_features / 4;
    return total;
}

int bitnet_hip_decoder_decode_layers(bitnet_hip_decoder *dec, size_t layer_begin, size_t layer_end,
                                     const float *x_in, size_t m, float *x_out, float *q_last, float *k_last,
                                     void *stream)
{
    if (!dec || !x_in || !x_out) return fail(BITNET_HIP_NULL_POINTER, "decoder_decode: null argument");
    if (layer_begin > layer_end || layer_end > dec->layers)
        return fail(BITNET_HIP_INVALID_CONFIG, "decoder_decode: layer range [%zu, %zu) outside [0, %zu)", layer_begin,
                    layer_end, dec->layers);
    if (m == 0 || layer_begin == layer_end) return BITNET_HIP_OK;
    if (m > dec->max_tokens) {
        size_t e[2] = {dec->max_tokens, dec->hidden}, a[2] = {m, dec->hidden};
        return fail_shape(e, 2, a, 2, "tokens per decode step exceed max_tokens");
    }
    hipStream_t s = as_stream(stream);
    const size_t H = dec->hidden, F = dec->ffn, KV = dec->kv_heads * dec->head_dim;
    const size_t group = dec->q_heads / dec->kv_heads;
    int rc = BITNET_HIP_OK;
    // readers of every projection involved (weight updates take the write lock and wait for the GPU), and one
    // decode at a time on this decoder's buffers
    std::vector<std::shared_lock<std::shared_mutex>> guards;
    guards.reserve((layer_end - layer_begin) * 7);
    for (size_t i = layer_begin * 7; i < layer_end * 7; ++i) {
        guards.emplace_back(dec->proj[i]->lock);
        if (!dec->proj[i]->has_weights)
            return fail(BITNET_HIP_NOT_INITIALIZED, "decoder_decode: a projection has no weights yet");
    }
    std::lock_guard<std::mutex> one_decode(dec->decode_lock);
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(s, &capturing);
    if (dec->done_recorded && dec->done_stream != s && capturing == hipStreamCaptureStatusNone)
        BITNET_HIP_TRY(hipStreamWaitEvent(s, dec->done, 0));  // the previous decode used these buffers on another stream
    // One chain: rows [row0, row0 + rows) through blocks layer_begin .. layer_end-1 on stream cs, in its own rows of the
    // decoder's activation buffers.
    const size_t widest = H > F ? H : F;
    auto run_chain = [&](size_t row0, size_t rows, hipStream_t cs) {
        // one launch group: `count` projections reading the same (transformed) input
        auto run = [&](bitnet_hip_bitlinear *const *layers, int count, const float *x, const float *x2, size_t ldx, int mode,
                       const float *gamma, const float *res0, float *const *outs) {
            if (rc != BITNET_HIP_OK) return;
            const float *res[GEMV_MAX_PROJ] = {res0, nullptr, nullptr};
            rc = run_projections(layers, count, x, x2, ldx, rows, mode, group, dec->head_dim, gamma, dec->eps, dec->sum_order,
                                 res, outs, nullptr, dec->a8 + row0 * widest, dec->a_scale + row0, dec->a_sum + row0, false, cs);
        };
        float *qb = dec->qb + row0 * H, *kb = dec->kb + row0 * KV, *vb = dec->vb + row0 * KV, *x1 = dec->x1 + row0 * H;
        float *gate = dec->gate + row0 * F, *up = dec->up + row0 * F, *ping = dec->ping + row0 * H;
        float *xo = x_out + row0 * H;
        const float *x = x_in + row0 * H;
        for (size_t l = layer_begin; l < layer_end; ++l) {
            bitnet_hip_bitlinear **P = &dec->proj[l * 7];
            const float *g_attn = dec->gamma + (l * 2) * H, *g_ffn = g_attn + H;
            const bool last = l + 1 == layer_end;
            // hidden states alternate between x_out and the internal buffer so that the last block writes x_out
            float *x2 = ((layer_end - 1 - l) % 2 == 0) ? xo : ping;
            float *qkv_out[3] = {(last && q_last) ? q_last + row0 * H : qb, (last && k_last) ? k_last + row0 * KV : kb, vb};
            run(&P[BITNET_HIP_PROJ_Q], 3, x, nullptr, H, BITNET_HIP_INPUT_PLAIN, g_attn, nullptr, qkv_out);
            float *o_out[1] = {x1};
            run(&P[BITNET_HIP_PROJ_O], 1, vb, nullptr, KV, BITNET_HIP_INPUT_GQA_BROADCAST, nullptr, x, o_out);
            float *gu_out[2] = {gate, up};
            run(&P[BITNET_HIP_PROJ_GATE], 2, x1, nullptr, H, BITNET_HIP_INPUT_PLAIN, g_ffn, nullptr, gu_out);
            float *d_out[1] = {x2};
            run(&P[BITNET_HIP_PROJ_DOWN], 1, gate, up, F, BITNET_HIP_INPUT_RELU2_MUL, nullptr, x1, d_out);
            x = x2;
        }
    };
    size_t chains = dec->chains ? dec->chains : 1;
    if (chains > m) chains = m;
    if (chains > dec->max_tokens) chains = dec->max_tokens;  // side streams exist for min(max_tokens, 8) chains
    if (chains <= 1) {
        run_chain(0, m, s);
    } else {
        // fork: the side streams start behind whatever the caller's stream holds; join: it continues behind them all.
        // Recorded into the caller's graph when s is being captured (the events pull the side streams into the capture).
        BITNET_HIP_TRY(hipEventRecord(dec->fork, s));
        const size_t base = m / chains, extra = m % chains;
        size_t row0 = base + (extra ? 1 : 0);
        for (size_t c = 1; c < chains; ++c) BITNET_HIP_TRY(hipStreamWaitEvent(dec->side[c - 1], dec->fork, 0));
        // every fork that was opened is joined again, also after a failed launch (an open fork would poison a capture)
        run_chain(0, row0, s);
        for (size_t c = 1; c < chains; ++c) {
            const size_t rows = base + (c < extra ? 1 : 0);
            run_chain(row0, rows, dec->side[c - 1]);
            row0 += rows;
            hipError_t e = hipEventRecord(dec->join[c - 1], dec->side[c - 1]);
            if (e == hipSuccess) e = hipStreamWaitEvent(s, dec->join[c - 1], 0);
            if (e != hipSuccess && rc == BITNET_HIP_OK)
                rc = fail(BITNET_HIP_DEVICE_ERROR, "decoder_decode: joining a row-group chain: %s", hipGetErrorString(e));
        }
    }
    if (rc == BITNET_HIP_OK && capturing == hipStreamCaptureStatusNone) {
        BITNET_HIP_TRY(hipEventRecord(dec->done, s));
        dec->done_stream = s;
        dec->done_recorded = true;
    }
    return rc;
}

int bitnet_hip_decoder_decode(bitnet_hip_decoder *dec, const float *x_in, size_t m, float *x_out, float *q_last,
                              float *k_last, void *stream)
{
    if (!dec) return fail(BITNET_HIP_NULL_POINTER, "decoder_decode: null argument");
    return bitnet_hip_decoder_decode_layers(dec, 0, dec->layers, x_in, m, x_out, q_last, k_last, stream);
}

}  // extern "C"

// ---------------------------------------------------------------------------------------------------
// A decode step recorded as a HIP graph
// ---------------------------------------------------------------------------------------------------
// A token step at batch 1 is 120 dependent launches of about 4 us each; enqueuing them one by one costs the host 2.8 to
// 4.5 us a launch (measured), which is as much as the GPU needs to run them, so the eager loop is bound by the host as
// often as not.  Replaying the recorded step costs the host under 0.1 ms and leaves the chain to the GPU alone.
struct bitnet_hip_decoder_graph {
    bitnet_hip_decoder *dec = nullptr;
    size_t layer_begin = 0, layer_end = 0;
    hipGraphExec_t exec = nullptr;

    ~bitnet_hip_decoder_graph()
    {
        if (exec) (void)hipGraphExecDestroy(exec);
    }
};

extern "C" {

int bitnet_hip_decoder_graph_create(bitnet_hip_decoder *dec, size_t layer_begin, size_t layer_end, const float *x_in,
                                    size_t m, float *x_out, float *q_last, float *k_last,
                                    bitnet_hip_decoder_graph **graph)
{
    if (!graph) return fail(BITNET_HIP_NULL_POINTER, "decoder_graph_create: graph is NULL");
    *graph = nullptr;
    if (!dec || !x_in || !x_out) return fail(BITNET_HIP_NULL_POINTER, "decoder_graph_create: null argument");
    if (m == 0 || layer_begin >= layer_end)
        return fail(BITNET_HIP_INVALID_CONFIG, "decoder_graph_create: nothing to record (m = %zu, layers [%zu, %zu))", m,
                    layer_begin, layer_end);
    std::unique_ptr<bitnet_hip_decoder_graph> g(new (std::nothrow) bitnet_hip_decoder_graph);
    if (!g) return fail(BITNET_HIP_MEMORY_ERROR, "decoder_graph_create: out of host memory");
    g->dec = dec; g->layer_begin = layer_begin; g->layer_end = layer_end;
    hipStream_t cs = nullptr;
    // a one-off: work queued on other streams that still writes x_in or reads x_out finishes first
    BITNET_HIP_TRY(hipDeviceSynchronize());
    BITNET_HIP_TRY(hipStreamCreateWithFlags(&cs, hipStreamNonBlocking));
    // The step runs once for real first: it validates the arguments, and every one-time set-up of the launchers
    // (a kernel's LDS limit) happens outside the recording.
    int rc = bitnet_hip_decoder_decode_layers(dec, layer_begin, layer_end, x_in, m, x_out, q_last, k_last, cs);
    if (rc == BITNET_HIP_OK && hipStreamSynchronize(cs) != hipSuccess)
        rc = fail(BITNET_HIP_KERNEL_ERROR, "decoder_graph_create: the step failed on the device");
    hipGraph_t recorded = nullptr;
    if (rc == BITNET_HIP_OK) {
        hipError_t e = hipStreamBeginCapture(cs, hipStreamCaptureModeThreadLocal);
        if (e != hipSuccess) {
            rc = fail(BITNET_HIP_DEVICE_ERROR, "decoder_graph_create: hipStreamBeginCapture: %s", hipGetErrorString(e));
        } else {
            rc = bitnet_hip_decoder_decode_layers(dec, layer_begin, layer_end, x_in, m, x_out, q_last, k_last, cs);
            e = hipStreamEndCapture(cs, &recorded);  // always ends the recording, also after a failed launch
            if (rc == BITNET_HIP_OK && e != hipSuccess)
                rc = fail(BITNET_HIP_DEVICE_ERROR, "decoder_graph_create: hipStreamEndCapture: %s", hipGetErrorString(e));
        }
    }
    if (rc == BITNET_HIP_OK) {
        hipError_t e = hipGraphInstantiate(&g->exec, recorded, nullptr, nullptr, 0);
        if (e != hipSuccess) rc = fail(BITNET_HIP_DEVICE_ERROR, "decoder_graph_create: hipGraphInstantiate: %s", hipGetErrorString(e));
    }
    if (recorded) (void)hipGraphDestroy(recorded);
    (void)hipStreamDestroy(cs);
    if (rc != BITNET_HIP_OK) return rc;
    *graph = g.release();
    return BITNET_HIP_OK;
}

int bitnet_hip_decoder_graph_launch(bitnet_hip_decoder_graph *graph, void *stream)
{
    if (!graph || !graph->exec) return fail(BITNET_HIP_NULL_POINTER, "decoder_graph_launch: null graph");
    bitnet_hip_decoder *dec = graph->dec;
    hipStream_t s = as_stream(stream);
    // as a decode call: readers of every projection involved, one step at a time on the decoder's buffers
    std::vector<std::shared_lock<std::shared_mutex>> guards;
    guards.reserve((graph->layer_end - graph->layer_begin) * 7);
    for (size_t i = graph->layer_begin * 7; i < graph->layer_end * 7; ++i) guards.emplace_back(dec->proj[i]->lock);
    std::lock_guard<std::mutex> one_decode(dec->decode_lock);
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(s, &capturing);
    if (dec->done_recorded && dec->done_stream != s && capturing == hipStreamCaptureStatusNone)
        BITNET_HIP_TRY(hipStreamWaitEvent(s, dec->done, 0));
    BITNET_HIP_TRY(hipGraphLaunch(graph->exec, s));
    if (capturing == hipStreamCaptureStatusNone) {
        BITNET_HIP_TRY(hipEventRecord(dec->done, s));
        dec->done_stream = s;
        dec->done_recorded = true;
    }
    return BITNET_HIP_OK;
}

void bitnet_hip_decoder_graph_destroy(bitnet_hip_decoder_graph *graph) { delete graph; }

}  // extern "C"

// ---------------------------------------------------------------------------------------------------
// Inference backend (InferenceBackend, bitnet-inference/src/engine/mod.rs:126-138)
// ---------------------------------------------------------------------------------------------------
struct bitnet_hip_backend {
    int device = 0;
    size_t total_mem = 0;
    bitnet_hip_decoder *model = nullptr;  // not owned
    float *stage_in = nullptr, *stage_out = nullptr;  // [max_tokens, hidden] each
    size_t stage_bytes = 0;
    std::mutex lock;  // execute_batch calls share the staging buffers
    // recorded behind the last call that used the staging buffers: a call on another stream waits for it
    hipEvent_t done = nullptr;
    hipStream_t done_stream = nullptr;
    bool done_recorded = false;

    ~bitnet_hip_backend()
    {
        if (stage_in) (void)hipFree(stage_in);
        if (stage_out) (void)hipFree(stage_out);
        if (done) (void)hipEventDestroy(done);
    }
};

namespace {
size_t decoder_device_bytes(const bitnet_hip_decoder *d)
{
    size_t total = 0;
    for (const bitnet_hip_bitlinear *p : d->proj) {
        total += (p->in_features * p->out_features + 3) / 4 + tiled_bytes(p->out_features, p->in_features) + sizeof(float);
        if (p->use_bias) total += sizeof(float) * p->out_features;
    }
    const size_t kv = d->kv_heads * d->head_dim, widest = d->hidden > d->ffn ? d->hidden : d->ffn, t = d->max_tokens;
    total += sizeof(float) * d->layers * 2 * d->hidden;                                        // norms
    total += t * widest + 2 * sizeof(float) * t;                                               // a8, a_scale, a_sum
    total += sizeof(float) * t * (d->hidden /*q*/ + 2 * kv + d->hidden /*x1*/ + 2 * d->ffn + d->hidden /*ping*/);
    return total;
}
}  // namespace

extern "C" {

int bitnet_hip_backend_create(int device, bitnet_hip_backend **backend)
{
    if (!backend) return fail(BITNET_HIP_NULL_POINTER, "backend_create: backend is NULL");
    *backend = nullptr;
    int rc = bitnet_hip_init(device);
    if (rc != BITNET_HIP_OK) return rc;
    bitnet_hip_backend *b = new (std::nothrow) bitnet_hip_backend;
    if (!b) return fail(BITNET_HIP_MEMORY_ERROR, "backend_create: out of host memory");
    b->device = device;
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) {
        delete b;
        return fail(BITNET_HIP_DEVICE_ERROR, "backend_create: hipGetDeviceProperties failed: %s", hipGetErrorString(e));
    }
    b->total_mem = prop.totalGlobalMem;
    e = hipEventCreateWithFlags(&b->done, hipEventDisableTiming);
    if (e != hipSuccess) {
        delete b;
        return fail(BITNET_HIP_DEVICE_ERROR, "backend_create: hipEventCreate failed: %s", hipGetErrorString(e));
    }
    *backend = b;
    return BITNET_HIP_OK;
}

void bitnet_hip_backend_destroy(bitnet_hip_backend *backend) { delete backend; }

int bitnet_hip_backend_optimize_model(bitnet_hip_backend *backend, bitnet_hip_decoder *model)
{
    if (!backend || !model) return fail(BITNET_HIP_NULL_POINTER, "backend_optimize_model: null argument");
    for (const bitnet_hip_bitlinear *p : model->proj)
        if (!p->has_weights) return fail(BITNET_HIP_NOT_INITIALIZED, "backend_optimize_model: a projection of the model has no weights yet");
    std::lock_guard<std::mutex> guard(backend->lock);
    const size_t bytes = sizeof(float) * model->max_tokens * model->hidden;
    if (bytes > backend->stage_bytes) {
        BITNET_HIP_TRY(hipDeviceSynchronize());
        if (backend->stage_in) (void)hipFree(backend->stage_in);
        if (backend->stage_out) (void)hipFree(backend->stage_out);
        backend->stage_in = backend->stage_out = nullptr;
        backend->stage_bytes = 0;
        hipError_t e = hipMalloc(reinterpret_cast<void **>(&backend->stage_in), bytes);
        if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&backend->stage_out), bytes);
        if (e != hipSuccess) return fail(BITNET_HIP_MEMORY_ERROR, "backend_optimize_model: hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
        backend->stage_bytes = bytes;
    }
    backend->model = model;
    return BITNET_HIP_OK;
}

int bitnet_hip_backend_execute_batch(bitnet_hip_backend *backend, const float *const *inputs, const size_t *rows,
                                     size_t count, float *const *outputs, void *stream)
{
    if (!backend) return fail(BITNET_HIP_NULL_POINTER, "backend_execute_batch: backend is NULL");
    std::lock_guard<std::mutex> guard(backend->lock);
    bitnet_hip_decoder *dec = backend->model;
    if (!dec) return fail(BITNET_HIP_NOT_INITIALIZED, "backend_execute_batch: no model bound (optimize_model first)");
    if (count == 0) return BITNET_HIP_OK;
    if (!inputs || !rows || !outputs) return fail(BITNET_HIP_NULL_POINTER, "backend_execute_batch: null argument");
    const size_t H = dec->hidden, cap = dec->max_tokens;
    hipStream_t s = as_stream(stream);
    for (size_t i = 0; i < count; ++i) {
        if (rows[i] != 0 && (!inputs[i] || !outputs[i])) return fail(BITNET_HIP_NULL_POINTER, "backend_execute_batch: input or output %zu is NULL", i);
        if (rows[i] > cap) {
            size_t e[2] = {cap, H}, a[2] = {rows[i], H};
            return fail_shape(e, 2, a, 2, "rows of one input exceed the model's max_tokens");
        }
    }
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(s, &capturing);
    if (backend->done_recorded && backend->done_stream != s && capturing == hipStreamCaptureStatusNone)
        BITNET_HIP_TRY(hipStreamWaitEvent(s, backend->done, 0));  // the staging buffers were last used on another stream
    bool staged = false;
    size_t i = 0;
    while (i < count) {
        // the longest run of inputs from i on whose rows fit one pass
        size_t j = i, total = 0;
        while (j < count && total + rows[j] <= cap) total += rows[j++];
        if (total == 0) { i = j > i ? j : i + 1; continue; }
        if (j == i + 1) {  // one input: no staging
            int rc = bitnet_hip_decoder_decode(dec, inputs[i], rows[i], outputs[i], nullptr, nullptr, stream);
            if (rc != BITNET_HIP_OK) return rc;
        } else {
            size_t at = 0;
            staged = true;
            for (size_t t = i; t < j; ++t) {
                if (rows[t] == 0) continue;
                BITNET_HIP_TRY(hipMemcpyAsync(backend->stage_in + at * H, inputs[t], sizeof(float) * rows[t] * H, hipMemcpyDeviceToDevice, s));
                at += rows[t];
            }
            int rc = bitnet_hip_decoder_decode(dec, backend->stage_in, total, backend->stage_out, nullptr, nullptr, stream);
            if (rc != BITNET_HIP_OK) return rc;
            at = 0;
            for (size_t t = i; t < j; ++t) {
                if (rows[t] == 0) continue;
                BITNET_HIP_TRY(hipMemcpyAsync(outputs[t], backend->stage_out + at * H, sizeof(float) * rows[t] * H, hipMemcpyDeviceToDevice, s));
                at += rows[t];
            }
        }
        i = j;
    }
    if (staged && capturing == hipStreamCaptureStatusNone) {
        BITNET_HIP_TRY(hipEventRecord(backend->done, s));
        backend->done_stream = s;
        backend->done_recorded = true;
    }
    return BITNET_HIP_OK;
}

size_t bitnet_hip_backend_get_memory_usage(const bitnet_hip_backend *backend)
{
    if (!backend || !backend->model) return 0;
    return decoder_device_bytes(backend->model) + 2 * backend->stage_bytes;
}

int bitnet_hip_backend_capabilities(const bitnet_hip_backend *backend, int *supports_batching, int *supports_streaming,
                                    size_t *max_batch_size, size_t *memory_limit, int *device)
{
    if (!backend) return fail(BITNET_HIP_NULL_POINTER, "backend_capabilities: backend is NULL");
    if (supports_batching) *supports_batching = 1;
    if (supports_streaming) *supports_streaming = 0;
    if (max_batch_size) *max_batch_size = backend->model ? backend->model->max_tokens : 0;
    if (memory_limit) *memory_limit = backend->total_mem;
    if (device) *device = backend->device;
    return BITNET_HIP_OK;
}

}  // extern "C"
