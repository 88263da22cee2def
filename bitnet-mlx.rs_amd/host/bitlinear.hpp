// C++ host-side mirror of the reference's Rust types for the BitLinear path, over the C ABI
// (include/bitnet_hip.h).  Header only.  Names, fields and error behaviour follow the reference so that
// call sites translate line by line:
//
//   bitnet::BitLinearError            bitnet-quant/src/bitlinear/error.rs:10-84 (variant + message; ShapeMismatch
//                                     carries expected / actual)
//   bitnet::BitLinearConfig           bitnet-quant/src/bitlinear/layer.rs:20-75
//   bitnet::BitLinear                 bitnet-quant/src/bitlinear/layer.rs:82-109,113-179,299-352 and the
//                                     BitLinearForward trait, bitnet-quant/src/bitlinear/forward.rs:14-51
//   bitnet::TernaryProcessor          bitnet-inference/src/engine/ternary_operations.rs:56-172
//   bitnet::QuantizedActivation, absmax_quantize_activations
//                                     bitnet-quant/src/quantization/activations.rs:95-112,530-641
//   bitnet::ActivationQuantizationConfig, DynamicActivationQuantizer
//                                     bitnet-quant/src/quantization/activations.rs:14-91,203-454
//   bitnet::WeightQuantizationConfig, BitNetWeightQuantizer, QuantizedWeight
//                                     bitnet-quant/src/quantization/weights.rs:58-95,158-175,341-611
//   bitnet::HipInferenceBackend       the InferenceBackend trait, bitnet-inference/src/engine/mod.rs:126-148
//   bitnet::BitLinearLayer            bitnet-inference/src/engine/transformer_layers.rs:68-202
//   bitnet::FeedForwardNetwork        bitnet-inference/src/engine/transformer_layers.rs:553-623
//
// Rust returns Result<T, E>; here every fallible call returns a Result<T> holding either the value or the
// error.  Nothing throws and nothing aborts.  Tensors are dense row-major f32 buffers in device memory
// (DeviceTensor owns its allocation, like the fresh Tensor the reference's forward returns).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <memory>
#include <mutex>
#include <optional>
#include <string>
#include <utility>
#include <vector>

#include "../../include/bitnet_hip.h"

namespace bitnet {

struct BitLinearError {
    enum Kind { ShapeMismatch = 1, ConfigError, DeviceError, MemoryError, QuantizationError, NotInitialized,
                KernelError, NullPointer, Unsupported };
    Kind kind;
    std::string message;
    std::vector<size_t> expected, actual;  // ShapeMismatch only
};

template <class T>
class Result {
public:
    Result(T v) : value_(std::move(v)) {}
    Result(BitLinearError e) : error_(std::move(e)) {}
    bool is_ok() const { return value_.has_value(); }
    bool is_err() const { return !is_ok(); }
    T &unwrap() { return *value_; }
    const BitLinearError &unwrap_err() const { return *error_; }

private:
    std::optional<T> value_;
    std::optional<BitLinearError> error_;
};
struct Unit {};

inline BitLinearError last_error(int status)
{
    BitLinearError e{static_cast<BitLinearError::Kind>(status), bitnet_hip_last_error(), {}, {}};
    if (status == BITNET_HIP_SHAPE_MISMATCH) {
        size_t ex[4], ac[4];
        int ar = 0;
        int er = bitnet_hip_last_shape_mismatch(ex, ac, &ar);
        e.expected.assign(ex, ex + er);
        e.actual.assign(ac, ac + ar);
    }
    return e;
}

// Dense f32 tensor in device memory.
class DeviceTensor {
public:
    DeviceTensor() = default;
    static Result<DeviceTensor> zeros(std::vector<size_t> dims)
    {
        DeviceTensor t;
        t.dims_ = std::move(dims);
        size_t n = t.elem_count();
        float *p = nullptr;
        if (hipMalloc(reinterpret_cast<void **>(&p), (n ? n : 1) * sizeof(float)) != hipSuccess)
            return BitLinearError{BitLinearError::MemoryError, "hipMalloc failed", {}, {}};
        (void)hipMemset(p, 0, n * sizeof(float));
        t.data_.reset(p, [](float *q) { (void)hipFree(q); });
        return t;
    }
    static Result<DeviceTensor> from_vec(const std::vector<float> &host, std::vector<size_t> dims)
    {
        auto r = zeros(std::move(dims));
        if (r.is_err()) return r;
        if (r.unwrap().elem_count() != host.size())
            return BitLinearError{BitLinearError::ShapeMismatch, "from_vec: element count", {r.unwrap().elem_count()}, {host.size()}};
        (void)hipMemcpy(r.unwrap().data(), host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice);
        return r;
    }
    std::vector<float> to_vec() const
    {
        std::vector<float> h(elem_count());
        (void)hipDeviceSynchronize();
        (void)hipMemcpy(h.data(), data_.get(), h.size() * sizeof(float), hipMemcpyDeviceToHost);
        return h;
    }
    const std::vector<size_t> &dims() const { return dims_; }
    size_t elem_count() const
    {
        size_t n = 1;
        for (size_t d : dims_) n *= d;
        return n;
    }
    float *data() const { return data_.get(); }

private:
    std::vector<size_t> dims_;
    std::shared_ptr<float> data_;
};

struct BitLinearConfig {
    size_t in_features = 512;
    size_t out_features = 512;
    bool use_bias = false;  // BitNet standard is bias-free
    int ternary_method = BITNET_HIP_TERNARY_ABSMEAN_ROUNDCLIP;
    float threshold_factor = 0.5f;
    float rms_norm_eps = 1e-5f;
    int sum_order = BITNET_HIP_SUM_BLOCK256;
};

class BitLinear {
public:
    // BitLinear::new(config, layer_name)
    static Result<std::shared_ptr<BitLinear>> create(const BitLinearConfig &config, std::string layer_name)
    {
        bitnet_hip_bitlinear *h = nullptr;
        int rc = bitnet_hip_bitlinear_create(config.in_features, config.out_features, config.use_bias, &h);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        return std::shared_ptr<BitLinear>(new BitLinear(config, std::move(layer_name), h));
    }
    ~BitLinear()
    {
        bitnet_hip_bitlinear_destroy(handle_);
        if (workspace_) (void)hipFree(workspace_);
        if (workspace_done_) (void)hipEventDestroy(workspace_done_);
    }
    BitLinear(const BitLinear &) = delete;
    BitLinear &operator=(const BitLinear &) = delete;

    const BitLinearConfig &config() const { return config_; }
    const std::string &layer_name() const { return layer_name_; }
    bitnet_hip_bitlinear *handle() const { return handle_; }
    // BitLinear::device (layer.rs:223): the ordinal of the GPU the layer's buffers were allocated on
    int device() const { return device_; }
    // BitLinear::clear_cache (layer.rs:353-361): the reference caches the quantised form of its latent f32 weights;
    // this layer holds only the quantised weights (update_weights quantises at once), so there is nothing to clear
    Result<Unit> clear_cache() const { return Unit{}; }
    // BitLinear::to_device (layer.rs:376-411): the same device is the reference's no-op, any other is refused
    Result<Unit> to_device(int device)
    {
        if (device == device_) return Unit{};
        return BitLinearError{BitLinearError::DeviceError, "Failed to move weights to device: the layer lives on one GPU", {}, {}};
    }

    // update_weights: latent f32 [out_features, in_features] in host memory
    Result<Unit> update_weights(const std::vector<float> &w, size_t rows, size_t cols)
    {
        int rc = bitnet_hip_bitlinear_set_weights_f32(handle_, w.data(), rows, cols, BITNET_HIP_LAYOUT_OUT_IN, 0,
                                                      config_.ternary_method, config_.threshold_factor, nullptr);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        return Unit{};
    }
    Result<Unit> update_bias(const std::vector<float> &b)
    {
        int rc = bitnet_hip_bitlinear_set_bias(handle_, b.data(), b.size(), 0, nullptr);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        return Unit{};
    }
    // BitLinearForward::forward: [.., in_features] -> [.., out_features]
    Result<DeviceTensor> forward(const DeviceTensor &input, const float *gamma = nullptr, hipStream_t stream = nullptr) const
    {
        std::vector<size_t> out_dims = input.dims();
        if (!out_dims.empty()) out_dims.back() = config_.out_features;
        auto out = DeviceTensor::zeros(out_dims.empty() ? std::vector<size_t>{config_.out_features} : out_dims);
        if (out.is_err()) return out;
        // the scratch for the quantised activations is kept by the layer and grown on demand: no allocation per call
        size_t rows = input.dims().empty() ? 0 : input.elem_count() / (input.dims().back() ? input.dims().back() : 1);
        std::lock_guard<std::mutex> guard(workspace_lock_);
        const size_t need = bitnet_hip_bitlinear_workspace_size(handle_, rows);
        if (need > workspace_bytes_) {
            (void)hipDeviceSynchronize();
            if (workspace_) (void)hipFree(workspace_);
            workspace_ = nullptr;
            workspace_bytes_ = 0;
            if (hipMalloc(&workspace_, need) != hipSuccess)
                return BitLinearError{BitLinearError::MemoryError, "hipMalloc failed", {}, {}};
            workspace_bytes_ = need;
        }
        // the scratch is shared by every forward of this layer: a call on another stream than the one before it waits,
        // on the GPU, for that call to finish with it (the lock above orders only the enqueue)
        if (!workspace_done_ && hipEventCreateWithFlags(&workspace_done_, hipEventDisableTiming) != hipSuccess)
            return BitLinearError{BitLinearError::DeviceError, "hipEventCreate failed", {}, {}};
        if (workspace_used_ && workspace_stream_ != stream && hipStreamWaitEvent(stream, workspace_done_, 0) != hipSuccess)
            return BitLinearError{BitLinearError::DeviceError, "hipStreamWaitEvent failed", {}, {}};
        int rc = bitnet_hip_bitlinear_forward(handle_, input.data(), input.dims().data(), (int)input.dims().size(), gamma,
                                              config_.rms_norm_eps, config_.sum_order, nullptr, out.unwrap().data(),
                                              workspace_, workspace_bytes_, nullptr, nullptr, nullptr, stream);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        if (hipEventRecord(workspace_done_, stream) != hipSuccess)
            return BitLinearError{BitLinearError::DeviceError, "hipEventRecord failed", {}, {}};
        workspace_stream_ = stream;
        workspace_used_ = true;
        return out;
    }
    Result<DeviceTensor> forward_batch(const DeviceTensor &inputs) const
    {
        if (inputs.dims().size() < 2)
            return BitLinearError{BitLinearError::ShapeMismatch, "forward_batch needs at least 2 dimensions",
                                  {1, 1, config_.in_features}, inputs.dims()};
        return forward(inputs);
    }

private:
    BitLinear(BitLinearConfig c, std::string n, bitnet_hip_bitlinear *h) : config_(c), layer_name_(std::move(n)), handle_(h)
    {
        (void)hipGetDevice(&device_);
    }
    BitLinearConfig config_;
    std::string layer_name_;
    bitnet_hip_bitlinear *handle_;
    int device_ = 0;
    mutable std::mutex workspace_lock_;  // forward calls of one layer share the scratch: one at a time through this mirror
    mutable void *workspace_ = nullptr;
    mutable size_t workspace_bytes_ = 0;
    mutable hipEvent_t workspace_done_ = nullptr;  // recorded behind every forward, on its stream
    mutable hipStream_t workspace_stream_ = nullptr;
    mutable bool workspace_used_ = false;
};

// TernaryProcessor: per-token int8 absmax quantisation and the ternary matmul on top of it.
struct QuantizedActivations {
    int8_t *values = nullptr;   // [m, k] device
    float *scales = nullptr;    // [m] device (127 / absmax)
    int32_t *row_sums = nullptr;
    size_t m = 0, k = 0;
    ~QuantizedActivations()
    {
        if (values) (void)hipFree(values);
        if (scales) (void)hipFree(scales);
        if (row_sums) (void)hipFree(row_sums);
    }
};

class TernaryProcessor {
public:
    // quantize_activations: input [m, k] (rank 1 is one token)
    Result<std::shared_ptr<QuantizedActivations>> quantize_activations(const DeviceTensor &input, hipStream_t stream = nullptr)
    {
        auto q = std::make_shared<QuantizedActivations>();
        q->k = input.dims().empty() ? 0 : input.dims().back();
        q->m = q->k ? input.elem_count() / q->k : 0;
        if (hipMalloc(reinterpret_cast<void **>(&q->values), q->m * q->k + 1) != hipSuccess ||
            hipMalloc(reinterpret_cast<void **>(&q->scales), (q->m + 1) * sizeof(float)) != hipSuccess ||
            hipMalloc(reinterpret_cast<void **>(&q->row_sums), (q->m + 1) * sizeof(int32_t)) != hipSuccess)
            return BitLinearError{BitLinearError::MemoryError, "hipMalloc failed", {}, {}};
        int rc = bitnet_hip_quantize_activations_i8(input.data(), nullptr, q->k, q->m, q->k, BITNET_HIP_INPUT_PLAIN, 1, 1,
                                                    nullptr, 0.0f, BITNET_HIP_SUM_BLOCK256, q->values, q->scales,
                                                    q->row_sums, nullptr, stream);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        ++activations_quantized;
        return q;
    }
    // ternary_matmul(weights, input, output): output [m, out] = input [m, in] through the layer's ternary weights
    Result<Unit> ternary_matmul(const BitLinear &weights, const DeviceTensor &input, DeviceTensor &output, hipStream_t stream = nullptr)
    {
        const size_t in = weights.config().in_features, outf = weights.config().out_features;
        if (input.dims().size() != 2 || input.dims()[1] != in)
            return BitLinearError{BitLinearError::ShapeMismatch, "ternary_matmul input", {input.dims().empty() ? 1 : input.dims()[0], in}, input.dims()};
        if (output.dims().size() != 2 || output.dims()[0] != input.dims()[0] || output.dims()[1] != outf)
            return BitLinearError{BitLinearError::ShapeMismatch, "ternary_matmul output", {input.dims()[0], outf}, output.dims()};
        auto q = quantize_activations(input, stream);
        if (q.is_err()) return q.unwrap_err();
        int rc = bitnet_hip_bitlinear_matmul(weights.handle(), q.unwrap()->values, q.unwrap()->row_sums, q.unwrap()->m,
                                             q.unwrap()->scales, nullptr, nullptr, output.data(), stream);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        (void)hipStreamSynchronize(stream);  // the quantised activations are released on return
        ++ternary_multiplications;
        return Unit{};
    }
    uint64_t ternary_multiplications = 0, activations_quantized = 0;  // TernaryStats
};

// BitLinearLayer::forward handles rank 2 and rank 3 inputs (transformer_layers.rs:119-201).
class BitLinearLayer {
public:
    static Result<std::shared_ptr<BitLinearLayer>> create(size_t in_features, size_t out_features, bool use_bias, std::string name)
    {
        BitLinearConfig c;
        c.in_features = in_features; c.out_features = out_features; c.use_bias = use_bias;
        auto l = BitLinear::create(c, std::move(name));
        if (l.is_err()) return l.unwrap_err();
        auto p = std::shared_ptr<BitLinearLayer>(new BitLinearLayer());
        p->in_features = in_features; p->out_features = out_features; p->layer = l.unwrap();
        return p;
    }
    Result<DeviceTensor> forward(const DeviceTensor &input) const { return layer->forward(input); }
    size_t in_features = 0, out_features = 0;
    std::shared_ptr<BitLinear> layer;
};

// FeedForwardNetwork::forward: down( up(x) * relu(gate(x))^2 ) (transformer_layers.rs:603-623).  gate and up
// share one activation quantisation; the ReLU^2 gating is fused into the quantiser in front of down.
class FeedForwardNetwork {
public:
    std::shared_ptr<BitLinear> up_proj, gate_proj, down_proj;
    Result<DeviceTensor> forward(const DeviceTensor &input, hipStream_t stream = nullptr) const
    {
        const size_t hidden = up_proj->config().in_features, ffn = up_proj->config().out_features;
        if (input.dims().size() != 2 || input.dims()[1] != hidden)
            return BitLinearError{BitLinearError::ShapeMismatch, "ffn input", {1, hidden}, input.dims()};
        const size_t m = input.dims()[0];
        auto gate = DeviceTensor::zeros({m, ffn}), up = DeviceTensor::zeros({m, ffn}), out = DeviceTensor::zeros({m, hidden});
        if (gate.is_err() || up.is_err() || out.is_err()) return BitLinearError{BitLinearError::MemoryError, "hipMalloc failed", {}, {}};
        bitnet_hip_bitlinear *layers[2] = {gate_proj->handle(), up_proj->handle()};
        float *outs[2] = {gate.unwrap().data(), up.unwrap().data()};
        int rc = bitnet_hip_bitlinear_forward_multi(layers, 2, input.data(), m, nullptr, 0.0f, BITNET_HIP_SUM_BLOCK256, outs,
                                                    nullptr, 0, stream);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        TernaryProcessor tp;
        QuantizedActivations q;
        q.m = m; q.k = ffn;
        if (hipMalloc(reinterpret_cast<void **>(&q.values), m * ffn) != hipSuccess ||
            hipMalloc(reinterpret_cast<void **>(&q.scales), m * sizeof(float)) != hipSuccess ||
            hipMalloc(reinterpret_cast<void **>(&q.row_sums), m * sizeof(int32_t)) != hipSuccess)
            return BitLinearError{BitLinearError::MemoryError, "hipMalloc failed", {}, {}};
        rc = bitnet_hip_quantize_activations_i8(gate.unwrap().data(), up.unwrap().data(), ffn, m, ffn, BITNET_HIP_INPUT_RELU2_MUL,
                                                1, 1, nullptr, 0.0f, BITNET_HIP_SUM_BLOCK256, q.values, q.scales, q.row_sums,
                                                nullptr, stream);
        if (rc == BITNET_HIP_OK)
            rc = bitnet_hip_bitlinear_matmul(down_proj->handle(), q.values, q.row_sums, m, q.scales, nullptr, nullptr,
                                             out.unwrap().data(), stream);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        (void)hipStreamSynchronize(stream);
        return out;
    }
};

// absmax_quantize_activations: ONE scale for the whole tensor, ternary codes (the default precision) or 8-bit values.
enum class QuantizationPrecision { OneFiveFiveBit = BITNET_HIP_PRECISION_ONE_FIVE_FIVE_BIT, EightBit = BITNET_HIP_PRECISION_EIGHT_BIT };
// QuantizationStats (bitnet-quant/src/quantization/mod.rs:118-148) with its defaults
struct QuantizationStats {
    size_t elements_count = 0;
    float quantization_error = 0.f, compression_ratio = 1.f, min_value = 0.f, max_value = 0.f, scale_factor = 1.f;
    std::optional<int> zero_point;
};
struct QuantizedActivation {
    std::shared_ptr<int8_t> values;  // device, original_shape elements (signed: the reference's U8 cast loses the sign)
    float scales = 1.f;              // the one scale of the tensor
    std::vector<size_t> original_shape;
    QuantizationPrecision precision = QuantizationPrecision::OneFiveFiveBit;
    QuantizationStats stats;
    float effective_bit_width() const { return precision == QuantizationPrecision::OneFiveFiveBit ? 1.58f : 8.0f; }
};
inline Result<QuantizedActivation> absmax_quantize_activations(const DeviceTensor &activations,
                                                               std::optional<QuantizationPrecision> precision = std::nullopt,
                                                               hipStream_t stream = nullptr)
{
    QuantizedActivation q;
    q.precision = precision.value_or(QuantizationPrecision::OneFiveFiveBit);
    q.original_shape = activations.dims();
    const size_t n = activations.elem_count();
    int8_t *v = nullptr;
    float *st = nullptr;
    if (hipMalloc(reinterpret_cast<void **>(&v), n ? n : 1) != hipSuccess || hipMalloc(reinterpret_cast<void **>(&st), 4 * sizeof(float)) != hipSuccess)
        return BitLinearError{BitLinearError::MemoryError, "hipMalloc failed", {}, {}};
    q.values.reset(v, [](int8_t *p) { (void)hipFree(p); });
    std::shared_ptr<float> st_guard(st, [](float *p) { (void)hipFree(p); });
    int rc = bitnet_hip_absmax_quantize_activations(activations.data(), n, static_cast<int>(q.precision), v, st, stream);
    if (rc != BITNET_HIP_OK) return last_error(rc);
    float h[4];
    (void)hipMemcpy(h, st, sizeof h, hipMemcpyDeviceToHost);
    q.scales = h[0];
    q.stats = {n, h[1], 32.0f / q.effective_bit_width(), h[2], h[3], h[0]};
    return q;
}

// DynamicActivationQuantizer (activations.rs:203-454): the state (exponential moving average of the scale, window of
// recent scales, warm-up counter, calibration flag) on the host in single precision, as the reference keeps it; abs-max and
// the quantisation with the current scale on the device.
struct ActivationQuantizationConfig {  // activations.rs:14-45, with its defaults
    QuantizationPrecision precision = QuantizationPrecision::OneFiveFiveBit;
    size_t moving_average_window = 100;
    float outlier_percentile = 99.9f;
    bool per_token = false;
    size_t calibration_warmup = 50;
    float ema_decay = 0.99f;
    bool quantize_attention = true;
    Result<Unit> validate() const  // :71-91
    {
        if (moving_average_window == 0) return BitLinearError{BitLinearError::ConfigError, "Moving average window cannot be zero", {}, {}};
        if (outlier_percentile <= 0.0f || outlier_percentile > 100.0f)
            return BitLinearError{BitLinearError::ConfigError, "Outlier percentile must be in range (0, 100]", {}, {}};
        if (ema_decay < 0.0f || ema_decay > 1.0f) return BitLinearError{BitLinearError::ConfigError, "EMA decay must be in range [0, 1]", {}, {}};
        return Unit{};
    }
};
class DynamicActivationQuantizer {
public:
    explicit DynamicActivationQuantizer(ActivationQuantizationConfig c = {}) : config_(c) {}
    const ActivationQuantizationConfig &config() const { return config_; }
    // quantize (:315-360): the moving average if there is one, else the tensor's own abs-max
    Result<QuantizedActivation> quantize(const DeviceTensor &activations, hipStream_t stream = nullptr) const
    {
        if (activations.dims().empty())
            return BitLinearError{BitLinearError::QuantizationError, "Activation tensor must have at least 1 dimension", {}, {}};
        const size_t n = activations.elem_count();
        float scale = 0.0f;
        if (ema_scale_) {
            scale = *ema_scale_;
        } else {
            int rc = bitnet_hip_abs_max(activations.data(), n, &scale, stream);
            if (rc != BITNET_HIP_OK) return last_error(rc);
        }
        QuantizedActivation q;
        q.precision = config_.precision;
        q.original_shape = activations.dims();
        int8_t *v = nullptr;
        if (hipMalloc(reinterpret_cast<void **>(&v), n ? n : 1) != hipSuccess)
            return BitLinearError{BitLinearError::MemoryError, "hipMalloc failed", {}, {}};
        q.values.reset(v, [](int8_t *p) { (void)hipFree(p); });
        int rc = bitnet_hip_quantize_activations_scaled(activations.data(), n, static_cast<int>(q.precision), scale, 0, v, stream);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        q.scales = scale;
        q.stats.elements_count = n;
        q.stats.scale_factor = scale;
        q.stats.compression_ratio = 32.0f / q.effective_bit_width();
        return q;
    }
    // quantize_dynamic (:372-383): count the step, update the moving average, quantise with it
    Result<QuantizedActivation> quantize_dynamic(const DeviceTensor &activations, hipStream_t stream = nullptr)
    {
        ++step_count_;
        auto up = update_dynamic_params(activations, stream);
        if (up.is_err()) return up.unwrap_err();
        return quantize(activations, stream);
    }
    // update_dynamic_params + compute_dynamic_scale (:241-267, 406-433)
    Result<Unit> update_dynamic_params(const DeviceTensor &activations, hipStream_t stream = nullptr)
    {
        float abs_max = 0.0f;
        int rc = bitnet_hip_abs_max(activations.data(), activations.elem_count(), &abs_max, stream);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        const float current = config_.precision == QuantizationPrecision::EightBit ? abs_max / 127.0f : abs_max / 1.0f;
        if (ema_scale_) {
            const float kept = config_.ema_decay * *ema_scale_, fresh = (1.0f - config_.ema_decay) * current;
            ema_scale_ = kept + fresh;
        } else {
            ema_scale_ = current;
        }
        if (scale_history_.size() >= config_.moving_average_window) scale_history_.erase(scale_history_.begin());
        scale_history_.push_back(current);
        if (step_count_ <= config_.calibration_warmup) {
            if (calibration_samples_ < config_.calibration_warmup) ++calibration_samples_;
        } else if (!calibrated_) {
            calibrated_ = true;
        }
        return Unit{};
    }
    float get_dynamic_scales() const { return ema_scale_.value_or(1.0f); }
    void reset_dynamic_state()
    {
        scale_history_.clear();
        ema_scale_.reset();
        calibrated_ = false;
        step_count_ = 0;
        calibration_samples_ = 0;
    }
    bool needs_calibration() const { return !calibrated_ || step_count_ <= config_.calibration_warmup; }
    const std::vector<float> &scale_history() const { return scale_history_; }

private:
    ActivationQuantizationConfig config_;
    std::vector<float> scale_history_;
    std::optional<float> ema_scale_;
    bool calibrated_ = false;
    size_t step_count_ = 0, calibration_samples_ = 0;
};

// BitNetWeightQuantizer::quantize with its whole configuration (weights.rs:568-611).
enum class TernaryMethod { MeanThreshold = 0, MedianThreshold, AdaptiveThreshold, OptimalThreshold, DetSTE };
struct WeightQuantizationConfig {
    bool normalize_weights = true;
    float outlier_threshold = 3.0f;
    TernaryMethod ternary_method = TernaryMethod::MeanThreshold;
    std::optional<float> custom_threshold_factor;
};
struct QuantizedWeight {
    std::vector<int8_t> values;   // ternary, [rows * cols]
    std::vector<uint8_t> packed;  // the reference's 2-bit bytes
    float scales = 1.f;
    std::vector<size_t> original_shape;
};
class BitNetWeightQuantizer {
public:
    explicit BitNetWeightQuantizer(WeightQuantizationConfig c = {}) : config_(c) {}
    const WeightQuantizationConfig &config() const { return config_; }
    // Quantizer::validate_input (weights.rs:625-639)
    Result<Unit> validate_input(const DeviceTensor &weights) const
    {
        if (weights.dims().size() < 2)
            return BitLinearError{BitLinearError::QuantizationError, "Weight tensor must have at least 2 dimensions", {}, {}};
        return Unit{};
    }
    // Quantizer::dequantize (weights.rs:616-619): values * scales, on the host
    std::vector<float> dequantize(const QuantizedWeight &q) const
    {
        std::vector<float> out(q.values.size());
        for (size_t i = 0; i < out.size(); ++i) out[i] = static_cast<float>(q.values[i]) * q.scales;
        return out;
    }
    // Quantizer::get_stats (weights.rs:638-640): the quantizer's own record, which quantize(&self) never updates in the
    // reference, so the defaults
    QuantizationStats get_stats() const { return QuantizationStats{}; }
    // weights: [rows, cols] f32 on the device
    Result<QuantizedWeight> quantize(const DeviceTensor &weights, hipStream_t stream = nullptr) const
    {
        if (weights.dims().size() < 2)
            return BitLinearError{BitLinearError::QuantizationError, "Weight tensor must have at least 2 dimensions", {}, {}};
        const size_t rows = weights.dims()[0], cols = weights.elem_count() / (rows ? rows : 1), n = rows * cols;
        uint8_t *packed = nullptr;
        int8_t *q = nullptr;
        float *scale = nullptr;
        if (hipMalloc(reinterpret_cast<void **>(&packed), (n + 3) / 4 + 1) != hipSuccess ||
            hipMalloc(reinterpret_cast<void **>(&q), n + 1) != hipSuccess || hipMalloc(reinterpret_cast<void **>(&scale), sizeof(float)) != hipSuccess) {
            (void)hipFree(packed); (void)hipFree(q); (void)hipFree(scale);  // hipFree(nullptr) is a no-op
            return BitLinearError{BitLinearError::MemoryError, "hipMalloc failed", {}, {}};
        }
        int rc = bitnet_hip_quantize_weights_reference(weights.data(), rows, cols, static_cast<int>(config_.ternary_method),
                                                       config_.normalize_weights, config_.outlier_threshold,
                                                       config_.custom_threshold_factor.value_or(0.0f), packed, scale, q, nullptr, stream);
        QuantizedWeight out;
        if (rc == BITNET_HIP_OK) {
            out.values.resize(n);
            out.packed.resize((n + 3) / 4);
            out.original_shape = weights.dims();
            (void)hipMemcpy(out.values.data(), q, n, hipMemcpyDeviceToHost);
            (void)hipMemcpy(out.packed.data(), packed, out.packed.size(), hipMemcpyDeviceToHost);
            (void)hipMemcpy(&out.scales, scale, sizeof(float), hipMemcpyDeviceToHost);
        }
        (void)hipFree(packed); (void)hipFree(q); (void)hipFree(scale);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        return out;
    }

private:
    WeightQuantizationConfig config_;
};

// The projections of a stack of decoder blocks, and the InferenceBackend that executes batches through them.
class DecoderProjections {
public:
    static Result<std::shared_ptr<DecoderProjections>> create(size_t layers, size_t hidden, size_t ffn, size_t q_heads, size_t kv_heads,
                                                              size_t head_dim, float eps, size_t max_tokens)
    {
        bitnet_hip_decoder *h = nullptr;
        int rc = bitnet_hip_decoder_create(layers, hidden, ffn, q_heads, kv_heads, head_dim, eps, BITNET_HIP_SUM_BLOCK256, max_tokens, &h);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        auto d = std::shared_ptr<DecoderProjections>(new DecoderProjections());
        d->handle_ = h; d->hidden = hidden; d->max_tokens = max_tokens; d->layers = layers;
        return d;
    }
    ~DecoderProjections() { bitnet_hip_decoder_destroy(handle_); }
    // latent f32 weights [out, in] of projection `proj` (BITNET_HIP_PROJ_*) of block `layer`, host memory
    Result<Unit> update_weights(size_t layer, int proj, const std::vector<float> &w, size_t rows, size_t cols)
    {
        bitnet_hip_bitlinear *bl = nullptr;
        int rc = bitnet_hip_decoder_projection(handle_, layer, proj, &bl);
        if (rc == BITNET_HIP_OK)
            rc = bitnet_hip_bitlinear_set_weights_f32(bl, w.data(), rows, cols, BITNET_HIP_LAYOUT_OUT_IN, 0,
                                                      BITNET_HIP_TERNARY_ABSMEAN_ROUNDCLIP, 0.5f, nullptr);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        return Unit{};
    }
    // row groups a step of several token rows is split into, each a chain of launches on its own stream (0 and 1 = one chain, the default)
    Result<Unit> set_chains(size_t chains)
    {
        int rc = bitnet_hip_decoder_set_chains(handle_, chains);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        return Unit{};
    }
    Result<DeviceTensor> decode(const DeviceTensor &x) const
    {
        auto out = DeviceTensor::zeros(x.dims());
        if (out.is_err()) return out;
        int rc = bitnet_hip_decoder_decode(handle_, x.data(), x.dims().empty() ? 0 : x.dims()[0], out.unwrap().data(), nullptr, nullptr, nullptr);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        return out;
    }
    // The decode step x -> out recorded as a HIP graph (the step runs once while it is recorded); replay() enqueues it
    // with one call.  The graph shares ownership of nothing: keep the decoder and both tensors alive while it is used.
    class Graph {
    public:
        Graph(Graph &&o) noexcept : handle_(o.handle_) { o.handle_ = nullptr; }
        Graph(const Graph &) = delete;
        Graph &operator=(const Graph &) = delete;
        ~Graph() { if (handle_) bitnet_hip_decoder_graph_destroy(handle_); }
        Result<Unit> replay(void *stream = nullptr) const
        {
            int rc = bitnet_hip_decoder_graph_launch(handle_, stream);
            if (rc != BITNET_HIP_OK) return last_error(rc);
            return Unit{};
        }
    private:
        friend class DecoderProjections;
        explicit Graph(bitnet_hip_decoder_graph *h) : handle_(h) {}
        bitnet_hip_decoder_graph *handle_ = nullptr;
    };
    Result<Graph> record(const DeviceTensor &x, DeviceTensor &out) const
    {
        if (x.dims().size() != 2 || x.dims() != out.dims())
            return BitLinearError{BitLinearError::ShapeMismatch, "record: x and out must be [m, hidden] tensors of one shape", x.dims(), out.dims()};
        bitnet_hip_decoder_graph *g = nullptr;
        int rc = bitnet_hip_decoder_graph_create(handle_, 0, layers, x.data(), x.dims()[0], out.data(), nullptr, nullptr, &g);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        return Graph(g);
    }
    bitnet_hip_decoder *handle() const { return handle_; }
    size_t hidden = 0, max_tokens = 0, layers = 0;

private:
    DecoderProjections() = default;
    bitnet_hip_decoder *handle_ = nullptr;
};

struct BackendCapabilities {
    bool supports_batching = false, supports_streaming = false;
    size_t max_batch_size = 0;
    std::optional<size_t> memory_limit;
    int device = 0;
};
class HipInferenceBackend {
public:
    static Result<std::shared_ptr<HipInferenceBackend>> create(int device = 0)
    {
        bitnet_hip_backend *h = nullptr;
        int rc = bitnet_hip_backend_create(device, &h);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        auto b = std::shared_ptr<HipInferenceBackend>(new HipInferenceBackend());
        b->handle_ = h;
        return b;
    }
    ~HipInferenceBackend() { bitnet_hip_backend_destroy(handle_); }
    Result<Unit> optimize_model(std::shared_ptr<DecoderProjections> model)
    {
        int rc = bitnet_hip_backend_optimize_model(handle_, model ? model->handle() : nullptr);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        model_ = std::move(model);
        return Unit{};
    }
    // execute_batch(&[Tensor]) -> Vec<Tensor>: every input [rows, hidden]
    Result<std::vector<DeviceTensor>> execute_batch(const std::vector<DeviceTensor> &inputs, hipStream_t stream = nullptr) const
    {
        std::vector<DeviceTensor> outs;
        std::vector<const float *> in_ptrs;
        std::vector<float *> out_ptrs;
        std::vector<size_t> rows;
        for (const DeviceTensor &t : inputs) {
            if (model_ && (t.dims().size() != 2 || t.dims()[1] != model_->hidden))
                return BitLinearError{BitLinearError::ShapeMismatch, "execute_batch input", {t.dims().empty() ? 1 : t.dims()[0], model_->hidden}, t.dims()};
            auto o = DeviceTensor::zeros(t.dims());
            if (o.is_err()) return o.unwrap_err();
            outs.push_back(o.unwrap());
            in_ptrs.push_back(t.data());
            out_ptrs.push_back(outs.back().data());
            rows.push_back(t.dims().empty() ? 0 : t.dims()[0]);
        }
        int rc = bitnet_hip_backend_execute_batch(handle_, in_ptrs.data(), rows.data(), inputs.size(), out_ptrs.data(), stream);
        if (rc != BITNET_HIP_OK) return last_error(rc);
        return outs;
    }
    size_t get_memory_usage() const { return bitnet_hip_backend_get_memory_usage(handle_); }
    BackendCapabilities capabilities() const
    {
        BackendCapabilities c;
        int sb = 0, ss = 0;
        size_t ml = 0;
        (void)bitnet_hip_backend_capabilities(handle_, &sb, &ss, &c.max_batch_size, &ml, &c.device);
        c.supports_batching = sb != 0; c.supports_streaming = ss != 0;
        if (ml) c.memory_limit = ml;
        return c;
    }

private:
    HipInferenceBackend() = default;
    bitnet_hip_backend *handle_ = nullptr;
    std::shared_ptr<DecoderProjections> model_;
};

}  // namespace bitnet
