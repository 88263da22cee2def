// Self-test of the C++ host mirror on a GPU.  The first three cases restate the reference's own BitLinear
// forward tests (bitnet-quant/src/bitlinear/forward.rs:304-371: basic shape, with bias, shape mismatch);
// the rest check that the different routes through the library agree bit for bit.
#include <cmath>
#include <cstdio>
#include <cstdlib>

#include "bitlinear.hpp"

using namespace bitnet;

static int failures = 0;
#define CHECK(cond)                                                                  \
    do {                                                                             \
        if (!(cond)) { std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond); ++failures; } \
    } while (0)

static std::vector<float> randn(size_t n, unsigned seed, float scale)
{
    std::vector<float> v(n);
    unsigned s = seed * 2654435761u + 12345u;
    for (auto &x : v) {  // sum of 12 uniforms, centred: close enough to normal for a self-test
        float acc = 0.f;
        for (int i = 0; i < 12; ++i) { s = s * 1664525u + 1013904223u; acc += (float)(s >> 8) / 16777216.0f; }
        x = (acc - 6.0f) * scale;
    }
    return v;
}

int main()
{
    if (bitnet_hip_init(0) != BITNET_HIP_OK) { std::printf("init failed: %s\n", bitnet_hip_last_error()); return 2; }

    {  // test_forward_basic
        BitLinearConfig c; c.in_features = 4; c.out_features = 3;
        auto layer = BitLinear::create(c, "test_layer");
        CHECK(layer.is_ok());
        CHECK(layer.unwrap()->update_weights(randn(12, 1, 0.02f), 3, 4).is_ok());
        auto input = DeviceTensor::from_vec(std::vector<float>(8, 1.0f), {2, 4});
        auto out = layer.unwrap()->forward(input.unwrap());
        CHECK(out.is_ok() && out.unwrap().dims() == (std::vector<size_t>{2, 3}));
    }
    {  // test_forward_with_bias
        BitLinearConfig c; c.in_features = 4; c.out_features = 3; c.use_bias = true;
        auto layer = BitLinear::create(c, "test_layer_bias");
        CHECK(layer.unwrap()->update_weights(randn(12, 2, 0.02f), 3, 4).is_ok());
        auto input = DeviceTensor::from_vec(std::vector<float>(8, 1.0f), {2, 4});
        auto out0 = layer.unwrap()->forward(input.unwrap());
        CHECK(layer.unwrap()->update_bias({1.0f, 2.0f, 3.0f}).is_ok());
        auto out1 = layer.unwrap()->forward(input.unwrap());
        CHECK(out1.is_ok() && out1.unwrap().dims() == (std::vector<size_t>{2, 3}));
        auto h0 = out0.unwrap().to_vec(), h1 = out1.unwrap().to_vec();
        for (int i = 0; i < 6; ++i) CHECK(h1[i] == h0[i] + (float)(i % 3 + 1));
    }
    {  // test_forward_shape_mismatch
        BitLinearConfig c; c.in_features = 4; c.out_features = 3;
        auto layer = BitLinear::create(c, "test_layer_shape");
        CHECK(layer.unwrap()->update_weights(randn(12, 3, 0.02f), 3, 4).is_ok());
        auto input = DeviceTensor::from_vec(std::vector<float>(10, 1.0f), {2, 5});
        auto out = layer.unwrap()->forward(input.unwrap());
        CHECK(out.is_err() && out.unwrap_err().kind == BitLinearError::ShapeMismatch);
        CHECK(out.unwrap_err().expected == (std::vector<size_t>{2, 4}) && out.unwrap_err().actual == (std::vector<size_t>{2, 5}));
        CHECK(layer.unwrap()->update_bias({1.f, 2.f, 3.f}).is_err());  // "Bias is not enabled for this layer"
        CHECK(layer.unwrap()->update_weights(randn(12, 3, 0.02f), 4, 3).is_err());
        auto noinit = BitLinear::create(c, "no_weights");
        auto ok_in = DeviceTensor::from_vec(std::vector<float>(8, 1.0f), {2, 4});
        auto r = noinit.unwrap()->forward(ok_in.unwrap());
        CHECK(r.is_err() && r.unwrap_err().kind == BitLinearError::NotInitialized);
    }
    {  // forward == TernaryProcessor::ternary_matmul, at decode and prefill token counts
        const size_t k = 2560, n = 640;
        BitLinearConfig c; c.in_features = k; c.out_features = n;
        auto layer = BitLinear::create(c, "tp");
        CHECK(layer.unwrap()->update_weights(randn(n * k, 4, 0.02f), n, k).is_ok());
        for (size_t m : {size_t(1), size_t(5), size_t(200)}) {
            auto x = DeviceTensor::from_vec(randn(m * k, 5 + (unsigned)m, 1.0f), {m, k});
            auto a = layer.unwrap()->forward(x.unwrap());
            auto b = DeviceTensor::zeros({m, n});
            TernaryProcessor tp;
            CHECK(tp.ternary_matmul(*layer.unwrap(), x.unwrap(), b.unwrap()).is_ok());
            CHECK(a.unwrap().to_vec() == b.unwrap().to_vec());
            auto x3 = DeviceTensor::from_vec(x.unwrap().to_vec(), {1, m, k});  // rank 3 flattens to the same rows
            auto a3 = layer.unwrap()->forward(x3.unwrap());
            CHECK(a3.is_ok() && a3.unwrap().dims() == (std::vector<size_t>{1, m, n}) && a3.unwrap().to_vec() == a.unwrap().to_vec());
        }
    }
    {  // FeedForwardNetwork == down(up * relu(gate)^2) composed by hand
        const size_t hidden = 256, ffn = 512, m = 3;
        BitLinearConfig cu; cu.in_features = hidden; cu.out_features = ffn;
        BitLinearConfig cd; cd.in_features = ffn; cd.out_features = hidden;
        FeedForwardNetwork net;
        net.up_proj = BitLinear::create(cu, "up").unwrap();
        net.gate_proj = BitLinear::create(cu, "gate").unwrap();
        net.down_proj = BitLinear::create(cd, "down").unwrap();
        net.up_proj->update_weights(randn(ffn * hidden, 7, 0.02f), ffn, hidden);
        net.gate_proj->update_weights(randn(ffn * hidden, 8, 0.02f), ffn, hidden);
        net.down_proj->update_weights(randn(ffn * hidden, 9, 0.02f), hidden, ffn);
        auto x = DeviceTensor::from_vec(randn(m * hidden, 10, 1.0f), {m, hidden});
        auto y = net.forward(x.unwrap());
        CHECK(y.is_ok());
        auto up = net.up_proj->forward(x.unwrap()).unwrap().to_vec();
        auto gate = net.gate_proj->forward(x.unwrap()).unwrap().to_vec();
        std::vector<float> h(m * ffn);
        for (size_t i = 0; i < h.size(); ++i) {  // ReLU^2 then gating, transformer_layers.rs:307-316,613-618
            volatile float r = gate[i] > 0.f ? gate[i] : 0.f;
            volatile float sq = r * r;
            h[i] = up[i] * sq;
        }
        auto ht = DeviceTensor::from_vec(h, {m, ffn});
        auto y2 = net.down_proj->forward(ht.unwrap());
        CHECK(y.unwrap().to_vec() == y2.unwrap().to_vec());
    }
    {  // absmax_quantize_activations: the reference's vectors (activations.rs:815-865)
        auto x = DeviceTensor::from_vec({100.0f, -50.0f, 25.0f, -75.0f}, {4});
        auto q8 = absmax_quantize_activations(x.unwrap(), QuantizationPrecision::EightBit);
        CHECK(q8.is_ok() && q8.unwrap().scales == 100.0f / 127.0f && q8.unwrap().effective_bit_width() == 8.0f);
        int8_t h[4];
        (void)hipMemcpy(h, q8.unwrap().values.get(), 4, hipMemcpyDeviceToHost);
        CHECK(h[0] == 127 && h[1] == -64 && h[2] == 32 && h[3] == -95);
        auto y = DeviceTensor::from_vec({4.0f, -2.0f, 1.0f, -3.0f}, {4});
        auto qt = absmax_quantize_activations(y.unwrap());
        CHECK(qt.is_ok() && qt.unwrap().stats.scale_factor == 4.0f && qt.unwrap().stats.elements_count == 4);
        (void)hipMemcpy(h, qt.unwrap().values.get(), 4, hipMemcpyDeviceToHost);
        CHECK(h[0] == 1 && h[1] == 0 && h[2] == 0 && h[3] == -1);  // |x| / 4 > 0.5 only for 4 and -3
    }
    {  // DynamicActivationQuantizer: the reference's own checks (activation_quantization_correctness_tests.rs:486-590)
        DynamicActivationQuantizer dq;  // default: ternary
        auto x = DeviceTensor::from_vec({0.2f, -1.5f, 3.0f, -0.4f, 2.9f, 0.0f, -3.0f, 1.4f}, {2, 4});
        auto q0 = dq.quantize(x.unwrap());  // no state yet: the tensor's own abs-max
        CHECK(q0.is_ok() && q0.unwrap().stats.scale_factor == 3.0f && q0.unwrap().original_shape == x.unwrap().dims());
        int8_t h[8];
        (void)hipMemcpy(h, q0.unwrap().values.get(), 8, hipMemcpyDeviceToHost);
        CHECK(h[0] == 0 && h[1] == 0 && h[2] == 1 && h[3] == 0 && h[4] == 1 && h[5] == 0 && h[6] == -1 && h[7] == 0);  // |x| / 3 > 0.5
        auto small = DeviceTensor::from_vec({0.01f, -0.02f, 0.015f, 0.005f}, {2, 2});
        auto large = DeviceTensor::from_vec({10.0f, -20.0f, 15.0f, 5.0f}, {2, 2});
        auto qs = dq.quantize_dynamic(small.unwrap());
        auto ql = dq.quantize_dynamic(large.unwrap());
        CHECK(qs.is_ok() && ql.is_ok() && qs.unwrap().stats.scale_factor == 0.02f);
        const float kept = 0.99f * 0.02f, fresh = (1.0f - 0.99f) * 20.0f;
        CHECK(ql.unwrap().stats.scale_factor == kept + fresh && qs.unwrap().stats.scale_factor < ql.unwrap().stats.scale_factor);
        CHECK(dq.scale_history().size() == 2 && dq.needs_calibration());
        dq.reset_dynamic_state();
        auto again = dq.quantize_dynamic(large.unwrap());
        CHECK(again.is_ok() && again.unwrap().stats.scale_factor == 20.0f && dq.get_dynamic_scales() == 20.0f);
        ActivationQuantizationConfig c8; c8.precision = QuantizationPrecision::EightBit;
        DynamicActivationQuantizer d8(c8);
        auto y = DeviceTensor::from_vec({100.0f, -50.0f, 25.0f, -75.0f}, {4});
        auto q8 = d8.quantize_dynamic(y.unwrap());
        CHECK(q8.is_ok() && q8.unwrap().stats.scale_factor == 100.0f / 127.0f);
        (void)hipMemcpy(h, q8.unwrap().values.get(), 4, hipMemcpyDeviceToHost);
        CHECK(h[0] == 127 && h[1] == -64 && h[2] == 32 && h[3] == -95);
        ActivationQuantizationConfig bad; bad.ema_decay = 1.5f;
        CHECK(bad.validate().is_err() && ActivationQuantizationConfig{}.validate().is_ok());
    }
    {  // BitNetWeightQuantizer: the packed bytes loaded into a layer give the forward the quantiser's codes imply
        const size_t n = 48, k = 256;
        auto w = DeviceTensor::from_vec(randn(n * k, 21, 1.0f), {n, k});
        BitNetWeightQuantizer quantizer;  // normalise, clip at 3.0, MeanThreshold
        auto qw = quantizer.quantize(w.unwrap());
        CHECK(qw.is_ok() && qw.unwrap().scales > 0.0f && qw.unwrap().values.size() == n * k);
        bool ternary = true, packs = true;
        for (size_t i = 0; i < n * k; ++i) {
            const int v = qw.unwrap().values[i];
            ternary = ternary && v >= -1 && v <= 1;
            packs = packs && ((qw.unwrap().packed[i / 4] >> (2 * (i % 4))) & 3) == v + 1;
        }
        CHECK(ternary && packs);
        BitLinearConfig c; c.in_features = k; c.out_features = n; c.ternary_method = BITNET_HIP_TERNARY_REF_MEAN_THRESHOLD; c.threshold_factor = 0.0f;
        auto layer = BitLinear::create(c, "refq");
        CHECK(layer.unwrap()->update_weights(w.unwrap().to_vec(), n, k).is_ok());
        float ws = 0.f;
        std::vector<uint8_t> held(n * k / 4);
        CHECK(bitnet_hip_bitlinear_get_quantized(layer.unwrap()->handle(), &ws, held.data(), held.size()) == BITNET_HIP_OK);
        CHECK(ws == qw.unwrap().scales && held == qw.unwrap().packed);
    }
    {  // HipInferenceBackend::execute_batch == one decode per input
        auto dec = DecoderProjections::create(2, 256, 512, 4, 2, 64, 1e-5f, 8);
        CHECK(dec.is_ok());
        const size_t outs[7] = {256, 128, 128, 256, 512, 512, 256}, ins[7] = {256, 256, 256, 256, 256, 256, 512};
        for (size_t l = 0; l < 2; ++l)
            for (int p = 0; p < 7; ++p)
                CHECK(dec.unwrap()->update_weights(l, p, randn(outs[p] * ins[p], 30 + (unsigned)(7 * l + p), 0.02f), outs[p], ins[p]).is_ok());
        auto backend = HipInferenceBackend::create(0);
        CHECK(backend.is_ok() && backend.unwrap()->get_memory_usage() == 0);
        std::vector<DeviceTensor> batch;
        for (size_t r : {size_t(1), size_t(3), size_t(2), size_t(8)}) batch.push_back(DeviceTensor::from_vec(randn(r * 256, 50 + (unsigned)r, 1.0f), {r, 256}).unwrap());
        auto none = backend.unwrap()->execute_batch(batch);
        CHECK(none.is_err() && none.unwrap_err().kind == BitLinearError::NotInitialized);
        CHECK(backend.unwrap()->optimize_model(dec.unwrap()).is_ok());
        auto caps = backend.unwrap()->capabilities();
        CHECK(caps.supports_batching && !caps.supports_streaming && caps.max_batch_size == 8 && caps.memory_limit.has_value());
        CHECK(backend.unwrap()->get_memory_usage() > 0);
        auto res = backend.unwrap()->execute_batch(batch);
        CHECK(res.is_ok() && res.unwrap().size() == batch.size());
        for (size_t i = 0; res.is_ok() && i < batch.size(); ++i) {
            auto one = dec.unwrap()->decode(batch[i]);
            CHECK(one.is_ok() && one.unwrap().to_vec() == res.unwrap()[i].to_vec());
        }
    }
    {  // a recorded decode step replays to the bits of the eager step, also after its input has changed
        auto dec = DecoderProjections::create(2, 256, 512, 4, 2, 64, 1e-5f, 4);
        CHECK(dec.is_ok());
        const size_t outs[7] = {256, 128, 128, 256, 512, 512, 256}, ins[7] = {256, 256, 256, 256, 256, 256, 512};
        for (size_t l = 0; l < 2; ++l)
            for (int p = 0; p < 7; ++p)
                CHECK(dec.unwrap()->update_weights(l, p, randn(outs[p] * ins[p], 70 + (unsigned)(7 * l + p), 0.02f), outs[p], ins[p]).is_ok());
        auto x = DeviceTensor::from_vec(randn(3 * 256, 90, 1.0f), {3, 256}).unwrap();
        auto out = DeviceTensor::zeros({3, 256}).unwrap();
        auto graph = dec.unwrap()->record(x, out);
        CHECK(graph.is_ok());
        for (unsigned round = 0; graph.is_ok() && round < 3; ++round) {
            auto fresh = randn(3 * 256, 91 + round, 1.0f);
            (void)hipMemcpy(x.data(), fresh.data(), fresh.size() * sizeof(float), hipMemcpyHostToDevice);
            auto eager = dec.unwrap()->decode(x);
            CHECK(graph.unwrap().replay().is_ok());
            CHECK(eager.is_ok() && eager.unwrap().to_vec() == out.to_vec());
        }
    }
    std::printf(failures ? "host selftest: %d FAILED\n" : "host selftest: all passed\n", failures);
    return failures ? 1 : 0;
}
