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
    std::printf(failures ? "host selftest: %d FAILED\n" : "host selftest: all passed\n", failures);
    return failures ? 1 : 0;
}
