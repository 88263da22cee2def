"""Parity of the HIP path (through the C ABI) with the CPU oracle on the same seeded inputs.

Bar: int8 activations, packed bytes and int32 accumulators bit-exact; f32 scales and outputs compared
bit-exact where the oracle and the kernel perform the same IEEE operations, and in any case within
1e-5 relative error (the tolerance the path's specification states)."""
import numpy as np
import pytest
import torch

import bitnet_hip as bh
from helpers import golden_vectors, rel_err, synth_activations, synth_weights
from oracle import oracle as orc

pytestmark = pytest.mark.gpu
G = golden_vectors()
f32 = np.float32
REL_TOL = 1e-5


@pytest.fixture(scope="module", autouse=True)
def _device():
    bh.init(0)
    info = bh.device_info()
    assert info["arch"].startswith("gfx950")
    yield
    torch.cuda.synchronize()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


# ---- P1 ------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("case", G["unpack_2bit"], ids=lambda c: c["source"].split(":")[0].split("/")[-1])
def test_unpack_reference_bytes(case):
    got = host(bh.unpack_ternary_2bit(dev(np.array(case["bytes"], dtype=np.uint8)), case["count"]))
    assert got.tolist() == case["expected"]


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 63, 64, 65, 1000, 10000, 2560 * 640])
def test_pack_unpack_match_oracle(n):
    rng = np.random.default_rng(n)
    w = rng.integers(-1, 2, size=n).astype(np.int8) if n not in (1000, 10000) else (np.arange(n) % 3 - 1).astype(np.int8)
    packed = bh.BitPacked2BitPacker().pack(dev(w))
    assert np.array_equal(host(packed), orc.pack_2bit(w))
    assert np.array_equal(host(bh.BitPacked2BitPacker().unpack(packed, n)), w)


def test_unpack_every_byte_value():
    allb = np.arange(256, dtype=np.uint8)
    assert np.array_equal(host(bh.unpack_ternary_2bit(dev(allb), 1024)), orc.unpack_2bit(allb, 1024))


@pytest.mark.parametrize("n,k", [(16, 256), (17, 257), (5, 7), (33, 100), (640, 2560), (2560, 6912)])
@pytest.mark.parametrize("layout", [bh.LAYOUT_OUT_IN, bh.LAYOUT_IN_OUT])
def test_retile_is_a_bijection(n, k, layout):
    rng = np.random.default_rng(n * 7 + k)
    w = rng.integers(-1, 2, size=(n, k)).astype(np.int8)
    src = w if layout == bh.LAYOUT_OUT_IN else np.ascontiguousarray(w.T)
    tiled = bh.retile_weights(dev(orc.pack_2bit(src)), n, k, layout)
    assert tiled.numel() == bh.tiled_size(n, k)
    back = host(bh.untile_weights(tiled, n, k))
    assert np.array_equal(back, orc.pack_2bit(w))


def test_retile_canonicalises_code_three():
    # code 3 decodes to weight 0 in every reference decoder; the tiled layout stores it as code 1
    n, k = 16, 256
    packed = np.full((n * k // 4,), 0xFF, dtype=np.uint8)
    tiled = bh.retile_weights(dev(packed), n, k)
    assert np.all(host(tiled) == 0x55)
    a = dev(np.full((1, k), 77, dtype=np.int8))
    acc, _ = bh.matmul_w2a8(tiled, a, n, want_out=False)
    assert not host(acc).any()


# ---- W1 ------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("n,k", [(4, 4), (3, 5), (64, 128), (640, 2560), (2560, 2560)])
def test_quantize_weights_absmean_bit_exact(n, k):
    rng = np.random.default_rng(n + k)
    w = synth_weights(rng, n, k)
    packed, w_scale, q = bh.quantize_weights(dev(w), want_i8=True)
    q_ref, s_ref = orc.quantize_weights_absmean(w)
    assert host(w_scale)[0] == s_ref
    assert np.array_equal(host(q), q_ref)
    assert np.array_equal(host(packed), orc.pack_2bit(q_ref))


def test_quantize_weights_reference_vectors():
    c = G["quantize_batch"]
    w = np.array([c["input"]], dtype=f32)
    # threshold form with the reference's factor 0.5 on its own vector (mean|w| of this vector is 1.2167)
    _, s, q = bh.quantize_weights(dev(w), method=bh.TERNARY_MEAN_THRESHOLD, threshold_factor=0.5, want_i8=True)
    assert host(s)[0] == orc.absmean(w)
    assert host(q)[0].tolist() == orc.ternarize_threshold(w, f32(0.5) * orc.absmean(w))[0].tolist()
    for case in G["absmean"]:
        _, s, _ = bh.quantize_weights(dev(np.array([case["input"]], dtype=f32)))
        assert abs(float(host(s)[0]) - case["expected"]) < 1e-6
    # ties and a zero matrix
    w = np.array([[0.5, -0.5, 0.25, 1.5, -7.0, 0.0, 1.0, -1.0]], dtype=f32)
    _, s, q = bh.quantize_weights(dev(w), want_i8=True)
    assert np.array_equal(host(q), orc.ternarize_roundclip(w, host(s)[0]))
    _, s, q = bh.quantize_weights(dev(np.zeros((4, 8), dtype=f32)), want_i8=True)
    assert host(s)[0] == 0.0 and not host(q).any()


@pytest.mark.parametrize("method", range(5))
@pytest.mark.parametrize("normalize,t,custom", [(True, 3.0, None), (False, 0.0, None), (True, 0.0, 0.45), (False, 2.0, None)])
def test_reference_weight_pipeline_bit_exact(method, normalize, t, custom):
    """BitNetWeightQuantizer::quantize with each TernaryMethod: ternary values, packed bytes, the scale and all twelve
    f32 scalars of the pipeline equal to the oracle's, bit for bit (stated bar: q exact, scale within 1e-6 relative)."""
    rng = np.random.default_rng(method * 10 + int(normalize) + int(t))
    for n, k in ((48, 200), (5, 7), (640, 2560)):
        w = (0.3 + 1.7 * rng.standard_normal((n, k))).astype(f32)
        w[rng.random(w.shape) < 0.01] *= f32(6.0)
        cfg = bh.WeightQuantizationConfig(normalize_weights=normalize, outlier_threshold=t, ternary_method=method,
                                          custom_threshold_factor=custom)
        got = bh.BitNetWeightQuantizer(cfg).quantize(dev(w))
        q_ref, s_ref, _, st_ref = orc.quantize_weights_reference(w, method=method, normalize=normalize, outlier_threshold=t,
                                                                 custom_factor=custom, want_details=True)
        assert np.array_equal(host(got.values), q_ref)
        assert np.array_equal(host(got.packed), orc.pack_2bit(q_ref))
        assert abs(float(host(got.scales)[0]) - float(s_ref)) <= 1e-6 * abs(float(s_ref))
        assert host(got.scales)[0] == s_ref
        for name, v in st_ref.items():
            assert f32(got.stats[name]) == v, (name, got.stats[name], v)


def test_reference_weight_pipeline_through_the_layer():
    """BitLinear with the reference's default quantiser (MeanThreshold, normalise, clip 3.0: layer.rs:53-63): the layer then
    holds the oracle's codes and scale, and forward follows from them."""
    rng = np.random.default_rng(21)
    n, k = 96, 512
    w = synth_weights(rng, n, k)
    for method, factor in ((bh.TERNARY_REF_MEAN_THRESHOLD, 0.0), (bh.TERNARY_REF_OPTIMAL_THRESHOLD, 0.0),
                           (bh.TERNARY_REF_ADAPTIVE_THRESHOLD, 0.0), (bh.TERNARY_REF_DETSTE, 0.9)):
        layer = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n, ternary_method=method, threshold_factor=factor), "ref")
        layer.update_weights(dev(w))
        q_ref, s_ref = orc.quantize_weights_reference(w, method=method - bh.TERNARY_REF_MEAN_THRESHOLD,
                                                      custom_factor=factor or None)
        packed, ws = layer.get_quantized_weights()
        assert ws == s_ref and np.array_equal(packed.numpy(), orc.pack_2bit(q_ref))
        x = synth_activations(rng, 3, k)
        ref = orc.bitlinear_forward(x, orc.pack_2bit(q_ref), n, float(s_ref))[0]
        assert np.array_equal(host(layer.forward(dev(x))), ref)
    with pytest.raises(bh.BitLinearError) as ei:
        bh.BitNetWeightQuantizer(bh.WeightQuantizationConfig(custom_threshold_factor=2.5))
    assert ei.value.kind == "InvalidConfig"
    with pytest.raises(bh.BitLinearError):
        bh.BitNetWeightQuantizer().quantize(torch.ones(4, device="cuda"))
    # an all-zero tensor: no non-zero code, scale 1.0 (compute_ternary_scale, weights.rs:554-556)
    z = bh.BitNetWeightQuantizer(bh.WeightQuantizationConfig(normalize_weights=False, outlier_threshold=0.0)).quantize(
        torch.zeros(4, 8, device="cuda"))
    assert not host(z.values).any() and host(z.scales)[0] == 1.0


# ---- A2 ------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("precision", [bh.QuantizationPrecision.OneFiveFiveBit, bh.QuantizationPrecision.EightBit])
@pytest.mark.parametrize("shape", [(4,), (32, 128), (3, 5, 7), (300, 4096 + 17), (1, 1)])
def test_absmax_quantize_activations_bit_exact(precision, shape):
    """absmax_quantize_activations (one scale per tensor): values, scale, error, min and max equal to the oracle's."""
    rng = np.random.default_rng(len(shape) * 10 + precision)
    x = (rng.standard_normal(shape) * 3).astype(f32)
    if x.size >= 4:
        x.flat[:4] = [100.0, -50.0, 25.0, -75.0]  # the reference's vector (activations.rs:815-840)
    got = bh.absmax_quantize_activations(dev(x), precision)
    q_ref, st = orc.absmax_quantize_activations(x, precision)
    assert np.array_equal(host(got.values), q_ref) and got.original_shape == shape
    assert f32(got.stats["scale_factor"]) == st["scale"] and host(got.scales)[0] == st["scale"]
    assert f32(got.stats["quantization_error"]) == st["mse"]
    assert f32(got.stats["min_value"]) == st["min"] and f32(got.stats["max_value"]) == st["max"]
    assert got.stats["elements_count"] == x.size and got.stats["compression_ratio"] > 1.0 and got.zero_points is None
    assert got.effective_bit_width() == (1.58 if precision == 0 else 8.0)
    deq = bh.ActivationQuantizer(precision).dequantize(got)
    assert tuple(deq.shape) == shape
    zeros = bh.absmax_quantize_activations(torch.zeros(2, 2, device="cuda"), precision)
    assert not host(zeros.values).any() and zeros.stats["scale_factor"] == 1.0
    with pytest.raises(bh.BitLinearError) as ei:
        bh.absmax_quantize_activations(dev(x), 7)
    assert ei.value.kind == "Unsupported"


@pytest.mark.parametrize("precision", [bh.QuantizationPrecision.OneFiveFiveBit, bh.QuantizationPrecision.EightBit])
@pytest.mark.parametrize("shape", [(5,), (32, 128), (3, 5, 7), (300, 4096 + 17), (1, 1)])
def test_dynamic_activation_quantizer_matches_the_oracle(precision, shape):
    """DynamicActivationQuantizer (activations.rs:203-454) on the device: abs-max and the quantiser with a given scale
    bit-equal to the oracle (signed and the reference's literal u8 form), and the stateful object step by step against
    the oracle driven by the same state machine: the moving average after every quantize_dynamic, the values it yields,
    reset, calibration, attention, and the reference's own assertions (ternary values only for the default precision,
    the scale grows with the magnitude, a reset quantizer scales by the tensor's own abs-max)."""
    rng = np.random.default_rng(len(shape) * 7 + precision)
    x = (rng.standard_normal(shape) * 3).astype(f32)
    assert f32(bh.abs_max(dev(x))) == orc.abs_max(x)
    for scale in (float(orc.abs_max(x)) / 127.0, 0.037, 1.0, 2.5):
        for u8 in (False, True):
            got = bh.quantize_activations_scaled(dev(x), precision, scale, reference_u8=u8)
            want = orc.quantize_activations_scaled(x, precision, scale, reference_u8=u8)
            assert np.array_equal(host(got).view(np.int8), want)
    cfg = bh.ActivationQuantizationConfig(precision=precision, ema_decay=0.8, calibration_warmup=2, moving_average_window=4)
    quant = bh.create_activation_quantizer(cfg)
    model = bh.DynamicScaleState(cfg)
    first = quant.quantize(dev(x))  # no state yet: the tensor's own abs-max is the scale
    assert f32(first.stats["scale_factor"]) == orc.abs_max(x)
    assert np.array_equal(host(first.values), orc.quantize_activations_scaled(x, precision, float(orc.abs_max(x))))
    scales = []
    for step, mag in enumerate((0.1, 1.0, 10.0, 3.0, 0.5)):
        xs = (x * f32(mag)).astype(f32)
        out = quant.quantize_dynamic(dev(xs))
        model.step_count += 1
        ema = model.update(orc.abs_max(xs))
        assert f32(out.stats["scale_factor"]) == ema == quant.state.ema_scale
        assert np.array_equal(host(out.values), orc.quantize_activations_scaled(xs, precision, float(ema)))
        assert out.original_shape == shape and out.stats["elements_count"] == x.size
        assert quant.needs_calibration() == model.needs_calibration()
        assert f32(float(quant.get_dynamic_scales())) == ema
        scales.append(float(ema))
        if precision == bh.QuantizationPrecision.OneFiveFiveBit:
            assert set(np.unique(host(out.values)).tolist()) <= {-1, 0, 1}
    assert scales[0] < scales[1] < scales[2]  # the scale adapts to the magnitude (test_..._dynamic_scaling)
    deq = quant.dequantize(out)
    assert tuple(deq.shape) == shape
    quant.reset_dynamic_state()
    again = quant.quantize_dynamic(dev(x))
    own = orc.abs_max(x) / f32(127.0) if precision == bh.QuantizationPrecision.EightBit else orc.abs_max(x)
    assert f32(again.stats["scale_factor"]) == own and again.stats["scale_factor"] > 0
    quant.calibrate([dev((x * f32(m)).astype(f32)) for m in (1.0, 4.0, 2.0)])
    assert f32(quant.state.ema_scale) == orc.abs_max((x * f32(4.0)).astype(f32)) and quant.state.calibrated
    att = quant.quantize_attention(dev(x), 64)
    assert att.sequence_length == 64
    off = bh.DynamicActivationQuantizer(bh.ActivationQuantizationConfig(quantize_attention=False))
    with pytest.raises(bh.BitLinearError):
        off.quantize_attention(dev(x), 8)
    with pytest.raises(bh.BitLinearError):
        quant.validate_input(torch.zeros((), device="cuda"))
    with pytest.raises(bh.BitLinearError):
        quant.validate_input(torch.zeros((4, 4), dtype=torch.uint8, device="cuda"))


# ---- R1 + A1 -------------------------------------------------------------------------------------------

@pytest.mark.parametrize("m,k", [(1, 2560), (4, 2560), (3, 6912), (2, 1024), (5, 4096), (2, 8192), (2, 12000),
                                 (3, 7), (2, 257), (1, 4), (9, 64), (33, 2560), (40, 6912), (35, 1028), (34, 20000),
                                 (2, 20000), (3, 16384), (33, 5)])
@pytest.mark.parametrize("norm", [False, True])
def test_activation_quant_bit_exact(m, k, norm):
    rng = np.random.default_rng(m * 100003 + k)
    x = synth_activations(rng, m, k, outliers=True)
    g = rng.standard_normal(k, dtype=f32) if norm else None
    q, s, asum, y = bh.quantize_activations_i8(dev(x), dev(g) if norm else None, eps=1e-5, want_sum=True, want_y=norm)
    q_ref, s_ref, rs_ref = orc.rmsnorm_quantize_i8(x, g, 1e-5, orc.SUM_BLOCK256)
    assert np.array_equal(host(s), s_ref)
    assert np.array_equal(host(q), q_ref)
    assert np.array_equal(host(asum), rs_ref)
    if norm:
        assert np.array_equal(host(y), orc.rmsnorm(x, g, 1e-5, orc.SUM_BLOCK256))


@pytest.mark.parametrize("m,k", [(3, 2560), (3, 300), (40, 2560), (40, 6912), (5, 12000), (2, 20000), (40, 301), (64, 8192),
                                 (300, 2560), (16, 6912)])
def test_activation_quant_sequential_order_bit_exact(m, k):
    """The reference's literal summation order (one running f32 sum) is available and also bit-exact: the kernels with
    16 and 4 wavefronts per row (the row's squares staged in LDS, every lane running the chain), unaligned rows, rows
    too long for the staging (the chain then reads global memory) and the wavefront-per-row kernel."""
    rng = np.random.default_rng(k + m)
    x = synth_activations(rng, m, k)
    g = rng.standard_normal(k, dtype=f32)
    q, s, _, y = bh.quantize_activations_i8(dev(x), dev(g), eps=1e-6, sum_order=bh.SUM_SEQUENTIAL, want_y=True)
    q_ref, s_ref, _ = orc.rmsnorm_quantize_i8(x, g, 1e-6, orc.SUM_SEQUENTIAL)
    assert np.array_equal(host(y), orc.rmsnorm(x, g, 1e-6, orc.SUM_SEQUENTIAL))
    assert np.array_equal(host(s), s_ref) and np.array_equal(host(q), q_ref)


def test_activation_quant_edge_rows():
    x = np.zeros((4, 256), dtype=f32)
    x[1, :9] = [127.0, 0.5, -0.5, 1.5, 2.5, -2.5, 0.49999997, -126.5, 126.4999]
    x[2, 3] = np.nan
    x[2, 4] = 2.0
    x[3, :] = 1e-30
    q, s, asum, _ = bh.quantize_activations_i8(dev(x), want_sum=True)
    q_ref, s_ref, rs_ref = orc.quantize_activations_i8(x)
    assert np.array_equal(host(q), q_ref) and np.array_equal(host(s), s_ref) and np.array_equal(host(asum), rs_ref)
    assert host(s)[0] == 1.0 and not host(q)[0].any()
    assert host(q)[1, :9].tolist() == [127, 1, -1, 2, 3, -3, 0, -127, 126]
    # the reference's own property test (ternary_operations.rs:445-461)
    xin = np.array([G["activation_quant_properties"]["input"]], dtype=f32)
    q, s, _, _ = bh.quantize_activations_i8(dev(xin))
    fq = host(q)[0].astype(f32) / host(s)[0]
    assert fq[1] > fq[0] and fq[2] < 0 and fq[3] < fq[2]
    c = G["absmax_8bit_scale"]
    _, s, _, _ = bh.quantize_activations_i8(dev(np.array([c["input"]], dtype=f32)))
    assert host(s)[0] == f32(127.0) / f32(c["absmax"])


def test_activation_quant_fused_inputs():
    rng = np.random.default_rng(21)
    m, ffn = 3, 6912
    gate, up = synth_activations(rng, m, ffn), synth_activations(rng, m, ffn)
    q, s, _, _ = bh.quantize_activations_i8(dev(gate), x2=dev(up), input_mode=bh.INPUT_RELU2_MUL)
    q_ref, s_ref, _ = orc.quantize_activations_i8(orc.relu2_mul(gate, up))
    assert np.array_equal(host(q), q_ref) and np.array_equal(host(s), s_ref)
    v = synth_activations(rng, m, 640)
    q, s, _, _ = bh.quantize_activations_i8(dev(v), input_mode=bh.INPUT_GQA_BROADCAST, gqa_group=4, head_dim=128)
    q_ref, s_ref, _ = orc.quantize_activations_i8(orc.gqa_broadcast_v(v, 20, 5, 128))
    assert np.array_equal(host(q), q_ref) and np.array_equal(host(s), s_ref)


def test_activation_quant_prefill_size_properties():
    """Full prefill size (2048 x 2560): size-independent properties plus a sampled comparison."""
    rng = np.random.default_rng(22)
    x = synth_activations(rng, 2048, 2560, outliers=True)
    g = np.ones(2560, dtype=f32)
    xd = dev(x)
    q, s, asum, _ = bh.quantize_activations_i8(xd, dev(g), want_sum=True)
    qh = host(q)
    assert np.all(np.abs(qh.astype(np.int32)).max(axis=1) == 127)
    assert np.array_equal(host(asum), qh.astype(np.int64).sum(axis=1))
    qn, sn, _, _ = bh.quantize_activations_i8(-xd, dev(g))
    assert np.array_equal(host(qn), -qh) and np.array_equal(host(sn), host(s))
    rows = rng.choice(2048, size=64, replace=False)
    q_ref, s_ref, _ = orc.rmsnorm_quantize_i8(x[rows], g, 1e-5)
    assert np.array_equal(qh[rows], q_ref) and np.array_equal(host(s)[rows], s_ref)


# ---- G1: reference contract on the reference's byte layout ---------------------------------------------------

@pytest.mark.parametrize("case", G["gemv"], ids=lambda c: f'{c["m"]}x{c["k"]}')
def test_w2a8_gemv_reference_vectors(case):
    w = np.array(case["a"], dtype=np.int8).reshape(case["m"], case["k"])
    out = torch.zeros(case["m"], dtype=torch.int32, device="cuda")
    bh.W2A8Backend().w2a8_gemv(dev(orc.pack_2bit(w)), dev(np.array(case["x"], dtype=np.int8)), out, case["m"], case["k"])
    assert (host(out) * case["scale"]).tolist() == case["expected"]


@pytest.mark.parametrize("n,k", [(1, 1), (3, 5), (7, 33), (64, 256), (100, 1000), (640, 2560), (2560, 6912)])
def test_w2a8_gemv_rowmajor_bit_exact(n, k):
    rng = np.random.default_rng(n * 31 + k)
    w = rng.integers(-1, 2, size=(n, k)).astype(np.int8)
    a = rng.integers(-128, 128, size=k).astype(np.int8)
    packed = orc.pack_2bit(w)
    out = torch.zeros(n, dtype=torch.int32, device="cuda")
    bh.W2A8Backend().w2a8_gemv(dev(packed), dev(a), out, n, k)
    assert np.array_equal(host(out), orc.gemv_w2a8(packed, a, n))


def test_w2a8_gemv_shape_errors():
    b = bh.W2A8Backend()
    w, a, o = dev(np.zeros(32, np.uint8)), dev(np.zeros(16, np.int8)), torch.zeros(8, dtype=torch.int32, device="cuda")
    with pytest.raises(bh.BitLinearError) as ei:
        b.w2a8_gemv(w[:31].contiguous(), a, o, 8, 16)
    assert ei.value.kind == "ShapeMismatch" and ei.value.expected == [32] and ei.value.actual == [31]
    with pytest.raises(bh.BitLinearError):
        b.w2a8_gemv(w, a[:15].contiguous(), o, 8, 16)
    with pytest.raises(bh.BitLinearError):
        b.w2a8_gemv(w, a, o[:7].contiguous(), 8, 16)


# ---- G1 / G2 / E1 on the tiled layout ---------------------------------------------------------------------

SHAPES = [(2560, 2560), (640, 2560), (6912, 2560), (2560, 6912)]


def make_problem(rng, m, n, k, outliers=False, full_range=False):
    w = synth_weights(rng, n, k)
    qw, ws = orc.quantize_weights_absmean(w)
    packed = orc.pack_2bit(qw)
    if full_range:
        a = rng.integers(-128, 128, size=(m, k)).astype(np.int8)
        a_scale = (rng.random(m, dtype=f32) * 50 + 1).astype(f32)
    else:
        a, a_scale, _ = orc.quantize_activations_i8(synth_activations(rng, m, k, outliers))
    return packed, ws, a, a_scale


@pytest.mark.parametrize("n,k", SHAPES)
@pytest.mark.parametrize("m", [1, 2, 3, 4, 8])
def test_decode_gemv_bit_exact(m, n, k):
    rng = np.random.default_rng(m * 1000 + n + k)
    packed, ws, a, a_scale = make_problem(rng, m, n, k, outliers=True)
    tiled = bh.retile_weights(dev(packed), n, k)
    acc, out = bh.matmul_w2a8(tiled, dev(a), n, dev(np.array([ws], dtype=f32)), dev(a_scale))
    acc_ref = orc.gemm_w2a8(packed, a, n)
    assert np.array_equal(host(acc), acc_ref)
    out_ref = orc.epilogue(acc_ref, ws, a_scale)
    assert np.array_equal(host(out), out_ref)
    assert rel_err(host(out), out_ref) <= REL_TOL


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (1, 5, 7), (2, 17, 257), (3, 33, 100), (1, 16, 255), (4, 15, 512),
                                   (1, 48, 16384), (8, 31, 3000), (17, 40, 512), (33, 100, 300), (48, 33, 768),
                                   (65, 50, 512), (95, 170, 1024), (20, 7000, 256)])
def test_decode_gemv_ragged_shapes(m, n, k):
    """Token counts 1, 2..16, 17..32, 33..64 and 65..95 take different variants of the decode GEMV (dot-product
    chain, MFMA with 1, 2 or 4 groups of 16 token rows, two launches); k a multiple of 256 or not selects the
    unconditional-load variant or the bounds-checked one."""
    rng = np.random.default_rng(m + 10 * n + 100 * k)
    packed, ws, a, a_scale = make_problem(rng, m, n, k, full_range=True)
    tiled = bh.retile_weights(dev(packed), n, k)
    bias = rng.standard_normal(n, dtype=f32)
    res = rng.standard_normal((m, n), dtype=f32)
    acc, out = bh.matmul_w2a8(tiled, dev(a), n, dev(np.array([ws], dtype=f32)), dev(a_scale), dev(bias), dev(res))
    acc_ref = orc.gemm_w2a8(packed, a, n)
    assert np.array_equal(host(acc), acc_ref)
    assert np.array_equal(host(out), orc.epilogue(acc_ref, ws, a_scale, bias, res))


@pytest.mark.parametrize("m,n,k", [(5, 40, 256), (16, 33, 3072), (8, 100, 3328), (8, 17, 8192), (5, 6500, 512),
                                   (16, 13000, 256), (7, 2560, 6912), (16, 6912, 2560), (9, 48, 3328), (4, 48, 2560)])
def test_decode_gemv_lds_staged_activations(m, n, k):
    """5..16 tokens with k a multiple of 256 whose rows fit LDS take the MFMA GEMV that copies the activations into
    LDS first: k <= 3072 (one chunk column per thread) or k <= 8192 with at most 8 tokens (two); n selects 1, 2 or 4
    row blocks per workgroup (400 / 800 row blocks), ragged n the partial last block.  The last two cases fall just
    outside (9 tokens at k > 3072, 4 tokens) and take the gathering variant."""
    rng = np.random.default_rng(m + 10 * n + 100 * k)
    packed, ws, a, a_scale = make_problem(rng, m, n, k, full_range=True)
    tiled = bh.retile_weights(dev(packed), n, k)
    bias = rng.standard_normal(n, dtype=f32)
    res = rng.standard_normal((m, n), dtype=f32)
    acc, out = bh.matmul_w2a8(tiled, dev(a), n, dev(np.array([ws], dtype=f32)), dev(a_scale), dev(bias), dev(res))
    acc_ref = orc.gemm_w2a8(packed, a, n)
    assert np.array_equal(host(acc), acc_ref)
    assert np.array_equal(host(out), orc.epilogue(acc_ref, ws, a_scale, bias, res))
    acc2, out2 = bh.matmul_w2a8(tiled, dev(a), n, dev(np.array([ws], dtype=f32)), dev(a_scale))
    assert np.array_equal(host(acc2), acc_ref)
    assert np.array_equal(host(out2), orc.epilogue(acc_ref, ws, a_scale))


def test_decode_gemv_extremes_and_identities():
    k, n = 6912, 32
    tiled_neg = bh.retile_weights(dev(orc.pack_2bit(-np.ones((n, k), np.int8))), n, k)
    acc, _ = bh.matmul_w2a8(tiled_neg, dev(np.full((1, k), -128, np.int8)), n, want_out=False)
    assert np.all(host(acc) == 128 * k)
    tiled_pos = bh.retile_weights(dev(orc.pack_2bit(np.ones((n, k), np.int8))), n, k)
    rng = np.random.default_rng(5)
    a = rng.integers(-128, 128, size=(2, k)).astype(np.int8)
    acc, _ = bh.matmul_w2a8(tiled_pos, dev(a), n, want_out=False)
    assert np.array_equal(host(acc), np.repeat(a.astype(np.int64).sum(1)[:, None], n, axis=1))
    # linearity in the activations: acc(a1 + a2) = acc(a1) + acc(a2) while a1 + a2 stays in int8
    w = rng.integers(-1, 2, size=(n, k)).astype(np.int8)
    tiled = bh.retile_weights(dev(orc.pack_2bit(w)), n, k)
    a1 = rng.integers(-60, 60, size=(1, k)).astype(np.int8)
    a2 = rng.integers(-60, 60, size=(1, k)).astype(np.int8)
    r1, _ = bh.matmul_w2a8(tiled, dev(a1), n, want_out=False)
    r2, _ = bh.matmul_w2a8(tiled, dev(a2), n, want_out=False)
    r12, _ = bh.matmul_w2a8(tiled, dev((a1 + a2).astype(np.int8)), n, want_out=False)
    assert np.array_equal(host(r12), host(r1) + host(r2))


@pytest.mark.parametrize("m", [16, 24, 64])
@pytest.mark.parametrize("n,k", [(6912, 2560), (2560, 6912)])
def test_batched_decode_sweep_bit_exact(m, n, k):
    rng = np.random.default_rng(m + n)
    packed, ws, a, a_scale = make_problem(rng, m, n, k, outliers=True)
    tiled = bh.retile_weights(dev(packed), n, k)
    acc, out = bh.matmul_w2a8(tiled, dev(a), n, dev(np.array([ws], dtype=f32)), dev(a_scale))
    acc_ref = orc.gemm_w2a8(packed, a, n)
    assert np.array_equal(host(acc), acc_ref)
    assert np.array_equal(host(out), orc.epilogue(acc_ref, ws, a_scale))


@pytest.mark.parametrize("m", [17, 31, 32, 33, 48, 80, 95])
@pytest.mark.parametrize("n,k", [(33, 256), (650, 2560), (6912, 2560), (2560, 6912), (100, 8192), (4000, 3072), (1000, 3328),
                                 (640, 2564)])
def test_token_group_gemv_bit_exact(m, n, k):
    """17 to 95 tokens: token groups of 16 with their rows in LDS (k a multiple of 256 up to 8192; one, two or four row
    blocks per workgroup; a last token group that is not full; output rows that do not fill a row block), with bias and
    residual; k = 2564 takes the gathering kernel instead."""
    rng = np.random.default_rng(m * 131 + n + k)
    packed, ws, a, a_scale = make_problem(rng, m, n, k, outliers=True)
    tiled = bh.retile_weights(dev(packed), n, k)
    bias = rng.standard_normal(n, dtype=f32)
    res = rng.standard_normal((m, n), dtype=f32)
    acc, out = bh.matmul_w2a8(tiled, dev(a), n, dev(np.array([ws], dtype=f32)), dev(a_scale), bias=dev(bias), residual=dev(res))
    acc_ref = orc.gemm_w2a8(packed, a, n)
    assert np.array_equal(host(acc), acc_ref)
    assert np.array_equal(host(out), orc.epilogue(acc_ref, ws, a_scale, bias, res))
    acc2, _ = bh.matmul_w2a8(tiled, dev(a), n, want_out=False)
    assert np.array_equal(host(acc2), acc_ref)


@pytest.mark.parametrize("m,n,k", [(96, 2560, 6912), (130, 2560, 6912), (256, 2560, 6912), (128, 6912, 2560), (200, 650, 2560),
                                   (256, 4800, 3072), (257, 2560, 6912), (192, 6912, 2560), (500, 2560, 6912), (700, 2577, 6912),
                                   (384, 6912, 2560), (1000, 2560, 2560), (160, 2560, 2560)])
def test_small_prefill_launches_bit_exact(m, n, k):
    """96 to 257 tokens, where the launch is too small for the 128 x 160 GEMM tiles to fill the chip: the token-group GEMV
    while its workgroups fit one round (96 tokens at 6912 -> 2560, 200 tokens at 650 rows), else the GEMM with narrow
    tiles and four stages of loads in flight (64 x 32 or 64 x 64).  Same results whichever runs."""
    rng = np.random.default_rng(m + n + k)
    packed, ws, a, a_scale = make_problem(rng, m, n, k, outliers=True)
    tiled = bh.retile_weights(dev(packed), n, k)
    res = rng.standard_normal((m, n), dtype=f32)
    a_sum = dev(a.astype(np.int32).sum(axis=1).astype(np.int32))
    acc, out = bh.matmul_w2a8(tiled, dev(a), n, dev(np.array([ws], dtype=f32)), dev(a_scale), residual=dev(res), a_sum=a_sum)
    acc_ref = orc.gemm_w2a8(packed, a, n)
    assert np.array_equal(host(acc), acc_ref)
    assert np.array_equal(host(out), orc.epilogue(acc_ref, ws, a_scale, None, res))


@pytest.mark.parametrize("n,k", [(6912, 2560), (2560, 6912)])
@pytest.mark.parametrize("with_sum", [True, False], ids=["lds_direct_kernel", "register_staged_kernel"])
def test_prefill_gemm_full_size(n, k, with_sum):
    """M = 2048 at the two prefill shapes (BASELINE config 4): every one of the 2048 x N accumulators against an f64 BLAS
    product of the unpacked operands (|acc| <= 127 K < 2^24, so every partial sum of the f64 product is an exact
    integer whatever the library's order), sampled rows also against the oracle's own loop, the f32 output of the whole
    matrix against the oracle's epilogue.  Supplying the activation row sums selects the LDS-direct kernel, omitting
    them the register-staged one."""
    m = 2048
    rng = np.random.default_rng(n)
    packed, ws, a, a_scale = make_problem(rng, m, n, k, outliers=False)
    tiled = bh.retile_weights(dev(packed), n, k)
    a_sum = dev(a.astype(np.int32).sum(axis=1).astype(np.int32)) if with_sum else None
    acc, out = bh.matmul_w2a8(tiled, dev(a), n, dev(np.array([ws], dtype=f32)), dev(a_scale), a_sum=a_sum)
    acc_h, out_h = host(acc), host(out)
    rows = np.sort(rng.choice(m, size=48, replace=False))
    acc_ref = orc.gemm_w2a8(packed, a[rows], n)
    assert np.array_equal(acc_h[rows], acc_ref)
    assert np.array_equal(out_h[rows], orc.epilogue(acc_ref, ws, a_scale[rows]))
    w = orc.unpack_2bit(packed, n * k).reshape(n, k)
    full = a.astype(np.float64) @ w.astype(np.float64).T  # exact: integers below 2^53 throughout
    assert np.array_equal(full[rows], acc_ref.astype(np.float64))  # the f64 product agrees with the oracle's loop
    assert np.array_equal(acc_h.astype(np.float64), full), "an accumulator of the full matrix differs"
    assert np.array_equal(out_h, orc.epilogue(acc_h, ws, a_scale))


@pytest.mark.parametrize("m,n,k", [(96, 160, 512), (100, 33, 512), (257, 170, 768), (130, 6912, 2560), (300, 16, 256),
                                   (128, 48, 300), (200, 200, 2561), (1500, 2602, 768), (1600, 2560, 512),
                                   (4100, 5002, 512)])
def test_gemm_ragged_shapes_both_kernels(m, n, k):
    """Token counts, widths and depths that do not fill the MFMA tiles, with bias and residual; with row sums
    (LDS-direct kernels where k allows it: the sizes cover the 64 x 160 tiles, the eight-wavefront 128 x 160
    workgroups (192..256 tiles) and the four-wavefront 128 x 160 workgroups (640 tiles and more)) and
    without."""
    rng = np.random.default_rng(m + 10 * n + 100 * k)
    packed, ws, a, a_scale = make_problem(rng, m, n, k, full_range=True)
    tiled = bh.retile_weights(dev(packed), n, k)
    bias = rng.standard_normal(n, dtype=f32)
    res = rng.standard_normal((m, n), dtype=f32)
    acc_ref = orc.gemm_w2a8(packed, a, n)
    out_ref = orc.epilogue(acc_ref, ws, a_scale, bias, res)
    for a_sum in (dev(a.astype(np.int32).sum(axis=1).astype(np.int32)), None):
        acc, out = bh.matmul_w2a8(tiled, dev(a), n, dev(np.array([ws], dtype=f32)), dev(a_scale), dev(bias), dev(res),
                                  a_sum=a_sum)
        assert np.array_equal(host(acc), acc_ref)
        assert np.array_equal(host(out), out_ref)


@pytest.mark.parametrize("m,n,k", [(100, 172, 512), (257, 2560, 768), (1600, 2564, 512), (1990, 6900, 768),
                                   (2048, 6912, 512), (1990, 6902, 512), (4100, 5000, 512)])
@pytest.mark.parametrize("extras", [False, True], ids=["plain", "bias_residual"])
def test_gemm_f32_only_epilogue_ragged(m, n, k, extras):
    """f32 output without the int32 accumulators: the straight-line epilogue of the LDS-direct kernels (64 x 160,
    eight-wavefront 128 x 160 and four-wavefront 128 x 160 workgroups), tiles cut by m and n, n not a multiple of 4 (general epilogue), and one activation scale outside the short division's
    range (whole wavefronts fall back to the plain division)."""
    rng = np.random.default_rng(7 * m + 3 * n + k + int(extras))
    packed, ws, a, a_scale = make_problem(rng, m, n, k, full_range=True)
    a_scale = a_scale.copy()
    a_scale[m // 2] = np.float32(2.0) ** 100  # invariant_divisor_ok fails for this row
    tiled = bh.retile_weights(dev(packed), n, k)
    bias = rng.standard_normal(n, dtype=f32) if extras else None
    res = rng.standard_normal((m, n), dtype=f32) if extras else None
    out_ref = orc.epilogue(orc.gemm_w2a8(packed, a, n), ws, a_scale, bias, res)
    a_sum = dev(a.astype(np.int32).sum(axis=1).astype(np.int32))
    _, out = bh.matmul_w2a8(tiled, dev(a), n, dev(np.array([ws], dtype=f32)), dev(a_scale),
                            dev(bias) if extras else None, dev(res) if extras else None, want_acc=False, a_sum=a_sum)
    assert np.array_equal(host(out), out_ref)


@pytest.mark.parametrize("m", [1, 4, 16, 128])
def test_forward_in_hip_graph_replays_match_eager(m):
    """forward() with caller-supplied output and workspace allocates nothing and records no memset, so a caller may
    capture it into a HIP graph: three replays, with eager work and synchronisations between them, each bit-equal
    to the eager result and to the oracle.  128 tokens take the GEMM that splits k across workgroups: its tile counters
    live in the workspace and are cleared by the quantiser kernel of the same call."""
    rng = np.random.default_rng(900 + m)
    n, k = 2560, 6912
    w = synth_weights(rng, n, k)
    layer = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), "graph")
    layer.update_weights(dev(w))
    qw, ws_ = orc.quantize_weights_absmean(w)
    x = synth_activations(rng, m, k, outliers=True)
    ref = orc.bitlinear_forward(x, orc.pack_2bit(qw), n, ws_)[0]
    xd = dev(x)
    y = torch.empty((m, n), device="cuda", dtype=torch.float32)
    scratch = torch.empty((max(layer.workspace_size(m), 16),), device="cuda", dtype=torch.uint8)
    layer.forward(xd, out=y, workspace=scratch)
    torch.cuda.synchronize()
    assert np.array_equal(host(y), ref)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layer.forward(xd, out=y, workspace=scratch)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        layer.forward(xd, out=y, workspace=scratch)
        layer.forward(xd, out=y, workspace=scratch)
    for _ in range(3):
        y.zero_()
        other = layer.forward(xd)  # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(host(y), ref)
        assert np.array_equal(host(other), ref)


@pytest.mark.parametrize("n", [1, 4, 5, 6, 1000, 10001, 2560 * 640])
def test_base3_pack_unpack_bit_exact(n):
    """Base3PackedPacker on the GPU against the oracle, ragged tails included; decoding every byte value."""
    rng = np.random.default_rng(n)
    q = rng.integers(-1, 2, size=n).astype(np.int8)
    packed = bh.pack_ternary_base3(dev(q))
    assert np.array_equal(host(packed), orc.pack_base3(q))
    assert np.array_equal(host(bh.unpack_ternary_base3(packed, n)), q)
    raw = rng.integers(0, 256, size=(n + 4) // 5).astype(np.uint8)  # any byte, also above 242
    assert np.array_equal(host(bh.unpack_ternary_base3(dev(raw), n)), orc.unpack_base3(raw, n))


@pytest.mark.parametrize("n,k", [(1, 4), (48, 300), (33, 7), (640, 2560)])
@pytest.mark.parametrize("on_device", [False, True])
def test_bitlinear_base3_weights_match_2bit_weights(n, k, on_device):
    """A layer loaded from base-3 bytes holds the same canonical 2-bit bytes and computes the same forward as a
    layer loaded from the 2-bit bytes of the same ternary matrix; short buffers are a shape mismatch."""
    rng = np.random.default_rng(31 * n + k)
    q = rng.integers(-1, 2, size=(n, k)).astype(np.int8)
    ws = np.float32(0.0173)
    b3 = torch.from_numpy(orc.pack_base3(q.ravel()))
    a = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), "b3")
    a.set_base3_weights(b3.cuda() if on_device else b3, float(ws))
    b = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), "b2")
    b.set_quantized_weights(dev(orc.pack_2bit(q.ravel())), float(ws))
    pa, sa = a.get_quantized_weights()
    pb, sb = b.get_quantized_weights()
    assert sa == sb == float(ws)
    assert np.array_equal(pa.numpy(), pb.numpy())
    assert np.array_equal(pa.numpy(), orc.pack_2bit(q.ravel()))
    x = synth_activations(rng, 3, k)
    ya, yb = host(a.forward(dev(x))), host(b.forward(dev(x)))
    assert np.array_equal(ya, yb)
    assert np.array_equal(ya, orc.bitlinear_forward(x, orc.pack_2bit(q.ravel()), n, ws)[0])
    if b3.numel() > 1:
        with pytest.raises(bh.BitLinearError) as err:
            a.set_base3_weights(b3[:-1].contiguous(), float(ws))
        assert err.value.status == bh.SHAPE_MISMATCH


@pytest.mark.parametrize("n,k", [(16, 320), (1, 5), (33, 7), (48, 300), (640, 2560), (2560, 6912), (100, 2561), (4096, 4096)])
def test_gemv_on_base3_bytes_bit_exact(n, k):
    """bitnet_hip_gemv_base3: the decode GEMV that consumes the base-3 bytes of Base3PackedPacker (packing.rs:421-501)
    themselves.  The streaming layout is built from the oracle's flat base-3 bytes; int32 accumulators equal the oracle's
    contraction of the same ternary matrix (and hence the 2-bit GEMV), the f32 output its epilogue; the reference's
    encoding fixture (140 = [1, 0, -1, 1, 0]) goes through the same path."""
    rng = np.random.default_rng(7 * n + k)
    q = rng.integers(-1, 2, size=(n, k)).astype(np.int8)
    a = rng.integers(-127, 128, size=(1, k)).astype(np.int8)
    b3 = orc.pack_base3(q.ravel())
    tiled = bh.retile_base3(dev(b3), n, k)
    assert tiled.numel() == bh.base3_tiled_size(n, k) == ((n + 15) // 16) * ((k + 319) // 320) * 1024
    ws, a_scale = f32(0.0171), np.array([f32(3.37)], dtype=f32)
    acc, out = bh.gemv_base3(tiled, dev(a.ravel()), n, w_scale=dev(np.array([ws], dtype=f32)), a_scale=dev(a_scale))
    acc_ref = orc.gemm_w2a8(orc.pack_2bit(q.ravel()), a, n)
    assert np.array_equal(host(acc), acc_ref[0])
    assert np.array_equal(host(out), orc.epilogue(acc_ref, ws, a_scale)[0])
    # the streaming layout, byte by byte: slot 16 kq + r of tile (row block, k-tile), byte t = columns 320 kt + 80 kq + 5 t ..
    th = host(tiled).reshape(-1, 64, 16)
    kt_count = (k + 319) // 320
    for _ in range(64):
        row, col = int(rng.integers(n)), int(rng.integers(k))
        kt, rem = divmod(col, 320)
        kq, rem = divmod(rem, 80)
        t, d = divmod(rem, 5)
        byte = int(th[(row // 16) * kt_count + kt, 16 * kq + row % 16, t])
        assert (byte // 3 ** d) % 3 - 1 == q[row, col]


def test_gemv_on_base3_bytes_reference_fixture_and_errors():
    """The reference's own base-3 vector (packing_correctness_tests.rs:159-176: [1, 0, -1, 1, 0] -> 140) as a 1 x 5 matrix,
    and the argument checks of the entry point."""
    b3 = np.array([140], dtype=np.uint8)
    assert np.array_equal(orc.unpack_base3(b3, 5), np.array([1, 0, -1, 1, 0], dtype=np.int8))
    tiled = bh.retile_base3(dev(b3), 1, 5)
    a = np.array([3, -7, 11, 5, 100], dtype=np.int8)
    acc, out = bh.gemv_base3(tiled, dev(a), 1)
    assert out is None and host(acc).tolist() == [3 - 11 + 5]
    with pytest.raises(bh.BitLinearError) as err:
        bh.gemv_base3(tiled[:-16].contiguous(), dev(a), 1)
    assert err.value.status == bh.SHAPE_MISMATCH
    with pytest.raises(bh.BitLinearError) as err:
        bh.retile_base3(dev(b3), 2, 5)
    assert err.value.status == bh.SHAPE_MISMATCH


@pytest.mark.parametrize("kind,cls", [(bh.LOOKUP_TERNARY, bh.HipTernaryLookupKernel), (bh.LOOKUP_I2S, bh.HipI2SLookupKernel)],
                         ids=["ternary", "i2s"])
def test_lookup_kernels_bit_exact(kind, cls):
    """TernaryLookupKernel / I2SLookupKernel::compute on the GPU: bit-identical to the oracle, out-of-table weights,
    non-finite inputs and signed zeros included; the shortest buffer decides the length; empty buffers are errors."""
    rng = np.random.default_rng(kind)
    kernel = cls()
    for n in (1, 5, 1000, 100003):
        w = rng.integers(-3, 4, size=n).astype(np.int8)
        x = rng.standard_normal(n, dtype=f32)
        x[rng.integers(0, n, size=max(1, n // 50))] = np.inf
        x[rng.integers(0, n, size=max(1, n // 50))] = np.nan
        out = torch.zeros((n,), device="cuda", dtype=torch.float32)
        kernel.compute(dev(w), dev(x), out)
        ref = orc.lookup_compute(kind, w, x)
        assert np.array_equal(host(out).view(np.uint32), ref.view(np.uint32))
    out = torch.full((6,), 7.0, device="cuda", dtype=torch.float32)
    kernel.compute(dev(np.array([1, -1, 1, 1], np.int8)), dev(np.array([2.0, 3.0, 4.0], f32)), out)
    assert host(out).tolist() == [2.0, -3.0, 4.0, 7.0, 7.0, 7.0]
    empty_w, empty_x = torch.empty((0,), dtype=torch.int8, device="cuda"), torch.empty((0,), dtype=torch.float32, device="cuda")
    for args in ((empty_w, dev(np.ones(2, f32)), out), (dev(np.ones(2, np.int8)), empty_x, out),
                 (dev(np.ones(2, np.int8)), dev(np.ones(2, f32)), empty_x)):
        with pytest.raises(bh.BitLinearError) as err:
            kernel.compute(*args)
        assert err.value.status == bh.INVALID_CONFIG
    assert kernel.name() and kernel.optimal_batch_size() > 0


def test_bitlinear_forward_prefill_uses_quantiser_row_sums():
    """BitLinear.forward at a prefill token count: quantiser -> row sums -> LDS-direct GEMM, bit-exact."""
    rng = np.random.default_rng(77)
    m, k, n = 384, 2560, 640
    w = synth_weights(rng, n, k)
    x = synth_activations(rng, m, k, outliers=True)
    g = (1 + 0.1 * rng.standard_normal(k, dtype=f32)).astype(f32)
    layer = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), "prefill")
    layer.update_weights(dev(w))
    out, q, a_scale, acc = layer.forward(dev(x), gamma=dev(g), debug=True)
    qw, ws = orc.quantize_weights_absmean(w)
    out_ref, q_ref, s_ref, acc_ref = orc.bitlinear_forward(x, orc.pack_2bit(qw), n, ws, g=g, eps=1e-5)
    assert np.array_equal(host(q), q_ref) and np.array_equal(host(a_scale), s_ref)
    assert np.array_equal(host(acc), acc_ref)
    assert np.array_equal(host(out), out_ref)


@pytest.mark.parametrize("m,k,n", [(97, 6912, 2560), (128, 6912, 2560), (200, 4096, 1000), (256, 6912, 2560), (130, 8192, 644),
                                   (255, 5120, 1408), (97, 4096, 16), (256, 8192, 2816), (300, 4352, 2240)])
def test_forward_split_k_bit_exact(m, k, n):
    """A long k with few output tiles (97 to 256 tokens at 6912 -> 2560): forward() splits k across workgroups, which
    exchange int32 partial tiles through the workspace.  Checked against the oracle (activations, accumulators, f32
    output with bias and residual); with a workspace that holds only the quantised activations (no split: same bits);
    on a workspace full of ones (the tile counters are cleared by the quantiser of the same call); and on the same
    workspace three times in a row (the counters are left at zero)."""
    rng = np.random.default_rng(m + k + n)
    w = synth_weights(rng, n, k)
    x = synth_activations(rng, m, k, outliers=True)
    bias = rng.standard_normal(n, dtype=f32)
    res = rng.standard_normal((m, n), dtype=f32)
    layer = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n, use_bias=True), "split")
    layer.update_weights(dev(w))
    layer.update_bias(dev(bias))
    qw, ws = orc.quantize_weights_absmean(w)
    out_ref, q_ref, s_ref, acc_ref = orc.bitlinear_forward(x, orc.pack_2bit(qw), n, ws, bias=bias, residual=res)
    out, q, a_scale, acc = layer.forward(dev(x), residual=dev(res), debug=True)
    assert np.array_equal(host(q), q_ref) and np.array_equal(host(a_scale), s_ref)
    assert np.array_equal(host(acc), acc_ref)
    assert np.array_equal(host(out), out_ref)
    full = layer.workspace_size(m)
    quant_only = ((m * k + 255) // 256) * 256 + 2 * (((4 * m) + 255) // 256) * 256 + 256
    assert full > quant_only, "this shape is expected to take the split"
    small = torch.full((quant_only,), 1, dtype=torch.uint8, device="cuda")
    assert np.array_equal(host(layer.forward(dev(x), residual=dev(res), workspace=small)), out_ref)
    big = torch.full((full,), 1, dtype=torch.uint8, device="cuda")
    for _ in range(3):
        assert np.array_equal(host(layer.forward(dev(x), residual=dev(res), workspace=big)), out_ref)


# ---- L1: BitLinear object ----------------------------------------------------------------------------------

def test_bitlinear_forward_config1_bit_exact():
    """BASELINE config 1: M=1, K=2560, N=2560, seed 0, W ~ N(0, 0.02), X ~ N(0, 1)."""
    rng = np.random.default_rng(0)
    w = synth_weights(rng, 2560, 2560)
    x = synth_activations(rng, 1, 2560)
    layer = bh.BitLinear(bh.BitLinearConfig(in_features=2560, out_features=2560), "config1")
    layer.update_weights(torch.from_numpy(w))  # host weights, quantised on the GPU
    out, q, a_scale, acc = layer.forward(dev(x), debug=True)
    qw, ws = orc.quantize_weights_absmean(w)
    packed_h, ws_h = layer.get_quantized_weights()
    assert ws_h == ws and np.array_equal(packed_h.numpy(), orc.pack_2bit(qw))
    out_ref, q_ref, s_ref, acc_ref = orc.bitlinear_forward(x, orc.pack_2bit(qw), 2560, ws)
    assert np.array_equal(host(q), q_ref)
    assert np.array_equal(host(a_scale), s_ref)
    assert np.array_equal(host(acc), acc_ref)
    assert np.array_equal(host(out), out_ref)
    assert rel_err(host(out), out_ref) <= REL_TOL
    # the non-debug call gives the same bits
    assert np.array_equal(host(layer.forward(dev(x))), out_ref)


def test_bitlinear_forward_shapes_bias_norm_and_layouts():
    rng = np.random.default_rng(31)
    k, n = 256, 80
    w = synth_weights(rng, n, k)
    qw, ws = orc.quantize_weights_absmean(w)
    packed = orc.pack_2bit(qw)
    bias = rng.standard_normal(n, dtype=f32)
    g = rng.standard_normal(k, dtype=f32)
    layer = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n, use_bias=True), "t")
    with pytest.raises(bh.BitLinearError) as ei:
        layer.forward(dev(np.zeros((2, k), f32)))
    assert ei.value.kind == "NotInitialized"
    layer.update_weights(dev(w))
    # bias starts at zero, like the reference's Tensor::zeros bias (layer.rs:127-133)
    x = synth_activations(rng, 6, k)
    ref0 = orc.bitlinear_forward(x, packed, n, ws)[0]
    assert np.array_equal(host(layer.forward(dev(x))), ref0)
    layer.update_bias(dev(bias))
    ref = orc.bitlinear_forward(x, packed, n, ws, bias=bias)[0]
    assert np.array_equal(host(layer.forward(dev(x))), ref)
    # rank 3 input is flattened to [b*s, in] and reshaped back (forward.rs:182-207)
    out3 = layer.forward(dev(x.reshape(2, 3, k)))
    assert tuple(out3.shape) == (2, 3, n) and np.array_equal(host(out3).reshape(6, n), ref)
    # fused RMSNorm + residual
    res = rng.standard_normal((6, n), dtype=f32)
    refn = orc.bitlinear_forward(x, packed, n, ws, g=g, eps=1e-5, bias=bias, residual=res)[0]
    assert np.array_equal(host(layer.forward(dev(x), gamma=dev(g), residual=dev(res))), refn)
    # [in, out] orientation (the GGUF-side convention) gives the same layer
    layer_t = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), "t_in_out")
    layer_t.update_weights(dev(np.ascontiguousarray(w.T)), layout=bh.LAYOUT_IN_OUT)
    p2, s2 = layer_t.get_quantized_weights()
    assert np.array_equal(p2.numpy(), packed)
    assert abs(s2 - float(ws)) <= 1e-7 * float(ws)  # the declared f64 summation order follows the given orientation
    # pre-quantised weights (forward_with_quantized_weights)
    layer_p = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), "t_packed")
    layer_p.set_quantized_weights(torch.from_numpy(packed), float(ws))
    assert np.array_equal(host(layer_p.forward(dev(x))), ref0)


@pytest.mark.parametrize("m", [1, 3, 8, 20, 40, 64, 200, 300, 1100])
def test_forward_multi_matches_single_forwards(m):
    """q/k/v-style: several layers on one input give exactly what each layer gives alone, and what the oracle gives.
    (m = 200: the token-group GEMV, which takes prefill launches too small for the GEMM to fill the chip; m = 300 and
    1100: the projections share launches of the 64 x 160 and of the eight-wavefront prefill GEMM.)"""
    rng = np.random.default_rng(40 + m)
    k = 2560
    ns = [2560, 640, 640, 96]
    g = (1 + 0.1 * rng.standard_normal(k, dtype=f32)).astype(f32)
    x = synth_activations(rng, m, k, outliers=True)
    layers, refs = [], []
    for i, n in enumerate(ns):
        w = synth_weights(rng, n, k)
        layer = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), f"multi{i}")
        layer.update_weights(dev(w))
        layers.append(layer)
        qw, ws = orc.quantize_weights_absmean(w)
        refs.append(orc.bitlinear_forward(x, orc.pack_2bit(qw), n, ws, g=g, eps=1e-5)[0])
    outs = bh.forward_multi(layers, dev(x), gamma=dev(g))
    for layer, out, ref in zip(layers, outs, refs):
        assert np.array_equal(host(out), ref)
        assert np.array_equal(host(layer.forward(dev(x), gamma=dev(g))), ref)
    other = bh.BitLinear(bh.BitLinearConfig(in_features=k + 4, out_features=8), "other")
    other.update_weights(torch.ones(8, k + 4))
    with pytest.raises(bh.BitLinearError) as ei:
        bh.forward_multi([layers[0], other], dev(x))
    assert ei.value.kind == "ShapeMismatch"


def test_forward_multi_prefill_gate_up_one_launch():
    """gate and up at M = 2048 share one launch of the 128 x 160 prefill GEMM (1408 tiles): sampled rows against the
    oracle, everything against the single-layer forwards."""
    rng = np.random.default_rng(4242)
    m, k, n = 2048, 2560, 6912
    g = (1 + 0.1 * rng.standard_normal(k, dtype=f32)).astype(f32)
    x = synth_activations(rng, m, k)
    rows = np.sort(rng.choice(m, size=24, replace=False))
    layers, refs = [], []
    for i in range(2):
        w = synth_weights(rng, n, k)
        layer = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), f"gu{i}")
        layer.update_weights(dev(w))
        layers.append(layer)
        qw, ws = orc.quantize_weights_absmean(w)
        refs.append(orc.bitlinear_forward(x[rows], orc.pack_2bit(qw), n, ws, g=g, eps=1e-5)[0])
    outs = bh.forward_multi(layers, dev(x), gamma=dev(g))
    for layer, out, ref in zip(layers, outs, refs):
        got = host(out)
        assert np.array_equal(got[rows], ref)
        assert np.array_equal(got, host(layer.forward(dev(x), gamma=dev(g))))


def test_forward_multi_prefill_qkv_128x128_tiles():
    """q, k and v at M = 3072 (and a ragged M just below) share one launch of the 128 x 128 instance of the prefill GEMM
    (720 tiles): sampled rows against the oracle, everything against the single-layer forwards, which take other
    instances (q alone 480 tiles, k and v alone 120)."""
    rng = np.random.default_rng(3072)
    k, ns = 2560, [2560, 640, 640]
    g = (1 + 0.1 * rng.standard_normal(k, dtype=f32)).astype(f32)
    layers, packed = [], []
    for i, n in enumerate(ns):
        w = synth_weights(rng, n, k)
        layer = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), f"qkv{i}")
        layer.update_weights(dev(w))
        layers.append(layer)
        qw, ws = orc.quantize_weights_absmean(w)
        packed.append((orc.pack_2bit(qw), n, ws))
    for m in (3072, 3072 - 37):
        x = synth_activations(rng, m, k, outliers=True)
        rows = np.sort(rng.choice(m, size=24, replace=False))
        rows[-1] = m - 1
        outs = bh.forward_multi(layers, dev(x), gamma=dev(g))
        for layer, out, (pk, n, ws) in zip(layers, outs, packed):
            got = host(out)
            assert np.array_equal(got[rows], orc.bitlinear_forward(x[rows], pk, n, ws, g=g, eps=1e-5)[0])
            assert np.array_equal(got, host(layer.forward(dev(x), gamma=dev(g))))


@pytest.mark.parametrize("m", [1, 2, 3, 4, 6, 7])
@pytest.mark.parametrize("n,k", [(1, 4), (17, 260), (1000, 2560), (2560, 6912), (6912 + 5, 2560), (40, 8192), (13824, 2560)])
def test_forward_fused_rows_bit_exact(m, n, k):
    """One to six tokens take the 16-wavefront kernel with the quantiser in its prologue and a set of workgroups per
    token, as long as those stay within 512 (otherwise, and from seven tokens on, the stand-alone quantiser and the MFMA
    GEMV run): row-block groups that do not fill the last 8 of the grid, one / two chunks per thread, one / four row
    blocks per workgroup, RMSNorm, bias and residual."""
    rng = np.random.default_rng(31 * m + n + k)
    w = synth_weights(rng, n, k)
    x = synth_activations(rng, m, k, outliers=True)
    g = (1 + 0.1 * rng.standard_normal(k, dtype=f32)).astype(f32)
    bias = rng.standard_normal(n, dtype=f32)
    res = rng.standard_normal((m, n), dtype=f32)
    layer = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n, use_bias=True), "rows")
    layer.update_weights(dev(w))
    layer.update_bias(dev(bias))
    qw, ws_ = orc.quantize_weights_absmean(w)
    for norm in (False, True):
        ref = orc.bitlinear_forward(x, orc.pack_2bit(qw), n, ws_, g=g if norm else None, eps=1e-5, bias=bias, residual=res)[0]
        got = host(layer.forward(dev(x), gamma=dev(g) if norm else None, residual=dev(res)))
        assert np.array_equal(got, ref)


@pytest.mark.parametrize("m", [1, 2, 3, 5, 8])
def test_bitlinear_forward_decode_debug_outputs(m):
    """At decode token counts the quantiser runs inside the GEMV launch; its int8 row, scale and the int32
    accumulators are still observable and bit-exact, with and without RMSNorm, at both FFN widths."""
    rng = np.random.default_rng(50 + m)
    for k, n, norm in [(2560, 640, True), (6912, 2560, False), (1024, 48, True)]:
        w = synth_weights(rng, n, k)
        x = synth_activations(rng, m, k, outliers=True)
        g = (1 + 0.1 * rng.standard_normal(k, dtype=f32)).astype(f32) if norm else None
        layer = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), "dbg")
        layer.update_weights(dev(w))
        out, q, a_scale, acc = layer.forward(dev(x), gamma=dev(g) if norm else None, debug=True)
        qw, ws = orc.quantize_weights_absmean(w)
        out_ref, q_ref, s_ref, acc_ref = orc.bitlinear_forward(x, orc.pack_2bit(qw), n, ws, g=g, eps=1e-5)
        assert np.array_equal(host(q), q_ref) and np.array_equal(host(a_scale), s_ref)
        assert np.array_equal(host(acc), acc_ref) and np.array_equal(host(out), out_ref)
    # the reference's literal summation order inside the fused launch
    layer = bh.BitLinear(bh.BitLinearConfig(in_features=1024, out_features=48, sum_order=bh.SUM_SEQUENTIAL), "seq")
    layer.update_weights(dev(w))
    out_ref = orc.bitlinear_forward(x, orc.pack_2bit(qw), n, ws, g=g, eps=1e-5, order=orc.SUM_SEQUENTIAL)[0]
    assert np.array_equal(host(layer.forward(dev(x), gamma=dev(g))), out_ref)


@pytest.mark.parametrize("k,ns", [(2560, (640,)), (6912, (2560,)), (2560, (6912, 6912))], ids=["short", "long_row", "two_row_blocks"])
def test_decode_sequential_sum_order_four_wavefront_kernel(k, ns):
    """One token with RMSNorm in the reference's literal (sequential) summation order: the launch shape that keeps four
    wavefronts per workgroup (every thread runs the whole chain), with short and long rows, one and two row blocks per
    workgroup, one and two projections per launch."""
    rng = np.random.default_rng(k + len(ns))
    g = (1 + 0.1 * rng.standard_normal(k, dtype=f32)).astype(f32)
    x = synth_activations(rng, 1, k, outliers=True)
    layers, refs = [], []
    for i, n in enumerate(ns):
        w = synth_weights(rng, n, k)
        layer = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n, sum_order=bh.SUM_SEQUENTIAL), f"seq{i}")
        layer.update_weights(dev(w))
        layers.append(layer)
        qw, ws = orc.quantize_weights_absmean(w)
        refs.append(orc.bitlinear_forward(x, orc.pack_2bit(qw), n, ws, g=g, eps=1e-5, order=orc.SUM_SEQUENTIAL)[0])
    outs = bh.forward_multi(layers, dev(x), gamma=dev(g)) if len(ns) > 1 else [layers[0].forward(dev(x), gamma=dev(g))]
    for out, ref in zip(outs, refs):
        assert np.array_equal(host(out), ref)


def test_forward_from_several_threads_and_streams():
    """BitLinear is Send + Sync in the reference (layer.rs:427-428): forward on one layer object from several host
    threads, each on a stream of its own, at decode and prefill token counts, while nothing is shared but the
    read-locked weights."""
    import threading

    rng = np.random.default_rng(99)
    k, n = 2560, 640
    w = synth_weights(rng, n, k)
    layer = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), "shared")
    layer.update_weights(dev(w))
    qw, ws = orc.quantize_weights_absmean(w)
    packed = orc.pack_2bit(qw)
    cases = []
    for t, m in enumerate([1, 1, 5, 130]):
        x = synth_activations(rng, m, k, outliers=True)
        cases.append((x, orc.bitlinear_forward(x, packed, n, ws)[0]))
    errors = []

    def worker(x, ref):
        try:
            stream = torch.cuda.Stream()  # default priority
            xd = dev(x)
            torch.cuda.current_stream().synchronize()
            for _ in range(25):
                with torch.cuda.stream(stream):
                    out = layer.forward(xd, stream=stream)
                stream.synchronize()
                if not np.array_equal(host(out), ref):
                    errors.append("mismatch")
                    return
        except Exception as e:  # noqa: BLE001 - reported below
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=c) for c in cases]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not errors, errors
    assert not any(th.is_alive() for th in threads)


def test_bitlinear_error_behaviour_matches_reference():
    """forward.rs:304-371: wrong last dimension -> ShapeMismatch; rank other than 2/3 -> ShapeMismatch."""
    layer = bh.BitLinear(bh.BitLinearConfig(in_features=4, out_features=3), "test_layer_shape")
    layer.update_weights(torch.ones(3, 4))
    out = layer.forward(torch.ones(2, 4, device="cuda"))
    assert tuple(out.shape) == (2, 3)
    with pytest.raises(bh.BitLinearError) as ei:
        layer.forward(torch.ones(2, 5, device="cuda"))
    assert ei.value.kind == "ShapeMismatch" and ei.value.expected == [2, 4] and ei.value.actual == [2, 5]
    with pytest.raises(bh.BitLinearError) as ei:
        layer.forward(torch.ones(4, device="cuda"))
    assert ei.value.kind == "ShapeMismatch"
    with pytest.raises(bh.BitLinearError) as ei:
        layer.forward(torch.ones(2, 2, 2, 4, device="cuda"))
    assert ei.value.kind == "ShapeMismatch"
    with pytest.raises(bh.BitLinearError) as ei:
        layer.update_weights(torch.ones(4, 3))
    assert ei.value.kind == "ShapeMismatch" and ei.value.expected == [3, 4]
    with pytest.raises(bh.BitLinearError) as ei:
        layer.update_bias(torch.ones(3))
    assert ei.value.kind == "InvalidConfig" and "Bias is not enabled" in str(ei.value)
    with pytest.raises(bh.BitLinearError):
        layer.forward_batch(torch.ones(4, device="cuda"))
    # empty batch: nothing to do
    assert tuple(layer.forward(torch.ones(0, 4, device="cuda")).shape) == (0, 3)


# ---- L1: decoder layer and stack ----------------------------------------------------------------------------

def build_decoder(rng, layers, hidden, ffn, qh, kvh, hd, max_tokens, eps=1e-5):
    dec = bh.DecoderProjections(layers, hidden, ffn, qh, kvh, hd, eps=eps, max_tokens=max_tokens)
    ref = []
    for l in range(layers):
        packed, scales = [], []
        for p in range(7):
            n, k = dec.proj_shape(p)
            w = synth_weights(rng, n, k)
            dec.projection(l, p).update_weights(dev(w))
            qw, s = orc.quantize_weights_absmean(w)
            packed.append(orc.pack_2bit(qw))
            scales.append(s)
        ga = (1 + 0.1 * rng.standard_normal(hidden, dtype=f32)).astype(f32)
        gf = (1 + 0.1 * rng.standard_normal(hidden, dtype=f32)).astype(f32)
        dec.set_norm(l, 0, torch.from_numpy(ga))
        dec.set_norm(l, 1, torch.from_numpy(gf))
        ref.append((packed, scales, ga, gf))
    return dec, ref


def oracle_stack(ref, x, hidden, ffn, qh, kvh, hd, eps=1e-5):
    q = k = None
    for packed, scales, ga, gf in ref:
        x, q, k = orc.decoder_layer(x, packed, scales, hidden, ffn, qh, kvh, hd, ga, gf, eps)
    return x, q, k


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 6, 7, 8])
def test_decoder_layer_config2_bit_exact(m):
    """BASELINE config 2: one decoder layer's seven projections at BitNet-2B shapes."""
    rng = np.random.default_rng(0)
    dec, ref = build_decoder(rng, 1, 2560, 6912, 20, 5, 128, max_tokens=8)
    assert dec.weight_bytes() == 17_367_040
    x = synth_activations(rng, m, 2560)
    out, q, k = dec.decode(dev(x), want_qk=True)
    x_ref, q_ref, k_ref = oracle_stack(ref, x, 2560, 6912, 20, 5, 128)
    assert np.array_equal(host(q), q_ref) and np.array_equal(host(k), k_ref)
    assert np.array_equal(host(out), x_ref)
    assert rel_err(host(out), x_ref) <= REL_TOL


@pytest.mark.parametrize("layers", [2, 3])
def test_decoder_stack_small_bit_exact(layers):
    rng = np.random.default_rng(layers)
    dims = (256, 512, 4, 2, 64)
    dec, ref = build_decoder(rng, layers, *dims, max_tokens=4)
    x = synth_activations(rng, 3, 256)
    out = dec.decode(dev(x))
    assert np.array_equal(host(out), oracle_stack(ref, x, *dims)[0])
    with pytest.raises(bh.BitLinearError) as ei:
        dec.decode(dev(synth_activations(rng, 5, 256)))
    assert ei.value.kind == "ShapeMismatch"


def random_packed_ternary(rng, n, k):
    """[n, k] ternary weights as flat 2-bit bytes drawn directly (code 3 folded onto code 1: weight 0), so a
    30-block stack of 521 MB is generated in a second: P(-1) = P(+1) = 1/4, P(0) = 1/2."""
    b = rng.integers(0, 256, size=n * k // 4, dtype=np.uint8)
    return b & ~((b & (b >> 1) & 0x55) << 1)


def build_decoder_packed(rng, layers, hidden, ffn, qh, kvh, hd, max_tokens, eps=1e-5):
    dec = bh.DecoderProjections(layers, hidden, ffn, qh, kvh, hd, eps=eps, max_tokens=max_tokens)
    ref = []
    for l in range(layers):
        packed, scales = [], []
        for p in range(7):
            n, k = dec.proj_shape(p)
            pk = random_packed_ternary(rng, n, k)
            s = f32(0.016 * (1 + 0.25 * rng.random()))
            dec.projection(l, p).set_quantized_weights(torch.from_numpy(pk), float(s))
            packed.append(pk)
            scales.append(s)
        ga = (1 + 0.1 * rng.standard_normal(hidden, dtype=f32)).astype(f32)
        gf = (1 + 0.1 * rng.standard_normal(hidden, dtype=f32)).astype(f32)
        dec.set_norm(l, 0, torch.from_numpy(ga))
        dec.set_norm(l, 1, torch.from_numpy(gf))
        ref.append((packed, scales, ga, gf))
    return dec, ref


def test_decoder_stack_config5_full_depth_bit_exact():
    """BASELINE config 5 at its real depth: 30 blocks at 2560 / 6912 / 20 / 5 / 128 (521,011,200 packed bytes) on a
    decoder sized for 8 tokens, one token and eight tokens per step, every block checked against the oracle's chain;
    then runs of blocks that start and end inside the stack, in place."""
    dims = (2560, 6912, 20, 5, 128)
    rng = np.random.default_rng(5)
    dec, ref = build_decoder_packed(rng, 30, *dims, max_tokens=8)
    assert dec.weight_bytes() == 521_011_200
    for m in (1, 8):
        x = synth_activations(rng, m, dims[0])
        # the oracle's hidden state after every block
        states, cur = [x], x
        for l in range(30):
            cur, q_ref, k_ref = oracle_stack(ref[l:l + 1], cur, *dims)
            states.append(cur)
        assert np.all(np.isfinite(states[-1]))
        out, q, k = dec.decode(dev(x), want_qk=True)
        assert np.array_equal(host(out), states[30]), f"m={m}: 30-block output differs from the oracle"
        assert np.array_equal(host(q), q_ref) and np.array_equal(host(k), k_ref)
        assert rel_err(host(out), states[30]) <= REL_TOL
        for lo, hi in ((2, 7), (4, 5), (3, 30), (29, 30)):
            buf = dev(states[lo].copy())
            dec.decode(buf, out=buf, layers=(lo, hi))
            assert np.array_equal(host(buf), states[hi]), f"m={m}: blocks {lo}..{hi - 1}"


@pytest.mark.parametrize("dims,layers", [((2560, 6912, 20, 5, 128), 4), ((256, 512, 4, 2, 64), 3),
                                         ((1024, 2816, 8, 8, 128), 2)])
def test_decoder_repeated_calls_subranges_and_streams(dims, layers):
    """One token: repeated calls, sub-ranges of blocks, in-place hidden states, one block at a time (as the benchmark
    does), and calls issued from two streams in turn (the decoder's buffers are shared: the second call waits for the
    first on the GPU)."""
    rng = np.random.default_rng(layers + dims[0])
    dec, ref = build_decoder(rng, layers, *dims, max_tokens=2)
    x = synth_activations(rng, 1, dims[0])
    x_ref, q_ref, k_ref = oracle_stack(ref, x, *dims)
    for _ in range(3):
        out, q, k = dec.decode(dev(x), want_qk=True)
        assert np.array_equal(host(out), x_ref)
        assert np.array_equal(host(q), q_ref) and np.array_equal(host(k), k_ref)
    x1_ref = oracle_stack(ref[:1], x, *dims)[0]
    buf = dev(x1_ref.copy())
    dec.decode(buf, out=buf, layers=(1, layers))
    assert np.array_equal(host(buf), x_ref)
    cur = dev(x)
    for l in range(layers):
        cur = dec.decode(cur, layers=(l, l + 1))
    assert np.array_equal(host(cur), x_ref)
    # two streams in alternation, no host synchronisation in between
    xs = [dev(synth_activations(rng, 2, dims[0])) for _ in range(4)]
    refs = [oracle_stack(ref, host(t), *dims)[0] for t in xs]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    outs = []
    for i, t in enumerate(xs):
        with torch.cuda.stream(streams[i % 2]):
            outs.append(dec.decode(t, stream=streams[i % 2]))
    torch.cuda.synchronize()
    for o, r in zip(outs, refs):
        assert np.array_equal(host(o), r)


@pytest.mark.parametrize("dims,layers,m", [((2560, 6912, 20, 5, 128), 3, 1), ((2560, 6912, 20, 5, 128), 2, 8),
                                           ((256, 512, 4, 2, 64), 3, 3), ((1024, 2816, 8, 8, 128), 2, 1)])
def test_decoder_recorded_step_replays_match_the_oracle(dims, layers, m):
    """A decode step recorded as a HIP graph (bitnet_hip_decoder_graph_*): every replay, with eager work and host
    synchronisations between the replays and with new inputs written into the recorded input tensor, equals the oracle's
    chain bit for bit; so do a recorded sub-range in place, replays on another stream, replays interleaved with eager
    decode calls on the same decoder, and replays after a weight update (the graph reads the layers' buffers, which an
    update keeps)."""
    rng = np.random.default_rng(17 * layers + m + dims[0])
    dec, ref = build_decoder_packed(rng, layers, *dims, max_tokens=max(m, 2))
    x = dev(synth_activations(rng, m, dims[0]))
    graph = dec.record(x, want_qk=True)
    other = torch.cuda.Stream()
    for round_ in range(4):
        fresh = synth_activations(rng, m, dims[0])
        x_ref, q_ref, k_ref = oracle_stack(ref, fresh, *dims)
        x.copy_(dev(fresh))
        graph.out.zero_()
        if round_ == 2:  # another stream, ordered behind the copy above by an explicit wait
            other.wait_stream(torch.cuda.current_stream())
            graph.replay(stream=other)
            torch.cuda.current_stream().wait_stream(other)
        else:
            graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(host(graph.out), x_ref), f"replay {round_}"
        assert np.array_equal(host(graph.q), q_ref) and np.array_equal(host(graph.k), k_ref)
        # eager work on the same decoder between the replays
        assert np.array_equal(host(dec.decode(dev(fresh))), x_ref)
    # a sub-range of blocks, in place
    if layers >= 3:
        start = oracle_stack(ref[:1], host(x), *dims)[0]
        want = oracle_stack(ref[1:], start, *dims)[0]
        buf = dev(start.copy())
        sub = dec.record(buf, out=buf, layers=(1, layers))
        for _ in range(2):
            buf.copy_(dev(start))
            sub.replay()
            assert np.array_equal(host(buf), want)
    # new weights in one projection: the recorded step reads them
    n, k = dec.proj_shape(6)  # down
    pk = random_packed_ternary(rng, n, k)
    dec.projection(layers - 1, 6).set_quantized_weights(torch.from_numpy(pk), 0.02)
    packed, scales, ga, gf = ref[-1]
    ref[-1] = (packed[:6] + [pk], scales[:6] + [f32(0.02)], ga, gf)
    x_ref = oracle_stack(ref, host(x), *dims)[0]
    graph.replay()
    assert np.array_equal(host(graph.out), x_ref)


@pytest.mark.parametrize("dims,layers,m,chains", [((2560, 6912, 20, 5, 128), 2, 8, 2), ((2560, 6912, 20, 5, 128), 2, 8, 4),
                                                  ((2560, 6912, 20, 5, 128), 2, 5, 8), ((256, 512, 4, 2, 64), 3, 3, 2),
                                                  ((1024, 2816, 8, 8, 128), 3, 16, 3)])
def test_decoder_row_group_chains_match_the_oracle(dims, layers, m, chains):
    """bitnet_hip_decoder_set_chains: a step of several token rows run as groups of rows side by side, each group a chain
    of launches on a stream of the decoder's own.  Eager calls, a recorded step replayed several times (with eager work
    and host synchronisations between the replays), a sub-range in place and the last block's q / k equal the oracle's
    chain bit for bit; more chains than rows are cut down to one row each; back to one chain afterwards."""
    rng = np.random.default_rng(31 * layers + 7 * m + chains + dims[0])
    dec, ref = build_decoder_packed(rng, layers, *dims, max_tokens=m)
    dec.set_chains(chains)
    xs = synth_activations(rng, m, dims[0])
    x_ref, q_ref, k_ref = oracle_stack(ref, xs, *dims)
    for _ in range(2):
        out, q, k = dec.decode(dev(xs), want_qk=True)
        assert np.array_equal(host(out), x_ref)
        assert np.array_equal(host(q), q_ref) and np.array_equal(host(k), k_ref)
    x = dev(xs)
    graph = dec.record(x, want_qk=True)
    for round_ in range(3):
        fresh = synth_activations(rng, m, dims[0])
        want, q_want, k_want = oracle_stack(ref, fresh, *dims)
        x.copy_(dev(fresh))
        graph.out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(host(graph.out), want), f"replay {round_}"
        assert np.array_equal(host(graph.q), q_want) and np.array_equal(host(graph.k), k_want)
        assert np.array_equal(host(dec.decode(dev(fresh))), want)  # eager work on the same decoder between the replays
    start = oracle_stack(ref[:1], xs, *dims)[0]
    buf = dev(start.copy())
    dec.decode(buf, out=buf, layers=(1, layers))
    assert np.array_equal(host(buf), x_ref)
    dec.set_chains(1)
    assert np.array_equal(host(dec.decode(dev(xs))), x_ref)
    with pytest.raises(bh.BitLinearError) as ei:
        dec.set_chains(9)
    assert ei.value.kind == "InvalidConfig"


def test_decoder_recorded_step_argument_errors():
    dec = bh.DecoderProjections(2, 256, 512, 4, 2, 64, max_tokens=2)
    x = torch.zeros((1, 256), device="cuda")
    with pytest.raises(bh.BitLinearError) as ei:  # no weights yet: nothing is recorded
        dec.record(x)
    assert ei.value.kind == "NotInitialized"
    with pytest.raises(bh.BitLinearError) as ei:
        dec.record(torch.zeros((3, 256), device="cuda"))
    assert ei.value.kind == "ShapeMismatch"
    with pytest.raises(bh.BitLinearError) as ei:
        dec.record(x, layers=(1, 1))
    assert ei.value.kind == "InvalidConfig"
    lib = bh.load_library()
    assert lib.bitnet_hip_decoder_graph_launch(None, None) == bh.NULL_POINTER
    lib.bitnet_hip_decoder_graph_destroy(None)


@pytest.mark.parametrize("layout", [bh.LAYOUT_OUT_IN, bh.LAYOUT_IN_OUT])
@pytest.mark.parametrize("n,k", [(1, 4), (48, 300), (640, 2560)])
def test_gguf_ternary_tensor_ingestion(n, k, layout):
    """A GGUF BitnetB158 tensor (8-byte header + 2-bit codes, either orientation, code 3 included) loaded straight
    into the layer: the layer then holds what the reference's decoder yields, and its forward matches the oracle."""
    rng = np.random.default_rng(n * 7 + k + layout)
    codes = rng.integers(0, 4, size=(n, k)).astype(np.uint8)  # code 3 decodes to 0 (gguf.rs:1139)
    if (n, k) == (1, 4):
        codes = np.array([[0, 1, 2, 0]], np.uint8)  # the reference's test vector 0x24 (gguf.rs:2421-2436)
    src = codes if layout == bh.LAYOUT_OUT_IN else codes.T
    flat = np.ascontiguousarray(src).reshape(-1)
    flat = np.concatenate([flat, np.zeros((-flat.size) % 4, np.uint8)])
    body = (flat[0::4] | (flat[1::4] << 2) | (flat[2::4] << 4) | (flat[3::4] << 6)).astype(np.uint8)
    scale = np.float32(0.0173)
    tensor = np.concatenate([np.frombuffer(np.array([scale, 0.5], "<f4").tobytes(), np.uint8), body])
    q_ref, s_ref, o_ref = orc.gguf_decode_ternary(tensor, n * k)
    w_ref = q_ref.reshape(src.shape) if layout == bh.LAYOUT_OUT_IN else q_ref.reshape(src.shape).T
    layer = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), "gguf")
    for data in (torch.from_numpy(tensor.copy()), dev(tensor)):
        got_scale, got_offset = layer.load_gguf_ternary(data, layout)
        assert (got_scale, got_offset) == (s_ref, o_ref)
        packed, ws = layer.get_quantized_weights()
        assert ws == s_ref
        assert np.array_equal(orc.unpack_2bit(packed.numpy(), n * k).reshape(n, k), w_ref)
    x = synth_activations(rng, 3, k)
    out = layer.forward(dev(x))
    ref = orc.bitlinear_forward(x, orc.pack_2bit(np.ascontiguousarray(w_ref).reshape(-1)), n, float(s_ref))[0]
    assert np.array_equal(host(out), ref)
    with pytest.raises(bh.BitLinearError) as ei:
        layer.load_gguf_ternary(torch.from_numpy(tensor[:-1].copy()), layout)
    assert ei.value.kind == "ShapeMismatch"


# ---- inference backend ---------------------------------------------------------------------------------------

def test_inference_backend_execute_batch_matches_per_input_oracle():
    """HipInferenceBackend (InferenceBackend, engine/mod.rs:126-138): a batch of inputs of different row counts, each
    result equal to the oracle's decoder chain on that input alone, however the inputs were grouped into passes."""
    dims = (256, 512, 4, 2, 64)
    rng = np.random.default_rng(77)
    dec, ref = build_decoder(rng, 2, *dims, max_tokens=8)
    backend = bh.create_backend("hip:0")
    caps = backend.capabilities()
    assert caps.supports_batching and not caps.supports_streaming and caps.max_batch_size == 0 and caps.device_type == "hip:0"
    assert backend.get_memory_usage() == 0
    with pytest.raises(bh.BitLinearError) as ei:
        backend.execute_batch([dev(synth_activations(rng, 1, dims[0]))])
    assert ei.value.kind == "NotInitialized"
    backend.optimize_model(dec)
    assert backend.capabilities().max_batch_size == 8 and backend.capabilities().memory_limit > 1 << 30
    assert backend.get_memory_usage() > dec.weight_bytes() * 2
    xs = [synth_activations(rng, r, dims[0]) for r in (1, 3, 2, 4, 8, 1, 1)]  # 1+3+2 | 4 | 8 | 1+1
    outs = backend.execute_batch([dev(x) for x in xs])
    assert len(outs) == len(xs)
    for x, o in zip(xs, outs):
        assert np.array_equal(host(o), oracle_stack(ref, x, *dims)[0])
    one = backend.execute_batch([dev(xs[0][0])])  # a rank-1 input is one row
    assert tuple(one[0].shape) == (dims[0],) and np.array_equal(host(one[0]), oracle_stack(ref, xs[0], *dims)[0][0])
    assert backend.execute_batch([]) == []
    with pytest.raises(bh.BitLinearError) as ei:
        backend.execute_batch([dev(synth_activations(rng, 9, dims[0]))])
    assert ei.value.kind == "ShapeMismatch"
    with pytest.raises(bh.BitLinearError) as ei:
        backend.execute_batch([dev(synth_activations(rng, 2, dims[0] + 4))])
    assert ei.value.kind == "ShapeMismatch"
    empty = bh.DecoderProjections(1, *dims, max_tokens=2)
    with pytest.raises(bh.BitLinearError) as ei:
        bh.HipInferenceBackend().optimize_model(empty)
    assert ei.value.kind == "NotInitialized"


# ---- C++ host mirror -----------------------------------------------------------------------------------------

def test_cpp_host_mirror_selftest():
    """bitnet-mlx.rs_amd/host/bitlinear.hpp (the C++ stand-in for the Rust types) against the reference's own
    BitLinear forward tests and against the other routes through the library."""
    import subprocess
    from pathlib import Path

    exe = Path(bh.LIB_PATH).parents[1] / "bin" / "host_selftest"
    assert exe.exists(), "build first: make -C bitnet-mlx.rs_amd"
    proc = subprocess.run([str(exe)], capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "all passed" in proc.stdout


def test_mfma_rate_diagnostic_is_plausible():
    """The matrix-unit loop bench.py quotes beside the prefill rates: between a tenth of and the published dense int8
    peak (5.0 POP/s), and constant operands are not slower than switching ones beyond run-to-run noise."""
    rand, const = bh.measure_mfma_i8_rate(True), bh.measure_mfma_i8_rate(False)
    assert 500.0 < rand < 5100.0 and 500.0 < const < 5100.0
    assert const > 0.9 * rand


def test_bitlinear_housekeeping_methods_of_the_reference():
    """clear_cache / cache_stats / to_device / device (layer.rs:223,353-411) and Quantizer::get_stats (weights.rs:638-640)
    as the reference's call sites use them: nothing to clear, the same device is a no-op, another device is refused."""
    layer = bh.BitLinear(bh.BitLinearConfig(in_features=64, out_features=32), "api")
    assert layer.clear_cache() is None and layer.cache_stats() is None
    assert layer.device.startswith("hip")
    assert layer.to_device(layer.device) is None and layer.to_device("cuda") is None
    with pytest.raises(bh.BitLinearError) as ei:
        layer.to_device("cpu")
    assert ei.value.kind == "DeviceError"
    stats = bh.BitNetWeightQuantizer().get_stats()
    assert (stats.elements_count, stats.quantization_error, stats.compression_ratio, stats.scale_factor, stats.zero_point) == (0, 0.0, 1.0, 1.0, None)


# ---- device diagnostics behind the C ABI -----------------------------------------------------------------------------------

def test_launch_chain_and_hand_over_diagnostics():
    """bitnet_hip_measure_launch_chain and bitnet_hip_measure_hop: plausible figures, argument checks, and the bounded
    waits of the hand-over kernel: with a spin limit of one look every wait gives up, the call reports that the vector did
    not arrive intact, and the kernel has ended normally (the next call on the device works)."""
    empty = bh.measure_launch_chain(60, replays=5)
    assert 10.0 < empty < 2000.0  # 60 dependent empty kernels: microseconds each, not nanoseconds and not milliseconds
    buf = torch.zeros(60 * 65536, dtype=torch.uint8, device="cuda")
    reads = bh.measure_launch_chain(60, replays=5, buf=buf, bytes_per_launch=[65536])
    assert reads >= 0.5 * empty
    with pytest.raises(bh.BitLinearError):
        bh.measure_launch_chain(61, replays=5, buf=buf, bytes_per_launch=[65536])  # needs more bytes than the buffer holds
    with pytest.raises(bh.BitLinearError):
        bh.measure_launch_chain(2, replays=5, buf=buf, bytes_per_launch=[24])
    for two_level in (False, True):
        us, intact = bh.measure_hop(640, hops=20, two_level=two_level)
        assert intact and 0.2 < us < 200.0
    us, intact = bh.measure_hop(2560, hops=8, two_level=False, spin_limit=1)
    assert not intact  # every wait gave up after one look; the kernel ended all the same
    us, intact = bh.measure_hop(640, hops=20)
    assert intact
    with pytest.raises(bh.BitLinearError):
        bh.measure_hop(0, hops=5)
