"""The C-ABI library: it loads, exports exactly what include/bitnet_hip.h declares, the Python binding
declares the same set, and argument validation that needs no device behaves like the reference's
validation code.  No GPU needed (no kernel is launched)."""
import ctypes as C
import re
import subprocess

import pytest

import bitnet_hip as bh


def header_functions():
    text = bh.HEADER_PATH.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bitnet_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_is_built_and_loads():
    assert bh.LIB_PATH.exists(), "build the library first: make -C bitnet-mlx.rs_amd"
    assert bh.load_library() is not None


def test_exports_match_header_and_binding():
    declared = header_functions()
    assert len(declared) >= 25
    out = subprocess.run(["nm", "-D", "--defined-only", str(bh.LIB_PATH)], capture_output=True, text=True, check=True).stdout
    exported = sorted(set(re.findall(r" T (bitnet_hip_[a-z0-9_]+)", out)))
    assert exported == declared
    assert bh.declared_symbols() == declared
    lib = bh.load_library()
    for name in declared:
        assert getattr(lib, name) is not None


def test_library_carries_gfx950_code_only():
    blob = bh.LIB_PATH.read_bytes()
    targets = set(re.findall(rb"amdgcn-amd-amdhsa--(gfx[0-9a-z]+)", blob))
    assert targets == {b"gfx950"}


def test_sizes_match_reference_formulas():
    # (count + 3) / 4: bitnet-cuda/src/backend.rs:226, bitnet-inference/src/engine/weight_conversion.rs:151
    for count in (0, 1, 3, 4, 5, 2560 * 2560, 6912 * 2560):
        assert bh.packed_size(count) == (count + 3) // 4
    assert bh.packed_size(2560 * 2560) == 1_638_400
    assert bh.packed_size(640 * 2560) == 409_600
    assert bh.packed_size(6912 * 2560) == 4_423_680
    # tiles of 16 rows x 256 columns, 1 KiB each: no padding at the BitNet-2B shapes
    assert bh.tiled_size(2560, 2560) == 1_638_400
    assert bh.tiled_size(6912, 2560) == 4_423_680
    assert bh.tiled_size(2560, 6912) == 4_423_680
    assert bh.tiled_size(17, 257) == 2 * 2 * 1024
    assert bh.tiled_size(0, 10) == 0


def _last_error():
    return bh.load_library().bitnet_hip_last_error().decode()


def test_w2a8_dimension_validation_matches_reference_order():
    """validate_w2a8_dimensions (bitnet-cuda/src/backend.rs:217-257): weights, then activations, then output."""
    lib = bh.load_library()
    m, k = 8, 16
    dummy = C.c_void_p(0x1000)  # never dereferenced: validation fails first
    rc = lib.bitnet_hip_gemv_w2a8_checked(dummy, 31, dummy, k, dummy, m, m, k, None)
    assert rc == bh.SHAPE_MISMATCH and "weight bytes" in _last_error()
    e, a, ar = (C.c_size_t * 4)(), (C.c_size_t * 4)(), C.c_int()
    assert lib.bitnet_hip_last_shape_mismatch(e, a, C.byref(ar)) == 1
    assert (e[0], a[0], ar.value) == ((m * k + 3) // 4, 31, 1)
    rc = lib.bitnet_hip_gemv_w2a8_checked(dummy, 32, dummy, k + 1, dummy, m, m, k, None)
    assert rc == bh.SHAPE_MISMATCH and "activation" in _last_error()
    rc = lib.bitnet_hip_gemv_w2a8_checked(dummy, 32, dummy, k, dummy, m - 1, m, k, None)
    assert rc == bh.SHAPE_MISMATCH and "output" in _last_error()


def test_null_and_config_validation_without_device():
    lib = bh.load_library()
    dummy = C.c_void_p(0x1000)
    assert lib.bitnet_hip_gemv_w2a8(None, None, None, 4, 4, None) == bh.NULL_POINTER
    assert lib.bitnet_hip_gemv_w2a8(dummy, dummy, dummy, 0, 4, None) == bh.OK  # nothing to do
    assert lib.bitnet_hip_matmul_w2a8(None, dummy, None, 1, 1, 16, dummy, None, None, None, None, None, None) == bh.NULL_POINTER
    assert lib.bitnet_hip_matmul_w2a8(dummy, dummy, None, 1, 1, 16, None, None, None, None, None, None, None) == bh.NULL_POINTER
    # out without scales
    assert lib.bitnet_hip_matmul_w2a8(dummy, dummy, None, 1, 1, 16, None, None, None, None, None, dummy, None) == bh.NULL_POINTER
    # misaligned tiled buffer
    assert lib.bitnet_hip_matmul_w2a8(C.c_void_p(0x1004), dummy, None, 1, 1, 16, dummy, None, None, None, None, None, None) == bh.INVALID_CONFIG
    rc = lib.bitnet_hip_quantize_activations_i8(dummy, None, 16, 1, 16, 7, 1, 1, None, 1e-5, 1, dummy, dummy, None, None, None)
    assert rc == bh.INVALID_CONFIG and "input_mode" in _last_error()
    rc = lib.bitnet_hip_quantize_activations_i8(dummy, None, 16, 1, 16, 0, 1, 1, None, 1e-5, 5, dummy, dummy, None, None, None)
    assert rc == bh.INVALID_CONFIG and "sum_order" in _last_error()
    rc = lib.bitnet_hip_quantize_activations_i8(dummy, None, 16, 1, 16, bh.INPUT_RELU2_MUL, 1, 1, None, 1e-5, 1, dummy, dummy, None, None, None)
    assert rc == bh.NULL_POINTER
    rc = lib.bitnet_hip_quantize_activations_i8(dummy, None, 8, 1, 16, 0, 1, 1, None, 1e-5, 1, dummy, dummy, None, None, None)
    assert rc == bh.SHAPE_MISMATCH
    rc = lib.bitnet_hip_quantize_weights(dummy, 4, 4, 9, 0.5, dummy, dummy, None, None)
    assert rc == bh.INVALID_CONFIG
    h = C.c_void_p()
    assert lib.bitnet_hip_bitlinear_create(0, 4, 0, C.byref(h)) == bh.INVALID_CONFIG and not h.value
    assert lib.bitnet_hip_bitlinear_create(4, 4, 0, None) == bh.NULL_POINTER
    d = C.c_void_p()
    # q_heads * head_dim must equal hidden
    assert lib.bitnet_hip_decoder_create(1, 64, 96, 4, 2, 8, 1e-5, 1, 1, C.byref(d)) == bh.INVALID_CONFIG


def test_binding_rejects_host_tensors_loudly():
    import torch

    with pytest.raises(bh.BitLinearError) as ei:
        bh.quantize_activations_i8(torch.zeros(2, 16))
    assert ei.value.kind == "DeviceError"


class _FakeDeviceTensor:
    """Stands in for a CUDA tensor so that the binding's host-side checks can be exercised without a device: the checks
    must raise before any pointer reaches the library."""

    def __init__(self, shape, dtype, device="cuda:0", contiguous=True):
        import torch

        self._t = torch.zeros(shape, dtype=dtype)
        self.shape, self.dtype, self.is_cuda = self._t.shape, dtype, True
        self.device = torch.device(device)
        self._contig = contiguous

    def dim(self):
        return self._t.dim()

    def numel(self):
        return self._t.numel()

    def is_contiguous(self):
        return self._contig

    def data_ptr(self):
        raise AssertionError("a pointer was taken before validation finished")


def test_binding_validates_operands_before_any_pointer_reaches_a_kernel():
    """A wrong optional tensor (host memory, wrong dtype, too short, wrong shape, non-contiguous) is a BitLinearError raised
    by the binding, never a launch with a wild pointer."""
    import torch

    F = _FakeDeviceTensor
    f32, i8, i32 = torch.float32, torch.int8, torch.int32
    layer = bh.BitLinear.__new__(bh.BitLinear)
    layer.config, layer._h, layer._owner = bh.BitLinearConfig(in_features=16, out_features=8), None, object()
    x = F((2, 16), f32)
    cases = [
        lambda: layer.forward(x, gamma=torch.ones(16)),                      # gamma in host memory
        lambda: layer.forward(x, gamma=F((15,), f32)),                       # gamma too short
        lambda: layer.forward(x, gamma=F((16,), torch.float64)),             # wrong dtype
        lambda: layer.forward(x, residual=F((2, 7), f32)),                   # residual of the wrong size
        lambda: layer.forward(x, residual=F((2, 8), f32, device="cuda:1")),  # another device
        lambda: layer.forward_noalloc(x, F((2, 7), f32)),                    # out of the wrong size
        lambda: layer.matmul_quantized(F((2, 16), i8), F((3,), f32)),        # a_scale length
        lambda: layer.matmul_quantized(F((2, 16), i8), F((2,), f32), a_sum=F((2,), f32)),  # a_sum dtype
        lambda: layer.matmul_quantized(F((2, 15), i8), F((2,), f32)),        # activation width
        lambda: bh.quantize_activations_i8(F((2, 16), f32), gamma=F((8,), f32)),
        lambda: bh.quantize_activations_i8(F((2, 16), f32), x2=F((2, 8), f32), input_mode=bh.INPUT_RELU2_MUL),
        lambda: bh.quantize_activations_i8(F((16,), f32)),
        lambda: bh.quantize_activations_i8(F((2, 16), f32, contiguous=False)),
        lambda: bh.matmul_w2a8(F((1024,), torch.uint8), F((2, 16), i8), 8, a_scale=F((1,), f32)),
        lambda: bh.matmul_w2a8(F((1024,), torch.uint8), F((2, 16), i8), 8, bias=F((7,), f32)),
        lambda: bh.forward_multi([layer], x, gamma=F((4,), f32)),
    ]
    for i, case in enumerate(cases):
        with pytest.raises(bh.BitLinearError):
            case()
    dec = bh.DecoderProjections.__new__(bh.DecoderProjections)
    dec._h, dec.layers, dec.hidden, dec.kv_dim = None, 2, 16, 8
    for bad in (lambda: dec.decode(F((2, 15), f32)), lambda: dec.decode(F((16,), f32)),
                lambda: dec.decode(F((2, 16), f32), out=F((3, 16), f32)), lambda: dec.decode(F((2, 16), f32), layers=(1, 3)),
                lambda: dec.decode(F((2, 16), torch.float64))):
        with pytest.raises(bh.BitLinearError):
            bad()
    # the recorded step takes the same operands through the same checks
    for bad in (lambda: dec.record(F((2, 15), f32)), lambda: dec.record(F((16,), f32)),
                lambda: dec.record(F((2, 16), f32), out=F((3, 16), f32)), lambda: dec.record(F((2, 16), f32), layers=(1, 3)),
                lambda: dec.record(F((2, 16), f32), layers=(1, 1)), lambda: dec.record(F((2, 16), torch.float64)),
                lambda: dec.record(torch.zeros(2, 16))):
        with pytest.raises(bh.BitLinearError):
            bad()


def test_missing_library_is_an_error_not_a_fallback(monkeypatch, tmp_path):
    monkeypatch.setattr(bh, "_lib", None)
    monkeypatch.setattr(bh, "LIB_PATH", tmp_path / "libbitnet_hip.so")
    with pytest.raises(ImportError):
        bh.load_library()
