"""ctypes binding of libbitnet_hip.so (the C ABI declared in include/bitnet_hip.h).

The library is the product; this module only moves pointers.  torch is used for device memory and
streams, nothing else: no function here computes a result on the host or through torch operators, and
loading fails loudly if the HIP library has not been built.

Class and method names mirror the reference's Rust API so call sites read alike:
  BitLinearConfig / BitLinear      bitnet-quant/src/bitlinear/layer.rs:20-109, forward.rs:14-51
  TernaryProcessor                 bitnet-inference/src/engine/ternary_operations.rs:56-172
  BitPacked2BitPacker              bitnet-quant/src/quantization/packing.rs:350-394
  W2A8Backend.w2a8_gemv            bitnet-cuda/src/backend.rs:129-157
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass
from pathlib import Path
from typing import Optional, Sequence

import torch

_PKG_ROOT = Path(__file__).resolve().parents[2]
LIB_PATH = _PKG_ROOT / "lib" / "libbitnet_hip.so"
HEADER_PATH = _PKG_ROOT.parent / "include" / "bitnet_hip.h"

OK = 0
SHAPE_MISMATCH = 1
INVALID_CONFIG = 2
DEVICE_ERROR = 3
MEMORY_ERROR = 4
QUANTIZATION_ERROR = 5
NOT_INITIALIZED = 6
KERNEL_ERROR = 7
NULL_POINTER = 8
UNSUPPORTED = 9

SUM_SEQUENTIAL = 0
SUM_BLOCK256 = 1
LAYOUT_OUT_IN = 0
LAYOUT_IN_OUT = 1
TERNARY_ABSMEAN_ROUNDCLIP = 0
TERNARY_MEAN_THRESHOLD = 1
TERNARY_REF_MEAN_THRESHOLD = 2
TERNARY_REF_MEDIAN_THRESHOLD = 3
TERNARY_REF_ADAPTIVE_THRESHOLD = 4
TERNARY_REF_OPTIMAL_THRESHOLD = 5
TERNARY_REF_DETSTE = 6
INPUT_PLAIN = 0
INPUT_RELU2_MUL = 1
INPUT_GQA_BROADCAST = 2
PROJ_NAMES = ("q", "k", "v", "o", "gate", "up", "down")

_STATUS_NAMES = {
    1: "ShapeMismatch", 2: "InvalidConfig", 3: "DeviceError", 4: "MemoryError", 5: "QuantizationError",
    6: "NotInitialized", 7: "KernelError", 8: "NullPointer", 9: "Unsupported",
}


class BitLinearError(RuntimeError):
    """Mirror of BitLinearError (bitnet-quant/src/bitlinear/error.rs:10-84): `kind` is the variant name."""

    def __init__(self, status: int, message: str, expected=None, actual=None):
        super().__init__(f"{_STATUS_NAMES.get(status, status)}: {message}")
        self.status = status
        self.kind = _STATUS_NAMES.get(status, str(status))
        self.expected = expected
        self.actual = actual


_lib = None


def load_library() -> C.CDLL:
    """Loads the built library; raises if it is missing (there is no fallback path)."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is not built: run `make -C {_PKG_ROOT}` (needs hipcc); "
            "the BitLinear HIP path has no CPU or PyTorch fallback"
        )
    lib = C.CDLL(str(LIB_PATH))
    vp, sz, i32, f32 = C.c_void_p, C.c_size_t, C.c_int, C.c_float
    sig = {
        "bitnet_hip_last_error": (C.c_char_p, []),
        "bitnet_hip_last_shape_mismatch": (i32, [C.POINTER(sz), C.POINTER(sz), C.POINTER(i32)]),
        "bitnet_hip_init": (i32, [i32]),
        "bitnet_hip_device_info": (i32, [C.c_char_p, sz, C.POINTER(i32), C.POINTER(i32), C.POINTER(sz)]),
        "bitnet_hip_measure_mfma_i8_rate": (i32, [i32, C.POINTER(C.c_double), vp]),
        "bitnet_hip_measure_launch_chain": (i32, [vp, C.POINTER(sz), sz, sz, sz, C.POINTER(C.c_double), vp]),
        "bitnet_hip_measure_hop": (i32, [i32, sz, sz, i32, C.POINTER(C.c_double), C.POINTER(i32), vp]),
        "bitnet_hip_quantize_activations_i8": (i32, [vp, vp, sz, sz, sz, i32, sz, sz, vp, f32, i32, vp, vp, vp, vp, vp]),
        "bitnet_hip_absmax_quantize_activations": (i32, [vp, sz, i32, vp, vp, vp]),
        "bitnet_hip_abs_max": (i32, [vp, sz, C.POINTER(C.c_float), vp]),
        "bitnet_hip_quantize_activations_scaled": (i32, [vp, sz, i32, f32, i32, vp, vp]),
        "bitnet_hip_lookup_compute": (i32, [i32, vp, sz, vp, sz, vp, sz, vp]),
        "bitnet_hip_packed_size": (sz, [sz]),
        "bitnet_hip_pack_ternary_2bit": (i32, [vp, sz, vp, vp]),
        "bitnet_hip_unpack_ternary_2bit": (i32, [vp, sz, vp, vp]),
        "bitnet_hip_base3_packed_size": (sz, [sz]),
        "bitnet_hip_pack_ternary_base3": (i32, [vp, sz, vp, vp]),
        "bitnet_hip_unpack_ternary_base3": (i32, [vp, sz, vp, vp]),
        "bitnet_hip_base3_tiled_size": (sz, [sz, sz]),
        "bitnet_hip_retile_base3": (i32, [vp, sz, sz, vp, vp]),
        "bitnet_hip_gemv_base3": (i32, [vp, vp, sz, sz, vp, vp, vp, vp, vp]),
        "bitnet_hip_quantize_weights": (i32, [vp, sz, sz, i32, f32, vp, vp, vp, vp]),
        "bitnet_hip_quantize_weights_reference": (i32, [vp, sz, sz, i32, i32, f32, f32, vp, vp, vp, vp, vp]),
        "bitnet_hip_tiled_size": (sz, [sz, sz]),
        "bitnet_hip_retile_weights": (i32, [vp, sz, sz, i32, vp, vp]),
        "bitnet_hip_untile_weights": (i32, [vp, sz, sz, vp, vp]),
        "bitnet_hip_gemv_w2a8": (i32, [vp, vp, vp, sz, sz, vp]),
        "bitnet_hip_gemv_w2a8_checked": (i32, [vp, sz, vp, sz, vp, sz, sz, sz, vp]),
        "bitnet_hip_matmul_w2a8": (i32, [vp, vp, vp, sz, sz, sz, vp, vp, vp, vp, vp, vp, vp]),
        "bitnet_hip_bitlinear_create": (i32, [sz, sz, i32, C.POINTER(vp)]),
        "bitnet_hip_bitlinear_destroy": (None, [vp]),
        "bitnet_hip_bitlinear_set_weights_f32": (i32, [vp, vp, sz, sz, i32, i32, i32, f32, vp]),
        "bitnet_hip_bitlinear_set_weights_packed": (i32, [vp, vp, sz, f32, i32, vp]),
        "bitnet_hip_bitlinear_set_weights_base3": (i32, [vp, vp, sz, f32, i32, vp]),
        "bitnet_hip_bitlinear_set_weights_gguf": (i32, [vp, vp, sz, sz, sz, i32, i32, C.POINTER(C.c_float),
                                                  C.POINTER(C.c_float), vp]),
        "bitnet_hip_bitlinear_set_bias": (i32, [vp, vp, sz, i32, vp]),
        "bitnet_hip_bitlinear_get_quantized": (i32, [vp, C.POINTER(f32), vp, sz]),
        "bitnet_hip_bitlinear_workspace_size": (sz, [vp, sz]),
        "bitnet_hip_bitlinear_forward": (i32, [vp, vp, C.POINTER(sz), i32, vp, f32, i32, vp, vp, vp, sz, vp, vp, vp, vp]),
        "bitnet_hip_bitlinear_forward_noalloc": (i32, [vp, vp, C.POINTER(sz), i32, vp, f32, i32, vp, vp, vp]),
        "bitnet_hip_bitlinear_forward_multi": (i32, [C.POINTER(vp), sz, vp, sz, vp, f32, i32, C.POINTER(vp), vp, sz, vp]),
        "bitnet_hip_bitlinear_matmul": (i32, [vp, vp, vp, sz, vp, vp, vp, vp, vp]),
        "bitnet_hip_decoder_decode_layers": (i32, [vp, sz, sz, vp, sz, vp, vp, vp, vp]),
        "bitnet_hip_decoder_create": (i32, [sz, sz, sz, sz, sz, sz, f32, i32, sz, C.POINTER(vp)]),
        "bitnet_hip_decoder_destroy": (None, [vp]),
        "bitnet_hip_decoder_projection": (i32, [vp, sz, i32, C.POINTER(vp)]),
        "bitnet_hip_decoder_set_norm": (i32, [vp, sz, i32, vp, i32, vp]),
        "bitnet_hip_decoder_set_chains": (i32, [vp, sz]),
        "bitnet_hip_decoder_weight_bytes": (sz, [vp]),
        "bitnet_hip_decoder_decode": (i32, [vp, vp, sz, vp, vp, vp, vp]),
        "bitnet_hip_decoder_graph_create": (i32, [vp, sz, sz, vp, sz, vp, vp, vp, C.POINTER(vp)]),
        "bitnet_hip_decoder_graph_launch": (i32, [vp, vp]),
        "bitnet_hip_decoder_graph_destroy": (None, [vp]),
        "bitnet_hip_backend_create": (i32, [i32, C.POINTER(vp)]),
        "bitnet_hip_backend_destroy": (None, [vp]),
        "bitnet_hip_backend_optimize_model": (i32, [vp, vp]),
        "bitnet_hip_backend_execute_batch": (i32, [vp, C.POINTER(vp), C.POINTER(sz), sz, C.POINTER(vp), vp]),
        "bitnet_hip_backend_get_memory_usage": (sz, [vp]),
        "bitnet_hip_backend_capabilities": (i32, [vp, C.POINTER(i32), C.POINTER(i32), C.POINTER(sz), C.POINTER(sz), C.POINTER(i32)]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    lib._bitnet_declared = tuple(sig)
    _lib = lib
    return lib


def declared_symbols():
    """Entry points this binding declares; tests compare them with the header and with the library."""
    lib = load_library()
    return sorted(lib._bitnet_declared)


def _check(status: int):
    if status == OK:
        return
    lib = load_library()
    msg = lib.bitnet_hip_last_error().decode()
    expected = actual = None
    if status == SHAPE_MISMATCH:
        e = (C.c_size_t * 4)()
        a = (C.c_size_t * 4)()
        ar = C.c_int(0)
        er = lib.bitnet_hip_last_shape_mismatch(e, a, C.byref(ar))
        expected, actual = list(e[:er]), list(a[: ar.value])
    raise BitLinearError(status, msg, expected, actual)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream(stream=None):
    s = stream if stream is not None else torch.cuda.current_stream()
    return C.c_void_p(s.cuda_stream)


def _dev(t: torch.Tensor, dtype, name: str):
    if not t.is_cuda:
        raise BitLinearError(DEVICE_ERROR, f"{name} must live on the GPU")
    if t.dtype != dtype:
        raise BitLinearError(INVALID_CONFIG, f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise BitLinearError(INVALID_CONFIG, f"{name} must be contiguous")
    return t


def _opt_dev(t: Optional[torch.Tensor], dtype, name: str, numel: int, like: torch.Tensor):
    """An optional device operand: right device, dtype, contiguity and element count, or a BitLinearError."""
    if t is None:
        return None
    _dev(t, dtype, name)
    if t.device != like.device:
        raise BitLinearError(DEVICE_ERROR, f"{name} lives on {t.device}, the input on {like.device}")
    if t.numel() != numel:
        raise BitLinearError(SHAPE_MISMATCH, name, [numel], [t.numel()])
    return t


def _check_optional_operands(layer: "BitLinear", x: torch.Tensor, gamma, residual, out=None):
    """gamma [in], residual [m, out], out [.., out]: checked on the host so that a wrong tensor is a BitLinearError and
    never a wild pointer inside a kernel.  Shape errors of x itself are left to the library (it reports them as the
    reference does)."""
    nin, nout = layer.config.in_features, layer.config.out_features
    if x.dim() not in (2, 3) or x.shape[-1] != nin:
        return
    m = 1
    for d in x.shape[:-1]:
        m *= d
    _opt_dev(gamma, torch.float32, "gamma", nin, x)
    _opt_dev(residual, torch.float32, "residual", m * nout, x)
    if out is not None:
        _opt_dev(out, torch.float32, "out", m * nout, x)


def init(device: int = 0):
    _check(load_library().bitnet_hip_init(device))


def device_info():
    lib = load_library()
    name = C.create_string_buffer(64)
    cus, mhz, mem = C.c_int(0), C.c_int(0), C.c_size_t(0)
    _check(lib.bitnet_hip_device_info(name, 64, C.byref(cus), C.byref(mhz), C.byref(mem)))
    return {"arch": name.value.decode(), "compute_units": cus.value, "clock_mhz": mhz.value, "total_mem": mem.value}


def measure_mfma_i8_rate(random_operands: bool = True, stream=None) -> float:
    """10^12 int8 operations per second of a loop of nothing but v_mfma_i32_16x16x64_i8 on the current device (about
    2.5 ms): the practical ceiling of the prefill GEMM there.  random_operands: int8 activations and 2-bit codes that
    differ from lane to lane, as the GEMM's do; otherwise every operand byte is 1."""
    tops = C.c_double(0.0)
    _check(load_library().bitnet_hip_measure_mfma_i8_rate(1 if random_operands else 0, C.byref(tops), _stream(stream)))
    return tops.value


def measure_launch_chain(launches: int, replays: int = 20, buf: Optional[torch.Tensor] = None,
                         bytes_per_launch: Optional[Sequence[int]] = None, stream=None) -> float:
    """Microseconds per replay of a recorded chain of `launches` dependent kernel launches on the current device: kernels
    that do nothing (buf None), or kernels that only read bytes_per_launch[i % len] bytes of buf each, one region after
    the other (the floor of a decode step with that many launches and those bytes)."""
    us = C.c_double(0.0)
    if buf is None:
        _check(load_library().bitnet_hip_measure_launch_chain(None, None, 0, launches, replays, C.byref(us), _stream(stream)))
        return us.value
    if not buf.is_cuda or not buf.is_contiguous():
        raise BitLinearError(INVALID_CONFIG, "measure_launch_chain: buf must be a contiguous device tensor")
    sizes = [int(b) for b in (bytes_per_launch or [])]
    if not sizes or any(b <= 0 or b % 16 for b in sizes):
        raise BitLinearError(INVALID_CONFIG, "measure_launch_chain: bytes_per_launch must be positive multiples of 16")
    total = sum(sizes[i % len(sizes)] for i in range(launches))
    if total > buf.numel() * buf.element_size():
        raise BitLinearError(SHAPE_MISMATCH, "measure_launch_chain buffer", [total], [buf.numel() * buf.element_size()])
    arr = (C.c_size_t * len(sizes))(*sizes)
    _check(load_library().bitnet_hip_measure_launch_chain(_ptr(buf), arr, len(sizes), launches, replays, C.byref(us),
                                                          _stream(stream)))
    return us.value


def measure_hop(values: int, hops: int = 200, two_level: bool = False, spin_limit: int = 0, stream=None):
    """(microseconds per hand-over, intact) of a vector of `values` 32-bit values passed from step to step through memory
    inside ONE launch of resident workgroups (bitnet_hip_measure_hop); intact is False if a bounded wait ran out or the
    final values are wrong (spin_limit = 1 forces that: every wait gives up after one look and the kernel still ends)."""
    us, ok = C.c_double(0.0), C.c_int(0)
    _check(load_library().bitnet_hip_measure_hop(1 if two_level else 0, values, hops, spin_limit, C.byref(us), C.byref(ok),
                                                 _stream(stream)))
    return us.value, bool(ok.value)


# ---- raw operators ------------------------------------------------------------------------------

def quantize_activations_i8(x: torch.Tensor, gamma: Optional[torch.Tensor] = None, eps: float = 1e-5,
                            sum_order: int = SUM_BLOCK256, x2: Optional[torch.Tensor] = None,
                            input_mode: int = INPUT_PLAIN, gqa_group: int = 1, head_dim: int = 1,
                            want_sum: bool = False, want_y: bool = False, stream=None):
    """Fused RMSNorm (if gamma) + per-token absmax int8 quantisation of a [m, k] f32 matrix."""
    lib = load_library()
    _dev(x, torch.float32, "x")
    if x.dim() != 2:
        raise BitLinearError(SHAPE_MISMATCH, "x must be a [m, k] matrix", [1, x.shape[-1] if x.dim() else 1], list(x.shape))
    m, src_cols = x.shape
    k = src_cols * gqa_group if input_mode == INPUT_GQA_BROADCAST else src_cols
    _opt_dev(gamma, torch.float32, "gamma", k, x)
    _opt_dev(x2, torch.float32, "x2", x.numel(), x)
    q = torch.empty((m, k), dtype=torch.int8, device=x.device)
    a_scale = torch.empty((m,), dtype=torch.float32, device=x.device)
    a_sum = torch.empty((m,), dtype=torch.int32, device=x.device) if want_sum else None
    y = torch.empty((m, k), dtype=torch.float32, device=x.device) if want_y else None
    _check(lib.bitnet_hip_quantize_activations_i8(_ptr(x), _ptr(x2), src_cols, m, k, input_mode, gqa_group, head_dim,
                                                  _ptr(gamma), eps, sum_order, _ptr(q), _ptr(a_scale), _ptr(a_sum),
                                                  _ptr(y), _stream(stream)))
    return q, a_scale, a_sum, y


class QuantizationPrecision:
    """The precisions of QuantizationPrecision (bitnet-quant/src/quantization/mod.rs) that absmax_quantize_activations
    implements."""
    OneFiveFiveBit, EightBit = 0, 1


@dataclass
class QuantizedActivation:
    """QuantizedActivation (activations.rs:95-112): values (int8, the tensor's shape), scales (one f32 on the device),
    zero_points (None: symmetric), original_shape, stats (scale_factor, quantization_error, min_value, max_value,
    elements_count, compression_ratio), sequence_length (None)."""
    values: torch.Tensor
    scales: torch.Tensor
    zero_points: Optional[torch.Tensor]
    original_shape: tuple
    precision: int
    stats: dict
    sequence_length: Optional[int] = None

    def effective_bit_width(self) -> float:
        return 1.58 if self.precision == QuantizationPrecision.OneFiveFiveBit else 8.0

    def memory_footprint(self) -> int:
        return self.values.numel() * self.values.element_size() + self.scales.numel() * self.scales.element_size()


def absmax_quantize_activations(activations: torch.Tensor, precision: Optional[int] = None, stream=None) -> QuantizedActivation:
    """absmax_quantize_activations (activations.rs:530-641): ONE scale for the whole tensor, ternary codes by default
    (precision None = OneFiveFiveBit) or 8-bit values.  The values keep their sign (the reference's U8 cast of the 8-bit
    branch loses it).  The per-token int8 quantiser of the BitLinear path is quantize_activations_i8."""
    _dev(activations, torch.float32, "activations")
    precision = QuantizationPrecision.OneFiveFiveBit if precision is None else precision
    values = torch.empty(activations.shape, dtype=torch.int8, device=activations.device)
    stats = torch.empty((4,), dtype=torch.float32, device=activations.device)
    _check(load_library().bitnet_hip_absmax_quantize_activations(_ptr(activations), activations.numel(), precision,
                                                                 _ptr(values), _ptr(stats), _stream(stream)))
    scale, mse, lo, hi = stats.cpu().tolist()
    bits = 1.58 if precision == QuantizationPrecision.OneFiveFiveBit else 8.0
    info = {"elements_count": activations.numel(), "quantization_error": mse, "compression_ratio": 32.0 / bits,
            "min_value": lo, "max_value": hi, "scale_factor": scale, "zero_point": None}
    return QuantizedActivation(values, stats[0:1], None, tuple(activations.shape), precision, info)


class ActivationQuantizer:
    """The quantize / dequantize pair of ActivationQuantizer (activations.rs:169-199) over absmax_quantize_activations."""

    def __init__(self, precision: int = QuantizationPrecision.OneFiveFiveBit):
        self.precision = precision

    def validate_activations(self, activations: torch.Tensor):
        if activations.numel() == 0:
            raise BitLinearError(QUANTIZATION_ERROR, "Activation tensor is empty")
        if activations.dtype != torch.float32:
            raise BitLinearError(QUANTIZATION_ERROR, "Activation tensor must be float type")

    def quantize(self, activations: torch.Tensor) -> QuantizedActivation:
        self.validate_activations(activations)
        return absmax_quantize_activations(activations, self.precision)

    def quantize_dynamic(self, activations: torch.Tensor) -> QuantizedActivation:
        return self.quantize(activations)

    def dequantize(self, quantized: QuantizedActivation) -> torch.Tensor:
        """values * scales (a host-side convenience through torch; not on the forward path)."""
        return quantized.values.to(torch.float32) * quantized.scales


@dataclass
class ActivationQuantizationConfig:
    """ActivationQuantizationConfig (activations.rs:14-45) with its defaults; `precision` stands for base.precision
    (QuantizationConfig::default() is OneFiveFiveBit, as ActivationQuantizationConfig::bitnet())."""
    precision: int = QuantizationPrecision.OneFiveFiveBit
    moving_average_window: int = 100
    outlier_percentile: float = 99.9
    per_token: bool = False
    calibration_warmup: int = 50
    ema_decay: float = 0.99
    quantize_attention: bool = True

    def validate(self):
        """activations.rs:71-91."""
        if self.moving_average_window == 0:
            raise BitLinearError(INVALID_CONFIG, "Moving average window cannot be zero")
        if self.outlier_percentile <= 0.0 or self.outlier_percentile > 100.0:
            raise BitLinearError(INVALID_CONFIG, "Outlier percentile must be in range (0, 100]")
        if self.ema_decay < 0.0 or self.ema_decay > 1.0:
            raise BitLinearError(INVALID_CONFIG, "EMA decay must be in range [0, 1]")


class DynamicScaleState:
    """The host-side state of DynamicActivationQuantizer (activations.rs:203-267, 406-447, 456-493): the exponential moving
    average of the scale, the window of recent scales, the warm-up counter and the calibration flag.  Every operation is
    single-precision arithmetic in the reference's order; it touches no device."""

    def __init__(self, config: ActivationQuantizationConfig):
        self.config = config
        self.scale_history: list = []
        self.ema_scale = None
        self.calibrated = False
        self.step_count = 0
        self.calibration_samples = 0  # the reference keeps the tensors themselves and never reads them again

    def current_scale(self, abs_max) -> "np.float32":
        """compute_dynamic_scale's per-step scale (:245-249): abs_max / 1.0 for ternary, abs_max / 127.0 for 8-bit."""
        import numpy as np
        a = np.float32(abs_max)
        if self.config.precision == QuantizationPrecision.OneFiveFiveBit:
            return a / np.float32(1.0)
        if self.config.precision == QuantizationPrecision.EightBit:
            return a / np.float32(127.0)
        raise BitLinearError(UNSUPPORTED, f"UnsupportedPrecision({self.config.precision})")

    def update(self, abs_max) -> "np.float32":
        """update_dynamic_params (:420-433) for a tensor whose max |x| is abs_max; returns the moving average."""
        import numpy as np
        cur = self.current_scale(abs_max)
        decay = np.float32(self.config.ema_decay)
        if self.ema_scale is None:
            self.ema_scale = cur
        else:
            self.ema_scale = decay * self.ema_scale + (np.float32(1.0) - decay) * cur
        if len(self.scale_history) >= self.config.moving_average_window:
            self.scale_history.pop(0)
        self.scale_history.append(cur)
        if self.step_count <= self.config.calibration_warmup:
            if self.calibration_samples < self.config.calibration_warmup:
                self.calibration_samples += 1
        elif not self.calibrated:
            self.calibrated = True
        return self.ema_scale

    def calibrate(self, abs_maxima: Sequence[float]):
        """calibrate (:459-483): the scale becomes the abs-max at index floor(len * outlier_percentile / 100) of the sorted
        list (the last one if that index is past the end)."""
        import numpy as np
        if len(abs_maxima) == 0:
            raise BitLinearError(QUANTIZATION_ERROR, "Calibration data cannot be empty")
        scales = sorted(np.float32(v) for v in abs_maxima)
        idx = int(np.float32(len(scales)) * np.float32(self.config.outlier_percentile) / np.float32(100.0))
        self.ema_scale = scales[min(idx, len(scales) - 1)]
        self.calibrated = True

    def needs_calibration(self) -> bool:
        return (not self.calibrated) or self.step_count <= self.config.calibration_warmup

    def reset(self):
        self.scale_history.clear()
        self.ema_scale = None
        self.calibrated = False
        self.step_count = 0
        self.calibration_samples = 0


def abs_max(x: torch.Tensor, stream=None) -> float:
    """max |x| over the tensor, on the host (activations.abs().max_all().to_scalar())."""
    _dev(x, torch.float32, "x")
    out = C.c_float(0.0)
    _check(load_library().bitnet_hip_abs_max(_ptr(x), x.numel(), C.byref(out), _stream(stream)))
    return out.value


def quantize_activations_scaled(x: torch.Tensor, precision: int, scale: float, reference_u8: bool = False, stream=None) -> torch.Tensor:
    """DynamicActivationQuantizer::quantize with the scale given: int8 values (uint8 with reference_u8, the reference's
    literal clamp(0, 255) of its 8-bit branch)."""
    _dev(x, torch.float32, "x")
    values = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    _check(load_library().bitnet_hip_quantize_activations_scaled(_ptr(x), x.numel(), precision, float(scale),
                                                                 1 if reference_u8 else 0, _ptr(values), _stream(stream)))
    return values.view(torch.uint8) if reference_u8 and precision == QuantizationPrecision.EightBit else values


class DynamicActivationQuantizer:
    """DynamicActivationQuantizer (activations.rs:203-454) over the HIP path: the tensor work (abs-max, quantisation with
    the current scale) runs on the device, the state (DynamicScaleState) on the host as in the reference.
    reference_u8: give the 8-bit values as the reference does (u8 after clamp(0, 255): negative activations become 0)
    instead of signed int8."""

    def __init__(self, config: Optional[ActivationQuantizationConfig] = None, reference_u8: bool = False):
        self.config = config or ActivationQuantizationConfig()
        self.state = DynamicScaleState(self.config)
        self.reference_u8 = reference_u8

    # -- Quantizer ------------------------------------------------------------------------------------------------
    def validate_input(self, activations: torch.Tensor):
        if activations.dim() < 1:
            raise BitLinearError(QUANTIZATION_ERROR, "Activation tensor must have at least 1 dimension")
        if activations.dtype not in (torch.float32, torch.float16):
            raise BitLinearError(QUANTIZATION_ERROR, "Activation tensor must be float type")

    validate_activations = validate_input

    def quantize(self, activations: torch.Tensor) -> QuantizedActivation:
        """quantize (:315-360): the moving-average scale if there is one, else the tensor's own abs-max."""
        self.validate_input(activations)
        if self.config.precision not in (QuantizationPrecision.OneFiveFiveBit, QuantizationPrecision.EightBit):
            raise BitLinearError(UNSUPPORTED, f"UnsupportedPrecision({self.config.precision})")
        x = activations if activations.dtype == torch.float32 else activations.float()
        x = x.contiguous()
        scale = float(self.state.ema_scale) if self.state.ema_scale is not None else abs_max(x)
        values = quantize_activations_scaled(x, self.config.precision, scale, self.reference_u8)
        bits = 1.58 if self.config.precision == QuantizationPrecision.OneFiveFiveBit else 8.0
        stats = {"elements_count": activations.numel(), "scale_factor": scale, "compression_ratio": 32.0 / bits}
        scales = torch.tensor([scale], dtype=torch.float32, device=activations.device)
        return QuantizedActivation(values, scales, None, tuple(activations.shape), self.config.precision, stats)

    def dequantize(self, quantized: QuantizedActivation) -> torch.Tensor:
        """values * scales (:362-368); a convenience through torch, not on the forward path."""
        return quantized.values.to(torch.float32) * quantized.scales

    def get_stats(self) -> dict:
        return {"elements_count": 0, "scale_factor": 1.0}  # the reference never updates the quantizer's own stats field

    # -- ActivationQuantizer --------------------------------------------------------------------------------------
    def quantize_dynamic(self, activations: torch.Tensor) -> QuantizedActivation:
        self.state.step_count += 1
        self.update_dynamic_params(activations)
        return self.quantize(activations)

    def quantize_attention(self, attention_scores: torch.Tensor, sequence_length: int) -> QuantizedActivation:
        if not self.config.quantize_attention:
            raise BitLinearError(QUANTIZATION_ERROR, "Attention quantization is disabled")
        out = self.quantize(attention_scores)
        out.sequence_length = sequence_length
        return out

    def update_dynamic_params(self, activations: torch.Tensor):
        x = activations if activations.dtype == torch.float32 else activations.float()
        self.state.update(abs_max(x.contiguous()))

    def get_dynamic_scales(self) -> torch.Tensor:
        return torch.tensor(float(self.state.ema_scale) if self.state.ema_scale is not None else 1.0, dtype=torch.float32)

    def reset_dynamic_state(self):
        self.state.reset()

    # -- CalibrationQuantizer -------------------------------------------------------------------------------------
    def calibrate(self, data: Sequence[torch.Tensor]):
        self.state.calibrate([abs_max(t.float().contiguous()) for t in data])

    def needs_calibration(self) -> bool:
        return self.state.needs_calibration()

    def reset_calibration(self):
        self.reset_dynamic_state()


def create_activation_quantizer(config: ActivationQuantizationConfig) -> DynamicActivationQuantizer:
    """create_activation_quantizer (activations.rs:496-504): validates the configuration first."""
    config.validate()
    return DynamicActivationQuantizer(config)


def packed_size(count: int) -> int:
    return load_library().bitnet_hip_packed_size(count)


def tiled_size(n: int, k: int) -> int:
    return load_library().bitnet_hip_tiled_size(n, k)


def pack_ternary_2bit(q: torch.Tensor, stream=None) -> torch.Tensor:
    _dev(q, torch.int8, "q")
    out = torch.empty((packed_size(q.numel()),), dtype=torch.uint8, device=q.device)
    _check(load_library().bitnet_hip_pack_ternary_2bit(_ptr(q), q.numel(), _ptr(out), _stream(stream)))
    return out


def unpack_ternary_2bit(packed: torch.Tensor, count: int, stream=None) -> torch.Tensor:
    _dev(packed, torch.uint8, "packed")
    if packed.numel() < packed_size(count):
        raise BitLinearError(SHAPE_MISMATCH, "packed buffer too short", [packed_size(count)], [packed.numel()])
    out = torch.empty((count,), dtype=torch.int8, device=packed.device)
    _check(load_library().bitnet_hip_unpack_ternary_2bit(_ptr(packed), count, _ptr(out), _stream(stream)))
    return out


def base3_packed_size(count: int) -> int:
    return (count + 4) // 5


def pack_ternary_base3(q: torch.Tensor, stream=None) -> torch.Tensor:
    _dev(q, torch.int8, "q")
    out = torch.empty((base3_packed_size(q.numel()),), dtype=torch.uint8, device=q.device)
    _check(load_library().bitnet_hip_pack_ternary_base3(_ptr(q), q.numel(), _ptr(out), _stream(stream)))
    return out


def unpack_ternary_base3(packed: torch.Tensor, count: int, stream=None) -> torch.Tensor:
    _dev(packed, torch.uint8, "packed")
    if packed.numel() < base3_packed_size(count):
        raise BitLinearError(SHAPE_MISMATCH, "packed buffer too short", [base3_packed_size(count)], [packed.numel()])
    out = torch.empty((count,), dtype=torch.int8, device=packed.device)
    _check(load_library().bitnet_hip_unpack_ternary_base3(_ptr(packed), count, _ptr(out), _stream(stream)))
    return out


def base3_tiled_size(n: int, k: int) -> int:
    return load_library().bitnet_hip_base3_tiled_size(n, k)


def retile_base3(base3: torch.Tensor, n: int, k: int, stream=None) -> torch.Tensor:
    """The bytes Base3PackedPacker emits for the flat [n, k] tensor, re-ordered into the streaming layout of
    gemv_base3 (tiles of 16 rows x 320 columns)."""
    _dev(base3, torch.uint8, "base3")
    if base3.numel() < base3_packed_size(n * k):
        raise BitLinearError(SHAPE_MISMATCH, "base-3 buffer too short", [base3_packed_size(n * k)], [base3.numel()])
    out = torch.empty((base3_tiled_size(n, k),), dtype=torch.uint8, device=base3.device)
    _check(load_library().bitnet_hip_retile_base3(_ptr(base3), n, k, _ptr(out), _stream(stream)))
    return out


def gemv_base3(tiled: torch.Tensor, a: torch.Tensor, n: int, w_scale: Optional[torch.Tensor] = None,
               a_scale: Optional[torch.Tensor] = None, want_acc: bool = True, out: Optional[torch.Tensor] = None, stream=None):
    """One token against base-3 weights in their streaming layout: returns (acc int32 [n] or None, out f32 [n] or None)."""
    _dev(tiled, torch.uint8, "tiled")
    _dev(a, torch.int8, "a")
    k = a.numel()
    if tiled.numel() != base3_tiled_size(n, k):
        raise BitLinearError(SHAPE_MISMATCH, "base-3 tiles", [base3_tiled_size(n, k)], [tiled.numel()])
    _opt_dev(w_scale, torch.float32, "w_scale", 1, a)
    _opt_dev(a_scale, torch.float32, "a_scale", 1, a)
    acc = torch.empty((n,), dtype=torch.int32, device=a.device) if want_acc else None
    if out is None and w_scale is not None:
        out = torch.empty((n,), dtype=torch.float32, device=a.device)
    elif out is not None:
        _dev(out, torch.float32, "out")
        if out.numel() != n or w_scale is None:
            raise BitLinearError(SHAPE_MISMATCH, "gemv_base3 output (needs w_scale)", [n], [out.numel()])
    _check(load_library().bitnet_hip_gemv_base3(_ptr(tiled), _ptr(a), n, k, _ptr(w_scale), _ptr(a_scale), _ptr(acc), _ptr(out),
                                                _stream(stream)))
    return acc, out


def quantize_weights(w: torch.Tensor, method: int = TERNARY_ABSMEAN_ROUNDCLIP, threshold_factor: float = 0.5,
                     want_i8: bool = False, stream=None):
    """Ternarise + pack an [n, k] f32 matrix on the GPU.  Returns (packed u8, w_scale f32[1], q i8 or None)."""
    _dev(w, torch.float32, "w")
    n, k = w.shape
    packed = torch.empty((packed_size(n * k),), dtype=torch.uint8, device=w.device)
    w_scale = torch.empty((1,), dtype=torch.float32, device=w.device)
    q = torch.empty((n, k), dtype=torch.int8, device=w.device) if want_i8 else None
    _check(load_library().bitnet_hip_quantize_weights(_ptr(w), n, k, method, threshold_factor, _ptr(packed),
                                                      _ptr(w_scale), _ptr(q), _stream(stream)))
    return packed, w_scale, q


class TernaryMethod:
    """TernaryMethod (bitnet-quant/src/quantization/weights.rs:17-30)."""
    MeanThreshold, MedianThreshold, AdaptiveThreshold, OptimalThreshold, DetSTE = range(5)


@dataclass
class WeightQuantizationConfig:
    """The fields of WeightQuantizationConfig (weights.rs:58-95) that affect arithmetic, with its defaults."""
    normalize_weights: bool = True
    outlier_threshold: float = 3.0
    ternary_method: int = TernaryMethod.MeanThreshold
    custom_threshold_factor: Optional[float] = None

    def validate(self):
        """WeightQuantizationConfig::validate (weights.rs:120-150)."""
        if self.outlier_threshold < 0.0:
            raise BitLinearError(INVALID_CONFIG, "Outlier threshold cannot be negative")
        f = self.custom_threshold_factor
        if f is not None and (f <= 0.0 or f > 2.0):
            raise BitLinearError(INVALID_CONFIG, "Custom threshold factor must be in range (0, 2]")


WQ_STATS = ("mean", "sd", "clip_mean", "clip_mad", "lo", "hi", "mean_abs", "max_abs", "threshold", "num", "den", "scale")


@dataclass
class QuantizationStats:
    """QuantizationStats (bitnet-quant/src/quantization/mod.rs:118-148) with its defaults."""
    elements_count: int = 0
    quantization_error: float = 0.0
    compression_ratio: float = 1.0
    min_value: float = 0.0
    max_value: float = 0.0
    scale_factor: float = 1.0
    zero_point: Optional[int] = None


@dataclass
class QuantizedWeight:
    """QuantizedWeight (weights.rs:158-175): ternary values (int8, the reference stores them as f32 in a tensor),
    the scalar scale, the original shape; plus the packed bytes the BitLinear layer takes."""
    values: torch.Tensor
    scales: torch.Tensor
    original_shape: tuple
    packed: torch.Tensor
    stats: dict


class BitNetWeightQuantizer:
    """BitNetWeightQuantizer (weights.rs:341-611): quantize / dequantize on the GPU."""

    def __init__(self, config: Optional[WeightQuantizationConfig] = None):
        self.config = config or WeightQuantizationConfig()
        self.config.validate()

    def validate_input(self, weights: torch.Tensor):
        """weights.rs:625-639."""
        if weights.dim() < 2:
            raise BitLinearError(QUANTIZATION_ERROR, "Weight tensor must have at least 2 dimensions")
        if weights.dtype != torch.float32:
            raise BitLinearError(QUANTIZATION_ERROR, "Weight tensor must be float type")

    def quantize(self, weights: torch.Tensor, stream=None) -> QuantizedWeight:
        self.validate_input(weights)
        _dev(weights, torch.float32, "weights")
        n, k = weights.shape[0], weights.numel() // weights.shape[0]
        packed = torch.empty((packed_size(n * k),), dtype=torch.uint8, device=weights.device)
        w_scale = torch.empty((1,), dtype=torch.float32, device=weights.device)
        q = torch.empty(weights.shape, dtype=torch.int8, device=weights.device)
        stats = torch.empty((12,), dtype=torch.float32, device=weights.device)
        c = self.config
        _check(load_library().bitnet_hip_quantize_weights_reference(
            _ptr(weights), n, k, c.ternary_method, int(c.normalize_weights), c.outlier_threshold,
            c.custom_threshold_factor or 0.0, _ptr(packed), _ptr(w_scale), _ptr(q), _ptr(stats), _stream(stream)))
        return QuantizedWeight(q, w_scale, tuple(weights.shape), packed, dict(zip(WQ_STATS, stats.cpu().tolist())))

    def dequantize(self, quantized: QuantizedWeight) -> torch.Tensor:
        """weights.rs:616-619: values * scales (a host-side convenience through torch; not on the forward path)."""
        return quantized.values.to(torch.float32) * quantized.scales

    def get_stats(self) -> QuantizationStats:
        """Quantizer::get_stats (weights.rs:638-640): the quantizer's own record, which `quantize(&self)` never updates
        in the reference, so the defaults; the figures of a call are in QuantizedWeight.stats."""
        return QuantizationStats()


def retile_weights(packed: torch.Tensor, n: int, k: int, layout: int = LAYOUT_OUT_IN, stream=None) -> torch.Tensor:
    _dev(packed, torch.uint8, "packed")
    if packed.numel() < packed_size(n * k):
        raise BitLinearError(SHAPE_MISMATCH, "packed buffer too short", [packed_size(n * k)], [packed.numel()])
    tiled = torch.empty((tiled_size(n, k),), dtype=torch.uint8, device=packed.device)
    _check(load_library().bitnet_hip_retile_weights(_ptr(packed), n, k, layout, _ptr(tiled), _stream(stream)))
    return tiled


def untile_weights(tiled: torch.Tensor, n: int, k: int, stream=None) -> torch.Tensor:
    _dev(tiled, torch.uint8, "tiled")
    packed = torch.empty((packed_size(n * k),), dtype=torch.uint8, device=tiled.device)
    _check(load_library().bitnet_hip_untile_weights(_ptr(tiled), n, k, _ptr(packed), _stream(stream)))
    return packed


def matmul_w2a8(tiled: torch.Tensor, a: torch.Tensor, n: int, w_scale: Optional[torch.Tensor] = None,
                a_scale: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
                residual: Optional[torch.Tensor] = None, want_acc: bool = True, want_out: bool = True, stream=None,
                a_sum: Optional[torch.Tensor] = None):
    """acc[m,n] (int32) and/or out[m,n] (f32) from re-tiled weights and int8 activations [m, k]."""
    _dev(tiled, torch.uint8, "tiled")
    _dev(a, torch.int8, "a")
    if a.dim() != 2:
        raise BitLinearError(SHAPE_MISMATCH, "a must be a [m, k] matrix", [1, a.shape[-1] if a.dim() else 1], list(a.shape))
    m, k = a.shape
    if tiled.numel() < tiled_size(n, k):
        raise BitLinearError(SHAPE_MISMATCH, "tiled buffer too short", [tiled_size(n, k)], [tiled.numel()])
    _opt_dev(w_scale, torch.float32, "w_scale", 1, a)
    _opt_dev(a_scale, torch.float32, "a_scale", m, a)
    _opt_dev(a_sum, torch.int32, "a_sum", m, a)
    _opt_dev(bias, torch.float32, "bias", n, a)
    _opt_dev(residual, torch.float32, "residual", m * n, a)
    acc = torch.empty((m, n), dtype=torch.int32, device=a.device) if want_acc else None
    out = torch.empty((m, n), dtype=torch.float32, device=a.device) if want_out else None
    _check(load_library().bitnet_hip_matmul_w2a8(_ptr(tiled), _ptr(a), _ptr(a_sum), m, n, k, _ptr(acc), _ptr(w_scale), _ptr(a_scale),
                                                 _ptr(bias), _ptr(residual), _ptr(out), _stream(stream)))
    return acc, out


class W2A8Backend:
    """Mirror of CudaBackend's W2A8 entry (bitnet-cuda/src/backend.rs:129-157)."""

    def w2a8_gemv(self, weights: torch.Tensor, activations: torch.Tensor, output: torch.Tensor, m: int, k: int,
                  stream=None):
        _dev(weights, torch.uint8, "weights")
        _dev(activations, torch.int8, "activations")
        _dev(output, torch.int32, "output")
        _check(load_library().bitnet_hip_gemv_w2a8_checked(_ptr(weights), weights.numel(), _ptr(activations),
                                                           activations.numel(), _ptr(output), output.numel(), m, k,
                                                           _stream(stream)))


class BitPacked2BitPacker:
    """Mirror of BitPacked2BitPacker (bitnet-quant/src/quantization/packing.rs:350-394)."""

    def pack(self, weights: torch.Tensor) -> torch.Tensor:
        return pack_ternary_2bit(weights.reshape(-1))

    def unpack(self, packed: torch.Tensor, element_count: int) -> torch.Tensor:
        return unpack_ternary_2bit(packed, element_count)


LOOKUP_TERNARY, LOOKUP_I2S = 0, 1


class _HipLookupKernel:
    """compute(weights i8, inputs f32, output f32) on device tensors: output[i] = inputs[i] * lut[weights[i]] over the
    shortest of the three; any empty tensor is an error (bitnet-core/src/cpu/kernels/generic.rs:54-75,118-139)."""
    _kind = LOOKUP_TERNARY
    _name = ""

    def compute(self, weights: torch.Tensor, inputs: torch.Tensor, output: torch.Tensor, stream=None):
        for t, dt, nm in ((weights, torch.int8, "weights"), (inputs, torch.float32, "inputs"), (output, torch.float32, "output")):
            if t.numel():
                _dev(t, dt, nm)
        _check(load_library().bitnet_hip_lookup_compute(self._kind, _ptr(weights) if weights.numel() else None, weights.numel(),
                                                        _ptr(inputs) if inputs.numel() else None, inputs.numel(),
                                                        _ptr(output) if output.numel() else None, output.numel(), _stream(stream)))

    def name(self) -> str:
        return self._name

    def optimal_batch_size(self) -> int:
        return 1 << 20  # elements per call from which the launch cost is small beside the 9 bytes per element moved


class HipTernaryLookupKernel(_HipLookupKernel):
    """Mirror of TernaryLookupKernel (bitnet-core/src/cpu/mod.rs:132-149): weights in {-1, 0, +1}."""
    _kind, _name = LOOKUP_TERNARY, "HIP-gfx950-Ternary"


class HipI2SLookupKernel(_HipLookupKernel):
    """Mirror of I2SLookupKernel (bitnet-core/src/cpu/mod.rs:151-169): weights in {-2, -1, 0, +1}."""
    _kind, _name = LOOKUP_I2S, "HIP-gfx950-I2S"


class Base3PackedPacker:
    """Mirror of Base3PackedPacker (bitnet-quant/src/quantization/packing.rs:421-501): 5 values per byte."""

    def pack(self, weights: torch.Tensor) -> torch.Tensor:
        return pack_ternary_base3(weights.reshape(-1))

    def unpack(self, packed: torch.Tensor, element_count: int) -> torch.Tensor:
        return unpack_ternary_base3(packed, element_count)


class TernaryProcessor:
    """Mirror of TernaryProcessor (bitnet-inference/src/engine/ternary_operations.rs:56-172), int8 kept."""

    def quantize_activations(self, x: torch.Tensor):
        x2 = x.reshape(-1, x.shape[-1]) if x.dim() != 2 else x
        q, a_scale, _, _ = quantize_activations_i8(x2.contiguous())
        return q, a_scale


# ---- BitLinear ------------------------------------------------------------------------------------

@dataclass
class BitLinearConfig:
    """Subset of BitLinearConfig (layer.rs:20-75) that affects arithmetic."""
    in_features: int = 512
    out_features: int = 512
    use_bias: bool = False
    ternary_method: int = TERNARY_ABSMEAN_ROUNDCLIP
    threshold_factor: float = 0.5
    rms_norm_eps: float = 1e-5
    sum_order: int = SUM_BLOCK256


class BitLinear:
    """Mirror of BitLinear + BitLinearForward (layer.rs:82-109,113-179; forward.rs:14-136)."""

    def __init__(self, config: BitLinearConfig, layer_name: str = "", _handle=None, _owner=None):
        self.config = config
        self.layer_name = layer_name
        self._owner = _owner
        lib = load_library()
        if _handle is not None:
            self._h = _handle
            return
        h = C.c_void_p()
        _check(lib.bitnet_hip_bitlinear_create(config.in_features, config.out_features, int(config.use_bias), C.byref(h)))
        self._h = h

    def __del__(self):
        if getattr(self, "_owner", None) is None and getattr(self, "_h", None) and _lib is not None:
            _lib.bitnet_hip_bitlinear_destroy(self._h)
            self._h = None

    def update_weights(self, w: torch.Tensor, layout: int = LAYOUT_OUT_IN, stream=None):
        """BitLinear::update_weights (layer.rs:299-326): latent f32 weights, host or device."""
        if w.dtype != torch.float32 or w.dim() != 2 or not w.is_contiguous():
            raise BitLinearError(INVALID_CONFIG, "weights must be a contiguous 2-D f32 tensor")
        _check(load_library().bitnet_hip_bitlinear_set_weights_f32(
            self._h, _ptr(w), w.shape[0], w.shape[1], layout, int(w.is_cuda), self.config.ternary_method,
            self.config.threshold_factor, _stream(stream)))

    def set_quantized_weights(self, packed: torch.Tensor, w_scale: float, stream=None):
        if packed.dtype != torch.uint8 or not packed.is_contiguous():
            raise BitLinearError(INVALID_CONFIG, "packed weights must be contiguous u8")
        _check(load_library().bitnet_hip_bitlinear_set_weights_packed(self._h, _ptr(packed), packed.numel(), w_scale,
                                                                      int(packed.is_cuda), _stream(stream)))

    def set_base3_weights(self, packed: torch.Tensor, w_scale: float, stream=None):
        """Weights in the reference's base-3 byte format (Base3PackedPacker, packing.rs:421-501), [out, in] flat,
        host or device; re-coded once into the 2-bit tiles."""
        if packed.dtype != torch.uint8 or not packed.is_contiguous():
            raise BitLinearError(INVALID_CONFIG, "packed weights must be contiguous u8")
        _check(load_library().bitnet_hip_bitlinear_set_weights_base3(self._h, _ptr(packed), packed.numel(), w_scale,
                                                                     int(packed.is_cuda), _stream(stream)))

    def load_gguf_ternary(self, data: torch.Tensor, layout: int = LAYOUT_OUT_IN, stream=None):
        """A GGUF BitnetB158 tensor (8-byte scale/offset header + 2-bit codes, GgufLoader::decode_ternary_weights,
        gguf.rs:1089-1165) as a contiguous u8 tensor, host or device.  Returns (scale, offset) of the header."""
        if data.dtype != torch.uint8 or not data.is_contiguous():
            raise BitLinearError(INVALID_CONFIG, "GGUF tensor bytes must be contiguous u8")
        n, k = self.config.out_features, self.config.in_features
        rows, cols = (n, k) if layout == LAYOUT_OUT_IN else (k, n)
        scale, offset = C.c_float(0), C.c_float(0)
        _check(load_library().bitnet_hip_bitlinear_set_weights_gguf(self._h, _ptr(data), data.numel(), rows, cols, layout,
                                                                    int(data.is_cuda), C.byref(scale), C.byref(offset),
                                                                    _stream(stream)))
        return scale.value, offset.value

    def update_bias(self, bias: torch.Tensor, stream=None):
        if bias.dtype != torch.float32 or not bias.is_contiguous():
            raise BitLinearError(INVALID_CONFIG, "bias must be contiguous f32")
        _check(load_library().bitnet_hip_bitlinear_set_bias(self._h, _ptr(bias), bias.numel(), int(bias.is_cuda),
                                                            _stream(stream)))

    def get_quantized_weights(self):
        """(packed bytes as a CPU u8 tensor in the reference format, w_scale)."""
        n = packed_size(self.config.in_features * self.config.out_features)
        buf = torch.empty((n,), dtype=torch.uint8)
        s = C.c_float(0)
        _check(load_library().bitnet_hip_bitlinear_get_quantized(self._h, C.byref(s), _ptr(buf), n))
        return buf, s.value

    def forward(self, x: torch.Tensor, gamma: Optional[torch.Tensor] = None, residual: Optional[torch.Tensor] = None,
                debug: bool = False, stream=None, out: Optional[torch.Tensor] = None,
                workspace: Optional[torch.Tensor] = None):
        """BitLinearForward::forward (forward.rs:55-92).  x: [m,in] or [b,s,in] f32 on the GPU.  out and workspace
        (uint8, at least workspace_size(m) bytes) may be supplied by callers that must not allocate per call."""
        _dev(x, torch.float32, "input")
        _check_optional_operands(self, x, gamma, residual)
        lib = load_library()
        dims = (C.c_size_t * max(x.dim(), 1))(*x.shape)
        nout = self.config.out_features
        out_shape = tuple(x.shape[:-1]) + (nout,) if x.dim() >= 1 else (nout,)
        m = 1
        for d in x.shape[:-1]:
            m *= d
        if out is None:
            out = torch.empty(out_shape, dtype=torch.float32, device=x.device)
        else:
            _dev(out, torch.float32, "out")
            if tuple(out.shape) != tuple(out_shape) or not out.is_contiguous():
                raise BitLinearError(SHAPE_MISMATCH, "out", list(out_shape), list(out.shape))
        q = a_scale = acc = None
        if debug and x.dim() in (2, 3) and x.shape[-1] == self.config.in_features:
            q = torch.empty((m, self.config.in_features), dtype=torch.int8, device=x.device)
            a_scale = torch.empty((m,), dtype=torch.float32, device=x.device)
            acc = torch.empty((m, nout), dtype=torch.int32, device=x.device)
        # scratch for the quantised activations comes from torch's caching allocator (the library would otherwise
        # allocate stream-ordered memory itself on every call)
        ws_bytes = lib.bitnet_hip_bitlinear_workspace_size(self._h, m) if m > 0 else 0
        if workspace is not None:
            _dev(workspace, torch.uint8, "workspace")
            ws, ws_bytes = workspace, workspace.numel()  # the library checks the size
        else:
            ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=x.device) if ws_bytes else None
        _check(lib.bitnet_hip_bitlinear_forward(self._h, _ptr(x), dims, x.dim(), _ptr(gamma), self.config.rms_norm_eps,
                                                self.config.sum_order, _ptr(residual), _ptr(out), _ptr(ws), ws_bytes,
                                                _ptr(q), _ptr(a_scale), _ptr(acc), _stream(stream)))
        if debug:
            return out, q, a_scale, acc
        return out

    def forward_noalloc(self, x: torch.Tensor, out: torch.Tensor, gamma: Optional[torch.Tensor] = None,
                        residual: Optional[torch.Tensor] = None, stream=None):
        """forward() into a caller-supplied `out` with the quantised activations in the library's static per-GPU
        scratch: no device allocation by the library or by this method.  At most 4096 rows and
        rows * in_features <= 1,048,576 per call; calls that overlap on one GPU race."""
        _dev(x, torch.float32, "input")
        _dev(out, torch.float32, "out")
        _check_optional_operands(self, x, gamma, residual, out)
        dims = (C.c_size_t * max(x.dim(), 1))(*x.shape)
        _check(load_library().bitnet_hip_bitlinear_forward_noalloc(
            self._h, _ptr(x), dims, x.dim(), _ptr(gamma), self.config.rms_norm_eps, self.config.sum_order,
            _ptr(residual), _ptr(out), _stream(stream)))
        return out

    def workspace_size(self, m: int) -> int:
        """Bytes of scratch forward() needs for m token rows."""
        return int(load_library().bitnet_hip_bitlinear_workspace_size(self._h, m)) if m > 0 else 0

    def matmul_quantized(self, a: torch.Tensor, a_scale: torch.Tensor, residual: Optional[torch.Tensor] = None,
                         want_acc: bool = False, out: Optional[torch.Tensor] = None, stream=None,
                         a_sum: Optional[torch.Tensor] = None):
        """Contraction + epilogue on already-quantised activations (TernaryProcessor::ternary_matmul,
        ternary_operations.rs:87-113, minus its quantiser).  a: [m, in] int8, a_scale: [m] f32."""
        _dev(a, torch.int8, "a")
        if a.dim() != 2 or a.shape[1] != self.config.in_features:
            raise BitLinearError(SHAPE_MISMATCH, "activation width", [a.shape[0] if a.dim() else 1, self.config.in_features],
                                 list(a.shape))
        m = a.shape[0]
        _opt_dev(a_scale, torch.float32, "a_scale", m, a)
        _opt_dev(a_sum, torch.int32, "a_sum", m, a)
        _opt_dev(residual, torch.float32, "residual", m * self.config.out_features, a)
        if a_scale is None:
            raise BitLinearError(NULL_POINTER, "a_scale is required")
        if out is None:
            out = torch.empty((m, self.config.out_features), dtype=torch.float32, device=a.device)
        else:
            _opt_dev(out, torch.float32, "out", m * self.config.out_features, a)
        acc = torch.empty((m, self.config.out_features), dtype=torch.int32, device=a.device) if want_acc else None
        _check(load_library().bitnet_hip_bitlinear_matmul(self._h, _ptr(a), _ptr(a_sum), m, _ptr(a_scale), _ptr(residual), _ptr(acc),
                                                          _ptr(out), _stream(stream)))
        return (out, acc) if want_acc else out

    @property
    def device(self) -> str:
        """BitLinear::device (layer.rs:223): always the GPU the library was initialised on."""
        return f"hip:{torch.cuda.current_device()}" if torch.cuda.is_available() else "hip"

    def clear_cache(self):
        """BitLinear::clear_cache (layer.rs:353-361).  The reference caches the quantised weights of the latent f32
        tensor; here the layer holds nothing but the quantised weights (update_weights quantises at once), so there is
        no cache to clear and the call succeeds without effect."""
        return None

    def cache_stats(self):
        """BitLinear::cache_stats (layer.rs:364-368): None, as for a reference layer built without a cache."""
        return None

    def to_device(self, device) -> None:
        """BitLinear::to_device (layer.rs:376-411).  A layer lives on the one GPU this library drives: a move to that
        device is the reference's same-device no-op, anything else is refused."""
        name = str(device)
        if name in ("hip", "cuda", self.device, self.device.replace("hip", "cuda")):
            return None
        raise BitLinearError(DEVICE_ERROR, f"Failed to move weights to device: {name} (this layer lives on {self.device})")

    def forward_batch(self, x: torch.Tensor):
        """BitLinear::forward_batch (forward.rs:270-297): rank >= 2 required."""
        if x.dim() < 2:
            raise BitLinearError(SHAPE_MISMATCH, "forward_batch needs at least 2 dimensions",
                                 [1, 1, self.config.in_features], list(x.shape))
        return self.forward(x)


def forward_multi(layers: Sequence["BitLinear"], x: torch.Tensor, gamma: Optional[torch.Tensor] = None, stream=None):
    """Several BitLinear layers on one input [m, in] (q/k/v, gate/up): one activation quantisation, shared launches."""
    _dev(x, torch.float32, "input")
    if x.dim() != 2:
        raise BitLinearError(SHAPE_MISMATCH, "forward_multi takes a [m, in] input", [1, layers[0].config.in_features],
                             list(x.shape))
    m = x.shape[0]
    if x.shape[1] != layers[0].config.in_features:
        raise BitLinearError(SHAPE_MISMATCH, "last input dimension", [m, layers[0].config.in_features], list(x.shape))
    _opt_dev(gamma, torch.float32, "gamma", layers[0].config.in_features, x)
    outs = [torch.empty((m, l.config.out_features), dtype=torch.float32, device=x.device) for l in layers]
    hs = (C.c_void_p * len(layers))(*[l._h for l in layers])
    os_ = (C.c_void_p * len(layers))(*[o.data_ptr() for o in outs])
    cfg = layers[0].config
    _check(load_library().bitnet_hip_bitlinear_forward_multi(hs, len(layers), _ptr(x), m, _ptr(gamma), cfg.rms_norm_eps,
                                                             cfg.sum_order, os_, None, 0, _stream(stream)))
    return outs


class DecoderProjections:
    """The seven BitLinear projections of a stack of decoder blocks at decode time."""

    def __init__(self, layers: int, hidden: int = 2560, ffn: int = 6912, q_heads: int = 20, kv_heads: int = 5,
                 head_dim: int = 128, eps: float = 1e-5, sum_order: int = SUM_BLOCK256, max_tokens: int = 8):
        lib = load_library()
        h = C.c_void_p()
        _check(lib.bitnet_hip_decoder_create(layers, hidden, ffn, q_heads, kv_heads, head_dim, eps, sum_order,
                                             max_tokens, C.byref(h)))
        self._h = h
        self.layers, self.hidden, self.ffn = layers, hidden, ffn
        self.q_heads, self.kv_heads, self.head_dim = q_heads, kv_heads, head_dim
        self.kv_dim = kv_heads * head_dim
        self.eps, self.sum_order = eps, sum_order

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.bitnet_hip_decoder_destroy(self._h)
            self._h = None

    def proj_shape(self, proj: int):
        outs = (self.hidden, self.kv_dim, self.kv_dim, self.hidden, self.ffn, self.ffn, self.hidden)
        ins = (self.hidden,) * 6 + (self.ffn,)
        return outs[proj], ins[proj]

    def projection(self, layer: int, proj: int) -> BitLinear:
        h = C.c_void_p()
        _check(load_library().bitnet_hip_decoder_projection(self._h, layer, proj, C.byref(h)))
        n, k = self.proj_shape(proj)
        return BitLinear(BitLinearConfig(in_features=k, out_features=n, rms_norm_eps=self.eps,
                                         sum_order=self.sum_order), f"layer{layer}.{PROJ_NAMES[proj]}",
                         _handle=h, _owner=self)

    def set_norm(self, layer: int, which: int, gamma: torch.Tensor, stream=None):
        if gamma.dtype != torch.float32 or gamma.numel() != self.hidden or not gamma.is_contiguous():
            raise BitLinearError(SHAPE_MISMATCH, "norm weight", [self.hidden], list(gamma.shape))
        _check(load_library().bitnet_hip_decoder_set_norm(self._h, layer, which, _ptr(gamma), int(gamma.is_cuda),
                                                          _stream(stream)))

    def set_chains(self, chains: int):
        """Row groups a decode step of several token rows is split into (each a chain of launches on its own stream);
        0 and 1 keep all rows in one chain (the default, and the faster form on the device measured)."""
        _check(load_library().bitnet_hip_decoder_set_chains(self._h, int(chains)))

    def weight_bytes(self) -> int:
        return load_library().bitnet_hip_decoder_weight_bytes(self._h)

    def decode(self, x: torch.Tensor, out: Optional[torch.Tensor] = None, want_qk: bool = False, stream=None,
               layers: Optional[Sequence[int]] = None):
        """One decode step through all blocks, or through blocks layers[0] .. layers[1]-1 only."""
        _dev(x, torch.float32, "x")
        if x.dim() != 2 or x.shape[1] != self.hidden:
            raise BitLinearError(SHAPE_MISMATCH, "decode input", [x.shape[0] if x.dim() else 1, self.hidden], list(x.shape))
        m = x.shape[0]
        lo_hi = (0, self.layers) if layers is None else tuple(layers)
        if len(lo_hi) != 2 or not (0 <= lo_hi[0] <= lo_hi[1] <= self.layers):
            raise BitLinearError(INVALID_CONFIG, f"layer range {lo_hi} outside [0, {self.layers}]")
        if out is None:
            out = torch.empty_like(x)
        else:
            _dev(out, torch.float32, "out")
            if tuple(out.shape) != tuple(x.shape) or out.device != x.device:
                raise BitLinearError(SHAPE_MISMATCH, "decode output", list(x.shape), list(out.shape))
        q = torch.empty((m, self.hidden), dtype=torch.float32, device=x.device) if want_qk else None
        k = torch.empty((m, self.kv_dim), dtype=torch.float32, device=x.device) if want_qk else None
        lo, hi = (0, self.layers) if layers is None else layers
        _check(load_library().bitnet_hip_decoder_decode_layers(self._h, lo, hi, _ptr(x), m, _ptr(out), _ptr(q), _ptr(k),
                                                               _stream(stream)))
        return (out, q, k) if want_qk else out

    def record(self, x: torch.Tensor, out: Optional[torch.Tensor] = None, want_qk: bool = False,
               layers: Optional[Sequence[int]] = None) -> "DecoderGraph":
        """The decode step on these tensors recorded as a HIP graph (the step runs once while it is recorded); replay() then
        reads x and writes out in place, for the price of one host call instead of four launches a block."""
        _dev(x, torch.float32, "x")
        if x.dim() != 2 or x.shape[1] != self.hidden:
            raise BitLinearError(SHAPE_MISMATCH, "decode input", [x.shape[0] if x.dim() else 1, self.hidden], list(x.shape))
        lo_hi = (0, self.layers) if layers is None else tuple(layers)
        if len(lo_hi) != 2 or not (0 <= lo_hi[0] < lo_hi[1] <= self.layers):
            raise BitLinearError(INVALID_CONFIG, f"layer range {lo_hi} outside [0, {self.layers}] or empty")
        if out is None:
            out = torch.empty_like(x)
        else:
            _dev(out, torch.float32, "out")
            if tuple(out.shape) != tuple(x.shape) or out.device != x.device:
                raise BitLinearError(SHAPE_MISMATCH, "decode output", list(x.shape), list(out.shape))
        m = x.shape[0]
        q = torch.empty((m, self.hidden), dtype=torch.float32, device=x.device) if want_qk else None
        k = torch.empty((m, self.kv_dim), dtype=torch.float32, device=x.device) if want_qk else None
        h = C.c_void_p()
        _check(load_library().bitnet_hip_decoder_graph_create(self._h, lo_hi[0], lo_hi[1], _ptr(x), m, _ptr(out), _ptr(q),
                                                              _ptr(k), C.byref(h)))
        return DecoderGraph(h, self, x, out, q, k)


class DecoderGraph:
    """A recorded decode step (bitnet_hip_decoder_graph): keeps the decoder and the tensors it reads and writes alive."""

    def __init__(self, handle, decoder, x, out, q, k):
        self._h, self._decoder = handle, decoder
        self.x, self.out, self.q, self.k = x, out, q, k

    def replay(self, stream=None) -> torch.Tensor:
        _check(load_library().bitnet_hip_decoder_graph_launch(self._h, _stream(stream)))
        return self.out

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.bitnet_hip_decoder_graph_destroy(self._h)
            self._h = None


@dataclass
class BackendCapabilities:
    """BackendCapabilities (bitnet-inference/src/engine/mod.rs:141-148)."""
    supports_batching: bool
    supports_streaming: bool
    max_batch_size: int
    memory_limit: Optional[int]
    device_type: str


class HipInferenceBackend:
    """InferenceBackend (bitnet-inference/src/engine/mod.rs:126-138) for this path: execute_batch runs every input
    through the bound decoder stack; the model is bound with optimize_model."""

    def __init__(self, device: int = 0):
        h = C.c_void_p()
        _check(load_library().bitnet_hip_backend_create(device, C.byref(h)))
        self._h = h
        self._model = None

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.bitnet_hip_backend_destroy(self._h)
            self._h = None

    def optimize_model(self, model: "DecoderProjections"):
        _check(load_library().bitnet_hip_backend_optimize_model(self._h, model._h))
        self._model = model  # keeps the decoder alive while the backend refers to it

    def execute_batch(self, inputs: Sequence[torch.Tensor], stream=None):
        if self._model is None:  # the library reports it the way the trait's implementations do
            _check(load_library().bitnet_hip_backend_execute_batch(self._h, None, None, 0, None, _stream(stream)))
        hidden = self._model.hidden
        mats = []
        for i, t in enumerate(inputs):
            _dev(t, torch.float32, f"input {i}")
            t2 = t.reshape(1, -1) if t.dim() == 1 else t
            if t2.dim() != 2 or t2.shape[1] != hidden:
                raise BitLinearError(SHAPE_MISMATCH, f"input {i}", [t2.shape[0] if t2.dim() else 1, hidden], list(t.shape))
            mats.append(t2)
        outs = [torch.empty_like(t) for t in mats]
        n = len(mats)
        ins = (C.c_void_p * n)(*[t.data_ptr() for t in mats])
        rows = (C.c_size_t * n)(*[t.shape[0] for t in mats])
        ous = (C.c_void_p * n)(*[t.data_ptr() for t in outs])
        _check(load_library().bitnet_hip_backend_execute_batch(self._h, ins, rows, n, ous, _stream(stream)))
        return [o.reshape(t.shape) for o, t in zip(outs, inputs)]

    def get_memory_usage(self) -> int:
        return int(load_library().bitnet_hip_backend_get_memory_usage(self._h))

    def capabilities(self) -> BackendCapabilities:
        sb, ss, dv = C.c_int(0), C.c_int(0), C.c_int(0)
        mb, ml = C.c_size_t(0), C.c_size_t(0)
        _check(load_library().bitnet_hip_backend_capabilities(self._h, C.byref(sb), C.byref(ss), C.byref(mb), C.byref(ml), C.byref(dv)))
        return BackendCapabilities(bool(sb.value), bool(ss.value), mb.value, ml.value or None, f"hip:{dv.value}")


def create_backend(device: str = "hip:0") -> HipInferenceBackend:
    """InferenceEngine::create_backend (bitnet-inference/src/api/mod.rs:426-460) for a HIP device string "hip:N"."""
    if not device.startswith("hip"):
        raise BitLinearError(UNSUPPORTED, f"this library serves HIP devices only, not {device!r}")
    return HipInferenceBackend(int(device.split(":")[1]) if ":" in device else 0)
