"""numpy-facing wrapper of the CPU oracle (oracle/libbitnet_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the benchmark's CPU-baseline
leg.  The shipped package never imports it.  Build the library with `make -C oracle`.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

_DIR = Path(__file__).resolve().parent
LIB_PATH = _DIR / "libbitnet_oracle.so"

SUM_SEQUENTIAL = 0
SUM_BLOCK256 = 1

_lib = None


def build():
    subprocess.run(["make", "-C", str(_DIR)], check=True, capture_output=True)


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        _lib = C.CDLL(str(LIB_PATH))
        _lib.orc_sum_squares.restype = C.c_float
        _lib.orc_absmean.restype = C.c_float
        _lib.orc_abs_max.restype = C.c_float
        _lib.orc_round_clip.restype = C.c_float
        _lib.orc_quantize_weights_reference.restype = C.c_float
        _lib.orc_pack_2bit.restype = C.c_size_t
        _lib.orc_packed_size.restype = C.c_size_t
        _lib.orc_gguf_decode_ternary.restype = C.c_size_t
        _lib.cpu_baseline_max_threads.restype = C.c_int
        _lib.cpu_baseline_isa.restype = C.c_int
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _sz(v):
    return C.c_size_t(int(v))


def sum_squares(x, order=SUM_BLOCK256) -> np.float32:
    x = _f32(x).reshape(-1)
    return np.float32(lib().orc_sum_squares(_p(x), _sz(x.size), C.c_int(order)))


def rmsnorm(x, g, eps, order=SUM_BLOCK256):
    x = _f32(x)
    g = _f32(g)
    m, k = x.shape
    y = np.empty_like(x)
    lib().orc_rmsnorm(_p(x), _p(g), C.c_float(eps), _sz(m), _sz(k), C.c_int(order), _p(y))
    return y


def quantize_activations_i8(x):
    """A1: returns (q int8 [m,k], a_scale f32 [m], row_sum int32 [m])."""
    x = _f32(x)
    m, k = x.shape
    q = np.empty((m, k), dtype=np.int8)
    s = np.empty((m,), dtype=np.float32)
    rs = np.empty((m,), dtype=np.int32)
    lib().orc_quantize_activations_i8(_p(x), _sz(m), _sz(k), _p(q), _p(s), _p(rs))
    return q, s, rs


def abs_max(x):
    x = _f32(x)
    return np.float32(lib().orc_abs_max(_p(x), _sz(x.size)))


def quantize_activations_scaled(x, precision, scale, reference_u8=False):
    """DynamicActivationQuantizer::quantize with a given scale: int8 values (the u8 bytes viewed as int8 with reference_u8)."""
    x = _f32(x)
    q = np.empty(x.shape, dtype=np.int8)
    lib().orc_quantize_activations_scaled(_p(x), _sz(x.size), C.c_int(precision), C.c_float(scale),
                                          C.c_int(1 if reference_u8 else 0), _p(q))
    return q


def fake_quantize_activations(x):
    x = _f32(x)
    m, k = x.shape
    out = np.empty_like(x)
    lib().orc_fake_quantize_activations(_p(x), _sz(m), _sz(k), _p(out))
    return out


def rmsnorm_quantize_i8(x, g, eps, order=SUM_BLOCK256):
    x = _f32(x)
    g = None if g is None else _f32(g)
    m, k = x.shape
    q = np.empty((m, k), dtype=np.int8)
    s = np.empty((m,), dtype=np.float32)
    rs = np.empty((m,), dtype=np.int32)
    lib().orc_rmsnorm_quantize_i8(_p(x), _p(g), C.c_float(eps), _sz(m), _sz(k), C.c_int(order), _p(q), _p(s), _p(rs))
    return q, s, rs


PRECISION_ONE_FIVE_FIVE_BIT, PRECISION_EIGHT_BIT = 0, 1


def absmax_quantize_activations(x, precision=PRECISION_ONE_FIVE_FIVE_BIT):
    """absmax_quantize_activations (activations.rs:530-641): returns (q int8 with x's shape, dict scale/mse/min/max)."""
    x = _f32(x)
    q = np.empty(x.shape, dtype=np.int8)
    stats = np.zeros(4, dtype=np.float32)
    lib().orc_absmax_quantize_activations(_p(x), _sz(x.size), C.c_int(int(precision)), _p(q), _p(stats))
    return q, dict(zip(("scale", "mse", "min", "max"), stats))


def round_clip(x, lo=-1.0, hi=1.0) -> float:
    return float(lib().orc_round_clip(C.c_float(x), C.c_float(lo), C.c_float(hi)))


def absmean(w) -> np.float32:
    w = _f32(w)
    if w.ndim == 1:
        w = w.reshape(1, -1)
    rows, cols = w.shape
    return np.float32(lib().orc_absmean(_p(w), _sz(rows), _sz(cols)))


def ternarize_roundclip(w, w_scale):
    w = _f32(w)
    q = np.empty(w.shape, dtype=np.int8)
    lib().orc_ternarize_roundclip(_p(w), _sz(w.size), C.c_float(w_scale), _p(q))
    return q


def ternarize_threshold(w, thr):
    w = _f32(w)
    q = np.empty(w.shape, dtype=np.int8)
    lib().orc_ternarize_threshold(_p(w), _sz(w.size), C.c_float(thr), _p(q))
    return q


def dequantize_ternary(q, scale):
    q = np.ascontiguousarray(q, dtype=np.int8)
    out = np.empty(q.shape, dtype=np.float32)
    lib().orc_dequantize_ternary(_p(q), _sz(q.size), C.c_float(scale), _p(out))
    return out


def quantize_weights_absmean(w):
    """BitNet b1.58 recipe: (q int8 [n,k], w_scale f32)."""
    w = _f32(w)
    s = absmean(w)
    return ternarize_roundclip(w, s), s


METHOD_MEAN, METHOD_MEDIAN, METHOD_ADAPTIVE, METHOD_OPTIMAL, METHOD_DETSTE = range(5)
WQ_STATS = ("mean", "sd", "clip_mean", "clip_mad", "lo", "hi", "mean_abs", "max_abs", "threshold", "num", "den", "scale")


def quantize_weights_reference(w, method=METHOD_MEAN, normalize=True, outlier_threshold=3.0, custom_factor=None,
                               want_details=False):
    """BitNetWeightQuantizer::quantize (weights.rs:568-611) on a 2-D f32 tensor; custom_factor None = method default.
    Returns (q, scale), or (q, scale, processed, stats dict) with want_details."""
    w = _f32(w)
    assert w.ndim == 2
    q = np.empty(w.shape, dtype=np.int8)
    processed = np.empty(w.shape, dtype=np.float32)
    stats = np.zeros(12, dtype=np.float32)
    s = lib().orc_quantize_weights_reference(_p(w), _sz(w.shape[0]), _sz(w.shape[1]), C.c_int(int(method)),
                                             C.c_int(int(normalize)), C.c_float(outlier_threshold),
                                             C.c_float(custom_factor if custom_factor else 0.0), _p(q), _p(processed),
                                             _p(stats))
    if want_details:
        return q, np.float32(s), processed, dict(zip(WQ_STATS, stats))
    return q, np.float32(s)


def pack_2bit(q):
    q = np.ascontiguousarray(q, dtype=np.int8).reshape(-1)
    out = np.empty(((q.size + 3) // 4,), dtype=np.uint8)
    lib().orc_pack_2bit(_p(q), _sz(q.size), _p(out))
    return out


def unpack_2bit(packed, n):
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    assert packed.size >= (n + 3) // 4
    q = np.empty((n,), dtype=np.int8)
    lib().orc_unpack_2bit(_p(packed), _sz(n), _p(q))
    return q


def lookup_compute(kind, w, x, nout=None):
    """TernaryLookupKernel / I2SLookupKernel::compute (bitnet-core/src/cpu/kernels/generic.rs:54-75,118-139);
    kind 0 = ternary, 1 = i2s.  Returns the output array (length nout, elements past min(len) left at zero) or None."""
    w = np.ascontiguousarray(w, dtype=np.int8).ravel()
    x = _f32(np.asarray(x).ravel())
    nout = min(w.size, x.size) if nout is None else nout
    out = np.zeros(nout, dtype=np.float32)
    rc = lib().orc_lookup_compute(C.c_int(kind), _p(w), _sz(w.size), _p(x), _sz(x.size), _p(out), _sz(nout))
    return None if rc != 0 else out


def pack_base3(q):
    """Base3PackedPacker::pack (packing.rs:424-447): 5 values per byte, value j weighs 3^j."""
    q = np.ascontiguousarray(q, dtype=np.int8).ravel()
    out = np.zeros((q.size + 4) // 5, dtype=np.uint8)
    lib().orc_pack_base3(_p(q), _sz(q.size), _p(out))
    return out


def unpack_base3(packed, count):
    """Base3PackedPacker::unpack (packing.rs:480-501)."""
    packed = np.ascontiguousarray(packed, dtype=np.uint8).ravel()
    assert packed.size * 5 >= count
    q = np.empty(count, dtype=np.int8)
    lib().orc_unpack_base3(_p(packed), _sz(count), _p(q))
    return q


def gguf_decode_ternary(data, count):
    """GgufLoader::decode_ternary_weights (gguf.rs:1089-1165): returns (q int8 [produced], scale, offset), or None
    where the reference reports "Insufficient packed data"."""
    data = np.ascontiguousarray(data, dtype=np.uint8)
    q = np.empty((max(count, 1),), dtype=np.int8)
    scale, offset = C.c_float(0), C.c_float(0)
    got = lib().orc_gguf_decode_ternary(_p(data), _sz(data.size), _sz(count), _p(q), C.byref(scale), C.byref(offset))
    if got == C.c_size_t(-1).value:
        return None
    return q[:got].copy(), scale.value, offset.value


def gemm_w2a8(packed, a, n_out):
    """acc int32 [m, n_out] from flat-packed [n_out, k] weights and int8 activations [m, k]."""
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    a = np.ascontiguousarray(a, dtype=np.int8)
    if a.ndim == 1:
        a = a.reshape(1, -1)
    m, k = a.shape
    assert packed.size >= (n_out * k + 3) // 4
    acc = np.empty((m, n_out), dtype=np.int32)
    lib().orc_gemm_w2a8(_p(packed), _p(a), _p(acc), _sz(m), _sz(n_out), _sz(k))
    return acc


def gemv_w2a8(packed, a, n_out):
    return gemm_w2a8(packed, np.asarray(a).reshape(1, -1), n_out)[0]


def gemm_ternary_i8(w, a):
    w = np.ascontiguousarray(w, dtype=np.int8)
    a = np.ascontiguousarray(a, dtype=np.int8)
    if a.ndim == 1:
        a = a.reshape(1, -1)
    n_out, k = w.shape
    m = a.shape[0]
    acc = np.empty((m, n_out), dtype=np.int32)
    lib().orc_gemm_ternary_i8(_p(w), _p(a), _p(acc), _sz(m), _sz(n_out), _sz(k))
    return acc


def epilogue(acc, w_scale, a_scale, bias=None, residual=None):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    m, n = acc.shape
    a_scale = _f32(a_scale)
    bias = None if bias is None else _f32(bias)
    residual = None if residual is None else _f32(residual)
    out = np.empty((m, n), dtype=np.float32)
    lib().orc_epilogue(_p(acc), C.c_float(w_scale), _p(a_scale), _p(bias), _p(residual), _sz(m), _sz(n), _p(out))
    return out


def bitlinear_forward(x, packed, n_out, w_scale, g=None, eps=1e-5, order=SUM_BLOCK256, bias=None, residual=None):
    """Returns (out f32 [m,n], q int8 [m,k], a_scale f32 [m], acc int32 [m,n])."""
    x = _f32(x)
    m, k = x.shape
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    g = None if g is None else _f32(g)
    bias = None if bias is None else _f32(bias)
    residual = None if residual is None else _f32(residual)
    out = np.empty((m, n_out), dtype=np.float32)
    q = np.empty((m, k), dtype=np.int8)
    a_scale = np.empty((m,), dtype=np.float32)
    acc = np.empty((m, n_out), dtype=np.int32)
    lib().orc_bitlinear_forward(_p(x), _sz(m), _sz(k), _p(g), C.c_float(eps), C.c_int(order), _p(packed), _sz(n_out),
                                C.c_float(w_scale), _p(bias), _p(residual), _p(out), _p(q), _p(a_scale), _p(acc))
    return out, q, a_scale, acc


def relu2_mul(gate, up):
    gate, up = _f32(gate), _f32(up)
    h = np.empty_like(gate)
    lib().orc_relu2_mul(_p(gate), _p(up), _sz(gate.size), _p(h))
    return h


def gqa_broadcast_v(v, q_heads, kv_heads, head_dim):
    v = _f32(v)
    m = v.shape[0]
    out = np.empty((m, q_heads * head_dim), dtype=np.float32)
    lib().orc_gqa_broadcast_v(_p(v), _sz(m), _sz(q_heads), _sz(kv_heads), _sz(head_dim), _p(out))
    return out


def decoder_layer(x, weights, w_scales, hidden, ffn, q_heads, kv_heads, head_dim, g_attn, g_ffn, eps=1e-5,
                  order=SUM_BLOCK256):
    """weights: 7 flat-packed u8 arrays (q,k,v,o,gate,up,down); returns (x_out, q, k)."""
    x = _f32(x)
    m = x.shape[0]
    ws = [np.ascontiguousarray(w, dtype=np.uint8) for w in weights]
    arr = (C.c_void_p * 7)(*[w.ctypes.data for w in ws])
    scales = (C.c_float * 7)(*[float(s) for s in w_scales])
    g_attn, g_ffn = _f32(g_attn), _f32(g_ffn)
    x_out = np.empty((m, hidden), dtype=np.float32)
    q = np.empty((m, hidden), dtype=np.float32)
    k = np.empty((m, kv_heads * head_dim), dtype=np.float32)
    lib().orc_decoder_layer(_p(x), _sz(m), _sz(hidden), _sz(ffn), _sz(q_heads), _sz(kv_heads), _sz(head_dim), _p(g_attn),
                            _p(g_ffn), C.c_float(eps), C.c_int(order), arr, scales, _p(x_out), _p(q), _p(k))
    return x_out, q, k


# ---- CPU baselines (timed by the benchmark, never used for results) ----------------------------------

def cpu_threads() -> int:
    return int(lib().cpu_baseline_max_threads())


def cpu_set_threads(n: int):
    lib().cpu_baseline_set_threads(C.c_int(n))


def cpu_isa() -> str:
    return {0: "scalar", 1: "avx2+fma", 2: "avx512f"}[int(lib().cpu_baseline_isa())]


def cpu_ref_f32_forward(x, q, scale, wf_scratch, out):
    m, k = x.shape
    n = q.shape[0]
    lib().cpu_ref_f32_forward(_p(x), _p(q), C.c_float(scale), None, _p(wf_scratch), _p(out), _sz(m), _sz(n), _sz(k))


def cpu_ref_simd_gemv(q, x, y, scale):
    m, k = x.shape
    n = q.shape[0]
    lib().cpu_ref_simd_gemv(_p(q), _p(x), _p(y), C.c_float(scale), _sz(m), _sz(n), _sz(k))
