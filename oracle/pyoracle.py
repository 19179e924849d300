"""ctypes binding of the CPU oracle (test infrastructure, never the product path).

Loads ``oracle/liboracle.so`` (built by ``oracle/Makefile``) and wraps each C
function with numpy in/out arrays.  Only tests, the smoke check and the CPU
baseline leg of the benchmark import this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

DTYPE_I8, DTYPE_U8, DTYPE_I16, DTYPE_I32, DTYPE_OTHER = range(5)
PER_TENSOR_AFFINE, PER_TENSOR_SYMMETRIC, PER_CHANNEL_AFFINE, PER_CHANNEL_SYMMETRIC = range(4)
ROUND_HALF_AWAY, ROUND_HALF_EVEN = 0, 1


class OracleError(ValueError):
    """Raised where the reference returns ``TorshError::InvalidArgument``."""


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (via its Makefile) and return the library path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


_f32p = C.POINTER(C.c_float)
_i32p = C.POINTER(C.c_int32)
_i8p = C.POINTER(C.c_int8)
_u8p = C.POINTER(C.c_uint8)
_szp = C.POINTER(C.c_size_t)


def _declare(l: C.CDLL) -> None:
    l.tq_time_roundtrip_c1.restype = C.c_double
    l.tq_time_matmul_rows.restype = C.c_double
    l.tq_nn_dequantize_value_asymmetric.restype = C.c_float
    l.tq_backend_dequantize_value.restype = C.c_float
    l.tq_qint8_quantize.restype = C.c_int8
    l.tq_quint8_quantize.restype = C.c_uint8
    for name in ("tq_nn_quantize_value_symmetric", "tq_nn_quantize_value_asymmetric", "tq_backend_quantize_value"):
        getattr(l, name).restype = C.c_int32
    l.tq_observer_new.restype = C.c_void_p
    l.tq_observer_new.argtypes = [C.c_int, C.c_size_t, C.c_float]
    for name in ("tq_observer_free", "tq_observer_reset"):
        getattr(l, name).restype = None
        getattr(l, name).argtypes = [C.c_void_p]
    l.tq_observer_update.argtypes = [C.c_void_p, _f32p, C.c_size_t]
    l.tq_observer_calculate_qparams.argtypes = [C.c_void_p, C.c_int, _f32p, _i32p]
    for name in ("tq_observer_get_min_max", "tq_observer_get_avg", "tq_observer_get_hist_range",
                 "tq_observer_histogram_range", "tq_observer_percentile_range"):
        getattr(l, name).restype = None
        getattr(l, name).argtypes = [C.c_void_p, _f32p, _f32p]
    for name in ("tq_observer_num_batches", "tq_observer_num_bins", "tq_observer_num_values"):
        getattr(l, name).restype = C.c_size_t
        getattr(l, name).argtypes = [C.c_void_p]
    l.tq_observer_histogram.restype = C.POINTER(C.c_uint64)
    l.tq_observer_histogram.argtypes = [C.c_void_p]
    l.tq_observer_values.restype = _f32p
    l.tq_observer_values.argtypes = [C.c_void_p]
    l.tq_value_to_bin_index.restype = C.c_size_t
    l.tq_value_to_bin_index.argtypes = [C.c_float, C.c_float, C.c_float, C.c_size_t]
    l.tq_histogram_accumulate.restype = None
    l.tq_histogram_accumulate.argtypes = [_f32p, C.c_size_t, C.c_float, C.c_float, C.c_size_t, C.POINTER(C.c_uint64)]
    l.tq_model_calculate_quantization_params.restype = None
    l.tq_model_calculate_quantization_params.argtypes = [C.c_float, C.c_float, C.c_int32, C.c_int32, _f32p, _i32p,
                                                         _f32p, _f32p]
    l.tq_fake_quantize_per_tensor_affine.restype = None
    l.tq_fake_quantize_per_tensor_affine.argtypes = [_f32p, C.c_size_t, C.c_float, C.c_int32, C.c_int32, C.c_int32, _f32p]
    l.tq_fake_quantize_auto.restype = C.c_int
    l.tq_fake_quantize_auto.argtypes = [_f32p, C.c_size_t, C.c_int, C.c_int, _f32p, C.POINTER(C.c_float),
                                        C.POINTER(C.c_int32)]
    l.tq_model_fake_quantize.restype = None
    l.tq_model_fake_quantize.argtypes = [_f32p, C.c_size_t, C.c_float, C.c_int32, C.c_int32, C.c_int32, _f32p]
    l.tq_quantize_int4_per_tensor.argtypes = [_f32p, C.c_size_t, _f32p, _f32p, _i32p]
    l.tq_quantize_int4_per_channel.argtypes = [_f32p, _szp, C.c_size_t, C.c_size_t, _f32p, _f32p, _i32p, _f32p, _i32p]
    l.tq_quantize_binary.argtypes = [_f32p, C.c_size_t, _f32p, _f32p, C.POINTER(C.c_double)]
    l.tq_quantize_ternary.argtypes = [_f32p, C.c_size_t, _f32p, _f32p, C.POINTER(C.c_double), _f32p]
    l.tq_quantize_binary_learned_threshold.argtypes = [_f32p, C.c_size_t, C.c_int, C.c_float, C.c_int, _f32p, _f32p,
                                                       C.POINTER(C.c_double), _f32p]
    l.tq_quantize_ternary_adaptive.argtypes = [_f32p, C.c_size_t, C.c_int, _f32p, _f32p, C.POINTER(C.c_double), _f32p,
                                               _f32p, C.POINTER(C.c_double)]
    l.tq_quantize_group_wise.argtypes = [_f32p, _szp, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int32, C.c_int32, _f32p,
                                         _f32p, _i32p, _f32p, _i32p]
    l.tq_model_mse_error.restype = C.c_double
    l.tq_model_mse_error.argtypes = [_f32p, _f32p, C.c_size_t]


def _p(a: np.ndarray, ty):
    return a.ctypes.data_as(ty)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise OracleError(f"{what}: invalid argument")


def set_round_mode(mode: int) -> None:
    lib().tq_set_round_mode(int(mode))


def num_threads() -> int:
    return int(lib().tq_num_threads())


def get_dtype_range(dtype: int):
    a, b = C.c_int32(), C.c_int32()
    lib().tq_get_dtype_range(int(dtype), C.byref(a), C.byref(b))
    return a.value, b.value


def find_min_max(x):
    x = _f32(x).ravel()
    mn, mx = C.c_float(), C.c_float()
    _check(lib().tq_find_min_max(_p(x, _f32p), C.c_size_t(x.size), C.byref(mn), C.byref(mx)), "find_min_max")
    return mn.value, mx.value


def min_max_fold(x):
    x = _f32(x).ravel()
    mn, mx = C.c_float(), C.c_float()
    lib().tq_min_max_fold(_p(x, _f32p), C.c_size_t(x.size), C.byref(mn), C.byref(mx))
    return mn.value, mx.value


def calculate_symmetric_params(mn, mx, dtype=DTYPE_I8):
    s, z = C.c_float(), C.c_int32()
    _check(lib().tq_calculate_symmetric_params(C.c_float(mn), C.c_float(mx), int(dtype), C.byref(s), C.byref(z)),
           "calculate_symmetric_quantization_params")
    return s.value, z.value


def calculate_affine_params(mn, mx, dtype=DTYPE_I8):
    s, z = C.c_float(), C.c_int32()
    _check(lib().tq_calculate_affine_params(C.c_float(mn), C.c_float(mx), int(dtype), C.byref(s), C.byref(z)),
           "calculate_affine_quantization_params")
    return s.value, z.value


def quantize_per_tensor_affine_simd(x, scale, zp):
    x = _f32(x)
    out = np.empty_like(x)
    _check(lib().tq_quantize_per_tensor_affine_simd(_p(x, _f32p), C.c_size_t(x.size), C.c_float(scale), int(zp),
                                                     _p(out, _f32p)), "quantize_per_tensor_affine_simd")
    return out


def quantize_to_int8_simd(x, scale, zp):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.int8)
    _check(lib().tq_quantize_to_int8_simd(_p(x, _f32p), C.c_size_t(x.size), C.c_float(scale), int(zp),
                                           _p(out, _i8p)), "quantize_to_int8_simd")
    return out


def quantize_cache_aware(x, scale, zp):
    """Element formula shared by the cache-aware, tiled, streaming and NEON quantizers (f32 carrier)."""
    x = _f32(x)
    out = np.empty_like(x)
    _check(lib().tq_quantize_cache_aware(_p(x, _f32p), C.c_size_t(x.size), C.c_float(scale), int(zp), _p(out, _f32p)),
           "quantize_cache_aware")
    return out


def quantize_mobile_optimized(x, scale, zp, reduced_precision=False):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.int8)
    _check(lib().tq_quantize_mobile_optimized(_p(x, _f32p), C.c_size_t(x.size), C.c_float(scale), int(zp),
                                              int(bool(reduced_precision)), _p(out, _i8p)), "quantize_mobile_optimized")
    return out


def calculate_tensor_stats_simd(x) -> dict:
    x = _f32(x)
    out = np.empty(5, dtype=np.float32)
    _check(lib().tq_calculate_tensor_stats_simd(_p(x, _f32p), C.c_size_t(x.size), _p(out, _f32p)),
           "calculate_tensor_stats_simd")
    return dict(zip(("min", "max", "mean", "std_dev", "variance"), out))


def calculate_tensor_stats_cache_optimized(x):
    """(min, max, mean, std_dev)"""
    x = _f32(x)
    out = np.empty(4, dtype=np.float32)
    _check(lib().tq_calculate_tensor_stats_cache_optimized(_p(x, _f32p), C.c_size_t(x.size), _p(out, _f32p)),
           "calculate_tensor_stats_cache_optimized")
    return tuple(out)


def quantize_per_tensor_affine(x, scale, zp):
    x = _f32(x)
    out = np.empty_like(x)
    _check(lib().tq_quantize_per_tensor_affine(_p(x, _f32p), C.c_size_t(x.size), C.c_float(scale), int(zp),
                                                _p(out, _f32p)), "quantize_per_tensor_affine")
    return out


def quantize_per_tensor_affine_i8(x, scale, zp):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.int8)
    _check(lib().tq_quantize_per_tensor_affine_i8(_p(x, _f32p), C.c_size_t(x.size), C.c_float(scale), int(zp),
                                                   _p(out, _i8p)), "quantize_per_tensor_affine_i8")
    return out


def dequantize_per_tensor_affine(q, scale, zp):
    q = _f32(q)
    out = np.empty_like(q)
    _check(lib().tq_dequantize_per_tensor_affine(_p(q, _f32p), C.c_size_t(q.size), C.c_float(scale), int(zp),
                                                  _p(out, _f32p)), "dequantize_per_tensor_affine")
    return out


def quantize_tensor_auto(x, dtype=DTYPE_I8, scheme=PER_TENSOR_SYMMETRIC):
    x = _f32(x)
    out = np.empty_like(x)
    s, z = C.c_float(), C.c_int32()
    _check(lib().tq_quantize_tensor_auto(_p(x, _f32p), C.c_size_t(x.size), int(dtype), int(scheme), _p(out, _f32p),
                                          C.byref(s), C.byref(z)), "quantize_tensor_auto")
    return out, s.value, z.value


def _shape_arr(shape):
    return (C.c_size_t * len(shape))(*[int(s) for s in shape])


def quantize_per_channel_auto(x, axis, dtype=DTYPE_I8, scheme=PER_CHANNEL_SYMMETRIC):
    x = _f32(x)
    out = np.empty_like(x)
    nch = x.shape[axis] if 0 <= axis < x.ndim else 1
    scales = np.empty(nch, dtype=np.float32)
    zps = np.empty(nch, dtype=np.int32)
    _check(lib().tq_quantize_per_channel_auto(_p(x, _f32p), _shape_arr(x.shape), C.c_size_t(x.ndim),
                                               C.c_size_t(axis), int(dtype), int(scheme), _p(out, _f32p),
                                               _p(scales, _f32p), _p(zps, _i32p)), "quantize_per_channel_auto")
    return out, scales, zps


def quantize_per_channel_simd(x, scales, zps, channel_size):
    x = _f32(x)
    scales = _f32(scales)
    zps = np.ascontiguousarray(zps, dtype=np.int32)
    out = np.empty_like(x)
    _check(lib().tq_quantize_per_channel_simd(_p(x, _f32p), C.c_size_t(x.size), _p(scales, _f32p), _p(zps, _i32p),
                                               C.c_size_t(scales.size), C.c_size_t(channel_size), _p(out, _f32p)),
           "quantize_per_channel_simd")
    return out


def quantize_per_channel_affine(x, scales, zps, axis):
    x = _f32(x)
    scales = _f32(scales)
    zps = np.ascontiguousarray(zps, dtype=np.int32)
    out = np.empty_like(x)
    _check(lib().tq_quantize_per_channel_affine(_p(x, _f32p), _shape_arr(x.shape), C.c_size_t(x.ndim),
                                                 C.c_size_t(axis), _p(scales, _f32p), _p(zps, _i32p),
                                                 C.c_size_t(scales.size), _p(out, _f32p)),
           "quantize_per_channel_affine")
    return out


def dequantize_per_channel_affine(q, scales, zps, axis):
    q = _f32(q)
    scales = _f32(scales)
    zps = np.ascontiguousarray(zps, dtype=np.int32)
    out = np.empty_like(q)
    _check(lib().tq_dequantize_per_channel_affine(_p(q, _f32p), _shape_arr(q.shape), C.c_size_t(q.ndim),
                                                   C.c_size_t(axis), _p(scales, _f32p), _p(zps, _i32p),
                                                   C.c_size_t(scales.size), _p(out, _f32p)),
           "dequantize_per_channel_affine")
    return out


def qint8_quantize(v, scale, zp):
    return int(lib().tq_qint8_quantize(C.c_float(v), C.c_float(scale), int(zp)))


def quint8_quantize(v, scale, zp):
    return int(lib().tq_quint8_quantize(C.c_float(v), C.c_float(scale), int(zp)))


def nn_quantize_value_symmetric(v, scale, qmin=-128, qmax=127):
    return int(lib().tq_nn_quantize_value_symmetric(C.c_float(v), C.c_float(scale), int(qmin), int(qmax)))


def nn_quantize_value_asymmetric(v, scale, zp, qmin, qmax):
    return int(lib().tq_nn_quantize_value_asymmetric(C.c_float(v), C.c_float(scale), int(zp), int(qmin), int(qmax)))


def nn_dequantize_value_asymmetric(q, scale, zp):
    return float(lib().tq_nn_dequantize_value_asymmetric(int(q), C.c_float(scale), int(zp)))


def nn_per_channel_quantize_weights_sym_i8(w):
    w = _f32(w)
    ch = w.shape[0]
    out = np.empty_like(w)
    scales = np.empty(ch, dtype=np.float32)
    lib().tq_nn_per_channel_quantize_weights_sym_i8(_p(w, _f32p), C.c_size_t(ch), C.c_size_t(w.size // max(ch, 1)),
                                                    _p(out, _f32p), _p(scales, _f32p))
    return out, scales


def nn_per_channel_quantize_weights_asym_u8(w):
    w = _f32(w)
    ch = w.shape[0]
    out = np.empty_like(w)
    scales = np.empty(ch, dtype=np.float32)
    zps = np.empty(ch, dtype=np.int32)
    lib().tq_nn_per_channel_quantize_weights_asym_u8(_p(w, _f32p), C.c_size_t(ch), C.c_size_t(w.size // max(ch, 1)),
                                                     _p(out, _f32p), _p(scales, _f32p), _p(zps, _i32p))
    return out, scales, zps


def backend_quantize_value(v, scale, zp, qmin=-128, qmax=127):
    return int(lib().tq_backend_quantize_value(C.c_float(v), C.c_float(scale), int(zp), int(qmin), int(qmax)))


def backend_dequantize_value(q, scale, zp):
    return float(lib().tq_backend_dequantize_value(int(q), C.c_float(scale), int(zp)))


def backend_params_symmetric(mn, mx, qmin=-128, qmax=127):
    s, z = C.c_float(), C.c_int32()
    _check(lib().tq_backend_params_symmetric(C.c_float(mn), C.c_float(mx), int(qmin), int(qmax), C.byref(s),
                                              C.byref(z)), "from_statistics(symmetric)")
    return s.value, z.value


def backend_params_asymmetric(mn, mx, qmin=0, qmax=255):
    s, z = C.c_float(), C.c_int32()
    _check(lib().tq_backend_params_asymmetric(C.c_float(mn), C.c_float(mx), int(qmin), int(qmax), C.byref(s),
                                               C.byref(z)), "from_statistics(asymmetric)")
    return s.value, z.value


def backend_quantize_f32(x, scales, zps, qmin, qmax):
    x = _f32(x)
    scales = _f32(np.atleast_1d(scales))
    zps = np.ascontiguousarray(np.atleast_1d(zps), dtype=np.int32)
    out = np.empty(x.shape, dtype=np.uint8)
    _check(lib().tq_backend_quantize_f32(_p(x, _f32p), C.c_size_t(x.size), _p(scales, _f32p), _p(zps, _i32p),
                                          C.c_size_t(scales.size), int(qmin), int(qmax), _p(out, _u8p)),
           "quantize_f32")
    return out


def backend_dequantize_f32(q, scales, zps, signed):
    q = np.ascontiguousarray(q).view(np.uint8)
    scales = _f32(np.atleast_1d(scales))
    zps = np.ascontiguousarray(np.atleast_1d(zps), dtype=np.int32)
    out = np.empty(q.shape, dtype=np.float32)
    _check(lib().tq_backend_dequantize_f32(_p(q, _u8p), C.c_size_t(q.size), _p(scales, _f32p), _p(zps, _i32p),
                                            C.c_size_t(scales.size), int(bool(signed)), _p(out, _f32p)),
           "dequantize_f32")
    return out


def backend_matmul_i32(a_bytes, b_kn_bytes):
    """Reference GEMM: A [M,K] bytes, B [K,N] bytes -> (i32 accumulators, clamped bytes)."""
    a = np.ascontiguousarray(a_bytes).view(np.uint8)
    b = np.ascontiguousarray(b_kn_bytes).view(np.uint8)
    m, k = a.shape
    k2, n = b.shape
    if k != k2:
        raise OracleError("qmatmul dimension mismatch")
    acc = np.empty((m, n), dtype=np.int32)
    cl = np.empty((m, n), dtype=np.uint8)
    lib().tq_backend_matmul_i32(_p(a, _u8p), _p(b, _u8p), C.c_size_t(m), C.c_size_t(k), C.c_size_t(n),
                                _p(acc, _i32p), _p(cl, _u8p))
    return acc, cl


def backend_conv2d_i32(x_q, zp_in, w_i8, stride=(1, 1), padding=(0, 0)):
    x_signed = x_q.dtype == np.int8
    xb = np.ascontiguousarray(x_q).view(np.uint8)
    w = np.ascontiguousarray(w_i8, dtype=np.int8)
    nb, c_in, h, wd = xb.shape
    c_out, c_in_w, kh, kw = w.shape
    if c_in != c_in_w:
        raise OracleError("qconv2d channel mismatch")
    ho = (h + 2 * padding[0] - kh) // stride[0] + 1
    wo = (wd + 2 * padding[1] - kw) // stride[1] + 1
    acc = np.empty((nb, c_out, ho, wo), dtype=np.int32)
    _check(lib().tq_backend_conv2d_i32(_p(xb, _u8p), int(x_signed), int(zp_in), _p(w, _i8p), C.c_size_t(nb),
                                        C.c_size_t(c_in), C.c_size_t(h), C.c_size_t(wd), C.c_size_t(c_out),
                                        C.c_size_t(kh), C.c_size_t(kw), C.c_size_t(stride[0]),
                                        C.c_size_t(stride[1]), C.c_size_t(padding[0]), C.c_size_t(padding[1]),
                                        _p(acc, _i32p)), "conv2d")
    return acc


def gemm_i8_nk(a_i8, w_nk_i8):
    a = np.ascontiguousarray(a_i8, dtype=np.int8)
    w = np.ascontiguousarray(w_nk_i8, dtype=np.int8)
    m, k = a.shape
    n, k2 = w.shape
    if k != k2:
        raise OracleError("gemm dimension mismatch")
    acc = np.empty((m, n), dtype=np.int32)
    lib().tq_gemm_i8_nk(_p(a, _i8p), _p(w, _i8p), C.c_size_t(m), C.c_size_t(n), C.c_size_t(k), _p(acc, _i32p))
    return acc


def linear_dequant_epilogue(acc, sa, sw, bias=None):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    m, n = acc.shape
    sa = _f32(np.atleast_1d(sa))
    sw = _f32(sw)
    per_row = int(sa.size > 1)
    out = np.empty((m, n), dtype=np.float32)
    b = _f32(bias) if bias is not None else None
    lib().tq_linear_dequant_epilogue(_p(acc, _i32p), C.c_size_t(m), C.c_size_t(n), _p(sa, _f32p), per_row,
                                     _p(sw, _f32p), _p(b, _f32p) if b is not None else None, _p(out, _f32p))
    return out


def requantize_epilogue(acc, sa, sw, bias, s_out, zp_out, qmin=-128, qmax=127, channel_axis_is_row=False, inner=1):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    rows, cols = acc.shape
    sa = _f32(np.atleast_1d(sa))
    sw = _f32(sw)
    per_row = int(sa.size > 1)
    out = np.empty((rows, cols), dtype=np.int8)
    b = _f32(bias) if bias is not None else None
    _check(lib().tq_requantize_epilogue(_p(acc, _i32p), C.c_size_t(rows), C.c_size_t(cols), _p(sa, _f32p), per_row,
                                         _p(sw, _f32p), _p(b, _f32p) if b is not None else None, C.c_float(s_out),
                                         int(zp_out), int(qmin), int(qmax), int(bool(channel_axis_is_row)),
                                         C.c_size_t(inner), _p(out, _i8p)), "requantize")
    return out


def layer_norm(x, gamma=None, beta=None, eps=1e-5):
    x = _f32(x)
    rows, cols = x.shape
    out = np.empty_like(x)
    g = _f32(gamma) if gamma is not None else None
    b = _f32(beta) if beta is not None else None
    lib().tq_layer_norm(_p(x, _f32p), C.c_size_t(rows), C.c_size_t(cols), _p(g, _f32p) if g is not None else None,
                        _p(b, _f32p) if b is not None else None, C.c_float(eps), _p(out, _f32p))
    return out


def gelu_tanh(x):
    x = _f32(x)
    out = np.empty_like(x)
    lib().tq_gelu_tanh(_p(x, _f32p), C.c_size_t(x.size), _p(out, _f32p))
    return out


def time_roundtrip_c1(x, reps=3):
    x = _f32(x).ravel()
    q = np.empty_like(x)
    y = np.empty_like(x)
    return float(lib().tq_time_roundtrip_c1(_p(x, _f32p), C.c_size_t(x.size), _p(q, _f32p), _p(y, _f32p), int(reps)))


def time_matmul_rows(a_bytes, b_kn_bytes, m_sample):
    a = np.ascontiguousarray(a_bytes).view(np.uint8)
    b = np.ascontiguousarray(b_kn_bytes).view(np.uint8)
    m, k = a.shape
    _, n = b.shape
    m_sample = min(int(m_sample), m)
    acc = np.empty((m_sample, n), dtype=np.int32)
    return float(lib().tq_time_matmul_rows(_p(a, _u8p), _p(b, _u8p), C.c_size_t(m_sample), C.c_size_t(k),
                                           C.c_size_t(n), _p(acc, _i32p)))


# ---- calibration observers, quality metrics, model-level fake quantization ----------------

OBS_MINMAX, OBS_MOVING_AVERAGE, OBS_HISTOGRAM, OBS_PERCENTILE, OBS_KL_DIVERGENCE, OBS_ENTROPY = range(6)

METRIC_FIELDS = ("mse", "psnr", "snr", "mae", "max_error", "zero_error_percentage", "cosine_similarity",
                 "compression_ratio")


class _Metrics(C.Structure):
    _fields_ = [(name, C.c_float) for name in METRIC_FIELDS]


def calculate_quantization_metrics(original, quantized, original_bits=32, quantized_bits=8) -> dict:
    """calculate_quantization_metrics (metrics.rs:67-175): sequential f32 sums, f32 results."""
    a, b = _f32(original).ravel(), _f32(quantized).ravel()
    if a.size != b.size:
        raise OracleError("calculate_quantization_metrics: shape mismatch")
    m = _Metrics()
    lib().tq_calculate_quantization_metrics(_p(a, _f32p), _p(b, _f32p), C.c_size_t(a.size), C.c_uint32(original_bits),
                                            C.c_uint32(quantized_bits), C.byref(m))
    return {name: np.float32(getattr(m, name)) for name in METRIC_FIELDS}


def calculate_quantization_metrics_f64(original, quantized, original_bits=32, quantized_bits=8) -> dict:
    """The same quantities with the sums carried in f64."""
    a, b = _f32(original).ravel(), _f32(quantized).ravel()
    out = (C.c_double * 8)()
    lib().tq_calculate_quantization_metrics_f64(_p(a, _f32p), _p(b, _f32p), C.c_size_t(a.size),
                                                C.c_uint32(original_bits), C.c_uint32(quantized_bits), out)
    return {name: float(out[i]) for i, name in enumerate(METRIC_FIELDS)}


class Observer:
    """Observer (observers.rs:36-556) driven through the C restatement."""

    def __init__(self, observer_type=OBS_MINMAX, num_bins=0, percentile=0.0):
        self._l = lib()
        self._h = self._l.tq_observer_new(int(observer_type), C.c_size_t(num_bins), C.c_float(percentile))

    def __del__(self):
        if getattr(self, "_h", None):
            self._l.tq_observer_free(self._h)
            self._h = None

    def update(self, x) -> None:
        x = _f32(x).ravel()
        _check(self._l.tq_observer_update(self._h, _p(x, _f32p), C.c_size_t(x.size)), "Observer::update")

    def calculate_qparams(self, dtype=DTYPE_I8):
        s, z = C.c_float(), C.c_int32()
        _check(self._l.tq_observer_calculate_qparams(self._h, int(dtype), C.byref(s), C.byref(z)),
               "Observer::calculate_qparams")
        return np.float32(s.value), z.value

    def reset(self) -> None:
        self._l.tq_observer_reset(self._h)

    def _pair(self, fn):
        a, b = C.c_float(), C.c_float()
        fn(self._h, C.byref(a), C.byref(b))
        return np.float32(a.value), np.float32(b.value)

    def get_min_max(self):
        return self._pair(self._l.tq_observer_get_min_max)

    def get_avg(self):
        return self._pair(self._l.tq_observer_get_avg)

    def get_hist_range(self):
        return self._pair(self._l.tq_observer_get_hist_range)

    def histogram_range(self):
        return self._pair(self._l.tq_observer_histogram_range)

    def percentile_range(self):
        return self._pair(self._l.tq_observer_percentile_range)

    def num_batches(self) -> int:
        return int(self._l.tq_observer_num_batches(self._h))

    def num_bins(self) -> int:
        return int(self._l.tq_observer_num_bins(self._h))

    def histogram(self) -> np.ndarray:
        n = self.num_bins()
        return np.ctypeslib.as_array(self._l.tq_observer_histogram(self._h), shape=(n,)).copy()

    def values(self) -> np.ndarray:
        n = int(self._l.tq_observer_num_values(self._h))
        if n == 0:
            return np.empty(0, dtype=np.float32)
        return np.ctypeslib.as_array(self._l.tq_observer_values(self._h), shape=(n,)).copy()


def value_to_bin_index(value, range_min, range_max, num_bins) -> int:
    return int(lib().tq_value_to_bin_index(C.c_float(value), C.c_float(range_min), C.c_float(range_max),
                                           C.c_size_t(num_bins)))


def histogram_accumulate(x, range_min, range_max, num_bins, counts=None) -> np.ndarray:
    x = _f32(x).ravel()
    counts = np.zeros(num_bins, dtype=np.uint64) if counts is None else np.ascontiguousarray(counts, dtype=np.uint64)
    lib().tq_histogram_accumulate(_p(x, _f32p), C.c_size_t(x.size), C.c_float(range_min), C.c_float(range_max),
                                  C.c_size_t(num_bins), _p(counts, C.POINTER(C.c_uint64)))
    return counts


def model_calculate_quantization_params(min_val, max_val, qmin=-128, qmax=127):
    """ModelQuantizer::calculate_quantization_params -> (scale, zero_point, adjusted_min, adjusted_max)."""
    s, z, a, b = C.c_float(), C.c_int32(), C.c_float(), C.c_float()
    lib().tq_model_calculate_quantization_params(C.c_float(min_val), C.c_float(max_val), qmin, qmax, C.byref(s),
                                                 C.byref(z), C.byref(a), C.byref(b))
    return np.float32(s.value), z.value, np.float32(a.value), np.float32(b.value)


def model_fake_quantize(x, scale, zp, qmin=-128, qmax=127) -> np.ndarray:
    x = _f32(x)
    out = np.empty_like(x)
    lib().tq_model_fake_quantize(_p(x, _f32p), C.c_size_t(x.size), C.c_float(scale), int(zp), qmin, qmax,
                                 _p(out, _f32p))
    return out


def fake_quantize_per_tensor_affine(x, scale, zp, qmin=-128, qmax=127) -> np.ndarray:
    x = _f32(x)
    out = np.empty_like(x)
    lib().tq_fake_quantize_per_tensor_affine(_p(x, _f32p), C.c_size_t(x.size), C.c_float(scale), int(zp), qmin, qmax,
                                             _p(out, _f32p))
    return out


def fake_quantize_auto(x, dtype=DTYPE_I8, scheme=0):
    """scheme 0 = PerTensorAffine, 1 = PerTensorSymmetric.  Returns (out, scale, zero_point)."""
    x = _f32(x)
    out = np.empty_like(x)
    s, z = C.c_float(), C.c_int32()
    _check(lib().tq_fake_quantize_auto(_p(x, _f32p), C.c_size_t(x.size), dtype, scheme, _p(out, _f32p), C.byref(s),
                                       C.byref(z)), "fake_quantize_auto")
    return out, float(s.value), int(z.value)


def model_mse_error(original, quantized) -> float:
    a, b = _f32(original).ravel(), _f32(quantized).ravel()
    return float(lib().tq_model_mse_error(_p(a, _f32p), _p(b, _f32p), C.c_size_t(a.size)))


# ---- special schemes (specialized.rs) ---------------------------------------------------------

def _shape(x):
    return (C.c_size_t * x.ndim)(*x.shape)


def quantize_int4_per_tensor(x):
    """-> (carrier, scale, zero_point)"""
    x = _f32(x)
    out = np.empty_like(x)
    s, z = C.c_float(), C.c_int32()
    lib().tq_quantize_int4_per_tensor(_p(x, _f32p), C.c_size_t(x.size), _p(out, _f32p), C.byref(s), C.byref(z))
    return out, np.float32(s.value), z.value


def quantize_int4_per_channel(x, axis):
    """-> (carrier, scales, zero_points, avg_scale, avg_zero_point)"""
    x = _f32(x)
    if axis >= x.ndim:
        raise OracleError("quantize_int4_per_channel: Axis out of bounds")
    ch = x.shape[axis]
    out = np.empty_like(x)
    scales, zps = np.empty(ch, np.float32), np.empty(ch, np.int32)
    s, z = C.c_float(), C.c_int32()
    _check(lib().tq_quantize_int4_per_channel(_p(x, _f32p), _shape(x), x.ndim, axis, _p(out, _f32p), _p(scales, _f32p),
                                              _p(zps, _i32p), C.byref(s), C.byref(z)), "quantize_int4_per_channel")
    return out, scales, zps, np.float32(s.value), z.value


def quantize_binary(x):
    """-> (carrier, scale, scale from an f64 sum)"""
    x = _f32(x)
    out = np.empty_like(x)
    s, d = C.c_float(), C.c_double()
    _check(lib().tq_quantize_binary(_p(x, _f32p), C.c_size_t(x.size), _p(out, _f32p), C.byref(s), C.byref(d)),
           "quantize_binary")
    return out, np.float32(s.value), d.value


def quantize_ternary(x):
    """-> (carrier, scale, scale from an f64 sum, threshold)"""
    x = _f32(x)
    out = np.empty_like(x)
    s, d, t = C.c_float(), C.c_double(), C.c_float()
    _check(lib().tq_quantize_ternary(_p(x, _f32p), C.c_size_t(x.size), _p(out, _f32p), C.byref(s), C.byref(d),
                                     C.byref(t)), "quantize_ternary")
    return out, np.float32(s.value), d.value, np.float32(t.value)


def quantize_binary_learned_threshold(x, threshold=None, f64_sums=False):
    """-> (carrier, scale, scale from an f64 sum, threshold used)"""
    x = _f32(x)
    out = np.empty_like(x)
    s, d, t = C.c_float(), C.c_double(), C.c_float()
    _check(lib().tq_quantize_binary_learned_threshold(_p(x, _f32p), C.c_size_t(x.size), int(threshold is not None),
                                                      C.c_float(threshold or 0.0), int(f64_sums), _p(out, _f32p),
                                                      C.byref(s), C.byref(d), C.byref(t)),
           "quantize_binary_learned_threshold")
    return out, np.float32(s.value), d.value, np.float32(t.value)


def quantize_ternary_adaptive(x, f64_sums=False):
    """-> (carrier, scale, scale from an f64 sum, threshold chosen, ten f32-sum errors, ten f64-sum errors)"""
    x = _f32(x)
    out = np.empty_like(x)
    s, d, t = C.c_float(), C.c_double(), C.c_float()
    e32, e64 = np.empty(10, np.float32), np.empty(10, np.float64)
    _check(lib().tq_quantize_ternary_adaptive(_p(x, _f32p), C.c_size_t(x.size), int(f64_sums), _p(out, _f32p),
                                              C.byref(s), C.byref(d), C.byref(t), _p(e32, _f32p),
                                              e64.ctypes.data_as(C.POINTER(C.c_double))), "quantize_ternary_adaptive")
    return out, np.float32(s.value), d.value, np.float32(t.value), e32, e64


def quantize_group_wise(x, axis, group_size, qmin=-128, qmax=127):
    """-> (carrier, group_scales, group_zero_points, avg_scale, avg_zero_point)"""
    x = _f32(x)
    if axis >= x.ndim or group_size == 0:
        raise OracleError("quantize_group_wise: invalid axis or group size")
    groups = -(-x.shape[axis] // group_size)
    out = np.empty_like(x)
    scales, zps = np.empty(groups, np.float32), np.empty(groups, np.int32)
    s, z = C.c_float(), C.c_int32()
    _check(lib().tq_quantize_group_wise(_p(x, _f32p), _shape(x), x.ndim, axis, group_size, qmin, qmax, _p(out, _f32p),
                                        _p(scales, _f32p), _p(zps, _i32p), C.byref(s), C.byref(z)), "quantize_group_wise")
    return out, scales, zps, np.float32(s.value), z.value


def backend_qadd(a, a_scale, a_zp, b, b_scale, b_zp, symmetric=False):
    """CpuQuantizationOps::qadd on int8 / uint8 arrays -> (bytes with a's dtype, scale, zero_point)."""
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    qmin, qmax = (-128, 127) if a.dtype == np.int8 else (0, 255)
    out = np.empty(a.shape, np.uint8)
    s, z = C.c_float(), C.c_int32()
    _check(lib().tq_backend_qadd_or_qrelu(a.ctypes.data_as(_u8p), int(a.dtype == np.int8), C.c_float(a_scale), int(a_zp),
                                          b.ctypes.data_as(_u8p), int(b.dtype == np.int8), C.c_float(b_scale), int(b_zp),
                                          C.c_size_t(a.size), int(symmetric), qmin, qmax, _p(out, _u8p), C.byref(s),
                                          C.byref(z)), "qadd")
    return out.view(a.dtype), np.float32(s.value), z.value


def backend_qrelu(q, scale, zp, symmetric=False):
    q = np.ascontiguousarray(q)
    qmin, qmax = (-128, 127) if q.dtype == np.int8 else (0, 255)
    out = np.empty(q.shape, np.uint8)
    s, z = C.c_float(), C.c_int32()
    _check(lib().tq_backend_qadd_or_qrelu(q.ctypes.data_as(_u8p), int(q.dtype == np.int8), C.c_float(scale), int(zp),
                                          None, 0, C.c_float(1.0), 0, C.c_size_t(q.size), int(symmetric), qmin, qmax,
                                          _p(out, _u8p), C.byref(s), C.byref(z)), "qrelu")
    return out.view(q.dtype), np.float32(s.value), z.value
