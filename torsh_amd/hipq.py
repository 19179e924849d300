"""ctypes binding of ``libtorsh_hipq.so`` for tests, the smoke check and the benchmark.

The binding is deliberately thin: every function forwards raw device pointers
(``torch.Tensor.data_ptr()``) to the C-ABI entry point of the same name and turns
a non-zero status into :class:`HipqError` carrying the library's last-error
string.  torch is used for device memory and streams only.  There is no
fallback: if the shared library is missing, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libtorsh_hipq.so")

SUCCESS, INVALID_ARGUMENT, SHAPE_ERROR, DIMENSION_MISMATCH, DEVICE_ERROR, ALLOCATION_ERROR, SYNCHRONIZATION_ERROR, UNKNOWN_ERROR = range(8)
ROUND_HALF_AWAY, ROUND_HALF_EVEN = 0, 1
ROUND_FLOOR_HALF_UP = 16  # hipq_quantize_per_tensor_f32_i8 only
FORM_MUL_INV, FORM_DIV = 0, 2
FORM_ZP_BEFORE_ROUND = 32  # round(x / scale + zp): the scalar quantized types of torsh-core
FORM_INT_CAST = 64         # (round(x / scale) as i32) + zp: torsh-nn's quantize_value_*; carrier output only
DTYPE_I8, DTYPE_U8 = 0, 1
PARAMS_SYMMETRIC, PARAMS_AFFINE, PARAMS_BACKEND_SYMMETRIC, PARAMS_BACKEND_ASYMMETRIC, PARAMS_ZERO_INCLUDED = range(5)
PARAMS_NN_SYMMETRIC, PARAMS_NN_ASYMMETRIC = 5, 6
FAKE_INT_CAST = 4
FAKE_NAN_TO_QMIN = 8
HISTOGRAM_MAX_BINS = 16384


class HipqError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"[hipq status {code}] {message}")
        self.code = code
        self.message = message


class BlockWeights(C.Structure):
    """hipq_block_weights: device pointers of one block of the projection stack."""
    _fields_ = [(n, C.c_void_p) for n in (
        "ln1_gamma", "ln1_beta", "ln2_gamma", "ln2_beta", "w_qkv", "s_qkv", "b_qkv", "w_out", "s_out", "b_out",
        "w_fc1", "s_fc1", "b_fc1", "w_fc2", "s_fc2", "b_fc2")]


class QParams(C.Structure):
    _fields_ = [("scale", C.c_float), ("zero_point", C.c_int32), ("min_val", C.c_float), ("max_val", C.c_float),
                ("status", C.c_int32), ("reserved", C.c_int32 * 3)]


class QuantMetrics(C.Structure):
    """hipq_quant_metrics: the fields of the reference's QuantizationMetrics, in its order."""
    _fields_ = [(n, C.c_float) for n in ("mse", "psnr", "snr", "mae", "max_error", "zero_error_percentage",
                                         "cosine_similarity", "compression_ratio")]

    def as_dict(self) -> dict:
        return {n: getattr(self, n) for n, _ in self._fields_}


class ObserveStats(C.Structure):
    _fields_ = [("min_val", C.c_float), ("max_val", C.c_float), ("nonfinite", C.c_uint64)]


class TensorStats(C.Structure):
    _fields_ = [("min_val", C.c_float), ("max_val", C.c_float), ("mean", C.c_float), ("std_dev", C.c_float),
                ("variance", C.c_float)]


_lib: Optional[C.CDLL] = None

_vp, _sz, _i32, _f32 = C.c_void_p, C.c_size_t, C.c_int32, C.c_float

# name -> argtypes (all return int32 status unless listed in _SPECIAL)
_SIGNATURES = {
    "hipq_ctx_create": [_i32, C.POINTER(_vp)],
    "hipq_ctx_create_on_stream": [_i32, _vp, C.POINTER(_vp)],
    "hipq_ctx_destroy": [_vp],
    "hipq_ctx_synchronize": [_vp],
    "hipq_device_malloc": [_vp, _sz, C.POINTER(_vp)],
    "hipq_device_free": [_vp, _vp],
    "hipq_memcpy_h2d": [_vp, _vp, _vp, _sz],
    "hipq_memcpy_d2h": [_vp, _vp, _vp, _sz],
    "hipq_minmax_f32": [_vp, _vp, _sz, _vp],
    "hipq_absmax_f32": [_vp, _vp, _sz, _vp],
    "hipq_qparams_from_minmax": [_vp, _vp, _i32, _i32, _i32, _vp],
    "hipq_quantize_per_tensor_f32_i8": [_vp, _vp, _sz, _f32, _i32, _i32, _vp],
    "hipq_quantize_per_tensor_f32_u8": [_vp, _vp, _sz, _f32, _i32, _i32, _vp],
    "hipq_quantize_per_tensor_f32_carrier": [_vp, _vp, _sz, _f32, _i32, _i32, _i32, _i32, _vp],
    "hipq_quantize_with_params_f32_i8": [_vp, _vp, _sz, _vp, _i32, _vp],
    "hipq_quantize_with_params_f32_u8": [_vp, _vp, _sz, _vp, _i32, _vp],
    "hipq_quantize_dynamic_per_tensor_f32": [_vp, _vp, _sz, _i32, _i32, _i32, _vp, _vp],
    "hipq_dequantize_i8_f32": [_vp, _vp, _sz, _f32, _i32, _vp],
    "hipq_dequantize_u8_f32": [_vp, _vp, _sz, _f32, _i32, _vp],
    "hipq_dequantize_carrier_f32": [_vp, _vp, _sz, _f32, _i32, _vp],
    "hipq_dequantize_with_params_i8_f32": [_vp, _vp, _sz, _vp, _vp],
    "hipq_quantize_per_row_f32_i8": [_vp, _vp, _sz, _sz, _i32, _i32, _vp, _vp, _vp, _vp],
    "hipq_quantize_per_channel_auto_f32_i8": [_vp, _vp, _sz, _sz, _sz, _i32, _i32, _vp, _vp, _vp, _vp],
    "hipq_quantize_per_group_auto_f32_i8": [_vp, _vp, _sz, _sz, _sz, _sz, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _vp],
    "hipq_quantize_binary_f32_i8": [_vp, _vp, _sz, _vp, _vp],
    "hipq_quantize_ternary_f32_i8": [_vp, _vp, _sz, _vp, _vp],
    "hipq_quantize_binary_learned_threshold_f32_i8": [_vp, _vp, _sz, _i32, _f32, _vp, _vp],
    "hipq_quantize_ternary_adaptive_f32_i8": [_vp, _vp, _sz, _vp, _vp],
    "hipq_quantize_per_channel_f32_i8": [_vp, _vp, _sz, _sz, _sz, _vp, _vp, _i32, _vp],
    "hipq_dequantize_per_channel_i8_f32": [_vp, _vp, _sz, _sz, _sz, _vp, _vp, _vp],
    "hipq_gemm_i8_i32": [_vp, _vp, _vp, _sz, _sz, _sz, _vp],
    "hipq_linear_i8_f32": [_vp, _vp, _vp, _i32, _vp, _vp, _vp, _sz, _sz, _sz, _vp],
    "hipq_linear_i8_i8": [_vp, _vp, _vp, _i32, _vp, _vp, _vp, _sz, _sz, _sz, _f32, _i32, _i32, _vp],
    "hipq_requantize_i32_i8": [_vp, _vp, _sz, _sz, _vp, _i32, _vp, _vp, _f32, _i32, _i32, _vp],
    "hipq_linear_dynamic_f32": [_vp, _vp, _i32, _vp, _vp, _vp, _sz, _sz, _sz, _i32, _vp],
    "hipq_linear_dynamic_f32_noalloc": [_vp, _vp, _i32, _vp, _vp, _vp, _sz, _sz, _sz, _i32, _vp],
    "hipq_pack_rows_i8": [_vp, _vp, _sz, _sz, _vp],
    "hipq_gemm_packed_i8_i32": [_vp, _vp, _vp, _sz, _sz, _sz, _vp],
    "hipq_linear_packed_i8_f32": [_vp, _vp, _vp, _i32, _vp, _vp, _vp, _sz, _sz, _sz, _vp],
    "hipq_linear_packed_i8_i8": [_vp, _vp, _vp, _i32, _vp, _vp, _vp, _sz, _sz, _sz, _f32, _i32, _i32, _vp],
    "hipq_quantize_per_tensor_packed_f32_i8": [_vp, _vp, _sz, _sz, _i32, _f32, _i32, _vp, _vp],
    "hipq_quantize_per_row_packed_f32_i8": [_vp, _vp, _sz, _sz, _i32, _vp, _vp],
    "hipq_linear_dynamic_packed_f32": [_vp, _vp, _i32, _vp, _vp, _vp, _sz, _sz, _sz, _i32, _vp],
    "hipq_linear_static_packed_f32": [_vp, _vp, _f32, _vp, _vp, _vp, _sz, _sz, _sz, _i32, _vp],
    "hipq_quantize_per_row_strided_f32_i8": [_vp, _vp, _sz, _sz, _sz, _i32, _i32, _vp, _vp, _vp, _vp],
    "hipq_linear_i8_f32_residual": [_vp, _vp, _vp, _i32, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp],
    "hipq_layer_norm_f32": [_vp, _vp, _sz, _sz, _vp, _vp, _f32, _vp],
    "hipq_quantize_static_per_tensor_f32_i8": [_vp, _vp, _sz, _f32, _i32, _i32, _vp, _vp],
    "hipq_set_gemm_kernel_variant": [_vp, _i32],
    "hipq_ctx_set_wait_spin_limit": [_vp, _i32],
    "hipq_ctx_set_resident_share": [_vp, _i32],
    "hipq_ctx_set_trace_buffer": [_vp, _vp, _sz],
    "hipq_probe_vector_memory_path": [_vp, _vp, _sz, _i32, _i32, _i32, _i32, _i32, _i32, _vp],
    "hipq_probe_buffer_range_check": [_vp, _vp, _sz, _i32, _i32, _vp],
    "hipq_linear_static_f32": [_vp, _vp, _f32, _vp, _vp, _vp, _sz, _sz, _sz, _i32, _vp],
    "hipq_layer_norm_quantize_f32_i8": [_vp, _vp, _sz, _sz, _vp, _vp, _f32, _i32, _vp, _vp],
    "hipq_add_layer_norm_quantize_f32_i8": [_vp, _vp, _vp, _sz, _sz, _vp, _vp, _f32, _i32, _vp, _vp],
    "hipq_gelu_tanh_f32": [_vp, _vp, _sz, _vp],
    "hipq_gelu_tanh_quantize_f32_i8": [_vp, _vp, _sz, _sz, _i32, _vp, _vp],
    "hipq_add_f32": [_vp, _vp, _vp, _sz, _vp],
    "hipq_linear_rows_packed_i8_f32": [_vp, _vp, _vp, _i32, _vp, _vp, _vp, _sz, _sz, _sz, _vp],
    "hipq_linear_gelu_quantize_packed_i8": [_vp, _vp, _vp, _i32, _vp, _vp, _vp, _sz, _sz, _sz, _i32, _vp, _vp],
    "hipq_linear_residual_layer_norm_quantize_packed_i8": [_vp, _vp, _vp, _i32, _vp, _vp, _vp, _sz, _sz, _sz, _vp, _vp,
                                                           _vp, _f32, _i32, _vp, _vp],
    "hipq_linear_from_f32_residual_layer_norm_quantize_packed_i8": [_vp, _vp, _sz, _vp, _vp, _vp, _sz, _sz, _sz, _vp, _vp,
                                                                    _vp, _f32, _i32, _vp, _vp],
    "hipq_transformer_stack_forward_f32": [_vp, _vp, _sz, _sz, _sz, _sz, _f32, _i32, _vp, _vp, _sz],
    "hipq_transformer_stack_forward_prepared_f32": [_vp, _vp, _sz, _sz, _sz, _sz, _f32, _i32, _vp, _vp, _sz],
    "hipq_qadd_u8": [_vp, _vp, _i32, _f32, _i32, _vp, _i32, _f32, _i32, _sz, _i32, _i32, _vp, _vp],
    "hipq_qrelu_u8": [_vp, _vp, _i32, _f32, _i32, _sz, _i32, _i32, _vp, _vp],
    "hipq_quantization_metrics_f32": [_vp, _vp, _vp, _sz, C.c_uint32, C.c_uint32, _vp],
    "hipq_fake_quantize_metrics_f32": [_vp, _vp, _sz, _f32, _i32, _vp, _i32, _i32, _i32, C.c_uint32, C.c_uint32, _vp],
    "hipq_fake_quantize_f32": [_vp, _vp, _sz, _f32, _i32, _vp, _i32, _i32, _i32, _vp],
    "hipq_observe_f32": [_vp, _vp, _sz, _vp],
    "hipq_tensor_stats_f32": [_vp, _vp, _sz, _i32, _vp],
    "hipq_histogram_f32": [_vp, _vp, _sz, _f32, _f32, _sz, _vp],
    "hipq_conv2d_u8i8_i32": [_vp, _vp, _i32, _vp] + [_sz] * 11 + [_vp],
    "hipq_conv2d_u8i8_i8": [_vp, _vp, _i32, _f32, _vp, _vp, _vp] + [_sz] * 11 + [_f32, _i32, _i32, _vp],
    "hipq_conv2d_u8i8_f32": [_vp, _vp, _i32, _f32, _vp, _vp, _vp] + [_sz] * 11 + [_vp],
    "hipq_conv2d_pack_weights_i8": [_vp, _vp, _sz, _sz, _sz, _sz, _vp, _vp],
    "hipq_conv2d_u8i8_i8_packed": [_vp, _vp, _i32, _f32, _vp, _vp, _vp, _vp] + [_sz] * 9 + [_f32, _i32, _i32, _vp],
    "hipq_conv2d_dynamic_f32_i8_packed": [_vp, _vp, _i32, _i32, _vp, _vp, _vp, _vp] + [_sz] * 9 +
                                         [_f32, _i32, _i32, _vp, _vp],
}

_SPECIAL = {
    "hipq_version": (C.c_char_p, []),
    "hipq_get_last_error": (C.c_char_p, []),
    "hipq_clear_last_error": (None, []),
    "hipq_has_error": (_i32, []),
    "hipq_ctx_stream": (_vp, [_vp]),
    "hipq_transformer_stack_workspace_bytes": (_sz, [_sz, _sz, _sz]),
    "hipq_transformer_stack_prepared_workspace_bytes": (_sz, [_sz, _sz, _sz]),
    "hipq_packed_size": (_i32, [_sz, _sz, C.POINTER(C.c_size_t)]),
    "hipq_conv2d_packed_weights_size": (_i32, [_sz, _sz, _sz, _sz, C.POINTER(C.c_size_t)]),
}


def exported_symbols() -> list[str]:
    """Every entry point ``include/torsh_hipq.h`` declares."""
    return sorted(list(_SIGNATURES) + list(_SPECIAL))


def lib_path() -> str:
    return _LIB_PATH


def load() -> C.CDLL:
    """Loads the shared library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise FileNotFoundError(
                f"{_LIB_PATH} is missing: build it with `python -m torsh_amd.build` (there is no CPU fallback)")
        lib = C.CDLL(_LIB_PATH)
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = _i32
        for name, (restype, argtypes) in _SPECIAL.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = lib
    return _lib


def last_error() -> str:
    return (load().hipq_get_last_error() or b"").decode()


def _check(code: int) -> None:
    if code != SUCCESS:
        raise HipqError(code, last_error())


def _ptr(t) -> Optional[int]:
    if t is None:
        return None
    if isinstance(t, int):
        return t
    if not t.is_contiguous():
        raise ValueError("hipq entry points take dense row-major tensors")
    return t.data_ptr()


class Context:
    """A ``hipq_ctx`` bound to a device; by default it enqueues on torch's current stream."""

    def __init__(self, device: int = 0, stream: Optional[torch.cuda.Stream] = None, own_stream: bool = False):
        self._lib = load()
        self.handle = _vp()
        self.device = device
        if own_stream:
            _check(self._lib.hipq_ctx_create(device, C.byref(self.handle)))
        else:
            st = stream if stream is not None else torch.cuda.current_stream(device)
            _check(self._lib.hipq_ctx_create_on_stream(device, _vp(st.cuda_stream), C.byref(self.handle)))

    def close(self) -> None:
        if self.handle:
            self._lib.hipq_ctx_destroy(self.handle)
            self.handle = _vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def call(self, name: str, *args) -> None:
        _check(getattr(self._lib, name)(self.handle, *args))

    def set_gemm_kernel_variant(self, variant: int) -> None:
        """Test / tuning hook: force one GEMM kernel form for later calls (0 = automatic)."""
        self.call("hipq_set_gemm_kernel_variant", int(variant))

    def set_trace_buffer(self, buf: Optional[torch.Tensor]) -> None:
        """Tuning aid: phase stamps of the packed GEMM go to `buf` (int64 device tensor) until None is set."""
        if buf is None:
            self.call("hipq_ctx_set_trace_buffer", None, 0)
        else:
            self.call("hipq_ctx_set_trace_buffer", _ptr(buf), buf.numel() * buf.element_size())

    def set_resident_share(self, contexts: int) -> None:
        """How many contexts launch concurrently on this device: the one-launch dynamic quantizers, whose grid has
        to be resident at once, then size it for 1 / contexts of the device."""
        self.call("hipq_ctx_set_resident_share", int(contexts))

    def set_wait_spin_limit(self, limit: int) -> None:
        """Test hook: polls a bounded wait (persistent GEMM, one-launch dynamic quantizer) makes before it gives
        up (< 0: default)."""
        self.call("hipq_ctx_set_wait_spin_limit", int(limit))

    def synchronize(self) -> None:
        self.call("hipq_ctx_synchronize")

    @property
    def stream_handle(self) -> int:
        return self._lib.hipq_ctx_stream(self.handle) or 0

    # ---- convenience wrappers over torch tensors (device memory only) -------------
    def _dev(self):
        return torch.device("cuda", self.device)

    def minmax(self, x: torch.Tensor) -> torch.Tensor:
        out = torch.empty(2, dtype=torch.float32, device=self._dev())
        self.call("hipq_minmax_f32", _ptr(x), x.numel(), _ptr(out))
        return out

    def absmax(self, x: torch.Tensor) -> torch.Tensor:
        out = torch.empty(1, dtype=torch.float32, device=self._dev())
        self.call("hipq_absmax_f32", _ptr(x), x.numel(), _ptr(out))
        return out

    def new_qparams(self) -> torch.Tensor:
        return torch.zeros(C.sizeof(QParams), dtype=torch.uint8, device=self._dev())

    @staticmethod
    def read_qparams(buf: torch.Tensor) -> QParams:
        return QParams.from_buffer_copy(bytes(buf.cpu().numpy().tobytes()))

    def qparams_from_minmax(self, minmax: torch.Tensor, flavor: int, qmin: int, qmax: int) -> torch.Tensor:
        out = self.new_qparams()
        self.call("hipq_qparams_from_minmax", _ptr(minmax), flavor, qmin, qmax, _ptr(out))
        return out

    # ---- quantized elementwise operators ---------------------------------------------
    def qadd(self, a, a_scale, a_zp, b, b_scale, b_zp, flavor=PARAMS_BACKEND_ASYMMETRIC):
        """a, b: int8 or uint8 tensors (per-tensor parameters); output has a's dtype.  -> (out, params record)"""
        out = torch.empty(a.shape, dtype=a.dtype, device=self._dev())
        params = self.new_qparams()
        self.call("hipq_qadd_u8", _ptr(a), int(a.dtype == torch.int8), float(a_scale), int(a_zp), _ptr(b),
                  int(b.dtype == torch.int8), float(b_scale), int(b_zp), a.numel(), flavor,
                  DTYPE_I8 if a.dtype == torch.int8 else DTYPE_U8, _ptr(out), _ptr(params))
        return out, params

    def qrelu(self, q, scale, zp, flavor=PARAMS_BACKEND_ASYMMETRIC):
        out = torch.empty(q.shape, dtype=q.dtype, device=self._dev())
        params = self.new_qparams()
        self.call("hipq_qrelu_u8", _ptr(q), int(q.dtype == torch.int8), float(scale), int(zp), q.numel(), flavor,
                  DTYPE_I8 if q.dtype == torch.int8 else DTYPE_U8, _ptr(out), _ptr(params))
        return out, params

    # ---- calibration observers and quality metrics --------------------------------
    def _record(self, ty):
        return torch.zeros(C.sizeof(ty), dtype=torch.uint8, device=self._dev())

    @staticmethod
    def _read(buf: torch.Tensor, ty):
        return ty.from_buffer_copy(bytes(buf.cpu().numpy().tobytes()))

    def quantization_metrics(self, original, quantized, original_bits=32, quantized_bits=8, out=None) -> torch.Tensor:
        """Device record (QuantMetrics); read it with read_metrics()."""
        out = out if out is not None else self._record(QuantMetrics)
        self.call("hipq_quantization_metrics_f32", _ptr(original), _ptr(quantized), original.numel(), original_bits,
                  quantized_bits, _ptr(out))
        return out

    def fake_quantize_metrics(self, x, scale, zp, qmin=-128, qmax=127, mode=0, params=None, original_bits=32,
                              quantized_bits=8, out=None) -> torch.Tensor:
        out = out if out is not None else self._record(QuantMetrics)
        self.call("hipq_fake_quantize_metrics_f32", _ptr(x), x.numel(), float(scale), int(zp), _ptr(params), qmin,
                  qmax, mode, original_bits, quantized_bits, _ptr(out))
        return out

    def read_metrics(self, buf: torch.Tensor) -> dict:
        return self._read(buf, QuantMetrics).as_dict()

    def fake_quantize(self, x, scale, zp, qmin=-128, qmax=127, mode=0, params=None, out=None) -> torch.Tensor:
        out = out if out is not None else torch.empty(x.shape, dtype=torch.float32, device=self._dev())
        self.call("hipq_fake_quantize_f32", _ptr(x), x.numel(), float(scale), int(zp), _ptr(params), qmin, qmax,
                  mode, _ptr(out))
        return out

    def observe(self, x, out=None) -> torch.Tensor:
        """Device record (ObserveStats): batch min, max and the number of non-finite values."""
        out = out if out is not None else self._record(ObserveStats)
        self.call("hipq_observe_f32", _ptr(x), x.numel(), _ptr(out))
        return out

    def tensor_stats(self, x, one_pass=False, out=None):
        """min, max, mean, std_dev, variance (population) of x; one_pass selects the raw-moment form.  Returns the
        record read back, or with `out` (a device record) leaves it there and returns `out`."""
        rec = out if out is not None else self._record(TensorStats)
        self.call("hipq_tensor_stats_f32", _ptr(x), x.numel(), int(one_pass), _ptr(rec))
        return rec if out is not None else self._read(rec, TensorStats)

    def read_observe(self, buf: torch.Tensor) -> ObserveStats:
        return self._read(buf, ObserveStats)

    def histogram(self, x, range_min, range_max, num_bins, counts=None) -> torch.Tensor:
        """counts[num_bins] (int64 tensor holding the uint64 counters) += histogram of x."""
        if counts is None:
            counts = torch.zeros(num_bins, dtype=torch.int64, device=self._dev())
        self.call("hipq_histogram_f32", _ptr(x), x.numel(), float(range_min), float(range_max), num_bins,
                  _ptr(counts))
        return counts

    def quantize_per_tensor_i8(self, x, scale, zp, mode=0, out=None):
        out = out if out is not None else torch.empty(x.shape, dtype=torch.int8, device=self._dev())
        self.call("hipq_quantize_per_tensor_f32_i8", _ptr(x), x.numel(), float(scale), int(zp), mode, _ptr(out))
        return out

    def quantize_per_tensor_u8(self, x, scale, zp, mode=FORM_DIV, out=None):
        out = out if out is not None else torch.empty(x.shape, dtype=torch.uint8, device=self._dev())
        self.call("hipq_quantize_per_tensor_f32_u8", _ptr(x), x.numel(), float(scale), int(zp), mode, _ptr(out))
        return out

    def quantize_per_tensor_carrier(self, x, scale, zp, mode=0, qmin=-128, qmax=127):
        out = torch.empty(x.shape, dtype=torch.float32, device=self._dev())
        self.call("hipq_quantize_per_tensor_f32_carrier", _ptr(x), x.numel(), float(scale), int(zp), mode, qmin, qmax,
                  _ptr(out))
        return out

    def quantize_dynamic_per_tensor(self, x, flavor=PARAMS_SYMMETRIC, dtype=DTYPE_I8, mode=0, out=None, params=None):
        tdt = torch.int8 if dtype == DTYPE_I8 else torch.uint8
        out = out if out is not None else torch.empty(x.shape, dtype=tdt, device=self._dev())
        params = params if params is not None else self.new_qparams()
        self.call("hipq_quantize_dynamic_per_tensor_f32", _ptr(x), x.numel(), flavor, dtype, mode, _ptr(out),
                  _ptr(params))
        return out, params

    def dequantize(self, q, scale, zp, out=None):
        out = out if out is not None else torch.empty(q.shape, dtype=torch.float32, device=self._dev())
        name = {torch.int8: "hipq_dequantize_i8_f32", torch.uint8: "hipq_dequantize_u8_f32",
                torch.float32: "hipq_dequantize_carrier_f32"}[q.dtype]
        self.call(name, _ptr(q), q.numel(), float(scale), int(zp), _ptr(out))
        return out

    def dequantize_with_params(self, q, params, out=None):
        out = out if out is not None else torch.empty(q.shape, dtype=torch.float32, device=self._dev())
        self.call("hipq_dequantize_with_params_i8_f32", _ptr(q), q.numel(), _ptr(params), _ptr(out))
        return out

    def quantize_per_row(self, x, flavor=PARAMS_SYMMETRIC, mode=0):
        rows, cols = x.shape
        out = torch.empty((rows, cols), dtype=torch.int8, device=self._dev())
        scales = torch.empty(rows, dtype=torch.float32, device=self._dev())
        zps = torch.empty(rows, dtype=torch.int32, device=self._dev())
        status = torch.empty(1, dtype=torch.int32, device=self._dev())
        self.call("hipq_quantize_per_row_f32_i8", _ptr(x), rows, cols, flavor, mode, _ptr(out), _ptr(scales),
                  _ptr(zps), _ptr(status))
        return out, scales, zps, status

    def quantize_per_group_auto(self, x, outer, channels, inner, group_size, flavor, qmin, qmax, mode=0):
        """Group-wise quantize of the dense [outer, channels, inner] view of x into [qmin, qmax]; parameters per group."""
        groups = -(-channels // group_size) if group_size > 0 else 1
        out = torch.empty(x.shape, dtype=torch.int8, device=self._dev())
        scales = torch.empty(groups, dtype=torch.float32, device=self._dev())
        zps = torch.empty(groups, dtype=torch.int32, device=self._dev())
        status = torch.empty(1, dtype=torch.int32, device=self._dev())
        self.call("hipq_quantize_per_group_auto_f32_i8", _ptr(x), outer, channels, inner, group_size, flavor, qmin,
                  qmax, mode, _ptr(out), _ptr(scales), _ptr(zps), _ptr(status))
        return out, scales, zps, status

    def quantize_binary(self, x):
        out = torch.empty(x.shape, dtype=torch.int8, device=self._dev())
        params = self.new_qparams()
        self.call("hipq_quantize_binary_f32_i8", _ptr(x), x.numel(), _ptr(out), _ptr(params))
        return out, params

    def quantize_ternary(self, x):
        out = torch.empty(x.shape, dtype=torch.int8, device=self._dev())
        params = self.new_qparams()
        self.call("hipq_quantize_ternary_f32_i8", _ptr(x), x.numel(), _ptr(out), _ptr(params))
        return out, params

    def quantize_binary_learned_threshold(self, x, threshold=None):
        """Codes in {-1, 0, 1}; params.min_val holds the threshold used (mean |x| when none is given)."""
        out = torch.empty(x.shape, dtype=torch.int8, device=self._dev())
        params = self.new_qparams()
        self.call("hipq_quantize_binary_learned_threshold_f32_i8", _ptr(x), x.numel(), int(threshold is not None),
                  float(threshold or 0.0), _ptr(out), _ptr(params))
        return out, params

    def quantize_ternary_adaptive(self, x):
        out = torch.empty(x.shape, dtype=torch.int8, device=self._dev())
        params = self.new_qparams()
        self.call("hipq_quantize_ternary_adaptive_f32_i8", _ptr(x), x.numel(), _ptr(out), _ptr(params))
        return out, params

    def quantize_per_channel_auto(self, x, axis, flavor=PARAMS_SYMMETRIC, mode=0):
        shape = list(x.shape)
        outer = 1
        for s in shape[:axis]:
            outer *= s
        inner = 1
        for s in shape[axis + 1:]:
            inner *= s
        ch = shape[axis]
        out = torch.empty(x.shape, dtype=torch.int8, device=self._dev())
        scales = torch.empty(ch, dtype=torch.float32, device=self._dev())
        zps = torch.empty(ch, dtype=torch.int32, device=self._dev())
        status = torch.empty(1, dtype=torch.int32, device=self._dev())
        self.call("hipq_quantize_per_channel_auto_f32_i8", _ptr(x), outer, ch, inner, flavor, mode, _ptr(out),
                  _ptr(scales), _ptr(zps), _ptr(status))
        return out, scales, zps, status

    def quantize_per_channel(self, x, scales, zps, axis, mode=FORM_DIV):
        shape = list(x.shape)
        outer = 1
        for s in shape[:axis]:
            outer *= s
        inner = 1
        for s in shape[axis + 1:]:
            inner *= s
        out = torch.empty(x.shape, dtype=torch.int8, device=self._dev())
        self.call("hipq_quantize_per_channel_f32_i8", _ptr(x), outer, shape[axis], inner, _ptr(scales), _ptr(zps),
                  mode, _ptr(out))
        return out

    def dequantize_per_channel(self, q, scales, zps, axis):
        shape = list(q.shape)
        outer = 1
        for s in shape[:axis]:
            outer *= s
        inner = 1
        for s in shape[axis + 1:]:
            inner *= s
        out = torch.empty(q.shape, dtype=torch.float32, device=self._dev())
        self.call("hipq_dequantize_per_channel_i8_f32", _ptr(q), outer, shape[axis], inner, _ptr(scales), _ptr(zps),
                  _ptr(out))
        return out

    def gemm_i8_i32(self, a, w, out=None):
        m, k = a.shape
        n, k2 = w.shape
        if k != k2:
            raise HipqError(DIMENSION_MISMATCH, f"gemm dimension mismatch: a has K={k} but w has K={k2}")
        out = out if out is not None else torch.empty((m, n), dtype=torch.int32, device=self._dev())
        self.call("hipq_gemm_i8_i32", _ptr(a), _ptr(w), m, n, k, _ptr(out))
        return out

    def linear_i8_f32(self, a, a_scale, w, w_scales, bias=None, out=None):
        m, k = a.shape
        n, _ = w.shape
        out = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=self._dev())
        self.call("hipq_linear_i8_f32", _ptr(a), _ptr(a_scale), int(a_scale.numel() > 1), _ptr(w), _ptr(w_scales),
                  _ptr(bias), m, n, k, _ptr(out))
        return out

    def quantize_static_per_tensor(self, x, scale, zp=0, mode=0, out=None, params=None):
        """Per-tensor int8 quantize with given parameters, which are also recorded in a device-side record."""
        out = out if out is not None else torch.empty(x.shape, dtype=torch.int8, device=self._dev())
        params = params if params is not None else self.new_qparams()
        self.call("hipq_quantize_static_per_tensor_f32_i8", _ptr(x), x.numel(), float(scale), int(zp), mode, _ptr(out),
                  _ptr(params))
        return out, params

    def linear_static(self, x, a_scale, w, w_scales, bias=None, mode=0, out=None):
        """Quantized Linear forward with a calibrated (static) per-tensor activation scale."""
        m, k = x.shape
        n, _ = w.shape
        out = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=self._dev())
        self.call("hipq_linear_static_f32", _ptr(x), float(a_scale), _ptr(w), _ptr(w_scales), _ptr(bias), m, n, k, mode,
                  _ptr(out))
        return out

    def linear_i8_i8(self, a, a_scale, w, w_scales, bias, out_scale, out_zp, mode=0, out=None):
        m, k = a.shape
        n, _ = w.shape
        out = out if out is not None else torch.empty((m, n), dtype=torch.int8, device=self._dev())
        self.call("hipq_linear_i8_i8", _ptr(a), _ptr(a_scale), int(a_scale.numel() > 1), _ptr(w), _ptr(w_scales),
                  _ptr(bias), m, n, k, float(out_scale), int(out_zp), mode, _ptr(out))
        return out

    def requantize(self, acc, a_scale, w_scales, bias, out_scale, out_zp, mode=0):
        rows, cols = acc.shape
        out = torch.empty((rows, cols), dtype=torch.int8, device=self._dev())
        self.call("hipq_requantize_i32_i8", _ptr(acc), rows, cols, _ptr(a_scale), int(a_scale.numel() > 1),
                  _ptr(w_scales), _ptr(bias), float(out_scale), int(out_zp), mode, _ptr(out))
        return out

    def linear_dynamic(self, x, w, w_scales, bias=None, per_token=False, mode=0, out=None):
        m, k = x.shape
        n, _ = w.shape
        out = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=self._dev())
        self.call("hipq_linear_dynamic_f32", _ptr(x), int(per_token), _ptr(w), _ptr(w_scales), _ptr(bias), m, n, k,
                  mode, _ptr(out))
        return out

    # ---- fragment-packed operands ------------------------------------------------------
    def packed_size(self, rows: int, k: int) -> int:
        n = C.c_size_t(0)
        _check(self._lib.hipq_packed_size(rows, k, C.byref(n)))
        return int(n.value)

    def pack_rows(self, q: torch.Tensor, out=None) -> torch.Tensor:
        """int8 [rows, k] -> the packed operand of the fast GEMM (a flat int8 buffer)."""
        rows, k = q.shape
        out = out if out is not None else torch.empty(self.packed_size(rows, k), dtype=torch.int8, device=self._dev())
        self.call("hipq_pack_rows_i8", _ptr(q), rows, k, _ptr(out))
        return out

    def gemm_packed_i8_i32(self, a_packed, w_packed, m, n, k, out=None):
        out = out if out is not None else torch.empty((m, n), dtype=torch.int32, device=self._dev())
        self.call("hipq_gemm_packed_i8_i32", _ptr(a_packed), _ptr(w_packed), m, n, k, _ptr(out))
        return out

    def linear_packed_i8_f32(self, a_packed, a_scale, w_packed, w_scales, bias, m, n, k, out=None):
        out = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=self._dev())
        self.call("hipq_linear_packed_i8_f32", _ptr(a_packed), _ptr(a_scale), int(a_scale.numel() > 1), _ptr(w_packed),
                  _ptr(w_scales), _ptr(bias), m, n, k, _ptr(out))
        return out

    def linear_packed_i8_i8(self, a_packed, a_scale, w_packed, w_scales, bias, m, n, k, out_scale, out_zp, mode=0):
        out = torch.empty((m, n), dtype=torch.int8, device=self._dev())
        self.call("hipq_linear_packed_i8_i8", _ptr(a_packed), _ptr(a_scale), int(a_scale.numel() > 1), _ptr(w_packed),
                  _ptr(w_scales), _ptr(bias), m, n, k, float(out_scale), int(out_zp), mode, _ptr(out))
        return out

    def quantize_per_tensor_packed(self, x, dynamic=True, scale=1.0, mode=0, out=None, params=None):
        """Symmetric per-tensor int8 quantize of fp32 [rows, cols] into the packed layout -> (packed, params)."""
        rows, cols = x.shape
        out = out if out is not None else torch.empty(self.packed_size(rows, cols), dtype=torch.int8,
                                                      device=self._dev())
        params = params if params is not None else self.new_qparams()
        self.call("hipq_quantize_per_tensor_packed_f32_i8", _ptr(x), rows, cols, int(dynamic), float(scale), mode,
                  _ptr(out), _ptr(params))
        return out, params

    def quantize_per_row_packed(self, x, mode=0, out=None, scales=None):
        """Symmetric per-row int8 quantize of fp32 [rows, cols] into the packed layout -> (packed, row scales)."""
        rows, cols = x.shape
        out = out if out is not None else torch.empty(self.packed_size(rows, cols), dtype=torch.int8,
                                                      device=self._dev())
        scales = scales if scales is not None else torch.empty(rows, dtype=torch.float32, device=self._dev())
        self.call("hipq_quantize_per_row_packed_f32_i8", _ptr(x), rows, cols, mode, _ptr(out), _ptr(scales))
        return out, scales

    def linear_dynamic_packed(self, x, w_packed, w_scales, bias=None, per_token=False, mode=0, out=None):
        m, k = x.shape
        n = w_scales.numel()
        out = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=self._dev())
        self.call("hipq_linear_dynamic_packed_f32", _ptr(x), int(per_token), _ptr(w_packed), _ptr(w_scales), _ptr(bias),
                  m, n, k, mode, _ptr(out))
        return out

    def linear_static_packed(self, x, a_scale, w_packed, w_scales, bias=None, mode=0, out=None):
        m, k = x.shape
        n = w_scales.numel()
        out = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=self._dev())
        self.call("hipq_linear_static_packed_f32", _ptr(x), float(a_scale), _ptr(w_packed), _ptr(w_scales), _ptr(bias),
                  m, n, k, mode, _ptr(out))
        return out

    # ---- a panel of whole rows per workgroup: the Linear and the row operation after it ----
    def linear_rows_packed_i8_f32(self, a_packed, a_scale, w_packed, w_scales, bias, m, n, k, out=None):
        out = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=self._dev())
        self.call("hipq_linear_rows_packed_i8_f32", _ptr(a_packed), _ptr(a_scale), int(a_scale.numel() > 1),
                  _ptr(w_packed), _ptr(w_scales), _ptr(bias), m, n, k, _ptr(out))
        return out

    def linear_gelu_quantize_packed(self, a_packed, a_scale, w_packed, w_scales, bias, m, n, k, mode=0, out=None,
                                    scales=None):
        """-> (packed int8 [m, n] of GELU(linear), row scales [m])"""
        out = out if out is not None else torch.empty(self.packed_size(m, n), dtype=torch.int8, device=self._dev())
        scales = scales if scales is not None else torch.empty(m, dtype=torch.float32, device=self._dev())
        self.call("hipq_linear_gelu_quantize_packed_i8", _ptr(a_packed), _ptr(a_scale), int(a_scale.numel() > 1),
                  _ptr(w_packed), _ptr(w_scales), _ptr(bias), m, n, k, mode, _ptr(out), _ptr(scales))
        return out, scales

    def linear_residual_layer_norm_quantize_packed(self, a_packed, a_scale, w_packed, w_scales, bias, m, n, k, x,
                                                   gamma=None, beta=None, eps=1e-5, mode=0, normalize=True, out=None,
                                                   scales=None):
        """x += linear (in place); with `normalize` -> (packed int8 [m, n] of LayerNorm(x), row scales [m])"""
        if normalize:
            out = out if out is not None else torch.empty(self.packed_size(m, n), dtype=torch.int8,
                                                          device=self._dev())
            scales = scales if scales is not None else torch.empty(m, dtype=torch.float32, device=self._dev())
        else:
            out = scales = None
        self.call("hipq_linear_residual_layer_norm_quantize_packed_i8", _ptr(a_packed), _ptr(a_scale),
                  int(a_scale.numel() > 1), _ptr(w_packed), _ptr(w_scales), _ptr(bias), m, n, k, _ptr(x), _ptr(gamma),
                  _ptr(beta), float(eps), mode, _ptr(out), _ptr(scales))
        return out, scales

    def linear_dynamic_noalloc(self, x, w, w_scales, bias=None, per_token=False, mode=0, out=None):
        """hipq_linear_dynamic_f32_noalloc: the same forward on the library's static device scratch.  `out`
        should be given by callers that must not allocate; it is created here only as a convenience."""
        m, k = x.shape
        n, _ = w.shape
        out = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=self._dev())
        self.call("hipq_linear_dynamic_f32_noalloc", _ptr(x), int(per_token), _ptr(w), _ptr(w_scales), _ptr(bias), m, n,
                  k, mode, _ptr(out))
        return out

    def conv2d_i32(self, x_u8, zp_in, w_i8, stride=(1, 1), padding=(0, 0)):
        nb, c, h, wd = x_u8.shape
        oc, c2, kh, kw = w_i8.shape
        if c != c2:
            raise HipqError(DIMENSION_MISMATCH, f"qconv2d channel mismatch: input C_in={c} but weight C_in={c2}")
        ho = max((h + 2 * padding[0] - kh) // stride[0] + 1, 0)  # the library rejects impossible geometry
        wo = max((wd + 2 * padding[1] - kw) // stride[1] + 1, 0)
        out = torch.empty((nb, oc, ho, wo), dtype=torch.int32, device=self._dev())
        self.call("hipq_conv2d_u8i8_i32", _ptr(x_u8), int(zp_in), _ptr(w_i8), nb, c, h, wd, oc, kh, kw, stride[0],
                  stride[1], padding[0], padding[1], _ptr(out))
        return out

    def conv2d_i8(self, x_u8, zp_in, s_in, w_i8, w_scales, bias, s_out, zp_out, stride=(1, 1), padding=(0, 0), mode=0,
                  out=None):
        nb, c, h, wd = x_u8.shape
        oc, c2, kh, kw = w_i8.shape
        if c != c2:
            raise HipqError(DIMENSION_MISMATCH, f"qconv2d channel mismatch: input C_in={c} but weight C_in={c2}")
        ho = max((h + 2 * padding[0] - kh) // stride[0] + 1, 0)  # the library rejects impossible geometry
        wo = max((wd + 2 * padding[1] - kw) // stride[1] + 1, 0)
        out = out if out is not None else torch.empty((nb, oc, ho, wo), dtype=torch.int8, device=self._dev())
        self.call("hipq_conv2d_u8i8_i8", _ptr(x_u8), int(zp_in), float(s_in), _ptr(w_i8), _ptr(w_scales), _ptr(bias), nb,
                  c, h, wd, oc, kh, kw, stride[0], stride[1], padding[0], padding[1], float(s_out), int(zp_out), mode,
                  _ptr(out))
        return out

    def conv2d_f32(self, x_u8, zp_in, s_in, w_i8, w_scales, bias, stride=(1, 1), padding=(0, 0), out=None):
        nb, c, h, wd = x_u8.shape
        oc, c2, kh, kw = w_i8.shape
        if c != c2:
            raise HipqError(DIMENSION_MISMATCH, f"qconv2d channel mismatch: input C_in={c} but weight C_in={c2}")
        ho = max((h + 2 * padding[0] - kh) // stride[0] + 1, 0)
        wo = max((wd + 2 * padding[1] - kw) // stride[1] + 1, 0)
        out = out if out is not None else torch.empty((nb, oc, ho, wo), dtype=torch.float32, device=self._dev())
        self.call("hipq_conv2d_u8i8_f32", _ptr(x_u8), int(zp_in), float(s_in), _ptr(w_i8), _ptr(w_scales), _ptr(bias), nb,
                  c, h, wd, oc, kh, kw, stride[0], stride[1], padding[0], padding[1], _ptr(out))
        return out

    def conv2d_pack_weights(self, w_i8):
        """int8 [OC, IC, KH, KW] filters -> (packed row operand of the matrix-core GEMM, per-filter sums)."""
        oc, ic, kh, kw = w_i8.shape
        n = C.c_size_t(0)
        _check(self._lib.hipq_conv2d_packed_weights_size(oc, ic, kh, kw, C.byref(n)))
        packed = torch.empty(int(n.value), dtype=torch.int8, device=self._dev())
        sums = torch.empty(oc, dtype=torch.int32, device=self._dev())
        self.call("hipq_conv2d_pack_weights_i8", _ptr(w_i8), oc, ic, kh, kw, _ptr(packed), _ptr(sums))
        return packed, sums

    def conv2d_i8_packed(self, x_u8, zp_in, s_in, w_packed, w_sums, kernel, w_scales, bias, s_out, zp_out,
                         padding=(0, 0), mode=0, out=None):
        nb, c, h, wd = x_u8.shape
        oc = w_sums.numel()
        kh, kw = kernel
        ho = h + 2 * padding[0] - kh + 1
        wo = wd + 2 * padding[1] - kw + 1
        out = out if out is not None else torch.empty((nb, oc, ho, wo), dtype=torch.int8, device=self._dev())
        self.call("hipq_conv2d_u8i8_i8_packed", _ptr(x_u8), int(zp_in), float(s_in), _ptr(w_packed), _ptr(w_sums),
                  _ptr(w_scales), _ptr(bias), nb, c, h, wd, oc, kh, kw, padding[0], padding[1], float(s_out),
                  int(zp_out), mode, _ptr(out))
        return out

    def conv2d_dynamic_packed(self, x, w_packed, w_sums, kernel, w_scales, bias, s_out, zp_out, padding=(0, 0),
                              flavor=PARAMS_BACKEND_ASYMMETRIC, quant_mode=0, mode=0, out=None, params=None):
        """Conv2d forward from fp32 activations: dynamic per-tensor uint8 quantize of x on the device, then the
        convolution on prepared filters -> (int8 output, device hipq_qparams of the input)."""
        nb, c, h, wd = x.shape
        oc = w_sums.numel()
        kh, kw = kernel
        ho = h + 2 * padding[0] - kh + 1
        wo = wd + 2 * padding[1] - kw + 1
        out = out if out is not None else torch.empty((nb, oc, ho, wo), dtype=torch.int8, device=self._dev())
        params = params if params is not None else self.new_qparams()
        self.call("hipq_conv2d_dynamic_f32_i8_packed", _ptr(x), flavor, quant_mode, _ptr(w_packed), _ptr(w_sums),
                  _ptr(w_scales), _ptr(bias), nb, c, h, wd, oc, kh, kw, padding[0], padding[1], float(s_out),
                  int(zp_out), mode, _ptr(out), _ptr(params))
        return out, params

    def quantize_per_row_strided(self, x_base, rows, cols, ld, elem_offset=0, flavor=PARAMS_SYMMETRIC, mode=0):
        out = torch.empty((rows, cols), dtype=torch.int8, device=self._dev())
        scales = torch.empty(rows, dtype=torch.float32, device=self._dev())
        self.call("hipq_quantize_per_row_strided_f32_i8", x_base.data_ptr() + 4 * elem_offset, rows, cols, ld, flavor,
                  mode, _ptr(out), _ptr(scales), None, None)
        return out, scales

    def linear_i8_f32_residual(self, a, a_scale, w, w_scales, bias, residual, out=None):
        m, k = a.shape
        n, _ = w.shape
        out = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=self._dev())
        self.call("hipq_linear_i8_f32_residual", _ptr(a), _ptr(a_scale), int(a_scale.numel() > 1), _ptr(w),
                  _ptr(w_scales), _ptr(bias), _ptr(residual), m, n, k, _ptr(out))
        return out

    def layer_norm(self, x, gamma=None, beta=None, eps=1e-5):
        rows, cols = x.shape
        out = torch.empty_like(x)
        self.call("hipq_layer_norm_f32", _ptr(x), rows, cols, _ptr(gamma), _ptr(beta), float(eps), _ptr(out))
        return out

    def layer_norm_quantize(self, x, gamma=None, beta=None, eps=1e-5, mode=0):
        rows, cols = x.shape
        out = torch.empty((rows, cols), dtype=torch.int8, device=self._dev())
        scales = torch.empty(rows, dtype=torch.float32, device=self._dev())
        self.call("hipq_layer_norm_quantize_f32_i8", _ptr(x), rows, cols, _ptr(gamma), _ptr(beta), float(eps), mode,
                  _ptr(out), _ptr(scales))
        return out, scales

    def linear_from_f32_residual_layer_norm_quantize_packed(self, a, w_packed, w_scales, bias, n, x, gamma=None,
                                                            beta=None, eps=1e-5, mode=0, normalize=True, out=None,
                                                            scales=None):
        """The same from fp32 activations a [m, k] (a view whose rows may be further apart than k): the per-token
        int8 quantizer of a runs inside the kernel."""
        m, k = a.shape
        assert a.stride(1) == 1
        if normalize:
            out = out if out is not None else torch.empty(self.packed_size(m, n), dtype=torch.int8,
                                                          device=self._dev())
            scales = scales if scales is not None else torch.empty(m, dtype=torch.float32, device=self._dev())
        else:
            out = scales = None
        self.call("hipq_linear_from_f32_residual_layer_norm_quantize_packed_i8", a.data_ptr(), a.stride(0),
                  _ptr(w_packed), _ptr(w_scales), _ptr(bias), m, n, k, _ptr(x), _ptr(gamma), _ptr(beta), float(eps), mode,
                  _ptr(out), _ptr(scales))
        return out, scales

    def add_layer_norm_quantize(self, x, delta, gamma=None, beta=None, eps=1e-5, mode=0):
        """x += delta in place, then LayerNorm + per-token int8 of the new x."""
        rows, cols = x.shape
        out = torch.empty((rows, cols), dtype=torch.int8, device=self._dev())
        scales = torch.empty(rows, dtype=torch.float32, device=self._dev())
        self.call("hipq_add_layer_norm_quantize_f32_i8", _ptr(x), _ptr(delta), rows, cols, _ptr(gamma), _ptr(beta),
                  float(eps), mode, _ptr(out), _ptr(scales))
        return out, scales

    def gelu_tanh(self, x):
        out = torch.empty_like(x)
        self.call("hipq_gelu_tanh_f32", _ptr(x), x.numel(), _ptr(out))
        return out

    def gelu_tanh_quantize(self, x, mode=0):
        rows, cols = x.shape
        out = torch.empty((rows, cols), dtype=torch.int8, device=self._dev())
        scales = torch.empty(rows, dtype=torch.float32, device=self._dev())
        self.call("hipq_gelu_tanh_quantize_f32_i8", _ptr(x), rows, cols, mode, _ptr(out), _ptr(scales))
        return out, scales

    def add(self, a, b):
        out = torch.empty_like(a)
        self.call("hipq_add_f32", _ptr(a), _ptr(b), a.numel(), _ptr(out))
        return out

    def stack_workspace(self, tokens, d_model, d_ff):
        nbytes = self._lib.hipq_transformer_stack_workspace_bytes(tokens, d_model, d_ff)
        return torch.empty(nbytes, dtype=torch.uint8, device=self._dev())

    def stack_prepare(self, blocks):
        """The blocks with every int8 weight matrix in packed order (done once per model)."""
        return [{k: (self.pack_rows(v) if k.startswith("w_") else v) for k, v in blk.items()} for blk in blocks]

    def stack_workspace_prepared(self, tokens, d_model, d_ff):
        nbytes = self._lib.hipq_transformer_stack_prepared_workspace_bytes(tokens, d_model, d_ff)
        return torch.empty(nbytes, dtype=torch.uint8, device=self._dev())

    def stack_forward(self, blocks, x, d_ff, workspace, eps=1e-5, mode=0, prepared=False):
        """blocks: list of dicts of device tensors keyed like BlockWeights; x [tokens, d_model] is updated in place.
        prepared: the blocks come from stack_prepare and the workspace from stack_workspace_prepared."""
        arr = (BlockWeights * len(blocks))()
        for rec, blk in zip(arr, blocks):
            for name, _ in BlockWeights._fields_:
                t = blk.get(name)
                setattr(rec, name, None if t is None else t.data_ptr())
        tokens, d_model = x.shape
        self.call("hipq_transformer_stack_forward_prepared_f32" if prepared else "hipq_transformer_stack_forward_f32",
                  C.cast(arr, C.c_void_p), len(blocks), tokens, d_model, d_ff, float(eps), mode, _ptr(x),
                  _ptr(workspace), workspace.numel())
        return x
