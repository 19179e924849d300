// torsh::quantization — the free functions of crates/torsh-quantization that sit on the
// quantized-inference path, with the reference's names, argument meaning and error
// behaviour, executed on the GPU through the torsh_hipq C-ABI.
//
//   quantize_with_config              crates/torsh-quantization/src/algorithms.rs:30-66
//   quantize_per_tensor               algorithms.rs:69-77
//   dequantize                        algorithms.rs:80-82
//   quantize_tensor_auto              algorithms.rs:85-123
//   quantize_per_channel_auto         algorithms.rs:126-242
//   quantize_per_tensor_affine_i8     algorithms.rs:245-274
//   quantize_per_tensor_affine        algorithms.rs:277-315
//   dequantize_per_tensor_affine      algorithms.rs:318-355
//   calculate_affine_quantization_params / calculate_symmetric_quantization_params
//                                     algorithms.rs:358-394 / 397-422
//   get_dtype_range                   algorithms.rs:425-433
//   quantize_auto                     algorithms.rs:436-438
//   quantize_per_tensor_affine_simd, dequantize_per_tensor_affine_simd, find_min_max_simd,
//   quantize_to_int8_simd             crates/torsh-quantization/src/simd_ops.rs:18,52,84,196
//   CacheAwareParams and the cache-aware / tiled / streaming quantizers, tensor statistics
//                                     algorithms.rs:440-735
//   quantize_batch_consistent_simd, calculate_tensor_stats_simd, the NEON and mobile twins
//                                     simd_ops.rs:170-193, 230-476
//   QScheme, QuantConfig              crates/torsh-quantization/src/config.rs:31-52, 95-128, 158-409
//
// quantize_with_config also dispatches the special schemes (int4, binary, ternary, group-wise) to
// specialized.hpp; mixed precision needs the reference's specialised API and is an error here too.
#pragma once

#include <cfloat>
#include <cmath>
#include <optional>
#include <string>
#include <tuple>
#include <vector>

#include "core.hpp"

namespace torsh {
namespace quantization {

enum class QScheme {
    PerTensorAffine,
    PerChannelAffine,
    PerTensorSymmetric,
    PerChannelSymmetric,
    Int4PerTensor,
    Int4PerChannel,
    MixedPrecision,
    Binary,
    Ternary,
    GroupWise,
};

enum class QuantBackend { Fbgemm, Qnnpack, Native, Xnnpack };
enum class ReduceRange { None, Reduce };
enum class ObserverType { MinMax, MovingAverage, Histogram, Percentile, KLDivergence, Entropy };

struct QuantConfig {
    DType dtype = DType::I8;
    QScheme scheme = QScheme::PerTensorAffine;
    bool enable_fake_quant = false;
    ObserverType observer_type = ObserverType::MinMax;
    QuantBackend backend = QuantBackend::Native;
    ReduceRange reduce_range = ReduceRange::None;
    std::optional<int32_t> qint_min, qint_max;
    float eps = 1e-8f;
    float averaging_constant = 0.01f;
    std::optional<size_t> ch_axis;
    std::optional<size_t> group_size;

    static QuantConfig make() { return QuantConfig{}; }
    // config.rs:163-170: int8() is per-tensor *affine*.
    static QuantConfig int8() {
        QuantConfig c;
        c.dtype = DType::I8;
        c.scheme = QScheme::PerTensorAffine;
        return c;
    }
    static QuantConfig uint8() {
        QuantConfig c;
        c.dtype = DType::U8;
        c.scheme = QScheme::PerTensorAffine;
        return c;
    }
    // config.rs:173-246
    static QuantConfig int4() {
        QuantConfig c;
        c.scheme = QScheme::Int4PerTensor;
        c.qint_min = -8, c.qint_max = 7;
        c.observer_type = ObserverType::Histogram;
        return c;
    }
    static QuantConfig binary() {
        QuantConfig c;
        c.scheme = QScheme::Binary;
        c.qint_min = -1, c.qint_max = 1;
        return c;
    }
    static QuantConfig ternary() {
        QuantConfig c;
        c.scheme = QScheme::Ternary;
        c.qint_min = -1, c.qint_max = 1;
        return c;
    }
    static QuantConfig group_wise(size_t ch_axis, size_t group_size) {
        QuantConfig c;
        c.scheme = QScheme::GroupWise;
        c.ch_axis = ch_axis;
        c.group_size = group_size;
        c.observer_type = ObserverType::Histogram;
        return c;
    }
    static QuantConfig per_channel(size_t axis) {
        QuantConfig c;
        c.scheme = QScheme::PerChannelAffine;
        c.ch_axis = axis;
        return c;
    }
    // config.rs:270-283: a per-channel scheme set through with_scheme gets channel axis 0 when none was chosen.
    QuantConfig with_scheme(QScheme s) const {
        QuantConfig c = *this;
        c.scheme = s;
        if ((s == QScheme::PerChannelAffine || s == QScheme::PerChannelSymmetric || s == QScheme::GroupWise) &&
            !c.ch_axis)
            c.ch_axis = 0;
        if (s == QScheme::GroupWise && !c.group_size) c.group_size = 32;
        return c;
    }
    QuantConfig with_observer(ObserverType o) const {  // config.rs:264-267
        QuantConfig c = *this;
        c.observer_type = o;
        return c;
    }
    QuantConfig with_reduce_range(ReduceRange r) const {
        QuantConfig c = *this;
        c.reduce_range = r;
        return c;
    }

    // config.rs:304-328
    std::pair<int32_t, int32_t> get_qint_range() const {
        int32_t base_min, base_max;
        switch (scheme) {
        case QScheme::Int4PerTensor:
        case QScheme::Int4PerChannel: base_min = -8, base_max = 7; break;
        case QScheme::Binary:
        case QScheme::Ternary: base_min = -1, base_max = 1; break;
        default:
            if (dtype == DType::I8) base_min = -128, base_max = 127;
            else if (dtype == DType::U8) base_min = 0, base_max = 255;
            else base_min = qint_min.value_or(-128), base_max = qint_max.value_or(127);
        }
        if (reduce_range == ReduceRange::None) return {base_min, base_max};
        const int32_t range = base_max - base_min, reduced = range / 2, mid = (base_min + base_max) / 2;
        return {mid - reduced / 2, mid + reduced / 2};
    }

    // config.rs:331-409
    Result<Unit> validate() const {
        const bool per_ch = scheme == QScheme::PerChannelAffine || scheme == QScheme::PerChannelSymmetric ||
                            scheme == QScheme::GroupWise;
        if (per_ch && !ch_axis)
            return TorshError::invalid_argument("Per-channel/Group-wise quantization requires channel axis");
        if (scheme == QScheme::GroupWise) {
            if (!group_size) return TorshError::invalid_argument("Group-wise quantization requires group size");
            if (*group_size == 0) return TorshError::invalid_argument("Group size must be greater than 0");
        }
        if ((scheme == QScheme::Binary || scheme == QScheme::Ternary) &&
            !(observer_type == ObserverType::MinMax || observer_type == ObserverType::MovingAverage))
            return TorshError::invalid_argument("Binary/ternary quantization requires MinMax or MovingAverage observer");
        if (scheme == QScheme::MixedPrecision &&
            !(observer_type == ObserverType::KLDivergence || observer_type == ObserverType::Entropy))
            return TorshError::invalid_argument("Mixed precision quantization requires KLDivergence or Entropy observer");
        if (!(eps > 0.0f)) return TorshError::invalid_argument("eps must be positive");
        if (averaging_constant <= 0.0f || averaging_constant >= 1.0f)
            return TorshError::invalid_argument("averaging_constant must be in (0, 1)");
        return Unit{};
    }
};

// algorithms.rs:425-433
inline std::pair<int32_t, int32_t> get_dtype_range(DType dtype) {
    switch (dtype) {
    case DType::I8: return {-128, 127};
    case DType::U8: return {0, 255};
    case DType::I16: return {-32768, 32767};
    case DType::I32: return {INT32_MIN, INT32_MAX};
    default: return {-128, 127};
    }
}

namespace detail {
inline float clamp_keep_nan(float v, float lo, float hi) {
    if (v < lo) v = lo;
    if (v > hi) v = hi;
    return v;
}
inline int32_t f32_as_i32(float v) {  // Rust `as i32`: saturating, NaN -> 0
    if (v != v) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return static_cast<int32_t>(v);
}
inline bool is_simd_available() { return true; }  // simd_ops.rs:274-283 is true on x86_64 / aarch64
}  // namespace detail

// algorithms.rs:358-394.  Scalar host arithmetic, as in the reference.
inline Result<std::pair<float, int32_t>> calculate_affine_quantization_params(float min_val, float max_val,
                                                                              DType dtype) {
    if (!std::isfinite(min_val) || !std::isfinite(max_val))
        return TorshError::invalid_argument("Min and max values must be finite");
    if (min_val > max_val) return TorshError::invalid_argument("Min value must be <= max value");
    auto [qmin_i, qmax_i] = get_dtype_range(dtype);
    const float qmin = static_cast<float>(qmin_i), qmax = static_cast<float>(qmax_i);
    if (std::fabs(max_val - min_val) < FLT_EPSILON) return std::make_pair(1.0f, qmin_i);
    const float scale = (max_val - min_val) / (qmax - qmin);
    const float zp = qmin - min_val / scale;
    return std::make_pair(scale, detail::f32_as_i32(detail::clamp_keep_nan(std::round(zp), qmin, qmax)));
}

// algorithms.rs:397-422
inline Result<std::pair<float, int32_t>> calculate_symmetric_quantization_params(float min_val, float max_val,
                                                                                 DType dtype) {
    if (!std::isfinite(min_val) || !std::isfinite(max_val))
        return TorshError::invalid_argument("Min and max values must be finite");
    const float abs_max = std::fmax(std::fabs(min_val), std::fabs(max_val));
    if (abs_max < FLT_EPSILON) return std::make_pair(1.0f, 0);
    const float qmax = static_cast<float>(get_dtype_range(dtype).second);
    return std::make_pair(abs_max / qmax, 0);
}

// ---- slice-level functions (simd_ops.rs): the narrowest seam, one C-ABI call each ----

// simd_ops.rs:84-121
inline Result<std::pair<float, float>> find_min_max_simd(const std::vector<float> &data) {
    if (data.empty()) return TorshError::invalid_argument("Cannot find min/max of empty array");
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
    TORSH_TRY(dmm, hip::DeviceBuffer::alloc(ctx, 2 * sizeof(float)));
    TORSH_CHECK(hip::check(hipq_minmax_f32(ctx, dx.as<float>(), data.size(), dmm.as<float>())));
    TORSH_TRY(mm, dmm.to_host<float>(2));
    return std::make_pair(mm[0], mm[1]);
}

// simd_ops.rs:18-49: q = clamp(round(x * (1/scale)) + zp, -128, 127), f32 carrier.
inline Result<Unit> quantize_per_tensor_affine_simd(const std::vector<float> &input, float scale, int32_t zero_point,
                                                    std::vector<float> &output) {
    if (input.size() != output.size())
        return TorshError::invalid_argument("Input and output length mismatch");
    if (scale <= 0.0f) return TorshError::invalid_argument("Scale must be positive");
    if (input.empty()) return Unit{};
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, input.data(), input.size()));
    TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, input.size() * sizeof(float)));
    TORSH_CHECK(hip::check(hipq_quantize_per_tensor_f32_carrier(ctx, dx.as<float>(), input.size(), scale, zero_point,
                                                                HIPQ_FORM_MUL_INV, -128, 127, dq.as<float>())));
    TORSH_TRY(q, dq.to_host<float>(input.size()));
    output = std::move(q);
    return Unit{};
}

// simd_ops.rs:196-227: same arithmetic, int8 output.
inline Result<Unit> quantize_to_int8_simd(const std::vector<float> &input, float scale, int32_t zero_point,
                                          std::vector<int8_t> &output) {
    if (input.size() != output.size())
        return TorshError::invalid_argument("Input and output length mismatch");
    if (scale <= 0.0f) return TorshError::invalid_argument("Scale must be positive");
    if (input.empty()) return Unit{};
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, input.data(), input.size()));
    TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, input.size()));
    TORSH_CHECK(hip::check(hipq_quantize_per_tensor_f32_i8(ctx, dx.as<float>(), input.size(), scale, zero_point,
                                                           HIPQ_FORM_MUL_INV, dq.as<int8_t>())));
    TORSH_TRY(q, dq.to_host<int8_t>(input.size()));
    output = std::move(q);
    return Unit{};
}

// simd_ops.rs:52-81: y = (q - zp) * scale on the f32 carrier.
inline Result<Unit> dequantize_per_tensor_affine_simd(const std::vector<float> &input, float scale,
                                                      int32_t zero_point, std::vector<float> &output) {
    if (input.size() != output.size())
        return TorshError::invalid_argument("Input and output length mismatch");
    if (scale <= 0.0f) return TorshError::invalid_argument("Scale must be positive");
    if (input.empty()) return Unit{};
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dq, hip::DeviceBuffer::from_host(ctx, input.data(), input.size()));
    TORSH_TRY(dy, hip::DeviceBuffer::alloc(ctx, input.size() * sizeof(float)));
    TORSH_CHECK(hip::check(hipq_dequantize_carrier_f32(ctx, dq.as<float>(), input.size(), scale, zero_point,
                                                       dy.as<float>())));
    TORSH_TRY(y, dy.to_host<float>(input.size()));
    output = std::move(y);
    return Unit{};
}

// ---- the slice-level twins: cache-aware, tiled, streaming, NEON, mobile, batch ----
// algorithms.rs:440-735 and simd_ops.rs:170-193, 230-476.  Their chunk sizes, tile shapes and
// prefetch hints steer a CPU's caches; the element arithmetic is one formula, so each is one call
// of the streaming kernel here, and the cache parameters are accepted and ignored.

// algorithms.rs:443-471
struct CacheAwareParams {
    size_t cache_line_size = 64;
    size_t l1_cache_size = 32 * 1024;
    size_t l2_cache_size = 256 * 1024;
    size_t l3_cache_size = 8 * 1024 * 1024;
    size_t prefetch_distance = 16;
    bool enable_chunking = true;
};

// algorithms.rs:473-522: q = clamp(round(x * (1/scale)) + zp, -128, 127), f32 carrier.
inline Result<Unit> quantize_per_tensor_affine_cache_aware(const std::vector<float> &input, float scale,
                                                           int32_t zero_point, std::vector<float> &output,
                                                           const CacheAwareParams & /*cache_params*/) {
    return quantize_per_tensor_affine_simd(input, scale, zero_point, output);  // same checks, same messages
}

// algorithms.rs:581-635
inline Result<Unit> quantize_matrix_cache_friendly(const std::vector<float> &matrix, size_t rows, size_t cols,
                                                   float scale, int32_t zero_point, std::vector<float> &output,
                                                   const CacheAwareParams & /*cache_params*/) {
    if (matrix.size() != rows * cols || output.size() != rows * cols)
        return TorshError::invalid_argument("Matrix dimensions don't match buffer sizes");
    return quantize_per_tensor_affine_simd(matrix, scale, zero_point, output);
}

// algorithms.rs:638-674
inline Result<Unit> quantize_streaming_with_prefetch(const std::vector<float> &input, float scale, int32_t zero_point,
                                                     std::vector<float> &output,
                                                     const CacheAwareParams & /*cache_params*/) {
    return quantize_per_tensor_affine_simd(input, scale, zero_point, output);
}

// algorithms.rs:711-735: every branch of the reference's size switch ends in the same arithmetic.
inline Result<Unit> quantize_with_cache_optimization(const std::vector<float> &input, float scale, int32_t zero_point,
                                                     std::vector<float> &output,
                                                     const CacheAwareParams * /*cache_params*/ = nullptr) {
    return quantize_per_tensor_affine_simd(input, scale, zero_point, output);
}

// simd_ops.rs:264-272
struct TensorStats {
    float min = 0, max = 0, mean = 0, std_dev = 0, variance = 0;
};

namespace detail {
inline Result<hipq_tensor_stats> tensor_stats(const std::vector<float> &data, bool one_pass) {
    if (data.empty()) return TorshError::invalid_argument("Cannot calculate stats of empty tensor");
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
    TORSH_TRY(ds, hip::DeviceBuffer::alloc(ctx, sizeof(hipq_tensor_stats)));
    TORSH_CHECK(hip::check(hipq_tensor_stats_f32(ctx, dx.as<float>(), data.size(), one_pass ? 1 : 0,
                                                 ds.as<hipq_tensor_stats>())));
    TORSH_TRY(st, ds.to_host<hipq_tensor_stats>(1));
    return st[0];
}
}  // namespace detail

// simd_ops.rs:230-262: range, f64 mean, population variance from a second pass.
inline Result<TensorStats> calculate_tensor_stats_simd(const std::vector<float> &data) {
    TORSH_TRY(st, detail::tensor_stats(data, false));
    return TensorStats{st.min_val, st.max_val, st.mean, st.std_dev, st.variance};
}

// algorithms.rs:525-578: (min, max, mean, std_dev) from the raw moments.
inline Result<std::tuple<float, float, float, float>> calculate_tensor_stats_cache_optimized(
    const std::vector<float> &data, const CacheAwareParams & /*cache_params*/) {
    TORSH_TRY(st, detail::tensor_stats(data, true));
    return std::make_tuple(st.min_val, st.max_val, st.mean, st.std_dev);
}

// simd_ops.rs:170-193: the same parameters for every tensor of the batch.
inline Result<Unit> quantize_batch_consistent_simd(const std::vector<const std::vector<float> *> &tensors, float scale,
                                                   int32_t zero_point, std::vector<std::vector<float> *> &outputs) {
    if (tensors.size() != outputs.size())
        return TorshError::invalid_argument("Number of input tensors must match output tensors");
    for (size_t i = 0; i < tensors.size(); ++i)
        TORSH_CHECK(quantize_per_tensor_affine_simd(*tensors[i], scale, zero_point, *outputs[i]));
    return Unit{};
}

// simd_ops.rs:302-350 and 354-387 (compiled for aarch64 only in the reference; same arithmetic).
inline Result<Unit> quantize_neon_optimized(const std::vector<float> &input, float scale, int32_t zero_point,
                                            std::vector<float> &output) {
    return quantize_per_tensor_affine_simd(input, scale, zero_point, output);
}
inline Result<std::pair<float, float>> find_min_max_neon(const std::vector<float> &data) {
    return find_min_max_simd(data);
}

// simd_ops.rs:390-446: int8 output; with use_reduced_precision and more than 256 elements the
// rounding is floor(x * inv + 0.5).
inline Result<Unit> quantize_mobile_optimized(const std::vector<float> &input, float scale, int32_t zero_point,
                                              std::vector<int8_t> &output, bool use_reduced_precision) {
    if (input.size() != output.size())
        return TorshError::invalid_argument("Input and output length mismatch");
    if (scale <= 0.0f) return TorshError::invalid_argument("Scale must be positive");
    if (input.empty()) return Unit{};
    const int32_t mode = HIPQ_FORM_MUL_INV |
                         ((use_reduced_precision && input.size() > 256) ? HIPQ_ROUND_FLOOR_HALF_UP : HIPQ_ROUND_HALF_AWAY);
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, input.data(), input.size()));
    TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, input.size()));
    TORSH_CHECK(hip::check(hipq_quantize_per_tensor_f32_i8(ctx, dx.as<float>(), input.size(), scale, zero_point, mode,
                                                           dq.as<int8_t>())));
    TORSH_TRY(q, dq.to_host<int8_t>(input.size()));
    output = std::move(q);
    return Unit{};
}

// ---- tensor-level functions (algorithms.rs) ----

using QuantizedTriple = std::tuple<Tensor, float, int32_t>;

// algorithms.rs:277-315.  len > 64: x * (1/scale) form; otherwise x / scale.  Clamp is the
// i8 range whatever the dtype, as in the reference.
inline Result<QuantizedTriple> quantize_per_tensor_affine(const Tensor &tensor, float scale, int32_t zero_point) {
    if (scale <= 0.0f) return TorshError::invalid_argument("Scale must be positive");
    const std::vector<float> &data = tensor.as_slice();
    std::vector<float> q(data.size());
    if (!data.empty()) {
        const int32_t mode =
            (data.size() > 64 && detail::is_simd_available()) ? HIPQ_FORM_MUL_INV : HIPQ_FORM_DIV;
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
        TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, data.size() * sizeof(float)));
        TORSH_CHECK(hip::check(hipq_quantize_per_tensor_f32_carrier(ctx, dx.as<float>(), data.size(), scale,
                                                                    zero_point, mode, -128, 127, dq.as<float>())));
        TORSH_TRY(out, dq.to_host<float>(data.size()));
        q = std::move(out);
    }
    TORSH_TRY(t, Tensor::from_data(std::move(q), tensor.shape().dims()));
    return QuantizedTriple{std::move(t), scale, zero_point};
}

// algorithms.rs:245-274: always x / scale, int8 tensor out.
inline Result<std::tuple<TensorI8, float, int32_t>> quantize_per_tensor_affine_i8(const Tensor &tensor, float scale,
                                                                                  int32_t zero_point) {
    if (scale <= 0.0f) return TorshError::invalid_argument("Scale must be positive");
    const std::vector<float> &data = tensor.as_slice();
    std::vector<int8_t> q(data.size());
    if (!data.empty()) {
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
        TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, data.size()));
        TORSH_CHECK(hip::check(hipq_quantize_per_tensor_f32_i8(ctx, dx.as<float>(), data.size(), scale, zero_point,
                                                               HIPQ_FORM_DIV, dq.as<int8_t>())));
        TORSH_TRY(out, dq.to_host<int8_t>(data.size()));
        q = std::move(out);
    }
    TORSH_TRY(t, TensorI8::from_data(std::move(q), tensor.shape().dims()));
    return std::make_tuple(std::move(t), scale, zero_point);
}

// algorithms.rs:318-355
inline Result<Tensor> dequantize_per_tensor_affine(const Tensor &tensor, float scale, int32_t zero_point) {
    if (scale <= 0.0f) return TorshError::invalid_argument("Scale must be positive");
    const std::vector<float> &data = tensor.as_slice();
    std::vector<float> y(data.size());
    if (!data.empty()) {
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(dq, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
        TORSH_TRY(dy, hip::DeviceBuffer::alloc(ctx, data.size() * sizeof(float)));
        TORSH_CHECK(hip::check(hipq_dequantize_carrier_f32(ctx, dq.as<float>(), data.size(), scale, zero_point,
                                                           dy.as<float>())));
        TORSH_TRY(out, dy.to_host<float>(data.size()));
        y = std::move(out);
    }
    return Tensor::from_data(std::move(y), tensor.shape().dims());
}

inline Result<Tensor> dequantize(const Tensor &tensor, float scale, int32_t zero_point) {
    return dequantize_per_tensor_affine(tensor, scale, zero_point);
}

// algorithms.rs:85-123: range on the device, parameters by the scalar formulas above,
// then quantize_per_tensor_affine.  The tensor is uploaded once for both device passes.
inline Result<QuantizedTriple> quantize_tensor_auto(const Tensor &tensor, DType dtype, QScheme scheme) {
    const std::vector<float> &data = tensor.as_slice();
    if (data.empty()) return TorshError::invalid_argument("Cannot quantize empty tensor");
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
    TORSH_TRY(dmm, hip::DeviceBuffer::alloc(ctx, 2 * sizeof(float)));
    TORSH_CHECK(hip::check(hipq_minmax_f32(ctx, dx.as<float>(), data.size(), dmm.as<float>())));
    TORSH_TRY(mm, dmm.to_host<float>(2));
    float scale;
    int32_t zero_point;
    if (scheme == QScheme::PerTensorAffine) {
        TORSH_TRY(p, calculate_affine_quantization_params(mm[0], mm[1], dtype));
        scale = p.first, zero_point = p.second;
    } else if (scheme == QScheme::PerTensorSymmetric) {
        TORSH_TRY(p, calculate_symmetric_quantization_params(mm[0], mm[1], dtype));
        scale = p.first, zero_point = p.second;
    } else {
        return TorshError::invalid_argument("Unsupported scheme for auto quantization");
    }
    if (scale <= 0.0f) return TorshError::invalid_argument("Scale must be positive");
    const int32_t mode = (data.size() > 64 && detail::is_simd_available()) ? HIPQ_FORM_MUL_INV : HIPQ_FORM_DIV;
    TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, data.size() * sizeof(float)));
    TORSH_CHECK(hip::check(hipq_quantize_per_tensor_f32_carrier(ctx, dx.as<float>(), data.size(), scale, zero_point,
                                                                mode, -128, 127, dq.as<float>())));
    TORSH_TRY(q, dq.to_host<float>(data.size()));
    TORSH_TRY(t, Tensor::from_data(std::move(q), tensor.shape().dims()));
    return QuantizedTriple{std::move(t), scale, zero_point};
}

inline Result<Tensor> quantize_per_tensor(const Tensor &tensor, float scale, int32_t zero_point, DType /*dtype*/) {
    TORSH_TRY(r, quantize_per_tensor_affine(tensor, scale, zero_point));
    return std::move(std::get<0>(r));
}

using PerChannelTriple = std::tuple<Tensor, std::vector<float>, std::vector<int32_t>>;

// algorithms.rs:126-242: per-channel range, parameters and x / scale quantization along `axis`;
// values come back in the f32 carrier.  The device path covers DType::I8.
inline Result<PerChannelTriple> quantize_per_channel_auto(const Tensor &tensor, size_t axis, DType dtype,
                                                          QScheme scheme) {
    const std::vector<size_t> &shape = tensor.shape().dims();
    if (axis >= shape.size()) return TorshError::invalid_argument("Axis out of bounds");
    int32_t flavor;
    if (scheme == QScheme::PerChannelAffine) flavor = HIPQ_PARAMS_AFFINE;
    else if (scheme == QScheme::PerChannelSymmetric) flavor = HIPQ_PARAMS_SYMMETRIC;
    else return TorshError::invalid_argument("Unsupported scheme for per-channel quantization");
    if (dtype != DType::I8)
        return TorshError::not_implemented("quantize_per_channel_auto on the HIP path supports DType::I8 only");
    const size_t channels = shape[axis];
    size_t outer = 1, inner = 1;
    for (size_t d = 0; d < axis; ++d) outer *= shape[d];
    for (size_t d = axis + 1; d < shape.size(); ++d) inner *= shape[d];
    const std::vector<float> &data = tensor.as_slice();
    std::vector<float> carrier(data.size());
    std::vector<float> scales(channels);
    std::vector<int32_t> zps(channels);
    if (!data.empty()) {
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
        TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, data.size()));
        TORSH_TRY(ds, hip::DeviceBuffer::alloc(ctx, channels * sizeof(float)));
        TORSH_TRY(dz, hip::DeviceBuffer::alloc(ctx, channels * sizeof(int32_t)));
        const int32_t zero = 0;
        TORSH_TRY(dst, hip::DeviceBuffer::from_host(ctx, &zero, 1));
        TORSH_CHECK(hip::check(hipq_quantize_per_channel_auto_f32_i8(ctx, dx.as<float>(), outer, channels, inner,
                                                                     flavor, HIPQ_FORM_DIV, dq.as<int8_t>(),
                                                                     ds.as<float>(), dz.as<int32_t>(),
                                                                     dst.as<int32_t>())));
        TORSH_TRY(st, dst.to_host<int32_t>(1));
        if (st[0] != HIPQ_SUCCESS)  // a channel's range was not finite (or min > max)
            return TorshError::invalid_argument("Min and max values must be finite");
        TORSH_TRY(q, dq.to_host<int8_t>(data.size()));
        TORSH_TRY(s, ds.to_host<float>(channels));
        TORSH_TRY(z, dz.to_host<int32_t>(channels));
        for (size_t i = 0; i < q.size(); ++i) carrier[i] = static_cast<float>(q[i]);
        scales = std::move(s);
        zps = std::move(z);
    }
    TORSH_TRY(t, Tensor::from_data(std::move(carrier), shape));
    return PerChannelTriple{std::move(t), std::move(scales), std::move(zps)};
}

// specialized.hpp (included below)
inline Result<QuantizedTriple> quantize_int4_per_tensor(const Tensor &tensor, const QuantConfig &config);
inline Result<QuantizedTriple> quantize_int4_per_channel(const Tensor &tensor, size_t axis, const QuantConfig &config);
inline Result<QuantizedTriple> quantize_binary(const Tensor &tensor);
inline Result<QuantizedTriple> quantize_ternary(const Tensor &tensor);
inline Result<QuantizedTriple> quantize_group_wise(const Tensor &tensor, size_t axis, size_t group_size,
                                                   const QuantConfig &config);

// algorithms.rs:30-66
inline Result<QuantizedTriple> quantize_with_config(const Tensor &tensor, const QuantConfig &config) {
    TORSH_CHECK(config.validate());
    switch (config.scheme) {
    case QScheme::PerTensorAffine:
    case QScheme::PerTensorSymmetric: return quantize_tensor_auto(tensor, config.dtype, config.scheme);
    case QScheme::PerChannelAffine:
    case QScheme::PerChannelSymmetric: {
        const size_t axis = config.ch_axis.value_or(0);
        TORSH_TRY(r, quantize_per_channel_auto(tensor, axis, config.dtype, config.scheme));
        // First channel's parameters, for compatibility (algorithms.rs:44-45).
        const float s0 = std::get<1>(r).empty() ? 1.0f : std::get<1>(r)[0];
        const int32_t z0 = std::get<2>(r).empty() ? 0 : std::get<2>(r)[0];
        return QuantizedTriple{std::move(std::get<0>(r)), s0, z0};
    }
    case QScheme::GroupWise:
        return quantize_group_wise(tensor, config.ch_axis.value_or(0), config.group_size.value_or(32), config);
    case QScheme::Int4PerTensor: return quantize_int4_per_tensor(tensor, config);
    case QScheme::Int4PerChannel: return quantize_int4_per_channel(tensor, config.ch_axis.value_or(0), config);
    case QScheme::Binary: return quantize_binary(tensor);
    case QScheme::Ternary: return quantize_ternary(tensor);
    case QScheme::MixedPrecision:
        return TorshError::invalid_argument("Mixed precision quantization requires specialized API");
    }
    return TorshError::invalid_argument("unknown quantization scheme");
}

inline Result<QuantizedTriple> quantize_auto(const Tensor &tensor, const QuantConfig &config) {
    return quantize_with_config(tensor, config);
}

}  // namespace quantization
}  // namespace torsh

#include "specialized.hpp"
