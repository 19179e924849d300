// torsh::quantization — the special schemes of crates/torsh-quantization/src/specialized.rs that
// quantize_with_config dispatches to, executed on the GPU.  Included at the end of quantization.hpp.
//
//   quantize_int4_per_tensor     specialized.rs:33-65
//   quantize_int4_per_channel    specialized.rs:68-160
//   quantize_binary              specialized.rs:163-188
//   quantize_ternary             specialized.rs:191-238
//   quantize_group_wise          specialized.rs:241-377
//   quantize_mixed_precision, determine_layer_precision, create_precision_config
//                                specialized.rs:379-436 (MixedPrecisionConfig: config.rs:131-154)
//   quantize_binary_learned_threshold, quantize_ternary_adaptive
//                                specialized.rs:439-552
//
// Values come back in the f32 carrier like the reference's.  Two documented differences, both
// only for non-finite inputs: a NaN element quantizes to clamp(0) (the int8 conversion used by the
// device path) where the reference keeps NaN (int4) or yields qmin (group-wise), and a range that
// is not finite is InvalidArgument.  The scale of the binary and ternary schemes is the mean of
// |x| formed from f64 partial sums; the reference adds f32 terms in element order.
#pragma once

#include <map>
#include <optional>
#include <string>

#include "quantization.hpp"

namespace torsh {
namespace quantization {

namespace detail {
// Group-wise quantization of the dense [outer, channels, inner] view (groups of `group`
// consecutive channels, the last may be shorter) with the zero-including range rule and integer
// range [qmin, qmax]; int8 codes, one (scale, zero point) per group.
struct ChannelResult {
    std::vector<int8_t> q;
    std::vector<float> scales;
    std::vector<int32_t> zps;
};
inline Result<ChannelResult> quantize_channels_zero_included(hipq_ctx *ctx, const float *dev_x, size_t outer,
                                                             size_t channels, size_t inner, size_t group,
                                                             int32_t qmin, int32_t qmax) {
    ChannelResult r;
    const size_t total = outer * channels * inner;
    const size_t groups = (channels + group - 1) / group;
    TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, total));
    TORSH_TRY(ds, hip::DeviceBuffer::alloc(ctx, groups * sizeof(float)));
    TORSH_TRY(dz, hip::DeviceBuffer::alloc(ctx, groups * sizeof(int32_t)));
    const int32_t zero = 0;
    TORSH_TRY(dst, hip::DeviceBuffer::from_host(ctx, &zero, 1));
    TORSH_CHECK(hip::check(hipq_quantize_per_group_auto_f32_i8(
        ctx, dev_x, outer, channels, inner, group, HIPQ_PARAMS_ZERO_INCLUDED, qmin, qmax, HIPQ_FORM_DIV,
        dq.as<int8_t>(), ds.as<float>(), dz.as<int32_t>(), dst.as<int32_t>())));
    TORSH_TRY(st, dst.to_host<int32_t>(1));
    if (st[0] != HIPQ_SUCCESS) return TorshError::invalid_argument("Min and max values must be finite");
    TORSH_TRY(q, dq.to_host<int8_t>(total));
    TORSH_TRY(s, ds.to_host<float>(groups));
    TORSH_TRY(z, dz.to_host<int32_t>(groups));
    r.q = std::move(q), r.scales = std::move(s), r.zps = std::move(z);
    return r;
}
inline std::pair<float, int32_t> average_params(const std::vector<float> &scales, const std::vector<int32_t> &zps) {
    float ssum = 0.0f;  // sequential f32 sum over a few channels, as the reference
    int32_t zsum = 0;
    for (float s : scales) ssum += s;
    for (int32_t z : zps) zsum += z;
    const float n = static_cast<float>(scales.size());
    return {ssum / n, f32_as_i32(std::round(static_cast<float>(zsum) / n))};
}
inline Result<Tensor> carrier_tensor(const std::vector<int8_t> &q, const std::vector<size_t> &dims) {
    std::vector<float> c(q.begin(), q.end());
    return Tensor::from_data(std::move(c), dims);
}
}  // namespace detail

// specialized.rs:33-65: range widened to 0, scale = range / 15, values in [-8, 7].
inline Result<QuantizedTriple> quantize_int4_per_tensor(const Tensor &tensor, const QuantConfig & /*config*/) {
    const std::vector<float> &data = tensor.as_slice();
    if (data.empty()) {  // fold over nothing: range (0, 0), scale 1, zero point -8
        TORSH_TRY(t, Tensor::from_data({}, tensor.shape().dims()));
        return QuantizedTriple{std::move(t), 1.0f, -8};
    }
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
    TORSH_TRY(r, detail::quantize_channels_zero_included(ctx, dx.as<float>(), 1, 1, data.size(), 1, -8, 7));
    TORSH_TRY(t, detail::carrier_tensor(r.q, tensor.shape().dims()));
    return QuantizedTriple{std::move(t), r.scales[0], r.zps[0]};
}

// specialized.rs:68-160: per-channel int4; the returned parameters are the averages over channels.
inline Result<QuantizedTriple> quantize_int4_per_channel(const Tensor &tensor, size_t axis,
                                                         const QuantConfig & /*config*/) {
    const std::vector<size_t> &shape = tensor.shape().dims();
    if (axis >= shape.size()) return TorshError::invalid_argument("Axis out of bounds");
    const std::vector<float> &data = tensor.as_slice();
    if (data.empty()) return TorshError::invalid_argument("Cannot quantize empty tensor");
    size_t outer = 1, inner = 1;
    for (size_t d = 0; d < axis; ++d) outer *= shape[d];
    for (size_t d = axis + 1; d < shape.size(); ++d) inner *= shape[d];
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
    TORSH_TRY(r, detail::quantize_channels_zero_included(ctx, dx.as<float>(), outer, shape[axis], inner, 1, -8, 7));
    const auto avg = detail::average_params(r.scales, r.zps);
    TORSH_TRY(t, detail::carrier_tensor(r.q, shape));
    return QuantizedTriple{std::move(t), avg.first, avg.second};
}

namespace detail {
inline Result<QuantizedTriple> sign_scheme(const Tensor &tensor, bool ternary) {
    const std::vector<float> &data = tensor.as_slice();
    if (data.empty()) return TorshError::invalid_argument("Cannot quantize empty tensor");
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
    TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, data.size()));
    TORSH_TRY(dp, hip::DeviceBuffer::alloc(ctx, sizeof(hipq_qparams)));
    TORSH_CHECK(hip::check(ternary ? hipq_quantize_ternary_f32_i8(ctx, dx.as<float>(), data.size(), dq.as<int8_t>(),
                                                                  dp.as<hipq_qparams>())
                                   : hipq_quantize_binary_f32_i8(ctx, dx.as<float>(), data.size(), dq.as<int8_t>(),
                                                                 dp.as<hipq_qparams>())));
    TORSH_TRY(q, dq.to_host<int8_t>(data.size()));
    TORSH_TRY(p, dp.to_host<hipq_qparams>(1));
    TORSH_TRY(t, carrier_tensor(q, tensor.shape().dims()));
    return QuantizedTriple{std::move(t), p[0].scale, 0};
}
}  // namespace detail

// specialized.rs:163-188
inline Result<QuantizedTriple> quantize_binary(const Tensor &tensor) { return detail::sign_scheme(tensor, false); }
// specialized.rs:191-238
inline Result<QuantizedTriple> quantize_ternary(const Tensor &tensor) { return detail::sign_scheme(tensor, true); }

// (tensor, scale, zero_point, threshold)
using ThresholdQuadruple = std::tuple<Tensor, float, int32_t, float>;

namespace detail {
inline Result<ThresholdQuadruple> searched_sign_scheme(const Tensor &tensor, bool adaptive,
                                                       std::optional<float> threshold) {
    const std::vector<float> &data = tensor.as_slice();
    if (data.empty()) return TorshError::invalid_argument("Cannot quantize empty tensor");
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
    TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, data.size()));
    TORSH_TRY(dp, hip::DeviceBuffer::alloc(ctx, sizeof(hipq_qparams)));
    TORSH_CHECK(hip::check(
        adaptive ? hipq_quantize_ternary_adaptive_f32_i8(ctx, dx.as<float>(), data.size(), dq.as<int8_t>(),
                                                         dp.as<hipq_qparams>())
                 : hipq_quantize_binary_learned_threshold_f32_i8(ctx, dx.as<float>(), data.size(),
                                                                 threshold.has_value() ? 1 : 0, threshold.value_or(0.0f),
                                                                 dq.as<int8_t>(), dp.as<hipq_qparams>())));
    TORSH_TRY(q, dq.to_host<int8_t>(data.size()));
    TORSH_TRY(p, dp.to_host<hipq_qparams>(1));
    TORSH_TRY(t, carrier_tensor(q, tensor.shape().dims()));
    return ThresholdQuadruple{std::move(t), p[0].scale, 0, p[0].min_val};
}
}  // namespace detail

// specialized.rs:439-492: the threshold is the given one or mean |x|; |x| <= threshold -> 0, else the
// sign with x >= 0 counted as positive; scale = mean |x| of the values above the threshold.
inline Result<ThresholdQuadruple> quantize_binary_learned_threshold(const Tensor &tensor,
                                                                    std::optional<float> threshold = std::nullopt) {
    return detail::searched_sign_scheme(tensor, false, threshold);
}

// specialized.rs:495-552: the first of the ten thresholds max|x| * (i * 0.1) with the least mean
// squared error of the unit ternary code.
inline Result<ThresholdQuadruple> quantize_ternary_adaptive(const Tensor &tensor) {
    return detail::searched_sign_scheme(tensor, true, std::nullopt);
}

// config.rs:131-154
struct MixedPrecisionConfig {
    std::map<std::string, DType> layer_precision{{"embedding", DType::I8}, {"attention", DType::F16},
                                                 {"output", DType::F32}};
    DType default_precision = DType::I8;
    float sensitivity_threshold = 0.1f;
};

// specialized.rs:401-412: the first pattern contained in the layer name decides.  (The reference walks
// a HashMap, so which of several matching patterns wins is unspecified there; here it is the
// alphabetically first.)
inline DType determine_layer_precision(const std::string &layer_name, const MixedPrecisionConfig &config) {
    for (const auto &[pattern, precision] : config.layer_precision)
        if (layer_name.find(pattern) != std::string::npos) return precision;
    return config.default_precision;
}

// specialized.rs:414-436
inline QuantConfig create_precision_config(DType precision) {
    switch (precision) {
    case DType::I8: return QuantConfig::int8();
    case DType::U8: return QuantConfig::uint8();
    case DType::F16:
    case DType::F32: {
        QuantConfig c;
        c.dtype = precision;
        c.enable_fake_quant = false;
        return c;
    }
    default: return QuantConfig::int8();
    }
}

// specialized.rs:241-377: groups of `group_size` consecutive channels along `axis` share one
// (scale, zero point), the last group may be shorter; integer range from config.get_qint_range().
inline Result<QuantizedTriple> quantize_group_wise(const Tensor &tensor, size_t axis, size_t group_size,
                                                   const QuantConfig &config) {
    const std::vector<size_t> &shape = tensor.shape().dims();
    if (axis >= shape.size()) return TorshError::invalid_argument("Axis out of bounds");
    if (group_size == 0) return TorshError::invalid_argument("Group size must be greater than 0");
    const auto [qmin, qmax] = config.get_qint_range();
    if (qmin < -128 || qmax > 127 || qmin >= qmax)
        return TorshError::not_implemented("group-wise quantization on the HIP path needs a range inside [-128, 127]");
    const std::vector<float> &data = tensor.as_slice();
    const size_t channels = shape[axis];
    size_t outer = 1, inner = 1;
    for (size_t d = 0; d < axis; ++d) outer *= shape[d];
    for (size_t d = axis + 1; d < shape.size(); ++d) inner *= shape[d];
    if (data.empty()) {  // no group has members: averages fall back to (1.0, 0), specialized.rs:361-371
        TORSH_TRY(t, Tensor::from_data({}, shape));
        return QuantizedTriple{std::move(t), 1.0f, 0};
    }
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
    TORSH_TRY(r, detail::quantize_channels_zero_included(ctx, dx.as<float>(), outer, channels, inner, group_size, qmin, qmax));
    const std::vector<int8_t> &q = r.q;
    const std::vector<float> &scales = r.scales;
    const std::vector<int32_t> &zps = r.zps;
    const auto avg = detail::average_params(scales, zps);
    TORSH_TRY(t, detail::carrier_tensor(q, shape));
    return QuantizedTriple{std::move(t), avg.first, avg.second};
}

// specialized.rs:379-399: every tensor through quantize_with_config with the configuration of the
// precision its layer name selects.  As in the reference, the F16 / F32 configurations still carry
// the default per-tensor affine scheme, whose integer range falls back to int8 (algorithms.rs:425-433).
inline Result<std::map<std::string, QuantizedTriple>> quantize_mixed_precision(
    const std::map<std::string, Tensor> &tensors, const MixedPrecisionConfig &config) {
    std::map<std::string, QuantizedTriple> results;
    for (const auto &[layer_name, tensor] : tensors) {
        const QuantConfig layer_config = create_precision_config(determine_layer_precision(layer_name, config));
        TORSH_TRY(r, quantize_with_config(tensor, layer_config));
        results.emplace(layer_name, std::move(r));
    }
    return results;
}

}  // namespace quantization
}  // namespace torsh
