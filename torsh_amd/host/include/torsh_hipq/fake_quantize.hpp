// Fake quantization for quantization-aware training: quantize, then immediately dequantize, in f32.
// Mirror of crates/torsh-quantization/src/fake_quantize.rs (same function and type names, argument
// meaning and error messages); the element loop runs on the device (hipq_fake_quantize_f32 with the
// division form and the clamp that maps NaN to qmin), the range of fake_quantize_auto through
// hipq_minmax_f32.
#pragma once

#include <algorithm>
#include <cmath>
#include <utility>
#include <vector>

#include "quantization.hpp"

namespace torsh {
namespace quantization {

// fake_quantize_per_tensor_affine, fake_quantize.rs:14-42:
//   q = round(x / scale) + zero_point;  q = q.max(quant_min).min(quant_max);  y = scale * (q - zero_point).
// The reference does not validate the scale; a non-positive one is rejected here as in
// quantize_per_tensor_affine (algorithms.rs:284-288), since 0 or a negative scale is never meant.
inline Result<Tensor> fake_quantize_per_tensor_affine(const Tensor &tensor, float scale, int32_t zero_point,
                                                      int32_t quant_min, int32_t quant_max) {
    const std::vector<float> &data = tensor.as_slice();
    std::vector<float> out(data.size());
    if (!data.empty()) {
        if (!(scale > 0.0f)) return TorshError::invalid_argument("Scale must be positive");
        if (quant_min > quant_max) return TorshError::invalid_argument("quant_min must not exceed quant_max");
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
        TORSH_TRY(dy, hip::DeviceBuffer::alloc(ctx, data.size() * sizeof(float)));
        TORSH_CHECK(hip::check(hipq_fake_quantize_f32(ctx, dx.as<float>(), data.size(), scale, zero_point, nullptr,
                                                      quant_min, quant_max, HIPQ_FORM_DIV | HIPQ_FAKE_NAN_TO_QMIN,
                                                      dy.as<float>())));
        TORSH_TRY(y, dy.to_host<float>(data.size()));
        out = std::move(y);
    }
    return Tensor::from_data(std::move(out), tensor.shape().dims());
}

// fake_quantize, fake_quantize.rs:9-11: the int8 range.
inline Result<Tensor> fake_quantize(const Tensor &tensor, float scale, int32_t zero_point) {
    return fake_quantize_per_tensor_affine(tensor, scale, zero_point, -128, 127);
}

// fake_quantize_per_tensor_symmetric, fake_quantize.rs:45-52: zero point 0.
inline Result<Tensor> fake_quantize_per_tensor_symmetric(const Tensor &tensor, float scale, int32_t quant_min,
                                                         int32_t quant_max) {
    return fake_quantize_per_tensor_affine(tensor, scale, 0, quant_min, quant_max);
}

// FakeQuantize, fake_quantize.rs:55-117: the module form with parameters that calibration updates.
class FakeQuantize {
  public:
    FakeQuantize(float scale, int32_t zero_point, int32_t quant_min, int32_t quant_max)
        : scale_(scale), zero_point_(zero_point), quant_min_(quant_min), quant_max_(quant_max) {}
    static FakeQuantize int8(float scale, int32_t zero_point) { return FakeQuantize(scale, zero_point, -128, 127); }
    static FakeQuantize uint8(float scale, int32_t zero_point) { return FakeQuantize(scale, zero_point, 0, 255); }
    void enable() { enabled_ = true; }
    void disable() { enabled_ = false; }
    bool enabled() const { return enabled_; }
    // Disabled: the input comes back unchanged (fake_quantize.rs:98-100).
    Result<Tensor> forward(const Tensor &tensor) const {
        if (!enabled_) return Tensor::from_data(tensor.as_slice(), tensor.shape().dims());
        return fake_quantize_per_tensor_affine(tensor, scale_, zero_point_, quant_min_, quant_max_);
    }
    void update_params(float scale, int32_t zero_point) {
        scale_ = scale;
        zero_point_ = zero_point;
    }
    float scale() const { return scale_; }
    int32_t zero_point() const { return zero_point_; }

  private:
    float scale_;
    int32_t zero_point_, quant_min_, quant_max_;
    bool enabled_ = true;
};

// The parameters fake_quantize_auto derives (fake_quantize.rs:129-147), exposed for tests and callers
// that want to keep them: the range is widened to include 0, a zero scale becomes 1, and only the
// affine scheme has a zero point.
inline Result<std::pair<float, int32_t>> fake_quantize_auto_params(const Tensor &tensor, DType dtype, QScheme scheme) {
    int32_t quant_min, quant_max;
    if (dtype == DType::I8) {
        quant_min = -128, quant_max = 127;
    } else if (dtype == DType::U8) {
        quant_min = 0, quant_max = 255;
    } else {
        return TorshError::invalid_argument("Unsupported quantization dtype");
    }
    if (scheme != QScheme::PerTensorAffine && scheme != QScheme::PerTensorSymmetric)
        return TorshError::invalid_argument("Quantization scheme not yet implemented");
    float min_val = 0.0f, max_val = 0.0f;  // the folds of an empty tensor end at min(inf, 0) and max(-inf, 0)
    if (tensor.numel() > 0) {
        TORSH_TRY(mm, find_min_max_simd(tensor.as_slice()));
        min_val = std::fmin(mm.first, 0.0f);  // f32::min / f32::max: the operand that is not NaN
        max_val = std::fmax(mm.second, 0.0f);
    }
    float scale = (max_val - min_val) / static_cast<float>(quant_max - quant_min);
    if (scale == 0.0f) scale = 1.0f;
    int32_t zero_point = 0;
    if (scheme == QScheme::PerTensorAffine) {
        const float z = std::fmin(std::fmax(std::round(static_cast<float>(quant_min) - min_val / scale),
                                            static_cast<float>(quant_min)),
                                  static_cast<float>(quant_max));
        zero_point = detail::f32_as_i32(z);
    }
    return std::make_pair(scale, zero_point);
}

// fake_quantize_auto, fake_quantize.rs:119-157.
inline Result<Tensor> fake_quantize_auto(const Tensor &tensor, DType dtype, QScheme scheme) {
    TORSH_TRY(p, fake_quantize_auto_params(tensor, dtype, scheme));
    const int32_t quant_min = dtype == DType::I8 ? -128 : 0, quant_max = dtype == DType::I8 ? 127 : 255;
    return fake_quantize_per_tensor_affine(tensor, p.first, p.second, quant_min, quant_max);
}

}  // namespace quantization
}  // namespace torsh
