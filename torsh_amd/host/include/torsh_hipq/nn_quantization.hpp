// torsh::nn::quantization and torsh::dtype::quantized — the two remaining "quantize a value" flavours
// of the reference, mirrored over the torsh_hipq C-ABI.
//
//   torsh-nn:   QuantizationParams::{symmetric, asymmetric, quantize, dequantize}
//               crates/torsh-nn/src/quantization/mod.rs:123-193
//               quantize_value_symmetric / _asymmetric, dequantize_value_*  ops.rs:153-172
//               per_channel_quantize_weights                                 ops.rs:296-373
//               Values go through Rust's `as i32` before the zero point is added (a NaN gives the code
//               `zero_point`), per-channel scales have no zero guard, and negative int8 codes travel as
//               256 + q in the f32 carrier (`as i8 as u8 as f32`).
//   torsh-core: QInt8 / QUInt8 / QInt32::{quantize, dequantize}
//               crates/torsh-core/src/dtype/quantized.rs:129-140, 285-296, 606-617
//               The zero point is added BEFORE rounding: round(v / scale + zp).
// Tensor-sized work runs on the device (hipq_quantize_per_tensor_f32_carrier with HIPQ_FORM_INT_CAST,
// hipq_quantize_per_group_auto_f32_i8 with HIPQ_PARAMS_NN_*, hipq_quantize_per_tensor_f32_i8 / _u8 with
// HIPQ_FORM_ZP_BEFORE_ROUND); the scalar types are scalar code in the reference and stay scalar here.
#pragma once

#include <algorithm>
#include <cmath>
#include <limits>

#include "core.hpp"

namespace torsh {
namespace nn {
namespace quantization {

enum class QuantizationScheme { Symmetric, Asymmetric, Dynamic, Static };

struct QuantizationParams {
    float scale = 1.0f;
    int32_t zero_point = 0;
    int32_t qmin = -128, qmax = 127;
    DType src_dtype = DType::F32;
    DType dst_dtype = DType::I8;

    static Result<std::pair<int32_t, int32_t>> range_of(DType dst) {
        switch (dst) {
        case DType::I8: return std::make_pair(-128, 127);
        case DType::U8: return std::make_pair(0, 255);
        case DType::I16: return std::make_pair(-32768, 32767);
        default: return TorshError::invalid_argument("Unsupported quantization dtype");  // the reference panics
        }
    }
    static Result<QuantizationParams> symmetric(float scale, DType src, DType dst) {
        TORSH_TRY(r, range_of(dst));
        return QuantizationParams{scale, 0, r.first, r.second, src, dst};
    }
    static Result<QuantizationParams> asymmetric(float scale, int32_t zero_point, DType src, DType dst) {
        TORSH_TRY(r, range_of(dst));
        return QuantizationParams{scale, zero_point, r.first, r.second, src, dst};
    }

    // quantize_tensor (ops.rs:16-35): int8 and int16 use the symmetric value formula (the zero point is
    // ignored), uint8 the asymmetric one; the result is the f32 carrier.
    Result<Tensor> quantize(const Tensor &tensor) const {
        if (dst_dtype != DType::I8 && dst_dtype != DType::U8 && dst_dtype != DType::I16)
            return TorshError::invalid_argument("Unsupported quantization target dtype");
        if (!(scale > 0.0f)) return TorshError::invalid_argument("Scale must be positive");
        const std::vector<float> &x = tensor.as_slice();
        std::vector<float> q(x.size());
        if (!x.empty()) {
            TORSH_TRY(ctx, hip::Runtime::ctx());
            TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, x.data(), x.size()));
            TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, x.size() * sizeof(float)));
            const int32_t zp = dst_dtype == DType::U8 ? zero_point : 0;
            TORSH_CHECK(hip::check(hipq_quantize_per_tensor_f32_carrier(ctx, dx.as<float>(), x.size(), scale, zp,
                                                                        HIPQ_FORM_DIV | HIPQ_FORM_INT_CAST, qmin, qmax,
                                                                        dq.as<float>())));
            TORSH_TRY(h, dq.to_host<float>(x.size()));
            q = std::move(h);
        }
        return Tensor::from_data(std::move(q), tensor.shape().dims());
    }

    // dequantize_tensor (ops.rs:38-57): (round(q) as i32 - zp) as f32 * scale, zp = 0 unless uint8.  The
    // carrier holds integers, so the device's (q - zp) * scale is the same value.
    Result<Tensor> dequantize(const Tensor &tensor) const {
        if (dst_dtype != DType::I8 && dst_dtype != DType::U8 && dst_dtype != DType::I16) {
            if (src_dtype == DType::F32) return tensor;  // "treat them as dequantized already"
            return TorshError::invalid_argument("Unsupported dequantization source dtype");
        }
        // (the reference does not look at the scale; the device entry point refuses a non-positive one)
        if (!(scale > 0.0f)) return TorshError::invalid_argument("Scale must be positive");
        const std::vector<float> &q = tensor.as_slice();
        std::vector<float> y(q.size());
        if (!q.empty()) {
            TORSH_TRY(ctx, hip::Runtime::ctx());
            TORSH_TRY(dq, hip::DeviceBuffer::from_host(ctx, q.data(), q.size()));
            TORSH_TRY(dy, hip::DeviceBuffer::alloc(ctx, q.size() * sizeof(float)));
            const int32_t zp = dst_dtype == DType::U8 ? zero_point : 0;
            TORSH_CHECK(hip::check(hipq_dequantize_carrier_f32(ctx, dq.as<float>(), q.size(), scale, zp, dy.as<float>())));
            TORSH_TRY(h, dy.to_host<float>(q.size()));
            y = std::move(h);
        }
        return Tensor::from_data(std::move(y), tensor.shape().dims());
    }
};

// per_channel_quantize_weights (ops.rs:296-373): channels along dimension 0; Symmetric -> int8 codes carried
// as `as i8 as u8 as f32` (256 + q for negatives), Asymmetric -> uint8 codes; one QuantizationParams per
// channel.  Target dtype I8 always uses the symmetric value formula, U8 the asymmetric one, as there.
inline Result<std::pair<Tensor, std::vector<QuantizationParams>>> per_channel_quantize_weights(
    const Tensor &weights, QuantizationScheme scheme, DType target_dtype) {
    if (scheme != QuantizationScheme::Symmetric && scheme != QuantizationScheme::Asymmetric)
        return TorshError::invalid_argument("Unsupported quantization scheme for per-channel quantization");
    if (target_dtype != DType::I8 && target_dtype != DType::U8)
        return TorshError::invalid_argument("Unsupported target dtype");
    const std::vector<size_t> &dims = weights.shape().dims();
    if (dims.empty()) return TorshError::invalid_argument("weights need a channel dimension");
    const size_t channels = dims[0], per = channels ? weights.numel() / channels : 0;
    std::vector<QuantizationParams> params;
    std::vector<float> carrier(weights.numel());
    if (channels == 0 || per == 0) return std::make_pair(Tensor::from_data(std::move(carrier), dims).unwrap(), params);
    const bool sym = scheme == QuantizationScheme::Symmetric;
    const bool as_i8 = target_dtype == DType::I8;
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dw, hip::DeviceBuffer::from_host(ctx, weights.as_slice().data(), weights.numel()));
    TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, weights.numel()));
    TORSH_TRY(ds, hip::DeviceBuffer::alloc(ctx, channels * sizeof(float)));
    TORSH_TRY(dz, hip::DeviceBuffer::alloc(ctx, channels * sizeof(int32_t)));
    // The parameters follow the scheme; the value formula follows the target dtype (int8: symmetric formula,
    // i.e. the zero point is not added).  The two agree except for Asymmetric + I8 / Symmetric + U8.
    if (sym != as_i8)
        return TorshError::not_implemented("per_channel_quantize_weights: scheme and target dtype that disagree "
                                           "(Symmetric + U8, Asymmetric + I8) are not offered on the device");
    TORSH_CHECK(hip::check(hipq_quantize_per_group_auto_f32_i8(
        ctx, dw.as<float>(), 1, channels, per, 1, sym ? HIPQ_PARAMS_NN_SYMMETRIC : HIPQ_PARAMS_NN_ASYMMETRIC,
        as_i8 ? -128 : 0, as_i8 ? 127 : 255, HIPQ_FORM_DIV, dq.as<int8_t>(), ds.as<float>(), dz.as<int32_t>(), nullptr)));
    TORSH_TRY(q, dq.to_host<uint8_t>(weights.numel()));
    TORSH_TRY(s, ds.to_host<float>(channels));
    TORSH_TRY(z, dz.to_host<int32_t>(channels));
    for (size_t i = 0; i < q.size(); ++i) carrier[i] = static_cast<float>(q[i]);  // u8 -> f32
    for (size_t c = 0; c < channels; ++c) {
        QuantizationParams p;
        p.scale = s[c];
        p.zero_point = sym ? 0 : z[c];
        p.qmin = as_i8 ? -128 : 0;
        p.qmax = as_i8 ? 127 : 255;
        p.dst_dtype = target_dtype;
        params.push_back(p);
    }
    TORSH_TRY(t, Tensor::from_data(std::move(carrier), dims));
    return std::make_pair(std::move(t), std::move(params));
}

}  // namespace quantization
}  // namespace nn

namespace dtype {
namespace quantized {

// Rust's `f32 as i32`: saturating, NaN -> 0.
inline int32_t f32_as_i32(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return std::numeric_limits<int32_t>::max();
    if (v <= -2147483648.0f) return std::numeric_limits<int32_t>::min();
    return static_cast<int32_t>(v);
}

// crates/torsh-core/src/dtype/quantized.rs:24-140
struct QInt8 {
    int8_t value;
    float scale;
    int8_t zero_point;
    static QInt8 quantize(float v, float scale, int8_t zero_point) {
        const int32_t q = f32_as_i32(std::round(v / scale + static_cast<float>(zero_point)));
        return QInt8{static_cast<int8_t>(std::clamp(q, -128, 127)), scale, zero_point};
    }
    float dequantize() const { return scale * (static_cast<float>(value) - static_cast<float>(zero_point)); }
};

// crates/torsh-core/src/dtype/quantized.rs:219-296
struct QUInt8 {
    uint8_t value;
    float scale;
    uint8_t zero_point;
    static QUInt8 quantize(float v, float scale, uint8_t zero_point) {
        const int32_t q = f32_as_i32(std::round(v / scale + static_cast<float>(zero_point)));
        return QUInt8{static_cast<uint8_t>(std::clamp(q, 0, 255)), scale, zero_point};
    }
    float dequantize() const { return scale * (static_cast<float>(value) - static_cast<float>(zero_point)); }
};

// crates/torsh-core/src/dtype/quantized.rs:540-617: the arithmetic is done in f64.
struct QInt32 {
    int32_t value;
    float scale;
    int32_t zero_point;
    static QInt32 quantize(float v, float scale, int32_t zero_point) {
        double q = std::round(static_cast<double>(v) / static_cast<double>(scale) + static_cast<double>(zero_point));
        if (q != q) return QInt32{0, scale, zero_point};  // `NaN as i32` is 0
        q = std::min(std::max(q, -2147483648.0), 2147483647.0);
        return QInt32{static_cast<int32_t>(q), scale, zero_point};
    }
    float dequantize() const {
        return scale * static_cast<float>(static_cast<double>(value) - static_cast<double>(zero_point));
    }
};

// Slices of QInt8 / QUInt8 values on the device: round(v / scale + zp), clamped to the type.
inline Result<std::vector<int8_t>> quantize_slice_qint8(const std::vector<float> &x, float scale, int8_t zero_point) {
    if (!(scale > 0.0f)) return TorshError::invalid_argument("Scale must be positive");
    std::vector<int8_t> out(x.size());
    if (x.empty()) return out;
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, x.data(), x.size()));
    TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, x.size()));
    TORSH_CHECK(hip::check(hipq_quantize_per_tensor_f32_i8(ctx, dx.as<float>(), x.size(), scale, zero_point,
                                                           HIPQ_FORM_ZP_BEFORE_ROUND, dq.as<int8_t>())));
    return dq.to_host<int8_t>(x.size());
}
inline Result<std::vector<uint8_t>> quantize_slice_quint8(const std::vector<float> &x, float scale,
                                                          uint8_t zero_point) {
    if (!(scale > 0.0f)) return TorshError::invalid_argument("Scale must be positive");
    std::vector<uint8_t> out(x.size());
    if (x.empty()) return out;
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, x.data(), x.size()));
    TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, x.size()));
    TORSH_CHECK(hip::check(hipq_quantize_per_tensor_f32_u8(ctx, dx.as<float>(), x.size(), scale, zero_point,
                                                           HIPQ_FORM_ZP_BEFORE_ROUND, dq.as<uint8_t>())));
    return dq.to_host<uint8_t>(x.size());
}

}  // namespace quantized
}  // namespace dtype
}  // namespace torsh
