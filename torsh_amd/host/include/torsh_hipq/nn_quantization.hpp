// torsh::nn::quantization and torsh::dtype::quantized — the two remaining "quantize a value" flavours
// of the reference, mirrored over the torsh_hipq C-ABI.
//
//   torsh-nn:   QuantizationParams::{symmetric, asymmetric, quantize, dequantize}
//               crates/torsh-nn/src/quantization/mod.rs:123-193
//               quantize_value_symmetric / _asymmetric, dequantize_value_*  ops.rs:153-172
//               per_channel_quantize_weights                                 ops.rs:296-373
//               quantized_matmul_int8 / quantized_conv2d_int8 / quantized_relu_int8   ops.rs:175-294
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

// Rust's `f32 as i32`: saturating, NaN -> 0.
inline int32_t dtype_cast_i32(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return std::numeric_limits<int32_t>::max();
    if (v <= -2147483648.0f) return std::numeric_limits<int32_t>::min();
    return static_cast<int32_t>(v);
}

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

namespace detail {
// The integer codes behind an f32 carrier of 8-bit values: `value.round() as i32` as the reference's dequantize
// reads them (ops.rs:110-143).  `as_u8`: uint8 codes; else int8.  Values outside the type are refused (a carrier of
// int16 codes has no 8-bit operand on the device).
inline Result<std::vector<uint8_t>> carrier_bytes(const Tensor &t, bool as_u8, const char *what) {
    const std::vector<float> &v = t.as_slice();
    std::vector<uint8_t> out(v.size());
    for (size_t i = 0; i < v.size(); ++i) {
        const float r = std::round(v[i]);
        if (!(r >= (as_u8 ? 0.0f : -128.0f) && r <= (as_u8 ? 255.0f : 127.0f)))
            return TorshError::invalid_argument(std::string(what) + ": carrier value outside the " +
                                                (as_u8 ? "uint8" : "int8") + " range");
        out[i] = as_u8 ? static_cast<uint8_t>(r) : static_cast<uint8_t>(static_cast<int8_t>(r));
    }
    return out;
}
inline bool is_8bit(DType d) { return d == DType::I8 || d == DType::U8; }
}  // namespace detail

// quantized_matmul_int8 (ops.rs:175-194): a [M,K] and b [K,N] are f32 carriers of quantized values; the result is
// the carrier of quantize_tensor(dequantize(a) x dequantize(b), output_params).  On the device the product is
// exact in int32 and scaled once, acc * (s_a * s_b), where the reference sums f32 products in an order its
// Tensor::matmul does not fix: the two agree to within that summation error (one output code).  int8 operands
// (the function's name; their zero points are not used, as in dequantize_from_int8); any 8- or 16-bit output type.
inline Result<Tensor> quantized_matmul_int8(const Tensor &a, const Tensor &b, const QuantizationParams &a_params,
                                            const QuantizationParams &b_params, const QuantizationParams &output_params) {
    const std::vector<size_t> &da = a.shape().dims(), &db = b.shape().dims();
    if (da.size() != 2 || db.size() != 2) return TorshError::invalid_argument("quantized_matmul_int8 requires 2D tensors");
    if (da[1] != db[0])
        return TorshError::invalid_argument("quantized_matmul_int8 dimension mismatch: a has K=" + std::to_string(da[1]) +
                                            " but b has K=" + std::to_string(db[0]));
    if (a_params.dst_dtype != DType::I8 || b_params.dst_dtype != DType::I8)
        return TorshError::not_implemented("quantized_matmul_int8 on the HIP path takes int8 operands");
    if (!(a_params.scale > 0.0f) || !(b_params.scale > 0.0f) || !(output_params.scale > 0.0f))
        return TorshError::invalid_argument("Scale must be positive");
    const size_t m = da[0], k = da[1], n = db[1];
    if (m * n == 0 || k == 0) return TorshError::invalid_argument("quantized_matmul_int8 of an empty tensor");
    TORSH_TRY(qa, detail::carrier_bytes(a, false, "quantized_matmul_int8"));
    TORSH_TRY(qb, detail::carrier_bytes(b, false, "quantized_matmul_int8"));
    std::vector<uint8_t> bt(n * k);  // [K,N] -> [N,K], once
    for (size_t l = 0; l < k; ++l)
        for (size_t j = 0; j < n; ++j) bt[j * k + l] = qb[l * n + j];
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(d_a, hip::DeviceBuffer::from_host(ctx, qa.data(), qa.size()));
    TORSH_TRY(d_w, hip::DeviceBuffer::from_host(ctx, bt.data(), bt.size()));
    const std::vector<float> sw(n, b_params.scale);
    TORSH_TRY(d_sa, hip::DeviceBuffer::from_host(ctx, &a_params.scale, 1));
    TORSH_TRY(d_sw, hip::DeviceBuffer::from_host(ctx, sw.data(), n));
    if (output_params.dst_dtype == DType::I8) {
        // int8 out: the fused requantizing epilogue, q = clamp(round(v / s_out), -128, 127) (the symmetric value
        // formula: the output zero point is not used)
        TORSH_TRY(d_q, hip::DeviceBuffer::alloc(ctx, m * n));
        TORSH_CHECK(hip::check(hipq_linear_i8_i8(ctx, d_a.as<int8_t>(), d_sa.as<float>(), 0, d_w.as<int8_t>(),
                                                 d_sw.as<float>(), nullptr, m, n, k, output_params.scale, 0, HIPQ_FORM_DIV,
                                                 d_q.as<int8_t>())));
        TORSH_TRY(q, d_q.to_host<int8_t>(m * n));
        std::vector<float> carrier(q.begin(), q.end());
        for (float &v : carrier) v = std::min(std::max(v, float(output_params.qmin)), float(output_params.qmax));
        return Tensor::from_data(std::move(carrier), {m, n});
    }
    TORSH_TRY(d_out, hip::DeviceBuffer::alloc(ctx, m * n * sizeof(float)));
    TORSH_CHECK(hip::check(hipq_linear_i8_f32(ctx, d_a.as<int8_t>(), d_sa.as<float>(), 0, d_w.as<int8_t>(),
                                              d_sw.as<float>(), nullptr, m, n, k, d_out.as<float>())));
    TORSH_TRY(f, d_out.to_host<float>(m * n));
    TORSH_TRY(ft, Tensor::from_data(std::move(f), {m, n}));
    return output_params.quantize(ft);
}

// quantized_conv2d_int8 (ops.rs:197-237): input [N,C,H,W] (int8 or uint8 carrier), weight [OC,IC,KH,KW] (int8
// carrier, one scale), optional bias (a carrier with its own parameters, dequantized on the host as the reference
// does before the convolution), dilation 1, one group.  int32 accumulation on the device, then
// acc * (s_in * s_w) + bias and quantize_tensor with the caller's output parameters; the same relation to the
// reference's f32 convolution as for the product above.
inline Result<Tensor> quantized_conv2d_int8(const Tensor &input, const Tensor &weight, const Tensor *bias,
                                            const QuantizationParams &input_params,
                                            const QuantizationParams &weight_params,
                                            const QuantizationParams *bias_params,
                                            const QuantizationParams &output_params, std::pair<size_t, size_t> stride,
                                            std::pair<size_t, size_t> padding) {
    const std::vector<size_t> &di = input.shape().dims(), &dw = weight.shape().dims();
    if (di.size() != 4 || dw.size() != 4)
        return TorshError::invalid_argument("quantized_conv2d_int8 requires 4D tensors [N, C, H, W] and [C_out, C_in, kH, kW]");
    if (di[1] != dw[1]) return TorshError::invalid_argument("quantized_conv2d_int8: channel mismatch between input and weight");
    if (!detail::is_8bit(input_params.dst_dtype) || weight_params.dst_dtype != DType::I8)
        return TorshError::not_implemented("quantized_conv2d_int8 on the HIP path takes an 8-bit input and int8 weights");
    if (stride.first == 0 || stride.second == 0) return TorshError::invalid_argument("stride must be positive");
    if (!(input_params.scale > 0.0f) || !(weight_params.scale > 0.0f) || !(output_params.scale > 0.0f))
        return TorshError::invalid_argument("Scale must be positive");
    const size_t nb = di[0], c = di[1], h = di[2], w = di[3], oc = dw[0], kh = dw[2], kw = dw[3];
    if (h + 2 * padding.first < kh || w + 2 * padding.second < kw)
        return TorshError::invalid_argument("quantized_conv2d_int8: kernel larger than the padded input");
    const size_t ho = (h + 2 * padding.first - kh) / stride.first + 1, wo = (w + 2 * padding.second - kw) / stride.second + 1;
    if (input.numel() == 0 || weight.numel() == 0) return TorshError::invalid_argument("quantized_conv2d_int8 of an empty tensor");
    const bool in_u8 = input_params.dst_dtype == DType::U8;
    TORSH_TRY(qx, detail::carrier_bytes(input, in_u8, "quantized_conv2d_int8"));
    TORSH_TRY(qw, detail::carrier_bytes(weight, false, "quantized_conv2d_int8"));
    // The device convolves uint8 codes with a zero point; int8 codes (whose zero point the reference's dequantize
    // does not use) are the uint8 codes q + 128 with zero point 128.
    int32_t zp_in = input_params.zero_point;
    if (!in_u8) {
        for (uint8_t &v : qx) v = static_cast<uint8_t>(v + 128);
        zp_in = 128;
    }
    std::vector<float> bias_f;
    if (bias && bias_params) {  // dequantize_tensor(bias, bias_params), ops.rs:216-220
        if (bias->numel() != oc) return TorshError::invalid_argument("quantized_conv2d_int8: bias length must equal C_out");
        bias_f.resize(oc);
        const bool b_u8 = bias_params->dst_dtype == DType::U8;
        for (size_t o = 0; o < oc; ++o) {
            const int32_t q = dtype_cast_i32(std::round(bias->as_slice()[o]));
            bias_f[o] = b_u8 ? static_cast<float>(q - bias_params->zero_point) * bias_params->scale
                             : static_cast<float>(q) * bias_params->scale;
        }
    }
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(d_x, hip::DeviceBuffer::from_host(ctx, qx.data(), qx.size()));
    TORSH_TRY(d_w, hip::DeviceBuffer::from_host(ctx, qw.data(), qw.size()));
    const std::vector<float> sw(oc, weight_params.scale);
    TORSH_TRY(d_sw, hip::DeviceBuffer::from_host(ctx, sw.data(), oc));
    hip::DeviceBuffer d_bias;
    if (!bias_f.empty()) {
        TORSH_TRY(db, hip::DeviceBuffer::from_host(ctx, bias_f.data(), oc));
        d_bias = std::move(db);
    }
    const float *bias_dev = bias_f.empty() ? nullptr : d_bias.as<float>();
    const size_t total = nb * oc * ho * wo;
    if (output_params.dst_dtype == DType::I8) {
        TORSH_TRY(d_q, hip::DeviceBuffer::alloc(ctx, total));
        TORSH_CHECK(hip::check(hipq_conv2d_u8i8_i8(ctx, d_x.as<uint8_t>(), zp_in, input_params.scale, d_w.as<int8_t>(),
                                                   d_sw.as<float>(), bias_dev, nb, c, h, w, oc, kh, kw, stride.first,
                                                   stride.second, padding.first, padding.second, output_params.scale, 0,
                                                   HIPQ_FORM_DIV, d_q.as<int8_t>())));
        TORSH_TRY(q, d_q.to_host<int8_t>(total));
        std::vector<float> carrier(q.begin(), q.end());
        for (float &v : carrier) v = std::min(std::max(v, float(output_params.qmin)), float(output_params.qmax));
        return Tensor::from_data(std::move(carrier), {nb, oc, ho, wo});
    }
    TORSH_TRY(d_out, hip::DeviceBuffer::alloc(ctx, total * sizeof(float)));
    TORSH_CHECK(hip::check(hipq_conv2d_u8i8_f32(ctx, d_x.as<uint8_t>(), zp_in, input_params.scale, d_w.as<int8_t>(),
                                                d_sw.as<float>(), bias_dev, nb, c, h, w, oc, kh, kw, stride.first,
                                                stride.second, padding.first, padding.second, d_out.as<float>())));
    TORSH_TRY(f, d_out.to_host<float>(total));
    TORSH_TRY(ft, Tensor::from_data(std::move(f), {nb, oc, ho, wo}));
    return output_params.quantize(ft);
}

// quantized_relu_int8 (ops.rs:261-294): max(value, zero) on the carrier, zero = the code of the real value 0 by
// the asymmetric value formula, clamp((round(0 / scale) as i32) + zero_point, qmin, qmax); the output parameters are
// not used, as in the reference.  On the device as a clamp from below of the carrier's integer values (carriers
// hold integers: every quantize of this module writes `q as f32`).
inline Result<Tensor> quantized_relu_int8(const Tensor &input, const QuantizationParams &input_params,
                                          const QuantizationParams & /*output_params*/) {
    const std::vector<float> &x = input.as_slice();
    const float r0 = std::round(0.0f / input_params.scale);  // NaN for a zero scale: `as i32` makes it 0
    const int64_t z = static_cast<int64_t>(dtype_cast_i32(r0)) + input_params.zero_point;
    const int32_t zero_q = static_cast<int32_t>(std::min<int64_t>(std::max<int64_t>(z, input_params.qmin), input_params.qmax));
    std::vector<float> y(x.size());
    if (!x.empty()) {
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, x.data(), x.size()));
        TORSH_TRY(dy, hip::DeviceBuffer::alloc(ctx, x.size() * sizeof(float)));
        TORSH_CHECK(hip::check(hipq_quantize_per_tensor_f32_carrier(ctx, dx.as<float>(), x.size(), 1.0f, 0,
                                                                    HIPQ_FORM_DIV | HIPQ_FORM_INT_CAST, zero_q, 1 << 24,
                                                                    dy.as<float>())));
        TORSH_TRY(h, dy.to_host<float>(x.size()));
        y = std::move(h);
    }
    return Tensor::from_data(std::move(y), input.shape().dims());
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
