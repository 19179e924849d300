// torsh::backend::quantization — byte-level quantized tensors and the QuantizationOps
// interface of crates/torsh-backend, with a HIP implementation next to the reference's
// CpuQuantizationOps.
//
//   QuantizedDType, QuantizationScheme   crates/torsh-backend/src/quantization/types.rs:11-140
//   QuantizationParams                   crates/torsh-backend/src/quantization/params.rs:16-363
//   QuantizedTensor                      crates/torsh-backend/src/quantization/tensor.rs:21-143
//   QuantizationOps (trait)              crates/torsh-backend/src/quantization/ops.rs:22-168
//   CpuQuantizationOps (what each method computes)  ops.rs:185-200, 295-660
//   VnniQuantizationOps::vnni_qmatmul_int8          crates/torsh-backend/src/quantization/specialized.rs:82-201
//
// HipQuantizationOps covers Int8 and UInt8 with per-tensor parameters for every method of the
// trait; sub-byte and 16-bit types, logarithmic parameters and channel-wise operands of qadd /
// qrelu return NotImplemented (they stay on the CPU implementation).
#pragma once

#include <cmath>
#include <optional>

#include "core.hpp"

namespace torsh {
namespace backend {
namespace quantization {

template <typename T>
using BackendResult = Result<T>;

enum class QuantizedDType { Int8, UInt8, Int16, UInt16, Int4, UInt4, Binary };
enum class QuantizationScheme { Linear, Symmetric, Asymmetric, Logarithmic, BlockWise, ChannelWise };

// types.rs:40-51
inline std::pair<int64_t, int64_t> value_range(QuantizedDType d) {
    switch (d) {
    case QuantizedDType::Int8: return {-128, 127};
    case QuantizedDType::UInt8: return {0, 255};
    case QuantizedDType::Int16: return {-32768, 32767};
    case QuantizedDType::UInt16: return {0, 65535};
    case QuantizedDType::Int4: return {-8, 7};
    case QuantizedDType::UInt4: return {0, 15};
    default: return {0, 1};
    }
}
inline int bits(QuantizedDType d) {
    switch (d) {
    case QuantizedDType::Int8:
    case QuantizedDType::UInt8: return 8;
    case QuantizedDType::Int16:
    case QuantizedDType::UInt16: return 16;
    case QuantizedDType::Int4:
    case QuantizedDType::UInt4: return 4;
    default: return 1;
    }
}
inline bool is_sub_byte(QuantizedDType d) { return bits(d) < 8; }

struct QuantizationParams {
    QuantizedDType dtype = QuantizedDType::UInt8;
    QuantizationScheme scheme = QuantizationScheme::Linear;
    std::vector<float> scale{1.0f};
    std::vector<int32_t> zero_point{0};
    std::optional<size_t> block_size;
    std::optional<float> min_val, max_val;

    static QuantizationParams int8_symmetric() {
        QuantizationParams p;
        p.dtype = QuantizedDType::Int8;
        p.scheme = QuantizationScheme::Symmetric;
        return p;
    }
    static QuantizationParams uint8_asymmetric() {
        QuantizationParams p;
        p.dtype = QuantizedDType::UInt8;
        p.scheme = QuantizationScheme::Asymmetric;
        p.zero_point = {128};
        return p;
    }
    static QuantizationParams make(float scale, int32_t zero_point) {  // QuantizationParams::new, params.rs:65-76
        QuantizationParams p;
        p.dtype = QuantizedDType::UInt8;
        p.scheme = QuantizationScheme::Asymmetric;
        p.scale = {scale};
        p.zero_point = {zero_point};
        return p;
    }
    static QuantizationParams channel_wise(size_t num_channels, QuantizedDType dtype) {
        QuantizationParams p;
        p.dtype = dtype;
        p.scheme = QuantizationScheme::ChannelWise;
        p.scale.assign(num_channels, 1.0f);
        p.zero_point.assign(num_channels, 0);
        return p;
    }

    // params.rs:282-363.  Symmetric: scale = 2*max_range/(qmax-qmin); asymmetric (also Linear,
    // BlockWise, ChannelWise): scale = (max-min)/(qmax-qmin), zp = clamp(round(qmin - min/scale)).
    Result<Unit> from_statistics(float mn, float mx) {
        if (mn > mx) return TorshError::invalid_argument("min_val must be <= max_val");
        if (!std::isfinite(mn) || !std::isfinite(mx))
            return TorshError::invalid_argument("min_val and max_val must be finite");
        min_val = mn;
        max_val = mx;
        const auto [qmin_i, qmax_i] = value_range(dtype);
        const float qmin = static_cast<float>(qmin_i), qmax = static_cast<float>(qmax_i);
        switch (scheme) {
        case QuantizationScheme::Symmetric: {
            const float max_range = std::fmax(std::fabs(mx), std::fabs(mn));
            scale[0] = max_range == 0.0f ? 1.0f : (2.0f * max_range) / (qmax - qmin);
            zero_point[0] = 0;
            return Unit{};
        }
        case QuantizationScheme::Logarithmic:
            return TorshError::not_implemented("logarithmic quantization is outside the int8 HIP path");
        default:
            if (mx == mn) {
                scale[0] = 1.0f;
                zero_point[0] = static_cast<int32_t>(qmin);
            } else {
                scale[0] = (mx - mn) / (qmax - qmin);
                float z = std::round(qmin - mn / scale[0]);
                z = z < qmin ? qmin : z;
                z = z > qmax ? qmax : z;
                zero_point[0] = (z != z) ? 0 : static_cast<int32_t>(z);
            }
            return Unit{};
        }
    }

    // params.rs:214-275
    Result<Unit> validate() const {
        if (scale.size() != zero_point.size())
            return TorshError::invalid_argument("Scale and zero_point vectors must have the same length");
        for (size_t i = 0; i < scale.size(); ++i)
            if (scale[i] <= 0.0f || !std::isfinite(scale[i]))
                return TorshError::invalid_argument("Scale factor at index " + std::to_string(i) +
                                                    " must be positive and finite, got " + std::to_string(scale[i]));
        const auto [qmin, qmax] = value_range(dtype);
        for (size_t i = 0; i < zero_point.size(); ++i)
            if (zero_point[i] < qmin || zero_point[i] > qmax)
                return TorshError::invalid_argument("Zero point at index " + std::to_string(i) + " (" +
                                                    std::to_string(zero_point[i]) + ") is outside valid range [" +
                                                    std::to_string(qmin) + ", " + std::to_string(qmax) + "]");
        if (scheme == QuantizationScheme::Symmetric)
            for (size_t i = 0; i < zero_point.size(); ++i)
                if (zero_point[i] != 0)
                    return TorshError::invalid_argument("Symmetric quantization requires zero_point[" +
                                                        std::to_string(i) + "] = 0, got " +
                                                        std::to_string(zero_point[i]));
        if (scheme == QuantizationScheme::BlockWise && !block_size)
            return TorshError::invalid_argument("Block-wise quantization requires block_size to be specified");
        if (scheme == QuantizationScheme::ChannelWise && scale.size() == 1)
            return TorshError::invalid_argument("Channel-wise quantization requires multiple scale/zero_point values");
        return Unit{};
    }
    bool is_per_channel() const { return scheme == QuantizationScheme::ChannelWise && scale.size() > 1; }
};

struct QuantizedTensor {
    std::vector<uint8_t> data;
    std::vector<size_t> shape;
    QuantizationParams params;

    static size_t data_size(size_t n, QuantizedDType d) {
        if (d == QuantizedDType::Int4 || d == QuantizedDType::UInt4) return (n + 1) / 2;
        if (d == QuantizedDType::Binary) return (n + 7) / 8;
        return n * (bits(d) / 8);
    }
    // tensor.rs:56-78
    static Result<QuantizedTensor> from_data(std::vector<uint8_t> data, std::vector<size_t> shape,
                                             QuantizationParams params) {
        size_t n = 1;
        for (size_t d : shape) n *= d;
        const size_t expect = data_size(n, params.dtype);
        if (data.size() != expect)
            return TorshError::invalid_argument("Data size mismatch: expected " + std::to_string(expect) +
                                                " bytes, got " + std::to_string(data.size()) + " bytes");
        QuantizedTensor t;
        t.data = std::move(data);
        t.shape = std::move(shape);
        t.params = std::move(params);
        return t;
    }
    size_t num_elements() const {
        size_t n = 1;
        for (size_t d : shape) n *= d;
        return n;
    }
    size_t ndim() const { return shape.size(); }
};

// ops.rs:22-168
class QuantizationOps {
  public:
    virtual ~QuantizationOps() = default;
    virtual BackendResult<std::vector<uint8_t>> quantize_f32(const std::vector<float> &input,
                                                             const QuantizationParams &params) const = 0;
    virtual BackendResult<std::vector<float>> dequantize_f32(const std::vector<uint8_t> &input,
                                                             const QuantizationParams &params) const = 0;
    virtual BackendResult<QuantizedTensor> qmatmul(const QuantizedTensor &a, const QuantizedTensor &b) const = 0;
    virtual BackendResult<QuantizedTensor> qconv2d(const QuantizedTensor &input, const QuantizedTensor &weight,
                                                   const QuantizedTensor *bias, std::pair<size_t, size_t> stride,
                                                   std::pair<size_t, size_t> padding) const = 0;
    virtual BackendResult<QuantizedTensor> qadd(const QuantizedTensor &a, const QuantizedTensor &b) const = 0;
    virtual BackendResult<QuantizedTensor> qrelu(const QuantizedTensor &input) const = 0;
    virtual BackendResult<QuantizationParams> calibrate(const std::vector<std::vector<float>> &samples,
                                                        QuantizedDType target_dtype) const = 0;
};

class HipQuantizationOps : public QuantizationOps {
  public:
    // ops.rs:295-364: q = clamp(round(v / scale) + zp, qmin, qmax), stored as a byte.
    // ChannelWise = contiguous equal chunks, one (scale, zp) per chunk.
    BackendResult<std::vector<uint8_t>> quantize_f32(const std::vector<float> &input,
                                                     const QuantizationParams &params) const override {
        if (input.empty()) return std::vector<uint8_t>{};
        TORSH_CHECK(params.validate());
        if (params.dtype != QuantizedDType::Int8 && params.dtype != QuantizedDType::UInt8)
            return TorshError::not_implemented("Quantization on the HIP path is implemented for Int8 and UInt8");
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, input.data(), input.size()));
        TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, input.size()));
        TORSH_CHECK(quantize_on_device(ctx, dx.as<float>(), input.size(), params, dq.as<uint8_t>()));
        return dq.to_host<uint8_t>(input.size());
    }

    // ops.rs:366-435: y = scale * (q - zp).
    BackendResult<std::vector<float>> dequantize_f32(const std::vector<uint8_t> &input,
                                                     const QuantizationParams &params) const override {
        if (input.empty()) return std::vector<float>{};
        TORSH_CHECK(params.validate());
        if (params.dtype != QuantizedDType::Int8 && params.dtype != QuantizedDType::UInt8)
            return TorshError::not_implemented("Dequantization on the HIP path is implemented for Int8 and UInt8");
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(dq, hip::DeviceBuffer::from_host(ctx, input.data(), input.size()));
        TORSH_TRY(dy, hip::DeviceBuffer::alloc(ctx, input.size() * sizeof(float)));
        const size_t n = input.size(), channels = params.scale.size();
        if (params.is_per_channel()) {
            if (n % channels != 0)
                return TorshError::invalid_argument("Channel-wise data length is not a multiple of the channel count");
            const size_t chunk = n / channels;
            if (params.dtype == QuantizedDType::Int8) {
                TORSH_TRY(ds, hip::DeviceBuffer::from_host(ctx, params.scale.data(), channels));
                TORSH_TRY(dz, hip::DeviceBuffer::from_host(ctx, params.zero_point.data(), channels));
                TORSH_CHECK(hip::check(hipq_dequantize_per_channel_i8_f32(ctx, dq.as<int8_t>(), 1, channels, chunk,
                                                                          ds.as<float>(), dz.as<int32_t>(),
                                                                          dy.as<float>())));
            } else {
                for (size_t c = 0; c < channels; ++c)
                    TORSH_CHECK(hip::check(hipq_dequantize_u8_f32(ctx, dq.as<uint8_t>() + c * chunk, chunk,
                                                                  params.scale[c], params.zero_point[c],
                                                                  dy.as<float>() + c * chunk)));
            }
        } else if (params.dtype == QuantizedDType::Int8) {
            TORSH_CHECK(hip::check(hipq_dequantize_i8_f32(ctx, dq.as<int8_t>(), n, params.scale[0],
                                                          params.zero_point[0], dy.as<float>())));
        } else {
            TORSH_CHECK(hip::check(hipq_dequantize_u8_f32(ctx, dq.as<uint8_t>(), n, params.scale[0],
                                                          params.zero_point[0], dy.as<float>())));
        }
        return dy.to_host<float>(n);
    }

    // Raw int32 accumulators of a [M,K] x b [K,N] (both Int8), the exact integer part of
    // specialized.rs:187-198.
    BackendResult<std::vector<int32_t>> qmatmul_i32(const QuantizedTensor &a, const QuantizedTensor &b) const {
        TORSH_CHECK(check_matmul(a, b, /*backend_error=*/false));
        const size_t m = a.shape[0], k = a.shape[1], n = b.shape[1];
        if (m * n == 0) return std::vector<int32_t>{};
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(acc, matmul_acc(ctx, a, b));
        return acc.to_host<int32_t>(m * n);
    }

    // specialized.rs:82-121 + 175-201: bytes = clamp(acc, -128, 127) as u8, parameters copied from `a`.
    BackendResult<QuantizedTensor> vnni_qmatmul_int8(const QuantizedTensor &a, const QuantizedTensor &b) const {
        TORSH_CHECK(check_matmul(a, b, /*backend_error=*/true));
        const size_t m = a.shape[0], k = a.shape[1], n = b.shape[1];
        std::vector<uint8_t> bytes(m * n);
        if (m * n) {
            TORSH_TRY(ctx, hip::Runtime::ctx());
            const std::vector<uint8_t> bt = transpose_kn(b.data, k, n);
            TORSH_TRY(da, hip::DeviceBuffer::from_host(ctx, a.data.data(), a.data.size()));
            TORSH_TRY(dw, hip::DeviceBuffer::from_host(ctx, bt.data(), bt.size()));
            const float one = 1.0f;
            const std::vector<float> ones(n, 1.0f);
            TORSH_TRY(dsa, hip::DeviceBuffer::from_host(ctx, &one, 1));
            TORSH_TRY(dsw, hip::DeviceBuffer::from_host(ctx, ones.data(), n));
            TORSH_TRY(dout, hip::DeviceBuffer::alloc(ctx, m * n));
            // With unit scales the requantize epilogue is clamp(acc): |acc| beyond 2^24 loses low bits
            // in the float conversion but is far outside [-128, 127] either way.
            TORSH_CHECK(hip::check(hipq_linear_i8_i8(ctx, da.as<int8_t>(), dsa.as<float>(), 0, dw.as<int8_t>(),
                                                     dsw.as<float>(), nullptr, m, n, k, 1.0f, 0,
                                                     HIPQ_ROUND_HALF_AWAY | HIPQ_FORM_DIV, dout.as<int8_t>())));
            TORSH_TRY(out, dout.to_host<uint8_t>(m * n));
            bytes = std::move(out);
        }
        QuantizedTensor t;
        t.data = std::move(bytes);
        t.shape = {m, n};
        t.params = a.params;
        return t;
    }

    // ops.rs:437-477 with the accumulation done in int32 on the matrix cores instead of the f32
    // triple loop: out_f = acc * (s_a * s_b) for zero-point-free Int8 operands (the exact value
    // of the sum the reference rounds term by term), then output parameters from the range of
    // out_f (`a`'s dtype and scheme) and requantization, as the reference does.
    BackendResult<QuantizedTensor> qmatmul(const QuantizedTensor &a, const QuantizedTensor &b) const override {
        if (a.ndim() != 2 || b.ndim() != 2) return TorshError::invalid_argument("qmatmul requires 2D tensors");
        if (a.shape[1] != b.shape[0])
            return TorshError::invalid_argument("qmatmul dimension mismatch: a has K=" + std::to_string(a.shape[1]) +
                                                " but b has K=" + std::to_string(b.shape[0]));
        TORSH_CHECK(a.params.validate());
        TORSH_CHECK(b.params.validate());
        if (a.params.dtype != QuantizedDType::Int8 || b.params.dtype != QuantizedDType::Int8 ||
            a.params.scale.size() != 1 || b.params.scale.size() != 1 || a.params.zero_point[0] != 0 ||
            b.params.zero_point[0] != 0)
            return TorshError::not_implemented("qmatmul on the HIP path takes per-tensor Int8 operands with zero point 0");
        const size_t m = a.shape[0], k = a.shape[1], n = b.shape[1];
        if (m * n == 0 || k == 0) return TorshError::invalid_argument("qmatmul of an empty tensor");
        TORSH_TRY(ctx, hip::Runtime::ctx());
        const std::vector<uint8_t> bt = transpose_kn(b.data, k, n);
        TORSH_TRY(da, hip::DeviceBuffer::from_host(ctx, a.data.data(), a.data.size()));
        TORSH_TRY(dw, hip::DeviceBuffer::from_host(ctx, bt.data(), bt.size()));
        const std::vector<float> sw(n, b.params.scale[0]);
        TORSH_TRY(dsa, hip::DeviceBuffer::from_host(ctx, a.params.scale.data(), 1));
        TORSH_TRY(dsw, hip::DeviceBuffer::from_host(ctx, sw.data(), n));
        TORSH_TRY(dout, hip::DeviceBuffer::alloc(ctx, m * n * sizeof(float)));
        TORSH_CHECK(hip::check(hipq_linear_i8_f32(ctx, da.as<int8_t>(), dsa.as<float>(), 0, dw.as<int8_t>(),
                                                  dsw.as<float>(), nullptr, m, n, k, dout.as<float>())));
        return requantize_from_range(ctx, dout, m * n, {m, n}, a.params);
    }

    // ops.rs:479-580 with the integer accumulation of operations.rs:672-713: UInt8 input
    // (per-tensor scale / zero point), Int8 filters (per-tensor or one scale per output
    // channel), optional quantized bias (dequantized to f32 and added in f32, ops.rs:561),
    // output parameters from the range of the f32 result with the input's dtype and scheme.
    BackendResult<QuantizedTensor> qconv2d(const QuantizedTensor &input, const QuantizedTensor &weight,
                                           const QuantizedTensor *bias, std::pair<size_t, size_t> stride,
                                           std::pair<size_t, size_t> padding) const override {
        if (input.ndim() != 4 || weight.ndim() != 4)
            return TorshError::invalid_argument(
                "qconv2d requires 4D tensors [N, C, H, W] for input and [C_out, C_in, kH, kW] for weight");
        const size_t nb = input.shape[0], c = input.shape[1], h = input.shape[2], w = input.shape[3];
        const size_t oc = weight.shape[0], kh = weight.shape[2], kw = weight.shape[3];
        if (c != weight.shape[1])
            return TorshError::invalid_argument("qconv2d channel mismatch: input C_in=" + std::to_string(c) +
                                                " but weight C_in=" + std::to_string(weight.shape[1]));
        TORSH_CHECK(input.params.validate());
        TORSH_CHECK(weight.params.validate());
        if (input.params.dtype != QuantizedDType::UInt8 || input.params.scale.size() != 1 ||
            weight.params.dtype != QuantizedDType::Int8)
            return TorshError::not_implemented("qconv2d on the HIP path takes a per-tensor UInt8 input and Int8 filters");
        for (int32_t z : weight.params.zero_point)
            if (z != 0) return TorshError::not_implemented("qconv2d on the HIP path takes symmetric filters");
        if (weight.params.scale.size() != 1 && weight.params.scale.size() != oc)
            return TorshError::invalid_argument("filter scales must be per tensor or one per output channel");
        if (stride.first == 0 || stride.second == 0) return TorshError::invalid_argument("stride must be positive");
        if (h + 2 * padding.first < kh || w + 2 * padding.second < kw)
            return TorshError::invalid_argument("kernel larger than the padded input");
        const size_t ho = (h + 2 * padding.first - kh) / stride.first + 1;
        const size_t wo = (w + 2 * padding.second - kw) / stride.second + 1;
        const size_t out_n = nb * oc * ho * wo;
        if (out_n == 0) return TorshError::invalid_argument("qconv2d of an empty tensor");
        std::vector<float> sw(oc, weight.params.scale[0]);
        if (weight.params.scale.size() == oc) sw = weight.params.scale;
        std::vector<float> bias_f;
        if (bias) {
            TORSH_TRY(bf, dequantize_f32(bias->data, bias->params));
            bias_f = std::move(bf);
            bias_f.resize(oc, 0.0f);  // missing entries count as 0 (ops.rs:533-536)
        }
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, input.data.data(), input.data.size()));
        TORSH_TRY(dw, hip::DeviceBuffer::from_host(ctx, weight.data.data(), weight.data.size()));
        TORSH_TRY(dsw, hip::DeviceBuffer::from_host(ctx, sw.data(), oc));
        TORSH_TRY(db, hip::DeviceBuffer::from_host(ctx, bias_f.data(), bias_f.size()));
        TORSH_TRY(dout, hip::DeviceBuffer::alloc(ctx, out_n * sizeof(float)));
        TORSH_CHECK(hip::check(hipq_conv2d_u8i8_f32(ctx, dx.as<uint8_t>(), input.params.zero_point[0],
                                                    input.params.scale[0], dw.as<int8_t>(), dsw.as<float>(),
                                                    bias ? db.as<float>() : nullptr, nb, c, h, w, oc, kh, kw,
                                                    stride.first, stride.second, padding.first, padding.second,
                                                    dout.as<float>())));
        return requantize_from_range(ctx, dout, out_n, {nb, oc, ho, wo}, input.params);
    }

    // ops.rs:582-606.  The f32 sum is formed twice from the bytes (once for its range, once to
    // quantize it) and never stored.
    BackendResult<QuantizedTensor> qadd(const QuantizedTensor &a, const QuantizedTensor &b) const override {
        if (a.shape != b.shape) return TorshError::invalid_argument("qadd shape mismatch");
        return elementwise(a, &b);
    }
    // ops.rs:608-624
    BackendResult<QuantizedTensor> qrelu(const QuantizedTensor &input) const override {
        return elementwise(input, nullptr);
    }

    // ops.rs:616-660: global range over all samples, then asymmetric parameters.  The reference
    // skips non-finite values; the device reduction skips NaN only, so samples holding +-Inf are
    // rejected here instead of being filtered.
    BackendResult<QuantizationParams> calibrate(const std::vector<std::vector<float>> &samples,
                                                QuantizedDType target_dtype) const override {
        if (samples.empty()) return TorshError::invalid_argument("Cannot calibrate with empty samples");
        float gmin = INFINITY, gmax = -INFINITY;
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(dmm, hip::DeviceBuffer::alloc(ctx, 2 * sizeof(float)));
        for (const auto &s : samples) {
            if (s.empty()) continue;
            TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, s.data(), s.size()));
            TORSH_CHECK(hip::check(hipq_minmax_f32(ctx, dx.as<float>(), s.size(), dmm.as<float>())));
            TORSH_TRY(mm, dmm.to_host<float>(2));
            gmin = std::fmin(gmin, mm[0]);
            gmax = std::fmax(gmax, mm[1]);
        }
        if (!std::isfinite(gmin) || !std::isfinite(gmax))
            return TorshError::invalid_argument("No finite values found in calibration samples");
        QuantizationParams p;
        p.dtype = target_dtype;
        p.scheme = QuantizationScheme::Asymmetric;
        TORSH_CHECK(p.from_statistics(gmin, gmax));
        return p;
    }

  private:
    // qadd (b != nullptr) / qrelu on per-tensor Int8 / UInt8 operands.
    static BackendResult<QuantizedTensor> elementwise(const QuantizedTensor &a, const QuantizedTensor *b) {
        auto supported = [](const QuantizationParams &p) {
            return (p.dtype == QuantizedDType::Int8 || p.dtype == QuantizedDType::UInt8) && p.scale.size() == 1 &&
                   p.zero_point.size() == 1;
        };
        TORSH_CHECK(a.params.validate());
        if (b) TORSH_CHECK(b->params.validate());
        if (!supported(a.params) || (b && !supported(b->params)))
            return TorshError::not_implemented("qadd / qrelu on the HIP path take per-tensor Int8 or UInt8 operands");
        if (a.params.scheme == QuantizationScheme::Logarithmic)
            return TorshError::not_implemented("logarithmic quantization is outside the int8 HIP path");
        const size_t n = a.data.size();
        if (b && b->data.size() != n) return TorshError::invalid_argument("qadd shape mismatch");
        // An empty tensor has range (+inf, -inf), which from_statistics rejects (params.rs:283-297).
        if (n == 0) return TorshError::invalid_argument("min_val must be <= max_val");
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(da, hip::DeviceBuffer::from_host(ctx, a.data.data(), n));
        hip::DeviceBuffer db;
        if (b) {
            TORSH_TRY(tmp, hip::DeviceBuffer::from_host(ctx, b->data.data(), n));
            db = std::move(tmp);
        }
        TORSH_TRY(dout, hip::DeviceBuffer::alloc(ctx, n));
        TORSH_TRY(dp, hip::DeviceBuffer::alloc(ctx, sizeof(hipq_qparams)));
        const int32_t flavor = a.params.scheme == QuantizationScheme::Symmetric ? HIPQ_PARAMS_BACKEND_SYMMETRIC
                                                                               : HIPQ_PARAMS_BACKEND_ASYMMETRIC;
        const int32_t out_dtype = a.params.dtype == QuantizedDType::Int8 ? HIPQ_DTYPE_I8 : HIPQ_DTYPE_U8;
        const int32_t a_signed = a.params.dtype == QuantizedDType::Int8;
        if (b)
            TORSH_CHECK(hip::check(hipq_qadd_u8(ctx, da.as<uint8_t>(), a_signed, a.params.scale[0],
                                                a.params.zero_point[0], db.as<uint8_t>(),
                                                b->params.dtype == QuantizedDType::Int8, b->params.scale[0],
                                                b->params.zero_point[0], n, flavor, out_dtype, dout.as<uint8_t>(),
                                                dp.as<hipq_qparams>())));
        else
            TORSH_CHECK(hip::check(hipq_qrelu_u8(ctx, da.as<uint8_t>(), a_signed, a.params.scale[0],
                                                 a.params.zero_point[0], n, flavor, out_dtype, dout.as<uint8_t>(),
                                                 dp.as<hipq_qparams>())));
        TORSH_TRY(p, dp.to_host<hipq_qparams>(1));
        if (p[0].status != HIPQ_SUCCESS) return TorshError::invalid_argument("min_val and max_val must be finite");
        QuantizationParams out_params = a.params;
        out_params.scale[0] = p[0].scale;
        out_params.zero_point[0] = p[0].zero_point;
        out_params.min_val = p[0].min_val;
        out_params.max_val = p[0].max_val;
        TORSH_TRY(bytes, dout.to_host<uint8_t>(n));
        return QuantizedTensor::from_data(std::move(bytes), a.shape, std::move(out_params));
    }

    static std::vector<uint8_t> transpose_kn(const std::vector<uint8_t> &b, size_t k, size_t n) {
        std::vector<uint8_t> t(b.size());
        for (size_t l = 0; l < k; ++l)
            for (size_t j = 0; j < n; ++j) t[j * k + l] = b[l * n + j];
        return t;
    }

    static Result<Unit> check_matmul(const QuantizedTensor &a, const QuantizedTensor &b, bool backend_error) {
        auto err = [&](const char *m) {
            return backend_error ? TorshError::backend(m) : TorshError::invalid_argument(m);
        };
        if (a.ndim() != 2 || b.ndim() != 2) return err("VNNI matrix multiplication requires 2D tensors");
        if (a.shape[1] != b.shape[0]) return err("Matrix dimensions incompatible for multiplication");
        if (a.data.size() != a.shape[0] * a.shape[1] || b.data.size() != b.shape[0] * b.shape[1])
            return err("int8 matrix multiplication takes one byte per element");
        return Unit{};
    }

    static Result<hip::DeviceBuffer> matmul_acc(hipq_ctx *ctx, const QuantizedTensor &a, const QuantizedTensor &b) {
        const size_t m = a.shape[0], k = a.shape[1], n = b.shape[1];
        const std::vector<uint8_t> bt = transpose_kn(b.data, k, n);
        TORSH_TRY(da, hip::DeviceBuffer::from_host(ctx, a.data.data(), a.data.size()));
        TORSH_TRY(dw, hip::DeviceBuffer::from_host(ctx, bt.data(), bt.size()));
        TORSH_TRY(dacc, hip::DeviceBuffer::alloc(ctx, m * n * sizeof(int32_t)));
        TORSH_CHECK(hip::check(hipq_gemm_i8_i32(ctx, da.as<int8_t>(), dw.as<int8_t>(), m, n, k, dacc.as<int32_t>())));
        return std::move(dacc);
    }

    static Result<Unit> quantize_on_device(hipq_ctx *ctx, const float *dx, size_t n, const QuantizationParams &params,
                                           uint8_t *dq) {
        const size_t channels = params.scale.size();
        const int32_t mode = HIPQ_FORM_DIV | HIPQ_ROUND_HALF_AWAY;
        if (params.is_per_channel()) {
            if (n % channels != 0)
                return TorshError::invalid_argument("Channel-wise data length is not a multiple of the channel count");
            const size_t chunk = n / channels;
            if (params.dtype == QuantizedDType::Int8) {
                TORSH_TRY(ds, hip::DeviceBuffer::from_host(ctx, params.scale.data(), channels));
                TORSH_TRY(dz, hip::DeviceBuffer::from_host(ctx, params.zero_point.data(), channels));
                return hip::check(hipq_quantize_per_channel_f32_i8(ctx, dx, 1, channels, chunk, ds.as<float>(),
                                                                   dz.as<int32_t>(), mode,
                                                                   reinterpret_cast<int8_t *>(dq)));
            }
            for (size_t c = 0; c < channels; ++c)
                TORSH_CHECK(hip::check(hipq_quantize_per_tensor_f32_u8(ctx, dx + c * chunk, chunk, params.scale[c],
                                                                       params.zero_point[c], mode, dq + c * chunk)));
            return Unit{};
        }
        if (params.dtype == QuantizedDType::Int8)
            return hip::check(hipq_quantize_per_tensor_f32_i8(ctx, dx, n, params.scale[0], params.zero_point[0], mode,
                                                              reinterpret_cast<int8_t *>(dq)));
        return hip::check(hipq_quantize_per_tensor_f32_u8(ctx, dx, n, params.scale[0], params.zero_point[0], mode, dq));
    }

    // Output parameters from the range of the f32 result (ops.rs:466-476 / 566-579), then quantize.
    static BackendResult<QuantizedTensor> requantize_from_range(hipq_ctx *ctx, const hip::DeviceBuffer &dout, size_t n,
                                                                std::vector<size_t> shape,
                                                                const QuantizationParams &like) {
        TORSH_TRY(dmm, hip::DeviceBuffer::alloc(ctx, 2 * sizeof(float)));
        TORSH_CHECK(hip::check(hipq_minmax_f32(ctx, dout.as<float>(), n, dmm.as<float>())));
        TORSH_TRY(mm, dmm.to_host<float>(2));
        QuantizationParams out_params = like;
        TORSH_CHECK(out_params.from_statistics(mm[0], mm[1]));
        if (out_params.dtype != QuantizedDType::Int8 && out_params.dtype != QuantizedDType::UInt8)
            return TorshError::not_implemented("output dtype must be Int8 or UInt8 on the HIP path");
        // from_statistics rewrites entry 0 only; a channel-wise operand keeps its other entries and
        // the reference then quantizes chunk-wise with them.  Follow that.
        TORSH_CHECK(out_params.validate());
        TORSH_TRY(dq, hip::DeviceBuffer::alloc(ctx, n));
        TORSH_CHECK(quantize_on_device(ctx, dout.as<float>(), n, out_params, dq.as<uint8_t>()));
        TORSH_TRY(bytes, dq.to_host<uint8_t>(n));
        return QuantizedTensor::from_data(std::move(bytes), std::move(shape), std::move(out_params));
    }
};

}  // namespace quantization
}  // namespace backend
}  // namespace torsh
