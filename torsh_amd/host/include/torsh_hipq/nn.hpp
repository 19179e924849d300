// torsh::nn — the Module interface of crates/torsh-nn and the quantized Linear / Conv2d
// modules that sit behind it.
//
//   Module (trait)     crates/torsh-nn/src/core/mod.rs:294-404   forward(&self,&Tensor)->Result<Tensor>,
//                                                                parameters() keyed "weight" / "bias"
//   Linear             crates/torsh-nn/src/layers/linear.rs:16-62  weight [in, out], input.matmul(weight) + bias
//   Conv2d             crates/torsh-nn/src/layers/conv/types.rs:108-160, conv2d_traits.rs:23-56
//                      weight [oc, ic/groups, kh, kw], bias broadcast [1, oc, 1, 1]
// The reference has no quantized Module; QuantizedLinear / QuantizedConv2d are what its
// `Linear::forward` / `Conv2d::forward` call sites switch to.  They keep int8 weights, scales
// and bias resident on the device and run:
//   QuantizedLinear : dynamic int8 activations (per tensor: algorithms.rs:85-123 symmetric;
//                     per token: algorithms.rs:126-242 axis 0) -> int32 GEMM -> acc*(s_a*s_w[n]) + bias[n]
//   QuantizedConv2d : asymmetric uint8 activations (crates/torsh-backend/src/quantization/params.rs:343-363)
//                     -> int32 conv (crates/torsh-quantization/src/operations.rs:672-713)
//                     -> bias + requantize to int8 with a calibrated output scale (operations.rs:716-724)
#pragma once

#include <cmath>
#include <map>

#include "core.hpp"
#include "serialize.hpp"

namespace torsh {
namespace nn {

using Parameter = Tensor;

class Module {
  public:
    virtual ~Module() = default;
    virtual Result<Tensor> forward(const Tensor &input) const = 0;
    virtual std::map<std::string, Parameter> parameters() const { return {}; }
    virtual std::map<std::string, Parameter> named_parameters() const { return parameters(); }
    virtual bool training() const { return training_; }
    virtual void train() { set_training(true); }
    virtual void eval() { set_training(false); }
    virtual void set_training(bool t) { training_ = t; }

  private:
    bool training_ = true;
};

// Parameter holder with the reference's layout.  Its fp32 forward is the reference's CPU
// code and is not part of the quantized path.
class Linear : public Module {
  public:
    Linear(size_t in_features, size_t out_features, bool bias)
        : in_(in_features), out_(out_features), use_bias_(bias) {
        weight_ = Tensor::from_data(std::vector<float>(in_ * out_, 0.0f), {in_, out_}).unwrap();
        if (bias) bias_ = Tensor::from_data(std::vector<float>(out_, 0.0f), {out_}).unwrap();
    }
    Result<Unit> set_weight(const Tensor &w) {
        if (w.shape().dims() != std::vector<size_t>{in_, out_})
            return TorshError::invalid_argument("Linear weight must have shape [in_features, out_features]");
        weight_ = w;
        return Unit{};
    }
    Result<Unit> set_bias(const Tensor &b) {
        if (!use_bias_ || b.shape().dims() != std::vector<size_t>{out_})
            return TorshError::invalid_argument("Linear bias must have shape [out_features]");
        bias_ = b;
        return Unit{};
    }
    Result<Tensor> forward(const Tensor &) const override {
        return TorshError::not_implemented("fp32 Linear::forward stays on the CPU implementation; convert with "
                                           "QuantizedLinear::from_linear");
    }
    std::map<std::string, Parameter> parameters() const override {
        std::map<std::string, Parameter> p{{"weight", weight_}};
        if (use_bias_) p["bias"] = bias_;
        return p;
    }
    size_t in_features() const { return in_; }
    size_t out_features() const { return out_; }
    bool has_bias() const { return use_bias_; }

  private:
    size_t in_, out_;
    bool use_bias_;
    Tensor weight_, bias_;
};

enum class ActivationQuant { PerTensor, PerToken };

class QuantizedLinear : public Module {
  public:
    // weight_nk: fp32 [out_features, in_features] (the layout of QATLinear,
    // crates/torsh-nn/src/quantization/qat.rs:266-343); quantized per output channel,
    // symmetric int8, division form, on the device.
    static Result<QuantizedLinear> from_weight_nk(const Tensor &weight_nk, const Tensor *bias,
                                                  ActivationQuant act = ActivationQuant::PerTensor) {
        const auto &d = weight_nk.shape().dims();
        if (d.size() != 2 || d[0] == 0 || d[1] == 0)
            return TorshError::invalid_argument("QuantizedLinear weight must be a non-empty 2D tensor");
        const size_t n = d[0], k = d[1];
        if (bias && bias->shape().dims() != std::vector<size_t>{n})
            return TorshError::invalid_argument("QuantizedLinear bias must have shape [out_features]");
        QuantizedLinear q;
        q.in_ = k;
        q.out_ = n;
        q.act_ = act;
        TORSH_TRY(ctx, hip::Runtime::ctx());
        q.ctx_ = ctx;
        TORSH_TRY(dwf, hip::DeviceBuffer::from_host(ctx, weight_nk.as_slice().data(), n * k));
        TORSH_TRY(dwq, hip::DeviceBuffer::alloc(ctx, n * k));
        TORSH_TRY(dsw, hip::DeviceBuffer::alloc(ctx, n * sizeof(float)));
        const int32_t zero = 0;
        TORSH_TRY(dst, hip::DeviceBuffer::from_host(ctx, &zero, 1));
        TORSH_CHECK(hip::check(hipq_quantize_per_row_f32_i8(ctx, dwf.as<float>(), n, k, HIPQ_PARAMS_SYMMETRIC,
                                                            HIPQ_ROUND_HALF_AWAY, dwq.as<int8_t>(), dsw.as<float>(),
                                                            nullptr, dst.as<int32_t>())));
        TORSH_TRY(st, dst.to_host<int32_t>(1));
        if (st[0] != HIPQ_SUCCESS) return TorshError::invalid_argument("Min and max values must be finite");
        q.w_ = std::move(dwq);
        q.sw_ = std::move(dsw);
        if (bias) {
            TORSH_TRY(db, hip::DeviceBuffer::from_host(ctx, bias->as_slice().data(), n));
            q.bias_ = std::move(db);
            q.has_bias_ = true;
        }
        TORSH_CHECK(q.pack());
        return std::move(q);
    }

    // From the reference's Linear: weight [in, out] is transposed once to [out, in].
    static Result<QuantizedLinear> from_linear(const Linear &lin, ActivationQuant act = ActivationQuant::PerTensor) {
        const auto params = lin.parameters();
        const std::vector<float> &w = params.at("weight").as_slice();
        const size_t k = lin.in_features(), n = lin.out_features();
        std::vector<float> wt(n * k);
        for (size_t i = 0; i < k; ++i)
            for (size_t j = 0; j < n; ++j) wt[j * k + i] = w[i * n + j];
        TORSH_TRY(wnk, Tensor::from_data(std::move(wt), {n, k}));
        if (lin.has_bias()) return from_weight_nk(wnk, &params.at("bias"), act);
        return from_weight_nk(wnk, nullptr, act);
    }

    // From prepared int8 weights (already quantized per output channel): one copy per section,
    // no arithmetic.  The counterpart of to_quantized_weights() / save().
    static Result<QuantizedLinear> from_quantized(const quantization::QuantizedWeights &w,
                                                  ActivationQuant act = ActivationQuant::PerTensor) {
        TORSH_CHECK(w.validate());
        if (w.kind != quantization::QuantizedWeights::Linear)
            return TorshError::invalid_argument("QuantizedLinear needs weights of kind Linear");
        QuantizedLinear q;
        q.out_ = w.dims[0];
        q.in_ = w.dims[1];
        q.act_ = act;
        if (q.in_ == 0 || q.out_ == 0)
            return TorshError::invalid_argument("QuantizedLinear weight must be a non-empty 2D tensor");
        TORSH_TRY(ctx, hip::Runtime::ctx());
        q.ctx_ = ctx;
        TORSH_TRY(dw, hip::DeviceBuffer::from_host(ctx, w.weight.data(), w.weight.size()));
        TORSH_TRY(ds, hip::DeviceBuffer::from_host(ctx, w.scales.data(), w.scales.size()));
        q.w_ = std::move(dw);
        q.sw_ = std::move(ds);
        if (!w.bias.empty()) {
            TORSH_TRY(db, hip::DeviceBuffer::from_host(ctx, w.bias.data(), w.bias.size()));
            q.bias_ = std::move(db);
            q.has_bias_ = true;
        }
        if (!w.packed.empty()) {
            // the file held the operand in tile order: it is what the forward reads, uploaded as it is
            TORSH_TRY(dp, hip::DeviceBuffer::from_host(ctx, w.packed.data(), w.packed.size()));
            q.wp_ = std::move(dp);
        } else {
            TORSH_CHECK(q.pack());
        }
        return std::move(q);
    }
    // prepared: also the rows in the operand order of the matrix cores, as the device holds them.
    Result<quantization::QuantizedWeights> to_quantized_weights(bool prepared = false) const {
        quantization::QuantizedWeights w;
        w.kind = quantization::QuantizedWeights::Linear;
        w.dims = {out_, in_};
        TORSH_TRY(wq, w_.to_host<int8_t>(out_ * in_));
        TORSH_TRY(sw, sw_.to_host<float>(out_));
        w.weight = std::move(wq);
        w.scales = std::move(sw);
        if (has_bias_) {
            TORSH_TRY(b, bias_.to_host<float>(out_));
            w.bias = std::move(b);
        }
        if (prepared) {
            TORSH_TRY(wp, wp_.to_host<int8_t>(wp_.bytes()));
            w.packed = std::move(wp);
        }
        return w;
    }
    Result<Unit> save(const std::string &path) const {
        TORSH_TRY(w, to_quantized_weights());
        return quantization::save_quantized_weights(w, path);
    }
    // The prepared-weight blob: int8 rows in tile order, scales, bias.  load() of it needs no packing pass.
    Result<Unit> save_prepared(const std::string &path) const {
        TORSH_TRY(w, to_quantized_weights(/*prepared=*/true));
        return quantization::save_quantized_weights(w, path);
    }
    static Result<QuantizedLinear> load(const std::string &path, ActivationQuant act = ActivationQuant::PerTensor) {
        TORSH_TRY(w, quantization::load_quantized_weights(path));
        return from_quantized(w, act);
    }

    // input [..., in_features] -> [..., out_features]
    Result<Tensor> forward(const Tensor &input) const override {
        const auto &d = input.shape().dims();
        if (d.empty() || d.back() != in_)
            return TorshError::invalid_argument("QuantizedLinear expects input [..., " + std::to_string(in_) + "]");
        const size_t m = input.numel() / in_;
        std::vector<size_t> out_dims = d;
        out_dims.back() = out_;
        if (m == 0) return TorshError::invalid_argument("Cannot quantize empty tensor");
        // The reference refuses a range that is not finite before it quantizes (algorithms.rs:403-407);
        // min / max skip a NaN (simd_ops.rs:95-108), so only an infinity makes the range non-finite.  The
        // device call is asynchronous and could only answer with NaN outputs, so the check is made here.
        for (float v : input.as_slice())
            if (std::isinf(v)) return TorshError::invalid_argument("Min and max values must be finite");
        TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx_, input.as_slice().data(), input.numel()));
        TORSH_TRY(dy, hip::DeviceBuffer::alloc(ctx_, m * out_ * sizeof(float)));
        // Activations follow the reference's branch for their size: x*(1/scale) above 64 elements
        // (algorithms.rs:292), x/scale otherwise; per-token always divides (algorithms.rs:230).
        const int32_t mode = (act_ == ActivationQuant::PerTensor && m * in_ > 64) ? HIPQ_FORM_MUL_INV : HIPQ_FORM_DIV;
        if (static_scale_ > 0.0f) {
            TORSH_CHECK(hip::check(hipq_linear_static_packed_f32(ctx_, dx.as<float>(), static_scale_,
                                                                 wp_.as<int8_t>(), sw_.as<float>(),
                                                                 has_bias_ ? bias_.as<float>() : nullptr, m, out_, in_,
                                                                 mode, dy.as<float>())));
            TORSH_TRY(ys, dy.to_host<float>(m * out_));
            return Tensor::from_data(std::move(ys), std::move(out_dims));
        }
        TORSH_CHECK(hip::check(hipq_linear_dynamic_packed_f32(ctx_, dx.as<float>(),
                                                              act_ == ActivationQuant::PerToken ? 1 : 0,
                                                              wp_.as<int8_t>(), sw_.as<float>(),
                                                              has_bias_ ? bias_.as<float>() : nullptr, m, out_, in_,
                                                              mode, dy.as<float>())));
        TORSH_TRY(y, dy.to_host<float>(m * out_));
        return Tensor::from_data(std::move(y), std::move(out_dims));
    }

    // "weight": int8 values in the f32 carrier, [out, in]; "weight_scale": [out]; "bias": [out].
    std::map<std::string, Parameter> parameters() const override {
        std::map<std::string, Parameter> p;
        auto wq = w_.to_host<int8_t>(out_ * in_);
        auto sw = sw_.to_host<float>(out_);
        if (wq.is_err() || sw.is_err()) return p;
        std::vector<float> carrier(wq.unwrap().begin(), wq.unwrap().end());
        p["weight"] = Tensor::from_data(std::move(carrier), {out_, in_}).unwrap();
        p["weight_scale"] = Tensor::from_data(sw.unwrap(), {out_}).unwrap();
        if (has_bias_) {
            auto b = bias_.to_host<float>(out_);
            if (b.is_ok()) p["bias"] = Tensor::from_data(b.unwrap(), {out_}).unwrap();
        }
        return p;
    }
    bool training() const override { return false; }
    size_t in_features() const { return in_; }
    size_t out_features() const { return out_; }

    // Static quantization: use a calibrated per-tensor activation scale (what
    // Observer::calculate_qparams returned for a symmetric int8 scheme, zero point 0) instead of
    // taking the range of every input.  A scale <= 0 switches back to dynamic quantization.
    Result<bool> set_static_activation_scale(float scale, int32_t zero_point = 0) {
        if (zero_point != 0)
            return TorshError::invalid_argument("QuantizedLinear: a static activation scale needs a symmetric scheme (zero point 0)");
        if (scale > 0.0f && act_ != ActivationQuant::PerTensor)
            return TorshError::invalid_argument("QuantizedLinear: a static activation scale is per tensor");
        static_scale_ = scale > 0.0f ? scale : 0.0f;
        return true;
    }
    float static_activation_scale() const { return static_scale_; }

  private:
    QuantizedLinear() = default;
    // Weight preparation, once per layer: the int8 rows in the operand order of the matrix cores, which is
    // what the forward reads; the row-major copy stays for parameters() and save().
    Result<Unit> pack() {
        size_t bytes = 0;
        TORSH_CHECK(hip::check(hipq_packed_size(out_, in_, &bytes)));
        TORSH_TRY(dp, hip::DeviceBuffer::alloc(ctx_, bytes));
        TORSH_CHECK(hip::check(hipq_pack_rows_i8(ctx_, w_.as<int8_t>(), out_, in_, dp.as<int8_t>())));
        wp_ = std::move(dp);
        return Unit{};
    }
    hipq_ctx *ctx_ = nullptr;
    size_t in_ = 0, out_ = 0;
    ActivationQuant act_ = ActivationQuant::PerTensor;
    hip::DeviceBuffer w_, wp_, sw_, bias_;
    bool has_bias_ = false;
    float static_scale_ = 0.0f;  // > 0: calibrated activation scale
};

class QuantizedConv2d : public Module {
  public:
    // weight fp32 [oc, ic, kh, kw] (groups = 1, dilation 1), quantized per output channel on the
    // device; out_scale / out_zero_point are the calibrated int8 output parameters.
    static Result<QuantizedConv2d> from_weight(const Tensor &weight, const Tensor *bias,
                                               std::pair<size_t, size_t> stride, std::pair<size_t, size_t> padding,
                                               float out_scale, int32_t out_zero_point) {
        const auto &d = weight.shape().dims();
        if (d.size() != 4 || weight.numel() == 0)
            return TorshError::invalid_argument("QuantizedConv2d weight must be [C_out, C_in, kH, kW]");
        if (bias && bias->shape().dims() != std::vector<size_t>{d[0]})
            return TorshError::invalid_argument("QuantizedConv2d bias must have shape [C_out]");
        if (!(out_scale > 0.0f)) return TorshError::invalid_argument("Scale must be positive");
        if (out_zero_point < -128 || out_zero_point > 127)
            return TorshError::invalid_argument("Zero point is outside valid range [-128, 127]");
        if (stride.first == 0 || stride.second == 0) return TorshError::invalid_argument("stride must be positive");
        QuantizedConv2d q;
        q.oc_ = d[0], q.ic_ = d[1], q.kh_ = d[2], q.kw_ = d[3];
        q.stride_ = stride, q.padding_ = padding;
        q.s_out_ = out_scale, q.zp_out_ = out_zero_point;
        TORSH_TRY(ctx, hip::Runtime::ctx());
        q.ctx_ = ctx;
        const size_t per = q.ic_ * q.kh_ * q.kw_;
        TORSH_TRY(dwf, hip::DeviceBuffer::from_host(ctx, weight.as_slice().data(), q.oc_ * per));
        TORSH_TRY(dwq, hip::DeviceBuffer::alloc(ctx, q.oc_ * per));
        TORSH_TRY(dsw, hip::DeviceBuffer::alloc(ctx, q.oc_ * sizeof(float)));
        const int32_t zero = 0;
        TORSH_TRY(dst, hip::DeviceBuffer::from_host(ctx, &zero, 1));
        TORSH_CHECK(hip::check(hipq_quantize_per_row_f32_i8(ctx, dwf.as<float>(), q.oc_, per, HIPQ_PARAMS_SYMMETRIC,
                                                            HIPQ_ROUND_HALF_AWAY, dwq.as<int8_t>(), dsw.as<float>(),
                                                            nullptr, dst.as<int32_t>())));
        TORSH_TRY(st, dst.to_host<int32_t>(1));
        if (st[0] != HIPQ_SUCCESS) return TorshError::invalid_argument("Min and max values must be finite");
        q.w_ = std::move(dwq);
        q.sw_ = std::move(dsw);
        if (bias) {
            TORSH_TRY(db, hip::DeviceBuffer::from_host(ctx, bias->as_slice().data(), q.oc_));
            q.bias_ = std::move(db);
            q.has_bias_ = true;
        }
        return std::move(q);
    }

    // From prepared int8 weights; stride, padding and the output parameters are not part of the
    // weight file (they belong to the layer's configuration).
    static Result<QuantizedConv2d> from_quantized(const quantization::QuantizedWeights &w,
                                                  std::pair<size_t, size_t> stride, std::pair<size_t, size_t> padding,
                                                  float out_scale, int32_t out_zero_point) {
        TORSH_CHECK(w.validate());
        if (w.kind != quantization::QuantizedWeights::Conv2d)
            return TorshError::invalid_argument("QuantizedConv2d needs weights of kind Conv2d");
        if (!(out_scale > 0.0f)) return TorshError::invalid_argument("Scale must be positive");
        if (out_zero_point < -128 || out_zero_point > 127)
            return TorshError::invalid_argument("Zero point is outside valid range [-128, 127]");
        if (stride.first == 0 || stride.second == 0) return TorshError::invalid_argument("stride must be positive");
        QuantizedConv2d q;
        q.oc_ = w.dims[0], q.ic_ = w.dims[1], q.kh_ = w.dims[2], q.kw_ = w.dims[3];
        q.stride_ = stride, q.padding_ = padding;
        q.s_out_ = out_scale, q.zp_out_ = out_zero_point;
        TORSH_TRY(ctx, hip::Runtime::ctx());
        q.ctx_ = ctx;
        TORSH_TRY(dw, hip::DeviceBuffer::from_host(ctx, w.weight.data(), w.weight.size()));
        TORSH_TRY(ds, hip::DeviceBuffer::from_host(ctx, w.scales.data(), w.scales.size()));
        q.w_ = std::move(dw);
        q.sw_ = std::move(ds);
        if (!w.bias.empty()) {
            TORSH_TRY(db, hip::DeviceBuffer::from_host(ctx, w.bias.data(), w.bias.size()));
            q.bias_ = std::move(db);
            q.has_bias_ = true;
        }
        return std::move(q);
    }
    Result<quantization::QuantizedWeights> to_quantized_weights() const {
        quantization::QuantizedWeights w;
        w.kind = quantization::QuantizedWeights::Conv2d;
        w.dims = {oc_, ic_, kh_, kw_};
        TORSH_TRY(wq, w_.to_host<int8_t>(oc_ * ic_ * kh_ * kw_));
        TORSH_TRY(sw, sw_.to_host<float>(oc_));
        w.weight = std::move(wq);
        w.scales = std::move(sw);
        if (has_bias_) {
            TORSH_TRY(b, bias_.to_host<float>(oc_));
            w.bias = std::move(b);
        }
        return w;
    }
    Result<Unit> save(const std::string &path) const {
        TORSH_TRY(w, to_quantized_weights());
        return quantization::save_quantized_weights(w, path);
    }

    // int8 NCHW output and the input parameters the activations were quantized with.
    Result<TensorI8> forward_quantized(const Tensor &input) const {
        const auto &d = input.shape().dims();
        if (d.size() < 4)
            return TorshError::invalid_argument("Conv2d expects 4D input (batch_size, channels, height, width), got " +
                                                std::to_string(d.size()) + "D");
        if (d[1] != ic_)
            return TorshError::invalid_argument("qconv2d channel mismatch: input C_in=" + std::to_string(d[1]) +
                                                " but weight C_in=" + std::to_string(ic_));
        if (input.numel() == 0) return TorshError::invalid_argument("Cannot quantize empty tensor");
        const size_t nb = d[0], h = d[2], w = d[3];
        if (h + 2 * padding_.first < kh_ || w + 2 * padding_.second < kw_)
            return TorshError::invalid_argument("kernel larger than the padded input");
        const size_t ho = (h + 2 * padding_.first - kh_) / stride_.first + 1;
        const size_t wo = (w + 2 * padding_.second - kw_) / stride_.second + 1;
        TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx_, input.as_slice().data(), input.numel()));
        TORSH_TRY(dxq, hip::DeviceBuffer::alloc(ctx_, input.numel()));
        TORSH_TRY(dp, hip::DeviceBuffer::alloc(ctx_, sizeof(hipq_qparams)));
        TORSH_CHECK(hip::check(hipq_quantize_dynamic_per_tensor_f32(ctx_, dx.as<float>(), input.numel(),
                                                                    HIPQ_PARAMS_BACKEND_ASYMMETRIC, HIPQ_DTYPE_U8,
                                                                    HIPQ_FORM_DIV, dxq.as<void>(),
                                                                    dp.as<hipq_qparams>())));
        TORSH_TRY(p, dp.to_host<hipq_qparams>(1));
        if (p[0].status != HIPQ_SUCCESS) return TorshError::invalid_argument("min_val and max_val must be finite");
        TORSH_TRY(dout, hip::DeviceBuffer::alloc(ctx_, nb * oc_ * ho * wo));
        TORSH_CHECK(hip::check(hipq_conv2d_u8i8_i8(ctx_, dxq.as<uint8_t>(), p[0].zero_point, p[0].scale,
                                                   w_.as<int8_t>(), sw_.as<float>(),
                                                   has_bias_ ? bias_.as<float>() : nullptr, nb, ic_, h, w, oc_, kh_,
                                                   kw_, stride_.first, stride_.second, padding_.first,
                                                   padding_.second, s_out_, zp_out_, HIPQ_ROUND_HALF_AWAY,
                                                   dout.as<int8_t>())));
        TORSH_TRY(q, dout.to_host<int8_t>(nb * oc_ * ho * wo));
        return TensorI8::from_data(std::move(q), {nb, oc_, ho, wo});
    }

    // Module::forward: the int8 result dequantized with the output parameters, (q - zp) * scale.
    Result<Tensor> forward(const Tensor &input) const override {
        TORSH_TRY(q, forward_quantized(input));
        const size_t n = q.numel();
        TORSH_TRY(dq, hip::DeviceBuffer::from_host(ctx_, q.as_slice().data(), n));
        TORSH_TRY(dy, hip::DeviceBuffer::alloc(ctx_, n * sizeof(float)));
        TORSH_CHECK(hip::check(hipq_dequantize_i8_f32(ctx_, dq.as<int8_t>(), n, s_out_, zp_out_, dy.as<float>())));
        TORSH_TRY(y, dy.to_host<float>(n));
        return Tensor::from_data(std::move(y), q.shape().dims());
    }

    std::map<std::string, Parameter> parameters() const override {
        std::map<std::string, Parameter> p;
        const size_t per = ic_ * kh_ * kw_;
        auto wq = w_.to_host<int8_t>(oc_ * per);
        auto sw = sw_.to_host<float>(oc_);
        if (wq.is_err() || sw.is_err()) return p;
        std::vector<float> carrier(wq.unwrap().begin(), wq.unwrap().end());
        p["weight"] = Tensor::from_data(std::move(carrier), {oc_, ic_, kh_, kw_}).unwrap();
        p["weight_scale"] = Tensor::from_data(sw.unwrap(), {oc_}).unwrap();
        if (has_bias_) {
            auto b = bias_.to_host<float>(oc_);
            if (b.is_ok()) p["bias"] = Tensor::from_data(b.unwrap(), {oc_}).unwrap();
        }
        return p;
    }
    bool training() const override { return false; }
    float out_scale() const { return s_out_; }
    int32_t out_zero_point() const { return zp_out_; }

  private:
    QuantizedConv2d() = default;
    hipq_ctx *ctx_ = nullptr;
    size_t oc_ = 0, ic_ = 0, kh_ = 0, kw_ = 0;
    std::pair<size_t, size_t> stride_{1, 1}, padding_{0, 0};
    float s_out_ = 1.0f;
    int32_t zp_out_ = 0;
    hip::DeviceBuffer w_, sw_, bias_;
    bool has_bias_ = false;
};

}  // namespace nn
}  // namespace torsh
