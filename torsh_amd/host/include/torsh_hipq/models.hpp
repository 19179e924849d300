// torsh::models::quantization — the model-level quantizer of crates/torsh-models, with the
// reference's names and formulas.  Per parameter it needs a range, a fake-quantized image and the
// error between the two: the range is one device pass, image and error are one fused device pass
// (the image is never written unless quantize_tensor asks for it).
//
//   QuantizationDType, QuantizationParams, QuantizationStats, LayerQuantizationStats
//                                            crates/torsh-models/src/quantization.rs:17-31, 183-224
//   QuantizationConfig, QuantizationStrategy, LayerQuantizationFilter, QuantizableLayerType
//                                            quantization.rs:33-131
//   ModelQuantizer                           quantization.rs:226-611
//   MinMaxObserver                           quantization.rs:614-652
//   quantization_utils                       quantization.rs:654-720
#pragma once

#include <map>

#include "calibration.hpp"
#include "nn.hpp"
#include "serialize.hpp"

namespace torsh {
namespace models {
namespace quantization {

enum class QuantizationDType { Int8, Uint8, Int16, Float16, BFloat16 };

enum class QuantizationStrategyKind { PostTraining, QuantizationAware, Dynamic };
struct QuantizationStrategy {
    QuantizationStrategyKind kind = QuantizationStrategyKind::PostTraining;
    size_t calibration_samples = 1000;    // PostTraining
    bool percentile_calibration = false;  // PostTraining
    bool fake_quantize = true;            // QuantizationAware
};

enum class QuantizableLayerType { Linear, Convolution, Embedding, Attention };

struct LayerQuantizationFilter {
    enum Kind { All, Include, Exclude, LayerTypes } kind = All;
    std::vector<std::string> names;
    std::vector<QuantizableLayerType> types;
};

struct QuantizationConfig {  // Default: quantization.rs:94-110
    QuantizationDType dtype = QuantizationDType::Int8;
    QuantizationStrategy strategy;
    LayerQuantizationFilter layer_filter;
    bool quantize_weights = true;
    bool quantize_activations = true;
};

struct QuantizationParams {
    float scale = 1.0f;
    int32_t zero_point = 0;
    float min_val = 0.0f;
    float max_val = 0.0f;
    QuantizationDType dtype = QuantizationDType::Int8;
};

struct LayerQuantizationStats {
    size_t original_params = 0;
    size_t quantized_params = 0;
    uint8_t bits_per_param = 8;
    double quantization_error = 0.0;
};

struct QuantizationStats {
    size_t original_size = 0;
    size_t quantized_size = 0;
    double compression_ratio = 0.0;
    std::map<std::string, LayerQuantizationStats> layer_stats;
    double theoretical_speedup = 1.0;
};

namespace detail {
inline const char *name_of(QuantizationDType d) {
    static const char *n[] = {"Int8", "Uint8", "Int16", "Float16", "BFloat16"};
    return n[static_cast<int>(d)];
}
}  // namespace detail

class ModelQuantizer {
  public:
    explicit ModelQuantizer(QuantizationConfig config) : config_(std::move(config)) {}

    // quantization.rs:351-363
    std::pair<int32_t, int32_t> get_quantization_range(QuantizationDType dtype) const {
        switch (dtype) {
        case QuantizationDType::Int8: return {-128, 127};
        case QuantizationDType::Uint8: return {0, 255};
        default: return {-32768, 32767};
        }
    }

    // quantization.rs:365-392
    QuantizationParams calculate_quantization_params(float min_val, float max_val, QuantizationDType dtype) const {
        const auto [qmin, qmax] = get_quantization_range(dtype);
        float amin = min_val, amax = max_val;
        if (std::fabs(max_val - min_val) < 1e-8f) {
            amin = min_val - 1e-4f;
            amax = max_val + 1e-4f;
        }
        const float scale = (amax - amin) / static_cast<float>(qmax - qmin);
        const float zf = static_cast<float>(qmin) - amin / scale;
        const int32_t zp = torsh::quantization::detail::f32_as_i32(torsh::quantization::detail::clamp_keep_nan(
            std::round(zf), static_cast<float>(qmin), static_cast<float>(qmax)));
        return {scale, zp, amin, amax, dtype};
    }

    // quantization.rs:395-408: an empty tensor has range (0, 0).
    Result<std::pair<float, float>> calculate_tensor_stats(const Tensor &tensor) const {
        const std::vector<float> &data = tensor.as_slice();
        if (data.empty()) return std::make_pair(0.0f, 0.0f);
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
        TORSH_TRY(dmm, hip::DeviceBuffer::alloc(ctx, 2 * sizeof(float)));
        TORSH_CHECK(hip::check(hipq_minmax_f32(ctx, dx.as<float>(), data.size(), dmm.as<float>())));
        TORSH_TRY(mm, dmm.to_host<float>(2));
        return std::make_pair(mm[0], mm[1]);
    }

    // quantization.rs:309-332: the fake-quantized image (quantize_value then dequantize_value).
    Result<Tensor> quantize_tensor(const Tensor &tensor, const QuantizationParams &params) const {
        const std::vector<float> &data = tensor.as_slice();
        std::vector<float> out(data.size());
        if (!data.empty()) {
            if (!(params.scale > 0.0f)) return TorshError::invalid_argument("Scale must be positive");
            const auto [qmin, qmax] = get_quantization_range(params.dtype);
            TORSH_TRY(ctx, hip::Runtime::ctx());
            TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
            TORSH_TRY(dy, hip::DeviceBuffer::alloc(ctx, data.size() * sizeof(float)));
            TORSH_CHECK(hip::check(hipq_fake_quantize_f32(ctx, dx.as<float>(), data.size(), params.scale,
                                                          params.zero_point, nullptr, qmin, qmax,
                                                          HIPQ_FORM_DIV | HIPQ_FAKE_INT_CAST, dy.as<float>())));
            TORSH_TRY(y, dy.to_host<float>(data.size()));
            out = std::move(y);
        }
        return Tensor::from_data(std::move(out), tensor.shape().dims());
    }

    // quantization.rs:248-257, 260-307: every strategy calibrates the filtered parameters, runs the
    // weight pass where it is enabled and then collects the statistics over all parameters.
    Result<QuantizationStats> quantize_model(const nn::Module &model) {
        return quantize_parameters(model.named_parameters());
    }
    Result<QuantizationStats> quantize_parameters(const std::map<std::string, Tensor> &parameters) {
        const auto filtered = filter_parameters(parameters);
        if (config_.strategy.kind != QuantizationStrategyKind::QuantizationAware) {
            for (const auto &[name, tensor] : filtered) {
                TORSH_TRY(mm, calculate_tensor_stats(tensor));
                quantization_params_[name] = calculate_quantization_params(mm.first, mm.second, config_.dtype);
            }
        }
        TORSH_TRY(stats, calculate_quantization_stats(parameters));
        stats_ = stats;
        has_stats_ = true;
        return stats;
    }

    const QuantizationStats *get_stats() const { return has_stats_ ? &stats_ : nullptr; }
    const std::map<std::string, QuantizationParams> &quantization_params() const { return quantization_params_; }

    // quantization.rs:586-611: serde_json of HashMap<String, QuantizationParams>, pretty printed.
    Result<Unit> save_quantization_params(const std::string &path) const {
        std::ostringstream o;
        o << "{";
        bool first = true;
        for (const auto &[name, p] : quantization_params_) {
            o << (first ? "\n" : ",\n") << "  \"" << name << "\": {\n"
              << "    \"scale\": " << torsh::quantization::detail::json_number(p.scale) << ",\n"
              << "    \"zero_point\": " << p.zero_point << ",\n"
              << "    \"min_val\": " << torsh::quantization::detail::json_number(p.min_val) << ",\n"
              << "    \"max_val\": " << torsh::quantization::detail::json_number(p.max_val) << ",\n"
              << "    \"dtype\": \"" << detail::name_of(p.dtype) << "\"\n  }";
            first = false;
        }
        o << (first ? "}" : "\n}");
        std::ofstream f(path, std::ios::trunc);
        if (!f) return TorshError::invalid_argument("Failed to write quantization params: cannot open " + path);
        f << o.str();
        return Unit{};
    }
    Result<Unit> load_quantization_params(const std::string &path) {
        std::ifstream f(path);
        if (!f) return TorshError::invalid_argument("Failed to read quantization params: cannot open " + path);
        std::stringstream ss;
        ss << f.rdbuf();
        auto outer = torsh::quantization::detail::FlatJson::parse_object(ss.str());
        if (outer.is_err())
            return TorshError::invalid_argument("Failed to deserialize quantization params: " +
                                                outer.unwrap_err().message);
        std::map<std::string, QuantizationParams> loaded;
        for (const auto &[name, text] : outer.unwrap()) {
            auto inner = torsh::quantization::detail::FlatJson::parse_object(text);
            if (inner.is_err())
                return TorshError::invalid_argument("Failed to deserialize quantization params: " +
                                                    inner.unwrap_err().message);
            const auto &m = inner.unwrap();
            for (const char *k : {"scale", "zero_point", "min_val", "max_val", "dtype"})
                if (!m.count(k))
                    return TorshError::invalid_argument(std::string("Failed to deserialize quantization params: "
                                                                    "missing field `") + k + "`");
            QuantizationParams p;
            p.scale = std::strtof(m.at("scale").c_str(), nullptr);
            p.zero_point = static_cast<int32_t>(std::strtol(m.at("zero_point").c_str(), nullptr, 10));
            p.min_val = std::strtof(m.at("min_val").c_str(), nullptr);
            p.max_val = std::strtof(m.at("max_val").c_str(), nullptr);
            const std::string dt = torsh::quantization::detail::FlatJson::unquote(m.at("dtype"));
            bool known = false;
            for (int i = 0; i < 5; ++i)
                if (dt == detail::name_of(static_cast<QuantizationDType>(i))) {
                    p.dtype = static_cast<QuantizationDType>(i);
                    known = true;
                }
            if (!known)
                return TorshError::invalid_argument("Failed to deserialize quantization params: unknown dtype " + dt);
            loaded[name] = p;
        }
        quantization_params_ = std::move(loaded);
        return Unit{};
    }

    // quantization.rs:411-457
    std::map<std::string, Tensor> filter_parameters(const std::map<std::string, Tensor> &parameters) const {
        const LayerQuantizationFilter &f = config_.layer_filter;
        if (f.kind == LayerQuantizationFilter::All) return parameters;
        auto contains_any = [&](const std::string &name) {
            for (const auto &n : f.names)
                if (name.find(n) != std::string::npos) return true;
            return false;
        };
        auto has = [](const std::string &s, const char *sub) { return s.find(sub) != std::string::npos; };
        auto matches_type = [&](const std::string &name) {
            for (QuantizableLayerType t : f.types) {
                switch (t) {
                case QuantizableLayerType::Linear:
                    if (has(name, "linear") || has(name, "fc")) return true;
                    break;
                case QuantizableLayerType::Convolution:
                    if (has(name, "conv")) return true;
                    break;
                case QuantizableLayerType::Embedding:
                    if (has(name, "embed")) return true;
                    break;
                case QuantizableLayerType::Attention:
                    if (has(name, "attn") || has(name, "attention")) return true;
                    break;
                }
            }
            return false;
        };
        std::map<std::string, Tensor> out;
        for (const auto &[name, t] : parameters) {
            const bool keep = f.kind == LayerQuantizationFilter::Include   ? contains_any(name)
                              : f.kind == LayerQuantizationFilter::Exclude ? !contains_any(name)
                                                                           : matches_type(name);
            if (keep) out.emplace(name, t);
        }
        return out;
    }

  private:
    // quantization.rs:491-546.  The per-layer error is quantize_tensor + calculate_mse_error
    // (:548-566) in one pass over the parameter.
    Result<QuantizationStats> calculate_quantization_stats(const std::map<std::string, Tensor> &parameters) const {
        QuantizationStats stats;
        const uint8_t bits = (config_.dtype == QuantizationDType::Int8 || config_.dtype == QuantizationDType::Uint8) ? 8 : 16;
        for (const auto &[name, tensor] : parameters) {
            const size_t count = tensor.numel();
            stats.original_size += count * 4;
            stats.quantized_size += count * (bits / 8);
            double error = 0.0;
            auto it = quantization_params_.find(name);
            if (it != quantization_params_.end()) {
                const QuantizationParams &p = it->second;
                const std::vector<float> &data = tensor.as_slice();
                if (data.empty()) {
                    error = std::numeric_limits<double>::quiet_NaN();  // 0.0 / 0.0 in the reference
                } else {
                    const auto [qmin, qmax] = get_quantization_range(p.dtype);
                    TORSH_TRY(ctx, hip::Runtime::ctx());
                    TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
                    TORSH_TRY(dm, hip::DeviceBuffer::alloc(ctx, sizeof(hipq_quant_metrics)));
                    TORSH_CHECK(hip::check(hipq_fake_quantize_metrics_f32(
                        ctx, dx.as<float>(), data.size(), p.scale, p.zero_point, nullptr, qmin, qmax,
                        HIPQ_FORM_DIV | HIPQ_FAKE_INT_CAST, 32, bits, dm.as<hipq_quant_metrics>())));
                    TORSH_TRY(m, dm.to_host<hipq_quant_metrics>(1));
                    error = static_cast<double>(m[0].mse);
                }
            }
            stats.layer_stats[name] = {count, count, bits, error};
        }
        stats.compression_ratio = static_cast<double>(stats.original_size) / static_cast<double>(stats.quantized_size);
        stats.theoretical_speedup = bits == 8 ? 2.0 : (config_.dtype == QuantizationDType::Int16 ? 1.5 : 1.3);  // :568-575
        return stats;
    }

    QuantizationConfig config_;
    std::map<std::string, QuantizationParams> quantization_params_;
    QuantizationStats stats_;
    bool has_stats_ = false;
};

// quantization.rs:614-652
class MinMaxObserver {
  public:
    Result<Unit> observe(const Tensor &tensor) {
        const std::vector<float> &data = tensor.as_slice();
        if (data.empty()) return Unit{};
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
        TORSH_TRY(dmm, hip::DeviceBuffer::alloc(ctx, 2 * sizeof(float)));
        TORSH_CHECK(hip::check(hipq_minmax_f32(ctx, dx.as<float>(), data.size(), dmm.as<float>())));
        TORSH_TRY(mm, dmm.to_host<float>(2));
        min_val_ = std::fmin(min_val_, mm[0]);
        max_val_ = std::fmax(max_val_, mm[1]);
        return Unit{};
    }
    std::pair<float, float> get_min_max() const { return {min_val_, max_val_}; }
    void reset() {
        min_val_ = std::numeric_limits<float>::infinity();
        max_val_ = -std::numeric_limits<float>::infinity();
    }

  private:
    float min_val_ = std::numeric_limits<float>::infinity();
    float max_val_ = -std::numeric_limits<float>::infinity();
};

namespace quantization_utils {  // quantization.rs:654-720
inline QuantizationConfig post_training_quantization_config(QuantizationDType dtype) {
    QuantizationConfig c;
    c.dtype = dtype;
    return c;
}
inline QuantizationConfig dynamic_quantization_config(QuantizationDType dtype) {
    QuantizationConfig c;
    c.dtype = dtype;
    c.strategy.kind = QuantizationStrategyKind::Dynamic;
    c.quantize_activations = false;
    return c;
}
inline QuantizationConfig quantization_aware_training_config(QuantizationDType dtype) {
    QuantizationConfig c;
    c.dtype = dtype;
    c.strategy.kind = QuantizationStrategyKind::QuantizationAware;
    c.strategy.fake_quantize = true;
    return c;
}
inline std::pair<double, double> calculate_memory_savings(size_t original_size, size_t quantized_size) {
    const double ratio = static_cast<double>(original_size) / static_cast<double>(quantized_size);
    const double savings = (1.0 - static_cast<double>(quantized_size) / static_cast<double>(original_size)) * 100.0;
    return {ratio, savings};
}
inline double estimate_inference_speedup(QuantizationDType dtype, const std::string &hardware_type) {
    const bool cpu = hardware_type == "cpu", gpu = hardware_type == "gpu";
    switch (dtype) {
    case QuantizationDType::Int8: return cpu ? 2.5 : gpu ? 1.8 : 1.0;
    case QuantizationDType::Uint8: return cpu ? 2.3 : gpu ? 1.7 : 1.0;
    case QuantizationDType::Int16: return cpu ? 1.6 : gpu ? 1.4 : 1.0;
    case QuantizationDType::Float16: return gpu ? 1.8 : 1.0;
    case QuantizationDType::BFloat16: return gpu ? 1.7 : 1.0;
    }
    return 1.0;
}
}  // namespace quantization_utils

}  // namespace quantization
}  // namespace models
}  // namespace torsh
