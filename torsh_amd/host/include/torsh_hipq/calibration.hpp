// torsh::quantization — calibration observers, quality metrics and batch utilities of
// crates/torsh-quantization, with the reference's names and error behaviour.  The passes over
// tensor data (range + non-finite check, histogram binning, metric sums, fake quantization) run
// on the GPU through the torsh_hipq C-ABI; the scalar bookkeeping around them (moving averages,
// outlier trimming of a 256-entry histogram, sorting at most ~10^5 retained samples) stays on the
// host, as it is not data-parallel work.
//
//   QuantizationMetrics, calculate_quantization_metrics   crates/torsh-quantization/src/metrics.rs:30-175
//   compare_quantization_configs                          metrics.rs:178-260
//   auto_calibrate_quantization                           metrics.rs:252-338
//   Observer                                              crates/torsh-quantization/src/observers.rs:36-556
//   quantize_batch_consistent                             crates/torsh-quantization/src/utils.rs:153-180
#pragma once

#include <algorithm>
#include <chrono>
#include <cmath>
#include <limits>
#include <map>
#include <string>

#include "quantization.hpp"

namespace torsh {
namespace quantization {

// metrics.rs:30-63
struct QuantizationMetrics {
    float mse = 0.0f;
    float psnr = 0.0f;
    float snr = 0.0f;
    float mae = 0.0f;
    float max_error = 0.0f;
    float zero_error_percentage = 100.0f;
    float cosine_similarity = 1.0f;
    float compression_ratio = 1.0f;
};

namespace detail {
inline QuantizationMetrics from_record(const hipq_quant_metrics &m) {
    QuantizationMetrics q;
    q.mse = m.mse, q.psnr = m.psnr, q.snr = m.snr, q.mae = m.mae, q.max_error = m.max_error;
    q.zero_error_percentage = m.zero_error_percentage, q.cosine_similarity = m.cosine_similarity;
    q.compression_ratio = m.compression_ratio;
    return q;
}
inline size_t f32_as_usize(float v) {  // Rust `as usize`: saturating, NaN and negatives -> 0
    if (!(v == v) || v <= 0.0f) return 0;
    if (v >= 18446744073709551616.0f) return std::numeric_limits<size_t>::max();
    return static_cast<size_t>(v);
}
inline uint32_t dtype_bits(DType d) {  // metrics.rs:203-216
    switch (d) {
    case DType::F32:
    case DType::I32: return 32;
    case DType::F16:
    case DType::I16: return 16;
    default: return 8;
    }
}
}  // namespace detail

// metrics.rs:67-175: one pass over both tensors on the device.
inline Result<QuantizationMetrics> calculate_quantization_metrics(const Tensor &original, const Tensor &quantized,
                                                                  uint32_t original_bits, uint32_t quantized_bits) {
    if (original.shape().dims() != quantized.shape().dims())
        return TorshError::invalid_argument("Shape mismatch between original and quantized tensors");
    const std::vector<float> &a = original.as_slice(), &b = quantized.as_slice();
    if (a.size() != b.size()) return TorshError::invalid_argument("Data length mismatch between tensors");
    if (a.empty()) return QuantizationMetrics{};
    TORSH_TRY(ctx, hip::Runtime::ctx());
    TORSH_TRY(da, hip::DeviceBuffer::from_host(ctx, a.data(), a.size()));
    TORSH_TRY(db, hip::DeviceBuffer::from_host(ctx, b.data(), b.size()));
    TORSH_TRY(dm, hip::DeviceBuffer::alloc(ctx, sizeof(hipq_quant_metrics)));
    TORSH_CHECK(hip::check(hipq_quantization_metrics_f32(ctx, da.as<float>(), db.as<float>(), a.size(), original_bits,
                                                         quantized_bits, dm.as<hipq_quant_metrics>())));
    TORSH_TRY(m, dm.to_host<hipq_quant_metrics>(1));
    return detail::from_record(m[0]);
}

struct ConfigComparison {
    QuantConfig config;
    QuantizationMetrics metrics;
    double seconds;
};

// metrics.rs:178-260: quantize with each configuration, dequantize, measure, rank by PSNR.  For
// the per-tensor schemes the three steps collapse into the range pass plus one fused pass that
// forms the dequantized image in registers; other schemes go through quantize_with_config and
// dequantize as the reference does.  A configuration that fails gets the worst-case record.
inline Result<std::vector<ConfigComparison>> compare_quantization_configs(const Tensor &tensor,
                                                                          const std::vector<QuantConfig> &configs) {
    std::vector<ConfigComparison> results;
    const std::vector<float> &data = tensor.as_slice();
    const float inf = std::numeric_limits<float>::infinity();
    const QuantizationMetrics worst{inf, -inf, -inf, inf, inf, 0.0f, 0.0f, 1.0f};
    for (const QuantConfig &config : configs) {
        const uint32_t qbits = detail::dtype_bits(config.dtype);
        auto one = [&]() -> Result<QuantizationMetrics> {
            const bool per_tensor =
                config.scheme == QScheme::PerTensorAffine || config.scheme == QScheme::PerTensorSymmetric;
            if (!per_tensor) {
                TORSH_TRY(q, quantize_with_config(tensor, config));
                TORSH_TRY(deq, dequantize(std::get<0>(q), std::get<1>(q), std::get<2>(q)));
                return calculate_quantization_metrics(tensor, deq, 32, qbits);
            }
            TORSH_CHECK(config.validate());
            if (data.empty()) return TorshError::invalid_argument("Cannot quantize empty tensor");
            TORSH_TRY(ctx, hip::Runtime::ctx());
            TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
            TORSH_TRY(dmm, hip::DeviceBuffer::alloc(ctx, 2 * sizeof(float)));
            TORSH_CHECK(hip::check(hipq_minmax_f32(ctx, dx.as<float>(), data.size(), dmm.as<float>())));
            TORSH_TRY(mm, dmm.to_host<float>(2));
            auto params = config.scheme == QScheme::PerTensorAffine
                              ? calculate_affine_quantization_params(mm[0], mm[1], config.dtype)
                              : calculate_symmetric_quantization_params(mm[0], mm[1], config.dtype);
            if (params.is_err()) return params.unwrap_err();
            const auto [scale, zp] = params.unwrap();
            if (scale <= 0.0f) return TorshError::invalid_argument("Scale must be positive");
            const int32_t mode = (data.size() > 64 && detail::is_simd_available()) ? HIPQ_FORM_MUL_INV : HIPQ_FORM_DIV;
            TORSH_TRY(dm, hip::DeviceBuffer::alloc(ctx, sizeof(hipq_quant_metrics)));
            // quantize_per_tensor_affine clamps to the i8 range whatever the dtype (algorithms.rs:296-305).
            TORSH_CHECK(hip::check(hipq_fake_quantize_metrics_f32(ctx, dx.as<float>(), data.size(), scale, zp, nullptr,
                                                                  -128, 127, mode, 32, qbits,
                                                                  dm.as<hipq_quant_metrics>())));
            TORSH_TRY(m, dm.to_host<hipq_quant_metrics>(1));
            return detail::from_record(m[0]);
        };
        const auto t0 = std::chrono::steady_clock::now();
        auto r = one();
        const double secs = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        results.push_back({config, r.is_ok() ? r.unwrap() : worst, secs});
    }
    // Higher PSNR first; incomparable pairs (NaN) count as equal (metrics.rs:252-256).
    std::stable_sort(results.begin(), results.end(), [](const ConfigComparison &a, const ConfigComparison &b) {
        return b.metrics.psnr < a.metrics.psnr;
    });
    return results;
}

// metrics.rs:252-338: the eight candidate configurations, each scored by its metrics averaged over the
// calibration tensors; a candidate that meets both thresholds is ranked by compression, the others by
// PSNR per unit of compression; the first best wins.
inline Result<QuantConfig> auto_calibrate_quantization(const std::vector<const Tensor *> &calibration_tensors,
                                                       float target_accuracy_threshold, float max_compression_ratio) {
    if (calibration_tensors.empty()) return TorshError::invalid_argument("No calibration tensors provided");
    const std::vector<QuantConfig> candidates{
        QuantConfig::int8(),           QuantConfig::int8().with_observer(ObserverType::Histogram),
        QuantConfig::per_channel(0),   QuantConfig::per_channel(1),
        QuantConfig::group_wise(0, 8), QuantConfig::group_wise(1, 16),
        QuantConfig::int4(),           QuantConfig::ternary()};
    bool found = false;
    QuantConfig best_config;
    float best_score = -std::numeric_limits<float>::infinity();
    for (const QuantConfig &config : candidates) {
        QuantizationMetrics total;  // QuantizationMetrics::default(): zero_error 100, cosine 1, ratio 1 (metrics.rs:50-63)
        int successful_tests = 0;
        for (const Tensor *tensor : calibration_tensors) {
            auto comparison = compare_quantization_configs(*tensor, {config});
            if (comparison.is_err() || comparison.unwrap().empty()) continue;
            const QuantizationMetrics &m = comparison.unwrap().front().metrics;
            if (!std::isfinite(m.psnr)) continue;
            total.mse += m.mse, total.psnr += m.psnr, total.snr += m.snr, total.mae += m.mae;
            total.max_error = std::fmax(total.max_error, m.max_error);
            total.zero_error_percentage += m.zero_error_percentage;
            total.cosine_similarity += m.cosine_similarity;
            total.compression_ratio += m.compression_ratio;
            ++successful_tests;
        }
        if (successful_tests == 0) continue;
        const float n = static_cast<float>(successful_tests);
        const float psnr = total.psnr / n, ratio = total.compression_ratio / n;
        const float score = (psnr >= target_accuracy_threshold && ratio <= max_compression_ratio)
                                ? ratio + psnr / 100.0f
                                : psnr / ratio;
        if (score > best_score) {
            best_score = score;
            best_config = config;
            found = true;
        }
    }
    if (!found) return TorshError::invalid_argument("No suitable configuration found");
    return best_config;
}

// observers.rs:36-556
class Observer {
  public:
    explicit Observer(ObserverType type) : type_(type), histogram_(256, 0), num_bins_(256) {}  // :57-73
    static Observer min_max() { return Observer(ObserverType::MinMax); }
    static Observer moving_average() { return Observer(ObserverType::MovingAverage); }
    static Observer histogram() { return Observer(ObserverType::Histogram); }
    static Observer new_histogram(size_t num_bins) { return histogram_with_bins(num_bins); }    // :76-91
    static Observer new_percentile(float percentile) { return percentile_with_value(percentile); }  // :94-109
    static Observer histogram_with_bins(size_t num_bins) {
        Observer o(ObserverType::Histogram);
        o.num_bins_ = num_bins;
        o.histogram_.assign(num_bins, 0);
        return o;
    }
    static Observer percentile() { return Observer(ObserverType::Percentile); }
    static Observer percentile_with_value(float percentile) {  // :94-109
        Observer o(ObserverType::Percentile);
        o.percentile_ = percentile;
        return o;
    }

    ObserverType observer_type() const { return type_; }
    std::pair<float, float> get_min_max() const { return {min_val_, max_val_}; }
    size_t num_batches() const { return num_batches_; }
    size_t num_bins() const { return num_bins_; }
    float percentile_value() const { return percentile_; }
    const std::vector<uint64_t> &histogram_counts() const { return histogram_; }
    const std::vector<float> &values() const { return values_; }

    // observers.rs:112-260
    Result<Unit> update(const Tensor &tensor) {
        const std::vector<float> &data = tensor.as_slice();
        num_batches_ += 1;  // counted even when the batch is empty or rejected
        if (data.empty()) return Unit{};
        TORSH_TRY(ctx, hip::Runtime::ctx());
        TORSH_TRY(dx, hip::DeviceBuffer::from_host(ctx, data.data(), data.size()));
        TORSH_TRY(dst, hip::DeviceBuffer::alloc(ctx, sizeof(hipq_observe_stats)));
        TORSH_CHECK(hip::check(hipq_observe_f32(ctx, dx.as<float>(), data.size(), dst.as<hipq_observe_stats>())));
        TORSH_TRY(st, dst.to_host<hipq_observe_stats>(1));
        if (st[0].nonfinite != 0)
            return TorshError::invalid_argument("Tensor contains non-finite values (NaN or infinity)");
        const float batch_min = st[0].min_val, batch_max = st[0].max_val;
        switch (type_) {
        case ObserverType::MovingAverage: {
            // The first-batch branch of the reference tests num_batches == 0 after the increment
            // above (:117, :160) and so never runs: the averages start from 0.
            const float alpha = 0.01f;
            avg_min_ = alpha * batch_min + (1.0f - alpha) * avg_min_;
            avg_max_ = alpha * batch_max + (1.0f - alpha) * avg_max_;
            min_val_ = std::fmin(min_val_, batch_min);
            max_val_ = std::fmax(max_val_, batch_max);
            break;
        }
        case ObserverType::Histogram: {
            min_val_ = std::fmin(min_val_, batch_min);
            max_val_ = std::fmax(max_val_, batch_max);
            hist_min_ = std::fmin(hist_min_, batch_min);
            hist_max_ = std::fmax(hist_max_, batch_max);
            if (num_bins_ == 0) break;
            if (num_bins_ > HIPQ_HISTOGRAM_MAX_BINS)
                return TorshError::not_implemented("histogram observers on the HIP path support up to 16384 bins");
            const float rmin = std::isfinite(hist_min_) ? hist_min_ : min_val_;
            const float rmax = std::isfinite(hist_max_) ? hist_max_ : max_val_;
            // Counters travel with the call: the observer's state lives on the host like the reference's.
            TORSH_TRY(dc, hip::DeviceBuffer::from_host(ctx, histogram_.data(), histogram_.size()));
            TORSH_CHECK(hip::check(hipq_histogram_f32(ctx, dx.as<float>(), data.size(), rmin, rmax, num_bins_,
                                                      dc.as<uint64_t>())));
            TORSH_TRY(counts, dc.to_host<uint64_t>(histogram_.size()));
            histogram_ = std::move(counts);
            break;
        }
        case ObserverType::Percentile: {
            min_val_ = std::fmin(min_val_, batch_min);
            max_val_ = std::fmax(max_val_, batch_max);
            if (values_.size() + data.size() > 100000) {  // :230-239
                const float sample_rate = 100000.0f / static_cast<float>(values_.size() + data.size());
                for (size_t i = 0; i < data.size(); ++i)
                    if (std::fmod(static_cast<float>(i) * sample_rate, 1.0f) < sample_rate) values_.push_back(data[i]);
            } else {
                values_.insert(values_.end(), data.begin(), data.end());
            }
            break;
        }
        default:
            min_val_ = std::fmin(min_val_, batch_min);
            max_val_ = std::fmax(max_val_, batch_max);
            break;
        }
        return Unit{};
    }

    // observers.rs:263-310
    Result<std::pair<float, int32_t>> calculate_qparams(DType dtype) const {
        int32_t qmin, qmax;
        if (dtype == DType::I8) qmin = -128, qmax = 127;
        else if (dtype == DType::U8) qmin = 0, qmax = 255;
        else return TorshError::invalid_argument("Unsupported quantization dtype");
        float mn, mx;
        if (type_ == ObserverType::Histogram && !histogram_.empty()) {
            std::tie(mn, mx) = calculate_histogram_range();
        } else if (type_ == ObserverType::Percentile && !values_.empty()) {
            std::tie(mn, mx) = calculate_percentile_range();
        } else {
            mn = std::fmin(min_val_, 0.0f), mx = std::fmax(max_val_, 0.0f);
        }
        float scale = (mx - mn) / static_cast<float>(qmax - qmin);
        if (scale == 0.0f) scale = 1.0f;
        const float z = std::fmin(std::fmax(std::round(static_cast<float>(qmin) - mn / scale), static_cast<float>(qmin)),
                                  static_cast<float>(qmax));
        return std::make_pair(scale, detail::f32_as_i32(z));
    }

    // observers.rs:336-402
    std::pair<float, float> calculate_histogram_range() const {
        const std::pair<float, float> fallback{min_val_, max_val_};
        if (histogram_.empty() || num_bins_ == 0) return fallback;
        uint64_t total = 0;
        for (uint64_t c : histogram_) total += c;
        if (total == 0) return fallback;
        const float thr = total > 10000 ? 0.001f : (total > 1000 ? 0.005f : 0.01f);
        const size_t threshold_count = detail::f32_as_usize(static_cast<float>(total) * thr);
        size_t start_bin = 0, end_bin = num_bins_ - 1;
        uint64_t cumsum = 0;
        for (size_t i = 0; i < histogram_.size(); ++i) {
            cumsum += histogram_[i];
            if (cumsum > threshold_count) {
                start_bin = i;
                break;
            }
        }
        cumsum = 0;
        for (size_t i = histogram_.size(); i-- > 0;) {
            cumsum += histogram_[i];
            if (cumsum > threshold_count) {
                end_bin = i;
                break;
            }
        }
        if (start_bin >= end_bin) return fallback;
        const float rmin = std::isfinite(hist_min_) ? hist_min_ : min_val_;
        const float rmax = std::isfinite(hist_max_) ? hist_max_ : max_val_;
        if (rmax <= rmin) return fallback;
        const float bin_width = (rmax - rmin) / static_cast<float>(num_bins_);
        const float lo = rmin + static_cast<float>(start_bin) * bin_width;
        const float hi = rmin + static_cast<float>(end_bin + 1) * bin_width;
        if (lo >= hi) return fallback;
        return {std::fmax(lo, min_val_), std::fmin(hi, max_val_)};
    }

    // observers.rs:405-423
    std::pair<float, float> calculate_percentile_range() const {
        if (values_.empty()) return {min_val_, max_val_};
        std::vector<float> sorted = values_;
        std::stable_sort(sorted.begin(), sorted.end());
        const size_t n = sorted.size();
        const float lower_percentile = 100.0f - percentile_, upper_percentile = percentile_;
        const size_t lower_idx = std::min(detail::f32_as_usize((lower_percentile / 100.0f) * static_cast<float>(n)), n - 1);
        const size_t upper_idx = std::min(detail::f32_as_usize((upper_percentile / 100.0f) * static_cast<float>(n)), n - 1);
        return {sorted[lower_idx], sorted[upper_idx]};
    }

    // observers.rs:426-475 (IQR rule on a host slice)
    std::pair<std::vector<float>, size_t> detect_outliers(const std::vector<float> &data, float factor) const {
        if (data.empty()) return {{}, 0};
        std::vector<float> sorted = data;
        std::stable_sort(sorted.begin(), sorted.end());
        const size_t n = sorted.size();
        float q1 = sorted[0], q3 = sorted[n - 1];
        if (n >= 4) {
            const size_t i1 = detail::f32_as_usize(static_cast<float>(n) * 0.25f);
            q1 = i1 > 0 ? sorted[std::min(i1, n - 1)] : sorted[0];
            q3 = sorted[std::min(detail::f32_as_usize(static_cast<float>(n) * 0.75f), n - 1)];
        }
        const float iqr = q3 - q1;
        if (iqr < 1e-6f) return {sorted, 0};
        const float lower = q1 - factor * iqr, upper = q3 + factor * iqr;
        std::vector<float> cleaned;
        for (float x : data)
            if (x >= lower && x <= upper) cleaned.push_back(x);
        const size_t removed = data.size() - cleaned.size();
        return {std::move(cleaned), removed};
    }

    // observers.rs:478-507
    std::map<std::string, float> get_statistics() const {
        std::map<std::string, float> stats;
        stats["min_val"] = min_val_;
        stats["max_val"] = max_val_;
        stats["range"] = max_val_ - min_val_;
        stats["num_batches"] = static_cast<float>(num_batches_);
        if (type_ == ObserverType::Histogram) {
            uint64_t total = 0, peak = 0;
            for (uint64_t c : histogram_) total += c, peak = std::max(peak, c);
            stats["num_bins"] = static_cast<float>(num_bins_);
            stats["total_samples"] = static_cast<float>(total);
            if (!histogram_.empty()) stats["max_bin_count"] = static_cast<float>(peak);
        } else if (type_ == ObserverType::Percentile) {
            stats["total_values"] = static_cast<float>(values_.size());
            stats["percentile"] = percentile_;
        }
        return stats;
    }

    // observers.rs:522-532
    void reset() {
        min_val_ = std::numeric_limits<float>::infinity();
        max_val_ = -std::numeric_limits<float>::infinity();
        num_batches_ = 0;
        avg_min_ = avg_max_ = 0.0f;
        hist_min_ = std::numeric_limits<float>::infinity();
        hist_max_ = -std::numeric_limits<float>::infinity();
        std::fill(histogram_.begin(), histogram_.end(), 0);
        values_.clear();
    }

    std::pair<float, float> get_moving_average() const { return {avg_min_, avg_max_}; }
    std::pair<float, float> get_histogram_bounds() const { return {hist_min_, hist_max_}; }

  private:
    ObserverType type_;
    float min_val_ = std::numeric_limits<float>::infinity();
    float max_val_ = -std::numeric_limits<float>::infinity();
    size_t num_batches_ = 0;
    float avg_min_ = 0.0f, avg_max_ = 0.0f;
    std::vector<uint64_t> histogram_;
    float hist_min_ = std::numeric_limits<float>::infinity();
    float hist_max_ = -std::numeric_limits<float>::infinity();
    size_t num_bins_;
    std::vector<float> values_;
    float percentile_ = 99.99f;
};

// utils.rs:153-180: one observer over all tensors, one (scale, zero_point) for all of them.
inline Result<std::vector<QuantizedTriple>> quantize_batch_consistent(const std::vector<const Tensor *> &tensors,
                                                                      const QuantConfig &config) {
    std::vector<QuantizedTriple> results;
    if (tensors.empty()) return results;
    Observer global_observer(config.observer_type);
    for (const Tensor *t : tensors) TORSH_CHECK(global_observer.update(*t));
    TORSH_TRY(qp, global_observer.calculate_qparams(config.dtype));
    for (const Tensor *t : tensors) {
        TORSH_TRY(q, quantize_per_tensor(*t, qp.first, qp.second, config.dtype));
        results.emplace_back(std::move(q), qp.first, qp.second);
    }
    return results;
}

}  // namespace quantization
}  // namespace torsh
