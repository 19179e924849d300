/*
 * CPU oracle, second part: calibration observers, quality metrics and the
 * model-level fake quantization of ToRSh.  TEST INFRASTRUCTURE ONLY, like
 * torsh_quant_oracle.h: a plain-C restatement of the reference's CPU formulas
 * used as the checker by the parity tests.  Nothing in the shipped library
 * links, loads or calls it.
 *
 * Every function names the reference lines it restates (paths relative to the
 * reference root).
 */
#ifndef TORSH_CALIB_ORACLE_H
#define TORSH_CALIB_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- quality metrics: crates/torsh-quantization/src/metrics.rs:30-175 ---- */
typedef struct {
    float mse, psnr, snr, mae, max_error, zero_error_percentage, cosine_similarity, compression_ratio;
} tq_metrics;

/* calculate_quantization_metrics, metrics.rs:67-175: sequential f32 sums in element order. */
int tq_calculate_quantization_metrics(const float *original, const float *quantized, size_t n,
                                      uint32_t original_bits, uint32_t quantized_bits, tq_metrics *out);
/* The same eight quantities with every sum carried in f64 (elementwise terms still f32, as
 * in the reference): the value the f32 formulas approach without the rounding a long
 * sequential f32 sum accumulates.  Used to separate kernel error from that rounding. */
int tq_calculate_quantization_metrics_f64(const float *original, const float *quantized, size_t n,
                                          uint32_t original_bits, uint32_t quantized_bits, double out[8]);

/* ---- observers: crates/torsh-quantization/src/observers.rs -------------- */
/* ObserverType, crates/torsh-quantization/src/config.rs:78-91 */
enum {
    TQ_OBS_MINMAX = 0,
    TQ_OBS_MOVING_AVERAGE = 1,
    TQ_OBS_HISTOGRAM = 2,
    TQ_OBS_PERCENTILE = 3,
    TQ_OBS_KL_DIVERGENCE = 4,
    TQ_OBS_ENTROPY = 5
};

typedef struct tq_observer tq_observer;

/* Observer::new / new_histogram / new_percentile, observers.rs:57-109.  num_bins 0 -> 256,
 * percentile <= 0 -> 99.99 (the defaults of Observer::new). */
tq_observer *tq_observer_new(int observer_type, size_t num_bins, float percentile);
void tq_observer_free(tq_observer *o);
/* Observer::update, observers.rs:112-260. */
int tq_observer_update(tq_observer *o, const float *x, size_t n);
/* Observer::calculate_qparams, observers.rs:263-310 (dtype: TQ_DTYPE_I8 = 0, TQ_DTYPE_U8 = 1). */
int tq_observer_calculate_qparams(const tq_observer *o, int dtype, float *scale, int32_t *zp);
/* Observer::reset, observers.rs:522-532. */
void tq_observer_reset(tq_observer *o);
/* State readers (get_min_max, num_batches, the histogram, the retained values). */
void tq_observer_get_min_max(const tq_observer *o, float *mn, float *mx);
void tq_observer_get_avg(const tq_observer *o, float *avg_min, float *avg_max);
void tq_observer_get_hist_range(const tq_observer *o, float *hist_min, float *hist_max);
size_t tq_observer_num_batches(const tq_observer *o);
size_t tq_observer_num_bins(const tq_observer *o);
const uint64_t *tq_observer_histogram(const tq_observer *o);
size_t tq_observer_num_values(const tq_observer *o);
const float *tq_observer_values(const tq_observer *o);
/* calculate_histogram_range / calculate_percentile_range, observers.rs:336-423. */
void tq_observer_histogram_range(const tq_observer *o, float *mn, float *mx);
void tq_observer_percentile_range(const tq_observer *o, float *mn, float *mx);

/* value_to_bin_index, observers.rs:313-333, as a free function of the range. */
size_t tq_value_to_bin_index(float value, float range_min, float range_max, size_t num_bins);
/* Histogram of x over [range_min, range_max] added into counts[num_bins]. */
void tq_histogram_accumulate(const float *x, size_t n, float range_min, float range_max, size_t num_bins,
                             uint64_t *counts);

/* ---- model-level quantizer: crates/torsh-models/src/quantization.rs ------ */
/* ModelQuantizer::calculate_quantization_params, quantization.rs:365-392.
 * Writes the adjusted range too (it is stored in QuantizationParams). */
void tq_model_calculate_quantization_params(float min_val, float max_val, int32_t qmin, int32_t qmax, float *scale,
                                            int32_t *zp, float *adj_min, float *adj_max);
/* ModelQuantizer::quantize_tensor, quantization.rs:309-349: quantize_value then
 * dequantize_value per element ("fake quantization"). */
void tq_model_fake_quantize(const float *x, size_t n, float scale, int32_t zp, int32_t qmin, int32_t qmax,
                            float *out);
/* ---- QAT fake quantization: crates/torsh-quantization/src/fake_quantize.rs ---- */
/* fake_quantize_per_tensor_affine, fake_quantize.rs:14-42: round(x / scale) + zp, clamped with
 * f32::max then f32::min (a NaN becomes qmin), out = scale * (clamped - zp). */
void tq_fake_quantize_per_tensor_affine(const float *x, size_t n, float scale, int32_t zp, int32_t qmin,
                                        int32_t qmax, float *out);
/* fake_quantize_auto, fake_quantize.rs:119-157 (range widened to include 0, scale 0 -> 1).
 * Returns non-zero for a dtype or scheme the reference rejects. */
int tq_fake_quantize_auto(const float *x, size_t n, int dtype, int scheme, float *out, float *out_scale,
                          int32_t *out_zp);
/* ModelQuantizer::calculate_mse_error, quantization.rs:548-566 (f32 sum, result widened). */
double tq_model_mse_error(const float *original, const float *quantized, size_t n);

/* ---- special schemes: crates/torsh-quantization/src/specialized.rs -------- */
/* quantize_int4_per_tensor, specialized.rs:33-65 (f32 carrier, range -8..7). */
int tq_quantize_int4_per_tensor(const float *x, size_t n, float *out, float *scale, int32_t *zp);
/* quantize_int4_per_channel, specialized.rs:68-160.  scales / zps (num_channels each) receive the
 * per-channel parameters; avg_scale / avg_zp are what the function returns. */
int tq_quantize_int4_per_channel(const float *x, const size_t *shape, size_t ndim, size_t axis, float *out,
                                 float *scales, int32_t *zps, float *avg_scale, int32_t *avg_zp);
/* quantize_binary, specialized.rs:163-188; scale_f64 (may be NULL) receives the mean of |x| from an
 * f64 sum. */
int tq_quantize_binary(const float *x, size_t n, float *out, float *scale, double *scale_f64);
/* quantize_ternary, specialized.rs:191-238; threshold (may be NULL) receives 0.7 * max|x|. */
int tq_quantize_ternary(const float *x, size_t n, float *out, float *scale, double *scale_f64, float *threshold);
/* quantize_binary_learned_threshold, specialized.rs:439-492.  has_threshold == 0 learns the
 * threshold as mean |x|.  f64_sums != 0 forms that mean (and nothing else) from an f64 sum instead
 * of the reference's sequential f32 sum: the threshold the f32 sum approaches, and the one a
 * reduction in any other order can be compared with element by element.  scale is always the
 * reference's f32 sum; scale_f64 (may be NULL) the f64 one.  threshold_out receives the threshold. */
int tq_quantize_binary_learned_threshold(const float *x, size_t n, int has_threshold, float threshold, int f64_sums,
                                         float *out, float *scale, double *scale_f64, float *threshold_out);
/* quantize_ternary_adaptive, specialized.rs:495-552 with calculate_ternary_error, :555-570.
 * errors (may be NULL) receives the ten mean errors as the reference forms them (f32 sums),
 * errors_f64 (may be NULL) the same from f64 sums; f64_sums != 0 selects the threshold by the
 * latter. */
int tq_quantize_ternary_adaptive(const float *x, size_t n, int f64_sums, float *out, float *scale, double *scale_f64,
                                 float *threshold_out, float errors[10], double errors_f64[10]);
/* quantize_group_wise, specialized.rs:241-377 with the integer range [qmin, qmax] of
 * config.get_qint_range().  group_scales / group_zps hold num_groups = ceil(shape[axis]/group_size). */
int tq_quantize_group_wise(const float *x, const size_t *shape, size_t ndim, size_t axis, size_t group_size,
                           int32_t qmin, int32_t qmax, float *out, float *group_scales, int32_t *group_zps,
                           float *avg_scale, int32_t *avg_zp);

#ifdef __cplusplus
}
#endif
#endif
