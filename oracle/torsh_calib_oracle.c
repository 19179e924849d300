/*
 * CPU oracle, second part (see torsh_calib_oracle.h).  TEST INFRASTRUCTURE ONLY.
 *
 * Rust semantics restated in C: `f32::min/max` ignore NaN (fminf/fmaxf), `f32::clamp` keeps
 * NaN, `as usize` / `as i32` from a float saturate with NaN -> 0, `f32 % f32` is fmodf,
 * `powi(2)` is one multiplication, `iter().sum::<f32>()` adds in element order, slice
 * `sort_by` is a stable sort.  Compiled with -ffp-contract=off, so no expression is fused.
 */
#include "torsh_calib_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

static size_t f32_as_usize(float v) {
    if (!(v == v) || v <= 0.0f) return 0;
    if (v >= 18446744073709551616.0f) return SIZE_MAX;
    return (size_t)v;
}

static int32_t f32_as_i32(float v) {
    if (!(v == v)) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}

static float clamp_keep_nan(float v, float lo, float hi) {
    if (v < lo) return lo;
    if (v > hi) return hi;
    return v;
}

/* ---- metrics ------------------------------------------------------------ */

/* metrics.rs:67-175 */
int tq_calculate_quantization_metrics(const float *original, const float *quantized, size_t n,
                                      uint32_t original_bits, uint32_t quantized_bits, tq_metrics *out) {
    if (n == 0) { /* QuantizationMetrics::default(), metrics.rs:50-63 */
        out->mse = 0.0f;
        out->psnr = 0.0f;
        out->snr = 0.0f;
        out->mae = 0.0f;
        out->max_error = 0.0f;
        out->zero_error_percentage = 100.0f;
        out->cosine_similarity = 1.0f;
        out->compression_ratio = 1.0f;
        return 0;
    }
    const float len = (float)n;
    float sse = 0.0f, sae = 0.0f, max_error = 0.0f, spow = 0.0f, max_signal = 0.0f, dot = 0.0f, qq = 0.0f;
    size_t zero_errors = 0;
    for (size_t i = 0; i < n; ++i) { /* :93-98 */
        const float d = original[i] - quantized[i];
        sse += d * d;
    }
    for (size_t i = 0; i < n; ++i) sae += fabsf(original[i] - quantized[i]);                 /* :101-106 */
    for (size_t i = 0; i < n; ++i) max_error = fmaxf(max_error, fabsf(original[i] - quantized[i])); /* :109-113 */
    for (size_t i = 0; i < n; ++i)                                                           /* :116-121 */
        if (fabsf(original[i] - quantized[i]) < 1e-7f) ++zero_errors;
    for (size_t i = 0; i < n; ++i) spow += original[i] * original[i];                       /* :124-125 */
    for (size_t i = 0; i < n; ++i) max_signal = fmaxf(max_signal, fabsf(original[i]));      /* :128-130 */
    const float mse = sse / len;
    const float mae = sae / len;
    const float signal_power = spow / len;
    out->mse = mse;
    out->mae = mae;
    out->max_error = max_error;
    out->zero_error_percentage = ((float)zero_errors / len) * 100.0f;
    out->psnr = mse > 0.0f ? 20.0f * log10f(max_signal / sqrtf(mse)) : INFINITY;            /* :131-135 */
    out->snr = (mse > 0.0f && signal_power > 0.0f) ? 10.0f * log10f(signal_power / mse) : INFINITY; /* :138-142 */
    for (size_t i = 0; i < n; ++i) dot += original[i] * quantized[i];                       /* :145-149 */
    for (size_t i = 0; i < n; ++i) qq += quantized[i] * quantized[i];
    const float on = sqrtf(spow), qn = sqrtf(qq);                                            /* :151-152 */
    out->cosine_similarity = (on > 0.0f && qn > 0.0f) ? dot / (on * qn) : 0.0f;              /* :154-158 */
    out->compression_ratio = (float)original_bits / (float)quantized_bits;                   /* :161 */
    return 0;
}

int tq_calculate_quantization_metrics_f64(const float *original, const float *quantized, size_t n,
                                          uint32_t original_bits, uint32_t quantized_bits, double out[8]) {
    if (n == 0) {
        const double d[8] = {0, 0, 0, 0, 0, 100, 1, 1};
        memcpy(out, d, sizeof d);
        return 0;
    }
    double sse = 0, sae = 0, spow = 0, dot = 0, qq = 0;
    float max_error = 0.0f, max_signal = 0.0f;
    size_t zero_errors = 0;
    for (size_t i = 0; i < n; ++i) {
        const float d = original[i] - quantized[i];
        sse += (double)(d * d);
        sae += (double)fabsf(d);
        max_error = fmaxf(max_error, fabsf(d));
        if (fabsf(d) < 1e-7f) ++zero_errors;
        spow += (double)(original[i] * original[i]);
        max_signal = fmaxf(max_signal, fabsf(original[i]));
        dot += (double)(original[i] * quantized[i]);
        qq += (double)(quantized[i] * quantized[i]);
    }
    const double len = (double)n, mse = sse / len, sp = spow / len;
    out[0] = mse;
    out[1] = mse > 0 ? 20.0 * log10((double)max_signal / sqrt(mse)) : INFINITY;
    out[2] = (mse > 0 && sp > 0) ? 10.0 * log10(sp / mse) : INFINITY;
    out[3] = sae / len;
    out[4] = max_error;
    out[5] = (double)(((float)zero_errors / (float)n) * 100.0f); /* an exact count: the f32 formula itself */
    out[6] = (spow > 0 && qq > 0) ? dot / (sqrt(spow) * sqrt(qq)) : 0.0;
    out[7] = (double)original_bits / (double)quantized_bits;
    return 0;
}

/* ---- observers ---------------------------------------------------------- */

struct tq_observer {
    int type;
    float min_val, max_val;
    size_t num_batches;
    float avg_min, avg_max;
    uint64_t *histogram;
    float hist_min, hist_max;
    size_t num_bins;
    float *values;
    size_t nvalues, cap;
    float percentile;
};

tq_observer *tq_observer_new(int observer_type, size_t num_bins, float percentile) {
    tq_observer *o = (tq_observer *)calloc(1, sizeof *o);
    if (!o) return NULL;
    o->type = observer_type;
    o->num_bins = num_bins ? num_bins : 256;          /* observers.rs:66-69 */
    o->percentile = percentile > 0.0f ? percentile : 99.99f; /* :71 */
    o->histogram = (uint64_t *)calloc(o->num_bins, sizeof(uint64_t));
    tq_observer_reset(o);
    return o;
}

void tq_observer_free(tq_observer *o) {
    if (!o) return;
    free(o->histogram);
    free(o->values);
    free(o);
}

/* observers.rs:522-532 */
void tq_observer_reset(tq_observer *o) {
    o->min_val = INFINITY;
    o->max_val = -INFINITY;
    o->num_batches = 0;
    o->avg_min = 0.0f;
    o->avg_max = 0.0f;
    o->hist_min = INFINITY;
    o->hist_max = -INFINITY;
    memset(o->histogram, 0, o->num_bins * sizeof(uint64_t));
    o->nvalues = 0;
}

/* observers.rs:313-333 */
size_t tq_value_to_bin_index(float value, float range_min, float range_max, size_t num_bins) {
    if (range_max <= range_min || !isfinite(value)) return 0;
    const float ratio = clamp_keep_nan((value - range_min) / (range_max - range_min), 0.0f, 1.0f);
    const size_t idx = f32_as_usize(floorf(ratio * (float)num_bins));
    return idx < num_bins - 1 ? idx : num_bins - 1;
}

void tq_histogram_accumulate(const float *x, size_t n, float range_min, float range_max, size_t num_bins,
                             uint64_t *counts) {
    for (size_t i = 0; i < n; ++i) {
        const size_t b = tq_value_to_bin_index(x[i], range_min, range_max, num_bins);
        if (b < num_bins) counts[b] += 1; /* the bound check of observers.rs:199-201 */
    }
}

static void values_push(tq_observer *o, float v) {
    if (o->nvalues == o->cap) {
        o->cap = o->cap ? o->cap * 2 : 1024;
        o->values = (float *)realloc(o->values, o->cap * sizeof(float));
    }
    o->values[o->nvalues++] = v;
}

/* observers.rs:112-260.  `num_batches` is incremented before the `num_batches == 0` tests of the
 * MovingAverage and Histogram arms (:117 vs :160, :178), so their first-batch branches never
 * run: the moving averages start from 0.0 and the histogram range from (+inf, -inf). */
int tq_observer_update(tq_observer *o, const float *x, size_t n) {
    o->num_batches += 1;
    if (n == 0) return 0;
    for (size_t i = 0; i < n; ++i)
        if (!isfinite(x[i])) return 1; /* InvalidArgument, :123-128 */
    float bmin = INFINITY, bmax = -INFINITY;
    for (size_t i = 0; i < n; ++i) {
        bmin = fminf(bmin, x[i]);
        bmax = fmaxf(bmax, x[i]);
    }
    switch (o->type) {
    case TQ_OBS_MOVING_AVERAGE: {
        const float alpha = 0.01f; /* :166 */
        o->avg_min = alpha * bmin + (1.0f - alpha) * o->avg_min;
        o->avg_max = alpha * bmax + (1.0f - alpha) * o->avg_max;
        o->min_val = fminf(o->min_val, bmin);
        o->max_val = fmaxf(o->max_val, bmax);
        break;
    }
    case TQ_OBS_HISTOGRAM: {
        o->min_val = fminf(o->min_val, bmin);
        o->max_val = fmaxf(o->max_val, bmax);
        o->hist_min = fminf(o->hist_min, bmin); /* :182-183 */
        o->hist_max = fmaxf(o->hist_max, bmax);
        /* value_to_bin_index falls back to min_val/max_val when the histogram range is not
         * finite (:315-324); after the two lines above it always is. */
        const float rmin = isfinite(o->hist_min) ? o->hist_min : o->min_val;
        const float rmax = isfinite(o->hist_max) ? o->hist_max : o->max_val;
        tq_histogram_accumulate(x, n, rmin, rmax, o->num_bins, o->histogram);
        break;
    }
    case TQ_OBS_PERCENTILE: {
        o->min_val = fminf(o->min_val, bmin);
        o->max_val = fmaxf(o->max_val, bmax);
        if (o->nvalues + n > 100000) { /* :230-239 */
            const float sample_rate = 100000.0f / (float)(o->nvalues + n);
            for (size_t i = 0; i < n; ++i)
                if (fmodf((float)i * sample_rate, 1.0f) < sample_rate) values_push(o, x[i]);
        } else {
            for (size_t i = 0; i < n; ++i) values_push(o, x[i]);
        }
        break;
    }
    default: /* MinMax and the types that fall back to it, :153-156, :245-249 */
        o->min_val = fminf(o->min_val, bmin);
        o->max_val = fmaxf(o->max_val, bmax);
        break;
    }
    return 0;
}

/* observers.rs:336-402 */
void tq_observer_histogram_range(const tq_observer *o, float *mn, float *mx) {
    *mn = o->min_val;
    *mx = o->max_val;
    if (o->num_bins == 0) return;
    uint64_t total = 0;
    for (size_t i = 0; i < o->num_bins; ++i) total += o->histogram[i];
    if (total == 0) return;
    const float thr = total > 10000 ? 0.001f : (total > 1000 ? 0.005f : 0.01f);
    const size_t threshold_count = f32_as_usize((float)total * thr);
    uint64_t cumsum = 0;
    size_t start_bin = 0, end_bin = o->num_bins - 1;
    for (size_t i = 0; i < o->num_bins; ++i) {
        cumsum += o->histogram[i];
        if (cumsum > threshold_count) {
            start_bin = i;
            break;
        }
    }
    cumsum = 0;
    for (size_t i = o->num_bins; i-- > 0;) {
        cumsum += o->histogram[i];
        if (cumsum > threshold_count) {
            end_bin = i;
            break;
        }
    }
    if (start_bin >= end_bin) return;
    const float rmin = isfinite(o->hist_min) ? o->hist_min : o->min_val;
    const float rmax = isfinite(o->hist_max) ? o->hist_max : o->max_val;
    if (rmax <= rmin) return;
    const float bin_width = (rmax - rmin) / (float)o->num_bins;
    const float lo = rmin + (float)start_bin * bin_width;
    const float hi = rmin + (float)(end_bin + 1) * bin_width;
    if (lo >= hi) return;
    *mn = fmaxf(lo, o->min_val);
    *mx = fminf(hi, o->max_val);
}

/* Stable merge sort by `<` (slice::sort_by with partial_cmp on finite values). */
static void merge_sort(float *a, float *tmp, size_t n) {
    if (n < 2) return;
    const size_t h = n / 2;
    merge_sort(a, tmp, h);
    merge_sort(a + h, tmp, n - h);
    size_t i = 0, j = h, k = 0;
    while (i < h && j < n) tmp[k++] = (a[j] < a[i]) ? a[j++] : a[i++];
    while (i < h) tmp[k++] = a[i++];
    while (j < n) tmp[k++] = a[j++];
    memcpy(a, tmp, n * sizeof(float));
}

/* observers.rs:405-423 */
void tq_observer_percentile_range(const tq_observer *o, float *mn, float *mx) {
    *mn = o->min_val;
    *mx = o->max_val;
    if (o->nvalues == 0) return;
    const size_t n = o->nvalues;
    float *s = (float *)malloc(2 * n * sizeof(float));
    memcpy(s, o->values, n * sizeof(float));
    merge_sort(s, s + n, n);
    const float lower_percentile = 100.0f - o->percentile;
    const float upper_percentile = o->percentile;
    size_t lower_idx = f32_as_usize((lower_percentile / 100.0f) * (float)n);
    size_t upper_idx = f32_as_usize((upper_percentile / 100.0f) * (float)n);
    if (lower_idx > n - 1) lower_idx = n - 1;
    if (upper_idx > n - 1) upper_idx = n - 1;
    *mn = s[lower_idx];
    *mx = s[upper_idx];
    free(s);
}

/* observers.rs:263-310 */
int tq_observer_calculate_qparams(const tq_observer *o, int dtype, float *scale, int32_t *zp) {
    int32_t qmin, qmax;
    if (dtype == 0) {
        qmin = -128;
        qmax = 127;
    } else if (dtype == 1) {
        qmin = 0;
        qmax = 255;
    } else {
        return 1; /* "Unsupported quantization dtype" */
    }
    float mn, mx;
    if (o->type == TQ_OBS_HISTOGRAM && o->num_bins != 0) {
        tq_observer_histogram_range(o, &mn, &mx);
    } else if (o->type == TQ_OBS_PERCENTILE && o->nvalues != 0) {
        tq_observer_percentile_range(o, &mn, &mx);
    } else {
        mn = fminf(o->min_val, 0.0f);
        mx = fmaxf(o->max_val, 0.0f);
    }
    float s = (mx - mn) / (float)(qmax - qmin);
    if (s == 0.0f) s = 1.0f;
    const float z = fminf(fmaxf(roundf((float)qmin - mn / s), (float)qmin), (float)qmax);
    *scale = s;
    *zp = f32_as_i32(z);
    return 0;
}

void tq_observer_get_min_max(const tq_observer *o, float *mn, float *mx) {
    *mn = o->min_val;
    *mx = o->max_val;
}
void tq_observer_get_avg(const tq_observer *o, float *avg_min, float *avg_max) {
    *avg_min = o->avg_min;
    *avg_max = o->avg_max;
}
void tq_observer_get_hist_range(const tq_observer *o, float *hist_min, float *hist_max) {
    *hist_min = o->hist_min;
    *hist_max = o->hist_max;
}
size_t tq_observer_num_batches(const tq_observer *o) { return o->num_batches; }
size_t tq_observer_num_bins(const tq_observer *o) { return o->num_bins; }
const uint64_t *tq_observer_histogram(const tq_observer *o) { return o->histogram; }
size_t tq_observer_num_values(const tq_observer *o) { return o->nvalues; }
const float *tq_observer_values(const tq_observer *o) { return o->values; }

/* ---- model-level quantizer ---------------------------------------------- */

/* crates/torsh-models/src/quantization.rs:365-392 */
void tq_model_calculate_quantization_params(float min_val, float max_val, int32_t qmin, int32_t qmax, float *scale,
                                            int32_t *zp, float *adj_min, float *adj_max) {
    float amin = min_val, amax = max_val;
    if (fabsf(max_val - min_val) < 1e-8f) {
        amin = min_val - 1e-4f;
        amax = max_val + 1e-4f;
    }
    const float s = (amax - amin) / (float)(qmax - qmin);
    const float zf = (float)qmin - amin / s;
    *scale = s;
    *zp = f32_as_i32(clamp_keep_nan(roundf(zf), (float)qmin, (float)qmax));
    *adj_min = amin;
    *adj_max = amax;
}

/* crates/torsh-models/src/quantization.rs:309-349 */
void tq_model_fake_quantize(const float *x, size_t n, float scale, int32_t zp, int32_t qmin, int32_t qmax,
                            float *out) {
    for (size_t i = 0; i < n; ++i) {
        const float q = roundf(x[i] / scale) + (float)zp;                       /* :337 */
        const int32_t qi = f32_as_i32(clamp_keep_nan(q, (float)qmin, (float)qmax)); /* :340-341 */
        out[i] = (float)(qi - zp) * scale;                                       /* :346 */
    }
}

/* f32::max / f32::min of Rust: the operand that is not NaN. */
static float rust_max(float a, float b) { return (a != a) ? b : ((b != b) ? a : (a > b ? a : b)); }
static float rust_min(float a, float b) { return (a != a) ? b : ((b != b) ? a : (a < b ? a : b)); }

/* crates/torsh-quantization/src/fake_quantize.rs:14-42 */
void tq_fake_quantize_per_tensor_affine(const float *x, size_t n, float scale, int32_t zp, int32_t qmin,
                                        int32_t qmax, float *out) {
    for (size_t i = 0; i < n; ++i) {
        const float quantized = roundf(x[i] / scale) + (float)zp;                     /* :27 */
        const float clamped = rust_min(rust_max(quantized, (float)qmin), (float)qmax); /* :29 */
        out[i] = scale * (clamped - (float)zp);                                       /* :31 */
    }
}

/* crates/torsh-quantization/src/fake_quantize.rs:119-157; dtype TQ_DTYPE_I8 = 0 / TQ_DTYPE_U8 = 1,
 * scheme 0 = PerTensorAffine, 1 = PerTensorSymmetric (the others are errors there). */
int tq_fake_quantize_auto(const float *x, size_t n, int dtype, int scheme, float *out, float *out_scale,
                          int32_t *out_zp) {
    int32_t qmin, qmax;
    if (dtype == 0) {
        qmin = -128, qmax = 127;
    } else if (dtype == 1) {
        qmin = 0, qmax = 255;
    } else {
        return 1; /* "Unsupported quantization dtype" */
    }
    float mn = INFINITY, mx = -INFINITY;
    for (size_t i = 0; i < n; ++i) mn = rust_min(mn, x[i]);  /* :132 */
    mn = rust_min(mn, 0.0f);
    for (size_t i = 0; i < n; ++i) mx = rust_max(mx, x[i]);  /* :133-136 */
    mx = rust_max(mx, 0.0f);
    float scale = (mx - mn) / (float)(qmax - qmin);          /* :138 */
    if (scale == 0.0f) scale = 1.0f;                         /* :139 */
    int32_t zp = 0;
    if (scheme == 0) {
        const float z = rust_min(rust_max(roundf((float)qmin - mn / scale), (float)qmin), (float)qmax); /* :143-146 */
        zp = (int32_t)z;
    } else if (scheme != 1) {
        return 1; /* "Quantization scheme not yet implemented" */
    }
    if (out_scale) *out_scale = scale;
    if (out_zp) *out_zp = zp;
    tq_fake_quantize_per_tensor_affine(x, n, scale, zp, qmin, qmax, out);
    return 0;
}

/* crates/torsh-models/src/quantization.rs:548-566 */
double tq_model_mse_error(const float *original, const float *quantized, size_t n) {
    float sum = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        const float d = original[i] - quantized[i];
        sum += d * d;
    }
    return (double)(sum / (float)n);
}

/* ---- special schemes ------------------------------------------------------ */

/* specialized.rs:33-65 */
int tq_quantize_int4_per_tensor(const float *x, size_t n, float *out, float *scale, int32_t *zp) {
    float mn = INFINITY, mx = -INFINITY;
    for (size_t i = 0; i < n; ++i) {
        mn = fminf(mn, x[i]);
        mx = fmaxf(mx, x[i]);
    }
    mn = fminf(mn, 0.0f);
    mx = fmaxf(mx, 0.0f);
    float s = (mx - mn) / 15.0f;
    if (s == 0.0f) s = 1.0f;
    const int32_t z = f32_as_i32(clamp_keep_nan(roundf(-8.0f - mn / s), -8.0f, 7.0f));
    for (size_t i = 0; i < n; ++i) out[i] = clamp_keep_nan(roundf(x[i] / s) + (float)z, -8.0f, 7.0f);
    *scale = s;
    *zp = z;
    return 0;
}

/* Channel coordinate of flat index i along `axis` (the stride walk of specialized.rs:106-117). */
static size_t channel_of(size_t i, const size_t *shape, size_t ndim, size_t axis) {
    size_t inner = 1;
    for (size_t d = axis + 1; d < ndim; ++d) inner *= shape[d];
    return (i / inner) % shape[axis];
}

/* specialized.rs:68-160 */
int tq_quantize_int4_per_channel(const float *x, const size_t *shape, size_t ndim, size_t axis, float *out,
                                 float *scales, int32_t *zps, float *avg_scale, int32_t *avg_zp) {
    if (axis >= ndim) return 1;
    size_t n = 1;
    for (size_t d = 0; d < ndim; ++d) n *= shape[d];
    const size_t channels = shape[axis];
    for (size_t i = 0; i < n; ++i) out[i] = 0.0f;
    for (size_t ch = 0; ch < channels; ++ch) {
        float mn = INFINITY, mx = -INFINITY;
        for (size_t i = 0; i < n; ++i)
            if (channel_of(i, shape, ndim, axis) == ch) {
                mn = fminf(mn, x[i]);
                mx = fmaxf(mx, x[i]);
            }
        mn = fminf(mn, 0.0f);
        mx = fmaxf(mx, 0.0f);
        float s = (mx - mn) / 15.0f;
        if (s == 0.0f) s = 1.0f;
        const int32_t z = f32_as_i32(clamp_keep_nan(roundf(-8.0f - mn / s), -8.0f, 7.0f));
        scales[ch] = s;
        zps[ch] = z;
        for (size_t i = 0; i < n; ++i)
            if (channel_of(i, shape, ndim, axis) == ch)
                out[i] = clamp_keep_nan(roundf(x[i] / s) + (float)z, -8.0f, 7.0f);
    }
    float ssum = 0.0f;
    int32_t zsum = 0;
    for (size_t ch = 0; ch < channels; ++ch) {
        ssum += scales[ch];
        zsum += zps[ch];
    }
    *avg_scale = ssum / (float)channels;                           /* :154 */
    *avg_zp = f32_as_i32(roundf((float)zsum / (float)channels));   /* :155-156 */
    return 0;
}

/* specialized.rs:163-188 */
int tq_quantize_binary(const float *x, size_t n, float *out, float *scale, double *scale_f64) {
    if (n == 0) return 1;
    float sum = 0.0f;
    double dsum = 0.0;
    for (size_t i = 0; i < n; ++i) {
        sum += fabsf(x[i]);
        dsum += (double)fabsf(x[i]);
    }
    float s = sum / (float)n;
    if (s == 0.0f) s = 1.0f;
    for (size_t i = 0; i < n; ++i) out[i] = x[i] >= 0.0f ? 1.0f : -1.0f;
    *scale = s;
    if (scale_f64) *scale_f64 = dsum == 0.0 ? 1.0 : dsum / (double)n;
    return 0;
}

/* specialized.rs:191-238 */
int tq_quantize_ternary(const float *x, size_t n, float *out, float *scale, double *scale_f64, float *threshold) {
    if (n == 0) return 1;
    float max_abs = 0.0f;
    for (size_t i = 0; i < n; ++i) max_abs = fmaxf(max_abs, fabsf(x[i]));
    const float thr = max_abs * 0.7f;
    float sum = 0.0f;
    double dsum = 0.0;
    size_t count = 0;
    for (size_t i = 0; i < n; ++i)
        if (fabsf(x[i]) > thr) {
            sum += fabsf(x[i]);
            dsum += (double)fabsf(x[i]);
            ++count;
        }
    *scale = count > 0 ? sum / (float)count : 1.0f;
    if (scale_f64) *scale_f64 = count > 0 ? dsum / (double)count : 1.0;
    if (threshold) *threshold = thr;
    for (size_t i = 0; i < n; ++i) out[i] = fabsf(x[i]) <= thr ? 0.0f : (x[i] > 0.0f ? 1.0f : -1.0f);
    return 0;
}

/* specialized.rs:439-492 */
int tq_quantize_binary_learned_threshold(const float *x, size_t n, int has_threshold, float threshold, int f64_sums,
                                         float *out, float *scale, double *scale_f64, float *threshold_out) {
    if (n == 0) return 1;
    float thr = threshold;
    if (!has_threshold) { /* :452-456 */
        float abs_sum = 0.0f;
        double abs_dsum = 0.0;
        for (size_t i = 0; i < n; ++i) {
            abs_sum += fabsf(x[i]);
            abs_dsum += (double)fabsf(x[i]);
        }
        thr = f64_sums ? (float)(abs_dsum / (double)n) : abs_sum / (float)n;
    }
    float sum = 0.0f;
    double dsum = 0.0;
    size_t count = 0;
    for (size_t i = 0; i < n; ++i)
        if (fabsf(x[i]) > thr) { /* :459-463 */
            sum += fabsf(x[i]);
            dsum += (double)fabsf(x[i]);
            ++count;
        }
    *scale = count > 0 ? sum / (float)count : 1.0f;
    if (scale_f64) *scale_f64 = count > 0 ? dsum / (double)count : 1.0;
    if (threshold_out) *threshold_out = thr;
    for (size_t i = 0; i < n; ++i) out[i] = fabsf(x[i]) <= thr ? 0.0f : (x[i] >= 0.0f ? 1.0f : -1.0f); /* :473-481 */
    return 0;
}

/* specialized.rs:555-570 */
static void ternary_error(const float *x, size_t n, float thr, float *err, double *err64) {
    float s = 0.0f;
    double d = 0.0;
    for (size_t i = 0; i < n; ++i) {
        const float q = fabsf(x[i]) <= thr ? 0.0f : (x[i] > 0.0f ? 1.0f : -1.0f);
        const float diff = x[i] - q;
        const float sq = diff * diff;
        s += sq;
        d += (double)sq;
    }
    *err = s / (float)n;
    *err64 = d / (double)n;
}

/* specialized.rs:495-552 */
int tq_quantize_ternary_adaptive(const float *x, size_t n, int f64_sums, float *out, float *scale, double *scale_f64,
                                 float *threshold_out, float errors[10], double errors_f64[10]) {
    if (n == 0) return 1;
    float max_abs = 0.0f;
    for (size_t i = 0; i < n; ++i) max_abs = fmaxf(max_abs, fabsf(x[i]));
    float best_thr = 0.0f, best_err = INFINITY;
    for (int i = 1; i <= 10; ++i) { /* :510-517 */
        const float thr = max_abs * ((float)i * 0.1f);
        float e;
        double e64;
        ternary_error(x, n, thr, &e, &e64);
        if (errors) errors[i - 1] = e;
        if (errors_f64) errors_f64[i - 1] = e64;
        const float cmp = f64_sums ? (float)e64 : e;
        if (cmp < best_err) {
            best_err = cmp;
            best_thr = thr;
        }
    }
    float sum = 0.0f;
    double dsum = 0.0;
    size_t count = 0;
    for (size_t i = 0; i < n; ++i)
        if (fabsf(x[i]) > best_thr) {
            sum += fabsf(x[i]);
            dsum += (double)fabsf(x[i]);
            ++count;
        }
    *scale = count > 0 ? sum / (float)count : 1.0f;
    if (scale_f64) *scale_f64 = count > 0 ? dsum / (double)count : 1.0;
    if (threshold_out) *threshold_out = best_thr;
    for (size_t i = 0; i < n; ++i) out[i] = fabsf(x[i]) <= best_thr ? 0.0f : (x[i] > 0.0f ? 1.0f : -1.0f);
    return 0;
}

/* specialized.rs:241-377 */
int tq_quantize_group_wise(const float *x, const size_t *shape, size_t ndim, size_t axis, size_t group_size,
                           int32_t qmin, int32_t qmax, float *out, float *group_scales, int32_t *group_zps,
                           float *avg_scale, int32_t *avg_zp) {
    if (axis >= ndim || group_size == 0) return 1;
    size_t n = 1;
    for (size_t d = 0; d < ndim; ++d) n *= shape[d];
    const size_t channels = shape[axis];
    const size_t groups = (channels + group_size - 1) / group_size;
    for (size_t i = 0; i < n; ++i) out[i] = 0.0f;
    size_t produced = 0;
    for (size_t g = 0; g < groups; ++g) {
        const size_t c0 = g * group_size, c1 = c0 + group_size < channels ? c0 + group_size : channels;
        float mn = INFINITY, mx = -INFINITY;
        size_t members = 0;
        for (size_t i = 0; i < n; ++i) {
            const size_t c = channel_of(i, shape, ndim, axis);
            if (c >= c0 && c < c1) {
                mn = fminf(mn, x[i]);
                mx = fmaxf(mx, x[i]);
                ++members;
            }
        }
        if (members == 0) continue; /* :301-303 */
        mn = fminf(mn, 0.0f);
        mx = fmaxf(mx, 0.0f);
        float s = (mx - mn) / (float)(qmax - qmin);
        if (s == 0.0f) s = 1.0f;
        const int32_t z = f32_as_i32(fminf(fmaxf(roundf((float)qmin - mn / s), (float)qmin), (float)qmax));
        group_scales[produced] = s;
        group_zps[produced] = z;
        ++produced;
        for (size_t i = 0; i < n; ++i) {
            const size_t c = channel_of(i, shape, ndim, axis);
            if (c >= c0 && c < c1) out[i] = fminf(fmaxf(roundf(x[i] / s) + (float)z, (float)qmin), (float)qmax);
        }
    }
    if (produced == 0) {
        *avg_scale = 1.0f;
        *avg_zp = 0;
        return 0;
    }
    float ssum = 0.0f;
    int32_t zsum = 0;
    for (size_t g = 0; g < produced; ++g) {
        ssum += group_scales[g];
        zsum += group_zps[g];
    }
    *avg_scale = ssum / (float)produced;
    *avg_zp = f32_as_i32(roundf((float)zsum / (float)produced));
    return 0;
}
