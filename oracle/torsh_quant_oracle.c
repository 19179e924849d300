/*
 * CPU oracle for ToRSh's quantized-inference path.  TEST INFRASTRUCTURE ONLY.
 *
 * Plain-C restatement of the reference's CPU formulas (the reference is Rust
 * and cannot be compiled where this is built).  It is the checker for the
 * device kernels and the timed CPU baseline; the shipped library never links,
 * loads or calls it.  Build: gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   - the known-answer vectors the reference's own unit tests hold
 *     (tests/golden/reference_vectors.json),
 *   - crafted tie / saturation / NaN / degenerate-range vectors whose answers
 *     follow from the Rust std definitions (round half away, NaN-ignoring
 *     min/max, saturating casts),
 *   - brute-force int64 numpy products for the integer GEMM / conv,
 *   - invariants from the reference's property tests (range, determinism).
 * Parity unpinned by any reference-held test: the fused Linear / Conv epilogues
 * (tq_linear_dequant_epilogue, tq_requantize_epilogue) - the reference has no
 * such fused function; they are pinned only by closed form against float64.
 *
 * Citations are paths under the reference root, file:line.
 */
#define _POSIX_C_SOURCE 200809L
#include "torsh_quant_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int g_round_mode = 0;

void tq_set_round_mode(int mode) { g_round_mode = mode ? 1 : 0; }
int tq_get_round_mode(void) { return g_round_mode; }

int tq_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* Rust f32::round = half away from zero; mode 1 = IEEE nearest-even. */
static inline float rnd(float v) { return g_round_mode ? rintf(v) : roundf(v); }

/* Rust f32::clamp: NaN stays NaN. */
static inline float clampf_rust(float v, float lo, float hi) {
    if (v < lo) return lo;
    if (v > hi) return hi;
    return v;
}

/* Rust `f32 as i32`: saturating, NaN -> 0. */
static inline int32_t f32_as_i32(float v) {
    if (isnan(v)) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}

static inline int8_t f32_as_i8(float v) {
    if (isnan(v)) return 0;
    if (v >= 127.0f) return 127;
    if (v <= -128.0f) return -128;
    return (int8_t)v;
}

static inline uint8_t f32_as_u8(float v) {
    if (isnan(v)) return 0;
    if (v >= 255.0f) return 255;
    if (v <= 0.0f) return 0;
    return (uint8_t)v;
}

static inline int32_t clampi(int32_t v, int32_t lo, int32_t hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* crates/torsh-quantization/src/algorithms.rs:425-433 */
void tq_get_dtype_range(int dtype, int32_t *qmin, int32_t *qmax) {
    switch (dtype) {
    case TQ_DTYPE_I8: *qmin = -128; *qmax = 127; break;
    case TQ_DTYPE_U8: *qmin = 0; *qmax = 255; break;
    case TQ_DTYPE_I16: *qmin = -32768; *qmax = 32767; break;
    case TQ_DTYPE_I32: *qmin = INT32_MIN; *qmax = INT32_MAX; break;
    default: *qmin = -128; *qmax = 127; break;
    }
}

/* crates/torsh-quantization/src/simd_ops.rs:84-121: chunks of 1024 reduced in
 * parallel; f32::min/max ignore NaN, so the result is order independent. */
int tq_find_min_max(const float *x, size_t n, float *mn, float *mx) {
    if (n == 0) return TQ_ERR_INVALID_ARGUMENT;
    float gmin = INFINITY, gmax = -INFINITY;
    const size_t chunk = 1024;
    if (n > chunk) {
        const long nchunks = (long)((n + chunk - 1) / chunk);
#pragma omp parallel
        {
            float lmin = INFINITY, lmax = -INFINITY;
#pragma omp for schedule(static) nowait
            for (long c = 0; c < nchunks; ++c) {
                size_t b = (size_t)c * chunk, e = b + chunk < n ? b + chunk : n;
                for (size_t i = b; i < e; ++i) {
                    lmin = fminf(lmin, x[i]);
                    lmax = fmaxf(lmax, x[i]);
                }
            }
#pragma omp critical
            {
                gmin = fminf(gmin, lmin);
                gmax = fmaxf(gmax, lmax);
            }
        }
    } else {
        for (size_t i = 0; i < n; ++i) {
            gmin = fminf(gmin, x[i]);
            gmax = fmaxf(gmax, x[i]);
        }
    }
    *mn = gmin;
    *mx = gmax;
    return TQ_OK;
}

/* crates/torsh-quantization/src/algorithms.rs:103-105 (small-tensor fold). */
int tq_min_max_fold(const float *x, size_t n, float *mn, float *mx) {
    float a = INFINITY, b = -INFINITY;
    for (size_t i = 0; i < n; ++i) {
        a = fminf(a, x[i]);
        b = fmaxf(b, x[i]);
    }
    *mn = a;
    *mx = b;
    return TQ_OK;
}

/* crates/torsh-quantization/src/algorithms.rs:397-422 */
int tq_calculate_symmetric_params(float mn, float mx, int dtype, float *scale, int32_t *zp) {
    if (!isfinite(mn) || !isfinite(mx)) return TQ_ERR_INVALID_ARGUMENT;
    int32_t qmin, qmax;
    tq_get_dtype_range(dtype, &qmin, &qmax);
    (void)qmin;
    float abs_max = fmaxf(fabsf(mn), fabsf(mx));
    if (abs_max < FLT_EPSILON) {
        *scale = 1.0f;
        *zp = 0;
        return TQ_OK;
    }
    *scale = abs_max / (float)qmax;
    *zp = 0;
    return TQ_OK;
}

/* crates/torsh-quantization/src/algorithms.rs:358-394 */
int tq_calculate_affine_params(float mn, float mx, int dtype, float *scale, int32_t *zp) {
    if (!isfinite(mn) || !isfinite(mx)) return TQ_ERR_INVALID_ARGUMENT;
    if (mn > mx) return TQ_ERR_INVALID_ARGUMENT;
    int32_t qmin_i, qmax_i;
    tq_get_dtype_range(dtype, &qmin_i, &qmax_i);
    float qmin = (float)qmin_i, qmax = (float)qmax_i;
    if (fabsf(mx - mn) < FLT_EPSILON) {
        *scale = 1.0f;
        *zp = f32_as_i32(qmin);
        return TQ_OK;
    }
    float s = (mx - mn) / (qmax - qmin);
    float zp_fp = qmin - mn / s;
    *scale = s;
    *zp = f32_as_i32(clampf_rust(roundf(zp_fp), qmin, qmax)); /* always f32::round */
    return TQ_OK;
}

/* crates/torsh-quantization/src/simd_ops.rs:18-49: x * (1/scale), round, + zp,
 * clamp to the i8 range whatever the dtype; f32 carrier output. */
int tq_quantize_per_tensor_affine_simd(const float *x, size_t n, float scale, int32_t zp, float *out) {
    if (scale <= 0.0f) return TQ_ERR_INVALID_ARGUMENT;
    const float inv = 1.0f / scale;
    const float zpf = (float)zp;
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)n; ++i) {
        float q = rnd(x[i] * inv) + zpf;
        out[i] = clampf_rust(q, -128.0f, 127.0f);
    }
    return TQ_OK;
}

/* crates/torsh-quantization/src/simd_ops.rs:196-227 */
int tq_quantize_to_int8_simd(const float *x, size_t n, float scale, int32_t zp, int8_t *out) {
    if (scale <= 0.0f) return TQ_ERR_INVALID_ARGUMENT;
    const float inv = 1.0f / scale;
    const float zpf = (float)zp;
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)n; ++i) {
        float q = rnd(x[i] * inv) + zpf;
        out[i] = f32_as_i8(clampf_rust(q, -128.0f, 127.0f));
    }
    return TQ_OK;
}

/* crates/torsh-quantization/src/simd_ops.rs:52-81 */
int tq_dequantize_per_tensor_affine_simd(const float *q, size_t n, float scale, int32_t zp, float *out) {
    if (scale <= 0.0f) return TQ_ERR_INVALID_ARGUMENT;
    const float zpf = (float)zp;
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)n; ++i) out[i] = (q[i] - zpf) * scale;
    return TQ_OK;
}

/* crates/torsh-quantization/src/algorithms.rs:277-315: len > 64 takes the
 * multiply-by-inverse body above, len <= 64 divides. */
int tq_quantize_per_tensor_affine(const float *x, size_t n, float scale, int32_t zp, float *out) {
    if (scale <= 0.0f) return TQ_ERR_INVALID_ARGUMENT;
    if (n > 64) return tq_quantize_per_tensor_affine_simd(x, n, scale, zp, out);
    for (size_t i = 0; i < n; ++i) {
        float q = rnd(x[i] / scale) + (float)zp;
        out[i] = clampf_rust(q, -128.0f, 127.0f);
    }
    return TQ_OK;
}

/* crates/torsh-quantization/src/algorithms.rs:245-274: always divides. */
int tq_quantize_per_tensor_affine_i8(const float *x, size_t n, float scale, int32_t zp, int8_t *out) {
    if (scale <= 0.0f) return TQ_ERR_INVALID_ARGUMENT;
    for (size_t i = 0; i < n; ++i) {
        float q = rnd(x[i] / scale) + (float)zp;
        out[i] = f32_as_i8(clampf_rust(q, -128.0f, 127.0f));
    }
    return TQ_OK;
}

/* crates/torsh-quantization/src/algorithms.rs:318-355 (both branches compute
 * (q - zp) * scale). */
int tq_dequantize_per_tensor_affine(const float *q, size_t n, float scale, int32_t zp, float *out) {
    if (scale <= 0.0f) return TQ_ERR_INVALID_ARGUMENT;
    if (n > 64) return tq_dequantize_per_tensor_affine_simd(q, n, scale, zp, out);
    for (size_t i = 0; i < n; ++i) out[i] = (q[i] - (float)zp) * scale;
    return TQ_OK;
}

/* crates/torsh-quantization/src/algorithms.rs:85-123 */
int tq_quantize_tensor_auto(const float *x, size_t n, int dtype, int scheme, float *out, float *scale,
                            int32_t *zp) {
    if (n == 0) return TQ_ERR_INVALID_ARGUMENT;
    float mn, mx;
    if (n > 64)
        tq_find_min_max(x, n, &mn, &mx);
    else
        tq_min_max_fold(x, n, &mn, &mx);
    int rc;
    if (scheme == TQ_PER_TENSOR_AFFINE)
        rc = tq_calculate_affine_params(mn, mx, dtype, scale, zp);
    else if (scheme == TQ_PER_TENSOR_SYMMETRIC)
        rc = tq_calculate_symmetric_params(mn, mx, dtype, scale, zp);
    else
        return TQ_ERR_INVALID_ARGUMENT;
    if (rc) return rc;
    return tq_quantize_per_tensor_affine(x, n, *scale, *zp, out);
}

static void row_major_strides(const size_t *shape, size_t ndim, size_t *strides) {
    strides[ndim - 1] = 1;
    for (size_t i = ndim - 1; i-- > 0;) strides[i] = strides[i + 1] * shape[i + 1];
}

/* crates/torsh-quantization/src/algorithms.rs:126-242.  The reference walks a
 * multi-dimensional index per element; the flat index it reaches for element i
 * of channel ch is outer*stride[axis]*shape[axis] + ch*stride[axis] + inner,
 * which is what is computed here.  Division form, dtype-range clamp. */
int tq_quantize_per_channel_auto(const float *x, const size_t *shape, size_t ndim, size_t axis, int dtype,
                                 int scheme, float *out, float *scales, int32_t *zps) {
    if (ndim == 0 || axis >= ndim) return TQ_ERR_INVALID_ARGUMENT;
    if (scheme != TQ_PER_CHANNEL_AFFINE && scheme != TQ_PER_CHANNEL_SYMMETRIC) return TQ_ERR_INVALID_ARGUMENT;
    size_t strides[16];
    if (ndim > 16) return TQ_ERR_INVALID_ARGUMENT;
    row_major_strides(shape, ndim, strides);
    size_t total = 1;
    for (size_t i = 0; i < ndim; ++i) total *= shape[i];
    const size_t nch = shape[axis];
    if (nch == 0) return TQ_OK;
    const size_t inner = strides[axis];
    const size_t outer = total / (nch * inner);
    int32_t qmin, qmax;
    tq_get_dtype_range(dtype, &qmin, &qmax);
    for (size_t ch = 0; ch < nch; ++ch) {
        float cmin = INFINITY, cmax = -INFINITY;
        for (size_t o = 0; o < outer; ++o)
            for (size_t in = 0; in < inner; ++in) {
                float v = x[(o * nch + ch) * inner + in];
                cmin = fminf(cmin, v);
                cmax = fmaxf(cmax, v);
            }
        float s;
        int32_t z;
        int rc = scheme == TQ_PER_CHANNEL_AFFINE ? tq_calculate_affine_params(cmin, cmax, dtype, &s, &z)
                                                 : tq_calculate_symmetric_params(cmin, cmax, dtype, &s, &z);
        if (rc) return rc;
        scales[ch] = s;
        zps[ch] = z;
        for (size_t o = 0; o < outer; ++o)
            for (size_t in = 0; in < inner; ++in) {
                size_t idx = (o * nch + ch) * inner + in;
                float q = rnd(x[idx] / s) + (float)z;
                out[idx] = clampf_rust(q, (float)qmin, (float)qmax);
            }
    }
    return TQ_OK;
}

/* crates/torsh-quantization/src/simd_ops.rs:124-169: contiguous channels, each
 * through the multiply-by-inverse per-tensor body. */
int tq_quantize_per_channel_simd(const float *x, size_t n, const float *scales, const int32_t *zps,
                                 size_t num_channels, size_t channel_size, float *out) {
    if (n != num_channels * channel_size) return TQ_ERR_INVALID_ARGUMENT;
    for (size_t ch = 0; ch < num_channels; ++ch) {
        if (scales[ch] <= 0.0f) return TQ_ERR_INVALID_ARGUMENT;
        int rc = tq_quantize_per_tensor_affine_simd(x + ch * channel_size, channel_size, scales[ch], zps[ch],
                                                    out + ch * channel_size);
        if (rc) return rc;
    }
    return TQ_OK;
}

/* crates/torsh-quantization/src/quantize.rs:287-331 */
int tq_quantize_per_channel_affine(const float *x, const size_t *shape, size_t ndim, size_t axis,
                                   const float *scales, const int32_t *zps, size_t nparams, float *out) {
    if (ndim == 0 || ndim > 16 || axis >= ndim) return TQ_ERR_INVALID_ARGUMENT;
    if (nparams != shape[axis]) return TQ_ERR_INVALID_ARGUMENT;
    size_t strides[16];
    row_major_strides(shape, ndim, strides);
    size_t total = 1;
    for (size_t i = 0; i < ndim; ++i) total *= shape[i];
    for (size_t idx = 0; idx < total; ++idx) {
        size_t ch = (idx / strides[axis]) % shape[axis];
        float q = rnd(x[idx] / scales[ch]) + (float)zps[ch];
        out[idx] = (float)f32_as_i8(clampf_rust(q, -128.0f, 127.0f));
    }
    return TQ_OK;
}

/* crates/torsh-quantization/src/dequantize.rs:46-89 */
int tq_dequantize_per_channel_affine(const float *q, const size_t *shape, size_t ndim, size_t axis,
                                     const float *scales, const int32_t *zps, size_t nparams, float *out) {
    if (ndim == 0 || ndim > 16 || axis >= ndim) return TQ_ERR_INVALID_ARGUMENT;
    if (nparams != shape[axis]) return TQ_ERR_INVALID_ARGUMENT;
    size_t strides[16];
    row_major_strides(shape, ndim, strides);
    size_t total = 1;
    for (size_t i = 0; i < ndim; ++i) total *= shape[i];
    for (size_t idx = 0; idx < total; ++idx) {
        size_t ch = (idx / strides[axis]) % shape[axis];
        out[idx] = scales[ch] * (q[idx] - (float)zps[ch]);
    }
    return TQ_OK;
}

/* crates/torsh-core/src/dtype/quantized.rs:129-134: zero point added BEFORE
 * rounding. */
int8_t tq_qint8_quantize(float v, float scale, int32_t zp) {
    int32_t q = f32_as_i32(rnd(v / scale + (float)zp));
    return (int8_t)clampi(q, -128, 127);
}

/* crates/torsh-core/src/dtype/quantized.rs:285-290 */
uint8_t tq_quint8_quantize(float v, float scale, int32_t zp) {
    int32_t q = f32_as_i32(rnd(v / scale + (float)zp));
    return (uint8_t)clampi(q, 0, 255);
}

/* crates/torsh-nn/src/quantization/ops.rs:153-156 */
int32_t tq_nn_quantize_value_symmetric(float v, float scale, int32_t qmin, int32_t qmax) {
    return clampi(f32_as_i32(rnd(v / scale)), qmin, qmax);
}

/* crates/torsh-nn/src/quantization/ops.rs:159-162 (i32 add wraps in release
 * builds; saturating input keeps it in range for every tested value). */
int32_t tq_nn_quantize_value_asymmetric(float v, float scale, int32_t zp, int32_t qmin, int32_t qmax) {
    int64_t q = (int64_t)f32_as_i32(rnd(v / scale)) + zp;
    if (q < qmin) q = qmin;
    if (q > qmax) q = qmax;
    return (int32_t)q;
}

/* crates/torsh-nn/src/quantization/ops.rs:170-172 */
float tq_nn_dequantize_value_asymmetric(int32_t q, float scale, int32_t zp) { return (float)(q - zp) * scale; }

/* crates/torsh-nn/src/quantization/ops.rs:296-373, Symmetric + I8 arm:
 * scale = max(|min|,|max|)/127 with no zero guard, value stored as the
 * two's-complement byte widened to f32 (so negatives appear as 256+q). */
int tq_nn_per_channel_quantize_weights_sym_i8(const float *w, size_t channels, size_t channel_size,
                                              float *out_carrier, float *scales) {
    for (size_t c = 0; c < channels; ++c) {
        float mn = INFINITY, mx = -INFINITY;
        for (size_t i = 0; i < channel_size; ++i) {
            mn = fminf(mn, w[c * channel_size + i]);
            mx = fmaxf(mx, w[c * channel_size + i]);
        }
        float s = fmaxf(fabsf(mx), fabsf(mn)) / 127.0f;
        scales[c] = s;
        for (size_t i = 0; i < channel_size; ++i) {
            int32_t q = tq_nn_quantize_value_symmetric(w[c * channel_size + i], s, -128, 127);
            out_carrier[c * channel_size + i] = (float)(uint8_t)(int8_t)q;
        }
    }
    return TQ_OK;
}

/* crates/torsh-nn/src/quantization/ops.rs:296-373, Asymmetric + U8 arm:
 * scale = (max - min)/255, zero_point = round(-min/scale) as i32 (not clamped), value =
 * clamp((round(v/scale) as i32) + zero_point, 0, 255) stored as the byte widened to f32. */
int tq_nn_per_channel_quantize_weights_asym_u8(const float *w, size_t channels, size_t channel_size,
                                               float *out_carrier, float *scales, int32_t *zps) {
    for (size_t c = 0; c < channels; ++c) {
        float mn = INFINITY, mx = -INFINITY;
        for (size_t i = 0; i < channel_size; ++i) {
            mn = fminf(mn, w[c * channel_size + i]);
            mx = fmaxf(mx, w[c * channel_size + i]);
        }
        float s = (mx - mn) / 255.0f;
        int32_t zp = f32_as_i32(roundf(-mn / s));
        scales[c] = s;
        zps[c] = zp;
        for (size_t i = 0; i < channel_size; ++i) {
            int32_t q = tq_nn_quantize_value_asymmetric(w[c * channel_size + i], s, zp, 0, 255);
            out_carrier[c * channel_size + i] = (float)(uint8_t)q;
        }
    }
    return TQ_OK;
}

/* One carrier value of a torsh-nn quantized tensor back to f32: dequantize_from_int8 / _int16
 * (crates/torsh-nn/src/quantization/ops.rs:110-125, 146-150: the zero point is not used) or
 * dequantize_from_uint8 (ops.rs:128-143). */
static inline float nn_dequantize_carrier(float v, float scale, int32_t zp, int is_u8) {
    const int32_t q = f32_as_i32(roundf(v));
    return is_u8 ? (float)(q - zp) * scale : (float)q * scale;
}
/* quantize_tensor (ops.rs:11-24) on one value: int8 / int16 take the symmetric formula, uint8 the asymmetric. */
static inline float nn_quantize_carrier(float v, float scale, int32_t zp, int is_u8, int32_t qmin, int32_t qmax) {
    return (float)(is_u8 ? tq_nn_quantize_value_asymmetric(v, scale, zp, qmin, qmax)
                         : tq_nn_quantize_value_symmetric(v, scale, qmin, qmax));
}

/* quantized_matmul_int8, crates/torsh-nn/src/quantization/ops.rs:175-194: dequantize both operands, multiply in
 * f32, quantize the product with the caller's output parameters.  a [m,k], b [k,n], f32 carriers.  The f32 product
 * is a plain i, j, l loop here; the reference's Tensor::matmul picks among several f32 kernels
 * (crates/torsh-tensor/src/ops/matrix.rs:83-160) whose order of summation is not fixed, so results are comparable
 * to within the f32 summation error, i.e. one output code. */
int tq_nn_quantized_matmul_int8(const float *a, const float *b, size_t m, size_t k, size_t n, float sa, int32_t zpa,
                                int a_u8, float sb, int32_t zpb, int b_u8, float so, int32_t zpo, int o_u8,
                                int32_t qmin, int32_t qmax, float *out) {
    for (size_t i = 0; i < m; ++i)
        for (size_t j = 0; j < n; ++j) {
            float acc = 0.0f;
            for (size_t l = 0; l < k; ++l)
                acc += nn_dequantize_carrier(a[i * k + l], sa, zpa, a_u8) * nn_dequantize_carrier(b[l * n + j], sb, zpb, b_u8);
            out[i * n + j] = nn_quantize_carrier(acc, so, zpo, o_u8, qmin, qmax);
        }
    return TQ_OK;
}

/* quantized_conv2d_int8, ops.rs:197-237: dequantize input, weight and (optional) bias, f32 convolution (dilation 1,
 * one group; padded taps are the real value 0), quantize with the caller's output parameters.  Summation order:
 * kh, kw, ic (the same caveat as for the product above). */
int tq_nn_quantized_conv2d_int8(const float *x, const float *w, const float *bias, size_t nb, size_t c_in, size_t h,
                                size_t wd, size_t c_out, size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                                size_t pad_h, size_t pad_w, float sx, int32_t zpx, int x_u8, float sw, int32_t zpw,
                                int w_u8, float sbias, int32_t zpb, int b_u8, float so, int32_t zpo, int o_u8,
                                int32_t qmin, int32_t qmax, float *out) {
    if (stride_h == 0 || stride_w == 0) return TQ_ERR_INVALID_ARGUMENT;
    if (h + 2 * pad_h < kh || wd + 2 * pad_w < kw) return TQ_ERR_INVALID_ARGUMENT;
    const size_t ho = (h + 2 * pad_h - kh) / stride_h + 1, wo = (wd + 2 * pad_w - kw) / stride_w + 1;
    for (size_t b = 0; b < nb; ++b)
        for (size_t oc = 0; oc < c_out; ++oc)
            for (size_t oh = 0; oh < ho; ++oh)
                for (size_t ow = 0; ow < wo; ++ow) {
                    float acc = 0.0f;
                    for (size_t r = 0; r < kh; ++r)
                        for (size_t s = 0; s < kw; ++s)
                            for (size_t ic = 0; ic < c_in; ++ic) {
                                size_t ih = oh * stride_h + r, iw = ow * stride_w + s;
                                if (ih < pad_h || iw < pad_w) continue;
                                ih -= pad_h;
                                iw -= pad_w;
                                if (ih >= h || iw >= wd) continue;
                                acc += nn_dequantize_carrier(x[((b * c_in + ic) * h + ih) * wd + iw], sx, zpx, x_u8) *
                                       nn_dequantize_carrier(w[((oc * c_in + ic) * kh + r) * kw + s], sw, zpw, w_u8);
                            }
                    if (bias) acc += nn_dequantize_carrier(bias[oc], sbias, zpb, b_u8);
                    out[((b * c_out + oc) * ho + oh) * wo + ow] = nn_quantize_carrier(acc, so, zpo, o_u8, qmin, qmax);
                }
    return TQ_OK;
}

/* quantized_relu_int8, ops.rs:261-294: the code of the real value 0 by the asymmetric formula (whatever the
 * dtype), then max on the carrier: `(value as i32) > zero ? value : zero as f32`. */
int tq_nn_quantized_relu_int8(const float *x, size_t n, float scale, int32_t zp, int32_t qmin, int32_t qmax, float *out) {
    const int32_t zero_q = tq_nn_quantize_value_asymmetric(0.0f, scale, zp, qmin, qmax);
    for (size_t i = 0; i < n; ++i) out[i] = f32_as_i32(x[i]) > zero_q ? x[i] : (float)zero_q;
    return TQ_OK;
}

/* crates/torsh-backend/src/quantization/ops.rs:185-195 */
int32_t tq_backend_quantize_value(float v, float scale, int32_t zp, int32_t qmin, int32_t qmax) {
    float q = rnd(v / scale) + (float)zp;
    return f32_as_i32(clampf_rust(q, (float)qmin, (float)qmax));
}

/* crates/torsh-backend/src/quantization/ops.rs:198-200 */
float tq_backend_dequantize_value(int32_t q, float scale, int32_t zp) { return scale * (float)(q - zp); }

/* crates/torsh-backend/src/quantization/params.rs:323-340 */
int tq_backend_params_symmetric(float mn, float mx, int32_t qmin, int32_t qmax, float *scale, int32_t *zp) {
    if (mn > mx || !isfinite(mn) || !isfinite(mx)) return TQ_ERR_INVALID_ARGUMENT;
    float max_range = fmaxf(fabsf(mx), fabsf(mn));
    *scale = max_range == 0.0f ? 1.0f : (2.0f * max_range) / ((float)qmax - (float)qmin);
    *zp = 0;
    return TQ_OK;
}

/* crates/torsh-backend/src/quantization/params.rs:343-363 */
int tq_backend_params_asymmetric(float mn, float mx, int32_t qmin, int32_t qmax, float *scale, int32_t *zp) {
    if (mn > mx || !isfinite(mn) || !isfinite(mx)) return TQ_ERR_INVALID_ARGUMENT;
    if (mx == mn) {
        *scale = 1.0f;
        *zp = qmin;
        return TQ_OK;
    }
    float fqmin = (float)qmin, fqmax = (float)qmax;
    float s = (mx - mn) / (fqmax - fqmin);
    float z = fqmin - mn / s;
    *scale = s;
    *zp = f32_as_i32(clampf_rust(roundf(z), fqmin, fqmax)); /* always f32::round */
    return TQ_OK;
}

/* crates/torsh-backend/src/quantization/ops.rs:295-364: per-value
 * quantize_value, ChannelWise = contiguous equal chunks, result byte = i32 as u8. */
int tq_backend_quantize_f32(const float *x, size_t n, const float *scales, const int32_t *zps,
                            size_t num_channels, int32_t qmin, int32_t qmax, uint8_t *out) {
    if (n == 0) return TQ_OK;
    if (num_channels == 0) return TQ_ERR_INVALID_ARGUMENT;
    size_t channel_size = num_channels > 1 ? n / num_channels : n;
    if (channel_size == 0) return TQ_ERR_INVALID_ARGUMENT;
    for (size_t i = 0; i < n; ++i) {
        size_t ch = num_channels > 1 ? i / channel_size : 0;
        if (ch >= num_channels) ch = num_channels - 1;
        out[i] = (uint8_t)tq_backend_quantize_value(x[i], scales[ch], zps[ch], qmin, qmax);
    }
    return TQ_OK;
}

/* crates/torsh-backend/src/quantization/ops.rs:366-435 */
int tq_backend_dequantize_f32(const uint8_t *q, size_t n, const float *scales, const int32_t *zps,
                              size_t num_channels, int is_signed, float *out) {
    if (n == 0) return TQ_OK;
    if (num_channels == 0) return TQ_ERR_INVALID_ARGUMENT;
    size_t channel_size = num_channels > 1 ? n / num_channels : n;
    if (channel_size == 0) return TQ_ERR_INVALID_ARGUMENT;
    for (size_t i = 0; i < n; ++i) {
        size_t ch = num_channels > 1 ? i / channel_size : 0;
        if (ch >= num_channels) ch = num_channels - 1;
        int32_t v = is_signed ? (int32_t)(int8_t)q[i] : (int32_t)q[i];
        out[i] = tq_backend_dequantize_value(v, scales[ch], zps[ch]);
    }
    return TQ_OK;
}

/* crates/torsh-backend/src/quantization/ops.rs:582-606 (qadd) and :608-624 (qrelu) */
int tq_backend_qadd_or_qrelu(const uint8_t *a, int a_signed, float a_scale, int32_t a_zp, const uint8_t *b,
                             int b_signed, float b_scale, int32_t b_zp, size_t n, int symmetric, int32_t qmin,
                             int32_t qmax, uint8_t *out, float *out_scale, int32_t *out_zp) {
    float *f = (float *)malloc((n ? n : 1) * sizeof(float));
    float *g = (float *)malloc((n ? n : 1) * sizeof(float));
    if (!f || !g) {
        free(f);
        free(g);
        return TQ_ERR_INVALID_ARGUMENT;
    }
    tq_backend_dequantize_f32(a, n, &a_scale, &a_zp, 1, a_signed, f);
    float mn = INFINITY, mx = -INFINITY;
    if (b) {
        tq_backend_dequantize_f32(b, n, &b_scale, &b_zp, 1, b_signed, g);
        for (size_t i = 0; i < n; ++i) f[i] = f[i] + g[i];
        for (size_t i = 0; i < n; ++i) mn = fminf(mn, f[i]);
        for (size_t i = 0; i < n; ++i) mx = fmaxf(mx, f[i]);
    } else {
        for (size_t i = 0; i < n; ++i) f[i] = fmaxf(f[i], 0.0f);
        for (size_t i = 0; i < n; ++i) mx = fmaxf(mx, f[i]);
        mn = 0.0f;
        mx = fmaxf(mx, 0.0f);
    }
    int rc = symmetric ? tq_backend_params_symmetric(mn, mx, qmin, qmax, out_scale, out_zp)
                       : tq_backend_params_asymmetric(mn, mx, qmin, qmax, out_scale, out_zp);
    if (rc == TQ_OK) rc = tq_backend_quantize_f32(f, n, out_scale, out_zp, 1, qmin, qmax, out);
    free(f);
    free(g);
    return rc;
}

/* crates/torsh-backend/src/quantization/specialized.rs:175-201: A [M,K] bytes
 * read as i8, B [K,N] row-major bytes read as i8, i32 accumulate in k order;
 * the reference then stores clamp(acc,-128,127) as a byte.  Both are returned
 * (either pointer may be NULL).  Loop order and the stride-N reads of B are the
 * reference's. */
int tq_backend_matmul_i32(const uint8_t *a, const uint8_t *b_kn, size_t m, size_t k, size_t n,
                          int32_t *acc_out, uint8_t *clamped_out) {
    for (size_t i = 0; i < m; ++i)
        for (size_t j = 0; j < n; ++j) {
            int32_t acc = 0;
            for (size_t l = 0; l < k; ++l) {
                int32_t av = (int32_t)(int8_t)a[i * k + l];
                int32_t bv = (int32_t)(int8_t)b_kn[l * n + j];
                acc += av * bv;
            }
            if (acc_out) acc_out[i * n + j] = acc;
            if (clamped_out) clamped_out[i * n + j] = (uint8_t)clampi(acc, -128, 127);
        }
    return TQ_OK;
}

/* crates/torsh-backend/src/quantization/operations.rs:637-713 (integer part):
 * NCHW, acc += (x_q - zp_in) * w_q over kh, kw, ic.  The reference lets padded
 * taps contribute (0 - zp_in) * w; a padded tap is the real value 0, i.e. the
 * quantized value zp_in, so it contributes 0 here (the two agree when
 * zp_in == 0, the only case the reference's formula is right for). */
int tq_backend_conv2d_i32(const uint8_t *x, int x_signed, int32_t zp_in, const int8_t *w, size_t nb,
                          size_t c_in, size_t h, size_t wd, size_t c_out, size_t kh, size_t kw,
                          size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w, int32_t *acc_out) {
    if (stride_h == 0 || stride_w == 0) return TQ_ERR_INVALID_ARGUMENT;
    if (h + 2 * pad_h < kh || wd + 2 * pad_w < kw) return TQ_ERR_INVALID_ARGUMENT;
    const size_t ho = (h + 2 * pad_h - kh) / stride_h + 1;
    const size_t wo = (wd + 2 * pad_w - kw) / stride_w + 1;
#pragma omp parallel for collapse(2) schedule(static)
    for (long b = 0; b < (long)nb; ++b)
        for (long oc = 0; oc < (long)c_out; ++oc)
            for (size_t oh = 0; oh < ho; ++oh)
                for (size_t ow = 0; ow < wo; ++ow) {
                    int32_t acc = 0;
                    for (size_t r = 0; r < kh; ++r)
                        for (size_t s = 0; s < kw; ++s)
                            for (size_t ic = 0; ic < c_in; ++ic) {
                                size_t ih = oh * stride_h + r, iw = ow * stride_w + s;
                                if (ih < pad_h || iw < pad_w) continue;
                                ih -= pad_h;
                                iw -= pad_w;
                                if (ih >= h || iw >= wd) continue;
                                uint8_t raw = x[(((size_t)b * c_in + ic) * h + ih) * wd + iw];
                                int32_t xv = (x_signed ? (int32_t)(int8_t)raw : (int32_t)raw) - zp_in;
                                int32_t wv = (int32_t)w[(((size_t)oc * c_in + ic) * kh + r) * kw + s];
                                acc += xv * wv;
                            }
                    acc_out[(((size_t)b * c_out + oc) * ho + oh) * wo + ow] = acc;
                }
    return TQ_OK;
}

/* Same integers as tq_backend_matmul_i32 with the weight held [N,K] (the
 * transpose of the reference's B): acc[m,n] = sum_k a[m,k] * w[n,k]. */
int tq_gemm_i8_nk(const int8_t *a, const int8_t *w_nk, size_t m, size_t n, size_t k, int32_t *acc) {
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)m; ++i)
        for (size_t j = 0; j < n; ++j) {
            int32_t s = 0;
            const int8_t *ar = a + (size_t)i * k, *wr = w_nk + j * k;
            for (size_t l = 0; l < k; ++l) s += (int32_t)ar[l] * (int32_t)wr[l];
            acc[(size_t)i * n + j] = s;
        }
    return TQ_OK;
}

/* Dequantize-with-bias epilogue of the quantized Linear:
 *   out[m,n] = (acc as f32) * (s_a * s_w[n]) + bias[n]
 * built from crates/torsh-backend/src/quantization/operations.rs:669,722
 * (acc as f32 * (s_in * s_w)) and the f32 bias add of
 * crates/torsh-backend/src/quantization/ops.rs:561.  No fused multiply-add. */
int tq_linear_dequant_epilogue(const int32_t *acc, size_t m, size_t n, const float *sa, int sa_per_row,
                               const float *sw, const float *bias, float *out) {
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)m; ++i) {
        const float s_a = sa_per_row ? sa[i] : sa[0];
        for (size_t j = 0; j < n; ++j) {
            float s = s_a * sw[j];
            float v = (float)acc[(size_t)i * n + j] * s;
            if (bias) v = v + bias[j];
            out[(size_t)i * n + j] = v;
        }
    }
    return TQ_OK;
}

/* Requantize epilogue (tail of operations.rs:716-724 generalised to a supplied
 * output scale): v = acc*(s_a*s_w[c]) (+ bias[c]); q = clamp(round(v / s_out)
 * + zp_out, qmin, qmax).  Layout: rows x cols accumulators; the weight channel
 * c is the column (Linear, channel_axis_is_row = 0) or (row / inner) % ... for
 * NCHW conv output viewed as [nb*c_out, ho*wo] (channel_axis_is_row = 1,
 * c = row % inner where inner = c_out). */
int tq_requantize_epilogue(const int32_t *acc, size_t rows, size_t cols, const float *sa, int sa_per_row,
                           const float *sw, const float *bias, float s_out, int32_t zp_out, int32_t qmin,
                           int32_t qmax, int channel_axis_is_row, size_t inner, int8_t *out) {
    if (s_out <= 0.0f) return TQ_ERR_INVALID_ARGUMENT;
    for (size_t i = 0; i < rows; ++i) {
        const float s_a = sa_per_row ? sa[i] : sa[0];
        for (size_t j = 0; j < cols; ++j) {
            size_t c = channel_axis_is_row ? i % inner : j;
            float s = s_a * sw[c];
            float v = (float)acc[i * cols + j] * s;
            if (bias) v = v + bias[c];
            float q = rnd(v / s_out) + (float)zp_out;
            out[i * cols + j] = (int8_t)f32_as_i32(clampf_rust(q, (float)qmin, (float)qmax));
        }
    }
    return TQ_OK;
}

/* LayerNorm over the last dimension, biased variance, eps inside the sqrt
 * (crates/torsh-nn/src/layers/normalization/layer_group/mod.rs, eps = 1e-5 at
 * :660).  Accumulated in double so the oracle is the more exact side. */
int tq_layer_norm(const float *x, size_t rows, size_t cols, const float *gamma, const float *beta, float eps,
                  float *out) {
    for (size_t r = 0; r < rows; ++r) {
        const float *xr = x + r * cols;
        double mean = 0.0;
        for (size_t c = 0; c < cols; ++c) mean += xr[c];
        mean /= (double)cols;
        double var = 0.0;
        for (size_t c = 0; c < cols; ++c) {
            double d = xr[c] - mean;
            var += d * d;
        }
        var /= (double)cols;
        double rstd = 1.0 / sqrt(var + (double)eps);
        for (size_t c = 0; c < cols; ++c) {
            double v = (xr[c] - mean) * rstd;
            if (gamma) v *= gamma[c];
            if (beta) v += beta[c];
            out[r * cols + c] = (float)v;
        }
    }
    return TQ_OK;
}

/* tanh-form GELU, crates/torsh-nn/src/layers/activation/modern.rs:124-136:
 * 0.5*x*(1+tanh(sqrt(2/pi)*(x+0.044715*x^3))). */
int tq_gelu_tanh(const float *x, size_t n, float *out) {
    const double c = sqrt(2.0 / 3.14159265358979323846);
    for (size_t i = 0; i < n; ++i) {
        double v = x[i];
        out[i] = (float)(0.5 * v * (1.0 + tanh(c * (v + 0.044715 * v * v * v))));
    }
    return TQ_OK;
}

static double now_s(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

/* CPU baseline, quantize -> dequantize round trip with the reference's call
 * structure: min/max reduce, symmetric params, multiply-by-inverse quantize to
 * an f32 carrier, dequantize (crates/torsh-quantization/src/algorithms.rs:85-123,
 * 318-355).  Returns the best-of-reps seconds for one round trip. */
double tq_time_roundtrip_c1(const float *x, size_t n, float *scratch_q, float *scratch_y, int reps) {
    double best = 1e30;
    for (int r = 0; r < reps; ++r) {
        double t0 = now_s();
        float scale;
        int32_t zp;
        tq_quantize_tensor_auto(x, n, TQ_DTYPE_I8, TQ_PER_TENSOR_SYMMETRIC, scratch_q, &scale, &zp);
        tq_dequantize_per_tensor_affine(scratch_q, n, scale, zp, scratch_y);
        double t1 = now_s();
        if (t1 - t0 < best) best = t1 - t0;
    }
    return best;
}

/* CPU baseline, integer GEMM: the reference's single-threaded i,j,l loop over
 * the first m_sample rows of A (crates/torsh-backend/src/quantization/
 * specialized.rs:187-198).  Returns seconds. */
double tq_time_matmul_rows(const uint8_t *a, const uint8_t *b_kn, size_t m_sample, size_t k, size_t n,
                           int32_t *acc) {
    double t0 = now_s();
    tq_backend_matmul_i32(a, b_kn, m_sample, k, n, acc, NULL);
    return now_s() - t0;
}

/* crates/torsh-quantization/src/algorithms.rs:473-522 (quantize_per_tensor_affine_cache_aware), 581-635
 * (quantize_matrix_cache_friendly), 638-674 (quantize_streaming_with_prefetch) and simd_ops.rs:302-350
 * (quantize_neon_optimized): chunking, tiling and prefetch hints differ, the element formula does not. */
int tq_quantize_cache_aware(const float *x, size_t n, float scale, int32_t zp, float *out) {
    if (scale <= 0.0f) return TQ_ERR_INVALID_ARGUMENT;
    const float inv = 1.0f / scale;
    const float zpf = (float)zp;
    for (size_t i = 0; i < n; ++i) out[i] = clampf_rust(roundf(x[i] * inv) + zpf, -128.0f, 127.0f);
    return TQ_OK;
}

/* crates/torsh-quantization/src/simd_ops.rs:390-446 */
int tq_quantize_mobile_optimized(const float *x, size_t n, float scale, int32_t zp, int reduced_precision,
                                 int8_t *out) {
    if (scale <= 0.0f) return TQ_ERR_INVALID_ARGUMENT;
    const float inv = 1.0f / scale; /* both branches of :409-414 */
    const float zpf = (float)zp;
    const int chunked = n > 256; /* :421 */
    for (size_t i = 0; i < n; ++i) {
        float q;
        if (chunked && reduced_precision)
            q = floorf(x[i] * inv + 0.5f) + zpf; /* :426-428 */
        else
            q = roundf(x[i] * inv) + zpf;
        out[i] = f32_as_i8(clampf_rust(q, -128.0f, 127.0f));
    }
    return TQ_OK;
}

/* crates/torsh-quantization/src/simd_ops.rs:230-262; the sums run in element order here, in
 * rayon's tree order there (f64 terms, so the two agree to ~1e-16 relative). */
int tq_calculate_tensor_stats_simd(const float *x, size_t n, float out[5]) {
    if (n == 0) return TQ_ERR_INVALID_ARGUMENT;
    float mn, mx;
    int rc = tq_find_min_max(x, n, &mn, &mx);
    if (rc != TQ_OK) return rc;
    double sum = 0.0;
    for (size_t i = 0; i < n; ++i) sum += (double)x[i];
    const double mean = sum / (double)n;
    double vs = 0.0;
    for (size_t i = 0; i < n; ++i) {
        const double d = (double)x[i] - mean;
        vs += d * d;
    }
    const double variance = vs / (double)n;
    out[0] = mn;
    out[1] = mx;
    out[2] = (float)mean;
    out[3] = (float)sqrt(variance);
    out[4] = (float)variance;
    return TQ_OK;
}

/* crates/torsh-quantization/src/algorithms.rs:525-578 */
int tq_calculate_tensor_stats_cache_optimized(const float *x, size_t n, float out[4]) {
    if (n == 0) return TQ_ERR_INVALID_ARGUMENT;
    float mn = INFINITY, mx = -INFINITY;
    double sum = 0.0, sumsq = 0.0;
    for (size_t i = 0; i < n; ++i) {
        mn = fminf(mn, x[i]);
        mx = fmaxf(mx, x[i]);
        const double v = (double)x[i];
        sum += v;
        sumsq += v * v;
    }
    const double nd = (double)n;
    const float mean = (float)(sum / nd);
    const float variance = (float)(sumsq / nd - (double)mean * (double)mean); /* :573 */
    out[0] = mn;
    out[1] = mx;
    out[2] = mean;
    out[3] = sqrtf(variance);
    return TQ_OK;
}
