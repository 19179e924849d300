/*
 * CPU oracle for ToRSh's quantized-inference path.  TEST INFRASTRUCTURE ONLY:
 * a plain-C restatement of the reference's CPU formulas, used as the checker by
 * the parity tests, by the smoke check and as the timed CPU baseline.  Nothing
 * in the shipped library links, loads or calls it.
 *
 * Every function names the reference lines it restates (paths relative to the
 * reference root).  The reference is Rust; `f32::round` is round-half-away-
 * from-zero (C `roundf`), `f32::min/max` ignore NaN (C `fminf/fmaxf`),
 * `f32::clamp` keeps NaN, `as i8/i32/u8` from float saturates with NaN -> 0.
 *
 * Return value: 0 on success, TQ_ERR_INVALID_ARGUMENT where the reference
 * returns `TorshError::InvalidArgument`.
 */
#ifndef TORSH_QUANT_ORACLE_H
#define TORSH_QUANT_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { TQ_OK = 0, TQ_ERR_INVALID_ARGUMENT = 1 };

/* torsh_core::DType subset used by get_dtype_range (algorithms.rs:425-433). */
enum { TQ_DTYPE_I8 = 0, TQ_DTYPE_U8 = 1, TQ_DTYPE_I16 = 2, TQ_DTYPE_I32 = 3, TQ_DTYPE_OTHER = 4 };

/* QScheme subset (config.rs:31-52). */
enum {
    TQ_PER_TENSOR_AFFINE = 0,
    TQ_PER_TENSOR_SYMMETRIC = 1,
    TQ_PER_CHANNEL_AFFINE = 2,
    TQ_PER_CHANNEL_SYMMETRIC = 3
};

/* Rounding used by every formula below.  0 = half away from zero (reference
 * behaviour), 1 = half to even.  Process-wide switch so one oracle serves both
 * the reference mode and the half-even variant the kernels also offer. */
void tq_set_round_mode(int mode);
int tq_get_round_mode(void);
/* Number of OpenMP threads the parallel (rayon-like) loops will use. */
int tq_num_threads(void);

/* ---- torsh-quantization ------------------------------------------------ */
void tq_get_dtype_range(int dtype, int32_t *qmin, int32_t *qmax);
int tq_find_min_max(const float *x, size_t n, float *mn, float *mx);
int tq_min_max_fold(const float *x, size_t n, float *mn, float *mx);
int tq_calculate_symmetric_params(float mn, float mx, int dtype, float *scale, int32_t *zp);
int tq_calculate_affine_params(float mn, float mx, int dtype, float *scale, int32_t *zp);
int tq_quantize_per_tensor_affine_simd(const float *x, size_t n, float scale, int32_t zp, float *out);
int tq_quantize_to_int8_simd(const float *x, size_t n, float scale, int32_t zp, int8_t *out);
int tq_dequantize_per_tensor_affine_simd(const float *q, size_t n, float scale, int32_t zp, float *out);
int tq_quantize_per_tensor_affine(const float *x, size_t n, float scale, int32_t zp, float *out);
int tq_quantize_per_tensor_affine_i8(const float *x, size_t n, float scale, int32_t zp, int8_t *out);
int tq_dequantize_per_tensor_affine(const float *q, size_t n, float scale, int32_t zp, float *out);
int tq_quantize_tensor_auto(const float *x, size_t n, int dtype, int scheme, float *out, float *scale, int32_t *zp);
int tq_quantize_per_channel_auto(const float *x, const size_t *shape, size_t ndim, size_t axis, int dtype,
                                 int scheme, float *out, float *scales, int32_t *zps);
int tq_quantize_per_channel_simd(const float *x, size_t n, const float *scales, const int32_t *zps,
                                 size_t num_channels, size_t channel_size, float *out);
/* The cache-aware, tiled, streaming and NEON twins of the per-tensor quantizer share one element
 * formula, clamp(round(x * (1/scale)) + zp, -128, 127) into an f32 carrier:
 * crates/torsh-quantization/src/algorithms.rs:473-522, 581-635, 638-674; simd_ops.rs:302-350. */
int tq_quantize_cache_aware(const float *x, size_t n, float scale, int32_t zp, float *out);
/* quantize_mobile_optimized, simd_ops.rs:390-446: int8 output; with reduced precision and more
 * than 256 elements the rounding is floor(x * inv + 0.5) instead of round. */
int tq_quantize_mobile_optimized(const float *x, size_t n, float scale, int32_t zp, int reduced_precision,
                                 int8_t *out);
/* calculate_tensor_stats_simd, simd_ops.rs:230-262: out = {min, max, mean, std_dev, variance}. */
int tq_calculate_tensor_stats_simd(const float *x, size_t n, float out[5]);
/* calculate_tensor_stats_cache_optimized, algorithms.rs:525-578: out = {min, max, mean, std_dev}. */
int tq_calculate_tensor_stats_cache_optimized(const float *x, size_t n, float out[4]);
int tq_quantize_per_channel_affine(const float *x, const size_t *shape, size_t ndim, size_t axis,
                                   const float *scales, const int32_t *zps, size_t nparams, float *out);
int tq_dequantize_per_channel_affine(const float *q, const size_t *shape, size_t ndim, size_t axis,
                                     const float *scales, const int32_t *zps, size_t nparams, float *out);

/* ---- torsh-core scalar Q types ---------------------------------------- */
int8_t tq_qint8_quantize(float v, float scale, int32_t zp);
uint8_t tq_quint8_quantize(float v, float scale, int32_t zp);

/* ---- torsh-nn::quantization ------------------------------------------- */
int32_t tq_nn_quantize_value_symmetric(float v, float scale, int32_t qmin, int32_t qmax);
int32_t tq_nn_quantize_value_asymmetric(float v, float scale, int32_t zp, int32_t qmin, int32_t qmax);
float tq_nn_dequantize_value_asymmetric(int32_t q, float scale, int32_t zp);
int tq_nn_per_channel_quantize_weights_sym_i8(const float *w, size_t channels, size_t channel_size,
                                              float *out_carrier, float *scales);
int tq_nn_per_channel_quantize_weights_asym_u8(const float *w, size_t channels, size_t channel_size,
                                               float *out_carrier, float *scales, int32_t *zps);

/* quantized_matmul_int8 / quantized_conv2d_int8 / quantized_relu_int8 (crates/torsh-nn/src/quantization/ops.rs:175-294)
 * on f32 carriers; *_u8 = 1 selects the uint8 (asymmetric) value formulas, 0 the int8 / int16 (symmetric) ones. */
int tq_nn_quantized_matmul_int8(const float *a, const float *b, size_t m, size_t k, size_t n, float sa, int32_t zpa,
                                int a_u8, float sb, int32_t zpb, int b_u8, float so, int32_t zpo, int o_u8,
                                int32_t qmin, int32_t qmax, float *out);
int tq_nn_quantized_conv2d_int8(const float *x, const float *w, const float *bias, size_t nb, size_t c_in, size_t h,
                                size_t wd, size_t c_out, size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                                size_t pad_h, size_t pad_w, float sx, int32_t zpx, int x_u8, float sw, int32_t zpw,
                                int w_u8, float sbias, int32_t zpb, int b_u8, float so, int32_t zpo, int o_u8,
                                int32_t qmin, int32_t qmax, float *out);
int tq_nn_quantized_relu_int8(const float *x, size_t n, float scale, int32_t zp, int32_t qmin, int32_t qmax, float *out);

/* ---- torsh-backend::quantization -------------------------------------- */
int32_t tq_backend_quantize_value(float v, float scale, int32_t zp, int32_t qmin, int32_t qmax);
float tq_backend_dequantize_value(int32_t q, float scale, int32_t zp);
int tq_backend_params_symmetric(float mn, float mx, int32_t qmin, int32_t qmax, float *scale, int32_t *zp);
int tq_backend_params_asymmetric(float mn, float mx, int32_t qmin, int32_t qmax, float *scale, int32_t *zp);
int tq_backend_quantize_f32(const float *x, size_t n, const float *scales, const int32_t *zps,
                            size_t num_channels, int32_t qmin, int32_t qmax, uint8_t *out);
int tq_backend_dequantize_f32(const uint8_t *q, size_t n, const float *scales, const int32_t *zps,
                              size_t num_channels, int is_signed, float *out);
int tq_backend_matmul_i32(const uint8_t *a, const uint8_t *b_kn, size_t m, size_t k, size_t n,
                          int32_t *acc_out, uint8_t *clamped_out);
int tq_backend_conv2d_i32(const uint8_t *x, int x_signed, int32_t zp_in, const int8_t *w, size_t nb,
                          size_t c_in, size_t h, size_t wd, size_t c_out, size_t kh, size_t kw,
                          size_t stride_h, size_t stride_w, size_t pad_h, size_t pad_w, int32_t *acc_out);

/* CpuQuantizationOps::qadd / qrelu, crates/torsh-backend/src/quantization/ops.rs:582-624: dequantize,
 * operate in f32, from_statistics on the result's range (symmetric != 0 selects the Symmetric
 * formula, else the Asymmetric one), quantize into [qmin, qmax].  b == NULL means qrelu. */
int tq_backend_qadd_or_qrelu(const uint8_t *a, int a_signed, float a_scale, int32_t a_zp, const uint8_t *b,
                             int b_signed, float b_scale, int32_t b_zp, size_t n, int symmetric, int32_t qmin,
                             int32_t qmax, uint8_t *out, float *out_scale, int32_t *out_zp);

/* ---- compositions the device path is checked against ------------------ */
int tq_gemm_i8_nk(const int8_t *a, const int8_t *w_nk, size_t m, size_t n, size_t k, int32_t *acc);
int tq_linear_dequant_epilogue(const int32_t *acc, size_t m, size_t n, const float *sa, int sa_per_row,
                               const float *sw, const float *bias, float *out);
int tq_requantize_epilogue(const int32_t *acc, size_t rows, size_t cols, const float *sa, int sa_per_row,
                           const float *sw, const float *bias, float s_out, int32_t zp_out, int32_t qmin,
                           int32_t qmax, int channel_axis_is_row, size_t inner, int8_t *out);
int tq_layer_norm(const float *x, size_t rows, size_t cols, const float *gamma, const float *beta, float eps,
                  float *out);
int tq_gelu_tanh(const float *x, size_t n, float *out);

/* Timed CPU baseline legs (reference loop structure, see the .c file). */
double tq_time_roundtrip_c1(const float *x, size_t n, float *scratch_q, float *scratch_y, int reps);
double tq_time_matmul_rows(const uint8_t *a, const uint8_t *b_kn, size_t m_sample, size_t k, size_t n,
                           int32_t *acc);

#ifdef __cplusplus
}
#endif
#endif
