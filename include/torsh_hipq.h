/*
 * torsh_hipq - C-ABI of the MI355X (gfx950) quantized-inference kernels that
 * sit behind ToRSh's quantization API.
 *
 * Every entry point returns an int32_t status using the numbering of the
 * reference's own C error enum (crates/torsh-core/src/ffi.rs:196-220) and
 * records a thread-local message readable through hipq_get_last_error(), the
 * convention of crates/torsh-ffi/src/c_api/utils.rs:162-190.  Pointers are
 * null-checked first (crates/torsh-ffi/src/c_api/neural.rs:106-113).
 *
 * Unless a parameter is documented as "host", data pointers are DEVICE
 * pointers valid on the context's GPU.  Work is enqueued on the context's HIP
 * stream and is asynchronous; hipq_ctx_synchronize() waits for it.  Inputs are
 * only read, outputs are caller-allocated, nothing is retained across calls
 * (the reference's functions borrow inputs and return fresh outputs,
 * crates/torsh-tensor/src/advanced_ops.rs:624-629).  A context must not be
 * used from two threads at once; distinct contexts are independent.
 *
 * Layouts: matrices are row-major and dense.  Linear weights are [N,K]
 * (output channel major, K contiguous) - the transpose of the [K,N] operand of
 * crates/torsh-backend/src/quantization/specialized.rs:191-193, same integers.
 * Conv tensors are NCHW / [OC,IC,KH,KW].
 */
#ifndef TORSH_HIPQ_H
#define TORSH_HIPQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HIPQ_API __attribute__((visibility("default")))

typedef struct hipq_ctx hipq_ctx;

/* crates/torsh-core/src/ffi.rs:196-220 */
enum {
    HIPQ_SUCCESS = 0,
    HIPQ_INVALID_ARGUMENT = 1,
    HIPQ_SHAPE_ERROR = 2,
    HIPQ_DIMENSION_MISMATCH = 3,
    HIPQ_DEVICE_ERROR = 4,
    HIPQ_ALLOCATION_ERROR = 5,
    HIPQ_SYNCHRONIZATION_ERROR = 6,
    HIPQ_UNKNOWN_ERROR = 7
};

/* `mode` bit field of the quantizing entry points.
 * Rounding: the reference rounds with Rust f32::round, half away from zero
 * (crates/torsh-quantization/src/simd_ops.rs:44); half-to-even is offered as a
 * variant.  Form: multiply by 1/scale (simd_ops.rs:36-46, the len > 64 branch
 * of algorithms.rs:292) or divide by scale (algorithms.rs:302-305, 230-233). */
enum {
    HIPQ_ROUND_HALF_AWAY = 0,
    HIPQ_ROUND_HALF_EVEN = 1,
    HIPQ_FORM_MUL_INV = 0,
    HIPQ_FORM_DIV = 2,
    /* floor(v + 0.5): the reduced-precision rounding of quantize_mobile_optimized
     * (simd_ops.rs:424-431); accepted by hipq_quantize_per_tensor_f32_i8 only. */
    HIPQ_ROUND_FLOOR_HALF_UP = 16,
    /* round(x / scale + zero_point): the zero point enters before the rounding, as in the scalar
     * quantized types QInt8 / QUInt8 (crates/torsh-core/src/dtype/quantized.rs:129-134, 285-290);
     * differs from round(x / scale) + zero_point on ties when the zero point is not 0.  Implies the
     * division form.  Accepted by hipq_quantize_per_tensor_f32_i8 / _u8. */
    HIPQ_FORM_ZP_BEFORE_ROUND = 32,
    /* ((x / scale).round() as i32) + zero_point: the value passes through Rust's `as i32` (NaN -> 0)
     * before the zero point is added, as in torsh-nn's quantize_value_symmetric / _asymmetric
     * (crates/torsh-nn/src/quantization/ops.rs:153-162), so a NaN input gives the code `zero_point`
     * instead of a NaN carrier.  Implies the division form.  Accepted by
     * hipq_quantize_per_tensor_f32_carrier. */
    HIPQ_FORM_INT_CAST = 64
};

/* Quantized integer types, ranges per get_dtype_range
 * (crates/torsh-quantization/src/algorithms.rs:425-433). */
enum { HIPQ_DTYPE_I8 = 0, HIPQ_DTYPE_U8 = 1 };

/* Which reference formula turns (min,max) into (scale, zero_point). */
enum {
    /* calculate_symmetric_quantization_params, algorithms.rs:397-422 */
    HIPQ_PARAMS_SYMMETRIC = 0,
    /* calculate_affine_quantization_params, algorithms.rs:358-394 */
    HIPQ_PARAMS_AFFINE = 1,
    /* torsh-backend from_statistics, symmetric: params.rs:323-340 */
    HIPQ_PARAMS_BACKEND_SYMMETRIC = 2,
    /* torsh-backend from_statistics, asymmetric: params.rs:343-363 */
    HIPQ_PARAMS_BACKEND_ASYMMETRIC = 3,
    /* The range is first widened to contain 0, a zero scale becomes 1:
     * Observer::calculate_qparams (crates/torsh-quantization/src/observers.rs:263-310),
     * quantize_int4_per_tensor / _per_channel and quantize_group_wise
     * (crates/torsh-quantization/src/specialized.rs:39-48, 126-133, 322-335). */
    HIPQ_PARAMS_ZERO_INCLUDED = 4,
    /* per_channel_quantize_weights of torsh-nn (crates/torsh-nn/src/quantization/ops.rs:296-373):
     * symmetric scale = max(|min|,|max|) / 127 with no zero guard (an all-zero channel gets scale 0),
     * asymmetric scale = (max - min) / 255 and zero_point = round(-min / scale), not clamped.  Both
     * always report HIPQ_SUCCESS, as the reference does not validate the range.  Accepted by the
     * per-row / per-group quantizers. */
    HIPQ_PARAMS_NN_SYMMETRIC = 5,
    HIPQ_PARAMS_NN_ASYMMETRIC = 6
};

/* Device-resident quantization parameters, written by the kernels that derive
 * them so that a dynamic quantize never round-trips to the host.  `status` is
 * HIPQ_SUCCESS or HIPQ_INVALID_ARGUMENT (non-finite or inverted range, where
 * the reference returns InvalidArgument, algorithms.rs:363-373,403-407). */
typedef struct hipq_qparams {
    float scale;
    int32_t zero_point;
    float min_val;
    float max_val;
    int32_t status;
    int32_t reserved[3];
} hipq_qparams;

/* ---- library, context, errors ---------------------------------------- */
HIPQ_API const char *hipq_version(void);
/* torsh_get_last_error / torsh_clear_last_error / torsh_has_error,
 * crates/torsh-ffi/src/c_api/utils.rs:162-190. */
HIPQ_API const char *hipq_get_last_error(void);
HIPQ_API void hipq_clear_last_error(void);
HIPQ_API int32_t hipq_has_error(void);

/* Creates a context on `device` with its own non-blocking stream. */
HIPQ_API int32_t hipq_ctx_create(int32_t device, hipq_ctx **out_ctx);
/* Creates a context that enqueues on a caller-owned hipStream_t (0 = the
 * legacy default stream). */
HIPQ_API int32_t hipq_ctx_create_on_stream(int32_t device, void *hip_stream, hipq_ctx **out_ctx);
HIPQ_API int32_t hipq_ctx_destroy(hipq_ctx *ctx);
/* Waits for the context's stream.  Also returns HIPQ_DEVICE_ERROR (once) if a kernel since the last
 * synchronize gave up on one of its bounded waits: its outputs are then invalid. */
HIPQ_API int32_t hipq_ctx_synchronize(hipq_ctx *ctx);
HIPQ_API void *hipq_ctx_stream(hipq_ctx *ctx);

/* Device-buffer helpers for callers whose tensors live on the host (the
 * reference's Tensor has no ROCm device, crates/torsh-core/src/device/types.rs:39-48). */
HIPQ_API int32_t hipq_device_malloc(hipq_ctx *ctx, size_t bytes, void **out_ptr);
HIPQ_API int32_t hipq_device_free(hipq_ctx *ctx, void *ptr);
HIPQ_API int32_t hipq_memcpy_h2d(hipq_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);
HIPQ_API int32_t hipq_memcpy_d2h(hipq_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);

/* ---- range reduction and parameters ---------------------------------- */
/* find_min_max_simd, crates/torsh-quantization/src/simd_ops.rs:84-121.
 * out_minmax: 2 floats {min, max}; NaNs are ignored as f32::min/max do.
 * n == 0 is InvalidArgument as in the reference. */
HIPQ_API int32_t hipq_minmax_f32(hipq_ctx *ctx, const float *x, size_t n, float *out_minmax);
/* max |x| (the symmetric-scheme reduction: max(|min|,|max|), algorithms.rs:410). */
HIPQ_API int32_t hipq_absmax_f32(hipq_ctx *ctx, const float *x, size_t n, float *out_absmax);
/* (min,max) -> (scale, zero_point) on the device; `flavor` is HIPQ_PARAMS_*.
 * qmin/qmax: -128/127 for I8, 0/255 for U8. */
HIPQ_API int32_t hipq_qparams_from_minmax(hipq_ctx *ctx, const float *minmax, int32_t flavor, int32_t qmin,
                                          int32_t qmax, hipq_qparams *out_params);

/* ---- per-tensor quantize / dequantize -------------------------------- */
/* quantize_to_int8_simd / quantize_per_tensor_affine_i8,
 * crates/torsh-quantization/src/simd_ops.rs:196-227, algorithms.rs:245-274:
 * q = clamp(round(x * (1/scale) | x / scale) + zp, -128, 127) as i8.
 * scale <= 0 is InvalidArgument (algorithms.rs:284-288).  Also the arithmetic of
 * quantize_mobile_optimized (simd_ops.rs:390-446; HIPQ_ROUND_FLOOR_HALF_UP is its
 * reduced-precision rounding for more than 256 elements). */
HIPQ_API int32_t hipq_quantize_per_tensor_f32_i8(hipq_ctx *ctx, const float *x, size_t n, float scale,
                                                 int32_t zero_point, int32_t mode, int8_t *out);
/* hipq_quantize_per_tensor_f32_i8 that also records the parameters it was given in a device-side
 * hipq_qparams, for the kernels that read their scale from device memory (hipq_linear_i8_f32,
 * hipq_dequantize_with_params_i8_f32). */
HIPQ_API int32_t hipq_quantize_static_per_tensor_f32_i8(hipq_ctx *ctx, const float *x, size_t n, float scale,
                                                        int32_t zero_point, int32_t mode, int8_t *out,
                                                        hipq_qparams *out_params);
/* CpuQuantizationOps::quantize_f32 for UInt8,
 * crates/torsh-backend/src/quantization/ops.rs:185-195,295-364:
 * q = clamp(round(x / scale) + zp, 0, 255). */
HIPQ_API int32_t hipq_quantize_per_tensor_f32_u8(hipq_ctx *ctx, const float *x, size_t n, float scale,
                                                 int32_t zero_point, int32_t mode, uint8_t *out);
/* quantize_per_tensor_affine_simd, simd_ops.rs:18-49: same arithmetic, result
 * kept in an f32 carrier clamped to [qmin,qmax] (NaN stays NaN), the form
 * torsh-quantization hands back (algorithms.rs:291,304-312). */
HIPQ_API int32_t hipq_quantize_per_tensor_f32_carrier(hipq_ctx *ctx, const float *x, size_t n, float scale,
                                                      int32_t zero_point, int32_t mode, int32_t qmin,
                                                      int32_t qmax, float *out);
/* As hipq_quantize_per_tensor_f32_i8 / _u8 with scale and zero point read from
 * a device hipq_qparams (no host round trip). */
HIPQ_API int32_t hipq_quantize_with_params_f32_i8(hipq_ctx *ctx, const float *x, size_t n,
                                                  const hipq_qparams *params, int32_t mode, int8_t *out);
HIPQ_API int32_t hipq_quantize_with_params_f32_u8(hipq_ctx *ctx, const float *x, size_t n,
                                                  const hipq_qparams *params, int32_t mode, uint8_t *out);
/* quantize_tensor_auto, algorithms.rs:85-123: min/max -> params (`flavor`) ->
 * quantize, all on the device.  dtype is HIPQ_DTYPE_I8 (out is int8_t*) or
 * HIPQ_DTYPE_U8 (out is uint8_t*).  out_params receives the parameters.
 * Up to 65536 * (compute units) elements (16 Mi on MI355X: a 4096 x 4096 tensor), n % 4 == 0, x 16-byte and
 * out 4-byte aligned, mode within HIPQ_FORM_DIV | HIPQ_ROUND_HALF_EVEN: one kernel that keeps the tensor in
 * registers between the range and the codes (up to 64 floats a lane, four workgroups per compute unit), so x
 * is read from memory once; its workgroups agree on the range through device words of the context (see
 * hipq_ctx_set_wait_spin_limit).  Anything else: a range pass, then a quantizer that folds its partials. */
HIPQ_API int32_t hipq_quantize_dynamic_per_tensor_f32(hipq_ctx *ctx, const float *x, size_t n, int32_t flavor,
                                                      int32_t dtype, int32_t mode, void *out,
                                                      hipq_qparams *out_params);
/* dequantize_per_tensor_affine, algorithms.rs:318-355: y = (q - zp) * scale. */
HIPQ_API int32_t hipq_dequantize_i8_f32(hipq_ctx *ctx, const int8_t *q, size_t n, float scale, int32_t zero_point,
                                        float *out);
HIPQ_API int32_t hipq_dequantize_u8_f32(hipq_ctx *ctx, const uint8_t *q, size_t n, float scale,
                                        int32_t zero_point, float *out);
/* The same on the f32 carrier form (simd_ops.rs:52-81). */
HIPQ_API int32_t hipq_dequantize_carrier_f32(hipq_ctx *ctx, const float *q, size_t n, float scale,
                                             int32_t zero_point, float *out);
/* Scale / zero point from a device hipq_qparams. */
HIPQ_API int32_t hipq_dequantize_with_params_i8_f32(hipq_ctx *ctx, const int8_t *q, size_t n,
                                                    const hipq_qparams *params, float *out);

/* ---- per-channel quantize / dequantize ------------------------------- */
/* quantize_per_channel_auto with axis 0 on a [rows, cols] view
 * (algorithms.rs:126-242): per row min/max -> params (`flavor`
 * HIPQ_PARAMS_SYMMETRIC or HIPQ_PARAMS_AFFINE) -> clamp(round(x / s) + zp,
 * qmin, qmax).  Used per output channel for weights and per token for
 * activations.  out_scales[rows], out_zero_points[rows] (may be NULL).
 * out_status: device int32, set non-zero if any row had a non-finite range. */
HIPQ_API int32_t hipq_quantize_per_row_f32_i8(hipq_ctx *ctx, const float *x, size_t rows, size_t cols,
                                              int32_t flavor, int32_t mode, int8_t *out, float *out_scales,
                                              int32_t *out_zero_points, int32_t *out_status);
/* The same for rows that are `ld` elements apart in memory (a column slice of
 * a wider matrix); the int8 output is dense [rows, cols]. */
HIPQ_API int32_t hipq_quantize_per_row_strided_f32_i8(hipq_ctx *ctx, const float *x, size_t rows, size_t cols,
                                                      size_t ld, int32_t flavor, int32_t mode, int8_t *out,
                                                      float *out_scales, int32_t *out_zero_points,
                                                      int32_t *out_status);
/* quantize_per_channel_auto for any axis of a dense tensor viewed as
 * [outer, channels, inner] (algorithms.rs:126-242).  A channel whose range is
 * not finite sets *out_status and keeps what `out` held for it.  From 256 Ki
 * elements on, a channel axis that is not the leading one takes two range keys
 * per channel from the context's scratch memory (grown on first use), so calls
 * on one context must not overlap, as for every entry point that uses it. */
HIPQ_API int32_t hipq_quantize_per_channel_auto_f32_i8(hipq_ctx *ctx, const float *x, size_t outer,
                                                       size_t channels, size_t inner, int32_t flavor,
                                                       int32_t mode, int8_t *out, float *out_scales,
                                                       int32_t *out_zero_points, int32_t *out_status);
/* Generalisation to groups of `group_size` consecutive channels that share
 * one (scale, zero point) - the last group may be shorter - with a caller-chosen
 * integer range [qmin, qmax] inside [-128, 127] (or inside [0, 255]: the codes are then the bytes of `out`
 * read as uint8) and any HIPQ_PARAMS_* flavor:
 * quantize_group_wise (crates/torsh-quantization/src/specialized.rs:241-377) and,
 * with group_size 1 and range -8..7, quantize_int4_per_channel (specialized.rs:68-160).
 * out_scales / out_zero_points hold ceil(channels / group_size) entries.  Values
 * are stored one per int8. */
HIPQ_API int32_t hipq_quantize_per_group_auto_f32_i8(hipq_ctx *ctx, const float *x, size_t outer, size_t channels,
                                                     size_t inner, size_t group_size, int32_t flavor, int32_t qmin,
                                                     int32_t qmax, int32_t mode, int8_t *out, float *out_scales,
                                                     int32_t *out_zero_points, int32_t *out_status);
/* quantize_binary, crates/torsh-quantization/src/specialized.rs:163-188:
 * out = x >= 0 ? 1 : -1 (int8), scale = mean |x| (1 if that is 0), zero point 0.
 * quantize_ternary, specialized.rs:191-238: threshold = 0.7 * max |x|;
 * out = 0 where |x| <= threshold, else sign(x); scale = mean of |x| over the
 * values above the threshold (1 if there are none).  out_params is a device
 * record; min_val / max_val hold the threshold (0 for binary) and max |x|.
 * n == 0 is InvalidArgument as in the reference.  The means are formed from
 * f64 sums (the reference adds f32 terms in element order). */
HIPQ_API int32_t hipq_quantize_binary_f32_i8(hipq_ctx *ctx, const float *x, size_t n, int8_t *out,
                                             hipq_qparams *out_params);
HIPQ_API int32_t hipq_quantize_ternary_f32_i8(hipq_ctx *ctx, const float *x, size_t n, int8_t *out,
                                              hipq_qparams *out_params);
/* quantize_binary_learned_threshold, crates/torsh-quantization/src/specialized.rs:439-492:
 * threshold = the given one (has_threshold != 0) or mean |x|; out = 0 where |x| <= threshold,
 * else x >= 0 ? 1 : -1; scale = mean of |x| over the values above the threshold (1 if none).
 * quantize_ternary_adaptive, specialized.rs:495-552: of the ten thresholds max|x| * (i * 0.1),
 * i = 1..10, the first with the smallest mean squared error of the unit ternary code
 * (specialized.rs:555-570); out and scale as quantize_ternary with that threshold.
 * out_params: scale, zero point 0, min_val = the threshold used, max_val = max |x| (adaptive)
 * or 0.  n == 0 is InvalidArgument.  Means and errors are formed from f64 sums. */
HIPQ_API int32_t hipq_quantize_binary_learned_threshold_f32_i8(hipq_ctx *ctx, const float *x, size_t n,
                                                               int32_t has_threshold, float threshold, int8_t *out,
                                                               hipq_qparams *out_params);
HIPQ_API int32_t hipq_quantize_ternary_adaptive_f32_i8(hipq_ctx *ctx, const float *x, size_t n, int8_t *out,
                                                       hipq_qparams *out_params);
/* quantize_per_channel_affine, explicit parameters,
 * crates/torsh-quantization/src/quantize.rs:287-331 (HIPQ_FORM_DIV) and
 * quantize_per_channel_simd, simd_ops.rs:124-169 (HIPQ_FORM_MUL_INV, inner
 * contiguous). */
HIPQ_API int32_t hipq_quantize_per_channel_f32_i8(hipq_ctx *ctx, const float *x, size_t outer, size_t channels,
                                                  size_t inner, const float *scales,
                                                  const int32_t *zero_points, int32_t mode, int8_t *out);
/* dequantize_per_channel_affine, crates/torsh-quantization/src/dequantize.rs:46-89:
 * y = scale[c] * (q - zp[c]). */
HIPQ_API int32_t hipq_dequantize_per_channel_i8_f32(hipq_ctx *ctx, const int8_t *q, size_t outer,
                                                    size_t channels, size_t inner, const float *scales,
                                                    const int32_t *zero_points, float *out);

/* ---- integer GEMM and the quantized Linear forward ------------------- */
/* vnni_matmul_kernel, crates/torsh-backend/src/quantization/specialized.rs:175-201:
 * acc[m,n] = sum_k a[m,k] * w[n,k] in int32 (raw accumulators, no clamp). */
HIPQ_API int32_t hipq_gemm_i8_i32(hipq_ctx *ctx, const int8_t *a, const int8_t *w, size_t m, size_t n, size_t k,
                                  int32_t *out);
/* Quantized Linear with dequantizing epilogue:
 *   out[m,n] = (acc as f32) * (s_a * s_w[n]) + bias[n]
 * (acc*(s_in*s_w): crates/torsh-backend/src/quantization/operations.rs:669,722;
 * f32 bias add: crates/torsh-backend/src/quantization/ops.rs:561).
 * a_scale: device, 1 float (per tensor) or m floats (per token) as
 * a_scale_per_row says; w_scales: device [n]; bias: device [n] or NULL. */
HIPQ_API int32_t hipq_linear_i8_f32(hipq_ctx *ctx, const int8_t *a, const float *a_scale,
                                    int32_t a_scale_per_row, const int8_t *w, const float *w_scales,
                                    const float *bias, size_t m, size_t n, size_t k, float *out);
/* hipq_linear_i8_f32 with a residual added after the bias:
 * out = acc * (s_a * s_w[n]) + bias[n] + residual[m,n]; out may alias residual
 * (Linear followed by the `.add()` of a skip connection). */
HIPQ_API int32_t hipq_linear_i8_f32_residual(hipq_ctx *ctx, const int8_t *a, const float *a_scale,
                                             int32_t a_scale_per_row, const int8_t *w, const float *w_scales,
                                             const float *bias, const float *residual, size_t m, size_t n, size_t k,
                                             float *out);
/* Same accumulators, requantizing epilogue (tail of operations.rs:716-724 with
 * a supplied output scale): q = clamp(round(v / s_out) + zp_out, -128, 127). */
HIPQ_API int32_t hipq_linear_i8_i8(hipq_ctx *ctx, const int8_t *a, const float *a_scale, int32_t a_scale_per_row,
                                   const int8_t *w, const float *w_scales, const float *bias, size_t m, size_t n,
                                   size_t k, float out_scale, int32_t out_zero_point, int32_t mode,
                                   int8_t *out);
/* Stand-alone requantize of int32 accumulators [rows, cols]; the weight
 * channel is the column. */
HIPQ_API int32_t hipq_requantize_i32_i8(hipq_ctx *ctx, const int32_t *acc, size_t rows, size_t cols,
                                        const float *a_scale, int32_t a_scale_per_row, const float *w_scales,
                                        const float *bias, float out_scale, int32_t out_zero_point,
                                        int32_t mode, int8_t *out);
/* No counterpart in the reference.  The one-launch dynamic quantizers need their whole grid resident on the device
 * at once and size it for the device being theirs: up to half of it (four light workgroups per compute unit) for
 * tensors of up to 4 Mi elements, all of its register files above that.  When `contexts` contexts launch such
 * work concurrently (one per serving thread, say), tell each of them so: it then sizes those grids for 1 / contexts
 * of the device and takes the two-launch path for what does not fit, instead of two half-resident grids waiting
 * for each other until their bounded waits give up.  Default 1; 1..64. */
HIPQ_API int32_t hipq_ctx_set_resident_share(hipq_ctx *ctx, int32_t contexts);
/* Whole forward of a quantized Linear with a static (calibrated) activation scale: the scale an
 * observer derived beforehand (Observer::calculate_qparams, crates/torsh-quantization/src/observers.rs:263-310,
 * symmetric: zero point 0) instead of a range pass over every input - per-tensor quantize
 * (algorithms.rs:277-315), int8 GEMM, dequantizing epilogue.  `mode` as hipq_quantize_per_tensor_f32_i8. */
HIPQ_API int32_t hipq_linear_static_f32(hipq_ctx *ctx, const float *x, float a_scale, const int8_t *w,
                                        const float *w_scales, const float *bias, size_t m, size_t n, size_t k,
                                        int32_t mode, float *out);
/* Whole forward of a quantized Linear on fp32 activations: dynamic activation
 * quantization (per tensor: algorithms.rs:85-123; per token: algorithms.rs:126-242
 * on axis 0), int8 GEMM, dequantizing epilogue.  Uses context-owned scratch
 * for the int8 activations and their scales.  Activations whose range is not finite (NaN / Inf
 * present; the reference returns InvalidArgument, algorithms.rs:403-407) cannot fail an asynchronous
 * call: the outputs that depend on them are NaN (the whole output per tensor, the row per token). */
HIPQ_API int32_t hipq_linear_dynamic_f32(hipq_ctx *ctx, const float *x, int32_t per_token, const int8_t *w,
                                         const float *w_scales, const float *bias, size_t m, size_t n, size_t k,
                                         int32_t mode, float *out);
/* hipq_linear_dynamic_f32 for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * arguments, same kernels, same results; the int8 activations, their scales and the range
 * partials go to a static device array of the library (about 4.3 MiB per GPU, held until the
 * process ends) instead of the context's growable scratch, and the call performs no hipMalloc /
 * hipFree.  Limits: m <= 16384 rows and m * k <= 4 Mi elements, else HIPQ_SHAPE_ERROR.  Every call
 * on one GPU shares that GPU's array: calls that overlap in time on one GPU (two streams, two
 * contexts) race; calls on one stream are ordered and safe. */
HIPQ_API int32_t hipq_linear_dynamic_f32_noalloc(hipq_ctx *ctx, const float *x, int32_t per_token, const int8_t *w,
                                                 const float *w_scales, const float *bias, size_t m, size_t n,
                                                 size_t k, int32_t mode, float *out);


/* ---- fragment-packed operands: the fast Linear forward ------------------ */
/* The int8 GEMM reads its operands fastest in the order the matrix cores consume them.  A packed
 * int8 matrix [rows, k] is [rows/32][k/32][1 KiB]: inside a 1 KiB fragment, 16-byte slot l holds
 * row 32*rb + l%32, bytes 32*kb + 16*(l/32) .. +15 (one operand of v_mfma_i32_32x32x32_i8).  Rows are
 * padded to a multiple of 32, the k blocks of a row block to a multiple of 4; padding along k is
 * zero.  This is the "tile order" of a prepared weight blob: weights are packed once when a layer
 * is converted (where QuantizedLinear::from_linear transposes Linear's [in,out] weight,
 * crates/torsh-nn/src/layers/linear.rs:28-31), activations are written packed by the quantize pass.
 * Same integers as the row-major form, so every result below is bit-identical to the row-major
 * entry point named beside it.  Packed buffers are device memory, 16-byte aligned, below 2 GiB. */
/* Bytes of the packed form of an int8 [rows, k] matrix (host call, no device work). */
HIPQ_API int32_t hipq_packed_size(size_t rows, size_t k, size_t *out_bytes);
/* Row-major int8 [rows, k] -> packed (weight preparation; also for callers that hold int8 activations). */
HIPQ_API int32_t hipq_pack_rows_i8(hipq_ctx *ctx, const int8_t *src, size_t rows, size_t k, int8_t *dst_packed);
/* hipq_gemm_i8_i32 on packed operands: vnni_matmul_kernel,
 * crates/torsh-backend/src/quantization/specialized.rs:175-201.  out is row-major [m, n]. */
HIPQ_API int32_t hipq_gemm_packed_i8_i32(hipq_ctx *ctx, const int8_t *a_packed, const int8_t *w_packed, size_t m,
                                         size_t n, size_t k, int32_t *out);
/* hipq_linear_i8_f32 on packed operands (acc * (s_a * s_w[n]) + bias[n]:
 * crates/torsh-backend/src/quantization/operations.rs:669,722 and ops.rs:561). */
HIPQ_API int32_t hipq_linear_packed_i8_f32(hipq_ctx *ctx, const int8_t *a_packed, const float *a_scale,
                                           int32_t a_scale_per_row, const int8_t *w_packed, const float *w_scales,
                                           const float *bias, size_t m, size_t n, size_t k, float *out);
/* hipq_linear_i8_i8 on packed operands (requantizing epilogue, operations.rs:722-728). */
HIPQ_API int32_t hipq_linear_packed_i8_i8(hipq_ctx *ctx, const int8_t *a_packed, const float *a_scale,
                                          int32_t a_scale_per_row, const int8_t *w_packed, const float *w_scales,
                                          const float *bias, size_t m, size_t n, size_t k, float out_scale,
                                          int32_t out_zero_point, int32_t mode, int8_t *out);
/* Symmetric per-tensor int8 quantize of fp32 [rows, cols] into the packed layout: with `dynamic` the
 * scale comes from the tensor's own range (quantize_tensor_auto, crates/torsh-quantization/src/algorithms.rs:85-123),
 * otherwise `scale` is used (quantize_per_tensor_affine, algorithms.rs:277-315).  Codes are those of
 * hipq_quantize_dynamic_per_tensor_f32 / hipq_quantize_per_tensor_f32_i8; a range that is not finite
 * gives status HIPQ_INVALID_ARGUMENT in out_params, a NaN scale and zero codes.
 * A dynamic call on up to 65536 * (compute units) elements (16 Mi on MI355X), cols % 16 == 0, x 16-byte aligned, is
 * one kernel: every wave holds its one or four fragments of 16 x 64 floats in registers while the workgroups agree on the range
 * through device words of the context (see hipq_ctx_set_wait_spin_limit), so x is read once.  It keeps no
 * host state per launch and can be captured and replayed.  Two such calls on one context must not overlap
 * (they cannot: a context has one stream). */
HIPQ_API int32_t hipq_quantize_per_tensor_packed_f32_i8(hipq_ctx *ctx, const float *x, size_t rows, size_t cols,
                                                        int32_t dynamic, float scale, int32_t mode,
                                                        int8_t *out_packed, hipq_qparams *out_params);
/* Symmetric per-row (per-token) int8 quantize of fp32 [rows, cols] into the packed layout: each row's range, scale
 * and codes in one pass (quantize_per_channel_auto over axis 0, algorithms.rs:126-242; the codes and scales of
 * hipq_quantize_per_row_f32_i8 with HIPQ_PARAMS_SYMMETRIC).  out_scales: rows floats.  A row whose range is
 * not finite gets a NaN scale and zero codes. */
HIPQ_API int32_t hipq_quantize_per_row_packed_f32_i8(hipq_ctx *ctx, const float *x, size_t rows, size_t cols,
                                                     int32_t mode, int8_t *out_packed, float *out_scales);
/* hipq_linear_dynamic_f32 with prepared (packed) weights: per tensor the dynamic quantizer of
 * hipq_quantize_per_tensor_packed_f32_i8 (one launch where its conditions hold, else a range pass and a quantizer)
 * and the packed GEMM with the dequantizing epilogue; per token the per-row quantizer (one pass) and the GEMM. */
HIPQ_API int32_t hipq_linear_dynamic_packed_f32(hipq_ctx *ctx, const float *x, int32_t per_token,
                                                const int8_t *w_packed, const float *w_scales, const float *bias,
                                                size_t m, size_t n, size_t k, int32_t mode, float *out);
/* hipq_linear_static_f32 with prepared (packed) weights. */
HIPQ_API int32_t hipq_linear_static_packed_f32(hipq_ctx *ctx, const float *x, float a_scale, const int8_t *w_packed,
                                               const float *w_scales, const float *bias, size_t m, size_t n,
                                               size_t k, int32_t mode, float *out);

/* ---- quantized Conv2d forward (NCHW, filters [OC,IC,KH,KW]) ------------ */
/* Integer part of perform_quantized_convolution,
 * crates/torsh-backend/src/quantization/operations.rs:637-713:
 *   acc[n,oc,oh,ow] = sum over kh,kw,ic of (x_q - zp_in) * w_q   (int32)
 * with padded taps contributing nothing (the real value 0), output size
 * (H + 2p - k)/s + 1 (crates/torsh-backend/src/quantization/ops.rs:513-514). */
HIPQ_API int32_t hipq_conv2d_u8i8_i32(hipq_ctx *ctx, const uint8_t *x, int32_t zp_in, const int8_t *w, size_t nb,
                                      size_t c, size_t h, size_t wd, size_t oc, size_t kh, size_t kw, size_t stride_h,
                                      size_t stride_w, size_t pad_h, size_t pad_w, int32_t *out);
/* The same accumulators followed by the fused bias + requantize tail
 * (operations.rs:716-724 with a supplied output scale):
 *   v = acc * (s_in * s_w[oc]) + bias[oc];  q = clamp(round(v / s_out) + zp_out, -128, 127).
 * s_in and s_out are host scalars; w_scales [oc] and bias [oc] (may be NULL) are device. */
HIPQ_API int32_t hipq_conv2d_u8i8_i8(hipq_ctx *ctx, const uint8_t *x, int32_t zp_in, float s_in, const int8_t *w,
                                     const float *w_scales, const float *bias, size_t nb, size_t c, size_t h, size_t wd,
                                     size_t oc, size_t kh, size_t kw, size_t stride_h, size_t stride_w, size_t pad_h,
                                     size_t pad_w, float out_scale, int32_t out_zero_point, int32_t mode, int8_t *out);
/* Convolution with the dequantize-with-bias epilogue: out[n,oc,oh,ow] = acc * (s_in * w_scales[oc]) + bias[oc], fp32
 * NCHW.  This is the fp32 result the reference forms before it derives output parameters from its range
 * (crates/torsh-backend/src/quantization/ops.rs:479-580; integer accumulation as in
 * crates/torsh-quantization/src/operations.rs:672-713 with zero-contribution padding). */
HIPQ_API int32_t hipq_conv2d_u8i8_f32(hipq_ctx *ctx, const uint8_t *x, int32_t zp_in, float s_in, const int8_t *w,
                                      const float *w_scales, const float *bias, size_t nb, size_t c, size_t h, size_t wd,
                                      size_t oc, size_t kh, size_t kw, size_t stride_h, size_t stride_w, size_t pad_h,
                                      size_t pad_w, float *out);
/* One-time filter preparation for the stride-1 fast path (offline weight preparation; no reference
 * counterpart, the reference keeps filters as stored): int8 [OC,IC,KH,KW] -> the packed row operand of the
 * matrix-core GEMM with K ordered (tap, channel), and the per-filter sums w_sums[oc].  `packed` is device
 * memory of hipq_conv2d_packed_weights_size bytes (>= OC*IC*KH*KW: rows are padded to 32, K to 128),
 * 16-byte aligned. */
HIPQ_API int32_t hipq_conv2d_packed_weights_size(size_t oc, size_t ic, size_t kh, size_t kw, size_t *out_bytes);
HIPQ_API int32_t hipq_conv2d_pack_weights_i8(hipq_ctx *ctx, const int8_t *w, size_t oc, size_t ic, size_t kh, size_t kw,
                                             int8_t *packed, int32_t *w_sums);
/* hipq_conv2d_u8i8_i8 on prepared filters (stride 1, channels a multiple of 32). */
HIPQ_API int32_t hipq_conv2d_u8i8_i8_packed(hipq_ctx *ctx, const uint8_t *x, int32_t zp_in, float s_in,
                                            const int8_t *w_packed, const int32_t *w_sums, const float *w_scales,
                                            const float *bias, size_t nb, size_t c, size_t h, size_t wd, size_t oc,
                                            size_t kh, size_t kw, size_t pad_h, size_t pad_w, float out_scale,
                                            int32_t out_zero_point, int32_t mode, int8_t *out);
/* The whole quantized Conv2d forward from fp32 activations, on the device: x [nb, c, h, w] fp32 is quantized per
 * tensor to uint8 with parameters from its own range (`flavor`, e.g. HIPQ_PARAMS_BACKEND_ASYMMETRIC as
 * QuantizationParams::from_statistics derives them, crates/torsh-backend/src/quantization/params.rs; quant_mode:
 * HIPQ_FORM_DIV / HIPQ_ROUND_HALF_EVEN bits of that quantize) and convolved as by hipq_conv2d_u8i8_i8_packed -
 * the codes, the parameters and the outputs are those of hipq_quantize_dynamic_per_tensor_f32 followed by
 * hipq_conv2d_u8i8_i8_packed, without the uint8 copy of the input and without reading the parameters back to the
 * host.  in_params (device) receives the input parameters; a range that is not finite leaves status
 * HIPQ_INVALID_ARGUMENT and a NaN scale there and outputs that carry no information.  Inputs whose image-layout
 * pass fits the device at once (the usual case) are quantized inside that pass, in one launch. */
HIPQ_API int32_t hipq_conv2d_dynamic_f32_i8_packed(hipq_ctx *ctx, const float *x, int32_t flavor, int32_t quant_mode,
                                                   const int8_t *w_packed, const int32_t *w_sums,
                                                   const float *w_scales, const float *bias, size_t nb, size_t c,
                                                   size_t h, size_t wd, size_t oc, size_t kh, size_t kw, size_t pad_h,
                                                   size_t pad_w, float out_scale, int32_t out_zero_point, int32_t mode,
                                                   int8_t *out, hipq_qparams *in_params);

/* ---- fp32 helpers of the int8 transformer stack ------------------------- */
/* LayerNorm over the last dimension (biased variance, eps inside the square
 * root, eps 1e-5 by default: crates/torsh-nn/src/layers/normalization/layer_group/mod.rs:130-166,660).
 * gamma / beta [cols] may be NULL.  cols % 4 == 0, cols <= 12288 (a row is held in registers). */
HIPQ_API int32_t hipq_layer_norm_f32(hipq_ctx *ctx, const float *x, size_t rows, size_t cols, const float *gamma,
                                     const float *beta, float eps, float *out);
/* LayerNorm followed by the per-token symmetric int8 quantizer
 * (quantize_per_channel_auto on axis 0, algorithms.rs:126-242) in one pass. */
HIPQ_API int32_t hipq_layer_norm_quantize_f32_i8(hipq_ctx *ctx, const float *x, size_t rows, size_t cols,
                                                 const float *gamma, const float *beta, float eps, int32_t mode,
                                                 int8_t *out, float *out_scales);
/* The skip connection and the LayerNorm + quantizer that follow it in one pass: x[r, :] += delta[r, :]
 * (Tensor::add, one rounding per element, written back over x), then the new row goes through
 * hipq_layer_norm_quantize_f32_i8.  Same results as hipq_add_f32 followed by that call. */
HIPQ_API int32_t hipq_add_layer_norm_quantize_f32_i8(hipq_ctx *ctx, float *x, const float *delta, size_t rows,
                                                     size_t cols, const float *gamma, const float *beta, float eps,
                                                     int32_t mode, int8_t *out, float *out_scales);
/* tanh-form GELU, crates/torsh-nn/src/layers/activation/modern.rs:124-136. */
HIPQ_API int32_t hipq_gelu_tanh_f32(hipq_ctx *ctx, const float *x, size_t n, float *out);
/* GELU followed by the per-token symmetric int8 quantizer in one pass. */
HIPQ_API int32_t hipq_gelu_tanh_quantize_f32_i8(hipq_ctx *ctx, const float *x, size_t rows, size_t cols, int32_t mode,
                                                int8_t *out, float *out_scales);
/* out = a + b (skip connection; Tensor::add). */
HIPQ_API int32_t hipq_add_f32(hipq_ctx *ctx, const float *a, const float *b, size_t n, float *out);

/* ---- Linear forward with the row operation that follows it in one kernel ---- */
/* In a transformer block every int8 product feeds an operation over whole rows (a per-token quantizer, a
 * LayerNorm).  These forms give a workgroup 32 whole rows of the output (all n columns, the accumulators in
 * registers), so that operation runs on the accumulators and the fp32 product never goes to memory.  Operands
 * are packed (above); n % 32 == 0 and n <= 3072 (outputs that are packed int8: n % 128 == 0); m, k any.
 * Results are those of the separate calls named with each: the same f32 operations per element in the same
 * order.  Only a LayerNorm's row sums are folded in another order, which moves its mean and variance in their
 * last bits (tests bound the effect: codes differ by at most one step where a value sits on a rounding edge). */
/* hipq_linear_packed_i8_f32 (operations.rs:669,722; ops.rs:561): same bits, fp32 row-major [m, n]. */
HIPQ_API int32_t hipq_linear_rows_packed_i8_f32(hipq_ctx *ctx, const int8_t *a_packed, const float *a_scale,
                                                int32_t a_scale_per_row, const int8_t *w_packed,
                                                const float *w_scales, const float *bias, size_t m, size_t n,
                                                size_t k, float *out);
/* hipq_linear_packed_i8_f32, then hipq_gelu_tanh_quantize_f32_i8 (GELU: modern.rs:124-136; per-token
 * quantizer: quantize_per_channel_auto on axis 0, algorithms.rs:126-242), the codes written as the packed
 * operand [m, n] of the next product: same bits as those two calls and hipq_pack_rows_i8. */
HIPQ_API int32_t hipq_linear_gelu_quantize_packed_i8(hipq_ctx *ctx, const int8_t *a_packed, const float *a_scale,
                                                     int32_t a_scale_per_row, const int8_t *w_packed,
                                                     const float *w_scales, const float *bias, size_t m, size_t n,
                                                     size_t k, int32_t mode, int8_t *out_packed, float *out_scales);
/* x[m, n] += the product (hipq_linear_i8_f32_residual: Tensor::add on the Linear's output), then, when
 * out_packed is not NULL, LayerNorm of the new rows (layer_group/mod.rs:130-166) and the per-token quantizer,
 * packed: hipq_add_layer_norm_quantize_f32_i8 and hipq_pack_rows_i8 on the same operands.  x is bit-identical
 * to the separate calls'.  gamma / beta [n] may be NULL. */
HIPQ_API int32_t hipq_linear_residual_layer_norm_quantize_packed_i8(
    hipq_ctx *ctx, const int8_t *a_packed, const float *a_scale, int32_t a_scale_per_row, const int8_t *w_packed,
    const float *w_scales, const float *bias, size_t m, size_t n, size_t k, float *x, const float *gamma,
    const float *beta, float eps, int32_t mode, int8_t *out_packed, float *out_scales);
/* The same forward from fp32 activations a [m, k] (rows lda floats apart, 16-byte aligned, k and lda multiples of
 * 4): every workgroup first quantizes its own 32 rows per token, symmetric int8 (quantize_per_channel_auto on axis
 * 0, algorithms.rs:126-242: hipq_quantize_per_row_packed_f32_i8 with HIPQ_PARAMS_SYMMETRIC; `mode` rounds these
 * codes and the output's alike) and keeps the codes on chip, so the quantizer's launch and its packed output are
 * gone.  Same bits as hipq_quantize_per_row_packed_f32_i8 (on the rows, dense) followed by the entry point above.
 * k <= 1536 and n <= 1536 (the panel of codes and the accumulators of a workgroup), n % 32 == 0 (% 128 with
 * out_packed); other shapes: HIPQ_SHAPE_ERROR, use the two calls. */
HIPQ_API int32_t hipq_linear_from_f32_residual_layer_norm_quantize_packed_i8(
    hipq_ctx *ctx, const float *a, size_t lda, const int8_t *w_packed, const float *w_scales, const float *bias,
    size_t m, size_t n, size_t k, float *x, const float *gamma, const float *beta, float eps, int32_t mode,
    int8_t *out_packed, float *out_scales);

/* ---- quantized elementwise operators of the backend trait --------------- */
/* CpuQuantizationOps::qadd, crates/torsh-backend/src/quantization/ops.rs:582-606:
 * out = quantize(dequantize(a) + dequantize(b)) with output parameters derived
 * from the range of the f32 sum by from_statistics (params.rs:282-363; `flavor`
 * = HIPQ_PARAMS_BACKEND_SYMMETRIC or _ASYMMETRIC for the scheme of `a`).
 * Operands are per-tensor quantized bytes; *_signed says the bytes are
 * two's-complement int8 (tensor.rs:103-143).  out_dtype: HIPQ_DTYPE_I8 / _U8
 * (the dtype of `a` in the reference).  out_params is a device record holding
 * the derived scale, zero point and range.  The f32 intermediate is never
 * stored: 5 bytes of traffic per element. */
HIPQ_API int32_t hipq_qadd_u8(hipq_ctx *ctx, const uint8_t *a, int32_t a_signed, float a_scale, int32_t a_zero_point,
                              const uint8_t *b, int32_t b_signed, float b_scale, int32_t b_zero_point, size_t n,
                              int32_t flavor, int32_t out_dtype, uint8_t *out, hipq_qparams *out_params);
/* CpuQuantizationOps::qrelu, ops.rs:608-624: out = quantize(max(dequantize(q), 0))
 * with parameters from_statistics(0, max(max_val, 0)).  3 bytes per element. */
HIPQ_API int32_t hipq_qrelu_u8(hipq_ctx *ctx, const uint8_t *q, int32_t is_signed, float scale, int32_t zero_point,
                               size_t n, int32_t flavor, int32_t out_dtype, uint8_t *out, hipq_qparams *out_params);

/* ---- calibration observers and quality metrics ------------------------ */
/* Extra `mode` bit of the fake-quantizing entry points: the clamped value goes
 * through `as i32` before it is dequantized (NaN becomes 0), as
 * ModelQuantizer::quantize_value does (crates/torsh-models/src/quantization.rs:336-342);
 * without it the value stays in its f32 carrier and a NaN stays a NaN
 * (crates/torsh-quantization/src/simd_ops.rs:36-46). */
enum { HIPQ_FAKE_INT_CAST = 4 };
/* Or (not both): the clamp is `.max(qmin).min(qmax)`, under which a NaN becomes qmin, and the
 * value is dequantized as scale * (q - zp): fake_quantize_per_tensor_affine,
 * crates/torsh-quantization/src/fake_quantize.rs:14-42 (use with HIPQ_FORM_DIV). */
enum { HIPQ_FAKE_NAN_TO_QMIN = 8 };

/* QuantizationMetrics, crates/torsh-quantization/src/metrics.rs:30-48 (same
 * fields, same order). */
typedef struct hipq_quant_metrics {
    float mse;
    float psnr;
    float snr;
    float mae;
    float max_error;
    float zero_error_percentage;
    float cosine_similarity;
    float compression_ratio;
} hipq_quant_metrics;

/* calculate_quantization_metrics, crates/torsh-quantization/src/metrics.rs:67-175,
 * over two f32 tensors of n elements in one pass; out_metrics is a device
 * record.  n == 0 yields QuantizationMetrics::default() (metrics.rs:50-63).
 * The sums are carried in f64 (the reference adds f32 terms in element
 * order); max_error and the zero-error count are exact. */
HIPQ_API int32_t hipq_quantization_metrics_f32(hipq_ctx *ctx, const float *original, const float *quantized, size_t n,
                                               uint32_t original_bits, uint32_t quantized_bits,
                                               hipq_quant_metrics *out_metrics);
/* The quantize -> dequantize -> metrics sequence of compare_quantization_configs
 * (metrics.rs:178-240) and of ModelQuantizer::calculate_quantization_stats
 * (crates/torsh-models/src/quantization.rs:504-533) fused into one pass over x:
 * the dequantized image is formed in registers and never written.  Quantizer:
 * q = clamp(round(x * (1/scale) | x / scale) + zp, qmin, qmax), y = (q - zp) * scale;
 * `mode` = HIPQ_ROUND_* | HIPQ_FORM_* | HIPQ_FAKE_INT_CAST or HIPQ_FAKE_NAN_TO_QMIN.  `params` (device,
 * may be NULL) overrides scale and zero_point. */
HIPQ_API int32_t hipq_fake_quantize_metrics_f32(hipq_ctx *ctx, const float *x, size_t n, float scale,
                                                int32_t zero_point, const hipq_qparams *params, int32_t qmin,
                                                int32_t qmax, int32_t mode, uint32_t original_bits,
                                                uint32_t quantized_bits, hipq_quant_metrics *out_metrics);
/* ModelQuantizer::quantize_tensor, crates/torsh-models/src/quantization.rs:309-332:
 * out = dequantize(quantize(x)) as f32 ("fake quantization"); same quantizer
 * and `mode` as above. */
HIPQ_API int32_t hipq_fake_quantize_f32(hipq_ctx *ctx, const float *x, size_t n, float scale, int32_t zero_point,
                                        const hipq_qparams *params, int32_t qmin, int32_t qmax, int32_t mode,
                                        float *out);

/* TensorStats, crates/torsh-quantization/src/simd_ops.rs:264-272 (same fields, same order). */
typedef struct hipq_tensor_stats {
    float min_val;
    float max_val;
    float mean;
    float std_dev;
    float variance;
} hipq_tensor_stats;
/* calculate_tensor_stats_simd, simd_ops.rs:230-262 (one_pass == 0: range, f64 mean, then the f64
 * sum of squared deviations from it in a second pass over x; population variance), or
 * calculate_tensor_stats_cache_optimized, algorithms.rs:525-578 (one_pass != 0: f64 sums of x and
 * x^2, mean rounded to f32, variance = E[x^2] - mean^2 rounded to f32, std_dev = its f32 square
 * root).  out_stats is a device record.  n == 0 is InvalidArgument as in both. */
HIPQ_API int32_t hipq_tensor_stats_f32(hipq_ctx *ctx, const float *x, size_t n, int32_t one_pass,
                                       hipq_tensor_stats *out_stats);

/* What Observer::update derives from one batch before it touches its state
 * (crates/torsh-quantization/src/observers.rs:122-150): the batch range (NaN
 * ignoring f32::min/max folds from +inf/-inf) and how many values are NaN or
 * infinite (the reference rejects the batch when this is not 0). */
typedef struct hipq_observe_stats {
    float min_val;
    float max_val;
    uint64_t nonfinite;
} hipq_observe_stats;
HIPQ_API int32_t hipq_observe_f32(hipq_ctx *ctx, const float *x, size_t n, hipq_observe_stats *out_stats);

/* Histogram update of the Histogram observer (observers.rs:186-225) with the
 * bin rule of Observer::value_to_bin_index (observers.rs:313-333) over the
 * range [range_min, range_max]: counts[bin] += occurrences, counts is a device
 * array of num_bins uint64 that the caller zeroes once and keeps across
 * batches.  Exact integer counts. */
#define HIPQ_HISTOGRAM_MAX_BINS 16384
HIPQ_API int32_t hipq_histogram_f32(hipq_ctx *ctx, const float *x, size_t n, float range_min, float range_max,
                                    size_t num_bins, uint64_t *counts);

/* Device pointers of one block of the projection stack: every Linear is
 * per-output-channel int8 ([out,in] weights, [out] scales, [out] fp32 bias). */
typedef struct hipq_block_weights {
    const float *ln1_gamma, *ln1_beta, *ln2_gamma, *ln2_beta;
    const int8_t *w_qkv;
    const float *s_qkv, *b_qkv; /* [3d, d] */
    const int8_t *w_out;
    const float *s_out, *b_out; /* [d, d] */
    const int8_t *w_fc1;
    const float *s_fc1, *b_fc1; /* [d_ff, d] */
    const int8_t *w_fc2;
    const float *s_fc2, *b_fc2; /* [d, d_ff] */
} hipq_block_weights;
/* Bytes of device workspace hipq_transformer_stack_forward_f32 needs. */
HIPQ_API size_t hipq_transformer_stack_workspace_bytes(size_t tokens, size_t d_model, size_t d_ff);
/* Forward of n_layers blocks on x [tokens, d_model] in place: per block
 *   x += Linear_out(quant(V(Linear_qkv(quant(LN1(x))))));  x += Linear_fc2(quant(GELU(Linear_fc1(quant(LN2(x))))))
 * with per-token dynamic int8 activations, LayerNorm and GELU in fp32, and the
 * attention mixing replaced by a pass-through of the value slice (it is not part
 * of the quantized path).  `blocks` is a HOST array of n_layers records. */
HIPQ_API int32_t hipq_transformer_stack_forward_f32(hipq_ctx *ctx, const hipq_block_weights *blocks, size_t n_layers,
                                                    size_t tokens, size_t d_model, size_t d_ff, float eps,
                                                    int32_t mode, float *x, void *workspace, size_t workspace_bytes);
/* The same forward on PREPARED weights: every w_* of `blocks` points to the packed form of the [out, in] matrix
 * (hipq_pack_rows_i8, once, when the model is converted).  Four kernels per layer: each Linear that feeds a row
 * operation applies it in its epilogue (hipq_linear_residual_layer_norm_quantize_packed_i8,
 * hipq_linear_gelu_quantize_packed_i8), the out-projection quantizes the fp32 value slice itself
 * (hipq_linear_from_f32_residual_layer_norm_quantize_packed_i8), and int8 activations stay packed between them.  x is what
 * hipq_transformer_stack_forward_f32 computes up to the fold order of the LayerNorm sums (see those entry
 * points).  d_model and d_ff: multiples of 128, at most 3072 (else HIPQ_SHAPE_ERROR: use the form above). */
HIPQ_API size_t hipq_transformer_stack_prepared_workspace_bytes(size_t tokens, size_t d_model, size_t d_ff);
HIPQ_API int32_t hipq_transformer_stack_forward_prepared_f32(hipq_ctx *ctx, const hipq_block_weights *blocks,
                                                             size_t n_layers, size_t tokens, size_t d_model,
                                                             size_t d_ff, float eps, int32_t mode, float *x,
                                                             void *workspace, size_t workspace_bytes);

#ifdef __cplusplus
}
#endif
#endif /* TORSH_HIPQ_H */
