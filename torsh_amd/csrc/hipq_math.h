// Device-side scalar arithmetic of the quantized path.  Each helper states the
// Rust semantics it reproduces; the translation units are compiled with
// -ffp-contract=off so no multiply-add is fused and every f32 operation rounds
// exactly as the reference's CPU code does.
#pragma once

#include <hip/hip_runtime.h>

#include <cfloat>
#include <cstdint>

#include "torsh_hipq.h"

namespace hipq {

constexpr int kWave = 64;

// Streaming (non-temporal) 16-byte and 4-byte accesses for data touched once.  Measured on
// MI355X over 16 Mi elements: quantize (64 MiB read, 16 MiB written) 19.8 us with ordinary
// accesses, 17.6 us with both streams non-temporal; dequantize (16 MiB read, 64 MiB written)
// 19.3 us ordinary, 13.4 us with ordinary loads and non-temporal stores (non-temporal loads
// of the small side cost 4 us there, so dequantize keeps ordinary loads).
typedef float hipq_vf4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 load_stream(const float4 *p) {
    const hipq_vf4 t = __builtin_nontemporal_load(reinterpret_cast<const hipq_vf4 *>(p));
    return make_float4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ uint32_t load_stream(const uint32_t *p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void store_stream(float4 *p, float4 v) {
    const hipq_vf4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<hipq_vf4 *>(p));
}
__device__ __forceinline__ void store_stream(uint32_t *p, uint32_t v) { __builtin_nontemporal_store(v, p); }

// RND 0: f32::round (half away from zero); 1: IEEE nearest-even; 2: floor(v + 0.5), the
// "faster rounding" of quantize_mobile_optimized (crates/torsh-quantization/src/simd_ops.rs:426-428),
// with the f32 sum rounded before the floor as there.  Callers that know two modes pass a bool.
// Half away from zero as trunc(v + copysign(h, v)) with h the largest float below 0.5: three
// instructions (v_bfi, v_add, v_trunc) instead of the six of the library roundf.  With 0.5 itself
// the sum rounds up across an integer for v = +-0.49999997; with h it never does, and ties still
// land on the integer away from zero because v + h then rounds to even = that integer.  Checked
// against roundf for every finite float (tests/host/round_away_check.c).
template <int RND>
__device__ __forceinline__ float round_mode(float v) {
    if constexpr (RND == 1)
        return rintf(v);
    else if constexpr (RND == 2)
        return floorf(v + 0.5f);
    else
        return truncf(v + copysignf(0x1.fffffep-2f, v));
}

// f32::clamp: NaN passes through.
__device__ __forceinline__ float clamp_keep_nan(float v, float lo, float hi) {
    v = (v < lo) ? lo : v;
    v = (v > hi) ? hi : v;
    return v;
}

// `f32 as i32` on a value already clamped to a small range: NaN -> 0.
__device__ __forceinline__ int to_int_nan0(float v) { return (v != v) ? 0 : static_cast<int>(v); }

// `f32 as i32`, saturating, NaN -> 0.
__device__ __forceinline__ int f32_as_i32(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return static_cast<int>(v);
}

// a / b, correctly rounded, from y = 1.0f / b (itself correctly rounded) with two FMAs
// (Markstein): q0 = RN(a*y), r = a - q0*b (exact in the FMA), q = RN(q0 + r*y).  Holds for every
// a while y is a normal number; an exhaustive CPU check over all 2^23 numerator significands x 22
// exponents x 3007 denominators (5.5e11 quotients) found no difference from a / b.  A division by
// one scale for a whole row or tensor then costs 3-4 instructions per element instead of the
// ~12 of the IEEE sequence.  y == 0 selects the plain division (recip_for_div returns 0 when
// 1/b is not normal); a NaN remainder (a or q0 infinite, or NaN input) means q0 already is the
// quotient.
__device__ __forceinline__ float recip_for_div(float b) {
    const float y = 1.0f / b;
    return (fabsf(y) >= FLT_MIN && fabsf(y) <= FLT_MAX) ? y : 0.0f;
}
__device__ __forceinline__ float div_rn(float a, float b, float y) {
    if (y == 0.0f) return a / b;
    const float q0 = a * y;
    const float r = fmaf(-q0, b, a);
    const float q1 = fmaf(r, y, q0);
    return (r == r) ? q1 : q0;
}

// The reference's "quantize one value" formulas differ in where the zero point enters:
//   FORM 0  round(x * (1/scale)) + zp     crates/torsh-quantization/src/simd_ops.rs:36-46
//   FORM 1  round(x / scale) + zp         crates/torsh-quantization/src/algorithms.rs:230-233, 302-305
//   FORM 2  round(x / scale + zp)         crates/torsh-core/src/dtype/quantized.rs:129-134 (QInt8 / QUInt8)
//   FORM 3  (round(x / scale) as i32) + zp   crates/torsh-nn/src/quantization/ops.rs:153-162 (NaN -> 0 before zp)
// A bool first argument reads as FORM 0 / 1.  `inv` is recip_for_div(scale) for the division forms, else 1/scale.
enum { QFORM_MUL = 0, QFORM_DIV = 1, QFORM_DIV_ZP_FIRST = 2, QFORM_DIV_INT_CAST = 3 };

// Saturating f32 -> i32 with NaN -> 0: exactly Rust's `as i32`, and exactly what
// v_cvt_i32_f32 does.  Inline asm so the conversion is never treated as undefined for
// out-of-range inputs.
__device__ __forceinline__ int cvt_i32_sat(float v) {
    int r;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(r) : "v"(v));
    return r;
}

// The quantized value, clamped; result still a float (the carrier).
template <int FORM, int RND>
__device__ __forceinline__ float quantize_value(float x, float scale, float inv, float zpf, float lo, float hi) {
    float t;
    if constexpr (FORM != QFORM_MUL)
        t = div_rn(x, scale, inv);
    else
        t = x * inv;
    float q;
    if constexpr (FORM == QFORM_DIV_ZP_FIRST)
        q = round_mode<RND>(t + zpf);
    else if constexpr (FORM == QFORM_DIV_INT_CAST)
        q = static_cast<float>(cvt_i32_sat(round_mode<RND>(t))) + zpf;  // clamped to a small range next
    else
        q = round_mode<RND>(t) + zpf;
    return clamp_keep_nan(q, lo, hi);
}

// Integer form of quantize_value for int8/uint8 outputs: the clamp is done after the
// conversion, on integers (round(..)+zp is integral, so converting first changes nothing;
// a NaN becomes 0 as `NaN.clamp(..) as i8` does, and +-Inf saturate).  About half the
// vector instructions of the float-clamp form.
template <int FORM, int RND>
__device__ __forceinline__ int quantize_int(float x, float scale, float inv, float zpf, int lo, int hi) {
    float t;
    if constexpr (FORM != QFORM_MUL)
        t = div_rn(x, scale, inv);
    else
        t = x * inv;
    int q;
    if constexpr (FORM == QFORM_DIV_ZP_FIRST) {
        q = cvt_i32_sat(round_mode<RND>(t + zpf));
    } else if constexpr (FORM == QFORM_DIV_INT_CAST) {
        // i32 sum of the reference; the inner clamp keeps it from wrapping and changes nothing after the outer one
        q = min(max(cvt_i32_sat(round_mode<RND>(t)), -(1 << 30)), 1 << 30) + static_cast<int>(zpf);
    } else {
        q = cvt_i32_sat(round_mode<RND>(t) + zpf);
    }
    return min(max(q, lo), hi);
}

// FORM 3 with the zero point as the integer it is: (round(x / scale) as i32) + zp, the sum taken in 64 bits (the
// reference's i32 sum never wraps where it does not panic), then the clamp.  A constant channel of torsh-nn's
// per-channel weights has scale 0 and a zero point at an end of the i32 range, which a float cannot carry.
template <int RND>
__device__ __forceinline__ int quantize_int_cast(float x, float scale, float inv, int zp, int lo, int hi) {
    const long long q = static_cast<long long>(cvt_i32_sat(round_mode<RND>(div_rn(x, scale, inv)))) + zp;
    return static_cast<int>(q < lo ? lo : (q > hi ? hi : q));
}

// quantize_int for a symmetric per-row quantizer (zero point 0, int8 range) whose scale was derived
// from the row's own finite maximum, scale = max|x| / 127: then |x * y| stays near 127, the
// remainder of div_rn is never NaN for a finite x, and the select that guards it can go; a NaN
// element still comes out as 0 (NaN propagates through both FMAs and the conversion maps it to 0).
template <bool EVEN>
__device__ __forceinline__ int quantize_int_sym(float x, float scale, float y) {
    float t;
    if (y == 0.0f) {
        t = x / scale;
    } else {
        const float q0 = x * y;
        t = fmaf(fmaf(-q0, scale, x), y, q0);
    }
    return min(max(cvt_i32_sat(round_mode<EVEN>(t)), -128), 127);
}

// clamp(round(v) ...) already formed as a float: convert and clamp on integers.
__device__ __forceinline__ int clamp_to_int(float q, int lo, int hi) { return min(max(cvt_i32_sat(q), lo), hi); }

// Low bytes of four ints -> one dword (three v_perm_b32 / v_or).
__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
    const uint32_t lo = __builtin_amdgcn_perm(static_cast<uint32_t>(b), static_cast<uint32_t>(a), 0x0c0c0400u);
    const uint32_t hi = __builtin_amdgcn_perm(static_cast<uint32_t>(d), static_cast<uint32_t>(c), 0x04000c0cu);
    return lo | hi;
}

// 4 x 4 byte transpose inside a quad of lanes: lane q holds bytes (row 0..3) of column q and ends with the bytes
// (column 0..3) of row q.  Two butterfly steps - swap with lane q ^ 1 and interleave bytes, swap with lane q ^ 2 and
// interleave halves - each a data-parallel move and a byte permute whose selector depends on the lane:
// sel1 = q & 1 ? 0x03070105 : 0x06020400, sel2 = q & 2 ? 0x03020706 : 0x05040100.
__device__ __forceinline__ uint32_t quad_byte_transpose(uint32_t d, uint32_t sel1, uint32_t sel2) {
    const uint32_t p1 = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(d), 0xB1, 0xf, 0xf, true));
    const uint32_t t = __builtin_amdgcn_perm(p1, d, sel1);
    const uint32_t p2 = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(t), 0x4E, 0xf, 0xf, true));
    return __builtin_amdgcn_perm(p2, t, sel2);
}

__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, kWave));
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

// (min,max) -> (scale, zero_point) with the reference formula `flavor` selects.
// Returns HIPQ_SUCCESS or HIPQ_INVALID_ARGUMENT.
//   HIPQ_PARAMS_SYMMETRIC          crates/torsh-quantization/src/algorithms.rs:397-422
//   HIPQ_PARAMS_AFFINE             crates/torsh-quantization/src/algorithms.rs:358-394
//   HIPQ_PARAMS_BACKEND_SYMMETRIC  crates/torsh-backend/src/quantization/params.rs:323-340
//   HIPQ_PARAMS_BACKEND_ASYMMETRIC crates/torsh-backend/src/quantization/params.rs:343-363
//   HIPQ_PARAMS_ZERO_INCLUDED      crates/torsh-quantization/src/observers.rs:263-310, specialized.rs:39-48, 322-335
//   HIPQ_PARAMS_NN_SYMMETRIC       crates/torsh-nn/src/quantization/ops.rs:322-325 (no guards: a zero range gives scale 0)
//   HIPQ_PARAMS_NN_ASYMMETRIC      crates/torsh-nn/src/quantization/ops.rs:326-330 (zero point not clamped)
__device__ __forceinline__ int params_from_minmax(float mn, float mx, int flavor, int qmin_i, int qmax_i,
                                                  float *scale, int *zp) {
    const bool finite = (fabsf(mn) <= FLT_MAX) && (fabsf(mx) <= FLT_MAX);  // false for NaN and Inf
    const float qmin = static_cast<float>(qmin_i), qmax = static_cast<float>(qmax_i);
    *scale = 1.0f;
    *zp = 0;
    switch (flavor) {
    case HIPQ_PARAMS_SYMMETRIC: {
        if (!finite) return HIPQ_INVALID_ARGUMENT;
        float abs_max = fmaxf(fabsf(mn), fabsf(mx));
        if (abs_max < FLT_EPSILON) return HIPQ_SUCCESS;
        *scale = abs_max / qmax;
        return HIPQ_SUCCESS;
    }
    case HIPQ_PARAMS_AFFINE: {
        if (!finite || mn > mx) return HIPQ_INVALID_ARGUMENT;
        if (fabsf(mx - mn) < FLT_EPSILON) {
            *zp = qmin_i;
            return HIPQ_SUCCESS;
        }
        float s = (mx - mn) / (qmax - qmin);
        float z = qmin - mn / s;
        *scale = s;
        *zp = f32_as_i32(clamp_keep_nan(roundf(z), qmin, qmax));
        return HIPQ_SUCCESS;
    }
    case HIPQ_PARAMS_BACKEND_SYMMETRIC: {
        if (!finite || mn > mx) return HIPQ_INVALID_ARGUMENT;
        float r = fmaxf(fabsf(mx), fabsf(mn));
        if (r != 0.0f) *scale = (2.0f * r) / (qmax - qmin);
        return HIPQ_SUCCESS;
    }
    case HIPQ_PARAMS_BACKEND_ASYMMETRIC: {
        if (!finite || mn > mx) return HIPQ_INVALID_ARGUMENT;
        if (mx == mn) {
            *zp = qmin_i;
            return HIPQ_SUCCESS;
        }
        float s = (mx - mn) / (qmax - qmin);
        float z = qmin - mn / s;
        *scale = s;
        *zp = f32_as_i32(clamp_keep_nan(roundf(z), qmin, qmax));
        return HIPQ_SUCCESS;
    }
    case HIPQ_PARAMS_ZERO_INCLUDED: {
        mn = fminf(mn, 0.0f);
        mx = fmaxf(mx, 0.0f);
        if (!((fabsf(mn) <= FLT_MAX) && (fabsf(mx) <= FLT_MAX))) return HIPQ_INVALID_ARGUMENT;
        float s = (mx - mn) / (qmax - qmin);
        if (s == 0.0f) s = 1.0f;
        *scale = s;
        *zp = f32_as_i32(fminf(fmaxf(roundf(qmin - mn / s), qmin), qmax));
        return HIPQ_SUCCESS;
    }
    case HIPQ_PARAMS_NN_SYMMETRIC: {
        *scale = fmaxf(fabsf(mx), fabsf(mn)) / 127.0f;
        return HIPQ_SUCCESS;
    }
    case HIPQ_PARAMS_NN_ASYMMETRIC: {
        const float s = (mx - mn) / 255.0f;
        *scale = s;
        *zp = f32_as_i32(roundf(-mn / s));
        return HIPQ_SUCCESS;
    }
    default:
        return HIPQ_INVALID_ARGUMENT;
    }
}

}  // namespace hipq
