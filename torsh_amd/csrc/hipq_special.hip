// Binary and ternary quantization (crates/torsh-quantization/src/specialized.rs:163-238): a sign
// or a thresholded sign per element plus one scale for the tensor, the mean of |x| over the
// elements that keep a sign.  One streaming pass writes the int8 codes and per-workgroup sums;
// a one-workgroup launch folds them.  The ternary threshold needs max|x| first (one more pass).
#include "hipq_internal.h"
#include "hipq_math.h"
#include "hipq_stream.h"

namespace hipq {

struct SignPartial {
    double sum;                 // sum of |x| over the counted elements
    unsigned long long count;   // counted elements
};

__device__ __forceinline__ void block_store_sign_partial(double sum, unsigned count, SignPartial *__restrict__ out) {
    __shared__ SignPartial lds[kCalBlock / kWave];
    SignPartial w{wave_sum(sum), wave_sum(static_cast<unsigned long long>(count))};
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == 0) lds[wave] = w;
    __syncthreads();
    if (threadIdx.x == 0) {
        SignPartial r = lds[0];
        for (int i = 1; i < kCalBlock / kWave; ++i) {
            r.sum += lds[i].sum;
            r.count += lds[i].count;
        }
        *out = r;
    }
}

// max|x| partial per workgroup (the fold `max(|x|)` from 0 of specialized.rs:200; NaN is ignored).
__global__ __launch_bounds__(kCalBlock) void absmax_partial_kernel(const float *__restrict__ x, size_t n,
                                                                    float *__restrict__ partials) {
    float m = 0.0f;
    stream1<kCalBlock>(
        x, n,
        [&](const float4 &v, size_t) {
            m = fmaxf(m, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        },
        [&](float v, size_t) { m = fmaxf(m, fabsf(v)); });
    __shared__ float lds[kCalBlock / kWave];
    m = wave_max(m);
    if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < kCalBlock / kWave; ++i) m = fmaxf(m, lds[i]);
        partials[blockIdx.x] = m;
    }
}

enum { SIGN_BINARY = 0, SIGN_TERNARY = 1, SIGN_GIVEN_GT = 2, SIGN_GIVEN_GE = 3 };

// SIGN_BINARY:   code = x >= 0 ? 1 : -1, every element counted (specialized.rs:172-180).
// SIGN_TERNARY:  threshold = 0.7 * max|x| folded from `absmax_partials` by every workgroup;
//                code = |x| <= threshold ? 0 : (x > 0 ? 1 : -1); elements with |x| > threshold
//                are counted (specialized.rs:201-227).
// SIGN_GIVEN_GT: the same with the threshold an earlier launch left in out_threshold[0]
//                (quantize_ternary_adaptive, specialized.rs:519-545).
// SIGN_GIVEN_GE: threshold from out_threshold[0], or `given` when has_given; the sign test is
//                x >= 0 (quantize_binary_learned_threshold, specialized.rs:452-483).
template <int MODE>
__global__ __launch_bounds__(kCalBlock) void sign_quantize_kernel(const float *__restrict__ x, size_t n,
                                                                   const float *__restrict__ absmax_partials,
                                                                   int nparts, int8_t *__restrict__ out,
                                                                   SignPartial *__restrict__ partials,
                                                                   float *__restrict__ out_threshold, int has_given,
                                                                   float given) {
    constexpr bool TERNARY = MODE != SIGN_BINARY;
    float threshold = 0.0f, max_abs = 0.0f;
    if constexpr (MODE == SIGN_GIVEN_GT || MODE == SIGN_GIVEN_GE) {
        // read before any workgroup could rewrite it: only `given` is ever written here, by the
        // thread that has just taken it from the argument
        threshold = has_given ? given : out_threshold[0];
        if (has_given && blockIdx.x == 0 && threadIdx.x == 0) {
            out_threshold[0] = given;
            out_threshold[1] = 0.0f;
        }
    }
    if constexpr (MODE == SIGN_TERNARY) {
        __shared__ float lds[kCalBlock / kWave];
        for (int i = threadIdx.x; i < nparts; i += kCalBlock) max_abs = fmaxf(max_abs, absmax_partials[i]);
        max_abs = wave_max(max_abs);
        if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = max_abs;
        __syncthreads();
        max_abs = lds[0];
        for (int i = 1; i < kCalBlock / kWave; ++i) max_abs = fmaxf(max_abs, lds[i]);
        threshold = max_abs * 0.7f;
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            out_threshold[0] = threshold;
            out_threshold[1] = max_abs;
        }
    }
    float sum4 = 0.0f;  // flushed into the f64 accumulator after every float4
    double sum = 0.0;
    unsigned count = 0;
    auto code = [&](float v) {
        const float a = fabsf(v);
        if constexpr (TERNARY) {
            if (a <= threshold) return 0;
            sum4 += a;
            ++count;
            if constexpr (MODE == SIGN_GIVEN_GE)
                return v >= 0.0f ? 1 : -1;
            else
                return v > 0.0f ? 1 : -1;
        } else {
            sum4 += a;
            ++count;
            return v >= 0.0f ? 1 : -1;
        }
    };
    const bool out_aligned = (reinterpret_cast<uintptr_t>(out) & 3u) == 0;
    stream1<kCalBlock>(
        x, n,
        [&](const float4 &v, size_t idx) {
            sum4 = 0.0f;
            const int a = code(v.x), b = code(v.y), c = code(v.z), d = code(v.w);
            sum += sum4;
            if (!out) return;  // sums only
            if (out_aligned) {
                store_stream(reinterpret_cast<uint32_t *>(out) + idx, pack4(a, b, c, d));
            } else {
                int8_t *o = out + idx * 4;
                o[0] = static_cast<int8_t>(a), o[1] = static_cast<int8_t>(b);
                o[2] = static_cast<int8_t>(c), o[3] = static_cast<int8_t>(d);
            }
        },
        [&](float v, size_t i) {
            sum4 = 0.0f;
            const int c = code(v);
            if (out) out[i] = static_cast<int8_t>(c);
            sum += sum4;
        });
    block_store_sign_partial(sum, count, partials + blockIdx.x);
}

// scale = sum / count (1 when nothing was counted, and for the binary scheme when the mean is 0).
__global__ __launch_bounds__(kCalBlock) void sign_final_kernel(const SignPartial *__restrict__ partials, int nparts,
                                                                int ternary, const float *__restrict__ threshold,
                                                                hipq_qparams *__restrict__ out) {
    double sum = 0.0;
    unsigned long long count = 0;
    for (int i = threadIdx.x; i < nparts; i += kCalBlock) {
        sum += partials[i].sum;
        count += partials[i].count;
    }
    __shared__ SignPartial lds[kCalBlock / kWave];
    SignPartial w{wave_sum(sum), wave_sum(count)};
    if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = w;
    __syncthreads();
    if (threadIdx.x != 0) return;
    SignPartial r = lds[0];
    for (int i = 1; i < kCalBlock / kWave; ++i) {
        r.sum += lds[i].sum;
        r.count += lds[i].count;
    }
    float scale = 1.0f;
    if (r.count > 0) {
        scale = static_cast<float>(r.sum / static_cast<double>(r.count));
        if (!ternary && scale == 0.0f) scale = 1.0f;  // specialized.rs:174
    }
    out->scale = scale;
    out->zero_point = 0;
    out->min_val = ternary ? threshold[0] : 0.0f;
    out->max_val = ternary ? threshold[1] : 0.0f;
    out->status = HIPQ_SUCCESS;
}

// threshold = mean |x| (quantize_binary_learned_threshold without a given threshold,
// specialized.rs:452-456), from the sums a SIGN_BINARY pass left.
__global__ __launch_bounds__(kCalBlock) void mean_abs_threshold_kernel(const SignPartial *__restrict__ partials,
                                                                        int nparts, size_t n,
                                                                        float *__restrict__ out_threshold) {
    double sum = 0.0;
    for (int i = threadIdx.x; i < nparts; i += kCalBlock) sum += partials[i].sum;
    __shared__ double lds[kCalBlock / kWave];
    sum = wave_sum(sum);
    if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = sum;
    __syncthreads();
    if (threadIdx.x != 0) return;
    for (int i = 1; i < kCalBlock / kWave; ++i) sum += lds[i];
    out_threshold[0] = static_cast<float>(sum / static_cast<double>(n));
    out_threshold[1] = 0.0f;
}

// quantize_ternary_adaptive's search (specialized.rs:505-517, 555-570): for the ten thresholds
// max|x| * (i * 0.1), i = 1..10, the squared error of the unit ternary code, all in one pass.
constexpr int kTernaryCandidates = 10;
struct SearchPartial {
    double err[kTernaryCandidates];
};

__device__ __forceinline__ float ternary_candidate(float max_abs, int i) {
    return max_abs * (static_cast<float>(i) * 0.1f);
}

__global__ __launch_bounds__(kCalBlock) void ternary_search_kernel(const float *__restrict__ x, size_t n,
                                                                    const float *__restrict__ absmax_partials,
                                                                    int nparts, SearchPartial *__restrict__ partials,
                                                                    float *__restrict__ out_threshold) {
    __shared__ float lds_max[kCalBlock / kWave];
    float max_abs = 0.0f;
    for (int i = threadIdx.x; i < nparts; i += kCalBlock) max_abs = fmaxf(max_abs, absmax_partials[i]);
    max_abs = wave_max(max_abs);
    if (threadIdx.x % kWave == 0) lds_max[threadIdx.x / kWave] = max_abs;
    __syncthreads();
    max_abs = lds_max[0];
    for (int i = 1; i < kCalBlock / kWave; ++i) max_abs = fmaxf(max_abs, lds_max[i]);
    if (blockIdx.x == 0 && threadIdx.x == 0) out_threshold[1] = max_abs;
    float thr[kTernaryCandidates];
#pragma unroll
    for (int i = 0; i < kTernaryCandidates; ++i) thr[i] = ternary_candidate(max_abs, i + 1);
    double err[kTernaryCandidates];
#pragma unroll
    for (int i = 0; i < kTernaryCandidates; ++i) err[i] = 0.0;
    auto one = [&](float v) {
        const float a = fabsf(v);
        const float away = v - (v > 0.0f ? 1.0f : -1.0f);  // x - q for a kept sign
        const double e_zero = static_cast<double>(v * v);          // the reference's f32 (x - q).powi(2)
        const double e_sign = static_cast<double>(away * away);
#pragma unroll
        for (int i = 0; i < kTernaryCandidates; ++i) err[i] += (a <= thr[i]) ? e_zero : e_sign;
    };
    stream1<kCalBlock>(
        x, n,
        [&](const float4 &v, size_t) {
            one(v.x);
            one(v.y);
            one(v.z);
            one(v.w);
        },
        [&](float v, size_t) { one(v); });
    __shared__ SearchPartial lds[kCalBlock / kWave];
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
#pragma unroll
    for (int i = 0; i < kTernaryCandidates; ++i) {
        const double w = wave_sum(err[i]);
        if (lane == 0) lds[wave].err[i] = w;
    }
    __syncthreads();
    if (threadIdx.x < kTernaryCandidates) {
        double r = lds[0].err[threadIdx.x];
        for (int w = 1; w < kCalBlock / kWave; ++w) r += lds[w].err[threadIdx.x];
        partials[blockIdx.x].err[threadIdx.x] = r;
    }
}

// First threshold with the strictly smallest mean error, in candidate order (specialized.rs:510-517).
__global__ __launch_bounds__(kCalBlock) void ternary_search_final_kernel(const SearchPartial *__restrict__ partials,
                                                                          int nparts, size_t n,
                                                                          float *__restrict__ out_threshold) {
    double err[kTernaryCandidates];
#pragma unroll
    for (int i = 0; i < kTernaryCandidates; ++i) err[i] = 0.0;
    for (int p = threadIdx.x; p < nparts; p += kCalBlock) {
#pragma unroll
        for (int i = 0; i < kTernaryCandidates; ++i) err[i] += partials[p].err[i];
    }
    __shared__ SearchPartial lds[kCalBlock / kWave];
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
#pragma unroll
    for (int i = 0; i < kTernaryCandidates; ++i) {
        const double w = wave_sum(err[i]);
        if (lane == 0) lds[wave].err[i] = w;
    }
    __syncthreads();
    if (threadIdx.x != 0) return;
    const float max_abs = out_threshold[1];
    float best_threshold = 0.0f, best_error = INFINITY;
    for (int i = 0; i < kTernaryCandidates; ++i) {
        double r = lds[0].err[i];
        for (int w = 1; w < kCalBlock / kWave; ++w) r += lds[w].err[i];
        const float mean_err = static_cast<float>(r / static_cast<double>(n));
        if (mean_err < best_error) {
            best_error = mean_err;
            best_threshold = ternary_candidate(max_abs, i + 1);
        }
    }
    out_threshold[0] = best_threshold;
}

static int32_t sign_quantize(const char *fn, hipq_ctx *ctx, const float *x, size_t n, bool ternary, int8_t *out,
                             hipq_qparams *out_params) {
    if (n == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: Cannot quantize empty tensor", fn);
    if (!x || !out || !out_params) return fail(HIPQ_INVALID_ARGUMENT, "%s: null pointer", fn);
    const size_t tiles = (n + size_t(kCalTile) * 4 - 1) / (size_t(kCalTile) * 4);
    const size_t cap = static_cast<size_t>(ctx->num_cus) * 4;
    const int grid = static_cast<int>(tiles < cap ? tiles : cap);
    void *scr = nullptr;
    // header: threshold and max|x| (2 floats); then absmax partials; then sign partials
    int32_t rc = scratch(ctx, kScratchHeader + cap * (sizeof(float) + sizeof(SignPartial)) + 64, &scr);
    if (rc != HIPQ_SUCCESS) return rc;
    float *threshold = reinterpret_cast<float *>(scr);
    SignPartial *partials = reinterpret_cast<SignPartial *>(static_cast<char *>(scr) + kScratchHeader);
    float *absmax_partials = reinterpret_cast<float *>(partials + cap);
    if (ternary) {
        absmax_partial_kernel<<<grid, kCalBlock, 0, ctx->stream>>>(x, n, absmax_partials);
        if ((rc = check_launch("absmax_partial_kernel")) != HIPQ_SUCCESS) return rc;
        sign_quantize_kernel<SIGN_TERNARY><<<grid, kCalBlock, 0, ctx->stream>>>(x, n, absmax_partials, grid, out,
                                                                                  partials, threshold, 0, 0.0f);
    } else {
        sign_quantize_kernel<SIGN_BINARY><<<grid, kCalBlock, 0, ctx->stream>>>(x, n, nullptr, 0, out, partials,
                                                                                 threshold, 0, 0.0f);
    }
    if ((rc = check_launch("sign_quantize_kernel")) != HIPQ_SUCCESS) return rc;
    sign_final_kernel<<<1, kCalBlock, 0, ctx->stream>>>(partials, grid, ternary ? 1 : 0, threshold, out_params);
    return check_launch("sign_final_kernel");
}

// The two searched-threshold schemes.  adaptive: max|x| -> ten-candidate search -> codes;
// learned: (mean |x| unless a threshold is given) -> codes.
static int32_t sign_quantize_searched(const char *fn, hipq_ctx *ctx, const float *x, size_t n, bool adaptive,
                                      int has_threshold, float given, int8_t *out, hipq_qparams *out_params) {
    if (n == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: Cannot quantize empty tensor", fn);
    if (!x || !out || !out_params) return fail(HIPQ_INVALID_ARGUMENT, "%s: null pointer", fn);
    const size_t tiles = (n + size_t(kCalTile) * 4 - 1) / (size_t(kCalTile) * 4);
    const size_t cap = static_cast<size_t>(ctx->num_cus) * 4;
    const int grid = static_cast<int>(tiles < cap ? tiles : cap);
    void *scr = nullptr;
    int32_t rc = scratch(ctx, kScratchHeader + cap * (sizeof(float) + sizeof(SignPartial) + sizeof(SearchPartial)) + 64,
                         &scr);
    if (rc != HIPQ_SUCCESS) return rc;
    float *threshold = reinterpret_cast<float *>(scr);
    SearchPartial *search = reinterpret_cast<SearchPartial *>(static_cast<char *>(scr) + kScratchHeader);
    SignPartial *partials = reinterpret_cast<SignPartial *>(search + cap);
    float *absmax_partials = reinterpret_cast<float *>(partials + cap);
    if (adaptive) {
        absmax_partial_kernel<<<grid, kCalBlock, 0, ctx->stream>>>(x, n, absmax_partials);
        ternary_search_kernel<<<grid, kCalBlock, 0, ctx->stream>>>(x, n, absmax_partials, grid, search, threshold);
        ternary_search_final_kernel<<<1, kCalBlock, 0, ctx->stream>>>(search, grid, n, threshold);
        if ((rc = check_launch("ternary_search")) != HIPQ_SUCCESS) return rc;
        sign_quantize_kernel<SIGN_GIVEN_GT><<<grid, kCalBlock, 0, ctx->stream>>>(x, n, nullptr, 0, out, partials,
                                                                                   threshold, 0, 0.0f);
    } else {
        if (!has_threshold) {
            // a pass for its sums only (no codes written): mean |x|
            sign_quantize_kernel<SIGN_BINARY><<<grid, kCalBlock, 0, ctx->stream>>>(x, n, nullptr, 0, nullptr, partials,
                                                                                     threshold, 0, 0.0f);
            mean_abs_threshold_kernel<<<1, kCalBlock, 0, ctx->stream>>>(partials, grid, n, threshold);
            if ((rc = check_launch("mean_abs_threshold_kernel")) != HIPQ_SUCCESS) return rc;
        }
        sign_quantize_kernel<SIGN_GIVEN_GE><<<grid, kCalBlock, 0, ctx->stream>>>(x, n, nullptr, 0, out, partials,
                                                                                   threshold, has_threshold, given);
    }
    if ((rc = check_launch("sign_quantize_kernel")) != HIPQ_SUCCESS) return rc;
    sign_final_kernel<<<1, kCalBlock, 0, ctx->stream>>>(partials, grid, 1, threshold, out_params);
    return check_launch("sign_final_kernel");
}

}  // namespace hipq

using namespace hipq;

extern "C" {

int32_t hipq_quantize_binary_f32_i8(hipq_ctx *ctx, const float *x, size_t n, int8_t *out, hipq_qparams *out_params) {
    HIPQ_ENTER(ctx);
    return sign_quantize(__func__, ctx, x, n, false, out, out_params);
}

int32_t hipq_quantize_ternary_f32_i8(hipq_ctx *ctx, const float *x, size_t n, int8_t *out, hipq_qparams *out_params) {
    HIPQ_ENTER(ctx);
    return sign_quantize(__func__, ctx, x, n, true, out, out_params);
}

int32_t hipq_quantize_binary_learned_threshold_f32_i8(hipq_ctx *ctx, const float *x, size_t n, int32_t has_threshold,
                                                      float threshold, int8_t *out, hipq_qparams *out_params) {
    HIPQ_ENTER(ctx);
    return sign_quantize_searched(__func__, ctx, x, n, false, has_threshold ? 1 : 0, threshold, out, out_params);
}

int32_t hipq_quantize_ternary_adaptive_f32_i8(hipq_ctx *ctx, const float *x, size_t n, int8_t *out,
                                              hipq_qparams *out_params) {
    HIPQ_ENTER(ctx);
    return sign_quantize_searched(__func__, ctx, x, n, true, 0, 0.0f, out, out_params);
}

}  // extern "C"
