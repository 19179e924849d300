// Calibration and quality kernels around the quantized path: observer statistics (range +
// non-finite count, fixed-range histogram), quantization quality metrics (two tensors, or one
// tensor against its own fake-quantized image computed on the fly), and fake quantization.
// All stream their inputs once from HBM; reductions use wave shuffles, LDS and per-workgroup
// partials folded by a second small launch (no global atomics: atomics from all XCDs on a few
// addresses serialise).
#include "hipq_internal.h"
#include "hipq_math.h"
#include "hipq_stream.h"

namespace hipq {

// ---- quality metrics -----------------------------------------------------------------------

// Running sums of calculate_quantization_metrics (crates/torsh-quantization/src/metrics.rs:93-152).
struct MetricSums {
    double sse, sae, spow, dot, qq;
    unsigned long long zeros;
    float max_err, max_sig;
};

struct MetricLane {
    // f32 sums of one float4 pair, flushed into the f64 accumulators per call.
    double sse = 0, sae = 0, spow = 0, dot = 0, qq = 0;
    unsigned zeros = 0;
    float max_err = 0.0f, max_sig = 0.0f;

    __device__ __forceinline__ void term(float a, float b, float &s0, float &s1, float &s2, float &s3, float &s4) {
        const float d = a - b;
        const float ad = fabsf(d);
        s0 = fmaf(d, d, s0);
        s1 += ad;
        s2 = fmaf(a, a, s2);
        s3 = fmaf(a, b, s3);
        s4 = fmaf(b, b, s4);
        max_err = fmaxf(max_err, ad);
        max_sig = fmaxf(max_sig, fabsf(a));
        zeros += (ad < 1e-7f) ? 1u : 0u;  // metrics.rs:119
    }
    __device__ __forceinline__ void add4(const float4 &a, const float4 &b) {
        float s0 = 0, s1 = 0, s2 = 0, s3 = 0, s4 = 0;
        term(a.x, b.x, s0, s1, s2, s3, s4);
        term(a.y, b.y, s0, s1, s2, s3, s4);
        term(a.z, b.z, s0, s1, s2, s3, s4);
        term(a.w, b.w, s0, s1, s2, s3, s4);
        sse += s0, sae += s1, spow += s2, dot += s3, qq += s4;
    }
    __device__ __forceinline__ void add1(float a, float b) {
        float s0 = 0, s1 = 0, s2 = 0, s3 = 0, s4 = 0;
        term(a, b, s0, s1, s2, s3, s4);
        sse += s0, sae += s1, spow += s2, dot += s3, qq += s4;
    }
};

__device__ __forceinline__ void block_store_sums(const MetricLane &m, MetricSums *__restrict__ out) {
    __shared__ MetricSums lds[kCalBlock / kWave];
    MetricSums w;
    w.sse = wave_sum(m.sse);
    w.sae = wave_sum(m.sae);
    w.spow = wave_sum(m.spow);
    w.dot = wave_sum(m.dot);
    w.qq = wave_sum(m.qq);
    w.zeros = wave_sum(static_cast<unsigned long long>(m.zeros));
    w.max_err = wave_max(m.max_err);
    w.max_sig = wave_max(m.max_sig);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == 0) lds[wave] = w;
    __syncthreads();
    if (threadIdx.x == 0) {
        MetricSums r = lds[0];
        for (int i = 1; i < kCalBlock / kWave; ++i) {
            r.sse += lds[i].sse, r.sae += lds[i].sae, r.spow += lds[i].spow, r.dot += lds[i].dot, r.qq += lds[i].qq;
            r.zeros += lds[i].zeros;
            r.max_err = fmaxf(r.max_err, lds[i].max_err);
            r.max_sig = fmaxf(r.max_sig, lds[i].max_sig);
        }
        *out = r;
    }
}

// The fake-quantized image of one value: quantize (either form), then dequantize.
//   carrier form: clamp(round(..) + zp) stays f32, y = (q - zp) * scale
//       (crates/torsh-quantization/src/simd_ops.rs:36-46, 52-81)
//   FQ_INT_CAST:  the clamped value goes through `as i32` (NaN -> 0), y = (q - zp) as f32 * scale
//       (crates/torsh-models/src/quantization.rs:336-347)
//   FQ_MAX_MIN:   the clamp is `.max(qmin).min(qmax)`, which maps NaN to qmin, y = scale * (q - zp)
//       (crates/torsh-quantization/src/fake_quantize.rs:24-33)
enum { FQ_CARRIER = 0, FQ_INT_CAST = 1, FQ_MAX_MIN = 2 };
template <bool DIV, bool EVEN, int KIND>
__device__ __forceinline__ float fake_quantize_value(float x, float scale, float inv, int zp, float zpf, float lo,
                                                     float hi) {
    if constexpr (KIND == FQ_MAX_MIN) {
        const float q = quantize_value<DIV, EVEN>(x, scale, inv, zpf, -INFINITY, INFINITY);
        return scale * (fminf(fmaxf(q, lo), hi) - zpf);  // fmaxf / fminf return the operand that is not NaN
    } else {
        const float q = quantize_value<DIV, EVEN>(x, scale, inv, zpf, lo, hi);
        if constexpr (KIND == FQ_INT_CAST) {
            return static_cast<float>(cvt_i32_sat(q) - zp) * scale;
        } else {
            return (q - zpf) * scale;
        }
    }
}

struct FakeQuantArgs {
    float scale;
    int zp;
    float lo, hi;
    const hipq_qparams *params;  // non-null: scale and zero point are read from device memory
};

__global__ __launch_bounds__(kCalBlock) void metrics_partial_kernel(const float *__restrict__ a,
                                                                     const float *__restrict__ b, size_t n,
                                                                     MetricSums *__restrict__ partials) {
    MetricLane m;
    stream2(
        a, b, n, [&](const float4 &va, const float4 &vb) { m.add4(va, vb); },
        [&](float va, float vb) { m.add1(va, vb); });
    block_store_sums(m, partials + blockIdx.x);
}

template <bool DIV, bool EVEN, int KIND>
__global__ __launch_bounds__(kCalBlock) void fake_quant_metrics_partial_kernel(const float *__restrict__ x, size_t n,
                                                                                FakeQuantArgs fq,
                                                                                MetricSums *__restrict__ partials) {
    if (fq.params) {
        fq.scale = fq.params->scale;
        fq.zp = fq.params->zero_point;
    }
    const float scale = fq.scale, zpf = static_cast<float>(fq.zp);
    const float inv = DIV ? recip_for_div(scale) : 1.0f / scale;
    MetricLane m;
    auto fqv = [&](float v) { return fake_quantize_value<DIV, EVEN, KIND>(v, scale, inv, fq.zp, zpf, fq.lo, fq.hi); };
    stream1<kCalBlock>(
        x, n,
        [&](const float4 &v, size_t) { m.add4(v, make_float4(fqv(v.x), fqv(v.y), fqv(v.z), fqv(v.w))); },
        [&](float v, size_t) { m.add1(v, fqv(v)); });
    block_store_sums(m, partials + blockIdx.x);
}

// One workgroup folds the partials and evaluates metrics.rs:93-172 on the totals.  The sums are
// carried in f64; each published quantity is rounded to f32 once.
__global__ __launch_bounds__(kCalBlock) void metrics_final_kernel(const MetricSums *__restrict__ partials,
                                                                   int nparts, size_t n, float compression_ratio,
                                                                   hipq_quant_metrics *__restrict__ out) {
    MetricLane m;
    unsigned long long zeros = 0;
    for (int i = threadIdx.x; i < nparts; i += kCalBlock) {
        const MetricSums p = partials[i];
        m.sse += p.sse, m.sae += p.sae, m.spow += p.spow, m.dot += p.dot, m.qq += p.qq;
        zeros += p.zeros;
        m.max_err = fmaxf(m.max_err, p.max_err);
        m.max_sig = fmaxf(m.max_sig, p.max_sig);
    }
    __shared__ MetricSums lds[kCalBlock / kWave];
    __shared__ unsigned long long lds_zeros[kCalBlock / kWave];
    MetricSums w;
    w.sse = wave_sum(m.sse);
    w.sae = wave_sum(m.sae);
    w.spow = wave_sum(m.spow);
    w.dot = wave_sum(m.dot);
    w.qq = wave_sum(m.qq);
    w.max_err = wave_max(m.max_err);
    w.max_sig = wave_max(m.max_sig);
    zeros = wave_sum(zeros);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == 0) {
        lds[wave] = w;
        lds_zeros[wave] = zeros;
    }
    __syncthreads();
    if (threadIdx.x != 0) return;
    if (n == 0) {  // QuantizationMetrics::default(), metrics.rs:50-63
        *out = hipq_quant_metrics{0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 100.0f, 1.0f, 1.0f};
        return;
    }
    MetricSums r = lds[0];
    unsigned long long z = lds_zeros[0];
    for (int i = 1; i < kCalBlock / kWave; ++i) {
        r.sse += lds[i].sse, r.sae += lds[i].sae, r.spow += lds[i].spow, r.dot += lds[i].dot, r.qq += lds[i].qq;
        z += lds_zeros[i];
        r.max_err = fmaxf(r.max_err, lds[i].max_err);
        r.max_sig = fmaxf(r.max_sig, lds[i].max_sig);
    }
    const double len = static_cast<double>(n);
    const double mse = r.sse / len, signal_power = r.spow / len;
    const float mse_f = static_cast<float>(mse), sp_f = static_cast<float>(signal_power);
    hipq_quant_metrics q;
    q.mse = mse_f;
    q.mae = static_cast<float>(r.sae / len);
    q.max_error = r.max_err;
    q.zero_error_percentage = (static_cast<float>(z) / static_cast<float>(n)) * 100.0f;  // exact count, f32 formula of :122
    q.psnr = mse_f > 0.0f ? static_cast<float>(20.0 * log10(static_cast<double>(r.max_sig) / sqrt(mse))) : INFINITY;
    q.snr = (mse_f > 0.0f && sp_f > 0.0f) ? static_cast<float>(10.0 * log10(signal_power / mse)) : INFINITY;
    const float on = static_cast<float>(sqrt(r.spow)), qn = static_cast<float>(sqrt(r.qq));
    q.cosine_similarity = (on > 0.0f && qn > 0.0f) ? static_cast<float>(r.dot / (sqrt(r.spow) * sqrt(r.qq))) : 0.0f;
    q.compression_ratio = compression_ratio;
    *out = q;
}

template <bool DIV, bool EVEN, int KIND>
__global__ __launch_bounds__(kCalBlock) void fake_quantize_kernel(const float *__restrict__ x, size_t n,
                                                                   FakeQuantArgs fq, float *__restrict__ out) {
    if (fq.params) {
        if (fq.params->status != HIPQ_SUCCESS) return;
        fq.scale = fq.params->scale;
        fq.zp = fq.params->zero_point;
    }
    const float scale = fq.scale, zpf = static_cast<float>(fq.zp);
    const float inv = DIV ? recip_for_div(scale) : 1.0f / scale;
    auto fqv = [&](float v) { return fake_quantize_value<DIV, EVEN, KIND>(v, scale, inv, fq.zp, zpf, fq.lo, fq.hi); };
    const bool out_aligned = (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
    if (out_aligned) {
        stream1<kCalBlock>(
            x, n,
            [&](const float4 &v, size_t idx) {
                store_stream(reinterpret_cast<float4 *>(out) + idx, make_float4(fqv(v.x), fqv(v.y), fqv(v.z), fqv(v.w)));
            },
            [&](float v, size_t i) { out[i] = fqv(v); });
    } else {
        for (size_t i = size_t(blockIdx.x) * kCalBlock + threadIdx.x; i < n; i += size_t(gridDim.x) * kCalBlock)
            out[i] = fqv(x[i]);
    }
}

// ---- tensor statistics ---------------------------------------------------------------------

struct StatsPartial {
    float mn, mx;
    double s1, s2;  // sum of x and of x^2, or (CENTERED) unused and the sum of (x - mean)^2
};

__device__ __forceinline__ void stats_block_store(float mn, float mx, double s1, double s2,
                                                  StatsPartial *__restrict__ out) {
    __shared__ StatsPartial lds[kCalBlock / kWave];
    StatsPartial w{wave_min(mn), wave_max(mx), wave_sum(s1), wave_sum(s2)};
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == 0) lds[wave] = w;
    __syncthreads();
    if (threadIdx.x == 0) {
        StatsPartial r = lds[0];
        for (int i = 1; i < kCalBlock / kWave; ++i) {
            r.mn = fminf(r.mn, lds[i].mn);
            r.mx = fmaxf(r.mx, lds[i].mx);
            r.s1 += lds[i].s1;
            r.s2 += lds[i].s2;
        }
        *out = r;
    }
}

// One pass of calculate_tensor_stats_simd (crates/torsh-quantization/src/simd_ops.rs:230-262) or of
// calculate_tensor_stats_cache_optimized (algorithms.rs:525-578): every element enters the sums as
// an f64, as there.  CENTERED = the second pass of the former, sum of (x - mean)^2 with the mean
// the first pass left in `totals`.
template <bool CENTERED>
__global__ __launch_bounds__(kCalBlock) void stats_partial_kernel(const float *__restrict__ x, size_t n,
                                                                   const StatsPartial *__restrict__ totals,
                                                                   StatsPartial *__restrict__ partials) {
    float mn = INFINITY, mx = -INFINITY;
    double s1 = 0.0, s2 = 0.0;
    double mean = 0.0;
    if constexpr (CENTERED) mean = totals->s1 / static_cast<double>(n);
    auto one = [&](float v) {
        const double d = static_cast<double>(v);
        if constexpr (CENTERED) {
            const double c = d - mean;
            s2 = fma(c, c, s2);
        } else {
            mn = fminf(mn, v);
            mx = fmaxf(mx, v);
            s1 += d;
            s2 = fma(d, d, s2);  // d * d is exact in f64
        }
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
    stats_block_store(mn, mx, s1, s2, partials + blockIdx.x);
}

// STAGE 0: fold the first pass into `totals` (and, ONE_PASS, finish with the raw-moment formulas of
// algorithms.rs:571-575).  STAGE 1: fold the centered sums and finish as simd_ops.rs:240-261.
template <int STAGE, bool ONE_PASS>
__global__ __launch_bounds__(kCalBlock) void stats_final_kernel(const StatsPartial *__restrict__ partials, int nparts,
                                                                 size_t n, StatsPartial *__restrict__ totals,
                                                                 hipq_tensor_stats *__restrict__ out) {
    float mn = INFINITY, mx = -INFINITY;
    double s1 = 0.0, s2 = 0.0;
    for (int i = threadIdx.x; i < nparts; i += kCalBlock) {
        const StatsPartial p = partials[i];
        mn = fminf(mn, p.mn);
        mx = fmaxf(mx, p.mx);
        s1 += p.s1;
        s2 += p.s2;
    }
    __shared__ StatsPartial folded;
    stats_block_store(mn, mx, s1, s2, &folded);
    if (threadIdx.x != 0) return;
    const StatsPartial r = folded;
    const double nd = static_cast<double>(n);
    if constexpr (STAGE == 0) {
        *totals = r;
        if constexpr (ONE_PASS) {
            const float mean = static_cast<float>(r.s1 / nd);
            const double md = static_cast<double>(mean);
            const float variance = static_cast<float>(r.s2 / nd - md * md);
            out->min_val = r.mn;
            out->max_val = r.mx;
            out->mean = mean;
            out->variance = variance;
            out->std_dev = sqrtf(variance);
        }
    } else {
        const double variance = r.s2 / nd;
        out->min_val = totals->mn;
        out->max_val = totals->mx;
        out->mean = static_cast<float>(totals->s1 / nd);
        out->variance = static_cast<float>(variance);
        out->std_dev = static_cast<float>(sqrt(variance));
    }
}

// ---- observer statistics -------------------------------------------------------------------

struct ObservePartial {
    float mn, mx;
    unsigned long long nonfinite;
};

// Range and count of non-finite values in one pass (Observer::update validates before it folds,
// crates/torsh-quantization/src/observers.rs:122-150).
__global__ __launch_bounds__(kCalBlock) void observe_partial_kernel(const float *__restrict__ x, size_t n,
                                                                     ObservePartial *__restrict__ partials) {
    float mn = INFINITY, mx = -INFINITY;
    unsigned bad = 0;
    auto one = [&](float v) {
        mn = fminf(mn, v);
        mx = fmaxf(mx, v);
        bad += (fabsf(v) <= FLT_MAX) ? 0u : 1u;  // true for NaN and +-Inf
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
    __shared__ ObservePartial lds[kCalBlock / kWave];
    ObservePartial w{wave_min(mn), wave_max(mx), wave_sum(static_cast<unsigned long long>(bad))};
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == 0) lds[wave] = w;
    __syncthreads();
    if (threadIdx.x == 0) {
        ObservePartial r = lds[0];
        for (int i = 1; i < kCalBlock / kWave; ++i) {
            r.mn = fminf(r.mn, lds[i].mn);
            r.mx = fmaxf(r.mx, lds[i].mx);
            r.nonfinite += lds[i].nonfinite;
        }
        partials[blockIdx.x] = r;
    }
}

__global__ __launch_bounds__(kCalBlock) void observe_final_kernel(const ObservePartial *__restrict__ partials,
                                                                   int nparts, hipq_observe_stats *__restrict__ out) {
    float mn = INFINITY, mx = -INFINITY;
    unsigned long long bad = 0;
    for (int i = threadIdx.x; i < nparts; i += kCalBlock) {
        const ObservePartial p = partials[i];
        mn = fminf(mn, p.mn);
        mx = fmaxf(mx, p.mx);
        bad += p.nonfinite;
    }
    __shared__ ObservePartial lds[kCalBlock / kWave];
    ObservePartial w{wave_min(mn), wave_max(mx), wave_sum(bad)};
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == 0) lds[wave] = w;
    __syncthreads();
    if (threadIdx.x == 0) {
        ObservePartial r = lds[0];
        for (int i = 1; i < kCalBlock / kWave; ++i) {
            r.mn = fminf(r.mn, lds[i].mn);
            r.mx = fmaxf(r.mx, lds[i].mx);
            r.nonfinite += lds[i].nonfinite;
        }
        out->min_val = r.mn;
        out->max_val = r.mx;
        out->nonfinite = r.nonfinite;
    }
}

// Histogram over a fixed range with the bin rule of Observer::value_to_bin_index
// (crates/torsh-quantization/src/observers.rs:313-333):
//   range_max <= range_min or value not finite -> bin 0
//   ratio = clamp((value - range_min) / (range_max - range_min), 0, 1)
//   bin   = min(floor(ratio * num_bins) as usize, num_bins - 1)
// Each wavefront counts into its own LDS copy (COPIES = waves per workgroup) or, for many bins,
// all share one; the workgroup's total goes to its row of `partials`.
constexpr int kHistBlock = 1024;

__global__ __launch_bounds__(kHistBlock) void histogram_partial_kernel(const float *__restrict__ x, size_t n,
                                                                        float range_min, float range_max,
                                                                        int num_bins, int copies,
                                                                        uint32_t *__restrict__ partials) {
    extern __shared__ uint32_t hist[];
    for (int i = threadIdx.x; i < num_bins * copies; i += kHistBlock) hist[i] = 0;
    __syncthreads();
    uint32_t *mine = hist + (copies > 1 ? (threadIdx.x / kWave) % copies : 0) * num_bins;
    const bool degenerate = range_max <= range_min;
    const float den = range_max - range_min;
    const float inv = recip_for_div(den);
    const float nb = static_cast<float>(num_bins);
    const int last = num_bins - 1;
    auto one = [&](float v) {
        int bin = 0;
        if (!degenerate && fabsf(v) <= FLT_MAX) {
            const float ratio = clamp_keep_nan(div_rn(v - range_min, den, inv), 0.0f, 1.0f);
            bin = min(max(cvt_i32_sat(floorf(ratio * nb)), 0), last);  // NaN -> 0, as `as usize`
        }
        atomicAdd(&mine[bin], 1u);
    };
    stream1<kHistBlock>(
        x, n,
        [&](const float4 &v, size_t) {
            one(v.x);
            one(v.y);
            one(v.z);
            one(v.w);
        },
        [&](float v, size_t) { one(v); });
    __syncthreads();
    uint32_t *row = partials + size_t(blockIdx.x) * num_bins;
    for (int i = threadIdx.x; i < num_bins; i += kHistBlock) {
        uint32_t s = 0;
        for (int c = 0; c < copies; ++c) s += hist[c * num_bins + i];
        row[i] = s;
    }
}

// counts[bin] += sum over workgroups of partials[wg][bin].  A workgroup owns 64 consecutive bins
// (one coalesced 256-byte load per row); its 16 wavefronts split the rows and issue their loads
// back to back, so the fold costs about one memory latency instead of one per row.
constexpr int kFoldBlock = 1024;
constexpr int kFoldUnroll = 8;

__global__ __launch_bounds__(kFoldBlock) void histogram_fold_kernel(const uint32_t *__restrict__ partials, int nparts,
                                                                     int num_bins,
                                                                     unsigned long long *__restrict__ counts) {
    __shared__ unsigned long long lds[kFoldBlock];
    constexpr int kWaves = kFoldBlock / kWave;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int bin = blockIdx.x * kWave + lane;
    unsigned long long s = 0;
    if (bin < num_bins) {
        for (int p0 = wave; p0 < nparts; p0 += kWaves * kFoldUnroll) {
            uint32_t v[kFoldUnroll];
#pragma unroll
            for (int u = 0; u < kFoldUnroll; ++u) {
                const int p = p0 + u * kWaves;
                v[u] = p < nparts ? partials[size_t(p) * num_bins + bin] : 0u;
            }
#pragma unroll
            for (int u = 0; u < kFoldUnroll; ++u) s += v[u];
        }
    }
    lds[threadIdx.x] = s;
    __syncthreads();
    if (wave == 0 && bin < num_bins) {
        for (int w = 1; w < kWaves; ++w) s += lds[w * kWave + lane];
        counts[bin] += s;
    }
}

// Workgroups per CU, measured on 16 Mi elements: the two-input metrics kernel is fastest with 3
// (26.8 us with 2, 23.1 with 3, 24.4 with 4), the fused fake-quantize metrics kernel with 4
// (17.1 / 15.9 / 15.4), the single-input range kernels do not care (2).
constexpr int kMaxWgPerCu = 4;

static int calib_grid(const hipq_ctx *ctx, size_t n, int tile_elems, int per_cu = 2) {
    const size_t tiles = (n + tile_elems - 1) / tile_elems;
    const size_t cap = static_cast<size_t>(ctx->num_cus) * per_cu;
    return static_cast<int>(tiles < 1 ? 1 : (tiles < cap ? tiles : cap));
}

static int32_t launch_metrics_final(hipq_ctx *ctx, const MetricSums *partials, int nparts, size_t n,
                                    uint32_t original_bits, uint32_t quantized_bits, hipq_quant_metrics *out) {
    const float ratio = static_cast<float>(original_bits) / static_cast<float>(quantized_bits);  // metrics.rs:161
    metrics_final_kernel<<<1, kCalBlock, 0, ctx->stream>>>(partials, nparts, n, ratio, out);
    return check_launch("metrics_final_kernel");
}

static int fq_kind(int32_t mode) {
    return (mode & HIPQ_FAKE_INT_CAST) ? FQ_INT_CAST : ((mode & HIPQ_FAKE_NAN_TO_QMIN) ? FQ_MAX_MIN : FQ_CARRIER);
}

template <bool DIV, bool EVEN>
static void launch_fq_metrics(int kind, int grid, hipStream_t s, const float *x, size_t n, FakeQuantArgs fq,
                              MetricSums *partials) {
    if (kind == FQ_INT_CAST)
        fake_quant_metrics_partial_kernel<DIV, EVEN, FQ_INT_CAST><<<grid, kCalBlock, 0, s>>>(x, n, fq, partials);
    else if (kind == FQ_MAX_MIN)
        fake_quant_metrics_partial_kernel<DIV, EVEN, FQ_MAX_MIN><<<grid, kCalBlock, 0, s>>>(x, n, fq, partials);
    else
        fake_quant_metrics_partial_kernel<DIV, EVEN, FQ_CARRIER><<<grid, kCalBlock, 0, s>>>(x, n, fq, partials);
}

template <bool DIV, bool EVEN>
static void launch_fq(int kind, int grid, hipStream_t s, const float *x, size_t n, FakeQuantArgs fq, float *out) {
    if (kind == FQ_INT_CAST)
        fake_quantize_kernel<DIV, EVEN, FQ_INT_CAST><<<grid, kCalBlock, 0, s>>>(x, n, fq, out);
    else if (kind == FQ_MAX_MIN)
        fake_quantize_kernel<DIV, EVEN, FQ_MAX_MIN><<<grid, kCalBlock, 0, s>>>(x, n, fq, out);
    else
        fake_quantize_kernel<DIV, EVEN, FQ_CARRIER><<<grid, kCalBlock, 0, s>>>(x, n, fq, out);
}

static int32_t check_fake_quant_args(const char *fn, float scale, const hipq_qparams *params, int32_t qmin,
                                     int32_t qmax, int32_t mode) {
    if (!params && !(scale > 0.0f))
        return fail(HIPQ_INVALID_ARGUMENT, "%s: Scale must be positive, got %g", fn, static_cast<double>(scale));
    if (qmin > qmax) return fail(HIPQ_INVALID_ARGUMENT, "%s: qmin %d > qmax %d", fn, qmin, qmax);
    if (mode & ~(HIPQ_ROUND_HALF_EVEN | HIPQ_FORM_DIV | HIPQ_FAKE_INT_CAST | HIPQ_FAKE_NAN_TO_QMIN))
        return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown mode bits 0x%x", fn, mode);
    if ((mode & HIPQ_FAKE_INT_CAST) && (mode & HIPQ_FAKE_NAN_TO_QMIN))
        return fail(HIPQ_INVALID_ARGUMENT, "%s: HIPQ_FAKE_INT_CAST and HIPQ_FAKE_NAN_TO_QMIN exclude each other", fn);
    return HIPQ_SUCCESS;
}

}  // namespace hipq

using namespace hipq;

extern "C" {

int32_t hipq_quantization_metrics_f32(hipq_ctx *ctx, const float *original, const float *quantized, size_t n,
                                      uint32_t original_bits, uint32_t quantized_bits,
                                      hipq_quant_metrics *out_metrics) {
    HIPQ_ENTER(ctx);
    HIPQ_REQUIRE_PTR(out_metrics);
    if (n) {
        HIPQ_REQUIRE_PTR(original);
        HIPQ_REQUIRE_PTR(quantized);
    }
    if (quantized_bits == 0 || original_bits == 0)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: bit widths must be positive", __func__);
    const int grid = n ? calib_grid(ctx, n, kCalTile * 2, 3) : 0;
    void *scr = nullptr;
    int32_t rc = scratch(ctx, kScratchHeader + sizeof(MetricSums) * static_cast<size_t>(ctx->num_cus) * kMaxWgPerCu, &scr);
    if (rc != HIPQ_SUCCESS) return rc;
    MetricSums *partials = reinterpret_cast<MetricSums *>(static_cast<char *>(scr) + kScratchHeader);
    if (grid) {
        metrics_partial_kernel<<<grid, kCalBlock, 0, ctx->stream>>>(original, quantized, n, partials);
        rc = check_launch("metrics_partial_kernel");
        if (rc != HIPQ_SUCCESS) return rc;
    }
    return launch_metrics_final(ctx, partials, grid, n, original_bits, quantized_bits, out_metrics);
}

int32_t hipq_fake_quantize_metrics_f32(hipq_ctx *ctx, const float *x, size_t n, float scale, int32_t zero_point,
                                       const hipq_qparams *params, int32_t qmin, int32_t qmax, int32_t mode,
                                       uint32_t original_bits, uint32_t quantized_bits,
                                       hipq_quant_metrics *out_metrics) {
    HIPQ_ENTER(ctx);
    HIPQ_REQUIRE_PTR(out_metrics);
    if (n) HIPQ_REQUIRE_PTR(x);
    int32_t rc = check_fake_quant_args(__func__, scale, params, qmin, qmax, mode);
    if (rc != HIPQ_SUCCESS) return rc;
    if (quantized_bits == 0 || original_bits == 0)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: bit widths must be positive", __func__);
    const int grid = n ? calib_grid(ctx, n, kCalTile * 4, kMaxWgPerCu) : 0;
    void *scr = nullptr;
    rc = scratch(ctx, kScratchHeader + sizeof(MetricSums) * static_cast<size_t>(ctx->num_cus) * kMaxWgPerCu, &scr);
    if (rc != HIPQ_SUCCESS) return rc;
    MetricSums *partials = reinterpret_cast<MetricSums *>(static_cast<char *>(scr) + kScratchHeader);
    if (grid) {
        const FakeQuantArgs fq{scale, zero_point, static_cast<float>(qmin), static_cast<float>(qmax), params};
        const int ic = fq_kind(mode);
        const bool div = (mode & HIPQ_FORM_DIV) != 0, even = (mode & HIPQ_ROUND_HALF_EVEN) != 0;
        if (div && even)
            launch_fq_metrics<true, true>(ic, grid, ctx->stream, x, n, fq, partials);
        else if (div)
            launch_fq_metrics<true, false>(ic, grid, ctx->stream, x, n, fq, partials);
        else if (even)
            launch_fq_metrics<false, true>(ic, grid, ctx->stream, x, n, fq, partials);
        else
            launch_fq_metrics<false, false>(ic, grid, ctx->stream, x, n, fq, partials);
        rc = check_launch("fake_quant_metrics_partial_kernel");
        if (rc != HIPQ_SUCCESS) return rc;
    }
    return launch_metrics_final(ctx, partials, grid, n, original_bits, quantized_bits, out_metrics);
}

int32_t hipq_fake_quantize_f32(hipq_ctx *ctx, const float *x, size_t n, float scale, int32_t zero_point,
                               const hipq_qparams *params, int32_t qmin, int32_t qmax, int32_t mode, float *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_fake_quant_args(__func__, scale, params, qmin, qmax, mode);
    if (rc != HIPQ_SUCCESS) return rc;
    if (n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out);
    const int grid = calib_grid(ctx, n, kCalTile * 4);
    const FakeQuantArgs fq{scale, zero_point, static_cast<float>(qmin), static_cast<float>(qmax), params};
    const int ic = fq_kind(mode);
    const bool div = (mode & HIPQ_FORM_DIV) != 0, even = (mode & HIPQ_ROUND_HALF_EVEN) != 0;
    if (div && even)
        launch_fq<true, true>(ic, grid, ctx->stream, x, n, fq, out);
    else if (div)
        launch_fq<true, false>(ic, grid, ctx->stream, x, n, fq, out);
    else if (even)
        launch_fq<false, true>(ic, grid, ctx->stream, x, n, fq, out);
    else
        launch_fq<false, false>(ic, grid, ctx->stream, x, n, fq, out);
    return check_launch("fake_quantize_kernel");
}

int32_t hipq_tensor_stats_f32(hipq_ctx *ctx, const float *x, size_t n, int32_t one_pass, hipq_tensor_stats *out_stats) {
    HIPQ_ENTER(ctx);
    HIPQ_REQUIRE_PTR(out_stats);
    if (n == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: Cannot calculate stats of empty tensor", __func__);
    HIPQ_REQUIRE_PTR(x);
    const int grid = calib_grid(ctx, n, kCalTile * 4);
    void *scr = nullptr;
    int32_t rc = scratch(ctx, kScratchHeader + sizeof(StatsPartial) * static_cast<size_t>(ctx->num_cus) * kMaxWgPerCu, &scr);
    if (rc != HIPQ_SUCCESS) return rc;
    StatsPartial *totals = reinterpret_cast<StatsPartial *>(scr);  // in the scratch header
    StatsPartial *partials = reinterpret_cast<StatsPartial *>(static_cast<char *>(scr) + kScratchHeader);
    stats_partial_kernel<false><<<grid, kCalBlock, 0, ctx->stream>>>(x, n, totals, partials);
    if (one_pass) {
        stats_final_kernel<0, true><<<1, kCalBlock, 0, ctx->stream>>>(partials, grid, n, totals, out_stats);
        return check_launch("tensor_stats");
    }
    stats_final_kernel<0, false><<<1, kCalBlock, 0, ctx->stream>>>(partials, grid, n, totals, out_stats);
    stats_partial_kernel<true><<<grid, kCalBlock, 0, ctx->stream>>>(x, n, totals, partials);
    stats_final_kernel<1, false><<<1, kCalBlock, 0, ctx->stream>>>(partials, grid, n, totals, out_stats);
    return check_launch("tensor_stats");
}

int32_t hipq_observe_f32(hipq_ctx *ctx, const float *x, size_t n, hipq_observe_stats *out_stats) {
    HIPQ_ENTER(ctx);
    HIPQ_REQUIRE_PTR(out_stats);
    if (n) HIPQ_REQUIRE_PTR(x);
    const int grid = n ? calib_grid(ctx, n, kCalTile * 4) : 0;
    void *scr = nullptr;
    int32_t rc = scratch(ctx, kScratchHeader + sizeof(ObservePartial) * static_cast<size_t>(ctx->num_cus) * kMaxWgPerCu, &scr);
    if (rc != HIPQ_SUCCESS) return rc;
    ObservePartial *partials = reinterpret_cast<ObservePartial *>(static_cast<char *>(scr) + kScratchHeader);
    if (grid) {
        observe_partial_kernel<<<grid, kCalBlock, 0, ctx->stream>>>(x, n, partials);
        rc = check_launch("observe_partial_kernel");
        if (rc != HIPQ_SUCCESS) return rc;
    }
    // n == 0 folds nothing: (+inf, -inf, 0), the state an empty batch leaves untouched.
    observe_final_kernel<<<1, kCalBlock, 0, ctx->stream>>>(partials, grid, out_stats);
    return check_launch("observe_final_kernel");
}

int32_t hipq_histogram_f32(hipq_ctx *ctx, const float *x, size_t n, float range_min, float range_max,
                           size_t num_bins, uint64_t *counts) {
    HIPQ_ENTER(ctx);
    if (num_bins == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: num_bins must be positive", __func__);
    if (num_bins > HIPQ_HISTOGRAM_MAX_BINS)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: num_bins %zu exceeds the supported maximum %d", __func__, num_bins,
                    HIPQ_HISTOGRAM_MAX_BINS);
    if (n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(counts);
    // A workgroup's LDS counters are 32 bits wide; with at most 2^32-1 elements per launch no
    // counter can wrap.  Longer inputs are walked in slices.
    const int nb = static_cast<int>(num_bins);
    const int waves = kHistBlock / kWave;
    const int copies = nb <= 1024 ? waves : (nb <= 4096 ? 4 : 1);
    const size_t lds_bytes = sizeof(uint32_t) * static_cast<size_t>(nb) * copies;
    const size_t kSlice = size_t(1) << 31;
    void *scr = nullptr;
    const size_t max_grid = static_cast<size_t>(ctx->num_cus);
    int32_t rc = scratch(ctx, kScratchHeader + sizeof(uint32_t) * max_grid * num_bins, &scr);
    if (rc != HIPQ_SUCCESS) return rc;
    uint32_t *partials = reinterpret_cast<uint32_t *>(static_cast<char *>(scr) + kScratchHeader);
    for (size_t off = 0; off < n; off += kSlice) {
        const size_t len = (n - off) < kSlice ? (n - off) : kSlice;
        const size_t tiles = (len + size_t(kHistBlock) * kCalVec * 4 - 1) / (size_t(kHistBlock) * kCalVec * 4);
        const int grid = static_cast<int>(tiles < max_grid ? tiles : max_grid);
        histogram_partial_kernel<<<grid, kHistBlock, lds_bytes, ctx->stream>>>(x + off, len, range_min, range_max, nb,
                                                                               copies, partials);
        rc = check_launch("histogram_partial_kernel");
        if (rc != HIPQ_SUCCESS) return rc;
        histogram_fold_kernel<<<(nb + kWave - 1) / kWave, kFoldBlock, 0, ctx->stream>>>(
            partials, grid, nb, reinterpret_cast<unsigned long long *>(counts));
        rc = check_launch("histogram_fold_kernel");
        if (rc != HIPQ_SUCCESS) return rc;
    }
    return HIPQ_SUCCESS;
}

}  // extern "C"
