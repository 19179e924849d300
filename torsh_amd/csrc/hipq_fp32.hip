// fp32 helpers of the int8 transformer stack: LayerNorm, tanh-GELU, residual add,
// and the fused forms that hand their result straight to the per-token int8
// quantizer (the normalised / activated row never makes a round trip through HBM
// as fp32).  One wavefront or one workgroup owns a row and keeps it in registers:
// a single HBM read per element, wave shuffles for the row statistics.
#include "hipq_internal.h"
#include "hipq_math.h"

namespace hipq {

constexpr int kRowBlock = 256;
constexpr int kRowCacheMax = 12;  // most float4 a thread keeps in registers (RC template parameter)

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

template <int TPR>
__device__ __forceinline__ float row_sum(float v, float *lds) {
    v = wave_sum(v);
    if constexpr (TPR == kWave) {
        return v;
    } else {
        const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
        __syncthreads();
        if (lane == 0) lds[wave] = v;
        __syncthreads();
        float r = 0.0f;
#pragma unroll
        for (int w = 0; w < TPR / kWave; ++w) r += lds[w];
        return r;
    }
}

template <int TPR>
__device__ __forceinline__ float row_max(float v, float *lds) {
    v = wave_max(v);
    if constexpr (TPR == kWave) {
        return v;
    } else {
        const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
        __syncthreads();
        if (lane == 0) lds[wave] = v;
        __syncthreads();
        float r = lds[0];
#pragma unroll
        for (int w = 1; w < TPR / kWave; ++w) r = fmaxf(r, lds[w]);
        return r;
    }
}

// tanh-form GELU, crates/torsh-nn/src/layers/activation/modern.rs:124-136:
//   0.5 * x * (1 + tanh(u)),  u = sqrt(2/pi) * (x + 0.044715 x^3).
// Evaluated as x / (1 + exp(-2u)), which is the same function (1 + tanh(u) = 2 / (1 + exp(-2u)))
// without the cancellation of 1 + tanh(u) for negative x, and costs one v_exp_f32 and one
// v_rcp_f32 instead of a tanhf call: the fused GELU + quantize kernel was bound by tanhf, not by
// HBM.  Against the reference's evaluation order in f32 the difference stays below 2e-6
// relative + 1e-7 absolute (the reference form itself carries up to |x| * 3e-8 of cancellation
// error).
// -2u * log2(e) = x * (K + K*c*x^2) with K = -2*log2(e)*sqrt(2/pi): one multiply, one fused
// multiply-add, one multiply (this function is compared at a tolerance, so the contraction is
// allowed here).  No clamp of the exponent: exp2 saturates to inf / 0, and rcp(1 + inf) = 0,
// rcp(1 + 0) = 1 give the right limits x * 0 and x.
__device__ __forceinline__ float gelu_tanh(float x) {
    constexpr float K = -2.8853900817779268f * 0.7978845608028654f;
    const float arg = x * fmaf(x * x, K * 0.044715f, K);
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(arg));
}

enum { ROW_LAYERNORM = 0, ROW_GELU = 1 };

// OP: LayerNorm over the row (biased variance, eps inside the square root) or GELU.
// QUANT: write the row as per-token symmetric int8 (scale = absmax/127,
// q = clamp(round(y / scale)), the division form of
// crates/torsh-quantization/src/algorithms.rs:126-242) instead of fp32.
// Rows are TPR threads wide and at most TPR * RC * 4 columns long (RC float4 per thread, all
// requested before the first is used); cols % 4 == 0.  The row is read once and written once,
// so both streams bypass the caches.
template <int TPR, int RC, int OP, bool QUANT, bool EVEN>
__device__ __forceinline__ void row_op_body(float4 (&v)[RC], size_t row, bool active, int lane, size_t cols,
                                            const float *__restrict__ gamma, const float *__restrict__ beta,
                                            float eps, float *__restrict__ out_f, int8_t *__restrict__ out_q,
                                            float *__restrict__ out_scales, float *lds) {
    const size_t nvec = cols / 4;
    if constexpr (OP == ROW_LAYERNORM) {
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < RC; ++i) s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
        const float mean = row_sum<TPR>(s, lds) / static_cast<float>(cols);
        float sq = 0.0f;
#pragma unroll
        for (int i = 0; i < RC; ++i) {
            const size_t idx = size_t(lane) + size_t(i) * TPR;
            if (idx < nvec) {
                const float a = v[i].x - mean, b = v[i].y - mean, c = v[i].z - mean, d = v[i].w - mean;
                sq += (a * a + b * b) + (c * c + d * d);
            }
        }
        const float var = row_sum<TPR>(sq, lds) / static_cast<float>(cols);
        const float rstd = 1.0f / sqrtf(var + eps);
        const float4 *g4 = reinterpret_cast<const float4 *>(gamma), *b4 = reinterpret_cast<const float4 *>(beta);
#pragma unroll
        for (int i = 0; i < RC; ++i) {
            const size_t idx = size_t(lane) + size_t(i) * TPR;
            if (idx < nvec) {
                float4 y = make_float4((v[i].x - mean) * rstd, (v[i].y - mean) * rstd, (v[i].z - mean) * rstd,
                                       (v[i].w - mean) * rstd);
                if (gamma) {
                    const float4 g = g4[idx];
                    y = make_float4(y.x * g.x, y.y * g.y, y.z * g.z, y.w * g.w);
                }
                if (beta) {
                    const float4 b = b4[idx];
                    y = make_float4(y.x + b.x, y.y + b.y, y.z + b.z, y.w + b.w);
                }
                v[i] = y;
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < RC; ++i) {
            const size_t idx = size_t(lane) + size_t(i) * TPR;
            if (idx < nvec) v[i] = make_float4(gelu_tanh(v[i].x), gelu_tanh(v[i].y), gelu_tanh(v[i].z), gelu_tanh(v[i].w));
        }
    }
    if constexpr (!QUANT) {
        if (!active) return;
        float4 *o4 = reinterpret_cast<float4 *>(out_f + row * cols);
#pragma unroll
        for (int i = 0; i < RC; ++i) {
            const size_t idx = size_t(lane) + size_t(i) * TPR;
            if (idx < nvec) store_stream(o4 + idx, v[i]);
        }
    } else {
        float am = 0.0f;
#pragma unroll
        for (int i = 0; i < RC; ++i) {
            const size_t idx = size_t(lane) + size_t(i) * TPR;
            if (idx < nvec) am = fmaxf(fmaxf(am, fmaxf(fabsf(v[i].x), fabsf(v[i].y))), fmaxf(fabsf(v[i].z), fabsf(v[i].w)));
        }
        am = row_max<TPR>(am, lds);
        if (!active) return;
        // calculate_symmetric_quantization_params, algorithms.rs:397-422 (a non-finite row
        // yields a NaN scale, which the caller can test for).
        float scale = am < FLT_EPSILON ? 1.0f : am / 127.0f;
        if (!(fabsf(am) <= FLT_MAX)) scale = NAN;
        if (lane == 0) out_scales[row] = scale;
        const float inv = recip_for_div(scale);  // once per row
        uint32_t *q4 = reinterpret_cast<uint32_t *>(out_q + row * cols);
#pragma unroll
        for (int i = 0; i < RC; ++i) {
            const size_t idx = size_t(lane) + size_t(i) * TPR;
            if (idx < nvec) {
                store_stream(q4 + idx, pack4(quantize_int_sym<EVEN>(v[i].x, scale, inv), quantize_int_sym<EVEN>(v[i].y, scale, inv),
                                             quantize_int_sym<EVEN>(v[i].z, scale, inv), quantize_int_sym<EVEN>(v[i].w, scale, inv)));
            }
        }
    }
}

// ADD: the row is x + delta (one rounding per element), written back over x before it is
// normalised: the residual update of the stream and the LayerNorm that follows it in one pass.
// STRIDE: workgroups walk the row groups with a grid stride and request the next group's row
// before the current one is processed, so loads, arithmetic and stores of different rows overlap in
// every wave.  Without it (as many workgroups as row groups) a wave handles one row and holds no
// second row buffer: fewer registers, more waves per SIMD to overlap the phases across waves.
template <int TPR, int RC, int OP, bool QUANT, bool EVEN, bool STRIDE, bool ADD>
__global__ __launch_bounds__(kRowBlock) void row_op_kernel(const float *x, const float *__restrict__ delta,
                                                            float *sum_out, size_t rows, size_t cols,
                                                            const float *__restrict__ gamma,
                                                            const float *__restrict__ beta, float eps,
                                                            float *__restrict__ out_f, int8_t *__restrict__ out_q,
                                                            float *__restrict__ out_scales) {
    constexpr int kRowsPerBlock = kRowBlock / TPR;
    __shared__ float lds[kRowBlock / kWave];
    const int sub = threadIdx.x / TPR, lane = threadIdx.x % TPR;
    const size_t nvec = cols / 4;
    const size_t groups = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
    constexpr int RD = ADD ? RC : 1;
    auto load_row = [&](size_t g, float4(&dst)[RC], float4(&dd)[RD]) {
        const size_t row = g * kRowsPerBlock + sub;
        const bool active = row < rows;
        const float4 *x4 = reinterpret_cast<const float4 *>(x + (active ? row : 0) * cols);
        const float4 *d4 = reinterpret_cast<const float4 *>(delta + (ADD && active ? row : 0) * cols);
#pragma unroll
        for (int i = 0; i < RC; ++i) {
            const size_t idx = size_t(lane) + size_t(i) * TPR;
            dst[i] = (active && idx < nvec) ? load_stream(x4 + idx) : make_float4(0.f, 0.f, 0.f, 0.f);
            if constexpr (ADD) dd[i] = (active && idx < nvec) ? load_stream(d4 + idx) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    // x + delta, stored back as the new row of the stream.
    auto add_row = [&](size_t g, float4(&dst)[RC], const float4(&dd)[RD]) {
        if constexpr (ADD) {
            const size_t row = g * kRowsPerBlock + sub;
            float4 *s4 = reinterpret_cast<float4 *>(sum_out + (row < rows ? row : 0) * cols);
#pragma unroll
            for (int i = 0; i < RC; ++i) {
                const size_t idx = size_t(lane) + size_t(i) * TPR;
                dst[i] = make_float4(dst[i].x + dd[i].x, dst[i].y + dd[i].y, dst[i].z + dd[i].z, dst[i].w + dd[i].w);
                if (row < rows && idx < nvec) store_stream(s4 + idx, dst[i]);
            }
        }
    };
    float4 v[RC], d[RD];
    size_t g = blockIdx.x;
    if (g >= groups) return;
    load_row(g, v, d);
    if constexpr (!STRIDE) {
        const size_t row = g * kRowsPerBlock + sub;
        add_row(g, v, d);
        row_op_body<TPR, RC, OP, QUANT, EVEN>(v, row, row < rows, lane, cols, gamma, beta, eps, out_f, out_q, out_scales,
                                              lds);
    } else {
        float4 nx[RC], nd[RD];
        for (; g < groups; g += gridDim.x) {
            const size_t gn = g + gridDim.x;
            if (gn < groups) load_row(gn, nx, nd);
            const size_t row = g * kRowsPerBlock + sub;
            add_row(g, v, d);
            row_op_body<TPR, RC, OP, QUANT, EVEN>(v, row, row < rows, lane, cols, gamma, beta, eps, out_f, out_q,
                                                  out_scales, lds);
#pragma unroll
            for (int i = 0; i < RC; ++i) v[i] = nx[i];
            if constexpr (ADD) {
#pragma unroll
                for (int i = 0; i < RC; ++i) d[i] = nd[i];
            }
        }
    }
}

__global__ __launch_bounds__(256) void gelu_kernel(const float *__restrict__ x, size_t n, float *__restrict__ out) {
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
    const size_t nvec = aligned ? n / 4 : 0;
    const float4 *x4 = reinterpret_cast<const float4 *>(x);
    float4 *o4 = reinterpret_cast<float4 *>(out);
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < nvec; i += size_t(gridDim.x) * 256) {
        const float4 p = x4[i];
        o4[i] = make_float4(gelu_tanh(p.x), gelu_tanh(p.y), gelu_tanh(p.z), gelu_tanh(p.w));
    }
    for (size_t i = nvec * 4 + size_t(blockIdx.x) * 256 + threadIdx.x; i < n; i += size_t(gridDim.x) * 256)
        out[i] = gelu_tanh(x[i]);
}

__global__ __launch_bounds__(256) void add_kernel(const float *__restrict__ a, const float *__restrict__ b, size_t n,
                                                   float *__restrict__ out) {
    const bool aligned = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) |
                           reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
    const size_t nvec = aligned ? n / 4 : 0;
    const float4 *a4 = reinterpret_cast<const float4 *>(a), *b4 = reinterpret_cast<const float4 *>(b);
    float4 *o4 = reinterpret_cast<float4 *>(out);
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < nvec; i += size_t(gridDim.x) * 256) {
        const float4 p = a4[i], q = b4[i];
        o4[i] = make_float4(p.x + q.x, p.y + q.y, p.z + q.z, p.w + q.w);
    }
    for (size_t i = nvec * 4 + size_t(blockIdx.x) * 256 + threadIdx.x; i < n; i += size_t(gridDim.x) * 256)
        out[i] = a[i] + b[i];
}

// Enough workgroups to fill the chip a few times over, few enough that each walks several
// row groups and overlaps their phases.
static int row_grid(hipq_ctx *ctx, size_t rows, int rows_per_block) {
    const size_t groups = (rows + rows_per_block - 1) / rows_per_block;
    constexpr int per_cu = 8;  // measured best of 1, 2, 4, 8 on [8192, 768] and [8192, 3072]
    const size_t cap = size_t(ctx->num_cus) * per_cu;
    return static_cast<int>(groups < cap ? groups : cap);
}

template <int OP, bool QUANT, bool ADD = false>
static int32_t launch_row_op(const char *fn, hipq_ctx *ctx, const float *x, size_t rows, size_t cols, const float *gamma,
                             const float *beta, float eps, int32_t mode, float *out_f, int8_t *out_q,
                             float *out_scales, const float *delta = nullptr, float *sum_out = nullptr) {
    if (rows == 0) return HIPQ_SUCCESS;
    if (cols == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: rows of zero length", fn);
    if (cols % 4 != 0 || cols > size_t(kRowBlock) * kRowCacheMax * 4)
        return fail(HIPQ_SHAPE_ERROR, "%s: row length %zu must be a multiple of 4 and at most %d", fn, cols,
                    kRowBlock * kRowCacheMax * 4);
    uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gamma) |
                     reinterpret_cast<uintptr_t>(beta) | reinterpret_cast<uintptr_t>(out_f) |
                     reinterpret_cast<uintptr_t>(delta) | reinterpret_cast<uintptr_t>(sum_out);
    if ((bits & 15u) || (reinterpret_cast<uintptr_t>(out_q) & 3u))
        return fail(HIPQ_INVALID_ARGUMENT, "%s: buffers must be 16-byte aligned", fn);
    if (rows >> 31) return fail(HIPQ_SHAPE_ERROR, "%s: too many rows", fn);
    const bool even = (mode & HIPQ_ROUND_HALF_EVEN) != 0;
    // A wavefront per row while the row fits 12 float4 per lane (no workgroup barrier in the row
    // reductions), else the whole workgroup; the register cache is sized to the row.
    const size_t vec_per_wave_lane = (cols / 4 + kWave - 1) / kWave, vec_per_block_lane = (cols / 4 + kRowBlock - 1) / kRowBlock;
#define HIPQ_ROW(TPR, RC, E, S)                                                                                   \
    hipLaunchKernelGGL((row_op_kernel<TPR, RC, OP, QUANT, E, S, ADD>), dim3(row_grid(ctx, rows, kRowBlock / TPR)), \
                       dim3(kRowBlock), 0, ctx->stream, x, delta, sum_out, rows, cols, gamma, beta, eps, out_f, out_q,   \
                       out_scales)
#define HIPQ_ROW_E(TPR, RC)                                                                              \
    do {                                                                                                 \
        const size_t groups = (rows + kRowBlock / TPR - 1) / (kRowBlock / TPR);                          \
        const bool stride = static_cast<size_t>(row_grid(ctx, rows, kRowBlock / TPR)) < groups;          \
        if (even && stride) HIPQ_ROW(TPR, RC, true, true);                                               \
        else if (even) HIPQ_ROW(TPR, RC, true, false);                                                   \
        else if (stride) HIPQ_ROW(TPR, RC, false, true);                                                 \
        else HIPQ_ROW(TPR, RC, false, false);                                                            \
    } while (0)
    if (vec_per_wave_lane <= 4) HIPQ_ROW_E(kWave, 4);
    else if (vec_per_wave_lane <= 8) HIPQ_ROW_E(kWave, 8);
    else if (vec_per_wave_lane <= 12) HIPQ_ROW_E(kWave, 12);
    else if (vec_per_block_lane <= 4) HIPQ_ROW_E(kRowBlock, 4);
    else if (vec_per_block_lane <= 8) HIPQ_ROW_E(kRowBlock, 8);
    else HIPQ_ROW_E(kRowBlock, 12);
#undef HIPQ_ROW_E
#undef HIPQ_ROW
    return check_launch(fn);
}

}  // namespace hipq

using namespace hipq;

extern "C" {

int32_t hipq_layer_norm_f32(hipq_ctx *ctx, const float *x, size_t rows, size_t cols, const float *gamma,
                            const float *beta, float eps, float *out) {
    HIPQ_ENTER(ctx);
    if (rows * cols != 0) {
        HIPQ_REQUIRE_PTR(x);
        HIPQ_REQUIRE_PTR(out);
    }
    return launch_row_op<ROW_LAYERNORM, false>(__func__, ctx, x, rows, cols, gamma, beta, eps, 0, out, nullptr, nullptr);
}

int32_t hipq_layer_norm_quantize_f32_i8(hipq_ctx *ctx, const float *x, size_t rows, size_t cols, const float *gamma,
                                        const float *beta, float eps, int32_t mode, int8_t *out, float *out_scales) {
    HIPQ_ENTER(ctx);
    if (rows * cols != 0) {
        HIPQ_REQUIRE_PTR(x);
        HIPQ_REQUIRE_PTR(out);
        HIPQ_REQUIRE_PTR(out_scales);
    }
    return launch_row_op<ROW_LAYERNORM, true>(__func__, ctx, x, rows, cols, gamma, beta, eps, mode, nullptr, out,
                                              out_scales);
}

int32_t hipq_add_layer_norm_quantize_f32_i8(hipq_ctx *ctx, float *x, const float *delta, size_t rows, size_t cols,
                                            const float *gamma, const float *beta, float eps, int32_t mode,
                                            int8_t *out, float *out_scales) {
    HIPQ_ENTER(ctx);
    if (rows * cols != 0) {
        HIPQ_REQUIRE_PTR(x);
        HIPQ_REQUIRE_PTR(delta);
        HIPQ_REQUIRE_PTR(out);
        HIPQ_REQUIRE_PTR(out_scales);
    }
    return launch_row_op<ROW_LAYERNORM, true, true>(__func__, ctx, x, rows, cols, gamma, beta, eps, mode, nullptr, out,
                                                    out_scales, delta, x);
}

int32_t hipq_gelu_tanh_f32(hipq_ctx *ctx, const float *x, size_t n, float *out) {
    HIPQ_ENTER(ctx);
    if (n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out);
    size_t blocks = (n / 4 + 255) / 256 + 1;
    const size_t cap = size_t(ctx->num_cus) * 16;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(gelu_kernel, dim3(static_cast<int>(blocks)), dim3(256), 0, ctx->stream, x, n, out);
    return check_launch(__func__);
}

int32_t hipq_gelu_tanh_quantize_f32_i8(hipq_ctx *ctx, const float *x, size_t rows, size_t cols, int32_t mode,
                                       int8_t *out, float *out_scales) {
    HIPQ_ENTER(ctx);
    if (rows * cols != 0) {
        HIPQ_REQUIRE_PTR(x);
        HIPQ_REQUIRE_PTR(out);
        HIPQ_REQUIRE_PTR(out_scales);
    }
    return launch_row_op<ROW_GELU, true>(__func__, ctx, x, rows, cols, nullptr, nullptr, 0.0f, mode, nullptr, out,
                                         out_scales);
}

int32_t hipq_add_f32(hipq_ctx *ctx, const float *a, const float *b, size_t n, float *out) {
    HIPQ_ENTER(ctx);
    if (n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(a);
    HIPQ_REQUIRE_PTR(b);
    HIPQ_REQUIRE_PTR(out);
    size_t blocks = (n / 4 + 255) / 256 + 1;
    const size_t cap = size_t(ctx->num_cus) * 16;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(add_kernel, dim3(static_cast<int>(blocks)), dim3(256), 0, ctx->stream, a, b, n, out);
    return check_launch(__func__);
}

}  // extern "C"
