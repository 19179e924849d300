// Quantized elementwise operators of the backend trait: qadd and qrelu
// (crates/torsh-backend/src/quantization/ops.rs:582-624).  The reference dequantizes its operands
// to f32 vectors, applies the operator, takes the range of the result, derives the output
// parameters from it and quantizes: five passes over f32 data.  Here the f32 result is never
// stored: pass 1 recomputes it from the bytes and reduces its range, pass 2 derives the
// parameters (every workgroup folds the few hundred range partials itself), recomputes the result
// and quantizes it.  Traffic per element: qadd 2 + 2 + 1 bytes, qrelu 1 + 1 + 1.
#include "hipq_internal.h"
#include "hipq_math.h"

namespace hipq {

constexpr int kQBlock = 256;
constexpr int kQInFlight = 2;  // 16-byte loads per operand in flight per lane (16 elements each)

struct QOperand {
    const uint8_t *q;
    float scale;
    int zp;
    int is_signed;  // bytes are two's-complement int8 (crates/torsh-backend/src/quantization/tensor.rs:103-143)
};

// dequantize_value, ops.rs:198-200: scale * (q - zp) as f32
__device__ __forceinline__ float deq(uint32_t byte, const QOperand &p) {
    const int v = p.is_signed ? static_cast<int>(static_cast<int8_t>(byte)) : static_cast<int>(byte);
    return p.scale * static_cast<float>(v - p.zp);
}

// The f32 value the reference would hold for element `byte(s)`.
template <bool ADD>
__device__ __forceinline__ float op_value(uint32_t a, uint32_t b, const QOperand &pa, const QOperand &pb) {
    if constexpr (ADD)
        return deq(a, pa) + deq(b, pb);  // ops.rs:592-596
    else
        return fmaxf(deq(a, pa), 0.0f);  // ops.rs:610
}

// Walks n bytes: 16 at a time through f16(uint4 a, uint4 b, vec index), the rest through f1.
template <bool ADD, typename F16, typename F1>
__device__ __forceinline__ void stream_bytes(const uint8_t *__restrict__ a, const uint8_t *__restrict__ b, size_t n,
                                             bool extra_aligned, F16 f16, F1 f1) {
    const bool aligned = extra_aligned && ((reinterpret_cast<uintptr_t>(a) & 15u) == 0) &&
                         (!ADD || (reinterpret_cast<uintptr_t>(b) & 15u) == 0);
    const size_t nvec = aligned ? n / 16 : 0;
    const uint4 *a4 = reinterpret_cast<const uint4 *>(a);
    const uint4 *b4 = reinterpret_cast<const uint4 *>(b);
    constexpr int kTile = kQBlock * kQInFlight;
    const size_t ntiles = (nvec + kTile - 1) / kTile;
    for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const size_t base = t * kTile + threadIdx.x;
        uint4 va[kQInFlight], vb[kQInFlight];
#pragma unroll
        for (int i = 0; i < kQInFlight; ++i) {
            const size_t idx = base + size_t(i) * kQBlock;
            if (idx < nvec) {
                va[i] = a4[idx];
                if constexpr (ADD) vb[i] = b4[idx];
            }
        }
#pragma unroll
        for (int i = 0; i < kQInFlight; ++i) {
            const size_t idx = base + size_t(i) * kQBlock;
            if (idx < nvec) f16(va[i], ADD ? vb[i] : va[i], idx);
        }
    }
    for (size_t i = nvec * 16 + size_t(blockIdx.x) * kQBlock + threadIdx.x; i < n; i += size_t(gridDim.x) * kQBlock)
        f1(a[i], ADD ? b[i] : a[i], i);
}

__device__ __forceinline__ uint32_t byte_of(const uint4 &v, int i) {
    const uint32_t w = i < 4 ? v.x : (i < 8 ? v.y : (i < 12 ? v.z : v.w));
    return (w >> (8 * (i & 3))) & 0xffu;
}

__device__ __forceinline__ float2 block_minmax2(float mn, float mx) {
    __shared__ float lds[2 * kQBlock / kWave];
    mn = wave_min(mn);
    mx = wave_max(mx);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    constexpr int nw = kQBlock / kWave;
    __syncthreads();
    if (lane == 0) {
        lds[wave] = mn;
        lds[nw + wave] = mx;
    }
    __syncthreads();
    float rmn = lds[0], rmx = lds[nw];
#pragma unroll
    for (int w = 1; w < nw; ++w) {
        rmn = fminf(rmn, lds[w]);
        rmx = fmaxf(rmx, lds[nw + w]);
    }
    return make_float2(rmn, rmx);
}

// Pass 1: range of the operator's f32 result (folds from +inf / -inf with f32::min / f32::max,
// ops.rs:600-601, 612).
template <bool ADD>
__global__ __launch_bounds__(kQBlock) void qop_range_kernel(QOperand pa, QOperand pb, size_t n,
                                                             float2 *__restrict__ partials) {
    float mn = INFINITY, mx = -INFINITY;
    stream_bytes<ADD>(
        pa.q, pb.q, n, true,
        [&](const uint4 &va, const uint4 &vb, size_t) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float v = op_value<ADD>(byte_of(va, i), byte_of(vb, i), pa, pb);
                mn = fminf(mn, v);
                mx = fmaxf(mx, v);
            }
        },
        [&](uint8_t a, uint8_t b, size_t) {
            const float v = op_value<ADD>(a, b, pa, pb);
            mn = fminf(mn, v);
            mx = fmaxf(mx, v);
        });
    const float2 r = block_minmax2(mn, mx);
    if (threadIdx.x == 0) partials[blockIdx.x] = r;
}

// Pass 2: output parameters from the folded range (from_statistics, params.rs:282-363, through
// `flavor`), then clamp(round(v / scale) + zp) as a byte (quantize_value, ops.rs:185-195).
template <bool ADD>
__global__ __launch_bounds__(kQBlock) void qop_quantize_kernel(QOperand pa, QOperand pb, size_t n,
                                                                const float2 *__restrict__ partials, int nparts,
                                                                int flavor, int qmin, int qmax,
                                                                uint8_t *__restrict__ out,
                                                                hipq_qparams *__restrict__ out_params) {
    float mn = INFINITY, mx = -INFINITY;
    for (int i = threadIdx.x; i < nparts; i += kQBlock) {
        const float2 p = partials[i];
        mn = fminf(mn, p.x);
        mx = fmaxf(mx, p.y);
    }
    float2 r = block_minmax2(mn, mx);
    if constexpr (!ADD) {  // qrelu: from_statistics(0.0, max_val.max(0.0)), ops.rs:612-615
        r.x = 0.0f;
        r.y = fmaxf(r.y, 0.0f);
    }
    float scale;
    int zp;
    const int st = params_from_minmax(r.x, r.y, flavor, qmin, qmax, &scale, &zp);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        out_params->scale = scale;
        out_params->zero_point = zp;
        out_params->min_val = r.x;
        out_params->max_val = r.y;
        out_params->status = st;
    }
    if (st != HIPQ_SUCCESS) return;
    const float inv = recip_for_div(scale), zpf = static_cast<float>(zp);
    auto quant = [&](uint32_t a, uint32_t b) {
        return static_cast<uint32_t>(quantize_int<true, false>(op_value<ADD>(a, b, pa, pb), scale, inv, zpf, qmin, qmax)) &
               0xffu;
    };
    const bool out_aligned = (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
    stream_bytes<ADD>(
        pa.q, pb.q, n, out_aligned,
        [&](const uint4 &va, const uint4 &vb, size_t idx) {
            uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < 16; ++i) w[i / 4] |= quant(byte_of(va, i), byte_of(vb, i)) << (8 * (i & 3));
            reinterpret_cast<uint4 *>(out)[idx] = make_uint4(w[0], w[1], w[2], w[3]);
        },
        [&](uint8_t a, uint8_t b, size_t i) { out[i] = static_cast<uint8_t>(quant(a, b)); });
}

template <bool ADD>
static int32_t run_qop(const char *fn, hipq_ctx *ctx, const QOperand &pa, const QOperand &pb, size_t n, int32_t flavor,
                       int32_t out_dtype, uint8_t *out, hipq_qparams *out_params) {
    if (flavor != HIPQ_PARAMS_BACKEND_SYMMETRIC && flavor != HIPQ_PARAMS_BACKEND_ASYMMETRIC)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: flavor must be HIPQ_PARAMS_BACKEND_SYMMETRIC or _ASYMMETRIC", fn);
    if (out_dtype != HIPQ_DTYPE_I8 && out_dtype != HIPQ_DTYPE_U8)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: output dtype must be HIPQ_DTYPE_I8 or HIPQ_DTYPE_U8", fn);
    if (!out_params) return fail(HIPQ_INVALID_ARGUMENT, "%s: null pointer 'out_params'", fn);
    if (n == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: the range of an empty tensor is not finite", fn);
    if (!pa.q || (ADD && !pb.q) || !out) return fail(HIPQ_INVALID_ARGUMENT, "%s: null data pointer", fn);
    const int qmin = out_dtype == HIPQ_DTYPE_I8 ? -128 : 0, qmax = out_dtype == HIPQ_DTYPE_I8 ? 127 : 255;
    const size_t per_tile = size_t(kQBlock) * kQInFlight * 16;
    const size_t tiles = (n + per_tile - 1) / per_tile;
    const size_t cap = static_cast<size_t>(ctx->num_cus) * 4;
    const int grid = static_cast<int>(tiles < cap ? tiles : cap);
    void *scr = nullptr;
    int32_t rc = scratch(ctx, kScratchHeader + cap * sizeof(float2), &scr);
    if (rc != HIPQ_SUCCESS) return rc;
    float2 *partials = reinterpret_cast<float2 *>(static_cast<char *>(scr) + kScratchHeader);
    qop_range_kernel<ADD><<<grid, kQBlock, 0, ctx->stream>>>(pa, pb, n, partials);
    if ((rc = check_launch("qop_range_kernel")) != HIPQ_SUCCESS) return rc;
    qop_quantize_kernel<ADD><<<grid, kQBlock, 0, ctx->stream>>>(pa, pb, n, partials, grid, flavor, qmin, qmax, out,
                                                                 out_params);
    return check_launch("qop_quantize_kernel");
}

}  // namespace hipq

using namespace hipq;

extern "C" {

int32_t hipq_qadd_u8(hipq_ctx *ctx, const uint8_t *a, int32_t a_signed, float a_scale, int32_t a_zero_point,
                     const uint8_t *b, int32_t b_signed, float b_scale, int32_t b_zero_point, size_t n,
                     int32_t flavor, int32_t out_dtype, uint8_t *out, hipq_qparams *out_params) {
    HIPQ_ENTER(ctx);
    const QOperand pa{a, a_scale, a_zero_point, a_signed ? 1 : 0}, pb{b, b_scale, b_zero_point, b_signed ? 1 : 0};
    return run_qop<true>(__func__, ctx, pa, pb, n, flavor, out_dtype, out, out_params);
}

int32_t hipq_qrelu_u8(hipq_ctx *ctx, const uint8_t *q, int32_t is_signed, float scale, int32_t zero_point, size_t n,
                      int32_t flavor, int32_t out_dtype, uint8_t *out, hipq_qparams *out_params) {
    HIPQ_ENTER(ctx);
    const QOperand pa{q, scale, zero_point, is_signed ? 1 : 0};
    return run_qop<false>(__func__, ctx, pa, pa, n, flavor, out_dtype, out, out_params);
}

}  // extern "C"
