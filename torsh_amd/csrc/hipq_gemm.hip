// int8 x int8 -> int32 GEMM on the CDNA4 matrix cores with fused epilogues:
//   acc[m,n] = sum_k a[m,k] * w[n,k]          (both operands K-contiguous)
// K-tiles of both operands are staged through LDS in 16-byte chunks with an XOR
// swizzle so the 16-byte-per-lane fragment reads of v_mfma_i32_16x16x64_i8 are
// conflict free, global loads for tile t+1 are in flight while tile t is being
// multiplied, and the epilogue (dequantize + bias, or requantize) runs on the
// accumulators in registers.  The weight fragment is the MFMA's row operand so
// that each lane ends up with four consecutive output channels of one
// activation row: 16-byte stores, 16-byte loads of the per-channel scales.
#include "hipq_internal.h"
#include "hipq_math.h"

namespace hipq {

typedef int v4i __attribute__((ext_vector_type(4)));

enum { EPI_I32 = 0, EPI_F32 = 1, EPI_I8 = 2 };

struct GemmEpilogue {
    const float *sa;    // activation scale(s)
    int sa_per_row;     // 0: sa[0], 1: sa[m]
    const float *sw;    // [N]
    const float *bias;  // [N] or null
    float s_out;        // requantize only
    int zp_out;
    void *out;  // int32 / float / int8 [M,N]
};

constexpr int kGemmThreads = 256;

template <int EPI, bool EVEN>
__device__ __forceinline__ void epilogue_store4(const GemmEpilogue &ep, int m, int n, int N, v4i acc, float s_a) {
    const size_t off = size_t(m) * N + n;
    constexpr unsigned kAlignMask = (EPI == EPI_I8) ? 3u : 15u;
    const bool vec = (N % 4 == 0) && (n + 3 < N) && ((reinterpret_cast<uintptr_t>(ep.out) & kAlignMask) == 0);
    if constexpr (EPI == EPI_I32) {
        int32_t *o = static_cast<int32_t *>(ep.out);
        if (vec) {
            *reinterpret_cast<v4i *>(o + off) = acc;
        } else {
            for (int r = 0; r < 4; ++r)
                if (n + r < N) o[off + r] = acc[r];
        }
    } else {
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int nn = (n + r < N) ? n + r : N - 1;
            const float s = s_a * ep.sw[nn];
            float t = static_cast<float>(acc[r]) * s;
            if (ep.bias) t = t + ep.bias[nn];
            v[r] = t;
        }
        if constexpr (EPI == EPI_F32) {
            float *o = static_cast<float *>(ep.out);
            if (vec) {
                *reinterpret_cast<float4 *>(o + off) = make_float4(v[0], v[1], v[2], v[3]);
            } else {
                for (int r = 0; r < 4; ++r)
                    if (n + r < N) o[off + r] = v[r];
            }
        } else {
            int8_t *o = static_cast<int8_t *>(ep.out);
            int q[4];
            const float zpf = static_cast<float>(ep.zp_out);
#pragma unroll
            for (int r = 0; r < 4; ++r)
                q[r] = to_int_nan0(clamp_keep_nan(round_mode<EVEN>(v[r] / ep.s_out) + zpf, -128.0f, 127.0f));
            if (vec) {
                *reinterpret_cast<uint32_t *>(o + off) = pack4(q[0], q[1], q[2], q[3]);
            } else {
                for (int r = 0; r < 4; ++r)
                    if (n + r < N) o[off + r] = static_cast<int8_t>(q[r]);
            }
        }
    }
}

// Maps the linear workgroup id to a tile so that the workgroups one XCD receives
// (ids congruent modulo 8) cover a contiguous band of weight panels: a panel of
// W is then pulled from HBM into one XCD's L2 only.
__device__ __forceinline__ void tile_of_block(int tiles_m, int tiles_n, int *tm, int *tn) {
    const int nblk = tiles_m * tiles_n;
    int b = blockIdx.x;
    if (nblk % 8 == 0) b = (b % 8) * (nblk / 8) + b / 8;
    *tm = b % tiles_m;
    *tn = b / tiles_m;
}

// BM x BN output tile per workgroup, BK = 128 bytes of K per stage, WM x WN
// waves each owning a (BM/WM) x (BN/WN) sub-tile.
template <int BM, int BN, int WM, int WN, int EPI, bool EVEN>
__global__ __launch_bounds__(kGemmThreads) void gemm_i8_mfma_kernel(const int8_t *__restrict__ A,
                                                                     const int8_t *__restrict__ W, int M, int N,
                                                                     int K, GemmEpilogue ep) {
    constexpr int BK = 128;
    constexpr int CPR = BK / 16;  // 16-byte chunks per tile row
    static_assert(WM * WN * kWave == kGemmThreads, "wave grid must use the whole workgroup");
    constexpr int TM = BM / WM, TN = BN / WN;
    constexpr int FM = TM / 16, FN = TN / 16;
    static_assert(TM % 16 == 0 && TN % 16 == 0, "wave tile is made of 16x16 MFMA blocks");
    constexpr int A_CHUNKS = BM * CPR, W_CHUNKS = BN * CPR;
    static_assert(A_CHUNKS % kGemmThreads == 0 && W_CHUNKS % kGemmThreads == 0, "tile loads divide evenly");
    constexpr int A_PER_T = A_CHUNKS / kGemmThreads, W_PER_T = W_CHUNKS / kGemmThreads;
    constexpr int STAGE = (BM + BN) * BK;

    __shared__ __attribute__((aligned(16))) int8_t lds[2 * STAGE];

    int tile_m, tile_n;
    tile_of_block((M + BM - 1) / BM, (N + BN - 1) / BN, &tile_m, &tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const int wm = wave % WM, wn = wave / WM;

    v4i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = v4i{0, 0, 0, 0};

    v4i ra[A_PER_T], rw[W_PER_T];
    const v4i zero = v4i{0, 0, 0, 0};

    auto load_global = [&](int k0) {
#pragma unroll
        for (int i = 0; i < A_PER_T; ++i) {
            const int c = tid + i * kGemmThreads;
            const int row = c / CPR, col = c % CPR;
            const int gm = m0 + row, gk = k0 + col * 16;
            ra[i] = (gm < M && gk < K) ? *reinterpret_cast<const v4i *>(A + size_t(gm) * K + gk) : zero;
        }
#pragma unroll
        for (int i = 0; i < W_PER_T; ++i) {
            const int c = tid + i * kGemmThreads;
            const int row = c / CPR, col = c % CPR;
            const int gn = n0 + row, gk = k0 + col * 16;
            rw[i] = (gn < N && gk < K) ? *reinterpret_cast<const v4i *>(W + size_t(gn) * K + gk) : zero;
        }
    };
    auto store_lds = [&](int stage) {
        int8_t *sa = lds + stage * STAGE;
        int8_t *sw = sa + BM * BK;
#pragma unroll
        for (int i = 0; i < A_PER_T; ++i) {
            const int c = tid + i * kGemmThreads;
            const int row = c / CPR, col = c % CPR;
            *reinterpret_cast<v4i *>(sa + row * BK + ((col ^ (row & (CPR - 1))) * 16)) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < W_PER_T; ++i) {
            const int c = tid + i * kGemmThreads;
            const int row = c / CPR, col = c % CPR;
            *reinterpret_cast<v4i *>(sw + row * BK + ((col ^ (row & (CPR - 1))) * 16)) = rw[i];
        }
    };

    const int nk = (K + BK - 1) / BK;
    load_global(0);
    store_lds(0);
    __syncthreads();

    const int frow = lane % 16, fcol = lane / 16;
    for (int kt = 0; kt < nk; ++kt) {
        if (kt + 1 < nk) load_global((kt + 1) * BK);
        const int8_t *sa = lds + (kt & 1) * STAGE;
        const int8_t *sw = sa + BM * BK;
#pragma unroll
        for (int ks = 0; ks < BK / 64; ++ks) {
            v4i fa[FM], fw[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                const int row = wm * TM + i * 16 + frow;
                const int col = ks * 4 + fcol;
                fa[i] = *reinterpret_cast<const v4i *>(sa + row * BK + ((col ^ (row & (CPR - 1))) * 16));
            }
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const int row = wn * TN + j * 16 + frow;
                const int col = ks * 4 + fcol;
                fw[j] = *reinterpret_cast<const v4i *>(sw + row * BK + ((col ^ (row & (CPR - 1))) * 16));
            }
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fw[j], fa[i], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) store_lds((kt + 1) & 1);
        __syncthreads();
    }

    // D = Wfrag (rows: n) x Afrag (cols: m): lane holds m = lane%16, n = 4*(lane/16)+r.
#pragma unroll
    for (int i = 0; i < FM; ++i) {
        const int m = m0 + wm * TM + i * 16 + (lane % 16);
        if (m >= M) continue;
        float s_a = 1.0f;
        if constexpr (EPI != EPI_I32) s_a = ep.sa_per_row ? ep.sa[m] : ep.sa[0];
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const int n = n0 + wn * TN + j * 16 + 4 * (lane / 16);
            if (n >= N) continue;
            epilogue_store4<EPI, EVEN>(ep, m, n, N, acc[i][j], s_a);
        }
    }
}

// Any shape, any alignment: one thread per output, plain integer dot product.
// Used when K is not a multiple of 16 or an operand is not 16-byte aligned.
template <int EPI, bool EVEN>
__global__ __launch_bounds__(kGemmThreads) void gemm_i8_generic_kernel(const int8_t *__restrict__ A,
                                                                        const int8_t *__restrict__ W, int M, int N,
                                                                        int K, GemmEpilogue ep) {
    const size_t total = size_t(M) * N;
    for (size_t idx = size_t(blockIdx.x) * kGemmThreads + threadIdx.x; idx < total;
         idx += size_t(gridDim.x) * kGemmThreads) {
        const int m = static_cast<int>(idx / N), n = static_cast<int>(idx % N);
        const int8_t *a = A + size_t(m) * K, *w = W + size_t(n) * K;
        int acc = 0;
        for (int k = 0; k < K; ++k) acc += static_cast<int>(a[k]) * static_cast<int>(w[k]);
        if constexpr (EPI == EPI_I32) {
            static_cast<int32_t *>(ep.out)[idx] = acc;
        } else {
            const float s = (ep.sa_per_row ? ep.sa[m] : ep.sa[0]) * ep.sw[n];
            float v = static_cast<float>(acc) * s;
            if (ep.bias) v = v + ep.bias[n];
            if constexpr (EPI == EPI_F32) {
                static_cast<float *>(ep.out)[idx] = v;
            } else {
                const float q = clamp_keep_nan(round_mode<EVEN>(v / ep.s_out) + static_cast<float>(ep.zp_out), -128.0f,
                                               127.0f);
                static_cast<int8_t *>(ep.out)[idx] = static_cast<int8_t>(to_int_nan0(q));
            }
        }
    }
}

template <int BM, int BN, int WM, int WN, int EPI, bool EVEN>
static void launch_tile(hipq_ctx *ctx, const int8_t *a, const int8_t *w, int M, int N, int K,
                        const GemmEpilogue &ep) {
    const int tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    hipLaunchKernelGGL((gemm_i8_mfma_kernel<BM, BN, WM, WN, EPI, EVEN>), dim3(tiles), dim3(kGemmThreads), 0,
                       ctx->stream, a, w, M, N, K, ep);
}

template <int EPI, bool EVEN>
static int32_t launch_gemm(hipq_ctx *ctx, const int8_t *a, const int8_t *w, size_t m, size_t n, size_t k,
                           const GemmEpilogue &ep) {
    const int M = static_cast<int>(m), N = static_cast<int>(n), K = static_cast<int>(k);
    const bool fast = (K % 16 == 0) && ((reinterpret_cast<uintptr_t>(a) & 15u) == 0) &&
                      ((reinterpret_cast<uintptr_t>(w) & 15u) == 0);
    if (!fast) {
        size_t blocks = (m * n + kGemmThreads - 1) / kGemmThreads;
        const size_t cap = size_t(ctx->num_cus) * 8;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL((gemm_i8_generic_kernel<EPI, EVEN>), dim3(static_cast<int>(blocks)), dim3(kGemmThreads), 0,
                           ctx->stream, a, w, M, N, K, ep);
        return check_launch("gemm_i8 (generic)");
    }
    // Tile choice: the largest tile that still gives every CU a workgroup.
    const size_t cus = static_cast<size_t>(ctx->num_cus);
    auto tiles = [&](size_t bm, size_t bn) { return ((m + bm - 1) / bm) * ((n + bn - 1) / bn); };
    if (tiles(128, 128) >= 2 * cus)
        launch_tile<128, 128, 2, 2, EPI, EVEN>(ctx, a, w, M, N, K, ep);
    else if (tiles(128, 64) >= cus || m > 64)
        launch_tile<128, 64, 2, 2, EPI, EVEN>(ctx, a, w, M, N, K, ep);
    else
        launch_tile<64, 64, 2, 2, EPI, EVEN>(ctx, a, w, M, N, K, ep);
    return check_launch("gemm_i8");
}

static int32_t check_gemm_shape(const char *fn, size_t m, size_t n, size_t k) {
    if ((m >> 30) || (n >> 30) || (k >> 30)) return fail(HIPQ_SHAPE_ERROR, "%s: dimension too large", fn);
    // |acc| <= K * 128 * 128 must fit int32.
    if (k > (size_t(1) << 17)) return fail(HIPQ_SHAPE_ERROR, "%s: K=%zu could overflow the int32 accumulator", fn, k);
    return HIPQ_SUCCESS;
}

}  // namespace hipq

using namespace hipq;

extern "C" {

int32_t hipq_gemm_i8_i32(hipq_ctx *ctx, const int8_t *a, const int8_t *w, size_t m, size_t n, size_t k,
                         int32_t *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_gemm_shape(__func__, m, n, k);
    if (rc) return rc;
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(out);
    if (k > 0) {
        HIPQ_REQUIRE_PTR(a);
        HIPQ_REQUIRE_PTR(w);
    }
    GemmEpilogue ep{nullptr, 0, nullptr, nullptr, 1.0f, 0, out};
    return launch_gemm<EPI_I32, false>(ctx, a, w, m, n, k, ep);
}

int32_t hipq_linear_i8_f32(hipq_ctx *ctx, const int8_t *a, const float *a_scale, int32_t a_scale_per_row,
                           const int8_t *w, const float *w_scales, const float *bias, size_t m, size_t n, size_t k,
                           float *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_gemm_shape(__func__, m, n, k);
    if (rc) return rc;
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(out);
    HIPQ_REQUIRE_PTR(a_scale);
    HIPQ_REQUIRE_PTR(w_scales);
    if (k > 0) {
        HIPQ_REQUIRE_PTR(a);
        HIPQ_REQUIRE_PTR(w);
    }
    GemmEpilogue ep{a_scale, a_scale_per_row ? 1 : 0, w_scales, bias, 1.0f, 0, out};
    return launch_gemm<EPI_F32, false>(ctx, a, w, m, n, k, ep);
}

int32_t hipq_linear_i8_i8(hipq_ctx *ctx, const int8_t *a, const float *a_scale, int32_t a_scale_per_row,
                          const int8_t *w, const float *w_scales, const float *bias, size_t m, size_t n, size_t k,
                          float out_scale, int32_t out_zero_point, int32_t mode, int8_t *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_gemm_shape(__func__, m, n, k);
    if (rc) return rc;
    if (out_scale <= 0.0f) return fail(HIPQ_INVALID_ARGUMENT, "%s: Scale must be positive", __func__);
    if (mode & ~(HIPQ_ROUND_HALF_EVEN | HIPQ_FORM_DIV)) return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown mode bits", __func__);
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(out);
    HIPQ_REQUIRE_PTR(a_scale);
    HIPQ_REQUIRE_PTR(w_scales);
    if (k > 0) {
        HIPQ_REQUIRE_PTR(a);
        HIPQ_REQUIRE_PTR(w);
    }
    GemmEpilogue ep{a_scale, a_scale_per_row ? 1 : 0, w_scales, bias, out_scale, out_zero_point, out};
    if (mode & HIPQ_ROUND_HALF_EVEN) return launch_gemm<EPI_I8, true>(ctx, a, w, m, n, k, ep);
    return launch_gemm<EPI_I8, false>(ctx, a, w, m, n, k, ep);
}

int32_t hipq_linear_dynamic_f32(hipq_ctx *ctx, const float *x, int32_t per_token, const int8_t *w,
                                const float *w_scales, const float *bias, size_t m, size_t n, size_t k, int32_t mode,
                                float *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_gemm_shape(__func__, m, n, k);
    if (rc) return rc;
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    if (k == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: Cannot quantize empty tensor", __func__);
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(w);
    HIPQ_REQUIRE_PTR(w_scales);
    HIPQ_REQUIRE_PTR(out);
    // Scratch layout after the header: per-row scales [m] floats, then int8 activations [m,k].
    const size_t scales_bytes = ((m * sizeof(float)) + 255) & ~size_t(255);
    // The range-reduction partials live at the start of the bulk area; keep clear of them.
    const size_t partial_bytes = size_t(ctx->num_cus) * 16 * sizeof(float2);
    void *s = nullptr;
    rc = scratch(ctx, kScratchHeader + partial_bytes + scales_bytes + m * k + 256, &s);
    if (rc) return rc;
    char *base = static_cast<char *>(s);
    hipq_qparams *params = reinterpret_cast<hipq_qparams *>(base);
    float *row_scales = reinterpret_cast<float *>(base + kScratchHeader + partial_bytes);
    int8_t *qa = reinterpret_cast<int8_t *>(base + kScratchHeader + partial_bytes + scales_bytes);
    if (per_token) {
        rc = hipq_quantize_per_row_f32_i8(ctx, x, m, k, HIPQ_PARAMS_SYMMETRIC, mode & HIPQ_ROUND_HALF_EVEN, qa,
                                          row_scales, nullptr, nullptr);
        if (rc) return rc;
        return hipq_linear_i8_f32(ctx, qa, row_scales, 1, w, w_scales, bias, m, n, k, out);
    }
    rc = hipq_quantize_dynamic_per_tensor_f32(ctx, x, m * k, HIPQ_PARAMS_SYMMETRIC, HIPQ_DTYPE_I8, mode, qa, params);
    if (rc) return rc;
    // hipq_qparams starts with the f32 scale.
    return hipq_linear_i8_f32(ctx, qa, &params->scale, 0, w, w_scales, bias, m, n, k, out);
}

}  // extern "C"
