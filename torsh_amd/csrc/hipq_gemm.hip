// int8 x int8 -> int32 GEMM on the CDNA4 matrix cores with fused epilogues:
//   acc[m,n] = sum_k a[m,k] * w[n,k]          (both operands K-contiguous)
// K-tiles of both operands are staged through LDS in 16-byte chunks with an XOR
// swizzle so the 16-byte-per-lane fragment reads of v_mfma_i32_16x16x64_i8 are
// conflict free, global loads for tile t+1 are in flight while tile t is being
// multiplied, and the epilogue (dequantize + bias, or requantize) runs on the
// accumulators in registers.  The weight fragment is the MFMA's row operand so
// that each lane ends up with four consecutive output channels of one
// activation row: 16-byte stores, 16-byte loads of the per-channel scales.

#include <mutex>

#include "hipq_gemm_kernels.h"
#include "hipq_gemm_persist.h"

namespace hipq {

// Epilogue of the skinny kernels: `sum` holds the accumulators of row m and channels
// n_out .. n_out+3.
template <int EPI, bool EVEN>
__device__ __forceinline__ void gemv_store(const GemmEpilogue &ep, v4i sum, int m, int n_out, int M, int N, float4 sw4,
                                           float4 b4, float s_a) {
    if (m >= M || n_out >= N) return;
    const size_t off = size_t(m) * N + n_out;
    constexpr unsigned kAlignMask = (EPI == EPI_I8) ? 3u : 15u;
    const bool vec = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(ep.out) & kAlignMask) == 0);
    if constexpr (EPI == EPI_I32) {
        int32_t *o = static_cast<int32_t *>(ep.out);
        if (vec) {
            *reinterpret_cast<v4i *>(o + off) = sum;
        } else {
            for (int i = 0; i < 4; ++i)
                if (n_out + i < N) o[off + i] = sum[i];
        }
    } else {
        const float swa[4] = {sw4.x, sw4.y, sw4.z, sw4.w}, ba[4] = {b4.x, b4.y, b4.z, b4.w};
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float s = s_a * swa[i];
            v[i] = static_cast<float>(sum[i]) * s;
            if (ep.bias) v[i] = v[i] + ba[i];
        }
        if constexpr (EPI == EPI_F32) {
            float *o = static_cast<float *>(ep.out);
            if (ep.residual)
                for (int i = 0; i < 4; ++i)
                    if (n_out + i < N) v[i] = v[i] + ep.residual[off + i];
            if (vec) {
                *reinterpret_cast<float4 *>(o + off) = make_float4(v[0], v[1], v[2], v[3]);
            } else {
                for (int i = 0; i < 4; ++i)
                    if (n_out + i < N) o[off + i] = v[i];
            }
        } else {
            int8_t *o = static_cast<int8_t *>(ep.out);
            int q[4];
            const float zpf = static_cast<float>(ep.zp_out);
#pragma unroll
            for (int i = 0; i < 4; ++i)
                q[i] = to_int_nan0(clamp_keep_nan(round_mode<EVEN>(div_rn(v[i], ep.s_out, ep.s_out_inv)) + zpf, -128.0f, 127.0f));
            if (vec) {
                *reinterpret_cast<uint32_t *>(o + off) = pack4(q[0], q[1], q[2], q[3]);
            } else {
                for (int i = 0; i < 4; ++i)
                    if (n_out + i < N) o[off + i] = static_cast<int8_t>(q[i]);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Skinny GEMM (M <= 16: decode-shaped Linear).  The weight matrix is read exactly
// once and nothing else matters: 16 weight rows per workgroup, the K range split
// between the four waves, each lane loading 16 bytes of "its" weight row straight
// into the MFMA operand layout (no LDS staging: there is no reuse to stage for).
// Vector-memory loads return in order, so the (L2-resident) activation fragments
// are requested first and all weight loads of the batch follow back to back; the
// MFMAs then run off registers while the next batch is already in flight.  The
// four partial 16x16 accumulators are summed through LDS (integer adds: order
// independent).
template <int G, int EPI, bool EVEN>
__global__ __launch_bounds__(kGemmThreads) void gemv_i8_kernel(const int8_t *__restrict__ A,
                                                               const int8_t *__restrict__ W, int M, int N, int K,
                                                               GemmEpilogue ep) {
    constexpr int NW = kGemmThreads / kWave;
    constexpr int BATCH = 16;  // k-steps of 64 bytes per batch: 16 KiB of weights per wave in flight
    __shared__ v4i red[NW][G][kWave];
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int n0 = blockIdx.x * (16 * G);
    const int frow = lane % 16, g = lane / 16;
    const int kw = K / NW;  // bytes of K per wave, a multiple of 64
    const int kbeg = wave * kw;
    const int mrow = frow < M ? frow : M - 1;
    const int8_t *ap = A + size_t(mrow) * K + kbeg + g * 16;
    const int8_t *wp[G];
#pragma unroll
    for (int r = 0; r < G; ++r) {
        int nrow = n0 + r * 16 + frow;
        nrow = nrow < N ? nrow : N - 1;  // rows past the edge are computed and discarded
        wp[r] = W + size_t(nrow) * K + kbeg + g * 16;
    }
    // Epilogue operands of the wave that will store row group `wave` (requested first, so
    // they are back long before they are needed).
    float4 sw4 = make_float4(1.f, 1.f, 1.f, 1.f), b4 = make_float4(0.f, 0.f, 0.f, 0.f);
    float s_a = 1.0f;
    const int n_out = n0 + wave * 16 + 4 * g;
    if constexpr (EPI != EPI_I32) {
        if (wave < G && n_out < N) {
            const int n1 = n_out + 1 < N ? n_out + 1 : N - 1, n2 = n_out + 2 < N ? n_out + 2 : N - 1,
                      n3 = n_out + 3 < N ? n_out + 3 : N - 1;
            sw4 = make_float4(ep.sw[n_out], ep.sw[n1], ep.sw[n2], ep.sw[n3]);
            if (ep.bias) b4 = make_float4(ep.bias[n_out], ep.bias[n1], ep.bias[n2], ep.bias[n3]);
            s_a = ep.sa_per_row ? ep.sa[mrow] : ep.sa[0];
        }
    }
    v4i acc[G];
#pragma unroll
    for (int r = 0; r < G; ++r) acc[r] = v4i{0, 0, 0, 0};
    for (int k0 = 0; k0 < kw; k0 += BATCH * 64) {
        v4i fa[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
            if (k0 + u * 64 < kw) fa[u] = *reinterpret_cast<const v4i *>(ap + k0 + u * 64);
#pragma unroll
        for (int r = 0; r < G; ++r) {
            v4i fw[BATCH];
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
                if (k0 + u * 64 < kw) fw[u] = *reinterpret_cast<const v4i *>(wp[r] + k0 + u * 64);
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
                if (k0 + u * 64 < kw) acc[r] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fw[u], fa[u], acc[r], 0, 0, 0);
        }
    }
#pragma unroll
    for (int r = 0; r < G; ++r) red[wave][r][lane] = acc[r];
    __syncthreads();
    // Wave r finishes row group r.  D = Wfrag (rows n) x Afrag (cols m): a lane holds
    // m = lane%16 and the four consecutive channels n = 4*(lane/16) + i.
    if (wave >= G) return;
    v4i sum = red[0][wave][lane];
#pragma unroll
    for (int w = 1; w < NW; ++w) sum += red[w][wave][lane];
    gemv_store<EPI, EVEN>(ep, sum, frow, n_out, M, N, sw4, b4, s_a);
}

// Skinny GEMM, LDS-staged form.  Reading weight rows straight into the MFMA operand layout
// makes every wave instruction touch 16 rows with 64 bytes each, and the memory pipeline then
// runs well below what HBM delivers.  Here a wave instruction copies 1 KiB of ONE weight row
// into LDS (global_load_lds, 16 bytes per lane, fully covered 128-byte lines), 16 rows per
// wave, and the MFMA fragments are read back from LDS (row pitch 1040 bytes: conflict free).
// There is still no reuse: LDS is used only to turn the coalesced layout into the operand
// layout.  Each wave owns a 1 KiB slice of K for the 16 rows of the workgroup, so it waits
// only for its own copies (vmcnt), never at a barrier, until the final 4-way sum.
template <int EPI, bool EVEN>
__global__ __launch_bounds__(kGemmThreads) void gemv_i8_lds_kernel(const int8_t *__restrict__ A,
                                                                   const int8_t *__restrict__ W, int M, int N, int K,
                                                                   GemmEpilogue ep) {
    constexpr int NW = kGemmThreads / kWave;
    constexpr int CHUNK = 1024, PITCH = CHUNK + 16, STEPS = CHUNK / 64;
    extern __shared__ __attribute__((aligned(16))) int8_t wlds[];  // [NW][16][PITCH]
    __shared__ v4i red[NW][kWave];
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int n0 = blockIdx.x * 16;
    const int frow = lane % 16, g = lane / 16;
    const int mrow = frow < M ? frow : M - 1;
    int8_t *wbuf = wlds + wave * (16 * PITCH);

    float4 sw4 = make_float4(1.f, 1.f, 1.f, 1.f), b4 = make_float4(0.f, 0.f, 0.f, 0.f);
    float s_a = 1.0f;
    const int n_out = n0 + 4 * g;
    if constexpr (EPI != EPI_I32) {
        if (wave == 0 && n_out < N) {
            const int n1 = n_out + 1 < N ? n_out + 1 : N - 1, n2 = n_out + 2 < N ? n_out + 2 : N - 1,
                      n3 = n_out + 3 < N ? n_out + 3 : N - 1;
            sw4 = make_float4(ep.sw[n_out], ep.sw[n1], ep.sw[n2], ep.sw[n3]);
            if (ep.bias) b4 = make_float4(ep.bias[n_out], ep.bias[n1], ep.bias[n2], ep.bias[n3]);
            s_a = ep.sa_per_row ? ep.sa[mrow] : ep.sa[0];
        }
    }
    v4i acc = v4i{0, 0, 0, 0};
    const int nchunks = (K + CHUNK - 1) / CHUNK;
    for (int c = wave; c < nchunks; c += NW) {
        const int k0 = c * CHUNK;
        const int len = K - k0 < CHUNK ? K - k0 : CHUNK;  // a multiple of 64
        // Activation fragments first (they hit in L2 and loads return in order).
        v4i fa[STEPS];
        const int8_t *ap = A + size_t(mrow) * K + k0 + g * 16;
#pragma unroll
        for (int st = 0; st < STEPS; ++st)
            if (st * 64 < len) fa[st] = *reinterpret_cast<const v4i *>(ap + st * 64);
        asm volatile("" ::: "memory");  // the copies below overwrite what the previous chunk's reads used
        if (lane * 16 < len) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                int nrow = n0 + r;
                nrow = nrow < N ? nrow : N - 1;  // rows past the edge are computed and discarded
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void *)(W + size_t(nrow) * K + k0 + lane * 16),
                    (__attribute__((address_space(3))) void *)(wbuf + r * PITCH), 16, 0, 2 /* nt: streamed once */);
            }
        }
        wait_vmcnt<0>();
        asm volatile("" ::: "memory");
#pragma unroll
        for (int st = 0; st < STEPS; ++st) {
            if (st * 64 < len) {
                const v4i fw = *reinterpret_cast<const v4i *>(wbuf + frow * PITCH + st * 64 + g * 16);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(fw, fa[st], acc, 0, 0, 0);
            }
        }
    }
    red[wave][lane] = acc;
    __syncthreads();
    if (wave != 0) return;
    v4i sum = red[0][lane];
#pragma unroll
    for (int w = 1; w < NW; ++w) sum += red[w][lane];
    gemv_store<EPI, EVEN>(ep, sum, frow, n_out, M, N, sw4, b4, s_a);
}

template <int EPI, bool EVEN>
static int32_t launch_gemv(hipq_ctx *ctx, const int8_t *a, const int8_t *w, int M, int N, int K,
                           const GemmEpilogue &ep) {
    // One weight row group per workgroup measured fastest for every M <= 16 (more row groups
    // per workgroup save activation re-reads from L2 but leave fewer loads in flight).
    // Measured at N = 11008, K = 4096: the direct form is ahead for M <= 4 (11.7 / 12.1 us against
    // 12.0 / 12.5 us), the LDS-staged form for M = 16 (13.9 against 14.8 us).
    if (M <= 4) {
        hipLaunchKernelGGL((gemv_i8_kernel<1, EPI, EVEN>), dim3((N + 15) / 16), dim3(kGemmThreads), 0, ctx->stream, a,
                           w, M, N, K, ep);
        return check_launch("gemv_i8");
    }
    constexpr int kLds = (kGemmThreads / kWave) * 16 * (1024 + 16);
    auto kernel = gemv_i8_lds_kernel<EPI, EVEN>;
    static bool configured[16] = {false};
    if (ctx->device < 16 && !configured[ctx->device]) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
        if (e != hipSuccess)
            return fail(HIPQ_DEVICE_ERROR, "gemv_i8: cannot reserve %d bytes of LDS: %s", kLds, hipGetErrorString(e));
        configured[ctx->device] = true;
    }
    hipLaunchKernelGGL(kernel, dim3((N + 15) / 16), dim3(kGemmThreads), kLds, ctx->stream, a, w, M, N, K, ep);
    return check_launch("gemv_i8 (LDS staged)");
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
                if (ep.residual) v = v + ep.residual[idx];
                static_cast<float *>(ep.out)[idx] = v;
            } else {
                const float q = clamp_keep_nan(round_mode<EVEN>(div_rn(v, ep.s_out, ep.s_out_inv)) + static_cast<float>(ep.zp_out), -128.0f,
                                               127.0f);
                static_cast<int8_t *>(ep.out)[idx] = static_cast<int8_t>(to_int_nan0(q));
            }
        }
    }
}

template <int BM, int BN, int WM, int WN, int EPI, bool EVEN>
static void launch_tile(hipq_ctx *ctx, const int8_t *a, const int8_t *w, int M, int N, int K,
                        const GemmEpilogue &ep) {
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    GemmEpilogue placed = ep;
    pick_xcd_rectangle(tiles_m, tiles_n, BM, BN, &placed.xcd_gm, &placed.xcd_gn);
    hipLaunchKernelGGL((gemm_i8_mfma_kernel<BM, BN, WM, WN, EPI, EVEN>), dim3(tiles_m * tiles_n), dim3(kGemmThreads), 0,
                       ctx->stream, a, w, M, N, K, placed);
}

// Tuning and test hook, per context: HIPQ_GEMM_VARIANT=<n> in the environment (read when the context is
// created), or hipq_set_gemm_kernel_variant(ctx, n), forces one kernel configuration wherever the shape
// allows it (0 = automatic).
static int gemm_variant_override(hipq_ctx *ctx) { return ctx->gemm_variant; }

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
    const size_t cus = static_cast<size_t>(ctx->num_cus);
    auto tiles = [&](size_t bm, size_t bn) { return ((m + bm - 1) / bm) * ((n + bn - 1) / bn); };
    int variant = gemm_variant_override(ctx);
    if (variant == 9 || variant == 11) variant = 0;  // switches of the packed forms only
    if (variant == 0 && M <= 16 && K % 256 == 0) return launch_gemv<EPI, EVEN>(ctx, a, w, M, N, K, ep);
    const bool pipe_ok = (K % 128 == 0) && K >= 256;
    if (variant == 0 && pipe_ok) {
        variant = 2;
        if (tiles(128, 64) >= 2 * cus) {
            // Many more tiles than CUs: the persistent kernel.  Its tile shape is picked with a
            // cost model fitted to measurements: a tile costs nk * L + E cycles, where the main
            // loop is bound by LDS traffic (L per K-tile: fills plus fragment reads) and E is the
            // epilogue of a tile of 4-byte outputs (conversion, transposition through LDS, stores);
            // a workgroup runs ceil(tiles / CUs) tiles.  Bigger tiles move fewer LDS bytes per MAC
            // but quantise worse.  The 256x128 and 128x192 forms have no room for residual values
            // in registers.
            const double nk = double(K / 128), out_scale = (EPI == EPI_I8) ? 0.25 : 1.0;
            auto cost = [&](size_t bm, size_t bn, double L, double E) {
                const size_t t = tiles(bm, bn);
                return double((t + cus - 1) / cus) * (nk * L + E * out_scale);
            };
            const bool with_residual = EPI == EPI_F32 && ep.residual;
            const double c5 = cost(128, 64, 900.0, 2700.0), c6 = cost(128, 128, 1350.0, 4700.0);
            const double c7 = with_residual ? 1e30 : cost(256, 128, 1950.0, 9600.0);
            // 128x192: between the two in LDS bytes per MAC; divides N = 768 and 2304 into whole rounds.
            const double c8 = with_residual ? 1e30 : cost(128, 192, 1600.0, 7200.0);
            variant = (c7 <= c6 && c7 <= c5 && c7 <= c8) ? 7 : (c8 <= c6 && c8 <= c5 ? 8 : (c6 <= c5 ? 6 : 5));
        }
    }
    if (variant == 0 || (variant != 10 && !pipe_ok)) variant = 10;
    switch (variant) {
    case 1: return launch_pipe<128, 64, 6, 4, 1, 1, 4, EPI, EVEN>(ctx, a, w, M, N, K, ep);
    case 2: return launch_pipe<128, 64, 6, 4, 2, 1, 2, EPI, EVEN>(ctx, a, w, M, N, K, ep);
    case 3: return launch_pipe<128, 64, 6, 4, 2, 2, 1, EPI, EVEN>(ctx, a, w, M, N, K, ep);
    case 5: return launch_persist<128, 64, 6, 4, 2, 2, 4, EPI, EVEN>(ctx, a, w, M, N, K, ep);
    case 6: return launch_persist<128, 128, 4, 4, 2, 2, 2, EPI, EVEN>(ctx, a, w, M, N, K, ep);
    case 7:
        if (!(EPI == EPI_F32 && ep.residual)) return launch_persist<256, 128, 3, 4, 2, 2, 1, EPI, EVEN>(ctx, a, w, M, N, K, ep);
        return launch_persist<128, 128, 4, 4, 2, 2, 2, EPI, EVEN>(ctx, a, w, M, N, K, ep);
    case 8:
        if (!(EPI == EPI_F32 && ep.residual)) return launch_persist<128, 192, 3, 4, 2, 2, 1, EPI, EVEN>(ctx, a, w, M, N, K, ep);
        return launch_persist<128, 128, 4, 4, 2, 2, 2, EPI, EVEN>(ctx, a, w, M, N, K, ep);
    default: break;
    }
    // Register-staged kernel: any K that is a multiple of 16.
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
    if (k >= (size_t(1) << 17)) return fail(HIPQ_SHAPE_ERROR, "%s: K=%zu could overflow the int32 accumulator", fn, k);
    return HIPQ_SUCCESS;
}

static int32_t check_linear_dynamic_args(const char *fn, const float *x, const int8_t *w, const float *w_scales,
                                         size_t m, size_t n, size_t k, float *out) {
    int32_t rc = check_gemm_shape(fn, m, n, k);
    if (rc) return rc;
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    if (k == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: Cannot quantize empty tensor", fn);
    if (!x || !w || !w_scales || !out) return fail(HIPQ_INVALID_ARGUMENT, "%s: null pointer", fn);
    return HIPQ_SUCCESS;
}

// Scratch layout of the fused dynamic Linear: header (hipq_qparams), the range-reduction partials,
// per-row scales [m] floats, then the int8 activations [m,k].
static size_t linear_dynamic_partial_bytes(int num_cus) { return size_t(num_cus) * 16 * sizeof(float2); }
static size_t linear_dynamic_scales_bytes(size_t m) { return ((m * sizeof(float)) + 255) & ~size_t(255); }
static size_t linear_dynamic_scratch_bytes(int num_cus, size_t m, size_t k) {
    return kScratchHeader + linear_dynamic_partial_bytes(num_cus) + linear_dynamic_scales_bytes(m) + m * k + 256;
}

// The fused dynamic Linear on a scratch area of linear_dynamic_scratch_bytes() at `base`.  Launches
// kernels only: no allocation, no synchronisation.
static int32_t linear_dynamic_on(hipq_ctx *ctx, char *base, const float *x, int32_t per_token, const int8_t *w,
                                 const float *w_scales, const float *bias, size_t m, size_t n, size_t k, int32_t mode,
                                 float *out) {
    const size_t partial_bytes = linear_dynamic_partial_bytes(ctx->num_cus);
    hipq_qparams *params = reinterpret_cast<hipq_qparams *>(base);
    void *partials = base + kScratchHeader;
    float *row_scales = reinterpret_cast<float *>(base + kScratchHeader + partial_bytes);
    int8_t *qa = reinterpret_cast<int8_t *>(base + kScratchHeader + partial_bytes + linear_dynamic_scales_bytes(m));
    int32_t rc;
    if (per_token) {
        rc = quantize_activations_per_row(ctx, x, m, k, mode & HIPQ_ROUND_HALF_EVEN, qa, row_scales);
        if (rc) return rc;
        return hipq_linear_i8_f32(ctx, qa, row_scales, 1, w, w_scales, bias, m, n, k, out);
    }
    rc = quantize_activations_per_tensor(ctx, x, m, k, true, 1.0f, mode, false, qa, params, partials, partial_bytes);
    if (rc) return rc;
    // hipq_qparams starts with the f32 scale.
    return hipq_linear_i8_f32(ctx, qa, &params->scale, 0, w, w_scales, bias, m, n, k, out);
}

// Scratch of hipq_linear_dynamic_f32_noalloc: device memory that exists from the moment the library is
// loaded, so the entry point never calls an allocator.  Every GPU holds its own copy at its own address;
// host code uses the per-device pointer from hipGetSymbolAddress, never the array's name.
constexpr int kMaxDevices = 64;
constexpr size_t kNoAllocMaxRows = 16384;
constexpr size_t kNoAllocMaxElems = size_t(4) << 20;  // m * k
constexpr size_t kNoAllocBytes = kScratchHeader + 1024 * 16 * sizeof(float2) + kNoAllocMaxRows * sizeof(float) +
                                 kNoAllocMaxElems + 256;
static __device__ __align__(256) unsigned char noalloc_scratch[kNoAllocBytes];
static void *g_noalloc_ptr[kMaxDevices] = {nullptr};
static std::mutex g_noalloc_mutex;

int32_t linear_noalloc_setup(int device) {
    if (device < 0 || device >= kMaxDevices) return HIPQ_SUCCESS;  // the no-alloc entry point reports it
    std::lock_guard<std::mutex> lock(g_noalloc_mutex);
    if (g_noalloc_ptr[device]) return HIPQ_SUCCESS;
    void *p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(noalloc_scratch));
    if (e != hipSuccess || !p)
        return fail(HIPQ_DEVICE_ERROR, "hipGetSymbolAddress(noalloc_scratch) on device %d: %s", device,
                    hipGetErrorString(e));
    g_noalloc_ptr[device] = p;
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

int32_t hipq_linear_i8_f32_residual(hipq_ctx *ctx, const int8_t *a, const float *a_scale, int32_t a_scale_per_row,
                                    const int8_t *w, const float *w_scales, const float *bias, const float *residual,
                                    size_t m, size_t n, size_t k, float *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_gemm_shape(__func__, m, n, k);
    if (rc) return rc;
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(out);
    HIPQ_REQUIRE_PTR(a_scale);
    HIPQ_REQUIRE_PTR(w_scales);
    HIPQ_REQUIRE_PTR(residual);
    if (k > 0) {
        HIPQ_REQUIRE_PTR(a);
        HIPQ_REQUIRE_PTR(w);
    }
    GemmEpilogue ep{a_scale, a_scale_per_row ? 1 : 0, w_scales, bias, 1.0f, 0, out};
    ep.residual = residual;
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
    ep.s_out_inv = host_recip_for_div(out_scale);
    if (mode & HIPQ_ROUND_HALF_EVEN) return launch_gemm<EPI_I8, true>(ctx, a, w, m, n, k, ep);
    return launch_gemm<EPI_I8, false>(ctx, a, w, m, n, k, ep);
}

int32_t hipq_linear_dynamic_f32(hipq_ctx *ctx, const float *x, int32_t per_token, const int8_t *w,
                                const float *w_scales, const float *bias, size_t m, size_t n, size_t k, int32_t mode,
                                float *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_linear_dynamic_args(__func__, x, w, w_scales, m, n, k, out);
    if (rc || m == 0 || n == 0) return rc;
    void *s = nullptr;
    rc = scratch(ctx, linear_dynamic_scratch_bytes(ctx->num_cus, m, k), &s);
    if (rc) return rc;
    return linear_dynamic_on(ctx, static_cast<char *>(s), x, per_token, w, w_scales, bias, m, n, k, mode, out);
}

int32_t hipq_linear_dynamic_f32_noalloc(hipq_ctx *ctx, const float *x, int32_t per_token, const int8_t *w,
                                        const float *w_scales, const float *bias, size_t m, size_t n, size_t k,
                                        int32_t mode, float *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_linear_dynamic_args(__func__, x, w, w_scales, m, n, k, out);
    if (rc || m == 0 || n == 0) return rc;
    if (m > kNoAllocMaxRows || m * k > kNoAllocMaxElems)
        return fail(HIPQ_SHAPE_ERROR,
                    "%s: activations [%zu,%zu] exceed the static scratch (at most %zu rows and %zu elements); "
                    "use hipq_linear_dynamic_f32",
                    __func__, m, k, kNoAllocMaxRows, kNoAllocMaxElems);
    if (ctx->device < 0 || ctx->device >= kMaxDevices || !g_noalloc_ptr[ctx->device])
        return fail(HIPQ_DEVICE_ERROR, "%s: the static scratch of device %d was not set up", __func__, ctx->device);
    if (linear_dynamic_scratch_bytes(ctx->num_cus, m, k) > kNoAllocBytes)
        return fail(HIPQ_SHAPE_ERROR, "%s: scratch layout does not fit the static array", __func__);
    return linear_dynamic_on(ctx, static_cast<char *>(g_noalloc_ptr[ctx->device]), x, per_token, w, w_scales, bias, m,
                             n, k, mode, out);
}

int32_t hipq_linear_static_f32(hipq_ctx *ctx, const float *x, float a_scale, const int8_t *w, const float *w_scales,
                               const float *bias, size_t m, size_t n, size_t k, int32_t mode, float *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_gemm_shape(__func__, m, n, k);
    if (rc) return rc;
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    if (k == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: Cannot quantize empty tensor", __func__);
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(w);
    HIPQ_REQUIRE_PTR(w_scales);
    HIPQ_REQUIRE_PTR(out);
    void *s = nullptr;
    rc = scratch(ctx, kScratchHeader + m * k + 256, &s);
    if (rc) return rc;
    char *base = static_cast<char *>(s);
    hipq_qparams *params = reinterpret_cast<hipq_qparams *>(base);
    int8_t *qa = reinterpret_cast<int8_t *>(base + kScratchHeader);
    rc = quantize_activations_per_tensor(ctx, x, m, k, false, a_scale, mode, false, qa, params, nullptr, 0);
    if (rc) return rc;
    return hipq_linear_i8_f32(ctx, qa, &params->scale, 0, w, w_scales, bias, m, n, k, out);
}

}  // extern "C"
