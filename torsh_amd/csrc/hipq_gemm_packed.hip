// Entry points of the fragment-packed int8 GEMM / Linear forward (kernels: hipq_gemm_packed.h).
//
// Weights are packed once when a layer is prepared (hipq_pack_rows_i8: the "MFMA-friendly tile
// order" of a prepared weight blob); activations are written in the packed layout by the quantize
// pass itself, so the forward costs no extra pass over either operand.
#include "hipq_gemm_packed.h"
#include "hipq_gemm_rows.h"
#include "hipq_conv_patch.h"

namespace hipq {

static int32_t check_packed_shape(const char *fn, size_t m, size_t n, size_t k) {
    if ((m >> 30) || (n >> 30) || (k >> 30)) return fail(HIPQ_SHAPE_ERROR, "%s: dimension too large", fn);
    // |acc| <= K * 128 * 128 must fit int32.
    if (k >= (size_t(1) << 17)) return fail(HIPQ_SHAPE_ERROR, "%s: K=%zu could overflow the int32 accumulator", fn, k);
    // fragment offsets are 32-bit
    if (packed_bytes(m, k) >= (size_t(1) << 31) || packed_bytes(n, k) >= (size_t(1) << 31))
        return fail(HIPQ_SHAPE_ERROR, "%s: a packed operand of 2 GiB or more is not supported", fn);
    return HIPQ_SUCCESS;
}

int32_t pack_rows(hipq_ctx *ctx, const int8_t *src, size_t rows, size_t k, int8_t *dst) {
    const size_t nfrag = packed_row_blocks(rows) * packed_k_blocks(k);
    size_t blocks = (nfrag + 3) / 4;
    const size_t cap = size_t(ctx->num_cus) * 16;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(pack_rows_i8_kernel, dim3(static_cast<int>(blocks)), dim3(256), 0, ctx->stream, src, rows, k, k,
                       dst);
    return check_launch("pack_rows_i8");
}

// Scratch of the fused forward: header (hipq_qparams), range partials, per-row scales, the packed activations.
struct PackedScratch {
    size_t partials, scales, packed, total;
};
static PackedScratch packed_scratch_layout(int num_cus, size_t m, size_t k) {
    PackedScratch L;
    auto up = [](size_t v) { return (v + 255) & ~size_t(255); };
    L.partials = kScratchHeader;
    L.scales = L.partials + up(size_t(num_cus) * 16 * sizeof(float2));
    L.packed = L.scales + up(m * sizeof(float));
    L.total = L.packed + up(packed_bytes(m, k)) + 256;
    return L;
}

size_t packed_operand_bytes(size_t rows, size_t k) { return packed_bytes(rows, k); }

// The pair form relies on the dispatcher handing workgroup ids b and b + 8 to one XCD.  Asked of the device once:
// a grid of one workgroup per compute unit records the XCD each workgroup ran on.
bool pairs_share_an_xcd(hipq_ctx *ctx) {
    static int known[16] = {0};  // 1 = yes, -1 = no
    if (ctx->device < 0 || ctx->device >= 16) return false;
    if (known[ctx->device] == 0) {
        int verdict = -1;
        const int n = ctx->num_cus;
        uint32_t *dev = nullptr;
        if (n >= 16 && n <= 4096 && hipMalloc(reinterpret_cast<void **>(&dev), size_t(n) * 4) == hipSuccess) {
            uint32_t host[4096];
            hipLaunchKernelGGL(xcc_probe_kernel, dim3(n), dim3(64), 0, ctx->stream, dev);
            if (hipGetLastError() == hipSuccess && hipStreamSynchronize(ctx->stream) == hipSuccess &&
                hipMemcpy(host, dev, size_t(n) * 4, hipMemcpyDeviceToHost) == hipSuccess) {
                verdict = 1;
                for (int b = 8; b < n; ++b)
                    if (host[b] != host[b - 8]) verdict = -1;
            }
            (void)hipFree(dev);
        }
        known[ctx->device] = verdict;
    }
    return known[ctx->device] > 0;
}

// Implicit-GEMM convolution on the packed kernel: picks the register depth (the largest of 4, 3, 2, 1 that
// divides the k blocks per wave) and the epilogue.
template <int EPI, bool EVEN>
static int32_t launch_conv_packed(hipq_ctx *ctx, const int8_t *filters, const int8_t *image, int M, int N, int K,
                                  const GemmEpilogue &ep) {
    const int steps = static_cast<int>(packed_k_blocks(size_t(K))) / 4;
    if constexpr (EPI == EPI_I8 && !EVEN) {
        // Phase stamps (hipq_ctx_set_trace_buffer): the depth-3 requantizing form only.
        const size_t tiles = ((packed_row_blocks(size_t(M)) + 3) / 4) * ((packed_row_blocks(size_t(N)) + 1) / 2);
        if (ctx->trace && steps % 4 != 0 && steps % 3 == 0 &&
            ctx->trace_bytes >= tiles * 4 * kTraceWords * sizeof(unsigned long long))
            return launch_packed<4, 2, 3, EPI, EVEN, true, true>(ctx, filters, image, M, N, K, ep);
    }
    if (steps % 4 == 0) return launch_packed<4, 2, 4, EPI, EVEN, false, true>(ctx, filters, image, M, N, K, ep);
    if (steps % 3 == 0) return launch_packed<4, 2, 3, EPI, EVEN, false, true>(ctx, filters, image, M, N, K, ep);
    if (steps % 2 == 0) return launch_packed<4, 2, 2, EPI, EVEN, false, true>(ctx, filters, image, M, N, K, ep);
    return launch_packed<4, 2, 1, EPI, EVEN, false, true>(ctx, filters, image, M, N, K, ep);
}

int32_t conv_gemm_packed(hipq_ctx *ctx, const int8_t *filters, const int8_t *image, int M, int N, int K,
                         const GemmEpilogue &ep, int epi, bool even) {
    if (epi == EPI_I32) return launch_conv_packed<EPI_I32, false>(ctx, filters, image, M, N, K, ep);
    if (epi == EPI_F32) return launch_conv_packed<EPI_F32, false>(ctx, filters, image, M, N, K, ep);
    if (even) return launch_conv_packed<EPI_I8, true>(ctx, filters, image, M, N, K, ep);
    return launch_conv_packed<EPI_I8, false>(ctx, filters, image, M, N, K, ep);
}

bool conv_patch_applicable(int nb, int c, int h, int w, int hp, int wp, int kh, int kw) {
    int patch = 0, lds_bytes = 0;
    return conv_patch_fits(c, h, w, hp, wp, kh, kw, static_cast<long long>(nb) * hp * wp, &patch, &lds_bytes);
}

template <int CBS>
static int32_t conv_patch_dispatch(hipq_ctx *ctx, const int8_t *filters, int M, int N, int K, const GemmEpilogue &ep,
                                   const ConvPatch &cp, int lds_bytes, int epi, bool even) {
    if (epi == EPI_I32) return launch_conv_patch<CBS, EPI_I32, false>(ctx, filters, M, N, K, ep, cp, lds_bytes);
    if (epi == EPI_F32) return launch_conv_patch<CBS, EPI_F32, false>(ctx, filters, M, N, K, ep, cp, lds_bytes);
    if (even) return launch_conv_patch<CBS, EPI_I8, true>(ctx, filters, M, N, K, ep, cp, lds_bytes);
    if (ctx->trace) return launch_conv_patch<CBS, EPI_I8, false, true>(ctx, filters, M, N, K, ep, cp, lds_bytes);
    return launch_conv_patch<CBS, EPI_I8, false>(ctx, filters, M, N, K, ep, cp, lds_bytes);
}

int32_t conv_gemm_patch(hipq_ctx *ctx, const int8_t *filters, const uint8_t *x, size_t x_bytes, int zp_in, int h, int w,
                        int ph, int pw, int kh, int M, int N, int K, const GemmEpilogue &ep, int epi, bool even) {
    int patch = 0, lds_bytes = 0;
    if (!conv_patch_fits(ep.cv_c, h, w, ep.cv_hp, ep.cv_wp, kh, ep.cv_kw, N, &patch, &lds_bytes) ||
        x_bytes >= (size_t(1) << 31) || (reinterpret_cast<uintptr_t>(x) & 3u))
        return fail(HIPQ_SHAPE_ERROR, "conv2d (patch): geometry not taken by this form");
    const uint32_t b = static_cast<uint32_t>(zp_in ^ 0x80) & 0xffu;
    const ConvPatch cp{x, h, w, ph, pw, kh, patch, b * 0x01010101u, static_cast<int>(x_bytes),
                       1.0f / static_cast<float>(ep.cv_hp * ep.cv_wp), 1.0f / static_cast<float>(ep.cv_wp)};
    if (ep.cv_c == 128) return conv_patch_dispatch<4>(ctx, filters, M, N, K, ep, cp, lds_bytes, epi, even);
    return conv_patch_dispatch<8>(ctx, filters, M, N, K, ep, cp, lds_bytes, epi, even);
}

}  // namespace hipq

using namespace hipq;

extern "C" {

int32_t hipq_packed_size(size_t rows, size_t k, size_t *out_bytes) {
    HIPQ_REQUIRE_PTR(out_bytes);
    if ((rows >> 30) || (k >> 30)) return fail(HIPQ_SHAPE_ERROR, "%s: dimension too large", __func__);
    *out_bytes = packed_bytes(rows, k);
    return HIPQ_SUCCESS;
}

int32_t hipq_pack_rows_i8(hipq_ctx *ctx, const int8_t *src, size_t rows, size_t k, int8_t *dst_packed) {
    HIPQ_ENTER(ctx);
    if ((rows >> 30) || (k >> 30)) return fail(HIPQ_SHAPE_ERROR, "%s: dimension too large", __func__);
    if (rows == 0 || k == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(src);
    HIPQ_REQUIRE_PTR(dst_packed);
    if (reinterpret_cast<uintptr_t>(dst_packed) & 15u)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: the packed buffer must be 16-byte aligned", __func__);
    return pack_rows(ctx, src, rows, k, dst_packed);
}

int32_t hipq_gemm_packed_i8_i32(hipq_ctx *ctx, const int8_t *a_packed, const int8_t *w_packed, size_t m, size_t n,
                                size_t k, int32_t *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_packed_shape(__func__, m, n, k);
    if (rc) return rc;
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    if (k == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: K must be positive", __func__);
    HIPQ_REQUIRE_PTR(out);
    HIPQ_REQUIRE_PTR(a_packed);
    HIPQ_REQUIRE_PTR(w_packed);
    GemmEpilogue ep{nullptr, 0, nullptr, nullptr, 1.0f, 0, out};
    return launch_gemm_packed<EPI_I32, false>(ctx, a_packed, w_packed, m, n, k, ep);
}

// The GEMM launch of hipq_linear_packed_i8_f32 (arguments already checked); `fresh`: a_packed was written by the
// kernel launched just before on this stream.
static int32_t linear_packed_launch(hipq_ctx *ctx, const int8_t *a_packed, const float *a_scale,
                                    int32_t a_scale_per_row, const int8_t *w_packed, const float *w_scales,
                                    const float *bias, size_t m, size_t n, size_t k, float *out, bool fresh) {
    GemmEpilogue ep{a_scale, a_scale_per_row ? 1 : 0, w_scales, bias, 1.0f, 0, out};
    ep.fresh_activations = fresh ? 1 : 0;
    return launch_gemm_packed<EPI_F32, false>(ctx, a_packed, w_packed, m, n, k, ep);
}

int32_t hipq_linear_packed_i8_f32(hipq_ctx *ctx, const int8_t *a_packed, const float *a_scale,
                                  int32_t a_scale_per_row, const int8_t *w_packed, const float *w_scales,
                                  const float *bias, size_t m, size_t n, size_t k, float *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_packed_shape(__func__, m, n, k);
    if (rc) return rc;
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    if (k == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: K must be positive", __func__);
    HIPQ_REQUIRE_PTR(out);
    HIPQ_REQUIRE_PTR(a_scale);
    HIPQ_REQUIRE_PTR(w_scales);
    HIPQ_REQUIRE_PTR(a_packed);
    HIPQ_REQUIRE_PTR(w_packed);
    return linear_packed_launch(ctx, a_packed, a_scale, a_scale_per_row, w_packed, w_scales, bias, m, n, k, out, false);
}

int32_t hipq_linear_packed_i8_i8(hipq_ctx *ctx, const int8_t *a_packed, const float *a_scale, int32_t a_scale_per_row,
                                 const int8_t *w_packed, const float *w_scales, const float *bias, size_t m, size_t n,
                                 size_t k, float out_scale, int32_t out_zero_point, int32_t mode, int8_t *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_packed_shape(__func__, m, n, k);
    if (rc) return rc;
    if (out_scale <= 0.0f) return fail(HIPQ_INVALID_ARGUMENT, "%s: Scale must be positive", __func__);
    if (mode & ~(HIPQ_ROUND_HALF_EVEN | HIPQ_FORM_DIV)) return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown mode bits", __func__);
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    if (k == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: K must be positive", __func__);
    HIPQ_REQUIRE_PTR(out);
    HIPQ_REQUIRE_PTR(a_scale);
    HIPQ_REQUIRE_PTR(w_scales);
    HIPQ_REQUIRE_PTR(a_packed);
    HIPQ_REQUIRE_PTR(w_packed);
    GemmEpilogue ep{a_scale, a_scale_per_row ? 1 : 0, w_scales, bias, out_scale, out_zero_point, out};
    ep.s_out_inv = host_recip_for_div(out_scale);
    if (mode & HIPQ_ROUND_HALF_EVEN) return launch_gemm_packed<EPI_I8, true>(ctx, a_packed, w_packed, m, n, k, ep);
    return launch_gemm_packed<EPI_I8, false>(ctx, a_packed, w_packed, m, n, k, ep);
}

int32_t hipq_quantize_per_tensor_packed_f32_i8(hipq_ctx *ctx, const float *x, size_t rows, size_t cols,
                                               int32_t dynamic, float scale, int32_t mode, int8_t *out_packed,
                                               hipq_qparams *out_params) {
    HIPQ_ENTER(ctx);
    if ((rows >> 30) || (cols >> 30)) return fail(HIPQ_SHAPE_ERROR, "%s: dimension too large", __func__);
    if (rows == 0 || cols == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: Cannot quantize empty tensor", __func__);
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out_packed);
    HIPQ_REQUIRE_PTR(out_params);
    if (reinterpret_cast<uintptr_t>(out_packed) & 15u)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: the packed buffer must be 16-byte aligned", __func__);
    return quantize_activations_per_tensor(ctx, x, rows, cols, dynamic != 0, scale, mode, true, out_packed, out_params,
                                           nullptr, 0);
}

int32_t hipq_quantize_per_row_packed_f32_i8(hipq_ctx *ctx, const float *x, size_t rows, size_t cols, int32_t mode,
                                            int8_t *out_packed, float *out_scales) {
    HIPQ_ENTER(ctx);
    if ((rows >> 30) || (cols >> 30)) return fail(HIPQ_SHAPE_ERROR, "%s: dimension too large", __func__);
    if (rows == 0 || cols == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: Cannot quantize empty tensor", __func__);
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out_packed);
    HIPQ_REQUIRE_PTR(out_scales);
    if (reinterpret_cast<uintptr_t>(out_packed) & 15u)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: the packed buffer must be 16-byte aligned", __func__);
    if (mode & ~HIPQ_ROUND_HALF_EVEN) return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown mode bits", __func__);
    return quantize_activations_per_row(ctx, x, rows, cols, mode, out_packed, out_scales, /*packed=*/true);
}

// Which lines of the packed weights the GEMM's workgroups of each die read, for the activation quantizer to touch
// while its grid waits for the range (WarmLines).  With the 128 x 64 tiles dealt to the dies as rectangles that span
// all row tiles (pick_xcd_rectangle), die d owns a run of consecutive weight row blocks: one contiguous slice of
// the packed matrix.  The sibling tiles of a weight panel start their K loops a quarter of K apart, so the lines
// read first are the runs behind those starts; half of each quarter is asked for.  Measured at M = 512,
// N = K = 4096 on three machines: GEMM -0.6 to -1.5 us, quantizer +0.2 to +1.0 us, the step -0.2 to -0.5 us with
// half of the lines; all of them gave -0.1 to -0.8 us, a quarter -0.1 to -0.6 us.  Only where a die's slice is at
// most half of its 4 MiB L2 and the tiles make one round over the compute units; variant 11 switches it off.
static void set_weight_warming(hipq_ctx *ctx, const int8_t *w_packed, size_t m, size_t n, size_t k) {
    ctx->warm = WarmLines{};
    const size_t rbW = packed_row_blocks(n), KB = packed_k_blocks(k);
    // (few rows, or few 64 x 64 tiles: the weight-streaming kernel runs, not the 128 x 64 tiles this is laid out for)
    if (ctx->gemm_variant == 11 || m <= 64 || ((packed_row_blocks(m) + 1) / 2) * ((rbW + 1) / 2) <= size_t(ctx->num_cus))
        return;
    const size_t tiles_m = (packed_row_blocks(m) + 3) / 4, tiles_n = (rbW + 1) / 2;
    if (tiles_m * tiles_n > size_t(ctx->num_cus) || rbW % 2 != 0 || KB % 32 != 0) return;
    int gm = 0, gn = 0;
    pick_xcd_rectangle(static_cast<int>(tiles_m), static_cast<int>(tiles_n), 128, 64, &gm, &gn);
    if (gm != static_cast<int>(tiles_m)) return;
    const size_t die_row_blocks = size_t(gn) * 2;
    if (die_row_blocks * KB * 1024 > (size_t(2) << 20)) return;
    WarmLines w;
    w.base = reinterpret_cast<const uint32_t *>(w_packed);
    w.row_block_lines = static_cast<uint32_t>(KB * 8);  // 1 KiB per k block
    w.die_stride_lines = static_cast<uint32_t>(die_row_blocks) * w.row_block_lines;
    w.starts = static_cast<uint32_t>(tiles_m < 4 ? tiles_m : 4);
    w.start_step_lines = w.row_block_lines / 4;
    w.run_lines = w.start_step_lines / 2;
    w.lines = static_cast<uint32_t>(die_row_blocks) * w.starts * w.run_lines;
    ctx->warm = w;
}

int32_t hipq_linear_dynamic_packed_f32(hipq_ctx *ctx, const float *x, int32_t per_token, const int8_t *w_packed,
                                       const float *w_scales, const float *bias, size_t m, size_t n, size_t k,
                                       int32_t mode, float *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_packed_shape(__func__, m, n, k);
    if (rc) return rc;
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    if (k == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: Cannot quantize empty tensor", __func__);
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(w_packed);
    HIPQ_REQUIRE_PTR(w_scales);
    HIPQ_REQUIRE_PTR(out);
    const PackedScratch L = packed_scratch_layout(ctx->num_cus, m, k);
    void *s = nullptr;
    rc = scratch(ctx, L.total, &s);
    if (rc) return rc;
    char *base = static_cast<char *>(s);
    hipq_qparams *params = reinterpret_cast<hipq_qparams *>(base);
    float *row_scales = reinterpret_cast<float *>(base + L.scales);
    int8_t *pa = reinterpret_cast<int8_t *>(base + L.packed);
    if (per_token) {
        // Decode, one or two rows: one launch, every workgroup quantizes the rows itself (variant 6 keeps the two).
        if (m <= 2 && ctx->gemm_variant != 6) {
            GemmEpilogue ep{nullptr, 1, w_scales, bias, 1.0f, 0, out};
            const bool fused = (mode & HIPQ_ROUND_HALF_EVEN)
                                   ? launch_gemv_packed_from_f32<true, false>(ctx, x, w_packed, m, n, k, ep, 0, &rc)
                                   : launch_gemv_packed_from_f32<false, false>(ctx, x, w_packed, m, n, k, ep, 0, &rc);
            if (fused) return rc;
        }
        // one pass over the activations: the per-row quantizer writes the packed operand itself
        rc = quantize_activations_per_row(ctx, x, m, k, mode & HIPQ_ROUND_HALF_EVEN, pa, row_scales, /*packed=*/true);
        if (rc) return rc;
        return linear_packed_launch(ctx, pa, row_scales, 1, w_packed, w_scales, bias, m, n, k, out, true);
    }
    set_weight_warming(ctx, w_packed, m, n, k);
    rc = quantize_activations_per_tensor(ctx, x, m, k, true, 1.0f, mode, true, pa, params, base + L.partials,
                                         L.scales - L.partials);
    ctx->warm = WarmLines{};
    if (rc) return rc;
    return linear_packed_launch(ctx, pa, &params->scale, 0, w_packed, w_scales, bias, m, n, k, out, true);
}

int32_t hipq_linear_static_packed_f32(hipq_ctx *ctx, const float *x, float a_scale, const int8_t *w_packed,
                                      const float *w_scales, const float *bias, size_t m, size_t n, size_t k,
                                      int32_t mode, float *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_packed_shape(__func__, m, n, k);
    if (rc) return rc;
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    if (k == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: Cannot quantize empty tensor", __func__);
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(w_packed);
    HIPQ_REQUIRE_PTR(w_scales);
    HIPQ_REQUIRE_PTR(out);
    // Decode, up to four rows: one launch, every workgroup quantizes the rows itself (variant 6 keeps the two).  A
    // scale or mode that is not valid goes on to the quantizer below, which says so.
    if (m <= 4 && ctx->gemm_variant != 6 && a_scale > 0.0f && !(mode & ~(HIPQ_ROUND_HALF_EVEN | HIPQ_FORM_DIV))) {
        GemmEpilogue ep{nullptr, 0, w_scales, bias, 1.0f, 0, out};
        ep.sa_scalar = a_scale;
        const int div = (mode & HIPQ_FORM_DIV) ? 1 : 0;
        const bool fused = (mode & HIPQ_ROUND_HALF_EVEN)
                               ? launch_gemv_packed_from_f32<true, true>(ctx, x, w_packed, m, n, k, ep, div, &rc)
                               : launch_gemv_packed_from_f32<false, true>(ctx, x, w_packed, m, n, k, ep, div, &rc);
        if (fused) return rc;
    }
    const PackedScratch L = packed_scratch_layout(ctx->num_cus, m, k);
    void *s = nullptr;
    rc = scratch(ctx, L.total, &s);
    if (rc) return rc;
    char *base = static_cast<char *>(s);
    hipq_qparams *params = reinterpret_cast<hipq_qparams *>(base);
    int8_t *pa = reinterpret_cast<int8_t *>(base + L.packed);
    rc = quantize_activations_per_tensor(ctx, x, m, k, false, a_scale, mode, true, pa, params, nullptr, 0);
    if (rc) return rc;
    return linear_packed_launch(ctx, pa, &params->scale, 0, w_packed, w_scales, bias, m, n, k, out, true);
}

// ---- row-panel forms: a workgroup owns 32 whole rows of the output (hipq_gemm_rows.h) -------------------------

static int32_t check_rows_args(const char *fn, hipq_ctx *ctx, size_t m, size_t n, size_t k) {
    int32_t rc = check_packed_shape(fn, m, n, k);
    if (rc) return rc;
    if (k == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: K must be positive", fn);
    (void)ctx;
    return HIPQ_SUCCESS;
}

int32_t hipq_linear_rows_packed_i8_f32(hipq_ctx *ctx, const int8_t *a_packed, const float *a_scale, int32_t a_scale_per_row,
                                       const int8_t *w_packed, const float *w_scales, const float *bias, size_t m,
                                       size_t n, size_t k, float *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_rows_args(__func__, ctx, m, n, k);
    if (rc) return rc;
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(a_packed);
    HIPQ_REQUIRE_PTR(a_scale);
    HIPQ_REQUIRE_PTR(w_packed);
    HIPQ_REQUIRE_PTR(w_scales);
    HIPQ_REQUIRE_PTR(out);
    RowPanel p{a_packed, a_scale, a_scale_per_row ? 1 : 0, w_packed, w_scales, bias, static_cast<int>(m),
               static_cast<int>(n), static_cast<int>(k), out, nullptr, nullptr, nullptr, nullptr, 0.0f};
    return launch_rows<RP_F32>(ctx, p, false);
}

int32_t hipq_linear_gelu_quantize_packed_i8(hipq_ctx *ctx, const int8_t *a_packed, const float *a_scale,
                                            int32_t a_scale_per_row, const int8_t *w_packed, const float *w_scales,
                                            const float *bias, size_t m, size_t n, size_t k, int32_t mode,
                                            int8_t *out_packed, float *out_scales) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_rows_args(__func__, ctx, m, n, k);
    if (rc) return rc;
    if (mode & ~HIPQ_ROUND_HALF_EVEN) return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown mode bits", __func__);
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(a_packed);
    HIPQ_REQUIRE_PTR(a_scale);
    HIPQ_REQUIRE_PTR(w_packed);
    HIPQ_REQUIRE_PTR(w_scales);
    HIPQ_REQUIRE_PTR(out_packed);
    HIPQ_REQUIRE_PTR(out_scales);
    RowPanel p{a_packed, a_scale, a_scale_per_row ? 1 : 0, w_packed, w_scales, bias, static_cast<int>(m),
               static_cast<int>(n), static_cast<int>(k), nullptr, out_packed, out_scales, nullptr, nullptr, 0.0f};
    return launch_rows<RP_GELU_Q>(ctx, p, (mode & HIPQ_ROUND_HALF_EVEN) != 0);
}

int32_t hipq_linear_residual_layer_norm_quantize_packed_i8(hipq_ctx *ctx, const int8_t *a_packed, const float *a_scale,
                                                           int32_t a_scale_per_row, const int8_t *w_packed,
                                                           const float *w_scales, const float *bias, size_t m, size_t n,
                                                           size_t k, float *x, const float *gamma, const float *beta,
                                                           float eps, int32_t mode, int8_t *out_packed,
                                                           float *out_scales) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_rows_args(__func__, ctx, m, n, k);
    if (rc) return rc;
    if (mode & ~HIPQ_ROUND_HALF_EVEN) return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown mode bits", __func__);
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(a_packed);
    HIPQ_REQUIRE_PTR(a_scale);
    HIPQ_REQUIRE_PTR(w_packed);
    HIPQ_REQUIRE_PTR(w_scales);
    HIPQ_REQUIRE_PTR(x);
    RowPanel p{a_packed, a_scale, a_scale_per_row ? 1 : 0, w_packed, w_scales, bias, static_cast<int>(m),
               static_cast<int>(n), static_cast<int>(k), x, out_packed, out_scales, gamma, beta, eps};
    if (!out_packed) return launch_rows<RP_RESID_F32>(ctx, p, false);  // no LayerNorm to feed: x += product only
    HIPQ_REQUIRE_PTR(out_scales);
    return launch_rows<RP_RESID_LN_Q>(ctx, p, (mode & HIPQ_ROUND_HALF_EVEN) != 0);
}

int32_t hipq_linear_from_f32_residual_layer_norm_quantize_packed_i8(hipq_ctx *ctx, const float *a, size_t lda,
                                                                    const int8_t *w_packed, const float *w_scales,
                                                                    const float *bias, size_t m, size_t n, size_t k,
                                                                    float *x, const float *gamma, const float *beta,
                                                                    float eps, int32_t mode, int8_t *out_packed,
                                                                    float *out_scales) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_rows_args(__func__, ctx, m, n, k);
    if (rc) return rc;
    if (mode & ~HIPQ_ROUND_HALF_EVEN) return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown mode bits", __func__);
    if (lda >= (size_t(1) << 31)) return fail(HIPQ_SHAPE_ERROR, "%s: row pitch %zu is too large", __func__, lda);
    if (m == 0 || n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(a);
    HIPQ_REQUIRE_PTR(w_packed);
    HIPQ_REQUIRE_PTR(w_scales);
    HIPQ_REQUIRE_PTR(x);
    RowPanel p{nullptr, nullptr, 1, w_packed, w_scales, bias, static_cast<int>(m), static_cast<int>(n),
               static_cast<int>(k), x, out_packed, out_scales, gamma, beta, eps, a, static_cast<int>(lda)};
    const bool even = (mode & HIPQ_ROUND_HALF_EVEN) != 0;
    if (!out_packed) return launch_rows_from_f32<RP_RESID_F32>(ctx, p, even);
    HIPQ_REQUIRE_PTR(out_scales);
    return launch_rows_from_f32<RP_RESID_LN_Q>(ctx, p, even);
}

}  // extern "C"
