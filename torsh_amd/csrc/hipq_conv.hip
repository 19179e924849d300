// Quantized Conv2d forward: u8 activations (NCHW) x per-channel int8 filters ->
// int32 accumulators -> requantized int8 (NCHW), bias fused.
//
// Fast path (stride 1, channels a multiple of 32): an im2col-free implicit GEMM on the
// fragment-packed MFMA kernel (hipq_gemm_packed.h, CONV).  The activations are rewritten
// once as signed bytes (x - 128) in a zero-point-padded image stored as
// [channel block of 32][pixel][32 bytes]: consecutive pixels of one channel block are 32
// bytes apart, so the 32 windows of an MFMA fragment, shifted by any filter tap, are one
// contiguous KiB that a wave loads with a single coalesced instruction, straight into the
// operand registers (no LDS, no gather).  The filters are packed once in the GEMM's
// fragment order with K = (tap, channel).  Shifting by 128 lets the signed int8 MFMA
// multiply unsigned activations; the shift and the zero point are undone in the epilogue
// with the per-filter weight sum:  sum (x - zp) w = sum (x - 128) w + (128 - zp) sum w,
// and a border pixel holds exactly zp so padded taps contribute nothing.
// Everything else runs through a direct per-output kernel (correct, not fast).
#include "hipq_gemm_kernels.h"
#include "hipq_meeting.h"

namespace hipq {

constexpr int kConvThreads = 256;

// u8 NCHW -> i8 [channel block][padded pixel][32] with a border of `pad` pixels holding (zp - 128); pixel
// index = (n * hp + y) * wp + x, `pixels` of them per channel block (the real ones, then zeroed slack that
// the last windows read into).  One thread per (channel block, padded pixel): it reads its pixel's byte from
// each of the block's 32 channel planes (consecutive lanes are consecutive pixels: consecutive bytes of a
// plane row), all 32 loads in flight at once, and writes the 32 bytes as two 16-byte stores (a wave writes
// 2 KiB contiguous).  x - 128 on a byte is a flip of its top bit.  No LDS.  The last cbs workgroups clear
// the slack.  C % 32 == 0.
__global__ __launch_bounds__(kConvThreads) void conv_pack_image_kernel(const uint8_t *__restrict__ x, int C, int H, int W,
                                                                         int pad_h, int pad_w, int zp,
                                                                         const int32_t *__restrict__ zp_dev, int nb,
                                                                         int groups_per_cb, int8_t *__restrict__ out,
                                                                         int pixels) {
    if (zp_dev) zp = *zp_dev;  // the zero point a dynamic quantize has left on the device
    const int hp = H + 2 * pad_h, wp = W + 2 * pad_w, cbs = C / 32;
    const int real_pixels = nb * hp * wp;
    const int work = cbs * groups_per_cb;
    if (static_cast<int>(blockIdx.x) >= work) {
        const int cb = blockIdx.x - work;
        uint4 *tail = reinterpret_cast<uint4 *>(out + (size_t(cb) * pixels + real_pixels) * 32);
        for (int i = threadIdx.x; i < (pixels - real_pixels) * 2; i += kConvThreads) tail[i] = make_uint4(0, 0, 0, 0);
        return;
    }
    const int cb = blockIdx.x / groups_per_cb;
    const int p = (blockIdx.x % groups_per_cb) * kConvThreads + threadIdx.x;  // padded pixel of the whole batch
    if (p >= real_pixels) return;
    const int n = p / (hp * wp), rem = p % (hp * wp);
    const int h = rem / wp - pad_h, w = rem % wp - pad_w;
    const uint32_t border4 = static_cast<uint32_t>(static_cast<uint8_t>(zp - 128)) * 0x01010101u;
    uint32_t d[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) d[i] = border4;
    if (h >= 0 && h < H && w >= 0 && w < W) {
        const size_t plane = size_t(H) * W;
        const uint8_t *src = x + ((size_t(n) * C + cb * 32) * H + h) * W + w;
        uint32_t b[32];
#pragma unroll
        for (int c = 0; c < 32; ++c) b[c] = src[size_t(c) * plane];
#pragma unroll
        for (int i = 0; i < 8; ++i)
            d[i] = (b[4 * i] | (b[4 * i + 1] << 8) | (b[4 * i + 2] << 16) | (b[4 * i + 3] << 24)) ^ 0x80808080u;
    }
    uint4 *dst = reinterpret_cast<uint4 *>(out + (size_t(cb) * pixels + p) * 32);
    dst[0] = make_uint4(d[0], d[1], d[2], d[3]);
    dst[1] = make_uint4(d[4], d[5], d[6], d[7]);
}

// The same image from fp32 activations, quantized on the way: per-tensor uint8 with parameters from the
// tensor's own range (flavor; codes 0..255).  A thread keeps the 32 channel values of its pixel in registers
// while the grid agrees on the range (hipq_meeting.h), quantizes them, and writes the 32 bytes; the border holds
// zp - 128 with the zero point just agreed on.  The input is read once and no uint8 copy of it is ever written.
// Workgroup 0 publishes the parameters in out_params for the convolution kernel that follows.  The caller
// guarantees that the grid can be resident at once.
template <bool DIV, int RND>
__global__ __launch_bounds__(kConvThreads, 4) void conv_quantize_pack_image_kernel(
    const float *__restrict__ x, int C, int H, int W, int pad_h, int pad_w, int flavor, int nb, int groups_per_cb,
    hipq_qparams *out_params, uint32_t *words, int spin_limit, int8_t *__restrict__ out, int pixels,
    const uint32_t *__restrict__ touch, uint32_t touch_lines) {
    __shared__ float lds[kMeetingLdsFloats];
    const int hp = H + 2 * pad_h, wp = W + 2 * pad_w, cbs = C / 32;
    const int real_pixels = nb * hp * wp;
    const int work = cbs * groups_per_cb;
    const bool slack = static_cast<int>(blockIdx.x) >= work;
    const int cb = slack ? blockIdx.x - work : blockIdx.x / groups_per_cb;
    const int p = (blockIdx.x % groups_per_cb) * kConvThreads + threadIdx.x;  // padded pixel of the whole batch
    bool inside = false;
    float v[32];
    if (!slack && p < real_pixels) {
        const int n = p / (hp * wp), rem = p % (hp * wp);
        const int h = rem / wp - pad_h, w = rem % wp - pad_w;
        if (h >= 0 && h < H && w >= 0 && w < W) {
            inside = true;
            const size_t plane = size_t(H) * W;
            const float *src = x + ((size_t(n) * C + cb * 32) * H + h) * W + w;
#pragma unroll
            for (int c = 0; c < 32; ++c) v[c] = src[size_t(c) * plane];
        }
    }
    const uint32_t gen = meeting_number(words);  // behind the data in program order: returned after it
    MinMax m{INFINITY, -INFINITY};
    if (inside) {
#pragma unroll
        for (int c = 0; c < 32; ++c) {
            m.mn = fminf(m.mn, v[c]);
            m.mx = fmaxf(m.mx, v[c]);
        }
    }
    const MinMax r = block_minmax(m, lds);
    if (slack) {
        // These workgroups only clear the slack behind the image: they take part in the meeting with a range
        // that changes nothing and do not wait for its result.
        meeting_publish_range(words, gen, r);
        uint4 *tail = reinterpret_cast<uint4 *>(out + (size_t(cb) * pixels + real_pixels) * 32);
        for (int i = threadIdx.x; i < (pixels - real_pixels) * 2; i += kConvThreads) tail[i] = make_uint4(0, 0, 0, 0);
        return;
    }
    // While the grid agrees on the range: one load per 128-byte line of the prepared filters, which every die's
    // workgroups of the convolution kernel read first thing (workgroups are dealt to the dies in turn, there as
    // here), by the waves that do not poll.  The values are not used.
    uint32_t touched = 0;
    if (touch_lines && threadIdx.x >= kWave && blockIdx.x != 0) {
        const uint32_t sharers = (work + 7 - blockIdx.x % 8) / 8, warmers = kConvThreads - kWave;
        for (uint32_t i = (blockIdx.x / 8) * warmers + (threadIdx.x - kWave); i < touch_lines; i += sharers * warmers)
            touched ^= touch[size_t(i) * 32];
    }
    const MeetingParams agreed = meet_on_range(words, gen, r, flavor, 0, 255, /*poison=*/true, spin_limit, lds, out_params);
    asm volatile("" ::"v"(touched));
    if (p >= real_pixels) return;
    const bool bad = agreed.scale != agreed.scale;
    const float scale = bad ? INFINITY : agreed.scale;  // x / inf: every code is the zero point
    const int zp = agreed.zero_point;
    const float inv = DIV ? recip_for_div(scale) : 1.0f / scale;
    const float zpf = static_cast<float>(zp);
    const uint32_t border4 = static_cast<uint32_t>(static_cast<uint8_t>(zp - 128)) * 0x01010101u;
    uint32_t d[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) d[i] = border4;
    if (inside) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            d[i] = pack4(quantize_int<DIV, RND>(v[4 * i], scale, inv, zpf, 0, 255),
                         quantize_int<DIV, RND>(v[4 * i + 1], scale, inv, zpf, 0, 255),
                         quantize_int<DIV, RND>(v[4 * i + 2], scale, inv, zpf, 0, 255),
                         quantize_int<DIV, RND>(v[4 * i + 3], scale, inv, zpf, 0, 255)) ^
                   0x80808080u;
    }
    uint4 *dst = reinterpret_cast<uint4 *>(out + (size_t(cb) * pixels + p) * 32);
    dst[0] = make_uint4(d[0], d[1], d[2], d[3]);
    dst[1] = make_uint4(d[4], d[5], d[6], d[7]);
}

// int8 [OC, IC, KH*KW] -> [OC, KH*KW, IC] and wsum[oc] = sum of the filter's weights.
__global__ __launch_bounds__(kConvThreads) void conv_pack_weights_kernel(const int8_t *__restrict__ w, int IC, int taps,
                                                                           int8_t *__restrict__ packed,
                                                                           int32_t *__restrict__ wsum) {
    __shared__ int part[kConvThreads / kWave];
    const int oc = blockIdx.x;
    const size_t base = size_t(oc) * IC * taps;
    int s = 0;
    for (int i = threadIdx.x; i < IC * taps; i += kConvThreads) {
        const int t = i / IC, c = i % IC;  // destination order
        const int8_t v = w[base + size_t(c) * taps + t];
        packed[base + i] = v;
        s += v;
    }
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, kWave);
    if (threadIdx.x % kWave == 0) part[threadIdx.x / kWave] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        int t = 0;
        for (int i = 0; i < kConvThreads / kWave; ++i) t += part[i];
        wsum[oc] = t;
    }
}

struct ConvGeom {
    int nb, c, h, w, oc, kh, kw, sh, sw, ph, pw, ho, wo;
};

// Direct convolution, one thread per output: acc = sum over valid taps (x - zp_in) * w.
template <int EPI, bool EVEN>
__global__ __launch_bounds__(kConvThreads) void conv_direct_kernel(const uint8_t *__restrict__ x, int zp_in,
                                                                    const int8_t *__restrict__ w, ConvGeom g,
                                                                    float s_in, const float *__restrict__ sw,
                                                                    const float *__restrict__ bias, float s_out,
                                                                    int zp_out, void *__restrict__ out) {
    const size_t total = size_t(g.nb) * g.oc * g.ho * g.wo;
    for (size_t idx = size_t(blockIdx.x) * kConvThreads + threadIdx.x; idx < total;
         idx += size_t(gridDim.x) * kConvThreads) {
        const int ow = static_cast<int>(idx % g.wo);
        const int oh = static_cast<int>((idx / g.wo) % g.ho);
        const int oc = static_cast<int>((idx / (size_t(g.wo) * g.ho)) % g.oc);
        const int n = static_cast<int>(idx / (size_t(g.wo) * g.ho * g.oc));
        int acc = 0;
        for (int r = 0; r < g.kh; ++r) {
            const int ih = oh * g.sh + r - g.ph;
            if (ih < 0 || ih >= g.h) continue;
            for (int s = 0; s < g.kw; ++s) {
                const int iw = ow * g.sw + s - g.pw;
                if (iw < 0 || iw >= g.w) continue;
                for (int c = 0; c < g.c; ++c) {
                    const int xv = static_cast<int>(x[((size_t(n) * g.c + c) * g.h + ih) * g.w + iw]) - zp_in;
                    const int wv = w[((size_t(oc) * g.c + c) * g.kh + r) * g.kw + s];
                    acc += xv * wv;
                }
            }
        }
        if constexpr (EPI == EPI_I32) {
            static_cast<int32_t *>(out)[idx] = acc;
        } else {
            float v = static_cast<float>(acc) * (s_in * sw[oc]);
            if (bias) v = v + bias[oc];
            if constexpr (EPI == EPI_F32) {
                static_cast<float *>(out)[idx] = v;
            } else {
                const float q =
                    clamp_keep_nan(round_mode<EVEN>(v / s_out) + static_cast<float>(zp_out), -128.0f, 127.0f);
                static_cast<int8_t *>(out)[idx] = static_cast<int8_t>(to_int_nan0(q));
            }
        }
    }
}

static int32_t check_geom(const char *fn, const ConvGeom &g) {
    if (g.sh <= 0 || g.sw <= 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: stride must be positive", fn);
    if (g.kh <= 0 || g.kw <= 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: empty kernel", fn);
    if (g.h + 2 * g.ph < g.kh || g.w + 2 * g.pw < g.kw)
        return fail(HIPQ_SHAPE_ERROR, "%s: kernel larger than the padded input", fn);
    if (size_t(g.c) * g.kh * g.kw > (size_t(1) << 16))
        return fail(HIPQ_SHAPE_ERROR, "%s: c*kh*kw = %zu could overflow the int32 accumulator", fn,
                    size_t(g.c) * g.kh * g.kw);
    return HIPQ_SUCCESS;
}

// Pixels per channel block of the packed image: the padded grid, what the last windows' taps reach past it,
// and the 32 windows of a fragment that starts at the last one.
static size_t image_pixels(const ConvGeom &g) {
    const size_t hp = g.h + 2 * g.ph, wp = g.w + 2 * g.pw;
    const size_t reach = size_t(g.kh - 1) * wp + g.kw + 32;
    return (size_t(g.nb) * hp * wp + reach + 31) / 32 * 32;
}

static bool fast_path_ok(const ConvGeom &g) {
    const size_t k = size_t(g.c) * g.kh * g.kw;
    // offsets into the packed image and the packed filters are 32-bit
    return g.sh == 1 && g.sw == 1 && g.c % 32 == 0 && g.oc >= 1 &&
           size_t(g.c / 32) * image_pixels(g) * 32 < (size_t(1) << 31) &&
           packed_operand_bytes(g.oc, k) < (size_t(1) << 31);
}

static size_t align256(size_t v) { return (v + 255) & ~size_t(255); }

// [OC, IC, taps] filters -> the GEMM's packed row operand with K = (tap, channel), and the per-filter sums.
// `staging` holds OC * IC * taps bytes.
static int32_t pack_filters(hipq_ctx *ctx, const int8_t *w, int oc, int ic, int taps, int8_t *staging, int8_t *packed,
                            int32_t *wsum) {
    hipLaunchKernelGGL(conv_pack_weights_kernel, dim3(oc), dim3(kConvThreads), 0, ctx->stream, w, ic, taps, staging, wsum);
    int32_t rc = check_launch("conv_pack_weights");
    if (rc) return rc;
    return pack_rows(ctx, staging, size_t(oc), size_t(ic) * taps, packed);
}

// Dynamic input of a convolution: fp32 activations to be quantized to uint8 on the device (flavor, quantize mode
// bits), and where the parameters go.  x null: the input is already uint8.
struct ConvDynamicInput {
    const float *x = nullptr;
    int flavor = 0, quant_mode = 0;
    hipq_qparams *params = nullptr;
};

template <int EPI, bool EVEN>
static int32_t conv_forward(const char *fn, hipq_ctx *ctx, const uint8_t *x, int zp_in, float s_in, const int8_t *w,
                            const int8_t *wpacked, const int32_t *wsum, const float *sw, const float *bias,
                            const ConvGeom &g, float s_out, int zp_out, void *out,
                            const ConvDynamicInput &dyn = ConvDynamicInput{}) {
    if (!fast_path_ok(g)) {
        if (dyn.x) return fail(HIPQ_INVALID_ARGUMENT, "%s: needs stride 1 and channels a multiple of 32", fn);
        if (!w) return fail(HIPQ_INVALID_ARGUMENT, "%s: this geometry needs the unpacked filters", fn);
        const size_t total = size_t(g.nb) * g.oc * g.ho * g.wo;
        size_t blocks = (total + kConvThreads - 1) / kConvThreads;
        const size_t cap = size_t(ctx->num_cus) * 32;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL((conv_direct_kernel<EPI, EVEN>), dim3(static_cast<int>(blocks)), dim3(kConvThreads), 0,
                           ctx->stream, x, zp_in, w, g, s_in, sw, bias, s_out, zp_out, out);
        return check_launch(fn);
    }
    const int hp = g.h + 2 * g.ph, wp = g.w + 2 * g.pw, taps = g.kh * g.kw, cbs = g.c / 32;
    // One launch, the image gathered by the convolution kernel itself (hipq_conv_patch.h): built, bit-exact, and
    // measured no faster than the two launches below on the shape it was built for (13.3 against 13.4 us at
    // [32, 256, 14, 14] x [256, 256, 3, 3]: the gather costs what the layout launch did, and the window fragments
    // leave LDS no faster than they leave the L2), so it runs only under test hook 14.
    if (!dyn.x && ctx->gemm_variant == 14 && conv_patch_applicable(g.nb, g.c, g.h, g.w, hp, wp, g.kh, g.kw) &&
        size_t(g.nb) * g.c * g.h * g.w < (size_t(1) << 31) && !(reinterpret_cast<uintptr_t>(x) & 3u)) {
        const size_t kk = size_t(g.c) * taps;
        int32_t rc;
        if (!wpacked) {
            void *s = nullptr;
            const size_t need = kScratchHeader + align256(size_t(g.oc) * kk) + align256(packed_operand_bytes(g.oc, kk)) +
                                align256(size_t(g.oc) * 4);
            if ((rc = scratch(ctx, need, &s))) return rc;
            int8_t *staging = reinterpret_cast<int8_t *>(static_cast<char *>(s) + kScratchHeader);
            int8_t *pbuf = staging + align256(size_t(g.oc) * kk);
            int32_t *wsbuf = reinterpret_cast<int32_t *>(pbuf + align256(packed_operand_bytes(g.oc, kk)));
            if ((rc = pack_filters(ctx, w, g.oc, g.c, taps, staging, pbuf, wsbuf))) return rc;
            wpacked = pbuf;
            wsum = wsbuf;
        }
        GemmEpilogue ep{nullptr, 0, sw, bias, s_out, zp_out, out};
        ep.s_out_inv = host_recip_for_div(s_out);
        ep.sa_scalar = s_in;
        ep.cv_kw = g.kw;
        ep.cv_wp = wp;
        ep.cv_hp = hp;
        ep.cv_c = g.c;
        ep.cv_ho = g.ho;
        ep.cv_wo = g.wo;
        ep.cv_oc = g.oc;
        ep.cv_nb = g.nb;
        ep.cv_wsum = wsum;
        ep.cv_corr_mul = 128 - zp_in;
        ep.cv_kblocks = taps * cbs;
        return conv_gemm_patch(ctx, wpacked, x, size_t(g.nb) * g.c * g.h * g.w, zp_in, g.h, g.w, g.ph, g.pw, g.kh, g.oc,
                               g.nb * hp * wp, static_cast<int>(kk), ep, EPI, EVEN);
    }
    const size_t pixels = image_pixels(g);
    const size_t img_bytes = size_t(cbs) * pixels * 32;
    const size_t k = size_t(g.c) * taps;
    const size_t w_bytes = wpacked ? 0 : align256(size_t(g.oc) * k) + align256(packed_operand_bytes(g.oc, k)) +
                                             align256(size_t(g.oc) * 4);
    const int groups_per_cb = (g.nb * hp * wp + kConvThreads - 1) / kConvThreads;
    const size_t pack_grid = size_t(cbs) * groups_per_cb + cbs;
    // Dynamic input: in one launch with the image pack when its grid can be resident at once (the kernel holds 32
    // floats a lane: four workgroups per compute unit), else quantized to a uint8 copy first.
    const bool fused_input = dyn.x && ctx->gemm_variant != 6 && pack_grid <= resident_workgroups(ctx, true);
    const size_t u8_bytes = (dyn.x && !fused_input) ? align256(size_t(g.nb) * g.c * g.h * g.w) : 0;
    void *s = nullptr;
    int32_t rc = scratch(ctx, kScratchHeader + align256(img_bytes) + w_bytes + u8_bytes, &s);
    if (rc) return rc;
    int8_t *ximg = reinterpret_cast<int8_t *>(static_cast<char *>(s) + kScratchHeader);
    if (fused_input) {
        const bool qdiv = (dyn.quant_mode & HIPQ_FORM_DIV) != 0, qeven = (dyn.quant_mode & HIPQ_ROUND_HALF_EVEN) != 0;
        // Prepared filters of at most 1 MiB: touched by the quantizer while it waits (variant 11 switches it off).
        const size_t filter_bytes = packed_operand_bytes(g.oc, k);
        const bool touching = wpacked && ctx->gemm_variant != 11 && filter_bytes <= (size_t(1) << 20);
        const uint32_t *touch = touching ? reinterpret_cast<const uint32_t *>(wpacked) : nullptr;
        const uint32_t touch_lines = touching ? static_cast<uint32_t>(filter_bytes / 128) : 0u;
#define HIPQ_LAUNCH_CQ(D, E)                                                                                          \
    hipLaunchKernelGGL((conv_quantize_pack_image_kernel<D, E>), dim3(static_cast<int>(pack_grid)), dim3(kConvThreads), 0, \
                       ctx->stream, dyn.x, g.c, g.h, g.w, g.ph, g.pw, dyn.flavor, g.nb, groups_per_cb, dyn.params,    \
                       ctx->wait_error, ctx->wait_spin_limit, ximg, static_cast<int>(pixels), touch, touch_lines)
        if (qdiv && qeven)
            HIPQ_LAUNCH_CQ(true, 1);
        else if (qdiv)
            HIPQ_LAUNCH_CQ(true, 0);
        else if (qeven)
            HIPQ_LAUNCH_CQ(false, 1);
        else
            HIPQ_LAUNCH_CQ(false, 0);
#undef HIPQ_LAUNCH_CQ
    } else {
        if (dyn.x) {
            uint8_t *xq = reinterpret_cast<uint8_t *>(ximg + align256(img_bytes) + w_bytes);
            rc = quantize_dynamic_per_tensor(ctx, dyn.x, size_t(g.nb) * g.c * g.h * g.w, dyn.flavor, HIPQ_DTYPE_U8,
                                             dyn.quant_mode, xq, dyn.params, nullptr, 0);
            if (rc) return rc;
            // the call above may have grown (moved) the scratch
            if ((rc = scratch(ctx, kScratchHeader + align256(img_bytes) + w_bytes + u8_bytes, &s))) return rc;
            if (static_cast<char *>(s) + kScratchHeader != reinterpret_cast<char *>(ximg))
                return fail(HIPQ_DEVICE_ERROR, "%s: scratch moved under a pending kernel", fn);
            x = xq;
        }
        hipLaunchKernelGGL(conv_pack_image_kernel, dim3(static_cast<int>(pack_grid)), dim3(kConvThreads), 0, ctx->stream,
                           x, g.c, g.h, g.w, g.ph, g.pw, zp_in, dyn.x ? &dyn.params->zero_point : nullptr, g.nb,
                           groups_per_cb, ximg, static_cast<int>(pixels));
    }
    if ((rc = check_launch(fn))) return rc;
    if (!wpacked) {
        int8_t *staging = ximg + align256(img_bytes);
        int8_t *pbuf = staging + align256(size_t(g.oc) * k);
        int32_t *wsbuf = reinterpret_cast<int32_t *>(pbuf + align256(packed_operand_bytes(g.oc, k)));
        if ((rc = pack_filters(ctx, w, g.oc, g.c, taps, staging, pbuf, wsbuf))) return rc;
        wpacked = pbuf;
        wsum = wsbuf;
    }
    GemmEpilogue ep{nullptr, 0, sw, bias, s_out, zp_out, out};
    ep.s_out_inv = host_recip_for_div(s_out);
    ep.sa_scalar = s_in;
    ep.cv_kw = g.kw;
    ep.cv_wp = wp;
    ep.cv_hp = hp;
    ep.cv_c = g.c;
    ep.cv_ho = g.ho;
    ep.cv_wo = g.wo;
    ep.cv_oc = g.oc;
    ep.cv_nb = g.nb;
    ep.cv_wsum = wsum;
    ep.cv_corr_mul = 128 - zp_in;
    if (dyn.x) {
        ep.sa = &dyn.params->scale;  // NaN for a range that is not finite: the outputs then carry no information
        ep.cv_zp_in = &dyn.params->zero_point;
    }
    ep.cv_pixels = static_cast<int>(pixels);
    ep.cv_kblocks = taps * cbs;
    ep.fresh_activations = 1;  // the image was written by the kernel just before
    return conv_gemm_packed(ctx, wpacked, ximg, g.oc, g.nb * hp * wp, static_cast<int>(k), ep, EPI, EVEN);
}

static int32_t make_geom(const char *fn, size_t nb, size_t c, size_t h, size_t w, size_t oc, size_t kh, size_t kw,
                         size_t sh, size_t sw, size_t ph, size_t pw, ConvGeom *g) {
    const size_t lim = size_t(1) << 24;
    if (nb >= lim || c >= lim || h >= lim || w >= lim || oc >= lim || kh >= lim || kw >= lim || sh >= lim || sw >= lim ||
        ph >= lim || pw >= lim)
        return fail(HIPQ_SHAPE_ERROR, "%s: dimension too large", fn);
    *g = ConvGeom{int(nb), int(c), int(h), int(w), int(oc), int(kh), int(kw), int(sh), int(sw), int(ph), int(pw), 0, 0};
    int32_t rc = check_geom(fn, *g);
    if (rc) return rc;
    // (H + 2p - k) / s + 1, crates/torsh-backend/src/quantization/ops.rs:513-514
    g->ho = (g->h + 2 * g->ph - g->kh) / g->sh + 1;
    g->wo = (g->w + 2 * g->pw - g->kw) / g->sw + 1;
    if (size_t(g->nb) * (g->h + 2 * g->ph) * (g->w + 2 * g->pw) >= (size_t(1) << 31))
        return fail(HIPQ_SHAPE_ERROR, "%s: too many pixels", fn);
    return HIPQ_SUCCESS;
}

}  // namespace hipq

using namespace hipq;

extern "C" {

int32_t hipq_conv2d_packed_weights_size(size_t oc, size_t ic, size_t kh, size_t kw, size_t *out_bytes) {
    HIPQ_REQUIRE_PTR(out_bytes);
    if (oc >> 24 || ic >> 24 || (kh * kw) >> 16 || (ic * kh * kw) >> 24)
        return fail(HIPQ_SHAPE_ERROR, "%s: dimension too large", __func__);
    *out_bytes = packed_operand_bytes(oc, ic * kh * kw);
    return HIPQ_SUCCESS;
}

int32_t hipq_conv2d_pack_weights_i8(hipq_ctx *ctx, const int8_t *w, size_t oc, size_t ic, size_t kh, size_t kw,
                                    int8_t *packed, int32_t *wsum) {
    HIPQ_ENTER(ctx);
    if (oc == 0 || ic * kh * kw == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(w);
    HIPQ_REQUIRE_PTR(packed);
    HIPQ_REQUIRE_PTR(wsum);
    if (oc >> 24 || ic >> 24 || (kh * kw) >> 16 || (ic * kh * kw) >> 24)
        return fail(HIPQ_SHAPE_ERROR, "%s: dimension too large", __func__);
    if (reinterpret_cast<uintptr_t>(packed) & 15u)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: the packed buffer must be 16-byte aligned", __func__);
    void *s = nullptr;
    int32_t rc = scratch(ctx, kScratchHeader + oc * ic * kh * kw, &s);
    if (rc) return rc;
    int8_t *staging = reinterpret_cast<int8_t *>(static_cast<char *>(s) + kScratchHeader);
    return pack_filters(ctx, w, static_cast<int>(oc), static_cast<int>(ic), static_cast<int>(kh * kw), staging, packed,
                        wsum);
}

int32_t hipq_conv2d_u8i8_i32(hipq_ctx *ctx, const uint8_t *x, int32_t zp_in, const int8_t *w, size_t nb, size_t c,
                             size_t h, size_t wd, size_t oc, size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                             size_t pad_h, size_t pad_w, int32_t *out) {
    HIPQ_ENTER(ctx);
    ConvGeom g;
    int32_t rc = make_geom(__func__, nb, c, h, wd, oc, kh, kw, stride_h, stride_w, pad_h, pad_w, &g);
    if (rc) return rc;
    if (zp_in < 0 || zp_in > 255) return fail(HIPQ_INVALID_ARGUMENT, "%s: zero point %d outside [0,255]", __func__, zp_in);
    if (nb == 0 || oc == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(w);
    HIPQ_REQUIRE_PTR(out);
    return conv_forward<EPI_I32, false>(__func__, ctx, x, zp_in, 1.0f, w, nullptr, nullptr, nullptr, nullptr, g, 1.0f, 0,
                                        out);
}

static int32_t conv_i8_common(const char *fn, hipq_ctx *ctx, const uint8_t *x, int32_t zp_in, float s_in,
                              const int8_t *w, const int8_t *wpacked, const int32_t *wsum, const float *sw,
                              const float *bias, const ConvGeom &g, float s_out, int32_t zp_out, int32_t mode,
                              int8_t *out) {
    if (s_in <= 0.0f || s_out <= 0.0f) return fail(HIPQ_INVALID_ARGUMENT, "%s: Scale must be positive", fn);
    if (zp_in < 0 || zp_in > 255) return fail(HIPQ_INVALID_ARGUMENT, "%s: zero point %d outside [0,255]", fn, zp_in);
    if (mode & ~(HIPQ_ROUND_HALF_EVEN | HIPQ_FORM_DIV)) return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown mode bits", fn);
    if (g.nb == 0 || g.oc == 0) return HIPQ_SUCCESS;
    if (!x || !sw || !out) return fail(HIPQ_INVALID_ARGUMENT, "%s: null pointer", fn);
    if (mode & HIPQ_ROUND_HALF_EVEN)
        return conv_forward<EPI_I8, true>(fn, ctx, x, zp_in, s_in, w, wpacked, wsum, sw, bias, g, s_out, zp_out, out);
    return conv_forward<EPI_I8, false>(fn, ctx, x, zp_in, s_in, w, wpacked, wsum, sw, bias, g, s_out, zp_out, out);
}

int32_t hipq_conv2d_u8i8_i8(hipq_ctx *ctx, const uint8_t *x, int32_t zp_in, float s_in, const int8_t *w,
                            const float *w_scales, const float *bias, size_t nb, size_t c, size_t h, size_t wd,
                            size_t oc, size_t kh, size_t kw, size_t stride_h, size_t stride_w, size_t pad_h,
                            size_t pad_w, float out_scale, int32_t out_zero_point, int32_t mode, int8_t *out) {
    HIPQ_ENTER(ctx);
    ConvGeom g;
    int32_t rc = make_geom(__func__, nb, c, h, wd, oc, kh, kw, stride_h, stride_w, pad_h, pad_w, &g);
    if (rc) return rc;
    if (nb != 0 && oc != 0) HIPQ_REQUIRE_PTR(w);
    return conv_i8_common(__func__, ctx, x, zp_in, s_in, w, nullptr, nullptr, w_scales, bias, g, out_scale,
                          out_zero_point, mode, out);
}

int32_t hipq_conv2d_u8i8_f32(hipq_ctx *ctx, const uint8_t *x, int32_t zp_in, float s_in, const int8_t *w,
                             const float *w_scales, const float *bias, size_t nb, size_t c, size_t h, size_t wd,
                             size_t oc, size_t kh, size_t kw, size_t stride_h, size_t stride_w, size_t pad_h,
                             size_t pad_w, float *out) {
    HIPQ_ENTER(ctx);
    ConvGeom g;
    int32_t rc = make_geom(__func__, nb, c, h, wd, oc, kh, kw, stride_h, stride_w, pad_h, pad_w, &g);
    if (rc) return rc;
    if (s_in <= 0.0f) return fail(HIPQ_INVALID_ARGUMENT, "%s: Scale must be positive", __func__);
    if (zp_in < 0 || zp_in > 255) return fail(HIPQ_INVALID_ARGUMENT, "%s: zero point %d outside [0,255]", __func__, zp_in);
    if (nb == 0 || oc == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(w);
    HIPQ_REQUIRE_PTR(w_scales);
    HIPQ_REQUIRE_PTR(out);
    return conv_forward<EPI_F32, false>(__func__, ctx, x, zp_in, s_in, w, nullptr, nullptr, w_scales, bias, g, 1.0f, 0,
                                        out);
}

int32_t hipq_conv2d_u8i8_i8_packed(hipq_ctx *ctx, const uint8_t *x, int32_t zp_in, float s_in, const int8_t *w_packed,
                                   const int32_t *w_sums, const float *w_scales, const float *bias, size_t nb, size_t c,
                                   size_t h, size_t wd, size_t oc, size_t kh, size_t kw, size_t pad_h, size_t pad_w,
                                   float out_scale, int32_t out_zero_point, int32_t mode, int8_t *out) {
    HIPQ_ENTER(ctx);
    ConvGeom g;
    int32_t rc = make_geom(__func__, nb, c, h, wd, oc, kh, kw, 1, 1, pad_h, pad_w, &g);
    if (rc) return rc;
    if (!fast_path_ok(g))
        return fail(HIPQ_INVALID_ARGUMENT, "%s: packed filters need stride 1 and channels a multiple of 32", __func__);
    if (nb != 0 && oc != 0) {
        HIPQ_REQUIRE_PTR(w_packed);
        HIPQ_REQUIRE_PTR(w_sums);
    }
    return conv_i8_common(__func__, ctx, x, zp_in, s_in, nullptr, w_packed, w_sums, w_scales, bias, g, out_scale,
                          out_zero_point, mode, out);
}

int32_t hipq_conv2d_dynamic_f32_i8_packed(hipq_ctx *ctx, const float *x, int32_t flavor, int32_t quant_mode,
                                          const int8_t *w_packed, const int32_t *w_sums, const float *w_scales,
                                          const float *bias, size_t nb, size_t c, size_t h, size_t wd, size_t oc,
                                          size_t kh, size_t kw, size_t pad_h, size_t pad_w, float out_scale,
                                          int32_t out_zero_point, int32_t mode, int8_t *out, hipq_qparams *in_params) {
    HIPQ_ENTER(ctx);
    ConvGeom g;
    int32_t rc = make_geom(__func__, nb, c, h, wd, oc, kh, kw, 1, 1, pad_h, pad_w, &g);
    if (rc) return rc;
    if (!fast_path_ok(g))
        return fail(HIPQ_INVALID_ARGUMENT, "%s: packed filters need stride 1 and channels a multiple of 32", __func__);
    if (flavor < HIPQ_PARAMS_SYMMETRIC || flavor > HIPQ_PARAMS_NN_ASYMMETRIC)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown flavor %d", __func__, flavor);
    if (quant_mode & ~(HIPQ_ROUND_HALF_EVEN | HIPQ_FORM_DIV))
        return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown quantize mode bits", __func__);
    if (mode & ~(HIPQ_ROUND_HALF_EVEN | HIPQ_FORM_DIV)) return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown mode bits", __func__);
    if (out_scale <= 0.0f) return fail(HIPQ_INVALID_ARGUMENT, "%s: Scale must be positive", __func__);
    if (nb == 0 || oc == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(w_packed);
    HIPQ_REQUIRE_PTR(w_sums);
    HIPQ_REQUIRE_PTR(w_scales);
    HIPQ_REQUIRE_PTR(out);
    HIPQ_REQUIRE_PTR(in_params);
    ConvDynamicInput dyn;
    dyn.x = x;
    dyn.flavor = flavor;
    dyn.quant_mode = quant_mode;
    dyn.params = in_params;
    if (mode & HIPQ_ROUND_HALF_EVEN)
        return conv_forward<EPI_I8, true>(__func__, ctx, nullptr, 0, 1.0f, nullptr, w_packed, w_sums, w_scales, bias, g,
                                          out_scale, out_zero_point, out, dyn);
    return conv_forward<EPI_I8, false>(__func__, ctx, nullptr, 0, 1.0f, nullptr, w_packed, w_sums, w_scales, bias, g,
                                       out_scale, out_zero_point, out, dyn);
}

}  // extern "C"
