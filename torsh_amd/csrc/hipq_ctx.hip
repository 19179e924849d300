// Context, error reporting and device-memory helpers of the torsh_hipq C-ABI.
#include <cstdio>
#include <cstring>
#include <new>

#include "hipq_internal.h"

namespace {
thread_local char g_last_error[512] = {0};
thread_local bool g_has_error = false;
}  // namespace

namespace hipq {

int32_t fail(int32_t code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    g_has_error = true;
    return code;
}

void clear_error() {
    g_last_error[0] = 0;
    g_has_error = false;
}

int32_t enter(hipq_ctx *ctx) {
    hipError_t e = hipSetDevice(ctx->device);
    if (e != hipSuccess) return fail(HIPQ_DEVICE_ERROR, "hipSetDevice(%d): %s", ctx->device, hipGetErrorString(e));
    return HIPQ_SUCCESS;
}

int32_t scratch(hipq_ctx *ctx, size_t bytes, void **out) {
    // Kernels recorded under stream capture keep pointers into the block of that moment.
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    const bool capturing = hipStreamIsCapturing(ctx->stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone;
    if (capturing) ctx->scratch_captured = true;
    if (bytes > ctx->scratch_bytes) {
        if (capturing)
            return fail(HIPQ_ALLOCATION_ERROR,
                        "scratch: this call needs %zu bytes of context scratch and the context holds %zu; memory cannot "
                        "be allocated while the stream is capturing - run the same call once before the capture",
                        bytes, ctx->scratch_bytes);
        // Round up so a sequence of slightly growing requests reallocates rarely.
        size_t want = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
        void *grown = nullptr;
        hipError_t e = hipMalloc(&grown, want);
        if (e != hipSuccess) return fail(HIPQ_ALLOCATION_ERROR, "scratch: hipMalloc(%zu): %s", want, hipGetErrorString(e));
        if (ctx->scratch) {
            if (ctx->scratch_captured) {
                ctx->retired.push_back(ctx->scratch);  // a captured graph may still be replayed on it
            } else {
                e = hipStreamSynchronize(ctx->stream);
                if (e != hipSuccess) {
                    (void)hipFree(grown);
                    return fail(HIPQ_SYNCHRONIZATION_ERROR, "scratch: %s", hipGetErrorString(e));
                }
                (void)hipFree(ctx->scratch);
            }
        }
        ctx->scratch = grown;
        ctx->scratch_bytes = want;
    }
    *out = ctx->scratch;
    return HIPQ_SUCCESS;
}

int32_t pair_area(hipq_ctx *ctx, size_t flag_bytes, size_t buf_bytes, uint32_t **flags, int8_t **buf) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    const bool capturing = hipStreamIsCapturing(ctx->stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone;
    if (capturing) ctx->scratch_captured = true;
    const size_t flags_up = (flag_bytes + 255) & ~size_t(255);
    if (flags_up > ctx->pair_flag_bytes || flags_up + buf_bytes > ctx->pair_bytes) {
        if (capturing)
            return fail(HIPQ_ALLOCATION_ERROR,
                        "pair exchange area: memory cannot be allocated while the stream is capturing - run the same "
                        "call once before the capture");
        // The flags of a larger area start further on, and flags must be zero: a fresh, zeroed block (the stream is
        // drained first, so no launch is using the old one).
        hipError_t e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) return fail(HIPQ_SYNCHRONIZATION_ERROR, "pair exchange area: %s", hipGetErrorString(e));
        const size_t fl = flags_up > ctx->pair_flag_bytes ? flags_up : ctx->pair_flag_bytes;
        const size_t want = (fl + buf_bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
        void *grown = nullptr;
        e = hipMalloc(&grown, want);
        if (e == hipSuccess) e = hipMemset(grown, 0, fl);
        if (e != hipSuccess) {
            if (grown) (void)hipFree(grown);
            return fail(HIPQ_ALLOCATION_ERROR, "pair exchange area: %zu bytes: %s", want, hipGetErrorString(e));
        }
        if (ctx->pair_area) {
            if (ctx->scratch_captured)
                ctx->retired.push_back(ctx->pair_area);
            else
                (void)hipFree(ctx->pair_area);
        }
        ctx->pair_area = grown;
        ctx->pair_flag_bytes = fl;
        ctx->pair_bytes = want;
    }
    *flags = static_cast<uint32_t *>(ctx->pair_area);
    *buf = static_cast<int8_t *>(ctx->pair_area) + ctx->pair_flag_bytes;
    return HIPQ_SUCCESS;
}

int32_t check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HIPQ_DEVICE_ERROR, "%s: kernel launch failed: %s", what, hipGetErrorString(e));
    return HIPQ_SUCCESS;
}

int32_t reset_ctx_words(hipq_ctx *ctx) {
    hipError_t e = hipMemset(ctx->wait_error, 0, kCtxWordsBytes);
    const uint32_t epoch = kCtxFirstEpoch;
    if (e == hipSuccess) e = hipMemcpy(ctx->wait_error + kCtxEpochWord, &epoch, sizeof(epoch), hipMemcpyHostToDevice);
    // (flags of the pair exchange: a launch that gave up may have left some set)
    if (e == hipSuccess && ctx->pair_area) e = hipMemset(ctx->pair_area, 0, ctx->pair_flag_bytes);
    if (e != hipSuccess) return fail(HIPQ_DEVICE_ERROR, "status words of the context: %s", hipGetErrorString(e));
    return HIPQ_SUCCESS;
}

}  // namespace hipq

extern "C" {

const char *hipq_version(void) { return "torsh_hipq 0.1.0 (gfx950)"; }

const char *hipq_get_last_error(void) { return g_last_error; }

void hipq_clear_last_error(void) { hipq::clear_error(); }

int32_t hipq_has_error(void) { return g_has_error ? 1 : 0; }

static int32_t ctx_new(int32_t device, hipStream_t stream, bool own, hipq_ctx **out_ctx) {
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0)
        return hipq::fail(HIPQ_DEVICE_ERROR, "hipq_ctx_create: no HIP device available (%s)",
                          e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    if (device < 0 || device >= count)
        return hipq::fail(HIPQ_INVALID_ARGUMENT, "hipq_ctx_create: device %d out of range [0,%d)", device, count);
    HIPQ_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    HIPQ_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return hipq::fail(HIPQ_DEVICE_ERROR, "hipq_ctx_create: device %d is %s; this library is built for gfx950 only",
                          device, prop.gcnArchName);
    hipq_ctx *ctx = new (std::nothrow) hipq_ctx();
    if (!ctx) return hipq::fail(HIPQ_ALLOCATION_ERROR, "hipq_ctx_create: out of host memory");
    ctx->device = device;
    ctx->num_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    if (own) {
        e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
        if (e != hipSuccess) {
            delete ctx;
            return hipq::fail(HIPQ_DEVICE_ERROR, "hipq_ctx_create: hipStreamCreate: %s", hipGetErrorString(e));
        }
        ctx->owns_stream = true;
    } else {
        ctx->stream = stream;
    }
    void *p = nullptr;
    int32_t rc = hipq::linear_noalloc_setup(device);
    if (rc == HIPQ_SUCCESS) rc = hipq::scratch(ctx, size_t(8) << 20, &p);
    if (rc == HIPQ_SUCCESS) {
        e = hipMalloc(reinterpret_cast<void **>(&ctx->wait_error), hipq::kCtxWordsBytes);
        if (e != hipSuccess)
            rc = hipq::fail(HIPQ_ALLOCATION_ERROR, "hipq_ctx_create: status words: %s", hipGetErrorString(e));
        else
            rc = hipq::reset_ctx_words(ctx);
    }
    if (rc != HIPQ_SUCCESS) {
        if (ctx->wait_error) (void)hipFree(ctx->wait_error);
        if (ctx->scratch) (void)hipFree(ctx->scratch);
        if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return rc;
    }
    (void)hipq::four_wide_workgroups_fit(ctx);  // asked here so that no later call is the first
    ctx->pair_ok = hipq::pairs_share_an_xcd(ctx);
    *out_ctx = ctx;
    return HIPQ_SUCCESS;
}

int32_t hipq_ctx_create(int32_t device, hipq_ctx **out_ctx) {
    HIPQ_REQUIRE_PTR(out_ctx);
    return ctx_new(device, nullptr, true, out_ctx);
}

int32_t hipq_ctx_create_on_stream(int32_t device, void *hip_stream, hipq_ctx **out_ctx) {
    HIPQ_REQUIRE_PTR(out_ctx);
    return ctx_new(device, static_cast<hipStream_t>(hip_stream), false, out_ctx);
}

int32_t hipq_ctx_destroy(hipq_ctx *ctx) {
    HIPQ_ENTER(ctx);
    (void)hipStreamSynchronize(ctx->stream);
    if (ctx->scratch) (void)hipFree(ctx->scratch);
    if (ctx->pair_area) (void)hipFree(ctx->pair_area);
    for (void *p : ctx->retired) (void)hipFree(p);
    if (ctx->wait_error) (void)hipFree(ctx->wait_error);
    if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return HIPQ_SUCCESS;
}

int32_t hipq_ctx_synchronize(hipq_ctx *ctx) {
    HIPQ_ENTER(ctx);
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess)
        return hipq::fail(HIPQ_SYNCHRONIZATION_ERROR, "hipq_ctx_synchronize: %s", hipGetErrorString(e));
    // A kernel whose bounded wait gave up has finished (every kernel drains) but its result is not the
    // product that was asked for: report it here, once, and clear the word.
    uint32_t gave_up = 0;
    HIPQ_HIP(hipMemcpy(&gave_up, ctx->wait_error, sizeof(gave_up), hipMemcpyDeviceToHost));
    if (gave_up) {
        // Workgroups that ran after their meeting was given up may have left words that a later meeting would
        // take for its own: start over.
        const int32_t rc = hipq::reset_ctx_words(ctx);
        if (rc) return rc;
        return hipq::fail(HIPQ_DEVICE_ERROR,
                          "hipq_ctx_synchronize: a bounded wait inside a kernel (persistent GEMM or one-launch "
                          "dynamic quantize) gave up (spin limit %d); results of the calls since the last "
                          "synchronize are invalid",
                          ctx->wait_spin_limit);
    }
    return HIPQ_SUCCESS;
}

int32_t hipq_set_gemm_kernel_variant(hipq_ctx *ctx, int32_t variant) {
    HIPQ_REQUIRE_PTR(ctx);
    if (variant < 0 || variant > 16 || variant == 13)
        return hipq::fail(HIPQ_INVALID_ARGUMENT, "%s: variant %d is not one of 0..12, 14..16", __func__, variant);
    ctx->gemm_variant = variant;
    return HIPQ_SUCCESS;
}

int32_t hipq_ctx_set_resident_share(hipq_ctx *ctx, int32_t contexts) {
    HIPQ_REQUIRE_PTR(ctx);
    if (contexts < 1 || contexts > 64)
        return hipq::fail(HIPQ_INVALID_ARGUMENT, "%s: %d is not in 1..64", __func__, contexts);
    ctx->resident_share = contexts;
    return HIPQ_SUCCESS;
}

int32_t hipq_ctx_set_wait_spin_limit(hipq_ctx *ctx, int32_t limit) {
    HIPQ_REQUIRE_PTR(ctx);
    ctx->wait_spin_limit = limit < 0 ? (1 << 20) : limit;
    return HIPQ_SUCCESS;
}

int32_t hipq_ctx_set_trace_buffer(hipq_ctx *ctx, void *device_buffer, size_t bytes) {
    HIPQ_REQUIRE_PTR(ctx);
    ctx->trace = device_buffer;
    ctx->trace_bytes = device_buffer ? bytes : 0;
    return HIPQ_SUCCESS;
}

void *hipq_ctx_stream(hipq_ctx *ctx) { return ctx ? static_cast<void *>(ctx->stream) : nullptr; }

int32_t hipq_device_malloc(hipq_ctx *ctx, size_t bytes, void **out_ptr) {
    HIPQ_ENTER(ctx);
    HIPQ_REQUIRE_PTR(out_ptr);
    *out_ptr = nullptr;
    if (bytes == 0) return HIPQ_SUCCESS;
    hipError_t e = hipMalloc(out_ptr, bytes);
    if (e != hipSuccess)
        return hipq::fail(HIPQ_ALLOCATION_ERROR, "hipq_device_malloc(%zu): %s", bytes, hipGetErrorString(e));
    return HIPQ_SUCCESS;
}

int32_t hipq_device_free(hipq_ctx *ctx, void *ptr) {
    HIPQ_ENTER(ctx);
    if (!ptr) return HIPQ_SUCCESS;
    HIPQ_HIP(hipFree(ptr));
    return HIPQ_SUCCESS;
}

int32_t hipq_memcpy_h2d(hipq_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes) {
    HIPQ_ENTER(ctx);
    if (bytes == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(dst_dev);
    HIPQ_REQUIRE_PTR(src_host);
    HIPQ_HIP(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
    HIPQ_HIP(hipStreamSynchronize(ctx->stream));
    return HIPQ_SUCCESS;
}

int32_t hipq_memcpy_d2h(hipq_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes) {
    HIPQ_ENTER(ctx);
    if (bytes == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(dst_host);
    HIPQ_REQUIRE_PTR(src_dev);
    HIPQ_HIP(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    HIPQ_HIP(hipStreamSynchronize(ctx->stream));
    return HIPQ_SUCCESS;
}

}  // extern "C"
