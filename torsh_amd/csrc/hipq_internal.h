// Internal declarations shared by the torsh_hipq translation units.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>

#include <vector>

#include "torsh_hipq.h"
#include "torsh_hipq_testing.h"

// Lines (128 bytes) of a packed operand wanted in the L2 of the die whose workgroups will read them: die d's share
// starts die_stride_lines * d lines after base; within it, per row block (row_block_lines apart), `starts` runs of
// run_lines lines, start_step_lines apart; `lines` of them per die in all.
struct WarmLines {
    const uint32_t *base = nullptr;
    uint32_t lines = 0, die_stride_lines = 0, row_block_lines = 0, starts = 1, run_lines = 0, start_step_lines = 0;
};

struct hipq_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    bool owns_stream = false;
    // Scratch owned by the context: partial reductions, device-side parameters,
    // int8 activations of the fused Linear forward.  Grown on demand, freed with
    // the context.
    void *scratch = nullptr;
    size_t scratch_bytes = 0;
    // Set once a call that uses the scratch was recorded under stream capture: the recorded kernels hold pointers
    // into the block of that moment, so from then on a block that is outgrown is kept (in `retired`, freed with
    // the context) instead of freed, and a replay of the graph still finds its memory.
    bool scratch_captured = false;
    std::vector<void *> retired;
    int num_cus = 256;
    // Exchange area of the GEMM form whose workgroup pairs hand partial sums to each other (hipq_gemm_pair.h):
    // flag words (zero between launches), then the buffer.  Grown like the scratch; pair_ok: the device hands
    // workgroup ids b and b + 8 to the same XCD (checked by hipq_ctx_create).
    void *pair_area = nullptr;
    size_t pair_flag_bytes = 0, pair_bytes = 0;
    bool pair_ok = false;
    // Device words of the context (kCtxWordsBytes of them, laid out as the kCtx* constants below say).  Word 0 is
    // set by a kernel whose bounded wait gave up; hipq_ctx_synchronize reads and clears it.
    uint32_t *wait_error = nullptr;
    // Test and tuning hooks, per context (torsh_hipq_testing.h): forced GEMM kernel form (0 = automatic) and the
    // spin limit of the kernels' bounded waits.
    int gemm_variant = 0;
    int wait_spin_limit = 1 << 20;
    // How many contexts launch concurrently on this device (hipq_ctx_set_resident_share): kernels whose grid has to
    // be resident at once size it for 1 / resident_share of the device.
    int resident_share = 1;
    // Set by a fused forward around its activation-quantize launch: lines of the operand that the next kernel reads
    // first, for the quantizer's workgroups to touch while they wait for the grid's range.  lines = 0: none.
    WarmLines warm;
    // Tuning aid (hipq_ctx_set_trace_buffer): caller-owned device memory for the packed GEMM's phase stamps.
    void *trace = nullptr;
    size_t trace_bytes = 0;
};

namespace hipq {

// Layout of hipq_ctx::wait_error, in 32-bit words.  Beyond the give-up flag it holds the meeting point of the
// one-launch dynamic quantizer (hipq_meeting.h): the number of the last meeting, the 64-bit word {tag, zero
// point, scale bits} that ends one, and per workgroup the two 64-bit words {meeting, min}, {meeting, max}.
constexpr size_t kCtxFlagWord = 0;
constexpr size_t kCtxEpochWord = 16;
constexpr size_t kCtxReadyWord = 32;
constexpr size_t kCtxRangeWord = 64;
constexpr size_t kCtxSlots = 2048;  // workgroups that can meet
constexpr size_t kCtxWordsBytes = (kCtxRangeWord + kCtxSlots * 4) * 4;
// Number the first meeting of a context gets, a few launches before the counter wraps, so that the wrap (which
// wipes the slots) is a path every context takes early, not once in 2^32 launches.
constexpr uint32_t kCtxFirstEpoch = 0xfffffff0u;
// Puts the device words of a context into their initial state (device current, stream idle).
int32_t reset_ctx_words(hipq_ctx *ctx);
// Workgroups of 256 threads per compute unit that a kernel of this context may count on being resident together
// with the rest of its grid.  The one-launch kernels, light or wide, are built with a launch bound of four
// workgroups per compute unit (at most 128 registers), so four is what the bound guarantees whatever the compiler
// made of a kernel, and the context's share of that is 1 / resident_share.
inline size_t resident_workgroups(const hipq_ctx *ctx, bool /*wide*/) {
    const int share = ctx->resident_share > 0 ? ctx->resident_share : 1;
    const int per_cu = 4 / share;
    size_t total = size_t(ctx->num_cus) * static_cast<size_t>(per_cu);
    return total < kCtxSlots ? total : kCtxSlots;
}

// Records `msg` (printf style) as the calling thread's last error and returns `code`.
int32_t fail(int32_t code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

// Makes the context's device current; returns HIPQ_SUCCESS or a recorded error.
int32_t enter(hipq_ctx *ctx);
// Ensures ctx->scratch holds at least `bytes`; returns pointer via out.
int32_t scratch(hipq_ctx *ctx, size_t bytes, void **out);
// Ensures the pair-exchange area holds `flag_bytes` of zeroed flag words followed (256-byte aligned) by
// `buf_bytes`; returns both pointers.  Same rules under stream capture as the scratch.
int32_t pair_area(hipq_ctx *ctx, size_t flag_bytes, size_t buf_bytes, uint32_t **flags, int8_t **buf);
// Whether workgroup ids 8 apart run on one XCD on this device (asked of the device once, remembered).
bool pairs_share_an_xcd(hipq_ctx *ctx);
// Checks the sticky launch error after a kernel launch.
int32_t check_launch(const char *what);

// hipq_quantize_dynamic_per_tensor_f32 with the room for its range partials given by the caller
// (`partials`, `partials_bytes` of device memory) instead of taken from the context scratch; null =
// context scratch.
int32_t quantize_dynamic_per_tensor(hipq_ctx *ctx, const float *x, size_t n, int32_t flavor, int32_t dtype,
                                    int32_t mode, void *out, hipq_qparams *out_params, void *partials,
                                    size_t partials_bytes);
// Activation quantizers of the fused Linear forwards: symmetric int8, per tensor (dynamic range or a given
// static scale; row-major or fragment-packed output) and per row (row-major).  A range that is not finite
// gives a NaN scale and zero codes, so the GEMM that follows turns it into NaN outputs.
int32_t quantize_activations_per_tensor(hipq_ctx *ctx, const float *x, size_t rows, size_t cols, bool dynamic,
                                        float static_scale, int32_t mode, bool packed, int8_t *out,
                                        hipq_qparams *out_params, void *partials, size_t partials_bytes);
int32_t quantize_activations_per_row(hipq_ctx *ctx, const float *x, size_t rows, size_t cols, int32_t mode,
                                     int8_t *out, float *out_scales, bool packed = false);
// The same for rows that lie `ld` floats apart (a column slice of a wider matrix).
int32_t quantize_activations_per_row_strided(hipq_ctx *ctx, const float *x, size_t rows, size_t cols, size_t ld,
                                             int32_t mode, int8_t *out, float *out_scales, bool packed);
// Looks up, once per device, the address of the static device array behind
// hipq_linear_dynamic_f32_noalloc; called by hipq_ctx_create with the device current.
int32_t linear_noalloc_setup(int device);
// Whether four workgroups of the widest one-launch quantizers fit a compute unit of the context's device (asked of
// the runtime once per device and remembered).
bool four_wide_workgroups_fit(const hipq_ctx *ctx);

// Bytes reserved at the head of the context scratch for small device records
// (hipq_qparams, min/max pairs, status words); bulk scratch starts after it.
constexpr size_t kScratchHeader = 4096;

}  // namespace hipq

#define HIPQ_REQUIRE_PTR(p)                                                              \
    do {                                                                                 \
        if ((p) == nullptr) return hipq::fail(HIPQ_INVALID_ARGUMENT, "%s: null pointer '%s'", __func__, #p); \
    } while (0)

#define HIPQ_ENTER(ctx)                                   \
    do {                                                  \
        HIPQ_REQUIRE_PTR(ctx);                            \
        int32_t _rc = hipq::enter(ctx);                   \
        if (_rc != HIPQ_SUCCESS) return _rc;              \
    } while (0)

#define HIPQ_HIP(call)                                                                              \
    do {                                                                                            \
        hipError_t _e = (call);                                                                     \
        if (_e != hipSuccess)                                                                       \
            return hipq::fail(HIPQ_DEVICE_ERROR, "%s: %s failed: %s", __func__, #call, hipGetErrorString(_e)); \
    } while (0)
