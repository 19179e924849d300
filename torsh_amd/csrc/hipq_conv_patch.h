// Quantized Conv2d forward (stride 1, u8 NCHW input) as an implicit GEMM whose workgroups build their own piece
// of the image: no layout pass over the input, no second launch.
//
// A workgroup owns 64 consecutive windows of the zero-point-padded pixel grid (two MFMA column blocks) and 128
// filters (one row block per wave, the whole K = taps x channels in that wave: no K split, no partial sums).
// The taps of those windows reach patch = 64 + (kh - 1) * wp + kw - 1 pixels of the padded grid, so the workgroup
// first gathers that patch from the NCHW planes into LDS as signed bytes (x - 128, a border pixel holds
// zp - 128), laid out [channel block of 32][half of 16 channels][pixel][16 bytes]: the fragment of (tap, channel
// block) for 32 windows is then 32 consecutive pixels of that array from the tap's offset on - one conflict-free
// 16-byte LDS read per lane, for every tap, with no im2col and nothing of the image on the vector-memory path
// after the gather (the layout pass and the per-tap window fragments of the two-launch form cost 2 KiB of that
// path per k block beside 4 KiB of filters; here it carries the filters alone).  Filter fragments come from the
// L2 straight into registers, sixteen in flight per wave.
//
// With one wave per SIMD a wave issues an instruction every four cycles at best, so every phase is written for
// instruction count: addresses are a per-lane base plus immediates or one scalar add, never a multiply per access.
//
// Gather, step 1: the plane bytes the patch can touch - whole rows of at most two images, contiguous in every
// channel plane, at most 128 bytes - go to LDS as they lie in memory, one dword per lane, 32 lanes along a plane
// and eight channels per instruction (byte loads straight from the planes cost the vector-memory path an
// instruction slot per 64 bytes: 4.5 us for this step, measured).  Step 2: a thread owns one pixel of the patch
// (its place in the raw rows, or "border", is worked out once) and collects that pixel's byte of each channel of
// its share with LDS byte reads at immediate offsets: lanes are consecutive pixels, consecutive bytes of a raw row.
//
// M = filters, N = padded pixels (n * hp * wp), K = taps * channels, tap-major.  Geometries taken: see
// conv_patch_fits; all others run the two-launch form.  Epilogue: conv_store_block (hipq_gemm_packed.h).
// Included by hipq_gemm_packed.hip.
#pragma once

#include "hipq_gemm_packed.h"

namespace hipq {

struct ConvPatch {
    const uint8_t *x;  // [nb, c, h, w]
    int h, w, ph, pw, kh;
    int patch;         // pixels of the padded grid a workgroup's taps reach
    uint32_t border;   // (zp_in ^ 0x80) in each byte
    int x_bytes;       // nb * c * h * w
    float r_per_img, r_wp;  // 1 / (hp * wp), 1 / wp: for the few divisions of the prologue
};

constexpr int kPatchMaxLds = 96 * 1024;
constexpr int kPatchRawPitch = 128;  // bytes of a channel's rows in the raw copy: 32 lanes of one dword
constexpr int kPatchSteps = 16;      // k blocks per trip of the main loop = filter fragments in flight per wave

// a / d for 0 <= a < 2^22 and 0 < d < 2^22 from rd ~ 1 / d: a float quotient is at most one off.
__device__ __forceinline__ int div_small(int a, int d, float rd) {
    int q = static_cast<int>(static_cast<float>(a) * rd);
    const int r = a - q * d;
    q += (r >= d) ? 1 : 0;
    q -= (r < 0) ? 1 : 0;
    return q;
}

// TRACE: shader-clock stamps of every wave at the phase boundaries (start, raw rows in LDS, patch built, last MFMA
// retired, stores issued, stores retired), in the layout of the packed kernel's stamps.
template <int CBS, int EPI, bool EVEN, bool TRACE = false>
__global__ __launch_bounds__(256) void conv_i8_patch_kernel(const int8_t *__restrict__ PF, int M, int N, int K,
                                                            GemmEpilogue ep, ConvPatch cp) {
    extern __shared__ __attribute__((aligned(1024))) int8_t lds[];
    constexpr int S = kPatchSteps, C = CBS * 32, R = kPatchRawPitch;
    constexpr int TPI = S / CBS;  // taps per trip
    static_assert(S % CBS == 0 && C % 128 == 0, "channel blocks: 4 or 8");
    const int tid = threadIdx.x, lane = tid % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int KB = static_cast<int>(packed_k_blocks(K));
    const int rbA = (M + 31) / 32;
    const int tiles_m = (rbA + 3) / 4;
    const int tile_m = blockIdx.x % tiles_m, tile_n = blockIdx.x / tiles_m;
    const int n0 = tile_n * 64;
    const int P = cp.patch, wp = ep.cv_wp, per_img = ep.cv_hp * ep.cv_wp;
    unsigned long long stamp[kTraceWords] = {};
    auto mark = [&](int i) {
        if constexpr (TRACE) stamp[i] = __builtin_readcyclecounter();
    };
    if constexpr (TRACE) stamp[kTracePoints] = __builtin_amdgcn_s_memrealtime();
    mark(0);

    // ---- gather, step 1: requested before anything else ----
    int8_t *raw = lds + CBS * 2 * P * 16;  // [image slot][channel][R bytes]
    const int plane = cp.h * cp.w;
    const int img0 = __builtin_amdgcn_readfirstlane(div_small(n0, per_img, cp.r_per_img));
    const int local0 = n0 - img0 * per_img;
    const bool second = local0 + P > per_img && img0 + 1 < ep.cv_nb;  // the patch runs into the next image
    int y0 = __builtin_amdgcn_readfirstlane(div_small(local0, wp, cp.r_wp)) - cp.ph;
    y0 = y0 < 0 ? 0 : (y0 > cp.h - 1 ? cp.h - 1 : y0);
    const int lo4_0 = (y0 * cp.w) & ~3;  // (the next image is entered at its first row: its raw rows start at 0)
    const __amdgpu_buffer_rsrc_t rx =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(cp.x), 0, cp.x_bytes, 0x00020000);
    {
        const int d = tid % 32, csub = tid / 32;  // dword of the raw row, channel within a group of eight
        const int v0 = (img0 * C + csub) * plane + lo4_0 + 4 * d;
        int8_t *dst = raw + csub * R + 4 * d;
#pragma unroll
        for (int sl = 0; sl < 2; ++sl) {
            if (sl == 1 && !second) break;  // (uniform)
            const int vsrc = sl == 0 ? v0 : v0 + C * plane - lo4_0;
            int8_t *dsl = dst + sl * C * R;
            for (int c0 = 0; c0 < C; c0 += 128) {  // 16 loads in flight per thread and trip
                int t[16];
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    t[i] = __builtin_amdgcn_raw_buffer_load_b32(rx, vsrc, (c0 + i * 8) * plane, 0);
#pragma unroll
                for (int i = 0; i < 16; ++i) *reinterpret_cast<int *>(dsl + c0 * R + i * 8 * R) = t[i];
            }
        }
    }

    // ---- epilogue operands and the first filter fragments: their latency hides behind the gather ----
    size_t cv_out_base[2];
    bool cv_valid[2];
    float cv_s = 1.0f, cv_b = 0.0f, sa0 = 1.0f;
    int cv_c = 0;
    const int fb = tile_m * 4 + wave;  // this wave's filter block (past the last: computed and discarded)
    const int row0 = fb * 32;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int q = n0 + j * 32 + lane % 32;
        const int img = div_small(q, per_img, cp.r_per_img), rem = q - img * per_img;
        const int oh = div_small(rem, wp, cp.r_wp), ow = rem - oh * wp;
        cv_valid[j] = q < N && oh < ep.cv_ho && ow < ep.cv_wo;
        cv_out_base[j] = (size_t(img) * ep.cv_oc * ep.cv_ho + oh) * ep.cv_wo + ow;  // + oc * ho * wo
    }
    {
        if constexpr (EPI != EPI_I32) sa0 = ep.sa ? ep.sa[0] : ep.sa_scalar;
        const int m = row0 + lane % 32;
        const int mc = m < M ? m : M - 1;
        cv_c = ep.cv_corr_mul * ep.cv_wsum[mc];
        if constexpr (EPI != EPI_I32) {
            cv_s = sa0 * ep.sw[mc];
            if (ep.bias) cv_b = ep.bias[mc];
        }
    }
    // (a block past the filters: an empty buffer, zeros)
    const __amdgpu_buffer_rsrc_t rf = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t *>(PF) + size_t(fb < rbA ? fb : 0) * KB * 1024, 0, fb < rbA ? KB * 1024 : 0, 0x00020000);
    const int voff = lane * 16;
    auto load_f = [&](int kb) {
        return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rf, voff, kb * 1024, 0));
    };
    v4i wf[S];
#pragma unroll
    for (int u = 0; u < S; ++u) wf[u] = load_f(u);
    __syncthreads();
    mark(1);

    // ---- gather, step 2 ----
    {
        const int slots = P <= 128 ? 128 : 256, groups = 256 / slots;
        const int pl = tid & (slots - 1);
        const int grp = __builtin_amdgcn_readfirstlane(tid / slots);  // (slots >= a wave: uniform, and known to be)
        const int p = n0 + pl;
        const int img = div_small(p, per_img, cp.r_per_img), rem = p - img * per_img;
        const int yp = div_small(rem, wp, cp.r_wp);
        const int y = yp - cp.ph, xx = rem - yp * wp - cp.pw;
        const int sl = img - img0;
        const bool real = pl < P && p < N && y >= 0 && y < cp.h && xx >= 0 && xx < cp.w && sl < 2;
        const int8_t *src = raw + (real ? sl * C * R + y * cp.w + xx - (sl ? 0 : lo4_0) : 0);
        int8_t *dst = lds + pl * 16;
        const int per_grp = CBS / groups;  // channel blocks of this thread: grp * per_grp ..
#pragma unroll
        for (int k = 0; k < CBS; ++k) {
            if (k >= per_grp) break;  // (uniform)
            const int cb = grp * per_grp + k;
            const int8_t *s = src + cb * 32 * R;
            uint32_t wds[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t b0 = *reinterpret_cast<const uint8_t *>(s + (4 * i + 0) * R);
                const uint32_t b1 = *reinterpret_cast<const uint8_t *>(s + (4 * i + 1) * R);
                const uint32_t b2 = *reinterpret_cast<const uint8_t *>(s + (4 * i + 2) * R);
                const uint32_t b3 = *reinterpret_cast<const uint8_t *>(s + (4 * i + 3) * R);
                const uint32_t v = (b0 | (b1 << 8)) | ((b2 | (b3 << 8)) << 16);
                wds[i] = real ? v ^ 0x80808080u : cp.border;
            }
            if (pl < P) {
                *reinterpret_cast<v4i *>(dst + (cb * 2 + 0) * P * 16) = v4i{int(wds[0]), int(wds[1]), int(wds[2]), int(wds[3])};
                *reinterpret_cast<v4i *>(dst + (cb * 2 + 1) * P * 16) = v4i{int(wds[4]), int(wds[5]), int(wds[6]), int(wds[7])};
            }
        }
    }
    __syncthreads();
    mark(2);

    // ---- main loop: k block = (tap, channel block), tap-major; a trip covers S k blocks = TPI whole taps ----
    // The window fragment of (tap, channel block cb) lies at tap offset + cb * 2 * P * 16 + this lane's place: the
    // lane part per channel block is kept in registers, the tap offset is a scalar, worked out once per tap.
    int vcb[CBS];
#pragma unroll
    for (int cb = 0; cb < CBS; ++cb) vcb[cb] = ((cb * 2 + lane / 32) * P + lane % 32) * 16;
    int ty = 0, tx = 0;
    // (past the taps the filters are zero: any fragment inside the patch will do, here the last tap row's)
    auto tap_offset = [&]() { return ((ty < cp.kh ? ty : cp.kh - 1) * wp + tx) * 16; };
    auto next_tap = [&]() {
        const int wrap = tx + 1 == ep.cv_kw ? 1 : 0;
        tx = wrap ? 0 : tx + 1;
        ty += wrap;
    };
    int tb[TPI], tbn[TPI];  // tap offsets of this trip and of the next
#pragma unroll
    for (int t = 0; t < TPI; ++t) {
        tb[t] = tap_offset();
        next_tap();
    }
#pragma unroll
    for (int t = 0; t < TPI; ++t) {
        tbn[t] = tap_offset();
        next_tap();
    }
    auto load_img = [&](int step, int j) {  // step: 0 .. 2 S - 1, counted from the start of this trip
        const int t = (step % S) / CBS, cb = step % CBS;
        const int base = step < S ? tb[t] : tbn[t];
        return *reinterpret_cast<const v4i *>(lds + base + vcb[cb] + j * 32 * 16);
    };
    v16i acc[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0;
    constexpr int ID = 4;  // window fragments are read from LDS four k blocks ahead
    static_assert(S % ID == 0, "static slots");
    v4i im[ID][2];
#pragma unroll
    for (int u = 0; u < ID; ++u) {
        im[u][0] = load_img(u, 0);
        im[u][1] = load_img(u, 1);
    }
    const int rounds_end = (KB + S - 1) / S * S;
    for (int kb0 = 0; kb0 < rounds_end; kb0 += S) {
#pragma unroll
        for (int u = 0; u < S; ++u) {
            acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[u], im[u % ID][0], acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[u], im[u % ID][1], acc[1], 0, 0, 0);
            wf[u] = load_f(kb0 + u + S);  // (past the last k block: beyond the buffer, zeros)
            im[u % ID][0] = load_img(u + ID, 0);
            im[u % ID][1] = load_img(u + ID, 1);
        }
#pragma unroll
        for (int t = 0; t < TPI; ++t) {
            tb[t] = tbn[t];
            tbn[t] = tap_offset();
            next_tap();
        }
    }

    v16i own[1][2];
#pragma unroll
    for (int j = 0; j < 2; ++j) own[0][j] = acc[j];
    if constexpr (TRACE) {
        // (the stamp waits for the accumulators: the last MFMA has retired)
        asm volatile("s_nop 0" ::"a"(own[0][0]), "a"(own[0][1]));
    }
    mark(3);
    conv_store_block<2, EPI, EVEN>(own, ep, M, row0, lane, cv_out_base, cv_valid, cv_c, cv_s, cv_b);
    if constexpr (TRACE) {
        mark(4);
        wait_vmcnt<0>();
        mark(5);
        stamp[kTracePoints + 1] = __builtin_amdgcn_s_memrealtime();
        if (lane == 0) {
            unsigned long long *t = ep.trace + (size_t(blockIdx.x) * 4 + wave) * kTraceWords;
#pragma unroll
            for (int i = 0; i < kTraceWords; ++i) t[i] = stamp[i];
        }
    }
}

// Whether the patch form takes this convolution, and its LDS bytes: 128 or 256 channels (the main loop is unrolled
// over the channel blocks of whole taps); planes of a multiple of 4 bytes and raw rows of at most 128 bytes (they
// are fetched as aligned dwords, one per lane); a patch that reaches into at most two images (an image of the
// padded grid is at least a patch long); pixel counts small enough for the float quotients of the prologue.
static inline bool conv_patch_fits(int c, int h, int w, int hp, int wp, int kh, int kw, long long padded_pixels,
                                   int *patch, int *lds_bytes) {
    const int p = 64 + (kh - 1) * wp + kw - 1;
    const int rows_bytes = ((p - 1) / wp + 2) * w + 3;
    *patch = p;
    *lds_bytes = (c / 32) * 2 * p * 16 + 2 * c * kPatchRawPitch;
    return (c == 128 || c == 256) && p <= 256 && rows_bytes <= kPatchRawPitch && (h * w) % 4 == 0 && hp * wp >= p &&
           padded_pixels + 256 < (1 << 22) && *lds_bytes <= kPatchMaxLds;
}

template <int CBS, int EPI, bool EVEN, bool TRACE = false>
static int32_t launch_conv_patch(hipq_ctx *ctx, const int8_t *filters, int M, int N, int K, const GemmEpilogue &ep,
                                 const ConvPatch &cp, int lds_bytes) {
    auto kernel = conv_i8_patch_kernel<CBS, EPI, EVEN, TRACE>;
    static bool configured[16] = {false};  // per device: raise the dynamic LDS limit once
    if (ctx->device < 16 && !configured[ctx->device]) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, kPatchMaxLds);
        if (e != hipSuccess)
            return fail(HIPQ_DEVICE_ERROR, "conv2d (patch): cannot reserve %d bytes of LDS: %s", kPatchMaxLds,
                        hipGetErrorString(e));
        configured[ctx->device] = true;
    }
    const int tiles_m = ((M + 31) / 32 + 3) / 4, tiles_n = (N + 63) / 64;
    GemmEpilogue placed = ep;
    if constexpr (TRACE) {
        // Phase stamps (hipq_ctx_set_trace_buffer): only if the buffer holds every wave's record.
        if (ctx->trace_bytes < size_t(tiles_m) * tiles_n * 4 * kTraceWords * sizeof(unsigned long long))
            return launch_conv_patch<CBS, EPI, EVEN, false>(ctx, filters, M, N, K, ep, cp, lds_bytes);
        placed.trace = static_cast<unsigned long long *>(ctx->trace);
    }
    hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n), dim3(256), lds_bytes, ctx->stream, filters, M, N, K, placed, cp);
    return check_launch("conv2d (patch)");
}

}  // namespace hipq
