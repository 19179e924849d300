// Device kernels shared by the Linear (hipq_gemm.hip) and Conv2d (hipq_conv.hip) entry points:
// the register-staged and the deep-pipelined int8 MFMA GEMM.
#pragma once

#include <cstdlib>

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
    const float *residual = nullptr;  // fp32 epilogue only: added after the bias, [M,N]; may alias out
    // Implicit-GEMM convolution (packed kernel, CONV): the row operand holds the packed filters, the column
    // operand is the padded int8 image as [channel block of 32][pixel][32 bytes]; column q is the window whose
    // top-left tap is padded pixel q = (n * hp + y) * wp + x, and K runs over (tap, channel).
    int cv_kw = 0, cv_wp = 0, cv_hp = 0, cv_c = 0;
    int cv_ho = 0, cv_wo = 0, cv_oc = 0, cv_nb = 0;
    const int32_t *cv_wsum = nullptr;  // [oc] sum of the filter's int8 weights
    int cv_corr_mul = 0;               // 128 - zp_in: accumulator += cv_corr_mul * cv_wsum[oc]
    const int32_t *cv_zp_in = nullptr; // when set: the input zero point on the device, used instead of cv_corr_mul
    int cv_pixels = 0;                 // pixels per channel block of the image buffer (with slack)
    int cv_kblocks = 0;                // taps * (c / 32): the k blocks that hold data
    float sa_scalar = 1.0f;            // activation scale used when sa is null
    float s_out_inv = 0.0f;            // recip_for_div(s_out), or 0 to divide directly (requantize only)
    // Tiles per XCD along M and N (pipelined kernel): the 8 XCDs each take a gm x gn rectangle of
    // tiles.  0 = not set (plain id order).
    int xcd_gm = 0, xcd_gn = 0;
    // Persistent kernel: how often a bounded wait polls before it gives up, and the device word
    // (owned by the context) in which a give-up is recorded.
    int spin_limit = 1 << 20;
    uint32_t *wait_error = nullptr;
    // Packed kernel, tuning aid: when set, every wave records the shader clock at its phase boundaries
    // (kTraceWords values per wave, workgroup-major: kTracePoints shader-clock stamps, then the constant
    // 100 MHz counter at the first and the last of them).
    unsigned long long *trace = nullptr;
    // Packed kernel: 1 = the activations were written by the kernel just before this one on the stream
    // (still in the memory-side cache), so the XCDs need not be kept from reading the same lines at once.
    int fresh_activations = 0;
};
constexpr int kTracePoints = 6, kTraceWords = 8;

// Defined with the packed kernel (hipq_gemm_packed.hip), used by the convolution.
// Row-major int8 [rows, k] -> fragment-packed operand (packed_operand_bytes(rows, k) bytes at dst).
int32_t pack_rows(hipq_ctx *ctx, const int8_t *src, size_t rows, size_t k, int8_t *dst);
size_t packed_operand_bytes(size_t rows, size_t k);
// Implicit-GEMM convolution: `filters` packed [M = output channels, K = taps x channels], `image` in
// [channel block][pixel][32] order, N = padded pixels; ep carries the cv_* geometry.  epi: EPI_I32 / _F32 / _I8.
int32_t conv_gemm_packed(hipq_ctx *ctx, const int8_t *filters, const int8_t *image, int M, int N, int K,
                         const GemmEpilogue &ep, int epi, bool even);
// The same convolution in one launch, from the u8 NCHW input itself (hipq_conv_patch.h): `fits` says whether
// that form takes the geometry (c channels, padded width wp, kh x kw taps).
bool conv_patch_applicable(int nb, int c, int h, int w, int hp, int wp, int kh, int kw);
int32_t conv_gemm_patch(hipq_ctx *ctx, const int8_t *filters, const uint8_t *x, size_t x_bytes, int zp_in, int h, int w,
                        int ph, int pw, int kh, int M, int N, int K, const GemmEpilogue &ep, int epi, bool even);

// Host-side twin of recip_for_div: the correctly rounded 1/b if it is a normal number, else 0.
static inline float host_recip_for_div(float b) {
    const float y = 1.0f / b;
    const float ay = y < 0.0f ? -y : y;
    return (ay >= 1.17549435e-38f && ay <= 3.40282347e+38f) ? y : 0.0f;
}

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
            if (ep.residual && n + r < N) t = t + ep.residual[off + r];
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
                q[r] = to_int_nan0(clamp_keep_nan(round_mode<EVEN>(div_rn(v[r], ep.s_out, ep.s_out_inv)) + zpf, -128.0f, 127.0f));
            if (vec) {
                *reinterpret_cast<uint32_t *>(o + off) = pack4(q[0], q[1], q[2], q[3]);
            } else {
                for (int r = 0; r < 4; ++r)
                    if (n + r < N) o[off + r] = static_cast<int8_t>(q[r]);
            }
        }
    }
}

// Maps the linear workgroup id to a tile.  Workgroups are handed to the 8 XCDs round robin (ids
// congruent modulo 8 share an XCD and its L2), so XCD x is given a gm x gn rectangle of tiles:
// it then pulls gm row blocks of the first operand and gn panels of the second through its L2
// once each.  The host picks the rectangle with the smallest gm*BM + gn*BN (for M = 512,
// N = 4096: all 4 row blocks x 8 weight panels, each weight panel read from HBM by one XCD only;
// for a tall M x 256 product: 8 row blocks x all 4 panels, instead of every XCD streaming half
// of the tall operand).
// a / d and a % d for small non-negative wave-uniform values; a power of two (the usual case) costs a
// shift instead of the ~25 instructions of an integer division, which sit in front of a kernel's first load.
__device__ __forceinline__ void divmod_uniform(int a, int d, int *q, int *r) {
    if ((d & (d - 1)) == 0) {
        *q = a >> (__builtin_ffs(d) - 1);
        *r = a & (d - 1);
    } else {
        *q = a / d;
        *r = a % d;
    }
}

// Tile of slot i (0, 1, ...) of XCD x: with a rectangle (gm > 0) the i-th tile of the XCD's rectangle, column
// major; without one, tile x + 8 * i in id order.
__device__ __forceinline__ void tile_of_xcd_slot(int tiles_m, int tiles_n, int gm, int gn, int x, int i, int *tm,
                                                 int *tn) {
    if (gm > 0) {
        int blocks_m, unused, xq, xr, iq, ir;   // rectangles along M
        divmod_uniform(tiles_m, gm, &blocks_m, &unused);
        divmod_uniform(x, blocks_m, &xq, &xr);
        divmod_uniform(i, gm, &iq, &ir);
        *tm = xr * gm + ir;
        *tn = xq * gn + iq;
        return;
    }
    const int b = x + 8 * i;
    *tm = b % tiles_m;
    *tn = b / tiles_m;
}

__device__ __forceinline__ void tile_of_block(int tiles_m, int tiles_n, int gm, int gn, int *tm, int *tn) {
    const int b = blockIdx.x;
    tile_of_xcd_slot(tiles_m, tiles_n, gm, gn, b % 8, b / 8, tm, tn);  // XCD, index within the XCD's rectangle
}

// Host side: the rectangle for tile_of_block, or (0, 0) when the tile grid does not split into 8
// equal rectangles.
static inline void pick_xcd_rectangle(int tiles_m, int tiles_n, int bm, int bn, int *gm_out, int *gn_out) {
    *gm_out = *gn_out = 0;
    const long nblk = static_cast<long>(tiles_m) * tiles_n;
    if (nblk % 8 != 0) return;
    const long per = nblk / 8;
    long best = -1;
    for (int gm = 1; gm <= tiles_m; ++gm) {
        if (tiles_m % gm != 0 || per % gm != 0) continue;
        const long gn = per / gm;
        if (gn > tiles_n || tiles_n % gn != 0) continue;
        const long cost = static_cast<long>(gm) * bm + gn * bn;
        if (best < 0 || cost < best) {
            best = cost;
            *gm_out = gm;
            *gn_out = static_cast<int>(gn);
        }
    }
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
    tile_of_block((M + BM - 1) / BM, (N + BN - 1) / BN, ep.xcd_gm, ep.xcd_gn, &tile_m, &tile_n);
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

// ---------------------------------------------------------------------------
// Deep-pipelined kernel for K % 128 == 0 (the shapes that matter).
//
// Occupancy for the headline shape is one workgroup per CU (256 tiles on 256
// CUs), so all latency hiding happens inside the workgroup:
//   * STAGES K-tiles of 128 bytes live in LDS (up to 144 KiB of the CU's 160 KiB)
//     and are filled by global_load_lds_dwordx4, which moves 16 bytes per lane
//     from global memory straight into LDS without passing through VGPRs.  A
//     wave instruction fills 1 KiB of contiguous LDS, so the XOR swizzle is
//     applied on the global side: lane l fetches the chunk that belongs in slot l.
//   * the MFMA fragments of stage kt+1 are read from LDS into a second register
//     set while the MFMAs of stage kt run, so LDS latency is off the MFMA path
//     even with a single wave per SIMD.
//   * vmcnt counts a wave's outstanding fills in order; waiting until only the
//     newest stages are outstanding, then a bare workgroup barrier, publishes a
//     stage to every wave and frees the buffer that the next fill reuses.
// v_mfma_i32_32x32x32_i8 is used (it sustains a higher rate than the 16x16x64
// form with one wave per SIMD).  The activation fragment is the row operand and
// the weight fragment the column operand, so a lane owns one output channel n
// and a wave-wide dword store writes 128 contiguous bytes of two output rows.
//
// Wave roles: WM x WN x WK.  WK > 1 splits the four k-steps of a stage between
// waves; the partial accumulators are summed through LDS after the main loop.
// Integer addition is associative, so the result is bit-identical for every WK.
typedef int v16i __attribute__((ext_vector_type(16)));

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    // gfx9 s_waitcnt encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | (0x7 << 4) | (0xF << 8));
}

__device__ __forceinline__ void wait_lgkmcnt0() {
    __builtin_amdgcn_s_waitcnt(0xF | (0x3 << 14) | (0x7 << 4) | (0x0 << 8));
}

template <int PER_STAGE, int MAX_STAGES>
__device__ __forceinline__ void wait_stages_outstanding(int stages) {
    // `stages` is wave-uniform; the immediate of s_waitcnt must be a constant.
    if constexpr (MAX_STAGES > 0) {
        if (stages >= MAX_STAGES) {
            wait_vmcnt<PER_STAGE * MAX_STAGES>();
            return;
        }
        wait_stages_outstanding<PER_STAGE, MAX_STAGES - 1>(stages);
    } else {
        wait_vmcnt<0>();
    }
}

// Sum of the K-split partial accumulators of a workgroup through LDS (integer adds: the result
// does not depend on the order).  Row block i of a wave-group tile is owned by wave (i % WK) of
// the group; every other wave of the group parks its partial for it.  Needs
// (waves / WK) * FM * (WK - 1) * FN * 4 KiB of LDS at `lds`, free of other use by the time the
// first wave arrives (LDS_BUSY: the main loop used it, so a workgroup barrier comes first).
template <int FM, int FN, int WK, bool LDS_BUSY = true>
__device__ __forceinline__ void ksplit_reduce(v16i (&acc)[FM][FN], int8_t *lds, int wk, int wmn, int lane) {
    if constexpr (WK > 1) {
        if constexpr (LDS_BUSY) __syncthreads();
        v4i *red = reinterpret_cast<v4i *>(lds);
        auto slot = [&](int i, int srcw, int j, int g) {
            const int owner = i % WK;
            const int sidx = (srcw - owner - 1 + WK) % WK;  // 0 .. WK-2
            return ((((wmn * FM + i) * (WK - 1) + sidx) * FN + j) * 4 + g) * kWave + lane;
        };
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            if (i % WK == wk) continue;
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    red[slot(i, wk, j, g)] =
                        v4i{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            if (i % WK != wk) continue;
#pragma unroll
            for (int p = 1; p < WK; ++p) {
                const int srcw = (wk + p) % WK;
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const v4i t = red[slot(i, srcw, j, g)];
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[i][j][4 * g + r] += t[r];
                    }
            }
        }
    }
}

// Dequantize / requantize / plain int32 epilogue of a wave's FM x FN grid of 32x32 accumulator
// blocks whose first row is `mrow0` (row blocks not owned by K-split wave `wk` are skipped).
// 32x32 accumulator block: lane holds column n = lane%32 and rows m = 8*(r/4) + 4*(lane/32) + r%4
// for r = 0..15.  nn / swv / bv: the lane's output channel per column block, its weight scale and
// bias; sa0: the per-tensor activation scale.
template <int FM, int FN, int WK, int EPI, bool EVEN>
__device__ __forceinline__ void store_tile(v16i (&acc)[FM][FN], const GemmEpilogue &ep, int M, int N, int mrow0,
                                           int wk, int lane, const int (&nn)[FN], const float (&swv)[FN],
                                           const float (&bv)[FN], float sa0) {
    const float zpf = static_cast<float>(ep.zp_out);
    const bool has_bias = ep.bias != nullptr;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
        if (WK > 1 && i % WK != wk) continue;
        // All loads of the row block first, then arithmetic and stores only: a load between
        // stores would wait for every earlier store to retire (stores count in vmcnt too).
        float s_row[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) s_row[r] = sa0;
        if constexpr (EPI != EPI_I32) {
            if (ep.sa_per_row) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = mrow0 + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
                    s_row[r] = ep.sa[m < M ? m : M - 1];
                }
            }
        }
        // Combined scales for the whole row block, computed before the first store so that no
        // loaded value is first touched between stores.
        float s_comb[16][FN], res[16][FN];
#pragma unroll
        for (int r = 0; r < 16; ++r)
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                s_comb[r][j] = s_row[r] * swv[j];
                res[r][j] = 0.0f;
            }
        if constexpr (EPI == EPI_F32) {
            if (ep.residual) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = mrow0 + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
#pragma unroll
                    for (int j = 0; j < FN; ++j)
                        if (m < M && nn[j] < N) res[r][j] = ep.residual[size_t(m) * N + nn[j]];
                }
            }
        }
        // Every load of this wave has landed (and the compiler's wait tracking knows it), so
        // the stores below are issued back to back without waiting on one another.
        wait_vmcnt<0>();
        if constexpr (EPI == EPI_I8) {
            // int8 output as dwords.  A lane holds one column of 16 rows; the four lanes of a quad
            // hold four consecutive columns.  Per group of four rows each lane packs its four
            // bytes, the quad transposes the 4x4 bytes (quad_byte_transpose: two lane swaps, two byte
            // permutes), and every lane stores one dword = four consecutive columns of one row:
            // a quarter of the store instructions of the byte form, none of them sub-dword.
            if (N % 4 == 0 && (reinterpret_cast<uintptr_t>(ep.out) & 3u) == 0) {
                const int qd = lane % 4;
                const uint32_t sel1 = (qd & 1) ? 0x03070105u : 0x06020400u, sel2 = (qd & 2) ? 0x03020706u : 0x05040100u;
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    const int col = nn[j] - qd;  // first column of the quad; N % 4 == 0 keeps quads whole
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        int q[4];
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            float v = static_cast<float>(acc[i][j][4 * t + k]) * s_comb[4 * t + k][j];
                            if (has_bias) v = v + bv[j];
                            q[k] = clamp_to_int(round_mode<EVEN>(div_rn(v, ep.s_out, ep.s_out_inv)) + zpf, -128, 127);
                        }
                        // byte k of the packed dword = row 8t + 4*(lane/32) + k
                        const uint32_t word = quad_byte_transpose(pack4(q[0], q[1], q[2], q[3]), sel1, sel2);
                        const int m = mrow0 + i * 32 + 8 * t + 4 * (lane / 32) + qd;
                        if (m < M && col < N)
                            __builtin_nontemporal_store(word, reinterpret_cast<uint32_t *>(static_cast<int8_t *>(ep.out) +
                                                                                           size_t(m) * N + col));
                    }
                }
                continue;
            }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = mrow0 + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
            if (m >= M) continue;
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                if (nn[j] >= N) continue;
                const size_t off = size_t(m) * N + nn[j];
                if constexpr (EPI == EPI_I32) {
                    __builtin_nontemporal_store(acc[i][j][r], static_cast<int32_t *>(ep.out) + off);
                } else {
                    float v = static_cast<float>(acc[i][j][r]) * s_comb[r][j];
                    if (has_bias) v = v + bv[j];
                    if constexpr (EPI == EPI_F32) {
                        if (ep.residual) v = v + res[r][j];
                        __builtin_nontemporal_store(v, static_cast<float *>(ep.out) + off);
                    } else {
                        const int q = clamp_to_int(round_mode<EVEN>(div_rn(v, ep.s_out, ep.s_out_inv)) + zpf, -128, 127);
                        __builtin_nontemporal_store(static_cast<int8_t>(q), static_cast<int8_t *>(ep.out) + off);
                    }
                }
            }
        }
    }
}

// PW producer waves do nothing but issue the fills; WM*WN*WK consumer waves do
// nothing but LDS reads and MFMAs.  A wave issues in order, and a fill blocks its
// wave while the texture path is busy, so mixing fills and MFMAs in one wave
// serialises the two pipes; with the roles split, MFMA issue never waits behind a
// memory instruction.  All waves meet at one barrier per K-tile.
template <int BM, int BN, int STAGES, int PW, int WM, int WN, int WK, int EPI, bool EVEN>
__global__ __launch_bounds__((PW + WM * WN * WK) * kWave) void gemm_i8_pipe_kernel(const int8_t *__restrict__ A,
                                                                                    const int8_t *__restrict__ W,
                                                                                    int M, int N, int K,
                                                                                    GemmEpilogue ep) {
    constexpr int BK = 128;
    constexpr int CPR = BK / 16;   // 16-byte chunks per tile row
    constexpr int RPI = 1024 / BK;  // tile rows filled by one wave-wide 1 KiB load
    constexpr int IPS = (BM + BN) / RPI;  // load instructions per stage
    static_assert(BM % RPI == 0 && IPS % PW == 0, "stage loads divide evenly between producer waves");
    constexpr int IPW = IPS / PW;
    static_assert(IPW * STAGES < 64, "outstanding loads must fit vmcnt");
    constexpr int STAGE = (BM + BN) * BK;
    constexpr int TM = BM / WM, TN = BN / WN;
    constexpr int FM = TM / 32, FN = TN / 32;
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile is made of 32x32 MFMA blocks");
    constexpr int KS = BK / 32;  // MFMA k-steps per stage
    static_assert(KS % WK == 0, "k-steps of a stage divide between the K-split waves");
    constexpr int KSW = KS / WK;
    static_assert(FM % WK == 0, "after the K-split reduction each wave owns FM/WK row blocks");
    constexpr int RED_BYTES = WM * WN * FM * (WK - 1) * FN * 4 * kWave * 16;
    static_assert(RED_BYTES <= STAGES * STAGE, "partial sums fit the pipeline buffers");

    extern __shared__ __attribute__((aligned(1024))) int8_t lds[];

    int tile_m, tile_n;
    tile_of_block((M + BM - 1) / BM, (N + BN - 1) / BN, ep.xcd_gm, ep.xcd_gn, &tile_m, &tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const int nk = K / BK;

    if (wave < PW) {
        // ---------------- producer ----------------
        const int8_t *src[IPW];
#pragma unroll
        for (int j = 0; j < IPW; ++j) {
            const int q = wave * IPW + j;
            const int trow = q * RPI + lane / CPR;  // row in the stacked [A rows | W rows] tile
            const int col = (lane % CPR) ^ ((trow >> 1) & 7);
            if (trow < BM) {
                int gm = m0 + trow;
                gm = gm < M ? gm : M - 1;  // rows past the edge are computed and discarded
                src[j] = A + size_t(gm) * K + col * 16;
            } else {
                int gn = n0 + (trow - BM);
                gn = gn < N ? gn : N - 1;
                src[j] = W + size_t(gn) * K + col * 16;
            }
        }
        auto issue_stage = [&](int kt, int buf) {
            int8_t *base = lds + buf * STAGE + wave * (IPW * 1024);
            const size_t koff_row = size_t(kt) * BK;
#pragma unroll
            for (int j = 0; j < IPW; ++j)
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void *)(src[j] + koff_row),
                    (__attribute__((address_space(3))) void *)(base + j * 1024), 16, 0, 0);
        };
        // Two stages before the first barrier so the consumers start after one memory
        // latency; the remaining buffers are requested while they work on stage 0.
        int issued = 0;  // stages [0, issued) have been requested
        for (; issued < 2 && issued < nk; ++issued) issue_stage(issued, issued);
        wait_stages_outstanding<IPW, STAGES - 1>(issued - 1);  // stage 0 has landed
        __builtin_amdgcn_s_barrier();
        for (; issued < STAGES && issued < nk; ++issued) issue_stage(issued, issued);
        for (int kt = 0; kt < nk; ++kt) {
            // Requests so far cover stages <= kt+STAGES-1; stage kt+1 must have landed.
            int newer = nk - 2 - kt;
            if (newer > STAGES - 2) newer = STAGES - 2;
            if (newer < 0) newer = 0;
            wait_stages_outstanding<IPW, STAGES - 2>(newer);
            // A bare barrier: __syncthreads() carries a release fence that would drain every
            // outstanding fill (vmcnt(0)) and serialise the pipeline.
            __builtin_amdgcn_s_barrier();
            // Every consumer holds stage kt in registers: its buffer is free for stage kt+STAGES.
            if (kt + STAGES < nk) issue_stage(kt + STAGES, kt % STAGES);
        }
        if constexpr (WK > 1) {
            __syncthreads();
            __syncthreads();
        }
        return;
    }

    // ---------------- consumer ----------------
    const int cw = wave - PW;
    const int wk = cw / (WM * WN), wmn = cw % (WM * WN);
    const int wm = wmn % WM, wn = wmn / WM;

    // Epilogue operands are fetched now so their latency hides behind the main loop.
    float swv[FN], bv[FN], sa0 = 1.0f;
    int nn[FN];
#pragma unroll
    for (int j = 0; j < FN; ++j) {
        nn[j] = n0 + wn * TN + j * 32 + lane % 32;
        const int nc = nn[j] < N ? nn[j] : N - 1;
        swv[j] = 1.0f;
        bv[j] = 0.0f;
        if constexpr (EPI != EPI_I32) {
            swv[j] = ep.sw[nc];
            if (ep.bias) bv[j] = ep.bias[nc];
        }
    }
    if constexpr (EPI != EPI_I32)
        if (!ep.sa_per_row) sa0 = ep.sa ? ep.sa[0] : ep.sa_scalar;
    // LDS byte offsets (within a stage) of this lane's fragment reads.
    int offA[FM][KSW], offW[FN][KSW];
#pragma unroll
    for (int s = 0; s < KSW; ++s) {
        const int col = (s * WK + wk) * 2 + lane / 32;
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            const int row = wm * TM + i * 32 + lane % 32;
            offA[i][s] = row * BK + ((col ^ ((row >> 1) & 7)) * 16);
        }
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const int row = BM + wn * TN + j * 32 + lane % 32;  // stacked-tile row
            offW[j][s] = row * BK + ((col ^ ((row >> 1) & 7)) * 16);
        }
    }
    v4i fa[2][KSW][FM], fw[2][KSW][FN];
    auto read_frags = [&](int buf, int set) {
        const int8_t *st = lds + buf * STAGE;
#pragma unroll
        for (int s = 0; s < KSW; ++s) {
#pragma unroll
            for (int i = 0; i < FM; ++i) fa[set][s][i] = *reinterpret_cast<const v4i *>(st + offA[i][s]);
#pragma unroll
            for (int j = 0; j < FN; ++j) fw[set][s][j] = *reinterpret_cast<const v4i *>(st + offW[j][s]);
        }
    };

    v16i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    auto compute = [&](int set) {
#pragma unroll
        for (int s = 0; s < KSW; ++s)
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[set][s][i], fw[set][s][j], acc[i][j], 0, 0, 0);
    };
    auto iteration = [&](int kt, int set) {
        wait_lgkmcnt0();  // this wave's fragment reads of stage kt are in registers
        asm volatile("" ::: "memory");  // compiler-only fence: keep LDS reads on their side of the barrier
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // Unconditional: after the last stage this re-reads a resident buffer whose values are
        // never used, which keeps reads and MFMAs in one basic block for the interleave below.
        read_frags((kt + 1) % STAGES, set ^ 1);
        compute(set);
        // Issue order: one MFMA, then one fragment read, ...: the reads slip into the issue
        // slots between MFMAs (an MFMA occupies the matrix pipe for 32 cycles) instead of
        // delaying the first MFMA of the stage.
#pragma unroll
        for (int q = 0; q < KSW * FM * FN; ++q) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (q < KSW * (FM + FN)) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
    };
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();  // stage 0 published
    asm volatile("" ::: "memory");
    read_frags(0, 0);
    int kt = 0;
    for (; kt + 1 < nk; kt += 2) {
        iteration(kt, 0);
        iteration(kt + 1, 1);
    }
    if (kt < nk) iteration(kt, 0);

    if constexpr (WK > 1) ksplit_reduce<FM, FN, WK>(acc, lds, wk, wmn, lane);
    store_tile<FM, FN, WK, EPI, EVEN>(acc, ep, M, N, m0 + wm * TM, wk, lane, nn, swv, bv, sa0);
}

template <int BM, int BN, int STAGES, int PW, int WM, int WN, int WK, int EPI, bool EVEN>
static int32_t launch_pipe(hipq_ctx *ctx, const int8_t *a, const int8_t *w, int M, int N, int K,
                           const GemmEpilogue &ep) {
    constexpr int kLds = STAGES * (BM + BN) * 128;
    constexpr int kThreads = (PW + WM * WN * WK) * kWave;
    auto kernel = gemm_i8_pipe_kernel<BM, BN, STAGES, PW, WM, WN, WK, EPI, EVEN>;
    static bool configured[16] = {false};  // per device: raise the dynamic LDS limit once
    if (ctx->device < 16 && !configured[ctx->device]) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
        if (e != hipSuccess)
            return fail(HIPQ_DEVICE_ERROR, "gemm_i8: cannot reserve %d bytes of LDS: %s", kLds, hipGetErrorString(e));
        configured[ctx->device] = true;
    }
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    GemmEpilogue placed = ep;
    pick_xcd_rectangle(tiles_m, tiles_n, BM, BN, &placed.xcd_gm, &placed.xcd_gn);
    hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n), dim3(kThreads), kLds, ctx->stream, a, w, M, N, K, placed);
    return check_launch("gemm_i8 (pipelined)");
}

}  // namespace hipq
