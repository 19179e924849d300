// int8 GEMM on fragment-packed operands: no LDS staging in the main loop.
//
// Packed layout of an int8 matrix [rows, K] (K contiguous):
//   P[row block rb = row / 32][k block kb = k / 32][1 KiB fragment]
// and inside a fragment lane l (16 bytes) holds row 32*rb + l%32, bytes 32*kb + 16*(l/32) .. +15:
// exactly one operand of v_mfma_i32_32x32x32_i8, fetched by ONE fully coalesced wave instruction
// (64 lanes x 16 bytes = 1 KiB contiguous).  Rows are padded to a multiple of 32 and the k blocks
// to a multiple of 4 (kPackKbAlign); k padding is zero in both operands, so it adds nothing.
//
// Why: with one 128x64 output tile per CU (256 tiles on 256 CUs for M = 512, N = 4096) a CU has to
// pull (128 + 64) * K bytes through its vector-memory path whatever the kernel does, and that
// path moves 64 bytes per clock.  Staging through LDS adds a second bottleneck (fills + fragment
// reads on one 128 B/clk port) and a barrier per K-tile.  Here the four waves of a workgroup split
// K (k block kb goes to wave kb % 4), every wave owns the whole 128x64 tile for its k blocks, and
// each operand byte enters the CU exactly once, straight into the registers that feed the MFMA:
// no LDS traffic, no barriers and no cross-wave dependency until the final 4-way sum of the
// partial accumulators (through LDS, integer adds, order independent).
#pragma once

#include "hipq_gemm_kernels.h"

namespace hipq {

constexpr int kPackKbAlign = 4;  // k blocks per row block are padded to a multiple of the K-split

__host__ __device__ inline size_t packed_row_blocks(size_t rows) { return (rows + 31) / 32; }
__host__ __device__ inline size_t packed_k_blocks(size_t k) {
    return ((k + 31) / 32 + kPackKbAlign - 1) / kPackKbAlign * kPackKbAlign;
}
__host__ __device__ inline size_t packed_bytes(size_t rows, size_t k) {
    return packed_row_blocks(rows) * packed_k_blocks(k) * 1024;
}

// TMB x TNB row blocks of 32 per workgroup tile; D register stages of (TMB + TNB) KiB per wave in
// flight.  Loads are buffer loads with a constant per-lane offset and scalar (SGPR) fragment
// offsets, so the loop spends no vector instruction on addressing.
//
// Sibling tiles (same weight panel, different tile_m) run on CUs of one XCD at the same time; each
// starts its K loop a quarter of the way further on (`rot`), so the four of them miss on
// different weight lines and every line is fetched from HBM by one of them and found in the L2 by
// the other three, instead of all four waiting on the same miss.
template <int TMB, int TNB, int D, int EPI, bool EVEN>
__global__ __launch_bounds__(256) void gemm_i8_packed_kernel(const int8_t *__restrict__ PA,
                                                             const int8_t *__restrict__ PW, int M, int N, int K,
                                                             GemmEpilogue ep) {
    extern __shared__ __attribute__((aligned(1024))) int8_t lds[];
    constexpr int WK = 4;
    const int KB = static_cast<int>(packed_k_blocks(K));
    const int rbA = (M + 31) / 32, rbW = (N + 31) / 32;
    const int tiles_m = (rbA + TMB - 1) / TMB, tiles_n = (rbW + TNB - 1) / TNB;
    int tile_m, tile_n;
    tile_of_block(tiles_m, tiles_n, ep.xcd_gm, ep.xcd_gn, &tile_m, &tile_n);
    const int m0 = tile_m * TMB * 32, n0 = tile_n * TNB * 32;
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);

    // Epilogue operands first: their latency hides behind the main loop.
    float swv[TNB], bv[TNB], sa0 = 1.0f;
    int nn[TNB];
#pragma unroll
    for (int j = 0; j < TNB; ++j) {
        nn[j] = n0 + j * 32 + lane % 32;
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

    // Byte offsets of this wave's first fragment of every row block of the tile (row blocks past
    // the matrix repeat the last one: computed and discarded).  Operands are below 2 GiB.
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(PA), 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(PW), 0, 0x7fffffff, 0x00020000);
    int soa[TMB], sow[TNB];
#pragma unroll
    for (int i = 0; i < TMB; ++i) {
        int rb = tile_m * TMB + i;
        rb = rb < rbA ? rb : rbA - 1;
        soa[i] = (rb * KB + wave) * 1024;
    }
#pragma unroll
    for (int j = 0; j < TNB; ++j) {
        int rb = tile_n * TNB + j;
        rb = rb < rbW ? rb : rbW - 1;
        sow[j] = (rb * KB + wave) * 1024;
    }
    const int steps = KB / WK;  // k blocks per wave
    const int rot = (tile_m % 4) * (steps / 4);
    const int voff = lane * 16;

    v4i fa[D][TMB], fb[D][TNB];
    auto issue = [&](int s, int slot) {
        int sr = s + rot;
        sr = sr >= steps ? sr - steps : sr;
        const int koff = sr * (WK * 1024);
#pragma unroll
        for (int i = 0; i < TMB; ++i)
            fa[slot][i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(ra, voff, soa[i] + koff, 0));
#pragma unroll
        for (int j = 0; j < TNB; ++j)
            fb[slot][j] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rw, voff, sow[j] + koff, 0));
    };

    v16i acc[TMB][TNB];
#pragma unroll
    for (int i = 0; i < TMB; ++i)
#pragma unroll
        for (int j = 0; j < TNB; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    auto compute = [&](int slot) {
#pragma unroll
        for (int i = 0; i < TMB; ++i)
#pragma unroll
            for (int j = 0; j < TNB; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[slot][i], fb[slot][j], acc[i][j], 0, 0, 0);
    };

    // steps is a positive multiple of D (the host picks D so).
#pragma unroll
    for (int u = 0; u < D; ++u) issue(u, u);
    for (int s0 = D; s0 < steps; s0 += D) {
#pragma unroll
        for (int u = 0; u < D; ++u) {
            compute(u);
            issue(s0 + u, u);
        }
    }
#pragma unroll
    for (int u = 0; u < D; ++u) compute(u);

    // wave `wave` holds the partial sums of its k blocks for the whole tile
    ksplit_reduce<TMB, TNB, WK, false>(acc, lds, wave, 0, lane);
    store_tile<TMB, TNB, WK, EPI, EVEN>(acc, ep, M, N, m0, wave, lane, nn, swv, bv, sa0);
}

// Row-major int8 [rows, k] -> packed.  One wave per fragment: a lane copies the 16 bytes of its
// (row, half k block); rows and k past the matrix become zero.
__global__ __launch_bounds__(256) void pack_rows_i8_kernel(const int8_t *__restrict__ src, size_t rows, size_t k,
                                                           size_t ld, int8_t *__restrict__ dst) {
    const size_t KB = packed_k_blocks(k);
    const size_t nfrag = packed_row_blocks(rows) * KB;
    const int lane = threadIdx.x % kWave;
    const bool vec = (ld % 16 == 0) && ((reinterpret_cast<uintptr_t>(src) & 15u) == 0);
    for (size_t f = size_t(blockIdx.x) * 4 + threadIdx.x / kWave; f < nfrag; f += size_t(gridDim.x) * 4) {
        const size_t rb = f / KB, kb = f % KB;
        const size_t row = rb * 32 + lane % 32, k0 = kb * 32 + 16 * (lane / 32);
        v4i v = v4i{0, 0, 0, 0};
        if (row < rows && k0 < k) {
            const int8_t *p = src + row * ld + k0;
            if (vec && k0 + 16 <= k) {
                v = *reinterpret_cast<const v4i *>(p);
            } else {
                uint32_t w[4] = {0, 0, 0, 0};
                for (int b = 0; b < 16; ++b)
                    if (k0 + b < k) w[b / 4] |= uint32_t(uint8_t(p[b])) << (8 * (b % 4));
                v = v4i{int(w[0]), int(w[1]), int(w[2]), int(w[3])};
            }
        }
        *reinterpret_cast<v4i *>(dst + f * 1024 + lane * 16) = v;
    }
}

template <int TMB, int TNB, int D, int EPI, bool EVEN>
static int32_t launch_packed(hipq_ctx *ctx, const int8_t *pa, const int8_t *pw, int M, int N, int K,
                             const GemmEpilogue &ep) {
    constexpr int kLds = TMB * TNB * 3 * 4096;
    auto kernel = gemm_i8_packed_kernel<TMB, TNB, D, EPI, EVEN>;
    static bool configured[16] = {false};  // per device: raise the dynamic LDS limit once
    if (ctx->device < 16 && !configured[ctx->device]) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
        if (e != hipSuccess)
            return fail(HIPQ_DEVICE_ERROR, "gemm_i8 (packed): cannot reserve %d bytes of LDS: %s", kLds,
                        hipGetErrorString(e));
        configured[ctx->device] = true;
    }
    const int tiles_m = ((M + 31) / 32 + TMB - 1) / TMB, tiles_n = ((N + 31) / 32 + TNB - 1) / TNB;
    GemmEpilogue placed = ep;
    pick_xcd_rectangle(tiles_m, tiles_n, TMB * 32, TNB * 32, &placed.xcd_gm, &placed.xcd_gn);
    hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n), dim3(256), kLds, ctx->stream, pa, pw, M, N, K, placed);
    return check_launch("gemm_i8 (packed)");
}

// Picks the register depth: the largest of 4, 2, 1 that divides the k blocks per wave.
template <int EPI, bool EVEN>
static int32_t launch_gemm_packed(hipq_ctx *ctx, const int8_t *pa, const int8_t *pw, size_t m, size_t n, size_t k,
                                  const GemmEpilogue &ep) {
    const int M = static_cast<int>(m), N = static_cast<int>(n), K = static_cast<int>(k);
    const int steps = static_cast<int>(packed_k_blocks(k)) / 4;
    if (steps % 4 == 0) return launch_packed<4, 2, 4, EPI, EVEN>(ctx, pa, pw, M, N, K, ep);
    if (steps % 2 == 0) return launch_packed<4, 2, 2, EPI, EVEN>(ctx, pa, pw, M, N, K, ep);
    return launch_packed<4, 2, 1, EPI, EVEN>(ctx, pa, pw, M, N, K, ep);
}

}  // namespace hipq
