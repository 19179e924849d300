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

#include <type_traits>

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

// fp32 / int32 epilogue of one 32-row block that lies wholly inside the output (first row `row0`, first
// column `n0`): the same arithmetic as store_tile, without per-element bounds checks and with buffer
// stores whose row and column-block offsets are scalar, so that an output costs a convert, a multiply,
// an add and a store instead of a predicate, a branch and a 64-bit address as well.
template <int TNB, int EPI>
__device__ __forceinline__ void store_block_interior(v16i (&own)[1][TNB], const GemmEpilogue &ep, int N, int row0,
                                                     int n0, int lane, const float (&swv)[TNB],
                                                     const float (&bv)[TNB], float sa0) {
    static_assert(EPI == EPI_F32 || EPI == EPI_I32, "interior epilogue: fp32 or int32 output");
    // 4-byte elements: a row block spans at most (31 * N + 64) * 4 bytes from its first element, far below
    // the 2 GiB a buffer offset can hold for any N the entry points accept.
    char *base = static_cast<char *>(ep.out) + (size_t(row0) * N + n0) * 4;
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(base, 0, 0x7fffffff, 0x00020000);
    const int voff = (4 * (lane / 32) * N + lane % 32) * 4;
    const int row_bytes = N * 4;
    auto put = [&](int r, int j, int bits) {
        __builtin_amdgcn_raw_buffer_store_b32(bits, ro, voff, (8 * (r / 4) + (r % 4)) * row_bytes + j * 128, /*nt*/ 2);
    };
    if constexpr (EPI == EPI_I32) {
#pragma unroll
        for (int r = 0; r < 16; ++r)
#pragma unroll
            for (int j = 0; j < TNB; ++j) put(r, j, own[0][j][r]);
    } else {
        const bool has_bias = ep.bias != nullptr;
        auto emit = [&](auto scale_of, auto with_bias) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
#pragma unroll
                for (int j = 0; j < TNB; ++j) {
                    float v = static_cast<float>(own[0][j][r]) * scale_of(r, j);
                    if constexpr (decltype(with_bias)::value) v = v + bv[j];
                    put(r, j, __builtin_bit_cast(int, v));
                }
        };
        if (ep.sa_per_row) {
            float s_row[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) s_row[r] = ep.sa[row0 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4)];
            wait_vmcnt<0>();
            auto sc = [&](int r, int j) { return s_row[r] * swv[j]; };
            if (has_bias)
                emit(sc, std::true_type{});
            else
                emit(sc, std::false_type{});
        } else {
            float s_comb[TNB];
#pragma unroll
            for (int j = 0; j < TNB; ++j) s_comb[j] = sa0 * swv[j];
            auto sc = [&](int, int j) { return s_comb[j]; };
            if (has_bias)
                emit(sc, std::true_type{});
            else
                emit(sc, std::false_type{});
        }
    }
}

// Convolution epilogue of one 32-row block (rows = output channels from `row0`, a lane = one window per column
// block): accumulator + (128 - zp_in) * sum of the filter's weights, then the Linear's dequantize / requantize
// arithmetic, stored to NCHW (consecutive lanes are consecutive ow: consecutive bytes).  c_l / s_l / b_l: the
// correction, combined scale and bias of row row0 + lane % 32, handed round by shuffles.
//
// With one wave per SIMD the epilogue is bound by instruction issue, so the common case - the whole row block
// inside the output channels, the output below 2 GiB - has no branch and no 64-bit address per element: the
// stores are buffer stores whose per-lane offset (the window's place in its image plus the lane half's four
// rows; beyond the buffer for a window of the padded grid that is not an output, which makes the hardware drop
// the store) is formed once, and whose row offset is scalar.
template <int TNB, int EPI, bool EVEN>
__device__ __forceinline__ void conv_store_block(v16i (&own)[1][TNB], const GemmEpilogue &ep, int M, int row0, int lane,
                                                 const size_t (&out_base)[TNB], const bool (&valid)[TNB], int c_l,
                                                 float s_l, float b_l) {
    constexpr int ES = EPI == EPI_I8 ? 1 : 4;  // bytes per output element
    const float zpf = static_cast<float>(ep.zp_out);
    const bool has_bias = ep.bias != nullptr;
    const size_t plane = size_t(ep.cv_ho) * ep.cv_wo;
    wait_vmcnt<0>();
    float s_row[16], b_row[16];
    int c_row[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int src = 8 * (r / 4) + 4 * (lane / 32) + (r % 4);  // row of the block = lane that holds its operands
        c_row[r] = __shfl(c_l, src, kWave);
        s_row[r] = __shfl(s_l, src, kWave);
        b_row[r] = __shfl(b_l, src, kWave);
    }
    // The element's bits (int8 in the low byte for EPI_I8).  FAST_DIV / BIAS are hoisted out of the element loop
    // so that its body is straight-line code the compiler can interleave across the 32 outputs of a lane.
    auto value = [&](int r, int j, auto fast_div, auto with_bias) -> int {
        const int a = own[0][j][r] + c_row[r];
        if constexpr (EPI == EPI_I32) {
            return a;
        } else {
            float v = static_cast<float>(a) * s_row[r];
            if constexpr (decltype(with_bias)::value) v = v + b_row[r];
            if constexpr (EPI == EPI_F32) {
                return __builtin_bit_cast(int, v);
            } else {
                float q;
                if constexpr (decltype(fast_div)::value) {
                    const float q0 = v * ep.s_out_inv;  // div_rn with a usable reciprocal
                    const float rem = fmaf(-q0, ep.s_out, v);
                    const float q1 = fmaf(rem, ep.s_out_inv, q0);
                    q = (rem == rem) ? q1 : q0;
                } else {
                    q = v / ep.s_out;
                }
                return clamp_to_int(round_mode<EVEN>(q) + zpf, -128, 127);  // NaN -> 0, as `as i8` after the clamp
            }
        }
    };
    const size_t out_bytes = size_t(ep.cv_nb) * ep.cv_oc * plane * ES;
    const bool whole = row0 + 32 <= M && out_bytes < (size_t(1) << 31);
    const __amdgpu_buffer_rsrc_t ro =
        __builtin_amdgcn_make_buffer_rsrc(ep.out, 0, whole ? static_cast<int>(out_bytes) : 0, 0x00020000);
    int voff[TNB];
#pragma unroll
    for (int j = 0; j < TNB; ++j)
        voff[j] = valid[j] ? static_cast<int>((out_base[j] + size_t(4 * (lane / 32)) * plane) * ES) : 0x7fffffff;
    const int plane_bytes = static_cast<int>(plane) * ES;
    auto emit = [&](auto fast_div, auto with_bias) {
        if (whole) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int soff = (row0 + 8 * (r / 4) + (r % 4)) * plane_bytes;
#pragma unroll
                for (int j = 0; j < TNB; ++j) {
                    const int bits = value(r, j, fast_div, with_bias);
                    if constexpr (EPI == EPI_I8)
                        __builtin_amdgcn_raw_buffer_store_b8(static_cast<char>(bits), ro, voff[j], soff, 0);
                    else
                        __builtin_amdgcn_raw_buffer_store_b32(bits, ro, voff[j], soff, 0);
                }
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = row0 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
                if (m >= M) continue;
#pragma unroll
                for (int j = 0; j < TNB; ++j) {
                    if (!valid[j]) continue;
                    const size_t off = out_base[j] + size_t(m) * plane;
                    const int bits = value(r, j, fast_div, with_bias);
                    if constexpr (EPI == EPI_I8)
                        static_cast<int8_t *>(ep.out)[off] = static_cast<int8_t>(bits);
                    else
                        static_cast<int32_t *>(ep.out)[off] = bits;
                }
            }
        }
    };
    const bool fast = ep.s_out_inv != 0.0f;
    if (fast && has_bias)
        emit(std::true_type{}, std::true_type{});
    else if (fast)
        emit(std::true_type{}, std::false_type{});
    else if (has_bias)
        emit(std::false_type{}, std::true_type{});
    else
        emit(std::false_type{}, std::false_type{});
}

// TMB x TNB row blocks of 32 per workgroup tile; D register stages of (TMB + TNB) KiB per wave in
// flight.  Loads are buffer loads with a constant per-lane offset and scalar (SGPR) fragment
// offsets, so the loop spends no vector instruction on addressing.
//
// Sibling tiles (same weight panel, different tile_m) run on CUs of one XCD at the same time; each
// starts its K loop a quarter of the way further on (`rot`), so the four of them miss on
// different weight lines and every line is fetched from HBM by one of them and found in the L2 by
// the other three, instead of all four waiting on the same miss.  The activation rows of a tile_m
// are read by all 8 XCDs (each has its own L2): every XCD starts a further (steps/8 | 1) steps on, so
// that the eight do not ask memory for the same lines at the same moment (17.9 -> 16.5 us at
// M = 512, N = K = 4096 with operands from HBM; with 32 steps every (tile_m, XCD) pair starts on a
// different step).  Activations that the previous kernel has just written are served by the memory-side
// cache, where the same stagger costs 0.4 us instead: the fused forwards switch it off.
//
// Issuing the loads of a stage between the MFMAs of the stage being multiplied (a third register slot, one load
// behind each of the first six MFMAs, the order pinned with sched_group_barrier) instead of behind all eight was
// measured: K loop 19.6 k -> 18.4 k cycles under the stamps, 14.7 us from launch to launch either way.  Not kept.
//
// CONV: implicit-GEMM convolution on the same loop.  The row operand PA holds the packed filters (M = output
// channels, K = taps x channels, tap-major), the column operand PW is the image as signed bytes in
// [channel block of 32][padded pixel][32 bytes] order (conv_pack_image_kernel), N = padded pixels = windows:
// window q's fragment for (tap, channel block) is the 32 pixels from q + tap offset on, 1 KiB contiguous, so a
// window fragment is one coalesced wave load like a packed one, with no im2col and no gather.
template <int TMB, int TNB, int D, int EPI, bool EVEN, bool TRACE = false, bool CONV = false, bool HALVES = false>
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
    // TRACE: shader-clock stamps at the phase boundaries of this wave (start, first operands in registers,
    // end of the K loop, partial sums reduced, stores issued, stores retired).
    unsigned long long stamp[kTraceWords] = {};
    auto mark = [&](int i) {
        if constexpr (TRACE) stamp[i] = __builtin_readcyclecounter();
    };
    if constexpr (TRACE) stamp[kTracePoints] = __builtin_amdgcn_s_memrealtime();
    mark(0);

    // Epilogue operands first: their latency hides behind the main loop.
    float swv[TNB], bv[TNB], sa0 = 1.0f;
    int nn[TNB];
#pragma unroll
    for (int j = 0; j < TNB; ++j) {
        nn[j] = n0 + j * 32 + lane % 32;
        const int nc = nn[j] < N ? nn[j] : N - 1;
        swv[j] = 1.0f;
        bv[j] = 0.0f;
        if constexpr (EPI != EPI_I32 && !CONV) {
            swv[j] = ep.sw[nc];
            if (ep.bias) bv[j] = ep.bias[nc];
        }
    }
    if constexpr (EPI != EPI_I32)
        if (CONV || !ep.sa_per_row) sa0 = ep.sa ? ep.sa[0] : ep.sa_scalar;
    // Convolution: where each window's outputs go and the per-filter operands of this wave's row block, also
    // ahead of the main loop.  Rows are output channels, columns are padded-grid windows; a lane owns one
    // window per column block.  Lane l fetches the operands of row l % 32 of the block; the 16 rows a lane
    // needs come back through shuffles in the epilogue.
    size_t cv_out_base[CONV ? TNB : 1];
    bool cv_valid[CONV ? TNB : 1];
    float cv_s = 1.0f, cv_b = 0.0f;
    int cv_c = 0;
    if constexpr (CONV) {
#pragma unroll
        for (int j = 0; j < TNB; ++j) {
            const int q = nn[j];
            const int per_img = ep.cv_hp * ep.cv_wp;
            const int img = q / per_img, rem = q % per_img;
            const int oh = rem / ep.cv_wp, ow = rem % ep.cv_wp;
            cv_valid[j] = q < N && oh < ep.cv_ho && ow < ep.cv_wo;
            cv_out_base[j] = (size_t(img) * ep.cv_oc * ep.cv_ho + oh) * ep.cv_wo + ow;  // + oc * ho * wo
        }
        const int m = m0 + wave * 32 + lane % 32;
        const int mc = m < M ? m : M - 1;
        cv_c = (ep.cv_zp_in ? 128 - *ep.cv_zp_in : ep.cv_corr_mul) * ep.cv_wsum[mc];
        if constexpr (EPI != EPI_I32) {
            cv_s = sa0 * ep.sw[mc];
            if (ep.bias) cv_b = ep.bias[mc];
        }
    }

    // Byte offsets of this wave's first fragment of every row block of the tile (row blocks past
    // the matrix repeat the last one: computed and discarded).  Operands are below 2 GiB.
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(PA), 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(PW), 0, 0x7fffffff, 0x00020000);
    // A wave numbers the tile's row blocks from the one it will own after the K-split sum: its block i is
    // row block (wave + i) % TMB of the tile.  Every wave then runs the same code on the same registers
    // (block 0 is kept, blocks 1.. are handed over), with no wave-dependent branch in the epilogue.
    static_assert(TMB == WK, "one row block per K-split wave");
    int soa[TMB], sow[TNB];
#pragma unroll
    for (int i = 0; i < TMB; ++i) {
        int rb = tile_m * TMB + (wave + i) % TMB;
        rb = rb < rbA ? rb : rbA - 1;
        soa[i] = (rb * KB + wave) * 1024;
    }
#pragma unroll
    for (int j = 0; j < TNB; ++j) {
        int rb = tile_n * TNB + j;
        rb = rb < rbW ? rb : rbW - 1;
        sow[j] = CONV ? rb * 1024 : (rb * KB + wave) * 1024;  // CONV: 32 pixels of 32 bytes per row block
    }
    const int steps = KB / WK;  // k blocks per wave
    int rot = (tile_m % 4) * (steps / 4) + (ep.fresh_activations ? 0 : int(blockIdx.x % 8) * ((steps / 8) | 1));
    while (rot >= steps) rot -= steps;  // at most a few rounds; cheaper than a division in front of the first load
    const int voff = lane * 16;
    // CONV: lane l reads window l % 32 (pixels are 32 bytes apart), bytes 16 * (l / 32) of the channel block.
    const int voffw = CONV ? (lane % 32) * 32 + (lane / 32) * 16 : voff;
    // CONV: this wave's k block as (channel block, tap row, tap column), advanced by 4 k blocks per step with
    // scalar adds (a division per step would cost more than the step's MFMAs).
    const int cv_cb_count = CONV ? ep.cv_c / 32 : 1;
    int cv_kb = 0, cv_cb = 0, cv_ty = 0, cv_tx = 0;
    auto conv_seek = [&](int sr) {
        int tap;
        cv_kb = wave + WK * sr;
        divmod_uniform(cv_kb, cv_cb_count, &tap, &cv_cb);
        divmod_uniform(tap, ep.cv_kw, &cv_ty, &cv_tx);
    };
    if constexpr (CONV) conv_seek(rot);

    v4i fa[D][TMB], fb[D][TNB];
    auto issue = [&](int s, int slot) {
        int sr = s + rot;
        sr = sr >= steps ? sr - steps : sr;
        const int koff = sr * (WK * 1024);
#pragma unroll
        for (int i = 0; i < TMB; ++i)
            fa[slot][i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(ra, voff, soa[i] + koff, 0));
        int koffw = koff;
        if constexpr (CONV) {
            if (sr == 0 && s != 0) conv_seek(0);  // wrapped round
            // k blocks past taps x channel blocks are zero in the filters: any valid address will do
            koffw = cv_kb < ep.cv_kblocks ? (cv_cb * ep.cv_pixels + cv_ty * ep.cv_wp + cv_tx) * 32 : 0;
            cv_kb += WK;
            cv_cb += WK;
            while (cv_cb >= cv_cb_count) {
                cv_cb -= cv_cb_count;
                if (++cv_tx == ep.cv_kw) {
                    cv_tx = 0;
                    ++cv_ty;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < TNB; ++j)
            fb[slot][j] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rw, voffw, sow[j] + koffw, 0));
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
    if constexpr (TRACE) {
        wait_vmcnt<(D - 1) * (TMB + TNB)>();  // the first stage has landed
        mark(1);
    }
    for (int s0 = D; s0 < steps; s0 += D) {
#pragma unroll
        for (int u = 0; u < D; ++u) {
            compute(u);
            issue(s0 + u, u);
        }
    }
#pragma unroll
    for (int u = 0; u < D; ++u) compute(u);
    if constexpr (TRACE) {
        // the last MFMA has retired once its result can be read
        asm volatile("s_nop 15\n\ts_nop 15" ::"v"(acc[TMB - 1][TNB - 1][0]));
        mark(2);
    }

    // Wave `wave` holds the partial sums of its k blocks for the whole tile.  Block i (i >= 1) goes to its
    // owner, wave (wave + i) % TMB, through LDS: [owner][slot i-1][column block][4 registers][lane] of 16
    // bytes; the three writers of one owner use three different slots.  Integer adds: any order, same bits.
    v4i *red = reinterpret_cast<v4i *>(lds);
    v16i own[1][TNB];
    if constexpr (HALVES) {
        // One column block at a time: half the LDS (48 KB), so that two workgroups share a compute unit and one
        // runs its loop while the other sums and stores.  [owner][slot i-1][4 registers][lane] of 16 bytes.
#pragma unroll
        for (int j = 0; j < TNB; ++j) {
            if (j) __syncthreads();  // the previous column block has been read
#pragma unroll
            for (int i = 1; i < TMB; ++i) {
                const int owner = (wave + i) % TMB;
                v4i *dst = red + ((owner * (TMB - 1) + (i - 1)) * 4) * kWave + lane;
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    dst[g * kWave] = v4i{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
            }
            __syncthreads();
            v4i part[TMB - 1][4];
            const v4i *src = red + (wave * (TMB - 1) * 4) * kWave + lane;
#pragma unroll
            for (int sl = 0; sl < TMB - 1; ++sl)
#pragma unroll
                for (int g = 0; g < 4; ++g) part[sl][g] = src[(sl * 4 + g) * kWave];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                int v = acc[0][j][r];
#pragma unroll
                for (int sl = 0; sl < TMB - 1; ++sl) v += part[sl][r / 4][r % 4];
                own[0][j][r] = v;
            }
        }
    } else {
#pragma unroll
    for (int i = 1; i < TMB; ++i) {
        const int owner = (wave + i) % TMB;
        v4i *dst = red + ((owner * (TMB - 1) + (i - 1)) * TNB * 4) * kWave + lane;
#pragma unroll
        for (int j = 0; j < TNB; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                dst[(j * 4 + g) * kWave] =
                    v4i{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
    }
    __syncthreads();
    // All reads first (the operand registers of the loop are free), then the adds: the LDS pipe streams
    // instead of paying its latency once per pair of reads.
    v4i part[TMB - 1][TNB][4];
    const v4i *src = red + (wave * (TMB - 1) * TNB * 4) * kWave + lane;
#pragma unroll
    for (int sl = 0; sl < TMB - 1; ++sl)
#pragma unroll
        for (int j = 0; j < TNB; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) part[sl][j][g] = src[((sl * TNB + j) * 4 + g) * kWave];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < TNB; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            int v = acc[0][j][r];
#pragma unroll
            for (int sl = 0; sl < TMB - 1; ++sl) v += part[sl][j][r / 4][r % 4];
            own[0][j][r] = v;
        }
    }
    mark(3);
    const int row0 = m0 + wave * 32;
    if constexpr (CONV) {
        conv_store_block<TNB, EPI, EVEN>(own, ep, M, row0, lane, cv_out_base, cv_valid, cv_c, cv_s, cv_b);
    } else {
        bool interior = false;
        if constexpr (EPI != EPI_I8) interior = m0 + TMB * 32 <= M && n0 + TNB * 32 <= N && ep.residual == nullptr;
        if (interior) {
            if constexpr (EPI != EPI_I8) store_block_interior<TNB, EPI>(own, ep, N, row0, n0, lane, swv, bv, sa0);
        } else {
            store_tile<1, TNB, 1, EPI, EVEN>(own, ep, M, N, row0, 0, lane, nn, swv, bv, sa0);
        }
    }
    if constexpr (TRACE) {
        mark(4);
        wait_vmcnt<0>();
        mark(5);
        stamp[kTracePoints + 1] = __builtin_amdgcn_s_memrealtime();
        if (lane == 0) {
            unsigned long long *t = ep.trace + (size_t(blockIdx.x) * WK + wave) * kTraceWords;
#pragma unroll
            for (int i = 0; i < kTraceWords; ++i) t[i] = stamp[i];
        }
    }
}

// Skinny product on packed operands (M <= 32: decode-shaped Linear).  The weight matrix is read exactly once and
// nothing else matters: one 32-row block of weights per workgroup, K split between the four waves, D stages of
// one weight fragment (1 KiB, contiguous in HBM) and one activation fragment (L2 resident) per wave in flight.
// The four partial 32x32 blocks are summed through LDS by wave 0, which runs the ordinary checked epilogue.
// The loop runs in rounds of D stages for any number of k steps: stages past the last ask for an offset beyond the
// buffers, which returns zeros without touching memory and adds nothing.  D is the host's choice by how many
// workgroups there are (see launch_gemv_packed).
template <int D, int EPI, bool EVEN>
__global__ __launch_bounds__(256) void gemv_i8_packed_kernel(const int8_t *__restrict__ PA, const int8_t *__restrict__ PW,
                                                             int M, int N, int K, GemmEpilogue ep) {
    __shared__ __attribute__((aligned(16))) v4i red[3][4][kWave];
    constexpr int WK = 4;
    const int KB = static_cast<int>(packed_k_blocks(K));
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int n0 = blockIdx.x * 32;
    float swv[1], bv[1], sa0 = 1.0f;
    int nn[1];
    nn[0] = n0 + lane % 32;
    swv[0] = 1.0f;
    bv[0] = 0.0f;
    if constexpr (EPI != EPI_I32) {
        if (wave == 0) {
            const int nc = nn[0] < N ? nn[0] : N - 1;
            swv[0] = ep.sw[nc];
            if (ep.bias) bv[0] = ep.bias[nc];
            if (!ep.sa_per_row) sa0 = ep.sa ? ep.sa[0] : ep.sa_scalar;
        }
    }
    // The activation fragments hold M real rows and 32 - M rows of zero padding: lanes of padding rows ask for an
    // offset beyond the buffer, which returns zeros without touching memory, so that for M = 1 an activation
    // fragment costs two 16-byte pieces instead of a KiB (every workgroup reads all of them).
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(PA), 0, KB * 1024, 0x00020000);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(PW), 0, 0x7fffffff, 0x00020000);
    const int soa = wave * 1024, sow = (static_cast<int>(blockIdx.x) * KB + wave) * 1024;
    const int steps = KB / WK, voff = lane * 16;
    const int voffa = lane % 32 < M ? voff : 0x7fffffff;
    v4i fa[D], fb[D];
    const int rounds_end = (steps + D - 1) / D * D;
    auto issue = [&](int s, int slot) {
        const int koff = s * (WK * 1024);
        const bool real = s < steps;
        fa[slot] = __builtin_bit_cast(
            v4i, __builtin_amdgcn_raw_buffer_load_b128(ra, real ? voffa : 0x7fffffff, real ? soa + koff : 0, 0));
        fb[slot] = __builtin_bit_cast(
            v4i, __builtin_amdgcn_raw_buffer_load_b128(rw, real ? voff : 0x7fffffff, real ? sow + koff : 0, 0));
    };
    v16i acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0;
#pragma unroll
    for (int u = 0; u < D; ++u) issue(u, u);
    for (int s0 = D; s0 < rounds_end; s0 += D) {
#pragma unroll
        for (int u = 0; u < D; ++u) {
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[u], fb[u], acc, 0, 0, 0);
            issue(s0 + u, u);
        }
    }
#pragma unroll
    for (int u = 0; u < D; ++u) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[u], fb[u], acc, 0, 0, 0);
    if (wave > 0) {
#pragma unroll
        for (int g = 0; g < 4; ++g) red[wave - 1][g][lane] = v4i{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
    }
    __syncthreads();
    if (wave > 0) return;
    v16i own[1][1];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const v4i t = red[0][g][lane] + red[1][g][lane] + red[2][g][lane];
#pragma unroll
        for (int c = 0; c < 4; ++c) own[0][0][4 * g + c] = acc[4 * g + c] + t[c];
    }
    store_tile<1, 1, 1, EPI, EVEN>(own, ep, M, N, 0, 0, lane, nn, swv, bv, sa0);
}

// The same with RB = 1 or 2 activation row blocks and TNB = 1 or 2 32-row blocks of weights per workgroup (a batch of
// decodes, a short prefill): K split between the four waves, each of which multiplies its TNB weight fragments with
// the RB activation fragments of the k block (L2 resident: RB KiB a step against TNB KiB from HBM).  Up to 64
// activation rows one row of workgroups covers the matrix and the weights are read from memory once; with more rows,
// blockIdx.y picks the pair of row blocks and the grid is one of 64 x 64 tiles.  The 128 x 64 tiles of the general
// kernel give such shapes 64-170 workgroups with 786 KB of operands each, and take as long for 64 rows as for 512.
// Wave b ends up owning output block b: the others park their partials of it in LDS.
template <int D, int RB, int TNB, int EPI, bool EVEN>
__global__ __launch_bounds__(256) void skinny_i8_packed_kernel(const int8_t *__restrict__ PA, const int8_t *__restrict__ PW,
                                                               int M, int N, int K, GemmEpilogue ep) {
    constexpr int NBLK = RB * TNB;  // 32 x 32 output blocks of the workgroup: block b = (row block b / TNB, column block b % TNB)
    static_assert(NBLK >= 2 && NBLK <= 4, "at most one output block per wave");
    __shared__ __attribute__((aligned(16))) v4i red[3][NBLK][4][kWave];
    constexpr int WK = 4;
    const int KB = static_cast<int>(packed_k_blocks(K));
    const int rbW = (N + 31) / 32;
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    // Epilogue operands of the block this wave will own.
    float swv[1], bv[1], sa0 = 1.0f;
    int nn[1];
    nn[0] = (static_cast<int>(blockIdx.x) * TNB + wave % TNB) * 32 + lane % 32;
    swv[0] = 1.0f;
    bv[0] = 0.0f;
    if constexpr (EPI != EPI_I32) {
        if (wave < NBLK) {
            const int nc = nn[0] < N ? nn[0] : N - 1;
            swv[0] = ep.sw[nc];
            if (ep.bias) bv[0] = ep.bias[nc];
            if (!ep.sa_per_row) sa0 = ep.sa ? ep.sa[0] : ep.sa_scalar;
        }
    }
    const __amdgpu_buffer_rsrc_t ra =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(PA), 0, 0x7ffffffe, 0x00020000);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(PW), 0, 0x7fffffff, 0x00020000);
    const int steps = KB / WK, voff = lane * 16;
    // blockIdx.y: which group of RB activation row blocks (more than RB of them: a grid of RB*32 x TNB*32 tiles)
    const int rb0 = static_cast<int>(blockIdx.y) * RB;
    int soa[RB], voffa[RB], sow[TNB];  // rows past M read zeros without touching memory
#pragma unroll
    for (int i = 0; i < RB; ++i) {
        soa[i] = ((rb0 + i) * KB + wave) * 1024;
        voffa[i] = (rb0 + i) * 32 + lane % 32 < M ? voff : 0x7fffffff;
    }
#pragma unroll
    for (int j = 0; j < TNB; ++j) {
        int rb = static_cast<int>(blockIdx.x) * TNB + j;
        rb = rb < rbW ? rb : rbW - 1;  // a column block past the matrix repeats the last one; its outputs are not stored
        sow[j] = (rb * KB + wave) * 1024;
    }
    v4i fa[D][RB], fb[D][TNB];
    const int rounds_end = (steps + D - 1) / D * D;
    auto issue = [&](int s, int slot) {
        const int koff = s * (WK * 1024);
        const bool real = s < steps;
#pragma unroll
        for (int i = 0; i < RB; ++i)
            fa[slot][i] = __builtin_bit_cast(
                v4i, __builtin_amdgcn_raw_buffer_load_b128(ra, real ? voffa[i] : 0x7fffffff, real ? soa[i] + koff : 0, 0));
#pragma unroll
        for (int j = 0; j < TNB; ++j)
            fb[slot][j] = __builtin_bit_cast(
                v4i, __builtin_amdgcn_raw_buffer_load_b128(rw, real ? voff : 0x7fffffff, real ? sow[j] + koff : 0, 0));
    };
    v16i acc[NBLK];
#pragma unroll
    for (int b = 0; b < NBLK; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[b][r] = 0;
    auto multiply = [&](int slot) {
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
            for (int j = 0; j < TNB; ++j)
                acc[i * TNB + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[slot][i], fb[slot][j], acc[i * TNB + j], 0, 0, 0);
    };
#pragma unroll
    for (int u = 0; u < D; ++u) issue(u, u);
    for (int s0 = D; s0 < rounds_end; s0 += D) {
#pragma unroll
        for (int u = 0; u < D; ++u) {
            multiply(u);
            issue(s0 + u, u);
        }
    }
#pragma unroll
    for (int u = 0; u < D; ++u) multiply(u);
    // Output block b goes to wave b; wave w parks its partial of it in slot (w - b - 1) mod 4 of the three.
#pragma unroll
    for (int b = 0; b < NBLK; ++b) {
        if (b == wave) continue;
        const int slot = (wave - b + 3) % 4;
#pragma unroll
        for (int g = 0; g < 4; ++g)
            red[slot][b][g][lane] = v4i{acc[b][4 * g], acc[b][4 * g + 1], acc[b][4 * g + 2], acc[b][4 * g + 3]};
    }
    __syncthreads();
    if (wave >= NBLK) return;
    v16i own[1][1];
#pragma unroll
    for (int b = 0; b < NBLK; ++b) {
        if (b != wave) continue;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const v4i t = red[0][b][g][lane] + red[1][b][g][lane] + red[2][b][g][lane];
#pragma unroll
            for (int c = 0; c < 4; ++c) own[0][0][4 * g + c] = acc[b][4 * g + c] + t[c];
        }
    }
    store_tile<1, 1, 1, EPI, EVEN>(own, ep, M, N, (rb0 + wave / TNB) * 32, 0, lane, nn, swv, bv, sa0);
}

// The same product straight from fp32 activations of at most four rows (decode), per-row dynamic int8: one launch
// instead of a quantizer and the product.  No workgroup depends on another: each one requests its first weight
// fragments, then reads the rows itself (they are 16 KiB each and come out of the L2 for all but the first
// workgroups), finds every row's range (waves by shuffles, the four waves through LDS), quantizes with the per-row
// quantizer's own arithmetic (params_from_minmax, symmetric; division form; a row whose range is not finite gets a
// NaN scale and zero codes) and leaves the codes in LDS in fragment order: [k block][half][row], 16 bytes each.
// The main loop takes its activation fragments from there.  A thread holds 16 consecutive floats per row and chunk
// of 4096 columns: MROWS * CH <= 4 chunks, i.e. at most 64 registers of data.  K % 16 == 0, x 16-byte aligned.
// Rounds of D stages as in gemv_i8_packed_kernel.  fp32 output: out = acc * (s_a[m] * s_w[n]) (+ bias[n]), as
// store_tile does it.  Every workgroup repeats the quantize arithmetic of all rows (16 values a thread and row at
// K = 4096), which is why this pays for one or two rows only: N = 11008, K = 4096 from fp32, one launch against
// the quantizer and the product: M = 1 11.7 / 14.7 us, M = 2 13.3 / 14.7, M = 3 15.4 / 14.8, M = 4 17.3 / 15.0.
// For more rows a hand-over inside one launch was built and measured (workgroup r quantizes row r into the packed
// scratch, fences at device scope and raises a flag word; every workgroup requests its first weight fragments,
// waits for the M flags, passes a device-scope acquire, then runs the product; an arrival counter lets the last
// workgroup clear the flags for the next launch).  Bit-identical, and slower: M = 4 27.6 us, M = 16 34.9 us against
// 13.9 / 14.9 us for the two launches (same shape); of that the acquire (an L2 invalidate per workgroup) costs
// 8.5 us, the arrival atomics on one word 4.4 us, the producers' fence 1.2 us - and with all three taken out
// (13.5 us, no longer correct) it only equals the two launches, because the chain "read the row, reduce, quantize,
// write through, flag seen by the other dies" is as long as the quantizer's launch and ramp.  Not kept.
template <int D, bool EVEN, int MROWS, int CH, bool STATIC = false>
__global__ __launch_bounds__(256) void gemv_i8_packed_from_f32_kernel(const float *__restrict__ x,
                                                                      const int8_t *__restrict__ PW, int M, int N, int K,
                                                                      GemmEpilogue ep, int static_div) {
    static_assert(MROWS * CH <= 4, "at most 64 data registers per thread");
    __shared__ __attribute__((aligned(16))) v4i red[3][4][kWave];
    __shared__ __attribute__((aligned(16))) v4i codes[MROWS * CH * 256];
    __shared__ float wave_mn[4][MROWS], wave_mx[4][MROWS];
    constexpr int WK = 4;
    const int KB = static_cast<int>(packed_k_blocks(K));
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int n = blockIdx.x * 32 + lane % 32;
    // Weights first: nothing below depends on them, and they are what the launch waits for.
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(PW), 0, 0x7fffffff, 0x00020000);
    const int sow = (static_cast<int>(blockIdx.x) * KB + wave) * 1024, steps = KB / WK, voff = lane * 16;
    const int rounds_end = (steps + D - 1) / D * D;
    v4i fb[D];
    auto issue = [&](int s, int slot) {
        const bool real = s < steps;
        fb[slot] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rw, real ? voff : 0x7fffffff,
                                                                                 real ? sow + s * (WK * 1024) : 0, 0));
    };
#pragma unroll
    for (int u = 0; u < D; ++u) issue(u, u);
    float sw = 1.0f, b = 0.0f;
    if (wave == 0) {
        const int nc = n < N ? n : N - 1;
        sw = ep.sw[nc];
        if (ep.bias) b = ep.bias[nc];
    }
    // The rows: thread t holds floats [16 g, 16 g + 16) of every row for g = t + 256 c.
    float4 v[MROWS][CH][4];
    bool have[MROWS][CH];
#pragma unroll
    for (int m = 0; m < MROWS; ++m)
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int k0 = (static_cast<int>(threadIdx.x) + 256 * c) * 16;
            have[m][c] = m < M && k0 < K;
            if (have[m][c]) {
#pragma unroll
                for (int i = 0; i < 4; ++i) v[m][c][i] = reinterpret_cast<const float4 *>(x + size_t(m) * K + k0)[i];
            }
        }
    if constexpr (!STATIC) {
#pragma unroll
        for (int m = 0; m < MROWS; ++m) {
            float mn = INFINITY, mx = -INFINITY;
#pragma unroll
            for (int c = 0; c < CH; ++c)
                if (have[m][c]) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        mn = fminf(mn, fminf(fminf(v[m][c][i].x, v[m][c][i].y), fminf(v[m][c][i].z, v[m][c][i].w)));
                        mx = fmaxf(mx, fmaxf(fmaxf(v[m][c][i].x, v[m][c][i].y), fmaxf(v[m][c][i].z, v[m][c][i].w)));
                    }
                }
            mn = wave_min(mn);
            mx = wave_max(mx);
            if (lane == 0) {
                wave_mn[wave][m] = mn;
                wave_mx[wave][m] = mx;
            }
        }
        __syncthreads();
    }
    float sa[MROWS];
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
        float scale, inv, zpf = 0.0f;
        if constexpr (STATIC) {
            // a given per-tensor scale: the packed quantizer's arithmetic in the caller's form (quantize_packed_kernel)
            scale = ep.sa_scalar;
            sa[m] = scale;
            inv = static_div ? recip_for_div(scale) : 1.0f / scale;
        } else {
            const float mn = fminf(fminf(wave_mn[0][m], wave_mn[1][m]), fminf(wave_mn[2][m], wave_mn[3][m]));
            const float mx = fmaxf(fmaxf(wave_mx[0][m], wave_mx[1][m]), fmaxf(wave_mx[2][m], wave_mx[3][m]));
            int zp;
            const bool bad = params_from_minmax(mn, mx, HIPQ_PARAMS_SYMMETRIC, -128, 127, &scale, &zp) != HIPQ_SUCCESS;
            sa[m] = bad ? __builtin_nanf("") : scale;
            if (bad) scale = INFINITY;  // x / inf: 0 for finite x, NaN -> code 0 otherwise
            inv = recip_for_div(scale);
            zpf = static_cast<float>(bad ? 0 : zp);
        }
        auto q = [&](float f) {
            if constexpr (STATIC) {
                return static_div ? quantize_int<true, EVEN>(f, scale, inv, zpf, -128, 127)
                                  : quantize_int<false, EVEN>(f, scale, inv, zpf, -128, 127);
            } else {
                return quantize_int<QFORM_DIV, EVEN>(f, scale, inv, zpf, -128, 127);
            }
        };
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int g = static_cast<int>(threadIdx.x) + 256 * c;
            if (m < M && g < KB * 2) {  // k past K up to the padded extent: zeros
                v4i w = v4i{0, 0, 0, 0};
                if (have[m][c]) {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        w[i] = static_cast<int>(pack4(q(v[m][c][i].x), q(v[m][c][i].y), q(v[m][c][i].z), q(v[m][c][i].w)));
                }
                codes[g * MROWS + m] = w;
            }
        }
    }
    __syncthreads();
    // Lane l of an activation fragment: row l % 32, bytes 16 * (l / 32) .. +15 of the k block; rows past M are zero.
    const int row = lane % 32, half = lane / 32;
    auto fragment = [&](int s) {
        const int kb = wave + WK * s;
        return (row < M && s < steps) ? codes[(kb * 2 + half) * MROWS + row] : v4i{0, 0, 0, 0};
    };
    v16i acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0;
    for (int s0 = D; s0 < rounds_end; s0 += D) {
#pragma unroll
        for (int u = 0; u < D; ++u) {
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fragment(s0 - D + u), fb[u], acc, 0, 0, 0);
            issue(s0 + u, u);
        }
    }
#pragma unroll
    for (int u = 0; u < D; ++u)
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fragment(rounds_end - D + u), fb[u], acc, 0, 0, 0);
    if (wave > 0) {
#pragma unroll
        for (int g = 0; g < 4; ++g) red[wave - 1][g][lane] = v4i{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
    }
    __syncthreads();
    if (wave > 0) return;
    // Rows 0..3 of the block are registers 0..3 of lanes 0..31 (lane = output column).
    const v4i t = red[0][0][lane] + red[1][0][lane] + red[2][0][lane];
    if (lane < 32 && n < N) {
#pragma unroll
        for (int m = 0; m < MROWS; ++m) {
            if (m >= M) continue;
            float o = static_cast<float>(acc[m] + t[m]) * (sa[m] * sw);
            if (ep.bias) o = o + b;
            __builtin_nontemporal_store(o, static_cast<float *>(ep.out) + size_t(m) * N + n);
        }
    }
}

// Whether the decode forward from fp32 can take the kernel above, and its launch.  Returns false when the shape is
// left to the two launches (quantizer into the packed layout, then the product).  STATIC: a given per-tensor scale
// (ep.sa_scalar; `static_div`: the division form) instead of per-row dynamic scales; without the range pass and its
// barrier the prologue is cheap enough for four rows.
template <bool EVEN, bool STATIC>
static bool launch_gemv_packed_from_f32(hipq_ctx *ctx, const float *x, const int8_t *pw, size_t m, size_t n, size_t k,
                                        const GemmEpilogue &ep, int static_div, int32_t *rc) {
    const size_t KB = packed_k_blocks(k);
    const size_t chunks = (KB * 2 + 255) / 256;  // 16-float groups per thread and row
    const size_t most_rows = STATIC ? 4 : 2;
    if (m == 0 || m > most_rows || k % 16 != 0 || (reinterpret_cast<uintptr_t>(x) & 15u) != 0 || KB < 16) return false;
    const int mrows = m <= 2 ? static_cast<int>(m) : 4, ch = chunks <= 1 ? 1 : (chunks == 2 ? 2 : 4);
    if (chunks > 4 || mrows * ch > 4) return false;
    const int M = static_cast<int>(m), N = static_cast<int>(n), K = static_cast<int>(k);
    const int row_blocks = (N + 31) / 32;
    const int depth = row_blocks >= 200 ? 4 : (row_blocks >= 100 ? 8 : 16);  // as launch_gemv_packed
    const dim3 grid(row_blocks);
#define HIPQ_LAUNCH_GFD(DEPTH, MR, C)                                                                                  \
    hipLaunchKernelGGL((gemv_i8_packed_from_f32_kernel<DEPTH, EVEN, MR, C, STATIC>), grid, dim3(256), 0, ctx->stream, x, pw, \
                       M, N, K, ep, static_div)
#define HIPQ_LAUNCH_GF(MR, C)              \
    do {                                   \
        if (depth == 4)                    \
            HIPQ_LAUNCH_GFD(4, MR, C);     \
        else if (depth == 8)               \
            HIPQ_LAUNCH_GFD(8, MR, C);     \
        else                               \
            HIPQ_LAUNCH_GFD(16, MR, C);    \
    } while (0)
    if (mrows == 1 && ch == 1)
        HIPQ_LAUNCH_GF(1, 1);
    else if (mrows == 1 && ch == 2)
        HIPQ_LAUNCH_GF(1, 2);
    else if (mrows == 1)
        HIPQ_LAUNCH_GF(1, 4);
    else if (mrows == 2 && ch == 1)
        HIPQ_LAUNCH_GF(2, 1);
    else if (mrows == 2)
        HIPQ_LAUNCH_GF(2, 2);
    else if constexpr (STATIC)
        HIPQ_LAUNCH_GF(4, 1);
#undef HIPQ_LAUNCH_GF
#undef HIPQ_LAUNCH_GFD
    *rc = check_launch("gemv_i8 (packed, from fp32)");
    return true;
}

template <int D, int EPI, bool EVEN>
static int32_t launch_gemv_packed_d(hipq_ctx *ctx, const int8_t *pa, const int8_t *pw, int M, int N, int K,
                                    const GemmEpilogue &ep) {
    hipLaunchKernelGGL((gemv_i8_packed_kernel<D, EPI, EVEN>), dim3((N + 31) / 32), dim3(256), 0, ctx->stream, pa, pw, M, N,
                       K, ep);
    return check_launch("gemv_i8 (packed)");
}

// Stages in flight per wave (1 KiB of weights each) by the number of workgroups, i.e. weight row blocks.  What
// streams well is 5-6 MB in flight over the chip.  Measured (M = 4, us; depth 2 / 4 / 8 / 16):
//   N = 11008, K = 4096  (344 workgroups):  13.0 / 10.9 / 11.7 / 11.9 - with more in flight the workgroups' streams
//     through their 128 KiB row blocks interleave more finely in memory and the stream as a whole gets slower;
//   N = 8192,  K = 2048  (256):   5.6 /  5.5 /  5.7 /  5.6
//   N = 4096,  K = 11008 (128):  24.2 / 16.3 / 12.5 / 12.7   (depth 2 was all that divided its 86 steps: 33.8 us)
//   N = 4096,  K = 4096  (128):   7.5 /  6.0 /  5.5 /  5.4
//   N = 2048,  K = 8192  (64):   11.8 /  8.4 /  6.8 /  6.5
// Splitting K over several workgroups per row block instead (partials written through to memory, a ticket per row
// block, the last to arrive sums and stores) was built and measured: level with depth 8 at N = 4096, K = 11008
// (12.3 us), 1.5-2 us slower at 16.8 MB of weights - the hand-over costs two trips through device-coherent memory.
// Starting the workgroups on different K steps does not help either (10.7 against 10.5 us).
template <int RB, int TNB, int EPI, bool EVEN>
static int32_t launch_skinny_packed_rb(hipq_ctx *ctx, const int8_t *pa, const int8_t *pw, int M, int N, int K,
                                       const GemmEpilogue &ep) {
    const int groups = ((N + 31) / 32 + TNB - 1) / TNB;
    const dim3 grid(groups, ((M + 31) / 32 + RB - 1) / RB);
    // (depth 8 at most: a stage is RB + TNB fragments of four registers)
    if (groups >= 200)
        hipLaunchKernelGGL((skinny_i8_packed_kernel<4, RB, TNB, EPI, EVEN>), grid, dim3(256), 0, ctx->stream, pa, pw, M, N, K,
                           ep);
    else
        hipLaunchKernelGGL((skinny_i8_packed_kernel<8, RB, TNB, EPI, EVEN>), grid, dim3(256), 0, ctx->stream, pa, pw, M, N, K,
                           ep);
    return check_launch("skinny_i8 (packed)");
}

// The weight-streaming kernel's forms.  Up to 64 activation rows: from 300 weight row blocks on a workgroup takes two
// of them: half the activation traffic per weight byte, and still more than one workgroup per compute unit.  One /
// two weight row blocks per workgroup, us:
//   N = 11008, K = 4096: M = 1 10.4 / 10.25, 16 11.3 / 10.9, 32 13.4 / 12.0, 33 14.9 / 12.9, 64 17.5 / 14.2
//   N = 32000, K = 4096: M = 1 26.6 / 24.0 (5.5 TB/s), 32 28.5 / 25.6, 64 35.9 / 28.6;   N = 128256: M = 1 87.6 / 86.1
//   N = 8192,  K = 2048: M = 1 4.7 / 5.1, 32 5.4 / 6.2, 64 7.3 / 7.9 (and the same below that); four per workgroup: slower.
constexpr int kTwoBlockRowBlocks = 300;

template <int EPI, bool EVEN>
static int32_t launch_skinny_packed(hipq_ctx *ctx, const int8_t *pa, const int8_t *pw, int M, int N, int K,
                                    const GemmEpilogue &ep) {
    const bool two = (N + 31) / 32 >= kTwoBlockRowBlocks;
    if (M <= 32) return launch_skinny_packed_rb<1, 2, EPI, EVEN>(ctx, pa, pw, M, N, K, ep);  // (callers: `two` only)
    if (M <= 64 && !two) return launch_skinny_packed_rb<2, 1, EPI, EVEN>(ctx, pa, pw, M, N, K, ep);
    return launch_skinny_packed_rb<2, 2, EPI, EVEN>(ctx, pa, pw, M, N, K, ep);  // more than 64 rows: a grid of 64 x 64 tiles
}

template <int EPI, bool EVEN>
static int32_t launch_gemv_packed(hipq_ctx *ctx, const int8_t *pa, const int8_t *pw, int M, int N, int K,
                                  const GemmEpilogue &ep) {
    const int steps = static_cast<int>(packed_k_blocks(size_t(K))) / 4, row_blocks = (N + 31) / 32;
    int depth = row_blocks >= 200 ? 4 : (row_blocks >= 100 ? 8 : 16);
    while (depth > 1 && depth > steps) depth /= 2;
    switch (depth) {
    case 16: return launch_gemv_packed_d<16, EPI, EVEN>(ctx, pa, pw, M, N, K, ep);
    case 8: return launch_gemv_packed_d<8, EPI, EVEN>(ctx, pa, pw, M, N, K, ep);
    case 4: return launch_gemv_packed_d<4, EPI, EVEN>(ctx, pa, pw, M, N, K, ep);
    case 2: return launch_gemv_packed_d<2, EPI, EVEN>(ctx, pa, pw, M, N, K, ep);
    default: return launch_gemv_packed_d<1, EPI, EVEN>(ctx, pa, pw, M, N, K, ep);
    }
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

}  // namespace hipq

#include "hipq_gemm_pair.h"

namespace hipq {

template <int TMB, int TNB, int D, int EPI, bool EVEN, bool TRACE = false, bool CONV = false, bool HALVES = false>
static int32_t launch_packed(hipq_ctx *ctx, const int8_t *pa, const int8_t *pw, int M, int N, int K,
                             const GemmEpilogue &ep) {
    constexpr int kLds = TMB * (HALVES ? 1 : TNB) * 3 * 4096;
    auto kernel = gemm_i8_packed_kernel<TMB, TNB, D, EPI, EVEN, TRACE, CONV, HALVES>;
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
    if constexpr (TRACE) placed.trace = static_cast<unsigned long long *>(ctx->trace);
    hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n), dim3(256), kLds, ctx->stream, pa, pw, M, N, K, placed);
    return check_launch("gemm_i8 (packed)");
}

// Register depth 2 where it divides the k blocks per wave (else 1): two stages of 6 KiB per wave in flight.  Depth
// 4 is as fast when the kernel is launched back to back at sustained clocks (14.8 us at M = 512, N = K = 4096) but
// slower from idle clocks (17.6 against 15.7 us) and inside the Linear step, where the kernel follows the small
// quantize kernels (24.2 against 23.5 us per step); depth 1 is 2-3 us slower everywhere.
template <int EPI, bool EVEN>
static int32_t launch_gemm_packed(hipq_ctx *ctx, const int8_t *pa, const int8_t *pw, size_t m, size_t n, size_t k,
                                  const GemmEpilogue &ep) {
    const int M = static_cast<int>(m), N = static_cast<int>(n), K = static_cast<int>(k);
    const int steps = static_cast<int>(packed_k_blocks(k)) / 4;
    if (M <= 32) {  // one row block of activations
        if ((N + 31) / 32 >= kTwoBlockRowBlocks && ctx->gemm_variant != 9)
            return launch_skinny_packed<EPI, EVEN>(ctx, pa, pw, M, N, K, ep);
        return launch_gemv_packed<EPI, EVEN>(ctx, pa, pw, M, N, K, ep);
    }
    // Up to 64 rows: the weight-streaming kernel.  More rows: the same kernel as a grid of 64 x 64 tiles, while those
    // make one round over the compute units at most - half the operand bytes per workgroup of a 128 x 64 tile
    // (512 KB against 786 KB at K = 4096), and twice the workgroups where the 128 x 64 tiles leave compute units idle
    // (variant 9: the 128 x 64 tiles always).  128 x 64 / 64 x 64 in us:
    //   N = K = 4096:        M = 96 12.6 / 8.5   128 12.2 / 8.9   192 13.7 / 9.0   256 13.4 / 9.3   384 13.2 / 15.0
    //   N = 4096, K = 11264: M = 128 36.9 / 26.3  256 34.0 / 25.4  384 32.9 / 38.3
    //   N = 8192, K = 2048:  M = 128  8.8 / 7.9;  N = 2304, K = 768: M = 384 6.0 / 5.3, 512 6.0 / 6.2
    //   N = 11008, K = 4096: M = 128 18.8 / 20.5  256 30.0 / 31.2  512 39.4 / 58.6   (344 and more 64 x 64 tiles)
    if (ctx->gemm_variant == 12) {
        // Test hook: one 128 x 128 tile per pair of compute units, K halved between them (hipq_gemm_pair.h), where
        // the shape allows it.  Measured slower than the forms below at every shape tried, so never the default.
        int32_t rc = HIPQ_SUCCESS;
        if (launch_pair_if_fits<EPI, EVEN>(ctx, pa, pw, m, n, k, ep, &rc)) return rc;
    }
    if (ctx->gemm_variant != 9 && !ctx->trace) {  // (the phase stamps are the 128 x 64 kernel's)
        const size_t tiles64 = ((packed_row_blocks(m) + 1) / 2) * ((packed_row_blocks(n) + 1) / 2);
        if (M <= 64 || tiles64 <= size_t(ctx->num_cus)) return launch_skinny_packed<EPI, EVEN>(ctx, pa, pw, M, N, K, ep);
    }
    if constexpr (EPI == EPI_F32 && !EVEN) {
        // Phase stamps (hipq_ctx_set_trace_buffer): the depth-2 fp32 form only, and only when the buffer holds
        // every wave's record.
        const size_t tiles = ((packed_row_blocks(m) + 3) / 4) * ((packed_row_blocks(n) + 1) / 2);
        if (ctx->trace && steps % 2 == 0 && ctx->trace_bytes >= tiles * 4 * kTraceWords * sizeof(unsigned long long))
            return launch_packed<4, 2, 2, EPI, EVEN, true>(ctx, pa, pw, M, N, K, ep);
    }
    if constexpr (EPI != EPI_I8) {
        // More tiles than compute units: the form that sums one column block at a time (48 KB of LDS), so that two
        // workgroups share a compute unit and one runs its loop while the other sums and stores (M = 8192, N = 2304,
        // K = 768: 43.6 -> 31.3 us; M = 2048, N = K = 4096: 50.2 -> 43.2 us).  The int8 epilogue needs more than
        // half the register file, so two of its workgroups would not fit anyway.
        const size_t tiles = ((packed_row_blocks(m) + 3) / 4) * ((packed_row_blocks(n) + 1) / 2);
        if (tiles > size_t(ctx->num_cus) && ctx->gemm_variant != 9) {
            if (steps % 2 == 0) return launch_packed<4, 2, 2, EPI, EVEN, false, false, true>(ctx, pa, pw, M, N, K, ep);
            return launch_packed<4, 2, 1, EPI, EVEN, false, false, true>(ctx, pa, pw, M, N, K, ep);
        }
    }
    if (steps % 2 == 0) return launch_packed<4, 2, 2, EPI, EVEN>(ctx, pa, pw, M, N, K, ep);
    return launch_packed<4, 2, 1, EPI, EVEN>(ctx, pa, pw, M, N, K, ep);
}

}  // namespace hipq
