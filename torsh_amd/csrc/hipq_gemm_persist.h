// Persistent, queue-coupled form of the pipelined int8 MFMA GEMM.
//
// One workgroup per CU walks a list of output tiles.  Producer waves stream K-tiles of the
// stacked [A rows | W rows] operand tile into a ring of LDS buffers with global_load_lds;
// consumer waves multiply them.  The two sides are coupled only through per-buffer counters
// in LDS (a software full/empty queue), not through workgroup barriers:
//   * a producer never waits for the consumers unless the ring is full, so the fill pipe stays
//     busy while the consumers convert and store a finished tile, and the first K-tiles of the
//     next tile are already in LDS when they come back;
//   * a consumer never waits for the producers unless its next K-tile has not landed.
// With a barrier per K-tile both sides advance in lock step, and a tile costs
// (fill time + epilogue time) instead of max(fill time, multiply + epilogue time).
//
// Counters (uint32 in LDS, zeroed before use, only ever incremented):
//   full[b]  += 1 by each producer wave when its share of a fill of buffer b has landed
//               (after s_waitcnt vmcnt proves it);  fill number f of buffer b is complete
//               when full[b] == PW * (f + 1).
//   empty[b] += 1 by each consumer wave when its fragments of the K-tile in buffer b are in
//               registers;  buffer b may be refilled for the f-th time when empty[b] == CW * f.
// A wave's LDS operations execute in order, and a fill's data is in LDS before vmcnt counts it,
// so "counter seen" implies "data visible".  Every wait is a bounded spin: if a counter never
// arrives (which would be a bug), the wave gives up after the spin limit, records that in a
// device word of the context (GemmEpilogue::wait_error) and runs on, so the grid always drains;
// the next hipq_ctx_synchronize reports the give-up as HIPQ_DEVICE_ERROR instead of returning a
// wrong product silently.
//
// Tile order: tile t -> (t % tiles_m, t / tiles_m).  With 256 workgroups and tiles_m a multiple
// of 64 a workgroup keeps one band of activation rows for its whole life and walks the weight
// panels; the workgroups of one XCD (ids congruent modulo 8) share 1/8 of the activation rows,
// which stay resident in that XCD's L2.
#pragma once

#include <type_traits>

#include "hipq_gemm_kernels.h"

namespace hipq {

constexpr int kSpinLimit = 1 << 20;  // default of hipq_ctx::wait_spin_limit

struct WaitPolicy {
    int spin_limit;
    uint32_t *error_word;  // device memory; set to 1 when a wait gives up
};

// The queue counters live in LDS.  They are read through an explicit LDS-address-space volatile
// pointer: a volatile access through a generic pointer is compiled to a flat load, which waits
// on vmcnt as well and so on every global store the wave has in flight.
typedef const volatile __attribute__((address_space(3))) uint32_t lds_counter_t;

__device__ __forceinline__ uint32_t read_counter(const uint32_t *counter) {
    return *(lds_counter_t *)counter;
}

// Spins until *counter >= target (wave-uniform), polling at most spin_limit more times after the
// first look; a wait that gives up is recorded in the policy's error word (one plain vector store).
__device__ __forceinline__ void wait_counter(const uint32_t *counter, uint32_t target, const WaitPolicy &wp,
                                             int lane) {
    bool reached = false;
    for (int spin = 0;; ++spin) {
        const uint32_t v = __builtin_amdgcn_readfirstlane(read_counter(counter));
        if (static_cast<int32_t>(v - target) >= 0) {
            reached = true;
            break;
        }
        if (spin >= wp.spin_limit) break;
        __builtin_amdgcn_s_sleep(1);
    }
    if (!reached && wp.error_word && lane == 0) *reinterpret_cast<volatile uint32_t *>(wp.error_word) = 1u;
    asm volatile("" ::: "memory");  // nothing that follows may be moved above the wait
}

__device__ __forceinline__ bool counter_reached(const uint32_t *counter, uint32_t target) {
    const uint32_t v = __builtin_amdgcn_readfirstlane(read_counter(counter));
    asm volatile("" ::: "memory");
    return static_cast<int32_t>(v - target) >= 0;
}

__device__ __forceinline__ void bump_counter(uint32_t *counter, int lane) {
    asm volatile("" ::: "memory");
    if (lane == 0) atomicAdd(counter, 1u);  // ds_add_u32; ordered after this wave's earlier LDS operations
}

template <int BM, int BN, int STAGES, int PW, int WM, int WN, int KG, int EPI, bool EVEN, bool RESIDUAL>
__global__ __launch_bounds__((PW + WM * WN) * kWave) void gemm_i8_persist_kernel(const int8_t *__restrict__ A,
                                                                                  const int8_t *__restrict__ W,
                                                                                  int M, int N, int K,
                                                                                  GemmEpilogue ep) {
    constexpr int BK = 128;
    constexpr int CPR = BK / 16;
    constexpr int RPI = 1024 / BK;
    constexpr int IPS = (BM + BN) / RPI;
    static_assert(BM % RPI == 0 && IPS % PW == 0, "stage loads divide evenly between producer waves");
    constexpr int IPW = IPS / PW;
    static_assert(IPW * STAGES < 64, "outstanding loads must fit vmcnt");
    constexpr int STAGE = (BM + BN) * BK;
    constexpr int CW = WM * WN;
    constexpr int TM = BM / WM, TN = BN / WN;
    constexpr int FM = TM / 32, FN = TN / 32;
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile is made of 32x32 MFMA blocks");
    constexpr int KS = BK / 32;
    constexpr int LAG = STAGES - 2;  // a producer wave reports fill q after it has requested fill q+LAG
    static_assert(LAG >= 1, "at least three buffers");
    static_assert(KS % KG == 0 && ((KS / KG) % 2 == 0 || KS / KG == 1), "k-steps of a K-tile divide into groups");

    extern __shared__ __attribute__((aligned(1024))) int8_t lds[];
    uint32_t *full = reinterpret_cast<uint32_t *>(lds + STAGES * STAGE);
    uint32_t *empty = full + STAGES;

    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const int ntiles = tiles_m * tiles_n;
    const int nk = K / BK;  // >= 1
    const int my_tiles = (ntiles - static_cast<int>(blockIdx.x) + static_cast<int>(gridDim.x) - 1) /
                         static_cast<int>(gridDim.x);
    const int T = my_tiles * nk;  // K-tiles this workgroup streams, in consumption order
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const WaitPolicy wp{ep.spin_limit, ep.wait_error};

    if (tid < 2 * STAGES) full[tid] = 0;
    __syncthreads();  // the only workgroup barrier: counters are zero before anyone uses them

    if (wave < PW) {
        // ---------------- producer ----------------
        const int8_t *src[IPW];
        auto set_tile = [&](int ti) {
            const int t = static_cast<int>(blockIdx.x) + ti * static_cast<int>(gridDim.x);
            const int m0 = (t % tiles_m) * BM, n0 = (t / tiles_m) * BN;
#pragma unroll
            for (int j = 0; j < IPW; ++j) {
                const int trow = (wave * IPW + j) * RPI + lane / CPR;  // row in the stacked [A rows | W rows] tile
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
        };
        int kt_issue = 0, ti_issue = 0;
        int buf = 0;        // buffer of the next fill
        uint32_t fill = 0;  // how many times that buffer has been filled before
        int sig_buf = 0;     // buffer of the oldest fill not yet reported
        int unreported = 0;  // fills requested but not yet reported (at most LAG between iterations)
        auto report_oldest = [&]() {
            // The oldest unreported fill has landed once only the newer ones are outstanding.
            wait_stages_outstanding<IPW, LAG>(unreported - 1);
            bump_counter(full + sig_buf, lane);
            sig_buf = sig_buf + 1 == STAGES ? 0 : sig_buf + 1;
            --unreported;
        };
        set_tile(0);
        for (int q = 0; q < T; ++q) {
            if (fill > 0 && !counter_reached(empty + buf, uint32_t(CW) * fill)) {
                // The ring is full.  Nothing is lost by waiting for the fills in flight, and the
                // consumers may be waiting for exactly those reports.
                while (unreported > 0) report_oldest();
                wait_counter(empty + buf, uint32_t(CW) * fill, wp, lane);  // consumers are done with the old contents
            }
            int8_t *base = lds + buf * STAGE + wave * (IPW * 1024);
            const size_t koff = size_t(kt_issue) * BK;
#pragma unroll
            for (int j = 0; j < IPW; ++j)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src[j] + koff),
                                                 (__attribute__((address_space(3))) void *)(base + j * 1024), 16, 0, 0);
            ++unreported;
            if (++buf == STAGES) {
                buf = 0;
                ++fill;
            }
            if (++kt_issue == nk) {
                kt_issue = 0;
                if (++ti_issue < my_tiles) set_tile(ti_issue);
            }
            if (unreported > LAG) report_oldest();
        }
        while (unreported > 0) report_oldest();
        return;
    }

    // ---------------- consumer ----------------
    const int cw = wave - PW;
    const int wm = cw % WM, wn = cw / WM;

    // LDS byte offsets (within a buffer) of this lane's fragment reads for row block 0 of each
    // operand.  Row block i lies 32 rows further on; the swizzle term (row>>1)&7 does not change
    // when the row advances by 32, so its offset is a compile-time constant more.
    int offA0[KS], offW0[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int col = s * 2 + lane / 32;
        const int rowA = wm * TM + lane % 32;
        const int rowW = BM + wn * TN + lane % 32;  // stacked-tile row
        offA0[s] = rowA * BK + ((col ^ ((rowA >> 1) & 7)) * 16);
        offW0[s] = rowW * BK + ((col ^ ((rowW >> 1) & 7)) * 16);
    }
    // Fragments are double buffered in groups of KG k-steps (32 bytes of K each): the reads of
    // group g+1 are in flight while the MFMAs of group g run, across K-tile and tile boundaries.
    // A group must hold enough MFMAs (KG*FM*FN of 32 cycles) to cover the LDS latency.
    constexpr int NGRP = KS / KG;
    v4i fa[2][KG][FM], fw[2][KG][FN];
    auto read_group = [&](int b, int g, int set) {
        const int8_t *st = lds + b * STAGE;
#pragma unroll
        for (int s = 0; s < KG; ++s) {
#pragma unroll
            for (int i = 0; i < FM; ++i) fa[set][s][i] = *reinterpret_cast<const v4i *>(st + offA0[g * KG + s] + i * 32 * BK);
#pragma unroll
            for (int j = 0; j < FN; ++j) fw[set][s][j] = *reinterpret_cast<const v4i *>(st + offW0[g * KG + s] + j * 32 * BK);
        }
    };
    v16i acc[FM][FN];
    // Ring position of the K-tile being multiplied (cur) and of the one after it (nxt).
    int cur_buf = 0, nxt_buf = 1 % STAGES;
    uint32_t nxt_fill = 0;  // fill number of the K-tile that will be read from nxt_buf
    int q_next = 1;         // index of the K-tile after the current one
    uint32_t full_seen = 0; // last value read of full[nxt_buf]
    // 16-byte (int8 output: 4-byte) accesses need rows that start on such a boundary.
    auto aligned_to = [](const void *ptr, unsigned a) { return (reinterpret_cast<uintptr_t>(ptr) & (a - 1)) == 0; };
    const bool vec_ok = (N % 4 == 0) && aligned_to(ep.out, EPI == EPI_I8 ? 4 : 16) &&
                        (EPI == EPI_I32 || (aligned_to(ep.sw, 16) && aligned_to(ep.bias, 16) && aligned_to(ep.residual, 16)));
    auto k_tile = [&](auto start_tag) {
        constexpr int START = decltype(start_tag)::value;  // fragment set that holds group 0 of this K-tile
#pragma unroll
        for (int g = 0; g < NGRP; ++g) {
            const int set = (START + g) & 1;
            wait_lgkmcnt0();  // fragments of this group are in registers
            if (g + 1 < NGRP) {
                read_group(cur_buf, g + 1, set ^ 1);
            } else {
                // Every fragment of the current K-tile is in registers: its buffer may be refilled.
                bump_counter(empty + cur_buf, lane);
                cur_buf = nxt_buf;
                if (q_next < T) {
                    // The counter of the next K-tile was requested one K-tile ago (its value came
                    // back with the fragments); only if it had not arrived by then is it polled.
                    const uint32_t want = uint32_t(PW) * (nxt_fill + 1);
                    if (static_cast<int32_t>(__builtin_amdgcn_readfirstlane(full_seen) - want) < 0) {
                        wait_counter(full + nxt_buf, want, wp, lane);  // next K-tile has landed
                    }
                    read_group(nxt_buf, 0, set ^ 1);
                }
                ++q_next;
                if (++nxt_buf == STAGES) {
                    nxt_buf = 0;
                    ++nxt_fill;
                }
                if (q_next < T) full_seen = read_counter(full + nxt_buf);
            }
#pragma unroll
            for (int s = 0; s < KG; ++s)
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int j = 0; j < FN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[set][s][i], fw[set][s][j], acc[i][j], 0, 0, 0);
            // Issue order: MFMAs with the fragment reads of the next group slipped in between.
#pragma unroll
            for (int q = 0; q < KG * FM * FN; ++q) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if (q < KG * (FM + FN)) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                if (q + KG * FM * FN < KG * (FM + FN)) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
        }
    };

    const float zpf = static_cast<float>(ep.zp_out);
    const bool has_bias = ep.bias != nullptr;
    wait_counter(full + 0, uint32_t(PW), wp, lane);  // first K-tile has landed
    read_group(0, 0, 0);
    if (T > 1) full_seen = read_counter(full + nxt_buf);

    for (int ti = 0; ti < my_tiles; ++ti) {
        const int t = static_cast<int>(blockIdx.x) + ti * static_cast<int>(gridDim.x);
        const int m0 = (t % tiles_m) * BM, n0 = (t / tiles_m) * BN;
        // Epilogue operands are requested now; they arrive while the tile is multiplied.
        // Interior tiles whose rows can be addressed in 16-byte pieces take the transposing
        // epilogue (lane = 4 consecutive columns of one row); the others the checked one
        // (lane = one column), which fetches its operands when it gets there.
        const bool fast = vec_ok && m0 + BM <= M && n0 + BN <= N;
        // Only the transposing epilogue reads these, and the bias only when there is one.  The
        // loads are nevertheless unconditional - where a value is not needed they read 16 valid
        // bytes of the activation matrix instead - because any other form (a constant first, or a
        // load under a condition) makes the register a merge of a loaded and a moved value, and
        // the compiler then waits at the top of every tile until all outstanding memory
        // operations, the previous epilogue's stores included, have completed.
        float4 sw4[FN], b4[FN];
        if constexpr (EPI != EPI_I32) {
            const float4 *dummy = reinterpret_cast<const float4 *>(A);
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const int nq = n0 + wn * TN + j * 32 + (lane % 8) * 4;
                sw4[j] = *(fast ? reinterpret_cast<const float4 *>(ep.sw + nq) : dummy);
                b4[j] = *((fast && has_bias) ? reinterpret_cast<const float4 *>(ep.bias + nq) : dummy);
            }
        }
        // Residual values of the whole wave tile, when they fit in registers: requested here, they
        // arrive while the tile is multiplied, and no load is issued between the epilogue's stores
        // (a load waits for every store issued before it: they share one counter).
        constexpr bool RES_PRE = RESIDUAL && EPI == EPI_F32 && FM * FN * 16 <= 32;
        float4 res_pre[RES_PRE ? FM : 1][RES_PRE ? FN : 1][4];
        if constexpr (RES_PRE) {
            if (fast) {
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int jj = 0; jj < FN; ++jj)
#pragma unroll
                        for (int hp = 0; hp < 4; ++hp) {
                            const int m = m0 + wm * TM + i * 32 + 16 * (hp / 2) + lane / 8 + 8 * (hp % 2);
                            const int nq = n0 + wn * TN + jj * 32 + (lane % 8) * 4;
                            res_pre[i][jj][hp] = *reinterpret_cast<const float4 *>(ep.residual + size_t(m) * N + nq);
                        }
            }
        }
        // Activation scales of this wave's rows, one row per lane (row block i in s_lane[i]); the
        // epilogue fetches the scale of each accumulator row with a lane shuffle.
        float s_lane[(TM + kWave - 1) / kWave];
        if constexpr (EPI != EPI_I32) {
            // One unconditional load per row block, for the same reason (a per-tensor scale is the
            // same address for every lane; the launcher checks that the scale is given).
#pragma unroll
            for (int u = 0; u < (TM + kWave - 1) / kWave; ++u) {
                const int m = m0 + wm * TM + u * kWave + lane;
                s_lane[u] = ep.sa[ep.sa_per_row ? (m < M ? m : M - 1) : 0];
            }
        }
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

        if constexpr (NGRP % 2 == 0) {
            for (int kt = 0; kt < nk; ++kt) k_tile(std::integral_constant<int, 0>{});
        } else {
            // One group per K-tile: the fragment sets alternate per K-tile, so two K-tiles are
            // unrolled to keep the set index static.  An odd K-tile at the end leaves the next
            // tile's first fragments in set 1; they are moved to set 0 (once per tile).
            int kt = 0;
            for (; kt + 1 < nk; kt += 2) {
                k_tile(std::integral_constant<int, 0>{});
                k_tile(std::integral_constant<int, 1>{});
            }
            if (kt < nk) {
                k_tile(std::integral_constant<int, 0>{});
                wait_lgkmcnt0();
#pragma unroll
                for (int sidx = 0; sidx < KG; ++sidx) {
#pragma unroll
                    for (int i = 0; i < FM; ++i) fa[0][sidx][i] = fa[1][sidx][i];
#pragma unroll
                    for (int j = 0; j < FN; ++j) fw[0][sidx][j] = fw[1][sidx][j];
                }
            }
        }

        // Epilogue.  32x32 accumulator block: lane holds column n = lane%32 and rows
        // m = 8*(r/4) + 4*(lane/32) + r%4 for r = 0..15.
        if (fast) {
            // Transposing epilogue.  The accumulators (lane = column) pass through a wave-private
            // 1 KiB LDS block, a quarter of a 32x32 block (8 rows) at a time, and come back with
            // lane l holding columns 4*(l%8)..+3 of row l/8: every global access is then a 16-byte
            // piece of a fully covered 128-byte line, a quarter of the store instructions of the
            // lane-per-column layout.  A wave's LDS operations execute in order, so it needs no
            // barrier to read back what it wrote.
            int32_t *tb = reinterpret_cast<int32_t *>(lds + STAGES * STAGE + 256) + cw * 256;
            // LDS traffic of block b+1 is issued before block b is converted and stored, so the
            // LDS round trip (long while the producers are refilling the ring) is overlapped.
            auto lds_block = [&](int b, v4i(&t)[4], float(&sr)[4]) {
                const int i = b / FN, j = b % FN;
#pragma unroll
                for (int hp = 0; hp < 4; ++hp) {
                    asm volatile("" ::: "memory");
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr)
                        tb[(4 * (lane / 32) + rr) * 32 + lane % 32] = acc[i][j][4 * hp + rr];
                    asm volatile("" ::: "memory");  // reads stay behind the writes (other lanes' data)
                    t[hp] = *reinterpret_cast<const v4i *>(tb + (lane / 8) * 32 + (lane % 8) * 4);
                }
                // The activation scales of the block's rows are fetched (lane shuffles, which go
                // through the LDS pipe) together with the block, one block ahead of their use.
                if constexpr (EPI != EPI_I32) {
#pragma unroll
                    for (int hp = 0; hp < 4; ++hp) {
                        const int wrow = i * 32 + 16 * (hp / 2) + lane / 8 + 8 * (hp % 2);  // row within the wave tile
                        sr[hp] = __shfl(s_lane[wrow / kWave], wrow % kWave, kWave);
                    }
                }
                asm volatile("" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);  // keep this block's LDS traffic ahead of the previous block's arithmetic
            };
            float4 res4[FN][4];
            auto out_block = [&](int b, v4i(&t)[4], float(&sr)[4]) {
                const int i = b / FN, j = b % FN;
                if constexpr (RESIDUAL && !RES_PRE) {
                    if (j == 0) {
#pragma unroll
                        for (int jj = 0; jj < FN; ++jj)
#pragma unroll
                            for (int hp = 0; hp < 4; ++hp) {
                                const int m = m0 + wm * TM + i * 32 + 16 * (hp / 2) + lane / 8 + 8 * (hp % 2);
                                const int nq = n0 + wn * TN + jj * 32 + (lane % 8) * 4;
                                res4[jj][hp] = *reinterpret_cast<const float4 *>(ep.residual + size_t(m) * N + nq);
                            }
                        wait_vmcnt<0>();  // before the stores below (see the checked path)
                    }
                }
#pragma unroll
                for (int hp = 0; hp < 4; ++hp) {
                    const int wrow = i * 32 + 16 * (hp / 2) + lane / 8 + 8 * (hp % 2);  // row within the wave tile
                    const int m = m0 + wm * TM + wrow;
                    const int nq = n0 + wn * TN + j * 32 + (lane % 8) * 4;
                    const size_t off = size_t(m) * N + nq;
                    if constexpr (EPI == EPI_I32) {
                        __builtin_nontemporal_store(t[hp], reinterpret_cast<v4i *>(static_cast<int32_t *>(ep.out) + off));
                    } else {
                        const float s_m = sr[hp];
                        const float swc[4] = {sw4[j].x, sw4[j].y, sw4[j].z, sw4[j].w};
                        const float bc[4] = {b4[j].x, b4[j].y, b4[j].z, b4[j].w};
                        float v[4];
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            v[c] = static_cast<float>(t[hp][c]) * (s_m * swc[c]);
                            if (has_bias) v[c] = v[c] + bc[c];
                        }
                        if constexpr (EPI == EPI_F32) {
                            if constexpr (RESIDUAL) {
                                const float4 rv = RES_PRE ? res_pre[RES_PRE ? i : 0][RES_PRE ? j : 0][hp] : res4[j][hp];
                                v[0] = v[0] + rv.x;
                                v[1] = v[1] + rv.y;
                                v[2] = v[2] + rv.z;
                                v[3] = v[3] + rv.w;
                            }
                            store_stream(reinterpret_cast<float4 *>(static_cast<float *>(ep.out) + off),
                                         make_float4(v[0], v[1], v[2], v[3]));
                        } else {
                            int q[4];
#pragma unroll
                            for (int c = 0; c < 4; ++c)
                                q[c] = clamp_to_int(round_mode<EVEN>(div_rn(v[c], ep.s_out, ep.s_out_inv)) + zpf, -128, 127);
                            store_stream(reinterpret_cast<uint32_t *>(static_cast<int8_t *>(ep.out) + off),
                                         pack4(q[0], q[1], q[2], q[3]));
                        }
                    }
                }
            };
            v4i tbuf[2][4];
            float srow[2][4];
            lds_block(0, tbuf[0], srow[0]);
#pragma unroll
            for (int b = 0; b < FM * FN; ++b) {
                if (b + 1 < FM * FN) lds_block(b + 1, tbuf[(b + 1) & 1], srow[(b + 1) & 1]);
                out_block(b, tbuf[b & 1], srow[b & 1]);
            }
            continue;
        }

        // Checked epilogue (edge tiles, unaligned outputs): lane = one column.
        float swv[FN], bv[FN];
        int nn[FN];
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            nn[j] = n0 + wn * TN + j * 32 + lane % 32;
            const int nc = nn[j] < N ? nn[j] : N - 1;
            swv[j] = 1.0f;
            bv[j] = 0.0f;
            if constexpr (EPI != EPI_I32) {
                swv[j] = ep.sw[nc];
                if (has_bias) bv[j] = ep.bias[nc];
            }
        }
        // Residual values: all row blocks at once when that fits in registers (then every load of
        // this wave has landed before the first store; a load issued between stores would wait for
        // all earlier stores to retire, since stores count in vmcnt too), else block by block.
        constexpr bool RES_ALL = FM * FN * 16 <= 64;
        float res[(RES_ALL ? FM : 1) * (RESIDUAL ? 1 : 0) + (RESIDUAL ? 0 : 1)][16][FN];
        auto load_residual = [&](int i, int slot) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * TM + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    res[slot][r][j] = 0.0f;
                    if constexpr (EPI == EPI_F32)
                        if (RESIDUAL && m < M && nn[j] < N) res[slot][r][j] = ep.residual[size_t(m) * N + nn[j]];
                }
            }
        };
        if constexpr (RES_ALL && RESIDUAL && EPI == EPI_F32) {
#pragma unroll
            for (int i = 0; i < FM; ++i) load_residual(i, i);
        }
        wait_vmcnt<0>();
        // Interior tiles (all but the last row / column of tiles) skip the per-element bounds
        // checks; addresses are one 64-bit base per column block plus row * (bytes per row).
        constexpr size_t ESZ = (EPI == EPI_I8) ? 1 : 4;
        const size_t row_bytes = size_t(N) * ESZ;
        auto store_tile = [&](auto checked_tag) {
            constexpr bool CHECKED = decltype(checked_tag)::value;
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                const int mrow = m0 + wm * TM + i * 32 + 4 * (lane / 32);
                if constexpr (!RES_ALL && EPI == EPI_F32 && RESIDUAL) {
                    load_residual(i, 0);
                    wait_vmcnt<0>();
                }
                float s_row[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    s_row[r] = 1.0f;
                    if constexpr (EPI != EPI_I32) {
                        const int row = i * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);  // row of the wave tile
                        s_row[r] = __shfl(s_lane[row / kWave], row % kWave, kWave);
                    }
                }
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    char *p0 = static_cast<char *>(ep.out) + (size_t(mrow) * N + nn[j]) * ESZ;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int cr = 8 * (r / 4) + (r % 4);
                        if (CHECKED && (mrow + cr >= M || nn[j] >= N)) continue;
                        char *p = p0 + size_t(cr) * row_bytes;
                        if constexpr (EPI == EPI_I32) {
                            __builtin_nontemporal_store(acc[i][j][r], reinterpret_cast<int32_t *>(p));
                        } else {
                            float v = static_cast<float>(acc[i][j][r]) * (s_row[r] * swv[j]);
                            if (has_bias) v = v + bv[j];
                            if constexpr (EPI == EPI_F32) {
                                if constexpr (RESIDUAL) v = v + res[RES_ALL ? i : 0][r][j];
                                __builtin_nontemporal_store(v, reinterpret_cast<float *>(p));
                            } else {
                                const int q = clamp_to_int(round_mode<EVEN>(div_rn(v, ep.s_out, ep.s_out_inv)) + zpf, -128, 127);
                                __builtin_nontemporal_store(static_cast<int8_t>(q), reinterpret_cast<int8_t *>(p));
                            }
                        }
                    }
                }
            }
        };
        if (m0 + BM <= M && n0 + BN <= N)
            store_tile(std::false_type{});
        else
            store_tile(std::true_type{});
    }
}

template <int BM, int BN, int STAGES, int PW, int WM, int WN, int KG, int EPI, bool EVEN>
static int32_t launch_persist(hipq_ctx *ctx, const int8_t *a, const int8_t *w, int M, int N, int K,
                              const GemmEpilogue &ep) {
    // ring of K-tile buffers + the queue counters + 1 KiB per consumer wave for the epilogue's transposition
    constexpr int kLds = STAGES * (BM + BN) * 128 + 256 + WM * WN * 1024;
    static_assert(kLds <= 160 * 1024, "LDS budget of one CU");
    constexpr int kThreads = (PW + WM * WN) * kWave;
    const bool with_residual = EPI == EPI_F32 && ep.residual != nullptr;
    auto kernel = with_residual ? gemm_i8_persist_kernel<BM, BN, STAGES, PW, WM, WN, KG, EPI, EVEN, EPI == EPI_F32>
                                : gemm_i8_persist_kernel<BM, BN, STAGES, PW, WM, WN, KG, EPI, EVEN, false>;
    static bool configured[16][2] = {};  // per device and instantiation: raise the dynamic LDS limit once
    if (ctx->device < 16 && !configured[ctx->device][with_residual]) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
        if (e != hipSuccess)
            return fail(HIPQ_DEVICE_ERROR, "gemm_i8: cannot reserve %d bytes of LDS: %s", kLds, hipGetErrorString(e));
        configured[ctx->device][with_residual] = true;
    }
    if (K % 128 != 0 || K < 128) return fail(HIPQ_INVALID_ARGUMENT, "gemm_i8 (persistent): K must be a multiple of 128");
    if (EPI != EPI_I32 && (!ep.sa || !ep.sw)) return fail(HIPQ_INVALID_ARGUMENT, "gemm_i8 (persistent): scales must be given");
    const int tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    const int grid = tiles < ctx->num_cus ? tiles : ctx->num_cus;
    GemmEpilogue placed = ep;
    placed.wait_error = ctx->wait_error;
    placed.spin_limit = ctx->wait_spin_limit;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), kLds, ctx->stream, a, w, M, N, K, placed);
    return check_launch("gemm_i8 (persistent)");
}

}  // namespace hipq
