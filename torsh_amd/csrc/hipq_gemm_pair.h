// int8 GEMM on fragment-packed operands with one 128 x 128 output tile per PAIR of compute units: the two
// workgroups of a pair take one half of K each and exchange partial sums through the L2 of the XCD they share.
//
// Why.  With one 128 x 64 tile per compute unit (gemm_i8_packed_kernel) a wave multiplies 4 x 2 blocks per k block:
// 6 KiB of operands for 8 MFMAs, 96 bytes per clock and compute unit against the 64 that the vector-memory path and
// the XCD's L2 (2 KiB per clock for 32 compute units) deliver.  A 4 x 4 block tile needs 8 KiB for 16 MFMAs,
// 64 bytes per clock: balanced, and a compute unit pulls (128 + 128) * K/2 bytes instead of (128 + 64) * K, two
// thirds.  The price: 256 accumulator registers per lane (the unified 512-register file of a wave that has its
// SIMD to itself), a K-split sum inside the workgroup of twice the size, and the exchange between the pair.
//
// Who is paired.  The dispatcher hands workgroups to the 8 XCDs round robin, so ids b and b + 8 run on one XCD and
// see one L2 (hipq_ctx_create checks this on the device, and a kernel that finds its partner on another XCD says
// so through the context's give-up word instead of using stale data).  Partial sums cross with plain stores, which
// land in that L2, followed - once the stores are acknowledged - by a flag word; the reader polls the flag past
// its L1 and then reads the partials past its L1 too.  No cache-wide fence, no trip through device-coherent memory.
// A flag is cleared by its reader, so every launch finds them zero and a captured launch can be replayed.
//
// Measured at M = 512, N = K = 4096 (256 workgroups, operands from memory; 128 x 64 tiles / this form, shader
// cycles): K loop 18.2-19.6 k / 14.4-15.3 k, K-split sum inside the workgroup 2.2 k / 5.0 k, exchange - / 5.0 k,
// stores 2.2 k / 1.7 k + 1.8 k to retire: 12.2 / 14.6 us from the first wave's start to the last one's end, and
// 14.7 / 18-22 us from launch to launch (the partial sums sit dirty in the L2 until the kernel ends).  The shorter
// loop does not pay for the larger sum and the exchange, so this form is reached through a test hook only.
// Polling the flag with a read-modify-write at workgroup scope (which executes in the L2) instead of an
// agent-scope load was slower still (exchange 8.6 k cycles); four register stages instead of two changed nothing.
//
// Both workgroups of a pair must be resident together (the grid is at most one workgroup per compute unit, and the
// host launches this form only then); waits are bounded like every wait of this library.
//
// Included by hipq_gemm_packed.h, after the kernels whose helpers it uses.
#pragma once

namespace hipq {

// Per context: flags (one 32-bit word per wave that receives) and the exchange buffer (8 KiB per wave).
struct PairExchange {
    uint32_t *flags = nullptr;
    int8_t *buf = nullptr;
};

constexpr size_t kPairBytesPerWorkgroup = 4 * 8192;  // four waves x two 32 x 32 int32 blocks
constexpr int kPairLds = 4 * 3 * 2 * 4096;           // K-split sum, two column blocks at a time

__device__ __forceinline__ uint32_t xcc_id() {
    uint32_t v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID, 0, 4)" : "=s"(v));
    return v;
}

// Records which XCD every workgroup of a (num_cus)-workgroup grid runs on (hipq_ctx_create's check).
__global__ void xcc_probe_kernel(uint32_t *out) {
    if (threadIdx.x == 0) out[blockIdx.x] = xcc_id();
}

// D register stages of 8 KiB per wave in flight.  M and N are multiples of 128, the k blocks a multiple of 8 * D,
// the grid is 2 * (M / 128) * (N / 128) workgroups with (M / 128) * (N / 128) a multiple of 8.  fp32 or int32
// epilogue on whole tiles (store_block_interior).  TRACE: stamps as gemm_i8_packed_kernel, with point 3 = K-split
// sum inside the workgroup done and point 4 = partner's partials added (instead of: stores issued).
template <int D, int EPI, bool TRACE = false>
__global__ __launch_bounds__(256) void gemm_i8_packed_pair_kernel(const int8_t *__restrict__ PA,
                                                                  const int8_t *__restrict__ PW, int M, int N, int K,
                                                                  GemmEpilogue ep, PairExchange px) {
    static_assert(EPI == EPI_F32 || EPI == EPI_I32, "whole-tile epilogues only");
    extern __shared__ __attribute__((aligned(1024))) int8_t lds[];
    constexpr int WK = 4, TB = 4;
    const int KB = static_cast<int>(packed_k_blocks(K));
    const int tiles_m = M / 128, tiles_n = N / 128;
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    // Slots 2t and 2t + 1 of an XCD (workgroup ids 8 apart) are the two K halves of the XCD's tile t.
    const int b = blockIdx.x;
    const int xcd = b % 8, slot = b / 8;
    const int half = slot % 2;
    int tile_m, tile_n;
    tile_of_xcd_slot(tiles_m, tiles_n, ep.xcd_gm, ep.xcd_gn, xcd, slot / 2, &tile_m, &tile_n);
    const int tile = tile_n * tiles_m + tile_m;
    unsigned long long stamp[kTraceWords] = {};
    auto mark = [&](int i) {
        if constexpr (TRACE) stamp[i] = __builtin_readcyclecounter();
    };
    if constexpr (TRACE) stamp[kTracePoints] = __builtin_amdgcn_s_memrealtime();
    mark(0);

    // A wave numbers the tile's row blocks from the one it will own after the K-split sum (row block
    // (wave + i) % 4) and its column blocks from the first of the two this workgroup finishes (column block
    // (2 * half + j) % 4): "keep block 0 of the rows, columns 0 and 1" is then the same code for every wave of
    // either workgroup.
    const int n0 = tile_n * 128 + half * 64;  // first column this workgroup stores
    float swv[2], bv[2], sa0 = 1.0f;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int n = n0 + j * 32 + lane % 32;
        swv[j] = 1.0f;
        bv[j] = 0.0f;
        if constexpr (EPI != EPI_I32) {
            swv[j] = ep.sw[n];
            if (ep.bias) bv[j] = ep.bias[n];
        }
    }
    if constexpr (EPI != EPI_I32)
        if (!ep.sa_per_row) sa0 = ep.sa ? ep.sa[0] : ep.sa_scalar;

    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(PA), 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(PW), 0, 0x7fffffff, 0x00020000);
    const int kb0 = half * (KB / 2) + wave;  // this wave's k blocks: kb0 + 4 * step
    int soa[TB], sow[TB];
#pragma unroll
    for (int i = 0; i < TB; ++i) soa[i] = ((tile_m * TB + (wave + i) % TB) * KB + kb0) * 1024;
#pragma unroll
    for (int j = 0; j < TB; ++j) sow[j] = ((tile_n * TB + (2 * half + j) % TB) * KB + kb0) * 1024;
    const int steps = KB / (2 * WK);
    // The four tiles of a weight panel (same XCD, same half) start a quarter of the way apart, so that each weight
    // line is fetched by one of them and found in the L2 by the other three; activations that come from memory are
    // staggered over the XCDs as well (see gemm_i8_packed_kernel).
    int rot = (tile_m % 4) * (steps / 4) + (ep.fresh_activations ? 0 : xcd * ((steps / 8) | 1));
    while (rot >= steps) rot -= steps;
    const int voff = lane * 16;

    v4i fa[D][TB], fb[D][TB];
    auto issue = [&](int s, int st) {
        int sr = s + rot;
        sr = sr >= steps ? sr - steps : sr;
        const int koff = sr * (WK * 1024);
#pragma unroll
        for (int i = 0; i < TB; ++i)
            fa[st][i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(ra, voff, soa[i] + koff, 0));
#pragma unroll
        for (int j = 0; j < TB; ++j)
            fb[st][j] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rw, voff, sow[j] + koff, 0));
    };
    v16i acc[TB][TB];
#pragma unroll
    for (int i = 0; i < TB; ++i)
#pragma unroll
        for (int j = 0; j < TB; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    auto compute = [&](int st) {
#pragma unroll
        for (int i = 0; i < TB; ++i)
#pragma unroll
            for (int j = 0; j < TB; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[st][i], fb[st][j], acc[i][j], 0, 0, 0);
    };
#pragma unroll
    for (int u = 0; u < D; ++u) issue(u, u);
    if constexpr (TRACE) {
        wait_vmcnt<(D - 1) * 2 * TB>();
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
        asm volatile("s_nop 15\n\ts_nop 15" ::"v"(acc[TB - 1][TB - 1][0]));
        mark(2);
    }

    // K-split sum inside the workgroup, two column blocks at a time: block i (i >= 1) of a wave goes to its owner,
    // wave (wave + i) % 4, through LDS: [owner][slot i - 1][column block of the round][4 registers][lane].
    v4i *red = reinterpret_cast<v4i *>(lds);
    auto ksum = [&](int j0) {
#pragma unroll
        for (int i = 1; i < TB; ++i) {
            const int owner = (wave + i) % TB;
            v4i *dst = red + ((owner * (TB - 1) + (i - 1)) * 2 * 4) * kWave + lane;
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    dst[(j * 4 + g) * kWave] = v4i{acc[i][j0 + j][4 * g], acc[i][j0 + j][4 * g + 1],
                                                   acc[i][j0 + j][4 * g + 2], acc[i][j0 + j][4 * g + 3]};
        }
    };
    auto kread = [&](int j0, v16i (&sum)[2]) {
        v4i part[TB - 1][2][4];
        const v4i *src = red + (wave * (TB - 1) * 2 * 4) * kWave + lane;
#pragma unroll
        for (int sl = 0; sl < TB - 1; ++sl)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) part[sl][j][g] = src[((sl * 2 + j) * 4 + g) * kWave];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                int v = acc[0][j0 + j][r];
#pragma unroll
                for (int sl = 0; sl < TB - 1; ++sl) v += part[sl][j][r / 4][r % 4];
                sum[j][r] = v;
            }
    };
    // First the two column blocks the partner finishes: they leave for its exchange slot while this workgroup sums
    // the two it keeps.
    v16i give[2], keep[1][2];
    ksum(2);
    __syncthreads();
    kread(2, give);
    const size_t my_slot = size_t(tile) * 2 + half, partner_slot = size_t(tile) * 2 + (1 - half);
    {
        v4i *dst = reinterpret_cast<v4i *>(px.buf + (partner_slot * 4 + wave) * 8192) + lane;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                dst[(j * 4 + g) * kWave] = v4i{give[j][4 * g], give[j][4 * g + 1], give[j][4 * g + 2], give[j][4 * g + 3]};
    }
    __syncthreads();  // every wave has read the first round
    ksum(0);
    // The stores above are acknowledged (they sit in the XCD's L2): tell the partner's wave of the same number.
    asm volatile("" ::: "memory");
    wait_vmcnt<0>();
    asm volatile("" ::: "memory");
    const uint32_t mine = 0x100u | xcc_id();
    if (lane == 0)
        __hip_atomic_store(px.flags + partner_slot * 4 + wave, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    kread(0, keep[0]);
    mark(3);
    // The partner's partial sums of the two blocks kept here.
    {
        uint32_t *flag = px.flags + my_slot * 4 + wave;
        uint32_t seen = 0;
        for (int spin = 0; spin <= ep.spin_limit; ++spin) {
            seen = __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (seen != 0) break;
            __builtin_amdgcn_s_sleep(1);
        }
        seen = __builtin_amdgcn_readfirstlane(seen);
        if (seen != mine) {
            // nothing came within the limit, or it came from another XCD, whose stores this L2 does not hold
            if (lane == 0) __hip_atomic_store(ep.wait_error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            asm volatile("" ::: "memory");
            const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(
                px.buf + (my_slot * 4 + wave) * 8192, 0, 8192, 0x00020000);
            v4i got[2][4];
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g)  // sc1: past this compute unit's L1
                    got[j][g] = __builtin_bit_cast(
                        v4i, __builtin_amdgcn_raw_buffer_load_b128(rx, voff, (j * 4 + g) * 1024, /*sc1*/ 16));
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) keep[0][j][r] += got[j][r / 4][r % 4];
        }
        if (lane == 0 && seen != 0) __hip_atomic_store(flag, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    mark(4);
    store_block_interior<2, EPI>(keep, ep, N, tile_m * 128 + wave * 32, n0, lane, swv, bv, sa0);
    if constexpr (TRACE) {
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

// Whether the product can run as pairs, and its launch.  Returns false when the shape is left to the other forms.
//   - whole 128 x 128 tiles, their number a multiple of 8 (every XCD gets whole pairs), two workgroups per tile
//     and all of them resident together: at most one workgroup per compute unit of this context's share;
//   - k blocks a multiple of 8 * D;
//   - no residual (store_block_interior has none), fp32 or int32 output;
//   - the device pairs workgroup ids 8 apart on one XCD (ctx->pair_ok).
// Reached through variant 12 only (a test hook): see the measurements at the top of this file.
template <int EPI, bool EVEN>
static bool launch_pair_if_fits(hipq_ctx *ctx, const int8_t *pa, const int8_t *pw, size_t m, size_t n, size_t k,
                                const GemmEpilogue &ep, int32_t *rc) {
    if constexpr (EPI == EPI_I8) {
        return false;
    } else {
        constexpr int D = 2;
        const size_t KB = packed_k_blocks(k);
        if (!ctx->pair_ok || ep.residual || m % 128 || n % 128 || KB % (8 * D)) return false;
        const size_t tiles_m = m / 128, tiles_n = n / 128, tiles = tiles_m * tiles_n;
        const int share = ctx->resident_share > 0 ? ctx->resident_share : 1;
        if (tiles % 8 || 2 * tiles > size_t(ctx->num_cus / share)) return false;
        // Worth it where the 128 x 64 tiles fill the device once: with fewer tiles the weight-streaming forms win.
        if (2 * tiles < size_t(ctx->num_cus)) return false;
        const bool trace = ctx->trace && ctx->trace_bytes >= 2 * tiles * 4 * kTraceWords * sizeof(unsigned long long);
        if (ctx->trace && !trace) return false;
        PairExchange px;
        *rc = pair_area(ctx, 2 * tiles * 4 * sizeof(uint32_t), 2 * tiles * kPairBytesPerWorkgroup, &px.flags, &px.buf);
        if (*rc) return true;
        static bool configured[16][2] = {};
        auto configure = [&](const void *kernel, int which) -> int32_t {
            if (ctx->device < 16 && !configured[ctx->device][which]) {
                const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kPairLds);
                if (e != hipSuccess)
                    return fail(HIPQ_DEVICE_ERROR, "gemm_i8 (pairs): cannot reserve %d bytes of LDS: %s", kPairLds,
                                hipGetErrorString(e));
                configured[ctx->device][which] = true;
            }
            return HIPQ_SUCCESS;
        };
        GemmEpilogue placed = ep;
        pick_xcd_rectangle(static_cast<int>(tiles_m), static_cast<int>(tiles_n), 128, 128, &placed.xcd_gm, &placed.xcd_gn);
        placed.spin_limit = ctx->wait_spin_limit;
        placed.wait_error = ctx->wait_error;
        const int M = static_cast<int>(m), N = static_cast<int>(n), K = static_cast<int>(k);
        const dim3 grid(static_cast<unsigned>(2 * tiles));
        if (trace) {
            auto kernel = gemm_i8_packed_pair_kernel<D, EPI, true>;
            if ((*rc = configure(reinterpret_cast<const void *>(kernel), 1))) return true;
            placed.trace = static_cast<unsigned long long *>(ctx->trace);
            hipLaunchKernelGGL(kernel, grid, dim3(256), kPairLds, ctx->stream, pa, pw, M, N, K, placed, px);
        } else {
            auto kernel = gemm_i8_packed_pair_kernel<D, EPI, false>;
            if ((*rc = configure(reinterpret_cast<const void *>(kernel), 0))) return true;
            hipLaunchKernelGGL(kernel, grid, dim3(256), kPairLds, ctx->stream, pa, pw, M, N, K, placed, px);
        }
        *rc = check_launch("gemm_i8 (pairs)");
        return true;
    }
}

}  // namespace hipq
