// Machine probes: what the vector-memory path of a compute unit and the matrix pipes deliver on the device at hand,
// measured by the kernel's own clocks.  The figures decide which GEMM tiling can pay (bytes per MFMA against bytes
// per clock), so they are part of the library's tuning aids (torsh_hipq_testing.h), not of the binding surface.
#include "hipq_gemm_kernels.h"

namespace hipq {

typedef int v16i __attribute__((ext_vector_type(16)));

// One workgroup of four waves per grid slot.  Every step a wave requests LOADS fragments of 1 KiB
// (buffer_load_dwordx4, one fully coalesced instruction each, as the packed GEMM does) and issues MFMAS
// v_mfma_i32_32x32x32_i8; two register stages, loads of a stage behind the MFMAs of the other, as in the GEMM's
// main loop.  Region r of `region_bytes` is walked round and round by the `share` workgroups of one XCD that have
// it in common (workgroup ids congruent modulo 8 share an XCD): share = 1: every compute unit streams lines of
// its own; share = 4: four compute units ask the XCD's L2 for the same lines.  region_bytes >= 64 KiB defeats the
// 32 KiB L1.  At most 256 registers, so that two workgroups share a compute unit (two waves per SIMD) when the grid
// has that many.  out[workgroup] = {shader-clock cycles, 100 MHz ticks, checksum} of wave 0.
template <int LOADS, int MFMAS>
__global__ __launch_bounds__(256, 2) void probe_vector_memory_kernel(const int8_t *__restrict__ buf, int region_bytes,
                                                                  int share, int steps, unsigned long long *out) {
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int b = blockIdx.x;
    const int region = b % 8 + 8 * ((b / 8) / share);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t *>(buf) + size_t(region) * region_bytes, 0, region_bytes, 0x00020000);
    const int voff = lane * 16;
    const int frags = region_bytes / 1024;  // a power of two
    // Workgroups that share a region start a quarter of it apart (as sibling tiles of the GEMM do).
    int pos = (wave + ((b / 8) % share) * (frags / 4)) & (frags - 1);
    constexpr int NL = LOADS > 0 ? LOADS : 1;
    v4i f[2][NL];
    v16i acc[8];
#pragma unroll
    for (int a = 0; a < 8; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][r] = 0;
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int q = 0; q < NL; ++q) f[st][q] = v4i{lane, st, q, 1};
    auto issue = [&](int st) {
#pragma unroll
        for (int q = 0; q < LOADS; ++q) {
            f[st][q] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rs, voff, pos * 1024, 0));
            pos = (pos + 4) & (frags - 1);
        }
    };
    auto compute = [&](int st) {
        if constexpr (MFMAS > 0) {
#pragma unroll
            for (int a = 0; a < MFMAS; ++a)
                acc[a % 8] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f[st][a % NL], f[st][(a + 1) % NL], acc[a % 8], 0, 0, 0);
        } else {
#pragma unroll
            for (int q = 0; q < LOADS; ++q) acc[0][q % 16] ^= f[st][q][0] ^ f[st][q][3];  // the data must arrive
        }
    };
    __syncthreads();
    const unsigned long long c0 = __builtin_readcyclecounter(), w0 = __builtin_amdgcn_s_memrealtime();
    issue(0);
    issue(1);
    for (int s = 2; s < steps; s += 2) {
        compute(0);
        issue(0);
        compute(1);
        issue(1);
    }
    compute(0);
    compute(1);
    int sum = 0;
#pragma unroll
    for (int a = 0; a < 8; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) sum ^= acc[a][r];
    const unsigned long long c1 = __builtin_readcyclecounter(), w1 = __builtin_amdgcn_s_memrealtime();
    if (threadIdx.x == 0) {
        out[size_t(b) * 3] = c1 - c0;
        out[size_t(b) * 3 + 1] = w1 - w0;
        out[size_t(b) * 3 + 2] = static_cast<unsigned>(sum);
    }
}

// What the hardware does with a raw buffer access whose scalar offset, alone or together with the lane's offset,
// reaches past the descriptor's extent.  The row-panel GEMM kernels give their descriptors exact extents and lean on
// the answer (loads give zeros and touch no memory, stores are dropped) for column blocks past N, k blocks past K and
// rows past M, so a test holds the device at hand to it.  One wave: lane l loads the dword at byte 4 l + soffset of a
// descriptor of `extent` bytes over `mem`, then stores 0x7777 there.
__global__ __launch_bounds__(kWave) void probe_range_check_kernel(int *mem, int extent, int soffset, int *loaded) {
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(mem, 0, extent, 0x00020000);
    const int lane = threadIdx.x;
    loaded[lane] = __builtin_amdgcn_raw_buffer_load_b32(r, lane * 4, soffset, 0);
    __builtin_amdgcn_raw_buffer_store_b32(0x7777, r, lane * 4, soffset, 0);
}

}  // namespace hipq

using namespace hipq;

extern "C" int32_t hipq_probe_buffer_range_check(hipq_ctx *ctx, int32_t *mem, size_t mem_bytes, int32_t extent,
                                                 int32_t soffset, int32_t *loaded) {
    HIPQ_ENTER(ctx);
    HIPQ_REQUIRE_PTR(mem);
    HIPQ_REQUIRE_PTR(loaded);
    // every address the wave could reach if nothing were checked lies inside the caller's allocation
    if (extent < 0 || soffset < 0 || size_t(extent) > mem_bytes || size_t(soffset) + kWave * 4 > mem_bytes)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: extent and soffset + 256 must lie within the %zu bytes of mem", __func__,
                    mem_bytes);
    hipLaunchKernelGGL(probe_range_check_kernel, dim3(1), dim3(kWave), 0, ctx->stream, mem, extent, soffset, loaded);
    return check_launch("probe_range_check");
}

extern "C" int32_t hipq_probe_vector_memory_path(hipq_ctx *ctx, const int8_t *buf, size_t buf_bytes, int32_t workgroups,
                                                 int32_t region_bytes, int32_t share, int32_t loads_per_step,
                                                 int32_t mfmas_per_step, int32_t steps, uint64_t *out) {
    HIPQ_ENTER(ctx);
    HIPQ_REQUIRE_PTR(buf);
    HIPQ_REQUIRE_PTR(out);
    if (workgroups < 1 || workgroups > 4096 || share < 1 || steps < 2 || steps % 2 != 0)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: workgroups in 1..4096, share >= 1, an even number of steps", __func__);
    if (region_bytes < 4096 || (region_bytes & (region_bytes - 1)))
        return fail(HIPQ_INVALID_ARGUMENT, "%s: region_bytes must be a power of two >= 4096", __func__);
    const size_t regions = 8 * ((size_t(workgroups) + 7) / 8 + size_t(share) - 1) / size_t(share) + 8;
    if (regions * size_t(region_bytes) > buf_bytes)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: the buffer holds fewer than %zu regions", __func__, regions);
    auto *o = reinterpret_cast<unsigned long long *>(out);
#define HIPQ_PROBE(L, M)                                                                                          \
    if (loads_per_step == L && mfmas_per_step == M) {                                                             \
        hipLaunchKernelGGL((probe_vector_memory_kernel<L, M>), dim3(workgroups), dim3(256), 0, ctx->stream, buf,  \
                           region_bytes, share, steps, o);                                                        \
        return check_launch("probe_vector_memory");                                                               \
    }
    HIPQ_PROBE(6, 0)
    HIPQ_PROBE(8, 0)
    HIPQ_PROBE(0, 8)
    HIPQ_PROBE(0, 16)
    HIPQ_PROBE(6, 8)
    HIPQ_PROBE(8, 16)
    HIPQ_PROBE(4, 8)
#undef HIPQ_PROBE
    return fail(HIPQ_INVALID_ARGUMENT, "%s: (loads, MFMAs) per step must be one of (6,0) (8,0) (0,8) (0,16) (6,8) (8,16) (4,8)",
                __func__);
}
