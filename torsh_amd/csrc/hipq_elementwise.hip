// HBM-streaming kernels of the quantized path: min/max reduction, per-tensor and
// per-row quantize, dequantize, requantize.  All are bandwidth bound; the design
// rule is one coalesced 16-byte load per lane per instruction (a wavefront reads
// 1 KiB contiguous), enough independent loads in flight per lane to cover HBM
// latency, and wave-level shuffles for the reductions.
#include "hipq_internal.h"
#include "hipq_math.h"
#include <type_traits>

#include "hipq_meeting.h"

namespace hipq {

constexpr int kVecPerThread = 4;                         // float4 loads in flight per lane
constexpr int kTileVec = kBlock * kVecPerThread;         // float4s per block iteration

// Stage 1 of the range reduction: each block folds a strided set of 4096-element
// tiles and writes one (min,max) partial.
__device__ __forceinline__ MinMax minmax_of_block_share(const float *__restrict__ x, size_t n, float *lds) {
    MinMax m{INFINITY, -INFINITY};
    const bool aligned = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
    const size_t nvec = aligned ? n / 4 : 0;
    const float4 *x4 = reinterpret_cast<const float4 *>(x);
    const size_t ntiles = (nvec + kTileVec - 1) / kTileVec;
    for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const size_t base = t * kTileVec + threadIdx.x;
        float4 v[kVecPerThread];
        if ((t + 1) * kTileVec <= nvec) {  // whole tile: unguarded loads issue back to back
#pragma unroll
            for (int i = 0; i < kVecPerThread; ++i) v[i] = load_stream(x4 + base + size_t(i) * kBlock);
        } else {
#pragma unroll
            for (int i = 0; i < kVecPerThread; ++i) {
                const size_t idx = base + size_t(i) * kBlock;
                // The filler leaves min and max as they are.
                v[i] = idx < nvec ? x4[idx] : make_float4(INFINITY, INFINITY, INFINITY, INFINITY);
            }
        }
#pragma unroll
        for (int i = 0; i < kVecPerThread; ++i) {
            m.mn = fminf(m.mn, fminf(fminf(v[i].x, v[i].y), fminf(v[i].z, v[i].w)));
        }
        if ((t + 1) * kTileVec > nvec) {
#pragma unroll
            for (int i = 0; i < kVecPerThread; ++i)
                if (base + size_t(i) * kBlock >= nvec) v[i] = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
        }
#pragma unroll
        for (int i = 0; i < kVecPerThread; ++i) {
            m.mx = fmaxf(m.mx, fmaxf(fmaxf(v[i].x, v[i].y), fmaxf(v[i].z, v[i].w)));
        }
    }
    for (size_t i = nvec * 4 + size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += size_t(gridDim.x) * kBlock)
        acc_minmax(m, x[i]);
    return block_minmax(m, lds);
}

__global__ __launch_bounds__(kBlock) void minmax_partial_kernel(const float *__restrict__ x, size_t n,
                                                                 float2 *__restrict__ partials) {
    __shared__ float lds[2 * kBlock / kWave];
    const MinMax r = minmax_of_block_share(x, n, lds);
    if (threadIdx.x == 0) partials[blockIdx.x] = make_float2(r.mn, r.mx);
}

// What a finished range reduction writes: {min, max}, max|x|, and/or a hipq_qparams derived with `flavor`.
struct RangeOutputs {
    float *minmax;
    float *absmax;
    hipq_qparams *params;
    int flavor, qmin, qmax;
};

__device__ __forceinline__ void write_range_outputs(const RangeOutputs &o, MinMax r) {
    if (o.minmax) {
        o.minmax[0] = r.mn;
        o.minmax[1] = r.mx;
    }
    if (o.absmax) *o.absmax = fmaxf(fabsf(r.mn), fabsf(r.mx));
    if (o.params) {
        float s;
        int zp;
        int st = params_from_minmax(r.mn, r.mx, o.flavor, o.qmin, o.qmax, &s, &zp);
        o.params->scale = s;
        o.params->zero_point = zp;
        o.params->min_val = r.mn;
        o.params->max_val = r.mx;
        o.params->status = st;
    }
}

// Both stages in one launch: every workgroup publishes its partial as tagged words of the context
// (hipq_meeting.h) and is done; workgroup 0, which the dispatcher starts first, stays to collect them and writes the
// outputs.  Nobody but workgroup 0 waits, so the grid need not be resident at once.  One trip through memory after
// the last partial instead of a second launch: 14.1 -> ~13 us for 16 Mi elements.
__global__ __launch_bounds__(kBlock) void minmax_one_launch_kernel(const float *__restrict__ x, size_t n,
                                                                    uint32_t *words, int spin_limit,
                                                                    RangeOutputs outs) {
    __shared__ float lds[kMeetingLdsFloats];
    const uint32_t gen = meeting_number(words);
    const MinMax r = minmax_of_block_share(x, n, lds);
    meeting_publish_range(words, gen, r);
    if (blockIdx.x != 0) return;
    MinMax t;
    const bool gave_up = meeting_collect_range(words, gen, spin_limit, lds, &t);
    meeting_close(words, gen, gave_up);
    if (threadIdx.x == 0) {
        meeting_mark_ready(words, gen);
        if (gave_up) t = MinMax{__builtin_nanf(""), __builtin_nanf("")};  // never a range made of some of the partials
        write_range_outputs(outs, t);
    }
}

// Stage 2: one block folds the partials and writes what the caller asked for:
// {min,max}, max|x|, and/or a hipq_qparams derived with `flavor`.
__global__ __launch_bounds__(kBlock) void minmax_final_kernel(const float2 *__restrict__ partials, int nparts,
                                                               float *__restrict__ out_minmax,
                                                               float *__restrict__ out_absmax,
                                                               hipq_qparams *__restrict__ out_params, int flavor,
                                                               int qmin, int qmax) {
    __shared__ float lds[2 * kBlock / kWave];
    MinMax m{INFINITY, -INFINITY};
    for (int i = threadIdx.x; i < nparts; i += kBlock) {
        float2 p = partials[i];
        m.mn = fminf(m.mn, p.x);
        m.mx = fmaxf(m.mx, p.y);
    }
    MinMax r = block_minmax(m, lds);
    if (threadIdx.x == 0) write_range_outputs(RangeOutputs{out_minmax, out_absmax, out_params, flavor, qmin, qmax}, r);
}

__global__ void qparams_kernel(const float *__restrict__ minmax, int flavor, int qmin, int qmax,
                               hipq_qparams *__restrict__ out) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        float s;
        int zp;
        const float mn = minmax[0], mx = minmax[1];
        int st = params_from_minmax(mn, mx, flavor, qmin, qmax, &s, &zp);
        out->scale = s;
        out->zero_point = zp;
        out->min_val = mn;
        out->max_val = mx;
        out->status = st;
    }
}

__global__ void fill_i32_kernel(int32_t *p, int32_t v, size_t n) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

template <typename OutT>
__device__ __forceinline__ OutT to_out(float q) {
    if constexpr (sizeof(OutT) == 4)
        return q;  // f32 carrier keeps NaN
    else
        return static_cast<OutT>(cvt_i32_sat(q));  // q is already clamped; NaN -> 0
}

// What a dynamic quantize folds in front of its element loop: the range partials of
// minmax_partial_kernel, the parameter formula, and where to publish the result.
struct DynamicRange {
    const float2 *partials;  // null: not a dynamic call
    int nparts;
    int flavor, qmin, qmax;
    hipq_qparams *out_params;
    // Fused Linear forward: a range that is not finite (where the reference returns InvalidArgument,
    // algorithms.rs:403-407) still has to leave defined operands for the GEMM that follows on the
    // stream.  With `poison` set the published scale is NaN and every code 0, so every output of that
    // GEMM is NaN and the status word says why; without it the kernel returns without writing codes.
    int poison = 0;
};

// Folds the range partials of a dynamic quantize, derives the parameters (identically in every
// workgroup) and lets workgroup 0 publish them; or takes the parameters from device memory; or records
// the ones given by value.  Returns false when the element loop must not run.  `lds` holds
// 2 * kBlock / kWave floats.
__device__ __forceinline__ bool resolve_quantize_params(const DynamicRange &dyn, const hipq_qparams *params,
                                                        float *lds, float &scale, int &zp) {
    if (dyn.partials) {
        MinMax m{INFINITY, -INFINITY};
        for (int i = threadIdx.x; i < dyn.nparts; i += kBlock) {
            const float2 p = dyn.partials[i];
            m.mn = fminf(m.mn, p.x);
            m.mx = fmaxf(m.mx, p.y);
        }
        const MinMax r = block_minmax(m, lds);
        const int st = params_from_minmax(r.mn, r.mx, dyn.flavor, dyn.qmin, dyn.qmax, &scale, &zp);
        const bool bad = st != HIPQ_SUCCESS;
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            dyn.out_params->scale = (bad && dyn.poison) ? __builtin_nanf("") : scale;
            dyn.out_params->zero_point = zp;
            dyn.out_params->min_val = r.mn;
            dyn.out_params->max_val = r.mx;
            dyn.out_params->status = st;
        }
        if (bad) {  // the reference errors before quantizing
            if (!dyn.poison) return false;
            scale = INFINITY;  // x * (1/inf) and x / inf: 0 for finite x, NaN -> code 0 otherwise
            zp = 0;
        }
    } else if (params) {
        if (params->status != HIPQ_SUCCESS) return false;
        scale = params->scale;
        zp = params->zero_point;
    } else if (dyn.out_params && blockIdx.x == 0 && threadIdx.x == 0) {
        // Parameters given by value, to be recorded on the device for the kernels that follow.
        dyn.out_params->scale = scale;
        dyn.out_params->zero_point = zp;
        dyn.out_params->min_val = 0.0f;
        dyn.out_params->max_val = 0.0f;
        dyn.out_params->status = HIPQ_SUCCESS;
    }
    return true;
}

// Per-tensor quantize.  Scale and zero point come from the launch arguments, from device
// memory when `params` is non-null, or (dynamic quantization) from the range partials: then
// every workgroup folds the same few hundred partials in the same order, derives the same
// parameters, and workgroup 0 publishes them, which saves the launch of a finalize kernel.
template <typename OutT, int DIV, int RND>
__global__ __launch_bounds__(kBlock) void quantize_kernel(const float *__restrict__ x, size_t n, float scale,
                                                           int zp, const hipq_qparams *__restrict__ params,
                                                           DynamicRange dyn, float lo, float hi,
                                                           OutT *__restrict__ out) {
    __shared__ float range_lds[2 * kBlock / kWave];
    if (!resolve_quantize_params(dyn, params, range_lds, scale, zp)) return;
    const float inv = DIV ? recip_for_div(scale) : 1.0f / scale;
    const float zpf = static_cast<float>(zp);
    const int ilo = static_cast<int>(lo), ihi = static_cast<int>(hi);
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) & 15u) == 0) &&
                         ((reinterpret_cast<uintptr_t>(out) & (4 * sizeof(OutT) - 1)) == 0);
    const size_t nvec = aligned ? n / 4 : 0;
    const float4 *x4 = reinterpret_cast<const float4 *>(x);
    const size_t ntiles = (nvec + kTileVec - 1) / kTileVec;
    auto emit = [&](size_t idx, const float4 &t) {
        if constexpr (sizeof(OutT) == 4) {
            const float a = quantize_value<DIV, RND>(t.x, scale, inv, zpf, lo, hi);
            const float b = quantize_value<DIV, RND>(t.y, scale, inv, zpf, lo, hi);
            const float c = quantize_value<DIV, RND>(t.z, scale, inv, zpf, lo, hi);
            const float d = quantize_value<DIV, RND>(t.w, scale, inv, zpf, lo, hi);
            store_stream(reinterpret_cast<float4 *>(out) + idx, make_float4(a, b, c, d));
        } else {
            const int a = quantize_int<DIV, RND>(t.x, scale, inv, zpf, ilo, ihi);
            const int b = quantize_int<DIV, RND>(t.y, scale, inv, zpf, ilo, ihi);
            const int c = quantize_int<DIV, RND>(t.z, scale, inv, zpf, ilo, ihi);
            const int d = quantize_int<DIV, RND>(t.w, scale, inv, zpf, ilo, ihi);
            store_stream(reinterpret_cast<uint32_t *>(out) + idx, pack4(a, b, c, d));
        }
    };
    for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const size_t base = t * kTileVec + threadIdx.x;
        float4 v[kVecPerThread];
        if ((t + 1) * kTileVec <= nvec) {  // whole tile: unguarded loads issue back to back
#pragma unroll
            for (int i = 0; i < kVecPerThread; ++i) v[i] = load_stream(x4 + base + size_t(i) * kBlock);
#pragma unroll
            for (int i = 0; i < kVecPerThread; ++i) emit(base + size_t(i) * kBlock, v[i]);
        } else {
#pragma unroll
            for (int i = 0; i < kVecPerThread; ++i) {
                const size_t idx = base + size_t(i) * kBlock;
                if (idx < nvec) emit(idx, x4[idx]);
            }
        }
    }
    for (size_t i = nvec * 4 + size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += size_t(gridDim.x) * kBlock)
        out[i] = to_out<OutT>(quantize_value<DIV, RND>(x[i], scale, inv, zpf, lo, hi));
}

// Per-tensor quantize of a matrix [rows, cols] straight into the fragment-packed operand layout of
// the packed GEMM (32-row x 32-byte fragments of 1 KiB, lane l = row l%32, bytes 16*(l/32)..+15;
// k blocks per row block padded to a multiple of 4).  One wave per fragment: a lane reads the 16
// floats of its (row, half k block) as four 16-byte loads and writes its 16 codes as one 16-byte
// store, so a wave reads 32 whole 128-byte lines and writes 1 KiB contiguous.  Rows and columns
// past the matrix become code 0 (zero padding along K adds nothing to a dot product).
// How the packed quantizer's waves walk the matrix: wave w of the grid takes fragments w, w + waves, ...;
// lane l of a fragment owns row 32 * rb + l % 32, floats 32 * kb + 16 * (l / 32) .. +15.  Shared with the range
// pass that runs just before it in a dynamic call, so that each workgroup reads the very same lines in both
// kernels, in the same order: the second read then finds them in the memory-side cache the way they went in
// (measured: the quantizer takes 5.2 us instead of 5.9 us after a range pass in flat order).
struct FragmentWalk {
    size_t rows, cols, KB, nfrag, fstep;
    int lane, kb_shift;
    bool vec, kb_pow2, frag32;
    __device__ FragmentWalk(const float *x, size_t rows_, size_t cols_) : rows(rows_), cols(cols_) {
        KB = ((cols + 31) / 32 + 3) / 4 * 4;
        nfrag = ((rows + 31) / 32) * KB;
        lane = threadIdx.x % kWave;
        vec = (cols % 4 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15u) == 0);
        fstep = size_t(gridDim.x) * (kBlock / kWave);
        // frag -> (row block, k block) without a 64-bit division where it can be avoided: it would sit, with
        // its ~100 instructions, in front of the kernel's first load.
        kb_pow2 = (KB & (KB - 1)) == 0;
        frag32 = nfrag + fstep < (size_t(1) << 32);
        kb_shift = __builtin_ffsll(static_cast<long long>(KB)) - 1;
    }
    __device__ size_t first() const { return size_t(blockIdx.x) * (kBlock / kWave) + threadIdx.x / kWave; }
    // The lane's (row, first float) in fragment `frag`; true when its 16 floats can be read as four float4.
    __device__ bool whole(size_t frag, size_t *row, size_t *k0) const {
        size_t rb, kb;
        if (kb_pow2) {
            rb = frag >> kb_shift;
            kb = frag & (KB - 1);
        } else if (frag32) {
            rb = static_cast<uint32_t>(frag) / static_cast<uint32_t>(KB);
            kb = static_cast<uint32_t>(frag) - static_cast<uint32_t>(rb) * static_cast<uint32_t>(KB);
        } else {
            rb = frag / KB;
            kb = frag % KB;
        }
        *row = rb * 32 + lane % 32;
        *k0 = kb * 32 + 16 * (lane / 32);
        return vec && frag < nfrag && *row < rows && *k0 + 16 <= cols;
    }
};

// Range pass over a matrix in the packed quantizer's order (see FragmentWalk): one (min, max) partial per
// workgroup, the same numbers as minmax_partial_kernel's fold whatever the order (min and max are exact).
__global__ __launch_bounds__(kBlock) void minmax_fragments_kernel(const float *__restrict__ x, size_t rows, size_t cols,
                                                                   float2 *__restrict__ partials) {
    __shared__ float lds[2 * kBlock / kWave];
    const FragmentWalk fw(x, rows, cols);
    MinMax m{INFINITY, -INFINITY};
    for (size_t f = fw.first(); f < fw.nfrag; f += fw.fstep) {
        size_t row, k0;
        if (fw.whole(f, &row, &k0)) {
            float4 v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = reinterpret_cast<const float4 *>(x + row * cols + k0)[i];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                m.mn = fminf(m.mn, fminf(fminf(v[i].x, v[i].y), fminf(v[i].z, v[i].w)));
                m.mx = fmaxf(m.mx, fmaxf(fmaxf(v[i].x, v[i].y), fmaxf(v[i].z, v[i].w)));
            }
        } else if (row < rows && k0 < cols) {
            const float *p = x + row * cols + k0;
            for (int b = 0; b < 16; ++b)
                if (k0 + b < cols) acc_minmax(m, p[b]);
        }
    }
    const MinMax r = block_minmax(m, lds);
    if (threadIdx.x == 0) partials[blockIdx.x] = make_float2(r.mn, r.mx);
}

// Dynamic per-tensor quantize into the packed layout in ONE launch, for matrices of at most FPW fragments per wave
// of the grid: every wave keeps its fragments in registers (16 floats a lane each) while the grid agrees on the
// range (hipq_meeting.h), so the matrix is read once.  The two-kernel form (range partials, then a quantizer that
// folds them) measured 1.7 us more at 512 x 4096 with FPW = 1; FPW = 4 with four workgroups per compute unit
// covers 16 Mi elements.  The launch bound keeps the kernel at 128 registers, so that four workgroups fit a
// compute unit: the caller relies on the grid being resident at once.  Wave w of the grid takes fragments
// w, w + waves, ...
template <bool DIV, int RND, int FPW>
__global__ __launch_bounds__(kBlock, 4) void quantize_packed_one_launch_kernel(const float *__restrict__ x, size_t rows,
                                                                                size_t cols, hipq_qparams *out_params,
                                                                                uint32_t *words, int spin_limit,
                                                                                int8_t *__restrict__ out,
                                                                                WarmLines warm) {
    __shared__ float lds[kMeetingLdsFloats];
    const FragmentWalk fw(x, rows, cols);
    size_t f[FPW];
    bool have[FPW];
    float4 v[FPW][4];
#pragma unroll
    for (int u = 0; u < FPW; ++u) {
        f[u] = fw.first() + u * fw.fstep;
        size_t row, k0;
        have[u] = fw.whole(f[u], &row, &k0);
        if (have[u]) {
#pragma unroll
            for (int i = 0; i < 4; ++i) v[u][i] = reinterpret_cast<const float4 *>(x + row * cols + k0)[i];
        }
    }
    // Behind the fragments' loads in program order: memory operations return in order, and the number is not
    // needed before the fragments have been folded.
    const uint32_t gen = meeting_number(words);
    MinMax m{INFINITY, -INFINITY};
#pragma unroll
    for (int u = 0; u < FPW; ++u)
        if (have[u]) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                m.mn = fminf(m.mn, fminf(fminf(v[u][i].x, v[u][i].y), fminf(v[u][i].z, v[u][i].w)));
                m.mx = fmaxf(m.mx, fmaxf(fmaxf(v[u][i].x, v[u][i].y), fmaxf(v[u][i].z, v[u][i].w)));
            }
        }
    const MinMax r = block_minmax(m, lds);
    // While the grid agrees on the range the memory system is idle: touch the lines of the next kernel's operand
    // that the workgroups of this die (workgroups are dealt to the dies in turn) will read first thing, one load
    // per line, so that they wait in this die's L2.  The values are not used.
    uint32_t touched = 0;
    // Not by the waves that poll (the first of every workgroup, all of workgroup 0): loads return in order, so a
    // poll issued behind such a load would not be seen before it.
    if (warm.lines && threadIdx.x >= kWave && blockIdx.x != 0) {
        constexpr uint32_t kWarmers = kBlock - kWave;
        const uint32_t die = blockIdx.x % 8, slot = blockIdx.x / 8, sharers = (gridDim.x + 7 - die) / 8;
        const uint32_t *base = warm.base + size_t(die) * warm.die_stride_lines * 32;
        for (uint32_t i = slot * kWarmers + (threadIdx.x - kWave); i < warm.lines; i += sharers * kWarmers) {
            // i counts the lines wanted: per row block, `starts` runs of `run_lines`, `start_step_lines` apart
            const uint32_t rb = i / (warm.starts * warm.run_lines), rem = i % (warm.starts * warm.run_lines);
            const uint32_t line = rb * warm.row_block_lines + (rem / warm.run_lines) * warm.start_step_lines +
                                  rem % warm.run_lines;
            touched ^= base[size_t(line) * 32];
        }
    }
    const MeetingParams agreed = meet_on_range(words, gen, r, HIPQ_PARAMS_SYMMETRIC, -128, 127, /*poison=*/true, spin_limit,
                                               lds, out_params);
    asm volatile("" ::"v"(touched));
    const float scale = agreed.scale == agreed.scale ? agreed.scale : INFINITY;  // x * (1/inf): 0; NaN -> code 0
    const float inv = DIV ? recip_for_div(scale) : 1.0f / scale;
#pragma unroll
    for (int u = 0; u < FPW; ++u) {
        uint32_t w[4] = {0u, 0u, 0u, 0u};
        if (have[u]) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                w[i] = pack4(quantize_int<DIV, RND>(v[u][i].x, scale, inv, 0.0f, -128, 127),
                             quantize_int<DIV, RND>(v[u][i].y, scale, inv, 0.0f, -128, 127),
                             quantize_int<DIV, RND>(v[u][i].z, scale, inv, 0.0f, -128, 127),
                             quantize_int<DIV, RND>(v[u][i].w, scale, inv, 0.0f, -128, 127));
        }
        if (f[u] < fw.nfrag)
            *reinterpret_cast<uint4 *>(out + f[u] * 1024 + size_t(fw.lane) * 16) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

// The same for a flat output, any parameter flavor and int8 / uint8 codes: a workgroup keeps VPT x 1024 consecutive
// elements in registers (VPT float4 per lane; each load and each store of a wave 1 KiB contiguous).  VPT = 16 is
// 64 registers of data per lane: with four workgroups per compute unit the chip's register files hold 16 Mi
// floats, so even a 4096 x 4096 tensor is read from memory once (29.5 -> ~20 us).  The launch bound keeps the
// kernel at 128 registers, which is what lets four workgroups share a compute unit: the grid has to be resident
// at once.  n is a multiple of 4, x is 16-byte and out 4-byte aligned.  `poison`: what a bad range leaves behind,
// see meet_on_range; without it no code is written, as in the two-launch path.
template <typename OutT, bool DIV, int RND, int VPT>
__global__ __launch_bounds__(kBlock, 4) void quantize_flat_one_launch_kernel(const float *__restrict__ x, size_t n,
                                                                              int flavor, int qmin, int qmax,
                                                                              int poison, hipq_qparams *out_params,
                                                                              uint32_t *words, int spin_limit,
                                                                              OutT *__restrict__ out) {
    static_assert(sizeof(OutT) == 1, "int8 or uint8 codes");
    __shared__ float lds[kMeetingLdsFloats];
    const size_t nvec = n / 4;
    const float4 *x4 = reinterpret_cast<const float4 *>(x);
    const size_t base = size_t(blockIdx.x) * (size_t(kBlock) * VPT) + threadIdx.x;
    const bool whole = (size_t(blockIdx.x) + 1) * (size_t(kBlock) * VPT) <= nvec;
    float4 v[VPT];
    if (whole) {
#pragma unroll
        for (int i = 0; i < VPT; ++i) v[i] = load_stream(x4 + base + size_t(i) * kBlock);
    } else {
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            // past the end: a value that changes neither the minimum nor the maximum (NaN is skipped by both)
            v[i] = make_float4(NAN, NAN, NAN, NAN);
            if (base + size_t(i) * kBlock < nvec) v[i] = x4[base + size_t(i) * kBlock];
        }
    }
    const uint32_t gen = meeting_number(words);  // behind the data in program order: returned after it
    MinMax m{INFINITY, -INFINITY};
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        m.mn = fminf(m.mn, fminf(fminf(v[i].x, v[i].y), fminf(v[i].z, v[i].w)));
        m.mx = fmaxf(m.mx, fmaxf(fmaxf(v[i].x, v[i].y), fmaxf(v[i].z, v[i].w)));
    }
    const MinMax r = block_minmax(m, lds);
    const MeetingParams agreed = meet_on_range(words, gen, r, flavor, qmin, qmax, poison != 0, spin_limit, lds, out_params);
    float scale = agreed.scale;
    if (scale != scale) {
        if (!poison) return;  // the reference errors before quantizing
        scale = INFINITY;      // x * (1/inf) and x / inf: 0 for finite x, NaN -> code 0 otherwise
    }
    const float inv = DIV ? recip_for_div(scale) : 1.0f / scale;
    const float zpf = static_cast<float>(agreed.zero_point);
    uint32_t *out4 = reinterpret_cast<uint32_t *>(out);
#pragma unroll
    for (int i = 0; i < VPT; ++i)
        if (whole || base + size_t(i) * kBlock < nvec)
            store_stream(out4 + base + size_t(i) * kBlock,
                         pack4(quantize_int<DIV, RND>(v[i].x, scale, inv, zpf, qmin, qmax),
                               quantize_int<DIV, RND>(v[i].y, scale, inv, zpf, qmin, qmax),
                               quantize_int<DIV, RND>(v[i].z, scale, inv, zpf, qmin, qmax),
                               quantize_int<DIV, RND>(v[i].w, scale, inv, zpf, qmin, qmax)));
}

// The one-launch quantizers that hold 64 floats a lane need four workgroups per compute unit resident: what the
// runtime says about the widest flat form (the packed one has the same launch bound), asked once per device -
// hipq_ctx_create does, so that no later call (one under stream capture, say) is the first to ask.
bool four_wide_workgroups_fit(const hipq_ctx *ctx) {
    static int resident[16] = {0};  // workgroups per compute unit; 0 = not asked yet, -1 = the query failed
    if (ctx->device < 0 || ctx->device >= 16) return false;
    if (resident[ctx->device] == 0) {
        int a = 0, b = 0;
        const hipError_t ea = hipOccupancyMaxActiveBlocksPerMultiprocessor(
            &a, reinterpret_cast<const void *>(quantize_flat_one_launch_kernel<int8_t, false, 0, 16>), kBlock, 0);
        const hipError_t eb = hipOccupancyMaxActiveBlocksPerMultiprocessor(
            &b, reinterpret_cast<const void *>(quantize_packed_one_launch_kernel<false, 0, 4>), kBlock, 0);
        resident[ctx->device] = (ea == hipSuccess && eb == hipSuccess && a > 0 && b > 0) ? (a < b ? a : b) : -1;
    }
    return resident[ctx->device] >= 4;
}

// Launches the kernel above when the call qualifies (returns true), else leaves the two-launch path to the caller.
// The grid must be resident at once: at most four workgroups per compute unit, which the kernel's launch bound
// makes room for; checked against the runtime's own occupancy figure the first time.
template <typename OutT>
static bool launch_flat_one_launch(hipq_ctx *ctx, const float *x, size_t n, int flavor, int qmin, int qmax, int mode,
                                   bool poison, hipq_qparams *out_params, OutT *out, int32_t *rc) {
    if (ctx->gemm_variant == 6 || n % 4 != 0 || (reinterpret_cast<uintptr_t>(x) & 15u) ||
        (reinterpret_cast<uintptr_t>(out) & 3u) || (mode & ~(HIPQ_FORM_DIV | HIPQ_ROUND_HALF_EVEN)))
        return false;
    // The torsh-nn flavours do not clamp their zero point to the code range (min = 2, max = 5 gives -170), and the
    // word the meeting ends with has room for -128..895 only: they take the two launches, whatever the size.
    if (flavor > HIPQ_PARAMS_ZERO_INCLUDED) return false;
    const size_t nvec = n / 4;
    const int vpt = nvec <= resident_workgroups(ctx, false) * kBlock * 4 ? 4 : 16;
    const size_t blocks = (nvec + size_t(kBlock) * vpt - 1) / (size_t(kBlock) * vpt);
    if (blocks > resident_workgroups(ctx, vpt == 16)) return false;
    if (vpt == 16 && !four_wide_workgroups_fit(ctx)) return false;
    const bool div = (mode & HIPQ_FORM_DIV) != 0, even = (mode & HIPQ_ROUND_HALF_EVEN) != 0;
#define HIPQ_LAUNCH_Q1F(D, E, V)                                                                                       \
    hipLaunchKernelGGL((quantize_flat_one_launch_kernel<OutT, D, E, V>), dim3(static_cast<int>(blocks)), dim3(kBlock), 0, \
                       ctx->stream, x, n, flavor, qmin, qmax, poison ? 1 : 0, out_params, ctx->wait_error,             \
                       ctx->wait_spin_limit, out)
#define HIPQ_LAUNCH_Q1F_MODE(V)          \
    do {                                 \
        if (div && even)                 \
            HIPQ_LAUNCH_Q1F(true, 1, V); \
        else if (div)                    \
            HIPQ_LAUNCH_Q1F(true, 0, V); \
        else if (even)                   \
            HIPQ_LAUNCH_Q1F(false, 1, V); \
        else                             \
            HIPQ_LAUNCH_Q1F(false, 0, V); \
    } while (0)
    if (vpt == 4)
        HIPQ_LAUNCH_Q1F_MODE(4);
    else
        HIPQ_LAUNCH_Q1F_MODE(16);
#undef HIPQ_LAUNCH_Q1F_MODE
#undef HIPQ_LAUNCH_Q1F
    *rc = check_launch("quantize (flat, one launch)");
    return true;
}

template <bool DIV, int RND>
__global__ __launch_bounds__(kBlock) void quantize_packed_kernel(const float *__restrict__ x, size_t rows,
                                                                  size_t cols, float scale, int zp,
                                                                  const hipq_qparams *__restrict__ params,
                                                                  DynamicRange dyn, int8_t *__restrict__ out) {
    const FragmentWalk fw(x, rows, cols);
    const size_t nfrag = fw.nfrag, fstep = fw.fstep;
    const int lane = fw.lane;
    size_t f = fw.first();
    // The first fragment's floats are requested before the parameters are resolved (a fold of the range
    // partials and two workgroup barriers in a dynamic call): the loads do not depend on the scale, and a
    // launch of this size is bound by latency, not by bandwidth.
    auto whole = [&](size_t frag, size_t *row, size_t *k0) { return fw.whole(frag, row, k0); };
    float4 v[4];
    size_t row, k0;
    bool have = whole(f, &row, &k0);
    if (have) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = reinterpret_cast<const float4 *>(x + row * cols + k0)[i];
    }
    __shared__ float range_lds[2 * kBlock / kWave];
    if (!resolve_quantize_params(dyn, params, range_lds, scale, zp)) return;
    const float inv = DIV ? recip_for_div(scale) : 1.0f / scale;
    const float zpf = static_cast<float>(zp);
    for (; f < nfrag; f += fstep) {
        uint32_t w[4] = {0u, 0u, 0u, 0u};
        if (have) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                w[i] = pack4(quantize_int<DIV, RND>(v[i].x, scale, inv, zpf, -128, 127),
                             quantize_int<DIV, RND>(v[i].y, scale, inv, zpf, -128, 127),
                             quantize_int<DIV, RND>(v[i].z, scale, inv, zpf, -128, 127),
                             quantize_int<DIV, RND>(v[i].w, scale, inv, zpf, -128, 127));
        } else if (row < rows && k0 < cols) {
            const float *p = x + row * cols + k0;
            for (int b = 0; b < 16; ++b)
                if (k0 + b < cols)
                    w[b / 4] |= (uint32_t(quantize_int<DIV, RND>(p[b], scale, inv, zpf, -128, 127)) & 0xffu)
                                << (8 * (b % 4));
        }
        *reinterpret_cast<uint4 *>(out + f * 1024 + size_t(lane) * 16) = make_uint4(w[0], w[1], w[2], w[3]);
        have = whole(f + fstep, &row, &k0);
        if (have) {
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = reinterpret_cast<const float4 *>(x + row * cols + k0)[i];
        }
    }
}

template <typename InT>
__device__ __forceinline__ float4 unpack4(uint32_t w) {
    if constexpr (sizeof(InT) == 1 && InT(-1) < InT(0)) {
        return make_float4(static_cast<float>(static_cast<int8_t>(w & 0xff)),
                           static_cast<float>(static_cast<int8_t>((w >> 8) & 0xff)),
                           static_cast<float>(static_cast<int8_t>((w >> 16) & 0xff)),
                           static_cast<float>(static_cast<int8_t>(w >> 24)));
    } else {
        return make_float4(static_cast<float>(w & 0xff), static_cast<float>((w >> 8) & 0xff),
                           static_cast<float>((w >> 16) & 0xff), static_cast<float>(w >> 24));
    }
}

// Per-tensor dequantize: y = (q - zp) * scale.
template <typename InT>
__global__ __launch_bounds__(kBlock) void dequantize_kernel(const InT *__restrict__ q, size_t n, float scale, int zp,
                                                             const hipq_qparams *__restrict__ params,
                                                             float *__restrict__ out) {
    if (params) {
        if (params->status != HIPQ_SUCCESS) return;
        scale = params->scale;
        zp = params->zero_point;
    }
    const float zpf = static_cast<float>(zp);
    const bool aligned = ((reinterpret_cast<uintptr_t>(q) & (4 * sizeof(InT) - 1)) == 0) &&
                         ((reinterpret_cast<uintptr_t>(out) & 15u) == 0);
    const size_t nvec = aligned ? n / 4 : 0;
    const size_t ntiles = (nvec + kTileVec - 1) / kTileVec;
    // Ordinary loads, non-temporal stores (the faster pairing for a small read stream).
    auto fetch = [&](size_t idx) {
        if constexpr (sizeof(InT) == 4)
            return reinterpret_cast<const float4 *>(q)[idx];
        else
            return unpack4<InT>(reinterpret_cast<const uint32_t *>(q)[idx]);
    };
    auto emit = [&](size_t idx, const float4 &t) {
        store_stream(reinterpret_cast<float4 *>(out) + idx,
                     make_float4((t.x - zpf) * scale, (t.y - zpf) * scale, (t.z - zpf) * scale, (t.w - zpf) * scale));
    };
    for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const size_t base = t * kTileVec + threadIdx.x;
        if ((t + 1) * kTileVec <= nvec) {
            float4 v[kVecPerThread];
#pragma unroll
            for (int i = 0; i < kVecPerThread; ++i) v[i] = fetch(base + size_t(i) * kBlock);
#pragma unroll
            for (int i = 0; i < kVecPerThread; ++i) emit(base + size_t(i) * kBlock, v[i]);
        } else {
#pragma unroll
            for (int i = 0; i < kVecPerThread; ++i) {
                const size_t idx = base + size_t(i) * kBlock;
                if (idx < nvec) emit(idx, fetch(idx));
            }
        }
    }
    for (size_t i = nvec * 4 + size_t(blockIdx.x) * kBlock + threadIdx.x; i < n; i += size_t(gridDim.x) * kBlock)
        out[i] = (static_cast<float>(q[i]) - zpf) * scale;
}

// Per-row (axis 0 of [rows, cols]) dynamic quantize: TPR threads own one row,
// read it once (rows up to TPR*16 floats stay in registers), reduce min/max
// across the row with wave shuffles, derive the row's parameters and quantize
// with the division form.
//
// PACKED: the codes go straight into the fragment-packed operand layout of the packed GEMM
// ([row block of 32][k block of 32 bytes][1 KiB]; lane l of a fragment = row l % 32, bytes 16 * (l / 32) .. +15)
// instead of a dense [rows, cols] matrix, so that a per-token Linear forward needs no packing pass.  The grid
// then covers the rows up to a multiple of 32, and the padding - rows past the matrix, k past cols up to a
// multiple of 128 - is written as zeros.
// KC: float4 per lane that stay in registers between the two phases (4: rows up to 4096 floats with a workgroup
// per row; 16: up to 16384).  What does not fit is read again, one dependent round trip per 1024 floats in each phase,
// which is what a long row costs (a single row of 11008 floats: 7.3 us with KC = 4, a round trip less per 4096 floats
// with 16).
// STREAM: a large dense tensor that is read and written once goes past the caches (non-temporal accesses), as in
// the per-tensor quantizer.
template <int TPR, bool EVEN, bool PACKED = false, int KC = 4, bool STREAM = false>
__global__ __launch_bounds__(kBlock) void quantize_per_row_kernel(const float *__restrict__ x, size_t rows,
                                                                   size_t cols, size_t ld, int flavor, int qmin,
                                                                   int qmax,
                                                                   int8_t *__restrict__ out,
                                                                   float *__restrict__ out_scales,
                                                                   int32_t *__restrict__ out_zps,
                                                                   int32_t *__restrict__ out_status, int poison) {
    constexpr int kRowsPerBlock = kBlock / TPR;
    constexpr int kCache = KC;
    __shared__ float lds[2 * kBlock / kWave];
    const int sub = threadIdx.x / TPR, lane = threadIdx.x % TPR;
    const size_t row = size_t(blockIdx.x) * kRowsPerBlock + sub;
    const bool active = row < rows;
    const float *xr = x + (active ? row : 0) * ld;  // input rows are ld elements apart, output is dense
    int8_t *qr = out + (active ? row : 0) * cols;
    // PACKED: where the byte of (row, k) lives, and the padded extent of K.
    const size_t kpad = ((cols + 31) / 32 + 3) / 4 * 4 * 32;
    int8_t *prow = out + (row / 32) * (kpad / 32) * 1024 + (row % 32) * 16;  // + packed_k(k)
    auto packed_k = [](size_t k) { return (k / 32) * 1024 + ((k % 32) / 16) * 512 + (k % 16); };
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) & 15u) == 0) && (cols % 4 == 0) && (ld % 4 == 0) &&
                         ((reinterpret_cast<uintptr_t>(out) & 3u) == 0);
    const size_t nvec = aligned ? cols / 4 : 0;
    const float4 *x4 = reinterpret_cast<const float4 *>(xr);

    MinMax m{INFINITY, -INFINITY};
    float4 cache[kCache];
    if (active) {
#pragma unroll
        for (int i = 0; i < kCache; ++i) {
            const size_t v = size_t(lane) + size_t(i) * TPR;
            if (v < nvec) cache[i] = STREAM ? load_stream(x4 + v) : x4[v];
        }
#pragma unroll
        for (int i = 0; i < kCache; ++i) {
            const size_t v = size_t(lane) + size_t(i) * TPR;
            if (v < nvec) {
                acc_minmax(m, cache[i].x);
                acc_minmax(m, cache[i].y);
                acc_minmax(m, cache[i].z);
                acc_minmax(m, cache[i].w);
            }
        }
        for (size_t v = size_t(lane) + size_t(kCache) * TPR; v < nvec; v += TPR) {
            float4 t = x4[v];
            acc_minmax(m, t.x);
            acc_minmax(m, t.y);
            acc_minmax(m, t.z);
            acc_minmax(m, t.w);
        }
        for (size_t c = nvec * 4 + lane; c < cols; c += TPR) acc_minmax(m, xr[c]);
    }
    if constexpr (TPR == kWave) {
        m.mn = wave_min(m.mn);
        m.mx = wave_max(m.mx);
    } else {
        static_assert(TPR == kBlock, "a row is owned by one wave or by the whole block");
        m = block_minmax(m, lds);
    }
    if (!active) {
        if constexpr (PACKED) {  // a padding row of the last row block
            if (row < (rows + 31) / 32 * 32)
                for (size_t k = size_t(lane) * 4; k < kpad; k += size_t(TPR) * 4)
                    *reinterpret_cast<uint32_t *>(prow + packed_k(k)) = 0u;
        }
        return;
    }

    float scale;
    int zp;
    const int st = params_from_minmax(m.mn, m.mx, flavor, qmin, qmax, &scale, &zp);
    const bool bad = st != HIPQ_SUCCESS;
    if (lane == 0) {
        // poison (fused Linear forward): a row whose range is not finite gets a NaN scale and zero codes,
        // so that every output of that row is NaN instead of a product of stale scratch.
        if (out_scales) out_scales[row] = (bad && poison) ? __builtin_nanf("") : scale;
        if (out_zps) out_zps[row] = zp;
        if (bad && out_status) *out_status = st;
    }
    if (bad) {
        if (!poison) return;
        scale = INFINITY;  // x / inf: 0 for finite x, NaN -> code 0 otherwise
        zp = 0;
    }
    const float zpf = static_cast<float>(zp);
    const float inv = recip_for_div(scale);  // once per row; each element then divides with two FMAs
    uint32_t *q4 = reinterpret_cast<uint32_t *>(qr);
    // torsh-nn's per-channel weights pass each value through `as i32` before the zero point is added
    const bool int_cast = flavor >= HIPQ_PARAMS_NN_SYMMETRIC;
    auto quant1 = [&](float v) {
        return int_cast ? quantize_int_cast<EVEN>(v, scale, inv, zp, qmin, qmax)
                        : quantize_int<QFORM_DIV, EVEN>(v, scale, inv, zpf, qmin, qmax);
    };
    auto quant4 = [&](float4 t) { return pack4(quant1(t.x), quant1(t.y), quant1(t.z), quant1(t.w)); };
    auto put4 = [&](size_t v, uint32_t w) {
        if constexpr (PACKED)
            *reinterpret_cast<uint32_t *>(prow + packed_k(v * 4)) = w;
        else if constexpr (STREAM)
            store_stream(q4 + v, w);
        else
            q4[v] = w;
    };
    auto put1 = [&](size_t c, int8_t b) {
        if constexpr (PACKED)
            prow[packed_k(c)] = b;
        else
            qr[c] = b;
    };
#pragma unroll
    for (int i = 0; i < kCache; ++i) {
        const size_t v = size_t(lane) + size_t(i) * TPR;
        if (v < nvec) put4(v, quant4(cache[i]));
    }
    for (size_t v = size_t(lane) + size_t(kCache) * TPR; v < nvec; v += TPR) put4(v, quant4(x4[v]));
    for (size_t c = nvec * 4 + lane; c < cols; c += TPR) put1(c, static_cast<int8_t>(quant1(xr[c])));
    if constexpr (PACKED)
        for (size_t c = cols + lane; c < kpad; c += TPR) put1(c, int8_t(0));  // k padding: zeros add nothing
}

// quantize_per_channel_auto for a channel axis that is not the leading one, and its group-wise
// form: one block per group of `group` consecutive channels (the last group may be shorter) walks
// the group's [outer, members * inner] runs twice.
template <bool EVEN>
__global__ __launch_bounds__(kBlock) void quantize_per_channel_auto_kernel(
    const float *__restrict__ x, size_t outer, size_t channels, size_t inner, size_t group, int flavor, int qmin,
    int qmax, int8_t *__restrict__ out, float *__restrict__ out_scales, int32_t *__restrict__ out_zps,
    int32_t *__restrict__ out_status) {
    __shared__ float lds[2 * kBlock / kWave];
    const size_t g = blockIdx.x;
    const size_t c0 = g * group;
    const size_t members = (c0 + group <= channels) ? group : channels - c0;
    const size_t run = members * inner;  // contiguous elements of this group per outer index
    const size_t per = outer * run;
    MinMax m{INFINITY, -INFINITY};
    for (size_t i = threadIdx.x; i < per; i += kBlock) {
        const size_t o = i / run, r = i % run;
        acc_minmax(m, x[(o * channels + c0) * inner + r]);
    }
    m = block_minmax(m, lds);
    float scale;
    int zp;
    const int st = params_from_minmax(m.mn, m.mx, flavor, qmin, qmax, &scale, &zp);
    if (threadIdx.x == 0) {
        if (out_scales) out_scales[g] = scale;
        if (out_zps) out_zps[g] = zp;
        if (st != HIPQ_SUCCESS && out_status) *out_status = st;
    }
    if (st != HIPQ_SUCCESS) return;
    const float zpf = static_cast<float>(zp), lo = static_cast<float>(qmin), hi = static_cast<float>(qmax);
    const float inv = recip_for_div(scale);
    for (size_t i = threadIdx.x; i < per; i += kBlock) {
        const size_t o = i / run, r = i % run;
        const size_t idx = (o * channels + c0) * inner + r;
        // (torsh-nn's flavours: `as i32` before the zero point is added, as in the row kernel)
        out[idx] = static_cast<int8_t>(flavor >= HIPQ_PARAMS_NN_SYMMETRIC
                                           ? quantize_int_cast<EVEN>(x[idx], scale, inv, zp, qmin, qmax)
                                           : to_int_nan0(quantize_value<true, EVEN>(x[idx], scale, inv, zpf, lo, hi)));
    }
}

// ---- the same over many workgroups: [outer, channels, inner] read as the matrix [outer, period = channels * inner],
// whose column j belongs to group j / (inner * group).  A thread owns one column unit (V = 4 consecutive columns
// where a channel's run is a multiple of four and the base is aligned, else 1) of a tile of `col_lanes` units and walks
// a share of the rows, so its group never changes; the workgroup's other threads (256 / col_lanes row lanes) walk other
// rows of the same tile.  Two passes after the keys are set: ranges by atomic min / max on order-preserving integer
// keys, then parameters (per thread, from its group's keys) and codes.  A workgroup per group, as above, leaves most of the chip idle when the groups are few or their
// runs short.
struct ChannelColumns {
    size_t outer, period, units, span;  // rows; elements per row; column units per row (period / V); inner * group
    unsigned col_tiles, slices;         // grid = col_tiles * slices
    int col_lanes_log2;
    int key_shift;  // a group's two keys start at keys[group << key_shift]: a 64-byte line of its own while that is cheap
};

// Floats as integers of the same order (-0 below +0), for atomicMin / atomicMax; its own inverse.
__device__ __forceinline__ int32_t ordered_key(int32_t bits) { return bits ^ ((bits >> 31) & 0x7fffffff); }

__global__ void channel_keys_init_kernel(int32_t *keys, uint32_t groups, int key_shift, int32_t *status) {
    const uint32_t g = blockIdx.x * blockDim.x + threadIdx.x;
    if (g < groups) {
        keys[size_t(g) << key_shift] = ordered_key(__float_as_int(INFINITY));
        keys[(size_t(g) << key_shift) + 1] = ordered_key(__float_as_int(-INFINITY));
    }
    if (g == 0 && status) *status = 0;
}

constexpr uint32_t kNoGroup = 0xffffffffu;

// Where thread `tid` of workgroup `block` starts: its column unit, first row and row step; false if it has no column.
struct ChannelWalk {
    size_t unit, row, row_step;
    __device__ bool start(const ChannelColumns &cc, unsigned block, unsigned tid) {
        const unsigned tile = block % cc.col_tiles, slice = block / cc.col_tiles;
        const unsigned col_lane = tid & ((1u << cc.col_lanes_log2) - 1), row_lane = tid >> cc.col_lanes_log2;
        const unsigned row_lanes = kBlock >> cc.col_lanes_log2;
        unit = (size_t(tile) << cc.col_lanes_log2) + col_lane;
        row = size_t(slice) * row_lanes + row_lane;
        row_step = size_t(cc.slices) * row_lanes;
        return unit < cc.units;
    }
};

template <int V>
__global__ __launch_bounds__(kBlock) void channel_range_kernel(const float *__restrict__ x, ChannelColumns cc,
                                                                int32_t *__restrict__ keys) {
    ChannelWalk w;
    const bool live = w.start(cc, blockIdx.x, threadIdx.x);
    uint32_t g = kNoGroup;
    MinMax m{INFINITY, -INFINITY};
    if (live) {
        g = static_cast<uint32_t>(w.unit * V / cc.span);
        auto take = [&](size_t row) {
            const float *p = x + row * cc.period + w.unit * V;
            if constexpr (V == 4) {
                const float4 t = *reinterpret_cast<const float4 *>(p);
                acc_minmax(m, t.x);
                acc_minmax(m, t.y);
                acc_minmax(m, t.z);
                acc_minmax(m, t.w);
            } else {
                acc_minmax(m, *p);
            }
        };
        size_t row = w.row;
        for (; row < cc.outer && cc.outer - row > 3 * w.row_step; row += 4 * w.row_step) {
            take(row);
            take(row + w.row_step);
            take(row + 2 * w.row_step);
            take(row + 3 * w.row_step);
        }
        for (; row < cc.outer; row += w.row_step) take(row);
    }
    // Column tiles of a wave's width or less: the workgroup's waves hold the same columns lane by lane (other rows),
    // so they combine through the LDS and the first wave alone goes on.
    if (cc.col_lanes_log2 <= 6) {
        __shared__ float lds_mn[kBlock], lds_mx[kBlock];
        lds_mn[threadIdx.x] = m.mn;
        lds_mx[threadIdx.x] = m.mx;
        __syncthreads();
        if (threadIdx.x >= kWave) return;
#pragma unroll
        for (int wv = 1; wv < kBlock / kWave; ++wv) {
            m.mn = fminf(m.mn, lds_mn[wv * kWave + threadIdx.x]);
            m.mx = fmaxf(m.mx, lds_mx[wv * kWave + threadIdx.x]);
        }
    }
    // Lanes of one group combine first (a wave's columns are consecutive, so a group's lanes are neighbours; where
    // equal groups are not neighbours the extra combination is of the same group and changes nothing), then the
    // first lane of every run of equal groups adds the run to the group's keys.
    const int lane = threadIdx.x % kWave;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const float omn = __shfl_down(m.mn, d), omx = __shfl_down(m.mx, d);
        const uint32_t og = __shfl_down(g, d);
        if (lane + d < kWave && og == g) {
            m.mn = fminf(m.mn, omn);
            m.mx = fmaxf(m.mx, omx);
        }
    }
    const uint32_t before = __shfl_up(g, 1);
    const bool head = g != kNoGroup && (lane == 0 || before != g);
    auto add_to_keys = [&](uint32_t group, float mn, float mx) {
        if (!(mn <= mx)) return;  // no finite or infinite value seen
        atomicMin(&keys[size_t(group) << cc.key_shift], ordered_key(__float_as_int(mn)));
        atomicMax(&keys[(size_t(group) << cc.key_shift) + 1], ordered_key(__float_as_int(mx)));
    };
    if (cc.col_lanes_log2 > 6) {
        // Wide tiles over long runs: mostly the four waves hold one group, the same one; then one thread adds for
        // all four.  (Atomics of many workgroups on a few keys queue up behind each other.)
        constexpr int nw = kBlock / kWave;
        constexpr uint32_t kMixed = kNoGroup - 1;
        __shared__ float wave_mn[nw], wave_mx[nw];
        __shared__ uint32_t wave_group[nw];
        const unsigned long long heads = __ballot(head);
        if (lane == 0) {
            wave_group[threadIdx.x / kWave] = heads == 1ull ? g : kMixed;
            wave_mn[threadIdx.x / kWave] = m.mn;
            wave_mx[threadIdx.x / kWave] = m.mx;
        }
        __syncthreads();
        bool same = wave_group[0] < kMixed;
#pragma unroll
        for (int wv = 1; wv < nw; ++wv) same = same && wave_group[wv] == wave_group[0];
        if (same) {
            if (threadIdx.x == 0) {
                MinMax all{wave_mn[0], wave_mx[0]};
#pragma unroll
                for (int wv = 1; wv < nw; ++wv) {
                    all.mn = fminf(all.mn, wave_mn[wv]);
                    all.mx = fmaxf(all.mx, wave_mx[wv]);
                }
                add_to_keys(wave_group[0], all.mn, all.mx);
            }
            return;
        }
    }
    if (head) add_to_keys(g, m.mn, m.mx);
}

// Parameters of the thread's group from the group's keys, then the codes of the thread's column.  The thread that
// owns a group's first column on the first row writes the group's parameters and, for a range that gives none, the
// status; such a group keeps what `out` held, as with a workgroup per group.
template <bool EVEN, int V>
__global__ __launch_bounds__(kBlock) void channel_quantize_kernel(const float *__restrict__ x, ChannelColumns cc,
                                                                   const int32_t *__restrict__ keys, int flavor, int qmin,
                                                                   int qmax, int8_t *__restrict__ out,
                                                                   float *__restrict__ out_scales,
                                                                   int32_t *__restrict__ out_zps,
                                                                   int32_t *__restrict__ out_status) {
    ChannelWalk w;
    if (!w.start(cc, blockIdx.x, threadIdx.x)) return;
    const size_t g = w.unit * V / cc.span;
    const float mn = __int_as_float(ordered_key(keys[g << cc.key_shift]));
    const float mx = __int_as_float(ordered_key(keys[(g << cc.key_shift) + 1]));
    float scale;
    int zp;
    const int st = params_from_minmax(mn, mx, flavor, qmin, qmax, &scale, &zp);
    if (w.row == 0 && w.unit * V == g * cc.span) {
        if (out_scales) out_scales[g] = scale;
        if (out_zps) out_zps[g] = zp;
        if (st != HIPQ_SUCCESS && out_status) *out_status = st;
    }
    if (st != HIPQ_SUCCESS) return;
    const float inv = recip_for_div(scale), zpf = static_cast<float>(zp);
    const float lo = static_cast<float>(qmin), hi = static_cast<float>(qmax);
    // torsh-nn's per-channel weights pass each value through `as i32` before the zero point is added
    // (crates/torsh-nn/src/quantization/ops.rs:153-162): a NaN becomes the code clamp(zero point).
    const bool int_cast = flavor >= HIPQ_PARAMS_NN_SYMMETRIC;
    auto one = [&](float v) {
        return int_cast ? quantize_int_cast<EVEN>(v, scale, inv, zp, qmin, qmax)
                        : to_int_nan0(quantize_value<true, EVEN>(v, scale, inv, zpf, lo, hi));
    };
    using Vec = typename std::conditional<V == 4, float4, float>::type;
    auto load = [&](size_t row) {
        const Vec *p = reinterpret_cast<const Vec *>(x + row * cc.period + w.unit * V);
        if constexpr (V == 4)
            return load_stream(p);
        else
            return *p;
    };
    auto store = [&](size_t row, const Vec &t) {
        int8_t *q = out + row * cc.period + w.unit * V;
        if constexpr (V == 4)
            store_stream(reinterpret_cast<uint32_t *>(q), pack4(one(t.x), one(t.y), one(t.z), one(t.w)));
        else
            *q = static_cast<int8_t>(one(t));
    };
    size_t row = w.row;
    for (; row < cc.outer && cc.outer - row > 3 * w.row_step; row += 4 * w.row_step) {
        const Vec a = load(row), b = load(row + w.row_step), c = load(row + 2 * w.row_step),
                  d = load(row + 3 * w.row_step);
        store(row, a);
        store(row + w.row_step, b);
        store(row + 2 * w.row_step, c);
        store(row + 3 * w.row_step, d);
    }
    for (; row < cc.outer; row += w.row_step) store(row, load(row));
}

// Explicit per-channel parameters over a dense [outer, channels, inner] view.
template <bool DIV, bool EVEN>
__global__ __launch_bounds__(kBlock) void quantize_per_channel_kernel(const float *__restrict__ x, size_t total,
                                                                       size_t channels, size_t inner,
                                                                       const float *__restrict__ scales,
                                                                       const int32_t *__restrict__ zps,
                                                                       int8_t *__restrict__ out) {
    for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < total; i += size_t(gridDim.x) * kBlock) {
        const size_t c = (i / inner) % channels;
        const float s = scales[c];
        const float inv = DIV ? 0.0f : 1.0f / s;  // a scale per element: the division form divides directly
        const float q = quantize_value<DIV, EVEN>(x[i], s, inv, static_cast<float>(zps[c]), -128.0f, 127.0f);
        out[i] = static_cast<int8_t>(to_int_nan0(q));
    }
}

// y = scale[c] * (q - zp[c])
__global__ __launch_bounds__(kBlock) void dequantize_per_channel_kernel(const int8_t *__restrict__ q, size_t total,
                                                                         size_t channels, size_t inner,
                                                                         const float *__restrict__ scales,
                                                                         const int32_t *__restrict__ zps,
                                                                         float *__restrict__ out) {
    for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < total; i += size_t(gridDim.x) * kBlock) {
        const size_t c = (i / inner) % channels;
        out[i] = scales[c] * (static_cast<float>(q[i]) - static_cast<float>(zps[c]));
    }
}

// The channel of vector j (four consecutive elements) of a dense [outer, channels, inner] view with inner % 4 == 0,
// so that a vector never straddles channels: (j / (inner / 4)) % channels, by shifts where the counts are powers
// of two and by 32-bit divisions where the index fits.
struct ChannelOfVector {
    size_t vpc, channels;  // vectors per channel run
    int vpc_shift;
    bool vpc_pow2, ch_pow2, small;
    __device__ ChannelOfVector(size_t inner, size_t channels_, size_t nvec) : vpc(inner / 4), channels(channels_) {
        vpc_pow2 = (vpc & (vpc - 1)) == 0;
        ch_pow2 = (channels & (channels - 1)) == 0;
        vpc_shift = __builtin_ffsll(static_cast<long long>(vpc)) - 1;
        small = nvec < (size_t(1) << 32);
    }
    __device__ size_t operator()(size_t j) const {
        size_t run;
        if (vpc_pow2)
            run = j >> vpc_shift;
        else if (small)
            run = static_cast<uint32_t>(j) / static_cast<uint32_t>(vpc);
        else
            run = j / vpc;
        if (ch_pow2) return run & (channels - 1);
        if (small) return static_cast<uint32_t>(run) % static_cast<uint32_t>(channels);
        return run % channels;
    }
};

// quantize_per_channel_kernel / dequantize_per_channel_kernel on vectors of four: 16-byte loads (4-byte for codes),
// 4-byte (16-byte) stores, four in flight per lane on whole tiles, the streams that are touched once past the
// caches; the element arithmetic is the scalar kernels'.  inner % 4 == 0, x / out aligned to their vector size.
template <bool DIV, bool EVEN>
__global__ __launch_bounds__(kBlock) void quantize_per_channel_vec_kernel(const float *__restrict__ x, size_t nvec,
                                                                           size_t channels, size_t inner,
                                                                           const float *__restrict__ scales,
                                                                           const int32_t *__restrict__ zps,
                                                                           int8_t *__restrict__ out) {
    const ChannelOfVector channel_of(inner, channels, nvec);
    const float4 *x4 = reinterpret_cast<const float4 *>(x);
    uint32_t *out4 = reinterpret_cast<uint32_t *>(out);
    // How a vector's channel is found (shifts / 32-bit divisions / 64-bit divisions) is decided once, outside the
    // loop: inside it the choice would be three branches per vector between the loads and the stores.
    auto run = [&](auto shifts, auto small) {
        auto channel = [&](size_t j) -> size_t {
            if constexpr (decltype(shifts)::value)
                return (j >> channel_of.vpc_shift) & (channels - 1);
            else if constexpr (decltype(small)::value)
                return (static_cast<uint32_t>(j) / static_cast<uint32_t>(channel_of.vpc)) % static_cast<uint32_t>(channels);
            else
                return channel_of(j);
        };
        auto emit = [&](size_t j, const float4 &t) {
            const size_t c = channel(j);
            const float s = scales[c], zpf = static_cast<float>(zps[c]);
            // One reciprocal per vector: the division form then gets the correctly rounded quotient from two FMAs
            // (div_rn: the same bits as the scalar kernel's x / s), the other form multiplies by it.
            const float inv = DIV ? recip_for_div(s) : 1.0f / s;
            auto one = [&](float v) { return quantize_int<DIV ? QFORM_DIV : QFORM_MUL, EVEN>(v, s, inv, zpf, -128, 127); };
            store_stream(out4 + j, pack4(one(t.x), one(t.y), one(t.z), one(t.w)));
        };
        const size_t ntiles = (nvec + kTileVec - 1) / kTileVec;
        for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
            const size_t base = t * kTileVec + threadIdx.x;
            if ((t + 1) * kTileVec <= nvec) {
                float4 v[kVecPerThread];
#pragma unroll
                for (int i = 0; i < kVecPerThread; ++i) v[i] = load_stream(x4 + base + size_t(i) * kBlock);
                // The usual case - runs of a channel much longer than a tile - has the thread's vectors in one
                // channel: its scale, zero point and reciprocal then once, not once per vector.
                size_t c[kVecPerThread];
                bool same = true;
#pragma unroll
                for (int i = 0; i < kVecPerThread; ++i) {
                    c[i] = channel(base + size_t(i) * kBlock);
                    same = same && c[i] == c[0];
                }
                if (same) {
                    const float s = scales[c[0]], zpf = static_cast<float>(zps[c[0]]);
                    const float inv = DIV ? recip_for_div(s) : 1.0f / s;
                    auto one = [&](float f) { return quantize_int<DIV ? QFORM_DIV : QFORM_MUL, EVEN>(f, s, inv, zpf, -128, 127); };
#pragma unroll
                    for (int i = 0; i < kVecPerThread; ++i)
                        store_stream(out4 + base + size_t(i) * kBlock, pack4(one(v[i].x), one(v[i].y), one(v[i].z), one(v[i].w)));
                } else {
#pragma unroll
                    for (int i = 0; i < kVecPerThread; ++i) emit(base + size_t(i) * kBlock, v[i]);
                }
            } else {
#pragma unroll
                for (int i = 0; i < kVecPerThread; ++i) {
                    const size_t j = base + size_t(i) * kBlock;
                    if (j < nvec) emit(j, x4[j]);
                }
            }
        }
    };
    if (channel_of.vpc_pow2 && channel_of.ch_pow2)
        run(std::true_type{}, std::true_type{});
    else if (channel_of.small)
        run(std::false_type{}, std::true_type{});
    else
        run(std::false_type{}, std::false_type{});
}

__global__ __launch_bounds__(kBlock) void dequantize_per_channel_vec_kernel(const int8_t *__restrict__ q, size_t nvec,
                                                                             size_t channels, size_t inner,
                                                                             const float *__restrict__ scales,
                                                                             const int32_t *__restrict__ zps,
                                                                             float *__restrict__ out) {
    const ChannelOfVector channel_of(inner, channels, nvec);
    const uint32_t *q4 = reinterpret_cast<const uint32_t *>(q);
    float4 *out4 = reinterpret_cast<float4 *>(out);
    auto emit = [&](size_t j, uint32_t w) {
        const size_t c = channel_of(j);
        const float s = scales[c], zpf = static_cast<float>(zps[c]);
        auto one = [&](int shift) { return s * (static_cast<float>(static_cast<int8_t>(w >> shift)) - zpf); };
        store_stream(out4 + j, make_float4(one(0), one(8), one(16), one(24)));
    };
    const size_t ntiles = (nvec + kTileVec - 1) / kTileVec;
    for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const size_t base = t * kTileVec + threadIdx.x;
        if ((t + 1) * kTileVec <= nvec) {
            uint32_t w[kVecPerThread];
#pragma unroll
            for (int i = 0; i < kVecPerThread; ++i) w[i] = q4[base + size_t(i) * kBlock];
#pragma unroll
            for (int i = 0; i < kVecPerThread; ++i) emit(base + size_t(i) * kBlock, w[i]);
        } else {
#pragma unroll
            for (int i = 0; i < kVecPerThread; ++i) {
                const size_t j = base + size_t(i) * kBlock;
                if (j < nvec) emit(j, q4[j]);
            }
        }
    }
}

// int32 accumulators -> int8: v = acc*(s_a*s_w[c]) (+bias[c]); q = clamp(round(v/s_out)+zp_out).
template <bool EVEN>
__global__ __launch_bounds__(kBlock) void requantize_kernel(const int32_t *__restrict__ acc, size_t rows, size_t cols,
                                                             const float *__restrict__ sa, int sa_per_row,
                                                             const float *__restrict__ sw,
                                                             const float *__restrict__ bias, float s_out, int zp_out,
                                                             int8_t *__restrict__ out) {
    const size_t total = rows * cols;
    const float zpf = static_cast<float>(zp_out);
    const float inv_out = recip_for_div(s_out);
    for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < total; i += size_t(gridDim.x) * kBlock) {
        const size_t r = i / cols, c = i % cols;
        const float s = (sa_per_row ? sa[r] : sa[0]) * sw[c];
        float v = static_cast<float>(acc[i]) * s;
        if (bias) v = v + bias[c];
        const float q = clamp_keep_nan(round_mode<EVEN>(div_rn(v, s_out, inv_out)) + zpf, -128.0f, 127.0f);
        out[i] = static_cast<int8_t>(to_int_nan0(q));
    }
}

// The same, four consecutive accumulators of a row per lane and instruction: one 16-byte load of accumulators, the
// four weight scales and biases as 16-byte loads (they stay in the caches), one 4-byte store of codes, four such
// groups in flight per lane on whole tiles; the streams that are touched once bypass the caches.  The element
// arithmetic is the scalar kernel's.  cols % 4 == 0; acc, sw, bias 16-byte and out 4-byte aligned.  A vector's
// row and column come from a shift when cols / 4 is a power of two, else from one 32- or 64-bit division per
// four elements.
// FIXED_COLUMNS: the grid is sized so that a thread meets the same four column vectors in every tile it takes
// ((gridDim.x * kTileVec) % (cols / 4) == 0, see requantize_grid): their weight scales and biases are loaded once,
// ahead of the accumulators, instead of with every vector.
template <bool EVEN, bool FIXED_COLUMNS>
__global__ __launch_bounds__(kBlock) void requantize_vec_kernel(const int32_t *__restrict__ acc, size_t rows, size_t cols,
                                                                 const float *__restrict__ sa, int sa_per_row,
                                                                 const float *__restrict__ sw,
                                                                 const float *__restrict__ bias, float s_out, int zp_out,
                                                                 int8_t *__restrict__ out) {
    const size_t vpr = cols / 4, nvec = rows * vpr;  // vectors per row, in all
    const float zpf = static_cast<float>(zp_out);
    const float inv_out = recip_for_div(s_out);
    const bool pow2 = (vpr & (vpr - 1)) == 0, small = nvec < (size_t(1) << 32);
    const int shift = __builtin_ffsll(static_cast<long long>(vpr)) - 1;
    const float sa0 = sa[0];
    const int4 *acc4 = reinterpret_cast<const int4 *>(acc);
    const float4 *sw4 = reinterpret_cast<const float4 *>(sw);
    const float4 *bias4 = reinterpret_cast<const float4 *>(bias);
    uint32_t *out4 = reinterpret_cast<uint32_t *>(out);
    // The uniform choices (how a vector's row and column are found, bias or none, one activation scale or one per
    // row) are made once, outside the loop: inside it they would be branches between the loads and the stores.
    auto run = [&](auto shifts, auto small32, auto with_bias, auto per_row) {
        auto row_col = [&](size_t j, size_t *r, size_t *cv) {
            if constexpr (decltype(shifts)::value) {
                *r = j >> shift;
                *cv = j & (vpr - 1);
            } else if constexpr (decltype(small32)::value) {
                *r = static_cast<uint32_t>(j) / static_cast<uint32_t>(vpr);
                *cv = static_cast<uint32_t>(j) - static_cast<uint32_t>(*r) * static_cast<uint32_t>(vpr);
            } else {
                *r = j / vpr;
                *cv = j % vpr;
            }
        };
        auto one = [&](int a, float s_w, float b, float s_a) {
            float v = static_cast<float>(a) * (s_a * s_w);
            if constexpr (decltype(with_bias)::value) v = v + b;
            // saturating conversion (NaN -> 0), then the clamp on integers: the scalar kernel's clamp-then-convert
            return clamp_to_int(round_mode<EVEN>(div_rn(v, s_out, inv_out)) + zpf, -128, 127);
        };
        const float4 none = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        auto emit4 = [&](size_t j, size_t r, const int4 &a, const float4 &w, const float4 &b) {
            float s_a = sa0;
            if constexpr (decltype(per_row)::value) s_a = sa[r];
            store_stream(out4 + j, pack4(one(a.x, w.x, b.x, s_a), one(a.y, w.y, b.y, s_a), one(a.z, w.z, b.z, s_a),
                                         one(a.w, w.w, b.w, s_a)));
        };
        auto emit = [&](size_t j, const int4 &a) {
            size_t r, cv;
            row_col(j, &r, &cv);
            emit4(j, r, a, sw4[cv], decltype(with_bias)::value ? bias4[cv] : none);
        };
        auto load_acc = [&](size_t j) {
            typedef int vi4 __attribute__((ext_vector_type(4)));
            const vi4 t = __builtin_nontemporal_load(reinterpret_cast<const vi4 *>(acc4 + j));
            return make_int4(t.x, t.y, t.z, t.w);
        };
        const size_t ntiles = (nvec + kTileVec - 1) / kTileVec;
        float4 w_fixed[kVecPerThread], b_fixed[kVecPerThread];
        if constexpr (FIXED_COLUMNS) {
#pragma unroll
            for (int i = 0; i < kVecPerThread; ++i) {
                size_t r, cv;  // (a first vector past nvec still has a valid column)
                row_col(size_t(blockIdx.x) * kTileVec + threadIdx.x + size_t(i) * kBlock, &r, &cv);
                w_fixed[i] = sw4[cv];
                b_fixed[i] = decltype(with_bias)::value ? bias4[cv] : none;
                if constexpr (!decltype(per_row)::value) {  // s_a * s_w once (the same product, rounded the same)
                    w_fixed[i].x = sa0 * w_fixed[i].x;
                    w_fixed[i].y = sa0 * w_fixed[i].y;
                    w_fixed[i].z = sa0 * w_fixed[i].z;
                    w_fixed[i].w = sa0 * w_fixed[i].w;
                }
            }
        }
        auto one_combined = [&](int a, float sc, float b) {
            float v = static_cast<float>(a) * sc;
            if constexpr (decltype(with_bias)::value) v = v + b;
            return clamp_to_int(round_mode<EVEN>(div_rn(v, s_out, inv_out)) + zpf, -128, 127);
        };
        for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
            const size_t base = t * kTileVec + threadIdx.x;
            if ((t + 1) * kTileVec <= nvec) {  // whole tile: unguarded loads issue back to back
                int4 a[kVecPerThread];
#pragma unroll
                for (int i = 0; i < kVecPerThread; ++i) a[i] = load_acc(base + size_t(i) * kBlock);
#pragma unroll
                for (int i = 0; i < kVecPerThread; ++i) {
                    const size_t j = base + size_t(i) * kBlock;
                    if constexpr (FIXED_COLUMNS && !decltype(per_row)::value) {
                        const float4 &w = w_fixed[i], &b = b_fixed[i];
                        store_stream(out4 + j, pack4(one_combined(a[i].x, w.x, b.x), one_combined(a[i].y, w.y, b.y),
                                                     one_combined(a[i].z, w.z, b.z), one_combined(a[i].w, w.w, b.w)));
                    } else if constexpr (FIXED_COLUMNS) {
                        size_t r, cv;
                        row_col(j, &r, &cv);
                        emit4(j, r, a[i], w_fixed[i], b_fixed[i]);
                    } else {
                        emit(j, a[i]);
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < kVecPerThread; ++i) {
                    const size_t j = base + size_t(i) * kBlock;
                    if (j < nvec) emit(j, acc4[j]);
                }
            }
        }
    };
    auto with_index = [&](auto with_bias, auto per_row) {
        if (pow2)
            run(std::true_type{}, std::true_type{}, with_bias, per_row);
        else if (small)
            run(std::false_type{}, std::true_type{}, with_bias, per_row);
        else
            run(std::false_type{}, std::false_type{}, with_bias, per_row);
    };
    if (bias && sa_per_row)
        with_index(std::true_type{}, std::true_type{});
    else if (bias)
        with_index(std::true_type{}, std::false_type{});
    else if (sa_per_row)
        with_index(std::false_type{}, std::true_type{});
    else
        with_index(std::false_type{}, std::false_type{});
}

static inline int grid_for_tiles(hipq_ctx *ctx, size_t n) {
    size_t tiles = (n / 4 + kTileVec - 1) / kTileVec;
    if (tiles == 0) tiles = 1;
    const size_t cap = size_t(ctx->num_cus) * 16;
    return static_cast<int>(tiles < cap ? tiles : cap);
}

// The range reduction wants few partials: its second stage is one block whose time grows
// with their count (16 Mi floats: 17.1 us for both stages with 4096 partials, 13.6 us with 512,
// the first stage taking 11.4 us either way).
static inline int grid_for_minmax(hipq_ctx *ctx, size_t n) {
    size_t tiles = (n / 4 + kTileVec - 1) / kTileVec;
    if (tiles == 0) tiles = 1;
    const size_t cap = size_t(ctx->num_cus) * 2;
    return static_cast<int>(tiles < cap ? tiles : cap);
}

static inline int grid_for_elems(hipq_ctx *ctx, size_t n) {
    size_t blocks = (n + kBlock - 1) / kBlock;
    if (blocks == 0) blocks = 1;
    const size_t cap = size_t(ctx->num_cus) * 16;
    return static_cast<int>(blocks < cap ? blocks : cap);
}

// Launches the two-stage range reduction.
static int32_t launch_minmax(hipq_ctx *ctx, const float *x, size_t n, float *out_minmax, float *out_absmax,
                             hipq_qparams *out_params, int flavor, int qmin, int qmax) {
    const int grid = grid_for_minmax(ctx, n);
    if (ctx->gemm_variant != 6 && size_t(grid) <= kCtxSlots) {
        hipLaunchKernelGGL(minmax_one_launch_kernel, dim3(grid), dim3(kBlock), 0, ctx->stream, x, n, ctx->wait_error,
                           ctx->wait_spin_limit, RangeOutputs{out_minmax, out_absmax, out_params, flavor, qmin, qmax});
        return check_launch("minmax (one launch)");
    }
    void *s = nullptr;
    int32_t rc = scratch(ctx, kScratchHeader + size_t(grid) * sizeof(float2), &s);
    if (rc != HIPQ_SUCCESS) return rc;
    float2 *partials = reinterpret_cast<float2 *>(static_cast<char *>(s) + kScratchHeader);
    hipLaunchKernelGGL(minmax_partial_kernel, dim3(grid), dim3(kBlock), 0, ctx->stream, x, n, partials);
    hipLaunchKernelGGL(minmax_final_kernel, dim3(1), dim3(kBlock), 0, ctx->stream, partials, grid, out_minmax,
                       out_absmax, out_params, flavor, qmin, qmax);
    return check_launch("minmax");
}

// First stage only; the quantize kernel that follows folds the partials itself.
static int32_t launch_minmax_partials(hipq_ctx *ctx, const float *x, size_t n, DynamicRange *dyn,
                                      float2 *partials = nullptr, size_t partials_cap = 0) {
    int grid = grid_for_minmax(ctx, n);
    if (partials) {
        // Caller-provided room for the partials (the entry point that must not allocate).
        if (size_t(grid) > partials_cap) grid = static_cast<int>(partials_cap);
    } else {
        void *s = nullptr;
        int32_t rc = scratch(ctx, kScratchHeader + size_t(grid) * sizeof(float2), &s);
        if (rc != HIPQ_SUCCESS) return rc;
        partials = reinterpret_cast<float2 *>(static_cast<char *>(s) + kScratchHeader);
    }
    hipLaunchKernelGGL(minmax_partial_kernel, dim3(grid), dim3(kBlock), 0, ctx->stream, x, n, partials);
    dyn->partials = partials;
    dyn->nparts = grid;
    return check_launch("minmax");
}

template <typename OutT>
static int32_t launch_quantize(hipq_ctx *ctx, const float *x, size_t n, float scale, int zp,
                               const hipq_qparams *params, int mode, float lo, float hi, OutT *out,
                               DynamicRange dyn = DynamicRange{nullptr, 0, 0, 0, 0, nullptr}) {
    const int grid = grid_for_tiles(ctx, n);
    const bool div = (mode & HIPQ_FORM_DIV) != 0, even = (mode & HIPQ_ROUND_HALF_EVEN) != 0;
    const bool half_up = (mode & HIPQ_ROUND_FLOOR_HALF_UP) != 0;
#define HIPQ_LAUNCH_Q(D, E)                                                                                   \
    hipLaunchKernelGGL((quantize_kernel<OutT, D, E>), dim3(grid), dim3(kBlock), 0, ctx->stream, x, n, scale, zp, \
                       params, dyn, lo, hi, out)
    if (mode & HIPQ_FORM_ZP_BEFORE_ROUND) {  // integer outputs only (checked by the entry points)
        if constexpr (sizeof(OutT) == 1) {
            if (even)
                HIPQ_LAUNCH_Q(QFORM_DIV_ZP_FIRST, 1);
            else
                HIPQ_LAUNCH_Q(QFORM_DIV_ZP_FIRST, 0);
        }
    } else if (mode & HIPQ_FORM_INT_CAST) {  // carrier output only
        if constexpr (sizeof(OutT) == 4) {
            if (even)
                HIPQ_LAUNCH_Q(QFORM_DIV_INT_CAST, 1);
            else
                HIPQ_LAUNCH_Q(QFORM_DIV_INT_CAST, 0);
        }
    } else if (half_up && div)
        HIPQ_LAUNCH_Q(1, 2);
    else if (half_up)
        HIPQ_LAUNCH_Q(0, 2);
    else if (div && even)
        HIPQ_LAUNCH_Q(1, 1);
    else if (div)
        HIPQ_LAUNCH_Q(1, 0);
    else if (even)
        HIPQ_LAUNCH_Q(0, 1);
    else
        HIPQ_LAUNCH_Q(0, 0);
#undef HIPQ_LAUNCH_Q
    return check_launch("quantize");
}

static int32_t check_mode(const char *fn, int32_t mode) {
    if (mode & ~(HIPQ_ROUND_HALF_EVEN | HIPQ_FORM_DIV)) return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown mode bits 0x%x", fn, mode);
    return HIPQ_SUCCESS;
}

static int32_t check_scale(const char *fn, float scale) {
    // `scale <= 0.0` in the reference: NaN passes that test there too.
    if (scale <= 0.0f) return fail(HIPQ_INVALID_ARGUMENT, "%s: Scale must be positive", fn);
    return HIPQ_SUCCESS;
}

template <typename InT>
static int32_t dequant_common(const char *fn, hipq_ctx *ctx, const InT *q, size_t n, float scale, int32_t zp,
                              const hipq_qparams *params, float *out) {
    if (!params) {
        int32_t rc = check_scale(fn, scale);
        if (rc) return rc;
    }
    if (n == 0) return HIPQ_SUCCESS;
    if (!q || !out) return fail(HIPQ_INVALID_ARGUMENT, "%s: null pointer", fn);
    const int grid = grid_for_tiles(ctx, n);
    hipLaunchKernelGGL((dequantize_kernel<InT>), dim3(grid), dim3(kBlock), 0, ctx->stream, q, n, scale, zp, params,
                       out);
    return check_launch(fn);
}

static int32_t check_row_flavor(const char *fn, int32_t flavor) {
    if (flavor != HIPQ_PARAMS_SYMMETRIC && flavor != HIPQ_PARAMS_AFFINE)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: Unsupported scheme for per-channel quantization (flavor %d)", fn, flavor);
    return HIPQ_SUCCESS;
}

}  // namespace hipq

using namespace hipq;

extern "C" {

int32_t hipq_minmax_f32(hipq_ctx *ctx, const float *x, size_t n, float *out_minmax) {
    HIPQ_ENTER(ctx);
    if (n == 0) return fail(HIPQ_INVALID_ARGUMENT, "hipq_minmax_f32: Cannot find min/max of empty array");
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out_minmax);
    return launch_minmax(ctx, x, n, out_minmax, nullptr, nullptr, 0, 0, 0);
}

int32_t hipq_absmax_f32(hipq_ctx *ctx, const float *x, size_t n, float *out_absmax) {
    HIPQ_ENTER(ctx);
    if (n == 0) return fail(HIPQ_INVALID_ARGUMENT, "hipq_absmax_f32: Cannot find min/max of empty array");
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out_absmax);
    return launch_minmax(ctx, x, n, nullptr, out_absmax, nullptr, 0, 0, 0);
}

int32_t hipq_qparams_from_minmax(hipq_ctx *ctx, const float *minmax, int32_t flavor, int32_t qmin, int32_t qmax,
                                 hipq_qparams *out_params) {
    HIPQ_ENTER(ctx);
    HIPQ_REQUIRE_PTR(minmax);
    HIPQ_REQUIRE_PTR(out_params);
    if (flavor < HIPQ_PARAMS_SYMMETRIC || flavor > HIPQ_PARAMS_NN_ASYMMETRIC)
        return fail(HIPQ_INVALID_ARGUMENT, "hipq_qparams_from_minmax: unknown flavor %d", flavor);
    if (qmin >= qmax) return fail(HIPQ_INVALID_ARGUMENT, "hipq_qparams_from_minmax: qmin %d >= qmax %d", qmin, qmax);
    hipLaunchKernelGGL(qparams_kernel, dim3(1), dim3(64), 0, ctx->stream, minmax, flavor, qmin, qmax, out_params);
    return check_launch("qparams");
}

int32_t hipq_quantize_per_tensor_f32_i8(hipq_ctx *ctx, const float *x, size_t n, float scale, int32_t zero_point,
                                        int32_t mode, int8_t *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_scale(__func__, scale);
    if (rc) return rc;
    // this entry point alone also knows the floor(v + 0.5) rounding of quantize_mobile_optimized; the integer
    // outputs know the zero-point-first form of the scalar quantized types
    if ((rc = check_mode(__func__, mode & ~(HIPQ_ROUND_FLOOR_HALF_UP | HIPQ_FORM_ZP_BEFORE_ROUND)))) return rc;
    if ((mode & HIPQ_ROUND_FLOOR_HALF_UP) && (mode & (HIPQ_ROUND_HALF_EVEN | HIPQ_FORM_ZP_BEFORE_ROUND)))
        return fail(HIPQ_INVALID_ARGUMENT, "%s: two rounding modes in mode 0x%x", __func__, mode);
    if (n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out);
    return launch_quantize<int8_t>(ctx, x, n, scale, zero_point, nullptr, mode, -128.0f, 127.0f, out);
}

int32_t hipq_quantize_static_per_tensor_f32_i8(hipq_ctx *ctx, const float *x, size_t n, float scale,
                                               int32_t zero_point, int32_t mode, int8_t *out,
                                               hipq_qparams *out_params) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_scale(__func__, scale);
    if (rc) return rc;
    if ((rc = check_mode(__func__, mode))) return rc;
    HIPQ_REQUIRE_PTR(out_params);
    if (n == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: Cannot quantize empty tensor", __func__);
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out);
    return launch_quantize<int8_t>(ctx, x, n, scale, zero_point, nullptr, mode, -128.0f, 127.0f, out,
                                   DynamicRange{nullptr, 0, 0, 0, 0, out_params});
}

int32_t hipq_quantize_per_tensor_f32_u8(hipq_ctx *ctx, const float *x, size_t n, float scale, int32_t zero_point,
                                        int32_t mode, uint8_t *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_scale(__func__, scale);
    if (rc) return rc;
    if ((rc = check_mode(__func__, mode & ~HIPQ_FORM_ZP_BEFORE_ROUND))) return rc;
    if (n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out);
    return launch_quantize<uint8_t>(ctx, x, n, scale, zero_point, nullptr, mode, 0.0f, 255.0f, out);
}

int32_t hipq_quantize_per_tensor_f32_carrier(hipq_ctx *ctx, const float *x, size_t n, float scale,
                                             int32_t zero_point, int32_t mode, int32_t qmin, int32_t qmax,
                                             float *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_scale(__func__, scale);
    if (rc) return rc;
    if ((rc = check_mode(__func__, mode & ~HIPQ_FORM_INT_CAST))) return rc;
    if (qmin > qmax) return fail(HIPQ_INVALID_ARGUMENT, "%s: qmin %d > qmax %d", __func__, qmin, qmax);
    if (n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out);
    return launch_quantize<float>(ctx, x, n, scale, zero_point, nullptr, mode, static_cast<float>(qmin),
                                  static_cast<float>(qmax), out);
}

int32_t hipq_quantize_with_params_f32_i8(hipq_ctx *ctx, const float *x, size_t n, const hipq_qparams *params,
                                         int32_t mode, int8_t *out) {
    HIPQ_ENTER(ctx);
    HIPQ_REQUIRE_PTR(params);
    int32_t rc = check_mode(__func__, mode);
    if (rc) return rc;
    if (n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out);
    return launch_quantize<int8_t>(ctx, x, n, 1.0f, 0, params, mode, -128.0f, 127.0f, out);
}

int32_t hipq_quantize_with_params_f32_u8(hipq_ctx *ctx, const float *x, size_t n, const hipq_qparams *params,
                                         int32_t mode, uint8_t *out) {
    HIPQ_ENTER(ctx);
    HIPQ_REQUIRE_PTR(params);
    int32_t rc = check_mode(__func__, mode);
    if (rc) return rc;
    if (n == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out);
    return launch_quantize<uint8_t>(ctx, x, n, 1.0f, 0, params, mode, 0.0f, 255.0f, out);
}

int32_t hipq_quantize_dynamic_per_tensor_f32(hipq_ctx *ctx, const float *x, size_t n, int32_t flavor, int32_t dtype,
                                             int32_t mode, void *out, hipq_qparams *out_params) {
    return hipq::quantize_dynamic_per_tensor(ctx, x, n, flavor, dtype, mode, out, out_params, nullptr, 0);
}

}  // extern "C"

int32_t hipq::quantize_dynamic_per_tensor(hipq_ctx *ctx, const float *x, size_t n, int32_t flavor, int32_t dtype,
                                          int32_t mode, void *out, hipq_qparams *out_params, void *partials,
                                          size_t partials_cap) {
    const char *fn = "hipq_quantize_dynamic_per_tensor_f32";
    HIPQ_ENTER(ctx);
    if (n == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: Cannot quantize empty tensor", fn);
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out);
    HIPQ_REQUIRE_PTR(out_params);
    int32_t rc = check_mode(fn, mode);
    if (rc) return rc;
    if (flavor < HIPQ_PARAMS_SYMMETRIC || flavor > HIPQ_PARAMS_NN_ASYMMETRIC)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown flavor %d", fn, flavor);
    if (dtype != HIPQ_DTYPE_I8 && dtype != HIPQ_DTYPE_U8)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown dtype %d", fn, dtype);
    const int qmin = dtype == HIPQ_DTYPE_I8 ? -128 : 0, qmax = dtype == HIPQ_DTYPE_I8 ? 127 : 255;
    if (dtype == HIPQ_DTYPE_I8) {
        if (launch_flat_one_launch<int8_t>(ctx, x, n, flavor, qmin, qmax, mode, false, out_params,
                                           static_cast<int8_t *>(out), &rc))
            return rc;
    } else if (launch_flat_one_launch<uint8_t>(ctx, x, n, flavor, qmin, qmax, mode, false, out_params,
                                               static_cast<uint8_t *>(out), &rc)) {
        return rc;
    }
    DynamicRange dyn{nullptr, 0, flavor, qmin, qmax, out_params};
    rc = launch_minmax_partials(ctx, x, n, &dyn, static_cast<float2 *>(partials), partials_cap / sizeof(float2));
    if (rc) return rc;
    if (dtype == HIPQ_DTYPE_I8)
        return launch_quantize<int8_t>(ctx, x, n, 1.0f, 0, nullptr, mode, -128.0f, 127.0f,
                                       static_cast<int8_t *>(out), dyn);
    return launch_quantize<uint8_t>(ctx, x, n, 1.0f, 0, nullptr, mode, 0.0f, 255.0f, static_cast<uint8_t *>(out),
                                    dyn);
}

extern "C" {

int32_t hipq_dequantize_i8_f32(hipq_ctx *ctx, const int8_t *q, size_t n, float scale, int32_t zero_point, float *out) {
    HIPQ_ENTER(ctx);
    return dequant_common<int8_t>(__func__, ctx, q, n, scale, zero_point, nullptr, out);
}

int32_t hipq_dequantize_u8_f32(hipq_ctx *ctx, const uint8_t *q, size_t n, float scale, int32_t zero_point,
                               float *out) {
    HIPQ_ENTER(ctx);
    return dequant_common<uint8_t>(__func__, ctx, q, n, scale, zero_point, nullptr, out);
}

int32_t hipq_dequantize_carrier_f32(hipq_ctx *ctx, const float *q, size_t n, float scale, int32_t zero_point,
                                    float *out) {
    HIPQ_ENTER(ctx);
    return dequant_common<float>(__func__, ctx, q, n, scale, zero_point, nullptr, out);
}

int32_t hipq_dequantize_with_params_i8_f32(hipq_ctx *ctx, const int8_t *q, size_t n, const hipq_qparams *params,
                                           float *out) {
    HIPQ_ENTER(ctx);
    HIPQ_REQUIRE_PTR(params);
    return dequant_common<int8_t>(__func__, ctx, q, n, 1.0f, 0, params, out);
}

}  // extern "C"

// Per-row quantize over rows `ld` apart, integer range [qmin, qmax]; `any_flavor` admits every
// HIPQ_PARAMS_* formula (the reference's per-channel function knows two).
static int32_t quantize_rows(const char *fn, hipq_ctx *ctx, const float *x, size_t rows, size_t cols, size_t ld,
                             int32_t flavor, bool any_flavor, int32_t qmin, int32_t qmax, int32_t mode, int8_t *out,
                             float *out_scales, int32_t *out_zero_points, int32_t *out_status, int poison = 0,
                             bool packed = false) {
    int32_t rc = any_flavor ? HIPQ_SUCCESS : check_row_flavor(fn, flavor);
    if (rc) return rc;
    if ((rc = check_mode(fn, mode))) return rc;
    if (out_status) hipLaunchKernelGGL(fill_i32_kernel, dim3(1), dim3(64), 0, ctx->stream, out_status, 0, size_t(1));
    if (rows == 0) return check_launch(fn);
    if (cols == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: rows of zero length have no range", fn);
    if (ld < cols) return fail(HIPQ_INVALID_ARGUMENT, "%s: row stride %zu smaller than the row length %zu", fn, ld, cols);
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out);
    const bool even = (mode & HIPQ_ROUND_HALF_EVEN) != 0;
    if (rows >> 31) return fail(HIPQ_INVALID_ARGUMENT, "%s: too many rows", fn);
    // Packed output: the grid also covers the padding rows of the last row block (they are written as zeros).
    const size_t grid_rows = packed ? (rows + 31) / 32 * 32 : rows;
    // A large dense tensor is read and written once: past the caches, as the per-tensor quantizer does it
    // (4096 x 4096: 19.9 -> 17.3 us).  Packed output is an operand of the GEMM that follows: it stays cached.
    const bool stream = !packed && rows * cols >= (size_t(1) << 22);
#define HIPQ_LAUNCH_ROWS(TPR, E, P, G)                                                                               \
    hipLaunchKernelGGL((quantize_per_row_kernel<TPR, E, P>), dim3(G), dim3(kBlock), 0, ctx->stream, x, rows, cols, ld, \
                       flavor, qmin, qmax, out, out_scales, out_zero_points, out_status, poison)
    if (cols > 4096 && ld % 4 == 0) {
        // long rows: four times the registers, so that up to 16384 floats are read once and all requested up front
        const int grid = static_cast<int>(grid_rows);
#define HIPQ_LAUNCH_LONG_ROWS(E, P)                                                                                   \
    hipLaunchKernelGGL((quantize_per_row_kernel<kBlock, E, P, 16>), dim3(grid), dim3(kBlock), 0, ctx->stream, x, rows,   \
                       cols, ld, flavor, qmin, qmax, out, out_scales, out_zero_points, out_status, poison)
        if (stream && even)
            hipLaunchKernelGGL((quantize_per_row_kernel<kBlock, true, false, 16, true>), dim3(grid), dim3(kBlock), 0,
                               ctx->stream, x, rows, cols, ld, flavor, qmin, qmax, out, out_scales, out_zero_points,
                               out_status, poison);
        else if (stream)
            hipLaunchKernelGGL((quantize_per_row_kernel<kBlock, false, false, 16, true>), dim3(grid), dim3(kBlock), 0,
                               ctx->stream, x, rows, cols, ld, flavor, qmin, qmax, out, out_scales, out_zero_points,
                               out_status, poison);
        else if (packed && even)
            HIPQ_LAUNCH_LONG_ROWS(true, true);
        else if (packed)
            HIPQ_LAUNCH_LONG_ROWS(false, true);
        else if (even)
            HIPQ_LAUNCH_LONG_ROWS(true, false);
        else
            HIPQ_LAUNCH_LONG_ROWS(false, false);
#undef HIPQ_LAUNCH_LONG_ROWS
    } else if (cols > 1024 && stream) {
        const int grid = static_cast<int>(grid_rows);
        if (even)
            hipLaunchKernelGGL((quantize_per_row_kernel<kBlock, true, false, 4, true>), dim3(grid), dim3(kBlock), 0,
                               ctx->stream, x, rows, cols, ld, flavor, qmin, qmax, out, out_scales, out_zero_points,
                               out_status, poison);
        else
            hipLaunchKernelGGL((quantize_per_row_kernel<kBlock, false, false, 4, true>), dim3(grid), dim3(kBlock), 0,
                               ctx->stream, x, rows, cols, ld, flavor, qmin, qmax, out, out_scales, out_zero_points,
                               out_status, poison);
    } else if (cols > 1024) {
        const int grid = static_cast<int>(grid_rows);
        if (packed) {
            if (even)
                HIPQ_LAUNCH_ROWS(kBlock, true, true, grid);
            else
                HIPQ_LAUNCH_ROWS(kBlock, false, true, grid);
        } else if (even) {
            HIPQ_LAUNCH_ROWS(kBlock, true, false, grid);
        } else {
            HIPQ_LAUNCH_ROWS(kBlock, false, false, grid);
        }
    } else if (stream) {
        const int grid = static_cast<int>((grid_rows + 3) / 4);
        if (even)
            hipLaunchKernelGGL((quantize_per_row_kernel<kWave, true, false, 4, true>), dim3(grid), dim3(kBlock), 0,
                               ctx->stream, x, rows, cols, ld, flavor, qmin, qmax, out, out_scales, out_zero_points,
                               out_status, poison);
        else
            hipLaunchKernelGGL((quantize_per_row_kernel<kWave, false, false, 4, true>), dim3(grid), dim3(kBlock), 0,
                               ctx->stream, x, rows, cols, ld, flavor, qmin, qmax, out, out_scales, out_zero_points,
                               out_status, poison);
    } else {
        const int grid = static_cast<int>((grid_rows + 3) / 4);
        if (packed) {
            if (even)
                HIPQ_LAUNCH_ROWS(kWave, true, true, grid);
            else
                HIPQ_LAUNCH_ROWS(kWave, false, true, grid);
        } else if (even) {
            HIPQ_LAUNCH_ROWS(kWave, true, false, grid);
        } else {
            HIPQ_LAUNCH_ROWS(kWave, false, false, grid);
        }
    }
#undef HIPQ_LAUNCH_ROWS
    return check_launch(fn);
}

// Below this many elements the per-group workgroups' one launch beats the three of the form spread over columns.
constexpr size_t kSpreadMinElems = size_t(1) << 18;

// quantize_per_channel_auto over a dense [outer, channels, inner] view with groups of `group`
// consecutive channels sharing their parameters (1 = per channel), integer range [qmin, qmax].
static int32_t quantize_channels(const char *fn, hipq_ctx *ctx, const float *x, size_t outer, size_t channels,
                                 size_t inner, size_t group, int32_t flavor, bool any_flavor, int32_t qmin,
                                 int32_t qmax, int32_t mode, int8_t *out, float *out_scales, int32_t *out_zero_points,
                                 int32_t *out_status) {
    if (group == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: Group size must be greater than 0", fn);
    if (outer == 1 && channels % group == 0)  // every group is one contiguous row
        return quantize_rows(fn, ctx, x, channels / group, group * inner, group * inner, flavor, any_flavor, qmin, qmax,
                             mode, out, out_scales, out_zero_points, out_status);
    int32_t rc = any_flavor ? HIPQ_SUCCESS : check_row_flavor(fn, flavor);
    if (rc) return rc;
    if ((rc = check_mode(fn, mode))) return rc;
    const size_t groups = (channels + group - 1) / group;
    const size_t period = channels * inner;
    // Many workgroups over the columns: a workgroup per group leaves the chip idle where the groups are few, reads
    // with a stride where their runs are short, and works element by element.  Small tensors stay with its one launch.
    const bool spread = x && out && !(groups >> 31) && outer * period >= kSpreadMinElems && period >= 16;
    // (the spread form clears the status word in its first kernel)
    if (out_status && !spread)
        hipLaunchKernelGGL(fill_i32_kernel, dim3(1), dim3(64), 0, ctx->stream, out_status, 0, size_t(1));
    if (channels == 0) return check_launch(fn);
    if (outer == 0 || inner == 0) return fail(HIPQ_INVALID_ARGUMENT, "%s: channels of zero length have no range", fn);
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(out);
    if (groups >> 31) return fail(HIPQ_INVALID_ARGUMENT, "%s: too many channels", fn);
    const bool even = (mode & HIPQ_ROUND_HALF_EVEN) != 0;
    if (spread) {
        const bool vec = inner % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0 &&
                         (reinterpret_cast<uintptr_t>(out) & 3u) == 0;
        ChannelColumns cc;
        cc.outer = outer;
        cc.period = period;
        cc.units = vec ? period / 4 : period;
        cc.span = inner * group;
        // Groups narrower than a wave's columns: every lane, or every few, ends in atomics of its own (they go past
        // the per-die caches and cost accordingly).  Tiles one wave wide then let the four waves combine first, and
        // at least eight rows per thread keep the atomics under one per 32 elements.
        const bool narrow = cc.span / (vec ? 4 : 1) < size_t(kWave);
        const int widest = narrow ? 6 : 8;
        cc.col_lanes_log2 = 0;
        while (cc.col_lanes_log2 < widest && (size_t(1) << cc.col_lanes_log2) < cc.units) ++cc.col_lanes_log2;
        const size_t col_lanes = size_t(1) << cc.col_lanes_log2, row_lanes = kBlock / col_lanes;
        const size_t col_tiles = (cc.units + col_lanes - 1) / col_lanes;
        const size_t row_sets = (outer + row_lanes - 1) / row_lanes;
        const size_t most = narrow ? (row_sets + 7) / 8 : row_sets;
        size_t slices = (size_t(ctx->num_cus) * 8 + col_tiles - 1) / col_tiles;
        if (slices > most) slices = most;
        if (col_tiles * slices >> 31) return fail(HIPQ_INVALID_ARGUMENT, "%s: too many columns", fn);
        cc.col_tiles = static_cast<unsigned>(col_tiles);
        cc.slices = static_cast<unsigned>(slices);
        void *s = nullptr;
        // (narrow groups: a wave's atomics go to neighbouring keys, which travel together when they share lines)
        cc.key_shift = (!narrow && groups <= 65536) ? 4 : 1;
        if ((rc = scratch(ctx, kScratchHeader + (groups << cc.key_shift) * sizeof(int32_t), &s))) return rc;
        int32_t *keys = reinterpret_cast<int32_t *>(static_cast<char *>(s) + kScratchHeader);
        const unsigned ngroups = static_cast<unsigned>(groups), gblocks = (ngroups + kBlock - 1) / kBlock;
        const dim3 grid(cc.col_tiles * cc.slices);
        hipLaunchKernelGGL(channel_keys_init_kernel, dim3(gblocks), dim3(kBlock), 0, ctx->stream, keys, ngroups,
                           cc.key_shift, out_status);
        if (vec)
            hipLaunchKernelGGL(channel_range_kernel<4>, grid, dim3(kBlock), 0, ctx->stream, x, cc, keys);
        else
            hipLaunchKernelGGL(channel_range_kernel<1>, grid, dim3(kBlock), 0, ctx->stream, x, cc, keys);
#define HIPQ_LAUNCH_CQ(E, V)                                                                                         \
    hipLaunchKernelGGL((channel_quantize_kernel<E, V>), grid, dim3(kBlock), 0, ctx->stream, x, cc, keys, flavor, qmin, \
                       qmax, out, out_scales, out_zero_points, out_status)
        if (even && vec)
            HIPQ_LAUNCH_CQ(true, 4);
        else if (even)
            HIPQ_LAUNCH_CQ(true, 1);
        else if (vec)
            HIPQ_LAUNCH_CQ(false, 4);
        else
            HIPQ_LAUNCH_CQ(false, 1);
#undef HIPQ_LAUNCH_CQ
        return check_launch(fn);
    }
    const int grid = static_cast<int>(groups);
    if (even)
        hipLaunchKernelGGL((quantize_per_channel_auto_kernel<true>), dim3(grid), dim3(kBlock), 0, ctx->stream, x, outer,
                           channels, inner, group, flavor, qmin, qmax, out, out_scales, out_zero_points, out_status);
    else
        hipLaunchKernelGGL((quantize_per_channel_auto_kernel<false>), dim3(grid), dim3(kBlock), 0, ctx->stream, x,
                           outer, channels, inner, group, flavor, qmin, qmax, out, out_scales, out_zero_points,
                           out_status);
    return check_launch(fn);
}

// Activation quantizers of the fused Linear forwards (declared in hipq_internal.h).  A range that is
// not finite poisons the operands (NaN scale, zero codes) instead of leaving stale scratch.
int32_t hipq::quantize_activations_per_tensor(hipq_ctx *ctx, const float *x, size_t rows, size_t cols, bool dynamic,
                                              float static_scale, int32_t mode, bool packed, int8_t *out,
                                              hipq_qparams *out_params, void *partials, size_t partials_bytes) {
    const char *fn = "hipq_linear (activation quantize)";
    int32_t rc = check_mode(fn, mode);
    if (rc) return rc;
    DynamicRange dyn{nullptr, 0, HIPQ_PARAMS_SYMMETRIC, -128, 127, out_params};
    dyn.poison = 1;
    float scale = 1.0f;
    const size_t KB = ((cols + 31) / 32 + 3) / 4 * 4, nfrag = ((rows + 31) / 32) * KB;
    size_t blocks = (nfrag + 3) / 4;
    const size_t cap = size_t(ctx->num_cus) * 8;
    int grid = static_cast<int>(blocks < cap ? blocks : cap);
    const bool div = (mode & HIPQ_FORM_DIV) != 0, even = (mode & HIPQ_ROUND_HALF_EVEN) != 0;
    // Fragments per wave of the one-launch form: one while that gives a workgroup per compute unit at most, two up to
    // four times that (fewer workgroups to meet: 512 x 4096 7.36 -> 7.27 us, 1024 x 4096 9.74 -> 9.18 us, the Linear
    // step at 512 rows -0.3 us), else four; more where the grid would not be resident otherwise.
    int fpw = blocks <= size_t(ctx->num_cus) ? 1 : (blocks <= size_t(ctx->num_cus) * 4 ? 2 : 4);
    while (fpw < 4 && (blocks + fpw - 1) / fpw > resident_workgroups(ctx, false)) fpw *= 2;
    const size_t q1_blocks = (blocks + fpw - 1) / fpw;
    if (dynamic && packed && ctx->gemm_variant != 6 && q1_blocks <= resident_workgroups(ctx, fpw == 4) && cols % 16 == 0 &&
        (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && (fpw == 1 || four_wide_workgroups_fit(ctx))) {
        // Every lane's 16 floats are all inside the matrix or all outside it, and four aligned float4.
#define HIPQ_LAUNCH_Q1(D, E, F)                                                                                           \
    hipLaunchKernelGGL((quantize_packed_one_launch_kernel<D, E, F>), dim3(static_cast<int>(q1_blocks)), dim3(kBlock), 0, \
                       ctx->stream, x, rows, cols, out_params, ctx->wait_error, ctx->wait_spin_limit, out,              \
                       ctx->warm)
#define HIPQ_LAUNCH_Q1_MODE(F)          \
    do {                                \
        if (div && even)                \
            HIPQ_LAUNCH_Q1(true, 1, F); \
        else if (div)                   \
            HIPQ_LAUNCH_Q1(true, 0, F); \
        else if (even)                  \
            HIPQ_LAUNCH_Q1(false, 1, F); \
        else                            \
            HIPQ_LAUNCH_Q1(false, 0, F); \
    } while (0)
        if (fpw == 1)
            HIPQ_LAUNCH_Q1_MODE(1);
        else if (fpw == 2)
            HIPQ_LAUNCH_Q1_MODE(2);
        else
            HIPQ_LAUNCH_Q1_MODE(4);
#undef HIPQ_LAUNCH_Q1_MODE
#undef HIPQ_LAUNCH_Q1
        return check_launch("quantize (packed, one launch)");
    }
    if (dynamic && packed) {
        // Range pass in the quantizer's own order and with its grid (FragmentWalk): one partial per workgroup.
        float2 *p = static_cast<float2 *>(partials);
        if (p) {
            const size_t room = partials_bytes / sizeof(float2);
            if (size_t(grid) > room) grid = static_cast<int>(room);
        } else {
            void *s = nullptr;
            if ((rc = scratch(ctx, kScratchHeader + size_t(grid) * sizeof(float2), &s))) return rc;
            p = reinterpret_cast<float2 *>(static_cast<char *>(s) + kScratchHeader);
        }
        hipLaunchKernelGGL(minmax_fragments_kernel, dim3(grid), dim3(kBlock), 0, ctx->stream, x, rows, cols, p);
        if ((rc = check_launch("minmax (fragments)"))) return rc;
        dyn.partials = p;
        dyn.nparts = grid;
    } else if (dynamic) {
        const size_t n = rows * cols;
        if (launch_flat_one_launch<int8_t>(ctx, x, n, HIPQ_PARAMS_SYMMETRIC, -128, 127, mode, /*poison=*/true, out_params,
                                           out, &rc))
            return rc;
        rc = launch_minmax_partials(ctx, x, n, &dyn, static_cast<float2 *>(partials),
                                    partials_bytes / sizeof(float2));
        if (rc) return rc;
    } else {
        if ((rc = check_scale(fn, static_scale))) return rc;
        scale = static_scale;
    }
    if (!packed) return launch_quantize<int8_t>(ctx, x, rows * cols, scale, 0, nullptr, mode, -128.0f, 127.0f, out, dyn);
#define HIPQ_LAUNCH_QP(D, E)                                                                                       \
    hipLaunchKernelGGL((quantize_packed_kernel<D, E>), dim3(grid), dim3(kBlock), 0, ctx->stream, x, rows, cols, scale, \
                       0, static_cast<const hipq_qparams *>(nullptr), dyn, out)
    if (div && even)
        HIPQ_LAUNCH_QP(true, 1);
    else if (div)
        HIPQ_LAUNCH_QP(true, 0);
    else if (even)
        HIPQ_LAUNCH_QP(false, 1);
    else
        HIPQ_LAUNCH_QP(false, 0);
#undef HIPQ_LAUNCH_QP
    return check_launch("quantize (packed)");
}

int32_t hipq::quantize_activations_per_row(hipq_ctx *ctx, const float *x, size_t rows, size_t cols, int32_t mode,
                                           int8_t *out, float *out_scales, bool packed) {
    return quantize_rows("hipq_linear (activation quantize)", ctx, x, rows, cols, cols, HIPQ_PARAMS_SYMMETRIC, false,
                         -128, 127, mode, out, out_scales, nullptr, nullptr, /*poison=*/1, packed);
}

int32_t hipq::quantize_activations_per_row_strided(hipq_ctx *ctx, const float *x, size_t rows, size_t cols, size_t ld,
                                                   int32_t mode, int8_t *out, float *out_scales, bool packed) {
    return quantize_rows("hipq_linear (activation quantize)", ctx, x, rows, cols, ld, HIPQ_PARAMS_SYMMETRIC, false,
                         -128, 127, mode, out, out_scales, nullptr, nullptr, /*poison=*/1, packed);
}

extern "C" {

int32_t hipq_quantize_per_row_strided_f32_i8(hipq_ctx *ctx, const float *x, size_t rows, size_t cols, size_t ld,
                                             int32_t flavor, int32_t mode, int8_t *out, float *out_scales,
                                             int32_t *out_zero_points, int32_t *out_status) {
    HIPQ_ENTER(ctx);
    return quantize_rows(__func__, ctx, x, rows, cols, ld, flavor, false, -128, 127, mode, out, out_scales,
                         out_zero_points, out_status);
}

int32_t hipq_quantize_per_row_f32_i8(hipq_ctx *ctx, const float *x, size_t rows, size_t cols, int32_t flavor,
                                     int32_t mode, int8_t *out, float *out_scales, int32_t *out_zero_points,
                                     int32_t *out_status) {
    return hipq_quantize_per_row_strided_f32_i8(ctx, x, rows, cols, cols, flavor, mode, out, out_scales,
                                                out_zero_points, out_status);
}

int32_t hipq_quantize_per_channel_auto_f32_i8(hipq_ctx *ctx, const float *x, size_t outer, size_t channels,
                                              size_t inner, int32_t flavor, int32_t mode, int8_t *out,
                                              float *out_scales, int32_t *out_zero_points, int32_t *out_status) {
    HIPQ_ENTER(ctx);
    return quantize_channels(__func__, ctx, x, outer, channels, inner, 1, flavor, false, -128, 127, mode, out,
                             out_scales, out_zero_points, out_status);
}

int32_t hipq_quantize_per_group_auto_f32_i8(hipq_ctx *ctx, const float *x, size_t outer, size_t channels,
                                            size_t inner, size_t group_size, int32_t flavor, int32_t qmin,
                                            int32_t qmax, int32_t mode, int8_t *out, float *out_scales,
                                            int32_t *out_zero_points, int32_t *out_status) {
    HIPQ_ENTER(ctx);
    if (flavor < HIPQ_PARAMS_SYMMETRIC || flavor > HIPQ_PARAMS_NN_ASYMMETRIC)
        return fail(HIPQ_INVALID_ARGUMENT, "%s: unknown flavor %d", __func__, flavor);
    // one byte per code: a signed range is stored as int8, an unsigned one (qmin >= 0) as the same byte read as uint8
    if (qmin >= qmax || !((qmin >= -128 && qmax <= 127) || (qmin >= 0 && qmax <= 255)))
        return fail(HIPQ_INVALID_ARGUMENT, "%s: range [%d, %d] must lie inside [-128, 127] or [0, 255]", __func__, qmin,
                    qmax);
    return quantize_channels(__func__, ctx, x, outer, channels, inner, group_size, flavor, true, qmin, qmax, mode, out,
                             out_scales, out_zero_points, out_status);
}

int32_t hipq_quantize_per_channel_f32_i8(hipq_ctx *ctx, const float *x, size_t outer, size_t channels, size_t inner,
                                         const float *scales, const int32_t *zero_points, int32_t mode,
                                         int8_t *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_mode(__func__, mode);
    if (rc) return rc;
    const size_t total = outer * channels * inner;
    if (total == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(x);
    HIPQ_REQUIRE_PTR(scales);
    HIPQ_REQUIRE_PTR(zero_points);
    HIPQ_REQUIRE_PTR(out);
    const bool div = (mode & HIPQ_FORM_DIV) != 0, even = (mode & HIPQ_ROUND_HALF_EVEN) != 0;
    if (inner % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && (reinterpret_cast<uintptr_t>(out) & 3u) == 0) {
        const int vgrid = grid_for_tiles(ctx, total);
#define HIPQ_LAUNCH_PCV(D, E)                                                                                          \
    hipLaunchKernelGGL((quantize_per_channel_vec_kernel<D, E>), dim3(vgrid), dim3(kBlock), 0, ctx->stream, x, total / 4, \
                       channels, inner, scales, zero_points, out)
        if (div && even)
            HIPQ_LAUNCH_PCV(true, true);
        else if (div)
            HIPQ_LAUNCH_PCV(true, false);
        else if (even)
            HIPQ_LAUNCH_PCV(false, true);
        else
            HIPQ_LAUNCH_PCV(false, false);
#undef HIPQ_LAUNCH_PCV
        return check_launch(__func__);
    }
    const int grid = grid_for_elems(ctx, total);
#define HIPQ_LAUNCH_PC(D, E)                                                                                       \
    hipLaunchKernelGGL((quantize_per_channel_kernel<D, E>), dim3(grid), dim3(kBlock), 0, ctx->stream, x, total,     \
                       channels, inner, scales, zero_points, out)
    if (div && even)
        HIPQ_LAUNCH_PC(true, true);
    else if (div)
        HIPQ_LAUNCH_PC(true, false);
    else if (even)
        HIPQ_LAUNCH_PC(false, true);
    else
        HIPQ_LAUNCH_PC(false, false);
#undef HIPQ_LAUNCH_PC
    return check_launch(__func__);
}

int32_t hipq_dequantize_per_channel_i8_f32(hipq_ctx *ctx, const int8_t *q, size_t outer, size_t channels,
                                           size_t inner, const float *scales, const int32_t *zero_points,
                                           float *out) {
    HIPQ_ENTER(ctx);
    const size_t total = outer * channels * inner;
    if (total == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(q);
    HIPQ_REQUIRE_PTR(scales);
    HIPQ_REQUIRE_PTR(zero_points);
    HIPQ_REQUIRE_PTR(out);
    if (inner % 4 == 0 && (reinterpret_cast<uintptr_t>(q) & 3u) == 0 && (reinterpret_cast<uintptr_t>(out) & 15u) == 0) {
        hipLaunchKernelGGL(dequantize_per_channel_vec_kernel, dim3(grid_for_tiles(ctx, total)), dim3(kBlock), 0,
                           ctx->stream, q, total / 4, channels, inner, scales, zero_points, out);
        return check_launch(__func__);
    }
    const int grid = grid_for_elems(ctx, total);
    hipLaunchKernelGGL(dequantize_per_channel_kernel, dim3(grid), dim3(kBlock), 0, ctx->stream, q, total, channels,
                       inner, scales, zero_points, out);
    return check_launch(__func__);
}

int32_t hipq_requantize_i32_i8(hipq_ctx *ctx, const int32_t *acc, size_t rows, size_t cols, const float *a_scale,
                               int32_t a_scale_per_row, const float *w_scales, const float *bias, float out_scale,
                               int32_t out_zero_point, int32_t mode, int8_t *out) {
    HIPQ_ENTER(ctx);
    int32_t rc = check_scale(__func__, out_scale);
    if (rc) return rc;
    if ((rc = check_mode(__func__, mode))) return rc;
    if (rows * cols == 0) return HIPQ_SUCCESS;
    HIPQ_REQUIRE_PTR(acc);
    HIPQ_REQUIRE_PTR(a_scale);
    HIPQ_REQUIRE_PTR(w_scales);
    HIPQ_REQUIRE_PTR(out);
    const bool vec = cols % 4 == 0 && (reinterpret_cast<uintptr_t>(acc) & 15u) == 0 &&
                     (reinterpret_cast<uintptr_t>(w_scales) & 15u) == 0 && (reinterpret_cast<uintptr_t>(bias) & 15u) == 0 &&
                     (reinterpret_cast<uintptr_t>(out) & 3u) == 0;
    if (vec) {
        // A grid of g workgroups hands a thread the vectors j, j + g * kTileVec, ...: the same column vector every
        // time when g * kTileVec is a multiple of the vectors per row.  With several tiles per workgroup that pays
        // (weight scales and biases loaded once per thread); g = the multiple of the period nearest 4 per compute unit (eight was slower: 17.1 against 16.4 us for 16 Mi).
        const size_t vpr = cols / 4, tiles = (rows * vpr + kTileVec - 1) / kTileVec;
        size_t a = vpr, b = kTileVec;
        while (b) {
            const size_t t = a % b;
            a = b;
            b = t;
        }
        const size_t period = vpr / a, want = size_t(ctx->num_cus) * 4;
        const size_t fixed_grid = period <= want ? want / period * period : 0;
        const bool fixed = fixed_grid && tiles >= 2 * fixed_grid;
        const int vgrid = fixed ? static_cast<int>(fixed_grid) : grid_for_tiles(ctx, rows * cols);
#define HIPQ_LAUNCH_RQ(E, F)                                                                                         \
    hipLaunchKernelGGL((requantize_vec_kernel<E, F>), dim3(vgrid), dim3(kBlock), 0, ctx->stream, acc, rows, cols, a_scale, \
                       a_scale_per_row, w_scales, bias, out_scale, out_zero_point, out)
        if (mode & HIPQ_ROUND_HALF_EVEN) {
            if (fixed)
                HIPQ_LAUNCH_RQ(true, true);
            else
                HIPQ_LAUNCH_RQ(true, false);
        } else {
            if (fixed)
                HIPQ_LAUNCH_RQ(false, true);
            else
                HIPQ_LAUNCH_RQ(false, false);
        }
#undef HIPQ_LAUNCH_RQ
        return check_launch(__func__);
    }
    const int grid = grid_for_elems(ctx, rows * cols);
    if (mode & HIPQ_ROUND_HALF_EVEN)
        hipLaunchKernelGGL((requantize_kernel<true>), dim3(grid), dim3(kBlock), 0, ctx->stream, acc, rows, cols,
                           a_scale, a_scale_per_row, w_scales, bias, out_scale, out_zero_point, out);
    else
        hipLaunchKernelGGL((requantize_kernel<false>), dim3(grid), dim3(kBlock), 0, ctx->stream, acc, rows, cols,
                           a_scale, a_scale_per_row, w_scales, bias, out_scale, out_zero_point, out);
    return check_launch(__func__);
}

}  // extern "C"
