// A meeting of all workgroups of one launch, through device words of the context: the grid agrees on the
// (min, max) of a tensor of which every workgroup has seen a part, without ending the kernel.
//
// Every word another workgroup waits for is a 64-bit {meeting number, payload} pair written by one atomic
// store, so a reader can tell a word of this meeting from what an earlier one left behind; nothing is reset
// between launches.  The number comes from device memory: every workgroup reads it first (meeting_number),
// and workgroup 0 advances it once all workgroups have published their range, which they do after reading it.
// A launch therefore needs no host state and a captured launch can be replayed.  When the number is about to
// wrap, workgroup 0 wipes the range words (nobody reads them any more once all have published), so that none
// can be taken for a word of a meeting 2^32 launches later.
//
// Every workgroup publishes {number, min} and {number, max}; workgroup 0 polls the words of all workgroups,
// folds them, derives the parameters and publishes them in one word (ready_word); thread 0 of every other
// workgroup polls that word.  That is two trips through device-coherent memory on the critical path (~1.5 us each).
// Measured alternatives: arrival counters need four trips and cross-XCD atomics on one address serialise
// (+1.3 us); every workgroup polling every workgroup's words needs one trip, but 512 workgroups reading the
// same 64 lines past their L2s round after round cost more than the trip saved (+1.2 us).
//
// All waits are bounded: a poll that gives up sets the context's flag word (hipq_ctx_synchronize reports
// it) and the kernel runs on with defined values, so a grid always drains.  The caller guarantees that the
// grid can be resident at once; launches that share a context's words must not overlap (they are on the
// context's one stream).  256 threads per workgroup.
#pragma once

#include "hipq_internal.h"
#include "hipq_math.h"

namespace hipq {

constexpr int kBlock = 256;

struct MinMax {
    float mn, mx;
};

__device__ __forceinline__ void acc_minmax(MinMax &m, float v) {
    m.mn = fminf(m.mn, v);
    m.mx = fmaxf(m.mx, v);
}

// Block-wide min/max; result valid in every thread.
__device__ __forceinline__ MinMax block_minmax(MinMax m, float *lds /* 2 * kBlock/kWave floats */) {
    m.mn = wave_min(m.mn);
    m.mx = wave_max(m.mx);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    constexpr int nw = kBlock / kWave;
    __syncthreads();
    if (lane == 0) {
        lds[wave] = m.mn;
        lds[nw + wave] = m.mx;
    }
    __syncthreads();
    MinMax r{lds[0], lds[nw]};
#pragma unroll
    for (int w = 1; w < nw; ++w) {
        r.mn = fminf(r.mn, lds[w]);
        r.mx = fmaxf(r.mx, lds[nw + w]);
    }
    return r;
}

constexpr int kMeetingLdsFloats = 2 * kBlock / kWave + 2;

// The number of the meeting this launch holds.  Call it before anything of the meeting is published.
__device__ __forceinline__ uint32_t meeting_number(const uint32_t *words) {
    return __hip_atomic_load(words + kCtxEpochWord, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
}

// {number, min}, {number, max} of workgroup `workgroup`.
__device__ __forceinline__ unsigned long long *meeting_range_slot(uint32_t *words, unsigned workgroup) {
    return reinterpret_cast<unsigned long long *>(words + kCtxRangeWord) + 2 * size_t(workgroup);
}
__device__ __forceinline__ void publish_tagged(unsigned long long *word, uint32_t gen, uint32_t payload) {
    __hip_atomic_store(word, (static_cast<unsigned long long>(gen) << 32) | payload, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

// Polls `word` until it carries meeting `gen` (at most spin_limit + 1 looks); false = gave up.
__device__ __forceinline__ bool poll_tagged(const unsigned long long *word, uint32_t gen, int spin_limit,
                                            uint32_t *payload) {
    for (int spin = 0; spin <= spin_limit; ++spin) {
        const unsigned long long w = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (static_cast<uint32_t>(w >> 32) == gen) {
            *payload = static_cast<uint32_t>(w);
            return true;
        }
        __builtin_amdgcn_s_sleep(1);
    }
    return false;
}

__device__ __forceinline__ void record_give_up(uint32_t *words) {
    __hip_atomic_store(words + kCtxFlagWord, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The word that ends the range part of a meeting carries the scale, the zero point and a tag in 64 bits, so that
// one look suffices: {meeting number mod 2^22, zero point + 128 in 10 bits, scale bits}.  The short tag is enough
// here because this word, unlike the range words, is rewritten by every meeting - also by those that only collect
// a range and have nobody waiting for it (meeting_mark_ready) - so it only has to differ from the one before (and
// from the all-zero initial state, which the first numbers of a context do).
constexpr uint32_t kReadyTagMask = 0x3fffffu;

// What a meeting agrees on: the parameters workgroup 0 derives from the folded range.  scale is NaN when the
// range is not acceptable to the flavor (not finite, ...) or a wait of the meeting was given up.
struct MeetingParams {
    float scale;
    int zero_point;
};

__device__ __forceinline__ unsigned long long ready_word(uint32_t gen, const MeetingParams &p) {
    return (static_cast<unsigned long long>(gen & kReadyTagMask) << 42) |
           (static_cast<unsigned long long>(static_cast<uint32_t>(p.zero_point + 128) & 0x3ffu) << 32) |
           __builtin_bit_cast(uint32_t, p.scale);
}

// Workgroup 0, thread 0, of a meeting in which nobody waits for parameters: leaves this meeting's tag in the ready
// word (NaN scale), so that the word always carries the number of the last meeting held.
__device__ __forceinline__ void meeting_mark_ready(uint32_t *words, uint32_t gen) {
    __hip_atomic_store(reinterpret_cast<unsigned long long *>(words + kCtxReadyWord),
                       ready_word(gen, MeetingParams{__builtin_nanf(""), 0}), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The whole grid agrees on the quantization parameters of a tensor: `r` is this workgroup's (min, max), uniform
// over its threads; flavor / qmin / qmax as for params_from_minmax.  Returns the same parameters in every thread of
// every workgroup.  Workgroup 0 also writes them to out_params, with the status; for a bad range it records a
// NaN scale if `poison` is set (the fused Linear forwards, whose GEMM must then produce NaN) and the neutral 1.0 of
// the two-launch path otherwise.  `lds`: kMeetingLdsFloats floats.
__device__ __forceinline__ void meeting_publish_range(uint32_t *words, uint32_t gen, MinMax r) {
    if (threadIdx.x == 0) {
        unsigned long long *mine = meeting_range_slot(words, blockIdx.x);
        publish_tagged(mine, gen, __builtin_bit_cast(uint32_t, r.mn));
        publish_tagged(mine + 1, gen, __builtin_bit_cast(uint32_t, r.mx));
    }
}

// Workgroup 0, all threads: waits for the range words of every workgroup of the grid and folds them; the result
// is valid in every thread.  Returns true if a wait was given up.
__device__ __forceinline__ bool meeting_collect_range(uint32_t *words, uint32_t gen, int spin_limit, float *lds,
                                                      MinMax *folded) {
    MinMax t{INFINITY, -INFINITY};
    bool all = true;
    for (unsigned i = threadIdx.x; i < gridDim.x; i += kBlock) {
        uint32_t lo = 0, hi = 0;
        const unsigned long long *slot = meeting_range_slot(words, i);
        const bool got = poll_tagged(slot, gen, spin_limit, &lo) && poll_tagged(slot + 1, gen, spin_limit, &hi);
        if (got) {
            t.mn = fminf(t.mn, __builtin_bit_cast(float, lo));
            t.mx = fmaxf(t.mx, __builtin_bit_cast(float, hi));
        }
        all &= got;
    }
    const bool gave_up = __syncthreads_or(!all) != 0;
    *folded = block_minmax(t, lds);
    return gave_up;
}

// Workgroup 0, all threads, after meeting_collect_range: every workgroup has published, so every workgroup has
// read the number, and nobody writes or reads a range word any more (or the meeting is lost anyway): advances the
// number, and at its wrap wipes the range words first.
__device__ __forceinline__ void meeting_close(uint32_t *words, uint32_t gen, bool gave_up) {
    const bool wrap = gen == 0xffffffffu;
    if (wrap) {
        unsigned long long *first = meeting_range_slot(words, 0);
        for (unsigned i = threadIdx.x; i < 2 * kCtxSlots; i += kBlock)
            __hip_atomic_store(first + i, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        __hip_atomic_store(words + kCtxEpochWord, wrap ? 0u : gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (gave_up) record_give_up(words);
    }
}

__device__ __forceinline__ MeetingParams meet_on_range(uint32_t *words, uint32_t gen, MinMax r, int flavor, int qmin,
                                                       int qmax, bool poison, int spin_limit, float *lds,
                                                       hipq_qparams *out_params) {
    unsigned long long *ready = reinterpret_cast<unsigned long long *>(words + kCtxReadyWord);
    meeting_publish_range(words, gen, r);
    MeetingParams p;
    if (blockIdx.x == 0) {
        MinMax t;
        const bool gave_up = meeting_collect_range(words, gen, spin_limit, lds, &t);
        float scale;
        int zp;
        int st = params_from_minmax(t.mn, t.mx, flavor, qmin, qmax, &scale, &zp);
        if (gave_up) st = HIPQ_DEVICE_ERROR;
        if (st == HIPQ_SUCCESS && (zp < -128 || zp > 895)) st = HIPQ_INVALID_ARGUMENT;  // not a code of an 8-bit type
        const bool bad = st != HIPQ_SUCCESS;
        p.scale = bad ? __builtin_nanf("") : scale;
        p.zero_point = bad ? 0 : zp;
        meeting_close(words, gen, gave_up);
        if (threadIdx.x == 0) {
            __hip_atomic_store(ready, ready_word(gen, p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            out_params->scale = (bad && !poison) ? scale : p.scale;
            out_params->zero_point = bad ? zp : p.zero_point;
            out_params->min_val = t.mn;
            out_params->max_val = t.mx;
            // A workgroup that stopped waiting for the word above has marked the context; the record says so as
            // well (it writes the status itself too, in case this store is the later one).
            const bool lost = __hip_atomic_load(words + kCtxFlagWord, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
            __hip_atomic_store(&out_params->status, lost ? HIPQ_DEVICE_ERROR : st, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        }
    } else {
        if (threadIdx.x == 0) {
            bool got = false;
            for (int spin = 0; spin <= spin_limit; ++spin) {
                const unsigned long long w = __hip_atomic_load(ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((w >> 42) == (gen & kReadyTagMask)) {
                    lds[kMeetingLdsFloats - 2] = __builtin_bit_cast(float, static_cast<uint32_t>(w));
                    lds[kMeetingLdsFloats - 1] = __builtin_bit_cast(float, static_cast<int>((w >> 32) & 0x3ffu) - 128);
                    got = true;
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
            if (!got) {
                record_give_up(words);
                __hip_atomic_store(&out_params->status, HIPQ_DEVICE_ERROR, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                lds[kMeetingLdsFloats - 2] = __builtin_nanf("");
                lds[kMeetingLdsFloats - 1] = 0.0f;
            }
        }
        __syncthreads();
        p.scale = lds[kMeetingLdsFloats - 2];
        p.zero_point = __builtin_bit_cast(int, lds[kMeetingLdsFloats - 1]);
    }
    return p;
}

}  // namespace hipq
