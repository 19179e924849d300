// int8 GEMM on fragment-packed operands with one PANEL OF ROWS per workgroup: 32 rows of the activations against
// ALL columns of the weights, the whole panel of accumulators in registers (N / 32 blocks of 32 x 32, an eighth of
// them per wave: up to 192 registers).
//
// Why.  In a transformer block the products are tall and short in K (8192 x 2304 x 768, 8192 x 3072 x 768, ...)
// and every one of them feeds an operation that needs whole rows: a per-token quantizer (the row's maximum), a
// LayerNorm (the row's mean and variance).  Tiles of 128 or 256 columns cannot apply those, so the fp32 product
// goes to memory and comes back through a row kernel: 100 MB out and 100 MB in for fc1 alone, more time than the
// multiply.  A workgroup that owns whole rows applies them in its epilogue, on the accumulators:
//   RP_F32         out = acc * (s_a[m] * s_w[n]) + bias[n]                                   (qkv)
//   RP_GELU_Q      per-token int8 of GELU(that), written as the packed operand of the next product      (fc1)
//   RP_RESID_F32   x += that                                                                 (the last fc2)
//   RP_RESID_LN_Q  x += that, then per-token int8 of LayerNorm(x), packed                     (out-proj, fc2)
// Every f32 operation is the one the separate kernels perform (same functions, same order per element); only the
// order in which a LayerNorm's row sums are folded differs (here: over a lane's column blocks, the 32 lanes of a
// half wave, the eight waves), which moves the mean and variance in their last bits, as any other order does.
//
// The price is operand traffic: every workgroup streams the whole weight matrix (out of its XCD's L2, which holds
// it), one 1 KiB fragment per MFMA - 128 bytes per clock and compute unit wanted, ~57 delivered - so the main loop
// runs at the vector-memory path's pace, N * K / 57 cycles.  The activations stay off that path: the panel's
// fragments go through LDS, 24 k blocks at a time (two buffers, one barrier per 24 k blocks), and every wave
// reads the fragment of a k block from there.  Weight fragments go from L2 straight into registers, D in flight
// per wave (48 KiB or more per compute unit: what the path needs to stay busy at its latency).
//
// M any; K any; N a multiple of 32 and at most 3072 (the *_Q forms: a multiple of 128, since their output is the
// K of the next product).  Included by hipq_gemm_packed.hip.
#pragma once

#include "hipq_gemm_packed.h"

namespace hipq {

enum { RP_F32 = 0, RP_GELU_Q = 1, RP_RESID_F32 = 2, RP_RESID_LN_Q = 3 };

struct RowPanel {
    const int8_t *pa;   // packed activations [M, K]
    const float *sa;    // activation scales: [M] (sa_per_row) or one
    int sa_per_row;
    const int8_t *pw;   // packed weights [N, K]
    const float *sw;    // [N]
    const float *bias;  // [N] or null
    int M, N, K;
    float *out_f;       // RP_F32: [M, N]; RP_RESID_*: the stream x [M, N], read and written
    int8_t *out_q;      // *_Q: packed int8 [M, N]
    float *out_scales;  // *_Q: [M]
    const float *gamma, *beta;  // RP_RESID_LN_Q: [N] or null
    float eps;
    const float *af;    // fp32 activations [M, K], rows lda floats apart (the kernels that quantize them themselves)
    int lda;
};

constexpr int kRowsWaves = 8;
constexpr int kRowsThreads = kRowsWaves * kWave;
constexpr int kRowsStage = 24;  // k blocks of the activation panel per LDS buffer (24 KiB)

// tanh-form GELU as the row kernels evaluate it (gelu_tanh in hipq_fp32.hip: the same three lines).
__device__ __forceinline__ float rp_gelu_tanh(float x) {
    constexpr float K = -2.8853900817779268f * 0.7978845608028654f;
    const float arg = x * fmaf(x * x, K * 0.044715f, K);
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(arg));
}

// Maximum or sum over the 32 lanes of a half wave, the result in every lane: four steps inside a row of 16 lanes
// on the data-parallel path (quad swaps, then the mirrors of 8 and 16 lanes: after each step the groups that were
// combined hold one value), one swizzle across the two rows.  Both partners of a step add the same two numbers,
// so all lanes end with the same bits.  MAX is for non-negative values that are no NaN: those order as their bit
// patterns do, and an integer maximum needs no quieting of its operands.
template <bool MAX>
__device__ __forceinline__ float half_wave_fold(float v) {
    auto combine = [](float a, float b) {
        if constexpr (MAX) {
            const uint32_t x = __builtin_bit_cast(uint32_t, a), y = __builtin_bit_cast(uint32_t, b);
            const uint32_t m = x > y ? x : y;
            return __builtin_bit_cast(float, m);
        } else {
            return a + b;
        }
    };
    auto dpp = [](float x, auto ctrl) {
        const int bits = __builtin_bit_cast(int, x);
        const int moved = __builtin_amdgcn_update_dpp(0, bits, decltype(ctrl)::value, 0xf, 0xf, false);
        return __builtin_bit_cast(float, moved);
    };
    v = combine(v, dpp(v, std::integral_constant<int, 0xB1>{}));   // quad_perm [1, 0, 3, 2]
    v = combine(v, dpp(v, std::integral_constant<int, 0x4E>{}));   // quad_perm [2, 3, 0, 1]
    v = combine(v, dpp(v, std::integral_constant<int, 0x141>{}));  // row_half_mirror
    v = combine(v, dpp(v, std::integral_constant<int, 0x140>{}));  // row_mirror
    const int bits = __builtin_bit_cast(int, v);
    const int other = __builtin_amdgcn_ds_swizzle(bits, 0x401F);  // lane ^ 16 (and 0x1f, or 0, xor 0x10)
    return combine(v, __builtin_bit_cast(float, other));
}

// The code of a value t = x / scale whose scale is its own row's max|x| / 127: round (ties away from zero, or to
// even) and convert.  v_cvt_i32_f32 truncates, so the ties-away form round_mode<0> = truncf(t + copysign(pred(0.5), t))
// needs no truncf of its own; |t| <= 127 (1 + 2^-22), so the result lies in [-127, 127] without a clamp; a NaN (a NaN
// element, or any element of a row whose scale is NaN: an infinity in the row, a row past M) converts to 0.
template <bool EVEN>
__device__ __forceinline__ int row_code(float t) {
    if constexpr (EVEN)
        return cvt_i32_sat(rintf(t));
    else
        return cvt_i32_sat(t + copysignf(0x1.fffffep-2f, t));
}

constexpr int rows_gcd(int a, int b) { return b == 0 ? a : rows_gcd(b, a % b); }

// AF32: the activations are fp32 rows (p.af, p.lda) and the workgroup quantizes its own 32 of them first, per token
// and symmetric, with the per-row quantizer's arithmetic (quantize_per_row_kernel: range by NaN-skipping min / max,
// params_from_minmax, division form; a row whose range is not finite gets a NaN scale and zero codes): a wave reads
// four rows, finds their ranges by shuffles, and writes the codes into LDS in fragment order, where the whole panel
// stays (K <= 1536) and the main loop reads it.  The quantizer's launch, its packed output and its scales are gone;
// the results are those of the two calls, bit for bit.
template <int NBW, int EPI, bool EVEN, bool AF32 = false>
__global__ __launch_bounds__(kRowsThreads) void gemm_i8_rows_kernel(RowPanel p) {
    constexpr int D = NBW <= 6 ? 12 : (NBW == 9 ? 9 : 6);  // weight fragments in flight per wave
    constexpr int U = D / rows_gcd(NBW, D);  // k blocks per trip of the main loop: U * NBW is a multiple of D
    static_assert((U * NBW) % D == 0 && kRowsStage % U == 0, "ring slots must be static");
    constexpr bool QUANT = EPI == RP_GELU_Q || EPI == RP_RESID_LN_Q;
    constexpr bool RESID = EPI == RP_RESID_F32 || EPI == RP_RESID_LN_Q;
    // The epilogue handles GS groups of four accumulator registers (= 4 rows per half wave) at a time: all 16 rows
    // where registers allow, else one group after the other (the row statistics then take a barrier per group).
    constexpr int GS = NBW <= 6 ? 4 : 1;
    constexpr int NR = 4 * GS;
    __shared__ __attribute__((aligned(1024))) int8_t apanel[2][kRowsStage * 1024];
    __shared__ __attribute__((aligned(16))) float red[3][kRowsWaves][32];  // [statistic][wave][row]: partial sums / maxima
    __shared__ __attribute__((aligned(16))) float fin[4][32];              // per row: mean, 1 / std, scale, 1 / scale
    __shared__ float sa_own[AF32 ? 32 : 1];                                // AF32: the rows' activation scales
    const int tid = threadIdx.x, lane = tid % kWave, half = lane / 32, cin = lane % 32;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int rb = blockIdx.x, m0 = rb * 32;
    const int KB = static_cast<int>(packed_k_blocks(p.K));  // (a multiple of 4)
    const int nblocks = p.N / 32;
    const int jb0 = wave * NBW;  // this wave's column blocks: jb0 .. jb0 + NBW - 1 (those past nblocks: no data)
    // Exact extents: a fragment past the operand (column blocks past N, k blocks past the last) reads as zeros
    // without touching memory, or as data of the next column block that no MFMA consumes.
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t *>(p.pa) + size_t(rb) * KB * 1024, 0, KB * 1024, 0x00020000);
    const __amdgpu_buffer_rsrc_t rw =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(p.pw), 0, nblocks * KB * 1024, 0x00020000);
    const int voff = lane * 16;
    const int wstride = KB * 1024;  // bytes between the column blocks of one k block
    const int wbase = jb0 * wstride;
    auto load_w = [&](int kb, int jj) {
        return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rw, voff, wbase + jj * wstride + kb * 1024, 0));
    };
    // one stage of the activation panel: 24 KiB = three 16-byte pieces per thread
    auto load_stage = [&](int s, v4i(&t)[3]) {
#pragma unroll
        for (int i = 0; i < 3; ++i)
            t[i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(
                                               ra, tid * 16, s * (kRowsStage * 1024) + i * (kRowsThreads * 16), 0));
    };

    // fp32 rows of this panel (output, or the stream that is read and written): rows past M lie beyond the buffer
    // and are dropped by the hardware.
    const int rows_here = p.M - m0 < 32 ? p.M - m0 : 32;
    const __amdgpu_buffer_rsrc_t rf = __builtin_amdgcn_make_buffer_rsrc(
        p.out_f ? reinterpret_cast<char *>(p.out_f) + size_t(m0) * p.N * 4 : nullptr, 0, p.out_f ? rows_here * p.N * 4 : 0,
        0x00020000);
    const int row_bytes = p.N * 4;
    auto load_x = [&](int jj, int r) {
        return __builtin_bit_cast(
            float, __builtin_amdgcn_raw_buffer_load_b32(rf, (4 * half * p.N + (jb0 + jj) * 32 + cin) * 4,
                                                        (8 * (r / 4) + (r % 4)) * row_bytes, 0));
    };

    // The weights are new to this XCD's L2 when the kernel starts (the previous layer used others), and all its
    // workgroups walk them in the same order at the same time: every fragment would be a miss for all of them at
    // once, and the walk would move at memory latency.  So each workgroup first touches its own thirty-second of
    // the matrix (workgroups b, b + 8, b + 16, ... share an XCD), one dword per 128-byte line: the whole matrix is
    // on its way into the L2 within one memory latency, and the walk below meets lines that are there or coming.
    {
        const int wbytes = nblocks * KB * 1024;
        const int chunk = ((wbytes + 31) / 32 + 127) & ~127;
        const int part = (blockIdx.x / 8) % 32;
        int touched = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int off = (tid + i * kRowsThreads) * 128;
            if (off < chunk) touched ^= __builtin_amdgcn_raw_buffer_load_b32(rw, off, part * chunk, 0);
        }
        // (keeps the loads alive; never true: p.M is positive)
        if (touched == 0x5a5a5a5a && p.M < 0) red[0][0][0] = 1.0f;
    }
    v4i wf[D];
#pragma unroll
    for (int u = 0; u < D; ++u) wf[u] = load_w(u / NBW, u % NBW);
    v4i astage[3];
    if constexpr (!AF32) load_stage(0, astage);
    if constexpr (AF32) {
        // rows 4 wave .. 4 wave + 3 of the panel: lane l holds floats 4 (l + 64 i) .. + 3 of each
        constexpr int kMaxVec = 6;  // K <= 1536
        int8_t *panel = &apanel[0][0];
        const int kpad = KB * 32;
        float4 v[4][kMaxVec];
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const int m = m0 + 4 * wave + rr;
            const float4 *row = reinterpret_cast<const float4 *>(p.af + size_t(m < p.M ? m : 0) * p.lda);
#pragma unroll
            for (int i = 0; i < kMaxVec; ++i) {
                const int k = 4 * (lane + kWave * i);
                if (m < p.M && k < p.K) v[rr][i] = row[lane + kWave * i];
            }
        }
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const int m = m0 + 4 * wave + rr;
            float mn = INFINITY, mx = -INFINITY;
#pragma unroll
            for (int i = 0; i < kMaxVec; ++i) {
                const int k = 4 * (lane + kWave * i);
                if (m < p.M && k < p.K) {
                    mn = fminf(mn, fminf(fminf(v[rr][i].x, v[rr][i].y), fminf(v[rr][i].z, v[rr][i].w)));
                    mx = fmaxf(mx, fmaxf(fmaxf(v[rr][i].x, v[rr][i].y), fmaxf(v[rr][i].z, v[rr][i].w)));
                }
            }
            mn = wave_min(mn);
            mx = wave_max(mx);
            float scale;
            int zp;
            const bool bad = params_from_minmax(mn, mx, HIPQ_PARAMS_SYMMETRIC, -128, 127, &scale, &zp) != HIPQ_SUCCESS;
            if (lane == 0) sa_own[4 * wave + rr] = bad ? __builtin_nanf("") : scale;
            if (bad) scale = INFINITY;  // x / inf: 0 for finite x, NaN -> code 0 otherwise
            const float inv = recip_for_div(scale);
            auto q = [&](float f) { return quantize_int<QFORM_DIV, EVEN>(f, scale, inv, 0.0f, -128, 127); };
#pragma unroll
            for (int i = 0; i < kMaxVec; ++i) {
                const int k = 4 * (lane + kWave * i);
                if (k < kpad) {  // (k past K up to the padded extent, rows past M: zeros)
                    uint32_t w4 = 0u;
                    if (m < p.M && k < p.K) w4 = pack4(q(v[rr][i].x), q(v[rr][i].y), q(v[rr][i].z), q(v[rr][i].w));
                    *reinterpret_cast<uint32_t *>(panel + (k / 32) * 1024 + ((k % 32) / 16) * 512 + (4 * wave + rr) * 16 +
                                                  (k % 16)) = w4;
                }
            }
        }
        __syncthreads();
    }
    // Residual values: with few column blocks per wave all of them are requested here, ahead of the main loop,
    // which hides them completely (and keeps loads from queueing behind the epilogue's stores: one counter).
    constexpr bool RES_EARLY = RESID && GS == 4;
    float res_all[RES_EARLY ? NBW : 1][16];
    if constexpr (RES_EARLY) {
#pragma unroll
        for (int jj = 0; jj < NBW; ++jj)
#pragma unroll
            for (int r = 0; r < 16; ++r) res_all[jj][r] = load_x(jj, r);
    }

    v16i acc[NBW];
#pragma unroll
    for (int j = 0; j < NBW; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0;

    if constexpr (AF32) {
        const int8_t *panel = &apanel[0][0];
        v4i a_cur = *reinterpret_cast<const v4i *>(panel + voff);
        for (int kl = 0; kl < KB; kl += U) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int nxt = kl + u + 1 < KB ? kl + u + 1 : KB - 1;
                const v4i a_nxt = *reinterpret_cast<const v4i *>(panel + nxt * 1024 + voff);
#pragma unroll
                for (int jj = 0; jj < NBW; ++jj) {
                    const int slot = (u * NBW + jj) % D;
                    acc[jj] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_cur, wf[slot], acc[jj], 0, 0, 0);
                    wf[slot] = load_w(kl + u + (jj + D) / NBW, (jj + D) % NBW);
                }
                a_cur = a_nxt;
            }
        }
    }
    const int stages = AF32 ? 0 : (KB + kRowsStage - 1) / kRowsStage;
    for (int s = 0; s < stages; ++s) {
        int8_t *buf = apanel[s & 1];
        // (the last reads of this buffer, two stages ago, lie before the previous stage's barrier)
#pragma unroll
        for (int i = 0; i < 3; ++i) *reinterpret_cast<v4i *>(buf + i * (kRowsThreads * 16) + tid * 16) = astage[i];
        __syncthreads();
        if (s + 1 < stages) load_stage(s + 1, astage);
        const int kb_first = s * kRowsStage;
        const int len = KB - kb_first < kRowsStage ? KB - kb_first : kRowsStage;  // (a multiple of 4)
        v4i a_cur = *reinterpret_cast<const v4i *>(buf + voff);
        for (int kl = 0; kl < len; kl += U) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int nxt = kl + u + 1 < kRowsStage ? kl + u + 1 : kRowsStage - 1;
                const v4i a_nxt = *reinterpret_cast<const v4i *>(buf + nxt * 1024 + voff);
                const int kb = kb_first + kl + u;
#pragma unroll
                for (int jj = 0; jj < NBW; ++jj) {
                    const int slot = (u * NBW + jj) % D;
                    acc[jj] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_cur, wf[slot], acc[jj], 0, 0, 0);
                    wf[slot] = load_w(kb + (jj + D) / NBW, (jj + D) % NBW);
                }
                a_cur = a_nxt;
            }
        }
    }

    // ---- epilogue: a 32 x 32 block has lane = column cin and register r = row 8 * (r / 4) + 4 * half + r % 4 ----
    // Instructions are what this part costs (the matrix pipe idles meanwhile), so everything that belongs to a row
    // rather than an element - the divisions of the mean, the variance, the scale and its reciprocal - is done by
    // ONE thread per row between two barriers, and handed to the row's lanes through LDS.
    auto row_of = [&](int r) { return 8 * (r / 4) + 4 * half + (r % 4); };
    // (through a copy: a bit cast applied to the element expression itself reads element 0 of the vector)
    auto value = [&](int jj, int r) {
        const int bits = acc[jj][r];
        return __builtin_bit_cast(float, bits);
    };
    // max(a, |b|) as fmaxf gives it for values that come out of arithmetic (a NaN b leaves a), in one instruction
    auto max_abs = [](float a, float b) {
        float o;
        asm("v_max_f32_e64 %0, %1, |%2|" : "=v"(o) : "v"(a), "v"(b));
        return o;
    };
    // Per-lane statistics of the rows of a pass -> one partial per wave and row in LDS.  MAX: non-negative values
    // that are no NaN, which order as their bit patterns do.
    auto partials_to_lds = [&](float(&t)[NR], int which, int g0, auto is_max) {
#pragma unroll
        for (int i = 0; i < NR; ++i) t[i] = half_wave_fold<decltype(is_max)::value>(t[i]);
        if (cin == 0) {
#pragma unroll
            for (int i = 0; i < NR; ++i) red[which][wave][row_of(4 * g0 + i)] = t[i];
        }
        __syncthreads();
    };
    // (one thread per row: tid < 8 * GS owns row 8 * g0 + tid of the panel)
    auto row_total = [&](int which, int row, auto is_max) {
        float w[kRowsWaves];
#pragma unroll
        for (int k = 0; k < kRowsWaves; ++k) w[k] = red[which][k][row];
        if constexpr (decltype(is_max)::value)
            return fmaxf(fmaxf(fmaxf(w[0], w[1]), fmaxf(w[2], w[3])), fmaxf(fmaxf(w[4], w[5]), fmaxf(w[6], w[7])));
        else
            return ((w[0] + w[1]) + (w[2] + w[3])) + ((w[4] + w[5]) + (w[6] + w[7]));
    };
    auto from_lds = [&](float(&t)[NR], int which, int g0) {
#pragma unroll
        for (int i = 0; i < NR; ++i) t[i] = fin[which][row_of(4 * g0 + i)];
    };
    const int KBo = p.N / 32;  // k blocks of the packed output (a multiple of 4 for the *_Q forms)
    const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc(
        QUANT ? p.out_q + size_t(rb) * KBo * 1024 : nullptr, 0, QUANT ? KBo * 1024 : 0, 0x00020000);
    const int qd = lane % 4;
    const uint32_t sel1 = (qd & 1) ? 0x03070105u : 0x06020400u, sel2 = (qd & 2) ? 0x03020706u : 0x05040100u;
    // after the byte exchange below a lane holds row 8 g + 4 half + qd, columns 4 * (cin / 4) .. + 3 of a block
    const int qoff = (4 * half + qd + 32 * (cin / 16)) * 16 + 4 * ((cin / 4) % 4);
    const float cols_f = static_cast<float>(p.N);

#pragma unroll
    for (int g0 = 0; g0 < 4; g0 += GS) {
        // rows of this pass: registers r = 4 * g0 + i, i < NR
        float s_row[NR];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const int m = m0 + row_of(4 * g0 + i);
            if constexpr (AF32)
                s_row[i] = sa_own[row_of(4 * g0 + i)];
            else
                s_row[i] = p.sa[p.sa_per_row ? (m < p.M ? m : p.M - 1) : 0];
        }
        // v = acc * (s_a * s_w) + bias (+ residual) (GELU), in place: the accumulator registers then hold float bits
        float sum[NR], am[NR];
#pragma unroll
        for (int i = 0; i < NR; ++i) sum[i] = am[i] = 0.0f;
#pragma unroll
        for (int jj = 0; jj < NBW; ++jj) {
            if (jb0 + jj >= nblocks) continue;  // (wave-uniform)
            const int col = (jb0 + jj) * 32 + cin;
            const float swv = p.sw[col];
            const float bv = p.bias ? p.bias[col] : -0.0f;  // (v + -0.0f is v, bit for bit)
            float res[NR];
            if constexpr (RESID) {
#pragma unroll
                for (int i = 0; i < NR; ++i) {
                    if constexpr (RES_EARLY)
                        res[i] = res_all[jj][4 * g0 + i];
                    else
                        res[i] = load_x(jj, 4 * g0 + i);
                }
            }
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                const int r = 4 * g0 + i;
                float v = static_cast<float>(acc[jj][r]) * (s_row[i] * swv) + bv;
                if constexpr (RESID) v = v + res[i];
                if constexpr (EPI == RP_GELU_Q) {
                    v = rp_gelu_tanh(v);
                    am[i] = max_abs(am[i], v);
                }
                if constexpr (EPI == RP_F32 || RESID)
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v), rf, (4 * half * p.N + col) * 4,
                                                          (8 * (r / 4) + (r % 4)) * row_bytes, EPI == RP_F32 ? 2 : 0);
                if constexpr (EPI == RP_RESID_LN_Q) sum[i] += v;
                acc[jj][r] = __builtin_bit_cast(int, v);
            }
        }
        if constexpr (QUANT) {
            if constexpr (EPI == RP_RESID_LN_Q) {
                // LayerNorm over the row (biased variance, eps inside the square root): passes over the registers
                partials_to_lds(sum, 0, g0, std::false_type{});
                if (tid < 8 * GS) fin[0][8 * g0 + tid] = row_total(0, 8 * g0 + tid, std::false_type{}) / cols_f;
                __syncthreads();
                float mean[NR], sq[NR];
                from_lds(mean, 0, g0);
#pragma unroll
                for (int i = 0; i < NR; ++i) sq[i] = 0.0f;
#pragma unroll
                for (int jj = 0; jj < NBW; ++jj) {
                    if (jb0 + jj >= nblocks) continue;
#pragma unroll
                    for (int i = 0; i < NR; ++i) {
                        const float d = value(jj, 4 * g0 + i) - mean[i];
                        sq[i] += d * d;
                    }
                }
                partials_to_lds(sq, 1, g0, std::false_type{});
                if (tid < 8 * GS)
                    fin[1][8 * g0 + tid] = 1.0f / sqrtf(row_total(1, 8 * g0 + tid, std::false_type{}) / cols_f + p.eps);
                __syncthreads();
                float rstd[NR];
                from_lds(rstd, 1, g0);
#pragma unroll
                for (int jj = 0; jj < NBW; ++jj) {
                    if (jb0 + jj >= nblocks) continue;
                    const int col = (jb0 + jj) * 32 + cin;
                    // (y * 1.0f and y + -0.0f are y, bit for bit)
                    const float g = p.gamma ? p.gamma[col] : 1.0f, b = p.beta ? p.beta[col] : -0.0f;
#pragma unroll
                    for (int i = 0; i < NR; ++i) {
                        const float y = (value(jj, 4 * g0 + i) - mean[i]) * rstd[i] * g + b;
                        am[i] = max_abs(am[i], y);
                        acc[jj][4 * g0 + i] = __builtin_bit_cast(int, y);
                    }
                }
            }
            // per-token symmetric int8: scale = max|v| / 127 (1 for an all-zero row, NaN for a row that is not
            // finite), q = clamp(round(v / scale)) with the row's reciprocal (calculate_symmetric_quantization_params
            // and the division form of quantize_per_channel_auto, as the row kernels apply them).  1 / scale is a
            // normal number for every scale this rule can give, or NaN with it; rows past M get a NaN scale here,
            // which makes their codes 0, as a NaN element's code is.
            partials_to_lds(am, 2, g0, std::true_type{});
            if (tid < 8 * GS) {
                const int row = 8 * g0 + tid;
                const float a = row_total(2, row, std::true_type{});
                float sc = a < FLT_EPSILON ? 1.0f : a / 127.0f;
                if (!(fabsf(a) <= FLT_MAX)) sc = NAN;
                if (m0 + row < p.M)
                    p.out_scales[m0 + row] = sc;
                else
                    sc = NAN;
                fin[2][row] = sc;
                fin[3][row] = 1.0f / sc;
            }
            __syncthreads();
            float scale[NR], inv[NR];
            from_lds(scale, 2, g0);
            from_lds(inv, 3, g0);
            // The codes, in the packed layout of the next product's activations: row block rb, k block = column
            // block, and inside the 1 KiB fragment slot (row + 32 * (column / 16)) of 16 bytes.  A lane holds one
            // column of four consecutive rows per register group; the four lanes of a quad transpose their 4 x 4
            // bytes (quad_byte_transpose) so that each holds four consecutive columns of ONE row: a dword.
#pragma unroll
            for (int jj = 0; jj < NBW; ++jj) {
                if (jb0 + jj >= nblocks) continue;
#pragma unroll
                for (int gi = 0; gi < GS; ++gi) {
                    int q[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const int i = 4 * gi + k;
                        // x / scale, correctly rounded, from the reciprocal (div_rn without its special cases: see above)
                        const float x = value(jj, 4 * g0 + i);
                        const float q0 = x * inv[i];
                        const float t = fmaf(fmaf(-q0, scale[i], x), inv[i], q0);
                        q[k] = row_code<EVEN>(t);
                    }
                    // byte k of the packed dword = row 8 g + 4 half + k; after the transpose: this lane's row, 4 columns
                    const uint32_t word = quad_byte_transpose(pack4(q[0], q[1], q[2], q[3]), sel1, sel2);
                    __builtin_amdgcn_raw_buffer_store_b32(static_cast<int>(word), rq, qoff,
                                                          (jb0 + jj) * 1024 + (g0 + gi) * 128, 0);
                }
            }
        }
    }
}

// ---- the same with a panel of 64 rows shared by a PAIR of compute units ----------------------------------------
// Every workgroup of gemm_i8_rows_kernel streams the whole weight matrix, which is what bounds its main loop
// (N * K bytes through a 57 B/clk path).  Here two workgroups on one XCD (ids b and b + 8, see hipq_gemm_pair.h)
// share 64 rows and take half of the columns each: a weight fragment feeds two MFMAs (one per row block), so the
// same matrix work needs half the weight stream per compute unit, and loop and MFMA time come level.  What the two
// halves of a row have to agree on - its maximum, its sum, its sum of squares - crosses through their XCD's L2 in
// one small exchange per statistic (64 floats each way, plain stores, then a flag word; the reader polls the flag
// past its L1, reads the partner's partials past its L1 and clears the flag, so every launch finds the flags zero
// and a captured launch can be replayed; a flag that does not come within the spin limit, or comes from another
// XCD, marks the context and the kernel runs on with defined values).  Both halves add the partials in the same
// order (columns' lower half first), so they hold the same bits.
// Results: the fp32 product, the skip connection, GELU and the per-token maxima are exactly those of the other
// forms; a LayerNorm's sums are folded in yet another order.
struct RowPairExchange {
    uint32_t *flags;  // four words per workgroup (three used: one per statistic)
    float *buf;       // three inboxes of 64 floats per workgroup
    uint32_t *wait_error;
    int spin_limit;
};

constexpr int kRowsPairStage = kRowsStage / 2;  // k blocks per LDS buffer and row block

template <int NBW, int EPI, bool EVEN>
__global__ __launch_bounds__(kRowsThreads) void gemm_i8_rows_pair_kernel(RowPanel p, RowPairExchange px) {
    constexpr int RB = 2;
    constexpr int D = NBW == 2 || NBW == 4 ? 8 : (NBW == 3 ? 12 : (NBW == 5 ? 10 : 6));  // weight fragments in flight per wave
    constexpr int U = D / rows_gcd(NBW, D);                // k blocks per trip of the main loop
    static_assert((U * NBW) % D == 0 && 4 % U == 0, "ring slots must be static; stages are multiples of 4 k blocks");
    constexpr bool QUANT = EPI == RP_GELU_Q || EPI == RP_RESID_LN_Q;
    constexpr bool RESID = EPI == RP_RESID_F32 || EPI == RP_RESID_LN_Q;
    __shared__ __attribute__((aligned(1024))) int8_t apanel[2][kRowsStage * 1024];  // [buffer][row block][k block]
    __shared__ __attribute__((aligned(16))) float red[3][kRowsWaves][64];           // [statistic][wave][row]
    __shared__ __attribute__((aligned(16))) float fin[4][64];  // per row: mean, 1 / std, scale, 1 / scale
    const int tid = threadIdx.x, lane = tid % kWave, half = lane / 32, cin = lane % 32;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int grp = blockIdx.x / 8;
    const int pair = (grp / 2) * 8 + blockIdx.x % 8, h = grp % 2;
    const int m0 = pair * 64;
    if (m0 >= p.M) return;  // (both workgroups of a pair)
    const int KB = static_cast<int>(packed_k_blocks(p.K));  // (a multiple of 4)
    const int nblocks = p.N / 32, nb2 = nblocks / 2;
    const int rbA = (p.M + 31) / 32, rb0 = pair * 2;
    // This wave's column blocks within the half: wave, wave + 8, wave + 16, ... (dealt round the waves, so that a
    // width that is no multiple of eight blocks leaves no wave idle), and within the matrix: jb(jj).
    auto mine_block = [&](int jj) { return wave + kRowsWaves * jj < nb2; };
    auto jb = [&](int jj) { return h * nb2 + wave + kRowsWaves * jj; };
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t *>(p.pa) + size_t(rb0) * KB * 1024, 0, (rbA - rb0 < 2 ? 1 : 2) * KB * 1024, 0x00020000);
    const __amdgpu_buffer_rsrc_t rw =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(p.pw), 0, nblocks * KB * 1024, 0x00020000);
    const int voff = lane * 16;
    const int wstride = KB * 1024;
    // (a block this wave does not have asks beyond the matrix: zeros, no memory access)
    int woff[NBW];
#pragma unroll
    for (int jj = 0; jj < NBW; ++jj) woff[jj] = mine_block(jj) ? jb(jj) * wstride : 0x7fffffff - 64 * 1024 * 1024;
    auto load_w = [&](int kb, int jj) {
        return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rw, voff, woff[jj] + kb * 1024, 0));
    };
    // one stage of the activation panel: 12 k blocks of both row blocks, three 16-byte pieces per thread
    int aoff[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        const int c = tid + i * kRowsThreads;  // 16-byte piece 0 .. 1535: row block c / 768
        aoff[i] = (c / 768) * KB * 1024 + (c % 768) * 16;
    }
    auto load_stage = [&](int s, v4i(&t)[3]) {
#pragma unroll
        for (int i = 0; i < 3; ++i)
            t[i] = __builtin_bit_cast(
                v4i, __builtin_amdgcn_raw_buffer_load_b128(ra, aoff[i], s * (kRowsPairStage * 1024), 0));
    };
    const int rows_here = p.M - m0 < 64 ? p.M - m0 : 64;
    const __amdgpu_buffer_rsrc_t rf = __builtin_amdgcn_make_buffer_rsrc(
        p.out_f ? reinterpret_cast<char *>(p.out_f) + size_t(m0) * p.N * 4 : nullptr, 0, p.out_f ? rows_here * p.N * 4 : 0,
        0x00020000);
    const int row_bytes = p.N * 4;
    auto load_x = [&](int rbk, int jj, int r) {
        return __builtin_bit_cast(
            float, __builtin_amdgcn_raw_buffer_load_b32(rf, (4 * half * p.N + jb(jj) * 32 + cin) * 4,
                                                        (32 * rbk + 8 * (r / 4) + (r % 4)) * row_bytes, 0));
    };
    // touch this workgroup's thirty-second of the weights (see gemm_i8_rows_kernel)
    {
        const int wbytes = nblocks * KB * 1024;
        const int chunk = ((wbytes + 31) / 32 + 127) & ~127;
        const int part = (blockIdx.x / 8) % 32;
        int touched = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int off = (tid + i * kRowsThreads) * 128;
            if (off < chunk) touched ^= __builtin_amdgcn_raw_buffer_load_b32(rw, off, part * chunk, 0);
        }
        if (touched == 0x5a5a5a5a && p.M < 0) red[0][0][0] = 1.0f;  // (keeps the loads alive; never true)
    }
    v4i wf[D];
#pragma unroll
    for (int u = 0; u < D; ++u) wf[u] = load_w(u / NBW, u % NBW);
    v4i astage[3];
    load_stage(0, astage);
    constexpr bool RES_EARLY = RESID && NBW <= 3;
    float res_all[RES_EARLY ? RB : 1][RES_EARLY ? NBW : 1][16];
    if constexpr (RES_EARLY) {
#pragma unroll
        for (int rbk = 0; rbk < RB; ++rbk)
#pragma unroll
            for (int jj = 0; jj < NBW; ++jj)
#pragma unroll
                for (int r = 0; r < 16; ++r) res_all[rbk][jj][r] = load_x(rbk, jj, r);
    }

    v16i acc[RB][NBW];
#pragma unroll
    for (int rbk = 0; rbk < RB; ++rbk)
#pragma unroll
        for (int j = 0; j < NBW; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[rbk][j][r] = 0;

    const int stages = (KB + kRowsPairStage - 1) / kRowsPairStage;
    for (int s = 0; s < stages; ++s) {
        int8_t *buf = apanel[s & 1];
#pragma unroll
        for (int i = 0; i < 3; ++i) *reinterpret_cast<v4i *>(buf + i * (kRowsThreads * 16) + tid * 16) = astage[i];
        __syncthreads();
        if (s + 1 < stages) load_stage(s + 1, astage);
        const int kb_first = s * kRowsPairStage;
        const int len = KB - kb_first < kRowsPairStage ? KB - kb_first : kRowsPairStage;  // (a multiple of 4)
        v4i a0 = *reinterpret_cast<const v4i *>(buf + voff);
        v4i a1 = *reinterpret_cast<const v4i *>(buf + kRowsPairStage * 1024 + voff);
        for (int kl = 0; kl < len; kl += U) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int nxt = kl + u + 1 < kRowsPairStage ? kl + u + 1 : kRowsPairStage - 1;
                const v4i n0 = *reinterpret_cast<const v4i *>(buf + nxt * 1024 + voff);
                const v4i n1 = *reinterpret_cast<const v4i *>(buf + (kRowsPairStage + nxt) * 1024 + voff);
                const int kb = kb_first + kl + u;
#pragma unroll
                for (int jj = 0; jj < NBW; ++jj) {
                    const int slot = (u * NBW + jj) % D;
                    acc[0][jj] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, wf[slot], acc[0][jj], 0, 0, 0);
                    acc[1][jj] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, wf[slot], acc[1][jj], 0, 0, 0);
                    wf[slot] = load_w(kb + (jj + D) / NBW, (jj + D) % NBW);
                }
                a0 = n0;
                a1 = n1;
            }
        }
    }

    // ---- epilogue (see gemm_i8_rows_kernel; rows 32 * rbk + row_of(r), statistics for all 64 rows at once) ----
    auto row_of = [&](int r) { return 8 * (r / 4) + 4 * half + (r % 4); };
    auto value = [&](int rbk, int jj, int r) {
        const int bits = acc[rbk][jj][r];
        return __builtin_bit_cast(float, bits);
    };
    auto max_abs = [](float a, float b) {
        float o;
        asm("v_max_f32_e64 %0, %1, |%2|" : "=v"(o) : "v"(a), "v"(b));
        return o;
    };
    auto partials_to_lds = [&](float(&t)[RB][16], int which, auto is_max) {
#pragma unroll
        for (int rbk = 0; rbk < RB; ++rbk)
#pragma unroll
            for (int r = 0; r < 16; ++r) t[rbk][r] = half_wave_fold<decltype(is_max)::value>(t[rbk][r]);
        if (cin == 0) {
#pragma unroll
            for (int rbk = 0; rbk < RB; ++rbk)
#pragma unroll
                for (int r = 0; r < 16; ++r) red[which][wave][32 * rbk + row_of(r)] = t[rbk][r];
        }
        __syncthreads();
    };
    // Wave 0, one lane per row: this half's statistic of the row, then the pair's.
    auto row_total = [&](int which, int round, auto is_max) {
        constexpr bool MAX = decltype(is_max)::value;
        float w[kRowsWaves];
#pragma unroll
        for (int k = 0; k < kRowsWaves; ++k) w[k] = red[which][k][tid];
        const float local = MAX ? fmaxf(fmaxf(fmaxf(w[0], w[1]), fmaxf(w[2], w[3])), fmaxf(fmaxf(w[4], w[5]), fmaxf(w[6], w[7])))
                                : ((w[0] + w[1]) + (w[2] + w[3])) + ((w[4] + w[5]) + (w[6] + w[7]));
        const size_t me = size_t(pair) * 2 + h, partner = size_t(pair) * 2 + (1 - h);
        px.buf[(partner * 3 + round) * 64 + tid] = local;  // (a plain store: it lands in the XCD's L2)
        asm volatile("" ::: "memory");
        wait_vmcnt<0>();
        asm volatile("" ::: "memory");
        const uint32_t mine = 0x100u | xcc_id();
        if (lane == 0) __hip_atomic_store(px.flags + partner * 4 + round, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        uint32_t *flag = px.flags + me * 4 + round;
        uint32_t seen = 0;
        for (int spin = 0; spin <= px.spin_limit; ++spin) {
            seen = __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (seen != 0) break;
            __builtin_amdgcn_s_sleep(1);
        }
        seen = __builtin_amdgcn_readfirstlane(seen);
        float other = MAX ? 0.0f : 0.0f;
        if (seen == mine) {
            asm volatile("" ::: "memory");
            const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(
                px.buf + (me * 3 + round) * 64, 0, 64 * 4, 0x00020000);
            other = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rx, tid * 4, 0, /*sc1*/ 16));
        } else if (lane == 0) {
            // nothing came within the limit, or it came from another XCD, whose stores this L2 does not hold
            __hip_atomic_store(px.wait_error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (lane == 0 && seen != 0) __hip_atomic_store(flag, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if constexpr (MAX) return fmaxf(local, other);
        return h == 0 ? local + other : other + local;
    };
    auto from_lds = [&](float(&t)[16], int which, int rbk) {
#pragma unroll
        for (int r = 0; r < 16; ++r) t[r] = fin[which][32 * rbk + row_of(r)];
    };
    const int KBo = p.N / 32;
    const int qd = lane % 4;
    const uint32_t sel1 = (qd & 1) ? 0x03070105u : 0x06020400u, sel2 = (qd & 2) ? 0x03020706u : 0x05040100u;
    const int qoff = (4 * half + qd + 32 * (cin / 16)) * 16 + 4 * ((cin / 4) % 4);
    const float cols_f = static_cast<float>(p.N);

    // v = acc * (s_a * s_w) + bias (+ residual) (GELU), in place
    float sum[RB][16], am[RB][16];
#pragma unroll
    for (int rbk = 0; rbk < RB; ++rbk) {
        float s_row[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = m0 + 32 * rbk + row_of(r);
            s_row[r] = p.sa[p.sa_per_row ? (m < p.M ? m : p.M - 1) : 0];
            sum[rbk][r] = am[rbk][r] = 0.0f;
        }
#pragma unroll
        for (int jj = 0; jj < NBW; ++jj) {
            if (!mine_block(jj)) continue;  // (wave-uniform)
            const int col = jb(jj) * 32 + cin;
            const float swv = p.sw[col];
            const float bv = p.bias ? p.bias[col] : -0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float v = static_cast<float>(acc[rbk][jj][r]) * (s_row[r] * swv) + bv;
                if constexpr (RESID) {
                    if constexpr (RES_EARLY)
                        v = v + res_all[rbk][jj][r];
                    else
                        v = v + load_x(rbk, jj, r);
                }
                if constexpr (EPI == RP_GELU_Q) {
                    v = rp_gelu_tanh(v);
                    am[rbk][r] = max_abs(am[rbk][r], v);
                }
                if constexpr (EPI == RP_F32 || RESID)
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v), rf, (4 * half * p.N + col) * 4,
                                                          (32 * rbk + 8 * (r / 4) + (r % 4)) * row_bytes,
                                                          EPI == RP_F32 ? 2 : 0);
                if constexpr (EPI == RP_RESID_LN_Q) sum[rbk][r] += v;
                acc[rbk][jj][r] = __builtin_bit_cast(int, v);
            }
        }
    }
    if constexpr (QUANT) {
        if constexpr (EPI == RP_RESID_LN_Q) {
            partials_to_lds(sum, 0, std::false_type{});
            if (wave == 0) fin[0][tid] = row_total(0, 0, std::false_type{}) / cols_f;
            __syncthreads();
            float sq[RB][16];
#pragma unroll
            for (int rbk = 0; rbk < RB; ++rbk) {
                float mean[16];
                from_lds(mean, 0, rbk);
#pragma unroll
                for (int r = 0; r < 16; ++r) sq[rbk][r] = 0.0f;
#pragma unroll
                for (int jj = 0; jj < NBW; ++jj) {
                    if (!mine_block(jj)) continue;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const float d = value(rbk, jj, r) - mean[r];
                        sq[rbk][r] += d * d;
                    }
                }
            }
            partials_to_lds(sq, 1, std::false_type{});
            if (wave == 0) fin[1][tid] = 1.0f / sqrtf(row_total(1, 1, std::false_type{}) / cols_f + p.eps);
            __syncthreads();
#pragma unroll
            for (int rbk = 0; rbk < RB; ++rbk) {
                float mean[16], rstd[16];
                from_lds(mean, 0, rbk);
                from_lds(rstd, 1, rbk);
#pragma unroll
                for (int jj = 0; jj < NBW; ++jj) {
                    if (!mine_block(jj)) continue;
                    const int col = jb(jj) * 32 + cin;
                    const float g = p.gamma ? p.gamma[col] : 1.0f, b = p.beta ? p.beta[col] : -0.0f;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const float y = (value(rbk, jj, r) - mean[r]) * rstd[r] * g + b;
                        am[rbk][r] = max_abs(am[rbk][r], y);
                        acc[rbk][jj][r] = __builtin_bit_cast(int, y);
                    }
                }
            }
        }
        partials_to_lds(am, 2, std::true_type{});
        if (wave == 0) {
            const float a = row_total(2, 2, std::true_type{});
            float sc = a < FLT_EPSILON ? 1.0f : a / 127.0f;
            if (!(fabsf(a) <= FLT_MAX)) sc = NAN;
            if (m0 + tid < p.M) {
                if (h == 0) p.out_scales[m0 + tid] = sc;
            } else {
                sc = NAN;  // rows past M: codes 0
            }
            fin[2][tid] = sc;
            fin[3][tid] = 1.0f / sc;
        }
        __syncthreads();
#pragma unroll
        for (int rbk = 0; rbk < RB; ++rbk) {
            float scale[16], inv[16];
            from_lds(scale, 2, rbk);
            from_lds(inv, 3, rbk);
            const bool there = rb0 + rbk < rbA;  // (the packed output has no row block past the matrix)
            const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc(
                p.out_q + size_t(there ? rb0 + rbk : 0) * KBo * 1024, 0, there ? KBo * 1024 : 0, 0x00020000);
#pragma unroll
            for (int jj = 0; jj < NBW; ++jj) {
                if (!mine_block(jj)) continue;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    int q[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const int r = 4 * g + k;
                        const float x = value(rbk, jj, r);
                        const float q0 = x * inv[r];
                        const float t = fmaf(fmaf(-q0, scale[r], x), inv[r], q0);
                        q[k] = row_code<EVEN>(t);
                    }
                    const uint32_t word = quad_byte_transpose(pack4(q[0], q[1], q[2], q[3]), sel1, sel2);
                    __builtin_amdgcn_raw_buffer_store_b32(static_cast<int>(word), rq, qoff, jb(jj) * 1024 + g * 128, 0);
                }
            }
        }
    }
}

// The pair form where it applies and pays: the device's workgroup pairs share an XCD, the whole grid is resident at
// once (one workgroup per compute unit of the context's share), N a multiple of 64 and at most 3072.  An exchange
// of row statistics costs about 2 us, and a workgroup's epilogue handles twice the rows, which the halved weight
// stream pays back when all eight waves have columns to work on (N >= 1536) and, for the three exchanges of a LayerNorm,
// when the matrix is large (N * K >= 2 Mi).  At M = 8192, K = 768 (3072 for N = 768), pairs against single panels,
// in us: fp32 11.0 / 11.7 (N = 768), 18.3 / 21.9 (1536), 26.6 / 32.1 (2304), 35.9 / 43.6 (3072), 26.1 / 29.8
// (768 x 3072); GELU + quantize 15.8 / 13.8, 22.4 / 24.0, 37.9 / 37.2, 40.1 / 48.4, 33.3 / 31.8; skip + LayerNorm +
// quantize 38.4 / 38.1 (1536), 60.8 / 60.7 (2304), 95.3 / 112.9 (3072), 43.6 / 41.2 (768 x 3072); skip alone 14.8 /
// 15.8 (768), 32.8 / 36.1 (768 x 3072), 76.2 / 57.0 (3072: the stream is then read inside the epilogue, value by
// value, by waves that hold twice the rows).  With the waits switched off (spin limit 0) the times are the same to
// 0.5 us: what an exchange costs is its own chain of L2 trips (store, acknowledge, flag, poll, read), not the
// partners' skew.  Raising the issue priority of one of the two waves of every SIMD during the main loop, so that
// its epilogue would overlap the other's loads and MFMAs, changes nothing (41.6 / 41.7 us at N = 3072 with GELU +
// quantize): the waves advance at the rate their loads return.
// Halving K instead of the columns between the partners (each multiplies both row blocks by its half of the weights,
// then every wave hands the partial sums of the partner's row block - 12 KiB a wave, 96 KiB a workgroup - to the
// partner's wave of the same columns and adds what it receives; integer sums, so bit-identical whatever the
// epilogue) was built for N <= 768 and measured: 36.7 against 32.9 us (fp32) and 44.2 against 43.0 us (skip +
// LayerNorm + quantize) at 768 x 3072, 21.6 against 12.8 us at 768 x 768.  The exchange of 24 MB through the L2s
// costs ~9 us, more than the halved weight stream saves (~5 us at K = 3072).
// Test hook 15 keeps the single-workgroup panels, 16 takes pairs wherever the shape allows them.  Returns false
// when the caller should launch the single panels.
template <int EPI>
static bool launch_rows_pair(hipq_ctx *ctx, const RowPanel &p, bool even, int32_t *rc) {
    const int share = ctx->resident_share > 0 ? ctx->resident_share : 1;
    const int pairs = (p.M + 63) / 64, grid = (pairs + 7) / 8 * 16;
    if (!ctx->pair_ok || ctx->gemm_variant == 15 || p.N % 64 != 0 || p.M <= 32 || grid > ctx->num_cus / share) return false;
    if (ctx->gemm_variant != 16) {
        if ((EPI == RP_GELU_Q || EPI == RP_RESID_LN_Q) && p.N < 1536) return false;
        if (EPI == RP_RESID_F32 && p.N > 1536) return false;
        if (EPI == RP_RESID_LN_Q && size_t(p.N) * p.K < (size_t(2) << 20)) return false;
    }
    RowPairExchange px;
    int8_t *buf = nullptr;
    *rc = pair_area(ctx, size_t(grid) * 4 * sizeof(uint32_t), size_t(grid) * 3 * 64 * sizeof(float), &px.flags, &buf);
    if (*rc) return true;
    px.buf = reinterpret_cast<float *>(buf);
    px.wait_error = ctx->wait_error;
    px.spin_limit = ctx->wait_spin_limit;
    const int nbw = (p.N / 64 + kRowsWaves - 1) / kRowsWaves;
#define HIPQ_LAUNCH_ROWS_PAIR(NBW)                                                                                        \
    do {                                                                                                                  \
        if (even)                                                                                                         \
            hipLaunchKernelGGL((gemm_i8_rows_pair_kernel<NBW, EPI, true>), dim3(grid), dim3(kRowsThreads), 0, ctx->stream, \
                               p, px);                                                                                    \
        else                                                                                                              \
            hipLaunchKernelGGL((gemm_i8_rows_pair_kernel<NBW, EPI, false>), dim3(grid), dim3(kRowsThreads), 0,            \
                               ctx->stream, p, px);                                                                       \
    } while (0)
    constexpr bool QUANT = EPI == RP_GELU_Q || EPI == RP_RESID_LN_Q;
    if (nbw <= 2) {
        HIPQ_LAUNCH_ROWS_PAIR(2);
    } else if (nbw <= 3) {
        HIPQ_LAUNCH_ROWS_PAIR(3);
    } else if (nbw <= 5 && !QUANT) {  // (the quantizing forms of these widths run with six, one or two blocks of zeros)
        if constexpr (!QUANT) {
            if (nbw == 4)
                HIPQ_LAUNCH_ROWS_PAIR(4);
            else
                HIPQ_LAUNCH_ROWS_PAIR(5);
        }
    } else {
        HIPQ_LAUNCH_ROWS_PAIR(6);
    }
#undef HIPQ_LAUNCH_ROWS_PAIR
    *rc = check_launch("gemm_i8 (row panels, pairs)");
    return true;
}

// Launch of the row-panel kernel that quantizes its own fp32 activations (gemm_i8_rows_kernel<.., AF32>): single
// panels, the whole panel of codes resident in LDS.
template <int EPI>
static int32_t launch_rows_from_f32(hipq_ctx *ctx, const RowPanel &p, bool even) {
    constexpr bool QUANT = EPI == RP_GELU_Q || EPI == RP_RESID_LN_Q;
    if (p.N % 32 != 0 || p.N > 1536 || p.N <= 0 || p.M <= 0 || p.K <= 0 || (QUANT && p.N % 128 != 0))
        return fail(HIPQ_SHAPE_ERROR,
                    "row-panel GEMM from fp32 rows: N = %d must be a multiple of 32 (of 128 for a packed int8 output) "
                    "and at most 1536", p.N);
    if (p.K > 1536 || p.K % 4 != 0 || p.lda % 4 != 0 || p.lda < p.K || (reinterpret_cast<uintptr_t>(p.af) & 15u))
        return fail(HIPQ_SHAPE_ERROR,
                    "row-panel GEMM from fp32 rows: K = %d (at most 1536) and the row pitch %d must be multiples of 4, "
                    "the rows 16-byte aligned", p.K, p.lda);
    const dim3 grid((p.M + 31) / 32);
    const int nbw = (p.N / 32 + kRowsWaves - 1) / kRowsWaves;
#define HIPQ_LAUNCH_ROWS_F32(NBW)                                                                                         \
    do {                                                                                                                  \
        if (even)                                                                                                         \
            hipLaunchKernelGGL((gemm_i8_rows_kernel<NBW, EPI, true, true>), grid, dim3(kRowsThreads), 0, ctx->stream, p); \
        else                                                                                                              \
            hipLaunchKernelGGL((gemm_i8_rows_kernel<NBW, EPI, false, true>), grid, dim3(kRowsThreads), 0, ctx->stream,    \
                               p);                                                                                        \
    } while (0)
    if (nbw <= 3)
        HIPQ_LAUNCH_ROWS_F32(3);
    else
        HIPQ_LAUNCH_ROWS_F32(6);
#undef HIPQ_LAUNCH_ROWS_F32
    return check_launch("gemm_i8 (row panels, fp32 activations)");
}

// Launch of the row-panel kernel: one workgroup of eight waves per 32 rows.  Returns HIPQ_SHAPE_ERROR for what it
// does not take (N not a multiple of 32 or above 3072; the *_Q forms: N not a multiple of 128).
template <int EPI>
static int32_t launch_rows(hipq_ctx *ctx, const RowPanel &p, bool even) {
    if (p.N % 32 != 0 || p.N > 3072 || p.N <= 0 || p.M <= 0 || p.K <= 0)
        return fail(HIPQ_SHAPE_ERROR, "row-panel GEMM: N = %d must be a multiple of 32 and at most 3072", p.N);
    constexpr bool QUANT = EPI == RP_GELU_Q || EPI == RP_RESID_LN_Q;
    if (QUANT && p.N % 128 != 0)
        return fail(HIPQ_SHAPE_ERROR, "row-panel GEMM: N = %d must be a multiple of 128 for a packed int8 output", p.N);
    // (offsets of column blocks past N, which read as zeros, are still computed: price the widest panel)
    if (packed_bytes(size_t(3072), size_t(p.K)) >= (size_t(1) << 31))
        return fail(HIPQ_SHAPE_ERROR, "row-panel GEMM: K = %d is too large (32-bit offsets into the weights)", p.K);
    {
        int32_t rc = HIPQ_SUCCESS;
        if (launch_rows_pair<EPI>(ctx, p, even, &rc)) return rc;
    }
    const dim3 grid((p.M + 31) / 32);
    const int nbw = (p.N / 32 + kRowsWaves - 1) / kRowsWaves;
#define HIPQ_LAUNCH_ROWS_NBW(NBW)                                                                                     \
    do {                                                                                                              \
        if (even)                                                                                                     \
            hipLaunchKernelGGL((gemm_i8_rows_kernel<NBW, EPI, true>), grid, dim3(kRowsThreads), 0, ctx->stream, p);  \
        else                                                                                                          \
            hipLaunchKernelGGL((gemm_i8_rows_kernel<NBW, EPI, false>), grid, dim3(kRowsThreads), 0, ctx->stream, p); \
    } while (0)
    if (nbw <= 3)
        HIPQ_LAUNCH_ROWS_NBW(3);
    else if (nbw <= 6)
        HIPQ_LAUNCH_ROWS_NBW(6);
    else if (nbw <= 9)
        HIPQ_LAUNCH_ROWS_NBW(9);
    else
        HIPQ_LAUNCH_ROWS_NBW(12);
#undef HIPQ_LAUNCH_ROWS_NBW
    return check_launch("gemm_i8 (row panels)");
}

}  // namespace hipq
