/*
 * torsh_hipq - test and tuning hooks of the library.  None of them has a counterpart in the
 * reference and none belongs to the surface a binding exposes: a maintainer's FFI crate binds
 * include/torsh_hipq.h only (the generated Rust declarations leave this file out).  They exist so
 * that the parity tests can run every kernel form on the same inputs, see the error path of a
 * bounded wait without hanging anything, and read the kernels' own phase stamps.  Results never
 * depend on them.  No environment variable changes which kernels run.
 */
#ifndef TORSH_HIPQ_TESTING_H
#define TORSH_HIPQ_TESTING_H

#include "torsh_hipq.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Forces one of the GEMM kernel forms for every later call on this context wherever the shape
 * allows it (0 = automatic choice, the default; 1-3 one-tile-per-workgroup forms, 5-8 persistent
 * forms, 10 register-staged form); 6 also makes the dynamic per-tensor activation quantizer of the
 * Linear forwards run as two launches (range partials, then a quantizer that folds them) where it
 * would run as one, and the per-token forward of one or two rows as a quantizer and a product where
 * it would be one kernel; 9 and 11 leave the choice automatic and switch off, on prepared operands,
 * the forms of the GEMM that are picked by occupancy - two workgroups per compute unit, the
 * weight-streaming kernel for 33..128 rows - (9) and the touching of weight / filter lines by the
 * one-launch activation quantizers of the dynamic Linear and Conv2d forwards while their grids wait
 * for the range (11); 12 runs shapes of whole 128 x 128 tiles that fill the device once as one tile
 * per PAIR of compute units, K halved between the two, partial sums exchanged through their XCD's L2
 * (measured slower than the default forms; kept as a measured alternative); 14 runs a Conv2d
 * forward on a uint8 input of 128 or 256 channels and small planes as ONE launch whose workgroups
 * gather their own patches of the image into LDS (measured no faster than the layout pass + implicit
 * GEMM it would replace; kept as a measured alternative); 15 makes the row-panel forwards (the
 * Linear forwards with a row operation in their epilogue) keep one workgroup per 32 rows where they
 * would let two workgroups of an XCD share 64 rows and half of the columns each; 16 makes them take
 * such pairs wherever the shape allows it, also where the single panels were measured faster. */
HIPQ_API int32_t hipq_set_gemm_kernel_variant(hipq_ctx *ctx, int32_t variant);
/* Some kernels couple their waves through device memory: the persistent GEMM kernel (counters
 * between producer and consumer waves), the one-launch dynamic quantizers (their workgroups meet to
 * agree on the range), the GEMM form whose workgroup pairs exchange partial sums and the row-panel
 * forwards whose workgroup pairs exchange row maxima and sums.  All bound
 * every wait, so that a grid always drains; a wait that gives up marks the context, and the next
 * hipq_ctx_synchronize returns HIPQ_DEVICE_ERROR once instead of handing back a wrong result
 * silently (the quantizers also leave zero codes, a NaN scale and status HIPQ_DEVICE_ERROR in
 * out_params).  `limit` is the number of polls after the first look (negative = the default, 2^20);
 * 0 lets a test see the error path without hanging anything. */
HIPQ_API int32_t hipq_ctx_set_wait_spin_limit(hipq_ctx *ctx, int32_t limit);
/* While a device buffer is set, hipq_linear_packed_i8_f32 (and the forwards built on it) run a
 * form of the packed GEMM kernel in which every wave records the shader clock at six points -
 * start, first operands in registers, end of the K loop, partial sums reduced, stores issued,
 * stores retired - followed by the constant 100 MHz counter at the first and the last point, as
 * uint64 values [workgroup][wave 0..3][8], provided the buffer holds one such record per wave of
 * the grid (otherwise the ordinary kernel runs).  The results are the same bits.  null removes the
 * buffer.  bench.py --profile gemm_phases prints the phase table from it. */
HIPQ_API int32_t hipq_ctx_set_trace_buffer(hipq_ctx *ctx, void *device_buffer, size_t bytes);

/* Machine probe: what a compute unit's vector-memory path and matrix pipes deliver, by the kernel's own clocks.
 * `workgroups` workgroups of four waves; every step a wave requests `loads_per_step` fragments of 1 KiB (one
 * coalesced 16-byte-per-lane load each, as the packed GEMM does) and issues `mfmas_per_step`
 * v_mfma_i32_32x32x32_i8; (loads, MFMAs) one of (6,0) (8,0) (0,8) (0,16) (6,8) (8,16) (4,8); `steps` even.  The
 * workgroups walk regions of `region_bytes` (a power of two) of `buf` round and round, `share` workgroups of one XCD
 * per region.  out (device): per workgroup {shader-clock cycles, 100 MHz ticks, checksum} as uint64.
 * bench.py --profile vmem_path prints the table. */
HIPQ_API int32_t hipq_probe_vector_memory_path(hipq_ctx *ctx, const int8_t *buf, size_t buf_bytes, int32_t workgroups,
                                               int32_t region_bytes, int32_t share, int32_t loads_per_step,
                                               int32_t mfmas_per_step, int32_t steps, uint64_t *out);

/* Machine probe: one wave accesses a raw buffer descriptor of `extent` bytes over `mem` with the scalar offset
 * `soffset`: lane l loads the dword at byte 4 l + soffset into loaded[l] (64 x int32, device), then stores 0x7777
 * there.  The row-panel GEMM kernels rely on accesses past the extent reading as zero and being dropped, scalar
 * offset included; every address the wave could reach must lie inside mem (soffset + 256 <= mem_bytes), so the
 * probe is safe whatever the hardware does. */
HIPQ_API int32_t hipq_probe_buffer_range_check(hipq_ctx *ctx, int32_t *mem, size_t mem_bytes, int32_t extent,
                                               int32_t soffset, int32_t *loaded);

#ifdef __cplusplus
}
#endif

#endif /* TORSH_HIPQ_TESTING_H */
