/*
 * cybq_debug.h - diagnostics exported by libcybq.so for the tests and the benchmark of this
 * repository.  NOT part of the operator interface (include/cybq.h): nothing a runtime binds,
 * no stability promise.  The tuning override is process-wide mutable state; use it from one
 * thread, with no launches in flight.
 */
#ifndef CYBQ_DEBUG_H
#define CYBQ_DEBUG_H

#include "../../include/cybq.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Overrides the decode kernels' launch heuristics for experiments: waves per
 * workgroup (1..16); which decode kernel runs (0 automatic, 1 always the
 * x-in-registers kernel, 2 never); tiles in flight per wave of the streaming
 * variant (2 or 4).  0 restores the automatic choice.  Any non-zero value also keeps
 * one-row calls away from the kernel of gemv1.hip. */
int cybq_debug_set_gemv_tuning(int waves_per_group, int rows_kernel, int unroll);

/* Which prefill kernel takes calls of up to 512 rows in FAST mode: 0 automatic (the kernel whose waves
 * split K where its workgroups of up to 64 rows fit one round of CUs and fill a quarter of it), 1 that kernel for
 * up to 64 rows whatever the width, 2 never that kernel (the tiled kernels - on small weights at up to 64 rows two
 * passes of the batched-rows decode kernel - take the call as they do for other shapes); 5: automatic, but the
 * staging launch asks for no weights ahead of the multiply; 6: automatic, it asks only ahead of that kernel. */
int cybq_debug_set_gemm_tuning(int rows_kernel);

/* Ceiling probes for the one-row decode kernel: a kernel that issues exactly that kernel's
 * memory requests for tensor `w` (one workgroup per 16-row strip, whole strip requested up
 * front) and does nothing with the data.
 *   with_io = 0  weights and scales only, nothing stored
 *   with_io = 1  also reads the activations x [K] f16 the way the kernel does and stores
 *                16 floats per strip to y [N]
 * `count` launches back to back, one per tensor of w[] (like cybq_matmul_many).
 * Needs K a multiple of 512 and at most 16384. */
int cybq_debug_read_weight(cybq_ctx* ctx, int64_t count, const cybq_weight* const* w, int with_io, const void* x, void* y,
                           void* stream);

/* The same bytes read in other ways, again with nothing done to the data: how long a launch that only
 * reads the tensor takes, whatever its decomposition.  `count` launches back to back, one per tensor.
 *   pattern 1  a strip per workgroup as in the decode kernel, but 4 waves x 2 sets (Q4, K = 4096 only)
 *   pattern 2  a strip per workgroup, 2 waves x 4 sets (Q4, K = 4096 only)
 *   pattern 3  flat: every wave reads one contiguous 8 KiB, all of it requested at once, one round
 *   pattern 4  persistent grid: one 16-wave workgroup per CU walks the tensor 4 KiB per wave and round
 *   pattern 5  persistent grid with the next chunk requested before the current one is consumed
 *   pattern 6  flat, 4 KiB per wave straight into LDS (no registers held while a request is in flight) */
int cybq_debug_read_pattern(cybq_ctx* ctx, int64_t count, const cybq_weight* const* w, int pattern, void* stream);

/* A loop of independent v_mfma_f32_16x16x32_f16 on every SIMD of the chip: `waves_per_simd`
 * waves each issue `iters` x 16 instructions.  flops = CUs * 4 * waves_per_simd * iters * 16 * 16384.
 * waves_per_simd = 0: one wave per SIMD issues `iters` x 8 independent v_mfma_f32_32x32x16_f16 instead
 * (flops = CUs * 4 * iters * 8 * 32768). */
int cybq_debug_mfma_loop(cybq_ctx* ctx, int waves_per_simd, int iters, float* sink, void* stream);

/* How fast the CUs take in bytes that sit in the L2: one workgroup of `waves` waves per CU, every workgroup
 * reads the same `bytes` at `buf` (device memory, a multiple of in_flight KiB, at most 1 GiB) `iters` times with
 * 1 KiB per wave instruction and `in_flight` (4, 8 or 16) instructions outstanding per wave; nothing is stored.
 * Bytes into the CUs = CUs * bytes * iters. */
int cybq_debug_cache_read(cybq_ctx* ctx, const void* buf, int64_t bytes, int waves, int in_flight, int iters, void* stream);

#ifdef __cplusplus
}
#endif
#endif
