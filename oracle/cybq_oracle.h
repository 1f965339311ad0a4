/*
 * cybq_oracle.h - CPU restatement of cyb's block-quantized matmul path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this code; only the test-suite, the smoke check and the cpu_baseline
 * leg of the benchmark do, and only as the checker / the CPU number printed
 * beside the GPU number.
 *
 * What it restates.  The operator itself (crate `run`, reached by cyb as the
 * path dependency `../glia/run`, /root/reference/Cargo.lock:8443-8462) is not
 * part of the reference tree, so no line of its arithmetic can be cited.  The
 * restatement follows what the tree does pin:
 *   - tensor data kinds Q4/Q8/F16/F32          decide/pipeline.md:28
 *   - weights named HF style, [out,in] = [N,K] decide/pipeline.md:30
 *   - import-time quantisation to Q4_0          decide/pipeline.md:38-40,59
 *   - Q8 = 8.5 bit per weight (34 B / 32 w)     shell/src/worlds/models/mod.rs:69-73
 *   - one op invocation per linear per token    decide/pipeline.md:51
 * and the workload definition this build was given: groups of 32 along K, one
 * f16 absmax scale per group, 4-bit signed two-per-byte (Q4) or int8 (Q8),
 * fp32 accumulation.
 *
 * Parity status of each function (what pins it, see tests/test_oracle_*.py):
 *   f16/bf16 conversions   pinned: exhaustive / tie cases against numpy.float16
 *   dequant                pinned: closed form, exact in f32 (11-bit x 8-bit)
 *   pack / unpack          pinned: exhaustive over byte values, hand vectors
 *   gemm (f32 and f64)     pinned: reduces to numpy float64 matmul
 *   quantize               PARITY UNPINNED against the reference: the scale
 *                          divisor (absmax/qmax), rounding mode and clamp are
 *                          this build's choice; pinned only against the
 *                          invariants the definition implies.
 *   interchange layouts    PARITY UNPINNED against the reference: nibble order,
 *                          signedness encoding and block order are this build's
 *                          choice (BLOCK_AOS follows the public GGML Q4_0/Q8_0
 *                          block shape that decide/pipeline.md:38 names).
 */
#ifndef CYBQ_ORACLE_H
#define CYBQ_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CYBQ_ORACLE_GROUP 32

/* ---- scalar conversions (IEEE-754 binary16 / bfloat16, round-to-nearest-even) */
float    cybq_oracle_f16_to_f32(uint16_t h);
uint16_t cybq_oracle_f32_to_f16(float f);
float    cybq_oracle_bf16_to_f32(uint16_t h);
uint16_t cybq_oracle_f32_to_bf16(float f);
void cybq_oracle_f16_to_f32_n(const uint16_t* h, float* out, size_t n);
void cybq_oracle_f32_to_f16_n(const float* f, uint16_t* out, size_t n);
void cybq_oracle_bf16_to_f32_n(const uint16_t* h, float* out, size_t n);
void cybq_oracle_f32_to_bf16_n(const float* f, uint16_t* out, size_t n);

/* ---- quantise (import stage).  bits = 4 or 8.  w is [N,K] row-major f32,
 * K % 32 == 0.  Outputs the canonical form: q int8 [N,K] (Q4: -8..7, Q8:
 * -127..127) and scales as f16 bit patterns [N,K/32].
 *   amax = max |w| over the group;  d = f16(amax / qmax)  (qmax 7 or 127)
 *   q    = clamp(round_half_away(w / f32(d)), lo, hi)    (lo,hi = -8,7 / -127,127)
 *   d == 0  =>  q = 0.
 * Returns 0, or -1 on a bad argument. */
int cybq_oracle_quantize(int bits, const float* w, size_t N, size_t K,
                         int8_t* q, uint16_t* scales);

/* ---- interchange layouts.
 * PLANAR   Q4: qplane [N][K/2], byte j = (q[2j] & 15) | (q[2j+1] & 15) << 4,
 *              two's-complement nibbles;  Q8: qplane [N][K] int8.
 *              scale plane [N][K/32] f16.
 * BLOCK_AOS Q4: [N][K/32] blocks of 18 B = f16 d, then 16 bytes, byte j =
 *              (q[j]+8) | (q[j+16]+8) << 4;  Q8: blocks of 34 B = f16 d, 32 int8. */
int cybq_oracle_pack_planar(int bits, const int8_t* q, size_t N, size_t K, uint8_t* qplane);
int cybq_oracle_unpack_planar(int bits, const uint8_t* qplane, size_t N, size_t K, int8_t* q);
int cybq_oracle_pack_blocks(int bits, const int8_t* q, const uint16_t* scales,
                            size_t N, size_t K, uint8_t* blocks);
int cybq_oracle_unpack_blocks(int bits, const uint8_t* blocks, size_t N, size_t K,
                              int8_t* q, uint16_t* scales);

/* ---- dequantise: w[n,k] = f32(scale[n,k/32]) * (float)q[n,k]   (exact in f32) */
int cybq_oracle_dequant(const int8_t* q, const uint16_t* scales, size_t N, size_t K, float* w);

/* ---- the op.  y[m,n] = sum_k x[m,k] * w[n,k],  x [M,K] f32 (already widened
 * from f16/bf16, which is exact), w as (q, scales).
 *   _f32 : fp32 accumulation, k ascending, separate multiply and add of the
 *          dequantised weight (no fused multiply-add)
 *   _f64 : the same contraction in double; the yardstick errors are measured on
 *   _blocked_mt : fp32, per group  acc += d * sum_k(x*q), rows split over
 *          `threads` OS threads - the timed CPU baseline. */
int cybq_oracle_matmul_f32(const int8_t* q, const uint16_t* scales, size_t N, size_t K,
                           const float* x, size_t M, float* y);
int cybq_oracle_matmul_f64(const int8_t* q, const uint16_t* scales, size_t N, size_t K,
                           const float* x, size_t M, double* y);
int cybq_oracle_matmul_blocked_mt(const int8_t* q, const uint16_t* scales, size_t N, size_t K,
                                  const float* x, size_t M, float* y, int threads);

/* relative L2 error  ||a-b|| / ||b||  in double */
double cybq_oracle_rel_l2(const float* a, const double* b, size_t n);

#ifdef __cplusplus
}
#endif
#endif
