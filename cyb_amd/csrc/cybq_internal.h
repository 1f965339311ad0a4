// cybq_internal.h - launcher prototypes shared between the C ABI (api.hip) and
// the kernel translation units.  Every launcher validates nothing: api.hip
// checks shapes, alignment and pointers before it calls down here.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "cybq_device.h"

namespace cybq {

// dtype codes mirror enum cybq_dtype
constexpr int kF32 = 0, kF16 = 1, kBF16 = 2;

// q: PLANAR q plane (4-byte aligned) with `scales`, or BLOCK_AOS blocks (2-byte aligned, scales unused)
// wide_flag: device word that receives 1 when some scale times the largest q leaves f16 (nullptr: no scan)
hipError_t launch_repack(int bits, int layout, const void* q, const void* scales, uint8_t* dst, int N, int K, int NT, int KT,
                         uint32_t* wide_flag, hipStream_t st);
hipError_t launch_dequant(const WeightView& w, float* out, hipStream_t st);

// decode path, 1 <= M <= 16 per call, and 17 .. 32 rows where gemv_serves_32 says so (api.hip
// walks the other 17..32-row calls 16 rows at a time)
bool gemv_serves_32(int xdt, int M, const Epilogue& epi);
// exact_operands: keep the weight operands exact integers for one and two f16 rows too (the LDS
// kernel) instead of the subnormal-operand kernel of gemv1.hip
// scratch: device memory the batched-rows kernel may use when it splits K over workgroups (few strips, a
// long K): a ticket word per strip group at its start - zero at rest - and the slabs of partial sums behind
// them; nullptr = never split.  Calls that share it must not overlap.
constexpr size_t kDecodeScratchBytes = (size_t)8 << 20;
hipError_t launch_gemv(const WeightView& w, const void* x, int xdt, int M, void* y, int ydt,
                       int num_cus, bool exact_operands, const Epilogue& epi, void* scratch, size_t scratch_bytes, hipStream_t st);
// decode kernel for one and two rows (f16 / bf16 activations, no folded norm): weight operands are f16 subnormals
// (bf16: 128 + u),
// the +8 / +128 bias comes off inside the MFMA accumulation (gemv1.hip)
bool gemv1_serves(const WeightView& w, int xdt, int M, const Epilogue& epi);
hipError_t launch_gemv1(const WeightView& w, const void* x, int xdt, int M, void* y, int ydt, const Epilogue& epi, hipStream_t st);
// prefill path (api.hip sends 16-bit activations with M > 32 here)
// exact: two MFMAs per group with losslessly split weights; otherwise one f16 MFMA
// per group with weights rounded once to f16
// workspace: device scratch owned by the context (activations restaged in MFMA operand
// order, fp32 slabs of a K split, per-row statistics of a folded norm)
hipError_t launch_gemm(const WeightView& w, const void* x, int xdt, int M, void* y, int ydt,
                       int num_cus, bool exact, void* workspace, size_t workspace_bytes, const Epilogue& epi,
                       hipStream_t st);

// few rows (17 .. 64 on an output wide enough, up to 512 on a narrow one), FAST mode, activations already staged as f16 operands
// (gemm_rows.hip); ssq_part / ssq_blocks / unscale: the staging pass's per-row statistics
int gemm_rows_blocks(const WeightView& w, int M, int num_cus, const Epilogue& epi);
bool gemm_rows_serves(const WeightView& w, int M, int num_cus, const Epilogue& epi);
hipError_t launch_gemm_rows(const WeightView& w, const void* x_staged, int M, void* y, int ydt, const Epilogue& epi,
                            const float* ssq_part, int ssq_blocks, const float* unscale, int num_cus, hipStream_t st);
// test/bench hook: 2 = never take the few-rows kernel, 1 = whatever the width, 0 = automatic
void set_gemm_tuning(int rows_kernel);
// whether launch_gemm hands a FAST-mode call of M rows with this epilogue to the few-rows kernel (the hook included)
bool gemm_rows_takes(const WeightView& w, int M, int num_cus, const Epilogue& epi);

hipError_t launch_quantize(int bits, const float* src, int N, int K, void* q_out, void* s_out,
                           hipStream_t st);

// Kernels that need more dynamic LDS than the default 64 KB say so when the library is loaded:
// naming LdsRequest<&kernel, bytes>::registered anywhere in a launcher puts the pair on a list
// (a static initialiser, run before any call).  cybq_init walks the list for its device, so
// no launch ever changes a function attribute: first calls behave like all others and may sit
// inside a stream capture.
void register_lds_request(const void* kernel, int bytes);
hipError_t raise_all_lds_limits();              // for the current device
template <auto Kernel, int Bytes>
struct LdsRequest {
    static inline const bool registered = (register_lds_request(reinterpret_cast<const void*>(Kernel), Bytes), true);
};

// measurement probes (debug.hip)
hipError_t launch_read_probe(const WeightView& w, bool io, const void* x, void* y, hipStream_t st);
// other pure-read patterns over the same bytes (pattern 1 .. 6, see cybq_debug.h)
hipError_t launch_read_pattern(const WeightView& w, int pattern, int num_cus, hipStream_t st);
hipError_t launch_mfma_loop(int num_cus, int waves_per_simd, int iters, float* sink, hipStream_t st);
hipError_t launch_cache_read(const void* buf, int64_t bytes, int waves, int in_flight, int iters, int num_cus, hipStream_t st);

// test/bench hook: overrides the decode kernel's launch heuristics (0 = automatic)
void set_gemv_tuning(int waves_per_group, int rows_kernel, int unroll);


}  // namespace cybq
