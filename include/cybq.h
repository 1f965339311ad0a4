/*
 * cybq.h - C ABI of libcybq, the MI355X (gfx950) implementation of cyb's
 * block-quantized matmul operator.
 *
 * What it replaces.  In cyb every linear layer of the decode loop
 * (QKV, O proj, FFN, LM head - /root/reference/decide/pipeline.md:51) is one
 * dequantize-and-multiply over Q4/Q8 tensor data
 * (/root/reference/decide/pipeline.md:28,38) executed by the model runtime
 * crate `run` on one of its backends (cpu | wgpu WGSL | Metal;
 * /root/reference/decide/model-lifecycle.md:25-26,37).  That crate is a path
 * dependency outside the tree (/root/reference/Cargo.lock:8443-8462), so its
 * backend trait cannot be cited line by line; the entry points below are what
 * a fourth backend of that runtime has to bind: create a device context,
 * hand over each weight tensor once at model load, run the op per graph node,
 * read back dequantised weights for verification.
 *
 * Conventions
 *   - every function returns 0 (CYBQ_OK) or a negative cybq_status; nothing
 *     aborts, nothing throws across the boundary (the caller surfaces errors
 *     as SomaEvent::Error - /root/reference/shell/src/worlds/soma_bridge.rs:322-333).
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *     cybq_matmul / cybq_dequant / cybq_quantize are asynchronous and
 *     stream-ordered; they allocate nothing.
 *   - x, y, out are DEVICE pointers owned by the caller; weight source
 *     buffers given to cybq_weight_upload are HOST pointers (the mmap'd
 *     .model file - /root/reference/shell/src/lib.rs:31-33).
 *   - a cybq_ctx is bound to one device and is used from one thread at a time
 *     (the runtime has a single inference thread -
 *     /root/reference/shell/src/worlds/soma_bridge.rs:49-50,65).
 *   - a cybq_weight is immutable after upload.
 */
#ifndef CYBQ_H
#define CYBQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CYBQ_GROUP 32            /* weights per scale, along K */

typedef struct cybq_ctx cybq_ctx;
typedef struct cybq_weight cybq_weight;

typedef enum cybq_status {
    CYBQ_OK = 0,
    CYBQ_ERR_INVALID = -1,       /* null pointer, bad enum, bad size */
    CYBQ_ERR_SHAPE = -2,         /* K % 32 != 0, M/N/K < 1, K mismatch */
    CYBQ_ERR_ALIGN = -3,         /* x / y / out not aligned as documented */
    CYBQ_ERR_NO_DEVICE = -4,     /* no HIP device, or not a gfx950 part */
    CYBQ_ERR_HIP = -5,           /* a HIP runtime call failed; see cybq_last_error */
    CYBQ_ERR_NOMEM = -6,
    CYBQ_ERR_UNSUPPORTED = -7    /* valid request this build does not implement */
} cybq_status;

/* tensor data kinds of the container (/root/reference/decide/pipeline.md:28) */
typedef enum cybq_quant { CYBQ_Q4 = 4, CYBQ_Q8 = 8 } cybq_quant;

/* Interchange layouts accepted at upload.  W is [N,K] = [out,in]
 * (/root/reference/decide/pipeline.md:30), groups of 32 run along K.
 *   PLANAR     q plane then a separate scale plane.
 *              Q4: q[N][K/2], byte j of a row = (w[2j] & 15) | (w[2j+1] & 15) << 4,
 *                  two's-complement nibbles in -8..7;  Q8: q[N][K] int8.
 *              scales[N][K/32] IEEE binary16.
 *   BLOCK_AOS  [N][K/32] blocks, the Q4_0 / Q8_0 block shape named at
 *              /root/reference/decide/pipeline.md:38 (18 B and 34 B per 32
 *              weights, cf. shell/src/worlds/models/mod.rs:69-73):
 *              Q4: f16 d, then 16 bytes, byte j = (w[j]+8) | (w[j+16]+8) << 4;
 *              Q8: f16 d, then 32 int8.   `scales` must be NULL.
 * On the device both are repacked once into one native tiled layout. */
typedef enum cybq_layout { CYBQ_LAYOUT_PLANAR = 0, CYBQ_LAYOUT_BLOCK_AOS = 1 } cybq_layout;

typedef enum cybq_dtype { CYBQ_F32 = 0, CYBQ_F16 = 1, CYBQ_BF16 = 2 } cybq_dtype;

/* How the prefill kernels (M > 32; in FAST mode also 17 .. 32 rows of fp32 activations, or of 16-bit
 * activations with a folded RMSNorm, on weights with K of 2048 .. 8192) feed the matrix cores.  Both stay
 * inside the operator's 1e-3 relative-L2 tolerance.  (Calls of up to 16 rows, other calls of up to 32 rows,
 * and 33 .. 64 rows on weights of up to 6144 x 4096 that the FAST kernels do not take - always so with
 * CYBQ_PREFILL_EXACT, which gives them the decode kernels' EXACT operands - take the decode kernels, whose
 * operand form cybq_decode_mode describes.)
 *   FAST   (default) one f16 MFMA per 32-group; the weight operand is
 *          round_f16(scale * q), relative error <= 2^-11 per weight (about 2e-4
 *          relative L2 on y).  bf16 and fp32 activations become f16 operands behind a
 *          power-of-two scale per row (taken from the row's largest magnitude and undone on
 *          output): rows of any finite magnitude keep that accuracy; within a row, elements
 *          below 2^-27 of the largest lose bits.  f16 activations are used as they are.
 *   EXACT  two MFMAs per 32-group in the activation type; scale * q is split
 *          without loss into a high and a low 16-bit operand, so y differs from
 *          the fp32 CPU path only by accumulation order.  Half the throughput. */
typedef enum cybq_prefill_mode { CYBQ_PREFILL_FAST = 0, CYBQ_PREFILL_EXACT = 1 } cybq_prefill_mode;

/* How the decode kernels form their weight operands.  Every form accumulates in fp32, applies the
 * f16 group scale in fp32 and stays far inside the 1e-3 tolerance.  Which form runs:
 *   f16 activations   1 - 2 rows: STREAM -> subnormal operands, EXACT -> exact integers.
 *                     3 - 32 rows (and the 33 - 64-row walk): STREAM -> subnormal operands for Q4 on
 *                     outputs wide enough for two to four 16-row strips per workgroup, exact integers
 *                     otherwise; EXACT -> exact integers.
 *   bf16 activations  any row count, either mode: the bf16 numbers 128 + (q + bias) with the bias
 *                     removed inside the accumulation (bf16 has no packed add to take it off
 *                     beforehand); the mode only chooses the kernel for 1 - 2 rows.
 *   fp32 activations  exact integers in either mode (activations split into two f16 halves).
 *   STREAM (default) the packed nibbles / bytes are used straight from memory - as f16 subnormals
 *          (q + bias) * 2^-22 with f16 activations - and the bias is removed inside the same fp32
 *          accumulation; about 4e-7 (bf16: 1e-6) relative L2.  The sums carry the bias until it
 *          cancels: a tensor of zeros gives values around 1e-7 of the activations' scale, not exact
 *          zeros (the same holds for bf16 activations in either mode).  The quickest form.
 *   EXACT  the weight operand is the exact integer q (more unpack arithmetic per byte);
 *          about 3e-7 relative L2, and a tensor of zeros gives exact zeros. */
typedef enum cybq_decode_mode { CYBQ_DECODE_STREAM = 0, CYBQ_DECODE_EXACT = 1 } cybq_decode_mode;

/* ---- context ---------------------------------------------------------- */

/* Replaces: backend construction when the runtime is spawned
 * (Soma::spawn(SomaConfig::default()) - shell/src/worlds/soma_bridge.rs:65). */
int cybq_init(int device, cybq_ctx** out);
void cybq_destroy(cybq_ctx* ctx);

const char* cybq_strerror(int status);
/* text of the last failure on this context (never NULL; "" when none) */
const char* cybq_last_error(const cybq_ctx* ctx);
/* "major.minor.patch" of the library */
const char* cybq_version(void);

/* ---- weights ---------------------------------------------------------- */

/* Replaces: the load of one quantised tensor from the mmap'd .model file at
 * model-switch time (use_model, lazy load - shell/src/worlds/models/mod.rs:7-8,386;
 * "all conversion happens at import" - decide/pipeline.md:59: the repack to the
 * device layout happens here, once, never in cybq_matmul).
 * `q` / `scales` are host pointers (see cybq_layout); requires K % 32 == 0.
 * A tensor with a scale so large that |scale| * 8 (Q4) or |scale| * 128 (Q8) leaves f16's range
 * (or a non-finite scale) is marked at upload and served by the decode kernels for every M: the
 * prefill kernels form scale * q in f16. */
int cybq_weight_upload(cybq_ctx* ctx, cybq_quant quant, cybq_layout layout,
                       int64_t N, int64_t K, const void* q, const void* scales,
                       cybq_weight** out);
/* A second device copy of the same tensor at a different address (used by
 * benchmarks to stream more bytes than the last-level cache holds). */
int cybq_weight_clone(cybq_ctx* ctx, const cybq_weight* src, cybq_weight** out);
int cybq_weight_free(cybq_ctx* ctx, cybq_weight* w);
/* any of the out pointers may be NULL.  device_bytes = bytes the tensor
 * occupies in HBM (with padding of N to 16 and K to 128). */
int cybq_weight_info(const cybq_weight* w, int* quant, int64_t* N, int64_t* K,
                     int64_t* device_bytes);

/* ---- the op ------------------------------------------------------------ */

/* Replaces: execution of one block-quantized matmul node of the graph IR
 * (decide/pipeline.md:28,51):   y[m,n] = sum_k x[m,k] * (scale[n,k/32] * q[n,k])
 * with fp32 accumulation.
 *   x  [M,K] row-major, xdt in {F16,BF16,F32}, 16-byte aligned
 *   y  [M,N] row-major, ydt in {F32,F16,BF16} (fp32 accumulator rounded once)
 *   M >= 1.  M <= 32 runs the HBM-streaming decode kernels (17..32 rows of 16-bit
 *   activations: one pass with two row blocks; with a folded norm two passes of 16
 *   rows; 33..64 rows of 16-bit activations on a weight of up to 6144 x 4096
 *   elements: two passes, 32 rows and the rest), larger M the LDS-tiled MFMA prefill kernel (fp32
 *   activations in CYBQ_PREFILL_EXACT mode: the decode kernel, 16 rows at a
 *   time; in FAST mode they are rounded once to f16 on the way in and take
 *   the prefill kernel from 17 rows on); there is no other path. */
int cybq_matmul(cybq_ctx* ctx, const cybq_weight* w, const void* x, cybq_dtype xdt,
                int64_t M, void* y, cybq_dtype ydt, void* stream);

/* cybq_matmul for callers that cannot allocate or cannot let a callee allocate: code under
 * stream capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the
 * reference.  Same arguments, same results to within summation order; the prefill path's
 * scratch (staged activations, partial sums of a K split) is a 64 MiB array inside the
 * library's code object, one copy per device, instead of the context's allocated workspace,
 * and the call makes no hipMalloc / hipFree and no call that allocates.  Limits: for M > 16,
 * K <= 32768 (CYBQ_ERR_UNSUPPORTED beyond).  All calls on one device share that array, whatever
 * context or stream they use: calls that overlap in time on one device race. */
int cybq_matmul_static(cybq_ctx* ctx, const cybq_weight* w, const void* x, cybq_dtype xdt,
                       int64_t M, void* y, cybq_dtype ydt, void* stream);

/* Replaces: a backend configuration knob (the reference picks a backend per run:
 * `--backend honeycrisp|wgpu|cpu`, shell/src/worlds/models/mod.rs:113-115); here
 * it selects the numeric mode of the prefill kernel for this context. */
int cybq_set_prefill_mode(cybq_ctx* ctx, cybq_prefill_mode mode);

/* Same knob for the decode kernel (see cybq_decode_mode). */
int cybq_set_decode_mode(cybq_ctx* ctx, cybq_decode_mode mode);

/* Replaces: the executor's walk over the quantised-matmul nodes of one decode
 * step (7 linears per layer x layers + LM head - decide/pipeline.md:51): `count`
 * independent invocations of cybq_matmul launched back to back on `stream`
 * from native code, so the host cost per node is one kernel launch.
 * w[i], x[i], y[i] as in cybq_matmul; all share M, xdt, ydt.  Stops at the
 * first failing node and returns its status. */
int cybq_matmul_many(cybq_ctx* ctx, int64_t count, const cybq_weight* const* w,
                     const void* const* x, void* const* y, cybq_dtype xdt, int64_t M,
                     cybq_dtype ydt, void* stream);

/* What the kernel does with an output element on its way to memory: the ops on
 * either side of a linear in the decode loop ("norm -> QKV -> ... -> O proj ->
 * residual -> norm -> FFN -> residual", decide/pipeline.md:51), fused so that
 * they cost no launch and no round trip through HBM.  The reference's own
 * definitions of these ops are not visible in its tree; the formulas below are
 * the LlamaStyle ones and are this library's choice. */
typedef enum cybq_epilogue {
    CYBQ_EPI_NONE = 0,
    CYBQ_EPI_ADD = 1,      /* y = residual + x W^T; residual: [M,N] of ydt; added in fp32, rounded once */
    CYBQ_EPI_SWIGLU = 2    /* w from cybq_weight_fuse_pairs(gate, up): y[M,N/2] = silu(x Wg^T) * (x Wu^T),
                              silu(t) = t / (1 + exp(-t)), all in fp32, rounded once */
} cybq_epilogue;

/* Replaces: the FFN's gate and up projections as one weight (both read the same
 * activations - decide/pipeline.md:51).  `gate` and `up`: same quant, same
 * [N,K], N a multiple of 16.  The result has 2N rows, gate and up interleaved in
 * strips of 16 rows (device to device, no requantisation); as a plain matmul
 * weight it yields those interleaved columns, with CYBQ_EPI_SWIGLU it yields
 * the N activated columns.  The inputs stay valid and independent. */
int cybq_weight_fuse_pairs(cybq_ctx* ctx, const cybq_weight* gate, const cybq_weight* up, cybq_weight** out);

/* cybq_matmul with an epilogue.  `residual` is read only for CYBQ_EPI_ADD (device
 * pointer, may alias y).  CYBQ_EPI_SWIGLU needs a weight made by
 * cybq_weight_fuse_pairs and writes y[M, N/2]. */
int cybq_matmul_ex(cybq_ctx* ctx, const cybq_weight* w, const void* x, cybq_dtype xdt, int64_t M,
                   void* y, cybq_dtype ydt, cybq_epilogue epilogue, const void* residual, void* stream);

/* cybq_matmul_ex with RMSNorm folded into the activation load (the norm in front of
 * QKV and of the FFN - decide/pipeline.md:51):
 *     rstd[m] = 1 / sqrt(mean_k x[m,k]^2 + eps)            (fp32, fixed summation order)
 *     y       = epilogue( rstd[m] * sum_k round(x[m,k] * gamma[k]) * W[n,k] )
 * x * gamma is formed in fp32 and rounded once to the kernel's operand type (the type
 * of x; f16 for bf16 and fp32 x in the FAST prefill mode; two f16 halves for fp32 x
 * elsewhere) - what an
 * unfused norm writing 16-bit activations would round too, minus its rounding of rstd.
 * gamma: [K] device pointer of type gdt, 16-byte aligned.  The definition is the LlamaStyle one and this
 * library's choice (the reference's is not visible in its tree). */
int cybq_matmul_norm(cybq_ctx* ctx, const cybq_weight* w, const void* x, cybq_dtype xdt, int64_t M,
                     const void* gamma, cybq_dtype gdt, float eps, void* y, cybq_dtype ydt,
                     cybq_epilogue epilogue, const void* residual, void* stream);

/* cybq_matmul_many with an epilogue per node: epilogue[i] is a cybq_epilogue,
 * residual[i] its residual (NULL unless CYBQ_EPI_ADD); either array may be NULL
 * (= no epilogues). */
int cybq_matmul_many_ex(cybq_ctx* ctx, int64_t count, const cybq_weight* const* w,
                        const void* const* x, void* const* y, const int* epilogue,
                        const void* const* residual, cybq_dtype xdt, int64_t M, cybq_dtype ydt,
                        void* stream);

/* cybq_matmul_many_ex with a folded RMSNorm per node: gamma[i] is the node's gamma ([K] of type
 * gdt) or NULL (no norm in front of that node); all norms share gdt and eps.  One native walk then
 * covers a whole decode layer as the loop runs it (decide/pipeline.md:51): norm + QKV, O + residual,
 * norm + gate/up with SwiGLU, down + residual.  gamma, epilogue and residual may each be NULL. */
int cybq_matmul_many_norm(cybq_ctx* ctx, int64_t count, const cybq_weight* const* w,
                          const void* const* x, const void* const* gamma, cybq_dtype gdt, float eps,
                          void* const* y, const int* epilogue, const void* const* residual,
                          cybq_dtype xdt, int64_t M, cybq_dtype ydt, void* stream);

/* Replaces: nothing the runtime calls per token; it is the verification hook
 * ("dequantised weights match bit-exactly"): out[N,K] f32 = f32(scale) * q. */
int cybq_dequant(cybq_ctx* ctx, const cybq_weight* w, float* out, void* stream);

/* Replaces: the quantise step of the import pipeline
 * (glia_import::pipeline::import_snapshot - shell/src/worlds/models/mod.rs:428;
 * decide/pipeline.md:38-40).  src [N,K] f32 on the device; writes the PLANAR
 * interchange layout to device buffers q_out ([N][K/2] or [N][K] bytes) and
 * scales_out ([N][K/32] f16):  d = f16(absmax/qmax), q = clamp(round(w/d)). */
int cybq_quantize(cybq_ctx* ctx, cybq_quant quant, const float* src, int64_t N, int64_t K,
                  void* q_out, void* scales_out, void* stream);
/* Builds a weight handle from PLANAR buffers that already live on the device
 * (the output of cybq_quantize); stream-ordered, allocates the handle.  The buffers must stay
 * valid until the work queued on `stream` has run; other calls that read the new weight
 * (cybq_weight_clone, cybq_weight_fuse_pairs, a matmul on another stream) must be ordered after it
 * by the caller.  The scales are scanned on the device by the same kernel (a tensor whose
 * |scale| * 8 (Q4) or |scale| * 128 (Q8) leaves f16's range is served by the decode kernels for
 * every M, as after cybq_weight_upload); the first call that needs the answer waits for that kernel. */
int cybq_weight_from_device(cybq_ctx* ctx, cybq_quant quant, int64_t N, int64_t K,
                            const void* q_dev, const void* scales_dev, void* stream,
                            cybq_weight** out);

#ifdef __cplusplus
}
#endif
#endif
