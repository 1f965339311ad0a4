// api.hip - the C ABI declared in include/cybq.h: argument checking, device
// memory ownership, dispatch to the kernels.  No torch, no C++ types cross
// this boundary.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "../../include/cybq.h"
#include "cybq_debug.h"
#include "cybq_internal.h"

struct cybq_ctx {
    int device = 0;
    int num_cus = 0;
    bool prefill_exact = false;
    bool decode_exact = false;
    void* workspace = nullptr;          // scratch for the prefill path, allocated once at init
    size_t workspace_bytes = 0;
    std::string last_error;
};

struct cybq_weight {
    int device = 0;
    int bits = 0;
    int64_t N = 0, K = 0;
    int NT = 0, KT = 0;
    uint8_t* data = nullptr;            // native tiles (q words + scales per tile), strip-major
    size_t bytes = 0;
    bool paired = false;                // made by cybq_weight_fuse_pairs: strips alternate gate / up
    // some |scale| * qmax exceeds what f16 holds: the prefill kernels, which form scale * q in
    // f16, would overflow; such a tensor takes the decode kernels (scale applied in fp32) for any M
    bool wide_scales = false;
    // cybq_weight_from_device: the repack kernel ORs "some scale is wide" into a word behind the tiles and a
    // copy of it to `scan_host` (pinned) is queued behind the kernel; the first call that needs the answer
    // waits for `scan_done` (long since complete in practice) and moves it into wide_scales
    hipEvent_t scan_done = nullptr;
    uint32_t* scan_host = nullptr;
    std::once_flag scan_once;
};

namespace cybq {

namespace {
struct LdsEntry {
    const void* kernel;
    int bytes;
};
std::vector<LdsEntry>& lds_requests()
{
    static std::vector<LdsEntry> list;        // built on first use: registrations come from static initialisers
    return list;
}
}  // namespace

void register_lds_request(const void* kernel, int bytes) { lds_requests().push_back({kernel, bytes}); }

hipError_t raise_all_lds_limits()
{
    for (const LdsEntry& r : lds_requests()) {
        hipError_t e = hipFuncSetAttribute(r.kernel, hipFuncAttributeMaxDynamicSharedMemorySize, r.bytes);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace cybq

namespace {

// Scratch of cybq_matmul_static, the entry point that allocates nothing: the prefill path's
// staging area and K-split slabs live in this array instead of a hipMalloc'ed workspace.
// Every device the library runs on holds its own copy at its own address until the process
// ends; the name below is only the host-side handle of the symbol, never a device address:
// cybq_init asks the runtime for the address on its device and kernels receive that pointer.
constexpr size_t kStaticScratchBytes = (size_t)64 << 20;
constexpr int64_t kStaticMaxK = 32768;          // 256 staged rows of 2-byte activations fit half the scratch with room to spare
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;              // contexts may be created from several threads

int fail(cybq_ctx* ctx, int code, const char* what)
{
    if (ctx) ctx->last_error = what ? what : "";
    return code;
}

int fail_hip(cybq_ctx* ctx, hipError_t e, const char* where)
{
    if (ctx) {
        ctx->last_error = std::string(where) + ": " + hipGetErrorString(e);
    }
    (void)hipGetLastError();   // clear the sticky error so the next call starts clean
    return e == hipErrorOutOfMemory ? CYBQ_ERR_NOMEM : CYBQ_ERR_HIP;
}

// The device is made current for every call: contexts may live on different
// devices inside one process.
struct DeviceGuard {
    hipError_t err;
    // (asking for the current device is a thread-local read; setting it again is not free, and a decode
    // launch is a few microseconds of host time in all)
    explicit DeviceGuard(int device)
    {
        int cur = -1;
        err = hipGetDevice(&cur);
        if (err != hipSuccess || cur != device) err = hipSetDevice(device);
    }
};

cybq::WeightView view_of(const cybq_weight* w)
{
    cybq::WeightView v;
    v.base = w->data;
    v.N = (int)w->N;
    v.K = (int)w->K;
    v.NT = w->NT;
    v.KT = w->KT;
    v.bits = w->bits;
    return v;
}

// largest finite f16 magnitude a scale may have for scale * q to stay inside f16: 65504 / qmax
bool scale_is_wide(uint16_t bits, int quant)
{
    const int e = (bits >> 10) & 31, m = bits & 1023;
    if (e == 31) return true;                                  // Inf / NaN
    const float v = e == 0 ? (float)m * (1.0f / 16777216.0f) : std::ldexp((float)(m + 1024), e - 25);
    return v * (quant == CYBQ_Q4 ? 8.0f : 128.0f) > 65504.0f;
}

bool any_wide_scale(int quant, int layout, int64_t groups, const void* q, const void* scales)
{
    if (layout == CYBQ_LAYOUT_PLANAR) {
        const uint16_t* s = static_cast<const uint16_t*>(scales);
        for (int64_t g = 0; g < groups; g++)
            if (scale_is_wide(s[g], quant)) return true;
        return false;
    }
    const size_t bs = quant == CYBQ_Q4 ? 18 : 34;
    const uint8_t* b = static_cast<const uint8_t*>(q);
    for (int64_t g = 0; g < groups; g++)
        if (scale_is_wide((uint16_t)(b[g * bs] | (b[g * bs + 1] << 8)), quant)) return true;
    return false;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

size_t dtype_size(int dt) { return dt == CYBQ_F32 ? 4 : 2; }
bool dtype_ok(int dt) { return dt == CYBQ_F32 || dt == CYBQ_F16 || dt == CYBQ_BF16; }

constexpr size_t kWeightTailBytes = 256;

int alloc_weight(cybq_ctx* ctx, int bits, int64_t N, int64_t K, cybq_weight** out)
{
    cybq_weight* w = new (std::nothrow) cybq_weight();
    if (!w) return fail(ctx, CYBQ_ERR_NOMEM, "host allocation failed");
    w->device = ctx->device;
    w->bits = bits;
    w->N = N;
    w->K = K;
    w->NT = (int)((N + cybq::kTileN - 1) / cybq::kTileN);
    w->KT = (int)((K + cybq::kTileK - 1) / cybq::kTileK);
    w->bytes = (size_t)w->NT * w->KT * cybq::tile_bytes(bits);
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&w->data), w->bytes + kWeightTailBytes);      // (tail: the scan's flag word)
    if (e != hipSuccess) {
        delete w;
        return fail_hip(ctx, e, "hipMalloc(weight)");
    }
    *out = w;
    return CYBQ_OK;
}

void release_weight(cybq_weight* w)
{
    if (w->scan_done) (void)hipEventDestroy(w->scan_done);
    if (w->scan_host) (void)hipHostFree(w->scan_host);
    (void)hipFree(w->data);
    delete w;
}

// wide_scales of a weight whose scales were scanned on the device: the answer is taken the first time it is needed
bool weight_is_wide(const cybq_weight* cw)
{
    cybq_weight* w = const_cast<cybq_weight*>(cw);
    if (w->scan_host) {
        std::call_once(w->scan_once, [w]() {
            if (w->scan_done) (void)hipEventSynchronize(w->scan_done);
            w->wide_scales = w->wide_scales || *w->scan_host != 0u;
        });
    }
    return w->wide_scales;
}

int check_weight_shape(cybq_ctx* ctx, int quant, int64_t N, int64_t K)
{
    if (quant != CYBQ_Q4 && quant != CYBQ_Q8) return fail(ctx, CYBQ_ERR_INVALID, "quant must be CYBQ_Q4 or CYBQ_Q8");
    if (N < 1 || K < 1) return fail(ctx, CYBQ_ERR_SHAPE, "N and K must be >= 1");
    if (K % CYBQ_GROUP) return fail(ctx, CYBQ_ERR_SHAPE, "K must be a multiple of 32");
    if (N > (int64_t)1 << 30 || K > (int64_t)1 << 30 || N * K > (int64_t)1 << 40)
        return fail(ctx, CYBQ_ERR_SHAPE, "tensor too large");
    return CYBQ_OK;
}

}  // namespace

extern "C" {

const char* cybq_version(void) { return "0.1.0"; }

const char* cybq_strerror(int status)
{
    switch (status) {
        case CYBQ_OK: return "ok";
        case CYBQ_ERR_INVALID: return "invalid argument";
        case CYBQ_ERR_SHAPE: return "bad shape";
        case CYBQ_ERR_ALIGN: return "misaligned pointer";
        case CYBQ_ERR_NO_DEVICE: return "no usable gfx950 device";
        case CYBQ_ERR_HIP: return "HIP runtime error";
        case CYBQ_ERR_NOMEM: return "out of memory";
        case CYBQ_ERR_UNSUPPORTED: return "unsupported";
        default: return "unknown status";
    }
}

const char* cybq_last_error(const cybq_ctx* ctx) { return ctx ? ctx->last_error.c_str() : ""; }

int cybq_init(int device, cybq_ctx** out)
{
    if (!out) return CYBQ_ERR_INVALID;
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count < 1) { (void)hipGetLastError(); return CYBQ_ERR_NO_DEVICE; }
    if (device < 0 || device >= count) return CYBQ_ERR_INVALID;
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) { (void)hipGetLastError(); return CYBQ_ERR_NO_DEVICE; }
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) return CYBQ_ERR_NO_DEVICE;
    e = hipSetDevice(device);
    if (e != hipSuccess) { (void)hipGetLastError(); return CYBQ_ERR_HIP; }
    // every kernel that wants more than the default dynamic LDS gets its limit raised now, for
    // this device: launches never touch function attributes
    e = cybq::raise_all_lds_limits();
    if (e != hipSuccess) { (void)hipGetLastError(); return CYBQ_ERR_HIP; }
    if (device < kMaxDevices) {       // this device's copy of the static scratch
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (!g_scratch_ptr[device]) {
            void* p = nullptr;
            e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
            if (e != hipSuccess || !p) { (void)hipGetLastError(); return CYBQ_ERR_HIP; }
            g_scratch_ptr[device] = p;
        }
    }
    cybq_ctx* ctx = new (std::nothrow) cybq_ctx();
    if (!ctx) return CYBQ_ERR_NOMEM;
    ctx->device = device;
    ctx->num_cus = prop.multiProcessorCount;
    // 256 MiB of scratch for the prefill path: the activations restaged in MFMA operand
    // order (larger M is walked in row chunks) and the partial sums of a K split
    ctx->workspace_bytes = (size_t)256 << 20;
    if (hipMalloc(&ctx->workspace, ctx->workspace_bytes) != hipSuccess) {
        (void)hipGetLastError();
        delete ctx;
        return CYBQ_ERR_NOMEM;
    }
    // the decode kernels' tickets (start of the scratch's tail) are zero at rest
    if (hipMemset(static_cast<char*>(ctx->workspace) + ctx->workspace_bytes - cybq::kDecodeScratchBytes, 0, (size_t)1 << 16) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipFree(ctx->workspace);
        delete ctx;
        return CYBQ_ERR_HIP;
    }
    *out = ctx;
    return CYBQ_OK;
}

void cybq_destroy(cybq_ctx* ctx)
{
    if (!ctx) return;
    if (ctx->workspace && hipSetDevice(ctx->device) == hipSuccess) (void)hipFree(ctx->workspace);
    delete ctx;
}

int cybq_weight_upload(cybq_ctx* ctx, cybq_quant quant, cybq_layout layout, int64_t N, int64_t K,
                       const void* q, const void* scales, cybq_weight** out)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (!out) return fail(ctx, CYBQ_ERR_INVALID, "out is NULL");
    *out = nullptr;
    if (!q) return fail(ctx, CYBQ_ERR_INVALID, "q is NULL");
    if (layout != CYBQ_LAYOUT_PLANAR && layout != CYBQ_LAYOUT_BLOCK_AOS)
        return fail(ctx, CYBQ_ERR_INVALID, "unknown layout");
    if (layout == CYBQ_LAYOUT_PLANAR && !scales) return fail(ctx, CYBQ_ERR_INVALID, "PLANAR needs a scale plane");
    if (layout == CYBQ_LAYOUT_BLOCK_AOS && scales) return fail(ctx, CYBQ_ERR_INVALID, "BLOCK_AOS carries its scales; pass NULL");
    int rc = check_weight_shape(ctx, quant, N, K);
    if (rc) return rc;
    DeviceGuard guard(ctx->device);
    if (guard.err != hipSuccess) return fail_hip(ctx, guard.err, "hipSetDevice");

    const int64_t groups = N * (K / CYBQ_GROUP);
    size_t q_src_bytes, s_src_bytes = 0;
    if (layout == CYBQ_LAYOUT_PLANAR) {
        q_src_bytes = (size_t)(quant == CYBQ_Q4 ? N * K / 2 : N * K);
        s_src_bytes = (size_t)groups * 2;
    } else {
        q_src_bytes = (size_t)groups * (quant == CYBQ_Q4 ? 18 : 34);
    }
    void *q_tmp = nullptr, *s_tmp = nullptr;
    hipError_t e = hipMalloc(&q_tmp, q_src_bytes);
    if (e == hipSuccess && s_src_bytes) e = hipMalloc(&s_tmp, s_src_bytes);
    if (e != hipSuccess) {
        if (q_tmp) (void)hipFree(q_tmp);
        return fail_hip(ctx, e, "hipMalloc(staging)");
    }
    cybq_weight* w = nullptr;
    rc = alloc_weight(ctx, quant, N, K, &w);
    if (rc == CYBQ_OK) {
        e = hipMemcpy(q_tmp, q, q_src_bytes, hipMemcpyHostToDevice);
        if (e == hipSuccess && s_src_bytes) e = hipMemcpy(s_tmp, scales, s_src_bytes, hipMemcpyHostToDevice);
        if (e == hipSuccess)
            e = cybq::launch_repack(quant, layout, q_tmp, s_tmp, w->data, (int)N, (int)K, w->NT, w->KT, nullptr, nullptr);
        if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
        if (e != hipSuccess) {
            rc = fail_hip(ctx, e, "weight upload");
            release_weight(w);
            w = nullptr;
        }
    }
    (void)hipFree(q_tmp);
    if (s_tmp) (void)hipFree(s_tmp);
    if (rc) return rc;
    w->wide_scales = any_wide_scale(quant, layout, groups, q, scales);
    *out = w;
    return CYBQ_OK;
}

int cybq_weight_from_device(cybq_ctx* ctx, cybq_quant quant, int64_t N, int64_t K, const void* q_dev,
                            const void* scales_dev, void* stream, cybq_weight** out)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (!out) return fail(ctx, CYBQ_ERR_INVALID, "out is NULL");
    *out = nullptr;
    if (!q_dev || !scales_dev) return fail(ctx, CYBQ_ERR_INVALID, "q_dev / scales_dev is NULL");
    if (reinterpret_cast<uintptr_t>(q_dev) % 4 || reinterpret_cast<uintptr_t>(scales_dev) % 2)
        return fail(ctx, CYBQ_ERR_ALIGN, "q_dev must be 4-byte and scales_dev 2-byte aligned");
    int rc = check_weight_shape(ctx, quant, N, K);
    if (rc) return rc;
    DeviceGuard guard(ctx->device);
    if (guard.err != hipSuccess) return fail_hip(ctx, guard.err, "hipSetDevice");
    cybq_weight* w = nullptr;
    rc = alloc_weight(ctx, quant, N, K, &w);
    if (rc) return rc;
    // the scales are scanned by the repack kernel itself: a word behind the tiles collects "some |scale| * qmax leaves
    // f16", its copy to pinned host memory is queued behind the kernel and read by the first call that needs it
    hipStream_t st = static_cast<hipStream_t>(stream);
    uint32_t* flag = reinterpret_cast<uint32_t*>(w->data + w->bytes);
    hipError_t e = hipHostMalloc(reinterpret_cast<void**>(&w->scan_host), sizeof(uint32_t), hipHostMallocDefault);
    if (e == hipSuccess) {
        *w->scan_host = 0u;
        e = hipEventCreateWithFlags(&w->scan_done, hipEventDisableTiming);
    }
    if (e == hipSuccess) e = hipMemsetAsync(flag, 0, sizeof(uint32_t), st);
    if (e == hipSuccess)
        e = cybq::launch_repack(quant, CYBQ_LAYOUT_PLANAR, q_dev, scales_dev, w->data, (int)N, (int)K, w->NT, w->KT, flag, st);
    if (e == hipSuccess) e = hipMemcpyAsync(w->scan_host, flag, sizeof(uint32_t), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipEventRecord(w->scan_done, st);
    if (e != hipSuccess) {
        (void)hipStreamSynchronize(st);          // nothing may still write the pinned word
        release_weight(w);
        return fail_hip(ctx, e, "repack launch");
    }
    *out = w;
    return CYBQ_OK;
}

int cybq_weight_clone(cybq_ctx* ctx, const cybq_weight* src, cybq_weight** out)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (!src || !out) return fail(ctx, CYBQ_ERR_INVALID, "src / out is NULL");
    *out = nullptr;
    if (src->device != ctx->device) return fail(ctx, CYBQ_ERR_INVALID, "weight lives on another device");
    DeviceGuard guard(ctx->device);
    if (guard.err != hipSuccess) return fail_hip(ctx, guard.err, "hipSetDevice");
    cybq_weight* w = nullptr;
    int rc = alloc_weight(ctx, src->bits, src->N, src->K, &w);
    if (rc) return rc;
    hipError_t e = hipMemcpy(w->data, src->data, src->bytes, hipMemcpyDeviceToDevice);
    if (e != hipSuccess) {
        release_weight(w);
        return fail_hip(ctx, e, "weight clone");
    }
    w->paired = src->paired;
    w->wide_scales = weight_is_wide(src);
    *out = w;
    return CYBQ_OK;
}

int cybq_weight_free(cybq_ctx* ctx, cybq_weight* w)
{
    if (!w) return CYBQ_OK;
    hipError_t e = hipSetDevice(w->device);
    if (e == hipSuccess) {
        if (w->scan_done) (void)hipEventDestroy(w->scan_done);
        if (w->scan_host) (void)hipHostFree(w->scan_host);
        e = hipFree(w->data);
    }
    delete w;
    if (e != hipSuccess) return fail_hip(ctx, e, "hipFree(weight)");
    return CYBQ_OK;
}

int cybq_weight_info(const cybq_weight* w, int* quant, int64_t* N, int64_t* K, int64_t* device_bytes)
{
    if (!w) return CYBQ_ERR_INVALID;
    if (quant) *quant = w->bits;
    if (N) *N = w->N;
    if (K) *K = w->K;
    if (device_bytes) *device_bytes = (int64_t)w->bytes;
    return CYBQ_OK;
}

namespace {
int matmul_fused(cybq_ctx* ctx, const cybq_weight* w, const void* x, cybq_dtype xdt, int64_t M, const void* gamma,
                 cybq_dtype gdt, float eps, void* y, cybq_dtype ydt, cybq_epilogue epilogue, const void* residual,
                 void* stream, void* workspace, size_t workspace_bytes)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (!w || !x || !y) return fail(ctx, CYBQ_ERR_INVALID, "w / x / y is NULL");
    if (!dtype_ok(xdt) || !dtype_ok(ydt)) return fail(ctx, CYBQ_ERR_INVALID, "unknown dtype");
    if (M < 1 || M > (1 << 24)) return fail(ctx, CYBQ_ERR_SHAPE, "M must be in 1..2^24");
    if (w->device != ctx->device) return fail(ctx, CYBQ_ERR_INVALID, "weight lives on another device");
    if (!aligned16(x)) return fail(ctx, CYBQ_ERR_ALIGN, "x must be 16-byte aligned");
    if (reinterpret_cast<uintptr_t>(y) % dtype_size(ydt)) return fail(ctx, CYBQ_ERR_ALIGN, "y is not aligned to its element size");
    cybq::Epilogue epi = {cybq::kEpiNone, nullptr, nullptr, 0, 0.f};
    if (gamma) {
        if (!dtype_ok(gdt)) return fail(ctx, CYBQ_ERR_INVALID, "unknown gamma dtype");
        if (!aligned16(gamma)) return fail(ctx, CYBQ_ERR_ALIGN, "gamma must be 16-byte aligned");
        if (!(eps >= 0.f)) return fail(ctx, CYBQ_ERR_INVALID, "eps must be >= 0");
    }
    if (epilogue == CYBQ_EPI_ADD) {
        if (!residual) return fail(ctx, CYBQ_ERR_INVALID, "CYBQ_EPI_ADD needs a residual");
        if (reinterpret_cast<uintptr_t>(residual) % dtype_size(ydt)) return fail(ctx, CYBQ_ERR_ALIGN, "residual is not aligned to its element size");
        epi.kind = cybq::kEpiAdd;
        epi.residual = residual;
    } else if (epilogue == CYBQ_EPI_SWIGLU) {
        if (!w->paired) return fail(ctx, CYBQ_ERR_INVALID, "CYBQ_EPI_SWIGLU needs a weight made by cybq_weight_fuse_pairs");
        epi.kind = cybq::kEpiSwiglu;
    } else if (epilogue != CYBQ_EPI_NONE) {
        return fail(ctx, CYBQ_ERR_INVALID, "unknown epilogue");
    }
    epi.gamma = gamma;
    epi.gamma_dt = (int)gdt;
    epi.eps = eps;
    DeviceGuard guard(ctx->device);
    if (guard.err != hipSuccess) return fail_hip(ctx, guard.err, "hipSetDevice");
    hipStream_t st = static_cast<hipStream_t>(stream);
    cybq::WeightView v = view_of(w);
    hipError_t e;
    // the tail of the scratch belongs to the decode kernels (tickets and slabs of a K split), the rest to prefill
    void* dscr = nullptr;
    size_t dscr_bytes = 0;
    if (workspace && workspace_bytes > 2 * cybq::kDecodeScratchBytes) {
        workspace_bytes -= cybq::kDecodeScratchBytes;
        dscr = static_cast<char*>(workspace) + workspace_bytes;
        dscr_bytes = cybq::kDecodeScratchBytes;
    }
    if (M <= 16 || (M <= 32 && cybq::gemv_serves_32((int)xdt, (int)M, epi))) {
        e = cybq::launch_gemv(v, x, xdt, (int)M, y, ydt, ctx->num_cus, ctx->decode_exact, epi, dscr, dscr_bytes, st);
    } else if (M <= 64 && (int64_t)w->N * w->K <= (int64_t)6144 * 4096 && cybq::gemv_serves_32((int)xdt, 32, epi) &&
               (ctx->prefill_exact || weight_is_wide(w) || !cybq::gemm_rows_takes(v, (int)M, ctx->num_cus, epi))) {
        // 33..64 rows on a small weight (up to 4096 -> 6144) that the few-rows MFMA kernel does not take (exact
        // mode, wide scales, K outside 2048 .. 8192, a folded SwiGLU): the tiled MFMA
        // kernel would split K over workgroups and add the slabs in a second pass; two passes of the
        // batched-rows decode kernel (32 rows, then the rest) are quicker although they stream the weights twice
        // (4096 -> 4096 at 64 rows 21.8 -> 14.8 us; the few-rows kernel 13.1) - and exact
        // (a context in CYBQ_PREFILL_EXACT mode asked for exact operands at this row count)
        const bool exact_ops = ctx->decode_exact || ctx->prefill_exact;
        const int64_t n_out = epi.kind == cybq::kEpiSwiglu ? w->N / 2 : w->N;
        const size_t yoff = (size_t)32 * n_out * dtype_size(ydt);
        cybq::Epilogue ec = epi;
        if (epi.kind == cybq::kEpiAdd) ec.residual = static_cast<const char*>(residual) + yoff;
        e = cybq::launch_gemv(v, x, xdt, 32, y, ydt, ctx->num_cus, exact_ops, epi, dscr, dscr_bytes, st);
        if (e == hipSuccess)
            e = cybq::launch_gemv(v, static_cast<const char*>(x) + (size_t)32 * w->K * dtype_size(xdt), xdt, (int)M - 32,
                                  static_cast<char*>(y) + yoff, ydt, ctx->num_cus, exact_ops, ec, dscr, dscr_bytes, st);
    } else if (!weight_is_wide(w) && (xdt == CYBQ_F32 ? !ctx->prefill_exact : (M > 32 || (!ctx->prefill_exact && cybq::gemm_rows_takes(v, (int)M, ctx->num_cus, epi))))) {
        e = cybq::launch_gemm(v, x, xdt, (int)M, y, ydt, ctx->num_cus, ctx->prefill_exact, workspace, workspace_bytes,
                              epi, st);
    } else {
        // fp32 activations keep full precision through the decode kernel's hi/lo split:
        // exact-mode prefill in fp32 is walked 16 rows at a time (FAST mode rounds them to f16
        // in the staging pass and takes the MFMA kernel from 17 rows on: the LDS decode kernel
        // needs 52 - 65 us for 24 - 32 fp32 rows, the few-row MFMA kernel 16).  So are 17..32
        // rows of 16-bit activations with a folded norm where the few-row MFMA kernel does not take
        // them (FAST mode: 4096 -> 14336 at 32 rows 18.1 us there against 23.0 here): two passes of
        // the batched-rows kernel stream the weights twice and are still quicker than a 128-row MFMA
        // tile mostly empty (without the norm they are one pass, two row blocks per weight operand).
        // A tensor with wide scales (scale * q leaves f16) is walked the same way for any M, 32 rows at a
        // time where the batched-rows kernel takes them in one pass: the weights stream once per 32 rows.
        e = hipSuccess;
        const int64_t n_out = epi.kind == cybq::kEpiSwiglu ? w->N / 2 : w->N;
        const int64_t step = cybq::gemv_serves_32((int)xdt, 32, epi) ? 32 : 16;
        for (int64_t m0 = 0; m0 < M && e == hipSuccess; m0 += step) {
            int mm = (int)((M - m0) < step ? (M - m0) : step);
            const char* xp = static_cast<const char*>(x) + (size_t)m0 * w->K * dtype_size(xdt);
            const size_t yoff = (size_t)m0 * n_out * dtype_size(ydt);
            cybq::Epilogue ec = epi;
            if (epi.kind == cybq::kEpiAdd) ec.residual = static_cast<const char*>(residual) + yoff;
            e = cybq::launch_gemv(v, xp, xdt, mm, static_cast<char*>(y) + yoff, ydt, ctx->num_cus, ctx->decode_exact, ec, dscr, dscr_bytes, st);
        }
    }
    if (e != hipSuccess) return fail_hip(ctx, e, "matmul launch");
    return CYBQ_OK;
}
}  // namespace

int cybq_matmul_ex(cybq_ctx* ctx, const cybq_weight* w, const void* x, cybq_dtype xdt, int64_t M, void* y,
                   cybq_dtype ydt, cybq_epilogue epilogue, const void* residual, void* stream)
{
    return matmul_fused(ctx, w, x, xdt, M, nullptr, CYBQ_F32, 0.f, y, ydt, epilogue, residual, stream, ctx ? ctx->workspace : nullptr,
                        ctx ? ctx->workspace_bytes : 0);
}

int cybq_matmul_norm(cybq_ctx* ctx, const cybq_weight* w, const void* x, cybq_dtype xdt, int64_t M, const void* gamma,
                     cybq_dtype gdt, float eps, void* y, cybq_dtype ydt, cybq_epilogue epilogue, const void* residual,
                     void* stream)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (!gamma) return fail(ctx, CYBQ_ERR_INVALID, "gamma is NULL");
    return matmul_fused(ctx, w, x, xdt, M, gamma, gdt, eps, y, ydt, epilogue, residual, stream, ctx->workspace, ctx->workspace_bytes);
}

int cybq_matmul(cybq_ctx* ctx, const cybq_weight* w, const void* x, cybq_dtype xdt, int64_t M, void* y,
                cybq_dtype ydt, void* stream)
{
    return cybq_matmul_ex(ctx, w, x, xdt, M, y, ydt, CYBQ_EPI_NONE, nullptr, stream);
}

int cybq_matmul_static(cybq_ctx* ctx, const cybq_weight* w, const void* x, cybq_dtype xdt, int64_t M, void* y,
                       cybq_dtype ydt, void* stream)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    void* static_scratch = nullptr;
    if (ctx->device < kMaxDevices) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        static_scratch = g_scratch_ptr[ctx->device];
    }
    if (!static_scratch) return fail(ctx, CYBQ_ERR_UNSUPPORTED, "no static scratch on this device");
    if (w && M > 16 && w->K > kStaticMaxK)
        return fail(ctx, CYBQ_ERR_UNSUPPORTED, "cybq_matmul_static: K beyond 32768 does not fit the static scratch for more than 16 rows");
    return matmul_fused(ctx, w, x, xdt, M, nullptr, CYBQ_F32, 0.f, y, ydt, CYBQ_EPI_NONE, nullptr, stream,
                        static_scratch, kStaticScratchBytes);
}

int cybq_weight_fuse_pairs(cybq_ctx* ctx, const cybq_weight* gate, const cybq_weight* up, cybq_weight** out)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (!gate || !up || !out) return fail(ctx, CYBQ_ERR_INVALID, "gate / up / out is NULL");
    *out = nullptr;
    if (gate->device != ctx->device || up->device != ctx->device) return fail(ctx, CYBQ_ERR_INVALID, "weight lives on another device");
    if (gate->bits != up->bits || gate->N != up->N || gate->K != up->K) return fail(ctx, CYBQ_ERR_SHAPE, "gate and up differ in quant or shape");
    if (gate->N % cybq::kTileN) return fail(ctx, CYBQ_ERR_SHAPE, "N must be a multiple of 16");
    if (gate->paired || up->paired) return fail(ctx, CYBQ_ERR_INVALID, "inputs are already fused");
    DeviceGuard guard(ctx->device);
    if (guard.err != hipSuccess) return fail_hip(ctx, guard.err, "hipSetDevice");
    cybq_weight* w = nullptr;
    int rc = alloc_weight(ctx, gate->bits, 2 * gate->N, gate->K, &w);
    if (rc) return rc;
    // the native layout is strip-major: output strip 2i is gate strip i, 2i+1 is up strip i
    const size_t sb = (size_t)gate->KT * cybq::tile_bytes(gate->bits);          // bytes of one strip
    hipError_t e = hipMemcpy2D(w->data, 2 * sb, gate->data, sb, sb, gate->NT, hipMemcpyDeviceToDevice);
    if (e == hipSuccess) e = hipMemcpy2D(w->data + sb, 2 * sb, up->data, sb, sb, up->NT, hipMemcpyDeviceToDevice);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        release_weight(w);
        return fail_hip(ctx, e, "weight fuse");
    }
    w->paired = true;
    w->wide_scales = weight_is_wide(gate) || weight_is_wide(up);
    *out = w;
    return CYBQ_OK;
}

int cybq_set_prefill_mode(cybq_ctx* ctx, cybq_prefill_mode mode)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (mode != CYBQ_PREFILL_FAST && mode != CYBQ_PREFILL_EXACT) return fail(ctx, CYBQ_ERR_INVALID, "unknown prefill mode");
    ctx->prefill_exact = mode == CYBQ_PREFILL_EXACT;
    return CYBQ_OK;
}

int cybq_set_decode_mode(cybq_ctx* ctx, cybq_decode_mode mode)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (mode != CYBQ_DECODE_STREAM && mode != CYBQ_DECODE_EXACT) return fail(ctx, CYBQ_ERR_INVALID, "unknown decode mode");
    ctx->decode_exact = mode == CYBQ_DECODE_EXACT;
    return CYBQ_OK;
}

int cybq_matmul_many(cybq_ctx* ctx, int64_t count, const cybq_weight* const* w, const void* const* x,
                     void* const* y, cybq_dtype xdt, int64_t M, cybq_dtype ydt, void* stream)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (count < 0 || (count > 0 && (!w || !x || !y))) return fail(ctx, CYBQ_ERR_INVALID, "bad node list");
    for (int64_t i = 0; i < count; i++) {
        int rc = cybq_matmul(ctx, w[i], x[i], xdt, M, y[i], ydt, stream);
        if (rc) return rc;
    }
    return CYBQ_OK;
}

int cybq_matmul_many_ex(cybq_ctx* ctx, int64_t count, const cybq_weight* const* w, const void* const* x,
                        void* const* y, const int* epilogue, const void* const* residual, cybq_dtype xdt, int64_t M,
                        cybq_dtype ydt, void* stream)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (count < 0 || (count > 0 && (!w || !x || !y))) return fail(ctx, CYBQ_ERR_INVALID, "bad node list");
    for (int64_t i = 0; i < count; i++) {
        const cybq_epilogue e = epilogue ? static_cast<cybq_epilogue>(epilogue[i]) : CYBQ_EPI_NONE;
        int rc = cybq_matmul_ex(ctx, w[i], x[i], xdt, M, y[i], ydt, e, residual ? residual[i] : nullptr, stream);
        if (rc) return rc;
    }
    return CYBQ_OK;
}

int cybq_matmul_many_norm(cybq_ctx* ctx, int64_t count, const cybq_weight* const* w, const void* const* x,
                          const void* const* gamma, cybq_dtype gdt, float eps, void* const* y, const int* epilogue,
                          const void* const* residual, cybq_dtype xdt, int64_t M, cybq_dtype ydt, void* stream)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (count < 0 || (count > 0 && (!w || !x || !y))) return fail(ctx, CYBQ_ERR_INVALID, "bad node list");
    for (int64_t i = 0; i < count; i++) {
        const cybq_epilogue e = epilogue ? static_cast<cybq_epilogue>(epilogue[i]) : CYBQ_EPI_NONE;
        int rc = matmul_fused(ctx, w[i], x[i], xdt, M, gamma ? gamma[i] : nullptr, gdt, eps, y[i], ydt, e,
                              residual ? residual[i] : nullptr, stream, ctx->workspace, ctx->workspace_bytes);
        if (rc) return rc;
    }
    return CYBQ_OK;
}

int cybq_dequant(cybq_ctx* ctx, const cybq_weight* w, float* out, void* stream)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (!w || !out) return fail(ctx, CYBQ_ERR_INVALID, "w / out is NULL");
    if (w->device != ctx->device) return fail(ctx, CYBQ_ERR_INVALID, "weight lives on another device");
    if (!aligned16(out)) return fail(ctx, CYBQ_ERR_ALIGN, "out must be 16-byte aligned");
    DeviceGuard guard(ctx->device);
    if (guard.err != hipSuccess) return fail_hip(ctx, guard.err, "hipSetDevice");
    hipError_t e = cybq::launch_dequant(view_of(w), out, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail_hip(ctx, e, "dequant launch");
    return CYBQ_OK;
}

int cybq_quantize(cybq_ctx* ctx, cybq_quant quant, const float* src, int64_t N, int64_t K, void* q_out,
                  void* scales_out, void* stream)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (!src || !q_out || !scales_out) return fail(ctx, CYBQ_ERR_INVALID, "src / q_out / scales_out is NULL");
    int rc = check_weight_shape(ctx, quant, N, K);
    if (rc) return rc;
    if (!aligned16(src)) return fail(ctx, CYBQ_ERR_ALIGN, "src must be 16-byte aligned");
    if (reinterpret_cast<uintptr_t>(q_out) % 4 || reinterpret_cast<uintptr_t>(scales_out) % 2)
        return fail(ctx, CYBQ_ERR_ALIGN, "q_out must be 4-byte and scales_out 2-byte aligned");
    DeviceGuard guard(ctx->device);
    if (guard.err != hipSuccess) return fail_hip(ctx, guard.err, "hipSetDevice");
    hipError_t e = cybq::launch_quantize(quant, src, (int)N, (int)K, q_out, scales_out, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail_hip(ctx, e, "quantize launch");
    return CYBQ_OK;
}

/* ---- diagnostics declared in cybq_debug.h (not part of the operator interface) ---- */

int cybq_debug_set_gemm_tuning(int rows_kernel)
{
    cybq::set_gemm_tuning(rows_kernel);
    return CYBQ_OK;
}

int cybq_debug_set_gemv_tuning(int waves_per_group, int rows_kernel, int unroll)
{
    cybq::set_gemv_tuning(waves_per_group, rows_kernel, unroll);
    return CYBQ_OK;
}

int cybq_debug_read_weight(cybq_ctx* ctx, int64_t count, const cybq_weight* const* w, int with_io, const void* x, void* y,
                           void* stream)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (count < 0 || (count > 0 && !w) || (with_io && (!x || !y))) return fail(ctx, CYBQ_ERR_INVALID, "w / x / y is NULL");
    DeviceGuard guard(ctx->device);
    if (guard.err != hipSuccess) return fail_hip(ctx, guard.err, "hipSetDevice");
    for (int64_t i = 0; i < count; i++) {
        if (!w[i]) return fail(ctx, CYBQ_ERR_INVALID, "w[i] is NULL");
        hipError_t e = cybq::launch_read_probe(view_of(w[i]), with_io != 0, x, y, static_cast<hipStream_t>(stream));
        if (e == hipErrorInvalidValue) {
            (void)hipGetLastError();
            return fail(ctx, CYBQ_ERR_UNSUPPORTED, "probe needs K % 512 == 0 and K <= 16384");
        }
        if (e != hipSuccess) return fail_hip(ctx, e, "probe launch");
    }
    return CYBQ_OK;
}

int cybq_debug_read_pattern(cybq_ctx* ctx, int64_t count, const cybq_weight* const* w, int pattern, void* stream)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (count < 0 || (count > 0 && !w)) return fail(ctx, CYBQ_ERR_INVALID, "w is NULL");
    DeviceGuard guard(ctx->device);
    if (guard.err != hipSuccess) return fail_hip(ctx, guard.err, "hipSetDevice");
    for (int64_t i = 0; i < count; i++) {
        if (!w[i]) return fail(ctx, CYBQ_ERR_INVALID, "w[i] is NULL");
        hipError_t e = cybq::launch_read_pattern(view_of(w[i]), pattern, ctx->num_cus, static_cast<hipStream_t>(stream));
        if (e == hipErrorInvalidValue) {
            (void)hipGetLastError();
            return fail(ctx, CYBQ_ERR_UNSUPPORTED, "unknown pattern, or a strip pattern on a tensor that is not Q4 with K = 4096");
        }
        if (e != hipSuccess) return fail_hip(ctx, e, "probe launch");
    }
    return CYBQ_OK;
}

int cybq_debug_mfma_loop(cybq_ctx* ctx, int waves_per_simd, int iters, float* sink, void* stream)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    if (!sink) return fail(ctx, CYBQ_ERR_INVALID, "sink is NULL");
    DeviceGuard guard(ctx->device);
    if (guard.err != hipSuccess) return fail_hip(ctx, guard.err, "hipSetDevice");
    hipError_t e = cybq::launch_mfma_loop(ctx->num_cus, waves_per_simd, iters, sink, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail_hip(ctx, e, "mfma loop launch");
    return CYBQ_OK;
}

int cybq_debug_cache_read(cybq_ctx* ctx, const void* buf, int64_t bytes, int waves, int in_flight, int iters, void* stream)
{
    if (!ctx) return CYBQ_ERR_INVALID;
    DeviceGuard guard(ctx->device);
    if (guard.err != hipSuccess) return fail_hip(ctx, guard.err, "hipSetDevice");
    hipError_t e = cybq::launch_cache_read(buf, bytes, waves, in_flight, iters, ctx->num_cus, static_cast<hipStream_t>(stream));
    if (e == hipErrorInvalidValue) return fail(ctx, CYBQ_ERR_INVALID, "cache read probe: bytes, waves or in_flight out of range");
    if (e != hipSuccess) return fail_hip(ctx, e, "cache read launch");
    return CYBQ_OK;
}

}  // extern "C"
