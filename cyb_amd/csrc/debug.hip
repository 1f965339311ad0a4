// debug.hip - measurement probes declared in cybq_debug.h (not part of the operator interface).
#include "cybq_device.h"
#include "cybq_internal.h"

namespace cybq {

namespace {

// The one-row decode kernel's requests without its arithmetic: wave wv of a strip's workgroup
// owns the sets (four consecutive K tiles) wv, wv + nwaves, ...
template <int BITS, int SETS, bool IO>
// (scalar arguments, delivered in registers at wave start like the decode kernel's)
__global__ __launch_bounds__(1024) void read_probe_kernel(const uint8_t* __restrict__ wbase, const _Float16* __restrict__ x, int KT,
                                                          int nwaves, float* __restrict__ y)
{
    constexpr int QV = BITS == 4 ? 1 : 2;
    constexpr int TB = kTileBytes<BITS>, QB = kTileQBytes<BITS>;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row = lane & 15, blk = lane >> 4;
    const int strip_tile = (int)blockIdx.x * KT;
    u32x4_t a[SETS], q[SETS][4][QV];
    u32x2_t sc[SETS];
#pragma unroll
    for (int h = 0; h < SETS; h++) {
        const int set = wv + nwaves * h;
        if (IO) a[h] = *reinterpret_cast<const u32x4_t*>(x + set * 512 + row * 32 + blk * 8);
        const uint8_t* sb = wbase + (int64_t)(strip_tile + 4 * set) * TB;
        sc[h] = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(sb + ((uint32_t)blk * TB + QB + row * 8)));
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
            for (int v = 0; v < QV; v++)
                q[h][b][v] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(sb + (b * TB + v * 1024) + lane * 16));
    }
    uint32_t r = 0;
#pragma unroll
    for (int h = 0; h < SETS; h++) {
        r ^= sc[h][0] ^ sc[h][1];
        if (IO) r ^= a[h][0] ^ a[h][3];
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
            for (int v = 0; v < QV; v++) r ^= q[h][b][v][0] ^ q[h][b][v][1] ^ q[h][b][v][2] ^ q[h][b][v][3];
    }
    if (IO && tid < 16) y[blockIdx.x * 16 + tid] = (float)r;
    if (r == 0x12345679u && y) y[0] = 1.f;              // never true in practice: keeps every wave's loads alive
}

__global__ __launch_bounds__(256) void mfma_loop_kernel(int iters, float* __restrict__ sink)
{
    Frag16 a, b;
    const uint32_t one2 = 0x3C003C00u;
    a.u = (u32x4_t){one2, one2, one2, one2};
    b.u = (u32x4_t){threadIdx.x, one2, one2, one2};
    float4_t acc[16];
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = (float4_t){0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 16; i++) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a.h, b.h, acc[i], 0, 0, 0);
    }
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) t += acc[i][0];
    if (t == 12345.678f) sink[0] = t;
}

}  // namespace

hipError_t launch_read_probe(const WeightView& w, bool io, const void* x, void* y, hipStream_t st)
{
    const int nsets = w.KT / 4;
    if (w.K % 512 || nsets < 1 || nsets > 32) return hipErrorInvalidValue;
    const int per_wave = (nsets + 15) / 16;
    if (nsets % per_wave) return hipErrorInvalidValue;
    const dim3 grid((unsigned)w.NT), block((unsigned)(nsets / per_wave) * 64);
    const _Float16* xp = reinterpret_cast<const _Float16*>(x);
    float* yp = reinterpret_cast<float*>(y);
#define CYBQ_PROBE(B, S)                                                                                            \
    do {                                                                                                            \
        if (io) hipLaunchKernelGGL((read_probe_kernel<B, S, true>), grid, block, 0, st, w.base, xp, w.KT, (int)block.x >> 6, yp); \
        else hipLaunchKernelGGL((read_probe_kernel<B, S, false>), grid, block, 0, st, w.base, xp, w.KT, (int)block.x >> 6, yp);  \
    } while (0)
    if (w.bits == 4 && per_wave == 1) CYBQ_PROBE(4, 1);
    else if (w.bits == 4) CYBQ_PROBE(4, 2);
    else if (per_wave == 1) CYBQ_PROBE(8, 1);
    else CYBQ_PROBE(8, 2);
#undef CYBQ_PROBE
    return hipGetLastError();
}

hipError_t launch_mfma_loop(int num_cus, int waves_per_simd, int iters, float* sink, hipStream_t st)
{
    if (waves_per_simd < 1 || waves_per_simd > 8 || iters < 1) return hipErrorInvalidValue;
    // 256 threads = one wave per SIMD of a CU; waves_per_simd such workgroups per CU
    hipLaunchKernelGGL(mfma_loop_kernel, dim3((unsigned)(num_cus * waves_per_simd)), dim3(256), 0, st, iters, sink);
    return hipGetLastError();
}

}  // namespace cybq
