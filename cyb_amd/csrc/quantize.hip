// quantize.hip - import-stage quantiser on the device: f32 [N,K] -> PLANAR
// interchange layout (q plane + f16 scale plane).  HBM-bound, one pass:
// 8 lanes share a 32-weight group, each lane owns 4 consecutive weights.
//   d = f16(absmax / qmax), q = clamp(round_half_away(w / f32(d))), d == 0 -> q = 0
#include "cybq_device.h"
#include "cybq_internal.h"

namespace cybq {

namespace {

template <int BITS>
__global__ void quantize_kernel(const float* __restrict__ src, int64_t ngroups, uint8_t* __restrict__ q_out,
                                uint16_t* __restrict__ s_out)
{
    const float qmax = BITS == 4 ? 7.0f : 127.0f;
    const float lo = BITS == 4 ? -8.0f : -127.0f;
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t g = t >> 3;
    const bool live = g < ngroups;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live) v = reinterpret_cast<const float4*>(src)[t];
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, __shfl_xor(amax, 1));
    amax = fmaxf(amax, __shfl_xor(amax, 2));
    amax = fmaxf(amax, __shfl_xor(amax, 4));
    _Float16 dh = (_Float16)(amax / qmax);
    uint16_t dbits = __builtin_bit_cast(uint16_t, dh);
    if ((dbits & 0x7fffu) >= 0x7c00u) { dbits = 0x7bffu; dh = __builtin_bit_cast(_Float16, dbits); }
    const float d = (float)dh;
    float w4[4] = {v.x, v.y, v.z, v.w};
    int qi[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float r = 0.f;
        if (d != 0.f) r = fminf(fmaxf(roundf(w4[i] / d), lo), qmax);
        qi[i] = (int)r;
    }
    if (!live) return;
    if (BITS == 4) {
        uint16_t packed = (uint16_t)((qi[0] & 15) | ((qi[1] & 15) << 4) | ((qi[2] & 15) << 8) | ((qi[3] & 15) << 12));
        reinterpret_cast<uint16_t*>(q_out)[t] = packed;
    } else {
        uint32_t packed = (uint32_t)(qi[0] & 255) | ((uint32_t)(qi[1] & 255) << 8) |
                          ((uint32_t)(qi[2] & 255) << 16) | ((uint32_t)(qi[3] & 255) << 24);
        reinterpret_cast<uint32_t*>(q_out)[t] = packed;
    }
    if ((t & 7) == 0) s_out[g] = dbits;
}

}  // namespace

hipError_t launch_quantize(int bits, const float* src, int N, int K, void* q_out, void* s_out, hipStream_t st)
{
    int64_t ngroups = (int64_t)N * (K / kGroup);
    int64_t threads_total = ngroups * 8;
    const int threads = 256;
    unsigned blocks = (unsigned)((threads_total + threads - 1) / threads);
    if (bits == 4)
        hipLaunchKernelGGL(quantize_kernel<4>, dim3(blocks), dim3(threads), 0, st, src, ngroups,
                           (uint8_t*)q_out, (uint16_t*)s_out);
    else
        hipLaunchKernelGGL(quantize_kernel<8>, dim3(blocks), dim3(threads), 0, st, src, ngroups,
                           (uint8_t*)q_out, (uint16_t*)s_out);
    return hipGetLastError();
}

}  // namespace cybq
