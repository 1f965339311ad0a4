// layout.hip - interchange layout -> native tiled layout (once, at upload) and
// the exact dequantise kernel used to verify "dequantised weights bit-exact".
#include "cybq_device.h"
#include "cybq_internal.h"

namespace cybq {

// signed weight and f16 scale bits from an interchange buffer ------------------

template <int BITS, int LAYOUT>
__device__ __forceinline__ int src_weight(const uint8_t* q, int64_t n, int64_t k, int64_t K)
{
    if (LAYOUT == 0) {                               // PLANAR
        if (BITS == 8) return (int)(int8_t)q[n * K + k];
        uint8_t b = q[(n * K + k) >> 1];
        int nib = (k & 1) ? (b >> 4) : (b & 15);
        return (nib & 8) ? nib - 16 : nib;
    } else {                                         // BLOCK_AOS
        const int bs = BITS == 4 ? 18 : 34;
        const uint8_t* blk = q + (n * (K / kGroup) + k / kGroup) * bs + 2;
        int i = (int)(k % kGroup);
        if (BITS == 8) return (int)(int8_t)blk[i];
        uint8_t b = blk[i & 15];
        return (int)((i < 16) ? (b & 15) : (b >> 4)) - 8;
    }
}

template <int BITS, int LAYOUT>
__device__ __forceinline__ uint16_t src_scale(const uint8_t* q, const uint16_t* scales,
                                              int64_t n, int64_t g, int64_t K)
{
    if (LAYOUT == 0) return scales[n * (K / kGroup) + g];
    const int bs = BITS == 4 ? 18 : 34;
    const uint8_t* blk = q + (n * (K / kGroup) + g) * bs;
    return (uint16_t)(blk[0] | (blk[1] << 8));
}

// One thread per native 32-bit q word.
template <int BITS, int LAYOUT>
__global__ void repack_q_kernel(const uint8_t* __restrict__ q, uint32_t* __restrict__ dst,
                                int N, int K, int NT, int KT)
{
    const int words_per_tile = BITS == 4 ? 256 : 512;
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t total = (int64_t)NT * KT * words_per_tile;
    if (idx >= total) return;
    int64_t tile = idx / words_per_tile;
    int r = (int)(idx % words_per_tile);
    int nt = (int)(tile / KT), kt = (int)(tile % KT);
    uint32_t out = 0;
    if (BITS == 4) {
        int lane = r >> 2, j = r & 3;
        int64_t n = (int64_t)nt * 16 + (lane & 15);
        int64_t k0 = (int64_t)kt * 128 + j * 32 + (lane >> 4) * 8;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            int v = 0;
            if (n < N && k0 + s < K) v = src_weight<4, LAYOUT>(q, n, k0 + s, K);
            out |= (uint32_t)((v + 8) & 15) << (4 * q4_nibble_pos(s));
        }
    } else {
        int h = r >> 8, lane = (r >> 2) & 63, wd = r & 3;     // half, lane, word in lane
        int64_t n = (int64_t)nt * 16 + (lane & 15);
        int j = 2 * h + (wd >> 1);
        int64_t k0 = (int64_t)kt * 128 + j * 32 + (lane >> 4) * 8 + (wd & 1) * 4;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            int v = 0;
            if (n < N && k0 + s < K) v = src_weight<8, LAYOUT>(q, n, k0 + s, K);
            out |= (uint32_t)((v + 128) & 255) << (8 * s);
        }
    }
    dst[idx] = out;
}

// One thread per native scale.
template <int BITS, int LAYOUT>
__global__ void repack_s_kernel(const uint8_t* __restrict__ q, const uint16_t* __restrict__ scales,
                                uint16_t* __restrict__ dst, int N, int K, int NT, int KT)
{
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t total = (int64_t)NT * KT * 64;
    if (idx >= total) return;
    int64_t tile = idx >> 6;
    int r = (int)(idx & 63);
    int nt = (int)(tile / KT), kt = (int)(tile % KT);
    int64_t n = (int64_t)nt * 16 + (r >> 2);
    int64_t g = (int64_t)kt * 4 + (r & 3);
    uint16_t v = 0;
    if (n < N && g * kGroup < K) v = src_scale<BITS, LAYOUT>(q, scales, n, g, K);
    dst[idx] = v;
}

// native -> f32 [N,K].  One thread per 8 consecutive k of one row.
template <int BITS>
__global__ void dequant_kernel(WeightView w, float* __restrict__ out)
{
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t octets_per_row = w.K / 8;
    if (idx >= (int64_t)w.N * octets_per_row) return;
    int64_t n = idx / octets_per_row;
    int64_t k0 = (idx % octets_per_row) * 8;
    int nt = (int)(n >> 4), row = (int)(n & 15);
    int kt = (int)(k0 >> 7), j = (int)((k0 >> 5) & 3), oct = (int)((k0 >> 3) & 3);
    int lane = oct * 16 + row;
    int64_t tile = (int64_t)nt * w.KT + kt;
    float d = f16_bits_to_f32(w.s[tile * 64 + row * 4 + j]);
    float v[8];
    if (BITS == 4) {
        uint32_t word = w.q[(tile * 64 + lane) * 4 + j];
#pragma unroll
        for (int s = 0; s < 8; s++) v[s] = d * (float)q4_slot_value(word, s);
    } else {
        const uint32_t* p = w.q + tile * 512 + (j >> 1) * 256 + lane * 4 + (j & 1) * 2;
        uint32_t w0 = p[0], w1 = p[1];
#pragma unroll
        for (int s = 0; s < 8; s++) v[s] = d * (float)q8_slot_value(w0, w1, s);
    }
    float4* o = reinterpret_cast<float4*>(out + n * w.K + k0);
    o[0] = make_float4(v[0], v[1], v[2], v[3]);
    o[1] = make_float4(v[4], v[5], v[6], v[7]);
}

template <int BITS, int LAYOUT>
static hipError_t launch_repack_t(const void* q, const void* scales, uint32_t* qdst, uint16_t* sdst,
                                  int N, int K, int NT, int KT, hipStream_t st)
{
    const int threads = 256;
    int64_t qwords = (int64_t)NT * KT * (BITS == 4 ? 256 : 512);
    int64_t swords = (int64_t)NT * KT * 64;
    hipLaunchKernelGGL((repack_q_kernel<BITS, LAYOUT>), dim3((unsigned)((qwords + threads - 1) / threads)),
                       dim3(threads), 0, st, (const uint8_t*)q, qdst, N, K, NT, KT);
    hipLaunchKernelGGL((repack_s_kernel<BITS, LAYOUT>), dim3((unsigned)((swords + threads - 1) / threads)),
                       dim3(threads), 0, st, (const uint8_t*)q, (const uint16_t*)scales, sdst, N, K, NT, KT);
    return hipGetLastError();
}

hipError_t launch_repack(int bits, int layout, const void* q, const void* scales, uint32_t* qdst,
                         uint16_t* sdst, int N, int K, int NT, int KT, hipStream_t st)
{
    if (bits == 4 && layout == 0) return launch_repack_t<4, 0>(q, scales, qdst, sdst, N, K, NT, KT, st);
    if (bits == 4 && layout == 1) return launch_repack_t<4, 1>(q, scales, qdst, sdst, N, K, NT, KT, st);
    if (bits == 8 && layout == 0) return launch_repack_t<8, 0>(q, scales, qdst, sdst, N, K, NT, KT, st);
    if (bits == 8 && layout == 1) return launch_repack_t<8, 1>(q, scales, qdst, sdst, N, K, NT, KT, st);
    return hipErrorInvalidValue;
}

hipError_t launch_dequant(const WeightView& w, float* out, hipStream_t st)
{
    const int threads = 256;
    int64_t total = (int64_t)w.N * (w.K / 8);
    unsigned blocks = (unsigned)((total + threads - 1) / threads);
    if (w.bits == 4) hipLaunchKernelGGL(dequant_kernel<4>, dim3(blocks), dim3(threads), 0, st, w, out);
    else             hipLaunchKernelGGL(dequant_kernel<8>, dim3(blocks), dim3(threads), 0, st, w, out);
    return hipGetLastError();
}

}  // namespace cybq
