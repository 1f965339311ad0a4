// layout.hip - interchange layout -> native tiled layout (once, at upload) and
// the exact dequantise kernel used to verify "dequantised weights bit-exact".
#include "cybq_device.h"
#include "cybq_internal.h"

namespace cybq {

namespace {

// Bytes one scale group occupies in a row of the interchange buffer.
template <int BITS, int LAYOUT>
constexpr int kSrcGroupBytes = LAYOUT == 0 ? (BITS == 4 ? 16 : 32) : (BITS == 4 ? 18 : 34);

// signed weight i (0..31) of group `gl` of a staged source row ---------------------
template <int BITS, int LAYOUT>
__device__ __forceinline__ int staged_weight(const uint8_t* row, int gl, int i)
{
    const uint8_t* g = row + gl * kSrcGroupBytes<BITS, LAYOUT>;
    if (LAYOUT == 0) {                               // PLANAR
        if (BITS == 8) return (int)(int8_t)g[i];
        const uint8_t b = g[i >> 1];
        const int nib = (i & 1) ? (b >> 4) : (b & 15);
        return (nib & 8) ? nib - 16 : nib;
    }
    if (BITS == 8) return (int)(int8_t)g[2 + i];     // BLOCK_AOS: f16 d, then the weights
    const uint8_t b = g[2 + (i & 15)];
    return (int)((i < 16) ? (b & 15) : (b >> 4)) - 8;
}

// A lane's share of one scale group (the 8 weights k = 8 * oct + s of row `row`) as eight
// offset-8 nibbles in native order within a word pair: weight s sits in byte {0, 2, 1, 3}[s & 3]
// of word s >> 2, low nibble (the caller shifts odd groups into the high nibbles).
template <int LAYOUT>
__device__ __forceinline__ void staged_q4_octet(const uint8_t* row, int gl, int oct, uint32_t& lo, uint32_t& hi)
{
    if (LAYOUT == 0) {
        // PLANAR: weight i is nibble i of the group's 16 bytes (two's complement): one aligned word
        const uint32_t src = *reinterpret_cast<const uint32_t*>(row + gl * 16 + oct * 4) ^ 0x88888888u;
        const uint32_t a = src & 0xffffu, b = src >> 16;
        lo = (a & 0x0f0fu) | (((a >> 4) & 0x0f0fu) << 16);
        hi = (b & 0x0f0fu) | (((b >> 4) & 0x0f0fu) << 16);
    } else {
        // BLOCK_AOS: weights 0..15 are the low nibbles of the 16 bytes behind the f16 scale, 16..31
        // the high nibbles (already offset-8); the bytes are only 2-byte aligned
        const uint16_t* p = reinterpret_cast<const uint16_t*>(row + gl * 18 + 2 + (oct & 1) * 8);
        const uint32_t w0 = (uint32_t)p[0] | ((uint32_t)p[1] << 16), w1 = (uint32_t)p[2] | ((uint32_t)p[3] << 16);
        const int sh = (oct >> 1) * 4;
        const uint32_t t0 = (w0 >> sh) & 0x0f0f0f0fu, t1 = (w1 >> sh) & 0x0f0f0f0fu;
        lo = __builtin_amdgcn_perm(t0, t0, 0x03010200u);       // bytes 1 and 2 change places
        hi = __builtin_amdgcn_perm(t1, t1, 0x03010200u);
    }
}

// One workgroup repacks CT consecutive K tiles of one 16-row strip.  The source rows of
// that piece are first copied into LDS with coalesced loads (a row's piece is one
// contiguous run in either interchange layout), then every thread assembles one lane's
// share of a native tile from LDS - a few aligned words and a handful of bit operations -
// and stores it with 128-bit stores: global memory only sees whole runs, the gathering
// stays inside the CU.
constexpr int kRepackTiles = 4;

template <int BITS, int LAYOUT>
__global__ __launch_bounds__(256) void repack_kernel(const uint8_t* __restrict__ q, const uint16_t* __restrict__ scales,
                                                      uint8_t* __restrict__ dst, int N, int K, int KT, uint32_t* __restrict__ wide_flag)
{
    constexpr int CT = kRepackTiles;
    constexpr int GB = kSrcGroupBytes<BITS, LAYOUT>;
    constexpr int ROWB = CT * kGroupsPerTile * GB;                  // bytes of one row's piece
    constexpr int UNIT = LAYOUT == 0 ? 16 : 2;                      // load width the source alignment allows
    constexpr int UPR = ROWB / UNIT;                                // units per row
    constexpr int PITCH = ROWB + (LAYOUT == 0 ? 16 : 4);            // (rows land in different LDS banks)
    __shared__ __attribute__((aligned(16))) uint8_t rows[kTileN][PITCH];

    const int t = threadIdx.x;
    const int chunks = (KT + CT - 1) / CT;
    const int nt = (int)(blockIdx.x / (unsigned)chunks), kt0 = (int)(blockIdx.x % (unsigned)chunks) * CT;
    const int G = K / kGroup;
    const int g0 = kt0 * kGroupsPerTile;
    const int ng = min(CT * kGroupsPerTile, G - g0);                // groups of this piece that exist
    for (int i = t; i < kTileN * UPR; i += 256) {
        const int r = i / UPR, u = i - r * UPR;
        const int64_t n = (int64_t)nt * kTileN + r;
        if (n < N && u * UNIT < ng * GB) {
            const uint8_t* src = q + (n * G + g0) * GB + u * UNIT;
            if (UNIT == 16) *reinterpret_cast<u32x4_t*>(&rows[r][u * 16]) = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(src));
            else *reinterpret_cast<uint16_t*>(&rows[r][u * 2]) = *reinterpret_cast<const uint16_t*>(src);
        }
    }
    __syncthreads();

    const int b = t >> 6, lane = t & 63;
    const int kt = kt0 + b;
    if (kt >= KT) return;
    const int row = lane & 15, oct = lane >> 4;
    const bool row_ok = (int64_t)nt * kTileN + row < N;
    uint8_t* tile = dst + ((int64_t)nt * KT + kt) * kTileBytes<BITS>;
    if (BITS == 4) {
        uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int gl = b * 4 + j;
            uint32_t lo = 0x08080808u, hi = 0x08080808u;             // q = 0 where the source has nothing
            if (row_ok && gl < ng) staged_q4_octet<LAYOUT>(rows[row], gl, oct, lo, hi);
            w[2 * (j >> 1)] |= lo << (4 * (j & 1));
            w[2 * (j >> 1) + 1] |= hi << (4 * (j & 1));
        }
        reinterpret_cast<u32x4_t*>(tile)[lane] = (u32x4_t){w[0], w[1], w[2], w[3]};
    } else {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int wd = 0; wd < 4; wd++) {
                const int gl = b * 4 + 2 * h + (wd >> 1);
                const bool ok = row_ok && gl < ng;
#pragma unroll
                for (int s = 0; s < 4; s++) {
                    const int v = ok ? staged_weight<8, LAYOUT>(rows[row], gl, oct * 8 + (wd & 1) * 4 + s) : 0;
                    w[wd] |= (uint32_t)((v + 128) & 255) << (8 * s);
                }
            }
            reinterpret_cast<u32x4_t*>(tile)[h * 64 + lane] = (u32x4_t){w[0], w[1], w[2], w[3]};
        }
    }
    // the tile's 64 scales: [row][group]
    {
        const int r = lane >> 2, j = lane & 3;
        const int gl = b * 4 + j;
        const int64_t n = (int64_t)nt * kTileN + r;
        uint16_t v = 0;
        if (n < N && gl < ng) {
            if (LAYOUT == 0) v = scales[n * G + g0 + gl];
            else v = (uint16_t)(rows[r][gl * GB] | (rows[r][gl * GB + 1] << 8));
        }
        reinterpret_cast<uint16_t*>(tile + kTileQBytes<BITS>)[lane] = v;
        // a scale whose product with the largest q leaves f16 (or that is not finite): the prefill kernels, which
        // form scale * q in f16, cannot serve this tensor; every thread that sees one stores the same 1
        if (wide_flag) {
            const bool wide = ((v >> 10) & 31u) == 31u || f16_bits_to_f32(v & 0x7fffu) * (BITS == 4 ? 8.0f : 128.0f) > 65504.0f;
            if (wide) *wide_flag = 1u;
        }
    }
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
    const uint16_t* sp = reinterpret_cast<const uint16_t*>(tile_s<BITS>(w, tile));
    float d = f16_bits_to_f32(sp[row * 4 + j]);
    float v[8];
    if (BITS == 4) {
        const u32x4_t lw = tile_q<4>(w, tile)[lane];
        const uint32_t words[4] = {lw[0], lw[1], lw[2], lw[3]};
#pragma unroll
        for (int s = 0; s < 8; s++) v[s] = d * (float)q4_slot_value(words, j, s);
    } else {
        const u32x4_t lw = tile_q<8>(w, tile)[(j >> 1) * 64 + lane];
        uint32_t w0 = lw[(j & 1) * 2], w1 = lw[(j & 1) * 2 + 1];
#pragma unroll
        for (int s = 0; s < 8; s++) v[s] = d * (float)q8_slot_value(w0, w1, s);
    }
    float4* o = reinterpret_cast<float4*>(out + n * w.K + k0);
    o[0] = make_float4(v[0], v[1], v[2], v[3]);
    o[1] = make_float4(v[4], v[5], v[6], v[7]);
}

template <int BITS, int LAYOUT>
hipError_t launch_repack_t(const void* q, const void* scales, uint8_t* dst, int N, int K, int NT, int KT, uint32_t* wide_flag,
                           hipStream_t st)
{
    const int64_t groups = (int64_t)((KT + kRepackTiles - 1) / kRepackTiles) * NT;
    if (groups > 0x7fffffff) return hipErrorInvalidValue;
    hipLaunchKernelGGL((repack_kernel<BITS, LAYOUT>), dim3((unsigned)groups), dim3(256), 0, st, (const uint8_t*)q, (const uint16_t*)scales, dst, N, K,
                       KT, wide_flag);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_repack(int bits, int layout, const void* q, const void* scales, uint8_t* dst, int N, int K, int NT, int KT,
                         uint32_t* wide_flag, hipStream_t st)
{
    if (bits == 4 && layout == 0) return launch_repack_t<4, 0>(q, scales, dst, N, K, NT, KT, wide_flag, st);
    if (bits == 4 && layout == 1) return launch_repack_t<4, 1>(q, scales, dst, N, K, NT, KT, wide_flag, st);
    if (bits == 8 && layout == 0) return launch_repack_t<8, 0>(q, scales, dst, N, K, NT, KT, wide_flag, st);
    if (bits == 8 && layout == 1) return launch_repack_t<8, 1>(q, scales, dst, N, K, NT, KT, wide_flag, st);
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
