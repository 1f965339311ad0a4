// gemm.hip - prefill kernel: Y[M,N] = X[M,K] * W^T for M > 16, LDS-tiled MFMA.
//
// A workgroup (4 waves) owns a BM x BN output tile and walks K in steps of 128
// (one native weight tile column = 4 scale groups).  Per step
//   - the NF = BN/16 native weight tiles are read once from HBM/L2 with 128-bit
//     loads, unpacked to exact 16-bit integers (bf16 or f16, matching X) and
//     written to LDS already in MFMA B-operand order;
//   - the X tile is written to LDS in MFMA A-operand order (each wave-wide
//     16 B load is one operand: 16 rows x 32 k);
//   - every wave multiplies its 16*MF rows against all NF column blocks with
//     v_mfma_f32_16x16x32, one scale group per instruction, and folds the f16
//     group scale in fp32 into the accumulators.
// The weight operand is an exact integer and the scale is applied in fp32, so
// the result differs from the fp32 CPU path only by accumulation order.
#include "cybq_device.h"
#include "cybq_internal.h"

namespace cybq {

namespace {

__device__ __forceinline__ uint16_t f32_to_bf16_rne_g(float f)
{
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__device__ __forceinline__ void store_out_g(void* y, int ydt, int64_t idx, float v)
{
    if (ydt == kF32) reinterpret_cast<float*>(y)[idx] = v;
    else if (ydt == kF16) reinterpret_cast<_Float16*>(y)[idx] = (_Float16)v;
    else reinterpret_cast<uint16_t*>(y)[idx] = f32_to_bf16_rne_g(v);
}

// XBF = 1: X is bf16 (bf16 MFMA), 0: X is f16 (f16 MFMA)
template <int BITS, int XBF, int NF, int MF>
__global__ __launch_bounds__(256) void gemm_kernel(WeightView w, const uint16_t* __restrict__ x, int M,
                                                   void* __restrict__ y, int ydt)
{
    constexpr int WAVES = 4;
    constexpr int MFRAGS = WAVES * MF;            // m-fragments per workgroup
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    u32x4_t* xs = reinterpret_cast<u32x4_t*>(smem);                    // [MFRAGS][4][64]
    u32x4_t* ws = xs + MFRAGS * 4 * 64;                                // [NF][4][64]
    const uint32_t magic = q4_magic_vgpr();

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = tid >> 6;
    const int row16 = lane & 15;
    const int oct = lane >> 4;
    const int nt0 = blockIdx.x * NF;
    const int m0 = blockIdx.y * (MFRAGS * 16);
    const int K = w.K;

    float4_t acc[MF][NF];
#pragma unroll
    for (int i = 0; i < MF; i++)
#pragma unroll
        for (int f = 0; f < NF; f++) acc[i][f] = (float4_t){0.f, 0.f, 0.f, 0.f};

    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    const u32x4_t* qp = reinterpret_cast<const u32x4_t*>(w.q);
    const u32x2_t* sp = reinterpret_cast<const u32x2_t*>(w.s);

    for (int kt = 0; kt < w.KT; kt++) {
        __syncthreads();
        // ---- X tile -> LDS, A-operand order
        for (int f = wv; f < MFRAGS * 4; f += WAVES) {
            int i = f >> 2, j = f & 3;
            int row = m0 + i * 16 + row16;
            int k = kt * kTileK + j * 32 + oct * 8;
            u32x4_t v = {0u, 0u, 0u, 0u};
            if (row < M && k < K) v = *reinterpret_cast<const u32x4_t*>(x + (int64_t)row * K + k);
            xs[f * 64 + lane] = v;
        }
        // ---- W tiles -> exact 16-bit integers -> LDS, B-operand order
        for (int f = wv; f < NF; f += WAVES) {
            int nt = nt0 + f;
            u32x4_t q0 = {0x88888888u, 0x88888888u, 0x88888888u, 0x88888888u}, q1 = q0;
            if (BITS == 8) q0 = q1 = (u32x4_t){0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u};
            if (nt < w.NT) {
                int64_t tile = (int64_t)nt * w.KT + kt;
                if (BITS == 4) q0 = qp[tile * 64 + lane];
                else { q0 = qp[tile * 128 + lane]; q1 = qp[tile * 128 + 64 + lane]; }
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                uint32_t bw[4];
                if (BITS == 4) unpack_q4_f16(q0[j], magic, bw);
                else if (j < 2) unpack_q8_f16(q0[(j & 1) * 2], q0[(j & 1) * 2 + 1], bw);
                else unpack_q8_f16(q1[(j & 1) * 2], q1[(j & 1) * 2 + 1], bw);
                if (XBF) f16frag_to_bf16frag(bw);
                ws[(f * 4 + j) * 64 + lane] = (u32x4_t){bw[0], bw[1], bw[2], bw[3]};
            }
        }
        // ---- group scales of this step for every column block (registers)
        float sc[NF][4];
#pragma unroll
        for (int f = 0; f < NF; f++) {
            int nt = nt0 + f;
            u32x2_t sv = {0u, 0u};
            if (nt < w.NT) sv = sp[((int64_t)nt * w.KT + kt) * 16 + row16];
            sc[f][0] = f16_bits_to_f32(sv[0] & 0xffffu);
            sc[f][1] = f16_bits_to_f32(sv[0] >> 16);
            sc[f][2] = f16_bits_to_f32(sv[1] & 0xffffu);
            sc[f][3] = f16_bits_to_f32(sv[1] >> 16);
        }
        __syncthreads();
        // ---- multiply
#pragma unroll
        for (int j = 0; j < 4; j++) {
            Frag16 a[MF];
#pragma unroll
            for (int i = 0; i < MF; i++) a[i].u = xs[((wv * MF + i) * 4 + j) * 64 + lane];
#pragma unroll
            for (int f = 0; f < NF; f++) {
                Frag16 b;
                b.u = ws[(f * 4 + j) * 64 + lane];
                const float s = sc[f][j];
#pragma unroll
                for (int i = 0; i < MF; i++) {
                    float4_t d;
                    if (XBF) d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i].b, b.b, zero, 0, 0, 0);
                    else d = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i].h, b.h, zero, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[i][f][r] = __builtin_fmaf(s, d[r], acc[i][f][r]);
                }
            }
        }
    }

    // ---- epilogue
#pragma unroll
    for (int i = 0; i < MF; i++)
#pragma unroll
        for (int f = 0; f < NF; f++) {
            int n = (nt0 + f) * 16 + row16;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                int m = m0 + (wv * MF + i) * 16 + oct * 4 + r;
                if (m < M && n < w.N) store_out_g(y, ydt, (int64_t)m * w.N + n, acc[i][f][r]);
            }
        }
}

template <int BITS, int XBF, int NF, int MF>
hipError_t launch_t(const WeightView& w, const void* x, int M, void* y, int ydt, hipStream_t st)
{
    constexpr int BM = 4 * MF * 16;
    size_t lds = (size_t)(4 * MF * 4 * 64 + NF * 4 * 64) * 16;
    auto kern = gemm_kernel<BITS, XBF, NF, MF>;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    dim3 grid((unsigned)((w.NT + NF - 1) / NF), (unsigned)((M + BM - 1) / BM));
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, w, reinterpret_cast<const uint16_t*>(x), M, y, ydt);
    return hipGetLastError();
}

template <int BITS, int XBF>
hipError_t launch_nf(const WeightView& w, const void* x, int M, void* y, int ydt, hipStream_t st)
{
    // 7 column blocks (BN = 112) tile N = 14336 = 128 * 112 exactly: with M = 512
    // that is 256 workgroups, one per CU; 8 column blocks otherwise
    if (w.NT % 7 == 0) return launch_t<BITS, XBF, 7, 4>(w, x, M, y, ydt, st);
    return launch_t<BITS, XBF, 8, 4>(w, x, M, y, ydt, st);
}

}  // namespace

hipError_t launch_gemm(const WeightView& w, const void* x, int xdt, int M, void* y, int ydt,
                       int num_cus, hipStream_t st)
{
    (void)num_cus;
    if (xdt == kF32) return hipErrorNotSupported;   // api.hip routes f32 prefill elsewhere
    if (w.bits == 4) {
        if (xdt == kBF16) return launch_nf<4, 1>(w, x, M, y, ydt, st);
        return launch_nf<4, 0>(w, x, M, y, ydt, st);
    }
    if (xdt == kBF16) return launch_nf<8, 1>(w, x, M, y, ydt, st);
    return launch_nf<8, 0>(w, x, M, y, ydt, st);
}

}  // namespace cybq
