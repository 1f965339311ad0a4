// gemm.hip - prefill kernel: Y[M,N] = X[M,K] * W^T for M > 16 on MFMA.
//
// Workgroup = 4 or 8 waves, output tile 256 or 128 rows x (16*NF) columns; wave w owns
// its share of the rows (4 or 2 row blocks of 16) against all NF column blocks.
//
//   X  never touches LDS.  An MFMA A operand is 16 rows x 32 k with lane l
//      holding row l%16, k 8*(l/16)..+8 - exactly a 16 B global load per lane -
//      and every wave consumes only its own rows, so X streams global ->
//      registers, one K tile (four scale groups) ahead of its use.
//   W  is shared by the four waves: per K tile (128 k = 4 groups) the NF native
//      weight tiles are read once with 128-bit loads and dequantised to
//      w = f32(scale) * q, which is exact in fp32 (11-bit x 4-bit significand).
//      A 16-bit MFMA operand cannot hold those 15 bits, so w is split without
//      loss into hi = round16(w) and lo = w - hi (both exactly representable)
//      and written to LDS as two operands, already in MFMA B-operand order.
//      LDS is double buffered, one barrier per K tile.
//   The inner loop is nothing but LDS operand reads and v_mfma_f32_16x16x32
//      accumulating hi and lo products in fp32: no per-group scaling on the
//      vector ALU, accumulators stay inside the matrix pipeline until the
//      epilogue.  The price is two MFMAs per scale group; the gain is that the
//      weights enter the contraction exactly, so the result differs from the
//      fp32 CPU path only by accumulation order.  (Q8 weights need 18 bits; lo
//      is then rounded and the split is exact to 2^-17 relative.)
//
// Two modes share this kernel:
//   EXACT  as described above: two MFMAs per scale group in the type of X.
//   FAST   one f16 MFMA per scale group.  The weight operand is round_f16(scale * q)
//          (one rounding, relative error <= 2^-11, about 2e-4 relative L2 on Y -
//          inside the operator's 1e-3 tolerance); bf16 activations are widened
//          to f16 in registers after a 2^-4 prescale that is undone in the
//          epilogue, exact for 2^-10 <= |x| < 2^20.
//
// Out-of-range rows / columns / k are clamped to valid addresses inside the hot
// loop (their results are never stored, padded weights are zero); the loop has
// no branches, so the compiler can count outstanding loads exactly.
#include <type_traits>

#include "cybq_device.h"
#include "cybq_internal.h"

namespace cybq {

namespace {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));

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


template <int BITS>
struct WRegs {               // one native weight tile as loaded by one lane, and its 4 group scales
    u32x4_t q[BITS == 4 ? 1 : 2];
    u32x2_t s;
};

template <int BITS>
__device__ __forceinline__ void load_wtile(WRegs<BITS>& r, const u32x4_t* qp, const u32x2_t* sp, int64_t tile,
                                           int lane)
{
    if (BITS == 4) {
        r.q[0] = qp[tile * 64 + lane];
    } else {
        r.q[0] = qp[tile * 128 + lane];
        r.q[BITS == 4 ? 0 : 1] = qp[tile * 128 + 64 + lane];
    }
    r.s = sp[tile * 16 + (lane & 15)];
}

// (w0, w1) fp32 -> packed 16-bit hi pair and lo pair with hi + lo == w
template <int XBF>
__device__ __forceinline__ void split_pair(float w0, float w1, uint32_t& hi, uint32_t& lo)
{
    if (XBF) {
        bf16x2_t h = __builtin_convertvector((float2_t){w0, w1}, bf16x2_t);
        hi = __builtin_bit_cast(uint32_t, h);
        float h0 = __builtin_bit_cast(float, hi << 16);
        float h1 = __builtin_bit_cast(float, hi & 0xffff0000u);
        bf16x2_t l = __builtin_convertvector((float2_t){w0 - h0, w1 - h1}, bf16x2_t);
        lo = __builtin_bit_cast(uint32_t, l);
    } else {
        half2_t h = {(_Float16)w0, (_Float16)w1};
        hi = as_u32(h);
        half2_t l = {(_Float16)(w0 - (float)h.x), (_Float16)(w1 - (float)h.y)};
        lo = as_u32(l);
    }
}

// group j of a native tile -> B operand(s) in LDS: hi and lo (EXACT) or one rounded f16 operand
template <int BITS, int XBF, bool EXACT>
__device__ __forceinline__ void dequant_group_to_lds(const WRegs<BITS>& r, int j, uint32_t magic, u32x4_t* dst,
                                                     int lane)
{
    uint32_t bw[4];
    if (BITS == 4) unpack_q4_f16(r.q[0][j], magic, bw);
    else unpack_q8_f16(r.q[(BITS == 4) ? 0 : (j >> 1)][(j & 1) * 2], r.q[(BITS == 4) ? 0 : (j >> 1)][(j & 1) * 2 + 1], bw);
    const uint32_t sb = (j & 1) ? (r.s[j >> 1] >> 16) : (r.s[j >> 1] & 0xffffu);
    if (!EXACT) {
        const _Float16 sh = __builtin_bit_cast(_Float16, (uint16_t)sb);
        const half2_t s2 = {sh, sh};
        uint32_t o[4];
#pragma unroll
        for (int p = 0; p < 4; p++) o[p] = as_u32(as_h2(bw[p]) * s2);     // round_f16(scale * q)
        dst[j * 64 + lane] = (u32x4_t){o[0], o[1], o[2], o[3]};
        return;
    }
    const float sc = f16_bits_to_f32(sb);
    uint32_t hi[4], lo[4];
#pragma unroll
    for (int p = 0; p < 4; p++) {
        half2_t qv = as_h2(bw[p]);
        split_pair<XBF>(sc * (float)qv.x, sc * (float)qv.y, hi[p], lo[p]);
    }
    dst[(j * 2 + 0) * 64 + lane] = (u32x4_t){hi[0], hi[1], hi[2], hi[3]};
    dst[(j * 2 + 1) * 64 + lane] = (u32x4_t){lo[0], lo[1], lo[2], lo[3]};
}

template <int XBF>
__device__ __forceinline__ float4_t mma(const Frag16& a, const Frag16& b, float4_t c)
{
    if (XBF) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, b.b, c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a.h, b.h, c, 0, 0, 0);
}

// bf16 A operand -> f16 A operand, prescaled by 2^-4
__device__ __forceinline__ Frag16 bf16_to_f16_frag(const Frag16& a)
{
    Frag16 o;
#pragma unroll
    for (int p = 0; p < 4; p++) {
        float f0 = __builtin_bit_cast(float, a.u[p] << 16);
        float f1 = __builtin_bit_cast(float, a.u[p] & 0xffff0000u);
        half2_t h = {(_Float16)(f0 * 0.0625f), (_Float16)(f1 * 0.0625f)};
        o.u[p] = as_u32(h);
    }
    return o;
}

// XBF = 1: X is bf16, 0: X is f16.  EXACT: see the header comment.
template <int BITS, int XBF, int NF, bool EXACT, int MF, int WAVES>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(MF == 4 ? 1 : 2, MF == 4 ? 1 : 2))) void gemm_kernel(WeightView w, const uint16_t* __restrict__ x, int M,
                                                   void* __restrict__ y, int ydt, int n_tiles, int m_tiles, float out_scale)
{
    // Workgroups are handed to the 8 XCDs round-robin (id % 8) and every XCD has
    // its own L2.  Give each XCD a contiguous run of tiles in row-block-major
    // order, so the workgroups sharing an L2 read the same rows of X and X is
    // fetched into every L2 once instead of once per column tile.
    const int per_xcd = (int)gridDim.x >> 3;
    const int item = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
    if (item >= n_tiles * m_tiles) return;
    const int tile_m = item / n_tiles;
    const int tile_n = item - tile_m * n_tiles;
    constexpr int BM = WAVES * MF * 16;               // MF = row blocks (of 16) per wave
    constexpr int WT = (NF + WAVES - 1) / WAVES;      // weight tiles a wave stages per K tile
    constexpr int OPS = EXACT ? 2 : 1;                // B operands per scale group
    constexpr int TILE16 = 4 * OPS * 64;              // u32x4 per column block per buffer
    constexpr int MMA_BF = EXACT ? XBF : 0;           // FAST always multiplies in f16
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    u32x4_t* ws = reinterpret_cast<u32x4_t*>(smem);   // [2][NF][4][2][64]
    const uint32_t magic = q4_magic_vgpr();

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row16 = lane & 15;
    const int oct = lane >> 4;
    const int nt0 = tile_n * NF;
    const int m0 = tile_m * BM + wv * (MF * 16);
    const int K = w.K, KT = w.KT;

    const u32x4_t* qp = reinterpret_cast<const u32x4_t*>(w.q);
    const u32x2_t* sp = reinterpret_cast<const u32x2_t*>(w.s);

    // X addressing: a wave-uniform byte pointer (row block base + k) plus a 32-bit
    // per-lane byte offset (row within the tile, k octet), so a load costs no vector
    // ALU work.  Rows past M-1 are clamped to M-1 (never stored); a scale group past
    // K (padding, zero weights) reads the last real group instead - K % 32 == 0, so
    // the clamp is uniform.
    const char* xtile = reinterpret_cast<const char*>(x + (int64_t)tile_m * BM * K);
    uint32_t xoff[MF];
#pragma unroll
    for (int i = 0; i < MF; i++) {
        const int row = min(m0 + i * 16 + row16, M - 1) - tile_m * BM;
        xoff[i] = (uint32_t)(((int64_t)row * K + oct * 8) * 2);
    }
    auto load_x = [&](Frag16 (&dst)[MF], int kstart) {
        const char* base = xtile + (int64_t)min(kstart, K - 32) * 2;
#pragma unroll
        for (int i = 0; i < MF; i++) dst[i].u = *reinterpret_cast<const u32x4_t*>(base + xoff[i]);
    };

    // the weight tiles this wave stages: column block f = wv + WAVES*t (clamped)
    int64_t wtile[WT];
    int wf[WT];
#pragma unroll
    for (int t = 0; t < WT; t++) {
        wf[t] = min(wv + WAVES * t, NF - 1);
        wtile[t] = (int64_t)min(nt0 + wf[t], w.NT - 1) * KT;
    }

    float4_t acc[MF][NF];
#pragma unroll
    for (int i = 0; i < MF; i++)
#pragma unroll
        for (int f = 0; f < NF; f++) acc[i][f] = (float4_t){0.f, 0.f, 0.f, 0.f};

    // ---- prologue: first K tile of X, W tile 0 -> LDS buffer 0, W tile 1 -> registers
    Frag16 xa[4][MF];          // one K tile (four scale groups) of X in flight
#pragma unroll
    for (int j = 0; j < 4; j++) load_x(xa[j], j * 32);
    WRegs<BITS> wreg[2][WT];   // packed weights: K tile t waits in wreg[t & 1]
    {
        WRegs<BITS> w0[WT];
#pragma unroll
        for (int t = 0; t < WT; t++) load_wtile<BITS>(w0[t], qp, sp, wtile[t], lane);
#pragma unroll
        for (int t = 0; t < WT; t++) load_wtile<BITS>(wreg[1][t], qp, sp, wtile[t] + min(1, KT - 1), lane);
#pragma unroll
        for (int t = 0; t < WT; t++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                dequant_group_to_lds<BITS, XBF, EXACT>(w0[t], j, magic, ws + wf[t] * TILE16, lane);
    }
    __syncthreads();

    // One K tile.  P = kt & 1 is a compile-time constant (the loop below is unrolled
    // by two), so LDS buffers and register sets alternate without copies or selects:
    //   multiply from LDS buffer P;  dequantise tile kt+1 (wreg[1-P], requested one
    //   iteration ago: its HBM latency is behind us) into LDS buffer 1-P;  request
    //   tile kt+2 into wreg[P].  Past the end indices are clamped: a tile is staged
    //   again but never read.
    auto k_tile = [&](int kt, auto parity) {
        constexpr int P = decltype(parity)::value;
        const u32x4_t* wcur = ws + P * (NF * TILE16);
        u32x4_t* wnxt = ws + (1 - P) * (NF * TILE16);
        const int ktn = min(kt + 2, KT - 1);
#pragma unroll
        for (int t = 0; t < WT; t++) load_wtile<BITS>(wreg[P][t], qp, sp, wtile[t] + ktn, lane);

#pragma unroll
        for (int j = 0; j < 4; j++) {
            Frag16 cv[MF];
            if (!EXACT && XBF) {
#pragma unroll
                for (int i = 0; i < MF; i++) cv[i] = bf16_to_f16_frag(xa[j][i]);
            }
            const Frag16 (&a)[MF] = (!EXACT && XBF) ? cv : xa[j];
#pragma unroll
            for (int f = 0; f < NF; f++) {
                Frag16 b[OPS];
#pragma unroll
                for (int o = 0; o < OPS; o++) b[o].u = wcur[f * TILE16 + (j * OPS + o) * 64 + lane];
#pragma unroll
                for (int o = 0; o < OPS; o++)
#pragma unroll
                    for (int i = 0; i < MF; i++) acc[i][f] = mma<MMA_BF>(a[i], b[o], acc[i][f]);
            }
            // After an odd group its pair of operand sets is free: refill both with
            // the same groups of the next K tile.  The two loads of a row hit the
            // two halves of one 128 B line back to back.
            if (j & 1) {
                load_x(xa[j - 1], (kt + 1) * kTileK + (j - 1) * 32);
                load_x(xa[j], (kt + 1) * kTileK + j * 32);
            }
            // a quarter of the next tile's dequantisation rides along with every group
            // (a wave whose tile index is clamped rewrites a neighbour's block with
            // identical values: no branch in the hot loop)
#pragma unroll
            for (int t = 0; t < WT; t++)
                dequant_group_to_lds<BITS, XBF, EXACT>(wreg[1 - P][t], j, magic, wnxt + wf[t] * TILE16, lane);
        }
        __syncthreads();
    };
    for (int kt = 0; kt < KT; kt += 2) {
        k_tile(kt, std::integral_constant<int, 0>{});
        if (kt + 1 < KT) k_tile(kt + 1, std::integral_constant<int, 1>{});
    }

    // ---- epilogue
#pragma unroll
    for (int i = 0; i < MF; i++)
#pragma unroll
        for (int f = 0; f < NF; f++) {
            const int n = (nt0 + f) * 16 + row16;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int m = m0 + i * 16 + oct * 4 + r;
                if (m < M && n < w.N) store_out_g(y, ydt, (int64_t)m * w.N + n, acc[i][f][r] * out_scale);
            }
        }
}

template <int BITS, int XBF, int NF, bool EXACT, int MF, int WAVES>
hipError_t launch_m(const WeightView& w, const void* x, int M, void* y, int ydt, float out_scale, hipStream_t st)
{
    constexpr int BM = WAVES * MF * 16;
    const size_t lds = (size_t)2 * NF * (4 * (EXACT ? 2 : 1) * 64) * 16;     // 56 .. 128 KB
    auto kern = gemm_kernel<BITS, XBF, NF, EXACT, MF, WAVES>;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int n_tiles = (w.NT + NF - 1) / NF, m_tiles = (M + BM - 1) / BM;
    const unsigned groups = (unsigned)(((int64_t)n_tiles * m_tiles + 7) / 8 * 8);
    hipLaunchKernelGGL(kern, dim3(groups), dim3(WAVES * 64), lds, st, w, reinterpret_cast<const uint16_t*>(x), M, y, ydt,
                       n_tiles, m_tiles, out_scale);
    return hipGetLastError();
}

// Workgroup shapes.
//   4 waves x 4 row blocks (256 rows): fewest LDS operand reads per MFMA; one wave per SIMD.
//   8 waves x 2 row blocks (256 rows): two waves per SIMD cover each other's stalls, the tile's
//       weights are still loaded and dequantised once; every wave reads all B operands, so
//       LDS reads per MFMA double - fine for FAST (one operand per group), too much for EXACT.
//   4 waves x 2 row blocks (128 rows): twice the tiles, for grids that would leave CUs idle.
template <int BITS, int XBF, int NF, bool EXACT>
hipError_t launch_t(const WeightView& w, const void* x, int M, void* y, int ydt, float out_scale, int num_cus,
                    hipStream_t st)
{
    const int64_t tiles256 = (int64_t)((w.NT + NF - 1) / NF) * ((M + 255) / 256);
    if (tiles256 < num_cus) return launch_m<BITS, XBF, NF, EXACT, 2, 4>(w, x, M, y, ydt, out_scale, st);
    if (!EXACT) return launch_m<BITS, XBF, NF, EXACT, 2, 8>(w, x, M, y, ydt, out_scale, st);
    return launch_m<BITS, XBF, NF, EXACT, 4, 4>(w, x, M, y, ydt, out_scale, st);
}

template <int BITS, int XBF>
hipError_t launch_nf(const WeightView& w, const void* x, int M, void* y, int ydt, bool exact, float out_scale,
                     int num_cus, hipStream_t st)
{
    // 7 column blocks (BN = 112) tile N = 14336 = 128 * 112 exactly: with M = 512
    // that is 256 workgroups, one per CU; 8 column blocks otherwise
    if (w.NT % 7 == 0) {
        if (exact) return launch_t<BITS, XBF, 7, true>(w, x, M, y, ydt, out_scale, num_cus, st);
        return launch_t<BITS, XBF, 7, false>(w, x, M, y, ydt, out_scale, num_cus, st);
    }
    if (exact) return launch_t<BITS, XBF, 8, true>(w, x, M, y, ydt, out_scale, num_cus, st);
    return launch_t<BITS, XBF, 8, false>(w, x, M, y, ydt, out_scale, num_cus, st);
}

// bf16 [n] -> f16 [n] scaled by 2^-4 (exact for 2^-10 <= |x| < 2^20); n % 8 == 0
__global__ void widen_bf16_kernel(const u32x4_t* __restrict__ src, u32x4_t* __restrict__ dst, int64_t n8)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8) return;
    Frag16 a;
    a.u = src[i];
    dst[i] = bf16_to_f16_frag(a).u;
}

}  // namespace

hipError_t launch_gemm(const WeightView& w, const void* x, int xdt, int M, void* y, int ydt,
                       int num_cus, bool exact, void* workspace, size_t workspace_bytes, hipStream_t st)
{
    if (xdt == kF32) return hipErrorNotSupported;   // api.hip walks fp32 prefill through the decode kernel
    float out_scale = 1.0f;
    if (!exact && xdt == kBF16) {
        out_scale = 16.0f;                          // undoes the 2^-4 prescale of the f16 activations
        const size_t need = (size_t)M * w.K * 2;
        if (workspace && need <= workspace_bytes) {
            // Widen X once instead of in every workgroup (each of the N/112 column
            // tiles would redo it): one elementwise pass, then the f16 kernel.
            const int64_t n8 = (int64_t)M * w.K / 8;
            hipLaunchKernelGGL(widen_bf16_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, st,
                               reinterpret_cast<const u32x4_t*>(x), reinterpret_cast<u32x4_t*>(workspace), n8);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return e;
            x = workspace;
            xdt = kF16;
        }
    }
    if (w.bits == 4) {
        if (xdt == kBF16) return launch_nf<4, 1>(w, x, M, y, ydt, exact, out_scale, num_cus, st);
        return launch_nf<4, 0>(w, x, M, y, ydt, exact, out_scale, num_cus, st);
    }
    if (xdt == kBF16) return launch_nf<8, 1>(w, x, M, y, ydt, exact, out_scale, num_cus, st);
    return launch_nf<8, 0>(w, x, M, y, ydt, exact, out_scale, num_cus, st);
}

}  // namespace cybq
