// gemm_rows.hip - prefill kernel for calls whose 64-row x 16/32/64-column pieces fill one round of workgroups
// (17 .. 64 rows on outputs from 1024 columns up - up to 32 they are fp32 rows -, up to 512 rows on narrow ones),
// FAST mode (f16 operands).
//
// With so little work per CU (64 rows x 56 columns at N = 14336) what the tiled kernels of gemm.hip spend
// per K tile - a barrier, every weight operand read from LDS by every multiplying wave - no longer hides
// behind arithmetic: their K loop costs 0.45 - 0.6 us per K tile whatever the tile holds, and narrow outputs
// make them split K over workgroups and add the slabs in a second pass.
//
// Here the waves of a workgroup share nothing until the end.  The workgroup owns MF row blocks of 16
// (blockIdx.y: which) and NF column blocks of 16; wave w takes the K tiles w, w + WAVES, ... and, for those,
// multiplies ALL its rows against ALL its column blocks (MF x NF accumulator blocks per wave).  A weight tile
// is then needed by exactly one wave: global memory -> registers -> dequantised in registers
// (round_f16(scale * q), the operand of FAST mode) -> MFMA B operand, no LDS, no barrier; and every row of X
// enters the CU once (staged operand order, 1 KB per load) and meets all NF column blocks from registers.  One
// wave per SIMD owns the register file (accumulators, a K tile of X and four K tiles of packed weights in
// flight).  At the end the waves' partial sums meet through LDS and are added in wave order (fixed order:
// results are reproducible and a row's bits do not depend on the other rows of the batch).
// Epilogues: residual add, folded RMSNorm / widened rows (a factor per row on the finished sums), SwiGLU (gate and
// up column blocks sit side by side in a workgroup: 4096 -> 28672 at 24 .. 64 rows 27 - 33 us against 47 - 48).
//
// What bounds it is what a CU takes in: all its rows of X (512 KB for 64 rows at K = 4096) plus its column
// blocks' weights, through an L1 that delivers 64 bytes a cycle (a workgroup per CU that does nothing but read
// the same 512 KB with 1-KB wave instructions reaches 21 - 31 TB/s over the chip with four waves, 33 with
// eight; this kernel takes in 156 MB in 16 us).  Hence: the fewest column blocks that still fit one round of
// workgroups, and only as many row blocks as the call has (two or three up to 48 rows: a row block costs
// 1.1 - 1.3 us).  Per call with the staging pass, bf16 rows, against the tiled kernels (up to 64 rows on small
// weights: against two passes of the batched-rows decode kernel):
//   4096 -> 14336 at 33 .. 48 / 64 rows  17.8 / 19.1 us against 21.5 / 22.1   4096 -> 28672   31 - 33 against 38 - 39
//   4096 ->  8192 at 33 / 64 / 128 rows  13.3 / 14.7 / 19.5 against 20.6 / 21.2 / 25.5
//   4096 ->  4096 at 64 / 128 / 256 rows 12.8 / 14.3 / 19.8 against 14.5 / 25.5 / 22.3
//   4096 ->  6144 at 64 / 128 rows       14.3 / 17.6 against 19.3 / 26.8     8192 -> 14336 at 33 .. 64 rows 30 - 32 against 36.5 - 38
//   4096 ->  1024 at 128 / 256 / 512 rows 12.9 / 14.2 / 20.7 against 18.7 / 21.6 / 27.6
//   fp32 rows, 17 .. 32: 4096 -> 14336 15.9 against 21, 4096 -> 4096 10.7 against 18
// The same kernel on v_mfma_f32_32x32x16_f16 (one wave per SIMD issues a 16x16x32 MFMA only every ~27 cycles, a
// 32x32x16 one back to back; both operands load in that shape from the same layouts as four 256-byte runs) measured
// the same to 0.3 us on every shape: the MFMAs are a quarter of a wave's cycles.  Two workgroups of two column
// blocks per CU (two waves per SIMD, twice the rows of X into every CU): 23.9 against 19.6 us.
// Two waves per SIMD (eight waves; wave (k share, half) takes two of the four scale groups of each of its K tiles:
// half the X registers, half of every tile record, nothing loaded or dequantised twice, eight partial sums at the
// end) is slower on every shape: 4096 -> 4096 at 64 rows 14.2 against 13.1 us, 4096 -> 8192 16.9 against 14.9,
// 4096 -> 1024 at 128 rows 13.9 against 12.8 (and it spills with four column blocks).
// Eight column blocks per workgroup on 32x32x16 (64 rows x 128 columns: 65 .. 128 rows on 4096 -> 14336 in one round,
// 0.8 MB into a CU instead of the tiled kernel's 1.15): 31.4 against 27.6 us at 128 rows, 30.3 against 24.5 at 65 -
// one wave's MFMAs, dequantisation and loads then add up instead of overlapping.
// With eight row blocks per wave (65 .. 128 rows in one workgroup, for wide outputs whose 64-row pieces would
// need two rounds) a wave has twice the MFMAs to issue per K tile next to the same dequantisation and the
// kernel is no quicker than the tiled one (X a whole K tile ahead: the operands no longer fit the register
// file next to 128 accumulator registers, 31 against 27 us; X half a K tile ahead: 27.5 against 27.4 at 128
// rows, 25.3 against 24.2 at 65): those calls stay there.
// Reading f16 rows where the caller has them (row-major: sixteen 64-byte runs per operand load instead of one
// KB) to save the restaging launch is slower, not quicker: 4096 -> 14336 at 64 rows 23.7 against 18.3 us with
// the pass, 4096 -> 4096 at 128 rows 21.9 against 15.9.
#include <algorithm>
#include <type_traits>

#include "cybq_device.h"
#include "cybq_internal.h"

namespace cybq {

namespace {

#include "gemm_parts.h"

template <int I, int N, class F>
__device__ __forceinline__ void static_for_r(F&& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for_r<I + 1, N>(f);
    }
}

// group j of a native tile -> the FAST-mode B operand round_f16(scale * q), in registers
template <int BITS>
__device__ __forceinline__ void dequant_group(const WRegs<BITS>& r, int j, uint32_t magic, Frag16& b)
{
    uint32_t bw[4];
    if (BITS == 4) unpack_q4_f16(r.q[0][2 * (j >> 1)], r.q[0][2 * (j >> 1) + 1], j & 1, magic, bw);
    else unpack_q8_f16(r.q[(BITS == 4) ? 0 : (j >> 1)][(j & 1) * 2], r.q[(BITS == 4) ? 0 : (j >> 1)][(j & 1) * 2 + 1], bw);
    const uint32_t sb = (j & 1) ? (r.s[j >> 1] >> 16) : (r.s[j >> 1] & 0xffffu);
    const _Float16 sh = __builtin_bit_cast(_Float16, (uint16_t)sb);
    const half2_t s2 = {sh, sh};
#pragma unroll
    for (int p = 0; p < 4; p++) b.u[p] = as_u32(as_h2(bw[p]) * s2);
}

// MF row blocks of 16 per workgroup (blockIdx.y-th MF * 16 rows of the call), NF column blocks per workgroup, WAVES
// waves that split K, DEPTH K tiles of packed weights and XD K tiles of X in flight per wave.
template <int BITS, int MF, int NF, int WAVES, int DEPTH, int XD>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(WAVES / 4, WAVES / 4))) void gemm_rows_kernel(
    const uint8_t* __restrict__ wbase, const u32x4_t* __restrict__ x, int KT_, int NT_, int x_row_blocks, int M, int N_,
    void* __restrict__ y, int ydt, int K_, Epilogue epi, NormStats ns)
{
    const WeightView w = {wbase, N_, K_, NT_, KT_, BITS};
    constexpr int FR = MF * NF;                        // accumulator blocks per wave
    static_assert(DEPTH % XD == 0 && MF >= 1 && MF <= WAVES, "shape");
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    float4_t* part = reinterpret_cast<float4_t*>(smem);                                    // [WAVES][FR][64]
    float* stg = reinterpret_cast<float*>(smem + (size_t)WAVES * FR * 1024);               // [MF][16 * NF * 16]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nt0 = (int)blockIdx.x * NF;
    const int KT = w.KT, K = w.K, G = K / kGroup;
    const uint32_t magic = q4_magic_vgpr();
    const int T = KT > wv ? (KT - wv + WAVES - 1) / WAVES : 0;        // my K tiles: number t is tile wv + WAVES * t
    // Workgroups that run side by side read the same rows of X: walking K in the same order they would all
    // ask the same L2 channels for the same lines at the same moment, so every column tile starts its walk
    // at another K tile and wraps around (the order depends on the column tile only, not on M).
    const int kt0 = (int)blockIdx.x % KT;
    // (a tile number past my last one is clamped to the last K tile: loaded again, never used)
    auto tile_of = [&](int t) __attribute__((always_inline)) {
        const int kt = min(wv + WAVES * t, KT - 1) + kt0;
        return kt >= KT ? kt - KT : kt;
    };
    // (row blocks and column blocks past the end are clamped to the last real one: computed again, never
    // stored; the offsets are wave-uniform, the lane's part of an address is one register)
    const u32x4_t* xl = x + lane;
    int xrow[MF];
    const int rb0 = (int)blockIdx.y * MF;              // my first row block (blockIdx.y: which MF * 16 rows of the call)
#pragma unroll
    for (int i = 0; i < MF; i++) xrow[i] = __builtin_amdgcn_readfirstlane(min(rb0 + i, x_row_blocks - 1) * G * 64);
    int64_t wtile[NF];
#pragma unroll
    for (int f = 0; f < NF; f++) wtile[f] = (int64_t)min(nt0 + f, w.NT - 1) * w.KT;
    auto load_x = [&](Frag16 (&dst)[MF], int t, int j) __attribute__((always_inline)) {
        const int g = min(tile_of(t) * 4 + j, G - 1);
#pragma unroll
        for (int i = 0; i < MF; i++) dst[i].u = xl[xrow[i] + g * 64];
    };
    auto fetch = [&](WRegs<BITS> (&dst)[NF], int t) __attribute__((always_inline)) {
        const int kt = tile_of(t);
#pragma unroll
        for (int f = 0; f < NF; f++) load_wtile<BITS>(dst[f], w, wtile[f] + kt, lane);
    };

    float4_t acc[MF][NF];
#pragma unroll
    for (int i = 0; i < MF; i++)
#pragma unroll
        for (int f = 0; f < NF; f++) acc[i][f] = (float4_t){0.f, 0.f, 0.f, 0.f};

    WRegs<BITS> wreg[DEPTH][NF];
    Frag16 xa[XD][4][MF];
#pragma unroll
    for (int d = 0; d < DEPTH; d++) fetch(wreg[d], d);
#pragma unroll
    for (int d = 0; d < XD; d++)
#pragma unroll
        for (int j = 0; j < 4; j++) load_x(xa[d][j], d, j);

    // my K tile number t (register sets R = t % DEPTH, R % XD): multiply; its X registers take the rows of tile
    // t + XD group by group as they fall free; its weight registers take tile t + DEPTH
    auto k_tile = [&](int t, auto residue) __attribute__((always_inline)) {
        constexpr int R = decltype(residue)::value;
#pragma unroll
        for (int j = 0; j < 4; j++) {
#pragma unroll
            for (int f = 0; f < NF; f++) {
                Frag16 b;
                dequant_group<BITS>(wreg[R][f], j, magic, b);
#pragma unroll
                for (int i = 0; i < MF; i++) acc[i][f] = mma<0>(xa[R % XD][j][i], b, acc[i][f]);
            }
            load_x(xa[R % XD][j], t + XD, j);
        }
        fetch(wreg[R], t + DEPTH);
    };
    int t = 0;
    for (; t + DEPTH <= T; t += DEPTH)
        static_for_r<0, DEPTH>([&](auto i) __attribute__((always_inline)) { k_tile(t + decltype(i)::value, i); });
    static_for_r<0, DEPTH - 1>([&](auto i) __attribute__((always_inline)) {
        if (t + decltype(i)::value < T) k_tile(t + decltype(i)::value, i);
    });

    // ---- the partial sums meet: every wave leaves all of its blocks, waves 0 .. MF-1 finish a row block each
#pragma unroll
    for (int i = 0; i < MF; i++)
#pragma unroll
        for (int f = 0; f < NF; f++) part[(wv * FR + i * NF + f) * 64 + lane] = acc[i][f];
    __syncthreads();
    if (wv >= MF) return;
    float4_t tot[1][NF];
#pragma unroll
    for (int f = 0; f < NF; f++) {
        const int blk = wv * NF + f;
        float4_t s = part[blk * 64 + lane];
#pragma unroll
        for (int p = 1; p < WAVES; p++) s += part[(p * FR + blk) * 64 + lane];
        tot[0][f] = s;
    }
    const int m0 = (rb0 + wv) * 16;
    if (epi.gamma || ns.unscale) {
#pragma unroll
        for (int r4 = 0; r4 < 4; r4++) {
            const float rs = row_factor(ns, epi.gamma != nullptr, min(m0 + (lane >> 4) * 4 + r4, M - 1), K, epi.eps);
#pragma unroll
            for (int f = 0; f < NF; f++) tot[0][f][r4] *= rs;
        }
    }
    if constexpr (NF >= 2) {
        if (epi.kind == kEpiSwiglu) {      // column blocks 2p / 2p+1 are gate / up of output block (nt0 >> 1) + p
            float4_t act[1][NF / 2];
#pragma unroll
            for (int p = 0; p < NF / 2; p++)
#pragma unroll
                for (int r4 = 0; r4 < 4; r4++) act[0][p][r4] = silu_mul(tot[0][2 * p][r4], tot[0][2 * p + 1][r4]);
            const Epilogue plain = {kEpiNone, nullptr, nullptr, 0, 0.f};
            write_rows<1, NF / 2>(act, stg + wv * (16 * NF * 16), m0, nt0 >> 1, M, w.N >> 1, y, ydt, 1.0f, plain, lane);
            return;
        }
    }
    write_rows<1, NF>(tot, stg + wv * (16 * NF * 16), m0, nt0, M, w.N, y, ydt, 1.0f, epi, lane);
}

template <int BITS, int MF, int NF, int WAVES, int DEPTH, int XD>
hipError_t launch_rows_t(const WeightView& w, const void* x, int M, void* y, int ydt, const Epilogue& epi, const NormStats& ns,
                         hipStream_t st)
{
    constexpr int lds = WAVES * MF * NF * 1024 + MF * 16 * NF * 16 * 4;
    (void)LdsRequest<&gemm_rows_kernel<BITS, MF, NF, WAVES, DEPTH, XD>, lds>::registered;
    const unsigned groups = (unsigned)((w.NT + NF - 1) / NF), row_parts = (unsigned)((M + 16 * MF - 1) / (16 * MF));
    hipLaunchKernelGGL((gemm_rows_kernel<BITS, MF, NF, WAVES, DEPTH, XD>), dim3(groups, row_parts), dim3(WAVES * 64), lds, st, w.base,
                       reinterpret_cast<const u32x4_t*>(x), w.KT, w.NT, (M + 15) / 16, M, w.N, y, ydt, w.K, epi, ns);
    return hipGetLastError();
}

}  // namespace

// Column blocks per workgroup (1, 2 or 4) for a call of M rows, or 0 when the kernel does not take it.
// A call takes about 1.6 us per K tile of a wave whatever the number of workgroups, and less per K tile the fewer
// column blocks a wave carries, so: the fewest column blocks that still fit one round of workgroups
// (4096 -> 4096 at 128 rows: 256 workgroups of two column blocks 14.3 us, 128 of four 17.0; 4096 -> 2048 at 24
// rows: 128 of one 11.6, the tiled kernels 17.5), at least a quarter of a round (4096 -> 1024 at 24 rows, 64
// workgroups: 11.4 against 17.4), K of 16 .. 64 tiles (beyond that the tiled kernels split K over workgroups:
// 14336 -> 4096 33.6 against 43 us here).  More than 64 rows are one workgroup per 64 rows and column group:
// narrow outputs only, where all of them fit one round.
int rows_column_blocks(const WeightView& w, int M, int num_cus, const Epilogue& epi)
{
    if (M <= 16 || M > 512 || w.KT < 16 || w.KT > 64) return 0;
    const int64_t parts = (M + 63) / 64;
    for (int nf : {1, 2, 4}) {
        if (nf == 1 && epi.kind == kEpiSwiglu) continue;        // (a gate block and its up block sit in one workgroup)
        const int64_t groups = (w.NT + nf - 1) / nf * parts;
        if (groups <= num_cus) return groups * 4 >= num_cus ? nf : 0;
    }
    return parts == 1 ? 4 : 0;       // (up to 64 rows a wide output may take more than one round)
}

int gemm_rows_blocks(const WeightView& w, int M, int num_cus, const Epilogue& epi) { return rows_column_blocks(w, M, num_cus, epi); }

bool gemm_rows_serves(const WeightView& w, int M, int num_cus, const Epilogue& epi)
{
    return rows_column_blocks(w, M, num_cus, epi) != 0;
}

hipError_t launch_gemm_rows(const WeightView& w, const void* x_staged, int M, void* y, int ydt, const Epilogue& epi,
                            const float* ssq_part, int ssq_blocks, const float* unscale, int num_cus, hipStream_t st)
{
    const NormStats ns = {ssq_part, ssq_blocks, unscale};
    const int nf = rows_column_blocks(w, M, num_cus, epi);
    // four waves, one per SIMD with the whole register file: four K tiles of packed weights and one K tile of
    // X in flight per wave.  Measured against it on 4096 -> 14336 at 64 bf16 rows (19.1 us per call with the
    // staging pass; the tiled kernel 22.1): eight waves with two / three weight tiles in flight 22.8 / 20.2;
    // X two / four K tiles ahead 21.7 / 20.4; eight weight tiles ahead 23.9; MFMAs and dequantisation
    // interleaved by scheduling hints 21.2; four staging + four multiplying waves sharing K slots through
    // LDS 26.7.
    // Up to 48 rows the workgroup carries two or three row blocks instead of four: the rows of X are most of what
    // a CU takes in, and its L1 delivers 64 bytes a cycle.
    const int mf = M > 48 ? 4 : M > 32 ? 3 : 2;
    auto go = [&](auto bits, auto nfc) {
        constexpr int B = decltype(bits)::value, F = decltype(nfc)::value;
        if (mf == 2) return launch_rows_t<B, 2, F, 4, 4, 1>(w, x_staged, M, y, ydt, epi, ns, st);
        if (mf == 3) return launch_rows_t<B, 3, F, 4, 4, 1>(w, x_staged, M, y, ydt, epi, ns, st);
        return launch_rows_t<B, 4, F, 4, 4, 1>(w, x_staged, M, y, ydt, epi, ns, st);
    };
    auto with_bits = [&](auto nfc) {
        if (w.bits == 8) return go(std::integral_constant<int, 8>{}, nfc);
        return go(std::integral_constant<int, 4>{}, nfc);
    };
    if (nf == 1) return with_bits(std::integral_constant<int, 1>{});
    if (nf == 2) return with_bits(std::integral_constant<int, 2>{});
    return with_bits(std::integral_constant<int, 4>{});
}

}  // namespace cybq
