// gemm.hip - prefill kernel: Y[M,N] = X[M,K] * W^T for M > 16 on MFMA.
//
// Workgroup = 8 or 4 waves, output tile 256 or 128 rows x (16*NF) columns; wave w owns
// two row blocks of 16 against all NF column blocks.
//
//   X  never touches LDS.  An MFMA A operand is 16 rows x 32 k with lane l
//      holding row l%16, k 8*(l/16)..+8.  Read straight from a row-major X that is
//      64 separate 16 B accesses per load (neighbouring lanes are different rows),
//      which saturates the address path long before the matrix cores.  So a small
//      kernel first restages X once per call in operand order - row block, scale
//      group, lane - and the multiply streams it global -> registers with
//      contiguous 1 KB loads, one K tile (four scale groups) ahead of its use.
//      The same pass turns bf16 / fp32 rows into f16 operands for FAST mode.
//   W  is shared by the waves of a workgroup: per K tile (128 k = 4 groups) the NF native
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
//          inside the operator's 1e-3 tolerance); bf16 and fp32 activations become
//          f16 operands in the staging pass behind a power-of-two scale per row that is
//          undone in the epilogue.
//
// Shapes with fewer tiles than CUs split K over workgroups: each split leaves fp32
// partial sums in its own slab of the workspace and a last kernel adds the slabs in a
// fixed order, so results are reproducible (no atomics).
//
// Out-of-range rows / columns / k are clamped to valid addresses inside the hot
// loop (their results are never stored, padded weights are zero); the loop has
// no branches, so the compiler can count outstanding loads exactly.
#include <algorithm>
#include <type_traits>

#include "cybq_device.h"
#include "cybq_internal.h"

namespace cybq {

namespace {

#include "gemm_parts.h"

// gamma[k0 .. k0+8) as fp32 (k0 a multiple of 8, gamma 16-byte aligned)
__device__ __forceinline__ void load_gamma8_g(const void* g, int gdt, int k0, float out[8])
{
    if (gdt == kF32) {
        const float4_t* p = reinterpret_cast<const float4_t*>(reinterpret_cast<const float*>(g) + k0);
        const float4_t a = p[0], b = p[1];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            out[i] = a[i];
            out[4 + i] = b[i];
        }
    } else {
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const uint16_t*>(g) + k0);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if (gdt == kF16) {
                const half2_t h = as_h2(v[i]);
                out[2 * i] = (float)h.x;
                out[2 * i + 1] = (float)h.y;
            } else {
                out[2 * i] = __builtin_bit_cast(float, v[i] << 16);
                out[2 * i + 1] = __builtin_bit_cast(float, v[i] & 0xffff0000u);
            }
        }
    }
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
    if (BITS == 4) unpack_q4_f16(r.q[0][2 * (j >> 1)], r.q[0][2 * (j >> 1) + 1], j & 1, magic, bw);
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

// XBF = 1: X is bf16, 0: X is f16.  EXACT: see the header comment.
// Wave wv of WAVES owns MF row blocks of 16 against all NF column blocks.
template <int BITS, int XBF, int NF, bool EXACT, int MF, int WAVES>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_kernel(const uint8_t* __restrict__ wbase, const u32x4_t* __restrict__ x, int KT_, int NT_, int x_row_blocks, int M,
                                                   int n_tiles, int m_tiles, int splits, int kt_per_split, int groups, int N_,
                                                   void* __restrict__ y, int ydt, int K_, float out_scale,
                                                   float* __restrict__ part, Epilogue epi, NormStats ns)
{
    // (leading scalar arguments in the order of their first use: they arrive in registers at wave start)
    const WeightView w = {wbase, N_, K_, NT_, KT_, BITS};
    // Workgroups are handed to the 8 XCDs round-robin (id % 8) and every XCD has
    // its own L2.  Give each XCD a contiguous run of tiles in row-block-major
    // order, so the workgroups sharing an L2 read the same rows of X and X is
    // fetched into every L2 once instead of once per column tile.
    const int per_xcd = groups >> 3;
    const int item = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
    if (item >= n_tiles * m_tiles * splits) return;
    // split-major: workgroups that run side by side share a K range of X
    const int split = item / (n_tiles * m_tiles);
    const int tile_m = (item - split * (n_tiles * m_tiles)) / n_tiles;
    const int tile_n = item - (split * m_tiles + tile_m) * n_tiles;
    constexpr int BM = WAVES * MF * 16;               // MF = row blocks (of 16) per wave
    constexpr int WT = (NF + WAVES - 1) / WAVES;      // weight tiles a wave stages per K tile
    constexpr int OPS = EXACT ? 2 : 1;                // B operands per scale group
    constexpr int TILE16 = 4 * OPS * 64;              // u32x4 per column block per K tile
    constexpr int BUF16 = NF * TILE16;                // u32x4 per LDS buffer
    constexpr int MMA_BF = EXACT ? XBF : 0;           // FAST always multiplies in f16
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    u32x4_t* ws = reinterpret_cast<u32x4_t*>(smem);   // [2][NF][4][OPS][64]
    const uint32_t magic = q4_magic_vgpr();

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row16 = lane & 15;
    const int oct = lane >> 4;
    const int nt0 = tile_n * NF;
    const int m0 = tile_m * BM + wv * (MF * 16);
    const int K = w.K;
    // this workgroup's K tiles: [kt_lo, kt_lo + KT) of the weight's w.KT (all of them unless K is split)
    const int kt_lo = split * kt_per_split;
    const int KT = min(kt_per_split, w.KT - kt_lo);
    // Workgroups that run side by side share rows of X.  Walking K in the same order
    // they would all ask the same few L2 channels for the same lines at the same
    // moment (a row of X is a multiple of the channel interleave long), so each
    // column tile starts its walk at a different K tile and wraps around.  The
    // order depends on the column tile only: a row of Y does not depend on M.
    const int kt0 = tile_n % KT;
    auto rot = [&](int kt) {
        const int r = min(kt, KT - 1) + kt0;
        return kt_lo + (r >= KT ? r - KT : r);
    };

    // X arrives staged in A-operand order (stage_x_kernel): row block rb, scale group
    // g is one contiguous KB, lane after lane, so a load is one wave-uniform base
    // plus lane * 16 B and adjacent lanes read adjacent memory.  Row blocks past the
    // last are clamped to it (never stored); a scale group past K (padding, zero
    // weights) reads the last real group instead.
    const int G = K / kGroup;
    const u32x4_t* xb[MF];
#pragma unroll
    for (int i = 0; i < MF; i++)
        xb[i] = x + ((int64_t)min(m0 / 16 + i, x_row_blocks - 1) * G) * 64 + lane;
    auto load_x = [&](Frag16 (&dst)[MF], int kt, int j) {
        const int g = min(rot(kt) * 4 + j, G - 1);
#pragma unroll
        for (int i = 0; i < MF; i++) dst[i].u = xb[i][g * 64];
    };

    // The weight tiles this wave stages: column block f = wv + WAVES*t (clamped: a wave
    // past the end stages a neighbour's block again with identical values, no branch).
    int64_t wtile[WT];
    int wdst[WT];
#pragma unroll
    for (int t = 0; t < WT; t++) {
        const int f = min(wv + WAVES * t, NF - 1);
        wdst[t] = f * TILE16;
        wtile[t] = (int64_t)min(nt0 + f, w.NT - 1) * w.KT;
    }
    auto load_units = [&](WRegs<BITS> (&dst)[WT], int kt) {
#pragma unroll
        for (int t = 0; t < WT; t++) load_wtile<BITS>(dst[t], w, wtile[t] + rot(kt), lane);
    };
    auto stage_units = [&](WRegs<BITS> (&src)[WT], int j, u32x4_t* buf) {
#pragma unroll
        for (int t = 0; t < WT; t++) dequant_group_to_lds<BITS, XBF, EXACT>(src[t], j, magic, buf + wdst[t], lane);
    };

    float4_t acc[MF][NF];
#pragma unroll
    for (int i = 0; i < MF; i++)
#pragma unroll
        for (int f = 0; f < NF; f++) acc[i][f] = (float4_t){0.f, 0.f, 0.f, 0.f};

    // ---- prologue: first K tile of X, W tile 0 -> LDS buffer 0, W tiles 1 .. SETS-1 -> registers
    Frag16 xa[4][MF];          // one K tile (four scale groups) of X in flight
#pragma unroll
    for (int j = 0; j < 4; j++) load_x(xa[j], 0, j);
    // Packed weights wait in registers: K tile t sits in wreg[t % SETS], requested SETS - 1
    // iterations before it is dequantised.  Loads retire in order and every iteration
    // also requests X, so two sets leave a weight tile one iteration (about 2 us) to
    // arrive - enough from cache, short for a first touch in HBM; Q4 FAST has the
    // registers for four.
    constexpr int SETS = (BITS == 4 && !EXACT) ? 4 : 2;
    WRegs<BITS> wreg[SETS][WT];
    {
        WRegs<BITS> w0[WT];
        load_units(w0, 0);
#pragma unroll
        for (int t = 1; t < SETS; t++) load_units(wreg[t], t);
#pragma unroll
        for (int j = 0; j < 4; j++) stage_units(w0, j, ws);
    }
    __syncthreads();

    // One K tile.  R = kt % SETS is a compile-time constant (the loop below is unrolled
    // SETS times), so LDS buffers (R & 1) and register sets alternate without copies
    // or selects:  multiply from LDS buffer R & 1;  dequantise tile kt+1 from its
    // register set into the other buffer;  request tile kt+SETS into the set tile kt
    // left free.  Past the end indices are clamped: a tile is staged again but never read.
    auto k_tile = [&](int kt, auto residue) {
        constexpr int R = decltype(residue)::value;
        constexpr int P = R & 1;
        const u32x4_t* wcur = ws + P * BUF16;
        u32x4_t* wnxt = ws + (1 - P) * BUF16;
        load_units(wreg[R], kt + SETS);

#pragma unroll
        for (int j = 0; j < 4; j++) {
            const Frag16 (&a)[MF] = xa[j];
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
            // the same groups of the next K tile.
            if (j & 1) {
                load_x(xa[j - 1], kt + 1, j - 1);
                load_x(xa[j], kt + 1, j);
            }
            // a quarter of the next tile's dequantisation rides along with every group
            stage_units(wreg[(R + 1) % SETS], j, wnxt);
        }
        // Order inside the K tile (two waves per SIMD): the dequantisation of the next tile is
        // spread between the MFMAs.  A wave issues in order: arithmetic queued behind a run of
        // MFMAs waits for all of them and the matrix pipe idles while it runs afterwards; and the
        // barrier keeps the two waves of a SIMD in the same phase, so they do not cover for each
        // other.  (With one wave per SIMD, the 128-row shape, the same order measured slower.)
        if constexpr (WAVES == 8 && !EXACT) {
            constexpr int READS = 4 * NF * OPS;
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);          // LDS reads run two ahead of their MFMAs
#pragma unroll
            for (int i = 0; i < READS; i++) {
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);      // one LDS read
                __builtin_amdgcn_sched_group_barrier(0x008, MF, 0);     // its MFMAs, one per row block
                __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);      // two vector ALU instructions
            }
        }
        __syncthreads();
    };
    for (int kt = 0; kt < KT; kt += SETS) {
        k_tile(kt, std::integral_constant<int, 0>{});
        if (kt + 1 < KT) k_tile(kt + 1, std::integral_constant<int, 1>{});
        if constexpr (SETS == 4) {
            if (kt + 2 < KT) k_tile(kt + 2, std::integral_constant<int, 2>{});
            if (kt + 3 < KT) k_tile(kt + 3, std::integral_constant<int, 3>{});
        }
    }

    // ---- epilogue: a K split leaves its partial sums in fp32 for splitk_reduce_kernel (whole runs of a row
    // through LDS, like the final sums)
    if (splits > 1) {
        const Epilogue plain = {kEpiNone, nullptr, nullptr, 0, 0.f};
        write_rows<MF, NF>(acc, reinterpret_cast<float*>(smem) + wv * (16 * NF * 16), m0, nt0, M, w.N, part + (int64_t)split * M * w.N, kF32,
                           1.0f, plain, lane);
        return;
    }
    if (epi.gamma || ns.unscale) {     // folded RMSNorm: rstd of the row; widened activations: the row's power of two
#pragma unroll
        for (int i = 0; i < MF; i++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float rs = row_factor(ns, epi.gamma != nullptr, min(m0 + i * 16 + oct * 4 + r, M - 1), K, epi.eps);
#pragma unroll
                for (int f = 0; f < NF; f++) acc[i][f][r] *= rs;
            }
    }
    if (epi.kind == kEpiSwiglu) {      // column blocks 2p / 2p+1 are gate / up of output block (nt0 >> 1) + p
        const int n_out = w.N >> 1;
#pragma unroll
        for (int i = 0; i < MF; i++)
#pragma unroll
            for (int p = 0; p < NF / 2; p++) {
                const int n = ((nt0 >> 1) + p) * 16 + row16;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int m = m0 + i * 16 + oct * 4 + r;
                    if (m < M && n < n_out)
                        store_out_g(y, ydt, (int64_t)m * n_out + n,
                                    silu_mul(acc[i][2 * p][r] * out_scale, acc[i][2 * p + 1][r] * out_scale));
                }
            }
        return;
    }
    write_rows<MF, NF>(acc, reinterpret_cast<float*>(smem) + wv * (16 * NF * 16), m0, nt0, M, w.N, y, ydt, out_scale, epi, lane);
}

// The same multiply (FAST mode, f16 operands) with the work of a workgroup split by role:
// MW waves only multiply - each owns MF row blocks against all NF column blocks, streams its X
// from global memory XD K tiles ahead and reads the weight operands from LDS - and four waves
// only fetch packed weight tiles and dequantise them into LDS, several K tiles ahead.  Loads
// retire in order within a wave: in gemm_kernel the wait for the next rows of X is also a wait
// for every weight tile requested before them, and a first touch in HBM holds the matrix pipe
// up; here the multiplying waves never wait for HBM.  Waves are dealt to the four SIMDs in turn,
// so every SIMD carries one staging wave: the dequantisation runs in the issue slots the MFMAs
// leave free.  MW*MF*16 x NF*16 outputs per workgroup, one barrier per K tile, no K split.
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

template <int BITS, int NF, int MF, int MW, int XD>
__global__ __launch_bounds__((MW + 4) * 64) __attribute__((amdgpu_waves_per_eu((MW + 7) / 4, (MW + 7) / 4))) void gemm_roles_kernel(
    const uint8_t* __restrict__ wbase, const u32x4_t* __restrict__ x, int KT_, int NT_, int x_row_blocks, int M, int n_tiles,
    int m_tiles, int groups, int N_, void* __restrict__ y, int ydt, int K_, float out_scale, Epilogue epi, NormStats ns)
{
    const WeightView w = {wbase, N_, K_, NT_, KT_, BITS};
    constexpr int SW = 4;                             // staging waves
    constexpr int WT = (NF + SW - 1) / SW;            // weight tiles a staging wave handles per K tile
    constexpr int TILE16 = 4 * 64;                    // u32x4 per column block per K tile
    constexpr int BUF16 = NF * TILE16;
    // K tiles of packed weights in flight per staging wave (8 measured the same at 64 and 128 rows, 16
    // slower: 23 -> 30 us at 64 rows)
    constexpr int DEPTH = 4;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    u32x4_t* ws = reinterpret_cast<u32x4_t*>(smem);   // [2][NF][4][64]

    const int per_xcd = groups >> 3;                  // (same tile order as gemm_kernel)
    const int item = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
    if (item >= n_tiles * m_tiles) return;
    const int tile_m = item / n_tiles, tile_n = item - tile_m * n_tiles;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nt0 = tile_n * NF;
    const int KT = w.KT, K = w.K;
    const int kt0 = tile_n % KT;
    auto rot = [&](int kt) {
        const int r = min(kt, KT - 1) + kt0;
        return r >= KT ? r - KT : r;
    };

    if (wave >= MW) {
        // ---- staging waves ----------------------------------------------------------------
        const int pw = wave - MW;
        const uint32_t magic = q4_magic_vgpr();
        int64_t wtile[WT];
        int wdst[WT];
#pragma unroll
        for (int t = 0; t < WT; t++) {
            const int f = min(pw + SW * t, NF - 1);     // (past the end: a neighbour's block again, same values)
            wdst[t] = f * TILE16;
            wtile[t] = (int64_t)min(nt0 + f, w.NT - 1) * w.KT;
        }
        WRegs<BITS> wreg[DEPTH][WT];
        auto fetch = [&](WRegs<BITS> (&dst)[WT], int kt) {
#pragma unroll
            for (int t = 0; t < WT; t++) load_wtile<BITS>(dst[t], w, wtile[t] + rot(kt), lane);
        };
        auto stage = [&](WRegs<BITS> (&src)[WT], u32x4_t* buf) {
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int t = 0; t < WT; t++) dequant_group_to_lds<BITS, 0, false>(src[t], j, magic, buf + wdst[t], lane);
        };
#pragma unroll
        for (int d = 0; d < DEPTH; d++) fetch(wreg[d], d);
        stage(wreg[0], ws);
        fetch(wreg[0], DEPTH);
        __syncthreads();
        // during K tile kt: tile kt + 1 (register set (kt + 1) % DEPTH) -> the other LDS buffer, then that
        // set is refilled with tile kt + 1 + DEPTH
        auto k_tile = [&](int kt, auto residue) {
            constexpr int R = decltype(residue)::value;            // = (kt + 1) % DEPTH
            stage(wreg[R], ws + ((R & 1) ? BUF16 : 0));
            fetch(wreg[R], kt + 1 + DEPTH);
            __syncthreads();
        };
        // Whole rounds in the loop, the remainder behind it: a tile skipped inside the loop is a path
        // into the loop head with fewer loads outstanding, the one wait count an instruction carries has
        // to be safe for that path, and the first use of a tile then also waits for the newest request.
        // With few rows there is little arithmetic per K tile to hide that behind (4096 -> 14336 at 64
        // rows 26.1 -> 22.8 us); the 256-row kernel measured better with the tighter counts (60.5 against
        // 63 us at 512 rows).
        int kt = 0;
        if constexpr (MW <= 4) {
            for (; kt + DEPTH <= KT; kt += DEPTH)
                static_for<0, DEPTH>([&](auto i) { k_tile(kt + decltype(i)::value, std::integral_constant<int, (decltype(i)::value + 1) % DEPTH>{}); });
            static_for<0, DEPTH - 1>([&](auto i) {
                if (kt + decltype(i)::value < KT) k_tile(kt + decltype(i)::value, std::integral_constant<int, (decltype(i)::value + 1) % DEPTH>{});
            });
            return;
        } else {
            for (; kt < KT; kt += DEPTH) {
                k_tile(kt, std::integral_constant<int, 1>{});
                if (kt + 1 < KT) k_tile(kt + 1, std::integral_constant<int, 2>{});
                if (kt + 2 < KT) k_tile(kt + 2, std::integral_constant<int, 3>{});
                if (kt + 3 < KT) k_tile(kt + 3, std::integral_constant<int, 0>{});
            }
            return;
        }
    }

    // ---- multiplying waves --------------------------------------------------------------------
    const int m0 = tile_m * (MW * MF * 16) + wave * (MF * 16);
    const int G = K / kGroup;
    const u32x4_t* xb[MF];
#pragma unroll
    for (int i = 0; i < MF; i++) xb[i] = x + ((int64_t)min(m0 / 16 + i, x_row_blocks - 1) * G) * 64 + lane;
    auto load_x = [&](Frag16 (&dst)[MF], int kt, int j) {
        const int g = min(rot(kt) * 4 + j, G - 1);
#pragma unroll
        for (int i = 0; i < MF; i++) dst[i].u = xb[i][g * 64];
    };
    float4_t acc[MF][NF];
#pragma unroll
    for (int i = 0; i < MF; i++)
#pragma unroll
        for (int f = 0; f < NF; f++) acc[i][f] = (float4_t){0.f, 0.f, 0.f, 0.f};
    Frag16 xa[XD][4][MF];          // XD K tiles of X in flight
#pragma unroll
    for (int d = 0; d < XD; d++)
#pragma unroll
        for (int j = 0; j < 4; j++) load_x(xa[d][j], d, j);
    __syncthreads();
    auto k_tile = [&](int kt, auto residue) {
        constexpr int D = decltype(residue)::value;                 // = kt % XD
        const u32x4_t* wcur = ws + ((kt & 1) ? BUF16 : 0);
#pragma unroll
        for (int j = 0; j < 4; j++) {
#pragma unroll
            for (int f = 0; f < NF; f++) {
                Frag16 b;
                b.u = wcur[f * TILE16 + j * 64 + lane];
#pragma unroll
                for (int i = 0; i < MF; i++) acc[i][f] = mma<0>(xa[D][j][i], b, acc[i][f]);
            }
            load_x(xa[D][j], kt + XD, j);      // this group's operands are free: those of K tile kt + XD take their place
        }
        constexpr int READS = 4 * NF;
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);          // LDS reads run two ahead of their MFMAs
#pragma unroll
        for (int i = 0; i < READS; i++) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, MF, 0);
            // (a group's X operands are requested again as soon as its last MFMA is out: left to itself
            // the scheduler moves all of a tile's requests to its end, one K tile less of lead)
            if (i % NF == NF - 1) __builtin_amdgcn_sched_group_barrier(0x020, MF, 0);
        }
        __syncthreads();
    };
    int kt = 0;
    if constexpr (MW <= 4) {                       // (whole rounds in the loop: see the staging waves)
        for (; kt + XD <= KT; kt += XD) {
            k_tile(kt, std::integral_constant<int, 0>{});
            if constexpr (XD > 1) k_tile(kt + 1, std::integral_constant<int, 1>{});
            if constexpr (XD > 2) k_tile(kt + 2, std::integral_constant<int, 2>{});
            if constexpr (XD > 3) k_tile(kt + 3, std::integral_constant<int, 3>{});
        }
    }
    for (; kt < KT; kt += XD) {
        k_tile(kt, std::integral_constant<int, 0>{});
        if constexpr (XD > 1) {
            if (kt + 1 < KT) k_tile(kt + 1, std::integral_constant<int, 1>{});
        }
        if constexpr (XD > 2) {
            if (kt + 2 < KT) k_tile(kt + 2, std::integral_constant<int, 2>{});
        }
        if constexpr (XD > 3) {
            if (kt + 3 < KT) k_tile(kt + 3, std::integral_constant<int, 3>{});
        }
    }
    if (epi.gamma || ns.unscale) {
#pragma unroll
        for (int i = 0; i < MF; i++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float rs = row_factor(ns, epi.gamma != nullptr, min(m0 + i * 16 + (lane >> 4) * 4 + r, M - 1), K, epi.eps);
#pragma unroll
                for (int f = 0; f < NF; f++) acc[i][f][r] *= rs;
            }
    }
    write_rows<MF, NF>(acc, reinterpret_cast<float*>(smem) + wave * (16 * NF * 16), m0, nt0, M, w.N, y, ydt, out_scale, epi, lane);
}

template <int BITS, int NF, int MF, int MW, int XD>
hipError_t launch_roles(const WeightView& w, const void* x, int M, void* y, int ydt, float out_scale, const Epilogue& epi,
                        const NormStats& ns, hipStream_t st)
{
    constexpr int lds = 2 * NF * (4 * 64) * 16;
    constexpr int BM = MW * MF * 16;
    (void)LdsRequest<&gemm_roles_kernel<BITS, NF, MF, MW, XD>, lds>::registered;
    const int n_tiles = (w.NT + NF - 1) / NF, m_tiles = (M + BM - 1) / BM;
    const unsigned groups = (unsigned)(((int64_t)n_tiles * m_tiles + 7) / 8 * 8);
    hipLaunchKernelGGL((gemm_roles_kernel<BITS, NF, MF, MW, XD>), dim3(groups), dim3((MW + 4) * 64), lds, st, w.base,
                       reinterpret_cast<const u32x4_t*>(x), w.KT, w.NT, (M + 15) / 16, M, n_tiles, m_tiles, (int)groups, w.N, y, ydt, w.K,
                       out_scale, epi, ns);
    return hipGetLastError();
}

// y = epilogue(out_scale * (part[0] + part[1] + ... + part[splits-1])), slabs added in that order.
// One thread per output element; N = columns of a slab (for SwiGLU y has N / 2).
__global__ void splitk_reduce_kernel(const float* __restrict__ part, int splits, int M, int N, void* __restrict__ y, int ydt,
                                     float out_scale, Epilogue epi, NormStats ns, int K)
{
    const int64_t slab = (int64_t)M * N;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (epi.kind == kEpiSwiglu) {
        const int n_out = N >> 1;
        if (i >= (int64_t)M * n_out) return;
        const int m = (int)(i / n_out), n = (int)(i - (int64_t)m * n_out);
        const int64_t ig = (int64_t)m * N + (n >> 4) * 32 + (n & 15);
        float g = part[ig], u = part[ig + 16];
        for (int s = 1; s < splits; s++) {
            g += part[s * slab + ig];
            u += part[s * slab + ig + 16];
        }
        const float sc = out_scale * row_factor(ns, epi.gamma != nullptr, m, K, epi.eps);
        store_out_g(y, ydt, i, silu_mul(g * sc, u * sc));
        return;
    }
    if (i >= slab) return;
    float v = part[i];
    for (int s = 1; s < splits; s++) v += part[s * slab + i];
    v *= out_scale;
    if (epi.gamma || ns.unscale) v *= row_factor(ns, epi.gamma != nullptr, (int)(i / N), K, epi.eps);
    if (epi.kind == kEpiAdd) v += load_out_g(epi.residual, ydt, i);
    store_out_g(y, ydt, i, v);
}

// The same sum, four neighbouring elements per thread with 128-bit slab reads (slab a multiple of
// four elements, no SwiGLU): the pass is pure memory traffic, splits + 1 times the output.
__global__ void splitk_reduce4_kernel(const float* __restrict__ part, int splits, int M, int N, void* __restrict__ y, int ydt,
                                      float out_scale, Epilogue epi, NormStats ns, int K)
{
    const int64_t slab = (int64_t)M * N;
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= slab) return;
    float4_t v = *reinterpret_cast<const float4_t*>(part + i);
    for (int s = 1; s < splits; s++) v += *reinterpret_cast<const float4_t*>(part + s * slab + i);
#pragma unroll
    for (int e = 0; e < 4; e++) {
        float t = v[e] * out_scale;
        if (epi.gamma || ns.unscale) t *= row_factor(ns, epi.gamma != nullptr, (int)((i + e) / N), K, epi.eps);
        if (epi.kind == kEpiAdd) t += load_out_g(epi.residual, ydt, i + e);
        v[e] = t;
    }
    if (ydt == kF32) {
        *reinterpret_cast<float4_t*>(reinterpret_cast<float*>(y) + i) = v;
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) store_out_g(y, ydt, i + e, v[e]);
    }
}

template <int BITS, int XBF, int NF, bool EXACT, int MF, int WAVES>
hipError_t launch_m(const WeightView& w, const void* x, int M, void* y, int ydt, float out_scale, float* part,
                    size_t part_bytes, int num_cus, const Epilogue& epi, const NormStats& ns, hipStream_t st)
{
    constexpr int BM = WAVES * MF * 16;
    constexpr int lds = 2 * NF * (4 * (EXACT ? 2 : 1) * 64) * 16;     // operand buffers, 56 .. 128 KB
    auto kern = gemm_kernel<BITS, XBF, NF, EXACT, MF, WAVES>;
    (void)LdsRequest<&gemm_kernel<BITS, XBF, NF, EXACT, MF, WAVES>, lds>::registered;
    const int n_tiles = (w.NT + NF - 1) / NF, m_tiles = (M + BM - 1) / BM;
    // Too few tiles to fill the chip: split K over workgroups.  Every split adds its
    // K range in fp32 into its own slab of `part`; a second kernel adds the slabs in
    // a fixed order (no atomics: results are reproducible).
    const int64_t tiles = (int64_t)n_tiles * m_tiles;
    int splits = (int)std::min<int64_t>(8, num_cus / tiles);
    splits = std::min(splits, w.KT / 4);                         // at least 4 K tiles per split
    while (splits > 1 && (size_t)splits * M * w.N * 4 > part_bytes) splits--;
    if (splits < 1) splits = 1;
    const int kt_per_split = (w.KT + splits - 1) / splits;
    splits = (w.KT + kt_per_split - 1) / kt_per_split;          // no empty split
    const unsigned groups = (unsigned)((tiles * splits + 7) / 8 * 8);
    hipLaunchKernelGGL(kern, dim3(groups), dim3(WAVES * 64), lds, st, w.base, reinterpret_cast<const u32x4_t*>(x), w.KT, w.NT,
                       (M + 15) / 16, M, n_tiles, m_tiles, splits, kt_per_split, (int)groups, w.N, y, ydt, w.K, out_scale, part, epi, ns);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || splits == 1) return e;
    const int64_t total = (int64_t)M * w.N;
    if (total % 4 == 0 && epi.kind != kEpiSwiglu && (ydt != kF32 || (reinterpret_cast<uintptr_t>(y) & 15u) == 0))
        hipLaunchKernelGGL(splitk_reduce4_kernel, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, st, part, splits, M, w.N, y,
                           ydt, out_scale, epi, ns, w.K);
    else
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, part, splits, M, w.N, y, ydt,
                           out_scale, epi, ns, w.K);
    return hipGetLastError();
}

// Workgroup shapes: every wave owns 2 row blocks.
//   8 waves (256 rows): two waves per SIMD cover each other's waits and the tile's
//       weights are dequantised once for all eight.
//   4 waves (128 rows): twice the tiles, for few rows on grids that would leave CUs idle.
//       From 256 rows up (a long K) or beyond, the 8-wave shape with a deeper K split is the
//       quicker way to fill the chip (14336 -> 4096 at M = 512: 86.7 -> 74.6 us).
template <int BITS, int XBF, int NF, bool EXACT>
hipError_t launch_t(const WeightView& w, const void* x, int M, void* y, int ydt, float out_scale, float* part,
                    size_t part_bytes, int num_cus, const Epilogue& epi, const NormStats& ns, hipStream_t st)
{
    const int64_t tiles256 = (int64_t)((w.NT + NF - 1) / NF) * ((M + 255) / 256);
    const bool few_rows = M < 256 || (M == 256 && w.KT < 64);
    // 512-row workgroups (four row blocks per wave: half the LDS operand reads per MFMA) once they
    // fill the chip by themselves
    if constexpr (!EXACT && NF == 7) {           // (eight column blocks x four row blocks spill)
        const int64_t tiles512 = (int64_t)((w.NT + NF - 1) / NF) * ((M + 511) / 512);
        const int rem = M % 512;                       // (a last tile at most half full: 256-row tiles waste less)
        if (tiles512 >= num_cus && (rem == 0 || rem > 256))
            return launch_m<BITS, XBF, NF, EXACT, 4, 8>(w, x, M, y, ydt, out_scale, part, part_bytes, num_cus, epi, ns, st);
    }
    // enough 256-row tiles to fill the chip without a K split: the role-split kernel (the SwiGLU
    // epilogue is not among what it writes)
    if constexpr (!EXACT) {
        if (tiles256 >= num_cus && epi.kind != kEpiSwiglu) return launch_roles<BITS, NF, 2, 8, 2>(w, x, M, y, ydt, out_scale, epi, ns, st);
    }
    if (tiles256 < num_cus && few_rows) return launch_m<BITS, XBF, NF, EXACT, 2, 4>(w, x, M, y, ydt, out_scale, part, part_bytes, num_cus, epi, ns, st);
    return launch_m<BITS, XBF, NF, EXACT, 2, 8>(w, x, M, y, ydt, out_scale, part, part_bytes, num_cus, epi, ns, st);
}

template <int BITS, int XBF>
hipError_t launch_nf(const WeightView& w, const void* x, int M, void* y, int ydt, bool exact, float out_scale,
                     float* part, size_t part_bytes, int num_cus, const Epilogue& epi, const NormStats& ns, hipStream_t st)
{
    // 7 column blocks (BN = 112) tile N = 14336 = 128 * 112 exactly: with M = 512
    // that is 256 workgroups, one per CU; 8 column blocks otherwise
    const bool nf7 = w.NT % 7 == 0 && epi.kind != kEpiSwiglu;      // gate / up pairs need an even number of column blocks
    if (exact) {
        if (nf7) return launch_t<BITS, XBF, 7, true>(w, x, M, y, ydt, out_scale, part, part_bytes, num_cus, epi, ns, st);
        return launch_t<BITS, XBF, 8, true>(w, x, M, y, ydt, out_scale, part, part_bytes, num_cus, epi, ns, st);
    }
    if constexpr (XBF == 0) {       // FAST multiplies in f16: bf16 activations were widened by the staging pass
        // up to 128 rows on a wide output: 128 x 64 tiles fill most of the chip without a K split and
        // its second pass over the partial sums
        if (M <= 128 && epi.kind != kEpiSwiglu) {
            const int64_t tiles64 = (w.NT + 3) / 4;                  // 64-column tiles
            if (tiles64 * 2 >= 3 * num_cus) {        // more than one round of them: the plain kernel (48 against 58 us at N = 28672),
                // up to 64 rows the role-split one with its smaller workgroups (41.5 -> 39.5 us)
                if (M <= 64) return launch_roles<BITS, 4, 2, 2, 2>(w, x, M, y, ydt, out_scale, epi, ns, st);
                return launch_m<BITS, 0, 4, false, 2, 4>(w, x, M, y, ydt, out_scale, part, part_bytes, num_cus, epi, ns, st);
            }
            if (tiles64 * 4 >= 3 * num_cus || (tiles64 * 2 >= num_cus && w.KT <= 48)) {      // (half a round still beats a K split on a short K)        // one round: the role-split kernel (30 against 34.5 us at N = 14336)
                // (every workgroup streams all the rows of X from the L2, and that stream is what these
                // calls wait for: two multiplying waves = 64 rows when that covers the batch)
                if (M <= 64) return launch_roles<BITS, 4, 2, 2, 2>(w, x, M, y, ydt, out_scale, epi, ns, st);
                return launch_roles<BITS, 4, 2, 4, 2>(w, x, M, y, ydt, out_scale, epi, ns, st);
            }
        }
        // A narrow output with a short K (the attention projections at a prefill chunk): 256 x 112 tiles
        // would leave most CUs idle and get a K split with its second pass over the partial sums.
        // One round of 128-row tiles of the role-split kernel, as wide as still gives every CU a tile,
        // does without (X then crosses from the L2 once per column tile: K stays short for this).
        if (epi.kind != kEpiSwiglu && w.KT <= 48 && M > 128) {
            const int64_t tiles256 = (int64_t)((w.NT + 6) / 7) * ((M + 255) / 256);
            if (tiles256 < num_cus) {
                // (128-row tiles first, 64-row ones for batches they cannot spread over the chip; the
                // width that fills most of one round, at least three quarters of it)
                int best_nf = 0, best_mw = 0;
                int64_t best_groups = 0;
                for (int mw : {4, 2})
                    for (int nf : {8, 6, 4}) {
                        const int64_t g = (int64_t)((M + mw * 32 - 1) / (mw * 32)) * ((w.NT + nf - 1) / nf);
                        if (g <= num_cus && g * 4 >= 3 * num_cus && (best_mw == 0 || (mw == best_mw && g > best_groups))) {
                            best_nf = nf;
                            best_mw = mw;
                            best_groups = g;
                        }
                    }
                if (best_mw == 4) {
                    if (best_nf == 8) return launch_roles<BITS, 8, 2, 4, 2>(w, x, M, y, ydt, out_scale, epi, ns, st);
                    if (best_nf == 6) return launch_roles<BITS, 6, 2, 4, 2>(w, x, M, y, ydt, out_scale, epi, ns, st);
                    return launch_roles<BITS, 4, 2, 4, 2>(w, x, M, y, ydt, out_scale, epi, ns, st);
                }
                if (best_mw == 2) {
                    if (best_nf == 8) return launch_roles<BITS, 8, 2, 2, 2>(w, x, M, y, ydt, out_scale, epi, ns, st);
                    if (best_nf == 6) return launch_roles<BITS, 6, 2, 2, 2>(w, x, M, y, ydt, out_scale, epi, ns, st);
                    return launch_roles<BITS, 4, 2, 2, 2>(w, x, M, y, ydt, out_scale, epi, ns, st);
                }
            }
        }
        if (nf7) return launch_t<BITS, 0, 7, false>(w, x, M, y, ydt, out_scale, part, part_bytes, num_cus, epi, ns, st);
        return launch_t<BITS, 0, 8, false>(w, x, M, y, ydt, out_scale, part, part_bytes, num_cus, epi, ns, st);
    }
    return hipErrorInvalidValue;
}

// The multiply that follows a staging launch starts on weights that come from HBM for the first time (2.4 of the
// 14.5 us of a 64-row call on 4096 -> 14336 pass before its K loops start).  Extra workgroups of the staging launch,
// which leaves most of the chip idle, ask for the first K tiles of every column group ahead of it - one dword per
// 128-byte line, nothing kept: workgroup number b here asks for what workgroup b of the multiply reads first (the
// hardware deals workgroups to the eight XCDs in turn, so with first_group a multiple of eight the lines land in
// that workgroup's L2; anywhere else they land in the memory-side cache).
struct Touch {
    const uint8_t* base;          // the weight tensor (first_group past the grid: nothing to do)
    int first_group, NT, KT, NF, tile_bytes, ahead;
    int per_xcd, tiles;           // the tiled kernels' order: workgroup b works on column tile (b % 8) * per_xcd + b / 8 of `tiles` (0: on b)
};

__device__ __forceinline__ void touch_weights(const Touch& tc, int b, int tid, int nthreads)
{
    const int lines = (tc.tile_bytes + 127) >> 7;
    if (tc.per_xcd) {
        b = (b & 7) * tc.per_xcd + (b >> 3);
        if (b >= tc.tiles) return;
    }
    const int kt0 = b % tc.KT;                     // (the multiply's workgroups start their K walk there)
    uint32_t acc = 0;
    for (int idx = tid; idx < tc.NF * tc.ahead * lines; idx += nthreads) {
        const int line = idx % lines, ft = idx / lines, t = ft % tc.ahead, f = ft / tc.ahead;
        const int nt = min(b * tc.NF + f, tc.NT - 1);
        int kt = kt0 + t;
        if (kt >= tc.KT) kt -= tc.KT;
        acc ^= *reinterpret_cast<const uint32_t*>(tc.base + ((int64_t)nt * tc.KT + kt) * tc.tile_bytes + min(line * 128, tc.tile_bytes - 4));
    }
    asm volatile("" ::"v"(acc));                   // (the loads have to be issued and waited for; nothing is stored)
}

// X [M, K] row major (16-bit elements, used as they are) -> A-operand order: for row block rb
// (16 rows, zero padded) and scale group g, 64 x 16 B where slot (oct, r) = oct*16 + r holds row
// 16*rb + r, k = 32*g + 8*oct .. +8.  A workgroup moves one row block x 16 groups through LDS:
// waves read 1 KB runs of a row and write whole 1 KB units.
constexpr int kStageGroups = 16;                       // scale groups per workgroup
constexpr int kStagePitch = kStageGroups * 4 + 1;      // 16 B slots per LDS row (odd: no bank conflicts)

// NORM: RMSNorm folded in.  x * gamma is formed in fp32 and rounded once to the operand type (XBF:
// bf16, else f16); the squares of the unscaled row are summed per (row, workgroup) in a fixed
// butterfly order into ssq_part[row * gridDim.y + blockIdx.y].
template <bool XBF, bool NORM>
__global__ __launch_bounds__(256) void stage_x_kernel(const u32x4_t* __restrict__ src, u32x4_t* __restrict__ dst, int M, int K8,
                                                      Epilogue epi, float* __restrict__ ssq_part)
{
    __shared__ u32x4_t tile[16 * kStagePitch];
    const int rb = blockIdx.x;
    const int c0 = blockIdx.y * (kStageGroups * 4);     // first 16 B chunk of the row handled here
    const int t = threadIdx.x;
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int r = it * 4 + (t >> 6), c = c0 + (t & 63);
        const int row = rb * 16 + r;
        Frag16 a;
        a.u = (u32x4_t){0u, 0u, 0u, 0u};
        if (row < M && c < K8) a.u = src[(int64_t)row * K8 + c];
        if (NORM) {
            float sq = 0.f;
            if (c < K8) {
                float g[8];
                load_gamma8_g(epi.gamma, epi.gamma_dt, c * 8, g);
#pragma unroll
                for (int p = 0; p < 4; p++) {
                    float v0, v1;
                    if (XBF) {
                        v0 = __builtin_bit_cast(float, a.u[p] << 16);
                        v1 = __builtin_bit_cast(float, a.u[p] & 0xffff0000u);
                    } else {
                        const half2_t h = as_h2(a.u[p]);
                        v0 = (float)h.x;
                        v1 = (float)h.y;
                    }
                    sq = fmaf(v1, v1, fmaf(v0, v0, sq));
                    v0 *= g[2 * p];
                    v1 *= g[2 * p + 1];
                    if (XBF) {
                        a.u[p] = pack_bf16x2(v0, v1);
                    } else {
                        const half2_t h = {(_Float16)v0, (_Float16)v1};
                        a.u[p] = as_u32(h);
                    }
                }
            }
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) sq += __shfl_xor(sq, off, 64);
            if ((t & 63) == 0) ssq_part[(int64_t)row * gridDim.y + blockIdx.y] = sq;      // (rows past M: zeros, never read)
        }
        tile[r * kStagePitch + (t & 63)] = a.u;
    }
    __syncthreads();
    const int G = K8 >> 2;
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int gl = it * 4 + (t >> 6), slot = t & 63;        // group within the workgroup, (oct, r)
        const int g = blockIdx.y * kStageGroups + gl;
        if (g < G) dst[((int64_t)rb * G + g) * 64 + slot] = tile[(slot & 15) * kStagePitch + gl * 4 + (slot >> 4)];
    }
}

// The same restaging for FAST mode when the activations are not f16 (bf16 or fp32 in, f16 operands
// out), with a power-of-two scale PER ROW: a workgroup owns four rows.  First a row is read for the
// largest magnitude (of x, or of x * gamma with a folded norm, whose sum of squares is also taken),
// which picks the power of two s that brings it just under 2^14 and leaves 1 / s in `unscale` for
// the multiply's epilogue; then the four rows go through LDS in pieces of 512 k, every value
// multiplied by its row's s on the way to f16, and leave as 64-byte runs (four neighbouring rows of
// one k octet in operand order).
// Whatever the magnitude of a row, its largest element lands in [2^13, 2^14) and elements down to
// 2^-27 of it stay normal f16 numbers.  Rows of up to 4 * CH * 512 elements stay in registers
// between the two steps (CH chunks of 8 values per lane in each of a row's four waves, all requested
// at once); longer rows are read again (the second read hits the L2).
template <int XT>
struct RowChunk {                 // 8 consecutive activations of a row as loaded
    u32x4_t v[XT == 2 ? 2 : 1];
};

template <int XT>
__device__ __forceinline__ RowChunk<XT> load_row_chunk(const void* src, int64_t row, int K, int c)
{
    RowChunk<XT> o;
    if (XT == 2) {
        const u32x4_t* p = reinterpret_cast<const u32x4_t*>(reinterpret_cast<const float*>(src) + row * K + c * 8);
        o.v[0] = p[0];
        o.v[XT == 2 ? 1 : 0] = p[1];
    } else {
        o.v[0] = *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const uint16_t*>(src) + row * K + c * 8);
    }
    return o;
}

template <int XT>
__device__ __forceinline__ void row_chunk_values(const RowChunk<XT>& c, float v[8])
{
#pragma unroll
    for (int e = 0; e < 4; e++) {
        if (XT == 2) {
            v[e] = __builtin_bit_cast(float, (uint32_t)c.v[0][e]);
            v[4 + e] = __builtin_bit_cast(float, (uint32_t)c.v[XT == 2 ? 1 : 0][e]);
        } else {
            v[2 * e] = __builtin_bit_cast(float, c.v[0][e] << 16);
            v[2 * e + 1] = __builtin_bit_cast(float, c.v[0][e] & 0xffff0000u);
        }
    }
}

// A workgroup owns four rows and gives every row four waves: wave (r, p) takes the pieces of 512 k
// numbered p, p + 4, ... of row r (CH of them at most stay in registers between the two steps), the
// four parts of a row meet once through LDS for the row's largest magnitude (and sum of squares, added
// in part order).  One wave per row took 5 - 7 us for 512 rows of 4096 and 10 - 12 us for rows of 14336,
// most of it the latency of one wave walking its row.
template <int XT, bool NORM, int CH>
__global__ __launch_bounds__(1024) void stage_rows_kernel(const void* __restrict__ src, u32x4_t* __restrict__ dst, int M, int K,
                                                          Epilogue epi, float* __restrict__ ssq, float* __restrict__ unscale, Touch touch)
{
    static_assert(XT == 1 || XT == 2, "bf16 or fp32 activations");
    if ((int)blockIdx.x >= touch.first_group) {
        touch_weights(touch, (int)blockIdx.x - touch.first_group, (int)threadIdx.x, 1024);
        return;
    }
    if ((int)(blockIdx.x >> 2) * 16 >= M) return;              // (padding up to first_group)
    constexpr int PW = 4;                                      // waves per row
    __shared__ u32x4_t tile[PW][2][4 * kStagePitch];
    __shared__ float amax_part[4][PW], sq_part[4][PW];
    const int rb = blockIdx.x >> 2, r0 = (blockIdx.x & 3) * 4;          // row block, first of this workgroup's rows in it
    const int t = threadIdx.x, lane = t & 63, wv = t >> 6;
    const int r = wv & 3, part = wv >> 2;                               // my row of the four, my part of the row
    const int64_t row = min(rb * 16 + r0 + r, M - 1);      // (rows past M repeat the last one and are never read back)
    const int K8 = K >> 3, G = K8 >> 2;
    const int pieces = (K8 + 63) >> 6;                     // pieces of 64 chunks (512 k) in a row
    const bool resident = pieces <= PW * CH;

    // ---- the row's largest magnitude (and sum of squares)
    RowChunk<XT> keep[CH];
    float amax = 0.f, sq = 0.f;
    for (int p0 = 0; p0 < pieces; p0 += PW * CH) {
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const int piece = p0 + i * PW + part;
            if (piece < pieces) keep[i] = load_row_chunk<XT>(src, row, K, min(piece * 64 + lane, K8 - 1));
        }
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const int piece = p0 + i * PW + part;
            const int c = piece * 64 + lane;
            float v[8];
            if (piece < pieces && c < K8) {
                row_chunk_values<XT>(keep[i], v);
                if (NORM) {
                    float g[8];
                    load_gamma8_g(epi.gamma, epi.gamma_dt, c * 8, g);
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        sq = fmaf(v[e], v[e], sq);
                        v[e] *= g[e];
                    }
                }
#pragma unroll
                for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(v[e]));
            }
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        amax = fmaxf(amax, __shfl_xor(amax, off, 64));
        if (NORM) sq += __shfl_xor(sq, off, 64);
    }
    if (lane == 0) {
        amax_part[r][part] = amax;
        if (NORM) sq_part[r][part] = sq;
    }
    __syncthreads();
    amax = fmaxf(fmaxf(amax_part[r][0], amax_part[r][1]), fmaxf(amax_part[r][2], amax_part[r][3]));
    if (NORM) sq = ((sq_part[r][0] + sq_part[r][1]) + sq_part[r][2]) + sq_part[r][3];
    // amax = f * 2^e with f in [0.5, 1): s = 2^(14 - e) puts it in [2^13, 2^14); zero, Inf and NaN rows keep s = 1
    float s = 1.0f;
    if (amax > 0.f && amax < __builtin_inff()) {
        int e;
        (void)frexpf(amax, &e);
        s = ldexpf(1.0f, min(14 - e, 126));        // (rows below 2^-112: 2^126 keeps s and 1 / s normal numbers)
    }
    if (lane == 0 && part == 0 && rb * 16 + r0 + r < M) {
        unscale[row] = 1.0f / s;
        if (NORM) ssq[row] = sq;
    }

    // ---- scale, round to f16, through LDS into operand order (two tiles per part: one barrier per piece)
    auto convert = [&](const RowChunk<XT>& ch, int c) {
        float v[8];
        row_chunk_values<XT>(ch, v);
        if (NORM) {
            float g[8];
            load_gamma8_g(epi.gamma, epi.gamma_dt, min(c, K8 - 1) * 8, g);
#pragma unroll
            for (int e = 0; e < 8; e++) v[e] *= g[e];
        }
        Frag16 a;
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const half2_t h = {(_Float16)(v[2 * p] * s), (_Float16)(v[2 * p + 1] * s)};
            a.u[p] = as_u32(h);
        }
        return a.u;
    };
    const int tp = r * 64 + lane;                           // my place among the 256 threads of my part
    const int gl = tp >> 4, oct = (tp >> 2) & 3, rr = tp & 3;  // when writing out: group within the piece, k octet, row
    int round = 0;
    for (int p0 = 0; p0 < pieces; p0 += PW * CH) {
        if (!resident) {
#pragma unroll
            for (int i = 0; i < CH; i++) {
                const int piece = p0 + i * PW + part;
                if (piece < pieces) keep[i] = load_row_chunk<XT>(src, row, K, min(piece * 64 + lane, K8 - 1));
            }
        }
#pragma unroll
        for (int i = 0; i < CH; i++) {
            if (p0 + i * PW < pieces) {                      // (uniform over the workgroup: some part has this piece)
                const int piece = p0 + i * PW + part;
                u32x4_t* tl = tile[part][round & 1];
                if (piece < pieces) tl[r * kStagePitch + lane] = convert(keep[i], piece * 64 + lane);
                __syncthreads();
                const int g = piece * 16 + gl;
                if (piece < pieces && g < G) dst[((int64_t)rb * G + g) * 64 + oct * 16 + r0 + rr] = tl[rr * kStagePitch + gl * 4 + oct];
                round++;
            }
        }
    }
}

}  // namespace

int g_rows_kernel = 0;        // (set_gemm_tuning: 2 = experiments switch the few-rows kernel off, 1 = on whatever the width)
int g_touch = 2;              // (5 = the staging launch asks for no weights ahead of the multiply, 6 = only ahead of the few-rows kernel)
void set_gemm_tuning(int rows_kernel) { g_rows_kernel = rows_kernel >= 5 ? 0 : rows_kernel; g_touch = rows_kernel == 5 ? 0 : rows_kernel == 6 ? 1 : 2; }

bool gemm_rows_takes(const WeightView& w, int M, int num_cus, const Epilogue& epi)
{
    return g_rows_kernel != 2 && gemm_rows_serves(w, M, g_rows_kernel == 1 ? 1 : num_cus, epi);
}

// the extra workgroups of a staging launch (grid_x grows by them) for a call of 33 rows or more that goes through the
// row-scaling pass (bf16 / fp32 rows) and on to the few-row kernel or to the tiled kernels' 64-column tiles: up to
// 16 MB of the tensor, from the K tile every column group starts at.  Per call: 4096 -> 14336 at 64 rows 19.6 -> 18.7
// us with 16 of the 32 K tiles (no gain with all of them: the launch then takes as long as the reads), 4096 -> 4096
// at 64 / 128 rows 13.6 / 14.6 -> 12.4 / 13.4, 4096 -> 1024 13.1 -> 11.7, 8192 -> 4096 at 128 rows 25.1 -> 22.9.  Not
// for f16 rows (their pass only reorders and is over before the reads are: 4096 -> 14336 at 64 rows 18.6 -> 19.1),
// for 17 .. 32 fp32 rows (12.5 -> 13.4 on 4096 -> 8192) or for K up to 2048.
// whether launch_nf gives a FAST-mode call of M rows the 64-column tiles (one row tile of up to 128 rows)
static bool few_rows_tiles64(const WeightView& w, int M, int num_cus, const Epilogue& epi)
{
    if (M > 128 || epi.kind == kEpiSwiglu) return false;
    const int64_t tiles64 = (w.NT + 3) / 4;
    return tiles64 * 4 >= 3 * num_cus || (tiles64 * 2 >= num_cus && w.KT <= 48);
}

static Touch plan_touch(const WeightView& w, int mc, int num_cus, const Epilogue& ec, bool exact, unsigned& grid_x)
{
    Touch tc = {nullptr, 0x7fffffff, w.NT, w.KT, 1, tile_bytes(w.bits), 0, 0, 0};
    if (g_touch == 0 || exact || mc < 33 || w.KT < 32) return tc;
    const int64_t per_k_tile = (int64_t)w.NT * tile_bytes(w.bits);
    int nf = 0, groups = 0;
    if (gemm_rows_takes(w, mc, num_cus, ec)) {
        nf = gemm_rows_blocks(w, mc, g_rows_kernel == 1 ? 1 : num_cus, ec);
        groups = (w.NT + nf - 1) / nf;
    } else if (g_touch >= 2 && per_k_tile * w.KT <= ((int64_t)40 << 20) && few_rows_tiles64(w, mc, num_cus, ec)) {
        // the 128 x 64 / 64 x 64 tiles of the tiled kernels (65 .. 128 rows on wide outputs; 4096 -> 14336 at 128 rows:
        // 27.5 us, 24.3 with the same tensor every call): 4096 -> 14336 at 65 / 100 / 128 rows 25.3 / 27.1 / 28.1 ->
        // 23.9 / 26.0 / 27.3 us, 4096 -> 11008 23.9 / 25.5 / 26.5 -> 23.3 / 24.6 / 25.2; nothing on tensors of 66 MB
        nf = 4;
        tc.tiles = (w.NT + 3) / 4;
        groups = (tc.tiles + 7) / 8 * 8;
        tc.per_xcd = groups / 8;
    } else {
        return tc;
    }
    tc.base = w.base;
    tc.NF = nf;
    tc.ahead = (int)std::min<int64_t>(w.KT, std::max<int64_t>(4, ((int64_t)16 << 20) / per_k_tile));
    tc.first_group = (int)((grid_x + 7) / 8 * 8);
    grid_x = (unsigned)(tc.first_group + groups);
    return tc;
}

hipError_t launch_gemm(const WeightView& w, const void* x, int xdt, int M, void* y, int ydt,
                       int num_cus, bool exact, void* workspace, size_t workspace_bytes, const Epilogue& epi,
                       hipStream_t st)
{
    if (xdt == kF32 && exact) return hipErrorNotSupported;   // api.hip walks exact fp32 prefill through the decode kernel
    // FAST multiplies in f16: bf16 activations are widened, fp32 activations rounded to f16
    // (both behind a power-of-two scale per row that the epilogue undoes)
    const bool widen = !exact && xdt != kF16;
    const float out_scale = 1.0f;
    const int kdt = widen ? kF16 : xdt;
    // Rows are staged through the workspace in chunks that fit it; work on one stream is
    // ordered, so a chunk's multiply is done before the next chunk overwrites the stage.
    // First half of the workspace: staged X; second half: partial sums of a K split.
    const size_t half = workspace_bytes / 2;
    float* part = reinterpret_cast<float*>(static_cast<char*>(workspace) + half);
    // The last MiB of the first half: per-row statistics - partial sums of squares of a folded
    // RMSNorm (rows of a chunk x K / 512 floats: less than half / 256 bytes) and, in its last
    // quarter, the per-row power of two of widened activations (at most 65536 rows per chunk).
    const size_t stats_bytes = (size_t)1 << 20;
    if (!workspace || half <= stats_bytes) return hipErrorOutOfMemory;
    float* ssq_part = reinterpret_cast<float*>(static_cast<char*>(workspace) + half - stats_bytes);
    float* unscale = reinterpret_cast<float*>(static_cast<char*>(workspace) + half - stats_bytes / 4);
    const int64_t row_bytes = (int64_t)w.K * (xdt == kF32 ? 4 : 2);        // a row of the caller's X
    const int64_t max_rows =
        std::min<int64_t>(65536, (int64_t)((half - stats_bytes) / (size_t)(w.K * 2)) / 256 * 256);    // staged rows are 16-bit
    if (max_rows < 256) return hipErrorOutOfMemory;
    const size_t ysize = ydt == kF32 ? 4 : 2;
    for (int64_t m_lo = 0; m_lo < M; m_lo += max_rows) {
        const int mc = (int)((M - m_lo) < max_rows ? (M - m_lo) : max_rows);
        const u32x4_t* xs = reinterpret_cast<const u32x4_t*>(static_cast<const char*>(x) + m_lo * row_bytes);
        const int64_t n_out = epi.kind == kEpiSwiglu ? w.N / 2 : w.N;
        void* yc = static_cast<char*>(y) + (size_t)m_lo * n_out * ysize;
        Epilogue ec = epi;                 // this row chunk's slice of the residual
        if (epi.kind == kEpiAdd) ec.residual = static_cast<const char*>(epi.residual) + (size_t)m_lo * n_out * ysize;
        const int K8 = w.K / 8;
        const dim3 grid((unsigned)((mc + 15) / 16), (unsigned)((K8 / 4 + kStageGroups - 1) / kStageGroups));
        u32x4_t* xst = reinterpret_cast<u32x4_t*>(workspace);
        NormStats ns = {ssq_part, (int)grid.y, nullptr};
        if (widen) {
            // per-row scaled f16 operands; one sum of squares per row
            ns = NormStats{ssq_part, 1, unscale};
            dim3 rgrid((unsigned)((mc + 15) / 16) * 4);
            const Touch touch = plan_touch(w, mc, num_cus, ec, exact, rgrid.x);
            // pieces of 512 k a lane keeps in registers (a row is split over four waves): the whole row when it has
            // at most 16384 (bf16) or 8192 (fp32) elements
            const int batches = ((K8 + 63) / 64 + 3) / 4;
#define CYBQ_STAGE_ROWS(XT, NORM, CH) \
    hipLaunchKernelGGL((stage_rows_kernel<XT, NORM, CH>), rgrid, dim3(1024), 0, st, xs, xst, mc, w.K, epi, ssq_part, unscale, touch)
#define CYBQ_STAGE_ROWS_CH(XT, NORM, C1, C2, C3)              \
    do {                                                      \
        if (batches <= C1) CYBQ_STAGE_ROWS(XT, NORM, C1);     \
        else if (batches <= C2) CYBQ_STAGE_ROWS(XT, NORM, C2); \
        else CYBQ_STAGE_ROWS(XT, NORM, C3);                   \
    } while (0)
            if (xdt == kF32 && epi.gamma) CYBQ_STAGE_ROWS_CH(2, true, 1, 2, 4);
            else if (xdt == kF32) CYBQ_STAGE_ROWS_CH(2, false, 1, 2, 4);
            else if (epi.gamma) CYBQ_STAGE_ROWS_CH(1, true, 2, 4, 8);
            else CYBQ_STAGE_ROWS_CH(1, false, 2, 4, 8);
#undef CYBQ_STAGE_ROWS_CH
#undef CYBQ_STAGE_ROWS
        } else if (epi.gamma) {
            if (xdt == kBF16) hipLaunchKernelGGL((stage_x_kernel<true, true>), grid, dim3(256), 0, st, xs, xst, mc, K8, epi, ssq_part);
            else hipLaunchKernelGGL((stage_x_kernel<false, true>), grid, dim3(256), 0, st, xs, xst, mc, K8, epi, ssq_part);
        } else {
            hipLaunchKernelGGL((stage_x_kernel<false, false>), grid, dim3(256), 0, st, xs, xst, mc, K8, epi, ssq_part);
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        // few rows on a wide output, FAST mode: the kernel of gemm_rows.hip (waves split K, no LDS on the way)
        if (!exact && kdt == kF16 && gemm_rows_takes(w, mc, num_cus, ec)) {
            e = launch_gemm_rows(w, workspace, mc, yc, ydt, ec, ns.part, ns.nblk, ns.unscale, g_rows_kernel == 1 ? 1 : num_cus, st);
            if (e != hipSuccess) return e;
            continue;
        }
        if (w.bits == 4) {
            e = kdt == kBF16 ? launch_nf<4, 1>(w, workspace, mc, yc, ydt, exact, out_scale, part, half, num_cus, ec, ns, st)
                             : launch_nf<4, 0>(w, workspace, mc, yc, ydt, exact, out_scale, part, half, num_cus, ec, ns, st);
        } else {
            e = kdt == kBF16 ? launch_nf<8, 1>(w, workspace, mc, yc, ydt, exact, out_scale, part, half, num_cus, ec, ns, st)
                             : launch_nf<8, 0>(w, workspace, mc, yc, ydt, exact, out_scale, part, half, num_cus, ec, ns, st);
        }
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace cybq
