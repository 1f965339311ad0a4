// gemv1.hip - decode kernel for one or two activation rows: y[M,N] = x[M,K] * W^T, f16 activations.
// (Described for one row; the two-row form is at the kernel's template parameters.)
//
// HBM-bound: a workgroup owns one 16-row strip of W (one contiguous run of memory) and
// requests all of it up front; everything else is arranged so that nothing stands between
// the kernel's start and those requests, and so that little remains to do once the last
// byte has arrived.
//
//  * No LDS staging of x, no barrier before the arithmetic.  A wave works on "sets" of four
//    consecutive K tiles (512 k, 16 scale groups).  Its MFMA A operand for a set is ONE
//    16-byte load per lane: lane (i = l & 15, o = l >> 4) reads x[512*set + 32*i + 8*o ..+8],
//    so row i of the 16x16x32 MFMA holds the activations of scale group i of the set.
//    Multiplying that operand with the weights of group g gives the wanted dot products in
//    output row g (rows != g pair the weights with another group's activations and are
//    ignored).  Output row g = 4*b + r lives in register r of lane block b (lanes 16b..16b+15):
//    lane block b ends up with tile b of the set, register r with scale group r - exactly
//    the four scales a lane gets from one 8-byte load of the tile's scale record.
//  * Weight operands cost two shifts and four ANDs per eight weights: the native nibble
//    order makes ((w << 2) & 0x003C003C) two f16 subnormals 4u * 2^-24 (u = q + 8), which the
//    matrix cores take at face value.  The bias comes off inside the same accumulation: the
//    MFMA's C operand is x times the constant -32 * 2^-24 (one extra MFMA per set, its row g is
//    exactly -8 * 4 * sum of group g's activations).  Odd groups sit in the high nibbles (64u *
//    2^-24, constant -512 * 2^-24); the 16 and the 2^22 are folded into the final scaling.
//    Q8 bytes u = q + 128 become subnormals with one byte permute per pair.
//  * Per-group f16 scales are applied in fp32 on the MFMA results; lanes add up what their
//    block owns, blocks meet through a 16x16x4 fp32 MFMA against ones, waves through LDS:
//    the order of all additions is fixed, results are reproducible.
#include "cybq_device.h"
#include "cybq_internal.h"

namespace cybq {

namespace {

__device__ __forceinline__ void store_out1(void* y, int ydt, int64_t idx, float v)
{
    if (ydt == kF32) reinterpret_cast<float*>(y)[idx] = v;
    else if (ydt == kF16) reinterpret_cast<_Float16*>(y)[idx] = (_Float16)v;
    else reinterpret_cast<uint16_t*>(y)[idx] = f32_to_bf16_bits(v);
}

__device__ __forceinline__ float load_out1(const void* p, int dt, int64_t idx)
{
    if (dt == kF32) return reinterpret_cast<const float*>(p)[idx];
    if (dt == kF16) return (float)reinterpret_cast<const _Float16*>(p)[idx];
    return __builtin_bit_cast(float, (uint32_t)reinterpret_cast<const uint16_t*>(p)[idx] << 16);
}

// B operand of scale group r of one tile as loaded by a lane
// (XBF: bf16 activations - the operand is the bf16 number 128 + u, there are no bf16 subnormals to use:
// their products with x would leave the fp32 range)
template <int BITS, bool XBF>
__device__ __forceinline__ Frag16 sub_operand(const u32x4_t (&q)[BITS == 4 ? 1 : 2], int r, uint32_t magic)
{
    Frag16 b;
    if (XBF) {
        uint32_t o[4];
        if (BITS == 4) unpack_q4_bf16_biased(q[0][2 * (r >> 1)], q[0][2 * (r >> 1) + 1], r & 1, magic, o);
        else unpack_q8_bf16_biased(q[BITS == 4 ? 0 : (r >> 1)][(r & 1) * 2], q[BITS == 4 ? 0 : (r >> 1)][(r & 1) * 2 + 1], o);
        b.u = (u32x4_t){o[0], o[1], o[2], o[3]};
    } else if (BITS == 4) {
        uint32_t o[4];
        unpack_q4_sub(q[0][2 * (r >> 1)], q[0][2 * (r >> 1) + 1], r & 1, o);
        b.u = (u32x4_t){o[0], o[1], o[2], o[3]};
    } else {
        // bytes [b0 b1 b2 b3] -> halves [b0, b1], [b2, b3] zero-extended (selector 0x0c = constant 0)
        const uint32_t w0 = q[BITS == 4 ? 0 : (r >> 1)][(r & 1) * 2], w1 = q[BITS == 4 ? 0 : (r >> 1)][(r & 1) * 2 + 1];
        b.u = (u32x4_t){__builtin_amdgcn_perm(0u, w0, 0x0c010c00u), __builtin_amdgcn_perm(0u, w0, 0x0c030c02u),
                        __builtin_amdgcn_perm(0u, w1, 0x0c010c00u), __builtin_amdgcn_perm(0u, w1, 0x0c030c02u)};
    }
    return b;
}

// SETS: sets a wave owns (set index wv + nwaves * h).  NS: strips per workgroup (2 = a gate strip
// and its up strip, SwiGLU epilogue).  EVEN: K is a multiple of 512 and every wave has SETS
// whole sets, so nothing needs clamping.  NW: waves that split K when known at compile time (0 = any).
// SPLIT (NS = 2, NW > 0): the workgroup has 2 * NW waves, waves [0, NW) take the gate strip and
// [NW, 2 NW) the up strip - per wave the same work as with one strip per workgroup (a wave that
// holds both strips' tiles has twice the requests in flight and half the waves to hide them).
// RES (MR = 1): the residual-add epilogue; the residual is requested first of all, so that it is there
// long before the sums are (asked for at the end it would cost the kernel one more trip to memory).
// MR: batch rows, 1 or 2.  The 16 rows of an A operand are MR batch rows x 16 / MR scale groups:
// an operand covers 4 / MR tiles of a set, a set takes MR operand loads and MR scale loads per lane,
// and lane block b ends up with batch row b / (4 / MR) and the tiles t = b mod (4 / MR), + 4 / MR, ...
// of the set.  (The scheme works for four rows as well - 12 load instructions per set instead of 6 -
// and was measured slower there than the batched-rows kernel: 8.8 against 8.6 us at 4096 -> 14336.)
// XBF: bf16 activations (bf16 MFMA, biased weight operands 128 + u, the constant operand is -136 / -128 for
// every group and nothing is left to fold into the final scaling).
// NORM: RMSNorm folded in (y = epilogue(rstd[m] * sum_k round(x * gamma) * W), rstd = 1 / sqrt(mean x^2 + eps)):
// gamma is requested next to x, the operand becomes x * gamma (fp32, rounded once to the operand type) in
// registers, the squares of x are summed per wave on the way and meet across waves with the partial sums.
template <int BITS, int SETS, int NS, bool EVEN, int NW, bool SPLIT = false, bool RES = false, int MR = 1, bool XBF = false,
          bool NORM = false>
// The arguments are scalars in the order the kernel needs them: the compiler is asked to have
// them delivered in registers at wave start (kernel argument preload), so the first requests do
// not wait for a load of the argument block.  (14 dwords are preloaded; the launch's wave count travels
// with them, the launch geometry is not among what is preloaded.  flags = output type | epilogue << 4 |
// M << 8 | gamma type << 16.  aux0: the residual, or gamma with a folded norm - then the residual is aux1.)
__global__ __launch_bounds__(1024) void gemv1_kernel(const uint8_t* __restrict__ wbase, const _Float16* __restrict__ x,
                                                     const void* __restrict__ aux0, void* __restrict__ y, int KT, int K,
                                                     int launch_waves, int n_rows, int flags, float eps,
                                                     const void* __restrict__ aux1)
{
    static_assert(!(NORM && RES), "the residual prefetch has no folded-norm form");
    const void* const residual = NORM ? aux1 : aux0;
    static_assert(MR == 1 || MR == 2, "batch rows per operand");
    static_assert(!RES || MR == 1, "the residual prefetch is the one-row form");
    constexpr int QV = BITS == 4 ? 1 : 2;
    constexpr int GPA = 16 / MR;                  // scale groups per A operand
    constexpr int TPA = 4 / MR;                   // tiles per A operand
    __shared__ float red[NS * MR * 16 * 16];
    __shared__ __attribute__((aligned(16))) float ssq_red[NORM ? MR * 16 : 4];       // [batch row][wave]
    const int out_dt = flags & 15, epi_kind = (flags >> 4) & 15, M = (flags >> 8) & 255, gdt = (flags >> 16) & 15;
    const int tid = threadIdx.x, lane = tid & 63;
    static_assert(!SPLIT || (NS == 2 && NW > 0), "split workgroups are gate / up pairs with a known wave count");
    constexpr int NL = SPLIT ? 1 : NS;            // strips a wave works on
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int wv = wave, half = 0;                      // my place among the waves that split K; SPLIT: my strip of the pair
    if constexpr (SPLIT) {
        wv = wave % NW;
        half = wave / NW;
    }
    const int nwaves = NW ? NW : launch_waves;          // NW = 0: whatever the launch says
    const int row = lane & 15, blk = lane >> 4;
    const int my_tile = blk % TPA;                // the tiles of a set this lane block ends up with: my_tile + TPA * c

    uint32_t res_word = 0;            // the aligned 32-bit word that holds this lane's residual element
    uint32_t res_addr = 0;
    if constexpr (RES) {
        const int n = min((int)blockIdx.x * 16 + row, n_rows - 1);
        const uintptr_t p = reinterpret_cast<uintptr_t>(residual) + (uintptr_t)n * (out_dt == kF32 ? 4u : 2u);
        res_addr = (uint32_t)p;
        res_word = *reinterpret_cast<const uint32_t*>(p & ~(uintptr_t)3);
    }
    // A row i of an operand: batch row i / GPA (rows past M repeat the last one, their sums are not stored),
    // scale group i % GPA of the operand's tiles
    const _Float16* xrow = x;
    if constexpr (MR > 1) xrow += min(row / GPA, M - 1) * K;
    const int xk = (row % GPA) * 32 + blk * 8;
    Frag16 a[SETS][MR];
    u32x4_t gam[NORM ? SETS : 1][MR][2];      // NORM: gamma at the operand's k (fp32: 32 bytes, else 16 and a repeat)
    u32x2_t sc[NL][SETS][MR];
    u32x4_t q[NL][SETS][4][QV];
    bool tile_ok[SETS][MR];           // this lane block's tiles of the set exist (!EVEN)
#pragma unroll
    for (int h = 0; h < SETS; h++) {
        const int set = wv + nwaves * h;
#pragma unroll
        for (int p = 0; p < MR; p++) {
            const int k = set * 512 + p * (TPA * 128) + xk;
            const int kc = EVEN ? k : min(k, K - 8);
            a[h][p].u = *reinterpret_cast<const u32x4_t*>(xrow + kc);
            if (!EVEN) tile_ok[h][p] = 4 * set + my_tile + TPA * p < KT;
            if constexpr (NORM) {
                const int esz = gdt == kF32 ? 4 : 2;
                const char* gp = static_cast<const char*>(aux0) + (int64_t)kc * esz;
                gam[h][p][0] = *reinterpret_cast<const u32x4_t*>(gp);
                gam[h][p][1] = *reinterpret_cast<const u32x4_t*>(gp + (esz == 4 ? 16 : 0));
            }
        }
    }
    // Addresses: one wave-uniform 64-bit base per (strip, set) plus a 32-bit lane offset, so the
    // requests go out after a handful of scalar instructions.
    constexpr int TB = kTileBytes<BITS>, QB = kTileQBytes<BITS>;
    const uint32_t lane_q = (uint32_t)lane * 16u;
    const uint32_t lane_s = (uint32_t)QB + (uint32_t)row * 8u;
#pragma unroll
    for (int st = 0; st < NL; st++) {
        const int strip_tile = ((int)blockIdx.x * NS + st + half) * KT;    // tile indices fit 32 bits
#pragma unroll
        for (int h = 0; h < SETS; h++) {
            const int t0 = 4 * (wv + nwaves * h);
            if (EVEN) {
                const uint8_t* sb = wbase + (int64_t)(strip_tile + t0) * TB;
#pragma unroll
                for (int c = 0; c < MR; c++)
                    sc[st][h][c] = __builtin_nontemporal_load(
                        reinterpret_cast<const u32x2_t*>(sb + ((uint32_t)(my_tile + TPA * c) * TB + lane_s)));
#pragma unroll
                for (int b = 0; b < 4; b++)
#pragma unroll
                    for (int v = 0; v < QV; v++)
                        q[st][h][b][v] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(sb + (b * TB + v * 1024) + lane_q));
            } else {
                const uint8_t* strip = wbase + (int64_t)strip_tile * TB;
#pragma unroll
                for (int c = 0; c < MR; c++)
                    sc[st][h][c] = __builtin_nontemporal_load(
                        reinterpret_cast<const u32x2_t*>(strip + ((uint32_t)min(t0 + my_tile + TPA * c, KT - 1) * TB + lane_s)));
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    const uint8_t* tp = strip + (int64_t)min(t0 + b, KT - 1) * TB;
#pragma unroll
                    for (int v = 0; v < QV; v++)
                        q[st][h][b][v] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(tp + v * 1024 + lane_q));
                }
            }
        }
    }
    // Everything the tail needs from the kernel arguments is kept live from here on: left to
    // itself the compiler fetches an argument where it is first used, i.e. after the final barrier.
    asm volatile("" ::"s"(n_rows), "s"(out_dt), "s"(epi_kind), "s"(residual), "s"(y), "s"(M));
    if (!NW) asm volatile("" ::"s"(nwaves));
    __builtin_amdgcn_sched_barrier(0);       // every request is out before any arithmetic

    if (!EVEN) {
#pragma unroll
        for (int h = 0; h < SETS; h++) {
#pragma unroll
            for (int p = 0; p < MR; p++) {
                // activations past K (the padded tail of the last tile) count as zero; a tile past
                // the end of the strip was clamped to the last one and gets scale zero
                const bool x_ok = (wv + nwaves * h) * 512 + p * (TPA * 128) + xk < K;
#pragma unroll
                for (int e = 0; e < 4; e++) a[h][p].u[e] = x_ok ? a[h][p].u[e] : 0u;
#pragma unroll
                for (int st = 0; st < NL; st++) {
                    sc[st][h][p][0] = tile_ok[h][p] ? sc[st][h][p][0] : 0u;
                    sc[st][h][p][1] = tile_ok[h][p] ? sc[st][h][p][1] : 0u;
                }
            }
        }
    }

    float ssq = 0.f;                  // NORM: squares of the activations this lane holds (batch row (lane & 15) / GPA)
    if constexpr (NORM) {
#pragma unroll
        for (int h = 0; h < SETS; h++)
#pragma unroll
            for (int p = 0; p < MR; p++) {
                float g[8];
                if (gdt == kF32) {
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const uint32_t lo = gam[h][p][0][e], hi = gam[h][p][1][e];       // (values first: a bit cast
                        g[e] = __builtin_bit_cast(float, lo);                             // straight from a vector
                        g[4 + e] = __builtin_bit_cast(float, hi);                         // element read element 0)
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const uint32_t v = gam[h][p][0][e];
                        g[2 * e] = gdt == kF16 ? f16_bits_to_f32(v & 0xffffu) : __builtin_bit_cast(float, v << 16);
                        g[2 * e + 1] = gdt == kF16 ? f16_bits_to_f32(v >> 16) : __builtin_bit_cast(float, v & 0xffff0000u);
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const uint32_t v = a[h][p].u[e];
                    float x0, x1;
                    if (XBF) {
                        x0 = __builtin_bit_cast(float, v << 16);
                        x1 = __builtin_bit_cast(float, v & 0xffff0000u);
                    } else {
                        x0 = f16_bits_to_f32(v & 0xffffu);
                        x1 = f16_bits_to_f32(v >> 16);
                    }
                    ssq = __builtin_fmaf(x1, x1, __builtin_fmaf(x0, x0, ssq));
                    x0 *= g[2 * e];
                    x1 *= g[2 * e + 1];
                    if (XBF) {
                        a[h][p].u[e] = pack_bf16x2(x0, x1);
                    } else {
                        const half2_t hh = {(_Float16)x0, (_Float16)x1};
                        a[h][p].u[e] = as_u32(hh);
                    }
                }
            }
    }
    Frag16 kL, kH;
    constexpr bool TWO = BITS == 4 && !XBF;           // even and odd groups carry different factors
    constexpr uint32_t cH = XBF ? (BITS == 4 ? kBf16Neg136x2 : kBf16Neg128x2) : (BITS == 4 ? kSubBiasH : kSubBiasQ8);
    constexpr float unscale = XBF ? 1.0f : (BITS == 4 ? kSubUnscale : kSubUnscaleQ8);
    uint32_t magic = 0;
    if constexpr (XBF && BITS == 4) magic = q4_magic_vgpr_bf16();
    auto mma = [](const Frag16& a, const Frag16& b, float4_t c) {
        if constexpr (XBF) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, b.b, c, 0, 0, 0);
        else return __builtin_amdgcn_mfma_f32_16x16x32_f16(a.h, b.h, c, 0, 0, 0);
    };
    kL.u = (u32x4_t){kSubBiasL, kSubBiasL, kSubBiasL, kSubBiasL};
    kH.u = (u32x4_t){cH, cH, cH, cH};
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    float4_t biasL[SETS][MR], biasH[SETS][MR];
#pragma unroll
    for (int h = 0; h < SETS; h++)
#pragma unroll
        for (int p = 0; p < MR; p++) {
            if (TWO) biasL[h][p] = mma(a[h][p], kL, zero);
            biasH[h][p] = mma(a[h][p], kH, zero);
        }

    // A lane block holds meaningful sums only for its own tiles of every set (one in TPA).  All
    // tiles are accumulated with the lane's own scales, TPA sums side by side (the others are
    // finite and unused), and the meaningful one is picked once at the end.  Even groups (low
    // nibbles) and odd groups (high nibbles, 16 times too large) are kept apart until the final scaling.
    float accL[NL][TPA], accH[NL][TPA];
#pragma unroll
    for (int st = 0; st < NL; st++)
#pragma unroll
        for (int b = 0; b < TPA; b++) accL[st][b] = accH[st][b] = 0.f;
    constexpr int T = NL * SETS * 4;
    float4_t dprev[4];
#pragma unroll
    for (int i = 0; i <= T; i++) {
        // MFMAs of tile i first, then the scaling of tile i - 1 whose results have landed meanwhile
        float4_t d[4];
        if (i < T) {
            const int st = i / (SETS * 4), h = (i / 4) % SETS, b = i % 4, p = b / TPA;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const Frag16 B = sub_operand<BITS, XBF>(q[st][h][b], r, magic);
                d[r] = mma(a[h][p], B, (!TWO || (r & 1)) ? biasH[h][p] : biasL[h][p]);
            }
        }
        if (i > 0) {
            const int st = (i - 1) / (SETS * 4), h = ((i - 1) / 4) % SETS, b = (i - 1) % 4, p = b / TPA, slot = b % TPA;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint32_t sb = (r & 1) ? (sc[st][h][p][r >> 1] >> 16) : (sc[st][h][p][r >> 1] & 0xffffu);
                const float sf = f16_bits_to_f32(sb);
                if (TWO && (r & 1)) accH[st][slot] = __builtin_fmaf(sf, dprev[r][r], accH[st][slot]);
                else accL[st][slot] = __builtin_fmaf(sf, dprev[r][r], accL[st][slot]);
            }
        }
#pragma unroll
        for (int r = 0; r < 4; r++) dprev[r] = d[r];
        __builtin_amdgcn_sched_barrier(0);
    }

    // Blocks meet inside the matrix pipe: with B[k = block][n] = the block's sum and A[m][k] = 1 where
    // block k belongs to batch row m, a 16x16x4 fp32 MFMA leaves sum_k B[k][n] in row m - one
    // instruction instead of two cross-lane round trips.  Waves meet through LDS; the last sum is the
    // same trick again: lane block j adds the partial sums of waves 4i + j in order of i, the MFMA
    // adds the four blocks.
    const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
    const float mine = (MR == 1 || blk / TPA == row) ? 1.0f : 0.0f;
#pragma unroll
    for (int st = 0; st < NL; st++) {
        float tb[TPA];
#pragma unroll
        for (int b = 0; b < TPA; b++) tb[b] = TWO ? accL[st][b] + accH[st][b] * 0.0625f : accL[st][b];
        float t = tb[0];
#pragma unroll
        for (int b = 1; b < TPA; b++) t = my_tile == b ? tb[b] : t;
        const float4_t sum = __builtin_amdgcn_mfma_f32_16x16x4f32(mine, t, zero4, 0, 0, 0);
        if (lane < 16) {
#pragma unroll
            for (int m = 0; m < MR; m++) red[(((st + half) * MR + m) * 16 + wv) * 16 + lane] = sum[m];
        }
    }
    if constexpr (NORM) {
        // rows of the operand first (the four lane blocks of a row meet in an fp32 MFMA against ones), then the
        // rows that belong to a batch row: the same 0/1 matrix that joins the lane blocks' sums
        const float4_t r1 = __builtin_amdgcn_mfma_f32_16x16x4f32(ssq, 1.0f, zero4, 0, 0, 0);
        const float t = (r1[0] + r1[1]) + (r1[2] + r1[3]);
        const float4_t r2 = __builtin_amdgcn_mfma_f32_16x16x4f32(mine, t, zero4, 0, 0, 0);
        if (lane == 0 && half == 0) {
#pragma unroll
            for (int m = 0; m < MR; m++) ssq_red[m * 16 + wv] = r2[m];
        }
    }
    __syncthreads();
    if (tid >= 64) return;
    constexpr int SLOTS = NW ? (NW + 3) / 4 : 4;
    float outv[NS][MR];
#pragma unroll
    for (int st = 0; st < NS; st++)
#pragma unroll
        for (int m = 0; m < MR; m++) {
            float t[SLOTS];
#pragma unroll
            for (int i = 0; i < SLOTS; i++) t[i] = red[((st * MR + m) * 16 + min(4 * i + blk, 15)) * 16 + row];
            float v = 0.f;
#pragma unroll
            for (int i = 0; i < SLOTS; i++) v += 4 * i + blk < nwaves ? t[i] : 0.f;
            outv[st][m] = __builtin_amdgcn_mfma_f32_16x16x4f32(1.0f, v, zero4, 0, 0, 0)[0] * unscale;
        }
    if constexpr (NORM) {
#pragma unroll
        for (int m = 0; m < MR; m++) {
            // (four vector reads in flight rather than a loop of dependent ones; hardware reciprocal
            // and reciprocal square root, 1 ulp each)
            float t = 0.f;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4_t v = *reinterpret_cast<const float4_t*>(ssq_red + m * 16 + 4 * q);
#pragma unroll
                for (int e = 0; e < 4; e++) t += 4 * q + e < nwaves ? v[e] : 0.f;
            }
            const float rstd = __builtin_amdgcn_rsqf(fmaf(t, __builtin_amdgcn_rcpf((float)K), eps));
#pragma unroll
            for (int st = 0; st < NS; st++) outv[st][m] *= rstd;
        }
    }
    if (lane >= 16) return;
    const int n = blockIdx.x * 16 + lane;
    if (NS == 2) {               // SwiGLU: strips 2i / 2i+1 are gate / up of output strip i
        const int n_out = n_rows >> 1;
#pragma unroll
        for (int m = 0; m < MR; m++)
            if (m < M && n < n_out) store_out1(y, out_dt, (int64_t)m * n_out + n, silu_mul(outv[0][m], outv[NS - 1][m]));
        return;
    }
    if (n < n_rows) {
#pragma unroll
        for (int m = 0; m < MR; m++) {
            float v = outv[0][m];
            if constexpr (RES) {
                const uint32_t h = (res_addr & 2u) ? res_word >> 16 : res_word & 0xffffu;
                v += out_dt == kF32 ? __builtin_bit_cast(float, res_word)
                                    : (out_dt == kF16 ? f16_bits_to_f32(h) : __builtin_bit_cast(float, h << 16));
            } else if ((MR > 1 || NORM) && epi_kind == kEpiAdd) {
                if (m < M) v += load_out1(residual, out_dt, (int64_t)m * n_rows + n);
            }
            if (m < M) store_out1(y, out_dt, (int64_t)m * n_rows + n, v);
        }
    }
}

// sets of four K tiles a wave may own (all of them in registers, 16 waves per workgroup at
// most: 128 registers per lane): two, three for Q4 with one strip per workgroup, one for
// Q8 gate / up pairs; with two batch rows per operand two (Q4, one strip) or one; with a folded norm
// (gamma travels in registers next to x) two for one row and one strip, else one
constexpr int max_sets_per_wave(int bits, int ns, int mr, bool norm)
{
    if (norm) return ns == 1 && mr == 1 ? 2 : 1;
    if (mr == 1) return bits == 4 ? (ns == 1 ? 3 : 2) : (ns == 1 ? 2 : 1);
    return bits == 4 && ns == 1 ? 2 : 1;
}

struct Shape1 {        // how a strip's K is split over waves
    int per_wave, nwaves;
    bool even, k8;
};

Shape1 shape_of(const WeightView& w)
{
    const int nsets = (w.KT + 3) / 4;
    Shape1 s;
    s.per_wave = (nsets + 15) / 16;
    s.nwaves = (nsets + s.per_wave - 1) / s.per_wave;
    s.even = w.K % 512 == 0 && nsets % s.nwaves == 0;
    s.k8 = s.even && s.nwaves == 8 && s.per_wave == 1;          // K = 4096: the shape most decode launches have
    return s;
}

template <int BITS, int SETS, int NS, int MR, bool XBF, bool NORM>
hipError_t launch1_e(const WeightView& w, const void* x, int M, void* y, int ydt, const Shape1& sh, const Epilogue& epi,
                     hipStream_t st)
{
    const int nwaves = sh.nwaves;
    const dim3 grid((unsigned)(w.NT / NS)), block((unsigned)nwaves * 64);
    const _Float16* xh = reinterpret_cast<const _Float16*>(x);
    const int flags = ydt | (epi.kind << 4) | (M << 8) | (epi.gamma_dt << 16);
    const void* aux0 = NORM ? epi.gamma : epi.residual;
#define CYBQ_GEMV1_LAUNCH(EVEN_, NW_, SPLIT_, RES_, BLOCK_)                                                                          \
    hipLaunchKernelGGL((gemv1_kernel<BITS, SETS, NS, EVEN_, NW_, SPLIT_, (RES_) && !NORM, MR, XBF, NORM>), grid, BLOCK_, 0, st, w.base, xh, \
                       aux0, y, w.KT, w.K, nwaves, w.N, flags, epi.eps, epi.residual)
    const bool k8 = sh.k8 && SETS == 1;
    if constexpr (NS == 2) {
        if constexpr (SETS == 1) {
            if (k8) CYBQ_GEMV1_LAUNCH(true, 8, true, false, dim3(1024));
            else if constexpr (MR > 1) return hipErrorInvalidValue;        // gemv1_serves() said no
            else if (sh.even) CYBQ_GEMV1_LAUNCH(true, 0, false, false, block);
            else CYBQ_GEMV1_LAUNCH(false, 0, false, false, block);
        } else if constexpr (MR == 1) {
            if (sh.even) CYBQ_GEMV1_LAUNCH(true, 0, false, false, block);
            else CYBQ_GEMV1_LAUNCH(false, 0, false, false, block);
        } else return hipErrorInvalidValue;
    } else if (MR == 1 && !NORM && epi.kind == kEpiAdd) {
        if constexpr (MR == 1 && !NORM) {
            if (k8) CYBQ_GEMV1_LAUNCH(true, (SETS == 1 ? 8 : 0), false, true, block);
            else if (sh.even) CYBQ_GEMV1_LAUNCH(true, 0, false, true, block);
            else CYBQ_GEMV1_LAUNCH(false, 0, false, true, block);
        }
    } else {
        if (k8) CYBQ_GEMV1_LAUNCH(true, (SETS == 1 ? 8 : 0), false, false, block);
        else if (sh.even) CYBQ_GEMV1_LAUNCH(true, 0, false, false, block);
        else CYBQ_GEMV1_LAUNCH(false, 0, false, false, block);
    }
#undef CYBQ_GEMV1_LAUNCH
    return hipGetLastError();
}

template <int BITS, int NS, int MR, bool XBF, bool NORM>
hipError_t launch1_s(const WeightView& w, const void* x, int M, void* y, int ydt, const Epilogue& epi, hipStream_t st)
{
    const Shape1 sh = shape_of(w);
    constexpr int MAXS = max_sets_per_wave(BITS, NS, MR, NORM);
    if (sh.per_wave == 1) return launch1_e<BITS, 1, NS, MR, XBF, NORM>(w, x, M, y, ydt, sh, epi, st);
    if constexpr (MAXS >= 2) {
        if (sh.per_wave == 2) return launch1_e<BITS, 2, NS, MR, XBF, NORM>(w, x, M, y, ydt, sh, epi, st);
    }
    if constexpr (MAXS >= 3) {
        if (sh.per_wave == 3) return launch1_e<BITS, 3, NS, MR, XBF, NORM>(w, x, M, y, ydt, sh, epi, st);
    }
    return hipErrorInvalidValue;         // gemv1_serves() said no
}

template <int BITS, int NS, bool NORM>
hipError_t launch1_x(const WeightView& w, const void* x, int xdt, int M, void* y, int ydt, const Epilogue& epi, hipStream_t st)
{
    if (xdt == kBF16) {
        if (M == 1) return launch1_s<BITS, NS, 1, true, NORM>(w, x, M, y, ydt, epi, st);
        return launch1_s<BITS, NS, 2, true, NORM>(w, x, M, y, ydt, epi, st);
    }
    if (M == 1) return launch1_s<BITS, NS, 1, false, NORM>(w, x, M, y, ydt, epi, st);
    return launch1_s<BITS, NS, 2, false, NORM>(w, x, M, y, ydt, epi, st);
}

template <int BITS, int NS>
hipError_t launch1_m(const WeightView& w, const void* x, int xdt, int M, void* y, int ydt, const Epilogue& epi, hipStream_t st)
{
    if (epi.gamma) return launch1_x<BITS, NS, true>(w, x, xdt, M, y, ydt, epi, st);
    return launch1_x<BITS, NS, false>(w, x, xdt, M, y, ydt, epi, st);
}

}  // namespace

bool gemv1_serves(const WeightView& w, int xdt, int M, const Epilogue& epi)
{
    if (M < 1 || M > 2 || xdt == kF32) return false;
    const int mr = M;
    const int ns = epi.kind == kEpiSwiglu ? 2 : 1;
    const Shape1 sh = shape_of(w);
    if (mr > 1 && ns == 2 && !sh.k8) return false;          // pairs with several rows: split workgroups only
    return sh.per_wave <= max_sets_per_wave(w.bits, ns, mr, epi.gamma != nullptr);
}

hipError_t launch_gemv1(const WeightView& w, const void* x, int xdt, int M, void* y, int ydt, const Epilogue& epi, hipStream_t st)
{
    if (epi.kind == kEpiSwiglu) {
        if (w.bits == 4) return launch1_m<4, 2>(w, x, xdt, M, y, ydt, epi, st);
        return launch1_m<8, 2>(w, x, xdt, M, y, ydt, epi, st);
    }
    if (w.bits == 4) return launch1_m<4, 1>(w, x, xdt, M, y, ydt, epi, st);
    return launch1_m<8, 1>(w, x, xdt, M, y, ydt, epi, st);
}

}  // namespace cybq
