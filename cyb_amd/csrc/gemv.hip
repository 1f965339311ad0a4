// gemv.hip - decode kernel: y[M,N] = x[M,K] * W^T for 1 <= M <= 16.
//
// HBM-bound: every weight byte is read exactly once with 128-bit loads; the
// only other traffic is x (staged once per workgroup into LDS) and y.
//
// Mapping.  One workgroup owns one 16-row strip of W (a contiguous stream in
// the native layout) and splits the strip's K tiles over its waves; tile kt
// goes to wave kt % waves, so neighbouring waves read neighbouring kilobytes.
// A lane's 16 B load is four MFMA B operands (one per scale group), x comes
// out of LDS as the A operand, and v_mfma_f32_16x16x32 does the 32-long dot
// product of one group for 16 columns x 16 batch rows at once.  The per-group
// f16 scale is applied in fp32 on the MFMA result, so the weight operand stays
// an exact small integer and the only rounding is the fp32 accumulation.
// Split-K partials meet in LDS in a fixed order: results are deterministic and
// row m of a batch is bit-identical to the same row run alone.
#include <type_traits>
#include "cybq_device.h"
#include "cybq_internal.h"

namespace cybq {

namespace {

constexpr int XF16 = 0, XBF16 = 1, XF32 = 2;

template <int BITS>
struct TileRegs {
    u32x4_t q[BITS == 4 ? 1 : 2];
    u32x2_t s;
};

template <int BITS>
__device__ __forceinline__ void load_tile(TileRegs<BITS>& t, const WeightView& w, int64_t tile, int lane)
{
    const u32x4_t* qp = tile_q<BITS>(w, tile);
    t.q[0] = __builtin_nontemporal_load(qp + lane);
    if (BITS == 8) t.q[BITS == 8 ? 1 : 0] = __builtin_nontemporal_load(qp + 64 + lane);
    t.s = __builtin_nontemporal_load(tile_s<BITS>(w, tile) + (lane & 15));
}

__device__ __forceinline__ void store_out(void* y, int ydt, int64_t idx, float v)
{
    if (ydt == kF32) reinterpret_cast<float*>(y)[idx] = v;
    else if (ydt == kF16) reinterpret_cast<_Float16*>(y)[idx] = (_Float16)v;
    else reinterpret_cast<uint16_t*>(y)[idx] = f32_to_bf16_bits(v);
}

__device__ __forceinline__ float load_out(const void* p, int dt, int64_t idx)
{
    if (dt == kF32) return reinterpret_cast<const float*>(p)[idx];
    if (dt == kF16) return (float)reinterpret_cast<const _Float16*>(p)[idx];
    return __builtin_bit_cast(float, (uint32_t)reinterpret_cast<const uint16_t*>(p)[idx] << 16);
}

// one finished output element: residual add (fp32, before the single rounding to ydt), store
__device__ __forceinline__ void emit(void* y, int ydt, const Epilogue& epi, int64_t idx, float v)
{
    if (epi.kind == kEpiAdd) v += load_out(epi.residual, ydt, idx);
    store_out(y, ydt, idx, v);
}

// x rows of one K slab -> LDS (row stride ldx 16-bit elements; XF32: a second
// plane of low halves follows the first at plane_elems).  Split in two so that
// the global loads can be issued BEFORE the weight loads: vmcnt retires in
// order, so an x load issued after them could only be waited for together with
// every weight tile, and nothing would overlap the HBM stream.
constexpr int kXChunks = 4;     // 8-element chunks of x a thread carries in registers

template <int XMODE>
struct XRegs {
    u32x4_t v[kXChunks][XMODE == XF32 ? 2 : 1];
};

// ONEROW (M == 1): chunk index = column, no division on the way to the first load.
template <int XMODE, bool ONEROW>
__device__ __forceinline__ void stage_x_load(XRegs<XMODE>& r, const void* x, int M, int K, int k_begin,
                                             int slab_k, int first_chunk, int tid, int nthreads)
{
    const int chunks_per_row = slab_k >> 3;
    const int total = M * chunks_per_row;
#pragma unroll
    for (int c = 0; c < kXChunks; c++) {
        const int idx = first_chunk + tid + c * nthreads;
        const int row = ONEROW ? 0 : idx / chunks_per_row;
        const int k = k_begin + ((idx - row * chunks_per_row) << 3);
        const bool live = idx < total && k < K;
        if (XMODE != XF32) {
            u32x4_t v = {0u, 0u, 0u, 0u};
            if (live) v = *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const uint16_t*>(x) + (int64_t)row * K + k);
            r.v[c][0] = v;
        } else {
            u32x4_t v0 = {0u, 0u, 0u, 0u}, v1 = v0;
            if (live) {
                const u32x4_t* p = reinterpret_cast<const u32x4_t*>(reinterpret_cast<const float*>(x) + (int64_t)row * K + k);
                v0 = p[0];
                v1 = p[1];
            }
            r.v[c][0] = v0;
            r.v[c][XMODE == XF32 ? 1 : 0] = v1;
        }
    }
}

template <int XMODE, bool ONEROW>
__device__ __forceinline__ void stage_x_store(const XRegs<XMODE>& r, uint16_t* xs, int M, int slab_k, int ldx,
                                              int plane_elems, int first_chunk, int tid, int nthreads)
{
    const int chunks_per_row = slab_k >> 3;
    const int total = M * chunks_per_row;
#pragma unroll
    for (int c = 0; c < kXChunks; c++) {
        const int idx = first_chunk + tid + c * nthreads;
        if (idx >= total) continue;
        const int row = ONEROW ? 0 : idx / chunks_per_row;
        const int col = (idx - row * chunks_per_row) << 3;
        u32x4_t* dst = reinterpret_cast<u32x4_t*>(xs + row * ldx + col);
        if (XMODE != XF32) {
            *dst = r.v[c][0];
        } else {
            Frag16 hi, lo;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float f = __builtin_bit_cast(float, (uint32_t)r.v[c][i >> 2][i & 3]);
                _Float16 h = (_Float16)f;
                hi.h[i] = h;
                lo.h[i] = (_Float16)(f - (float)h);
            }
            *dst = hi.u;
            *reinterpret_cast<u32x4_t*>(xs + plane_elems + row * ldx + col) = lo.u;
        }
    }
}

// chunks beyond the first kXChunks per thread (large M * slab): plain loop
template <int XMODE, bool ONEROW>
__device__ __forceinline__ void stage_x_rest(uint16_t* xs, const void* x, int M, int K, int k_begin, int slab_k,
                                             int ldx, int plane_elems, int tid, int nthreads)
{
    const int total = M * (slab_k >> 3);
    for (int first = kXChunks * nthreads; first < total; first += kXChunks * nthreads) {
        XRegs<XMODE> r;
        stage_x_load<XMODE, ONEROW>(r, x, M, K, k_begin, slab_k, first, tid, nthreads);
        stage_x_store<XMODE, ONEROW>(r, xs, M, slab_k, ldx, plane_elems, first, tid, nthreads);
    }
}

// One tile = 4 scale groups.  tile_issue reads the four x operands from LDS,
// unpacks the four weight operands and issues the four MFMAs back to back into
// separate result registers; tile_accum folds the group scales in afterwards.
// Callers run tile_accum one tile late, so the MFMA latency is covered by the
// next tile's unpack instead of by wait states.
template <int BITS, int XMODE>
__device__ __forceinline__ void tile_issue(const TileRegs<BITS>& t, const uint16_t* xrow, int plane_elems,
                                           uint32_t magic, float4_t d[4])
{
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    Frag16 a[4], al[4], b[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        a[j].u = *reinterpret_cast<const u32x4_t*>(xrow + j * 32);
        if (XMODE == XF32) al[j].u = *reinterpret_cast<const u32x4_t*>(xrow + plane_elems + j * 32);
    }
#pragma unroll
    for (int j = 0; j < 4; j++) {
        uint32_t bw[4];
        if (BITS == 4 && XMODE == XBF16) {
            unpack_q4_bf16_biased(t.q[0][2 * (j >> 1)], t.q[0][2 * (j >> 1) + 1], j & 1, magic, bw);
        } else if (XMODE == XBF16) {
            unpack_q8_bf16_biased(t.q[j >> 1][(j & 1) * 2], t.q[j >> 1][(j & 1) * 2 + 1], bw);
        } else {
            if (BITS == 4) unpack_q4_f16(t.q[0][2 * (j >> 1)], t.q[0][2 * (j >> 1) + 1], j & 1, magic, bw);
            else unpack_q8_f16(t.q[j >> 1][(j & 1) * 2], t.q[j >> 1][(j & 1) * 2 + 1], bw);
        }
        b[j].u = (u32x4_t){bw[0], bw[1], bw[2], bw[3]};
    }
    Frag16 off;
    const uint32_t offw = BITS == 4 ? kBf16Neg136x2 : kBf16Neg128x2;
    off.u = (u32x4_t){offw, offw, offw, offw};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        if (XMODE == XBF16) {
            d[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j].b, b[j].b, zero, 0, 0, 0);
            d[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j].b, off.b, d[j], 0, 0, 0);
        } else {
            d[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j].h, b[j].h, zero, 0, 0, 0);
            if (XMODE == XF32) d[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al[j].h, b[j].h, d[j], 0, 0, 0);
        }
    }
}

template <int RMAX>
__device__ __forceinline__ void tile_accum(u32x2_t s, const float4_t d[4], float acc[RMAX])
{
#pragma unroll
    for (int j = 0; j < 4; j++) {
        uint32_t sb = (j & 1) ? (s[j >> 1] >> 16) : (s[j >> 1] & 0xffffu);
        float sc = f16_bits_to_f32(sb);
#pragma unroll
        for (int r = 0; r < RMAX; r++) acc[r] = __builtin_fmaf(sc, d[j][r], acc[r]);
    }
}

// The hot region is kept free of branches on purpose: vmcnt retires in order
// and the compiler can only count outstanding loads along straight-line code;
// a conditional load forces it to wait for everything (vmcnt(0)) and nothing
// overlaps.  Tiles past the end of the slab are therefore clamped to the last
// valid tile (a cache hit) and their scale is forced to zero.
template <int BITS, int U>
__device__ __forceinline__ void load_batch(TileRegs<BITS> (&buf)[U], const WeightView& w, int64_t base, int i0,
                                           int nwaves, int limit, int lane)
{
#pragma unroll
    for (int u = 0; u < U; u++) load_tile<BITS>(buf[u], w, base + min(i0 + u * nwaves, limit - 1), lane);
}

// Runs a batch of U tiles (tile index i0 + u * nwaves, contributing while < limit).
template <int BITS, int XMODE, int RMAX, int U>
__device__ __forceinline__ void compute_batch(const TileRegs<BITS> (&buf)[U], int i0, int nwaves, int limit,
                                              const uint16_t* xbase, int plane_elems, uint32_t magic,
                                              float acc[RMAX])
{
    float4_t dprev[4];
    u32x2_t sprev = {0u, 0u};
#pragma unroll
    for (int j = 0; j < 4; j++) dprev[j] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int i = i0 + u * nwaves;
        const bool valid = i < limit;
        float4_t d[4];
        tile_issue<BITS, XMODE>(buf[u], xbase + min(i, limit - 1) * kTileK, plane_elems, magic, d);
        u32x2_t sc = buf[u].s;
        sc[0] = valid ? sc[0] : 0u;
        sc[1] = valid ? sc[1] : 0u;
        tile_accum<RMAX>(sprev, dprev, acc);
#pragma unroll
        for (int j = 0; j < 4; j++) dprev[j] = d[j];
        sprev = sc;
    }
    tile_accum<RMAX>(sprev, dprev, acc);
}

// Sum of the waves' partial sums red[k * stride], k = 0 .. nwaves-1, added in wave
// order.  The reads go out eight at a time: one LDS round trip per eight waves
// instead of one per wave.  (Slots past nwaves add +0, which changes nothing: a sum
// that starts from +0 is never -0.)
__device__ __forceinline__ float sum_partials(const float* red, int nwaves, int stride)
{
    float v = 0.f;
    for (int k0 = 0; k0 < nwaves; k0 += 8) {
        float t[8];
#pragma unroll
        for (int i = 0; i < 8; i++) t[i] = red[min(k0 + i, nwaves - 1) * stride];
#pragma unroll
        for (int i = 0; i < 8; i++) v += (k0 + i < nwaves) ? t[i] : 0.f;
    }
    return v;
}

// ---- RMSNorm folded into the staged x (LDS kernel) ------------------------------
// gamma[k0 .. k0+8) as fp32 (k0 a multiple of 8; gamma is 16-byte aligned at such k for f32 and 16-bit types)
__device__ __forceinline__ void load_gamma8(const void* g, int gdt, int k0, float out[8])
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

// eight staged values (one 16 B piece of a row) as fp32, and back
template <int XMODE>
__device__ __forceinline__ void staged_piece(const uint16_t* row, int plane_elems, int c, float out[8])
{
    const u32x4_t v = reinterpret_cast<const u32x4_t*>(row)[c];
    u32x4_t lo = {0u, 0u, 0u, 0u};
    if (XMODE == XF32) lo = reinterpret_cast<const u32x4_t*>(row + plane_elems)[c];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        if (XMODE == XBF16) {
            out[2 * i] = __builtin_bit_cast(float, v[i] << 16);
            out[2 * i + 1] = __builtin_bit_cast(float, v[i] & 0xffff0000u);
        } else {
            const half2_t h = as_h2(v[i]);
            out[2 * i] = (float)h.x;
            out[2 * i + 1] = (float)h.y;
            if (XMODE == XF32) {
                const half2_t l = as_h2(lo[i]);
                out[2 * i] += (float)l.x;
                out[2 * i + 1] += (float)l.y;
            }
        }
    }
}

template <int XMODE>
__device__ __forceinline__ void store_staged_piece(uint16_t* row, int plane_elems, int c, const float in[8])
{
    u32x4_t v, lo;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        if (XMODE == XBF16) {
            v[i] = pack_bf16x2(in[2 * i], in[2 * i + 1]);
        } else {
            const half2_t h = {(_Float16)in[2 * i], (_Float16)in[2 * i + 1]};
            v[i] = as_u32(h);
            if (XMODE == XF32) {
                const half2_t l = {(_Float16)(in[2 * i] - (float)h.x), (_Float16)(in[2 * i + 1] - (float)h.y)};
                lo[i] = as_u32(l);
            }
        }
    }
    reinterpret_cast<u32x4_t*>(row)[c] = v;
    if (XMODE == XF32) reinterpret_cast<u32x4_t*>(row + plane_elems)[c] = lo;
}

// One staged K slab: adds this slab's sum of squares of every row to ssq[row] and replaces
// x by x * gamma, in 16 B pieces (ldx, slab_k and K are multiples of 8).  Every thread
// takes pieces tid, tid + threads, ... of each row; lanes meet in a fixed butterfly, waves
// through `part` in wave order: the order of the additions never changes.  Two barriers inside.
// gamma of the first two pieces a thread will scale (pieces tid and tid + threads of every row),
// requested together with x so that it is there when the slab is staged
struct GammaPre {
    float g[2][8];
};
__device__ __forceinline__ void prefetch_gamma(GammaPre& gp, const Epilogue& epi, int slab_k, int k_begin, int K, int tid,
                                               int nthreads)
{
    const int pieces = max(min(slab_k, K - k_begin) >> 3, 1);
    load_gamma8(epi.gamma, epi.gamma_dt, k_begin + min(tid, pieces - 1) * 8, gp.g[0]);
    load_gamma8(epi.gamma, epi.gamma_dt, k_begin + min(tid + nthreads, pieces - 1) * 8, gp.g[1]);
}

template <int XMODE>
__device__ __forceinline__ void norm_staged_slab(uint16_t* xs, int M, int slab_k, int k_begin, int K, int ldx,
                                                 int plane_elems, const Epilogue& epi, const GammaPre& gp, float* ssq,
                                                 float* part, int tid, int nthreads)
{
    const int lane = tid & 63, wv = tid >> 6, nw = nthreads >> 6;
    const int pieces = min(slab_k, K - k_begin) >> 3;
    for (int m = 0; m < M; m++) {
        const uint16_t* row = xs + m * ldx;
        float a = 0.f;
        for (int c = tid; c < pieces; c += nthreads) {
            float v[8];
            staged_piece<XMODE>(row, plane_elems, c, v);
#pragma unroll
            for (int i = 0; i < 8; i++) a = fmaf(v[i], v[i], a);
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) a += __shfl_xor(a, off, 64);
        if (lane == 0) part[m * 16 + wv] = a;
    }
    __syncthreads();
    if (tid < M) {
        float t = ssq[tid];
        for (int k = 0; k < nw; k++) t += part[tid * 16 + k];
        ssq[tid] = t;
    }
    for (int m = 0; m < M; m++) {
        uint16_t* row = xs + m * ldx;
        int it = 0;
        for (int c = tid; c < pieces; c += nthreads, it++) {
            float v[8], g[8];
            staged_piece<XMODE>(row, plane_elems, c, v);
            if (it < 2) {
#pragma unroll
                for (int i = 0; i < 8; i++) g[i] = it == 0 ? gp.g[0][i] : gp.g[1][i];
            } else {
                load_gamma8(epi.gamma, epi.gamma_dt, k_begin + c * 8, g);
            }
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] *= g[i];
            store_staged_piece<XMODE>(row, plane_elems, c, v);
        }
    }
    __syncthreads();
}

// U = tiles a wave keeps in flight per batch.  ONESHOT: the wave's whole share
// of the strip is at most U tiles, all requested before anything else happens
// (one register set); otherwise two batches are live and ping-pong.
// NORM: RMSNorm folded into the staged x (only instantiated for the streaming variant U = 2).
template <int BITS, int XMODE, int RMAX, int U, bool ONESHOT, int PAIR, bool NORM>
// (leading scalar arguments, in the order of their first use: they arrive in registers at wave start)
// (the launch's thread count travels with them: the launch geometry is not among what is preloaded)
__global__ __launch_bounds__(1024) void gemv_kernel(const uint8_t* __restrict__ wbase, const void* __restrict__ x, int KT, int K, int M,
                            int nthreads, int slab_tiles, int ldx, int red_offset, void* __restrict__ y, int N, int ydt, int NT,
                            Epilogue epi)
{
    const WeightView w = {wbase, N, K, NT, KT, BITS};
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint16_t* xs = reinterpret_cast<uint16_t*>(smem);
    const uint32_t magic = (BITS == 4 && XMODE == XBF16) ? q4_magic_vgpr_bf16() : q4_magic_vgpr();

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    // SwiGLU: the workgroup owns a gate strip and its up strip; the first half of its
    // waves splits the K tiles of one, the second half those of the other, x is staged once
    // (PAIR = 2)
    const int wv_all = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = (nthreads >> 6) / PAIR;                 // waves per strip
    const int sub = (PAIR == 2 && wv_all >= nwaves) ? 1 : 0;
    const int wv = wv_all - sub * nwaves;
    const int nt = blockIdx.x * PAIR + sub;
    const int mrow = min(lane & 15, M - 1);
    const int oct = lane >> 4;
    const int plane_elems = M * ldx;
    const int64_t strip = (int64_t)nt * w.KT;
    const int stride = nwaves * U;

    float acc[RMAX];
#pragma unroll
    for (int r = 0; r < RMAX; r++) acc[r] = 0.f;

    // folded RMSNorm: per-row sums of squares live behind the partial sums
    float* ssq = reinterpret_cast<float*>(smem + red_offset) + PAIR * nwaves * RMAX * 64;
    float* ssq_part = ssq + 16;                      // [row][wave] partial sums of squares
    if (NORM && tid < 16) ssq[tid] = 0.f;            // (ordered before its first use by the staging barrier)

    if (ONESHOT) {
        TileRegs<BITS> buf[U];
        XRegs<XMODE> xr;
        stage_x_rest<XMODE, RMAX == 1>(xs, x, M, w.K, 0, w.KT * kTileK, ldx, plane_elems, tid, nthreads);
        stage_x_load<XMODE, RMAX == 1>(xr, x, M, w.K, 0, w.KT * kTileK, 0, tid, nthreads);
        GammaPre gp;
        if (NORM) prefetch_gamma(gp, epi, w.KT * kTileK, 0, w.K, tid, nthreads);
        load_batch<BITS, U>(buf, w, strip, wv, nwaves, w.KT, lane);
        stage_x_store<XMODE, RMAX == 1>(xr, xs, M, w.KT * kTileK, ldx, plane_elems, 0, tid, nthreads);
        __syncthreads();
        if (NORM) norm_staged_slab<XMODE>(xs, M, w.KT * kTileK, 0, w.K, ldx, plane_elems, epi, gp, ssq, ssq_part, tid, nthreads);
        const uint16_t* xbase = xs + mrow * ldx + oct * 8;
        compute_batch<BITS, XMODE, RMAX, U>(buf, wv, nwaves, w.KT, xbase, plane_elems, magic, acc);
    } else {
        TileRegs<BITS> bufA[U], bufB[U];
        for (int slab0 = 0; slab0 < w.KT; slab0 += slab_tiles) {
            const int st = min(slab_tiles, w.KT - slab0);
            const int64_t base = strip + slab0;
            if (slab0 > 0) __syncthreads();          // every wave is done with the previous slab of x
            // x loads first, then the first weight batch of this slab: the HBM
            // latency of the weights overlaps the staging and the barrier
            XRegs<XMODE> xr;
            stage_x_rest<XMODE, RMAX == 1>(xs, x, M, w.K, slab0 * kTileK, st * kTileK, ldx, plane_elems, tid, nthreads);
            stage_x_load<XMODE, RMAX == 1>(xr, x, M, w.K, slab0 * kTileK, st * kTileK, 0, tid, nthreads);
            GammaPre gp;
            if (NORM) prefetch_gamma(gp, epi, st * kTileK, slab0 * kTileK, w.K, tid, nthreads);
            load_batch<BITS, U>(bufA, w, base, wv, nwaves, st, lane);
            stage_x_store<XMODE, RMAX == 1>(xr, xs, M, st * kTileK, ldx, plane_elems, 0, tid, nthreads);
            __syncthreads();
            if (NORM)
                norm_staged_slab<XMODE>(xs, M, st * kTileK, slab0 * kTileK, w.K, ldx, plane_elems, epi, gp, ssq, ssq_part, tid, nthreads);

            const uint16_t* xbase = xs + mrow * ldx + oct * 8;
            for (int r0 = 0; r0 < st; r0 += 2 * stride) {
                // bufA holds batch r0; fetch batch r0 + stride into bufB, and so on.  A batch that
                // starts past the end of the slab is not requested at all (its loads would only
                // be cache hits, but they would still queue in the address path).  Every arm is
                // straight-line code of its own, so the load counters stay exact.
                const int i0 = r0 + wv;
                if (r0 + stride < st) {
                    load_batch<BITS, U>(bufB, w, base, i0 + stride, nwaves, st, lane);
                    compute_batch<BITS, XMODE, RMAX, U>(bufA, i0, nwaves, st, xbase, plane_elems, magic, acc);
                    if (r0 + 2 * stride < st) {
                        load_batch<BITS, U>(bufA, w, base, i0 + 2 * stride, nwaves, st, lane);
                        compute_batch<BITS, XMODE, RMAX, U>(bufB, i0 + stride, nwaves, st, xbase, plane_elems, magic, acc);
                    } else {
                        compute_batch<BITS, XMODE, RMAX, U>(bufB, i0 + stride, nwaves, st, xbase, plane_elems, magic, acc);
                    }
                } else {
                    compute_batch<BITS, XMODE, RMAX, U>(bufA, i0, nwaves, st, xbase, plane_elems, magic, acc);
                }
            }
        }
    }

    // split-K partials -> LDS (their own area behind x: no barrier to wait for the last
    // reader of x), summed in wave order; wave r finishes output register r
    float* red = reinterpret_cast<float*>(smem + red_offset);
#pragma unroll
    for (int r = 0; r < RMAX; r++) red[(wv_all * RMAX + r) * 64 + lane] = acc[r];
    __syncthreads();
    if (PAIR == 2) {
        const int n_out = w.N >> 1;
        const int n = blockIdx.x * 16 + (lane & 15);
        for (int r = wv_all; r < RMAX; r += 2 * nwaves) {
            float g = sum_partials(red + r * 64 + lane, nwaves, RMAX * 64);
            float u = sum_partials(red + (nwaves * RMAX + r) * 64 + lane, nwaves, RMAX * 64);
            const int m = 4 * oct + r;
            if (NORM) {
                const float rstd = 1.0f / sqrtf(ssq[min(m, M - 1)] / (float)w.K + epi.eps);
                g *= rstd;
                u *= rstd;
            }
            if (m < M && n < n_out) store_out(y, ydt, (int64_t)m * n_out + n, silu_mul(g, u));
        }
        return;
    }
    const int n = nt * 16 + (lane & 15);
    for (int r = wv; r < RMAX; r += nwaves) {
        float v = sum_partials(red + r * 64 + lane, nwaves, RMAX * 64);
        const int m = 4 * oct + r;
        if (NORM) v *= 1.0f / sqrtf(ssq[min(m, M - 1)] / (float)w.K + epi.eps);
        if (m < M && n < w.N) emit(y, ydt, epi, (int64_t)m * w.N + n, v);
    }
}

// ---------------------------------------------------------------------------
// Batch rows 3..16: x operands live in REGISTERS and are reused across strips.
//
// With more than a few batch rows the LDS kernel above spends its time moving
// x: every 16-row strip's workgroup stages all M rows of x (128 KB at M = 16,
// K = 4096, against 37 KB of weights).  Here a workgroup owns NS consecutive
// strips; each wave loads the x of ITS K tiles once (coalesced, then moved across
// lanes into A-operand order: lane = batch row l%16, k octet l/16; no LDS
// staging, no barrier), requests the weight tiles two strips ahead and walks over
// the strips with the same operands.  Tile kt belongs to wave kt % waves and
// partials are summed in wave order: deterministic, and a row's bits do not depend
// on the batch it is part of (within this kernel; the LDS kernel may split K over
// a different number of waves).
template <int BITS, int XMODE>
__device__ __forceinline__ void tile_operands(const TileRegs<BITS>& t, uint32_t magic, Frag16 (&b)[4])
{
#pragma unroll
    for (int j = 0; j < 4; j++) {
        uint32_t bw[4];
        if (BITS == 4 && XMODE == XBF16) {
            unpack_q4_bf16_biased(t.q[0][2 * (j >> 1)], t.q[0][2 * (j >> 1) + 1], j & 1, magic, bw);
        } else if (XMODE == XBF16) {
            unpack_q8_bf16_biased(t.q[j >> 1][(j & 1) * 2], t.q[j >> 1][(j & 1) * 2 + 1], bw);
        } else {
            if (BITS == 4) unpack_q4_f16(t.q[0][2 * (j >> 1)], t.q[0][2 * (j >> 1) + 1], j & 1, magic, bw);
            else unpack_q8_f16(t.q[j >> 1][(j & 1) * 2], t.q[j >> 1][(j & 1) * 2 + 1], bw);
        }
        b[j].u = (u32x4_t){bw[0], bw[1], bw[2], bw[3]};
    }
}

template <int BITS, int XMODE>
__device__ __forceinline__ void tile_multiply(const Frag16 (&a)[4], const Frag16 (&b)[4], float4_t d[4])
{
    const float4_t zero = {0.f, 0.f, 0.f, 0.f};
    Frag16 off;
    const uint32_t offw = BITS == 4 ? kBf16Neg136x2 : kBf16Neg128x2;
    off.u = (u32x4_t){offw, offw, offw, offw};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        if (XMODE == XBF16) {
            d[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j].b, b[j].b, zero, 0, 0, 0);
            d[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j].b, off.b, d[j], 0, 0, 0);
        } else d[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j].h, b[j].h, zero, 0, 0, 0);
    }
}

template <int BITS, int XMODE>
__device__ __forceinline__ void tile_issue_regs(const TileRegs<BITS>& t, const Frag16 (&a)[4], uint32_t magic,
                                                float4_t d[4])
{
    Frag16 b[4];
    tile_operands<BITS, XMODE>(t, magic, b);
    tile_multiply<BITS, XMODE>(a, b, d);
}

// NORM: RMSNorm folded into the activation load (epi.gamma / epi.eps).  A lane multiplies the 16 B
// piece of x it loaded (eight neighbouring k of one row) by gamma and adds up its squares while the
// piece is still as loaded: every element of the batch is touched once per workgroup, where the
// operand fragments made from the pieces repeat a batch of four rows four times.  Rows meet
// across lanes and waves in the final exchange.
// GH: x and gamma are both f16 - gamma sits in LDS as loaded and the product is one packed f16
// multiply per pair (the product of two f16 is exact in fp32, so its single rounding to f16 is the
// rounding the fp32 form makes); otherwise gamma is fp32 in LDS and the pair goes through fp32.
// v as the lanes named by a DPP control see it (quad permutations, mirrors within a row of 16)
template <int CTRL>
__device__ __forceinline__ float lane_cross(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// (the LDS reads of a tile's pieces are issued together, ahead of the arithmetic)
struct GammaPiece {
    u32x4_t lo, hi;           // 8 x fp32, or (GH) 8 x f16 in lo
};

template <bool GH>
__device__ __forceinline__ GammaPiece gamma_piece(const void* gamma_lds, int k)
{
    GammaPiece g;
    if constexpr (GH) {
        g.lo = *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const uint16_t*>(gamma_lds) + k);
        g.hi = g.lo;
    } else {
        g.lo = reinterpret_cast<const u32x4_t*>(reinterpret_cast<const float*>(gamma_lds) + k)[0];
        g.hi = reinterpret_cast<const u32x4_t*>(reinterpret_cast<const float*>(gamma_lds) + k)[1];
    }
    return g;
}

template <int XMODE, bool GH>
__device__ __forceinline__ void norm_piece(u32x4_t& v, const GammaPiece& gp, bool counts, float& ssq)
{
    float sq = ssq;
    if constexpr (GH) {
        const u32x4_t g = gp.lo;
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const half2_t h = as_h2(v[p]);
            sq = __builtin_amdgcn_fdot2(h, h, sq, false);
            v[p] = as_u32(h * as_h2(g[p]));
        }
    } else {
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const uint32_t ua = p < 2 ? gp.lo[2 * p] : gp.hi[2 * p - 4], ub = p < 2 ? gp.lo[2 * p + 1] : gp.hi[2 * p - 3];
            const float ga = __builtin_bit_cast(float, ua), gb = __builtin_bit_cast(float, ub);
            if (XMODE == XBF16) {
                const float v0 = __builtin_bit_cast(float, v[p] << 16);
                const float v1 = __builtin_bit_cast(float, v[p] & 0xffff0000u);
                sq = fmaf(v1, v1, fmaf(v0, v0, sq));
                v[p] = pack_bf16x2(v0 * ga, v1 * gb);
            } else {
                const half2_t h = as_h2(v[p]);
                sq = __builtin_amdgcn_fdot2(h, h, sq, false);
                const half2_t o = {(_Float16)((float)h.x * ga), (_Float16)((float)h.y * gb)};
                v[p] = as_u32(o);
            }
        }
    }
    ssq = counts ? sq : ssq;
}

// MB: blocks of 16 batch rows (2 = 17..32 rows: every unpacked weight operand is multiplied with
// two activation operands, the weights still stream once).
// gamma / gamma_dt (NORM) sit ahead of y in the argument list: everything the first loads need is
// then in the argument registers the hardware fills before the kernel starts.
// SUB (f16 activations, Q4, decode mode STREAM): the weights enter the MFMA as the f16 subnormals
// 4u * 2^-24 / 64u * 2^-24 (six vector instructions per eight weights instead of nine), the bias comes off
// through the MFMA's C operand like with bf16 activations, 1/16 for the odd groups rides on their scale
// and 2^22 on the final sums.
// KS: K is split over `splits` workgroups per strip group (few strips and a long K: with one workgroup per
// strip every CU pulls all of x out of the L2, M x K x 2 bytes against its 37 KB x strips of weights).  Workgroup
// (group, split) walks the K tiles [split * kt_per_split, ...) of the group's NS strips and leaves its sums in
// its slab of `slabs`; a ticket per group tells the workgroup that arrives last, which adds the slabs in split
// order - a fixed order whoever arrives when - and writes y.  Slabs and ticket travel past the caches (stores
// and loads at system scope, waited for before the ticket is taken): nothing is flushed, nothing invalidated.
// The ticket is left at zero again for the next launch; launches that share `slabs` must not overlap.
template <int BITS, int XMODE, int TS, int NS, bool NORM, int XR, int MB = 1, bool SUB = false, bool KS = false>
// (waves_per_eu: the scheduler would otherwise trade the up-front loads for occupancy)
__global__ __launch_bounds__((TS <= 2 && MB == 1 && !NORM) ? 1024 : 512)
__attribute__((amdgpu_waves_per_eu(2, (TS <= 2 && MB == 1 && !NORM) ? 4 : 2)))
void gemv_rows_kernel(const uint8_t* __restrict__ wbase, const uint16_t* __restrict__ x, const void* __restrict__ gamma, int KT_, int K,
                      int NT, int M, int nwaves, int gamma_dt, int N, void* __restrict__ y, int ydt, Epilogue epi, int splits,
                      int kt_per_split, float* __restrict__ slabs, unsigned* __restrict__ tickets)
{
    static_assert(!KS || !NORM, "the K split has no folded-norm form");
    const WeightView w = {wbase, N, K, NT, KT_, BITS};
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t magic = (BITS == 4 && XMODE == XBF16) ? q4_magic_vgpr_bf16() : q4_magic_vgpr();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int oct = lane >> 4;
    int group = blockIdx.x, split = 0, kt_lo = 0;
    int KT = w.KT;                                   // K tiles this workgroup walks: [kt_lo, kt_lo + KT)
    if constexpr (KS) {
        group = (int)blockIdx.x / splits;
        split = (int)blockIdx.x - group * splits;
        kt_lo = split * kt_per_split;
        KT = min(kt_per_split, w.KT - kt_lo);
    }
    const int strip0 = group * NS;
    // x is read the way memory likes it - one load instruction covers XR rows (the batch rounded
    // up to 4, 8 or 16) x P = 64 / XR neighbouring 16 B pieces, lane l takes piece l % P of row
    // l / P - and then moved across lanes into MFMA A-operand order (lane l: row l%16, k octet
    // l/16).  Reading in operand order directly costs 64 separate accesses per load instead of
    // 16; and the address path takes 16 cycles per load whatever the lanes ask for, so a batch of
    // four rows gets a whole tile (128 k) with one load where sixteen rows need four.
    constexpr int P = 64 / XR;                  // 16 B pieces per row and load
    constexpr int L = 16 / P;                   // loads per tile: 1, 2, 4
    constexpr int GPL = 4 / L;                  // scale groups per load
    static_assert(MB == 1 || (XR == 16 && !NORM), "two row blocks: full loads, no folded norm");
    const uint16_t* xrow = x + (int64_t)min(lane / P, M - 1) * w.K + (lane % P) * 8;
    const int64_t xblock = MB > 1 ? (int64_t)(min(16 + lane / P, M - 1) - min(lane / P, M - 1)) * w.K : 0;     // to my row of the second block
    const int klast = w.K - 8 - (lane % P) * 8;          // last start at which this lane's piece is inside the row
    const int from_lane = ((((lane & 15) & (XR - 1)) * P) | oct) << 2;       // byte address for ds_bpermute (+ 16 per group)
    // NORM: each wave keeps the gamma of the K tiles it is working on in an LDS area of its own,
    // behind the exchange areas
    uint8_t* gamma_lds = smem + ((size_t)NS * MB * nwaves * 4 * 64 + 8 * 16 + (size_t)wv * TS * kTileK) * sizeof(float);
    const bool gamma_h = NORM && XMODE == XF16 && gamma_dt == kF16;
    const bool gamma_f32 = NORM && gamma_dt == kF32;
    const int g_count = gamma_f32 ? 4 : 8;               // values of a tile's gamma a lane loads,
    const int g_first = (lane & (gamma_f32 ? 31 : 15)) * g_count;       // the first of them,
    const int g_shift = gamma_f32 ? 2 : 1;               // log2 of their size

    float acc[NS][MB][4];
#pragma unroll
    for (int s = 0; s < NS; s++)
#pragma unroll
        for (int b = 0; b < MB; b++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[s][b][r] = 0.f;
    float ssq = 0.f;          // NORM: squares of the x values this lane loaded (row lane / P)

    int64_t sbase[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) sbase[s] = (int64_t)min(strip0 + s, w.NT - 1) * w.KT;

    for (int slab0 = 0; slab0 < KT; slab0 += nwaves * TS) {
        // my K tiles of this slab and their x operands (clamped past the end; such tiles get scale 0)
        int kt[TS];
        bool valid[TS];
        Frag16 a[MB][TS][4];
        u32x4_t graw[NORM ? TS : 1];        // NORM: gamma of my tiles, 8 values in each of 16 lanes (4 in each of 32: fp32)
#pragma unroll
        for (int u = 0; u < TS; u++) {
            const int t = slab0 + wv + nwaves * u;
            valid[u] = t < KT;
            kt[u] = kt_lo + min(t, KT - 1);
            if (NORM)
                graw[u] = *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const uint8_t*>(gamma) +
                                                            ((size_t)min(kt[u] * kTileK + g_first, w.K - g_count) << g_shift));
#pragma unroll
            for (int h = 0; h < L; h++) {
                // (past the end of K: any x inside the row will do, the padded weights are zero)
                const int k0 = kt[u] * kTileK + h * (GPL * 32);
                if (XR == 16) {
#pragma unroll
                    for (int b = 0; b < MB; b++)
                        a[b][u][h].u = *reinterpret_cast<const u32x4_t*>(xrow + b * xblock + min(k0, w.K - 32));
                } else a[0][u][h].u = *reinterpret_cast<const u32x4_t*>(xrow + min(k0, klast));
            }
        }
        // The memory pipeline takes requests at its own pace: a wave that asks for all its
        // tiles first sits in the issue queue for microseconds and only then starts on
        // its arithmetic.  So the strips are walked two requests ahead: strip s+2 is
        // requested, then strip s (whose tiles were requested two steps ago) is
        // multiplied while the others are on their way.
        // bf16 activations with two to four strips: the weights enter the bf16 MFMA as 128 + u (256 + u for
        // Q8) and one more MFMA of the activations against a constant operand takes the bias off.  That
        // second product does not depend on the strip, so the tiles are walked K tile by K tile with all
        // strips of a tile behind one bias product (its result is the C operand of their MFMAs):
        // 4 + 4 NS instead of 8 NS MFMAs per tile.  Each strip still sums its tiles in the same order.
        constexpr bool BY_TILE = (XMODE == XBF16 || SUB) && BITS == 4 && NS >= 2 && NS <= 4 && (TS == 4 || MB == 2);       // (the others would spill)
        static_assert(!SUB || (BY_TILE && XMODE == XF16 && !NORM), "subnormal operands: f16 activations, walked by tile");
        constexpr int WU = NS == 4 ? (TS < 2 ? TS : 2) : TS;       // BY_TILE: K tiles requested ahead (about eight weight tiles)
        TileRegs<BITS> buf[NS][TS];
        constexpr int AHEAD = NS < 2 ? NS : 2;
        if constexpr (BY_TILE) {
#pragma unroll
            for (int u = 0; u < WU; u++)
#pragma unroll
                for (int s = 0; s < NS; s++) load_tile<BITS>(buf[s][u], w, sbase[s] + kt[u], lane);
        } else {
#pragma unroll
            for (int s = 0; s < AHEAD; s++)
#pragma unroll
                for (int u = 0; u < TS; u++) load_tile<BITS>(buf[s][u], w, sbase[s] + kt[u], lane);
        }
        if (NORM) {
            // my tiles' gamma -> my LDS area (16 or 32 lanes hold a tile's 128 values; fp32, or as loaded
            // when x and gamma are both f16), read back below piece by piece: no other wave is involved
            if (gamma_h) {
                if (lane < 16) {
#pragma unroll
                    for (int u = 0; u < TS; u++) reinterpret_cast<u32x4_t*>(gamma_lds)[u * 16 + lane] = graw[u];
                }
            } else if (gamma_f32) {
                if (lane < 32) {
#pragma unroll
                    for (int u = 0; u < TS; u++) reinterpret_cast<u32x4_t*>(gamma_lds)[u * 32 + lane] = graw[u];
                }
            } else if (lane < 16) {
                const bool gh = gamma_dt == kF16;
#pragma unroll
                for (int u = 0; u < TS; u++) {
                    float g[8];
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const half2_t h = as_h2(graw[u][i]);
                        g[2 * i] = gh ? (float)h.x : __builtin_bit_cast(float, graw[u][i] << 16);
                        g[2 * i + 1] = gh ? (float)h.y : __builtin_bit_cast(float, graw[u][i] & 0xffff0000u);
                    }
                    reinterpret_cast<float4_t*>(gamma_lds)[u * 32 + 2 * lane] = (float4_t){g[0], g[1], g[2], g[3]};
                    reinterpret_cast<float4_t*>(gamma_lds)[u * 32 + 2 * lane + 1] = (float4_t){g[4], g[5], g[6], g[7]};
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            auto norm_all = [&](auto packed) {
                constexpr bool GH = decltype(packed)::value;
#pragma unroll
                for (int u = 0; u < TS; u++) {
                    GammaPiece g[L];
                    bool counts[L];
#pragma unroll
                    for (int h = 0; h < L; h++) {
                        const int k0 = kt[u] * kTileK + h * (GPL * 32);
                        const int kp = k0 + (lane % P) * 8;             // my piece (one past K repeats one inside: not counted)
                        const int kk = (XR == 16 ? min(k0, w.K - 32) + (lane % P) * 8 : min(kp, w.K - 8)) - kt[u] * kTileK + u * kTileK;
                        g[h] = gamma_piece<GH>(gamma_lds, kk);
                        counts[h] = valid[u] && kp < w.K;
                    }
#pragma unroll
                    for (int h = 0; h < L; h++) norm_piece<XMODE, GH>(a[0][u][h].u, g[h], counts[h], ssq);
                }
            };
            if constexpr (XMODE == XF16) {
                if (gamma_h) norm_all(std::true_type{});
                else norm_all(std::false_type{});
            } else norm_all(std::false_type{});
        }
#pragma unroll
        for (int b = 0; b < MB; b++)
#pragma unroll
            for (int u = 0; u < TS; u++) {
                u32x4_t raw[L];
#pragma unroll
                for (int h = 0; h < L; h++) raw[h] = a[b][u][h].u;
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int p = 0; p < 4; p++)
                        a[b][u][j].u[p] =
                            (uint32_t)__builtin_amdgcn_ds_bpermute(from_lane + (j % GPL) * 16, (int)raw[j / GPL][p]);
            }
        if constexpr (BY_TILE) {
            const float4_t zero = {0.f, 0.f, 0.f, 0.f};
            Frag16 off, off_odd;            // the constant operand(s) that take the bias off
            const uint32_t offw = SUB ? kSubBiasL : (BITS == 4 ? kBf16Neg136x2 : kBf16Neg128x2);
            const uint32_t offw_odd = SUB ? kSubBiasH : offw;
            off.u = (u32x4_t){offw, offw, offw, offw};
            off_odd.u = (u32x4_t){offw_odd, offw_odd, offw_odd, offw_odd};
#pragma unroll
            for (int u = 0; u < TS; u++) {
                if (NS > 2) __builtin_amdgcn_sched_barrier(0);
                if (u + WU < TS) {
#pragma unroll
                    for (int s = 0; s < NS; s++) load_tile<BITS>(buf[s][u + WU], w, sbase[s] + kt[u + WU], lane);
                }
                if (NS > 2) __builtin_amdgcn_sched_barrier(0);
                float4_t bias[MB][4];
#pragma unroll
                for (int b = 0; b < MB; b++)
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        if constexpr (SUB)
                            bias[b][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[b][u][j].h, ((j & 1) ? off_odd : off).h, zero, 0, 0, 0);
                        else bias[b][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[b][u][j].b, off.b, zero, 0, 0, 0);
                    }
#pragma unroll
                for (int s = 0; s < NS; s++) {
                    Frag16 bop[4];
                    if constexpr (SUB) {
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            uint32_t bw[4];
                            unpack_q4_sub(buf[s][u].q[0][2 * (j >> 1)], buf[s][u].q[0][2 * (j >> 1) + 1], j & 1, bw);
                            bop[j].u = (u32x4_t){bw[0], bw[1], bw[2], bw[3]};
                        }
                    } else tile_operands<BITS, XMODE>(buf[s][u], magic, bop);
                    u32x2_t sc = buf[s][u].s;
                    sc[0] = valid[u] ? sc[0] : 0u;
                    sc[1] = valid[u] ? sc[1] : 0u;
#pragma unroll
                    for (int b = 0; b < MB; b++) {
                        float4_t d[4];
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            if constexpr (SUB) d[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[b][u][j].h, bop[j].h, bias[b][j], 0, 0, 0);
                            else d[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[b][u][j].b, bop[j].b, bias[b][j], 0, 0, 0);
                        }
                        if constexpr (SUB) {
#pragma unroll
                            for (int j = 0; j < 4; j++) {
                                const uint32_t sb = (j & 1) ? (sc[j >> 1] >> 16) : (sc[j >> 1] & 0xffffu);
                                const float sf = (j & 1) ? f16_bits_to_f32(sb) * 0.0625f : f16_bits_to_f32(sb);
#pragma unroll
                                for (int r = 0; r < 4; r++) acc[s][b][r] = __builtin_fmaf(sf, d[j][r], acc[s][b][r]);
                            }
                        } else tile_accum<4>(sc, d, acc[s][b]);
                    }
                }
            }
        }
#pragma unroll
        for (int s = 0; s < (BY_TILE ? 0 : NS); s++) {
            if (NS > 2) __builtin_amdgcn_sched_barrier(0);
            if (s + AHEAD < NS) {
#pragma unroll
                for (int u = 0; u < TS; u++) load_tile<BITS>(buf[s + AHEAD][u], w, sbase[s + AHEAD] + kt[u], lane);
            }
            if (NS > 2) __builtin_amdgcn_sched_barrier(0);
            float4_t dprev[MB][4];
            u32x2_t sprev = {0u, 0u};
#pragma unroll
            for (int b = 0; b < MB; b++)
#pragma unroll
                for (int j = 0; j < 4; j++) dprev[b][j] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < TS; u++) {
                float4_t d[MB][4];
                Frag16 bop[4];
                tile_operands<BITS, XMODE>(buf[s][u], magic, bop);
#pragma unroll
                for (int b = 0; b < MB; b++) tile_multiply<BITS, XMODE>(a[b][u], bop, d[b]);
                u32x2_t sc = buf[s][u].s;
                sc[0] = valid[u] ? sc[0] : 0u;
                sc[1] = valid[u] ? sc[1] : 0u;
#pragma unroll
                for (int b = 0; b < MB; b++) {
                    tile_accum<4>(sprev, dprev[b], acc[s][b]);
#pragma unroll
                    for (int j = 0; j < 4; j++) dprev[b][j] = d[b][j];
                }
                sprev = sc;
            }
#pragma unroll
            for (int b = 0; b < MB; b++) tile_accum<4>(sprev, dprev[b], acc[s][b]);
        }
    }

    // split-K partials -> LDS, summed in wave order
    // (slot = strip * MB + row block)
    float* red = reinterpret_cast<float*>(smem);
#pragma unroll
    for (int s = 0; s < NS; s++)
#pragma unroll
        for (int b = 0; b < MB; b++)
#pragma unroll
            for (int r = 0; r < 4; r++) red[(((s * MB + b) * nwaves + wv) * 4 + r) * 64 + lane] = acc[s][b][r];
    float* ssq_part = red + NS * MB * nwaves * 4 * 64;      // [wave][row]
    if (NORM) {
        // lane l holds pieces of row l / P: sum over each run of P lanes with lane-crossing moves
        // inside the ALU (pairs, quads, then the mirror images within 8 and within 16 lanes)
        ssq += lane_cross<0xB1>(ssq);
        ssq += lane_cross<0x4E>(ssq);
        if (P >= 8) ssq += lane_cross<0x141>(ssq);
        if (P >= 16) ssq += lane_cross<0x140>(ssq);
        if (lane % P == 0) {
            ssq_part[wv * 16 + lane / P] = ssq;
            if (wv == 0) {                              // the slots of waves this launch does not have
#pragma unroll
                for (int k = 1; k < 8; k++)
                    if (k >= nwaves) ssq_part[k * 16 + lane / P] = 0.f;
            }
        }
    }
    __syncthreads();
    constexpr float kOut = SUB ? kSubUnscale : 1.f;
    float rstd[4] = {kOut, kOut, kOut, kOut};         // of the rows this lane's outputs belong to (SUB: 2^22 of the operands)
    if (NORM) {
        // (eight slots whatever the wave count, all reads in flight at once; rows past the batch read
        // slots nobody wrote and are not stored)
        float4_t t = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < 8; k++) t += *reinterpret_cast<const float4_t*>(ssq_part + k * 16 + 4 * oct);
        // (hardware reciprocal and reciprocal square root, 1 ulp each: the correctly rounded divisions
        // and root are some 140 instructions here, half a microsecond between the barrier and the stores)
        const float inv_k = __builtin_amdgcn_rcpf((float)w.K);
#pragma unroll
        for (int r = 0; r < 4; r++) rstd[r] = __builtin_amdgcn_rsqf(fmaf(t[r], inv_k, epi.eps));
    }
    // wave v finishes (strip, output register) pairs v, v + waves, ...
    if (NS >= 2 && epi.kind == kEpiSwiglu) {       // strips 2j / 2j+1 of the group are gate / up of output strip (strip0 >> 1) + j
        const int n_out = w.N >> 1;
        for (int p = wv; p < NS * MB * 2; p += nwaves) {
            const int r = p & 3, b = (p >> 2) % MB, j = (p >> 2) / MB;
            const int nt = (strip0 >> 1) + j;
            const int n = nt * 16 + (lane & 15);
            const float g = sum_partials(red + (((2 * j) * MB + b) * nwaves * 4 + r) * 64 + lane, nwaves, 4 * 64) * rstd[r];
            const float u = sum_partials(red + (((2 * j + 1) * MB + b) * nwaves * 4 + r) * 64 + lane, nwaves, 4 * 64) * rstd[r];
            const int m = 16 * b + 4 * oct + r;
            if (2 * nt + 1 < w.NT && m < M && n < n_out) store_out(y, ydt, (int64_t)m * n_out + n, silu_mul(g, u));
        }
        return;
    }
    if constexpr (KS) {
        constexpr int OUTS = NS * MB * 4;                 // output registers of a workgroup, 64 lanes each
        const int groups = (int)gridDim.x / splits;
        float* mine = slabs + ((size_t)split * groups + group) * (OUTS * 64);
        for (int p = wv; p < OUTS; p += nwaves) {
            const int r = p & 3, sb = p >> 2;
            const float v = sum_partials(red + (sb * nwaves * 4 + r) * 64 + lane, nwaves, 4 * 64) * rstd[r];
            __hip_atomic_store(mine + p * 64 + lane, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");          // my part of the slab has reached memory
        __syncthreads();                                          // (and everybody is done reading `red`)
        unsigned* flag = reinterpret_cast<unsigned*>(red);
        if (tid == 0) {
            const unsigned old = __hip_atomic_fetch_add(tickets + group, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const bool last = old + 1u == (unsigned)splits;
            if (last) __hip_atomic_store(tickets + group, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *flag = last ? 1u : 0u;
        }
        __syncthreads();
        if (*flag == 0u) return;
        const size_t slab_stride = (size_t)groups * (OUTS * 64);
        const float* first = slabs + (size_t)group * (OUTS * 64);
        for (int p = wv; p < OUTS; p += nwaves) {
            const int r = p & 3, b = (p >> 2) % MB, s = (p >> 2) / MB;
            float part[4];                                 // (at most four splits: rows_split_plan)
#pragma unroll
            for (int k = 0; k < 4; k++)
                part[k] = __hip_atomic_load(first + (size_t)min(k, splits - 1) * slab_stride + p * 64 + lane, __ATOMIC_RELAXED,
                                            __HIP_MEMORY_SCOPE_SYSTEM);
            float v = part[0];
#pragma unroll
            for (int k = 1; k < 4; k++) v += k < splits ? part[k] : 0.f;
            const int nt = strip0 + s;
            const int n = nt * 16 + (lane & 15);
            const int m = 16 * b + 4 * oct + r;
            if (nt < w.NT && m < M && n < w.N) emit(y, ydt, epi, (int64_t)m * w.N + n, v);
        }
        return;
    }
    for (int p = wv; p < NS * MB * 4; p += nwaves) {
        const int r = p & 3, b = (p >> 2) % MB, s = (p >> 2) / MB;
        const int nt = strip0 + s;
        const int n = nt * 16 + (lane & 15);
        const float v = sum_partials(red + ((s * MB + b) * nwaves * 4 + r) * 64 + lane, nwaves, 4 * 64) * rstd[r];
        const int m = 16 * b + 4 * oct + r;
        if (nt < w.NT && m < M && n < w.N) emit(y, ydt, epi, (int64_t)m * w.N + n, v);
    }
}

template <int BITS, int XMODE, int TS, int NS, int XR, int MB = 1>
hipError_t launch_rows_x(const WeightView& w, const void* x, int M, void* y, int ydt, int nwaves, const Epilogue& epi,
                         bool sub, hipStream_t st)
{
    size_t lds = (size_t)NS * MB * nwaves * 4 * 64 * sizeof(float) + 8 * 16 * sizeof(float);
    const unsigned groups = (unsigned)((w.NT + NS - 1) / NS);
    if constexpr (MB == 1) {
        if (epi.gamma) {
            lds += (size_t)nwaves * TS * kTileK * sizeof(float);            // each wave's tiles of gamma as fp32
            auto kern = gemv_rows_kernel<BITS, XMODE, TS, NS, true, XR>;
            (void)LdsRequest<&gemv_rows_kernel<BITS, XMODE, TS, NS, true, XR>, 150 * 1024>::registered;
            if (lds > 150 * 1024) return hipErrorInvalidValue;
            hipLaunchKernelGGL(kern, dim3(groups), dim3(nwaves * 64), lds, st, w.base, reinterpret_cast<const uint16_t*>(x), epi.gamma,
                               w.KT, w.K, w.NT, M, nwaves, epi.gamma_dt, w.N, y, ydt, epi, 1, 0, nullptr, nullptr);
            return hipGetLastError();
        }
    }
    // decode mode STREAM, Q4 and f16 activations, two to four strips: subnormal operands
    // (with two row blocks, 17..32 rows, it measures 0.3 us slower than the integer operands, but a row keeps
    // the bits it has in a batch of up to 16)
    if constexpr (BITS == 4 && XMODE == XF16 && NS >= 2 && NS <= 4 && (TS == 4 || MB == 2)) {
        if (sub && !epi.gamma) {
            if constexpr (NS * MB * 8 * 1024 + 512 > 64 * 1024)
                (void)LdsRequest<&gemv_rows_kernel<BITS, XMODE, TS, NS, false, XR, MB, true>, 150 * 1024>::registered;
            hipLaunchKernelGGL((gemv_rows_kernel<BITS, XMODE, TS, NS, false, XR, MB, true>), dim3(groups), dim3(nwaves * 64), lds, st,
                               w.base, reinterpret_cast<const uint16_t*>(x), nullptr, w.KT, w.K, w.NT, M, nwaves, 0, w.N, y, ydt, epi, 1, 0, nullptr,
                               nullptr);
            return hipGetLastError();
        }
    }
    // (the exchange area alone passes 64 KB with eight strips, or four strips and two row blocks)
    if constexpr (NS * MB * 8 * 1024 + 512 > 64 * 1024)
        (void)LdsRequest<&gemv_rows_kernel<BITS, XMODE, TS, NS, false, XR, MB>, 150 * 1024>::registered;
    hipLaunchKernelGGL((gemv_rows_kernel<BITS, XMODE, TS, NS, false, XR, MB>), dim3(groups), dim3(nwaves * 64), lds, st, w.base,
                       reinterpret_cast<const uint16_t*>(x), nullptr, w.KT, w.K, w.NT, M, nwaves, 0, w.N, y, ydt, epi, 1, 0, nullptr, nullptr);
    return hipGetLastError();
}

// Few strips and a long K (the down projection): four strips per workgroup, K split four ways over
// workgroups, the slabs added by the workgroup that arrives last (gemv_rows_kernel, KS).
struct SplitPlan {
    int splits, kt_per_split, nwaves, groups;
};

constexpr int kSplitStrips = 4, kSplitWays = 4;

bool rows_split_plan(const WeightView& w, int xdt, int M, int num_cus, const Epilogue& epi, size_t scratch_bytes, SplitPlan& sp)
{
    if (w.bits != 4 || xdt == kF32 || epi.gamma || epi.kind == kEpiSwiglu) return false;
    // a long K and about one strip per CU (14336 -> 4096 on 256 CUs: 12.6 against 13.9 us at 16 rows, 17.4 against
    // 21.5 at 32; with K = 11008 or a quarter of the strips the split only costs: its slabs and ticket add 2.5 - 3 us)
    if (w.KT < 96 || (int64_t)w.NT * 2 > (int64_t)num_cus * 3 || (int64_t)w.NT * 4 < (int64_t)num_cus * 3) return false;
    sp.splits = kSplitWays;
    sp.kt_per_split = (w.KT + sp.splits - 1) / sp.splits;
    sp.splits = (w.KT + sp.kt_per_split - 1) / sp.kt_per_split;                         // no empty split
    sp.nwaves = min(8, (sp.kt_per_split + 3) / 4);
    sp.groups = (w.NT + kSplitStrips - 1) / kSplitStrips;
    const size_t need = (size_t)sp.splits * sp.groups * (kSplitStrips * 2 * 4 * 64) * sizeof(float) + (size_t)sp.groups * sizeof(unsigned) + 256;
    return sp.splits > 1 && sp.splits <= 4 && sp.groups * sizeof(unsigned) <= ((size_t)1 << 16) && need <= scratch_bytes;
}

template <int XMODE, int XR, int MB>
hipError_t launch_rows_split_x(const WeightView& w, const void* x, int M, void* y, int ydt, const Epilogue& epi, bool sub,
                               const SplitPlan& sp, void* scratch, hipStream_t st)
{
    constexpr int NS = kSplitStrips, TS = MB == 1 ? 4 : 2;
    // tickets first (one word per group, zero at rest), slabs behind them
    unsigned* tickets = reinterpret_cast<unsigned*>(scratch);
    float* slabs = reinterpret_cast<float*>(static_cast<char*>(scratch) + (((size_t)sp.groups * sizeof(unsigned) + 255) & ~(size_t)255));
    const size_t lds = (size_t)NS * MB * sp.nwaves * 4 * 64 * sizeof(float) + 8 * 16 * sizeof(float);
    const dim3 grid((unsigned)(sp.groups * sp.splits)), block((unsigned)sp.nwaves * 64);
    const uint16_t* xp = reinterpret_cast<const uint16_t*>(x);
    if constexpr (XMODE == XF16) {
        if (sub) {
            if constexpr (NS * MB * 8 * 1024 + 512 > 64 * 1024)
                (void)LdsRequest<&gemv_rows_kernel<4, XMODE, TS, NS, false, XR, MB, true, true>, 150 * 1024>::registered;
            hipLaunchKernelGGL((gemv_rows_kernel<4, XMODE, TS, NS, false, XR, MB, true, true>), grid, block, lds, st, w.base, xp, nullptr, w.KT,
                               w.K, w.NT, M, sp.nwaves, 0, w.N, y, ydt, epi, sp.splits, sp.kt_per_split, slabs, tickets);
            return hipGetLastError();
        }
    }
    if constexpr (NS * MB * 8 * 1024 + 512 > 64 * 1024)
        (void)LdsRequest<&gemv_rows_kernel<4, XMODE, TS, NS, false, XR, MB, false, true>, 150 * 1024>::registered;
    hipLaunchKernelGGL((gemv_rows_kernel<4, XMODE, TS, NS, false, XR, MB, false, true>), grid, block, lds, st, w.base, xp, nullptr, w.KT, w.K,
                       w.NT, M, sp.nwaves, 0, w.N, y, ydt, epi, sp.splits, sp.kt_per_split, slabs, tickets);
    return hipGetLastError();
}

template <int XMODE>
hipError_t launch_rows_split(const WeightView& w, const void* x, int M, void* y, int ydt, const Epilogue& epi, bool sub,
                             const SplitPlan& sp, void* scratch, hipStream_t st)
{
    if (M > 16) return launch_rows_split_x<XMODE, 16, 2>(w, x, M, y, ydt, epi, sub, sp, scratch, st);
    if (M <= 4) return launch_rows_split_x<XMODE, 4, 1>(w, x, M, y, ydt, epi, sub, sp, scratch, st);
    if (M <= 8) return launch_rows_split_x<XMODE, 8, 1>(w, x, M, y, ydt, epi, sub, sp, scratch, st);
    return launch_rows_split_x<XMODE, 16, 1>(w, x, M, y, ydt, epi, sub, sp, scratch, st);
}

// (the x load pattern follows the batch: up to 4, up to 8, up to 16 rows per load)
template <int BITS, int XMODE, int TS, int NS>
hipError_t launch_rows_t(const WeightView& w, const void* x, int M, void* y, int ydt, int nwaves, const Epilogue& epi,
                         bool sub, hipStream_t st)
{
    if (M <= 4) return launch_rows_x<BITS, XMODE, TS, NS, 4>(w, x, M, y, ydt, nwaves, epi, sub, st);
    if (M <= 8) return launch_rows_x<BITS, XMODE, TS, NS, 8>(w, x, M, y, ydt, nwaves, epi, sub, st);
    return launch_rows_x<BITS, XMODE, TS, NS, 16>(w, x, M, y, ydt, nwaves, epi, sub, st);
}

// strips per workgroup: as many as keeps about one workgroup per CU, at most 4
int strips_per_group(const WeightView& w, int num_cus, const Epilogue& epi)
{
    int ns = (w.NT + num_cus / 2) / num_cus;
    ns = ns >= 3 ? 4 : (ns >= 2 ? 2 : 1);
    if (epi.kind == kEpiSwiglu && ns < 2) ns = 2;          // a gate strip and its up strip share a workgroup
    return ns;
}

template <int BITS, int XMODE>
hipError_t launch_rows(const WeightView& w, const void* x, int M, void* y, int ydt, int tuned_waves, int num_cus,
                       const Epilogue& epi, bool sub, hipStream_t st)
{
    // 8 waves split K (fewer when the strip has fewer tiles), 4 tiles of x per wave and slab
    const int ns = strips_per_group(w, num_cus, epi);
    // seven strips per workgroup when that is exactly one workgroup per CU (N = 28672 on 256 CUs:
    // with four strips the 448 workgroups need a second, mostly empty round); SwiGLU pairs need an
    // even count: eight strips there, 224 workgroups in one round
    const bool seven = w.NT == 7 * num_cus;
    int nwaves = tuned_waves > 0 ? min(tuned_waves, 8) : 8;
    while (nwaves > 1 && nwaves * 2 > w.KT) nwaves >>= 1;
    if constexpr (BITS == 4) {
        // several rounds of workgroups per CU (the LM head: 2004 of them): two tiles per wave and slab
        // instead of four halve the registers, two workgroups share a CU and one's ramp and tail
        // overlap the other's stream (128256 rows at 8 rows: 70 -> 54 us)
        if (ns == 4 && (int64_t)w.NT >= (int64_t)8 * num_cus && !epi.gamma)
            return launch_rows_t<BITS, XMODE, 2, 4>(w, x, M, y, ydt, nwaves, epi, sub, st);
        if (seven && epi.kind == kEpiSwiglu) return launch_rows_t<BITS, XMODE, 4, 8>(w, x, M, y, ydt, nwaves, epi, sub, st);
        if (seven && epi.kind != kEpiSwiglu) return launch_rows_t<BITS, XMODE, 4, 7>(w, x, M, y, ydt, nwaves, epi, sub, st);
        if (ns == 4) return launch_rows_t<BITS, XMODE, 4, 4>(w, x, M, y, ydt, nwaves, epi, sub, st);
    } else if constexpr (XMODE == XF16) {
        // Q8 tiles are twice the registers: four strips x four tiles of f16 operands would spill.  Two
        // strips x two tiles (80 registers, six waves per SIMD) stream best there; bf16 operands fit
        if (ns == 4) return launch_rows_t<BITS, XMODE, 2, 2>(w, x, M, y, ydt, nwaves, epi, sub, st);
    } else {
        if (ns == 4) return launch_rows_t<BITS, XMODE, 4, 4>(w, x, M, y, ydt, nwaves, epi, sub, st);
    }
    if (ns == 2) return launch_rows_t<BITS, XMODE, 4, 2>(w, x, M, y, ydt, nwaves, epi, sub, st);
    if constexpr (BITS == 4) {
        // one strip per workgroup and a long K: eight tiles per wave and slab (fewer round trips), unless
        // that leaves more of the last slab empty than seven or four would - tiles past the end are still loaded
        // (11008 -> 4096: 86 tiles are 2 slabs of 64 or 3 of 32, 15.6 -> 11.7 us at 16 rows; 14336 -> 4096:
        // 112 tiles are 2 slabs of 56, seven tiles per wave)
        auto pad = [&](int ts) { return (w.KT + nwaves * ts - 1) / (nwaves * ts) * (nwaves * ts) - w.KT; };
        if (w.KT > nwaves * 4) {
            // (seven or eight tiles of full-width x loads and a folded norm do not fit the registers)
            const bool fits = !epi.gamma || M <= 8;
            if (pad(8) <= pad(7) && pad(8) <= pad(4) && fits) return launch_rows_t<BITS, XMODE, 8, 1>(w, x, M, y, ydt, nwaves, epi, sub, st);
            if (pad(7) <= pad(4) && fits) return launch_rows_t<BITS, XMODE, 7, 1>(w, x, M, y, ydt, nwaves, epi, sub, st);
        }
    }
    return launch_rows_t<BITS, XMODE, 4, 1>(w, x, M, y, ydt, nwaves, epi, sub, st);
}

// 17 .. 32 rows: two activation operands per weight operand.  Two tiles of x per wave and slab
// (a wave holds 2 x 2 x 4 operand fragments) when a workgroup has several strips, four with one.
template <int BITS, int XMODE>
hipError_t launch_rows2(const WeightView& w, const void* x, int M, void* y, int ydt, int tuned_waves, int num_cus,
                        const Epilogue& epi, bool sub, hipStream_t st)
{
    const int ns = strips_per_group(w, num_cus, epi);
    int nwaves = tuned_waves > 0 ? min(tuned_waves, 8) : 8;
    while (nwaves > 1 && nwaves * 2 > w.KT) nwaves >>= 1;
    if constexpr (BITS == 4) {
        if (w.NT == 7 * num_cus && epi.kind != kEpiSwiglu)
            return launch_rows_x<BITS, XMODE, 2, 7, 16, 2>(w, x, M, y, ydt, nwaves, epi, sub, st);
        if (ns == 4) return launch_rows_x<BITS, XMODE, 2, 4, 16, 2>(w, x, M, y, ydt, nwaves, epi, sub, st);
    }
    if (ns >= 2) return launch_rows_x<BITS, XMODE, 2, 2, 16, 2>(w, x, M, y, ydt, nwaves, epi, sub, st);
    if constexpr (BITS == 4) return launch_rows_x<BITS, XMODE, 4, 1, 16, 2>(w, x, M, y, ydt, nwaves, epi, sub, st);
    return launch_rows_x<BITS, XMODE, 2, 1, 16, 2>(w, x, M, y, ydt, nwaves, epi, sub, st);
}

int g_tune_waves = 0, g_tune_unroll = 0, g_tune_rows = 0;
constexpr int kSplitMinRows = 12;

constexpr int kLdsBudget = 64 * 1024;      // what a slab of x aims for
constexpr int kLdsCap = 150 * 1024;         // what a launch may ask for

template <int BITS, int XMODE, int RMAX, int U, bool ONESHOT, int PAIR, bool NORM>
hipError_t launch_p(const WeightView& w, const void* x, int M, void* y, int ydt, int nwaves, const Epilogue& epi,
                    hipStream_t st)
{
    const int planes = XMODE == XF32 ? 2 : 1;
    // x is staged in K slabs that fit the LDS budget.  A slab is a whole number
    // of rounds over the waves, so which wave owns tile kt (kt % nwaves) - and
    // with it the summation order - does not depend on M.
    int slab_tiles = w.KT;
    if (!ONESHOT && (int64_t)M * (w.KT * kTileK + 8) * 2 * planes > kLdsBudget) {
        int k_fit = kLdsBudget / (2 * M * planes) - 8;
        slab_tiles = k_fit / kTileK;
        int step = nwaves * U;
        if (slab_tiles >= step) slab_tiles -= slab_tiles % step;
        else slab_tiles -= slab_tiles % nwaves;
        if (slab_tiles < nwaves) slab_tiles = nwaves;
    }
    int ldx = slab_tiles * kTileK + 8;
    const size_t xbytes = ((size_t)M * ldx * 2 * planes + 255) & ~(size_t)255;
    // x, then the waves' partial sums, then 16 row sums of squares and their 16 x 16 per-wave parts (folded RMSNorm)
    const size_t lds = xbytes + (size_t)PAIR * nwaves * RMAX * 64 * sizeof(float) + (16 + 256) * sizeof(float);
    auto kern = gemv_kernel<BITS, XMODE, RMAX, U, ONESHOT, PAIR, NORM>;
    // A slab is at least one tile per wave, whatever the budget says: 16 rows of fp32 activations
    // (two 16-bit planes) on 16 waves stage 16 x 2056 x 4 B = 129 KB, plus 16 KB of partial sums
    // and the norm's row sums - the largest request there is, 146 KB.
    (void)LdsRequest<&gemv_kernel<BITS, XMODE, RMAX, U, ONESHOT, PAIR, NORM>, kLdsCap>::registered;
    if (lds > (size_t)kLdsCap) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kern, dim3(w.NT / PAIR), dim3(nwaves * PAIR * 64), lds, st, w.base, x, w.KT, w.K, M, nwaves * PAIR * 64, slab_tiles, ldx,
                       (int)xbytes, y, w.N, ydt, w.NT, epi);
    return hipGetLastError();
}

template <int BITS, int XMODE, int RMAX, int U, bool ONESHOT, bool NORM>
hipError_t launch_t(const WeightView& w, const void* x, int M, void* y, int ydt, int nwaves, const Epilogue& epi,
                    hipStream_t st)
{
    if (epi.kind == kEpiSwiglu) return launch_p<BITS, XMODE, RMAX, U, ONESHOT, 2, NORM>(w, x, M, y, ydt, nwaves, epi, st);
    return launch_p<BITS, XMODE, RMAX, U, ONESHOT, 1, NORM>(w, x, M, y, ydt, nwaves, epi, st);
}

template <int BITS, int XMODE, int U, bool ONESHOT, bool NORM = false>
hipError_t launch_r(const WeightView& w, const void* x, int M, void* y, int ydt, int nwaves, const Epilogue& epi,
                    hipStream_t st)
{
    if (M == 1) return launch_t<BITS, XMODE, 1, U, ONESHOT, NORM>(w, x, M, y, ydt, nwaves, epi, st);
    if (M == 2) return launch_t<BITS, XMODE, 2, U, ONESHOT, NORM>(w, x, M, y, ydt, nwaves, epi, st);
    return launch_t<BITS, XMODE, 4, U, ONESHOT, NORM>(w, x, M, y, ydt, nwaves, epi, st);
}

template <int BITS, int XMODE>
hipError_t launch_u(const WeightView& w, const void* x, int M, void* y, int ydt, int nwaves, int unroll,
                    const Epilogue& epi, hipStream_t st)
{
    const int planes = XMODE == XF32 ? 2 : 1;
    const bool one_slab = (int64_t)M * (w.KT * kTileK + 8) * 2 * planes <= kLdsBudget;
    const int per_wave = (w.KT + nwaves - 1) / nwaves;
    if (epi.gamma) return launch_r<BITS, XMODE, 2, false, true>(w, x, M, y, ydt, nwaves, epi, st);    // folded RMSNorm
    if (one_slab && unroll == 0) {
        if (per_wave <= 2) return launch_r<BITS, XMODE, 2, true>(w, x, M, y, ydt, nwaves, epi, st);
        if (per_wave <= 4) return launch_r<BITS, XMODE, 4, true>(w, x, M, y, ydt, nwaves, epi, st);
        // (fp32 activations carry two operand planes: 8 tiles in flight would spill)
        if (per_wave <= 8 && XMODE != XF32) return launch_r<BITS, XMODE, 8, true>(w, x, M, y, ydt, nwaves, epi, st);
    }
    if (unroll == 4 && XMODE != XF32) return launch_r<BITS, XMODE, 4, false>(w, x, M, y, ydt, nwaves, epi, st);
    return launch_r<BITS, XMODE, 2, false>(w, x, M, y, ydt, nwaves, epi, st);
}

}  // namespace

void set_gemv_tuning(int waves_per_group, int rows_kernel, int unroll)
{
    g_tune_waves = waves_per_group;
    g_tune_rows = rows_kernel;       // 0 automatic, 1 always the register kernel, 2 never, 3 / 4: always, K split never / whenever it applies
    g_tune_unroll = unroll;
}

// 17 .. 32 rows in one pass (weights streamed once): 16-bit activations, no folded norm
bool gemv_serves_32(int xdt, int M, const Epilogue& epi)
{
    return M > 16 && M <= 32 && xdt != kF32 && !epi.gamma && g_tune_rows != 2;
}

hipError_t launch_gemv(const WeightView& w, const void* x, int xdt, int M, void* y, int ydt,
                       int num_cus, bool exact_operands, const Epilogue& epi, void* scratch, size_t scratch_bytes, hipStream_t st)
{
    // Waves per workgroup (= split of a strip's K tiles).  Depends on the weight
    // shape only, never on M, so that the summation order is the same for every
    // batch size: up to 4 waves (2 when there are strips enough for 8 waves per CU anyway), then
    // more if that is what it takes to bring a wave's share down to 8 tiles, all requested
    // up front.  (K = 4096 is 4 waves x 8 tiles for every N: with few strips 8 waves x 4 tiles
    // measured 2 - 4 % slower.)
    // one or two f16 rows: the kernel of gemv1.hip (unless the caller asked for exact integer weight
    // operands, or a test forces one of the kernels below)
    if (!exact_operands && g_tune_waves == 0 && g_tune_rows == 0 && g_tune_unroll == 0 && gemv1_serves(w, xdt, M, epi))
        return launch_gemv1(w, x, xdt, M, y, ydt, epi, st);
    int nwaves = g_tune_waves;
    if (nwaves <= 0) {
        nwaves = 2;
        while (nwaves < 4 && (int64_t)w.NT * nwaves < (int64_t)num_cus * 8) nwaves *= 2;
        while (nwaves < 16 && w.KT > 8 * nwaves) nwaves *= 2;
    }
    if (nwaves > 16) nwaves = 16;
    if (epi.kind == kEpiSwiglu && nwaves > 8) nwaves = 8;      // two strips per workgroup: 2 x 8 waves at most
    while (nwaves > 1 && nwaves > w.KT) nwaves >>= 1;
    // 0: request a wave's whole share up front when it fits, else stream in batches of 2
    int unroll = g_tune_unroll;
    // One workgroup per CU and a long K (the down projection): nothing else runs on the CU while a
    // wave sits in the issue of its up-front requests, so stream in batches of two there -
    // arithmetic in between the requests (14336 -> 4096: 10.2 -> 8.8 us, 11008 -> 4096: 9.4 -> 7.9 us).
    // Which wave owns which tile, and with it every sum, is the same either way.
    if (g_tune_waves <= 0 && g_tune_unroll == 0 && w.NT <= num_cus && w.KT > 64 && epi.kind != kEpiSwiglu) {
        nwaves = w.KT >= 96 ? 16 : 8;
        unroll = 2;
    }

    // three or more batch rows (16-bit activations): x in registers, shared across strips
    // (Q8 on wide outputs: up to four rows the LDS kernel is still the quicker one, 24.0 against
    // 27.6 us at 4096 -> 28672)
    const bool wide_q8 = w.bits == 8 && (w.NT + num_cus / 2) / num_cus >= 3;
    const bool rows_kernel = g_tune_rows == 1 || g_tune_rows >= 3 || (g_tune_rows == 0 && M >= (wide_q8 ? 5 : 3));
    if (M > 16 && !gemv_serves_32(xdt, M, epi)) return hipErrorInvalidValue;
    // few strips, a long K, twelve rows or more: K split over workgroups (tuning 3: never, 4: from three rows on)
    if (rows_kernel && xdt != kF32 && scratch && g_tune_rows != 3 && g_tune_waves == 0 && (M >= kSplitMinRows || g_tune_rows == 4)) {
        SplitPlan sp;
        if (rows_split_plan(w, xdt, M, num_cus, epi, scratch_bytes, sp)) {
            if (xdt == kF16) return launch_rows_split<XF16>(w, x, M, y, ydt, epi, !exact_operands, sp, scratch, st);
            return launch_rows_split<XBF16>(w, x, M, y, ydt, epi, !exact_operands, sp, scratch, st);
        }
    }
    if (M > 16) {
        if (w.bits == 4) {
            if (xdt == kF16) return launch_rows2<4, XF16>(w, x, M, y, ydt, g_tune_waves, num_cus, epi, !exact_operands, st);
            return launch_rows2<4, XBF16>(w, x, M, y, ydt, g_tune_waves, num_cus, epi, !exact_operands, st);
        }
        if (xdt == kF16) return launch_rows2<8, XF16>(w, x, M, y, ydt, g_tune_waves, num_cus, epi, !exact_operands, st);
        return launch_rows2<8, XBF16>(w, x, M, y, ydt, g_tune_waves, num_cus, epi, !exact_operands, st);
    }
    if (rows_kernel && xdt != kF32) {
        if (w.bits == 4) {
            if (xdt == kF16) return launch_rows<4, XF16>(w, x, M, y, ydt, g_tune_waves, num_cus, epi, !exact_operands, st);
            return launch_rows<4, XBF16>(w, x, M, y, ydt, g_tune_waves, num_cus, epi, !exact_operands, st);
        }
        if (xdt == kF16) return launch_rows<8, XF16>(w, x, M, y, ydt, g_tune_waves, num_cus, epi, !exact_operands, st);
        return launch_rows<8, XBF16>(w, x, M, y, ydt, g_tune_waves, num_cus, epi, !exact_operands, st);
    }

    if (w.bits == 4) {
        if (xdt == kF16) return launch_u<4, XF16>(w, x, M, y, ydt, nwaves, unroll, epi, st);
        if (xdt == kBF16) return launch_u<4, XBF16>(w, x, M, y, ydt, nwaves, unroll, epi, st);
        return launch_u<4, XF32>(w, x, M, y, ydt, nwaves, unroll, epi, st);
    }
    if (xdt == kF16) return launch_u<8, XF16>(w, x, M, y, ydt, nwaves, unroll, epi, st);
    if (xdt == kBF16) return launch_u<8, XBF16>(w, x, M, y, ydt, nwaves, unroll, epi, st);
    return launch_u<8, XF32>(w, x, M, y, ydt, nwaves, unroll, epi, st);
}

}  // namespace cybq
