// gemm_parts.h - pieces shared by the prefill kernels (gemm.hip, gemm_rows.hip): output element
// access, the row statistics of a folded norm / widened activations, a weight tile in registers,
// the MFMA wrapper and the epilogue that writes a wave's finished sums.  Included inside
// namespace cybq { namespace { ... } } of each translation unit.
#ifndef CYBQ_GEMM_PARTS_H
#define CYBQ_GEMM_PARTS_H

typedef float float2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void store_out_g(void* y, int ydt, int64_t idx, float v)
{
    if (ydt == kF32) reinterpret_cast<float*>(y)[idx] = v;
    else if (ydt == kF16) reinterpret_cast<_Float16*>(y)[idx] = (_Float16)v;
    else reinterpret_cast<uint16_t*>(y)[idx] = f32_to_bf16_bits(v);
}


__device__ __forceinline__ float load_out_g(const void* p, int dt, int64_t idx)
{
    if (dt == kF32) return reinterpret_cast<const float*>(p)[idx];
    if (dt == kF16) return (float)reinterpret_cast<const _Float16*>(p)[idx];
    return __builtin_bit_cast(float, (uint32_t)reinterpret_cast<const uint16_t*>(p)[idx] << 16);
}

// Folded RMSNorm on the prefill path: the staging pass leaves, per row of the chunk, `nblk`
// partial sums of squares; rstd of a row adds them in index order.
// `unscale` (FAST mode with widened activations): the power of two every staged row was
// divided by on its way to f16, to be multiplied back onto the finished sums.
struct NormStats {
    const float* part;
    int nblk;
    const float* unscale;
};

__device__ __forceinline__ float rstd_of(const NormStats& ns, int row, int K, float eps)
{
    float t = 0.f;
    for (int j = 0; j < ns.nblk; j++) t += ns.part[(int64_t)row * ns.nblk + j];
    return 1.0f / sqrtf(t / (float)K + eps);
}

// what a finished sum of row `row` is multiplied by before the epilogue
__device__ __forceinline__ float row_factor(const NormStats& ns, bool norm, int row, int K, float eps)
{
    float f = ns.unscale ? ns.unscale[row] : 1.0f;
    if (norm) f *= rstd_of(ns, row, K, eps);
    return f;
}

template <int BITS>
struct WRegs {               // one native weight tile as loaded by one lane, and its 4 group scales
    u32x4_t q[BITS == 4 ? 1 : 2];
    u32x2_t s;
};

template <int BITS>
__device__ __forceinline__ void load_wtile(WRegs<BITS>& r, const WeightView& w, int64_t tile, int lane)
{
    const u32x4_t* qp = tile_q<BITS>(w, tile);
    r.q[0] = qp[lane];
    if (BITS == 8) r.q[BITS == 4 ? 0 : 1] = qp[64 + lane];
    r.s = tile_s<BITS>(w, tile)[lane & 15];
}

template <int XBF>
__device__ __forceinline__ float4_t mma(const Frag16& a, const Frag16& b, float4_t c)
{
    if (XBF) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, b.b, c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a.h, b.h, c, 0, 0, 0);
}

// The finished sums of one wave (MF row blocks x NF column blocks, lane = column, four rows per lane;
// first row m0, first column block nt0) -> y, with the residual-add epilogue.  `stg`: 16 x NF*16
// floats of LDS that belong to this wave.
template <int MF, int NF>
__device__ __forceinline__ void write_rows(const float4_t (&acc)[MF][NF], float* stg, int m0, int nt0, int M, int N, void* y, int ydt,
                                           float out_scale, const Epilogue& epi, int lane)
{
    const int row16 = lane & 15, oct = lane >> 4;
    // Output rows that start on a 16-byte boundary (8 for 16-bit outputs): the accumulators (lane =
    // column, four rows per lane) go through LDS - the operand buffers are free after the last K
    // tile's barrier, a wave's share of them holds one of its row blocks - and leave four
    // elements per lane, 64 lanes writing whole runs of a row instead of 64-byte pieces of four rows.
    const uintptr_t amask = ydt == kF32 ? 15u : 7u;
    const bool rows_aligned = (N & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & amask) == 0 &&
                              (epi.kind != kEpiAdd || (reinterpret_cast<uintptr_t>(epi.residual) & amask) == 0);
    if (rows_aligned) {
        constexpr int ROWF = NF * 16;               // floats of a tile row
        constexpr int V4 = ROWF / 4;                // four-element pieces of a tile row
        const float4_t* stg4 = reinterpret_cast<const float4_t*>(stg);
#pragma unroll
        for (int i = 0; i < MF; i++) {
#pragma unroll
            for (int f = 0; f < NF; f++)
#pragma unroll
                for (int r = 0; r < 4; r++) stg[(oct * 4 + r) * ROWF + f * 16 + row16] = acc[i][f][r] * out_scale;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int p = lane; p < 16 * V4; p += 64) {
                const int row = p / V4, c4 = p - row * V4;
                const int m = m0 + i * 16 + row, n = nt0 * 16 + c4 * 4;
                if (m < M && n < N) {
                    float4_t v = stg4[p];
                    const int64_t at = (int64_t)m * N + n;
                    if (ydt == kF32) {
                        if (epi.kind == kEpiAdd) v += *reinterpret_cast<const float4_t*>(reinterpret_cast<const float*>(epi.residual) + at);
                        *reinterpret_cast<float4_t*>(reinterpret_cast<float*>(y) + at) = v;
                    } else {
                        if (epi.kind == kEpiAdd) {
                            const u32x2_t rr = *reinterpret_cast<const u32x2_t*>(reinterpret_cast<const uint16_t*>(epi.residual) + at);
#pragma unroll
                            for (int e = 0; e < 4; e++) {
                                const uint32_t h = (e & 1) ? rr[e >> 1] >> 16 : rr[e >> 1] & 0xffffu;
                                v[e] += ydt == kF16 ? f16_bits_to_f32(h) : __builtin_bit_cast(float, h << 16);
                            }
                        }
                        u32x2_t o;
                        if (ydt == kF16) {
                            const half2_t a = {(_Float16)v[0], (_Float16)v[1]}, b = {(_Float16)v[2], (_Float16)v[3]};
                            o = (u32x2_t){as_u32(a), as_u32(b)};
                        } else {
                            o = (u32x2_t){(uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16),
                                          (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16)};
                        }
                        *reinterpret_cast<u32x2_t*>(reinterpret_cast<uint16_t*>(y) + at) = o;
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < MF; i++)
#pragma unroll
        for (int f = 0; f < NF; f++) {
            const int n = (nt0 + f) * 16 + row16;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int m = m0 + i * 16 + oct * 4 + r;
                if (m < M && n < N) {
                    float v = acc[i][f][r] * out_scale;
                    if (epi.kind == kEpiAdd) v += load_out_g(epi.residual, ydt, (int64_t)m * N + n);
                    store_out_g(y, ydt, (int64_t)m * N + n, v);
                }
            }
        }
}

#endif
