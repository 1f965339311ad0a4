/*
 * cybq_cpu_baseline.c - the CPU path timed beside the GPU numbers.  Test infrastructure like
 * the rest of oracle/: only bench.py's cpu_baseline leg (and the test that checks it against
 * cybq_oracle_matmul_f64) loads it; nothing under cyb_amd/ does.
 *
 * What it restates: the reference runs this operator on the CPU with rayon (row-parallel
 * threads) and `wide` (portable SIMD) over the tensor data of the mmap'd .model file
 * (/root/reference/Cargo.lock:8443-8462; Q4_0 blocks, /root/reference/decide/pipeline.md:38,59).
 * That source is not in the tree, so this is a restatement of the same plan, not the
 * reference's code:   y[n] = sum_g f32(d[n,g]) * sum_{k in g} x[k] * q[n,k]   in fp32,
 * reading packed BLOCK_AOS Q4_0 bytes (18 B per 32 weights: f16 d, then byte j =
 * (w[j]+8) | (w[j+16]+8) << 4), rows split over all host cores (OpenMP), the inner loops
 * written with SIMD intrinsics, one build per instruction set picked at run time
 * (AVX-512, AVX2+FMA, plain C) because the box that runs it is not the box that
 * builds it.  Unlike cybq_oracle.c it is built with contraction allowed: it is the thing
 * timed, and it is checked against the oracle before it is timed.
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#include <omp.h>

typedef float (*row_dot_fn)(const uint8_t*, const float*, size_t);
static float g_f16_lut[65536];
static int g_lut_ready;

static float f16_bits_to_f32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 31u, m = h & 1023u, bits;
    if (e == 0) {
        if (m == 0) bits = sign;
        else {
            int sh = 0;
            while (!(m & 1024u)) { m <<= 1; sh++; }
            bits = sign | ((uint32_t)(113 - sh) << 23) | ((m & 1023u) << 13);
        }
    } else if (e == 31) bits = sign | 0x7f800000u | (m << 13);
    else bits = sign | ((e + 112u) << 23) | (m << 13);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* One row: G blocks of 18 bytes against x[32*G].  SIMD lanes run across the 16 (or 8) positions
 * of a half block; the block's products are summed per lane, scaled by d with one FMA into a
 * per-lane running sum, lanes are folded at the end.  Three builds of the same loop, picked
 * once at run time. */
#include <immintrin.h>

__attribute__((target("avx512f,avx512bw,avx512vl")))
static float row_dot_avx512(const uint8_t* blocks, const float* x, size_t G)
{
    __m512 acc = _mm512_setzero_ps();
    const __m128i m4 = _mm_set1_epi8(15);
    const __m512i eight = _mm512_set1_epi32(8);
    for (size_t g = 0; g < G; g++) {
        const uint8_t* b = blocks + g * 18;
        const __m128i raw = _mm_loadu_si128((const __m128i*)(b + 2));
        const __m512 lo = _mm512_cvtepi32_ps(_mm512_sub_epi32(_mm512_cvtepu8_epi32(_mm_and_si128(raw, m4)), eight));
        const __m512 hi = _mm512_cvtepi32_ps(_mm512_sub_epi32(_mm512_cvtepu8_epi32(_mm_and_si128(_mm_srli_epi16(raw, 4), m4)), eight));
        __m512 t = _mm512_mul_ps(lo, _mm512_loadu_ps(x + g * 32));
        t = _mm512_fmadd_ps(hi, _mm512_loadu_ps(x + g * 32 + 16), t);
        acc = _mm512_fmadd_ps(_mm512_set1_ps(g_f16_lut[(uint16_t)(b[0] | (b[1] << 8))]), t, acc);
    }
    return _mm512_reduce_add_ps(acc);
}

__attribute__((target("avx2,fma")))
static float row_dot_avx2(const uint8_t* blocks, const float* x, size_t G)
{
    __m256 acc = _mm256_setzero_ps();
    const __m128i m4 = _mm_set1_epi8(15);
    const __m256i eight = _mm256_set1_epi32(8);
    for (size_t g = 0; g < G; g++) {
        const uint8_t* b = blocks + g * 18;
        const __m128i raw = _mm_loadu_si128((const __m128i*)(b + 2));
        const __m128i lo8 = _mm_and_si128(raw, m4), hi8 = _mm_and_si128(_mm_srli_epi16(raw, 4), m4);
        const float* xg = x + g * 32;
        __m256 t = _mm256_mul_ps(_mm256_cvtepi32_ps(_mm256_sub_epi32(_mm256_cvtepu8_epi32(lo8), eight)), _mm256_loadu_ps(xg));
        t = _mm256_fmadd_ps(_mm256_cvtepi32_ps(_mm256_sub_epi32(_mm256_cvtepu8_epi32(_mm_srli_si128(lo8, 8)), eight)), _mm256_loadu_ps(xg + 8), t);
        t = _mm256_fmadd_ps(_mm256_cvtepi32_ps(_mm256_sub_epi32(_mm256_cvtepu8_epi32(hi8), eight)), _mm256_loadu_ps(xg + 16), t);
        t = _mm256_fmadd_ps(_mm256_cvtepi32_ps(_mm256_sub_epi32(_mm256_cvtepu8_epi32(_mm_srli_si128(hi8, 8)), eight)), _mm256_loadu_ps(xg + 24), t);
        acc = _mm256_fmadd_ps(_mm256_set1_ps(g_f16_lut[(uint16_t)(b[0] | (b[1] << 8))]), t, acc);
    }
    __m128 r = _mm_add_ps(_mm256_castps256_ps128(acc), _mm256_extractf128_ps(acc, 1));
    r = _mm_add_ps(r, _mm_movehl_ps(r, r));
    r = _mm_add_ss(r, _mm_shuffle_ps(r, r, 1));
    return _mm_cvtss_f32(r);
}

static float row_dot_plain(const uint8_t* blocks, const float* x, size_t G)
{
    float acc[32];
    for (int j = 0; j < 32; j++) acc[j] = 0.f;
    for (size_t g = 0; g < G; g++) {
        const uint8_t* b = blocks + g * 18;
        const float d = g_f16_lut[(uint16_t)(b[0] | (b[1] << 8))];
        const float* xg = x + g * 32;
        for (int j = 0; j < 16; j++) {
            acc[j] += d * (float)((int)(b[2 + j] & 15) - 8) * xg[j];
            acc[j + 16] += d * (float)((int)(b[2 + j] >> 4) - 8) * xg[j + 16];
        }
    }
    for (int h = 16; h >= 1; h >>= 1)
        for (int j = 0; j < h; j++) acc[j] += acc[j + h];
    return acc[0];
}



static row_dot_fn g_row_dot = row_dot_plain;
static const char* g_isa = "plain";

void cybq_cpu_baseline_init(void)
{
    if (g_lut_ready) return;
    for (uint32_t i = 0; i < 65536; i++) g_f16_lut[i] = f16_bits_to_f32((uint16_t)i);
    __builtin_cpu_init();
    if (__builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") && __builtin_cpu_supports("avx512vl")) {
        g_row_dot = row_dot_avx512;
        g_isa = "avx512";
    } else if (__builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma")) {
        g_row_dot = row_dot_avx2;
        g_isa = "avx2";
    }
    g_lut_ready = 1;
}

const char* cybq_cpu_baseline_isa(void)
{
    cybq_cpu_baseline_init();
    return g_isa;
}

/* y[M,N] = x[M,K] * W^T, W as N x (K/32) Q4_0 blocks.  Returns the number of threads used. */
int cybq_cpu_q4_0_matmul(const uint8_t* blocks, size_t N, size_t K, const float* x, size_t M, float* y, int threads)
{
    cybq_cpu_baseline_init();
    const size_t G = K / 32;
    if (threads < 1) threads = 1;
    int used = 1;
#pragma omp parallel num_threads(threads)
    {
#pragma omp single
        used = omp_get_num_threads();
#pragma omp for schedule(static)
        for (long n = 0; n < (long)N; n++) {
            const uint8_t* row = blocks + (size_t)n * G * 18;
            for (size_t m = 0; m < M; m++) y[m * N + (size_t)n] = g_row_dot(row, x + m * K, G);
        }
    }
    return used;
}
