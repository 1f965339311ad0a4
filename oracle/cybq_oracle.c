/*
 * cybq_oracle.c - CPU restatement of the block-quantized matmul path.
 * Test infrastructure only; see cybq_oracle.h for what it follows in the
 * reference tree and which functions are pinned by what.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math (see oracle/Makefile); the
 * f32 path must not be contracted into fused multiply-adds, its definition is
 * "round the product, then round the sum".
 */
#include "cybq_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#define G CYBQ_ORACLE_GROUP

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ------------------------------------------------------------------ f16 */

float cybq_oracle_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: man * 2^-24, exact in f32 */
        float v = (float)man * (1.0f / 16777216.0f);
        return sign ? -v : v;
    }
    if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t cybq_oracle_f32_to_f16(float f)
{
    uint32_t u = f32_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a >= 0x7f800000u) {                       /* inf / nan */
        if (a == 0x7f800000u) return (uint16_t)(sign | 0x7c00u);
        return (uint16_t)(sign | 0x7c00u | 0x200u | ((a >> 13) & 0x3ffu)); /* quiet nan */
    }
    if (a >= 0x477ff000u)                         /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    if (a < 0x33000001u)                          /* <= 2^-25 rounds to zero (tie to even) */
        return sign;
    int32_t e = (int32_t)(a >> 23) - 127;         /* unbiased exponent */
    uint32_t m = (a & 0x7fffffu) | 0x800000u;     /* 24-bit significand */
    uint32_t shift;                               /* bits dropped from m */
    uint32_t base;                                /* exponent field contribution */
    if (e < -14) { shift = (uint32_t)(13 + (-14 - e)); base = 0; }
    else         { shift = 13; base = (uint32_t)(e + 15) << 10; }
    uint32_t kept = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (kept & 1u))) kept++;
    /* normal: kept carries the hidden bit at 0x400; adding it to (e+14)<<10
     * makes a carry out of the mantissa bump the exponent for free. */
    uint32_t r = (e < -14) ? kept : (base - 0x400u + kept);
    return (uint16_t)(sign | r);
}

float cybq_oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

uint16_t cybq_oracle_f32_to_bf16(float f)
{
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

void cybq_oracle_f16_to_f32_n(const uint16_t* h, float* out, size_t n)
{ for (size_t i = 0; i < n; i++) out[i] = cybq_oracle_f16_to_f32(h[i]); }
void cybq_oracle_f32_to_f16_n(const float* f, uint16_t* out, size_t n)
{ for (size_t i = 0; i < n; i++) out[i] = cybq_oracle_f32_to_f16(f[i]); }
void cybq_oracle_bf16_to_f32_n(const uint16_t* h, float* out, size_t n)
{ for (size_t i = 0; i < n; i++) out[i] = cybq_oracle_bf16_to_f32(h[i]); }
void cybq_oracle_f32_to_bf16_n(const float* f, uint16_t* out, size_t n)
{ for (size_t i = 0; i < n; i++) out[i] = cybq_oracle_f32_to_bf16(f[i]); }

/* ------------------------------------------------------------- quantise */

static int bits_ok(int bits) { return bits == 4 || bits == 8; }

int cybq_oracle_quantize(int bits, const float* w, size_t N, size_t K,
                         int8_t* q, uint16_t* scales)
{
    if (!bits_ok(bits) || !w || !q || !scales || K % G) return -1;
    const float qmax = bits == 4 ? 7.0f : 127.0f;
    const float lo = bits == 4 ? -8.0f : -127.0f;
    const float hi = qmax;
    const size_t ng = K / G;
    for (size_t n = 0; n < N; n++) {
        for (size_t g = 0; g < ng; g++) {
            const float* src = w + n * K + g * G;
            int8_t* dst = q + n * K + g * G;
            float amax = 0.0f;
            for (int i = 0; i < G; i++) {
                float a = fabsf(src[i]);
                if (a > amax) amax = a;
            }
            uint16_t d16 = cybq_oracle_f32_to_f16(amax / qmax);
            if ((d16 & 0x7fffu) >= 0x7c00u) d16 = 0x7bffu;   /* saturate at 65504 */
            float d = cybq_oracle_f16_to_f32(d16);
            scales[n * ng + g] = d16;
            for (int i = 0; i < G; i++) {
                float r = 0.0f;
                if (d != 0.0f) {
                    r = roundf(src[i] / d);               /* half away from zero */
                    if (r < lo) r = lo;
                    if (r > hi) r = hi;
                }
                dst[i] = (int8_t)r;
            }
        }
    }
    return 0;
}

/* -------------------------------------------------------------- layouts */

int cybq_oracle_pack_planar(int bits, const int8_t* q, size_t N, size_t K, uint8_t* qplane)
{
    if (!bits_ok(bits) || !q || !qplane || K % G) return -1;
    if (bits == 8) { memcpy(qplane, q, N * K); return 0; }
    for (size_t i = 0; i < N * K / 2; i++)
        qplane[i] = (uint8_t)((q[2 * i] & 15) | ((q[2 * i + 1] & 15) << 4));
    return 0;
}

static inline int8_t sext4(uint8_t nib) { return (int8_t)((nib & 8) ? (int)nib - 16 : (int)nib); }

int cybq_oracle_unpack_planar(int bits, const uint8_t* qplane, size_t N, size_t K, int8_t* q)
{
    if (!bits_ok(bits) || !q || !qplane || K % G) return -1;
    if (bits == 8) { memcpy(q, qplane, N * K); return 0; }
    for (size_t i = 0; i < N * K / 2; i++) {
        q[2 * i] = sext4(qplane[i] & 15);
        q[2 * i + 1] = sext4(qplane[i] >> 4);
    }
    return 0;
}

int cybq_oracle_pack_blocks(int bits, const int8_t* q, const uint16_t* scales,
                            size_t N, size_t K, uint8_t* blocks)
{
    if (!bits_ok(bits) || !q || !scales || !blocks || K % G) return -1;
    const size_t nb = N * (K / G);
    const size_t bs = bits == 4 ? 18 : 34;
    for (size_t b = 0; b < nb; b++) {
        uint8_t* o = blocks + b * bs;
        const int8_t* s = q + b * G;
        o[0] = (uint8_t)(scales[b] & 0xff);
        o[1] = (uint8_t)(scales[b] >> 8);
        if (bits == 4) {
            for (int j = 0; j < 16; j++)
                o[2 + j] = (uint8_t)(((s[j] + 8) & 15) | (((s[j + 16] + 8) & 15) << 4));
        } else {
            memcpy(o + 2, s, G);
        }
    }
    return 0;
}

int cybq_oracle_unpack_blocks(int bits, const uint8_t* blocks, size_t N, size_t K,
                              int8_t* q, uint16_t* scales)
{
    if (!bits_ok(bits) || !q || !scales || !blocks || K % G) return -1;
    const size_t nb = N * (K / G);
    const size_t bs = bits == 4 ? 18 : 34;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t* o = blocks + b * bs;
        int8_t* s = q + b * G;
        scales[b] = (uint16_t)(o[0] | (o[1] << 8));
        if (bits == 4) {
            for (int j = 0; j < 16; j++) {
                s[j] = (int8_t)((o[2 + j] & 15) - 8);
                s[j + 16] = (int8_t)((o[2 + j] >> 4) - 8);
            }
        } else {
            memcpy(s, o + 2, G);
        }
    }
    return 0;
}

/* -------------------------------------------------------------- dequant */

int cybq_oracle_dequant(const int8_t* q, const uint16_t* scales, size_t N, size_t K, float* w)
{
    if (!q || !scales || !w || K % G) return -1;
    const size_t ng = K / G;
    for (size_t n = 0; n < N; n++)
        for (size_t g = 0; g < ng; g++) {
            float d = cybq_oracle_f16_to_f32(scales[n * ng + g]);
            for (int i = 0; i < G; i++)
                w[n * K + g * G + i] = d * (float)q[n * K + g * G + i];
        }
    return 0;
}

/* --------------------------------------------------------------- matmul */

int cybq_oracle_matmul_f32(const int8_t* q, const uint16_t* scales, size_t N, size_t K,
                           const float* x, size_t M, float* y)
{
    if (!q || !scales || !x || !y || K % G) return -1;
    const size_t ng = K / G;
    for (size_t n = 0; n < N; n++)
        for (size_t m = 0; m < M; m++) {
            float acc = 0.0f;
            for (size_t g = 0; g < ng; g++) {
                float d = cybq_oracle_f16_to_f32(scales[n * ng + g]);
                for (int i = 0; i < G; i++) {
                    size_t k = g * G + i;
                    float wv = d * (float)q[n * K + k];     /* exact */
                    float p = x[m * K + k] * wv;
                    acc = acc + p;
                }
            }
            y[m * N + n] = acc;
        }
    return 0;
}

int cybq_oracle_matmul_f64(const int8_t* q, const uint16_t* scales, size_t N, size_t K,
                           const float* x, size_t M, double* y)
{
    if (!q || !scales || !x || !y || K % G) return -1;
    const size_t ng = K / G;
    for (size_t n = 0; n < N; n++)
        for (size_t m = 0; m < M; m++) {
            double acc = 0.0;
            for (size_t g = 0; g < ng; g++) {
                double d = (double)cybq_oracle_f16_to_f32(scales[n * ng + g]);
                for (int i = 0; i < G; i++) {
                    size_t k = g * G + i;
                    acc += (double)x[m * K + k] * (d * (double)q[n * K + k]);
                }
            }
            y[m * N + n] = acc;
        }
    return 0;
}

struct mt_job {
    const int8_t* q; const uint16_t* scales; size_t K; const float* x; size_t M; size_t N;
    float* y; size_t n0, n1;
};

static void* mt_worker(void* arg)
{
    struct mt_job* j = (struct mt_job*)arg;
    const size_t K = j->K, ng = K / G;
    for (size_t n = j->n0; n < j->n1; n++) {
        const int8_t* qr = j->q + n * K;
        for (size_t m = 0; m < j->M; m++) {
            const float* xr = j->x + m * K;
            float acc = 0.0f;
            for (size_t g = 0; g < ng; g++) {
                float d = cybq_oracle_f16_to_f32(j->scales[n * ng + g]);
                float part[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                for (int i = 0; i < G; i += 8)
                    for (int l = 0; l < 8; l++)
                        part[l] += xr[g * G + i + l] * (float)qr[g * G + i + l];
                float s = ((part[0] + part[4]) + (part[1] + part[5])) +
                          ((part[2] + part[6]) + (part[3] + part[7]));
                acc += d * s;
            }
            j->y[m * j->N + n] = acc;
        }
    }
    return NULL;
}

int cybq_oracle_matmul_blocked_mt(const int8_t* q, const uint16_t* scales, size_t N, size_t K,
                                  const float* x, size_t M, float* y, int threads)
{
    if (!q || !scales || !x || !y || K % G || threads < 1) return -1;
    if ((size_t)threads > N) threads = (int)(N ? N : 1);
    struct mt_job* jobs = (struct mt_job*)calloc((size_t)threads, sizeof *jobs);
    pthread_t* tid = (pthread_t*)calloc((size_t)threads, sizeof *tid);
    if (!jobs || !tid) { free(jobs); free(tid); return -1; }
    size_t per = (N + (size_t)threads - 1) / (size_t)threads;
    int started = 0;
    for (int t = 0; t < threads; t++) {
        size_t n0 = (size_t)t * per, n1 = n0 + per;
        if (n0 >= N) break;
        if (n1 > N) n1 = N;
        jobs[t] = (struct mt_job){q, scales, K, x, M, N, y, n0, n1};
        if (t == threads - 1 || n1 == N) { mt_worker(&jobs[t]); tid[t] = 0; started = t; break; }
        if (pthread_create(&tid[t], NULL, mt_worker, &jobs[t]) != 0) {
            mt_worker(&jobs[t]); tid[t] = 0;
        }
        started = t;
    }
    for (int t = 0; t <= started; t++)
        if (tid[t]) pthread_join(tid[t], NULL);
    free(jobs); free(tid);
    return 0;
}

double cybq_oracle_rel_l2(const float* a, const double* b, size_t n)
{
    double num = 0.0, den = 0.0;
    for (size_t i = 0; i < n; i++) {
        double d = (double)a[i] - b[i];
        num += d * d;
        den += b[i] * b[i];
    }
    if (den == 0.0) return num == 0.0 ? 0.0 : INFINITY;
    return sqrt(num / den);
}
