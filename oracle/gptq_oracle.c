/*
 * CPU oracle for the GPTQ int3/int4 QuantLinear path, in plain C.
 * TEST INFRASTRUCTURE ONLY: it is the checker the HIP kernels are compared
 * with (and a single-thread CPU timing), never part of the product path.
 *
 * It restates auto_gptq/nn_modules/qlinear.py of the reference:
 *   oracle_unpack_rows  : 198-240 (shift table :62-70, straddling codes :233-234)
 *   oracle_unpack_zeros : 202-209, 217-227 (same layout along N, then +1)
 *   oracle_dequant      : 242  W = scales[g_idx[k]] * (q - zero[g_idx[k]]), fp16, one rounding
 *   oracle_forward      : 243-245  y = x @ W (+ bias); accumulated in double here, returned as float
 *
 * fp16 values travel as uint16_t bit patterns; the conversions below are
 * written out by hand so nothing depends on compiler half support.
 *
 * Pinned by tests/test_oracle.py against the closed-form bit stream and the
 * numpy/torch restatement in oracle/gptq_oracle.py.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static float half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while ((man & 0x400u) == 0);
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* round-to-nearest-even float -> half */
static uint16_t float_to_half(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((absx > 0x7f800000u) ? 0x200u : 0));
    }
    if (absx >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absx < 0x33000001u) { /* below half of the smallest subnormal */
        return (uint16_t)sign;
    }
    int32_t exp = (int32_t)(absx >> 23) - 127;
    uint32_t man = (absx & 0x7fffffu) | 0x800000u;
    uint32_t shift;
    uint32_t base;
    if (exp < -14) { /* subnormal result */
        shift = (uint32_t)(13 + (-14 - exp));
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(exp + 15) << 10;
        man &= 0x7fffffu;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) {
        q++;
    }
    return (uint16_t)(sign | (base + q)); /* a mantissa carry walks into the exponent */
}

uint16_t oracle_float_to_half(float f) { return float_to_half(f); }
float oracle_half_to_float(uint16_t h) { return half_to_float(h); }

static const int WF3[3][12] = {
    {0, 3, 6, 9, 12, 15, 18, 21, 24, 27, 30, 0},
    {0, 1, 4, 7, 10, 13, 16, 19, 22, 25, 28, 31},
    {0, 2, 5, 8, 11, 14, 17, 20, 23, 26, 29, 0},
};

/* 32 codes out of three words, the way the reference's table does it */
static void unpack3_block(int32_t w0, int32_t w1, int32_t w2, int32_t out[32])
{
    int32_t t[3][12];
    const int32_t w[3] = {w0, w1, w2};
    for (int r = 0; r < 3; r++) {
        for (int c = 0; c < 12; c++) {
            t[r][c] = (w[r] >> WF3[r][c]) & 0x7; /* arithmetic shift, then mask */
        }
    }
    t[0][10] = (t[0][10] & 0x3) | ((t[1][0] << 2) & 0x4);
    t[1][11] = (t[1][11] & 0x1) | ((t[2][0] << 1) & 0x6);
    int o = 0;
    for (int c = 0; c < 11; c++) out[o++] = t[0][c] & 0x7;
    for (int c = 1; c < 12; c++) out[o++] = t[1][c] & 0x7;
    for (int c = 1; c < 11; c++) out[o++] = t[2][c] & 0x7;
}

/* qweight int32 [K/32*bits, N] -> codes int32 [K, N] */
int oracle_unpack_rows(const int32_t *qweight, int K, int N, int bits, int32_t *codes)
{
    if (bits == 2 || bits == 4 || bits == 8) {
        /* 32 / bits codes per word, code j at bit bits * j (qlinear.py:211-215) */
        const int per = 32 / bits;
        const int32_t mask = (1 << bits) - 1;
        for (int r = 0; r < K / per; r++) {
            for (int j = 0; j < per; j++) {
                for (int n = 0; n < N; n++) {
                    codes[(size_t)(per * r + j) * N + n] = (qweight[(size_t)r * N + n] >> (bits * j)) & mask;
                }
            }
        }
        return 0;
    }
    if (bits == 3) {
        int32_t blk[32];
        for (int r = 0; r < K / 32; r++) {
            for (int n = 0; n < N; n++) {
                unpack3_block(qweight[(size_t)(3 * r) * N + n], qweight[(size_t)(3 * r + 1) * N + n],
                              qweight[(size_t)(3 * r + 2) * N + n], blk);
                for (int j = 0; j < 32; j++) {
                    codes[(size_t)(32 * r + j) * N + n] = blk[j];
                }
            }
        }
        return 0;
    }
    return -1;
}

/* qzeros int32 [G, N/32*bits] -> zero points int32 [G, N], already +1 */
int oracle_unpack_zeros(const int32_t *qzeros, int G, int N, int bits, int32_t *zeros)
{
    const int words = N / 32 * bits;
    if (bits == 2 || bits == 4 || bits == 8) {
        const int per = 32 / bits;
        const int32_t mask = (1 << bits) - 1;
        for (int g = 0; g < G; g++) {
            for (int n = 0; n < N; n++) {
                zeros[(size_t)g * N + n] = ((qzeros[(size_t)g * words + n / per] >> (bits * (n % per))) & mask) + 1;
            }
        }
        return 0;
    }
    if (bits == 3) {
        int32_t blk[32];
        for (int g = 0; g < G; g++) {
            for (int b = 0; b < N / 32; b++) {
                const int32_t *w = qzeros + (size_t)g * words + 3 * b;
                unpack3_block(w[0], w[1], w[2], blk);
                for (int j = 0; j < 32; j++) {
                    zeros[(size_t)g * N + 32 * b + j] = blk[j] + 1;
                }
            }
        }
        return 0;
    }
    return -1;
}

/* W fp16 bits [K, N] */
int oracle_dequant(const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales, const int32_t *g_idx,
                   int K, int N, int G, int bits, uint16_t *W)
{
    int32_t *codes = (int32_t *)malloc((size_t)K * N * sizeof(int32_t));
    int32_t *zeros = (int32_t *)malloc((size_t)G * N * sizeof(int32_t));
    if (!codes || !zeros) {
        free(codes);
        free(zeros);
        return -2;
    }
    int rc = oracle_unpack_rows(qweight, K, N, bits, codes);
    if (rc == 0) rc = oracle_unpack_zeros(qzeros, G, N, bits, zeros);
    if (rc == 0) {
        for (int k = 0; k < K; k++) {
            const int g = g_idx[k];
            if (g < 0 || g >= G) {
                rc = -3;
                break;
            }
            for (int n = 0; n < N; n++) {
                /* scale (11 significant bits) times an integer of magnitude <= 256 is exact in
                 * float, so one rounding to half equals the reference's fp16 multiply */
                const float s = half_to_float(scales[(size_t)g * N + n]);
                const float d = (float)(codes[(size_t)k * N + n] - zeros[(size_t)g * N + n]);
                W[(size_t)k * N + n] = float_to_half(s * d);
            }
        }
    }
    free(codes);
    free(zeros);
    return rc;
}

/* y float [M, N] = x[M, K] @ W[K, N] (+ bias), accumulated in double */
int oracle_forward(const uint16_t *x, const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales,
                   const int32_t *g_idx, const uint16_t *bias, int M, int K, int N, int G, int bits, float *y)
{
    uint16_t *W = (uint16_t *)malloc((size_t)K * N * sizeof(uint16_t));
    double *acc = (double *)malloc((size_t)N * sizeof(double));
    if (!W || !acc) {
        free(W);
        free(acc);
        return -2;
    }
    int rc = oracle_dequant(qweight, qzeros, scales, g_idx, K, N, G, bits, W);
    if (rc == 0) {
        for (int m = 0; m < M; m++) {
            for (int n = 0; n < N; n++) acc[n] = 0.0;
            for (int k = 0; k < K; k++) {
                const double xv = (double)half_to_float(x[(size_t)m * K + k]);
                const uint16_t *wr = W + (size_t)k * N;
                for (int n = 0; n < N; n++) acc[n] += xv * (double)half_to_float(wr[n]);
            }
            for (int n = 0; n < N; n++) {
                double v = acc[n];
                if (bias) v += (double)half_to_float(bias[n]);
                y[(size_t)m * N + n] = (float)v;
            }
        }
    }
    free(W);
    free(acc);
    return rc;
}
