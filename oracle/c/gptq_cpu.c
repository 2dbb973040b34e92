/*
 * CPU restatement, in plain C, of the reference's GPTQ quantized linear:
 * TEST INFRASTRUCTURE ONLY -- it is the checker and the timed CPU baseline,
 * never part of the product path.
 *
 *   W[k, n] = fp16( (q[k, n] - (z[g, n] + 1)) * s[g, n] ),  g = g_idx[k]
 *             (minit/quantize/dispatch.py:14-20, computed in fp16)
 *   y[m, n] = fp16( sum_k x[m, k] * W[k, n] )
 *             (minit/quantize/dispatch.py:8-11; fp32-or-better accumulate,
 *              one rounding: minit/cuda/kernel/cublas.py:116-127)
 * with the sub-word layout of examples/qwen1_5_int8.py:97-138: sub-word i of a
 * 32-bit word at bit i * bits, qweight packed along K, qzeros along N.
 *
 * Accumulation is in double so the result is the correctly rounded fp16 of the
 * exact sum up to double round-off, like the numpy oracle (oracle/gptq.py).
 * Parallelised over output columns with OpenMP.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1Fu;
    const uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: man * 2^-24 */
            float f = (float)man * 5.9604644775390625e-08f;
            memcpy(&bits, &f, 4);
            bits |= sign;
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

/* round-to-nearest-even double -> binary16 */
static uint16_t double_to_half(double v) {
    uint16_t sign = 0;
    if (signbit(v)) {
        sign = 0x8000u;
        v = -v;
    }
    if (isnan(v)) return (uint16_t)(sign | 0x7E00u);
    if (v >= 65520.0) return (uint16_t)(sign | 0x7C00u); /* rounds to inf */
    if (v < 6.103515625e-05) {                           /* subnormal or zero: units of 2^-24 */
        const double q = nearbyint(v * 16777216.0);
        return (uint16_t)(sign | (uint16_t)q);           /* q == 1024 is the smallest normal */
    }
    int e;
    const double m = frexp(v, &e); /* v = m * 2^e, m in [0.5, 1) */
    double q = nearbyint(m * 2048.0); /* 11 significant bits */
    if (q == 2048.0) {
        q = 1024.0;
        e += 1;
    }
    const int biased = e - 1 + 15;
    if (biased >= 31) return (uint16_t)(sign | 0x7C00u);
    return (uint16_t)(sign | (uint16_t)(biased << 10) | ((uint16_t)q & 0x3FFu));
}

int oracle_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* number of OpenMP threads of the following calls (the timed CPU baseline runs with all threads and with one) */
void oracle_set_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

uint16_t oracle_double_to_half(double v) { return double_to_half(v); }
float oracle_half_to_float(uint16_t h) { return half_to_float(h); }

/* out[k, n] fp16 bits */
void oracle_gptq_dequant(const int32_t* qweight, const int32_t* qzeros, const uint16_t* scales,
                         const int32_t* g_idx, uint16_t* out, int N, int K, int group_size, int bits) {
    const int P = 32 / bits;
    const uint32_t mask = (1u << bits) - 1u;
#pragma omp parallel for schedule(static)
    for (int k = 0; k < K; ++k) {
        const int g = g_idx ? g_idx[k] : k / group_size;
        const uint32_t* qrow = (const uint32_t*)qweight + (size_t)(k / P) * N;
        const int shift = (k % P) * bits;
        for (int n = 0; n < N; ++n) {
            const int q = (int)((qrow[n] >> shift) & mask);
            const int z = (int)((((const uint32_t*)qzeros)[(size_t)g * (N / P) + n / P] >> ((n % P) * bits)) & mask);
            /* integer part exact; one rounding at the multiply */
            const double w = (double)(q - (z + 1)) * (double)half_to_float(scales[(size_t)g * N + n]);
            out[(size_t)k * N + n] = double_to_half(w);
        }
    }
}

/* y[M, N] = x[M, K] @ dequant(W)[K, N]; all fp16 as raw bits */
void oracle_gptq_matmul(const uint16_t* x, const int32_t* qweight, const int32_t* qzeros,
                        const uint16_t* scales, const int32_t* g_idx, uint16_t* y, int M, int N, int K,
                        int group_size, int bits) {
    const int P = 32 / bits;
    const uint32_t mask = (1u << bits) - 1u;
    const int CB = 256; /* column block per task */
    const int nblocks = (N + CB - 1) / CB;
    float* xf = (float*)malloc((size_t)M * K * sizeof(float));
    for (size_t i = 0; i < (size_t)M * K; ++i) xf[i] = half_to_float(x[i]);
#pragma omp parallel for schedule(dynamic, 1)
    for (int blk = 0; blk < nblocks; ++blk) {
        const int n0 = blk * CB, n1 = n0 + CB < N ? n0 + CB : N;
        const int nb = n1 - n0;
        double* acc = (double*)calloc((size_t)M * nb, sizeof(double));
        float* w = (float*)malloc((size_t)nb * sizeof(float));
        for (int k = 0; k < K; ++k) {
            const int g = g_idx ? g_idx[k] : k / group_size;
            const uint32_t* qrow = (const uint32_t*)qweight + (size_t)(k / P) * N;
            const int shift = (k % P) * bits;
            for (int n = n0; n < n1; ++n) {
                const int q = (int)((qrow[n] >> shift) & mask);
                const int z = (int)((((const uint32_t*)qzeros)[(size_t)g * (N / P) + n / P] >> ((n % P) * bits)) & mask);
                const double wd = (double)(q - (z + 1)) * (double)half_to_float(scales[(size_t)g * N + n]);
                w[n - n0] = half_to_float(double_to_half(wd));
            }
            for (int m = 0; m < M; ++m) {
                const double xv = (double)xf[(size_t)m * K + k];
                double* a = acc + (size_t)m * nb;
                for (int j = 0; j < nb; ++j) a[j] += xv * (double)w[j];
            }
        }
        for (int m = 0; m < M; ++m)
            for (int j = 0; j < nb; ++j) y[(size_t)m * N + n0 + j] = double_to_half(acc[(size_t)m * nb + j]);
        free(acc);
        free(w);
    }
    free(xf);
}
