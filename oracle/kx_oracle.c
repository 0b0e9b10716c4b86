/*
 * CPU oracle: see kx_oracle.h for scope, layout and pin status.
 * TEST INFRASTRUCTURE ONLY - never linked into the shipped library.
 *
 * Style follows the reference's CPU kernels (single thread, raw pointers, no stream:
 * kuiper/source/op/kernel/cpu/add_kernel.cpp:5-26); the arithmetic follows the closed
 * form w = (q - z) * s, for which the reference holds no code
 * (kuiper/include/op/matmul.h:7-9 is empty).
 */
#include "kx_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

static const int KXO_ORDER[8] = {0, 2, 4, 6, 1, 3, 5, 7};

/* ------------------------------------------------------------------ conversions */

static inline uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

static inline float bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

uint16_t kxo_f32_to_bf16(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        /* NaN: keep the sign and the top payload bits, force the quiet bit */
        return (uint16_t)((u >> 16) | 0x0040u);
    }
    /* round to nearest, ties to even on bit 16 */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

float kxo_bf16_to_f32(uint16_t h) {
    return bits_f32((uint32_t)h << 16);
}

float kxo_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) {
            return bits_f32(sign);
        }
        /* subnormal: man * 2^-24, exact in fp32 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    if (exp == 31) {
        return bits_f32(sign | 0x7f800000u | (man << 13));
    }
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t kxo_f32_to_f16(float f) {
    uint32_t u = f32_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) {
        return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x3ffu)); /* quiet NaN */
    }
    if (a >= 0x47800000u) {
        /* |f| >= 65536: infinity. Values in [65520, 65536) are handled by the rounding below. */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (a < 0x38800000u) {
        /* below the smallest normal half (2^-14): the result is a multiple of 2^-24 */
        if (a < 0x33000000u) {
            return sign; /* < 2^-25 rounds to zero (2^-25 itself ties to even = 0) */
        }
        int e = (int)(a >> 23);              /* biased fp32 exponent, 102..112 */
        uint32_t m = (a & 0x7fffffu) | 0x800000u; /* 24-bit significand */
        int shift = 126 - e;                 /* bits to drop so that the unit is 2^-24 */
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) {
            q++;
        }
        return (uint16_t)(sign | q); /* q == 0x400 lands on the smallest normal, as it should */
    }
    /* normal range: re-bias and round the 13 dropped bits to nearest even */
    uint32_t v = a - 0x38000000u;
    uint32_t lsb = (v >> 13) & 1u;
    v += 0xfffu + lsb;
    v >>= 13;
    if (v >= 0x7c00u) {
        v = 0x7c00u; /* rounded up to infinity */
    }
    return (uint16_t)(sign | v);
}

void kxo_f32_to_bf16_n(const float* src, uint16_t* dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = kxo_f32_to_bf16(src[i]);
}
void kxo_bf16_to_f32_n(const uint16_t* src, float* dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = kxo_bf16_to_f32(src[i]);
}
void kxo_f32_to_f16_n(const float* src, uint16_t* dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = kxo_f32_to_f16(src[i]);
}
void kxo_f16_to_f32_n(const uint16_t* src, float* dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = kxo_f16_to_f32(src[i]);
}

/* ------------------------------------------------------------------ nibble stream */

int kxo_awq_pack(const uint8_t* codes, int64_t rows, int64_t cols, int32_t* words) {
    if (rows < 0 || cols < 0 || (cols % 8) != 0) return 1;
    int64_t wcols = cols / 8;
    for (int64_t r = 0; r < rows; r++) {
        for (int64_t j = 0; j < wcols; j++) {
            uint32_t w = 0;
            for (int i = 0; i < 8; i++) {
                uint32_t c = codes[r * cols + 8 * j + KXO_ORDER[i]];
                if (c > 15u) return 2;
                w |= c << (4 * i);
            }
            words[r * wcols + j] = (int32_t)w;
        }
    }
    return 0;
}

int kxo_awq_unpack(const int32_t* words, int64_t rows, int64_t cols, uint8_t* codes) {
    if (rows < 0 || cols < 0 || (cols % 8) != 0) return 1;
    int64_t wcols = cols / 8;
    for (int64_t r = 0; r < rows; r++) {
        for (int64_t j = 0; j < wcols; j++) {
            uint32_t w = (uint32_t)words[r * wcols + j];
            for (int i = 0; i < 8; i++) {
                codes[r * cols + 8 * j + KXO_ORDER[i]] = (uint8_t)((w >> (4 * i)) & 0xfu);
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ dequant */

uint16_t kxo_awq_dequant_one(uint32_t q, uint32_t z, uint16_t scale_f16) {
    /* (q - z) is an integer in [-15, 15]; its product with an 11-bit significand is exact in
     * fp32 (fp16 subnormal scales included), so one rounding happens, at the bf16 store. */
    float d = (float)((int)(q & 0xfu) - (int)(z & 0xfu));
    float s = kxo_f16_to_f32(scale_f16);
    return kxo_f32_to_bf16(d * s);
}

int kxo_awq_dequant_bf16(const int32_t* qweight, const uint16_t* scales_f16, const int32_t* qzeros,
                         int64_t K, int64_t N, int64_t group, uint16_t* w_bf16) {
    if (group <= 0 || (K % group) != 0 || (N % 8) != 0) return 1;
    int64_t wcols = N / 8;
    for (int64_t k = 0; k < K; k++) {
        int64_t g = k / group;
        for (int64_t j = 0; j < wcols; j++) {
            uint32_t qw = (uint32_t)qweight[k * wcols + j];
            uint32_t zw = (uint32_t)qzeros[g * wcols + j];
            for (int i = 0; i < 8; i++) {
                int64_t n = 8 * j + KXO_ORDER[i];
                w_bf16[k * N + n] = kxo_awq_dequant_one((qw >> (4 * i)) & 0xfu,
                                                        (zw >> (4 * i)) & 0xfu,
                                                        scales_f16[g * N + n]);
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ AWQ GEMV */

int kxo_gemv_awq_f64(const uint16_t* x_bf16, const int32_t* qweight, const uint16_t* scales_f16,
                     const int32_t* qzeros, int64_t M, int64_t K, int64_t N, int64_t group,
                     double* y_f64) {
    if (group <= 0 || (K % group) != 0 || (N % 8) != 0) return 1;
    int64_t wcols = N / 8;
    uint8_t* qrow = (uint8_t*)malloc((size_t)N);
    uint8_t* zrow = (uint8_t*)malloc((size_t)N);
    if (!qrow || !zrow) {
        free(qrow);
        free(zrow);
        return 3;
    }
    for (int64_t i = 0; i < M * N; i++) y_f64[i] = 0.0;
    for (int64_t k = 0; k < K; k++) {
        int64_t g = k / group;
        kxo_awq_unpack(qweight + k * wcols, 1, N, qrow);
        if (k % group == 0) {
            kxo_awq_unpack(qzeros + g * wcols, 1, N, zrow);
        }
        for (int64_t m = 0; m < M; m++) {
            double xv = (double)kxo_bf16_to_f32(x_bf16[m * K + k]);
            double* y = y_f64 + m * N;
            for (int64_t n = 0; n < N; n++) {
                double w = (double)((int)qrow[n] - (int)zrow[n]) *
                           (double)kxo_f16_to_f32(scales_f16[g * N + n]);
                y[n] += xv * w;
            }
        }
    }
    free(qrow);
    free(zrow);
    return 0;
}

/* word columns [j_begin, j_end) of the fp32 evaluation; the arithmetic of a column does not depend
 * on the range it is computed in */
int kxo_gemv_awq_f32_range(const uint16_t* x_bf16, const int32_t* qweight, const uint16_t* scales_f16,
                           const int32_t* qzeros, int64_t M, int64_t K, int64_t N, int64_t group,
                           int64_t j_begin, int64_t j_end, uint16_t* y_bf16) {
    if (group <= 0 || (K % group) != 0 || (N % 8) != 0) return 1;
    int64_t wcols = N / 8;
    int64_t groups = K / group;
    if (j_begin < 0 || j_end > wcols || j_begin > j_end) return 1;
    float* acc = (float*)malloc((size_t)N * sizeof(float));
    float* sg = (float*)malloc((size_t)N * sizeof(float));
    float* zg = (float*)malloc((size_t)N * sizeof(float));
    if (!acc || !sg || !zg) {
        free(acc);
        free(sg);
        free(zg);
        return 3;
    }
    for (int64_t m = 0; m < M; m++) {
        for (int64_t n = 8 * j_begin; n < 8 * j_end; n++) acc[n] = 0.0f;
        for (int64_t g = 0; g < groups; g++) {
            /* per-group scales and zero points, unpacked once */
            for (int64_t j = j_begin; j < j_end; j++) {
                uint32_t zw = (uint32_t)qzeros[g * wcols + j];
                for (int i = 0; i < 8; i++) {
                    int64_t n = 8 * j + KXO_ORDER[i];
                    zg[n] = (float)((zw >> (4 * i)) & 0xfu);
                    sg[n] = kxo_f16_to_f32(scales_f16[g * N + n]);
                }
            }
            for (int64_t k = g * group; k < (g + 1) * group; k++) {
                float xv = kxo_bf16_to_f32(x_bf16[m * K + k]);
                const int32_t* row = qweight + k * wcols;
                for (int64_t j = j_begin; j < j_end; j++) {
                    uint32_t qw = (uint32_t)row[j];
                    for (int i = 0; i < 8; i++) {
                        int64_t n = 8 * j + KXO_ORDER[i];
                        float w = ((float)((qw >> (4 * i)) & 0xfu) - zg[n]) * sg[n];
                        acc[n] += xv * w;
                    }
                }
            }
        }
        for (int64_t n = 8 * j_begin; n < 8 * j_end; n++) y_bf16[m * N + n] = kxo_f32_to_bf16(acc[n]);
    }
    free(acc);
    free(sg);
    free(zg);
    return 0;
}

int kxo_gemv_awq_f32(const uint16_t* x_bf16, const int32_t* qweight, const uint16_t* scales_f16,
                     const int32_t* qzeros, int64_t M, int64_t K, int64_t N, int64_t group,
                     uint16_t* y_bf16) {
    if ((N % 8) != 0) return 1;
    return kxo_gemv_awq_f32_range(x_bf16, qweight, scales_f16, qzeros, M, K, N, group, 0, N / 8, y_bf16);
}

/* ------------------------------------------------------------------ BF16 GEMV */

int kxo_gemv_bf16_f64(const uint16_t* x_bf16, const uint16_t* w_bf16, int64_t M, int64_t K,
                      int64_t N, double* y_f64) {
    for (int64_t m = 0; m < M; m++) {
        for (int64_t n = 0; n < N; n++) {
            double s = 0.0;
            const uint16_t* wr = w_bf16 + n * K;
            const uint16_t* xr = x_bf16 + m * K;
            for (int64_t k = 0; k < K; k++) {
                s += (double)kxo_bf16_to_f32(xr[k]) * (double)kxo_bf16_to_f32(wr[k]);
            }
            y_f64[m * N + n] = s;
        }
    }
    return 0;
}

int kxo_gemv_bf16_f32(const uint16_t* x_bf16, const uint16_t* w_bf16, int64_t M, int64_t K,
                      int64_t N, uint16_t* y_bf16) {
    for (int64_t m = 0; m < M; m++) {
        for (int64_t n = 0; n < N; n++) {
            float s = 0.0f;
            const uint16_t* wr = w_bf16 + n * K;
            const uint16_t* xr = x_bf16 + m * K;
            for (int64_t k = 0; k < K; k++) {
                s += kxo_bf16_to_f32(xr[k]) * kxo_bf16_to_f32(wr[k]);
            }
            y_bf16[m * N + n] = kxo_f32_to_bf16(s);
        }
    }
    return 0;
}
