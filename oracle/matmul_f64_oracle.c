/*
 * Oracle: native fp64 tier and reduced-precision tier.
 * TEST INFRASTRUCTURE ONLY - see eshkol_oracle.h.
 *
 * Compile with -ffp-contract=off: every fused multiply-add below is spelled
 * fma() so the rounding sequence does not depend on the optimiser.
 */
#include "eshkol_oracle.h"
#include <math.h>
#include <string.h>
#include <stdlib.h>

/* 1 (default): the reference built with -mavx2 -mfma (AVX 4x8 kernel, fused
 * multiply-add). 0: the reference's flag-less x86-64 build (SSE2 4x4 kernel,
 * blas_backend.cpp:669-763, multiply and add rounded separately). The loop
 * nest and accumulation order are the same in both. */
static int g_fused = 1;
void oracle_matmul_set_fused(int fused) { g_fused = fused ? 1 : 0; }

static inline double madd(double a, double b, double c) {
    if (g_fused) return fma(a, b, c);
    double p = a * b;
    return p + c;
}

/* blas_backend.cpp:407-419 (with -mfma, sum += a*b contracts to fma). */
void oracle_matmul_scalar_f64(const double* A, const double* B, double* C,
                              uint64_t M, uint64_t K, uint64_t N) {
    for (uint64_t i = 0; i < M; ++i)
        for (uint64_t j = 0; j < N; ++j) {
            double sum = 0.0;
            for (uint64_t k = 0; k < K; ++k)
                sum = madd(A[i * K + k], B[k * N + j], sum);
            C[i * N + j] = sum;
        }
}

/* blas_backend.cpp:616-658 with the 4x8 micro-kernel (550-598) and the scalar
 * edge block (601-614). Both accumulate one output over the k-block with fma
 * from 0.0 and then add into C, so one loop states both. */
void oracle_matmul_blocked_f64(const double* A, const double* B, double* C,
                               uint64_t M, uint64_t K, uint64_t N) {
    const uint64_t BLK = 64;
    memset(C, 0, (size_t)(M * N) * sizeof(double));
    for (uint64_t i0 = 0; i0 < M; i0 += BLK) {
        uint64_t mb = (M - i0 < BLK) ? M - i0 : BLK;
        for (uint64_t j0 = 0; j0 < N; j0 += BLK) {
            uint64_t nb = (N - j0 < BLK) ? N - j0 : BLK;
            for (uint64_t k0 = 0; k0 < K; k0 += BLK) {
                uint64_t kb = (K - k0 < BLK) ? K - k0 : BLK;
                for (uint64_t i = 0; i < mb; ++i) {
                    const double* arow = A + (i0 + i) * K + k0;
                    double acc[64];
                    for (uint64_t j = 0; j < nb; ++j) acc[j] = 0.0;
                    for (uint64_t k = 0; k < kb; ++k) {
                        const double a = arow[k];
                        const double* brow = B + (k0 + k) * N + j0;
                        for (uint64_t j = 0; j < nb; ++j)
                            acc[j] = madd(a, brow[j], acc[j]);
                    }
                    double* crow = C + (i0 + i) * N + j0;
                    for (uint64_t j = 0; j < nb; ++j) crow[j] += acc[j];
                }
            }
        }
    }
}

/* blas_backend.cpp:791-906, non-BLAS build (M*N < 1e9 always takes the SIMD path). */
void oracle_matmul_f64(const double* A, const double* B, double* C,
                       uint64_t M, uint64_t K, uint64_t N) {
    if (M * N <= 16) oracle_matmul_scalar_f64(A, B, C, M, K, N);
    else             oracle_matmul_blocked_f64(A, B, C, M, K, N);
}

/* runtime_tensor_math.cpp:796-817. C += a*b contracts to fma when the file is
 * built with -mfma and rounds twice in the flag-less build (same switch). */
void oracle_batch_matmul_f64(const double* a, const double* b, double* c,
                             int64_t batch, int64_t M, int64_t K, int64_t N) {
    for (int64_t bs = 0; bs < batch; bs++) {
        const double* A = a + bs * M * K;
        const double* B = b + bs * K * N;
        double*       C = c + bs * M * N;
        for (int64_t idx = 0; idx < M * N; idx++) C[idx] = 0.0;
        for (int64_t i = 0; i < M; i++)
            for (int64_t kk = 0; kk < K; kk++) {
                double a_ik = A[i * K + kk];
                for (int64_t j = 0; j < N; j++) {
                    C[i * N + j] = madd(a_ik, B[kk * N + j], C[i * N + j]);
                }
            }
    }
}

/* eshkol_matmul_backward_f64, blas_backend.cpp:924-1039, non-BLAS non-GPU
 * build: both the tiny-matrix branch (941-954) and the scalar fallback
 * (1029-1038) are the same two accumulation loops, n ascending for grad_A and
 * i ascending for grad_B, `+=` contracting to fma with -mfma. */
void oracle_matmul_backward_f64(const double* grad_out, const double* saved_A, const double* saved_B,
                                double* grad_A, double* grad_B,
                                uint64_t M, uint64_t K, uint64_t N) {
    memset(grad_A, 0, (size_t)(M * K) * sizeof(double));
    for (uint64_t i = 0; i < M; i++)
        for (uint64_t j = 0; j < K; j++)
            for (uint64_t n = 0; n < N; n++)
                grad_A[i * K + j] = madd(grad_out[i * N + n], saved_B[j * N + n], grad_A[i * K + j]);
    memset(grad_B, 0, (size_t)(K * N) * sizeof(double));
    for (uint64_t j = 0; j < K; j++)
        for (uint64_t n = 0; n < N; n++)
            for (uint64_t i = 0; i < M; i++)
                grad_B[j * N + n] = madd(saved_A[i * K + j], grad_out[i * N + n], grad_B[j * N + n]);
}

/* ---- reduced precision --------------------------------------------------- */

/* runtime_tensor_dtype.cpp:37-93 */
static double f64_to_f16_to_f64(double x) {
    float f = (float)x;
    uint32_t bits;
    memcpy(&bits, &f, sizeof bits);
    uint32_t sign = (bits >> 16) & 0x8000u;
    int32_t  e    = (int32_t)((bits >> 23) & 0xFFu) - 127;
    uint32_t mant = bits & 0x7FFFFFu;
    uint16_t h;
    if (((bits >> 23) & 0xFFu) == 0xFFu) {
        h = (uint16_t)(sign | 0x7C00u | (mant ? 0x0200u : 0u));
    } else if (e >= 16) {
        h = (uint16_t)(sign | 0x7C00u);
    } else if (e >= -14) {
        uint32_t hexp = (uint32_t)(e + 15);
        uint32_t hm = mant >> 13, rem = mant & 0x1FFFu;
        h = (uint16_t)(sign | (hexp << 10) | hm);
        if (rem > 0x1000u || (rem == 0x1000u && (hm & 1u))) h++;
    } else if (e >= -24) {
        mant |= 0x800000u;
        int32_t shift = -e - 1;
        uint32_t hm = mant >> (shift + 1);
        uint32_t rem = mant & ((1u << (shift + 1)) - 1u);
        uint32_t halfway = 1u << shift;
        h = (uint16_t)(sign | hm);
        if (rem > halfway || (rem == halfway && (hm & 1u))) h++;
    } else {
        h = (uint16_t)sign;
    }
    uint32_t hs = (h & 0x8000u) >> 15, he = (h & 0x7C00u) >> 10, hm = h & 0x03FFu;
    double sgn = hs ? -1.0 : 1.0;
    if (he == 0) {
        if (hm == 0) return sgn * 0.0;
        return sgn * ldexp((double)hm, -24);
    }
    if (he == 0x1F) return hm ? (x != x ? x : nan("")) : sgn * HUGE_VAL;
    return sgn * ldexp(1.0 + (double)hm / 1024.0, (int)he - 15);
}

/* runtime_tensor_dtype.cpp:97-109 */
static double f64_to_bf16_to_f64(double x) {
    float f = (float)x;
    uint32_t bits;
    memcpy(&bits, &f, sizeof bits);
    if (((bits >> 23) & 0xFFu) == 0xFFu) return (double)f;
    bits += 0x7FFFu + ((bits >> 16) & 1u);
    bits &= 0xFFFF0000u;
    memcpy(&f, &bits, sizeof f);
    return (double)f;
}

/* runtime_tensor_dtype.cpp:126-145 */
double oracle_reduce_precision(double v, int64_t dtype) {
    switch (dtype) {
        case 1: return (double)(float)v;
        case 2: return f64_to_f16_to_f64(v);
        case 3: return f64_to_bf16_to_f64(v);
        case 4: {
            if (!(v == v)) return 0.0;
            double r = nearbyint(v);
            if (r < -128.0) r = -128.0;
            if (r > 127.0) r = 127.0;
            return (double)(int8_t)r;
        }
        default: return v;
    }
}

void oracle_reduce_precision_array(const double* in, double* out, size_t n, int64_t dtype) {
    for (size_t i = 0; i < n; i++) out[i] = oracle_reduce_precision(in[i], dtype);
}

void oracle_matmul_reduced(const double* A, const double* B, double* C,
                           uint64_t M, uint64_t K, uint64_t N, int64_t dtype) {
    double* Ar = (double*)malloc((size_t)(M * K) * sizeof(double));
    double* Br = (double*)malloc((size_t)(K * N) * sizeof(double));
    oracle_reduce_precision_array(A, Ar, (size_t)(M * K), dtype);
    oracle_reduce_precision_array(B, Br, (size_t)(K * N), dtype);
    oracle_matmul_f64(Ar, Br, C, M, K, N);
    free(Ar); free(Br);
}

void oracle_matmul_reduced_f32acc(const double* A, const double* B, double* C,
                                  uint64_t M, uint64_t K, uint64_t N,
                                  int64_t dtype, int round_output) {
    float* Ar = (float*)malloc((size_t)(M * K) * sizeof(float));
    float* Bt = (float*)malloc((size_t)(K * N) * sizeof(float));
    for (uint64_t i = 0; i < M * K; i++) Ar[i] = (float)oracle_reduce_precision(A[i], dtype);
    for (uint64_t k = 0; k < K; k++)
        for (uint64_t j = 0; j < N; j++)
            Bt[j * K + k] = (float)oracle_reduce_precision(B[k * N + j], dtype);
    #pragma omp parallel for schedule(static)
    for (uint64_t i = 0; i < M; i++)
        for (uint64_t j = 0; j < N; j++) {
            float acc = 0.0f;
            const float* a = Ar + i * K;
            const float* b = Bt + j * K;
            for (uint64_t k = 0; k < K; k++) acc = fmaf(a[k], b[k], acc);
            double v = (double)acc;
            C[i * N + j] = round_output ? oracle_reduce_precision(v, dtype) : v;
        }
    free(Ar); free(Bt);
}
