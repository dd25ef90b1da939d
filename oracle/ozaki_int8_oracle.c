/*
 * Oracle: INT8 slice tier (Ootomo-Ozaki-Yokota base-128 slicing).
 * TEST INFRASTRUCTURE ONLY - see eshkol_oracle.h.
 *
 * The reference has no CPU implementation of this tier; these functions restate
 * its device kernels (lib/backend/gpu/gpu_cuda_kernels.cu:663-741) and the host
 * orchestration (lib/backend/gpu/gpu_memory_cuda.cpp:339-452) in C.
 * Compile with -ffp-contract=off: the device kernels' `res -= a`, `acc += w*g`
 * are stated unfused here because w*g is a power of two times an int32 (exact),
 * so fusing cannot change the result, and res*128 is exact.
 */
#include "eshkol_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* gpu_cuda_kernels.cu:664-673 */
void oracle_ozaki_rowmax_f64(const double* A, uint64_t M, uint64_t K, double* rmax) {
    for (uint64_t i = 0; i < M; i++) {
        double m = 0.0;
        const double* row = A + i * K;
        for (uint64_t k = 0; k < K; k++) { double v = fabs(row[k]); if (v > m) m = v; }
        rmax[i] = (m > 0.0) ? m : 1.0;
    }
}

/* gpu_cuda_kernels.cu:676-684 */
void oracle_ozaki_colmax_f64(const double* B, uint64_t K, uint64_t N, double* cmax) {
    for (uint64_t j = 0; j < N; j++) {
        double m = 0.0;
        for (uint64_t k = 0; k < K; k++) { double v = fabs(B[k * N + j]); if (v > m) m = v; }
        cmax[j] = (m > 0.0) ? m : 1.0;
    }
}

/* gpu_cuda_kernels.cu:694-701: shared by both operands. */
static inline void slice_value(double res, int s, int8_t* out, uint64_t stride) {
    for (int p = 0; p < s; p++) {
        res *= 128.0;
        double a = rint(res);
        if (a > 127.0) a = 127.0; else if (a < -127.0) a = -127.0;
        out[(uint64_t)p * stride] = (int8_t)a;
        res -= a;
    }
}

/* gpu_cuda_kernels.cu:688-703 */
void oracle_ozaki_split_a_f64(const double* A, uint64_t M, uint64_t K,
                              const double* rmax, int s, int8_t* slices) {
    uint64_t tot = M * K;
    for (uint64_t idx = 0; idx < tot; idx++) {
        uint64_t i = idx / K;
        slice_value(A[idx] / rmax[i], s, slices + idx, tot);
    }
}

/* gpu_cuda_kernels.cu:707-723 */
void oracle_ozaki_split_b_f64(const double* B, uint64_t K, uint64_t N,
                              const double* cmax, int s, int8_t* slices) {
    uint64_t tot = K * N;
    for (uint64_t idx = 0; idx < tot; idx++) {
        uint64_t k = idx / N, j = idx % N;
        slice_value(B[idx] / cmax[j], s, slices + (k + j * K), tot);
    }
}

/* gpu_memory_cuda.cpp:353,363-389 */
int oracle_ozaki_int8_plan(uint64_t K, int T, int max_buf, int max_pairs,
                           double* weights, int* buf_first,
                           int* pair_p, int* pair_q) {
    if (K > 133000) return -1;
    const int s = T + 1;
    long long cap = (long long)(2147483647.0 / ((double)K * 16129.0));
    if (cap < 1) return -1;
    int nbuf = 0, npairs = 0;
    for (int d = 0; d <= T; d++) {
        int ps_p[64], ps_q[64], n = 0;
        for (int p = 0; p < s; p++) { int q = d - p; if (q >= 0 && q < s) { ps_p[n] = p; ps_q[n] = q; n++; } }
        double w = pow(2.0, -7.0 * (d + 2));
        for (long long off = 0; off < n; off += cap) {
            if (nbuf >= max_buf) return -1;
            weights[nbuf] = w;
            buf_first[nbuf] = npairs;
            for (long long t = off; t < n && t < off + cap; t++) {
                if (npairs >= max_pairs) return -1;
                pair_p[npairs] = ps_p[t]; pair_q[npairs] = ps_q[t]; npairs++;
            }
            nbuf++;
        }
    }
    buf_first[nbuf] = npairs;
    return nbuf;
}

/* gpu_memory_cuda.cpp:415-434: exact integer sums (int64 here, stored as int32;
 * the plan guarantees they fit). */
void oracle_ozaki_int8_products(const int8_t* As, const int8_t* Bs,
                                uint64_t M, uint64_t K, uint64_t N,
                                int nbuf, const int* buf_first,
                                const int* pair_p, const int* pair_q,
                                int32_t* Gall) {
    const uint64_t totA = M * K, totB = K * N, totC = M * N;
    for (int b = 0; b < nbuf; b++) {
        int32_t* G = Gall + (uint64_t)b * totC;
        #pragma omp parallel for schedule(static)
        for (uint64_t i = 0; i < M; i++)
            for (uint64_t j = 0; j < N; j++) {
                int64_t acc = 0;
                for (int t = buf_first[b]; t < buf_first[b + 1]; t++) {
                    const int8_t* a = As + (uint64_t)pair_p[t] * totA + i * K;
                    const int8_t* bb = Bs + (uint64_t)pair_q[t] * totB + j * K;
                    int32_t part = 0;
                    for (uint64_t k = 0; k < K; k++) part += (int32_t)a[k] * (int32_t)bb[k];
                    acc += part;
                }
                G[i * N + j] = (int32_t)acc;
            }
    }
}

/* gpu_cuda_kernels.cu:728-741 */
void oracle_ozaki_reconstruct_f64(double* C, const int32_t* Gall,
                                  const double* weights, int nbuf,
                                  const double* rmax, const double* cmax,
                                  uint64_t M, uint64_t N) {
    uint64_t tot = M * N;
    for (uint64_t idx = 0; idx < tot; idx++) {
        uint64_t i = idx / N, j = idx % N;
        double acc = 0.0;
        for (int b = 0; b < nbuf; b++) {
            double term = weights[b] * (double)Gall[(uint64_t)b * tot + idx];
            acc = acc + term;
        }
        double t = acc * rmax[i];
        C[idx] = t * cmax[j];
    }
}

/* gpu_memory_cuda.cpp:339-452 */
int oracle_matmul_ozaki_int8_f64(const double* A, const double* B, double* C,
                                 uint64_t M, uint64_t K, uint64_t N, int T) {
    if (!A || !B || !C || M == 0 || K == 0 || N == 0) return -1;
    if (M > 0x7fffffffULL || K > 0x7fffffffULL || N > 0x7fffffffULL) return -1;
    if (T < 1 || T > 8) return -1;
    double weights[128]; int buf_first[129], pp[128], pq[128];
    int nbuf = oracle_ozaki_int8_plan(K, T, 128, 128, weights, buf_first, pp, pq);
    if (nbuf < 0) return -1;
    const int s = T + 1;
    int8_t* As = (int8_t*)malloc((size_t)s * M * K);
    int8_t* Bs = (int8_t*)malloc((size_t)s * K * N);
    int32_t* G = (int32_t*)malloc((size_t)nbuf * M * N * sizeof(int32_t));
    double* r = (double*)malloc((size_t)M * sizeof(double));
    double* c = (double*)malloc((size_t)N * sizeof(double));
    int rc = -1;
    if (As && Bs && G && r && c) {
        oracle_ozaki_rowmax_f64(A, M, K, r);
        oracle_ozaki_colmax_f64(B, K, N, c);
        oracle_ozaki_split_a_f64(A, M, K, r, s, As);
        oracle_ozaki_split_b_f64(B, K, N, c, s, Bs);
        oracle_ozaki_int8_products(As, Bs, M, K, N, nbuf, buf_first, pp, pq, G);
        oracle_ozaki_reconstruct_f64(C, G, weights, nbuf, r, c, M, N);
        rc = 0;
    }
    free(As); free(Bs); free(G); free(r); free(c);
    return rc;
}
