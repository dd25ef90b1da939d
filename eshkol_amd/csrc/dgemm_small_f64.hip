/*
 * fp64 products of matrices far smaller than a tile: at most 1024 outputs and operands
 * of a few kilobytes, one or a batch of them stored back to back (hip_dgemm_f64_batched, the
 * reference's cublasDgemmStridedBatched, lib/backend/gpu/gpu_memory_cuda.cpp:700-760,
 * and the same shapes through hip_dgemm_f64 / _ex).
 *
 * The tiled kernels give every matrix a workgroup and a 64 x 64 tile: 4096 products
 * of 8 x 8 x 8 took 53 us for 1.5 MB of operands and results, 100000 of them 1.2 ms.
 * Here a workgroup takes as many consecutive matrices as its 256 threads have
 * outputs for (at least one), copies their operands into LDS with coalesced loads
 * (the batch is contiguous in memory), and every thread sums one output element at
 * a time over k ascending: bound by HBM and by launch latency, not by tiles.
 */
#include "hip_common.h"
#include "kernels.h"

namespace {

constexpr int SMALL_LDS_BYTES = 48 * 1024;

__global__ __launch_bounds__(256)
void dgemm_small_batched_kernel(const double* __restrict__ A, const double* __restrict__ B, double* __restrict__ C,
                                int M, int K, int N, int ta, int tb, long batch, int G) {
    extern __shared__ __align__(16) double small_smem[];
    const int asz = M * K, bsz = K * N, csz = M * N;
    const long g0 = (long)blockIdx.x * G;
    const int ng = (int)((batch - g0 < G) ? batch - g0 : G);
    double* sA = small_smem;
    double* sB = small_smem + (size_t)G * asz;
    const int tid = (int)threadIdx.x;
    const double* gA = A + (size_t)g0 * asz;
    const double* gB = B + (size_t)g0 * bsz;
    for (int i = tid; i < ng * asz; i += 256) sA[i] = gA[i];
    for (int i = tid; i < ng * bsz; i += 256) sB[i] = gB[i];
    __syncthreads();
    double* gC = C + (size_t)g0 * csz;
    /* strides of op(A)(i, k) and op(B)(k, j) inside a matrix as stored */
    const int a_i = ta ? 1 : K, a_k = ta ? M : 1;
    const int b_k = tb ? 1 : N, b_j = tb ? K : 1;
    for (int e = tid; e < ng * csz; e += 256) {
        const int g = e / csz, r = e - g * csz;
        const int i = r / N, j = r - i * N;
        const double* a = sA + g * asz + i * a_i;
        const double* b = sB + g * bsz + j * b_j;
        double acc = 0.0;
        for (int k = 0; k < K; k++) acc = fma(a[k * a_k], b[k * b_k], acc);
        gC[e] = acc;
    }
}

/* One product with few outputs and a long k (1 x 6699 x 139, 13 x 6701 x 11): a single tile
 * would walk all of K in one workgroup (0.38 ms for the first of the two). Here workgroup
 * p takes k in [p kc, (p + 1) kc), copies its slices of both operands into LDS (op(A) as
 * sA[i][kk], op(B) as sB[kk][j], whatever form the caller holds them in), sums one output
 * per thread over its slice, and leaves part[p][i][j]; dgemm_small_sum_kernel adds the
 * pieces, p ascending. */
__global__ __launch_bounds__(256)
void dgemm_small_splitk_kernel(const double* __restrict__ A, const double* __restrict__ B,
                               int M, int K, int N, int ta, int tb, int kc, double* __restrict__ part) {
    extern __shared__ __align__(16) double small_smem[];
    const int k0 = (int)blockIdx.x * kc;
    const int nk = (K - k0 < kc) ? K - k0 : kc;
    const int pa = kc + 1;                        /* pitch of sA: rows of one k-slice land in different banks */
    double* sA = small_smem;
    double* sB = small_smem + (size_t)M * pa;
    const int tid = (int)threadIdx.x;
    if (ta) {                                     /* A is [K][M]: i contiguous */
        for (int e = tid; e < nk * M; e += 256) { const int kk = e / M, i = e - kk * M; sA[i * pa + kk] = A[(size_t)(k0 + kk) * M + i]; }
    } else {                                      /* A is [M][K]: k contiguous */
        for (int e = tid; e < M * nk; e += 256) { const int i = e / nk, kk = e - i * nk; sA[i * pa + kk] = A[(size_t)i * K + k0 + kk]; }
    }
    if (tb) {                                     /* B is [N][K]: k contiguous */
        for (int e = tid; e < N * nk; e += 256) { const int j = e / nk, kk = e - j * nk; sB[kk * N + j] = B[(size_t)j * K + k0 + kk]; }
    } else {                                      /* B is [K][N]: j contiguous */
        for (int e = tid; e < nk * N; e += 256) sB[e] = B[(size_t)k0 * N + e];
    }
    __syncthreads();
    double* out = part + (size_t)blockIdx.x * M * N;
    for (int e = tid; e < M * N; e += 256) {
        const int i = e / N, j = e - i * N;
        const double* a = sA + i * pa;
        const double* b = sB + j;
        double acc = 0.0;
        for (int kk = 0; kk < nk; kk++) acc = fma(a[kk], b[kk * N], acc);
        out[e] = acc;
    }
}

__global__ __launch_bounds__(256)
void dgemm_small_sum_kernel(const double* __restrict__ part, int pieces, int outputs, double* __restrict__ C) {
    const int e = (int)(blockIdx.x * 256 + threadIdx.x);
    if (e >= outputs) return;
    double r = 0.0;
    int p = 0;
    for (; p + 8 <= pieces; p += 8) {             /* eight loads in flight, added in order */
        double v[8];
#pragma unroll
        for (int q = 0; q < 8; q++) v[q] = part[(size_t)(p + q) * outputs + e];
#pragma unroll
        for (int q = 0; q < 8; q++) r += v[q];
    }
    for (; p < pieces; p++) r += part[(size_t)p * outputs + e];
    C[e] = r;
}

}  // namespace

/* One product of few outputs and a long k: eshkol_hip_dgemm_small_long_k takes it. */
bool eshkol_hip_dgemm_is_small_long_k(uint64_t M, uint64_t K, uint64_t N) {
    return M * N <= 1024 && M + N <= 256 && K >= 256 && K <= 0x7fffffffULL;
}

int eshkol_hip_dgemm_small_long_k(const double* A, const double* B, double* C, uint64_t M, uint64_t K, uint64_t N,
                                  int trans_a, int trans_b, hipStream_t st) {
    const int m = (int)M, k = (int)K, n = (int)N;
    /* slices of k: as long as 32 KiB of LDS hold (at least 16), at most 512, and enough of them for every CU */
    int kc = (int)(4096 / (m + n)) - 1;
    if (kc > 512) kc = 512;
    const int per_cu = (k + eshkol_hip_num_cus() - 1) / eshkol_hip_num_cus();
    if (kc > per_cu) kc = per_cu < 16 ? 16 : per_cu;
    if (kc < 15) return -1;
    const int pieces = (k + kc - 1) / kc;
    double* part = (double*)eshkol_hip_workspace(WS_DGEMM_PARTIAL, (size_t)pieces * m * n * sizeof(double));
    if (!part) return -1;
    const size_t lds = ((size_t)m * (kc + 1) + (size_t)kc * n) * sizeof(double);
    hipLaunchKernelGGL(dgemm_small_splitk_kernel, dim3((unsigned)pieces), dim3(256), lds, st, A, B, m, k, n, trans_a, trans_b, kc, part);
    hipLaunchKernelGGL(dgemm_small_sum_kernel, dim3((unsigned)((m * n + 255) / 256)), dim3(256), 0, st, part, pieces, m * n, C);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

/* Shapes eshkol_hip_dgemm_small takes. */
bool eshkol_hip_dgemm_is_small(uint64_t M, uint64_t K, uint64_t N) {
    return M <= 64 && N <= 64 && M * N <= 1024 && K <= 4096 && (M * K + K * N) * sizeof(double) <= 16 * 1024;
}

/* C[b] = op(A[b]) op(B[b]) for b < batch, matrices stored back to back. */
int eshkol_hip_dgemm_small(const double* A, const double* B, double* C, uint64_t M, uint64_t K, uint64_t N,
                           int trans_a, int trans_b, uint64_t batch, hipStream_t st) {
    const int m = (int)M, k = (int)K, n = (int)N;
    const size_t per = (size_t)(m * k + k * n) * sizeof(double);
    /* matrices per workgroup: one output per thread, as far as LDS goes */
    long G = 256 / (m * n);
    if (G < 1) G = 1;
    if ((size_t)G * per > (size_t)SMALL_LDS_BYTES) G = (long)(SMALL_LDS_BYTES / per);
    if (G < 1) return -1;
    if ((uint64_t)G > batch) G = (long)batch;
    const uint64_t nwg = (batch + (uint64_t)G - 1) / (uint64_t)G;
    if (nwg > 0x7fffffffULL) return -1;
    hipLaunchKernelGGL(dgemm_small_batched_kernel, dim3((unsigned)nwg), dim3(256), (size_t)G * per, st,
                       A, B, C, m, k, n, trans_a, trans_b, (long)batch, (int)G);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}
