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

}  // namespace

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
