/*
 * A matrix held with k contiguous times one vector, in fp64: C[M x N] = A[M x K] * B[K x N]
 * with N = 1, or M = 1 and B held transposed. Behind the same entry points as the
 * matrix-core GEMM (hip_dgemm_f64 / hip_dgemm_f64_ex), which replace cublasDgemm
 * (lib/backend/gpu/gpu_memory_cuda.cpp:611-650) for every shape.
 *
 * Such a product reads the matrix once and does one fma per element: it is bound by HBM,
 * and a tile of the matrix-core kernels wastes them on rows that do not exist
 * (1 x 8192 x 8192: 0.42 ms through the tiled kernel, 0.10 ms at what HBM delivers). A
 * workgroup owns R rows o of big[O][K]; lanes run along k, 16 bytes of each row per step,
 * the four waves a quarter of K each; a lane multiplies its two k of every row by the
 * vector's values at those k (through L2) and the partial sums meet across lanes and
 * waves at the end, in a fixed order: the same call gives the same bits every time. The
 * order differs from the tiled kernel's; the tolerance of the fp64 tier (1e-14 normwise)
 * covers both. Every other thin shape (a vector against a matrix with the output index
 * contiguous, two to sixty-four vectors against either) goes through the matrix cores:
 * dgemm_thin_f64.hip.
 */
#include "hip_common.h"
#include "kernels.h"

typedef double d2u_t __attribute__((ext_vector_type(2), aligned(8)));

namespace {

/* big[O][K] (pitch ldb) times x[K]; C(o) = C[o * co] */
template <int R>
__global__ __launch_bounds__(256)
void dgemv_klast_kernel(const double* __restrict__ big, long ldb, int O, int K,
                        const double* __restrict__ x, double* __restrict__ C, long co) {
    __shared__ double red[4][R];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int o0 = (int)blockIdx.x * R;
    const double* rows[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int o = (o0 + r < O) ? o0 + r : O - 1;          /* rows beyond the matrix repeat the last one */
        rows[r] = big + (long)o * ldb;
    }
    double acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0;

    /* blocks of 128 k (two per lane), dealt to the four waves in turn */
    for (int kb = wave * 128; kb + 1 < K; kb += 512) {
        const int k = kb + 2 * lane;
        if (k + 1 < K) {
            const d2u_t t = *(const d2u_t*)(x + k);
#pragma unroll
            for (int r = 0; r < R; r++) {
                const d2u_t v = *(const d2u_t*)(rows[r] + k);
                acc[r] = fma(v.y, t.y, fma(v.x, t.x, acc[r]));
            }
        }
    }
    /* an odd K's last value: one lane of wave 0 */
    if ((K & 1) && wave == 0 && lane == 0) {
        const int k = K - 1;
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = fma(rows[r][k], x[k], acc[r]);
    }
    /* across the lanes of a wave (a fixed tree), then across the waves */
#pragma unroll
    for (int r = 0; r < R; r++) {
        double v = acc[r];
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
        if (lane == 0) red[wave][r] = v;
    }
    __syncthreads();
    const int t = (int)threadIdx.x;
    if (t < R && o0 + t < O)
        C[(long)(o0 + t) * co] = ((red[0][t] + red[1][t]) + red[2][t]) + red[3][t];
}

}  // namespace

/* Whether eshkol_hip_dgemm_matvec takes the product: one vector against a matrix held with
 * k contiguous, long enough in both directions for the launch to matter. */
bool eshkol_hip_dgemm_is_matvec(uint64_t M, uint64_t K, uint64_t N, int trans_a, int trans_b) {
    const uint64_t thin = M < N ? M : N, wide = M < N ? N : M;
    if (thin != 1 || wide < 128 || K < 64 || K > 0x7fffffffULL || wide > 0x7fffffffULL) return false;
    const bool thin_m = M <= N;
    const bool klast = thin_m ? (trans_b != 0) : (trans_a == 0);     /* the matrix has k contiguous */
    return klast && wide * K >= (1ull << 17);
}

/* C = op(A) op(B) for a product eshkol_hip_dgemm_is_matvec() accepts. */
int eshkol_hip_dgemm_matvec(const double* A, const double* B, double* C, uint64_t M, uint64_t K, uint64_t N,
                            int trans_a, int trans_b, hipStream_t st) {
    (void)trans_a; (void)trans_b;
    const bool thin_m = M <= N;
    const int O = (int)(thin_m ? N : M), k = (int)K;
    const double* big = thin_m ? B : A;
    const double* x = thin_m ? A : B;               /* K values, contiguous whichever form the caller holds it in */
    constexpr int R = 8;
    hipLaunchKernelGGL(dgemv_klast_kernel<R>, dim3((unsigned)((O + R - 1) / R)), dim3(256), 0, st,
                       big, (long)K, O, k, x, C, 1L);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}
