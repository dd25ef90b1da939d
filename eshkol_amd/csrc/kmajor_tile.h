/*
 * Reading an operand the caller stores k-major (X[K][R], the row index
 * contiguous: B as the runtime holds it) as if it were X^T[R][K], without a
 * transposed copy in HBM. The split, slice and narrowing kernels all want two
 * consecutive k of one row per thread, so that a wave writes 128 contiguous
 * output bytes per plane; this helper gives them exactly that view.
 *
 * A block owns 32 rows of X^T by 128 k. It reads the 128 x 32 tile with the row
 * index across lanes (256 contiguous bytes per k, 16 bytes per lane), parks it
 * in LDS as [32][128+2] doubles, and hands thread t the pairs (row q/64,
 * k 2(q%64)), q = t, t+256, ... The pad keeps the 16-byte LDS reads
 * conflict-free.
 */
#ifndef ESHKOL_HIP_KMAJOR_TILE_H
#define ESHKOL_HIP_KMAJOR_TILE_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace kmaj {

typedef double d2_t __attribute__((ext_vector_type(2)));

constexpr int TK = 128;
constexpr int TR = 32;
constexpr int LD = TK + 2;
constexpr int SMEM_DOUBLES = TR * LD;

/* blocks needed to cover rows_ext rows by k_ext k-values (both may exceed the matrix: padding) */
inline uint64_t grid_blocks(uint64_t rows_ext, uint64_t k_ext) {
    return ((rows_ext + TR - 1) / TR) * ((k_ext + TK - 1) / TK);
}

/* emit(row, k, x0, x1) for every even k < k_ext and every row < rows_ext of the
 * block's tile; x is 0 outside the R x K matrix. 256 threads.
 * KFAST picks which neighbours run together: consecutive blocks along k write
 * whole output rows (best when the kernel writes more than it reads, as the
 * 16-plane CRT split does); consecutive blocks along the rows read whole rows
 * of X (best for the lighter slice and narrowing kernels). Measured at 8192^2:
 * CRT split 560 vs 740 us, slices 410 vs 385 us, narrowing 164 vs 149 us. */
template <bool KFAST, class Emit>
__device__ __forceinline__ void for_each_pair(const double* __restrict__ X, uint64_t R, uint64_t K,
                                              uint64_t rows_ext, uint64_t k_ext, double* lds, Emit emit) {
    const uint32_t rt = (uint32_t)((rows_ext + TR - 1) / TR), kt = (uint32_t)((k_ext + TK - 1) / TK);
    const uint32_t rtile = KFAST ? blockIdx.x / kt : blockIdx.x % rt;
    const uint32_t ktile = KFAST ? blockIdx.x % kt : blockIdx.x / rt;
    const uint64_t r0 = (uint64_t)rtile * TR;
    const uint64_t k0 = (uint64_t)ktile * TK;
    const int tid = threadIdx.x;
    /* a lane takes two neighbouring rows of one k: 16 lanes read 256 contiguous bytes */
    const int lr = 2 * (tid & 15), lk = tid >> 4;
    const bool vec = ((R & 1) == 0) && (((uintptr_t)X & 15) == 0);
#pragma unroll
    for (int i = 0; i < TK / 16; i++) {
        const int kk = lk + 16 * i;
        const uint64_t gk = k0 + kk, gr = r0 + lr;
        double v0 = 0.0, v1 = 0.0;
        if (gk < K) {
            const double* p = X + gk * R + gr;
            if (vec) {
                if (gr < R) { const d2_t v = *(const d2_t*)p; v0 = v.x; v1 = v.y; }
            } else {
                if (gr < R) v0 = p[0];
                if (gr + 1 < R) v1 = p[1];
            }
        }
        lds[lr * LD + kk] = v0;
        lds[(lr + 1) * LD + kk] = v1;
    }
    __syncthreads();
    /* not unrolled: the emit bodies are long, and keeping four waves per SIMD
     * resident matters more here than instruction-level overlap (measured
     * 560 vs 770 us for the 16-modulus split at 8192^2) */
#pragma unroll 1
    for (int i = 0; i < TR * TK / 2 / 256; i++) {
        const int q = tid + 256 * i;
        const int r = q >> 6, kp = q & 63;
        const uint64_t row = r0 + r, k = k0 + 2 * kp;
        if (row < rows_ext && k < k_ext) {
            const d2_t v = *(const d2_t*)(lds + r * LD + 2 * kp);
            emit(row, k, v.x, v.y);
        }
    }
}

}  // namespace kmaj
#endif
