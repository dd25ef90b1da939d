/*
 * Streaming (HBM-bound) kernels shared by the tiers: transpose, per-row
 * absolute maximum, the elementwise family and the dense-layer epilogue.
 */
#include "hip_common.h"
#include <hip/hip_ext.h>
#include "kernels.h"
#include "crt_shared.h"
#include "tanh_f64.h"

namespace {

/* 64x64 tile through LDS, 256 threads; reads and writes are both 512-byte
 * contiguous per wave row. (+1 pad: conflict-free column reads.) */
__global__ __launch_bounds__(256)
void transpose_f64_kernel(const double* __restrict__ in, double* __restrict__ out,
                          uint64_t rows, uint64_t cols) {
    __shared__ double tile[64][65];
    const uint64_t r0 = (uint64_t)blockIdx.y * 64, c0 = (uint64_t)blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const uint64_t r = r0 + ty + 4 * i, c = c0 + tx;
        if (r < rows && c < cols) tile[ty + 4 * i][tx] = in[r * cols + c];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const uint64_t c = c0 + ty + 4 * i, r = r0 + tx;
        if (r < rows && c < cols) out[c * rows + r] = tile[tx][ty + 4 * i];
    }
}

/* One wave per row: lanes stride the row 16 bytes at a time, then a butterfly
 * max across the wave. A NaN or infinity anywhere in the row makes the result
 * +inf, which the tiers read as "not representable, use the native GEMM". */
__global__ __launch_bounds__(256)
void rowabsmax_f64_kernel(const double* __restrict__ A, uint64_t M, uint64_t K,
                          double zero_value, double* __restrict__ rmax, int32_t* __restrict__ shift, int E) {
    const int lane = threadIdx.x & 63;
    const uint64_t row = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;
    const double* p = A + row * K;
    double m = 0.0;
    const bool vec = ((K & 1) == 0) && (((uintptr_t)A & 15) == 0);
    if (vec) {
        typedef double d2_t __attribute__((ext_vector_type(2)));
        const d2_t* p2 = (const d2_t*)p;
        const uint64_t n2 = K >> 1;
        for (uint64_t k = lane; k < n2; k += 64) {
            d2_t v = p2[k];
            eshkol_absmax_step(v.x, &m);
            eshkol_absmax_step(v.y, &m);
        }
    } else {
        for (uint64_t k = lane; k < K; k += 64) eshkol_absmax_step(p[k], &m);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        double o = __shfl_xor(m, off, 64);
        if (o > m) m = o;
    }
    if (lane == 0) {
        rmax[row] = (m > 0.0) ? m : zero_value;
        if (shift) shift[row] = eshkol_shift_of_maximum(m, E);
    }
}

/* The same for a few long rows (a handful of activation rows in front of a layer): a wave
 * per row walks 4096 elements from one memory latency to the next (12 us for one row).
 * Here a workgroup takes a row, every thread with four loads in flight. */
__global__ __launch_bounds__(256)
void rowabsmax_few_rows_f64_kernel(const double* __restrict__ A, uint64_t K,
                                   double zero_value, double* __restrict__ rmax, int32_t* __restrict__ shift, int E) {
    __shared__ double red[4];
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint64_t row = blockIdx.x;
    const double* p = A + row * K;
    double m = 0.0;
    const bool vec = ((K & 1) == 0) && (((uintptr_t)A & 15) == 0);
    if (vec) {
        typedef double d2_t __attribute__((ext_vector_type(2)));
        const d2_t* p2 = (const d2_t*)p;
        const uint64_t n2 = K >> 1;
        for (uint64_t k = tid; k < n2; k += 1024) {
            d2_t v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) v[u] = (k + 256 * u < n2) ? p2[k + 256 * u] : (d2_t){0.0, 0.0};
#pragma unroll
            for (int u = 0; u < 4; u++) { eshkol_absmax_step(v[u].x, &m); eshkol_absmax_step(v[u].y, &m); }
        }
    } else {
        for (uint64_t k = tid; k < K; k += 1024) {
            double v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) v[u] = (k + 256 * u < K) ? p[k + 256 * u] : 0.0;
#pragma unroll
            for (int u = 0; u < 4; u++) eshkol_absmax_step(v[u], &m);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        double o = __shfl_xor(m, off, 64);
        if (o > m) m = o;
    }
    if (lane == 0) red[wave] = m;
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 4; w++) if (red[w] > m) m = red[w];
        rmax[row] = (m > 0.0) ? m : zero_value;
        if (shift) shift[row] = eshkol_shift_of_maximum(m, E);
    }
}

/* Column maxima of a row-major X[K][R] in two steps: a block takes 64 columns
 * by one slice of the rows (a wave reads 512 contiguous bytes per row) and
 * writes its partial maxima; the second kernel folds the slices. */
constexpr int COLMAX_SLICES = 64;

__global__ __launch_bounds__(256)
void colabsmax_partial_kernel(const double* __restrict__ X, uint64_t K, uint64_t R,
                              uint64_t rows_per_slice, double* __restrict__ partial) {
    __shared__ double red[4][64];
    const int c = threadIdx.x & 63, part = threadIdx.x >> 6;
    const uint64_t col = (uint64_t)blockIdx.x * 64 + c;
    const uint64_t k0 = (uint64_t)blockIdx.y * rows_per_slice;
    const uint64_t k1 = (k0 + rows_per_slice < K) ? k0 + rows_per_slice : K;
    double m = 0.0;
    if (col < R) {
        uint64_t k = k0 + part;
        for (; k + 28 < k1; k += 32) {          /* eight loads in flight per thread, not one */
            double v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = X[(k + 4 * u) * R + col];
#pragma unroll
            for (int u = 0; u < 8; u++) eshkol_absmax_step(v[u], &m);
        }
        for (; k < k1; k += 4) eshkol_absmax_step(X[k * R + col], &m);
    }
    red[part][c] = m;
    __syncthreads();
    if (part == 0 && col < R) {
        for (int p = 1; p < 4; p++) { const double o = red[p][c]; if (o > m) m = o; }
        partial[(uint64_t)blockIdx.y * R + col] = m;
    }
}

__global__ __launch_bounds__(256)
void colabsmax_fold_kernel(const double* __restrict__ partial, uint64_t R, int slices,
                           double zero_value, double* __restrict__ out, int32_t* __restrict__ shift, int E) {
    const uint64_t col = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (col >= R) return;
    double m = 0.0;
    int s = 0;
    for (; s + 8 <= slices; s += 8) {           /* eight loads in flight, not one */
        double o[8];
#pragma unroll
        for (int u = 0; u < 8; u++) o[u] = partial[(uint64_t)(s + u) * R + col];
#pragma unroll
        for (int u = 0; u < 8; u++) if (o[u] > m) m = o[u];
    }
    for (; s < slices; s++) { const double o = partial[(uint64_t)s * R + col]; if (o > m) m = o; }
    out[col] = (m > 0.0) ? m : zero_value;
    if (shift) shift[col] = eshkol_shift_of_maximum(m, E);
}

__device__ __forceinline__ double apply_op(int op, double a, double b, bool has_b) {
    switch (op) {
        case 0:  return a + (has_b ? b : 0.0);
        case 1:  return a - (has_b ? b : 0.0);
        case 2:  return a * (has_b ? b : 1.0);
        case 3:  return a / (has_b ? b : 1.0);
        case 4:  return -a;
        case 5:  return fabs(a);
        case 6:  return exp(a);
        case 7:  return log(a);
        case 8:  return sin(a);
        case 9:  return cos(a);
        case 10: return eshkol_tanh_f64(a);
        case 11: return a > 0.0 ? a : 0.0;
        case 12: return 1.0 / (1.0 + exp(-a));
        case 13: return sqrt(a);
        default: return 1.0 / a;
    }
}

__global__ __launch_bounds__(256)
void elementwise_f64_kernel(const double* __restrict__ a, const double* __restrict__ b,
                            double* __restrict__ out, uint64_t n, int op) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        out[i] = apply_op(op, a[i], b ? b[i] : 0.0, b != nullptr);
}

__global__ __launch_bounds__(256)
void bias_act_f64_kernel(double* __restrict__ Y, const double* __restrict__ bias,
                         uint64_t rows, uint64_t cols, int act) {
    const uint64_t n = rows * cols;
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        double v = Y[i];
        if (bias) v += bias[i % cols];
        if (act == 1) v = eshkol_tanh_f64(v);
        Y[i] = v;
    }
}

inline unsigned grid_1d(uint64_t n, unsigned block, unsigned cap) {
    uint64_t g = (n + block - 1) / block;
    if (g > cap) g = cap;
    if (g < 1) g = 1;
    return (unsigned)g;
}

}  // namespace

extern "C" int hip_transpose_f64(const double* in, double* out, uint64_t rows, uint64_t cols, void* stream) {
    if (!in || !out || rows == 0 || cols == 0) return -1;
    const uint64_t gx = (cols + 63) / 64, gy = (rows + 63) / 64;
    if (gx > 0x7fffffffULL || gy > 65535ULL) return -1;
    hipLaunchKernelGGL(transpose_f64_kernel, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0,
                       (hipStream_t)stream, in, out, rows, cols);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

int eshkol_rowabsmax_shift_f64(const double* A, uint64_t M, uint64_t K, double zero_value,
                               double* rmax, int32_t* shift, int E, hipStream_t stream, hipEvent_t done) {
    if (!A || !rmax || M == 0 || K == 0) return -1;
    const uint64_t g = (M + 3) / 4;
    if (g > 0x7fffffffULL) return -1;
    if (M <= 256 && K >= 1024) {        /* fewer waves than SIMDs, rows long enough to feel it */
        hipExtLaunchKernelGGL(rowabsmax_few_rows_f64_kernel, dim3((unsigned)M), dim3(256), 0, stream, nullptr, done, 0,
                              A, K, zero_value, rmax, shift, E);
        return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
    }
    hipExtLaunchKernelGGL(rowabsmax_f64_kernel, dim3((unsigned)g), dim3(256), 0, stream, nullptr, done, 0,
                          A, M, K, zero_value, rmax, shift, E);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

extern "C" int hip_rowabsmax_f64(const double* A, uint64_t M, uint64_t K, double zero_value,
                                 double* rmax, void* stream) {
    return eshkol_rowabsmax_shift_f64(A, M, K, zero_value, rmax, nullptr, 0, (hipStream_t)stream);
}

extern "C" int hip_colabsmax_f64(const double* X, uint64_t K, uint64_t R, double zero_value,
                                 double* cmax, void* stream) {
    return eshkol_colabsmax_shift_f64(X, K, R, zero_value, cmax, nullptr, 0, (hipStream_t)stream);
}

int eshkol_colabsmax_shift_f64(const double* X, uint64_t K, uint64_t R, double zero_value,
                               double* cmax, int32_t* shift, int E, hipStream_t stream, hipEvent_t done) {
    EshkolHipCall bracket(stream);
    if (!X || !cmax || K == 0 || R == 0) return -1;
    const uint64_t gx = (R + 63) / 64;
    if (gx > 0x7fffffffULL) return -1;
    int slices = (int)((K + 63) / 64);                 /* at least 64 rows per slice */
    if (slices > COLMAX_SLICES) slices = COLMAX_SLICES;
    const uint64_t rows_per_slice = (K + slices - 1) / slices;
    slices = (int)((K + rows_per_slice - 1) / rows_per_slice);
    double* partial = (double*)eshkol_hip_workspace(WS_COLPARTIAL, (size_t)slices * R * sizeof(double));
    if (!partial) return -1;
    hipLaunchKernelGGL(colabsmax_partial_kernel, dim3((unsigned)gx, (unsigned)slices), dim3(256), 0,
                       (hipStream_t)stream, X, K, R, rows_per_slice, partial);
    hipExtLaunchKernelGGL(colabsmax_fold_kernel, dim3((unsigned)((R + 255) / 256)), dim3(256), 0,
                          (hipStream_t)stream, nullptr, done, 0, partial, R, slices, zero_value, cmax, shift, E);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

extern "C" int hip_elementwise_f64(const double* a, const double* b, double* out, uint64_t n, int op,
                                   void* stream) {
    if (!a || !out || n == 0 || op < 0 || op > 14) return -1;
    hipLaunchKernelGGL(elementwise_f64_kernel, dim3(grid_1d(n, 256, 256 * 32)), dim3(256), 0,
                       (hipStream_t)stream, a, b, out, n, op);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

extern "C" int hip_bias_act_f64(double* Y, const double* bias, uint64_t rows, uint64_t cols, int act,
                                void* stream) {
    if (!Y || rows == 0 || cols == 0 || act < 0 || act > 1) return -1;
    hipLaunchKernelGGL(bias_act_f64_kernel, dim3(grid_1d(rows * cols, 256, 256 * 32)), dim3(256), 0,
                       (hipStream_t)stream, Y, bias, rows, cols, act);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

