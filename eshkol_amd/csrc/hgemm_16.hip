/*
 * Reduced-precision tier: f16 or bf16 operands, fp32 accumulation on the gfx950
 * matrix cores (v_mfma_f32_32x32x16_f16 / _bf16). Takes the place of
 * cuda_matmul_f16_from_f64 (lib/backend/gpu/gpu_memory_cuda.cpp:678-728): there
 * the f64 -> half conversion and back run on the host around cublasGemmEx; here
 * they are device kernels and the operands never leave HBM.
 *
 * The narrowing is the reference's two-step one: f64 -> f32 (round to nearest
 * even), then f32 -> 16-bit (round to nearest even), as in reduce_precision
 * (lib/core/runtime_tensor_dtype.cpp:37-109) and in the CUDA path's
 * __float2half((float)x). dtype 3 multiplies true bf16 operands; the reference's
 * CUDA unit sends bf16 tensors through half (gpu_memory_cuda.cpp:1125), which
 * overflows for |x| > 65504.
 *
 * The contraction has the same shape as the int8 one: K-contiguous operands
 * (B is transposed once in fp64), 64-byte k-blocks double-buffered in LDS with
 * a 16-byte row pad, 2x2 waves of 4x4 (or 2x2) MFMA tiles, B fragment as the
 * first MFMA operand so a lane owns 4 consecutive output columns.
 */
#include "hip_common.h"
#include "kernels.h"
#include "gemm_pipe.h"
#include "gemm_pipe2.h"
#include "kmajor_tile.h"

#include <cstring>
#include <mutex>

typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef float v4f_t __attribute__((ext_vector_type(4)));
typedef float v16f_t __attribute__((ext_vector_type(16)));
typedef _Float16 v8h_t __attribute__((ext_vector_type(8)));
typedef __bf16 v8b_t __attribute__((ext_vector_type(8)));
typedef double d2_t __attribute__((ext_vector_type(2)));

namespace {

constexpr int BKB = 64;            /* bytes of K per block = 32 elements */
constexpr int LDS_PITCH = BKB + 16;

/* runtime_tensor_dtype.cpp:97-109, NaN kept quiet instead of truncated */
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t bits = __float_as_uint(f);
    if (((bits >> 23) & 0xffu) == 0xffu) {
        uint16_t h = (uint16_t)(bits >> 16);
        if (bits & 0x7fffffu) h |= 0x0040u;
        return h;
    }
    bits += 0x7fffu + ((bits >> 16) & 1u);
    return (uint16_t)(bits >> 16);
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
    _Float16 h = (_Float16)f;                 /* v_cvt_f16_f32: round to nearest even */
    uint16_t u;
    __builtin_memcpy(&u, &h, 2);
    return u;
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t u) {
    _Float16 h;
    __builtin_memcpy(&h, &u, 2);
    return (float)h;
}

template <bool BF16>
__device__ __forceinline__ uint32_t narrow_pair(double x0, double x1) {
    const uint16_t h0 = BF16 ? f32_to_bf16_bits((float)x0) : f32_to_f16_bits((float)x0);
    const uint16_t h1 = BF16 ? f32_to_bf16_bits((float)x1) : f32_to_f16_bits((float)x1);
    return (uint32_t)h0 | ((uint32_t)h1 << 16);
}

/* Every narrowing kernel converts `gridDim.y` matrices stored back to back
 * (X + b * rows * K -> out + b * rows_padded * ld). */

/* Row-major X[rows][K]. One thread: two consecutive k of one row. */
template <bool BF16>
__global__ __launch_bounds__(256)
void convert_kernel(const double* __restrict__ X, uint64_t rows, uint64_t K,
                    uint16_t* __restrict__ out, uint64_t rows_padded, uint64_t ld) {
    X += (uint64_t)blockIdx.y * rows * K;
    out += (uint64_t)blockIdx.y * rows_padded * ld;
    const uint32_t cpr = (uint32_t)((ld / 2 + 255) / 256);
    const uint64_t row = blockIdx.x / cpr;
    const uint64_t k = ((uint64_t)(blockIdx.x % cpr) * 256 + threadIdx.x) * 2;
    if (k >= ld) return;
    double x0 = 0.0, x1 = 0.0;
    if (row < rows) {
        const double* p = X + row * K + k;
        if (k + 1 < K) {
            if ((K & 1) == 0 && (((uintptr_t)X & 15) == 0)) { d2_t v = *(const d2_t*)p; x0 = v.x; x1 = v.y; }
            else { x0 = p[0]; x1 = p[1]; }
        } else if (k < K) {
            x0 = p[0];
        }
    }
    *(uint32_t*)(out + row * ld + k) = narrow_pair<BF16>(x0, x1);
}

/* Row-major X[rows][K] into the interleaved layout (rows_padded a multiple of 32,
 * ld of 64 elements). A block takes 32 rows x 64 k: eight lanes read 512
 * contiguous bytes of a row, a lane narrows eight k into one 16-byte chunk, and
 * the chunks of eight consecutive rows are 128 contiguous output bytes. */
template <bool BF16>
__global__ __launch_bounds__(256)
void convert_il_kernel(const double* __restrict__ X, uint64_t rows, uint64_t K,
                       uint16_t* __restrict__ out, uint64_t rows_padded, uint64_t ld) {
    X += (uint64_t)blockIdx.y * rows * K;
    out += (uint64_t)blockIdx.y * rows_padded * ld;
    const uint32_t kt = (uint32_t)(ld / 64);
    const uint64_t rb = blockIdx.x / kt, kb = blockIdx.x % kt;
    const int tid = threadIdx.x;
    const uint64_t row = rb * 32 + (uint64_t)(tid >> 3), k = kb * 64 + 8 * (uint64_t)(tid & 7);
    double x[8] = {0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0};
    if (row < rows && k < K) {
        const double* p = X + row * K + k;
        if (k + 8 <= K && (K & 1) == 0 && (((uintptr_t)X & 15) == 0)) {
#pragma unroll
            for (int e = 0; e < 8; e += 2) { const d2_t v = *(const d2_t*)(p + e); x[e] = v.x; x[e + 1] = v.y; }
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) if (k + e < K) x[e] = p[e];
        }
    }
    v4i_t w;
#pragma unroll
    for (int e = 0; e < 4; e++) w[e] = (int)narrow_pair<BF16>(x[2 * e], x[2 * e + 1]);
    eshkol_store_streaming((v4i_t*)((int8_t*)out + eshkol_plane_offset(1, row, 2 * k, 2 * ld)), w);
}

/* k-major X[K][rows] (B as the runtime stores it), same output. */
template <bool BF16>
__global__ __launch_bounds__(256, 4)
void convert_kmajor_kernel(const double* __restrict__ X, uint64_t rows, uint64_t K,
                           uint16_t* __restrict__ out, uint64_t rows_padded, uint64_t ld, int layout) {
    __shared__ __align__(16) double tile[kmaj::SMEM_DOUBLES];
    X += (uint64_t)blockIdx.y * rows * K;
    out += (uint64_t)blockIdx.y * rows_padded * ld;
    if (layout == 1) {
        /* sixteen k per thread: two 16-byte chunks of one row */
        kmaj::for_each_16(X, rows, K, rows_padded, ld, 0xffffffffu, tile,
            [](uint64_t) { return 0; },
            [&](uint64_t row, uint64_t k, const double* x, int) {
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    v4i_t w;
#pragma unroll
                    for (int e = 0; e < 4; e++) w[e] = (int)narrow_pair<BF16>(x[8 * c + 2 * e], x[8 * c + 2 * e + 1]);
                    eshkol_store_streaming((v4i_t*)((int8_t*)out + eshkol_plane_offset(1, row, 2 * k + 16 * c, 2 * ld)), w);
                }
            });
        return;
    }
    kmaj::for_each_pair(X, rows, K, rows_padded, ld, 0xffffffffu, tile,
        [](uint64_t) { return 0; },
        [&](uint64_t row, uint64_t k, double x0, double x1, int) {
            *(uint32_t*)(out + row * ld + k) = narrow_pair<BF16>(x0, x1);
        });
}

/* k-major X[K][rows], interleaved planes: no LDS (kmajor_tile.h); sixteen k of one
 * row are two 16-byte chunks. */
template <bool BF16>
__global__ __launch_bounds__(256, 4)
void convert_kmajor_il_kernel(const double* __restrict__ X, uint64_t rows, uint64_t K,
                              uint16_t* __restrict__ out, uint64_t rows_padded, uint64_t ld) {
    X += (uint64_t)blockIdx.y * rows * K;
    out += (uint64_t)blockIdx.y * rows_padded * ld;
    uint64_t row, k;
    kmaj::il_thread(rows_padded, &row, &k);
    if (row >= rows_padded || k >= ld) return;
    double x[16];
    kmaj::load_k16(X, rows, K, row, k, x);
#pragma unroll
    for (int c = 0; c < 2; c++) {
        v4i_t w;
#pragma unroll
        for (int e = 0; e < 4; e++) w[e] = (int)narrow_pair<BF16>(x[8 * c + 2 * e], x[8 * c + 2 * e + 1]);
        eshkol_store_streaming((v4i_t*)((int8_t*)out + eshkol_plane_offset(1, row, 2 * k + 16 * c, 2 * ld)), w);
    }
}

template <int TM, int TN> struct Cfg {
    static constexpr int NT = 256;
    static constexpr int BM = 2 * TM * 32;
    static constexpr int BN = 2 * TN * 32;
    static constexpr int A_TILE = BM * LDS_PITCH;
    static constexpr int B_TILE = BN * LDS_PITCH;
    static constexpr int SMEM_BYTES = 2 * (A_TILE + B_TILE);
    static constexpr int A_CHUNKS = BM * BKB / 16 / NT;
    static constexpr int B_CHUNKS = BN * BKB / 16 / NT;
};

/* out_mode 0: fp32 C; 1: f64 C; 2: f64 C after rounding to the 16-bit type */
template <bool BF16, int TM, int TN>
__global__ __launch_bounds__(256)
void hgemm_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ Bt,
                  int M, int N, int ld_bytes, int out_mode, void* __restrict__ Cout,
                  int tiles_m, int tiles_n, uint64_t a_stride, uint64_t b_stride) {
    using C = Cfg<TM, TN>;
    extern __shared__ __align__(16) int8_t smem_h[];
    /* blockIdx.y: one of the products stored back to back (strides in bytes) */
    A = (const uint16_t*)((const int8_t*)A + (uint64_t)blockIdx.y * a_stride);
    Bt = (const uint16_t*)((const int8_t*)Bt + (uint64_t)blockIdx.y * b_stride);
    Cout = (int8_t*)Cout + (uint64_t)blockIdx.y * (uint64_t)M * (uint64_t)N * (out_mode == 0 ? 4u : 8u);
    int8_t* As = smem_h;
    int8_t* Bs = smem_h + 2 * C::A_TILE;

    int tm, tn;
    {
        const int nwg = gridDim.x, wg = blockIdx.x;
        const int q = nwg >> 3, r = nwg & 7;
        const int xcd = wg & 7, seq = wg >> 3;
        const int L = xcd * q + (xcd < r ? xcd : r) + seq;
        const int GM = 8;
        const int width = GM * tiles_n;
        const int group = L / width;
        const int first_m = group * GM;
        const int gsize = (tiles_m - first_m < GM) ? tiles_m - first_m : GM;
        const int in_group = L - group * width;
        tm = first_m + in_group % gsize;
        tn = in_group / gsize;
    }
    const int m0 = tm * C::BM, n0 = tn * C::BN;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 31, lh = lane >> 5;

    const int8_t* Ap = (const int8_t*)A + (size_t)m0 * ld_bytes;
    const int8_t* Bp = (const int8_t*)Bt + (size_t)n0 * ld_bytes;
    const int nkb = ld_bytes / BKB;

    v4i_t ra[C::A_CHUNKS], rb[C::B_CHUNKS];
    auto gload = [&](int kb) {
        const int k0 = kb * BKB;
#pragma unroll
        for (int r = 0; r < C::A_CHUNKS; r++) {
            const int c = tid + C::NT * r;
            ra[r] = *(const v4i_t*)(Ap + (size_t)(c >> 2) * ld_bytes + k0 + (c & 3) * 16);
        }
#pragma unroll
        for (int r = 0; r < C::B_CHUNKS; r++) {
            const int c = tid + C::NT * r;
            rb[r] = *(const v4i_t*)(Bp + (size_t)(c >> 2) * ld_bytes + k0 + (c & 3) * 16);
        }
    };
    auto sstore = [&](int buf) {
#pragma unroll
        for (int r = 0; r < C::A_CHUNKS; r++) {
            const int c = tid + C::NT * r;
            *(v4i_t*)(As + buf * C::A_TILE + (c >> 2) * LDS_PITCH + (c & 3) * 16) = ra[r];
        }
#pragma unroll
        for (int r = 0; r < C::B_CHUNKS; r++) {
            const int c = tid + C::NT * r;
            *(v4i_t*)(Bs + buf * C::B_TILE + (c >> 2) * LDS_PITCH + (c & 3) * 16) = rb[r];
        }
    };

    v16f_t acc[TM][TN];
#pragma unroll
    for (int t = 0; t < TM; t++)
#pragma unroll
        for (int u = 0; u < TN; u++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[t][u][r] = 0.0f;

    gload(0);
    sstore(0);
    __syncthreads();

    int cur = 0;
    for (int kb = 0; kb < nkb; kb++) {
        const bool more = (kb + 1 < nkb);
        if (more) gload(kb + 1);
        const int8_t* a_base = As + cur * C::A_TILE + (wm * TM * 32 + li) * LDS_PITCH + lh * 16;
        const int8_t* b_base = Bs + cur * C::B_TILE + (wn * TN * 32 + li) * LDS_PITCH + lh * 16;
#pragma unroll
        for (int ks = 0; ks < BKB / 32; ks++) {
            v4i_t a[TM], b[TN];
#pragma unroll
            for (int t = 0; t < TM; t++) a[t] = *(const v4i_t*)(a_base + t * 32 * LDS_PITCH + ks * 32);
#pragma unroll
            for (int u = 0; u < TN; u++) b[u] = *(const v4i_t*)(b_base + u * 32 * LDS_PITCH + ks * 32);
#pragma unroll
            for (int t = 0; t < TM; t++)
#pragma unroll
                for (int u = 0; u < TN; u++) {
                    if (BF16)
                        acc[t][u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            __builtin_bit_cast(v8b_t, b[u]), __builtin_bit_cast(v8b_t, a[t]), acc[t][u], 0, 0, 0);
                    else
                        acc[t][u] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                            __builtin_bit_cast(v8h_t, b[u]), __builtin_bit_cast(v8h_t, a[t]), acc[t][u], 0, 0, 0);
                }
        }
        if (more) sstore(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }

    /* lane column is the output row; registers 4v..4v+3 are output columns
     * 8v + 4*(lane/32) + 0..3 of the 32x32 tile */
#pragma unroll
    for (int t = 0; t < TM; t++) {
        const int row = m0 + wm * TM * 32 + t * 32 + li;
        if (row >= M) continue;
#pragma unroll
        for (int u = 0; u < TN; u++) {
            /* With 256 accumulator registers, keep each 16-register tile in the
             * accumulator file until it is stored: otherwise the allocator copies
             * all of them into vector registers on entry and spills. */
            if constexpr (TM * TN >= 16) asm volatile("" : "+a"(acc[t][u]));
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int col = n0 + wn * TN * 32 + u * 32 + 8 * v + 4 * lh;
                float f[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float x = acc[t][u][4 * v + e];
                    if (out_mode == 2)
                        x = BF16 ? bf16_bits_to_f32(f32_to_bf16_bits(x)) : f16_bits_to_f32(f32_to_f16_bits(x));
                    f[e] = x;
                }
                if (out_mode == 0) {
                    float* p = (float*)Cout + (size_t)row * N + col;
                    if ((N & 3) == 0 && col + 3 < N) *(v4f_t*)p = (v4f_t){f[0], f[1], f[2], f[3]};
                    else for (int e = 0; e < 4; e++) if (col + e < N) p[e] = f[e];
                } else {
                    double* p = (double*)Cout + (size_t)row * N + col;
                    if ((N & 1) == 0 && col + 3 < N) {
                        *(d2_t*)p = (d2_t){(double)f[0], (double)f[1]};
                        *(d2_t*)(p + 2) = (d2_t){(double)f[2], (double)f[3]};
                    } else {
                        for (int e = 0; e < 4; e++) if (col + e < N) p[e] = (double)f[e];
                    }
                }
            }
        }
    }
}

/* ---- pipelined kernel (gemm_pipe.h): 256x256 tile, 128-byte k-blocks ------- */

template <bool BF16> struct H16Op {
    typedef v16f_t acc_t;
    static __device__ __forceinline__ void mfma(const v4i_t& first, const v4i_t& second, v16f_t& acc) {
        if (BF16)
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8b_t, first),
                                                          __builtin_bit_cast(v8b_t, second), acc, 0, 0, 0);
        else
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h_t, first),
                                                         __builtin_bit_cast(v8h_t, second), acc, 0, 0, 0);
    }
    /* the first product of a sum: the instruction takes the constant 0 as its addend */
    static __device__ __forceinline__ void mfma_first(const v4i_t& first, const v4i_t& second, v16f_t& acc) {
        const v16f_t none = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        if (BF16)
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8b_t, first),
                                                          __builtin_bit_cast(v8b_t, second), none, 0, 0, 0);
        else
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h_t, first),
                                                         __builtin_bit_cast(v8h_t, second), none, 0, 0, 0);
    }
    static __device__ __forceinline__ void zero(v16f_t& acc) {
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0.0f;
    }
};

/* x rounded to the 16-bit type and widened again. The bf16 form is
 * f32_to_bf16_bits() above written with selects: an epilogue applies it to 256
 * values per lane, and a branch for the Inf/NaN case around each of them costs
 * more than the rounding. */
template <bool BF16>
__device__ __forceinline__ float round16(float x) {
    if constexpr (BF16) {
        const uint32_t bits = __float_as_uint(x);
        const uint32_t rounded = (bits + 0x7fffu + ((bits >> 16) & 1u)) & 0xffff0000u;
        const uint32_t special = (bits & 0xffff0000u) | ((bits & 0x7fffffu) ? 0x00400000u : 0u);
        return __uint_as_float((bits & 0x7f800000u) == 0x7f800000u ? special : rounded);
    } else {
        return f16_bits_to_f32(f32_to_f16_bits(x));
    }
}

/* lane column is the output row; registers 4v..4v+3 are output columns
 * 8v + 4*(lane/32) + 0..3 of the 32x32 tile */
template <bool BF16, int TM, int TN>
__device__ __forceinline__ void store_tile(v16f_t (&acc)[TM][TN], int m0, int n0, int M, int N,
                                           int out_mode, void* Cout) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 31, lh = lane >> 5;
#pragma unroll
    for (int t = 0; t < TM; t++) {
        const int row = m0 + wm * TM * 32 + t * 32 + li;
        if (row >= M) continue;
#pragma unroll
        for (int u = 0; u < TN; u++) {
            /* With 256 accumulator registers, keep each 16-register tile in the
             * accumulator file until it is stored: otherwise the allocator copies
             * all of them into vector registers on entry and spills. */
            if constexpr (TM * TN >= 16) asm volatile("" : "+a"(acc[t][u]));
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int col = n0 + wn * TN * 32 + u * 32 + 8 * v + 4 * lh;
                float f[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float x = acc[t][u][4 * v + e];
                    if (out_mode == 2) x = round16<BF16>(x);
                    f[e] = x;
                }
                if (out_mode == 0) {
                    float* p = (float*)Cout + (size_t)row * N + col;
                    if ((N & 3) == 0 && col + 3 < N) *(v4f_t*)p = (v4f_t){f[0], f[1], f[2], f[3]};
                    else for (int e = 0; e < 4; e++) if (col + e < N) p[e] = f[e];
                } else {
                    double* p = (double*)Cout + (size_t)row * N + col;
                    if ((N & 1) == 0 && col + 3 < N) {
                        *(d2_t*)p = (d2_t){(double)f[0], (double)f[1]};
                        *(d2_t*)(p + 2) = (d2_t){(double)f[2], (double)f[3]};
                    } else {
                        for (int e = 0; e < 4; e++) if (col + e < N) p[e] = (double)f[e];
                    }
                }
            }
        }
    }
}

/* One workgroup per CU walks the tile ids blockIdx.x, blockIdx.x + gridDim.x, ...
 * (gridDim.x is a multiple of 8, so an id stays on its XCD); ids are laid out so
 * that each XCD owns a contiguous run of tiles, 8 tile-rows at a time. The
 * operand stream runs on across tile boundaries (pipe::run_tiles). */
template <bool BF16, int PF>
__global__ __launch_bounds__(256, 1)
void hgemm_pipe_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ Bt,
                       int M, int N, int ld_bytes, int out_mode, void* __restrict__ Cout,
                       int tiles_m, int tiles_n, int n_ids) {
    extern __shared__ __align__(16) int8_t smem_h[];
    pipe::Source cm;
    cm.a_planes = (const int8_t*)A; cm.b_planes = (const int8_t*)Bt;
    cm.a_plane_stride = 0; cm.b_plane_stride = 0;
    cm.ld = ld_bytes;

    const int n_tiles = tiles_m * tiles_n;
    int next_id = (int)blockIdx.x;
    auto next_tile = [&](pipe::Tile& t) -> bool {
        while (next_id < n_ids) {
            const int id = next_id;
            next_id += (int)gridDim.x;
            /* XCD x owns tiles [x * per, (x + 1) * per) */
            const int per = n_ids >> 3;
            const int L = (id & 7) * per + (id >> 3);
            if (L >= n_tiles) continue;
            const int GM = 8;
            const int width = GM * tiles_n;
            const int group = L / width;
            const int first_m = group * GM;
            const int gsize = (tiles_m - first_m < GM) ? tiles_m - first_m : GM;
            const int in_group = L - group * width;
            t.m0 = (first_m + in_group % gsize) * 256;
            t.n0 = (in_group / gsize) * 256;
            t.tag = 0; t.a_idx = nullptr; t.b_idx = nullptr; t.npairs = 1;
            return true;
        }
        return false;
    };
    auto epi = [&](v16f_t (&acc)[4][4], const pipe::Tile& t) {
        store_tile<BF16, 4, 4>(acc, t.m0, t.n0, M, N, out_mode, Cout);
    };
    pipe::run_tiles<H16Op<BF16>, 4, 4, PF>(smem_h, cm, next_tile, epi);
}

/* ---- interleaved operands, loaded straight into LDS and MFMA registers
 * (gemm_pipe2.h): four waves stacked along M, wave tile 64 x 256. acc[t][u] is
 * the transposed 32 x 32 tile of rows m0 + 64 wave + 32 t + lane%32, columns
 * n0 + 32 u + 8 v + 4 (lane/32) + 0..3 in registers 4v .. 4v+3. A batch of
 * products is one launch: a tile's batch index is its operand plane. */
/* INTERIOR: the tile lies inside the matrix: the stores then carry no bounds and no
 * branches, and one address serves a block. Rows move as 16-byte pieces whatever N is:
 * the vector types below promise the element's alignment only (global memory takes
 * 16-byte accesses at any 4-byte boundary), so an odd N costs no more than lines
 * written in two parts.
 * OM: the output mode where the caller has already branched on it (-1: read out_mode_arg). */
template <bool BF16, bool INTERIOR, int OM = -1>
__device__ __forceinline__ void store_tile_direct(v16f_t (&acc)[pipe2::TM][pipe2::TN], int m0, int n0, int M, int N,
                                                  int out_mode_arg, void* Cout, int8_t* stage) {
    const int out_mode = OM >= 0 ? OM : out_mode_arg;      /* OM >= 0: known when compiled, nothing decided per value */
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    typedef int v4iu_t __attribute__((ext_vector_type(4), aligned(4)));
    typedef double d2u_t __attribute__((ext_vector_type(2), aligned(8)));
#pragma unroll
    for (int t = 0; t < pipe2::TM; t++) {
        const int row0 = m0 + wave * 64 + t * 32;
#pragma unroll
        for (int u = 0; u < pipe2::TN; u++) {
            asm volatile("" : "+a"(acc[t][u]));          /* keep the tile in the accumulator file until here */
            /* the block goes through the wave's LDS stage so that a store instruction
             * writes whole lines: eight lanes a 128-byte row segment of fp32, sixteen
             * lanes 256 bytes of fp64 */
#pragma unroll
            for (int v = 0; v < 4; v++) {
                float f[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float x = acc[t][u][4 * v + e];
                    if (out_mode == 2) x = round16<BF16>(x);
                    f[e] = x;
                }
                pipe2::park_block(stage, v, (v4i_t){__float_as_int(f[0]), __float_as_int(f[1]),
                                                    __float_as_int(f[2]), __float_as_int(f[3])});
                __builtin_amdgcn_sched_barrier(0);
            }
            const int cb = n0 + u * 32;
            if constexpr (INTERIOR) {
                if (out_mode == 0) {
                    v4i_t w[4];
#pragma unroll
                    for (int i = 0; i < 4; i++) w[i] = pipe2::parked_row16(stage, i);
                    float* p = (float*)Cout + (size_t)(row0 + (lane >> 3)) * N + cb + 4 * (lane & 7);
#pragma unroll
                    /* streaming: 2 per cent of the 8192^3 product (0.818 -> 0.802 ms); the fp64
                     * form below gains nothing from it */
                    for (int i = 0; i < 4; i++) __builtin_nontemporal_store((v4iu_t)w[i], (v4iu_t*)(p + (size_t)(8 * i) * N));
                } else {
                    pipe2::v2i_t w[8];
#pragma unroll
                    for (int i = 0; i < 8; i++) w[i] = pipe2::parked_row8(stage, i);
                    double* p = (double*)Cout + (size_t)(row0 + (lane >> 4)) * N + cb + 2 * (lane & 15);
#pragma unroll
                    for (int i = 0; i < 8; i++)
                        *(d2u_t*)(p + (size_t)(4 * i) * N) = (d2u_t){(double)__int_as_float(w[i][0]), (double)__int_as_float(w[i][1])};
                }
            } else if (out_mode == 0) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const v4i_t w = pipe2::parked_row16(stage, i);
                    const int row = row0 + (lane >> 3) + 8 * i, col = cb + 4 * (lane & 7);
                    if (row < M && col < N) {
                        float* p = (float*)Cout + (size_t)row * N + col;
                        if (col + 3 < N) *(v4iu_t*)p = (v4iu_t)w;
                        else for (int e = 0; e < 4; e++) if (col + e < N) p[e] = __int_as_float(w[e]);
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const pipe2::v2i_t w = pipe2::parked_row8(stage, i);
                    const int row = row0 + (lane >> 4) + 4 * i, col = cb + 2 * (lane & 15);
                    if (row < M && col < N) {
                        double* p = (double*)Cout + (size_t)row * N + col;
                        if (col + 1 < N) *(d2u_t*)p = (d2u_t){(double)__int_as_float(w[0]), (double)__int_as_float(w[1])};
                        else for (int e = 0; e < 2; e++) if (col + e < N) p[e] = (double)__int_as_float(w[e]);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

template <bool BF16>
__global__ __launch_bounds__(256, 1)
void hgemm_direct_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ Bt,
                         int M, int N, int ld_bytes, int out_mode, void* __restrict__ Cout,
                         int tiles_m, int tiles_n, int n_ids, uint64_t a_stride, uint64_t b_stride, int batch) {
    extern __shared__ __align__(16) int8_t smem_h[];
    pipe::Source cm;
    cm.a_planes = (const int8_t*)A; cm.b_planes = (const int8_t*)Bt;
    cm.a_plane_stride = a_stride; cm.b_plane_stride = b_stride;
    cm.ld = ld_bytes;

    const int per_matrix = tiles_m * tiles_n;
    const int per_xcd = n_ids >> 3;                  /* XCD x owns tile numbers [x * per_xcd, (x + 1) * per_xcd) */
    int next_id = (int)blockIdx.x;
    auto next_tile = [&](pipe::Tile& t) -> bool {
        while (next_id < n_ids) {
            const int id = next_id;
            next_id += (int)gridDim.x;
            const int L = (id & 7) * per_xcd + (id >> 3);
            const int b = L / per_matrix, in_matrix = L - b * per_matrix;
            if (b >= batch) continue;                /* padding ids of the last XCD */
            const int GM = 8;
            const int width = GM * tiles_n;
            const int group = in_matrix / width;
            const int first_m = group * GM;
            const int gsize = (tiles_m - first_m < GM) ? tiles_m - first_m : GM;
            const int in_group = in_matrix - group * width;
            t.m0 = (first_m + in_group % gsize) * 256;
            t.n0 = (in_group / gsize) * 256;
            t.tag = b; t.a_idx = nullptr; t.b_idx = nullptr; t.npairs = 1;
            t.a_plane0 = b; t.b_plane0 = b;
            return true;
        }
        return false;
    };
    const uint64_t c_bytes = (uint64_t)M * (uint64_t)N * (out_mode == 0 ? 4u : 8u);
    auto epi = [&](v16f_t (&acc)[pipe2::TM][pipe2::TN], const pipe::Tile& t, int8_t* stage) {
        void* Ct = (int8_t*)Cout + (uint64_t)t.tag * c_bytes;
        const bool interior = t.m0 + pipe2::BM <= M && t.n0 + pipe2::BN <= N;
        if (!interior) store_tile_direct<BF16, false>(acc, t.m0, t.n0, M, N, out_mode, Ct, stage);
        else if (out_mode == 0) store_tile_direct<BF16, true, 0>(acc, t.m0, t.n0, M, N, 0, Ct, stage);
        else if (out_mode == 1) store_tile_direct<BF16, true, 1>(acc, t.m0, t.n0, M, N, 1, Ct, stage);
        else store_tile_direct<BF16, true, 2>(acc, t.m0, t.n0, M, N, 2, Ct, stage);
    };
    pipe2::run_tiles<H16Op<BF16>>(smem_h, cm, next_tile, epi);
}

/* The dynamic-LDS attribute of a kernel, set once per kernel and process: a list
 * under a mutex instead of a static flag per launcher, so that the first calls
 * of two threads do not race and so that hip_matmul_reduced_f64_noalloc's
 * set-up can run every launcher's part ahead of its first call. */
bool kernel_ready(const void* kern, int smem) {
    static std::mutex m;
    static const void* done[16];
    static int n_done = 0;
    std::lock_guard<std::mutex> lk(m);
    for (int i = 0; i < n_done; i++) if (done[i] == kern) return true;
    if (!ESHKOL_HIP_OK(hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem))) return false;
    if (n_done < 16) done[n_done++] = kern;
    return true;
}

template <bool BF16>
int launch_direct(const uint16_t* A, const uint16_t* Bt, int M, int N, int ld_bytes, int out_mode, void* C,
                  int batch, uint64_t a_stride, uint64_t b_stride, hipStream_t st) {
    constexpr int SMEM = pipe2::SMEM_BYTES;
    auto kern = hgemm_direct_kernel<BF16>;
    if (!kernel_ready((const void*)kern, SMEM)) return -1;
    const int num_cus = eshkol_hip_num_cus();
    if (!A) return 0;                                        /* set-up only */
    const int tiles_m = (M + 255) / 256, tiles_n = (N + 255) / 256;
    const long long total = (long long)tiles_m * tiles_n * batch;
    if (total > 0x7ffffff0LL) return -1;
    const int n_ids = (int)((total + 7) / 8 * 8);            /* padded so every XCD owns the same count */
    int grid = (num_cus / 8) * 8;
    if (grid < 8) grid = 8;
    if (grid > n_ids) grid = n_ids;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), SMEM, st,
                       A, Bt, M, N, ld_bytes, out_mode, C, tiles_m, tiles_n, n_ids, a_stride, b_stride, batch);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

template <bool BF16>
int launch_pipe(const uint16_t* A, const uint16_t* Bt, int M, int N, int ld_bytes, int out_mode, void* C,
                hipStream_t st) {
    constexpr int SMEM = pipe::TilesCfg<4, 4>::SMEM_MAIN;
    auto kern = hgemm_pipe_kernel<BF16, 2>;
    if (!kernel_ready((const void*)kern, SMEM)) return -1;
    const int num_cus = eshkol_hip_num_cus();
    if (!A) return 0;                                        /* set-up only */
    const int tiles_m = (M + 255) / 256, tiles_n = (N + 255) / 256;
    const int n_ids = (tiles_m * tiles_n + 7) / 8 * 8;      /* padded so every XCD owns the same count */
    int grid = (num_cus / 8) * 8;
    if (grid < 8) grid = 8;
    if (grid > n_ids) grid = n_ids;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), SMEM, st,
                       A, Bt, M, N, ld_bytes, out_mode, C, tiles_m, tiles_n, n_ids);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

template <bool BF16, int TM, int TN>
int launch(const uint16_t* A, const uint16_t* Bt, int M, int N, int ld_bytes, int out_mode, void* C,
           int batch, uint64_t a_stride, uint64_t b_stride, hipStream_t st) {
    using Cf = Cfg<TM, TN>;
    auto kern = hgemm_kernel<BF16, TM, TN>;
    if (!kernel_ready((const void*)kern, Cf::SMEM_BYTES)) return -1;
    if (!A) return 0;                                        /* set-up only */
    const int tiles_m = (M + Cf::BM - 1) / Cf::BM, tiles_n = (N + Cf::BN - 1) / Cf::BN;
    const long long nwg = (long long)tiles_m * tiles_n;
    if (nwg > 0x7fffffffLL) return -1;
    /* the batch rides on the grid's y axis, at most 65535 products per launch */
    const uint64_t c_bytes = (uint64_t)M * (uint64_t)N * (out_mode == 0 ? 4u : 8u);
    for (int b0 = 0; b0 < batch; b0 += 65535) {
        const int nb = (batch - b0 < 65535) ? batch - b0 : 65535;
        hipLaunchKernelGGL(kern, dim3((unsigned)nwg, (unsigned)nb), dim3(256), Cf::SMEM_BYTES, st,
                           (const uint16_t*)((const int8_t*)A + (uint64_t)b0 * a_stride),
                           (const uint16_t*)((const int8_t*)Bt + (uint64_t)b0 * b_stride),
                           M, N, ld_bytes, out_mode, (void*)((int8_t*)C + (uint64_t)b0 * c_bytes),
                           tiles_m, tiles_n, a_stride, b_stride);
    }
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

/* batch products stored back to back: A [batch][rows_a][ld], Bt [batch][rows_b][ld]
 * (rows_a, rows_b the padded row counts), C [batch][M][N]. */
int hgemm_thin16(const uint16_t* A, const uint16_t* Bt, uint64_t M, uint64_t N, uint64_t ld,
                 int is_bf16, int out_mode, void* C, hipStream_t st);

int hgemm_any(const uint16_t* A, const uint16_t* Bt, uint64_t batch, uint64_t M, uint64_t K, uint64_t N,
              uint64_t rows_a, uint64_t rows_b, uint64_t ld,
              int is_bf16, int layout, int out_mode, void* C, hipStream_t st, bool may_use_workspace = false) {
    if (!A || !Bt || !C || M == 0 || K == 0 || N == 0 || batch == 0) return -1;
    if (M > 0x7fffffffULL || N > 0x7fffffffULL || batch > 0x7fffffffULL) return -1;
    if (ld < K || ld % 64 != 0 || ld * 2 > 0x7fffffffULL) return -1;
    if (rows_a < M || rows_b < N || rows_a % 256 != 0 || rows_b % 256 != 0) return -1;
    if (((uintptr_t)A & 15) || ((uintptr_t)Bt & 15)) return -1;
    const int m = (int)M, n = (int)N, ldb = (int)(ld * 2), nb = (int)batch;
    const uint64_t a_stride = rows_a * ld * 2, b_stride = rows_b * ld * 2;
    if (layout == 1) {
        /* interleaved operands: whole groups of four 128-byte k-blocks */
        if (ldb % 512 != 0) return -1;
        return is_bf16 ? launch_direct<true>(A, Bt, m, n, ldb, out_mode, C, nb, a_stride, b_stride, st)
                       : launch_direct<false>(A, Bt, m, n, ldb, out_mode, C, nb, a_stride, b_stride, st);
    }
    if (layout != 0) return -1;
    /* up to 128 rows against a big second operand: stream it once (callers that may use the
     * library workspace, i.e. the entry points for 16-bit operands; the f64 pipelines have
     * the kernels that read fp64 directly) */
    if (may_use_workspace && batch == 1 && M <= 128 && N >= 128 && N * ld >= (1ull << 21) &&
        hgemm_thin16(A, Bt, M, N, ld, is_bf16, out_mode, C, st) == 0) return 0;
    const long long big = (long long)((M + 255) / 256) * ((N + 255) / 256);
    /* the pipelined kernel wants whole pairs of 128-byte k-blocks and more than two per tile */
    if (batch == 1 && big >= 128 && ldb % 256 == 0 && ldb >= 512)
        return is_bf16 ? launch_pipe<true>(A, Bt, m, n, ldb, out_mode, C, st)
                       : launch_pipe<false>(A, Bt, m, n, ldb, out_mode, C, st);
    if (big * (long long)batch >= 256 && M >= 192 && N >= 192)
        return is_bf16 ? launch<true, 4, 4>(A, Bt, m, n, ldb, out_mode, C, nb, a_stride, b_stride, st)
                       : launch<false, 4, 4>(A, Bt, m, n, ldb, out_mode, C, nb, a_stride, b_stride, st);
    return is_bf16 ? launch<true, 2, 2>(A, Bt, m, n, ldb, out_mode, C, nb, a_stride, b_stride, st)
                   : launch<false, 2, 2>(A, Bt, m, n, ldb, out_mode, C, nb, a_stride, b_stride, st);
}

}  // namespace

namespace {
int g_direct16 = 1;

int convert_any(const double* in, uint16_t* out, uint64_t batch, uint64_t rows, uint64_t cols,
                uint64_t rows_padded, uint64_t ld, int is_bf16, bool kmajor, int layout, void* stream) {
    if (!in || !out || rows == 0 || cols == 0 || batch == 0 || rows_padded < rows || ld < cols || (ld & 1)) return -1;
    if (layout != 0 && layout != 1) return -1;
    if (layout == 1 && ((rows_padded & 31) || (ld & 63) || ((uintptr_t)out & 15))) return -1;
    const uint64_t nblk = kmajor ? (layout ? kmaj::il_blocks(rows_padded, ld)
                                           : kmaj::grid_blocks(rows_padded, ld, eshkol_hip_num_cus()))
                        : layout ? (rows_padded / 32) * (ld / 64) : ((ld / 2 + 255) / 256) * rows_padded;
    if (nblk > 0x7fffffffULL || (kmajor && kmaj::tile_count(rows_padded, ld) > 0x7fffffffULL)) return -1;
    hipStream_t st = (hipStream_t)stream;
    for (uint64_t b0 = 0; b0 < batch; b0 += 65535) {
        const uint64_t nb = (batch - b0 < 65535) ? batch - b0 : 65535;
        const double* x = in + b0 * rows * cols;
        uint16_t* o = out + b0 * rows_padded * ld;
        const dim3 grid((unsigned)nblk, (unsigned)nb), block(256);
        if (kmajor && layout == 1) {
            if (is_bf16) hipLaunchKernelGGL(convert_kmajor_il_kernel<true>, grid, block, 0, st, x, rows, cols, o, rows_padded, ld);
            else         hipLaunchKernelGGL(convert_kmajor_il_kernel<false>, grid, block, 0, st, x, rows, cols, o, rows_padded, ld);
        } else if (kmajor) {
            if (is_bf16) hipLaunchKernelGGL(convert_kmajor_kernel<true>, grid, block, 0, st, x, rows, cols, o, rows_padded, ld, layout);
            else         hipLaunchKernelGGL(convert_kmajor_kernel<false>, grid, block, 0, st, x, rows, cols, o, rows_padded, ld, layout);
        } else if (layout == 1) {
            if (is_bf16) hipLaunchKernelGGL(convert_il_kernel<true>, grid, block, 0, st, x, rows, cols, o, rows_padded, ld);
            else         hipLaunchKernelGGL(convert_il_kernel<false>, grid, block, 0, st, x, rows, cols, o, rows_padded, ld);
        } else {
            if (is_bf16) hipLaunchKernelGGL(convert_kernel<true>, grid, block, 0, st, x, rows, cols, o, rows_padded, ld);
            else         hipLaunchKernelGGL(convert_kernel<false>, grid, block, 0, st, x, rows, cols, o, rows_padded, ld);
        }
    }
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

/* ---- a few rows against a big second operand held as fp64 [K][N] ------------------------
 * The tier on such a product spends its time on the second operand: read once as fp64 to
 * narrow it, written as 16 bits, read again by a contraction that has a handful of tiles
 * (32 x 4096 x 4096: 92 us, of which the operand read once is 27). Here it is read once:
 * a workgroup takes a strip of 32 CW columns and a slice of k, its four waves deal the
 * slice out sixteen k at a time; a lane loads CW consecutive columns of eight rows of k
 * (the 32 lanes of a half-wave 256 CW contiguous bytes of each row), narrows them in
 * registers and has, for each of its columns, the eight consecutive k of one matrix-core
 * operand: CW instructions per block of 32 rows, column j of instruction c being column
 * CW j + c of the strip. CW = 2: strips of 64 columns measured faster than of 128 at every
 * row count (32 rows: 38 -> 31 us, 64 rows: 48 -> 36), and leave registers for the sums of
 * 128 rows. The first operand is narrowed beforehand (it is small) and its fragments come
 * from L2. Same arithmetic as the tier's other kernels (16-bit operands, fp32 sums); the
 * sums of the four waves meet in LDS, slices of k leave fp32 partial results that a second
 * kernel adds in ascending order, rounds if asked and stores. */
typedef double d4u_t __attribute__((ext_vector_type(4), aligned(8)));

template <bool BF16>
__device__ __forceinline__ void store_reduced(void* Cout, int out_mode, size_t idx, float x) {
    if (out_mode == 2) x = round16<BF16>(x);
    if (out_mode == 0) ((float*)Cout)[idx] = x;
    else ((double*)Cout)[idx] = (double)x;
}

template <bool BF16, int RB, int CW>
__global__ __launch_bounds__(256)
void reduced_thin_kernel(const uint16_t* __restrict__ A16, int lda, int M,
                         const double* __restrict__ B, int K, int N, int kc,
                         float* __restrict__ part, long slice_stride, void* Cout, int out_mode, long c_r, long c_o) {
    __shared__ v4f_t red[4][4][64];
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, lh = lane >> 5;
    typedef double dcu_t __attribute__((ext_vector_type(CW), aligned(8)));
    const int n0 = (int)blockIdx.x * (32 * CW), col = n0 + CW * li;
    const int ks = (int)blockIdx.y * kc;
    const int ke = (ks + kc < K) ? ks + kc : K;
    const bool edge = n0 + 32 * CW > N;                              /* the same for the whole workgroup */
    int oc[CW];
#pragma unroll
    for (int c = 0; c < CW; c++) oc[c] = (col + c < N) ? col + c : N - 1;
    v16f_t acc[RB][CW];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int c = 0; c < CW; c++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[rb][c][r] = 0.0f;

    for (int k0 = ks + 16 * wave; k0 < ke; k0 += 64) {
        const int kk = k0 + 8 * lh;
        double v[8][CW];
        if (k0 + 16 <= ke && !edge) {                           /* the same for the whole wave */
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const dcu_t x = *(const dcu_t*)(B + (size_t)(kk + j) * N + col);
#pragma unroll
                for (int c = 0; c < CW; c++) v[j][c] = x[c];
            }
        } else {
            /* the last, partial round of the slice and the last strip: clamped addresses,
             * zeros beyond the slice (the first operand is not zero there) */
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const bool in = kk + j < ke;
                const size_t kr = (size_t)(in ? kk + j : ke - 1);
#pragma unroll
                for (int c = 0; c < CW; c++) { const double x = B[kr * N + oc[c]]; v[j][c] = in ? x : 0.0; }
            }
        }
        v4i_t op[CW];
#pragma unroll
        for (int c = 0; c < CW; c++)
#pragma unroll
            for (int q = 0; q < 4; q++) op[c][q] = (int)narrow_pair<BF16>(v[2 * q][c], v[2 * q + 1][c]);
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            const v4i_t a = *(const v4i_t*)(A16 + (size_t)(rb * 32 + li) * lda + kk);
#pragma unroll
            for (int c = 0; c < CW; c++) H16Op<BF16>::mfma(op[c], a, acc[rb][c]);
        }
    }
    /* acc[rb][c]: lane%32 is the output row, registers 4v .. 4v+3 are columns j = 8v + 4 (lane/32) + 0..3
     * of instruction c, i.e. columns n0 + CW j + c. One (rb, c) at a time through LDS. */
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
#pragma unroll
        for (int c = 0; c < CW; c++) {
            if (rb + c) __syncthreads();
#pragma unroll
            for (int vv = 0; vv < 4; vv++)
                red[wave][vv][lane] = (v4f_t){acc[rb][c][4 * vv], acc[rb][c][4 * vv + 1], acc[rb][c][4 * vv + 2], acc[rb][c][4 * vv + 3]};
            __syncthreads();
            const int row = rb * 32 + li;
            if (row >= M) continue;                              /* the barriers sit above */
            v4f_t s = red[0][wave][lane];
#pragma unroll
            for (int w = 1; w < 4; w++) s += red[w][wave][lane];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int cx = n0 + CW * (8 * wave + 4 * lh + e) + c;
                if (cx >= N) continue;
                if (part) part[(size_t)blockIdx.y * slice_stride + (size_t)row * N + cx] = s[e];
                else store_reduced<BF16>(Cout, out_mode, (size_t)((long)row * c_r + (long)cx * c_o), s[e]);
            }
        }
    }
}

/* The same against a big operand with k contiguous, G[O][K] (the second operand held
 * transposed, or a matrix against a few columns): a lane loads eight consecutive k of one
 * output's row (64 bytes; the two halves of a wave the sixteen k of a round) and narrows
 * them into one matrix-core operand; a workgroup's strip is NB blocks of 32 outputs. */
/* G16: the big operand is 16-bit already (rows of ldg elements, zero padded in k and in rows,
 * as hip_hgemm_16 takes its operands): loaded as it is, K counts the padded k. */
template <bool BF16, int RB, int NB, bool G16 = false>
__global__ __launch_bounds__(256)
void reduced_thin_klast_kernel(const uint16_t* __restrict__ T16, int ldt, int R,
                               const void* __restrict__ Gv, int K, int O, int kc,
                               float* __restrict__ part, long slice_stride, void* Cout, int out_mode, long c_r, long c_o) {
    __shared__ v4f_t red[4][4][64];
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, lh = lane >> 5;
    const int o0 = (int)blockIdx.x * (32 * NB);
    const int ks = (int)blockIdx.y * kc;
    const int ke = (ks + kc < K) ? ks + kc : K;
    size_t g_off[NB];
#pragma unroll
    for (int cb = 0; cb < NB; cb++) {
        const int o = o0 + 32 * cb + li;
        g_off[cb] = (size_t)(o < O ? o : O - 1) * K;            /* rows beyond the operand repeat the last: never stored */
    }
    const double* G = (const double*)Gv;
    const uint16_t* Gh = (const uint16_t*)Gv;
    v16f_t acc[RB][NB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int cb = 0; cb < NB; cb++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[rb][cb][r] = 0.0f;

    for (int k0 = ks + 16 * wave; k0 < ke; k0 += 64) {
        const int kk = k0 + 8 * lh;
        v4i_t op[NB];
        if (G16) {
#pragma unroll
            for (int cb = 0; cb < NB; cb++) op[cb] = *(const v4i_t*)(Gh + g_off[cb] + kk);
        } else if (k0 + 16 <= ke) {                             /* the same for the whole wave */
#pragma unroll
            for (int cb = 0; cb < NB; cb++) {
                const d4u_t x0 = *(const d4u_t*)(G + g_off[cb] + kk), x1 = *(const d4u_t*)(G + g_off[cb] + kk + 4);
                op[cb] = (v4i_t){(int)narrow_pair<BF16>(x0[0], x0[1]), (int)narrow_pair<BF16>(x0[2], x0[3]),
                                 (int)narrow_pair<BF16>(x1[0], x1[1]), (int)narrow_pair<BF16>(x1[2], x1[3])};
            }
        } else {
#pragma unroll
            for (int cb = 0; cb < NB; cb++) {
                double x[8];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const bool in = kk + j < ke;
                    const double g = G[g_off[cb] + (in ? kk + j : ke - 1)];
                    x[j] = in ? g : 0.0;
                }
                op[cb] = (v4i_t){(int)narrow_pair<BF16>(x[0], x[1]), (int)narrow_pair<BF16>(x[2], x[3]),
                                 (int)narrow_pair<BF16>(x[4], x[5]), (int)narrow_pair<BF16>(x[6], x[7])};
            }
        }
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            const v4i_t a = *(const v4i_t*)(T16 + (size_t)(rb * 32 + li) * ldt + kk);
#pragma unroll
            for (int cb = 0; cb < NB; cb++) H16Op<BF16>::mfma(op[cb], a, acc[rb][cb]);
        }
    }
    /* acc[rb][cb]: lane%32 is the thin row, registers 4v .. 4v+3 are outputs o0 + 32 cb + 8v + 4 (lane/32) + 0..3 */
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
#pragma unroll
        for (int cb = 0; cb < NB; cb++) {
            if (rb + cb) __syncthreads();
#pragma unroll
            for (int vv = 0; vv < 4; vv++)
                red[wave][vv][lane] = (v4f_t){acc[rb][cb][4 * vv], acc[rb][cb][4 * vv + 1], acc[rb][cb][4 * vv + 2], acc[rb][cb][4 * vv + 3]};
            __syncthreads();
            const int row = rb * 32 + li;
            if (row >= R) continue;                              /* the barriers sit above */
            v4f_t s = red[0][wave][lane];
#pragma unroll
            for (int w = 1; w < 4; w++) s += red[w][wave][lane];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int o = o0 + 32 * cb + 8 * wave + 4 * lh + e;
                if (o >= O) continue;
                if (part) part[(size_t)blockIdx.y * slice_stride + (size_t)row * O + o] = s[e];
                else store_reduced<BF16>(Cout, out_mode, (size_t)((long)row * c_r + (long)o * c_o), s[e]);
            }
        }
    }
}

/* C(r, o) = the slices' partial sums [slice][r][o] added in ascending order, rounded if asked */
template <bool BF16>
__global__ __launch_bounds__(256)
void reduced_thin_sum_kernel(const float* __restrict__ part, int slices, long n, int O, void* Cout, int out_mode,
                             long c_r, long c_o) {
    const long e = (long)blockIdx.x * 256 + threadIdx.x;
    if (e >= n) return;
    float s = 0.0f;
    int y = 0;
    for (; y + 8 <= slices; y += 8) {                            /* eight loads in flight, added in ascending order */
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = part[(size_t)(y + u) * n + e];
#pragma unroll
        for (int u = 0; u < 8; u++) s += v[u];
    }
    for (; y < slices; y++) s += part[(size_t)y * n + e];
    const long r = e / O, o = e - r * O;
    store_reduced<BF16>(Cout, out_mode, (size_t)(r * c_r + o * c_o), s);
}

int g_reduced_thin = 1;

/* Slices of k for the kernels above: about three workgroups per CU, at least 256 k each
 * (128 where the strips are few), at most 64 slices. By the shape alone. R: rows on the
 * thin side, O: outputs on the wide one. */
struct ThinPlan { int slices, kc; size_t part_bytes; };
ThinPlan reduced_thin_plan(uint64_t R, uint64_t K, uint64_t O) {
    const int width = 64;           /* outputs per strip */
    const int strips = (int)((O + width - 1) / width);
    const int min_kc = strips <= 4 ? 128 : 256;
    int slices = (3 * eshkol_hip_num_cus()) / strips;
    if (slices > (int)(K / min_kc)) slices = (int)(K / min_kc);
    if (slices > 64) slices = 64;
    if (slices < 1) slices = 1;
    int kc = (int)((K + slices - 1) / slices);
    kc = (kc + 63) / 64 * 64;
    slices = (int)((K + kc - 1) / kc);
    return { slices, kc, slices > 1 ? (size_t)slices * R * O * sizeof(float) : 0 };
}

/* up to 128 rows (or columns) against a big operand that is worth streaming, every operand
 * form; everything else keeps the narrowing kernels and the tiled contraction */
bool reduced_is_thin(uint64_t batch, uint64_t M, uint64_t K, uint64_t N) {
    const uint64_t thin = M <= N ? M : N, wide = M <= N ? N : M;
    return g_reduced_thin && batch == 1 && thin <= 128 && wide >= 128 && K >= 64 && wide * K >= (1ull << 21) &&
           K <= 0x3fffff00ULL && wide <= 0x7fffff00ULL;
}
ThinPlan reduced_thin_plan_for(uint64_t M, uint64_t K, uint64_t N) {
    return M <= N ? reduced_thin_plan(M, K, N) : reduced_thin_plan(N, K, M);
}

/* T16: 128 rows of ld elements for the thin operand's 16-bit copy, written here; part:
 * reduced_thin_plan_for().part_bytes. */
int reduced_thin(const double* A, const double* B, double* C, uint64_t M, uint64_t K, uint64_t N, int trans_a, int trans_b,
                 int is_bf16, int round_output, uint16_t* T16, uint64_t ld, float* part, hipStream_t st) {
    const bool thin_m = M <= N;
    const uint64_t R = thin_m ? M : N, O = thin_m ? N : M;
    /* the thin operand as rows of k: A (k-major when the caller holds A^T), or B's columns
     * (k-major as the runtime stores B, rows of k when the caller holds B^T) */
    const double* T = thin_m ? A : B;
    const bool t_kmajor = thin_m ? trans_a != 0 : trans_b == 0;
    if (convert_any(T, T16, 1, R, K, 128, ld, is_bf16, t_kmajor, 0, st) != 0) return -1;
    const double* G = thin_m ? B : A;
    const bool kfirst = thin_m ? trans_b == 0 : trans_a != 0;    /* the big operand has the output index contiguous */
    const long c_r = thin_m ? (long)N : 1, c_o = thin_m ? 1 : (long)N;
    const ThinPlan pl = reduced_thin_plan(R, K, O);
    const int width = 64;
    const dim3 grid((unsigned)((O + width - 1) / width), (unsigned)pl.slices);
    const int out_mode = round_output ? 2 : 1;
    float* p = pl.slices > 1 ? part : nullptr;
    const long stride = (long)(R * O);
#define THIN(KERN, BF, RB, W) hipLaunchKernelGGL((KERN<BF, RB, W>), grid, dim3(256), 0, st, T16, (int)ld, (int)R, G, (int)K, \
                                                 (int)O, pl.kc, p, stride, (void*)C, out_mode, c_r, c_o)
#define THIN_BY_ROWS(KERN, BF) do { if (R <= 32) THIN(KERN, BF, 1, 2); else if (R <= 64) THIN(KERN, BF, 2, 2); \
                                    else if (R <= 96) THIN(KERN, BF, 3, 2); else THIN(KERN, BF, 4, 2); } while (0)
    if (kfirst) { if (is_bf16) THIN_BY_ROWS(reduced_thin_kernel, true); else THIN_BY_ROWS(reduced_thin_kernel, false); }
    else        { if (is_bf16) THIN_BY_ROWS(reduced_thin_klast_kernel, true); else THIN_BY_ROWS(reduced_thin_klast_kernel, false); }
#undef THIN_BY_ROWS
#undef THIN
    if (p) {
        const long n = (long)(R * O);
        const dim3 sgrid((unsigned)((n + 255) / 256));
        if (is_bf16) hipLaunchKernelGGL(reduced_thin_sum_kernel<true>, sgrid, dim3(256), 0, st, p, pl.slices, n, (int)O, (void*)C, out_mode, c_r, c_o);
        else         hipLaunchKernelGGL(reduced_thin_sum_kernel<false>, sgrid, dim3(256), 0, st, p, pl.slices, n, (int)O, (void*)C, out_mode, c_r, c_o);
    }
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

/* hip_hgemm_16 on up to 128 rows: A [rows padded][ld] and Bt [rows padded][ld] 16-bit, zero
 * padded; the big operand streamed once by the kernel for k-contiguous operands. */
int hgemm_thin16(const uint16_t* A, const uint16_t* Bt, uint64_t M, uint64_t N, uint64_t ld,
                 int is_bf16, int out_mode, void* C, hipStream_t st) {
    if (!g_reduced_thin) return -1;
    const ThinPlan pl = reduced_thin_plan(M, ld, N);
    float* p = nullptr;
    if (pl.slices > 1) {
        p = (float*)eshkol_hip_workspace(WS_DGEMM_PARTIAL, pl.part_bytes);
        if (!p) return -1;
    }
    const dim3 grid((unsigned)((N + 63) / 64), (unsigned)pl.slices);
    const long stride = (long)(M * N), c_r = (long)N, c_o = 1;
#define THIN16(BF, RB) hipLaunchKernelGGL((reduced_thin_klast_kernel<BF, RB, 2, true>), grid, dim3(256), 0, st, A, (int)ld, (int)M, \
                                          (const void*)Bt, (int)ld, (int)N, pl.kc, p, stride, C, out_mode, c_r, c_o)
#define THIN16_BY_ROWS(BF) do { if (M <= 32) THIN16(BF, 1); else if (M <= 64) THIN16(BF, 2); else if (M <= 96) THIN16(BF, 3); else THIN16(BF, 4); } while (0)
    if (is_bf16) THIN16_BY_ROWS(true); else THIN16_BY_ROWS(false);
#undef THIN16_BY_ROWS
#undef THIN16
    if (p) {
        const long n = (long)(M * N);
        const dim3 sgrid((unsigned)((n + 255) / 256));
        if (is_bf16) hipLaunchKernelGGL(reduced_thin_sum_kernel<true>, sgrid, dim3(256), 0, st, p, pl.slices, n, (int)N, C, out_mode, c_r, c_o);
        else         hipLaunchKernelGGL(reduced_thin_sum_kernel<false>, sgrid, dim3(256), 0, st, p, pl.slices, n, (int)N, C, out_mode, c_r, c_o);
    }
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

/* Padded operand shape and plane layout of the reduced tier for a batch of
 * M x K x N products: interleaved 16-bit operands (and a k pitch of whole
 * 512-byte groups) when the launch has enough 256 x 256 tiles for the
 * direct-to-LDS kernel and the matrices are not much smaller than a tile. */
struct ReducedShape { uint64_t Mp, Np, ld; int layout; };
ReducedShape reduced_shape(uint64_t batch, uint64_t M, uint64_t K, uint64_t N) {
    ReducedShape r;
    r.Mp = round_up_sz(M, 256); r.Np = round_up_sz(N, 256);
    r.layout = hip_hgemm_plane_layout(M, N, batch);
    r.ld = round_up_sz(K, r.layout ? 256 : 128);
    return r;
}

/* Narrow both operands into the 16-bit copies A16 [batch][Mp][ld] and B16
 * [batch][Np][ld] the caller provides (every element of both, padding included,
 * is written), then multiply. One stored k-major (B as given, A when the caller
 * holds A^T) is narrowed through LDS tiles, so no transposed fp64 copy is made. */
int reduced_pipeline(const double* A, const double* B, double* C, uint64_t batch, uint64_t M, uint64_t K, uint64_t N,
                     int trans_a, int trans_b, int is_bf16, int round_output,
                     uint16_t* A16, uint16_t* B16, const ReducedShape& sh, hipStream_t st) {
    if (convert_any(A, A16, batch, M, K, sh.Mp, sh.ld, is_bf16, trans_a != 0, sh.layout, st) != 0) return -1;
    if (convert_any(B, B16, batch, N, K, sh.Np, sh.ld, is_bf16, trans_b == 0, sh.layout, st) != 0) return -1;
    return hgemm_any(A16, B16, batch, M, K, N, sh.Mp, sh.Np, sh.ld, is_bf16, sh.layout, round_output ? 2 : 1, C, st);
}
}  // namespace

/* Tuning hook: 0 keeps the 16-bit tier on row-major operands and the
 * register-staged kernels. Same results. */
extern "C" void hip_hgemm_set_direct(int on) { EshkolHipLock lk; g_direct16 = on ? 1 : 0; }
/* Tuning hook: 0 keeps a few rows against a big second operand on the narrowing kernels
 * and the tiled contraction. Same arithmetic, another order of the fp32 sums. */
extern "C" void hip_reduced_set_thin(int on) { EshkolHipLock lk; g_reduced_thin = on ? 1 : 0; }

extern "C" int hip_hgemm_plane_layout(uint64_t M, uint64_t N, uint64_t batch) {
    const uint64_t tiles = ((M + 255) / 256) * ((N + 255) / 256) * batch;
    return (g_direct16 && tiles >= 128 && M >= 192 && N >= 192) ? 1 : 0;
}

extern "C" int hip_convert_f64_to_16(const double* in, uint16_t* out, uint64_t rows, uint64_t cols,
                                     uint64_t rows_padded, uint64_t ld, int is_bf16, void* stream) {
    return convert_any(in, out, 1, rows, cols, rows_padded, ld, is_bf16, false, 0, stream);
}

extern "C" int hip_convert_f64_to_16_kmajor(const double* in, uint16_t* out, uint64_t rows, uint64_t cols,
                                            uint64_t rows_padded, uint64_t ld, int is_bf16, void* stream) {
    return convert_any(in, out, 1, rows, cols, rows_padded, ld, is_bf16, true, 0, stream);
}

extern "C" int hip_convert_f64_to_16_planes(const double* in, uint16_t* out, uint64_t batch, uint64_t rows, uint64_t cols,
                                            uint64_t rows_padded, uint64_t ld, int is_bf16,
                                            int kmajor, int layout, void* stream) {
    return convert_any(in, out, batch, rows, cols, rows_padded, ld, is_bf16, kmajor != 0, layout, stream);
}

extern "C" int hip_hgemm_16(const uint16_t* A, const uint16_t* Bt, uint64_t M, uint64_t K, uint64_t N,
                            uint64_t ld, int is_bf16, float* C, void* stream) {
    EshkolHipCall bracket(stream);
    return hgemm_any(A, Bt, 1, M, K, N, round_up_sz(M, 256), round_up_sz(N, 256), ld, is_bf16, 0, 0, C, (hipStream_t)stream, true);
}

extern "C" int hip_hgemm_16_batched(const uint16_t* A, const uint16_t* Bt, uint64_t batch,
                                    uint64_t M, uint64_t K, uint64_t N,
                                    uint64_t rows_a_padded, uint64_t rows_b_padded, uint64_t ld,
                                    int is_bf16, int layout, float* C, void* stream) {
    EshkolHipCall bracket(stream);
    return hgemm_any(A, Bt, batch, M, K, N, rows_a_padded, rows_b_padded, ld, is_bf16, layout, 0, C, (hipStream_t)stream, true);
}

extern "C" int hip_matmul_reduced_f64_batched_ex(const double* A, const double* B, double* C,
                                                 uint64_t batch, uint64_t M, uint64_t K, uint64_t N,
                                                 int trans_a, int trans_b,
                                                 int dtype, int round_output, void* stream) {
    EshkolHipCall bracket(stream);
    if (!A || !B || !C || M == 0 || K == 0 || N == 0 || batch == 0) return -1;
    if (dtype != 2 && dtype != 3) return -1;
    if (M > 0x7fffffffULL || K > 0x3fffffffULL || N > 0x7fffffffULL || batch > 0x7fffffffULL) return -1;
    hipStream_t st = (hipStream_t)stream;
    const ReducedShape sh = reduced_shape(batch, M, K, N);
    if (reduced_is_thin(batch, M, K, N)) {
        /* a few rows or columns: the big operand is read once, as fp64, and never copied */
        const ThinPlan pl = reduced_thin_plan_for(M, K, N);
        uint16_t* A16 = (uint16_t*)eshkol_hip_workspace(WS_HALF_A, 128 * sh.ld * 2);
        float* part = pl.part_bytes ? (float*)eshkol_hip_workspace(WS_DGEMM_PARTIAL, pl.part_bytes) : nullptr;
        if (A16 && (part || !pl.part_bytes))
            return reduced_thin(A, B, C, M, K, N, trans_a, trans_b, dtype == 3, round_output, A16, sh.ld, part, st);
    }
    uint16_t* A16 = (uint16_t*)eshkol_hip_workspace(WS_HALF_A, batch * sh.Mp * sh.ld * 2);
    uint16_t* B16 = (uint16_t*)eshkol_hip_workspace(WS_HALF_B, batch * sh.Np * sh.ld * 2);
    if (!A16 || !B16) return -1;
    return reduced_pipeline(A, B, C, batch, M, K, N, trans_a, trans_b, dtype == 3, round_output, A16, B16, sh, st);
}

extern "C" int hip_matmul_reduced_f64_batched(const double* A, const double* B, double* C,
                                              uint64_t batch, uint64_t M, uint64_t K, uint64_t N,
                                              int dtype, int round_output, void* stream) {
    return hip_matmul_reduced_f64_batched_ex(A, B, C, batch, M, K, N, 0, 0, dtype, round_output, stream);
}

extern "C" int hip_matmul_reduced_f64_ex(const double* A, const double* B, double* C,
                                         uint64_t M, uint64_t K, uint64_t N,
                                         int trans_a, int trans_b,
                                         int dtype, int round_output, void* stream) {
    return hip_matmul_reduced_f64_batched_ex(A, B, C, 1, M, K, N, trans_a, trans_b, dtype, round_output, stream);
}

/* ---- the reduced tier without any allocation ------------------------------------
 * The 16-bit operand copies live in a device array that is part of the code
 * object, so the call reaches neither hipMalloc nor the grow-only workspace.
 * Host code never uses the array's name as an address: each device holds its
 * own copy, whose address hipGetSymbolAddress returns once per device. */
namespace {
constexpr size_t NOALLOC_SCRATCH_BYTES = 32u << 20;
constexpr int NOALLOC_MAX_DEVICES = 16;
__device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];
unsigned char* g_scratch_ptr[NOALLOC_MAX_DEVICES] = {};
std::mutex g_scratch_mutex;

/* The current device's copy of the array, or NULL. */
unsigned char* noalloc_scratch(void) {
    int dev = -1;
    if (!ESHKOL_HIP_OK(hipGetDevice(&dev)) || dev < 0 || dev >= NOALLOC_MAX_DEVICES) return nullptr;
    std::lock_guard<std::mutex> lk(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        if (!ESHKOL_HIP_OK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch))) || !ptr) {
            (void)hipGetLastError();
            return nullptr;
        }
        g_scratch_ptr[dev] = (unsigned char*)ptr;
    }
    return g_scratch_ptr[dev];
}
}  // namespace

/* Everything hip_matmul_reduced_f64_noalloc would otherwise do on its first
 * call with some shape: the scratch address, every contraction kernel's LDS
 * attribute, the CU count. After it the entry point only launches kernels. */
int eshkol_hip_noalloc_setup(void) {
    if (!noalloc_scratch()) return -1;
    (void)eshkol_hip_num_cus();
    int rc = 0;
    rc |= launch_direct<true>(nullptr, nullptr, 0, 0, 0, 0, nullptr, 0, 0, 0, nullptr);
    rc |= launch_direct<false>(nullptr, nullptr, 0, 0, 0, 0, nullptr, 0, 0, 0, nullptr);
    rc |= launch_pipe<true>(nullptr, nullptr, 0, 0, 0, 0, nullptr, nullptr);
    rc |= launch_pipe<false>(nullptr, nullptr, 0, 0, 0, 0, nullptr, nullptr);
    rc |= launch<true, 4, 4>(nullptr, nullptr, 0, 0, 0, 0, nullptr, 0, 0, 0, nullptr);
    rc |= launch<false, 4, 4>(nullptr, nullptr, 0, 0, 0, 0, nullptr, 0, 0, 0, nullptr);
    rc |= launch<true, 2, 2>(nullptr, nullptr, 0, 0, 0, 0, nullptr, 0, 0, 0, nullptr);
    rc |= launch<false, 2, 2>(nullptr, nullptr, 0, 0, 0, 0, nullptr, 0, 0, 0, nullptr);
    return rc == 0 ? 0 : -1;
}

extern "C" size_t hip_matmul_reduced_f64_noalloc_limit(void) { return NOALLOC_SCRATCH_BYTES; }

extern "C" int hip_matmul_reduced_f64_noalloc(const double* A, const double* B, double* C,
                                              uint64_t M, uint64_t K, uint64_t N,
                                              int dtype, int round_output, void* stream) {
    if (!A || !B || !C || M == 0 || K == 0 || N == 0) return -1;
    if (dtype != 2 && dtype != 3) return -1;
    if (M > 0x7fffffffULL || K > 0x3fffffffULL || N > 0x7fffffffULL) return -1;
    const ReducedShape sh = reduced_shape(1, M, K, N);
    const uint64_t a_bytes = sh.Mp * sh.ld * 2, b_bytes = sh.Np * sh.ld * 2;          /* multiples of 256 */
    if (a_bytes + b_bytes > NOALLOC_SCRATCH_BYTES) {
        fprintf(stderr, "[GPU] hip_matmul_reduced_f64_noalloc: %llux%llux%llu needs %llu bytes of 16-bit "
                        "operand copies, the static scratch holds %llu; use hip_matmul_reduced_f64\n",
                (unsigned long long)M, (unsigned long long)K, (unsigned long long)N,
                (unsigned long long)(a_bytes + b_bytes), (unsigned long long)NOALLOC_SCRATCH_BYTES);
        return -3;
    }
    unsigned char* base = noalloc_scratch();
    if (!base) return -1;
    if (reduced_is_thin(1, M, K, N)) {
        /* the same kernel and slices as the workspace entry point: the thin operand's 128
         * rows of 16-bit values and the fp32 partial sums take the place of the copies */
        const ThinPlan pl = reduced_thin_plan_for(M, K, N);
        const uint64_t a16 = round_up_sz(128 * sh.ld * 2, 256);
        if (a16 + pl.part_bytes > NOALLOC_SCRATCH_BYTES) {
            fprintf(stderr, "[GPU] hip_matmul_reduced_f64_noalloc: %llux%llux%llu needs %llu bytes of partial sums, "
                            "the static scratch holds %llu; use hip_matmul_reduced_f64\n",
                    (unsigned long long)M, (unsigned long long)K, (unsigned long long)N,
                    (unsigned long long)(a16 + pl.part_bytes), (unsigned long long)NOALLOC_SCRATCH_BYTES);
            return -3;
        }
        return reduced_thin(A, B, C, M, K, N, 0, 0, dtype == 3, round_output, (uint16_t*)base, sh.ld,
                            (float*)(base + a16), (hipStream_t)stream);
    }
    return reduced_pipeline(A, B, C, 1, M, K, N, 0, 0, dtype == 3, round_output,
                            (uint16_t*)base, (uint16_t*)(base + a_bytes), sh, (hipStream_t)stream);
}

extern "C" int hip_matmul_reduced_f64(const double* A, const double* B, double* C,
                                      uint64_t M, uint64_t K, uint64_t N,
                                      int dtype, int round_output, void* stream) {
    return hip_matmul_reduced_f64_ex(A, B, C, M, K, N, 0, 0, dtype, round_output, stream);
}
