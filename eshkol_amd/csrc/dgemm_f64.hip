/*
 * Native fp64 tier: C[MxN] = A[MxK] * B[KxN], row-major, on the gfx950 matrix
 * cores (v_mfma_f64_16x16x4_f64). Takes the place of the cublasDgemm call of
 * the reference (lib/backend/gpu/gpu_memory_cuda.cpp:633-640).
 *
 * Work decomposition
 *   workgroup  256 threads = 4 waves in a 2x2 grid, block tile BM x BN, BK = 16
 *   wave       (BM/2) x (BN/2) = TM x TN MFMA tiles of 16x16, fp64 accumulators
 *              in registers
 *   LDS        double-buffered: A tile [BM][16(+2)] k-contiguous, B tile
 *              [16][BN(+4)] n-contiguous; the pads make every ds_read hit
 *              distinct banks
 *   pipeline   global loads of block kb+1 are issued before the MFMAs of block
 *              kb and written to the other LDS buffer after them: one barrier
 *              per k-block
 *
 * k-order inside a k-block: lane group g = lane/16 feeds k = 4g+s at MFMA step
 * s for both operands, so a lane reads its four A values as two 16-byte LDS
 * loads. Summation order therefore differs from a k-ascending loop; the tier's
 * contract is the normwise bound, not bitwise order.
 *
 * Workgroup ids are remapped so that each XCD (ids congruent mod 8 land on the
 * same XCD) walks a contiguous run of tiles, grouped 8 tile-rows at a time, so
 * concurrently resident workgroups share A rows and B columns in that XCD's L2.
 */
#include "hip_common.h"
#include "kernels.h"

typedef double d4_t __attribute__((ext_vector_type(4)));
typedef double d2_t __attribute__((ext_vector_type(2)));

namespace {

constexpr int BK = 16;
constexpr int LDA_S = BK + 2;      /* doubles per A row in LDS: 144 B */

template <int BM, int BN> struct Tile {
    static constexpr int LDB_S = BN + 4;              /* doubles per B row in LDS */
    static constexpr int A_TILE = BM * LDA_S;
    static constexpr int B_TILE = BK * LDB_S;
    static constexpr int SMEM_BYTES = 2 * (A_TILE + B_TILE) * (int)sizeof(double);
    static constexpr int TM = BM / 32;                /* 16x16 tiles per wave, rows */
    static constexpr int TN = BN / 32;
    static constexpr int A_CHUNKS = BM * BK / 2 / 256; /* 16-byte chunks per thread */
    static constexpr int B_CHUNKS = BK * BN / 2 / 256;
};

__device__ __forceinline__ void tile_of_workgroup(int tiles_m, int tiles_n, int* tm, int* tn) {
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
    *tm = first_m + in_group % gsize;
    *tn = in_group / gsize;
}

/* VEC: K and N even and A, B 16-byte aligned, so operands move as 16-byte pairs. */
template <int BM, int BN, bool VEC>
__global__ __launch_bounds__(256)
void dgemm_mfma_kernel(const double* __restrict__ A, const double* __restrict__ B,
                       double* __restrict__ C, int M, int N, int K,
                       int tiles_m, int tiles_n) {
    using T = Tile<BM, BN>;
    extern __shared__ __align__(16) double smem[];
    double* As = smem;
    double* Bs = smem + 2 * T::A_TILE;

    int tm, tn;
    tile_of_workgroup(tiles_m, tiles_n, &tm, &tn);
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 15, lg = lane >> 4;

    d2_t ra[T::A_CHUNKS], rb[T::B_CHUNKS];

    auto gload = [&](int kb) {
        const int k0 = kb * BK;
#pragma unroll
        for (int r = 0; r < T::A_CHUNKS; r++) {
            const int c = tid + 256 * r;
            const int row = c >> 3, kc = c & 7;
            const int gr = m0 + row, gk = k0 + 2 * kc;
            const double* p = A + (size_t)gr * K + gk;
            d2_t v = {0.0, 0.0};
            if (VEC) {
                if (gr < M && gk < K) v = *(const d2_t*)p;
            } else {
                if (gr < M && gk < K) v.x = p[0];
                if (gr < M && gk + 1 < K) v.y = p[1];
            }
            ra[r] = v;
        }
#pragma unroll
        for (int r = 0; r < T::B_CHUNKS; r++) {
            const int c = tid + 256 * r;
            const int kr = c / (BN / 2), nc = c % (BN / 2);
            const int gk = k0 + kr, gn = n0 + 2 * nc;
            const double* p = B + (size_t)gk * N + gn;
            d2_t v = {0.0, 0.0};
            if (VEC) {
                if (gk < K && gn < N) v = *(const d2_t*)p;
            } else {
                if (gk < K && gn < N) v.x = p[0];
                if (gk < K && gn + 1 < N) v.y = p[1];
            }
            rb[r] = v;
        }
    };
    auto sstore = [&](int buf) {
#pragma unroll
        for (int r = 0; r < T::A_CHUNKS; r++) {
            const int c = tid + 256 * r;
            const int row = c >> 3, kc = c & 7;
            *(d2_t*)(As + buf * T::A_TILE + row * LDA_S + 2 * kc) = ra[r];
        }
#pragma unroll
        for (int r = 0; r < T::B_CHUNKS; r++) {
            const int c = tid + 256 * r;
            const int kr = c / (BN / 2), nc = c % (BN / 2);
            *(d2_t*)(Bs + buf * T::B_TILE + kr * T::LDB_S + 2 * nc) = rb[r];
        }
    };

    d4_t acc[T::TM][T::TN];
#pragma unroll
    for (int t = 0; t < T::TM; t++)
#pragma unroll
        for (int u = 0; u < T::TN; u++) acc[t][u] = (d4_t){0.0, 0.0, 0.0, 0.0};

    const int nkb = (K + BK - 1) / BK;
    gload(0);
    sstore(0);
    __syncthreads();

    int cur = 0;
    for (int kb = 0; kb < nkb; kb++) {
        const bool more = (kb + 1 < nkb);
        if (more) gload(kb + 1);

        const double* a_base = As + cur * T::A_TILE + (wm * (BM / 2) + li) * LDA_S + 4 * lg;
        const double* b_base = Bs + cur * T::B_TILE + (4 * lg) * T::LDB_S + wn * (BN / 2) + li;

        d2_t a_lo[T::TM], a_hi[T::TM];
#pragma unroll
        for (int t = 0; t < T::TM; t++) {
            a_lo[t] = *(const d2_t*)(a_base + t * 16 * LDA_S);
            a_hi[t] = *(const d2_t*)(a_base + t * 16 * LDA_S + 2);
        }
#pragma unroll
        for (int s = 0; s < 4; s++) {
            double b[T::TN];
#pragma unroll
            for (int u = 0; u < T::TN; u++) b[u] = b_base[s * T::LDB_S + u * 16];
#pragma unroll
            for (int t = 0; t < T::TM; t++) {
                const double a = (s == 0) ? a_lo[t].x : (s == 1) ? a_lo[t].y
                               : (s == 2) ? a_hi[t].x : a_hi[t].y;
#pragma unroll
                for (int u = 0; u < T::TN; u++)
                    acc[t][u] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b[u], acc[t][u], 0, 0, 0);
            }
        }

        if (more) sstore(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }

    /* accumulator layout: register r of the lane is row 4*r + lane/16, column lane%16 */
#pragma unroll
    for (int t = 0; t < T::TM; t++)
#pragma unroll
        for (int u = 0; u < T::TN; u++) {
            const int col = n0 + wn * (BN / 2) + u * 16 + li;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int row = m0 + wm * (BM / 2) + t * 16 + 4 * r + lg;
                if (row < M && col < N) C[(size_t)row * N + col] = acc[t][u][r];
            }
        }
}

template <int BM, int BN, bool VEC>
int launch(const double* A, const double* B, double* C, int M, int N, int K, hipStream_t st) {
    using T = Tile<BM, BN>;
    static bool attr_set = false;
    auto kern = dgemm_mfma_kernel<BM, BN, VEC>;
    if (!attr_set) {
        if (!ESHKOL_HIP_OK(hipFuncSetAttribute((const void*)kern,
                hipFuncAttributeMaxDynamicSharedMemorySize, T::SMEM_BYTES))) return -1;
        attr_set = true;
    }
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const long long nwg = (long long)tiles_m * tiles_n;
    if (nwg > 0x7fffffffLL) return -1;
    hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(256), T::SMEM_BYTES, st,
                       A, B, C, M, N, K, tiles_m, tiles_n);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

}  // namespace

extern "C" int hip_dgemm_f64(const double* A, const double* B, double* C,
                             uint64_t M, uint64_t K, uint64_t N, void* stream) {
    if (!A || !B || !C || M == 0 || K == 0 || N == 0) return -1;
    if (M > 0x7fffffffULL || K > 0x7fffffffULL || N > 0x7fffffffULL) return -1;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = (K % 2 == 0) && (N % 2 == 0) &&
                     ((uintptr_t)A % 16 == 0) && ((uintptr_t)B % 16 == 0);
    const int m = (int)M, n = (int)N, k = (int)K;
    /* Small outputs cannot fill 256 CUs with 128x128 tiles: use 64x64 there. */
    const long long big_tiles = (long long)((M + 127) / 128) * (long long)((N + 127) / 128);
    if (big_tiles >= 256) {
        return vec ? launch<128, 128, true>(A, B, C, m, n, k, st)
                   : launch<128, 128, false>(A, B, C, m, n, k, st);
    }
    return vec ? launch<64, 64, true>(A, B, C, m, n, k, st)
               : launch<64, 64, false>(A, B, C, m, n, k, st);
}
