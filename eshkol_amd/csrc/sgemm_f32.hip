/*
 * Single-precision GEMM on the fp32 matrix cores (v_mfma_f32_32x32x2_f32), behind
 * eshkol_gpu_matmul_f32: C[MxN] = A[MxK] * B[KxN], row-major, alpha 1, beta 0. It
 * replaces the cublasSgemm call of the reference
 * (lib/backend/gpu/gpu_memory_cuda.cpp:658-665); no language construct reaches
 * this entry, the runtime's tensors being fp64 storage.
 *
 *   block      256 threads = 2 x 2 waves, block tile 128 x 128, wave tile 64 x 64
 *              (2 x 2 MFMA tiles of 32 x 32, 64 accumulator registers), k-block of
 *              32 floats: every global row segment of A is a whole 128-byte line;
 *              two workgroups per CU (68 KiB of LDS each)
 *   global     the loads of block g+1 are issued before the MFMAs of block g and
 *              written to the other LDS buffer half-way through them: one barrier
 *              per block, with nothing left to wait for
 *   LDS        A tile [128 rows][32 k] with a pitch of 36 floats (the 16-byte
 *              fragment reads of eight lanes cover all banks); B tile as it comes,
 *              [32 k][128 n], so B is never transposed: a lane's fragment element
 *              is one float of a row of 32 consecutive ones
 *   fragments  lane l feeds k = 16 (l / 32) + s at step s = 0 .. 15 to BOTH
 *              operands, so its sixteen A values are 64 contiguous bytes; the sum
 *              over k does not care in which order the steps take it
 *   result     B's fragment is the MFMA's first operand: a lane ends up with four
 *              consecutive columns of one output row per register quad and stores
 *              them as one 16-byte word
 *
 * Two instances: products whose sizes are multiples of the tile (M, N of 128, K
 * of 32) with 16-byte aligned operands run a loop without a single bounds check
 * or branch, one straight-line region per k-block that the compiler interleaves
 * freely; everything else takes the instance whose loads and stores are guarded
 * (vector ones for tiles inside the matrix, scalar ones at the edges). Same
 * arithmetic in the same order: the two give the same bits.
 */
#include "hip_common.h"
#include "kernels.h"

#include <mutex>

typedef float v4f_t __attribute__((ext_vector_type(4)));
typedef float v16f_t __attribute__((ext_vector_type(16)));

namespace {

constexpr int BM = 128, BN = 128, BK = 32;
constexpr int A_PITCH = BK + 4;                 /* floats */
constexpr int A_TILE = BM * A_PITCH;            /* floats per buffer */
constexpr int B_TILE = BK * BN;
constexpr int SMEM_BYTES = 2 * (A_TILE + B_TILE) * (int)sizeof(float);

template <bool FAST>
__global__ __launch_bounds__(256, 2)
void sgemm_mfma_kernel(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C,
                       int M, int N, int K, int tiles_m, int tiles_n, int vec_ok) {
    extern __shared__ __align__(16) float smem_f32[];
    float* As = smem_f32;
    float* Bs = smem_f32 + 2 * A_TILE;

    /* eight tile rows at a time, so that the workgroups resident together share operand panels */
    const int GM = 8;
    const int pid = (int)blockIdx.x;
    const int width = GM * tiles_n;
    const int group = pid / width;
    const int first_m = group * GM;
    const int gsize = (tiles_m - first_m < GM) ? tiles_m - first_m : GM;
    const int tm = first_m + (pid - group * width) % gsize;
    const int tn = (pid - group * width) / gsize;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 31, lh = lane >> 5;
    const bool interior = FAST || (vec_ok && m0 + BM <= M && n0 + BN <= N);

    v4f_t ga[4], gb[4];                         /* one k-block of each operand on its way to LDS */
    auto load_global = [&](int k0) {
        const bool whole = FAST || (interior && k0 + BK <= K);
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int c = tid + 256 * r;
            const int arow = c >> 3, ak = (c & 7) * 4;          /* A: 128 rows x 8 chunks of 4 floats */
            const int bk = c >> 5, bn = (c & 31) * 4;           /* B: 32 k x 32 chunks */
            if (whole) {
                ga[r] = *(const v4f_t*)(A + (size_t)(m0 + arow) * K + k0 + ak);
                gb[r] = *(const v4f_t*)(B + (size_t)(k0 + bk) * N + n0 + bn);
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int gm = m0 + arow, gk = k0 + ak + e;
                    ga[r][e] = (gm < M && gk < K) ? A[(size_t)gm * K + gk] : 0.0f;
                    const int gk2 = k0 + bk, gn = n0 + bn + e;
                    gb[r][e] = (gk2 < K && gn < N) ? B[(size_t)gk2 * N + gn] : 0.0f;
                }
            }
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int c = tid + 256 * r;
            *(v4f_t*)(As + buf * A_TILE + (c >> 3) * A_PITCH + (c & 7) * 4) = ga[r];
            *(v4f_t*)(Bs + buf * B_TILE + (c >> 5) * BN + (c & 31) * 4) = gb[r];
        }
    };

    v16f_t acc[2][2];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[t][u][r] = 0.0f;

    const int nkb = (K + BK - 1) / BK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int g = 0; g < nkb; g++) {
        const int buf = g & 1;
        const bool more = g + 1 < nkb;
        if (more) load_global((g + 1) * BK);
        /* the lane's sixteen k of each of its two A rows: 64 contiguous bytes */
        const float* ap = As + buf * A_TILE + (wm * 64 + li) * A_PITCH + 16 * lh;
        const float* bp = Bs + buf * B_TILE + (16 * lh) * BN + wn * 64 + li;
        /* The fragment reads of the block in quarters of four k-steps, each issued as a
         * group ahead of the MFMAs that use it and under the MFMAs of the quarter before.
         * Left alone the compiler reads each step's two B values right before the four
         * MFMAs that need them and waits for LDS sixteen times per block: the matrix pipe
         * was busy 0.66 of the cycles at a clock of 2.3 GHz. */
        v4f_t af[2][4];
        float bf[16][2];
        auto read_quarter = [&](int h) {         /* k-steps 4h .. 4h+3: one 16-byte piece of each A row, four pairs of B values */
#pragma unroll
            for (int t = 0; t < 2; t++) af[t][h] = *(const v4f_t*)(ap + t * 32 * A_PITCH + 4 * h);
#pragma unroll
            for (int s = 4 * h; s < 4 * h + 4; s++) { bf[s][0] = bp[s * BN]; bf[s][1] = bp[s * BN + 32]; }
        };
        auto mfma_steps = [&](int s0, int s1) {
#pragma unroll
            for (int s = s0; s < s1; s++)
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    const float a = af[t][s >> 2][s & 3];
                    acc[t][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[s][0], a, acc[t][0], 0, 0, 0);
                    acc[t][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[s][1], a, acc[t][1], 0, 0, 0);
                }
        };
        read_quarter(0);
        __builtin_amdgcn_sched_barrier(0);
        mfma_steps(0, 1);                       /* each later quarter is requested under the MFMAs of the one before */
        __builtin_amdgcn_sched_barrier(0);
        read_quarter(1);
        __builtin_amdgcn_sched_barrier(0);
        mfma_steps(1, 4);
        __builtin_amdgcn_sched_barrier(0);
        read_quarter(2);
        __builtin_amdgcn_sched_barrier(0);
        mfma_steps(4, 8);
        __builtin_amdgcn_sched_barrier(0);
        read_quarter(3);
        /* the other buffer was last read before the previous barrier, and the loads issued
         * at the top of this block have had half a block to land: written here, the LDS
         * writes finish under the second half's MFMAs and the barrier finds them done */
        if (more) store_lds(buf ^ 1);
        __builtin_amdgcn_sched_barrier(0);
        mfma_steps(8, 16);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
    }

    /* lane: output row m0 + 64 wm + 32 t + li; registers 4v .. 4v+3: columns 8v + 4 lh + 0..3 of tile u */
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int row = m0 + wm * 64 + t * 32 + li;
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int col = n0 + wn * 64 + u * 32 + 8 * v + 4 * lh;
                if (interior) {
                    *(v4f_t*)(C + (size_t)row * N + col) =
                        (v4f_t){acc[t][u][4 * v], acc[t][u][4 * v + 1], acc[t][u][4 * v + 2], acc[t][u][4 * v + 3]};
                } else if (row < M) {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (col + e < N) C[(size_t)row * N + col + e] = acc[t][u][4 * v + e];
                }
            }
    }
}

}  // namespace

extern "C" int hip_sgemm_f32(const float* A, const float* B, float* C,
                             uint64_t M, uint64_t K, uint64_t N, void* stream) {
    if (!A || !B || !C || M == 0 || K == 0 || N == 0) return -1;
    if (M > 0x7fffffffULL || N > 0x7fffffffULL || K > 0x7fffffffULL) return -1;
    static bool attr_set = false;
    static std::mutex attr_mutex;
    {
        std::lock_guard<std::mutex> lk(attr_mutex);
        if (!attr_set) {
            if (!ESHKOL_HIP_OK(hipFuncSetAttribute((const void*)sgemm_mfma_kernel<true>,
                    hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES)) ||
                !ESHKOL_HIP_OK(hipFuncSetAttribute((const void*)sgemm_mfma_kernel<false>,
                    hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES))) return -1;
            attr_set = true;
        }
    }
    const uint64_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    if (tiles_m * tiles_n > 0x7fffffffULL) return -1;
    /* vector loads and stores want rows of A, B and C that start on 16-byte boundaries */
    const int vec_ok = (K % 4 == 0) && (N % 4 == 0) && (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15) == 0;
    const bool fast = vec_ok && M % BM == 0 && N % BN == 0 && K % BK == 0;
    if (fast)
        hipLaunchKernelGGL(sgemm_mfma_kernel<true>, dim3((unsigned)(tiles_m * tiles_n)), dim3(256), SMEM_BYTES,
                           (hipStream_t)stream, A, B, C, (int)M, (int)N, (int)K, (int)tiles_m, (int)tiles_n, 1);
    else
        hipLaunchKernelGGL(sgemm_mfma_kernel<false>, dim3((unsigned)(tiles_m * tiles_n)), dim3(256), SMEM_BYTES,
                           (hipStream_t)stream, A, B, C, (int)M, (int)N, (int)K, (int)tiles_m, (int)tiles_n, vec_ok);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}
