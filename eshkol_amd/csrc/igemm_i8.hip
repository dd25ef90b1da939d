/*
 * int8 x int8 -> int32 contraction on the gfx950 matrix cores
 * (v_mfma_i32_32x32x32_i8), shared by the Ozaki-II CRT tier (one product per
 * modulus, result reduced modulo p) and the INT8 slice tier (several slice
 * pairs summed into one int32 diagonal buffer). It replaces the cublasGemmEx
 * loop of the reference (lib/backend/gpu/gpu_memory_cuda.cpp:415-434) and the
 * modular GEMM matmul_ozaki_gemm (lib/backend/gpu/metal_softfloat.h:3907-4100).
 *
 * Operands are K-contiguous int8 planes (row pitch ldk, zero padded), so both
 * MFMA operands are 16-byte LDS reads along K; which k each lane feeds does not
 * matter as long as both operands agree, because the int32 sum is exact.
 *
 * Work decomposition
 *   workgroup  WGM x WGN waves, block tile (WGM*TM*32) x (WGN*TN*32), BK = 64 bytes
 *   wave       TM x TN MFMA tiles of 32x32, int32 accumulators in registers
 *   LDS        double-buffered [rows][64(+16)] bytes per operand; the 16-byte pad
 *              spreads the 16-byte reads of 16 consecutive rows over all banks
 *   operands   the B fragment is passed as the MFMA's first operand, so a lane
 *              ends up with 4 consecutive columns of one output row and can
 *              store them as one word (int8) or one 16-byte vector (int32)
 *   epilogue   mode 1 reduces modulo p in fp64 (exact: |sum| < 2^31), stages
 *              the int8 tile through LDS and writes whole 16-byte chunks
 *
 * One launch covers every output plane: the flattened workgroup id is remapped
 * so each XCD works through whole planes, 8 tile-rows at a time, and the
 * workgroups resident together share operand rows in that XCD's L2.
 */
#include "hip_common.h"
#include "kernels.h"

typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef int v16i_t __attribute__((ext_vector_type(16)));

namespace {

constexpr int BKB = 64;            /* bytes of K per block */
constexpr int LDS_PITCH = BKB + 16;

template <int WGM, int WGN, int TM, int TN> struct Cfg {
    static constexpr int NT = 64 * WGM * WGN;
    static constexpr int BM = WGM * TM * 32;
    static constexpr int BN = WGN * TN * 32;
    static constexpr int A_TILE = BM * LDS_PITCH;
    static constexpr int B_TILE = BN * LDS_PITCH;
    static constexpr int SMEM_MAIN = 2 * (A_TILE + B_TILE);
    static constexpr int SMEM_EPI = BM * (BN + 16);
    static constexpr int SMEM_BYTES = SMEM_MAIN > SMEM_EPI ? SMEM_MAIN : SMEM_EPI;
    static constexpr int A_CHUNKS = BM * BKB / 16 / NT;
    static constexpr int B_CHUNKS = BN * BKB / 16 / NT;
    static_assert(BM * BKB / 16 % NT == 0 && BN * BKB / 16 % NT == 0, "tile/thread mismatch");
};

template <int WGM, int WGN, int TM, int TN>
__global__ __launch_bounds__(64 * WGM * WGN)
void igemm_i8_kernel(HipIgemmArgs g, int tiles_m, int tiles_n) {
    using C = Cfg<WGM, WGN, TM, TN>;
    extern __shared__ __align__(16) int8_t smem_i8[];
    int8_t* As = smem_i8;
    int8_t* Bs = smem_i8 + 2 * C::A_TILE;

    /* workgroup -> (output plane, tile) */
    int o, tm, tn;
    {
        const int nwg = gridDim.x, wg = blockIdx.x;
        const int q = nwg >> 3, r = nwg & 7;
        const int xcd = wg & 7, seq = wg >> 3;
        const int L = xcd * q + (xcd < r ? xcd : r) + seq;
        const int per_plane = tiles_m * tiles_n;
        o = L / per_plane;
        const int in_plane = L - o * per_plane;
        const int GM = 8;
        const int width = GM * tiles_n;
        const int group = in_plane / width;
        const int first_m = group * GM;
        const int gsize = (tiles_m - first_m < GM) ? tiles_m - first_m : GM;
        const int in_group = in_plane - group * width;
        tm = first_m + in_group % gsize;
        tn = in_group / gsize;
    }
    const int m0 = tm * C::BM, n0 = tn * C::BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int li = lane & 31, lh = lane >> 5;

    const int pair_lo = g.pair_first[o], pair_hi = g.pair_first[o + 1];
    const int nkb_per = (int)(g.ldk / BKB);
    const int nkb = (pair_hi - pair_lo) * nkb_per;

    v4i_t ra[C::A_CHUNKS], rb[C::B_CHUNKS];

    auto gload = [&](int kb) {
        const int t = pair_lo + kb / nkb_per;
        const int k0 = (kb % nkb_per) * BKB;
        const int8_t* Ap = g.a_planes + (size_t)g.pair_a[t] * g.a_plane_stride + (size_t)m0 * g.ldk + k0;
        const int8_t* Bp = g.b_planes + (size_t)g.pair_b[t] * g.b_plane_stride + (size_t)n0 * g.ldk + k0;
#pragma unroll
        for (int r = 0; r < C::A_CHUNKS; r++) {
            const int c = tid + C::NT * r;
            ra[r] = *(const v4i_t*)(Ap + (size_t)(c >> 2) * g.ldk + (c & 3) * 16);
        }
#pragma unroll
        for (int r = 0; r < C::B_CHUNKS; r++) {
            const int c = tid + C::NT * r;
            rb[r] = *(const v4i_t*)(Bp + (size_t)(c >> 2) * g.ldk + (c & 3) * 16);
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

    v16i_t acc[TM][TN];
#pragma unroll
    for (int t = 0; t < TM; t++)
#pragma unroll
        for (int u = 0; u < TN; u++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[t][u][r] = 0;

    if (nkb > 0) {
        gload(0);
        sstore(0);
    }
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
                for (int u = 0; u < TN; u++)
                    acc[t][u] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[u], a[t], acc[t][u], 0, 0, 0);
        }

        if (more) sstore(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }

    /* With B as the first operand the accumulator is the transposed tile:
     * lane column (lane%32) is the output row, and registers 4v..4v+3 are the
     * output columns 8v + 4*(lane/32) + 0..3. */
    if (g.mode == 0) {
        int32_t* out = g.out_i32 + (size_t)o * g.M * g.N;
        const bool vec_ok = (g.N % 4 == 0);
#pragma unroll
        for (int t = 0; t < TM; t++) {
            const int row = m0 + wm * TM * 32 + t * 32 + li;
#pragma unroll
            for (int u = 0; u < TN; u++)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int col = n0 + wn * TN * 32 + u * 32 + 8 * v + 4 * lh;
                    if (row < (int)g.M) {
                        int32_t* p = out + (size_t)row * g.N + col;
                        if (vec_ok && col + 3 < (int)g.N) {
                            v4i_t w = {acc[t][u][4 * v], acc[t][u][4 * v + 1],
                                       acc[t][u][4 * v + 2], acc[t][u][4 * v + 3]};
                            *(v4i_t*)p = w;
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                if (col + e < (int)g.N) p[e] = acc[t][u][4 * v + e];
                        }
                    }
                }
        }
        return;
    }

    /* mode 1: residues modulo p, staged through LDS */
    const int p = g.modulus[o];
    const double pinv = 1.0 / (double)p;
    constexpr int EPITCH = C::BN + 16;
    int8_t* stage = smem_i8;     /* the main loop's last barrier has passed */
#pragma unroll
    for (int t = 0; t < TM; t++) {
        const int lrow = wm * TM * 32 + t * 32 + li;
#pragma unroll
        for (int u = 0; u < TN; u++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int lcol = wn * TN * 32 + u * 32 + 8 * v + 4 * lh;
                uint32_t packed = 0;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int s = acc[t][u][4 * v + e];
                    const int qd = (int)rint((double)s * pinv);
                    int r = s - qd * p;
                    if (2 * r >= p) r -= p;
                    else if (2 * r < -p) r += p;
                    packed |= ((uint32_t)(uint8_t)(int8_t)r) << (8 * e);
                }
                *(uint32_t*)(stage + lrow * EPITCH + lcol) = packed;
            }
    }
    __syncthreads();
    {
        int8_t* out = g.out_i8 + (size_t)o * g.M * g.N;
        const bool vec_ok = (g.N % 16 == 0) && (((uintptr_t)out & 15) == 0);
        constexpr int CHUNKS_PER_ROW = C::BN / 16;
        constexpr int TOTAL = C::BM * CHUNKS_PER_ROW;
        for (int c = tid; c < TOTAL; c += C::NT) {
            const int lrow = c / CHUNKS_PER_ROW, lc = (c % CHUNKS_PER_ROW) * 16;
            const int row = m0 + lrow, col = n0 + lc;
            if (row >= (int)g.M || col >= (int)g.N) continue;
            const int8_t* src = stage + lrow * EPITCH + lc;
            int8_t* dst = out + (size_t)row * g.N + col;
            if (vec_ok && col + 15 < (int)g.N) {
                *(v4i_t*)dst = *(const v4i_t*)src;
            } else {
                for (int e = 0; e < 16 && col + e < (int)g.N; e++) dst[e] = src[e];
            }
        }
    }
}

template <int WGM, int WGN, int TM, int TN>
int launch(const HipIgemmArgs& a, hipStream_t st) {
    using C = Cfg<WGM, WGN, TM, TN>;
    static bool attr_set = false;
    auto kern = igemm_i8_kernel<WGM, WGN, TM, TN>;
    if (!attr_set) {
        if (!ESHKOL_HIP_OK(hipFuncSetAttribute((const void*)kern,
                hipFuncAttributeMaxDynamicSharedMemorySize, C::SMEM_BYTES))) return -1;
        attr_set = true;
    }
    const int tiles_m = (int)((a.M + C::BM - 1) / C::BM), tiles_n = (int)((a.N + C::BN - 1) / C::BN);
    const long long nwg = (long long)tiles_m * tiles_n * a.n_out;
    if (nwg > 0x7fffffffLL || nwg <= 0) return -1;
    hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(C::NT), C::SMEM_BYTES, st, a, tiles_m, tiles_n);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

}  // namespace

extern "C" int hip_igemm_i8(const HipIgemmArgs* args, void* stream) {
    if (!args || !args->a_planes || !args->b_planes || !args->pair_first || !args->pair_a || !args->pair_b)
        return -1;
    const HipIgemmArgs& a = *args;
    if (a.M == 0 || a.N == 0 || a.n_out == 0 || a.ldk == 0 || a.ldk % 128 != 0) return -1;
    if (a.M > 0x7fffffffu || a.N > 0x7fffffffu) return -1;
    if (((uintptr_t)a.a_planes & 15) || ((uintptr_t)a.b_planes & 15) ||
        (a.a_plane_stride & 15) || (a.b_plane_stride & 15)) return -1;
    if (a.mode == 0) { if (!a.out_i32) return -1; }
    else if (a.mode == 1) { if (!a.out_i8 || !a.modulus) return -1; }
    else return -1;
    hipStream_t st = (hipStream_t)stream;
    /* 256x256 tiles when they fill the chip, else 128x128. Operand planes are
     * padded to multiples of 256 rows, so either tiling reads in bounds. */
    const long long big = (long long)((a.M + 255) / 256) * ((a.N + 255) / 256) * a.n_out;
    if (big >= 256) return launch<2, 2, 4, 4>(a, st);
    return launch<2, 2, 2, 2>(a, st);
}
