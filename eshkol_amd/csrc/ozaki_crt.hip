/*
 * Ozaki-II CRT exact tier: C = A*B in fp64 recovered from int8 matrix-core
 * products modulo up to 16 pairwise-coprime moduli. Follows ozaki_ii_dispatch
 * of the reference (lib/backend/gpu/gpu_memory.mm:2474-2665), whose scaling,
 * residue and reconstruction steps run on the CPU; here every O(MK+KN+MN) pass
 * is a device kernel and only the O(M+N) scalar bookkeeping (log2 of the row
 * and column maxima, the exponent E, the shifts) stays on the host, where it
 * uses the same libm as the reference's host code.
 *
 * Pipeline (all on the library stream):
 *   amax[i], bmax[j]                          row maxima of A, column maxima of B
 *   -> host: frac bounds, E, mu[i], nu[j]     gpu_memory.mm:376-420, 2510-2532
 *   A planes, B planes                        trunc(x*2^shift) mod p_l as int8, both
 *                                              [row][k]; B is read k-major through
 *                                              LDS tiles, never transposed in HBM
 *   W_l = (A_l * B_l^T) mod p_l               int8 MFMA, int32 accumulate
 *   C = CRT(W) * 2^-mu * 2^-nu                gpu_memory.mm:2626-2655, verbatim
 *
 * Residues are taken with exact integer arithmetic on the bit pattern of the
 * input (the reference's float formula x - p*rint(x/p) loses exactness at the
 * top of the range); the representative lies in [-p/2, p/2), so 128 mod 256 is
 * stored as -128. Both choices are invisible modulo p.
 */
#include "hip_common.h"
#include "kernels.h"
#include "tanh_f64.h"
#include "kmajor_tile.h"
#include "crt_shared.h"

#include <atomic>
#include <chrono>
#include <climits>
#include <cmath>
#include <cstring>
#include <mutex>

typedef double d2_t __attribute__((ext_vector_type(2)));
typedef uint32_t v4u_t __attribute__((ext_vector_type(4)));

namespace {

/* gpu_memory.mm:227-233 (first 16 of 49; 16 is the most whose product fits
 * a signed 128-bit integer, gpu_memory.mm:246-255) */
#define OZAKI_MODULI_16 256, 255, 253, 251, 247, 241, 239, 233, 229, 227, 223, 217, 211, 199, 197, 193
constexpr int MAX_MODULI = 16;
const int H_MODULI[MAX_MODULI] = { OZAKI_MODULI_16 };

struct ModuliTable { int p[MAX_MODULI]; uint32_t wlo[MAX_MODULI]; uint32_t whi[MAX_MODULI]; };
constexpr ModuliTable make_table() {
    ModuliTable t{};
    const int m[MAX_MODULI] = { OZAKI_MODULI_16 };
    for (int l = 0; l < MAX_MODULI; l++) {
        const ByteWeights w = byte_weights(m[l]);
        t.p[l] = m[l]; t.wlo[l] = w.lo; t.whi[l] = w.hi;
    }
    return t;
}
constexpr ModuliTable TBL = make_table();

/* A word whose low byte is the int8 residue of s modulo p_L, the representative
 * in [-p/2, p/2). Five full-rate instructions: two byte dot products give
 * x = sum b_i w_i < 2^19, congruent to s; q = nearest integer to x/p comes out of
 * one fma against 1.5 * 2^23 (x/p < 2^12 is off by at most 2e-4 in the product
 * and, p being odd, at least 1/(2p) >= 2e-3 from a half-integer), left in the low
 * bits of the float as 2^22 + q; x - (2^22 + q) p then differs from the residue by
 * a multiple of 256. For p = 256 the residue is the low byte of s itself. */
template <int L>
__device__ __forceinline__ uint32_t residue_byte(Scaled s) {
    constexpr int p = TBL.p[L];
    if (p == 256) return s.lo;
    const uint32_t x = __builtin_amdgcn_udot4(s.lo, TBL.wlo[L], __builtin_amdgcn_udot4(s.hi, TBL.whi[L], 0u, false), false);
    const float qm = fmaf((float)x, 1.0f / (float)p, 12582912.0f);
    return (uint32_t)(__mul24(__float_as_int(qm), -p) + (int)x);
}

/* Residues of two consecutive k of one row: one 16-bit store per plane. */
template <int NMOD>
__device__ __forceinline__ void split_pair(double x0, double x1, int sh, int8_t* out, uint64_t plane_stride) {
    const Scaled s0 = scaled_integer<false>(x0, sh), s1 = scaled_integer<false>(x1, sh);
#define ESHKOL_SPLIT_ONE(L)                                                           \
    if (L < NMOD)                                                                     \
        *(uint16_t*)(out + (uint64_t)L * plane_stride) =                              \
            (uint16_t)__builtin_amdgcn_perm(residue_byte<L>(s1), residue_byte<L>(s0), 0x0c0c0400u);
    ESHKOL_SPLIT_ONE(0)  ESHKOL_SPLIT_ONE(1)  ESHKOL_SPLIT_ONE(2)  ESHKOL_SPLIT_ONE(3)
    ESHKOL_SPLIT_ONE(4)  ESHKOL_SPLIT_ONE(5)  ESHKOL_SPLIT_ONE(6)  ESHKOL_SPLIT_ONE(7)
    ESHKOL_SPLIT_ONE(8)  ESHKOL_SPLIT_ONE(9)  ESHKOL_SPLIT_ONE(10) ESHKOL_SPLIT_ONE(11)
    ESHKOL_SPLIT_ONE(12) ESHKOL_SPLIT_ONE(13) ESHKOL_SPLIT_ONE(14) ESHKOL_SPLIT_ONE(15)
#undef ESHKOL_SPLIT_ONE
}

/* Residues of sixteen consecutive k of one row: one 16-byte store per plane. */
template <int NMOD>
__device__ __forceinline__ void split_16(const double* x, int sh, int8_t* out, uint64_t plane_stride) {
    Scaled s[16];
#pragma unroll
    for (int e = 0; e < 16; e++) s[e] = scaled_integer<false>(x[e], sh);
#define ESHKOL_SPLIT_ONE(L)                                                           \
    if (L < NMOD) {                                                                   \
        v4u_t w;                                                                      \
        _Pragma("unroll")                                                             \
        for (int g = 0; g < 4; g++) {                                                 \
            const uint32_t w01 = __builtin_amdgcn_perm(residue_byte<L>(s[4 * g + 1]), residue_byte<L>(s[4 * g]), 0x0c0c0400u); \
            const uint32_t w23 = __builtin_amdgcn_perm(residue_byte<L>(s[4 * g + 3]), residue_byte<L>(s[4 * g + 2]), 0x0c0c0400u); \
            w[g] = __builtin_amdgcn_perm(w23, w01, 0x05040100u);                      \
        }                                                                             \
        eshkol_store_streaming((v4u_t*)(out + (uint64_t)L * plane_stride), w);        \
    }
    ESHKOL_SPLIT_ONE(0)  ESHKOL_SPLIT_ONE(1)  ESHKOL_SPLIT_ONE(2)  ESHKOL_SPLIT_ONE(3)
    ESHKOL_SPLIT_ONE(4)  ESHKOL_SPLIT_ONE(5)  ESHKOL_SPLIT_ONE(6)  ESHKOL_SPLIT_ONE(7)
    ESHKOL_SPLIT_ONE(8)  ESHKOL_SPLIT_ONE(9)  ESHKOL_SPLIT_ONE(10) ESHKOL_SPLIT_ONE(11)
    ESHKOL_SPLIT_ONE(12) ESHKOL_SPLIT_ONE(13) ESHKOL_SPLIT_ONE(14) ESHKOL_SPLIT_ONE(15)
#undef ESHKOL_SPLIT_ONE
}

/* Row-major X[rows][K]. One thread: two consecutive k of one row. */
template <int NMOD>
__global__ __launch_bounds__(256)
void crt_split_kernel(const double* __restrict__ X, uint64_t rows, uint64_t K,
                      const int32_t* __restrict__ shift, int8_t* __restrict__ planes,
                      uint64_t rows_padded, uint64_t ldk) {
    const uint32_t cpr = (uint32_t)((ldk / 2 + 255) / 256);      /* blocks per row */
    const uint64_t row = blockIdx.x / cpr;
    const uint64_t k = ((uint64_t)(blockIdx.x % cpr) * 256 + threadIdx.x) * 2;
    if (k >= ldk) return;
    double x0 = 0.0, x1 = 0.0;
    int sh = 0;
    if (row < rows) {
        sh = shift[row];
        const double* p = X + row * K + k;
        if (k + 1 < K) {
            if ((K & 1) == 0 && (((uintptr_t)X & 15) == 0)) { d2_t v = *(const d2_t*)p; x0 = v.x; x1 = v.y; }
            else { x0 = p[0]; x1 = p[1]; }
        } else if (k < K) {
            x0 = p[0];
        }
    }
    split_pair<NMOD>(x0, x1, sh, planes + row * ldk + k, rows_padded * ldk);
}

/* Row-major X[rows][K], pitches that are multiples of 16 bytes. One thread: four
 * consecutive k of one row. The residues of a block (1024 k of one row, all
 * planes) are collected in LDS as one word per thread and plane, then leave as
 * 16-byte stores: four store instructions per thread instead of a 2-byte store
 * per plane and pair. */
template <int NMOD>
__global__ __launch_bounds__(256)
void crt_split_staged_kernel(const double* __restrict__ X, uint64_t rows, uint64_t K,
                             const int32_t* __restrict__ shift, int8_t* __restrict__ planes,
                             uint64_t rows_padded, uint64_t ldk) {
    __shared__ __align__(16) uint32_t stage[NMOD][256];
    const uint32_t cpr = (uint32_t)((ldk + 1023) / 1024);        /* blocks per row */
    const uint64_t row = blockIdx.x / cpr;
    const uint64_t kbase = (uint64_t)(blockIdx.x % cpr) * 1024;
    const int tid = threadIdx.x;
    const uint64_t k = kbase + 4 * (uint64_t)tid;
    double x[4] = {0.0, 0.0, 0.0, 0.0};
    int sh = 0;
    if (row < rows && k < K) {
        sh = shift[row];
        const double* p = X + row * K + k;
        if (k + 3 < K && (K & 1) == 0 && (((uintptr_t)X & 15) == 0)) {
            const d2_t v0 = *(const d2_t*)p, v1 = *(const d2_t*)(p + 2);
            x[0] = v0.x; x[1] = v0.y; x[2] = v1.x; x[3] = v1.y;
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) if (k + e < K) x[e] = p[e];
        }
    }
    Scaled t[4];
#pragma unroll
    for (int e = 0; e < 4; e++) t[e] = scaled_integer<false>(x[e], sh);
#define ESHKOL_SPLIT_ONE(L)                                                           \
    if (L < NMOD) {                                                                   \
        const uint32_t w01 = __builtin_amdgcn_perm(residue_byte<L>(t[1]), residue_byte<L>(t[0]), 0x0c0c0400u); \
        const uint32_t w23 = __builtin_amdgcn_perm(residue_byte<L>(t[3]), residue_byte<L>(t[2]), 0x0c0c0400u); \
        stage[L][tid] = __builtin_amdgcn_perm(w23, w01, 0x05040100u);                 \
    }
    ESHKOL_SPLIT_ONE(0)  ESHKOL_SPLIT_ONE(1)  ESHKOL_SPLIT_ONE(2)  ESHKOL_SPLIT_ONE(3)
    ESHKOL_SPLIT_ONE(4)  ESHKOL_SPLIT_ONE(5)  ESHKOL_SPLIT_ONE(6)  ESHKOL_SPLIT_ONE(7)
    ESHKOL_SPLIT_ONE(8)  ESHKOL_SPLIT_ONE(9)  ESHKOL_SPLIT_ONE(10) ESHKOL_SPLIT_ONE(11)
    ESHKOL_SPLIT_ONE(12) ESHKOL_SPLIT_ONE(13) ESHKOL_SPLIT_ONE(14) ESHKOL_SPLIT_ONE(15)
#undef ESHKOL_SPLIT_ONE
    __syncthreads();
    const uint64_t plane_stride = rows_padded * ldk;
#pragma unroll
    for (int j = 0; j < NMOD * 64 / 256 + (NMOD * 64 % 256 != 0); j++) {
        const int c = tid + 256 * j;
        const int plane = c >> 6, ch = c & 63;
        const uint64_t kk = kbase + 16 * (uint64_t)ch;
        if (plane < NMOD && kk < ldk)
            *(v4u_t*)(planes + (uint64_t)plane * plane_stride + row * ldk + kk) = *(const v4u_t*)&stage[plane][4 * ch];
    }
}

/* Row-major X[rows][K], interleaved planes (rows_padded and ldk multiples of 32).
 * A block takes 32 rows x 32 k, a thread four consecutive k of one row (eight
 * lanes read 256 contiguous bytes of a row). What the block produces is, per
 * plane, one operand fragment: 1 KiB of contiguous memory, written by one wave
 * as 16-byte stores. */
template <int NMOD>
__global__ __launch_bounds__(256)
void crt_split_il_kernel(const double* __restrict__ X, uint64_t rows, uint64_t K,
                         const int32_t* __restrict__ shift, int8_t* __restrict__ planes,
                         uint64_t rows_padded, uint64_t ldk) {
    __shared__ __align__(16) uint32_t stage[NMOD][256];
    const uint32_t kt = (uint32_t)(ldk / 32);
    const uint64_t rb = blockIdx.x / kt, kb = blockIdx.x % kt;
    const int tid = threadIdx.x;
    const uint64_t row = rb * 32 + (uint64_t)(tid >> 3), k = kb * 32 + 4 * (uint64_t)(tid & 7);
    double x[4] = {0.0, 0.0, 0.0, 0.0};
    int sh = 0;
    if (row < rows && k < K) {
        sh = shift[row];
        const double* p = X + row * K + k;
        if (k + 3 < K && (K & 1) == 0 && (((uintptr_t)X & 15) == 0)) {
            const d2_t v0 = *(const d2_t*)p, v1 = *(const d2_t*)(p + 2);
            x[0] = v0.x; x[1] = v0.y; x[2] = v1.x; x[3] = v1.y;
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) if (k + e < K) x[e] = p[e];
        }
    }
    Scaled t[4];
#pragma unroll
    for (int e = 0; e < 4; e++) t[e] = scaled_integer<false>(x[e], sh);
#define ESHKOL_SPLIT_ONE(L)                                                           \
    if (L < NMOD) {                                                                   \
        const uint32_t w01 = __builtin_amdgcn_perm(residue_byte<L>(t[1]), residue_byte<L>(t[0]), 0x0c0c0400u); \
        const uint32_t w23 = __builtin_amdgcn_perm(residue_byte<L>(t[3]), residue_byte<L>(t[2]), 0x0c0c0400u); \
        stage[L][tid] = __builtin_amdgcn_perm(w23, w01, 0x05040100u);                 \
    }
    ESHKOL_SPLIT_ONE(0)  ESHKOL_SPLIT_ONE(1)  ESHKOL_SPLIT_ONE(2)  ESHKOL_SPLIT_ONE(3)
    ESHKOL_SPLIT_ONE(4)  ESHKOL_SPLIT_ONE(5)  ESHKOL_SPLIT_ONE(6)  ESHKOL_SPLIT_ONE(7)
    ESHKOL_SPLIT_ONE(8)  ESHKOL_SPLIT_ONE(9)  ESHKOL_SPLIT_ONE(10) ESHKOL_SPLIT_ONE(11)
    ESHKOL_SPLIT_ONE(12) ESHKOL_SPLIT_ONE(13) ESHKOL_SPLIT_ONE(14) ESHKOL_SPLIT_ONE(15)
#undef ESHKOL_SPLIT_ONE
    __syncthreads();
    /* stage[plane][8 r + j] holds k 4j .. 4j+3 of row r; fragment order is
     * [k-chunk c][row r][16 bytes]: chunk c of row r is words 8 r + 4 c .. + 3 */
    const uint64_t plane_stride = rows_padded * ldk;
    int8_t* frag = planes + rb * (32 * ldk) + kb * 1024;
#pragma unroll
    for (int j = 0; j < NMOD * 64 / 256 + (NMOD * 64 % 256 != 0); j++) {
        const int c = tid + 256 * j;
        const int plane = c >> 6, q = c & 63;
        if (plane < NMOD)
            eshkol_store_streaming((v4u_t*)(frag + (uint64_t)plane * plane_stride + 16 * q),
                                   *(const v4u_t*)&stage[plane][8 * (q & 31) + 4 * (q >> 5)]);
    }
}

/* k-major X[K][rows] (B as the runtime stores it), same output. */
template <int NMOD>
__global__ __launch_bounds__(256, 4)
void crt_split_kmajor_kernel(const double* __restrict__ X, uint64_t rows, uint64_t K,
                             const int32_t* __restrict__ shift, int8_t* __restrict__ planes,
                             uint64_t rows_padded, uint64_t ldk, uint32_t group, int layout) {
    __shared__ __align__(16) double tile[kmaj::SMEM_DOUBLES];
    const uint64_t plane_stride = rows_padded * ldk;
    if ((ldk & 15) == 0 && (((uintptr_t)planes & 15) == 0)) {
        kmaj::for_each_16(X, rows, K, rows_padded, ldk, group, tile,
            [&](uint64_t row) { return (row < rows) ? shift[row] : 0; },
            [&](uint64_t row, uint64_t k, const double* x, int sh) {
                split_16<NMOD>(x, sh, planes + eshkol_plane_offset(layout, row, k, ldk), plane_stride);
            });
        return;
    }
    kmaj::for_each_pair(X, rows, K, rows_padded, ldk, group, tile,
        [&](uint64_t row) { return (row < rows) ? shift[row] : 0; },
        [&](uint64_t row, uint64_t k, double x0, double x1, int sh) {
            split_pair<NMOD>(x0, x1, sh, planes + eshkol_plane_offset(layout, row, k, ldk), plane_stride);
        });
}

/* k-major X[K][rows], interleaved planes: no LDS (kmajor_tile.h). */
template <int NMOD>
__global__ __launch_bounds__(256, 4)
void crt_split_kmajor_il_kernel(const double* __restrict__ X, uint64_t rows, uint64_t K,
                                const int32_t* __restrict__ shift, int8_t* __restrict__ planes,
                                uint64_t rows_padded, uint64_t ldk) {
    uint64_t row, k;
    kmaj::il_thread(rows_padded, &row, &k);
    if (row >= rows_padded || k >= ldk) return;
    double x[16];
    kmaj::load_k16(X, rows, K, row, k, x);
    const int sh = (row < rows) ? shift[row] : 0;
    split_16<NMOD>(x, sh, planes + eshkol_plane_offset(1, row, k, ldk), rows_padded * ldk);
}

struct CrtConsts {
    double sl1[MAX_MODULI], sl2[MAX_MODULI];
    double P1, P2, Pinv;
    int n;
};

/* One thread: four consecutive columns of one row. The arithmetic is the
 * reference's, operation for operation: S1 = fma(sl1_l, w, S1), S2 likewise,
 * l ascending; s = S1 + S2; Q = round(s*Pinv); c' = fma(-P1,Q,S1) + fma(-P2,Q,S2);
 * C = (c' * 2^-mu) * 2^-nu. The number of planes is a compile-time constant so
 * that a thread's loads of all planes are issued together, before the first
 * use: the kernel moves 24 bytes per element and has to keep HBM busy. So is
 * the tanh epilogue: its code would otherwise cost every launch three quarters
 * of its occupancy in registers. */
/* W is [NMOD][wrows][ldw]: the product planes as the contraction left them.
 * VEC 1: N is a multiple of four and W and C are aligned for 4- and 16-byte
 * accesses (the launcher checks): every thread then has four whole elements, and
 * the kernel carries none of the byte-wise path, whose address arithmetic the
 * compiler would otherwise place in front of both paths (a third of the
 * kernel's vector instructions: it is bound by them, not by HBM).
 * VEC 2: W's pitch and base allow the 4-byte loads, but N is not a multiple of
 * four or C's rows do not start on 16-byte boundaries: whole groups of four are
 * stored as two 16-byte words at 8-byte alignment, the last group of a row
 * element by element.
 * VEC 0: nothing is known about W's alignment either (dense planes of any N). */
typedef double d2u_t __attribute__((ext_vector_type(2), aligned(8)));
template <int NMOD, bool TANH, int VEC>
__global__ __launch_bounds__(256)
void crt_reconstruct_kernel(const int8_t* __restrict__ W, uint64_t wrows, uint64_t ldw, uint64_t M, uint64_t N, CrtConsts cc,
                            const int32_t* __restrict__ mu, const int32_t* __restrict__ nu,
                            const double* __restrict__ bias, double* __restrict__ C) {
    const uint32_t cpr = (uint32_t)(((N + 3) / 4 + 255) / 256);   /* blocks per row */
    const uint64_t row = blockIdx.x / cpr;
    const uint64_t col = ((uint64_t)(blockIdx.x % cpr) * 256 + threadIdx.x) * 4;
    if (col >= N) return;
    const uint64_t tot = wrows * ldw, idx = row * N + col, widx = row * ldw + col;
    const int nvalid = (VEC == 1) ? 4 : ((N - col < 4) ? (int)(N - col) : 4);
    uint32_t u[NMOD];
    if (VEC != 0) {
        const int8_t* p = W + widx;                /* one address, then a step per plane */
#pragma unroll
        for (int l = 0; l < NMOD; l++) { u[l] = *(const uint32_t*)p; p += tot; }
    } else {
#pragma unroll
        for (int l = 0; l < NMOD; l++) {
            const int8_t* w = W + (uint64_t)l * tot + widx;
            u[l] = 0;
#pragma unroll
            for (int e = 0; e < 4; e++) if (e < nvalid) u[l] |= (uint32_t)(uint8_t)w[e] << (8 * e);
        }
    }
    int sh[4] = {0, 0, 0, 0};
    double bv[4] = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < 4; e++) {
        if (e < nvalid) {
            sh[e] = nu[col + e];
            if (bias) bv[e] = bias[col + e];
        }
    }
    const double mu_inv = ldexp(1.0, -mu[row]);
    double S1[4] = {0, 0, 0, 0}, S2[4] = {0, 0, 0, 0};
#pragma unroll
    for (int l = 0; l < NMOD; l++) {
        const double a = cc.sl1[l], b = cc.sl2[l];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const double wd = (double)(int8_t)(u[l] >> (8 * e));
            S1[e] = fma(a, wd, S1[e]);
            S2[e] = fma(b, wd, S2[e]);
        }
    }
    double out[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const double s = S1[e] + S2[e];
        const double Q = round(s * cc.Pinv);
        const double h1 = fma(-cc.P1, Q, S1[e]);
        const double h2 = fma(-cc.P2, Q, S2[e]);
        const double cp = h1 + h2;
        double v = (cp * mu_inv) * ldexp(1.0, -sh[e]);
        if (bias) v = v + bv[e];
        if (TANH) v = eshkol_tanh_f64(v);
        out[e] = v;
    }
    if (VEC == 1) {
        d2_t* o = (d2_t*)(C + idx);
        d2_t lo, hi;
        lo.x = out[0]; lo.y = out[1]; hi.x = out[2]; hi.y = out[3];
        o[0] = lo; o[1] = hi;
    } else if (VEC == 2 && nvalid == 4) {
        d2u_t* o = (d2u_t*)(C + idx);
        d2u_t lo, hi;
        lo.x = out[0]; lo.y = out[1]; hi.x = out[2]; hi.y = out[3];
        o[0] = lo; o[1] = hi;
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) if (e < nvalid) C[idx + e] = out[e];
    }
}

/* ---- shifts without a host pass over the maxima ---------------------------------
 *
 * The reference takes log2 of every row and column maximum on the host
 * (gpu_memory.mm:376-420) for two things: floor(log2 m) per row, and the largest
 * fractional part frac = log2 m - floor(log2 m) per operand. Both can be had
 * without M + N libm calls. floor(log2 m) is the exponent of m unless its
 * mantissa sits within 2^-40 of a power of two, where a libm result may round
 * across the integer. And frac is within 2^-42 of log2 of the mantissa (a libm
 * accurate to an ulp, results below 1024 in magnitude), so only maxima whose
 * mantissa lies within 2^-40 of the largest one can carry the largest frac. The
 * scan below leaves the exponents on the device and hands the host those few
 * maxima; the host calls log2 on them exactly as the reference does. An operand
 * with a mantissa next to a power of two, or with more than SCAN_CAND distinct
 * candidates, takes the full host pass instead. */
constexpr int SCAN_CAND = 64;
constexpr int SCAN_THREADS = 1024;
constexpr int32_t FL_ZERO = CRT_FL_ZERO;        /* marks a maximum of zero: shift 0 */
constexpr unsigned long long MANT_ONE = 1ull << 52, MANT_WINDOW = 1ull << 12;

struct CrtScan {
    unsigned long long mant_max;
    int32_t nonfinite, extreme, nonzero, e_min, e_max, ncand;
    double cand[SCAN_CAND];
    uint32_t ready;             /* the launch's ticket, written last */
    uint32_t pad;
};

/* m > 0 finite -> exponent e = floor(log2 m) and mantissa n in [2^52, 2^53), m = n 2^(e-52) */
__device__ __forceinline__ void decode_positive(double m, int* e, unsigned long long* n) {
    const unsigned long long bits = (unsigned long long)__double_as_longlong(m);
    const int ef = (int)(bits >> 52);
    const unsigned long long mant = bits & (MANT_ONE - 1);
    if (ef != 0) { *e = ef - 1023; *n = mant | MANT_ONE; }
    else { const int p = 63 - __clzll((long long)mant); *e = p - 1074; *n = mant << (52 - p); }
}

/* One workgroup of THREADS threads scans the n_rows maxima x[] (global or LDS memory) and
 * leaves their summary in *o, the ticket last. */
template <int THREADS>
__device__ __forceinline__ void scan_block(const double* x, uint64_t n_rows, int32_t* fl, CrtScan* o, uint32_t ticket) {
    constexpr int SCAN_THREADS = THREADS;
    __shared__ unsigned long long s_max, keys[256];
    __shared__ int s_nonfinite, s_extreme, s_nonzero, s_emin, s_emax, s_ncand;
    const int tid = threadIdx.x;
    if (tid == 0) { s_max = 0; s_nonfinite = 0; s_extreme = 0; s_nonzero = 0; s_emin = INT32_MAX; s_emax = INT32_MIN; s_ncand = 0; }
    if (tid < 256) keys[tid] = 0;
    __syncthreads();
    unsigned long long my_max = 0;
    int my_nonfinite = 0, my_extreme = 0, my_nonzero = 0, my_emin = INT32_MAX, my_emax = INT32_MIN;
    /* four loads in flight per thread: a single block must not crawl from one
     * memory latency to the next */
    for (uint64_t base = 0; base < n_rows; base += 4 * SCAN_THREADS) {
        double v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const uint64_t i = base + (uint64_t)u * SCAN_THREADS + tid;
            v[u] = (i < n_rows) ? x[i] : 0.0;
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const uint64_t i = base + (uint64_t)u * SCAN_THREADS + tid;
            if (i >= n_rows) continue;
            const double m = v[u];
            int32_t f = FL_ZERO;
            if (!(m <= 1.79769313486231570815e308)) my_nonfinite = 1;   /* NaN or +Inf; maxima are >= 0 */
            else if (m > 0.0) {
                int e; unsigned long long n;
                decode_positive(m, &e, &n);
                f = e;
                my_nonzero = 1;
                if (n > my_max) my_max = n;
                if (e < my_emin) my_emin = e;
                if (e > my_emax) my_emax = e;
                if ((n != MANT_ONE && n < MANT_ONE + MANT_WINDOW) || n >= 2 * MANT_ONE - MANT_WINDOW) my_extreme = 1;
            }
            if (fl) fl[i] = f;
        }
    }
    /* fold within the wave first: a thousand atomics on one LDS word would take
     * longer than the scan itself */
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const unsigned long long om = __shfl_xor(my_max, d);
        const int on = __shfl_xor(my_emin, d), ox = __shfl_xor(my_emax, d);
        const int flags = __shfl_xor(my_nonfinite | my_extreme << 1 | my_nonzero << 2, d);
        if (om > my_max) my_max = om;
        if (on < my_emin) my_emin = on;
        if (ox > my_emax) my_emax = ox;
        my_nonfinite |= flags & 1; my_extreme |= flags >> 1 & 1; my_nonzero |= flags >> 2 & 1;
    }
    if ((tid & 63) == 0) {
        if (my_max) atomicMax(&s_max, my_max);
        if (my_nonfinite) atomicOr(&s_nonfinite, 1);
        if (my_extreme) atomicOr(&s_extreme, 1);
        if (my_nonzero) { atomicOr(&s_nonzero, 1); atomicMin(&s_emin, my_emin); atomicMax(&s_emax, my_emax); }
    }
    __syncthreads();
    /* second pass: the distinct maxima whose mantissa is within the window of the largest */
    const unsigned long long floor_n = (s_max > MANT_ONE + MANT_WINDOW) ? s_max - MANT_WINDOW : MANT_ONE;
    if (s_nonzero && !s_nonfinite) {
        for (uint64_t base = 0; base < n_rows; base += 4 * SCAN_THREADS) {
            double v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const uint64_t i = base + (uint64_t)u * SCAN_THREADS + tid;
                v[u] = (i < n_rows) ? x[i] : 0.0;
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const double m = v[u];
                if (!(m > 0.0)) continue;
                int e; unsigned long long n;
                decode_positive(m, &e, &n);
                if (n < floor_n) continue;
                const unsigned long long bits = (unsigned long long)__double_as_longlong(m);
                unsigned h = (unsigned)((bits * 0x9E3779B97F4A7C15ull) >> 56);
                int probes = 0;
                for (; probes < 256; probes++, h = (h + 1) & 255) {
                    const unsigned long long old = atomicCAS(&keys[h], 0ull, bits);
                    if (old == bits) break;
                    if (old == 0ull) {
                        const int slot = atomicAdd(&s_ncand, 1);
                        if (slot < SCAN_CAND) o->cand[slot] = m;
                        break;
                    }
                }
                if (probes == 256) atomicAdd(&s_ncand, SCAN_CAND + 1);
            }
        }
    }
    /* `out` is host memory the CPU is polling: every thread's candidate stores must
     * be out before the ticket that announces them */
    __threadfence_system();
    __syncthreads();
    if (tid == 0) {
        o->mant_max = s_max; o->nonfinite = s_nonfinite; o->extreme = s_extreme; o->nonzero = s_nonzero;
        o->e_min = s_emin; o->e_max = s_emax; o->ncand = s_ncand;
        __threadfence_system();
        *(volatile uint32_t*)&o->ready = ticket;
    }
}

/* block 0: the M row maxima of A; block 1: the N maxima of B */
__global__ __launch_bounds__(SCAN_THREADS)
void crt_scan_kernel(const double* __restrict__ amax, uint64_t M, const double* __restrict__ bmax, uint64_t N,
                     int32_t* __restrict__ fl_a, int32_t* __restrict__ fl_b, CrtScan* out, uint32_t ticket) {
    scan_block<SCAN_THREADS>(blockIdx.x ? bmax : amax, blockIdx.x ? N : M, blockIdx.x ? fl_b : fl_a,
                             out + blockIdx.x, ticket);
}

/* A few long rows in front of prepared planes: their maxima, their shifts and the scan of
 * the maxima in one launch (three launch-sized kernels otherwise, 8 us of the 50 a layer
 * takes). A workgroup per row, every thread with four loads in flight; the workgroup
 * that finishes last (a counter in device memory, left at zero again) scans the M <= 256
 * maxima, which it reads with atomic loads into LDS: no cache of its CU has seen them. */
constexpr int FUSED_MAX_ROWS = 256;
__global__ __launch_bounds__(256)
void crt_rowmax_scan_kernel(const double* __restrict__ A, uint64_t M, uint64_t K, double* rmax, int32_t* __restrict__ shift,
                            int E, unsigned* counter, CrtScan* out, uint32_t ticket) {
    __shared__ double red[4];
    __shared__ double maxima[FUSED_MAX_ROWS];
    __shared__ int s_last;
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint64_t row = blockIdx.x;
    const double* p = A + row * K;
    double m = 0.0;
    if (((K & 1) == 0) && (((uintptr_t)A & 15) == 0)) {
        typedef double d2_t __attribute__((ext_vector_type(2)));
        const d2_t* p2 = (const d2_t*)p;
        const uint64_t n2 = K >> 1;
        for (uint64_t k = tid; k < n2; k += 2048) {
            d2_t v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = (k + 256 * u < n2) ? p2[k + 256 * u] : (d2_t){0.0, 0.0};
#pragma unroll
            for (int u = 0; u < 8; u++) { eshkol_absmax_step(v[u].x, &m); eshkol_absmax_step(v[u].y, &m); }
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
        const double o = __shfl_xor(m, off, 64);
        if (o > m) m = o;
    }
    if (lane == 0) red[wave] = m;
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 4; w++) if (red[w] > m) m = red[w];
        __hip_atomic_store(&rmax[row], m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        shift[row] = eshkol_shift_of_maximum(m, E);
        __threadfence();
        s_last = atomicAdd(counter, 1u) == gridDim.x - 1 ? 1 : 0;
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    if (tid == 0) *counter = 0;                       /* the next launch on the stream starts from zero */
    for (uint64_t i = tid; i < M; i += 256)
        maxima[i] = __hip_atomic_load(&rmax[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    scan_block<256>(maxima, M, nullptr, out, ticket);
}

/* shift = E - floor(log2 max), 0 for a maximum of zero (gpu_memory.mm:2524-2532), in place */
__global__ __launch_bounds__(256)
void crt_shift_kernel(int32_t* __restrict__ fl_a, uint64_t M, int32_t* __restrict__ fl_b, uint64_t N, int E) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= M + N) return;
    int32_t* p = (i < M) ? fl_a + i : fl_b + (i - M);
    const int32_t f = *p;
    *p = (f == FL_ZERO) ? 0 : E - f;
}

/* ---- host bookkeeping ------------------------------------------------------ */

struct HostCrt { double P1, P2, Pinv, log2P; double sl1[MAX_MODULI], sl2[MAX_MODULI]; int q[MAX_MODULI]; bool ready; };
HostCrt g_crt[2][MAX_MODULI + 1];        /* [weights split as the reference does / at a common bit][moduli] */
std::mutex g_crt_mutex;
bool g_aligned_weights = false;

int64_t ext_gcd(int64_t a, int64_t b, int64_t* x, int64_t* y) {
    if (a == 0) { *x = 0; *y = 1; return b; }
    int64_t x1, y1;
    int64_t g = ext_gcd(b % a, a, &x1, &y1);
    *x = y1 - (b / a) * x1;
    *y = x1;
    return g;
}
int mod_inverse(int64_t a, int64_t m) {
    int64_t x, y;
    ext_gcd(a % m, m, &x, &y);
    return (int)((x % m + m) % m);
}

/* precompute_ozaki_constants, gpu_memory.mm:301-341. The volatile temporaries
 * keep the Dekker split free of fused contraction.
 * The reference splits each weight s_l = (P / p_l) q_l relative to the weight's
 * own exponent, so the lowest bits of the upper parts sl1 lie between 2^81 and
 * 2^88 (sixteen moduli) and the sum of sl1_l w_l, up to 2^137, is not always
 * representable: on N(0,1) operands about one element in 150 is off by a
 * multiple of 2^81 in the scaled integer (2^-25 of a typical element; normwise
 * 1e-11 ... 1e-10). That is the reference's result and the default here. With
 * `aligned` every sl1 is a multiple of 2^e, e = bits(P) + 7 + ceil(log2 n) - 53,
 * the partial sums are exact and the tier delivers what its scaling allows
 * (normwise 1e-17); the kernels are the same, only these constants differ. */
const HostCrt& crt_constants(int n, bool aligned) {
    std::lock_guard<std::mutex> lk(g_crt_mutex);
    HostCrt& c = g_crt[aligned ? 1 : 0][n];
    if (c.ready) return c;
    __int128 P = 1;
    for (int l = 0; l < n; l++) P *= H_MODULI[l];
    c.P1 = (double)P;
    c.P2 = (double)(P - (__int128)c.P1);
    c.Pinv = 1.0 / (double)P;
    c.log2P = log2((double)P);
    int bits_P = 0;
    for (__int128 t = P; t > 0; t >>= 1) bits_P++;
    for (int l = 0; l < n; l++) {
        const int p = H_MODULI[l];
        const __int128 Pp = P / p;
        c.q[l] = mod_inverse((int64_t)(Pp % p), p);
        const __int128 s = Pp * (__int128)c.q[l];
        const int bits_to_remove = 8 + (int)ceil(log2((double)n));
        if (aligned) {
            const int e = bits_P + (bits_to_remove - 1) - 53;
            __int128 hi = s;
            if (e > 0) hi = ((s + ((__int128)1 << (e - 1))) >> e) << e;
            c.sl1[l] = (double)hi;
            c.sl2[l] = (double)(s - hi);
            continue;
        }
        const double s_d = (double)s;
        const double factor = (double)(1LL << (bits_to_remove + 1)) + 1.0;
        volatile double t = factor * s_d;
        volatile double hi = t - s_d;
        c.sl1[l] = t - hi;
        c.sl2[l] = (double)(s - (__int128)c.sl1[l]);
    }
    c.ready = true;
    return c;
}
const HostCrt& crt_constants(int n) { return crt_constants(n, g_aligned_weights); }

double g_log2_cumul[MAX_MODULI + 1];
std::once_flag g_cumul_once;

/* pinned host staging for the maxima and shifts */
void* g_pinned = nullptr;
size_t g_pinned_bytes = 0;
void* pinned(size_t bytes) {
    if (g_pinned_bytes >= bytes) return g_pinned;
    if (g_pinned) (void)hipHostFree(g_pinned);
    g_pinned = nullptr; g_pinned_bytes = 0;
    if (!ESHKOL_HIP_OK(hipHostMalloc(&g_pinned, bytes, hipHostMallocDefault))) return nullptr;
    g_pinned_bytes = bytes;
    return g_pinned;
}

/* The scan's result goes straight into pinned host memory that the device can
 * write (no copy command, no stream synchronisation: those cost 25 us of GPU idle
 * time per call, a tenth of a small layer). The host polls the ticket the kernel
 * writes last and falls back to a stream synchronisation if it does not show. */
CrtScan* g_mailbox = nullptr;         /* host address; [2] */
CrtScan* g_mailbox_dev = nullptr;     /* the same memory as the device sees it */
uint32_t g_ticket = 0;
hipStream_t g_scan_stream = nullptr;  /* where a scan that nothing on the device waits for runs */
hipEvent_t g_scan_event = nullptr;
bool ensure_mailbox() {
    if (g_mailbox) return true;
    void* h = nullptr;
    void* d = nullptr;
    if (!g_scan_stream && !ESHKOL_HIP_OK(hipStreamCreateWithFlags(&g_scan_stream, hipStreamNonBlocking))) return false;
    if (!g_scan_event && !ESHKOL_HIP_OK(hipEventCreateWithFlags(&g_scan_event, hipEventDisableTiming | hipEventReleaseToDevice))) return false;
    if (!ESHKOL_HIP_OK(hipHostMalloc(&h, 2 * sizeof(CrtScan), hipHostMallocMapped))) return false;
    if (!ESHKOL_HIP_OK(hipHostGetDevicePointer(&d, h, 0))) { (void)hipHostFree(h); return false; }
    memset(h, 0, 2 * sizeof(CrtScan));
    g_mailbox = (CrtScan*)h; g_mailbox_dev = (CrtScan*)d;
    return true;
}
/* 0 when both halves carry `ticket` (halves == 1: the first, the only one that scan wrote) */
int await_mailbox(uint32_t ticket, hipStream_t st, int halves) {
    volatile uint32_t* r0 = &g_mailbox[0].ready;
    volatile uint32_t* r1 = &g_mailbox[halves == 2 ? 1 : 0].ready;
    const auto t0 = std::chrono::steady_clock::now();
    for (unsigned spin = 0; *r0 != ticket || *r1 != ticket; spin++) {
        if ((spin & 1023) == 1023 &&
            std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(20)) {
            if (!ESHKOL_HIP_OK(hipStreamSynchronize(st))) return -1;
            return (*r0 == ticket && *r1 == ticket) ? 0 : -1;
        }
        __builtin_ia32_pause();
    }
    std::atomic_thread_fence(std::memory_order_acquire);
    return 0;
}

/* Queues the scan of the two vectors of maxima; 0 on failure, else the ticket its
 * summary will carry. */
hipStream_t g_scan_ran_on = nullptr;  /* the stream the last scan was queued on: what a wait drains if the ticket does not show */
int g_scan_halves = 2;                /* 1: the last scan looked at A's maxima only (B's summary was kept when B was prepared) */
uint32_t scan_launch(const double* amax, uint64_t M, const double* bmax, uint64_t N,
                     int32_t* fl_a, int32_t* fl_b, hipStream_t st, int halves = 2) {
    if (!ensure_mailbox()) return 0;
    g_scan_ran_on = st;
    g_scan_halves = halves;
    const uint32_t ticket = ++g_ticket ? g_ticket : ++g_ticket;            /* never 0: the mailbox starts zeroed */
    hipLaunchKernelGGL(crt_scan_kernel, dim3(halves), dim3(SCAN_THREADS), 0, st, amax, M, bmax, N, fl_a, fl_b,
                       g_mailbox_dev, ticket);
    return ESHKOL_HIP_OK(hipGetLastError()) ? ticket : 0;
}
/* The same scan for its summary alone, on the library's side stream behind what
 * st holds so far. operand_elems = M K + K N of the product: below ASIDE_FROM the
 * pipeline's kernels last a few microseconds each and the device waits for the
 * host to queue them, so the event, the wait and the launch on a second stream
 * cost more (three calls) than the scan's ten microseconds in line do. */
constexpr uint64_t ASIDE_FROM = 6u << 20;
hipEvent_t scan_event(uint64_t operand_elems) {
    return (operand_elems >= ASIDE_FROM && ensure_mailbox()) ? g_scan_event : nullptr;
}
/* event_attached: the caller made scan_event() the completion event of the last
 * kernel the scan depends on, so no marker needs to be queued behind st. */
uint32_t scan_launch_aside(const double* amax, uint64_t M, const double* bmax, uint64_t N, hipStream_t st,
                           uint64_t operand_elems, bool event_attached, int halves = 2) {
    if (!ensure_mailbox()) return 0;
    if (operand_elems < ASIDE_FROM) return scan_launch(amax, M, bmax, N, nullptr, nullptr, st, halves);
    if ((!event_attached && !ESHKOL_HIP_OK(hipEventRecord(g_scan_event, st))) ||
        !ESHKOL_HIP_OK(hipStreamWaitEvent(g_scan_stream, g_scan_event, 0))) return 0;
    return scan_launch(amax, M, bmax, N, nullptr, nullptr, g_scan_stream, halves);
}
/* the mailbox once the scan that carries `ticket` has written it (its second half is that scan's only if it had two) */
const CrtScan* scan_await(uint32_t ticket) {
    return (ticket != 0 && await_mailbox(ticket, g_scan_ran_on, g_scan_halves) == 0) ? g_mailbox : nullptr;
}

/* device-resident constant tables for the contraction: identity pair lists and moduli */
int32_t* g_tables = nullptr;   /* [0..16] pair_first, [17..32] pair index, [33..48] moduli, [49] the fused scan's counter */
int ensure_tables(hipStream_t st) {
    if (g_tables) return 0;
    int32_t h[17 + 16 + 16 + 1];
    h[49] = 0;
    for (int i = 0; i <= 16; i++) h[i] = i;
    for (int i = 0; i < 16; i++) { h[17 + i] = i; h[33 + i] = H_MODULI[i]; }
    if (!ESHKOL_HIP_OK(hipMalloc((void**)&g_tables, sizeof h))) { g_tables = nullptr; return -1; }
    if (!ESHKOL_HIP_OK(hipMemcpyAsync(g_tables, h, sizeof h, hipMemcpyHostToDevice, st)) ||
        !ESHKOL_HIP_OK(hipStreamSynchronize(st))) { (void)hipFree(g_tables); g_tables = nullptr; return -1; }
    return 0;
}

/* Row maxima, shifts (E fixed) and the scan of A's maxima alone in one launch on st, for a
 * few long rows in front of prepared planes; the ticket, 0 on failure. */
uint32_t rowmax_scan_launch(const double* A, uint64_t M, uint64_t K, double* amax, int32_t* mu, int E, hipStream_t st) {
    if (!ensure_mailbox() || !g_tables || M == 0 || M > (uint64_t)FUSED_MAX_ROWS) return 0;
    g_scan_ran_on = st;
    g_scan_halves = 1;
    const uint32_t ticket = ++g_ticket ? g_ticket : ++g_ticket;
    hipLaunchKernelGGL(crt_rowmax_scan_kernel, dim3((unsigned)M), dim3(256), 0, st, A, M, K, amax, mu, E,
                       (unsigned*)(g_tables + 49), g_mailbox_dev, ticket);
    return ESHKOL_HIP_OK(hipGetLastError()) ? ticket : 0;
}

HipOzakiCrtStages g_last = {};
bool g_force_host_pass = false;
bool g_fused_scan = true;      /* tuning: false keeps the three kernels apart */

template <int NMOD>
void launch_split(const double* X, uint64_t rows, uint64_t K, const int32_t* shift, int8_t* planes,
                  uint64_t rows_padded, uint64_t ldk, bool kmajor, int layout, hipStream_t st) {
    if (kmajor && layout == 1) {
        dim3 grid((unsigned)kmaj::il_blocks(rows_padded, ldk));
        hipLaunchKernelGGL(crt_split_kmajor_il_kernel<NMOD>, grid, dim3(256), 0, st, X, rows, K, shift, planes,
                           rows_padded, ldk);
        return;
    }
    if (kmajor) {
        dim3 grid((unsigned)kmaj::grid_blocks(rows_padded, ldk, eshkol_hip_num_cus()));
        hipLaunchKernelGGL(crt_split_kmajor_kernel<NMOD>, grid, dim3(256), 0, st, X, rows, K, shift, planes,
                           rows_padded, ldk, 0xffffffffu, layout);
        return;
    }
    if (layout == 1) {
        dim3 grid((unsigned)((rows_padded / 32) * (ldk / 32)));
        hipLaunchKernelGGL(crt_split_il_kernel<NMOD>, grid, dim3(256), 0, st, X, rows, K, shift, planes,
                           rows_padded, ldk);
        return;
    }
    if (ldk % 16 == 0 && ((uintptr_t)planes & 15) == 0) {
        dim3 grid((unsigned)(((ldk + 1023) / 1024) * rows_padded));
        hipLaunchKernelGGL(crt_split_staged_kernel<NMOD>, grid, dim3(256), 0, st, X, rows, K, shift, planes,
                           rows_padded, ldk);
        return;
    }
    dim3 grid((unsigned)(((ldk / 2 + 255) / 256) * rows_padded));
    hipLaunchKernelGGL(crt_split_kernel<NMOD>, grid, dim3(256), 0, st, X, rows, K, shift, planes,
                       rows_padded, ldk);
}

}  // namespace

namespace {
int crt_split_any(const double* X, uint64_t rows, uint64_t K, const int32_t* shift, int num_moduli,
                  int8_t* planes, uint64_t rows_padded, uint64_t ldk, bool kmajor, int layout, void* stream) {
    if (!X || !shift || !planes || rows == 0 || K == 0) return -1;
    if (num_moduli < 2 || num_moduli > MAX_MODULI) return -1;
    if (rows_padded < rows || ldk < K || (ldk & 1)) return -1;
    if (layout != 0 && layout != 1) return -1;
    if (layout == 1 && ((rows_padded & 31) || (ldk & 31) || ((uintptr_t)planes & 15))) return -1;
    if (((ldk / 2 + 255) / 256) * rows_padded > 0x7fffffffULL) return -1;
    if (kmaj::tile_count(rows_padded, ldk) > 0x7fffffffULL) return -1;
    hipStream_t st = (hipStream_t)stream;
    switch (num_moduli) {
#define CASE(n) case n: launch_split<n>(X, rows, K, shift, planes, rows_padded, ldk, kmajor, layout, st); break;
        CASE(2) CASE(3) CASE(4) CASE(5) CASE(6) CASE(7) CASE(8) CASE(9)
        CASE(10) CASE(11) CASE(12) CASE(13) CASE(14) CASE(15) CASE(16)
#undef CASE
    }
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}
}  // namespace

static int g_crt_quiet = 0;
void eshkol_crt_set_quiet(int quiet) { g_crt_quiet = quiet; }
int eshkol_crt_quiet(void) { return g_crt_quiet; }

uint32_t eshkol_crt_scan_launch_aside(const double* amax, uint64_t M, const double* bmax, uint64_t N, hipStream_t st,
                                      uint64_t operand_elems, bool event_attached) {
    return scan_launch_aside(amax, M, bmax, N, st, operand_elems, event_attached);
}
hipEvent_t eshkol_crt_scan_event(uint64_t operand_elems) { return scan_event(operand_elems); }

int eshkol_crt_scan_result(uint32_t ticket, CrtMaxima out[2], hipStream_t st) {
    (void)st;
    const CrtScan* h = scan_await(ticket);
    if (!h) return -1;
    for (int o = 0; o < 2; o++) {
        out[o].nonfinite = h[o].nonfinite; out[o].nonzero = h[o].nonzero;
        out[o].e_min = h[o].e_min; out[o].e_max = h[o].e_max;
    }
    return 0;
}

extern "C" int hip_ozaki_crt_split_f64(const double* X, uint64_t rows, uint64_t K,
                                       const int32_t* shift, int num_moduli,
                                       int8_t* planes, uint64_t rows_padded, uint64_t ldk, void* stream) {
    return crt_split_any(X, rows, K, shift, num_moduli, planes, rows_padded, ldk, false, 0, stream);
}

extern "C" int hip_ozaki_crt_split_kmajor_f64(const double* X, uint64_t rows, uint64_t K,
                                              const int32_t* shift, int num_moduli,
                                              int8_t* planes, uint64_t rows_padded, uint64_t ldk, void* stream) {
    return crt_split_any(X, rows, K, shift, num_moduli, planes, rows_padded, ldk, true, 0, stream);
}

extern "C" int hip_ozaki_crt_split_planes_f64(const double* X, uint64_t rows, uint64_t K,
                                              const int32_t* shift, int num_moduli,
                                              int8_t* planes, uint64_t rows_padded, uint64_t ldk,
                                              int kmajor, int layout, void* stream) {
    return crt_split_any(X, rows, K, shift, num_moduli, planes, rows_padded, ldk, kmajor != 0, layout, stream);
}

/* Reconstruction from product planes of wrows rows of ldw bytes each. */
static int crt_reconstruct(const int8_t* w_planes, uint64_t wrows, uint64_t ldw, uint64_t M, uint64_t N, int num_moduli,
                           const double* sl1, const double* sl2, double P1, double P2, double Pinv,
                           const int32_t* mu, const int32_t* nu, const double* bias, int act,
                           double* C, void* stream) {
    if (!w_planes || !sl1 || !sl2 || !mu || !nu || !C || M == 0 || N == 0 || wrows < M || ldw < N) return -1;
    if (num_moduli < 2 || num_moduli > MAX_MODULI || act < 0 || act > 1) return -1;
    if ((((N + 3) / 4 + 255) / 256) * M > 0x7fffffffULL) return -1;
    CrtConsts cc;
    memset(&cc, 0, sizeof cc);
    for (int l = 0; l < num_moduli; l++) { cc.sl1[l] = sl1[l]; cc.sl2[l] = sl2[l]; }
    cc.P1 = P1; cc.P2 = P2; cc.Pinv = Pinv; cc.n = num_moduli;
    dim3 grid((unsigned)((((N + 3) / 4 + 255) / 256) * M));
    /* 4-byte loads of W: its base, pitch and plane size multiples of four (N itself, for dense planes) */
    const bool wvec = (ldw % 4 == 0) && ((wrows * ldw) % 4 == 0) && (((uintptr_t)w_planes & 3) == 0);
    const int vec = !wvec ? 0 : ((N % 4 == 0) && (((uintptr_t)C & 15) == 0)) ? 1 : 2;
    switch (num_moduli) {
#define LAUNCH(n, tanh, v) hipLaunchKernelGGL((crt_reconstruct_kernel<n, tanh, v>), grid, dim3(256), 0,    \
                                              (hipStream_t)stream, w_planes, wrows, ldw, M, N, cc, mu, nu, bias, C)
#define CASE(n) case n:                                                                                   \
        if (act == 1) { if (vec == 1) LAUNCH(n, true, 1); else if (vec == 2) LAUNCH(n, true, 2); else LAUNCH(n, true, 0); } \
        else { if (vec == 1) LAUNCH(n, false, 1); else if (vec == 2) LAUNCH(n, false, 2); else LAUNCH(n, false, 0); }       \
        break;
        CASE(2) CASE(3) CASE(4) CASE(5) CASE(6) CASE(7) CASE(8) CASE(9)
        CASE(10) CASE(11) CASE(12) CASE(13) CASE(14) CASE(15) CASE(16)
#undef CASE
#undef LAUNCH
        default: return -1;
    }
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

extern "C" int hip_ozaki_crt_reconstruct_f64(const int8_t* w_planes, uint64_t M, uint64_t N, int num_moduli,
                                             const double* sl1, const double* sl2,
                                             double P1, double P2, double Pinv,
                                             const int32_t* mu, const int32_t* nu,
                                             const double* bias, int act,
                                             double* C, void* stream) {
    return crt_reconstruct(w_planes, M, N, M, N, num_moduli, sl1, sl2, P1, P2, Pinv, mu, nu, bias, act, C, stream);
}

void eshkol_hip_crt_release(void) {
    if (g_tables) { (void)hipFree(g_tables); g_tables = nullptr; }
    if (g_mailbox) { (void)hipHostFree(g_mailbox); g_mailbox = nullptr; g_mailbox_dev = nullptr; }
    if (g_pinned) { (void)hipHostFree(g_pinned); g_pinned = nullptr; g_pinned_bytes = 0; }
    if (g_scan_event) { (void)hipEventDestroy(g_scan_event); g_scan_event = nullptr; }
    if (g_scan_stream) { (void)hipStreamDestroy(g_scan_stream); g_scan_stream = nullptr; }
    g_scan_ran_on = nullptr;
    g_ticket = 0;
    g_last = HipOzakiCrtStages{};
}

extern "C" void hip_ozaki_crt_set_host_pass(int on) { EshkolHipLock lk; g_force_host_pass = on != 0; }
extern "C" void hip_ozaki_crt_set_fused_scan(int on) { EshkolHipLock lk; g_fused_scan = on != 0; }

extern "C" int hip_ozaki_crt_set_aligned_weights(int on) {
    EshkolHipLock lk;
    const int was = g_aligned_weights ? 1 : 0;
    g_aligned_weights = on != 0;
    return was;
}

extern "C" int hip_ozaki_crt_last_stages(HipOzakiCrtStages* out) {
    EshkolHipLock lk;
    if (!out || !g_last.a_planes) return -1;
    *out = g_last;
    return 0;
}

/* ---- a second operand prepared once (constant weights) ----------------------------
 * What the tier derives from B alone: its column maxima and its residue planes.
 * With sixteen moduli the exponent E is 52 whatever the operands are, so the
 * planes of a B that does not change do not change either, and a layer that
 * multiplies fresh activations by the same weights need only split the
 * activations. The planes are the bytes the tier would compute itself, so the
 * result is the same bit for bit. */
int eshkol_hip_igemm_direct_mode(void);     /* igemm_i8.hip: 1 unless a test forces a kernel */
namespace {
struct CrtPreparedB {
    uint32_t magic;
    const double* src;          /* the operand the planes were made from */
    uint64_t K, N, rows_padded, ldk;
    int trans_b, n_mod, layout;
    double* bmax;               /* [N] column maxima, device */
    int32_t* nu;                /* [N] shifts 52 - floor(log2 max), device */
    int8_t* planes;             /* [n_mod][rows_padded][ldk], device */
    CrtScan scan;               /* the scan's summary of bmax: it does not change either */
};
constexpr uint32_t PREPARED_MAGIC = 0x43525442u;
}  // namespace

static int crt_matmul_impl(const double* A, const double* B, double* C,
                           uint64_t M, uint64_t K, uint64_t N,
                           int trans_a, int trans_b,
                           int num_moduli, int adaptive,
                           const double* bias, int act, void* stream, const CrtPreparedB* prepared) {
    EshkolHipCall bracket(stream);
    if (!A || !B || !C || M == 0 || K == 0 || N == 0) return -1;
    if (M > 0x7fffffffULL || N > 0x7fffffffULL) return -1;
    /* int32 accumulation of |a*b| <= 128*128 is exact while K*16384 < 2^31 */
    if (K > 131071) {
        static bool warned = false;
        if (!warned) {
            warned = true;
            fprintf(stderr, "[GPU] Ozaki-II: K=%llu exceeds the int32-exact bound 131071; "
                            "falling back to the native fp64 GEMM\n", (unsigned long long)K);
        }
        return -1;
    }
    if (num_moduli < 2) num_moduli = 2;
    if (num_moduli > MAX_MODULI) {
        fprintf(stderr, "[GPU] Ozaki-II: requested N=%d exceeds max %d (would overflow "
                        "__int128 P); clamping to %d\n", num_moduli, MAX_MODULI, MAX_MODULI);
        num_moduli = MAX_MODULI;
    }
    hipStream_t st = (hipStream_t)stream;
    if (ensure_tables(st) != 0) return -1;

    /* planes interleaved (and the k pitch padded to whole groups of four 128-byte
     * blocks) when the contraction will take the kernel that wants them so */
    /* Interleaved planes serve every row count (the kernels that take them run with any
     * number of tiles), so a second operand prepared in that layout keeps it; row-major
     * planes serve only the products that would make row-major planes themselves. */
    const bool keep_interleaved = prepared && prepared->layout == 1 && !adaptive && !g_force_host_pass &&
                                  prepared->n_mod == num_moduli && eshkol_hip_igemm_direct_mode() == 1;
    const int layout = keep_interleaved ? 1 : hip_igemm_plane_layout_single(M, K, N, num_moduli);
    /* a first operand of a few rows goes to the kernel that streams the second operand's
     * planes: its own planes then need whole blocks of 32 rows only */
    const bool thin = layout == 1 && eshkol_hip_igemm_is_thin(M, N);
    const uint64_t Mp = round_up_sz(M, thin ? 32 : 256), Np = round_up_sz(N, 256), ldk = round_up_sz(K, layout ? 512 : 256);
    /* Both operands come out as planes [row][k]. An operand stored with k
     * contiguous (A as given, B when the caller holds B^T) is read row by row;
     * one stored k-major (B as given, A when the caller holds A^T) is read
     * through LDS tiles: no transposed fp64 copy is made either way. */
    const bool a_kmajor = trans_a != 0, b_kmajor = trans_b == 0;
    /* prepared planes apply when they are what this call would compute: same
     * operand shape, moduli, layout and pitch, and E fixed at 52 (checked below) */
    const bool use_prepared = prepared && !adaptive && !g_force_host_pass && prepared->n_mod == num_moduli &&
                              prepared->K == K && prepared->N == N && prepared->trans_b == trans_b &&
                              prepared->layout == layout && prepared->ldk == ldk && prepared->rows_padded == Np &&
                              floor((crt_constants(num_moduli).log2P - 3.0 - log2((double)K)) / 2.0) >= 52.0;
    double* amax = (double*)eshkol_hip_workspace(WS_ROWSCALE, M * sizeof(double));
    double* bmax = use_prepared ? prepared->bmax : (double*)eshkol_hip_workspace(WS_COLSCALE, N * sizeof(double));
    int32_t* dmu = (int32_t*)eshkol_hip_workspace(WS_ROWSHIFT, M * sizeof(int32_t));
    int32_t* dnu = (int32_t*)eshkol_hip_workspace(WS_COLSHIFT, N * sizeof(int32_t));
    if (!amax || !bmax || !dmu || !dnu) return -1;
    char* host = (char*)pinned((M + N) * (sizeof(double) + sizeof(int32_t)));
    if (!host) return -1;
    double* h_amax = (double*)host;
    double* h_bmax = h_amax + M;
    int32_t* h_mu = (int32_t*)(h_bmax + N);
    int32_t* h_nu = h_mu + M;

    /* E = min(52, floor((log2 P - 1 - log2 K - frac_A - frac_B) / 2)) with both
     * fractions below 1 (gpu_memory.mm:2510-2512): where even frac_A + frac_B = 2
     * leaves 52 (16 moduli: every K this tier accepts), E does not depend on the
     * operands. Then the kernels that find the maxima write the shifts as well, the
     * scan of the maxima (non-finite input? shifts in range? a maximum so close to a
     * power of two that libm's log2 may round across it?) runs beside the pipeline
     * on a stream of its own, and nothing on the device waits for it. */
    const double log2K = log2((double)K);
    const bool fixed_E = !adaptive && !g_force_host_pass &&
                         floor((crt_constants(num_moduli).log2P - 3.0 - log2K) / 2.0) >= 52.0;
    int32_t* const mu_out = fixed_E ? dmu : nullptr;
    int32_t* const nu_out = fixed_E ? dnu : nullptr;
    /* a few long rows in front of prepared planes: maxima, shifts and scan in one launch */
    /* (up to 160 rows: beyond, the workgroups' fences and their additions to the one counter cost what the launches saved) */
    const bool fused_scan = use_prepared && !a_kmajor && M <= 160 && K >= 1024 && g_fused_scan;
    uint32_t ticket = 0;
    if (fused_scan) {
        ticket = rowmax_scan_launch(A, M, K, amax, dmu, 52, st);
    } else {
        /* the last kernel that writes maxima carries the event the scan's stream waits for */
        const hipEvent_t fork = fixed_E ? scan_event(M * K + K * N) : nullptr;
        const hipEvent_t fork_a = use_prepared ? fork : nullptr, fork_b = use_prepared ? nullptr : fork;
        if ((a_kmajor ? eshkol_colabsmax_shift_f64(A, K, M, 0.0, amax, mu_out, 52, st, fork_a)
                      : eshkol_rowabsmax_shift_f64(A, M, K, 0.0, amax, mu_out, 52, st, fork_a)) != 0) return -1;
        if (!use_prepared &&
            (b_kmajor ? eshkol_colabsmax_shift_f64(B, K, N, 0.0, bmax, nu_out, 52, st, fork_b)
                      : eshkol_rowabsmax_shift_f64(B, N, K, 0.0, bmax, nu_out, 52, st, fork_b)) != 0) return -1;
        /* prepared planes: the scan looks at A's maxima only, B's summary was kept with the planes */
        ticket = fixed_E ? scan_launch_aside(amax, M, bmax, N, st, M * K + K * N, fork != nullptr, use_prepared ? 1 : 2)
                         : scan_launch(amax, M, bmax, N, dmu, dnu, st);
    }
    if (!ticket) return -1;
    CrtScan merged[2];
    auto await_scan = [&]() -> const CrtScan* {
        const CrtScan* h = scan_await(ticket);
        if (!h || !use_prepared) return h;
        merged[0] = h[0];
        merged[1] = prepared->scan;
        return merged;
    };

    /* Everything after the shifts, queued in one go. */
    auto enqueue_products = [&](int n_mod, const HostCrt& crt, int E, bool b_ready) -> int {
        const int32_t* nu = b_ready ? prepared->nu : dnu;
        int8_t* Ap = (int8_t*)eshkol_hip_workspace(WS_APLANES, (size_t)n_mod * Mp * ldk);
        int8_t* Bp = b_ready ? prepared->planes : (int8_t*)eshkol_hip_workspace(WS_BPLANES, (size_t)n_mod * Np * ldk);
        const uint64_t Mw = eshkol_product_rows(M), Nw = eshkol_product_pitch(N);
        int8_t* Wp = (int8_t*)eshkol_hip_workspace(WS_PRODUCTS, (size_t)n_mod * Mw * Nw);
        if (!Ap || !Bp || !Wp) return -1;
        if (crt_split_any(A, M, K, dmu, n_mod, Ap, Mp, ldk, a_kmajor, layout, st) != 0) return -1;
        if (!b_ready && crt_split_any(B, N, K, dnu, n_mod, Bp, Np, ldk, b_kmajor, layout, st) != 0) return -1;
        HipIgemmArgs ga;
        memset(&ga, 0, sizeof ga);
        ga.a_planes = Ap; ga.b_planes = Bp;
        ga.a_plane_stride = Mp * ldk; ga.b_plane_stride = Np * ldk;
        ga.ldk = (uint32_t)ldk; ga.M = (uint32_t)M; ga.N = (uint32_t)N; ga.n_out = (uint32_t)n_mod;
        ga.pair_first = g_tables; ga.pair_a = g_tables + 17; ga.pair_b = g_tables + 17;
        ga.mode = 1; ga.max_pairs = 1; ga.modulus = g_tables + 33; ga.out_i8 = Wp;
        ga.layout = layout;
        ga.out_rows = (uint32_t)Mw; ga.ldn = (uint32_t)Nw;
        if (hip_igemm_i8(&ga, st) != 0) return -1;
        if (crt_reconstruct(Wp, Mw, Nw, M, N, n_mod, crt.sl1, crt.sl2, crt.P1, crt.P2, crt.Pinv,
                            dmu, nu, bias, act, C, st) != 0) return -1;
        g_last.a_planes = Ap; g_last.b_planes = Bp; g_last.w_planes = Wp;
        g_last.w_rows = Mw; g_last.w_ld = Nw;
        g_last.mu = dmu; g_last.nu = (int32_t*)nu;
        g_last.rows_a_padded = Mp; g_last.rows_b_padded = Np; g_last.ldk = ldk;
        g_last.num_moduli = n_mod; g_last.E = E; g_last.layout = layout;
        return 0;
    };
    auto announce = [&](int n_mod, const HostCrt& crt) {
        if (!eshkol_crt_quiet()) fprintf(stderr, "[GPU] Ozaki-II: N=%d%s, log2(P)=%.1f\n", n_mod,
                adaptive ? " (adaptive)" : "", crt.log2P);       /* gpu_memory.mm:2503 */
    };
    auto in_range = [](int E, bool any, int e_min, int e_max) {
        /* every shift E - floor(log2 max) must be an exponent ldexp can apply exactly */
        return !any || (E - e_min <= 1023 && E - e_max >= -1022);
    };

    /* With E fixed the whole pipeline is queued at once. The scan's summary is read
     * afterwards; what it may still demand is a refusal (non-finite input, shifts
     * out of range: C then holds no result) or the reference's own pass over the
     * maxima, after which the products are queued a second time. */
    const CrtScan* h_scan = nullptr;
    bool announced = false;
    if (fixed_E) {
        const HostCrt& crt = crt_constants(num_moduli);
        const int E = 52;
        if (enqueue_products(num_moduli, crt, E, use_prepared) != 0) return -1;
        announce(num_moduli, crt);
        announced = true;
        h_scan = await_scan();
        if (!h_scan) return -1;
        if (h_scan[0].nonfinite || h_scan[1].nonfinite) return -1;  /* NaN/Inf input */
        if (!h_scan[0].extreme && !h_scan[1].extreme) {
            for (int o = 0; o < 2; o++)
                if (!in_range(E, h_scan[o].nonzero != 0, h_scan[o].e_min, h_scan[o].e_max)) return -1;
            return 0;
        }
    }
    if (!h_scan) h_scan = await_scan();
    if (!h_scan) return -1;
    if (h_scan[0].nonfinite || h_scan[1].nonfinite) return -1;          /* NaN/Inf input */

    /* frac bounds (gpu_memory.mm:403-417) and the range of floor(log2 max) per operand */
    double frac[2] = {0.0, 0.0};
    int e_min[2], e_max[2];
    bool any[2];
    const bool full_pass = g_force_host_pass || h_scan[0].extreme || h_scan[1].extreme ||
                           h_scan[0].ncand > SCAN_CAND || h_scan[1].ncand > SCAN_CAND;
    if (!full_pass) {
        for (int o = 0; o < 2; o++) {
            for (int c = 0; c < h_scan[o].ncand; c++) {
                const double lg = log2(h_scan[o].cand[c]), f = lg - floor(lg);
                if (f > frac[o]) frac[o] = f;
            }
            any[o] = h_scan[o].nonzero != 0; e_min[o] = h_scan[o].e_min; e_max[o] = h_scan[o].e_max;
        }
    } else {
        /* the reference's own pass: one log2 per maximum */
        if (!ESHKOL_HIP_OK(hipMemcpyAsync(h_amax, amax, M * sizeof(double), hipMemcpyDeviceToHost, st))) return -1;
        if (!ESHKOL_HIP_OK(hipMemcpyAsync(h_bmax, bmax, N * sizeof(double), hipMemcpyDeviceToHost, st))) return -1;
        if (!ESHKOL_HIP_OK(hipStreamSynchronize(st))) return -1;
        const double* h_max[2] = { h_amax, h_bmax };
        int32_t* h_fl[2] = { h_mu, h_nu };
        const uint64_t cnt[2] = { M, N };
        for (int o = 0; o < 2; o++) {
            any[o] = false; e_min[o] = INT32_MAX; e_max[o] = INT32_MIN;
            for (uint64_t i = 0; i < cnt[o]; i++) {
                const double m = h_max[o][i];
                h_fl[o][i] = FL_ZERO;
                if (m > 0.0) {
                    const double lg = log2(m), fl = floor(lg), f = lg - fl;
                    const int e = (int)fl;
                    h_fl[o][i] = e;
                    if (f > frac[o]) frac[o] = f;
                    any[o] = true;
                    if (e < e_min[o]) e_min[o] = e;
                    if (e > e_max[o]) e_max[o] = e;
                }
            }
        }
        if (!ESHKOL_HIP_OK(hipMemcpyAsync(dmu, h_mu, M * sizeof(int32_t), hipMemcpyHostToDevice, st))) return -1;
        if (!ESHKOL_HIP_OK(hipMemcpyAsync(dnu, h_nu, N * sizeof(int32_t), hipMemcpyHostToDevice, st))) return -1;
    }
    const double frac_A = frac[0], frac_B = frac[1];
    if (adaptive) {                                   /* gpu_memory.mm:433-453 */
        std::call_once(g_cumul_once, [] {
            g_log2_cumul[0] = 0.0;
            for (int i = 0; i < MAX_MODULI; i++) g_log2_cumul[i + 1] = g_log2_cumul[i] + log2((double)H_MODULI[i]);
        });
        int chosen = num_moduli;
        for (int n = 2; n <= num_moduli; n++) {
            double emax = floor((g_log2_cumul[n] - 1.0 - log2K - frac_A - frac_B) / 2.0);
            if (emax >= 52.0) { chosen = n; break; }
        }
        num_moduli = chosen;
    }
    const HostCrt& crt = crt_constants(num_moduli);
    int E = (int)floor((crt.log2P - 1.0 - log2K - frac_A - frac_B) / 2.0);   /* gpu_memory.mm:2510-2512 */
    if (E > 52) E = 52;
    if (E < 0) E = 0;
    for (int o = 0; o < 2; o++)
        if (!in_range(E, any[o], e_min[o], e_max[o])) return -1;
    hipLaunchKernelGGL(crt_shift_kernel, dim3((unsigned)((M + N + 255) / 256)), dim3(256), 0, st, dmu, M, dnu, N, E);
    /* this path recomputes the shifts (libm on every maximum, or another E): the
     * planes are split again from B itself, prepared or not */
    if (enqueue_products(num_moduli, crt, E, false) != 0) return -1;
    if (!announced) announce(num_moduli, crt);
    return 0;
}

extern "C" int hip_matmul_ozaki_crt_f64_ex(const double* A, const double* B, double* C,
                                           uint64_t M, uint64_t K, uint64_t N,
                                           int trans_a, int trans_b,
                                           int num_moduli, int adaptive,
                                           const double* bias, int act, void* stream) {
    return crt_matmul_impl(A, B, C, M, K, N, trans_a, trans_b, num_moduli, adaptive, bias, act, stream, nullptr);
}

extern "C" int hip_ozaki_crt_prepare_operand_b(const double* B, uint64_t K, uint64_t N, int trans_b,
                                               int num_moduli, uint64_t M_expected, void** handle, void* stream) {
    if (!B || !handle || K == 0 || N == 0 || K > 131071 || N > 0x7fffffffULL) return -1;
    *handle = nullptr;
    if (num_moduli < 2 || num_moduli > MAX_MODULI) return -1;
    EshkolHipCall bracket(stream);
    hipStream_t st = (hipStream_t)stream;
    const HostCrt& crt = crt_constants(num_moduli);
    /* only where E does not depend on the operands (gpu_memory.mm:2510-2512) */
    if (!(floor((crt.log2P - 3.0 - log2((double)K)) / 2.0) >= 52.0)) return -1;
    const int layout = hip_igemm_plane_layout_single(M_expected ? M_expected : 1, K, N, num_moduli);
    const uint64_t Np = round_up_sz(N, 256), ldk = round_up_sz(K, layout ? 512 : 256);
    const bool b_kmajor = trans_b == 0;
    CrtPreparedB* pb = new CrtPreparedB();
    pb->magic = PREPARED_MAGIC; pb->src = B; pb->K = K; pb->N = N; pb->rows_padded = Np; pb->ldk = ldk;
    pb->trans_b = trans_b; pb->n_mod = num_moduli; pb->layout = layout;
    pb->bmax = nullptr; pb->nu = nullptr; pb->planes = nullptr;
    auto fail = [&]() {
        if (pb->bmax) (void)hipFree(pb->bmax);
        if (pb->nu) (void)hipFree(pb->nu);
        if (pb->planes) (void)hipFree(pb->planes);
        delete pb;
        return -1;
    };
    if (!ESHKOL_HIP_OK(hipMalloc((void**)&pb->bmax, N * sizeof(double))) ||
        !ESHKOL_HIP_OK(hipMalloc((void**)&pb->nu, N * sizeof(int32_t))) ||
        !ESHKOL_HIP_OK(hipMalloc((void**)&pb->planes, (size_t)num_moduli * Np * ldk))) { (void)hipGetLastError(); fail(); return -2; }
    if ((b_kmajor ? eshkol_colabsmax_shift_f64(B, K, N, 0.0, pb->bmax, pb->nu, 52, st)
                  : eshkol_rowabsmax_shift_f64(B, N, K, 0.0, pb->bmax, pb->nu, 52, st)) != 0)
        return fail();
    /* the scan takes two vectors of maxima: B's stand in for both */
    const CrtScan* h = scan_await(scan_launch(pb->bmax, N, pb->bmax, N, nullptr, nullptr, st));
    if (!h || h[1].nonfinite || h[1].extreme) return fail();     /* such a B takes the full pass on every call */
    if (h[1].nonzero && !(52 - h[1].e_min <= 1023 && 52 - h[1].e_max >= -1022)) return fail();
    pb->scan = h[1];
    if (crt_split_any(B, N, K, pb->nu, num_moduli, pb->planes, Np, ldk, b_kmajor, layout, st) != 0) return fail();
    if (!ESHKOL_HIP_OK(hipStreamSynchronize(st))) return fail();
    *handle = pb;
    return 0;
}

extern "C" void hip_ozaki_crt_release_prepared(void* handle) {
    CrtPreparedB* pb = (CrtPreparedB*)handle;
    if (!pb || pb->magic != PREPARED_MAGIC) return;
    EshkolHipCall bracket(eshkol_hip_stream());     /* queues nothing: no caller's stream to order against */
    (void)hipDeviceSynchronize();
    (void)hipFree(pb->bmax);
    (void)hipFree(pb->nu);
    (void)hipFree(pb->planes);
    pb->magic = 0;
    delete pb;
}

extern "C" int hip_matmul_ozaki_crt_prepared_f64(const double* A, const void* prepared_b, double* C,
                                                 uint64_t M, uint64_t K, uint64_t N, int trans_a,
                                                 int num_moduli, int adaptive,
                                                 const double* bias, int act, void* stream) {
    const CrtPreparedB* pb = (const CrtPreparedB*)prepared_b;
    if (!pb || pb->magic != PREPARED_MAGIC || pb->K != K || pb->N != N) return -1;
    return crt_matmul_impl(A, pb->src, C, M, K, N, trans_a, pb->trans_b, num_moduli, adaptive, bias, act, stream, pb);
}

extern "C" int hip_matmul_ozaki_crt_f64(const double* A, const double* B, double* C,
                                        uint64_t M, uint64_t K, uint64_t N,
                                        int num_moduli, int adaptive,
                                        const double* bias, int act, void* stream) {
    return hip_matmul_ozaki_crt_f64_ex(A, B, C, M, K, N, 0, 0, num_moduli, adaptive, bias, act, stream);
}
