/*
 * Ozaki-II reduced-precision ("fast") CRT tier: C = A*B from int8 matrix-core
 * products modulo a handful of small prime powers, reconstructed by a
 * fractional CRT. Follows ozaki_ii_fast_dispatch of the reference
 * (lib/backend/gpu/gpu_memory.mm:2802-3012) and its kernels
 * (lib/backend/gpu/metal_softfloat.h:4126-4246):
 *
 *   moduli   the n largest prime powers <= cap; cap is the reference's, the
 *            largest p with K floor(p/2)^2 < 2^24 (there it keeps an f32 GEMM
 *            exact; here it keeps the moduli, hence every integer of the tier,
 *            the reference's)
 *   E        floor((log2 P - log2 K - 2) / 2) in [1, 52]: a function of K and n only
 *   e_i,f_j  exponents of the row / column maxima (frexp), so all scaling is by
 *            powers of two and nothing in the pipeline needs libm
 *   split    round-half-up(|x| 2^(E-e)) with x's sign, modulo p, in [-p/2, p/2]
 *            with +p/2 for the even moduli's tie; int8 planes [row][k]
 *   product  W_l = (A_l B_l^T) mod p_l               int8 MFMA, int32 accumulate
 *   C        frac(sum_l ((W_l q_l) mod p_l) / p_l) centred, times P 2^(e_i+f_j-2E)
 *
 * The reference carries the last step in float pairs (Apple GPUs have no fp64);
 * here it is plain fp64, which resolves 2^-52 of P instead of about 2^-45. The
 * integers (residues, products modulo p) are the reference's bit for bit.
 */
#include "hip_common.h"
#include "kernels.h"
#include "kmajor_tile.h"
#include "crt_shared.h"

#include <cmath>
#include <cstring>
#include <vector>
#include <algorithm>

typedef double d2_t __attribute__((ext_vector_type(2)));
typedef uint32_t v4u_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int FAST_MAX_MODULI = 16;             /* gpu_memory.mm:264 */

/* What the split needs to know about the moduli; passed by value. */
struct FastTable {
    int n;
    int p[FAST_MAX_MODULI];
    uint32_t wlo[FAST_MAX_MODULI], whi[FAST_MAX_MODULI];
    float pinv[FAST_MAX_MODULI];
    uint32_t neg_half[FAST_MAX_MODULI];         /* the byte of -p/2 for even p, else 0x100 (never a byte) */
};

/* The int8 residues of four integers modulo p_l, packed into a word. Two byte
 * dot products give x < 2^19 congruent to s; one fma against 1.5 * 2^23 leaves the
 * nearest integer to x/p in the low bits of a float; the low byte of
 * x - (2^22 + q) p is the residue in [-p/2, p/2]: five instructions, and the four
 * low bytes are gathered by two byte permutes and an or. The even moduli are
 * powers of two, their 1/p is exact, so their tie x = p/2 (mod p) comes out as
 * +p/2 or -p/2 with the parity of q: -p/2 is folded to the +p/2 the reference
 * stores (metal_softfloat.h:4174-4177). Only an even modulus pays for that test
 * (the branch is the same for every lane): there is at most one among the
 * moduli, and the split is bound by its vector instructions. */
__device__ __forceinline__ uint32_t fast_residue_raw(Scaled s, const FastTable& t, int l) {
    const uint32_t x = __builtin_amdgcn_udot4(s.lo, t.wlo[l], __builtin_amdgcn_udot4(s.hi, t.whi[l], 0u, false), false);
    const float qm = fmaf((float)x, t.pinv[l], 12582912.0f);
    return (uint32_t)(__mul24(__float_as_int(qm), -t.p[l]) + (int)x);         /* the residue is the low byte */
}

__device__ __forceinline__ uint32_t fast_residues4(Scaled s0, Scaled s1, Scaled s2, Scaled s3, const FastTable& t, int l) {
    uint32_t r0 = fast_residue_raw(s0, t, l), r1 = fast_residue_raw(s1, t, l);
    uint32_t r2 = fast_residue_raw(s2, t, l), r3 = fast_residue_raw(s3, t, l);
    if (t.neg_half[l] != 0x100u) {
        const uint32_t nh = t.neg_half[l], half = (uint32_t)t.p[l] >> 1;
        r0 = ((r0 & 0xffu) == nh) ? half : r0;
        r1 = ((r1 & 0xffu) == nh) ? half : r1;
        r2 = ((r2 & 0xffu) == nh) ? half : r2;
        r3 = ((r3 & 0xffu) == nh) ? half : r3;
    }
    return __builtin_amdgcn_perm(r1, r0, 0x0c0c0400u) | __builtin_amdgcn_perm(r3, r2, 0x04000c0cu);
}

/* Row-major X[rows][K], pitch a multiple of 16: a block takes 1024 k of one row,
 * a thread four of them; the residues are collected in LDS and leave as 16-byte
 * stores (the layout of the exact tier's split). */
__global__ __launch_bounds__(256)
void fast_split_kernel(const double* __restrict__ X, uint64_t rows, uint64_t K,
                       const int32_t* __restrict__ shift, FastTable tbl, int8_t* __restrict__ planes,
                       uint64_t rows_padded, uint64_t ldk) {
    __shared__ __align__(16) uint32_t stage[FAST_MAX_MODULI][256];
    const uint32_t cpr = (uint32_t)((ldk + 1023) / 1024);
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
    Scaled s[4];
#pragma unroll
    for (int e = 0; e < 4; e++) s[e] = scaled_integer<true>(x[e], sh);
#pragma unroll
    for (int l = 0; l < FAST_MAX_MODULI; l++)
        if (l < tbl.n)
            stage[l][tid] = fast_residues4(s[0], s[1], s[2], s[3], tbl, l);
    __syncthreads();
    const uint64_t plane_stride = rows_padded * ldk;
    for (int c = tid; c < tbl.n * 64; c += 256) {
        const int plane = c >> 6, ch = c & 63;
        const uint64_t kk = kbase + 16 * (uint64_t)ch;
        if (kk < ldk)
            *(v4u_t*)(planes + (uint64_t)plane * plane_stride + row * ldk + kk) = *(const v4u_t*)&stage[plane][4 * ch];
    }
}

/* Row-major X[rows][K], interleaved planes (rows_padded and ldk multiples of 32):
 * a block takes 32 rows x 32 k, a thread four consecutive k of one row, and each
 * plane's share of the block is one operand fragment, 1 KiB of contiguous memory
 * (the layout of the exact tier's interleaved split). */
__global__ __launch_bounds__(256)
void fast_split_il_kernel(const double* __restrict__ X, uint64_t rows, uint64_t K,
                          const int32_t* __restrict__ shift, FastTable tbl, int8_t* __restrict__ planes,
                          uint64_t rows_padded, uint64_t ldk) {
    __shared__ __align__(16) uint32_t stage[FAST_MAX_MODULI][256];
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
    Scaled s[4];
#pragma unroll
    for (int e = 0; e < 4; e++) s[e] = scaled_integer<true>(x[e], sh);
#pragma unroll
    for (int l = 0; l < FAST_MAX_MODULI; l++)
        if (l < tbl.n)
            stage[l][tid] = fast_residues4(s[0], s[1], s[2], s[3], tbl, l);
    __syncthreads();
    const uint64_t plane_stride = rows_padded * ldk;
    int8_t* frag = planes + rb * (32 * ldk) + kb * 1024;
    for (int c = tid; c < tbl.n * 64; c += 256) {
        const int plane = c >> 6, q = c & 63;
        eshkol_store_streaming((v4u_t*)(frag + (uint64_t)plane * plane_stride + 16 * q),
                               *(const v4u_t*)&stage[plane][8 * (q & 31) + 4 * (q >> 5)]);
    }
}

/* k-major X[K][rows] (B as the runtime stores it), same planes. */
__global__ __launch_bounds__(256, 4)
void fast_split_kmajor_kernel(const double* __restrict__ X, uint64_t rows, uint64_t K,
                              const int32_t* __restrict__ shift, FastTable tbl, int8_t* __restrict__ planes,
                              uint64_t rows_padded, uint64_t ldk, int layout) {
    __shared__ __align__(16) double tile[kmaj::SMEM_DOUBLES];
    const uint64_t plane_stride = rows_padded * ldk;
    kmaj::for_each_16(X, rows, K, rows_padded, ldk, 0xffffffffu, tile,
        [&](uint64_t row) { return (row < rows) ? shift[row] : 0; },
        [&](uint64_t row, uint64_t k, const double* x, int sh) {
            Scaled s[16];
#pragma unroll
            for (int e = 0; e < 16; e++) s[e] = scaled_integer<true>(x[e], sh);
            int8_t* out = planes + eshkol_plane_offset(layout, row, k, ldk);
#pragma unroll 1
            for (int l = 0; l < tbl.n; l++) {
                v4u_t w;
#pragma unroll
                for (int g = 0; g < 4; g++)
                    w[g] = fast_residues4(s[4 * g], s[4 * g + 1], s[4 * g + 2], s[4 * g + 3], tbl, l);
                eshkol_store_streaming((v4u_t*)(out + (uint64_t)l * plane_stride), w);
            }
        });
}

/* k-major X[K][rows], interleaved planes: no LDS (kmajor_tile.h). */
__global__ __launch_bounds__(256, 4)
void fast_split_kmajor_il_kernel(const double* __restrict__ X, uint64_t rows, uint64_t K,
                                 const int32_t* __restrict__ shift, FastTable tbl, int8_t* __restrict__ planes,
                                 uint64_t rows_padded, uint64_t ldk) {
    uint64_t row, k;
    kmaj::il_thread(rows_padded, &row, &k);
    if (row >= rows_padded || k >= ldk) return;
    double x[16];
    kmaj::load_k16(X, rows, K, row, k, x);
    const int sh = (row < rows) ? shift[row] : 0;
    Scaled s[16];
#pragma unroll
    for (int e = 0; e < 16; e++) s[e] = scaled_integer<true>(x[e], sh);
    int8_t* out = planes + eshkol_plane_offset(1, row, k, ldk);
    const uint64_t plane_stride = rows_padded * ldk;
#pragma unroll 1
    for (int l = 0; l < tbl.n; l++) {
        v4u_t w;
#pragma unroll
        for (int g = 0; g < 4; g++)
            w[g] = fast_residues4(s[4 * g], s[4 * g + 1], s[4 * g + 2], s[4 * g + 3], tbl, l);
        eshkol_store_streaming((v4u_t*)(out + (uint64_t)l * plane_stride), w);
    }
}

/* Fractional CRT (metal_softfloat.h:4183-4246): frac(sum_l ((w_l q_l) mod p_l) / p_l),
 * centred, times P 2^(e_i + f_j - 2E). The fractions are added in 64-bit fixed
 * point, where "modulo 1" is the wrap of the integer and "centred" is reading it
 * as signed: with d_l = floor(2^64 q_l / p_l), w_l d_l mod 2^64 is
 * frac(w_l q_l / p_l) to within |w_l| 2^-64, so no modular reduction of w_l q_l is
 * needed at all. d_l is held as four 16-bit limbs and each limb's sum over the
 * moduli is one 24-bit multiply-add per residue into a 32-bit register
 * (16 * 128 * 65535 < 2^27); the limbs are put together once per element. Total
 * error below 2^-53 of P (the reference's float pairs resolve about 2^-45).
 * One thread: four consecutive columns of a row. The number of planes is a
 * template parameter so that a thread's loads of all planes are issued together
 * (the kernel moves 8 + n bytes per element and has to keep HBM busy). */
struct FracLimbs { int32_t d[FAST_MAX_MODULI][4]; };

/* W is [NMOD][wrows][ldw], the product planes as the contraction left them.
 * VEC 1: N is a multiple of four and W and C are aligned for 4- and 16-byte
 * accesses (the launcher checks): the kernel then carries none of the byte-wise
 * path, whose address arithmetic would otherwise sit in front of both paths.
 * VEC 2: W allows the 4-byte loads, but N is not a multiple of four or C's rows
 * do not start on 16-byte boundaries: whole groups of four leave as two 16-byte
 * words at 8-byte alignment, a row's last group element by element.
 * VEC 0: nothing is known about W either (dense planes of any N). */
typedef double d2u_t __attribute__((ext_vector_type(2), aligned(8)));
template <int NMOD, int VEC>
__global__ __launch_bounds__(256)
void fast_reconstruct_kernel(const int8_t* __restrict__ W, uint64_t wrows, uint64_t ldw, uint64_t M, uint64_t N,
                             FracLimbs fl, double P_over_2_64,
                             const int32_t* __restrict__ sh_a, const int32_t* __restrict__ sh_b,
                             double* __restrict__ C) {
    const uint32_t cpr = (uint32_t)(((N + 3) / 4 + 255) / 256);
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
    int sb[4] = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < 4; e++) if (e < nvalid) sb[e] = sh_b[col + e];
    int32_t acc[4][4];
#pragma unroll
    for (int e = 0; e < 4; e++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[e][j] = 0;
#pragma unroll
    for (int l = 0; l < NMOD; l++) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int w = (int)(int8_t)(u[l] >> (8 * e));
#pragma unroll
            for (int j = 0; j < 4; j++) acc[e][j] += __mul24(w, fl.d[l][j]);
        }
    }
    const int sa = sh_a[row];
    double out[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int64_t S = (int64_t)acc[e][0] + ((int64_t)acc[e][1] << 16) + ((int64_t)acc[e][2] << 32) +
                          (int64_t)((uint64_t)(int64_t)acc[e][3] << 48);
        /* S / 2^64 is the centred fraction; (double)S in two halves */
        const double f = fma((double)(int32_t)(S >> 32), 4294967296.0, (double)(uint32_t)S);
        out[e] = ldexp(f * P_over_2_64, -(sa + sb[e]));
    }
    if (VEC == 1) {
        d2_t lo, hi;
        lo.x = out[0]; lo.y = out[1]; hi.x = out[2]; hi.y = out[3];
        ((d2_t*)(C + idx))[0] = lo; ((d2_t*)(C + idx))[1] = hi;
    } else if (VEC == 2 && nvalid == 4) {
        d2u_t lo, hi;
        lo.x = out[0]; lo.y = out[1]; hi.x = out[2]; hi.y = out[3];
        ((d2u_t*)(C + idx))[0] = lo; ((d2u_t*)(C + idx))[1] = hi;
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) if (e < nvalid) C[idx + e] = out[e];
    }
}

/* ---- host side -------------------------------------------------------------- */

struct FastPlan {
    int n = 0, cap = 0, E = 0;
    int moduli[FAST_MAX_MODULI] = {}, q[FAST_MAX_MODULI] = {};
    double log2P = 0.0, P = 0.0;
    FastTable table = {};
    FracLimbs limbs = {};
};

/* gpu_memory.mm:2802-2814 */
std::vector<int> build_moduli(int cap, int n_mod) {
    std::vector<int> pp;
    for (int p = 2; p <= cap; p++) {
        bool pr = true;
        for (int d = 2; d * d <= p; d++) if (p % d == 0) { pr = false; break; }
        if (!pr) continue;
        long v = p, best = p;
        while (v * p <= cap) { v *= p; best = v; }
        pp.push_back((int)best);
    }
    std::sort(pp.begin(), pp.end(), std::greater<int>());
    if ((int)pp.size() > n_mod) pp.resize((size_t)n_mod);
    return pp;
}

long mod_inverse(long a, long m) {
    long t = 0, nt = 1, r = m, nr = ((a % m) + m) % m;
    while (nr != 0) { const long qq = r / nr; long x = t - qq * nt; t = nt; nt = x; x = r - qq * nr; r = nr; nr = x; }
    return (t % m + m) % m;
}

/* gpu_memory.mm:2831-2857; 0, or -4 where the reference gives up */
int make_plan(uint64_t K, int n_mod, FastPlan* out, bool quiet = false) {
    FastPlan f;
    int cap = (int)floor(2.0 * sqrt(16777216.0 / (double)K));
    if (cap > 255) cap = 255;
    while (cap > 2 && (double)K * floor(cap / 2.0) * floor(cap / 2.0) >= 16777216.0) cap--;
    if (cap < 2) {
        if (!quiet) fprintf(stderr, "[GPU] Ozaki-II FAST: K=%llu too large for the tier's moduli; falling back\n", (unsigned long long)K);
        return -4;
    }
    if (n_mod > FAST_MAX_MODULI) n_mod = FAST_MAX_MODULI;
    if (n_mod < 2) n_mod = 2;
    const std::vector<int> mod = build_moduli(cap, n_mod);
    if (mod.size() < 2) {
        if (!quiet) fprintf(stderr, "[GPU] Ozaki-II FAST: too few coprime moduli <= cap %d; falling back\n", cap);
        return -4;
    }
    f.n = (int)mod.size(); f.cap = cap;
    unsigned __int128 P = 1;
    for (int p : mod) P *= (unsigned)p;
    for (int l = 0; l < f.n; l++) {
        const int p = mod[(size_t)l];
        f.moduli[l] = p;
        f.q[l] = (int)mod_inverse((long)((P / (unsigned)p) % (unsigned)p), p);
        f.log2P += log2((double)p);
        const ByteWeights w = byte_weights(p);
        f.table.p[l] = p; f.table.wlo[l] = w.lo; f.table.whi[l] = w.hi;
        f.table.pinv[l] = 1.0f / (float)p;
        f.table.neg_half[l] = (p % 2 == 0) ? (uint32_t)(256 - p / 2) & 0xffu : 0x100u;
        const unsigned __int128 d = (((unsigned __int128)(unsigned)f.q[l]) << 64) / (unsigned)p;   /* < 2^64: q < p */
        for (int j = 0; j < 4; j++) f.limbs.d[l][j] = (int32_t)((uint64_t)(d >> (16 * j)) & 0xffffu);
    }
    f.table.n = f.n;
    int E = (int)floor((f.log2P - log2((double)K) - 2.0) / 2.0);
    if (E > 52) E = 52;
    if (E < 1) E = 1;
    f.E = E;
    f.P = (double)P;
    *out = f;
    return 0;
}

/* Device-resident tables of the current moduli: identity pair lists and the
 * moduli for the contraction. */
int32_t* g_tables = nullptr;    /* [0..16] pair_first, [17..32] plane index, [33..48] moduli */
int g_tables_key[FAST_MAX_MODULI + 1] = {};

int ensure_tables(const FastPlan& f, hipStream_t st) {
    int key[FAST_MAX_MODULI + 1] = {};
    key[0] = f.n;
    for (int l = 0; l < f.n; l++) key[l + 1] = f.moduli[l];
    if (g_tables && memcmp(key, g_tables_key, sizeof key) == 0) return 0;
    if (!g_tables && !ESHKOL_HIP_OK(hipMalloc((void**)&g_tables, 49 * sizeof(int32_t)))) return -1;
    int32_t h[49] = {};
    for (int i = 0; i <= 16; i++) h[i] = i;
    for (int i = 0; i < 16; i++) h[17 + i] = i;
    for (int l = 0; l < f.n; l++) h[33 + l] = f.moduli[l];
    /* pageable source: the copy is complete when the calls return */
    if (!ESHKOL_HIP_OK(hipMemcpyAsync(g_tables, h, sizeof h, hipMemcpyHostToDevice, st)) ||
        !ESHKOL_HIP_OK(hipStreamSynchronize(st))) return -1;
    memcpy(g_tables_key, key, sizeof key);
    return 0;
}

HipOzakiFastStages g_last = {};

int split_any(const double* X, uint64_t rows, uint64_t K, const int32_t* shift, const FastTable& tbl,
              int8_t* planes, uint64_t rows_padded, uint64_t ldk, bool kmajor, int layout, hipStream_t st) {
    if (kmajor && layout == 1) {
        const uint64_t nblk = kmaj::il_blocks(rows_padded, ldk);
        if (nblk > 0x7fffffffULL) return -1;
        hipLaunchKernelGGL(fast_split_kmajor_il_kernel, dim3((unsigned)nblk), dim3(256), 0, st, X, rows, K, shift, tbl,
                           planes, rows_padded, ldk);
    } else if (kmajor) {
        if (kmaj::tile_count(rows_padded, ldk) > 0x7fffffffULL) return -1;
        const dim3 grid((unsigned)kmaj::grid_blocks(rows_padded, ldk, eshkol_hip_num_cus()));
        hipLaunchKernelGGL(fast_split_kmajor_kernel, grid, dim3(256), 0, st, X, rows, K, shift, tbl, planes,
                           rows_padded, ldk, layout);
    } else if (layout == 1) {
        const uint64_t nblk = (rows_padded / 32) * (ldk / 32);
        if (nblk > 0x7fffffffULL) return -1;
        hipLaunchKernelGGL(fast_split_il_kernel, dim3((unsigned)nblk), dim3(256), 0, st, X, rows, K, shift, tbl, planes,
                           rows_padded, ldk);
    } else {
        const uint64_t nblk = ((ldk + 1023) / 1024) * rows_padded;
        if (nblk > 0x7fffffffULL) return -1;
        hipLaunchKernelGGL(fast_split_kernel, dim3((unsigned)nblk), dim3(256), 0, st, X, rows, K, shift, tbl, planes,
                           rows_padded, ldk);
    }
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

}  // namespace

extern "C" int hip_ozaki_fast_plan(uint64_t K, int num_moduli, int32_t* E, int32_t* cap, int32_t* moduli) {
    if (K == 0 || K > 131071) return -4;
    FastPlan f;
    const int rc = make_plan(K, num_moduli, &f, true);
    if (rc != 0) return rc;
    if (E) *E = f.E;
    if (cap) *cap = f.cap;
    if (moduli) for (int l = 0; l < FAST_MAX_MODULI; l++) moduli[l] = (l < f.n) ? f.moduli[l] : 0;
    return f.n;
}

/* The tier's two streaming stages on their own (moduli and E from the plan for K). */
extern "C" int hip_ozaki_fast_split_planes_f64(const double* X, uint64_t rows, uint64_t K, const int32_t* shift,
                                               int num_moduli, int8_t* planes, uint64_t rows_padded, uint64_t ldk,
                                               int kmajor, int layout, void* stream) {
    if (!X || !shift || !planes || rows == 0 || K == 0 || K > 131071) return -1;
    if (rows_padded < rows || ldk < K || (ldk & 15) || ((uintptr_t)planes & 15)) return -1;
    if (layout != 0 && layout != 1) return -1;
    if (layout == 1 && ((rows_padded & 31) || (ldk & 31))) return -1;
    FastPlan f;
    if (make_plan(K, num_moduli, &f, true) != 0) return -1;
    return split_any(X, rows, K, shift, f.table, planes, rows_padded, ldk, kmajor != 0, layout, (hipStream_t)stream);
}

/* Reconstruction from product planes of wrows rows of ldw bytes each. */
static int fast_reconstruct(const int8_t* w_planes, uint64_t wrows, uint64_t ldw, uint64_t M, uint64_t N,
                            const FastPlan& f, const int32_t* shift_a, const int32_t* shift_b, double* C, hipStream_t st) {
    if (wrows < M || ldw < N) return -1;
    const uint64_t nblk = (((N + 3) / 4 + 255) / 256) * M;
    if (nblk > 0x7fffffffULL) return -1;
    const bool wvec = (ldw % 4 == 0) && ((wrows * ldw) % 4 == 0) && (((uintptr_t)w_planes & 3) == 0);
    const int vec = !wvec ? 0 : ((N % 4 == 0) && (((uintptr_t)C & 15) == 0)) ? 1 : 2;
    switch (f.n) {
#define LAUNCH(n, v) hipLaunchKernelGGL((fast_reconstruct_kernel<n, v>), dim3((unsigned)nblk), dim3(256), 0, st,  \
                                        w_planes, wrows, ldw, M, N, f.limbs, ldexp(f.P, -64), shift_a, shift_b, C)
#define CASE(n) case n:                                                                                          \
        if (vec == 1) LAUNCH(n, 1); else if (vec == 2) LAUNCH(n, 2); else LAUNCH(n, 0);                           \
        break;
        CASE(2) CASE(3) CASE(4) CASE(5) CASE(6) CASE(7) CASE(8) CASE(9)
        CASE(10) CASE(11) CASE(12) CASE(13) CASE(14) CASE(15) CASE(16)
#undef CASE
#undef LAUNCH
        default: return -1;
    }
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -3;
}

extern "C" int hip_ozaki_fast_reconstruct_f64(const int8_t* w_planes, uint64_t M, uint64_t N, uint64_t K, int num_moduli,
                                              const int32_t* shift_a, const int32_t* shift_b, double* C, void* stream) {
    if (!w_planes || !shift_a || !shift_b || !C || M == 0 || N == 0 || K == 0 || K > 131071) return -1;
    FastPlan f;
    if (make_plan(K, num_moduli, &f, true) != 0) return -1;
    return fast_reconstruct(w_planes, M, N, M, N, f, shift_a, shift_b, C, (hipStream_t)stream) == 0 ? 0 : -1;
}

void eshkol_hip_fast_release(void) {
    if (g_tables) { (void)hipFree(g_tables); g_tables = nullptr; }
    memset(g_tables_key, 0, sizeof g_tables_key);
    g_last = HipOzakiFastStages{};
}

extern "C" int hip_ozaki_fast_last_stages(HipOzakiFastStages* out) {
    EshkolHipLock lk;
    if (!out || !g_last.a_planes) return -1;
    *out = g_last;
    return 0;
}

extern "C" int hip_matmul_ozaki_fast_f64_ex(const double* A, const double* B, double* C,
                                            uint64_t M, uint64_t K, uint64_t N,
                                            int trans_a, int trans_b, int num_moduli, void* stream) {
    EshkolHipCall bracket(stream);
    if (!A || !B || !C || M == 0 || K == 0 || N == 0) return -1;
    if (M > 0x7fffffffULL || N > 0x7fffffffULL) return -1;
    if (K > 131071) return -4;          /* the contraction's int32 bound; the reference's f32 bound is 2^24 / (p/2)^2 */
    FastPlan f;
    const int prc = make_plan(K, num_moduli, &f);
    if (prc != 0) return prc;
    hipStream_t st = (hipStream_t)stream;
    if (ensure_tables(f, st) != 0) return -1;
    if (!eshkol_crt_quiet()) fprintf(stderr, "[GPU] Ozaki-II FAST: n_mod=%d E=%d cap=%d log2(P)=%.1f (int8 MFMA GEMMs)\n",
            f.n, f.E, f.cap, f.log2P);                                  /* gpu_memory.mm:2859 */

    const int layout = hip_igemm_plane_layout_single(M, K, N, f.n);
    const uint64_t Mp = round_up_sz(M, 256), Np = round_up_sz(N, 256), ldk = round_up_sz(K, layout ? 512 : 256);
    const bool a_kmajor = trans_a != 0, b_kmajor = trans_b == 0;
    double* amax = (double*)eshkol_hip_workspace(WS_ROWSCALE, M * sizeof(double));
    double* bmax = (double*)eshkol_hip_workspace(WS_COLSCALE, N * sizeof(double));
    int32_t* sha = (int32_t*)eshkol_hip_workspace(WS_ROWSHIFT, M * sizeof(int32_t));
    int32_t* shb = (int32_t*)eshkol_hip_workspace(WS_COLSHIFT, N * sizeof(int32_t));
    int8_t* Ap = (int8_t*)eshkol_hip_workspace(WS_APLANES, (size_t)f.n * Mp * ldk);
    int8_t* Bp = (int8_t*)eshkol_hip_workspace(WS_BPLANES, (size_t)f.n * Np * ldk);
    const uint64_t Mw = eshkol_product_rows(M), Nw = eshkol_product_pitch(N);
    int8_t* Wp = (int8_t*)eshkol_hip_workspace(WS_PRODUCTS, (size_t)f.n * Mw * Nw);
    if (!amax || !bmax || !sha || !shb || !Ap || !Bp || !Wp) return -2;

    /* frexp exponent e = floor(log2 max) + 1 (gpu_memory.mm:2886-2905); the split
     * scales by 2^(E - e), so the per-row shift is (E - 1) - floor(log2 max): the
     * kernels that find the maxima write it beside them. Nothing the host computes
     * depends on the operands, so the whole pipeline is queued at once; the scan of
     * the maxima (non-finite input?) runs beside it and is read at the end. */
    if ((a_kmajor ? eshkol_colabsmax_shift_f64(A, K, M, 0.0, amax, sha, f.E - 1, st)
                  : eshkol_rowabsmax_shift_f64(A, M, K, 0.0, amax, sha, f.E - 1, st)) != 0) return -1;
    /* the last kernel that writes maxima carries the event the scan's stream waits for */
    const hipEvent_t fork = eshkol_crt_scan_event(M * K + K * N);
    if ((b_kmajor ? eshkol_colabsmax_shift_f64(B, K, N, 0.0, bmax, shb, f.E - 1, st, fork)
                  : eshkol_rowabsmax_shift_f64(B, N, K, 0.0, bmax, shb, f.E - 1, st, fork)) != 0) return -1;
    const uint32_t ticket = eshkol_crt_scan_launch_aside(amax, M, bmax, N, st, M * K + K * N, fork != nullptr);
    if (!ticket) return -1;

    if (split_any(A, M, K, sha, f.table, Ap, Mp, ldk, a_kmajor, layout, st) != 0) return -1;
    if (split_any(B, N, K, shb, f.table, Bp, Np, ldk, b_kmajor, layout, st) != 0) return -1;

    HipIgemmArgs ga;
    memset(&ga, 0, sizeof ga);
    ga.a_planes = Ap; ga.b_planes = Bp;
    ga.a_plane_stride = Mp * ldk; ga.b_plane_stride = Np * ldk;
    ga.ldk = (uint32_t)ldk; ga.M = (uint32_t)M; ga.N = (uint32_t)N; ga.n_out = (uint32_t)f.n;
    ga.pair_first = g_tables; ga.pair_a = g_tables + 17; ga.pair_b = g_tables + 17;
    ga.mode = 1; ga.max_pairs = 1; ga.modulus = g_tables + 33; ga.out_i8 = Wp;
    ga.layout = layout;
    ga.out_rows = (uint32_t)Mw; ga.ldn = (uint32_t)Nw;
    if (hip_igemm_i8(&ga, st) != 0) return -1;

    { const int rc = fast_reconstruct(Wp, Mw, Nw, M, N, f, sha, shb, C, st); if (rc != 0) return rc; }
    CrtMaxima mx[2];
    if (eshkol_crt_scan_result(ticket, mx, st) != 0) return -1;
    if (mx[0].nonfinite || mx[1].nonfinite) return -1;                  /* NaN / Inf: not this tier's business; C holds no result */

    g_last.a_planes = Ap; g_last.b_planes = Bp; g_last.w_planes = Wp;
    g_last.w_rows = Mw; g_last.w_ld = Nw;
    g_last.shift_a = sha; g_last.shift_b = shb;
    g_last.rows_a_padded = Mp; g_last.rows_b_padded = Np; g_last.ldk = ldk;
    g_last.num_moduli = f.n; g_last.E = f.E; g_last.cap = f.cap; g_last.layout = layout;
    for (int l = 0; l < FAST_MAX_MODULI; l++) g_last.moduli[l] = (l < f.n) ? f.moduli[l] : 0;
    return 0;
}

extern "C" int hip_matmul_ozaki_fast_f64(const double* A, const double* B, double* C,
                                         uint64_t M, uint64_t K, uint64_t N, int num_moduli, void* stream) {
    return hip_matmul_ozaki_fast_f64_ex(A, B, C, M, K, N, 0, 0, num_moduli, stream);
}
