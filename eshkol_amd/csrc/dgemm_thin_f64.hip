/*
 * fp64 products with one thin side: up to sixty-four rows (or columns) against a big
 * operand, C[M][N] = A[M][K] B[K][N] with M small: a batch of activation rows in front
 * of a layer, a vector against a matrix, a matrix against a few columns. Behind the same
 * entry points as the tiled GEMM (hip_dgemm_f64 / hip_dgemm_f64_ex), which replace
 * cublasDgemm (lib/backend/gpu/gpu_memory_cuda.cpp:611-650) for every shape.
 *
 * Such a product is bound by reading the big operand once. The tiled kernels pad the thin
 * side to a 64- or 128-row tile and have few tiles to hand out (1 ... 2 TB/s); fma loops
 * on the vector ALU, whose fp64 rate equals the matrix cores' on this chip, keep up with
 * HBM for a handful of rows only (32 rows: 1.9 TB/s) and lose to the kernel below even at
 * one row (the thin operand's values as scalar loads, a lane per two columns: 33 us
 * against 27 for 1 x 4096 x 4096). Here the matrix cores multiply
 * (v_mfma_f64_16x16x4_f64: rows that do not exist cost nothing while the stream is the
 * bound) and nothing is staged:
 *
 *   - a workgroup takes a strip of 64 output columns and a slice of k; its four waves
 *     deal the slice out sixteen k at a time. With the output index contiguous in the big
 *     operand (G[k][o]) a lane loads four consecutive columns of one row of k (32 bytes;
 *     the sixteen lanes of a row 512 contiguous bytes) and feeds them to four matrix-core
 *     instructions per block of 16 rows: column j of instruction c is column 4 j + c of
 *     the strip, so a lane ends up with four consecutive columns of its rows and stores
 *     them as one vector. With k contiguous (G[o][k]) see the second kernel;
 *   - the thin operand's fragments (16 rows x 4 k, a double per lane) come from the L2,
 *     addressed by strides, so every operand form is served;
 *   - a wave loads sixteen k, multiplies them, loads the next: the other waves of its SIMD
 *     (two to five, by the row count) multiply meanwhile;
 *   - the four waves' sums meet in LDS; slices of k (when the strips alone do not fill
 *     the device) leave partial results that a second kernel adds in ascending order.
 *
 * Sums are taken in a fixed order: the same call gives the same bits every time. The order
 * differs from the tiled kernel's; the tolerance of the fp64 tier (1e-14 normwise) covers
 * both. One vector against a matrix with k contiguous stays on the vector ALU
 * (dgemv_f64.hip: 24 us against 28 for 4096 x 4096).
 */
#include "hip_common.h"
#include "kernels.h"
#include <type_traits>

typedef double v4d_t __attribute__((ext_vector_type(4)));
typedef double d4u_t __attribute__((ext_vector_type(4), aligned(8)));

namespace {

template <int RB>
__global__ __launch_bounds__(256)
void dgemm_thin_rows_kernel(const double* __restrict__ T, long t_r, long t_k, int R,
                            const double* __restrict__ G, long ldg, int K, int O, int kc,
                            double* __restrict__ out, long c_r, long c_o, long slice_stride) {
    __shared__ double red[4][16][64];
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 15, lg = lane >> 4;
    const int o = (int)blockIdx.x * 64 + 4 * li;
    const int ks = (int)blockIdx.y * kc;
    const int ke = (ks + kc < K) ? ks + kc : K;
    const bool cols_in = o + 3 < O;
    /* more than 64 thin rows: a chunk of 64 per blockIdx.z */
    T += (long)blockIdx.z * 64 * t_r;
    out += (long)blockIdx.z * 64 * c_r;
    R = (R - 64 * (int)blockIdx.z < 64) ? R - 64 * (int)blockIdx.z : 64;
    v4d_t acc[RB][4];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int c = 0; c < 4; c++) acc[rb][c] = (v4d_t){0.0, 0.0, 0.0, 0.0};

    /* Loads carry no branches. Rows of the thin operand beyond R are read from row R - 1
     * (their sums are never stored); an edge strip reads its columns one by one from
     * clamped addresses; the last, partial round of k reads from clamped rows and
     * replaces what lies beyond the slice with zeros on both sides (a zero on one side
     * only would turn an infinity on the other into a NaN). */
    long t_off[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        const int r = 16 * rb + li;
        t_off[rb] = (long)(r < R ? r : R - 1) * t_r;
    }
    int oc[4];
#pragma unroll
    for (int c = 0; c < 4; c++) oc[c] = (o + c < O) ? o + c : O - 1;
    const bool edge = (int)blockIdx.x * 64 + 64 > O;              /* the same for the whole workgroup */

    v4d_t g[4];
    double a[RB][4];
    auto fetch = [&](int kb, v4d_t (&gd)[4], double (&ad)[RB][4], auto is_edge, auto is_tail) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int k = kb + 4 * u + lg;
            const bool in = !decltype(is_tail)::value || k < ke;
            const int kr = in ? k : ke - 1;
            const double* p = G + (size_t)kr * ldg;
            v4d_t v;
            if (decltype(is_edge)::value) {
#pragma unroll
                for (int c = 0; c < 4; c++) v[c] = p[oc[c]];
            } else {
                v = *(const d4u_t*)(p + o);
            }
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                const double t = T[t_off[rb] + (long)kr * t_k];
                ad[rb][u] = in ? t : 0.0;
            }
            if (decltype(is_tail)::value) {
#pragma unroll
                for (int c = 0; c < 4; c++) v[c] = in ? v[c] : 0.0;
            }
            gd[u] = v;
        }
    };
    auto fetch_any = [&](int kb, v4d_t (&gd)[4], double (&ad)[RB][4]) {
        const bool tail = kb + 16 > ke;                            /* the same for the whole wave */
        if (edge) { if (tail) fetch(kb, gd, ad, std::true_type{}, std::true_type{}); else fetch(kb, gd, ad, std::true_type{}, std::false_type{}); }
        else      { if (tail) fetch(kb, gd, ad, std::false_type{}, std::true_type{}); else fetch(kb, gd, ad, std::false_type{}, std::false_type{}); }
    };
    for (int k0 = ks + 16 * wave; k0 < ke; k0 += 64) {
        fetch_any(k0, g, a);
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int rb = 0; rb < RB; rb++)
#pragma unroll
                for (int c = 0; c < 4; c++)
                    acc[rb][c] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[rb][u], g[u][c], acc[rb][c], 0, 0, 0);
    }
    /* acc[rb][c][r]: row 16 rb + 4 r + lane/16, column o + c. One block of 16 rows at a time
     * through LDS; thread (wave w, lane) then sums row 16 rb + 4 w + lane/16, columns o .. o + 3. */
    double* dst0 = out + (size_t)blockIdx.y * slice_stride;
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        if (rb) __syncthreads();
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int r = 0; r < 4; r++) red[wave][4 * c + r][lane] = acc[rb][c][r];
        __syncthreads();
        const int row = 16 * rb + 4 * wave + lg;
        if (row >= R) continue;                                  /* the barriers sit above */
        v4d_t s;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            double t = red[0][4 * c + wave][lane];
#pragma unroll
            for (int w = 1; w < 4; w++) t += red[w][4 * c + wave][lane];
            s[c] = t;
        }
        double* dst = dst0 + (long)row * c_r + (long)o * c_o;
        if (cols_in && c_o == 1) *(d4u_t*)dst = s;
        else {
#pragma unroll
            for (int c = 0; c < 4; c++) if (o + c < O) dst[(long)c * c_o] = s[c];
        }
    }
}

/* The same against a big operand with k contiguous, G[o][k] (a layer's weights held
 * transposed, or a matrix against a few columns): a lane loads four consecutive k of one
 * output column (the sixteen lanes of a k-quarter sixteen rows, 128 bytes each); element c
 * of the load goes to instruction c, whose k index then stands for k0 + 4 (lane/16) + c on
 * both sides. A workgroup's strip is four blocks of 16 output columns. TVEC: the thin
 * operand has k contiguous as well and is loaded the same way. */
template <int RB, bool TVEC>
__global__ __launch_bounds__(256)
void dgemm_thin_rows_klast_kernel(const double* __restrict__ T, long t_r, long t_k, int R,
                                  const double* __restrict__ G, long ldg, int K, int O, int kc,
                                  double* __restrict__ out, long c_r, long c_o, long slice_stride) {
    __shared__ double red[4][16][64];
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 15, lg = lane >> 4;
    const int ob = (int)blockIdx.x * 64;
    const int ks = (int)blockIdx.y * kc;
    const int ke = (ks + kc < K) ? ks + kc : K;
    T += (long)blockIdx.z * 64 * t_r;
    out += (long)blockIdx.z * 64 * c_r;
    R = (R - 64 * (int)blockIdx.z < 64) ? R - 64 * (int)blockIdx.z : 64;
    v4d_t acc[RB][4];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int cb = 0; cb < 4; cb++) acc[rb][cb] = (v4d_t){0.0, 0.0, 0.0, 0.0};
    /* rows beyond the operands are read from the last row: their sums are never stored */
    long g_off[4], t_off[RB];
#pragma unroll
    for (int cb = 0; cb < 4; cb++) {
        const int oo = ob + 16 * cb + li;
        g_off[cb] = (long)(oo < O ? oo : O - 1) * ldg;
    }
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        const int r = 16 * rb + li;
        t_off[rb] = (long)(r < R ? r : R - 1) * t_r;
    }
    for (int k0 = ks + 16 * wave; k0 < ke; k0 += 64) {
        const int kk = k0 + 4 * lg;
        v4d_t v[4], t[RB];
        if (k0 + 16 <= ke) {                                      /* the same for the whole wave */
#pragma unroll
            for (int cb = 0; cb < 4; cb++) v[cb] = *(const d4u_t*)(G + g_off[cb] + kk);
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                if (TVEC) t[rb] = *(const d4u_t*)(T + t_off[rb] + kk);
                else {
#pragma unroll
                    for (int c = 0; c < 4; c++) t[rb][c] = T[t_off[rb] + (long)(kk + c) * t_k];
                }
            }
        } else {
            /* the slice's last, partial round: clamped addresses, zeros on both sides beyond it */
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const bool in = kk + c < ke;
                const int kr = in ? kk + c : ke - 1;
#pragma unroll
                for (int cb = 0; cb < 4; cb++) { const double x = G[g_off[cb] + kr]; v[cb][c] = in ? x : 0.0; }
#pragma unroll
                for (int rb = 0; rb < RB; rb++) { const double x = T[t_off[rb] + (long)kr * t_k]; t[rb][c] = in ? x : 0.0; }
            }
        }
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int rb = 0; rb < RB; rb++)
#pragma unroll
                for (int cb = 0; cb < 4; cb++)
                    acc[rb][cb] = __builtin_amdgcn_mfma_f64_16x16x4f64(t[rb][c], v[cb][c], acc[rb][cb], 0, 0, 0);
    }
    /* acc[rb][cb][r]: row 16 rb + 4 r + lane/16, column ob + 16 cb + lane%16 */
    double* dst0 = out + (size_t)blockIdx.y * slice_stride;
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        if (rb) __syncthreads();
#pragma unroll
        for (int cb = 0; cb < 4; cb++)
#pragma unroll
            for (int r = 0; r < 4; r++) red[wave][4 * cb + r][lane] = acc[rb][cb][r];
        __syncthreads();
        const int row = 16 * rb + 4 * wave + lg;
        if (row >= R) continue;                                  /* the barriers sit above */
#pragma unroll
        for (int cb = 0; cb < 4; cb++) {
            double s = red[0][4 * cb + wave][lane];
#pragma unroll
            for (int w = 1; w < 4; w++) s += red[w][4 * cb + wave][lane];
            const int col = ob + 16 * cb + li;
            if (col < O) dst0[(long)row * c_r + (long)col * c_o] = s;
        }
    }
}

/* C(r, o) = the slices' partial results added in ascending order */
__global__ __launch_bounds__(256)
void dgemm_thin_rows_sum_kernel(const double* __restrict__ part, int slices, int R, int O,
                                double* __restrict__ C, long c_r, long c_o) {
    const long n = (long)R * O;
    const long e = (long)blockIdx.x * 256 + threadIdx.x;
    if (e >= n) return;
    /* eight loads in flight, added in ascending order all the same */
    double s = 0.0;
    int y = 0;
    for (; y + 8 <= slices; y += 8) {
        double v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = part[(size_t)(y + u) * n + e];
#pragma unroll
        for (int u = 0; u < 8; u++) s += v[u];
    }
    for (; y < slices; y++) s += part[(size_t)y * n + e];
    const long r = e / O, o = e - r * O;
    C[r * c_r + o * c_o] = s;
}

template <int RB>
void launch_rows(bool klast, const double* T, long t_r, long t_k, int R, const double* G, long ldg, int K, int O, int kc,
                 int slices, double* out, long c_r, long c_o, long slice_stride, hipStream_t st) {
    const dim3 grid((unsigned)((O + 63) / 64), (unsigned)slices, (unsigned)((R + 63) / 64));
    if (!klast)
        hipLaunchKernelGGL(dgemm_thin_rows_kernel<RB>, grid, dim3(256), 0, st,
                           T, t_r, t_k, R, G, ldg, K, O, kc, out, c_r, c_o, slice_stride);
    else if (t_k == 1)
        hipLaunchKernelGGL((dgemm_thin_rows_klast_kernel<RB, true>), grid, dim3(256), 0, st,
                           T, t_r, t_k, R, G, ldg, K, O, kc, out, c_r, c_o, slice_stride);
    else
        hipLaunchKernelGGL((dgemm_thin_rows_klast_kernel<RB, false>), grid, dim3(256), 0, st,
                           T, t_r, t_k, R, G, ldg, K, O, kc, out, c_r, c_o, slice_stride);
}

int g_thin_rows = 1;        /* fewest rows sent here; 0: none (tuning) */
int g_thin_rows_klast = 1;
constexpr int THIN_MIN_WIDE = 16;      /* narrowest big operand */
int g_thin_chunks = 1;       /* 0: no more than 64 thin rows (tuning) */
constexpr int THIN_MIN_LOG2 = 13;      /* smallest big operand, log2 of its elements */

}  // namespace

extern "C" void hip_dgemm_set_thin_rows(int from) { EshkolHipLock lk; g_thin_rows = from > 0 ? from : 0; }
extern "C" void hip_dgemm_set_thin_chunks(int on) { EshkolHipLock lk; g_thin_chunks = on ? 1 : 0; }
extern "C" void hip_dgemm_set_thin_rows_klast(int on) { EshkolHipLock lk; g_thin_rows_klast = on ? 1 : 0; }

/* Up to 64 rows on the thin side. The other side may be narrow too where k is long
 * (32 x 4109 x 36: 34 us on the tiled kernels, which have one tile to cut along k, 10
 * here); what the tiled kernels keep is the widest thin sides on a short k
 * (64 x 300 x 4000: 17 us here, 13 there) and operands of a few thousand elements. One
 * vector against a matrix with k contiguous is left to dgemv_f64.hip. */
bool eshkol_hip_dgemm_is_thin_rows(uint64_t M, uint64_t K, uint64_t N, int trans_a, int trans_b) {
    if (!g_thin_rows) return false;
    const bool thin_m = M <= N;
    const uint64_t thin = thin_m ? M : N, wide = thin_m ? N : M;
    const bool kfirst = thin_m ? !trans_b : (trans_a != 0);
    if (!kfirst && (!g_thin_rows_klast || thin < 2)) return false;
    if (thin < (uint64_t)g_thin_rows || wide < (uint64_t)THIN_MIN_WIDE || K < 64) return false;
    if (thin > 48 && K < 512) return false;
    if (thin > 64) {
        /* chunks of 64 rows, each reading the big operand again: where the tiled kernels would
         * have a few dozen tiles and a long k to walk, and the big operand stays in the caches
         * (135 x 2559 x 349: 50 -> 23 us, 70 x 32768 x 128: 71 -> 38; 250 x 4096 x 700 would
         * go from 43 to 54) */
        if (!g_thin_chunks || thin > 256 || K < 1024) return false;
        const uint64_t blocks = ((thin + 63) / 64) * ((wide + 63) / 64);
        if (blocks > 48 || (wide * K > (2ull << 20) && blocks > 8)) return false;
    }
    if (K > 0x7fffff00ULL || wide > 0x7fffff00ULL) return false;      /* strip and round indices are ints */
    return wide * K >= (1ull << THIN_MIN_LOG2);
}

int eshkol_hip_dgemm_thin_rows(const double* A, const double* B, double* C, uint64_t M, uint64_t K, uint64_t N,
                               int trans_a, int trans_b, hipStream_t st) {
    const bool thin_m = M <= N;
    const int R = (int)(thin_m ? M : N), O = (int)(thin_m ? N : M), k = (int)K;
    const double* G = thin_m ? B : A;
    const double* T = thin_m ? A : B;
    long t_r, t_k, c_r, c_o;
    if (thin_m) { t_r = trans_a ? 1 : (long)K; t_k = trans_a ? (long)M : 1; c_r = (long)N; c_o = 1; }
    else        { t_r = trans_b ? (long)K : 1; t_k = trans_b ? 1 : (long)N; c_r = 1; c_o = (long)N; }
    const bool klast = !(thin_m ? !trans_b : (trans_a != 0));
    const long ldg = klast ? (long)K : (long)O;
    /* slices of k where the strips alone leave CUs idle: about three workgroups per CU,
     * at least four rounds of 64 k per workgroup */
    const int strips = (O + 63) / 64;
    const int chunks = (R + 63) / 64;
    int slices = (3 * eshkol_hip_num_cus()) / (strips * chunks);
    /* a slice of at least 256 k, shorter where the strips are few or k is short (more slices
     * are all the parallelism such a launch has) */
    const int min_kc = strips <= 2 ? 64 : (strips <= 4 || k < 2048) ? 128 : 256;
    if (slices > k / min_kc) slices = k / min_kc;
    if (slices > 128) slices = 128;                 /* the sum walks them one thread per output */
    if (slices < 1) slices = 1;
    int kc = (k + slices - 1) / slices;
    kc = (kc + 63) / 64 * 64;
    slices = (k + kc - 1) / kc;
    double* out = C;
    long o_r = c_r, o_o = c_o, slice_stride = 0;
    if (slices > 1) {
        out = (double*)eshkol_hip_workspace(WS_DGEMM_PARTIAL, (size_t)slices * R * O * sizeof(double));
        if (!out) return -1;
        o_r = O; o_o = 1; slice_stride = (long)R * O;
    }
    switch ((R + 15) / 16) {
        case 1: launch_rows<1>(klast, T, t_r, t_k, R, G, ldg, k, O, kc, slices, out, o_r, o_o, slice_stride, st); break;
        case 2: launch_rows<2>(klast, T, t_r, t_k, R, G, ldg, k, O, kc, slices, out, o_r, o_o, slice_stride, st); break;
        case 3: launch_rows<3>(klast, T, t_r, t_k, R, G, ldg, k, O, kc, slices, out, o_r, o_o, slice_stride, st); break;
        default: launch_rows<4>(klast, T, t_r, t_k, R, G, ldg, k, O, kc, slices, out, o_r, o_o, slice_stride, st); break;
    }
    if (slices > 1)
        hipLaunchKernelGGL(dgemm_thin_rows_sum_kernel, dim3((unsigned)(((long)R * O + 255) / 256)), dim3(256), 0, st,
                           out, slices, R, O, C, c_r, c_o);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}
