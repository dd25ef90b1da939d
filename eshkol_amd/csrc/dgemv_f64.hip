/*
 * fp64 products with one thin side: C[M x N] = A[M x K] * B[K x N] where M or N is
 * small (a vector or a handful of vectors against a matrix: up to 8, or up to 32 where
 * the big operand has the output index contiguous). Behind the same
 * entry points as the matrix-core GEMM (hip_dgemm_f64 / hip_dgemm_f64_ex), which
 * replace cublasDgemm (lib/backend/gpu/gpu_memory_cuda.cpp:611-650) for every shape.
 *
 * Such a product reads its big operand once and does almost no arithmetic per byte:
 * it is bound by HBM, and a 64 x 64 or 128 x 128 tile wastes the matrix cores on
 * rows that do not exist (1 x 8192 x 8192: 0.42 ms through the tiled kernel, 0.11 ms
 * at what HBM delivers). On this chip the vector ALU's fp64 fma rate equals the
 * matrix cores', so plain fma loops lose nothing. Two kernels, by how the big
 * operand lies in memory; the thin one and the result are addressed by strides, so
 * that transposed operands need no third:
 *
 *   big[K][O], the output index contiguous (B as given with M thin; A held transposed
 *   with N thin). A lane owns two adjacent outputs o and reads 16 bytes of every row k;
 *   the thin operand's value for (s, k) is the same for the whole wave: a scalar load.
 *   The four waves of a workgroup take groups of four k of the workgroup's k-range in
 *   turn and add up through LDS; workgroups split K further where O alone cannot fill the
 *   device, each leaving a partial result that a second kernel adds in a fixed order.
 *
 *   big[O][K], k contiguous (A as given with N thin; B held transposed with M thin). A
 *   workgroup owns R rows o; lanes run along k, 16 bytes of each row per step, the four
 *   waves a quarter of K each. A lane multiplies its two k of every row by the thin
 *   operand's values at those k (read through L2: the thin operand is small) and the
 *   partial sums meet across lanes and waves at the end.
 *
 * Sums are taken in a fixed order: the same call gives the same bits every time. The
 * order differs from the tiled kernel's; the tolerance of the fp64 tier (1e-14
 * normwise) covers both.
 */
#include "hip_common.h"
#include "kernels.h"

typedef double d2u_t __attribute__((ext_vector_type(2), aligned(8)));

namespace {

constexpr int COLS_PER_WG = 128;     /* kfirst: two per lane */

/* big[K][O] (pitch ldb), thin(s, k) = thin[s * ts + k * tk], s < S.
 * out(s, o): C[s * cs + o * co] when gridDim.y == 1, else part[(y * S + s) * O + o].
 * CONTIG says what the launcher knows about the thin operand's strides, so that the
 * scalar loads of a group of four k can be merged: 1: tk == 1 (four consecutive k of
 * one s are 32 contiguous bytes), 2: ts == 1 and tk == S (dense [K][S]: the values of
 * one k are contiguous, and reading SP of them where S exist stays inside the buffer
 * except behind its last row), 0: nothing. */
template <int SP, int CONTIG>
__global__ __launch_bounds__(256)
void skinny_kfirst_kernel(const double* __restrict__ big, long ldb, int K, int O,
                          const double* __restrict__ thin, long ts, long tk, int S,
                          double* __restrict__ C, long cs, long co, double* __restrict__ part, int kchunk) {
    constexpr int RB = SP < 16 ? SP : 16;
    __shared__ double red[3][RB][COLS_PER_WG];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int o = (int)blockIdx.x * COLS_PER_WG + 2 * lane;
    const int k_lo = (int)blockIdx.y * kchunk;
    const int k_hi = (k_lo + kchunk < K) ? k_lo + kchunk : K;
    const bool two = o + 1 < O, one = o < O;
    /* lanes beyond the matrix read the last pair of the row: valid memory, results dropped */
    const int oc = two ? o : (O >= 2 ? O - 2 : 0);
    const double* bp = big + oc;

    double acc0[SP], acc1[SP];
#pragma unroll
    for (int s = 0; s < SP; s++) { acc0[s] = 0.0; acc1[s] = 0.0; }

    /* groups of four consecutive k, dealt to the four waves in turn: four rows of the big
     * operand in flight per wave */
    /* CONTIG 2 reads SP values where a row of the thin operand holds S: beyond its last row
     * that would leave the buffer, so the group that holds row K - 1 takes the loop below */
    const int k_vec_hi = (CONTIG == 2 && S < SP && k_hi > K - 1) ? K - 1 : k_hi;
    int k = k_lo + 4 * wave;
    for (; k + 3 < k_vec_hi; k += 16) {
        double b0[4], b1[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if (O >= 2) { const d2u_t v = *(const d2u_t*)(bp + (long)(k + i) * ldb); b0[i] = v.x; b1[i] = v.y; }
            else { b0[i] = big[(long)(k + i) * ldb]; b1[i] = 0.0; }
        }
        /* the thin operand's values are the same for every lane: scalar loads, eight s at a
         * time (more than 64 scalar registers of them at once and the compiler spills) */
        constexpr int SB = SP < 8 ? SP : 8;
#pragma unroll
        for (int s0 = 0; s0 < SP; s0 += SB) {
            double a[SB][4];
            if (CONTIG == 1) {
#pragma unroll
                for (int s = 0; s < SB; s++) {
                    const double* t = thin + (long)(s0 + s < S ? s0 + s : 0) * ts + k;
#pragma unroll
                    for (int i = 0; i < 4; i++) a[s][i] = (s0 + s < S) ? t[i] : 0.0;
                }
            } else if (CONTIG == 2) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const double* t = thin + (long)(k + i) * tk + s0;
#pragma unroll
                    for (int s = 0; s < SB; s++) a[s][i] = t[s];
                }
            } else {
#pragma unroll
                for (int s = 0; s < SB; s++)
#pragma unroll
                    for (int i = 0; i < 4; i++) a[s][i] = (s0 + s < S) ? thin[(long)(s0 + s) * ts + (long)(k + i) * tk] : 0.0;
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int s = 0; s < SB; s++) {
                    acc0[s0 + s] = fma(a[s][i], b0[i], acc0[s0 + s]);
                    acc1[s0 + s] = fma(a[s][i], b1[i], acc1[s0 + s]);
                }
            if (SP > SB) __builtin_amdgcn_sched_barrier(0);
        }
    }
    /* what is left of a k-range that is not a multiple of four: its owner is the wave whose turn it is */
    if (k < k_hi) {
        for (; k < k_hi; k++) {
            double b0, b1;
            if (O >= 2) { const d2u_t v = *(const d2u_t*)(bp + (long)k * ldb); b0 = v.x; b1 = v.y; }
            else { b0 = big[(long)k * ldb]; b1 = 0.0; }
#pragma unroll
            for (int s = 0; s < SP; s++) {
                const double a = (s < S) ? thin[(long)s * ts + (long)k * tk] : 0.0;
                acc0[s] = fma(a, b0, acc0[s]);
                acc1[s] = fma(a, b1, acc1[s]);
            }
        }
    }
    /* a lane clamped to the last pair holds that pair's sums: only o == O - 1 of an odd O
     * is a real output among them, and it is the pair's second value */
    const bool shifted = !two && O >= 2;          /* this lane's o is O - 1, held as the second value of the clamped pair */
#pragma unroll
    for (int s0 = 0; s0 < SP; s0 += RB) {         /* through LDS, at most sixteen s at a time */
        if (s0 > 0) __syncthreads();
        if (wave > 0) {
#pragma unroll
            for (int s = 0; s < RB; s++) { red[wave - 1][s][2 * lane] = acc0[s0 + s]; red[wave - 1][s][2 * lane + 1] = acc1[s0 + s]; }
        }
        __syncthreads();
        if (wave == 0 && one) {
#pragma unroll
            for (int s = 0; s < RB; s++) {
                if (s0 + s >= S) break;
                double r0 = acc0[s0 + s], r1 = acc1[s0 + s];
#pragma unroll
                for (int w = 0; w < 3; w++) { r0 += red[w][s][2 * lane]; r1 += red[w][s][2 * lane + 1]; }
                if (shifted) r0 = r1;
                if (gridDim.y == 1) {
                    C[(long)(s0 + s) * cs + (long)o * co] = r0;
                    if (two) C[(long)(s0 + s) * cs + (long)(o + 1) * co] = r1;
                } else {
                    double* p = part + ((size_t)blockIdx.y * S + s0 + s) * (size_t)O + o;
                    p[0] = r0;
                    if (two) p[1] = r1;
                }
            }
        }
    }
}

/* dst[k][s] = src[s * ts + k]: the thin operand from rows of k to dense [K][S] */
__global__ __launch_bounds__(256)
void skinny_thin_to_dense_kernel(const double* __restrict__ src, long ts, int S, int K, double* __restrict__ dst) {
    const int k = (int)(blockIdx.x * 256 + threadIdx.x);
    if (k >= K) return;
    for (int s = 0; s < S; s++) dst[(size_t)k * S + s] = src[(long)s * ts + k];
}

/* C(s, o) = sum over pieces y of part[(y * S + s) * O + o], y ascending */
__global__ __launch_bounds__(256)
void skinny_fixup_kernel(const double* __restrict__ part, int pieces, int S, int O,
                         double* __restrict__ C, long cs, long co) {
    const int o = (int)(blockIdx.x * 256 + threadIdx.x), s = (int)blockIdx.y;
    if (o >= O) return;
    double r = 0.0;
    for (int y = 0; y < pieces; y++) r += part[((size_t)y * S + s) * (size_t)O + o];
    C[(long)s * cs + (long)o * co] = r;
}

/* big[O][K] (pitch ldb), C(o, s) = C[o * co + s * cs]; a workgroup owns rows R * blockIdx.x
 * .. + R - 1. The thin operand in one of the two forms it can have here, so that a lane's
 * values for its two k come as 16-byte loads:
 *   DENSE false: thin(k, s) = thin[s * ts + k], k contiguous (the operand held with k
 *     along its rows): the two k of one s are one 16-byte word, lanes side by side;
 *     SP is S rounded up to a power of two, rows beyond S repeat row 0 and are dropped.
 *   DENSE true: thin is [K][SP] with SP == S exactly: the lane's 2 x S values are 16 S
 *     contiguous bytes, S loads, each lane in a cache line of its own that the S loads
 *     use up between them. (Read value by value, 2 S loads of 8 bytes that touch 64
 *     lines each, the loads and not HBM set the pace from S = 5 on: 0.40 ms for
 *     8192 x 8192 x 8 against 0.11.) */
template <int SP, int R, bool DENSE>
__global__ __launch_bounds__(256)
void skinny_klast_kernel(const double* __restrict__ big, long ldb, int O, int K,
                         const double* __restrict__ thin, long ts, int S,
                         double* __restrict__ C, long co, long cs) {
    __shared__ double red[4][R][SP];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int o0 = (int)blockIdx.x * R;
    const double* rows[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int o = (o0 + r < O) ? o0 + r : O - 1;          /* rows beyond the matrix repeat the last one */
        rows[r] = big + (long)o * ldb;
    }
    double acc[R][SP];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int s = 0; s < SP; s++) acc[r][s] = 0.0;

    /* blocks of 128 k (two per lane), dealt to the four waves in turn */
    for (int kb = wave * 128; kb + 1 < K; kb += 512) {
        const int k = kb + 2 * lane;
        if (k + 1 < K) {
            double t0[SP], t1[SP];
            if (DENSE) {
                double tv[2 * SP];
#pragma unroll
                for (int j = 0; j < SP; j++) {
                    const d2u_t t = *(const d2u_t*)(thin + (long)k * SP + 2 * j);
                    tv[2 * j] = t.x; tv[2 * j + 1] = t.y;
                }
#pragma unroll
                for (int s = 0; s < SP; s++) { t0[s] = tv[s]; t1[s] = tv[SP + s]; }
            } else {
#pragma unroll
                for (int s = 0; s < SP; s++) {
                    const d2u_t t = *(const d2u_t*)(thin + (long)(s < S ? s : 0) * ts + k);
                    t0[s] = t.x; t1[s] = t.y;
                }
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                const d2u_t v = *(const d2u_t*)(rows[r] + k);
#pragma unroll
                for (int s = 0; s < SP; s++) acc[r][s] = fma(v.y, t1[s], fma(v.x, t0[s], acc[r][s]));
            }
        }
    }
    /* an odd K's last value: one lane of wave 0 */
    if ((K & 1) && wave == 0 && lane == 0) {
        const int k = K - 1;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const double a = rows[r][k];
#pragma unroll
            for (int s = 0; s < SP; s++)
                if (s < S) acc[r][s] = fma(a, DENSE ? thin[(long)k * SP + s] : thin[(long)s * ts + k], acc[r][s]);
        }
    }
    /* across the lanes of a wave (a fixed tree), then across the waves */
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int s = 0; s < SP; s++) {
            double v = acc[r][s];
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
            if (lane == 0) red[wave][r][s] = v;
        }
    __syncthreads();
    const int t = (int)threadIdx.x;
    if (t < R * SP) {
        const int r = t / SP, s = t % SP;
        if (o0 + r < O && s < S)
            C[(long)(o0 + r) * co + (long)s * cs] = ((red[0][r][s] + red[1][r][s]) + red[2][r][s]) + red[3][r][s];
    }
}

template <int SP>
int launch_kfirst(const double* big, long ldb, int K, int O, const double* thin, long ts, long tk, int S,
                  double* C, long cs, long co, hipStream_t st) {
    const int gx = (O + COLS_PER_WG - 1) / COLS_PER_WG;
    /* enough workgroups for four per CU; a workgroup's k-range at least 64 rows, a multiple of 16 */
    const int want = 4 * eshkol_hip_num_cus();
    int pieces = (want + gx - 1) / gx;
    if (pieces > K / 64) pieces = K / 64;
    if (pieces < 1) pieces = 1;
    int kchunk = ((K + pieces - 1) / pieces + 15) & ~15;
    pieces = (K + kchunk - 1) / kchunk;
    double* part = nullptr;
    if (pieces > 1) {
        part = (double*)eshkol_hip_workspace(WS_DGEMM_PARTIAL, (size_t)pieces * S * O * sizeof(double));
        if (!part) { pieces = 1; kchunk = (K + 15) & ~15; }
    }
    const dim3 grid((unsigned)gx, (unsigned)pieces);
    const int contig = (tk == 1) ? 1 : (ts == 1 && tk == S) ? 2 : 0;
    if (contig == 1)
        hipLaunchKernelGGL((skinny_kfirst_kernel<SP, 1>), grid, dim3(256), 0, st, big, ldb, K, O, thin, ts, tk, S, C, cs, co, part, kchunk);
    else if (contig == 2)
        hipLaunchKernelGGL((skinny_kfirst_kernel<SP, 2>), grid, dim3(256), 0, st, big, ldb, K, O, thin, ts, tk, S, C, cs, co, part, kchunk);
    else
        hipLaunchKernelGGL((skinny_kfirst_kernel<SP, 0>), grid, dim3(256), 0, st, big, ldb, K, O, thin, ts, tk, S, C, cs, co, part, kchunk);
    if (pieces > 1)
        hipLaunchKernelGGL(skinny_fixup_kernel, dim3((unsigned)((O + 255) / 256), (unsigned)S), dim3(256), 0, st,
                           part, pieces, S, O, C, cs, co);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

template <int SP, int R, bool DENSE>
int launch_klast(const double* big, long ldb, int O, int K, const double* thin, long ts, int S,
                 double* C, long co, long cs, hipStream_t st) {
    hipLaunchKernelGGL((skinny_klast_kernel<SP, R, DENSE>), dim3((unsigned)((O + R - 1) / R)), dim3(256), 0, st,
                       big, ldb, O, K, thin, ts, S, C, co, cs);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

}  // namespace

/* Whether eshkol_hip_dgemm_skinny takes the product: one side thin, the other long
 * enough to give every CU work, and the big operand worth a pass of its own. */
bool eshkol_hip_dgemm_is_skinny(uint64_t M, uint64_t K, uint64_t N, int trans_a, int trans_b) {
    const uint64_t thin = M < N ? M : N, wide = M < N ? N : M;
    if (thin == 0 || wide < 128 || K < 64 || K > 0x7fffffffULL || wide > 0x7fffffffULL) return false;
    /* The kernel for k-contiguous big operands holds R x S sums per lane and is out of
     * registers after eight thin columns; the other one carries up to thirty-two thin rows
     * (3 TB/s at 32 x 8192 x 8192, where the tiled kernel reaches 2), from seventeen on only
     * where the big operand is large enough for the difference to show. */
    const bool thin_m = M <= N;
    const bool kfirst = thin_m ? !trans_b : (trans_a != 0);     /* the big operand has the output index contiguous */
    const uint64_t limit = !kfirst ? 8u : (wide * K >= (1ull << 24)) ? 32u : 16u;
    return thin <= limit && wide * K >= (1ull << 17);
}

/* C = op(A) op(B) for a product eshkol_hip_dgemm_is_skinny() accepts. */
int eshkol_hip_dgemm_skinny(const double* A, const double* B, double* C, uint64_t M, uint64_t K, uint64_t N,
                            int trans_a, int trans_b, hipStream_t st) {
    const bool thin_m = M <= N;
    const int S = (int)(thin_m ? M : N), O = (int)(thin_m ? N : M), k = (int)K;
    const double* big = thin_m ? B : A;
    const double* thin = thin_m ? A : B;
    /* element (row of the product's thin index s, k) of the thin operand, and C(s, o) */
    long ts, tk, cs, co;
    if (thin_m) { ts = trans_a ? 1 : (long)K; tk = trans_a ? (long)M : 1; cs = (long)N; co = 1; }
    else        { ts = trans_b ? (long)K : 1; tk = trans_b ? 1 : (long)N; cs = 1; co = (long)N; }
    const bool kfirst = thin_m ? !trans_b : (trans_a != 0);
    const long ldb = kfirst ? (long)O : (long)K;
    const int sp = S <= 1 ? 1 : S <= 2 ? 2 : S <= 4 ? 4 : S <= 8 ? 8 : S <= 16 ? 16 : 32;
    if (kfirst && sp >= 16 && tk == 1) {
        /* From nine thin rows of k on: sixteen streams of scalar loads, one per row, run at
         * less than half the rate of the same values held densely as [K][S] (16 x 8192 x 8192:
         * 0.29 ms against 0.12): a megabyte, transposed first. */
        double* dense = (double*)eshkol_hip_workspace(WS_DGEMM_PAD_A, (size_t)K * S * sizeof(double));
        if (!dense) return -1;
        hipLaunchKernelGGL(skinny_thin_to_dense_kernel, dim3((unsigned)((k + 255) / 256)), dim3(256), 0, st, thin, ts, S, k, dense);
        thin = dense; ts = 1; tk = S;
    }
    if (kfirst) {
        switch (sp) {
            case 1: return launch_kfirst<1>(big, ldb, k, O, thin, ts, tk, S, C, cs, co, st);
            case 2: return launch_kfirst<2>(big, ldb, k, O, thin, ts, tk, S, C, cs, co, st);
            case 4: return launch_kfirst<4>(big, ldb, k, O, thin, ts, tk, S, C, cs, co, st);
            case 8: return launch_kfirst<8>(big, ldb, k, O, thin, ts, tk, S, C, cs, co, st);
            case 16: return launch_kfirst<16>(big, ldb, k, O, thin, ts, tk, S, C, cs, co, st);
            default: return launch_kfirst<32>(big, ldb, k, O, thin, ts, tk, S, C, cs, co, st);
        }
    }
    /* the thin operand with k last: k contiguous (tk == 1), or dense [K][S] (ts == 1, tk == S) */
    constexpr int R = 8;
    if (tk == 1) {
        switch (sp) {
            case 1: return launch_klast<1, R, false>(big, ldb, O, k, thin, ts, S, C, co, cs, st);
            case 2: return launch_klast<2, R, false>(big, ldb, O, k, thin, ts, S, C, co, cs, st);
            case 4: return launch_klast<4, R, false>(big, ldb, O, k, thin, ts, S, C, co, cs, st);
            default: return launch_klast<8, R, false>(big, ldb, O, k, thin, ts, S, C, co, cs, st);
        }
    }
    switch (S) {
        case 1: return launch_klast<1, R, true>(big, ldb, O, k, thin, ts, S, C, co, cs, st);
        case 2: return launch_klast<2, R, true>(big, ldb, O, k, thin, ts, S, C, co, cs, st);
        case 3: return launch_klast<3, R, true>(big, ldb, O, k, thin, ts, S, C, co, cs, st);
        case 4: return launch_klast<4, R, true>(big, ldb, O, k, thin, ts, S, C, co, cs, st);
        case 5: return launch_klast<5, R, true>(big, ldb, O, k, thin, ts, S, C, co, cs, st);
        case 6: return launch_klast<6, R, true>(big, ldb, O, k, thin, ts, S, C, co, cs, st);
        case 7: return launch_klast<7, R, true>(big, ldb, O, k, thin, ts, S, C, co, cs, st);
        default: return launch_klast<8, R, true>(big, ldb, O, k, thin, ts, S, C, co, cs, st);
    }
}
