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
 *              distinct banks. An operand the caller holds transposed (the
 *              backward products G*B^T and A^T*G) takes the other operand's
 *              tile form, so no transposed copy is ever made
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

#include <type_traits>

typedef double d4_t __attribute__((ext_vector_type(4)));
typedef double d2_t __attribute__((ext_vector_type(2)));

namespace {

constexpr int BK = 16;

/* One operand of a block tile: R rows (the m or the n extent) by BK k-values.
 * KMAJ = false: the matrix is stored row by row with k contiguous (A as given,
 *   B when the caller holds its transpose); LDS tile [R][BK+2], a lane reads
 *   its four k-values as two 16-byte loads.
 * KMAJ = true:  the matrix is stored k by k with the row index contiguous (B
 *   as given, A when the caller holds its transpose); LDS tile [BK][R+4], a
 *   lane reads one 8-byte value per MFMA step.
 * The pads make every LDS access of a wave hit distinct banks. Both forms hand
 * the MFMA the value at (row li + 16 t, k = 4 lg + s), so they are
 * interchangeable on either side of the instruction. */
template <int R, bool KMAJ, bool VEC, bool LK = KMAJ> struct Operand {
    /* LK: the LDS tile is k-major. Always so for a k-major matrix; for a
     * row-major one it means the pair a thread loaded is written as two 8-byte
     * values one LDS row apart (a transpose on the way in). */
    static_assert(LK || !KMAJ, "a k-major matrix keeps its form in LDS");
    /* k-major tile of a k-major matrix: a thread writes 16 bytes of one LDS row,
     * pitch R + 4. k-major tile of a row-major matrix: the eight lanes that loaded
     * 128 contiguous bytes of a matrix row write sixteen LDS rows, two apart per
     * lane: an odd pitch puts those rows 4 banks apart, so that sixteen lanes'
     * 8-byte writes cover all 32 banks (with R + 4 they fell on two bank pairs,
     * four deep, and the writes held up the fragment reads behind them). */
    static constexpr int LD_S = LK ? (KMAJ ? R + 4 : R + 1) : BK + 2;
    static constexpr int TILE = LK ? BK * LD_S : R * LD_S;
    static constexpr int CHUNKS = R * BK / 2 / 256;   /* 16-byte chunks per thread */
    static constexpr int T = R / 32;                  /* 16-row tiles per wave */
    d2_t reg[CHUNKS];
    d2_t lo[LK ? 1 : T], hi[LK ? 1 : T];
    const double* base;

    /* rows = row count of the whole matrix, K = its k extent */
    __device__ __forceinline__ void gload(const double* __restrict__ P, int rows, int K,
                                          int r0, int k0, int tid) {
#pragma unroll
        for (int r = 0; r < CHUNKS; r++) {
            const int c = tid + 256 * r;
            d2_t v = {0.0, 0.0};
            if (KMAJ) {
                const int kr = c / (R / 2), rc = c % (R / 2);
                const int gk = k0 + kr, gr = r0 + 2 * rc;
                const double* p = P + (size_t)gk * rows + gr;
                if (VEC) {
                    if (gk < K && gr < rows) v = *(const d2_t*)p;
                } else {
                    if (gk < K && gr < rows) v.x = p[0];
                    if (gk < K && gr + 1 < rows) v.y = p[1];
                }
            } else {
                const int row = c >> 3, kc = c & 7;
                const int gr = r0 + row, gk = k0 + 2 * kc;
                const double* p = P + (size_t)gr * K + gk;
                if (VEC) {
                    if (gr < rows && gk < K) v = *(const d2_t*)p;
                } else {
                    if (gr < rows && gk < K) v.x = p[0];
                    if (gr < rows && gk + 1 < K) v.y = p[1];
                }
            }
            reg[r] = v;
        }
    }
    __device__ __forceinline__ void sstore(double* S, int tid) const {
#pragma unroll
        for (int r = 0; r < CHUNKS; r++) {
            const int c = tid + 256 * r;
            if (KMAJ) {
                const int kr = c / (R / 2), rc = c % (R / 2);
                *(d2_t*)(S + kr * LD_S + 2 * rc) = reg[r];
            } else if (LK) {
                const int row = c >> 3, kc = c & 7;
                S[(2 * kc) * LD_S + row] = reg[r].x;
                S[(2 * kc + 1) * LD_S + row] = reg[r].y;
            } else {
                const int row = c >> 3, kc = c & 7;
                *(d2_t*)(S + row * LD_S + 2 * kc) = reg[r];
            }
        }
    }
    /* woff = first row of this wave inside the block tile */
    __device__ __forceinline__ void frag_begin(const double* S, int woff, int li, int lg) {
        if (LK) {
            base = S + (4 * lg) * LD_S + woff + li;
        } else {
            base = S + (woff + li) * LD_S + 4 * lg;
#pragma unroll
            for (int t = 0; t < T; t++) {
                lo[t] = *(const d2_t*)(base + t * 16 * LD_S);
                hi[t] = *(const d2_t*)(base + t * 16 * LD_S + 2);
            }
        }
    }
    __device__ __forceinline__ double frag(int s, int t) const {
        if (LK) return base[s * LD_S + t * 16];
        return (s == 0) ? lo[t].x : (s == 1) ? lo[t].y : (s == 2) ? hi[t].x : hi[t].y;
    }
};

/* Position L in the tile order -> tile: groups of eight tile rows, the row index
 * running fastest inside a group. */
__device__ __forceinline__ void tile_of_index(int L, int tiles_m, int tiles_n, int* tm, int* tn) {
    const int GM = 8;
    const int width = GM * tiles_n;
    const int group = L / width;
    const int first_m = group * GM;
    const int gsize = (tiles_m - first_m < GM) ? tiles_m - first_m : GM;
    const int in_group = L - group * width;
    *tm = first_m + in_group % gsize;
    *tn = in_group / gsize;
}

/* Workgroup -> position in the tile order: XCD x (workgroups x, x+8, ...) takes
 * the x-th eighth of the launch's positions, so neighbours in the order share an L2. */
__device__ __forceinline__ void tile_of_workgroup(int nwg, int tiles_m, int tiles_n, int* tm, int* tn) {
    const int wg = blockIdx.x;
    const int q = nwg >> 3, r = nwg & 7;
    const int xcd = wg & 7, seq = wg >> 3;
    const int L = xcd * q + (xcd < r ? xcd : r) + seq;
    tile_of_index(L, tiles_m, tiles_n, tm, tn);
}

/* C[MxN] = op(A) * op(B). TA: A is stored as its transpose [K][M]; TB: B is
 * stored as its transpose [N][K]. VEC: every row pitch is even and both bases
 * are 16-byte aligned, so operands move as 16-byte pairs. */
template <int BM, int BN, bool VEC, bool TA, bool TB, bool ALK, bool BLK>
__global__ __launch_bounds__(256)
void dgemm_mfma_kernel(const double* __restrict__ A, const double* __restrict__ B,
                       double* __restrict__ C, int M, int N, int K,
                       int tiles_m, int tiles_n) {
    using OpA = Operand<BM, TA, VEC, ALK>;
    using OpB = Operand<BN, !TB, VEC, BLK>;
    extern __shared__ __align__(16) double smem[];
    double* As = smem;
    double* Bs = smem + 2 * OpA::TILE;

    /* blockIdx.y walks a batch of dense products stored back to back */
    A += (size_t)blockIdx.y * M * K;
    B += (size_t)blockIdx.y * K * N;
    C += (size_t)blockIdx.y * M * N;

    int tm, tn;
    tile_of_workgroup((int)gridDim.x, tiles_m, tiles_n, &tm, &tn);
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 15, lg = lane >> 4;

    OpA a;
    OpB b;

    d4_t acc[OpA::T][OpB::T];
#pragma unroll
    for (int t = 0; t < OpA::T; t++)
#pragma unroll
        for (int u = 0; u < OpB::T; u++) acc[t][u] = (d4_t){0.0, 0.0, 0.0, 0.0};

    const int nkb = (K + BK - 1) / BK;
    a.gload(A, M, K, m0, 0, tid);
    b.gload(B, N, K, n0, 0, tid);
    a.sstore(As, tid);
    b.sstore(Bs, tid);
    __syncthreads();

    int cur = 0;
    for (int kb = 0; kb < nkb; kb++) {
        const bool more = (kb + 1 < nkb);
        if (more) {
            a.gload(A, M, K, m0, (kb + 1) * BK, tid);
            b.gload(B, N, K, n0, (kb + 1) * BK, tid);
        }

        a.frag_begin(As + cur * OpA::TILE, wm * (BM / 2), li, lg);
        b.frag_begin(Bs + cur * OpB::TILE, wn * (BN / 2), li, lg);
#pragma unroll
        for (int s = 0; s < 4; s++) {
            double av[OpA::T], bv[OpB::T];
#pragma unroll
            for (int t = 0; t < OpA::T; t++) av[t] = a.frag(s, t);
#pragma unroll
            for (int u = 0; u < OpB::T; u++) bv[u] = b.frag(s, u);
#pragma unroll
            for (int t = 0; t < OpA::T; t++)
#pragma unroll
                for (int u = 0; u < OpB::T; u++)
                    acc[t][u] = __builtin_amdgcn_mfma_f64_16x16x4f64(av[t], bv[u], acc[t][u], 0, 0, 0);
        }

        if (more) {
            a.sstore(As + (cur ^ 1) * OpA::TILE, tid);
            b.sstore(Bs + (cur ^ 1) * OpB::TILE, tid);
        }
        __syncthreads();
        cur ^= 1;
    }

    /* accumulator layout: register r of the lane is row 4*r + lane/16, column lane%16 */
#pragma unroll
    for (int t = 0; t < OpA::T; t++)
#pragma unroll
        for (int u = 0; u < OpB::T; u++) {
            const int col = n0 + wn * (BN / 2) + u * 16 + li;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int row = m0 + wm * (BM / 2) + t * 16 + 4 * r + lg;
                if (row < M && col < N) C[(size_t)row * N + col] = acc[t][u][r];
            }
        }
}

/* ---- straight-line kernel -----------------------------------------------------
 * For launches of at least 256 tiles whose operands move as 16-byte chunks
 * (even row pitches, aligned bases). The loads carry no bounds checks: rows of
 * an edge tile are clamped to the matrix (their outputs are never stored) and a
 * k-tail is zeroed with selects in a variant of its own. A k-block is therefore
 * one straight-line region and its memory operations can be placed between the
 * MFMAs instead of around them:
 *
 *   step 0   MFMAs of k 0..3    | LDS reads of the step-1 fragments
 *   step 1   MFMAs of k 4..7    | LDS reads of step 2
 *   step 2   MFMAs of k 8..11   | LDS reads of step 3, LDS writes of block g+1
 *            LDS-only barrier (s_waitcnt lgkmcnt(0); s_barrier: a __syncthreads
 *            would also wait for the global loads issued below)
 *   step 3   MFMAs of k 12..15  | LDS reads of block g+1's step-0 fragments,
 *                                 global loads of block g+2 into the staging
 *                                 registers step 2 has just emptied
 *
 * A global load therefore has a whole k-block of MFMA time to land, the wave
 * never waits on a barrier with its next operands unread, and the staging
 * registers are reused without a second set. Both LDS tiles are k-major (a
 * row-major operand is transposed by its LDS writes), so every fragment is an
 * 8-byte read at a compile-time offset. */
using I0 = std::integral_constant<int, 0>;
using I1 = std::integral_constant<int, 1>;

__device__ __forceinline__ void lds_only_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

/* SPLIT: the launch covers the last `tail` tiles of the tile order, each cut
 * along k into pieces of kb_per_piece k-blocks; workgroup whole + piece * tail + i
 * multiplies piece `piece` of tail tile i and leaves the whole partial tile in
 * `partial` (dgemm_fixup_kernel adds the pieces up in order). The first `whole`
 * workgroups of such a launch compute the tiles at positions 0 .. whole - 1 of
 * the tile order whole, as an unsplit launch of `whole` workgroups would (small
 * tiles only; 0 for large ones). */
struct SplitArgs { int first_tile, tail, kb_per_piece; double* partial; int whole; int lda, ldb; };
/* lda, ldb: row pitches of the operands as stored, in doubles; 0 for the dense pitch
 * the shape implies. Set (by dgemm_any, under the library lock every entry point
 * holds) when an operand was copied to an even pitch first; the launchers below put
 * them into every SplitArgs they build. */
int g_lda = 0, g_ldb = 0;

template <bool TA, bool TB, bool KTAIL, bool SPLIT, int TS = 128, int PF = 1>
__global__ __launch_bounds__(256, TS == 128 ? 2 : 4)
void dgemm_fast_kernel(const double* __restrict__ A, const double* __restrict__ B,
                       double* __restrict__ C, int M, int N, int K,
                       int tiles_m, int tiles_n, SplitArgs sp) {
    /* TS: edge of the block tile. 128 (wave tile 64 x 64) is the kernel of large
     * launches; 64 (wave tile 32 x 32, four workgroups to a CU) serves launches
     * that would leave CUs idle or half a round empty with the large tile. */
    /* PF: how many k-blocks ahead of the LDS writes the global loads run. With 1 a
     * load has three steps of MFMAs to land (one staging set, refilled as soon as
     * the LDS writes have emptied it): enough when other workgroups share the CU
     * or a step is 1024 cycles long. With 2 (two staging sets, block j in set
     * j % 2) it has a whole k-block more: for the small tile, whose step is 256
     * cycles, when a CU holds one workgroup. */
    static_assert(TS == 128 || TS == 64, "tile edges");
    static_assert(PF == 1 || PF == 2, "one or two staging sets");
    constexpr int BM = TS, BN = TS;
    constexpr int TT = TS / 32;                  /* 16 x 16 MFMA tiles per wave and dimension */
    using OpA = Operand<BM, TA, true, true>;
    using OpB = Operand<BN, !TB, true, true>;
    constexpr int LDA = OpA::LD_S, LDB = OpB::LD_S;
    extern __shared__ __align__(16) double smem[];
    double* As = smem;
    double* Bs = smem + 2 * OpA::TILE;

    A += (size_t)blockIdx.y * M * K;
    B += (size_t)blockIdx.y * K * N;
    C += (size_t)blockIdx.y * M * N;

    int tm, tn;
    /* in a cut launch: this workgroup multiplies a piece (else one of the leading whole
     * tiles, which only launches of small tiles have: the large tile's cut variants
     * have no register to spare for the distinction) */
    const bool is_piece = SPLIT && (TS == 128 || (int)blockIdx.x >= sp.whole);
    const int piece_wg = !SPLIT ? 0 : (TS == 128) ? (int)blockIdx.x : (int)blockIdx.x - sp.whole;
    if (is_piece) tile_of_index(sp.first_tile + (int)((unsigned)piece_wg % (unsigned)sp.tail), tiles_m, tiles_n, &tm, &tn);
    else tile_of_workgroup(SPLIT ? sp.whole : (int)gridDim.x, tiles_m, tiles_n, &tm, &tn);
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 15, lg = lane >> 4;

    /* This thread's four 16-byte chunks of each operand tile: global pointers
     * for k-block 0. Rows beyond the matrix (edge tiles) are clamped to its last
     * rows: they load valid memory and feed outputs that are never stored. */
    const int lda = sp.lda ? sp.lda : (TA ? M : K), ldb = sp.ldb ? sp.ldb : (TB ? K : N);
    const double* pa[OpA::CHUNKS];
    const double* pb[OpB::CHUNKS];
    /* first k of chunk r inside a k-block (recomputed where the k-tail needs it: the few
     * registers it would take to keep them are the ones this kernel does not have) */
    auto ka_of = [&](int r) { const int c = tid + 256 * r; return TA ? c / (BM / 2) : 2 * (c & 7); };
    auto kbo_of = [&](int r) { const int c = tid + 256 * r; return TB ? 2 * (c & 7) : c / (BN / 2); };
#pragma unroll
    for (int r = 0; r < OpA::CHUNKS; r++) {
        const int c = tid + 256 * r;
        if (TA) {
            int m = m0 + 2 * (c % (BM / 2));
            m = (m < lda - 2) ? m : lda - 2;         /* a pair may end in the pitch's padding, not beyond it */
            pa[r] = A + (size_t)ka_of(r) * lda + m;
        } else {
            int m = m0 + (c >> 3);
            m = (m < M - 1) ? m : M - 1;
            pa[r] = A + (size_t)m * lda + ka_of(r);
        }
    }
#pragma unroll
    for (int r = 0; r < OpB::CHUNKS; r++) {
        const int c = tid + 256 * r;
        if (TB) {
            int n = n0 + (c >> 3);
            n = (n < N - 1) ? n : N - 1;
            pb[r] = B + (size_t)n * ldb + kbo_of(r);
        } else {
            int n = n0 + 2 * (c % (BN / 2));
            n = (n < ldb - 2) ? n : ldb - 2;
            pb[r] = B + (size_t)kbo_of(r) * ldb + n;
        }
    }
    const size_t a_step = TA ? (size_t)BK * lda : (size_t)BK;   /* doubles per k-block */
    const size_t b_step = TB ? (size_t)BK : (size_t)BK * ldb;

    OpA a[PF];
    OpB b[PF];
    /* KTAIL: K is not a multiple of 16. A chunk whose k lies beyond K reads the
     * same chunk of k-block 0 instead (valid memory, K >= 16) and is zeroed. */
    /* `masked` (a compile-time flag): the block may be the one that holds the k-tail.
     * Only the last requests of a workgroup pay for the selects; all others are plain
     * loads, as in the variant without a tail. */
    auto gload = [&](int kb, auto set, auto masked) {
        constexpr int S = decltype(set)::value;
        constexpr bool MASK = KTAIL && decltype(masked)::value;
#pragma unroll
        for (int r = 0; r < OpA::CHUNKS; r++) {
            const bool ok = !MASK || (kb * BK + ka_of(r) < K);
            const d2_t v = *(const d2_t*)(pa[r] + (size_t)(ok ? kb : 0) * a_step);
            a[S].reg[r] = ok ? v : (d2_t){0.0, 0.0};
        }
#pragma unroll
        for (int r = 0; r < OpB::CHUNKS; r++) {
            const bool ok = !MASK || (kb * BK + kbo_of(r) < K);
            const d2_t v = *(const d2_t*)(pb[r] + (size_t)(ok ? kb : 0) * b_step);
            b[S].reg[r] = ok ? v : (d2_t){0.0, 0.0};
        }
    };

    d4_t acc[TT][TT];
#pragma unroll
    for (int t = 0; t < TT; t++)
#pragma unroll
        for (int u = 0; u < TT; u++) acc[t][u] = (d4_t){0.0, 0.0, 0.0, 0.0};

    double af[2][TT], bf[2][TT];
    const int a_off = (4 * lg) * LDA + wm * (BM / 2) + li;
    const int b_off = (4 * lg) * LDB + wn * (BN / 2) + li;
    auto ldfrag = [&](int buf, int st, auto which) {
        constexpr int W = decltype(which)::value;
        const double* ab = As + buf * OpA::TILE + a_off + st * LDA;
        const double* bb = Bs + buf * OpB::TILE + b_off + st * LDB;
#pragma unroll
        for (int t = 0; t < TT; t++) af[W][t] = ab[t * 16];
#pragma unroll
        for (int u = 0; u < TT; u++) bf[W][u] = bb[u * 16];
    };
    auto mfma_step = [&](auto which) {
        constexpr int W = decltype(which)::value;
#pragma unroll
        for (int t = 0; t < TT; t++)
#pragma unroll
            for (int u = 0; u < TT; u++)
                acc[t][u] = __builtin_amdgcn_mfma_f64_16x16x4f64(af[W][t], bf[W][u], acc[t][u], 0, 0, 0);
    };

    /* this workgroup's k-blocks [kb_lo, kb_hi): all of them unless the tile is split */
    const int nkb_all = (K + BK - 1) / BK;
    const int piece = is_piece ? (int)((unsigned)piece_wg / (unsigned)sp.tail) : 0;
    const int kb_lo = is_piece ? piece * sp.kb_per_piece : 0;
    const int kb_hi = is_piece ? ((kb_lo + sp.kb_per_piece < nkb_all) ? kb_lo + sp.kb_per_piece : nkb_all) : nkb_all;
    auto clamped = [&](int kb) { return kb < kb_hi ? kb : kb_hi - 1; };   /* requests past the end are never consumed */
    gload(kb_lo, I0{}, I1{});
    a[0].sstore(As, tid);
    b[0].sstore(Bs, tid);
    if constexpr (PF == 2) {
        gload(clamped(kb_lo + 1), I1{}, I1{});
        gload(clamped(kb_lo + 2), I0{}, I1{});
    } else {
        gload(clamped(kb_lo + 1), I0{}, I1{});
    }
    __syncthreads();
    ldfrag(0, 0, I0{});

    /* one k-block; `parity` = (kb - kb_lo) % 2 is its LDS buffer and, with two
     * staging sets, the set the block after it is not in */
    auto block = [&](int kb, auto parity, auto masked) {
        constexpr int cur = decltype(parity)::value;
        using NextSet = std::integral_constant<int, PF == 2 ? (cur ^ 1) : 0>;    /* holds block kb + 1 */
        const int kb2 = clamped(kb + 1 + PF);

        /* per step: NM MFMAs, TT fragment reads (pairs), and in step 2 the LDS writes of
         * the next block (3 per chunk pair), in step 3 its successor's global loads */
        constexpr int NM = TT * TT;
        constexpr int WR_PER = 2;                  /* 64 x 64: six LDS writes behind three of the four MFMAs */
        constexpr int GL = OpA::CHUNKS + OpB::CHUNKS;

        /* With two staging sets block kb + 1 has been in registers for a whole k-block:
         * its LDS writes go here, into the buffer every wave left behind at the last
         * barrier, and are long finished when this block's barrier asks for them. */
        ldfrag(cur, 1, I1{});
        if constexpr (PF == 2) {
            a[NextSet::value].sstore(As + (cur ^ 1) * OpA::TILE, tid);
            b[NextSet::value].sstore(Bs + (cur ^ 1) * OpB::TILE, tid);
        }
        mfma_step(I0{});
#pragma unroll
        for (int i = 0; i < NM; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i < TT) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (PF == 2) {
                if (TS == 128) { if (i >= 2 && i < 14) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0); }
                else if (i >= 1) __builtin_amdgcn_sched_group_barrier(0x200, WR_PER, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);

        ldfrag(cur, 2, I0{});
        mfma_step(I1{});
#pragma unroll
        for (int i = 0; i < NM; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i < TT) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);

        ldfrag(cur, 3, I1{});
        if constexpr (PF == 1) {
            a[NextSet::value].sstore(As + (cur ^ 1) * OpA::TILE, tid);
            b[NextSet::value].sstore(Bs + (cur ^ 1) * OpB::TILE, tid);
        }
        mfma_step(I0{});
#pragma unroll
        for (int i = 0; i < NM; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i < TT) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (PF == 1) {
                if (TS == 128) { if (i >= 2 && i < 14) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0); }
                else if (i >= 1) __builtin_amdgcn_sched_group_barrier(0x200, WR_PER, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        lds_only_barrier();

        ldfrag(cur ^ 1, 0, I0{});
        gload(kb2, NextSet{}, masked);
        mfma_step(I1{});
#pragma unroll
        for (int i = 0; i < NM; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i < TT) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (i < GL) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    /* the blocks whose request (1 + PF blocks ahead) cannot reach the last block of k
     * run without the tail's selects; the few that follow run with them */
    int kb = kb_lo;
    if constexpr (KTAIL) {
        for (; kb + 1 + (1 + PF) < kb_hi - 1; kb += 2) {     /* block kb + 1 requests block kb + 2 + PF: not the last */
            block(kb, I0{}, I0{});
            block(kb + 1, I1{}, I0{});
        }
        for (; kb + 1 < kb_hi; kb += 2) {          /* kb - kb_lo is even here: the parities stay compile-time */
            block(kb, I0{}, I1{});
            block(kb + 1, I1{}, I1{});
        }
        if (kb < kb_hi) block(kb, I0{}, I1{});
    } else {
        for (; kb + 1 < kb_hi; kb += 2) {
            block(kb, I0{}, I0{});
            block(kb + 1, I1{}, I0{});
        }
        if (kb < kb_hi) block(kb, I0{}, I0{});
    }

    if (is_piece) {
        double* out = sp.partial + (size_t)piece_wg * (BM * BN);
#pragma unroll
        for (int t = 0; t < TT; t++)
#pragma unroll
            for (int u = 0; u < TT; u++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                    out[(wm * (BM / 2) + t * 16 + 4 * r + lg) * BN + wn * (BN / 2) + u * 16 + li] = acc[t][u][r];
        return;
    }
#pragma unroll
    for (int t = 0; t < TT; t++)
#pragma unroll
        for (int u = 0; u < TT; u++) {
            const int col = n0 + wn * (BN / 2) + u * 16 + li;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int row = m0 + wm * (BM / 2) + t * 16 + 4 * r + lg;
                if (row < M && col < N) C[(size_t)row * N + col] = acc[t][u][r];
            }
        }
}

/* Adds up the partial tiles of dgemm_fast_kernel<..., SPLIT>: piece 0 first, so the
 * result does not depend on which workgroup finished when. TS: the tile's edge.
 * grid (tail, TS / (1024 / TS)): a thread sums four consecutive columns of a row,
 * TS / 4 threads a row, a workgroup 1024 / TS rows of one tile. */
template <int TS>
__global__ __launch_bounds__(256)
void dgemm_fixup_kernel(const double* __restrict__ partial, int tail, int pieces, int first_tile,
                        int tiles_m, int tiles_n, double* __restrict__ C, int M, int N) {
    constexpr int PER_ROW = TS / 4, ROWS = 256 / PER_ROW;
    int tm, tn;
    tile_of_index(first_tile + (int)blockIdx.x, tiles_m, tiles_n, &tm, &tn);
    const int lrow = (int)blockIdx.y * ROWS + (int)(threadIdx.x / PER_ROW), lcol = 4 * (int)(threadIdx.x % PER_ROW);
    const double* p = partial + (size_t)blockIdx.x * (TS * TS) + lrow * TS + lcol;
    d2_t s0 = *(const d2_t*)p, s1 = *(const d2_t*)(p + 2);
    for (int q = 1; q < pieces; q++) {
        const double* pq = p + (size_t)q * tail * (TS * TS);
        const d2_t v0 = *(const d2_t*)pq, v1 = *(const d2_t*)(pq + 2);
        s0.x += v0.x; s0.y += v0.y; s1.x += v1.x; s1.y += v1.y;
    }
    const int row = tm * TS + lrow, col = tn * TS + lcol;
    if (row >= M) return;
    double* c = C + (size_t)row * N + col;
    if (col < N) c[0] = s0.x;
    if (col + 1 < N) c[1] = s0.y;
    if (col + 2 < N) c[2] = s1.x;
    if (col + 3 < N) c[3] = s1.y;
}

int g_tail_split = 1;

/* What a launch of the straight-line kernels is expected to take, in microseconds,
 * from fits to measurements on this device (16 ... 6400 tiles, K = 256 ... 8192; the
 * fits are within a few per cent of the measurements they came from). A CU works
 * through the tiles it is given at a fixed rate per k-block whether they share the
 * CU or follow one another, so a launch takes as long as its fullest CU:
 *   128 x 128 tiles: 10 + 1.82 per k-block and tile of the fullest CU;
 *   64 x 64 tiles:   10 + 0.46 per k-block and tile of the fullest CU (0.483 where
 *                    no CU holds more than one): four small tiles cost 2 % more
 *                    than a large one, and fill the device four times finer;
 *   large tiles cut along k into p pieces (launches that do not fill the device):
 *                    10 + 0.04 per workgroup (two launches, the partial tiles' round
 *                    trip) + 2.2 per k-block of a piece, times 1.7 once some CUs
 *                    hold two workgroups;
 *   a last round of large tiles cut along k: the full rounds, plus that round's
 *                    share ceil(p tail / slots) / p + 0.006 p, plus 15 for the two
 *                    extra launches. */
constexpr double US_KB_128 = 1.82, US_KB_64 = 0.46, US_KB_64_ALONE = 0.483, US_LAUNCH = 10.0;

/* pieces per tile for a launch of `nwg` large tiles that does not fill the device (1 = whole) and its time */
int small_launch_pieces(long long nwg, int nkb, double* us = nullptr) {
    const int cus = eshkol_hip_num_cus();
    int best_p = 1;
    double best = US_LAUNCH + US_KB_128 * nkb * (double)((nwg + cus - 1) / cus);
    if (4 * nwg < 3 * (long long)cus) {
        for (int p = 2; p <= 128 && nkb / p >= 4 && nwg * p <= 2 * cus; p++) {
            const double crowd = (nwg * p <= cus) ? 1.0 : 1.7;
            const double cost = 10.0 + 0.04 * (double)(nwg * p) + crowd * 2.2 * ((double)nkb / p);
            if (cost < 0.95 * best) { best = cost; best_p = p; }
        }
    }
    if (us) *us = best;
    return best_p;
}

/* pieces per tile of the last, partial round of a launch of more than `slots` large tiles (1 = whole) and the launch's time */
int tail_round_pieces(long long nwg, int nkb, double* share = nullptr) {
    const int slots = 2 * eshkol_hip_num_cus();
    const int tail = (int)(nwg % slots);
    int best_p = 1;
    double best = 1.0;
    if (nwg > slots && tail > 0) {
        for (int p = 2; p <= 32 && nkb / p >= 4; p++) {
            const long long rounds = ((long long)p * tail + slots - 1) / slots;
            const double cost = (double)rounds / p + 0.006 * p;
            if (cost < best - 1e-9) { best = cost; best_p = p; }
        }
        if (!(best < 0.9)) { best = 1.0; best_p = 1; }
    }
    if (share) *share = best;
    return best_p;
}

/* time of the large-tile path as launch_fast_k would run it */
double large_tile_us(long long nwg, int nkb, bool may_cut) {
    const int cus = eshkol_hip_num_cus(), slots = 2 * cus;
    if (may_cut && nwg > slots && nwg % slots != 0) {
        double share;
        if (tail_round_pieces(nwg, nkb, &share) >= 2)
            return US_LAUNCH + 15.0 + 2.0 * US_KB_128 * nkb * ((double)(nwg / slots) + share);
    }
    if (may_cut && 4 * nwg < 3 * (long long)cus) {
        double us;
        small_launch_pieces(nwg, nkb, &us);
        return us;
    }
    return US_LAUNCH + US_KB_128 * nkb * (double)((nwg + cus - 1) / cus);
}

/* Small tiles beyond the last multiple of the CU count make some CUs work a whole
 * tile longer than the others (1536^3: 576 tiles on 256 CUs, three on some, two on
 * most). Those leftover tiles are cut along k into p pieces each, in the same
 * launch behind the whole tiles, so that every CU gets a piece or so of them:
 * pieces per leftover tile (1 = whole) and the launch's expected time, which is
 * the fullest CU's whole tiles and pieces plus 8 us for the launch that adds the
 * pieces up and the partial tiles' round trip. */
int small_tile_tail_pieces(long long nwg64, int nkb, bool may_cut, double* us = nullptr) {
    const int cus = eshkol_hip_num_cus();
    const long long full = nwg64 / cus, rem = nwg64 % cus;
    const long long per_cu = (nwg64 + cus - 1) / cus;
    double best = US_LAUNCH + (per_cu <= 1 ? US_KB_64_ALONE : US_KB_64) * nkb * (double)per_cu;
    int best_p = 1;
    if (may_cut && full >= 1 && rem > 0) {
        for (int p = 2; p <= 16 && nkb / p >= 4; p++) {
            const long long rounds = (p * rem + cus - 1) / cus;
            const double cost = US_LAUNCH + 8.0 + US_KB_64 * nkb * ((double)full + (double)rounds / p) + 0.5 * (double)rounds;
            /* cutting must beat the whole launch by 5 per cent; among cuts the cheapest wins */
            if (best_p == 1 ? cost < 0.95 * best : cost < best) { best = cost; best_p = p; }
        }
    }
    if (us) *us = best;
    return best_p;
}

double small_tile_us(long long nwg64, int nkb, bool may_cut) {
    double us;
    small_tile_tail_pieces(nwg64, nkb, may_cut, &us);
    return us;
}

/* 0 (default) and 2: global loads two k-blocks ahead of their LDS writes wherever that
 * variant holds its registers (all but the 128-tile kernel with a k-tail); 1: one ahead. */
int g_prefetch_depth = 0;

template <bool TA, bool TB, bool KTAIL>
int launch_fast_k(const double* A, const double* B, double* C, int M, int N, int K, int batch, hipStream_t st) {
    constexpr int SMEM_BYTES = 2 * (Operand<128, TA, true, true>::TILE + Operand<128, !TB, true, true>::TILE)
                               * (int)sizeof(double);
    static bool attr_set = false;
    /* with a k-tail the two-set variant of this tile size runs out of registers */
    constexpr int DEEP = KTAIL ? 1 : 2;
    auto kern1 = dgemm_fast_kernel<TA, TB, KTAIL, false, 128, 1>;
    auto kern2 = dgemm_fast_kernel<TA, TB, KTAIL, false, 128, DEEP>;
    auto kern_split1 = dgemm_fast_kernel<TA, TB, KTAIL, true, 128, 1>;
    auto kern_split2 = dgemm_fast_kernel<TA, TB, KTAIL, true, 128, DEEP>;
    if (!attr_set) {
        for (const void* f : {(const void*)kern1, (const void*)kern2, (const void*)kern_split1, (const void*)kern_split2})
            if (!ESHKOL_HIP_OK(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES))) return -1;
        attr_set = true;
    }
    auto kern = g_prefetch_depth == 1 ? kern1 : kern2;
    auto kern_split = g_prefetch_depth == 1 ? kern_split1 : kern_split2;
    const int tiles_m = (M + 127) / 128, tiles_n = (N + 127) / 128;
    const long long nwg = (long long)tiles_m * tiles_n;
    if (nwg > 0x7fffffffLL || batch < 1 || batch > 65535) return -1;
    SplitArgs sp = {0, 1, 0, nullptr, 0, g_lda, g_ldb};

    /* Two workgroups fit on a CU, so a launch runs in rounds of `slots` tiles, and
     * a last round of a few tiles takes as long as a full one. Its tiles are
     * therefore cut along k into p pieces each: p * tail workgroups of 1/p the
     * length, in ceil(p * tail / slots) short rounds (5000^3: 1600 tiles on 512
     * slots, 4.4 -> 4.0 ms; 7680^3: 13.7 -> 12.5 ms). p minimises that time plus
     * a small charge per piece for the extra prologues and the workspace traffic;
     * the pieces go through a workspace and are added in a fixed order. */
    const int slots = 2 * eshkol_hip_num_cus();
    const int tail = (int)(nwg % slots), nkb = (K + BK - 1) / BK;
    const int best_p = (g_tail_split && batch == 1) ? tail_round_pieces(nwg, nkb) : 1;
    if (best_p >= 2) {
        const int kbpp = (nkb + best_p - 1) / best_p;
        const int pieces = (nkb + kbpp - 1) / kbpp;
        double* ws = (pieces >= 2) ? (double*)eshkol_hip_workspace(WS_DGEMM_PARTIAL,
                                         (size_t)tail * pieces * 128 * 128 * sizeof(double)) : nullptr;
        if (ws) {
            sp.first_tile = (int)(nwg - tail); sp.tail = tail; sp.kb_per_piece = kbpp; sp.partial = ws;
            hipLaunchKernelGGL(kern, dim3((unsigned)(nwg - tail), 1), dim3(256), SMEM_BYTES, st,
                               A, B, C, M, N, K, tiles_m, tiles_n, sp);
            hipLaunchKernelGGL(kern_split, dim3((unsigned)(tail * pieces), 1), dim3(256), SMEM_BYTES, st,
                               A, B, C, M, N, K, tiles_m, tiles_n, sp);
            hipLaunchKernelGGL(dgemm_fixup_kernel<128>, dim3((unsigned)tail, 16), dim3(256), 0, st,
                               ws, tail, pieces, sp.first_tile, tiles_m, tiles_n, C, M, N);
            return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
        }
    }
    /* A launch of fewer tiles than CUs leaves CUs idle for its whole length: all
     * its tiles are cut along k the same way (1024^3: 64 tiles, 59 -> 53 us;
     * 512 x 2048 x 512: 16 tiles, 104 -> 33 us; 128 x 8192 x 128: 400 -> 47 us). */
    const int small_p = (g_tail_split && batch == 1) ? small_launch_pieces(nwg, nkb) : 1;
    if (small_p >= 2) {
        const int kbpp = (nkb + small_p - 1) / small_p;
        const int pieces = (nkb + kbpp - 1) / kbpp;
        double* ws = pieces >= 2 ? (double*)eshkol_hip_workspace(WS_DGEMM_PARTIAL,
                                         (size_t)nwg * pieces * 128 * 128 * sizeof(double)) : nullptr;
        if (ws) {
            sp.first_tile = 0; sp.tail = (int)nwg; sp.kb_per_piece = kbpp; sp.partial = ws;
            hipLaunchKernelGGL(kern_split, dim3((unsigned)(nwg * pieces), 1), dim3(256), SMEM_BYTES, st,
                               A, B, C, M, N, K, tiles_m, tiles_n, sp);
            hipLaunchKernelGGL(dgemm_fixup_kernel<128>, dim3((unsigned)nwg, 16), dim3(256), 0, st,
                               ws, (int)nwg, pieces, 0, tiles_m, tiles_n, C, M, N);
            return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
        }
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)nwg, (unsigned)batch), dim3(256), SMEM_BYTES, st,
                       A, B, C, M, N, K, tiles_m, tiles_n, sp);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

template <bool TA, bool TB>
int launch_fast(const double* A, const double* B, double* C, int M, int N, int K, int batch, hipStream_t st) {
    return (K % BK == 0) ? launch_fast_k<TA, TB, false>(A, B, C, M, N, K, batch, st)
                         : launch_fast_k<TA, TB, true>(A, B, C, M, N, K, batch, st);
}

/* The straight-line kernel with 64 x 64 tiles, every tile whole: four workgroups
 * to a CU, four times as many tiles to spread over the device. */
template <bool TA, bool TB, bool KTAIL>
int launch_fast64_k(const double* A, const double* B, double* C, int M, int N, int K, int batch, hipStream_t st) {
    constexpr int SMEM_BYTES = 2 * (Operand<64, TA, true, true>::TILE + Operand<64, !TB, true, true>::TILE)
                               * (int)sizeof(double);
    auto kern = g_prefetch_depth == 1 ? dgemm_fast_kernel<TA, TB, KTAIL, false, 64, 1> : dgemm_fast_kernel<TA, TB, KTAIL, false, 64, 2>;
    const int tiles_m = (M + 63) / 64, tiles_n = (N + 63) / 64;
    const long long nwg = (long long)tiles_m * tiles_n;
    if (nwg > 0x7fffffffLL || batch < 1 || batch > 65535) return -1;
    SplitArgs sp = {0, 1, 0, nullptr, 0, g_lda, g_ldb};
    /* leftover tiles cut along k, in one launch with the whole ones (small_tile_tail_pieces) */
    const int nkb = (K + BK - 1) / BK;
    const int p = small_tile_tail_pieces(nwg, nkb, g_tail_split && batch == 1);
    if (p >= 2) {
        const int cus = eshkol_hip_num_cus();
        const int tail = (int)(nwg % cus), whole = (int)(nwg - tail);
        const int kbpp = (nkb + p - 1) / p;
        const int pieces = (nkb + kbpp - 1) / kbpp;
        double* ws = pieces >= 2 ? (double*)eshkol_hip_workspace(WS_DGEMM_PARTIAL,
                                         (size_t)tail * pieces * 64 * 64 * sizeof(double)) : nullptr;
        if (ws) {
            auto kern_cut = g_prefetch_depth == 1 ? dgemm_fast_kernel<TA, TB, KTAIL, true, 64, 1>
                                                  : dgemm_fast_kernel<TA, TB, KTAIL, true, 64, 2>;
            sp.first_tile = whole; sp.tail = tail; sp.kb_per_piece = kbpp; sp.partial = ws; sp.whole = whole;
            hipLaunchKernelGGL(kern_cut, dim3((unsigned)(whole + tail * pieces), 1), dim3(256), SMEM_BYTES, st,
                               A, B, C, M, N, K, tiles_m, tiles_n, sp);
            hipLaunchKernelGGL(dgemm_fixup_kernel<64>, dim3((unsigned)tail, 4), dim3(256), 0, st,
                               ws, tail, pieces, whole, tiles_m, tiles_n, C, M, N);
            return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
        }
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)nwg, (unsigned)batch), dim3(256), SMEM_BYTES, st,
                       A, B, C, M, N, K, tiles_m, tiles_n, sp);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}
template <bool TA, bool TB>
int launch_fast64(const double* A, const double* B, double* C, int M, int N, int K, int batch, hipStream_t st) {
    return (K % BK == 0) ? launch_fast64_k<TA, TB, false>(A, B, C, M, N, K, batch, st)
                         : launch_fast64_k<TA, TB, true>(A, B, C, M, N, K, batch, st);
}

int g_small_tile = 1;       /* 0 never, 1 where it measures faster, 2 wherever it is legal */

int g_fast_path = 1;

template <int BM, int BN, bool VEC, bool TA, bool TB, bool ALK, bool BLK>
int launch(const double* A, const double* B, double* C, int M, int N, int K, int batch, hipStream_t st) {
    constexpr int SMEM_BYTES = 2 * (Operand<BM, TA, VEC, ALK>::TILE + Operand<BN, !TB, VEC, BLK>::TILE)
                               * (int)sizeof(double);
    static bool attr_set = false;
    auto kern = dgemm_mfma_kernel<BM, BN, VEC, TA, TB, ALK, BLK>;
    if (!attr_set) {
        if (!ESHKOL_HIP_OK(hipFuncSetAttribute((const void*)kern,
                hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES))) return -1;
        attr_set = true;
    }
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const long long nwg = (long long)tiles_m * tiles_n;
    if (nwg > 0x7fffffffLL || batch < 1 || batch > 65535) return -1;
    hipLaunchKernelGGL(kern, dim3((unsigned)nwg, (unsigned)batch), dim3(256), SMEM_BYTES, st,
                       A, B, C, M, N, K, tiles_m, tiles_n);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

enum class Kernel { Fast64, Fast128, General128, General64 };

/* Which kernel a shape takes. */
Kernel choose_kernel(int m, int n, int k, int batch, bool vec) {
    /* Small outputs cannot fill 256 CUs with 128x128 tiles: use 64x64 there. */
    const long long big_tiles = (long long)((m + 127) / 128) * (long long)((n + 127) / 128) * batch;
    /* 16-byte operand chunks (even pitches, aligned bases) and at least one whole k-block */
    const int nkb = (k + BK - 1) / BK;
    const bool may_cut = g_tail_split && batch == 1;
    const bool cut = may_cut && small_launch_pieces(big_tiles, nkb) >= 2;
    const bool straight = g_fast_path && vec && m >= 2 && n >= 2 && k >= BK;
    /* Tile size of the straight-line kernel: whichever the fits above expect to finish
     * first. Small tiles win where large ones would leave CUs idle or a round half
     * empty and k is too short for cutting them to pay (1024^3: 41 us against 55 for
     * the cut large tiles and 58 for whole ones; 2304 x 2304 x 2048: 360 against 463;
     * 3072^3: 1075 against 1078 cut and 1385 whole); large tiles win full rounds by
     * 2 % and, cut along k, launches of a few tiles with a long k. */
    const long long small_tiles = (long long)((m + 63) / 64) * (long long)((n + 63) / 64) * batch;
    /* (the small tile's rate holds up to about two rounds of large tiles; beyond, its
     * four-fold operand traffic tells: 5120^3 3.86 ms against 3.63 for large tiles with
     * a cut last round, where the fits call it even) */
    if (straight && (g_small_tile == 2 ||
                     (g_small_tile == 1 && big_tiles < 4LL * eshkol_hip_num_cus() &&
                      small_tile_us(small_tiles, nkb, may_cut) < large_tile_us(big_tiles, nkb, may_cut))))
        return Kernel::Fast64;
    if (straight && (big_tiles >= 192 || cut)) return Kernel::Fast128;
    return big_tiles >= 256 ? Kernel::General128 : Kernel::General64;
}

template <bool TA, bool TB>
int launch_shape(const double* A, const double* B, double* C, int m, int n, int k, int batch, bool vec,
                 hipStream_t st) {
    /* Row-major A next to a k-major B: writing A's tile k-major into LDS (so both
     * operands are read the same way) measured 1 % faster than keeping A's rows
     * at 8192^3; with both operands row-major the natural forms are faster. */
    constexpr bool ALK = TA || !TB;
    switch (choose_kernel(m, n, k, batch, vec)) {
        case Kernel::Fast64: return launch_fast64<TA, TB>(A, B, C, m, n, k, batch, st);
        case Kernel::Fast128: return launch_fast<TA, TB>(A, B, C, m, n, k, batch, st);
        case Kernel::General128:
            return vec ? launch<128, 128, true, TA, TB, ALK, !TB>(A, B, C, m, n, k, batch, st)
                       : launch<128, 128, false, TA, TB, TA, !TB>(A, B, C, m, n, k, batch, st);
        default:
            return vec ? launch<64, 64, true, TA, TB, TA, !TB>(A, B, C, m, n, k, batch, st)
                       : launch<64, 64, false, TA, TB, TA, !TB>(A, B, C, m, n, k, batch, st);
    }
}

/* dst[r][c] = src[r][c] for c < cols, 0 for cols <= c < ld: an operand whose rows do
 * not start on 16-byte boundaries (odd cols, or a base that is not aligned) copied
 * to an even pitch. One launch copies both operands of a product (blockIdx.z says
 * which); an operand that needs no copy comes with rows == 0. */
struct PadCopy { const double* src; double* dst; int rows, cols, ld; };
__global__ __launch_bounds__(256)
void dgemm_pad_copy_kernel(PadCopy a, PadCopy b) {
    const PadCopy& p = blockIdx.z == 0 ? a : b;
    const int c = (int)(blockIdx.x * 256 + threadIdx.x);
    if (c >= p.ld) return;
    for (int r = (int)blockIdx.y; r < p.rows; r += (int)gridDim.y)
        p.dst[(size_t)r * p.ld + c] = (c < p.cols) ? p.src[(size_t)r * p.cols + c] : 0.0;
}

}  // namespace

namespace {
int dgemm_any(const double* A, const double* B, double* C, uint64_t M, uint64_t K, uint64_t N,
              int trans_a, int trans_b, uint64_t batch, void* stream) {
    if (!A || !B || !C || M == 0 || K == 0 || N == 0 || batch == 0) return -1;
    if (M > 0x7fffffffULL || K > 0x7fffffffULL || N > 0x7fffffffULL) return -1;
    if (trans_a && trans_b) return -1;   /* no caller needs it: (B*A)^T, transpose the result instead */
    hipStream_t st = (hipStream_t)stream;
    /* row pitches: A is [M][K] or [K][M]; B is [K][N] or [N][K]. In a batch every
     * matrix must start on a 16-byte boundary as well. */
    const uint64_t pitch_a = trans_a ? M : K, pitch_b = trans_b ? K : N;
    const bool vec = (pitch_a % 2 == 0) && (pitch_b % 2 == 0) &&
                     ((uintptr_t)A % 16 == 0) && ((uintptr_t)B % 16 == 0) &&
                     (batch == 1 || ((M * K) % 2 == 0 && (K * N) % 2 == 0));
    const int m = (int)M, n = (int)N, k = (int)K;
    /* Shapes with kernels of their own; one that cannot run (no workspace to be had) leaves the
     * product to the tiled kernels below. */
    /* matrices far smaller than a tile, one or many: several to a workgroup (dgemm_small_f64.hip) */
    if (g_fast_path && eshkol_hip_dgemm_is_small(M, K, N) &&
        eshkol_hip_dgemm_small(A, B, C, M, K, N, trans_a, trans_b, batch, st) == 0) return 0;
    /* up to 64 rows (or columns) against a matrix: streamed through the matrix cores (dgemm_thin_f64.hip) */
    if (g_fast_path && batch == 1 && eshkol_hip_dgemm_is_thin_rows(M, K, N, trans_a, trans_b) &&
        eshkol_hip_dgemm_thin_rows(A, B, C, M, K, N, trans_a, trans_b, st) == 0) return 0;
    /* few outputs, a long k: slices of k over the workgroups */
    if (g_fast_path && batch == 1 && eshkol_hip_dgemm_is_small_long_k(M, K, N) &&
        eshkol_hip_dgemm_small_long_k(A, B, C, M, K, N, trans_a, trans_b, st) == 0) return 0;
    /* a vector against a matrix with k contiguous: plain fma loops at the rate of HBM (dgemv_f64.hip) */
    if (g_fast_path && batch == 1 && eshkol_hip_dgemm_is_matvec(M, K, N, trans_a, trans_b) &&
        eshkol_hip_dgemm_matvec(A, B, C, M, K, N, trans_a, trans_b, st) == 0) return 0;
    /* Operands whose rows do not start on 16-byte boundaries (an odd pitch, a base that
     * is not aligned) would take the kernel of 8-byte loads, at two thirds of the rate
     * (4096 x 4096 x 4097: 3.0 ms against 2.1). Where the shape would otherwise run the
     * straight-line kernel and is large enough (20 MFLOP: some ten microseconds in the other kernel) for
     * another launch and two passes over an operand not to matter, or has a k long enough
     * to want cutting (only that kernel's launches are cut along k), the operand is copied to an even pitch first and the kernel told the
     * pitch; the k-tail and edge logic work on the logical sizes as before, and a pair
     * of values that straddles the end of a row ends in the copy's zero. C needs no
     * copy: the kernel stores it value by value. */
    if (!vec && batch == 1 && (2.0 * (double)M * (double)N * (double)K >= 2.0e7 || K >= 512)) {
        const Kernel would = choose_kernel(m, n, k, 1, true);
        if (would == Kernel::Fast64 || would == Kernel::Fast128) {
            const int rows_a = trans_a ? k : m, rows_b = trans_b ? n : k;
            const bool copy_a = (pitch_a % 2 != 0) || ((uintptr_t)A % 16 != 0);
            const bool copy_b = (pitch_b % 2 != 0) || ((uintptr_t)B % 16 != 0);
            const int lda = (int)(pitch_a + (pitch_a & 1)), ldb = (int)(pitch_b + (pitch_b & 1));
            const double* a2 = A;
            const double* b2 = B;
            bool ok = pitch_a < 0x7fffffffULL && pitch_b < 0x7fffffffULL;
            PadCopy ca = {A, nullptr, 0, (int)pitch_a, lda}, cb = {B, nullptr, 0, (int)pitch_b, ldb};
            if (ok && copy_a) {
                ca.dst = (double*)eshkol_hip_workspace(WS_DGEMM_PAD_A, (size_t)rows_a * lda * sizeof(double));
                ca.rows = rows_a;
                if (ca.dst) a2 = ca.dst; else ok = false;
            }
            if (ok && copy_b) {
                cb.dst = (double*)eshkol_hip_workspace(WS_DGEMM_PAD_B, (size_t)rows_b * ldb * sizeof(double));
                cb.rows = rows_b;
                if (cb.dst) b2 = cb.dst; else ok = false;
            }
            if (ok) {
                const int wide = (copy_a && (!copy_b || lda > ldb)) ? lda : ldb;
                const int tall = (ca.rows > cb.rows) ? ca.rows : cb.rows;
                hipLaunchKernelGGL(dgemm_pad_copy_kernel, dim3((unsigned)((wide + 255) / 256), (unsigned)(tall < 65535 ? tall : 65535), 2),
                                   dim3(256), 0, st, ca, cb);
            }
            if (ok) {
                g_lda = copy_a ? lda : 0;
                g_ldb = copy_b ? ldb : 0;
                int rc;
                if (trans_a) rc = launch_shape<true, false>(a2, b2, C, m, n, k, 1, true, st);
                else if (trans_b) rc = launch_shape<false, true>(a2, b2, C, m, n, k, 1, true, st);
                else rc = launch_shape<false, false>(a2, b2, C, m, n, k, 1, true, st);
                g_lda = 0; g_ldb = 0;
                return rc;
            }
        }
    }
    /* the grid's y extent is limited to 65535 */
    for (uint64_t done = 0; done < batch; ) {
        const int nb = (int)((batch - done < 65535) ? batch - done : 65535);
        const double* a = A + done * M * K;
        const double* b = B + done * K * N;
        double* c = C + done * M * N;
        int rc;
        if (trans_a) rc = launch_shape<true, false>(a, b, c, m, n, k, nb, vec, st);
        else if (trans_b) rc = launch_shape<false, true>(a, b, c, m, n, k, nb, vec, st);
        else rc = launch_shape<false, false>(a, b, c, m, n, k, nb, vec, st);
        if (rc != 0) return rc;
        done += (uint64_t)nb;
    }
    return 0;
}
}  // namespace

/* 0 routes every shape through the bounds-checked kernel (for comparisons). */
extern "C" void hip_dgemm_set_fast_path(int on) { EshkolHipLock lk; g_fast_path = on ? 1 : 0; }
/* 0 keeps every tile whole (results then equal the bounds-checked kernel's bit for bit). */
extern "C" void hip_dgemm_set_tail_split(int on) { EshkolHipLock lk; g_tail_split = on ? 1 : 0; }
/* 0: the straight-line kernel uses 128 x 128 tiles only; 1 (default): 64 x 64 tiles where
 * they measure faster; 2: 64 x 64 tiles wherever the straight-line kernel applies. */
extern "C" void hip_dgemm_set_prefetch_depth(int depth) { EshkolHipLock lk; g_prefetch_depth = (depth == 1 || depth == 2) ? depth : 0; }
extern "C" void hip_dgemm_set_small_tile(int mode) { EshkolHipLock lk; if (mode >= 0 && mode <= 2) g_small_tile = mode; }

extern "C" int hip_dgemm_f64_ex(const double* A, const double* B, double* C,
                                uint64_t M, uint64_t K, uint64_t N,
                                int trans_a, int trans_b, void* stream) {
    EshkolHipCall bracket(stream);
    return dgemm_any(A, B, C, M, K, N, trans_a, trans_b, 1, stream);
}

extern "C" int hip_dgemm_f64(const double* A, const double* B, double* C,
                             uint64_t M, uint64_t K, uint64_t N, void* stream) {
    EshkolHipCall bracket(stream);
    return dgemm_any(A, B, C, M, K, N, 0, 0, 1, stream);
}

extern "C" int hip_dgemm_f64_batched(const double* A, const double* B, double* C,
                                     uint64_t batch, uint64_t M, uint64_t K, uint64_t N, void* stream) {
    EshkolHipCall bracket(stream);
    return dgemm_any(A, B, C, M, K, N, 0, 0, batch, stream);
}
