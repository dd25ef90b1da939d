/*
 * Software-pipelined main loop shared by the int8 and the 16-bit matrix-core
 * GEMMs. Both move K-contiguous operand rows as bytes: a k-step of one 32x32
 * MFMA consumes 32 bytes of each operand row (32 int8 or 16 half/bf16 values),
 * 16 bytes per lane, so the data path is identical and only the MFMA differs.
 *
 *   block      256 threads = 2x2 waves; wave tile (TM*32) x (TN*32); k-block of
 *              128 bytes = 4 k-steps, so every global row segment is a whole
 *              128-byte line
 *   global     a register ring of PF k-blocks in flight: block g+1+PF is
 *              requested during the last two k-steps of block g (A's rows in
 *              the third, B's in the fourth: sixteen requests in one k-step
 *              queue up behind the address unit), into the ring slot the
 *              second k-step has just emptied. The ring, not occupancy, hides
 *              the ~1.3 us a miss takes: the accumulators leave room for one
 *              wave per SIMD only.
 *   LDS        two buffers, each [A rows][128(+16)] then [B rows][128(+16)]
 *              bytes; block g+1 is written during the second k-step of block g
 *   fragments  double-buffered: the 16-byte LDS reads of k-step s+1 are issued
 *              between the MFMAs of k-step s (sched_group_barrier pins that
 *              interleaving; left alone the scheduler sinks each read next to
 *              its use and waits for it)
 *   barrier    one per k-block, LDS-only (s_waitcnt lgkmcnt(0); s_barrier): a
 *              full __syncthreads would also wait for the prefetched global
 *              loads and undo the ring
 *
 * The loop body is branch-free (prefetches past the end of the last tile are
 * clamped to its last block and never consumed), so it is one scheduling region.
 */
#ifndef ESHKOL_HIP_GEMM_PIPE_H
#define ESHKOL_HIP_GEMM_PIPE_H

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace pipe {

typedef int v4i_t __attribute__((ext_vector_type(4)));

constexpr int BKB = 128;                /* bytes of K per block */
constexpr int PITCH = BKB + 16;         /* LDS row pitch: 16 consecutive rows hit 64 distinct banks */
constexpr int NKS = BKB / 32;
constexpr int MAX_PAIRS = 64;

template <int TM, int TN> struct Cfg {
    static constexpr int NT = 256;
    static constexpr int BM = 2 * TM * 32;
    static constexpr int BN = 2 * TN * 32;
    static constexpr int A_TILE = BM * PITCH;
    static constexpr int B_TILE = BN * PITCH;
    static constexpr int TABLE_BYTES = 2 * MAX_PAIRS * 4;
    static constexpr int SMEM_MAIN = 2 * (A_TILE + B_TILE) + TABLE_BYTES;
    static constexpr int A_CH = BM * BKB / 16 / NT;      /* 16-byte chunks per thread per block */
    static constexpr int B_CH = BN * BKB / 16 / NT;
};

template <int V> using IC = std::integral_constant<int, V>;

template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

/* Buffer descriptor of the 256 plane rows that start at `rows` (wave-uniform):
 * untyped, no stride, so a load's address is rows + the lane's 32-bit offset +
 * a scalar offset, and none of it is vector arithmetic. */
__device__ __forceinline__ __amdgpu_buffer_rsrc_t plane_rsrc(const int8_t* rows) {
    return __builtin_amdgcn_make_buffer_rsrc((void*)rows, 0, 0x7fffffff, 0x00020000);
}

__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

/* The operand planes a launch multiplies: every plane is [rows][ld] bytes. */
struct Source {
    const int8_t* a_planes;
    const int8_t* b_planes;
    uint64_t a_plane_stride, b_plane_stride;
    int ld;                     /* bytes per row, multiple of BKB*PF */
};

/* ---- several tiles per workgroup ------------------------------------------------
 * The same main loop for a workgroup that walks a list of output tiles. The
 * stream of k-blocks is continuous across tiles: when the request cursor runs
 * past the last block of a tile it moves on to the first blocks of the next
 * one, so those loads are in flight while the tile's epilogue runs and the
 * next tile starts with its operands already in registers. What a workgroup
 * launch costs (dispatch, cold first loads, a drained pipe) is paid once.
 * The cursor runs PF + 1 blocks ahead and the tile after the current one is
 * always known; every tile must have at least max(2 PF, PF + 2) k-blocks so
 * that the cursor has left a tile's index table before the table of the tile
 * after the next replaces it. A tile's first block reaches LDS buffer 0 during
 * the last block of the tile before it, so an epilogue that needs LDS takes
 * buffer 1 (epilogue_stage). */
struct Tile {
    int m0, n0;                 /* first row of the A planes / of the B planes */
    int tag;                    /* caller's: output plane */
    const int32_t* a_idx;       /* plane indices of the tile's products (device memory), or NULL: */
    const int32_t* b_idx;
    int npairs;                 /* >= 1 */
    int a_plane0 = 0;           /* the one plane a list-less tile multiplies (run_tiles of gemm_pipe2.h only) */
    int b_plane0 = 0;
};

template <int TM, int TN> struct TilesCfg {
    static constexpr int SMEM_MAIN = Cfg<TM, TN>::SMEM_MAIN + Cfg<TM, TN>::TABLE_BYTES;   /* two index tables */
};

/* next_tile(Tile&) -> bool hands out this workgroup's tiles in order;
 * epilogue(acc, tile) consumes a finished accumulator (LDS buffer 1 is free for
 * it, buffer 0 is not). A launch of single tiles needs one index table only:
 * the second half of `table` is written when a next tile exists. */
template <class Op, int TM, int TN, int PF, class Next, class Epi>
__device__ __forceinline__ void run_tiles(int8_t* smem, const Source& cm, Next next_tile, Epi epilogue) {
    using C = Cfg<TM, TN>;
    constexpr int BUF = C::A_TILE + C::B_TILE;                            /* LDS: [A0][B0][A1][B1][tables] */
    int32_t* table = (int32_t*)(smem + 2 * BUF);                          /* [2][2 * MAX_PAIRS] */

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 31, lh = lane >> 5;

    const int nkb_per = cm.ld / BKB;
    /* A thread's chunks of a k-block: rows tid/8 + 32 r, bytes 16 (tid%8) of the
     * 128. Kept as 32-bit offsets from a wave-uniform block address, so the
     * loads take their base from scalar registers and the cursor is scalar work. */
    uint32_t voff[(C::A_CH > C::B_CH) ? C::A_CH : C::B_CH];
#pragma unroll
    for (int r = 0; r < ((C::A_CH > C::B_CH) ? C::A_CH : C::B_CH); r++)
        voff[r] = (uint32_t)((tid >> 3) + 32 * r) * (uint32_t)cm.ld + (uint32_t)(tid & 7) * 16u;
    const int s_off = (tid >> 3) * PITCH + (tid & 7) * 16;

    /* The current tile and the one after it: the request cursor may cross into the
     * next tile at any time, so that tile is always known one tile ahead. */
    Tile cur, nxt;
    if (!next_tile(cur)) return;
    int tab = 0;                                   /* table half that describes `cur` */
    if (tid < cur.npairs) {
        table[tid] = cur.a_idx ? cur.a_idx[tid] : 0;
        table[MAX_PAIRS + tid] = cur.b_idx ? cur.b_idx[tid] : 0;
    }
    const int8_t* nx_a = nullptr;
    const int8_t* nx_b = nullptr;
    int nx_np = 1;
    bool nx_has = false;
    auto learn_next = [&]() {
        nx_has = next_tile(nxt);
        if (nx_has) {
            if (tid < nxt.npairs) {
                table[(tab ^ 1) * 2 * MAX_PAIRS + tid] = nxt.a_idx ? nxt.a_idx[tid] : 0;
                table[(tab ^ 1) * 2 * MAX_PAIRS + MAX_PAIRS + tid] = nxt.b_idx ? nxt.b_idx[tid] : 0;
            }
            nx_a = cm.a_planes + (size_t)nxt.m0 * cm.ld;
            nx_b = cm.b_planes + (size_t)nxt.n0 * cm.ld;
            nx_np = nxt.npairs;
        }
    };
    learn_next();
    __syncthreads();

    /* request cursor */
    const int8_t* a_t = cm.a_planes + (size_t)cur.m0 * cm.ld;
    const int8_t* b_t = cm.b_planes + (size_t)cur.n0 * cm.ld;
    int gl_t = 0, gl_j = 0, gl_np = cur.npairs, gl_tab = 0;
    int v_ia = table[0], v_ib = table[MAX_PAIRS];

    v4i_t ra[PF][C::A_CH], rb[PF][C::B_CH];
    /* One k-block is requested in two halves, A's rows and then B's, in two
     * consecutive k-steps; the cursor moves on after the second. */
    auto gload_a = [&](auto slot) {
        constexpr int S = decltype(slot)::value;
        const int ia = __builtin_amdgcn_readfirstlane(v_ia);
        const __amdgpu_buffer_rsrc_t rs = plane_rsrc(a_t + (size_t)ia * cm.a_plane_stride);
        const int soff = gl_j * BKB;
#pragma unroll
        for (int r = 0; r < C::A_CH; r++) ra[S][r] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff[r], soff, 0);
    };
    auto gload_b = [&](auto slot) {
        constexpr int S = decltype(slot)::value;
        const int ib = __builtin_amdgcn_readfirstlane(v_ib);
        const __amdgpu_buffer_rsrc_t rs = plane_rsrc(b_t + (size_t)ib * cm.b_plane_stride);
        const int soff = gl_j * BKB;
#pragma unroll
        for (int r = 0; r < C::B_CH; r++) rb[S][r] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff[r], soff, 0);
        /* advance: next k-block, next product, next tile; with no next tile the
         * cursor stays on the last block (those requests are never consumed) */
        const int nj = gl_j + 1;
        const bool wrap = (nj == nkb_per);
        const bool last = wrap && (gl_t + 1 == gl_np);
        const bool hop = last && nx_has;
        gl_j = hop ? 0 : (last ? gl_j : (wrap ? 0 : nj));
        gl_t = hop ? 0 : ((wrap && !last) ? gl_t + 1 : gl_t);
        a_t = hop ? nx_a : a_t;
        b_t = hop ? nx_b : b_t;
        gl_np = hop ? nx_np : gl_np;
        gl_tab = hop ? (gl_tab ^ 1) : gl_tab;
        v_ia = table[gl_tab * 2 * MAX_PAIRS + gl_t];
        v_ib = table[gl_tab * 2 * MAX_PAIRS + MAX_PAIRS + gl_t];
    };
    auto sstore = [&](int buf, auto slot) {
        constexpr int S = decltype(slot)::value;
        int8_t* ad = smem + buf * BUF + s_off;
        int8_t* bd = ad + C::A_TILE;
#pragma unroll
        for (int r = 0; r < C::A_CH; r++) *(v4i_t*)(ad + 32 * r * PITCH) = ra[S][r];
#pragma unroll
        for (int r = 0; r < C::B_CH; r++) *(v4i_t*)(bd + 32 * r * PITCH) = rb[S][r];
    };

    v4i_t fa[2][TM], fb[2][TN];
    const int a_frag_off = (wm * TM * 32 + li) * PITCH + lh * 16;
    const int b_frag_off = C::A_TILE + (wn * TN * 32 + li) * PITCH + lh * 16;
    typename Op::acc_t acc[TM][TN];
    auto ldfrag = [&](int buf, int ks, auto which) {
        constexpr int W = decltype(which)::value;
        const int8_t* ab = smem + buf * BUF + a_frag_off + ks * 32;
        const int8_t* bb = smem + buf * BUF + b_frag_off + ks * 32;
#pragma unroll
        for (int t = 0; t < TM; t++) fa[W][t] = *(const v4i_t*)(ab + t * 32 * PITCH);
#pragma unroll
        for (int u = 0; u < TN; u++) fb[W][u] = *(const v4i_t*)(bb + u * 32 * PITCH);
    };
    auto mfma_all = [&](auto which) {
        constexpr int W = decltype(which)::value;
#pragma unroll
        for (int t = 0; t < TM; t++)
#pragma unroll
            for (int u = 0; u < TN; u++) Op::mfma(fb[W][u], fa[W][t], acc[t][u]);
    };
    using I0 = IC<0>;
    using I1 = IC<1>;
    constexpr int NM = TM * TN, NF = TM + TN;

    /* Start of the stream: block 0 into LDS buffer 0, blocks 1..PF into the ring
     * (block j in slot j % PF). Every later tile finds the same state: its block
     * 0 was written to buffer 0 during the last block of the tile before it. */
    static_for<PF>([&](auto s) { gload_a(s); gload_b(s); });
    sstore(0, I0{});
    gload_a(I0{});
    gload_b(I0{});

    for (;;) {
#pragma unroll
        for (int t = 0; t < TM; t++)
#pragma unroll
            for (int u = 0; u < TN; u++) Op::zero(acc[t][u]);

        const int nkb = cur.npairs * nkb_per;      /* even: the row pitch is a multiple of 2 * BKB */
        lds_barrier();                             /* block 0 and the parked table are visible */
        ldfrag(0, 0, I0{});

        for (int g0 = 0; g0 < nkb; g0 += PF) {
            static_for<PF>([&](auto s) {
                constexpr int S = decltype(s)::value;
                using NextSlot = IC<(S + 1) % PF>;           /* holds block g+1, then block g+1+PF */
                const int cb = (g0 + S) & 1;

                ldfrag(cb, 1, I1{});
                mfma_all(I0{});
#pragma unroll
                for (int i = 0; i < NM; i++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if (i < NF) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
                __builtin_amdgcn_sched_barrier(0);

                ldfrag(cb, 2, I0{});
                sstore(cb ^ 1, NextSlot{});
                mfma_all(I1{});
#pragma unroll
                for (int i = 0; i < NM; i++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if (i < NF) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    if (i < C::A_CH + C::B_CH) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                }
                __builtin_amdgcn_sched_barrier(0);

                ldfrag(cb, 3, I1{});
                gload_a(NextSlot{});
                mfma_all(I0{});
#pragma unroll
                for (int i = 0; i < NM; i++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if (i < NF) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    if (i >= NF && i - NF < C::A_CH) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                lds_barrier();

                ldfrag(cb ^ 1, 0, I0{});
                gload_b(NextSlot{});
                mfma_all(I1{});
#pragma unroll
                for (int i = 0; i < NM; i++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if (i < NF) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    if (i >= NF && i - NF < C::B_CH) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        }
        lds_barrier();                 /* every wave is done with LDS buffer 1 */
        epilogue(acc, cur);            /* may stage in buffer 1 (epilogue_stage): buffer 0 holds the next tile's block 0 */
        if (!nx_has) break;
        cur = nxt;
        tab ^= 1;
        learn_next();                  /* parks the table in the half the cursor has left behind */
    }
}

/* LDS an epilogue may use while the stream continues: the second operand buffer. */
template <int TM, int TN>
__device__ __forceinline__ int8_t* epilogue_stage(int8_t* smem) {
    return smem + Cfg<TM, TN>::A_TILE + Cfg<TM, TN>::B_TILE;
}
template <int TM, int TN> struct StageCfg {
    static constexpr int BYTES = Cfg<TM, TN>::A_TILE + Cfg<TM, TN>::B_TILE;
};

}  // namespace pipe
#endif
