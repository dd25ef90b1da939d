/*
 * Main loop of the int8 and 16-bit matrix-core GEMMs for operand planes stored
 * fragment-major ("interleaved"), with no operand staged through registers.
 *
 * Plane layout. Rows come in blocks of 32; inside a block the 16-byte k-chunks
 * are the slow index and the row the fast one:
 *     offset(row, k) = (row / 32) * 32 * ld + (k / 16) * 512 + (row % 32) * 16 + k % 16
 * so the operand fragment of one 32x32 MFMA k-step (32 rows x 32 bytes of k, a
 * lane holding 16 bytes of row lane%32, k-half lane/32) is 1 KiB of contiguous
 * memory read as base + 16 * lane. Both operands use it; which k a lane feeds
 * does not matter as long as both agree.
 *
 *   block      256 threads = 4 waves stacked along M; wave tile 64 x 256 (2 x 8
 *              MFMA tiles, 256 accumulator registers); block tile 256 x 256;
 *              k-block of 128 bytes = 4 k-steps
 *   A          private to a wave: its fragments go straight from global memory
 *              into MFMA operand registers as coalesced 1 KiB loads, through a
 *              ring of DEPTH k-blocks (no LDS traffic at all for this operand)
 *   B          shared by the four waves: buffer_load ... lds moves it from
 *              global memory into a ring of DEPTH LDS stages of 32 KiB without
 *              touching registers; a stage is [col-block 8][k-step 4][1 KiB], so
 *              a fragment read is 16 * lane again, conflict-free without padding
 *   depth      k-block b+DEPTH is requested while block b is multiplied: every
 *              load has more than two k-blocks of MFMA time to land, where a
 *              register-staged tile has one and a half
 *   counters   all loads of the loop are issued from inline assembly, so the
 *              compiler's own wait-count bookkeeping does not see them (it would
 *              make every LDS read wait for every earlier load to LDS). One
 *              s_waitcnt vmcnt per k-block, just before the block's barrier,
 *              covers everything the next block needs; the count is fixed by
 *              the issue order below (loads return in issue order).
 *   barrier    one per k-block, after the third k-step: behind it the stage the
 *              block used is free (every wave holds its last fragments in
 *              registers) and the next block's stage is complete
 *
 * Issue order of block b, slot S = b % DEPTH, cursor = the block DEPTH ahead:
 *   k-step 0   A(cursor)(k-step 3) -> slot S-1, then the cursor advances   2 loads
 *   k-step 1   A(cursor)(k-step 0) -> slot S                               2
 *   k-step 2   A(cursor)(k-step 1) -> slot S; wait; barrier                2
 *   k-step 3   A(cursor)(k-step 2) -> slot S; B(cursor) -> stage S         2 + 8
 * A register of slot S is overwritten one k-step after the MFMAs that read it
 * have been issued. At the wait of block b the youngest load block b+1 needs is
 * A(b+1)(k-step 3), issued in k-step 0 of block b-2; 14 + 16 + 6 = 36 loads
 * follow it.
 *
 * The stream of k-blocks is continuous across the tiles a workgroup walks: the
 * cursor moves on to the next tile's first blocks while the current tile is
 * still being multiplied, and they land during its epilogue. Every tile needs a
 * multiple of DEPTH k-blocks (row pitch a multiple of 512 bytes), so the cursor,
 * DEPTH blocks ahead, is never more than one tile ahead.
 */
#ifndef ESHKOL_HIP_GEMM_PIPE2_H
#define ESHKOL_HIP_GEMM_PIPE2_H

#include <hip/hip_runtime.h>
#include <stdint.h>
#include "gemm_pipe.h"

namespace pipe2 {

typedef int v2i_t __attribute__((ext_vector_type(2)));

using pipe::v4i_t;
using pipe::IC;
using pipe::static_for;
using pipe::Source;
using pipe::Tile;

constexpr int BKB = 128;
constexpr int DEPTH = 4;
constexpr int TM = 2, TN = 8;
constexpr int BM = 256, BN = 256;
constexpr int FRAG = 1024;
constexpr int STAGE = BN * BKB;                       /* 32 KiB of B per k-block */
constexpr int RING = DEPTH * STAGE;
constexpr int EPI_PITCH = 128 + 16;
constexpr int EPI_WAVE_BYTES = 32 * EPI_PITCH;        /* per wave: 32 rows x 128 output bytes */
constexpr int SMEM_BYTES = RING + 4 * EPI_WAVE_BYTES;

/* A 32 x 32 block of 4-byte words on its way out of a wave. The 32x32 MFMAs
 * leave it transposed: lane l holds row l % 32, and its registers 4v .. 4v+3 the
 * columns 8v + 4 (l / 32) + 0..3, so a store straight from the registers would
 * put 16 bytes into each of 64 places. park_block() writes the block into the
 * wave's LDS stage as rows of 128 bytes (pitch EPI_PITCH: the 16-byte accesses of
 * eight lanes, in either direction, fall into distinct banks); afterwards eight
 * lanes read a row and a store instruction writes whole 128-byte lines. The
 * wave's LDS accesses complete in order: its reads see its writes, and the next
 * block's writes come after this block's reads. */
__device__ __forceinline__ void park_block(int8_t* stage, int v, v4i_t words) {
    const int lane = threadIdx.x & 63;
    *(v4i_t*)(stage + (lane & 31) * EPI_PITCH + 32 * v + 16 * (lane >> 5)) = words;
}
/* i = 0..3: the 16 bytes of row lane/8 + 8 i, words 4 (lane % 8) .. + 3 */
__device__ __forceinline__ v4i_t parked_row16(const int8_t* stage, int i) {
    const int lane = threadIdx.x & 63;
    return *(const v4i_t*)(stage + ((lane >> 3) + 8 * i) * EPI_PITCH + 16 * (lane & 7));
}
/* i = 0..7: the 8 bytes of row lane/16 + 4 i, words 2 (lane % 16), + 1 */
__device__ __forceinline__ v2i_t parked_row8(const int8_t* stage, int i) {
    const int lane = threadIdx.x & 63;
    return *(const v2i_t*)(stage + ((lane >> 4) + 4 * i) * EPI_PITCH + 8 * (lane & 15));
}
constexpr int WAIT_STEADY = 36;                       /* see the issue order above */
constexpr int WAIT_START = 3 * 16 + 8 + 6 - 16;       /* after the prologue: all but block 0's loads may be pending */

/* untyped buffer descriptor on a wave-uniform address, as four scalar words */
__device__ __forceinline__ v4i_t rsrc_words(const void* p) {
    const uint64_t a = (uint64_t)p;
    v4i_t r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((a >> 32) & 0xffffu));
    r[2] = 0x7fffffff;
    r[3] = 0x00020000;
    return r;
}

/* 16 bytes per lane from global memory into registers; the data arrives later,
 * behind the compiler's back: nothing may read dst before wait_loads. */
template <int IMM>
__device__ __forceinline__ void load_hidden(v4i_t& dst, const v4i_t& rs, uint32_t voff, uint32_t soff) {
    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4"
                 : "=v"(dst) : "v"(voff), "s"(rs), "s"(soff), "n"(IMM));
}

/* 16 bytes per lane from global memory to LDS address lds + IMM + 16 * lane */
template <int IMM>
__device__ __forceinline__ void load_to_lds(uint32_t lds, const v4i_t& rs, uint32_t voff, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen offset:%4 lds"
                 :: "s"(lds), "v"(voff), "s"(rs), "s"(soff), "n"(IMM) : "memory", "m0");
}

/* at most N loads still pending; the eight registers are the A fragments of the
 * slot that becomes readable (the operands tie the wait to their first use) */
template <int N>
__device__ __forceinline__ void wait_loads(v4i_t (&slot)[TM][4]) {
    asm volatile("s_waitcnt vmcnt(%8)"
                 : "+v"(slot[0][0]), "+v"(slot[0][1]), "+v"(slot[0][2]), "+v"(slot[0][3]),
                   "+v"(slot[1][0]), "+v"(slot[1][1]), "+v"(slot[1][2]), "+v"(slot[1][3])
                 : "n"(N));
}

__device__ __forceinline__ void drain_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

/* One word from a wave-uniform address through the scalar cache. A vector load
 * here would make the compiler wait for vmcnt(0), which drains every request the
 * pipeline has in flight. For tables the launch does not write. */
__device__ __forceinline__ int32_t scalar_load(const int32_t* p) {
    const uint64_t a = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32));
    const uint64_t u = ((uint64_t)hi << 32) | lo;
    int32_t v;
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(u) : "memory");
    return v;
}

/* next_tile(Tile&) -> bool hands out this workgroup's tiles in order;
 * epilogue(acc, tile, stage) consumes a finished accumulator: acc[t][u] is the
 * transposed 32x32 tile of rows m0 + 64 wave + 32 t, columns n0 + 32 u; stage is
 * EPI_WAVE_BYTES of LDS private to the wave. */
template <class Op, class Next, class Epi>
__device__ __forceinline__ void run_tiles(int8_t* smem, const Source& cm, Next next_tile, Epi epilogue) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t rb_stride = 32u * (uint32_t)cm.ld;                       /* bytes per 32-row block of a plane */
    const int nkb_per = cm.ld / BKB;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) int8_t*)smem;
    const uint32_t voff[2] = { (uint32_t)lane * 16u, (uint32_t)lane * 16u + rb_stride };
    int8_t* epi_stage = smem + RING + wave * EPI_WAVE_BYTES;

    /* The current tile and the one after it: the request cursor crosses into the
     * next tile while the current one is still being multiplied. */
    Tile cur, nxt;
    if (!next_tile(cur)) return;
    bool nx_has = next_tile(nxt);
    /* a wave's share of a tile: its 64 rows of A, its 64 of the 256 rows of B it stages */
    auto wave_rows_a = [&](const Tile& t) { return cm.a_planes + (size_t)(t.m0 / 32 + 2 * wave) * rb_stride; };
    auto wave_rows_b = [&](const Tile& t) { return cm.b_planes + (size_t)(t.n0 / 32 + 2 * wave) * rb_stride; };

    /* request cursor: tile, product within the tile, k-block within the product.
     * A tile's plane indices are read from its lists when the cursor reaches a
     * product (scalar loads: once per product, not per k-block). */
    const int8_t* c_a = wave_rows_a(cur);
    const int8_t* c_b = wave_rows_b(cur);
    const int32_t* c_ai = cur.a_idx;
    const int32_t* c_bi = cur.b_idx;
    int c_pa = cur.a_plane0, c_pb = cur.b_plane0;
    int c_t = 0, c_j = 0, c_np = cur.npairs;
    bool c_in_next = false;                     /* the cursor has crossed into nxt */
    v4i_t rs_a, rs_b;
    auto point_at_product = [&]() {
        const int ia = c_ai ? scalar_load(c_ai + c_t) : c_pa;
        const int ib = c_bi ? scalar_load(c_bi + c_t) : c_pb;
        rs_a = rsrc_words(c_a + (size_t)ia * cm.a_plane_stride);
        rs_b = rsrc_words(c_b + (size_t)ib * cm.b_plane_stride);
    };
    point_at_product();
    uint32_t c_soff = 0;
    auto advance = [&]() {
        const int nj = c_j + 1;
        if (nj != nkb_per) { c_j = nj; c_soff = (uint32_t)nj * (uint32_t)(4 * FRAG); return; }
        /* end of a product */
        if (c_t + 1 < c_np) {
            c_t++; c_j = 0; c_soff = 0;
            point_at_product();
        } else if (nx_has && !c_in_next) {
            c_in_next = true;
            c_a = wave_rows_a(nxt); c_b = wave_rows_b(nxt);
            c_ai = nxt.a_idx; c_bi = nxt.b_idx; c_np = nxt.npairs;
            c_pa = nxt.a_plane0; c_pb = nxt.b_plane0;
            c_t = 0; c_j = 0; c_soff = 0;
            point_at_product();
        }
        /* else: no tile to move on to (or the tile after the next is not known
         * yet, which the minimum tile length excludes): the cursor stays on the
         * last block, whose repeated requests are never consumed */
    };

    v4i_t ra[DEPTH][TM][4];                     /* A fragments: [slot][row block][k-step] */
    v4i_t fb[2][TN];                            /* B fragments of the current and the next k-step */
    typename Op::acc_t acc[TM][TN];

    auto issue_a = [&](auto slot, auto kstep) {
        constexpr int S = decltype(slot)::value, KS = decltype(kstep)::value;
        load_hidden<KS * FRAG>(ra[S][0][KS], rs_a, voff[0], c_soff);
        load_hidden<KS * FRAG>(ra[S][1][KS], rs_a, voff[1], c_soff);
    };
    auto issue_b_one = [&](auto stage, auto which) {
        constexpr int S = decltype(stage)::value, J = decltype(which)::value / 4, KS = decltype(which)::value % 4;
        const uint32_t dst = lds_base + (uint32_t)(S * STAGE) + (uint32_t)(2 * wave + J) * (uint32_t)(4 * FRAG);
        load_to_lds<KS * FRAG>(dst, rs_b, voff[J], c_soff);
    };
    using I0 = IC<0>;
    using I1 = IC<1>;

    /* One k-step: sixteen MFMAs on the fragments fb[W] and slot S's A fragments of
     * k-step KS, with one memory operation after each (a wave has a single
     * instruction stream: what is not placed between two MFMAs is issued while
     * the matrix pipe runs dry). After MFMA i < 8 the B fragment i of the next
     * k-step (LDS stage nstage, k-step nks) is read into fb[W ^ 1]; after MFMA
     * 8 ... 15 comes mem(i - 8). The order is pinned: nothing crosses a
     * sched_barrier(0). */
    auto kstep = [&](auto which, auto slot, auto kstep_c, int nstage, int nks, auto mem, auto fresh) {
        constexpr int W = decltype(which)::value, S = decltype(slot)::value, KS = decltype(kstep_c)::value;
        constexpr bool FRESH = decltype(fresh)::value != 0;
        const int8_t* nb = smem + nstage * STAGE + nks * FRAG + lane * 16;
        static_for<TM * TN>([&](auto idx) {
            constexpr int I = decltype(idx)::value, T = I / TN, U = I % TN;
            if constexpr (FRESH) Op::mfma_first(fb[W][U], ra[S][T][KS], acc[T][U]);
            else Op::mfma(fb[W][U], ra[S][T][KS], acc[T][U]);
            if constexpr (I < TN) fb[W ^ 1][I] = *(const v4i_t*)(nb + I * 4 * FRAG);
            else mem(IC<I - TN>{});
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    /* Start of the stream: blocks 0, 1, 2 whole, block 3 without its last A k-step
     * (the first block's k-step 0 requests it), 62 loads in all. */
    static_for<DEPTH - 1>([&](auto s) {
        static_for<8>([&](auto w) { issue_b_one(s, w); });
        static_for<4>([&](auto ks) { issue_a(s, ks); });
        advance();
    });
    static_for<8>([&](auto w) { issue_b_one(IC<DEPTH - 1>{}, w); });
    static_for<3>([&](auto ks) { issue_a(IC<DEPTH - 1>{}, ks); });
    wait_loads<WAIT_START>(ra[0]);
    bool first_tile = true;

    /* DEPTH k-blocks. In a tile's first group the sixteen sums start with their
     * first product (the instruction adds it to the constant 0): no accumulator
     * is cleared, which would be 256 instructions per tile with the matrix pipe idle. */
    auto group = [&](auto first_of_tile) {
        constexpr int FIRST = decltype(first_of_tile)::value;
        static_for<DEPTH>([&](auto s) {
            constexpr int S = decltype(s)::value;
            constexpr int SP = (S + DEPTH - 1) % DEPTH, SN = (S + 1) % DEPTH;

            kstep(I0{}, IC<S>{}, IC<0>{}, S, 1, [&](auto m) {
                constexpr int Mi = decltype(m)::value;
                if constexpr (Mi == 0) load_hidden<3 * FRAG>(ra[SP][0][3], rs_a, voff[0], c_soff);
                if constexpr (Mi == 1) load_hidden<3 * FRAG>(ra[SP][1][3], rs_a, voff[1], c_soff);
                if constexpr (Mi == 2) advance();
            }, IC<(FIRST && S == 0) ? 1 : 0>{});
            kstep(I1{}, IC<S>{}, IC<1>{}, S, 2, [&](auto m) {
                constexpr int Mi = decltype(m)::value;
                if constexpr (Mi == 0) load_hidden<0>(ra[S][0][0], rs_a, voff[0], c_soff);
                if constexpr (Mi == 1) load_hidden<0>(ra[S][1][0], rs_a, voff[1], c_soff);
            }, I0{});
            kstep(I0{}, IC<S>{}, IC<2>{}, S, 3, [&](auto m) {
                constexpr int Mi = decltype(m)::value;
                if constexpr (Mi == 0) load_hidden<FRAG>(ra[S][0][1], rs_a, voff[0], c_soff);
                if constexpr (Mi == 1) load_hidden<FRAG>(ra[S][1][1], rs_a, voff[1], c_soff);
            }, I0{});
            wait_loads<WAIT_STEADY>(ra[SN]);
            pipe::lds_barrier();
            kstep(I1{}, IC<S>{}, IC<3>{}, SN, 0, [&](auto m) {
                constexpr int Mi = decltype(m)::value;
                if constexpr (Mi == 0) load_hidden<2 * FRAG>(ra[S][0][2], rs_a, voff[0], c_soff);
                if constexpr (Mi == 1) load_hidden<2 * FRAG>(ra[S][1][2], rs_a, voff[1], c_soff);
                issue_b_one(IC<S>{}, m);
            }, I0{});
        });
    };

    for (;;) {
        if (first_tile) {
            first_tile = false;
            pipe::lds_barrier();                   /* block 0 is in its stage, whichever wave requested it */
#pragma unroll
            for (int u = 0; u < TN; u++) fb[0][u] = *(const v4i_t*)(smem + lane * 16 + u * 4 * FRAG);
        }

        const int nkb = cur.npairs * nkb_per;      /* a multiple of DEPTH, at least DEPTH */
        group(I1{});
        for (int g0 = DEPTH; g0 < nkb; g0 += DEPTH) group(I0{});
        epilogue(acc, cur, epi_stage);
        if (!nx_has) break;
        cur = nxt;
        nx_has = next_tile(nxt);
        c_in_next = false;                         /* the cursor is inside the new current tile */
    }
    /* requests past the end of the stream are still on their way to LDS: they
     * must land before the workgroup gives its LDS back */
    drain_loads();
}

}  // namespace pipe2
#endif
