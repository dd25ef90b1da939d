/*
 * The main loop of gemm_pipe2.h on half the accumulator: wave tile 64 x 128 (2 x 4
 * MFMA tiles, 128 accumulator registers), block tile 256 x 128, so that a wave
 * needs 256 registers and TWO workgroups share a CU, two waves on every SIMD.
 *
 * Why. With 256 accumulators a wave owns its SIMD, and whenever it does not issue
 * MFMAs (the epilogue of a finished tile, the barrier of every k-block, a wait
 * for LDS) the SIMD's matrix pipe idles. The epilogue does not depend on K, so it
 * weighs most on short contractions (K = 1024: about half of a tile). With two
 * workgroups per CU the pair settles by itself into opposite phases: while one
 * is in its epilogue the other is in its main loop (time stamps per workgroup and
 * CU, 4096 x 1024 x 1024, sixteen planes: epilogue 6 us, main loop 8 us, two tiles
 * per 14.5 us and CU, where one workgroup alone would need 10 us per tile).
 *
 * What bounds it. A SIMD does run a wave's vector ALU instructions beside another
 * wave's MFMAs, at about half their speed alone (v_dot4 not at all: the matrix pipe
 * executes it), so the epilogue beside a main loop takes 6 us where it takes 3
 * alone. Time stamps per k-block: the matrix pipe is busy 0.6 of the cycles while
 * the sibling is in its epilogue and 0.96 while both multiply, at a clock of 1.65
 * GHz; with the epilogue taken out it is busy 0.99 and the chip lowers the clock
 * to 1.43 GHz. The kernel's time follows the energy it spends under the power
 * limit rather than the cycles its pipe is busy: taking the byte dot product out
 * of the epilogue (a 16-bit fold instead: 6.2 -> 5.0 us beside a main loop, one
 * instruction more per element, clock 1.59 GHz), raising either phase's wave
 * priority and reading the B fragments of a k-step earlier were each measured
 * and change the kernel's time by less than the 2 per cent two runs differ by;
 * none is in.
 * Measured on sixteen residue planes of 4096 x 4096: K = 512 -6 %, K = 1024 -5 %
 * (-8 % at 8192 x 8192), K = 2048 +2 %, K >= 4096 +7 ... +10 % against the
 * 256 x 256 kernel: this one is for K <= 1024.
 *
 * What it costs. The plane layout, the fragment-major addressing, the loads
 * issued from asm and the per-k-block barrier are those of gemm_pipe2.h. Per
 * MFMA the wave loads twice as many A fragments (two per eight MFMAs instead of
 * two per sixteen) and the CU moves half as much more from L2 (48 KiB per 128
 * MFMAs against 64 KiB per 256): three quarters of what the vector memory path
 * of a CU carries at the matrix pipe's full rate, where the large tile needs
 * half. That is why it loses when K is long.
 *
 * Rings. 256 registers leave room for two k-blocks of A fragments, not four, so
 * the two operands have cursors of their own:
 *   A   ring of DEPTH_A = 2 k-blocks in registers: block b+2 is requested while
 *       block b is multiplied (each load has 1.75 k-blocks to land);
 *   B   ring of DEPTH_B = 3 stages of 16 KiB in LDS: block b+3 is requested in
 *       the last k-step of block b, into the stage block b has just left (two
 *       k-blocks to land). Stage of block b = b mod 3, counted across tiles.
 *
 * Issue order of block b (A slot S = b % 2, B stage b % 3):
 *   k-step 0   A(b+1)(k-step 3) -> slot S^1, then the A cursor advances      2 loads
 *   k-step 1   A(b+2)(k-step 0) -> slot S                                    2
 *   k-step 2   A(b+2)(k-step 1) -> slot S; wait; barrier                     2
 *   k-step 3   A(b+2)(k-step 2) -> slot S; B(b+3) -> stage b % 3, B cursor   2 + 4
 * At the wait of block b the youngest load that block b+1 needs is
 * A(b+1)(k-step 3) from this block's k-step 0, with 4 loads behind it; B(b+1)
 * went out in block b-2 with 18 behind it. Hence vmcnt(4).
 */
#ifndef ESHKOL_HIP_GEMM_PIPE3_H
#define ESHKOL_HIP_GEMM_PIPE3_H

#include "gemm_pipe2.h"

namespace pipe3 {

using pipe::v4i_t;
using pipe::IC;
using pipe::static_for;
using pipe::Source;
using pipe::Tile;
using pipe2::FRAG;
using pipe2::BKB;
using pipe2::EPI_WAVE_BYTES;

constexpr int DEPTH_A = 2, DEPTH_B = 3;
constexpr int TM = 2, TN = 4;
constexpr int BM = 256, BN = 128;
constexpr int STAGE = BN * BKB;                       /* 16 KiB of B per k-block */
constexpr int RING = DEPTH_B * STAGE;
constexpr int SMEM_BYTES = RING + 4 * EPI_WAVE_BYTES; /* 66 KiB: two workgroups per CU */
constexpr int WAIT_STEADY = 4;                        /* see the issue order above */
constexpr int WAIT_START = 4 + 6 + 4;                 /* after the prologue: all but block 0's loads may be pending */

/* request cursor of one operand: product within the tile, k-block within the product */
struct Cursor {
    const int8_t* rows;         /* the wave's rows of the tile the cursor is in */
    const int32_t* idx;         /* the tile's plane index list, or NULL */
    int plane0;
    int t, j, np;
    bool in_next;               /* the cursor has crossed into the tile after the current one */
    v4i_t rs;                   /* buffer descriptor of the product's plane rows */
    uint32_t soff;              /* byte offset of the k-block */
};

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

    Tile cur, nxt;
    if (!next_tile(cur)) return;
    bool nx_has = next_tile(nxt);
    /* a wave's share of a tile: its 64 rows of A, its 32 of the 128 rows of B it stages */
    auto wave_rows_a = [&](const Tile& t) { return cm.a_planes + (size_t)(t.m0 / 32 + 2 * wave) * rb_stride; };
    auto wave_rows_b = [&](const Tile& t) { return cm.b_planes + (size_t)(t.n0 / 32 + wave) * rb_stride; };

    Cursor ca, cb;
    auto point = [&](Cursor& c, uint64_t plane_stride) {
        const int i = c.idx ? pipe2::scalar_load(c.idx + c.t) : c.plane0;
        c.rs = pipe2::rsrc_words(c.rows + (size_t)i * plane_stride);
    };
    auto enter = [&](Cursor& c, const Tile& t, auto is_a) {
        constexpr bool A = decltype(is_a)::value != 0;
        c.rows = A ? wave_rows_a(t) : wave_rows_b(t);
        c.idx = A ? t.a_idx : t.b_idx;
        c.plane0 = A ? t.a_plane0 : t.b_plane0;
        c.np = t.npairs;
        c.t = 0; c.j = 0; c.soff = 0;
        point(c, A ? cm.a_plane_stride : cm.b_plane_stride);
    };
    auto advance = [&](Cursor& c, auto is_a) {
        constexpr bool A = decltype(is_a)::value != 0;
        const int nj = c.j + 1;
        if (nj != nkb_per) { c.j = nj; c.soff = (uint32_t)nj * (uint32_t)(4 * FRAG); return; }
        if (c.t + 1 < c.np) {
            c.t++; c.j = 0; c.soff = 0;
            point(c, A ? cm.a_plane_stride : cm.b_plane_stride);
        } else if (nx_has && !c.in_next) {
            c.in_next = true;
            enter(c, nxt, is_a);
        }
        /* else: nothing to move on to: the cursor stays on the last block, whose
         * repeated requests are never consumed */
    };
    using IsA = IC<1>;
    using IsB = IC<0>;
    ca.in_next = false; cb.in_next = false;
    enter(ca, cur, IsA{});
    enter(cb, cur, IsB{});

    v4i_t ra[DEPTH_A][TM][4];                   /* A fragments: [slot][row block][k-step] */
    v4i_t fb[2][TN];                            /* B fragments of the current and the next k-step */
    typename Op::acc_t acc[TM][TN];

    auto issue_a = [&](auto slot, auto kstep) {
        constexpr int S = decltype(slot)::value, KS = decltype(kstep)::value;
        pipe2::load_hidden<KS * FRAG>(ra[S][0][KS], ca.rs, voff[0], ca.soff);
        pipe2::load_hidden<KS * FRAG>(ra[S][1][KS], ca.rs, voff[1], ca.soff);
    };
    /* the wave's k-step KS of the block at the B cursor into LDS stage `stage` */
    auto issue_b_one = [&](int stage, auto kstep) {
        constexpr int KS = decltype(kstep)::value;
        const uint32_t dst = lds_base + (uint32_t)(stage * STAGE) + (uint32_t)wave * (uint32_t)(4 * FRAG);
        pipe2::load_to_lds<KS * FRAG>(dst, cb.rs, voff[0], cb.soff);
    };
    using I0 = IC<0>;
    using I1 = IC<1>;

    /* One k-step: eight MFMAs on the fragments fb[W] and slot S's A fragments of
     * k-step KS, with memory operations after each: after MFMA i < 4 the B
     * fragment i of the next k-step (LDS stage nstage, k-step nks) is read into
     * fb[W ^ 1]; after MFMA 4 ... 7 comes mem(i - 4). Nothing crosses a
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

    /* Start of the stream: B blocks 0, 1, 2 into stages 0, 1, 2; A block 0 whole and
     * block 1 without its last k-step (block 0's k-step 0 requests it). */
    static_for<4>([&](auto ks) { issue_b_one(0, ks); });
    advance(cb, IsB{});
    static_for<4>([&](auto ks) { issue_a(I0{}, ks); });
    advance(ca, IsA{});
    static_for<4>([&](auto ks) { issue_b_one(1, ks); });
    advance(cb, IsB{});
    static_for<3>([&](auto ks) { issue_a(I1{}, ks); });
    static_for<4>([&](auto ks) { issue_b_one(2, ks); });
    advance(cb, IsB{});
    pipe2::wait_loads<WAIT_START>(ra[0]);
    bool first_tile = true;
    int sb = 0;                                 /* LDS stage of the block being multiplied */

    /* Four k-blocks (A slots 0, 1, 0, 1). In a tile's first block the eight sums
     * start with their first product instead of cleared registers. */
    auto group = [&](auto first_of_tile) {
        constexpr int FIRST = decltype(first_of_tile)::value;
        static_for<4>([&](auto s) {
            constexpr int Q = decltype(s)::value, S = Q % DEPTH_A, SN = S ^ 1;
            const int sn = (sb == DEPTH_B - 1) ? 0 : sb + 1;

            kstep(I0{}, IC<S>{}, IC<0>{}, sb, 1, [&](auto m) {
                constexpr int Mi = decltype(m)::value;
                if constexpr (Mi == 0) pipe2::load_hidden<3 * FRAG>(ra[SN][0][3], ca.rs, voff[0], ca.soff);
                if constexpr (Mi == 1) pipe2::load_hidden<3 * FRAG>(ra[SN][1][3], ca.rs, voff[1], ca.soff);
                if constexpr (Mi == 2) advance(ca, IsA{});
            }, IC<(FIRST && Q == 0) ? 1 : 0>{});
            kstep(I1{}, IC<S>{}, IC<1>{}, sb, 2, [&](auto m) {
                constexpr int Mi = decltype(m)::value;
                if constexpr (Mi == 0) pipe2::load_hidden<0>(ra[S][0][0], ca.rs, voff[0], ca.soff);
                if constexpr (Mi == 1) pipe2::load_hidden<0>(ra[S][1][0], ca.rs, voff[1], ca.soff);
            }, I0{});
            kstep(I0{}, IC<S>{}, IC<2>{}, sb, 3, [&](auto m) {
                constexpr int Mi = decltype(m)::value;
                if constexpr (Mi == 0) pipe2::load_hidden<FRAG>(ra[S][0][1], ca.rs, voff[0], ca.soff);
                if constexpr (Mi == 1) pipe2::load_hidden<FRAG>(ra[S][1][1], ca.rs, voff[1], ca.soff);
            }, I0{});
            pipe2::wait_loads<WAIT_STEADY>(ra[SN]);
            pipe::lds_barrier();
            kstep(I1{}, IC<S>{}, IC<3>{}, sn, 0, [&](auto m) {
                constexpr int Mi = decltype(m)::value;
                if constexpr (Mi == 0) pipe2::load_hidden<2 * FRAG>(ra[S][0][2], ca.rs, voff[0], ca.soff);
                if constexpr (Mi == 1) pipe2::load_hidden<2 * FRAG>(ra[S][1][2], ca.rs, voff[1], ca.soff);
                issue_b_one(sb, m);
                if constexpr (Mi == 3) advance(cb, IsB{});
            }, I0{});
            sb = sn;
        });
    };

    for (;;) {
        if (first_tile) {
            first_tile = false;
            pipe::lds_barrier();                   /* block 0 is in its stage, whichever wave requested it */
        }
        /* The first fragments of a tile are read here, behind the epilogue of the tile
         * before (their stage was complete at the last barrier), although that tile's
         * last k-step has read them already: sixteen registers that are not live across
         * the epilogue, which has none to spare. */
#pragma unroll
        for (int u = 0; u < TN; u++) fb[0][u] = *(const v4i_t*)(smem + sb * STAGE + lane * 16 + u * 4 * FRAG);

        const int nkb = cur.npairs * nkb_per;      /* a multiple of 4, at least 4 */
        group(I1{});
        for (int g0 = 4; g0 < nkb; g0 += 4) group(I0{});
        epilogue(acc, cur, epi_stage);
        if (!nx_has) break;
        cur = nxt;
        nx_has = next_tile(nxt);
        ca.in_next = false;                        /* both cursors are inside the new current tile */
        cb.in_next = false;
    }
    /* requests past the end of the stream are still on their way to LDS: they
     * must land before the workgroup gives its LDS back */
    pipe2::drain_loads();
}

}  // namespace pipe3
#endif
