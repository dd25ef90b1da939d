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
 * Two kernels share the tile mapping and the epilogue:
 *   pipelined  256x256 tile, 128-byte k-blocks, register-ring prefetch
 *              (gemm_pipe.h); used when the launch fills the chip and the row
 *              pitch is a multiple of 256 bytes
 *   simple     128x128 tile, 64-byte k-blocks, one block in flight; small or
 *              oddly padded problems
 *
 * The B fragment is passed as the MFMA's first operand, so a lane ends up with
 * 4 consecutive columns of one output row and stores them as one word (int8)
 * or one 16-byte vector (int32). Mode 1 reduces modulo p exactly (two integer
 * folds of 2^14, then a nearest-multiple step in fp32), stages the int8 tile
 * through LDS and writes 16-byte chunks.
 *
 * One launch covers every output plane. Workgroup ids congruent mod 8 run on
 * the same XCD; the id is remapped so that XCD x owns the x-th eighth of every
 * plane's tiles (8 tile-rows at a time inside it). All XCDs then carry the same
 * work whatever the per-plane cost, and the workgroups resident together on an
 * XCD share operand rows in its L2.
 */
#include "hip_common.h"
#include "kernels.h"
#include "gemm_pipe.h"
#include "gemm_pipe2.h"
#include "gemm_pipe3.h"

typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef int v16i_t __attribute__((ext_vector_type(16)));

/* igemm_thin_i8.hip: a first operand of a few rows, interleaved planes */
int eshkol_hip_igemm_thin(const HipIgemmArgs& a, hipStream_t st);

namespace {

struct I8Op {
    typedef v16i_t acc_t;
    static __device__ __forceinline__ void mfma(const v4i_t& first, const v4i_t& second, v16i_t& acc) {
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(first, second, acc, 0, 0, 0);
    }
    /* the first product of a sum: the instruction takes the constant 0 as its addend */
    static __device__ __forceinline__ void mfma_first(const v4i_t& first, const v4i_t& second, v16i_t& acc) {
        const v16i_t none = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(first, second, none, 0, 0, 0);
    }
    static __device__ __forceinline__ void zero(v16i_t& acc) {
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0;
    }
};

/* workgroup -> (output plane, tile); false for the padding workgroups of an XCD */
__device__ __forceinline__ bool map_workgroup(int wg, int tiles_m, int tiles_n, int n_out, int chunk,
                                              int* o, int* tm, int* tn) {
    const int xcd = wg & 7, seq = wg >> 3;
    const int per_plane = tiles_m * tiles_n;
    /* planes from last to first: in the slice tier later planes sum more products */
    *o = n_out - 1 - seq / chunk;
    const int in_plane = xcd * chunk + seq % chunk;
    if (in_plane >= per_plane) return false;
    const int GM = 8;
    const int width = GM * tiles_n;
    const int group = in_plane / width;
    const int first_m = group * GM;
    const int gsize = (tiles_m - first_m < GM) ? tiles_m - first_m : GM;
    const int in_group = in_plane - group * width;
    *tm = first_m + in_group % gsize;
    *tn = in_group / gsize;
    return true;
}

/* The accumulator is the transposed tile (B was the first operand): lane
 * column (lane%32) is the output row, registers 4v..4v+3 are output columns
 * 8v + 4*(lane/32) + 0..3. `stage` is LDS of at least BM*(BN+16) bytes that no
 * wave is still reading. */
template <int TM, int TN>
__device__ __forceinline__ void epilogue(const HipIgemmArgs& g, int o, int m0, int n0,
                                         v16i_t (&acc)[TM][TN], int8_t* stage) {
    constexpr int BM = 2 * TM * 32, BN = 2 * TN * 32, NT = 256;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 31, lh = lane >> 5;

    if (g.mode == 0) {
        int32_t* out = g.out_i32 + (size_t)o * g.out_rows * g.ldn;
        const bool vec_ok = (g.ldn % 4 == 0);
#pragma unroll
        for (int t = 0; t < TM; t++) {
            const int row = m0 + wm * TM * 32 + t * 32 + li;
#pragma unroll
            for (int u = 0; u < TN; u++) {
                asm volatile("" : "+a"(acc[t][u]));      /* see mode 1 */
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int col = n0 + wn * TN * 32 + u * 32 + 8 * v + 4 * lh;
                    if (row < (int)g.out_rows) {
                        int32_t* p = out + (size_t)row * g.ldn + col;
                        if (vec_ok && col + 3 < (int)g.ldn) {
                            v4i_t w = {acc[t][u][4 * v], acc[t][u][4 * v + 1],
                                       acc[t][u][4 * v + 2], acc[t][u][4 * v + 3]};
                            *(v4i_t*)p = w;
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                if (col + e < (int)g.ldn) p[e] = acc[t][u][4 * v + e];
                        }
                    }
                    /* one 4-register group at a time: without the fence the
                     * scheduler reads all 256 accumulators out first and spills */
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        return;
    }

    /* mode 1: residues modulo p, staged through LDS.
     * |sum| <= K * 128 * 128 <= 2^31. One fold of 2^20 into the modulus
     * (sum = hi 2^20 + lo, hi 2^20 = hi c20 mod p) leaves |x| < 2^21, exact in
     * fp32. One fma against 1.5 * 2^23 then rounds x/p to the nearest integer
     * q and leaves 2^22 + q in the low 24 bits of the float: x/p < 2^14 is off
     * by at most 7e-4 in the product and, unless it is a tie, lies at least
     * 1/(2p) >= 2e-3 from a half-integer. x - (2^22 + q) p differs from the
     * residue x - q p in [-p/2, p/2] by a multiple of 256, so its low byte is the
     * int8 residue; the tie (p = 256, +-128) is the same byte either way.
     * Six full-rate instructions per element after the accumulator read: the
     * epilogue is VALU time the matrix pipe sits idle for, so it is kept short. */
    const int p = g.modulus[o];
    const int c20 = (1 << 20) % p;
    const float pinv = 1.0f / (float)p;
    constexpr int EPITCH = BN + 16;
#pragma unroll
    for (int t = 0; t < TM; t++) {
        const int lrow = wm * TM * 32 + t * 32 + li;
#pragma unroll
        for (int u = 0; u < TN; u++) {
            /* Keep this 16-register tile in the accumulator file until here.
             * Otherwise the allocator copies all 256 accumulators into vector
             * registers on entry and spills what does not fit. */
            asm volatile("" : "+a"(acc[t][u]));
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int lcol = wn * TN * 32 + u * 32 + 8 * v + 4 * lh;
                int r[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int s = acc[t][u][4 * v + e];
                    const int x = __mul24(s >> 20, c20) + (s & 0xfffff);
                    const float qm = fmaf((float)x, pinv, 12582912.0f);
                    r[e] = __mul24(__float_as_int(qm), -p) + x;
                }
                /* low bytes of r[0..3] into one word */
                const uint32_t lo2 = __builtin_amdgcn_perm((uint32_t)r[1], (uint32_t)r[0], 0x0c0c0400u);
                const uint32_t hi2 = __builtin_amdgcn_perm((uint32_t)r[3], (uint32_t)r[2], 0x04000c0cu);
                const uint32_t packed = lo2 | hi2;
                *(uint32_t*)(stage + lrow * EPITCH + lcol) = packed;
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    __syncthreads();
    int8_t* out = g.out_i8 + (size_t)o * g.out_rows * g.ldn;
    const bool vec_ok = (g.ldn % 16 == 0) && (((uintptr_t)out & 15) == 0);
    constexpr int CHUNKS_PER_ROW = BN / 16;
    constexpr int TOTAL = BM * CHUNKS_PER_ROW;
    for (int c = tid; c < TOTAL; c += NT) {
        const int lrow = c / CHUNKS_PER_ROW, lc = (c % CHUNKS_PER_ROW) * 16;
        const int row = m0 + lrow, col = n0 + lc;
        if (row >= (int)g.out_rows || col >= (int)g.ldn) continue;
        const int8_t* src = stage + lrow * EPITCH + lc;
        int8_t* dst = out + (size_t)row * g.ldn + col;
        if (vec_ok && col + 15 < (int)g.ldn) {
            *(v4i_t*)dst = *(const v4i_t*)src;
        } else {
            for (int e = 0; e < 16 && col + e < (int)g.ldn; e++) dst[e] = src[e];
        }
    }
}

/* ---- pipelined kernel ------------------------------------------------------ */

/* One workgroup per tile: the same pipeline with a tile list of one. */
template <int TM, int TN, int PF>
__global__ __launch_bounds__(256, 1)
void igemm_i8_pipe_kernel(HipIgemmArgs g, int tiles_m, int tiles_n, int chunk) {
    extern __shared__ __align__(16) int8_t smem_i8[];
    int o, tm, tn;
    if (!map_workgroup((int)blockIdx.x, tiles_m, tiles_n, (int)g.n_out, chunk, &o, &tm, &tn)) return;
    constexpr int BM = 2 * TM * 32, BN = 2 * TN * 32;
    pipe::Source cm;
    cm.a_planes = g.a_planes; cm.b_planes = g.b_planes;
    cm.a_plane_stride = g.a_plane_stride; cm.b_plane_stride = g.b_plane_stride;
    cm.ld = (int)g.ldk;

    const int pair_lo = g.pair_first[o];
    const int npairs = g.pair_first[o + 1] - pair_lo;
    if (npairs <= 0) return;             /* the caller promises every plane a product */
    bool handed_out = false;
    auto next_tile = [&](pipe::Tile& t) -> bool {
        if (handed_out) return false;
        handed_out = true;
        t.m0 = tm * BM; t.n0 = tn * BN; t.tag = o;
        t.a_idx = g.pair_a + pair_lo; t.b_idx = g.pair_b + pair_lo;
        t.npairs = npairs;
        return true;
    };
    auto epi = [&](v16i_t (&acc)[TM][TN], const pipe::Tile& t) {
        epilogue<TM, TN>(g, t.tag, t.m0, t.n0, acc, pipe::epilogue_stage<TM, TN>(smem_i8));
    };
    pipe::run_tiles<I8Op, TM, TN, PF>(smem_i8, cm, next_tile, epi);
}

/* ---- persistent pipelined kernel ------------------------------------------------
 * One workgroup per CU walks the tile ids blockIdx.x, blockIdx.x + gridDim.x, ...
 * (gridDim.x is a multiple of 8, so an id keeps the XCD the tile mapping meant
 * for it). The operand stream runs on across tile boundaries (pipe::run_tiles). */
template <int TM, int TN, int PF>
__global__ __launch_bounds__(256, 1)
void igemm_i8_persistent_kernel(HipIgemmArgs g, int tiles_m, int tiles_n, int chunk, int n_ids) {
    extern __shared__ __align__(16) int8_t smem_i8[];
    constexpr int BM = 2 * TM * 32, BN = 2 * TN * 32;
    pipe::Source cm;
    cm.a_planes = g.a_planes; cm.b_planes = g.b_planes;
    cm.a_plane_stride = g.a_plane_stride; cm.b_plane_stride = g.b_plane_stride;
    cm.ld = (int)g.ldk;

    int next_id = (int)blockIdx.x;
    auto next_tile = [&](pipe::Tile& t) -> bool {
        while (next_id < n_ids) {
            int o, tm, tn;
            const bool real = map_workgroup(next_id, tiles_m, tiles_n, (int)g.n_out, chunk, &o, &tm, &tn);
            next_id += (int)gridDim.x;
            if (!real) continue;
            const int pair_lo = g.pair_first[o];
            t.m0 = tm * BM; t.n0 = tn * BN; t.tag = o;
            t.a_idx = g.pair_a + pair_lo; t.b_idx = g.pair_b + pair_lo;
            t.npairs = g.pair_first[o + 1] - pair_lo;
            /* the caller promises every output plane at least one product
             * (max_pairs >= 1 selects this kernel); an empty one is skipped */
            if (t.npairs > 0) return true;
        }
        return false;
    };
    auto epi = [&](v16i_t (&acc)[TM][TN], const pipe::Tile& t) {
        epilogue<TM, TN>(g, t.tag, t.m0, t.n0, acc, pipe::epilogue_stage<TM, TN>(smem_i8));
    };
    pipe::run_tiles<I8Op, TM, TN, PF>(smem_i8, cm, next_tile, epi);
}

/* Per modulus p <= 256, for the direct kernel's residue epilogue: the smallest
 * multiple of p that is >= 2^31, and the byte weights 256^i mod p (i = 0..3)
 * packed into a word. Tables instead of divisions per tile: the kernel has no
 * vector registers to spare for them. */
struct ModulusTables { uint32_t start[257]; uint32_t wbytes[257]; };
constexpr ModulusTables make_modulus_tables() {
    ModulusTables t{};
    for (uint32_t p = 1; p <= 256; p++) {
        t.start[p] = (uint32_t)(((0x80000000ull + p - 1) / p) * p);
        const uint32_t w0 = 1u % p, w1 = 256u % p, w2 = w1 * w1 % p, w3 = w2 * w1 % p;
        t.wbytes[p] = w0 | w1 << 8 | w2 << 16 | w3 << 24;
    }
    return t;
}
__device__ const ModulusTables MOD_TABLES = make_modulus_tables();

/* ---- interleaved planes: operands never pass through registers on their way
 * to LDS (gemm_pipe2.h) ---------------------------------------------------------
 * Four waves stacked along M, each with a 64 x 256 accumulator: acc[t][u] is
 * the transposed 32 x 32 tile of rows m0 + 64 wave + 32 t + lane%32 and columns
 * n0 + 32 u + 8 v + 4 (lane/32) + 0..3 in registers 4v .. 4v+3. The epilogue
 * is private to a wave (no workgroup barrier): residues are packed four to a
 * word, parked in the wave's own 32 x 128-byte LDS stage and leave as 16-byte
 * stores, eight lanes to a 128-byte row segment. */
template <int TN>
__device__ __forceinline__ void epilogue_direct(const HipIgemmArgs& g, int o, int m0, int n0,
                                                v16i_t (&acc)[2][TN], int8_t* stage) {
    constexpr int TM = 2, TILE_M = 256, TILE_N = 32 * TN;         /* the block tile: four waves of 64 rows */
    static_assert(TN % 4 == 0, "whole 128-column halves");
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, lh = lane >> 5;

    if (g.mode == 0) {
        int32_t* out = g.out_i32 + (size_t)o * g.out_rows * g.ldn;
        const bool vec_ok = (g.ldn % 4 == 0);
        /* a tile inside the matrix: no bounds, no branches, one address per block (the same for every lane) */
        const bool interior0 = vec_ok && (((uintptr_t)out & 15) == 0) &&
                               m0 + TILE_M <= (int)g.out_rows && n0 + TILE_N <= (int)g.ldn;
#pragma unroll
        for (int t = 0; t < TM; t++) {
            const int row = m0 + wave * 64 + t * 32 + li;
#pragma unroll
            for (int u = 0; u < TN; u++) {
                asm volatile("" : "+a"(acc[t][u]));      /* keep the tile in the accumulator file until here */
                /* through the wave's LDS stage, so that eight lanes write a 128-byte row segment */
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    pipe2::park_block(stage, v, (v4i_t){acc[t][u][4 * v], acc[t][u][4 * v + 1],
                                                        acc[t][u][4 * v + 2], acc[t][u][4 * v + 3]});
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (interior0) {
                    constexpr int AB = (TN >= 8) ? 4 : 2;        /* rows in flight: registers are short on the 128-column tile */
                    int32_t* p = out + (size_t)(row - li + (lane >> 3)) * g.ldn + (n0 + u * 32 + 4 * (lane & 7));
#pragma unroll
                    for (int i0 = 0; i0 < 4; i0 += AB) {
                        v4i_t w[AB];
#pragma unroll
                        for (int i = 0; i < AB; i++) w[i] = pipe2::parked_row16(stage, i0 + i);
#pragma unroll
                        for (int i = 0; i < AB; i++) *(v4i_t*)(p + (size_t)(8 * (i0 + i)) * g.ldn) = w[i];
                        if (AB < 4) __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const v4i_t w = pipe2::parked_row16(stage, i);
                        const int orow = row - li + (lane >> 3) + 8 * i, col = n0 + u * 32 + 4 * (lane & 7);
                        if (orow < (int)g.out_rows && col < (int)g.ldn) {
                            int32_t* p = out + (size_t)orow * g.ldn + col;
                            if (vec_ok && col + 3 < (int)g.ldn) *(v4i_t*)p = w;
                            else for (int e = 0; e < 4; e++) if (col + e < (int)g.ldn) p[e] = w[e];
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        return;
    }

    /* mode 1. Adding the smallest multiple of p that is not below 2^31 makes the
     * sum (|sum| < 2^31 for every K the tiers accept) a non-negative 32-bit word
     * of the same residue class. One byte dot product with 256^i mod p gives
     * x < 2^18 congruent to it; the nearest-multiple step of epilogue() above then
     * leaves the residue in the low byte: five instructions per element. */
    const int p = pipe2::scalar_load(g.modulus + o);
    const uint32_t wbytes = (uint32_t)pipe2::scalar_load((const int32_t*)&MOD_TABLES.wbytes[p & 0x1ff]);
    const uint32_t lift = (uint32_t)pipe2::scalar_load((const int32_t*)&MOD_TABLES.start[p & 0x1ff]);
    const float pinv = 1.0f / (float)p;
    constexpr int EP = pipe2::EPI_PITCH;
    int8_t* out = g.out_i8 + (size_t)o * g.out_rows * g.ldn;
    const bool vec_ok = (g.ldn % 16 == 0) && (((uintptr_t)out & 15) == 0);
    const bool interior = vec_ok && m0 + TILE_M <= (int)g.out_rows && n0 + TILE_N <= (int)g.ldn;    /* the same for every lane */
#pragma unroll
    for (int t = 0; t < TM; t++) {
#pragma unroll
        for (int h = 0; h < TN / 4; h++) {                /* columns 128 h .. 128 h + 127 of the tile */
#pragma unroll
            for (int uu = 0; uu < 4; uu++) {
                const int u = 4 * h + uu;
                asm volatile("" : "+a"(acc[t][u]));
                /* Eight elements abreast, one operation of the chain at a time: every
                 * instruction depends on the one eight back, not on its neighbour (a wave
                 * alone on its SIMD has nobody to fill the gaps a dependent chain leaves:
                 * 9.3 -> 8.9 us per tile). Four abreast where two waves share the SIMD and
                 * registers are short (the 128-column tile). */
                constexpr int VG = (TN >= 8) ? 2 : 1;             /* groups of four columns per pass */
#pragma unroll
                for (int vv = 0; vv < 4; vv += VG) {
                    uint32_t a8[4 * VG];
                    int x[4 * VG], r[4 * VG];
                    float q[4 * VG];
#pragma unroll
                    for (int e = 0; e < 4 * VG; e++) a8[e] = (uint32_t)acc[t][u][4 * vv + e] + lift;
#pragma unroll
                    for (int e = 0; e < 4 * VG; e++) x[e] = (int)__builtin_amdgcn_udot4(a8[e], wbytes, 0u, false);
#pragma unroll
                    for (int e = 0; e < 4 * VG; e++) q[e] = (float)x[e];
#pragma unroll
                    for (int e = 0; e < 4 * VG; e++) q[e] = fmaf(q[e], pinv, 12582912.0f);
#pragma unroll
                    for (int e = 0; e < 4 * VG; e++) r[e] = __mul24(__float_as_int(q[e]), -p) + x[e];
#pragma unroll
                    for (int w = 0; w < VG; w++) {
                        const uint32_t lo2 = __builtin_amdgcn_perm((uint32_t)r[4 * w + 1], (uint32_t)r[4 * w], 0x0c0c0400u);
                        const uint32_t hi2 = __builtin_amdgcn_perm((uint32_t)r[4 * w + 3], (uint32_t)r[4 * w + 2], 0x04000c0cu);
                        *(uint32_t*)(stage + li * EP + uu * 32 + 8 * (vv + w) + 4 * lh) = lo2 | hi2;
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            /* the wave's LDS accesses complete in order: its reads see its writes */
            if (interior) {
                /* a tile inside the matrix: no bounds, no branches, one address per wave
                 * and row block (2.8 of this epilogue's 9 us per tile were the guarded
                 * stores below: a branch and a 64-bit product each) */
                constexpr int AB = (TN >= 8) ? 4 : 2;            /* rows in flight, as above */
                int8_t* dst = out + (size_t)(m0 + wave * 64 + t * 32 + (lane >> 3)) * g.ldn + (n0 + 128 * h + 16 * (lane & 7));
#pragma unroll
                for (int i0 = 0; i0 < 4; i0 += AB) {
                    v4i_t val[AB];
#pragma unroll
                    for (int i = 0; i < AB; i++)
                        val[i] = *(const v4i_t*)(stage + ((lane >> 3) + 8 * (i0 + i)) * EP + (lane & 7) * 16);
#pragma unroll
                    for (int i = 0; i < AB; i++) *(v4i_t*)(dst + (size_t)(8 * (i0 + i)) * g.ldn) = val[i];
                    if (AB < 4) __builtin_amdgcn_sched_barrier(0);
                }
                continue;
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int c = lane + 64 * i;
                const int lrow = c >> 3, ch = c & 7;
                const int row = m0 + wave * 64 + t * 32 + lrow, col = n0 + 128 * h + 16 * ch;
                const v4i_t val = *(const v4i_t*)(stage + lrow * EP + ch * 16);
                if (row < (int)g.out_rows && col < (int)g.ldn) {
                    int8_t* dst = out + (size_t)row * g.ldn + col;
                    if (vec_ok && col + 15 < (int)g.ldn) {
                        *(v4i_t*)dst = val;
                    } else {
                        const int8_t* src = stage + lrow * EP + ch * 16;
                        for (int e = 0; e < 16 && col + e < (int)g.ldn; e++) dst[e] = src[e];
                    }
                }
            }
        }
    }
}

/* One workgroup per CU walks the tile ids blockIdx.x, blockIdx.x + gridDim.x, ...
 * as the persistent kernel above does. */
__global__ __launch_bounds__(256, 1)
void igemm_i8_direct_kernel(HipIgemmArgs g, int tiles_m, int tiles_n, int chunk, int n_ids) {
    extern __shared__ __align__(16) int8_t smem_i8[];
    pipe::Source cm;
    cm.a_planes = g.a_planes; cm.b_planes = g.b_planes;
    cm.a_plane_stride = g.a_plane_stride; cm.b_plane_stride = g.b_plane_stride;
    cm.ld = (int)g.ldk;

    int next_id = (int)blockIdx.x;
    auto next_tile = [&](pipe::Tile& t) -> bool {
        while (next_id < n_ids) {
            int o, tm, tn;
            const bool real = map_workgroup(next_id, tiles_m, tiles_n, (int)g.n_out, chunk, &o, &tm, &tn);
            next_id += (int)gridDim.x;
            if (!real) continue;
            const int pair_lo = pipe2::scalar_load(g.pair_first + o);
            t.m0 = tm * pipe2::BM; t.n0 = tn * pipe2::BN; t.tag = o;
            t.a_idx = g.pair_a + pair_lo; t.b_idx = g.pair_b + pair_lo;
            t.npairs = pipe2::scalar_load(g.pair_first + o + 1) - pair_lo;
            if (t.npairs > 0) return true;
        }
        return false;
    };
    auto epi = [&](v16i_t (&acc)[pipe2::TM][pipe2::TN], const pipe::Tile& t, int8_t* stage) {
        epilogue_direct<pipe2::TN>(g, t.tag, t.m0, t.n0, acc, stage);
    };
    pipe2::run_tiles<I8Op>(smem_i8, cm, next_tile, epi);
}

/* The same on 256 x 128 tiles with 128 accumulators per wave, two workgroups per
 * CU (gemm_pipe3.h): while one workgroup is in its epilogue the other multiplies.
 * For contractions whose K is short enough for the time between tiles to matter. */
__global__ __launch_bounds__(256, 2)
void igemm_i8_direct_half_kernel(HipIgemmArgs g, int tiles_m, int tiles_n, int chunk, int n_ids) {
    extern __shared__ __align__(16) int8_t smem_i8[];
    pipe::Source cm;
    cm.a_planes = g.a_planes; cm.b_planes = g.b_planes;
    cm.a_plane_stride = g.a_plane_stride; cm.b_plane_stride = g.b_plane_stride;
    cm.ld = (int)g.ldk;

    int next_id = (int)blockIdx.x;
    auto next_tile = [&](pipe::Tile& t) -> bool {
        while (next_id < n_ids) {
            int o, tm, tn;
            const bool real = map_workgroup(next_id, tiles_m, tiles_n, (int)g.n_out, chunk, &o, &tm, &tn);
            next_id += (int)gridDim.x;
            if (!real) continue;
            const int pair_lo = pipe2::scalar_load(g.pair_first + o);
            t.m0 = tm * pipe3::BM; t.n0 = tn * pipe3::BN; t.tag = o;
            t.a_idx = g.pair_a + pair_lo; t.b_idx = g.pair_b + pair_lo;
            t.npairs = pipe2::scalar_load(g.pair_first + o + 1) - pair_lo;
            if (t.npairs > 0) return true;
        }
        return false;
    };
    auto epi = [&](v16i_t (&acc)[pipe3::TM][pipe3::TN], const pipe::Tile& t, int8_t* stage) {
        epilogue_direct<pipe3::TN>(g, t.tag, t.m0, t.n0, acc, stage);
    };
    pipe3::run_tiles<I8Op>(smem_i8, cm, next_tile, epi);
}

/* ---- simple kernel --------------------------------------------------------- */

constexpr int SBK = 64;
constexpr int SPITCH = SBK + 16;

template <int TM, int TN>
__global__ __launch_bounds__(256, 2)
void igemm_i8_simple_kernel(HipIgemmArgs g, int tiles_m, int tiles_n, int chunk) {
    constexpr int BM = 2 * TM * 32, BN = 2 * TN * 32, NT = 256;
    constexpr int A_TILE = BM * SPITCH, B_TILE = BN * SPITCH;
    constexpr int A_CH = BM * SBK / 16 / NT, B_CH = BN * SBK / 16 / NT;
    extern __shared__ __align__(16) int8_t smem_i8[];
    int8_t* As = smem_i8;
    int8_t* Bs = smem_i8 + 2 * A_TILE;

    int o, tm, tn;
    if (!map_workgroup((int)blockIdx.x, tiles_m, tiles_n, (int)g.n_out, chunk, &o, &tm, &tn)) return;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 31, lh = lane >> 5;

    const int pair_lo = g.pair_first[o], pair_hi = g.pair_first[o + 1];
    const int nkb_per = (int)(g.ldk / SBK);
    const int nkb = (pair_hi - pair_lo) * nkb_per;

    v4i_t ra[A_CH], rb[B_CH];
    auto gload = [&](int kb) {
        const int t = pair_lo + kb / nkb_per;
        const int k0 = (kb % nkb_per) * SBK;
        const int8_t* Ap = g.a_planes + (size_t)g.pair_a[t] * g.a_plane_stride + (size_t)m0 * g.ldk + k0;
        const int8_t* Bp = g.b_planes + (size_t)g.pair_b[t] * g.b_plane_stride + (size_t)n0 * g.ldk + k0;
#pragma unroll
        for (int r = 0; r < A_CH; r++) {
            const int c = tid + NT * r;
            ra[r] = *(const v4i_t*)(Ap + (size_t)(c >> 2) * g.ldk + (c & 3) * 16);
        }
#pragma unroll
        for (int r = 0; r < B_CH; r++) {
            const int c = tid + NT * r;
            rb[r] = *(const v4i_t*)(Bp + (size_t)(c >> 2) * g.ldk + (c & 3) * 16);
        }
    };
    auto sstore = [&](int buf) {
#pragma unroll
        for (int r = 0; r < A_CH; r++) {
            const int c = tid + NT * r;
            *(v4i_t*)(As + buf * A_TILE + (c >> 2) * SPITCH + (c & 3) * 16) = ra[r];
        }
#pragma unroll
        for (int r = 0; r < B_CH; r++) {
            const int c = tid + NT * r;
            *(v4i_t*)(Bs + buf * B_TILE + (c >> 2) * SPITCH + (c & 3) * 16) = rb[r];
        }
    };

    v16i_t acc[TM][TN];
#pragma unroll
    for (int t = 0; t < TM; t++)
#pragma unroll
        for (int u = 0; u < TN; u++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[t][u][r] = 0;

    if (nkb > 0) { gload(0); sstore(0); }
    __syncthreads();
    int cur = 0;
    for (int kb = 0; kb < nkb; kb++) {
        const bool more = (kb + 1 < nkb);
        if (more) gload(kb + 1);
        const int8_t* a_base = As + cur * A_TILE + (wm * TM * 32 + li) * SPITCH + lh * 16;
        const int8_t* b_base = Bs + cur * B_TILE + (wn * TN * 32 + li) * SPITCH + lh * 16;
#pragma unroll
        for (int ks = 0; ks < SBK / 32; ks++) {
            v4i_t a[TM], b[TN];
#pragma unroll
            for (int t = 0; t < TM; t++) a[t] = *(const v4i_t*)(a_base + t * 32 * SPITCH + ks * 32);
#pragma unroll
            for (int u = 0; u < TN; u++) b[u] = *(const v4i_t*)(b_base + u * 32 * SPITCH + ks * 32);
#pragma unroll
            for (int t = 0; t < TM; t++)
#pragma unroll
                for (int u = 0; u < TN; u++) I8Op::mfma(b[u], a[t], acc[t][u]);
        }
        if (more) sstore(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }
    epilogue<TM, TN>(g, o, m0, n0, acc, smem_i8);
}

int g_direct = 1;       /* big launches take interleaved planes and the direct-to-LDS kernel */
int g_prefetch = 2;     /* blocks in flight in the pipelined kernel */
int g_persistent = 1;   /* pipelined kernel as one workgroup per CU walking a tile list */

template <class K>
int launch_kernel(K kern, int smem, bool* attr_set, const HipIgemmArgs& a, int BM, int BN, hipStream_t st) {
    if (!*attr_set) {
        if (!ESHKOL_HIP_OK(hipFuncSetAttribute((const void*)kern,
                hipFuncAttributeMaxDynamicSharedMemorySize, smem))) return -1;
        *attr_set = true;
    }
    const int tiles_m = (int)((a.M + BM - 1) / BM), tiles_n = (int)((a.N + BN - 1) / BN);
    const int chunk = (tiles_m * tiles_n + 7) / 8;
    const long long nwg = 8LL * chunk * a.n_out;
    if (nwg > 0x7fffffffLL || nwg <= 0) return -1;
    hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(256), smem, st, a, tiles_m, tiles_n, chunk);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

template <int PF>
int launch_pipe(const HipIgemmArgs& a, hipStream_t st) {
    using C = pipe::Cfg<4, 4>;
    constexpr int EPI = C::BM * (C::BN + 16);
    static_assert(EPI <= pipe::StageCfg<4, 4>::BYTES, "the epilogue stages its tile in one LDS operand buffer");
    constexpr int MAIN = pipe::TilesCfg<4, 4>::SMEM_MAIN;
    constexpr int SMEM = MAIN > EPI ? MAIN : EPI;
    static bool attr_set = false;
    return launch_kernel(igemm_i8_pipe_kernel<4, 4, PF>, SMEM, &attr_set, a, C::BM, C::BN, st);
}

template <int PF>
int launch_persistent(const HipIgemmArgs& a, hipStream_t st) {
    using C = pipe::Cfg<4, 4>;
    constexpr int EPI = C::BM * (C::BN + 16);
    static_assert(EPI <= pipe::StageCfg<4, 4>::BYTES, "the epilogue stages its tile in one LDS operand buffer");
    constexpr int MAIN = pipe::TilesCfg<4, 4>::SMEM_MAIN;
    constexpr int SMEM = MAIN > EPI ? MAIN : EPI;
    static bool attr_set = false;
    static int num_cus = 0;
    auto kern = igemm_i8_persistent_kernel<4, 4, PF>;
    if (!attr_set) {
        if (!ESHKOL_HIP_OK(hipFuncSetAttribute((const void*)kern,
                hipFuncAttributeMaxDynamicSharedMemorySize, SMEM))) return -1;
        int dev = 0;
        hipDeviceProp_t prop;
        if (!ESHKOL_HIP_OK(hipGetDevice(&dev)) || !ESHKOL_HIP_OK(hipGetDeviceProperties(&prop, dev))) return -1;
        num_cus = prop.multiProcessorCount;
        attr_set = true;
    }
    const int tiles_m = (int)((a.M + C::BM - 1) / C::BM), tiles_n = (int)((a.N + C::BN - 1) / C::BN);
    const int chunk = (tiles_m * tiles_n + 7) / 8;
    const long long n_ids = 8LL * chunk * a.n_out;
    if (n_ids > 0x7fffffffLL || n_ids <= 0) return -1;
    long long grid = (num_cus / 8) * 8;             /* one workgroup per CU, a multiple of the XCD count */
    if (grid < 8) grid = 8;
    if (grid > n_ids) grid = n_ids;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), SMEM, st, a, tiles_m, tiles_n, chunk, (int)n_ids);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

int g_cu_limit = 0;      /* > 0: the persistent 256 x 256 kernel leaves the other CUs to whatever else runs */

int launch_direct(const HipIgemmArgs& a, hipStream_t st) {
    constexpr int SMEM = pipe2::SMEM_BYTES;
    static bool attr_set = false;
    static int num_cus = 0;
    auto kern = igemm_i8_direct_kernel;
    if (!attr_set) {
        if (!ESHKOL_HIP_OK(hipFuncSetAttribute((const void*)kern,
                hipFuncAttributeMaxDynamicSharedMemorySize, SMEM))) return -1;
        int dev = 0;
        hipDeviceProp_t prop;
        if (!ESHKOL_HIP_OK(hipGetDevice(&dev)) || !ESHKOL_HIP_OK(hipGetDeviceProperties(&prop, dev))) return -1;
        num_cus = prop.multiProcessorCount;
        attr_set = true;
    }
    const int tiles_m = (int)((a.M + pipe2::BM - 1) / pipe2::BM), tiles_n = (int)((a.N + pipe2::BN - 1) / pipe2::BN);
    const int chunk = (tiles_m * tiles_n + 7) / 8;
    const long long n_ids = 8LL * chunk * a.n_out;
    if (n_ids > 0x7fffffffLL || n_ids <= 0) return -1;
    long long grid = (num_cus / 8) * 8;             /* one workgroup per CU, a multiple of the XCD count */
    if (g_cu_limit > 0 && grid > g_cu_limit) grid = (g_cu_limit / 8) * 8;
    if (grid < 8) grid = 8;
    if (grid > n_ids) grid = n_ids;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), SMEM, st, a, tiles_m, tiles_n, chunk, (int)n_ids);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

int launch_direct_half(const HipIgemmArgs& a, hipStream_t st) {
    constexpr int SMEM = pipe3::SMEM_BYTES;
    static bool attr_set = false;
    static int num_cus = 0;
    auto kern = igemm_i8_direct_half_kernel;
    if (!attr_set) {
        if (!ESHKOL_HIP_OK(hipFuncSetAttribute((const void*)kern,
                hipFuncAttributeMaxDynamicSharedMemorySize, SMEM))) return -1;
        num_cus = eshkol_hip_num_cus();
        attr_set = true;
    }
    const int tiles_m = (int)((a.M + pipe3::BM - 1) / pipe3::BM), tiles_n = (int)((a.N + pipe3::BN - 1) / pipe3::BN);
    const int chunk = (tiles_m * tiles_n + 7) / 8;
    const long long n_ids = 8LL * chunk * a.n_out;
    if (n_ids > 0x7fffffffLL || n_ids <= 0) return -1;
    long long grid = 2LL * ((num_cus / 8) * 8);     /* two workgroups per CU, a multiple of the XCD count */
    if (grid < 8) grid = 8;
    if (grid > n_ids) grid = n_ids;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256), SMEM, st, a, tiles_m, tiles_n, chunk, (int)n_ids);
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}

int launch_simple(const HipIgemmArgs& a, hipStream_t st) {
    constexpr int BM = 128, BN = 128;
    constexpr int MAIN = 2 * (BM + BN) * SPITCH, EPI = BM * (BN + 16);
    constexpr int SMEM = MAIN > EPI ? MAIN : EPI;
    static bool attr_set = false;
    return launch_kernel(igemm_i8_simple_kernel<2, 2>, SMEM, &attr_set, a, BM, BN, st);
}

}  // namespace

/* Tuning hook: k-blocks in flight in the pipelined kernel (1..3), 0 = simple kernel only. */
extern "C" void hip_igemm_set_prefetch(int pf) { EshkolHipLock lk; if (pf >= 0 && pf <= 3) g_prefetch = pf; }
/* Tuning hook: 1 (default) runs the pipelined kernel as one workgroup per CU
 * walking a list of tiles, 0 as one workgroup per tile. Same results. */
extern "C" void hip_igemm_set_persistent(int on) { EshkolHipLock lk; g_persistent = on ? 1 : 0; }

/* Tuning hook: 0 keeps every launch on row-major planes and the register-staged
 * kernels. Same results. */
extern "C" void hip_igemm_set_direct(int on) { EshkolHipLock lk; g_direct = (on >= 0 && on <= 3) ? on : 1; }

extern "C" void hip_igemm_set_cu_limit(int cus) { EshkolHipLock lk; g_cu_limit = cus > 0 ? cus : 0; }

int eshkol_hip_igemm_direct_mode(void) { return g_direct; }

/* The plane layout the tiers should produce for a contraction of n_out output
 * planes of M x N: 1 (interleaved, for the direct-to-LDS kernel) when the launch
 * has enough 256 x 256 tiles to be worth a workgroup per CU, else 0. */
extern "C" int hip_igemm_plane_layout(uint64_t M, uint64_t N, int n_out) {
    const uint64_t big = ((M + 255) / 256) * ((N + 255) / 256) * (uint64_t)(n_out > 0 ? n_out : 0);
    if (eshkol_hip_igemm_is_thin(M, N)) return 1;     /* streams the second operand's planes */
    return (g_direct != 0 && big >= 128) ? 1 : 0;
}

/* The same for contractions of one product per output plane over K of k (the two CRT
 * tiers), which the 256 x 128 kernel may take: from sixteen tiles of 256 x 256 and 1024 of
 * k on, that kernel on interleaved planes is at least as fast as the kernels for row-major
 * planes (256 x 1024 x 256, sixteen planes: 12.7 us against 13.2; 256 x 4096 x 1024: 38.7
 * against 47.3; 256 x 16384 x 256: 102 against 152), so such launches are interleaved too. */
extern "C" int hip_igemm_plane_layout_single(uint64_t M, uint64_t K, uint64_t N, int n_out) {
    if (hip_igemm_plane_layout(M, N, n_out)) return 1;
    const uint64_t big = ((M + 255) / 256) * ((N + 255) / 256) * (uint64_t)(n_out > 0 ? n_out : 0);
    return ((g_direct == 1 || g_direct == 2) && K >= 1024 && big >= 16) ? 1 : 0;
}

extern "C" int hip_igemm_i8(const HipIgemmArgs* args, void* stream) {
    EshkolHipCall bracket(stream);
    if (!args || !args->a_planes || !args->b_planes || !args->pair_first || !args->pair_a || !args->pair_b)
        return -1;
    HipIgemmArgs a = *args;
    if (a.M == 0 || a.N == 0 || a.n_out == 0 || a.ldk == 0 || a.ldk % 128 != 0) return -1;
    if (a.M > 0x7fffffffu || a.N > 0x7fffffffu) return -1;
    /* output planes of out_rows x ldn elements: dense unless the caller allocated them larger */
    if (a.ldn == 0) a.ldn = a.N;
    if (a.out_rows == 0) a.out_rows = a.M;
    if (a.ldn < a.N || a.out_rows < a.M || a.ldn > 0x7fffffffu || a.out_rows > 0x7fffffffu) return -1;
    if (((uintptr_t)a.a_planes & 15) || ((uintptr_t)a.b_planes & 15) ||
        (a.a_plane_stride & 15) || (a.b_plane_stride & 15)) return -1;
    if (a.mode == 0) { if (!a.out_i32) return -1; }
    else if (a.mode == 1) { if (!a.out_i8 || !a.modulus) return -1; }
    else return -1;
    hipStream_t st = (hipStream_t)stream;
    if (a.layout == 1) {
        /* interleaved planes: whole groups of four 128-byte k-blocks per product,
         * every output plane with 1..64 products, row counts padded to 256 */
        if (a.ldk % 512 != 0 || a.max_pairs < 1) return -1;
        if ((a.a_plane_stride % (32ull * a.ldk)) || (a.b_plane_stride % (32ull * a.ldk))) return -1;
        /* a few rows against the second operand's planes: bound by reading those once */
        if (eshkol_hip_igemm_is_thin(a.M, a.N)) return eshkol_hip_igemm_thin(a, st);
        /* Products of at most 1024 bytes of k per row take the 256 x 128 kernel with
         * two workgroups per CU (measured 5 ... 13 % faster there, slower from 2048 on), and
         * so do launches with no more 256 x 256 tiles than CUs, whatever their k: twice the
         * workgroups (64 tiles of k = 4096: 50 -> 39 us, 32 of k = 8192: 86 -> 53, 256 of
         * k = 4096: 100 -> 92, of k = 2048: 48 -> 44). Row counts
         * of B padded to 256 cover its tiles too. g_direct 2 / 3: always / never. */
        const uint64_t tiles256 = (uint64_t)((a.M + 255) / 256) * ((a.N + 255) / 256) * a.n_out;
        const bool half = g_direct == 2 || (g_direct == 1 && a.max_pairs == 1 &&
                                            (a.ldk <= 1024 || tiles256 <= (uint64_t)eshkol_hip_num_cus()));
        return half ? launch_direct_half(a, st) : launch_direct(a, st);
    }
    if (a.layout != 0) return -1;
    /* Operand planes are padded to multiples of 256 rows, so either tiling reads
     * in bounds. The pipelined kernel needs whole groups of prefetched blocks
     * per product and at most 64 products per output plane. */
    const long long big = (long long)((a.M + 255) / 256) * ((a.N + 255) / 256) * a.n_out;
    int pf = g_prefetch;
    while (pf > 0 && a.ldk % (128u * pf) != 0) pf--;
    if (pf > 0 && big >= 128 && a.max_pairs >= 1 && a.max_pairs <= pipe::MAX_PAIRS) {
        /* the persistent kernel's request cursor must have left a tile before the
         * tile after the next is announced: max(2 PF, PF + 2) blocks per tile */
        if (g_persistent && a.ldk >= 128u * (unsigned)(2 * pf > pf + 2 ? 2 * pf : pf + 2)) {
            switch (pf) {
                case 1: return launch_persistent<1>(a, st);
                case 2: return launch_persistent<2>(a, st);
                default: return launch_persistent<3>(a, st);
            }
        }
        switch (pf) {
            case 1: return launch_pipe<1>(a, st);
            case 2: return launch_pipe<2>(a, st);
            default: return launch_pipe<3>(a, st);
        }
    }
    return launch_simple(a, st);
}
