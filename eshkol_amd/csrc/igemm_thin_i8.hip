/*
 * The int8 contraction (hip_igemm_i8) for a first operand of a few rows (up to 160): a batch
 * of activation rows against a layer's residue planes. The tiled kernels pad such a product
 * to 256 rows and hand every workgroup a 256-column tile with all of k to walk: 16 planes
 * of 4096 x 1024 gave 128 ... 512 workgroups and 1.3 ... 2.4 TB/s on planes that are read
 * exactly once, 16 of 4096 x 4096 3.1 ... 3.9. Here the second operand's planes are
 * streamed and nothing else matters. Interleaved planes only (HipIgemmArgs.layout 1): the
 * 32 rows x 32 bytes of k that one v_mfma_i32_32x32x32_i8 takes are 1 KiB of contiguous
 * memory, and a block of 32 rows is one contiguous run of 32 ldk bytes. Two kernels:
 *
 *   up to 64 rows, igemm_i8_thin_kernel: a workgroup takes one or two blocks of the second
 *     operand (32 or 64 output columns) of one output plane; its four waves deal the run
 *     out in pieces of 8 KiB, every lane with eight 16-byte loads in flight, so that the
 *     launch has thousands of waves and tens of megabytes on their way at any time. The
 *     first operand comes from the L2, every wave fetching the fragments it needs for
 *     itself: the L2 delivered about 11 TB/s to the CUs whatever the split, so with R
 *     blocks of 32 rows and C column blocks per workgroup the stream gets 1 / (1 + R / C)
 *     of it (5.7 TB/s at R 1 C 2, 4.5 at R 2 C 2, 3.2 at R 4 C 2). The four partial sums
 *     meet in LDS.
 *
 *   33 ... 160 rows, igemm_i8_rows_kernel: the four waves of a workgroup take four
 *     neighbouring column blocks and walk k together; the first operand's fragments for
 *     a group of steps are fetched once per workgroup into LDS. See there.
 *
 * Every thread ends up with four consecutive columns of one row, reduces them modulo p
 * (mode 1, the arithmetic of the tiled kernels' epilogue) and stores one word, or the four
 * int32 sums (mode 0). Same plans as the tiled kernels (an output plane may sum several
 * products), same bits.
 */
#include "hip_common.h"
#include "kernels.h"

typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef int v16i_t __attribute__((ext_vector_type(16)));

namespace {

/* Four consecutive columns of one output row: the int32 sums (mode 0) or their residues
 * modulo p packed into one word (mode 1). col is a multiple of 4.
 * |sum| < 2^31: one fold of 2^20 leaves |x| < 2^21, exact in fp32; the fma against
 * 1.5 * 2^23 leaves 2^22 + round(x / p) in the float's low bits, and x - (2^22 + q) p
 * differs from the residue in [-p/2, p/2] by a multiple of 256: its low byte is the result. */
__device__ __forceinline__ void store_four(const HipIgemmArgs& g, int o, int row, int col, const v4i_t& s,
                                           int p, int c20, float pinv) {
    if (g.mode == 0) {
        int32_t* dst = g.out_i32 + ((size_t)o * g.out_rows + row) * g.ldn + col;
        if (g.ldn % 4 == 0 && ((uintptr_t)g.out_i32 & 15) == 0) *(v4i_t*)dst = s;
        else for (int e = 0; e < 4; e++) if (col + e < (int)g.ldn) dst[e] = s[e];
        return;
    }
    int r[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int x = __mul24(s[e] >> 20, c20) + (s[e] & 0xfffff);
        const float qm = fmaf((float)x, pinv, 12582912.0f);
        r[e] = __mul24(__float_as_int(qm), -p) + x;
    }
    int8_t* dst = g.out_i8 + ((size_t)o * g.out_rows + row) * g.ldn + col;
    if (g.ldn % 4 == 0 && ((uintptr_t)g.out_i8 & 3) == 0) {
        const uint32_t lo2 = __builtin_amdgcn_perm((uint32_t)r[1], (uint32_t)r[0], 0x0c0c0400u);
        const uint32_t hi2 = __builtin_amdgcn_perm((uint32_t)r[3], (uint32_t)r[2], 0x04000c0cu);
        *(uint32_t*)dst = lo2 | hi2;
    } else {
        for (int e = 0; e < 4; e++) if (col + e < (int)g.ldn) dst[e] = (int8_t)r[e];
    }
}

template <int RB, int CB, int GROUP_STEPS>
__global__ __launch_bounds__(256)
void igemm_i8_thin_kernel(HipIgemmArgs g) {
    constexpr int GROUP_BYTES = GROUP_STEPS * 1024;
    __shared__ v4i_t red[4][4][64];
    const int o = (int)blockIdx.y, cb0 = (int)blockIdx.x * CB;
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, lh = lane >> 5;
    v16i_t acc[RB][CB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int c = 0; c < CB; c++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[rb][c][r] = 0;

    const int groups = (int)(g.ldk / (32 * GROUP_STEPS));
    const size_t block_bytes = (size_t)32 * g.ldk;
    const int first = g.pair_first[o], last = g.pair_first[o + 1];
    for (int t = first; t < last; t++) {
        const int8_t* bp = g.b_planes + (size_t)g.pair_b[t] * g.b_plane_stride + (size_t)cb0 * block_bytes + lane * 16;
        const int8_t* ap = g.a_planes + (size_t)g.pair_a[t] * g.a_plane_stride + lane * 16;
        for (int gi = wave; gi < groups; gi += 4) {
            v4i_t b[CB][GROUP_STEPS];
#pragma unroll
            for (int c = 0; c < CB; c++)
#pragma unroll
                for (int s = 0; s < GROUP_STEPS; s++)
                    b[c][s] = __builtin_nontemporal_load((const v4i_t*)(bp + c * block_bytes + (size_t)gi * GROUP_BYTES + s * 1024));
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                v4i_t a[GROUP_STEPS];
#pragma unroll
                for (int s = 0; s < GROUP_STEPS; s++)
                    a[s] = *(const v4i_t*)(ap + rb * block_bytes + (size_t)gi * GROUP_BYTES + s * 1024);
#pragma unroll
                for (int c = 0; c < CB; c++)
#pragma unroll
                    for (int s = 0; s < GROUP_STEPS; s++)
                        acc[rb][c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[c][s], a[s], acc[rb][c], 0, 0, 0);
            }
        }
    }
    int p = 1, c20 = 0;
    float pinv = 1.0f;
    if (g.mode == 1) { p = g.modulus[o]; c20 = (1 << 20) % p; pinv = 1.0f / (float)p; }
    /* The accumulator is the transposed tile (the second operand's fragment went first):
     * lane%32 is the output row, registers 4v .. 4v+3 are columns 8v + 4 (lane/32) + 0..3.
     * One 32 x 32 block at a time through LDS: thread (wave v, lane) then owns row
     * 32 rb + lane%32, columns 32 (cb0 + c) + 8 v + 4 (lane/32) + 0..3. */
    const int v = wave;
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
#pragma unroll
        for (int c = 0; c < CB; c++) {
            if (rb + c) __syncthreads();                            /* the block before has been read */
#pragma unroll
            for (int vv = 0; vv < 4; vv++)
                red[wave][vv][lane] = (v4i_t){acc[rb][c][4 * vv], acc[rb][c][4 * vv + 1], acc[rb][c][4 * vv + 2], acc[rb][c][4 * vv + 3]};
            __syncthreads();
            const int row = rb * 32 + li, col = (cb0 + c) * 32 + 8 * v + 4 * lh;
            if (row >= (int)g.out_rows || col >= (int)g.ldn) continue;      /* no barrier is skipped: they sit above */
            v4i_t s = red[0][v][lane];
#pragma unroll
            for (int w = 1; w < 4; w++) s += red[w][v][lane];
            store_four(g, o, row, col, s, p, c20, pinv);
        }
    }
}

/* 33 ... 160 rows: with more than two blocks of rows the first operand's fragments, fetched
 * from the L2 by every wave for itself, outweigh the stream they are multiplied with. Here
 * the four waves of a workgroup take four neighbouring column blocks and walk k together,
 * GS matrix-core steps at a time: the group's RB x GS fragments of the first operand are
 * fetched once per workgroup into LDS, each wave's own 1 KiB x GS of the second operand into
 * registers, then RB x GS matrix-core instructions per wave. Nothing is prefetched and the
 * LDS has one buffer (two barriers per group): what hides a group's memory latency is the
 * other workgroups of the CU, which is why registers and LDS are kept small (a version
 * with two LDS buffers and the next group's loads in flight measured 83 us where this one
 * takes 60, 16 planes of 4096 x 4096 against 128 rows: it had half the waves per CU). A wave
 * owns its 32 columns, so no sums are combined. 16 planes of 4096 x 4096: 54 us at 64 rows,
 * 60 at 128 (the tiled kernels 74 ... 90), 73 at 160; from 192 rows on the tiled kernels win. */
template <int RB, int GS>
__global__ __launch_bounds__(256)
void igemm_i8_rows_kernel(HipIgemmArgs g) {
    constexpr int FRAGS = RB * GS;                 /* 1 KiB fragments of the first operand per group */
    constexpr int PASSES = (FRAGS + 3) / 4;        /* each wave fetches one fragment per pass */
    __shared__ __align__(16) int8_t abuf[FRAGS * 1024];
    const int o = (int)blockIdx.y;
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, lh = lane >> 5;
    const int cb = (int)blockIdx.x * 4 + wave;
    v16i_t acc[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[rb][r] = 0;
    const int groups = (int)(g.ldk / (32 * GS));
    const size_t block_bytes = (size_t)32 * g.ldk;
    const int first = g.pair_first[o], last = g.pair_first[o + 1];
    for (int t = first; t < last; t++) {
        const int8_t* ap = g.a_planes + (size_t)g.pair_a[t] * g.a_plane_stride + lane * 16;
        const int8_t* bp = g.b_planes + (size_t)g.pair_b[t] * g.b_plane_stride + (size_t)cb * block_bytes + lane * 16;
        for (int gi = 0; gi < groups; gi++) {
            v4i_t b[GS], areg[PASSES];
#pragma unroll
            for (int s = 0; s < GS; s++)
                b[s] = __builtin_nontemporal_load((const v4i_t*)(bp + (size_t)gi * (GS * 1024) + s * 1024));
#pragma unroll
            for (int ps = 0; ps < PASSES; ps++) {
                const int f = ps * 4 + wave;
                if (FRAGS % 4 == 0 || f < FRAGS)
                    areg[ps] = *(const v4i_t*)(ap + (size_t)(f / GS) * block_bytes + (size_t)gi * (GS * 1024) + (f % GS) * 1024);
            }
            __syncthreads();                      /* the group before has been multiplied */
#pragma unroll
            for (int ps = 0; ps < PASSES; ps++) {
                const int f = ps * 4 + wave;
                if (FRAGS % 4 == 0 || f < FRAGS) *(v4i_t*)(abuf + f * 1024 + lane * 16) = areg[ps];
            }
            __syncthreads();
#pragma unroll
            for (int s = 0; s < GS; s++)
#pragma unroll
                for (int rb = 0; rb < RB; rb++)
                    acc[rb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[s], *(const v4i_t*)(abuf + (rb * GS + s) * 1024 + lane * 16),
                                                                    acc[rb], 0, 0, 0);
        }
    }
    int p = 1, c20 = 0;
    float pinv = 1.0f;
    if (g.mode == 1) { p = g.modulus[o]; c20 = (1 << 20) % p; pinv = 1.0f / (float)p; }
    /* lane%32 is the output row, registers 4v .. 4v+3 are columns 8v + 4 (lane/32) + 0..3 */
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        const int row = rb * 32 + li;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int col = cb * 32 + 8 * v + 4 * lh;
            if (row >= (int)g.out_rows || col >= (int)g.ldn) continue;
            const v4i_t s = {acc[rb][4 * v], acc[rb][4 * v + 1], acc[rb][4 * v + 2], acc[rb][4 * v + 3]};
            store_four(g, o, row, col, s, p, c20, pinv);
        }
    }
}

int g_thin_variant = 0;      /* tuning: 1, 2: column blocks per workgroup of the first kernel; 3: the second kernel; 0: by the shape */

}  // namespace

extern "C" void hip_igemm_set_thin_variant(int v) { EshkolHipLock lk; g_thin_variant = (v >= 1 && v <= 3) ? v : 0; }

/* Whether hip_igemm_i8 sends interleaved planes of an M x N product here (not while a test
 * forces a tiled kernel). By M and N alone, so that a tier that pads its planes for these
 * kernels and the entry point that routes to them cannot disagree. */
int eshkol_hip_igemm_direct_mode(void);
bool eshkol_hip_igemm_is_thin(uint64_t M, uint64_t N) {
    if (eshkol_hip_igemm_direct_mode() != 1 || M < 1) return false;
    return M <= 128 || (M <= 160 && N >= 4096);
}

/* Arguments as hip_igemm_i8 has checked them (layout 1, output pitch and rows filled in);
 * the first operand's planes need M rounded up to 32 rows only. */
int eshkol_hip_igemm_thin(const HipIgemmArgs& a, hipStream_t st) {
    if (a.M < 1 || a.M > 160 || a.layout != 1 || a.ldk % 512 != 0) return -1;
    const unsigned col_blocks = (a.N + 31) / 32;
    if (a.n_out > 65535u) return -1;
    const int rb = (int)((a.M + 31) / 32);
    const bool many = (uint64_t)col_blocks * a.n_out >= 2048;     /* column blocks over all output planes */
    /* 33 ... 64 rows: the second kernel where it has a workgroup or two for every CU */
    const bool rows = g_thin_variant == 3 || rb > 2 || (rb == 2 && many && g_thin_variant == 0);
    if (rows) {
        const dim3 grid((col_blocks + 3) / 4, a.n_out);
#define ROWS(RB, GS) hipLaunchKernelGGL((igemm_i8_rows_kernel<RB, GS>), grid, dim3(256), 0, st, a)
        switch (rb) {
            case 1: ROWS(1, 8); break;
            case 2: ROWS(2, 8); break;
            case 3: ROWS(3, 8); break;
            case 4: ROWS(4, 8); break;
            default: ROWS(5, 4); break;
        }
#undef ROWS
        return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
    }
    /* two column blocks per workgroup (the first operand's fragments then serve both) where
     * that still leaves a couple of thousand workgroups */
    const int cb = (g_thin_variant == 1 || g_thin_variant == 2) ? g_thin_variant : (many ? 2 : 1);
    const dim3 grid((col_blocks + cb - 1) / cb, a.n_out);
#define THIN(RB, CB, ST) hipLaunchKernelGGL((igemm_i8_thin_kernel<RB, CB, ST>), grid, dim3(256), 0, st, a)
    if (rb == 1) { if (cb == 1) THIN(1, 1, 8); else THIN(1, 2, 8); }
    else { if (cb == 1) THIN(2, 1, 8); else THIN(2, 2, 8); }
#undef THIN
    return ESHKOL_HIP_OK(hipGetLastError()) ? 0 : -1;
}
