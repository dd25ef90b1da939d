/*
 * Reading an operand the caller stores k-major (X[K][R], the row index
 * contiguous: B as the runtime holds it) as if it were X^T[R][K], without a
 * transposed copy in HBM. The split, slice and narrowing kernels all want two
 * consecutive k of one row per thread, so that a wave writes 128 contiguous
 * output bytes per plane; this helper gives them exactly that view.
 *
 * A block owns 32 rows of X^T by 128 k. It reads the 128 x 32 tile with the row
 * index across lanes (256 contiguous bytes per k, 16 bytes per lane), parks it
 * in LDS as [32][128+2] doubles, and hands thread t the pairs (row q/64,
 * k 2(q%64)), q = t, t+256, ... The pad keeps the 16-byte LDS reads
 * conflict-free.
 */
#ifndef ESHKOL_HIP_KMAJOR_TILE_H
#define ESHKOL_HIP_KMAJOR_TILE_H

#include <hip/hip_runtime.h>
#include <stdint.h>

/* Byte offset of element (row, k) inside one int8 / 16-bit operand plane with a
 * row pitch of ld bytes (k counted in bytes). layout 0: [rows][ld]. layout 1,
 * "interleaved": rows in blocks of 32, inside a block the 16-byte k-chunks slow
 * and the row fast, so that the 32-row x 32-byte operand fragment of a 32x32
 * matrix-core instruction is 1 KiB of contiguous memory (gemm_pipe2.h). */
__device__ __forceinline__ uint64_t eshkol_plane_offset(int layout, uint64_t row, uint64_t k, uint64_t ld) {
    return layout ? (row >> 5) * (32 * ld) + (k >> 4) * 512 + (row & 31) * 16 + (k & 15) : row * ld + k;
}

namespace kmaj {

typedef double d2_t __attribute__((ext_vector_type(2)));

constexpr int TK = 128;
constexpr int TR = 32;
constexpr int LD = TK + 2;
constexpr int SMEM_DOUBLES = TR * LD;

/* tiles covering rows_ext rows by k_ext k-values (both may exceed the matrix: padding) */
inline uint64_t tile_count(uint64_t rows_ext, uint64_t k_ext) {
    return ((rows_ext + TR - 1) / TR) * ((k_ext + TK - 1) / TK);
}

/* Tile number -> tile. Tiles are numbered in groups of `group` row tiles: inside
 * a group the row tile runs fastest, then k, so blocks that run together read
 * group * 256 contiguous bytes of each k-line of X and, between them, write whole
 * output rows. group = 1 walks k first; group >= the number of row tiles walks
 * the rows first. */
__device__ __forceinline__ void tile_of_index(uint32_t idx, uint32_t group, uint32_t rt, uint32_t kt,
                                              uint32_t* rtile, uint32_t* ktile) {
    if (group > rt) group = rt;
    const uint32_t per = group * kt;
    const uint32_t g = idx / per, rem = idx - g * per;
    const uint32_t left = rt - g * group, gl = left < group ? left : group;
    *ktile = rem / gl;
    *rtile = g * group + rem % gl;
}

/* A block's share of a 128 x 32 tile of X, held in registers on its way to LDS:
 * a lane takes two neighbouring rows of eight k, so 16 lanes read 256 contiguous
 * bytes; zero outside the R x K matrix. */
struct TileRegs { double v0[TK / 16], v1[TK / 16]; uint32_t ok0, ok1; };

/* No branch around a load and no use of a loaded value: a lane outside the
 * matrix reads element 0 and remembers to discard it, so all eight loads of a
 * tile are in flight together and stay in flight until park_tile. */
__device__ __forceinline__ void load_tile(const double* __restrict__ X, uint64_t R, uint64_t K,
                                          uint64_t r0, uint64_t k0, TileRegs& t) {
    const int tid = threadIdx.x;
    const int lr = 2 * (tid & 15), lk = tid >> 4;
    const uint64_t gr = r0 + lr;
    const bool in0 = gr < R, in1 = gr + 1 < R;
    t.ok0 = 0; t.ok1 = 0;
    if (((R & 1) == 0) && (((uintptr_t)X & 15) == 0)) {
        const double* p = X + (k0 + lk) * R + gr;
#pragma unroll
        for (int i = 0; i < TK / 16; i++) {
            const bool ok = in0 && k0 + lk + 16 * i < K;
            const d2_t v = *(const d2_t*)(ok ? p + (uint64_t)(16 * i) * R : X);
            t.v0[i] = v.x; t.v1[i] = v.y;
            t.ok0 |= (uint32_t)ok << i;
        }
        t.ok1 = t.ok0;
    } else {
        const double* p = X + (k0 + lk) * R + gr;
#pragma unroll
        for (int i = 0; i < TK / 16; i++) {
            const bool kin = k0 + lk + 16 * i < K;
            const bool ok0 = kin && in0, ok1 = kin && in1;
            const double* q = p + (uint64_t)(16 * i) * R;
            t.v0[i] = *(ok0 ? q : X);
            t.v1[i] = *(ok1 ? q + 1 : X);
            t.ok0 |= (uint32_t)ok0 << i;
            t.ok1 |= (uint32_t)ok1 << i;
        }
    }
}

__device__ __forceinline__ void park_tile(const TileRegs& t, double* lds) {
    const int tid = threadIdx.x;
    const int lr = 2 * (tid & 15), lk = tid >> 4;
#pragma unroll
    for (int i = 0; i < TK / 16; i++) {
        lds[lr * LD + lk + 16 * i] = (t.ok0 >> i & 1) ? t.v0[i] : 0.0;
        lds[(lr + 1) * LD + lk + 16 * i] = (t.ok1 >> i & 1) ? t.v1[i] : 0.0;
    }
}

/* The tiles of a block: blockIdx.x, blockIdx.x + gridDim.x, ... While one tile is
 * worked on out of LDS, the next is already on its way from HBM into registers,
 * so a block always has 32 KiB of reads in flight. rowval(row) is the per-row
 * parameter of the caller (a shift, a scale); it travels with the tile, so the
 * consumer never waits on a dependent global load. body(r0, k0, rowvals) consumes
 * the tile in LDS; rowvals[r] belongs to row r0 + r. */
template <class RowVal, class Body>
__device__ __forceinline__ void for_each_tile(const double* __restrict__ X, uint64_t R, uint64_t K,
                                              uint64_t rows_ext, uint64_t k_ext, uint32_t group, double* lds,
                                              RowVal rowval, Body body) {
    typedef decltype(rowval((uint64_t)0)) RV;
    __shared__ RV rowvals[TR];
    const uint32_t rt = (uint32_t)((rows_ext + TR - 1) / TR), kt = (uint32_t)((k_ext + TK - 1) / TK);
    const uint32_t total = rt * kt;
    const int tid = threadIdx.x;
    uint32_t rtile, ktile;
    TileRegs regs;
    RV rv = RV();
    uint32_t idx = blockIdx.x;
    if (idx >= total) return;
    tile_of_index(idx, group, rt, kt, &rtile, &ktile);
    load_tile(X, R, K, (uint64_t)rtile * TR, (uint64_t)ktile * TK, regs);
    if (tid < TR) rv = rowval((uint64_t)rtile * TR + tid);
    while (true) {
        const uint64_t r0 = (uint64_t)rtile * TR, k0 = (uint64_t)ktile * TK;
        park_tile(regs, lds);
        if (tid < TR) rowvals[tid] = rv;
        __syncthreads();
        idx += gridDim.x;
        const bool more = idx < total;
        if (more) {
            tile_of_index(idx, group, rt, kt, &rtile, &ktile);
            load_tile(X, R, K, (uint64_t)rtile * TR, (uint64_t)ktile * TK, regs);
            if (tid < TR) rv = rowval((uint64_t)rtile * TR + tid);
        }
        body(r0, k0, rowvals);
        if (!more) break;
        __syncthreads();
    }
}

/* how many blocks to launch for that loop: every tile if they all fit on the chip
 * at once (four blocks per CU), else exactly that many blocks */
inline uint64_t grid_blocks(uint64_t rows_ext, uint64_t k_ext, int num_cus) {
    const uint64_t total = ((rows_ext + TR - 1) / TR) * ((k_ext + TK - 1) / TK);
    const uint64_t resident = 4ull * (uint64_t)(num_cus > 0 ? num_cus : 256);
    return total < resident ? total : resident;
}

/* emit(row, k, x0, x1, rowval(row)) for every even k < k_ext and every row <
 * rows_ext; x is 0 outside the R x K matrix. 256 threads. A wave writes 128
 * contiguous output bytes per plane.
 * The emit loops are not unrolled: the bodies are long, and keeping four waves
 * per SIMD resident matters more here than instruction-level overlap. */
template <class RowVal, class Emit>
__device__ __forceinline__ void for_each_pair(const double* __restrict__ X, uint64_t R, uint64_t K,
                                              uint64_t rows_ext, uint64_t k_ext, uint32_t group, double* lds,
                                              RowVal rowval, Emit emit) {
    for_each_tile(X, R, K, rows_ext, k_ext, group, lds, rowval, [&](uint64_t r0, uint64_t k0, const auto* rowvals) {
        const int tid = threadIdx.x;
#pragma unroll 1
        for (int i = 0; i < TR * TK / 2 / 256; i++) {
            const int q = tid + 256 * i;
            const int r = q >> 6, kp = q & 63;
            const uint64_t row = r0 + r, k = k0 + 2 * kp;
            if (row < rows_ext && k < k_ext) {
                const d2_t v = *(const d2_t*)(lds + r * LD + 2 * kp);
                emit(row, k, v.x, v.y, rowvals[r]);
            }
        }
    });
}

/* The same handed out sixteen k at a time: emit(row, k, x[16], rowval(row)) for
 * every k < k_ext that is a multiple of 16 (k_ext must be one); one group per
 * thread and tile. Eight lanes write 128 contiguous output bytes per plane with
 * 16-byte stores. */
template <class RowVal, class Emit>
__device__ __forceinline__ void for_each_16(const double* __restrict__ X, uint64_t R, uint64_t K,
                                            uint64_t rows_ext, uint64_t k_ext, uint32_t group, double* lds,
                                            RowVal rowval, Emit emit) {
    static_assert(TR * TK / 16 == 256, "one group of sixteen per thread");
    for_each_tile(X, R, K, rows_ext, k_ext, group, lds, rowval, [&](uint64_t r0, uint64_t k0, const auto* rowvals) {
        const int tid = threadIdx.x;
        const int r = tid >> 3, kc = tid & 7;
        const uint64_t row = r0 + r, k = k0 + 16 * kc;
        if (row < rows_ext && k < k_ext) {
            double x[16];
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const d2_t v = *(const d2_t*)(lds + r * LD + 16 * kc + 2 * e);
                x[2 * e] = v.x; x[2 * e + 1] = v.y;
            }
            emit(row, k, x, rowvals[r]);
        }
    });
}

/* Interleaved planes need no trip through LDS. There a thread that owns sixteen
 * consecutive k of one row writes one 16-byte chunk per plane, and 32 such
 * threads on 32 neighbouring rows write 512 contiguous bytes; a wave on 64
 * neighbouring rows reads 512 contiguous bytes of every k-line of X. A block of
 * 256 threads takes 64 rows x 64 k: row r0 + tid % 64, k from k0 + 16 (tid / 64).
 * (Measured at 8192^2 with sixteen planes: 319 us, against 327 for 32 rows x 128 k,
 * 321-324 for 128 or 256 rows, 330-337 for a loop that prefetches its next tile,
 * and 345 for the tile parked in LDS above; the row block runs fastest over the
 * grid, every other order measured 1-10 % slower.) */
constexpr int IL_ROWS = 64, IL_K = 64;

/* blocks covering rows_ext x k_ext */
inline uint64_t il_blocks(uint64_t rows_ext, uint64_t k_ext) {
    return ((rows_ext + IL_ROWS - 1) / IL_ROWS) * ((k_ext + IL_K - 1) / IL_K);
}

__device__ __forceinline__ void il_thread(uint64_t rows_ext, uint64_t* row, uint64_t* k) {
    const uint32_t rt = (uint32_t)((rows_ext + IL_ROWS - 1) / IL_ROWS);
    const uint32_t kb = blockIdx.x / rt, rb = blockIdx.x - kb * rt;
    *row = (uint64_t)rb * IL_ROWS + (threadIdx.x & 63);
    *k = (uint64_t)kb * IL_K + 16 * (threadIdx.x >> 6);
}

/* x[e] = X[k + e][row], zero outside the R x K matrix. All sixteen loads are
 * issued before the first value is looked at (a lane outside the matrix reads
 * element 0 and discards it). */
__device__ __forceinline__ void load_k16(const double* __restrict__ X, uint64_t R, uint64_t K,
                                         uint64_t row, uint64_t k, double* x) {
    const bool rin = row < R;
    const double* p = X + k * R + row;
    uint32_t ok = 0;
#pragma unroll
    for (int e = 0; e < 16; e++) {
        const bool in = rin && k + e < K;
        x[e] = *(in ? p + (uint64_t)e * R : X);
        ok |= (uint32_t)in << e;
    }
#pragma unroll
    for (int e = 0; e < 16; e++) x[e] = (ok >> e & 1) ? x[e] : 0.0;
}

}  // namespace kmaj
#endif
