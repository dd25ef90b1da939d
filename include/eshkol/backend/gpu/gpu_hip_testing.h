/*
 * Test and benchmark hooks of libeshkol_gpu_hip.so, and the device probe of
 * libeshkol_gpu_probe.so. NOT part of the product ABI: a runtime that links the
 * library needs gpu_memory.h (and gpu_hip_tiers.h if it calls tiers directly)
 * and nothing from this file. None of these has a counterpart in the reference.
 *
 * The hip_*_set_* switches are process-wide and read by later calls; each takes
 * the library's recursive mutex, so a switch never changes under a call that is
 * inside the library, but a caller that wants one setting for a group of calls
 * has to keep other threads out itself. The *_last_stages read-outs hand out
 * pointers into the library's workspace: valid until the next tier call on any
 * thread.
 */
#ifndef ESHKOL_GPU_HIP_TESTING_H
#define ESHKOL_GPU_HIP_TESTING_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- stage read-outs, for parity checks of each stage on its own ------------ */

/* Stage outputs of the last hip_matmul_ozaki_crt_f64 call, for parity checks:
 * device pointers into the library workspace (valid until the next call). */
typedef struct {
    const int8_t* a_planes; const int8_t* b_planes; const int8_t* w_planes;
    const int32_t* mu; const int32_t* nu;
    uint64_t rows_a_padded, rows_b_padded, ldk;
    int32_t num_moduli, E;
    int32_t layout;             /* of a_planes and b_planes: HipIgemmArgs.layout */
    uint64_t w_rows, w_ld;      /* w_planes is [num_moduli][w_rows][w_ld]: the products' M x N corner counts */
} HipOzakiCrtStages;
int hip_ozaki_crt_last_stages(HipOzakiCrtStages* out);

/* Device pointers to the stages of the last hip_matmul_ozaki_fast_f64 call (valid
 * until the next tier call): residue planes [l][row padded to 256][ldk] of A and
 * of B^T, product residues [l][w_rows][w_ld] (the M x N corner counts), the per-row and per-column shifts
 * E - frexp exponent (0 for an all-zero row), and the moduli. */
typedef struct {
    const int8_t* a_planes;
    const int8_t* b_planes;
    const int8_t* w_planes;
    const int32_t* shift_a;
    const int32_t* shift_b;
    uint64_t rows_a_padded, rows_b_padded, ldk;
    int32_t num_moduli, E, cap;
    int32_t moduli[16];
    int32_t layout;             /* of a_planes and b_planes: HipIgemmArgs.layout */
    uint64_t w_rows, w_ld;      /* w_planes is [num_moduli][w_rows][w_ld] */
} HipOzakiFastStages;
int hip_ozaki_fast_last_stages(HipOzakiFastStages* out);

/* Stages of the last hip_matmul_ozaki_int8_f64 call. */
typedef struct {
    const int8_t* a_slices; const int8_t* b_slices; const int32_t* products;
    const double* rmax; const double* cmax;
    uint64_t rows_a_padded, rows_b_padded, ldk;
    int32_t s, nbuf;
    int32_t layout;             /* of a_slices and b_slices: HipIgemmArgs.layout */
    uint64_t g_rows, g_ld;      /* products is [nbuf][g_rows][g_ld] */
} HipOzakiInt8Stages;
int hip_ozaki_int8_last_stages(HipOzakiInt8Stages* out);

/* ---- switches between code paths that give the same results ------------------ */

/* 0 sends every fp64 product through the bounds-checked kernel; 1 (default)
 * lets launches of at least 256 tiles with even row pitches, 16-byte aligned
 * operands and K >= 16 take the straight-line kernel. Both give the same bits;
 * the switch exists to compare them. */
void hip_dgemm_set_fast_path(int on);

/* 1 (default): when the last round of 128 x 128 tiles of a large product would
 * leave more than half of the CUs idle, or a product has too few tiles to fill
 * the device at all, those tiles are cut along k, the pieces multiplied side by
 * side and added in a fixed order (deterministic, but the summation order of
 * those tiles differs from an unsplit launch); 0: every tile is multiplied
 * whole. */
void hip_dgemm_set_tail_split(int on);

/* Tile size of the straight-line fp64 kernel. 0: 128 x 128 only; 1 (default):
 * 64 x 64 tiles for the launches expected to finish sooner with them (large
 * tiles would leave CUs idle or a round of tiles half empty, and k is too short
 * for cutting them along k to pay: 1024^3, 2304 x 2304 x 2048, 3072^3 ...);
 * 2: 64 x 64 wherever that kernel applies. The summation order inside a tile
 * is the same, so all three give the same bits as long as no tile is cut
 * along k. */
void hip_dgemm_set_small_tile(int mode);

/* How many k-blocks the straight-line fp64 kernels' global loads run ahead of
 * their LDS writes. 0 (default) and 2: two, wherever that variant holds its
 * registers; 1: one. Same bits; the switch exists to compare them. */
void hip_dgemm_set_prefetch_depth(int depth);

/* Fewest rows on the thin side that take the kernels which stream the big operand
 * through the matrix cores without tiles (1, the default: every product with up to 64
 * thin rows that qualifies; 0: none, such shapes then take the tiled kernels). The
 * summation order differs between the two, the tolerance is the tier's. */
void hip_dgemm_set_thin_rows(int from);
/* The same for the two refinements of that path, for measurements: big operands with k
 * contiguous (1 default), and more than 64 thin rows in chunks of 64 (1 default). */
void hip_dgemm_set_thin_rows_klast(int on);
void hip_dgemm_set_thin_chunks(int on);

/* Which of the int8 kernels for a first operand of a few rows runs: 0 (default) by the
 * shape; 1 or 2: the kernel for up to 64 rows with that many column blocks per workgroup;
 * 3: the kernel that shares the rows through LDS. Same results. */
void hip_igemm_set_thin_variant(int column_blocks);

/* k-blocks kept in flight by the pipelined int8 kernel (1..3; 0 = simple kernel only). */
void hip_igemm_set_prefetch(int pf);

/* 1 (default): contractions with at least 128 tiles (the CRT tiers: 16 tiles and
 * 1024 of k) take interleaved operand
 * planes and the kernels that load them straight into LDS and MFMA registers
 * (256 x 128 tiles and two workgroups per CU for products of at most 1024 bytes
 * of k and for launches with no more 256 x 256 tiles than CUs, 256 x 256 tiles and
 * one otherwise); 2: the 256 x 128 kernel for all of
 * them; 3: the 256 x 256 kernel for all of them; 0: row-major planes and the
 * register-staged kernels everywhere. With 1, a first operand of a few rows
 * takes the kernels that stream the second operand's planes (any other value
 * keeps such products on the kernels named). Same results; the switch exists to
 * compare them. */
void hip_igemm_set_direct(int on);

/* Workgroups of the persistent 256 x 256 int8 kernel: 0 (default) one per CU;
 * n > 0 at most n (rounded down to a multiple of 8), which leaves the other CUs
 * to kernels queued on other streams. For measuring what running the streaming
 * stages beside the contraction would cost and gain. */
void hip_igemm_set_cu_limit(int cus);

/* The same switch for the 16-bit tier. */
void hip_hgemm_set_direct(int on);

/* 1 (default): the reduced tier on up to 128 rows or columns against a big operand reads
 * that operand once, as fp64, and narrows it in registers on its way to the matrix cores;
 * 0: narrowing kernels and the tiled contraction, as for every other shape. Same
 * arithmetic, another order of the fp32 sums. */
void hip_reduced_set_thin(int on);

/* 1 (default): the pipelined int8 kernel runs as one workgroup per CU walking a
 * list of tiles, its operand stream continuous across tile boundaries; 0: one
 * workgroup per tile. Same results; the switch exists to compare them. */
void hip_igemm_set_persistent(int on);

/* 1 (default): a few long rows (at most 160, k from 1024 on) in front of a prepared second
 * operand get their maxima, their shifts and the scan of the maxima from one launch; 0:
 * from the three kernels every other shape uses. Same results. */
void hip_ozaki_crt_set_fused_scan(int on);

/* 0 (default): the CRT tier finds floor(log2) of the row and column maxima and
 * the few maxima that can carry the largest fractional part of log2 on the
 * device, and the host calls log2 on those few only; 1: the host takes log2 of
 * every maximum, as gpu_memory.mm:376-420 does. Same E, shifts and results (the
 * first falls back to the second whenever a maximum lies within 2^-40 of a power
 * of two); the switch exists to compare them. */
void hip_ozaki_crt_set_host_pass(int on);

/* ---- libeshkol_gpu_probe.so (built beside the library, loaded by bench.py only) --
 * Rate the device sustains on a register-only MFMA loop (kind 0 fp64 flop/s,
 * 1 int8 op/s, 2 bf16 flop/s; random_operands != 0 uses random operand bits,
 * under which the chip clocks down to hold its power limit) or on a large copy
 * (kind 3, bytes/s read+written). The counterpart of the reference's
 * self-calibrating peak model (gpu_memory_cuda.cpp:499-522), measured rather
 * than seeded. Synchronises the stream; allocates and frees
 * its own buffers. */
int hip_probe_peak(int kind, int random_operands, double* rate, void* stream);

/* Which vector ALU instructions a SIMD runs beside another wave's MFMAs: the time
 * (ms) of four waves of back-to-back int8 MFMAs per CU (constant or random operand
 * bits), of four waves of vector ALU instructions per CU (kind 0: v_fma_f32, 1:
 * v_dot4_u32_u8, 2: the instruction mix of a residue epilogue, which holds one byte
 * dot product in nine instructions, 3: that mix with a shift and a 24-bit
 * multiply-add in the dot product's place; valu_iters iterations), and of both
 * sharing the SIMDs two waves each. With the vector ALU waves the shorter ones,
 * both = mfma: entirely beside the MFMAs; both = mfma + valu: not at all. With
 * them the longer ones, (mfma + valu - both) / mfma is their rate beside the MFMAs
 * relative to their rate alone. What the 256 x 128 int8 contraction with two
 * workgroups per CU rests on. */
int hip_probe_coissue(int kind, int random_operands, int valu_iters,
                      double* mfma_ms, double* valu_ms, double* both_ms, void* stream);

#ifdef __cplusplus
}
#endif
#endif
