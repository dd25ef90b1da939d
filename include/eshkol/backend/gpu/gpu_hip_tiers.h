/*
 * Per-tier and per-stage entry points of libeshkol_gpu_hip.so.
 *
 * These are the AMD counterparts of the launchers the reference's CUDA
 * translation unit binds from its kernel file
 * (lib/backend/gpu/gpu_memory_cuda.cpp:52-100: cuda_launch_*_f64,
 * cuda_ozaki_split_a_f64, cuda_ozaki_split_b_f64, cuda_ozaki_reconstruct_f64)
 * and of its static tier functions (cuda_matmul_ozaki_int8_f64 :339-452,
 * cuda_matmul_f16_from_f64 :678-728, ozaki_ii_dispatch gpu_memory.mm:2474-2771).
 * The runtime reaches them through eshkol_gpu_matmul_f64 /
 * eshkol_matmul_dispatch; they are exported so that each stage can be checked
 * on its own against the reference arithmetic.
 *
 * Conventions: plain C, device pointers, sizes as uint64_t in (M, K, N) order,
 * `stream` is a hipStream_t passed as void* (NULL = the null stream). Return 0
 * on success, -1 on a bad argument, an unsupported shape or a launch failure.
 * Launchers do not synchronise. eshkol_gpu_init() must have succeeded first.
 *
 * Threads and streams. The tier pipelines (hip_matmul_*), hip_dgemm_f64*,
 * hip_igemm_i8, hip_hgemm_16 and hip_colabsmax_f64 share the library's cached
 * device workspace and per-process tables. Each of them takes the library's
 * one recursive mutex (the same the eshkol_* entry points hold) for the length
 * of the call and, when its stream differs from the stream of the previous such
 * call, first waits on the host until the device is idle (consecutive calls on
 * one stream, the usual case, are ordered by the stream and pay nothing): they
 * may be called from any thread, on any stream, beside eshkol_* calls, and are
 * serialised on the host and on the device. The stage launchers (split, slice, convert, reconstruct,
 * rowabsmax, transpose, elementwise, bias) touch only the memory they are
 * given and take no lock. hip_matmul_reduced_f64_noalloc takes no lock and
 * orders nothing (see there). The switches and stage read-outs that tests and
 * the benchmark use are not part of this header: gpu_hip_testing.h.
 */
#ifndef ESHKOL_GPU_HIP_TIERS_H
#define ESHKOL_GPU_HIP_TIERS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The stream all library work is issued on (hipStream_t), for callers that
 * bracket calls with their own events. NULL before eshkol_gpu_init(). */
void* eshkol_hip_get_stream(void);

/* ---- native fp64 tier ------------------------------------------------------
 * C = A*B on the fp64 matrix cores; replaces the cublasDgemm call at
 * gpu_memory_cuda.cpp:633-640 (alpha 1, beta 0, row-major, no leading dims). */
int hip_dgemm_f64(const double* A, const double* B, double* C,
                  uint64_t M, uint64_t K, uint64_t N, void* stream);

/* C[MxN] = op(A)*op(B) with an operand held transposed: trans_a != 0 means A
 * points at A^T stored [K][M]; trans_b != 0 means B points at B^T stored
 * [N][K] (not both). What cblas_dgemm's CblasTrans flags give the reference's
 * backward pass (lib/backend/blas_backend.cpp:1013-1024); its GPU branch makes
 * transposed host copies instead (:969-977). */
int hip_dgemm_f64_ex(const double* A, const double* B, double* C,
                     uint64_t M, uint64_t K, uint64_t N,
                     int trans_a, int trans_b, void* stream);

/* batch dense products stored back to back (A [batch][M][K], B [batch][K][N],
 * C [batch][M][N]) in one launch, the batch index on the grid's second axis:
 * the f64 counterpart of the strided-batched call the reference has for 16-bit
 * tensors only (gpu_memory_cuda.cpp:763-771); its f64 batches run the CPU loop
 * (lib/core/runtime_tensor_math.cpp:796-817). */
int hip_dgemm_f64_batched(const double* A, const double* B, double* C,
                          uint64_t batch, uint64_t M, uint64_t K, uint64_t N, void* stream);

/* Single precision, replaces cublasSgemm at gpu_memory_cuda.cpp:658-665. */
int hip_sgemm_f32(const float* A, const float* B, float* C,
                  uint64_t M, uint64_t K, uint64_t N, void* stream);

/* ---- shared streaming kernels --------------------------------------------- */

/* out[cols x rows] = in[rows x cols]^T; cuda_launch_transpose_f64,
 * gpu_cuda_kernels.cu:189-213. */
int hip_transpose_f64(const double* in, double* out, uint64_t rows, uint64_t cols, void* stream);

/* rmax[i] = max_k |A[i,k]|, with zero_value substituted for an all-zero row:
 * 1.0 gives ozaki_rowmax_f64_kernel (gpu_cuda_kernels.cu:664-673), 0.0 gives
 * the row maxima of ozaki_ii_dispatch (gpu_memory.mm:2517-2524). One wave per
 * row instead of the reference's one thread per row. */
int hip_rowabsmax_f64(const double* A, uint64_t M, uint64_t K, double zero_value,
                      double* rmax, void* stream);

/* cmax[j] = max_k |X[k,j]| of a row-major X[K][R], same conventions as
 * hip_rowabsmax_f64: the column maxima of B without transposing it
 * (ozaki_colmax_f64_kernel, gpu_cuda_kernels.cu:675-685). Uses the library
 * workspace. */
int hip_colabsmax_f64(const double* X, uint64_t K, uint64_t R, double zero_value,
                      double* cmax, void* stream);

/* The 15 operations of EshkolElementwiseOp; cuda_launch_elementwise_f64,
 * gpu_cuda_kernels.cu:21-43. b may be NULL (identity operand). */
int hip_elementwise_f64(const double* a, const double* b, double* out, uint64_t n, int op, void* stream);

/* In place Y[i,j] = act(Y[i,j] + bias[j]); act 0 none, 1 tanh. bias may be
 * NULL. The dense-layer epilogue (broadcast add runtime_tensor_math.cpp:672-740,
 * tanh lib/core/model_io.cpp:709) for tiers that do not fuse it. */
int hip_bias_act_f64(double* Y, const double* bias, uint64_t rows, uint64_t cols, int act, void* stream);

/* ---- int8 matrix-core contraction ------------------------------------------
 * Replaces the cublasGemmEx(int8 x int8 -> int32) loop at
 * gpu_memory_cuda.cpp:415-434 and the modular GEMM matmul_ozaki_gemm
 * (metal_softfloat.h:3907-4100). Operand planes are K-contiguous int8 with a
 * row pitch of ldk bytes (multiple of 128, zero padded beyond K) and row counts
 * padded with zero rows to multiples of 256 (interleaved planes of a first operand
 * of at most 128 rows, or 160 where N >= 4096: to multiples of 32; such products take
 * kernels of their own that stream the second operand's planes once). The pipelined kernel needs ldk to
 * be a multiple of 256, 1 <= max_pairs <= 64 and every output plane to have at
 * least one product (pair_first strictly increasing); pass max_pairs = 0 for
 * plans with empty planes: they take the simple kernel, which writes zeros. */
typedef struct {
    const int8_t* a_planes;   /* [n_a_planes][rows_a_padded][ldk]                */
    const int8_t* b_planes;   /* [n_b_planes][rows_b_padded][ldk]                */
    uint64_t a_plane_stride;  /* bytes between consecutive A planes              */
    uint64_t b_plane_stride;
    uint32_t ldk;
    uint32_t M, N;            /* logical output size                             */
    uint32_t n_out;           /* number of output planes                         */
    /* Output plane o is the int32 sum of the products pair_first[o] ..
     * pair_first[o+1]-1; product t multiplies A plane pair_a[t] by B plane
     * pair_b[t]. The three arrays live in device memory.                        */
    const int32_t* pair_first;
    const int32_t* pair_a;
    const int32_t* pair_b;
    /* mode 0: out_i32[o][out_rows][ldn] = the int32 sums
     * mode 1: out_i8[o][out_rows][ldn]  = the sum modulo modulus[o], representative
     *         in [-p/2, p/2); modulus[] in device memory                        */
    int32_t mode;
    int32_t max_pairs;        /* upper bound on products per output plane (host knows the plan) */
    const int32_t* modulus;
    int32_t* out_i32;
    int8_t*  out_i8;
    /* 0: planes are [rows][ldk]. 1: interleaved, the layout the tiers use for
     * products that fill the device: rows in blocks of 32, inside a block the
     * 16-byte k-chunks slow and the row fast,
     *   offset(row, k) = (row/32) * 32*ldk + (k/16) * 512 + (row%32) * 16 + k%16,
     * so the 32-row x 32-byte operand fragment of one matrix-core instruction is
     * 1 KiB of contiguous memory. Needs ldk % 512 == 0 and max_pairs >= 1 (every
     * output plane at least one product). */
    int32_t layout;
    /* The output planes as allocated: out_rows rows of ldn elements each (0: M and
     * N, dense planes). With ldn a multiple of 16 (4 for mode 0) every store is a
     * 16-byte one whatever N is, and with out_rows and ldn multiples of 256 no tile
     * has a bound to check. Elements outside M x N come from the operands' zero
     * padding: they are written as zeros, or not at all where no tile covers them. */
    uint32_t ldn;
    uint32_t out_rows;
} HipIgemmArgs;
int hip_igemm_i8(const HipIgemmArgs* args, void* stream);

/* The layout (HipIgemmArgs.layout) the tiers give their operand planes for a
 * contraction of n_out output planes of M x N: 1 when the launch has at least
 * 128 tiles of 256 x 256 and so takes the direct-to-LDS kernel, or when M is at
 * most 128 (160 where N >= 4096: the kernels for a few rows), else 0. With 1 the k
 * pitch is padded to a multiple of 512. */
int hip_igemm_plane_layout(uint64_t M, uint64_t N, int n_out);
/* The rule of the two CRT tiers, whose contractions are one product per output plane over
 * K of k: 1 as above, and also from sixteen tiles of 256 x 256 and K >= 1024 on (such
 * launches take a kernel on 256 x 128 tiles that the plans of several products per plane
 * cannot use). */
int hip_igemm_plane_layout_single(uint64_t M, uint64_t K, uint64_t N, int n_out);

/* ---- Ozaki-II CRT exact tier ------------------------------------------------
 * Residue planes of trunc(X[i,k] * 2^shift[i]) modulo the first num_moduli
 * entries of the reference's modulus table (gpu_memory.mm:227-233, 2538-2583):
 * planes[l][i][k], representative in [-p/2, p/2), pitch ldk, rows_padded rows
 * per plane (padding written as zeros). Used for A directly and for B through
 * its transpose, so both operands come out K-contiguous. */
int hip_ozaki_crt_split_f64(const double* X, uint64_t rows, uint64_t K,
                            const int32_t* shift, int num_moduli,
                            int8_t* planes, uint64_t rows_padded, uint64_t ldk, void* stream);

/* The same planes from a k-major operand X[K][rows] (B as the runtime stores
 * it): output identical to hip_ozaki_crt_split_f64 on X^T. */
int hip_ozaki_crt_split_kmajor_f64(const double* X, uint64_t rows, uint64_t K,
                                   const int32_t* shift, int num_moduli,
                                   int8_t* planes, uint64_t rows_padded, uint64_t ldk, void* stream);

/* Either of the two with the plane layout as an argument (HipIgemmArgs.layout;
 * layout 1 needs rows_padded and ldk to be multiples of 32 and planes 16-byte
 * aligned). */
int hip_ozaki_crt_split_planes_f64(const double* X, uint64_t rows, uint64_t K,
                                   const int32_t* shift, int num_moduli,
                                   int8_t* planes, uint64_t rows_padded, uint64_t ldk,
                                   int kmajor, int layout, void* stream);

/* CRT accumulation, reconstruction and inverse scaling (gpu_memory.mm:2626-2655)
 * from the int8 residue products w_planes[l][M][N]; optional fused dense-layer
 * epilogue C = act(C + bias[j]) (act 0 none, 1 tanh; bias may be NULL). */
int hip_ozaki_crt_reconstruct_f64(const int8_t* w_planes, uint64_t M, uint64_t N, int num_moduli,
                                  const double* sl1, const double* sl2,
                                  double P1, double P2, double Pinv,
                                  const int32_t* mu, const int32_t* nu,
                                  const double* bias, int act,
                                  double* C, void* stream);

/* Whole tier: ozaki_ii_dispatch (gpu_memory.mm:2474-2665). num_moduli in
 * [2,16]; adaptive != 0 picks the count as ESHKOL_OZAKI_ADAPTIVE=1 does.
 * Returns -1 (caller falls back to the native tier) for K > 131071, non-finite
 * input, or scale factors outside the double range; the last two are found
 * after the products have been queued, so C then holds no result. */
int hip_matmul_ozaki_crt_f64(const double* A, const double* B, double* C,
                             uint64_t M, uint64_t K, uint64_t N,
                             int num_moduli, int adaptive,
                             const double* bias, int act, void* stream);

/* A second operand that does not change between calls (a layer's weights),
 * prepared once: the tier keeps what it derives from B alone (column maxima,
 * residue planes: num_moduli * roundup(N,256) * roundup(K,512) bytes of device
 * memory) in *handle, and hip_matmul_ozaki_crt_prepared_f64 then splits only A.
 * No counterpart in the reference, which re-wraps and re-splits every operand
 * on every call (gpu_memory_cuda.cpp:1136-1145, gpu_memory.mm:2538-2583). The
 * result is the one hip_matmul_ozaki_crt_f64_ex gives on the same operands, bit
 * for bit: the planes are the same bytes. Prepared only where the exponent E
 * does not depend on the operands (sixteen moduli at every K the tier accepts;
 * -1 otherwise, and for a B with non-finite entries or a column maximum within
 * 2^-40 of a power of two; -2 when device memory for the planes cannot be had). M_expected is the row count of the products to
 * come: it selects the plane layout (hip_igemm_plane_layout). Interleaved planes
 * (layout 1) then serve products of every row count; row-major planes serve the
 * products that would make row-major planes themselves, and a call whose shape
 * wants interleaved ones, or adaptive != 0, simply splits B again. B
 * must stay valid and unchanged while the handle lives; eshkol_gpu_resident_pin
 * tensors get this treatment by themselves when the dispatcher routes a product
 * to this tier. */
int hip_ozaki_crt_prepare_operand_b(const double* B, uint64_t K, uint64_t N, int trans_b,
                                    int num_moduli, uint64_t M_expected, void** handle, void* stream);
int hip_matmul_ozaki_crt_prepared_f64(const double* A, const void* prepared_b, double* C,
                                      uint64_t M, uint64_t K, uint64_t N, int trans_a,
                                      int num_moduli, int adaptive,
                                      const double* bias, int act, void* stream);
void hip_ozaki_crt_release_prepared(void* handle);

/* How the CRT weights s_l = (P / p_l) q_l are split into the two doubles the
 * accumulation uses. 0 (default): as the reference does (gpu_memory.mm:322-337),
 * each relative to its own exponent; results equal the reference's bit for bit,
 * including its defect: the upper parts then end at different bits, their
 * weighted sum is not always representable, and on general operands about one
 * element in 150 is wrong by 2^-25 of a typical element. 1: at one common bit
 * position, which makes that sum exact (normwise error about 1e-17; same
 * kernels, same residues and products). The environment variable
 * ESHKOL_OZAKI_CRT_WEIGHTS=aligned selects 1 for the dispatcher's calls, and
 * the accuracy-budget selector uses 1 when it picks this tier. Returns the
 * previous setting. */
int hip_ozaki_crt_set_aligned_weights(int on);

/* ---- Ozaki-II reduced-precision ("fast") CRT tier -------------------------------
 * ozaki_ii_fast_dispatch (lib/backend/gpu/gpu_memory.mm:2816-3012): the n largest
 * prime powers below a K-dependent cap as moduli (gpu_memory.mm:2802-2842),
 * power-of-two scaling by the frexp exponents of the row / column maxima,
 * round-half-up integer split (metal_softfloat.h:4148-4178), exact modular
 * products, fractional CRT (metal_softfloat.h:4183-4246; here in fp64 instead of
 * float pairs). num_moduli is the accuracy knob, [2, 16], clamped; the
 * reference's default is 11 (about 1e-8). Returns 0, -4 where the reference
 * gives up (K too large for the moduli, fewer than two moduli under the cap),
 * -1 on non-finite input (found after the products were queued: C then holds
 * no result) or a device error, -2 when workspace cannot be had. */
int hip_matmul_ozaki_fast_f64(const double* A, const double* B, double* C,
                              uint64_t M, uint64_t K, uint64_t N, int num_moduli, void* stream);

/* The tier's two streaming stages on their own, with the moduli hip_ozaki_fast_plan
 * gives for (K, num_moduli): the split of one operand into residue planes
 * (shift[i] = E - 1 - floor(log2 max_i), 0 for an all-zero row; ldk a multiple
 * of 16; layout as HipIgemmArgs.layout) and the fractional CRT of the product
 * residues w_planes[l][M][N] back to fp64. */
int hip_ozaki_fast_split_planes_f64(const double* X, uint64_t rows, uint64_t K, const int32_t* shift,
                                    int num_moduli, int8_t* planes, uint64_t rows_padded, uint64_t ldk,
                                    int kmajor, int layout, void* stream);
int hip_ozaki_fast_reconstruct_f64(const int8_t* w_planes, uint64_t M, uint64_t N, uint64_t K, int num_moduli,
                                   const int32_t* shift_a, const int32_t* shift_b, double* C, void* stream);

/* What ESHKOL_MATMUL_ACCURACY=<budget> would choose for a product of this shape
 * (the selector of gpu_memory_cuda.cpp:546-566 with the two Ozaki-II tiers as
 * further candidates), without running anything; host arithmetic only. Returns
 * 0 native fp64, 1 INT8 slices (*T), 2 Ozaki-II exact tier with aligned
 * weights, 3 Ozaki-II reduced-precision tier (*fast_moduli); *speedup is the
 * cost model's predicted ratio to native. Pointers may be NULL. */
int hip_select_tier_for_budget(uint64_t M, uint64_t K, uint64_t N, double budget,
                               int32_t* T, int32_t* fast_moduli, double* speedup);

/* What that tier would use for a contraction length K and a requested moduli
 * count (gpu_memory.mm:2802-2857), without running anything: returns the number
 * of moduli (it can be below the request when too few prime powers fit under
 * the cap) or -4 where the tier gives up, and fills E (bits kept per operand),
 * cap and moduli[16] where the pointers are not NULL. The accuracy-budget
 * selector asks it for the smallest count whose E meets a budget. */
int hip_ozaki_fast_plan(uint64_t K, int num_moduli, int32_t* E, int32_t* cap, int32_t* moduli);

/* ---- INT8 slice tier ----------------------------------------------------------
 * s base-128 slices of X[i,k] / scale[i] (gpu_cuda_kernels.cu:688-723):
 * planes[p][i][k], pitch ldk, rows_padded rows per plane, padding zero. With
 * rows_padded == rows and ldk == K this is the reference's layout for A, and
 * for B when X is B transposed. */
int hip_ozaki_slice_f64(const double* X, uint64_t rows, uint64_t K, const double* scale, int s,
                        int8_t* planes, uint64_t rows_padded, uint64_t ldk, void* stream);

/* The same planes from a k-major operand X[K][rows]: the reference's B kernel
 * (gpu_cuda_kernels.cu:706-723); output identical to hip_ozaki_slice_f64 on X^T. */
int hip_ozaki_slice_kmajor_f64(const double* X, uint64_t rows, uint64_t K, const double* scale, int s,
                               int8_t* planes, uint64_t rows_padded, uint64_t ldk, void* stream);

/* Either of the two with the plane layout as an argument (HipIgemmArgs.layout). */
int hip_ozaki_slice_planes_f64(const double* X, uint64_t rows, uint64_t K, const double* scale, int s,
                               int8_t* planes, uint64_t rows_padded, uint64_t ldk,
                               int kmajor, int layout, void* stream);

/* cuda_ozaki_reconstruct_f64 (gpu_cuda_kernels.cu:728-741, 779-798), weights
 * already in device memory. */
int hip_ozaki_reconstruct_f64(double* C, const int32_t* Gall, const double* d_weights, int nbuf,
                              const double* rmax, const double* cmax,
                              uint64_t M, uint64_t N, void* stream);

/* Whole tier: cuda_matmul_ozaki_int8_f64 (gpu_memory_cuda.cpp:339-452), T in [1,8]. */
int hip_matmul_ozaki_int8_f64(const double* A, const double* B, double* C,
                              uint64_t M, uint64_t K, uint64_t N, int T, void* stream);

/* ---- reduced-precision tier ----------------------------------------------------
 * cuda_matmul_f16_from_f64 (gpu_memory_cuda.cpp:678-728) with the conversions
 * on the device: operands in f64 storage are narrowed to dtype 2 (f16) or 3
 * (bf16), multiplied on the matrix cores with fp32 accumulation, and written
 * back as f64. round_output != 0 rounds the fp32 result to the 16-bit type
 * first, as the reference's 16F output does. */
int hip_matmul_reduced_f64(const double* A, const double* B, double* C,
                           uint64_t M, uint64_t K, uint64_t N,
                           int dtype, int round_output, void* stream);

/* batch products stored back to back (A [batch][M][K], B [batch][K][N],
 * C [batch][M][N]) in one launch each of the two narrowing kernels and of the
 * contraction: the strided-batched call of the reference's 16-bit tier
 * (cuda_batch_matmul_f16_from_f64, gpu_memory_cuda.cpp:736-784). */
int hip_matmul_reduced_f64_batched(const double* A, const double* B, double* C,
                                   uint64_t batch, uint64_t M, uint64_t K, uint64_t N,
                                   int dtype, int round_output, void* stream);

/* The same product as hip_matmul_reduced_f64, for callers that cannot allocate
 * device memory: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc. It has no counterpart in the reference. The 16-bit
 * operand copies live in a device array that is part of the library's code
 * object (hip_matmul_reduced_f64_noalloc_limit() bytes per GPU, held until the
 * process ends) instead of the grow-only workspace, and the call reaches no
 * hipMalloc, hipFree or allocating library routine. Returns -3 with a message
 * on stderr when 2 * (roundup(M,256) + roundup(N,256)) * roundup(K,256) bytes
 * exceed that limit (for up to 128 rows or columns against an operand of two million
 * elements or more, which both entry points multiply without a 16-bit copy of it: also when
 * the fp32 partial sums of that kernel, at most 25 MiB, do not fit beside the
 * first operand's copy), otherwise what hip_matmul_reduced_f64 returns, and the
 * same bits in C. Every call on a GPU shares that GPU's array: calls that
 * overlap on one GPU (two streams, two threads) race. */
int hip_matmul_reduced_f64_noalloc(const double* A, const double* B, double* C,
                                   uint64_t M, uint64_t K, uint64_t N,
                                   int dtype, int round_output, void* stream);
size_t hip_matmul_reduced_f64_noalloc_limit(void);

/* 16-bit operands already in device memory (A [M][K], Bt [N][K], pitch ld
 * elements, multiple of 64, rows padded to multiples of 256 with zeros), fp32
 * result C[M][N]: the contraction alone (BASELINE configuration 4). Up to 128
 * rows against a second operand of two million elements or more read that
 * operand once, in slices of k whose fp32 partial sums (in the library's
 * workspace) a second kernel adds in ascending order. */
int hip_hgemm_16(const uint16_t* A, const uint16_t* Bt, uint64_t M, uint64_t K, uint64_t N,
                 uint64_t ld, int is_bf16, float* C, void* stream);

/* The contraction for a batch of products whose 16-bit operands are stored back
 * to back (A [batch][rows_a_padded][ld], Bt [batch][rows_b_padded][ld], both row
 * counts multiples of 256), result C [batch][M][N] fp32, one launch. layout 0:
 * operands [row][ld]. layout 1: interleaved (HipIgemmArgs.layout with k counted
 * in bytes; needs ld to be a multiple of 256 elements), the layout
 * hip_hgemm_plane_layout() says the tier uses when the launch has at least 128
 * tiles of 256 x 256 and M, N >= 192. */
int hip_hgemm_16_batched(const uint16_t* A, const uint16_t* Bt, uint64_t batch,
                         uint64_t M, uint64_t K, uint64_t N,
                         uint64_t rows_a_padded, uint64_t rows_b_padded, uint64_t ld,
                         int is_bf16, int layout, float* C, void* stream);
int hip_hgemm_plane_layout(uint64_t M, uint64_t N, uint64_t batch);

/* RNE narrowing of f64 storage to f16/bf16 (runtime_tensor_dtype.cpp:37-109),
 * out[i][k] with pitch ld and rows_padded rows, padding zero. */
int hip_convert_f64_to_16(const double* in, uint16_t* out, uint64_t rows, uint64_t cols,
                          uint64_t rows_padded, uint64_t ld, int is_bf16, void* stream);

/* The same narrowing from a k-major operand in[cols][rows]: out[i][k] = in[k][i]. */
int hip_convert_f64_to_16_kmajor(const double* in, uint16_t* out, uint64_t rows, uint64_t cols,
                                 uint64_t rows_padded, uint64_t ld, int is_bf16, void* stream);

/* Both narrowing kernels with batch and plane layout as arguments: `batch`
 * matrices stored back to back, kmajor != 0 for in[cols][rows], layout as in
 * hip_hgemm_16_batched (layout 1 needs rows_padded % 32 == 0, ld % 64 == 0). */
int hip_convert_f64_to_16_planes(const double* in, uint16_t* out, uint64_t batch, uint64_t rows, uint64_t cols,
                                 uint64_t rows_padded, uint64_t ld, int is_bf16,
                                 int kmajor, int layout, void* stream);

/* ---- operands held transposed, and the backward pass ---------------------------
 * The tier pipelines with the trans_a / trans_b meaning of hip_dgemm_f64_ex.
 * The Ozaki and reduced tiers turn both operands into planes [row][k]; an
 * operand stored k-major is read through LDS tiles, so neither form costs a
 * transposed copy. */
int hip_matmul_ozaki_fast_f64_ex(const double* A, const double* B, double* C,
                                 uint64_t M, uint64_t K, uint64_t N,
                                 int trans_a, int trans_b, int num_moduli, void* stream);
int hip_matmul_ozaki_crt_f64_ex(const double* A, const double* B, double* C,
                                uint64_t M, uint64_t K, uint64_t N,
                                int trans_a, int trans_b, int num_moduli, int adaptive,
                                const double* bias, int act, void* stream);
int hip_matmul_ozaki_int8_f64_ex(const double* A, const double* B, double* C,
                                 uint64_t M, uint64_t K, uint64_t N,
                                 int trans_a, int trans_b, int T, void* stream);
int hip_matmul_reduced_f64_ex(const double* A, const double* B, double* C,
                              uint64_t M, uint64_t K, uint64_t N,
                              int trans_a, int trans_b,
                              int dtype, int round_output, void* stream);

/* Gradients of C = A*B (eshkol_matmul_backward_f64, lib/backend/blas_backend.cpp:
 * 924-1039): grad_A[MxK] = grad_out[MxN] * B^T and grad_B[KxN] = A^T * grad_out,
 * straight from the saved row-major A[MxK] and B[KxN] with no transposed
 * copies (the reference's GPU branch transposes both on the host, :969-977).
 * tier: 0 native fp64, 1 INT8 slices with T, 2 Ozaki-II CRT (16 moduli).
 * Either gradient pointer may be NULL to skip it. */
int hip_matmul_backward_f64(const double* grad_out, const double* A, const double* B,
                            double* grad_A, double* grad_B,
                            uint64_t M, uint64_t K, uint64_t N,
                            int tier, int T, void* stream);

#ifdef __cplusplus
}
#endif
#endif
