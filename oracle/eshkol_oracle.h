/*
 * CPU oracle for the Eshkol tensor-matmul GPU hot path.
 *
 * TEST INFRASTRUCTURE ONLY. This is a plain-C restatement of the reference's
 * arithmetic for each matmul tier. It exists to check the HIP kernels; nothing
 * in the shipped library links, loads or calls it. Only tests/, the smoke check
 * and the cpu_baseline leg of bench.py may use it.
 *
 * Every function cites the reference file:line it follows (paths are relative
 * to the root of tsotchke/eshkol).
 *
 * Pinning status (how each restatement is itself checked):
 *   oracle_matmul_f64 / oracle_batch_matmul_f64 / oracle_reduce_precision:
 *       bit-for-bit against the reference's own translation units compiled
 *       into oracle/_ref/libeshkol_ref.so, plus committed golden vectors.
 *   oracle_ozaki_int8_*: closed forms (slice recomposition, brute-force int64
 *       products) and the reference's buffer-plan invariants.
 *   oracle_ozaki_crt_*: exact __int128 dot products on integer inputs, the
 *       reference's certification witness, CRT constant identities.
 *   The cBLAS branch of the reference CPU matmul lives in a third-party
 *   library (system OpenBLAS / Accelerate) that is not in the tree:
 *   parity unpinned beyond the small exact-integer cases the reference tests.
 */
#ifndef ESHKOL_ORACLE_H
#define ESHKOL_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- native fp64 tier (lib/backend/blas_backend.cpp) -------------------- */

/* Select which build of the reference the fp64 restatement mirrors: 1 (default)
 * = -mavx2 -mfma (AVX 4x8 kernel, fused multiply-add); 0 = flag-less x86-64
 * build (SSE2 4x4 kernel, blas_backend.cpp:669-763, unfused). */
void oracle_matmul_set_fused(int fused);

/* matmul_scalar, blas_backend.cpp:407-419: i-j-k, one accumulator per output.
 * The reference is built with -mfma and GCC's default contraction, so the
 * multiply-add is a fused one; stated here with explicit fma(). */
void oracle_matmul_scalar_f64(const double* A, const double* B, double* C,
                              uint64_t M, uint64_t K, uint64_t N);

/* matmul_simd_avx + avx_microkernel_4x8 + avx_scalar_block,
 * blas_backend.cpp:550-658: C zeroed, 64^3 blocking (i0,j0,k0 nest), inside a
 * k-block every output accumulates fma over k ascending from 0.0, then C += acc. */
void oracle_matmul_blocked_f64(const double* A, const double* B, double* C,
                               uint64_t M, uint64_t K, uint64_t N);

/* eshkol_matmul_f64, blas_backend.cpp:791-906, non-BLAS build: M*N <= 16 ->
 * scalar, otherwise the blocked kernel. */
void oracle_matmul_f64(const double* A, const double* B, double* C,
                       uint64_t M, uint64_t K, uint64_t N);

/* eshkol_batch_matmul_f64, lib/core/runtime_tensor_math.cpp:796-817: naive
 * i-k-j per batch entry, C zeroed first (fused or not per oracle_matmul_set_fused). */
void oracle_batch_matmul_f64(const double* a, const double* b, double* c,
                             int64_t batch, int64_t M, int64_t K, int64_t N);

/* eshkol_matmul_backward_f64, blas_backend.cpp:924-1039 (the scalar loops of a
 * non-BLAS, non-GPU build): grad_A[MxK] = grad_out[MxN] * B^T, grad_B[KxN] =
 * A^T * grad_out, each output accumulated in ascending contraction order. */
void oracle_matmul_backward_f64(const double* grad_out, const double* saved_A, const double* saved_B,
                                double* grad_A, double* grad_B,
                                uint64_t M, uint64_t K, uint64_t N);

/* ---- reduced-precision tier (lib/core/runtime_tensor_dtype.cpp) ---------- */

/* reduce_precision, runtime_tensor_dtype.cpp:37-145. dtype codes: 0 f64,
 * 1 f32, 2 f16, 3 bf16, 4 i8. Round to nearest even; storage stays double. */
double oracle_reduce_precision(double v, int64_t dtype);
void   oracle_reduce_precision_array(const double* in, double* out, size_t n, int64_t dtype);

/* Reference CPU statement of the reduced tier: the f64 GEMM over inputs already
 * rounded to the 16-bit format (gpu_memory_stub.cpp:391-397 ignores dtype).
 * Rounds A and B through `dtype` first, then oracle_matmul_f64. */
void oracle_matmul_reduced(const double* A, const double* B, double* C,
                           uint64_t M, uint64_t K, uint64_t N, int64_t dtype);

/* cuda_matmul_f16_from_f64, gpu_memory_cuda.cpp:678-728: operands narrowed to
 * the 16-bit type, products accumulated in fp32 (k ascending here; the GPU
 * library's order is unspecified), optional rounding of the result to the
 * 16-bit type (round_output != 0 is what the CUDA path does). */
void oracle_matmul_reduced_f32acc(const double* A, const double* B, double* C,
                                  uint64_t M, uint64_t K, uint64_t N,
                                  int64_t dtype, int round_output);

/* ---- INT8 slice tier (gpu_cuda_kernels.cu:663-741, gpu_memory_cuda.cpp:339-452) */

/* ozaki_rowmax_f64_kernel / ozaki_colmax_f64_kernel, gpu_cuda_kernels.cu:664-684. */
void oracle_ozaki_rowmax_f64(const double* A, uint64_t M, uint64_t K, double* rmax);
void oracle_ozaki_colmax_f64(const double* B, uint64_t K, uint64_t N, double* cmax);

/* ozaki_split_a_f64_kernel, gpu_cuda_kernels.cu:688-703. slices[p*M*K + i*K + k]. */
void oracle_ozaki_split_a_f64(const double* A, uint64_t M, uint64_t K,
                              const double* rmax, int s, int8_t* slices);
/* ozaki_split_b_f64_kernel, gpu_cuda_kernels.cu:707-723. Stored transposed:
 * slices[q*K*N + j*K + k]. */
void oracle_ozaki_split_b_f64(const double* B, uint64_t K, uint64_t N,
                              const double* cmax, int s, int8_t* slices);

/* Buffer plan of cuda_matmul_ozaki_int8_f64, gpu_memory_cuda.cpp:363-389.
 * Returns nbuf (<= max_buf) or -1 (K beyond the int32-exact bound, or overflow
 * of the caller's arrays). pair_p/pair_q hold the (p,q) pairs buffer after
 * buffer; buf_first[b]..buf_first[b+1] indexes them (buf_first has nbuf+1 slots). */
int oracle_ozaki_int8_plan(uint64_t K, int T, int max_buf, int max_pairs,
                           double* weights, int* buf_first,
                           int* pair_p, int* pair_q);

/* The cublasGemmEx loop, gpu_memory_cuda.cpp:415-434: exact int32
 * G_b[i,j] = sum over the buffer's pairs of sum_k A_p[i,k]*B_q[k,j]. */
void oracle_ozaki_int8_products(const int8_t* As, const int8_t* Bs,
                                uint64_t M, uint64_t K, uint64_t N,
                                int nbuf, const int* buf_first,
                                const int* pair_p, const int* pair_q,
                                int32_t* Gall);

/* ozaki_reconstruct_f64_kernel, gpu_cuda_kernels.cu:728-741. */
void oracle_ozaki_reconstruct_f64(double* C, const int32_t* Gall,
                                  const double* weights, int nbuf,
                                  const double* rmax, const double* cmax,
                                  uint64_t M, uint64_t N);

/* Whole pipeline. Returns 0, or -1 where the reference returns -1. */
int oracle_matmul_ozaki_int8_f64(const double* A, const double* B, double* C,
                                 uint64_t M, uint64_t K, uint64_t N, int T);

/* ---- Ozaki-II CRT exact tier (gpu_memory.mm:227-453, 2474-2665) ---------- */

#define ORACLE_OZAKI_MAX_MODULI 16
extern const int ORACLE_OZAKI_MODULI[49];   /* gpu_memory.mm:227-233 */

typedef struct {
    double P1, P2;              /* P = P1 + P2 exactly (to the bits P2 keeps) */
    double Pinv;
    double sl1[ORACLE_OZAKI_MAX_MODULI], sl2[ORACLE_OZAKI_MAX_MODULI];
    int    q[ORACLE_OZAKI_MAX_MODULI];
    int    num_moduli;
    double log2P;
} OracleCRTConstants;

/* precompute_ozaki_constants, gpu_memory.mm:301-341 (n clamped to [2,16] as
 * get_ozaki_crt does, 344-359). */
void oracle_ozaki_crt_constants(int n, OracleCRTConstants* crt);
/* the same constants with the weights split at one common bit position (not the reference's split) */
void oracle_ozaki_crt_constants_aligned(int n, OracleCRTConstants* crt);
void oracle_ozaki_crt_use_aligned_weights(int on);

/* ozaki_compute_frac_bounds, gpu_memory.mm:376-420. */
void oracle_ozaki_frac_bounds(const double* A, const double* B,
                              uint64_t M, uint64_t K, uint64_t N,
                              double* frac_A, double* frac_B);
/* ozaki_compute_adaptive_N, gpu_memory.mm:433-453. */
int oracle_ozaki_adaptive_n(const double* A, const double* B,
                            uint64_t M, uint64_t K, uint64_t N, int max_moduli);

/* Scaling exponent and shifts, gpu_memory.mm:2510-2532. mu[M], nu[N]. */
int oracle_ozaki_crt_scaling(const double* A, const double* B,
                             uint64_t M, uint64_t K, uint64_t N,
                             const OracleCRTConstants* crt,
                             int* mu, int* nu);

/* Residue planes, gpu_memory.mm:2538-2583 with the residue taken by exact
 * integer arithmetic: A' = trunc(A*2^mu_i) as an integer, residue in
 * [-p/2, p/2) (so p = 256 maps 128 to -128; the reference's float formula may
 * give +128 there, the same class mod 256).
 * a_planes[l*M*K + i*K + k]; b_planes[l*N*K + j*K + k] (transposed, K contiguous). */
void oracle_ozaki_crt_split_a(const double* A, uint64_t M, uint64_t K,
                              const int* mu, int num_moduli, int8_t* a_planes);
void oracle_ozaki_crt_split_b(const double* B, uint64_t K, uint64_t N,
                              const int* nu, int num_moduli, int8_t* b_planes);

/* matmul_ozaki_gemm, metal_softfloat.h:3907-4100: W_l = symmetric residue of
 * sum_k a_l[i,k]*b_l[k,j] mod p_l, as int8 in [-p/2, p/2). w_planes[l*M*N + i*N + j].
 * If acc32 is not NULL it also receives the raw int32 sums (same layout). */
void oracle_ozaki_crt_products(const int8_t* a_planes, const int8_t* b_planes,
                               uint64_t M, uint64_t K, uint64_t N, int num_moduli,
                               int8_t* w_planes, int32_t* acc32);

/* CRT accumulation + reconstruction + inverse scaling, gpu_memory.mm:2626-2655. */
void oracle_ozaki_crt_reconstruct(const int8_t* w_planes, uint64_t M, uint64_t N,
                                  const OracleCRTConstants* crt,
                                  const int* mu, const int* nu, double* C);

/* ozaki_ii_dispatch, gpu_memory.mm:2474-2665. num_moduli in [2,16]; adaptive
 * != 0 selects the count as ESHKOL_OZAKI_ADAPTIVE=1 does. Returns 0, or -1 when
 * an input is non-finite or a scale factor leaves the double range (the
 * reference is undefined there; the GPU library falls back to native fp64). */
int oracle_matmul_ozaki_crt_f64(const double* A, const double* B, double* C,
                                uint64_t M, uint64_t K, uint64_t N,
                                int num_moduli, int adaptive);

/* The same tier with the representatives the reference's floating-point residue
 * formulas give (mode 1: gpu_memory.mm:2573-2583 applied to the exact sum; mode 2:
 * the Metal kernel's partial reductions every 1008 k, metal_softfloat.h:3907-4100):
 * the half-way class of the modulus 256 comes out as +128 or -128 there, always
 * -128 above. n_half / n_plus count the elements in that class / those returned
 * as +128. Test infrastructure for quantifying what the choice changes. */
void oracle_ozaki_crt_products_refrep(const double* A, const double* B,
                                      uint64_t M, uint64_t K, uint64_t N,
                                      const int* mu, const int* nu, int num_moduli, int mode,
                                      int16_t* w16);
int oracle_matmul_ozaki_crt_refrep_f64(const double* A, const double* B, double* C,
                                       uint64_t M, uint64_t K, uint64_t N,
                                       int num_moduli, int mode,
                                       uint64_t* n_half, uint64_t* n_plus);

/* ---- MLP layer (BASELINE config 5) --------------------------------------- */

/* y = tanh(x*W + b): matmul via the exact tier, then the broadcast add
 * (runtime_tensor_math.cpp:672-740) and glibc tanh (lib/core/model_io.cpp:709).
 * X[batch x in], W[in x out], b[out] (may be NULL), Y[batch x out]. */
int oracle_mlp_layer_f64(const double* X, const double* W, const double* b, double* Y,
                         uint64_t batch, uint64_t in_f, uint64_t out_f,
                         int num_moduli);

#ifdef __cplusplus
}
#endif
/* ---- Ozaki-II reduced-precision ("fast") CRT tier (gpu_memory.mm:2802-3012,
 *      metal_softfloat.h:4126-4246) ------------------------------------------ */
typedef struct {
    int num_moduli, cap, E;
    int moduli[16];
    int q[16];                  /* (P / p_l)^-1 mod p_l */
    double log2P, P;
    float P_hi, P_lo;           /* P as a float pair */
} OracleFastConstants;

int  oracle_ozaki_fast_cap(uint64_t K);
int  oracle_ozaki_fast_moduli(int cap, int n_mod, int* out);
int  oracle_ozaki_fast_constants(uint64_t K, int n_mod_req, OracleFastConstants* c);
void oracle_ozaki_fast_exponents(const double* A, const double* B, uint64_t M, uint64_t K, uint64_t N,
                                 int32_t* ei, int32_t* fj);
/* planes [n][rows][K] int8; scaled (optional) [rows][K] int64: the integers the residues are taken of */
void oracle_ozaki_fast_split_a(const double* A, uint64_t M, uint64_t K, const int32_t* ei,
                               const OracleFastConstants* c, int8_t* planes, int64_t* scaled);
void oracle_ozaki_fast_split_b(const double* B, uint64_t K, uint64_t N, const int32_t* fj,
                               const OracleFastConstants* c, int8_t* planes, int64_t* scaled);
void oracle_ozaki_fast_products(const int8_t* a_planes, const int8_t* b_planes, uint64_t M, uint64_t K, uint64_t N,
                                int n, int32_t* G);
void oracle_ozaki_fast_reconstruct(const int32_t* G, uint64_t M, uint64_t N, const OracleFastConstants* c,
                                   const int32_t* ei, const int32_t* fj, double* C);
void oracle_ozaki_fast_exact_value(const int64_t* a_scaled, const int64_t* b_scaled, uint64_t M, uint64_t K, uint64_t N,
                                   const OracleFastConstants* c, const int32_t* ei, const int32_t* fj, double* C);
int  oracle_matmul_ozaki_fast_f64(const double* A, const double* B, double* C,
                                  uint64_t M, uint64_t K, uint64_t N, int n_mod);

#endif
