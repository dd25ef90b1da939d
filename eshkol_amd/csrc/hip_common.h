/*
 * Internal declarations shared by the translation units of libeshkol_gpu_hip.so.
 * Nothing here is part of the public ABI.
 */
#ifndef ESHKOL_HIP_COMMON_H
#define ESHKOL_HIP_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <stdio.h>

#define ESHKOL_HIP_OK(call) ((call) == hipSuccess)

/* Log to stderr with the reference's "[GPU] " prefix when ESHKOL_GPU_VERBOSE is
 * set (reference gpu_memory_cuda.cpp:25-38). */
int eshkol_hip_verbose(void);
#define GPU_LOG(fmt, ...) \
    do { if (eshkol_hip_verbose()) fprintf(stderr, "[GPU] " fmt "\n", ##__VA_ARGS__); } while (0)

/* The one stream every kernel of the library is launched on. */
hipStream_t eshkol_hip_stream(void);

/* Grow-only device workspace slots, kept for the life of the process so a
 * matmul does not pay hipMalloc/hipFree per call. Returns NULL on failure. */
enum {
    WS_APLANES = 0, /* int8 planes of A                                   */
    WS_BPLANES,     /* int8 planes of B (transposed, K contiguous)        */
    WS_PRODUCTS,    /* int8 residue products / int32 diagonal buffers     */
    WS_ROWSCALE,    /* per-row fp64 scale or max, then int shifts         */
    WS_COLSCALE,    /* per-column fp64 scale or max, then int shifts      */
    WS_ROWSHIFT,
    WS_COLSHIFT,
    WS_HALF_A,      /* 16-bit copies of A, B and fp32 C for the reduced tier */
    WS_HALF_B,
    WS_F32_C,
    WS_COLPARTIAL,  /* per-slice partial column maxima                       */
    WS_DGEMM_PARTIAL, /* partial tiles of a k-split last round of the fp64 GEMM */
    WS_DGEMM_PAD_A, /* copies of fp64 operands whose rows do not start on 16-byte  */
    WS_DGEMM_PAD_B, /* boundaries, at an even pitch                                */
    WS_MISC,
    WS_COUNT
};
void* eshkol_hip_workspace(int slot, size_t bytes);
void  eshkol_hip_workspace_release(void);

/* What each tier keeps for the life of the process besides the workspace (small
 * device tables, the scan's pinned mailbox, stream and event): released by
 * eshkol_gpu_shutdown(), with the library mutex held and the device idle; the
 * next call after a new eshkol_gpu_init() makes them again. */
void eshkol_hip_crt_release(void);
void eshkol_hip_fast_release(void);
void eshkol_hip_int8_release(void);

/* Brackets a public tier entry point (hip_matmul_*, hip_dgemm_*, hip_igemm_i8,
 * hip_colabsmax_f64): takes the library's recursive mutex, the one the eshkol_*
 * entry points hold, and, if the previous bracketed call queued its work on
 * another stream, waits until the device is idle. The tiers share the grow-only workspace, the scan
 * mailbox and per-process tables; with the bracket, callers on several threads
 * or streams are serialised on the host and their kernels on the device. */
void eshkol_hip_enter(hipStream_t stream);
void eshkol_hip_leave(hipStream_t stream);
struct EshkolHipCall {
    hipStream_t st;
    explicit EshkolHipCall(void* stream) : st((hipStream_t)stream) { eshkol_hip_enter(st); }
    ~EshkolHipCall() { eshkol_hip_leave(st); }
    EshkolHipCall(const EshkolHipCall&) = delete;
    EshkolHipCall& operator=(const EshkolHipCall&) = delete;
};

/* The same mutex without the stream bookkeeping: for the process-wide switches
 * and read-outs of gpu_hip_testing.h, so that none changes under a call that
 * is inside the library. */
void eshkol_hip_lock(void);
void eshkol_hip_unlock(void);
struct EshkolHipLock {
    EshkolHipLock() { eshkol_hip_lock(); }
    ~EshkolHipLock() { eshkol_hip_unlock(); }
    EshkolHipLock(const EshkolHipLock&) = delete;
    EshkolHipLock& operator=(const EshkolHipLock&) = delete;
};

/* Looks up, once per device, the current device's address of the static scratch
 * array behind hip_matmul_reduced_f64_noalloc (hgemm_16.hip). 0 on success. */
int eshkol_hip_noalloc_setup(void);

/* compute units of the current device (256 if the query fails) */
static inline int eshkol_hip_num_cus(void) {
    static int cached = 0;
    if (cached == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached = n;
    }
    return cached;
}

static inline size_t round_up_sz(size_t v, size_t m) { return (v + m - 1) / m * m; }

/* Rows and row pitch of the product planes a tier puts between its contraction and
 * its reconstruction (HipIgemmArgs.out_rows, ldn). A pitch of a multiple of 16
 * elements keeps every store of the contraction and every load of the
 * reconstruction a vector one whatever N is; from 1024 on both are rounded up to
 * the contraction's 256 x 256 tile, which then has no bound to check anywhere. */
static inline uint64_t eshkol_product_rows(uint64_t M) { return M >= 1024 ? round_up_sz(M, 256) : M; }
static inline uint64_t eshkol_product_pitch(uint64_t N) { return N >= 1024 ? round_up_sz(N, 256) : round_up_sz(N, 16); }

/* A store whose line nothing on the device reads again soon (operand planes on
 * their way to HBM: gigabytes written once, read by a later kernel): the
 * non-temporal form keeps such lines from displacing what the caches hold and
 * measured 5-7 % on the kernels that mix reads and writes about evenly
 * (slices of 8192^2: 0.203 -> 0.190 ms). Only for stores that fill whole lines by
 * themselves or with their neighbours in the wave: 8-byte pieces of a line sent
 * this way are not merged on the way out (the slice tier's reconstruction ran
 * twice as long with them). */
/* The int8 contraction for a first operand of a few rows (igemm_thin_i8.hip): whether a
 * product of M x N output planes is one (up to 128 rows, up to 160 against 4096 columns or
 * more); hip_igemm_i8 sends interleaved planes of such a product there, and the tiers then
 * pad the first operand's planes to whole blocks of 32 rows instead of 256. */
bool eshkol_hip_igemm_is_thin(uint64_t M, uint64_t N);

/* fp64 products of matrices far smaller than a tile, one or a batch (dgemm_small_f64.hip) */
bool eshkol_hip_dgemm_is_small(uint64_t M, uint64_t K, uint64_t N);
int eshkol_hip_dgemm_small(const double* A, const double* B, double* C, uint64_t M, uint64_t K, uint64_t N,
                           int trans_a, int trans_b, uint64_t batch, hipStream_t st);

bool eshkol_hip_dgemm_is_small_long_k(uint64_t M, uint64_t K, uint64_t N);
int eshkol_hip_dgemm_small_long_k(const double* A, const double* B, double* C, uint64_t M, uint64_t K, uint64_t N,
                                  int trans_a, int trans_b, hipStream_t st);

/* One vector against a matrix held with k contiguous (dgemv_f64.hip): whether the shape is
 * one, and the product itself. hip_dgemm_f64 and hip_dgemm_f64_ex send such shapes there. */
bool eshkol_hip_dgemm_is_matvec(uint64_t M, uint64_t K, uint64_t N, int trans_a, int trans_b);
int eshkol_hip_dgemm_matvec(const double* A, const double* B, double* C, uint64_t M, uint64_t K, uint64_t N,
                            int trans_a, int trans_b, hipStream_t st);

/* fp64 products with up to 64 rows on the thin side: the big operand streamed through the
 * matrix cores (dgemm_thin_f64.hip) */
bool eshkol_hip_dgemm_is_thin_rows(uint64_t M, uint64_t K, uint64_t N, int trans_a, int trans_b);
int eshkol_hip_dgemm_thin_rows(const double* A, const double* B, double* C, uint64_t M, uint64_t K, uint64_t N,
                               int trans_a, int trans_b, hipStream_t st);

#ifdef __HIPCC__
template <class T>
__device__ __forceinline__ void eshkol_store_streaming(T* p, T v) { __builtin_nontemporal_store(v, p); }
#endif

#endif
