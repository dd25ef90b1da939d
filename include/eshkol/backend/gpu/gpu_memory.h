/*
 * C ABI of the Eshkol GPU runtime, as exported by the MI355X (gfx950) backend.
 *
 * This header declares the same symbols, with the same signatures, argument
 * order (M, K, N) and return conventions, as the reference's
 * inc/eshkol/backend/gpu/gpu_memory.h:33-68 (types) and :90-474 (functions).
 * One translation unit per build provides them (reference CMakeLists.txt:
 * 1513-1514, 1622-1624, 1641); libeshkol_gpu_hip.so is that unit for AMD.
 * The only addition to the reference ABI is the enum value ESHKOL_GPU_HIP.
 *
 * Return conventions (reference gpu_memory.h:72-90, gpu_memory_cuda.cpp:839-1157):
 *   eshkol_gpu_init           1 = a GPU backend is active, 0 = CPU only
 *   every other int function  0 = success, negative = failure
 *   void dispatchers          never fail: they fall back to the runtime's CPU
 *                             matmul (eshkol_matmul_f64 / eshkol_batch_matmul_f64,
 *                             imported from the host runtime at link/load time)
 */
#ifndef ESHKOL_GPU_MEMORY_H
#define ESHKOL_GPU_MEMORY_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* reference gpu_memory.h:33-38; value 4 is new */
typedef enum {
    ESHKOL_GPU_NONE = 0,
    ESHKOL_GPU_METAL = 1,
    ESHKOL_GPU_CUDA = 2,
    ESHKOL_GPU_VULKAN = 3,
    ESHKOL_GPU_HIP = 4      /* AMD HIP, gfx950 */
} EshkolGPUBackend;

/* reference gpu_memory.h:40-45 */
typedef enum {
    ESHKOL_MEM_HOST = 0,
    ESHKOL_MEM_HOST_PINNED = 1,
    ESHKOL_MEM_DEVICE = 2,
    ESHKOL_MEM_UNIFIED = 3
} EshkolMemoryType;

/* reference gpu_memory.h:47-52 */
typedef enum {
    ESHKOL_SYNC_NONE = 0,
    ESHKOL_SYNC_HOST_TO_DEVICE,
    ESHKOL_SYNC_DEVICE_TO_HOST,
    ESHKOL_SYNC_BIDIRECTIONAL
} EshkolSyncDirection;

/* reference gpu_memory.h:60-68. Caller owns the struct; alloc/wrap fill it,
 * free releases what it names and zeroes it. */
typedef struct EshkolGPUBuffer {
    void* host_ptr;
    void* device_ptr;
    size_t size_bytes;
    EshkolMemoryType mem_type;
    EshkolGPUBackend backend;
    uint32_t flags;          /* bit0 wrapped host memory, bit1 copy back on sync/free */
    void* backend_data;      /* original host pointer of a staged wrap */
} EshkolGPUBuffer;

/* ---- device management: reference gpu_memory.h:90-149 -------------------- */
int eshkol_gpu_init(void);
void eshkol_gpu_shutdown(void);
EshkolGPUBackend eshkol_gpu_get_backend(void);
const char* eshkol_gpu_backend_name(EshkolGPUBackend backend);
int eshkol_gpu_backend_available(EshkolGPUBackend backend);
int eshkol_gpu_supports_f64(void);
int eshkol_gpu_has_fp64(void);

/* ---- memory: reference gpu_memory.h:164-224 ------------------------------ */
int eshkol_gpu_alloc(size_t size_bytes, EshkolMemoryType mem_type, EshkolGPUBuffer* out_buffer);
int eshkol_gpu_alloc_aligned(size_t size_bytes, size_t alignment,
                             EshkolMemoryType mem_type, EshkolGPUBuffer* out_buffer);
void eshkol_gpu_free(EshkolGPUBuffer* buffer);
int eshkol_gpu_wrap_host(void* host_ptr, size_t size_bytes, EshkolGPUBuffer* out_buffer);
int eshkol_gpu_sync(EshkolGPUBuffer* buffer, EshkolSyncDirection direction);
int eshkol_gpu_sync_async(EshkolGPUBuffer* buffer, EshkolSyncDirection direction,
                          void* stream_handle);
void eshkol_gpu_wait(EshkolGPUBuffer* buffer);

/* ---- matmul: reference gpu_memory.h:242-252 ------------------------------
 * C[MxN] = A[MxK] * B[KxN], row-major dense, alpha 1, beta 0, C overwritten.
 * Buffers carry device pointers. The f64 entry selects the tier from the
 * environment exactly where the reference's cuda_matmul_f64 does
 * (gpu_memory_cuda.cpp:577-650). */
int eshkol_gpu_matmul_f64(EshkolGPUBuffer* A, EshkolGPUBuffer* B, EshkolGPUBuffer* C,
                          uint64_t M, uint64_t K, uint64_t N);
int eshkol_gpu_matmul_f32(EshkolGPUBuffer* A, EshkolGPUBuffer* B, EshkolGPUBuffer* C,
                          uint64_t M, uint64_t K, uint64_t N);

/* Gradients of C = A*B: grad_A[MxK] = grad_out[MxN] * B^T and grad_B[KxN] =
 * A^T * grad_out from the saved row-major operands, same tier selection as
 * the forward product. An addition to the reference header: it replaces the
 * GPU branch inside eshkol_matmul_backward_f64 (lib/backend/blas_backend.cpp:
 * 968-1003), which transposes both operands on the host and calls
 * eshkol_gpu_matmul_f64 twice. Either gradient buffer may be NULL. */
int eshkol_gpu_matmul_backward_f64(EshkolGPUBuffer* grad_out, EshkolGPUBuffer* A, EshkolGPUBuffer* B,
                                   EshkolGPUBuffer* grad_A, EshkolGPUBuffer* grad_B,
                                   uint64_t M, uint64_t K, uint64_t N);

/* ---- resident host tensors -------------------------------------------------
 * An addition to the reference header. The reference's dispatchers wrap and
 * upload every operand on every call (gpu_memory_cuda.cpp:1136-1145), so a
 * weight matrix crosses the host link once per matmul. A tensor the runtime
 * declares stable keeps a device copy: eshkol_matmul_dispatch and
 * eshkol_batch_matmul_dispatch then use that copy for an input operand whose
 * host pointer matches, moving no bytes.
 *   pin      upload now (again if already pinned); 0 on success
 *   refresh  the host contents changed: upload again; -1 if not pinned
 *   unpin    drop the device copy
 *   bytes    device memory currently held by pinned tensors
 * The caller owns the contract that a pinned tensor is not modified on the
 * host without a refresh. eshkol_gpu_shutdown drops every copy. */
int eshkol_gpu_resident_pin(const void* host_ptr, size_t size_bytes);
int eshkol_gpu_resident_refresh(const void* host_ptr);
void eshkol_gpu_resident_unpin(const void* host_ptr);
size_t eshkol_gpu_resident_bytes(void);

/* ---- thresholds: reference gpu_memory.h:261-280 -------------------------- */
extern size_t g_gpu_threshold;
void eshkol_gpu_set_threshold(size_t threshold);
size_t eshkol_gpu_get_threshold(void);
int eshkol_gpu_should_use(size_t num_elements);

/* ---- elementwise / reductions: reference gpu_memory.h:284-397 ------------ */
typedef enum {
    ESHKOL_ELEMWISE_ADD = 0, ESHKOL_ELEMWISE_SUB = 1, ESHKOL_ELEMWISE_MUL = 2,
    ESHKOL_ELEMWISE_DIV = 3, ESHKOL_ELEMWISE_NEG = 4, ESHKOL_ELEMWISE_ABS = 5,
    ESHKOL_ELEMWISE_EXP = 6, ESHKOL_ELEMWISE_LOG = 7, ESHKOL_ELEMWISE_SIN = 8,
    ESHKOL_ELEMWISE_COS = 9, ESHKOL_ELEMWISE_TANH = 10, ESHKOL_ELEMWISE_RELU = 11,
    ESHKOL_ELEMWISE_SIGMOID = 12, ESHKOL_ELEMWISE_SQRT = 13, ESHKOL_ELEMWISE_RECIPROCAL = 14
} EshkolElementwiseOp;

typedef enum {
    ESHKOL_REDUCE_SUM = 0, ESHKOL_REDUCE_PROD = 1, ESHKOL_REDUCE_MIN = 2,
    ESHKOL_REDUCE_MAX = 3, ESHKOL_REDUCE_MEAN = 4
} EshkolReduceOp;

int eshkol_gpu_elementwise_f64(EshkolGPUBuffer* a, EshkolGPUBuffer* b, EshkolGPUBuffer* out,
                               uint64_t n, EshkolElementwiseOp op);
int eshkol_gpu_reduce_f64(EshkolGPUBuffer* in, EshkolGPUBuffer* out, uint64_t n, EshkolReduceOp op);
int eshkol_gpu_reduce_axis_f64(EshkolGPUBuffer* in, EshkolGPUBuffer* out, uint64_t rank,
                               const uint64_t* shape, uint64_t axis, EshkolReduceOp op);
int eshkol_gpu_transpose_f64(EshkolGPUBuffer* in, EshkolGPUBuffer* out, uint64_t rows, uint64_t cols);
int eshkol_gpu_softmax_f64(EshkolGPUBuffer* in, EshkolGPUBuffer* out,
                           uint64_t num_slices, uint64_t slice_len);
int eshkol_gpu_normalize_f64(EshkolGPUBuffer* in, EshkolGPUBuffer* out,
                             uint64_t num_slices, uint64_t slice_len,
                             double gamma, double beta, double epsilon);

/* ---- backward ops: reference gpu_memory.h:404-442. As in the reference's
 * no-GPU unit (gpu_memory_stub.cpp:417-449) these return -1 and the caller
 * runs its CPU rule; they are outside the matmul path. */
int eshkol_gpu_conv2d_backward_input_f64(
    EshkolGPUBuffer* grad_out, EshkolGPUBuffer* kernel_weights, EshkolGPUBuffer* grad_input,
    uint64_t in_h, uint64_t in_w, uint64_t k_h, uint64_t k_w, uint64_t out_h, uint64_t out_w,
    uint64_t stride_h, uint64_t stride_w, uint64_t channels_in, uint64_t channels_out,
    uint64_t batch_size);
int eshkol_gpu_conv2d_backward_kernel_f64(
    EshkolGPUBuffer* grad_out, EshkolGPUBuffer* saved_input, EshkolGPUBuffer* grad_kernel,
    uint64_t in_h, uint64_t in_w, uint64_t k_h, uint64_t k_w, uint64_t out_h, uint64_t out_w,
    uint64_t stride_h, uint64_t stride_w, uint64_t channels_in, uint64_t channels_out,
    uint64_t batch_size);
int eshkol_gpu_batchnorm_backward_f64(
    EshkolGPUBuffer* grad_out, EshkolGPUBuffer* saved_input, EshkolGPUBuffer* saved_mean,
    EshkolGPUBuffer* saved_inv_std, EshkolGPUBuffer* saved_gamma, EshkolGPUBuffer* grad_input,
    EshkolGPUBuffer* grad_gamma, EshkolGPUBuffer* grad_beta,
    uint64_t batch_size, uint64_t feature_size);
int eshkol_gpu_layernorm_backward_f64(
    EshkolGPUBuffer* grad_out, EshkolGPUBuffer* saved_input, EshkolGPUBuffer* saved_mean,
    EshkolGPUBuffer* saved_inv_std, EshkolGPUBuffer* saved_gamma, EshkolGPUBuffer* grad_input,
    uint64_t num_samples, uint64_t feature_size);

/* ---- runtime entry points: reference gpu_memory.h:466-474 ----------------
 * Host pointers, row-major. dtype is the result tensor's dtype code
 * (0 f64, 1 f32, 2 f16, 3 bf16, 4 i8); 2 and 3 take the reduced tier. */
void eshkol_matmul_dispatch(const double* A, const double* B, double* C,
                            uint64_t M, uint64_t K, uint64_t N, int32_t dtype);
void eshkol_batch_matmul_dispatch(const double* a, const double* b, double* c,
                                  int64_t batch, int64_t M, int64_t K, int64_t N,
                                  int32_t dtype);

#ifdef __cplusplus
}
#endif
#endif /* ESHKOL_GPU_MEMORY_H */
