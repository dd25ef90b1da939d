/*
 * TEST INFRASTRUCTURE ONLY - see eshkol_oracle.h.
 *
 * Plays the CPU side of the Eshkol runtime for tests of the GPU library's
 * fallback ladder: the GPU translation unit imports eshkol_matmul_f64
 * (lib/backend/blas_backend.cpp:791) and eshkol_batch_matmul_f64
 * (lib/core/runtime_tensor_math.cpp:796) from the runtime it is linked into;
 * here the oracle's restatements answer under those names and count the calls
 * so a test can tell which side ran.
 */
#include "eshkol_oracle.h"

static volatile long g_matmul_calls = 0;
static volatile long g_batch_calls = 0;

void eshkol_matmul_f64(const double* A, const double* B, double* C,
                       uint64_t M, uint64_t K, uint64_t N) {
    g_matmul_calls++;
    oracle_matmul_f64(A, B, C, M, K, N);
}

void eshkol_batch_matmul_f64(const double* a, const double* b, double* c,
                             int64_t batch, int64_t M, int64_t K, int64_t N) {
    g_batch_calls++;
    oracle_batch_matmul_f64(a, b, c, batch, M, K, N);
}

long oracle_hostrt_matmul_calls(void) { return g_matmul_calls; }
long oracle_hostrt_batch_calls(void)  { return g_batch_calls; }
void oracle_hostrt_reset(void) { g_matmul_calls = 0; g_batch_calls = 0; }
