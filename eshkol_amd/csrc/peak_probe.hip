/*
 * What the device sustains, measured in place, so that every throughput figure
 * can be quoted against both the published peak and the rate the silicon holds
 * under the same kind of data.
 *
 * The matrix-core probes run a register-only MFMA loop (no memory traffic, every
 * SIMD occupied by several waves, operand registers fixed at compile time). With
 * constant operands the int8 and bf16 loops reach the published rates; with
 * random operand bits the chip lowers its clock to hold its power limit and
 * sustains markedly less (about 3.0 of 5.0 POP/s for int8 and 1.7 of 2.5 PFLOP/s
 * for bf16 were measured). The figures are context for the GEMM numbers, not
 * bounds: a GEMM also spends power on LDS and cache traffic.
 *
 * The memory probe is a plain 16-byte-per-lane copy of a buffer much larger
 * than the caches: the read+write rate HBM sustains.
 *
 * Built into libeshkol_gpu_probe.so, which only the benchmark loads: it is not
 * part of libeshkol_gpu_hip.so and shares nothing with it.
 */
#include <hip/hip_runtime.h>
#include <stddef.h>
#include "eshkol/backend/gpu/gpu_hip_testing.h"

#define ESHKOL_HIP_OK(call) ((call) == hipSuccess)

typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef int v16i_t __attribute__((ext_vector_type(16)));
typedef float v16f_t __attribute__((ext_vector_type(16)));
typedef double d4_t __attribute__((ext_vector_type(4)));
typedef __bf16 v8b_t __attribute__((ext_vector_type(8)));

namespace {

__device__ __forceinline__ unsigned mix(unsigned x) {
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}

__global__ __launch_bounds__(256)
void probe_f64(int iters, int random, int* sink) {
    d4_t acc[8];
    double a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        acc[i] = (d4_t){0.0, 0.0, 0.0, 0.0};
        const unsigned h1 = mix(threadIdx.x * 64 + i + blockIdx.x * 7919), h2 = mix(h1 + 1);
        a[i] = random ? ((double)h1 / 4294967296.0 - 0.5) * 1.37 : 1.0;
        b[i] = random ? ((double)h2 / 4294967296.0 - 0.5) * 0.73 : 0.5;
    }
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 8; i++)
            acc[i] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[i], b[(i + 3) & 7], acc[i], 0, 0, 0);
    }
    double s = 0.0;
    for (int i = 0; i < 8; i++) for (int r = 0; r < 4; r++) s += acc[i][r];
    if (s == 12345.678) sink[0] = 1;
}

__global__ __launch_bounds__(256)
void probe_i8(int iters, int random, int* sink) {
    v16i_t acc[8];
    v4i_t a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const unsigned h1 = mix(threadIdx.x * 64 + i * 8 + c + blockIdx.x * 7919), h2 = mix(h1 + 12345);
            a[i][c] = random ? (int)h1 : 0x01010101;
            b[i][c] = random ? (int)h2 : 0x02020202;
        }
    }
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 8; i++)
            acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[(i + 3) & 7], acc[i], 0, 0, 0);
    }
    int s = 0;
    for (int i = 0; i < 8; i++) for (int r = 0; r < 16; r++) s += acc[i][r];
    if (s == 123456789) sink[0] = s;
}

__global__ __launch_bounds__(256)
void probe_bf16(int iters, int random, int* sink) {
    v16f_t acc[8];
    v4i_t a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0.0f;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const unsigned h1 = mix(threadIdx.x * 64 + i * 8 + c + blockIdx.x * 7919), h2 = mix(h1 + 12345);
            /* random sign and mantissa, exponent near 1.0 so nothing overflows */
            a[i][c] = random ? (int)((h1 & 0x807f807fu) | 0x3c003c00u) : 0x3f803f80;
            b[i][c] = random ? (int)((h2 & 0x807f807fu) | 0x3c003c00u) : 0x3f803f80;
        }
    }
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 8; i++)
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8b_t, a[i]),
                                                             __builtin_bit_cast(v8b_t, b[(i + 3) & 7]),
                                                             acc[i], 0, 0, 0);
    }
    float s = 0.0f;
    for (int i = 0; i < 8; i++) for (int r = 0; r < 16; r++) s += acc[i][r];
    if (s == 12345.678f) sink[0] = 1;
}

__global__ __launch_bounds__(256)
void probe_copy(const v4i_t* __restrict__ src, v4i_t* __restrict__ dst, size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

/* Which of a wave's vector ALU instructions run while another wave's MFMAs occupy
 * the same SIMD? 512 threads = eight waves per workgroup, one workgroup per CU, two
 * waves on every SIMD: waves 0-3 issue int8 MFMAs back to back (constant or random
 * operand bits), waves 4-7 forty instructions per iteration of one kind, eight
 * independent chains:
 *   KIND 0  v_fma_f32                 (stands for the plain vector ALU instructions)
 *   KIND 1  v_dot4_u32_u8             (the byte dot product of a residue epilogue)
 *   KIND 2  the epilogue's mix: add, byte dot product, convert, fma, 24-bit multiply-add
 *   KIND 3  the same mix with the byte dot product replaced by a 16-bit fold
 *           (shift, 24-bit multiply-add), which reduces modulo p as well
 * Either half can be switched off with a count of 0. */
template <int KIND>
__global__ __launch_bounds__(512, 1)
void probe_coissue(int mfma_iters, int valu_iters, int random, int* sink) {
    const int wave = threadIdx.x >> 6;
    if (wave < 4) {
        v16i_t acc[4];
        v4i_t a, b;
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][r] = 0;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const unsigned h1 = mix(threadIdx.x * 4 + r + blockIdx.x * 7919), h2 = mix(h1 + 12345);
            a[r] = random ? (int)h1 : 0x01010101 * (int)(threadIdx.x & 3);
            b[r] = random ? (int)h2 : 0x02020202;
        }
        for (int it = 0; it < mfma_iters; it++) {
#pragma unroll
            for (int i = 0; i < 4; i++) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[i], 0, 0, 0);
        }
        int s = 0;
        for (int i = 0; i < 4; i++) for (int r = 0; r < 16; r++) s += acc[i][r];
        if (s == 0x12345678) sink[0] = s;
    } else {
        unsigned x[8];
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] = mix(threadIdx.x * 8 + e);
        if (KIND == 0) {
            const unsigned c = 0x3f7fbe77u;     /* 0.999 */
            for (int it = 0; it < valu_iters; it++) {
#pragma unroll
                for (int r = 0; r < 5; r++)
#pragma unroll
                    for (int e = 0; e < 8; e++) asm volatile("v_fma_f32 %0, %0, %1, %1" : "+v"(x[e]) : "v"(c));
            }
        } else if (KIND == 1) {
            const unsigned wb = 0x01100401u;
            for (int it = 0; it < valu_iters; it++) {
#pragma unroll
                for (int r = 0; r < 5; r++)
#pragma unroll
                    for (int e = 0; e < 8; e++) asm volatile("v_dot4_u32_u8 %0, %0, %1, %0" : "+v"(x[e]) : "v"(wb));
            }
        } else {
            float q[8];
            const unsigned wb = 0x01100401u;
            const int p = 251;
            const float pinv = 1.0f / 251.0f;
            for (int it = 0; it < valu_iters; it++) {
#pragma unroll
                for (int e = 0; e < 8; e++) x[e] = x[e] + 0x80000000u + (unsigned)it;
                if (KIND == 2) {
#pragma unroll
                    for (int e = 0; e < 8; e++) x[e] = __builtin_amdgcn_udot4(x[e], wb, x[e] >> 24, false);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; e++) x[e] = (unsigned)(__mul24((int)(x[e] >> 16), 25 - 65536) + (int)x[e]);
                }
#pragma unroll
                for (int e = 0; e < 8; e++) q[e] = fmaf((float)(int)x[e], pinv, 12582912.0f);
#pragma unroll
                for (int e = 0; e < 8; e++) x[e] = (unsigned)(__mul24(__float_as_int(q[e]), -p) + (int)x[e]) ^ (x[e] << 13);
            }
        }
        unsigned s = 0;
        for (int e = 0; e < 8; e++) s += x[e];
        if (s == 0x12345678u) sink[1] = (int)s;
    }
}

}  // namespace

/* Times (ms) of the MFMA waves alone (20000 iterations of four MFMAs), the vector
 * ALU waves alone (valu_iters iterations) and both together, each wave's work the
 * same in all three. With the vector ALU waves the shorter ones, both = the MFMA
 * time means they ran entirely beside the MFMAs and both = the sum that they did
 * not run beside them at all; with the vector ALU waves the longer ones,
 * (mfma + valu - both) / mfma is the rate at which they advance beside the MFMAs,
 * relative to their rate alone. */
extern "C" int hip_probe_coissue(int kind, int random_operands, int valu_iters,
                                 double* mfma_ms, double* valu_ms, double* both_ms, void* stream) {
    if (!mfma_ms || !valu_ms || !both_ms || kind < 0 || kind > 3 || valu_iters <= 0) return -1;
    hipStream_t st = (hipStream_t)stream;
    int* sink = nullptr;
    hipEvent_t e0, e1;
    if (!ESHKOL_HIP_OK(hipMalloc((void**)&sink, 256))) return -1;
    if (!ESHKOL_HIP_OK(hipEventCreate(&e0)) || !ESHKOL_HIP_OK(hipEventCreate(&e1))) { (void)hipFree(sink); return -1; }
    const int M = 20000, V = valu_iters;
    const int counts[3][2] = {{M, 0}, {0, V}, {M, V}};
    double out[3] = {0.0, 0.0, 0.0};
    int rc = 0;
    for (int c = 0; c < 3 && rc == 0; c++) {
        float best = 1e30f;
        for (int rep = 0; rep < 3; rep++) {
            (void)hipEventRecord(e0, st);
            if (kind == 0) hipLaunchKernelGGL(probe_coissue<0>, dim3(256), dim3(512), 0, st, counts[c][0], counts[c][1], random_operands, sink);
            else if (kind == 1) hipLaunchKernelGGL(probe_coissue<1>, dim3(256), dim3(512), 0, st, counts[c][0], counts[c][1], random_operands, sink);
            else if (kind == 2) hipLaunchKernelGGL(probe_coissue<2>, dim3(256), dim3(512), 0, st, counts[c][0], counts[c][1], random_operands, sink);
            else hipLaunchKernelGGL(probe_coissue<3>, dim3(256), dim3(512), 0, st, counts[c][0], counts[c][1], random_operands, sink);
            (void)hipEventRecord(e1, st);
            float ms = 0.0f;
            if (!ESHKOL_HIP_OK(hipEventSynchronize(e1)) || !ESHKOL_HIP_OK(hipEventElapsedTime(&ms, e0, e1))) { rc = -1; break; }
            if (rep > 0 && ms < best) best = ms;
        }
        out[c] = best;
    }
    *mfma_ms = out[0]; *valu_ms = out[1]; *both_ms = out[2];
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    return rc;
}

/* kind 0: fp64 MFMA flop/s, 1: int8 MFMA op/s, 2: bf16 MFMA flop/s, 3: HBM copy
 * bytes/s (read + written). random_operands selects random operand bits for the
 * matrix-core kinds. Synchronises the stream. */
extern "C" int hip_probe_peak(int kind, int random_operands, double* rate, void* stream) {
    if (!rate || kind < 0 || kind > 3) return -1;
    hipStream_t st = (hipStream_t)stream;
    hipEvent_t e0, e1;
    if (!ESHKOL_HIP_OK(hipEventCreate(&e0)) || !ESHKOL_HIP_OK(hipEventCreate(&e1))) return -1;
    int rc = -1;
    float ms = 0.0f;
    if (kind == 3) {
        const size_t bytes = (size_t)1 << 30;
        char* buf = nullptr;
        if (ESHKOL_HIP_OK(hipMalloc((void**)&buf, 2 * bytes))) {
            for (int rep = 0; rep < 2; rep++) {
                if (rep == 1) (void)hipEventRecord(e0, st);
                hipLaunchKernelGGL(probe_copy, dim3(256 * 16), dim3(256), 0, st,
                                   (const v4i_t*)buf, (v4i_t*)(buf + bytes), bytes / 16);
            }
            (void)hipEventRecord(e1, st);
            if (ESHKOL_HIP_OK(hipEventSynchronize(e1)) && ESHKOL_HIP_OK(hipEventElapsedTime(&ms, e0, e1)) && ms > 0) {
                *rate = 2.0 * (double)bytes / (ms * 1e-3);
                rc = 0;
            }
            (void)hipFree(buf);
        }
    } else {
        int* sink = nullptr;
        if (!ESHKOL_HIP_OK(hipMalloc((void**)&sink, 256))) sink = nullptr;
        const int wgs = 1024;
        const int iters = (kind == 0) ? 20000 : 40000;
        const double per_mfma = (kind == 0) ? 2048.0 : (kind == 1) ? 65536.0 : 32768.0;
        if (sink) {
            for (int rep = 0; rep < 2; rep++) {
                if (rep == 1) (void)hipEventRecord(e0, st);
                if (kind == 0) hipLaunchKernelGGL(probe_f64, dim3(wgs), dim3(256), 0, st, iters, random_operands, sink);
                else if (kind == 1) hipLaunchKernelGGL(probe_i8, dim3(wgs), dim3(256), 0, st, iters, random_operands, sink);
                else hipLaunchKernelGGL(probe_bf16, dim3(wgs), dim3(256), 0, st, iters, random_operands, sink);
            }
            (void)hipEventRecord(e1, st);
            if (ESHKOL_HIP_OK(hipEventSynchronize(e1)) && ESHKOL_HIP_OK(hipEventElapsedTime(&ms, e0, e1)) && ms > 0) {
                *rate = (double)wgs * 4.0 * iters * 8.0 * per_mfma / (ms * 1e-3);
                rc = 0;
            }
            (void)hipFree(sink);
        }
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return rc;
}
