"""Write golden vectors for the native fp64 tier from the reference's own CPU
matmul, compiled from its sources in place by oracle/Makefile into
oracle/_ref/libeshkol_ref.so (AVX2+FMA build) and libeshkol_ref_sse2.so
(flag-less build). Run in the build container (needs /root/reference):

    make -C oracle ref && python tests/golden/make_golden.py

Outputs (committed): tests/golden/fp64_matmul.npz, fp64_batch.npz,
fp64_backward.npz, reduce_precision.npz. Inputs come from eshkol_amd.synth (seeded), small cases
are stored whole, the 256^3 case as a checksum plus sampled entries.
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
from eshkol_amd import synth  # noqa: E402

dp = C.POINTER(C.c_double)
u64, i64 = C.c_uint64, C.c_int64


def ref(path):
    lib = C.CDLL(path)
    lib.eshkol_matmul_f64.argtypes = [dp, dp, dp, u64, u64, u64]
    lib.eshkol_batch_matmul_f64.argtypes = [dp, dp, dp, i64, i64, i64, i64]
    lib.eshkol_matmul_backward_f64.argtypes = [dp, dp, dp, dp, dp, u64, u64, u64]
    lib.eshkol_tensor_reduce_precision_value.argtypes = [C.c_double, i64]
    lib.eshkol_tensor_reduce_precision_value.restype = C.c_double
    return lib


def P(a):
    return a.ctypes.data_as(dp)


CASES = [(2, 2, 2), (4, 4, 4), (3, 5, 4), (5, 7, 3), (1, 100, 1), (64, 64, 64), (65, 67, 66), (37, 130, 9)]
BACKWARD_CASES = [(2, 2, 2), (4, 4, 4), (3, 5, 4), (17, 23, 11), (64, 48, 80), (1, 33, 1)]
SAMPLES_256 = [(0, 0), (0, 255), (255, 0), (255, 255), (128, 128), (17, 201), (64, 63), (63, 64), (100, 3)]


def main():
    avx = ref(os.path.join(ROOT, "oracle", "_ref", "libeshkol_ref.so"))
    sse = ref(os.path.join(ROOT, "oracle", "_ref", "libeshkol_ref_sse2.so"))
    out = {}
    for ci, (M, K, N) in enumerate(CASES):
        A = synth.uniform(1000 + ci, (M, K))
        B = synth.uniform(2000 + ci, (K, N))
        for tag, lib in (("avx", avx), ("sse2", sse)):
            Cc = np.empty((M, N))
            lib.eshkol_matmul_f64(P(A), P(B), P(Cc), M, K, N)
            out["case%d_%s" % (ci, tag)] = Cc
        out["case%d_shape" % ci] = np.array([M, K, N])
        out["case%d_seeds" % ci] = np.array([1000 + ci, 2000 + ci])
    # configuration 1: 256^3 uniform[-1,1]
    A = synth.uniform(42, (256, 256))
    B = synth.uniform(43, (256, 256))
    for tag, lib in (("avx", avx), ("sse2", sse)):
        Cc = np.empty((256, 256))
        lib.eshkol_matmul_f64(P(A), P(B), P(Cc), 256, 256, 256)
        out["c1_%s_sum" % tag] = np.array([np.sum(Cc.astype(np.longdouble)).astype(np.float64)])
        out["c1_%s_samples" % tag] = np.array([Cc[i, j] for i, j in SAMPLES_256])
        out["c1_%s_row17" % tag] = Cc[17].copy()
    out["c1_sample_idx"] = np.array(SAMPLES_256)
    np.savez(os.path.join(HERE, "fp64_matmul.npz"), **out)

    a = synth.normal(7, (3, 17, 23))
    b = synth.normal(8, (3, 23, 11))
    bo = {}
    for tag, lib in (("avx", avx), ("sse2", sse)):
        c = np.empty((3, 17, 11))
        lib.eshkol_batch_matmul_f64(P(a), P(b), P(c), 3, 17, 23, 11)
        bo[tag] = c
    np.savez(os.path.join(HERE, "fp64_batch.npz"), **bo)

    # matmul backward (eshkol_matmul_backward_f64): grad_A, grad_B for seeded G, A, B
    wo = {}
    for ci, (M, K, N) in enumerate(BACKWARD_CASES):
        G = synth.normal(300 + ci, (M, N))
        A = synth.normal(400 + ci, (M, K))
        B = synth.normal(500 + ci, (K, N))
        for tag, lib in (("avx", avx), ("sse2", sse)):
            gA, gB = np.empty((M, K)), np.empty((K, N))
            lib.eshkol_matmul_backward_f64(P(G), P(A), P(B), P(gA), P(gB), M, K, N)
            wo["case%d_%s_gradA" % (ci, tag)] = gA
            wo["case%d_%s_gradB" % (ci, tag)] = gB
        wo["case%d_shape" % ci] = np.array([M, K, N])
    np.savez(os.path.join(HERE, "fp64_backward.npz"), **wo)

    vals = np.concatenate([
        synth.normal(11, (3000,)), synth.normal(12, (2000,)) * 1e-6, synth.normal(13, (1000,)) * 1e5,
        synth.normal(14, (500,)) * 6e-8,
        np.array([0.0, -0.0, 1.0009765625, 3.7, -3.5, 2.5, 65504.0, 65519.99, 65520.0, 1e-8, 5.96e-8,
                  2.98e-8, 6.1e-5, np.inf, -np.inf, 1e39, 3.3e38, 3.4e38, 127.5, -128.5, 300.0])])
    ro = {"values": vals}
    for d in (1, 2, 3, 4):
        ro["dtype%d" % d] = np.array([avx.eshkol_tensor_reduce_precision_value(float(v), d) for v in vals])
    np.savez(os.path.join(HERE, "reduce_precision.npz"), **ro)
    print("wrote golden fixtures")


if __name__ == "__main__":
    main()
