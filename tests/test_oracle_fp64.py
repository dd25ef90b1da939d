"""The fp64 oracle against the reference's own outputs: golden vectors written
from the compiled reference (tests/golden/make_golden.py), the reference
library itself when it has been built in this container, and the known-answer
catalogue of the reference's matmul tests."""
import ctypes as C
import os

import numpy as np
import pytest

import oracle
from eshkol_amd import synth
from conftest import GOLDEN

CASES = 8


def test_golden_small_cases_bitexact():
    g = np.load(os.path.join(GOLDEN, "fp64_matmul.npz"))
    for ci in range(CASES):
        M, K, N = (int(v) for v in g["case%d_shape" % ci])
        sa, sb = (int(v) for v in g["case%d_seeds" % ci])
        A, B = synth.uniform(sa, (M, K)), synth.uniform(sb, (K, N))
        assert np.array_equal(oracle.matmul_f64(A, B, fused=True), g["case%d_avx" % ci]), (M, K, N)
        assert np.array_equal(oracle.matmul_f64(A, B, fused=False), g["case%d_sse2" % ci]), (M, K, N)


def test_golden_config1_256cubed():
    g = np.load(os.path.join(GOLDEN, "fp64_matmul.npz"))
    A, B = synth.uniform(42, (256, 256)), synth.uniform(43, (256, 256))
    for tag, fused in (("avx", True), ("sse2", False)):
        Cc = oracle.matmul_f64(A, B, fused=fused)
        idx = g["c1_sample_idx"]
        assert np.array_equal(np.array([Cc[i, j] for i, j in idx]), g["c1_%s_samples" % tag])
        assert np.array_equal(Cc[17], g["c1_%s_row17" % tag])
        assert float(np.sum(Cc.astype(np.longdouble))) == float(g["c1_%s_sum" % tag][0])


def test_golden_batch():
    g = np.load(os.path.join(GOLDEN, "fp64_batch.npz"))
    a, b = synth.normal(7, (3, 17, 23)), synth.normal(8, (3, 23, 11))
    assert np.array_equal(oracle.batch_matmul_f64(a, b), g["avx"])
    oracle.lib().oracle_matmul_set_fused(0)
    try:
        assert np.array_equal(oracle.batch_matmul_f64(a, b), g["sse2"])
    finally:
        oracle.lib().oracle_matmul_set_fused(1)


@pytest.mark.skipif(not os.path.exists(oracle.REF_PATH), reason="reference library not built here")
def test_against_compiled_reference_random_shapes():
    dp = C.POINTER(C.c_double)
    ref = C.CDLL(oracle.REF_PATH)
    ref.eshkol_matmul_f64.argtypes = [dp, dp, dp, C.c_uint64, C.c_uint64, C.c_uint64]
    rng = np.random.default_rng(5)
    for _ in range(25):
        M, K, N = (int(v) for v in rng.integers(1, 150, 3))
        A, B = rng.standard_normal((M, K)), rng.standard_normal((K, N))
        out = np.empty((M, N))
        ref.eshkol_matmul_f64(A.ctypes.data_as(dp), B.ctypes.data_as(dp), out.ctypes.data_as(dp), M, K, N)
        assert np.array_equal(oracle.matmul_f64(A, B), out), (M, K, N)


# ---- the reference's known-answer tests -----------------------------------------

def test_known_answers_small():
    mm = oracle.matmul_f64
    # tests/gpu/matmul_correctness_test.esk:4-63
    a = np.array([[1., 2.], [3., 4.]]); b = np.array([[5., 6.], [7., 8.]])
    assert np.array_equal(mm(a, b), [[19, 22], [43, 50]])
    assert np.array_equal(mm(np.eye(2), a), a)
    a23 = np.array([[1., 2., 3.], [4., 5., 6.]]); b32 = np.array([[7., 8.], [9., 10.], [11., 12.]])
    assert np.array_equal(mm(a23, b32), [[58, 64], [139, 154]])
    assert np.array_equal(mm(a, b).T, mm(b.T, a.T))
    assert np.array_equal(mm(mm(a, b), a), [[85, 126], [193, 286]])
    # tests/ml/matmul_test.esk:5-19
    assert np.array_equal(mm(np.arange(6.).reshape(2, 3), np.arange(6.).reshape(3, 2)), [[10, 13], [28, 40]])
    # tests/xla/matmul_accuracy.esk:21-55
    assert mm(np.ones((1, 100)), np.arange(100.).reshape(100, 1))[0, 0] == 4950.0
    assert abs(mm(np.full((2, 2), 1e-6), np.diag([1e6, 1e6]))[0, 0] - 1.0) < 1e-4


@pytest.mark.parametrize("n", [4, 8, 10, 16, 32, 46, 47, 49, 50, 51, 53, 64, 100, 192])
def test_known_answers_ones(n):
    # tests/gpu/gpu_diagnostic_test.esk:25-49, tests/backend/blas_provider_test.cpp:85-95
    assert np.all(oracle.matmul_f64(np.ones((n, n)), np.ones((n, n))) == float(n))


def test_known_answers_row_index_and_identity():
    # tests/gpu/sf64_nonuniform_test.esk:40-72
    n = 50
    A = np.repeat(np.arange(1., n + 1)[:, None], n, axis=1)
    assert np.array_equal(oracle.matmul_f64(A, np.ones((n, n)))[:, 0], 50.0 * np.arange(1, n + 1))
    # tests/gpu/gpu_large_matmul_test.esk:12-63, cuda_host_sync_regression_test.esk:14-39
    for n in (8, 50):
        S = np.arange(float(n * n)).reshape(n, n)
        assert np.array_equal(oracle.matmul_f64(S, np.eye(n)), S)


def test_normwise_error_vs_long_double():
    A, B = synth.uniform(42, (256, 256)), synth.uniform(43, (256, 256))
    ref = A.astype(np.longdouble) @ B.astype(np.longdouble)
    err = np.linalg.norm((oracle.matmul_f64(A, B) - ref).astype(np.float64)) / (np.linalg.norm(A) * np.linalg.norm(B))
    assert err < 1e-15
