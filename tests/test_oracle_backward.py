"""The matmul-backward oracle against the reference's own outputs: golden
gradients written from the compiled reference (tests/golden/make_golden.py),
the reference library itself when it has been built here, and what the
mathematics fixes (integer cases that are exact in any order, the transpose
identities, a finite-difference check of d<G, A@B>)."""
import ctypes as C
import os

import numpy as np
import pytest

import oracle
from eshkol_amd import synth
from conftest import GOLDEN

CASES = 6


def test_golden_gradients_bitexact():
    g = np.load(os.path.join(GOLDEN, "fp64_backward.npz"))
    for ci in range(CASES):
        M, K, N = (int(v) for v in g["case%d_shape" % ci])
        G, A, B = synth.normal(300 + ci, (M, N)), synth.normal(400 + ci, (M, K)), synth.normal(500 + ci, (K, N))
        for tag, fused in (("avx", True), ("sse2", False)):
            gA, gB = oracle.matmul_backward_f64(G, A, B, fused=fused)
            assert np.array_equal(gA, g["case%d_%s_gradA" % (ci, tag)]), (M, K, N, tag)
            assert np.array_equal(gB, g["case%d_%s_gradB" % (ci, tag)]), (M, K, N, tag)


@pytest.mark.skipif(not os.path.exists(oracle.REF_PATH), reason="reference library not built here")
def test_against_compiled_reference_random_shapes():
    dp = C.POINTER(C.c_double)
    ref = C.CDLL(oracle.REF_PATH)
    ref.eshkol_matmul_backward_f64.argtypes = [dp] * 5 + [C.c_uint64] * 3
    rng = np.random.default_rng(11)
    for _ in range(20):
        M, K, N = (int(v) for v in rng.integers(1, 90, 3))
        G, A, B = rng.standard_normal((M, N)), rng.standard_normal((M, K)), rng.standard_normal((K, N))
        gA, gB = np.empty((M, K)), np.empty((K, N))
        ref.eshkol_matmul_backward_f64(*(x.ctypes.data_as(dp) for x in (G, A, B, gA, gB)), M, K, N)
        oA, oB = oracle.matmul_backward_f64(G, A, B)
        assert np.array_equal(oA, gA) and np.array_equal(oB, gB), (M, K, N)


def test_integer_cases_are_exact_and_not_transposed():
    # small integers: every summation order gives the same bits, so a wrong
    # index or a swapped operand cannot hide behind rounding
    rng = np.random.default_rng(3)
    for (M, K, N) in [(1, 1, 1), (2, 3, 4), (5, 2, 7), (16, 9, 3), (31, 33, 29)]:
        G = rng.integers(-9, 10, (M, N)).astype(np.float64)
        A = rng.integers(-9, 10, (M, K)).astype(np.float64)
        B = rng.integers(-9, 10, (K, N)).astype(np.float64)
        gA, gB = oracle.matmul_backward_f64(G, A, B)
        assert np.array_equal(gA, G @ B.T)
        assert np.array_equal(gB, A.T @ G)


def test_gradients_are_the_derivative_of_the_forward_product():
    # d/dt <G, (A + t dA) @ (B + t dB)> at 0 equals <grad_A, dA> + <grad_B, dB>
    rng = np.random.default_rng(4)
    M, K, N = 13, 17, 11
    G, A, B = rng.standard_normal((M, N)), rng.standard_normal((M, K)), rng.standard_normal((K, N))
    dA, dB = rng.standard_normal((M, K)), rng.standard_normal((K, N))
    gA, gB = oracle.matmul_backward_f64(G, A, B)
    f = lambda t: float(np.sum(G * oracle.matmul_f64(A + t * dA, B + t * dB)))
    h = 1e-6
    fd = (f(h) - f(-h)) / (2 * h)
    an = float(np.sum(gA * dA) + np.sum(gB * dB))
    assert abs(fd - an) <= 1e-7 * max(1.0, abs(an))


def test_agrees_with_forward_oracle_on_transposed_copies():
    # the reference's GPU branch computes the same gradients as two forward
    # products on explicit transposes (blas_backend.cpp:969-993)
    G, A, B = synth.normal(1, (40, 24)), synth.normal(2, (40, 56)), synth.normal(3, (56, 24))
    gA, gB = oracle.matmul_backward_f64(G, A, B)
    fA = oracle.matmul_f64(G, np.ascontiguousarray(B.T))
    fB = oracle.matmul_f64(np.ascontiguousarray(A.T), G)
    scale = np.sqrt(np.sum(G * G))
    assert np.abs(gA - fA).max() <= 1e-14 * scale * np.sqrt(np.sum(B * B))
    assert np.abs(gB - fB).max() <= 1e-14 * scale * np.sqrt(np.sum(A * A))
