"""Reduced-precision tier: the rounding primitives against the reference's own
outputs (golden), against library casts known to round to nearest even, and the
reference's dtype known answers (tests/v1_3_edge_cases/tensor_dtype_test.esk)."""
import os

import numpy as np

import oracle
from eshkol_amd import synth
from conftest import GOLDEN


def same(a, b):
    return np.all((a == b) | (np.isnan(a) & np.isnan(b))) and np.array_equal(np.signbit(a), np.signbit(b))


def test_reduce_precision_golden():
    g = np.load(os.path.join(GOLDEN, "reduce_precision.npz"))
    for d in (1, 2, 3, 4):
        assert same(oracle.reduce_precision(g["values"], d), g["dtype%d" % d]), d


def test_reduce_precision_vs_library_casts():
    x = np.concatenate([synth.normal(1, (20000,)), synth.normal(2, (5000,)) * 1e-5,
                        synth.normal(3, (5000,)) * 3e4, synth.normal(4, (2000,)) * 1e-7])
    f32 = x.astype(np.float32)
    assert same(oracle.reduce_precision(x, 1), f32.astype(np.float64))
    # f16: IEEE round-to-nearest-even on the normal range. Below 2^-14 the reference's
    # subnormal branch (runtime_tensor_dtype.cpp:66-77) shifts one bit too far and
    # returns half the IEEE value; the oracle keeps that (golden-pinned) behaviour.
    normal = np.abs(x) >= 2.0 ** -14
    with np.errstate(over="ignore"):
        ieee = f32.astype(np.float16).astype(np.float64)
    assert same(oracle.reduce_precision(x, 2)[normal], ieee[normal])
    sub = (~normal) & (np.abs(x) > 2.0 ** -23)
    assert sub.sum() > 100
    quirk = oracle.reduce_precision(x, 2)[sub]
    assert np.all(np.abs(quirk) <= np.abs(ieee[sub])) and np.any(quirk != ieee[sub])
    import torch
    bf = torch.from_numpy(f32).to(torch.bfloat16).to(torch.float64).numpy()
    assert same(oracle.reduce_precision(x, 3), bf)


def test_dtype_known_answers():
    assert abs(oracle.reduce_precision(np.array([1.0009765625]), 2)[0] - 1.0009765625) < 1e-3
    assert oracle.reduce_precision(np.array([3.7]), 4)[0] == 4.0
    assert oracle.reduce_precision(np.array([2.5, 3.5, -2.5, 200.0, -200.0, np.nan]), 4).tolist() == \
        [2.0, 4.0, -2.0, 127.0, -128.0, 0.0]
    assert oracle.reduce_precision(np.array([65520.0]), 2)[0] == np.inf


def test_reduced_matmul_statements_agree_within_tier_tolerance():
    M = K = N = 96
    A = synth.normal(5, (M, K), 1.0 / np.sqrt(K))
    B = synth.normal(6, (K, N), 1.0 / np.sqrt(K))
    for d in (2, 3):
        ref = oracle.matmul_reduced(A, B, d)                  # f64 GEMM over rounded inputs
        Ar, Br = oracle.reduce_precision(A, d), oracle.reduce_precision(B, d)
        assert np.array_equal(ref, oracle.matmul_f64(Ar, Br))
        f32acc = oracle.matmul_reduced_f32acc(A, B, d, False)
        rounded = oracle.matmul_reduced_f32acc(A, B, d, True)
        den = np.linalg.norm(Ar) * np.linalg.norm(Br)
        assert np.linalg.norm(f32acc - ref) / den < 1e-6
        assert np.linalg.norm(rounded - ref) / den < 1e-2
        assert same(rounded, oracle.reduce_precision(f32acc, d))
