"""INT8 slice tier on the GPU, stage by stage against the oracle. Bars: int8
slices and int32 products bit-exact; C equal to the reference statement (same
fp64 operations in the same order), checked to 2 ulp."""
import numpy as np
import pytest

import oracle
from eshkol_amd import synth
from gpu_util import run_int8, ulp_distance
from test_oracle_ozaki import regimes

pytestmark = pytest.mark.gpu


def check_all_stages(A, B, T):
    rc, Cg, st = run_int8(A, B, T)
    assert rc == 0
    so = oracle.ozaki_int8_stages(A, B, T)
    assert st["s"] == T + 1 and st["nbuf"] == so["plan"]["nbuf"]
    assert np.array_equal(st["rmax"], so["rmax"]) and np.array_equal(st["cmax"], so["cmax"])
    assert np.array_equal(st["a_slices"], so["a_slices"])
    assert np.array_equal(st["b_slices"], so["b_slices"])
    assert st["pad_clear"]
    assert np.array_equal(st["products"], so["products"])
    assert ulp_distance(Cg, so["C"]).max() <= 2
    return Cg


@pytest.mark.parametrize("M,K,N,T", [(1, 1, 1, 6), (5, 3, 4, 6), (64, 128, 64, 6), (100, 200, 90, 4),
                                     (257, 129, 255, 6), (300, 260, 280, 7), (512, 512, 512, 6),
                                     (33, 2049, 65, 2), (640, 1024, 384, 8), (96, 96, 96, 1),
                                     (3, 133000, 2, 6), (3001, 2, 2, 6), (2, 2, 3001, 4), (1, 1031, 513, 6)])
def test_all_stages(gpu, M, K, N, T):
    print("int8", M, K, N, T, flush=True)
    A, B = synth.normal(500 + M, (M, K)), synth.normal(600 + N, (K, N))
    check_all_stages(A, B, T)


def test_random_shapes_with_a_few_rows_all_stages(gpu):
    """Twenty random products with up to 170 rows and a random slice count: whichever contraction kernel the shape
    picks (its plans sum several products per output plane), every stage is the oracle's."""
    rng = np.random.default_rng(32)
    done = 0
    while done < 20:
        M = int(rng.integers(1, 171)); K = int(2 ** rng.uniform(6, 11.5)); N = int(2 ** rng.uniform(4, 12.3))
        if M * K * N > 1.0e8:
            continue
        done += 1
        T = int(rng.integers(1, 9))
        print("int8, random", M, K, N, T, flush=True)
        check_all_stages(synth.normal(5000 + done, (M, K)), synth.normal(6000 + done, (K, N)), T)


def test_wide_range_and_zero_rows(gpu):
    A = synth.wide_range(1, (80, 120), -12, 12); B = synth.wide_range(2, (120, 60), -12, 12)
    A[4, :] = 0.0; B[:, 11] = 0.0
    Cg = check_all_stages(A, B, 6)
    assert np.all(Cg[4] == 0.0) and np.all(Cg[:, 11] == 0.0)


@pytest.mark.parametrize("T,tol", [(6, 1e-9), (4, 1e-6)])
def test_reference_gate_regimes(gpu, T, tol):
    # tests/gpu/cuda_ozaki_correctness_gate.sh:106,112-118: normwise on a 5x5 probe grid
    n = 1024
    for A, B in regimes(n):
        rc, Cg, _ = run_int8(A, B, T, want_stages=False)
        assert rc == 0
        grid = [int(p * (n - 1) / 4) for p in range(5)]
        ref = (A[grid].astype(np.longdouble) @ B[:, grid].astype(np.longdouble)).astype(np.float64)
        assert np.linalg.norm(Cg[grid][:, grid] - ref) / np.linalg.norm(ref) < tol


def test_k_guard_and_bad_arguments(gpu):
    assert run_int8(np.ones((2, 133001)), np.ones((133001, 2)), 6)[0] == -1
    assert run_int8(np.ones((4, 4)), np.ones((4, 4)), 0)[0] == -1
    assert run_int8(np.ones((4, 4)), np.ones((4, 4)), 9)[0] == -1
    A = np.ones((8, 8)); A[1, 1] = np.nan
    assert run_int8(A, np.ones((8, 8)), 6)[0] == -1


def test_full_size_sampled(gpu):
    """8192^3 at T=6: sampled rows and columns against the oracle run on the same
    rows and columns (every stage of this tier is local to a row or a column)."""
    n = 8192
    print("int8 full", n, flush=True)
    A, B = synth.normal(41, (n, n)), synth.normal(42, (n, n))
    rc, Cg, st = run_int8(A, B, 6)
    assert rc == 0
    rows = [0, 1, 255, 256, 4097, n - 257, n - 1]
    cols = [0, 3, 255, 256, 5000, n - 256, n - 1]
    so = oracle.ozaki_int8_stages(A[rows], B[:, cols], 6)
    assert np.array_equal(st["rmax"][rows], so["rmax"]) and np.array_equal(st["cmax"][cols], so["cmax"])
    assert np.array_equal(st["a_slices"][:, rows, :], so["a_slices"])
    assert np.array_equal(st["b_slices"][:, cols, :], so["b_slices"])
    assert np.array_equal(st["products"][:, rows][:, :, cols], so["products"])
    assert ulp_distance(Cg[rows][:, cols], so["C"]).max() <= 2
    assert st["pad_clear"]


@pytest.mark.parametrize("M,K,N,T", [(3001, 1030, 3005, 6), (4095, 515, 4097, 4)])
def test_large_sizes_that_are_multiples_of_nothing_sampled(gpu, M, K, N, T):
    """Sizes that end inside a tile in every dimension, with an N that puts C's rows off 16-byte
    boundaries (the int32 product buffers then have a pitch of their own): sampled rows and columns,
    the edges among them, against the oracle run on those rows and columns."""
    print("int8 ragged", M, K, N, T, flush=True)
    A, B = synth.normal(43 + M, (M, K)), synth.normal(44 + N, (K, N))
    rc, Cg, st = run_int8(A, B, T)
    assert rc == 0
    rows = [0, 1, 255, 256, M // 2 + 1, M - 257, M - 2, M - 1]
    cols = [0, 3, 255, 256, N // 2, N - 256, N - 2, N - 1]
    so = oracle.ozaki_int8_stages(A[rows], B[:, cols], T)
    assert np.array_equal(st["rmax"][rows], so["rmax"]) and np.array_equal(st["cmax"][cols], so["cmax"])
    assert np.array_equal(st["a_slices"][:, rows, :], so["a_slices"])
    assert np.array_equal(st["b_slices"][:, cols, :], so["b_slices"])
    assert np.array_equal(st["products"][:, rows][:, :, cols], so["products"])
    assert ulp_distance(Cg[rows][:, cols], so["C"]).max() <= 2
    assert st["pad_clear"]
    # every element: the same slices multiplied in float64 (exact: the sums stay far below 2^53)
    plan = so["plan"]
    for b in range(st["nbuf"]):
        lo, hi = plan["first"][b], plan["first"][b + 1]
        acc = sum(st["a_slices"][plan["pair_p"][t]].astype(np.float64) @ st["b_slices"][plan["pair_q"][t]].astype(np.float64).T
                  for t in range(lo, hi))
        assert np.array_equal(acc.astype(np.int64), st["products"][b].astype(np.int64)), b
