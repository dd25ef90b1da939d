"""The reduced-precision ("fast") CRT tier on the GPU, stage by stage against the
oracle's restatement of the reference. Bars: moduli, E, exponents, int8 residue
planes bit-exact; product residues equal modulo p; C within the resolution of an
fp64 fractional CRT (num_moduli 2^-50 P at the element's scale) of the exactly
scaled integer product, and within the resolution of the reference's float-pair
reconstruction (2^-40 P) of the oracle's restatement of it."""
import math

import numpy as np
import pytest

import oracle
from eshkol_amd import synth
from gpu_util import run_fast
from test_oracle_ozaki import regimes

pytestmark = pytest.mark.gpu


def check_all_stages(A, B, n_mod=11, trans=None):
    rc, Cg, st = run_fast(A, B, n_mod, trans=trans)
    assert rc == 0
    so = oracle.ozaki_fast_stages(A, B, n_mod)
    assert st["num_moduli"] == so["num_moduli"] and st["moduli"] == so["moduli"]
    assert st["E"] == so["E"] and st["cap"] == so["consts"].cap
    E = so["E"]
    nz_a, nz_b = np.abs(A).max(axis=1) > 0, np.abs(B).max(axis=0) > 0
    assert np.array_equal(st["shift_a"][nz_a], E - so["ei"][nz_a]) and not st["shift_a"][~nz_a].any()
    assert np.array_equal(st["shift_b"][nz_b], E - so["fj"][nz_b]) and not st["shift_b"][~nz_b].any()
    assert np.array_equal(st["a_planes"], so["a_planes"])           # bit-exact residues
    assert np.array_equal(st["b_planes"], so["b_planes"])
    assert st["a_pad_clear"] and st["b_pad_clear"]
    for l, p in enumerate(so["moduli"]):                             # exact products modulo p
        assert np.array_equal(np.mod(st["w_planes"][l].astype(np.int64), p), np.mod(so["G"][l].astype(np.int64), p)), l
        assert np.abs(st["w_planes"][l].astype(np.int64)).max() <= p // 2 + (p % 2 == 0)
    P = float(math.prod(so["moduli"]))
    scale = np.ldexp(1.0, (so["ei"][:, None] + so["fj"][None, :] - 2 * E).astype(np.int64))
    exact = so["C_exact"]
    assert np.all(np.abs(Cg - exact) <= so["num_moduli"] * 2.0 ** -50 * P * scale)
    # and the reference's own float-pair result (where its float scaling does not leave the
    # range) sits within its 2^-40 P of the same value: the two agree to that resolution
    ok = np.isfinite(so["C"]) & (scale > 2.0 ** -100) & (scale < 2.0 ** 60)
    assert np.all(np.abs(Cg - so["C"])[ok] <= 2.0 ** -39 * P * scale[ok])
    return Cg, so


SHAPES = [(1, 1, 1), (5, 3, 4), (64, 128, 64), (100, 200, 90), (257, 129, 255), (33, 2049, 65), (512, 640, 384),
          (3, 131071, 2), (3001, 2, 2), (2, 2, 3001), (1, 1031, 513),
          # fewer tiles than CUs and k from 1024 on: interleaved planes on the 256 x 128 kernel (not yet at 11 tiles)
          (200, 1024, 300), (300, 2048, 257), (256, 1024, 256)]


@pytest.mark.parametrize("M,K,N", SHAPES)
def test_wide_range_inputs_all_stages(gpu, M, K, N):
    A = synth.wide_range(500 + M, (M, K))
    B = synth.wide_range(600 + N, (K, N))
    check_all_stages(A, B)


def test_random_shapes_with_a_few_rows_all_stages(gpu):
    """Twenty random products with up to 170 rows: whichever contraction kernel the shape picks, every stage is the
    oracle's."""
    rng = np.random.default_rng(31)
    done = 0
    while done < 20:
        M = int(rng.integers(1, 171)); K = int(2 ** rng.uniform(6, 11.5)); N = int(2 ** rng.uniform(4, 12.3))
        if M * K * N > 1.0e8:
            continue
        done += 1
        print("fast, random", M, K, N, flush=True)
        check_all_stages(synth.wide_range(3000 + done, (M, K)), synth.wide_range(4000 + done, (K, N)),
                         n_mod=int(rng.integers(2, 17)))


@pytest.mark.parametrize("n", [2, 5, 8, 11, 16])
def test_moduli_counts(gpu, n):
    A, B = synth.normal(13, (96, 160)), synth.normal(14, (160, 80))
    check_all_stages(A, B, n_mod=n)
    rc, _, st = run_fast(A, B, 40)                     # clamped like the reference (gpu_memory.mm:2838)
    assert rc == 0 and st["num_moduli"] == 16


def test_zero_rows_subnormals_signs_and_ties(gpu):
    A = synth.normal(21, (70, 90)); B = synth.normal(22, (90, 50))
    A[3, :] = 0.0; A[10, :] = -0.0; B[:, 7] = 0.0; A[20, 5] = 5e-324; B[4, 4] = -2.0 ** -1030
    A[30, :] = 2.0 ** -600; B[:, 9] = 2.0 ** 500
    A[40, :] = np.ldexp(np.arange(90) + 0.5, -30)      # exact halves after scaling: round half up, both signs
    A[41, :] = -A[40, :]
    Cg, so = check_all_stages(A, B)
    assert np.all(Cg[3] == 0.0) and np.all(Cg[:, 7] == 0.0)


def test_even_modulus_keeps_the_positive_half(gpu):
    """At K = 8192 the cap is 90 and 64 is among the moduli: residues of 32 (mod 64) are stored
    as +32 for either sign of the element (metal_softfloat.h:4172-4177)."""
    M, K, N = 24, 8192, 20
    A, B = synth.normal(23, (M, K)), synth.normal(24, (K, N))
    A[:, 0] = 4.0                                       # every row maximum 4 = 0.5 * 2^3: e = 3
    A[0, 1:200] = np.ldexp(32.0 + 64.0 * np.arange(199), 3 - 26)        # 32 (mod 64) after scaling by 2^(E-e)
    A[1, 1:200] = -A[0, 1:200]
    Cg, so = check_all_stages(A, B)
    assert so["consts"].cap == 90 and so["E"] == 26 and 64 in so["moduli"]
    l = so["moduli"].index(64)
    assert np.all(so["a_planes"][l][0, 1:200] == 32) and np.all(so["a_planes"][l][1, 1:200] == 32)
    assert not (so["a_planes"][l] == -32).any()


def test_operands_held_transposed(gpu):
    A, B = synth.wide_range(31, (130, 300), -6, 6), synth.wide_range(32, (300, 70), -6, 6)
    base, _ = check_all_stages(A, B)
    for trans in ((1, 0), (0, 1)):
        Cg, _ = check_all_stages(A, B, trans=trans)
        assert np.array_equal(Cg, base)


def test_accuracy_over_the_reference_gate_regimes(gpu):
    """The reference calls 11 moduli its ~1e-8 tier, 'worst ~2.4e-8 over 4 gate regimes'."""
    worst = 0.0
    for A, B in regimes(256):
        rc, Cg, _ = run_fast(A, B, 11, want_stages=False)
        assert rc == 0
        ref = (A.astype(np.longdouble) @ B.astype(np.longdouble)).astype(np.float64)
        worst = max(worst, float(np.abs(Cg - ref).max() / np.abs(ref).max()))
    assert worst <= 5e-8, worst


def test_rejects_what_the_tier_cannot_represent(gpu):
    A, B = synth.normal(41, (64, 64)), synth.normal(42, (64, 64))
    An = A.copy(); An[5, 5] = np.nan
    assert run_fast(An, B)[0] == -1
    Bi = B.copy(); Bi[1, 2] = np.inf
    assert run_fast(A, Bi)[0] == -1


@pytest.mark.parametrize("n_mod", [3, 5, 8, 11, 14, 16])
def test_error_stays_inside_the_tolerance_the_budget_selector_assumes(gpu, n_mod):
    """The accuracy-budget selector credits this tier with a relative error of
    2^(5 - E) for E bits kept per operand (32 times what well-conditioned operands
    show). Checked here on N(0,1) operands, on operands of equal magnitude and
    random sign (every rounding as large as it can be) and on rows of very
    different scale (each row is scaled by its own maximum)."""
    import ctypes as C
    import eshkol_amd as ea
    M, K, N = 256, 2048, 192
    E = C.c_int32()
    got_n = ea.load().hip_ozaki_fast_plan(K, n_mod, C.byref(E), None, None)
    assert got_n == n_mod
    tol = 2.0 ** (5 - E.value)
    rng = np.random.default_rng(n_mod)
    cases = [(synth.normal(3, (M, K)), synth.normal(4, (K, N))),
             (np.where(rng.random((M, K)) < 0.5, -0.7, 0.7) * (1 + 1e-3 * rng.random((M, K))),
              np.where(rng.random((K, N)) < 0.5, -1.3, 1.3) * (1 + 1e-3 * rng.random((K, N)))),
             (synth.normal(5, (M, K)) * 2.0 ** rng.integers(-20, 20, (M, 1)),
              synth.normal(6, (K, N)) * 2.0 ** rng.integers(-20, 20, (1, N)))]
    for A, B in cases:
        rc, Cg, _ = run_fast(A, B, n_mod, want_stages=False)
        assert rc == 0
        ref = A.astype(np.longdouble) @ B.astype(np.longdouble)
        # row by row and column by column, so that small rows are not hidden behind large ones
        err = np.abs((Cg - ref).astype(np.float64))
        scale = np.linalg.norm(A, axis=1)[:, None] * np.linalg.norm(B, axis=0)[None, :]
        assert (err / scale).max() <= tol, (n_mod, E.value, float((err / scale).max()), tol)


@pytest.mark.parametrize("M,K,N", [(3001, 1030, 3005), (4095, 515, 4097)])
def test_large_sizes_that_are_multiples_of_nothing_sampled(gpu, M, K, N):
    """Sizes that end inside a tile in every dimension, with an N that puts C's rows off 16-byte
    boundaries (the product planes then have a pitch of their own): every residue product recomputed
    from the device's own planes with exact integers, and sampled rows and columns against the oracle."""
    print("fast ragged", M, K, N, flush=True)
    A = synth.wide_range(45 + M, (M, K)); B = synth.wide_range(46 + N, (K, N))
    rc, Cg, st = run_fast(A, B, 11)
    assert rc == 0
    for l, p in enumerate(st["moduli"]):
        acc = st["a_planes"][l].astype(np.float64) @ st["b_planes"][l].astype(np.float64).T
        w = st["w_planes"][l].astype(np.int64)
        assert np.all((acc.astype(np.int64) - w) % p == 0) and np.abs(w).max() <= p // 2 + (p % 2 == 0), l
    rows = [0, 1, 255, 256, M // 2 + 1, M - 257, M - 2, M - 1]
    cols = [0, 3, 255, 256, N // 2, N - 256, N - 2, N - 1]
    rc, Cs, _ = run_fast(A[rows], B[:, cols], 11)
    assert rc == 0
    # every stage is local to a row of A or a column of B once E is fixed by K and the moduli count
    assert np.array_equal(Cg[rows][:, cols], Cs)
    check_all_stages(np.ascontiguousarray(A[rows]), np.ascontiguousarray(B[:, cols]))
