"""Pins for the Ozaki restatements that do not come from running the reference
(it has no CPU implementation of these tiers): closed forms, exact integer
brute force, the reference's own invariants and gate tolerances."""
from fractions import Fraction

import numpy as np
import pytest

import oracle
from eshkol_amd import synth

MOD = oracle.MODULI


def regimes(n):
    """The four fill regimes of tests/gpu/cuda_ozaki_correctness_test.esk:28-39."""
    i = np.arange(n * n, dtype=np.float64)
    A = [(i % 7) - 3, 1.0 + 0.5 * (i % 7), np.pi * (1.0 + (i % 11)),
         2.0 ** ((i % 20) - 10) * (1.0 + 0.1 * (i % 3))]
    B = [(i % 5) - 2, 0.5 + 0.25 * (i % 5), np.e * ((i % 9) - 4.0),
         2.0 ** ((i % 18) - 9) * (1.0 + 0.1 * (i % 4))]
    return [(a.reshape(n, n), b.reshape(n, n)) for a, b in zip(A, B)]


def exact_dot(A, B):
    """Exact products of doubles as Fractions (tiny sizes only)."""
    Af = [[Fraction(float(v)) for v in row] for row in A]
    Bf = [[Fraction(float(v)) for v in row] for row in B]
    return [[sum(Af[i][k] * Bf[k][j] for k in range(len(Bf))) for j in range(len(Bf[0]))]
            for i in range(len(Af))]


# ---- INT8 slice tier ------------------------------------------------------------

def test_slice_plan_invariants():
    p = oracle.ozaki_int8_plan(8192, 6)
    assert p["nbuf"] == 7 and len(p["pair_p"]) == 28                      # (T+1)(T+2)/2, cap = 16
    assert np.array_equal(p["weights"], 2.0 ** (-7.0 * (np.arange(7) + 2)))
    for b in range(7):
        sl = slice(p["first"][b], p["first"][b + 1])
        assert np.all(p["pair_p"][sl] + p["pair_q"][sl] == b)
    assert int(2147483647.0 / (8192 * 16129.0)) == 16
    assert oracle.ozaki_int8_plan(133001, 6) is None                       # K guard
    big = oracle.ozaki_int8_plan(100000, 6)                                # cap = 1: one pair per buffer
    assert big["nbuf"] == 28 and np.all(np.diff(big["first"]) == 1)
    for T in range(1, 9):
        assert len(oracle.ozaki_int8_plan(1024, T)["pair_p"]) == (T + 1) * (T + 2) // 2


def test_slices_recompose_and_ranges():
    A = synth.wide_range(3, (40, 70), -12, 12)
    B = synth.normal(4, (70, 30))
    A[5, :] = 0.0
    st = oracle.ozaki_int8_stages(A, B, 6)
    assert st["rmax"][5] == 1.0 and np.array_equal(st["rmax"][:5], np.abs(A[:5]).max(axis=1))
    assert np.array_equal(st["cmax"], np.abs(B).max(axis=0))
    sl = st["a_slices"].astype(np.float64)
    assert np.abs(sl).max() <= 127
    inside = np.abs(A / st["rmax"][:, None]) < 0.99        # away from the clamp at the row maximum
    assert np.abs(sl[1:][:, inside]).max() <= 64
    recomposed = sum(sl[p] * 128.0 ** -(p + 1) for p in range(7))
    assert np.abs(recomposed - A / st["rmax"][:, None]).max() <= 128.0 ** -7
    # the row maximum itself decomposes as 127, 127, ...
    i, k = 0, int(np.argmax(np.abs(A[0])))
    assert np.all(np.abs(sl[:, i, k]) == 127)
    # B slices are stored transposed
    slb = st["b_slices"].astype(np.float64)
    rb = sum(slb[q] * 128.0 ** -(q + 1) for q in range(7))
    assert np.abs(rb.T - B / st["cmax"][None, :]).max() <= 128.0 ** -7


def test_slice_products_bruteforce_int64():
    A, B = synth.normal(5, (33, 257)), synth.normal(6, (257, 29))
    st = oracle.ozaki_int8_stages(A, B, 4)
    p = st["plan"]
    for b in range(p["nbuf"]):
        G = np.zeros((33, 29), dtype=np.int64)
        for t in range(p["first"][b], p["first"][b + 1]):
            G += st["a_slices"][p["pair_p"][t]].astype(np.int64) @ st["b_slices"][p["pair_q"][t]].astype(np.int64).T
        assert np.array_equal(G, st["products"][b])
    # reconstruction, recomputed independently with numpy in the same order
    acc = np.zeros((33, 29))
    for b in range(p["nbuf"]):
        acc = acc + p["weights"][b] * st["products"][b].astype(np.float64)
    assert np.array_equal((acc * st["rmax"][:, None]) * st["cmax"][None, :], st["C"])


@pytest.mark.parametrize("T,tol", [(6, 1e-9), (4, 1e-6)])
def test_slice_tier_meets_reference_gate(T, tol):
    # tests/gpu/cuda_ozaki_correctness_gate.sh:106,112-118: normwise on the four regimes
    for A, B in regimes(96):
        ref = A.astype(np.longdouble) @ B.astype(np.longdouble)
        Cc = oracle.matmul_ozaki_int8(A, B, T)
        err = np.linalg.norm((Cc - ref).astype(np.float64)) / np.linalg.norm(ref.astype(np.float64))
        assert err < tol


def test_slice_tier_guaranteed_tolerances():
    # gpu_memory_cuda.cpp:485-487, well-conditioned inputs
    A, B = synth.normal(9, (64, 300)), synth.normal(10, (300, 48))
    ref = A.astype(np.longdouble) @ B.astype(np.longdouble)
    tol = [None, 1e-3, 1e-5, 1e-7, 1e-9, 1e-11, 1e-13, 1e-14, 1e-14]
    for T in range(1, 9):
        Cc = oracle.matmul_ozaki_int8(A, B, T)
        err = np.linalg.norm((Cc - ref).astype(np.float64)) / (np.linalg.norm(A) * np.linalg.norm(B))
        assert err < tol[T], (T, err)


# ---- CRT exact tier --------------------------------------------------------------

def test_crt_constants_identities():
    for n in (2, 7, 16):
        c = oracle.crt_constants(n)
        P = 1
        for m in MOD[:n]:
            P *= m
        assert c.num_moduli == n and c.P1 == float(P)
        assert abs(int(c.P1) + int(c.P2) - P) < (P >> 100) + 1
        assert c.Pinv == 1.0 / float(P)
        for l, m in enumerate(MOD[:n]):
            s = (P // m) * c.q[l]
            assert 0 < c.q[l] < m and s % m == 1
            for other in MOD[:n]:
                if other != m:
                    assert s % other == 0
            bits = 8 + int(np.ceil(np.log2(n)))
            mant = int(np.frexp(c.sl1[l])[0] * 2.0 ** 53)     # normalised 53-bit significand
            assert mant % (1 << bits) == 0                    # its low bits are zero
            assert abs(int(c.sl1[l]) + int(c.sl2[l]) - s) < (s >> 90) + 1
    assert abs(oracle.crt_constants(16).log2P - 125.4) < 0.05     # gpu_memory.mm:248, 1316
    assert oracle.crt_constants(40).num_moduli == 16 and oracle.crt_constants(1).num_moduli == 2


def test_crt_scaling_formulas():
    A = np.array([[1.0, -0.5, 0.25], [0.0, 0.0, 0.0], [3.0, 2.0, -7.9], [1e-3, 2.0 ** -20, 0.0]])
    B = np.array([[2.0, 0.0], [1.0, 0.0], [-4.0, 0.0]])
    st = oracle.ozaki_crt_stages(A, B)
    assert st["E"] == 52
    assert list(st["mu"]) == [52, 0, 50, 52 + 10]
    assert list(st["nu"]) == [50, 0]
    # E drops below 52 when few moduli are used
    st2 = oracle.ozaki_crt_stages(A, B, num_moduli=4)
    fa = np.log2(7.9) - 2
    assert st2["E"] == int(np.floor((np.log2(256 * 255 * 253 * 251) - 1 - np.log2(3) - fa) / 2))


def test_crt_residues_and_products_exact_integers():
    A = synth.wide_range(21, (9, 40), -30, 30)
    B = synth.wide_range(22, (40, 7), -30, 30)
    st = oracle.ozaki_crt_stages(A, B)
    Ai = [[int(np.trunc(np.ldexp(A[i, k], int(st["mu"][i])))) for k in range(40)] for i in range(9)]
    Bi = [[int(np.trunc(np.ldexp(B[k, j], int(st["nu"][j])))) for j in range(7)] for k in range(40)]
    D = [[sum(Ai[i][k] * Bi[k][j] for k in range(40)) for j in range(7)] for i in range(9)]
    P = 1
    for m in MOD:
        P *= m
    for l, m in enumerate(MOD):
        ap, bp, wp = st["a_planes"][l], st["b_planes"][l], st["w_planes"][l]
        assert ap.min() >= -(m // 2) and ap.max() <= (m - 1) // 2
        assert all((int(ap[i, k]) - Ai[i][k]) % m == 0 for i in range(9) for k in range(40))
        assert all((int(bp[j, k]) - Bi[k][j]) % m == 0 for j in range(7) for k in range(40))
        assert all((int(wp[i, j]) - D[i][j]) % m == 0 for i in range(9) for j in range(7))
        assert np.array_equal(st["acc32"][l], ap.astype(np.int64) @ bp.astype(np.int64).T)
    # the residues determine the exact integer (CRT with exact coefficients)
    for i in range(9):
        for j in range(7):
            S = sum(((P // m) * st["crt"].q[l]) * int(st["w_planes"][l][i, j]) for l, m in enumerate(MOD))
            c = S % P
            if c > P // 2:
                c -= P
            assert c == D[i][j]


def _fma(a, b, c):
    return float(Fraction(a) * Fraction(b) + Fraction(c))       # one rounding, to nearest even


def test_crt_reconstruction_arithmetic_independent_restatement():
    A, B = synth.normal(31, (6, 64)), synth.normal(32, (64, 5))
    st = oracle.ozaki_crt_stages(A, B)
    c = st["crt"]
    for i in range(6):
        for j in range(5):
            S1 = S2 = 0.0
            for l in range(16):
                w = float(st["w_planes"][l][i, j])
                S1 = _fma(c.sl1[l], w, S1)
                S2 = _fma(c.sl2[l], w, S2)
            s = S1 + S2
            x = s * c.Pinv
            Q = float(np.floor(abs(x) + 0.5) * np.sign(x))           # round half away from zero
            cp = _fma(-c.P1, Q, S1) + _fma(-c.P2, Q, S2)
            expect = (cp * 2.0 ** -int(st["mu"][i])) * 2.0 ** -int(st["nu"][j])
            assert expect == st["C"][i, j]


def test_crt_certification_witness_sample_points():
    # tests/gpu/ozaki_certification_test.esk:14-106
    n = 512
    r = np.arange(n, dtype=np.int64)[:, None]
    c = np.arange(n, dtype=np.int64)[None, :]
    a = (16777216 + ((97 * r + 53 * c) % 257)) * np.where((131 * r + 13 * c) % 2 == 0, 1, -1)
    b = (16777216 + ((71 * r + 29 * c + r * c) % 257)) * np.where((73 * r + 23 * c) % 2 == 0, 1, -1)
    exact = a @ b                                            # |dot| < 2^58: exact in int64
    assert np.abs(exact).max() < 2 ** 58
    Cc = oracle.matmul_ozaki_crt(a.astype(np.float64), b.astype(np.float64))
    pts = [0, 128, 256, 384, 511]
    for i in pts:
        for j in pts:
            assert Cc[i, j] == float(int(exact[i, j])), (i, j)
    plain = a.astype(np.float64) @ b.astype(np.float64)
    assert (plain != exact.astype(np.float64)).sum() >= 1     # ordinary f64 misses at least once
    # away from the sample points the reference's double-double accumulation is
    # not always exact; it stays within its own per-element gate
    rel = np.abs(Cc - exact.astype(np.float64)) / np.abs(exact.astype(np.float64))
    assert rel.max() < 1e-9


def test_crt_tier_meets_reference_gate_on_regimes():
    # tests/gpu/ozaki_correctness_test.esk:33: per-element relative error < 1e-9 on a 5x5 grid
    n = 128
    for A, B in regimes(n):
        Cc = oracle.matmul_ozaki_crt(A, B)
        ref = (A.astype(np.longdouble) @ B.astype(np.longdouble)).astype(np.float64)
        grid = [int(p * (n - 1) / 4) for p in range(5)]
        for i in grid:
            for j in grid:
                denom = abs(ref[i, j]) if abs(ref[i, j]) > 1e-9 else 1.0    # the reference test's denominator
                assert abs(Cc[i, j] - ref[i, j]) / denom < 1e-9


def _scaled_integer_products(A, B, mu, nu):
    """The exact integers the tier multiplies: sum_k trunc(a 2^mu) trunc(b 2^nu)."""
    import math
    M, K = A.shape
    N = B.shape[1]
    ai = [[int(math.trunc(math.ldexp(float(A[i, k]), int(mu[i])))) for k in range(K)] for i in range(M)]
    bi = [[int(math.trunc(math.ldexp(float(B[k, j]), int(nu[j])))) for k in range(K)] for j in range(N)]
    return [[sum(x * y for x, y in zip(ai[i], bi[j])) for j in range(N)] for i in range(M)]


def test_crt_weight_split_of_the_reference_loses_bits_and_the_aligned_one_does_not():
    """The reference splits every CRT weight relative to the weight's own exponent
    (gpu_memory.mm:322-337): the upper parts end at different bits, and their
    weighted sum is not always representable. Pinned here as a fact of the reference
    (the default mode reproduces it bit for bit), next to the split at a common bit
    position, whose sum is exact."""
    n = 16
    P = 1
    for m in MOD[:n]:
        P *= m
    ref_c, al_c = oracle.crt_constants(n), oracle.crt_constants(n, aligned=True)
    lsb = lambda x: (int(x) & -int(x)).bit_length() - 1
    ref_lsb = [lsb(ref_c.sl1[l]) for l in range(n)]
    assert min(ref_lsb) == 81 and max(ref_lsb) == 88          # sum of 16 * 128 * 2^126 needs bits >= 2^84 only
    e = P.bit_length() + 7 + 4 - 53
    assert e == 84
    for l, m in enumerate(MOD[:n]):
        s = (P // m) * al_c.q[l]
        assert al_c.q[l] == ref_c.q[l] and s % m == 1
        assert int(al_c.sl1[l]) % (1 << e) == 0 and abs(s - int(al_c.sl1[l])) <= 1 << (e - 1)
        assert abs(s - int(al_c.sl1[l]) - int(al_c.sl2[l])) <= 1 << (e - 1 - 52)
    assert (al_c.P1, al_c.P2, al_c.Pinv) == (ref_c.P1, ref_c.P2, ref_c.Pinv)

    A, B = synth.normal(1, (24, 256)), synth.normal(2, (256, 20))
    so, sa = oracle.ozaki_crt_stages(A, B), oracle.ozaki_crt_stages(A, B, aligned=True)
    assert np.array_equal(so["w_planes"], sa["w_planes"]) and np.array_equal(so["mu"], sa["mu"])
    X = _scaled_integer_products(A, B, so["mu"], so["nu"])
    bad_ref = 0
    for i in range(A.shape[0]):
        for j in range(B.shape[1]):
            sh = int(so["mu"][i] + so["nu"][j])
            exact = Fraction(X[i][j], 1 << sh)
            err_ref = abs(Fraction(float(so["C"][i, j])) - exact) * (1 << sh)       # in units of the scaled integer
            err_al = abs(Fraction(float(sa["C"][i, j])) - exact) * (1 << sh)
            if err_ref > 2 ** 70:
                bad_ref += 1
                assert 2 ** 80 < err_ref < 2 ** 86                                  # a rounding at 2^134 ... 2^137
            # aligned: roundings of the low parts (below 2^47) and of the result itself
            assert err_al <= 2 ** 47 + abs(X[i][j]) // 2 ** 52, (i, j, float(err_al))
    assert 1 <= bad_ref <= 24                                                        # about one element in 150
    # whole-tier entry: the same numbers, and what they mean against the true product
    ref = (A.astype(np.longdouble) @ B.astype(np.longdouble))
    scale = np.linalg.norm(A) * np.linalg.norm(B)
    Ca, Cr = oracle.matmul_ozaki_crt(A, B, aligned=True), oracle.matmul_ozaki_crt(A, B)
    assert np.array_equal(Ca, sa["C"]) and np.array_equal(Cr, so["C"])
    assert float(np.linalg.norm((Ca - ref).astype(np.float64))) / scale < 1e-16
    assert float(np.linalg.norm((Cr - ref).astype(np.float64))) / scale > 1e-12


def test_crt_small_exact_integer_products():
    # with 2-bit integers the true product is far below 2^53: it must come back exactly
    rng = np.random.default_rng(2)
    A = rng.integers(-3, 4, (20, 30)).astype(np.float64)
    B = rng.integers(-3, 4, (30, 10)).astype(np.float64)
    Cc = oracle.matmul_ozaki_crt(A, B)
    assert np.abs(Cc - A @ B).max() <= 1e-9 * np.abs(A @ B).max()


def test_crt_rejects_nonfinite_and_extreme_scale():
    A = np.ones((4, 4)); B = np.ones((4, 4))
    A2 = A.copy(); A2[1, 2] = np.nan
    assert oracle.matmul_ozaki_crt(A2, B) is None
    A3 = A.copy(); A3[0, 0] = np.inf
    assert oracle.matmul_ozaki_crt(A3, B) is None
    assert oracle.matmul_ozaki_crt(A * 1e-300, B) is None      # 2^mu would overflow


def test_crt_adaptive_moduli_count():
    A = 1.0 + synth.uniform(40, (8, 8), 0.0, 0.4)
    B = 1.0 + synth.uniform(41, (8, 8), 0.0, 0.4)
    st = oracle.ozaki_crt_stages(A, B, adaptive=True)
    n = st["num_moduli"]
    cum = np.cumsum(np.log2(MOD))
    fa = np.log2(A.max(axis=1)).max() % 1.0
    fb = np.log2(B.max(axis=0)).max() % 1.0
    emax = lambda k: np.floor((cum[k - 1] - 1 - 3 - fa - fb) / 2)
    assert emax(n) >= 52 and emax(n - 1) < 52 and st["E"] == 52


def test_mlp_layer():
    X = synth.normal(50, (12, 24))
    W = synth.xavier_uniform(51, 24, 16)
    b = synth.uniform(52, (16,), -0.1, 0.1)
    Y = oracle.mlp_layer(X, W, b)
    expect = np.tanh(oracle.matmul_ozaki_crt(X, W) + b[None, :])
    assert np.abs(Y - expect).max() <= 4 * np.finfo(np.float64).eps


def test_crt_exact_tier_guarantee_is_normwise_not_componentwise():
    """What the accuracy-budget selector may promise for the exact tier. Every element of A
    is truncated at 2^-52 of its row's largest magnitude, every element of B at 2^-52 of its
    column's, and the rest is exact: |C - AB|_ij <= K 2^-51 rmax_i cmax_j (plus the final
    rounding), which bounds the error in the norm the budget is stated in but not per
    element. Rows whose entries span 2^60 show it: the product of the small entries of row 0
    with the small entries of a column is lost entirely, where native fp64 keeps it."""
    K = 512
    A = synth.uniform(91, (4, K), 0.5, 1.0)
    B = synth.uniform(92, (K, 3), 0.5, 1.0)
    A[0, 1:] *= 2.0 ** -60                      # row 0: one entry of size 1, the rest 2^-60 of it
    B[1:, 0] *= 2.0 ** -60                      # column 0 likewise
    A[0, 0] = 0.0                               # ... and the two large entries never meet
    A[0, 5] = 0.75
    B[0, 0] = 0.625
    exact = [[sum(Fraction(float(A[i, k])) * Fraction(float(B[k, j])) for k in range(K)) for j in range(3)]
             for i in range(4)]
    rmax, cmax = np.abs(A).max(axis=1), np.abs(B).max(axis=0)
    for aligned in (True, False):
        C = oracle.matmul_ozaki_crt(A, B, aligned=aligned)
        for i in range(4):
            for j in range(3):
                err = abs(Fraction(float(C[i, j])) - exact[i][j])
                bound = Fraction(K) * Fraction(1, 2 ** 51) * Fraction(float(rmax[i])) * Fraction(float(cmax[j]))
                if aligned:
                    assert err <= bound + abs(exact[i][j]) * Fraction(1, 2 ** 52), (i, j, float(err), float(bound))
    Ca = oracle.matmul_ozaki_crt(A, B, aligned=True)
    # C[0,0] is a sum of products of order 2^-60: all of them are below the truncation, which
    # cuts at 2^-52 of the row's maximum 0.75 (and of the column's 0.625)
    assert exact[0][0] > 0 and float(exact[0][0]) < 2.0 ** -55
    assert abs(Fraction(float(Ca[0, 0])) - exact[0][0]) > exact[0][0] / 4          # componentwise: lost
    native = float(np.dot(A[0], B[:, 0]))
    assert abs(Fraction(native) - exact[0][0]) <= exact[0][0] * Fraction(K, 2 ** 52)   # native fp64 keeps it
    # ... while in the norm of the budget the tier is far inside 1e-15
    num = sum((Fraction(float(Ca[i, j])) - exact[i][j]) ** 2 for i in range(4) for j in range(3))
    den = sum(Fraction(float(x)) ** 2 for x in A.ravel()) * sum(Fraction(float(x)) ** 2 for x in B.ravel())
    assert float(num) ** 0.5 / float(den) ** 0.5 < 1e-15


@pytest.mark.parametrize("kind", ["normal", "wide"])
def test_crt_half_way_class_of_modulus_256_reference_representative(kind):
    """The one place where this oracle and the reference can return different bits for the
    exact tier: when a product's residue modulo 256 is the half-way class, the oracle (and the
    GPU) carry -128, the reference's floating-point residue formulas +128 or -128 by the parity
    of a rounded quotient (gpu_memory.mm:2573-2583; metal_softfloat.h:3907-4100 with its partial
    reductions every 1008 k). Modulo 256 that is the same number; the reference's weighted sum
    is inexact, so the choice can move its rounding error. Counted here on N(0,1) and on
    wide-range operands (BASELINE configuration 3's law), K = 2304 = three partial reductions:
    about one element in 256 is in the class, about half of those come out as +128, and of
    those a handful per 65536 elements change at all; the ones that do move by the
    reference's own error quantum (far more than 2 ulp, far inside its 1e-9 gate). With
    aligned weights the sum is exact and no element changes."""
    M, K, N = 256, 2304, 256
    if kind == "normal":
        A, B = synth.normal(41, (M, K)), synth.normal(42, (K, N))
    else:
        A, B = synth.wide_range(43, (M, K), -30, 30), synth.wide_range(44, (K, N), -30, 30)
    exact = A.astype(np.longdouble) @ B.astype(np.longdouble)
    scale = np.abs(A).max(axis=1)[:, None] * np.abs(B).max(axis=0)[None, :] * K
    for aligned in (False, True):
        base = oracle.matmul_ozaki_crt(A, B, aligned=aligned)
        for mode in (1, 2):
            got, n_half, n_plus = oracle.matmul_ozaki_crt_refrep(A, B, mode, aligned=aligned)
            changed = got != base
            print(kind, "aligned" if aligned else "reference weights", "mode", mode, "half-way class", n_half,
                  "as +128", n_plus, "elements that change", int(changed.sum()))
            assert M * N / 400 < n_half < M * N / 170            # one element in 256
            assert 0.35 * n_half < n_plus < 0.65 * n_half        # parity of a quotient: about half
            if aligned:
                assert not changed.any()
            else:
                assert changed.sum() <= 8                        # of 65536: at most about one in ten thousand
                # where it changes, both values are the reference's arithmetic with its inexact sum:
                # each within the reference's 1e-9 gate of the exact product, neither within 2 ulp of the other
                for v in (got, base):
                    assert float(np.max(np.abs(v[changed] - exact[changed]) / scale[changed], initial=0.0)) < 1e-9
