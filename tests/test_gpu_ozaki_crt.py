"""Ozaki-II CRT exact tier on the GPU, stage by stage against the oracle.
Bars (BASELINE.json): int8 residue planes and residue products bit-exact;
C within 2 ulp per element of the reference statement of the tier."""
import numpy as np
import pytest

import oracle
from eshkol_amd import synth
from gpu_util import run_crt, ulp_distance
from test_oracle_ozaki import regimes

pytestmark = pytest.mark.gpu
MAX_ULP = 2


def check_all_stages(A, B, num_moduli=16, adaptive=False):
    rc, Cg, st = run_crt(A, B, num_moduli, adaptive)
    assert rc == 0
    so = oracle.ozaki_crt_stages(A, B, num_moduli, adaptive)
    assert st["num_moduli"] == so["num_moduli"] and st["E"] == so["E"]
    assert np.array_equal(st["mu"], so["mu"]) and np.array_equal(st["nu"], so["nu"])
    assert np.array_equal(st["a_planes"], so["a_planes"])          # bit-exact residues
    assert np.array_equal(st["b_planes"], so["b_planes"])
    assert st["a_pad_clear"] and st["b_pad_clear"]
    assert np.array_equal(st["w_planes"], so["w_planes"])          # bit-exact residue products
    assert ulp_distance(Cg, so["C"]).max() <= MAX_ULP
    return Cg, so


SHAPES = [(1, 1, 1), (5, 3, 4), (64, 128, 64), (100, 200, 90), (257, 129, 255), (300, 1000, 17),
          (512, 512, 512), (33, 2049, 65), (768, 640, 1024),
          (3, 131071, 2),                      # the largest K the tier accepts
          (3001, 2, 2), (2, 2, 3001), (1, 1031, 513),
          (8, 4096, 1024), (32, 1024, 2048), (64, 1000, 777), (65, 1000, 777),      # a few rows against a layer
          # fewer tiles than CUs and k from 1024 on: interleaved planes on the 256 x 128 kernel
          (200, 1024, 300), (161, 1100, 1000), (300, 2048, 257), (256, 4100, 256)]


@pytest.mark.parametrize("M,K,N", SHAPES)
def test_wide_range_inputs_all_stages(gpu, M, K, N):
    print("crt", M, K, N, flush=True)
    A = synth.wide_range(300 + M, (M, K))          # configuration 3's input law
    B = synth.wide_range(400 + N, (K, N))
    check_all_stages(A, B)


def test_zero_rows_columns_and_negative_zero(gpu):
    A = synth.normal(1, (70, 90)); B = synth.normal(2, (90, 50))
    A[3, :] = 0.0; A[10, :] = -0.0; B[:, 7] = 0.0; A[20, 5] = 0.0; B[4, 4] = -0.0
    A[30, :] = 2.0 ** -600; B[:, 9] = 2.0 ** 500       # extreme but representable scales
    Cg, so = check_all_stages(A, B)
    assert np.all(Cg[3] == 0.0) and np.all(Cg[:, 7] == 0.0)


@pytest.mark.parametrize("n", [2, 3, 7, 12, 15, 16])
def test_moduli_counts(gpu, n):
    A, B = synth.normal(3, (96, 160)), synth.normal(4, (160, 80))
    check_all_stages(A, B, num_moduli=n)


def test_adaptive_moduli_selection(gpu):
    A = 1.0 + synth.uniform(40, (64, 8), 0.0, 0.4)
    B = 1.0 + synth.uniform(41, (8, 64), 0.0, 0.4)
    _, so = check_all_stages(A, B, adaptive=True)
    assert so["num_moduli"] < 16


def test_reference_gate_regimes(gpu):
    # tests/gpu/ozaki_correctness_test.esk:33-90: four regimes, per-element rel < 1e-9 on a 5x5 grid
    for n in (512, 1024):
        for A, B in regimes(n):
            rc, Cg, _ = run_crt(A, B, want_stages=False)
            assert rc == 0
            grid = [int(p * (n - 1) / 4) for p in range(5)]
            ref = A[grid].astype(np.longdouble) @ B[:, grid].astype(np.longdouble)
            got = Cg[grid][:, grid]
            denom = np.where(np.abs(ref) > 1e-9, np.abs(ref), 1.0)     # the reference test's denominator
            assert np.all(np.abs(got - ref) / denom < 1e-9)


def test_certification_witness(gpu):
    # tests/gpu/ozaki_certification_test.esk:14-106
    n = 512
    r = np.arange(n, dtype=np.int64)[:, None]
    c = np.arange(n, dtype=np.int64)[None, :]
    a = (16777216 + ((97 * r + 53 * c) % 257)) * np.where((131 * r + 13 * c) % 2 == 0, 1, -1)
    b = (16777216 + ((71 * r + 29 * c + r * c) % 257)) * np.where((73 * r + 23 * c) % 2 == 0, 1, -1)
    exact = a @ b
    Cg, _ = check_all_stages(a.astype(np.float64), b.astype(np.float64))
    pts = [0, 128, 256, 384, 511]
    for i in pts:
        for j in pts:
            assert Cg[i, j] == float(int(exact[i, j]))


def test_rejects_what_the_tier_cannot_represent(gpu):
    A = np.ones((8, 8)); B = np.ones((8, 8))
    for bad in (np.nan, np.inf, -np.inf):
        A2 = A.copy(); A2[2, 3] = bad
        assert run_crt(A2, B)[0] == -1
        B2 = B.copy(); B2[5, 1] = bad
        assert run_crt(A, B2)[0] == -1
    assert run_crt(A * 1e-300, B)[0] == -1                      # 2^mu outside the double range
    A3 = A.copy(); A3[4, :] = 5e-324                            # subnormal row: same
    assert run_crt(A3, B)[0] == -1
    assert run_crt(np.ones((2, 131072)), np.ones((131072, 2)))[0] == -1   # int32-exact bound on K


def test_fused_bias_tanh_epilogue(gpu):
    X = synth.normal(50, (96, 200)); W = synth.xavier_uniform(51, 200, 72)
    b = synth.uniform(52, (72,), -0.1, 0.1)
    rc, Y, _ = run_crt(X, W, bias=b, act=1, want_stages=False)
    assert rc == 0
    expect = oracle.mlp_layer(X, W, b)
    assert np.abs(Y - expect).max() <= 4 * np.finfo(np.float64).eps    # device tanh vs glibc tanh
    rc, Y0, _ = run_crt(X, W, bias=b, act=0, want_stages=False)
    assert np.array_equal(Y0, oracle.matmul_ozaki_crt(X, W) + b[None, :])


def test_full_size_config3_sampled(gpu):
    """Configuration 3 at 8192^3: sampled residue products recomputed from the
    device's own planes with exact integers, and a sampled block of C against the
    oracle run on the same rows and columns (mu, nu depend only on the row or
    column; E is clamped to 52 at this K for both)."""
    n = 8192
    print("crt full", n, flush=True)
    A = synth.wide_range(31, (n, n)); B = synth.wide_range(32, (n, n))
    rc, Cg, st = run_crt(A, B)
    assert rc == 0 and st["E"] == 52 and st["num_moduli"] == 16
    rows = [0, 1, 255, 256, 4097, n - 257, n - 1]
    cols = [0, 3, 255, 256, 5000, n - 256, n - 1]
    so = oracle.ozaki_crt_stages(A[rows], B[:, cols])
    assert so["E"] == 52
    assert np.array_equal(st["mu"][rows], so["mu"]) and np.array_equal(st["nu"][cols], so["nu"])
    assert np.array_equal(st["a_planes"][:, rows, :], so["a_planes"])
    assert np.array_equal(st["b_planes"][:, cols, :], so["b_planes"])
    for l, p in enumerate(oracle.MODULI):
        acc = st["a_planes"][l][rows].astype(np.int64) @ st["b_planes"][l][cols].astype(np.int64).T
        w = st["w_planes"][l][rows][:, cols].astype(np.int64)
        assert np.all((acc - w) % p == 0) and w.min() >= -(p // 2) and w.max() <= (p - 1) // 2
    assert np.array_equal(st["w_planes"][:, rows][:, :, cols], so["w_planes"])
    assert ulp_distance(Cg[rows][:, cols], so["C"]).max() <= MAX_ULP
    assert st["a_pad_clear"] and st["b_pad_clear"]


@pytest.mark.parametrize("M,K,N", [(3001, 1030, 3005), (4095, 515, 4097), (2303, 2049, 2561)])
def test_large_sizes_that_are_multiples_of_nothing_sampled(gpu, M, K, N):
    """Products large enough for the kernels that load straight into LDS and MFMA registers, with
    sizes that end inside a tile in every dimension and an N that puts C's rows off 16-byte
    boundaries: the product planes then have a pitch of their own. Sampled rows and columns, the
    edges among them, against the oracle run on those rows and columns; every residue product
    recomputed from the device's own planes with exact integers."""
    print("crt ragged", M, K, N, flush=True)
    A = synth.wide_range(41 + M, (M, K)); B = synth.wide_range(42 + N, (K, N))
    rc, Cg, st = run_crt(A, B)
    assert rc == 0 and st["num_moduli"] == 16
    rows = [0, 1, 255, 256, M // 2 + 1, M - 257, M - 2, M - 1]
    cols = [0, 3, 255, 256, N // 2, N - 256, N - 2, N - 1]
    so = oracle.ozaki_crt_stages(A[rows], B[:, cols])
    assert so["E"] == st["E"]
    assert np.array_equal(st["mu"][rows], so["mu"]) and np.array_equal(st["nu"][cols], so["nu"])
    assert np.array_equal(st["a_planes"][:, rows, :], so["a_planes"])
    assert np.array_equal(st["b_planes"][:, cols, :], so["b_planes"])
    assert st["a_pad_clear"] and st["b_pad_clear"]
    assert np.array_equal(st["w_planes"][:, rows][:, :, cols], so["w_planes"])
    assert ulp_distance(Cg[rows][:, cols], so["C"]).max() <= MAX_ULP
    for l, p in enumerate(oracle.MODULI):            # every element of every plane, exactly
        acc = st["a_planes"][l].astype(np.float64) @ st["b_planes"][l].astype(np.float64).T
        w = st["w_planes"][l].astype(np.int64)
        assert np.all((acc.astype(np.int64) - w) % p == 0) and w.min() >= -(p // 2) and w.max() <= (p - 1) // 2
    # The whole result against the oracle's own product is too slow here. With the aligned weights
    # (the reference's own lose low bits in the weighted sum) the tier is exact on small integers,
    # which checks every element of C, edges included.
    import eshkol_amd as ea
    rng = np.random.default_rng(M)
    Ai = rng.integers(-50, 51, (M, K)).astype(np.float64); Bi = rng.integers(-50, 51, (K, N)).astype(np.float64)
    was = ea.load().hip_ozaki_crt_set_aligned_weights(1)
    try:
        rc, Ci, _ = run_crt(Ai, Bi, want_stages=False)
    finally:
        ea.load().hip_ozaki_crt_set_aligned_weights(was)
    assert rc == 0 and np.array_equal(Ci, Ai @ Bi)


def both_bookkeeping_paths(A, B, **kw):
    """The device scan with a handful of host log2 calls, and the host pass over every
    maximum, must give the same E, shifts, planes and result; returns the first."""
    import eshkol_amd as ea
    lib = ea.load()
    fast = check_all_stages(A, B, **kw)
    lib.hip_ozaki_crt_set_host_pass(1)
    try:
        rc, Ch, sh = run_crt(A, B, kw.get("num_moduli", 16), kw.get("adaptive", False))
    finally:
        lib.hip_ozaki_crt_set_host_pass(0)
    assert rc == 0
    so = fast[1]
    assert sh["E"] == so["E"] and np.array_equal(sh["mu"], so["mu"]) and np.array_equal(sh["nu"], so["nu"])
    assert np.array_equal(Ch, fast[0])
    return fast


def test_shift_bookkeeping_structured_maxima(gpu):
    """Maxima that are powers of two, equal in every row, subnormal, or spread over a
    hundred binades with one mantissa (more distinct candidates than the scan keeps)."""
    rng = np.random.default_rng(11)
    A = rng.standard_normal((130, 70)); B = rng.standard_normal((70, 90))
    both_bookkeeping_paths(np.ones((40, 30)), np.full((30, 50), 0.5))
    both_bookkeeping_paths(np.eye(64), np.eye(64) * 3.0)
    As = A.copy(); As[5, :] = 0.0; As[6, :] *= 2.0 ** -900           # a zero row and a tiny one
    both_bookkeeping_paths(As, B)
    As[6, :] *= 2.0 ** -140                                           # a subnormal maximum: no shift reaches it
    import eshkol_amd as ea
    for host_pass in (0, 1):
        ea.load().hip_ozaki_crt_set_host_pass(host_pass)
        try:
            assert run_crt(As, B)[0] == -1
        finally:
            ea.load().hip_ozaki_crt_set_host_pass(0)
    Aw = A / np.abs(A).max(axis=1, keepdims=True) * 1.75             # every row maximum 1.75 ...
    Aw *= 2.0 ** np.arange(-65, 65)[:, None]                         # ... in 130 different binades
    both_bookkeeping_paths(Aw, B)
    Bw = B / np.abs(B).max(axis=0, keepdims=True) * (1.0 + 2.0 ** -30)
    Bw *= 2.0 ** rng.integers(-3, 4, 90)[None, :]                    # seven binades: few candidates
    both_bookkeeping_paths(A, Bw)


def test_shift_bookkeeping_mantissas_next_to_a_power_of_two(gpu):
    """Within 2^-40 of a power of two libm may round log2 across the integer: the scan
    must notice and leave such operands to the host pass. Results equal the oracle's."""
    rng = np.random.default_rng(12)
    A = rng.standard_normal((50, 40)); B = rng.standard_normal((40, 60))
    for val in (np.nextafter(2.0, 0.0), np.nextafter(1.0, 2.0), 4.0 - 2.0 ** -45, 8.0 * (1.0 + 2.0 ** -50)):
        Ax = A / np.abs(A).max() * 0.9; Ax[7, 3] = val
        Bx = B / np.abs(B).max() * 0.9; Bx[5, 9] = -val
        both_bookkeeping_paths(Ax, B)
        both_bookkeeping_paths(A, Bx)


@pytest.mark.parametrize("M,K,N", [(1, 1024, 512), (8, 4096, 300), (64, 1031, 1000), (160, 1500, 300), (161, 1500, 300), (200, 2048, 256),
                                   (256, 1024, 64)])
def test_few_rows_in_front_of_prepared_planes(gpu, M, K, N):
    """A few long rows against a prepared second operand: row maxima, shifts and the scan of the maxima are one
    launch there (the workgroup that finishes last scans). Results are the plain entry point's bit for bit and the
    oracle's within the tier's bar, also with zero rows, tiny and huge rows, a maximum next to a power of two (the
    scan hands such operands to the host pass), and a NaN or an infinity is refused; with the three kernels kept
    apart the same again."""
    import ctypes as C
    import eshkol_amd as ea
    lib = ea.load()
    st = lib.eshkol_hip_get_stream()
    B = synth.normal(50 + N, (K, N))
    dB = ea.DeviceArray.from_host(B)
    h = C.c_void_p()
    assert lib.hip_ozaki_crt_prepare_operand_b(dB.ptr, K, N, 0, 16, M, C.byref(h), st) == 0

    def run(A, prepared):
        dA, dC = ea.DeviceArray.from_host(A), ea.DeviceArray((M, N))
        if prepared:
            rc = lib.hip_matmul_ozaki_crt_prepared_f64(dA.ptr, h, dC.ptr, M, K, N, 0, 16, 0, None, 0, st)
        else:
            rc = lib.hip_matmul_ozaki_crt_f64(dA.ptr, dB.ptr, dC.ptr, M, K, N, 16, 0, None, 0, st)
        ea.synchronize()
        return rc, dC.download()

    base = synth.normal(60 + M, (M, K))
    cases = [base]
    A = base.copy(); A[0, :] = 0.0; cases.append(A)
    A = base.copy(); A[M - 1, :] *= 2.0 ** -600; A[M // 2, :] *= 2.0 ** 500; cases.append(A)
    A = base / np.abs(base).max() * 0.9; A[0, K - 1] = 4.0 - 2.0 ** -45; cases.append(A)     # an extreme mantissa
    A = base / np.abs(base).max(axis=1, keepdims=True) * 1.75; cases.append(A)              # every maximum the same
    try:
        for fused in (1, 0):
            lib.hip_ozaki_crt_set_fused_scan(fused)
            for i in range(2):                      # twice: the counter the last workgroup leaves must be zero again
                for A in cases:
                    rc, got = run(A, True)
                    assert rc == 0
                    rc, want = run(A, False)
                    assert rc == 0 and np.array_equal(got, want)
                    assert ulp_distance(got, oracle.matmul_ozaki_crt(A, B)).max() <= MAX_ULP
            for bad in (np.nan, np.inf, -np.inf):
                A = base.copy(); A[M - 1, 7] = bad
                assert run(A, True)[0] == -1
            rc, got = run(base, True)               # and the call after a refusal is whole again
            assert rc == 0 and np.array_equal(got, run(base, False)[1])
    finally:
        lib.hip_ozaki_crt_set_fused_scan(1)
        lib.hip_ozaki_crt_release_prepared(h)


def test_random_shapes_with_a_few_rows_match_the_oracle(gpu):
    """Thirty random products with up to 170 rows: whichever contraction kernel the row count and the width pick
    (the two for a few rows, or tiles), residue products and results are the oracle's."""
    rng = np.random.default_rng(2024)
    done = 0
    while done < 30:
        M = int(rng.integers(1, 171)); K = int(2 ** rng.uniform(6, 11.5)); N = int(2 ** rng.uniform(4, 12.3))
        if M * K * N > 1.5e8:
            continue
        done += 1
        print("crt, random", M, K, N, flush=True)
        A = synth.wide_range(1000 + done, (M, K))
        B = synth.wide_range(2000 + done, (K, N))
        check_all_stages(A, B)


def test_aligned_weight_split_matches_the_oracle_and_is_accurate(gpu):
    """hip_ozaki_crt_set_aligned_weights(1): the CRT weights split at a common bit.
    Residues and products are those of the default mode, the result equals the
    oracle's aligned restatement within the tier's 2 ulp, and on operands where the
    reference's split loses bits (N(0,1): about one element in 150) the error
    against the true product drops from 1e-11 to 1e-17 normwise."""
    import eshkol_amd as ea
    lib = ea.load()
    A, B = synth.normal(1, (300, 1024)), synth.normal(2, (1024, 260))
    ref = A.astype(np.longdouble) @ B.astype(np.longdouble)
    scale = np.linalg.norm(A) * np.linalg.norm(B)
    rc, C_ref_split, st0 = run_crt(A, B)
    assert rc == 0
    was = lib.hip_ozaki_crt_set_aligned_weights(1)
    try:
        assert was == 0
        rc, C_aligned, st1 = run_crt(A, B)
    finally:
        assert lib.hip_ozaki_crt_set_aligned_weights(0) == 1
    assert rc == 0
    assert np.array_equal(st0["w_planes"], st1["w_planes"]) and np.array_equal(st0["mu"], st1["mu"])
    assert ulp_distance(C_ref_split, oracle.matmul_ozaki_crt(A, B)).max() <= MAX_ULP
    assert ulp_distance(C_aligned, oracle.matmul_ozaki_crt(A, B, aligned=True)).max() <= MAX_ULP
    err = lambda X: float(np.linalg.norm((X - ref).astype(np.float64))) / scale
    assert err(C_aligned) < 1e-16 and err(C_ref_split) > 1e-12
