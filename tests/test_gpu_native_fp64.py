"""Native fp64 tier on the GPU (hip_dgemm_f64, through the C ABI) against the
oracle's restatement of the reference CPU matmul. Bar (BASELINE.json):
||C - C_ref||_F / (||A||_F ||B||_F) <= 1e-14."""
import os

import numpy as np
import pytest

import oracle
from eshkol_amd import synth
from conftest import GOLDEN
from gpu_util import normwise, run_dgemm

pytestmark = pytest.mark.gpu
TOL = 1e-14


@pytest.fixture
def tiled(gpu):
    """For the tests of the tiled kernels' own variants (tile sizes, cuts along k): shapes with a
    thin side or a small output would otherwise take the kernels of dgemm_thin_f64.hip."""
    import eshkol_amd as ea
    lib = ea.load()
    lib.hip_dgemm_set_thin_rows(0)
    yield
    lib.hip_dgemm_set_thin_rows(1)

SHAPES = [(1, 1, 1), (2, 2, 2), (1, 100, 1), (3, 5, 4), (5, 7, 3), (16, 16, 16), (64, 64, 64),
          (65, 67, 66), (37, 130, 9), (128, 128, 128), (129, 257, 131), (256, 256, 256),
          (300, 17, 500), (512, 1000, 64), (1000, 33, 1000), (1024, 1024, 1024),
          (1, 100003, 1), (70001, 3, 5), (5, 3, 70001), (2, 2, 65537), (65537, 2, 2), (9, 70000, 131)]


@pytest.mark.parametrize("M,K,N", SHAPES)
def test_dgemm_matches_reference_cpu_statement(gpu, M, K, N):
    print("dgemm", M, K, N, flush=True)
    A, B = synth.uniform(100 + M, (M, K)), synth.uniform(200 + N, (K, N))
    Cg = run_dgemm(A, B)
    assert normwise(Cg, oracle.matmul_f64(A, B), A, B) <= TOL


def test_dgemm_against_golden_vectors(gpu):
    g = np.load(os.path.join(GOLDEN, "fp64_matmul.npz"))
    for ci in range(8):
        M, K, N = (int(v) for v in g["case%d_shape" % ci])
        sa, sb = (int(v) for v in g["case%d_seeds" % ci])
        A, B = synth.uniform(sa, (M, K)), synth.uniform(sb, (K, N))
        assert normwise(run_dgemm(A, B), g["case%d_avx" % ci], A, B) <= TOL
    A, B = synth.uniform(42, (256, 256)), synth.uniform(43, (256, 256))      # configuration 1
    Cg = run_dgemm(A, B)
    assert np.abs(Cg[17] - g["c1_avx_row17"]).max() <= 1e-13
    assert abs(float(np.sum(Cg.astype(np.longdouble))) - float(g["c1_avx_sum"][0])) <= 1e-9


def test_known_answers_are_exact(gpu):
    a = np.array([[1., 2.], [3., 4.]]); b = np.array([[5., 6.], [7., 8.]])
    assert np.array_equal(run_dgemm(a, b), [[19, 22], [43, 50]])
    assert np.array_equal(run_dgemm(np.eye(2), a), a)
    a23 = np.array([[1., 2., 3.], [4., 5., 6.]]); b32 = np.array([[7., 8.], [9., 10.], [11., 12.]])
    assert np.array_equal(run_dgemm(a23, b32), [[58, 64], [139, 154]])
    assert np.array_equal(run_dgemm(run_dgemm(a, b), a), [[85, 126], [193, 286]])
    assert np.array_equal(run_dgemm(np.arange(6.).reshape(2, 3), np.arange(6.).reshape(3, 2)), [[10, 13], [28, 40]])
    assert run_dgemm(np.ones((1, 100)), np.arange(100.).reshape(100, 1))[0, 0] == 4950.0
    for n in (4, 8, 10, 16, 32, 46, 47, 49, 50, 51, 53, 64, 100, 192):
        assert np.all(run_dgemm(np.ones((n, n)), np.ones((n, n))) == float(n)), n
    S = np.arange(2500.).reshape(50, 50)
    assert np.array_equal(run_dgemm(S, np.eye(50)), S)
    R = np.repeat(np.arange(1., 51.)[:, None], 50, axis=1)
    assert np.array_equal(run_dgemm(R, np.ones((50, 50)))[:, 0], 50.0 * np.arange(1, 51))


def test_nonsquare_tile_edges_config2b_reduced(gpu):
    # configuration 2b is M=8192, N=1024, K=8192; same aspect at a size the oracle finishes
    A, B = synth.normal(7, (1024, 1024)), synth.normal(8, (1024, 128))
    assert normwise(run_dgemm(A, B), oracle.matmul_f64(A, B), A, B) <= TOL


@pytest.mark.parametrize("M,K,N", [(8192, 8192, 8192), (8192, 8192, 1024)])
def test_full_size_properties(gpu, M, K, N):
    """Configuration 2 at full size: exact integer identities that hold for any
    summation order, plus sampled rows and columns against the oracle."""
    print("dgemm full", M, K, N, flush=True)
    i = np.arange(M * K, dtype=np.int64).reshape(M, K)
    j = np.arange(K * N, dtype=np.int64).reshape(K, N)
    A = ((i * 7 + i // K) % 7 - 3).astype(np.float64)
    B = ((j * 5 + j // N) % 5 - 2).astype(np.float64)
    Cg = run_dgemm(A, B)
    # checksum of checksums: all quantities are integers far below 2^53
    assert np.array_equal(Cg.sum(axis=1), A @ B.sum(axis=1))
    assert np.array_equal(Cg.sum(axis=0), A.sum(axis=0) @ B)
    rows = [0, 1, 127, 128, 4095, M - 129, M - 1]
    cols = [0, 1, 127, 128, 777, N - 129, N - 1]
    assert np.array_equal(Cg[rows][:, cols], A[rows] @ B[:, cols])
    # real-valued inputs of the configuration, sampled block against the oracle
    A, B = synth.normal(11, (M, K)), synth.normal(12, (K, N))
    Cg = run_dgemm(A, B)
    ref = oracle.matmul_f64(A[rows], B[:, cols])
    assert normwise(Cg[rows][:, cols], ref, A[rows], B[:, cols]) <= TOL


@pytest.mark.parametrize("M,K,N", [(2048, 16, 2048), (2048, 48, 2048), (2048, 1024, 2048), (4096, 2064, 1024),
                                   (1024, 512, 4096), (2050, 130, 2046), (2049, 1000, 2050), (3000, 72, 1500),
                                   (1922, 4098, 2174), (2048, 18, 2048), (2176, 30, 1930)])
def test_straight_line_kernel_matches_bounds_checked_kernel_bitwise(gpu, tiled, M, K, N):
    """Large launches take a kernel without bounds checks (edge rows clamped,
    k-tail zeroed): same tiles, same summation order, so the same bits as the
    bounds-checked kernel, for all three operand forms. The output buffer is
    pre-filled with NaN and framed by guard rows to catch stray stores."""
    import eshkol_amd as ea
    from gpu_util import stream
    lib = ea.load()
    A, B = synth.normal(M + K, (M, K)), synth.normal(K + N, (K, N))
    ref = oracle.matmul_f64(A, B) if M * K * N <= 2 ** 32 else None
    forms = [(A, B, 0, 0), (A, np.ascontiguousarray(B.T), 0, 1), (np.ascontiguousarray(A.T), B, 1, 0)]
    for X, Y, ta, tb in forms:
        dX, dY = ea.DeviceArray.from_host(X), ea.DeviceArray.from_host(Y)
        outs = []
        try:
            for fast in (0, 1):
                lib.hip_dgemm_set_fast_path(fast)
                lib.hip_dgemm_set_tail_split(0)
                guard = np.full((M + 2, N), np.nan)
                guard[0] = guard[-1] = 12345.0
                dC = ea.DeviceArray.from_host(guard)
                assert lib.hip_dgemm_f64_ex(dX.ptr, dY.ptr, dC.ptr + N * 8, M, K, N, ta, tb, stream()) == 0
                ea.synchronize()
                got = dC.download()
                assert np.all(got[0] == 12345.0) and np.all(got[-1] == 12345.0)
                outs.append(got[1:-1])
        finally:
            lib.hip_dgemm_set_fast_path(1)
            lib.hip_dgemm_set_tail_split(1)
        assert np.array_equal(outs[0], outs[1]), (ta, tb)
        if ref is not None:
            assert normwise(outs[1], ref, A, B) <= TOL


def test_straight_line_kernel_in_a_batch(gpu):
    import eshkol_amd as ea
    from gpu_util import stream
    lib = ea.load()
    bt, M, K, N = 3, 2048, 64, 2048
    a, b = synth.normal(5, (bt, M, K)), synth.normal(6, (bt, K, N))
    da, db, dc = ea.DeviceArray.from_host(a), ea.DeviceArray.from_host(b), ea.DeviceArray((bt, M, N))
    assert lib.hip_dgemm_f64_batched(da.ptr, db.ptr, dc.ptr, bt, M, K, N, stream()) == 0
    ea.synchronize()
    got = dc.download()
    for i in range(bt):
        assert normwise(got[i], oracle.matmul_f64(a[i], b[i]), a[i], b[i]) <= TOL


@pytest.mark.parametrize("M,K,N", [(3072, 256, 3072), (3072, 1000, 3072), (3000, 520, 3100), (3200, 160, 3072),
                                   (2944, 4100, 3060)])
def test_k_split_last_round(gpu, tiled, M, K, N):
    """More than one round of tiles with a nearly empty last round: those tiles are cut
    along k and the pieces added in a fixed order. Same result on every run, the tiles
    of the full rounds bit-identical to an unsplit launch, everything within the tier's
    bound, nothing stored outside C; for all three operand forms."""
    import eshkol_amd as ea
    from gpu_util import stream
    lib = ea.load()
    A, B = synth.normal(M + 3 * K, (M, K)), synth.normal(K + 3 * N, (K, N))
    ref = oracle.matmul_f64(A, B) if M * K * N <= 2 ** 33 else None
    forms = [(A, B, 0, 0), (A, np.ascontiguousarray(B.T), 0, 1), (np.ascontiguousarray(A.T), B, 1, 0)]
    for X, Y, ta, tb in forms:
        dX, dY = ea.DeviceArray.from_host(X), ea.DeviceArray.from_host(Y)
        outs = []
        try:
            lib.hip_dgemm_set_small_tile(0)     # this test is about the large tiles of a cut last round
            for split in (0, 1, 1):
                lib.hip_dgemm_set_tail_split(split)
                guard = np.full((M + 2, N), np.nan)
                guard[0] = guard[-1] = 12345.0
                dC = ea.DeviceArray.from_host(guard)
                assert lib.hip_dgemm_f64_ex(dX.ptr, dY.ptr, dC.ptr + N * 8, M, K, N, ta, tb, stream()) == 0
                ea.synchronize()
                got = dC.download()
                assert np.all(got[0] == 12345.0) and np.all(got[-1] == 12345.0)
                outs.append(got[1:-1])
        finally:
            lib.hip_dgemm_set_tail_split(1)
            lib.hip_dgemm_set_small_tile(1)
        whole, cut, again = outs
        assert np.array_equal(cut, again), (ta, tb)
        same = (whole == cut)
        assert not same.all(), "the launch was expected to split its last round"
        assert same.mean() > 0.5                      # the full rounds are untouched
        assert np.isfinite(cut).all()
        if ref is not None:
            assert normwise(cut, ref, A, B) <= TOL, (ta, tb)
        else:
            assert np.abs(cut - whole).max() <= 1e-11 * np.sqrt(K)


@pytest.mark.parametrize("M,K,N", [(512, 2048, 512), (128, 8192, 128), (400, 1000, 400), (300, 1002, 1100),
                                   (1536, 1024, 1536), (130, 4098, 258), (1152, 1152, 1152)])
def test_k_split_of_a_launch_that_does_not_fill_the_device(gpu, tiled, M, K, N):
    """Fewer 128 x 128 tiles than CUs: every tile is cut along k and the pieces are added in
    a fixed order. Same bits on every run, within the tier's bound (against the whole launch
    too), nothing stored outside C; for all three operand forms."""
    import eshkol_amd as ea
    from gpu_util import stream
    lib = ea.load()
    A, B = synth.normal(M + 5 * K, (M, K)), synth.normal(K + 5 * N, (K, N))
    ref = oracle.matmul_f64(A, B)
    forms = [(A, B, 0, 0), (A, np.ascontiguousarray(B.T), 0, 1), (np.ascontiguousarray(A.T), B, 1, 0)]
    for X, Y, ta, tb in forms:
        dX, dY = ea.DeviceArray.from_host(X), ea.DeviceArray.from_host(Y)
        outs = []
        try:
            lib.hip_dgemm_set_small_tile(0)     # this test is about the large tiles cut along k
            for split in (0, 1, 1):
                lib.hip_dgemm_set_tail_split(split)
                guard = np.full((M + 2, N), np.nan)
                guard[0] = guard[-1] = 12345.0
                dC = ea.DeviceArray.from_host(guard)
                assert lib.hip_dgemm_f64_ex(dX.ptr, dY.ptr, dC.ptr + N * 8, M, K, N, ta, tb, stream()) == 0
                ea.synchronize()
                got = dC.download()
                assert np.all(got[0] == 12345.0) and np.all(got[-1] == 12345.0)
                outs.append(got[1:-1])
        finally:
            lib.hip_dgemm_set_tail_split(1)
            lib.hip_dgemm_set_small_tile(1)
        whole, cut, again = outs
        assert np.array_equal(cut, again), (ta, tb)
        assert not np.array_equal(whole, cut), "the launch was expected to be cut along k"
        assert normwise(cut, ref, A, B) <= 1e-14 and normwise(cut, whole, A, B) <= 1e-14


@pytest.mark.parametrize("M,K,N", [(1024, 1024, 1024), (1000, 700, 1300), (130, 4098, 258), (64, 16, 64), (2, 16, 2),
                                   (900, 1001 * 2, 1100), (2048, 512, 2048)])
def test_small_tile_kernel_gives_the_bits_of_the_large_one(gpu, tiled, M, K, N):
    """The straight-line kernel with 64 x 64 tiles (launches that would otherwise be cut along k)
    sums every output element in the same order as the 128 x 128 one: with whole tiles the two
    must agree bit for bit, for all three operand forms, edge tiles and k-tails included, and
    store nothing outside C."""
    import eshkol_amd as ea
    from gpu_util import stream
    lib = ea.load()
    A, B = synth.normal(M + 11 * K, (M, K)), synth.normal(K + 11 * N, (K, N))
    forms = [(A, B, 0, 0), (A, np.ascontiguousarray(B.T), 0, 1), (np.ascontiguousarray(A.T), B, 1, 0)]
    try:
        lib.hip_dgemm_set_tail_split(0)
        for X, Y, ta, tb in forms:
            dX, dY = ea.DeviceArray.from_host(X), ea.DeviceArray.from_host(Y)
            outs = []
            for mode in (0, 2):
                lib.hip_dgemm_set_small_tile(mode)
                guard = np.full((M + 2, N), np.nan)
                guard[0] = guard[-1] = 12345.0
                dC = ea.DeviceArray.from_host(guard)
                assert lib.hip_dgemm_f64_ex(dX.ptr, dY.ptr, dC.ptr + N * 8, M, K, N, ta, tb, stream()) == 0
                ea.synchronize()
                got = dC.download()
                assert np.all(got[0] == 12345.0) and np.all(got[-1] == 12345.0)
                outs.append(got[1:-1])
            assert np.array_equal(outs[0], outs[1]), (ta, tb)
            assert normwise(outs[1], oracle.matmul_f64(A, B), A, B) <= TOL
    finally:
        lib.hip_dgemm_set_tail_split(1)
        lib.hip_dgemm_set_small_tile(1)


@pytest.mark.parametrize("M,K,N", [(1536, 1024, 1536), (1280, 1288, 1280), (1300, 2000, 1250), (1792, 1024, 1800)])
def test_k_split_of_the_small_tiles_left_over(gpu, tiled, M, K, N):
    """64 x 64 tiles beyond the last multiple of the CU count are cut along k, in the same
    launch behind the whole ones, and their pieces added in a fixed order. Same result on
    every run, the whole tiles bit-identical to an uncut launch, everything within the
    tier's bound, nothing stored outside C; for all three operand forms, with edge tiles
    and k-tails."""
    import eshkol_amd as ea
    from gpu_util import stream
    lib = ea.load()
    A, B = synth.normal(M + 17 * K, (M, K)), synth.normal(K + 17 * N, (K, N))
    ref = oracle.matmul_f64(A, B)
    forms = [(A, B, 0, 0), (A, np.ascontiguousarray(B.T), 0, 1), (np.ascontiguousarray(A.T), B, 1, 0)]
    for X, Y, ta, tb in forms:
        dX, dY = ea.DeviceArray.from_host(X), ea.DeviceArray.from_host(Y)
        outs = []
        try:
            lib.hip_dgemm_set_small_tile(2)
            for split in (0, 1, 1):
                lib.hip_dgemm_set_tail_split(split)
                guard = np.full((M + 2, N), np.nan)
                guard[0] = guard[-1] = 12345.0
                dC = ea.DeviceArray.from_host(guard)
                assert lib.hip_dgemm_f64_ex(dX.ptr, dY.ptr, dC.ptr + N * 8, M, K, N, ta, tb, stream()) == 0
                ea.synchronize()
                got = dC.download()
                assert np.all(got[0] == 12345.0) and np.all(got[-1] == 12345.0)
                outs.append(got[1:-1])
        finally:
            lib.hip_dgemm_set_tail_split(1)
            lib.hip_dgemm_set_small_tile(1)
        whole, cut, again = outs
        assert np.array_equal(cut, again), (ta, tb)
        same = (whole == cut)
        assert not same.all(), "the launch was expected to cut its leftover tiles"
        assert same.mean() > 0.5                      # the whole tiles are untouched
        assert np.isfinite(cut).all()
        assert normwise(cut, ref, A, B) <= TOL, (ta, tb)
        assert normwise(cut, whole, A, B) <= 1e-14


@pytest.mark.parametrize("M,K,N", [(1024, 1024, 1024), (2304, 512, 2304), (3072, 640, 3072), (520, 4096, 500), (2048, 2048, 2048),
                                   (4096, 256, 4100), (300, 1002, 1100)])
def test_the_tile_size_chosen_by_itself_changes_no_bits_of_whole_tiles(gpu, tiled, M, K, N):
    """The library picks the tile size of the straight-line kernel from the launch's shape.
    With every tile whole (no cuts along k) all choices sum in the same order: the default
    must give the bits of both forced sizes, and with cuts allowed stay within the tier's bound."""
    import eshkol_amd as ea
    from gpu_util import stream
    lib = ea.load()
    A, B = synth.normal(M + 13 * K, (M, K)), synth.normal(K + 13 * N, (K, N))
    dA, dB, dC = ea.DeviceArray.from_host(A), ea.DeviceArray.from_host(B), ea.DeviceArray((M, N))
    outs = {}
    try:
        for split, mode in ((0, 0), (0, 1), (0, 2), (1, 1)):
            lib.hip_dgemm_set_tail_split(split); lib.hip_dgemm_set_small_tile(mode)
            assert lib.hip_dgemm_f64(dA.ptr, dB.ptr, dC.ptr, M, K, N, stream()) == 0
            ea.synchronize()
            outs[split, mode] = dC.download()
    finally:
        lib.hip_dgemm_set_tail_split(1); lib.hip_dgemm_set_small_tile(1)
    assert np.array_equal(outs[0, 0], outs[0, 1]) and np.array_equal(outs[0, 0], outs[0, 2])
    assert normwise(outs[1, 1], oracle.matmul_f64(A, B), A, B) <= TOL
    for depth in (1, 2):                      # both prefetch depths of the kernels: same bits
        lib.hip_dgemm_set_prefetch_depth(depth)
        try:
            lib.hip_dgemm_set_tail_split(0)
            assert lib.hip_dgemm_f64(dA.ptr, dB.ptr, dC.ptr, M, K, N, stream()) == 0
            ea.synchronize()
            assert np.array_equal(dC.download(), outs[0, 0]), depth
        finally:
            lib.hip_dgemm_set_prefetch_depth(0); lib.hip_dgemm_set_tail_split(1)
