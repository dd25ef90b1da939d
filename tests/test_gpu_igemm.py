"""The int8 matrix-core contraction on its own (hip_igemm_i8), against exact
integer arithmetic in numpy, for each of its kernels: the simple one, the
pipelined one (a workgroup per tile) and the persistent one (a workgroup per
CU walking a tile list). All three must give the same bits: int32 sums for
the slice tier's plans, symmetric residues for the CRT tier's."""
import ctypes as C

import numpy as np
import pytest

import eshkol_amd as ea
from gpu_util import stream

pytestmark = pytest.mark.gpu

MODULI = [256, 255, 253, 251, 247, 241, 239, 233, 229, 227, 223, 217, 211, 199, 197, 193]
KERNELS = {"simple": (0, 0), "pipelined": (2, 0), "persistent": (2, 1), "pipelined-1": (1, 0), "persistent-1": (1, 1),
           "direct": (2, 1),           # interleaved planes, operands loaded straight into LDS / MFMA registers
           "direct-half": (2, 1)}      # the same on 256 x 128 tiles, two workgroups per CU
DIRECT_MODE = {"direct": 3, "direct-half": 2}
# interleaved planes; "thin": what the entry point picks by itself for at most 64 rows of A
INTERLEAVED = set(DIRECT_MODE) | {"thin"}


def pad(n, m):
    return (n + m - 1) // m * m


def planes(rng, n_planes, rows, K, lo=-128, hi=128, row_pad=256):
    """[n_planes][rows padded to 256][K padded to 256] int8, padding zero."""
    out = np.zeros((n_planes, pad(rows, row_pad), pad(K, 256)), np.int8)
    out[:, :rows, :K] = rng.integers(lo, hi, (n_planes, rows, K), dtype=np.int8)
    return out


def interleave(x):
    """[n][rows][ldk] -> the interleaved layout: rows in blocks of 32, inside a block the
    16-byte k-chunks slow and the row fast; ldk padded to a multiple of 512 first."""
    n, rows, ldk = x.shape
    if ldk % 512:
        x = np.concatenate([x, np.zeros((n, rows, pad(ldk, 512) - ldk), np.int8)], axis=2)
        ldk = x.shape[2]
    y = x.reshape(n, rows // 32, 32, ldk // 16, 16).transpose(0, 1, 3, 2, 4)
    return np.ascontiguousarray(y).reshape(n, rows, ldk)


def run(a, b, M, N, plan, mode, kernel, out_rows=0, ldn=0):
    """plan: list of lists of (a_plane, b_plane) per output plane. out_rows, ldn: the output planes as
    allocated (0: M x N); the whole planes come back."""
    lib = ea.load()
    pf, pers = KERNELS.get(kernel, (2, 1))
    if kernel in INTERLEAVED:
        a, b = interleave(a), interleave(b)
    first = np.cumsum([0] + [len(p) for p in plan]).astype(np.int32)
    pa = np.array([t[0] for p in plan for t in p], np.int32)
    pb = np.array([t[1] for p in plan for t in p], np.int32)
    dA, dB = ea.DeviceArray.from_host(a), ea.DeviceArray.from_host(b)
    dF, dPa, dPb = (ea.DeviceArray.from_host(x) for x in (first, pa, pb))
    dMod = ea.DeviceArray.from_host(np.array(MODULI[:len(plan)] if mode == 1 else [1], np.int32))
    n_out = len(plan)
    out = ea.DeviceArray.from_host(np.full((n_out, out_rows or M, ldn or N), 0x55, np.int8 if mode == 1 else np.int32))
    g = ea.HipIgemmArgs()
    g.out_rows, g.ldn = out_rows, ldn
    g.a_planes, g.b_planes = dA.ptr, dB.ptr
    g.a_plane_stride, g.b_plane_stride = a.shape[1] * a.shape[2], b.shape[1] * b.shape[2]
    g.ldk, g.M, g.N, g.n_out = a.shape[2], M, N, n_out
    g.pair_first, g.pair_a, g.pair_b = dF.ptr, dPa.ptr, dPb.ptr
    g.mode, g.max_pairs, g.modulus = mode, max(len(p) for p in plan), dMod.ptr
    g.layout = 1 if kernel in INTERLEAVED else 0
    if mode == 1:
        g.out_i8 = out.ptr
    else:
        g.out_i32 = out.ptr
    lib.hip_igemm_set_prefetch(pf)
    lib.hip_igemm_set_persistent(pers)
    lib.hip_igemm_set_direct(DIRECT_MODE.get(kernel, 1))
    try:
        assert lib.hip_igemm_i8(C.byref(g), stream()) == 0
        ea.synchronize()
    finally:
        lib.hip_igemm_set_prefetch(2)
        lib.hip_igemm_set_persistent(1)
        lib.hip_igemm_set_direct(1)
    return out.download()


def exact(a, b, M, N, K, plan):
    """Sums of int8 products are integers far below 2^53: a float64 GEMM computes them exactly."""
    af, bf = a[:, :M, :K].astype(np.float64), b[:, :N, :K].astype(np.float64)
    return np.stack([sum(af[i] @ bf[j].T for i, j in p) for p in plan]).astype(np.int64)


def symmetric(v, p):
    r = np.mod(v, p)
    return np.where(2 * r >= p, r - p, r)


@pytest.mark.parametrize("kernel", list(KERNELS))
@pytest.mark.parametrize("M,K,N", [(1024, 1024, 1024), (1000, 700, 1300), (2048, 256, 1024), (1536, 1000, 1792)])
def test_residue_products(gpu, M, K, N, kernel):
    rng = np.random.default_rng(M + K)
    a, b = planes(rng, 16, M, K), planes(rng, 16, N, K)
    plan = [[(l, l)] for l in range(16)]
    got = run(a, b, M, N, plan, 1, kernel)
    want = exact(a, b, M, N, K, plan)
    for l, p in enumerate(MODULI):
        assert np.array_equal(got[l].astype(np.int64), symmetric(want[l], p)), (l, p)


@pytest.mark.parametrize("kernel", list(KERNELS))
@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("M,K,N,out_rows,ldn", [(1000, 700, 1300, 1024, 1536), (1000, 700, 1300, 1000, 1312),
                                                (2041, 512, 2051, 2048, 2304), (1023, 256, 1025, 1023, 1028)])
def test_output_planes_larger_than_the_product(gpu, M, K, N, out_rows, ldn, mode, kernel):
    """Output planes allocated with a row pitch and a row count of their own: the M x N corner holds what the
    dense call gives, the rest zeros (products of the operands' zero padding) or what was there before."""
    rng = np.random.default_rng(M + N + mode)
    n = 16 if mode == 1 else 3
    a, b = planes(rng, n, M, K), planes(rng, n, N, K)
    plan = [[(l, l)] for l in range(n)] if mode == 1 else [[(0, 0)], [(1, 1), (2, 2)], [(0, 2), (1, 0), (2, 1)]]
    dense = run(a, b, M, N, plan, mode, kernel)
    got = run(a, b, M, N, plan, mode, kernel, out_rows, ldn)
    assert got.shape == (len(plan), out_rows, ldn)
    assert np.array_equal(got[:, :M, :N], dense)
    rest = got.copy()
    rest[:, :M, :N] = 0
    fill = 0x55
    assert np.all((rest == 0) | (rest == fill))


THIN_SHAPES = [(1, 512, 32), (5, 700, 100), (32, 4096, 1024), (33, 1000, 1300), (64, 2049, 257), (17, 130, 4096),
               (64, 512, 4100), (32, 1, 1), (2, 513, 33),
               # 33 ... 160 rows: rows shared through LDS (two row blocks only against many column blocks)
               (40, 512, 4100), (65, 700, 100), (96, 4096, 1024), (128, 513, 300), (100, 1, 1), (129, 512, 4096),
               (160, 1000, 4100), (97, 2049, 129)]


@pytest.mark.parametrize("M,K,N", THIN_SHAPES)
def test_thin_first_operand_residues(gpu, M, K, N):
    """A few rows of A (up to 128, up to 160 against 4096 columns or more), planes padded to whole blocks of 32
    rows only: the kernels that stream B's planes."""
    rng = np.random.default_rng(M + K + N)
    a, b = planes(rng, 16, M, K, row_pad=32), planes(rng, 16, N, K)
    plan = [[(l, l)] for l in range(16)]
    got = run(a, b, M, N, plan, 1, "thin")
    want = exact(a, b, M, N, K, plan)
    for l, p in enumerate(MODULI):
        assert np.array_equal(got[l].astype(np.int64), symmetric(want[l], p)), (l, p)
    # the tiled kernel on the same operands (rows padded to its 256): the same bytes
    a256 = np.zeros((16, 256, a.shape[2]), np.int8)
    a256[:, :a.shape[1]] = a
    assert np.array_equal(run(a256, b, M, N, plan, 1, "direct"), got)


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("M,K,N,out_rows,ldn", [(7, 700, 100, 7, 112), (40, 512, 1030, 40, 1280), (64, 300, 33, 64, 33),
                                                (3, 1024, 95, 5, 95), (32, 520, 64, 32, 66), (100, 700, 90, 101, 96),
                                                (128, 512, 257, 128, 259), (50, 600, 4100, 64, 4112)])
def test_thin_first_operand_plans_and_output_pitches(gpu, M, K, N, out_rows, ldn, mode):
    """Several products per output plane (the slice tier's plans), int32 sums and residues, output planes with
    a pitch of their own, also one that keeps no store aligned."""
    rng = np.random.default_rng(M + N + mode)
    a, b = planes(rng, 3, M, K, row_pad=32), planes(rng, 3, N, K)
    plan = [[(0, 0)], [(1, 1), (2, 2)], [(0, 2), (1, 0), (2, 1)]]
    got = run(a, b, M, N, plan, mode, "thin", out_rows, ldn)
    want = exact(a, b, M, N, K, plan)
    if mode == 1:
        want = np.stack([symmetric(want[l], MODULI[l]) for l in range(3)])
    assert np.array_equal(got[:, :M, :N].astype(np.int64), want)
    rest = got.copy()
    rest[:, :M, :N] = 0
    assert np.all((rest == 0) | (rest == 0x55))


def test_thin_first_operand_extremes_of_the_accumulator(gpu):
    """All -128 against -128 and against 127 at the largest K: both ends of the int32 range."""
    M, N, K = 9, 96, 131072 - 256
    a = np.full((16, 32, K), -128, np.int8)
    a[:, M:] = 0
    b = np.full((16, 256, K), -128, np.int8)
    b[:, 1::2, :] = 127
    b[:, N:] = 0
    plan = [[(l, l)] for l in range(16)]
    got = run(a, b, M, N, plan, 1, "thin")
    want = exact(a, b, M, N, K, plan)
    for l, p in enumerate(MODULI):
        assert np.array_equal(got[l].astype(np.int64), symmetric(want[l], p)), (l, p)


@pytest.mark.parametrize("kernel", list(KERNELS))
def test_residues_at_the_extremes_of_the_accumulator(gpu, kernel):
    """All operands -128 (sums up to +K 2^14) and mixed signs (down to -K 127 128):
    the reduction must stay exact at both ends of the int32 range it is specified for."""
    M = N = 1024
    for K in (8192, 131072 - 256):
        a = np.full((16, M, pad(K, 256)), -128, np.int8)
        b = np.full((16, N, pad(K, 256)), -128, np.int8)
        a[:, :, K:] = 0
        b[:, 1::2, :] = 127
        b[:, :, K:] = 0
        if K > 8192:                      # keep the large case cheap: eight planes still fill the chip
            a, b = a[:8], b[:8]
        plan = [[(l, l)] for l in range(a.shape[0])]
        got = run(a, b, M, N, plan, 1, kernel)
        for l in range(a.shape[0]):
            p = MODULI[l]
            even, odd = K * 128 * 128, -K * 128 * 127
            assert np.all(got[l][:, 0::2] == symmetric(np.int64(even), p)), (K, l)
            assert np.all(got[l][:, 1::2] == symmetric(np.int64(odd), p)), (K, l)


@pytest.mark.parametrize("kernel", list(KERNELS))
@pytest.mark.parametrize("M,K,N,s", [(1024, 512, 1024, 7), (900, 300, 1100, 5), (2048, 256, 2048, 3), (2048, 512, 2048, 5),
                                     (1800, 1100, 2300, 7)])
def test_slice_diagonal_sums(gpu, M, K, N, s, kernel):
    """The slice tier's plan: output d sums the products (p, d - p); several products per output."""
    rng = np.random.default_rng(s * M)
    a, b = planes(rng, s, M, K, -127, 128), planes(rng, s, N, K, -127, 128)
    plan = [[(p, d - p) for p in range(s) if 0 <= d - p < s] for d in range(s)]
    got = run(a, b, M, N, plan, 0, kernel)
    assert np.array_equal(got.astype(np.int64), exact(a, b, M, N, K, plan))


@pytest.mark.parametrize("M,K,N", [(4096, 1024, 4096), (4096, 4096, 4096), (4096, 4096, 1024), (4096, 512, 4096)])
def test_direct_kernel_on_the_mlp_shapes_and_the_shortest_tiles(gpu, M, K, N):
    """The direct kernel's loads are issued from asm statements and waited for by count, so a
    late operand would show as a wrong residue and nowhere else. The layer shapes of BASELINE
    configuration 5 (16 planes, K = 1024 and 4096: 4096 or 1024 tiles on 256 CUs, the request
    cursor crossing a tile boundary every 8 or 32 k-blocks) and the shortest tile there is
    (K = 512: one ring of four k-blocks, so the cursor is in the next tile during every block):
    all residues against the persistent kernel's, bit for bit, and sampled rows against exact
    integer arithmetic."""
    print("case: direct kernel %dx%dx%d, 16 planes" % (M, K, N), flush=True)
    rng = np.random.default_rng(M + 3 * K + 7 * N)
    a, b = planes(rng, 16, M, K), planes(rng, 16, N, K)
    plan = [[(l, l)] for l in range(16)]
    got = run(a, b, M, N, plan, 1, "direct")
    assert np.array_equal(got, run(a, b, M, N, plan, 1, "persistent"))
    assert np.array_equal(got, run(a, b, M, N, plan, 1, "direct-half"))
    rows = np.unique(np.concatenate([np.arange(0, M, 257), [63, 64, 255, 256, M - 1]]))
    for l, p in enumerate(MODULI):
        want = a[l][rows, :K].astype(np.float64) @ b[l][:N, :K].astype(np.float64).T
        assert np.array_equal(got[l][rows].astype(np.int64), symmetric(want.astype(np.int64), p)), (l, p)


def test_bad_arguments(gpu):
    lib = ea.load()
    g = ea.HipIgemmArgs()
    assert lib.hip_igemm_i8(C.byref(g), stream()) == -1
    assert lib.hip_igemm_i8(None, stream()) == -1
