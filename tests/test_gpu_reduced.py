"""Reduced-precision tier on the GPU. Bar (BASELINE.json): normwise error
<= 1e-2 against the reference's reduced tier, whose CPU statement is the f64
GEMM over operands already rounded to the 16-bit type."""
import ctypes as C

import numpy as np
import pytest

import eshkol_amd as ea
import oracle
from eshkol_amd import synth
from gpu_util import Operands, normwise, run_reduced, stream

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.mark.parametrize("dtype", [2, 3])
@pytest.mark.parametrize("M,K,N", [(1, 1, 1), (5, 3, 4), (64, 128, 64), (100, 200, 90), (257, 129, 255),
                                   (512, 512, 512), (33, 2049, 65), (1024, 768, 640),
                                   (1, 20001, 1), (9001, 3, 5), (5, 3, 9001), (2, 2, 65537)])
def test_reduced_matches_reference_statement(gpu, M, K, N, dtype):
    print("reduced", M, K, N, dtype, flush=True)
    A = synth.normal(700 + M, (M, K), 1.0 / np.sqrt(K))      # configuration 4's input law
    B = synth.normal(800 + N, (K, N), 1.0 / np.sqrt(K))
    # The runtime hands this tier tensors whose f64 storage was already rounded to the
    # 16-bit type when they were created (runtime_tensor_dtype.cpp:194-229).
    Ar, Br = oracle.reduce_precision(A, dtype), oracle.reduce_precision(B, dtype)
    ref = oracle.matmul_f64(Ar, Br)
    assert np.array_equal(ref, oracle.matmul_reduced(A, B, dtype))
    wide = run_reduced(Ar, Br, dtype, round_output=False)
    assert normwise(wide, ref, Ar, Br) <= 1e-6               # fp32 accumulation only
    narrow = run_reduced(Ar, Br, dtype, round_output=True)   # what the reference's 16F output does
    assert normwise(narrow, ref, Ar, Br) <= TOL
    ok = (np.abs(wide) >= 2.0 ** -14) | (wide == 0)         # outside the reference's f16 subnormal quirk
    assert np.array_equal(narrow[ok], oracle.reduce_precision(wide, dtype)[ok])
    if dtype == 3:
        # fp32 accumulation order is unspecified; the sum is close to a k-ascending one
        assert normwise(wide, oracle.matmul_reduced_f32acc(A, B, dtype, False), Ar, Br) <= 1e-6


@pytest.mark.parametrize("dtype", [2, 3])
@pytest.mark.parametrize("M,K,N", [(1, 8192, 256), (5, 7000, 300), (32, 4096, 1024), (33, 2049, 1030), (64, 520, 4099),
                                   (17, 512, 4100), (40, 16400, 130), (100, 4096, 1024), (128, 1031, 2050)])
def test_a_few_rows_against_a_big_second_operand(gpu, M, K, N, dtype):
    """Up to 128 rows against B as the runtime stores it: B is read once as fp64 and narrowed in registers on
    its way to the matrix cores. Same arithmetic as the tier's other kernels (16-bit operands, fp32 sums), so:
    the reference statement within the fp32 bar, the rounded output the unrounded one rounded, the tiled path
    within the scatter of fp32 summation orders, an infinity in B in its own column only, the entry point that
    allocates nothing the same bits."""
    print("reduced, few rows", M, K, N, dtype, flush=True)
    lib = ea.load()
    A = oracle.reduce_precision(synth.normal(700 + M, (M, K), 1.0 / np.sqrt(K)), dtype)
    B = oracle.reduce_precision(synth.normal(800 + N, (K, N), 1.0 / np.sqrt(K)), dtype)
    ref = oracle.matmul_f64(A, B)
    wide = run_reduced(A, B, dtype, round_output=False)
    assert normwise(wide, ref, A, B) <= 1e-6
    narrow = run_reduced(A, B, dtype, round_output=True)
    ok = (np.abs(wide) >= 2.0 ** -14) | (wide == 0)
    assert np.array_equal(narrow[ok], oracle.reduce_precision(wide, dtype)[ok])
    lib.hip_reduced_set_thin(0)
    try:
        tiled = run_reduced(A, B, dtype, round_output=False)
    finally:
        lib.hip_reduced_set_thin(1)
    assert normwise(wide, tiled, A, B) <= 1e-6 and not np.array_equal(wide, tiled) or M * N < 64
    # operands that are not 16-bit values yet are narrowed on the way, as by the narrowing kernels
    A2, B2 = synth.normal(1 + M, (M, K)), synth.normal(2 + N, (K, N))
    got = run_reduced(A2, B2, dtype, round_output=False)
    want = oracle.matmul_f64(oracle.reduce_precision(A2, dtype), oracle.reduce_precision(B2, dtype))
    assert normwise(got, want, A2, B2) <= 1e-6
    # an infinity in the last row of k and in the last column shows in its own column only
    B3 = B.copy(); B3[K - 1, 3] = np.inf; B3[0, N - 1] = -np.inf
    A3 = A.copy(); A3[:, K - 1] = np.abs(A3[:, K - 1]) + 2.0 ** -6; A3[:, 0] = np.abs(A3[:, 0]) + 2.0 ** -6
    A3 = oracle.reduce_precision(A3, dtype)
    got = run_reduced(A3, B3, dtype, round_output=False)
    assert np.all(got[:, 3] == np.inf) and np.all(got[:, N - 1] == -np.inf)
    keep = np.ones(N, bool); keep[[3, N - 1]] = False
    assert np.isfinite(got[:, keep]).all()
    if M * K <= (1 << 20) and K * N <= (4 << 20):
        ops = Operands(A, B)
        assert lib.hip_matmul_reduced_f64_noalloc(ops.dA.ptr, ops.dB.ptr, ops.dC.ptr, M, K, N, dtype, 0, stream()) == 0
        assert np.array_equal(ops.result(), wide)


@pytest.mark.parametrize("dtype", [2, 3])
@pytest.mark.parametrize("thin,K,wide", [(1, 8192, 300), (7, 2049, 1030), (33, 4100, 520), (64, 515, 4099), (65, 2049, 1030),
                                         (96, 4100, 520), (128, 515, 4099)])
def test_a_few_rows_or_columns_in_every_operand_form(gpu, thin, K, wide, dtype):
    """The thin side may be M or N, and either operand may be held transposed: two kernels (the big operand
    with the output index contiguous, or with k contiguous) serve all of them. Against the reference statement
    within the fp32 bar, and the tiled path within the scatter of fp32 summation orders."""
    print("reduced, thin side, forms", thin, K, wide, dtype, flush=True)
    lib = ea.load()
    for (M, N) in ((thin, wide), (wide, thin)):
        A = oracle.reduce_precision(synth.normal(70 + M, (M, K), 1.0 / np.sqrt(K)), dtype)
        B = oracle.reduce_precision(synth.normal(80 + N, (K, N), 1.0 / np.sqrt(K)), dtype)
        ref = oracle.matmul_f64(A, B)
        for ta, tb in ((0, 0), (0, 1), (1, 0)):
            X = np.ascontiguousarray(A.T) if ta else A
            Y = np.ascontiguousarray(B.T) if tb else B
            dX, dY, dC = ea.DeviceArray.from_host(X), ea.DeviceArray.from_host(Y), ea.DeviceArray((M, N))
            outs = []
            for on in (1, 0):
                lib.hip_reduced_set_thin(on)
                try:
                    assert lib.hip_matmul_reduced_f64_ex(dX.ptr, dY.ptr, dC.ptr, M, K, N, ta, tb, dtype, 0, stream()) == 0
                    ea.synchronize()
                finally:
                    lib.hip_reduced_set_thin(1)
                outs.append(dC.download())
            assert normwise(outs[0], ref, A, B) <= 1e-6, (M, N, ta, tb)
            assert normwise(outs[0], outs[1], A, B) <= 1e-6
            assert lib.hip_matmul_reduced_f64_ex(dX.ptr, dY.ptr, dC.ptr, M, K, N, ta, tb, dtype, 1, stream()) == 0
            ea.synchronize()
            narrow = dC.download()
            ok = (np.abs(outs[0]) >= 2.0 ** -14) | (outs[0] == 0)
            assert np.array_equal(narrow[ok], oracle.reduce_precision(outs[0], dtype)[ok])


def test_random_shapes_with_a_thin_side_take_whichever_kernel_and_agree(gpu):
    """Sixty random shapes with one side of at most 140 and a random operand form: whichever kernel the tier picks
    (the ones that read the big operand once, or narrowing and tiles), the result is the reference statement's within
    the fp32 bar. Small integers that are 16-bit values make the sums exact in fp32 whatever their order: those
    must come out bit for bit."""
    lib = ea.load()
    rng = np.random.default_rng(77)
    for it in range(60):
        thin = int(rng.integers(1, 141))
        wide = int(2 ** rng.uniform(7, 12.3))
        K = int(2 ** rng.uniform(6, 13))
        M, N = (thin, wide) if rng.integers(0, 2) else (wide, thin)
        ta, tb = [(0, 0), (0, 0), (0, 1), (1, 0)][int(rng.integers(0, 4))]
        dtype = 2 + int(rng.integers(0, 2))
        print("reduced, random", M, K, N, ta, tb, dtype, flush=True)
        A = rng.integers(-3, 4, (M, K)).astype(np.float64)
        B = rng.integers(-3, 4, (K, N)).astype(np.float64)
        X = np.ascontiguousarray(A.T) if ta else A
        Y = np.ascontiguousarray(B.T) if tb else B
        dX, dY, dC = ea.DeviceArray.from_host(X), ea.DeviceArray.from_host(Y), ea.DeviceArray((M, N))
        assert lib.hip_matmul_reduced_f64_ex(dX.ptr, dY.ptr, dC.ptr, M, K, N, ta, tb, dtype, 0, stream()) == 0
        ea.synchronize()
        assert np.array_equal(dC.download(), A @ B), (M, K, N, ta, tb, dtype)
        A = oracle.reduce_precision(rng.standard_normal((M, K)) / np.sqrt(K), dtype)
        B = oracle.reduce_precision(rng.standard_normal((K, N)) / np.sqrt(K), dtype)
        X = np.ascontiguousarray(A.T) if ta else A
        Y = np.ascontiguousarray(B.T) if tb else B
        dX, dY = ea.DeviceArray.from_host(X), ea.DeviceArray.from_host(Y)
        assert lib.hip_matmul_reduced_f64_ex(dX.ptr, dY.ptr, dC.ptr, M, K, N, ta, tb, dtype, 0, stream()) == 0
        ea.synchronize()
        assert normwise(dC.download(), A @ B, A, B) <= 1e-6, (M, K, N, ta, tb, dtype)


@pytest.mark.parametrize("dtype", [2, 3])
@pytest.mark.parametrize("M,K,N", [(3072, 256, 3072), (3000, 200, 2900), (3001, 200, 2901), (3072, 256, 3073)])
def test_rounded_output_of_the_kernel_for_large_products(gpu, M, K, N, dtype):
    """From 128 tiles of 256 x 256 on, the tier's contraction is the kernel that loads its
    operands straight into LDS and MFMA registers, with an epilogue of its own for every
    output form. Its rounded f64 output must be its unrounded one rounded to the 16-bit type,
    value for value: whole tiles (3072^2) and ragged edges, with infinities, an infinity minus
    infinity and a sum beyond the 16-bit type's range among the results."""
    print("reduced, large, rounded", M, K, N, dtype, flush=True)
    A = oracle.reduce_precision(synth.normal(900 + M, (M, K), 1.0 / np.sqrt(K)), dtype)
    B = oracle.reduce_precision(synth.normal(950 + N, (K, N), 1.0 / np.sqrt(K)), dtype)
    A[0, 0] = np.inf; B[0, 0] = 1.0                   # row 0: infinities
    A[1, 0] = np.inf; A[1, 1] = -np.inf; B[0, 1] = 1.0; B[1, 1] = 1.0     # inf - inf: NaN
    A[2, :] = (65504.0 if dtype == 2 else 1.0e38) / K; B[:, 2] = 2.0      # finite in fp32, beyond f16 once rounded
    A, B = oracle.reduce_precision(A, dtype), oracle.reduce_precision(B, dtype)
    wide = run_reduced(A, B, dtype, round_output=False)
    narrow = run_reduced(A, B, dtype, round_output=True)
    assert np.isinf(wide[0, 0]) and np.isnan(wide[1, 1]) and np.isfinite(wide[2, 2])
    if dtype == 2:
        assert np.isinf(narrow[2, 2])
    ref = oracle.matmul_f64(A[3:67], B[:, 3:])
    assert normwise(wide[3:67, 3:], ref, A[3:67], B[:, 3:]) <= 1e-6
    ok = (np.abs(wide) >= 2.0 ** -14) | (wide == 0) | np.isnan(wide)    # outside the reference's f16 subnormal quirk
    assert np.array_equal(narrow[ok], oracle.reduce_precision(wide, dtype)[ok], equal_nan=True)


@pytest.mark.parametrize("is_bf16", [0, 1])
def test_device_narrowing_is_round_to_nearest_even(gpu, is_bf16):
    lib = ea.load()
    rows, cols, rp, ld = 37, 150, 256, 192
    x = np.concatenate([synth.normal(1, (3000,)), synth.normal(2, (1500,)) * 300.0,
                        synth.normal(3, (1000,)) * 1e-3, np.array([0.0, -0.0, 1.0009765625, 65504.0, 65520.0, 1e6])])
    x = np.resize(x, rows * cols).reshape(rows, cols)
    d_in = ea.DeviceArray.from_host(x)
    d_out = ea.DeviceArray((rp, ld), np.uint16)
    assert lib.hip_convert_f64_to_16(d_in.ptr, d_out.ptr, rows, cols, rp, ld, is_bf16, stream()) == 0
    ea.synchronize()
    got = d_out.download()
    assert not got[rows:].any() and not got[:, cols:].any()
    bits = got[:rows, :cols]
    if is_bf16:
        val = (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    else:
        val = bits.view(np.float16).astype(np.float64)
    normal_range = (np.abs(x) >= 2.0 ** -14) | (x == 0)
    expect = oracle.reduce_precision(x, 3 if is_bf16 else 2)
    assert np.array_equal(val[normal_range], expect[normal_range])
    assert np.array_equal(np.signbit(val), np.signbit(expect))


def test_hgemm_fp32_output_config4_reduced_size(gpu):
    """The contraction alone, bf16 in / fp32 out (configuration 4 at 1024^3)."""
    lib = ea.load()
    n = 1024
    A = synth.normal(4, (n, n), 1.0 / np.sqrt(n)); B = synth.normal(5, (n, n), 1.0 / np.sqrt(n))
    dA, dBt = ea.DeviceArray.from_host(A), ea.DeviceArray.from_host(np.ascontiguousarray(B.T))
    a16, b16 = ea.DeviceArray((n, n), np.uint16), ea.DeviceArray((n, n), np.uint16)
    assert lib.hip_convert_f64_to_16(dA.ptr, a16.ptr, n, n, n, n, 1, stream()) == 0
    assert lib.hip_convert_f64_to_16(dBt.ptr, b16.ptr, n, n, n, n, 1, stream()) == 0
    dC = ea.DeviceArray((n, n), np.float32)
    assert lib.hip_hgemm_16(a16.ptr, b16.ptr, n, n, n, n, 1, dC.ptr, stream()) == 0
    ea.synchronize()
    Cg = dC.download().astype(np.float64)
    Ar, Br = oracle.reduce_precision(A, 3), oracle.reduce_precision(B, 3)
    assert normwise(Cg, oracle.matmul_f64(Ar, Br), Ar, Br) <= 1e-6


@pytest.mark.parametrize("is_bf16", [0, 1])
@pytest.mark.parametrize("M,K,N", [(1, 8192, 256), (7, 2050, 1030), (32, 4096, 4096), (33, 1000, 2100), (100, 520, 4099),
                                   (128, 4096, 1024)])
def test_a_few_rows_of_16_bit_operands_stream_the_second_operand(gpu, M, K, N, is_bf16):
    """hip_hgemm_16 on up to 128 rows against a big second operand reads that operand once
    instead of tiling it: against the oracle on the narrowed operands, and, on small
    integers (exact in fp32 whatever the order of the sums), equal to the tiled kernel."""
    print("hgemm16 thin", M, K, N, is_bf16, flush=True)
    lib = ea.load()
    dtype = 3 if is_bf16 else 2
    rp = lambda r: -(-r // 256) * 256
    ld = -(-K // 64) * 64

    def run(A, Bt):
        dA, dBt = ea.DeviceArray.from_host(A), ea.DeviceArray.from_host(Bt)
        a16 = ea.DeviceArray.from_host(np.full((rp(M), ld), 0x7777, np.uint16))
        b16 = ea.DeviceArray.from_host(np.full((rp(N), ld), 0x7777, np.uint16))
        assert lib.hip_convert_f64_to_16(dA.ptr, a16.ptr, M, K, rp(M), ld, is_bf16, stream()) == 0
        assert lib.hip_convert_f64_to_16(dBt.ptr, b16.ptr, N, K, rp(N), ld, is_bf16, stream()) == 0
        dC = ea.DeviceArray.from_host(np.full((M, N), np.nan, np.float32))
        assert lib.hip_hgemm_16(a16.ptr, b16.ptr, M, K, N, ld, is_bf16, dC.ptr, stream()) == 0
        ea.synchronize()
        return dC.download().astype(np.float64)

    A = synth.normal(70 + M, (M, K), 1.0 / np.sqrt(K)); Bt = synth.normal(71 + N, (N, K), 1.0 / np.sqrt(K))
    if is_bf16:
        Ar, Br = oracle.reduce_precision(A, dtype), oracle.reduce_precision(Bt, dtype).T
    else:       # IEEE narrowing, subnormals included (the device's; the reference's f16 narrowing differs below 2^-14)
        Ar, Br = A.astype(np.float16).astype(np.float64), Bt.astype(np.float16).astype(np.float64).T
    assert normwise(run(A, Bt), oracle.matmul_f64(Ar, Br), Ar, Br) <= 1e-6
    i = np.arange(M * K, dtype=np.int64).reshape(M, K); j = np.arange(N * K, dtype=np.int64).reshape(N, K)
    Ai = ((i * 7 + i // K) % 7 - 3).astype(np.float64); Bi = ((j * 5 + j // K) % 5 - 2).astype(np.float64)
    want = Ai @ Bi.T
    assert np.array_equal(run(Ai, Bi), want)
    lib.hip_reduced_set_thin(0)
    try:
        assert np.array_equal(run(Ai, Bi), want)
    finally:
        lib.hip_reduced_set_thin(1)


def test_full_size_config4_sampled(gpu):
    n = 8192
    print("reduced full", n, flush=True)
    A = synth.normal(61, (n, n), 1.0 / np.sqrt(n)); B = synth.normal(62, (n, n), 1.0 / np.sqrt(n))
    Cg = run_reduced(A, B, 3, round_output=False)
    rows = [0, 1, 255, 256, 4097, n - 257, n - 1]
    cols = [0, 3, 255, 256, 5000, n - 256, n - 1]
    Ar, Br = oracle.reduce_precision(A[rows], 3), oracle.reduce_precision(B[:, cols], 3)
    assert normwise(Cg[rows][:, cols], oracle.matmul_f64(Ar, Br), Ar, Br) <= TOL
    # linearity in exact arithmetic: small integers are exact in bf16 and in fp32 sums
    i = np.arange(n * n, dtype=np.int64).reshape(n, n)
    Ai = ((i * 7 + i // n) % 7 - 3).astype(np.float64); Bi = ((i * 5 + i // n) % 5 - 2).astype(np.float64)
    Ci = run_reduced(Ai, Bi, 3, round_output=False)
    assert np.array_equal(Ci.sum(axis=1), Ai @ Bi.sum(axis=1))
    assert np.array_equal(Ci[rows][:, cols], Ai[rows] @ Bi[:, cols])


def _interleaved16(x):
    """uint16 [rows][ld] -> the interleaved plane: rows in blocks of 32, 16-byte chunks slow, rows fast."""
    rows, ld = x.shape
    y = x.reshape(rows // 32, 32, ld // 8, 8).transpose(0, 2, 1, 3)
    return np.ascontiguousarray(y).reshape(rows, ld)


@pytest.mark.parametrize("is_bf16", [0, 1])
@pytest.mark.parametrize("rows,cols", [(1, 1), (37, 150), (300, 70), (513, 1000), (1024, 1024)])
def test_interleaved_narrowing_holds_the_same_values(gpu, rows, cols, is_bf16):
    """The interleaved 16-bit planes, from either operand order and for a batch, are the
    row-major planes element for element, padding included."""
    lib = ea.load()
    batch = 3
    x = synth.normal(rows + 3 * cols, (batch, rows, cols)) * 3.0
    rp, ld = -(-rows // 256) * 256, -(-cols // 256) * 256
    d_in = ea.DeviceArray.from_host(x)
    d_in_t = ea.DeviceArray.from_host(np.ascontiguousarray(x.transpose(0, 2, 1)))
    ref = ea.DeviceArray.from_host(np.full((batch, rp, ld), 0x7878, np.uint16))
    assert lib.hip_convert_f64_to_16_planes(d_in.ptr, ref.ptr, batch, rows, cols, rp, ld, is_bf16, 0, 0, stream()) == 0
    ea.synchronize()
    want = ref.download()
    assert not want[:, rows:].any() and not want[:, :, cols:].any()
    one = ea.DeviceArray.from_host(np.full((rp, ld), 0x7777, np.uint16))
    assert lib.hip_convert_f64_to_16(ea.DeviceArray.from_host(x[1]).ptr, one.ptr, rows, cols, rp, ld, is_bf16, stream()) == 0
    ea.synchronize()
    assert np.array_equal(one.download(), want[1])
    for kmajor, src in ((0, d_in), (1, d_in_t)):
        for layout in (0, 1):
            out = ea.DeviceArray.from_host(np.full((batch, rp, ld), 0x7777, np.uint16))
            assert lib.hip_convert_f64_to_16_planes(src.ptr, out.ptr, batch, rows, cols, rp, ld, is_bf16,
                                                    kmajor, layout, stream()) == 0
            ea.synchronize()
            got = out.download()
            for b in range(batch):
                expect = _interleaved16(want[b]) if layout else want[b]
                assert np.array_equal(got[b], expect), (kmajor, layout, b)


@pytest.mark.parametrize("dtype", [2, 3])
@pytest.mark.parametrize("batch,M,K,N", [(64, 128, 256, 128), (5, 33, 70, 65), (3, 300, 129, 257), (8, 1024, 512, 1024),
                                         (2, 2048, 300, 2304)])
def test_batched_reduced_tier_in_one_launch(gpu, batch, M, K, N, dtype):
    """hip_matmul_reduced_f64_batched: many small experts (the simple kernel, batch on the grid)
    and batches that fill the device (interleaved operands, batch as the operand plane) give,
    matrix for matrix, the bits of the single-product entry point, and meet the tier's bound
    against the reference statement."""
    print("batched reduced", batch, M, K, N, dtype, flush=True)
    lib = ea.load()
    a = synth.normal(batch + M, (batch, M, K), 1.0 / np.sqrt(K))
    b = synth.normal(batch + N, (batch, K, N), 1.0 / np.sqrt(K))
    da, db, dc = ea.DeviceArray.from_host(a), ea.DeviceArray.from_host(b), ea.DeviceArray((batch, M, N))
    assert lib.hip_matmul_reduced_f64_batched(da.ptr, db.ptr, dc.ptr, batch, M, K, N, dtype, 1, stream()) == 0
    ea.synchronize()
    got = dc.download()
    for i in sorted({0, 1, batch // 2, batch - 1}):
        single = run_reduced(a[i], b[i], dtype, round_output=True)
        ar, br = oracle.reduce_precision(a[i], dtype), oracle.reduce_precision(b[i], dtype)
        assert normwise(got[i], oracle.matmul_f64(ar, br), ar, br) <= TOL, i
        # fp32 sums of the same operands in a possibly different order, then rounded to 16 bits:
        # equal up to one unit of that rounding, and exactly equal when both took the same kernel
        assert normwise(got[i], single, ar, br) <= 1e-4, i
    assert lib.hip_matmul_reduced_f64_batched(da.ptr, db.ptr, dc.ptr, 0, M, K, N, dtype, 1, stream()) == -1


def test_interleaved_contraction_config4_reduced_size(gpu):
    """bf16 operands resident in the interleaved layout, fp32 out, through hip_hgemm_16_batched:
    the direct-to-LDS kernel against the row-major one on the same operands. Integer operands make
    every fp32 sum exact, so the two must agree bit for bit there."""
    lib = ea.load()
    n = 2048
    i = np.arange(n * n, dtype=np.int64).reshape(n, n)
    cases = [(((i * 7 + i // n) % 7 - 3).astype(np.float64), ((i * 5 + i // n) % 5 - 2).astype(np.float64), True),
             (synth.normal(4, (n, n), 1.0 / np.sqrt(n)), synth.normal(5, (n, n), 1.0 / np.sqrt(n)), False)]
    for A, B, exact in cases:
        dA, dB = ea.DeviceArray.from_host(A), ea.DeviceArray.from_host(B)
        outs = []
        for layout in (0, 1):
            a16, b16 = ea.DeviceArray((n, n), np.uint16), ea.DeviceArray((n, n), np.uint16)
            assert lib.hip_convert_f64_to_16_planes(dA.ptr, a16.ptr, 1, n, n, n, n, 1, 0, layout, stream()) == 0
            assert lib.hip_convert_f64_to_16_planes(dB.ptr, b16.ptr, 1, n, n, n, n, 1, 1, layout, stream()) == 0
            dC = ea.DeviceArray((n, n), np.float32)
            assert lib.hip_hgemm_16_batched(a16.ptr, b16.ptr, 1, n, n, n, n, n, n, 1, layout, dC.ptr, stream()) == 0
            ea.synchronize()
            outs.append(dC.download().astype(np.float64))
        Ar, Br = oracle.reduce_precision(A, 3), oracle.reduce_precision(B, 3)
        ref = oracle.matmul_f64(Ar[:64], Br)
        for o in outs:
            assert normwise(o[:64], ref, Ar[:64], Br) <= 1e-6
        if exact:
            assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0][:64], ref)


@pytest.mark.parametrize("M,N", [(3000, 2901), (3072, 3073), (3001, 3070)])
def test_direct_kernel_fp32_rows_that_start_off_16_byte_boundaries(gpu, M, N):
    """fp32 results whose rows do not start on 16-byte boundaries (N not a multiple of four) leave the
    direct kernel as 16-byte stores all the same; integer operands make every sum exact, so the result
    must equal the integer product bit for bit, ragged edges included, and nothing may be written
    beyond the M x N values."""
    print("case: hip_hgemm_16_batched fp32 out", M, N, flush=True)
    lib = ea.load()
    K = 512
    rng = np.random.default_rng(M + N)
    A = rng.integers(-7, 8, (M, K)).astype(np.float64)
    B = rng.integers(-7, 8, (K, N)).astype(np.float64)
    dA, dB = ea.DeviceArray.from_host(A), ea.DeviceArray.from_host(B)
    Mp, Np = (M + 255) // 256 * 256, (N + 255) // 256 * 256
    assert lib.hip_hgemm_plane_layout(M, N, 1) == 1
    a16, b16 = ea.DeviceArray((Mp, K), np.uint16), ea.DeviceArray((Np, K), np.uint16)
    assert lib.hip_convert_f64_to_16_planes(dA.ptr, a16.ptr, 1, M, K, Mp, K, 1, 0, 1, stream()) == 0
    assert lib.hip_convert_f64_to_16_planes(dB.ptr, b16.ptr, 1, N, K, Np, K, 1, 1, 1, stream()) == 0
    guard = 64
    dC = ea.DeviceArray.from_host(np.full(M * N + guard, -1.5, np.float32))
    assert lib.hip_hgemm_16_batched(a16.ptr, b16.ptr, 1, M, K, N, Mp, Np, K, 1, 1, dC.ptr, stream()) == 0
    ea.synchronize()
    out = dC.download()
    assert np.all(out[M * N:] == -1.5)
    assert np.array_equal(out[:M * N].reshape(M, N).astype(np.float64), A @ B)


def test_direct_kernel_batched_with_integer_operands(gpu):
    """A batch through hip_hgemm_16_batched on interleaved operands (the direct kernel walks
    all matrices' tiles in one persistent launch, the batch index as the operand plane) against
    the row-major kernels on the same operands and against the exact integer product: small
    integers are exact in bf16 and every fp32 sum of their products is exact, so all three
    must agree bit for bit. K = 512 is the shortest tile the kernel has (one ring of four
    k-blocks); 24 matrices of 4 x 4 tiles are more tiles than CUs."""
    print("case: hip_hgemm_16_batched 24 x 1024x512x1024 integer operands", flush=True)
    lib = ea.load()
    batch, M, K, N = 24, 1024, 512, 1024
    rng = np.random.default_rng(5)
    A = rng.integers(-7, 8, (batch, M, K)).astype(np.float64)
    B = rng.integers(-7, 8, (batch, K, N)).astype(np.float64)
    dA, dB = ea.DeviceArray.from_host(A), ea.DeviceArray.from_host(B)
    assert lib.hip_hgemm_plane_layout(M, N, batch) == 1
    outs = []
    for layout in (0, 1):
        a16, b16 = ea.DeviceArray((batch, M, K), np.uint16), ea.DeviceArray((batch, N, K), np.uint16)
        assert lib.hip_convert_f64_to_16_planes(dA.ptr, a16.ptr, batch, M, K, M, K, 1, 0, layout, stream()) == 0
        assert lib.hip_convert_f64_to_16_planes(dB.ptr, b16.ptr, batch, N, K, N, K, 1, 1, layout, stream()) == 0
        dC = ea.DeviceArray((batch, M, N), np.float32)
        assert lib.hip_hgemm_16_batched(a16.ptr, b16.ptr, batch, M, K, N, M, N, K, 1, layout, dC.ptr, stream()) == 0
        ea.synchronize()
        outs.append(dC.download())
    assert np.array_equal(outs[0], outs[1])
    assert np.array_equal(outs[1].astype(np.float64), A @ B)
