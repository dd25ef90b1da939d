"""Matmul backward on the GPU through the C ABI: the transposed-operand forms
of the native fp64 kernel, the tier pipelines fed operands the caller holds
transposed, hip_matmul_backward_f64 and eshkol_gpu_matmul_backward_f64,
against the oracle's restatement of eshkol_matmul_backward_f64
(lib/backend/blas_backend.cpp:924-1039).

Bars: native fp64 normwise <= 1e-14; Ozaki tiers bit-identical to the same
tier on explicit transposed copies (the pipelines see the same k-contiguous
operands either way) and to the oracle of that tier; integer cases exact."""
import ctypes as C

import numpy as np
import pytest

import eshkol_amd as ea
import oracle
from eshkol_amd import synth
from gpu_util import normwise, run_crt, run_int8, stream
from test_gpu_dispatch import run_child

pytestmark = pytest.mark.gpu
TOL = 1e-14

SHAPES = [(1, 1, 1), (2, 3, 4), (5, 7, 3), (16, 16, 16), (64, 64, 64), (65, 67, 66), (37, 130, 9),
          (129, 257, 131), (256, 256, 256), (300, 17, 500), (512, 1000, 64), (1000, 33, 1000),
          (1024, 1024, 1024), (2050, 130, 2046)]


def dev(x):
    return ea.DeviceArray.from_host(np.ascontiguousarray(x, dtype=np.float64))


def dgemm_ex(X, Y, m, k, n, ta, tb):
    """C[m x n] = op(X) op(Y) with X, Y as the caller holds them."""
    dX, dY, dZ = dev(X), dev(Y), ea.DeviceArray((m, n))
    assert ea.load().hip_dgemm_f64_ex(dX.ptr, dY.ptr, dZ.ptr, m, k, n, ta, tb, stream()) == 0
    ea.synchronize()
    return dZ.download()


def backward(G, A, B, tier, T=0):
    M, K = A.shape
    N = B.shape[1]
    dG, dA, dB = dev(G), dev(A), dev(B)
    gA, gB = ea.DeviceArray((M, K)), ea.DeviceArray((K, N))
    rc = ea.load().hip_matmul_backward_f64(dG.ptr, dA.ptr, dB.ptr, gA.ptr, gB.ptr, M, K, N, tier, T, stream())
    assert rc == 0
    ea.synchronize()
    return gA.download(), gB.download()


@pytest.mark.parametrize("M,K,N", SHAPES)
def test_native_transposed_operands_match_oracle(gpu, M, K, N):
    print("dgemm_ex", M, K, N, flush=True)
    A, B = synth.uniform(100 + M, (M, K)), synth.uniform(200 + N, (K, N))
    ref = oracle.matmul_f64(A, B)
    At, Bt = np.ascontiguousarray(A.T), np.ascontiguousarray(B.T)
    assert normwise(dgemm_ex(A, Bt, M, K, N, 0, 1), ref, A, B) <= TOL
    assert normwise(dgemm_ex(At, B, M, K, N, 1, 0), ref, A, B) <= TOL


def test_native_rejects_both_transposed(gpu):
    dX, dZ = dev(np.ones((4, 4))), ea.DeviceArray((4, 4))
    assert ea.load().hip_dgemm_f64_ex(dX.ptr, dX.ptr, dZ.ptr, 4, 4, 4, 1, 1, stream()) == -1


@pytest.mark.parametrize("M,K,N", [(1, 1, 1), (2, 3, 4), (31, 33, 29), (130, 64, 258), (257, 300, 129)])
def test_native_backward_integers_exact(gpu, M, K, N):
    rng = np.random.default_rng(M * 7 + N)
    G = rng.integers(-9, 10, (M, N)).astype(np.float64)
    A = rng.integers(-9, 10, (M, K)).astype(np.float64)
    B = rng.integers(-9, 10, (K, N)).astype(np.float64)
    gA, gB = backward(G, A, B, 0)
    assert np.array_equal(gA, G @ B.T) and np.array_equal(gB, A.T @ G)


@pytest.mark.parametrize("M,K,N", [(64, 48, 80), (17, 23, 11), (300, 513, 130), (1024, 768, 512)])
def test_native_backward_matches_oracle(gpu, M, K, N):
    G, A, B = synth.normal(1 + M, (M, N)), synth.normal(2 + K, (M, K)), synth.normal(3 + N, (K, N))
    gA, gB = backward(G, A, B, 0)
    oA, oB = oracle.matmul_backward_f64(G, A, B)
    assert normwise(gA, oA, G, B) <= TOL
    assert normwise(gB, oB, A, G) <= TOL


def test_skipping_one_gradient(gpu):
    G, A, B = synth.normal(1, (40, 24)), synth.normal(2, (40, 56)), synth.normal(3, (56, 24))
    dG, dA, dB = dev(G), dev(A), dev(B)
    gA = ea.DeviceArray.from_host(np.full((40, 56), 7.0))
    gB = ea.DeviceArray.from_host(np.full((56, 24), 7.0))
    lib = ea.load()
    assert lib.hip_matmul_backward_f64(dG.ptr, dA.ptr, dB.ptr, gA.ptr, None, 40, 56, 24, 0, 0, stream()) == 0
    ea.synchronize()
    assert np.all(gB.download() == 7.0) and normwise(gA.download(), G @ B.T, G, B) <= TOL
    assert lib.hip_matmul_backward_f64(dG.ptr, dA.ptr, dB.ptr, None, None, 40, 56, 24, 0, 0, stream()) == -1


@pytest.mark.parametrize("M,K,N", [(512, 512, 512), (520, 777, 300)])
def test_crt_tier_backward_is_bit_identical_to_forward_on_transposed_copies(gpu, M, K, N):
    G, A, B = synth.normal(5, (M, N)), synth.wide_range(6, (M, K)), synth.normal(7, (K, N))
    gA, gB = backward(G, A, B, 2)
    # the same tier on explicit copies, and the oracle of the tier
    rc, fA, _ = run_crt(G, np.ascontiguousarray(B.T), want_stages=False)
    assert rc == 0 and np.array_equal(gA, fA)
    rc, fB, _ = run_crt(np.ascontiguousarray(A.T), G, want_stages=False)
    assert rc == 0 and np.array_equal(gB, fB)
    assert np.array_equal(gA, oracle.matmul_ozaki_crt(G, np.ascontiguousarray(B.T)))
    assert np.array_equal(gB, oracle.matmul_ozaki_crt(np.ascontiguousarray(A.T), G))


@pytest.mark.parametrize("T", [1, 4, 6])
def test_int8_tier_backward_is_bit_identical_to_forward_on_transposed_copies(gpu, T):
    M, K, N = 384, 300, 260
    G, A, B = synth.normal(8, (M, N)), synth.normal(9, (M, K)), synth.uniform(10, (K, N))
    gA, gB = backward(G, A, B, 1, T)
    rc, fA, _ = run_int8(G, np.ascontiguousarray(B.T), T, want_stages=False)
    assert rc == 0 and np.array_equal(gA, fA)
    rc, fB, _ = run_int8(np.ascontiguousarray(A.T), G, T, want_stages=False)
    assert rc == 0 and np.array_equal(gB, fB)
    assert np.array_equal(gA, oracle.matmul_ozaki_int8(G, np.ascontiguousarray(B.T), T))
    assert np.array_equal(gB, oracle.matmul_ozaki_int8(np.ascontiguousarray(A.T), G, T))


def test_reduced_tier_with_operands_held_transposed(gpu):
    M, K, N = 200, 330, 140
    A = oracle.reduce_precision(synth.normal(11, (M, K)), 3)
    B = oracle.reduce_precision(synth.normal(12, (K, N)), 3)
    lib = ea.load()
    dA, dB, dAt, dBt = dev(A), dev(B), dev(A.T), dev(B.T)
    outs = []
    for (x, y, ta, tb) in ((dA, dB, 0, 0), (dA, dBt, 0, 1), (dAt, dB, 1, 0)):
        dC = ea.DeviceArray((M, N))
        assert lib.hip_matmul_reduced_f64_ex(x.ptr, y.ptr, dC.ptr, M, K, N, ta, tb, 3, 0, stream()) == 0
        ea.synchronize()
        outs.append(dC.download())
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


def test_buffer_entry_default_tier(gpu):
    lib = ea.load()
    M, K, N = 260, 140, 330
    G, A, B = synth.normal(13, (M, N)), synth.normal(14, (M, K)), synth.normal(15, (K, N))
    dG, dA, dB = dev(G), dev(A), dev(B)
    gA, gB = ea.DeviceArray((M, K)), ea.DeviceArray((K, N))
    rc = lib.eshkol_gpu_matmul_backward_f64(C.byref(dG.buf), C.byref(dA.buf), C.byref(dB.buf),
                                            C.byref(gA.buf), C.byref(gB.buf), M, K, N)
    assert rc == 0
    oA, oB = oracle.matmul_backward_f64(G, A, B)
    assert normwise(gA.download(), oA, G, B) <= TOL and normwise(gB.download(), oB, A, G) <= TOL
    # a buffer too small for its shape is refused
    small = ea.DeviceArray((M, K - 1))
    assert lib.eshkol_gpu_matmul_backward_f64(C.byref(dG.buf), C.byref(dA.buf), C.byref(dB.buf),
                                              C.byref(small.buf), C.byref(gB.buf), M, K, N) == -1


def test_buffer_entry_follows_the_tier_override(gpu):
    r = run_child(r"""
assert lib.eshkol_gpu_init() == 1
M, K, N = 640, 512, 576
G, A, B = synth.normal(16, (M, N)), synth.normal(17, (M, K)), synth.normal(18, (K, N))
dG, dA, dB = (ea.DeviceArray.from_host(x) for x in (G, A, B))
gA, gB = ea.DeviceArray((M, K)), ea.DeviceArray((K, N))
assert lib.eshkol_gpu_matmul_backward_f64(C.byref(dG.buf), C.byref(dA.buf), C.byref(dB.buf),
                                          C.byref(gA.buf), C.byref(gB.buf), M, K, N) == 0
assert np.array_equal(gA.download(), oracle.matmul_ozaki_crt(G, np.ascontiguousarray(B.T)))
assert np.array_equal(gB.download(), oracle.matmul_ozaki_crt(np.ascontiguousarray(A.T), G))
""", env={"ESHKOL_HIP_F64_KERNEL": "ozaki-crt", "ESHKOL_GPU_VERBOSE": "1"})
    assert r.stderr.count("[GPU] Ozaki-II: N=16") == 2
    assert r.stderr.count("Ozaki-II CRT exact") == 2


def test_full_size_backward_properties(gpu):
    """8192-wide gradients: integer identities that hold in any summation order."""
    M, K, N = 8192, 2048, 4096
    i = np.arange(M * N, dtype=np.int64).reshape(M, N)
    G = ((i * 7 + i // N) % 7 - 3).astype(np.float64)
    i = np.arange(M * K, dtype=np.int64).reshape(M, K)
    A = ((i * 5 + i // K) % 5 - 2).astype(np.float64)
    i = np.arange(K * N, dtype=np.int64).reshape(K, N)
    B = ((i * 3 + i // N) % 11 - 5).astype(np.float64)
    gA, gB = backward(G, A, B, 0)
    assert np.array_equal(gA.sum(axis=1), G @ B.sum(axis=0))          # row sums of G B^T
    assert np.array_equal(gB.sum(axis=1), A.T @ G.sum(axis=1))        # row sums of A^T G
    rows = [0, 1, 127, 128, 4095, M - 1]
    assert np.array_equal(gA[rows], G[rows] @ B.T)
    cols = [0, 1, 127, 128, 777, N - 1]
    assert np.array_equal(gB[:, cols], A.T @ G[:, cols])


@pytest.mark.parametrize("M,K,N", [(1537, 1601, 1409), (2049, 1024, 2047), (2048, 1025, 2048), (1409, 2001, 1538),
                                   (513, 515, 517), (301, 1999, 303), (33, 2048, 2048)])
def test_native_large_operands_with_rows_off_16_byte_boundaries(gpu, M, K, N):
    """Large products whose operands have an odd pitch are copied to an even one and run the straight-line
    kernel with that pitch. Small integers make every sum exact, so all three operand forms must give the
    integer product bit for bit, edges included; random operands must stay within the tier's tolerance."""
    print("dgemm_ex, odd pitches", M, K, N, flush=True)
    rng = np.random.default_rng(M + K + N)
    A = rng.integers(-9, 10, (M, K)).astype(np.float64)
    B = rng.integers(-9, 10, (K, N)).astype(np.float64)
    ref = A @ B
    At, Bt = np.ascontiguousarray(A.T), np.ascontiguousarray(B.T)
    assert np.array_equal(dgemm_ex(A, B, M, K, N, 0, 0), ref)
    assert np.array_equal(dgemm_ex(A, Bt, M, K, N, 0, 1), ref)
    assert np.array_equal(dgemm_ex(At, B, M, K, N, 1, 0), ref)
    A, B = synth.uniform(100 + M, (M, K)), synth.uniform(200 + N, (K, N))
    rows = np.array([0, 1, M // 2, M - 2, M - 1])
    got = dgemm_ex(A, B, M, K, N, 0, 0)
    assert normwise(got[rows], oracle.matmul_f64(A[rows], B), A[rows], B) <= TOL
    assert normwise(got, A @ B, A, B) <= TOL


def test_native_large_operands_with_a_base_off_16_byte_boundaries(gpu):
    """Even pitches, but the operands start 8 bytes into their buffers."""
    M, K, N = 1536, 1600, 1408
    rng = np.random.default_rng(3)
    A = rng.integers(-9, 10, (M, K)).astype(np.float64)
    B = rng.integers(-9, 10, (K, N)).astype(np.float64)
    bufA = ea.DeviceArray.from_host(np.concatenate([[777.0], A.ravel()]))
    bufB = ea.DeviceArray.from_host(np.concatenate([[777.0], B.ravel()]))
    dC = ea.DeviceArray((M, N))
    assert ea.load().hip_dgemm_f64_ex(bufA.ptr + 8, bufB.ptr + 8, dC.ptr, M, K, N, 0, 0, stream()) == 0
    ea.synchronize()
    assert np.array_equal(dC.download(), A @ B)


@pytest.mark.parametrize("thin", [1, 2, 3, 5, 8, 9, 16, 17, 32, 33, 48, 64, 65])
@pytest.mark.parametrize("wide,K", [(1024, 1024), (1025, 1031), (4096, 100), (3001, 2050), (4097, 4100)])
def test_native_products_with_one_thin_side(gpu, thin, wide, K):
    """A vector or a few against a matrix take kernels of their own, bound by HBM (up to 64 rows where the big
    operand has the output index contiguous: the matrix cores stream it), in all three operand forms and with
    either side thin. Integer operands make every sum exact, so the result must
    be the integer product bit for bit; random operands must stay within the tier's tolerance."""
    print("dgemm_ex, thin side", thin, wide, K, flush=True)
    rng = np.random.default_rng(thin * 7 + wide + K)
    for (M, N) in ((thin, wide), (wide, thin)):
        A = rng.integers(-9, 10, (M, K)).astype(np.float64)
        B = rng.integers(-9, 10, (K, N)).astype(np.float64)
        ref = A @ B
        At, Bt = np.ascontiguousarray(A.T), np.ascontiguousarray(B.T)
        assert np.array_equal(dgemm_ex(A, B, M, K, N, 0, 0), ref)
        assert np.array_equal(dgemm_ex(A, Bt, M, K, N, 0, 1), ref)
        assert np.array_equal(dgemm_ex(At, B, M, K, N, 1, 0), ref)
        A, B = synth.uniform(100 + M, (M, K)), synth.uniform(200 + N, (K, N))
        ref = oracle.matmul_f64(A, B) if M * N * K <= (1 << 27) else A @ B
        At, Bt = np.ascontiguousarray(A.T), np.ascontiguousarray(B.T)
        assert normwise(dgemm_ex(A, B, M, K, N, 0, 0), ref, A, B) <= TOL
        assert normwise(dgemm_ex(A, Bt, M, K, N, 0, 1), ref, A, B) <= TOL
        assert normwise(dgemm_ex(At, B, M, K, N, 1, 0), ref, A, B) <= TOL


@pytest.mark.parametrize("M,K,N", [(1, 1 << 19, 2), (2, 1 << 19, 2), (2, 1 << 19, 1), (3, 70000, 900)])
def test_native_products_thin_on_both_sides_keep_the_tiled_kernel(gpu, M, K, N):
    """Neither side is wide: not a shape for the thin kernels; the result must not care."""
    rng = np.random.default_rng(M + N)
    A = rng.integers(-9, 10, (M, K)).astype(np.float64)
    B = rng.integers(-9, 10, (K, N)).astype(np.float64)
    assert np.array_equal(dgemm_ex(A, B, M, K, N, 0, 0), A @ B)
    assert np.array_equal(dgemm_ex(A, np.ascontiguousarray(B.T), M, K, N, 0, 1), A @ B)
    assert np.array_equal(dgemm_ex(np.ascontiguousarray(A.T), B, M, K, N, 1, 0), A @ B)


def test_native_thin_products_write_nothing_else(gpu):
    """The result of a thin product lies in a buffer with guard values around it."""
    lib = ea.load()
    for (M, K, N) in ((3, 777, 2049), (2049, 777, 3), (1, 4096, 4097), (4097, 4096, 1), (33, 1031, 2049), (2049, 1031, 48),
                      (135, 2559, 349), (20, 3000, 18)):
        rng = np.random.default_rng(M + N)
        A = rng.integers(-9, 10, (M, K)).astype(np.float64)
        B = rng.integers(-9, 10, (K, N)).astype(np.float64)
        dA, dB = dev(A), dev(B)
        buf = ea.DeviceArray.from_host(np.full(M * N + 128, -7.25))
        assert lib.hip_dgemm_f64(dA.ptr, dB.ptr, buf.ptr + 64 * 8, M, K, N, stream()) == 0
        ea.synchronize()
        out = buf.download()
        assert np.all(out[:64] == -7.25) and np.all(out[64 + M * N:] == -7.25)
        assert np.array_equal(out[64:64 + M * N].reshape(M, N), A @ B)


@pytest.mark.parametrize("M,K,N", [(135, 2559, 349), (100, 8192, 100), (256, 4096, 256), (65, 1500, 300), (70, 32768, 128),
                                   (32, 4109, 36), (51, 7755, 52), (12, 215, 60), (49, 5536, 2), (129, 1024, 1024),
                                   (64, 512, 16), (16, 64, 2048), (2, 65, 128), (256, 1024, 64), (65, 1024, 17), (48, 511, 4000),
                                   (49, 511, 4000), (64, 16384, 33)])
def test_native_small_outputs_with_a_long_k(gpu, M, K, N):
    """Up to 256 rows against a narrow operand with a long k: chunks of 64 rows through the kernel that streams the
    big operand, all operand forms and either side as the thin one; integers exact, random operands within tolerance."""
    print("dgemm_ex, small outputs, long k", M, K, N, flush=True)
    rng = np.random.default_rng(M + K + N)
    for (m, n) in ((M, N), (N, M)):
        A = rng.integers(-9, 10, (m, K)).astype(np.float64)
        B = rng.integers(-9, 10, (K, n)).astype(np.float64)
        ref = A @ B
        At, Bt = np.ascontiguousarray(A.T), np.ascontiguousarray(B.T)
        assert np.array_equal(dgemm_ex(A, B, m, K, n, 0, 0), ref)
        assert np.array_equal(dgemm_ex(A, Bt, m, K, n, 0, 1), ref)
        assert np.array_equal(dgemm_ex(At, B, m, K, n, 1, 0), ref)
        A, B = synth.uniform(100 + m, (m, K)), synth.uniform(200 + n, (K, n))
        assert normwise(dgemm_ex(A, B, m, K, n, 0, 0), A @ B, A, B) <= TOL


def test_native_batch_of_rows_against_a_matrix_with_infinities_and_an_odd_base(gpu):
    """9 ... 64 rows against a matrix read through the matrix cores: an infinity in the big operand shows in its
    own column only (the zeros that pad the last round of k must not meet it), also when k is not a multiple of
    the round and the strip of columns is cut; operands whose base is 8 bytes off a 16-byte boundary."""
    lib = ea.load()
    M, K, N = 20, 1031, 1100
    rng = np.random.default_rng(5)
    A = rng.integers(-9, 10, (M, K)).astype(np.float64)
    B = rng.integers(-9, 10, (K, N)).astype(np.float64)
    A[:, K - 1] = np.abs(A[:, K - 1]) + 1.0
    B[K - 1, 7] = np.inf
    B[3, N - 1] = -np.inf
    A[:, 3] = np.abs(A[:, 3]) + 1.0
    bufA = ea.DeviceArray.from_host(np.concatenate([[0.0], A.ravel()]))
    bufB = ea.DeviceArray.from_host(np.concatenate([[0.0], B.ravel()]))
    out = ea.DeviceArray.from_host(np.zeros(M * N + 1))
    assert lib.hip_dgemm_f64(bufA.ptr + 8, bufB.ptr + 8, out.ptr + 8, M, K, N, stream()) == 0
    ea.synchronize()
    got = out.download()[1:].reshape(M, N)
    with np.errstate(invalid="ignore"):
        want = A @ B
    assert np.all(got[:, 7] == np.inf) and np.all(got[:, N - 1] == -np.inf)
    keep = np.ones(N, bool)
    keep[[7, N - 1]] = False
    assert np.array_equal(got[:, keep], want[:, keep])


@pytest.mark.parametrize("batch,M,K,N", [(1, 1, 1, 1), (1, 3, 3, 3), (7, 3, 3, 3), (4096, 8, 8, 8), (1000, 5, 7, 6), (513, 16, 16, 16),
                                         (300, 32, 32, 32), (33, 32, 31, 1), (65, 1, 64, 32), (100, 2, 500, 2), (2, 32, 32, 32),
                                         (70001, 4, 4, 4), (1000, 33, 17, 29), (40, 64, 5, 16), (40, 16, 9, 64)])
def test_native_batches_of_matrices_far_smaller_than_a_tile(gpu, batch, M, K, N):
    """Matrices of a few kilobytes, several to a workgroup: small integers make every sum exact, so
    the batch must equal the integer products bit for bit, the buffer's guard values untouched;
    random operands within the tier's tolerance of the oracle's batch loop."""
    print("dgemm small batched", batch, M, K, N, flush=True)
    lib = ea.load()
    rng = np.random.default_rng(batch + M + K + N)
    A = rng.integers(-9, 10, (batch, M, K)).astype(np.float64)
    B = rng.integers(-9, 10, (batch, K, N)).astype(np.float64)
    dA, dB = dev(A), dev(B)
    buf = ea.DeviceArray.from_host(np.full(batch * M * N + 128, -7.25))
    assert lib.hip_dgemm_f64_batched(dA.ptr, dB.ptr, buf.ptr + 64 * 8, batch, M, K, N, stream()) == 0
    ea.synchronize()
    out = buf.download()
    assert np.all(out[:64] == -7.25) and np.all(out[64 + batch * M * N:] == -7.25)
    assert np.array_equal(out[64:64 + batch * M * N].reshape(batch, M, N), A @ B)
    nb = min(batch, 50)
    A, B = synth.uniform(1 + M, (nb, M, K)), synth.uniform(2 + N, (nb, K, N))
    dA, dB, dC = dev(A), dev(B), ea.DeviceArray((nb, M, N))
    assert lib.hip_dgemm_f64_batched(dA.ptr, dB.ptr, dC.ptr, nb, M, K, N, stream()) == 0
    ea.synchronize()
    got = dC.download()
    for b in range(nb):
        assert normwise(got[b], oracle.matmul_f64(A[b], B[b]), A[b], B[b]) <= TOL
        # one matrix on its own, in every operand form, gives the batch's bits
        if b < 3:
            assert np.array_equal(dgemm_ex(A[b], B[b], M, K, N, 0, 0), got[b])
            assert np.array_equal(dgemm_ex(A[b], np.ascontiguousarray(B[b].T), M, K, N, 0, 1), got[b])
            assert np.array_equal(dgemm_ex(np.ascontiguousarray(A[b].T), B[b], M, K, N, 1, 0), got[b])


@pytest.mark.parametrize("M,K,N", [(1, 6699, 139), (13, 6701, 11), (108, 5980, 3), (6, 3945, 1), (1, 1919, 1), (27, 3215, 6),
                                   (31, 300, 33), (16, 100000, 16), (255, 257, 1), (64, 256, 16), (1, 256, 255), (32, 4097, 32)])
def test_native_products_of_few_outputs_and_a_long_k(gpu, M, K, N):
    """Few outputs, long k: the contraction is cut into slices over the workgroups and the pieces are
    added in a fixed order. Integer operands: exact, bit for bit, in every operand form; random
    operands within the tier's tolerance; the same call twice gives the same bits."""
    print("dgemm small long k", M, K, N, flush=True)
    rng = np.random.default_rng(M + K + N)
    A = rng.integers(-9, 10, (M, K)).astype(np.float64)
    B = rng.integers(-9, 10, (K, N)).astype(np.float64)
    ref = A @ B
    At, Bt = np.ascontiguousarray(A.T), np.ascontiguousarray(B.T)
    assert np.array_equal(dgemm_ex(A, B, M, K, N, 0, 0), ref)
    assert np.array_equal(dgemm_ex(A, Bt, M, K, N, 0, 1), ref)
    assert np.array_equal(dgemm_ex(At, B, M, K, N, 1, 0), ref)
    A, B = synth.uniform(100 + M, (M, K)), synth.uniform(200 + N, (K, N))
    got = dgemm_ex(A, B, M, K, N, 0, 0)
    assert normwise(got, oracle.matmul_f64(A, B), A, B) <= TOL
    assert np.array_equal(got, dgemm_ex(A, B, M, K, N, 0, 0))
    assert normwise(dgemm_ex(np.ascontiguousarray(A.T), B, M, K, N, 1, 0), oracle.matmul_f64(A, B), A, B) <= TOL
    assert normwise(dgemm_ex(A, np.ascontiguousarray(B.T), M, K, N, 0, 1), oracle.matmul_f64(A, B), A, B) <= TOL


def test_native_random_shapes_take_whichever_kernel_and_agree_with_integers(gpu):
    """Eighty shapes drawn log-uniformly (1 ... 3000 per dimension), random operand form: whichever of
    the fp64 kernels a shape is routed to (tiles with or without a cut k, copies to an even pitch, the
    thin-side kernels, the kernels for matrices smaller than a tile), small integers must come out as
    the exact integer product."""
    rng = np.random.default_rng(20240)
    for case in range(80):
        M, K, N = (max(1, int(2 ** rng.uniform(0, 11.55))) for _ in range(3))
        ta, tb = [(0, 0), (0, 1), (1, 0)][rng.integers(0, 3)]
        print("dgemm_ex random", case, M, K, N, ta, tb, flush=True)
        A = rng.integers(-9, 10, (M, K)).astype(np.float64)
        B = rng.integers(-9, 10, (K, N)).astype(np.float64)
        X = np.ascontiguousarray(A.T) if ta else A
        Y = np.ascontiguousarray(B.T) if tb else B
        assert np.array_equal(dgemm_ex(X, Y, M, K, N, ta, tb), A @ B), (M, K, N, ta, tb)
