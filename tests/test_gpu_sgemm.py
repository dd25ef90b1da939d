"""hip_sgemm_f32 / eshkol_gpu_matmul_f32 (the reference's cublasSgemm call,
lib/backend/gpu/gpu_memory_cuda.cpp:658-665) on the fp32 matrix cores, against a float64
product of the same fp32 operands: 1e-6 in the norm the native tier is held to at 1e-14."""
import ctypes as C

import numpy as np
import pytest

import eshkol_amd as ea
from eshkol_amd import synth
from gpu_util import normwise, stream
from test_gpu_native_fp64 import SHAPES

pytestmark = pytest.mark.gpu


def sgemm(A, B):
    lib = ea.load()
    M, K = A.shape
    N = B.shape[1]
    dA, dB, dC = ea.DeviceArray.from_host(A), ea.DeviceArray.from_host(B), ea.DeviceArray((M, N), np.float32)
    assert lib.hip_sgemm_f32(dA.ptr, dB.ptr, dC.ptr, M, K, N, stream()) == 0
    ea.synchronize()
    return dC.download()


@pytest.mark.parametrize("M,K,N", SHAPES + [(2048, 2048, 2048), (1000, 1001, 1003), (4096, 64, 4096), (384, 4100, 260)])
def test_sgemm_against_float64_product_of_the_same_operands(gpu, M, K, N):
    print("case: sgemm %dx%dx%d" % (M, K, N), flush=True)
    A = synth.normal(M + 3 * K, (M, K)).astype(np.float32)
    B = synth.normal(N + 5 * K, (K, N)).astype(np.float32)
    got = sgemm(A, B)
    want = A.astype(np.float64) @ B.astype(np.float64)
    assert normwise(got.astype(np.float64), want, A.astype(np.float64), B.astype(np.float64)) <= 1e-6
    assert np.isfinite(got).all()


def test_sgemm_known_answers_and_integer_products_are_exact(gpu):
    """Small integers are exact in fp32 and so is every partial sum below 2^24: whatever order
    the matrix cores add in, the result is the integer product bit for bit (tile edges, a
    k-tail, odd pitches and an unaligned view included)."""
    a = np.array([[1, 2], [3, 4]], np.float32)
    b = np.array([[5, 6], [7, 8]], np.float32)
    assert np.array_equal(sgemm(a, b), np.array([[19, 22], [43, 50]], np.float32))
    rng = np.random.default_rng(3)
    for M, K, N in ((128, 32, 128), (256, 96, 384), (130, 70, 129), (257, 1000, 131), (512, 2048, 640)):
        A = rng.integers(-8, 9, (M, K)).astype(np.float32)
        B = rng.integers(-8, 9, (K, N)).astype(np.float32)
        assert np.array_equal(sgemm(A, B), (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32)), (M, K, N)
    ones = np.ones((640, 640), np.float32)
    assert np.all(sgemm(ones, ones) == 640.0)


def test_sgemm_rejects_bad_arguments(gpu):
    lib = ea.load()
    d = ea.DeviceArray((4,), np.float32)
    assert lib.hip_sgemm_f32(None, d.ptr, d.ptr, 2, 2, 2, stream()) == -1
    assert lib.hip_sgemm_f32(d.ptr, d.ptr, d.ptr, 0, 2, 2, stream()) == -1
