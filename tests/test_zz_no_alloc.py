"""hip_matmul_reduced_f64_noalloc: the reduced tier with its 16-bit operand copies in a
static device array instead of the library workspace. Same kernels, so the result must equal
hip_matmul_reduced_f64's bit for bit; the second call is smaller than the first, so stale
contents of the shared array would show."""
import numpy as np
import pytest

import eshkol_amd as ea
from eshkol_amd import synth
from gpu_util import Operands, stream

pytestmark = pytest.mark.gpu


def both(A, B, dtype, round_output):
    lib = ea.init()
    ops = Operands(A, B)
    assert lib.hip_matmul_reduced_f64_noalloc(ops.dA.ptr, ops.dB.ptr, ops.dC.ptr, ops.M, ops.K, ops.N,
                                              dtype, round_output, stream()) == 0
    got = ops.result()
    assert lib.hip_matmul_reduced_f64(ops.dA.ptr, ops.dB.ptr, ops.dC.ptr, ops.M, ops.K, ops.N,
                                      dtype, round_output, stream()) == 0
    return got, ops.result()


def test_noalloc_equals_workspace_entry_point_twice_in_a_row():
    print("case: noalloc 700x900x520 bf16 then 130x77x260 f16", flush=True)
    A, B = synth.normal(11, (700, 900), 1.0), synth.normal(12, (900, 520), 1.0)
    got, want = both(A, B, 3, 0)
    assert np.array_equal(got, want)
    assert np.isfinite(got).all() and np.abs(got).max() > 1.0
    A2, B2 = synth.normal(13, (130, 77), 1.0), synth.normal(14, (77, 260), 1.0)
    got2, want2 = both(A2, B2, 2, 1)
    assert np.array_equal(got2, want2)
    ref = A2 @ B2
    assert np.abs(got2 - ref).max() <= 2e-2 * np.abs(ref).max() + 0.2


def test_noalloc_takes_no_device_memory_on_first_use_of_a_shape():
    """Shapes this process has not multiplied before, one per contraction kernel the entry point
    can reach (the direct kernel on interleaved operands, the small-tile kernel): the device's
    free memory is the same before and after, i.e. neither the call nor anything it sets up on
    first use (kernel attributes, the CU count) allocates. Results against the workspace entry
    point afterwards, which may allocate."""
    import ctypes as C
    lib = ea.init()
    hip = ea.hip_runtime()
    hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]

    def free_bytes():
        free, total = C.c_size_t(), C.c_size_t()
        assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
        return free.value

    cases = [((4096, 384, 4096), 3, 0), ((310, 205, 99), 2, 1)]
    held = []
    for (M, K, N), dtype, rnd in cases:
        print("case: noalloc first use %dx%dx%d dtype %d" % (M, K, N, dtype), flush=True)
        held.append((Operands(synth.normal(21, (M, K), 1.0), synth.normal(22, (K, N), 1.0)), dtype, rnd))
    ea.synchronize()
    before = free_bytes()
    got = []
    for ops, dtype, rnd in held:
        assert lib.hip_matmul_reduced_f64_noalloc(ops.dA.ptr, ops.dB.ptr, ops.dC.ptr, ops.M, ops.K, ops.N,
                                                  dtype, rnd, stream()) == 0
        ea.synchronize()
        assert free_bytes() == before
        got.append(ops.result())
    for (ops, dtype, rnd), g in zip(held, got):
        assert lib.hip_matmul_reduced_f64(ops.dA.ptr, ops.dB.ptr, ops.dC.ptr, ops.M, ops.K, ops.N,
                                          dtype, rnd, stream()) == 0
        assert np.array_equal(g, ops.result())


def test_noalloc_rejects_sizes_beyond_its_scratch():
    lib = ea.init()
    limit = lib.hip_matmul_reduced_f64_noalloc_limit()
    assert limit == 32 << 20
    M = N = K = 4096                                    # 2 * 4096 * 4096 * 2 bytes = 64 MiB
    d = ea.DeviceArray((8,))                            # never touched: the size check comes first
    assert lib.hip_matmul_reduced_f64_noalloc(d.ptr, d.ptr, d.ptr, M, K, N, 3, 0, stream()) == -3
