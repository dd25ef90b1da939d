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


def test_noalloc_rejects_sizes_beyond_its_scratch():
    lib = ea.init()
    limit = lib.hip_matmul_reduced_f64_noalloc_limit()
    assert limit == 32 << 20
    M = N = K = 4096                                    # 2 * 4096 * 4096 * 2 bytes = 64 MiB
    d = ea.DeviceArray((8,))                            # never touched: the size check comes first
    assert lib.hip_matmul_reduced_f64_noalloc(d.ptr, d.ptr, d.ptr, M, K, N, 3, 0, stream()) == -3
