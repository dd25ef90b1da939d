"""The drop-in boundary on a GPU: buffer lifecycle, eshkol_gpu_matmul_f64 and
its environment-driven tier selection, eshkol_matmul_dispatch with its threshold
and fallback ladder, the batched entry, elementwise and transpose. Environment
variables are parsed once per process, so each configuration runs in a child
process that calls the library through the same ctypes binding."""
import ctypes as C
import os
import subprocess
import sys

import numpy as np
import pytest

import eshkol_amd as ea
import oracle
from eshkol_amd import synth
from conftest import ROOT
from gpu_util import normwise

pytestmark = pytest.mark.gpu

CHILD = r"""
import ctypes as C, os, sys
import numpy as np
sys.path.insert(0, %(root)r); sys.path.insert(0, os.path.join(%(root)r, "tests"))
import oracle, eshkol_amd as ea
from eshkol_amd import synth
from gpu_util import normwise, ulp_distance
rt = C.CDLL(oracle.HOSTRT_PATH, mode=C.RTLD_GLOBAL)
rt.oracle_hostrt_matmul_calls.restype = C.c_long
rt.oracle_hostrt_batch_calls.restype = C.c_long
lib = ea.load()
%(body)s
print("CHILD-OK")
"""


def run_child(body, env=None):
    e = dict(os.environ)
    for k in list(e):
        if k.startswith("ESHKOL_"):
            del e[k]
    if env:
        e.update(env)
    r = subprocess.run([sys.executable, "-u", "-c", CHILD % {"root": ROOT, "body": body}],
                       capture_output=True, text=True, env=e, timeout=600)
    assert r.returncode == 0 and "CHILD-OK" in r.stdout, "stdout:\n%s\nstderr:\n%s" % (r.stdout, r.stderr)
    return r


def test_buffer_lifecycle(gpu):
    lib = ea.load()
    b = ea.EshkolGPUBuffer()
    assert lib.eshkol_gpu_get_backend() == ea.GPU_HIP and lib.eshkol_gpu_init() == 1
    assert lib.eshkol_gpu_supports_f64() == 1 and lib.eshkol_gpu_has_fp64() == 1
    assert lib.eshkol_gpu_backend_available(ea.GPU_HIP) == 1 and lib.eshkol_gpu_backend_available(ea.GPU_CUDA) == 0
    assert lib.eshkol_gpu_alloc(4096, ea.MEM_DEVICE, C.byref(b)) == 0
    assert b.host_ptr is None and b.device_ptr and b.mem_type == ea.MEM_DEVICE and b.backend == ea.GPU_HIP
    lib.eshkol_gpu_free(C.byref(b)); assert not b.device_ptr and b.size_bytes == 0
    assert lib.eshkol_gpu_alloc(4096, ea.MEM_UNIFIED, C.byref(b)) == 0
    assert b.host_ptr == b.device_ptr and b.host_ptr
    lib.eshkol_gpu_free(C.byref(b))
    assert lib.eshkol_gpu_alloc(4096, ea.MEM_HOST_PINNED, C.byref(b)) == 0
    assert b.host_ptr and b.device_ptr is None
    lib.eshkol_gpu_free(C.byref(b))
    assert lib.eshkol_gpu_alloc_aligned(1000, 256, ea.MEM_DEVICE, C.byref(b)) == 0 and b.size_bytes == 1024
    lib.eshkol_gpu_free(C.byref(b))
    # wrap: device copy, sync D2H lands in the caller's memory, free never frees it
    x = np.arange(1024.0); y = np.zeros(1024)
    bx, by = ea.EshkolGPUBuffer(), ea.EshkolGPUBuffer()
    assert lib.eshkol_gpu_wrap_host(x.ctypes.data, x.nbytes, C.byref(bx)) == 0 and (bx.flags & 1)
    assert lib.eshkol_gpu_wrap_host(y.ctypes.data, y.nbytes, C.byref(by)) == 0
    assert lib.eshkol_gpu_elementwise_f64(C.byref(bx), C.byref(bx), C.byref(by), 1024, 0) == 0   # y = x + x
    assert lib.eshkol_gpu_sync(C.byref(by), ea.SYNC_DEVICE_TO_HOST) == 0
    assert np.array_equal(y, 2 * x)
    assert lib.eshkol_gpu_elementwise_f64(C.byref(by), None, C.byref(by), 1024, 4) == 0          # y = -y
    lib.eshkol_gpu_free(C.byref(by))                       # copy-back on free
    assert np.array_equal(y, -2 * x)
    lib.eshkol_gpu_free(C.byref(bx)); assert x[5] == 5.0
    lib.eshkol_gpu_wait(None)


@pytest.mark.parametrize("nbytes", [(1 << 20) - 8, (1 << 20) + 8, (16 << 20), (16 << 20) + 24,
                                    5 * (16 << 20) + 4096 + 8, 9 * (16 << 20) - 8])
def test_wrapped_host_memory_round_trip_through_the_staging_ring(gpu, nbytes):
    """Uploads and downloads of caller-owned memory are staged through a ring of
    pinned chunks by several threads; every byte has to arrive, whatever the
    size is relative to a chunk, the ring, or a thread's share."""
    lib = ea.load()
    n = nbytes // 8
    x = synth.normal(90 + (nbytes % 97), (n,))
    y = np.full(n, np.nan)
    bx, by = ea.EshkolGPUBuffer(), ea.EshkolGPUBuffer()
    assert lib.eshkol_gpu_wrap_host(x.ctypes.data, x.nbytes, C.byref(bx)) == 0
    assert lib.eshkol_gpu_wrap_host(y.ctypes.data, y.nbytes, C.byref(by)) == 0
    assert lib.eshkol_gpu_elementwise_f64(C.byref(bx), None, C.byref(by), n, 4) == 0      # y = -x
    assert lib.eshkol_gpu_sync(C.byref(by), ea.SYNC_DEVICE_TO_HOST) == 0
    assert np.array_equal(y, -x)
    # host -> device of changed contents, then the copy-back on free
    y[:] = x * 2.0
    assert lib.eshkol_gpu_sync(C.byref(by), ea.SYNC_HOST_TO_DEVICE) == 0
    assert lib.eshkol_gpu_elementwise_f64(C.byref(by), None, C.byref(by), n, 4) == 0      # y = -y
    lib.eshkol_gpu_free(C.byref(by))
    assert np.array_equal(y, -2.0 * x)
    lib.eshkol_gpu_free(C.byref(bx))


def test_staged_copies_can_be_switched_off(gpu):
    run_child("""
assert lib.eshkol_gpu_init() == 1
n = (40 << 20) // 8
x = synth.normal(7, (n,)); y = np.zeros(n)
bx, by = ea.EshkolGPUBuffer(), ea.EshkolGPUBuffer()
assert lib.eshkol_gpu_wrap_host(x.ctypes.data, x.nbytes, C.byref(bx)) == 0
assert lib.eshkol_gpu_wrap_host(y.ctypes.data, y.nbytes, C.byref(by)) == 0
assert lib.eshkol_gpu_elementwise_f64(C.byref(bx), None, C.byref(by), n, 4) == 0
lib.eshkol_gpu_free(C.byref(by)); lib.eshkol_gpu_free(C.byref(bx))
assert np.array_equal(y, -x)
""", {"ESHKOL_GPU_COPY_THREADS": "0"})


def test_gpu_matmul_f64_on_device_buffers(gpu):
    lib = ea.load()
    M, K, N = 300, 200, 260
    A, B = synth.normal(1, (M, K)), synth.normal(2, (K, N))
    dA, dB, dC = ea.DeviceArray.from_host(A), ea.DeviceArray.from_host(B), ea.DeviceArray((M, N))
    assert lib.eshkol_gpu_matmul_f64(C.byref(dA.buf), C.byref(dB.buf), C.byref(dC.buf), M, K, N) == 0
    assert normwise(dC.download(), oracle.matmul_f64(A, B), A, B) <= 1e-14
    small = ea.DeviceArray((4, 4))
    assert lib.eshkol_gpu_matmul_f64(C.byref(dA.buf), C.byref(dB.buf), C.byref(small.buf), M, K, N) == -1
    host = ea.EshkolGPUBuffer()
    assert lib.eshkol_gpu_matmul_f64(C.byref(host), C.byref(dB.buf), C.byref(dC.buf), M, K, N) == -1
    # single precision entry
    Af, Bf = A.astype(np.float32), B.astype(np.float32)
    fa, fb, fc = ea.DeviceArray.from_host(Af), ea.DeviceArray.from_host(Bf), ea.DeviceArray((M, N), np.float32)
    assert lib.eshkol_gpu_matmul_f32(C.byref(fa.buf), C.byref(fb.buf), C.byref(fc.buf), M, K, N) == 0
    assert normwise(fc.download(), Af.astype(np.float64) @ Bf.astype(np.float64), Af, Bf) <= 1e-6


def test_elementwise_family_and_transpose(gpu):
    lib = ea.load()
    n = 5000
    a = synth.uniform(3, (n,), 0.1, 3.0); b = synth.uniform(4, (n,), 0.5, 2.0)
    da, db, do = ea.DeviceArray.from_host(a), ea.DeviceArray.from_host(b), ea.DeviceArray((n,))
    expect = [a + b, a - b, a * b, a / b, -a, np.abs(a), np.exp(a), np.log(a), np.sin(a), np.cos(a),
              np.tanh(a), np.maximum(a, 0), 1 / (1 + np.exp(-a)), np.sqrt(a), 1 / a]
    for op, want in enumerate(expect):
        bb = C.byref(db.buf) if op < 4 else None
        assert lib.eshkol_gpu_elementwise_f64(C.byref(da.buf), bb, C.byref(do.buf), n, op) == 0
        got = do.download()
        if op in (0, 1, 2, 3, 4, 5, 11, 13, 14):
            assert np.array_equal(got, want), op          # correctly rounded operations
        else:
            assert np.abs(got - want).max() <= 4e-16 * max(1.0, np.abs(want).max()), op
    assert lib.eshkol_gpu_elementwise_f64(C.byref(da.buf), None, C.byref(do.buf), n, 15) == -1
    X = synth.normal(5, (130, 70))
    dx, dt = ea.DeviceArray.from_host(X), ea.DeviceArray((70, 130))
    assert lib.eshkol_gpu_transpose_f64(C.byref(dx.buf), C.byref(dt.buf), 130, 70) == 0
    assert np.array_equal(dt.download(), X.T)
    # the operations left to the caller's CPU rules report failure
    assert lib.eshkol_gpu_reduce_f64(C.byref(da.buf), C.byref(do.buf), n, 0) == -1
    assert lib.eshkol_gpu_softmax_f64(C.byref(da.buf), C.byref(do.buf), 10, 500) == -1


def test_known_answers_of_the_reference_elementwise_and_transpose_tests(gpu):
    """tests/gpu/elementwise_correctness_test.esk and transpose_correctness_test.esk,
    through eshkol_gpu_elementwise_f64 / eshkol_gpu_transpose_f64."""
    lib = ea.load()

    def ew(op, a, b=None):
        a = np.ascontiguousarray(a, dtype=np.float64)
        da, do = ea.DeviceArray.from_host(a), ea.DeviceArray(a.shape)
        db = ea.DeviceArray.from_host(np.ascontiguousarray(b, dtype=np.float64)) if b is not None else None
        assert lib.eshkol_gpu_elementwise_f64(C.byref(da.buf), C.byref(db.buf) if db else None, C.byref(do.buf),
                                              a.size, op) == 0
        return do.download()

    def tr(a):
        a = np.ascontiguousarray(a, dtype=np.float64)
        da, dt = ea.DeviceArray.from_host(a), ea.DeviceArray(a.shape[::-1])
        assert lib.eshkol_gpu_transpose_f64(C.byref(da.buf), C.byref(dt.buf), a.shape[0], a.shape[1]) == 0
        return dt.download()

    A, B = np.array([[1., 2.], [3., 4.]]), np.array([[5., 6.], [7., 8.]])
    assert np.array_equal(ew(0, A, B), [[6, 8], [10, 12]])
    assert np.array_equal(ew(1, A, B), [[-4, -4], [-4, -4]])
    assert np.array_equal(ew(2, A, B), [[5, 12], [21, 32]])
    assert abs(ew(3, A, B)[0, 0] - 0.2) < 1e-10
    Cm, D = np.arange(1., 10.).reshape(3, 3), np.arange(9., 0., -1.).reshape(3, 3)
    cd = ew(0, Cm, D)
    assert np.all(cd == 10.0)
    assert np.array_equal(ew(2, cd, Cm), 10.0 * Cm)                       # chained
    assert np.array_equal(ew(0, A, B), ew(0, B, A))                      # commutative
    AB = np.array([[6., 8.], [10., 12.]])
    assert np.array_equal(ew(0, ew(0, A, B), AB), ew(0, A, ew(0, B, AB)))   # associative on these values
    A23 = np.array([[1., 2., 3.], [4., 5., 6.]])
    assert np.array_equal(tr(A23), [[1, 4], [2, 5], [3, 6]]) and np.array_equal(tr(tr(A23)), A23)
    assert np.array_equal(tr(A), [[1, 3], [2, 4]])
    M2 = np.arange(5000.).reshape(50, 100)
    M2T = tr(M2)
    assert (M2T[0, 0], M2T[1, 0], M2T[0, 1]) == (0.0, 1.0, 100.0) and abs(M2T.sum() - M2.sum()) < 1e-6


def test_differential_gate_workload_gpu_against_the_compiled_reference_cpu(gpu):
    """tests/gpu/gpu_correctness_gate.esk:22-76 with gpu_correctness_gate.sh:55,364-390:
    the gate's sin/cos workload through the GPU entry points and through the CPU
    matmul of the reference itself (compiled in place by the oracle's recipe), its
    RESULT values compared at the gate's relative tolerance 1e-4 (they agree to
    1e-13 and better)."""
    if not os.path.exists(oracle.REF_PATH):
        pytest.skip("the compiled reference is not in this tree")
    lib = ea.load()
    n = k = 512
    i = np.arange(n * k, dtype=np.float64)
    A = (1.0001 + np.sin(i * 0.001)).reshape(n, k)
    B = (1.0002 + np.cos(i * 0.0013)).reshape(k, n)
    old = lib.eshkol_gpu_get_threshold()
    lib.eshkol_gpu_set_threshold(1)
    try:
        Cg = ea.matmul_dispatch(A, B)
    finally:
        lib.eshkol_gpu_set_threshold(old)
    ref = C.CDLL(oracle.REF_PATH)
    dp = C.POINTER(C.c_double)
    ref.eshkol_matmul_f64.argtypes = [dp, dp, dp, C.c_uint64, C.c_uint64, C.c_uint64]
    Cc = np.empty((n, n))
    ref.eshkol_matmul_f64(A.ctypes.data_as(dp), B.ctypes.data_as(dp), Cc.ctypes.data_as(dp), n, k, n)
    da, db, do = ea.DeviceArray.from_host(A.ravel()), ea.DeviceArray.from_host(B.ravel()), ea.DeviceArray((n * k,))
    assert lib.eshkol_gpu_elementwise_f64(C.byref(da.buf), C.byref(db.buf), C.byref(do.buf), n * k, 0) == 0
    add = do.download()
    assert lib.eshkol_gpu_elementwise_f64(C.byref(da.buf), C.byref(db.buf), C.byref(do.buf), n * k, 2) == 0
    mul = do.download()
    dc, dt, dtt = ea.DeviceArray.from_host(Cg), ea.DeviceArray((n, n)), ea.DeviceArray((n, n))
    assert lib.eshkol_gpu_transpose_f64(C.byref(dc.buf), C.byref(dt.buf), n, n) == 0
    assert lib.eshkol_gpu_transpose_f64(C.byref(dt.buf), C.byref(dtt.buf), n, n) == 0
    Ctt = dtt.download()
    gpu_results = {"matmul-checksum": Cg.sum(), "matmul-c00": Cg[0, 0], "matmul-cmid": Cg[256, 256],
                   "matmul-clast": Cg[511, 511], "add-checksum": add.sum(), "mul-checksum": mul.sum(),
                   "transpose-roundtrip-c00": Ctt[0, 0], "transpose-roundtrip-clast": Ctt[511, 511]}
    cpu_results = {"matmul-checksum": Cc.sum(), "matmul-c00": Cc[0, 0], "matmul-cmid": Cc[256, 256],
                   "matmul-clast": Cc[511, 511], "add-checksum": (A + B).sum(), "mul-checksum": (A * B).sum(),
                   "transpose-roundtrip-c00": Cc[0, 0], "transpose-roundtrip-clast": Cc[511, 511]}
    for name, g in gpu_results.items():
        c = cpu_results[name]
        assert abs(g - c) / max(abs(c), 1e-300) <= 1e-4, name          # the gate's bar
        assert abs(g - c) / abs(c) <= 1e-13, name                      # what the two actually differ by


def test_dispatch_threshold_and_fallback_ladder(gpu):
    body = r"""
A = synth.normal(1, (200, 150)); B = synth.normal(2, (150, 300))
ref = oracle.matmul_f64(A, B)
# default threshold 100000: 200*300 = 60000 outputs stay on the runtime's CPU path
got = ea.matmul_dispatch(A, B)
assert rt.oracle_hostrt_matmul_calls() == 1 and np.array_equal(got, ref)
lib.eshkol_gpu_set_threshold(1)
got = ea.matmul_dispatch(A, B)
assert rt.oracle_hostrt_matmul_calls() == 1               # GPU took it
assert normwise(got, ref, A, B) <= 1e-14
assert lib.eshkol_gpu_should_use(1) == 1
# known answers through the dispatcher (tests/gpu/matmul_correctness_test.esk)
assert np.array_equal(ea.matmul_dispatch(np.array([[1., 2.], [3., 4.]]), np.array([[5., 6.], [7., 8.]])), [[19, 22], [43, 50]])
# tests/gpu/gpu_scale_correctness_test.esk:14-80
n = 4096
Cc = ea.matmul_dispatch(np.ones((n, n)), np.ones((n, n)))
assert np.all(Cc == 4096.0)
R = np.repeat(np.arange(1., n + 1)[:, None], n, axis=1)
Cc = ea.matmul_dispatch(R, np.ones((n, n)))
assert np.array_equal(Cc[:, 0], 4096.0 * np.arange(1, n + 1))
# f16 / bf16 dtype codes take the reduced tier
A = synth.normal(3, (256, 512), 1 / np.sqrt(512)); B = synth.normal(4, (512, 128), 1 / np.sqrt(512))
for d in (2, 3):
    got = ea.matmul_dispatch(A, B, d)
    Ar, Br = oracle.reduce_precision(A, d), oracle.reduce_precision(B, d)
    assert normwise(got, oracle.matmul_f64(Ar, Br), Ar, Br) <= 1e-2
    ok = np.abs(got) >= 2.0 ** -14                                   # away from the reference's f16 subnormal quirk
    assert np.array_equal(got[ok], oracle.reduce_precision(got, d)[ok])   # result carries the 16-bit rounding
assert rt.oracle_hostrt_matmul_calls() == 1
# batched entry: dtype 3 on the GPU, dtype 0 on the runtime's CPU path
a = synth.normal(5, (4, 96, 160), 0.1); b = synth.normal(6, (4, 160, 64), 0.1); c = np.empty((4, 96, 64))
lib.eshkol_batch_matmul_dispatch(a.ctypes.data, b.ctypes.data, c.ctypes.data, 4, 96, 160, 64, 3)
assert rt.oracle_hostrt_batch_calls() == 0
for i in range(4):
    Ar, Br = oracle.reduce_precision(a[i], 3), oracle.reduce_precision(b[i], 3)
    assert normwise(c[i], oracle.matmul_f64(Ar, Br), Ar, Br) <= 1e-2
# f64 batches: below the element threshold (4*96*64 outputs) the runtime's CPU loop, above it one strided launch
lib.eshkol_gpu_set_threshold(100000)
lib.eshkol_batch_matmul_dispatch(a.ctypes.data, b.ctypes.data, c.ctypes.data, 4, 96, 160, 64, 0)
assert rt.oracle_hostrt_batch_calls() == 1 and np.array_equal(c, oracle.batch_matmul_f64(a, b))
lib.eshkol_gpu_set_threshold(1)
c[:] = 0
lib.eshkol_batch_matmul_dispatch(a.ctypes.data, b.ctypes.data, c.ctypes.data, 4, 96, 160, 64, 0)
assert rt.oracle_hostrt_batch_calls() == 1
ref = oracle.batch_matmul_f64(a, b)
for i in range(4):
    assert normwise(c[i], ref[i], a[i], b[i]) <= 1e-14
"""
    r = run_child(body, {"ESHKOL_GPU_VERBOSE": "1"})
    assert "native fp64 MFMA" in r.stderr and "reduced tier" in r.stderr
    assert "batch matmul 4 x (96x160 @ 160x64) -> native fp64 MFMA, one strided launch" in r.stderr


PANELLED = r"""
assert lib.eshkol_gpu_init() == 1
lib.eshkol_gpu_set_threshold(1)
lib.hip_dgemm_set_tail_split(0)                  # a split last round reorders sums in the tiles it takes
M, K, N = 4100, 2048, 2056                       # 7 panels of 640 rows, the last one of 260
A = synth.normal(11, (M, K)); B = synth.normal(12, (K, N))
got = ea.matmul_dispatch(A, B, DTYPE)
dA, dB, dC = ea.DeviceArray.from_host(A), ea.DeviceArray.from_host(B), ea.DeviceArray((M, N))
if DTYPE:
    assert lib.hip_matmul_reduced_f64(dA.ptr, dB.ptr, dC.ptr, M, K, N, DTYPE, 1, None) == 0
else:
    assert lib.eshkol_gpu_matmul_f64(C.byref(dA.buf), C.byref(dB.buf), C.byref(dC.buf), M, K, N) == 0
lib.eshkol_gpu_wait(None)
whole = dC.download()
assert np.array_equal(got, whole)
# the same call again reuses the device copies' memory, and resident weights skip their upload
assert lib.eshkol_gpu_resident_pin(B.ctypes.data, B.nbytes) == 0
again = ea.matmul_dispatch(A, B, DTYPE)
assert np.array_equal(again, got)
lib.eshkol_gpu_resident_unpin(B.ctypes.data)
"""


@pytest.mark.parametrize("env,dtype,tier_line", [
    ({}, 0, "native fp64 MFMA"),
    ({"ESHKOL_HIP_F64_KERNEL": "ozaki-crt"}, 0, "Ozaki-II CRT exact"),
    ({"ESHKOL_OZAKI_FAST": "1"}, 0, "Ozaki-II FAST"),
    ({"ESHKOL_HIP_F64_KERNEL": "ozaki-int8"}, 0, "INT8-Ozaki T=6"),
    ({}, 3, "row panels"),
    ({}, 2, "row panels"),
    # two kernels meet this budget at nearly the same predicted cost: either is a right answer
    ({"ESHKOL_MATMUL_ACCURACY": "1e-6"}, 0, ("Ozaki-II FAST (9 moduli; accuracy-budget selector)",
                                             "INT8-Ozaki T=3 (accuracy-budget selector")),
], ids=["native", "crt", "crt-fast", "int8-slices", "bf16", "f16", "budget-1e-6"])
def test_host_memory_dispatch_in_row_panels(gpu, env, dtype, tier_line):
    """Large products on host memory go through the device in row panels of A
    and C so that copies and products overlap; the result is the one-piece one."""
    body = PANELLED.replace("DTYPE", str(dtype))
    e = dict(env); e["ESHKOL_GPU_VERBOSE"] = "1"
    r = run_child(body, e)
    lines = tier_line if isinstance(tier_line, tuple) else (tier_line,)
    assert "in 7 row panels of 640" in r.stderr and any(l in r.stderr for l in lines)
    e["ESHKOL_GPU_OVERLAP"] = "0"
    r = run_child(body, e)
    assert "row panels" not in r.stderr and (dtype or any(l in r.stderr for l in lines))


def test_concurrent_callers_serialise_on_the_library(gpu):
    """Calls from several host threads (the reference guards only initialisation,
    gpu_memory_cuda.cpp:111, 844; this library serialises every call on one mutex):
    large panelled products and small ones share the streams, the workspaces and
    the staging ring, and give the bits of the same calls made one at a time."""
    import threading
    lib = ea.load()
    assert lib.eshkol_gpu_init() == 1
    old = lib.eshkol_gpu_get_threshold()
    lib.eshkol_gpu_set_threshold(1)
    shapes = [(4100, 2048, 2056), (300, 200, 260), (1024, 1024, 1024), (4096, 2048, 2048), (64, 4096, 96), (700, 50, 900),
              (32, 2048, 4096), (1, 8192, 1024), (2048, 4096, 3)]
    ops = [(synth.normal(20 + i, (m, k)), synth.normal(40 + i, (k, n))) for i, (m, k, n) in enumerate(shapes)]
    want = [ea.matmul_dispatch(a, b) for a, b in ops]            # one at a time
    got = [[None] * len(ops) for _ in range(2)]
    errors = []

    def worker(rep, i):
        try:
            got[rep][i] = ea.matmul_dispatch(*ops[i])
        except Exception as e:                                     # pragma: no cover
            errors.append(e)

    try:
        threads = [threading.Thread(target=worker, args=(rep, i)) for rep in range(2) for i in range(len(ops))]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
    finally:
        lib.eshkol_gpu_set_threshold(old)
    assert not errors
    for rep in range(2):
        for i, (a, b) in enumerate(ops):
            assert np.array_equal(got[rep][i], want[i]), shapes[i]
            if rep == 0 and a.shape[0] * a.shape[1] * b.shape[1] <= 2 ** 28:
                assert normwise(want[i], oracle.matmul_f64(a, b), a, b) <= 1e-14


def test_calls_that_change_streams_wait_for_the_call_before(gpu):
    """The tier pipelines share one workspace (planes, partial sums), so a call on
    another stream than the call before it must not start before that call's work
    is over. Products queued alternately on two streams of the caller and on the
    library's, with no synchronisation of the caller's between them, give the bits
    of the same products made one at a time, and so does a call made after a
    stream it followed has been destroyed."""
    lib = ea.init(); hip = ea.hip_runtime()
    streams = [C.c_void_p(), C.c_void_p()]
    for s in streams:
        assert hip.hipStreamCreate(C.byref(s)) == 0
    own = C.c_void_p(lib.eshkol_hip_get_stream())
    shapes = [(1024, 1024, 1024), (768, 512, 640), (1536, 1024, 1280), (512, 2048, 512)]
    ops = [(ea.DeviceArray.from_host(synth.normal(60 + i, (m, k))), ea.DeviceArray.from_host(synth.normal(70 + i, (k, n))))
           for i, (m, k, n) in enumerate(shapes)]

    def product(kind, i, stream, out):
        m, k, n = shapes[i]
        a, b = ops[i]
        if kind == 0:
            return lib.hip_dgemm_f64(a.ptr, b.ptr, out.ptr, m, k, n, stream)
        if kind == 1:
            return lib.hip_matmul_ozaki_crt_f64(a.ptr, b.ptr, out.ptr, m, k, n, 16, 0, None, 0, stream)
        return lib.hip_matmul_ozaki_int8_f64(a.ptr, b.ptr, out.ptr, m, k, n, 4, stream)

    plan = [(kind, i) for kind in (1, 0, 2) for i in range(len(shapes))]
    want = []
    for kind, i in plan:                                   # one at a time on the library's stream
        out = ea.DeviceArray((shapes[i][0], shapes[i][2]))
        assert product(kind, i, own, out) == 0
        assert hip.hipDeviceSynchronize() == 0
        want.append(out.download()); out.free()
    outs = [ea.DeviceArray((shapes[i][0], shapes[i][2])) for _, i in plan]
    order = [streams[0], streams[1], own]
    for j, (kind, i) in enumerate(plan):                   # back to back, the stream changing every call
        assert product(kind, i, order[j % 3], outs[j]) == 0
    assert hip.hipDeviceSynchronize() == 0
    for j, (kind, i) in enumerate(plan):
        assert np.array_equal(outs[j].download(), want[j]), (kind, shapes[i])
    # a stream that is gone by the time the next call arrives
    assert product(1, 0, streams[1], outs[0]) == 0
    assert hip.hipStreamSynchronize(streams[1]) == 0 and hip.hipStreamDestroy(streams[1]) == 0
    assert product(1, 1, streams[0], outs[1]) == 0
    assert hip.hipStreamSynchronize(streams[0]) == 0
    assert np.array_equal(outs[0].download(), want[0]) and np.array_equal(outs[1].download(), want[1])
    assert hip.hipStreamDestroy(streams[0]) == 0
    assert product(0, 2, own, outs[6]) == 0 and hip.hipDeviceSynchronize() == 0
    assert np.array_equal(outs[6].download(), want[6])
    for o in outs:
        o.free()
    for a, b in ops:
        a.free(); b.free()


def test_batched_native_kernel(gpu):
    """hip_dgemm_f64_batched against the oracle's batch loop: even and odd shapes
    (the odd ones leave matrices of the batch off 16-byte boundaries), integer
    cases exact, a batch larger than one grid axis allows."""
    lib = ea.load()
    st = lib.eshkol_hip_get_stream()
    for (bt, M, K, N) in [(1, 64, 64, 64), (3, 17, 23, 11), (5, 33, 7, 9), (8, 128, 96, 160), (2, 300, 257, 129),
                          (16, 256, 256, 256)]:
        a, b = synth.normal(bt + M, (bt, M, K)), synth.normal(bt + N, (bt, K, N))
        da, db, dc = ea.DeviceArray.from_host(a), ea.DeviceArray.from_host(b), ea.DeviceArray((bt, M, N))
        assert lib.hip_dgemm_f64_batched(da.ptr, db.ptr, dc.ptr, bt, M, K, N, st) == 0
        ea.synchronize()
        got, ref = dc.download(), oracle.batch_matmul_f64(a, b)
        for i in range(bt):
            assert normwise(got[i], ref[i], a[i], b[i]) <= 1e-14, (bt, M, K, N, i)
    rng = np.random.default_rng(9)
    bt, M, K, N = 70000, 4, 6, 2
    a = rng.integers(-5, 6, (bt, M, K)).astype(np.float64)
    b = rng.integers(-5, 6, (bt, K, N)).astype(np.float64)
    da, db, dc = ea.DeviceArray.from_host(a), ea.DeviceArray.from_host(b), ea.DeviceArray((bt, M, N))
    assert lib.hip_dgemm_f64_batched(da.ptr, db.ptr, dc.ptr, bt, M, K, N, st) == 0
    ea.synchronize()
    assert np.array_equal(dc.download(), np.einsum("bmk,bkn->bmn", a, b))
    assert lib.hip_dgemm_f64_batched(da.ptr, db.ptr, dc.ptr, 0, M, K, N, st) == -1


def test_batched_dispatch_of_16_bit_tensors_is_one_launch(gpu):
    """eshkol_batch_matmul_dispatch with dtype 2 / 3 (gpu_memory_cuda.cpp:736-784: one strided
    launch for all experts): many small experts from host memory, against the reference's reduced
    statement per matrix, with the dispatcher's own log line as evidence of the single launch."""
    body = r"""
batch, M, K, N = 64, 128, 256, 128
a = synth.normal(1, (batch, M, K), 1.0 / np.sqrt(K)); b = synth.normal(2, (batch, K, N), 1.0 / np.sqrt(K))
for dtype in (2, 3):
    ar, br = oracle.reduce_precision(a, dtype), oracle.reduce_precision(b, dtype)
    c = np.full((batch, M, N), np.nan)
    lib.eshkol_batch_matmul_dispatch(ar.ctypes.data, br.ctypes.data, c.ctypes.data, batch, M, K, N, dtype)
    for i in range(batch):
        assert normwise(c[i], oracle.matmul_f64(ar[i], br[i]), ar[i], br[i]) <= 1e-2, (dtype, i)
assert rt.oracle_hostrt_batch_calls() == 0
"""
    r = run_child(body, {"ESHKOL_GPU_VERBOSE": "1"})
    assert r.stderr.count("reduced tier (f16 in, fp32 accumulate), one strided launch") == 1
    assert r.stderr.count("reduced tier (bf16 in, fp32 accumulate), one strided launch") == 1


def test_batched_f64_products_follow_the_tier_selection(gpu):
    """A batch of f64 products that an override (or the accuracy budget) sends to an Ozaki tier
    takes that tier matrix by matrix: the same bits as dispatching each product on its own.
    Products too small for the tier stay on the one strided native launch."""
    body = r"""
lib.eshkol_gpu_set_threshold(1)
batch, n = 3, 512
a = synth.wide_range(1, (batch, n, n)); b = synth.wide_range(2, (batch, n, n))
c = np.full((batch, n, n), np.nan)
lib.eshkol_batch_matmul_dispatch(a.ctypes.data, b.ctypes.data, c.ctypes.data, batch, n, n, n, 0)
for i in range(batch):
    assert np.array_equal(c[i], ea.matmul_dispatch(a[i], b[i])), i
    assert ulp_distance(c[i], oracle.matmul_ozaki_crt(a[i], b[i])).max() <= 2
m = 96
cs = np.full((batch, m, m), np.nan)
sa, sb = np.ascontiguousarray(a[:, :m, :m]), np.ascontiguousarray(b[:, :m, :m])
lib.eshkol_batch_matmul_dispatch(sa.ctypes.data, sb.ctypes.data, cs.ctypes.data, batch, m, m, m, 0)
for i in range(batch):
    assert normwise(cs[i], oracle.matmul_f64(sa[i], sb[i]), sa[i], sb[i]) <= 1e-14
assert rt.oracle_hostrt_batch_calls() == 0
"""
    r = run_child(body, {"ESHKOL_HIP_F64_KERNEL": "ozaki-crt", "ESHKOL_GPU_VERBOSE": "1"})
    assert r.stderr.count("tier chosen per product, 3 launches of it") == 1
    assert r.stderr.count("native fp64 MFMA, one strided launch") == 1
    assert r.stderr.count("[GPU] Ozaki-II: N=16") == 1 + 3          # one marker for the batch, one per single dispatch


def test_resident_tensors_skip_the_upload(gpu):
    body = r"""
lib.eshkol_gpu_set_threshold(1)
W = synth.normal(1, (300, 200)); X = synth.normal(2, (150, 300))
assert lib.eshkol_gpu_resident_bytes() == 0
assert lib.eshkol_gpu_resident_pin(W.ctypes.data, W.nbytes) == 0
assert lib.eshkol_gpu_resident_bytes() == W.nbytes
ref = oracle.matmul_f64(X, W)
assert normwise(ea.matmul_dispatch(X, W), ref, X, W) <= 1e-14
# the device copy is what the product reads: a host change is invisible until refresh
keep = W.copy()
W[:] = 0.0
assert normwise(ea.matmul_dispatch(X, W), ref, X, keep) <= 1e-14
assert lib.eshkol_gpu_resident_refresh(W.ctypes.data) == 0
assert np.all(ea.matmul_dispatch(X, W) == 0.0)
W[:] = keep
assert lib.eshkol_gpu_resident_pin(W.ctypes.data, W.nbytes) == 0          # pin again = upload again
assert normwise(ea.matmul_dispatch(X, W), ref, X, W) <= 1e-14
# as the first operand too, and in the batched entry
assert normwise(ea.matmul_dispatch(W.T.copy(), X.T.copy()), ref.T, X, W) <= 1e-14
lib.eshkol_gpu_resident_unpin(W.ctypes.data)
assert lib.eshkol_gpu_resident_bytes() == 0 and lib.eshkol_gpu_resident_refresh(W.ctypes.data) == -1
W[:] = 1.0
assert np.array_equal(ea.matmul_dispatch(np.ones((150, 300)), W), np.full((150, 200), 300.0))
assert rt.oracle_hostrt_matmul_calls() == 0
# staging buffers are reused: many calls, no growth in device memory in use
free0, total = C.c_size_t(), C.c_size_t()
ea.hip_runtime().hipMemGetInfo(C.byref(free0), C.byref(total))
for _ in range(20):
    ea.matmul_dispatch(X, W)
free1 = C.c_size_t()
ea.hip_runtime().hipMemGetInfo(C.byref(free1), C.byref(total))
assert free0.value - free1.value <= (8 << 20)
lib.eshkol_gpu_shutdown()
"""
    run_child(body)


def test_resident_weights_keep_their_residue_planes(gpu):
    """A pinned weight matrix used as the second operand of the exact tier is split once:
    later products (fresh activations) reuse its planes and give the bits of the unpinned
    path; eshkol_gpu_resident_refresh drops them, so changed weights are split again."""
    body = r"""
M, K, N = 1024, 1024, 1536
W = synth.xavier_uniform(5, K, N)
want = {}
for seed in (1, 2):
    X = synth.normal(seed, (M, K))
    want[seed] = ea.matmul_dispatch(X, W)                       # nothing pinned: W is split on every call
    assert np.array_equal(want[seed], oracle.matmul_ozaki_crt(X, W))
assert lib.eshkol_gpu_resident_pin(W.ctypes.data, W.nbytes) == 0
for rep in range(2):
    for seed in (1, 2):
        assert np.array_equal(ea.matmul_dispatch(synth.normal(seed, (M, K)), W), want[seed])
W[17, :] *= 3.0                                                 # the host tensor changes ...
assert lib.eshkol_gpu_resident_refresh(W.ctypes.data) == 0      # ... and the runtime says so
X = synth.normal(1, (M, K))
assert np.array_equal(ea.matmul_dispatch(X, W), oracle.matmul_ozaki_crt(X, W))
lib.eshkol_gpu_resident_unpin(W.ctypes.data)
assert np.array_equal(ea.matmul_dispatch(X, W), oracle.matmul_ozaki_crt(X, W))
"""
    r = run_child(body, {"ESHKOL_HIP_F64_KERNEL": "ozaki-crt", "ESHKOL_GPU_THRESHOLD": "1", "ESHKOL_GPU_VERBOSE": "1"})
    assert r.stderr.count("residue planes of the exact tier prepared") == 2      # once after pin, once after refresh


def test_resident_planes_follow_the_plane_layout_and_the_byte_cap(gpu):
    """Row-major planes (512 rows: 64 tiles, and k too short for the kernel that would take
    interleaved planes on so few) are made again, interleaved, when a product wants
    interleaved ones (1024 rows: 128 tiles), with a line in the verbose log, instead of staying
    in memory unused while B is split on every call; interleaved planes then serve every row
    count that follows (512 again, 700). ESHKOL_GPU_PREPARED_BYTES
    bounds what they may take (0: none). Results are the unpinned path's either way."""
    body = r"""
K, N = 512, 512
W = synth.xavier_uniform(5, K, N)
assert lib.eshkol_gpu_resident_pin(W.ctypes.data, W.nbytes) == 0
for M in (512, 1024, 1024, 512, 700):
    X = synth.normal(M, (M, K))
    assert np.array_equal(ea.matmul_dispatch(X, W), oracle.matmul_ozaki_crt(X, W)), M
lib.eshkol_gpu_resident_unpin(W.ctypes.data)
"""
    env = {"ESHKOL_HIP_F64_KERNEL": "ozaki-crt", "ESHKOL_GPU_THRESHOLD": "1", "ESHKOL_GPU_VERBOSE": "1"}
    r = run_child(body, env)
    assert r.stderr.count("residue planes of the exact tier prepared") == 2
    assert r.stderr.count("this product wants the other: preparing them again") == 1
    r = run_child(body, dict(env, ESHKOL_GPU_PREPARED_BYTES="0"))
    assert "residue planes of the exact tier prepared" not in r.stderr
    assert r.stderr.count("would exceed ESHKOL_GPU_PREPARED_BYTES=0") == 1       # said once, then remembered


def test_shutdown_releases_what_the_tiers_keep_and_a_new_init_starts_over(gpu):
    """eshkol_gpu_shutdown() frees the tiers' own tables, the scan's mailbox, stream and event
    besides workspace, staging and resident memory; after eshkol_gpu_init() every tier works
    again and gives the same bits."""
    body = r"""
n = 1024
A = synth.wide_range(1, (n, n), -6, 6); B = synth.wide_range(2, (n, n), -6, 6)
def all_tiers():
    st = lib.eshkol_hip_get_stream()
    dA, dB, dC = ea.DeviceArray.from_host(A), ea.DeviceArray.from_host(B), ea.DeviceArray((n, n))
    out = []
    for call in (lambda: lib.hip_matmul_ozaki_crt_f64(dA.ptr, dB.ptr, dC.ptr, n, n, n, 16, 0, None, 0, st),
                 lambda: lib.hip_matmul_ozaki_fast_f64(dA.ptr, dB.ptr, dC.ptr, n, n, n, 11, st),
                 lambda: lib.hip_matmul_ozaki_int8_f64(dA.ptr, dB.ptr, dC.ptr, n, n, n, 4, st),
                 lambda: lib.hip_matmul_reduced_f64(dA.ptr, dB.ptr, dC.ptr, n, n, n, 3, 0, st)):
        assert call() == 0
        ea.synchronize()
        out.append(dC.download())
    for d in (dA, dB, dC):
        d.free()
    return out
assert lib.eshkol_gpu_init() == 1
hip = ea.hip_runtime()
def free_bytes():
    f, t = C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(f), C.byref(t)) == 0
    return f.value
base = free_bytes()
first = all_tiers()
assert np.array_equal(first[0], oracle.matmul_ozaki_crt(A, B))
held = base - free_bytes()
lib.eshkol_gpu_shutdown()
assert lib.eshkol_gpu_get_backend() == ea.GPU_NONE
after_first = free_bytes()
released = held - (base - after_first)
print("HELD %d RELEASED %d" % (held, released))
# the workspace (64 MiB of planes and products at this size) and the tiers' tables are gone; what the HIP
# runtime itself took on the first launches stays with it
assert held > (48 << 20) and released >= held - (16 << 20)
assert lib.eshkol_gpu_init() == 1
again = all_tiers()
for a, b in zip(first, again):
    assert np.array_equal(a, b)
lib.eshkol_gpu_shutdown()
assert after_first - free_bytes() <= (2 << 20)                   # a second cycle leaves nothing behind
"""
    run_child(body)


def test_threshold_env_forces_gpu(gpu):
    body = r"""
A = synth.normal(1, (8, 8)); B = np.eye(8)
got = ea.matmul_dispatch(A, B)                 # tests/gpu/cuda_host_sync_regression_test.esk:14-39
assert np.array_equal(got, A) and rt.oracle_hostrt_matmul_calls() == 0
"""
    r = run_child(body, {"ESHKOL_GPU_THRESHOLD": "1", "ESHKOL_GPU_VERBOSE": "1"})
    assert "[GPU] matmul 8x8 @ 8x8 -> native fp64 MFMA" in r.stderr


def test_tier_override_crt(gpu):
    body = r"""
n = 512
A = synth.wide_range(1, (n, n)); B = synth.wide_range(2, (n, n))
got = ea.matmul_dispatch(A, B)
assert ulp_distance(got, oracle.matmul_ozaki_crt(A, B)).max() <= 2
small = ea.matmul_dispatch(A[:256, :256], B[:256, :256])     # below 512: native tier
assert normwise(small, oracle.matmul_f64(A[:256, :256], B[:256, :256]), A[:256, :256], B[:256, :256]) <= 1e-14
"""
    for env in ({"ESHKOL_HIP_F64_KERNEL": "ozaki-crt"}, {"ESHKOL_SF64_KERNEL": "ozaki"}):
        env = dict(env, ESHKOL_GPU_THRESHOLD="1", ESHKOL_GPU_VERBOSE="1", ESHKOL_OZAKI_PROFILE="1")
        r = run_child(body, env)
        assert r.stderr.count("[GPU] Ozaki-II: N=16, log2(P)=125.4") == 1      # one marker per dispatch
        assert "Ozaki-II CRT exact" in r.stderr and "[OZAKI_PROFILE] exact M=512" in r.stderr
        assert "native fp64 MFMA" in r.stderr
    r = run_child(body, {"ESHKOL_HIP_F64_KERNEL": "ozaki-crt", "ESHKOL_GPU_THRESHOLD": "1",
                         "ESHKOL_OZAKI_NUM_MODULI": "32"})
    assert "out of range" in r.stderr                                          # loud clamp, still correct


def test_tier_override_fast_crt(gpu):
    """ESHKOL_OZAKI_FAST / ESHKOL_SF64_KERNEL=ozaki-fast (gpu_memory.mm:1319-1343): the reduced-precision
    CRT tier first, the exact tier behind it when it declines; the moduli knob clamps loudly."""
    body = r"""
n = 512
A = synth.normal(1, (n, n)); B = synth.normal(2, (n, n))
got = ea.matmul_dispatch(A, B)
n_mod = int(os.environ.get("EXPECT_MODULI", "11"))
rc, want = oracle.matmul_ozaki_fast(A, B, n_mod)
ref = A @ B
# the oracle reconstructs in float pairs (2^-45 of P), the device in fp64: with 16 moduli P outgrows
# the products and the float pairs lose more than the 11-modulus tier does
assert rc == 0 and np.abs(got - want).max() <= (1e-9 if n_mod == 11 else 2e-8) * np.abs(ref).max()
assert np.abs(got - ref).max() <= 5e-8 * np.abs(ref).max()
bad = A.copy(); bad[3, 3] = np.inf                      # the fast tier declines, the exact tier declines, native answers
out = ea.matmul_dispatch(bad, B)
assert np.isinf(out[3]).any() or np.isnan(out[3]).any()
"""
    for env in ({"ESHKOL_OZAKI_FAST": "1"}, {"ESHKOL_SF64_KERNEL": "ozaki-fast"}, {"ESHKOL_HIP_F64_KERNEL": "ozaki-fast"}):
        env = dict(env, ESHKOL_GPU_THRESHOLD="1", ESHKOL_GPU_VERBOSE="1", ESHKOL_OZAKI_PROFILE="1")
        r = run_child(body, env)
        assert "[GPU] Ozaki-II FAST tier ENABLED: N=11 moduli" in r.stderr
        assert "[GPU] Ozaki-II FAST: n_mod=11 E=" in r.stderr and "[OZAKI_PROFILE] fast M=512" in r.stderr
        assert "[GPU] Ozaki-II FAST dispatch returned -1; falling back to exact tier" in r.stderr
    r = run_child(body, {"ESHKOL_OZAKI_FAST": "1", "ESHKOL_OZAKI_FAST_MODULI": "40", "EXPECT_MODULI": "16",
                         "ESHKOL_GPU_THRESHOLD": "1"})
    assert "ESHKOL_OZAKI_FAST_MODULI=40 out of range [2,16]; clamping to 16" in r.stderr
    r = run_child("A = synth.normal(1, (512, 512)); ea.matmul_dispatch(A, A)",
                  {"ESHKOL_OZAKI_FAST": "0", "ESHKOL_GPU_THRESHOLD": "1", "ESHKOL_GPU_VERBOSE": "1"})
    assert "FAST" not in r.stderr and "native fp64 MFMA" in r.stderr           # "0" leaves it off


GATE = r"""
import re
TOL = float(os.environ["GATE_TOL"])
assert lib.eshkol_gpu_init() == 1
fails = 0
for regime in range(4):
    for n in (512, 1024, 2048, 4096):
        i = np.arange(n * n, dtype=np.float64)
        A = [(i % 7) - 3, 1.0 + 0.5 * (i % 7), np.pi * (1.0 + (i % 11)), 2.0 ** ((i % 20) - 10) * (1.0 + 0.1 * (i % 3))][regime].reshape(n, n)
        B = [(i % 5) - 2, 0.5 + 0.25 * (i % 5), np.e * ((i % 9) - 4.0), 2.0 ** ((i % 18) - 9) * (1.0 + 0.1 * (i % 4))][regime].reshape(n, n)
        Cd = ea.matmul_dispatch(A, B)
        worst = 0.0
        for pr in range(5):
            for pc in range(5):
                ii, jj = (pr * (n - 1)) // 4, (pc * (n - 1)) // 4
                ref = 0.0
                for a, b in zip(A[ii].tolist(), B[:, jj].tolist()):          # the probe's own k-ascending f64 sum
                    ref += a * b
                denom = abs(ref) if abs(ref) > 1e-9 else 1.0
                worst = max(worst, abs(Cd[ii, jj] - ref) / denom)
        print("REGIME=%d N=%d MAXREL=%g VERDICT=%s" % (regime, n, worst, "PASS" if worst < TOL else "FAIL"))
        fails += worst >= TOL
print("SUMMARY total_fail=%d" % fails)
assert fails == 0
"""


@pytest.mark.parametrize("kernel,tol", [("ozaki", "1e-9"), ("ozaki-fast", "1e-7")], ids=["exact", "fast"])
def test_reference_gates_for_the_ozaki_tiers_through_the_dispatcher(gpu, kernel, tol):
    """tests/gpu/ozaki_correctness_test.esk + ozaki_correctness_gate.sh:79-136 and
    tests/gpu/ozaki_fast_test.esk + ozaki_fast_gate.sh: four fill regimes at
    N = 512 ... 4096, a 5 x 5 grid of probes against a plain f64 sum, the gates'
    own tolerance and denominator; and what the gates read off stderr: one
    dispatch marker per product and no other Ozaki-II line for the exact tier
    (sixteen products, also at 4096 where the dispatcher works in row panels), the
    FAST marker and no fall-back for the reduced-precision tier."""
    r = run_child(GATE, {"ESHKOL_SF64_KERNEL": kernel, "ESHKOL_GPU_THRESHOLD": "1", "ESHKOL_GPU_VERBOSE": "1",
                         "GATE_TOL": tol})
    assert "SUMMARY total_fail=0" in r.stdout and "VERDICT=FAIL" not in r.stdout
    lines = r.stderr.splitlines()
    import re
    if kernel == "ozaki":
        pat = re.compile(r"^\[GPU\] Ozaki-II: N=[0-9]+( \(adaptive\))?, log2\(P\)=")
        assert sum(1 for l in lines if pat.match(l)) == 16
        assert not [l for l in lines if l.startswith("[GPU] Ozaki-II:") and not pat.match(l)]      # the gate's poison guard
    else:
        assert sum(1 for l in lines if l.startswith("[GPU] Ozaki-II FAST: n_mod=11")) == 16
        assert "falling back to exact tier" not in r.stderr


def test_tier_override_int8_and_budget_selector(gpu):
    body = r"""
n = 1024
A = synth.normal(1, (n, n)); B = synth.normal(2, (n, n))
T = int(os.environ.get("EXPECT_T", "6"))
got = ea.matmul_dispatch(A, B)
assert ulp_distance(got, oracle.matmul_ozaki_int8(A, B, T)).max() <= 2
"""
    r = run_child(body, {"ESHKOL_CUDA_F64_KERNEL": "ozaki-int8", "ESHKOL_GPU_THRESHOLD": "1", "ESHKOL_GPU_VERBOSE": "1"})
    assert "INT8-Ozaki T=6" in r.stderr
    r = run_child(body, {"ESHKOL_HIP_F64_KERNEL": "ozaki-int8", "ESHKOL_OZAKI_CUDA_T": "4", "EXPECT_T": "4",
                         "ESHKOL_GPU_THRESHOLD": "1", "ESHKOL_GPU_VERBOSE": "1"})
    assert "INT8-Ozaki T=4" in r.stderr
    r = run_child(body, {"ESHKOL_CUDA_F64_KERNEL": "ozaki-int8", "ESHKOL_OZAKI_CUDA_T": "99",
                         "ESHKOL_GPU_THRESHOLD": "1"})
    assert "out of range" in r.stderr
    # accuracy budget: a loose budget picks a small T, a strict one stays native
    body2 = r"""
n = 4096
A = synth.normal(1, (n, n)); B = synth.normal(2, (n, n))
got = ea.matmul_dispatch(A, B)
rows = list(range(0, n, 587))
ref = A[rows].astype(np.longdouble) @ B.astype(np.longdouble)
err = normwise(got[rows], ref, A[rows], B)
assert err <= float(os.environ["EXPECT_ERR"]), err
"""
    r = run_child(body2, {"ESHKOL_MATMUL_ACCURACY": "fast", "EXPECT_ERR": "1e-3", "ESHKOL_GPU_THRESHOLD": "1",
                          "ESHKOL_GPU_VERBOSE": "1"})
    assert "INT8-Ozaki T=1 (accuracy-budget selector" in r.stderr
    # the names exact / full are the reference's strictest request: native fp64, never an Ozaki tier ...
    for name in ("exact", "full"):
        r = run_child(body2, {"ESHKOL_MATMUL_ACCURACY": name, "EXPECT_ERR": "1e-15", "ESHKOL_GPU_THRESHOLD": "1",
                              "ESHKOL_GPU_VERBOSE": "1"})
        assert "native fp64 MFMA (budget met cheapest by native fp64)" in r.stderr and "Ozaki" not in r.stderr
    # ... a numeric budget the exact tier's normwise bound meets (sqrt(K) 2^-51 = 2.85e-14 at K = 4096) is met
    # cheapest by that tier ...
    for budget in ("1e-13", "3e-14"):
        r = run_child(body2, {"ESHKOL_MATMUL_ACCURACY": budget, "EXPECT_ERR": budget, "ESHKOL_GPU_THRESHOLD": "1",
                              "ESHKOL_GPU_VERBOSE": "1"})
        assert "Ozaki-II CRT exact (accuracy-budget selector), aligned weights" in r.stderr
    # ... and a tighter one stays native like the names do, although the tier measures 1e-17 on such operands:
    # an entry far below its row's largest keeps its low bits there. Row 0 of A carries one entry of 2^60
    # that meets a zero row of B, so the row's result is made of the small entries alone; the exact tier
    # would cut them at 2^8.
    wide = r"""
n = 4096
A = synth.normal(1, (n, n)); B = synth.normal(2, (n, n))
A[0, 0] = 2.0 ** 60; B[0, :] = 0.0
got = ea.matmul_dispatch(A, B)
ref = A[:1].astype(np.longdouble) @ B.astype(np.longdouble)
rel = float(np.max(np.abs(got[0] - ref[0]) / (np.abs(A[0, 1:]) @ np.abs(B[1:]))))
print("ROW0 %.3e" % rel)
assert rel <= 1e-14, rel
"""
    r = run_child(wide, {"ESHKOL_MATMUL_ACCURACY": "1e-15", "ESHKOL_GPU_THRESHOLD": "1", "ESHKOL_GPU_VERBOSE": "1"})
    assert "native fp64 MFMA (budget met cheapest by native fp64)" in r.stderr and "Ozaki" not in r.stderr
    # the override by name keeps the reference's weights (and its error on such operands) unless told otherwise
    r = run_child(body2, {"ESHKOL_HIP_F64_KERNEL": "ozaki-crt", "EXPECT_ERR": "1e-9", "ESHKOL_GPU_THRESHOLD": "1",
                          "ESHKOL_GPU_VERBOSE": "1"})
    assert "Ozaki-II CRT exact (" in r.stderr and "aligned weights" not in r.stderr
    r = run_child(body2, {"ESHKOL_HIP_F64_KERNEL": "ozaki-crt", "ESHKOL_OZAKI_CRT_WEIGHTS": "aligned", "EXPECT_ERR": "1e-15",
                          "ESHKOL_GPU_THRESHOLD": "1", "ESHKOL_GPU_VERBOSE": "1"})
    assert "aligned weights" in r.stderr
    # ... a middling one by the reduced-precision CRT tier with just enough moduli ...
    r = run_child(body2, {"ESHKOL_MATMUL_ACCURACY": "1e-10", "EXPECT_ERR": "1e-10", "ESHKOL_GPU_THRESHOLD": "1",
                          "ESHKOL_GPU_VERBOSE": "1"})
    assert "Ozaki-II FAST (" in r.stderr and "accuracy-budget selector)" in r.stderr
    # ... and with the exact tier cut down to fewer moduli (no longer exact) it is not a candidate
    r = run_child(body2, {"ESHKOL_MATMUL_ACCURACY": "1e-15", "ESHKOL_OZAKI_NUM_MODULI": "12", "EXPECT_ERR": "1e-14",
                          "ESHKOL_GPU_THRESHOLD": "1", "ESHKOL_GPU_VERBOSE": "1"})
    assert "native fp64 MFMA (budget met cheapest by native fp64)" in r.stderr
    # small products stay native whatever the budget
    body3 = body2.replace("n = 4096", "n = 1024").replace("range(0, n, 587)", "range(0, n, 97)")
    r = run_child(body3, {"ESHKOL_MATMUL_ACCURACY": "1e-15", "EXPECT_ERR": "1e-14", "ESHKOL_GPU_THRESHOLD": "1",
                          "ESHKOL_GPU_VERBOSE": "1"})
    assert "native fp64 MFMA (budget met cheapest by native fp64)" in r.stderr


def test_precision_settings_keep_the_error_level_of_the_reference_tiers(gpu):
    """ESHKOL_GPU_PRECISION=fast is the reference's f32 tier (about 6e-8) and =ml its fp24
    tier (about 1e-5), gpu_memory.mm:174, 1346-1351. Here they are accuracy budgets of 1e-7
    and 1e-5 on f64 tensors: the error stays at that level (never the 4e-3 of a 16-bit
    product), and an explicit ESHKOL_MATMUL_ACCURACY wins."""
    body = r"""
n = 4096
A = synth.normal(1, (n, n)); B = synth.normal(2, (n, n))
got = ea.matmul_dispatch(A, B)
rows = list(range(0, n, 587))
ref = A[rows].astype(np.longdouble) @ B.astype(np.longdouble)
err = normwise(got[rows], ref, A[rows], B)
print("ERR %.3e" % err)
assert err <= float(os.environ["EXPECT_ERR"]), err
"""
    common = {"ESHKOL_GPU_THRESHOLD": "1", "ESHKOL_GPU_VERBOSE": "1"}
    r = run_child(body, dict(common, ESHKOL_GPU_PRECISION="fast", EXPECT_ERR="1e-7"))
    assert "accuracy-budget selector" in r.stderr and "reduced tier" not in r.stderr
    r = run_child(body, dict(common, ESHKOL_GPU_PRECISION="ml", EXPECT_ERR="1e-5"))
    assert "accuracy-budget selector" in r.stderr and "reduced tier" not in r.stderr
    r = run_child(body, dict(common, ESHKOL_GPU_PRECISION="high", EXPECT_ERR="1e-15"))
    assert "native fp64 MFMA (default)" in r.stderr
    r = run_child(body, dict(common, ESHKOL_GPU_PRECISION="ml", ESHKOL_MATMUL_ACCURACY="1e-13", EXPECT_ERR="1e-13"))
    assert "Ozaki-II CRT exact (accuracy-budget selector)" in r.stderr
    # small products: native fp64 whatever the setting
    small = body.replace("n = 4096", "n = 600").replace("range(0, n, 587)", "range(0, n, 97)")
    r = run_child(small, dict(common, ESHKOL_GPU_PRECISION="fast", EXPECT_ERR="1e-15"))
    assert "native fp64 MFMA" in r.stderr


def test_cut_down_exact_tier_is_not_multiplied_in_row_panels(gpu):
    """With fewer than sixteen moduli (or the adaptive count) the exact tier's exponent E
    depends on all rows of A together, so the host-memory dispatcher must not cut A into row
    panels: the result has to be the one-piece result, which is the oracle's bit for bit."""
    body = r"""
M, K, N = 8192 + 512, 1536, 512                          # A and C together above the panel threshold
A = synth.wide_range(5, (M, K), -6, 6); B = synth.wide_range(6, (K, N), -6, 6)
got = ea.matmul_dispatch(A, B)
rows = [0, 1, 777, 4095, 4096, 8191, 8192, M - 1]
want = oracle.matmul_ozaki_crt(A, B, num_moduli=12)
assert np.array_equal(got, want), int((got != want).sum())
"""
    r = run_child(body, {"ESHKOL_HIP_F64_KERNEL": "ozaki-crt", "ESHKOL_OZAKI_NUM_MODULI": "12",
                         "ESHKOL_GPU_THRESHOLD": "1", "ESHKOL_GPU_VERBOSE": "1"})
    assert "row panels" not in r.stderr and "Ozaki-II CRT exact" in r.stderr
    # sixteen moduli: E is 52 whatever the data, panels are used and the bits are still the oracle's
    body16 = body.replace("num_moduli=12", "num_moduli=16")
    r = run_child(body16, {"ESHKOL_HIP_F64_KERNEL": "ozaki-crt", "ESHKOL_GPU_THRESHOLD": "1", "ESHKOL_GPU_VERBOSE": "1"})
    assert "row panels" in r.stderr


def test_device_tanh_accuracy(gpu):
    """The fused epilogues use the library's own fp64 tanh. Against a reference of twice
    the precision (numpy longdouble) it must stay within 2 ulp everywhere: dense samples of
    the whole range, tiny arguments (relative accuracy), the saturation edge, specials."""
    import eshkol_amd as ea
    from gpu_util import stream
    lib = ea.load()
    rng = np.random.default_rng(77)
    x = np.concatenate([
        rng.uniform(-20.0, 20.0, 400000), rng.uniform(-1.0, 1.0, 400000),
        np.ldexp(rng.uniform(0.5, 1.0, 200000), rng.integers(-60, 6, 200000)) * rng.choice([-1.0, 1.0], 200000),
        rng.uniform(18.5, 19.5, 1000), np.linspace(0.17, 0.18, 1001), np.linspace(0.34, 0.36, 1001),
        [0.0, -0.0, 1e-300, -1e-300, 5e-324, 2.0 ** -28, 2.0 ** -27, 19.1, 19.2, 40.0, 710.0, -710.0, 1e308,
         np.inf, -np.inf]])
    dx, dy = ea.DeviceArray.from_host(x), ea.DeviceArray((x.size,))
    assert lib.hip_elementwise_f64(dx.ptr, None, dy.ptr, x.size, 10, stream()) == 0
    ea.synchronize()
    got = dy.download()
    want_ld = np.tanh(x.astype(np.longdouble))
    want = want_ld.astype(np.float64)
    err_ulp = np.abs((got.astype(np.longdouble) - want_ld) / np.spacing(np.maximum(np.abs(want), 5e-324)).astype(np.longdouble))
    assert err_ulp.max() <= 2.0, (err_ulp.max(), x[np.argmax(err_ulp)])
    assert np.array_equal(np.signbit(got), np.signbit(x))
    out = ea.DeviceArray((1,))
    assert lib.hip_elementwise_f64(ea.DeviceArray.from_host(np.array([np.nan])).ptr, None, out.ptr, 1, 10, stream()) == 0
    ea.synchronize()
    assert np.isnan(out.download()[0])
