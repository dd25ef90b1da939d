"""The reference's own C++ caller drives the library. oracle/_ref/libeshkol_ref_gpu.so is the
reference's CPU matmul translation units compiled unmodified with -DESHKOL_GPU_ENABLED (what the
runtime is when a GPU backend is linked) and linked against libeshkol_gpu_hip.so: its
eshkol_matmul_f64 (lib/backend/blas_backend.cpp:859-879) and eshkol_matmul_backward_f64
(:957-1007) wrap host memory, call eshkol_gpu_matmul_f64 and rely on eshkol_gpu_free to bring
the result back. The environment is the one the reference's gates force the GPU with
(tests/gpu/ozaki_correctness_gate.sh:79-87); it is read by static initialisers of that
library, hence a child process per setting. Compared with the same sources built without
the GPU branch (oracle/_ref/libeshkol_ref.so)."""
import os
import subprocess
import sys

import pytest

import oracle
from conftest import ROOT

pytestmark = pytest.mark.gpu

CHILD = r"""
import ctypes as C, os, sys
import numpy as np
sys.path.insert(0, %(root)r); sys.path.insert(0, os.path.join(%(root)r, "tests"))
import oracle, eshkol_amd as ea
from eshkol_amd import synth
from gpu_util import normwise
gpu = ea.load()                                            # RTLD_GLOBAL; the caller's NEEDED entry resolves to it
caller = C.CDLL(oracle.REF_GPU_PATH, mode=C.RTLD_GLOBAL)   # one image, as in the runtime: the library finds
cpu = C.CDLL(oracle.REF_PATH)                              # eshkol_matmul_f64 for its own fallback there
u64, vp = C.c_uint64, C.c_void_p
for l in (caller, cpu):
    l.eshkol_matmul_f64.argtypes = [vp, vp, vp, u64, u64, u64]; l.eshkol_matmul_f64.restype = None
    l.eshkol_matmul_backward_f64.argtypes = [vp] * 5 + [u64] * 3; l.eshkol_matmul_backward_f64.restype = None
def fwd(l, A, B):
    M, K = A.shape; N = B.shape[1]
    Cm = np.full((M, N), np.nan)
    l.eshkol_matmul_f64(A.ctypes.data, B.ctypes.data, Cm.ctypes.data, M, K, N)
    return Cm
def bwd(l, G, A, B):
    M, K = A.shape; N = B.shape[1]
    gA, gB = np.full((M, K), np.nan), np.full((K, N), np.nan)
    l.eshkol_matmul_backward_f64(G.ctypes.data, A.ctypes.data, B.ctypes.data, gA.ctypes.data, gB.ctypes.data, M, K, N)
    return gA, gB
%(body)s
print("CHILD-OK")
"""

FORCE_GPU = {"ESHKOL_GPU_MATMUL_THRESHOLD": "0", "ESHKOL_GPU_THRESHOLD": "1", "ESHKOL_GPU_VERBOSE": "1",
             "ESHKOL_BLAS_PEAK_GFLOPS": "0.001", "ESHKOL_GPU_PEAK_GFLOPS": "1000000"}


def run_child(body, env):
    assert os.path.exists(oracle.REF_GPU_PATH), "oracle/_ref/libeshkol_ref_gpu.so is not built (make -C oracle ref)"
    e = {k: v for k, v in os.environ.items() if not k.startswith("ESHKOL_")}
    e.update(env)
    r = subprocess.run([sys.executable, "-u", "-c", CHILD % {"root": ROOT, "body": body}],
                       capture_output=True, text=True, env=e, timeout=600)
    assert r.returncode == 0 and "CHILD-OK" in r.stdout, "stdout:\n%s\nstderr:\n%s" % (r.stdout, r.stderr)
    return r


def test_reference_matmul_and_backward_run_on_the_native_tier():
    print("case: reference caller, native tier, 1024x768x640 forward and backward", flush=True)
    body = r"""
M, K, N = 1024, 768, 640
A, B, G = synth.normal(1, (M, K)), synth.normal(2, (K, N)), synth.normal(3, (M, N))
got, want = fwd(caller, A, B), fwd(cpu, A, B)
assert np.isfinite(got).all()                              # the copy-back on eshkol_gpu_free reached host memory
assert normwise(got, want, A, B) <= 1e-14
assert not np.array_equal(got, want)                       # and it is not the CPU kernel's summation order
gA, gB = bwd(caller, G, A, B)
wA, wB = bwd(cpu, G, A, B)
assert np.isfinite(gA).all() and np.isfinite(gB).all()
assert normwise(gA, wA, G, B) <= 1e-14 and normwise(gB, wB, A, G) <= 1e-14
# a product of at most 16 outputs never reaches the boundary (blas_backend.cpp:800-803)
small = fwd(caller, A[:4, :8].copy(), B[:8, :4].copy())
assert np.array_equal(small, fwd(cpu, A[:4, :8].copy(), B[:8, :4].copy()))
"""
    r = run_child(body, FORCE_GPU)
    lines = [l for l in r.stderr.splitlines() if l.startswith("[GPU] matmul ")]
    assert [l.split(" -> ")[0] for l in lines] == ["[GPU] matmul 1024x768 @ 768x640", "[GPU] matmul 1024x640 @ 640x768",
                                                   "[GPU] matmul 768x1024 @ 1024x640"]
    assert all("-> native fp64 MFMA" in l for l in lines)


def test_reference_matmul_reaches_the_exact_tier_by_the_gates_setting():
    print("case: reference caller, ESHKOL_SF64_KERNEL=ozaki, 640x1024x768", flush=True)
    body = r"""
M, K, N = 640, 1024, 768
A, B = synth.wide_range(4, (M, K), -8, 8), synth.wide_range(5, (K, N), -8, 8)
got = fwd(caller, A, B)
assert np.array_equal(got, oracle.matmul_ozaki_crt(A, B))
"""
    r = run_child(body, dict(FORCE_GPU, ESHKOL_SF64_KERNEL="ozaki"))
    assert r.stderr.count("[GPU] Ozaki-II: N=16, log2(P)=125.4") == 1 and "Ozaki-II CRT exact" in r.stderr


def test_reference_caller_keeps_small_products_on_its_cpu_path_by_default():
    print("case: reference caller, default thresholds, 512^3 stays on the CPU", flush=True)
    body = r"""
n = 512
A, B = synth.normal(6, (n, n)), synth.normal(7, (n, n))
assert np.array_equal(fwd(caller, A, B), fwd(cpu, A, B))   # 2.6e5 outputs < 1e9: the SIMD path, same bits
"""
    r = run_child(body, {"ESHKOL_GPU_VERBOSE": "1"})
    assert "[GPU] matmul" not in r.stderr
