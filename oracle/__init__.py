"""ctypes binding of the CPU oracle (oracle/liboracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
cpu_baseline leg of bench.py. The shipped library never touches it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")
HOSTRT_PATH = os.path.join(HERE, "liboracle_hostrt.so")
REF_PATH = os.path.join(HERE, "_ref", "libeshkol_ref.so")
REF_SSE2_PATH = os.path.join(HERE, "_ref", "libeshkol_ref_sse2.so")
# the same reference sources built with -DESHKOL_GPU_ENABLED: the caller side of the GPU boundary
REF_GPU_PATH = os.path.join(HERE, "_ref", "libeshkol_ref_gpu.so")

u64, i64 = C.c_uint64, C.c_int64
dp = C.POINTER(C.c_double)
ip = C.POINTER(C.c_int)
bp = C.POINTER(C.c_int8)
i32p = C.POINTER(C.c_int32)

MODULI = [256, 255, 253, 251, 247, 241, 239, 233, 229, 227, 223, 217, 211, 199, 197, 193]


class CRTConstants(C.Structure):
    _fields_ = [("P1", C.c_double), ("P2", C.c_double), ("Pinv", C.c_double),
                ("sl1", C.c_double * 16), ("sl2", C.c_double * 16), ("q", C.c_int * 16),
                ("num_moduli", C.c_int), ("log2P", C.c_double)]


def build():
    subprocess.run(["make", "-C", HERE, "-s"], check=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        L.oracle_reduce_precision.restype = C.c_double
        L.oracle_reduce_precision.argtypes = [C.c_double, i64]
        _lib = L
    return _lib


def _d(a):
    return a.ctypes.data_as(dp)


def _f64(a):
    return np.ascontiguousarray(a, dtype=np.float64)


def matmul_f64(A, B, fused=True):
    A, B = _f64(A), _f64(B)
    M, K = A.shape
    N = B.shape[1]
    out = np.empty((M, N))
    L = lib()
    L.oracle_matmul_set_fused(1 if fused else 0)
    L.oracle_matmul_f64(_d(A), _d(B), _d(out), u64(M), u64(K), u64(N))
    L.oracle_matmul_set_fused(1)
    return out


def matmul_backward_f64(G, A, B, fused=True):
    """(grad_A, grad_B) for C = A @ B given grad_out G."""
    G, A, B = _f64(G), _f64(A), _f64(B)
    M, K = A.shape
    N = B.shape[1]
    assert G.shape == (M, N) and B.shape[0] == K
    gA, gB = np.empty((M, K)), np.empty((K, N))
    L = lib()
    L.oracle_matmul_set_fused(1 if fused else 0)
    L.oracle_matmul_backward_f64(_d(G), _d(A), _d(B), _d(gA), _d(gB), u64(M), u64(K), u64(N))
    L.oracle_matmul_set_fused(1)
    return gA, gB


def batch_matmul_f64(a, b):
    a, b = _f64(a), _f64(b)
    batch, M, K = a.shape
    N = b.shape[2]
    out = np.empty((batch, M, N))
    lib().oracle_batch_matmul_f64(_d(a), _d(b), _d(out), i64(batch), i64(M), i64(K), i64(N))
    return out


def reduce_precision(x, dtype):
    x = _f64(x)
    out = np.empty_like(x)
    lib().oracle_reduce_precision_array(_d(x), _d(out), C.c_size_t(x.size), i64(dtype))
    return out


def matmul_reduced(A, B, dtype):
    A, B = _f64(A), _f64(B)
    M, K = A.shape
    N = B.shape[1]
    out = np.empty((M, N))
    lib().oracle_matmul_reduced(_d(A), _d(B), _d(out), u64(M), u64(K), u64(N), i64(dtype))
    return out


def matmul_reduced_f32acc(A, B, dtype, round_output):
    A, B = _f64(A), _f64(B)
    M, K = A.shape
    N = B.shape[1]
    out = np.empty((M, N))
    lib().oracle_matmul_reduced_f32acc(_d(A), _d(B), _d(out), u64(M), u64(K), u64(N), i64(dtype),
                                       C.c_int(1 if round_output else 0))
    return out


# ---- INT8 slice tier ---------------------------------------------------------

def ozaki_int8_plan(K, T):
    w = (C.c_double * 128)()
    first = (C.c_int * 129)()
    pp = (C.c_int * 128)()
    pq = (C.c_int * 128)()
    n = lib().oracle_ozaki_int8_plan(u64(K), C.c_int(T), 128, 128, w, first, pp, pq)
    if n < 0:
        return None
    npairs = first[n]
    return dict(nbuf=n, weights=np.array(w[:n]), first=np.array(first[:n + 1], dtype=np.int32),
                pair_p=np.array(pp[:npairs], dtype=np.int32), pair_q=np.array(pq[:npairs], dtype=np.int32))


def ozaki_int8_stages(A, B, T):
    """Every stage of the slice tier: rmax, cmax, slices, int32 products, C."""
    A, B = _f64(A), _f64(B)
    M, K = A.shape
    N = B.shape[1]
    L = lib()
    s = T + 1
    plan = ozaki_int8_plan(K, T)
    if plan is None:
        return None
    rmax, cmax = np.empty(M), np.empty(N)
    L.oracle_ozaki_rowmax_f64(_d(A), u64(M), u64(K), _d(rmax))
    L.oracle_ozaki_colmax_f64(_d(B), u64(K), u64(N), _d(cmax))
    As = np.empty((s, M, K), dtype=np.int8)
    Bs = np.empty((s, N, K), dtype=np.int8)
    L.oracle_ozaki_split_a_f64(_d(A), u64(M), u64(K), _d(rmax), C.c_int(s), As.ctypes.data_as(bp))
    L.oracle_ozaki_split_b_f64(_d(B), u64(K), u64(N), _d(cmax), C.c_int(s), Bs.ctypes.data_as(bp))
    G = np.empty((plan["nbuf"], M, N), dtype=np.int32)
    L.oracle_ozaki_int8_products(As.ctypes.data_as(bp), Bs.ctypes.data_as(bp), u64(M), u64(K), u64(N),
                                 C.c_int(plan["nbuf"]), plan["first"].ctypes.data_as(ip),
                                 plan["pair_p"].ctypes.data_as(ip), plan["pair_q"].ctypes.data_as(ip),
                                 G.ctypes.data_as(i32p))
    out = np.empty((M, N))
    L.oracle_ozaki_reconstruct_f64(_d(out), G.ctypes.data_as(i32p), _d(plan["weights"]),
                                   C.c_int(plan["nbuf"]), _d(rmax), _d(cmax), u64(M), u64(N))
    return dict(rmax=rmax, cmax=cmax, a_slices=As, b_slices=Bs, products=G, C=out, plan=plan)


def matmul_ozaki_int8(A, B, T):
    A, B = _f64(A), _f64(B)
    M, K = A.shape
    N = B.shape[1]
    out = np.empty((M, N))
    rc = lib().oracle_matmul_ozaki_int8_f64(_d(A), _d(B), _d(out), u64(M), u64(K), u64(N), C.c_int(T))
    return out if rc == 0 else None


# ---- CRT exact tier -----------------------------------------------------------

def crt_constants(n, aligned=False):
    c = CRTConstants()
    if aligned:
        lib().oracle_ozaki_crt_constants_aligned(C.c_int(n), C.byref(c))
    else:
        lib().oracle_ozaki_crt_constants(C.c_int(n), C.byref(c))
    return c


def ozaki_crt_stages(A, B, num_moduli=16, adaptive=False, aligned=False):
    """Every stage of the CRT tier: mu, nu, E, residue planes, products, C."""
    A, B = _f64(A), _f64(B)
    M, K = A.shape
    N = B.shape[1]
    L = lib()
    if adaptive:
        L.oracle_ozaki_adaptive_n.restype = C.c_int
        num_moduli = L.oracle_ozaki_adaptive_n(_d(A), _d(B), u64(M), u64(K), u64(N), C.c_int(num_moduli))
    crt = crt_constants(num_moduli, aligned)
    n = crt.num_moduli
    mu = np.empty(M, dtype=np.int32)
    nu = np.empty(N, dtype=np.int32)
    E = L.oracle_ozaki_crt_scaling(_d(A), _d(B), u64(M), u64(K), u64(N), C.byref(crt),
                                   mu.ctypes.data_as(ip), nu.ctypes.data_as(ip))
    ap = np.empty((n, M, K), dtype=np.int8)
    bpl = np.empty((n, N, K), dtype=np.int8)
    L.oracle_ozaki_crt_split_a(_d(A), u64(M), u64(K), mu.ctypes.data_as(ip), C.c_int(n), ap.ctypes.data_as(bp))
    L.oracle_ozaki_crt_split_b(_d(B), u64(K), u64(N), nu.ctypes.data_as(ip), C.c_int(n), bpl.ctypes.data_as(bp))
    wp = np.empty((n, M, N), dtype=np.int8)
    acc = np.empty((n, M, N), dtype=np.int32)
    L.oracle_ozaki_crt_products(ap.ctypes.data_as(bp), bpl.ctypes.data_as(bp), u64(M), u64(K), u64(N),
                                C.c_int(n), wp.ctypes.data_as(bp), acc.ctypes.data_as(i32p))
    out = np.empty((M, N))
    L.oracle_ozaki_crt_reconstruct(wp.ctypes.data_as(bp), u64(M), u64(N), C.byref(crt),
                                   mu.ctypes.data_as(ip), nu.ctypes.data_as(ip), _d(out))
    return dict(E=E, mu=mu, nu=nu, a_planes=ap, b_planes=bpl, w_planes=wp, acc32=acc, C=out,
                crt=crt, num_moduli=n)


def matmul_ozaki_crt(A, B, num_moduli=16, adaptive=False, aligned=False):
    A, B = _f64(A), _f64(B)
    M, K = A.shape
    N = B.shape[1]
    out = np.empty((M, N))
    L = lib()
    L.oracle_ozaki_crt_use_aligned_weights(C.c_int(1 if aligned else 0))
    try:
        rc = L.oracle_matmul_ozaki_crt_f64(_d(A), _d(B), _d(out), u64(M), u64(K), u64(N),
                                           C.c_int(num_moduli), C.c_int(1 if adaptive else 0))
    finally:
        L.oracle_ozaki_crt_use_aligned_weights(C.c_int(0))
    return out if rc == 0 else None


def matmul_ozaki_crt_refrep(A, B, mode, num_moduli=16, aligned=False):
    """The exact tier with the reference's own choice of representative at the half-way
    class of the modulus 256 (mode 1: its residue formula on the exact sum; mode 2: the
    Metal kernel's partial reductions). Returns (C, n_half, n_plus)."""
    A, B = _f64(A), _f64(B)
    M, K = A.shape
    N = B.shape[1]
    out = np.empty((M, N))
    half, plus = u64(0), u64(0)
    L = lib()
    L.oracle_ozaki_crt_use_aligned_weights(C.c_int(1 if aligned else 0))
    try:
        rc = L.oracle_matmul_ozaki_crt_refrep_f64(_d(A), _d(B), _d(out), u64(M), u64(K), u64(N),
                                                  C.c_int(num_moduli), C.c_int(mode), C.byref(half), C.byref(plus))
    finally:
        L.oracle_ozaki_crt_use_aligned_weights(C.c_int(0))
    assert rc == 0
    return out, half.value, plus.value


def mlp_layer(X, W, b, num_moduli=16):
    X, W = _f64(X), _f64(W)
    batch, in_f = X.shape
    out_f = W.shape[1]
    out = np.empty((batch, out_f))
    bptr = _d(_f64(b)) if b is not None else None
    rc = lib().oracle_mlp_layer_f64(_d(X), _d(W), bptr, _d(out), u64(batch), u64(in_f), u64(out_f),
                                    C.c_int(num_moduli))
    return out if rc == 0 else None


class FastConstants(C.Structure):
    _fields_ = [("num_moduli", C.c_int), ("cap", C.c_int), ("E", C.c_int), ("moduli", C.c_int * 16),
                ("q", C.c_int * 16), ("log2P", C.c_double), ("P", C.c_double),
                ("P_hi", C.c_float), ("P_lo", C.c_float)]


def fast_constants(K, n_mod=11):
    c = FastConstants()
    L = lib()
    L.oracle_ozaki_fast_constants.restype = C.c_int
    rc = L.oracle_ozaki_fast_constants(u64(K), C.c_int(n_mod), C.byref(c))
    return rc, c


def ozaki_fast_stages(A, B, n_mod=11):
    """Every stage of the reduced-precision CRT tier: exponents, residue planes, the
    integers they are residues of, exact products, the reference's float-float C and
    the exactly scaled integer product."""
    A, B = _f64(A), _f64(B)
    M, K = A.shape
    N = B.shape[1]
    L = lib()
    rc, c = fast_constants(K, n_mod)
    if rc != 0:
        return None
    n = c.num_moduli
    ei, fj = np.empty(M, np.int32), np.empty(N, np.int32)
    L.oracle_ozaki_fast_exponents(_d(A), _d(B), u64(M), u64(K), u64(N), ei.ctypes.data_as(i32p), fj.ctypes.data_as(i32p))
    ap, bpl = np.empty((n, M, K), np.int8), np.empty((n, N, K), np.int8)
    a_int, b_int = np.empty((M, K), np.int64), np.empty((N, K), np.int64)
    i64p = C.POINTER(C.c_int64)
    L.oracle_ozaki_fast_split_a(_d(A), u64(M), u64(K), ei.ctypes.data_as(i32p), C.byref(c), ap.ctypes.data_as(bp),
                                a_int.ctypes.data_as(i64p))
    L.oracle_ozaki_fast_split_b(_d(B), u64(K), u64(N), fj.ctypes.data_as(i32p), C.byref(c), bpl.ctypes.data_as(bp),
                                b_int.ctypes.data_as(i64p))
    G = np.empty((n, M, N), np.int32)
    L.oracle_ozaki_fast_products(ap.ctypes.data_as(bp), bpl.ctypes.data_as(bp), u64(M), u64(K), u64(N), C.c_int(n),
                                 G.ctypes.data_as(i32p))
    out, exact = np.empty((M, N)), np.empty((M, N))
    L.oracle_ozaki_fast_reconstruct(G.ctypes.data_as(i32p), u64(M), u64(N), C.byref(c), ei.ctypes.data_as(i32p),
                                    fj.ctypes.data_as(i32p), _d(out))
    L.oracle_ozaki_fast_exact_value(a_int.ctypes.data_as(i64p), b_int.ctypes.data_as(i64p), u64(M), u64(K), u64(N),
                                    C.byref(c), ei.ctypes.data_as(i32p), fj.ctypes.data_as(i32p), _d(exact))
    return dict(consts=c, num_moduli=n, E=c.E, moduli=list(c.moduli[:n]), q=list(c.q[:n]), ei=ei, fj=fj,
                a_planes=ap, b_planes=bpl, a_int=a_int, b_int=b_int, G=G, C=out, C_exact=exact)


def matmul_ozaki_fast(A, B, n_mod=11):
    A, B = _f64(A), _f64(B)
    M, K = A.shape
    N = B.shape[1]
    out = np.empty((M, N))
    L = lib()
    L.oracle_matmul_ozaki_fast_f64.restype = C.c_int
    rc = L.oracle_matmul_ozaki_fast_f64(_d(A), _d(B), _d(out), u64(M), u64(K), u64(N), C.c_int(n_mod))
    return rc, out
