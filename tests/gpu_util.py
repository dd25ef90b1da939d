"""Helpers for the GPU parity tests: every call goes through the C ABI of
libeshkol_gpu_hip.so; the oracle is only the checker."""
import ctypes as C

import numpy as np

import eshkol_amd as ea


def nrm(x):
    return float(np.sqrt(np.sum(np.asarray(x, dtype=np.longdouble) ** 2)))


def normwise(Cg, Cref, A, B):
    """||C - C_ref||_F / (||A||_F ||B||_F), the bound BASELINE.json states."""
    return nrm(np.asarray(Cg, dtype=np.longdouble) - np.asarray(Cref, dtype=np.longdouble)) / (nrm(A) * nrm(B))


def ulp_distance(a, b):
    """Distance in units in the last place between two float64 arrays."""
    ai = np.ascontiguousarray(a, dtype=np.float64).view(np.int64).astype(np.int64)
    bi = np.ascontiguousarray(b, dtype=np.float64).view(np.int64).astype(np.int64)
    ai = np.where(ai < 0, np.int64(-2 ** 63) - ai, ai)
    bi = np.where(bi < 0, np.int64(-2 ** 63) - bi, bi)
    return np.abs(ai - bi)


class Operands:
    """A, B on the device, C allocated."""

    def __init__(self, A, B):
        self.A, self.B = np.ascontiguousarray(A, dtype=np.float64), np.ascontiguousarray(B, dtype=np.float64)
        self.M, self.K = self.A.shape
        self.N = self.B.shape[1]
        self.dA = ea.DeviceArray.from_host(self.A)
        self.dB = ea.DeviceArray.from_host(self.B)
        self.dC = ea.DeviceArray((self.M, self.N))

    def result(self):
        ea.synchronize()
        return self.dC.download()


def stream():
    return ea.load().eshkol_hip_get_stream()


def run_dgemm(A, B):
    ops = Operands(A, B)
    rc = ea.load().hip_dgemm_f64(ops.dA.ptr, ops.dB.ptr, ops.dC.ptr, ops.M, ops.K, ops.N, stream())
    assert rc == 0
    return ops.result()


def run_crt(A, B, num_moduli=16, adaptive=False, bias=None, act=0, want_stages=True):
    lib = ea.load()
    ops = Operands(A, B)
    dbias = ea.DeviceArray.from_host(np.asarray(bias, dtype=np.float64)) if bias is not None else None
    rc = lib.hip_matmul_ozaki_crt_f64(ops.dA.ptr, ops.dB.ptr, ops.dC.ptr, ops.M, ops.K, ops.N,
                                      num_moduli, 1 if adaptive else 0,
                                      dbias.ptr if dbias is not None else None, act, stream())
    if rc != 0:
        return rc, None, None
    Cg = ops.result()
    if not want_stages:
        return 0, Cg, None
    sg = ea.HipOzakiCrtStages()
    assert lib.hip_ozaki_crt_last_stages(C.byref(sg)) == 0
    n, M, K, N = sg.num_moduli, ops.M, ops.K, ops.N
    ap = ea.deinterleave(ea.download_raw(sg.a_planes, (n, sg.rows_a_padded, sg.ldk), np.int8), sg.layout)
    bp = ea.deinterleave(ea.download_raw(sg.b_planes, (n, sg.rows_b_padded, sg.ldk), np.int8), sg.layout)
    st = dict(num_moduli=n, E=sg.E,
              mu=ea.download_raw(sg.mu, (M,), np.int32), nu=ea.download_raw(sg.nu, (N,), np.int32),
              a_planes=ap[:, :M, :K], b_planes=bp[:, :N, :K],
              a_pad_clear=(not ap[:, M:, :].any()) and (not ap[:, :, K:].any()),
              b_pad_clear=(not bp[:, N:, :].any()) and (not bp[:, :, K:].any()),
              w_planes=ea.download_raw(sg.w_planes, (n, sg.w_rows, sg.w_ld), np.int8)[:, :M, :N])
    return 0, Cg, st


def run_int8(A, B, T, want_stages=True):
    lib = ea.load()
    ops = Operands(A, B)
    rc = lib.hip_matmul_ozaki_int8_f64(ops.dA.ptr, ops.dB.ptr, ops.dC.ptr, ops.M, ops.K, ops.N, T, stream())
    if rc != 0:
        return rc, None, None
    Cg = ops.result()
    if not want_stages:
        return 0, Cg, None
    sg = ea.HipOzakiInt8Stages()
    assert lib.hip_ozaki_int8_last_stages(C.byref(sg)) == 0
    s, M, K, N = sg.s, ops.M, ops.K, ops.N
    As = ea.deinterleave(ea.download_raw(sg.a_slices, (s, sg.rows_a_padded, sg.ldk), np.int8), sg.layout)
    Bs = ea.deinterleave(ea.download_raw(sg.b_slices, (s, sg.rows_b_padded, sg.ldk), np.int8), sg.layout)
    st = dict(s=s, nbuf=sg.nbuf, a_slices=As[:, :M, :K], b_slices=Bs[:, :N, :K],
              pad_clear=not (As[:, M:, :].any() or As[:, :, K:].any() or Bs[:, N:, :].any() or Bs[:, :, K:].any()),
              products=ea.download_raw(sg.products, (sg.nbuf, sg.g_rows, sg.g_ld), np.int32)[:, :M, :N],
              rmax=ea.download_raw(sg.rmax, (M,), np.float64), cmax=ea.download_raw(sg.cmax, (N,), np.float64))
    return 0, Cg, st


def run_reduced(A, B, dtype, round_output):
    ops = Operands(A, B)
    rc = ea.load().hip_matmul_reduced_f64(ops.dA.ptr, ops.dB.ptr, ops.dC.ptr, ops.M, ops.K, ops.N,
                                          dtype, 1 if round_output else 0, stream())
    assert rc == 0
    return ops.result()


def run_fast(A, B, n_mod=11, want_stages=True, trans=None):
    """The reduced-precision CRT tier on the device; trans = (trans_a, trans_b) hands the
    operands over transposed (A as [K][M] / B as [N][K])."""
    lib = ea.load()
    ops = Operands(A, B)
    if trans is None:
        rc = lib.hip_matmul_ozaki_fast_f64(ops.dA.ptr, ops.dB.ptr, ops.dC.ptr, ops.M, ops.K, ops.N, n_mod, stream())
    else:
        ta, tb = trans
        dA = ea.DeviceArray.from_host(np.ascontiguousarray(A.T)) if ta else ops.dA
        dB = ea.DeviceArray.from_host(np.ascontiguousarray(B.T)) if tb else ops.dB
        rc = lib.hip_matmul_ozaki_fast_f64_ex(dA.ptr, dB.ptr, ops.dC.ptr, ops.M, ops.K, ops.N, ta, tb, n_mod, stream())
    if rc != 0:
        return rc, None, None
    Cg = ops.result()
    if not want_stages:
        return 0, Cg, None
    sg = ea.HipOzakiFastStages()
    assert lib.hip_ozaki_fast_last_stages(C.byref(sg)) == 0
    n, M, K, N = sg.num_moduli, ops.M, ops.K, ops.N
    ap = ea.deinterleave(ea.download_raw(sg.a_planes, (n, sg.rows_a_padded, sg.ldk), np.int8), sg.layout)
    bp = ea.deinterleave(ea.download_raw(sg.b_planes, (n, sg.rows_b_padded, sg.ldk), np.int8), sg.layout)
    st = dict(num_moduli=n, E=sg.E, cap=sg.cap, moduli=list(sg.moduli[:n]),
              shift_a=ea.download_raw(sg.shift_a, (M,), np.int32), shift_b=ea.download_raw(sg.shift_b, (N,), np.int32),
              a_planes=ap[:, :M, :K], b_planes=bp[:, :N, :K],
              a_pad_clear=(not ap[:, M:, :].any()) and (not ap[:, :, K:].any()),
              b_pad_clear=(not bp[:, N:, :].any()) and (not bp[:, :, K:].any()),
              w_planes=ea.download_raw(sg.w_planes, (n, sg.w_rows, sg.w_ld), np.int8)[:, :M, :N])
    return 0, Cg, st
