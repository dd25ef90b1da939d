"""Operands read k-major (B as the runtime stores it) without a transposed copy:
column maxima, CRT residue planes, INT8 slice planes and 16-bit narrowing must
be bit-identical to the row-major kernels applied to an explicit transpose,
padding included. The row-major kernels are themselves checked against the
oracle in the tier tests, so equality here carries that parity over."""
import numpy as np
import pytest

import eshkol_amd as ea
from eshkol_amd import synth
from gpu_util import stream

pytestmark = pytest.mark.gpu

# (K, R): k extent, number of rows of the transposed view (columns of the stored matrix)
SHAPES = [(1, 1), (2, 3), (7, 5), (64, 64), (128, 32), (129, 33), (130, 257), (300, 70), (1000, 513),
          (1024, 1024), (2049, 511)]


def dev(x, dtype=np.float64):
    return ea.DeviceArray.from_host(np.ascontiguousarray(x, dtype=dtype))


def pad(n, m):
    return (n + m - 1) // m * m


@pytest.mark.parametrize("K,R", SHAPES)
def test_column_maxima(gpu, K, R):
    lib = ea.load()
    X = synth.wide_range(K * 31 + R, (K, R))
    X[:, R // 2] = 0.0                                   # an all-zero column takes zero_value
    dX, dXt = dev(X), dev(X.T)
    for zero_value in (0.0, 1.0):
        a, b = ea.DeviceArray((R,)), ea.DeviceArray((R,))
        assert lib.hip_colabsmax_f64(dX.ptr, K, R, zero_value, a.ptr, stream()) == 0
        assert lib.hip_rowabsmax_f64(dXt.ptr, R, K, zero_value, b.ptr, stream()) == 0
        ea.synchronize()
        got = a.download()
        assert np.array_equal(got, b.download())
        want = np.abs(X).max(axis=0)
        want[want == 0.0] = zero_value
        assert np.array_equal(got, want)


@pytest.mark.parametrize("rows,K", [(1, 1024), (5, 4096), (64, 4097), (256, 1031), (3, 131071), (7, 5002)])
def test_row_maxima_of_a_few_long_rows(gpu, rows, K):
    """A handful of rows in front of a layer: a workgroup per row. Also from a base that is
    not a multiple of 16 bytes, with a zero row and a row that holds a NaN."""
    lib = ea.load()
    X = synth.wide_range(rows * 7 + K, (rows, K))
    if rows > 2:
        X[1, :] = 0.0
        X[2, K - 1] = np.nan
    flat = dev(np.concatenate([[0.0], X.ravel()]))
    for base, zero_value in ((dev(X).ptr, 0.0), (flat.ptr + 8, 1.0)):
        out = ea.DeviceArray((rows,))
        assert lib.hip_rowabsmax_f64(base, rows, K, zero_value, out.ptr, stream()) == 0
        ea.synchronize()
        got = out.download()
        want = np.abs(X).max(axis=1)
        want[want == 0.0] = zero_value
        want[np.isnan(want)] = np.inf
        assert np.array_equal(got, want)


def test_column_maxima_flag_non_finite_input(gpu):
    lib = ea.load()
    X = synth.normal(3, (200, 70))
    X[17, 5] = np.nan
    X[199, 69] = -np.inf
    out = ea.DeviceArray((70,))
    assert lib.hip_colabsmax_f64(dev(X).ptr, 200, 70, 0.0, out.ptr, stream()) == 0
    ea.synchronize()
    got = out.download()
    assert np.isposinf(got[5]) and np.isposinf(got[69]) and np.isfinite(np.delete(got, [5, 69])).all()


@pytest.mark.parametrize("K,R", SHAPES)
@pytest.mark.parametrize("nmod", [2, 9, 16])
def test_crt_planes(gpu, K, R, nmod):
    lib = ea.load()
    X = synth.wide_range(K + 7 * R, (K, R), -8, 8)
    shift = (20 - np.floor(np.log2(np.maximum(np.abs(X).max(axis=0), 1e-300)))).astype(np.int32)
    Rp, ldk = pad(R, 256), pad(K, 256)
    dX, dXt, dsh = dev(X), dev(X.T), dev(shift, np.int32)
    pa = ea.DeviceArray.from_host(np.full((nmod, Rp, ldk), 77, np.int8))
    pb = ea.DeviceArray.from_host(np.full((nmod, Rp, ldk), 78, np.int8))
    assert lib.hip_ozaki_crt_split_kmajor_f64(dX.ptr, R, K, dsh.ptr, nmod, pa.ptr, Rp, ldk, stream()) == 0
    assert lib.hip_ozaki_crt_split_f64(dXt.ptr, R, K, dsh.ptr, nmod, pb.ptr, Rp, ldk, stream()) == 0
    ea.synchronize()
    a = pa.download()
    assert np.array_equal(a, pb.download())
    assert not a[:, R:, :].any() and not a[:, :, K:].any()


@pytest.mark.parametrize("K,R", [(7, 5), (130, 257), (300, 70), (1000, 513)])
def test_crt_planes_at_any_even_pitch(gpu, K, R):
    """The kernels pick wider stores when the pitch allows: every variant must write the same residues."""
    lib = ea.load()
    X = synth.wide_range(3 * K + R, (K, R), -8, 8)
    shift = (20 - np.floor(np.log2(np.maximum(np.abs(X).max(axis=0), 1e-300)))).astype(np.int32)
    dX, dXt, dsh = dev(X), dev(X.T), dev(shift, np.int32)
    want = None
    for Rp, ldk in [(pad(R, 256), pad(K, 256)), (R, K + (K & 1)), (R + 3, K + (K & 1) + 2), (R + 1, pad(K, 4) + 4),
                    (R, pad(K, 16)), (R + 2, pad(K, 16) + 16)]:
        pa = ea.DeviceArray.from_host(np.full((16, Rp, ldk), 77, np.int8))
        pb = ea.DeviceArray.from_host(np.full((16, Rp, ldk), 78, np.int8))
        assert lib.hip_ozaki_crt_split_kmajor_f64(dX.ptr, R, K, dsh.ptr, 16, pa.ptr, Rp, ldk, stream()) == 0
        assert lib.hip_ozaki_crt_split_f64(dXt.ptr, R, K, dsh.ptr, 16, pb.ptr, Rp, ldk, stream()) == 0
        ea.synchronize()
        a, b = pa.download(), pb.download()
        assert np.array_equal(a, b), (Rp, ldk)
        assert not a[:, R:, :].any() and not a[:, :, K:].any(), (Rp, ldk)
        if want is None:
            want = a[:, :R, :K].copy()
        assert np.array_equal(a[:, :R, :K], want), (Rp, ldk)


@pytest.mark.parametrize("K,R", SHAPES)
def test_slice_planes(gpu, K, R):
    lib = ea.load()
    s = 7
    X = synth.normal(K + 3 * R, (K, R))
    scale = np.abs(X).max(axis=0)
    scale[scale == 0.0] = 1.0
    Rp, ldk = pad(R, 256), pad(K, 256)
    dX, dXt, dsc = dev(X), dev(X.T), dev(scale)
    pa = ea.DeviceArray.from_host(np.full((s, Rp, ldk), 77, np.int8))
    pb = ea.DeviceArray.from_host(np.full((s, Rp, ldk), 78, np.int8))
    assert lib.hip_ozaki_slice_kmajor_f64(dX.ptr, R, K, dsc.ptr, s, pa.ptr, Rp, ldk, stream()) == 0
    assert lib.hip_ozaki_slice_f64(dXt.ptr, R, K, dsc.ptr, s, pb.ptr, Rp, ldk, stream()) == 0
    ea.synchronize()
    a = pa.download()
    assert np.array_equal(a, pb.download())
    assert not a[:, R:, :].any() and not a[:, :, K:].any()


@pytest.mark.parametrize("K,R", [(7, 5), (130, 257), (300, 70), (1000, 513)])
def test_slice_planes_at_any_even_pitch(gpu, K, R):
    lib = ea.load()
    X = synth.wide_range(5 * K + R, (K, R), -8, 8)
    scale = np.abs(X).max(axis=0)
    scale[scale == 0.0] = 1.0
    dX, dXt, dsc = dev(X), dev(X.T), dev(scale)
    want = None
    for Rp, ldk in [(pad(R, 256), pad(K, 256)), (R, K + (K & 1)), (R + 3, K + (K & 1) + 2), (R + 1, pad(K, 4) + 4),
                    (R, pad(K, 16)), (R + 2, pad(K, 16) + 16)]:
        pa = ea.DeviceArray.from_host(np.full((7, Rp, ldk), 77, np.int8))
        pb = ea.DeviceArray.from_host(np.full((7, Rp, ldk), 78, np.int8))
        assert lib.hip_ozaki_slice_kmajor_f64(dX.ptr, R, K, dsc.ptr, 7, pa.ptr, Rp, ldk, stream()) == 0
        assert lib.hip_ozaki_slice_f64(dXt.ptr, R, K, dsc.ptr, 7, pb.ptr, Rp, ldk, stream()) == 0
        ea.synchronize()
        a, b = pa.download(), pb.download()
        assert np.array_equal(a, b), (Rp, ldk)
        assert not a[:, R:, :].any() and not a[:, :, K:].any(), (Rp, ldk)
        if want is None:
            want = a[:, :R, :K].copy()
        assert np.array_equal(a[:, :R, :K], want), (Rp, ldk)


@pytest.mark.parametrize("K,R", SHAPES)
@pytest.mark.parametrize("is_bf16", [0, 1])
def test_narrowing(gpu, K, R, is_bf16):
    lib = ea.load()
    X = synth.normal(K + 5 * R, (K, R))
    Rp, ld = pad(R, 256), pad(K, 128)
    dX, dXt = dev(X), dev(X.T)
    pa = ea.DeviceArray.from_host(np.full((Rp, ld), 0x7777, np.uint16))
    pb = ea.DeviceArray.from_host(np.full((Rp, ld), 0x7878, np.uint16))
    assert lib.hip_convert_f64_to_16_kmajor(dX.ptr, pa.ptr, R, K, Rp, ld, is_bf16, stream()) == 0
    assert lib.hip_convert_f64_to_16(dXt.ptr, pb.ptr, R, K, Rp, ld, is_bf16, stream()) == 0
    ea.synchronize()
    a = pa.download()
    assert np.array_equal(a, pb.download())
    assert not a[R:, :].any() and not a[:, K:].any()


@pytest.mark.parametrize("K,R", [(1, 1), (7, 5), (129, 33), (300, 70), (1000, 513), (1024, 1024), (2049, 511)])
@pytest.mark.parametrize("nmod", [2, 16])
def test_interleaved_crt_planes_hold_the_same_residues(gpu, K, R, nmod):
    """Interleaved planes (rows in blocks of 32, 16-byte k-chunks slow, rows fast) from both
    operand orders, put back in order, are the row-major planes byte for byte, padding included."""
    lib = ea.load()
    X = synth.wide_range(K + 11 * R, (K, R), -8, 8)
    shift = (20 - np.floor(np.log2(np.maximum(np.abs(X).max(axis=0), 1e-300)))).astype(np.int32)
    Rp, ldk = pad(R, 256), pad(K, 512)
    dX, dXt, dsh = dev(X), dev(X.T), dev(shift, np.int32)
    ref = ea.DeviceArray.from_host(np.full((nmod, Rp, ldk), 78, np.int8))
    assert lib.hip_ozaki_crt_split_f64(dXt.ptr, R, K, dsh.ptr, nmod, ref.ptr, Rp, ldk, stream()) == 0
    for kmajor, src in ((1, dX), (0, dXt)):
        out = ea.DeviceArray.from_host(np.full((nmod, Rp, ldk), 77, np.int8))
        assert lib.hip_ozaki_crt_split_planes_f64(src.ptr, R, K, dsh.ptr, nmod, out.ptr, Rp, ldk, kmajor, 1, stream()) == 0
        ea.synchronize()
        assert np.array_equal(ea.deinterleave(out.download(), 1), ref.download()), kmajor
    odd = ea.DeviceArray((nmod, Rp + 1, ldk), np.int8)
    assert lib.hip_ozaki_crt_split_planes_f64(dXt.ptr, R, K, dsh.ptr, nmod, odd.ptr, Rp + 1, ldk, 0, 1, stream()) == -1


@pytest.mark.parametrize("K,R", [(1, 1), (7, 5), (129, 33), (300, 70), (1000, 513), (1024, 1024), (2049, 511)])
def test_interleaved_slice_planes_hold_the_same_slices(gpu, K, R):
    lib = ea.load()
    s = 7
    X = synth.normal(K + 13 * R, (K, R))
    scale = np.abs(X).max(axis=0)
    scale[scale == 0.0] = 1.0
    Rp, ldk = pad(R, 256), pad(K, 512)
    dX, dXt, dsc = dev(X), dev(X.T), dev(scale)
    ref = ea.DeviceArray.from_host(np.full((s, Rp, ldk), 78, np.int8))
    assert lib.hip_ozaki_slice_f64(dXt.ptr, R, K, dsc.ptr, s, ref.ptr, Rp, ldk, stream()) == 0
    for kmajor, src in ((1, dX), (0, dXt)):
        out = ea.DeviceArray.from_host(np.full((s, Rp, ldk), 77, np.int8))
        assert lib.hip_ozaki_slice_planes_f64(src.ptr, R, K, dsc.ptr, s, out.ptr, Rp, ldk, kmajor, 1, stream()) == 0
        ea.synchronize()
        assert np.array_equal(ea.deinterleave(out.download(), 1), ref.download()), kmajor


@pytest.mark.parametrize("K,R", [(40, 33), (97, 96), (129, 160), (500, 289)])
def test_interleaved_planes_with_the_least_padding_the_layout_allows(gpu, K, R):
    """Rows padded to 32 and the k pitch to 32 bytes only (64 elements for 16-bit planes): the
    k-major kernels, whose blocks are larger than that, must stay inside the planes (sentinel
    bytes behind the last one) and still fill the padding with zeros."""
    lib = ea.load()
    nmod, s = 5, 3
    X = synth.normal(K + 17 * R, (K, R))
    shift = (20 - np.floor(np.log2(np.abs(X).max(axis=0)))).astype(np.int32)
    scale = np.abs(X).max(axis=0)
    Rp, ldk = pad(R, 32), pad(K, 32)
    dX, dXt, dsh, dsc = dev(X), dev(X.T), dev(shift, np.int32), dev(scale)

    def run(planes, call_ref, call):
        ref = ea.DeviceArray.from_host(np.full((planes, Rp, ldk), 78, np.int8))
        assert call_ref(ref.ptr) == 0
        for kmajor, src in ((1, dX), (0, dXt)):
            out = ea.DeviceArray.from_host(np.full((planes + 1, Rp, ldk), 77, np.int8))
            assert call(src.ptr, out.ptr, kmajor) == 0
            ea.synchronize()
            got = out.download()
            assert np.all(got[planes] == 77), kmajor
            assert np.array_equal(ea.deinterleave(got[:planes], 1), ref.download()), kmajor

    run(nmod, lambda r: lib.hip_ozaki_crt_split_f64(dXt.ptr, R, K, dsh.ptr, nmod, r, Rp, ldk, stream()),
        lambda x, o, km: lib.hip_ozaki_crt_split_planes_f64(x, R, K, dsh.ptr, nmod, o, Rp, ldk, km, 1, stream()))
    run(s, lambda r: lib.hip_ozaki_slice_f64(dXt.ptr, R, K, dsc.ptr, s, r, Rp, ldk, stream()),
        lambda x, o, km: lib.hip_ozaki_slice_planes_f64(x, R, K, dsc.ptr, s, o, Rp, ldk, km, 1, stream()))
    ld = pad(K, 64)
    for is_bf16 in (0, 1):
        ref = ea.DeviceArray.from_host(np.full((Rp, ld), 7, np.uint16))
        assert lib.hip_convert_f64_to_16(dXt.ptr, ref.ptr, R, K, Rp, ld, is_bf16, stream()) == 0
        for kmajor, src in ((1, dX), (0, dXt)):
            out = ea.DeviceArray.from_host(np.full((2, Rp, ld), 9, np.uint16))
            assert lib.hip_convert_f64_to_16_planes(src.ptr, out.ptr, 1, R, K, Rp, ld, is_bf16, kmajor, 1, stream()) == 0
            ea.synchronize()
            got = out.download()
            assert np.all(got[1] == 9), kmajor
            assert np.array_equal(ea.deinterleave(got[:1], 1)[0], ref.download()), kmajor
    # the reduced-precision CRT tier has no entry for plain row-major planes: all four forms must agree
    nf = 8
    got = {}
    for kmajor, src in ((1, dX), (0, dXt)):
        for layout in (0, 1):
            out = ea.DeviceArray.from_host(np.full((nf + 1, Rp, ldk), 77, np.int8))
            assert lib.hip_ozaki_fast_split_planes_f64(src.ptr, R, K, dsh.ptr, nf, out.ptr, Rp, ldk, kmajor, layout, stream()) == 0
            ea.synchronize()
            g = out.download()
            assert np.all(g[nf] == 77), (kmajor, layout)
            got[kmajor, layout] = ea.deinterleave(g[:nf], layout)
    assert all(np.array_equal(got[0, 0], g) for g in got.values())
    assert got[0, 0].any() and not got[0, 0][:, R:].any() and not got[0, 0][:, :, K:].any()
