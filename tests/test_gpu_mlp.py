"""BASELINE configuration 5: a dense-layer forward pass y = tanh(x W + b) with
every GEMM through the exact tier and the bias add and tanh fused into its
epilogue. Checked against the oracle layer by layer; tanh is glibc's on the CPU
and the device library's on the GPU, so the bar on the activations is 4 ulp of
1.0 (|tanh| <= 1), while the pre-activation GEMM keeps the exact tier's 2 ulp."""
import numpy as np
import pytest

import eshkol_amd as ea
import oracle
from eshkol_amd import synth
from gpu_util import run_crt, ulp_distance

pytestmark = pytest.mark.gpu
ATOL = 4 * np.finfo(np.float64).eps


def forward(X, layers):
    h = X
    outs = []
    for W, b in layers:
        rc, h, _ = run_crt(h, W, bias=b, act=1, want_stages=False)
        assert rc == 0
        outs.append(h)
    return outs


@pytest.mark.parametrize("batch,dims", [(128, [64, 256, 256, 64]), (130, [63, 255, 129, 65]), (37, [100, 1030, 77, 3])])
def test_mlp_reduced_size(gpu, batch, dims):
    """Layer sizes that are multiples of four, and sizes that are multiples of nothing (rows of the
    activations off 16-byte boundaries, a last group of columns that is not whole)."""
    X = synth.normal(1, (batch, dims[0]))
    layers = [(synth.xavier_uniform(10 + i, dims[i], dims[i + 1]), synth.uniform(20 + i, (dims[i + 1],), -0.05, 0.05))
              for i in range(3)]
    outs = forward(X, layers)
    h = X
    for (W, b), got in zip(layers, outs):
        want = oracle.mlp_layer(h, W, b)
        assert np.abs(got - want).max() <= ATOL
        h = got                               # feed the device activations forward: per-layer check


def test_mlp_config5_full_size_sampled(gpu):
    batch, dims = 4096, [1024, 4096, 4096, 1024]
    print("mlp full", flush=True)
    X = synth.normal(1, (batch, dims[0]))
    layers = [(synth.xavier_uniform(10 + i, dims[i], dims[i + 1]), np.zeros(dims[i + 1])) for i in range(3)]
    outs = forward(X, layers)
    rows = [0, 1, 255, 256, 2049, batch - 257, batch - 1]
    h = X
    for (W, b), got in zip(layers, outs):
        cols = [0, 5, 255, 256, W.shape[1] // 2 + 1, W.shape[1] - 1]
        want = oracle.mlp_layer(h[rows], W[:, cols], b[cols])
        assert np.abs(got[rows][:, cols] - want).max() <= ATOL
        assert np.all(np.abs(got) <= 1.0)
        h = got


@pytest.mark.parametrize("batch,dims", [(128, [512, 640, 512]), (2048, [1024, 2048, 1024])])
def test_prepared_weights_give_the_same_bits(gpu, batch, dims):
    """Weights prepared once (hip_ozaki_crt_prepare_operand_b: their column maxima and residue
    planes kept between calls) against the ordinary entry point that splits them on every call:
    the planes are the same bytes, so every activation must be identical, for fresh inputs too;
    a call whose shape the prepared form does not fit (other layout) still gives the same result."""
    import ctypes as C
    lib = ea.load()
    st = lib.eshkol_hip_get_stream()
    layers = [(synth.xavier_uniform(30 + i, dims[i], dims[i + 1]), synth.uniform(40 + i, (dims[i + 1],), -0.05, 0.05))
              for i in range(len(dims) - 1)]
    dW = [ea.DeviceArray.from_host(W) for W, _ in layers]
    dB = [ea.DeviceArray.from_host(b) for _, b in layers]
    handles = []
    for i, (W, _) in enumerate(layers):
        h = C.c_void_p()
        assert lib.hip_ozaki_crt_prepare_operand_b(dW[i].ptr, W.shape[0], W.shape[1], 0, 16, batch, C.byref(h), st) == 0
        handles.append(h)

    def run(X, prepared, rows):
        src = ea.DeviceArray.from_host(X)
        outs = []
        for i, (W, _) in enumerate(layers):
            out = ea.DeviceArray((rows, W.shape[1]))
            if prepared:
                rc = lib.hip_matmul_ozaki_crt_prepared_f64(src.ptr, handles[i], out.ptr, rows, W.shape[0], W.shape[1],
                                                           0, 16, 0, dB[i].ptr, 1, st)
            else:
                rc = lib.hip_matmul_ozaki_crt_f64(src.ptr, dW[i].ptr, out.ptr, rows, W.shape[0], W.shape[1],
                                                  16, 0, dB[i].ptr, 1, st)
            assert rc == 0
            ea.synchronize()
            outs.append(out.download())
            src = out
        return outs

    for seed in (1, 2):
        X = synth.normal(seed, (batch, dims[0]))
        for got, want in zip(run(X, True, batch), run(X, False, batch)):
            assert np.array_equal(got, want)
    # 40 rows: the kernel for a few rows takes interleaved planes (kept where the larger size made them so, made so for
    # this call where it made row-major ones); 300 rows after that: interleaved planes serve tiled kernels with few tiles too
    for rows in (40, 300):
        X = synth.normal(3, (rows, dims[0]))
        for got, want in zip(run(X, True, rows), run(X, False, rows)):
            assert np.array_equal(got, want)
    for h in handles:
        lib.hip_ozaki_crt_release_prepared(h)
    # what cannot be prepared is refused, not approximated: fewer moduli make E depend on the data
    h = C.c_void_p()
    assert lib.hip_ozaki_crt_prepare_operand_b(dW[0].ptr, dims[0], dims[1], 0, 12, batch, C.byref(h), st) == -1
    bad = layers[0][0].copy(); bad[3, 4] = np.inf
    assert lib.hip_ozaki_crt_prepare_operand_b(ea.DeviceArray.from_host(bad).ptr, dims[0], dims[1], 0, 16, batch,
                                               C.byref(h), st) == -1
