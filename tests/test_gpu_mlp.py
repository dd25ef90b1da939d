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


def test_mlp_reduced_size(gpu):
    dims = [64, 256, 256, 64]
    X = synth.normal(1, (128, dims[0]))
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
