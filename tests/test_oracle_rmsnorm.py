"""Pins the RMS-normalisation oracle (oracle/rmsnorm_oracle.c) without the GPU.

The reference holds no stored vectors for this op: its test compares the CUDA kernel with
F.rms_norm live, unseeded, at atol 1e-3 (reference: test/kernels.py:59-74).  Pins: the reference's
own oracle call (F.rms_norm over the last dimension, refs.py:10) in float64, a committed golden file
made the same way, and what the mathematics fixes."""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle


@pytest.mark.parametrize("shape", [(2, 7, 48), (1, 3, 4, 128), (2, 2, 6144), (1, 5, 3, 10)])
@pytest.mark.parametrize("eps", [1e-6, 1e-2])
def test_matches_torch_rms_norm(shape, eps):
    g = torch.Generator().manual_seed(len(shape) * 100 + shape[-1])
    x = torch.randn(*shape, generator=g)
    w = torch.randn(shape[-1], generator=g) / shape[-1] ** 0.5
    want = F.rms_norm(x.double(), (shape[-1],), weight=w.double(), eps=eps).numpy()
    assert np.abs(oracle.rmsnorm(x, w, eps) - want).max() < 1e-6


def test_known_answers_and_invariants():
    # one non-zero element c at index i, eps = 0: mean square = c^2/dim, so out[i] = sign(c) * w[i] * sqrt(dim)
    x = np.zeros((1, 1, 16), np.float32)
    x[0, 0, 5] = -3.0
    w = np.arange(1, 17, dtype=np.float32)
    y = oracle.rmsnorm(x, w, 0.0)
    assert y[0, 0, 5] == pytest.approx(-6.0 * 4.0, rel=1e-7) and np.count_nonzero(y) == 1
    # a constant vector a, eps = 0: out = sign(a) * w
    y = oracle.rmsnorm(np.full((1, 2, 16), -0.25, np.float32), w, 0.0)
    assert np.allclose(y, -w, rtol=1e-7)
    # eps enters under the root: x = 0 gives 0; with x = e_i and dim = 4, out = w / sqrt(1/4 + eps)
    assert np.array_equal(oracle.rmsnorm(np.zeros((1, 1, 8), np.float32), w[:8], 1e-6), np.zeros((1, 1, 8), np.float32))
    x4 = np.array([[[0, 2.0, 0, 0]]], np.float32)
    assert oracle.rmsnorm(x4, np.ones(4, np.float32), 3.0)[0, 0, 1] == pytest.approx(2.0 / np.sqrt(1.0 + 3.0), rel=1e-7)
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 3, 64)).astype(np.float32)
    w = rng.standard_normal(64).astype(np.float32)
    y = oracle.rmsnorm(x, w, 0.0)
    # scale invariance in x (eps = 0), linearity in w, output mean square equals that of w-weighted unit vector
    assert np.allclose(oracle.rmsnorm(4.0 * x, w, 0.0), y, rtol=1e-6)
    assert np.allclose(oracle.rmsnorm(x, 2.0 * w, 0.0), 2.0 * y, rtol=1e-6)
    assert np.allclose(((y / w) ** 2).mean(-1), 1.0, rtol=1e-5)
    # vectors are independent and the vector length is the weight's: [2,3,64] with a 32-long weight is 12 vectors
    w32 = w[:32]
    y32 = oracle.rmsnorm(x, w32, 1e-6)
    assert np.allclose(y32.reshape(-1, 32)[7], oracle.rmsnorm(x.reshape(-1, 32)[7:8].reshape(1, 1, 32), w32, 1e-6).ravel(), rtol=1e-6)
    with pytest.raises(ValueError):
        oracle.rmsnorm(x, w, -1.0)


def test_golden_vectors():
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "rmsnorm_small.npz"))
    assert np.abs(oracle.rmsnorm(z["x"], z["w"], float(z["eps"])) - z["y"]).max() < 1e-6
