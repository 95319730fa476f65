"""Pins the GEMM oracle (oracle/gemm_oracle.c) without the GPU: the reference's oracle call torch.addmm
(reference: refs.py:49-51) and its test's expression alpha*(A@W) + beta*bias (test/kernels.py:139) in float64,
the QKV test's x @ W^T (test/kernels.py:193-195), known answers, and a committed golden file."""
import os

import numpy as np
import pytest
import torch

import oracle


@pytest.mark.parametrize("M,N,K", [(5, 7, 3), (33, 17, 50), (64, 64, 64), (1, 130, 257)])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (2.0, 3.0), (0.5, -1.0)])
def test_matches_torch_addmm(M, N, K, alpha, beta):
    g = torch.Generator().manual_seed(M * N + K)
    a, b, c = torch.randn(M, K, generator=g), torch.randn(K, N, generator=g), torch.randn(M, N, generator=g)
    want = torch.addmm(c.double(), a.double(), b.double(), beta=beta, alpha=alpha).numpy()
    assert np.abs(oracle.gemm(a, b, c, alpha, beta) - want).max() < 1e-5
    # the same product with the weight stored [N, K]
    assert np.abs(oracle.gemm(a, b.T.contiguous(), c, alpha, beta, oracle.GEMM_B_NK) - want).max() < 1e-5
    # leading dimensions of A and C are flattened (reference: gemm/op.cuh:278)
    assert np.array_equal(oracle.gemm(a.view(1, M, K), b, c.view(1, M, N), alpha, beta), oracle.gemm(a, b, c, alpha, beta))


def test_known_answers():
    a = np.arange(6, dtype=np.float32).reshape(2, 3)           # [[0,1,2],[3,4,5]]
    b = np.array([[1, 0], [0, 1], [1, 1]], np.float32)         # [K=3, N=2]
    c = np.ones((2, 2), np.float32)
    assert np.array_equal(oracle.gemm(a, b, None, 1.0, 0.0), np.array([[2, 3], [8, 9]], np.float32))
    assert np.array_equal(oracle.gemm(a, b, c, 2.0, -3.0), np.array([[1, 3], [13, 15]], np.float32))
    assert np.array_equal(oracle.gemm(a, np.ascontiguousarray(b.T), None, 1.0, 0.0, oracle.GEMM_B_NK), np.array([[2, 3], [8, 9]], np.float32))
    eye = np.eye(4, dtype=np.float32)
    x = np.random.default_rng(0).standard_normal((3, 4)).astype(np.float32)
    assert np.array_equal(oracle.gemm(x, eye, None, 1.0, 0.0), x)
    # a non-symmetric weight tells the two layouts apart
    w = np.triu(np.ones((4, 4), np.float32))
    assert np.array_equal(oracle.gemm(x, w, None, 1.0, 0.0, oracle.GEMM_B_NK), oracle.gemm(x, np.ascontiguousarray(w.T), None, 1.0, 0.0))
    assert not np.array_equal(oracle.gemm(x, w, None, 1.0, 0.0, oracle.GEMM_B_NK), oracle.gemm(x, w, None, 1.0, 0.0))
    with pytest.raises(ValueError):
        oracle.gemm(x, w, None, 1.0, 1.0)          # beta != 0 needs C


def test_golden_vectors():
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "gemm_small.npz"))
    got = oracle.gemm(z["a"], z["b"], z["c"], float(z["alpha"]), float(z["beta"]))
    assert np.abs(got - z["d"]).max() < 1e-5
    got = oracle.gemm(z["a"], np.ascontiguousarray(z["b"].T), z["c"], float(z["alpha"]), float(z["beta"]), oracle.GEMM_B_NK)
    assert np.abs(got - z["d"]).max() < 1e-5
