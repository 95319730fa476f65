"""GPU parity tests (-m gpu) of the RMS-normalisation kernels through the C ABI (and the registered torch
op) against the fp64 CPU oracle on identical seeded inputs.

Tolerance: the reference's test allows atol 1e-3 on N(0,1) data with weights ~ N(0,1)/sqrt(dim)
(reference: test/kernels.py:59-74).  Here every element must lie within 0.51 units in the last place of
the output format of the oracle's exact value (0.5 for the final rounding, the rest for fp32 arithmetic),
which for such data is far inside 1e-3."""
import os

import numpy as np
import pytest
import torch

import capi
import oracle
import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda"
MANT = {torch.float16: 10, torch.bfloat16: 7}
MIN_EXP = {torch.float16: -14, torch.bfloat16: -126}


def assert_close(got, exact, dtype, what=""):
    got = got.float().cpu().numpy().astype(np.float64)
    e = np.floor(np.log2(np.maximum(np.abs(exact.astype(np.float64)), 2.0 ** MIN_EXP[dtype])))
    bound = 0.51 * 2.0 ** (e - MANT[dtype])
    err = np.abs(got - exact)
    worst = np.unravel_index(np.argmax(err - bound), err.shape)
    assert not (err > bound).any(), (f"{what}: {(err > bound).sum()} elements beyond 0.51 ulp; at {worst} got {got[worst]!r}, "
                                     f"exact {float(exact[worst])!r}")


def run(x, w, eps, out=None):
    out = torch.full_like(x, float("nan")) if out is None else out
    rc = capi.rmsnorm(x, w, out, eps)
    assert rc == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [
    (2, 9, 5, 128),      # per head, the reference's head size: 16 lanes per vector
    (3, 7, 64), (1, 50, 3, 40), (2, 3, 8),           # 8 lanes per vector, ragged tails of the wave
    (2, 5, 256), (1, 11, 512), (1, 7, 1024), (1, 3, 2048), (2, 3, 1536),
    (2, 5, 6144),        # per token, the reference's hidden size: one workgroup per vector
    (1, 2, 16384), (1, 3, 40000),                    # beyond what a workgroup keeps in registers
    (2, 7, 3, 10), (1, 5, 4100),                     # not a multiple of 8: element-wise kernel
])
def test_rmsnorm_matches_oracle(dtype, shape):
    g = torch.Generator().manual_seed(sum(shape))
    x = torch.randn(*shape, generator=g).to(dtype)
    w = (torch.randn(shape[-1], generator=g) / shape[-1] ** 0.5).to(dtype)
    exact = oracle.rmsnorm(x, w, 1e-6)
    y = run(x.to(DEV), w.to(DEV), 1e-6)
    assert_close(y, exact, dtype, "rmsnorm")


def test_rmsnorm_golden_in_place_and_weight_shorter_than_last_dim():
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "rmsnorm_small.npz"))
    x, w = torch.from_numpy(z["x"]).to(DEV), torch.from_numpy(z["w"]).to(DEV)
    y = run(x, w, float(z["eps"]))
    assert_close(y, z["y"].astype(np.float64), torch.float16, "golden")
    xi = x.clone()
    run(xi, w, float(z["eps"]), out=xi)                 # in place
    assert torch.equal(xi, y)
    # the vector length is the weight's (reference: rmsnorm/op.cuh:52-53): last dim 40 with an 8-long weight
    w8 = w[:8].contiguous()
    assert_close(run(x, w8, 1e-6), oracle.rmsnorm(x, w8, 1e-6), torch.float16, "short weight")


@pytest.mark.parametrize("shape", [(8, 4096, 6144), (8, 4096, 48, 128)])
def test_rmsnorm_reference_test_shapes(shape):
    """The two shapes of the reference's test (test/kernels.py:60-63): oracle on slices, and on the whole
    tensor what holds at any size: (out / w) has unit mean square per vector."""
    x, w = workloads.rmsnorm_input(shape, seed=1, device=DEV)
    y = run(x, w, 1e-6)
    flat_x, flat_y = x.view(-1, shape[-1]), y.view(-1, shape[-1])
    for lo in (0, 12345, flat_x.shape[0] - 64):
        exact = oracle.rmsnorm(flat_x[lo:lo + 64].cpu()[None], w.cpu(), 1e-6)[0]
        assert_close(flat_y[lo:lo + 64], exact, torch.float16, f"rows {lo}")
    assert torch.isfinite(flat_y.float()).all()
    keep = w.float().abs() > 1e-3                        # columns whose weight is not nearly 0
    ms = (flat_y[:, keep].float() / w[keep].float()).square().mean(-1)
    ms_x = flat_x[:, keep].float().square().mean(-1) / flat_x.float().square().mean(-1)
    assert float((ms / ms_x - 1).abs().max()) < 5e-3


def test_torch_op_equals_c_abi_and_keeps_the_reference_checks(kerns):
    x, w = workloads.rmsnorm_input((2, 33, 6, 128), seed=2, device=DEV)
    out = torch.zeros_like(x)
    assert kerns.rmsnorm(1e-6, x, w, out) is None
    torch.cuda.synchronize()
    assert torch.equal(out, run(x, w, 1e-6))
    from minfer.kernels import refs
    assert torch.allclose(refs.rmsnorm(x, w, 1e-6).float(), out.float(), atol=1e-3)      # the reference's own bar
    # reference checks (rmsnorm/op.cuh:27-42): contiguous, one dtype, 3-D or 4-D, equal shapes, divisible last dim
    with pytest.raises(RuntimeError):
        kerns.rmsnorm(1e-6, x.transpose(1, 2), w, out.transpose(1, 2))
    with pytest.raises(RuntimeError):
        kerns.rmsnorm(1e-6, x, w.float(), out)
    with pytest.raises(RuntimeError):
        kerns.rmsnorm(1e-6, x[0, 0], w, out[0, 0])
    with pytest.raises(RuntimeError):
        kerns.rmsnorm(1e-6, x, w, out[:1])
    with pytest.raises(RuntimeError):
        kerns.rmsnorm(1e-6, x, w[:100].contiguous(), out)
    with pytest.raises((RuntimeError, NotImplementedError)):
        kerns.rmsnorm(1e-6, x.cpu(), w.cpu(), out.cpu())
