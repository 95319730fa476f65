"""GPU checks (-m gpu) of the calibration entry points (include/minfer_attn.h: minfer_calib_mfma_rate,
minfer_calib_mfma_rate_32x32x16, minfer_calib_attn_mix; measurement loops with no counterpart in the reference).
The MFMA-only loops add up known products, so what a lane writes to the sink is fixed by the operand and result
layouts of the two matrix instructions, the layouts the prefill and GEMM kernels are built on: the expected values
are evaluated in float64 from the same operand buffer."""
import ctypes

import numpy as np
import pytest
import torch

import capi

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _fns():
    L = capi.lib()
    i64 = ctypes.c_int64
    for fn in (L.minfer_calib_mfma_rate, L.minfer_calib_mfma_rate_32x32x16):
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.c_int, ctypes.c_void_p, i64, i64, ctypes.c_void_p, ctypes.c_void_p]
    L.minfer_calib_attn_mix.restype = ctypes.c_int
    L.minfer_calib_attn_mix.argtypes = [ctypes.c_int, ctypes.c_void_p, i64, i64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    return L


def _operands(dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return (0.5 * torch.randn(16, 64, 8, generator=g)).to(dtype)     # 16 fragments x 64 lanes x 8 values


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("iters", [1, 3])
def test_mfma_16x16x32_loop_sums_the_products_its_layout_implies(dtype, iters):
    L = _fns()
    ops = _operands(dtype, 1)
    f = ops.double().numpy()
    # fragment -> matrix: A[row][k] is lane row + 16 (k // 8), value k % 8; B[k][col] is lane col + 16 (k // 8), value k % 8
    lane = np.arange(16)[:, None] + 16 * (np.arange(32)[None, :] // 8)
    val = np.broadcast_to(np.arange(32)[None, :] % 8, (16, 32))
    A = [f[c][lane, val] for c in range(8)]                     # [16 rows][32 k]
    B = [f[8 + c][lane, val].T for c in range(8)]               # [32 k][16 cols]
    # iteration: MFMA j (0..15) multiplies a[j & 7] with b[(j + (j >> 3)) & 7] into block j & 7
    D = [A[c] @ (B[c] + B[(c + 1) & 7]) for c in range(8)]      # [16 rows][16 cols]
    expect = np.zeros(64)
    for ln in range(64):
        col, quad = ln & 15, ln >> 4
        expect[ln] = iters * sum(D[c][4 * quad + e][col] for c in range(8) for e in range(4))
    dev_ops = ops.to(DEV)
    sink = torch.full((2 * 512,), float("nan"), dtype=torch.float32, device=DEV)
    assert L.minfer_calib_mfma_rate(capi._dtype_code(dev_ops), dev_ops.data_ptr(), iters, 2, sink.data_ptr(), _stream()) == capi.OK, capi.last_error()
    got = sink.cpu().double().numpy().reshape(2, 8, 64)        # workgroup, wave, lane: every wave adds up the same
    scale = iters * sum(np.abs(A[c]) @ (np.abs(B[c]) + np.abs(B[(c + 1) & 7])) for c in range(8)).max() * 16
    assert np.abs(got - expect[None, None, :]).max() <= 1e-5 * scale


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_mfma_32x32x16_loop_sums_the_products_its_layout_implies(dtype):
    L = _fns()
    ops = _operands(dtype, 2)
    f = ops.double().numpy()
    # A[row][k] is lane row + 32 (k // 8), value k % 8 (32 rows, 16 k); B likewise by column
    lane = np.arange(32)[:, None] + 32 * (np.arange(16)[None, :] // 8)
    val = np.broadcast_to(np.arange(16)[None, :] % 8, (32, 16))
    D = [f[j][lane, val] @ f[8 + j][lane, val].T for j in range(8)]     # MFMA j multiplies a[j] with b[j] into block j & 3
    iters = 2
    expect = np.zeros(64)
    for ln in range(64):
        col, h = ln & 31, ln >> 5
        rows = [8 * (r // 4) + 4 * h + r % 4 for r in range(16)]        # result register r of a lane
        expect[ln] = iters * sum(D[j][row][col] for j in range(8) for row in rows)
    dev_ops = ops.to(DEV)
    sink = torch.full((512,), float("nan"), dtype=torch.float32, device=DEV)
    assert L.minfer_calib_mfma_rate_32x32x16(capi._dtype_code(dev_ops), dev_ops.data_ptr(), iters, 1, sink.data_ptr(), _stream()) == capi.OK, capi.last_error()
    got = sink.cpu().double().numpy().reshape(8, 64)
    scale = iters * sum(np.abs(f[j][lane, val]) @ np.abs(f[8 + j][lane, val]).T for j in range(8)).max() * 16
    assert np.abs(got - expect[None, :]).max() <= 1e-5 * scale


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("lds_reads,softmax", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_attention_mix_loop_runs_and_is_deterministic(dtype, lds_reads, softmax):
    L = _fns()
    dev_ops = _operands(dtype, 3).to(DEV)
    outs = []
    for _ in range(2):
        sink = torch.full((3 * 512,), float("nan"), dtype=torch.float32, device=DEV)
        assert L.minfer_calib_attn_mix(capi._dtype_code(dev_ops), dev_ops.data_ptr(), 4, 3, lds_reads, softmax, sink.data_ptr(), _stream()) == capi.OK, capi.last_error()
        outs.append(sink.cpu())
    assert torch.isfinite(outs[0]).all()
    assert torch.equal(outs[0], outs[1])
    w = outs[0].view(3, 8, 64)
    assert torch.equal(w[0], w[1]) and torch.equal(w[0], w[2])          # every workgroup computes the same
