"""Calibration measurements next to the operator benchmarks: what the chip sustains on the matrix instruction
alone.  Calls the library's calibration entry point (include/minfer_attn.h: minfer_calib_mfma_rate) through ctypes;
it is not an operator and has no counterpart in the reference."""
import ctypes
import os

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(HERE), "lib", "libminfer_attn.so")
DTYPE_CODE = {torch.float16: 1, torch.bfloat16: 30}
OPERAND_BYTES = 16384
FLOP_PER_ITER = 8 * 8 * 32768     # per workgroup, minfer_calib_mfma_rate (and _32x32x16)
MIX_FLOP_PER_ITER = 8 * 32 * 32768  # per workgroup, minfer_calib_attn_mix (one 64-key tile per wave)

_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is not built; run python minfer-python_amd/build.py")
        _lib = ctypes.CDLL(LIB_PATH)
        for fn in (_lib.minfer_calib_mfma_rate, _lib.minfer_calib_mfma_rate_32x32x16):
            fn.restype = ctypes.c_int
            fn.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
        _lib.minfer_calib_attn_mix.restype = ctypes.c_int
        _lib.minfer_calib_attn_mix.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                               ctypes.c_void_p, ctypes.c_void_p]
        _lib.minfer_attn_last_error.restype = ctypes.c_char_p
    return _lib


def mfma_operands(dtype, kind: str, device="cuda", seed=0):
    """16 KiB of operand fragments: 'random' = 0.5 * N(0,1) (the value distribution of the prefill benchmarks),
    'constant' = every element 0.25, 'zero'."""
    n = OPERAND_BYTES // 2
    if kind == "random":
        g = torch.Generator().manual_seed(seed)
        return (0.5 * torch.randn(n, generator=g)).to(dtype).to(device)
    if kind == "constant":
        return torch.full((n,), 0.25, dtype=dtype, device=device)
    if kind == "zero":
        return torch.zeros(n, dtype=dtype, device=device)
    raise ValueError(f"unknown operand kind {kind}")


def launch_mfma_rate(operands, iters: int, workgroups: int, sink, shape32: bool = False):
    fn = _load().minfer_calib_mfma_rate_32x32x16 if shape32 else _load().minfer_calib_mfma_rate
    rc = fn(DTYPE_CODE[operands.dtype], operands.data_ptr(), iters, workgroups, sink.data_ptr(),
            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    if rc != 0:
        raise RuntimeError(_load().minfer_attn_last_error().decode())


def launch_attn_mix(operands, iters: int, workgroups: int, lds_reads: bool, softmax: bool, sink):
    rc = _load().minfer_calib_attn_mix(DTYPE_CODE[operands.dtype], operands.data_ptr(), iters, workgroups, int(lds_reads), int(softmax),
                                       sink.data_ptr(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    if rc != 0:
        raise RuntimeError(_load().minfer_attn_last_error().decode())


def _sustained(launch, flop_per_iter, first_iters, timed_ms, prewarm_ms, device):
    wgs = torch.cuda.get_device_properties(0).multi_processor_count
    sink = torch.empty(wgs * 512, dtype=torch.float32, device=device)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    iters = first_iters
    launch(iters, wgs, sink)
    a.record(); launch(iters, wgs, sink); b.record(); b.synchronize()
    iters = max(50, int(iters * 5.0 / max(a.elapsed_time(b), 1e-3)))          # ~5 ms per launch
    per_launch_ms = 5.0
    for _ in range(max(1, int(prewarm_ms / per_launch_ms))):
        launch(iters, wgs, sink)
    n = max(1, int(timed_ms / per_launch_ms))
    a.record()
    for _ in range(n):
        launch(iters, wgs, sink)
    b.record(); b.synchronize()
    ms = a.elapsed_time(b) / n
    flop = float(wgs) * iters * flop_per_iter
    return {"tflops": flop / (ms * 1e-3) / 1e12, "ms_per_launch": ms, "iters": iters, "workgroups": wgs, "launches": n}


def mfma_rate(dtype=torch.float16, kind="random", timed_ms=200.0, prewarm_ms=150.0, device="cuda", shape32=False):
    """Sustained rate of v_mfma_f32_16x16x32 (shape32: v_mfma_f32_32x32x16) on the whole chip, TFLOP/s: one workgroup of 8
    waves per compute unit, launches of ~5 ms run back to back for `prewarm_ms` (the clocks settle), then for `timed_ms`
    between two events."""
    ops = mfma_operands(dtype, kind, device)
    r = _sustained(lambda iters, wgs, sink: launch_mfma_rate(ops, iters, wgs, sink, shape32), FLOP_PER_ITER, 2000, timed_ms, prewarm_ms, device)
    r.update({"operands": kind, "dtype": str(dtype).replace("torch.", ""), "instruction": "v_mfma_f32_32x32x16" if shape32 else "v_mfma_f32_16x16x32"})
    return r


def attn_mix_rate(dtype=torch.float16, kind="random", lds_reads=True, softmax=True, timed_ms=200.0, prewarm_ms=150.0, device="cuda"):
    """Sustained rate of the prefill kernel's per-tile instruction mix (head_dim 128) with no memory traffic, barrier or
    bookkeeping in the loop (minfer_calib_attn_mix), TFLOP/s of its MFMAs; measured like mfma_rate."""
    ops = mfma_operands(dtype, kind, device)
    r = _sustained(lambda iters, wgs, sink: launch_attn_mix(ops, iters, wgs, lds_reads, softmax, sink), MIX_FLOP_PER_ITER, 500,
                   timed_ms, prewarm_ms, device)
    r.update({"operands": kind, "dtype": str(dtype).replace("torch.", ""), "lds_reads": lds_reads, "softmax": softmax})
    return r
