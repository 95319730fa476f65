"""Reports the GPU core clock (rocm-smi) while one operator runs in a loop, next to the time per call.

    python minfer-python_amd/apps/clock_probe.py [--seconds 4]

On the MI355X boxes this was written on the core clock is 2.4 GHz when idle and drops as soon as the matrix units are
kept busy, so the published peak (which assumes 2.4 GHz) is not what a sustained kernel can reach: the numbers printed
here say what the clock was while each kernel's throughput was measured.
"""
import argparse
import json
import os
import subprocess
import sys
import threading
import time

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

import workloads  # noqa: E402
from minfer.const import GGML_QUANT_SIZES, GGMLQuantizationType  # noqa: E402
from minfer.kernels import KernelBackend  # noqa: E402

QT = GGMLQuantizationType.F16
QB, QS = GGML_QUANT_SIZES[QT]


def sclk_mhz():
    out = subprocess.run(["rocm-smi", "--showclocks", "--json"], capture_output=True, text=True, timeout=10).stdout
    card = json.loads(out)
    card = card[sorted(card)[0]]
    return int(card["sclk clock speed:"].strip("()Mhz"))


def measure(name, fn, seconds, flops=None, nbytes=None):
    samples, stop = [], threading.Event()

    def sampler():
        while not stop.is_set():
            try:
                samples.append(sclk_mhz())
            except Exception:
                pass
            time.sleep(0.25)

    for _ in range(300):
        fn()
    torch.cuda.synchronize()
    th = threading.Thread(target=sampler)
    th.start()
    t0, n = time.time(), 0
    while time.time() - t0 < seconds:
        for _ in range(200):
            fn()
        torch.cuda.synchronize()
        n += 200
    per_call = (time.time() - t0) / n
    stop.set()
    th.join()
    mid = sorted(samples[1:])[len(samples[1:]) // 2] if len(samples) > 1 else -1
    rate = f"{flops / per_call / 1e12:7.0f} TFLOP/s" if flops else f"{nbytes / per_call / 1e9:7.0f} GB/s"
    print(f"{name:34s} {per_call * 1e6:8.1f} us/call {rate}   core clock {mid} MHz (median of {len(samples) - 1} samples)", flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--seconds", type=float, default=4.0)
    args = ap.parse_args()
    kerns = KernelBackend("torch_ext")
    print(f"idle core clock {sclk_mhz()} MHz")
    q, k, v, mask = workloads.llama8b_prefill(device="cuda")
    out = torch.zeros_like(q)
    measure("flash_attn S=4096 (Llama-3-8B)", lambda: kerns.flash_attn(QT, QB, QS, q, k, v, mask, out), args.seconds,
            flops=workloads.prefill_flops(32, 128, [4096]))
    a, w, bias = workloads.gemm_input(4096, 4096, 4096, device="cuda")
    o = torch.empty_like(bias)
    measure("gemm 4096^3", lambda: kerns.gemm(QT, QB, QS, 1.0, 0.0, a, w, bias, o), args.seconds, flops=workloads.gemm_flops(4096, 4096, 4096))
    measure("torch.matmul 4096^3 (vendor library)", lambda: torch.matmul(a[0], w, out=o[0]), args.seconds, flops=workloads.gemm_flops(4096, 4096, 4096))
    qd, kc, vc, ctx = workloads.decode_cache(device="cuda")
    od = torch.zeros_like(qd)
    measure("flash_attn_decode B=64", lambda: kerns.flash_attn_decode(QT, QB, QS, qd, kc, vc, ctx, od), args.seconds,
            nbytes=workloads.decode_bytes(ctx.tolist(), 32, 8, 128))


if __name__ == "__main__":
    main()
