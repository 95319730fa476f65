"""Times the attention ops against the PyTorch reference statements, one table per op.

Same command-line shape and timing method as the reference's benchmark script
(reference: apps/benchmark.py:210-290): torch.utils.benchmark.Timer.blocked_autorange per shape,
Compare(...).print(); for `--which ref` the GQA expansion of K/V is outside the timed closure.
"""
import argparse
import gc
import os
import sys

import torch
from torch.utils.benchmark import Compare, Timer

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

import workloads  # noqa: E402
from minfer.const import GGML_QUANT_SIZES, GGMLQuantizationType  # noqa: E402
from minfer.kernels import KernelBackend, refs  # noqa: E402

QT = GGMLQuantizationType.F16
QB, QS = GGML_QUANT_SIZES[QT]


def _measure(fn, sub_label, which, label):
    return Timer(stmt="fn()", globals={"fn": fn}, label=label, sub_label=sub_label, description=which).blocked_autorange()


def flash_attn(backend: str, which: str):
    """flash_attn against pytorch SDPA at the reference's shapes (B=4, 48 heads over 8 KV heads)."""
    kerns = KernelBackend(backend)
    B, Hq, Hkv, D = 4, 48, 8, 128
    results = []
    for L in [4096, 8192, 16384]:
        q, k, v = workloads.dense_prefill(B, Hq, Hkv, L, D, torch.float16, scale=D ** -0.5, views=True, device="cuda")
        mask = workloads.causal_mask(B, L, device="cuda")
        out = torch.zeros((B, Hq, L, D), dtype=torch.float16, device="cuda")
        if which == "minfer":
            fn = lambda: kerns.flash_attn(QT, QB, QS, q, k, v, mask, out)
        else:
            k_exp, v_exp = k.repeat_interleave(Hq // Hkv, dim=1), v.repeat_interleave(Hq // Hkv, dim=1)
            fn = lambda: refs.flash_attn(q, k_exp, v_exp, mask)
        results.append(_measure(fn, f"B={B}, L={L}, n_heads={Hq}, n_kv_heads={Hkv}, head_dim={D}", which, "flash_attn"))
        del q, k, v, mask, out
        gc.collect()
        torch.cuda.empty_cache()
    Compare(results).print()


def flash_attn_decode(backend: str, which: str):
    kerns = KernelBackend(backend)
    results = []
    for B in [16, 64]:
        q, kc, vc, ctx = workloads.decode_cache(device="cuda", B=B)
        out = torch.zeros_like(q)
        if which == "minfer":
            fn = lambda: kerns.flash_attn_decode(QT, QB, QS, q, kc, vc, ctx, out)
        else:
            k_exp, v_exp = kc.repeat_interleave(4, dim=1), vc.repeat_interleave(4, dim=1)
            fn = lambda: refs.flash_attn_decode(q, k_exp, v_exp, ctx)
        results.append(_measure(fn, f"B={B}, ctx~U[512,8192], n_heads=32, n_kv_heads=8, head_dim=128", which, "flash_attn_decode"))
        del q, kc, vc, out
        gc.collect()
        torch.cuda.empty_cache()
    Compare(results).print()


def flash_attn_varlen(backend: str, which: str):
    kerns = KernelBackend(backend)
    q, k, v, cu = workloads.ragged_prefill(device="cuda")
    out = torch.zeros_like(q)
    max_len = int((cu[1:] - cu[:-1]).max())
    if which == "minfer":
        fn = lambda: kerns.flash_attn_varlen(QT, QB, QS, q, k, v, cu, max_len, out)
    else:
        k_exp, v_exp = k.repeat_interleave(8, dim=1), v.repeat_interleave(8, dim=1)
        fn = lambda: refs.flash_attn_varlen(q, k_exp, v_exp, cu)
    Compare([_measure(fn, f"16 seqs, T={q.shape[2]}, n_heads=64, n_kv_heads=8, head_dim=128", which, "flash_attn_varlen")]).print()


if __name__ == "__main__":
    KERNELS = {"flash_attn": flash_attn, "flash_attn_decode": flash_attn_decode, "flash_attn_varlen": flash_attn_varlen}
    parser = argparse.ArgumentParser()
    parser.add_argument("--backend", choices=["torch_ext"], default="torch_ext")
    parser.add_argument("--kernel", choices=sorted(KERNELS), required=True)
    parser.add_argument("--which", choices=["minfer", "ref"], required=True)
    args = parser.parse_args()
    KERNELS[args.kernel](backend=args.backend, which=args.which)
