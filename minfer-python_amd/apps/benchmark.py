"""Times the ops of the attention path against the PyTorch reference statements, one table per op.

Same command-line shape, test cases and timing method as the reference's benchmark script
(reference: apps/benchmark.py:18-290): torch.utils.benchmark.Timer.blocked_autorange per shape,
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


def flash_attn_operand_data(backend: str, which: str):
    """The prefill kernel on one shape (B=1, 32 heads over 8 KV heads, L=8192) with random and with constant operands,
    fp16 and bf16: the instruction stream is the same in all cases, so any difference is what the values cost the
    chip in power (the matrix units switch less on constant data) and the clock it can then hold."""
    kerns = KernelBackend(backend)
    B, Hq, Hkv, L, D = 1, 32, 8, 8192, 128
    mask = workloads.causal_mask(B, L, device="cuda")
    results = []
    for dtype, qt in ((torch.float16, GGMLQuantizationType.F16), (torch.bfloat16, GGMLQuantizationType.BF16)):
        qb, qs = GGML_QUANT_SIZES[qt]
        q, k, v = workloads.dense_prefill(B, Hq, Hkv, L, D, dtype, scale=0.5, device="cuda")
        for name, (qq, kk, vv) in (("N(0, 0.5)", (q, k, v)),
                                   ("all 0.25", (torch.full_like(q, 0.25), torch.full_like(k, 0.25), torch.full_like(v, 0.25))),
                                   ("all 0", (torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)))):
            out = torch.zeros_like(q)
            if which == "minfer":
                fn = lambda: kerns.flash_attn(qt, qb, qs, qq, kk, vv, mask, out)
            else:
                k_exp, v_exp = kk.repeat_interleave(Hq // Hkv, dim=1), vv.repeat_interleave(Hq // Hkv, dim=1)
                fn = lambda: refs.flash_attn(qq, k_exp, v_exp, mask)
            results.append(_measure(fn, f"L={L}, {str(dtype).split('.')[-1]}, operands {name}", which, "flash_attn"))
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


def _table(label, cases, make, which):
    """One Timer row per case; make(case) returns (sub_label, minfer closure, ref closure)."""
    results = []
    for case in cases:
        sub_label, mine, ref = make(case)
        with torch.no_grad():
            results.append(_measure(mine if which == "minfer" else ref, sub_label, which, label))
        del mine, ref
        gc.collect()
        torch.cuda.empty_cache()
    Compare(results).print()


def flash_attn_decode_q8_0(backend: str, which: str):
    """Decode over Q8_0 caches; `ref` is the fp16 decode op over the dequantised caches."""
    kerns = KernelBackend(backend)
    q8 = GGMLQuantizationType.Q8_0

    def make(B):
        q, kc, vc, ctx = workloads.decode_cache(device="cuda", B=B)
        out = torch.zeros_like(q)
        kq, vq = workloads.q8_0_rows(kc), workloads.q8_0_rows(vc)
        return (f"B={B}, ctx~U[512,8192], n_heads=32, n_kv_heads=8, head_dim=128",
                lambda: kerns.flash_attn_decode(q8, *GGML_QUANT_SIZES[q8], q, kq, vq, ctx, out),
                lambda: kerns.flash_attn_decode(QT, QB, QS, q, kc, vc, ctx, out))
    _table("flash_attn_decode_q8_0", [16, 64], make, which)


def rmsnorm(backend: str, which: str):
    """The reference's cases (reference: apps/benchmark.py:23-32): per token and per head, L = 1024..16384."""
    kerns = KernelBackend(backend)

    def make(case):
        B, L, shape, eps = case
        x = torch.randn((B, L, *shape), dtype=torch.float16, device="cuda")
        w = shape[-1] ** -0.5 * torch.randn(shape[-1], dtype=torch.float16, device="cuda")
        out = torch.zeros_like(x)
        what = f"hidden_dim={shape[-1]}" if len(shape) == 1 else f"n_heads={shape[0]}, head_dim={shape[1]}"
        return f"B={B}, L={L}, {what}", lambda: kerns.rmsnorm(eps, x, w, out), lambda: refs.rmsnorm(x, w, eps)
    _table("rmsnorm", [(8, L, shape, 1e-6) for shape in ((6144,), (48, 128)) for L in (1024, 4096, 8192, 16384)], make, which)


def _rope(name, backend, which):
    """The reference's cases (reference: apps/benchmark.py:74-79, :118-123): x [8, L, 48, 128], rotary 64, base 1e6."""
    kerns = KernelBackend(backend)

    def make(L):
        x = torch.randn((8, L, 48, 128), dtype=torch.float16, device="cuda")
        return (f"B=8, L={L}, n_heads=48, head_dim=128, rotary_dim=64",
                lambda: getattr(kerns, name)(64, 0, 1e6, x), lambda: getattr(refs, name)(x, 64, 0, 1e6))
    _table(name, [1024, 4096, 8192, 16384], make, which)


def il_rope(backend: str, which: str):
    _rope("il_rope", backend, which)


def neox_rope(backend: str, which: str):
    _rope("neox_rope", backend, which)


def rope_kv_append(backend: str, which: str):
    """The fused producer at the Llama-3-8B head shape, into fp16 and into Q8_0 caches; `ref` is the statements it
    replaces (rope q, rope k, two transposed copies)."""
    kerns = KernelBackend(backend)

    def make(case):
        L, q8 = case
        q, k, v, pos, kc, vc = workloads.kv_append(device="cuda", B=8, L=L)
        if q8:
            kc = torch.zeros(kc.shape[:-1] + (kc.shape[-1] // 32 * 34,), dtype=torch.uint8, device="cuda")
            vc = torch.zeros_like(kc)

        def ref():
            refs.neox_rope(q, 128, 0, 5e5)
            rk = refs.neox_rope(k, 128, 0, 5e5).transpose(1, 2)
            if q8:
                rk, rv = workloads.q8_0_rows(rk.contiguous()), workloads.q8_0_rows(v.transpose(1, 2).contiguous())
                kc[:, :, :L], vc[:, :, :L] = rk, rv
            else:
                kc[:, :, :L], vc[:, :, :L] = rk, v.transpose(1, 2)
        return (f"B=8, L={L}, n_heads=32, n_kv_heads=8, head_dim=128, {'Q8_0' if q8 else 'fp16'} caches",
                lambda: kerns.rope_kv_append(1, 128, 5e5, q, k, v, pos, kc, vc), ref)
    _table("rope_kv_append", [(L, q8) for q8 in (False, True) for L in (1024, 4096)], make, which)


def gemm(backend: str, which: str):
    """The reference's cases (reference: apps/benchmark.py:164-166): M = K = N = 512..8192, four (alpha, beta)."""
    kerns = KernelBackend(backend)

    def make(case):
        s, alpha, beta = case
        a, w, bias = workloads.gemm_input(s, s, s, device="cuda")
        out = torch.zeros_like(bias)
        return (f"alpha={alpha}, beta={beta}, M={s}, K={s}, N={s}",
                lambda: kerns.gemm(QT, QB, QS, alpha, beta, a, w, bias, out),
                lambda: refs.gemm(a[0], w, bias[0], out[0], alpha, beta))
    _table("gemm", [(s, al, be) for s in (512, 1024, 2048, 4096, 8192) for al, be in ((1.0, 0.0), (1.0, 1.0), (2.0, 3.0), (0.5, 2.0))],
           make, which)


def mfma_rate(backend: str, which: str):
    """Calibration, not an operator: the rate the chip sustains on v_mfma_f32_16x16x32 alone, the instruction the prefill
    and GEMM kernels use, and on v_mfma_f32_32x32x16 (two waves per SIMD on every compute unit, nothing else in the
    loop), for random, constant and zero operand values, fp16 and bf16.  `ref` runs torch.matmul (the vendor library) at
    8192^3 for comparison.  The nominal dense peak is 2500 TFLOP/s."""
    import calibration
    if which == "minfer":
        print(f"{'instruction':<22}{'dtype':<10}{'operands':<12}{'TFLOP/s':>10}{'of 2500':>10}   (launches of ~5 ms back to back, 200 ms timed after 150 ms of warm-up)")
        for shape32 in (False, True):
            for dtype in (torch.float16, torch.bfloat16):
                for kind in ("random", "constant", "zero"):
                    r = calibration.mfma_rate(dtype, kind, shape32=shape32)
                    print(f"{r['instruction']:<22}{r['dtype']:<10}{kind:<12}{r['tflops']:>10.1f}{r['tflops'] / 2500.0:>10.3f}")
        # the prefill kernel's per-tile instruction mix without any memory traffic, barrier or bookkeeping: what each kind
        # of co-running work costs the matrix rate, and what a kernel with no fixed cost at all would reach
        print(f"{'dtype':<10}{'operands':<12}{'fragments':<12}{'softmax':<10}{'TFLOP/s':>10}{'of 2500':>10}   (64 MFMAs of 16x16x32 per wave and 64-key tile, head_dim 128)")
        for dtype in (torch.float16, torch.bfloat16):
            for kind in ("random", "zero"):
                for lds_reads, softmax in ((False, False), (True, False), (False, True), (True, True)):
                    r = calibration.attn_mix_rate(dtype, kind, lds_reads, softmax)
                    print(f"{r['dtype']:<10}{kind:<12}{'from LDS' if lds_reads else 'registers':<12}{'yes' if softmax else 'no':<10}{r['tflops']:>10.1f}{r['tflops'] / 2500.0:>10.3f}")
    else:
        results = []
        for dtype in (torch.float16, torch.bfloat16):
            a = (0.5 * torch.randn(8192, 8192, device="cuda")).to(dtype)
            b = (0.5 * torch.randn(8192, 8192, device="cuda")).to(dtype)
            results.append(_measure(lambda: torch.matmul(a, b), f"torch.matmul 8192^3 {str(dtype).split('.')[-1]} (1.0995e12 flop)", which, "mfma_rate"))
        Compare(results).print()


if __name__ == "__main__":
    KERNELS = {"mfma_rate": mfma_rate, "flash_attn": flash_attn, "flash_attn_operand_data": flash_attn_operand_data, "flash_attn_decode": flash_attn_decode, "flash_attn_varlen": flash_attn_varlen,
               "flash_attn_decode_q8_0": flash_attn_decode_q8_0, "rmsnorm": rmsnorm, "il_rope": il_rope, "neox_rope": neox_rope,
               "rope_kv_append": rope_kv_append, "gemm": gemm}
    parser = argparse.ArgumentParser()
    parser.add_argument("--backend", choices=["torch_ext"], default="torch_ext")
    parser.add_argument("--kernel", choices=sorted(KERNELS), required=True)
    parser.add_argument("--which", choices=["minfer", "ref"], required=True)
    args = parser.parse_args()
    KERNELS[args.kernel](backend=args.backend, which=args.which)
