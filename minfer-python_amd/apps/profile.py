"""One un-timed call of an op of the attention path, for an external profiler, e.g.

    rocprofv3 --kernel-trace --stats --output-format csv -- python minfer-python_amd/apps/profile.py --kernel flash_attn --which minfer
    rocprofv3 --pmc SQ_INSTS_VALU_MFMA_MOPS_F16 SQ_BUSY_CYCLES -- python minfer-python_amd/apps/profile.py --kernel flash_attn --which minfer

Same command-line shape as the reference's profiling script (reference: apps/profile.py:96-143);
`--workload` chooses between the reference's own shape and the shapes the benchmarks use.
"""
import argparse
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)

import workloads  # noqa: E402
from minfer.const import GGML_QUANT_SIZES, GGMLQuantizationType  # noqa: E402
from minfer.kernels import KernelBackend, refs  # noqa: E402

QT = GGMLQuantizationType.F16
QB, QS = GGML_QUANT_SIZES[QT]


def flash_attn(backend: str, which: str, workload: str, repeat: int):
    kerns = KernelBackend(backend)
    if workload == "reference":   # reference: apps/profile.py:98 (B=4, L=4096, 48 heads over 8 KV heads)
        B, L, Hq, Hkv, D = 4, 4096, 48, 8, 128
        q, k, v = workloads.dense_prefill(B, Hq, Hkv, L, D, torch.float16, scale=1.0, views=True, device="cuda")
        mask = workloads.causal_mask(B, L, device="cuda")
    elif workload == "long":
        q, k, v, mask = workloads.long_context_prefill(device="cuda")
    else:
        q, k, v, mask = workloads.llama8b_prefill(device="cuda")
    out = torch.zeros(q.shape, dtype=q.dtype, device="cuda")
    n_rep = q.shape[1] // k.shape[1]
    if which == "minfer":
        fn = lambda: kerns.flash_attn(QT, QB, QS, q, k, v, mask, out)
    else:
        k_exp, v_exp = k.repeat_interleave(n_rep, dim=1), v.repeat_interleave(n_rep, dim=1)
        fn = lambda: refs.flash_attn(q, k_exp, v_exp, mask)
    with torch.no_grad():
        for _ in range(repeat):
            fn()
    torch.cuda.synchronize()


def flash_attn_decode(backend: str, which: str, workload: str, repeat: int):
    kerns = KernelBackend(backend)
    q, kc, vc, ctx = workloads.decode_cache(device="cuda")
    out = torch.zeros_like(q)
    if which == "minfer":
        fn = lambda: kerns.flash_attn_decode(QT, QB, QS, q, kc, vc, ctx, out)
    else:
        n_rep = q.shape[1] // kc.shape[1]
        fn = lambda: [refs.flash_attn_decode(q[b:b + 1], kc[b:b + 1].repeat_interleave(n_rep, 1),
                                             vc[b:b + 1].repeat_interleave(n_rep, 1), ctx[b:b + 1]) for b in range(q.shape[0])]
    with torch.no_grad():
        for _ in range(repeat):
            fn()
    torch.cuda.synchronize()


def flash_attn_decode_q8_0(backend: str, which: str, workload: str, repeat: int):
    """The decode workload over Q8_0 caches (quantised on the device from the same fp16 caches); `ref` attends the
    dequantised caches with the fp16 decode op."""
    kerns = KernelBackend(backend)
    q, kc, vc, ctx = workloads.decode_cache(device="cuda")
    out = torch.zeros_like(q)
    q8 = GGMLQuantizationType.Q8_0
    kq, vq = workloads.q8_0_rows(kc), workloads.q8_0_rows(vc)
    if which == "minfer":
        del kc, vc
        fn = lambda: kerns.flash_attn_decode(q8, *GGML_QUANT_SIZES[q8], q, kq, vq, ctx, out)
    else:
        k16, v16 = torch.empty_like(kc), torch.empty_like(vc)
        kerns._dequant(q8, *GGML_QUANT_SIZES[q8], kq.view(-1, kq.shape[-1]), k16.view(-1, 128))
        kerns._dequant(q8, *GGML_QUANT_SIZES[q8], vq.view(-1, vq.shape[-1]), v16.view(-1, 128))
        fn = lambda: kerns.flash_attn_decode(QT, QB, QS, q, k16, v16, ctx, out)
    with torch.no_grad():
        for _ in range(repeat):
            fn()
    torch.cuda.synchronize()


def flash_attn_varlen(backend: str, which: str, workload: str, repeat: int):
    kerns = KernelBackend(backend)
    q, k, v, cu = workloads.ragged_prefill(device="cuda")
    out = torch.zeros_like(q)
    max_len = int((cu[1:] - cu[:-1]).max())
    if which == "minfer":
        fn = lambda: kerns.flash_attn_varlen(QT, QB, QS, q, k, v, cu, max_len, out)
    else:
        n_rep = q.shape[1] // k.shape[1]
        k_exp, v_exp = k.repeat_interleave(n_rep, dim=1), v.repeat_interleave(n_rep, dim=1)
        fn = lambda: refs.flash_attn_varlen(q, k_exp, v_exp, cu)
    with torch.no_grad():
        for _ in range(repeat):
            fn()
    torch.cuda.synchronize()


def il_rope(backend: str, which: str, workload: str, repeat: int):
    """The reference test's shape (reference: test/kernels.py:80): x [8,4096,48,128], rotary 64, base 1e6."""
    kerns = KernelBackend(backend)
    x = workloads.rope_input(device="cuda")
    fn = (lambda: kerns.il_rope(64, 2048, 1e6, x)) if which == "minfer" else (lambda: refs.il_rope(x, 64, 2048, 1e6))
    for _ in range(repeat):
        fn()
    torch.cuda.synchronize()


def rope_kv_append(backend: str, which: str, workload: str, repeat: int):
    """NeoX rope(q), rope(k) -> cache, v -> cache at the Llama-3-8B head shape, B=8, L=4096."""
    kerns = KernelBackend(backend)
    q, k, v, pos, kc, vc = workloads.kv_append(device="cuda", B=8, L=4096)
    if which == "minfer":
        fn = lambda: kerns.rope_kv_append(1, 128, 5e5, q, k, v, pos, kc, vc)
    else:
        def fn():
            refs.neox_rope(q, 128, 0, 5e5)
            kc[:, :, :4096] = refs.neox_rope(k, 128, 0, 5e5).transpose(1, 2)
            vc[:, :, :4096] = v.transpose(1, 2)
    for _ in range(repeat):
        fn()
    torch.cuda.synchronize()


def rope_kv_append_q8_0(backend: str, which: str, workload: str, repeat: int):
    """rope_kv_append at the same shape into Q8_0 caches."""
    kerns = KernelBackend(backend)
    q, k, v, pos, kc, vc = workloads.kv_append(device="cuda", B=8, L=4096)
    kq = torch.zeros(kc.shape[:-1] + (kc.shape[-1] // 32 * 34,), dtype=torch.uint8, device="cuda")
    vq = torch.zeros_like(kq)
    if which == "minfer":
        fn = lambda: kerns.rope_kv_append(1, 128, 5e5, q, k, v, pos, kq, vq)
    else:
        q8 = GGMLQuantizationType.Q8_0

        def fn():
            kerns.rope_kv_append(1, 128, 5e5, q, k, v, pos, kc, vc)
            kerns._quant(q8, *GGML_QUANT_SIZES[q8], kc.view(-1, 128), kq.view(-1, kq.shape[-1]))
            kerns._quant(q8, *GGML_QUANT_SIZES[q8], vc.view(-1, 128), vq.view(-1, vq.shape[-1]))
    for _ in range(repeat):
        fn()
    torch.cuda.synchronize()


def rope_kv_append_norm(backend: str, which: str, workload: str, repeat: int):
    """rope_kv_append at the same shape with the per-head RMSNorm of q and k in front (the models whose attention
    normalises q and k per head: reference src/minfer/core.py:134-141); `ref` is the three separate steps."""
    kerns = KernelBackend(backend)
    q, k, v, pos, kc, vc = workloads.kv_append(device="cuda", B=8, L=4096)
    wq = torch.ones(128, dtype=q.dtype, device="cuda")
    wk = torch.ones(128, dtype=q.dtype, device="cuda")
    if which == "minfer":
        fn = lambda: kerns.rope_kv_append_norm(1, 128, 5e5, 1e-6, q, k, v, wq, wk, pos, kc, vc)
    else:
        def fn():
            kerns.rmsnorm(1e-6, q, wq, q)
            kerns.rmsnorm(1e-6, k, wk, k)
            kerns.rope_kv_append(1, 128, 5e5, q, k, v, pos, kc, vc)
    for _ in range(repeat):
        fn()
    torch.cuda.synchronize()


def quant(backend: str, which: str, workload: str, repeat: int):
    """The reference test's larger shape (reference: test/kernels.py:25): fp32 [16384, 6144] into Q8_0 rows and back."""
    kerns = KernelBackend(backend)
    q8 = GGMLQuantizationType.Q8_0
    x = torch.randn(16384, 6144, device="cuda")
    y = torch.empty(16384, 6144 // 32 * 34, dtype=torch.uint8, device="cuda")
    back = torch.empty_like(x)
    for _ in range(repeat):
        kerns._quant(q8, *GGML_QUANT_SIZES[q8], x, y)
        kerns._dequant(q8, *GGML_QUANT_SIZES[q8], y, back)
    torch.cuda.synchronize()


def rmsnorm(backend: str, which: str, workload: str, repeat: int):
    """The reference test's shapes (reference: test/kernels.py:60-63): per token [8,4096,6144] (default) or,
    with --workload reference, per head [8,4096,48,128]."""
    kerns = KernelBackend(backend)
    x, w = workloads.rmsnorm_input((8, 4096, 48, 128) if workload == "reference" else (8, 4096, 6144), device="cuda")
    out = torch.empty_like(x)
    fn = (lambda: kerns.rmsnorm(1e-6, x, w, out)) if which == "minfer" else (lambda: refs.rmsnorm(x, w, 1e-6))
    for _ in range(repeat):
        fn()
    torch.cuda.synchronize()


def gemm(backend: str, which: str, workload: str, repeat: int):
    """M=K=N=4096, alpha 1, beta 0: a size of the reference's published HGEMM table (reference: README.md:84-109)."""
    kerns = KernelBackend(backend)
    a, w, bias = workloads.gemm_input(4096, 4096, 4096, device="cuda")
    out = torch.empty_like(bias)
    fn = (lambda: kerns.gemm(QT, QB, QS, 1.0, 0.0, a, w, bias, out)) if which == "minfer" else (lambda: refs.gemm(a[0], w, bias[0], out[0], 1.0, 0.0))
    for _ in range(repeat):
        fn()
    torch.cuda.synchronize()


DECODE_TOKENS = 64   # --tokens


def gemm_decode(backend: str, which: str, workload: str, repeat: int):
    """A batch of decode tokens (64 unless --tokens says otherwise) against an fp16 weight stored [N, K]:
    x [1,tokens,4096], W [14336,4096] (Llama-3-8B FFN up)."""
    kerns = KernelBackend(backend)
    w = workloads.gemm_input(16, 14336, 4096, seed=3, device="cuda")[1].t().contiguous()
    x = workloads.gemm_input(DECODE_TOKENS, 16, 4096, seed=5, device="cuda")[0]
    out = torch.zeros(1, DECODE_TOKENS, 14336, dtype=torch.float16, device="cuda")
    fn = (lambda: kerns.gemm(QT, QB, QS, 1.0, 0.0, x, w, out, out)) if which == "minfer" else (lambda: torch.matmul(x, w.t(), out=out))
    for _ in range(repeat):
        fn()
    torch.cuda.synchronize()


def qkv(backend: str, which: str, workload: str, repeat: int):
    """The Llama-3-8B QKV projection of a 4096-token prefill: x [1,4096,4096], wq [4096,4096], wk and wv [1024,4096];
    `ref` is three separate gemm calls."""
    kerns = KernelBackend(backend)
    x, w, _ = workloads.gemm_input(4096, 4096, 4096, device="cuda")
    wq = w.t().contiguous()
    wk, wv = wq[:1024].clone(), wq[1024:2048].clone()
    qo = torch.empty(1, 4096, 4096, dtype=x.dtype, device="cuda")
    ko = torch.empty(1, 4096, 1024, dtype=x.dtype, device="cuda")
    vo = torch.empty_like(ko)
    if which == "minfer":
        fn = lambda: kerns.qkv(QT, QT, QT, QB, QB, QB, QS, QS, QS, x, wq, wk, wv, qo, ko, vo)
    else:
        def fn():
            for wt, o in ((wq, qo), (wk, ko), (wv, vo)):
                kerns.gemm(QT, QB, QS, 1.0, 0.0, x, wt, o, o)
    for _ in range(repeat):
        fn()
    torch.cuda.synchronize()


def gemm_q8_0(backend: str, which: str, workload: str, repeat: int):
    """A decode step's projection against a weight kept as Q8_0 blocks: one token x [1,1,4096] against W uint8
    [14336, 4352] (Llama-3-8B FFN up; the reference routes this case to an empty launcher, gemm/op.cuh:199-210).
    `ref` multiplies with the dequantised fp16 weight."""
    kerns = KernelBackend(backend)
    q8 = GGMLQuantizationType.Q8_0
    wf = workloads.gemm_input(16, 14336, 4096, seed=3, device="cuda")[1].t().contiguous()
    wq8 = torch.empty(14336, 4096 // 32 * 34, dtype=torch.uint8, device="cuda")
    kerns._quant(q8, *GGML_QUANT_SIZES[q8], wf, wq8)
    x = workloads.gemm_input(1, 16, 4096, seed=4, device="cuda")[0]
    out = torch.zeros(1, 1, 14336, dtype=torch.float16, device="cuda")
    if which == "minfer":
        fn = lambda: kerns.gemm(q8, *GGML_QUANT_SIZES[q8], 1.0, 0.0, x, wq8, out, out)
    else:
        fn = lambda: kerns.gemm(QT, QB, QS, 1.0, 0.0, x, wf, out, out)
    for _ in range(repeat):
        fn()
    torch.cuda.synchronize()


def copy(backend: str, which: str, workload: str, repeat: int):
    """A plain device-to-device copy of 1 GiB: the known-size kernel that HBM byte counters
    (FETCH_SIZE / WRITE_SIZE) are calibrated against."""
    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
    dst = torch.empty_like(src)
    for _ in range(repeat):
        dst.copy_(src)
    torch.cuda.synchronize()


def mfma_rate(backend: str, which: str, workload: str, repeat: int):
    """Calibration like `copy`: the library's matrix-instruction-only loop (v_mfma_f32_16x16x32_f16, two waves per SIMD
    on every compute unit), ~5 ms per launch, on random operand values (--workload reference: constant ones).  The
    kernel's duration in a trace, or MFMA counters over it, give the rate the matrix pipes sustain when nothing else
    runs: 256 workgroups x 8 waves x 16 x iters instructions of 16 384 flop."""
    import calibration
    ops = calibration.mfma_operands(torch.float16, "constant" if workload == "reference" else "random")
    wgs = torch.cuda.get_device_properties(0).multi_processor_count
    sink = torch.empty(wgs * 512, dtype=torch.float32, device="cuda")
    iters = 40000
    print(f"mfma_rate: {wgs} workgroups x {iters} iterations = {wgs * iters * calibration.FLOP_PER_ITER:.4e} flop per launch")
    for _ in range(repeat):
        calibration.launch_mfma_rate(ops, iters, wgs, sink)
    torch.cuda.synchronize()


if __name__ == "__main__":
    KERNELS = {"mfma_rate": mfma_rate, "gemm_q8_0": gemm_q8_0, "flash_attn": flash_attn, "flash_attn_decode": flash_attn_decode, "flash_attn_varlen": flash_attn_varlen,
               "flash_attn_decode_q8_0": flash_attn_decode_q8_0, "il_rope": il_rope, "rope_kv_append": rope_kv_append,
               "rope_kv_append_q8_0": rope_kv_append_q8_0, "rope_kv_append_norm": rope_kv_append_norm, "qkv": qkv, "quant": quant, "rmsnorm": rmsnorm, "gemm": gemm, "gemm_decode": gemm_decode, "copy": copy}
    parser = argparse.ArgumentParser()
    parser.add_argument("--backend", choices=["torch_ext"], default="torch_ext")
    parser.add_argument("--kernel", choices=sorted(KERNELS), required=True)
    parser.add_argument("--which", choices=["minfer", "ref"], required=True)
    parser.add_argument("--workload", choices=["llama8b", "reference", "long"], default="llama8b")
    parser.add_argument("--repeat", type=int, default=1)
    parser.add_argument("--tokens", type=int, default=64, help="gemm_decode: rows of the activation matrix (1-64 take the stripe kernel)")
    args = parser.parse_args()
    DECODE_TOKENS = args.tokens
    KERNELS[args.kernel](args.backend, args.which, args.workload, args.repeat)
