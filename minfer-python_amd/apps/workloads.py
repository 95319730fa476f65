"""Seeded synthetic inputs for the attention workloads that tests, benchmarks and profiles share.

Every generator draws from ``torch.Generator().manual_seed(seed)`` on the CPU (so the same seed
gives the same bytes on any machine) and returns CPU tensors unless ``device`` is given.  The
input recipes follow the reference's callers (reference: test/kernels.py:225-244,
apps/benchmark.py:215-237): q/k/v are drawn as [B, L, H*D] and handed over as the transposed
view [B, H, L, D] when ``views=True``.
"""
import torch


def _qkv(gen, B, H, L, D, scale, dtype, views):
    if views:
        x = (scale * torch.randn(B, L, H * D, generator=gen)).to(dtype)
        return x.view(B, L, H, D).transpose(1, 2)
    return (scale * torch.randn(B, H, L, D, generator=gen)).to(dtype)


def causal_mask(B, L, device="cpu"):
    i = torch.arange(L, device=device)
    return (i[None, :] <= i[:, None])[None, None].expand(B, 1, L, L).contiguous()


def window_mask(B, L, window, device="cpu"):
    i = torch.arange(L, device=device)
    return ((i[None, :] - i[:, None]).abs() < window)[None, None].expand(B, 1, L, L).contiguous()


def dense_prefill(B, Hq, Hkv, L, D, dtype, seed=0, scale=0.5, views=False, device="cpu"):
    """q [B,Hq,L,D], k/v [B,Hkv,L,D] ~ scale * N(0,1)."""
    gen = torch.Generator().manual_seed(seed)
    q = _qkv(gen, B, Hq, L, D, scale, dtype, views)
    k = _qkv(gen, B, Hkv, L, D, scale, dtype, views)
    v = _qkv(gen, B, Hkv, L, D, scale, dtype, views)
    if device != "cpu":
        if views:  # keep the strided layout on the device
            q, k, v = (t.transpose(1, 2).to(device).transpose(1, 2) for t in (q, k, v))
        else:
            q, k, v = q.to(device), k.to(device), v.to(device)
    return q, k, v


def cpu_plumbing(seed=0):
    """B=1, Hq=8, Hkv=2, S=256, D=64, fp32, N(0,1), causal."""
    q, k, v = dense_prefill(1, 8, 2, 256, 64, torch.float32, seed=seed, scale=1.0)
    return q, k, v, causal_mask(1, 256)


def llama8b_prefill(seed=0, device="cpu", views=False, L=4096):
    """B=1, Hq=32, Hkv=8, S=4096, D=128, fp16, 0.5*N(0,1), causal."""
    q, k, v = dense_prefill(1, 32, 8, L, 128, torch.float16, seed=seed, scale=0.5, views=views, device=device)
    return q, k, v, causal_mask(1, L, device=device)


def reference_test_prefill(seed=0, device="cpu", B=8, L=4096, Hq=48, Hkv=8, D=128, window=None):
    """The reference test's recipe (reference: test/kernels.py:225-244, 263-280): q ~ N(0,1), k and v ~ N(0,1)/sqrt(D),
    drawn as [B,L,H*D] fp16 and handed over as transposed [B,H,L,D] views; mask causal (case A) or, with
    ``window`` (256 there, case B), |i - j| < window."""
    gen = torch.Generator().manual_seed(seed)
    q = _qkv(gen, B, Hq, L, D, 1.0, torch.float16, True)
    k = _qkv(gen, B, Hkv, L, D, D ** -0.5, torch.float16, True)
    v = _qkv(gen, B, Hkv, L, D, D ** -0.5, torch.float16, True)
    if device != "cpu":
        q, k, v = (t.transpose(1, 2).to(device).transpose(1, 2) for t in (q, k, v))
    mask = causal_mask(B, L, device=device) if window is None else window_mask(B, L, window, device=device)
    return q, k, v, mask


def reference_benchmark_prefill(seed=0, device="cpu", B=4, L=16384, Hq=48, Hkv=8, D=128):
    """The reference benchmark's recipe (reference: apps/benchmark.py:215-237; L in 4096, 8192, 16384): q, k, v all
    ~ N(0,1)/sqrt(D) as transposed views, causal mask."""
    gen = torch.Generator().manual_seed(seed)
    q, k, v = (_qkv(gen, B, H, L, D, D ** -0.5, torch.float16, True) for H in (Hq, Hkv, Hkv))
    if device != "cpu":
        q, k, v = (t.transpose(1, 2).to(device).transpose(1, 2) for t in (q, k, v))
    return q, k, v, causal_mask(B, L, device=device)


def long_context_prefill(seed=0, device="cpu", L=32768):
    """B=1, Hq=32, Hkv=8, S=32768, D=128, bf16, 0.5*N(0,1), causal."""
    q, k, v = dense_prefill(1, 32, 8, L, 128, torch.bfloat16, seed=seed, scale=0.5, device=device)
    return q, k, v, causal_mask(1, L, device=device)


def decode_cache(seed=0, device="cpu", B=64, Hq=32, Hkv=8, Lmax=8192, D=128, dtype=torch.float16,
                 ctx_lo=512, ctx_hi=8192):
    """q [B,Hq,1,D] ~ N(0,1); caches [B,Hkv,Lmax,D] ~ N(0,1); ctx_lens uniform in [ctx_lo, ctx_hi]."""
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, 1, D, generator=gen).to(dtype)
    ctx = torch.randint(ctx_lo, ctx_hi + 1, (B,), generator=gen, dtype=torch.int32)
    if device == "cpu":
        kc = torch.randn(B, Hkv, Lmax, D, generator=gen).to(dtype)
        vc = torch.randn(B, Hkv, Lmax, D, generator=gen).to(dtype)
    else:  # the 2 GiB of cache entries are drawn on the device from the same seed
        dgen = torch.Generator(device=device).manual_seed(seed)
        kc = torch.randn(B, Hkv, Lmax, D, generator=dgen, device=device, dtype=dtype)
        vc = torch.randn(B, Hkv, Lmax, D, generator=dgen, device=device, dtype=dtype)
        q, ctx = q.to(device), ctx.to(device)
    return q, kc, vc, ctx


def q8_0_rows(x):
    """Device tensor [..., D] (D a multiple of 32) -> its rows as Q8_0 blocks, uint8 [..., D/32*34], quantised on the
    device by the library's own quantiser (reference format: common/types.hpp:141-146)."""
    from minfer.const import GGML_QUANT_SIZES, GGMLQuantizationType
    from minfer.kernels import KernelBackend
    qt = GGMLQuantizationType.Q8_0
    D = x.shape[-1]
    y = torch.empty(x.shape[:-1] + (D // 32 * 34,), dtype=torch.uint8, device=x.device)
    KernelBackend("torch_ext")._quant(qt, *GGML_QUANT_SIZES[qt], x.reshape(-1, D), y.view(-1, D // 32 * 34))
    return y


def decode_bytes_q8_0(ctx_lens, Hq, Hkv, D):
    """K and V rows of D/32 34-byte blocks read once per KV head, plus fp16 q and out."""
    B = len(ctx_lens)
    return int(sum(int(c) for c in ctx_lens)) * Hkv * (D // 32 * 34) * 2 + 2 * B * Hq * D * 2


def ragged_prefill(seed=0, device="cpu", n_seqs=16, len_lo=128, len_hi=2048, Hq=64, Hkv=8, D=128,
                   dtype=torch.float16, scale=1.0):
    """Packed sequences with lengths uniform in [len_lo, len_hi]: q [1,Hq,T,D], k/v [1,Hkv,T,D] ~ N(0,1),
    cu_seqlens int32 [n_seqs+1]."""
    gen = torch.Generator().manual_seed(seed)
    lens = torch.randint(len_lo, len_hi + 1, (n_seqs,), generator=gen)
    cu = torch.zeros(n_seqs + 1, dtype=torch.int32)
    cu[1:] = lens.cumsum(0).to(torch.int32)
    T = int(cu[-1])
    q = (scale * torch.randn(1, Hq, T, D, generator=gen)).to(dtype)
    k = (scale * torch.randn(1, Hkv, T, D, generator=gen)).to(dtype)
    v = (scale * torch.randn(1, Hkv, T, D, generator=gen)).to(dtype)
    if device != "cpu":
        q, k, v, cu = q.to(device), k.to(device), v.to(device), cu.to(device)
    return q, k, v, cu


def prefill_flops(Hq, D, lens):
    """4*D*Hq*(attended pairs) for causal sequences of the given lengths."""
    return 2 * D * Hq * sum(int(n) * (int(n) + 1) for n in lens)


def decode_bytes(ctx_lens, Hq, Hkv, D, itemsize=2):
    """K and V rows read once per KV head, plus q and out."""
    B = len(ctx_lens)
    return int(sum(int(c) for c in ctx_lens)) * Hkv * D * 2 * itemsize + 2 * B * Hq * D * itemsize


def rope_input(seed=0, device="cpu", B=8, L=4096, H=48, D=128, dtype=torch.float16):
    """x [B,L,H,D] ~ N(0,1): the shape the reference tests its rotary kernels on
    (reference: test/kernels.py:80-82; rotary_dim 64, base 1e6, start_pos 0 or 2048 there)."""
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(B, L, H, D, generator=gen).to(dtype)
    return x.to(device) if device != "cpu" else x


def kv_append(seed=0, device="cpu", B=1, L=4096, Hq=32, Hkv=8, D=128, Lmax=None, dtype=torch.float16, pos_hi=1):
    """Inputs of the rope + cache-append step at the Llama-3-8B shape: q [B,L,Hq,D], k/v [B,L,Hkv,D]
    ~ N(0,1), positions int32 [B] uniform in [0, pos_hi), zero-filled caches [B,Hkv,Lmax,D]
    (Lmax defaults to pos_hi - 1 + L, so that every row fits)."""
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(B, L, Hq, D, generator=gen).to(dtype)
    k = torch.randn(B, L, Hkv, D, generator=gen).to(dtype)
    v = torch.randn(B, L, Hkv, D, generator=gen).to(dtype)
    positions = torch.randint(0, pos_hi, (B,), generator=gen, dtype=torch.int32)
    Lmax = Lmax if Lmax is not None else pos_hi - 1 + L
    if device != "cpu":
        q, k, v, positions = q.to(device), k.to(device), v.to(device), positions.to(device)
    k_cache = torch.zeros(B, Hkv, Lmax, D, dtype=dtype, device=device)
    v_cache = torch.zeros(B, Hkv, Lmax, D, dtype=dtype, device=device)
    return q, k, v, positions, k_cache, v_cache


def rope_bytes(B, L, H, rotary_dim, itemsize=2):
    """Algorithmic HBM bytes of an in-place rotary embedding: the rotary part, read and written once."""
    return 2 * B * L * H * rotary_dim * itemsize


def kv_append_bytes(B, L, Hq, Hkv, D, rotary_dim, itemsize=2):
    """q's rotary part read and written; k and v read once; their cache rows written once."""
    return (2 * B * L * Hq * rotary_dim + 4 * B * L * Hkv * D) * itemsize


def kv_append_bytes_q8_0(B, L, Hq, Hkv, D, rotary_dim, itemsize=2):
    """As kv_append_bytes, with the cache rows written as D/32 blocks of 34 bytes."""
    return B * L * (2 * Hq * rotary_dim * itemsize + 2 * Hkv * D * itemsize + 2 * Hkv * (D // 32 * 34))


def rmsnorm_input(shape=(8, 4096, 6144), seed=0, device="cpu", dtype=torch.float16):
    """x ~ N(0,1) of `shape`, w ~ N(0,1)/sqrt(shape[-1]) (reference: test/kernels.py:60-69; its two shapes are
    (8,4096,6144) per token and (8,4096,48,128) per head)."""
    gen = torch.Generator().manual_seed(seed)
    w = ((1 / shape[-1] ** 0.5) * torch.randn(shape[-1], generator=gen)).to(dtype)
    n = 1
    for s in shape:
        n *= s
    x = torch.empty(shape, dtype=dtype)
    flat = x.view(-1)
    for lo in range(0, n, 1 << 26):          # in pieces: the fp32 staging of 2e8 elements is large
        hi = min(n, lo + (1 << 26))
        flat[lo:hi] = torch.randn(hi - lo, generator=gen).to(dtype)
    return (x.to(device), w.to(device)) if device != "cpu" else (x, w)


def rmsnorm_bytes(shape, itemsize=2):
    """Every element read once and written once, plus the weight."""
    n = 1
    for s in shape:
        n *= s
    return (2 * n + shape[-1]) * itemsize


def gemm_input(M, N, K, seed=0, device="cpu", dtype=torch.float16):
    """The reference test's recipe (reference: test/kernels.py:133-136): A [1,M,K] ~ N(0,1), weight [K,N] ~
    N(0,1)/sqrt(K), bias [1,M,N] ~ N(0,1)."""
    gen = torch.Generator().manual_seed(seed)
    a = torch.randn(1, M, K, generator=gen).to(dtype)
    w = ((1 / K ** 0.5) * torch.randn(K, N, generator=gen)).to(dtype)
    bias = torch.randn(1, M, N, generator=gen).to(dtype)
    return (a.to(device), w.to(device), bias.to(device)) if device != "cpu" else (a, w, bias)


def gemm_flops(M, N, K):
    return 2 * M * N * K
