"""PyTorch statements of what each attention op computes, for callers that want to compare or
time against them the way the reference's apps do (reference: src/minfer/kernels/refs.py:53-55,
apps/benchmark.py:240-248).  Nothing in the operator path calls these."""
import torch
import torch.nn.functional as F


def flash_attn(Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """SDPA with a bool mask (True = attend).  Q/K/V: (B, n_heads, L, head_dim); K/V must already be
    expanded to n_heads for GQA (``repeat_interleave(n_rep, dim=1)``)."""
    return F.scaled_dot_product_attention(Q, K, V, attn_mask=mask)


def flash_attn_decode(Q: torch.Tensor, K_cache: torch.Tensor, V_cache: torch.Tensor, ctx_lens: torch.Tensor) -> torch.Tensor:
    """Q: (B, n_heads, 1, head_dim); caches (B, n_heads, Lmax, head_dim), pre-expanded; query b sees
    cache rows 0..ctx_lens[b]-1."""
    Lmax = K_cache.shape[2]
    mask = (torch.arange(Lmax, device=Q.device)[None, :] < ctx_lens.to(Q.device)[:, None])[:, None, None, :]
    return F.scaled_dot_product_attention(Q, K_cache, V_cache, attn_mask=mask)


def flash_attn_varlen(Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, cu_seqlens: torch.Tensor) -> torch.Tensor:
    """Q/K/V: (1, n_heads, T, head_dim), pre-expanded; causal attention inside each packed sequence."""
    out = torch.empty_like(Q)
    cu = cu_seqlens.tolist()
    for lo, hi in zip(cu[:-1], cu[1:]):
        if hi > lo:
            out[:, :, lo:hi] = F.scaled_dot_product_attention(Q[:, :, lo:hi], K[:, :, lo:hi], V[:, :, lo:hi], is_causal=True)
    return out
