"""PyTorch statements of what each op computes, for callers that want to compare or time against
them the way the reference's apps do (reference: src/minfer/kernels/refs.py:12-55,
apps/benchmark.py:240-248).  Nothing in the operator path calls these."""
import torch
import torch.nn.functional as F


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x: (B, L, n_heads, head_dim) (per head) or (B, L, hidden) (per vector); normalised over the last dimension."""
    return F.rms_norm(x, (x.shape[-1],), weight=weight, eps=eps)


def gemm(input: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, out: torch.Tensor, alpha: float, beta: float):
    """alpha * input @ weight + beta * bias -> out; all 2-D (squeeze 3-D activations first)."""
    torch.addmm(bias, input, weight, beta=beta, alpha=alpha, out=out)


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


def _rope_angles(L: int, rotary_dim: int, start_pos: int, base_freq: float, device) -> torch.Tensor:
    """angle[l, i] = (start_pos + l) * base_freq^(-2i/rotary_dim), fp32 like the reference's."""
    i = torch.arange(rotary_dim // 2, dtype=torch.float32, device=device)
    inv = base_freq ** (-2.0 * i / rotary_dim)
    return (torch.arange(L, dtype=torch.float32, device=device) + start_pos)[:, None] * inv[None, :]


def il_rope(x: torch.Tensor, rotary_dim: int, start_pos: int, base_freq: float) -> torch.Tensor:
    """Interleaved rotary embedding; x: (B, L, n_heads, head_dim).  Pairs (2i, 2i+1) rotate by angle[l, i]."""
    ang = _rope_angles(x.shape[1], rotary_dim, start_pos, base_freq, x.device)
    cos, sin = ang.cos()[None, :, None, :], ang.sin()[None, :, None, :]
    y = x.float().clone()
    x0, x1 = y[..., 0:rotary_dim:2].clone(), y[..., 1:rotary_dim:2].clone()
    y[..., 0:rotary_dim:2] = cos * x0 - sin * x1
    y[..., 1:rotary_dim:2] = sin * x0 + cos * x1
    return y.to(x.dtype)


def neox_rope(x: torch.Tensor, rotary_dim: int, start_pos: int, base_freq: float) -> torch.Tensor:
    """NeoX rotary embedding; x: (B, L, n_heads, head_dim).  Pairs (i, i + rotary_dim/2) rotate by angle[l, i]."""
    ang = _rope_angles(x.shape[1], rotary_dim, start_pos, base_freq, x.device)
    cos, sin = ang.cos()[None, :, None, :], ang.sin()[None, :, None, :]
    y = x.float().clone()
    h = rotary_dim // 2
    x0, x1 = y[..., :h].clone(), y[..., h:rotary_dim].clone()
    y[..., :h] = cos * x0 - sin * x1
    y[..., h:rotary_dim] = sin * x0 + cos * x1
    return y.to(x.dtype)
