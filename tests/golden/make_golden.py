"""Writes the golden vectors in this directory.

The reference holds no stored vectors for attention (its test compares against a live
torch SDPA call with unseeded inputs: reference test/kernels.py:222-298).  These fixtures pin
that same call on seeded inputs: expected = F.scaled_dot_product_attention(Q, K_exp, V_exp,
attn_mask=mask) on CPU in fp32 with torch 2.10, K/V expanded by repeat_interleave(n_rep, dim=1),
which is the reference's refs.flash_attn (reference src/minfer/kernels/refs.py:53-55).  Nothing
from the reference is imported.  Inputs are fp16-representable (q, k ~ N(0,1), v ~ 0.5*N(0,1), so that |out| stays below 2 and
the fp16 output format itself does not eat the 2e-3 tolerance) and stored as fp16, so the
fp16 kernels see exactly the values the expected output was computed from.

The rotary-embedding fixture (rope_small.npz) pins the reference's torch formulation of both styles
(reference src/minfer/kernels/refs.py:12-47) in float64 on seeded fp16-representable inputs, and
rmsnorm_small.npz the reference's F.rms_norm call (refs.py:10) in float64, gemm_small.npz its torch.addmm call
(refs.py:49-51) in float64.

Run:  python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))


def sdpa(q, k, v, mask):
    n_rep = q.shape[1] // k.shape[1]
    return F.scaled_dot_product_attention(q, k.repeat_interleave(n_rep, 1), v.repeat_interleave(n_rep, 1), attn_mask=mask)


def make(name, B, Hq, Hkv, L, D, kind, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, L, D, generator=g).half().float()
    k = torch.randn(B, Hkv, L, D, generator=g).half().float()
    v = (0.5 * torch.randn(B, Hkv, L, D, generator=g)).half().float()
    i = torch.arange(L)
    if kind == "causal":
        m = i[None, :] <= i[:, None]
    elif kind == "window":
        m = (i[None, :] - i[:, None]).abs() < 7
    else:
        m = torch.rand(L, L, generator=g) < 0.4
        m[3, :] = False  # a row that attends nothing
    mask = m[None, None].expand(B, 1, L, L).contiguous()
    out = sdpa(q, k, v, mask)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), q=q.numpy().astype(np.float16), k=k.numpy().astype(np.float16),
                        v=v.numpy().astype(np.float16), mask=mask.numpy(), out=out.numpy().astype(np.float32))


def make_decode(name, B, Hq, Hkv, Lmax, D, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, 1, D, generator=g).half().float()
    k = torch.randn(B, Hkv, Lmax, D, generator=g).half().float()
    v = (0.5 * torch.randn(B, Hkv, Lmax, D, generator=g)).half().float()
    ctx = torch.randint(1, Lmax + 1, (B,), generator=g, dtype=torch.int32)
    mask = (torch.arange(Lmax)[None, :] < ctx[:, None])[:, None, None, :]
    out = sdpa(q, k, v, mask)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), q=q.numpy().astype(np.float16), k=k.numpy().astype(np.float16),
                        v=v.numpy().astype(np.float16), ctx=ctx.numpy(), out=out.numpy().astype(np.float32))


def make_varlen(name, Hq, Hkv, D, lens, seed):
    g = torch.Generator().manual_seed(seed)
    T = sum(lens)
    q = torch.randn(1, Hq, T, D, generator=g).half().float()
    k = torch.randn(1, Hkv, T, D, generator=g).half().float()
    v = (0.5 * torch.randn(1, Hkv, T, D, generator=g)).half().float()
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    out = torch.zeros_like(q)
    for lo, hi in zip(cu[:-1], cu[1:]):
        if hi > lo:
            n = hi - lo
            m = torch.ones(n, n, dtype=torch.bool).tril()[None, None]
            out[:, :, lo:hi] = sdpa(q[:, :, lo:hi], k[:, :, lo:hi], v[:, :, lo:hi], m)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), q=q.numpy().astype(np.float16), k=k.numpy().astype(np.float16),
                        v=v.numpy().astype(np.float16), cu=cu, out=out.numpy().astype(np.float32))


def make_rope(name, B, L, H, D, rotary_dim, start_pos, freq_base, seed):
    """Expected values of both rotary styles from the reference's torch formulation, complex multiplication
    by exp(i*theta) (reference src/minfer/kernels/refs.py:19-27 and 37-47), evaluated in float64."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, L, H, D, generator=g).half().double()
    f = freq_base ** (-2.0 * torch.arange(rotary_dim // 2, dtype=torch.float64) / rotary_dim)
    ang = (torch.arange(L, dtype=torch.float64) + start_pos)[:, None] * f[None, :]
    rot = torch.polar(torch.ones_like(ang), ang)[None, :, None, :]
    y_il = x.clone()
    xc = torch.view_as_complex(x[..., :rotary_dim].reshape(B, L, H, rotary_dim // 2, 2).contiguous())
    y_il[..., :rotary_dim] = torch.view_as_real(xc * rot).flatten(-2)
    y_neox = x.clone()
    h = rotary_dim // 2
    xc = torch.view_as_complex(torch.stack([x[..., :h], x[..., h:rotary_dim]], dim=-1).contiguous())
    yr = torch.view_as_real(xc * rot)
    y_neox[..., :h] = yr[..., 0]
    y_neox[..., h:rotary_dim] = yr[..., 1]
    np.savez_compressed(os.path.join(HERE, name + ".npz"), x=x.numpy().astype(np.float16), rotary_dim=rotary_dim,
                        start_pos=start_pos, freq_base=freq_base, y_il=y_il.numpy().astype(np.float32),
                        y_neox=y_neox.numpy().astype(np.float32))


def make_rmsnorm(name, shape, eps, seed):
    """Expected values from the reference's oracle call, F.rms_norm over the last dimension (reference
    src/minfer/kernels/refs.py:10), evaluated in float64."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(*shape, generator=g).half().double()
    w = ((1 / shape[-1] ** 0.5) * torch.randn(shape[-1], generator=g)).half().double()
    y = F.rms_norm(x, (shape[-1],), weight=w, eps=eps)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), x=x.numpy().astype(np.float16), w=w.numpy().astype(np.float16),
                        eps=eps, y=y.numpy().astype(np.float32))


def make_gemm(name, M, N, K, alpha, beta, seed):
    """Expected values from the reference's oracle call torch.addmm (reference src/minfer/kernels/refs.py:49-51)
    evaluated in float64; inputs drawn as in the reference's test (reference test/kernels.py:133-136)."""
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(M, K, generator=g).half().double()
    b = ((1 / K ** 0.5) * torch.randn(K, N, generator=g)).half().double()
    c = torch.randn(M, N, generator=g).half().double()
    d = torch.addmm(c, a, b, beta=beta, alpha=alpha)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), a=a.numpy().astype(np.float16), b=b.numpy().astype(np.float16),
                        c=c.numpy().astype(np.float16), alpha=alpha, beta=beta, d=d.numpy().astype(np.float32))


if __name__ == "__main__":
    torch.set_num_threads(1)
    make("dense_causal_b1_h4_kv2_l16_d64", 1, 4, 2, 16, 64, "causal", 1)
    make("dense_window_b2_h6_kv2_l40_d128", 2, 6, 2, 40, 128, "window", 2)
    make("dense_random_b1_h8_kv1_l70_d64", 1, 8, 1, 70, 64, "random", 3)
    make_decode("decode_b3_h8_kv2_l50_d128", 3, 8, 2, 50, 128, 4)
    make_varlen("varlen_h4_kv2_d64", 4, 2, 64, [5, 1, 33, 70], 5)
    make_rope("rope_small", 2, 9, 3, 64, 32, 2048, 1e6, 6)
    make_rmsnorm("rmsnorm_small", (2, 5, 3, 40), 1e-6, 7)
    make_gemm("gemm_small", 70, 72, 128, 2.0, 3.0, 8)
    print("golden vectors written to", HERE)
