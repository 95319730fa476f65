"""Pins the CPU oracle (oracle/attn_oracle.c) before anything is compared against it.

The reference has no stored vectors for attention, so the oracle is pinned by
  * the reference's own oracle call, torch SDPA on K/V expanded with repeat_interleave
    (reference: src/minfer/kernels/refs.py:53-55, test/kernels.py:252-257), run live on CPU,
  * an independent numpy float64 evaluation of the closed form,
  * committed golden vectors (tests/golden),
  * closed-form invariants chosen so that a dropped scale, a transposed mask, a wrong GQA head
    mapping or an off-by-one in a causal / context bound each fail at least one of them.
"""
import glob
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def np_attention(q, k, v, mask):
    """softmax(q k^T / sqrt(D) | mask) v in float64 with explicit loops over heads."""
    q, k, v = (np.asarray(x, dtype=np.float64) for x in (q, k, v))
    B, Hq, Lq, D = q.shape
    Hkv = k.shape[1]
    out = np.zeros((B, Hq, Lq, D))
    for b in range(B):
        for h in range(Hq):
            g = h // (Hq // Hkv)
            s = q[b, h] @ k[b, g].T / np.sqrt(D)
            s = np.where(mask[b, 0], s, -np.inf)
            m = s.max(axis=1, keepdims=True)
            m = np.where(np.isfinite(m), m, 0.0)
            p = np.exp(s - m)
            den = p.sum(axis=1, keepdims=True)
            out[b, h] = np.where(den > 0, p / np.where(den > 0, den, 1.0), 0.0) @ v[b, g]
    return out


def rand_case(B, Hq, Hkv, L, D, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(B, Hq, L, D, generator=g), torch.randn(B, Hkv, L, D, generator=g),
            torch.randn(B, Hkv, L, D, generator=g), g)


def sdpa_ref(q, k, v, mask):
    n_rep = q.shape[1] // k.shape[1]
    return F.scaled_dot_product_attention(q, k.repeat_interleave(n_rep, 1), v.repeat_interleave(n_rep, 1), attn_mask=mask)


@pytest.mark.parametrize("B,Hq,Hkv,L,D", [(1, 8, 2, 256, 64), (2, 6, 2, 37, 128), (1, 4, 4, 65, 64), (1, 3, 1, 9, 128)])
@pytest.mark.parametrize("kind", ["causal", "window", "random"])
def test_oracle_matches_sdpa_and_numpy(B, Hq, Hkv, L, D, kind):
    q, k, v, g = rand_case(B, Hq, Hkv, L, D, seed=L + D)
    i = torch.arange(L)
    if kind == "causal":
        m = i[None, :] <= i[:, None]                       # reference: test/kernels.py:242
    elif kind == "window":
        m = (i[None, :] - i[:, None]).abs() < 5            # reference: test/kernels.py:276-278
    else:
        m = torch.rand(L, L, generator=g) < 0.5
        m[L // 2, :] = False
    mask = m[None, None].expand(B, 1, L, L).contiguous()
    got = oracle.flash_attn(q, k, v, mask)
    np.testing.assert_allclose(got, sdpa_ref(q, k, v, mask).numpy(), atol=2e-6, rtol=0)
    np.testing.assert_allclose(got, np_attention(q.numpy(), k.numpy(), v.numpy(), mask.numpy()), atol=2e-6, rtol=0)


def test_cpu_plumbing_config():
    """benchmark configuration 1: B=1, Hq=8, Hkv=2, S=256, D=64, fp32, causal, scale 1/sqrt(64)."""
    import workloads
    q, k, v, mask = workloads.cpu_plumbing(seed=0)
    got = oracle.flash_attn(q, k, v, mask)
    assert got.shape == (1, 8, 256, 64)
    np.testing.assert_allclose(got, sdpa_ref(q, k, v, mask).numpy(), atol=2e-6, rtol=0)
    # scale really is 1/8: logits scaled any other way change the result measurably
    wrong = sdpa_ref(q * 2.0, k, v, mask).numpy()
    assert np.abs(got - wrong).max() > 1e-2


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "dense_*.npz"))))
def test_golden_dense(path):
    z = np.load(path)
    got = oracle.flash_attn(z["q"], z["k"], z["v"], z["mask"])
    np.testing.assert_allclose(got, z["out"], atol=2e-6, rtol=0)


def test_golden_decode_and_varlen():
    z = np.load(os.path.join(GOLDEN, "decode_b3_h8_kv2_l50_d128.npz"))
    np.testing.assert_allclose(oracle.flash_attn_decode(z["q"], z["k"], z["v"], z["ctx"]), z["out"], atol=2e-6, rtol=0)
    z = np.load(os.path.join(GOLDEN, "varlen_h4_kv2_d64.npz"))
    np.testing.assert_allclose(oracle.flash_attn_varlen(z["q"], z["k"], z["v"], z["cu"]), z["out"], atol=2e-6, rtol=0)


def test_invariants_masking_exact():
    B, Hq, Hkv, L, D = 1, 4, 2, 33, 64
    q, k, v, g = rand_case(B, Hq, Hkv, L, D, seed=7)
    causal = torch.ones(L, L, dtype=torch.bool).tril()[None, None]
    out = oracle.flash_attn(q, k, v, causal)
    # causal row 0 sees key 0 only: exact copy of V row 0 of the head's KV head
    for h in range(Hq):
        assert np.array_equal(out[0, h, 0], v[0, h // 2, 0].numpy())
    # one-hot rows copy exactly the selected V row (mask orientation: row = query, column = key)
    sel = torch.randint(0, L, (L,), generator=g)
    onehot = torch.zeros(L, L, dtype=torch.bool)
    onehot[torch.arange(L), sel] = True
    out = oracle.flash_attn(q, k, v, onehot[None, None])
    for h in range(Hq):
        assert np.array_equal(out[0, h], v[0, h // 2, sel].numpy())
    # a row with no attended key gives zeros (torch 2.10 CPU SDPA does the same)
    none = causal.clone()
    none[0, 0, 5, :] = False
    out = oracle.flash_attn(q, k, v, none)
    assert np.all(out[0, :, 5] == 0)
    assert np.all(sdpa_ref(q, k, v, none)[0, :, 5].numpy() == 0)


def test_invariants_closed_forms():
    B, Hq, Hkv, L, D = 2, 8, 2, 40, 64
    q, k, v, g = rand_case(B, Hq, Hkv, L, D, seed=11)
    causal = torch.ones(L, L, dtype=torch.bool).tril()[None, None].expand(B, 1, L, L)
    # Q = 0: uniform weights -> running mean of V
    out = oracle.flash_attn(torch.zeros_like(q), k, v, causal)
    run_mean = (v.double().cumsum(2) / torch.arange(1, L + 1)[None, None, :, None]).numpy()
    for h in range(Hq):
        np.testing.assert_allclose(out[:, h], run_mean[:, h // 4], atol=1e-6)
    # V constant per KV head exposes the GQA mapping h -> h // n_rep exactly
    vconst = torch.zeros_like(v)
    for gidx in range(Hkv):
        vconst[:, gidx] = float(gidx + 1)
    out = oracle.flash_attn(q, k, vconst, causal)
    for h in range(Hq):
        np.testing.assert_allclose(out[:, h], float(h // 4 + 1), atol=1e-6)
    # permuting keys together with mask columns leaves the result unchanged
    full = torch.rand(L, L, generator=g) < 0.7
    full[:, 0] = True
    perm = torch.randperm(L, generator=g)
    a = oracle.flash_attn(q, k, v, full[None, None].expand(B, 1, L, L))
    b = oracle.flash_attn(q, k[:, :, perm], v[:, :, perm], full[:, perm][None, None].expand(B, 1, L, L))
    np.testing.assert_allclose(a, b, atol=1e-6)
    # softmax shift invariance: adding a constant vector c to every key adds q.c to every logit of a row
    c = torch.randn(D, generator=g)
    np.testing.assert_allclose(a, oracle.flash_attn(q, k + c, v, full[None, None].expand(B, 1, L, L)), atol=2e-5)


def test_rows_decode_varlen_consistency():
    B, Hq, Hkv, L, D = 2, 4, 2, 50, 128
    q, k, v, g = rand_case(B, Hq, Hkv, L, D, seed=3)
    causal = torch.ones(L, L, dtype=torch.bool).tril()[None, None].expand(B, 1, L, L).contiguous()
    dense = oracle.flash_attn(q, k, v, causal)
    rows = [0, 7, 49]
    np.testing.assert_array_equal(oracle.flash_attn_rows(q, k, v, causal[:, 0, rows], rows), dense[:, :, rows])
    # decode with ctx = i+1 is row i of causal prefill
    ctx = torch.tensor([13, 50], dtype=torch.int32)
    qd = torch.stack([q[b, :, ctx[b] - 1] for b in range(B)])[:, :, None]
    dec = oracle.flash_attn_decode(qd, k, v, ctx)
    for b in range(B):
        np.testing.assert_array_equal(dec[b, :, 0], dense[b, :, ctx[b] - 1])
    # ctx = 0 -> zeros; rows beyond ctx never matter
    k2, v2 = k.clone(), v.clone()
    k2[0, :, 13:] = float("nan")
    v2[0, :, 13:] = float("inf")
    np.testing.assert_array_equal(oracle.flash_attn_decode(qd, k2, v2, ctx)[0], dec[0])
    assert np.all(oracle.flash_attn_decode(qd, k, v, torch.tensor([0, 50], dtype=torch.int32))[0] == 0)
    # varlen equals per-sequence causal prefill and the block-diagonal-causal dense mask
    lens = [20, 0, 30]
    cu = np.array([0, 20, 20, 50], dtype=np.int32)
    var = oracle.flash_attn_varlen(q[:1], k[:1], v[:1], cu)
    blk = torch.zeros(L, L, dtype=torch.bool)
    for lo, hi in zip(cu[:-1], cu[1:]):
        blk[lo:hi, lo:hi] = torch.ones(hi - lo, hi - lo, dtype=torch.bool).tril()
    np.testing.assert_array_equal(var, oracle.flash_attn(q[:1], k[:1], v[:1], blk[None, None]))
    np.testing.assert_array_equal(var[:, :, :20], oracle.flash_attn(q[:1, :, :20], k[:1, :, :20], v[:1, :, :20], causal[:1, :, :20, :20]))


def test_oracle_rejects_bad_arguments():
    q = np.zeros((1, 3, 4, 64), np.float32)
    k = np.zeros((1, 2, 4, 64), np.float32)
    with pytest.raises(ValueError):
        oracle.flash_attn(q, k, k, np.ones((1, 1, 4, 4), bool))          # Hq % Hkv != 0
    q = np.zeros((1, 2, 1, 64), np.float32)
    with pytest.raises(ValueError):
        oracle.flash_attn_decode(q, k, k, np.array([5], np.int32))          # ctx > Lmax
    q = np.zeros((1, 2, 4, 64), np.float32)
    with pytest.raises(ValueError):
        oracle.flash_attn_varlen(q, k, k, np.array([0, 3], np.int32))       # cu_seqlens[-1] != T
