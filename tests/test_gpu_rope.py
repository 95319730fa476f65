"""GPU parity tests (-m gpu) of the rotary-embedding kernels and of the rope + KV-cache append producer,
called through the C ABI (and the registered torch ops), against the fp64 CPU oracle on identical
seeded inputs.

Tolerance.  The reference's own test allows atol 5e-3 on N(0,1) fp16 data because it evaluates the
angle in fp32 (reference: test/kernels.py:94-95).  The kernels here reduce the angle in fp64, so the
bar is the output format itself: every element must lie within 0.51 units in the last place of the
oracle's exact value (0.5 for the final rounding, 0.01 for the fp32 arithmetic before it) plus 2^-20 of
the tensor's largest magnitude (the fp32 cos/sin, which shows only where cos*x0 and sin*x1 cancel to a
result far smaller than its terms); for |x| < 8 that is always inside the reference's 5e-3 as well.  Elements the operator must not touch (past
rotary_dim, cache rows that are not appended) are compared for exact equality.
"""
import numpy as np
import pytest
import torch

import capi
import oracle
import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda"
IL, NEOX = capi.ROPE_INTERLEAVED, capi.ROPE_NEOX
MANT = {torch.float16: 10, torch.bfloat16: 7}
MIN_EXP = {torch.float16: -14, torch.bfloat16: -126}


def ulp(exact, dtype):
    e = np.floor(np.log2(np.maximum(np.abs(exact.astype(np.float64)), 2.0 ** MIN_EXP[dtype])))
    return 2.0 ** (e - MANT[dtype])


def assert_close(got, exact, dtype, what=""):
    got = got.float().cpu().numpy().astype(np.float64)
    err = np.abs(got - exact)
    bound = 0.51 * ulp(exact, dtype) + 2.0 ** -20 * float(np.abs(exact).max())
    bad = err > bound
    worst = np.unravel_index(np.argmax(err - bound), err.shape)
    assert not bad.any(), (f"{what}: {bad.sum()} elements beyond 0.51 ulp; at {worst} got {got[worst]!r}, "
                           f"exact {float(exact[worst])!r}, error {err[worst]:.3e}")
    if dtype == torch.float16:   # the reference's own bar (it tests fp16 only)
        assert err.max() <= 5e-3 or np.abs(exact).max() >= 8.0


def run_rope(style, x, rd, start, base):
    y = x.clone()
    rc = capi.rope(style, y, rd, start, base)
    assert rc == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    return y


@pytest.mark.parametrize("style", [IL, NEOX])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape,rd,start,base", [
    ((2, 33, 5, 128), 64, 0, 1e6),        # the reference test's head shape (rotary 64 of 128)
    ((1, 70, 8, 128), 128, 2048, 5e5),    # Llama-3: the whole head rotates
    ((3, 17, 3, 64), 32, 100000, 1e4),    # far positions
    ((1, 300, 2, 256), 256, 7, 1e4),      # largest rotary_dim
    ((2, 9, 3, 80), 16, 31, 1e4),         # head_dim that is only a multiple of 8
    ((2, 11, 3, 12), 6, 5, 1e4),          # nothing vectorisable: one-pair-per-thread kernel
    ((1, 6, 2, 128), 2, 1000, 1e4),
])
def test_rope_matches_oracle(style, dtype, shape, rd, start, base):
    g = torch.Generator().manual_seed(sum(shape) + rd)
    x = torch.randn(*shape, generator=g).to(dtype)
    exact = oracle.rope(style, x, rd, start, base)
    y = run_rope(style, x.to(DEV), rd, start, base)
    assert_close(y, exact, dtype, "rope")
    assert torch.equal(y[..., rd:].cpu(), x[..., rd:])      # tail untouched


def test_rope_golden_vectors():
    import os
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "rope_small.npz"))
    x = torch.from_numpy(z["x"]).to(DEV)
    for style, name in ((IL, "il"), (NEOX, "neox")):
        y = run_rope(style, x, int(z["rotary_dim"]), int(z["start_pos"]), float(z["freq_base"]))
        assert_close(y, z[f"y_{name}"].astype(np.float64), torch.float16, name)


@pytest.mark.parametrize("style", [IL, NEOX])
@pytest.mark.parametrize("start", [0, 2048])
def test_rope_reference_test_shape(style, start):
    """B=8, L=4096, 48 heads of 128, rotary 64, base 1e6, start 0 / 2048 (reference: test/kernels.py:76-96):
    oracle on slices of tokens, and on the whole tensor what holds at any size: pair norms are kept,
    the tail is untouched, token 0 at start 0 is unchanged."""
    rd, base = 64, 1e6
    x = workloads.rope_input(seed=start, device=DEV)
    y = run_rope(style, x, rd, start, base)
    for b, l0 in ((0, 0), (3, 1777), (7, 4096 - 16)):
        exact = oracle.rope(style, x[b:b + 1, l0:l0 + 16].cpu(), rd, start + l0, base)
        assert_close(y[b:b + 1, l0:l0 + 16], exact, torch.float16, f"slice {b},{l0}")
    assert torch.equal(y[..., rd:], x[..., rd:])
    if start == 0:
        assert torch.equal(y[:, 0], x[:, 0])
    xf, yf = x[..., :rd].float(), y[..., :rd].float()
    if style == IL:
        nx, ny = xf.view(*xf.shape[:-1], rd // 2, 2).square().sum(-1), yf.view(*yf.shape[:-1], rd // 2, 2).square().sum(-1)
    else:
        nx, ny = xf[..., :rd // 2].square() + xf[..., rd // 2:].square(), yf[..., :rd // 2].square() + yf[..., rd // 2:].square()
    assert float((nx.sqrt() - ny.sqrt()).abs().max()) < 6e-3     # two roundings of values below 8


def run_append(style, q, k, v, pos, kc, vc, rd, base):
    q2, kc2, vc2 = q.clone(), kc.clone(), vc.clone()
    rc = capi.rope_kv_append(style, q2, k, v, pos, kc2, vc2, rd, base)
    assert rc == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    return q2, kc2, vc2


@pytest.mark.parametrize("style", [IL, NEOX])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,L,Hq,Hkv,D,Lmax,rd,pos", [
    (3, 5, 4, 2, 64, 12, 32, [0, 7, 9]),          # sequence 2 runs past the end of the cache
    (2, 40, 8, 2, 128, 64, 128, [24, 0]),
    (4, 1, 32, 8, 128, 96, 64, [95, 0, 50, 96]),  # decode step; sequence 3 is full (row 96 does not exist)
    (1, 3, 2, 1, 16, 8, 0, [2]),                  # rotary_dim 0: pure append
    (1, 6, 80, 10, 128, 16, 96, [3]),             # more chunks per token than one pass of the workgroup takes
])
def test_kv_append_matches_oracle(style, dtype, B, L, Hq, Hkv, D, Lmax, rd, pos):
    g = torch.Generator().manual_seed(B * 100 + L)
    q = torch.randn(B, L, Hq, D, generator=g).to(dtype)
    k = torch.randn(B, L, Hkv, D, generator=g).to(dtype)
    v = torch.randn(B, L, Hkv, D, generator=g).to(dtype)
    kc = torch.randn(B, Hkv, Lmax, D, generator=g).to(dtype)     # pre-existing content must survive
    vc = torch.randn(B, Hkv, Lmax, D, generator=g).to(dtype)
    p = torch.tensor(pos, dtype=torch.int32)
    eq, ekc, evc = oracle.rope_kv_append(style, q, k, v, p, kc, vc, rd, 1e4)
    q2, kc2, vc2 = run_append(style, q.to(DEV), k.to(DEV), v.to(DEV), p.to(DEV), kc.to(DEV), vc.to(DEV), rd, 1e4)
    assert_close(q2, eq, dtype, "q")
    assert_close(kc2, ekc, dtype, "k_cache")
    assert torch.equal(vc2.cpu().float(), torch.from_numpy(evc))            # copies are exact
    for b in range(B):                                                     # rows not appended: bit-identical
        keep = torch.ones(Lmax, dtype=torch.bool)
        keep[max(0, pos[b]):max(0, min(Lmax, pos[b] + L))] = False
        assert torch.equal(kc2[b].cpu()[:, keep], kc[b][:, keep])
        assert torch.equal(vc2[b].cpu()[:, keep], vc[b][:, keep])


def test_kv_append_strided_cache():
    """Caches that are views of a larger allocation (other strides than [Hkv*Lmax*D, Lmax*D, D])."""
    B, L, Hq, Hkv, D, Lmax = 2, 6, 4, 2, 64, 16
    g = torch.Generator().manual_seed(9)
    q, k, v = (torch.randn(B, L, h, D, generator=g).half() for h in (Hq, Hkv, Hkv))
    big_k = torch.randn(B, Hkv + 1, Lmax + 8, D, generator=g).half()
    big_v = torch.randn(B, Hkv + 1, Lmax + 8, D, generator=g).half()
    p = torch.tensor([3, 10], dtype=torch.int32)
    bk, bv = big_k.to(DEV), big_v.to(DEV)
    kc, vc = bk[:, 1:, 8:], bv[:, 1:, 8:]
    eq, ekc, evc = oracle.rope_kv_append(IL, q, k, v, p, big_k[:, 1:, 8:], big_v[:, 1:, 8:], 64, 1e4)
    q2 = q.to(DEV)
    assert capi.rope_kv_append(IL, q2, k.to(DEV), v.to(DEV), p.to(DEV), kc, vc, 64, 1e4) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert_close(kc, ekc, torch.float16, "k_cache view")
    assert torch.equal(vc.cpu().float(), torch.from_numpy(evc))
    assert torch.equal(bk[:, 0].cpu(), big_k[:, 0]) and torch.equal(bk[:, :, :8].cpu(), big_k[:, :, :8])


def test_kv_append_llama_shape_then_decode_reads_it():
    """Llama-3-8B prefill shape (B=1, L=4096, 32/8 heads of 128, whole head rotates, base 5e5): sampled
    tokens against the oracle, then the decode kernel attends over the cache this producer wrote and must
    agree with the attention oracle run on the oracle's cache."""
    q, k, v, pos, kc, vc = workloads.kv_append(seed=1, device=DEV, Lmax=4096 + 64)
    q2, kc2, vc2 = run_append(NEOX, q, k, v, pos, kc, vc, 128, 5e5)
    for l0 in (0, 2049, 4096 - 8):
        sl = slice(l0, l0 + 8)
        eq, ekc, evc = oracle.rope_kv_append(NEOX, q[:, sl].cpu(), k[:, sl].cpu(), v[:, sl].cpu(), torch.tensor([l0], dtype=torch.int32),
                                             torch.zeros(1, 8, 4096 + 64, 128), torch.zeros(1, 8, 4096 + 64, 128), 128, 5e5)
        assert_close(q2[:, sl], eq, torch.float16, "q")
        assert_close(kc2[:, :, sl], ekc[:, :, sl], torch.float16, "k_cache")
        assert torch.equal(vc2[:, :, sl].cpu().float(), torch.from_numpy(evc[:, :, sl]))
    assert float(kc2[:, :, 4096:].abs().max()) == 0.0 and float(vc2[:, :, 4096:].abs().max()) == 0.0
    # the last token as a decode query over the 4096 rows just written
    qd = q2[:, -1:].transpose(1, 2).contiguous()                  # [1, 32, 1, 128]
    ctx = torch.tensor([4096], dtype=torch.int32, device=DEV)
    out = torch.empty_like(qd)
    assert capi.flash_attn_decode(qd, kc2, vc2, ctx, out) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    want = oracle.flash_attn_decode(qd, kc2, vc2, ctx)
    assert float((out.float().cpu() - torch.from_numpy(want)).abs().max()) <= 2e-3


def test_large_launches_equal_the_same_work_in_small_ones():
    """A launch that touches more than the memory-side cache holds marks its loads and stores non-temporal; one
    batch entry at a time stays below that.  Both must give the same bits: in place over whole heads, the producer
    into fp16 caches and into Q8_0 caches."""
    B, L = 8, 4096
    x = workloads.rope_input(seed=5, device=DEV)                       # [8, 4096, 48, 128]
    big = run_rope(NEOX, x, 128, 7, 5e5)
    for b in range(B):
        assert torch.equal(big[b:b + 1], run_rope(NEOX, x[b:b + 1].contiguous(), 128, 7, 5e5)), b
    del big, x
    q, k, v, pos, kc, vc = workloads.kv_append(seed=2, device=DEV, B=B, L=L, pos_hi=9)
    q2, kc2, vc2 = run_append(NEOX, q, k, v, pos, kc, vc, 128, 5e5)
    kq = torch.zeros(B, 8, kc.shape[2], 136, dtype=torch.uint8, device=DEV)
    vq = torch.zeros_like(kq)
    q3 = q.clone()
    assert capi.rope_kv_append_q8_0(NEOX, q3, k, v, pos, kq, vq, 128, 5e5) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert torch.equal(q3, q2)
    for b in range(B):
        one = slice(b, b + 1)
        qs, ks, vs = run_append(NEOX, q[one].contiguous(), k[one].contiguous(), v[one].contiguous(), pos[one], kc[one].contiguous(), vc[one].contiguous(), 128, 5e5)
        assert torch.equal(q2[one], qs) and torch.equal(kc2[one], ks) and torch.equal(vc2[one], vs), b
        kqs, vqs, qq = torch.zeros_like(kq[one]), torch.zeros_like(vq[one]), q[one].contiguous()
        assert capi.rope_kv_append_q8_0(NEOX, qq, k[one].contiguous(), v[one].contiguous(), pos[one], kqs, vqs, 128, 5e5) == capi.OK
        torch.cuda.synchronize()
        assert torch.equal(kq[one], kqs) and torch.equal(vq[one], vqs), b


def test_torch_ops_equal_c_abi_and_keep_the_reference_checks(kerns):
    g = torch.Generator().manual_seed(4)
    x = torch.randn(2, 50, 6, 128, generator=g).half().to(DEV)
    for style, fn in ((IL, kerns.il_rope), (NEOX, kerns.neox_rope)):
        a = run_rope(style, x, 64, 2048, 1e6)
        b = x.clone()
        assert fn(64, 2048, 1e6, b) is None
        torch.cuda.synchronize()
        assert torch.equal(a, b)
    assert torch.equal(run_rope(IL, x, 64, 3, 1e4), (lambda t: (torch.ops.minfer.il_rope.default(64, 3, 1e4, t), t)[1])(x.clone()))
    # the reference's checks (il_rope/op.cuh:26-30): contiguous, 4-D, half (or bfloat16 here), rotary_dim <= head_dim
    with pytest.raises(RuntimeError):
        kerns.il_rope(64, 0, 1e4, x.transpose(1, 2))
    with pytest.raises(RuntimeError):
        kerns.neox_rope(64, 0, 1e4, x[0])
    with pytest.raises(RuntimeError):
        kerns.il_rope(64, 0, 1e4, x.float())
    with pytest.raises(RuntimeError):
        kerns.il_rope(256, 0, 1e4, x.clone())
    with pytest.raises((RuntimeError, NotImplementedError)):
        kerns.il_rope(64, 0, 1e4, x.cpu())            # no CPU implementation is registered
    # fused producer through the op
    q, k, v, pos, kc, vc = workloads.kv_append(seed=2, device=DEV, B=3, L=20, Lmax=40, pos_hi=20)
    qa, kca, vca = run_append(IL, q, k, v, pos, kc, vc, 128, 1e4)
    qb, kcb, vcb = q.clone(), kc.clone(), vc.clone()
    assert kerns.rope_kv_append(IL, 128, 1e4, qb, k, v, pos, kcb, vcb) is None
    torch.cuda.synchronize()
    assert torch.equal(qa, qb) and torch.equal(kca, kcb) and torch.equal(vca, vcb)
    with pytest.raises(RuntimeError):
        kerns.rope_kv_append(IL, 128, 1e4, qb, k, v, pos.long(), kcb, vcb)
    with pytest.raises(RuntimeError):
        kerns.rope_kv_append(2, 128, 1e4, qb, k, v, pos, kcb, vcb)


def test_rope_agrees_with_the_fp32_torch_statement():
    """refs.il_rope / refs.neox_rope restate the reference's fp32 torch expressions; at the reference's
    own tolerance (atol 5e-3, test/kernels.py:95) the kernels agree with them too."""
    from minfer.kernels import refs
    x = workloads.rope_input(seed=5, device=DEV, B=2, L=512)
    for style, ref in ((IL, refs.il_rope), (NEOX, refs.neox_rope)):
        for start in (0, 2048):
            y = run_rope(style, x, 64, start, 1e6)
            assert torch.allclose(ref(x, 64, start, 1e6).float(), y.float(), atol=5e-3)
