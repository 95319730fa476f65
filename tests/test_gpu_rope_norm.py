"""GPU parity tests (-m gpu) of the rope + KV-cache append producer with the per-head RMS normalisation of q and k
fused in front of the rotation (reference: the optional rmsnorm(q), rmsnorm(k) calls before the two rope calls,
src/minfer/core.py:224-230), through the C ABI and the registered torch op.

Two bars.  (1) The fused call must equal the three separate operators (rmsnorm on q, rmsnorm on k, then the plain
producer) bit for bit: the intermediate is rounded to the element type exactly where the separate operators
round it.  (2) Against the fp64 oracle, composed the same way (oracle rmsnorm, rounded to the element type, then
the oracle producer): within 0.51 ulp of the output format wherever the rounded intermediate agrees, which is all
but a few elements in ten thousand (an intermediate that falls within 1e-2 ulp of a rounding boundary may round
the other way in fp32); those move by at most the intermediate's own unit in the last place.
"""
import numpy as np
import pytest
import torch

import capi
import oracle
import workloads
from test_gpu_rope import IL, NEOX, ulp

pytestmark = pytest.mark.gpu
DEV = "cuda"
EPS = 1e-6


def make(B, L, Hq, Hkv, D, Lmax, dtype, seed, q8=False):
    g = torch.Generator().manual_seed(seed)
    q = (2.0 * torch.randn(B, L, Hq, D, generator=g)).to(dtype)
    k = (0.5 * torch.randn(B, L, Hkv, D, generator=g)).to(dtype)
    v = torch.randn(B, L, Hkv, D, generator=g).to(dtype)
    wq = (1.0 + 0.3 * torch.randn(D, generator=g)).to(dtype)
    wk = (1.0 + 0.3 * torch.randn(D, generator=g)).to(dtype)
    if q8:
        kc = torch.randint(0, 256, (B, Hkv, Lmax, D // 32 * 34), generator=g, dtype=torch.uint8)
        vc = torch.randint(0, 256, (B, Hkv, Lmax, D // 32 * 34), generator=g, dtype=torch.uint8)
    else:
        kc = torch.randn(B, Hkv, Lmax, D, generator=g).to(dtype)
        vc = torch.randn(B, Hkv, Lmax, D, generator=g).to(dtype)
    return q, k, v, wq, wk, kc, vc


def separate_ops(style, q, k, v, wq, wk, pos, kc, vc, rd, base):
    """rmsnorm(q), rmsnorm(k), then the plain producer: three launches, the intermediates rounded to the dtype."""
    qn, kn = torch.empty_like(q), torch.empty_like(k)
    assert capi.rmsnorm(q, wq, qn, EPS) == capi.OK and capi.rmsnorm(k, wk, kn, EPS) == capi.OK, capi.last_error()
    kc2, vc2 = kc.clone(), vc.clone()
    fn = capi.rope_kv_append_q8_0 if kc.dtype == torch.uint8 else capi.rope_kv_append
    assert fn(style, qn, kn, v, pos, kc2, vc2, rd, base) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    return qn, kc2, vc2


CASES = [
    (2, 40, 8, 2, 128, 64, 128, [24, 0]),          # whole head rotates; sequence 0 runs past the end of the cache
    (3, 5, 4, 2, 64, 12, 32, [0, 7, 9]),           # half the head rotates, D = 64
    (4, 1, 32, 8, 128, 96, 64, [95, 0, 50, 96]),   # decode step; sequence 3 is full
    (1, 6, 80, 10, 128, 16, 96, [3]),              # 100 heads per token: several passes of the workgroup; NeoX half = 3 chunks
    (2, 3, 3, 1, 64, 8, 0, [2, 0]),                # nothing rotates: normalise and append; head sections cut waves
    (1, 9, 5, 5, 128, 16, 128, [1]),               # n_rep = 1, odd head counts
]


@pytest.mark.parametrize("style", [IL, NEOX])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,L,Hq,Hkv,D,Lmax,rd,pos", CASES)
def test_fused_norm_equals_separate_operators_and_oracle(style, dtype, B, L, Hq, Hkv, D, Lmax, rd, pos):
    if style == NEOX and rd % 16:
        pytest.skip("NeoX rotary_dim must be a multiple of 16")
    q, k, v, wq, wk, kc, vc = make(B, L, Hq, Hkv, D, Lmax, dtype, seed=B * 100 + L + D)
    p = torch.tensor(pos, dtype=torch.int32)
    dq, dk, dv, dwq, dwk, dp, dkc, dvc = (t.to(DEV) for t in (q, k, v, wq, wk, p, kc, vc))
    q_sep, kc_sep, vc_sep = separate_ops(style, dq, dk, dv, dwq, dwk, dp, dkc, dvc, rd, 1e4)
    q_f, kc_f, vc_f = dq.clone(), dkc.clone(), dvc.clone()
    assert capi.rope_kv_append_norm(style, q_f, dk, dv, dwq, dwk, EPS, dp, kc_f, vc_f, rd, 1e4) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert torch.equal(q_f, q_sep) and torch.equal(kc_f, kc_sep) and torch.equal(vc_f, vc_sep)

    # the oracle, composed the same way
    qn = torch.from_numpy(oracle.rmsnorm(q, wq, EPS)).to(dtype)
    kn = torch.from_numpy(oracle.rmsnorm(k, wk, EPS)).to(dtype)
    eq, ekc, evc = oracle.rope_kv_append(style, qn, kn, v, p, kc, vc, rd, 1e4)
    assert torch.equal(vc_f.cpu().float(), torch.from_numpy(evc))
    for got, exact, mid, what in ((q_f, eq, qn, "q"), (kc_f, ekc, kn, "k_cache")):
        err = np.abs(got.float().cpu().numpy().astype(np.float64) - exact)
        slack = 2.0 ** -20 * float(np.abs(exact).max())
        far = err > 0.51 * ulp(exact, dtype) + slack
        assert far.mean() <= 1e-3, f"{what}: {far.sum()} of {far.size} elements beyond 0.51 ulp"
        # where the rounded intermediate differs by one unit in its last place, the rotated value moves by at most
        # that unit (a rotation keeps the length of a pair), whatever the size of the rotated value itself
        mid_ulp = float(ulp(mid.float().abs().max().numpy(), dtype))
        assert (err <= 0.51 * ulp(exact, dtype) + 1.5 * mid_ulp + slack).all(), f"{what}: an element moved by more than the intermediate's rounding"
    for b in range(B):   # rows not appended keep their bits
        keep = torch.ones(Lmax, dtype=torch.bool)
        keep[max(0, pos[b]):max(0, min(Lmax, pos[b] + L))] = False
        assert torch.equal(kc_f[b].cpu()[:, keep], kc[b][:, keep]) and torch.equal(vc_f[b].cpu()[:, keep], vc[b][:, keep])


@pytest.mark.parametrize("style", [IL, NEOX])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_norm_into_q8_0_caches(style, dtype):
    B, L, Hq, Hkv, D, Lmax, rd = 2, 33, 8, 2, 128, 48, 128
    q, k, v, wq, wk, kc, vc = make(B, L, Hq, Hkv, D, Lmax, dtype, seed=77, q8=True)
    p = torch.tensor([20, 0], dtype=torch.int32)     # sequence 0 runs past the cache
    dq, dk, dv, dwq, dwk, dp, dkc, dvc = (t.to(DEV) for t in (q, k, v, wq, wk, p, kc, vc))
    q_sep, kc_sep, vc_sep = separate_ops(style, dq, dk, dv, dwq, dwk, dp, dkc, dvc, rd, 5e5)
    q_f, kc_f, vc_f = dq.clone(), dkc.clone(), dvc.clone()
    assert capi.rope_kv_append_norm(style, q_f, dk, dv, dwq, dwk, EPS, dp, kc_f, vc_f, rd, 5e5) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert torch.equal(q_f, q_sep) and torch.equal(kc_f, kc_sep) and torch.equal(vc_f, vc_sep)
    # v rows are the oracle quantiser's bytes of v
    want_v = torch.from_numpy(oracle.quant_q8_0(v.float())).view(B, L, Hkv, D // 32 * 34)
    for b, lo, n in ((0, 20, 28), (1, 0, 33)):
        assert torch.equal(vc_f[b, :, lo:lo + n].cpu(), want_v[b, :n].transpose(0, 1))


def test_one_weight_only_and_torch_op(kerns):
    B, L, Hq, Hkv, D, Lmax, rd = 2, 7, 8, 4, 128, 16, 64
    q, k, v, wq, wk, kc, vc = make(B, L, Hq, Hkv, D, Lmax, torch.float16, seed=5)
    p = torch.tensor([0, 9], dtype=torch.int32)
    dq, dk, dv, dwq, dwk, dp, dkc, dvc = (t.to(DEV) for t in (q, k, v, wq, wk, p, kc, vc))
    # only k is normalised: q must equal the plain producer's q, the cache the separate path's cache
    q_f, kc_f, vc_f = dq.clone(), dkc.clone(), dvc.clone()
    assert capi.rope_kv_append_norm(NEOX, q_f, dk, dv, None, dwk, EPS, dp, kc_f, vc_f, rd, 1e4) == capi.OK, capi.last_error()
    q_plain, kc_plain, vc_plain = dq.clone(), dkc.clone(), dvc.clone()
    assert capi.rope_kv_append(NEOX, q_plain, dk, dv, dp, kc_plain, vc_plain, rd, 1e4) == capi.OK
    _, kc_sep, _ = separate_ops(NEOX, dq, dk, dv, dwq, dwk, dp, dkc, dvc, rd, 1e4)
    torch.cuda.synchronize()
    assert torch.equal(q_f, q_plain) and torch.equal(kc_f, kc_sep) and torch.equal(vc_f, vc_plain)
    # the registered op gives the C ABI's bits, and keeps the argument checks
    q_c, kc_c, vc_c = dq.clone(), dkc.clone(), dvc.clone()
    assert capi.rope_kv_append_norm(IL, q_c, dk, dv, dwq, dwk, EPS, dp, kc_c, vc_c, rd, 1e4) == capi.OK
    q_o, kc_o, vc_o = dq.clone(), dkc.clone(), dvc.clone()
    assert kerns.rope_kv_append_norm(IL, rd, 1e4, EPS, q_o, dk, dv, dwq, dwk, dp, kc_o, vc_o) is None
    torch.cuda.synchronize()
    assert torch.equal(q_c, q_o) and torch.equal(kc_c, kc_o) and torch.equal(vc_c, vc_o)
    with pytest.raises(RuntimeError):
        kerns.rope_kv_append_norm(IL, rd, 1e4, EPS, q_o, dk, dv, dwq[:64], dwk, dp, kc_o, vc_o)
    with pytest.raises(RuntimeError):
        kerns.rope_kv_append_norm(IL, rd, 1e4, EPS, q_o, dk, dv, dwq.float(), dwk, dp, kc_o, vc_o)


def test_fused_norm_llama_shape_large_launch():
    """B=8, L=4096, 32/8 heads of 128 (805 MB touched: the launch streams past the caches): equal to the separate
    operators on every byte."""
    q, k, v, pos, kc, vc = workloads.kv_append(seed=3, device=DEV, B=8, L=4096, pos_hi=9)
    g = torch.Generator().manual_seed(3)
    wq = (1.0 + 0.3 * torch.randn(128, generator=g)).half().to(DEV)
    wk = (1.0 + 0.3 * torch.randn(128, generator=g)).half().to(DEV)
    q_sep, kc_sep, vc_sep = separate_ops(NEOX, q, k, v, wq, wk, pos, kc, vc, 128, 5e5)
    q_f = q.clone()
    assert capi.rope_kv_append_norm(NEOX, q_f, k, v, wq, wk, EPS, pos, kc, vc, 128, 5e5) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert torch.equal(q_f, q_sep) and torch.equal(kc, kc_sep) and torch.equal(vc, vc_sep)
