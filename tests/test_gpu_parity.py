"""GPU parity tests (-m gpu): the HIP kernels, called through the C ABI of libminfer_attn.so (and
through the registered torch ops), against the CPU oracle on identical seeded inputs.

Tolerances are the ones the task fixes: max-abs error <= 2e-3 for fp16 and <= 1e-2 for bf16 against
an fp32-or-better reference.  Masking and the GQA head mapping are checked for exact equality.
At the full benchmark sizes the oracle is evaluated on a sample of query rows (it is a scalar CPU
program) and the whole output is additionally compared with a plain fp32 torch evaluation of the
same formula on the GPU.
"""
import math

import numpy as np
import pytest
import torch

import capi
import oracle
import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float16: 2e-3, torch.bfloat16: 1e-2}


# ------------------------------------------------------------------------------------------------
def torch_ref(q, k, v, mask, row_chunk=1024):
    """softmax(q k^T / sqrt(D) | mask) v in fp32 on the GPU, a chunk of query rows at a time."""
    B, Hq, L, D = q.shape
    n_rep = Hq // k.shape[1]
    kf = k.float().repeat_interleave(n_rep, 1).transpose(-1, -2).contiguous()
    vf = v.float().repeat_interleave(n_rep, 1).contiguous()
    out = torch.empty(B, Hq, L, D, dtype=torch.float32, device=q.device)
    for lo in range(0, L, row_chunk):
        hi = min(lo + row_chunk, L)
        s = (q[:, :, lo:hi].float() @ kf) / math.sqrt(D)
        s.masked_fill_(~mask[:, :, lo:hi], float("-inf"))
        p = torch.nan_to_num(torch.softmax(s, -1), nan=0.0)
        out[:, :, lo:hi] = p @ vf
    return out


def run_prefill(q, k, v, mask, out=None):
    if out is None:
        out = torch.full(q.shape, float("nan"), dtype=q.dtype, device=q.device)
    rc = capi.flash_attn(q, k, v, mask, out)
    assert rc == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    return out


def max_err(a, b):
    return float((torch.as_tensor(a).float().cpu() - torch.as_tensor(b).float().cpu()).abs().max())


def make_mask(kind, B, L, gen):
    i = torch.arange(L)
    if kind == "causal":
        m = (i[None, :] <= i[:, None])[None].expand(B, L, L)
    elif kind == "window":
        m = ((i[None, :] - i[:, None]).abs() < 37)[None].expand(B, L, L)
    elif kind == "full":
        m = torch.ones(B, L, L, dtype=torch.bool)
    elif kind == "random":       # different per batch element, with rows that attend nothing
        m = torch.rand(B, L, L, generator=gen) < 0.5
        m[:, L // 3, :] = False
    elif kind == "blocky":       # whole 64x64 tiles switched off, to exercise tile skipping with holes
        t = (L + 63) // 64
        tiles = torch.rand(B, t, t, generator=gen) < 0.5
        tiles[:, :, 0] = True
        m = tiles.repeat_interleave(64, 1).repeat_interleave(64, 2)[:, :L, :L]
    return m[:, None].contiguous()


# ------------------------------------------------------------------------------------------------
# golden vectors (pin: torch SDPA on the reference's call, see tests/golden/make_golden.py)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["dense_causal_b1_h4_kv2_l16_d64", "dense_window_b2_h6_kv2_l40_d128",
                                  "dense_random_b1_h8_kv1_l70_d64"])
def test_golden_dense(name):
    z = np.load(f"{capi.ROOT}/tests/golden/{name}.npz")
    q, k, v = (torch.from_numpy(z[n]).to(DEV) for n in ("q", "k", "v"))
    out = run_prefill(q, k, v, torch.from_numpy(z["mask"]).to(DEV))
    assert max_err(out, z["out"]) <= TOL[torch.float16]


def test_golden_decode_and_varlen():
    z = np.load(f"{capi.ROOT}/tests/golden/decode_b3_h8_kv2_l50_d128.npz")
    q, k, v = (torch.from_numpy(z[n]).to(DEV) for n in ("q", "k", "v"))
    out = torch.full(q.shape, float("nan"), dtype=q.dtype, device=DEV)
    assert capi.flash_attn_decode(q, k, v, torch.from_numpy(z["ctx"]).to(DEV), out) == capi.OK, capi.last_error()
    assert max_err(out, z["out"]) <= TOL[torch.float16]
    z = np.load(f"{capi.ROOT}/tests/golden/varlen_h4_kv2_d64.npz")
    q, k, v = (torch.from_numpy(z[n]).to(DEV) for n in ("q", "k", "v"))
    out = torch.full(q.shape, float("nan"), dtype=q.dtype, device=DEV)
    assert capi.flash_attn_varlen(q, k, v, torch.from_numpy(z["cu"]).to(DEV), 70, out) == capi.OK, capi.last_error()
    assert max_err(out, z["out"]) <= TOL[torch.float16]


# ------------------------------------------------------------------------------------------------
# dense prefill against the oracle: shapes, masks, dtypes, layouts
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,Hq,Hkv,L,D,kind,views", [
    (1, 8, 2, 256, 64, "causal", False),     # benchmark configuration 1 shape
    (2, 8, 2, 320, 128, "causal", True),     # reference-style transposed views
    (2, 6, 2, 200, 128, "window", False),    # n_rep = 3, symmetric window (reference test case B)
    (2, 4, 4, 333, 128, "random", False),    # L % 4 != 0: byte-wise mask path, per-batch masks
    (1, 16, 2, 520, 64, "random", True),     # n_rep = 8
    (1, 12, 2, 136, 128, "blocky", False),   # n_rep = 6
    (1, 16, 1, 264, 128, "causal", False),   # n_rep = 16
    (1, 2, 2, 1, 128, "full", False),        # single token
    (1, 4, 2, 63, 64, "causal", False),
    (3, 4, 1, 65, 128, "full", False),
    (1, 4, 1, 1040, 128, "blocky", False),
    # above 1024 rows the launch uses 8-wave workgroups (4-wave ones below): the same kinds of edges there
    (1, 6, 2, 1093, 128, "random", False),   # n_rep = 3, byte-wise mask path
    (1, 8, 1, 1100, 64, "window", True),     # n_rep = 8, D = 64, transposed views
    (2, 4, 4, 1029, 128, "causal", False),   # n_rep = 1, a last tile of 5 rows
])
def test_dense_matches_oracle(dtype, B, Hq, Hkv, L, D, kind, views):
    gen = torch.Generator().manual_seed(1000 * L + D + Hq)
    q, k, v = workloads.dense_prefill(B, Hq, Hkv, L, D, dtype, seed=L + Hq, scale=0.5, views=views, device=DEV)
    q = q * 2 if dtype == torch.float16 else q   # fp16: logits with a wider spread
    mask = make_mask(kind, B, L, gen)
    out = run_prefill(q, k, v, mask.to(DEV))
    want = oracle.flash_attn(q, k, v, mask)
    assert not torch.isnan(out).any()
    assert max_err(out, want) <= TOL[dtype]


@pytest.mark.parametrize("B,Hq,Hkv,L,D,kind", [
    (1, 4, 4, 16, 128, "random"),      # n_rep = 1: four query blocks per workgroup, of which one has rows
    (2, 4, 2, 48, 64, "full"),         # n_rep = 2
    (1, 6, 2, 208, 128, "window"),     # n_rep = 3
    (2, 8, 2, 320, 128, "blocky"),     # n_rep = 4, key tiles that no row of a query block attends
    (1, 16, 2, 512, 64, "random"),     # n_rep = 8: two head groups
    (1, 16, 1, 1008, 128, "blocky"),   # n_rep = 16, a last key tile of 48 columns
    (1, 8, 2, 1024, 128, "random"),    # the longest mask whose rows one wave-wide load covers
    (3, 32, 8, 512, 128, "blocky"),    # more workgroups than fit on the chip at once: the pre-pass classifies
])
def test_short_dense_masks_classified_inside_the_kernel(B, Hq, Hkv, L, D, kind):
    """A short dense problem with 16-byte readable mask rows launches no classification pre-pass: each workgroup
    classifies its own mask rows.  Checked against the oracle, and bit for bit against the same call with the mask at an
    odd address, which takes the pre-pass and the byte-wise mask reads."""
    dtype = torch.float16
    gen = torch.Generator().manual_seed(77 * L + Hq)
    q, k, v = workloads.dense_prefill(B, Hq, Hkv, L, D, dtype, seed=L + Hq + 1, scale=0.5, device=DEV)
    mask = make_mask(kind, B, L, gen)
    md = mask.to(DEV)
    out = run_prefill(q, k, v, md)
    assert not torch.isnan(out).any()
    assert max_err(out, oracle.flash_attn(q, k, v, mask)) <= TOL[dtype]
    shifted = torch.zeros(md.numel() + 1, dtype=torch.bool, device=DEV)[1:].view(md.shape)
    shifted.copy_(md)
    assert shifted.data_ptr() % 16 == 1
    assert torch.equal(run_prefill(q, k, v, shifted), out)


def test_cpu_plumbing_config_on_gpu():
    """benchmark configuration 1 (fp32 N(0,1) inputs, S=256, D=64): the same seeded inputs rounded to fp16."""
    q, k, v, mask = workloads.cpu_plumbing(seed=0)
    want = oracle.flash_attn(q.half(), k.half(), v.half(), mask)
    out = run_prefill(q.half().to(DEV), k.half().to(DEV), v.half().to(DEV), mask.to(DEV))
    assert out.shape == (1, 8, 256, 64)
    assert max_err(out, want) <= TOL[torch.float16]


def test_strided_out_and_determinism():
    B, Hq, Hkv, L, D = 2, 8, 2, 192, 128
    q, k, v = workloads.dense_prefill(B, Hq, Hkv, L, D, torch.float16, seed=5, views=True, device=DEV)
    mask = workloads.causal_mask(B, L, device=DEV)
    a = run_prefill(q, k, v, mask)
    out_t = torch.full((B, L, Hq, D), float("nan"), dtype=torch.float16, device=DEV).transpose(1, 2)
    b = run_prefill(q, k, v, mask, out=out_t)
    assert torch.equal(a, b)
    assert torch.equal(a, run_prefill(q, k, v, mask))
    assert max_err(a, oracle.flash_attn(q, k, v, mask)) <= TOL[torch.float16]


# ------------------------------------------------------------------------------------------------
# exact properties: masking and GQA mapping are bit-identical
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_masking_and_gqa_mapping_exact(dtype):
    B, Hq, Hkv, L, D = 2, 8, 2, 200, 128
    gen = torch.Generator().manual_seed(9)
    q, k, v = workloads.dense_prefill(B, Hq, Hkv, L, D, dtype, seed=9, scale=1.0, device=DEV)
    n_rep = Hq // Hkv
    # one attended key per row: the output row is that V row, bit for bit
    sel = torch.randint(0, L, (B, L), generator=gen)
    onehot = torch.zeros(B, L, L, dtype=torch.bool)
    onehot.scatter_(2, sel[:, :, None], True)
    out = run_prefill(q, k, v, onehot[:, None].contiguous().to(DEV))
    for b in range(B):
        for h in range(Hq):
            assert torch.equal(out[b, h], v[b, h // n_rep, sel[b].to(DEV)])
    # causal: row 0 is V row 0
    out = run_prefill(q, k, v, workloads.causal_mask(B, L, device=DEV))
    for h in range(Hq):
        assert torch.equal(out[:, h, 0], v[:, h // n_rep, 0])
    # V constant per KV head: every row of query head h equals the constant of KV head h // n_rep
    vc = torch.empty_like(v)
    for g in range(Hkv):
        vc[:, g] = float(g + 1)
    out = run_prefill(q, k, vc, workloads.causal_mask(B, L, device=DEV))
    for h in range(Hq):
        assert torch.equal(out[:, h], torch.full_like(out[:, h], float(h // n_rep + 1)))
    # rows that attend nothing give zeros, their neighbours are unaffected
    m = workloads.causal_mask(B, L)
    m[:, :, 70, :] = False
    out2 = run_prefill(q, k, v, m.to(DEV))
    assert torch.all(out2[:, :, 70] == 0)
    ref = run_prefill(q, k, v, workloads.causal_mask(B, L, device=DEV))
    keep = torch.arange(L) != 70
    assert torch.equal(out2[:, :, keep], ref[:, :, keep])


# ------------------------------------------------------------------------------------------------
# the benchmark configurations at full size
# ------------------------------------------------------------------------------------------------
def sample_rows(L, n, gen):
    fixed = [0, 1, 31, 32, 63, 64, 65, L // 2, L - 65, L - 2, L - 1]
    extra = torch.randint(0, L, (n,), generator=gen).tolist()
    return sorted(set(r for r in fixed + extra if 0 <= r < L))


@pytest.mark.parametrize("views", [False, True])
def test_llama8b_prefill_full(views):
    """benchmark configuration 2: B=1, Hq=32, Hkv=8, S=4096, D=128, fp16, causal, 0.5*N(0,1)."""
    q, k, v, mask = workloads.llama8b_prefill(seed=0, device=DEV, views=views)
    out = run_prefill(q, k, v, mask)
    assert max_err(out, torch_ref(q, k, v, mask)) <= TOL[torch.float16]
    rows = sample_rows(4096, 150, torch.Generator().manual_seed(1))
    want = oracle.flash_attn_rows(q, k, v, mask[:, 0, rows].cpu(), rows)
    assert max_err(out[:, :, rows], want) <= TOL[torch.float16]
    assert torch.equal(out[0, :, 0], v[0].repeat_interleave(4, 0)[:, 0])


def test_long_context_prefill_full():
    """benchmark configuration 4: B=1, Hq=32, Hkv=8, S=32768, D=128, bf16, causal, 0.5*N(0,1)."""
    L = 32768
    q, k, v, mask = workloads.long_context_prefill(seed=0, device=DEV, L=L)
    out = run_prefill(q, k, v, mask)
    rows = sample_rows(L, 40, torch.Generator().manual_seed(2))
    want = oracle.flash_attn_rows(q, k, v, mask[:, 0, rows].cpu(), rows)
    assert max_err(out[:, :, rows], want) <= TOL[torch.bfloat16]
    assert torch.equal(out[0, :, 0], v[0].repeat_interleave(4, 0)[:, 0])
    assert max_err(out, torch_ref(q, k, v, mask, row_chunk=512)) <= TOL[torch.bfloat16]


def test_decode_full():
    """benchmark configuration 3: B=64, Hq=32, Hkv=8, D=128, fp16, ctx in [512, 8192], cache [B,Hkv,8192,128]."""
    q, kc, vc, ctx = workloads.decode_cache(seed=0, device=DEV)
    # rows beyond ctx are garbage that must not reach the result
    for b in range(0, 64, 7):
        kc[b, :, int(ctx[b]):] = float("nan")
        vc[b, :, int(ctx[b]):] = float("inf")
    out = torch.full(q.shape, float("nan"), dtype=q.dtype, device=DEV)
    assert capi.flash_attn_decode(q, kc, vc, ctx, out) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert not torch.isnan(out).any()
    want = oracle.flash_attn_decode(q, kc, vc, ctx)
    assert max_err(out, want) <= TOL[torch.float16]


def test_ragged_prefill_full():
    """benchmark configuration 5: 16 sequences, lengths in [128, 2048], Hq=64, Hkv=8, D=128, fp16, N(0,1)."""
    q, k, v, cu = workloads.ragged_prefill(seed=0, device=DEV)
    lens = (cu[1:] - cu[:-1]).tolist()
    out = torch.full(q.shape, float("nan"), dtype=q.dtype, device=DEV)
    assert capi.flash_attn_varlen(q, k, v, cu, max(lens), out) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert not torch.isnan(out).any()
    worst, lo = 0.0, 0
    for n in lens:
        m = workloads.causal_mask(1, n, device=DEV)
        worst = max(worst, max_err(out[:, :, lo:lo + n], torch_ref(q[:, :, lo:lo + n], k[:, :, lo:lo + n], v[:, :, lo:lo + n], m)))
        lo += n
    assert worst <= TOL[torch.float16]
    # the shortest sequence in full against the oracle
    s = int(np.argmin(lens))
    lo, hi = int(cu[s]), int(cu[s + 1])
    want = oracle.flash_attn(q[:, :, lo:hi], k[:, :, lo:hi], v[:, :, lo:hi], workloads.causal_mask(1, hi - lo))
    assert max_err(out[:, :, lo:hi], want) <= TOL[torch.float16]


# ------------------------------------------------------------------------------------------------
# decode and varlen edge cases against the oracle
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,Hq,Hkv,Lmax,D,lo,hi", [
    (2, 8, 2, 256, 128, 1, 256),
    (5, 8, 2, 1000, 64, 0, 1000),      # ctx = 0 allowed, Lmax not a multiple of 16
    (2, 40, 2, 700, 128, 500, 700),    # n_rep = 20: two head groups
    (3, 6, 6, 1537, 128, 1537, 1537),  # ctx = Lmax, n_rep = 1, 4 chunks with a 1-row tail
    (4, 4, 1, 17, 64, 1, 17),
    (3, 8, 2, 0, 128, 0, 0),           # an empty cache: zeros, with the workspace size the library reports for it
])
def test_decode_matches_oracle(dtype, B, Hq, Hkv, Lmax, D, lo, hi):
    scale = 1.0 if dtype == torch.float16 else 0.5
    q, kc, vc, ctx = workloads.decode_cache(seed=Lmax, device="cpu", B=B, Hq=Hq, Hkv=Hkv, Lmax=Lmax, D=D, dtype=dtype,
                                            ctx_lo=lo, ctx_hi=hi)
    vc = (vc.float() * scale).to(dtype)
    out = torch.full(q.shape, float("nan"), dtype=dtype, device=DEV)
    assert capi.flash_attn_decode(q.to(DEV), kc.to(DEV), vc.to(DEV), ctx.to(DEV), out) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert max_err(out, oracle.flash_attn_decode(q, kc, vc, ctx)) <= TOL[dtype]
    assert torch.all(out[ctx.to(DEV) == 0] == 0)


@pytest.mark.parametrize("B,Hq,Hkv,Lmax,D,ctx", [
    (200, 8, 2, 64, 64, "tiny"),          # shares of the work span many short sequences, some empty; B > 64
    (1, 4, 1, 40000, 128, "full"),        # one (sequence, KV head) cut into ~57 shares: as many partials per row
    (70, 40, 2, 1000, 128, "gaps"),       # empty sequences at both ends and in between, two head groups
    (3, 16, 16, 5000, 64, "full"),
])
def test_decode_work_is_shared_out_evenly_whatever_the_lengths(B, Hq, Hkv, Lmax, D, ctx):
    g = torch.Generator().manual_seed(B + Lmax)
    q = torch.randn(B, Hq, 1, D, generator=g).half()
    kc = torch.randn(B, Hkv, Lmax, D, generator=g).half()
    vc = torch.randn(B, Hkv, Lmax, D, generator=g).half()
    if ctx == "tiny":
        lens = torch.randint(0, 41, (B,), generator=g, dtype=torch.int32)
    elif ctx == "full":
        lens = torch.full((B,), Lmax, dtype=torch.int32)
    else:
        lens = torch.randint(1, Lmax + 1, (B,), generator=g, dtype=torch.int32)
        lens[:3] = 0
        lens[-2:] = 0
        lens[10:40:7] = 0
    out = torch.full(q.shape, float("nan"), dtype=q.dtype, device=DEV)
    assert capi.flash_attn_decode(q.to(DEV), kc.to(DEV), vc.to(DEV), lens.to(DEV), out) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert max_err(out, oracle.flash_attn_decode(q, kc, vc, lens)) <= TOL[torch.float16]
    assert torch.all(out[lens.to(DEV) == 0] == 0)
    # the same caches as Q8_0 blocks
    kq, vq = torch.from_numpy(oracle.quant_q8_0(kc.float())), torch.from_numpy(oracle.quant_q8_0(vc.float()))
    out8 = torch.full(q.shape, float("nan"), dtype=q.dtype, device=DEV)
    assert capi.flash_attn_decode_q8_0(q.to(DEV), kq.to(DEV), vq.to(DEV), lens.to(DEV), out8) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert max_err(out8, oracle.flash_attn_decode_q8_0(q, kq, vq, lens)) <= TOL[torch.float16]
    assert torch.all(out8[lens.to(DEV) == 0] == 0)


def test_decode_equals_last_prefill_row():
    """Splitting the KV range and merging by log-sum-exp must not change the result: the decode of
    position ctx-1 equals the last row of a causal prefill over the same ctx rows."""
    B, Hq, Hkv, Lmax, D = 1, 8, 2, 2048, 128
    q, k, v = workloads.dense_prefill(B, Hq, Hkv, Lmax, D, torch.float16, seed=21, device=DEV)
    pre = run_prefill(q, k, v, workloads.causal_mask(B, Lmax, device=DEV))
    for ctx_len in (1, 511, 512, 513, 2048):
        out = torch.empty(B, Hq, 1, D, dtype=torch.float16, device=DEV)
        ctx = torch.tensor([ctx_len], dtype=torch.int32, device=DEV)
        assert capi.flash_attn_decode(q[:, :, ctx_len - 1:ctx_len].contiguous(), k, v, ctx, out) == capi.OK
        assert max_err(out[:, :, 0], pre[:, :, ctx_len - 1]) <= 1e-3


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv,D,lens", [
    (8, 2, 128, [5, 64, 100, 1, 257]),
    (8, 1, 64, [130, 31, 0, 77]),
    (6, 2, 128, [1, 1, 1]),
    (4, 4, 64, [300]),
    (8, 2, 128, [(7 * i) % 41 for i in range(150)]),      # more sequences than a wave has lanes, some empty
    (8, 2, 64, [700, 333, 0, 20, 64, 1]),
])
def test_varlen_matches_oracle_and_dense(dtype, Hq, Hkv, D, lens):
    g = torch.Generator().manual_seed(sum(lens))
    T = sum(lens)
    q = torch.randn(1, Hq, T, D, generator=g).to(dtype)
    k = torch.randn(1, Hkv, T, D, generator=g).to(dtype)
    v = (0.5 * torch.randn(1, Hkv, T, D, generator=g)).to(dtype)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
    out = torch.full(q.shape, float("nan"), dtype=dtype, device=DEV)
    assert capi.flash_attn_varlen(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), max(lens), out) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert max_err(out, oracle.flash_attn_varlen(q, k, v, cu)) <= TOL[dtype]
    # max_seqlen chooses the workgroup shape (4 waves up to 1024 rows, 8 above; 0 = not known = T): the same bits either way
    out0 = torch.full(q.shape, float("nan"), dtype=dtype, device=DEV)
    assert capi.flash_attn_varlen(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), 0, out0) == capi.OK, capi.last_error()
    out_big = torch.full(q.shape, float("nan"), dtype=dtype, device=DEV)
    assert capi.flash_attn_varlen(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), 5000, out_big) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert torch.equal(out0, out) and torch.equal(out_big, out)
    # same result as the reference-signature op under the block-diagonal causal mask
    blk = torch.zeros(T, T, dtype=torch.bool)
    for lo, hi in zip(cu[:-1].tolist(), cu[1:].tolist()):
        blk[lo:hi, lo:hi] = torch.ones(hi - lo, hi - lo, dtype=torch.bool).tril()
    dense = run_prefill(q.to(DEV), k.to(DEV), v.to(DEV), blk[None, None].contiguous().to(DEV))
    # (two bf16 results may round an element above 1 to neighbouring values, 2^-7 apart)
    one_ulp = float(dense.float().abs().max()) * 2.0 ** -8 if dtype == torch.bfloat16 else 0.0
    assert max_err(out, dense) <= TOL[dtype] / 2 + one_ulp


def test_varlen_malformed_cu_seqlens_stay_in_bounds():
    """cu_seqlens lives on the device and is never checked by the host: a decreasing entry, a negative one and one
    past T must not move any access outside q/k/v/out.  The tensors are views with guard rows on both sides of every
    head (NaN in q/k/v, which would poison any result that read them; a sentinel in out); sequences that are valid
    and overlap no other come out as the oracle computes them."""
    Hq, Hkv, D, T, G = 8, 2, 128, 600, 96
    g = torch.Generator().manual_seed(77)

    def guarded(H, fill, scale=1.0):
        buf = torch.full((1, H, T + 2 * G, D), fill, dtype=torch.float16)
        buf[:, :, G:G + T] = (scale * torch.randn(1, H, T, D, generator=g)).to(torch.float16)
        buf = buf.to(DEV)
        return buf, buf[:, :, G:G + T]

    qb, q = guarded(Hq, float("nan"))
    kb, k = guarded(Hkv, float("nan"))
    vb, v = guarded(Hkv, float("nan"), 0.5)
    ob = torch.full((1, Hq, T + 2 * G, D), 7.0, dtype=torch.float16, device=DEV)
    out = ob[:, :, G:G + T]
    # sequence 0 = rows [0,200); 1 ends before it starts (empty); 2 = [150,400) overlaps the end of 0; 3 starts at 400
    # and claims rows far past T (cut to [400,600)); 4 starts past T (empty); 5 has a negative start and end (empty)
    cu = torch.tensor([0, 200, 150, 400, 2_000_000_000, -5, -3], dtype=torch.int32, device=DEV)
    assert capi.flash_attn_varlen(q, k, v, cu, 0, out) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert torch.all(ob[:, :, :G] == 7.0) and torch.all(ob[:, :, G + T:] == 7.0)     # guard rows of out untouched
    assert not torch.isnan(out).any()                                                 # no guard row of q/k/v was read
    qc, kc, vc = q.cpu(), k.cpu(), v.cpu()
    for lo, hi, rows in [(0, 200, slice(0, 150)), (150, 400, slice(50, 250)), (400, 600, slice(0, 200))]:
        want = oracle.flash_attn(qc[:, :, lo:hi], kc[:, :, lo:hi], vc[:, :, lo:hi], workloads.causal_mask(1, hi - lo))
        assert max_err(out[:, :, lo:hi][:, :, rows], want[:, :, rows]) <= TOL[torch.float16]
    # the same with max_seqlen given: rows of a sequence past it are left alone, the others are as before
    ob.fill_(7.0)
    assert capi.flash_attn_varlen(q, k, v, cu, 100, out) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert torch.all(ob[:, :, :G] == 7.0) and torch.all(ob[:, :, G + T:] == 7.0)
    assert torch.all(out[:, :, 500:] == 7.0)                                          # rows 100.. of the last sequence
    want = oracle.flash_attn(qc[:, :, 400:500], kc[:, :, 400:500], vc[:, :, 400:500], workloads.causal_mask(1, 100))
    assert max_err(out[:, :, 400:500], want) <= TOL[torch.float16]


# ------------------------------------------------------------------------------------------------
# the registered torch ops (the reference's call path) give the same bits and the same errors
# ------------------------------------------------------------------------------------------------
def test_torch_ops_match_c_abi(kerns):
    from minfer.const import GGML_QUANT_SIZES, GGMLQuantizationType
    qt = GGMLQuantizationType.F16
    qb, qs = GGML_QUANT_SIZES[qt]
    B, Hq, Hkv, L, D = 2, 12, 2, 300, 128
    q, k, v = workloads.dense_prefill(B, Hq, Hkv, L, D, torch.float16, seed=31, views=True, device=DEV)
    mask = workloads.window_mask(B, L, 100, device=DEV)
    a = torch.zeros(B, Hq, L, D, dtype=torch.float16, device=DEV)
    kerns.flash_attn(qt, qb, qs, q, k, v, mask, a)           # reference call shape: test/kernels.py:246-248
    torch.cuda.synchronize()
    assert torch.equal(a, run_prefill(q, k, v, mask))

    qd, kc, vc, ctx = workloads.decode_cache(seed=3, device=DEV, B=4, Lmax=1024, ctx_lo=1, ctx_hi=1024)
    a = torch.zeros_like(qd)
    kerns.flash_attn_decode(qt, qb, qs, qd, kc, vc, ctx, a)
    b = torch.zeros_like(qd)
    assert capi.flash_attn_decode(qd, kc, vc, ctx, b) == capi.OK
    torch.cuda.synchronize()
    assert torch.equal(a, b)

    qv, kv, vv, cu = workloads.ragged_prefill(seed=3, device=DEV, n_seqs=4, len_lo=1, len_hi=200, Hq=8, Hkv=2)
    a = torch.zeros_like(qv)
    kerns.flash_attn_varlen(qt, qb, qs, qv, kv, vv, cu, 200, a)
    b = torch.zeros_like(qv)
    assert capi.flash_attn_varlen(qv, kv, vv, cu, 200, b) == capi.OK
    torch.cuda.synchronize()
    assert torch.equal(a, b)


def test_torch_op_validation(kerns):
    """The checks of the reference host function (flash_attn/op.cuh:32-96) raise RuntimeError."""
    B, Hq, Hkv, L, D = 1, 4, 2, 64, 128
    q, k, v = workloads.dense_prefill(B, Hq, Hkv, L, D, torch.float16, seed=1, device=DEV)
    mask = workloads.causal_mask(B, L, device=DEV)
    out = torch.empty_like(q)
    args = lambda **kw: [1, 1, 2] + [kw.get(n, d) for n, d in (("q", q), ("k", k), ("v", v), ("mask", mask), ("out", out))]
    with pytest.raises(RuntimeError):
        kerns.flash_attn(*args(q=q.float()))                                   # dtype
    with pytest.raises(RuntimeError):
        kerns.flash_attn(*args(mask=mask.to(torch.uint8)))                     # mask dtype
    with pytest.raises(RuntimeError):
        kerns.flash_attn(*args(mask=mask.expand(B, 1, L, L).transpose(2, 3)))  # mask not contiguous
    with pytest.raises(RuntimeError):
        kerns.flash_attn(*args(q=q[..., ::2].repeat_interleave(2, -1)[..., ::1].transpose(2, 3).transpose(2, 3)[:, :, :, :64]))  # head_dim 64 vs k 128
    with pytest.raises(RuntimeError):
        kerns.flash_attn(*args(k=k[:, :, :32]))                                # Lk != Lq
    with pytest.raises(RuntimeError):
        kerns.flash_attn(*args(out=out[0]))                                    # rank
    with pytest.raises(RuntimeError):
        kerns.flash_attn(*args(v=v.transpose(1, 2).contiguous().transpose(1, 2)))  # k/v strides differ
    with pytest.raises(RuntimeError):
        kerns.flash_attn(*args(mask=mask.cpu()))                               # device
    kerns.flash_attn(*args())                                                  # and the good call passes
    torch.cuda.synchronize()
