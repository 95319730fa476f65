"""GPU parity tests (-m gpu) of the Q8_0 path through the C ABI: the block quantiser and dequantiser, decode
attention over Q8_0 caches, and the rope + cache append that writes them.

Bars: quantised bytes and dequantised values are integer/bit work and must equal the CPU oracle's exactly
(the oracle equals the reference's own quantiser source byte for byte, tests/test_oracle_quant.py); decode over
Q8_0 caches must be within the fp16 attention tolerance (max-abs 2e-3) of the oracle, which dequantises the
caches as the reference's device dequantiser does and attends in fp64.  The reference's own test of this
format round-trips rows of 6144 values through its CPU quantiser and compares the device dequantiser with the
CPU one (reference: test/kernels.py:24-56); test_round_trip_as_the_reference_tests_it is that test."""
import numpy as np
import pytest
import torch

import capi
import oracle
import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = 2e-3


def gpu_quant(x):
    k = x.shape[-1]
    y = torch.full(x.shape[:-1] + (k // 32 * 34,), 0xAB, dtype=torch.uint8, device=DEV)
    assert capi.quant_q8_0(x.to(DEV), y) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    return y


def gpu_dequant(y, dtype):
    out = torch.full(y.shape[:-1] + (y.shape[-1] // 34 * 32,), float("nan"), dtype=dtype, device=DEV)
    assert capi.dequant_q8_0(y.to(DEV), out) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    return out


def rows(seed, shape, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


@pytest.mark.parametrize("shape,scale", [((1024, 6144), 1.0), ((3, 32), 1.0), ((7, 5, 96), 40.0), ((130, 2048), 1e-3),
                                         ((1, 64 * 1031), 1.0)])
def test_quant_bytes_equal_oracle(shape, scale):
    x = rows(sum(shape), shape, scale)
    x.view(-1)[:32] = 0.0                                                   # a zero block
    x.view(-1)[32:40] = torch.tensor([0.5, -0.5, 1.5, -1.5, 2.5, 127.0, 63.5, -63.5])   # ties
    want = oracle.quant_q8_0(x)
    got = gpu_quant(x).cpu().numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_quant_of_16_bit_input_quantises_its_values(dtype):
    x = rows(11, (64, 512), 3.0).to(dtype)
    assert np.array_equal(gpu_quant(x).cpu().numpy(), oracle.quant_q8_0(x.float()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_dequant_bits_equal_oracle(dtype):
    np_dtype = np.float32 if dtype == torch.float32 else np.float16
    y = oracle.quant_q8_0(rows(5, (257, 1024), 2.0))
    got = gpu_dequant(torch.from_numpy(y), dtype).cpu().numpy()
    want = oracle.dequant_q8_0(y, np_dtype)
    assert np.array_equal(got.view(np.uint32 if dtype == torch.float32 else np.uint16),
                          want.view(np.uint32 if dtype == torch.float32 else np.uint16))
    # arbitrary quants under finite scales of every size, subnormal ones included
    g = np.random.default_rng(3)
    raw = g.integers(0, 256, (96, 8 * 34), dtype=np.uint8)
    sc = (g.standard_normal((96, 8)) * np.exp2(g.integers(-24, 8, (96, 8)))).astype(np.float16)
    raw.reshape(96, 8, 34)[:, :, :2] = sc.view(np.uint8).reshape(96, 8, 2)
    got = gpu_dequant(torch.from_numpy(raw), dtype).cpu().numpy()
    want = oracle.dequant_q8_0(raw, np_dtype)
    assert np.array_equal(got, want) and np.array_equal(np.signbit(got), np.signbit(want))


@pytest.mark.parametrize("shape", [(1024, 6144), (16384, 6144)])
def test_round_trip_as_the_reference_tests_it(shape):
    # reference: test/kernels.py:24-56 (quantise on the CPU, dequantise on both sides, compare)
    data = torch.randn(shape, generator=torch.Generator().manual_seed(shape[0]))
    quantized = torch.from_numpy(oracle.quant_q8_0(data))
    expected = torch.from_numpy(oracle.dequant_q8_0(quantized.numpy()))
    actual = gpu_dequant(quantized, torch.float32)
    assert torch.equal(actual.cpu(), expected)
    # and the device quantiser writes the same bytes
    assert torch.equal(gpu_quant(data).cpu(), quantized)


# ------------------------------------------------------------------------------------------------
# decode attention over Q8_0 caches
# ------------------------------------------------------------------------------------------------
def q8_cache(seed, B, Hkv, Lmax, D, scale=1.0):
    return torch.from_numpy(oracle.quant_q8_0(rows(seed, (B, Hkv, Lmax, D), scale)))


def run_decode_q8(q, kq, vq, ctx):
    out = torch.full(q.shape, float("nan"), dtype=q.dtype, device=DEV)
    assert capi.flash_attn_decode_q8_0(q, kq, vq, ctx, out) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("B,Hq,Hkv,Lmax,D,lo,hi", [
    (2, 8, 2, 256, 128, 1, 256),
    (5, 8, 2, 1000, 64, 0, 1000),      # ctx = 0 allowed, Lmax not a multiple of 16
    (2, 40, 2, 700, 128, 500, 700),    # n_rep = 20: two head groups
    (3, 6, 6, 1537, 128, 1537, 1537),  # ctx = Lmax, n_rep = 1, chunks with a 1-row tail
    (4, 4, 1, 17, 64, 1, 17),
    (3, 32, 8, 2500, 128, 100, 2500),
])
def test_decode_q8_matches_oracle_and_fp16_path(B, Hq, Hkv, Lmax, D, lo, hi):
    g = torch.Generator().manual_seed(Lmax)
    q = torch.randn(B, Hq, 1, D, generator=g).half()
    ctx = torch.randint(lo, hi + 1, (B,), generator=g, dtype=torch.int32)
    kq, vq = q8_cache(Lmax, B, Hkv, Lmax, D), q8_cache(Lmax + 1, B, Hkv, Lmax, D)
    out = run_decode_q8(q.to(DEV), kq.to(DEV), vq.to(DEV), ctx.to(DEV))
    want = oracle.flash_attn_decode_q8_0(q, kq, vq, ctx)
    assert float(np.abs(out.float().cpu().numpy() - want).max()) <= TOL
    assert torch.all(out[ctx.to(DEV) == 0] == 0)
    # the fp16 decode kernel over the device-dequantised caches computes the same thing in another order
    k16, v16 = gpu_dequant(kq, torch.float16), gpu_dequant(vq, torch.float16)
    out16 = torch.full(q.shape, float("nan"), dtype=q.dtype, device=DEV)
    assert capi.flash_attn_decode(q.to(DEV), k16, v16, ctx.to(DEV), out16) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert float((out.float() - out16.float()).abs().max()) <= TOL


def test_decode_q8_ignores_rows_past_ctx_and_takes_strided_caches():
    B, Hq, Hkv, Lmax, D = 4, 16, 4, 600, 128
    g = torch.Generator().manual_seed(1)
    q = torch.randn(B, Hq, 1, D, generator=g).half().to(DEV)
    ctx = torch.tensor([1, 333, 600, 47], dtype=torch.int32)
    # caches as views of a larger allocation: batch and head strides are not the dense ones
    big_k = torch.zeros(B, Hkv + 1, Lmax + 6, D // 32 * 34, dtype=torch.uint8)
    big_v = torch.zeros_like(big_k)
    kq, vq = big_k[:, 1:, :Lmax], big_v[:, :Hkv, 6:]
    kq.copy_(q8_cache(2, B, Hkv, Lmax, D))
    vq.copy_(q8_cache(3, B, Hkv, Lmax, D, 2.0))
    want = oracle.flash_attn_decode_q8_0(q, kq, vq, ctx)
    for b in range(B):   # rows past ctx: NaN scales and wild quants that must not reach the result
        kq[b, :, int(ctx[b]):] = 0xFF
        vq[b, :, int(ctx[b]):] = 0x7F
    dk, dv = big_k.to(DEV), big_v.to(DEV)
    out = run_decode_q8(q, dk[:, 1:, :Lmax], dv[:, :Hkv, 6:], ctx.to(DEV))
    assert not torch.isnan(out).any()
    assert float(np.abs(out.float().cpu().numpy() - want).max()) <= TOL


def test_decode_q8_full():
    """The decode benchmark's shape (B=64, Hq=32, Hkv=8, D=128, ctx in [512, 8192], Lmax 8192) over Q8_0 caches:
    the caches are quantised on the device, the oracle checks a sample of sequences and the fp16 decode kernel over
    the dequantised caches checks all of them."""
    q, kc, vc, ctx = workloads.decode_cache(seed=0, device=DEV)
    kq, vq = gpu_quant(kc), gpu_quant(vc)
    del kc, vc
    out = run_decode_q8(q, kq, vq, ctx)
    assert not torch.isnan(out).any()
    k16, v16 = gpu_dequant(kq, torch.float16), gpu_dequant(vq, torch.float16)
    out16 = torch.full(q.shape, float("nan"), dtype=q.dtype, device=DEV)
    assert capi.flash_attn_decode(q, k16, v16, ctx, out16) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert float((out.float() - out16.float()).abs().max()) <= TOL
    pick = [0, 17, 40, 63]
    want = oracle.flash_attn_decode_q8_0(q[pick].cpu(), kq[pick].cpu(), vq[pick].cpu(), ctx[pick].cpu())
    assert float(np.abs(out[pick].float().cpu().numpy() - want).max()) <= TOL


# ------------------------------------------------------------------------------------------------
# rope + append into Q8_0 caches
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("style", [capi.ROPE_INTERLEAVED, capi.ROPE_NEOX])
@pytest.mark.parametrize("B,L,Hq,Hkv,D,rd,Lmax,pos_hi", [
    (2, 37, 8, 2, 128, 128, 64, 20),
    (3, 5, 4, 4, 64, 64, 40, 30),
    (1, 130, 32, 8, 128, 64, 200, 60),     # rotary part shorter than the head: tail chunks are copied
    (2, 9, 6, 3, 96, 0, 16, 8),            # no rotary part: the producer only quantises
    (2, 12, 4, 2, 128, 128, 10, 6),        # some rows fall beyond Lmax and are dropped
])
def test_rope_kv_append_q8_writes_the_quantised_fp16_rows(dtype, style, B, L, Hq, Hkv, D, rd, Lmax, pos_hi):
    q, k, v, pos, kc, vc = workloads.kv_append(seed=L, device=DEV, B=B, L=L, Hq=Hq, Hkv=Hkv, D=D, Lmax=Lmax,
                                               dtype=dtype, pos_hi=pos_hi)
    q2 = q.clone()
    assert capi.rope_kv_append(style, q, k, v, pos, kc, vc, rd, 1e4) == capi.OK, capi.last_error()
    kq = torch.full((B, Hkv, Lmax, D // 32 * 34), 0x5A, dtype=torch.uint8, device=DEV)
    vq = torch.full_like(kq, 0x5A)
    assert capi.rope_kv_append_q8_0(style, q2, k, v, pos, kq, vq, rd, 1e4) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert torch.equal(q, q2)
    # rows the fp16/bf16 producer wrote, quantised by the oracle; every other row untouched
    want_k = oracle.quant_q8_0(kc.float().cpu())
    want_v = oracle.quant_q8_0(vc.float().cpu())
    written = np.zeros((B, Lmax), bool)
    for b in range(B):
        lo = int(pos[b])
        written[b, lo:min(lo + L, Lmax)] = True
    m = np.broadcast_to(written[:, None, :, None], want_k.shape)
    gk, gv = kq.cpu().numpy(), vq.cpu().numpy()
    assert np.array_equal(gk[m], want_k[m]) and np.array_equal(gv[m], want_v[m])
    assert (gk[~m] == 0x5A).all() and (gv[~m] == 0x5A).all()
    if rd == 0:   # nothing rotated: the bytes follow from the inputs alone
        for b in range(B):
            n = int(written[b].sum())
            lo = int(pos[b])
            assert np.array_equal(gv[b, :, lo:lo + n], oracle.quant_q8_0(v[b, :n].float().cpu().permute(1, 0, 2)))


def test_append_then_decode_over_q8_caches():
    B, L, Hq, Hkv, D, Lmax = 3, 300, 16, 4, 128, 320
    q, k, v, pos, _, _ = workloads.kv_append(seed=9, device=DEV, B=B, L=L, Hq=Hq, Hkv=Hkv, D=D, Lmax=Lmax, pos_hi=1)
    kq = torch.zeros(B, Hkv, Lmax, D // 32 * 34, dtype=torch.uint8, device=DEV)
    vq = torch.zeros_like(kq)
    q_in, k_in, v_in = q.cpu().clone(), k.cpu(), v.cpu()
    assert capi.rope_kv_append_q8_0(capi.ROPE_NEOX, q, k, v, pos, kq, vq, D, 5e5) == capi.OK, capi.last_error()
    ctx = torch.tensor([300, 17, 200], dtype=torch.int32)
    qd = torch.randn(B, Hq, 1, D, generator=torch.Generator().manual_seed(2)).half()
    out = run_decode_q8(qd.to(DEV), kq, vq, ctx.to(DEV))
    # oracle pipeline: exact rope -> fp16 rows -> oracle quantiser -> oracle decode
    zk = np.zeros((B, Hkv, Lmax, D), np.float32)
    _, ek, ev = oracle.rope_kv_append(oracle.ROPE_NEOX, q_in, k_in, v_in, pos.cpu(), zk, zk.copy(), D, 5e5)
    ekq = oracle.quant_q8_0(ek.astype(np.float16).astype(np.float32))
    evq = oracle.quant_q8_0(ev.astype(np.float16).astype(np.float32))
    want = oracle.flash_attn_decode_q8_0(qd, ekq, evq, ctx)
    assert float(np.abs(out.float().cpu().numpy() - want).max()) <= TOL


# ------------------------------------------------------------------------------------------------
# prefill over k, v given as Q8_0 blocks (the operator's (qtype_int, qblock_size, qtype_size) = (8, 32, 34))
# ------------------------------------------------------------------------------------------------
def _q8_rows(x):
    """[..., D] values -> uint8 [..., D/32*34] Q8_0 rows (the oracle's quantiser), and the fp16 values they dequantise to."""
    yq = torch.from_numpy(oracle.quant_q8_0(x.float()))
    back = torch.from_numpy(oracle.dequant_q8_0(yq.numpy(), np.float16)).view(x.shape)
    return yq, back


@pytest.mark.parametrize("B,Hq,Hkv,L,D,kind,cache_rows", [
    (2, 8, 2, 200, 128, "causal", 0),
    (1, 12, 2, 333, 64, "window", 0),        # n_rep = 6, L not a multiple of anything
    (2, 8, 4, 130, 128, "causal", 500),      # k, v are the first L rows of longer caches: strided batch and head dims
    (1, 32, 8, 1024, 128, "causal", 0),
])
def test_prefill_over_q8_0_kv(B, Hq, Hkv, L, D, kind, cache_rows):
    """Equal, bit for bit, to the fp16 operator on the dequantised rows (the same kernel reads the same fp16 values),
    and within the fp16 attention tolerance of the oracle on those rows."""
    q, k, v = workloads.dense_prefill(B, Hq, Hkv, L, D, torch.float16, seed=L + D, scale=1.0)
    rows_total = max(L, cache_rows)
    kq_all, k_back = _q8_rows(torch.cat([k, torch.zeros(B, Hkv, rows_total - L, D, dtype=torch.float16)], 2))
    vq_all, v_back = _q8_rows(torch.cat([v, torch.zeros(B, Hkv, rows_total - L, D, dtype=torch.float16)], 2))
    kq, vq = kq_all.to(DEV)[:, :, :L], vq_all.to(DEV)[:, :, :L]
    assert kq.is_contiguous() == (cache_rows == 0)
    mask = workloads.causal_mask(B, L) if kind == "causal" else workloads.window_mask(B, L, 50)
    out = torch.full(q.shape, float("nan"), dtype=torch.float16, device=DEV)
    assert capi.flash_attn_q8_0(q.to(DEV), kq, vq, mask.to(DEV), out) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    ref = torch.full_like(out, float("nan"))
    assert capi.flash_attn(q.to(DEV), k_back[:, :, :L].contiguous().to(DEV), v_back[:, :, :L].contiguous().to(DEV), mask.to(DEV), ref) == capi.OK
    torch.cuda.synchronize()
    assert torch.equal(out, ref)
    want = oracle.flash_attn(q, k_back[:, :, :L], v_back[:, :, :L], mask)
    assert float((out.float().cpu() - torch.from_numpy(want)).abs().max()) <= TOL


def test_varlen_prefill_over_q8_0_kv_and_torch_ops(kerns):
    from minfer.const import GGML_QUANT_SIZES, GGMLQuantizationType
    q8 = GGMLQuantizationType.Q8_0
    qb, qs = GGML_QUANT_SIZES[q8]
    qv, kv, vv, cu = workloads.ragged_prefill(seed=4, n_seqs=5, len_lo=1, len_hi=300, Hq=8, Hkv=2)
    kq, k_back = _q8_rows(kv)
    vq, v_back = _q8_rows(vv)
    out = torch.full(qv.shape, float("nan"), dtype=torch.float16, device=DEV)
    assert capi.flash_attn_varlen_q8_0(qv.to(DEV), kq.to(DEV), vq.to(DEV), cu.to(DEV), 300, out) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    want = oracle.flash_attn_varlen(qv, k_back, v_back, cu)
    assert float((out.float().cpu() - torch.from_numpy(want)).abs().max()) <= TOL
    # the registered ops take the same tensors with the Q8_0 type triple and give the same bits
    out2 = torch.zeros_like(out)
    assert kerns.flash_attn_varlen(q8, qb, qs, qv.to(DEV), kq.to(DEV), vq.to(DEV), cu.to(DEV), 300, out2) is None
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    B, Hq, Hkv, L, D = 2, 8, 2, 192, 128
    q, k, v = workloads.dense_prefill(B, Hq, Hkv, L, D, torch.float16, seed=8, scale=1.0, device=DEV)
    kq, _ = _q8_rows(k.cpu())
    vq, _ = _q8_rows(v.cpu())
    mask = workloads.causal_mask(B, L, device=DEV)
    a, b = torch.zeros_like(q), torch.zeros_like(q)
    assert kerns.flash_attn(q8, qb, qs, q, kq.to(DEV), vq.to(DEV), mask, a) is None
    assert capi.flash_attn_q8_0(q, kq.to(DEV), vq.to(DEV), mask, b) == capi.OK
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    with pytest.raises(RuntimeError):
        kerns.flash_attn(1, 1, 2, q, kq.to(DEV), vq.to(DEV), mask, a)            # byte k/v without the Q8_0 type
    with pytest.raises(RuntimeError):
        kerns.flash_attn(q8, qb, qs, q.bfloat16(), kq.to(DEV), vq.to(DEV), mask, a.bfloat16())   # q must be float16
    with pytest.raises(RuntimeError):
        kerns.flash_attn(q8, qb, qs, q, k, v, mask, a)                           # float k/v with the Q8_0 type
