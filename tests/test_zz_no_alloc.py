"""The decode entry point that allocates nothing (minfer_flash_attn_decode_noalloc), through the C ABI, against
minfer_flash_attn_decode on the same inputs: two calls in a row, the second on a smaller problem, so that the
second call finds the first call's partial results in the library's scratch array.  Bit equality is the bar: both
entry points run the same kernels on the same split of the work."""
import pytest
import torch

import capi
import oracle
import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _both(q, kc, vc, ctx):
    want = torch.full(q.shape, float("nan"), dtype=q.dtype, device=DEV)
    assert capi.flash_attn_decode(q, kc, vc, ctx, want) == capi.OK, capi.last_error()
    got = torch.full(q.shape, float("nan"), dtype=q.dtype, device=DEV)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    assert capi.flash_attn_decode_noalloc(q, kc, vc, ctx, got) == capi.OK, capi.last_error()
    after = torch.cuda.memory_stats()["allocation.all.allocated"]
    torch.cuda.synchronize()
    assert after == before                      # nothing went through torch's allocator either
    return got, want


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_noalloc_decode_matches_workspace_decode_twice(dtype):
    # first call: 12 sequences of up to 3000 rows (several shares and partial results per row)
    q, kc, vc, ctx = workloads.decode_cache(seed=7, device=DEV, B=12, Hq=32, Hkv=8, Lmax=3000, D=128, dtype=dtype,
                                            ctx_lo=0, ctx_hi=3000)
    got, want = _both(q, kc, vc, ctx)
    assert torch.equal(got, want)
    assert float((got.float().cpu() - torch.from_numpy(oracle.flash_attn_decode(q, kc, vc, ctx))).abs().max()) <= \
        (2e-3 if dtype == torch.float16 else 1e-2)
    # second call, smaller in every dimension: fewer slots per row, other head count, other head_dim
    q2, kc2, vc2, ctx2 = workloads.decode_cache(seed=8, device=DEV, B=3, Hq=8, Hkv=2, Lmax=700, D=64, dtype=dtype,
                                                ctx_lo=1, ctx_hi=700)
    got2, want2 = _both(q2, kc2, vc2, ctx2)
    assert torch.equal(got2, want2)
    assert float((got2.float().cpu() - torch.from_numpy(oracle.flash_attn_decode(q2, kc2, vc2, ctx2))).abs().max()) <= \
        (2e-3 if dtype == torch.float16 else 1e-2)
    # and the first problem again gives the first result again
    got3, _ = _both(q, kc, vc, ctx)
    assert torch.equal(got3, want)


def test_noalloc_decode_full_size_and_limit():
    # the benchmark's decode workload fits the scratch array
    q, kc, vc, ctx = workloads.decode_cache(seed=0, device=DEV)
    assert capi.lib().minfer_flash_attn_decode_workspace_bytes(64, 32, 8192, 128) <= capi.DECODE_NOALLOC_SCRATCH_BYTES
    got, want = _both(q, kc, vc, ctx)
    assert torch.equal(got, want)
    del kc, vc
    # a problem beyond it is refused on the host, nothing launched, out untouched
    B, Hq, Lmax = 256, 64, 8192
    assert capi.lib().minfer_flash_attn_decode_workspace_bytes(B, Hq, Lmax, 128) > capi.DECODE_NOALLOC_SCRATCH_BYTES
    qb = torch.zeros(B, Hq, 1, 128, dtype=torch.float16, device=DEV)
    cache = torch.zeros(B, 8, 16, 128, dtype=torch.float16, device=DEV).as_strided((B, 8, Lmax, 128), (8 * 16 * 128, 16 * 128, 0, 1))
    out = torch.full_like(qb, 3.0)
    ctx_b = torch.ones(B, dtype=torch.int32, device=DEV)
    assert capi.flash_attn_decode_noalloc(qb, cache, cache, ctx_b, out) == capi.EWORKSPACE
    assert "scratch" in capi.last_error()
    torch.cuda.synchronize()
    assert torch.all(out == 3.0)
