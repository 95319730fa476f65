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
    # the first call on a device looks up the scratch array's address (and may load the code object): a call
    # before the measured one takes that out of the picture
    warm = torch.empty_like(got)
    assert capi.flash_attn_decode_noalloc(q, kc, vc, ctx, warm) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    # the device's own count of free memory (hipMemGetInfo): the library does not go through torch's allocator,
    # so torch's statistics would not see a hipMalloc inside the call
    free_before, _ = torch.cuda.mem_get_info()
    stats_before = torch.cuda.memory_stats()["allocation.all.allocated"]
    assert capi.flash_attn_decode_noalloc(q, kc, vc, ctx, got) == capi.OK, capi.last_error()
    free_during, _ = torch.cuda.mem_get_info()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_during == free_before and free_after == free_before
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == stats_before
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


def test_noalloc_decode_under_graph_capture():
    """The use the entry point is for: captured into a HIP graph (where hipMalloc is not allowed) after a first call
    outside the capture, replayed several times with eager work in between, every replay bit-equal to the workspace
    entry point.  The two kernels clear nothing with a memset, so the graph holds kernel nodes only."""
    q, kc, vc, ctx = workloads.decode_cache(seed=11, device=DEV, B=6, Hq=16, Hkv=4, Lmax=2048, D=128, ctx_lo=1, ctx_hi=2048)
    want = torch.empty_like(q)
    assert capi.flash_attn_decode(q, kc, vc, ctx, want) == capi.OK, capi.last_error()
    got = torch.full(q.shape, float("nan"), dtype=q.dtype, device=DEV)
    assert capi.flash_attn_decode_noalloc(q, kc, vc, ctx, got) == capi.OK, capi.last_error()   # address looked up here
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):               # capi passes torch's current stream: the capture stream
        assert capi.flash_attn_decode_noalloc(q, kc, vc, ctx, got) == capi.OK, capi.last_error()
    for i in range(4):
        got.fill_(float("nan"))
        q2 = (q.float() * (1.0 + i)).to(q.dtype)    # eager work between replays, and other inputs for this replay
        q.copy_(q2)
        assert capi.flash_attn_decode(q, kc, vc, ctx, want) == capi.OK, capi.last_error()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {i} differs from the eager result"
