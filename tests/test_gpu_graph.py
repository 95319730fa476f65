"""The attention operators under HIP graph capture (-m gpu): one graph that holds a prefill call and a decode call
through the registered ops (the reference's call path, torch_ext/ops.py:234-247) and a decode call through the C ABI
entry point that allocates nothing, replayed several times with eager work and synchronisations in between; every
replay must equal the eager result bit for bit.  None of the launches clears memory with a memset (such nodes have
replayed wrongly on this platform), which is what makes the operators capturable as they are.
"""
import pytest
import torch

import capi
import workloads
from minfer.const import GGML_QUANT_SIZES, GGMLQuantizationType

pytestmark = pytest.mark.gpu
DEV = "cuda"


def test_prefill_decode_and_noalloc_decode_in_one_graph(kerns):
    qt = GGMLQuantizationType.F16
    qb, qs = GGML_QUANT_SIZES[qt]
    B, Hq, Hkv, L, D = 2, 8, 2, 320, 128
    q, k, v = workloads.dense_prefill(B, Hq, Hkv, L, D, torch.float16, seed=41, views=True, device=DEV)
    mask = workloads.causal_mask(B, L, device=DEV)
    out_p = torch.zeros(B, Hq, L, D, dtype=torch.float16, device=DEV)
    qd, kc, vc, ctx = workloads.decode_cache(seed=42, device=DEV, B=5, Hq=8, Hkv=2, Lmax=1500, D=128, ctx_lo=1, ctx_hi=1500)
    out_d = torch.zeros_like(qd)
    out_n = torch.zeros_like(qd)

    def calls():
        kerns.flash_attn(qt, qb, qs, q, k, v, mask, out_p)
        kerns.flash_attn_decode(qt, qb, qs, qd, kc, vc, ctx, out_d)
        assert capi.flash_attn_decode_noalloc(qd, kc, vc, ctx, out_n) == capi.OK, capi.last_error()

    def eager():
        calls()
        torch.cuda.synchronize()
        return out_p.clone(), out_d.clone(), out_n.clone()

    # warm-up on a side stream, as torch asks before a capture (first-call set-up, allocator pools, the scratch address)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        calls()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        calls()

    gq = torch.Generator(device="cpu").manual_seed(43)
    for i in range(4):
        if i:   # new operand values in the same buffers, written by eager kernels between the replays
            q.copy_(torch.randn(q.shape, generator=gq).to(torch.float16).to(DEV))
            qd.copy_(torch.randn(qd.shape, generator=gq).to(torch.float16).to(DEV))
            ctx.copy_(torch.randint(1, 1501, ctx.shape, generator=gq, dtype=torch.int32).to(DEV))
        want_p, want_d, want_n = eager()
        assert torch.equal(want_d, want_n)
        for t in (out_p, out_d, out_n):
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_p, want_p), f"replay {i}: prefill differs from eager"
        assert torch.equal(out_d, want_d), f"replay {i}: decode differs from eager"
        assert torch.equal(out_n, want_n), f"replay {i}: allocation-free decode differs from eager"
