"""GPU parity on the reference's own caller recipes (-m gpu): the flash_attn test of the reference
(reference: test/kernels.py:222-298: B=8, L=4096, 48 query heads over 8 KV heads, D=128, transposed views, case A
causal, case B a symmetric window of 256), its benchmark's largest case (reference: apps/benchmark.py:210-237,
L=16384), the stride-0 mask its profiling script builds (reference: apps/profile.py:105), and
torch.library.opcheck on the registered ops, which the reference runs for gemm (reference: test/kernels.py:150-170).

The reference's own tolerance is atol 3e-1 against torch SDPA; here the bar is 2e-3 against the CPU oracle on
sampled query rows and against an fp32 torch evaluation of the whole output.
"""
import pytest
import torch

import capi
import oracle
import workloads
from minfer.const import GGML_QUANT_SIZES, GGMLQuantizationType
from test_gpu_parity import max_err, sample_rows, torch_ref

pytestmark = pytest.mark.gpu
DEV = "cuda"
QT = GGMLQuantizationType.F16
QB, QS = GGML_QUANT_SIZES[QT]


@pytest.mark.parametrize("window", [None, 256], ids=["caseA_causal", "caseB_window256"])
def test_reference_test_recipe(kerns, window):
    B, L, Hq, Hkv, D = 8, 4096, 48, 8, 128
    q, k, v, mask = workloads.reference_test_prefill(seed=11 if window is None else 12, device=DEV, window=window)
    assert q.shape == (B, Hq, L, D) and q.stride() == (L * Hq * D, D, Hq * D, 1) and not q.is_contiguous()
    out = torch.zeros(B, Hq, L, D, dtype=torch.float16, device=DEV)
    kerns.flash_attn(QT, QB, QS, q, k, v, mask, out)           # the call of test/kernels.py:246-248
    torch.cuda.synchronize()
    assert max_err(out, torch_ref(q, k, v, mask, row_chunk=512)) <= 2e-3
    rows = sample_rows(L, 12, torch.Generator().manual_seed(3)) + [255, 256, 257, 511, 512]
    rows = sorted(set(rows))
    want = oracle.flash_attn_rows(q, k, v, mask[:, 0, rows].cpu(), rows)
    assert max_err(out[:, :, rows], want) <= 2e-3
    # the C ABI called directly gives the same bits as the registered op
    out2 = torch.full_like(out, float("nan"))
    assert capi.flash_attn(q, k, v, mask, out2) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


def test_reference_benchmark_recipe_longest(kerns):
    B, L, Hq, Hkv, D = 4, 16384, 48, 8, 128
    q, k, v, mask = workloads.reference_benchmark_prefill(seed=13, device=DEV, B=B, L=L)
    out = torch.zeros(B, Hq, L, D, dtype=torch.float16, device=DEV)
    kerns.flash_attn(QT, QB, QS, q, k, v, mask, out)           # the call of apps/benchmark.py:245
    torch.cuda.synchronize()
    rows = sample_rows(L, 6, torch.Generator().manual_seed(4))
    want = oracle.flash_attn_rows(q, k, v, mask[:, 0, rows].cpu(), rows)
    assert max_err(out[:, :, rows], want) <= 2e-3
    for b in range(B):   # the whole output against fp32 torch, one batch entry at a time
        assert max_err(out[b:b + 1], torch_ref(q[b:b + 1], k[b:b + 1], v[b:b + 1], mask[b:b + 1], row_chunk=1024)) <= 2e-3


def test_profile_script_mask_is_rejected(kerns):
    """apps/profile.py:105 builds its mask with expand(B, 1, L, L).to(torch.bool): a stride-0 view, which the
    reference host function rejects (op.cuh:50: the mask must be contiguous).  Same error here, nothing launched."""
    B, L = 4, 256
    q, k, v, _ = workloads.reference_test_prefill(seed=1, device=DEV, B=B, L=L)
    i = torch.arange(L, device=DEV)
    mask = (i.unsqueeze(0) <= i.unsqueeze(1)).unsqueeze(0).unsqueeze(0).expand(B, 1, L, L).to(torch.bool)
    assert mask.stride(0) == 0 and not mask.is_contiguous()
    out = torch.zeros(B, 48, L, 128, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="contiguous"):
        kerns.flash_attn(QT, QB, QS, q, k, v, mask, out)
    assert torch.all(out == 0)
    kerns.flash_attn(QT, QB, QS, q, k, v, mask.contiguous(), out)
    torch.cuda.synchronize()
    assert max_err(out, torch_ref(q, k, v, mask.contiguous())) <= 2e-3


# ------------------------------------------------------------------------------------------------
# torch.library.opcheck: schema (what is mutated, what aliases), fake kernels, dispatch under tracing
# ------------------------------------------------------------------------------------------------
OPCHECKS = ("test_schema", "test_faketensor", "test_aot_dispatch_dynamic")   # no autograd formula is registered, as in the reference


def _opcheck(op, args):
    import minfer.kernels.torch_ext  # noqa: F401  (registers the ops and their fakes)
    torch.library.opcheck(op, args, test_utils=OPCHECKS)


def test_opcheck_flash_attn():
    q, k, v = workloads.dense_prefill(2, 8, 2, 192, 128, torch.float16, seed=2, views=True, device=DEV)
    mask = workloads.causal_mask(2, 192, device=DEV)
    _opcheck(torch.ops.minfer.flash_attn.default, (QT, QB, QS, q, k, v, mask, torch.zeros_like(q)))


def test_opcheck_flash_attn_decode_and_varlen():
    qd, kc, vc, ctx = workloads.decode_cache(seed=2, device=DEV, B=3, Hq=8, Hkv=2, Lmax=300, ctx_lo=1, ctx_hi=300)
    _opcheck(torch.ops.minfer.flash_attn_decode.default, (QT, QB, QS, qd, kc, vc, ctx, torch.zeros_like(qd)))
    qv, kv, vv, cu = workloads.ragged_prefill(seed=2, device=DEV, n_seqs=3, len_lo=5, len_hi=90, Hq=8, Hkv=2)
    _opcheck(torch.ops.minfer.flash_attn_varlen.default, (QT, QB, QS, qv, kv, vv, cu, 90, torch.zeros_like(qv)))


@pytest.mark.parametrize("size", [64, 256])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (2.0, 3.0)])
def test_opcheck_gemm(size, alpha, beta):
    """The reference's own opcheck (test/kernels.py:150-170) on two of its sizes and scale pairs."""
    a, w, bias = workloads.gemm_input(size, size, size, seed=size, device=DEV)
    _opcheck(torch.ops.minfer.gemm.default, (QT, QB, QS, alpha, beta, a, w, bias, torch.zeros_like(bias)))


def test_opcheck_rmsnorm_and_rope():
    x, w = workloads.rmsnorm_input((2, 16, 256), seed=5, device=DEV)
    _opcheck(torch.ops.minfer.rmsnorm.default, (1e-6, x, w, torch.empty_like(x)))
    r = workloads.rope_input(seed=5, device=DEV, B=2, L=8, H=4, D=128)
    _opcheck(torch.ops.minfer.il_rope.default, (64, 3, 1e6, r))
    _opcheck(torch.ops.minfer.neox_rope.default, (64, 3, 1e6, r))


def test_opcheck_producers_and_quantised_operands():
    """The ops beyond the reference's set: the cache producers, the Q8_0 operands of gemm / qkv / the attention ops."""
    q8 = GGMLQuantizationType.Q8_0
    q8b, q8s = GGML_QUANT_SIZES[q8]
    q, k, v, pos, kc, vc = workloads.kv_append(seed=3, device=DEV, B=2, L=5, Hq=8, Hkv=2, D=128, Lmax=16)
    _opcheck(torch.ops.minfer.rope_kv_append.default, (1, 128, 5e5, q.clone(), k, v, pos, kc.clone(), vc.clone()))
    w = torch.ones(128, dtype=q.dtype, device=DEV)
    _opcheck(torch.ops.minfer.rope_kv_append_norm.default, (1, 128, 5e5, 1e-6, q.clone(), k, v, w, w, pos, kc.clone(), vc.clone()))
    kq = torch.zeros(2, 2, 16, 136, dtype=torch.uint8, device=DEV)
    _opcheck(torch.ops.minfer.rope_kv_append.default, (1, 128, 5e5, q.clone(), k, v, pos, kq, kq.clone()))
    # a weight of Q8_0 blocks
    a, wf, bias = workloads.gemm_input(8, 256, 512, seed=4, device=DEV)
    wq = torch.empty(256, 512 // 32 * 34, dtype=torch.uint8, device=DEV)
    torch.ops.minfer.quant.default(q8, q8b, q8s, wf.t().contiguous(), wq)
    _opcheck(torch.ops.minfer.gemm.default, (q8, q8b, q8s, 1.0, 1.0, a, wq, bias, torch.zeros_like(bias)))
    outs = [torch.zeros(1, 8, 256, dtype=torch.float16, device=DEV) for _ in range(3)]
    _opcheck(torch.ops.minfer.qkv.default, (q8, q8, q8, q8b, q8b, q8b, q8s, q8s, q8s, a, wq, wq, wq, *outs))
    # decode over Q8_0 caches
    qd, kcf, vcf, ctx = workloads.decode_cache(seed=2, device=DEV, B=2, Hq=8, Hkv=2, Lmax=64, ctx_lo=1, ctx_hi=64)
    kc8 = torch.empty(2, 2, 64, 136, dtype=torch.uint8, device=DEV)
    vc8 = torch.empty_like(kc8)
    torch.ops.minfer.quant.default(q8, q8b, q8s, kcf.reshape(-1, 128), kc8.view(-1, 136))
    torch.ops.minfer.quant.default(q8, q8b, q8s, vcf.reshape(-1, 128), vc8.view(-1, 136))
    _opcheck(torch.ops.minfer.flash_attn_decode.default, (q8, q8b, q8s, qd, kc8, vc8, ctx, torch.zeros_like(qd)))
