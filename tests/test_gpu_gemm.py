"""GPU parity tests (-m gpu) of the GEMM kernels and of the gemm / qkv operators, through the C ABI and the
registered torch ops, against the fp64 CPU oracle on identical seeded inputs.

Tolerance: the reference's tests allow atol 6e-1 (gemm) and 2e-1 (qkv) (reference: test/kernels.py:145,
212-214).  Here every element must lie within 0.51 units in the last place of the output format of the
oracle's exact value, plus 2^-17 of the largest magnitude of the result for the fp32 accumulation (which
shows only where a sum of a few hundred terms cancels to something far smaller than its terms)."""
import os

import numpy as np
import pytest
import torch

import capi
import oracle
import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda"
MANT = {torch.float16: 10, torch.bfloat16: 7}
MIN_EXP = {torch.float16: -14, torch.bfloat16: -126}
KN, NK = capi.GEMM_B_KN, capi.GEMM_B_NK


def assert_close(got, exact, dtype, what=""):
    got = got.float().cpu().numpy().astype(np.float64)
    exact = exact.astype(np.float64)
    e = np.floor(np.log2(np.maximum(np.abs(exact), 2.0 ** MIN_EXP[dtype])))
    bound = 0.51 * 2.0 ** (e - MANT[dtype]) + 2.0 ** -17 * float(np.abs(exact).max())
    err = np.abs(got - exact)
    worst = np.unravel_index(np.argmax(err - bound), err.shape)
    assert not (err > bound).any(), (f"{what}: {(err > bound).sum()} elements out of bound; at {worst} got {got[worst]!r}, "
                                     f"exact {float(exact[worst])!r}")


def make(M, N, K, layout, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(M, K, generator=g).to(dtype)
    b = ((1 / K ** 0.5) * torch.randn((K, N) if layout == KN else (N, K), generator=g)).to(dtype)
    c = torch.randn(M, N, generator=g).to(dtype)
    return a, b, c


@pytest.mark.parametrize("layout", [KN, NK])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K,alpha,beta", [
    (256, 256, 64, 1.0, 0.0),        # four tiles of the 128 x 128 kernel, one K step
    (512, 384, 256, 2.0, 3.0),
    (300, 264, 192, 0.5, 2.0),       # ragged rows and columns (N a multiple of 8 only)
    (100, 72, 64, 1.0, 1.0),
    (1, 128, 128, 1.0, 0.0),         # a single row (decode-time projection)
    (4096, 4096, 128, 1.0, 1.0),     # enough tiles for the 256 x 256 kernel
    (3000, 4104, 64, 2.0, 0.0),      # the same with ragged edges
    (33, 17, 50, 1.0, 1.0),          # nothing tileable: plain kernel
    (64, 64, 72, 1.0, 0.0),          # K not a multiple of 64: plain kernel
    (8, 4096, 4096, 1.0, 0.0),       # a decode step's tokens: with an [N, K] weight, the kernel that streams it once
    (64, 1024, 1792, 2.0, 3.0),      # its largest row count; K steps not a multiple of the eight waves
    (48, 8192, 8192, 1.0, 0.0),      # more than 32 rows against a large weight: the tiled kernel again
    (2048, 6144, 128, 1.0, 1.0),     # [N, K]: 256 x 192 tiles (one full round instead of three quarters of one)
    (1800, 6144, 64, 2.0, 3.0),      # the same with a ragged last tile row
    (30, 5200, 128, 2.0, 1.0),       # wide enough for two column groups per workgroup, the last one ragged
    (37, 24, 192, 0.5, 1.0),         # ragged rows, a last group of 16 columns that is half empty
    (17, 4104, 64, 1.0, 1.0),        # one K step: seven of the eight waves have nothing to add
    (64, 6144, 4096, 2.0, 3.0),      # 64 rows, two column groups per workgroup: the few-row kernel's largest instantiation
    (40, 5128, 1024, 1.0, 1.0),      # 40 rows (three row blocks), two column groups, the last one ragged
    # up to 16 rows against an [N, K] weight with K a multiple of 512: weight and activation rows copied to LDS along the rows
    (2, 4096, 4096, 1.0, 0.0),
    (5, 264, 512, 1.0, 1.0),         # one segment per wave; rows 5..7 of the second activation copy do not exist
    (12, 1000, 1536, 2.0, 3.0),      # three activation copies, a last group of 8 columns
    (16, 4104, 1024, 1.0, 1.0),
    (3, 8, 512, 1.0, 0.0),           # a single half-empty group
    (9, 2048, 14336, 0.5, 0.0),      # 28 segments per wave
    # 1-64 rows against a weight of 12288 columns or more, K a multiple of 256: 64-column stripes over the whole of K
    (2, 12288, 256, 1.0, 0.0),       # one segment
    (1, 12296, 1024, 2.0, 3.0),      # one row
    (1, 6144, 4096, 1.0, 0.0),       # 96 stripes: the narrowest weight it takes at any row count
    (8, 5120, 768, 2.0, 3.0),        # 80 stripes from 8 rows on
    (40, 4104, 1024, 1.0, 1.0),      # 65 stripes from 32 rows on, the last one of 8 columns
    (9, 12296, 512, 2.0, 3.0),       # a last stripe of 8 columns; two segments (fewer than the three stages)
    (16, 14336, 1024, 1.0, 1.0),
    (17, 12288, 768, 1.0, 0.0),      # two blocks of activation rows, the second with one row
    (32, 12352, 1280, 0.5, 1.0),
    (33, 12288, 512, 1.0, 1.0),      # four blocks of activation rows, two stages
    (64, 14336, 1792, 2.0, 0.0),
    # one row against an [N, K] weight: whole weight rows per wave (segments of 4096 values)
    (1, 4096, 4096, 1.0, 0.0),       # one segment, the activations in registers; two rows per wave
    (1, 1000, 4160, 2.0, 3.0),       # a second segment of 64 values, the activations in LDS
    (1, 1000, 8192, 2.0, 3.0),       # longer than a segment and a multiple of 512: the LDS-staged few-row kernel instead
    (1, 20000, 64, 2.0, 3.0),        # ten short rows per wave
    (1, 264, 16384, 1.0, 1.0),       # the longest activation row its LDS area holds
    (1, 264, 16448, 1.0, 0.0),       # longer: the 16-rows-per-instruction kernel
    (1, 8, 192, 1.0, 1.0),           # two waves with rows, the others none
    # two to four rows against long rows of a wide weight: whole weight rows per wave, every piece times the same piece of each activation row
    (2, 10240, 8192, 1.0, 0.0),
    (3, 10248, 8192, 2.0, 3.0),      # a last wave with fewer rows
    (4, 16384, 8192, 1.0, 1.0),
])
def test_gemm_matches_oracle(layout, dtype, M, N, K, alpha, beta):
    a, b, c = make(M, N, K, layout, dtype, M + N + K)
    if M * N * K <= 1 << 26 or M <= 64:
        exact = oracle.gemm(a, b, c, alpha, beta, layout)
        rows = slice(None)
    else:       # the oracle is a scalar CPU program: a sample of rows at this size
        rows = torch.tensor(sorted({0, 1, 255, 256, 257, M // 2, M - 257, M - 2, M - 1} | set(range(1000, 1064))))
        exact = oracle.gemm(a[rows], b, c[rows], alpha, beta, layout)
    d = torch.full((M, N), float("nan"), dtype=dtype, device=DEV)
    assert capi.gemm(a.to(DEV), b.to(DEV), c.to(DEV), d, alpha, beta, layout) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert_close(d[rows], exact, dtype, "gemm")
    if not isinstance(rows, slice):   # the whole result against an fp32 torch evaluation of the same expression
        ref = alpha * (a.to(DEV).float() @ (b.to(DEV).float() if layout == KN else b.to(DEV).float().T)) + beta * c.to(DEV).float()
        assert float((d.float() - ref).abs().max()) <= 2.0 ** -MANT[dtype] * float(ref.abs().max())


def test_gemm_golden_strided_and_in_place():
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "gemm_small.npz"))
    a, b, c = (torch.from_numpy(z[k]).to(DEV) for k in "abc")
    alpha, beta = float(z["alpha"]), float(z["beta"])
    d = torch.empty_like(c)
    assert capi.gemm(a, b, c, d, alpha, beta) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert_close(d, z["d"], torch.float16, "golden")
    # C aliasing D
    d2 = c.clone()
    assert capi.gemm(a, b, d2, d2, alpha, beta) == capi.OK
    torch.cuda.synchronize()
    assert torch.equal(d2, d)
    # row strides larger than the rows (views of wider buffers), beta = 0 with no C
    big_a = torch.randn(70, 200, device=DEV).half()
    big_d = torch.full((70, 96), float("nan"), dtype=torch.float16, device=DEV)
    av, dv = big_a[:, 8:136], big_d[:, 16:88]
    assert capi.gemm(av, b, None, dv, 1.0, 0.0) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    assert_close(dv, oracle.gemm(av.cpu().contiguous(), b.cpu(), None, 1.0, 0.0), torch.float16, "strided")
    assert torch.isnan(big_d[:, :16]).all() and torch.isnan(big_d[:, 88:]).all()


@pytest.mark.parametrize("S", [1024, 2048])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (2.0, 3.0)])
def test_gemm_op_reference_test_recipe(kerns, S, alpha, beta):
    """The reference's test recipe (test/kernels.py:119-147): A [1,S,S] ~ N(0,1), weight [S,S] ~ N(0,1)/sqrt(S), bias
    ~ N(0,1), through the op with the reference's signature; sampled rows against the oracle, everything against
    the reference's own expression at its own tolerance."""
    a, w, bias = workloads.gemm_input(S, S, S, seed=S, device=DEV)
    out = torch.zeros_like(bias)
    assert kerns.gemm(1, 1, 2, alpha, beta, a, w, bias, out) is None
    torch.cuda.synchronize()
    rows = torch.arange(0, S, S // 16)
    assert_close(out[0, rows], oracle.gemm(a[0, rows].cpu(), w.cpu(), bias[0, rows].cpu(), alpha, beta), torch.float16, "op")
    assert torch.allclose((alpha * (a @ w) + beta * bias).float(), out.float(), atol=6e-1)
    d = torch.empty(S, S, dtype=torch.float16, device=DEV)
    ws = torch.empty(max(capi.lib().minfer_gemm_workspace_bytes(S, S, S), 16), dtype=torch.uint8, device=DEV)   # the op brings one too
    assert capi.gemm_ws(a[0], w, bias[0], d, alpha, beta, ws) == capi.OK
    torch.cuda.synchronize()
    assert torch.equal(d, out[0])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,K,Nq,Nk,Nv", [
    (4096, 4096, 4096, 1024, 1024),    # Llama-3-8B prefill: 256 x 192 tiles over the weights' columns numbered through (two full rounds)
    (2000, 128, 4096, 1024, 1024),     # the same tiling with a ragged last tile row; tiles that hold columns of q and k, of k and v
    (4096, 128, 4096, 2048, 2048),     # 8192 columns: no multiple of 192, 256 x 256 tiles per weight
    (512, 6144, 6144, 1024, 1024),     # the reference test's head shape at a smaller batch: 128 x 128 tiles
    (300, 256, 200, 72, 136),          # ragged rows, widths that end inside a tile
    (1, 4096, 4096, 1024, 1024),       # a decode step: whole weight rows per wave, the three weights' rows numbered through
    (1, 8192, 1032, 8, 520),           # the same with the activations in LDS and runs of rows that cross from one weight to the next
    (2, 4096, 4096, 1024, 1024),       # up to 16 rows, K a multiple of 512: the LDS-staged few-row kernel over the three weights' column groups
    (13, 1024, 520, 264, 8),           # the same with ragged last groups
    (16, 576, 4096, 1024, 1024),       # K not a multiple of 512: the few-row kernel that loads fragments directly
    (24, 1024, 5120, 1280, 1288),      # few rows, two column groups per workgroup, a ragged last group
    (64, 512, 768, 256, 256),          # few-row kernel at its largest row count
    (33, 50, 17, 17, 9),               # nothing tileable: three plain launches
    # 5-64 rows, K a multiple of 256, 96 stripes of 64 columns or more over the three weights: the stripe kernel, every weight
    # with workgroups of its own in proportion to its width
    (5, 4096, 4096, 1024, 1024),
    (16, 512, 4096, 1024, 1032),       # a last stripe of 8 columns in the third weight
    (40, 1024, 4104, 1024, 1024),      # ... in the first; three blocks of activation rows
    (64, 256, 5120, 520, 8),           # one segment; a weight of a single partial stripe
])
def test_qkv_one_launch_equals_three_gemms(dtype, M, K, Nq, Nk, Nv):
    """minfer_qkv (one grid over the column tiles of the three weights) against minfer_gemm per weight: from 65 rows on
    the same tiles run the same arithmetic and the results are equal bit for bit; up to 64 rows which few-row kernel runs
    depends on the width, which is the three weights' together in one case and one weight's in the other, and the
    results are equal up to the order of the fp32 sums (every output against the oracle there); k always against the
    oracle."""
    g = torch.Generator().manual_seed(M + K + Nq)
    x = torch.randn(M, K, generator=g).to(dtype).to(DEV)
    ws = [((1 / K ** 0.5) * torch.randn(n, K, generator=g)).to(dtype).to(DEV) for n in (Nq, Nk, Nv)]
    outs = [torch.full((M, n), float("nan"), dtype=dtype, device=DEV) for n in (Nq, Nk, Nv)]
    assert capi.qkv(x, *ws, *outs) == capi.OK, capi.last_error()
    torch.cuda.synchronize()
    for w, o, name in zip(ws, outs, "qkv"):
        ref = torch.full_like(o, float("nan"))
        assert capi.gemm(x, w, None, ref, 1.0, 0.0, NK) == capi.OK, capi.last_error()
        torch.cuda.synchronize()
        if M > 64:
            assert torch.equal(o, ref), name
        else:
            assert_close(o, oracle.gemm(x.cpu(), w.cpu(), None, 1.0, 0.0, NK), dtype, name + " against the oracle")
            assert float((o.float() - ref.float()).abs().max()) <= 2.0 ** -MANT[dtype] * float(ref.float().abs().max()), name
    rows = torch.arange(0, M, max(1, M // 24))
    assert_close(outs[1][rows], oracle.gemm(x[rows].cpu(), ws[1].cpu(), None, 1.0, 0.0, NK), dtype, "k against the oracle")


def test_qkv_op_and_reference_checks(kerns):
    """The QKV recipe of the reference's test at a smaller batch (test/kernels.py:173-214: hidden 6144, 48 query and
    8 KV heads of 128): x @ W^T for the three weights stored [out, hidden]."""
    B, L, hidden, q_dim, kv_dim = 2, 512, 6144, 48 * 128, 8 * 128
    g = torch.Generator().manual_seed(3)
    x = torch.randn(B, L, hidden, generator=g).half().to(DEV)
    wq, wk, wv = (((1 / hidden ** 0.5) * torch.randn(n, hidden, generator=g)).half().to(DEV) for n in (q_dim, kv_dim, kv_dim))
    q, k, v = (torch.zeros(B, L, n, dtype=torch.float16, device=DEV) for n in (q_dim, kv_dim, kv_dim))
    assert kerns.qkv(1, 1, 1, 1, 1, 1, 2, 2, 2, x, wq, wk, wv, q, k, v) is None
    torch.cuda.synchronize()
    rows = torch.arange(0, B * L, 64)
    xs = x.view(B * L, hidden)[rows].cpu()
    for out, w, name in ((q, wq, "q"), (k, wk, "k"), (v, wv, "v")):
        assert_close(out.view(B * L, -1)[rows], oracle.gemm(xs, w.cpu(), None, 1.0, 0.0, oracle.GEMM_B_NK), torch.float16, name)
        assert torch.allclose((x @ w.T).float(), out.float(), atol=2e-1)
    # weights stored [hidden, out] are recognised by their shape
    k2 = torch.zeros_like(k)
    kerns.qkv(1, 1, 1, 1, 1, 1, 2, 2, 2, x, wq, wk.T.contiguous(), wv, q, k2, v)
    torch.cuda.synchronize()
    assert float((k2.float() - k.float()).abs().max()) <= 4e-3
    with pytest.raises(RuntimeError):
        kerns.qkv(1, 1, 1, 1, 1, 1, 2, 2, 2, x, wq, wk[:, :100].contiguous(), wv, q, k, v)
    with pytest.raises(RuntimeError):
        kerns.qkv(2, 2, 2, 32, 32, 32, 18, 18, 18, x, wq, wk, wv, q, k, v)          # quantised weights: not implemented
    # gemm's reference checks (gemm/op.cuh:229-273)
    a, w, bias = workloads.gemm_input(64, 64, 64, seed=1, device=DEV)
    out = torch.zeros_like(bias)
    with pytest.raises(RuntimeError):
        kerns.gemm(1, 1, 2, 0.0, 1.0, a, w, bias, out)                              # alpha == 0
    with pytest.raises(RuntimeError):
        kerns.gemm(1, 1, 2, 1.0, 0.0, a[0], w, bias, out)                           # A must be 3-D
    with pytest.raises(RuntimeError):
        kerns.gemm(1, 1, 2, 1.0, 0.0, a, w[:, :32], bias, out)                      # not contiguous / wrong shape
    with pytest.raises(RuntimeError):
        kerns.gemm(1, 1, 2, 1.0, 0.0, a, w.float(), bias, out)
    with pytest.raises((RuntimeError, NotImplementedError)):
        kerns.gemm(1, 1, 2, 1.0, 0.0, a.cpu(), w.cpu(), bias.cpu(), out.cpu())


# ---- K slices through a workspace (minfer_gemm_ws) -------------------------------------------------------------
@pytest.mark.parametrize("layout", [KN, NK])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K,alpha,beta", [
    (64, 4096, 4096, 1.0, 0.0),      # 32 tiles, 8 slices of 8 steps
    (100, 1032, 2048, 2.0, 3.0),     # ragged rows and columns, C read by the second kernel
    (256, 2048, 1024, 0.5, 1.0),     # two tile rows
    (40, 512, 1984, 1.0, 0.0),       # K steps (31) not a multiple of the slice count
    (1, 4096, 4096, 1.0, 1.0),       # one row: with [K, N] the sliced tiles, with [N, K] still the few-row kernel
    (24, 1024, 2048, 1.0, 1.0),      # 17-32 rows: with a workspace the sliced tiles for both layouts
    (256, 8192, 1024, 1.0, 1.0),     # 128 tiles: two slices, so that two workgroups share a compute unit
    # [N, K] weights of fewer than 192 stripes of 64 columns: K slices of the stripe kernel
    (8, 5120, 5120, 2.0, 3.0),       # 80 stripes, three slices of 6, 7 and 7 segments
    (16, 4104, 8192, 1.0, 1.0),      # a last stripe of 8 columns
    (33, 8192, 2048, 0.5, 0.0),      # three blocks of activation rows, two slices of four segments
    (1, 8192, 4096, 1.0, 0.0),       # one row
    (64, 6144, 4096, 1.0, 1.0),
    (12, 1024, 14336, 1.0, 0.0),     # long rows of a small weight: 16 stripes, 14 slices of 4 segments
    (24, 2048, 4096, 2.0, 1.0),      # 8 M weight values from 17 rows on: 8 slices of 2 segments, two blocks of rows
    (3, 1536, 8960, 1.0, 1.0),       # long rows, 24 stripes: slices from 2 rows on (10 slices of 3 or 4 segments)
])
def test_gemm_k_slices_against_oracle(layout, dtype, M, N, K, alpha, beta):
    a, b, c = make(M, N, K, layout, dtype, seed=M + N + K)
    need = capi.lib().minfer_gemm_workspace_bytes(M, N, K)
    assert need > 0 and need % (4 * M * N) == 0, need
    exact = oracle.gemm(a.float().numpy(), b.float().numpy(), c.float().numpy(), alpha, beta, layout)
    da, db, dc = a.to(DEV), b.to(DEV), c.to(DEV)
    d = torch.zeros(M, N, dtype=dtype, device=DEV)
    ws = torch.full((need,), 0xFF, dtype=torch.uint8, device=DEV)      # NaN patterns: every slot read must have been written
    assert capi.gemm_ws(da, db, dc, d, alpha, beta, ws, layout) == capi.OK, capi.last_error()
    assert_close(d, exact, dtype, "k slices")
    # a workspace that is too small, or none, is the plain call
    d2 = torch.zeros_like(d)
    assert capi.gemm_ws(da, db, dc, d2, alpha, beta, ws[: 4 * M * N], layout) == capi.OK, capi.last_error()   # room for one slice: no path takes it
    d3 = torch.zeros_like(d)
    assert capi.gemm(da, db, dc, d3, alpha, beta, layout) == capi.OK, capi.last_error()
    assert torch.equal(d2, d3)
    assert_close(d2, exact, dtype, "fallback")


def test_gemm_workspace_bytes_is_zero_where_tiles_fill_the_chip():
    L = capi.lib()
    assert L.minfer_gemm_workspace_bytes(4096, 4096, 4096) == 0
    assert L.minfer_gemm_workspace_bytes(64, 4096, 100) == 0       # K not a multiple of 64
    assert L.minfer_gemm_workspace_bytes(64, 4096, 256) == 0       # too few K steps to slice
    assert L.minfer_gemm_workspace_bytes(0, 4096, 4096) == 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_gemm_op_uses_k_slices_and_matches_oracle(dtype):
    from minfer.kernels import KernelBackend
    from minfer.const import GGMLQuantizationType, GGML_QUANT_SIZES
    kerns = KernelBackend("torch_ext")
    qt = GGMLQuantizationType.F16 if dtype == torch.float16 else GGMLQuantizationType.BF16
    qb, qs = GGML_QUANT_SIZES[qt]
    M, N, K = 96, 2048, 4096
    a, b, c = make(M, N, K, KN, dtype, seed=5)
    exact = oracle.gemm(a.float().numpy(), b.float().numpy(), c.float().numpy(), 1.0, 1.0, KN)
    A, Cc = a.view(2, 48, K).to(DEV), c.view(2, 48, N).to(DEV)
    D = torch.empty_like(Cc)
    kerns.gemm(qt, qb, qs, 1.0, 1.0, A, b.to(DEV), Cc, D)
    assert_close(D.view(M, N), exact, dtype, "gemm op, k slices")


# ---- weights stored as Q8_0 blocks (minfer_gemm_q8_0; the gemm op with the type triple (8, 32, 34)) -----------------
def make_q8(M, N, K, seed):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(M, K, generator=g).half()
    w = (1 / K ** 0.5) * torch.randn(N, K, generator=g)
    c = torch.randn(M, N, generator=g).half()
    wq = torch.from_numpy(oracle.quant_q8_0(w.numpy()))                        # uint8 [N, K/32*34]
    w_deq = torch.from_numpy(oracle.dequant_q8_0(wq.numpy(), np.float16))      # what every kernel must multiply with
    return a, wq, c, w_deq


@pytest.mark.parametrize("M,N,K,alpha,beta", [
    (1, 4096, 4096, 1.0, 0.0),       # a decode step against a Llama-3-8B projection: the kernel that streams the blocks
    (8, 1024, 4096, 1.0, 1.0),
    (16, 256, 14336, 2.0, 3.0),      # a long contraction split over the eight waves
    (17, 5152, 256, 1.0, 0.0),       # two column groups per workgroup, a ragged last one
    (4, 5200, 512, 1.0, 1.0),        # the same with one block of rows
    (40, 5152, 512, 2.0, 1.0),       # three and four blocks of rows with two column groups
    (64, 5120, 256, 1.0, 0.0),
    (64, 264, 192, 0.5, 1.0),        # its largest row count; K a multiple of 64 but not of 128: a short last step
    (37, 24, 64, 1.0, 1.0),          # one step, half-empty column group
    (65, 256, 256, 1.0, 2.0),        # above 64 rows: dequantise into the workspace, then the fp16 kernels
    (300, 1032, 512, 2.0, 0.0),
    (5, 64, 96, 1.0, 1.0),           # an odd number of blocks per row: workspace path at any row count
    (3, 18, 256, 1.0, 1.0),          # out_dim not a multiple of 4 with few rows: workspace path as well
    (64, 1030, 128, 2.0, 0.0),
    # one row with K a multiple of 256: the kernel that streams whole weight rows (segments of 128 blocks)
    (1, 264, 14336, 2.0, 1.0),       # three whole segments and one of 64 blocks, the activations in LDS
    (1, 520, 4352, 1.0, 0.0),        # a last segment of 8 blocks
    (1, 2052, 768, 0.5, 1.0),        # a single segment of 24 blocks, the activations in registers
    (1, 20000, 256, 1.0, 1.0),       # ten weight rows per wave
    (1, 4, 256, 1.0, 0.0),           # one wave with four rows, the others none
    (1, 4096, 16384, 1.0, 0.0),      # the longest activation row its LDS area holds
    (1, 512, 16640, 1.0, 0.0),       # longer: back to the 16-rows-per-instruction kernel
    (2, 2052, 768, 0.5, 1.0),        # two rows: that kernel as well
    # 2-64 rows with K a multiple of 256: the stripe kernel over the raw blocks (16-column blocks shared out, chunks of four)
    (9, 12296, 256, 1.0, 1.0),       # 769 blocks over 256 workgroups, the last one half empty; one segment
    (33, 6152, 1024, 2.0, 3.0),      # from 33 rows on narrower weights too; three blocks of rows, chunks of one and two blocks
    (48, 12288, 2560, 1.0, 0.0),     # ten segments
    (64, 12304, 512, 0.5, 1.0),      # chunks of four and of three blocks
    (16, 8192, 4096, 1.0, 0.0),      # two blocks per workgroup
    (2, 14336, 4096, 1.0, 0.0),
    # fewer than 192 stripes and a workspace: K slices of the stripe kernel, summed by a second launch
    (16, 4096, 14336, 1.0, 1.0),     # 4 slices of 14 segments
    (33, 5120, 5120, 2.0, 0.0),      # 3 slices of 7, 7 and 6 segments; three blocks of rows
    (8, 8192, 8192, 1.0, 0.0),       # 2 slices
    (64, 4104, 2048, 0.5, 1.0),      # 65 stripes, the last of 8 columns: 2 slices of 4 segments; a small weight, from 16 rows
    (2, 6144, 4096, 1.0, 0.0),
    (3, 1536, 8960, 1.0, 1.0),       # long rows, 24 stripes: 10 slices of 3 or 4 segments
])
def test_gemm_q8_0_weights_against_oracle(M, N, K, alpha, beta):
    a, wq, c, w_deq = make_q8(M, N, K, seed=M * 7 + N + K)
    exact = oracle.gemm(a.float().numpy(), w_deq.float().numpy(), c.float().numpy(), alpha, beta, NK)
    da, dwq, dc = a.to(DEV), wq.to(DEV), c.to(DEV)
    d = torch.zeros(M, N, dtype=torch.float16, device=DEV)
    need = capi.lib().minfer_gemm_q8_0_workspace_bytes(M, N, K)
    streams = M <= 64 and (K // 32) % 2 == 0 and N % 4 == 0      # the raw blocks are multiplied: a workspace only for K slices
    assert streams or need > 0
    if streams:
        stripes = (N + 63) // 64
        slices = min(256 // stripes, K // 1024, 16) if M >= 2 and K % 256 == 0 and N % 8 == 0 and stripes < 192 and (N * K > 1 << 24 or M >= 16 or (K >= 6144 and M >= 8) or (K >= 8192 and stripes <= 24)) else 1
        assert need == (slices * M * N * 4 if slices > 1 else 0)
    ws = torch.full((max(need, 16),), 0xFF, dtype=torch.uint8, device=DEV)
    assert capi.gemm_q8_0(da, dwq, dc, d, alpha, beta, ws if need else None) == capi.OK, capi.last_error()
    assert_close(d, exact, torch.float16, "q8_0 weight")
    if streams and need:            # the slices are optional: without the workspace, or with too small a one, one launch
        for small in (None, ws[:need // 2]):
            d.fill_(float("nan"))
            assert capi.gemm_q8_0(da, dwq, dc, d, alpha, beta, small) == capi.OK, capi.last_error()
            assert_close(d, exact, torch.float16, "q8_0 weight, no slices")
    # the same numbers as the fp16 kernel on the dequantised weight, up to the order of the fp32 sums
    d_ref = torch.zeros_like(d)
    assert capi.gemm(da, w_deq.to(DEV), dc, d_ref, alpha, beta, NK) == capi.OK, capi.last_error()
    assert_close(d_ref, exact, torch.float16, "fp16 kernel on the dequantised weight")
    if not streams:
        assert capi.gemm_q8_0(da, dwq, dc, d, alpha, beta, None) == capi.EWORKSPACE and "workspace" in capi.last_error()


def test_gemm_op_with_q8_0_weight(kerns):
    M, N, K = 8, 2048, 4096
    a, wq, c, w_deq = make_q8(M, N, K, seed=3)
    exact = oracle.gemm(a.float().numpy(), w_deq.float().numpy(), c.float().numpy(), 1.0, 1.0, NK)
    A, Cc = a.view(2, 4, K).to(DEV), c.view(2, 4, N).to(DEV)
    D = torch.empty_like(Cc)
    assert kerns.gemm(8, 32, 34, 1.0, 1.0, A, wq.to(DEV), Cc, D) is None
    assert_close(D.view(M, N), exact, torch.float16, "gemm op, q8_0 weight")
    A2 = torch.randn(1, 200, K, dtype=torch.float16, device=DEV)
    C2 = torch.zeros(1, 200, N, dtype=torch.float16, device=DEV)
    D2 = torch.empty_like(C2)
    kerns.gemm(8, 32, 34, 1.0, 0.0, A2, wq.to(DEV), C2, D2)                      # prefill-sized: workspace path
    exact2 = oracle.gemm(A2[0].float().cpu().numpy(), w_deq.float().numpy(), None, 1.0, 0.0, NK)
    assert_close(D2[0], exact2, torch.float16, "gemm op, q8_0 weight, 200 rows")
    with pytest.raises(RuntimeError, match="Unsupported dims"):
        kerns.gemm(8, 32, 34, 1.0, 0.0, A2, wq.to(DEV)[:, :-34].contiguous(), C2, D2)
    with pytest.raises(RuntimeError, match="float16"):
        kerns.gemm(8, 32, 34, 1.0, 0.0, A2.bfloat16(), wq.to(DEV), C2.bfloat16(), D2.bfloat16())


def test_qkv_op_with_q8_0_weights(kerns):
    """The reference's QKV recipe (test/kernels.py:173-214) with the k and v weights as Q8_0 blocks and q as float16."""
    B, L, K, Nq, Nkv = 2, 3, 2048, 1024, 256
    g = torch.Generator().manual_seed(11)
    x = torch.randn(B, L, K, generator=g).half()
    wq = ((1 / K ** 0.5) * torch.randn(Nq, K, generator=g)).half()
    wk = (1 / K ** 0.5) * torch.randn(Nkv, K, generator=g)
    wv = (1 / K ** 0.5) * torch.randn(Nkv, K, generator=g)
    wk8, wv8 = (torch.from_numpy(oracle.quant_q8_0(w.numpy())) for w in (wk, wv))
    q, k, v = (torch.empty(B, L, n, dtype=torch.float16, device=DEV) for n in (Nq, Nkv, Nkv))
    assert kerns.qkv(1, 8, 8, 1, 32, 32, 2, 34, 34, x.to(DEV), wq.to(DEV), wk8.to(DEV), wv8.to(DEV), q, k, v) is None
    x2 = x.view(B * L, K).float().numpy()
    assert_close(q.view(B * L, Nq), oracle.gemm(x2, wq.float().numpy(), None, 1.0, 0.0, NK), torch.float16, "q")
    for out, w8, name in ((k, wk8, "k"), (v, wv8, "v")):
        w_deq = torch.from_numpy(oracle.dequant_q8_0(w8.numpy(), np.float16)).float().numpy()
        assert_close(out.view(B * L, Nkv), oracle.gemm(x2, w_deq, None, 1.0, 0.0, NK), torch.float16, name)
    with pytest.raises(RuntimeError, match="Q8_0 weight is uint8"):
        kerns.qkv(1, 8, 8, 1, 32, 32, 2, 34, 34, x.to(DEV), wq.to(DEV), wk8.to(DEV)[:, :-34].contiguous(), wv8.to(DEV), q, k, v)
