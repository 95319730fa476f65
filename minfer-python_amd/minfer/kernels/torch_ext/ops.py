"""Python wrappers and fake (meta) kernels of the attention ops and of the rotary-embedding step
before them, mirroring the reference's wrapper layer (reference:
src/minfer/kernels/torch_ext/ops.py:60-266): positional pass-through
to ``torch.ops.minfer.<op>.default``; the result is written into ``out``."""
import torch

_ACT_DTYPES = (torch.float16, torch.bfloat16)
_Q8_0 = 8   # GGML type number of the one block format built here: 32 values in 34 bytes


def dequant(qtype: int, qblock_size: int, qtype_size: int, x: torch.Tensor, y: torch.Tensor):
    """Dequantises the rows of x (uint8 [M, N/32*34], Q8_0 blocks) into y (float32 or float16 [M, N]);
    qblock_size is the number of values per block, qtype_size its bytes (reference: ops.py:8-21)."""
    return torch.ops.minfer.dequant.default(qtype, qblock_size, qtype_size, x, y)


@torch.library.register_fake("minfer::dequant")
def _(qtype, qblock_size, qtype_size, x, y):
    torch._check(x.dtype == torch.uint8)
    torch._check(y.dtype in (torch.float32, torch.float16))
    torch._check(x.device == y.device)
    torch._check(x.device.type == "cuda")
    torch._check(x.size(0) == y.size(0))


def quant(qtype: int, qblock_size: int, qtype_size: int, x: torch.Tensor, y: torch.Tensor):
    """Quantises the rows of x (float32 [M, N]; float16/bfloat16 also taken) into y (uint8 [M, N/32*34], Q8_0
    blocks), on the device (reference: ops.py:33-46, CPU only there)."""
    return torch.ops.minfer.quant.default(qtype, qblock_size, qtype_size, x, y)


@torch.library.register_fake("minfer::quant")
def _(qtype, qblock_size, qtype_size, x, y):
    torch._check(x.dtype in (torch.float32, torch.float16, torch.bfloat16))
    torch._check(y.dtype == torch.uint8)
    torch._check(x.device == y.device)
    torch._check(x.device.type == "cuda")
    torch._check(x.size(0) == y.size(0))


def flash_attn(
    qtype_int: int,
    qblock_size: int,
    qtype_size: int,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    mask: torch.Tensor,
    out: torch.Tensor,
):
    """Fused GQA attention under a dense bool mask [B,1,L,L] (True = attend).
    q/out [B,n_heads,L,D], k/v [B,n_kv_heads,L,D], any strides with unit stride on D.  With (qtype_int, qblock_size,
    qtype_size) = (8, 32, 34), k and v are Q8_0 blocks, uint8 [B,n_kv_heads,L,D/32*34], and q/out float16."""
    return torch.ops.minfer.flash_attn.default(qtype_int, qblock_size, qtype_size, q, k, v, mask, out)


@torch.library.register_fake("minfer::flash_attn")
def _(qtype_int, qblock_size, qtype_size, q, k, v, mask, out):
    torch._check(q.dtype in _ACT_DTYPES)
    kv_dtype = torch.uint8 if qtype_int == _Q8_0 else q.dtype
    torch._check(k.dtype == kv_dtype and v.dtype == kv_dtype and out.dtype == q.dtype)
    torch._check(mask.dtype == torch.bool)
    torch._check(q.device == k.device == v.device == out.device)
    torch._check(q.device.type == "cuda")
    torch._check(q.dim() == 4 and k.dim() == 4 and v.dim() == 4 and mask.dim() == 4 and out.dim() == 4)


def flash_attn_decode(
    qtype_int: int,
    qblock_size: int,
    qtype_size: int,
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    ctx_lens: torch.Tensor,
    out: torch.Tensor,
):
    """Single-token decode: q/out [B,n_heads,1,D] against caches [B,n_kv_heads,Lmax,D]; query b
    attends cache rows 0..ctx_lens[b]-1 (ctx_lens int32 [B]).  With (qtype_int, qblock_size, qtype_size) =
    (8, 32, 34) the caches are Q8_0 blocks, uint8 [B,n_kv_heads,Lmax,D/32*34], and q/out float16."""
    return torch.ops.minfer.flash_attn_decode.default(qtype_int, qblock_size, qtype_size, q, k_cache, v_cache, ctx_lens, out)


@torch.library.register_fake("minfer::flash_attn_decode")
def _(qtype_int, qblock_size, qtype_size, q, k_cache, v_cache, ctx_lens, out):
    torch._check(q.dtype in _ACT_DTYPES and out.dtype == q.dtype)
    cache_dtype = torch.uint8 if qtype_int == _Q8_0 else q.dtype
    torch._check(k_cache.dtype == cache_dtype and v_cache.dtype == cache_dtype)
    torch._check(ctx_lens.dtype == torch.int32)
    torch._check(q.device == k_cache.device == v_cache.device == ctx_lens.device == out.device)
    torch._check(q.device.type == "cuda")
    torch._check(q.dim() == 4 and k_cache.dim() == 4 and v_cache.dim() == 4 and out.dim() == 4 and ctx_lens.dim() == 1)


def flash_attn_varlen(
    qtype_int: int,
    qblock_size: int,
    qtype_size: int,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens: torch.Tensor,
    max_seqlen: int,
    out: torch.Tensor,
):
    """Packed ragged causal prefill: q/out [1,n_heads,T,D], k/v [1,n_kv_heads,T,D], cu_seqlens
    int32 [n_seqs+1]; rows cu_seqlens[s]..cu_seqlens[s+1]-1 attend causally among themselves."""
    return torch.ops.minfer.flash_attn_varlen.default(qtype_int, qblock_size, qtype_size, q, k, v, cu_seqlens, max_seqlen, out)


@torch.library.register_fake("minfer::flash_attn_varlen")
def _(qtype_int, qblock_size, qtype_size, q, k, v, cu_seqlens, max_seqlen, out):
    torch._check(q.dtype in _ACT_DTYPES)
    kv_dtype = torch.uint8 if qtype_int == _Q8_0 else q.dtype
    torch._check(k.dtype == kv_dtype and v.dtype == kv_dtype and out.dtype == q.dtype)
    torch._check(cu_seqlens.dtype == torch.int32)
    torch._check(q.device == k.device == v.device == cu_seqlens.device == out.device)
    torch._check(q.device.type == "cuda")
    torch._check(q.dim() == 4 and k.dim() == 4 and v.dim() == 4 and out.dim() == 4 and cu_seqlens.dim() == 1)



def il_rope(rotary_dim: int, start_pos: int, freq_base: float, x: torch.Tensor):
    """Interleaved rotary embedding, in place; x [B,L,n_heads,head_dim], token l at position start_pos + l."""
    return torch.ops.minfer.il_rope.default(rotary_dim, start_pos, freq_base, x)


@torch.library.register_fake("minfer::il_rope")
def _(rotary_dim, start_pos, freq_base, x):
    torch._check(x.dtype in _ACT_DTYPES)
    torch._check(x.dim() == 4)
    torch._check(x.device.type == "cuda")
    torch._check(rotary_dim <= x.size(3))


def neox_rope(rotary_dim: int, start_pos: int, freq_base: float, x: torch.Tensor):
    """NeoX (two-halves) rotary embedding, in place; x [B,L,n_heads,head_dim]."""
    return torch.ops.minfer.neox_rope.default(rotary_dim, start_pos, freq_base, x)


@torch.library.register_fake("minfer::neox_rope")
def _(rotary_dim, start_pos, freq_base, x):
    torch._check(x.dtype in _ACT_DTYPES)
    torch._check(x.dim() == 4)
    torch._check(x.device.type == "cuda")
    torch._check(rotary_dim <= x.size(3))


def rope_kv_append(
    style: int,
    rotary_dim: int,
    freq_base: float,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    positions: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
):
    """Rotates q [B,L,n_heads,D] in place, writes the rotated k [B,L,n_kv_heads,D] and v into rows
    positions[b] + l of the caches [B,n_kv_heads,Lmax,D]; style 0 = interleaved, 1 = NeoX; positions
    int32 [B].  uint8 caches [B,n_kv_heads,Lmax,D/32*34] receive the rows as Q8_0 blocks."""
    return torch.ops.minfer.rope_kv_append.default(style, rotary_dim, freq_base, q, k, v, positions, k_cache, v_cache)


@torch.library.register_fake("minfer::rope_kv_append")
def _(style, rotary_dim, freq_base, q, k, v, positions, k_cache, v_cache):
    torch._check(q.dtype in _ACT_DTYPES)
    torch._check(k.dtype == q.dtype and v.dtype == q.dtype)
    torch._check(k_cache.dtype in (q.dtype, torch.uint8) and v_cache.dtype == k_cache.dtype)
    torch._check(positions.dtype == torch.int32)
    torch._check(q.device.type == "cuda")
    torch._check(q.dim() == 4 and k.dim() == 4 and v.dim() == 4 and k_cache.dim() == 4 and v_cache.dim() == 4)
    torch._check(rotary_dim <= q.size(3))


def rope_kv_append_norm(
    style: int,
    rotary_dim: int,
    freq_base: float,
    eps: float,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    wq_norm: torch.Tensor,
    wk_norm: torch.Tensor,
    positions: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
):
    """rope_kv_append with the per-head RMS normalisation of q (weight wq_norm [D]) and k (wk_norm [D]) in front of
    the rotation: equals rmsnorm(q), rmsnorm(k), rope_kv_append in one pass (the reference model's optional q/k norm)."""
    return torch.ops.minfer.rope_kv_append_norm.default(style, rotary_dim, freq_base, eps, q, k, v, wq_norm, wk_norm,
                                                        positions, k_cache, v_cache)


@torch.library.register_fake("minfer::rope_kv_append_norm")
def _(style, rotary_dim, freq_base, eps, q, k, v, wq_norm, wk_norm, positions, k_cache, v_cache):
    torch._check(q.dtype in _ACT_DTYPES)
    torch._check(k.dtype == q.dtype and v.dtype == q.dtype and wq_norm.dtype == q.dtype and wk_norm.dtype == q.dtype)
    torch._check(k_cache.dtype in (q.dtype, torch.uint8) and v_cache.dtype == k_cache.dtype)
    torch._check(positions.dtype == torch.int32)
    torch._check(q.device.type == "cuda")
    torch._check(q.dim() == 4 and k.dim() == 4 and v.dim() == 4 and k_cache.dim() == 4 and v_cache.dim() == 4)
    torch._check(wq_norm.dim() == 1 and wk_norm.dim() == 1)
    torch._check(rotary_dim <= q.size(3))


def rmsnorm(eps: float, input: torch.Tensor, w: torch.Tensor, out: torch.Tensor):
    """RMS normalisation over vectors of length len(w) (the whole hidden dimension, or per head)."""
    return torch.ops.minfer.rmsnorm.default(eps, input, w, out)


@torch.library.register_fake("minfer::rmsnorm")
def _(eps, input, w, out):
    torch._check(input.dtype in _ACT_DTYPES)
    torch._check(w.dtype == input.dtype and out.dtype == input.dtype)
    torch._check(input.device == w.device == out.device)
    torch._check(input.device.type == "cuda")
    torch._check(input.shape == out.shape)
    torch._check(input.dim() in (3, 4))
    torch._check(input.size(-1) == w.size(0) or input.size(-1) % w.size(0) == 0)


def gemm(qtype_int: int, qblock_size: int, qtype_size: int, alpha: float, beta: float,
         A: torch.Tensor, B: torch.Tensor, C: torch.Tensor, D: torch.Tensor):
    """D = alpha * A B + beta * C; A [B,L,in_dim], weight B [in_dim,out_dim] (or [out_dim,in_dim]: A B^T), C and D
    [B,L,out_dim].  With (qtype_int, qblock_size, qtype_size) = (8, 32, 34) the weight is uint8 [out_dim, in_dim/32*34],
    rows of Q8_0 blocks, and the product is A B^T over the dequantised weight."""
    return torch.ops.minfer.gemm.default(qtype_int, qblock_size, qtype_size, alpha, beta, A, B, C, D)


@torch.library.register_fake("minfer::gemm")
def _(qtype_int, qblock_size, qtype_size, alpha, beta, A, B, C, D):
    torch._check(A.dtype in _ACT_DTYPES)
    torch._check(C.dtype == A.dtype and D.dtype == A.dtype)
    torch._check(B.dtype == (torch.uint8 if qtype_int == 8 else A.dtype))
    torch._check(A.device == B.device == C.device == D.device)
    torch._check(A.device.type == "cuda")
    torch._check(A.dim() == 3 and B.dim() == 2 and C.dim() == 3 and D.dim() == 3)
    torch._check(A.size(0) * A.size(1) == C.size(0) * C.size(1))
    torch._check(B.size(-1) == C.size(-1) or B.size(0) == C.size(-1))
    torch._check(C.shape == D.shape)
    torch._check(alpha != 0.0)


def qkv(q_qtype_int: int, k_qtype_int: int, v_qtype_int: int, q_qblock_size: int, k_qblock_size: int, v_qblock_size: int,
        q_qtype_size: int, k_qtype_size: int, v_qtype_size: int,
        x: torch.Tensor, wq: torch.Tensor, wk: torch.Tensor, wv: torch.Tensor,
        q_out: torch.Tensor, k_out: torch.Tensor, v_out: torch.Tensor):
    """The three projections q_out = x wq^T, k_out = x wk^T, v_out = x wv^T; x [B,L,hidden], weights [out,hidden]; a
    weight whose type triple is (8, 32, 34) is uint8 [out, hidden/32*34], rows of Q8_0 blocks."""
    return torch.ops.minfer.qkv.default(q_qtype_int, k_qtype_int, v_qtype_int, q_qblock_size, k_qblock_size, v_qblock_size,
                                        q_qtype_size, k_qtype_size, v_qtype_size, x, wq, wk, wv, q_out, k_out, v_out)


@torch.library.register_fake("minfer::qkv")
def _(q_qtype_int, k_qtype_int, v_qtype_int, q_qblock_size, k_qblock_size, v_qblock_size, q_qtype_size, k_qtype_size,
      v_qtype_size, x, wq, wk, wv, q_out, k_out, v_out):
    torch._check(x.dtype in _ACT_DTYPES)
    torch._check(all(t.dtype == x.dtype for t in (q_out, k_out, v_out)))
    torch._check(all(w.dtype == (torch.uint8 if qt == 8 else x.dtype) for w, qt in ((wq, q_qtype_int), (wk, k_qtype_int), (wv, v_qtype_int))))
    torch._check(x.device == wq.device == wk.device == wv.device == q_out.device == k_out.device == v_out.device)
    torch._check(x.device.type == "cuda")
    torch._check(x.dim() == 3 and q_out.dim() == 3 and k_out.dim() == 3 and v_out.dim() == 3)
    torch._check(wq.dim() == 2 and wk.dim() == 2 and wv.dim() == 2)
