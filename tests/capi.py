"""ctypes view of libminfer_attn.so for the tests: calls the C ABI of include/minfer_attn.h with the
device pointers, strides and current stream of torch tensors.  No torch types cross the boundary."""
import ctypes
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(ROOT, "minfer-python_amd", "lib", "libminfer_attn.so")
HEADER = os.path.join(ROOT, "include", "minfer_attn.h")

F16, BF16, F32 = 1, 30, 0
Q8_0, Q8_0_BLOCK, Q8_0_BLOCK_BYTES = 8, 32, 34
ROPE_INTERLEAVED, ROPE_NEOX = 0, 1
GEMM_B_KN, GEMM_B_NK = 0, 1
OK, EINVAL, EWORKSPACE, ELAUNCH = 0, -1, -2, -3


class Strides(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in ("q0", "q1", "q2", "kv0", "kv1", "kv2", "o0", "o1", "o2")]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is not built; run python minfer-python_amd/build.py")
        L = ctypes.CDLL(LIB_PATH)
        i64, vp, sz = ctypes.c_int64, ctypes.c_void_p, ctypes.c_size_t
        L.minfer_attn_version.restype = ctypes.c_int
        L.minfer_attn_last_error.restype = ctypes.c_char_p
        L.minfer_flash_attn_workspace_bytes.restype = sz
        L.minfer_flash_attn_workspace_bytes.argtypes = [i64, i64]
        L.minfer_flash_attn.restype = ctypes.c_int
        L.minfer_flash_attn.argtypes = [ctypes.c_int, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64,
                                        ctypes.POINTER(Strides), vp, sz, vp]
        L.minfer_flash_attn_decode_workspace_bytes.restype = sz
        L.minfer_flash_attn_decode_workspace_bytes.argtypes = [i64, i64, i64, i64]
        L.minfer_flash_attn_decode.restype = ctypes.c_int
        L.minfer_flash_attn_decode.argtypes = [ctypes.c_int, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64,
                                               ctypes.POINTER(Strides), vp, sz, vp]
        L.minfer_flash_attn_decode_noalloc.restype = ctypes.c_int
        L.minfer_flash_attn_decode_noalloc.argtypes = [ctypes.c_int, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64,
                                                       ctypes.POINTER(Strides), vp]
        L.minfer_flash_attn_varlen.restype = ctypes.c_int
        L.minfer_flash_attn_varlen.argtypes = [ctypes.c_int, vp, vp, vp, vp, i64, i64, vp, i64, i64, i64, i64,
                                               ctypes.POINTER(Strides), vp]
        dbl = ctypes.c_double
        L.minfer_rope.restype = ctypes.c_int
        L.minfer_rope.argtypes = [ctypes.c_int, ctypes.c_int, vp, i64, i64, i64, i64, i64, i64, dbl, vp]
        L.minfer_rope_kv_append.restype = ctypes.c_int
        L.minfer_rope_kv_append.argtypes = [ctypes.c_int, ctypes.c_int, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64,
                                            i64, i64, i64, i64, i64, dbl, vp]
        L.minfer_rope_kv_append_norm.restype = ctypes.c_int
        L.minfer_rope_kv_append_norm.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp, vp, vp, vp, dbl, vp, vp, vp,
                                                 i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, dbl, vp]
        L.minfer_rmsnorm.restype = ctypes.c_int
        L.minfer_rmsnorm.argtypes = [ctypes.c_int, vp, vp, vp, i64, i64, dbl, vp]
        L.minfer_gemm.restype = ctypes.c_int
        L.minfer_gemm.argtypes = [ctypes.c_int, ctypes.c_int, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, dbl, dbl, vp]
        L.minfer_gemm_ws.restype = ctypes.c_int
        L.minfer_gemm_ws.argtypes = [ctypes.c_int, ctypes.c_int, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, dbl, dbl, vp, ctypes.c_size_t, vp]
        L.minfer_gemm_workspace_bytes.restype = ctypes.c_size_t
        L.minfer_gemm_workspace_bytes.argtypes = [i64, i64, i64]
        L.minfer_gemm_q8_0.restype = ctypes.c_int
        L.minfer_gemm_q8_0.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, dbl, dbl, vp, ctypes.c_size_t, vp]
        L.minfer_gemm_q8_0_workspace_bytes.restype = ctypes.c_size_t
        L.minfer_gemm_q8_0_workspace_bytes.argtypes = [i64, i64, i64]
        L.minfer_qkv.restype = ctypes.c_int
        L.minfer_qkv.argtypes = [ctypes.c_int, vp, vp, vp, vp, vp, vp, vp] + [i64] * 12 + [vp]
        L.minfer_quant_q8_0.restype = ctypes.c_int
        L.minfer_quant_q8_0.argtypes = [ctypes.c_int, vp, vp, i64, i64, vp]
        L.minfer_dequant_q8_0.restype = ctypes.c_int
        L.minfer_dequant_q8_0.argtypes = [ctypes.c_int, vp, vp, i64, i64, vp]
        L.minfer_flash_attn_decode_q8_0.restype = ctypes.c_int
        L.minfer_flash_attn_decode_q8_0.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64,
                                                    ctypes.POINTER(Strides), vp, sz, vp]
        L.minfer_flash_attn_q8_0_workspace_bytes.restype = sz
        L.minfer_flash_attn_q8_0_workspace_bytes.argtypes = [i64, i64, i64, i64]
        L.minfer_flash_attn_q8_0.restype = ctypes.c_int
        L.minfer_flash_attn_q8_0.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, ctypes.POINTER(Strides), vp, sz, vp]
        L.minfer_flash_attn_varlen_q8_0_workspace_bytes.restype = sz
        L.minfer_flash_attn_varlen_q8_0_workspace_bytes.argtypes = [i64, i64, i64]
        L.minfer_flash_attn_varlen_q8_0.restype = ctypes.c_int
        L.minfer_flash_attn_varlen_q8_0.argtypes = [vp, vp, vp, vp, i64, i64, vp, i64, i64, i64, i64, ctypes.POINTER(Strides), vp, sz, vp]
        L.minfer_rope_kv_append_q8_0.restype = ctypes.c_int
        L.minfer_rope_kv_append_q8_0.argtypes = [ctypes.c_int, ctypes.c_int, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64,
                                                 i64, i64, i64, i64, i64, dbl, vp]
        _lib = L
    return _lib


def last_error():
    return lib().minfer_attn_last_error().decode()


def _dtype_code(t):
    import torch
    return {torch.float16: F16, torch.bfloat16: BF16, torch.float32: F32}[t.dtype]


def _strides(q, k, o):
    return Strides(q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
                   o.stride(0), o.stride(1), o.stride(2))


def _stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def flash_attn(q, k, v, mask, out, workspace=None):
    """Returns the C ABI's return code; `out` is written in place."""
    import torch
    B, Hq, L, D = q.shape
    need = lib().minfer_flash_attn_workspace_bytes(B, L)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    st = _strides(q, k, out)
    return lib().minfer_flash_attn(_dtype_code(q), q.data_ptr(), k.data_ptr(), v.data_ptr(), mask.data_ptr(),
                                   out.data_ptr(), B, Hq, k.shape[1], L, D, ctypes.byref(st),
                                   workspace.data_ptr(), workspace.numel(), _stream())


def flash_attn_decode(q, k_cache, v_cache, ctx_lens, out, workspace=None):
    import torch
    B, Hq, _, D = q.shape
    Hkv, Lmax = k_cache.shape[1], k_cache.shape[2]
    need = lib().minfer_flash_attn_decode_workspace_bytes(B, Hq, Lmax, D)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    st = _strides(q, k_cache, out)
    return lib().minfer_flash_attn_decode(_dtype_code(q), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                          ctx_lens.data_ptr(), out.data_ptr(), B, Hq, Hkv, Lmax, D,
                                          ctypes.byref(st), workspace.data_ptr(), workspace.numel(), _stream())


DECODE_NOALLOC_SCRATCH_BYTES = 64 << 20


def flash_attn_decode_noalloc(q, k_cache, v_cache, ctx_lens, out):
    """The decode entry point that takes no workspace and allocates nothing."""
    B, Hq, _, D = q.shape
    st = _strides(q, k_cache, out)
    return lib().minfer_flash_attn_decode_noalloc(_dtype_code(q), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                                  ctx_lens.data_ptr(), out.data_ptr(), B, Hq, k_cache.shape[1],
                                                  k_cache.shape[2], D, ctypes.byref(st), _stream())


def flash_attn_varlen(q, k, v, cu_seqlens, max_seqlen, out):
    _, Hq, T, D = q.shape
    st = _strides(q, k, out)
    return lib().minfer_flash_attn_varlen(_dtype_code(q), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                          cu_seqlens.data_ptr(), cu_seqlens.numel() - 1, max_seqlen, out.data_ptr(),
                                          Hq, k.shape[1], T, D, ctypes.byref(st), _stream())


def rope(style, x, rotary_dim, start_pos, freq_base):
    """In-place rotary embedding of x [B,L,H,D] (contiguous)."""
    B, L, H, D = x.shape
    return lib().minfer_rope(_dtype_code(x), style, x.data_ptr(), B, L, H, D, rotary_dim, start_pos, freq_base, _stream())


def rope_kv_append(style, q, k, v, positions, k_cache, v_cache, rotary_dim, freq_base):
    """q [B,L,Hq,D] in place; k, v [B,L,Hkv,D] into rows positions[b]+l of the caches [B,Hkv,Lmax,D]."""
    B, L, Hq, D = q.shape
    return lib().minfer_rope_kv_append(_dtype_code(q), style, q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                       positions.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), B, L, Hq,
                                       k.shape[2], D, k_cache.shape[2], k_cache.stride(0), k_cache.stride(1),
                                       k_cache.stride(2), rotary_dim, freq_base, _stream())


def rope_kv_append_norm(style, q, k, v, wq_norm, wk_norm, eps, positions, k_cache, v_cache, rotary_dim, freq_base):
    """rope_kv_append with per-head RMS normalisation of q and k first (a weight may be None); uint8 caches are Q8_0."""
    import torch
    B, L, Hq, D = q.shape
    cache_type = Q8_0 if k_cache.dtype == torch.uint8 else _dtype_code(q)
    return lib().minfer_rope_kv_append_norm(_dtype_code(q), style, cache_type, q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                            wq_norm.data_ptr() if wq_norm is not None else None,
                                            wk_norm.data_ptr() if wk_norm is not None else None, eps,
                                            positions.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), B, L, Hq,
                                            k.shape[2], D, k_cache.shape[2], k_cache.stride(0), k_cache.stride(1),
                                            k_cache.stride(2), rotary_dim, freq_base, _stream())


def rmsnorm(x, w, out, eps):
    """RMS normalisation of contiguous x over vectors of length len(w), into out."""
    dim = w.shape[0]
    return lib().minfer_rmsnorm(_dtype_code(x), x.data_ptr(), w.data_ptr(), out.data_ptr(), x.numel() // dim, dim, eps, _stream())


def gemm(a, b, c, d, alpha, beta, b_layout=GEMM_B_KN):
    """d[M,N] = alpha * a[M,K] x b + beta * c; 2-D tensors with unit stride on their last dimension; b is
    [K,N] (GEMM_B_KN) or [N,K] (GEMM_B_NK); c may be None when beta == 0."""
    M, K = a.shape
    N = d.shape[1]
    return lib().minfer_gemm(_dtype_code(a), b_layout, a.data_ptr(), b.data_ptr(), c.data_ptr() if c is not None else None,
                             d.data_ptr(), M, N, K, a.stride(0), b.stride(0), c.stride(0) if c is not None else N, d.stride(0),
                             alpha, beta, _stream())


def gemm_ws(a, b, c, d, alpha, beta, ws, b_layout=GEMM_B_KN):
    """gemm with a workspace tensor (uint8, device) that lets a few-row problem run as K slices; ws may be None."""
    M, K = a.shape
    N = d.shape[1]
    return lib().minfer_gemm_ws(_dtype_code(a), b_layout, a.data_ptr(), b.data_ptr(), c.data_ptr() if c is not None else None,
                                d.data_ptr(), M, N, K, a.stride(0), b.stride(0), c.stride(0) if c is not None else N, d.stride(0),
                                alpha, beta, ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, _stream())


def gemm_q8_0(a, bq, c, d, alpha, beta, ws=None):
    """d[M,N] = alpha * a[M,K] x dequant(bq)^T + beta * c; bq uint8 [N, K/32*34] rows of Q8_0 blocks; fp16 a, c, d."""
    M, K = a.shape
    N = d.shape[1]
    return lib().minfer_gemm_q8_0(a.data_ptr(), bq.data_ptr(), c.data_ptr() if c is not None else None, d.data_ptr(), M, N, K,
                                  a.stride(0), c.stride(0) if c is not None else N, d.stride(0), alpha, beta,
                                  ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, _stream())


def qkv(x, wq, wk, wv, q_out, k_out, v_out):
    """The three projections x [M,K] against weights [N,K] into outputs [M,N], one launch."""
    M, K = x.shape
    return lib().minfer_qkv(_dtype_code(x), x.data_ptr(), wq.data_ptr(), wk.data_ptr(), wv.data_ptr(), q_out.data_ptr(),
                            k_out.data_ptr(), v_out.data_ptr(), M, K, wq.shape[0], wk.shape[0], wv.shape[0], x.stride(0),
                            wq.stride(0), wk.stride(0), wv.stride(0), q_out.stride(0), k_out.stride(0), v_out.stride(0),
                            _stream())


def quant_q8_0(x, y):
    """Rows of contiguous x [n, k] (fp32, fp16 or bf16) into rows of Q8_0 blocks y, uint8 [n, k/32*34]."""
    k = x.shape[-1]
    return lib().minfer_quant_q8_0(_dtype_code(x), x.data_ptr(), y.data_ptr(), x.numel() // max(k, 1), k, _stream())


def dequant_q8_0(x, y):
    """Rows of Q8_0 blocks x, uint8 [n, k/32*34], into contiguous y [n, k] (fp32 or fp16)."""
    k = y.shape[-1]
    return lib().minfer_dequant_q8_0(_dtype_code(y), x.data_ptr(), y.data_ptr(), y.numel() // max(k, 1), k, _stream())


def flash_attn_decode_q8_0(q, k_cache, v_cache, ctx_lens, out, workspace=None):
    """q, out fp16 [B,Hq,1,D]; caches uint8 [B,Hkv,Lmax,D/32*34] (dims 0, 1 may be strided)."""
    import torch
    B, Hq, _, D = q.shape
    Hkv, Lmax = k_cache.shape[1], k_cache.shape[2]
    need = lib().minfer_flash_attn_decode_workspace_bytes(B, Hq, Lmax, D)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    st = _strides(q, k_cache, out)   # a uint8 tensor's strides are byte strides
    return lib().minfer_flash_attn_decode_q8_0(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                               ctx_lens.data_ptr(), out.data_ptr(), B, Hq, Hkv, Lmax, D,
                                               ctypes.byref(st), workspace.data_ptr(), workspace.numel(), _stream())


def flash_attn_q8_0(q, k, v, mask, out):
    """Dense-mask prefill with k, v as Q8_0 blocks, uint8 [B,Hkv,L,D/32*34] (dims 0, 1 may be strided)."""
    import torch
    B, Hq, L, D = q.shape
    need = lib().minfer_flash_attn_q8_0_workspace_bytes(B, k.shape[1], L, D)
    ws = torch.empty(need, dtype=torch.uint8, device=q.device)
    st = _strides(q, k, out)
    return lib().minfer_flash_attn_q8_0(q.data_ptr(), k.data_ptr(), v.data_ptr(), mask.data_ptr(), out.data_ptr(), B, Hq,
                                        k.shape[1], L, D, ctypes.byref(st), ws.data_ptr(), ws.numel(), _stream())


def flash_attn_varlen_q8_0(q, k, v, cu_seqlens, max_seqlen, out):
    """Packed ragged prefill with k, v as Q8_0 blocks, uint8 [1,Hkv,T,D/32*34]."""
    import torch
    _, Hq, T, D = q.shape
    need = lib().minfer_flash_attn_varlen_q8_0_workspace_bytes(k.shape[1], T, D)
    ws = torch.empty(need, dtype=torch.uint8, device=q.device)
    st = _strides(q, k, out)
    return lib().minfer_flash_attn_varlen_q8_0(q.data_ptr(), k.data_ptr(), v.data_ptr(), cu_seqlens.data_ptr(),
                                               cu_seqlens.numel() - 1, max_seqlen, out.data_ptr(), Hq, k.shape[1], T, D,
                                               ctypes.byref(st), ws.data_ptr(), ws.numel(), _stream())


def rope_kv_append_q8_0(style, q, k, v, positions, k_cache, v_cache, rotary_dim, freq_base):
    """As rope_kv_append, into Q8_0 caches, uint8 [B,Hkv,Lmax,D/32*34] with dense rows."""
    B, L, Hq, D = q.shape
    return lib().minfer_rope_kv_append_q8_0(_dtype_code(q), style, q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                            positions.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), B, L, Hq,
                                            k.shape[2], D, k_cache.shape[2], k_cache.stride(0), k_cache.stride(1),
                                            rotary_dim, freq_base, _stream())
