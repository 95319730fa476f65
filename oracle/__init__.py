"""TEST INFRASTRUCTURE ONLY: ctypes access to the CPU oracle in attn_oracle.c, rope_oracle.c, rmsnorm_oracle.c,
gemm_oracle.c and quant_oracle.c.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this
package.  The shipped operator never does: it launches HIP kernels or raises.

Each wrapper takes numpy arrays or torch CPU tensors of any float dtype, up-casts them to
contiguous fp32 and returns a float32 numpy array in the reference operator's layout
([B,Hq,L,D]; reference: src/minfer/kernels/torch_ext/csrc/cuda/flash_attn/op.cuh:21-30).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


class _Strides(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in ("q0", "q1", "q2", "kv0", "kv1", "kv2", "o0", "o1", "o2")]


def build(force=False):
    """Compile the oracle's C files into liboracle.so (gcc + OpenMP)."""
    so = os.path.join(_HERE, "liboracle.so")
    if force and os.path.exists(so):
        os.remove(so)
    subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, stdout=subprocess.DEVNULL)
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(so):
            build()
        _LIB = ctypes.CDLL(so)
        for name in ("oracle_flash_attn", "oracle_flash_attn_rows", "oracle_flash_attn_decode",
                     "oracle_flash_attn_varlen", "oracle_rope", "oracle_rope_kv_append", "oracle_rmsnorm", "oracle_gemm",
                     "oracle_quant_q8_0", "oracle_dequant_q8_0", "oracle_dequant_q8_0_f16"):
            getattr(_LIB, name).restype = ctypes.c_int
        _LIB.oracle_f32_to_f16.restype = ctypes.c_uint16
        _LIB.oracle_f32_to_f16.argtypes = [ctypes.c_float]
        _LIB.oracle_f16_to_f32.restype = ctypes.c_float
        _LIB.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
    return _LIB


def _f32(x):
    if hasattr(x, "detach"):
        x = x.detach().to("cpu").float().numpy()
    return np.ascontiguousarray(np.asarray(x, dtype=np.float32))


def _ptr(a, ty=ctypes.c_float):
    return a.ctypes.data_as(ctypes.POINTER(ty))


def _contig_strides(q, k, o):
    s = lambda a: [x // a.itemsize for x in a.strides[:3]]
    return _Strides(*s(q), *s(k), *s(o))


def flash_attn(q, k, v, mask):
    """Dense bool-mask GQA attention; the reference op's semantics (refs.py:53-55)."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    if hasattr(mask, "detach"):
        mask = mask.detach().to("cpu").numpy()
    B, Hq, L, D = q.shape
    Hkv = k.shape[1]
    mask = np.ascontiguousarray(np.broadcast_to(np.asarray(mask, dtype=np.bool_), (B, 1, L, L))).view(np.uint8)
    out = np.empty_like(q)
    st = _contig_strides(q, k, out)
    rc = lib().oracle_flash_attn(_ptr(q), _ptr(k), _ptr(v), _ptr(mask, ctypes.c_uint8), _ptr(out),
                                 *[ctypes.c_int64(x) for x in (B, Hq, Hkv, L, D)], ctypes.byref(st))
    if rc != 0:
        raise ValueError(f"oracle_flash_attn rc={rc}")
    return out


def flash_attn_rows(q, k, v, mask_rows, rows):
    """flash_attn restricted to query rows `rows`; mask_rows is bool [B,n,L] (= mask[:,0,rows,:]).
    Returns [B,Hq,n,D]."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    if hasattr(mask_rows, "detach"):
        mask_rows = mask_rows.detach().to("cpu").numpy()
    B, Hq, L, D = q.shape
    Hkv = k.shape[1]
    rows = np.ascontiguousarray(np.asarray(rows, dtype=np.int64))
    n = len(rows)
    mask_rows = np.ascontiguousarray(np.broadcast_to(np.asarray(mask_rows, dtype=np.bool_), (B, n, L))).view(np.uint8)
    out = np.empty((B, Hq, n, D), dtype=np.float32)
    st = _contig_strides(q, k, q)
    rc = lib().oracle_flash_attn_rows(_ptr(q), _ptr(k), _ptr(v), _ptr(mask_rows, ctypes.c_uint8),
                                      _ptr(rows, ctypes.c_int64), ctypes.c_int64(n), _ptr(out),
                                      *[ctypes.c_int64(x) for x in (B, Hq, Hkv, L, D)], ctypes.byref(st))
    if rc != 0:
        raise ValueError(f"oracle_flash_attn_rows rc={rc}")
    return out


def flash_attn_decode(q, k_cache, v_cache, ctx_lens):
    """q [B,Hq,1,D] against caches [B,Hkv,Lmax,D], keys 0..ctx_lens[b]-1."""
    q, k_cache, v_cache = _f32(q), _f32(k_cache), _f32(v_cache)
    if hasattr(ctx_lens, "detach"):
        ctx_lens = ctx_lens.detach().to("cpu").numpy()
    ctx = np.ascontiguousarray(np.asarray(ctx_lens, dtype=np.int32))
    B, Hq, _, D = q.shape
    Hkv, Lmax = k_cache.shape[1], k_cache.shape[2]
    out = np.empty_like(q)
    st = _contig_strides(q, k_cache, out)
    rc = lib().oracle_flash_attn_decode(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(ctx, ctypes.c_int32),
                                        _ptr(out), *[ctypes.c_int64(x) for x in (B, Hq, Hkv, Lmax, D)],
                                        ctypes.byref(st))
    if rc != 0:
        raise ValueError(f"oracle_flash_attn_decode rc={rc}")
    return out


def flash_attn_varlen(q, k, v, cu_seqlens):
    """Packed ragged causal prefill: q [1,Hq,T,D], k/v [1,Hkv,T,D], cu_seqlens [N+1]."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    if hasattr(cu_seqlens, "detach"):
        cu_seqlens = cu_seqlens.detach().to("cpu").numpy()
    cu = np.ascontiguousarray(np.asarray(cu_seqlens, dtype=np.int32))
    _, Hq, T, D = q.shape
    Hkv = k.shape[1]
    out = np.empty_like(q)
    st = _contig_strides(q, k, out)
    rc = lib().oracle_flash_attn_varlen(_ptr(q), _ptr(k), _ptr(v), _ptr(cu, ctypes.c_int32),
                                        ctypes.c_int64(len(cu) - 1), _ptr(out),
                                        *[ctypes.c_int64(x) for x in (Hq, Hkv, T, D)], ctypes.byref(st))
    if rc != 0:
        raise ValueError(f"oracle_flash_attn_varlen rc={rc}")
    return out


ROPE_INTERLEAVED, ROPE_NEOX = 0, 1


def rope(style, x, rotary_dim, start_pos, freq_base):
    """Rotary embedding of x [B,L,H,D] (reference: refs.py:12-47), fp64 arithmetic; returns a new
    float32 array, unrounded."""
    x = _f32(x).copy()
    B, L, H, D = x.shape
    rc = lib().oracle_rope(ctypes.c_int(style), _ptr(x), *[ctypes.c_int64(v) for v in (B, L, H, D, rotary_dim, start_pos)],
                           ctypes.c_double(freq_base))
    if rc != 0:
        raise ValueError(f"oracle_rope rc={rc}")
    return x


def rope_kv_append(style, q, k, v, positions, k_cache, v_cache, rotary_dim, freq_base):
    """rope(q), rope(k) -> k_cache rows positions[b]+l, v -> v_cache rows (reference: core.py:228-232,
    cache layout core.py:105-127).  q/k/v [B,L,H*,D], caches [B,Hkv,Lmax,D].  Returns new float32
    arrays (q, k_cache, v_cache)."""
    q, k, v = _f32(q).copy(), _f32(k), _f32(v)
    k_cache, v_cache = _f32(k_cache).copy(), _f32(v_cache).copy()
    if hasattr(positions, "detach"):
        positions = positions.detach().to("cpu").numpy()
    pos = np.ascontiguousarray(np.asarray(positions, dtype=np.int32))
    B, L, Hq, D = q.shape
    Hkv, Lmax = k_cache.shape[1], k_cache.shape[2]
    rc = lib().oracle_rope_kv_append(ctypes.c_int(style), _ptr(q), _ptr(k), _ptr(v), _ptr(pos, ctypes.c_int32),
                                     _ptr(k_cache), _ptr(v_cache),
                                     *[ctypes.c_int64(x) for x in (B, L, Hq, Hkv, D, Lmax, rotary_dim)],
                                     ctypes.c_double(freq_base))
    if rc != 0:
        raise ValueError(f"oracle_rope_kv_append rc={rc}")
    return q, k_cache, v_cache


def rmsnorm(x, w, eps):
    """x * w / sqrt(mean(x^2 over vectors of len(w)) + eps) (reference: refs.py:4-10, rmsnorm/kernel.cuh:24-38),
    fp64 arithmetic; returns a new float32 array of x's shape, unrounded."""
    x, w = _f32(x), _f32(w)
    dim = w.shape[0]
    out = np.empty_like(x)
    rc = lib().oracle_rmsnorm(_ptr(x), _ptr(w), _ptr(out), ctypes.c_int64(x.size // dim), ctypes.c_int64(dim), ctypes.c_double(eps))
    if rc != 0:
        raise ValueError(f"oracle_rmsnorm rc={rc}")
    return out


GEMM_B_KN, GEMM_B_NK = 0, 1


def gemm(a, b, c, alpha, beta, b_layout=GEMM_B_KN):
    """alpha * A @ B + beta * C with B stored [K,N] (b_layout 0) or [N,K] (1); a [..., K] with leading dims
    flattened (reference: gemm/op.cuh:284-297, refs.py:49-51); fp64 sums; returns float32 [M, N], unrounded."""
    a, b = _f32(a), _f32(b)
    K = a.shape[-1]
    a2 = np.ascontiguousarray(a.reshape(-1, K))
    M = a2.shape[0]
    N = b.shape[1] if b_layout == GEMM_B_KN else b.shape[0]
    c2 = np.ascontiguousarray(_f32(c).reshape(M, N)) if c is not None else None
    out = np.empty((M, N), dtype=np.float32)
    rc = lib().oracle_gemm(ctypes.c_int(b_layout), _ptr(a2), _ptr(b), _ptr(c2) if c2 is not None else None, _ptr(out),
                           *[ctypes.c_int64(x) for x in (M, N, K)], ctypes.c_double(alpha), ctypes.c_double(beta))
    if rc != 0:
        raise ValueError(f"oracle_gemm rc={rc}")
    return out


Q8_0_BLOCK, Q8_0_BLOCK_BYTES = 32, 34


def quant_q8_0(x):
    """Rows of floats [..., k] -> rows of Q8_0 blocks, uint8 [..., k/32*34] (reference:
    csrc/quants/impl.cpp:1169-1193)."""
    x = _f32(x)
    k = x.shape[-1]
    y = np.empty(x.shape[:-1] + (k // 32 * 34,), dtype=np.uint8)
    rc = lib().oracle_quant_q8_0(_ptr(x), _ptr(y, ctypes.c_uint8), ctypes.c_int64(x.size // max(k, 1)), ctypes.c_int64(k))
    if rc != 0:
        raise ValueError(f"oracle_quant_q8_0 rc={rc}")
    return y


def dequant_q8_0(y, dtype=np.float32):
    """Rows of Q8_0 blocks, uint8 [..., nb*34] -> values [..., nb*32] as float32 (q * d) or float16
    ((half)(q * d)) (reference: csrc/quants/impl.cpp:1152-1167, cuda/quants/impls.cuh:121-143)."""
    if hasattr(y, "detach"):
        y = y.detach().to("cpu").numpy()
    y = np.ascontiguousarray(np.asarray(y, dtype=np.uint8))
    nbytes = y.shape[-1]
    if nbytes % 34 != 0:
        raise ValueError("row bytes must be a multiple of 34")
    k = nbytes // 34 * 32
    n_rows = y.size // max(nbytes, 1)
    if np.dtype(dtype) == np.float16:
        out = np.empty(y.shape[:-1] + (k,), dtype=np.uint16)
        rc = lib().oracle_dequant_q8_0_f16(_ptr(y, ctypes.c_uint8), _ptr(out, ctypes.c_uint16), ctypes.c_int64(n_rows), ctypes.c_int64(k))
        out = out.view(np.float16)
    else:
        out = np.empty(y.shape[:-1] + (k,), dtype=np.float32)
        rc = lib().oracle_dequant_q8_0(_ptr(y, ctypes.c_uint8), _ptr(out), ctypes.c_int64(n_rows), ctypes.c_int64(k))
    if rc != 0:
        raise ValueError(f"oracle_dequant_q8_0 rc={rc}")
    return out


def flash_attn_decode_q8_0(q, k_cache_q8, v_cache_q8, ctx_lens):
    """Decode attention over Q8_0 caches (uint8 [B,Hkv,Lmax,D/32*34]): the caches are dequantised to fp16 as
    the reference's device dequantiser does, then attended as fp16 caches are."""
    return flash_attn_decode(q, dequant_q8_0(k_cache_q8, np.float16), dequant_q8_0(v_cache_q8, np.float16), ctx_lens)


_REF = None


def ref_quants():
    """The reference's own quantiser source compiled into oracle/_ref/libref_quants.so (make -C oracle ref), or
    None when that library has not been built.  Returns (quant, dequant_f32, dequant_f16) taking numpy arrays."""
    global _REF
    so = os.path.join(_HERE, "_ref", "libref_quants.so")
    if not os.path.exists(so):
        return None
    if _REF is None:
        L = ctypes.CDLL(so)
        qf = getattr(L, "_ZN6minfer4impl14quant_row_q8_0EPKfPhl")
        d32 = getattr(L, "_ZN6minfer4impl16dequant_row_q8_0IfEEvPKhPT_l")
        d16 = getattr(L, "_ZN6minfer4impl16dequant_row_q8_0IN3c104HalfEEEvPKhPT_l")
        for f in (qf, d32, d16):
            f.restype = None

        def quant(x):
            x = _f32(x)
            k = x.shape[-1]
            y = np.empty(x.shape[:-1] + (k // 32 * 34,), dtype=np.uint8)
            qf(_ptr(x), _ptr(y, ctypes.c_uint8), ctypes.c_int64(x.size))   # rows are whole blocks: one long row
            return y

        def dequant32(y):
            y = np.ascontiguousarray(y, dtype=np.uint8)
            out = np.empty(y.shape[:-1] + (y.shape[-1] // 34 * 32,), dtype=np.float32)
            d32(_ptr(y, ctypes.c_uint8), _ptr(out), ctypes.c_int64(out.size))
            return out

        def dequant16(y):
            y = np.ascontiguousarray(y, dtype=np.uint8)
            out = np.empty(y.shape[:-1] + (y.shape[-1] // 34 * 32,), dtype=np.uint16)
            d16(_ptr(y, ctypes.c_uint8), _ptr(out, ctypes.c_uint16), ctypes.c_int64(out.size))
            return out.view(np.float16)

        _REF = (quant, dequant32, dequant16)
    return _REF


def build_ref():
    """Compile oracle/_ref from the reference's source tree (only where that tree exists)."""
    if os.path.isdir("/root/reference"):
        subprocess.run(["make", "-C", _HERE, "ref"], check=True, stdout=subprocess.DEVNULL)
