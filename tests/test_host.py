"""CPU-only checks of the boundary: the C-ABI library loads and exports what the header declares,
argument validation rejects bad calls before anything is launched, and the Python surface keeps
the reference's names (reference: src/minfer/kernels/__init__.py, torch_ext/ops.py:234-266)."""
import ctypes
import inspect
import re

import pytest
import torch

import capi


def declared_functions():
    text = open(capi.HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(minfer_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert {"minfer_flash_attn", "minfer_flash_attn_decode", "minfer_flash_attn_varlen",
            "minfer_flash_attn_workspace_bytes", "minfer_flash_attn_decode_workspace_bytes",
            "minfer_attn_last_error", "minfer_attn_version"} <= set(names)
    L = capi.lib()
    for n in names:
        assert hasattr(L, n), n
    assert L.minfer_attn_version() >= 1000


def test_workspace_sizes():
    L = capi.lib()
    # one class byte per 64x64 mask tile
    assert L.minfer_flash_attn_workspace_bytes(1, 4096) >= 64 * 64
    assert L.minfer_flash_attn_workspace_bytes(2, 100) >= 2 * 2 * 2
    assert L.minfer_flash_attn_workspace_bytes(1, 32768) >= 512 * 512
    # fp32 partials (D values + max + sum), one per share of at least 256 rows that can overlap a (sequence, head)'s rows
    # (8192/256 + 2 of them), plus one line offset per sequence
    need = L.minfer_flash_attn_decode_workspace_bytes(64, 32, 8192, 128)
    assert 64 * 32 * 34 * 130 * 4 + 65 * 4 <= need <= 2 * 64 * 32 * 34 * 130 * 4
    # never more than 64 partials per row, however long the cache
    assert L.minfer_flash_attn_decode_workspace_bytes(1, 8, 1 << 20, 128) <= 8 * 64 * 130 * 4 + 4096


def _call_prefill(dtype=capi.F16, q=0x1000, k=0x2000, v=0x3000, mask=0x4000, out=0x5000, B=1, Hq=8, Hkv=2,
                  L=64, D=128, st=None, ws=0x6000, ws_bytes=1 << 20):
    st = st or capi.Strides(Hq * L * D, L * D, D, Hkv * L * D, L * D, D, Hq * L * D, L * D, D)
    return capi.lib().minfer_flash_attn(dtype, q, k, v, mask, out, B, Hq, Hkv, L, D, ctypes.byref(st), ws, ws_bytes, None)


def test_validation_rejects_before_launch():
    """Every case must be refused on the host: the pointers are fake, so a launch would fault."""
    assert _call_prefill(dtype=7) == capi.EINVAL and "dtype" in capi.last_error()
    assert _call_prefill(D=96) == capi.EINVAL and "head_dim" in capi.last_error()
    assert _call_prefill(Hq=6, Hkv=4) == capi.EINVAL
    assert _call_prefill(q=0) == capi.EINVAL
    assert _call_prefill(k=0x2004) == capi.EINVAL and "aligned" in capi.last_error()
    assert _call_prefill(st=capi.Strides(1, 1, 130, 1, 1, 128, 1, 1, 128)) == capi.EINVAL and "strides" in capi.last_error()
    assert _call_prefill(mask=0) == capi.EINVAL
    assert _call_prefill(ws=0) == capi.EWORKSPACE
    assert _call_prefill(ws_bytes=0) == capi.EWORKSPACE and "workspace" in capi.last_error()
    assert _call_prefill(L=1 << 20) == capi.EINVAL
    # a K/V row stride the tile copies' 32-bit lane offsets cannot span
    assert _call_prefill(st=capi.Strides(8 * 64 * 128, 64 * 128, 128, 2 << 31, 1 << 31, 1 << 25, 8 * 64 * 128, 64 * 128, 128)) == capi.EINVAL \
        and "row stride" in capi.last_error()
    # empty problems are accepted and launch nothing
    assert _call_prefill(B=0) == capi.OK and capi.last_error() == ""
    assert _call_prefill(L=0) == capi.OK

    L = capi.lib()
    st = capi.Strides(1024, 128, 128, 1024, 128, 128, 1024, 128, 128)
    assert L.minfer_flash_attn_decode(capi.F16, 0x1000, 0x2000, 0x3000, None, 0x5000, 1, 8, 2, 64, 128,
                                      ctypes.byref(st), 0x6000, 1 << 20, None) == capi.EINVAL
    assert L.minfer_flash_attn_decode(capi.F16, 0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 1, 8, 2, 64, 128,
                                      ctypes.byref(st), 0x6000, 16, None) == capi.EWORKSPACE
    assert L.minfer_flash_attn_decode(capi.F16, 0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 0, 8, 2, 64, 128,
                                      ctypes.byref(st), 0x6000, 1 << 20, None) == capi.OK
    assert L.minfer_flash_attn_varlen(capi.BF16, 0x1000, 0x2000, 0x3000, None, 2, 64, 0x5000, 8, 2, 64, 128,
                                      ctypes.byref(st), None) == capi.EINVAL
    assert L.minfer_flash_attn_varlen(capi.BF16, 0x1000, 0x2000, 0x3000, 0x4000, 0, 64, 0x5000, 8, 2, 64, 128,
                                      ctypes.byref(st), None) == capi.OK
    big = capi.Strides(1024, 128, 128, 1 << 32, 1 << 31, 1 << 25, 1024, 128, 128)
    assert L.minfer_flash_attn_varlen(capi.BF16, 0x1000, 0x2000, 0x3000, 0x4000, 2, 64, 0x5000, 8, 2, 64, 128,
                                      ctypes.byref(big), None) == capi.EINVAL and "row stride" in capi.last_error()
    # the allocation-free decode refuses, on the host, a problem its built-in scratch array cannot hold
    assert L.minfer_flash_attn_decode_workspace_bytes(256, 64, 8192, 128) > capi.DECODE_NOALLOC_SCRATCH_BYTES
    assert L.minfer_flash_attn_decode_noalloc(capi.F16, 0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 256, 64, 8, 8192, 128,
                                              ctypes.byref(st), None) == capi.EWORKSPACE and "scratch" in capi.last_error()
    assert L.minfer_flash_attn_decode_noalloc(capi.F16, 0x1000, 0x2000, 0x3000, None, 0x5000, 1, 8, 2, 64, 128,
                                              ctypes.byref(st), None) == capi.EINVAL
    # an empty cache (Lmax = 0) is a valid call: the size the library asks for is the size it accepts
    need0 = L.minfer_flash_attn_decode_workspace_bytes(2, 8, 0, 128)
    assert need0 >= 2 * 8 * 130 * 4
    assert L.minfer_flash_attn_decode(capi.F16, 0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 2, 8, 2, 0, 128,
                                      ctypes.byref(st), 0x6000, need0 - 256, None) == capi.EWORKSPACE


def test_rope_validation_rejects_before_launch():
    """Fake pointers again: every call must be refused (or be an accepted empty problem) on the host."""
    L = capi.lib()
    rope = lambda dtype=capi.F16, style=0, x=0x1000, B=1, Ln=4, H=2, D=128, rd=64, start=0, base=1e4: \
        L.minfer_rope(dtype, style, x, B, Ln, H, D, rd, start, base, None)
    assert rope(dtype=7) == capi.EINVAL and "dtype" in capi.last_error()
    assert rope(style=2) == capi.EINVAL and "style" in capi.last_error()
    assert rope(rd=130) == capi.EINVAL and "rotary_dim" in capi.last_error()
    assert rope(rd=7) == capi.EINVAL and "even" in capi.last_error()
    assert rope(D=512, rd=512) == capi.EINVAL
    assert rope(base=0.0) == capi.EINVAL and "freq_base" in capi.last_error()
    assert rope(x=0) == capi.EINVAL
    assert rope(start=-1) == capi.EINVAL
    assert rope(start=1 << 31) == capi.EINVAL
    assert rope(B=0) == capi.OK and rope(rd=0) == capi.OK and capi.last_error() == ""

    app = lambda q=0x1000, k=0x2000, v=0x3000, pos=0x4000, kc=0x5000, vc=0x6000, B=1, Ln=4, Hq=4, Hkv=2, D=128, \
        Lmax=16, s=(4096, 2048, 128), rd=64, style=0: \
        L.minfer_rope_kv_append(capi.F16, style, q, k, v, pos, kc, vc, B, Ln, Hq, Hkv, D, Lmax, *s, rd, 1e4, None)
    assert app(pos=0) == capi.EINVAL and "null" in capi.last_error()
    assert app(kc=0x5008) == capi.EINVAL and "aligned" in capi.last_error()
    assert app(s=(4096, 2048, 100)) == capi.EINVAL and "strides" in capi.last_error()
    assert app(D=100, rd=64) == capi.EINVAL
    assert app(rd=24, style=1) == capi.EINVAL          # NeoX halves must be whole 16-byte chunks
    assert app(Hkv=0) == capi.EINVAL
    assert app(B=0) == capi.OK and app(Ln=0) == capi.OK


def test_rmsnorm_validation_rejects_before_launch():
    L = capi.lib()
    norm = lambda dtype=capi.F16, x=0x1000, w=0x2000, out=0x3000, n=4, dim=128, eps=1e-6: \
        L.minfer_rmsnorm(dtype, x, w, out, n, dim, eps, None)
    assert norm(dtype=3) == capi.EINVAL and "dtype" in capi.last_error()
    assert norm(dim=0) == capi.EINVAL
    assert norm(n=-1) == capi.EINVAL
    assert norm(eps=-1.0) == capi.EINVAL and "eps" in capi.last_error()
    assert norm(w=0) == capi.EINVAL and "null" in capi.last_error()
    assert norm(n=0) == capi.OK and capi.last_error() == ""


def test_gemm_validation_rejects_before_launch():
    L = capi.lib()
    gemm = lambda dtype=capi.F16, layout=0, a=0x1000, b=0x2000, c=0x3000, d=0x4000, M=64, N=64, K=64, lda=64, ldb=64, \
        ldc=64, ldd=64, alpha=1.0, beta=1.0: L.minfer_gemm(dtype, layout, a, b, c, d, M, N, K, lda, ldb, ldc, ldd, alpha, beta, None)
    assert gemm(dtype=2) == capi.EINVAL and "dtype" in capi.last_error()
    assert gemm(layout=2) == capi.EINVAL and "b_layout" in capi.last_error()
    assert gemm(M=-1) == capi.EINVAL
    assert gemm(a=0) == capi.EINVAL and "null" in capi.last_error()
    assert gemm(c=0) == capi.EINVAL                      # beta != 0 needs C
    assert gemm(lda=32) == capi.EINVAL and "leading" in capi.last_error()
    assert gemm(N=128, ldd=64) == capi.EINVAL
    assert gemm(M=0) == capi.OK and gemm(N=0) == capi.OK and capi.last_error() == ""
    # the entry point with a workspace checks the same things first
    gemm_ws = lambda dtype=capi.F16, layout=0, a=0x1000, b=0x2000, d=0x4000, M=64, N=4096, K=4096, lda=4096, ldd=4096: \
        L.minfer_gemm_ws(dtype, layout, a, b, None, d, M, N, K, lda, N, N, ldd, 1.0, 0.0, 0x10000, 1 << 30, None)
    assert gemm_ws(dtype=2) == capi.EINVAL and "dtype" in capi.last_error()
    assert gemm_ws(a=0) == capi.EINVAL and gemm_ws(lda=64) == capi.EINVAL and gemm_ws(ldd=64) == capi.EINVAL
    assert gemm_ws(M=0) == capi.OK


def test_gemm_q8_0_validation_rejects_before_launch():
    L = capi.lib()
    g = lambda a=0x1000, b=0x2000, c=None, d=0x4000, M=4, N=64, K=256, lda=256, ldc=64, ldd=64, alpha=1.0, beta=0.0, ws=None, wsb=0: \
        L.minfer_gemm_q8_0(a, b, c, d, M, N, K, lda, ldc, ldd, alpha, beta, ws, wsb, None)
    assert g(K=100) == capi.EINVAL and "multiple of the block size" in capi.last_error()
    assert g(a=0) == capi.EINVAL and "null" in capi.last_error()
    assert g(beta=1.0) == capi.EINVAL                                  # beta != 0 needs C
    assert g(lda=128) == capi.EINVAL and "leading" in capi.last_error()
    assert g(b=0x2002) == capi.EINVAL and "4-byte" in capi.last_error()
    # operands the streaming kernel cannot take (A off a 16-byte boundary, N not a multiple of 4) go through the
    # dequantised weight, i.e. ask for the workspace instead of being refused
    assert g(a=0x1008) == capi.EWORKSPACE and "not aligned" in capi.last_error()
    assert g(N=18, ldc=18, ldd=18) == capi.EWORKSPACE
    assert g(M=100) == capi.EWORKSPACE and "workspace" in capi.last_error()   # more than 64 rows: needs the dequantised weight
    assert g(K=96, lda=96) == capi.EWORKSPACE                               # an odd number of blocks per row as well
    assert g(M=0) == capi.OK and g(N=0) == capi.OK and capi.last_error() == ""
    ws = L.minfer_gemm_q8_0_workspace_bytes
    assert ws(1, 4096, 4096) == 0 and ws(64, 14336, 4096) == 0
    assert ws(65, 4096, 4096) == 4096 * 4096 * 2 + L.minfer_gemm_workspace_bytes(65, 4096, 4096)
    assert ws(4, 64, 96) == (64 * 96 * 2 + 255) // 256 * 256 and ws(4, 64, 100) == 0 and ws(0, 64, 128) == 0
    assert ws(4, 18, 256) == (18 * 256 * 2 + 255) // 256 * 256      # N not a multiple of 4: the query and the call agree


def test_gemm_workspace_sizes():
    L = capi.lib()
    ws = L.minfer_gemm_workspace_bytes
    assert ws(64, 4096, 4096) == 8 * 64 * 4096 * 4            # 32 tiles of 128 x 128: 8 slices of 8 steps
    assert ws(256, 4096, 4096) == 4 * 256 * 4096 * 4          # 64 tiles: 4 slices
    assert ws(100, 14336, 4096) == 4 * 100 * 14336 * 4        # 112 tiles: 2 slices fill the chip once, 4 of 16 steps each are taken
    assert ws(4096, 4096, 4096) == 0 and ws(64, 4096, 256) == 0 and ws(64, 4096, 100) == 0 and ws(64, 4100, 4096) == 0
    assert ws(0, 4096, 4096) == 0 and ws(-1, 4096, 4096) == 0 and ws(64, 4096, 1 << 40) == 0


def test_q8_0_validation_rejects_before_launch():
    L = capi.lib()
    quant = lambda dtype=capi.F32, x=0x1000, y=0x2000, n=4, k=128: L.minfer_quant_q8_0(dtype, x, y, n, k, None)
    assert quant(dtype=8) == capi.EINVAL and "dtype" in capi.last_error()
    assert quant(k=100) == capi.EINVAL and "multiple of 32" in capi.last_error()
    assert quant(x=0) == capi.EINVAL and "null" in capi.last_error()
    assert quant(x=0x1004) == capi.EINVAL and quant(y=0x2001) == capi.EINVAL and quant(n=-1) == capi.EINVAL
    assert quant(n=0) == capi.OK and quant(k=0) == capi.OK and capi.last_error() == ""
    dequant = lambda dtype=capi.F16, x=0x1000, y=0x2000, n=4, k=128: L.minfer_dequant_q8_0(dtype, x, y, n, k, None)
    assert dequant(dtype=capi.BF16) == capi.EINVAL and "dtype" in capi.last_error()   # the reference dequantises to float or half
    assert dequant(k=31) == capi.EINVAL and dequant(y=0x2002) == capi.EINVAL and dequant(x=0x1001) == capi.EINVAL
    assert dequant(n=0) == capi.OK

    def dec(B=2, Hq=8, Hkv=2, Lmax=64, D=128, q=0x1000, k=0x2000, v=0x3000, ctx=0x4000, out=0x5000, ws=0x6000, ws_bytes=None, **st):
        s = dict(q0=Hq * D, q1=D, q2=D, kv0=Hkv * Lmax * (D // 32 * 34), kv1=Lmax * (D // 32 * 34), kv2=D // 32 * 34,
                 o0=Hq * D, o1=D, o2=D)
        s.update(st)
        need = L.minfer_flash_attn_decode_workspace_bytes(B, Hq, Lmax, D)
        return L.minfer_flash_attn_decode_q8_0(q, k, v, ctx, out, B, Hq, Hkv, Lmax, D, ctypes.byref(capi.Strides(**s)), ws,
                                               need if ws_bytes is None else ws_bytes, None)
    assert dec(D=96) == capi.EINVAL and "head_dim" in capi.last_error()
    assert dec(Hq=7) == capi.EINVAL
    assert dec(k=0x2001) == capi.EINVAL and "2-byte" in capi.last_error()
    assert dec(kv2=256) == capi.EINVAL and "dense" in capi.last_error()
    assert dec(kv1=64 * 136 + 1) == capi.EINVAL and "even" in capi.last_error()
    assert dec(ctx=0) == capi.EINVAL and dec(q=0x1008) == capi.EINVAL
    assert dec(ws_bytes=16) == capi.EWORKSPACE
    assert dec(B=0) == capi.OK and capi.last_error() == ""

    def app(dtype=capi.F16, style=0, q=0x1000, k=0x2000, v=0x3000, pos=0x4000, kc=0x5000, vc=0x6000, B=1, Ln=4, Hq=8, Hkv=2, D=128,
            Lmax=16, c0=None, c1=None, rd=128, base=1e4):
        row = D // 32 * 34
        return L.minfer_rope_kv_append_q8_0(dtype, style, q, k, v, pos, kc, vc, B, Ln, Hq, Hkv, D, Lmax,
                                            Hkv * Lmax * row if c0 is None else c0, Lmax * row if c1 is None else c1, rd, base, None)
    assert app(D=80, rd=0) == capi.EINVAL and "multiple of 32" in capi.last_error()
    assert app(rd=48) == capi.EINVAL                      # a block must not straddle the rotary part's end
    assert app(rd=96, style=1) == capi.EINVAL             # NeoX halves must be whole blocks
    assert app(kc=0x5001) == capi.EINVAL and app(c1=137) == capi.EINVAL and app(pos=0) == capi.EINVAL
    assert app(dtype=capi.F32) == capi.EINVAL
    assert app(B=0) == capi.OK and app(Ln=0) == capi.OK


def test_calibration_validation_rejects_before_launch():
    L = capi.lib()
    i64 = ctypes.c_int64
    for fn in (L.minfer_calib_mfma_rate, L.minfer_calib_mfma_rate_32x32x16):
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.c_int, ctypes.c_void_p, i64, i64, ctypes.c_void_p, ctypes.c_void_p]
        assert fn(7, 0x1000, 10, 1, 0x2000, None) == capi.EINVAL and "dtype" in capi.last_error()
        assert fn(capi.F16, 0x1008, 10, 1, 0x2000, None) == capi.EINVAL and "aligned" in capi.last_error()
        assert fn(capi.F16, 0x1000, -1, 1, 0x2000, None) == capi.EINVAL and "iters" in capi.last_error()
        assert fn(capi.F16, 0x1000, 10, 0, 0x2000, None) == capi.EINVAL
        assert fn(capi.F16, 0x1000, 10, 1, None, None) == capi.EINVAL
    mix = L.minfer_calib_attn_mix
    mix.restype = ctypes.c_int
    mix.argtypes = [ctypes.c_int, ctypes.c_void_p, i64, i64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    assert mix(7, 0x1000, 10, 1, 1, 1, 0x2000, None) == capi.EINVAL and "dtype" in capi.last_error()
    assert mix(capi.BF16, None, 10, 1, 1, 1, 0x2000, None) == capi.EINVAL


def test_python_surface_matches_reference_names(kerns):
    from minfer.const import GGML_QUANT_SIZES, GGMLQuantizationType
    from minfer.kernels import KernelBackend, refs
    import minfer.kernels.torch_ext as te
    import oracle

    assert GGMLQuantizationType.F16 == 1 and GGML_QUANT_SIZES[GGMLQuantizationType.F16] == (1, 2)
    # the reference's table value for BF16 (reference: src/minfer/const.py:67), kept for callers that compare tables
    assert GGMLQuantizationType.BF16 == 30 and GGML_QUANT_SIZES[GGMLQuantizationType.BF16] == (256, 512)
    assert list(inspect.signature(te.flash_attn).parameters) == [
        "qtype_int", "qblock_size", "qtype_size", "q", "k", "v", "mask", "out"]
    assert callable(kerns.flash_attn) and callable(kerns.flash_attn_decode) and callable(kerns.flash_attn_varlen)
    with pytest.raises(ValueError):
        KernelBackend("triton")
    schema = str(torch.ops.minfer.flash_attn.default._schema)
    assert schema == ("minfer::flash_attn(int qtype_int, int qblock_size, int qtype_size, Tensor q, Tensor k, "
                      "Tensor v, Tensor(a!) mask, Tensor(a!) out) -> ()")
    # rotary embedding: names, argument order and schemas of the reference (torch_ext/ops.py:86-126, reg.cpp:25-26)
    for name in ("il_rope", "neox_rope"):
        assert list(inspect.signature(getattr(te, name)).parameters) == ["rotary_dim", "start_pos", "freq_base", "x"]
        assert callable(getattr(kerns, name))
        assert str(getattr(torch.ops.minfer, name).default._schema) == \
            f"minfer::{name}(int rotary_dim, int start_pos, float freq_base, Tensor(a!) x) -> ()"
    assert callable(kerns.rope_kv_append)
    # the quantisers: private names, argument order and schemas of the reference (kernels/__init__.py:5-7,
    # torch_ext/ops.py:8-46, reg.cpp:22-23); Q8_0 numbered and sized as there (const.py:11, :46)
    assert GGMLQuantizationType.Q8_0 == 8 and GGML_QUANT_SIZES[GGMLQuantizationType.Q8_0] == (32, 34)
    for name in ("dequant", "quant"):
        assert callable(getattr(kerns, "_" + name)) and getattr(te, "_" + name) is getattr(kerns, "_" + name)
        assert list(inspect.signature(getattr(kerns, "_" + name)).parameters) == ["qtype", "qblock_size", "qtype_size", "x", "y"]
        assert str(getattr(torch.ops.minfer, name).default._schema) == \
            f"minfer::{name}(int qtype, int qblock_size, int qtype_size, Tensor x, Tensor(a!) y) -> ()"
    assert list(inspect.signature(te.gemm).parameters) == ["qtype_int", "qblock_size", "qtype_size", "alpha", "beta", "A", "B", "C", "D"]
    assert str(torch.ops.minfer.gemm.default._schema) == ("minfer::gemm(int qtype_int, int qblock_size, int qtype_size, float alpha, "
                                                          "float beta, Tensor A, Tensor B, Tensor C, Tensor(a!) out) -> ()")
    assert list(inspect.signature(te.qkv).parameters)[9:] == ["x", "wq", "wk", "wv", "q_out", "k_out", "v_out"]
    assert str(torch.ops.minfer.qkv.default._schema).endswith("Tensor x, Tensor wq, Tensor wk, Tensor wv, Tensor(a!) q_out, "
                                                              "Tensor(a!) k_out, Tensor(a!) v_out) -> ()")
    assert callable(kerns.gemm) and callable(kerns.qkv)
    ga, gw, gb = torch.randn(5, 7), torch.randn(7, 3), torch.randn(5, 3)
    go = torch.empty(5, 3)
    refs.gemm(ga, gw, gb, go, 2.0, 3.0)
    assert float((go - torch.from_numpy(oracle.gemm(ga, gw, gb, 2.0, 3.0))).abs().max()) < 1e-5
    assert list(inspect.signature(te.rmsnorm).parameters) == ["eps", "input", "w", "out"] and callable(kerns.rmsnorm)
    assert str(torch.ops.minfer.rmsnorm.default._schema) == "minfer::rmsnorm(float eps, Tensor input, Tensor w, Tensor(a!) out) -> ()"
    xn, wn = torch.randn(2, 3, 16), torch.randn(16)
    assert float((refs.rmsnorm(xn, wn, 1e-6) - torch.from_numpy(oracle.rmsnorm(xn, wn, 1e-6))).abs().max()) < 1e-5
    x = torch.randn(2, 5, 3, 16).half()
    for style, ref in ((0, refs.il_rope), (1, refs.neox_rope)):
        assert ref(x, 8, 3, 1e4).dtype == torch.float16
        assert float((ref(x, 8, 3, 1e4).float() - torch.from_numpy(oracle.rope(style, x, 8, 3, 1e4))).abs().max()) < 4e-3
    q = torch.randn(1, 2, 4, 8)
    m = torch.ones(1, 1, 4, 4, dtype=torch.bool).tril()
    assert torch.equal(refs.flash_attn(q, q, q, m), torch.nn.functional.scaled_dot_product_attention(q, q, q, attn_mask=m))


def test_no_cpu_fallback(kerns):
    """CPU tensors must fail loudly: there is no CPU implementation behind the ops."""
    q = torch.zeros(1, 2, 64, 128, dtype=torch.float16)
    mask = torch.ones(1, 1, 64, 64, dtype=torch.bool)
    with pytest.raises((NotImplementedError, RuntimeError)):
        kerns.flash_attn(1, 1, 2, q, q, q, mask, torch.empty_like(q))
    with pytest.raises((NotImplementedError, RuntimeError)):
        kerns.flash_attn_decode(1, 1, 2, q[:, :, :1], q, q, torch.ones(1, dtype=torch.int32), torch.empty_like(q[:, :, :1]))
    with pytest.raises((NotImplementedError, RuntimeError)):
        kerns.flash_attn_varlen(1, 1, 2, q, q, q, torch.tensor([0, 64], dtype=torch.int32), 64, torch.empty_like(q))
    x = torch.zeros(1, 4, 2, 128, dtype=torch.float16)
    with pytest.raises((NotImplementedError, RuntimeError)):
        kerns.rmsnorm(1e-6, x, torch.ones(128, dtype=torch.float16), torch.empty_like(x))
    h = torch.zeros(1, 4, 64, dtype=torch.float16)
    with pytest.raises((NotImplementedError, RuntimeError)):
        kerns.gemm(1, 1, 2, 1.0, 0.0, h, torch.zeros(64, 64, dtype=torch.float16), h, torch.empty_like(h))
    with pytest.raises((NotImplementedError, RuntimeError)):
        kerns.qkv(1, 1, 1, 1, 1, 1, 2, 2, 2, h, *[torch.zeros(64, 64, dtype=torch.float16)] * 3, *[torch.empty_like(h) for _ in range(3)])
    with pytest.raises((NotImplementedError, RuntimeError)):
        kerns._quant(8, 32, 34, torch.zeros(2, 64), torch.zeros(2, 68, dtype=torch.uint8))
    with pytest.raises((NotImplementedError, RuntimeError)):
        kerns._dequant(8, 32, 34, torch.zeros(2, 68, dtype=torch.uint8), torch.zeros(2, 64))
    with pytest.raises((NotImplementedError, RuntimeError)):
        kerns.flash_attn_decode(8, 32, 34, q[:, :, :1], torch.zeros(1, 2, 64, 136, dtype=torch.uint8), torch.zeros(1, 2, 64, 136, dtype=torch.uint8),
                                torch.ones(1, dtype=torch.int32), torch.empty_like(q[:, :, :1]))
    with pytest.raises((NotImplementedError, RuntimeError)):
        kerns.il_rope(64, 0, 1e4, x)
    with pytest.raises((NotImplementedError, RuntimeError)):
        kerns.neox_rope(64, 0, 1e4, x)
    with pytest.raises((NotImplementedError, RuntimeError)):
        kerns.rope_kv_append(0, 64, 1e4, x, x, x, torch.zeros(1, dtype=torch.int32), torch.zeros(1, 2, 8, 128).half(),
                             torch.zeros(1, 2, 8, 128).half())


def test_workload_generators_are_seeded():
    import workloads
    a = workloads.llama8b_prefill(seed=3, L=128)
    b = workloads.llama8b_prefill(seed=3, L=128)
    c = workloads.llama8b_prefill(seed=4, L=128)
    assert all(torch.equal(x, y) for x, y in zip(a, b)) and not torch.equal(a[0], c[0])
    qv = workloads.llama8b_prefill(seed=3, L=128, views=True)[0]
    assert qv.shape == (1, 32, 128, 128) and qv.stride() == (128 * 32 * 128, 128, 32 * 128, 1)
    q, k, v, cu = workloads.ragged_prefill(seed=0)
    lens = (cu[1:] - cu[:-1]).tolist()
    assert len(lens) == 16 and min(lens) >= 128 and max(lens) <= 2048 and q.shape == (1, 64, int(cu[-1]), 128)
    assert workloads.prefill_flops(32, 128, [4096]) == 2 * 128 * 32 * 4096 * 4097
    assert workloads.decode_bytes([10, 20], 32, 8, 128) == 30 * 4096 + 2 * 2 * 32 * 128 * 2
    ga, gw, gb = workloads.gemm_input(8, 16, 32, seed=2)
    assert ga.shape == (1, 8, 32) and gw.shape == (32, 16) and gb.shape == (1, 8, 16) and workloads.gemm_flops(8, 16, 32) == 8192
    xs, ws = workloads.rmsnorm_input((2, 3, 64), seed=5)
    assert xs.shape == (2, 3, 64) and ws.shape == (64,) and torch.equal(xs, workloads.rmsnorm_input((2, 3, 64), seed=5)[0])
    assert workloads.rmsnorm_bytes((2, 3, 64)) == (2 * 384 + 64) * 2
    x = workloads.rope_input(seed=1, B=1, L=8)
    assert x.shape == (1, 8, 48, 128) and torch.equal(x, workloads.rope_input(seed=1, B=1, L=8))
    assert workloads.rope_bytes(8, 4096, 48, 64) == 2 * 8 * 4096 * 48 * 64 * 2
    q, k, v, pos, kc, vc = workloads.kv_append(seed=0, L=16)
    assert q.shape == (1, 16, 32, 128) and k.shape == v.shape == (1, 16, 8, 128) and kc.shape == (1, 8, 16, 128)
    assert workloads.kv_append_bytes(1, 16, 32, 8, 128, 128) == (2 * 16 * 32 * 128 + 4 * 16 * 8 * 128) * 2
    assert workloads.kv_append_bytes_q8_0(1, 16, 32, 8, 128, 128) == 16 * (2 * 32 * 128 * 2 + 2 * 8 * 128 * 2 + 2 * 8 * 136)
    assert workloads.decode_bytes_q8_0([10, 20], 32, 8, 128) == 30 * 8 * 136 * 2 + 2 * 2 * 32 * 128 * 2


def test_build_scan_finds_dependences_too_close_to_an_asm_statement():
    """build.py scans the generated device code for the two distances the compiler cannot keep when one end lies inside
    an asm statement; the scan itself is checked here on small pieces of assembly text."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("minfer_build", f"{capi.ROOT}/minfer-python_amd/build.py")
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    copy = lambda nop: f"\t;;#ASMSTART\n\ts_mov_b32 m0, s2\n\ts_nop {nop}\n\tglobal_load_lds_dwordx4 v16, s[24:25]\n\t;;#ASMEND\n"
    head = "kernel_a:\n\tv_readfirstlane_b32 s25, v11\n\tv_readfirstlane_b32 s24, v10\n"
    assert len(build.asm_hazards(head + copy(0))) == 2                       # two issue slots between: too close
    assert build.asm_hazards(head + copy(3)) == []                          # s_mov + s_nop 3 = five slots
    assert build.asm_hazards(head + "\tv_add_u32_e32 v1, v2, v3\n" * 3 + copy(0)) == []
    assert build.asm_hazards(head.replace("s24", "s30").replace("s25", "s31") + copy(0)) == []   # other registers
    assert build.asm_hazards(head + ".LBB0_1:\n" + copy(0)) != []           # a branch target does not reset the distance
    cvt = "\t;;#ASMSTART\n\tv_cvt_f16_i16_sdwa v51, sext(v68) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_3\n\t;;#ASMEND\n"
    mfma = "\tv_mfma_f32_16x16x32_f16 v[26:29], v[50:53], v[58:61], v[26:29]\n"
    assert len(build.asm_hazards("kernel_b:\n" + cvt + "\tv_pk_mul_f16 v63, v63, v136\n" + mfma)) == 1
    assert build.asm_hazards("kernel_b:\n" + cvt + "\tv_pk_mul_f16 v63, v63, v136\n" * 2 + mfma) == []
    assert build.asm_hazards("kernel_b:\n" + cvt.replace("v51", "v70") + mfma) == []
