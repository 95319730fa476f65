"""Kernel facade, same shape as the reference's (reference: src/minfer/kernels/__init__.py:2-18):
an attribute bag of callables for one backend.  Only the attention path, the normalisation,
projection and rotary-embedding steps that feed it, and the Q8_0 quantisers of its KV cache live here."""


class KernelBackend:
    def __init__(self, backend: str):
        if backend == "torch_ext":
            from .torch_ext import (_dequant, _quant, flash_attn, flash_attn_decode, flash_attn_varlen, gemm, il_rope,
                                    neox_rope, qkv, rmsnorm, rope_kv_append, rope_kv_append_norm)
            self._dequant = _dequant
            self._quant = _quant
            self.rmsnorm = rmsnorm
            self.gemm = gemm
            self.qkv = qkv
            self.il_rope = il_rope
            self.neox_rope = neox_rope
            self.rope_kv_append = rope_kv_append
            self.rope_kv_append_norm = rope_kv_append_norm
            self.flash_attn = flash_attn
            self.flash_attn_decode = flash_attn_decode
            self.flash_attn_varlen = flash_attn_varlen
        else:
            raise ValueError(f"KernelBackend init: unsupported backend {backend}")
