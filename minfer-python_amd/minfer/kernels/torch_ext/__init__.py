# Importing _C loads the shared object, whose static initialisers register the minfer::* ops
# (reference: src/minfer/kernels/torch_ext/__init__.py:1).  There is no fallback: without the
# built extension this import fails.
try:
    from . import _C  # noqa: F401
except ImportError as e:  # pragma: no cover
    raise ImportError(
        "minfer.kernels.torch_ext._C is not built; run `python minfer-python_amd/build.py` "
        "(hipcc, gfx950) first"
    ) from e
from .ops import (flash_attn, flash_attn_decode, flash_attn_varlen, gemm, il_rope, neox_rope,  # noqa: E402,F401
                  qkv, rmsnorm, rope_kv_append, rope_kv_append_norm)
from .ops import dequant as _dequant, quant as _quant  # noqa: E402,F401  (reference: torch_ext/__init__.py:2)
