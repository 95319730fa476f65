"""Element-type identifiers the attention operators are called with.

Callers pass ``qtype, *GGML_QUANT_SIZES[qtype]`` as the three leading integers of every op
(reference: test/kernels.py:226-227, apps/benchmark.py:216-217).  The numbering is GGML's
(reference: src/minfer/const.py:4-35).  Only the types an attention activation can have and the one
block format a KV cache may be kept in (Q8_0) are listed; the other quantised weight formats of the
reference belong to its dequant/gemm ops.
"""
from enum import IntEnum


class GGMLQuantizationType(IntEnum):
    F32 = 0
    F16 = 1
    Q8_0 = 8
    BF16 = 30


# (elements per block, bytes per block); reference: src/minfer/const.py:39-41.  BF16 is (256, 512) as in
# the reference's table (const.py:67): the same two bytes per element; the operators ignore the pair for
# 16-bit types.
GGML_QUANT_SIZES: dict[GGMLQuantizationType, tuple[int, int]] = {
    GGMLQuantizationType.F32: (1, 4),
    GGMLQuantizationType.F16: (1, 2),
    GGMLQuantizationType.Q8_0: (32, 2 + 32),   # reference: src/minfer/const.py:46
    GGMLQuantizationType.BF16: (256, 512),
}
