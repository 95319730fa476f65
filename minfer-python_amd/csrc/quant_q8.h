// Device helpers for the Q8_0 block format: 32 values as an fp16 scale d followed by 32 int8, 34 bytes, so
// blocks start on 2-byte boundaries only (reference: src/minfer/kernels/torch_ext/csrc/common/types.hpp:141-146).
#pragma once

#include "attn_common.h"

namespace minfer_attn {

// One Q8_0 block as a lane holds it: the 32 int8 in eight words, the scale's fp16 bits.
struct Q8Block { uint4 lo, hi; uint32_t d; };

// (half)(q * d) for the four int8 of a word (reference: cuda/quants/impls.cuh:121-143): q + 1152 is built
// exactly by placing (q ^ 0x80) under the exponent of 1024, the subtraction is exact, and the packed
// multiply rounds the exact product once, as the conversion of the fp32 product does.
MA_DEV void dequant4(uint32_t w, h16x2 d2, uint32_t& out_lo, uint32_t& out_hi) {
    const uint32_t x = w ^ 0x80808080u;
    const h16x2 bias = {(_Float16)1152.f, (_Float16)1152.f};
    const h16x2 a = __builtin_bit_cast(h16x2, __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u));
    const h16x2 b = __builtin_bit_cast(h16x2, __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u));
    out_lo = __builtin_bit_cast(uint32_t, (a - bias) * d2);
    out_hi = __builtin_bit_cast(uint32_t, (b - bias) * d2);
}
// the 8 fp16 values of words w0, w1 of a block
MA_DEV s16x8 dequant8(uint32_t w0, uint32_t w1, h16x2 d2) {
    uint4 u;
    dequant4(w0, d2, u.x, u.y);
    dequant4(w1, d2, u.z, u.w);
    return __builtin_bit_cast(s16x8, u);
}

// The same from a block that is only 2-byte aligned, read as aligned words: `lo`, `hi` are consecutive words of
// memory and the four int8 wanted start at byte 2 of `lo` (block on a 4-byte boundary: sel_a, sel_b =
// kQ8SelEvenA, kQ8SelEvenB) or are `hi` itself (block 2 bytes past one: kQ8SelOddA, kQ8SelOddB).  The byte
// permute that spreads the quants under the exponent bytes does the shift on the way.
constexpr uint32_t kQ8SelEvenA = 0x0c030c02u, kQ8SelEvenB = 0x0c050c04u, kQ8SelOddA = 0x0c050c04u, kQ8SelOddB = 0x0c070c06u;
MA_DEV void dequant4_shifted(uint32_t lo, uint32_t hi, uint32_t sel_a, uint32_t sel_b, h16x2 d2, uint32_t& out_lo, uint32_t& out_hi) {
    const h16x2 bias = {(_Float16)1152.f, (_Float16)1152.f};
    // selector 0x0c yields a zero byte; (q ^ 0x80) | 0x6400 in each half is one exclusive or
    const h16x2 a = __builtin_bit_cast(h16x2, __builtin_amdgcn_perm(hi, lo, sel_a) ^ 0x64806480u);
    const h16x2 b = __builtin_bit_cast(h16x2, __builtin_amdgcn_perm(hi, lo, sel_b) ^ 0x64806480u);
    out_lo = __builtin_bit_cast(uint32_t, (a - bias) * d2);
    out_hi = __builtin_bit_cast(uint32_t, (b - bias) * d2);
}
// the 8 fp16 values of quant words j, j+1 of such a block, given memory words w[j], w[j+1], w[j+2]
MA_DEV s16x8 dequant8_shifted(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t sel_a, uint32_t sel_b, h16x2 d2) {
    uint4 u;
    dequant4_shifted(w0, w1, sel_a, sel_b, d2, u.x, u.y);
    dequant4_shifted(w1, w2, sel_a, sel_b, d2, u.z, u.w);
    return __builtin_bit_cast(s16x8, u);
}

// Quantises the lane's 8 values of a block whose 32 values are spread over the 4 lanes 4i..4i+3 (all four
// must be active): returns the 8 int8, and the block's scale as fp16 bits (reference:
// csrc/quants/impl.cpp:1169-1193; the division, the reciprocal and the product are single IEEE operations
// and roundf rounds ties away from zero, as there).
MA_DEV uint2 quant8_q8_0(const float (&f)[8], uint16_t& d_bits) {
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(f[j]));
    // lanes l ^ 1 and l ^ 2 through quad permutes of the vector ALU (no trip through LDS)
    amax = fmaxf(amax, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, amax), 0xB1, 0xf, 0xf, true)));
    amax = fmaxf(amax, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, amax), 0x4E, 0xf, 0xf, true)));
    const float d = amax / 127.f;
    const float id = d != 0.f ? 1.f / d : 0.f;
    d_bits = __builtin_bit_cast(uint16_t, (_Float16)d);
    uint32_t w[2] = {0u, 0u};
#pragma unroll
    for (int j = 0; j < 8; ++j) w[j >> 2] |= ((uint32_t)(int)roundf(f[j] * id) & 0xffu) << (8 * (j & 3));
    return uint2{w[0], w[1]};
}

// Stores the 8 int8 of values off..off+7 of the block at blk, and the scale from the lane that holds off 0.
MA_DEV void store_q8_piece(char* blk, int off, uint2 q, uint16_t d_bits) {
    char* dst = (char*)__builtin_assume_aligned(blk + 2 + off, 2);
    __builtin_memcpy(dst, &q, 8);
    if (off == 0) __builtin_memcpy(__builtin_assume_aligned(blk, 2), &d_bits, 2);
}

}  // namespace minfer_attn
