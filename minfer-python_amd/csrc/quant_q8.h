// Device helpers for the Q8_0 block format: 32 values as an fp16 scale d followed by 32 int8, 34 bytes, so
// blocks start on 2-byte boundaries only (reference: src/minfer/kernels/torch_ext/csrc/common/types.hpp:141-146).
#pragma once

#include "attn_common.h"

namespace minfer_attn {

// One Q8_0 block as a lane holds it: the 32 int8 in eight words, the scale's fp16 bits.
struct Q8Block { uint4 lo, hi; uint32_t d; };

// The four int8 of a word as fp16, exactly: sub-dword addressing lets the int16 -> fp16 conversion take one byte,
// sign-extended, as its source and one half of the destination as its target, so a value costs one instruction
// (building q + 1152 under the exponent byte of 1024 with a byte permute and an exclusive or, then subtracting, costs 1.5).
// The results must pass through an instruction the compiler emits (the multiply by the scale, here) before a matrix
// instruction reads them: a matrix instruction may read a register two instructions after a vector instruction wrote
// it at the earliest, and the compiler cannot keep that distance for a write it does not see (measured: stale operands).
MA_DEV void int8x4_to_f16(uint32_t w, uint32_t& out_lo, uint32_t& out_hi) {
    asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_0" : "=v"(out_lo) : "v"(w));
    asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_1" : "+v"(out_lo) : "v"(w));
    asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(out_hi) : "v"(w));
    asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_3" : "+v"(out_hi) : "v"(w));
}
// (half)(q * d) for the 8 int8 of two quant words (reference: cuda/quants/impls.cuh:121-143): conversion, then one
// packed multiply per pair, which rounds the exact product once, as the conversion of the fp32 product does.
MA_DEV s16x8 dequant8_words(uint32_t a0, uint32_t a1, h16x2 d2) {
    uint4 u;
    int8x4_to_f16(a0, u.x, u.y);
    int8x4_to_f16(a1, u.z, u.w);
    u.x = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h16x2, u.x) * d2);
    u.y = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h16x2, u.y) * d2);
    u.z = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h16x2, u.z) * d2);
    u.w = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h16x2, u.w) * d2);
    return __builtin_bit_cast(s16x8, u);
}

// The same from a block that is only 2-byte aligned, read as aligned words w0, w1, w2 of memory: quant word j of the
// block is bytes 2..5 of {w[j+1], w[j]} when the block starts on a 4-byte boundary (kQ8SelEven) and w[j+1] itself when
// it starts 2 bytes past one (kQ8SelOdd); one byte permute per word, its selector a per-lane constant, does the shift.
constexpr uint32_t kQ8SelEven = 0x05040302u, kQ8SelOdd = 0x07060504u;
MA_DEV s16x8 dequant8_shifted(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t sel, h16x2 d2) {
    return dequant8_words(__builtin_amdgcn_perm(w1, w0, sel), __builtin_amdgcn_perm(w2, w1, sel), d2);
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
