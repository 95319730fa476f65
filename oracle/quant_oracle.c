/*
 * TEST INFRASTRUCTURE ONLY: CPU restatement of the reference's Q8_0 block quantiser and dequantiser.
 * Nothing that ships links or calls this file.
 *
 * Block layout (reference: src/minfer/kernels/torch_ext/csrc/common/types.hpp:141-146): 32 values as an fp16
 * scale d followed by 32 int8, 34 bytes, rows are whole blocks.
 * Quantise (reference: src/minfer/kernels/torch_ext/csrc/quants/impl.cpp:1169-1193): amax = max |x|,
 * d = amax / 127, id = d ? 1 / d : 0, q = roundf(x * id), d stored rounded to fp16 -- all in fp32.
 * Dequantise (reference: csrc/quants/impl.cpp:1152-1167, cuda/quants/impls.cuh:121-143): y = (T)(q * (float)d).
 *
 * Pinned by tests/test_oracle_quant.py: byte equality with the reference's own source compiled into
 * oracle/_ref where that library is present, the fp16 conversions against numpy's for every fp16 bit
 * pattern and random floats, hand-computed blocks (ties round away from zero, all-zero block), and the
 * error bound |x - dq| <= d/2 (+ the rounding of d) on random rows.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* IEEE binary32 -> binary16, round to nearest even, overflow to infinity, subnormals kept. */
uint16_t oracle_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t mag = x & 0x7fffffffu;
    if (mag >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (mag > 0x7f800000u ? 0x200u | ((mag >> 13) & 0x3ffu) : 0u));
    if (mag >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);           /* >= 65520 rounds to infinity */
    if (mag < 0x33000001u) return (uint16_t)sign;                         /* <= 2^-25 rounds to zero */
    int e = (int)(mag >> 23) - 127;
    uint32_t m = (mag & 0x7fffffu) | 0x800000u;                           /* 24-bit significand */
    int shift;                                                            /* bits to drop */
    uint32_t base;
    if (e >= -14) { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7fffffu; }
    else { shift = 13 + (-14 - e); base = 0; }
    uint32_t kept = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (kept & 1u))) kept += 1;           /* may carry into the exponent: still right */
    return (uint16_t)(sign | (base + kept));
}

float oracle_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    float out;
    uint32_t bits;
    if (e == 0) {
        out = ldexpf((float)m, -24);
        memcpy(&bits, &out, 4);
        bits |= sign;
    } else if (e == 31) {
        bits = sign | 0x7f800000u | (m << 13);
    } else {
        bits = sign | ((e + 112u) << 23) | (m << 13);
    }
    memcpy(&out, &bits, 4);
    return out;
}

/* x [n_rows, k] fp32 -> y [n_rows, k/32*34] bytes. */
int oracle_quant_q8_0(const float* x, uint8_t* y, int64_t n_rows, int64_t k) {
    if (k % 32 != 0 || n_rows < 0) return -1;
    const int64_t nb = n_rows * (k / 32);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < nb; ++i) {
        const float* xb = x + 32 * i;
        uint8_t* yb = y + 34 * i;
        float amax = 0.0f;
        for (int j = 0; j < 32; ++j) {
            const float a = fabsf(xb[j]);
            if (a > amax) amax = a;
        }
        const float d = amax / 127.0f;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        const uint16_t dh = oracle_f32_to_f16(d);
        memcpy(yb, &dh, 2);
        for (int j = 0; j < 32; ++j) {
            const float x0 = xb[j] * id;
            yb[2 + j] = (uint8_t)(int8_t)roundf(x0);
        }
    }
    return 0;
}

/* y fp32 [n_rows, k] = q * (float)d. */
int oracle_dequant_q8_0(const uint8_t* x, float* y, int64_t n_rows, int64_t k) {
    if (k % 32 != 0 || n_rows < 0) return -1;
    const int64_t nb = n_rows * (k / 32);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < nb; ++i) {
        uint16_t dh;
        memcpy(&dh, x + 34 * i, 2);
        const float d = oracle_f16_to_f32(dh);
        for (int j = 0; j < 32; ++j) y[32 * i + j] = (float)(int8_t)x[34 * i + 2 + j] * d;
    }
    return 0;
}

/* y fp16 bits [n_rows, k] = (half)(q * (float)d). */
int oracle_dequant_q8_0_f16(const uint8_t* x, uint16_t* y, int64_t n_rows, int64_t k) {
    if (k % 32 != 0 || n_rows < 0) return -1;
    const int64_t nb = n_rows * (k / 32);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < nb; ++i) {
        uint16_t dh;
        memcpy(&dh, x + 34 * i, 2);
        const float d = oracle_f16_to_f32(dh);
        for (int j = 0; j < 32; ++j) y[32 * i + j] = oracle_f32_to_f16((float)(int8_t)x[34 * i + 2 + j] * d);
    }
    return 0;
}
