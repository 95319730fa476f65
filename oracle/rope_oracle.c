/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for rotary position embedding and the
 * rope + KV-cache append producer.
 *
 * Nothing in the shipped package may import, link or call this file; it is the
 * checker used by tests/ and by the cpu_baseline legs of bench.py.
 *
 * What it restates.  The reference defines both styles twice, in agreement:
 * as CUDA kernels (reference: src/minfer/kernels/torch_ext/csrc/cuda/il_rope/kernel.cuh:21-38,
 * neox_rope/kernel.cuh:22-37) and as torch expressions (reference:
 * src/minfer/kernels/refs.py:12-47).  For token index l of a tensor x [B,L,H,D]:
 *   pos   = start_pos + l
 *   theta = pos * freq_base^(-2 i / rotary_dim)            i = 0 .. rotary_dim/2 - 1
 *   (x0, x1) <- (cos(theta) x0 - sin(theta) x1,  sin(theta) x0 + cos(theta) x1)
 * with (x0, x1) = elements (2i, 2i+1) of the head for the interleaved style and
 * (i, i + rotary_dim/2) for the NeoX style; elements rotary_dim..D-1 are unchanged.
 * (The torch form multiplies the complex number x0 + i x1 by exp(i theta), which is
 * the same thing.)  The reference evaluates theta in fp32; here everything is fp64,
 * which is what the mathematics fixes: the reference's own test allows atol 5e-3
 * for that reason (reference: test/kernels.py:94-95).
 *
 * The append producer has no single counterpart in the reference: it is its
 * intended sequence rope(q), rope(k), store k and v in the cache
 * (reference: src/minfer/core.py:228-232) with the cache laid out
 * [B, Hkv, Lmax, D] (reference: src/minfer/core.py:105-127) and the position of
 * token l of sequence b equal to positions[b] + l.
 *
 * Inputs and outputs are fp32 (callers up-cast fp16/bf16 first and round the
 * result themselves); arithmetic is fp64.  Return 0, or -1 on a bad argument.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define ORACLE_ROPE_INTERLEAVED 0
#define ORACLE_ROPE_NEOX 1

static void rotate_head(float* xh, int style, int64_t rotary_dim, int64_t pos, double freq_base) {
    const int64_t half = rotary_dim / 2;
    for (int64_t i = 0; i < half; ++i) {
        const double theta = (double)pos * pow(freq_base, -2.0 * (double)i / (double)rotary_dim);
        const double c = cos(theta), s = sin(theta);
        const int64_t i0 = style == ORACLE_ROPE_INTERLEAVED ? 2 * i : i;
        const int64_t i1 = style == ORACLE_ROPE_INTERLEAVED ? 2 * i + 1 : i + half;
        const double x0 = xh[i0], x1 = xh[i1];
        xh[i0] = (float)(c * x0 - s * x1);
        xh[i1] = (float)(s * x0 + c * x1);
    }
}

/* x [B,L,H,D] contiguous, rotated in place. */
int oracle_rope(int style, float* x, int64_t B, int64_t L, int64_t H, int64_t D, int64_t rotary_dim,
                int64_t start_pos, double freq_base) {
    if ((style != ORACLE_ROPE_INTERLEAVED && style != ORACLE_ROPE_NEOX) || !x || B < 0 || L < 0 || H < 0 ||
        D <= 0 || rotary_dim < 0 || rotary_dim > D || rotary_dim % 2 != 0 || !(freq_base > 0.0))
        return -1;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t b = 0; b < B; ++b)
        for (int64_t l = 0; l < L; ++l)
            for (int64_t h = 0; h < H; ++h)
                rotate_head(x + ((b * L + l) * H + h) * D, style, rotary_dim, start_pos + l, freq_base);
    return 0;
}

/* q [B,L,Hq,D] rotated in place; k, v [B,L,Hkv,D] read; caches [B,Hkv,Lmax,D] contiguous, rows
 * positions[b] + l written (rows outside 0..Lmax-1 skipped), every other cache element untouched. */
int oracle_rope_kv_append(int style, float* q, const float* k, const float* v, const int32_t* positions,
                          float* k_cache, float* v_cache, int64_t B, int64_t L, int64_t Hq, int64_t Hkv,
                          int64_t D, int64_t Lmax, int64_t rotary_dim, double freq_base) {
    if ((style != ORACLE_ROPE_INTERLEAVED && style != ORACLE_ROPE_NEOX) || !q || !k || !v || !positions ||
        !k_cache || !v_cache || B < 0 || L < 0 || Hq < 0 || Hkv < 0 || D <= 0 || D > 4096 || Lmax < 0 ||
        rotary_dim < 0 || rotary_dim > D || rotary_dim % 2 != 0 || !(freq_base > 0.0))
        return -1;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t b = 0; b < B; ++b)
        for (int64_t l = 0; l < L; ++l) {
            const int64_t pos = (int64_t)positions[b] + l;
            for (int64_t h = 0; h < Hq; ++h)
                rotate_head(q + ((b * L + l) * Hq + h) * D, style, rotary_dim, pos, freq_base);
            if (pos < 0 || pos >= Lmax) continue;
            for (int64_t g = 0; g < Hkv; ++g) {
                float row[4096];
                memcpy(row, k + ((b * L + l) * Hkv + g) * D, (size_t)D * sizeof(float));
                rotate_head(row, style, rotary_dim, pos, freq_base);
                memcpy(k_cache + ((b * Hkv + g) * Lmax + pos) * D, row, (size_t)D * sizeof(float));
                memcpy(v_cache + ((b * Hkv + g) * Lmax + pos) * D, v + ((b * L + l) * Hkv + g) * D,
                       (size_t)D * sizeof(float));
            }
        }
    return 0;
}
