/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the fused-attention path.
 *
 * Nothing in the shipped package may import, link or call this file; it is the
 * checker used by tests/, by __graft_entry__.smoke() and by the cpu_baseline
 * leg of bench.py.
 *
 * What it restates.  The reference's attention arithmetic is one library call,
 *   F.scaled_dot_product_attention(Q, K_exp, V_exp, attn_mask=mask)
 * (reference: src/minfer/kernels/refs.py:53-55), where K_exp/V_exp are the KV
 * heads repeated n_rep = Hq/Hkv times along the head axis
 * (reference: test/kernels.py:252-257), mask is bool with True = attend and
 * mask[b,0,i,j] gating query i against key j (reference: test/kernels.py:242),
 * and the scale is the SDPA default 1/sqrt(D).  The arithmetic itself lives in
 * third-party torch (pinned 2.10.0 in the reference's uv.lock:601-602); what is
 * restated here is its published definition
 *   out[b,h,i,:] = sum_j softmax_j( q[b,h,i,:].k[b,h/n_rep,j,:]/sqrt(D) | mask ) v[b,h/n_rep,j,:]
 * with a row whose mask is entirely False producing zeros (what torch 2.10's
 * CPU SDPA returns for such a row).
 *
 * Tensor arguments follow the reference operator's layouts
 * (reference: src/minfer/kernels/torch_ext/csrc/cuda/flash_attn/op.cuh:21-30):
 * q/out [B,Hq,L,D], k/v [B,Hkv,L,D], element strides for dims 0..2 and unit
 * stride on D.  The decode and varlen entry points have no counterpart in the
 * reference (its op demands Lq == Lk, op.cuh:74-78); they are the same closed
 * form restricted to one query row per sequence over a KV cache laid out as
 * the reference's cache (reference: src/minfer/core.py:105-127), and to
 * causal attention inside each packed sequence.
 *
 * Inputs are fp32 (callers up-cast fp16/bf16 first); accumulation is fp64 so
 * the oracle is at least as accurate as an fp32 reference.
 *
 * Pinning (see tests/test_oracle.py): checked against torch's CPU SDPA on the
 * reference's exact call, against an independent numpy fp64 evaluation, against
 * committed golden vectors, and against closed-form invariants (row 0 of a
 * causal mask copies V row 0, one-hot mask rows copy a V row, Q=0 gives running
 * means, constant-per-KV-head V exposes the GQA head mapping).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
    int64_t q0, q1, q2;    /* q strides, dims 0..2 (elements)   */
    int64_t kv0, kv1, kv2; /* k and v strides (shared)          */
    int64_t o0, o1, o2;    /* out strides                       */
} oracle_strides;

/* One query row against keys [key_lo, key_hi) of one KV head; mask_row may be NULL
 * (all attend) or points at the row's bool bytes indexed by absolute key index. */
static void attend_row(const float* q, const float* k, const float* v, int64_t kv2,
                       int64_t key_lo, int64_t key_hi, const uint8_t* mask_row,
                       int64_t D, double scale, float* out, double* s_buf)
{
    double m = -INFINITY;
    for (int64_t j = key_lo; j < key_hi; ++j) {
        if (mask_row && !mask_row[j]) { s_buf[j - key_lo] = -INFINITY; continue; }
        const float* kj = k + j * kv2;
        double acc = 0.0;
        for (int64_t d = 0; d < D; ++d) acc += (double)q[d] * (double)kj[d];
        acc *= scale;
        s_buf[j - key_lo] = acc;
        if (acc > m) m = acc;
    }
    if (m == -INFINITY) { /* nothing attended: zeros */
        for (int64_t d = 0; d < D; ++d) out[d] = 0.0f;
        return;
    }
    double l = 0.0;
    double o[512];
    for (int64_t d = 0; d < D; ++d) o[d] = 0.0;
    for (int64_t j = key_lo; j < key_hi; ++j) {
        double s = s_buf[j - key_lo];
        if (s == -INFINITY) continue;
        double p = exp(s - m);
        l += p;
        const float* vj = v + j * kv2;
        for (int64_t d = 0; d < D; ++d) o[d] += p * (double)vj[d];
    }
    for (int64_t d = 0; d < D; ++d) out[d] = (float)(o[d] / l);
}

/* Dense-mask attention, the reference operator's contract (op.cuh:21-30, refs.py:53-55).
 * mask: contiguous bool bytes [B,1,L,L].  Returns 0, or -1 on unsupported D. */
int oracle_flash_attn(const float* q, const float* k, const float* v, const uint8_t* mask,
                      float* out, int64_t B, int64_t Hq, int64_t Hkv, int64_t L, int64_t D,
                      const oracle_strides* st)
{
    if (D > 512 || Hq % Hkv != 0) return -1;
    const int64_t n_rep = Hq / Hkv;
    const double scale = 1.0 / sqrt((double)D);
    const int64_t rows = B * Hq * L;
    #pragma omp parallel
    {
        double* s_buf = (double*)malloc(sizeof(double) * (size_t)(L > 0 ? L : 1));
        #pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < rows; ++r) {
            int64_t i = r % L, h = (r / L) % Hq, b = r / (L * Hq);
            int64_t g = h / n_rep; /* repeat_interleave(n_rep, dim=1): test/kernels.py:252-255 */
            attend_row(q + b * st->q0 + h * st->q1 + i * st->q2,
                       k + b * st->kv0 + g * st->kv1, v + b * st->kv0 + g * st->kv1, st->kv2,
                       0, L, mask + (b * L + i) * L, D, scale,
                       out + b * st->o0 + h * st->o1 + i * st->o2, s_buf);
        }
        free(s_buf);
    }
    return 0;
}

/* Same as oracle_flash_attn for a subset of query rows only (so that full-size problems can be
 * spot-checked in seconds): rows[n] are query indices, mask_rows is [B,n,L] bool bytes holding
 * mask[b,0,rows[r],:]; out is contiguous [B,Hq,n,D]. */
int oracle_flash_attn_rows(const float* q, const float* k, const float* v, const uint8_t* mask_rows,
                           const int64_t* rows, int64_t n, float* out,
                           int64_t B, int64_t Hq, int64_t Hkv, int64_t L, int64_t D,
                           const oracle_strides* st)
{
    if (D > 512 || Hq % Hkv != 0) return -1;
    for (int64_t r = 0; r < n; ++r) if (rows[r] < 0 || rows[r] >= L) return -2;
    const int64_t n_rep = Hq / Hkv;
    const double scale = 1.0 / sqrt((double)D);
    #pragma omp parallel
    {
        double* s_buf = (double*)malloc(sizeof(double) * (size_t)(L > 0 ? L : 1));
        #pragma omp for schedule(dynamic, 4)
        for (int64_t t = 0; t < B * Hq * n; ++t) {
            int64_t r = t % n, h = (t / n) % Hq, b = t / (n * Hq), g = h / n_rep;
            attend_row(q + b * st->q0 + h * st->q1 + rows[r] * st->q2,
                       k + b * st->kv0 + g * st->kv1, v + b * st->kv0 + g * st->kv1, st->kv2,
                       0, L, mask_rows + (b * n + r) * L, D, scale,
                       out + ((b * Hq + h) * n + r) * D, s_buf);
        }
        free(s_buf);
    }
    return 0;
}

/* Single-token decode over a KV cache [B,Hkv,Lmax,D] (layout of core.py:105-127):
 * query b attends keys 0..ctx_lens[b]-1; q/out are [B,Hq,1,D] (q2/o2 unused). */
int oracle_flash_attn_decode(const float* q, const float* k_cache, const float* v_cache,
                             const int32_t* ctx_lens, float* out,
                             int64_t B, int64_t Hq, int64_t Hkv, int64_t Lmax, int64_t D,
                             const oracle_strides* st)
{
    if (D > 512 || Hq % Hkv != 0) return -1;
    const int64_t n_rep = Hq / Hkv;
    const double scale = 1.0 / sqrt((double)D);
    for (int64_t b = 0; b < B; ++b) if (ctx_lens[b] < 0 || ctx_lens[b] > Lmax) return -2;
    #pragma omp parallel
    {
        double* s_buf = (double*)malloc(sizeof(double) * (size_t)(Lmax > 0 ? Lmax : 1));
        #pragma omp for schedule(dynamic, 1)
        for (int64_t r = 0; r < B * Hq; ++r) {
            int64_t h = r % Hq, b = r / Hq, g = h / n_rep;
            attend_row(q + b * st->q0 + h * st->q1,
                       k_cache + b * st->kv0 + g * st->kv1, v_cache + b * st->kv0 + g * st->kv1,
                       st->kv2, 0, ctx_lens[b], NULL, D, scale,
                       out + b * st->o0 + h * st->o1, s_buf);
        }
        free(s_buf);
    }
    return 0;
}

/* Packed ragged prefill: q/out [1,Hq,T,D], k/v [1,Hkv,T,D]; sequence s owns token rows
 * cu_seqlens[s]..cu_seqlens[s+1]-1 and attends causally inside itself only. */
int oracle_flash_attn_varlen(const float* q, const float* k, const float* v,
                             const int32_t* cu_seqlens, int64_t n_seqs, float* out,
                             int64_t Hq, int64_t Hkv, int64_t T, int64_t D,
                             const oracle_strides* st)
{
    if (D > 512 || Hq % Hkv != 0) return -1;
    if (cu_seqlens[0] != 0 || cu_seqlens[n_seqs] != T) return -2;
    for (int64_t s = 0; s < n_seqs; ++s) if (cu_seqlens[s + 1] < cu_seqlens[s]) return -2;
    const int64_t n_rep = Hq / Hkv;
    const double scale = 1.0 / sqrt((double)D);
    #pragma omp parallel
    {
        double* s_buf = (double*)malloc(sizeof(double) * (size_t)(T > 0 ? T : 1));
        #pragma omp for schedule(dynamic, 16)
        for (int64_t r = 0; r < Hq * T; ++r) {
            int64_t i = r % T, h = r / T, g = h / n_rep;
            int64_t s = 0;
            while (cu_seqlens[s + 1] <= i) ++s;
            attend_row(q + h * st->q1 + i * st->q2, k + g * st->kv1, v + g * st->kv1, st->kv2,
                       cu_seqlens[s], i + 1, NULL, D, scale, out + h * st->o1 + i * st->o2, s_buf);
        }
        free(s_buf);
    }
    return 0;
}
