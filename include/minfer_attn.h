/*
 * C ABI of the MI355X (gfx950) fused-attention library, libminfer_attn.so.
 *
 * Every entry point takes plain device pointers, sizes, element strides and a HIP stream
 * (as void*), launches asynchronously on that stream and never synchronises or allocates.
 * Scratch memory is a caller-provided workspace whose size the *_workspace_bytes
 * functions report.  Return value: 0 on success, a negative MINFER_ATTN_E* code on a
 * rejected call (nothing was launched); minfer_attn_last_error() then describes it.
 *
 * The operator-level contract these functions implement is the reference's
 *   flash_attn(int qtype_int, int qblock_size, int qtype_size,
 *              Tensor q, Tensor k, Tensor v, Tensor(a!) mask, Tensor(a!) out) -> ()
 * (reference: src/minfer/kernels/torch_ext/csrc/reg.cpp:30), whose host function is
 * flash_attn_cuda (reference: src/minfer/kernels/torch_ext/csrc/cuda/flash_attn/op.cuh:21-106).
 */
#ifndef MINFER_ATTN_H
#define MINFER_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types, numbered as the reference numbers its activations' GGML types
 * (reference: src/minfer/const.py:4-35: F16 = 1, BF16 = 30). */
#define MINFER_ATTN_F16 1
#define MINFER_ATTN_BF16 30
#define MINFER_ATTN_F32 0    /* only as the float side of minfer_quant_q8_0 / minfer_dequant_q8_0 */

#define MINFER_ATTN_OK 0
#define MINFER_ATTN_EINVAL (-1)    /* shape, stride, dtype or alignment rejected        */
#define MINFER_ATTN_EWORKSPACE (-2) /* workspace missing or smaller than required       */
#define MINFER_ATTN_ELAUNCH (-3)   /* the HIP runtime refused the launch                */

/* Element strides of dims 0..2 of q, of k (v must share them) and of out; dim 3 (head_dim)
 * always has stride 1.  Replaces the reference's QKVStrides, which carries no out strides
 * (reference: src/minfer/kernels/torch_ext/csrc/cuda/flash_attn/kernels/kernel.cuh:12-15,
 * filled at op.cuh:80-83). */
typedef struct minfer_attn_strides {
    int64_t q0, q1, q2;
    int64_t kv0, kv1, kv2;
    int64_t o0, o1, o2;
} minfer_attn_strides;

/* Library/ABI version (major * 1000 + minor). */
int minfer_attn_version(void);

/* Message for the most recent non-zero return on the calling thread ("" if none). */
const char* minfer_attn_last_error(void);

/* Bytes of workspace minfer_flash_attn needs for batch B and sequence length L (holds the
 * per-tile mask classification). */
size_t minfer_flash_attn_workspace_bytes(int64_t B, int64_t L);

/*
 * Dense-mask GQA attention (prefill):
 *   out[b,h,i,:] = sum_j softmax_j(q[b,h,i,:].k[b,h/n_rep,j,:]/sqrt(D) | mask[b,0,i,j]) v[b,h/n_rep,j,:]
 * q,out [B,Hq,L,D]; k,v [B,Hkv,L,D]; mask contiguous bool bytes [B,1,L,L], non-zero = attend;
 * n_rep = Hq/Hkv.  A query row with no attended key yields zeros.
 * Replaces flash_attn_cuda + flash_attn_cuda_impl (reference: flash_attn/op.cuh:21-106,
 * flash_attn/kernels/kernel.cuh:16-27).  Beyond the reference's checks (op.cuh:32-96):
 * dtype may be MINFER_ATTN_F16 or MINFER_ATTN_BF16, D may be 64 or 128, all data pointers must
 * be 16-byte aligned and all strides multiples of 8 elements.
 */
int minfer_flash_attn(int dtype, const void* q, const void* k, const void* v,
                      const uint8_t* mask, void* out,
                      int64_t B, int64_t Hq, int64_t Hkv, int64_t L, int64_t D,
                      const minfer_attn_strides* strides,
                      void* workspace, size_t workspace_bytes, void* stream);

/* Bytes of workspace minfer_flash_attn_decode needs (split-KV partial results). */
size_t minfer_flash_attn_decode_workspace_bytes(int64_t B, int64_t Hq, int64_t Lmax, int64_t D);

/*
 * Single-token decode over a KV cache: q,out [B,Hq,1,D]; k_cache,v_cache [B,Hkv,Lmax,D]
 * (the reference's cache layout, src/minfer/core.py:105-127); ctx_lens int32 [B] on the device;
 * query b attends cache rows 0..ctx_lens[b]-1 (rows beyond are never read into the result;
 * ctx_lens[b] == 0 yields zeros).  The KV range is split across workgroups and merged by a
 * log-sum-exp combine kernel.  No counterpart in the reference (its op requires Lq == Lk,
 * flash_attn/op.cuh:74-78); strides->q2 and strides->o2 are ignored.
 */
int minfer_flash_attn_decode(int dtype, const void* q, const void* k_cache, const void* v_cache,
                             const int32_t* ctx_lens, void* out,
                             int64_t B, int64_t Hq, int64_t Hkv, int64_t Lmax, int64_t D,
                             const minfer_attn_strides* strides,
                             void* workspace, size_t workspace_bytes, void* stream);

/*
 * minfer_flash_attn_decode without a workspace argument, for callers that cannot allocate device memory: code
 * under HIP graph capture, serving loops and harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  The split-KV partial results go to a device array that is part of the library's code object
 * (MINFER_DECODE_NOALLOC_SCRATCH_BYTES bytes on every GPU the library is used on, held until the process ends);
 * a problem whose minfer_flash_attn_decode_workspace_bytes(B, Hq, Lmax, D) exceeds that size is rejected with
 * MINFER_ATTN_EWORKSPACE (nothing launched).  The call allocates and frees nothing.  Its first call on a device
 * looks the array's address up (which may load the code object): make that call outside a graph capture.  All calls
 * on one GPU share the array: calls that overlap in time on one GPU (two streams, two threads) race; calls that
 * follow each other on one stream do not.  The array used is the copy on the device that owns `stream` (the
 * current device for the null stream); that device must be the current one, a stream of another device is
 * rejected with MINFER_ATTN_EINVAL.  Arguments, results and errors are otherwise those of
 * minfer_flash_attn_decode (16-bit caches only).
 */
#ifndef MINFER_DECODE_NOALLOC_SCRATCH_BYTES   /* a build that never calls the entry point may shrink the array (define it when compiling the library) */
#define MINFER_DECODE_NOALLOC_SCRATCH_BYTES (64u << 20)
#endif
int minfer_flash_attn_decode_noalloc(int dtype, const void* q, const void* k_cache, const void* v_cache,
                                     const int32_t* ctx_lens, void* out,
                                     int64_t B, int64_t Hq, int64_t Hkv, int64_t Lmax, int64_t D,
                                     const minfer_attn_strides* strides, void* stream);

/*
 * Packed ragged causal prefill: q,out [1,Hq,T,D]; k,v [1,Hkv,T,D]; cu_seqlens int32 [n_seqs+1]
 * on the device with cu_seqlens[0] == 0 and cu_seqlens[n_seqs] == T; token rows
 * cu_seqlens[s]..cu_seqlens[s+1]-1 form sequence s and attend causally inside it only.
 * Equals minfer_flash_attn with B = 1, L = T under the block-diagonal causal mask.  Needs no
 * workspace.  No counterpart in the reference; strides->q0, kv0, o0 are ignored.
 * max_seqlen: an upper bound of the sequence lengths (0 = not known); it sizes the launch and selects the
 * workgroup shape, and rows of a sequence past max_seqlen are not computed.  cu_seqlens is read on the
 * device only and is not trusted: every sequence is cut to its part inside [0, T) and an end before its
 * start is an empty sequence, so malformed entries (decreasing, negative, past T) cannot cause an access
 * outside q/k/v/out; which rows such a call computes is unspecified beyond that, valid ones excepted.
 */
int minfer_flash_attn_varlen(int dtype, const void* q, const void* k, const void* v,
                             const int32_t* cu_seqlens, int64_t n_seqs, int64_t max_seqlen,
                             void* out, int64_t Hq, int64_t Hkv, int64_t T, int64_t D,
                             const minfer_attn_strides* strides, void* stream);

/* Rotary embedding styles. */
#define MINFER_ROPE_INTERLEAVED 0   /* pairs (2i, 2i+1) of a head   (reference: il_rope) */
#define MINFER_ROPE_NEOX 1          /* pairs (i, i + rotary_dim/2)  (reference: neox_rope) */

/*
 * Rotary position embedding, in place: x [B,L,H,D] contiguous; for the token at index l the position is
 * start_pos + l; pair i < rotary_dim/2 of every head is rotated by the angle
 * pos * freq_base^(-2i/rotary_dim): (x0, x1) -> (cos*x0 - sin*x1, sin*x0 + cos*x1); elements
 * rotary_dim..D-1 are not touched.  Replaces il_rope_cuda / neox_rope_cuda and their kernels
 * (reference: il_rope/op.cuh:20-58, il_rope/kernel.cuh:9-39, neox_rope/op.cuh, neox_rope/kernel.cuh:9-38;
 * oracle refs.py:12-47).  Beyond the reference: dtype may be MINFER_ATTN_BF16; rotary_dim must be even
 * and at most 256.
 */
int minfer_rope(int dtype, int style, void* x, int64_t B, int64_t L, int64_t H, int64_t D,
                int64_t rotary_dim, int64_t start_pos, double freq_base, void* stream);

/*
 * The step before attention, fused (reference: the il_rope(q), il_rope(k) calls and the cache they feed,
 * src/minfer/core.py:228-232, cache layout core.py:105-127): q [B,L,Hq,D] is rotated in place; k [B,L,Hkv,D]
 * is rotated and written to k_cache[b, g, positions[b] + l, :]; v [B,L,Hkv,D] is copied to the same row of
 * v_cache.  positions is int32 [B] on the device (the number of rows sequence b already holds); token l of
 * sequence b has position positions[b] + l.  Caches are [B,Hkv,Lmax,D] with the given element strides
 * (multiples of 8) for their first three dims; rows outside 0..Lmax-1 are not written (q is still
 * rotated).  k and v are only read.  All pointers 16-byte aligned, D a multiple of 8, rotary_dim a
 * multiple of 8 (interleaved) or 16 (NeoX).  No counterpart as one call in the reference.
 */
int minfer_rope_kv_append(int dtype, int style, void* q, const void* k, const void* v,
                          const int32_t* positions, void* k_cache, void* v_cache,
                          int64_t B, int64_t L, int64_t Hq, int64_t Hkv, int64_t D, int64_t Lmax,
                          int64_t cache_stride_b, int64_t cache_stride_h, int64_t cache_stride_row,
                          int64_t rotary_dim, double freq_base, void* stream);

/*
 * The producer with the per-head RMS normalisation of q and k in front of the rotation (reference: the optional
 * rmsnorm(q), rmsnorm(k) calls between the QKV projection and the rotary embedding, src/minfer/core.py:224-230, each
 * being rmsnorm_cuda over [B,L,n_heads,head_dim], rmsnorm/op.cuh:20-70): every head of q is replaced by
 * rope(round(rmsnorm(head, wq_norm, eps))), every head of k goes through the same with wk_norm on its way into the
 * cache, v is copied; the result equals minfer_rmsnorm on q and on k followed by minfer_rope_kv_append (or
 * minfer_rope_kv_append_q8_0) bit for bit, with one pass over q, k and v instead of two.  wq_norm / wk_norm are
 * [D] in the activations' dtype; a null weight leaves that tensor un-normalised.  cache_type is the activations'
 * dtype (caches [B,Hkv,Lmax,D], element strides) or MINFER_Q8_0 (caches of Q8_0 blocks, byte strides, rows dense:
 * cache_stride_row = D/32 * 34).  D must be 64 or 128; the other requirements are those of minfer_rope_kv_append.
 * No counterpart as one call in the reference.
 */
int minfer_rope_kv_append_norm(int dtype, int style, int cache_type, void* q, const void* k, const void* v,
                               const void* wq_norm, const void* wk_norm, double eps,
                               const int32_t* positions, void* k_cache, void* v_cache,
                               int64_t B, int64_t L, int64_t Hq, int64_t Hkv, int64_t D, int64_t Lmax,
                               int64_t cache_stride_b, int64_t cache_stride_h, int64_t cache_stride_row,
                               int64_t rotary_dim, double freq_base, void* stream);

/*
 * RMS normalisation: in, out are n_vectors contiguous vectors of length dim; w has dim elements;
 *   out[v, i] = in[v, i] * w[i] / sqrt(mean_i(in[v, :]^2) + eps)      (fp32 arithmetic, one rounding)
 * The reference's [B,L,hidden] and [B,L,n_heads,head_dim] inputs are both this with dim = |w| and
 * n_vectors = numel / dim.  in and out may be the same buffer.  Replaces rmsnorm_cuda and its kernel
 * (reference: rmsnorm/op.cuh:20-70, rmsnorm/kernel.cuh:11-40; oracle refs.py:4-10).  Beyond the reference:
 * dtype may be MINFER_ATTN_BF16.
 */
int minfer_rmsnorm(int dtype, const void* in, const void* w, void* out, int64_t n_vectors, int64_t dim,
                   double eps, void* stream);

/* Layout of the weight operand of minfer_gemm. */
#define MINFER_GEMM_B_KN 0   /* B is [K, N]: D = alpha * A B + beta * C     (reference: dispatch_f16_ab)  */
#define MINFER_GEMM_B_NK 1   /* B is [N, K]: D = alpha * A B^T + beta * C   (reference: dispatch_f16_abt, empty there) */

/*
 * D[M,N] = alpha * A[M,K] x B + beta * C[M,N], 16-bit operands, fp32 accumulation, one rounding.  lda..ldd
 * are row strides in elements (ldb: of B as stored).  C may be null when beta == 0 and may alias D.
 * Replaces gemm_cuda's F16 paths and their kernels (reference: gemm/op.cuh:218-316, gemm/kernels/gemm_f16.cuh;
 * oracle refs.py:49-51), and is what the QKV projection runs on (reference: qkv/op.cuh, a stub).  The tiled
 * MFMA kernel needs K % 64 == 0, N % 8 == 0, 16-byte aligned A and B with strides that are multiples of 8 and
 * 8-byte aligned C and D with strides that are multiples of 4; anything else runs a plain kernel.
 */
int minfer_gemm(int dtype, int b_layout, const void* A, const void* B, const void* C, void* D,
                int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t ldd,
                double alpha, double beta, void* stream);

/*
 * minfer_gemm with a workspace.  A problem of a few dozen rows against a wide weight (a batch of decode steps, a short
 * prefill chunk) has too few output tiles to occupy the chip; given minfer_gemm_workspace_bytes(M, N, K) bytes of
 * device memory (16-byte aligned; 0 = this shape does not use any), the K dimension is cut into slices that run as
 * separate workgroups and meet in the workspace as fp32 partial sums, which a second kernel adds up (alpha, beta and
 * C applied there, one rounding): slices of the 128 x 128 tiles, or, up to 64 rows against an [N, K] weight of fewer
 * than 12288 columns, of 64-column stripes (where two launches pay: from 9 rows on below 6144 columns, from 2 on rows
 * of 8192 values and more of at most 1536 columns, from 33 between 6144 and 12288 columns).  With a null workspace the
 * call is minfer_gemm; a workspace smaller than minfer_gemm_workspace_bytes is used only by a path whose slices fit
 * in it.  No counterpart in the
 * reference, whose gemm_cuda takes no scratch memory (reference: gemm/op.cuh:218-316); same contract for the
 * workspace as the attention entry points (contents need not be initialised; one per stream).
 */
size_t minfer_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);
int minfer_gemm_ws(int dtype, int b_layout, const void* A, const void* B, const void* C, void* D,
                   int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t ldd,
                   double alpha, double beta, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The projection against a weight stored as Q8_0 blocks: D[M,N] = alpha * A[M,K] x W^T + beta * C[M,N] with W given as N
 * dense rows of K/32 blocks of 34 bytes (4-byte aligned), every weight dequantised to fp16 exactly as
 * minfer_dequant_q8_0 does, fp16 A, C and D, fp32 accumulation, one rounding: the result is that of minfer_gemm
 * (MINFER_GEMM_B_NK) on the dequantised weight, element for element up to the order of the fp32 sums.  Up to 64 rows of A
 * and an even number of blocks per weight row, a kernel streams the blocks once (34 bytes per 32 weights instead of
 * 64: the projections of a decode step) and no workspace is needed; for 2-64 rows against fewer than 12288 columns
 * minfer_gemm_q8_0_workspace_bytes still names one, for K slices as in minfer_gemm_ws (fp32 partial sums, a second
 * launch), which the call uses when it is given in full and does without otherwise.  Other shapes dequantise the
 * weight into the workspace and run the fp16 kernels on it: for them a missing or too small workspace is
 * MINFER_ATTN_EWORKSPACE.  This is the case the reference's
 * gemm_cuda routes to dispatch_quant_abt, whose body is empty (reference: gemm/op.cuh:199-210, 299-312); block format
 * common/types.hpp:141-146, dequantisation cuda/quants/impls.cuh:121-143.
 */
size_t minfer_gemm_q8_0_workspace_bytes(int64_t M, int64_t N, int64_t K);
int minfer_gemm_q8_0(const void* A, const void* Bq, const void* C, void* D, int64_t M, int64_t N, int64_t K,
                     int64_t lda, int64_t ldc, int64_t ldd, double alpha, double beta,
                     void* workspace, size_t workspace_bytes, void* stream);

/*
 * The QKV projection in one launch: q_out[M,Nq] = x[M,K] wq^T, k_out[M,Nk] = x wk^T, v_out[M,Nv] = x wv^T, the three
 * weights stored [N, K] (the reference's layout for them), 16-bit operands, fp32 accumulation, one rounding; ld* are
 * row strides in elements.  What the reference's fused qkv operator is meant to be (reference:
 * src/minfer/kernels/torch_ext/csrc/cuda/qkv/op.cuh:21-34, a stub there; the model's call src/minfer/core.py:222-223;
 * expected values test/kernels.py:172-216).  One grid covers the column tiles of all three weights, so x is
 * read by one kernel and the narrow k and v projections share the launch with the wide q projection; every element
 * equals what minfer_gemm with MINFER_GEMM_B_NK, alpha 1, beta 0 gives for its weight, up to the order of the fp32
 * sums (bit for bit from 65 rows on, where both run the same tiles; up to 64 rows the few-row kernel is chosen by the
 * width, which is the three weights' together here and one weight's there).  Shapes the tiled kernels cannot take (see
 * minfer_gemm) run as three plain launches.
 */
int minfer_qkv(int dtype, const void* x, const void* wq, const void* wk, const void* wv,
               void* q_out, void* k_out, void* v_out, int64_t M, int64_t K, int64_t Nq, int64_t Nk, int64_t Nv,
               int64_t ldx, int64_t ldwq, int64_t ldwk, int64_t ldwv, int64_t ldq, int64_t ldk, int64_t ldv,
               void* stream);

/*
 * Q8_0 blocks: 32 consecutive values of a row as an fp16 scale d followed by 32 int8, 34 bytes, no padding
 * (reference: src/minfer/kernels/torch_ext/csrc/common/types.hpp:141-146; GGML type 8, sizes const.py:46).
 */
#define MINFER_Q8_0 8
#define MINFER_Q8_0_BLOCK 32        /* values per block */
#define MINFER_Q8_0_BLOCK_BYTES 34  /* bytes per block  */

/*
 * Quantises n_rows contiguous rows of k values (k a multiple of 32) into rows of k/32 blocks: per block
 * d = max|x| / 127, q = roundf(x / d) (ties away from zero; all zero when d is), d stored as fp16.
 * x is fp32 (MINFER_ATTN_F32), fp16 or bf16, 16-byte aligned; y 2-byte aligned.  Replaces quant_cpu's Q8_0
 * case, which runs on the host (reference: csrc/quants/op.cpp:156-196, csrc/quants/impl.cpp:1169-1193), byte
 * for byte on fp32 input.
 */
int minfer_quant_q8_0(int src_dtype, const void* x, void* y, int64_t n_rows, int64_t k, void* stream);

/*
 * The inverse: y[i] = (T)(q[i] * (float)d), T fp32 (MINFER_ATTN_F32) or fp16; x 2-byte aligned, y 16-byte
 * aligned.  Replaces dequant_cuda's Q8_0 case and its kernel (reference: cuda/quants/op.cuh,
 * cuda/quants/kernel.cuh:10-40, cuda/quants/impls.cuh:121-143), bit for bit.
 */
int minfer_dequant_q8_0(int dst_dtype, const void* x, void* y, int64_t n_rows, int64_t k, void* stream);

/*
 * minfer_flash_attn_decode over Q8_0 caches: q and out are fp16 [B,Hq,1,D] with element strides st->q0, q1 and
 * st->o0, o1; k_cache and v_cache are [B,Hkv,Lmax] rows of D/32 blocks, 2-byte aligned, with st->kv0 and
 * st->kv1 the BYTE strides of their first two dims (even) and st->kv2 = D/32 * 34 (rows are dense).  The kernel
 * reads whole aligned 16-byte pieces, so up to 15 bytes on either side of a (sequence, head)'s rows, inside the
 * same 16-byte lines, are read and ignored (an aligned 16-byte line never straddles a page, so those bytes lie in pages
 * that hold bytes of the cache itself and the read cannot fault).  Every
 * block is dequantised to fp16 exactly as minfer_dequant_q8_0 does and the result is that of
 * minfer_flash_attn_decode on the dequantised cache; workspace as for minfer_flash_attn_decode.  This is what
 * the reference's unused (qtype_int, qblock_size, qtype_size) operator arguments are for (reference:
 * cuda/flash_attn/op.cuh:22-24); it has no kernel for it.
 */
int minfer_flash_attn_decode_q8_0(const void* q, const void* k_cache, const void* v_cache,
                                  const int32_t* ctx_lens, void* out, int64_t B, int64_t Hq, int64_t Hkv,
                                  int64_t Lmax, int64_t D, const minfer_attn_strides* st, void* workspace,
                                  size_t workspace_bytes, void* stream);

/*
 * minfer_flash_attn and minfer_flash_attn_varlen with k and v given as rows of Q8_0 blocks (prefill over a quantised
 * KV cache): q and out are fp16; k, v are [B,Hkv,L] (varlen: [1,Hkv,T]) rows of D/32 blocks, 2-byte aligned, with
 * st->kv0 and st->kv1 the BYTE strides of their first two dims (even) and st->kv2 = D/32 * 34 (rows dense), so a view of
 * the first L rows of a longer cache is accepted.  One pass dequantises k and v into the workspace exactly as
 * minfer_dequant_q8_0 does (every K/V row is read by many query tiles, so it is done once up front), then the fp16
 * kernel runs: the result is that of minfer_flash_attn / minfer_flash_attn_varlen on the dequantised rows, bit for
 * bit.  This is what the reference's unused (qtype_int, qblock_size, qtype_size) operator arguments are for
 * (reference: cuda/flash_attn/op.cuh:22-24); it has no kernel for it.  The workspace holds the mask classification
 * (dense call only) and the two fp16 copies.
 */
size_t minfer_flash_attn_q8_0_workspace_bytes(int64_t B, int64_t Hkv, int64_t L, int64_t D);
int minfer_flash_attn_q8_0(const void* q, const void* k, const void* v, const uint8_t* mask, void* out,
                           int64_t B, int64_t Hq, int64_t Hkv, int64_t L, int64_t D,
                           const minfer_attn_strides* st, void* workspace, size_t workspace_bytes, void* stream);
size_t minfer_flash_attn_varlen_q8_0_workspace_bytes(int64_t Hkv, int64_t T, int64_t D);
int minfer_flash_attn_varlen_q8_0(const void* q, const void* k, const void* v, const int32_t* cu_seqlens,
                                  int64_t n_seqs, int64_t max_seqlen, void* out, int64_t Hq, int64_t Hkv,
                                  int64_t T, int64_t D, const minfer_attn_strides* st, void* workspace,
                                  size_t workspace_bytes, void* stream);

/*
 * minfer_rope_kv_append into Q8_0 caches: q is rotated in place as there; the rotated k and v, rounded to
 * `dtype` as an fp16/bf16 cache would hold them, are quantised as minfer_quant_q8_0 does and written to row
 * positions[b] + l of caches laid out as minfer_flash_attn_decode_q8_0 reads them (cache_stride_b,
 * cache_stride_h in bytes, even; rows dense).  D must be a multiple of 32 and rotary_dim of 32 (interleaved)
 * or 64 (NeoX); q, k, v 16-byte aligned, caches 2-byte aligned.  No counterpart in the reference.
 */
int minfer_rope_kv_append_q8_0(int dtype, int style, void* q, const void* k, const void* v,
                               const int32_t* positions, void* k_cache, void* v_cache,
                               int64_t B, int64_t L, int64_t Hq, int64_t Hkv, int64_t D, int64_t Lmax,
                               int64_t cache_stride_b, int64_t cache_stride_h,
                               int64_t rotary_dim, double freq_base, void* stream);

/*
 * Calibration, not an operator (no counterpart in the reference): `workgroups` workgroups of 8 waves issue
 * 16 * iters v_mfma_f32_16x16x32 (f16 or bf16) each, the instruction the prefill and GEMM kernels are built on, back to
 * back on eight accumulator blocks, from 16 operand fragments (64 lanes x 16 bytes each, 16 KiB in all) that every wave
 * reads once from `operands`; 16 384 flop per instruction, i.e. workgroups * 8 * 8 * iters * 32768 flop per launch.
 * Timed by the caller, it gives the matrix rate the chip sustains on the caller's operand values (random values cost
 * more power than constant ones), the figure the attention and GEMM kernels' fractions of the nominal peak can be read
 * against.  minfer_calib_mfma_rate_32x32x16 issues 8 * iters v_mfma_f32_32x32x16 on four blocks instead (the same
 * flops): on random fp16 operands the chip sustains 15-18 % less of that instruction.  sink: workgroups * 512 floats.
 */
#define MINFER_CALIB_MFMA_OPERAND_BYTES 16384
#define MINFER_CALIB_MFMA_FLOP_PER_ITER (8 * 8 * 32768)   /* per workgroup */
int minfer_calib_mfma_rate(int dtype, const void* operands, int64_t iters, int64_t workgroups, float* sink, void* stream);
int minfer_calib_mfma_rate_32x32x16(int dtype, const void* operands, int64_t iters, int64_t workgroups, float* sink, void* stream);

/*
 * Calibration as well: the prefill kernel's per-tile instruction mix at head_dim 128 (64 MFMAs, 16 + 32 LDS fragment
 * reads, the softmax's maximum / exponential / pack / denominator instructions) on one K and one V tile that stay in
 * LDS, with no global memory traffic, barrier, mask or bookkeeping in the loop; `iters` tiles per wave, 32 * 32768
 * flop each, workgroups * 8 waves.  lds_reads = 0 keeps the fragments in registers, softmax = 0 feeds the second GEMM
 * from registers.  With both set this is the rate an attention kernel free of every fixed cost would reach on the
 * caller's operand values.  operands and sink as for minfer_calib_mfma_rate.  No counterpart in the reference.
 */
#define MINFER_CALIB_ATTN_MIX_FLOP_PER_ITER (8 * 32 * 32768)   /* per workgroup */
int minfer_calib_attn_mix(int dtype, const void* operands, int64_t iters, int64_t workgroups, int lds_reads, int softmax,
                          float* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MINFER_ATTN_H */
