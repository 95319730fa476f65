// PyTorch (stable ABI) registration of the attention operators, and of the normalisation, projection
// and rotary-embedding steps that feed them, in namespace `minfer`.
//
// This file is the only place where torch types appear: it validates tensors exactly as the
// reference host function does, turns them into pointers/strides and calls the C ABI of
// libminfer_attn.so (include/minfer_attn.h) on the current torch stream.  Loading the shared
// object as the Python module `_C` runs the static registrations, which is how the reference
// exposes its ops (reference: src/minfer/kernels/torch_ext/csrc/reg.cpp:7-33,
// src/minfer/kernels/torch_ext/csrc/cuda/reg.cu:16-27).
//
// Only the accelerator dispatch key gets an implementation: calling these ops with CPU tensors
// fails in the dispatcher instead of falling back to anything.
#include <Python.h>

#include <torch/csrc/inductor/aoti_torch/c/shim.h>
#include <torch/csrc/stable/accelerator.h>
#include <torch/csrc/stable/library.h>
#include <torch/csrc/stable/ops.h>
#include <torch/csrc/stable/tensor.h>
#include <torch/headeronly/core/ScalarType.h>
#include <torch/headeronly/util/Exception.h>

#include "minfer_attn.h"

extern "C" {
PyObject* PyInit__C(void) {
    static struct PyModuleDef module_def = {PyModuleDef_HEAD_INIT, "_C", NULL, -1, NULL};
    return PyModule_Create(&module_def);
}
}

namespace minfer {

using torch::headeronly::DeviceType;
using torch::headeronly::ScalarType;
using torch::stable::Tensor;

namespace {

void* current_stream() {
    auto device_index = torch::stable::accelerator::getCurrentDeviceIndex();
    void* stream = nullptr;
    TORCH_ERROR_CODE_CHECK(aoti_torch_get_current_cuda_stream(device_index, &stream));
    return stream;
}

bool on_gpu(const Tensor& t) { return t.device().type() == DeviceType::CUDA; }

int dtype_code(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& out, const char* op) {
    const ScalarType t = q.scalar_type();
    STD_TORCH_CHECK(t == ScalarType::Half || t == ScalarType::BFloat16, op, ": q must be float16 or bfloat16");
    STD_TORCH_CHECK(k.scalar_type() == t && v.scalar_type() == t && out.scalar_type() == t, op,
                    ": q, k, v and out must share one dtype");
    return t == ScalarType::Half ? MINFER_ATTN_F16 : MINFER_ATTN_BF16;
}

Tensor byte_workspace(const Tensor& like, size_t nbytes) {
    const int64_t n = (int64_t)nbytes;
    return torch::stable::new_empty(like, {n}, ScalarType::Byte);
}

void check_rc(int rc, const char* op) {
    STD_TORCH_CHECK(rc == MINFER_ATTN_OK, op, ": ", minfer_attn_last_error());
}

minfer_attn_strides strides_of(const Tensor& q, const Tensor& k, const Tensor& out) {
    return minfer_attn_strides{q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1),
                               k.stride(2), out.stride(0), out.stride(1), out.stride(2)};
}

}  // namespace

// Prefill over k and v given as Q8_0 blocks: uint8 [B, n_kv_heads, L, HEAD_DIM/32 * 34] (dims 0 and 1 may be strided,
// e.g. the first L rows of a longer cache), q and out float16.
static void flash_attn_q8_0(int64_t qblock_size, int64_t qtype_size, const Tensor& q, const Tensor& k, const Tensor& v,
                            Tensor& mask, Tensor& out) {
    STD_TORCH_CHECK(qblock_size == MINFER_Q8_0_BLOCK && qtype_size == MINFER_Q8_0_BLOCK_BYTES,
                    "flash_attn: Q8_0 has qblock_size 32 and qtype_size 34");
    STD_TORCH_CHECK(q.dim() == 4 && k.dim() == 4 && v.dim() == 4 && out.dim() == 4 && mask.dim() == 4,
                    "flash_attn: q, k, v, mask and out must be 4-D");
    STD_TORCH_CHECK(q.scalar_type() == ScalarType::Half && out.scalar_type() == ScalarType::Half,
                    "flash_attn: q and out must be float16 over Q8_0 k/v");
    STD_TORCH_CHECK(k.scalar_type() == ScalarType::Byte && v.scalar_type() == ScalarType::Byte, "flash_attn: Q8_0 k and v must be uint8");
    STD_TORCH_CHECK(q.stride(-1) == 1 && k.stride(-1) == 1 && v.stride(-1) == 1 && out.stride(-1) == 1,
                    "flash_attn: q, k, v and out must be contiguous in their last dimension");
    STD_TORCH_CHECK(k.stride(0) == v.stride(0) && k.stride(1) == v.stride(1) && k.stride(2) == v.stride(2),
                    "flash_attn: k and v must share strides");
    STD_TORCH_CHECK(mask.is_contiguous() && mask.scalar_type() == ScalarType::Bool, "flash_attn: mask must be contiguous bool");
    STD_TORCH_CHECK(q.sizes().equals(out.sizes()) && k.sizes().equals(v.sizes()), "flash_attn: q/out or k/v shapes differ");
    const int64_t B = q.size(0), Hq = q.size(1), Hkv = k.size(1), L = q.size(2), D = q.size(3);
    STD_TORCH_CHECK(D == 128 || D == 64, "flash_attn: head_dim must be 128 or 64");
    STD_TORCH_CHECK(B == k.size(0) && B == mask.size(0) && mask.size(1) == 1 && L == k.size(2) && L == mask.size(2) &&
                    L == mask.size(3) && k.size(3) == D / 32 * 34 && k.stride(2) == k.size(3),
                    "flash_attn: expected q [B,Hq,L,D], Q8_0 k/v [B,Hkv,L,D/32*34] with dense rows, mask [B,1,L,L]");
    if (B == 0 || L == 0) return;
    const minfer_attn_strides st = strides_of(q, k, out);   // a byte tensor's strides are byte strides
    const size_t ws_bytes = minfer_flash_attn_q8_0_workspace_bytes(B, Hkv, L, D);
    Tensor ws = byte_workspace(q, ws_bytes);
    check_rc(minfer_flash_attn_q8_0(q.const_data_ptr(), k.const_data_ptr(), v.const_data_ptr(),
                                    static_cast<const uint8_t*>(mask.const_data_ptr()), out.mutable_data_ptr(), B, Hq, Hkv, L, D,
                                    &st, ws.mutable_data_ptr(), ws_bytes, current_stream()),
             "flash_attn");
}

// Same signature, argument meaning and checks as the reference's flash_attn_cuda
// (reference: src/minfer/kernels/torch_ext/csrc/cuda/flash_attn/op.cuh:21-106); the dtype check
// also admits bfloat16 and head_dim may be 64 as well as 128.
void flash_attn_hip(int64_t qtype_int, int64_t qblock_size, int64_t qtype_size,
                    const Tensor& q,   // [B, n_heads, L, HEAD_DIM]
                    const Tensor& k,   // [B, n_kv_heads, L, HEAD_DIM]
                    const Tensor& v,   // [B, n_kv_heads, L, HEAD_DIM]
                    Tensor& mask,      // [B, 1, L, L] bool, True = attend
                    Tensor& out) {     // [B, n_heads, L, HEAD_DIM]
    // The reference leaves its three leading arguments unused; here (8, 32, 34) announces k and v as Q8_0 blocks,
    // any other value k and v of q's own type, as the reference's callers pass it (F16 = 1).
    STD_TORCH_CHECK(on_gpu(q) && on_gpu(k) && on_gpu(v) && on_gpu(mask) && on_gpu(out),
                    "flash_attn: all tensors must be on the GPU");
    if (qtype_int == MINFER_Q8_0) {
        flash_attn_q8_0(qblock_size, qtype_size, q, k, v, mask, out);
        return;
    }
    STD_TORCH_CHECK(k.scalar_type() != ScalarType::Byte, "flash_attn: byte k/v need qtype_int = 8 (Q8_0)");
    STD_TORCH_CHECK(q.dim() == 4 && k.dim() == 4 && v.dim() == 4 && out.dim() == 4 && mask.dim() == 4,
                    "flash_attn: q, k, v, mask and out must be 4-D");
    STD_TORCH_CHECK(q.stride(-1) == 1 && k.stride(-1) == 1 && v.stride(-1) == 1 && out.stride(-1) == 1,
                    "flash_attn: q, k, v and out must be contiguous in head_dim");
    STD_TORCH_CHECK(k.stride(0) == v.stride(0) && k.stride(1) == v.stride(1) && k.stride(2) == v.stride(2),
                    "flash_attn: k and v must share strides");
    STD_TORCH_CHECK(mask.is_contiguous(), "flash_attn: mask must be contiguous");
    const int dtype = dtype_code(q, k, v, out, "flash_attn");
    STD_TORCH_CHECK(mask.scalar_type() == ScalarType::Bool, "flash_attn: mask must be bool");
    STD_TORCH_CHECK(q.sizes().equals(out.sizes()), "flash_attn: q and out shapes differ");
    STD_TORCH_CHECK(k.sizes().equals(v.sizes()), "flash_attn: k and v shapes differ");
    STD_TORCH_CHECK(q.size(0) == k.size(0) && q.size(0) == mask.size(0) && mask.size(1) == 1 &&
                    q.size(2) == k.size(2) && q.size(2) == mask.size(2) && q.size(2) == mask.size(3) &&
                    q.size(3) == k.size(3),
                    "flash_attn: expected q [B,Hq,L,D], k/v [B,Hkv,L,D], mask [B,1,L,L]");
    const int64_t B = q.size(0), Hq = q.size(1), Hkv = k.size(1), L = q.size(2), D = q.size(3);
    STD_TORCH_CHECK(D == 128 || D == 64, "flash_attn: head_dim must be 128 (or 64)");
    if (B == 0 || L == 0) return;

    const minfer_attn_strides st = strides_of(q, k, out);
    const size_t ws_bytes = minfer_flash_attn_workspace_bytes(B, L);
    Tensor ws = byte_workspace(q, ws_bytes);
    check_rc(minfer_flash_attn(dtype, q.const_data_ptr(), k.const_data_ptr(), v.const_data_ptr(),
                               static_cast<const uint8_t*>(mask.const_data_ptr()), out.mutable_data_ptr(),
                               B, Hq, Hkv, L, D, &st, ws.mutable_data_ptr(), ws_bytes, current_stream()),
             "flash_attn");
}

// Decode over Q8_0 caches: uint8 [B, n_kv_heads, Lmax, HEAD_DIM/32 * 34], selected by the operator's
// (qtype_int, qblock_size, qtype_size) = (8, 32, 34) (reference: the unused leading arguments of
// flash_attn_cuda, cuda/flash_attn/op.cuh:22-24; sizes src/minfer/const.py:46).
static void flash_attn_decode_q8_0(int64_t qblock_size, int64_t qtype_size, const Tensor& q, const Tensor& k_cache,
                                   const Tensor& v_cache, const Tensor& ctx_lens, Tensor& out) {
    STD_TORCH_CHECK(qblock_size == MINFER_Q8_0_BLOCK && qtype_size == MINFER_Q8_0_BLOCK_BYTES,
                    "flash_attn_decode: Q8_0 has qblock_size 32 and qtype_size 34");
    STD_TORCH_CHECK(q.dim() == 4 && k_cache.dim() == 4 && v_cache.dim() == 4 && out.dim() == 4 && ctx_lens.dim() == 1,
                    "flash_attn_decode: q, k_cache, v_cache, out must be 4-D and ctx_lens 1-D");
    STD_TORCH_CHECK(q.scalar_type() == ScalarType::Half && out.scalar_type() == ScalarType::Half,
                    "flash_attn_decode: q and out must be float16 over Q8_0 caches");
    STD_TORCH_CHECK(k_cache.scalar_type() == ScalarType::Byte && v_cache.scalar_type() == ScalarType::Byte,
                    "flash_attn_decode: Q8_0 caches must be uint8");
    STD_TORCH_CHECK(q.stride(-1) == 1 && k_cache.stride(-1) == 1 && v_cache.stride(-1) == 1 && out.stride(-1) == 1,
                    "flash_attn_decode: tensors must be contiguous in their last dimension");
    STD_TORCH_CHECK(k_cache.stride(0) == v_cache.stride(0) && k_cache.stride(1) == v_cache.stride(1) &&
                    k_cache.stride(2) == v_cache.stride(2), "flash_attn_decode: k_cache and v_cache must share strides");
    STD_TORCH_CHECK(ctx_lens.scalar_type() == ScalarType::Int && ctx_lens.is_contiguous(),
                    "flash_attn_decode: ctx_lens must be contiguous int32");
    STD_TORCH_CHECK(q.sizes().equals(out.sizes()), "flash_attn_decode: q and out shapes differ");
    STD_TORCH_CHECK(k_cache.sizes().equals(v_cache.sizes()), "flash_attn_decode: cache shapes differ");
    const int64_t B = q.size(0), Hq = q.size(1), Hkv = k_cache.size(1), Lmax = k_cache.size(2), D = q.size(3);
    STD_TORCH_CHECK(D == 128 || D == 64, "flash_attn_decode: head_dim must be 128 or 64");
    STD_TORCH_CHECK(q.size(2) == 1 && B == k_cache.size(0) && B == ctx_lens.size(0) &&
                    k_cache.size(3) == D / 32 * 34 && k_cache.stride(2) == k_cache.size(3),
                    "flash_attn_decode: expected q [B,Hq,1,D], caches [B,Hkv,Lmax,D/32*34] with dense rows, ctx_lens [B]");
    if (B == 0) return;
    const minfer_attn_strides st = strides_of(q, k_cache, out);   // a byte tensor's strides are byte strides
    const size_t ws_bytes = minfer_flash_attn_decode_workspace_bytes(B, Hq, Lmax, D);
    Tensor ws = byte_workspace(q, ws_bytes);
    check_rc(minfer_flash_attn_decode_q8_0(q.const_data_ptr(), k_cache.const_data_ptr(), v_cache.const_data_ptr(),
                                           static_cast<const int32_t*>(ctx_lens.const_data_ptr()), out.mutable_data_ptr(),
                                           B, Hq, Hkv, Lmax, D, &st, ws.mutable_data_ptr(), ws_bytes, current_stream()),
             "flash_attn_decode");
}

// Decode over a KV cache laid out like the reference's cache (reference: src/minfer/core.py:105-127).
void flash_attn_decode_hip(int64_t qtype_int, int64_t qblock_size, int64_t qtype_size,
                           const Tensor& q,         // [B, n_heads, 1, HEAD_DIM]
                           const Tensor& k_cache,   // [B, n_kv_heads, Lmax, HEAD_DIM]
                           const Tensor& v_cache,   // [B, n_kv_heads, Lmax, HEAD_DIM]
                           const Tensor& ctx_lens,  // [B] int32
                           Tensor& out) {           // [B, n_heads, 1, HEAD_DIM]
    STD_TORCH_CHECK(on_gpu(q) && on_gpu(k_cache) && on_gpu(v_cache) && on_gpu(ctx_lens) && on_gpu(out),
                    "flash_attn_decode: all tensors must be on the GPU");
    if (qtype_int == MINFER_Q8_0) {
        flash_attn_decode_q8_0(qblock_size, qtype_size, q, k_cache, v_cache, ctx_lens, out);
        return;
    }
    // any other value describes caches of q's own type, as the reference's callers pass it (F16 = 1)
    STD_TORCH_CHECK(k_cache.scalar_type() != ScalarType::Byte, "flash_attn_decode: byte caches need qtype_int = 8 (Q8_0)");
    STD_TORCH_CHECK(q.dim() == 4 && k_cache.dim() == 4 && v_cache.dim() == 4 && out.dim() == 4 && ctx_lens.dim() == 1,
                    "flash_attn_decode: q, k_cache, v_cache, out must be 4-D and ctx_lens 1-D");
    STD_TORCH_CHECK(q.stride(-1) == 1 && k_cache.stride(-1) == 1 && v_cache.stride(-1) == 1 && out.stride(-1) == 1,
                    "flash_attn_decode: tensors must be contiguous in head_dim");
    STD_TORCH_CHECK(k_cache.stride(0) == v_cache.stride(0) && k_cache.stride(1) == v_cache.stride(1) &&
                    k_cache.stride(2) == v_cache.stride(2), "flash_attn_decode: k_cache and v_cache must share strides");
    const int dtype = dtype_code(q, k_cache, v_cache, out, "flash_attn_decode");
    STD_TORCH_CHECK(ctx_lens.scalar_type() == ScalarType::Int && ctx_lens.is_contiguous(),
                    "flash_attn_decode: ctx_lens must be contiguous int32");
    STD_TORCH_CHECK(q.sizes().equals(out.sizes()), "flash_attn_decode: q and out shapes differ");
    STD_TORCH_CHECK(k_cache.sizes().equals(v_cache.sizes()), "flash_attn_decode: cache shapes differ");
    STD_TORCH_CHECK(q.size(2) == 1 && q.size(0) == k_cache.size(0) && q.size(0) == ctx_lens.size(0) &&
                    q.size(3) == k_cache.size(3),
                    "flash_attn_decode: expected q [B,Hq,1,D], caches [B,Hkv,Lmax,D], ctx_lens [B]");
    const int64_t B = q.size(0), Hq = q.size(1), Hkv = k_cache.size(1), Lmax = k_cache.size(2), D = q.size(3);
    STD_TORCH_CHECK(D == 128 || D == 64, "flash_attn_decode: head_dim must be 128 or 64");
    if (B == 0) return;

    const minfer_attn_strides st = strides_of(q, k_cache, out);
    const size_t ws_bytes = minfer_flash_attn_decode_workspace_bytes(B, Hq, Lmax, D);
    Tensor ws = byte_workspace(q, ws_bytes);
    check_rc(minfer_flash_attn_decode(dtype, q.const_data_ptr(), k_cache.const_data_ptr(), v_cache.const_data_ptr(),
                                      static_cast<const int32_t*>(ctx_lens.const_data_ptr()), out.mutable_data_ptr(),
                                      B, Hq, Hkv, Lmax, D, &st, ws.mutable_data_ptr(), ws_bytes, current_stream()),
             "flash_attn_decode");
}

// Packed ragged causal prefill.
void flash_attn_varlen_hip(int64_t qtype_int, int64_t qblock_size, int64_t qtype_size,
                           const Tensor& q,           // [1, n_heads, T, HEAD_DIM]
                           const Tensor& k,           // [1, n_kv_heads, T, HEAD_DIM]
                           const Tensor& v,           // [1, n_kv_heads, T, HEAD_DIM]
                           const Tensor& cu_seqlens,  // [n_seqs + 1] int32
                           int64_t max_seqlen,
                           Tensor& out) {             // [1, n_heads, T, HEAD_DIM]
    STD_TORCH_CHECK(on_gpu(q) && on_gpu(k) && on_gpu(v) && on_gpu(cu_seqlens) && on_gpu(out),
                    "flash_attn_varlen: all tensors must be on the GPU");
    STD_TORCH_CHECK(q.dim() == 4 && k.dim() == 4 && v.dim() == 4 && out.dim() == 4 && cu_seqlens.dim() == 1,
                    "flash_attn_varlen: q, k, v, out must be 4-D and cu_seqlens 1-D");
    if (qtype_int == MINFER_Q8_0) {   // k and v as Q8_0 blocks: uint8 [1, n_kv_heads, T, HEAD_DIM/32 * 34], q and out float16
        STD_TORCH_CHECK(qblock_size == MINFER_Q8_0_BLOCK && qtype_size == MINFER_Q8_0_BLOCK_BYTES,
                        "flash_attn_varlen: Q8_0 has qblock_size 32 and qtype_size 34");
        STD_TORCH_CHECK(q.scalar_type() == ScalarType::Half && out.scalar_type() == ScalarType::Half &&
                        k.scalar_type() == ScalarType::Byte && v.scalar_type() == ScalarType::Byte,
                        "flash_attn_varlen: over Q8_0 k/v, q and out must be float16 and k, v uint8");
        STD_TORCH_CHECK(q.stride(-1) == 1 && k.stride(-1) == 1 && v.stride(-1) == 1 && out.stride(-1) == 1 &&
                        k.stride(1) == v.stride(1) && k.stride(2) == v.stride(2),
                        "flash_attn_varlen: tensors must be contiguous in their last dimension, k and v share strides");
        STD_TORCH_CHECK(cu_seqlens.scalar_type() == ScalarType::Int && cu_seqlens.is_contiguous() && cu_seqlens.size(0) >= 1,
                        "flash_attn_varlen: cu_seqlens must be contiguous int32 with at least one entry");
        STD_TORCH_CHECK(q.sizes().equals(out.sizes()) && k.sizes().equals(v.sizes()), "flash_attn_varlen: q/out or k/v shapes differ");
        const int64_t Hq8 = q.size(1), Hkv8 = k.size(1), T8 = q.size(2), D8 = q.size(3);
        STD_TORCH_CHECK(D8 == 128 || D8 == 64, "flash_attn_varlen: head_dim must be 128 or 64");
        STD_TORCH_CHECK(q.size(0) == 1 && k.size(0) == 1 && T8 == k.size(2) && k.size(3) == D8 / 32 * 34 && k.stride(2) == k.size(3),
                        "flash_attn_varlen: expected q [1,Hq,T,D], Q8_0 k/v [1,Hkv,T,D/32*34] with dense rows");
        const int64_t n8 = cu_seqlens.size(0) - 1;
        if (n8 == 0 || T8 == 0) return;
        const minfer_attn_strides st8 = strides_of(q, k, out);
        const size_t ws_bytes = minfer_flash_attn_varlen_q8_0_workspace_bytes(Hkv8, T8, D8);
        Tensor ws = byte_workspace(q, ws_bytes);
        check_rc(minfer_flash_attn_varlen_q8_0(q.const_data_ptr(), k.const_data_ptr(), v.const_data_ptr(),
                                               static_cast<const int32_t*>(cu_seqlens.const_data_ptr()), n8, max_seqlen,
                                               out.mutable_data_ptr(), Hq8, Hkv8, T8, D8, &st8, ws.mutable_data_ptr(), ws_bytes,
                                               current_stream()),
                 "flash_attn_varlen");
        return;
    }
    STD_TORCH_CHECK(k.scalar_type() != ScalarType::Byte, "flash_attn_varlen: byte k/v need qtype_int = 8 (Q8_0)");
    STD_TORCH_CHECK(q.stride(-1) == 1 && k.stride(-1) == 1 && v.stride(-1) == 1 && out.stride(-1) == 1,
                    "flash_attn_varlen: tensors must be contiguous in head_dim");
    STD_TORCH_CHECK(k.stride(1) == v.stride(1) && k.stride(2) == v.stride(2), "flash_attn_varlen: k and v must share strides");
    const int dtype = dtype_code(q, k, v, out, "flash_attn_varlen");
    STD_TORCH_CHECK(cu_seqlens.scalar_type() == ScalarType::Int && cu_seqlens.is_contiguous() && cu_seqlens.size(0) >= 1,
                    "flash_attn_varlen: cu_seqlens must be contiguous int32 with at least one entry");
    STD_TORCH_CHECK(q.sizes().equals(out.sizes()), "flash_attn_varlen: q and out shapes differ");
    STD_TORCH_CHECK(k.sizes().equals(v.sizes()), "flash_attn_varlen: k and v shapes differ");
    STD_TORCH_CHECK(q.size(0) == 1 && k.size(0) == 1 && q.size(2) == k.size(2) && q.size(3) == k.size(3),
                    "flash_attn_varlen: expected q [1,Hq,T,D], k/v [1,Hkv,T,D]");
    const int64_t Hq = q.size(1), Hkv = k.size(1), T = q.size(2), D = q.size(3);
    STD_TORCH_CHECK(D == 128 || D == 64, "flash_attn_varlen: head_dim must be 128 or 64");
    const int64_t n_seqs = cu_seqlens.size(0) - 1;
    if (n_seqs == 0 || T == 0) return;

    const minfer_attn_strides st = strides_of(q, k, out);
    check_rc(minfer_flash_attn_varlen(dtype, q.const_data_ptr(), k.const_data_ptr(), v.const_data_ptr(),
                                      static_cast<const int32_t*>(cu_seqlens.const_data_ptr()), n_seqs, max_seqlen,
                                      out.mutable_data_ptr(), Hq, Hkv, T, D, &st, current_stream()),
             "flash_attn_varlen");
}

// Rotary embedding in place, same signature, argument meaning and checks as the reference's il_rope_cuda /
// neox_rope_cuda (reference: src/minfer/kernels/torch_ext/csrc/cuda/il_rope/op.cuh:20-58 and
// neox_rope/op.cuh); bfloat16 is admitted as well.
namespace {
void rope_hip(int style, const char* op, int64_t rotary_dim, int64_t start_pos, double freq_base,
              Tensor& x) {   // [B, L, n_heads, head_dim] (before the transpose for flash_attn)
    STD_TORCH_CHECK(on_gpu(x), op, ": x must be on the GPU");
    STD_TORCH_CHECK(x.is_contiguous(), op, ": x must be contiguous");
    STD_TORCH_CHECK(x.dim() == 4, op, ": x must be 4-D");
    const ScalarType t = x.scalar_type();
    STD_TORCH_CHECK(t == ScalarType::Half || t == ScalarType::BFloat16, op, ": x must be float16 or bfloat16");
    STD_TORCH_CHECK(rotary_dim <= x.size(3), op, ": rotary_dim exceeds head_dim");
    check_rc(minfer_rope(t == ScalarType::Half ? MINFER_ATTN_F16 : MINFER_ATTN_BF16, style, x.mutable_data_ptr(),
                         x.size(0), x.size(1), x.size(2), x.size(3), rotary_dim, start_pos, freq_base,
                         current_stream()),
             op);
}
}  // namespace

void il_rope_hip(int64_t rotary_dim, int64_t start_pos, double freq_base, Tensor& x) {
    rope_hip(MINFER_ROPE_INTERLEAVED, "il_rope", rotary_dim, start_pos, freq_base, x);
}

void neox_rope_hip(int64_t rotary_dim, int64_t start_pos, double freq_base, Tensor& x) {
    rope_hip(MINFER_ROPE_NEOX, "neox_rope", rotary_dim, start_pos, freq_base, x);
}

// rope(q) in place, rope(k) -> k_cache, v -> v_cache in one pass: the step before attention
// (reference: src/minfer/core.py:228-232) writing the reference's cache layout (core.py:105-127).
void rope_kv_append_hip(int64_t style, int64_t rotary_dim, double freq_base,
                        Tensor& q,                 // [B, L, n_heads, head_dim], rotated in place
                        const Tensor& k,           // [B, L, n_kv_heads, head_dim]
                        const Tensor& v,           // [B, L, n_kv_heads, head_dim]
                        const Tensor& positions,   // [B] int32: rows each sequence already holds
                        Tensor& k_cache,           // [B, n_kv_heads, Lmax, head_dim]
                        Tensor& v_cache) {
    STD_TORCH_CHECK(on_gpu(q) && on_gpu(k) && on_gpu(v) && on_gpu(positions) && on_gpu(k_cache) && on_gpu(v_cache),
                    "rope_kv_append: all tensors must be on the GPU");
    STD_TORCH_CHECK(q.dim() == 4 && k.dim() == 4 && v.dim() == 4 && k_cache.dim() == 4 && v_cache.dim() == 4 && positions.dim() == 1,
                    "rope_kv_append: q, k, v and the caches must be 4-D and positions 1-D");
    STD_TORCH_CHECK(q.is_contiguous() && k.is_contiguous() && v.is_contiguous(), "rope_kv_append: q, k and v must be contiguous");
    STD_TORCH_CHECK(style == MINFER_ROPE_INTERLEAVED || style == MINFER_ROPE_NEOX, "rope_kv_append: style must be 0 (interleaved) or 1 (NeoX)");
    const bool q8 = k_cache.scalar_type() == ScalarType::Byte;   // Q8_0 caches: [B, n_kv_heads, Lmax, head_dim/32 * 34] bytes
    const int dtype = dtype_code(q, k, v, q8 ? q : k_cache, "rope_kv_append");
    STD_TORCH_CHECK(v_cache.scalar_type() == k_cache.scalar_type(), "rope_kv_append: caches must share q's dtype, or both be uint8 (Q8_0)");
    STD_TORCH_CHECK(positions.scalar_type() == ScalarType::Int && positions.is_contiguous(), "rope_kv_append: positions must be contiguous int32");
    STD_TORCH_CHECK(k.sizes().equals(v.sizes()) && k_cache.sizes().equals(v_cache.sizes()), "rope_kv_append: k/v or cache shapes differ");
    STD_TORCH_CHECK(k_cache.stride(-1) == 1 && v_cache.stride(-1) == 1 && k_cache.stride(0) == v_cache.stride(0) &&
                    k_cache.stride(1) == v_cache.stride(1) && k_cache.stride(2) == v_cache.stride(2),
                    "rope_kv_append: caches must be contiguous in head_dim and share strides");
    STD_TORCH_CHECK(q.size(0) == k.size(0) && q.size(1) == k.size(1) && q.size(3) == k.size(3) && q.size(0) == k_cache.size(0) &&
                    k.size(2) == k_cache.size(1) && positions.size(0) == q.size(0) &&
                    k_cache.size(3) == (q8 ? q.size(3) / 32 * 34 : q.size(3)) && (!q8 || q.size(3) % 32 == 0),
                    "rope_kv_append: expected q [B,L,Hq,D], k/v [B,L,Hkv,D], caches [B,Hkv,Lmax,D] (or [B,Hkv,Lmax,D/32*34] bytes), positions [B]");
    STD_TORCH_CHECK(rotary_dim <= q.size(3), "rope_kv_append: rotary_dim exceeds head_dim");
    if (q8) {
        STD_TORCH_CHECK(k_cache.stride(2) == k_cache.size(3), "rope_kv_append: Q8_0 cache rows must be dense");
        check_rc(minfer_rope_kv_append_q8_0(dtype, (int)style, q.mutable_data_ptr(), k.const_data_ptr(), v.const_data_ptr(),
                                            static_cast<const int32_t*>(positions.const_data_ptr()), k_cache.mutable_data_ptr(),
                                            v_cache.mutable_data_ptr(), q.size(0), q.size(1), q.size(2), k.size(2), q.size(3),
                                            k_cache.size(2), k_cache.stride(0), k_cache.stride(1), rotary_dim, freq_base,
                                            current_stream()),
                 "rope_kv_append");
        return;
    }
    check_rc(minfer_rope_kv_append(dtype, (int)style, q.mutable_data_ptr(), k.const_data_ptr(), v.const_data_ptr(),
                                   static_cast<const int32_t*>(positions.const_data_ptr()), k_cache.mutable_data_ptr(),
                                   v_cache.mutable_data_ptr(), q.size(0), q.size(1), q.size(2), k.size(2), q.size(3),
                                   k_cache.size(2), k_cache.stride(0), k_cache.stride(1), k_cache.stride(2), rotary_dim,
                                   freq_base, current_stream()),
             "rope_kv_append");
}

// The same producer with the optional per-head normalisation of q and k in front of the rotation
// (reference: src/minfer/core.py:224-230: rmsnorm(q), rmsnorm(k), then the two rope calls).
void rope_kv_append_norm_hip(int64_t style, int64_t rotary_dim, double freq_base, double eps,
                             Tensor& q,                 // [B, L, n_heads, head_dim], normalised and rotated in place
                             const Tensor& k,           // [B, L, n_kv_heads, head_dim]
                             const Tensor& v,           // [B, L, n_kv_heads, head_dim]
                             const Tensor& wq_norm,     // [head_dim]
                             const Tensor& wk_norm,     // [head_dim]
                             const Tensor& positions,   // [B] int32
                             Tensor& k_cache,           // [B, n_kv_heads, Lmax, head_dim] (or Q8_0 bytes)
                             Tensor& v_cache) {
    STD_TORCH_CHECK(on_gpu(q) && on_gpu(k) && on_gpu(v) && on_gpu(wq_norm) && on_gpu(wk_norm) && on_gpu(positions) &&
                    on_gpu(k_cache) && on_gpu(v_cache), "rope_kv_append_norm: all tensors must be on the GPU");
    STD_TORCH_CHECK(q.dim() == 4 && k.dim() == 4 && v.dim() == 4 && k_cache.dim() == 4 && v_cache.dim() == 4 &&
                    positions.dim() == 1 && wq_norm.dim() == 1 && wk_norm.dim() == 1,
                    "rope_kv_append_norm: q, k, v and the caches must be 4-D, positions and the norm weights 1-D");
    STD_TORCH_CHECK(q.is_contiguous() && k.is_contiguous() && v.is_contiguous() && wq_norm.is_contiguous() && wk_norm.is_contiguous(),
                    "rope_kv_append_norm: q, k, v and the norm weights must be contiguous");
    STD_TORCH_CHECK(style == MINFER_ROPE_INTERLEAVED || style == MINFER_ROPE_NEOX, "rope_kv_append_norm: style must be 0 (interleaved) or 1 (NeoX)");
    const bool q8 = k_cache.scalar_type() == ScalarType::Byte;
    const int dtype = dtype_code(q, k, v, q8 ? q : k_cache, "rope_kv_append_norm");
    STD_TORCH_CHECK(wq_norm.scalar_type() == q.scalar_type() && wk_norm.scalar_type() == q.scalar_type(),
                    "rope_kv_append_norm: norm weights must have q's dtype");
    STD_TORCH_CHECK(v_cache.scalar_type() == k_cache.scalar_type(), "rope_kv_append_norm: caches must share q's dtype, or both be uint8 (Q8_0)");
    STD_TORCH_CHECK(positions.scalar_type() == ScalarType::Int && positions.is_contiguous(), "rope_kv_append_norm: positions must be contiguous int32");
    STD_TORCH_CHECK(k.sizes().equals(v.sizes()) && k_cache.sizes().equals(v_cache.sizes()), "rope_kv_append_norm: k/v or cache shapes differ");
    STD_TORCH_CHECK(k_cache.stride(-1) == 1 && v_cache.stride(-1) == 1 && k_cache.stride(0) == v_cache.stride(0) &&
                    k_cache.stride(1) == v_cache.stride(1) && k_cache.stride(2) == v_cache.stride(2),
                    "rope_kv_append_norm: caches must be contiguous in head_dim and share strides");
    STD_TORCH_CHECK(q.size(0) == k.size(0) && q.size(1) == k.size(1) && q.size(3) == k.size(3) && q.size(0) == k_cache.size(0) &&
                    k.size(2) == k_cache.size(1) && positions.size(0) == q.size(0) && wq_norm.size(0) == q.size(3) &&
                    wk_norm.size(0) == q.size(3) && k_cache.size(3) == (q8 ? q.size(3) / 32 * 34 : q.size(3)),
                    "rope_kv_append_norm: expected q [B,L,Hq,D], k/v [B,L,Hkv,D], weights [D], caches [B,Hkv,Lmax,D] (or [B,Hkv,Lmax,D/32*34] bytes), positions [B]");
    STD_TORCH_CHECK(rotary_dim <= q.size(3), "rope_kv_append_norm: rotary_dim exceeds head_dim");
    check_rc(minfer_rope_kv_append_norm(dtype, (int)style, q8 ? MINFER_Q8_0 : dtype, q.mutable_data_ptr(), k.const_data_ptr(),
                                        v.const_data_ptr(), wq_norm.const_data_ptr(), wk_norm.const_data_ptr(), eps,
                                        static_cast<const int32_t*>(positions.const_data_ptr()), k_cache.mutable_data_ptr(),
                                        v_cache.mutable_data_ptr(), q.size(0), q.size(1), q.size(2), k.size(2), q.size(3),
                                        k_cache.size(2), k_cache.stride(0), k_cache.stride(1), k_cache.stride(2), rotary_dim,
                                        freq_base, current_stream()),
             "rope_kv_append_norm");
}

// Same signature, argument meaning and checks as the reference's rmsnorm_cuda
// (reference: src/minfer/kernels/torch_ext/csrc/cuda/rmsnorm/op.cuh:20-70); bfloat16 is admitted as well.
void rmsnorm_hip(double eps,
                 const Tensor& in,   // [B, L, hidden] or [B, L, n_heads, head_dim]
                 const Tensor& w,    // [dim]: the vector length that is normalised
                 Tensor& out) {      // same shape as in
    STD_TORCH_CHECK(on_gpu(in) && on_gpu(w) && on_gpu(out), "rmsnorm: all tensors must be on the GPU");
    STD_TORCH_CHECK(in.is_contiguous() && out.is_contiguous() && w.is_contiguous(), "rmsnorm: tensors must be contiguous");
    const ScalarType t = in.scalar_type();
    STD_TORCH_CHECK(t == ScalarType::Half || t == ScalarType::BFloat16, "rmsnorm: input must be float16 or bfloat16");
    STD_TORCH_CHECK(out.scalar_type() == t && w.scalar_type() == t, "rmsnorm: input, w and out must share one dtype");
    STD_TORCH_CHECK(in.dim() == 3 || in.dim() == 4, "rmsnorm: input must be 3-D or 4-D");
    STD_TORCH_CHECK(in.sizes().equals(out.sizes()), "rmsnorm: input and out shapes differ");
    STD_TORCH_CHECK(w.dim() == 1 && w.size(0) > 0 && (in.size(-1) == w.size(0) || in.size(-1) % w.size(0) == 0),
                    "rmsnorm: the last dimension must be a multiple of the weight length");
    const int64_t dim = w.size(0);
    check_rc(minfer_rmsnorm(t == ScalarType::Half ? MINFER_ATTN_F16 : MINFER_ATTN_BF16, in.const_data_ptr(), w.const_data_ptr(),
                            out.mutable_data_ptr(), in.numel() / dim, dim, eps, current_stream()),
             "rmsnorm");
}

// D = alpha * A B + beta * C.  Same signature, argument meaning and checks as the reference's gemm_cuda for
// 16-bit weights (reference: src/minfer/kernels/torch_ext/csrc/cuda/gemm/op.cuh:218-297): B stored [in_dim,
// out_dim] selects A B, B stored [out_dim, in_dim] selects A B^T (the first wins when both fit, as there).
// Quantised (byte) weights are not implemented here.  bfloat16 is admitted as well.
void gemm_hip(int64_t qtype_int, int64_t qblock_size, int64_t qtype_size, double alpha, double beta,
              const Tensor& A,   // [B, L, in_dim]
              const Tensor& B,   // [in_dim, out_dim] or [out_dim, in_dim]
              const Tensor& C,   // [B, L, out_dim]
              Tensor& D) {       // [B, L, out_dim]
    STD_TORCH_CHECK(qtype_int == 1 || qtype_int == 30 || qtype_int == 8,
                    "gemm: weights must be 16-bit (qtype F16 = 1, BF16 = 30) or Q8_0 blocks (qtype 8)");
    STD_TORCH_CHECK(on_gpu(A) && on_gpu(B) && on_gpu(C) && on_gpu(D), "gemm: all tensors must be on the GPU");
    if (qtype_int == 8) {
        // B [out_dim, in_dim / 32 * 34] bytes: alpha * A B^T + beta * C over the dequantised weight (reference:
        // gemm/op.cuh:299-312 routes this case to dispatch_quant_abt, which is empty there)
        STD_TORCH_CHECK(qblock_size == 32 && qtype_size == 34, "gemm: Q8_0 is (qblock_size, qtype_size) = (32, 34)");
        STD_TORCH_CHECK(A.scalar_type() == ScalarType::Half && C.scalar_type() == ScalarType::Half && D.scalar_type() == ScalarType::Half,
                        "gemm: A, C and D must be float16 with a Q8_0 weight");
        STD_TORCH_CHECK(B.scalar_type() == ScalarType::Byte, "gemm: a Q8_0 weight is a uint8 tensor");
        STD_TORCH_CHECK(A.dim() == 3 && B.dim() == 2 && C.dim() == 3 && D.dim() == 3, "gemm: A, C, D must be 3-D and B 2-D");
        STD_TORCH_CHECK(A.is_contiguous() && B.is_contiguous() && C.is_contiguous() && D.is_contiguous(), "gemm: tensors must be contiguous");
        const int64_t K = A.size(-1), M = A.numel() / (K > 0 ? K : 1), N = B.size(0);
        STD_TORCH_CHECK(K % 32 == 0, "gemm: in_dim must be a multiple of the block size");
        STD_TORCH_CHECK(B.size(1) == K / 32 * 34, "Unsupported dims for quant matmul");
        STD_TORCH_CHECK(A.size(0) * A.size(1) == C.size(0) * C.size(1) && C.size(-1) == N, "gemm: C does not have the shape of A B^T");
        STD_TORCH_CHECK(C.sizes().equals(D.sizes()), "gemm: C and D shapes differ");
        STD_TORCH_CHECK(alpha != 0.0, "gemm: alpha must not be 0");
        size_t ws_bytes = minfer_gemm_q8_0_workspace_bytes(M, N, K);
        // a view that starts off a 16-byte boundary cannot feed the kernel that streams the blocks: such a call goes
        // through the dequantised weight like the shapes that kernel does not take
        const auto misaligned = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) != 0; };
        if (ws_bytes == 0 && (misaligned(A.const_data_ptr()) || misaligned(D.const_data_ptr()) || (beta != 0.0 && misaligned(C.const_data_ptr()))))
            ws_bytes = ((static_cast<size_t>(N) * static_cast<size_t>(K) * 2 + 255) & ~static_cast<size_t>(255)) + minfer_gemm_workspace_bytes(M, N, K);
        Tensor ws = byte_workspace(A, ws_bytes);
        check_rc(minfer_gemm_q8_0(A.const_data_ptr(), B.const_data_ptr(), C.const_data_ptr(), D.mutable_data_ptr(), M, N, K, K, N, N,
                                  alpha, beta, ws_bytes ? ws.mutable_data_ptr() : nullptr, ws_bytes, current_stream()),
                 "gemm");
        return;
    }
    (void)qblock_size; (void)qtype_size;
    const ScalarType t = A.scalar_type();
    STD_TORCH_CHECK(t == ScalarType::Half || t == ScalarType::BFloat16, "gemm: A must be float16 or bfloat16");
    STD_TORCH_CHECK(B.scalar_type() == t && C.scalar_type() == t && D.scalar_type() == t, "gemm: A, B, C and D must share one dtype");
    STD_TORCH_CHECK(A.dim() == 3 && B.dim() == 2 && C.dim() == 3 && D.dim() == 3, "gemm: A, C, D must be 3-D and B 2-D");
    STD_TORCH_CHECK(A.is_contiguous() && B.is_contiguous() && C.is_contiguous() && D.is_contiguous(), "gemm: tensors must be contiguous");
    const int64_t K = A.size(-1), M = A.numel() / (K > 0 ? K : 1);
    STD_TORCH_CHECK(B.size(0) == K || B.size(1) == K, "gemm: A and B cannot be multiplied");
    const bool kn = B.size(0) == K;
    const int64_t N = kn ? B.size(1) : B.size(0);
    STD_TORCH_CHECK(A.size(0) * A.size(1) == C.size(0) * C.size(1) && C.size(-1) == N, "gemm: C does not have the shape of A B");
    STD_TORCH_CHECK(C.sizes().equals(D.sizes()), "gemm: C and D shapes differ");
    STD_TORCH_CHECK(alpha != 0.0, "gemm: alpha must not be 0");
    // a few dozen rows against a wide weight run as K slices that meet in a workspace
    const size_t ws_bytes = minfer_gemm_workspace_bytes(M, N, K);
    Tensor ws = byte_workspace(A, ws_bytes);
    check_rc(minfer_gemm_ws(t == ScalarType::Half ? MINFER_ATTN_F16 : MINFER_ATTN_BF16, kn ? MINFER_GEMM_B_KN : MINFER_GEMM_B_NK,
                            A.const_data_ptr(), B.const_data_ptr(), C.const_data_ptr(), D.mutable_data_ptr(), M, N, K, K,
                            kn ? N : K, N, N, alpha, beta, ws_bytes ? ws.mutable_data_ptr() : nullptr, ws_bytes, current_stream()),
             "gemm");
}

// q_out = x wq^T, k_out = x wk^T, v_out = x wv^T.  The reference's op of this name and signature is a stub
// (reference: src/minfer/kernels/torch_ext/csrc/cuda/qkv/op.cuh:21-34); what it must compute is fixed by its test
// (reference: test/kernels.py:173-214): weights stored [out_dim, hidden_dim].  A weight stored
// [hidden_dim, out_dim] (the layout the stub's comments name) is accepted when its shape says so unambiguously.
void qkv_hip(int64_t q_qtype_int, int64_t k_qtype_int, int64_t v_qtype_int, int64_t q_qblock_size, int64_t k_qblock_size,
             int64_t v_qblock_size, int64_t q_qtype_size, int64_t k_qtype_size, int64_t v_qtype_size,
             const Tensor& x,    // [B, L, hidden_dim]
             const Tensor& wq,   // [q_dim, hidden_dim]
             const Tensor& wk,   // [kv_dim, hidden_dim]
             const Tensor& wv,   // [kv_dim, hidden_dim]
             Tensor& q_out,      // [B, L, q_dim]
             Tensor& k_out,      // [B, L, kv_dim]
             Tensor& v_out) {    // [B, L, kv_dim]
    const int64_t qtypes[3] = {q_qtype_int, k_qtype_int, v_qtype_int};
    const int64_t qblocks[3] = {q_qblock_size, k_qblock_size, v_qblock_size}, qsizes[3] = {q_qtype_size, k_qtype_size, v_qtype_size};
    const ScalarType t = x.scalar_type();
    STD_TORCH_CHECK(t == ScalarType::Half || t == ScalarType::BFloat16, "qkv: x must be float16 or bfloat16");
    STD_TORCH_CHECK(x.dim() == 3 && x.is_contiguous() && on_gpu(x), "qkv: x must be a contiguous 3-D GPU tensor");
    const int64_t K = x.size(-1), M = x.numel() / (K > 0 ? K : 1);
    const int dtype = t == ScalarType::Half ? MINFER_ATTN_F16 : MINFER_ATTN_BF16;
    void* stream = current_stream();
    const Tensor* ws[3] = {&wq, &wk, &wv};
    Tensor* outs[3] = {&q_out, &k_out, &v_out};
    const char* names[3] = {"qkv: q", "qkv: k", "qkv: v"};
    if (qtypes[0] == MINFER_Q8_0 || qtypes[1] == MINFER_Q8_0 || qtypes[2] == MINFER_Q8_0) {
        // weights as rows of Q8_0 blocks, uint8 [out_dim, hidden_dim / 32 * 34] (each may also be 16-bit): one projection per weight
        STD_TORCH_CHECK(t == ScalarType::Half, "qkv: x must be float16 with a Q8_0 weight");
        STD_TORCH_CHECK(K % 32 == 0, "qkv: hidden_dim must be a multiple of the block size");
        // one workspace, sized for the projection that needs most, serves the three calls one after the other (they run
        // in stream order): the dequantised weight of a Q8_0 projection with many rows, the K slices of a 16-bit one
        size_t ws_max = 0;
        for (int i = 0; i < 3; ++i) {
            const int64_t N = outs[i]->dim() == 3 ? outs[i]->size(-1) : 0;
            const size_t need = qtypes[i] == MINFER_Q8_0 ? minfer_gemm_q8_0_workspace_bytes(M, N, K) : minfer_gemm_workspace_bytes(M, N, K);
            ws_max = need > ws_max ? need : ws_max;
        }
        Tensor wsp = byte_workspace(x, ws_max);
        void* wsp_ptr = ws_max ? wsp.mutable_data_ptr() : nullptr;
        for (int i = 0; i < 3; ++i) {
            const Tensor& w = *ws[i];
            Tensor& o = *outs[i];
            STD_TORCH_CHECK(on_gpu(w) && on_gpu(o) && o.scalar_type() == t, names[i], ": dtype or device mismatch");
            STD_TORCH_CHECK(w.dim() == 2 && o.dim() == 3 && w.is_contiguous() && o.is_contiguous(), names[i], ": weight must be contiguous 2-D, output contiguous 3-D");
            STD_TORCH_CHECK(o.size(0) == x.size(0) && o.size(1) == x.size(1), names[i], ": output must be [B, L, out_dim]");
            const int64_t N = o.size(-1);
            if (qtypes[i] == MINFER_Q8_0) {
                STD_TORCH_CHECK(qblocks[i] == MINFER_Q8_0_BLOCK && qsizes[i] == MINFER_Q8_0_BLOCK_BYTES, names[i], ": Q8_0 is (qblock_size, qtype_size) = (32, 34)");
                STD_TORCH_CHECK(w.scalar_type() == ScalarType::Byte && w.size(0) == N && w.size(1) == K / 32 * 34, names[i],
                                ": a Q8_0 weight is uint8 [out_dim, hidden_dim / 32 * 34]");
                check_rc(minfer_gemm_q8_0(x.const_data_ptr(), w.const_data_ptr(), nullptr, o.mutable_data_ptr(), M, N, K, K, N, N, 1.0, 0.0,
                                          wsp_ptr, ws_max, stream),
                         names[i]);
            } else {
                STD_TORCH_CHECK(qtypes[i] == 1 && w.scalar_type() == t && w.size(0) == N && w.size(1) == K, names[i],
                                ": next to a Q8_0 weight, a 16-bit weight must be float16 [out_dim, hidden_dim]");
                check_rc(minfer_gemm_ws(dtype, MINFER_GEMM_B_NK, x.const_data_ptr(), w.const_data_ptr(), nullptr, o.mutable_data_ptr(), M, N, K, K, K, N, N,
                                        1.0, 0.0, wsp_ptr, ws_max, stream),
                         names[i]);
            }
        }
        return;
    }
    STD_TORCH_CHECK((q_qtype_int == 1 || q_qtype_int == 30) && k_qtype_int == q_qtype_int && v_qtype_int == q_qtype_int,
                    "qkv: weights must be 16-bit (qtype F16 = 1, BF16 = 30), all alike, or Q8_0 blocks (qtype 8)");
    bool all_nk = true;
    for (int i = 0; i < 3; ++i) {
        const Tensor& w = *ws[i];
        Tensor& o = *outs[i];
        STD_TORCH_CHECK(on_gpu(w) && on_gpu(o) && w.scalar_type() == t && o.scalar_type() == t, names[i], ": dtype or device mismatch");
        STD_TORCH_CHECK(w.dim() == 2 && o.dim() == 3 && w.is_contiguous() && o.is_contiguous(), names[i], ": weight must be contiguous 2-D, output contiguous 3-D");
        const int64_t N = o.size(-1);
        STD_TORCH_CHECK(o.size(0) == x.size(0) && o.size(1) == x.size(1), names[i], ": output must be [B, L, out_dim]");
        const bool nk = w.size(0) == N && w.size(1) == K;
        STD_TORCH_CHECK(nk || (w.size(0) == K && w.size(1) == N), names[i], ": weight must be [out_dim, hidden_dim] (or [hidden_dim, out_dim])");
        all_nk = all_nk && nk;
    }
    if (all_nk) {   // the reference's layout: one launch for the three projections
        const int64_t Nq = q_out.size(-1), Nk = k_out.size(-1), Nv = v_out.size(-1);
        check_rc(minfer_qkv(dtype, x.const_data_ptr(), wq.const_data_ptr(), wk.const_data_ptr(), wv.const_data_ptr(),
                            q_out.mutable_data_ptr(), k_out.mutable_data_ptr(), v_out.mutable_data_ptr(), M, K, Nq, Nk, Nv,
                            K, K, K, K, Nq, Nk, Nv, stream),
                 "qkv");
        return;
    }
    for (int i = 0; i < 3; ++i) {
        const Tensor& w = *ws[i];
        Tensor& o = *outs[i];
        const int64_t N = o.size(-1);
        const bool nk = w.size(0) == N && w.size(1) == K;
        check_rc(minfer_gemm(dtype, nk ? MINFER_GEMM_B_NK : MINFER_GEMM_B_KN, x.const_data_ptr(), w.const_data_ptr(), nullptr,
                             o.mutable_data_ptr(), M, N, K, K, nk ? K : N, N, N, 1.0, 0.0, stream),
                 names[i]);
    }
}

// Same signatures and checks as the reference's dequant_cuda and quant_cpu (reference:
// src/minfer/kernels/torch_ext/csrc/cuda/quants/op.cuh:25-78, csrc/quants/op.cpp:156-196), for the one block
// format on this path, Q8_0; the quantiser runs on the device here.  x and y are 2-D, rows are whole blocks.
void dequant_hip(int64_t qtype_int, int64_t qblock_size, int64_t qtype_size, const Tensor& x, Tensor& y) {
    STD_TORCH_CHECK(qtype_int == MINFER_Q8_0, "dequant: only Q8_0 (qtype 8) is built here, got qtype ", qtype_int);
    STD_TORCH_CHECK(qblock_size == MINFER_Q8_0_BLOCK && qtype_size == MINFER_Q8_0_BLOCK_BYTES, "dequant: Q8_0 has qblock_size 32 and qtype_size 34");
    STD_TORCH_CHECK(on_gpu(x) && on_gpu(y), "dequant: x and y must be on the GPU");
    STD_TORCH_CHECK(x.dim() == 2 && y.dim() == 2);
    STD_TORCH_CHECK(x.size(0) == y.size(0), "x and y must have the same number of rows");
    STD_TORCH_CHECK(x.scalar_type() == ScalarType::Byte, "x must be uint8 (byte)");
    STD_TORCH_CHECK(y.scalar_type() == ScalarType::Float || y.scalar_type() == ScalarType::Half, "y must be float32 or float16");
    STD_TORCH_CHECK(x.is_contiguous(), "x must be contiguous");
    STD_TORCH_CHECK(y.is_contiguous(), "y must be contiguous");
    STD_TORCH_CHECK(y.size(1) % 32 == 0 && x.size(1) == y.size(1) / 32 * 34, "dequant: x rows must hold y.size(1)/32 blocks of 34 bytes");
    check_rc(minfer_dequant_q8_0(y.scalar_type() == ScalarType::Float ? MINFER_ATTN_F32 : MINFER_ATTN_F16, x.const_data_ptr(),
                                 y.mutable_data_ptr(), y.size(0), y.size(1), current_stream()),
             "dequant");
}

void quant_hip(int64_t qtype_int, int64_t qblock_size, int64_t qtype_size, const Tensor& x, Tensor& y) {
    STD_TORCH_CHECK(qtype_int == MINFER_Q8_0, "quant: only Q8_0 (qtype 8) is built here, got qtype ", qtype_int);
    STD_TORCH_CHECK(qblock_size == MINFER_Q8_0_BLOCK && qtype_size == MINFER_Q8_0_BLOCK_BYTES, "quant: Q8_0 has qblock_size 32 and qtype_size 34");
    STD_TORCH_CHECK(on_gpu(x) && on_gpu(y), "quant: x and y must be on the GPU");
    STD_TORCH_CHECK(x.dim() == 2 && y.dim() == 2);
    STD_TORCH_CHECK(x.size(0) == y.size(0), "x and y must have same number of rows");
    const ScalarType t = x.scalar_type();
    STD_TORCH_CHECK(t == ScalarType::Float || t == ScalarType::Half || t == ScalarType::BFloat16, "x must be float32 (or float16 / bfloat16)");
    STD_TORCH_CHECK(y.scalar_type() == ScalarType::Byte, "y must be uint8 (byte)");
    STD_TORCH_CHECK(x.is_contiguous(), "x must be contiguous");
    STD_TORCH_CHECK(y.is_contiguous(), "y must be contiguous");
    STD_TORCH_CHECK(x.size(1) % 32 == 0 && y.size(1) == x.size(1) / 32 * 34, "quant: y rows must hold x.size(1)/32 blocks of 34 bytes");
    const int src = t == ScalarType::Float ? MINFER_ATTN_F32 : t == ScalarType::Half ? MINFER_ATTN_F16 : MINFER_ATTN_BF16;
    check_rc(minfer_quant_q8_0(src, x.const_data_ptr(), y.mutable_data_ptr(), x.size(0), x.size(1), current_stream()), "quant");
}

STABLE_TORCH_LIBRARY(minfer, m) {
    // verbatim the reference's schema (reference: src/minfer/kernels/torch_ext/csrc/reg.cpp:30)
    m.def("dequant(int qtype, int qblock_size, int qtype_size, Tensor x, Tensor(a!) y) -> ()");
    m.def("quant(int qtype, int qblock_size, int qtype_size, Tensor x, Tensor(a!) y) -> ()");
    m.def("flash_attn(int qtype_int, int qblock_size, int qtype_size, Tensor q, Tensor k, Tensor v, Tensor(a!) mask, Tensor(a!) out) -> ()");
    // verbatim the reference's schemas (reference: src/minfer/kernels/torch_ext/csrc/reg.cpp:24-29)
    m.def("gemm(int qtype_int, int qblock_size, int qtype_size, float alpha, float beta, Tensor A, Tensor B, Tensor C, Tensor(a!) out) -> ()");
    m.def("qkv(int q_qtype_int, int k_qtype_int, int v_qtype_int, int q_qblock_size, int k_qblock_size, int v_qblock_size, int q_qtype_size, int k_qtype_size, int v_qtype_size, Tensor x, Tensor wq, Tensor wk, Tensor wv, Tensor(a!) q_out, Tensor(a!) k_out, Tensor(a!) v_out) -> ()");
    m.def("rmsnorm(float eps, Tensor input, Tensor w, Tensor(a!) out) -> ()");
    m.def("il_rope(int rotary_dim, int start_pos, float freq_base, Tensor(a!) x) -> ()");
    m.def("neox_rope(int rotary_dim, int start_pos, float freq_base, Tensor(a!) x) -> ()");
    // extensions in the same style: ints first, inputs, out-parameter last, no return value
    m.def("flash_attn_decode(int qtype_int, int qblock_size, int qtype_size, Tensor q, Tensor k_cache, Tensor v_cache, Tensor ctx_lens, Tensor(a!) out) -> ()");
    m.def("flash_attn_varlen(int qtype_int, int qblock_size, int qtype_size, Tensor q, Tensor k, Tensor v, Tensor cu_seqlens, int max_seqlen, Tensor(a!) out) -> ()");
    m.def("rope_kv_append(int style, int rotary_dim, float freq_base, Tensor(a!) q, Tensor k, Tensor v, Tensor positions, Tensor(b!) k_cache, Tensor(c!) v_cache) -> ()");
    m.def("rope_kv_append_norm(int style, int rotary_dim, float freq_base, float eps, Tensor(a!) q, Tensor k, Tensor v, Tensor wq_norm, Tensor wk_norm, Tensor positions, Tensor(b!) k_cache, Tensor(c!) v_cache) -> ()");
}

STABLE_TORCH_LIBRARY_IMPL(minfer, CUDA, m) {  // "CUDA" is PyTorch's dispatch-key name for ROCm devices too
    m.impl("dequant", TORCH_BOX(&dequant_hip));
    m.impl("quant", TORCH_BOX(&quant_hip));
    m.impl("flash_attn", TORCH_BOX(&flash_attn_hip));
    m.impl("flash_attn_decode", TORCH_BOX(&flash_attn_decode_hip));
    m.impl("flash_attn_varlen", TORCH_BOX(&flash_attn_varlen_hip));
    m.impl("rmsnorm", TORCH_BOX(&rmsnorm_hip));
    m.impl("gemm", TORCH_BOX(&gemm_hip));
    m.impl("qkv", TORCH_BOX(&qkv_hip));
    m.impl("il_rope", TORCH_BOX(&il_rope_hip));
    m.impl("neox_rope", TORCH_BOX(&neox_rope_hip));
    m.impl("rope_kv_append", TORCH_BOX(&rope_kv_append_hip));
    m.impl("rope_kv_append_norm", TORCH_BOX(&rope_kv_append_norm_hip));
}

}  // namespace minfer
