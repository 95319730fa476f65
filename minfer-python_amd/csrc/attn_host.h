// Host-side helpers shared by the C-ABI entry points: per-thread error text and the argument
// checks every entry point applies before launching anything.
#pragma once

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "minfer_attn.h"

// Everything is compiled with hidden visibility; only the C ABI is exported.
#define MINFER_ATTN_EXPORT extern "C" __attribute__((visibility("default")))

namespace minfer_attn {

inline char* error_buf() {
    static thread_local char buf[512] = {0};
    return buf;
}
inline void clear_error() { error_buf()[0] = '\0'; }
inline int fail(int code, const char* msg) {
    snprintf(error_buf(), 512, "%s", msg);
    return code;
}
inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        snprintf(error_buf(), 512, "%s: launch failed: %s", what, hipGetErrorString(e));
        return MINFER_ATTN_ELAUNCH;
    }
    return MINFER_ATTN_OK;
}
inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// A launch of a byte mover (rope, rmsnorm, dequantiser) that touches more distinct bytes than this marks its loads and
// stores non-temporal: a working set beyond the 256 MiB memory-side cache only churns it, and streaming past it is
// 9-20 % faster; a smaller one is left in the caches for the kernel that consumes it next (an in-place rope over
// 200 MB that is run again, or read by the next kernel, is 15 % faster that way).
constexpr int64_t kStreamBytes = INT64_C(256) << 20;

// Checks shared by the three operators.  Mirrors the reference host function's validation
// (reference: src/minfer/kernels/torch_ext/csrc/cuda/flash_attn/op.cuh:32-96) at the pointer
// level: dtype (Half there; Half or BFloat16 here), head_dim (128 there; 64 or 128 here), GQA
// divisibility, plus the 16-byte vector-access requirements of these kernels.
inline int check_common(int dtype, const void* q, const void* k, const void* v, const void* out,
                        int64_t Hq, int64_t Hkv, int64_t D, const minfer_attn_strides* st) {
    if (dtype != MINFER_ATTN_F16 && dtype != MINFER_ATTN_BF16)
        return fail(MINFER_ATTN_EINVAL, "dtype must be MINFER_ATTN_F16 or MINFER_ATTN_BF16");
    if (D != 64 && D != 128) return fail(MINFER_ATTN_EINVAL, "head_dim must be 64 or 128");
    if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0)
        return fail(MINFER_ATTN_EINVAL, "n_heads must be a positive multiple of n_kv_heads");
    if (Hq > 65535) return fail(MINFER_ATTN_EINVAL, "n_heads > 65535 unsupported");
    if (!st) return fail(MINFER_ATTN_EINVAL, "strides is null");
    if (!q || !k || !v || !out) return fail(MINFER_ATTN_EINVAL, "q, k, v and out must be non-null");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out))
        return fail(MINFER_ATTN_EINVAL, "q, k, v and out must be 16-byte aligned");
    const int64_t s[9] = {st->q0, st->q1, st->q2, st->kv0, st->kv1, st->kv2, st->o0, st->o1, st->o2};
    for (int i = 0; i < 9; ++i)
        if (s[i] % 8 != 0 || s[i] < 0)
            return fail(MINFER_ATTN_EINVAL, "strides of dims 0..2 must be non-negative multiples of 8 elements");
    return MINFER_ATTN_OK;
}

// Dequantises K and V rows of Q8_0 blocks ([B, Hkv, L] rows of D/32 blocks; byte strides s0, s1 between batch
// entries and heads; rows dense) into contiguous fp16 [B, Hkv, L, D] (csrc/quant.hip).
int launch_dequant_q8_0_kv(const void* k, const void* v, void* k_out, void* v_out, int64_t B, int64_t Hkv, int64_t L,
                           int64_t D, int64_t s0, int64_t s1, hipStream_t stream);

}  // namespace minfer_attn
