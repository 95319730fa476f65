// Q8_0 block quantisation for gfx950: rows of floats <-> rows of 34-byte blocks.
//
// A block holds 32 consecutive values of a row as an fp16 scale d followed by 32 int8
// (reference: src/minfer/kernels/torch_ext/csrc/common/types.hpp:141-146).  Quantising (reference:
// csrc/quants/impl.cpp:1169-1193, CPU only there): amax = max |x|, d = amax / 127, id = d ? 1 / d : 0,
// q = roundf(x * id) (ties away from zero), d stored rounded to fp16.  Dequantising (reference:
// cuda/quants/impls.cuh:121-143, csrc/quants/impl.cpp:1152-1167): y = (T)(q * (float)d).  Both are exact
// restatements: IEEE division, one rounding per step, so the bytes equal the reference's.
//
// HBM-bound byte movers.  Four lanes share a block, eight values each (the amax goes through two
// lane exchanges), so a wave reads 2 KB (fp32) or 1 KB (fp16) of contiguous input per step and writes 544
// contiguous bytes; blocks start on 2-byte boundaries, which global accesses on this target allow.
#include <algorithm>

#include "attn_common.h"
#include "attn_host.h"
#include "quant_q8.h"

namespace minfer_attn {

constexpr int kQuantThreads = 256;

// x: n_blocks * 32 values, contiguous; y: n_blocks * 34 bytes.  SRC: 0 fp32, 1 fp16, 2 bf16.
template <int SRC>
__global__ __launch_bounds__(kQuantThreads) void quant_q8_0_kernel(const void* x, char* y, int64_t n_blocks) {
    const int64_t n_pieces = n_blocks * 4;
    for (int64_t i = (int64_t)blockIdx.x * kQuantThreads + threadIdx.x; i < ((n_pieces + 3) & ~(int64_t)3);
         i += (int64_t)gridDim.x * kQuantThreads) {
        const bool on = i < n_pieces;   // a block's four lanes are on or off together (n_pieces is a multiple of 4)
        float f[8];
        if (SRC == 0) {
            const f32x4* src = (const f32x4*)x + 2 * i;
            const f32x4 a = on ? src[0] : f32x4{0.f, 0.f, 0.f, 0.f};
            const f32x4 b = on ? src[1] : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 4; ++j) { f[j] = a[j]; f[4 + j] = b[j]; }
        } else {
            const s16x8 a = on ? ((const s16x8*)x)[i] : s16x8{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < 8; ++j) f[j] = SRC == 1 ? F16::to_float(a[j]) : BF16::to_float(a[j]);
        }
        uint16_t d_bits;
        const uint2 q = quant8_q8_0(f, d_bits);
        if (on) {
            char* blk = y + (i >> 2) * 34;
            store_q8_piece(blk, (int)(i & 3) * 8, q, d_bits);
        }
    }
}

// x: n_blocks * 34 bytes; y: n_blocks * 32 values.  DST: 0 fp32, 1 fp16.
template <int DST, bool STREAM>
__global__ __launch_bounds__(kQuantThreads) void dequant_q8_0_kernel(const char* x, void* y, int64_t n_blocks) {
    if (DST == 0) {
        // fp32 output is 4 bytes out per byte in: a lane takes 4 quants and stores one 16-byte piece, so that every
        // store instruction of a wave writes 1 KB in one run (8 quants and two strided stores per lane ran 35 % slower)
        const int64_t n4 = n_blocks * 8;
        for (int64_t i = (int64_t)blockIdx.x * kQuantThreads + threadIdx.x; i < n4; i += (int64_t)gridDim.x * kQuantThreads) {
            const char* blk = (const char*)__builtin_assume_aligned(x + (i >> 3) * 34, 2);
            uint16_t d_bits, lo, hi;
            __builtin_memcpy(&d_bits, blk, 2);
            __builtin_memcpy(&lo, blk + 2 + 4 * (i & 7), 2);
            __builtin_memcpy(&hi, blk + 4 + 4 * (i & 7), 2);
            const float d = (float)__builtin_bit_cast(_Float16, d_bits);
            const uint32_t q = (uint32_t)lo | ((uint32_t)hi << 16);
            f32x4 a;
#pragma unroll
            for (int j = 0; j < 4; ++j) a[j] = (float)(int8_t)(q >> (8 * j)) * d;
            store_once<STREAM>((f32x4*)y + i, a);
        }
        return;
    }
    const int64_t n_pieces = n_blocks * 4;
    for (int64_t i = (int64_t)blockIdx.x * kQuantThreads + threadIdx.x; i < n_pieces; i += (int64_t)gridDim.x * kQuantThreads) {
        const char* blk = (const char*)__builtin_assume_aligned(x + (i >> 2) * 34, 2);
        uint16_t d_bits;
        uint2 q;
        __builtin_memcpy(&d_bits, blk, 2);
        __builtin_memcpy(&q, blk + 2 + 8 * (i & 3), 8);
        if (DST == 1) {
            const _Float16 dh = __builtin_bit_cast(_Float16, d_bits);
            const h16x2 d2 = {dh, dh};
            store_once<STREAM>((s16x8*)y + i, dequant8_words(q.x, q.y, d2));
        } else {
            const float d = (float)__builtin_bit_cast(_Float16, d_bits);
            f32x4 a, b;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                a[j] = (float)(int8_t)(q.x >> (8 * j)) * d;
                b[j] = (float)(int8_t)(q.y >> (8 * j)) * d;
            }
            f32x4* dst = (f32x4*)y + 2 * i;
            dst[0] = a;
            dst[1] = b;
        }
    }
}

// K and V rows of Q8_0 blocks, [B, Hkv, L] rows of D/32 blocks with byte strides s0, s1 between batch entries and
// heads (rows dense), into two contiguous fp16 tensors [B, Hkv, L, D]: what prefill attention over quantised K/V
// reads.  grid (pieces of one (batch, head), B * Hkv, 2): z = 0 is K, 1 is V.
__global__ __launch_bounds__(kQuantThreads) void dequant_q8_0_kv_kernel(const char* k, const char* v, short* k_out, short* v_out,
                                                                      int Hkv, int64_t s0, int64_t s1, int64_t pieces_per_head) {
    const int bg = blockIdx.y, b = bg / Hkv, g = bg - b * Hkv;
    const char* src = (blockIdx.z ? v : k) + (int64_t)b * s0 + (int64_t)g * s1;
    s16x8* dst = (s16x8*)(blockIdx.z ? v_out : k_out) + (int64_t)bg * pieces_per_head;
    for (int64_t i = (int64_t)blockIdx.x * kQuantThreads + threadIdx.x; i < pieces_per_head; i += (int64_t)gridDim.x * kQuantThreads) {
        const char* blk = (const char*)__builtin_assume_aligned(src + (i >> 2) * 34, 2);
        uint16_t d_bits;
        uint2 q;
        __builtin_memcpy(&d_bits, blk, 2);
        __builtin_memcpy(&q, blk + 2 + 8 * (i & 3), 8);
        const _Float16 dh = __builtin_bit_cast(_Float16, d_bits);
        const h16x2 d2 = {dh, dh};
        dst[i] = dequant8_words(q.x, q.y, d2);
    }
}

int launch_dequant_q8_0_kv(const void* k, const void* v, void* k_out, void* v_out, int64_t B, int64_t Hkv, int64_t L,
                           int64_t D, int64_t s0, int64_t s1, hipStream_t stream) {
    const int64_t pieces = L * (D / 8);
    const dim3 grid((unsigned)std::min<int64_t>((pieces + kQuantThreads - 1) / kQuantThreads, 4096), (unsigned)(B * Hkv), 2);
    hipLaunchKernelGGL(dequant_q8_0_kv_kernel, grid, dim3(kQuantThreads), 0, stream, (const char*)k, (const char*)v,
                       (short*)k_out, (short*)v_out, (int)Hkv, s0, s1, pieces);
    return check_launch("dequant_q8_0_kv_kernel");
}

static int check_rows(const char* op, const void* x, const void* y, int64_t n_rows, int64_t k) {
    char msg[160];
    auto bad = [&](const char* what) {
        snprintf(msg, sizeof msg, "%s: %s", op, what);
        return fail(MINFER_ATTN_EINVAL, msg);
    };
    if (n_rows < 0 || k < 0) return bad("negative size");
    if (k % 32 != 0) return bad("row length must be a multiple of 32 (the Q8_0 block)");
    if (!x || !y) return bad("null pointer");
    if (n_rows > 0 && k > 0 && n_rows > (INT64_C(1) << 56) / k) return bad("problem too large");
    return MINFER_ATTN_OK;
}

static int grid_for(int64_t n_pieces) {
    return (int)std::min<int64_t>((n_pieces + kQuantThreads - 1) / kQuantThreads, 256 * 32);
}

}  // namespace minfer_attn

using namespace minfer_attn;

MINFER_ATTN_EXPORT int minfer_quant_q8_0(int src_dtype, const void* x, void* y, int64_t n_rows, int64_t k, void* stream_v) {
    clear_error();
    if (src_dtype != MINFER_ATTN_F32 && src_dtype != MINFER_ATTN_F16 && src_dtype != MINFER_ATTN_BF16)
        return fail(MINFER_ATTN_EINVAL, "quant_q8_0: source dtype must be MINFER_ATTN_F32, MINFER_ATTN_F16 or MINFER_ATTN_BF16");
    if (int rc = check_rows("quant_q8_0", x, y, n_rows, k)) return rc;
    if (!aligned16(x)) return fail(MINFER_ATTN_EINVAL, "quant_q8_0: x must be 16-byte aligned");
    if ((uintptr_t)y & 1u) return fail(MINFER_ATTN_EINVAL, "quant_q8_0: y must be 2-byte aligned");
    const int64_t n_blocks = n_rows * (k / 32);
    if (n_blocks == 0) return MINFER_ATTN_OK;
    hipStream_t stream = (hipStream_t)stream_v;
    const dim3 grid(grid_for(n_blocks * 4)), block(kQuantThreads);
    if (src_dtype == MINFER_ATTN_F32) hipLaunchKernelGGL((quant_q8_0_kernel<0>), grid, block, 0, stream, x, (char*)y, n_blocks);
    else if (src_dtype == MINFER_ATTN_F16) hipLaunchKernelGGL((quant_q8_0_kernel<1>), grid, block, 0, stream, x, (char*)y, n_blocks);
    else hipLaunchKernelGGL((quant_q8_0_kernel<2>), grid, block, 0, stream, x, (char*)y, n_blocks);
    return check_launch("quant_q8_0_kernel");
}

MINFER_ATTN_EXPORT int minfer_dequant_q8_0(int dst_dtype, const void* x, void* y, int64_t n_rows, int64_t k, void* stream_v) {
    clear_error();
    if (dst_dtype != MINFER_ATTN_F32 && dst_dtype != MINFER_ATTN_F16)
        return fail(MINFER_ATTN_EINVAL, "dequant_q8_0: destination dtype must be MINFER_ATTN_F32 or MINFER_ATTN_F16");
    if (int rc = check_rows("dequant_q8_0", x, y, n_rows, k)) return rc;
    if (!aligned16(y)) return fail(MINFER_ATTN_EINVAL, "dequant_q8_0: y must be 16-byte aligned");
    if ((uintptr_t)x & 1u) return fail(MINFER_ATTN_EINVAL, "dequant_q8_0: x must be 2-byte aligned");
    const int64_t n_blocks = n_rows * (k / 32);
    if (n_blocks == 0) return MINFER_ATTN_OK;
    hipStream_t stream = (hipStream_t)stream_v;
    const dim3 grid(grid_for(n_blocks * 4)), block(kQuantThreads);
    const bool streamed = n_blocks * (34 + 32 * (dst_dtype == MINFER_ATTN_F32 ? 4 : 2)) > kStreamBytes;
    if (dst_dtype == MINFER_ATTN_F32) {
        if (streamed) hipLaunchKernelGGL((dequant_q8_0_kernel<0, true>), grid, block, 0, stream, (const char*)x, y, n_blocks);
        else hipLaunchKernelGGL((dequant_q8_0_kernel<0, false>), grid, block, 0, stream, (const char*)x, y, n_blocks);
    } else {
        if (streamed) hipLaunchKernelGGL((dequant_q8_0_kernel<1, true>), grid, block, 0, stream, (const char*)x, y, n_blocks);
        else hipLaunchKernelGGL((dequant_q8_0_kernel<1, false>), grid, block, 0, stream, (const char*)x, y, n_blocks);
    }
    return check_launch("dequant_q8_0_kernel");
}
