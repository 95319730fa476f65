// RMS normalisation for gfx950: out = x * w * rsqrt(mean(x^2) + eps) over vectors of length dim = |w|.
//
// What the reference computes (reference: src/minfer/kernels/torch_ext/csrc/cuda/rmsnorm/kernel.cuh:11-40,
// host side rmsnorm/op.cuh:20-70, oracle src/minfer/kernels/refs.py:4-10): the input, [B,L,hidden] or
// [B,L,n_heads,head_dim], is a list of numel/dim contiguous vectors; each is scaled by the reciprocal root of
// its mean square (fp32 arithmetic) and multiplied elementwise by the weight.  The reference runs one block
// per vector and reads the vector twice from memory.
//
// HBM-bound: every element is read once and written once, in 16-byte lane accesses, and stays in registers
// between the sum of squares and the scaling, as does the lane's share of the weight.  Vectors up to 8192 elements (per-head norm, and per-token norm
// of the usual hidden sizes) are handled by a group of 8..64 lanes of one wave, several short vectors per
// wave, reduced with lane exchanges only and with no barrier; longer vectors by one 256-thread workgroup
// with one LDS exchange.
#include <algorithm>

#include "attn_common.h"
#include "attn_host.h"

namespace minfer_attn {

constexpr int kNormThreads = 256;

struct NormParams {
    const void* in; const void* w; void* out;
    int64_t n_vec;
    int dim;
    float eps, inv_dim;
};

// LANES lanes per vector, NCH 16-byte chunks per lane (dim <= LANES * 8 * NCH, dim % 8 == 0): chunk j of a
// lane covers elements 8 * (j * LANES + lane_in_group) .., so a group reads contiguous 16 * LANES bytes.
template <class T, int LANES, int NCH, bool STREAM>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_rows_kernel(const NormParams p) {
    const int lane = threadIdx.x & 63, gl = lane & (LANES - 1);
    constexpr int VPW = 64 / LANES;                               // vectors per wave
    const int64_t wave = (int64_t)blockIdx.x * (kNormThreads / 64) + (threadIdx.x >> 6);
    const int64_t n_waves = (int64_t)gridDim.x * (kNormThreads / 64);
    const int chunks = p.dim >> 3;
    // the lane's share of the weight stays in registers for all the vectors the wave handles (re-reading it from
    // cache per vector cost 5 % at 4096-6144 elements)
    s16x8 wv[NCH];
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        const int c = j * LANES + gl;
        wv[j] = c < chunks ? *reinterpret_cast<const s16x8*>((const short*)p.w + 8 * c) : s16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
    for (int64_t v0 = wave * VPW; v0 < p.n_vec; v0 += n_waves * VPW) {
        const int64_t vec = v0 + lane / LANES;
        const bool on = vec < p.n_vec;
        const short* src = (const short*)p.in + vec * p.dim;
        s16x8 x[NCH];
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            const int c = j * LANES + gl;
            x[j] = (on && c < chunks) ? load_once<STREAM>(reinterpret_cast<const s16x8*>(src + 8 * c)) : s16x8{0, 0, 0, 0, 0, 0, 0, 0};
        }
#pragma unroll
        for (int j = 0; j < NCH; ++j) ss += sum_sq8<T>(x[j]);
#pragma unroll
        for (int m = 1; m < LANES; m <<= 1) ss += __shfl_xor(ss, m);
        const float sc = rsqrtf(ss * p.inv_dim + p.eps);
        short* dst = (short*)p.out + vec * p.dim;
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            const int c = j * LANES + gl;
            if (on && c < chunks) store_once<STREAM>(reinterpret_cast<s16x8*>(dst + 8 * c), scale8w<T>(x[j], wv[j], sc));
        }
    }
}

// One workgroup per vector.  VEC: 16-byte chunks, up to NCH per thread held in registers (dim <= 2048 * NCH
// elements), anything beyond that re-read; !VEC: any dim and alignment, element by element.
template <class T, bool VEC, int NCH>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_block_kernel(const NormParams p) {
    __shared__ float part[kNormThreads / 64];
    const int tid = threadIdx.x;
    for (int64_t vec = blockIdx.x; vec < p.n_vec; vec += gridDim.x) {
        const short* src = (const short*)p.in + vec * p.dim;
        short* dst = (short*)p.out + vec * p.dim;
        const short* wp = (const short*)p.w;
        float ss = 0.f;
        s16x8 x[NCH];
        const int chunks = p.dim >> 3;
        if (VEC) {
#pragma unroll
            for (int j = 0; j < NCH; ++j) {
                const int c = j * kNormThreads + tid;
                x[j] = c < chunks ? *reinterpret_cast<const s16x8*>(src + 8 * c) : s16x8{0, 0, 0, 0, 0, 0, 0, 0};
            }
#pragma unroll
            for (int j = 0; j < NCH; ++j) ss += sum_sq8<T>(x[j]);
            for (int c = NCH * kNormThreads + tid; c < chunks; c += kNormThreads)
                ss += sum_sq8<T>(*reinterpret_cast<const s16x8*>(src + 8 * c));
        } else {
            for (int i = tid; i < p.dim; i += kNormThreads) { const float f = T::to_float(src[i]); ss += f * f; }
        }
#pragma unroll
        for (int m = 1; m < 64; m <<= 1) ss += __shfl_xor(ss, m);
        __syncthreads();                 // the previous vector's partial sums have been read
        if ((tid & 63) == 0) part[tid >> 6] = ss;
        __syncthreads();
        float tot = 0.f;
#pragma unroll
        for (int i = 0; i < kNormThreads / 64; ++i) tot += part[i];
        const float sc = rsqrtf(tot * p.inv_dim + p.eps);
        if (VEC) {
#pragma unroll
            for (int j = 0; j < NCH; ++j) {
                const int c = j * kNormThreads + tid;
                if (c < chunks)
                    *reinterpret_cast<s16x8*>(dst + 8 * c) = scale8w<T>(x[j], *reinterpret_cast<const s16x8*>(wp + 8 * c), sc);
            }
            for (int c = NCH * kNormThreads + tid; c < chunks; c += kNormThreads)
                *reinterpret_cast<s16x8*>(dst + 8 * c) =
                    scale8w<T>(*reinterpret_cast<const s16x8*>(src + 8 * c), *reinterpret_cast<const s16x8*>(wp + 8 * c), sc);
        } else {
            for (int i = tid; i < p.dim; i += kNormThreads) {
                const uint32_t pk = T::pack2(T::to_float(src[i]) * T::to_float(wp[i]) * sc, 0.f);
                dst[i] = (short)(pk & 0xffffu);
            }
        }
    }
}

template <class T>
static void launch_norm(const NormParams& p, bool vec_ok, hipStream_t stream) {
    const int waves_cap = 256 * 8 * 4;   // resident waves of the chip, times a few
    if (vec_ok && p.dim <= 8192) {
        const int chunks = p.dim >> 3;
        const bool streamed = 2 * p.n_vec * p.dim * 2 > kStreamBytes;   // input and output
#define MINFER_ROWS(LANES, NCH)                                                                                   \
    {                                                                                                             \
        const int64_t waves = (p.n_vec + (64 / LANES) - 1) / (64 / LANES);                                        \
        const int grid = (int)std::min<int64_t>((waves + 3) / 4, waves_cap / 4);                                  \
        if (streamed) hipLaunchKernelGGL((rmsnorm_rows_kernel<T, LANES, NCH, true>), dim3(grid), dim3(kNormThreads), 0, stream, p);  \
        else hipLaunchKernelGGL((rmsnorm_rows_kernel<T, LANES, NCH, false>), dim3(grid), dim3(kNormThreads), 0, stream, p);          \
    }
        if (chunks <= 8) MINFER_ROWS(8, 1)
        else if (chunks <= 16) MINFER_ROWS(16, 1)
        else if (chunks <= 32) MINFER_ROWS(32, 1)
        else if (chunks <= 64) MINFER_ROWS(64, 1)
        else if (chunks <= 128) MINFER_ROWS(64, 2)
        else if (chunks <= 256) MINFER_ROWS(64, 4)
        else if (chunks <= 384) MINFER_ROWS(64, 6)
        else if (chunks <= 512) MINFER_ROWS(64, 8)
        else if (chunks <= 768) MINFER_ROWS(64, 12)
        else MINFER_ROWS(64, 16)
#undef MINFER_ROWS
    } else {
        const int grid = (int)std::min<int64_t>(p.n_vec, 256 * 8);
        if (vec_ok) hipLaunchKernelGGL((rmsnorm_block_kernel<T, true, 4>), dim3(grid), dim3(kNormThreads), 0, stream, p);
        else hipLaunchKernelGGL((rmsnorm_block_kernel<T, false, 1>), dim3(grid), dim3(kNormThreads), 0, stream, p);
    }
}

}  // namespace minfer_attn

using namespace minfer_attn;

MINFER_ATTN_EXPORT int minfer_rmsnorm(int dtype, const void* in, const void* w, void* out, int64_t n_vectors,
                                      int64_t dim, double eps, void* stream_v) {
    clear_error();
    if (dtype != MINFER_ATTN_F16 && dtype != MINFER_ATTN_BF16)
        return fail(MINFER_ATTN_EINVAL, "rmsnorm: dtype must be MINFER_ATTN_F16 or MINFER_ATTN_BF16");
    if (n_vectors < 0 || dim <= 0 || dim > 0x7fffffffLL) return fail(MINFER_ATTN_EINVAL, "rmsnorm: bad n_vectors or dim");
    if (!(eps >= 0.0)) return fail(MINFER_ATTN_EINVAL, "rmsnorm: eps must be non-negative");
    if (!in || !w || !out) return fail(MINFER_ATTN_EINVAL, "rmsnorm: null pointer");
    if (n_vectors == 0) return MINFER_ATTN_OK;
    NormParams p{};
    p.in = in; p.w = w; p.out = out; p.n_vec = n_vectors; p.dim = (int)dim;
    p.eps = (float)eps; p.inv_dim = (float)(1.0 / (double)dim);
    const bool vec_ok = dim % 8 == 0 && aligned16(in) && aligned16(w) && aligned16(out);
    hipStream_t stream = (hipStream_t)stream_v;
    if (dtype == MINFER_ATTN_F16) launch_norm<F16>(p, vec_ok, stream);
    else launch_norm<BF16>(p, vec_ok, stream);
    return check_launch("rmsnorm kernel");
}
