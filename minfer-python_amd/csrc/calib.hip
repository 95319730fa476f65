// Calibration kernel: the matrix pipes alone.  Every wave keeps eight A and eight B operand fragments in
// registers (read once from a caller-provided buffer, so the caller chooses the values: random, constant, zero) and
// issues v_mfma_f32_32x32x16 back to back on four independent accumulators, two waves per SIMD, nothing else in the
// loop.  What this reaches is the rate the chip sustains on the matrix instruction the attention and GEMM kernels use
// when no other unit competes for issue slots or power; it depends on the operand values (multipliers that toggle
// draw more power, and the chip lowers its clock to stay inside its budget), which is why the buffer is an argument.
// No counterpart in the reference.
#include "attn_common.h"
#include "attn_host.h"

namespace minfer_attn {

constexpr int kCalibWaves = 8;     // per workgroup: two per SIMD, as in the prefill kernel
constexpr int kCalibFrags = 16;    // 8 A + 8 B fragments of 64 lanes x 16 bytes

template <class T>
__global__ __launch_bounds__(kCalibWaves * 64, 1) void mfma_rate_kernel(const s16x8* __restrict__ operands, int iters,
                                                                         float* __restrict__ sink) {
    const int lane = threadIdx.x & 63;
    s16x8 a[8], b[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        a[j] = operands[j * 64 + lane];
        b[j] = operands[(8 + j) * 64 + lane];
    }
    f32x16 acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j & 3] = T::mfma32(a[j], b[j], acc[j & 3]);
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[c][r];
    sink[(size_t)blockIdx.x * (kCalibWaves * 64) + threadIdx.x] = s;
}

}  // namespace minfer_attn

using namespace minfer_attn;

MINFER_ATTN_EXPORT int minfer_calib_mfma_rate(int dtype, const void* operands, int64_t iters, int64_t workgroups, float* sink,
                                              void* stream_v) {
    clear_error();
    if (dtype != MINFER_ATTN_F16 && dtype != MINFER_ATTN_BF16)
        return fail(MINFER_ATTN_EINVAL, "calib_mfma_rate: dtype must be MINFER_ATTN_F16 or MINFER_ATTN_BF16");
    if (!operands || !sink || !aligned16(operands)) return fail(MINFER_ATTN_EINVAL, "calib_mfma_rate: operands (16-byte aligned) and sink must be non-null");
    if (iters < 0 || iters > (1 << 24) || workgroups <= 0 || workgroups > (1 << 20))
        return fail(MINFER_ATTN_EINVAL, "calib_mfma_rate: iters must be in [0, 2^24] and workgroups in [1, 2^20]");
    hipStream_t stream = (hipStream_t)stream_v;
    if (dtype == MINFER_ATTN_F16)
        hipLaunchKernelGGL(mfma_rate_kernel<F16>, dim3((unsigned)workgroups), dim3(kCalibWaves * 64), 0, stream,
                           (const s16x8*)operands, (int)iters, sink);
    else
        hipLaunchKernelGGL(mfma_rate_kernel<BF16>, dim3((unsigned)workgroups), dim3(kCalibWaves * 64), 0, stream,
                           (const s16x8*)operands, (int)iters, sink);
    return check_launch("mfma_rate_kernel");
}
