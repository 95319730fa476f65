/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for RMS normalisation.
 *
 * Nothing in the shipped package may import, link or call this file; it is the
 * checker used by tests/ and by the cpu_baseline legs of bench.py.
 *
 * What it restates.  The reference's kernel (reference:
 * src/minfer/kernels/torch_ext/csrc/cuda/rmsnorm/kernel.cuh:24-38) treats its input as
 * numel/dim contiguous vectors with dim = the weight's length (rmsnorm/op.cuh:52-53) and
 * computes, per vector,
 *     sc = rsqrt(sum(x^2) / dim + eps),   out[i] = x[i] * w[i] * sc.
 * Its oracle is torch's F.rms_norm over the last dimension (reference:
 * src/minfer/kernels/refs.py:4-10), the same closed form.  Here it is evaluated in fp64
 * on fp32 inputs (callers up-cast fp16/bf16 first and round the result themselves).
 * Returns 0, or -1 on a bad argument.
 */
#include <math.h>
#include <stdint.h>

int oracle_rmsnorm(const float* in, const float* w, float* out, int64_t n_vectors, int64_t dim, double eps) {
    if (!in || !w || !out || n_vectors < 0 || dim <= 0 || !(eps >= 0.0)) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t v = 0; v < n_vectors; ++v) {
        const float* x = in + v * dim;
        double ss = 0.0;
        for (int64_t i = 0; i < dim; ++i) ss += (double)x[i] * (double)x[i];
        const double sc = 1.0 / sqrt(ss / (double)dim + eps);
        for (int64_t i = 0; i < dim; ++i) out[v * dim + i] = (float)((double)x[i] * (double)w[i] * sc);
    }
    return 0;
}
