/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the half-precision GEMM.
 *
 * Nothing in the shipped package may import, link or call this file; it is the
 * checker used by tests/ and by the cpu_baseline legs of bench.py.
 *
 * What it restates.  The reference's op computes D = alpha * A B + beta * C for a weight
 * stored [K, N], or alpha * A B^T + beta * C for a weight stored [N, K] (reference:
 * src/minfer/kernels/torch_ext/csrc/cuda/gemm/op.cuh:284-297); its oracle is
 * torch.addmm(bias, input, weight, beta=beta, alpha=alpha) (reference:
 * src/minfer/kernels/refs.py:49-51) and, in its test, alpha*(A@W) + beta*bias
 * (reference: test/kernels.py:139); the QKV projection is x @ W^T per weight
 * (reference: test/kernels.py:193-195).  Here the sum is evaluated in fp64 on fp32
 * inputs (callers up-cast first and round the result themselves).
 * Returns 0, or -1 on a bad argument.
 */
#include <stdint.h>

/* b_layout 0: B is [K,N]; 1: B is [N,K].  All matrices contiguous.  C may be null when beta == 0. */
int oracle_gemm(int b_layout, const float* A, const float* B, const float* C, float* D, int64_t M, int64_t N,
                int64_t K, double alpha, double beta) {
    if ((b_layout != 0 && b_layout != 1) || !A || !B || !D || (beta != 0.0 && !C) || M < 0 || N < 0 || K < 0) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double s = 0.0;
            if (b_layout == 0)
                for (int64_t k = 0; k < K; ++k) s += (double)A[m * K + k] * (double)B[k * N + n];
            else
                for (int64_t k = 0; k < K; ++k) s += (double)A[m * K + k] * (double)B[n * K + k];
            D[m * N + n] = (float)(alpha * s + (beta != 0.0 ? beta * (double)C[m * N + n] : 0.0));
        }
    return 0;
}
