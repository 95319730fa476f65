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

// SHAPE32 = false: v_mfma_f32_16x16x32, the instruction the prefill and GEMM kernels are built on (16 per iteration on 8
// accumulator blocks); true: v_mfma_f32_32x32x16 (8 per iteration on 4 blocks).  The same flops per iteration.
template <class T, bool SHAPE32>
__global__ __launch_bounds__(kCalibWaves * 64, 1) void mfma_rate_kernel(const s16x8* __restrict__ operands, int iters,
                                                                         float* __restrict__ sink) {
    const int lane = threadIdx.x & 63;
    s16x8 a[8], b[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        a[j] = operands[j * 64 + lane];
        b[j] = operands[(8 + j) * 64 + lane];
    }
    float s = 0.f;
    if (SHAPE32) {
        f32x16 acc[4];
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j & 3] = T::mfma32(a[j], b[j], acc[j & 3]);
        }
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int r = 0; r < 16; ++r) s += acc[c][r];
    } else {
        f32x4 acc[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[j & 7] = T::mfma16(a[j & 7], b[(j + (j >> 3)) & 7], acc[j & 7]);
        }
#pragma unroll
        for (int c = 0; c < 8; ++c)
#pragma unroll
            for (int r = 0; r < 4; ++r) s += acc[c][r];
    }
    sink[(size_t)blockIdx.x * (kCalibWaves * 64) + threadIdx.x] = s;
}

// The prefill kernel's per-tile instruction mix with everything removed that is not matrix, LDS-read or softmax work: no
// global->LDS copies, no barrier, no masking, no tile bookkeeping, the same K and V tile (64 keys x 128, written to LDS
// once) for every iteration.  Per "tile" a wave issues what the attention kernel issues for head_dim 128 and its 32 query
// rows (two blocks of 16): 32 MFMAs (16x16x32) for S^T = K Q^T with the K fragments read from LDS (16 ds_read_b128), the
// lane's largest exponent of its two rows (16 v_max3) and the reference test, 32 exponentials, 16 packs, 16 dot products for the denominators, and 32
// MFMAs for O^T += V^T P^T with the V^T fragments from 32 transpose reads.  LDS_READS = false keeps the fragments in
// registers instead, SOFTMAX = false feeds the second GEMM from registers: the four combinations show what each kind of
// co-running work costs the matrix rate, and the full mix is what an attention kernel with no fixed costs at all would
// reach.
template <class T, bool LDS_READS, bool SOFTMAX>
__global__ __launch_bounds__(kCalibWaves * 64, 2) void attn_mix_kernel(const s16x8* __restrict__ operands, int iters,
                                                                        float* __restrict__ sink) {
    constexpr int RB = 256, TILE = 64 * RB;
    __shared__ __attribute__((aligned(1024))) char lds[2 * TILE];
    const int lane = threadIdx.x & 63, l16 = lane & 15, quad = lane >> 4;
    // fill both tiles from the 16 KiB of operands (K = the buffer, V = the buffer again)
    for (int i = threadIdx.x; i < 2 * TILE / 16; i += kCalibWaves * 64)
        reinterpret_cast<s16x8*>(lds)[i] = operands[i & (kCalibFrags * 64 - 1)];
    __syncthreads();
    s16x8 qf[2][4];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int c = 0; c < 4; ++c) qf[qb][c] = T::scale8(operands[(4 * qb + c) * 64 + lane], 0.1275f);   // 1/sqrt(128) * log2(e)
    // conflict-free read addresses as in the attention kernel (XOR swizzles by row)
    uint32_t k_rd[4], v_rd[8];
#pragma unroll
    for (int c = 0; c < 4; ++c) k_rd[c] = lds_addr(lds) + l16 * RB + 16 * ((4 * c + quad) ^ l16);
    {
        const int vrow = 4 * quad + (l16 >> 2), swv = (vrow & 7) << 1;
#pragma unroll
        for (int db = 0; db < 8; ++db) {
            const int dcol = 16 * db + 4 * (l16 & 3);
            v_rd[db] = lds_addr(lds) + TILE + vrow * RB + 16 * ((dcol >> 3) ^ swv) + 2 * (dcol & 7);
        }
    }
    s16x8 kreg[4], vreg[4];   // the register-resident operands of the variants without LDS reads
#pragma unroll
    for (int j = 0; j < 4; ++j) { kreg[j] = operands[(8 + j) * 64 + lane]; vreg[j] = operands[(12 + j) * 64 + lane]; }
    f32x4 o_acc[8][2], neg_ref = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int db = 0; db < 8; ++db) o_acc[db][0] = o_acc[db][1] = f32x4{0.f, 0.f, 0.f, 0.f};
    float l_sum = 0.f, m_run = 0.f;
    const float grow_at = 8.f + (float)(iters >> 30);   // the attention kernel's threshold, in a register
    for (int it = 0; it < iters; ++it) {
        asm volatile("" ::: "memory");   // every iteration reads its fragments from LDS again, as a new tile would need
        f32x4 e_acc[4][2];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
#pragma unroll
            for (int kb = 0; kb < 4; ++kb) {
                const s16x8 kf = LDS_READS ? lds_read_b128(k_rd[c], 16 * kb * RB) : kreg[(c + kb) & 3];
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) e_acc[kb][qb] = T::mfma16(kf, qf[qb][c], c == 0 ? neg_ref : e_acc[kb][qb]);
            }
        }
        s16x8 pk[2][2];   // [key chunk][query block]
        if (SOFTMAX) {
            float ls = 0.f;
            float mx[2];
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {   // the lane's largest exponent of the row, as the attention kernel takes it
                float x = max3(e_acc[0][qb][0], e_acc[0][qb][1], e_acc[0][qb][2]);
                x = max3(x, e_acc[0][qb][3], e_acc[1][qb][0]);
#pragma unroll
                for (int kb = 1; kb < 4; ++kb) {
                    x = max3(x, e_acc[kb][qb][1], e_acc[kb][qb][2]);
                    x = kb < 3 ? max3(x, e_acc[kb][qb][3], e_acc[kb + 1][qb][0]) : max2(x, e_acc[kb][qb][3]);
                }
                mx[qb] = x;
            }
            // the reference test; with these operands the exponents stay small and the branch (the row maxima across lanes)
            // is never taken, as in all but the first tiles of a real call
            if (__any(mx[0] > grow_at || mx[1] > grow_at)) m_run = fmaxf(m_run, fmaxf(max_across_quads(mx[0]), max_across_quads(mx[1])));
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
                for (int ck = 0; ck < 2; ++ck) {
                    uint32_t w4[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int kb = 2 * ck + (i >> 1), r = 2 * (i & 1);
                        w4[i] = T::pack2(fast_exp2(e_acc[kb][qb][r]), fast_exp2(e_acc[kb][qb][r + 1]));
                        ls = T::add_pair(w4[i], ls);
                    }
                    uint4 pu; pu.x = w4[0]; pu.y = w4[1]; pu.z = w4[2]; pu.w = w4[3];
                    pk[ck][qb] = __builtin_bit_cast(s16x8, pu);
                }
            }
            l_sum += ls;
        } else {
            // keep the first GEMM's result live without vector work on it: one register of each block joins the sink value
#pragma unroll
            for (int kb = 0; kb < 4; ++kb) l_sum += e_acc[kb][0][0] + e_acc[kb][1][0];
#pragma unroll
            for (int ck = 0; ck < 2; ++ck) { pk[ck][0] = qf[0][ck]; pk[ck][1] = qf[1][ck]; }
        }
#pragma unroll
        for (int ck = 0; ck < 2; ++ck) {
#pragma unroll
            for (int db = 0; db < 8; ++db) {
                s16x8 va;
                if (LDS_READS) {
                    const s16x4 t0 = lds_read_tr16(v_rd[db], (32 * ck) * RB);
                    const s16x4 t1 = lds_read_tr16(v_rd[db], (32 * ck + 16) * RB);
                    va = s16x8{t0[0], t0[1], t0[2], t0[3], t1[0], t1[1], t1[2], t1[3]};
                } else {
                    va = vreg[(ck + db) & 3];
                }
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) o_acc[db][qb] = T::mfma16(va, pk[ck][qb], o_acc[db][qb]);
            }
        }
    }
    float s = l_sum + m_run;
#pragma unroll
    for (int db = 0; db < 8; ++db)
#pragma unroll
        for (int r = 0; r < 4; ++r) s += o_acc[db][0][r] + o_acc[db][1][r];
    sink[(size_t)blockIdx.x * (kCalibWaves * 64) + threadIdx.x] = s;
}

}  // namespace minfer_attn

using namespace minfer_attn;

MINFER_ATTN_EXPORT int minfer_calib_attn_mix(int dtype, const void* operands, int64_t iters, int64_t workgroups, int lds_reads,
                                             int softmax, float* sink, void* stream_v) {
    clear_error();
    if (dtype != MINFER_ATTN_F16 && dtype != MINFER_ATTN_BF16)
        return fail(MINFER_ATTN_EINVAL, "calib_attn_mix: dtype must be MINFER_ATTN_F16 or MINFER_ATTN_BF16");
    if (!operands || !sink || !aligned16(operands)) return fail(MINFER_ATTN_EINVAL, "calib_attn_mix: operands (16-byte aligned) and sink must be non-null");
    if (iters < 0 || iters > (1 << 24) || workgroups <= 0 || workgroups > (1 << 20))
        return fail(MINFER_ATTN_EINVAL, "calib_attn_mix: iters must be in [0, 2^24] and workgroups in [1, 2^20]");
    hipStream_t stream = (hipStream_t)stream_v;
    const dim3 grid((unsigned)workgroups), block(kCalibWaves * 64);
    const s16x8* ops = (const s16x8*)operands;
    const int it = (int)iters;
#define MINFER_MIX(T, L, S) hipLaunchKernelGGL((attn_mix_kernel<T, L, S>), grid, block, 0, stream, ops, it, sink)
    if (dtype == MINFER_ATTN_F16) {
        if (lds_reads) { if (softmax) MINFER_MIX(F16, true, true); else MINFER_MIX(F16, true, false); }
        else { if (softmax) MINFER_MIX(F16, false, true); else MINFER_MIX(F16, false, false); }
    } else {
        if (lds_reads) { if (softmax) MINFER_MIX(BF16, true, true); else MINFER_MIX(BF16, true, false); }
        else { if (softmax) MINFER_MIX(BF16, false, true); else MINFER_MIX(BF16, false, false); }
    }
#undef MINFER_MIX
    return check_launch("attn_mix_kernel");
}

static int launch_mfma_rate(bool shape32, int dtype, const void* operands, int64_t iters, int64_t workgroups, float* sink, void* stream_v) {
    clear_error();
    if (dtype != MINFER_ATTN_F16 && dtype != MINFER_ATTN_BF16)
        return fail(MINFER_ATTN_EINVAL, "calib_mfma_rate: dtype must be MINFER_ATTN_F16 or MINFER_ATTN_BF16");
    if (!operands || !sink || !aligned16(operands)) return fail(MINFER_ATTN_EINVAL, "calib_mfma_rate: operands (16-byte aligned) and sink must be non-null");
    if (iters < 0 || iters > (1 << 24) || workgroups <= 0 || workgroups > (1 << 20))
        return fail(MINFER_ATTN_EINVAL, "calib_mfma_rate: iters must be in [0, 2^24] and workgroups in [1, 2^20]");
    hipStream_t stream = (hipStream_t)stream_v;
    const dim3 grid((unsigned)workgroups), block(kCalibWaves * 64);
    const s16x8* ops = (const s16x8*)operands;
    const int it = (int)iters;
    if (dtype == MINFER_ATTN_F16) {
        if (shape32) hipLaunchKernelGGL((mfma_rate_kernel<F16, true>), grid, block, 0, stream, ops, it, sink);
        else hipLaunchKernelGGL((mfma_rate_kernel<F16, false>), grid, block, 0, stream, ops, it, sink);
    } else {
        if (shape32) hipLaunchKernelGGL((mfma_rate_kernel<BF16, true>), grid, block, 0, stream, ops, it, sink);
        else hipLaunchKernelGGL((mfma_rate_kernel<BF16, false>), grid, block, 0, stream, ops, it, sink);
    }
    return check_launch("mfma_rate_kernel");
}

MINFER_ATTN_EXPORT int minfer_calib_mfma_rate(int dtype, const void* operands, int64_t iters, int64_t workgroups, float* sink,
                                              void* stream_v) {
    return launch_mfma_rate(false, dtype, operands, iters, workgroups, sink, stream_v);
}

MINFER_ATTN_EXPORT int minfer_calib_mfma_rate_32x32x16(int dtype, const void* operands, int64_t iters, int64_t workgroups, float* sink,
                                                       void* stream_v) {
    return launch_mfma_rate(true, dtype, operands, iters, workgroups, sink, stream_v);
}
