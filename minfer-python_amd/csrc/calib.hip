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

// The prefill kernel's per-tile instruction mix with everything removed that is not matrix, LDS-read or softmax work: no
// global->LDS copies, no barrier, no masking, no tile bookkeeping, the same K and V tile (64 keys x 128, written to LDS
// once) for every iteration.  Per "tile" a wave issues what the attention kernel issues for head_dim 128: 16 MFMAs for
// S^T = K Q^T with the K fragments read from LDS (16 ds_read_b128), the row maximum (16 v_max3 + a half swap), 32
// exponentials, 16 packs, 16 dot products for the denominator, and 16 MFMAs for O^T += V^T P^T with the V^T fragments
// from 32 transpose reads.  LDS_READS = false keeps the fragments in registers instead, SOFTMAX = false feeds the
// second GEMM from registers: the four combinations show what each kind of co-running work costs the matrix rate, and
// the full mix is what an attention kernel with no fixed costs at all would reach.
template <class T, bool LDS_READS, bool SOFTMAX>
__global__ __launch_bounds__(kCalibWaves * 64, 2) void attn_mix_kernel(const s16x8* __restrict__ operands, int iters,
                                                                        float* __restrict__ sink) {
    constexpr int RB = 256, TILE = 64 * RB;
    __shared__ __attribute__((aligned(1024))) char lds[2 * TILE];
    const int lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5, li = lane & 15, blk = lane >> 4;
    // fill both tiles from the 16 KiB of operands (K = the buffer, V = the buffer again)
    for (int i = threadIdx.x; i < 2 * TILE / 16; i += kCalibWaves * 64)
        reinterpret_cast<s16x8*>(lds)[i] = operands[i & (kCalibFrags * 64 - 1)];
    __syncthreads();
    s16x8 qf[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) qf[c] = T::scale8(operands[c * 64 + lane], 0.1275f);   // 1/sqrt(128) * log2(e)
    // conflict-free read addresses as in the attention kernel (XOR swizzles by row)
    uint32_t k_rd[8], v_rd[4];
#pragma unroll
    for (int c = 0; c < 8; ++c) k_rd[c] = lds_addr(lds) + l32 * RB + 16 * ((2 * c + h) ^ (l32 & 15));
    {
        const int vrow = 4 * h + (li >> 2), swv = (vrow & 3) << 2;
#pragma unroll
        for (int db = 0; db < 4; ++db) {
            const int dcol = 32 * db + 16 * (blk & 1) + 4 * (li & 3);
            v_rd[db] = lds_addr(lds) + TILE + vrow * RB + 16 * ((dcol >> 3) ^ swv) + 2 * (dcol & 7);
        }
    }
    s16x8 kreg[4], vreg[4];   // the register-resident operands of the variants without LDS reads
#pragma unroll
    for (int j = 0; j < 4; ++j) { kreg[j] = operands[(8 + j) * 64 + lane]; vreg[j] = operands[(12 + j) * 64 + lane]; }
    f32x16 o_acc[4], neg_ref;
#pragma unroll
    for (int r = 0; r < 16; ++r) { neg_ref[r] = 0.f; o_acc[0][r] = o_acc[1][r] = o_acc[2][r] = o_acc[3][r] = 0.f; }
    float l_sum = 0.f, m_run = 0.f;
    for (int it = 0; it < iters; ++it) {
        asm volatile("" ::: "memory");   // every iteration reads its fragments from LDS again, as a new tile would need
        f32x16 e_acc[2];
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const s16x8 k0 = LDS_READS ? lds_read_b128(k_rd[c], 0) : kreg[c & 3];
            const s16x8 k1 = LDS_READS ? lds_read_b128(k_rd[c], 32 * RB) : kreg[(c + 1) & 3];
            e_acc[0] = T::mfma32(k0, qf[c], c == 0 ? neg_ref : e_acc[0]);
            e_acc[1] = T::mfma32(k1, qf[c], c == 0 ? neg_ref : e_acc[1]);
        }
        s16x8 pk[4];
        if (SOFTMAX) {
            float mx = e_acc[0][0];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) mx = fmaxf(mx, e_acc[kb][r]);
            mx = max_across_halves(mx);
            m_run = fmaxf(m_run, mx);   // kept live; the reference itself never moves (the exponents stay small)
            float ls = 0.f;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                uint32_t w4[4];
#pragma unroll
                for (int i = 0; i < 8; i += 2) {
                    const int kb = c >> 1, r = 8 * (c & 1) + i;
                    w4[i >> 1] = T::pack2(fast_exp2(e_acc[kb][r]), fast_exp2(e_acc[kb][r + 1]));
                    ls = T::add_pair(w4[i >> 1], ls);
                }
                uint4 pu; pu.x = w4[0]; pu.y = w4[1]; pu.z = w4[2]; pu.w = w4[3];
                pk[c] = __builtin_bit_cast(s16x8, pu);
            }
            l_sum += ls;
        } else {
            // keep the first GEMM's result live without vector work on it: one register of it joins the sink value
            l_sum += e_acc[0][0] + e_acc[1][0];
#pragma unroll
            for (int c = 0; c < 4; ++c) pk[c] = qf[c];
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
#pragma unroll
            for (int db = 0; db < 4; ++db) {
                s16x8 va;
                if (LDS_READS) {
                    const s16x4 t0 = lds_read_tr16(v_rd[db], (16 * c) * RB);
                    const s16x4 t1 = lds_read_tr16(v_rd[db], (16 * c + 8) * RB);
                    va = s16x8{t0[0], t0[1], t0[2], t0[3], t1[0], t1[1], t1[2], t1[3]};
                } else {
                    va = vreg[(c + db) & 3];
                }
                o_acc[db] = T::mfma32(va, pk[c], o_acc[db]);
            }
        }
    }
    float s = l_sum + m_run;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += o_acc[db][r];
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
