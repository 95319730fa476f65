// Single-token decode attention for gfx950: split-KV partial kernel + log-sum-exp combine.
//
// The op is HBM-bound (each K/V byte is used once per query head of its GQA group), so the
// design goal is bytes in flight, not FLOPs.  A workgroup (4 waves) owns one (sequence, KV
// head, chunk of `chunk` cache rows).  Every wave runs a private two-stage pipeline over
// 16-row groups of that chunk: K and V rows are copied global->LDS directly (full 256-byte rows,
// no VGPRs held while in flight), the wave waits on its own vmcnt only -- no workgroup barrier
// in the loop -- and while one stage is consumed the other is in flight.  With two workgroups
// per CU about 100 KB per CU are in flight.
//
// Compute per group: S^T[16 keys x 16 heads] = K Q^T (16x16x32 MFMA; the GQA group's query heads
// are the 16 columns, unused columns are zero), online softmax per head (a lane holds 4 keys of
// one head), then O^T[D x heads] += V^T P^T with 16x16x16 MFMAs whose B operand is the score
// registers as they are and whose A operand comes from LDS transpose reads.
//
// Every (sequence, head, chunk) writes an un-normalised fp32 partial (O, max, sum) to the
// workspace; the combine kernel merges the chunks of a row with the usual log-sum-exp weights.
#include "attn_common.h"
#include "attn_host.h"

namespace minfer_attn {

constexpr int kDecodeWaves = 4;
constexpr int kGroupRows = 16;   // cache rows per pipeline stage of one wave

struct DecodeParams {
    const void* q; const void* k; const void* v;
    const int32_t* ctx;
    float* part_o;   // [B][Hq][S][D]
    float* part_ml;  // [B][Hq][S][2]: reference max (raw score units), sum
    int64_t q0, q1, kv0, kv1, kv2;
    int B, Hq, Hkv, n_rep, Lmax;
    int chunk;       // cache rows per workgroup (multiple of 64)
    int S;           // chunks per sequence = ceil(Lmax / chunk)
    int n_hg;        // head groups of <= 16 heads per KV head
    float scale_log2;
};

template <int D> struct DecodeGeom {
    static constexpr int RB = D * 2;
    static constexpr int G = RB / 16;
    static constexpr int RPI = 1024 / RB;              // rows per copy instruction
    static constexpr int NI = kGroupRows / RPI;        // copy instructions per tensor per group
    static constexpr int RPW = 256 / RB;
    static constexpr int STAGE_BYTES = 2 * kGroupRows * RB;   // K rows then V rows
    static MA_DEV int swz_k(int row) { return (row / RPW) & (G - 1); }
    // transpose reads touch 8 rows x 32 bytes per half-wave: spread the 32-byte chunks over the banks
    static MA_DEV int swz_v(int row) { return D == 128 ? ((row & 7) << 1) : (((row >> 1) & 3) << 1); }
};

template <class T, int D>
__global__ __launch_bounds__(kDecodeWaves * 64, 2) void decode_split_kernel(const DecodeParams p) {
    using GEO = DecodeGeom<D>;
    constexpr int RB = GEO::RB, G = GEO::G, RPI = GEO::RPI, NI = GEO::NI;
    constexpr int KC = D / 32;   // 32-wide contraction chunks of K Q^T
    constexpr int DB = D / 16;   // 16-row blocks of O^T
    constexpr int kWaveLds = 2 * GEO::STAGE_BYTES;
    constexpr int PS = D + 4;    // floats per head in a wave's partial result (O, max, sum, pad)
    static_assert(kWaveLds >= 16 * PS * 4, "per-wave LDS also holds the wave's partial result");

    __shared__ __attribute__((aligned(1024))) char lds[kDecodeWaves][kWaveLds];

    const int tid = threadIdx.x, lane = tid & 63, w = wave_id();
    const int l16 = lane & 15, quad = lane >> 4;
    const int split = blockIdx.x;
    const int g = blockIdx.y % p.Hkv, hg = blockIdx.y / p.Hkv;
    const int b = blockIdx.z;

    const int ctx = min(max(p.ctx[b], 0), p.Lmax);
    const int row_lo = split * p.chunk;
    if (row_lo >= ctx) return;                       // chunk entirely beyond this sequence
    const int row_hi = min(row_lo + p.chunk, ctx);
    const int n_groups = (row_hi - row_lo + kGroupRows - 1) / kGroupRows;
    const int my_groups = (n_groups - w + kDecodeWaves - 1) / kDecodeWaves;  // groups w, w+4, ...

    const int heads_here = min(16, p.n_rep - hg * 16);
    const int head0 = g * p.n_rep + hg * 16;
    const short* Kb = (const short*)p.k + (int64_t)b * p.kv0 + (int64_t)g * p.kv1;
    const short* Vb = (const short*)p.v + (int64_t)b * p.kv0 + (int64_t)g * p.kv1;
    char* my_lds = lds[w];

    // ---- Q^T fragments (B operand): column = head l16, k = d = 32c + 8*quad + 0..7 ------------
    s16x8 qf[KC];
    {
        const bool valid = l16 < heads_here;
        const short* src = (const short*)p.q + (int64_t)b * p.q0 + (int64_t)(head0 + (valid ? l16 : 0)) * p.q1 + 8 * quad;
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            s16x8 x = *reinterpret_cast<const s16x8*>(src + 32 * c);
            if (!valid) x = s16x8{0, 0, 0, 0, 0, 0, 0, 0};
            qf[c] = x;
        }
    }

    auto issue_group = [&](int gi, int stage) {  // gi = group index inside the chunk
        const int r0 = row_lo + gi * kGroupRows;
        char* kdst = my_lds + stage * GEO::STAGE_BYTES;
        char* vdst = kdst + kGroupRows * RB;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int row = j * RPI + lane / G;
            const int pg = lane % G;
            const int64_t grow = (int64_t)min(r0 + row, row_hi - 1) * p.kv2;
            copy16_global_to_lds(Kb + grow + 8 * (pg ^ GEO::swz_k(row)), kdst + j * 1024);
        }
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int row = j * RPI + lane / G;
            const int pg = lane % G;
            const int64_t grow = (int64_t)min(r0 + row, row_hi - 1) * p.kv2;
            copy16_global_to_lds(Vb + grow + 8 * (pg ^ GEO::swz_v(row)), vdst + j * 1024);
        }
    };

    f32x4 o_acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) o_acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_ref = -INFINITY, l_sum = 0.f;
    const float c2 = p.scale_log2;
    constexpr float kLazyLog2 = 6.f;

    if (my_groups > 0) issue_group(w, 0);
    if (my_groups > 1) issue_group(w + kDecodeWaves, 1);

    for (int i = 0; i < my_groups; ++i) {
        const int stage = i & 1;
        const int gi = w + i * kDecodeWaves;
        // the copies of group i are older than those of group i+1 (if any): wait for all but the newest 2*NI
        if (i + 1 < my_groups) wait_vmcnt<2 * NI>();
        else wait_vmcnt<0>();
        const char* kst = my_lds + stage * GEO::STAGE_BYTES;
        const char* vst = kst + kGroupRows * RB;

        // ---- S^T = K Q^T: lane gets head l16, keys 4*quad + r --------------------------------
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
        {
            const char* rowp = kst + l16 * RB;
            const int sw = GEO::swz_k(l16);
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                const s16x8 a = *reinterpret_cast<const s16x8*>(rowp + 16 * ((4 * c + quad) ^ sw));
                s = T::mfma16(a, qf[c], s);
            }
        }
        const int key0 = row_lo + gi * kGroupRows + 4 * quad;
        if (key0 + 4 > row_hi) {
#pragma unroll
            for (int r = 0; r < 4; ++r) s[r] = (key0 + r < row_hi) ? s[r] : -INFINITY;
        }

        // ---- online softmax over this group's 16 keys ------------------------------------------
        float mx = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const bool grow = (mx - m_ref) * c2 > kLazyLog2 || (m_ref == -INFINITY && mx > -INFINITY);
        if (__any(grow)) {
            const float m_new = grow ? mx : m_ref;
            const float alpha = (m_ref == -INFINITY) ? 0.f : fast_exp2((m_ref - m_new) * c2);
            m_ref = m_new;
            l_sum *= alpha;
#pragma unroll
            for (int db = 0; db < DB; ++db) o_acc[db] *= alpha;
        }
        const float mc = (m_ref == -INFINITY) ? 0.f : m_ref * c2;
        const float p0 = fast_exp2(fmaf(s[0], c2, -mc)), p1 = fast_exp2(fmaf(s[1], c2, -mc));
        const float p2 = fast_exp2(fmaf(s[2], c2, -mc)), p3 = fast_exp2(fmaf(s[3], c2, -mc));
        uint2 pu; pu.x = T::pack2(p0, p1); pu.y = T::pack2(p2, p3);
        l_sum = T::add_pair(pu.y, T::add_pair(pu.x, l_sum));   // sums the rounded weights the MFMA uses
        const s16x4 pfrag = __builtin_bit_cast(s16x4, pu);

        // ---- O^T += V^T P^T: A = V^T block (row d = 16db + l16, k = keys 4*quad + 0..3) -----------
        {
            const int row = 4 * quad + (l16 >> 2);
            const char* rowp = vst + row * RB;
            const int sw = GEO::swz_v(row);
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const int dcol = 16 * db + 4 * (l16 & 3);
                const s16x4 a = lds_read_tr16(rowp + 16 * ((dcol >> 3) ^ sw) + 2 * (dcol & 7));
                o_acc[db] = T::mfma16k16(a, pfrag, o_acc[db]);
            }
        }

        if (i + 2 < my_groups) {
            issue_group(gi + 2 * kDecodeWaves, stage);   // refill the stage just consumed
        }
    }

    // ---- merge the four waves' partial results through LDS, write the chunk's partial ----------
    l_sum += __shfl_xor(l_sum, 16);
    l_sum += __shfl_xor(l_sum, 32);
    float* mine = reinterpret_cast<float*>(my_lds);   // [16 heads][PS]
    if (l16 < heads_here) {
#pragma unroll
        for (int db = 0; db < DB; ++db) *reinterpret_cast<f32x4*>(mine + l16 * PS + 16 * db + 4 * quad) = o_acc[db];
        if (quad == 0) { mine[l16 * PS + D] = m_ref; mine[l16 * PS + D + 1] = l_sum; }
    }
    __syncthreads();
    for (int idx = tid; idx < heads_here * D; idx += kDecodeWaves * 64) {
        const int hh = idx / D, d = idx % D;
        float M = -INFINITY;
#pragma unroll
        for (int ww = 0; ww < kDecodeWaves; ++ww) {
            const float* src = reinterpret_cast<const float*>(lds[ww]) + hh * PS;
            if (ww < n_groups) M = fmaxf(M, src[D]);
        }
        float o = 0.f, l = 0.f;
#pragma unroll
        for (int ww = 0; ww < kDecodeWaves; ++ww) {
            const float* src = reinterpret_cast<const float*>(lds[ww]) + hh * PS;
            if (ww < n_groups && src[D] > -INFINITY) {
                const float wgt = fast_exp2((src[D] - M) * c2);
                o += src[d] * wgt;
                l += src[D + 1] * wgt;
            }
        }
        const int64_t slot = ((int64_t)b * p.Hq + head0 + hh) * p.S + split;
        p.part_o[slot * D + d] = o;
        if (d == 0) { p.part_ml[slot * 2] = M; p.part_ml[slot * 2 + 1] = l; }
    }
}

// out[b,h,:] = sum_s O_s w_s / sum_s l_s w_s with w_s = 2^((m_s - max m) * scale_log2).
// grid (Hq, B), block D threads.
template <class T, int D>
__global__ __launch_bounds__(D) void decode_combine_kernel(const DecodeParams p, void* out, int64_t o0, int64_t o1) {
    const int hq = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
    const int ctx = min(max(p.ctx[b], 0), p.Lmax);
    const int ns = (ctx + p.chunk - 1) / p.chunk;
    const int64_t slot0 = ((int64_t)b * p.Hq + hq) * p.S;
    float M = -INFINITY;
    for (int s = 0; s < ns; ++s) M = fmaxf(M, p.part_ml[(slot0 + s) * 2]);
    float o = 0.f, l = 0.f;
    for (int s = 0; s < ns; ++s) {
        const float m = p.part_ml[(slot0 + s) * 2];
        if (m > -INFINITY) {
            const float wgt = fast_exp2((m - M) * p.scale_log2);
            o += p.part_o[(slot0 + s) * D + d] * wgt;
            l += p.part_ml[(slot0 + s) * 2 + 1] * wgt;
        }
    }
    const float r = l > 0.f ? o / l : 0.f;
    const uint32_t pk = T::pack2(r, 0.f);
    reinterpret_cast<uint16_t*>(out)[(int64_t)b * o0 + (int64_t)hq * o1 + d] = (uint16_t)(pk & 0xffffu);
}

constexpr int kDecodeChunk = 512;

static size_t decode_ws_bytes(int64_t B, int64_t Hq, int64_t Lmax, int64_t D) {
    const int64_t S = (Lmax + kDecodeChunk - 1) / kDecodeChunk;
    return (size_t)(B * Hq * S * (D + 2) * 4 + 255) / 256 * 256 + 256;
}

template <class T, int D>
static int launch_decode(const DecodeParams& p, void* out, int64_t o0, int64_t o1, hipStream_t stream) {
    hipLaunchKernelGGL((decode_split_kernel<T, D>), dim3(p.S, p.Hkv * p.n_hg, p.B), dim3(kDecodeWaves * 64), 0, stream, p);
    if (int rc = check_launch("decode_split_kernel")) return rc;
    hipLaunchKernelGGL((decode_combine_kernel<T, D>), dim3(p.Hq, p.B), dim3(D), 0, stream, p, out, o0, o1);
    return check_launch("decode_combine_kernel");
}

}  // namespace minfer_attn

using namespace minfer_attn;

MINFER_ATTN_EXPORT size_t minfer_flash_attn_decode_workspace_bytes(int64_t B, int64_t Hq, int64_t Lmax, int64_t D) {
    if (B <= 0 || Hq <= 0 || Lmax <= 0 || D <= 0) return 256;
    return decode_ws_bytes(B, Hq, Lmax, D);
}

MINFER_ATTN_EXPORT int minfer_flash_attn_decode(int dtype, const void* q, const void* k_cache, const void* v_cache,
                                        const int32_t* ctx_lens, void* out, int64_t B, int64_t Hq, int64_t Hkv,
                                        int64_t Lmax, int64_t D, const minfer_attn_strides* st, void* workspace,
                                        size_t workspace_bytes, void* stream_v) {
    clear_error();
    if (int rc = check_common(dtype, q, k_cache, v_cache, out, Hq, Hkv, D, st)) return rc;
    if (!ctx_lens) return fail(MINFER_ATTN_EINVAL, "flash_attn_decode: ctx_lens is null");
    if (B < 0 || Lmax < 0) return fail(MINFER_ATTN_EINVAL, "flash_attn_decode: negative B or Lmax");
    if (B == 0) return MINFER_ATTN_OK;
    if (B > 65535 || Hq > 65535) return fail(MINFER_ATTN_EINVAL, "flash_attn_decode: B or n_heads > 65535 unsupported");
    if (Lmax > (1 << 30)) return fail(MINFER_ATTN_EINVAL, "flash_attn_decode: Lmax too large");
    if (!workspace || workspace_bytes < decode_ws_bytes(B, Hq, Lmax, D) || !aligned16(workspace))
        return fail(MINFER_ATTN_EWORKSPACE, "flash_attn_decode: workspace too small or misaligned (see minfer_flash_attn_decode_workspace_bytes)");
    hipStream_t stream = (hipStream_t)stream_v;

    DecodeParams p{};
    p.q = q; p.k = k_cache; p.v = v_cache; p.ctx = ctx_lens;
    p.q0 = st->q0; p.q1 = st->q1; p.kv0 = st->kv0; p.kv1 = st->kv1; p.kv2 = st->kv2;
    p.B = (int)B; p.Hq = (int)Hq; p.Hkv = (int)Hkv; p.n_rep = (int)(Hq / Hkv); p.Lmax = (int)Lmax;
    p.chunk = kDecodeChunk;
    p.S = (int)((Lmax + kDecodeChunk - 1) / kDecodeChunk);
    if (p.S < 1) p.S = 1;
    p.n_hg = (p.n_rep + 15) / 16;
    p.scale_log2 = (float)(1.4426950408889634 / sqrt((double)D));
    const size_t o_bytes = (size_t)B * Hq * p.S * D * 4;
    p.part_o = (float*)workspace;
    p.part_ml = (float*)((char*)workspace + (o_bytes + 255) / 256 * 256);

    if (dtype == MINFER_ATTN_F16)
        return D == 128 ? launch_decode<F16, 128>(p, out, st->o0, st->o1, stream) : launch_decode<F16, 64>(p, out, st->o0, st->o1, stream);
    return D == 128 ? launch_decode<BF16, 128>(p, out, st->o0, st->o1, stream) : launch_decode<BF16, 64>(p, out, st->o0, st->o1, stream);
}
