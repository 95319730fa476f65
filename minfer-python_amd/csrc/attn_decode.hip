// Single-token decode attention for gfx950: split-KV partial kernel + log-sum-exp combine.
//
// The op is HBM-bound (each K/V byte is used once per query head of its GQA group), so the
// design goal is bytes in flight, not FLOPs.  A workgroup (4 waves) owns one (sequence, KV
// head, chunk of `chunk` cache rows); only chunks that exist are enumerated (a wave-level prefix
// sum over ctx_lens maps the linear chunk id to its sequence), so no workgroup is launched just
// to find out that it has nothing to do while others wait for its slot.  Every wave runs a
// private NS-deep register ring over 16-row groups of the chunk: K rows are loaded straight into
// the MFMA A-operand layout, V rows as full 256-byte rows; the wave waits only on its own loads
// -- no workgroup barrier in the loop -- and with 8 waves per CU and NS-1 groups of 8 KB in
// flight per wave well over 100 KB per CU are outstanding.
//
// Compute per group: S^T[16 keys x 16 heads] = K Q^T (16x16x32 MFMA; the GQA group's query heads
// are the 16 columns, unused columns are zero), online softmax per head (a lane holds 4 keys of
// one head), then O^T[D x heads] += V^T P^T with 16x16x16 MFMAs whose B operand is the score
// registers as they are and whose A operand comes from LDS transpose reads of the V rows the
// wave has just parked in its private 4 KB of LDS.
//
// Every (sequence, head, chunk) writes an un-normalised fp32 partial (O, max, sum) to the
// workspace; the combine kernel merges the chunks of a row with the usual log-sum-exp weights.
#include "attn_common.h"
#include "attn_host.h"

namespace minfer_attn {

// Tunables (overridable at compile time for sweeps).
#ifndef MINFER_DECODE_WAVES
#define MINFER_DECODE_WAVES 4
#endif
#ifndef MINFER_DECODE_STAGES
#define MINFER_DECODE_STAGES 3
#endif
#ifndef MINFER_DECODE_MIN_WAVES_PER_SIMD
#define MINFER_DECODE_MIN_WAVES_PER_SIMD 2
#endif
constexpr int kDecodeWaves = MINFER_DECODE_WAVES;
constexpr int kGroupRows = 16;   // cache rows per ring slot of one wave
constexpr int kDecodeStages = MINFER_DECODE_STAGES; // ring depth

struct DecodeParams {
    const void* q; const void* k; const void* v;
    const int32_t* ctx;
    float* part_o;   // [B][Hq][S][D]
    float* part_ml;  // [B][Hq][S][2]: reference max (raw score units), sum
    int64_t q0, q1, kv0, kv1, kv2;
    int B, Hq, Hkv, n_rep, Lmax;
    int chunk;       // cache rows per workgroup (multiple of 64)
    int S;           // chunks per sequence = ceil(Lmax / chunk), at most 64
    int n_hg;        // head groups of <= 16 heads per KV head
    float scale_log2;
};

MA_DEV int chunks_of(int ctx, int Lmax, int chunk) { return (min(max(ctx, 0), Lmax) + chunk - 1) / chunk; }

// Maps a linear chunk id to (sequence, chunk inside the sequence) by a wave-wide inclusive scan of
// the per-sequence chunk counts; returns false when the id is past the last chunk.
MA_DEV bool locate_chunk(const DecodeParams& p, int id, int lane, int& b_out, int& split_out, int& ctx_out) {
    int offset = 0;
    for (int base = 0; base < p.B; base += 64) {
        const int b = base + lane;
        const int c = b < p.B ? p.ctx[b] : 0;
        const int n = chunks_of(c, p.Lmax, p.chunk);
        int incl = n;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d);
            if (lane >= d) incl += up;
        }
        const int total = __builtin_amdgcn_readfirstlane(__shfl(incl, 63));   // wave-uniform, and known to be
        if (id < offset + total) {
            const uint64_t hit = __ballot(id < offset + incl);
            const int src = __ffsll((unsigned long long)hit) - 1;
            // every lane holds the same values; saying so keeps the kernel's control flow (and with it
            // the compiler's wait-count bookkeeping in the main loop) scalar
            b_out = __builtin_amdgcn_readfirstlane(base + src);
            split_out = __builtin_amdgcn_readfirstlane(id - offset - __shfl(incl - n, src));
            ctx_out = __builtin_amdgcn_readfirstlane(__shfl(c, src));
            return true;
        }
        offset += total;
    }
    return false;
}

template <int D> struct DecodeGeom {
    static constexpr int RB = D * 2;
    static constexpr int G = RB / 16;
    static constexpr int RPI = 1024 / RB;              // rows one wave-wide 16-byte load covers
    static constexpr int NI = kGroupRows / RPI;        // such loads per group of V rows
    // transpose reads touch 8 rows x 32 bytes per half-wave: spread the 32-byte chunks over the banks
    static MA_DEV int swz_v(int row) { return D == 128 ? ((row & 7) << 1) : (((row >> 1) & 3) << 1); }
    // K rows are read back 16 rows x one 16-byte granule at a time
    static MA_DEV int swz_k(int row) { return D == 128 ? (row & 15) : ((row >> 1) & 7); }
};

template <class T, int D>
__global__ __launch_bounds__(kDecodeWaves * 64, MINFER_DECODE_MIN_WAVES_PER_SIMD) void decode_split_kernel(const DecodeParams p) {
    using GEO = DecodeGeom<D>;
    constexpr int RB = GEO::RB, G = GEO::G, RPI = GEO::RPI, NI = GEO::NI;
    constexpr int KC = D / 32;   // 32-wide contraction chunks of K Q^T
    constexpr int DB = D / 16;   // 16-row blocks of O^T
    constexpr int NS = kDecodeStages;
    constexpr int PS = D + 4;    // floats per head in a wave's partial result (O, max, sum, pad)

    __shared__ __attribute__((aligned(1024))) char v_lds[kDecodeWaves][kGroupRows * RB];
    __shared__ __attribute__((aligned(1024))) char k_lds[kDecodeWaves][kGroupRows * RB];
    __shared__ __attribute__((aligned(16))) float part_lds[kDecodeWaves][16 * PS];

    const int tid = threadIdx.x, lane = tid & 63, w = wave_id();
    const int l16 = lane & 15, quad = lane >> 4;
    const int per_chunk = p.Hkv * p.n_hg;
    const int y = blockIdx.x % per_chunk;
    const int g = y % p.Hkv, hg = y / p.Hkv;
    int b, split, ctx_raw;
    if (!locate_chunk(p, blockIdx.x / per_chunk, lane, b, split, ctx_raw)) return;   // past the last chunk

    const int ctx = min(max(ctx_raw, 0), p.Lmax);
    const int row_lo = split * p.chunk;
    const int row_hi = min(row_lo + p.chunk, ctx);
    const int n_groups = (row_hi - row_lo + kGroupRows - 1) / kGroupRows;
    const int my_groups = (n_groups - w + kDecodeWaves - 1) / kDecodeWaves;  // groups w, w+4, ...
    auto group_of = [&](int t) { return w + t * kDecodeWaves; };
    auto wave_has_work = [&](int ww) { return ww < n_groups; };

    const int heads_here = min(16, p.n_rep - hg * 16);
    const int head0 = g * p.n_rep + hg * 16;
    const short* Kb = (const short*)p.k + (int64_t)b * p.kv0 + (int64_t)g * p.kv1;
    const short* Vb = (const short*)p.v + (int64_t)b * p.kv0 + (int64_t)g * p.kv1;
    char* my_v = v_lds[w];
    char* my_k = k_lds[w];

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

    // ring of groups in flight: K and V as full rows (16 lanes x 16 bytes per row)
    s16x8 kr[NS][NI], vr[NS][NI];
    static_assert(NI == KC, "a 16-row group is NI row loads and KC contraction chunks");
    auto load_group = [&](int t, s16x8 (&kk)[NI], s16x8 (&vv)[NI]) {
        const int r0 = row_lo + group_of(t) * kGroupRows;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int row = j * RPI + lane / G;
            kk[j] = *reinterpret_cast<const s16x8*>(Kb + (int64_t)min(r0 + row, row_hi - 1) * p.kv2 + 8 * (lane % G));
        }
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int row = j * RPI + lane / G;
            vv[j] = *reinterpret_cast<const s16x8*>(Vb + (int64_t)min(r0 + row, row_hi - 1) * p.kv2 + 8 * (lane % G));
        }
    };
    // Loads and the consume step below are issued unconditionally (rows are clamped into the chunk and
    // out-of-range keys masked), so the loop body is straight-line code and the compiler's wait
    // counts let NS-1 groups stay in flight instead of draining the queue at every branch join.
#pragma unroll
    for (int s = 0; s < NS; ++s) load_group(s, kr[s], vr[s]);

    f32x4 o_acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) o_acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_ref = -INFINITY, l_sum = 0.f;
    const float c2 = p.scale_log2;
    constexpr float kLazyLog2 = 6.f;

    auto consume = [&](int t, const s16x8 (&kk)[NI], const s16x8 (&vv)[NI]) {
        // ---- S^T = K Q^T: lane gets head l16, keys 4*quad + r --------------------------------
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
        {   // park the K rows in LDS (swizzled) and read them back as A operands (row l16, d = 32c + 8*quad + 0..7)
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int row = j * RPI + lane / G;
                *reinterpret_cast<s16x8*>(my_k + row * RB + 16 * ((lane % G) ^ GEO::swz_k(row))) = kk[j];
            }
            const char* rowp = my_k + l16 * RB;
            const int sw = GEO::swz_k(l16);
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                const s16x8 a = *reinterpret_cast<const s16x8*>(rowp + 16 * ((4 * c + quad) ^ sw));
                s = T::mfma16(a, qf[c], s);
            }
        }
        const int key0 = row_lo + group_of(t) * kGroupRows + 4 * quad;
#pragma unroll
        for (int r = 0; r < 4; ++r) s[r] = (key0 + r < row_hi) ? s[r] : -INFINITY;
        // ---- park the V rows in LDS (swizzled) for the transpose reads -------------------------
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int row = j * RPI + lane / G;
            *reinterpret_cast<s16x8*>(my_v + row * RB + 16 * ((lane % G) ^ GEO::swz_v(row))) = vv[j];
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
            const char* rowp = my_v + row * RB;
            const int sw = GEO::swz_v(row);
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const int dcol = 16 * db + 4 * (l16 & 3);
                const s16x4 a = lds_read_tr16(rowp + 16 * ((dcol >> 3) ^ sw) + 2 * (dcol & 7));
                o_acc[db] = T::mfma16k16(a, pfrag, o_acc[db]);
            }
        }
    };

    for (int t0 = 0; t0 < my_groups; t0 += NS) {
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            consume(t0 + s, kr[s], vr[s]);
            load_group(t0 + s + NS, kr[s], vr[s]);
        }
    }

    // ---- merge the four waves' partial results through LDS, write the chunk's partial ----------
    l_sum += __shfl_xor(l_sum, 16);
    l_sum += __shfl_xor(l_sum, 32);
    float* mine = part_lds[w];   // [16 heads][PS]
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
        for (int ww = 0; ww < kDecodeWaves; ++ww)
            if (wave_has_work(ww)) M = fmaxf(M, part_lds[ww][hh * PS + D]);
        float o = 0.f, l = 0.f;
#pragma unroll
        for (int ww = 0; ww < kDecodeWaves; ++ww) {
            const float* src = part_lds[ww] + hh * PS;
            if (wave_has_work(ww) && src[D] > -INFINITY) {
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
// One wave per (sequence, head) row; lane s holds chunk s's (max, sum), every lane owns D/64
// output elements.  grid ceil(B*Hq/4), 256 threads.
template <class T, int D>
__global__ __launch_bounds__(256) void decode_combine_kernel(const DecodeParams p, void* out, int64_t o0, int64_t o1) {
    constexpr int EPL = D / 64;   // output elements per lane
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + wave_id();
    if (row >= p.B * p.Hq) return;
    const int b = row / p.Hq, hq = row % p.Hq;
    const int ns = chunks_of(p.ctx[b], p.Lmax, p.chunk);
    const int64_t slot0 = (int64_t)row * p.S;
    float m = -INFINITY, l = 0.f;
    if (lane < ns) { m = p.part_ml[(slot0 + lane) * 2]; l = p.part_ml[(slot0 + lane) * 2 + 1]; }
    float M = m;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) M = fmaxf(M, __shfl_xor(M, d));
    const float wgt = (m > -INFINITY) ? fast_exp2((m - M) * p.scale_log2) : 0.f;
    float L = l * wgt;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) L += __shfl_xor(L, d);
    float acc[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] = 0.f;
    const float* src = p.part_o + slot0 * D + EPL * lane;
    for (int s0 = 0; s0 < ns; s0 += 8) {   // 8 chunk partials at a time, all loads in flight together
        float x[8][EPL];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float* ptr = src + (int64_t)min(s0 + u, ns - 1) * D;
            if (EPL == 2) {
                const f32x2 v2 = *reinterpret_cast<const f32x2*>(ptr);
                x[u][0] = v2[0]; x[u][EPL - 1] = v2[1];
            } else {
                x[u][0] = ptr[0];
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float ws = (s0 + u < ns) ? __shfl(wgt, s0 + u) : 0.f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[e] += x[u][e] * ws;
        }
    }
    const float inv = L > 0.f ? 1.f / L : 0.f;
    uint16_t* dst = reinterpret_cast<uint16_t*>(out) + (int64_t)b * o0 + (int64_t)hq * o1 + EPL * lane;
    if (EPL == 2) {
        *reinterpret_cast<uint32_t*>(dst) = T::pack2(acc[0] * inv, acc[EPL - 1] * inv);
    } else {
        dst[0] = (uint16_t)(T::pack2(acc[0] * inv, 0.f) & 0xffffu);
    }
}

// Cache rows per workgroup.  Smallest: 256 (or more for very long caches, so that a row never has more
// than 64 chunks, which is what one wave of the combine kernel merges).  Larger chunks mean fewer
// partials and fewer workgroup start-ups, so the launcher doubles the chunk while the grid would still
// hold well over a thousand workgroups.  The workspace is sized for the smallest chunk.
static int decode_min_chunk_rows(int64_t Lmax) {
    int64_t c = (Lmax + 63) / 64;
    c = (c + 63) / 64 * 64;
    return (int)(c > 256 ? c : 256);
}
static int decode_chunk_rows(int64_t B, int64_t Hkv, int64_t n_hg, int64_t Lmax) {
#ifdef MINFER_DECODE_CHUNK
    const int forced = MINFER_DECODE_CHUNK;
    return forced > decode_min_chunk_rows(Lmax) ? forced : decode_min_chunk_rows(Lmax);
#else
    int chunk = decode_min_chunk_rows(Lmax);
    while (chunk < 1024 && B * Hkv * n_hg * ((Lmax + 2 * chunk - 1) / (2 * chunk)) >= 2048) chunk *= 2;
    return chunk;
#endif
}

static size_t decode_ws_bytes(int64_t B, int64_t Hq, int64_t Lmax, int64_t D) {
    const int64_t chunk = decode_min_chunk_rows(Lmax);
    const int64_t S = (Lmax + chunk - 1) / chunk;
    return (size_t)(B * Hq * S * (D + 2) * 4 + 255) / 256 * 256 + 256;
}

template <class T, int D>
static int launch_decode(const DecodeParams& p, void* out, int64_t o0, int64_t o1, hipStream_t stream) {
    // chunk id is the slow index, so every chunk that exists is dispatched before the ids past the end
    const int64_t grid = (int64_t)p.B * p.S * p.Hkv * p.n_hg;
    hipLaunchKernelGGL((decode_split_kernel<T, D>), dim3((unsigned)grid), dim3(kDecodeWaves * 64), 0, stream, p);
    if (int rc = check_launch("decode_split_kernel")) return rc;
    hipLaunchKernelGGL((decode_combine_kernel<T, D>), dim3((p.B * p.Hq + 3) / 4), dim3(256), 0, stream, p, out, o0, o1);
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
    p.n_hg = (p.n_rep + 15) / 16;
    p.chunk = decode_chunk_rows(B, Hkv, p.n_hg, Lmax);
    p.S = (int)((Lmax + p.chunk - 1) / p.chunk);
    if (p.S < 1) p.S = 1;
    if ((int64_t)B * p.S * Hkv * ((Hq / Hkv + 15) / 16) > 0x7fffffffLL)
        return fail(MINFER_ATTN_EINVAL, "flash_attn_decode: problem too large for one launch");
    p.scale_log2 = (float)(1.4426950408889634 / sqrt((double)D));
    const size_t o_bytes = (size_t)B * Hq * p.S * D * 4;
    p.part_o = (float*)workspace;
    p.part_ml = (float*)((char*)workspace + (o_bytes + 255) / 256 * 256);

    if (dtype == MINFER_ATTN_F16)
        return D == 128 ? launch_decode<F16, 128>(p, out, st->o0, st->o1, stream) : launch_decode<F16, 64>(p, out, st->o0, st->o1, stream);
    return D == 128 ? launch_decode<BF16, 128>(p, out, st->o0, st->o1, stream) : launch_decode<BF16, 64>(p, out, st->o0, st->o1, stream);
}
