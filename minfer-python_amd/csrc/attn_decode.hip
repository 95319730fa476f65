// Single-token decode attention for gfx950: split-KV partial kernel + log-sum-exp combine.
//
// The op is HBM-bound (each K/V byte is used once per query head of its GQA group), so the design goal is
// bytes in flight, not FLOPs.  All the cache rows that have to be read -- every sequence, every KV head, rows
// 0..ctx-1 -- are laid out on one line in 16-row groups, and the line is cut into as many equal shares as the
// chip holds waves of this kernel (two workgroups of four waves per compute unit): a wave streams its share
// from start to end on its own, with no barrier and no exchange with its neighbours, and all waves finish
// together whatever the mix of context lengths.  Where a share crosses from one (sequence, KV head) to the next
// the wave writes the partial result of the piece it has finished (a segment) and goes on.
//
// Every wave runs a private NS-deep register ring over its 16-row groups: K and V rows are loaded as full
// 256-byte rows; the wave waits only on its own loads, and with 8 waves per CU and NS-1 groups of 8 KB in
// flight per wave well over 100 KB per CU are outstanding.
//
// Compute per group: S^T[16 keys x 16 heads] = K Q^T (16x16x32 MFMA; the GQA group's query heads
// are the 16 columns, unused columns are zero), online softmax per head (a lane holds 4 keys of
// one head), then O^T[D x heads] += V^T P^T with 16x16x16 MFMAs whose B operand is the score
// registers as they are and whose A operand comes from LDS transpose reads of the V rows the
// wave has just parked in its private 4 KB of LDS (K goes through the wave's other 4 KB the same way).
//
// Every segment writes an un-normalised fp32 partial (O, max, sum) to the workspace; the combine kernel
// merges the partials of a (sequence, head) with the usual log-sum-exp weights.
//
// Q8_0 caches (decode_split_q8_kernel): a cache row is D/32 blocks of 34 bytes, an fp16 scale d followed by
// 32 int8 (reference: src/minfer/kernels/torch_ext/csrc/common/types.hpp:141-146), so blocks start on 2-byte
// boundaries.  Global memory is read in aligned 16-byte pieces all the same (2-byte-aligned wide loads run at a
// fraction of the rate): a wave's ring holds 32-row groups as the flat run of aligned pieces that covers them,
// the pieces are dropped into the wave's LDS area, and every lane picks its own blocks out of it as aligned
// words.  A block becomes the 32 fp16 values (half)(q * d) the reference's dequantiser produces
// (reference: cuda/quants/impls.cuh:121-143).  K needs no further LDS pass: lane (key, quad) holds values
// D/4 * quad .. of its key, which is a valid MFMA contraction order as long as Q^T is loaded in the same
// order.  V is parked as fp16 rows and read back transposed, as on the fp16 path.
#include <atomic>
#include <mutex>

#include <type_traits>

#include "attn_common.h"
#include "attn_host.h"
#include "quant_q8.h"

namespace minfer_attn {

constexpr int kDecodeWaves = 4;         // waves per workgroup
constexpr int kDecodeWavesPerSimd = 2;  // resident waves per SIMD the register budget is set for
constexpr int kDecodeWgPerCu = 2;       // workgroups of the split launch per compute unit
constexpr int kGroupRows = 16;          // cache rows per ring slot of one wave
constexpr int kDecodeStages = 3;        // ring depth

struct DecodeParams {
    const void* q; const void* k; const void* v;
    const int32_t* ctx;
    float* part_o;     // [B][Hq][S][D]
    float* part_ml;    // [B][Hq][S][2]: reference max (raw score units), sum
    int32_t* seq_off;  // [B + 1]: linear start of every sequence's work, written by workgroup 0 for the combine kernel
    int64_t q0, q1, kv0, kv1, kv2;
    int B, Hq, Hkv, n_rep, Lmax;
    int n_wg;          // workgroups of the split launch (kDecodeWaves waves each)
    int min_quota;     // smallest share of the work a wave takes, in groups
    int group_rows;    // cache rows per group: the unit the work is counted in
    int S;             // partial results a (sequence, head) can have: slots per row of the workspace, at most 64
    int n_hg;          // head groups of <= 16 heads per KV head
    float scale_log2;
};

// The work, laid out on a line: for every sequence, for every (head group, KV head) pair, the pair's cache rows in
// groups of `group_rows`.  Wave i of the launch takes groups [i * quota, (i + 1) * quota) of that line, whatever
// sequences and pairs they belong to, so every wave streams the same number of cache rows, on its own, and all of them
// end together; a piece of one pair inside one wave's share is a segment, and yields one partial result.
MA_DEV int groups_of(const DecodeParams& p, int ctx) { return (min(max(ctx, 0), p.Lmax) + p.group_rows - 1) / p.group_rows; }

// Length of the line (every lane gets it).  With `publish`, also stores every sequence's start on the line and,
// at index B, the length.
MA_DEV int work_total(const DecodeParams& p, int lane, bool publish) {
    const int pairs = p.Hkv * p.n_hg;
    int offset = 0;
    for (int base = 0; base < p.B; base += 64) {
        const int b = base + lane;
        const int n = b < p.B ? groups_of(p, p.ctx[b]) * pairs : 0;
        const int incl = wave_inclusive_scan(n, lane);
        if (publish && b < p.B) p.seq_off[b] = offset + incl - n;
        offset += __builtin_amdgcn_readfirstlane(__shfl(incl, 63));
    }
    if (publish && lane == 0) p.seq_off[p.B] = offset;
    return offset;
}
MA_DEV int work_quota(const DecodeParams& p, int total) {
    const int n_waves = p.n_wg * kDecodeWaves;
    return max((total + n_waves - 1) / n_waves, p.min_quota);
}

// The sequence that holds position x (< total) of the line, its start on the line and its context length.
MA_DEV void locate_sequence(const DecodeParams& p, int x, int lane, int& b_out, int& off_out, int& ctx_out) {
    const int pairs = p.Hkv * p.n_hg;
    int offset = 0;
    b_out = 0; off_out = 0; ctx_out = 0;
    for (int base = 0; base < p.B; base += 64) {
        const int b = base + lane;
        const int c = b < p.B ? p.ctx[b] : 0;
        const int n = b < p.B ? groups_of(p, c) * pairs : 0;
        const int incl = wave_inclusive_scan(n, lane);
        const int total = __builtin_amdgcn_readfirstlane(__shfl(incl, 63));
        if (x < offset + total) {
            const uint64_t hit = __ballot(x < offset + incl);
            const int src = __ffsll((unsigned long long)hit) - 1;
            // every lane holds the same values; saying so keeps the kernel's control flow (and with it
            // the compiler's wait-count bookkeeping in the main loop) scalar
            b_out = __builtin_amdgcn_readfirstlane(base + src);
            off_out = __builtin_amdgcn_readfirstlane(offset + __shfl(incl - n, src));
            ctx_out = __builtin_amdgcn_readfirstlane(__shfl(c, src));
            return;
        }
        offset += total;
    }
}

// Walks a wave's share of the line segment by segment.
struct SegmentWalk {
    int x, x_end, quota;     // position on the line, end of the share
    int b, off_b, ctx, n_b;  // current sequence: index, start on the line, context length, groups per pair
    // set by next():
    int pair, g0, g1, slot;  // (head group, KV head) pair, its groups [g0, g1), index of the partial result among the pair's

    int wave;                // index of the wave's share of the line
    // Shares are dealt to the waves of a workgroup in turn; when there are no more shares than workgroups (few or
    // short sequences), every share goes to a workgroup of its own instead, so that as many compute units as
    // possible pull on the memory system (B = 1 over 131072 rows: 107 -> 94 us, over 8192 rows: 19.4 -> 17.7 us).
    MA_DEV void take_share(int total, int w) {
        const int n_shares = (total + quota - 1) / quota;
        wave = n_shares <= (int)gridDim.x ? w * (int)gridDim.x + (int)blockIdx.x : (int)blockIdx.x * kDecodeWaves + w;
        x = wave * quota;
        x_end = min(total, x + quota);
    }
    MA_DEV bool start(const DecodeParams& p, int lane, int w) {
        const bool first = blockIdx.x == 0 && w == 0;   // the wave that also stores the sequences' offsets
        int c;
        if (p.B <= 64) {   // one scan gives the line's length and the share's first sequence
            c = lane < p.B ? p.ctx[lane] : 0;
            const int n = lane < p.B ? groups_of(p, c) * p.Hkv * p.n_hg : 0;
            const int incl = wave_inclusive_scan(n, lane);
            const int total = __builtin_amdgcn_readfirstlane(__shfl(incl, 63));
            if (first) {
                if (lane < p.B) p.seq_off[lane] = incl - n;
                if (lane == 0) p.seq_off[p.B] = total;
            }
            quota = work_quota(p, total);
            take_share(total, w);
            if (x >= x_end) return false;
            const int src = __ffsll((unsigned long long)__ballot(x < incl)) - 1;
            b = __builtin_amdgcn_readfirstlane(src);
            off_b = __builtin_amdgcn_readfirstlane(__shfl(incl - n, src));
            c = __builtin_amdgcn_readfirstlane(__shfl(c, src));
        } else {
            const int total = work_total(p, lane, first);
            quota = work_quota(p, total);
            take_share(total, w);
            if (x >= x_end) return false;
            locate_sequence(p, x, lane, b, off_b, c);
        }
        ctx = min(max(c, 0), p.Lmax);
        n_b = groups_of(p, ctx);
        return true;
    }
    MA_DEV bool next(const DecodeParams& p) {
        if (x >= x_end) return false;
        const int pairs = p.Hkv * p.n_hg;
        if (x >= off_b + pairs * n_b) {        // the sequence is done: on to the next one that has rows
            off_b += pairs * n_b;
            do {
                ++b;
                ctx = min(max(p.ctx[b], 0), p.Lmax);
                n_b = groups_of(p, ctx);
            } while (n_b == 0);
        }
        const int y = x - off_b;
        pair = y / n_b;
        g0 = y - pair * n_b;
        g1 = min(n_b, g0 + (x_end - x));
        slot = wave - (off_b + pair * n_b) / quota;
        x += g1 - g0;
        return true;
    }
};

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
__global__ __launch_bounds__(kDecodeWaves * 64, kDecodeWavesPerSimd) void decode_split_kernel(const DecodeParams p) {
    using GEO = DecodeGeom<D>;
    constexpr int RB = GEO::RB, G = GEO::G, RPI = GEO::RPI, NI = GEO::NI;
    constexpr int KC = D / 32;   // 32-wide contraction chunks of K Q^T
    constexpr int DB = D / 16;   // 16-row blocks of O^T
    constexpr int NS = kDecodeStages;

    __shared__ __attribute__((aligned(1024))) char v_lds[kDecodeWaves][kGroupRows * RB];
    __shared__ __attribute__((aligned(1024))) char k_lds[kDecodeWaves][kGroupRows * RB];

    const int tid = threadIdx.x, lane = tid & 63, w = wave_id();
    const int l16 = lane & 15, quad = lane >> 4;
    SegmentWalk walk;
    if (!walk.start(p, lane, w)) return;   // no share of the work
    while (walk.next(p)) {
    const int b = walk.b, split = walk.slot;
    const int g = walk.pair % p.Hkv, hg = walk.pair / p.Hkv;
    const int ctx = walk.ctx;
    const int row_lo = walk.g0 * kGroupRows;
    const int row_hi = min(walk.g1 * kGroupRows, ctx);
    const int n_groups = walk.g1 - walk.g0;

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
        const int r0 = row_lo + t * kGroupRows;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int row = j * RPI + lane / G;
            kk[j] = stream_load(reinterpret_cast<const s16x8*>(Kb + (int64_t)min(r0 + row, row_hi - 1) * p.kv2 + 8 * (lane % G)));
        }
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int row = j * RPI + lane / G;
            vv[j] = stream_load(reinterpret_cast<const s16x8*>(Vb + (int64_t)min(r0 + row, row_hi - 1) * p.kv2 + 8 * (lane % G)));
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
        const int key0 = row_lo + t * kGroupRows + 4 * quad;
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

    for (int t0 = 0; t0 < n_groups; t0 += NS) {
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            if (t0 + s < n_groups) consume(t0 + s, kr[s], vr[s]);
            load_group(t0 + s + NS, kr[s], vr[s]);
        }
    }

    // ---- the segment's partial result: un-normalised O, reference max and sum of every head -------------
    l_sum += __shfl_xor(l_sum, 16);
    l_sum += __shfl_xor(l_sum, 32);
    if (l16 < heads_here) {
        const int64_t slot = ((int64_t)b * p.Hq + head0 + l16) * p.S + split;
        float* dst = p.part_o + slot * D + 4 * quad;
#pragma unroll
        for (int db = 0; db < DB; ++db) *reinterpret_cast<f32x4*>(dst + 16 * db) = o_acc[db];
        if (quad == 0) { p.part_ml[slot * 2] = m_ref; p.part_ml[slot * 2 + 1] = l_sum; }
    }
    }
}

// ---- decode over Q8_0 caches -----------------------------------------------------------------------
constexpr int kDecodeStagesQ8 = 2;   // ring depth, in 32-row groups
constexpr int kGroupRowsQ8 = 32;

template <int D> struct DecodeGeomQ8 {
    static constexpr int BPR = D / 32;                        // blocks per cache row
    static constexpr int ROWB = BPR * 34;                     // bytes per cache row
    static constexpr int RAWB = kGroupRowsQ8 * ROWB;          // bytes of a group's K (or V) rows, a multiple of 16
    static constexpr int NG = (RAWB + 14 + 15) / 16;          // aligned 16-byte pieces that cover them (base any even address)
    static constexpr int NL = (NG + 63) / 64;                 // wave-wide loads per group and tensor
    static constexpr int RAW_LDS = NG * 16;
    static constexpr int RB = D * 2;                          // bytes of a parked fp16 row
    static constexpr int PARK = kGroupRowsQ8 * RB;
    // K's pieces are consumed into registers before V's arrive, so one raw area serves both
    static constexpr int WAVE_LDS = RAW_LDS + PARK;
};

// kv0/kv1 of DecodeParams are byte strides here; q and out are fp16.
template <int D>
__global__ __launch_bounds__(kDecodeWaves * 64, kDecodeWavesPerSimd) void decode_split_q8_kernel(const DecodeParams p) {
    using T = F16;
    using GEO = DecodeGeom<D>;
    using Q = DecodeGeomQ8<D>;
    constexpr int RB = Q::RB, BPR = Q::BPR, ROWB = Q::ROWB, NL = Q::NL, NG = Q::NG;
    constexpr int KC = D / 32;   // 32-wide contraction steps of K Q^T
    constexpr int DB = D / 16;   // 16-row blocks of O^T
    constexpr int NS = kDecodeStagesQ8;
    constexpr int GR = kGroupRowsQ8;

    __shared__ __attribute__((aligned(1024))) char lds[kDecodeWaves][(Q::WAVE_LDS + 1023) / 1024 * 1024];

    const int tid = threadIdx.x, lane = tid & 63, w = wave_id();
    const int l16 = lane & 15, quad = lane >> 4;
    SegmentWalk walk;
    if (!walk.start(p, lane, w)) return;   // no share of the work
    while (walk.next(p)) {
    const int b = walk.b, split = walk.slot;
    const int g = walk.pair % p.Hkv, hg = walk.pair / p.Hkv;
    const int ctx = walk.ctx;
    const int row_lo = walk.g0 * GR;                         // a multiple of 32
    const int row_hi = min(walk.g1 * GR, ctx);
    const int n_groups = walk.g1 - walk.g0;

    const int heads_here = min(16, p.n_rep - hg * 16);
    const int head0 = g * p.n_rep + hg * 16;
    char* raw_k = lds[w];
    char* raw_v = lds[w];                    // after K's blocks have been read (a wave's LDS operations execute in order)
    char* park_v = lds[w] + Q::RAW_LDS;

    // The (sequence, KV head)'s rows start at kb; pieces are counted from the 16-byte boundary at or below it.
    // (plain pointer arithmetic, so that the loads below stay global-memory loads)
    const char* kb = (const char*)p.k + ((int64_t)b * p.kv0 + (int64_t)g * p.kv1);
    const char* vb = (const char*)p.v + ((int64_t)b * p.kv0 + (int64_t)g * p.kv1);
    const int pre_k = (int)((uintptr_t)kb & 15), pre_v = (int)((uintptr_t)vb & 15);   // even, wave-uniform
    const char* kb16 = kb - pre_k;
    const char* vb16 = vb - pre_v;
    // last piece that holds a byte of the chunk's rows, relative to the aligned base
    const int64_t last_k = ((int64_t)pre_k + (int64_t)row_hi * ROWB - 1) & ~(int64_t)15;
    const int64_t last_v = ((int64_t)pre_v + (int64_t)row_hi * ROWB - 1) & ~(int64_t)15;

    // ---- Q^T fragments (B operand): column = head l16; step s takes d = D/4 * quad + 8s + 0..7, the order in
    // which the K fragments below come out of a lane's share of its key's row
    s16x8 qf[KC];
    {
        const bool valid = l16 < heads_here;
        const short* src = (const short*)p.q + (int64_t)b * p.q0 + (int64_t)(head0 + (valid ? l16 : 0)) * p.q1 + (D / 4) * quad;
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            s16x8 x = *reinterpret_cast<const s16x8*>(src + 8 * c);
            if (!valid) x = s16x8{0, 0, 0, 0, 0, 0, 0, 0};
            qf[c] = x;
        }
    }

    // ring of groups in flight: piece 64j + lane of the group's K bytes and of its V bytes
    struct Stage { u32x4 k[NL], v[NL]; };
    Stage ring[NS];
    // Pieces past the chunk's last one re-read that one (and land on its LDS slot again); ring slots past the
    // wave's last group have every lane re-read one piece of the last group, which costs one cache line.  The
    // loop body stays straight-line code that way, which lets the compiler's wait counts keep NS-1 groups in flight.
    auto piece_offset = [&](int t, int j, int64_t last, int64_t& group_off) {
        const bool real = t < n_groups;
        const int grp = min(t, n_groups - 1);
        group_off = (int64_t)(row_lo + grp * GR) * ROWB;              // a multiple of 16, wave-uniform
        // the group's own pieces only (they are what its LDS area holds), and none past the chunk's last one
        const int rel_last = real ? (int)min(last - group_off, (int64_t)16 * (NG - 1)) : 0;   // >= 0
        return min(16 * (64 * j + lane), rel_last);
    };
    // A group that is not the wave's last lies wholly inside the chunk: its pieces need no clamping (their offsets are
    // constants of the lane) and its keys no masking.  `inner_tag` says so at compile time; the loop below runs such
    // groups through code without the clamps and falls back to the general code for the last ones.
    int inner_off[NL];
#pragma unroll
    for (int j = 0; j < NL; ++j) inner_off[j] = min(16 * (64 * j + lane), 16 * (NG - 1));
    // K's and V's pieces of a group are requested separately: each as soon as the registers that receive them have
    // handed the group before over to LDS (at the start and in the middle of that group's turn, not after it), so that
    // a request has the better part of two turns to come back.
    auto load_k = [&](auto inner_tag, int t, Stage& st) __attribute__((always_inline)) {
        constexpr bool INNER = decltype(inner_tag)::value;
        const int64_t inner_goff = (int64_t)(row_lo + t * GR) * ROWB;
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            int64_t goff = inner_goff;
            const int off = INNER ? inner_off[j] : piece_offset(t, j, last_k, goff);
            st.k[j] = stream_load(reinterpret_cast<const u32x4*>(kb16 + goff + off));
        }
    };
    auto load_v = [&](auto inner_tag, int t, Stage& st) __attribute__((always_inline)) {
        constexpr bool INNER = decltype(inner_tag)::value;
        const int64_t inner_goff = (int64_t)(row_lo + t * GR) * ROWB;
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            int64_t goff = inner_goff;
            const int off = INNER ? inner_off[j] : piece_offset(t, j, last_v, goff);
            st.v[j] = stream_load(reinterpret_cast<const u32x4*>(vb16 + goff + off));
        }
    };
    const std::false_type general_tag{};
    const std::true_type inner_group_tag{};
#pragma unroll
    for (int s = 0; s < NS; ++s) { load_k(general_tag, s, ring[s]); load_v(general_tag, s, ring[s]); }

    f32x4 o_acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) o_acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_ref = -INFINITY, l_sum = 0.f;
    const float c2 = p.scale_log2;
    constexpr float kLazyLog2 = 6.f;

    // A block sits at an even offset of a raw area and is read as the aligned words that cover it (2-byte aligned
    // LDS reads stall for tens of cycles): whether it starts on a word or in the middle of one is a property of
    // the lane, fixed for the whole kernel (rows and 64-block strides are multiples of 4 bytes).
    const bool k_odd = ((pre_k + (D == 128 ? quad : quad >> 1) * 34) & 2) != 0;
    const bool v_odd = ((pre_v + lane * 34) & 2) != 0;
    const uint32_t k_sel = k_odd ? kQ8SelOdd : kQ8SelEven, v_sel = v_odd ? kQ8SelOdd : kQ8SelEven;
    // the block's scale from its first memory word (zero for rows past the chunk's end, whose bytes were never loaded)
    auto scale_of = [&](uint32_t w0, bool odd, bool row_ok) {
        const uint16_t bits = (uint16_t)(odd ? w0 >> 16 : w0);
        const _Float16 dh = row_ok ? __builtin_bit_cast(_Float16, bits) : (_Float16)0.f;
        return h16x2{dh, dh};
    };

    // (next_tag: whether group t + NS, requested during this turn, is an inner one)
    auto consume = [&](auto inner_tag, auto next_tag, int t, Stage& st) __attribute__((always_inline)) {
        constexpr bool INNER = decltype(inner_tag)::value;
        const int r0 = row_lo + t * GR;
        int64_t goff;
        // ---- the group's pieces into the wave's raw areas ----------------------------------------------
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            const int off = INNER ? inner_off[j] : piece_offset(t, j, last_k, goff);
            *reinterpret_cast<u32x4*>(raw_k + off) = st.k[j];
        }
        load_k(next_tag, t + NS, st);
        // ---- S^T = K Q^T for the two 16-key halves: lane gets head l16, keys 16h + 4*quad + r ---------------
        f32x4 s[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int row = 16 * h + l16;
            // the lane's share of its key's row: D/4 values starting at D/4 * quad (one block at D = 128, half a block at 64)
            const int at = pre_k + row * ROWB + (D == 128 ? quad : quad >> 1) * 34;
            const uint32_t* wp = reinterpret_cast<const uint32_t*>(raw_k + (at & ~3));
            const h16x2 d2 = scale_of(wp[0], k_odd, INNER || r0 + row < row_hi);
            constexpr int NW = D / 16;                       // quant words of the lane's share
            const uint32_t* qp = wp + (D == 128 ? 0 : 4 * (quad & 1));
            uint32_t wq[NW + 1];
#pragma unroll
            for (int i = 0; i <= NW; ++i) wq[i] = qp[i];
            s[h] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < KC; ++c)
                s[h] = T::mfma16(dequant8_shifted(wq[2 * c], wq[2 * c + 1], wq[2 * c + 2], k_sel, d2), qf[c], s[h]);
            if (!INNER) {
                const int key0 = r0 + 16 * h + 4 * quad;
#pragma unroll
                for (int r = 0; r < 4; ++r) s[h][r] = (key0 + r < row_hi) ? s[h][r] : -INFINITY;
            }
        }
        // ---- V: its pieces over K's, then every lane dequantises GR * BPR / 64 blocks and parks them as fp16 rows (swizzled)
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            const int off = INNER ? inner_off[j] : piece_offset(t, j, last_v, goff);
            *reinterpret_cast<u32x4*>(raw_v + off) = st.v[j];
        }
        load_v(next_tag, t + NS, st);
#pragma unroll
        for (int i = 0; i < GR * BPR / 64; ++i) {
            const int idx = 64 * i + lane, row = idx / BPR, c = idx % BPR;
            const int at = pre_v + idx * 34;
            const uint32_t* wp = reinterpret_cast<const uint32_t*>(raw_v + (at & ~3));
            uint32_t wv[9];
#pragma unroll
            for (int j = 0; j < 9; ++j) wv[j] = wp[j];
            const h16x2 d2 = scale_of(wv[0], v_odd, INNER || r0 + row < row_hi);
            char* rowp = park_v + row * RB;
            const int sw = GEO::swz_v(row);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<s16x8*>(rowp + 16 * ((4 * c + j) ^ sw)) =
                    dequant8_shifted(wv[2 * j], wv[2 * j + 1], wv[2 * j + 2], v_sel, d2);
        }
        // ---- online softmax over this group's 32 keys ----------------------------------------------------
        float mx = fmaxf(fmaxf(fmaxf(s[0][0], s[0][1]), fmaxf(s[0][2], s[0][3])), fmaxf(fmaxf(s[1][0], s[1][1]), fmaxf(s[1][2], s[1][3])));
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
        uint4 pu;
        {
            uint32_t pk[4];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                pk[2 * h] = T::pack2(fast_exp2(fmaf(s[h][0], c2, -mc)), fast_exp2(fmaf(s[h][1], c2, -mc)));
                pk[2 * h + 1] = T::pack2(fast_exp2(fmaf(s[h][2], c2, -mc)), fast_exp2(fmaf(s[h][3], c2, -mc)));
            }
            pu = uint4{pk[0], pk[1], pk[2], pk[3]};
            l_sum = T::add_pair(pk[3], T::add_pair(pk[2], T::add_pair(pk[1], T::add_pair(pk[0], l_sum))));   // the rounded weights
        }
        const s16x8 pfrag = __builtin_bit_cast(s16x8, pu);   // contraction index j: key 4*quad + j (j < 4), 16 + 4*quad + j - 4
        // ---- O^T += V^T P^T over the 32 keys: A = V^T block (row d = 16db + l16), same key order ---------------
        {
            const int row = 4 * quad + (l16 >> 2);
            const char* rowp = park_v + row * RB;
            const int sw = GEO::swz_v(row);         // rows 16 apart share a swizzle
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const int dcol = 16 * db + 4 * (l16 & 3);
                const int at = 16 * ((dcol >> 3) ^ sw) + 2 * (dcol & 7);
                const s16x4 a0 = lds_read_tr16(rowp + at);
                const s16x4 a1 = lds_read_tr16(rowp + 16 * RB + at);
                const s16x8 a = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
                o_acc[db] = T::mfma16(a, pfrag, o_acc[db]);
            }
        }
    };

    int t0 = 0;
    // rounds in which every group consumed and every group requested is an inner one
    for (; t0 + 2 * NS < n_groups; t0 += NS) {
#pragma unroll
        for (int s = 0; s < NS; ++s) consume(inner_group_tag, inner_group_tag, t0 + s, ring[s]);
    }
    for (; t0 < n_groups; t0 += NS) {
#pragma unroll
        for (int s = 0; s < NS; ++s)
            if (t0 + s < n_groups) consume(general_tag, general_tag, t0 + s, ring[s]);
    }

    // ---- the segment's partial result: un-normalised O, reference max and sum of every head -------------
    l_sum += __shfl_xor(l_sum, 16);
    l_sum += __shfl_xor(l_sum, 32);
    if (l16 < heads_here) {
        const int64_t slot = ((int64_t)b * p.Hq + head0 + l16) * p.S + split;
        float* dst = p.part_o + slot * D + 4 * quad;
#pragma unroll
        for (int db = 0; db < DB; ++db) *reinterpret_cast<f32x4*>(dst + 16 * db) = o_acc[db];
        if (quad == 0) { p.part_ml[slot * 2] = m_ref; p.part_ml[slot * 2 + 1] = l_sum; }
    }
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
    const int64_t slot0 = (int64_t)row * p.S;
    const float* src = p.part_o + slot0 * D + EPL * lane;
    auto load_o = [&](int slot, float (&x)[EPL]) {
        const float* ptr = src + (int64_t)slot * D;
        if (EPL == 2) {
            const f32x2 v2 = *reinterpret_cast<const f32x2*>(ptr);
            x[0] = v2[0]; x[EPL - 1] = v2[1];
        } else {
            x[0] = ptr[0];
        }
    };
    // Everything is requested at once: how many partial results the row has, and, before that is known, every
    // slot's (max, sum) and the first four slots' O (slots past the count hold stale bytes and are discarded).
    const int sl = min(lane, p.S - 1);
    const float m_raw = p.part_ml[(slot0 + sl) * 2], l_raw = p.part_ml[(slot0 + sl) * 2 + 1];
    constexpr int kEarly = 4;
    float x[8][EPL];
#pragma unroll
    for (int u = 0; u < kEarly; ++u) load_o(min(u, p.S - 1), x[u]);
    // the partial results of this row: one per share of the line that overlaps the rows of its (sequence, KV head)
    const int n_b = groups_of(p, p.ctx[b]);
    const int quota = work_quota(p, p.seq_off[p.B]);
    const int g = hq / p.n_rep, hg = (hq % p.n_rep) / 16;
    const int start = p.seq_off[b] + (hg * p.Hkv + g) * n_b;
    const int ns = n_b > 0 ? (start + n_b - 1) / quota - start / quota + 1 : 0;
    const float m = lane < ns ? m_raw : -INFINITY, l = lane < ns ? l_raw : 0.f;
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
    for (int s0 = 0; s0 < ns; s0 += 8) {   // 8 partial results at a time, all loads in flight together
        if (s0 > 0) {
#pragma unroll
            for (int u = 0; u < 8; ++u) load_o(min(s0 + u, ns - 1), x[u]);
        } else {
#pragma unroll
            for (int u = kEarly; u < 8; ++u) load_o(min(u, ns - 1), x[u]);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const bool on = s0 + u < ns;
            const float ws = __shfl(wgt, min(s0 + u, 63));
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[e] += on ? x[u][e] * ws : 0.f;
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

// Smallest share of the work a workgroup takes, in cache rows: 256, or more for very long caches, so that a
// (sequence, head) never has more than 64 partial results, which is what one wave of the combine kernel merges.
static int decode_min_share_rows(int64_t Lmax) {
    int64_t c = (Lmax + 59) / 60;
    c = (c + 63) / 64 * 64;
    return (int)(c > 256 ? c : 256);
}
// Partial results a (sequence, head) can have: a pair's rows overlap at most this many shares.
static int decode_slots(int64_t Lmax) { return (int)(Lmax / decode_min_share_rows(Lmax)) + 3; }

static size_t decode_ws_bytes(int64_t B, int64_t Hq, int64_t Lmax, int64_t D) {
    const int64_t S = decode_slots(Lmax);
    return (size_t)(B * Hq * S * (D + 2) * 4 + 255) / 256 * 256 + (size_t)((B + 1) * 4 + 255) / 256 * 256 + 256;
}

// Workgroups of the split launch: as many as the chip holds at once (kDecodeWgPerCu per compute unit: LDS and
// registers allow no more), so that each gets one equal share of the work and all run from start to end.
// The per-device count is cached in atomics: concurrent first calls at worst both query the attribute.
static int decode_workgroups() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        n = cus * kDecodeWgPerCu;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

template <class T, int D>
static int launch_decode(const DecodeParams& p, void* out, int64_t o0, int64_t o1, hipStream_t stream) {
    hipLaunchKernelGGL((decode_split_kernel<T, D>), dim3((unsigned)p.n_wg), dim3(kDecodeWaves * 64), 0, stream, p);
    if (int rc = check_launch("decode_split_kernel")) return rc;
    hipLaunchKernelGGL((decode_combine_kernel<T, D>), dim3((p.B * p.Hq + 3) / 4), dim3(256), 0, stream, p, out, o0, o1);
    return check_launch("decode_combine_kernel");
}

template <int D>
static int launch_decode_q8(const DecodeParams& p, void* out, int64_t o0, int64_t o1, hipStream_t stream) {
    hipLaunchKernelGGL((decode_split_q8_kernel<D>), dim3((unsigned)p.n_wg), dim3(kDecodeWaves * 64), 0, stream, p);
    if (int rc = check_launch("decode_split_q8_kernel")) return rc;
    hipLaunchKernelGGL((decode_combine_kernel<F16, D>), dim3((p.B * p.Hq + 3) / 4), dim3(256), 0, stream, p, out, o0, o1);
    return check_launch("decode_combine_kernel");
}

}  // namespace minfer_attn

using namespace minfer_attn;

MINFER_ATTN_EXPORT size_t minfer_flash_attn_decode_workspace_bytes(int64_t B, int64_t Hq, int64_t Lmax, int64_t D) {
    if (B <= 0 || Hq <= 0 || Lmax < 0 || D <= 0) return 256;
    return decode_ws_bytes(B, Hq, Lmax, D);   // Lmax == 0 (an empty cache) still has its rows' slots: the call writes zeros
}

// Fills the launch parameters both decode entry points share; returns an error code or MINFER_ATTN_OK.
static int fill_decode(DecodeParams& p, const void* q, const void* k_cache, const void* v_cache, const int32_t* ctx_lens,
                       int64_t B, int64_t Hq, int64_t Hkv, int64_t Lmax, int64_t D, const minfer_attn_strides* st,
                       void* workspace, size_t workspace_bytes, int group_rows) {
    if (!ctx_lens) return fail(MINFER_ATTN_EINVAL, "flash_attn_decode: ctx_lens is null");
    if (B < 0 || Lmax < 0) return fail(MINFER_ATTN_EINVAL, "flash_attn_decode: negative B or Lmax");
    if (B > 65535 || Hq > 65535) return fail(MINFER_ATTN_EINVAL, "flash_attn_decode: B or n_heads > 65535 unsupported");
    if (Lmax > (1 << 30)) return fail(MINFER_ATTN_EINVAL, "flash_attn_decode: Lmax too large");
    if (B == 0) return MINFER_ATTN_OK;
    if (!workspace || workspace_bytes < decode_ws_bytes(B, Hq, Lmax, D) || !aligned16(workspace))
        return fail(MINFER_ATTN_EWORKSPACE, "flash_attn_decode: workspace too small or misaligned (see minfer_flash_attn_decode_workspace_bytes)");
    p.q = q; p.k = k_cache; p.v = v_cache; p.ctx = ctx_lens;
    p.q0 = st->q0; p.q1 = st->q1; p.kv0 = st->kv0; p.kv1 = st->kv1; p.kv2 = st->kv2;
    p.B = (int)B; p.Hq = (int)Hq; p.Hkv = (int)Hkv; p.n_rep = (int)(Hq / Hkv); p.Lmax = (int)Lmax;
    p.n_hg = (p.n_rep + 15) / 16;
    p.group_rows = group_rows;
    p.min_quota = decode_min_share_rows(Lmax) / group_rows;
    p.S = decode_slots(Lmax);
    p.n_wg = decode_workgroups();
    // the line of work is indexed with 32-bit integers
    if ((int64_t)B * Hkv * p.n_hg * ((Lmax + group_rows - 1) / group_rows) > 0x7fffffffLL - 65536)
        return fail(MINFER_ATTN_EINVAL, "flash_attn_decode: problem too large for one launch");
    p.scale_log2 = (float)(1.4426950408889634 / sqrt((double)D));
    const size_t o_bytes = ((size_t)B * Hq * p.S * D * 4 + 255) / 256 * 256;
    const size_t ml_bytes = ((size_t)B * Hq * p.S * 2 * 4 + 255) / 256 * 256;
    p.part_o = (float*)workspace;
    p.part_ml = (float*)((char*)workspace + o_bytes);
    p.seq_off = (int32_t*)((char*)workspace + o_bytes + ml_bytes);
    return MINFER_ATTN_OK;
}

MINFER_ATTN_EXPORT int minfer_flash_attn_decode(int dtype, const void* q, const void* k_cache, const void* v_cache,
                                        const int32_t* ctx_lens, void* out, int64_t B, int64_t Hq, int64_t Hkv,
                                        int64_t Lmax, int64_t D, const minfer_attn_strides* st, void* workspace,
                                        size_t workspace_bytes, void* stream_v) {
    clear_error();
    if (Lmax == 0) { k_cache = k_cache ? k_cache : q; v_cache = v_cache ? v_cache : q; }   // an empty cache has no rows to point at
    if (int rc = check_common(dtype, q, k_cache, v_cache, out, Hq, Hkv, D, st)) return rc;
    DecodeParams p{};
    if (int rc = fill_decode(p, q, k_cache, v_cache, ctx_lens, B, Hq, Hkv, Lmax, D, st, workspace, workspace_bytes, kGroupRows)) return rc;
    if (B == 0) return MINFER_ATTN_OK;
    hipStream_t stream = (hipStream_t)stream_v;

    if (dtype == MINFER_ATTN_F16)
        return D == 128 ? launch_decode<F16, 128>(p, out, st->o0, st->o1, stream) : launch_decode<F16, 64>(p, out, st->o0, st->o1, stream);
    return D == 128 ? launch_decode<BF16, 128>(p, out, st->o0, st->o1, stream) : launch_decode<BF16, 64>(p, out, st->o0, st->o1, stream);
}

MINFER_ATTN_EXPORT int minfer_flash_attn_decode_q8_0(const void* q, const void* k_cache, const void* v_cache,
                                             const int32_t* ctx_lens, void* out, int64_t B, int64_t Hq, int64_t Hkv,
                                             int64_t Lmax, int64_t D, const minfer_attn_strides* st, void* workspace,
                                             size_t workspace_bytes, void* stream_v) {
    clear_error();
    if (D != 64 && D != 128) return fail(MINFER_ATTN_EINVAL, "head_dim must be 64 or 128");
    if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0)
        return fail(MINFER_ATTN_EINVAL, "n_heads must be a positive multiple of n_kv_heads");
    if (!st) return fail(MINFER_ATTN_EINVAL, "strides is null");
    if (!q || !k_cache || !v_cache || !out) return fail(MINFER_ATTN_EINVAL, "q, k_cache, v_cache and out must be non-null");
    if (!aligned16(q) || !aligned16(out)) return fail(MINFER_ATTN_EINVAL, "q and out must be 16-byte aligned");
    if (st->q0 % 8 || st->q1 % 8 || st->o0 % 8 || st->o1 % 8 || st->q0 < 0 || st->q1 < 0 || st->o0 < 0 || st->o1 < 0)
        return fail(MINFER_ATTN_EINVAL, "strides of q and out must be non-negative multiples of 8 elements");
    if (((uintptr_t)k_cache | (uintptr_t)v_cache) & 1u)
        return fail(MINFER_ATTN_EINVAL, "flash_attn_decode_q8_0: caches must be 2-byte aligned");
    if (st->kv2 != D / 32 * 34)
        return fail(MINFER_ATTN_EINVAL, "flash_attn_decode_q8_0: cache rows must be dense (row stride = D/32 * 34 bytes)");
    if (st->kv0 < 0 || st->kv1 < 0 || st->kv0 % 2 || st->kv1 % 2)
        return fail(MINFER_ATTN_EINVAL, "flash_attn_decode_q8_0: cache strides must be non-negative even byte counts");
    DecodeParams p{};
    if (int rc = fill_decode(p, q, k_cache, v_cache, ctx_lens, B, Hq, Hkv, Lmax, D, st, workspace, workspace_bytes, kGroupRowsQ8)) return rc;
    if (B == 0) return MINFER_ATTN_OK;
    hipStream_t stream = (hipStream_t)stream_v;
    return D == 128 ? launch_decode_q8<128>(p, out, st->o0, st->o1, stream) : launch_decode_q8<64>(p, out, st->o0, st->o1, stream);
}

// ------------------------------------------------------------------------------------------------
// Decode for callers that cannot allocate (code under HIP graph capture, serving loops that must not touch the
// allocator): the split-KV partial results live in a file-scope device array instead of a caller workspace.
// Every GPU the library runs on holds its own copy of the array, at its own address, until the process ends; the
// array's name is only a host-side handle, the device address comes from hipGetSymbolAddress, once per device.
// The partial slots a call reads are all written by that call's split kernel first (slots past a row's count are
// loaded and discarded), so nothing needs clearing between calls; calls that overlap in time on one GPU would
// share the slots and race.
// ------------------------------------------------------------------------------------------------
namespace minfer_attn {
static __device__ __align__(256) unsigned char scratch[MINFER_DECODE_NOALLOC_SCRATCH_BYTES];

// The kernels run on the device that owns the caller's stream, so that device's copy of the array is the one to
// hand them.  The address is looked up once per device, with that device current (hipGetSymbolAddress answers for
// the current device); a stream that belongs to another device than the current one is refused, as a launch on it
// would be.
static int decode_scratch(hipStream_t stream, void** ptr_out) {
    static std::mutex mu;
    static void* ptrs[64] = {nullptr};
    int cur = 0, dev = 0;
    if (hipGetDevice(&cur) != hipSuccess) return fail(MINFER_ATTN_ELAUNCH, "flash_attn_decode_noalloc: hipGetDevice failed");
    dev = cur;
    if (stream) {   // the null stream belongs to the current device
        hipDevice_t sd = 0;
        if (hipStreamGetDevice(stream, &sd) != hipSuccess) return fail(MINFER_ATTN_EINVAL, "flash_attn_decode_noalloc: hipStreamGetDevice failed for the given stream");
        dev = (int)sd;
    }
    if (dev < 0 || dev >= 64) return fail(MINFER_ATTN_EINVAL, "flash_attn_decode_noalloc: device index above 63 unsupported");
    if (dev != cur) return fail(MINFER_ATTN_EINVAL, "flash_attn_decode_noalloc: the stream belongs to another device than the current one (hipSetDevice to the stream's device before the call)");
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            snprintf(error_buf(), 512, "flash_attn_decode_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
            return MINFER_ATTN_ELAUNCH;
        }
        ptrs[dev] = ptr;
    }
    *ptr_out = ptrs[dev];
    return MINFER_ATTN_OK;
}
}  // namespace minfer_attn

MINFER_ATTN_EXPORT int minfer_flash_attn_decode_noalloc(int dtype, const void* q, const void* k_cache, const void* v_cache,
                                                const int32_t* ctx_lens, void* out, int64_t B, int64_t Hq, int64_t Hkv,
                                                int64_t Lmax, int64_t D, const minfer_attn_strides* st, void* stream_v) {
    clear_error();
    if (Lmax == 0) { k_cache = k_cache ? k_cache : q; v_cache = v_cache ? v_cache : q; }   // an empty cache has no rows to point at
    if (int rc = check_common(dtype, q, k_cache, v_cache, out, Hq, Hkv, D, st)) return rc;
    if (!ctx_lens) return fail(MINFER_ATTN_EINVAL, "flash_attn_decode_noalloc: ctx_lens is null");
    if (B < 0 || Lmax < 0) return fail(MINFER_ATTN_EINVAL, "flash_attn_decode_noalloc: negative B or Lmax");
    if (B > 65535 || Lmax > (1 << 30)) return fail(MINFER_ATTN_EINVAL, "flash_attn_decode_noalloc: B > 65535 or Lmax > 2^30 unsupported");
    if (B == 0) return MINFER_ATTN_OK;
    if (decode_ws_bytes(B, Hq, Lmax, D) > (size_t)MINFER_DECODE_NOALLOC_SCRATCH_BYTES) {
        snprintf(error_buf(), 512, "flash_attn_decode_noalloc: B=%lld Hq=%lld Lmax=%lld D=%lld needs %zu bytes of partial results, "
                 "the built-in scratch holds %zu; use minfer_flash_attn_decode with a workspace",
                 (long long)B, (long long)Hq, (long long)Lmax, (long long)D, decode_ws_bytes(B, Hq, Lmax, D),
                 (size_t)MINFER_DECODE_NOALLOC_SCRATCH_BYTES);
        return MINFER_ATTN_EWORKSPACE;
    }
    void* ws = nullptr;
    if (int rc = decode_scratch((hipStream_t)stream_v, &ws)) return rc;
    DecodeParams p{};
    if (int rc = fill_decode(p, q, k_cache, v_cache, ctx_lens, B, Hq, Hkv, Lmax, D, st, ws,
                             (size_t)MINFER_DECODE_NOALLOC_SCRATCH_BYTES, kGroupRows)) return rc;
    hipStream_t stream = (hipStream_t)stream_v;
    if (dtype == MINFER_ATTN_F16)
        return D == 128 ? launch_decode<F16, 128>(p, out, st->o0, st->o1, stream) : launch_decode<F16, 64>(p, out, st->o0, st->o1, stream);
    return D == 128 ? launch_decode<BF16, 128>(p, out, st->o0, st->o1, stream) : launch_decode<BF16, 64>(p, out, st->o0, st->o1, stream);
}
