// Half-precision GEMM for gfx950: D = alpha * A x B + beta * C with fp32 accumulation on the MFMA units.
//
// What the reference computes (reference: src/minfer/kernels/torch_ext/csrc/cuda/gemm/op.cuh:218-316,
// oracle src/minfer/kernels/refs.py:49-51, tests test/kernels.py:119-216): A is [M, K] activations (leading
// dims flattened), B is the weight either as [K, N] ("A x B", what its tuned kernel handles) or as [N, K]
// ("A x B^T", the layout of its QKV projection, whose launcher is empty in the reference), C and D are [M, N].
//
// Design.  A workgroup (8 waves, two per SIMD) owns a 256 x 256 tile of D (128 x 128 with 4 waves for problems
// too small to fill the chip with large tiles) and walks K in steps of 64; the A and B panels of a step (32 KB
// each) are copied global->LDS without passing through registers, double-buffered, one barrier per step
// (placed inside the step, so that the matrix pipe keeps running across step boundaries).
// Every wave owns 128 (64) rows (m) x 64 columns (n) as 8 (4) x 4 accumulator blocks of 16x16
// (v_mfma_f32_16x16x32) and computes the transposed product D^T = B^T A^T, so that a lane ends up with 4
// consecutive n of one row m and the epilogue stores 8 bytes per block: B supplies the MFMA A operand (for the
// [K, N] layout through LDS transpose reads, the same way the attention kernel reads V^T; for [N, K] through
// plain 16-byte reads) and A supplies the B operand (16-byte reads).  LDS panels are split into sub-tiles
// with XOR swizzles of the kind the attention kernel's K and V tiles use, so both read patterns are free of bank
// conflicts.  Workgroup ids are dealt so that one XCD works on consecutive tiles of a tile row (they share the
// A panel in that XCD's L2).
#include <algorithm>
#include <atomic>

#include "attn_common.h"
#include "attn_host.h"
#include "quant_q8.h"

namespace minfer_attn {


constexpr int kBK = 64;
// Two tile shapes: 8 waves (2 x 4) on 256 x 256 for problems that fill the chip with such tiles, 4 waves (2 x 2) on
// 128 x 128 otherwise.  A wave owns 32*MB rows x 32*NB columns (as blocks of 16 x 16); OCC waves per SIMD.
template <int MB_, int NB_, int WAVES_N_, int OCC_, int WAVES_M_ = 2, int NS_ = 2> struct GemmShape {
    static constexpr int MB = MB_, NB = NB_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, WAVES = WAVES_M * WAVES_N, OCC = OCC_;
    static constexpr int NS = NS_;   // stages of the K ring in LDS: NS - 1 steps in flight while one is multiplied
    static constexpr int BM = 32 * MB * WAVES_M, BN = 32 * NB * WAVES_N;
    static constexpr int A_PANEL = BM * 128, B_PANEL = BN * 128;   // bytes of one K step
    static constexpr int A_COPIES = A_PANEL / 1024 / WAVES, B_COPIES = B_PANEL / 1024 / WAVES;   // wave-wide copies per wave
};
// (4 waves with 128 x 128 each, GemmShape<4, 4, 2, 1>, read a third fewer LDS bytes per flop.  Compiled as it stands
// that shape spills: its 256 accumulators leave the allocator no register to move anything with.  On 32 x 32 blocks,
// with 14 of the 16 accumulator blocks pinned to the accumulation registers and 2 to the vector registers by inline
// assembly, it was spill-free and ended level with the 8-wave shape at 4096^3 and 4 % behind at 8192^3.)
using GemmBig = GemmShape<4, 2, 4, 2>;
using GemmSmall = GemmShape<2, 2, 2, 2>;
// The same tile with three stages (96 KiB of LDS: one workgroup per compute unit) for launches of at most one workgroup per
// compute unit anyway: two steps in flight instead of one (clocks settled, 512 x 6144 x 4096 as 192 tiles 43.6 -> 36.6 us,
// 1024 x 4096 x 4096 as 256 tiles 44.9 -> 40.1, 256 x 14336 x 4096 44.9 -> 38.5; with more workgroups than compute units
// two resident workgroups of two stages are ahead, 2048 x 4096 x 4096 66.9 against 78.6; four stages lose to three throughout).
using GemmSmall3 = GemmShape<2, 2, 2, 2, 2, 3>;
static bool one_workgroup_per_unit(int64_t workgroups) { return workgroups <= 256; }
// 256 x 192 (8 waves as 4 x 2, a wave owns 64 x 96): for widths that are multiples of 192 whose 256 x 256 tiles would
// leave half the chip idle in their last round (4096 x 6144 is 384 large tiles, one and a half rounds on 256 compute
// units, but 512 of these, two full rounds of three quarters the work each).  [N, K] weights only: its 192 columns are
// three 64-row sub-tiles of such a weight, but one and a half of the 128-column sub-tiles of a [K, N] one.
using GemmWide = GemmShape<2, 3, 2, 2, 4>;
constexpr int kRowTile = 8192;              // sub-tile [64 rows][64 k], 128-byte rows (A, and B as [N, K])
constexpr int kColTile = 16384;             // sub-tile [64 k][128 n], 256-byte rows (B as [K, N])

// Several weights that share A in one launch (the QKV projection): the column tiles (tiled kernel) or column groups
// (few-row kernel) of weight s follow those of weight s - 1; `end` holds the cumulative counts.  No C operand.
constexpr int kMaxGroup = 3;
struct GemmGroup {
    const void* B[kMaxGroup]; void* D[kMaxGroup];
    int N[kMaxGroup], end[kMaxGroup];
    int64_t ldb[kMaxGroup], ldd[kMaxGroup];
};
struct GemmParams {
    const void* A; const void* B; const void* C; void* D;
    int M, N, K;
    int64_t lda, ldb, ldc, ldd;   // row strides in elements
    float alpha, beta;
    int tiles_m, tiles_n, per_xcd;
    int splits;                   // SPLIT instantiations: K is cut into this many slices, one workgroup per (tile, slice)
    float* part;                  // their fp32 partial products, [splits][M][N]
    GemmGroup grp;                // used by the GROUPED instantiations only
};
// Which weight column unit `c` (a tile column or a column group) belongs to, and its index inside that weight.
MA_DEV int group_of_unit(const GemmGroup& g, int c, int& local) {
    const int s = c < g.end[0] ? 0 : (c < g.end[1] ? 1 : 2);
    local = c - (s == 0 ? 0 : (s == 1 ? g.end[0] : g.end[1]));
    return s;
}

// swizzles: granule index of a row XORed with a function of the row (see the attention kernel's TileGeom)
MA_DEV int swz_row_tile(int row) { return (row >> 1) & 7; }        // 128-byte rows, read 32 rows x 16 bytes
MA_DEV int swz_col_tile(int row) { return ((row & 3) << 2) | ((row >> 2) & 2); }   // 256-byte rows, transposing reads of 4 rows x 32 bytes by each of two 16-lane groups 8 rows apart

// CONCAT (with GROUPED, [N, K] weights whose widths are multiples of 64): the weights' columns are numbered through as
// one wide matrix and tiled without regard to where one weight ends, so a tile may hold columns of two weights; every
// 64-column sub-tile of the B panel and every 32-column block of a wave lies inside one weight, which is looked up
// per copy instruction and per block (grp.end = cumulative column counts).
template <class T, bool NT, class SH, bool GROUPED = false, bool SPLIT = false, bool CONCAT = false>
__global__ __launch_bounds__(SH::WAVES * 64, SH::OCC) void gemm_kernel(const GemmParams p) {
    static_assert(!CONCAT || (GROUPED && NT && !SPLIT && SH::WAVES == 8), "CONCAT: grouped [N, K] weights, one sub-tile per copy index");
    constexpr int kBM = SH::BM, kBN = SH::BN, NW = SH::WAVES, MB = SH::MB, NB = SH::NB, CA = SH::A_COPIES, CB = SH::B_COPIES;
    constexpr int NS = SH::NS;
    static_assert(NS >= 2 && NS <= 4, "two to four stages");
    __shared__ __attribute__((aligned(1024))) char a_lds[NS][SH::A_PANEL];
    __shared__ __attribute__((aligned(1024))) char b_lds[NS][SH::B_PANEL];

    const int lane = threadIdx.x & 63, w = wave_id();
    const int h = lane >> 5, l32 = lane & 31;
    const int wm = w % SH::WAVES_M, wn = w / SH::WAVES_M;   // wave's place in the tile: rows 32*MB*wm .., columns 32*NB*wn ..
    static_assert(NT || SH::BN % 128 == 0, "a [K, N] weight is staged in sub-tiles of 128 columns");

    // ---- which tile ----------------------------------------------------------------------------------
    // (SPLIT: consecutive workgroup ids are the K slices of one tile, so the slices of a tile run on different XCDs)
    const int unit = SPLIT ? (int)blockIdx.x : (int)(blockIdx.x & 7) * p.per_xcd + (int)(blockIdx.x >> 3);
    const int slice = SPLIT ? unit % p.splits : 0;
    const int t = SPLIT ? unit / p.splits : unit;
    if (t >= p.tiles_m * p.tiles_n) return;
    // Tiles are numbered down bands of kGroupM tile rows, so that the tiles an XCD runs at one time form a block that
    // shares A row panels as well as B column panels in its L2 (row-major numbering made every XCD read all of B).
    constexpr int kGroupM = 4;
    const int band = t / (kGroupM * p.tiles_n), in_band = t % (kGroupM * p.tiles_n);
    const int first_m = band * kGroupM, gm = min(kGroupM, p.tiles_m - first_m);
    const int m0 = (first_m + in_band % gm) * kBM;
    int n0 = (in_band / gm) * kBN;

    const short* Ag = (const short*)p.A;
    const short* Bg = (const short*)p.B;
    short* Dg = (short*)p.D;
    int N = p.N;
    int64_t ldb = p.ldb, ldd = p.ldd;
    if (GROUPED && !CONCAT) {   // the tile column's weight, output and place inside them (all wave-uniform)
        int local;
        const int sg = group_of_unit(p.grp, in_band / gm, local);
        n0 = local * kBN;
        Bg = (const short*)(sg == 0 ? p.grp.B[0] : sg == 1 ? p.grp.B[1] : p.grp.B[2]);
        Dg = (short*)(sg == 0 ? p.grp.D[0] : sg == 1 ? p.grp.D[1] : p.grp.D[2]);
        N = sg == 0 ? p.grp.N[0] : sg == 1 ? p.grp.N[1] : p.grp.N[2];
        ldb = sg == 0 ? p.grp.ldb[0] : sg == 1 ? p.grp.ldb[1] : p.grp.ldb[2];
        ldd = sg == 0 ? p.grp.ldd[0] : sg == 1 ? p.grp.ldd[1] : p.grp.ldd[2];
    }

    // ---- global -> LDS copies: lane offsets (bytes) from the panel's first element ---------------------
    // Every wave issues 4 wave-wide copies (1 KB each) per panel and K step; copy q = j*NW + w of a panel covers
    //   A (and B as [N, K]): rows 8*(q%8) .. +7 of sub-tile q/8 (64 rows of 128 bytes each);
    //   B as [K, N]:         k rows 4*(q%16) .. +3 of sub-tile q/16 (64 k rows of 256 bytes, 128 columns).
    uint32_t a_off[CA], b_off[CB];
    int a_dst[CA], b_dst[CB];
    const short* b_src[CONCAT ? CB : 1];   // CONCAT: first weight row of copy j's sub-tile (wave-uniform)
#pragma unroll
    for (int j = 0; j < CA; ++j) {
        const int q = j * NW + w;
        const int sub = q >> 3, row = 8 * (q & 7) + (lane >> 3), pg = lane & 7;
        const int m = min(m0 + 64 * sub + row, p.M - 1) - m0;
        a_off[j] = (uint32_t)((int64_t)m * p.lda + 8 * (pg ^ swz_row_tile(row))) * 2u;
        a_dst[j] = sub * kRowTile + 8 * (q & 7) * 128;
    }
#pragma unroll
    for (int j = 0; j < CB; ++j) {
        const int q = j * NW + w;
        if (CONCAT) {   // copy j of every wave lies in sub-tile j, whose 64 weight rows belong to one weight
            const int row = 8 * (q & 7) + (lane >> 3), pg = lane & 7;
            int local;
            const int sg = group_of_unit(p.grp, n0 + 64 * j, local);
            const int64_t ldj = sg == 0 ? p.grp.ldb[0] : sg == 1 ? p.grp.ldb[1] : p.grp.ldb[2];
            b_src[j] = (const short*)(sg == 0 ? p.grp.B[0] : sg == 1 ? p.grp.B[1] : p.grp.B[2]) + (int64_t)local * ldj;
            b_off[j] = (uint32_t)((int64_t)row * ldj + 8 * (pg ^ swz_row_tile(row))) * 2u;
            b_dst[j] = j * kRowTile + 8 * (q & 7) * 128;
        } else if (NT) {
            const int sub = q >> 3, row = 8 * (q & 7) + (lane >> 3), pg = lane & 7;
            const int n = min(n0 + 64 * sub + row, N - 1) - n0;
            b_off[j] = (uint32_t)((int64_t)n * ldb + 8 * (pg ^ swz_row_tile(row))) * 2u;
            b_dst[j] = sub * kRowTile + 8 * (q & 7) * 128;
        } else {
            const int sub = q >> 4, row = 4 * (q & 15) + (lane >> 4), pg = lane & 15;
            const int col = min(n0 + 128 * sub + 8 * (pg ^ swz_col_tile(row)), N - 8) - n0;
            b_off[j] = (uint32_t)((int64_t)row * ldb + col) * 2u;
            b_dst[j] = sub * kColTile + 4 * (q & 15) * 256;
        }
    }
    // K steps of this workgroup: all of them, or its slice
    const int kt_all = p.K / kBK;
    const int kt_first = SPLIT ? (int)((int64_t)slice * kt_all / p.splits) : 0;
    const int KT = SPLIT ? (int)((int64_t)(slice + 1) * kt_all / p.splits) - kt_first : kt_all;
    // (With three stages the compiler runs out of scalar registers in some instantiations and moves the panel bases from
    // vector registers right in front of every copy, closer than a copy may follow such a move: those wait the documented
    // distance inside the copy, see copy16_global_to_lds; the build's scan of the generated code is what finds such cases.)
    constexpr bool kFreshBases = SH::NS > 2;
    // copy c of a step (the wave's A copies, then its B copies) into a stage
    auto copy_one = [&](int kt_rel, int stage, int c) __attribute__((always_inline)) {
        const int kt = kt_first + kt_rel;
        if (c < CA) {
            copy16_global_to_lds<kFreshBases>(Ag + (int64_t)m0 * p.lda + (int64_t)kt * kBK, a_off[c], &a_lds[stage][a_dst[c]]);
        } else {
            const int j = c - CA;
            const short* bbase = NT ? Bg + (int64_t)n0 * ldb + (int64_t)kt * kBK : Bg + (int64_t)kt * kBK * ldb + n0;
            copy16_global_to_lds<kFreshBases>(CONCAT ? b_src[CONCAT ? j : 0] + (int64_t)kt * kBK : bbase, b_off[j], &b_lds[stage][b_dst[j]]);
        }
    };
    auto issue = [&](int kt_rel, int stage) __attribute__((always_inline)) {
#pragma unroll
        for (int c = 0; c < CA + CB; ++c) copy_one(kt_rel, stage, c);
    };

    // ---- per-lane LDS read addresses (stage 0; stage, sub-tile and block offsets are immediates) ---------
    // The matrix instruction is v_mfma_f32_16x16x32 (on random fp16 operands the chip sustains 1.80-1.90 PFLOP/s of it and
    // 1.56-1.62 of v_mfma_f32_32x32x16, and a power-bound GEMM runs at what its matrix instruction sustains).  A K step is two slices of
    // 32 values; a fragment is 16 rows x 32 k, lane (l16, quad) holding row l16, k = 8 quad + 0..7 of the slice: 16 bytes
    // at granule (4 slice + quad) ^ swizzle of the row.  A 16-row block is a quarter of a 64-row sub-tile; the swizzle of
    // row 16 b + l16 does not depend on b.
    constexpr int M16 = 2 * MB, N16 = 2 * NB, BLK = kRowTile / 4;
    const int l16 = lane & 15, quad = lane >> 4;
    constexpr int NRD = N16 < 4 ? 4 : N16;
    uint32_t m_rd[2], n_rd[NRD];
    {
        const int sw = swz_row_tile(l16);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const uint32_t o = l16 * 128 + 16 * ((4 * ks + quad) ^ sw);
            m_rd[ks] = lds_addr(&a_lds[0][0]) + M16 * wm * BLK + o;
            if (NT) n_rd[ks] = lds_addr(&b_lds[0][0]) + N16 * wn * BLK + o;    // n fragments: as the m fragments
        }
        if (!NT) {
            // n fragments through transpose reads of the [k][n] sub-tile: the 16-lane group `quad` addresses k rows
            // 8 quad + 0..3 (second read: + 4) of the slice, 16 columns, and lane l16 receives column l16
            const int krow = 8 * quad + (l16 >> 2);
            const int swv = swz_col_tile(krow);
#pragma unroll
            for (int nb = 0; nb < NRD; ++nb) {
                const int n = 16 * (N16 * wn + (nb < N16 ? nb : 0)), col = (n & 127) + 4 * (l16 & 3);
                n_rd[nb] = lds_addr(&b_lds[0][0]) + (n >> 7) * kColTile + krow * 256 + 16 * ((col >> 3) ^ swv) + 2 * (col & 7);
            }
        }
    }

    f32x4 acc[N16][M16];
#pragma unroll
    for (int nb = 0; nb < N16; ++nb)
#pragma unroll
        for (int mb = 0; mb < M16; ++mb) acc[nb][mb] = f32x4{0.f, 0.f, 0.f, 0.f};

    // n fragment nb / m fragment mb of slice ks of a stage
    auto read_n = [&](auto stage_tag, int ks, int nb) __attribute__((always_inline)) -> s16x8 {
        constexpr int BOFF = decltype(stage_tag)::value * SH::B_PANEL;
        if (NT) return lds_read_b128(n_rd[ks], BOFF + nb * BLK);
        const s16x4 t0 = lds_read_tr16(n_rd[nb], BOFF + (32 * ks) * 256);
        const s16x4 t1 = lds_read_tr16(n_rd[nb], BOFF + (32 * ks + 4) * 256);
        return s16x8{t0[0], t0[1], t0[2], t0[3], t1[0], t1[1], t1[2], t1[3]};
    };
    auto read_m = [&](auto stage_tag, int ks, int mb) __attribute__((always_inline)) -> s16x8 {
        constexpr int AOFF = decltype(stage_tag)::value * SH::A_PANEL;
        return lds_read_b128(m_rd[ks], AOFF + mb * BLK);
    };
    // ---- main loop ---------------------------------------------------------------------------------------
    // A slice is N16 groups of M16 MFMAs (group nb: n fragment nb against every m fragment).  The n fragments are
    // double-buffered: the next slice's are read during groups 1 .. N16-2, one read after an MFMA; the m fragments have
    // one buffer, refilled in the last group, fragment mb right after the last MFMA that uses it.  The workgroup's only
    // barrier per K step sits after group 0 of the step's second slice: by then every read of the stage has returned
    // (the last were issued a group earlier) and the wave's share of the next stage's copy, issued a whole step
    // before, has landed; what follows the barrier reads the next stage and copies the step after next into the stage
    // just vacated, one copy after an MFMA.  Every MFMA, read and copy is pinned where it is written (scheduling
    // barriers): left alone the compiler moves reads down to just before their use, where nothing of the wave covers
    // their latency.
    s16x8 nf[2][N16], mf[M16];
    constexpr int NC = CA + CB;
    constexpr int MID = (N16 - 2) * M16;    // MFMAs of groups 1 .. N16-2
    auto pin = [&]() __attribute__((always_inline)) { __builtin_amdgcn_sched_barrier(0); };
    // one slice: MFMAs on nf[buf] and mf; `next_tag`/`ks_next` name the slice read meanwhile (has_next: there is one);
    // SECOND: the step's second slice, with the barrier after group 0 and, if copy_kt >= 0, that step's copies after it
    // this wave's copies of all but the `later` most recently issued steps have landed (copies retire in order)
    auto wait_stages = [&](int later) __attribute__((always_inline)) {
        if (NS >= 4 && later >= 3) wait_vmcnt<(NS >= 4 ? 3 : 0) * NC>();
        else if (NS >= 3 && later == 2) wait_vmcnt<(NS >= 3 ? 2 : 0) * NC>();
        else if (later == 1) wait_vmcnt<NC>();
        else wait_vmcnt<0>();
    };
    auto k_slice = [&](auto next_tag, int ks_next, int buf, bool has_next, auto second_tag, int copy_kt, auto stage_tag, int later = 0) __attribute__((always_inline)) {
        constexpr bool SECOND = decltype(second_tag)::value;
        constexpr int STAGE = decltype(stage_tag)::value;
#pragma unroll
        for (int nb = 0; nb < N16; ++nb) {
#pragma unroll
            for (int mb = 0; mb < M16; ++mb) {
                acc[nb][mb] = T::mfma16(nf[buf][nb], mf[mb], acc[nb][mb]);
                pin();
                if (nb >= 1 && nb <= N16 - 2) {
                    const int i = (nb - 1) * M16 + mb;   // 0 .. MID-1
                    if (has_next) {
#pragma unroll
                        for (int r = (N16 * i + MID - 1) / MID; r < (N16 * (i + 1) + MID - 1) / MID; ++r) nf[buf ^ 1][r] = read_n(next_tag, ks_next, r);
                    }
                    if (SECOND && copy_kt >= 0) {
#pragma unroll
                        for (int c = (NC * i + MID - 1) / MID; c < (NC * (i + 1) + MID - 1) / MID; ++c) copy_one(copy_kt, STAGE, c);
                    }
                } else if (nb == N16 - 1) {
                    if (has_next) mf[mb] = read_m(next_tag, ks_next, mb);
                }
                pin();
            }
            if (SECOND && nb == 0) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // this wave has read everything it needs from this stage
                wait_stages(later);                                    // and its share of the next stage has landed
                __syncthreads();
                pin();
            }
        }
    };
    auto step = [&](auto stage_tag, int kt) __attribute__((always_inline)) {
        constexpr int STAGE = decltype(stage_tag)::value;
        using Next = std::integral_constant<int, (STAGE + 1) % NS>;
        pin();
        k_slice(stage_tag, 1, 0, true, std::false_type{}, -1, stage_tag);
        // at the barrier the next step's stage must have landed; the steps after it, up to NS - 2 of them, may be in flight
        k_slice(Next{}, 0, 1, kt + 1 < KT, std::true_type{}, kt + NS < KT ? kt + NS : -1, stage_tag, min(NS - 2, KT - 2 - kt));
    };
#pragma unroll
    for (int st = 0; st < NS; ++st)
        if (st < KT) issue(st, st);
    wait_stages(min(NS, KT) - 1);   // the copies of step 0 retire first
    __syncthreads();
#pragma unroll
    for (int nb = 0; nb < N16; ++nb) nf[0][nb] = read_n(std::integral_constant<int, 0>{}, 0, nb);
#pragma unroll
    for (int mb = 0; mb < M16; ++mb) mf[mb] = read_m(std::integral_constant<int, 0>{}, 0, mb);
    for (int kt = 0; kt < KT; kt += NS) {
        step(std::integral_constant<int, 0>{}, kt);
        if (kt + 1 < KT) step(std::integral_constant<int, 1>{}, kt + 1);
        if constexpr (NS > 2) if (kt + 2 < KT) step(std::integral_constant<int, 2 % NS>{}, kt + 2);
        if constexpr (NS > 3) if (kt + 3 < KT) step(std::integral_constant<int, 3 % NS>{}, kt + 3);
    }

    // ---- epilogue: D = alpha * acc + beta * C; register e of a block is n = 4 quad + e, m = l16 ----
    const short* Cg = (const short*)p.C;
#pragma unroll
    for (int mb = 0; mb < M16; ++mb) {
        const int m = m0 + 16 * M16 * wm + 16 * mb + l16;
        if (m >= p.M) continue;
#pragma unroll
        for (int nb = 0; nb < N16; ++nb) {
            int nb0 = n0 + 16 * N16 * wn + 16 * nb;   // first column of the block
            if (CONCAT) {                              // ... inside the weight that holds the block
                int local;
                const int sg = group_of_unit(p.grp, nb0, local);
                nb0 = local;
                Dg = (short*)(sg == 0 ? p.grp.D[0] : sg == 1 ? p.grp.D[1] : p.grp.D[2]);
                ldd = sg == 0 ? p.grp.ldd[0] : sg == 1 ? p.grp.ldd[1] : p.grp.ldd[2];
            }
            const int n = nb0 + 4 * quad;
            if (!CONCAT && n >= N) continue;
            if (SPLIT) {   // the slice's raw sums; gemm_reduce_kernel adds the slices up and applies alpha, beta and C
                *reinterpret_cast<f32x4*>(p.part + ((int64_t)slice * p.M + m) * N + n) = acc[nb][mb];
                continue;
            }
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = p.alpha * acc[nb][mb][e];
            if (p.beta != 0.f) {
                const s16x4 c = *reinterpret_cast<const s16x4*>(Cg + (int64_t)m * p.ldc + n);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] += p.beta * T::to_float(c[e]);
            }
            uint2 pk;
            pk.x = T::pack2(v[0], v[1]);
            pk.y = T::pack2(v[2], v[3]);
            *reinterpret_cast<uint2*>(Dg + (int64_t)m * ldd + n) = pk;
        }
    }
}

// Few rows of A (the tokens of a decode step) against a weight stored [N, K]: the work is reading the weight once.
// A workgroup owns 16 columns n of D and all K; its 8 waves split K, each streaming its slice of the 16 weight rows
// (non-temporal 32-byte pieces per lane, four lanes covering one 128-byte line of a row) into the A operand of
// v_mfma_f32_16x16x32, the rows of A (from L2) being the B operand, 16 at a time; the waves' partial sums meet in LDS.
// Within a 64-wide K step lane (row, quad) takes k = 16*quad + 0..15 for both operands, which is just another order
// of the contraction.  MB = ceil(M / 16) <= 4.
constexpr int kSkinnyWaves = 8;
// NR groups of 16 columns per workgroup (2 for wide weights: half as many workgroups, each A fragment used twice)
template <class T, int MB, int NR, bool GROUPED = false>
__global__ __launch_bounds__(kSkinnyWaves * 64) void gemm_skinny_kernel(const GemmParams p) {
    __shared__ f32x4 part[kSkinnyWaves][NR][MB][64];
    const int lane = threadIdx.x & 63, w = wave_id();
    const int l16 = lane & 15, quad = lane >> 4;
    int n0 = (int)blockIdx.x * 16 * NR;
    const short* Bg = (const short*)p.B;
    short* Dg = (short*)p.D;
    int N = p.N;
    int64_t ldb = p.ldb, ldd = p.ldd;
    if (GROUPED) {   // the workgroup's weight, output and place inside them (uniform)
        int local;
        const int sg = group_of_unit(p.grp, (int)blockIdx.x, local);
        n0 = local * 16 * NR;
        Bg = (const short*)(sg == 0 ? p.grp.B[0] : sg == 1 ? p.grp.B[1] : p.grp.B[2]);
        Dg = (short*)(sg == 0 ? p.grp.D[0] : sg == 1 ? p.grp.D[1] : p.grp.D[2]);
        N = sg == 0 ? p.grp.N[0] : sg == 1 ? p.grp.N[1] : p.grp.N[2];
        ldb = sg == 0 ? p.grp.ldb[0] : sg == 1 ? p.grp.ldb[1] : p.grp.ldb[2];
        ldd = sg == 0 ? p.grp.ldd[0] : sg == 1 ? p.grp.ldd[1] : p.grp.ldd[2];
    }
    const int steps = p.K / 64, per = (steps + kSkinnyWaves - 1) / kSkinnyWaves;
    const int s0 = w * per, s1 = min(steps, s0 + per);
    const short* wrow[NR];
#pragma unroll
    for (int nr = 0; nr < NR; ++nr) wrow[nr] = Bg + (int64_t)min(n0 + 16 * nr + l16, N - 1) * ldb + 16 * quad;
    const short* xrow[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) xrow[mb] = (const short*)p.A + (int64_t)min(16 * mb + l16, p.M - 1) * p.lda + 16 * quad;
    f32x4 acc[NR][MB];
#pragma unroll
    for (int nr = 0; nr < NR; ++nr)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[nr][mb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int s = s0; s < s1; ++s) {
        const int k0 = 64 * s;
        s16x8 w0[NR], w1[NR];
#pragma unroll
        for (int nr = 0; nr < NR; ++nr) {
            w0[nr] = stream_load(reinterpret_cast<const s16x8*>(wrow[nr] + k0));
            w1[nr] = stream_load(reinterpret_cast<const s16x8*>(wrow[nr] + k0 + 8));
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const s16x8 x0 = *reinterpret_cast<const s16x8*>(xrow[mb] + k0);
            const s16x8 x1 = *reinterpret_cast<const s16x8*>(xrow[mb] + k0 + 8);
#pragma unroll
            for (int nr = 0; nr < NR; ++nr) {
                acc[nr][mb] = T::mfma16(w0[nr], x0, acc[nr][mb]);
                acc[nr][mb] = T::mfma16(w1[nr], x1, acc[nr][mb]);
            }
        }
    }
#pragma unroll
    for (int nr = 0; nr < NR; ++nr)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) part[w][nr][mb][lane] = acc[nr][mb];
    __syncthreads();
    // wave j adds up block (nr, mb) = (j / MB, j % MB): register r of a lane is n = n0 + 16*nr + 4*quad + r, m = 16*mb + l16
    if (w >= NR * MB) return;
    const int nr = w / MB, mb = w - nr * MB;
    f32x4 sum = part[0][nr][mb][lane];
#pragma unroll
    for (int ww = 1; ww < kSkinnyWaves; ++ww) sum += part[ww][nr][mb][lane];
    const int m = 16 * mb + l16, n = n0 + 16 * nr + 4 * quad;
    if (m >= p.M || n >= N) return;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = p.alpha * sum[e];
    if (p.beta != 0.f) {
        const s16x4 c = *reinterpret_cast<const s16x4*>((const short*)p.C + (int64_t)m * p.ldc + n);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += p.beta * T::to_float(c[e]);
    }
    uint2 pk;
    pk.x = T::pack2(v[0], v[1]);
    pk.y = T::pack2(v[2], v[3]);
    *reinterpret_cast<uint2*>(Dg + (int64_t)m * ldd + n) = pk;
}

template <class T, int NR>
static void launch_skinny_nr(const GemmParams& p, hipStream_t stream) {
    const dim3 grid((p.N + 16 * NR - 1) / (16 * NR)), block(kSkinnyWaves * 64);
    const int mb = (p.M + 15) / 16;
    if (mb == 1) hipLaunchKernelGGL((gemm_skinny_kernel<T, 1, NR>), grid, block, 0, stream, p);
    else if (mb == 2) hipLaunchKernelGGL((gemm_skinny_kernel<T, 2, NR>), grid, block, 0, stream, p);
    else if (mb == 3) hipLaunchKernelGGL((gemm_skinny_kernel<T, 3, NR>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((gemm_skinny_kernel<T, 4, NR>), grid, block, 0, stream, p);
}
// The few-row kernel for large weights.  gemm_skinny_kernel's weight loads put 16 different weight rows into every
// quarter of a wave, 16 cache lines touched for 256 bytes, and that, not HBM, is what it runs at (4.5 TB/s of the weight
// at any row count).  Here the weight rows and the activation rows take the long way round: global -> LDS copies whose
// lanes walk along the rows (a copy instruction moves 256 consecutive bytes of each of four rows, 4 lines per quarter
// wave), and the MFMA fragments are read back from LDS.  A workgroup of four waves owns 16 columns; wave w takes every
// fourth 128-wide K segment, each wave with its own two-stage LDS area (no barrier until the final sum): per segment
// 4 copies for the 16 weight rows, 4 for up to 16 activation rows, 4 MFMAs.  Four rows of a copy share a 1 KiB block
// of LDS, blocks 64 bytes apart in the banks, so that the 16 rows of a fragment read hit 16 different bank groups.
constexpr int kRowsSeg = 128;                                  // K values per segment
constexpr int kRowsBlock = 1024 + 64;                          // LDS bytes of four rows' segment, padded
constexpr int kRowsStage = 4 * kRowsBlock;                     // 16 rows
// XI: copy instructions that hold activation rows (four rows each, M <= 4 * XI); fragment columns past them multiply
// whatever their LDS block holds into output columns that are never stored.
// GROUPED: the 16-column groups of up to three weights numbered through (p.grp.end in groups), alpha = 1 and no C.
template <class T, int XI, bool GROUPED>
__global__ __launch_bounds__(4 * 64) void gemm_rows_lds_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) char wx[4][2][2][kRowsStage];   // [wave][stage][weights, activations]
    __shared__ f32x4 part[4][64];
    const int lane = threadIdx.x & 63, w = wave_id();
    const int l16 = lane & 15, quad = lane >> 4;
    int n0 = (int)blockIdx.x * 16;
    const short* Bg = (const short*)p.B;
    short* Dg = (short*)p.D;
    int N = p.N;
    int64_t ldb = p.ldb, ldd = p.ldd;
    if (GROUPED) {   // the workgroup's weight, output and place inside them (uniform)
        int local;
        const int sg = group_of_unit(p.grp, (int)blockIdx.x, local);
        n0 = local * 16;
        Bg = (const short*)(sg == 0 ? p.grp.B[0] : sg == 1 ? p.grp.B[1] : p.grp.B[2]);
        Dg = (short*)(sg == 0 ? p.grp.D[0] : sg == 1 ? p.grp.D[1] : p.grp.D[2]);
        N = sg == 0 ? p.grp.N[0] : sg == 1 ? p.grp.N[1] : p.grp.N[2];
        ldb = sg == 0 ? p.grp.ldb[0] : sg == 1 ? p.grp.ldb[1] : p.grp.ldb[2];
        ldd = sg == 0 ? p.grp.ldd[0] : sg == 1 ? p.grp.ldd[1] : p.grp.ldd[2];
    }
    const int nseg = p.K / kRowsSeg;                           // a multiple of 4: every wave the same number
    const int per = nseg / 4;
    // copy instruction i of a segment: lane L takes piece L >> 2 of row 4i + (L & 3)
    const short* wsrc[4];
    const short* xsrc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        wsrc[i] = Bg + (int64_t)min(n0 + 4 * i + (lane & 3), N - 1) * ldb + 8 * (lane >> 2);
        xsrc[i] = (const short*)p.A + (int64_t)min(4 * i + (lane & 3), p.M - 1) * p.lda + 8 * (lane >> 2);
    }
    auto issue = [&](int t, int stage) {                       // the wave's t-th segment
        const int k0 = (4 * t + w) * kRowsSeg;
#pragma unroll
        for (int i = 0; i < 4; ++i) copy16_global_to_lds(wsrc[i] + k0, &wx[w][stage][0][i * kRowsBlock]);
#pragma unroll
        for (int i = 0; i < XI; ++i) copy16_global_to_lds(xsrc[i] + k0, &wx[w][stage][1][i * kRowsBlock]);
    };
    // fragment of k step s (32 values) for row r = l16: piece 4s + quad of the row, inside the row's block of four
    const int frag = (l16 >> 2) * kRowsBlock + 16 * (l16 & 3) + 64 * quad;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    issue(0, 0);
    for (int t = 0; t < per; ++t) {
        if (t + 1 < per) { issue(t + 1, (t + 1) & 1); wait_vmcnt<4 + XI>(); } else wait_vmcnt<0>();
        const char* wb = &wx[w][t & 1][0][frag];
        const char* xb = &wx[w][t & 1][1][frag];
#pragma unroll
        for (int s = 0; s < kRowsSeg / 32; ++s) {
            const s16x8 a = *reinterpret_cast<const s16x8*>(wb + 256 * s);
            const s16x8 b = *reinterpret_cast<const s16x8*>(xb + 256 * s);
            acc = T::mfma16(a, b, acc);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // the fragments are in registers before the stage is refilled
    }
    part[w][lane] = acc;
    __syncthreads();
    if (w != 0) return;
    f32x4 sum = part[0][lane];
#pragma unroll
    for (int ww = 1; ww < 4; ++ww) sum += part[ww][lane];
    const int m = l16, n = n0 + 4 * quad;      // register r of a lane: weight row n + r, activation row m
    if (m >= p.M || n >= N) return;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = GROUPED ? sum[e] : p.alpha * sum[e];
    if (!GROUPED && p.beta != 0.f) {
        const s16x4 c = *reinterpret_cast<const s16x4*>((const short*)p.C + (int64_t)m * p.ldc + n);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += p.beta * T::to_float(c[e]);
    }
    uint2 pk;
    pk.x = T::pack2(v[0], v[1]);
    pk.y = T::pack2(v[2], v[3]);
    *reinterpret_cast<uint2*>(Dg + (int64_t)m * ldd + n) = pk;
}
// (16 rows at most, K a multiple of 512)
static bool rows_lds_takes(int64_t M, int64_t K) { return M <= 16 && K % (4 * kRowsSeg) == 0; }
template <class T, bool GROUPED = false>
static int launch_rows_lds(const GemmParams& p, int groups, hipStream_t stream) {
    const dim3 grid(groups), block(4 * 64);
    if (p.M <= 4) hipLaunchKernelGGL((gemm_rows_lds_kernel<T, 1, GROUPED>), grid, block, 0, stream, p);
    else if (p.M <= 8) hipLaunchKernelGGL((gemm_rows_lds_kernel<T, 2, GROUPED>), grid, block, 0, stream, p);
    else if (p.M <= 12) hipLaunchKernelGGL((gemm_rows_lds_kernel<T, 3, GROUPED>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((gemm_rows_lds_kernel<T, 4, GROUPED>), grid, block, 0, stream, p);
    return check_launch("gemm_rows_lds_kernel");
}

// Up to 64 rows against a wide [N, K] weight (a batch of decode steps against an FFN or output-head weight): a workgroup
// of four waves owns a stripe of 64 columns over the whole of K; K goes by in segments of 256 values, the 64 weight rows
// and the activation rows copied global -> LDS with instructions whose lanes walk along the rows (512 consecutive bytes
// of each of two rows, 2 lines per quarter wave); three weight stages (two segments in flight) and two or three
// activation stages, one workgroup per compute unit (segments of 128 values and two workgroups per unit are 15-25 %
// slower from 24 rows on).  No K slices across workgroups, so no partial sums in memory: the activations are read once
// per stripe (N / 64 times in all) and the weight once.  Two rows of a copy share a 1 KiB block of LDS; inside block i
// the 16-byte pieces of a row sit at piece ^ (i & 7), so the 16 rows of a fragment read hit 16 different bank groups
// without padding (160 KiB exactly at 49-64 rows).  It needs N / 64 stripes to fill the chip.
constexpr int kStripeSeg = 256;                                // K values per segment
constexpr int kStripeBlock = 1024;                             // LDS bytes of two rows' segment
template <int MB> struct StripeGeom {
    static constexpr int W_BYTES = 4 * 8 * kStripeBlock;       // 64 weight rows
    static constexpr int X_BYTES = MB * 8 * kStripeBlock;      // 16 * MB activation rows
    static constexpr int WST = MB >= 4 ? 2 : 3, XST = MB >= 3 ? 2 : 3;   // 120 / 144 / 144 / 128 KiB
    static constexpr int CW = 8, CX = 2 * MB;                  // copies per wave and segment
};
// SLICED: p.splits workgroups per stripe, each over its share of the segments; they leave raw fp32 sums in p.part
// ([slice][M][N]) for gemm_reduce_kernel.
// GROUPED: the stripes of up to three weights numbered through (p.grp.end in stripes), alpha = 1 and no C.
template <class T, int MB, bool SLICED = false, bool GROUPED = false>
__global__ __launch_bounds__(4 * 64) void gemm_stripe_kernel(const GemmParams p) {
    static_assert(!(SLICED && GROUPED), "the grouped launch has no workspace");
    using G = StripeGeom<MB>;
    constexpr int WST = G::WST, XST = G::XST;
    __shared__ __attribute__((aligned(16))) char w_lds[WST][G::W_BYTES];
    __shared__ __attribute__((aligned(16))) char x_lds[XST][G::X_BYTES];
    const int lane = threadIdx.x & 63, w = wave_id();
    const int l16 = lane & 15, quad = lane >> 4;
    int slice = 0, seg0 = 0, nseg = p.K / kStripeSeg;
    if (SLICED) {
        slice = (int)blockIdx.x % p.splits;
        seg0 = slice * nseg / p.splits;
        nseg = (slice + 1) * nseg / p.splits - seg0;
    }
    // Which columns.  SLICED: workgroup b / splits owns stripe b / splits.  Plain launches: the 16-column blocks of the weight
    // are shared out evenly: workgroup g of G owns blocks g * blocks / G ..
    // (g + 1) * blocks / G - 1 and goes through them four at a time, a chunk ending early at the end of the workgroup's
    // range; the waves without a block of their own in such a chunk copy its last row again (from L2) and
    // multiply what is never stored.  Every compute unit so streams the same share of the weight to within one block,
    // whatever the number of columns (448 stripes of 64 columns are one and three quarter rounds of 256 workgroups:
    // 28672 x 4096 from memory 46.5 -> 41.5-42.3 us), and a narrow weight is spread over the whole chip (6144 x 4096 at
    // 9-16 rows: 96 stripes 15.2-15.9 us, 256 workgroups of one or two blocks 12.3-12.7).
    // GROUPED: every weight has a run of workgroups of its own (p.grp.end counts them, cumulatively; the host hands them
    // out in proportion to the weights' blocks), and a workgroup's share is worked out inside its weight, once, before the
    // chunk loop: with the lookup of a chunk's weight inside the loop the grouped launch ran 20 us where the plain one ran
    // 11, for the same instructions and the same L2 traffic.
    int blk_first = SLICED ? 4 * ((int)blockIdx.x / p.splits) : (int)((int64_t)blockIdx.x * p.tiles_n / (int)gridDim.x);
    int blk_last = SLICED ? min(blk_first + 4, p.tiles_n) : (int)((int64_t)(blockIdx.x + 1) * p.tiles_n / (int)gridDim.x);
    const short* Bg = (const short*)p.B;
    short* Dg = (short*)p.D;
    int Nw = p.N;
    int64_t ldb = p.ldb, ldd = p.ldd;
    if (GROUPED) {   // the workgroup's weight, output and place among that weight's workgroups (uniform)
        int idx;
        const int sg = group_of_unit(p.grp, (int)blockIdx.x, idx);
        Bg = (const short*)(sg == 0 ? p.grp.B[0] : sg == 1 ? p.grp.B[1] : p.grp.B[2]);
        Dg = (short*)(sg == 0 ? p.grp.D[0] : sg == 1 ? p.grp.D[1] : p.grp.D[2]);
        Nw = sg == 0 ? p.grp.N[0] : sg == 1 ? p.grp.N[1] : p.grp.N[2];
        ldb = sg == 0 ? p.grp.ldb[0] : sg == 1 ? p.grp.ldb[1] : p.grp.ldb[2];
        ldd = sg == 0 ? p.grp.ldd[0] : sg == 1 ? p.grp.ldd[1] : p.grp.ldd[2];
        const int wgs = (sg == 0 ? p.grp.end[0] : sg == 1 ? p.grp.end[1] - p.grp.end[0] : p.grp.end[2] - p.grp.end[1]);
        const int blocks = (Nw + 15) / 16;
        blk_first = (int)((int64_t)idx * blocks / wgs);
        blk_last = (int)((int64_t)(idx + 1) * blocks / wgs);
    }
    for (int cb = blk_first; cb < blk_last;) {
    const int local = cb;
    const int nb = min(4, blk_last - cb);
    int N = Nw;
    N = min(N, 16 * (local + nb));                             // rows past the chunk are not this chunk's
    const int n0 = 16 * local + 16 * w;                        // the columns this wave copies and, at the end, writes
    // copy instruction for row pair i: lane L lands at byte 16 L of the block and fetches piece (L >> 1) ^ (i & 7) of
    // row 2i + (L & 1)
    const short* wsrc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        wsrc[i] = Bg + (int64_t)min(n0 + 2 * i + (lane & 1), N - 1) * ldb + 8 * ((lane >> 1) ^ i);
    const short* xsrc[2 * MB];                                 // this wave's share of the activation rows: row pairs w, w + 4, ...
#pragma unroll
    for (int j = 0; j < 2 * MB; ++j)
        xsrc[j] = (const short*)p.A + (int64_t)min(2 * (w + 4 * j) + (lane & 1), p.M - 1) * p.lda + 8 * ((lane >> 1) ^ ((w + 4 * j) & 7));
    // A chunk starts at segment (its place in the weight) mod nseg and wraps: the chunks running at one time then read
    // different segments of the activation rows instead of the same few lines of the same few L2 channels
    const int rot = (int)((SLICED ? blockIdx.x : (unsigned)(local >> 2)) % (unsigned)nseg);
    auto seg_k0 = [&](int t) { const int sg = t + rot; return (seg0 + (sg >= nseg ? sg - nseg : sg)) * kStripeSeg; };
    auto issue_w = [&](int t) {
        char* st = w_lds[t % WST];
        const int k0 = seg_k0(t);
#pragma unroll
        for (int i = 0; i < 8; ++i) copy16_global_to_lds(wsrc[i] + k0, st + (w * 8 + i) * kStripeBlock);
    };
    auto issue_x = [&](int t) {
        char* st = x_lds[t % XST];
        const int k0 = seg_k0(t);
#pragma unroll
        for (int j = 0; j < 2 * MB; ++j) copy16_global_to_lds(xsrc[j] + k0, st + (w + 4 * j) * kStripeBlock);
    };
    // Wave w multiplies k steps 2w and 2w + 1 of every segment for all 64 columns and all rows: every fragment is read
    // from LDS once per workgroup (a wave that owned 16 columns over the whole segment would read all activation
    // fragments, four times the traffic), and the four partial sums meet in LDS after the last segment.  Fragment of k
    // step s for row r = l16 of a 16-row set: piece 4s + quad of the row, in pair block r >> 1.
    const int row_off = (l16 >> 1) * kStripeBlock + 16 * (l16 & 1);
    int frag[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) frag[s] = row_off + 32 * ((4 * (2 * w + s) + quad) ^ (l16 >> 1));
    f32x4 acc[4][MB];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[c][mb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < WST - 1; ++t) {
        if (t < XST - 1 && t < nseg) issue_x(t);
        if (t < nseg) issue_w(t);
    }
    for (int t = 0; t < nseg; ++t) {
        __syncthreads();                                       // every wave has read segment t - 1: its stages may be refilled
        if (t + XST - 1 < nseg) issue_x(t + XST - 1);
        if (t + WST - 1 < nseg) issue_w(t + WST - 1);
        // segment t has landed once at most the copies issued after it are outstanding: the weight of the next two
        // segments and the activations of the next XST - 1
        const int after = nseg - 1 - t;
        if (after >= 2) wait_vmcnt<(WST - 1) * G::CW + (XST - 1) * G::CX>(); else if (after == 1) wait_vmcnt<G::CW + G::CX>(); else wait_vmcnt<0>();
        __syncthreads();                                       // ... for every wave's copies
        const char* wb = w_lds[t % WST];
        const char* xb = x_lds[t % XST];
        // all fragments of the wave's two k steps first, then the MFMAs: left to itself the compiler pipelines these reads
        // in one instantiation and waits for each before its MFMA in another (the grouped one ran twice as long for it)
        s16x8 a[2][4], b[2][MB];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) b[s][mb] = *reinterpret_cast<const s16x8*>(xb + mb * 8 * kStripeBlock + frag[s]);
#pragma unroll
            for (int c = 0; c < 4; ++c) a[s][c] = *reinterpret_cast<const s16x8*>(wb + c * 8 * kStripeBlock + frag[s]);
        }
        __builtin_amdgcn_sched_barrier(0);                     // (the scheduler moves nothing across this)
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) acc[c][mb] = T::mfma16(a[s][c], b[s][mb], acc[c][mb]);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // fragments in registers before the barrier that frees the stage
    }
    // partial sums of the four waves: wave u leaves column block c at red[u][c][mb][lane]; wave w adds up column block w
    // in the order of the waves
    __syncthreads();
    f32x4* red = reinterpret_cast<f32x4*>(&w_lds[0][0]);   // 16 MB KiB of the 96
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) red[((w * 4 + c) * MB + mb) * 64 + lane] = acc[c][mb];
    __syncthreads();
    const int n = n0 + 4 * quad;                               // register r of a lane: weight row n + r, activation row 16mb + l16
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int m = 16 * mb + l16;
        if (m >= p.M || n >= N) continue;
        f32x4 sum = red[((0 * 4 + w) * MB + mb) * 64 + lane];
#pragma unroll
        for (int u = 1; u < 4; ++u) sum += red[((u * 4 + w) * MB + mb) * 64 + lane];
        if (SLICED) {
            *reinterpret_cast<f32x4*>(p.part + ((int64_t)slice * p.M + m) * p.N + n) = sum;
            continue;
        }
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = p.alpha * sum[e];
        if (!GROUPED && p.beta != 0.f) {
            const s16x4 c = *reinterpret_cast<const s16x4*>((const short*)p.C + (int64_t)m * p.ldc + n);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += p.beta * T::to_float(c[e]);
        }
        uint2 pk;
        pk.x = T::pack2(v[0], v[1]);
        pk.y = T::pack2(v[2], v[3]);
        *reinterpret_cast<uint2*>(Dg + (int64_t)m * ldd + n) = pk;
    }
    cb += nb;
    if (cb < blk_last) __syncthreads();                        // the sums have been read: the next chunk's copies may land there
    }
}
// Which widths it takes (in stripes of 64 columns; weights coming from memory): from 96 on every row count that reaches
// it (14336 x 4096 at 2-32 rows 22.8-23.7 us, the 16-column kernel 24.3-32.4; 6144 x 4096 at 9-32 rows 12.3-15.5 against
// 14.4-21.5); 80 from 8 rows on and 64 from 32 rows on, where no workspace allows K slices (5120 x 5120 at 16 rows 15.8
// against 20.5; 4096 x 4096 at 32 rows 13.6 against 16.3); an output head from 5 rows on (128256 x 4096 at 8 rows 179 against
// 183, 57344 x 8192 166 against 185; up to 4 rows the kernels that keep more workgroups on a compute unit are ahead).
static bool stripe_takes(int64_t M, int64_t stripes, int64_t K) {
    if (M < 1 || M > 64 || K % kStripeSeg != 0) return false;
    if (stripes > 640) return M >= 5;
    return stripes >= 96 || (stripes >= 80 && M >= 8) || (stripes >= 64 && M >= 32);
}
// `blocks`: 16-column blocks in all (GROUPED: workgroups in all, p.grp.end counting them per weight).
template <class T, bool SLICED = false, bool GROUPED = false>
static int launch_stripe(const GemmParams& p0, int blocks, hipStream_t stream) {
    GemmParams p = p0;
    p.tiles_n = blocks;
    const dim3 grid(SLICED ? (blocks + 3) / 4 * p.splits : GROUPED ? blocks : std::min(blocks, 256)), block(4 * 64);   // (GROUPED: `blocks` is the number of workgroups)
    if (p.M <= 16) hipLaunchKernelGGL((gemm_stripe_kernel<T, 1, SLICED, GROUPED>), grid, block, 0, stream, p);
    else if (p.M <= 32) hipLaunchKernelGGL((gemm_stripe_kernel<T, 2, SLICED, GROUPED>), grid, block, 0, stream, p);
    else if (p.M <= 48) hipLaunchKernelGGL((gemm_stripe_kernel<T, 3, SLICED, GROUPED>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((gemm_stripe_kernel<T, 4, SLICED, GROUPED>), grid, block, 0, stream, p);
    return check_launch("gemm_stripe_kernel");
}
// A weight of fewer than 192 stripes: with a workspace, K slices bring the workgroups up to the chip's 256 compute units
// (every slice four segments at least); the slices' sums are added up by gemm_reduce_kernel.  1 = no slices.
static int stripe_slices(int64_t M, int64_t N, int64_t K) {
    const int64_t stripes = (N + 63) / 64;
    if (M < 1 || M > 64 || K % kStripeSeg != 0 || N % 8 != 0 || stripes >= 192) return 1;
    return (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(256 / stripes, K / kStripeSeg / 4), 16));
}

// One row against an [N, K] weight (a decode step's projection): a wave streams whole weight rows as consecutive 16-byte
// pieces (1 KiB per instruction, where the MFMA kernel above takes 128 bytes of each of 16 rows) and multiplies in the
// vector ALU, which one activation row leaves mostly idle; one fp32 sum per lane, added up over the lanes at the end of
// a row.  A row is cut into segments of 4096 values (8 pieces per lane); when it is a single segment the lane keeps the
// activations it needs in registers (XREG), otherwise the workgroup keeps the activation row in LDS.  A wave owns a run
// of consecutive rows and has the next two segments in flight.
constexpr int kGemvSegHalfs = 4096;
constexpr int kGemvSegPieces = kGemvSegHalfs / 8 / 64;     // 16-byte pieces per lane and segment
template <class T> MA_DEV float dot8(uint4 a, uint4 b, float acc);
template <> MA_DEV float dot8<F16>(uint4 a, uint4 b, float acc) {
    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h16x2, a.x), __builtin_bit_cast(h16x2, b.x), acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h16x2, a.y), __builtin_bit_cast(h16x2, b.y), acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h16x2, a.z), __builtin_bit_cast(h16x2, b.z), acc, false);
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(h16x2, a.w), __builtin_bit_cast(h16x2, b.w), acc, false);
}
template <> MA_DEV float dot8<BF16>(uint4 a, uint4 b, float acc) {   // a bf16 is the upper half of the fp32 of the same value
    const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, bw[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        acc = __builtin_fmaf(__builtin_bit_cast(float, aw[i] << 16), __builtin_bit_cast(float, bw[i] << 16), acc);
        acc = __builtin_fmaf(__builtin_bit_cast(float, aw[i] & 0xffff0000u), __builtin_bit_cast(float, bw[i] & 0xffff0000u), acc);
    }
    return acc;
}
constexpr int kGemvMaxKHalfs = 16384;                      // activation row kept in LDS: 32 KiB
// GROUPED: the rows of up to three weights numbered through (p.grp.end[s] = rows of weights 0 .. s), every weight with
// its own output; alpha = 1, no C.
// MR: activation rows (1-4; more than one only ungrouped): every weight piece is multiplied with the same piece of each.
template <class T, bool XREG, bool GROUPED, int MR = 1>
__global__ __launch_bounds__(4 * 64) void gemv_kernel(const GemmParams p, int rows_per_wave) {
    static_assert(MR == 1 || !GROUPED, "several activation rows: one weight only");
    __shared__ __attribute__((aligned(16))) short x_lds[XREG ? 8 : (MR == 1 ? kGemvMaxKHalfs : 2 * kGemvMaxKHalfs)];   // MR rows of K values: MR * K <= 32768
    const int tid = threadIdx.x, lane = tid & 63, w = wave_id();
    const int npiece = p.K / 8, nseg = XREG ? 1 : (p.K + kGemvSegHalfs - 1) / kGemvSegHalfs;
    const int wave = (int)blockIdx.x * 4 + w;
    const int n_rows = GROUPED ? p.grp.end[kMaxGroup - 1] : p.N;
    const int r0 = min(wave * rows_per_wave, n_rows - 1), r1 = min(n_rows, wave * rows_per_wave + rows_per_wave);
    const int units = max(r1 - r0, 0) * nseg;              // (row, segment) pairs of this wave (none for a wave past the rows)
    // where row number `row` lives: its weight row and its output element (wave-uniform)
    auto locate = [&](int row, const short*& wrow, short*& out) {
        if (GROUPED) {
            const int sg = (row >= p.grp.end[0]) + (row >= p.grp.end[1]);
            const int local = row - (sg == 0 ? 0 : sg == 1 ? p.grp.end[0] : p.grp.end[1]);
            wrow = (const short*)(sg == 0 ? p.grp.B[0] : sg == 1 ? p.grp.B[1] : p.grp.B[2]) +
                   (int64_t)local * (sg == 0 ? p.grp.ldb[0] : sg == 1 ? p.grp.ldb[1] : p.grp.ldb[2]);
            out = (short*)(sg == 0 ? p.grp.D[0] : sg == 1 ? p.grp.D[1] : p.grp.D[2]) + local;
        } else {
            wrow = (const short*)p.B + (int64_t)row * p.ldb;
            out = (short*)p.D + row;
        }
    };
    struct Unit { uint4 piece[kGemvSegPieces]; };
    auto request = [&](int u, Unit& un) {
        u = max(min(u, units - 1), 0);                     // past the end: the last unit again, never used
        const int row = r0 + u / nseg, seg = u % nseg;
        const short* base; short* unused;
        locate(row, base, unused);
#pragma unroll
        for (int j = 0; j < kGemvSegPieces; ++j)
            un.piece[j] = __builtin_bit_cast(uint4, stream_load(reinterpret_cast<const u32x4*>(base + 8 * min(seg * (kGemvSegHalfs / 8) + 64 * j + lane, npiece - 1))));
    };
    Unit ring[2];
    request(0, ring[0]);
    request(1, ring[1]);
    uint4 xr[MR][kGemvSegPieces];
    if (XREG) {
#pragma unroll
        for (int m = 0; m < MR; ++m)
#pragma unroll
            for (int j = 0; j < kGemvSegPieces; ++j)
                xr[m][j] = *reinterpret_cast<const uint4*>((const short*)p.A + (int64_t)min(m, p.M - 1) * p.lda + 8 * min(64 * j + lane, npiece - 1));
    } else {
        for (int i = tid; i < MR * npiece; i += 4 * 64) {
            const int m = i / npiece, pc = i - m * npiece;
            *reinterpret_cast<uint4*>(x_lds + 8 * i) = *reinterpret_cast<const uint4*>((const short*)p.A + (int64_t)min(m, p.M - 1) * p.lda + 8 * pc);
        }
        __syncthreads();
    }
    float acc[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[m] = 0.f;
    auto consume = [&](int u, Unit& un) {
        const int row = r0 + u / nseg, seg = u % nseg;
        uint4 wv[kGemvSegPieces];
#pragma unroll
        for (int j = 0; j < kGemvSegPieces; ++j) wv[j] = un.piece[j];
        request(u + 2, un);
#pragma unroll
        for (int j = 0; j < kGemvSegPieces; ++j) {
            const int piece = seg * (kGemvSegHalfs / 8) + 64 * j + lane;
            if (piece < npiece) {
#pragma unroll
                for (int m = 0; m < MR; ++m)
                    acc[m] = dot8<T>(wv[j], XREG ? xr[m][j] : *reinterpret_cast<const uint4*>(x_lds + 8 * (m * npiece + piece)), acc[m]);
            }
        }
        if (seg == nseg - 1) {
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                float v = acc[m];
                acc[m] = 0.f;
#pragma unroll
                for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off);
                if (lane == 0 && m < p.M) {
                    const short* unused; short* out;
                    locate(row, unused, out);
                    if (!GROUPED) {
                        v *= p.alpha;
                        if (p.beta != 0.f) v += p.beta * T::to_float(((const short*)p.C)[(int64_t)m * p.ldc + row]);
                        out += (int64_t)m * p.ldd;
                    }
                    *out = (short)(T::pack2(v, 0.f) & 0xffffu);
                }
            }
        }
    };
    for (int u = 0; u < units; u += 2) {
        consume(u, ring[0]);
        if (u + 1 < units) consume(u + 1, ring[1]);
    }
}
template <class T, bool GROUPED = false>
static int launch_gemv(const GemmParams& p, int n_rows, hipStream_t stream) {
    const int max_waves = 256 * 2 * 4;   // two workgroups of four waves per compute unit
    const int rows_per_wave = (n_rows + max_waves - 1) / max_waves;
    const int waves = (n_rows + rows_per_wave - 1) / rows_per_wave;
    const dim3 grid((waves + 3) / 4), block(4 * 64);
    const bool xreg = p.K <= kGemvSegHalfs;
#define MINFER_GEMV(XR, MR) hipLaunchKernelGGL((gemv_kernel<T, XR, GROUPED, MR>), grid, block, 0, stream, p, rows_per_wave)
    if (GROUPED || p.M == 1) { if (xreg) MINFER_GEMV(true, 1); else MINFER_GEMV(false, 1); }
    else if (p.M == 2) MINFER_GEMV(false, GROUPED ? 1 : 2);   // (several rows: rows longer than a segment only, see gemv_takes)
    else if (p.M == 3) MINFER_GEMV(false, GROUPED ? 1 : 3);
    else MINFER_GEMV(false, GROUPED ? 1 : 4);
#undef MINFER_GEMV
    return check_launch("gemv_kernel");
}
// which calls it takes: one row, or up to four rows longer than a segment whose activations fit its LDS area
static bool gemv_takes(int64_t M, int64_t K) { return M >= 1 && M <= 4 && K <= kGemvMaxKHalfs && (M == 1 || (K > kGemvSegHalfs && M * K <= 2 * kGemvMaxKHalfs)); }

template <class T>
static int launch_skinny(const GemmParams& p, hipStream_t stream) {
    // two column groups per workgroup once that still leaves 160 workgroups and there is more than one block of rows
    // to share between them (32 rows x 14336 columns: 52 -> 40 us; 64 x 6144: 38 -> 27; a single block of rows loses 5-10 %)
    if (p.M > 16 && p.N >= 160 * 32) launch_skinny_nr<T, 2>(p, stream);
    else launch_skinny_nr<T, 1>(p, stream);
    return check_launch("gemm_skinny_kernel");
}

// The few-row kernel over a weight stored as rows of Q8_0 blocks, [N][K/32] blocks of 34 bytes (an fp16 scale and 32
// int8; reference block format: csrc/common/types.hpp:141-146): every weight is dequantised to fp16 exactly as
// minfer_dequant_q8_0 does (reference: cuda/quants/impls.cuh:121-143) on its way into the MFMA, so the result is that of
// the fp16 kernel on the dequantised weight while the launch streams 34 bytes per 32 weights instead of 64.
// A K step is 128 wide: lane (row n, quad q) owns block 4s + q of its weight row, which is one MFMA A fragment per
// 8 values, and the activations of the same k for the B operand (64 contiguous bytes of row m).  Blocks start on
// 2-byte boundaries; a lane reads its block as the nine aligned words that cover it, and whether the block starts on a
// word or in the middle of one depends only on q (rows are multiples of 4 bytes), so one byte permute per quant word with
// a per-lane constant selector undoes the shift (dequant8_shifted).  fp16 activations only.
// The weight loads carry no non-temporal hint, unlike the fp16 kernel's: a 128-byte line of a weight row holds 3.8
// blocks, so the line a step ends in is the line the next step starts in, and a line loaded with the hint is not kept
// for that second touch (14336 x 4096 at one row: 31 us with the hint, 17.5 us without).
template <int MB, int NR>
__global__ __launch_bounds__(kSkinnyWaves * 64) void gemm_skinny_q8_kernel(const GemmParams p) {
    using T = F16;
    __shared__ f32x4 part[kSkinnyWaves][NR][MB][64];
    const int lane = threadIdx.x & 63, w = wave_id();
    const int l16 = lane & 15, quad = lane >> 4;
    const int n0 = (int)blockIdx.x * 16 * NR;
    const int nblk = p.K / 32;                                  // blocks per weight row
    const int steps = (nblk + 3) / 4, per = (steps + kSkinnyWaves - 1) / kSkinnyWaves;
    const int s0 = w * per, s1 = min(steps, s0 + per);
    const bool odd = (quad & 1) != 0;                           // block 4s + q starts 2 bytes past a word boundary
    const uint32_t sel = odd ? kQ8SelOdd : kQ8SelEven;
    const char* wrow[NR];
#pragma unroll
    for (int nr = 0; nr < NR; ++nr) wrow[nr] = (const char*)p.B + (int64_t)min(n0 + 16 * nr + l16, p.N - 1) * p.ldb;   // ldb in bytes here
    const short* xrow[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) xrow[mb] = (const short*)p.A + (int64_t)min(16 * mb + l16, p.M - 1) * p.lda;
    f32x4 acc[NR][MB];
#pragma unroll
    for (int nr = 0; nr < NR; ++nr)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[nr][mb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
    for (int s = s0; s < s1; ++s) {
        const int blk = 4 * s + quad;
        const bool real = blk < nblk;                           // K need not be a multiple of 128: the last step may be short
        const int bc = real ? blk : (quad & 1);               // a block of the same alignment class that exists (nblk is even)
        uint32_t wq[NR][9];
#pragma unroll
        for (int nr = 0; nr < NR; ++nr) {
            // four words per load, at addresses that are only word-aligned: the vector type says so
            typedef uint32_t u32x4_w __attribute__((ext_vector_type(4), aligned(4)));
            const uint32_t* src = reinterpret_cast<const uint32_t*>(wrow[nr] + (int64_t)bc * 34 - (odd ? 2 : 0));
            const u32x4_w a = *reinterpret_cast<const u32x4_w*>(src);
            const u32x4_w b = *reinterpret_cast<const u32x4_w*>(src + 4);
            wq[nr][0] = a[0]; wq[nr][1] = a[1]; wq[nr][2] = a[2]; wq[nr][3] = a[3];
            wq[nr][4] = b[0]; wq[nr][5] = b[1]; wq[nr][6] = b[2]; wq[nr][7] = b[3];
            wq[nr][8] = src[8];
        }
        s16x8 x[MB][4];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int j = 0; j < 4; ++j)   // a lane past the last block contributes exact zeros, whatever block 0 or 1 holds
                x[mb][j] = real ? *reinterpret_cast<const s16x8*>(xrow[mb] + 32 * bc + 8 * j) : s16x8{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int nr = 0; nr < NR; ++nr) {
            const uint16_t bits = (uint16_t)(odd ? wq[nr][0] >> 16 : wq[nr][0]);
            const _Float16 dh = real ? __builtin_bit_cast(_Float16, bits) : (_Float16)0.f;
            const h16x2 d2 = {dh, dh};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const s16x8 wf = dequant8_shifted(wq[nr][2 * j], wq[nr][2 * j + 1], wq[nr][2 * j + 2], sel, d2);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) acc[nr][mb] = T::mfma16(wf, x[mb][j], acc[nr][mb]);
            }
        }
    }
#pragma unroll
    for (int nr = 0; nr < NR; ++nr)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) part[w][nr][mb][lane] = acc[nr][mb];
    __syncthreads();
    // wave j adds up block (nr, mb) = (j / MB, j % MB): register r of a lane is n = n0 + 16*nr + 4*quad + r, m = 16*mb + l16
    if (w >= NR * MB) return;
    const int nr = w / MB, mb = w - nr * MB;
    f32x4 sum = part[0][nr][mb][lane];
#pragma unroll
    for (int ww = 1; ww < kSkinnyWaves; ++ww) sum += part[ww][nr][mb][lane];
    const int m = 16 * mb + l16, n = n0 + 16 * nr + 4 * quad;
    if (m >= p.M || n >= p.N) return;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = p.alpha * sum[e];
    if (p.beta != 0.f) {
        const s16x4 c = *reinterpret_cast<const s16x4*>((const short*)p.C + (int64_t)m * p.ldc + n);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += p.beta * T::to_float(c[e]);
    }
    uint2 pk;
    pk.x = T::pack2(v[0], v[1]);
    pk.y = T::pack2(v[2], v[3]);
    *reinterpret_cast<uint2*>((short*)p.D + (int64_t)m * p.ldd + n) = pk;
}

// One row against Q8_0 weights (a decode step's projections): the MFMA kernel above reads 136 bytes of each of 16 weight
// rows per instruction, which this chip's memory system serves at about half its rate.  Here a wave streams whole weight
// rows instead, as consecutive aligned 16-byte pieces (1 KiB per instruction), and does the arithmetic in the vector
// ALU, of which one activation row needs little: a weight row is cut into segments of 128 blocks (4352 bytes, a multiple
// of 16, which is why K must be a multiple of 256 and the rows 16-byte aligned); a segment's pieces go through the wave's
// LDS area, from which lane l takes blocks l and l + 64 as the nine aligned words that cover each (as
// gemm_skinny_q8_kernel does), dequantises them exactly as minfer_dequant_q8_0 does and multiplies them with the
// activations of the same positions into one fp32 sum per lane; after a row's last segment the 64 sums are added up.
// The activations a lane needs are the same for every weight row when a row is one segment (K <= 4096, XREG): it keeps
// them in registers; otherwise the workgroup keeps the activation row in LDS.  A wave owns a run of consecutive weight
// rows and always has the next two segments' pieces in flight.  (Two rows this way cost as much as the MFMA kernel, four
// half as much again: the dot products fill the vector ALU.)
constexpr int kGemvWaves = 4;
constexpr int kGemvSegBlocks = 128;                       // blocks per segment: two per lane
constexpr int kGemvSegBytes = kGemvSegBlocks * 34;        // 4352
constexpr int kGemvPieces = (kGemvSegBytes + 1023) / 1024;   // 16-byte pieces per lane and segment (5, the last one partly)
constexpr int kGemvMaxK = 16384;                          // activation row kept in LDS: 32 KiB
template <bool XREG>
__global__ __launch_bounds__(kGemvWaves * 64) void gemv_q8_kernel(const GemmParams p, int rows_per_wave) {
    using T = F16;
    __shared__ __attribute__((aligned(16))) char raw[kGemvWaves][kGemvSegBytes + 48];   // + the words a last block's read runs over
    __shared__ __attribute__((aligned(16))) short x_lds[XREG ? 8 : kGemvMaxK];
    const int tid = threadIdx.x, lane = tid & 63, w = wave_id();
    const int nblk = p.K / 32, nseg = XREG ? 1 : (nblk + kGemvSegBlocks - 1) / kGemvSegBlocks;
    const int wave = (int)blockIdx.x * kGemvWaves + w;
    const int r0 = min(wave * rows_per_wave, p.N - 1), r1 = min(p.N, wave * rows_per_wave + rows_per_wave);
    const int units = max(r1 - r0, 0) * nseg;              // (row, segment) pairs of this wave, row-major (none for a wave past the rows)
    const bool odd = (lane & 1) != 0;                      // blocks l and l + 64 start 2 bytes past a word boundary
    const uint32_t sel = odd ? kQ8SelOdd : kQ8SelEven;
    char* my_raw = raw[w];

    struct Unit { u32x4 piece[kGemvPieces]; };
    auto request = [&](int u, Unit& un) {
        u = max(min(u, units - 1), 0);                     // past the end: the last unit again (one cache line, never used)
        const int row = r0 + u / nseg, seg = u % nseg;
        const int pieces = min(kGemvSegBlocks, nblk - seg * kGemvSegBlocks) * 34 / 16;   // a multiple of 8 blocks: whole pieces
        const char* base = (const char*)p.B + (int64_t)row * p.ldb + (int64_t)seg * kGemvSegBytes;
#pragma unroll
        for (int j = 0; j < kGemvPieces; ++j)
            un.piece[j] = *reinterpret_cast<const u32x4*>(base + 16 * min(64 * j + lane, pieces - 1));
    };
    Unit ring[2];
    request(0, ring[0]);
    request(1, ring[1]);
    // ---- the activations, while the first weight pieces are on their way ---------------------------------
    uint4 xr[2][4];
    if (XREG) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                xr[i][j] = *reinterpret_cast<const uint4*>((const short*)p.A + 32 * min(lane + 64 * i, nblk - 1) + 8 * j);
    } else {
        for (int i = tid; i < p.K / 8; i += kGemvWaves * 64)
            *reinterpret_cast<s16x8*>(x_lds + 8 * i) = *reinterpret_cast<const s16x8*>((const short*)p.A + 8 * i);
        __syncthreads();
    }
    float acc = 0.f;
    auto consume = [&](int u, Unit& un) {
        const int row = r0 + u / nseg, seg = u % nseg;
        const int seg_blocks = min(kGemvSegBlocks, nblk - seg * kGemvSegBlocks);
        const int pieces = seg_blocks * 34 / 16;
#pragma unroll
        for (int j = 0; j < kGemvPieces; ++j)
            *reinterpret_cast<u32x4*>(my_raw + 16 * min(64 * j + lane, pieces - 1)) = un.piece[j];
        request(u + 2, un);                                // the registers are free again: two units ahead
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int b = lane + 64 * i;
            if (b < seg_blocks) {
                const uint32_t* wp = reinterpret_cast<const uint32_t*>(my_raw + ((34 * b) & ~3));
                uint32_t wq[9];
#pragma unroll
                for (int j = 0; j < 9; ++j) wq[j] = wp[j];
                const uint16_t bits = (uint16_t)(odd ? wq[0] >> 16 : wq[0]);
                const _Float16 dh = __builtin_bit_cast(_Float16, bits);
                const h16x2 d2 = {dh, dh};
                const short* xb = x_lds + (XREG ? 0 : 32 * (seg * kGemvSegBlocks + b));
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint4 wf = __builtin_bit_cast(uint4, dequant8_shifted(wq[2 * j], wq[2 * j + 1], wq[2 * j + 2], sel, d2));
                    const uint4 xv = XREG ? xr[i][j] : *reinterpret_cast<const uint4*>(xb + 8 * j);
                    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h16x2, wf.x), __builtin_bit_cast(h16x2, xv.x), acc, false);
                    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h16x2, wf.y), __builtin_bit_cast(h16x2, xv.y), acc, false);
                    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h16x2, wf.z), __builtin_bit_cast(h16x2, xv.z), acc, false);
                    acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h16x2, wf.w), __builtin_bit_cast(h16x2, xv.w), acc, false);
                }
            }
        }
        if (seg == nseg - 1) {                             // the row is complete: add the lanes' sums up and store
            float v = acc;
            acc = 0.f;
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off);
            if (lane == 0) {
                v *= p.alpha;
                if (p.beta != 0.f) v += p.beta * T::to_float(((const short*)p.C)[row]);
                ((short*)p.D)[row] = (short)(T::pack2(v, 0.f) & 0xffffu);
            }
        }
    };
    for (int u = 0; u < units; u += 2) {
        consume(u, ring[0]);
        if (u + 1 < units) consume(u + 1, ring[1]);
    }
}

// which calls the row-streaming kernel takes: one row, whole segments of 16-byte pieces, an activation row that fits its LDS area
static bool q8_gemv_ok(int64_t M, int64_t K, const void* Bq, int64_t row_bytes) {
    return M == 1 && K % 256 == 0 && K <= kGemvMaxK && aligned16(Bq) && row_bytes % 16 == 0;
}
static int launch_gemv_q8(const GemmParams& p, hipStream_t stream) {
    // as many waves as the chip holds at a time when there are rows enough for them: two workgroups per compute unit
    const int max_waves = 256 * 2 * kGemvWaves;
    const int rows_per_wave = (p.N + max_waves - 1) / max_waves;
    const int waves = (p.N + rows_per_wave - 1) / rows_per_wave;
    const dim3 grid((waves + kGemvWaves - 1) / kGemvWaves), block(kGemvWaves * 64);
    if (p.K <= 32 * kGemvSegBlocks) hipLaunchKernelGGL((gemv_q8_kernel<true>), grid, block, 0, stream, p, rows_per_wave);
    else hipLaunchKernelGGL((gemv_q8_kernel<false>), grid, block, 0, stream, p, rows_per_wave);
    return check_launch("gemv_q8_kernel");
}

static int launch_skinny_q8(const GemmParams& p, hipStream_t stream) {
    const int mb = (p.M + 15) / 16;
    // two column groups per workgroup as soon as there is more than one row and the weight is wide enough to leave 160
    // workgroups: the activations are re-read from L2 for every group of columns, and from 8 rows on they are more bytes than
    // a group's blocks (14336 columns, 8 / 16 rows: 22.2 -> 18.4 us, 27.1 -> 20.7 us)
    const bool two = p.M > 1 && p.N >= 160 * 32;
    const dim3 grid((p.N + (two ? 32 : 16) - 1) / (two ? 32 : 16)), block(kSkinnyWaves * 64);
#define MINFER_SKINNY_Q8(MB, NR) hipLaunchKernelGGL((gemm_skinny_q8_kernel<MB, NR>), grid, block, 0, stream, p)
    if (!two) { if (mb == 1) MINFER_SKINNY_Q8(1, 1); else if (mb == 2) MINFER_SKINNY_Q8(2, 1); else if (mb == 3) MINFER_SKINNY_Q8(3, 1); else MINFER_SKINNY_Q8(4, 1); }
    else { if (mb == 1) MINFER_SKINNY_Q8(1, 2); else if (mb == 2) MINFER_SKINNY_Q8(2, 2); else if (mb == 3) MINFER_SKINNY_Q8(3, 2); else MINFER_SKINNY_Q8(4, 2); }
#undef MINFER_SKINNY_Q8
    return check_launch("gemm_skinny_q8_kernel");
}

// The stripe kernel over a weight of Q8_0 blocks ([N][K/32] blocks of 34 bytes, K a multiple of 256, rows 16-byte
// aligned): the same sharing out of 16-column blocks, chunks of four, segments of 256 values, split of a segment's k
// steps over the four waves and sum through LDS as gemm_stripe_kernel, with the weight staged as the raw blocks.  A
// segment of a row is 8 blocks = 272 bytes = 17 pieces of 16 bytes; the 64 rows of a chunk are 1088 pieces = 17 copy
// instructions of 64 lanes, lane L of instruction j taking piece 64 j + L of the chunk (row (64 j + L) / 17), so that
// a stage is the 64 row segments one after the other, 272 bytes each (a fragment's 16 rows are 68 words apart: 16
// different groups of four banks).  Every wave issues five of them per segment (j = w, w + 4, ..; the three past the
// seventeenth fetch the chunk's last piece again and land behind the stage).  A k step is one block: the lane of row
// r, k quarter q reads the three aligned words that cover values 8 q .. 8 q + 7 of block 2 w + s of its row's segment
// and dequantises them exactly as minfer_dequant_q8_0 does (dequant8_shifted; block 2 w starts on a word boundary,
// block 2 w + 1 two bytes past one), so the result is that of the fp16 kernels on the dequantised weight.
constexpr int kQ8SegBytes = 272;
constexpr int kQ8Stage = 22 * 1024;                            // 17 KiB of row segments, 3 KiB the extra copies land in; three stages hold the 64 KiB of partial sums
// SLICED: p.splits workgroups per chunk of four blocks, each over its share of the segments; raw fp32 sums into p.part
// ([slice][M][N]) for gemm_reduce_kernel (a narrow weight with a workspace, as gemm_stripe_kernel has it).
template <int MB, bool SLICED = false>
__global__ __launch_bounds__(4 * 64) void gemm_stripe_q8_kernel(const GemmParams p) {
    using T = F16;
    using G = StripeGeom<MB>;
    constexpr int WST = 3, XST = MB >= 3 ? 2 : 3, CW = 5, CX = 2 * MB;   // 90 / 114 / 114 / 130 KiB
    static_assert(WST * kQ8Stage >= 4 * 4 * MB * 64 * 16, "the partial sums reuse the weight stages");
    __shared__ __attribute__((aligned(16))) char w_lds[WST][kQ8Stage];
    __shared__ __attribute__((aligned(16))) char x_lds[XST][G::X_BYTES];
    const int lane = threadIdx.x & 63, w = wave_id();
    const int l16 = lane & 15, quad = lane >> 4;
    int slice = 0, seg0 = 0, nseg = p.K / kStripeSeg;
    if (SLICED) {
        slice = (int)blockIdx.x % p.splits;
        seg0 = slice * nseg / p.splits;
        nseg = (slice + 1) * nseg / p.splits - seg0;
    }
    const int blk_first = SLICED ? 4 * ((int)blockIdx.x / p.splits) : (int)((int64_t)blockIdx.x * p.tiles_n / (int)gridDim.x);
    const int blk_last = SLICED ? min(blk_first + 4, p.tiles_n) : (int)((int64_t)(blockIdx.x + 1) * p.tiles_n / (int)gridDim.x);
    // x fragments as in gemm_stripe_kernel; weight fragment of (column block c, k step s): three words at
    // 272 (16 c + l16) + 68 w + 32 s + 8 quad, the block's scale two bytes further for s = 1
    const int row_off = (l16 >> 1) * kStripeBlock + 16 * (l16 & 1);
    int frag[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) frag[s] = row_off + 32 * ((4 * (2 * w + s) + quad) ^ (l16 >> 1));
    const int wfrag = kQ8SegBytes * l16 + 68 * w + 8 * quad;
    for (int cb = blk_first; cb < blk_last;) {
    const int nb = min(4, blk_last - cb);
    const int N = min(p.N, 16 * (cb + nb));                    // rows past the chunk are not this chunk's
    const char* wsrc[CW];
#pragma unroll
    for (int i = 0; i < CW; ++i) {
        const int pc = min(64 * (w + 4 * i) + lane, 64 * 17 - 1), row = pc / 17;
        wsrc[i] = (const char*)p.B + (int64_t)min(16 * cb + row, N - 1) * p.ldb + 16 * (pc - 17 * row);
    }
    const short* xsrc[CX];
#pragma unroll
    for (int j = 0; j < CX; ++j)
        xsrc[j] = (const short*)p.A + (int64_t)min(2 * (w + 4 * j) + (lane & 1), p.M - 1) * p.lda + 8 * ((lane >> 1) ^ ((w + 4 * j) & 7));
    const int rot = (int)((SLICED ? blockIdx.x : (unsigned)(cb >> 2)) % (unsigned)nseg);
    auto seg_of = [&](int t) { const int sg = t + rot; return seg0 + (sg >= nseg ? sg - nseg : sg); };
    auto issue_w = [&](int t) {
        char* st = w_lds[t % WST];
        const int off = seg_of(t) * kQ8SegBytes;
#pragma unroll
        for (int i = 0; i < CW; ++i) copy16_global_to_lds(wsrc[i] + off, st + 1024 * (w + 4 * i));
    };
    auto issue_x = [&](int t) {
        char* st = x_lds[t % XST];
        const int k0 = seg_of(t) * kStripeSeg;
#pragma unroll
        for (int j = 0; j < CX; ++j) copy16_global_to_lds(xsrc[j] + k0, st + (w + 4 * j) * kStripeBlock);
    };
    f32x4 acc[4][MB];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[c][mb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < WST - 1; ++t) {
        if (t < XST - 1 && t < nseg) issue_x(t);
        if (t < nseg) issue_w(t);
    }
    for (int t = 0; t < nseg; ++t) {
        __syncthreads();                                       // every wave has read segment t - 1: its stages may be refilled
        if (t + XST - 1 < nseg) issue_x(t + XST - 1);
        if (t + WST - 1 < nseg) issue_w(t + WST - 1);
        const int after = nseg - 1 - t;
        if (after >= 2) wait_vmcnt<(WST - 1) * CW + (XST - 1) * CX>(); else if (after == 1) wait_vmcnt<CW + CX>(); else wait_vmcnt<0>();
        __syncthreads();                                       // ... for every wave's copies
        const char* wb = w_lds[t % WST] + wfrag;
        const char* xb = x_lds[t % XST];
        uint32_t wq[2][4][3], dbits[2][4];
        s16x8 b[2][MB];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) b[s][mb] = *reinterpret_cast<const s16x8*>(xb + mb * 8 * kStripeBlock + frag[s]);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t* wp = reinterpret_cast<const uint32_t*>(wb + 16 * kQ8SegBytes * c + 32 * s);
                wq[s][c][0] = wp[0]; wq[s][c][1] = wp[1]; wq[s][c][2] = wp[2];
                dbits[s][c] = *reinterpret_cast<const uint16_t*>(wb + 16 * kQ8SegBytes * c + 34 * s - 8 * quad);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const _Float16 dh = __builtin_bit_cast(_Float16, (uint16_t)dbits[s][c]);
                const s16x8 a = dequant8_shifted(wq[s][c][0], wq[s][c][1], wq[s][c][2], s == 0 ? kQ8SelEven : kQ8SelOdd, h16x2{dh, dh});
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) acc[c][mb] = T::mfma16(a, b[s][mb], acc[c][mb]);
            }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // fragments in registers before the barrier that frees the stage
    }
    __syncthreads();
    f32x4* red = reinterpret_cast<f32x4*>(&w_lds[0][0]);   // 16 MB KiB of the 66
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) red[((w * 4 + c) * MB + mb) * 64 + lane] = acc[c][mb];
    __syncthreads();
    const int n = 16 * cb + 16 * w + 4 * quad;               // register r of a lane: weight row n + r, activation row 16mb + l16
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int m = 16 * mb + l16;
        if (m >= p.M || n >= N) continue;
        f32x4 sum = red[((0 * 4 + w) * MB + mb) * 64 + lane];
#pragma unroll
        for (int u = 1; u < 4; ++u) sum += red[((u * 4 + w) * MB + mb) * 64 + lane];
        if (SLICED) {
            *reinterpret_cast<f32x4*>(p.part + ((int64_t)slice * p.M + m) * p.N + n) = sum;
            continue;
        }
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = p.alpha * sum[e];
        if (p.beta != 0.f) {
            const s16x4 c = *reinterpret_cast<const s16x4*>((const short*)p.C + (int64_t)m * p.ldc + n);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += p.beta * T::to_float(c[e]);
        }
        uint2 pk;
        pk.x = T::pack2(v[0], v[1]);
        pk.y = T::pack2(v[2], v[3]);
        *reinterpret_cast<uint2*>((short*)p.D + (int64_t)m * p.ldd + n) = pk;
    }
    cb += nb;
    if (cb < blk_last) __syncthreads();
    }
}
// Which calls it takes: 2-64 rows, whole segments of 8 blocks, rows that start on 16-byte boundaries, and a weight wide
// enough for two and a half blocks per workgroup, or two from 16 rows, or one and a half above 32 (weights coming from memory:
// 14336 x 4096 at 2-16 rows 16.7-16.9 us against 20.8-26.8 for gemm_skinny_q8_kernel, 64 rows 23.4 against 50.9; 28672 x
// 4096 29.7-43.4 against 36.8-97.7; 8192 x 8192 at 2 rows 27.0 against 23.5, at 16 rows 27.4 against 28.4; 6144 x 4096 at
// 16 rows 15.7 against 15.2, at 64 rows 22.9 against 25.9).  A chunk of fewer than four blocks dequantises and multiplies
// all four all the same: skipping the missing ones by a branch cost the full chunks a third (16.7 -> 22.8 us).
// K slices of it for a weight of fewer than 192 stripes when a workspace is given (1 = none): 256 / stripes workgroups
// per chunk of four blocks, full chunks whatever the width (weights coming from memory: 4096 x 14336 at 16 / 32 / 64 rows
// 19.0 / 21.8 / 26.4 us against 29.6 / 43.0 / 68.4 for gemm_skinny_q8_kernel, 8192 x 8192 at 2-64 rows 19.6-28.5 against
// 23.7-40.3, 6144 x 4096 12.4-17.7 against 12.7-22.2; 4096 x 4096 up to 8 rows 10.2 against 7.7-8.3: two launches, so a
// weight of 16 M values or fewer only from 16 rows on, or from 8 when its rows are 6144 values and longer, or from 2
// when they are 8192 values and longer and the stripes 24 at most, as for the 16-bit weights).
static int q8_slices(int64_t M, int64_t N, int64_t K) {
    if (M < 2 || M > 64 || K % kStripeSeg != 0 || N % 8 != 0) return 1;
    const bool long_rows = (K >= 6144 && M >= 8) || (K >= 8192 && N <= 24 * 64);
    if (N * K <= (INT64_C(1) << 24) && M < 16 && !long_rows) return 1;
    return stripe_slices(M, N, K);
}
static bool q8_stripe_ok(int64_t M, int64_t N, int64_t K, const void* Bq, int64_t row_bytes) {
    return M >= 2 && M <= 64 && K % kStripeSeg == 0 && aligned16(Bq) && row_bytes % 16 == 0 &&
           (N >= 10240 || (N >= 8192 && M >= 16) || (N >= 6144 && M > 32));
}
template <bool SLICED = false>
static int launch_stripe_q8(const GemmParams& p0, hipStream_t stream) {
    GemmParams p = p0;
    p.tiles_n = (p.N + 15) / 16;
    const dim3 grid(SLICED ? (p.tiles_n + 3) / 4 * p.splits : std::min(p.tiles_n, 256)), block(4 * 64);
    if (p.M <= 16) hipLaunchKernelGGL((gemm_stripe_q8_kernel<1, SLICED>), grid, block, 0, stream, p);
    else if (p.M <= 32) hipLaunchKernelGGL((gemm_stripe_q8_kernel<2, SLICED>), grid, block, 0, stream, p);
    else if (p.M <= 48) hipLaunchKernelGGL((gemm_stripe_q8_kernel<3, SLICED>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((gemm_stripe_q8_kernel<4, SLICED>), grid, block, 0, stream, p);
    return check_launch("gemm_stripe_q8_kernel");
}

// Any shape and alignment: one thread per element of D, fp32 accumulation.  Small or odd problems only.
template <class T, bool NT>
__global__ __launch_bounds__(256) void gemm_plain_kernel(const GemmParams p) {
    const int64_t total = (int64_t)p.M * p.N;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int m = (int)(i / p.N), n = (int)(i % p.N);
        const short* a = (const short*)p.A + (int64_t)m * p.lda;
        const short* b = (const short*)p.B + (NT ? (int64_t)n * p.ldb : (int64_t)n);
        float s = 0.f;
        for (int k = 0; k < p.K; ++k) s += T::to_float(a[k]) * T::to_float(b[NT ? k : (int64_t)k * p.ldb]);
        float v = p.alpha * s;
        if (p.beta != 0.f) v += p.beta * T::to_float(((const short*)p.C)[(int64_t)m * p.ldc + n]);
        ((short*)p.D)[(int64_t)m * p.ldd + n] = (short)(T::pack2(v, 0.f) & 0xffffu);
    }
}

// D = alpha * (sum of the K slices' partial products) + beta * C, four columns per thread.
template <class T>
__global__ __launch_bounds__(256) void gemm_reduce_kernel(const GemmParams p) {
    const int n4 = p.N >> 2;
    const int64_t total = (int64_t)p.M * n4;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int m = (int)(i / n4), n = 4 * (int)(i % n4);
        f32x4 sum = *reinterpret_cast<const f32x4*>(p.part + (int64_t)m * p.N + n);
        for (int sl = 1; sl < p.splits; ++sl) sum += *reinterpret_cast<const f32x4*>(p.part + ((int64_t)sl * p.M + m) * p.N + n);
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = p.alpha * sum[e];
        if (p.beta != 0.f) {
            const s16x4 c = *reinterpret_cast<const s16x4*>((const short*)p.C + (int64_t)m * p.ldc + n);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += p.beta * T::to_float(c[e]);
        }
        uint2 pk;
        pk.x = T::pack2(v[0], v[1]);
        pk.y = T::pack2(v[2], v[3]);
        *reinterpret_cast<uint2*>((short*)p.D + (int64_t)m * p.ldd + n) = pk;
    }
}

static int launch_stripe_q8_slices(GemmParams& p, hipStream_t stream) {
    if (int rc = launch_stripe_q8<true>(p, stream)) return rc;
    const int grid = (int)std::min<int64_t>(((int64_t)p.M * (p.N / 4) + 255) / 256, 256 * 8);
    hipLaunchKernelGGL((gemm_reduce_kernel<F16>), dim3(grid), dim3(256), 0, stream, p);
    return check_launch("gemm_reduce_kernel");
}

// How many K slices a problem is cut into when a workspace is at hand: problems whose 128 x 128 tiles would leave most
// of the chip idle (a few dozen rows against a wide weight), every slice at least 4 steps of 64 long.  1 = no split.
// Up to 256 tiles: one workgroup of these tiles per compute unit leaves its matrix pipes waiting for every K step, two
// overlap (256 x 8192 x 8192, 128 tiles: 75 -> 52 us; 512 x 8192 x 28672, 256 tiles: 400 -> 317).
static int gemm_splits(int64_t M, int64_t N, int64_t K) {
    if (K % kBK != 0 || N % 8 != 0) return 1;
    const int64_t tiles = ((M + GemmSmall::BM - 1) / GemmSmall::BM) * ((N + GemmSmall::BN - 1) / GemmSmall::BN);
    const int64_t kt = K / kBK;
    if (tiles > 256 || kt < 8) return 1;
    int64_t s = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(256 / tiles, kt / 4), 32));
    // 64-127 tiles get two or three slices that way and fill the chip once; twice as many, while a slice stays 16 steps long,
    // keep two workgroups on a compute unit ([K,N] 4096 x 14336 at 1-16 rows: 27.5 -> 22 us; 128 rows 37 -> 32).  Tiles that
    // fill the chip by themselves (129-256) are cut in two only for long rows: the second launch and the partial sums cost
    // what the second workgroup per unit gains at K = 8192 and less (clocks settled, sliced / not: 512 x 8192 x 8192 89.0 /
    // 76.8 us, 1024 x 4096 x 4096 47.0 / 44.7, 256 x 14336 x 4096 47.5 / 44.9; 1024 x 4096 x 14336 134 / 146)
    if (tiles >= 64 && tiles * s <= 256 && kt / (2 * s) >= 16 && (s >= 2 || kt >= 192)) s *= 2;
    return (int)s;
}

template <class T>
static int launch_stripe_slices(GemmParams& p, hipStream_t stream) {
    if (int rc = launch_stripe<T, true>(p, (p.N + 15) / 16, stream)) return rc;
    const int grid = (int)std::min<int64_t>(((int64_t)p.M * (p.N / 4) + 255) / 256, 256 * 8);
    hipLaunchKernelGGL((gemm_reduce_kernel<T>), dim3(grid), dim3(256), 0, stream, p);
    return check_launch("gemm_reduce_kernel");
}

template <class T, bool NT>
static int launch_split(GemmParams& p, hipStream_t stream) {
    using SH = GemmSmall;
    p.tiles_m = (p.M + SH::BM - 1) / SH::BM;
    p.tiles_n = (p.N + SH::BN - 1) / SH::BN;
    p.per_xcd = 0;
    const int64_t wgs = (int64_t)p.tiles_m * p.tiles_n * p.splits;
    if (one_workgroup_per_unit(wgs)) hipLaunchKernelGGL((gemm_kernel<T, NT, GemmSmall3, false, true>), dim3((unsigned)wgs), dim3(SH::WAVES * 64), 0, stream, p);
    else hipLaunchKernelGGL((gemm_kernel<T, NT, SH, false, true>), dim3((unsigned)wgs), dim3(SH::WAVES * 64), 0, stream, p);
    if (int rc = check_launch("gemm_kernel (K slices)")) return rc;
    const int grid = (int)std::min<int64_t>(((int64_t)p.M * (p.N / 4) + 255) / 256, 256 * 8);
    hipLaunchKernelGGL((gemm_reduce_kernel<T>), dim3(grid), dim3(256), 0, stream, p);
    return check_launch("gemm_reduce_kernel");
}

template <class T, bool NT, class SH>
static int launch_tiled(GemmParams& p, hipStream_t stream) {
    p.tiles_m = (p.M + SH::BM - 1) / SH::BM;
    p.tiles_n = (p.N + SH::BN - 1) / SH::BN;
    p.per_xcd = (p.tiles_m * p.tiles_n + 7) / 8;
    hipLaunchKernelGGL((gemm_kernel<T, NT, SH>), dim3(p.per_xcd * 8), dim3(SH::WAVES * 64), 0, stream, p);
    return check_launch("gemm_kernel");
}

// Rounds of the chip a launch of `tiles` workgroups (one per compute unit at a time) costs: full rounds count 1; a last
// round that fills only part of the chip counts 0.55 + 0.45 x that part (its compute units run faster, the chip being
// less loaded: 4096 x 6144 x 4096 as 384 large tiles takes 1.76 rounds' time, 2048 x 6144 x 4096 as 192 takes 0.87).
static double rounds_cost(int64_t tiles) {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    int cus = cached[dev].load(std::memory_order_relaxed);
    if (cus == 0) {
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        cached[dev].store(cus, std::memory_order_relaxed);
    }
    const int64_t full = tiles / cus, rest = tiles % cus;
    return (double)full + (rest ? 0.55 + 0.45 * (double)rest / cus : 0.0);
}
// A 256 x 192 tile is 0.75 of a 256 x 256 one and runs 5 % below its rate per flop (8192 x 6144 x 4096: 366 against 347 us).
static bool wide_shape_pays(int64_t big_tiles, int64_t wide_tiles) {
    return 0.75 * 1.05 * rounds_cost(wide_tiles) < 0.97 * rounds_cost(big_tiles);
}

template <class T, bool NT>
static int launch_gemm(GemmParams& p, bool fast, hipStream_t stream) {
    if (fast) {
        // large tiles halve the LDS and L2 traffic per flop; they are worth it once they fill most of the chip
        const int64_t big_tiles = (int64_t)((p.M + GemmBig::BM - 1) / GemmBig::BM) * ((p.N + GemmBig::BN - 1) / GemmBig::BN);
        if constexpr (NT) {
            if (big_tiles >= 160 && p.N % GemmWide::BN == 0 &&
                wide_shape_pays(big_tiles, (int64_t)((p.M + GemmWide::BM - 1) / GemmWide::BM) * (p.N / GemmWide::BN)))
                return launch_tiled<T, NT, GemmWide>(p, stream);
        }
        if (big_tiles >= 160) return launch_tiled<T, NT, GemmBig>(p, stream);
        const int64_t small_tiles = (int64_t)((p.M + GemmSmall::BM - 1) / GemmSmall::BM) * ((p.N + GemmSmall::BN - 1) / GemmSmall::BN);
        return one_workgroup_per_unit(small_tiles) ? launch_tiled<T, NT, GemmSmall3>(p, stream) : launch_tiled<T, NT, GemmSmall>(p, stream);
    }
    const int grid = (int)std::min<int64_t>(((int64_t)p.M * p.N + 255) / 256, 256 * 16);
    hipLaunchKernelGGL((gemm_plain_kernel<T, NT>), dim3(grid), dim3(256), 0, stream, p);
    return check_launch("gemm_plain_kernel");
}

// Up to three weights [N_s, K] against one A in one launch (alpha = 1, no C): the tiled kernel over the concatenated
// column tiles of the weights, or, for a decode step's few rows, the few-row kernel over their column groups.
template <class T>
static int launch_grouped(GemmParams& p, int n_w, hipStream_t stream) {
    int64_t n_sum = 0;
    for (int s = 0; s < n_w; ++s) n_sum += p.grp.N[s];
    auto fill_ends = [&](int unit) {
        int acc = 0;
        for (int s = 0; s < kMaxGroup; ++s) {
            if (s < n_w) acc += (p.grp.N[s] + unit - 1) / unit;
            p.grp.end[s] = acc;
        }
        return acc;
    };
    if (p.M == 1 && p.K <= kGemvMaxKHalfs && (n_sum * p.K >= (INT64_C(1) << 25) || !rows_lds_takes(p.M, p.K)) && n_sum <= 0x7fffffffLL) {   // one row: whole weight rows per wave, numbered through (the rule of gemm_impl)
        int acc = 0;
        for (int s = 0; s < kMaxGroup; ++s) { if (s < n_w) acc += p.grp.N[s]; p.grp.end[s] = acc; }
        return launch_gemv<T, true>(p, (int)n_sum, stream);
    }
    // a batch of decode steps: the stripe kernel over the three weights from 5 rows on (4096 + 1024 + 1024 columns of 4096
    // values, weights coming from memory: 8 rows 12.3 us against 14.2 for the 16-column kernel, 16 rows 12.7 against 17.4,
    // 32 rows 15.6 against 21.5; up to 4 rows both take 12.1-12.6)
    {
        int64_t stripes = 0;
        for (int s = 0; s < n_w; ++s) stripes += (p.grp.N[s] + 63) / 64;
        if (p.M >= 5 && stripes <= 640 && stripe_takes(p.M, stripes, p.K)) {
            // every weight a run of workgroups in proportion to its 16-column blocks, 256 or nearly in all
            int64_t blocks = 0;
            for (int s = 0; s < n_w; ++s) blocks += (p.grp.N[s] + 15) / 16;
            const int64_t total = std::min<int64_t>(blocks, 256);
            int acc = 0;
            for (int s = 0; s < kMaxGroup; ++s) {
                if (s < n_w) {
                    const int64_t bs = (p.grp.N[s] + 15) / 16;
                    acc += (int)std::max<int64_t>(1, std::min<int64_t>(bs, total * bs / blocks));
                }
                p.grp.end[s] = acc;
            }
            return launch_stripe<T, false, true>(p, acc, stream);
        }
    }
    if (rows_lds_takes(p.M, p.K)) return launch_rows_lds<T, true>(p, fill_ends(16), stream);
    if (p.M <= 32 || (p.M <= 64 && n_sum * p.K <= (INT64_C(1) << 25))) {
        const int nr = (p.M > 16 && n_sum >= 160 * 32) ? 2 : 1;
        const int groups = fill_ends(16 * nr);
        const dim3 grid(groups), block(kSkinnyWaves * 64);
        const int mb = (p.M + 15) / 16;
#define MINFER_SKINNY(MB, NR) hipLaunchKernelGGL((gemm_skinny_kernel<T, MB, NR, true>), grid, block, 0, stream, p)
        if (nr == 1) { if (mb == 1) MINFER_SKINNY(1, 1); else if (mb == 2) MINFER_SKINNY(2, 1); else if (mb == 3) MINFER_SKINNY(3, 1); else MINFER_SKINNY(4, 1); }
        else { if (mb == 2) MINFER_SKINNY(2, 2); else if (mb == 3) MINFER_SKINNY(3, 2); else MINFER_SKINNY(4, 2); }
#undef MINFER_SKINNY
        return check_launch("gemm_skinny_kernel (grouped)");
    }
    int64_t big_tiles = 0;
    for (int s = 0; s < n_w; ++s) big_tiles += (int64_t)((p.M + GemmBig::BM - 1) / GemmBig::BM) * ((p.grp.N[s] + GemmBig::BN - 1) / GemmBig::BN);
    const bool big = big_tiles >= 160;
    // 256 x 192 tiles over the weights' columns numbered through, when that fills the chip's rounds better (the Llama-3-8B
    // QKV projection of 4096 tokens: 384 large tiles, one and a half rounds, or 512 of these, two rounds of 3/4 the work)
    bool concat = big && n_sum % GemmWide::BN == 0 && n_sum < (INT64_C(1) << 31);
    for (int s = 0; s < n_w; ++s) concat = concat && p.grp.N[s] % 64 == 0;
    if (concat) {
        const int64_t wide_tiles = (int64_t)((p.M + GemmWide::BM - 1) / GemmWide::BM) * (n_sum / GemmWide::BN);
        concat = wide_shape_pays(big_tiles, wide_tiles);
    }
    if (concat) {
        int acc = 0;
        for (int s = 0; s < kMaxGroup; ++s) { if (s < n_w) acc += p.grp.N[s]; p.grp.end[s] = acc; }
        p.N = (int)n_sum;
        p.tiles_m = (p.M + GemmWide::BM - 1) / GemmWide::BM;
        p.tiles_n = (int)(n_sum / GemmWide::BN);
        p.per_xcd = (p.tiles_m * p.tiles_n + 7) / 8;
        hipLaunchKernelGGL((gemm_kernel<T, true, GemmWide, true, false, true>), dim3(p.per_xcd * 8), dim3(GemmWide::WAVES * 64), 0, stream, p);
        return check_launch("gemm_kernel (grouped, columns numbered through)");
    }
    const int bm = big ? GemmBig::BM : GemmSmall::BM, bn = big ? GemmBig::BN : GemmSmall::BN;
    p.tiles_m = (p.M + bm - 1) / bm;
    p.tiles_n = fill_ends(bn);
    p.per_xcd = (p.tiles_m * p.tiles_n + 7) / 8;
    if (big) hipLaunchKernelGGL((gemm_kernel<T, true, GemmBig, true>), dim3(p.per_xcd * 8), dim3(GemmBig::WAVES * 64), 0, stream, p);
    else if (one_workgroup_per_unit((int64_t)p.per_xcd * 8)) hipLaunchKernelGGL((gemm_kernel<T, true, GemmSmall3, true>), dim3(p.per_xcd * 8), dim3(GemmSmall::WAVES * 64), 0, stream, p);
    else hipLaunchKernelGGL((gemm_kernel<T, true, GemmSmall, true>), dim3(p.per_xcd * 8), dim3(GemmSmall::WAVES * 64), 0, stream, p);
    return check_launch("gemm_kernel (grouped)");
}

}  // namespace minfer_attn

using namespace minfer_attn;

MINFER_ATTN_EXPORT int minfer_qkv(int dtype, const void* x, const void* wq, const void* wk, const void* wv,
                                  void* q_out, void* k_out, void* v_out, int64_t M, int64_t K,
                                  int64_t Nq, int64_t Nk, int64_t Nv, int64_t ldx, int64_t ldwq, int64_t ldwk, int64_t ldwv,
                                  int64_t ldq, int64_t ldk, int64_t ldv, void* stream_v) {
    clear_error();
    if (dtype != MINFER_ATTN_F16 && dtype != MINFER_ATTN_BF16)
        return fail(MINFER_ATTN_EINVAL, "qkv: dtype must be MINFER_ATTN_F16 or MINFER_ATTN_BF16");
    const int64_t Ns[3] = {Nq, Nk, Nv}, ldw[3] = {ldwq, ldwk, ldwv}, ldo[3] = {ldq, ldk, ldv};
    const void* W[3] = {wq, wk, wv};
    void* O[3] = {q_out, k_out, v_out};
    if (M < 0 || K < 0 || M > 0x7fffffffLL || K > 0x7fffffffLL) return fail(MINFER_ATTN_EINVAL, "qkv: bad M or K");
    if (!x || ldx < K) return fail(MINFER_ATTN_EINVAL, "qkv: x is null or its leading dimension is smaller than K");
    bool fast = K > 0 && K % kBK == 0 && ldx % 8 == 0 && aligned16(x) && (int64_t)GemmBig::BM * ldx < (1LL << 30);
    for (int s = 0; s < 3; ++s) {
        if (Ns[s] < 0 || Ns[s] > 0x7fffffffLL) return fail(MINFER_ATTN_EINVAL, "qkv: bad output width");
        if (!W[s] || !O[s]) return fail(MINFER_ATTN_EINVAL, "qkv: null pointer");
        if (ldw[s] < K || ldo[s] < Ns[s]) return fail(MINFER_ATTN_EINVAL, "qkv: a leading dimension is smaller than its row");
        fast = fast && Ns[s] % 8 == 0 && ldw[s] % 8 == 0 && ldo[s] % 4 == 0 && aligned16(W[s]) && ((uintptr_t)O[s] & 7u) == 0 &&
               (int64_t)std::max<int64_t>(GemmBig::BN, kBK) * ldw[s] < (1LL << 30);
    }
    if (M == 0) return MINFER_ATTN_OK;
    if (!fast || Nq == 0 || Nk == 0 || Nv == 0) {   // shapes the tiled kernels cannot take: three separate launches
        for (int s = 0; s < 3; ++s)
            if (int rc = minfer_gemm(dtype, MINFER_GEMM_B_NK, x, W[s], nullptr, O[s], M, Ns[s], K, ldx, ldw[s], Ns[s], ldo[s], 1.0, 0.0, stream_v))
                return rc;
        return MINFER_ATTN_OK;
    }
    GemmParams p{};
    p.A = x; p.M = (int)M; p.K = (int)K; p.lda = ldx; p.alpha = 1.f; p.beta = 0.f; p.C = nullptr;
    p.B = wq; p.D = q_out; p.N = (int)Nq; p.ldb = ldwq; p.ldd = ldq; p.ldc = ldq;
    for (int s = 0; s < 3; ++s) { p.grp.B[s] = W[s]; p.grp.D[s] = O[s]; p.grp.N[s] = (int)Ns[s]; p.grp.ldb[s] = ldw[s]; p.grp.ldd[s] = ldo[s]; }
    hipStream_t stream = (hipStream_t)stream_v;
    return dtype == MINFER_ATTN_F16 ? launch_grouped<F16>(p, 3, stream) : launch_grouped<BF16>(p, 3, stream);
}

static int gemm_impl(int dtype, int b_layout, const void* A, const void* B, const void* C, void* D,
                     int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t ldd,
                     double alpha, double beta, void* workspace, size_t workspace_bytes, void* stream_v) {
    clear_error();
    if (dtype != MINFER_ATTN_F16 && dtype != MINFER_ATTN_BF16)
        return fail(MINFER_ATTN_EINVAL, "gemm: dtype must be MINFER_ATTN_F16 or MINFER_ATTN_BF16");
    if (b_layout != MINFER_GEMM_B_KN && b_layout != MINFER_GEMM_B_NK)
        return fail(MINFER_ATTN_EINVAL, "gemm: b_layout must be MINFER_GEMM_B_KN or MINFER_GEMM_B_NK");
    if (M < 0 || N < 0 || K < 0 || M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL)
        return fail(MINFER_ATTN_EINVAL, "gemm: bad M, N or K");
    if (!A || !B || !D || (beta != 0.0 && !C)) return fail(MINFER_ATTN_EINVAL, "gemm: null pointer");
    const bool nt = b_layout == MINFER_GEMM_B_NK;
    if (lda < K || ldd < N || (beta != 0.0 && ldc < N) || ldb < (nt ? K : N))
        return fail(MINFER_ATTN_EINVAL, "gemm: a leading dimension is smaller than its row");
    if (M == 0 || N == 0) return MINFER_ATTN_OK;
    GemmParams p{};
    p.A = A; p.B = B; p.C = C; p.D = D; p.M = (int)M; p.N = (int)N; p.K = (int)K;
    p.lda = lda; p.ldb = ldb; p.ldc = ldc; p.ldd = ldd; p.alpha = (float)alpha; p.beta = (float)beta;
    // the tiled kernel moves 16-byte pieces and whole 64-wide K steps, and addresses a panel with 32-bit offsets
    const bool fast = K > 0 && K % kBK == 0 && N % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0 && ldc % 4 == 0 && ldd % 4 == 0 &&
                      aligned16(A) && aligned16(B) && ((uintptr_t)D & 7u) == 0 && ((uintptr_t)C & 7u) == 0 &&
                      (int64_t)GemmBig::BM * lda < (1LL << 30) && (int64_t)std::max<int64_t>(GemmBig::BN, kBK) * ldb < (1LL << 30);
    hipStream_t stream = (hipStream_t)stream_v;
    // A decode step's few tokens against an [N, K] weight: stream the weight once.  Which kernel does that best was
    // measured with the calls cycling over copies of the weight, 640 MiB in all: a weight of up to 256 MiB called again
    // and again is served by the chip's last-level cache, where the order of the kernels is a different one (14336 x
    // 4096 at one row: stripes 18.0 us against 19.5 for whole rows per wave from the cache, 24.2 against 21.9 from memory).
    const int splits = fast && workspace && aligned16(workspace) ? gemm_splits(M, N, K) : 1;
    const bool can_split = splits > 1 && workspace_bytes >= (size_t)splits * (size_t)M * (size_t)N * sizeof(float);
    const int64_t stripes = (N + 63) / 64;
    const bool rows_takes = rows_lds_takes(M, K);
    // one row: whole weight rows per wave (14336 x 4096: 21.9 us, the 16-column kernel 23.6, stripes 24.2; 28672 x 8192:
    // 75.8 / 91 / 97); a weight under 32 M values goes to the 16-column kernel when it takes it (4096 x 4096: 8.5 against 10.5)
    if (fast && nt && M == 1 && K <= kGemvMaxKHalfs && (N * K >= (INT64_C(1) << 25) || !rows_takes))
        return dtype == MINFER_ATTN_F16 ? launch_gemv<F16>(p, p.N, stream) : launch_gemv<BF16>(p, p.N, stream);
    // two to four rows against long rows of a wide weight go the same way, every weight piece multiplied with the same
    // piece of each activation row (28672 x 8192 at 2-4 rows: 78.6-82.6 us against 93-95 for the 16-column kernel, 10240 x
    // 8192 at 2-3 rows 33.2-34.6 against 36.3; 8192 x 8192 30.5-33.9 against 29.2-29.6, and rows of 4096 values gain nothing)
    if (fast && nt && M >= 2 && gemv_takes(M, K) && K >= 8192 && N >= 10240 && (M <= 3 || N >= 16384))
        return dtype == MINFER_ATTN_F16 ? launch_gemv<F16>(p, p.N, stream) : launch_gemv<BF16>(p, p.N, stream);
    // up to 8 rows against fewer than 96 stripes, and up to 4 against an output head: the 16-column kernel (4096 x 14336 at
    // 2-8 rows: 23.5-24.4 us against 32.5 for the stripes' blocks shared out; 128256 x 4096 at 2-4 rows 166-170 against
    // 176-178; 28672 x 4096 at 2-8 rows 42.2-44.5 against 41.5-41.7 and 14336 x 4096 24.3-25.8 against 22.8-23.0: those go on)
    const bool rows_first = rows_takes && ((M <= 8 && stripes < 96) || (M <= 4 && stripes > 640));
    const int slices = fast && nt && workspace && aligned16(workspace) ? stripe_slices(M, N, K) : 1;
    const bool sliceable = slices > 1 && workspace_bytes >= (size_t)slices * (size_t)M * (size_t)N * sizeof(float);
    // ... except long rows of a narrow weight when a workspace allows K slices: one wave per 16 columns walks a whole row
    // by itself (1024 x 14336 at 2-8 rows 16.5-20.8 us, in slices 13.1-14.1; 1536 x 8960 15.2-17.4 and 11.8-12.5; 2048 x
    // 8192 at 5-8 rows 12.5-13.4 and 12.5-12.6, at 2-4 rows and for rows of 6144 values no gain)
    const bool long_rows_few_stripes = K >= 8192 && ((M >= 5 && stripes <= 32) || (M >= 2 && stripes <= 24));
    if (fast && nt && rows_first && !(sliceable && long_rows_few_stripes))
        return dtype == MINFER_ATTN_F16 ? launch_rows_lds<F16>(p, (int)((N + 15) / 16), stream) : launch_rows_lds<BF16>(p, (int)((N + 15) / 16), stream);
    // with a workspace, K slices of the stripes: fewer than 96 stripes from 9 rows on (4096 x 14336 at 16 rows 24.5 us against
    // 29.1 for the 16-column kernel and 33 for the blocks shared out; 5120 x 5120 14.6 / 20.5 / 15.8), 96-191 stripes from 33
    // rows on (6144 x 4096 at 64 rows 18.6 against 20.2, 8192 x 8192 33.9 against 37.8; up to 32 rows the blocks shared out
    // are ahead: 6144 x 4096 at 16 rows 12.7 against 14.3).  Two launches, 10.5 us at least, where one launch over rows of
    // 4096 values takes 8-10 at 9-16 rows: up to 16 rows only for 25 M weight values or rows of 6144 values and more (2048 x
    // 8192 at 9-16 rows 12.7-13.0 against 13.9-16.5, 1024 x 14336 13.7-14.6 against 21.5-26.7; 4096 x 4096 12.0 against
    // 9.3-10.2), from 17 rows on for 8 M values where the other choice is gemm_skinny_kernel (2048 x 4096 at 24-64 rows
    // 10.9-13.0 against 13.9-16.7, 4096 x 2048 at 24 rows 10.8 against 12.3) and 16 M where it is the blocks shared out
    // (4096 x 2048 at 32 / 64 rows: 10.8 / 12.6 against 8.9 / 11.5).
    const bool slices_pay = stripes >= 96 ? M > 32 && N * K >= (INT64_C(1) << 24)
        : long_rows_few_stripes || (M >= 9 && (N * K >= INT64_C(25000000) || K >= 6144 || (M >= 17 && N * K >= (INT64_C(1) << (stripe_takes(M, stripes, K) ? 24 : 23)))));
    if (sliceable && slices_pay) {
        p.splits = slices; p.part = (float*)workspace;
        return dtype == MINFER_ATTN_F16 ? launch_stripe_slices<F16>(p, stream) : launch_stripe_slices<BF16>(p, stream);
    }
    if (fast && nt && stripe_takes(M, stripes, K))
        return dtype == MINFER_ATTN_F16 ? launch_stripe<F16>(p, (int)((N + 15) / 16), stream) : launch_stripe<BF16>(p, (int)((N + 15) / 16), stream);
    if (fast && nt && rows_takes)
        return dtype == MINFER_ATTN_F16 ? launch_rows_lds<F16>(p, (int)((N + 15) / 16), stream) : launch_rows_lds<BF16>(p, (int)((N + 15) / 16), stream);
    if (fast && nt && M == 1 && K <= kGemvMaxKHalfs)
        return dtype == MINFER_ATTN_F16 ? launch_gemv<F16>(p, p.N, stream) : launch_gemv<BF16>(p, p.N, stream);
    if (fast && nt && (M <= 16 || (!can_split && (M <= 32 || (M <= 64 && N * K <= (INT64_C(1) << 25))))))
        return dtype == MINFER_ATTN_F16 ? launch_skinny<F16>(p, stream) : launch_skinny<BF16>(p, stream);
    if (can_split) {
        p.splits = splits; p.part = (float*)workspace;
        if (dtype == MINFER_ATTN_F16) return nt ? launch_split<F16, true>(p, stream) : launch_split<F16, false>(p, stream);
        return nt ? launch_split<BF16, true>(p, stream) : launch_split<BF16, false>(p, stream);
    }
    if (dtype == MINFER_ATTN_F16) return nt ? launch_gemm<F16, true>(p, fast, stream) : launch_gemm<F16, false>(p, fast, stream);
    return nt ? launch_gemm<BF16, true>(p, fast, stream) : launch_gemm<BF16, false>(p, fast, stream);
}

MINFER_ATTN_EXPORT int minfer_gemm(int dtype, int b_layout, const void* A, const void* B, const void* C, void* D,
                                   int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t ldd,
                                   double alpha, double beta, void* stream_v) {
    return gemm_impl(dtype, b_layout, A, B, C, D, M, N, K, lda, ldb, ldc, ldd, alpha, beta, nullptr, 0, stream_v);
}

MINFER_ATTN_EXPORT size_t minfer_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0 || M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL) return 0;
    const int splits = std::max(gemm_splits(M, N, K), stripe_slices(M, N, K));
    return splits > 1 ? (size_t)splits * (size_t)M * (size_t)N * sizeof(float) : 0;
}

MINFER_ATTN_EXPORT int minfer_gemm_ws(int dtype, int b_layout, const void* A, const void* B, const void* C, void* D,
                                      int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t ldd,
                                      double alpha, double beta, void* workspace, size_t workspace_bytes, void* stream_v) {
    return gemm_impl(dtype, b_layout, A, B, C, D, M, N, K, lda, ldb, ldc, ldd, alpha, beta, workspace, workspace_bytes, stream_v);
}

// ---- weights stored as Q8_0 blocks ------------------------------------------------------------------------------
constexpr int64_t kQ8SkinnyRows = 64;    // up to here the kernel that streams the blocks; above, dequantise once and run the tiles

static size_t q8_dequant_bytes(int64_t N, int64_t K) { return ((size_t)N * (size_t)K * 2 + 255) & ~(size_t)255; }

// the streaming kernel takes up to 64 rows, needs weight rows that are multiples of 4 bytes (an even number of blocks)
// and stores 8-byte pieces of D (N a multiple of 4); every other shape goes through the dequantised weight
static bool q8_streams(int64_t M, int64_t N, int64_t K) { return M <= kQ8SkinnyRows && (K / 32) % 2 == 0 && N % 4 == 0; }
// ... and it reads 16-byte pieces of A and aligned 8-byte pieces of C (only when beta != 0) and D
static bool q8_stream_operands(const void* A, const void* C, const void* D, int64_t lda, int64_t ldc, int64_t ldd, double beta) {
    return aligned16(A) && lda % 8 == 0 && ldd % 4 == 0 && ((uintptr_t)D & 7u) == 0 &&
           (beta == 0.0 || (ldc % 4 == 0 && ((uintptr_t)C & 7u) == 0));
}

MINFER_ATTN_EXPORT size_t minfer_gemm_q8_0_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0 || K % 32 != 0 || M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL) return 0;
    if (q8_streams(M, N, K)) {   // optional: K slices of the stripe kernel for a narrow weight
        const int slices = q8_slices(M, N, K);
        return slices > 1 ? (size_t)slices * (size_t)M * (size_t)N * sizeof(float) : 0;
    }
    return q8_dequant_bytes(N, K) + minfer_gemm_workspace_bytes(M, N, K);
}

MINFER_ATTN_EXPORT int minfer_gemm_q8_0(const void* A, const void* Bq, const void* C, void* D, int64_t M, int64_t N, int64_t K,
                                        int64_t lda, int64_t ldc, int64_t ldd, double alpha, double beta,
                                        void* workspace, size_t workspace_bytes, void* stream_v) {
    clear_error();
    if (M < 0 || N < 0 || K < 0 || M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL)
        return fail(MINFER_ATTN_EINVAL, "gemm_q8_0: bad M, N or K");
    if (K % 32 != 0) return fail(MINFER_ATTN_EINVAL, "gemm_q8_0: K must be a multiple of the block size 32");
    if (!A || !Bq || !D || (beta != 0.0 && !C)) return fail(MINFER_ATTN_EINVAL, "gemm_q8_0: null pointer");
    if (lda < K || ldd < N || (beta != 0.0 && ldc < N)) return fail(MINFER_ATTN_EINVAL, "gemm_q8_0: a leading dimension is smaller than its row");
    if (M == 0 || N == 0) return MINFER_ATTN_OK;
    if (K == 0) return fail(MINFER_ATTN_EINVAL, "gemm_q8_0: K must be positive");
    hipStream_t stream = (hipStream_t)stream_v;
    const int64_t row_bytes = K / 32 * 34;
    if (((uintptr_t)Bq & 3u) != 0) return fail(MINFER_ATTN_EINVAL, "gemm_q8_0: the weight must be 4-byte aligned");
    if (q8_streams(M, N, K) && q8_stream_operands(A, C, D, lda, ldc, ldd, beta)) {
        GemmParams p{};
        p.A = A; p.B = Bq; p.C = beta != 0.0 ? C : nullptr; p.D = D; p.M = (int)M; p.N = (int)N; p.K = (int)K;
        p.lda = lda; p.ldb = row_bytes; p.ldc = ldc; p.ldd = ldd; p.alpha = (float)alpha; p.beta = (float)beta;
        if (q8_gemv_ok(M, K, Bq, row_bytes)) return launch_gemv_q8(p, stream);
        const int slices = aligned16(Bq) && row_bytes % 16 == 0 ? q8_slices(M, N, K) : 1;
        if (slices > 1 && workspace && aligned16(workspace) && workspace_bytes >= (size_t)slices * (size_t)M * (size_t)N * sizeof(float)) {
            p.splits = slices; p.part = (float*)workspace;
            return launch_stripe_q8_slices(p, stream);
        }
        if (q8_stripe_ok(M, N, K, Bq, row_bytes)) return launch_stripe_q8(p, stream);
        return launch_skinny_q8(p, stream);
    }
    // otherwise: the weight as fp16 in the workspace, then the fp16 kernels on it
    const size_t deq = q8_dequant_bytes(N, K);
    if (!workspace || !aligned16(workspace) || workspace_bytes < deq)
        return fail(MINFER_ATTN_EWORKSPACE, "gemm_q8_0: this call needs a workspace of N*K*2 bytes (rounded up to 256) for the dequantised weight "
                                            "(more than 64 rows, an odd number of blocks per row, N not a multiple of 4, or A/C/D not aligned for the streaming kernel: "
                                            "A 16 bytes with lda a multiple of 8, C and D 8 bytes with strides multiples of 4)");
    if (int rc = minfer_dequant_q8_0(MINFER_ATTN_F16, Bq, workspace, N, K, stream_v)) return rc;
    return gemm_impl(MINFER_ATTN_F16, MINFER_GEMM_B_NK, A, workspace, C, D, M, N, K, lda, K, ldc, ldd, alpha, beta,
                     (char*)workspace + deq, workspace_bytes - deq, stream_v);
}
