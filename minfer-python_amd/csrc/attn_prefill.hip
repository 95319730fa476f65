// Prefill attention for gfx950: single-pass online-softmax kernel over 64-key tiles.
//
// Work decomposition.  One workgroup = 8 waves (two per SIMD, so one wave's softmax overlaps the
// other's MFMAs) = one KV head x (HPW query heads of that KV head's GQA group) x (QBW consecutive
// 32-row query blocks), HPW*QBW = 8, so the K/V tiles a workgroup stages in LDS are shared by
// every query head of the group.  Each wave owns 32 query rows of one head (two blocks of 16) and keeps
// its Q fragments, the 64x32 score tile and the Dx32 output accumulator in registers.
//
// Per 64-key tile a wave computes S^T = K Q^T with v_mfma_f32_16x16x32 (K from LDS as the MFMA A operand,
// Q as B), so that a lane holds four keys of each of its two query rows per 16x16 block: a row maximum /
// row sum needs two lane swaps (lanes l ^ 16, l ^ 32).  The exponentiated scores of two key blocks are,
// without any data movement, the B operand of a 32-key chunk of O^T += V^T P^T; V^T fragments come from
// LDS transpose reads.  K and V tiles are copied global->LDS directly (no VGPR staging) and
// double-buffered: the copy of tile t+1 is issued right after the barrier that opens tile t.  The K
// fragments of a tile pass through a ring of two register buffers, refilled two chunks ahead.
//
// Query rows in, output rows out.  Every wave has a private 8 KiB LDS area.  Its 32 query rows
// are copied there global->LDS as whole rows (full 128/256-byte lines per request) and read back
// as MFMA fragments; at the end the normalised output goes through the same area so that the
// wave stores whole rows as well.  Read straight into fragment layout, a load or store
// instruction would touch 32 different rows with 16 bytes each.  The area is the wave's own:
// no barrier is involved.
//
// Masking.  The reference operator takes an arbitrary dense bool mask [B,1,L,L]
// (reference: src/minfer/kernels/torch_ext/csrc/cuda/flash_attn/op.cuh:28).  A pre-pass
// classifies every 64x64 mask tile as none / all / mixed; the main kernel skips "none" tiles,
// runs "all" tiles unmasked and reads mask bytes only for "mixed" tiles, which keeps arbitrary
// masks bit-exact while a causal mask costs one byte-read tile per row of tiles.
#include <type_traits>

#include "attn_common.h"
#include "attn_host.h"

namespace minfer_attn {

enum : uint32_t { TILE_NONE = 0, TILE_ALL = 1, TILE_MIXED = 2 };
constexpr int kMaxKeyTiles = 2048;  // active-tile list capacity (L <= 131072)

// ------------------------------------------------------------------------------------------
// Mask classification: cls[b][qt][kt] for 64x64 tiles.  grid (ceil(NKT/16), NQT, B), 256 threads.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void classify_mask_kernel(const uint8_t* __restrict__ mask,
                                                            uint8_t* __restrict__ cls, int L, int NQT,
                                                            int NKT, int vec) {
    __shared__ uint32_t any_s[16], all_s[16];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int strip = blockIdx.x, qt = blockIdx.y, b = blockIdx.z;
    if (tid < 16) { any_s[tid] = 0u; all_s[tid] = 0x01010101u; }
    __syncthreads();
    const uint8_t* mb = mask + (size_t)b * L * L;
    const int col0 = strip * 1024 + lane * 16;  // this lane's 16 key columns
    uint32_t any_acc = 0u, all_acc = 0x01010101u;
    if (vec) {
        if (col0 < L) {
            // all 16 row segments of this lane are requested before any is used (rows past the end
            // re-read the last row, which changes neither the OR nor the AND)
            uint4 x[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int row = min(qt * 64 + w + 4 * i, L - 1);
                x[i] = *reinterpret_cast<const uint4*>(mb + (size_t)row * L + col0);
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                any_acc |= x[i].x | x[i].y | x[i].z | x[i].w;
                all_acc &= x[i].x & x[i].y & x[i].z & x[i].w;
            }
        }
    } else {
        for (int r = w; r < 64; r += 4) {
            const int row = qt * 64 + r;
            if (row >= L) break;
            for (int e = 0; e < 16; ++e) {
                const int col = col0 + e;
                if (col < L) {
                    const uint32_t x = mb[(size_t)row * L + col] ? 1u : 0u;
                    any_acc |= x;
                    all_acc &= x * 0x01010101u;
                }
            }
        }
    }
    // lanes 4t..4t+3 of each wave cover key tile (strip*16 + t)
    any_acc |= __shfl_xor(any_acc, 1); any_acc |= __shfl_xor(any_acc, 2);
    all_acc &= __shfl_xor(all_acc, 1); all_acc &= __shfl_xor(all_acc, 2);
    if ((lane & 3) == 0) {
        atomicOr(&any_s[lane >> 2], any_acc);
        atomicAnd(&all_s[lane >> 2], all_acc);
    }
    __syncthreads();
    if (tid < 16) {
        const int kt = strip * 16 + tid;
        if (kt < NKT) {
            const uint32_t c = any_s[tid] == 0u ? TILE_NONE : (all_s[tid] == 0x01010101u ? TILE_ALL : TILE_MIXED);
            cls[((size_t)b * NQT + qt) * NKT + kt] = (uint8_t)c;
        }
    }
}

// The same for masks whose rows can be read in aligned 16-byte pieces, 64 rows x 256 columns (4 key tiles) per workgroup:
// a lane takes 16 bytes of one row, the workgroup 16 rows per pass, 4 passes, all requested before any is used.  Four times
// the workgroups of the general kernel and a quarter of the loads per lane: the pass is latency-bound, not byte-bound
// (16 MiB at S=4096: 4.4 us instead of 5.1).  grid (ceil(NKT/4), NQT, B).
__global__ __launch_bounds__(256) void classify_mask_kernel_256(const uint8_t* __restrict__ mask, uint8_t* __restrict__ cls,
                                                                int L, int NQT, int NKT) {
    __shared__ uint32_t any_s[4][4], all_s[4][4];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int strip = blockIdx.x, qt = blockIdx.y, b = blockIdx.z;
    const uint8_t* mb = mask + (size_t)b * L * L;
    const int col0 = strip * 256 + (tid & 15) * 16;     // this lane's 16 key columns
    const int r0 = tid >> 4;                            // row inside a pass of 16 rows
    uint32_t any_acc = 0u, all_acc = 0x01010101u;
    if (col0 < L) {
        uint4 x[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = min(qt * 64 + 16 * i + r0, L - 1);
            x[i] = *reinterpret_cast<const uint4*>(mb + (size_t)row * L + col0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            any_acc |= x[i].x | x[i].y | x[i].z | x[i].w;
            all_acc &= x[i].x & x[i].y & x[i].z & x[i].w;
        }
    }
    // lanes 4t..4t+3 (mod 16) cover key tile t of the strip; rows differ across lane / 16 and across waves
    any_acc |= __shfl_xor(any_acc, 1); any_acc |= __shfl_xor(any_acc, 2);
    all_acc &= __shfl_xor(all_acc, 1); all_acc &= __shfl_xor(all_acc, 2);
    any_acc |= __shfl_xor(any_acc, 16); any_acc |= __shfl_xor(any_acc, 32);
    all_acc &= __shfl_xor(all_acc, 16); all_acc &= __shfl_xor(all_acc, 32);
    if (lane < 16 && (lane & 3) == 0) { any_s[w][lane >> 2] = any_acc; all_s[w][lane >> 2] = all_acc; }
    __syncthreads();
    if (tid < 4) {
        const int kt = strip * 4 + tid;
        if (kt < NKT) {
            const uint32_t a = any_s[0][tid] | any_s[1][tid] | any_s[2][tid] | any_s[3][tid];
            const uint32_t l = all_s[0][tid] & all_s[1][tid] & all_s[2][tid] & all_s[3][tid];
            cls[((size_t)b * NQT + qt) * NKT + kt] = (uint8_t)(a == 0u ? TILE_NONE : (l == 0x01010101u ? TILE_ALL : TILE_MIXED));
        }
    }
}

// ------------------------------------------------------------------------------------------
// Main kernel
// ------------------------------------------------------------------------------------------
struct PrefillParams {
    const void* q; const void* k; const void* v; void* out;
    const uint8_t* mask;   // dense mode: [B,1,L,L]
    const uint8_t* cls;    // dense mode: [B,NQT,NKT]
    const int32_t* cu;     // varlen mode: [n_seqs+1]
    int64_t q0, q1, q2, kv0, kv1, kv2, o0, o1, o2;
    int L;                 // dense: sequence length; varlen: total packed tokens
    int B, Hq, Hkv, n_rep;
    int hpw_log2;          // query heads per workgroup = 1 << hpw_log2 (<= 8)
    int n_hg;              // head groups per KV head = n_rep >> hpw_log2
    int NQT, NKT;          // dense: 64-row query / key tile counts of the mask classification
    int NQ;                // workgroup-level query tiles (dense: exact; varlen: upper bound)
    int n_seqs;
    int max_len;           // varlen: rows of a sequence past this many are not computed (>= every length for a valid call)
    int mask_vec;          // dense: mask rows may be read as aligned 32-bit words
    float scale_log2;      // softmax scale * log2(e)
};

// MODE_DENSE: dense bool mask, tile classes from the pre-pass.  MODE_VARLEN: packed sequences, causal by index.
// MODE_DENSE_SELF: dense bool mask of a short problem (L <= 1024, rows readable in 16-byte pieces): every workgroup
// classifies its own rows of the mask in its prologue, one wave-wide load per row, and no pre-pass is launched.
enum { MODE_DENSE = 0, MODE_VARLEN = 1, MODE_DENSE_SELF = 2 };
constexpr int kSelfClassifyMaxGrid = 512;
constexpr int kSelfClassifyMaxL = 1024;   // 16 key tiles: lane l of a wave-wide load holds columns 16l .. 16l+15 of one row
// Waves per workgroup, a template argument of the kernel: 8 (one workgroup per compute unit: 256 query rows share every
// K/V tile staged in LDS) or 4 (two workgroups per compute unit, 128 rows per tile: twice the tile copies per flop, but
// one workgroup's prologue, epilogue and hand-over run under the other's tiles, which is what counts when sequences
// are short).
constexpr int kWavesBig = 8, kWavesSmall = 4;

template <int D, int NW> struct TileGeom {
    static constexpr int RB = D * 2;          // bytes per K/V row
    static constexpr int G = RB / 16;         // 16-byte granules per row
    static constexpr int RPI = 1024 / RB;     // rows one wave-wide copy instruction covers
    static constexpr int NLD = 64 / (NW * RPI);  // copy instructions per wave, per tile, per tensor
    static constexpr int RPW = 256 / RB;      // rows per 256-byte bank window
    static constexpr int TILE_BYTES = 64 * RB;
    // XOR swizzles applied to the granule index of a row.  K is read 16 rows x one granule at a
    // time (ds_read_b128), V 4 rows x 32 bytes by each 16-lane group, the groups on consecutive
    // 4-row blocks (transpose reads); both become conflict-free.
    static MA_DEV int swz_k(int row) { return (row / RPW) & (G - 1); }
    static MA_DEV int swz_v(int row) { return D == 128 ? ((row & 7) << 1) : (((row >> 1) & 3) << 1); }
};

template <class T, int D, int MODE, int NW>
__global__ __launch_bounds__(NW * 64, 2) void prefill_kernel(const PrefillParams p) {
    using GEO = TileGeom<D, NW>;
    constexpr int RB = GEO::RB, G = GEO::G, RPI = GEO::RPI, NLD = GEO::NLD;
    constexpr int KC = D / 32;   // 32-wide contraction chunks of Q K^T
    constexpr int DB = D / 16;   // 16-row blocks of O^T
    constexpr int kWaves = NW;
    constexpr int STAGE_BYTES = 2 * GEO::TILE_BYTES;   // a stage = the K tile followed by the V tile
    constexpr int ROWS_BYTES = 32 * RB;                // a wave's 32 query (or output) rows

    __shared__ __attribute__((aligned(1024))) char kv_lds[2][STAGE_BYTES];
    constexpr bool kDense = MODE != MODE_VARLEN;
    __shared__ uint32_t tile_list[MODE == MODE_DENSE ? kMaxKeyTiles : (MODE == MODE_DENSE_SELF ? kSelfClassifyMaxL / 64 : 1)];
    __shared__ int n_active_s;
    // A wave's own 32 query rows on their way in (whole rows, copied global->LDS) and its 32 output rows on their way
    // out (so that a store instruction writes whole rows).  With 8 waves the area is separate memory, the wave's own, so
    // neither step needs a barrier.  With 4 waves (4 x ROWS_BYTES = one stage) it lies inside the K/V stages, which is
    // what lets two workgroups fit a compute unit: the query rows in stage 1, which no tile copy touches before the
    // barrier that opens tile 0 (by then every wave has its fragments in registers); the output rows in the stage the
    // last tile did not use, which every wave finished reading before the barrier that opened the last tile.
    constexpr bool kAliasRows = NW * ROWS_BYTES <= STAGE_BYTES;
    __shared__ __attribute__((aligned(1024))) char q_lds_own[kAliasRows ? 1 : NW][kAliasRows ? 16 : ROWS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63, w = wave_id();
    const int l16 = lane & 15, quad = lane >> 4;
    const int HPW = 1 << p.hpw_log2, QBW = kWaves >> p.hpw_log2;  // heads, 32-row query blocks per workgroup
    char* const q_stage = kAliasRows ? &kv_lds[1][w * ROWS_BYTES] : &q_lds_own[kAliasRows ? 0 : w][0];

    // ---- which (batch, KV head, head group, query tile) is this workgroup -------------------
    const int BG = p.B * p.Hkv;
    const int NG = BG * p.n_hg;
    int pidx, rank;
    {
        const int n = blockIdx.x;
        if ((NG & 7) == 0) {  // keep all workgroups of one (batch, KV head) on one XCD (ids go round-robin)
            const int per = NG >> 3, mm = n >> 3;
            pidx = (mm % per) * 8 + (n & 7);
            rank = mm / per;
        } else {
            pidx = n % NG;
            rank = n / NG;
        }
    }
    const int bg = pidx % BG, hg = pidx / BG;
    const int g = bg % p.Hkv, b = bg / p.Hkv;

    int seq_lo = 0, seq_len = p.L;  // token rows of the attended sequence
    int qtile;                      // workgroup-level query tile (32*QBW rows) inside the sequence
    if (kDense) {
        qtile = p.NQ - 1 - rank;    // longest rows of a causal mask first
    } else {
        // the sequence that holds query tile `rank` of the packed batch: 64 sequences per step, a prefix sum of their
        // tile counts over the lanes (one sequence per step cost a workgroup ~40 ns per sequence before its tile)
        int x = rank, nt = 0;
        bool found = false;
        for (int base = 0; base < p.n_seqs && !found; base += 64) {
            const int sq = base + lane;
            // cu_seqlens is device data nobody has checked: every sequence is cut to the part of it that lies
            // inside the packed tensors ([0, L) rows) and to max_seqlen rows, and an end before its start is an
            // empty sequence, so no entry can produce an address outside q/k/v/out or a negative tile count.
            int lo = 0, len = 0;
            if (sq < p.n_seqs) {
                lo = min(max(p.cu[sq], 0), p.L);
                len = min(min(max(p.cu[sq + 1], lo), p.L) - lo, p.max_len);
            }
            const int n = (len + 32 * QBW - 1) / (32 * QBW);
            const int incl = wave_inclusive_scan(n, lane);
            const int total = __builtin_amdgcn_readfirstlane(__shfl(incl, 63));
            if (x < total) {
                const int src = __ffsll((unsigned long long)__ballot(x < incl)) - 1;
                seq_lo = __builtin_amdgcn_readfirstlane(__shfl(lo, src));
                seq_len = __builtin_amdgcn_readfirstlane(__shfl(len, src));
                nt = __builtin_amdgcn_readfirstlane(__shfl(n, src));
                x -= __builtin_amdgcn_readfirstlane(__shfl(incl - n, src));
                found = true;
            } else {
                x -= total;
            }
        }
        if (!found) return;
        qtile = nt - 1 - x;
    }

    const int head = g * p.n_rep + hg * HPW + (w & (HPW - 1));
    const int qblk = qtile * QBW + (w >> p.hpw_log2);           // 32-row block index inside the sequence
    const int q_row0 = qblk * 32;                                // first query row (sequence-local)
    const bool wave_on = q_row0 < seq_len;
    const int last_row = seq_len - 1;
    const int qrow[2] = {q_row0 + l16, q_row0 + 16 + l16};       // this lane's two query rows (one per 16-row block)

    const short* Qh = (const short*)p.q + (kDense ? (int64_t)b * p.q0 : 0) + (int64_t)head * p.q1 + (int64_t)seq_lo * p.q2;
    const short* Kh = (const short*)p.k + (kDense ? (int64_t)b * p.kv0 : 0) + (int64_t)g * p.kv1 + (int64_t)seq_lo * p.kv2;
    const short* Vh = (const short*)p.v + (kDense ? (int64_t)b * p.kv0 : 0) + (int64_t)g * p.kv1 + (int64_t)seq_lo * p.kv2;
    short* Oh = (short*)p.out + (kDense ? (int64_t)b * p.o0 : 0) + (int64_t)head * p.o1 + (int64_t)seq_lo * p.o2;
    const uint8_t* mrow[2] = {kDense ? p.mask + ((size_t)b * p.L + min(qrow[0], last_row)) * p.L : nullptr,
                              kDense ? p.mask + ((size_t)b * p.L + min(qrow[1], last_row)) * p.L : nullptr};

    // The wave's Q rows are requested now and used after the tile list is built, so that the two latencies overlap.
    // They are copied global->LDS as whole rows (RPI rows per instruction, with the K tile's swizzle) and read back as
    // fragments: fetched straight into fragment registers every instruction would touch 32 rows for 32 bytes each.
    // A block that lies wholly inside its sequence (all but a sequence's last one) takes the short way: a wave-uniform
    // base per instruction plus one 32-bit lane offset (swz_k of the instruction's first row and of the lane's row
    // within it occupy different bits, so the instruction's share of the swizzle is a constant).  Otherwise rows past
    // the end of the sequence re-read its last row.
    if (q_row0 + 32 <= seq_len) {
        const int row_in = lane / G, pg = lane % G;
        const uint32_t lane_row = (uint32_t)((int64_t)row_in * p.q2) * 2u;
        const int g0 = pg ^ GEO::swz_k(row_in);
        const short* qbase = Qh + (int64_t)q_row0 * p.q2;
#pragma unroll
        for (int j = 0; j < 32 / RPI; ++j)
            copy16_global_to_lds<true>(qbase + (int64_t)(j * RPI) * p.q2, lane_row + 16u * (uint32_t)(g0 ^ GEO::swz_k(j * RPI)), q_stage + j * RPI * RB);
    } else {
#pragma unroll
        for (int j = 0; j < 32 / RPI; ++j) {
            const int row = j * RPI + lane / G, pg = lane % G;
            const short* src = Qh + (int64_t)min(q_row0 + row, last_row) * p.q2 + 8 * (pg ^ GEO::swz_k(row));
            copy16_global_to_lds(src, q_stage + j * RPI * RB);
        }
    }

    // ---- list of key tiles this workgroup visits ---------------------------------------------
    // entry = key tile | (2-bit class for each 64-row query tile the workgroup overlaps) << 16
    const int qt64_first = (qtile * QBW * 32) >> 6;
    const int n_qt64 = QBW >= 2 ? QBW / 2 : 1;
    // (a workgroup that classifies its own rows does so per 32-row query block: slot = the wave's block)
    const int my_qt64_slot = MODE == MODE_DENSE_SELF ? (w >> p.hpw_log2) : (q_row0 >> 6) - qt64_first;
    int n_active;
    if (MODE == MODE_DENSE_SELF) {
        // Every wave reads 32/HPW rows of its own query block (the HPW waves of a block share its rows), 8 rows in flight:
        // lane l holds the 16 mask bytes of key columns 16l .. 16l+15, so lanes 4t .. 4t+3 cover key tile t.  Rows past the
        // end re-read the last row, which changes neither the OR nor the AND.
        __shared__ uint32_t any_s[NW][kSelfClassifyMaxL / 64], all_s[NW][kSelfClassifyMaxL / 64];
        const int rpw = 32 >> p.hpw_log2;
        const int row_first = q_row0 + (w & (HPW - 1)) * rpw;
        uint32_t any_acc = 0u, all_acc = 0x01010101u;
        if (16 * lane < p.L) {
            const uint8_t* mb = p.mask + (size_t)b * p.L * p.L + 16 * lane;
            for (int r0 = 0; r0 < rpw; r0 += 8) {
                uint4 x[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) x[i] = *reinterpret_cast<const uint4*>(mb + (size_t)min(row_first + r0 + i, last_row) * p.L);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    any_acc |= x[i].x | x[i].y | x[i].z | x[i].w;
                    all_acc &= x[i].x & x[i].y & x[i].z & x[i].w;
                }
            }
        }
        any_acc |= __shfl_xor(any_acc, 1); any_acc |= __shfl_xor(any_acc, 2);
        all_acc &= __shfl_xor(all_acc, 1); all_acc &= __shfl_xor(all_acc, 2);
        if ((lane & 3) == 0) { any_s[w][lane >> 2] = any_acc; all_s[w][lane >> 2] = all_acc; }
        __syncthreads();
        if (w == 0) {
            const int kt = lane;
            uint32_t c = 0;
            if (kt < p.NKT) {
                for (int sb = 0; sb < QBW; ++sb) {
                    uint32_t a = 0u, l = 0x01010101u;
                    for (int ww = sb * HPW; ww < (sb + 1) * HPW; ++ww) { a |= any_s[ww][kt]; l &= all_s[ww][kt]; }
                    c |= (a == 0u ? TILE_NONE : (l == 0x01010101u ? TILE_ALL : TILE_MIXED)) << (2 * sb);
                }
            }
            const uint64_t bal = __ballot(c != 0);
            if (c) tile_list[__popcll(bal & ((1ull << lane) - 1ull))] = (uint32_t)kt | (c << 16);
            if (lane == 0) n_active_s = __popcll(bal);
        }
        __syncthreads();
        n_active = n_active_s;
    } else if (MODE == MODE_DENSE) {
        if (w == 0) {
            int cnt = 0;
            for (int base = 0; base < p.NKT; base += 64) {
                const int kt = base + lane;
                uint32_t c = 0;
                if (kt < p.NKT) {
                    for (int s = 0; s < n_qt64; ++s) {
                        const int qs = qt64_first + s;
                        if (qs < p.NQT) c |= (uint32_t)p.cls[((size_t)b * p.NQT + qs) * p.NKT + kt] << (2 * s);
                    }
                }
                const uint64_t bal = __ballot(c != 0);
                const int pos = cnt + __popcll(bal & ((1ull << lane) - 1ull));
                if (c) tile_list[pos] = (uint32_t)kt | (c << 16);
                cnt += __popcll(bal);
            }
            if (lane == 0) n_active_s = cnt;
        }
        __syncthreads();
        n_active = n_active_s;
    } else {
        const int top_row = min(qtile * QBW * 32 + QBW * 32, seq_len) - 1;  // causal: keys 0..top_row
        n_active = (top_row >> 6) + 1;
    }

    const float c2 = p.scale_log2;
    s16x8 qf[2][KC];   // the wave's query rows as B-operand fragments; filled once the first K/V tile has been requested

    // ---- global -> LDS tile copy ----------------------------------------------------------
    // Instruction j of this wave fills rows (j*kWaves + w)*RPI .. +RPI-1 of the tile.  The lane's byte offset from the
    // first of the instruction's rows is a constant (row and swizzled granule; kWaves*RPI is a multiple of every
    // swizzle period, so it is the same for every j), and the instruction's first row goes into the scalar base: a
    // full tile costs no vector ALU work.
    static_assert((kWaves * RPI) % 16 == 0, "the swizzles repeat every 16 rows at most");
    uint32_t k_off0, v_off0;
    {
        const int row = w * RPI + lane / G, pg = lane % G;
        k_off0 = (uint32_t)((int64_t)(lane / G) * p.kv2 + 8 * (pg ^ GEO::swz_k(row))) * 2u;
        v_off0 = (uint32_t)((int64_t)(lane / G) * p.kv2 + 8 * (pg ^ GEO::swz_v(row))) * 2u;
    }
    // In this one instantiation the compiler (out of scalar registers) keeps the row bases in vector registers and moves
    // them to scalar ones right in front of every copy, closer than a copy may follow such a move (copy16_global_to_lds);
    // the build's scan of the generated code is what says which instantiations need this.
    constexpr bool kFreshBases = MODE == MODE_VARLEN && NW == 4 && D == 128;
    auto issue_tile = [&](int kt, int stage) {
        const int key0 = kt * 64;
        const short* kbase = Kh + (int64_t)key0 * p.kv2;
        const short* vbase = Vh + (int64_t)key0 * p.kv2;
        if (key0 + 64 <= seq_len) {
#pragma unroll
            for (int j = 0; j < NLD; ++j) {
                const int row0 = (j * kWaves + w) * RPI;
                copy16_global_to_lds<kFreshBases>(kbase + (int64_t)row0 * p.kv2, k_off0, &kv_lds[stage][row0 * RB]);
                copy16_global_to_lds<kFreshBases>(vbase + (int64_t)row0 * p.kv2, v_off0, &kv_lds[stage][GEO::TILE_BYTES + row0 * RB]);
            }
        } else {   // tile crossing the end of the sequence: rows past it re-read the last row
#pragma unroll
            for (int j = 0; j < NLD; ++j) {
                const int row0 = (j * kWaves + w) * RPI;
                const int row = row0 + lane / G, pg = lane % G;
                const int64_t grow = (int64_t)(min(key0 + row, last_row) - key0) * p.kv2;
                copy16_global_to_lds<kFreshBases>(kbase, (uint32_t)(grow + 8 * (pg ^ GEO::swz_k(row))) * 2u, &kv_lds[stage][row0 * RB]);
                copy16_global_to_lds<kFreshBases>(vbase, (uint32_t)(grow + 8 * (pg ^ GEO::swz_v(row))) * 2u, &kv_lds[stage][GEO::TILE_BYTES + row0 * RB]);
            }
        }
    };

    // ---- per-lane LDS read addresses (stage 0; the other stage and the row blocks are immediates) ----
    // The matrix instruction is v_mfma_f32_16x16x32: lane (l16, quad) holds row l16, contraction values 8 quad + 0..7 of
    // an A or B fragment and rows 4 quad + 0..3, column l16 of a result block.  K fragment (chunk c of 32 head
    // dimensions, key block kb of 16): row 16kb + l16, granule (4c + quad) ^ swz_k(row); swz_k is the same for rows l16
    // and 16kb + l16.  V^T fragment (chunk ck of 32 keys, block db of 16 head dimensions): two transpose reads, the
    // 16-lane group `quad` addressing key rows 32ck + 4 quad + 0..3 and 32ck + 16 + 4 quad + 0..3, columns 16db + 4(li&3);
    // swz_v depends on quad and li only.
    const int li = l16;
    uint32_t k_rd[KC], v_rd[DB];
    {
        const int sw = GEO::swz_k(l16);
#pragma unroll
        for (int c = 0; c < KC; ++c) k_rd[c] = lds_addr(&kv_lds[0][0]) + l16 * RB + 16 * ((4 * c + quad) ^ sw);
        const int vrow = 4 * quad + (li >> 2);
        const int swv = GEO::swz_v(vrow);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            const int dcol = 16 * db + 4 * (li & 3);
            v_rd[db] = lds_addr(&kv_lds[0][GEO::TILE_BYTES]) + vrow * RB + 16 * ((dcol >> 3) ^ swv) + 2 * (dcol & 7);
        }
    }

    f32x4 o_acc[DB][2];   // [block of 16 head dimensions][block of 16 query rows]: rows d = 16db + 4 quad + 0..3, column l16
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) o_acc[db][qb] = f32x4{0.f, 0.f, 0.f, 0.f};
    // Reference exponent of each of the lane's two query rows (log2 units; -inf until a key has been seen) and the
    // lane's share of the softmax denominators.  The reference moves only when a tile's largest exponent
    // exceeds it by more than kLazyLog2, so most tiles rescale nothing and weights stay below 2^kLazyLog2.
    float m_ref[2] = {-INFINITY, -INFINITY}, l_sum[2] = {0.f, 0.f};
    constexpr float kLazyLog2 = 8.f;
    float grow_at[2] = {-INFINITY, -INFINITY};
    f32x4 neg_ref[2];   // -m_ref in every register (0 while there is no reference): the MFMA C operand of Q K^T
    neg_ref[0] = neg_ref[1] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto tile_of = [&](uint32_t e, int it, int& kt, uint32_t& cls_w) {
        if (kDense) {
            kt = (int)(e & 0xffffu);
            cls_w = (e >> (16 + 2 * my_qt64_slot)) & 3u;
        } else {
            kt = it;
            cls_w = (64 * kt + 63 <= q_row0) ? TILE_ALL : ((64 * kt > q_row0 + 31) ? TILE_NONE : TILE_MIXED);
        }
        if (!wave_on) cls_w = TILE_NONE;
    };
    auto list_entry = [&](int it) -> uint32_t {   // wave-uniform
        if (!kDense || n_active <= 0) return 0u;
        return __builtin_amdgcn_readfirstlane(tile_list[min(it, n_active - 1)]);
    };
    // mask words of a MIXED dense tile: word [qb][kb] covers keys key0 + 16kb + 4 quad + 0..3 of query row qrow[qb]
    uint32_t mw[2][4] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
    auto fetch_mask = [&](int kt) {
        const int key0 = kt * 64;
        if (p.mask_vec && key0 + 64 <= seq_len) {
#pragma unroll
            for (int qb = 0; qb < 2; ++qb)
#pragma unroll
                for (int kb = 0; kb < 4; ++kb)
                    mw[qb][kb] = *reinterpret_cast<const uint32_t*>(mrow[qb] + key0 + 16 * kb + 4 * quad);
        } else {  // unaligned rows or a tile crossing the end: bytes, clamped (the range test comes later)
#pragma unroll
            for (int qb = 0; qb < 2; ++qb)
#pragma unroll
                for (int kb = 0; kb < 4; ++kb) {
                    const int kbase = key0 + 16 * kb + 4 * quad;
                    uint32_t x = 0;
#pragma unroll
                    for (int e = 0; e < 4; ++e) x |= (uint32_t)mrow[qb][min(kbase + e, last_row)] << (8 * e);
                    mw[qb][kb] = x;
                }
        }
    };

    // ---- one key tile, K/V in LDS stage STAGE (compile-time, so every LDS address is base + immediate) ----
    auto process_tile = [&](auto stage_tag, int kt, uint32_t cls_w) {
        constexpr int STAGE = decltype(stage_tag)::value;
        constexpr int SOFF = STAGE * STAGE_BYTES;
        const int key0 = kt * 64;
        auto pin = [&]() __attribute__((always_inline)) { __builtin_amdgcn_sched_barrier(0); };

        // V^T fragment of key chunk ck (32 keys), block db (16 head dimensions)
        auto read_v = [&](int ck, int db) __attribute__((always_inline)) -> s16x8 {
            const s16x4 t0 = lds_read_tr16(v_rd[db], SOFF + (32 * ck) * RB);
            const s16x4 t1 = lds_read_tr16(v_rd[db], SOFF + (32 * ck + 16) * RB);
            return s16x8{t0[0], t0[1], t0[2], t0[3], t1[0], t1[1], t1[2], t1[3]};
        };
        s16x8 va[DB];   // the V^T fragments of one key chunk; refilled with the next chunk's as they are used the last time

        // S^T = K Q^T, accumulated on top of -reference: register e of block [kb][qb] is key 16kb + 4 quad + e, query row
        // 16qb + l16.  K fragments go through two register buffers of one contraction chunk each (four key blocks): the
        // fragment just used for the last time is refilled two chunks ahead, between the MFMAs (every MFMA and read is
        // pinned where it is written: left alone the compiler moved every read down to just before the MFMAs that use it).
        // Between the MFMAs of the last chunk, whose fragments are not refilled, the first key chunk's V^T fragments are
        // requested.  The accumulators start from -reference (neg_ref, a register block that changes only when the
        // reference does), so the MFMA output is the exponent relative to the reference.
        f32x4 e_acc[4][2];
        {
            s16x8 kf[2][4];   // [buffer][key block]
#pragma unroll
            for (int c = 0; c < 2 && c < KC; ++c)
#pragma unroll
                for (int kb = 0; kb < 4; ++kb) kf[c][kb] = lds_read_b128(k_rd[c], SOFF + 16 * kb * RB);
            pin();
#pragma unroll
            for (int c = 0; c < KC; ++c) {
#pragma unroll
                for (int kb = 0; kb < 4; ++kb) {
#pragma unroll
                    for (int qb = 0; qb < 2; ++qb)
                        e_acc[kb][qb] = T::mfma16(kf[c & 1][kb], qf[qb][c], c == 0 ? neg_ref[qb] : e_acc[kb][qb]);
                    pin();
                    if (c + 2 < KC) {
                        kf[c & 1][kb] = lds_read_b128(k_rd[c + 2], SOFF + 16 * kb * RB);
                    } else if (c + 1 == KC) {
#pragma unroll
                        for (int db = kb * (DB / 4); db < (kb + 1) * (DB / 4); ++db) va[db] = read_v(0, db);
                    }
                    pin();
                }
            }
        }

        // ---- masking ----------------------------------------------------------------------
        // The test by position (keys past the end of the sequence; in a packed batch also keys after the lane's query
        // row) is one compare of a constant with a per-lane limit; dense MIXED tiles test their mask bytes as well.
        if (cls_w == TILE_MIXED || key0 + 64 > seq_len) {
            const bool use_bytes = kDense && cls_w == TILE_MIXED;
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
                int lim = last_row - key0 - 4 * quad;                              // largest kept 16kb + e
                if (MODE == MODE_VARLEN) lim = min(lim, qrow[qb] - key0 - 4 * quad);
#pragma unroll
                for (int kb = 0; kb < 4; ++kb)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        bool keep = 16 * kb + e <= lim;
                        if (kDense) keep = keep && (!use_bytes || ((mw[qb][kb] >> (8 * e)) & 0xffu) != 0u);
                        e_acc[kb][qb][e] = keep ? e_acc[kb][qb][e] : -INFINITY;
                    }
            }
        }
        // ---- reference update (rare after the first tiles) --------------------------------------
        {
            // The lane's largest exponent of each row (16 registers; three-operand maxima written out: through fmaxf every
            // operand that comes out of an MFMA is first passed through an instruction of its own that quiets a signalling
            // NaN).  A row moves its reference when its largest exponent exceeds grow_at (kLazyLog2 once the row has a
            // reference, -inf before), which is the case exactly when one of the row's four lanes sees it: the lane swaps
            // that make the row's maximum are left to the branch.
            float mx[2];
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
                float x = max3(e_acc[0][qb][0], e_acc[0][qb][1], e_acc[0][qb][2]);
                x = max3(x, e_acc[0][qb][3], e_acc[1][qb][0]);
#pragma unroll
                for (int kb = 1; kb < 4; ++kb) {
                    x = max3(x, e_acc[kb][qb][1], e_acc[kb][qb][2]);
                    x = kb < 3 ? max3(x, e_acc[kb][qb][3], e_acc[kb + 1][qb][0]) : max2(x, e_acc[kb][qb][3]);
                }
                mx[qb] = x;
            }
            if (__any(mx[0] > grow_at[0] || mx[1] > grow_at[1])) {  // wave-uniform branch
                mx[0] = max_across_quads(mx[0]);   // largest exponent of the row in this tile, relative to the reference
                mx[1] = max_across_quads(mx[1]);
                const bool grow0 = mx[0] > grow_at[0], grow1 = mx[1] > grow_at[1];
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) {
                    const bool grow = qb == 0 ? grow0 : grow1;
                    const float delta = grow ? mx[qb] : 0.f;
                    const float alpha = (m_ref[qb] == -INFINITY) ? 0.f : fast_exp2(-delta);
                    m_ref[qb] = grow ? ((m_ref[qb] == -INFINITY) ? mx[qb] : m_ref[qb] + mx[qb]) : m_ref[qb];
                    grow_at[qb] = (m_ref[qb] == -INFINITY) ? -INFINITY : kLazyLog2;
                    const float nr = (m_ref[qb] == -INFINITY) ? 0.f : -m_ref[qb];
                    neg_ref[qb] = f32x4{nr, nr, nr, nr};
                    l_sum[qb] *= alpha;
#pragma unroll
                    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
                        for (int e = 0; e < 4; ++e) e_acc[kb][qb][e] -= delta;
#pragma unroll
                    for (int db = 0; db < DB; ++db)
#pragma unroll
                        for (int e = 0; e < 4; ++e) o_acc[db][qb][e] *= alpha;
                }
            }
        }
        // ---- P = 2^E and O^T += V^T P^T, one 32-key chunk and one 16-row query block at a time ---------
        // Chunk ck contracts keys 32ck .. 32ck+31 in the order 32ck + 16(i/4) + 4 quad + i%4 (i = element of the lane's
        // 8-wide slice), which is the order the exponent registers of key blocks 2ck and 2ck+1 already have and the
        // order the two transpose reads of a V^T fragment deliver.  The weights of the next (chunk, query block) are
        // computed before the MFMAs of the current one are issued, so they run while those are in the matrix pipe.
        float ls[2] = {0.f, 0.f};
        // quarter i of the weights of (chunk ck, query block qb): two exponentials, packed
        auto weights_quarter = [&](int ck, int qb, int i) __attribute__((always_inline)) -> uint32_t {
            const int kb = 2 * ck + (i >> 1), r = 2 * (i & 1);
            const uint32_t pk = T::pack2(fast_exp2(e_acc[kb][qb][r]), fast_exp2(e_acc[kb][qb][r + 1]));
            ls[qb] = T::add_pair(pk, ls[qb]);   // the denominator sums the rounded weights the MFMA uses
            asm volatile("" : "+v"(ls[qb]));     // ... here, not in one run after the tile's last MFMA
            return pk;
        };
        uint32_t pw[2][4];   // the packed weights in use and the next ones in the making
#pragma unroll
        for (int i = 0; i < 4; ++i) pw[0][i] = weights_quarter(0, 0, i);
        pin();
#pragma unroll
        for (int s = 0; s < 4; ++s) {   // (ck, qb) = (s >> 1, s & 1)
            const int ck = s >> 1, qb = s & 1;
            uint4 pu; pu.x = pw[s & 1][0]; pu.y = pw[s & 1][1]; pu.z = pw[s & 1][2]; pu.w = pw[s & 1][3];
            const s16x8 pcur = __builtin_bit_cast(s16x8, pu);
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                o_acc[db][qb] = T::mfma16(va[db], pcur, o_acc[db][qb]);
                pin();
                if (qb == 1 && ck == 0) va[db] = read_v(1, db);   // used for the last time: the next chunk's fragment takes its place
                if (s + 1 < 4 && db < 4) pw[(s + 1) & 1][db] = weights_quarter((s + 1) >> 1, (s + 1) & 1, db);
                pin();
            }
        }
        l_sum[0] += ls[0];
        l_sum[1] += ls[1];
    };

    // ---- main loop: one barrier per tile; the copy of tile t+1 is issued right after the barrier that
    // opens tile t, into the stage tile t-1 has just vacated ---------------------------------------
    uint32_t e_cur = list_entry(0), e_next = list_entry(1);
    int kt_first = 0; uint32_t cls_first = TILE_NONE;
    if (n_active > 0) {
        tile_of(e_cur, 0, kt_first, cls_first);
        issue_tile(kt_first, 0);
    }
    // ---- Q fragments (B operand): lane = query row 16qb + l16, d = 32c + 8 quad + 0..7 --------------------
    // Q is multiplied by scale*log2(e) once, here, so that the MFMA accumulator of Q K^T is directly
    // the base-2 exponent of the softmax weight (minus the running reference it is initialised with).
    // The rows were requested before the tile list was built, and the first K/V tile after them: copies retire in
    // order, so the rows have landed once no more than that tile's copies are outstanding.
    if (n_active > 0) wait_vmcnt<2 * NLD>(); else wait_vmcnt<0>();
    {
        const uint32_t qa = lds_addr(q_stage) + l16 * RB;
        const int sw = GEO::swz_k(l16);   // the same for row 16 + l16
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
            for (int c = 0; c < KC; ++c) qf[qb][c] = T::scale8(lds_read_b128(qa + 16 * ((4 * c + quad) ^ sw), 16 * qb * RB), c2);
    }
    if (kDense && n_active > 0 && cls_first == TILE_MIXED) fetch_mask(kt_first);
    auto iteration = [&](auto stage_tag, int it) {
        constexpr int STAGE = decltype(stage_tag)::value;
        int kt, ktn; uint32_t cls_w, cn;
        tile_of(e_cur, it, kt, cls_w);
        tile_of(e_next, it + 1, ktn, cn);
        const uint32_t e_after = list_entry(it + 2);   // read early, used next iteration
        wait_vmcnt<0>();       // this wave's share of tile `it` (and its mask words) has landed
        __syncthreads();       // everyone's has; stage STAGE^1 is no longer being read
        if (it + 1 < n_active) issue_tile(ktn, STAGE ^ 1);
        if (cls_w != TILE_NONE) process_tile(stage_tag, kt, cls_w);
        if (kDense && it + 1 < n_active && cn == TILE_MIXED) fetch_mask(ktn);   // after this tile's words were used
        e_cur = e_next; e_next = e_after;
    };
    for (int it = 0; it < n_active; it += 2) {
        iteration(std::integral_constant<int, 0>{}, it);
        if (it + 1 < n_active) iteration(std::integral_constant<int, 1>{}, it + 1);
    }

    // ---- epilogue: normalise, transpose through the wave's staging area, store whole rows ---------------
    // A lane holds 4 consecutive columns of ONE row per register quadruple: stored from the registers, an instruction
    // would write 16 bytes to each of 32 rows (2.2 us per item for the 16 stores of a wave).  Written to LDS (8 bytes
    // per lane, granules XOR-swizzled by row) and read back 16 bytes per lane, RPI whole rows per instruction, the same
    // data leaves in 32/RPI stores of whole rows.
    if (!wave_on) return;
    float inv[2];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
        const float l = sum_across_quads(l_sum[qb]);
        inv[qb] = l > 0.f ? 1.f / l : 0.f;
    }
    {
        const int free_stage = (n_active & 1);   // the last tile sat in stage (n_active - 1) & 1
        const uint32_t so = kAliasRows ? lds_addr(&kv_lds[0][0]) + free_stage * STAGE_BYTES + w * ROWS_BYTES : lds_addr(q_stage);
        typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
        typedef __attribute__((address_space(3))) u32x2 lds_u32x2;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
                u32x2 pk;
                pk.x = T::pack2(o_acc[db][qb][0] * inv[qb], o_acc[db][qb][1] * inv[qb]);
                pk.y = T::pack2(o_acc[db][qb][2] * inv[qb], o_acc[db][qb][3] * inv[qb]);
                const int row = 16 * qb + l16;
                const int gi = 2 * db + (quad >> 1);   // 16-byte granule of the row: columns 8gi..8gi+7, this lane's half 4(quad&1)..+3
                *(lds_u32x2*)(uintptr_t)(so + row * RB + 16 * (gi ^ (row & (G - 1))) + 8 * (quad & 1)) = pk;
            }
        }
        if (q_row0 + 32 <= seq_len) {   // every row exists: a wave-uniform base per store plus one 32-bit lane offset
            const int row_in = lane / G, gi = lane % G;
            const uint32_t lane_off = (uint32_t)((int64_t)row_in * p.o2 + 8 * gi) * 2u;
            char* obase = reinterpret_cast<char*>(Oh + (int64_t)q_row0 * p.o2);
#pragma unroll
            for (int i = 0; i < 32 / RPI; ++i) {
                const int r = i * RPI + row_in;
                const s16x8 val = lds_read_b128(so + r * RB + 16 * (gi ^ (r & (G - 1))), 0);
                *reinterpret_cast<s16x8*>(obase + (int64_t)(i * RPI) * p.o2 * 2 + lane_off) = val;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 32 / RPI; ++i) {
                const int r = i * RPI + lane / G, gi = lane % G;
                const s16x8 val = lds_read_b128(so + r * RB + 16 * (gi ^ (r & (G - 1))), 0);
                if (q_row0 + r < seq_len) *reinterpret_cast<s16x8*>(Oh + (int64_t)(q_row0 + r) * p.o2 + 8 * gi) = val;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// Host side
// ------------------------------------------------------------------------------------------
static size_t cls_bytes(int64_t B, int64_t L) {
    const int64_t nt = (L + 63) / 64;
    return (size_t)(B * nt * nt + 255) / 256 * 256;
}

template <class T, int D, int MODE, int NW>
static int launch_prefill(const PrefillParams& p, int grid, hipStream_t stream) {
    hipLaunchKernelGGL((prefill_kernel<T, D, MODE, NW>), dim3(grid), dim3(NW * 64), 0, stream, p);
    return check_launch("prefill_kernel");
}

template <int MODE, int NW>
static int dispatch_prefill_nw(int dtype, int64_t D, const PrefillParams& p, int grid, hipStream_t stream) {
    if (dtype == MINFER_ATTN_F16) {
        return D == 128 ? launch_prefill<F16, 128, MODE, NW>(p, grid, stream) : launch_prefill<F16, 64, MODE, NW>(p, grid, stream);
    }
    return D == 128 ? launch_prefill<BF16, 128, MODE, NW>(p, grid, stream) : launch_prefill<BF16, 64, MODE, NW>(p, grid, stream);
}

template <int MODE>
static int dispatch_prefill(int dtype, int64_t D, const PrefillParams& p, int waves, int grid, hipStream_t stream) {
    return waves == kWavesSmall ? dispatch_prefill_nw<MODE, kWavesSmall>(dtype, D, p, grid, stream)
                                : dispatch_prefill_nw<MODE, kWavesBig>(dtype, D, p, grid, stream);
}

// Waves per workgroup for a launch whose sequences have at most `longest` rows.  Short sequences mean few key tiles per
// workgroup, so the cost a workgroup pays once (query rows in, first tile, output rows out, hand-over of the compute
// unit) is a large share: two small workgroups per compute unit hide it under each other's tiles.  Long sequences
// amortise it and gain more from sharing every staged K/V tile among 256 rows.
#ifndef MINFER_PREFILL_FORCE_WAVES
#define MINFER_PREFILL_FORCE_WAVES 0
#endif
// Measured, 4 against 8 waves, 32 query heads over 8 KV heads: 128 packed sequences of 128 rows 87 / 98 us, 64 of 512
// rows 256 / 263 us, dense B=16 L=512 68 / 73 us, B=8 L=1024 95.5 / 97.8 us, B=4 L=2048 159 / 156 us, L=4096 157 / 146 us.
// At head_dim 64 a tile has half the MFMAs for the same vector work and the small workgroups win at every length
// (clocks settled, 4 / 8 waves: B=8 L=1024 54.6 / 65.2 us, B=4 L=2048 88 / 102, B=1 L=8192 292 / 330, L=16384 1113 / 1267;
// head_dim 128 for comparison: L=1536 180 / 182, L=2048 151.5 / 149.6, L=4096 143.7 / 134.4, L=8192 506 / 494).
constexpr int64_t kSmallWorkgroupMaxRows = 1024;
static int prefill_waves(int64_t longest, int64_t D) {
    if (MINFER_PREFILL_FORCE_WAVES) return MINFER_PREFILL_FORCE_WAVES;
    return (D == 64 || longest <= kSmallWorkgroupMaxRows) ? kWavesSmall : kWavesBig;
}

// The global->LDS copies of K/V tiles and query rows and the output stores address a block's rows with a 32-bit unsigned
// per-lane byte offset from the block's first row (a few rows of it, plus a granule inside the row): the row strides
// must keep that below 2^32.
static int check_row_stride(const minfer_attn_strides* st, const char* op) {
    if (st->kv2 >= (INT64_C(1) << 25) || st->q2 >= (INT64_C(1) << 25) || st->o2 >= (INT64_C(1) << 25)) {
        snprintf(error_buf(), 512, "%s: row strides (dim 2) of q, k/v and out must be below 2^25 elements", op);
        return MINFER_ATTN_EINVAL;
    }
    return MINFER_ATTN_OK;
}

static void fill_common(PrefillParams& p, const void* q, const void* k, const void* v, void* out,
                        int64_t Hq, int64_t Hkv, int64_t D, const minfer_attn_strides* st, int kWaves) {
    p.q = q; p.k = k; p.v = v; p.out = out;
    p.q0 = st->q0; p.q1 = st->q1; p.q2 = st->q2;
    p.kv0 = st->kv0; p.kv1 = st->kv1; p.kv2 = st->kv2;
    p.o0 = st->o0; p.o1 = st->o1; p.o2 = st->o2;
    p.Hq = (int)Hq; p.Hkv = (int)Hkv; p.n_rep = (int)(Hq / Hkv);
    p.hpw_log2 = (p.n_rep % 8 == 0 && kWaves >= 8) ? 3 : (p.n_rep % 4 == 0) ? 2 : ((p.n_rep % 2 == 0) ? 1 : 0);
    p.n_hg = p.n_rep >> p.hpw_log2;
    p.scale_log2 = (float)(1.4426950408889634 / sqrt((double)D));
}

}  // namespace minfer_attn

using namespace minfer_attn;

MINFER_ATTN_EXPORT size_t minfer_flash_attn_workspace_bytes(int64_t B, int64_t L) {
    if (B <= 0 || L <= 0) return 256;
    return cls_bytes(B, L);
}

MINFER_ATTN_EXPORT int minfer_flash_attn(int dtype, const void* q, const void* k, const void* v,
                                 const uint8_t* mask, void* out, int64_t B, int64_t Hq, int64_t Hkv,
                                 int64_t L, int64_t D, const minfer_attn_strides* st, void* workspace,
                                 size_t workspace_bytes, void* stream_v) {
    clear_error();
    if (int rc = check_common(dtype, q, k, v, out, Hq, Hkv, D, st)) return rc;
    if (int rc = check_row_stride(st, "flash_attn")) return rc;
    if (!mask) return fail(MINFER_ATTN_EINVAL, "flash_attn: mask is null");
    if (B < 0 || L < 0) return fail(MINFER_ATTN_EINVAL, "flash_attn: negative B or L");
    if (B == 0 || L == 0) return MINFER_ATTN_OK;
    if (L > 64 * (int64_t)kMaxKeyTiles) return fail(MINFER_ATTN_EINVAL, "flash_attn: L > 131072 unsupported");
    if (B > 65535) return fail(MINFER_ATTN_EINVAL, "flash_attn: B > 65535 unsupported");
    if (!workspace || workspace_bytes < cls_bytes(B, L))
        return fail(MINFER_ATTN_EWORKSPACE, "flash_attn: workspace too small (see minfer_flash_attn_workspace_bytes)");
    hipStream_t stream = (hipStream_t)stream_v;

    PrefillParams p{};
    const int kWaves = prefill_waves(L, D);
    fill_common(p, q, k, v, out, Hq, Hkv, D, st, kWaves);
    p.mask = mask; p.cls = (const uint8_t*)workspace; p.cu = nullptr;
    p.L = (int)L; p.B = (int)B;
    p.NQT = p.NKT = (int)((L + 63) / 64);
    const int rows_per_wg = 32 * (kWaves >> p.hpw_log2);
    p.NQ = (int)((L + rows_per_wg - 1) / rows_per_wg);
    p.n_seqs = 0;
    p.mask_vec = ((L & 15) == 0 && aligned16(mask)) ? 1 : 0;
    const int64_t grid = (int64_t)p.NQ * B * Hkv * p.n_hg;
    if (grid > 0x7fffffffLL) return fail(MINFER_ATTN_EINVAL, "flash_attn: problem too large for one launch");

    // A short problem whose mask rows can be read in 16-byte pieces and whose workgroups all fit on the chip at once
    // (2 per CU, 256 CUs) needs no pre-pass: its workgroups classify their own rows, which takes 2-3 us off a call of
    // 9-28 us.  With more workgroups than that the pre-pass is cheaper than every head re-reading the mask rows.
    if (p.mask_vec && L <= kSelfClassifyMaxL && kWaves == kWavesSmall && grid <= kSelfClassifyMaxGrid) {
        p.cls = nullptr;
        return dispatch_prefill_nw<MODE_DENSE_SELF, kWavesSmall>(dtype, D, p, (int)grid, stream);
    }
    if (p.mask_vec)
        hipLaunchKernelGGL(classify_mask_kernel_256, dim3((p.NKT + 3) / 4, p.NQT, (unsigned)B), dim3(256), 0, stream,
                           mask, (uint8_t*)workspace, p.L, p.NQT, p.NKT);
    else
        hipLaunchKernelGGL(classify_mask_kernel, dim3((p.NKT + 15) / 16, p.NQT, (unsigned)B), dim3(256), 0, stream,
                           mask, (uint8_t*)workspace, p.L, p.NQT, p.NKT, p.mask_vec);
    if (int rc = check_launch("classify_mask_kernel")) return rc;
    return dispatch_prefill<MODE_DENSE>(dtype, D, p, kWaves, (int)grid, stream);
}

MINFER_ATTN_EXPORT int minfer_flash_attn_varlen(int dtype, const void* q, const void* k, const void* v,
                                        const int32_t* cu_seqlens, int64_t n_seqs, int64_t max_seqlen,
                                        void* out, int64_t Hq, int64_t Hkv, int64_t T, int64_t D,
                                        const minfer_attn_strides* st, void* stream_v) {
    clear_error();
    if (int rc = check_common(dtype, q, k, v, out, Hq, Hkv, D, st)) return rc;
    if (int rc = check_row_stride(st, "flash_attn_varlen")) return rc;
    if (!cu_seqlens) return fail(MINFER_ATTN_EINVAL, "flash_attn_varlen: cu_seqlens is null");
    if (n_seqs < 0 || T < 0 || max_seqlen < 0) return fail(MINFER_ATTN_EINVAL, "flash_attn_varlen: negative size");
    if (n_seqs == 0 || T == 0) return MINFER_ATTN_OK;
    if (T > 0x7fffffffLL / 2) return fail(MINFER_ATTN_EINVAL, "flash_attn_varlen: T too large");
    hipStream_t stream = (hipStream_t)stream_v;

    // max_seqlen 0 means "not known".  Rows of a sequence past max_seqlen are not computed, so a caller's bound
    // must be at least the longest sequence (as in every varlen attention interface).
    const int64_t max_len = (max_seqlen > 0 && max_seqlen < T) ? max_seqlen : T;
    PrefillParams p{};
    const int kWaves = prefill_waves(max_len, D);
    fill_common(p, q, k, v, out, Hq, Hkv, D, st, kWaves);
    p.mask = nullptr; p.cls = nullptr; p.cu = cu_seqlens;
    p.L = (int)T; p.B = 1;
    p.NQT = p.NKT = 0;
    const int rows_per_wg = 32 * (kWaves >> p.hpw_log2);
    // query tiles: sum over sequences of ceil(len / rows_per_wg) <= both bounds below (cu_seqlens lives on the device,
    // so the exact count is not known here; workgroups past it exit at once)
    const int64_t nq_packed = (T + rows_per_wg - 1) / rows_per_wg + n_seqs;
    const int64_t nq_each = n_seqs * ((max_len + rows_per_wg - 1) / rows_per_wg);
    p.NQ = (int)(nq_each < nq_packed ? nq_each : nq_packed);
    p.n_seqs = (int)n_seqs;
    p.max_len = (int)max_len;
    const int64_t grid = (int64_t)p.NQ * Hkv * p.n_hg;
    if (grid > 0x7fffffffLL) return fail(MINFER_ATTN_EINVAL, "flash_attn_varlen: problem too large for one launch");
    return dispatch_prefill<MODE_VARLEN>(dtype, D, p, kWaves, (int)grid, stream);
}

// ------------------------------------------------------------------------------------------------
// Prefill over K/V given as Q8_0 blocks (the operator's (qtype_int, qblock_size, qtype_size) = (8, 32, 34);
// reference: the unused leading arguments of flash_attn_cuda, cuda/flash_attn/op.cuh:22-24).  In a prefill every K/V
// tile is read by every query tile that attends it, so dequantising inside the attention kernel would repeat the work
// once per query tile; instead one pass turns the rows into fp16 (exactly the values the reference's dequantiser gives,
// cuda/quants/impls.cuh:121-143) in the caller's workspace, read back from the caches by the fp16 kernel.
// ------------------------------------------------------------------------------------------------
namespace minfer_attn {
static size_t kv_f16_bytes(int64_t B, int64_t Hkv, int64_t L, int64_t D) {
    return ((size_t)(B * Hkv * L * D * 2) + 255) / 256 * 256;
}
static int check_q8_kv(const char* op, int dtype, const void* q, const void* k, const void* v, const void* out, int64_t Hq,
                       int64_t Hkv, int64_t D, const minfer_attn_strides* st) {
    char msg[200];
    auto bad = [&](const char* what) { snprintf(msg, sizeof msg, "%s: %s", op, what); return fail(MINFER_ATTN_EINVAL, msg); };
    if (dtype != MINFER_ATTN_F16) return bad("q and out must be fp16 over Q8_0 k/v (the dequantiser produces fp16)");
    if (D != 64 && D != 128) return bad("head_dim must be 64 or 128");
    if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0) return bad("n_heads must be a positive multiple of n_kv_heads");
    if (!st) return bad("strides is null");
    if (!q || !k || !v || !out) return bad("q, k, v and out must be non-null");
    if (!aligned16(q) || !aligned16(out)) return bad("q and out must be 16-byte aligned");
    if (((uintptr_t)k | (uintptr_t)v) & 1u) return bad("Q8_0 k and v must be 2-byte aligned");
    const int64_t e[6] = {st->q0, st->q1, st->q2, st->o0, st->o1, st->o2};
    for (int i = 0; i < 6; ++i)
        if (e[i] % 8 != 0 || e[i] < 0) return bad("strides of q and out must be non-negative multiples of 8 elements");
    if (st->kv2 != D / 32 * 34) return bad("Q8_0 rows must be dense (row stride = D/32 * 34 bytes)");
    if (st->kv0 < 0 || st->kv1 < 0 || st->kv0 % 2 || st->kv1 % 2) return bad("Q8_0 k/v strides must be non-negative even byte counts");
    return MINFER_ATTN_OK;
}
}  // namespace minfer_attn

MINFER_ATTN_EXPORT size_t minfer_flash_attn_q8_0_workspace_bytes(int64_t B, int64_t Hkv, int64_t L, int64_t D) {
    if (B <= 0 || Hkv <= 0 || L <= 0 || D <= 0) return 256;
    return cls_bytes(B, L) + 2 * kv_f16_bytes(B, Hkv, L, D);
}

MINFER_ATTN_EXPORT int minfer_flash_attn_q8_0(const void* q, const void* k, const void* v, const uint8_t* mask, void* out,
                                              int64_t B, int64_t Hq, int64_t Hkv, int64_t L, int64_t D,
                                              const minfer_attn_strides* st, void* workspace, size_t workspace_bytes,
                                              void* stream_v) {
    clear_error();
    if (int rc = check_q8_kv("flash_attn_q8_0", MINFER_ATTN_F16, q, k, v, out, Hq, Hkv, D, st)) return rc;
    if (!mask) return fail(MINFER_ATTN_EINVAL, "flash_attn_q8_0: mask is null");
    if (B < 0 || L < 0) return fail(MINFER_ATTN_EINVAL, "flash_attn_q8_0: negative B or L");
    if (B == 0 || L == 0) return MINFER_ATTN_OK;
    if (B * Hkv > 65535) return fail(MINFER_ATTN_EINVAL, "flash_attn_q8_0: B * n_kv_heads > 65535 unsupported");
    const size_t cls = cls_bytes(B, L), kvb = kv_f16_bytes(B, Hkv, L, D);
    if (!workspace || workspace_bytes < cls + 2 * kvb || !aligned16(workspace))
        return fail(MINFER_ATTN_EWORKSPACE, "flash_attn_q8_0: workspace too small or misaligned (see minfer_flash_attn_q8_0_workspace_bytes)");
    char* ws = (char*)workspace;
    void* kf = ws + cls;
    void* vf = ws + cls + kvb;
    if (int rc = launch_dequant_q8_0_kv(k, v, kf, vf, B, Hkv, L, D, st->kv0, st->kv1, (hipStream_t)stream_v)) return rc;
    minfer_attn_strides s2 = *st;
    s2.kv0 = Hkv * L * D; s2.kv1 = L * D; s2.kv2 = D;
    return minfer_flash_attn(MINFER_ATTN_F16, q, kf, vf, mask, out, B, Hq, Hkv, L, D, &s2, workspace, cls, stream_v);
}

MINFER_ATTN_EXPORT size_t minfer_flash_attn_varlen_q8_0_workspace_bytes(int64_t Hkv, int64_t T, int64_t D) {
    if (Hkv <= 0 || T <= 0 || D <= 0) return 256;
    return 2 * kv_f16_bytes(1, Hkv, T, D);
}

MINFER_ATTN_EXPORT int minfer_flash_attn_varlen_q8_0(const void* q, const void* k, const void* v, const int32_t* cu_seqlens,
                                                     int64_t n_seqs, int64_t max_seqlen, void* out, int64_t Hq, int64_t Hkv,
                                                     int64_t T, int64_t D, const minfer_attn_strides* st, void* workspace,
                                                     size_t workspace_bytes, void* stream_v) {
    clear_error();
    if (int rc = check_q8_kv("flash_attn_varlen_q8_0", MINFER_ATTN_F16, q, k, v, out, Hq, Hkv, D, st)) return rc;
    if (!cu_seqlens) return fail(MINFER_ATTN_EINVAL, "flash_attn_varlen_q8_0: cu_seqlens is null");
    if (n_seqs < 0 || T < 0 || max_seqlen < 0) return fail(MINFER_ATTN_EINVAL, "flash_attn_varlen_q8_0: negative size");
    if (n_seqs == 0 || T == 0) return MINFER_ATTN_OK;
    if (Hkv > 65535) return fail(MINFER_ATTN_EINVAL, "flash_attn_varlen_q8_0: n_kv_heads > 65535 unsupported");
    const size_t kvb = kv_f16_bytes(1, Hkv, T, D);
    if (!workspace || workspace_bytes < 2 * kvb || !aligned16(workspace))
        return fail(MINFER_ATTN_EWORKSPACE, "flash_attn_varlen_q8_0: workspace too small or misaligned (see minfer_flash_attn_varlen_q8_0_workspace_bytes)");
    void* kf = workspace;
    void* vf = (char*)workspace + kvb;
    if (int rc = launch_dequant_q8_0_kv(k, v, kf, vf, 1, Hkv, T, D, 0, st->kv1, (hipStream_t)stream_v)) return rc;
    minfer_attn_strides s2 = *st;
    s2.kv0 = Hkv * T * D; s2.kv1 = T * D; s2.kv2 = D;
    return minfer_flash_attn_varlen(MINFER_ATTN_F16, q, kf, vf, cu_seqlens, n_seqs, max_seqlen, out, Hq, Hkv, T, D, &s2, stream_v);
}
