// Rotary position embedding for gfx950, in place and fused with the KV-cache append.
//
// What the reference computes (reference: src/minfer/kernels/torch_ext/csrc/cuda/il_rope/kernel.cuh:9-39,
// neox_rope/kernel.cuh:9-38, oracle src/minfer/kernels/refs.py:12-47): for token position `pos` and pair
// index i < rotary_dim/2, angle = pos * freq_base^(-2i/rotary_dim), and the pair (x0, x1) becomes
// (cos*x0 - sin*x1, sin*x0 + cos*x1).  Interleaved style pairs elements (2i, 2i+1) of a head, NeoX style
// pairs (i, i + rotary_dim/2).  Elements past rotary_dim are left alone.  x is [B, L, n_heads, head_dim].
//
// These are HBM-bound byte movers, so the design is about touching each byte once in 16-byte lane
// accesses and about not paying for the transcendental per element as the reference's one-thread-per-pair
// kernels do: the angle depends only on (position, pair), so a workgroup computes one cos/sin table per
// token in LDS (rotary_dim/2 entries; the frequencies arrive as kernel arguments, the angle is reduced in
// fp64 so that positions in the hundreds of thousands lose nothing) and every head of the token reuses
// it.  Only the rotary part of a head is read and written.
//
// The fused producer does what the model does right before attention (reference: src/minfer/core.py:228-232,
// cache layout core.py:105-127): rotate q in place, rotate k while copying it into the KV cache
// [B, n_kv_heads, Lmax, head_dim] at row positions[b] + l, copy v into the cache.  k is read once and never
// written back, the cache row is written once.  With Q8_0 caches (Q8 = true; rows of D/32 blocks of 34 bytes,
// strides in bytes) the rotated k and the v values are quantised on the way, from the values an fp16/bf16 cache
// would have held: the four lanes that hold a block's 32 values agree on its scale through two lane exchanges.
#include <algorithm>

#include "attn_common.h"
#include "attn_host.h"
#include "quant_q8.h"

namespace minfer_attn {

constexpr int kRopeThreads = 256;
constexpr int kMaxPairs = 128;    // rotary_dim <= 256

enum { ROPE_IL = MINFER_ROPE_INTERLEAVED, ROPE_NEOX = MINFER_ROPE_NEOX };

struct RopeParams {
    void* x;                  // [B, L, H, D], rotated in place (q of the fused producer)
    const void* k;            // fused: [B, L, Hkv, D]
    const void* v;            // fused: [B, L, Hkv, D]
    void* k_cache;            // fused: [B, Hkv, Lmax, D] with element strides c0, c1, c2 (Q8_0: byte strides)
    void* v_cache;
    const int32_t* positions; // fused: [B] first cache row of each sequence; otherwise null
    int64_t c0, c1, c2;
    int B, L, H, Hkv, D, rd, Lmax;
    int start_pos;            // not fused: position of token l is start_pos + l
    double inv_freq[kMaxPairs];
};

// The rotated pair, rounded to the element type: low half = cos*x0 - sin*x1, high half = sin*x0 + cos*x1.
// Each output is one product and one fused multiply-add, written out so that every kernel rounds alike:
// cos*x0 - sin*x1 = fma(cos, x0, -(sin*x1)), sin*x0 + cos*x1 = fma(cos, x1, sin*x0).
MA_DEV float fma_of_product(float c, float mine, float s, float other) {
    float t;
    {
#pragma clang fp contract(off)
        t = s * other;
    }
    return __builtin_fmaf(c, mine, t);
}
template <class T> MA_DEV uint32_t rotate_pair(float c, float s, short a, short b) {
    const float x0 = T::to_float(a), x1 = T::to_float(b);
    return T::pack2(fma_of_product(c, x0, -s, x1), fma_of_product(c, x1, s, x0));
}
// One output of a pair for a lane that holds one element and has fetched the other: signed_s is -sin for the lane
// with x0, +sin for the lane with x1.
template <class T> MA_DEV float rotate_one(float c, float signed_s, short mine, short other) {
    return fma_of_product(c, T::to_float(mine), signed_s, T::to_float(other));
}

// cos/sin of pos * inv_freq[i]: the product and its reduction to a fraction of a turn are done in fp64
// (exact enough for any int32 position), the sine and cosine of the reduced angle in fp32.
MA_DEV f32x2 table_entry(double inv_freq, int pos) {
    const double turns = (double)pos * inv_freq * 0.15915494309189535;   // angle / 2pi
    const float r = (float)((turns - rint(turns)) * 6.283185307179586);  // in [-pi, pi]
    float s, c;
    sincosf(r, &s, &c);
    return f32x2{c, s};
}

// Per token: every thread requests the 16-byte chunks it owns (a few in flight), the first rd/2 threads
// meanwhile fill the token's cos/sin table, one barrier, then rotate and store.  The producer into Q8_0 caches
// requests the first chunks of its next token before it works on the current one.
//
// Chunk numbering inside a token.  Rotary chunks of a tensor with NH heads: interleaved style, chunk c of
// head hd covers elements 8c..8c+7 (pairs 4c..4c+3), rd/8 chunks per head; NeoX style, chunk c covers
// elements 8c..8c+7 and their partners rd/2 + 8c.., rd/16 chunks per head.  Sections, in order: q rotary,
// then (fused only) k rotary, k tail (elements rd..D-1, copied), v (copied).
template <class T, int STYLE, bool FUSED, bool Q8, bool STREAM>
__global__ __launch_bounds__(kRopeThreads, FUSED ? 1 : 8) void rope_kernel(const RopeParams p) {
    static_assert(FUSED || !Q8, "only the fused producer writes a cache");
    __shared__ f32x2 tab[2][kMaxPairs];
    __shared__ double freq[kMaxPairs];   // the kernel argument array, where a thread can index it cheaply
    const int tid = threadIdx.x;
    const int half_rd = p.rd >> 1;
    const int cph = STYLE == ROPE_IL ? p.rd >> 3 : p.rd >> 4;   // rotary chunks per head
    const int tail = (p.D - p.rd) >> 3;                         // copy chunks per head past the rotary part
    const int n_q = p.H * cph;
    const int n_kr = FUSED ? p.Hkv * cph : 0;
    const int n_kt = FUSED ? p.Hkv * tail : 0;
    const int n_v = FUSED ? p.Hkv * (p.D >> 3) : 0;
    // Chunk numbers of a token: sections in the order above, each starting at a multiple of the wave size, so that the
    // 64 chunks a wave takes at a time are of one kind and its base pointers and branches are scalar.
    const int k_begin = FUSED ? (n_q + 63) & ~63 : n_q;
    const int kt_begin = FUSED ? (k_begin + n_kr + 63) & ~63 : n_q;
    const int v_begin = FUSED ? (kt_begin + n_kt + 63) & ~63 : n_q;
    const int n_all = FUSED ? v_begin + n_v : n_q;
    const int tokens = p.B * p.L;
    // The token's table is filled by the workgroup's first rd/2 threads, or, into Q8_0 caches, by its last: there
    // the first threads rotate and quantise k in their second chunk slot, which for the last ones is the lightest
    // (often empty); +2.4 %, while the other kernels lose 0.7 % that way.
    const int tab_i = Q8 ? tid - (kRopeThreads - half_rd) : (tid < half_rd ? tid : -1);
    if (tab_i >= 0) freq[tab_i] = p.inv_freq[tab_i];   // read back by the same thread only

    // what a token's chunks are addressed from
    struct Token {
        int pos; bool row_ok;
        short* xq; const short* xk; const short* xv;
        short* ck; short* cv;      // the token's cache row of head 0: element pointers ...
        char* qk; char* qv;        // ... or byte pointers (Q8_0)
    };
    auto token_at = [&](int tok) __attribute__((always_inline)) {
        Token k;
        const int b = __builtin_amdgcn_readfirstlane(tok / p.L), l = tok - b * p.L;
        // positions is an input nothing writes: read as constant memory the load is a scalar one, and waiting for it
        // does not wait for the chunk loads and stores in flight
        typedef const __attribute__((address_space(4))) int32_t* const_i32_ptr;
        k.pos = FUSED ? *((const_i32_ptr)(uintptr_t)p.positions + b) + l : p.start_pos + l;
        k.row_ok = !FUSED || (k.pos >= 0 && k.pos < p.Lmax);   // cache row exists
        k.xq = (short*)p.x + (int64_t)tok * p.H * p.D;
        k.xk = FUSED ? (const short*)p.k + (int64_t)tok * p.Hkv * p.D : nullptr;
        k.xv = FUSED ? (const short*)p.v + (int64_t)tok * p.Hkv * p.D : nullptr;
        k.ck = FUSED && !Q8 ? (short*)p.k_cache + (int64_t)b * p.c0 + (int64_t)k.pos * p.c2 : nullptr;
        k.cv = FUSED && !Q8 ? (short*)p.v_cache + (int64_t)b * p.c0 + (int64_t)k.pos * p.c2 : nullptr;
        k.qk = Q8 ? (char*)p.k_cache + (int64_t)b * p.c0 + (int64_t)k.pos * p.c2 : nullptr;
        k.qv = Q8 ? (char*)p.v_cache + (int64_t)b * p.c0 + (int64_t)k.pos * p.c2 : nullptr;
        return k;
    };
    // Which chunk of a token a thread works on, and where that chunk sits inside the token's q, k, v and cache rows,
    // does not depend on the token: a slot is worked out once (integer divisions) and then only added to the token's
    // base pointers.  sect is the same for all lanes of a wave; elem is the chunk's first element inside its head.
    enum { Q_ROT = 0, K_ROT = 1, K_COPY = 2, V_COPY = 3 };
    struct Slot {
        int sect; uint32_t where;     // where: head << 16 | elem, all ones = no chunk for this lane
        MA_DEV bool valid() const { return where != ~0u; }
        MA_DEV int hd() const { return (int)(where >> 16); }
        MA_DEV int elem() const { return (int)(where & 0xffffu); }
    };
    auto place = [&](int t) __attribute__((always_inline)) {
        const int w0 = __builtin_amdgcn_readfirstlane(t) & ~63;   // a wave's lanes hold 64 consecutive numbers
        int sect = Q_ROT, begin = 0, n = n_q, per = cph, elem0 = 0;
        if (FUSED && w0 >= k_begin) {
            if (w0 < kt_begin) { sect = K_ROT; begin = k_begin; n = n_kr; }
            else if (w0 < v_begin) { sect = K_COPY; begin = kt_begin; n = n_kt; per = tail; elem0 = p.rd; }
            else { sect = V_COPY; begin = v_begin; n = n_v; per = p.D >> 3; }
        }
        const int i = t - begin, hd = i / per;
        return Slot{sect, i < n ? (uint32_t)hd << 16 | (uint32_t)(elem0 + 8 * (i - hd * per)) : ~0u};
    };
    auto live = [&](const Token& k, const Slot& s) __attribute__((always_inline)) {
        return s.valid() && (s.sect == Q_ROT || k.row_ok);
    };
    // chunks in flight per thread and buffer: a NeoX rotary chunk is two 16-byte pieces, so half as many
    constexpr int UN = STYLE == ROPE_IL ? 4 : 2;
    struct Buffer { s16x8 lo[UN], hi[UN]; };
    struct Slots { Slot s[UN]; };
    auto place_batch = [&](int t0) __attribute__((always_inline)) {
        Slots b;
#pragma unroll
        for (int u = 0; u < UN; ++u) b.s[u] = place(t0 + u * kRopeThreads);
        return b;
    };
    auto request = [&](const Token& k, const Slots slots, Buffer& buf) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const Slot s = slots.s[u];
            const short* src = (s.sect == Q_ROT ? k.xq : s.sect == V_COPY ? k.xv : k.xk) + (s.hd() * p.D + s.elem());
            buf.lo[u] = s16x8{0, 0, 0, 0, 0, 0, 0, 0};
            if (live(k, s)) buf.lo[u] = load_once<STREAM>(reinterpret_cast<const s16x8*>(src));
            buf.hi[u] = buf.lo[u];
            if (STYLE == ROPE_NEOX && live(k, s) && s.sect <= K_ROT) buf.hi[u] = load_once<STREAM>(reinterpret_cast<const s16x8*>(src + half_rd));
        }
    };
    // 8 values to their place: as they are, or (Q8_0 cache) quantised with the block's three other lanes
    auto put = [&](short* dst, char* crow, int elem, s16x8 val) __attribute__((always_inline)) {
        if (Q8 && crow) {
            float f[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) f[j] = T::to_float(val[j]);
            uint16_t d_bits;
            const uint2 q = quant8_q8_0(f, d_bits);
            store_q8_piece(crow + (elem >> 5) * 34, elem & 31, q, d_bits);
        } else {
            store_once<STREAM>(reinterpret_cast<s16x8*>(dst), val);
        }
    };
    auto finish = [&](const Token& k, const Slots slots, const Buffer& buf, int parity) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const Slot s = slots.s[u];
            if (!live(k, s)) continue;
            short* dst = nullptr; char* crow = nullptr;
            const int elem = s.elem(), chunk = elem >> 3;
            if (s.sect == Q_ROT) dst = k.xq + (s.hd() * p.D + elem);
            else if (Q8) crow = (s.sect == V_COPY ? k.qv : k.qk) + s.hd() * p.c1;
            else dst = (s.sect == V_COPY ? k.cv : k.ck) + (s.hd() * p.c1 + elem);
            s16x8 a = buf.lo[u];
            if (s.sect <= K_ROT) {
                if (STYLE == ROPE_IL) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const f32x2 cs = tab[parity][4 * chunk + j];
                        const uint32_t pk = rotate_pair<T>(cs[0], cs[1], a[2 * j], a[2 * j + 1]);
                        a[2 * j] = (short)(pk & 0xffffu);
                        a[2 * j + 1] = (short)(pk >> 16);
                    }
                } else {
                    s16x8 b = buf.hi[u];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const f32x2 cs = tab[parity][8 * chunk + j];
                        const uint32_t pk = rotate_pair<T>(cs[0], cs[1], a[j], b[j]);
                        a[j] = (short)(pk & 0xffffu);
                        b[j] = (short)(pk >> 16);
                    }
                    put(dst + half_rd, crow, elem + half_rd, b);
                }
            }
            put(dst, crow, elem, a);
        }
    };
    // the slots of a thread's first batch of chunks, and the frequency of the table entry it computes
    const Slots first = place_batch(tid);
    // One token: its table (the token's first chunks are already on their way in `buf`), the one barrier of the
    // token (the next token writes the other table), rotate and store, then any further batches of chunks.
    auto one_token = [&](const Token& k, Buffer& buf, int parity) __attribute__((always_inline)) {
        if (tab_i >= 0) tab[parity][tab_i] = table_entry(freq[tab_i], k.pos);
        __syncthreads();
        finish(k, first, buf, parity);
        for (int t0 = tid + UN * kRopeThreads; t0 < n_all; t0 += UN * kRopeThreads) {
            const Slots more = place_batch(t0);
            request(k, more, buf);
            finish(k, more, buf, parity);
        }
    };

    const int stride = gridDim.x;
    int tok = blockIdx.x;
    if (tok >= tokens) return;
    if (!(FUSED && Q8)) {
        // One token at a time.  With every compute unit holding 7-8 workgroups the memory system is saturated as it
        // is: fetching a token ahead costs registers, hence resident workgroups, and is 2-6 % slower, in place as
        // into fp16 caches.
        Buffer buf;
        int parity = 0;
        for (; tok < tokens; tok += stride, parity ^= 1) {
            const Token k = token_at(tok);
            request(k, first, buf);
            one_token(k, buf, parity);
        }
        return;
    }
    // Into Q8_0 caches the quantiser's dependent chain makes a token long, and fetching ahead pays (+7 %): two
    // tokens per trip, so that the two buffers are fixed registers; while a token is rotated, quantised and stored,
    // the first chunks of the workgroup's next token are already in flight in the other buffer.
    Buffer buf_a, buf_b;
    Token cur = token_at(tok);
    request(cur, first, buf_a);
    for (;;) {
        const bool more_b = tok + stride < tokens;
        const Token nxt = token_at(more_b ? tok + stride : tok);
        if (more_b) request(nxt, first, buf_b);
        one_token(cur, buf_a, 0);
        if (!more_b) break;
        tok += stride;
        const bool more_a = tok + stride < tokens;
        cur = token_at(more_a ? tok + stride : tok);
        if (more_a) request(cur, first, buf_a);
        one_token(nxt, buf_b, 1);
        if (!more_a) break;
        tok += stride;
    }
}

// Any even rotary_dim, any alignment: one thread per (token, head, pair), as the reference launches it.
template <class T, int STYLE>
__global__ __launch_bounds__(kRopeThreads) void rope_scalar_kernel(const RopeParams p) {
    const int half_rd = p.rd >> 1;
    const int64_t total = (int64_t)p.B * p.L * p.H * half_rd;
    for (int64_t i = (int64_t)blockIdx.x * kRopeThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kRopeThreads) {
        const int pair = (int)(i % half_rd);
        const int64_t row = i / half_rd;                 // (token, head)
        const int l = (int)((row / p.H) % p.L);
        const f32x2 cs = table_entry(p.inv_freq[pair], p.start_pos + l);
        short* xh = (short*)p.x + row * p.D;
        const int i0 = STYLE == ROPE_IL ? 2 * pair : pair, i1 = STYLE == ROPE_IL ? 2 * pair + 1 : pair + half_rd;
        const uint32_t pk = rotate_pair<T>(cs[0], cs[1], xh[i0], xh[i1]);
        xh[i0] = (short)(pk & 0xffffu);
        xh[i1] = (short)(pk >> 16);
    }
}

// ------------------------------------------------------------------------------------------------
// The producer with the per-head RMS normalisation of q and k in front of the rotation (reference: the optional
// rmsnorm(q), rmsnorm(k) calls between the QKV projection and the rotary embedding, src/minfer/core.py:224-230).
// A head is in registers between its load and its rotation anyway, so the normalisation costs no memory traffic:
// G = D/8 neighbouring lanes hold one head (a 16-byte chunk each), sum their squares with lane exchanges, scale,
// round to the element type exactly as rmsnorm_rows_kernel does (same grouping, same order of additions: the
// result equals rmsnorm followed by the producer bit for bit), then rotate.  The NeoX partner of a chunk sits in
// another lane of the group and is fetched by lane exchange.  v is copied (or quantised) as in the plain producer.
// ------------------------------------------------------------------------------------------------
struct NormRopeParams {
    RopeParams r;
    const void* wq; const void* wk;   // per-head weights [D]; null = that tensor is not normalised
    float eps, inv_dim;
};

// A lane's value from another lane of its row of 16 (quad permutation, mirror or rotation, chosen by CTRL).
template <int CTRL> MA_DEV uint32_t row_exchange(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}
// ss summed over the G lanes of a head.  The partners are those of `ss += __shfl_xor(ss, m)`, m = 1, 2, 4, 8 (after
// the quad steps every lane of a quad holds the same sum, so mirroring the half row or the row reads the same value
// as the lane m away), the additions therefore the same, at a few cycles each instead of a trip through the LDS.
template <int G> MA_DEV float sum_over_head(float ss) {
    ss += __builtin_bit_cast(float, row_exchange<0xB1>(__builtin_bit_cast(uint32_t, ss)));            // lanes 1 0 3 2
    ss += __builtin_bit_cast(float, row_exchange<0x4E>(__builtin_bit_cast(uint32_t, ss)));            // lanes 2 3 0 1
    ss += __builtin_bit_cast(float, row_exchange<0x141>(__builtin_bit_cast(uint32_t, ss)));           // half row mirrored
    if (G == 16) ss += __builtin_bit_cast(float, row_exchange<0x140>(__builtin_bit_cast(uint32_t, ss)));   // row mirrored
    return ss;
}

template <class T, int STYLE, bool Q8, int G, bool STREAM>
__global__ __launch_bounds__(kRopeThreads) void rope_norm_append_kernel(const NormRopeParams np) {
    const RopeParams& p = np.r;
    __shared__ f32x2 tab[2][kMaxPairs];
    static_assert(G == 8 || G == 16, "a head is 8 or 16 chunks");
    constexpr int D = 8 * G;
    constexpr int UN = 4;             // chunks in flight per thread and batch
    const int tid = threadIdx.x;
    const int half_rd = p.rd >> 1;
    const int heads = p.H + 2 * p.Hkv;
    const int units = heads * G;
    const int batches = (units + UN * kRopeThreads - 1) / (UN * kRopeThreads);
    const int c = tid & (G - 1);      // the lane's chunk inside its head: elements 8c..8c+7
    const int rot_chunks = STYLE == ROPE_IL ? p.rd >> 3 : p.rd >> 4;   // IL: chunks that rotate; NeoX: chunks per half
    // NeoX: chunk c < rd/16 holds the x0 of pairs 8c.., chunk c + rd/16 their x1
    const bool neox_lo = STYLE == ROPE_NEOX && c < rot_chunks;
    const bool neox_hi = STYLE == ROPE_NEOX && c >= rot_chunks && c < 2 * rot_chunks;
    const int partner = neox_lo ? (int)(threadIdx.x & 63) + rot_chunks : neox_hi ? (int)(threadIdx.x & 63) - rot_chunks : (int)(threadIdx.x & 63);
    const bool partner_half_row = STYLE == ROPE_NEOX && G == 16 && rot_chunks == 8;   // the partner is the lane 8 further round the row
    const bool rotates = STYLE == ROPE_IL ? c < rot_chunks : (neox_lo || neox_hi);
    const int pair0 = STYLE == ROPE_IL ? 4 * c : 8 * (neox_hi ? c - rot_chunks : c);   // first table entry of the chunk
    const double my_freq = tid < half_rd ? p.inv_freq[tid] : 0.0;
    const s16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    float wq32[8], wk32[8];           // the lane's share of the two weights
    {
        const s16x8 wq8 = np.wq ? *reinterpret_cast<const s16x8*>((const short*)np.wq + 8 * c) : zero8;
        const s16x8 wk8 = np.wk ? *reinterpret_cast<const s16x8*>((const short*)np.wk + 8 * c) : zero8;
#pragma unroll
        for (int j = 0; j < 8; ++j) { wq32[j] = T::to_float(wq8[j]); wk32[j] = T::to_float(wk8[j]); }
    }
    const int tokens = p.B * p.L;
    const uintptr_t kc_addr = (uintptr_t)p.k_cache, vc_addr = (uintptr_t)p.v_cache;   // chosen per lane by value, not by a table in memory

    // the chunks of batch `bi` of a token: unit (bi*UN + u)*threads + tid is chunk c of head unit / G
    // (the token's position comes back: it is read through the scalar cache, once per token)
    auto request = [&](int tok, int bi, s16x8 (&x)[UN]) __attribute__((always_inline)) {
        const int b = __builtin_amdgcn_readfirstlane(tok / p.L), l = tok - b * p.L;
        // positions is an input nothing writes: read it as constant memory, so that the load is a scalar one and
        // waiting for it does not wait for the chunk loads in flight
        typedef const __attribute__((address_space(4))) int32_t* const_i32_ptr;
        const int pos = *((const_i32_ptr)(uintptr_t)p.positions + b) + l;
        const bool row_ok = pos >= 0 && pos < p.Lmax;
        const uintptr_t xq = (uintptr_t)((const short*)p.x + (int64_t)tok * p.H * D);
        const uintptr_t xk = (uintptr_t)((const short*)p.k + (int64_t)tok * p.Hkv * D);
        const uintptr_t xv = (uintptr_t)((const short*)p.v + (int64_t)tok * p.Hkv * D);
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int unit = (bi * UN + u) * kRopeThreads + tid;
            const int hd = (int)((unsigned)unit / G);
            x[u] = zero8;
            if (unit < units) {
                const bool from_k = hd >= p.H, from_v = hd >= p.H + p.Hkv;
                const uintptr_t src = from_v ? xv : from_k ? xk : xq;
                const int local = hd - (from_v ? p.H + p.Hkv : from_k ? p.H : 0);
                if (!from_k || row_ok) x[u] = load_once<STREAM>(reinterpret_cast<const s16x8*>((const short*)src + local * D + 8 * c));
            }
        }
        return pos;
    };

    // The work is the sequence of (token, batch) items of this workgroup; the chunks of the next item are requested
    // before the current one is worked on.
    int tok = blockIdx.x, bi = 0, parity = 0;
    if (tok >= tokens) return;
    s16x8 x[UN], xn[UN];
    int pos = request(tok, 0, x), npos = 0;
    float cs_c[8], cs_s[8];           // the lane's cos and signed sin: out = cos * mine + sin * partner's (NeoX)
    while (tok < tokens) {
        const int b = __builtin_amdgcn_readfirstlane(tok / p.L);
        const bool row_ok = pos >= 0 && pos < p.Lmax;
        short* xq = (short*)p.x + (int64_t)tok * p.H * D;
        const int64_t crow = (int64_t)b * p.c0 + (int64_t)pos * p.c2;   // elements, or bytes into Q8_0 caches
        int ntok = tok, nbi = bi + 1;
        if (nbi == batches) { ntok = tok + gridDim.x; nbi = 0; }
        if (ntok < tokens) npos = request(ntok, nbi, xn);
        if (bi == 0) {   // the token's table; one barrier per token (the next token writes the other buffer)
            if (tid < half_rd) tab[parity][tid] = table_entry(my_freq, pos);
            __syncthreads();
            if (rotates) {
#pragma unroll
                for (int j = 0; j < (STYLE == ROPE_IL ? 4 : 8); ++j) {
                    const f32x2 e = tab[parity][pair0 + j];
                    cs_c[j] = e[0];
                    cs_s[j] = neox_lo ? -e[1] : e[1];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int unit = (bi * UN + u) * kRopeThreads + tid;
            if (__builtin_amdgcn_readfirstlane(unit) >= units) continue;   // units grow with the lane: none of this wave's is real
            const bool valid = unit < units;
            const int hd = (int)((unsigned)unit / G);
            const bool is_q = valid && hd < p.H, is_k = valid && hd >= p.H && hd < p.H + p.Hkv;
            // normalise: every lane takes part in the exchanges, the result is used by q and k heads only
            const float ss = sum_over_head<G>(sum_sq8<T>(x[u]));
            const float sc = rsqrtf(ss * np.inv_dim + np.eps);
            s16x8 a = x[u];
            if ((is_q && np.wq) || (is_k && np.wk)) {
                uint32_t r[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float w0 = is_q ? wq32[2 * j] : wk32[2 * j], w1 = is_q ? wq32[2 * j + 1] : wk32[2 * j + 1];
                    r[j] = T::pack2(T::to_float(a[2 * j]) * w0 * sc, T::to_float(a[2 * j + 1]) * w1 * sc);
                }
                uint4 v4; v4.x = r[0]; v4.y = r[1]; v4.z = r[2]; v4.w = r[3];
                a = __builtin_bit_cast(s16x8, v4);
            }
            // rotate
            if (STYLE == ROPE_NEOX) {
                const uint4 mine = __builtin_bit_cast(uint4, a);
                uint4 other;
                if (partner_half_row) {
                    other.x = row_exchange<0x128>(mine.x); other.y = row_exchange<0x128>(mine.y);
                    other.z = row_exchange<0x128>(mine.z); other.w = row_exchange<0x128>(mine.w);
                } else {
                    other.x = __shfl(mine.x, partner); other.y = __shfl(mine.y, partner);
                    other.z = __shfl(mine.z, partner); other.w = __shfl(mine.w, partner);
                }
                const s16x8 o = __builtin_bit_cast(s16x8, other);
                if ((is_q || is_k) && rotates) {
                    uint32_t r[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        r[j] = T::pack2(rotate_one<T>(cs_c[2 * j], cs_s[2 * j], a[2 * j], o[2 * j]),
                                        rotate_one<T>(cs_c[2 * j + 1], cs_s[2 * j + 1], a[2 * j + 1], o[2 * j + 1]));
                    uint4 v4; v4.x = r[0]; v4.y = r[1]; v4.z = r[2]; v4.w = r[3];
                    a = __builtin_bit_cast(s16x8, v4);
                }
            } else if ((is_q || is_k) && rotates) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t pk = rotate_pair<T>(cs_c[j], cs_s[j], a[2 * j], a[2 * j + 1]);
                    a[2 * j] = (short)(pk & 0xffffu);
                    a[2 * j + 1] = (short)(pk >> 16);
                }
            }
            // store
            if (is_q) {
                store_once<STREAM>(reinterpret_cast<s16x8*>(xq + hd * D + 8 * c), a);
            } else if (valid && row_ok) {
                const int g = is_k ? hd - p.H : hd - p.H - p.Hkv;
                void* cache = (void*)(is_k ? kc_addr : vc_addr);
                if (Q8) {
                    float f[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) f[j] = T::to_float(a[j]);
                    uint16_t d_bits;
                    const uint2 q8 = quant8_q8_0(f, d_bits);
                    store_q8_piece((char*)cache + crow + (int64_t)g * p.c1 + (c >> 2) * 34, 8 * (c & 3), q8, d_bits);
                } else {
                    store_once<STREAM>(reinterpret_cast<s16x8*>((short*)cache + crow + (int64_t)g * p.c1 + 8 * c), a);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) x[u] = xn[u];
        if (nbi == 0) parity ^= 1;
        tok = ntok; bi = nbi; pos = npos;
    }
}

static int fill_rope(RopeParams& p, int dtype, int style, int64_t B, int64_t L, int64_t H, int64_t D,
                     int64_t rotary_dim, double freq_base, const char* op) {
    char msg[160];
    auto bad = [&](const char* what) {
        snprintf(msg, sizeof msg, "%s: %s", op, what);
        return fail(MINFER_ATTN_EINVAL, msg);
    };
    if (dtype != MINFER_ATTN_F16 && dtype != MINFER_ATTN_BF16) return bad("dtype must be MINFER_ATTN_F16 or MINFER_ATTN_BF16");
    if (style != ROPE_IL && style != ROPE_NEOX) return bad("style must be MINFER_ROPE_INTERLEAVED or MINFER_ROPE_NEOX");
    if (B < 0 || L < 0 || H < 0 || D <= 0) return bad("negative size");
    if (rotary_dim < 0 || rotary_dim > D) return bad("rotary_dim must be in 0..head_dim");
    if (rotary_dim % 2 != 0) return bad("rotary_dim must be even");
    if (rotary_dim > 2 * kMaxPairs) return bad("rotary_dim > 256 unsupported");
    if (!(freq_base > 0.0)) return bad("freq_base must be positive");
    if (B * L > 0x7fffffffLL || H > 65535 || D > 65535 || H * D > 0x7fffffffLL) return bad("problem too large");
    p.B = (int)B; p.L = (int)L; p.H = (int)H; p.D = (int)D; p.rd = (int)rotary_dim;
    for (int i = 0; i < rotary_dim / 2; ++i) p.inv_freq[i] = pow(freq_base, -2.0 * i / (double)rotary_dim);
    return MINFER_ATTN_OK;
}

static bool vector_ok(int style, int64_t D, int64_t rd) {
    return D % 8 == 0 && rd % (style == ROPE_IL ? 8 : 16) == 0;
}

template <bool FUSED, bool Q8, bool STREAM>
static void launch_rope_as(int dtype, int style, const RopeParams& p, int grid, hipStream_t stream) {
    if (dtype == MINFER_ATTN_F16) {
        if (style == ROPE_IL) hipLaunchKernelGGL((rope_kernel<F16, ROPE_IL, FUSED, Q8, STREAM>), dim3(grid), dim3(kRopeThreads), 0, stream, p);
        else hipLaunchKernelGGL((rope_kernel<F16, ROPE_NEOX, FUSED, Q8, STREAM>), dim3(grid), dim3(kRopeThreads), 0, stream, p);
    } else {
        if (style == ROPE_IL) hipLaunchKernelGGL((rope_kernel<BF16, ROPE_IL, FUSED, Q8, STREAM>), dim3(grid), dim3(kRopeThreads), 0, stream, p);
        else hipLaunchKernelGGL((rope_kernel<BF16, ROPE_NEOX, FUSED, Q8, STREAM>), dim3(grid), dim3(kRopeThreads), 0, stream, p);
    }
}

template <bool FUSED, bool Q8 = false>
static int launch_rope(int dtype, int style, const RopeParams& p, hipStream_t stream) {
    const int tokens = p.B * p.L;
    const int grid = std::min(tokens, 256 * 16);
    // distinct bytes the launch touches: q's rotary part (in place), and for the producer k, v and their cache rows
    int64_t touched = (int64_t)tokens * p.H * p.rd * 2;
    if (FUSED) touched += (int64_t)tokens * p.Hkv * p.D * 2 * (Q8 ? 3 : 4);
    if (touched > kStreamBytes) launch_rope_as<FUSED, Q8, true>(dtype, style, p, grid, stream);
    else launch_rope_as<FUSED, Q8, false>(dtype, style, p, grid, stream);
    return check_launch("rope_kernel");
}

}  // namespace minfer_attn

using namespace minfer_attn;

MINFER_ATTN_EXPORT int minfer_rope(int dtype, int style, void* x, int64_t B, int64_t L, int64_t H, int64_t D,
                                   int64_t rotary_dim, int64_t start_pos, double freq_base, void* stream_v) {
    clear_error();
    RopeParams p{};
    if (int rc = fill_rope(p, dtype, style, B, L, H, D, rotary_dim, freq_base, "rope")) return rc;
    if (!x) return fail(MINFER_ATTN_EINVAL, "rope: x is null");
    if (start_pos < 0 || start_pos + L > 0x7fffffffLL) return fail(MINFER_ATTN_EINVAL, "rope: positions must fit in int32");
    if (B == 0 || L == 0 || H == 0 || rotary_dim == 0) return MINFER_ATTN_OK;
    p.x = x; p.start_pos = (int)start_pos;
    hipStream_t stream = (hipStream_t)stream_v;
    if (vector_ok(style, D, rotary_dim) && aligned16(x)) return launch_rope<false>(dtype, style, p, stream);

    const int64_t pairs = B * L * H * (rotary_dim / 2);
    const int grid = (int)std::min<int64_t>((pairs + kRopeThreads - 1) / kRopeThreads, 256 * 32);
    if (dtype == MINFER_ATTN_F16) {
        if (style == ROPE_IL) hipLaunchKernelGGL((rope_scalar_kernel<F16, ROPE_IL>), dim3(grid), dim3(kRopeThreads), 0, stream, p);
        else hipLaunchKernelGGL((rope_scalar_kernel<F16, ROPE_NEOX>), dim3(grid), dim3(kRopeThreads), 0, stream, p);
    } else {
        if (style == ROPE_IL) hipLaunchKernelGGL((rope_scalar_kernel<BF16, ROPE_IL>), dim3(grid), dim3(kRopeThreads), 0, stream, p);
        else hipLaunchKernelGGL((rope_scalar_kernel<BF16, ROPE_NEOX>), dim3(grid), dim3(kRopeThreads), 0, stream, p);
    }
    return check_launch("rope_scalar_kernel");
}

MINFER_ATTN_EXPORT int minfer_rope_kv_append(int dtype, int style, void* q, const void* k, const void* v,
                                             const int32_t* positions, void* k_cache, void* v_cache, int64_t B,
                                             int64_t L, int64_t Hq, int64_t Hkv, int64_t D, int64_t Lmax,
                                             int64_t cache_stride_b, int64_t cache_stride_h, int64_t cache_stride_row,
                                             int64_t rotary_dim, double freq_base, void* stream_v) {
    clear_error();
    RopeParams p{};
    if (int rc = fill_rope(p, dtype, style, B, L, Hq, D, rotary_dim, freq_base, "rope_kv_append")) return rc;
    if (!q || !k || !v || !positions || !k_cache || !v_cache) return fail(MINFER_ATTN_EINVAL, "rope_kv_append: null pointer");
    if (Hkv <= 0 || Hkv > 65535 || Lmax < 0 || Lmax > 0x7fffffffLL) return fail(MINFER_ATTN_EINVAL, "rope_kv_append: bad n_kv_heads or Lmax");
    if (!vector_ok(style, D, rotary_dim))
        return fail(MINFER_ATTN_EINVAL, "rope_kv_append: head_dim must be a multiple of 8 and rotary_dim of 8 (interleaved) or 16 (NeoX)");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(k_cache) || !aligned16(v_cache))
        return fail(MINFER_ATTN_EINVAL, "rope_kv_append: tensors must be 16-byte aligned");
    if (cache_stride_b % 8 || cache_stride_h % 8 || cache_stride_row % 8 || cache_stride_b < 0 || cache_stride_h < 0 || cache_stride_row < 0)
        return fail(MINFER_ATTN_EINVAL, "rope_kv_append: cache strides must be non-negative multiples of 8 elements");
    if (B == 0 || L == 0) return MINFER_ATTN_OK;
    p.x = q; p.k = k; p.v = v; p.k_cache = k_cache; p.v_cache = v_cache; p.positions = positions;
    p.Hkv = (int)Hkv; p.Lmax = (int)Lmax;
    p.c0 = cache_stride_b; p.c1 = cache_stride_h; p.c2 = cache_stride_row;
    return launch_rope<true>(dtype, style, p, (hipStream_t)stream_v);
}

MINFER_ATTN_EXPORT int minfer_rope_kv_append_q8_0(int dtype, int style, void* q, const void* k, const void* v,
                                                  const int32_t* positions, void* k_cache, void* v_cache, int64_t B,
                                                  int64_t L, int64_t Hq, int64_t Hkv, int64_t D, int64_t Lmax,
                                                  int64_t cache_stride_b, int64_t cache_stride_h, int64_t rotary_dim,
                                                  double freq_base, void* stream_v) {
    clear_error();
    RopeParams p{};
    if (int rc = fill_rope(p, dtype, style, B, L, Hq, D, rotary_dim, freq_base, "rope_kv_append_q8_0")) return rc;
    if (!q || !k || !v || !positions || !k_cache || !v_cache) return fail(MINFER_ATTN_EINVAL, "rope_kv_append_q8_0: null pointer");
    if (Hkv <= 0 || Hkv > 65535 || Lmax < 0 || Lmax > 0x7fffffffLL) return fail(MINFER_ATTN_EINVAL, "rope_kv_append_q8_0: bad n_kv_heads or Lmax");
    // a block's 32 values must sit in four neighbouring 8-value chunks of one kind
    if (D % 32 != 0 || rotary_dim % (style == ROPE_IL ? 32 : 64) != 0)
        return fail(MINFER_ATTN_EINVAL, "rope_kv_append_q8_0: head_dim must be a multiple of 32 and rotary_dim of 32 (interleaved) or 64 (NeoX)");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v)) return fail(MINFER_ATTN_EINVAL, "rope_kv_append_q8_0: q, k and v must be 16-byte aligned");
    if (((uintptr_t)k_cache | (uintptr_t)v_cache) & 1u) return fail(MINFER_ATTN_EINVAL, "rope_kv_append_q8_0: caches must be 2-byte aligned");
    if (cache_stride_b % 2 || cache_stride_h % 2 || cache_stride_b < 0 || cache_stride_h < 0)
        return fail(MINFER_ATTN_EINVAL, "rope_kv_append_q8_0: cache strides must be non-negative even byte counts");
    if (B == 0 || L == 0) return MINFER_ATTN_OK;
    p.x = q; p.k = k; p.v = v; p.k_cache = k_cache; p.v_cache = v_cache; p.positions = positions;
    p.Hkv = (int)Hkv; p.Lmax = (int)Lmax;
    p.c0 = cache_stride_b; p.c1 = cache_stride_h; p.c2 = D / 32 * 34;
    return launch_rope<true, true>(dtype, style, p, (hipStream_t)stream_v);
}

namespace minfer_attn {
template <class T, int STYLE, bool Q8>
static void launch_norm_append_as(const NormRopeParams& np, int D, bool stream_hint, int grid, hipStream_t stream) {
#define MINFER_NORM_APPEND(G, STREAM) \
    hipLaunchKernelGGL((rope_norm_append_kernel<T, STYLE, Q8, G, STREAM>), dim3(grid), dim3(kRopeThreads), 0, stream, np)
    if (D == 128) { if (stream_hint) MINFER_NORM_APPEND(16, true); else MINFER_NORM_APPEND(16, false); }
    else { if (stream_hint) MINFER_NORM_APPEND(8, true); else MINFER_NORM_APPEND(8, false); }
#undef MINFER_NORM_APPEND
}
}  // namespace minfer_attn

MINFER_ATTN_EXPORT int minfer_rope_kv_append_norm(int dtype, int style, int cache_type, void* q, const void* k, const void* v,
                                                  const void* wq_norm, const void* wk_norm, double eps,
                                                  const int32_t* positions, void* k_cache, void* v_cache, int64_t B,
                                                  int64_t L, int64_t Hq, int64_t Hkv, int64_t D, int64_t Lmax,
                                                  int64_t cache_stride_b, int64_t cache_stride_h, int64_t cache_stride_row,
                                                  int64_t rotary_dim, double freq_base, void* stream_v) {
    clear_error();
    NormRopeParams np{};
    RopeParams& p = np.r;
    if (int rc = fill_rope(p, dtype, style, B, L, Hq, D, rotary_dim, freq_base, "rope_kv_append_norm")) return rc;
    const bool q8 = cache_type == MINFER_Q8_0;
    if (!q8 && cache_type != dtype)
        return fail(MINFER_ATTN_EINVAL, "rope_kv_append_norm: cache_type must be the activations' dtype or MINFER_Q8_0");
    if (!q || !k || !v || !positions || !k_cache || !v_cache) return fail(MINFER_ATTN_EINVAL, "rope_kv_append_norm: null pointer");
    if (!(eps >= 0.0)) return fail(MINFER_ATTN_EINVAL, "rope_kv_append_norm: eps must be non-negative");
    if (Hkv <= 0 || Hkv > 65535 || Lmax < 0 || Lmax > 0x7fffffffLL) return fail(MINFER_ATTN_EINVAL, "rope_kv_append_norm: bad n_kv_heads or Lmax");
    if (D != 64 && D != 128) return fail(MINFER_ATTN_EINVAL, "rope_kv_append_norm: head_dim must be 64 or 128");
    if (!vector_ok(style, D, rotary_dim))
        return fail(MINFER_ATTN_EINVAL, "rope_kv_append_norm: rotary_dim must be a multiple of 8 (interleaved) or 16 (NeoX)");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || (wq_norm && !aligned16(wq_norm)) || (wk_norm && !aligned16(wk_norm)))
        return fail(MINFER_ATTN_EINVAL, "rope_kv_append_norm: q, k, v and the norm weights must be 16-byte aligned");
    if (q8) {
        if (((uintptr_t)k_cache | (uintptr_t)v_cache) & 1u) return fail(MINFER_ATTN_EINVAL, "rope_kv_append_norm: Q8_0 caches must be 2-byte aligned");
        if (cache_stride_b % 2 || cache_stride_h % 2 || cache_stride_b < 0 || cache_stride_h < 0 || cache_stride_row != D / 32 * 34)
            return fail(MINFER_ATTN_EINVAL, "rope_kv_append_norm: Q8_0 cache strides are even byte counts, rows dense (D/32 * 34 bytes)");
    } else {
        if (!aligned16(k_cache) || !aligned16(v_cache)) return fail(MINFER_ATTN_EINVAL, "rope_kv_append_norm: caches must be 16-byte aligned");
        if (cache_stride_b % 8 || cache_stride_h % 8 || cache_stride_row % 8 || cache_stride_b < 0 || cache_stride_h < 0 || cache_stride_row < 0)
            return fail(MINFER_ATTN_EINVAL, "rope_kv_append_norm: cache strides must be non-negative multiples of 8 elements");
    }
    if (B == 0 || L == 0) return MINFER_ATTN_OK;
    p.x = q; p.k = k; p.v = v; p.k_cache = k_cache; p.v_cache = v_cache; p.positions = positions;
    p.Hkv = (int)Hkv; p.Lmax = (int)Lmax;
    p.c0 = cache_stride_b; p.c1 = cache_stride_h; p.c2 = cache_stride_row;
    np.wq = wq_norm; np.wk = wk_norm; np.eps = (float)eps; np.inv_dim = (float)(1.0 / (double)D);
    const int tokens = p.B * p.L;
    const int grid = std::min(tokens, 256 * 16);
    const int64_t touched = (int64_t)tokens * (2 * Hq * D * 2 + Hkv * D * 2 * (q8 ? 3 : 4));   // q in place (whole heads), k, v, cache rows
    const bool hint = touched > kStreamBytes;
    hipStream_t stream = (hipStream_t)stream_v;
    if (dtype == MINFER_ATTN_F16) {
        if (style == ROPE_IL) { if (q8) launch_norm_append_as<F16, ROPE_IL, true>(np, (int)D, hint, grid, stream); else launch_norm_append_as<F16, ROPE_IL, false>(np, (int)D, hint, grid, stream); }
        else { if (q8) launch_norm_append_as<F16, ROPE_NEOX, true>(np, (int)D, hint, grid, stream); else launch_norm_append_as<F16, ROPE_NEOX, false>(np, (int)D, hint, grid, stream); }
    } else {
        if (style == ROPE_IL) { if (q8) launch_norm_append_as<BF16, ROPE_IL, true>(np, (int)D, hint, grid, stream); else launch_norm_append_as<BF16, ROPE_IL, false>(np, (int)D, hint, grid, stream); }
        else { if (q8) launch_norm_append_as<BF16, ROPE_NEOX, true>(np, (int)D, hint, grid, stream); else launch_norm_append_as<BF16, ROPE_NEOX, false>(np, (int)D, hint, grid, stream); }
    }
    return check_launch("rope_norm_append_kernel");
}
