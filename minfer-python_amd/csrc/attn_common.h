// Shared device helpers for the gfx950 attention kernels: element-type traits over the CDNA4
// MFMA builtins, wave64 cross-lane helpers, direct global->LDS copies and LDS swizzles.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace minfer_attn {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 h16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 h16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 h16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 b16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 b16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 b16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define MA_DEV __device__ __forceinline__

// 16-bit element types.  Operand fragments travel as raw 16-bit lanes (s16x8 / s16x4) and are
// bit-cast at the MFMA call, so one kernel body serves both.
struct F16 {
    // D[32x32] += A[32x16] * B[16x32]; lane l holds A row l%32, k = 8*(l/32)+0..7 (B alike, by
    // column); D register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32.
    static MA_DEV f32x16 mfma32(s16x8 a, s16x8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h16x8, a),
                                                      __builtin_bit_cast(h16x8, b), c, 0, 0, 0);
    }
    // D[16x16] += A[16x32] * B[32x16]; lane l holds A row l%16, k = 8*(l/16)+0..7; D register r
    // of lane l is row 4*(l/16) + r, column l%16.
    static MA_DEV f32x4 mfma16(s16x8 a, s16x8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h16x8, a),
                                                      __builtin_bit_cast(h16x8, b), c, 0, 0, 0);
    }
    // D[16x16] += A[16x16] * B[16x16]; lane l holds A row l%16, k = 4*(l/16)+0..3.
    static MA_DEV f32x4 mfma16k16(s16x4 a, s16x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(h16x4, a),
                                                     __builtin_bit_cast(h16x4, b), c, 0, 0, 0);
    }
    static MA_DEV uint32_t pack2(float lo, float hi) {  // round-to-nearest-even pair
        f32x2 f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, h16x2));
    }
    static MA_DEV float to_float(short bits) { return (float)__builtin_bit_cast(_Float16, bits); }
    // x * f elementwise, computed in fp32 and rounded back (round-to-nearest-even)
    static MA_DEV s16x8 scale8(s16x8 x, float f) {
        const h16x8 v = __builtin_bit_cast(h16x8, x);
        h16x8 r;
#pragma unroll
        for (int i = 0; i < 8; ++i) r[i] = (_Float16)__builtin_fmaf((float)v[i], f, 0.f);   // one mixed-precision fma each
        return __builtin_bit_cast(s16x8, r);
    }
    // acc + lo + hi of a packed pair, in fp32: sums exactly the rounded values the MFMA consumes
    static MA_DEV float add_pair(uint32_t pair, float acc) {
        const h16x2 ones = {(_Float16)1.f, (_Float16)1.f};
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(h16x2, pair), ones, acc, false);
    }
};

struct BF16 {
    static MA_DEV f32x16 mfma32(s16x8 a, s16x8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(b16x8, a),
                                                       __builtin_bit_cast(b16x8, b), c, 0, 0, 0);
    }
    static MA_DEV f32x4 mfma16(s16x8 a, s16x8 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b16x8, a),
                                                       __builtin_bit_cast(b16x8, b), c, 0, 0, 0);
    }
    static MA_DEV f32x4 mfma16k16(s16x4 a, s16x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
    }
    static MA_DEV uint32_t pack2(float lo, float hi) {
        f32x2 f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, b16x2));
    }
    static MA_DEV float to_float(short bits) {
        return __builtin_bit_cast(float, (uint32_t)(uint16_t)bits << 16);
    }
    static MA_DEV s16x8 scale8(s16x8 x, float f) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = pack2(to_float(x[2 * i]) * f, to_float(x[2 * i + 1]) * f);
        uint4 u; u.x = w[0]; u.y = w[1]; u.z = w[2]; u.w = w[3];
        return __builtin_bit_cast(s16x8, u);
    }
    static MA_DEV float add_pair(uint32_t pair, float acc) {
        const b16x2 ones = {(__bf16)1.f, (__bf16)1.f};
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b16x2, pair), ones, acc, false);
    }
};

typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void glb_cvoid;

// Copies 16 bytes per lane from global memory straight into LDS without passing through VGPRs.
// `lds_base` must be wave-uniform: lane i's 16 bytes land at lds_base + 16*i, whatever address
// the lane read from.  Completion is tracked by vmcnt, and it is the caller who waits
// (s_waitcnt vmcnt + barrier) before anyone reads the destination: the copy is issued from
// inline assembly so that the compiler does not serialise every later LDS read behind it.
MA_DEV void copy16_global_to_lds(const void* src, void* lds_base) {
    const uint32_t dst = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_void*)lds_base);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(dst), "v"(src)
                 : "memory", "m0");
}
// Same, with the source given as a wave-uniform base plus a 32-bit unsigned per-lane byte offset, which
// costs no vector ALU work when the offset is loop-invariant.
//
// A vector-memory instruction must not read a scalar register earlier than five instructions after a vector
// instruction (readfirstlane) wrote it.  The compiler keeps that distance for the instructions it emits but cannot see
// into an asm statement, which itself puts two instructions between.  BASE_FRESH = false is for bases that are scalar
// values long before the call (a tile loop's row base); BASE_FRESH = true (three more idle issue slots) is for a base
// computed from per-wave values right before the call.  build.py scans the generated code of every kernel for a copy
// that reads a scalar register written by a vector instruction fewer than five instructions earlier and fails on one.
template <bool BASE_FRESH = false>
MA_DEV void copy16_global_to_lds(const void* uniform_base, uint32_t lane_byte_offset, void* lds_base) {
    const uint32_t dst = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_void*)lds_base);
    const uint64_t b = (uint64_t)(uintptr_t)uniform_base;
    // readfirstlane returns a signed int: go through uint32_t, or a low word with bit 31 set would be
    // sign-extended into the high word of the address
    const uint64_t sb = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32)) << 32) |
                        (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    if (BASE_FRESH)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(dst), "v"(lane_byte_offset), "s"(sb)
                     : "memory", "m0");
    else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(dst), "v"(lane_byte_offset), "s"(sb)
                     : "memory", "m0");
}

// 32-bit LDS address of a __shared__ object, and reads at such an address plus a compile-time offset
// (which the instruction carries as an immediate, so one address register serves many reads).
MA_DEV uint32_t lds_addr(const void* p) { return (uint32_t)(uintptr_t)(lds_void*)p; }
MA_DEV s16x8 lds_read_b128(uint32_t addr, int imm) {
    typedef __attribute__((address_space(3))) s16x8 lds_s16x8;
    return *(const lds_s16x8*)(uintptr_t)(addr + imm);
}

// Waits until at most N of this wave's vector-memory operations (global loads and global->LDS
// copies, which retire in order) are outstanding.  Also a compiler barrier, so LDS reads of the
// copied data cannot be hoisted above the wait.
template <int N> MA_DEV void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// LDS transpose read: within each group of 16 lanes, lanes 4e..4e+3 together address row e of a
// 4x16 tile of 16-bit elements (4 contiguous elements per lane); lane i receives column i, i.e.
// {row0[i], row1[i], row2[i], row3[i]}.
MA_DEV s16x4 lds_read_tr16(const void* lds_ptr) {
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)lds_ptr);
}
MA_DEV s16x4 lds_read_tr16(uint32_t addr, int imm) {
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(uintptr_t)(addr + imm));
}

// Value of x held by lane (l ^ 32), combined with the lane's own by max / sum.  (The maximum of the two values of a lane
// swap as one instruction: fmaxf on them costs three, the compiler quieting each possible signalling NaN first.)
MA_DEV float max2(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
MA_DEV float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
MA_DEV float max_across_halves(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return max2(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
// The same over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (the 16-lane groups of a 16x16 MFMA block's column): rows
// 1 and 3 of one operand are swapped with rows 0 and 2 of the other, then the halves.
MA_DEV float max_across_quads(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return max_across_halves(max2(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1])));
}
MA_DEV float sum_across_halves(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}

MA_DEV float sum_across_quads(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return sum_across_halves(__builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]));
}

MA_DEV float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Inclusive prefix sum of x over the lanes of a wave.
MA_DEV int wave_inclusive_scan(int x, int lane) {
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(x, d);
        if (lane >= d) x += up;
    }
    return x;
}

// Loads and stores of bytes that a kernel touches once (cache rows being streamed, rows of a normalisation):
// marked non-temporal, so that the caches between the compute units and HBM do not keep the lines.  On this chip
// that alone raises the HBM throughput of a streaming kernel by 10-15 %.
template <class V> MA_DEV V stream_load(const V* p) { return __builtin_nontemporal_load(p); }
template <class V> MA_DEV void stream_store(V* p, V v) { __builtin_nontemporal_store(v, p); }
// The same with the choice made per launch (template argument): see kStreamBytes on the host side.
template <bool STREAM, class V> MA_DEV V load_once(const V* p) { return STREAM ? __builtin_nontemporal_load(p) : *p; }
template <bool STREAM, class V> MA_DEV void store_once(V* p, V v) { if (STREAM) __builtin_nontemporal_store(v, p); else *p = v; }

// Pieces of the RMS normalisation that the normalisation kernels and the rope producer that normalises heads share
// (the same code on both sides, so their results agree bit for bit): the sum of squares of 8 elements, and
// x * w * scale rounded once to the element type.
template <class T> MA_DEV float sum_sq8(s16x8 v) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) { const float f = T::to_float(v[i]); s += f * f; }
    return s;
}
template <class T> MA_DEV s16x8 scale8w(s16x8 v, s16x8 w, float sc) {
    uint32_t r[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        r[i] = T::pack2(T::to_float(v[2 * i]) * T::to_float(w[2 * i]) * sc, T::to_float(v[2 * i + 1]) * T::to_float(w[2 * i + 1]) * sc);
    uint4 u; u.x = r[0]; u.y = r[1]; u.z = r[2]; u.w = r[3];
    return __builtin_bit_cast(s16x8, u);
}

MA_DEV int wave_id() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

}  // namespace minfer_attn
