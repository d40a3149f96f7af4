// Types and device helpers shared by the gfx950 MFMA kernels (bf16 and fp16 elements).
#pragma once

#include "sa2_common.h"

namespace sa2 {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float floatx16;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;

constexpr int BQ = 32;       // queries per workgroup
constexpr int TJ = 32;       // keys per LDS tile
constexpr int NTHREADS = 256;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
constexpr float LOG2_EPS = -26.575424759098897f;   // log2(1e-8)
constexpr float LN_EPS = -18.420680743952367f;     // ln(1e-8)

__device__ __forceinline__ float bf16_lo(uint32_t x) { return __uint_as_float(x << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t x) { return __uint_as_float(x & 0xffff0000u); }
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// The 16-bit element type of a call: how its pairs unpack to fp32, its MFMA and its
// two-element dot product.  WEIGHT_LIMIT bounds the row sum of one tile of softmax weights
// in the forward's fast kernel: above it the block is recomputed by the repair kernel (bf16
// shares fp32's exponent range; an fp16 weight must stay below 65504).
struct ElemBF16 {
    typedef __bf16 scalar;
    typedef bf16x8 x8;
    typedef bf16x2 x2;
    static constexpr int DTYPE = SA2_BF16;
    static constexpr float WEIGHT_LIMIT = 1.0e30f;
    static __device__ __forceinline__ float lo(uint32_t x) { return __uint_as_float(x << 16); }
    static __device__ __forceinline__ float hi(uint32_t x) { return __uint_as_float(x & 0xffff0000u); }
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        union { __bf16 h[2]; uint32_t u; } v;
        v.h[0] = (__bf16)a;
        v.h[1] = (__bf16)b;
        return v.u;
    }
    static __device__ __forceinline__ floatx16 mfma(x8 a, x8 b, floatx16 c, int, int, int) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float dot2(x2 a, x2 b, float c, bool) {
        return __builtin_amdgcn_fdot2_f32_bf16(a, b, c, false);
    }
};
struct ElemF16 {
    typedef _Float16 scalar;
    typedef f16x8 x8;
    typedef f16x2 x2;
    static constexpr int DTYPE = SA2_F16;
    static constexpr float WEIGHT_LIMIT = 3.0e4f;
    static __device__ __forceinline__ float lo(uint32_t x) {
        union { uint32_t u; _Float16 h[2]; } v;
        v.u = x;
        return (float)v.h[0];
    }
    static __device__ __forceinline__ float hi(uint32_t x) {
        union { uint32_t u; _Float16 h[2]; } v;
        v.u = x;
        return (float)v.h[1];
    }
    static __device__ __forceinline__ uint32_t pack(float a, float b) {
        union { _Float16 h[2]; uint32_t u; } v;
        v.h[0] = (_Float16)a;
        v.h[1] = (_Float16)b;
        return v.u;
    }
    static __device__ __forceinline__ floatx16 mfma(x8 a, x8 b, floatx16 c, int, int, int) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float dot2(x2 a, x2 b, float c, bool) {
        return __builtin_amdgcn_fdot2(a, b, c, false);
    }
};

// Exchange between lane l and lane l^32 (one VALU op): returns the partner's value.
__device__ __forceinline__ float other_half(float x) {
    const unsigned u = __float_as_uint(x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    // r[0] holds the low half's value in every lane, r[1] the high half's
    return __uint_as_float((threadIdx.x & 32) ? r[0] : r[1]);
}

// Tiles in LDS (written by direct global->LDS loads, or by wavefronts in the same order) keep
// groups of RPW rows together: within a group the 16-byte chunk c of row q sits at byte
// (c * RPW + q) * 16, groups lie GROUP bytes apart.  Row operand reads (16 bytes per lane) and the
// transposed reads below are both free of bank conflicts in this layout.
//
// Transposed MFMA operand out of such a tile: eight 16-bit elements of one COLUMN of the tile, as
// the A/B operand of a 32x32x16 MFMA whose contraction index runs over the tile's rows.  For a
// 32-column block, lane l gets column l%32 and, for its half h = l/32, the rows
//   16*ks + 4*h + {0,1,2,3}   and   16*ks + 8 + 4*h + {0,1,2,3}
// which is exactly the k-slot order in which a 32x32 accumulator tile (rows = those rows) hands
// its values to the other operand.  Uses the LDS transpose read: within 16 lanes, lane s supplies
// the address of row s/4, columns 4*(s%4)..+3, and lane i receives column i of those four rows.
// lds_group_column_lane_offset() is the lane part of the address (bytes, for ks = 0); the reads
// take the sum of the tile's LDS byte address, the block's offset (block * 64 * RPW) and that lane
// part, so that inside a loop the address is one add and everything else sits in immediate offsets.
template <int RPW, int GROUP>
__device__ __forceinline__ uint32_t lds_group_column_lane_offset(int lane) {
    const int grp = lane >> 4, s = lane & 15;
    const int rr = 4 * (grp >> 1) + (s >> 2);            // row within the 8-row slice
    const int cc = 16 * (grp & 1) + 4 * (s & 3);         // column within the 32-column block
    return (uint32_t)((rr / RPW) * GROUP + ((cc / 8) * RPW + rr % RPW) * 16 + (cc % 8) * 2);
}
// The operand itself (compiler-visible reads): `addr` = tile + lane part + block * 64 * RPW; k-step ks
// takes rows 16*ks .. 16*ks+15.  CFG supplies row_off(r), the byte offset of row r.
template <class CFG, class X8 = bf16x8>
__device__ __forceinline__ X8 lds_group_column_operand_at(uint32_t addr, int ks) {
    typedef short v4s __attribute__((ext_vector_type(4)));
    typedef v4s __attribute__((address_space(3)))* lds_v4s;
    const uint32_t o0 = ks ? (uint32_t)CFG::row_off(16) : 0u, o1 = ks ? (uint32_t)CFG::row_off(24) : (uint32_t)CFG::row_off(8);
    const v4s a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)(uintptr_t)(addr + o0));
    const v4s b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)(uintptr_t)(addr + o1));
    union { v4s h[2]; X8 v; } u;
    u.h[0] = a;
    u.h[1] = b;
    return u.v;
}
// The same operand read in two phases for loops that keep direct global->LDS loads in
// flight: the compiler would wait for every outstanding vector-memory operation before a
// transpose-read builtin, so the reads are issued as opaque instructions and the wait for
// their results is placed by hand (lds_settle) before the first use.
typedef short lds_half_operand __attribute__((ext_vector_type(4)));
template <int OFF_A, int OFF_B>
__device__ __forceinline__ void lds_tr_issue(uint32_t addr, lds_half_operand& a, lds_half_operand& b) {
    asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
                 : "=&v"(a), "=&v"(b)
                 : "v"(addr), "n"(OFF_A), "n"(OFF_B));
}
// all LDS reads issued so far have returned; the operands named here are only used afterwards
__device__ __forceinline__ void lds_settle(lds_half_operand (&x)[16]) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7]),
                   "+v"(x[8]), "+v"(x[9]), "+v"(x[10]), "+v"(x[11]), "+v"(x[12]), "+v"(x[13]), "+v"(x[14]), "+v"(x[15]));
}
__device__ __forceinline__ void lds_settle(lds_half_operand (&x)[4]) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]));
}
__device__ __forceinline__ void lds_settle(lds_half_operand (&x)[8]) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7]));
}
template <class X8 = bf16x8>
__device__ __forceinline__ X8 lds_join(const lds_half_operand& a, const lds_half_operand& b) {
    union { lds_half_operand h[2]; X8 v; } u;
    u.h[0] = a;
    u.h[1] = b;
    return u.v;
}
// NW consecutive 32-bit words (2*NW 16-bit elements) from / to a NW*4-byte aligned address
template <int NW>
__device__ __forceinline__ void load_words(const void* p, uint32_t (&w)[NW]) {
    static_assert(NW == 1 || NW == 2 || NW == 4, "one 4-, 8- or 16-byte access");
    if constexpr (NW == 4) {
        const uint4 x = *(const uint4*)p;
        w[0] = x.x; w[1] = x.y; w[2] = x.z; w[3] = x.w;
    } else if constexpr (NW == 2) {
        const uint2 x = *(const uint2*)p;
        w[0] = x.x; w[1] = x.y;
    } else {
        w[0] = *(const uint32_t*)p;
    }
}
template <int NW>
__device__ __forceinline__ void store_words(void* p, const uint32_t (&w)[NW]) {
    static_assert(NW == 1 || NW == 2 || NW == 4, "one 4-, 8- or 16-byte access");
    if constexpr (NW == 4) *(uint4*)p = make_uint4(w[0], w[1], w[2], w[3]);
    else if constexpr (NW == 2) *(uint2*)p = make_uint2(w[0], w[1]);
    else *(uint32_t*)p = w[0];
}
// LDS byte address of a pointer into shared memory
__device__ __forceinline__ uint32_t lds_address(const void* p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}
template <class X8 = bf16x8>
__device__ __forceinline__ X8 lds_read_x8(uint32_t addr) {
    return *(const X8 __attribute__((address_space(3)))*)(uintptr_t)addr;
}
// Row operand reads as opaque instructions, like lds_tr_issue: r[FIRST + i] = the 16 bytes at
// addr + (FIRST + i) * STEP for i < N.  The compiler's own wait-count bookkeeping does not see
// them (nor the transposed reads), so it neither waits for them nor makes a wait for one of its
// own loads cover them; lds_wait<PENDING>() names the registers that may be used once at most
// PENDING of the LDS reads issued so far are still outstanding (they return in order).
template <int FIRST, int N, int STEP, class X8>
__device__ __forceinline__ void lds_row_issue(uint32_t addr, X8* r) {
    if constexpr (N > 0) {
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(r[FIRST]) : "v"(addr), "n"(FIRST * STEP));
        lds_row_issue<FIRST + 1, N - 1, STEP>(addr, r);
    }
}
template <int PENDING, class X8>
__device__ __forceinline__ void lds_wait(X8 (&x)[1]) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(x[0]) : "n"(PENDING));
}
template <int PENDING, class X8>
__device__ __forceinline__ void lds_wait(X8 (&x)[2]) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(x[0]), "+v"(x[1]) : "n"(PENDING));
}
template <int PENDING, class X8>
__device__ __forceinline__ void lds_wait(X8 (&x)[4]) {
    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]) : "n"(PENDING));
}
template <int PENDING, class X8>
__device__ __forceinline__ void lds_wait(X8 (&x)[8]) {
    asm volatile("s_waitcnt lgkmcnt(%8)"
                 : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]), "+v"(x[4]), "+v"(x[5]), "+v"(x[6]), "+v"(x[7])
                 : "n"(PENDING));
}

}  // namespace
}  // namespace sa2
