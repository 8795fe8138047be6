// Device helpers shared by the fast kernels: wave-uniform table loads and the per-lane
// payload loads of the prepared layout (wave_layout.h).
#pragma once

#include <type_traits>
#include <utility>

#include "wave_layout.h"

namespace bitsmoe {

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef const u32x2 __attribute__((address_space(1)))* gptr_u32x2;
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));

__device__ inline float gload_half(gptr<__half> p) {
    const uint16_t bits = *reinterpret_cast<gptr<uint16_t>>(p);
    return __half2float(__ushort_as_half(bits));
}

// Calls f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>): an unrolled loop whose
// index is a compile-time constant (register-array indices must be static).
template <class F, int... Q>
__device__ inline void static_for(F&& f, std::integer_sequence<int, Q...>) {
    (f(std::integral_constant<int, Q>{}), ...);
}

// The index is wave-uniform at every call site; readfirstlane tells the compiler so (scalar
// registers, scalar branches, scalar-base addressing downstream).
__device__ inline FastSlab load_fast_slab(const FastSlab* __restrict__ tab, int idx) {
    const i32x4 v = *reinterpret_cast<const i32x4*>(tab + idx);
    return FastSlab{__builtin_amdgcn_readfirstlane(v[0]), __builtin_amdgcn_readfirstlane(v[1]),
                    __builtin_amdgcn_readfirstlane(v[2]), __builtin_amdgcn_readfirstlane(v[3])};
}

// The fields of an expert's record held in scalar registers from HERE on.  They are first used behind the routing scan's
// workgroup barriers; loads from tables the kernel only reads may be moved, and left alone the compiler moves them down
// to those uses, where each is one more dependent round trip in front of the first payload request.  Called after
// everything else the start-up needs has been requested.
__device__ __forceinline__ void hold_fast_expert(FastExpert& fe) {
    uint64_t p0 = (uint64_t)fe.payload, p1 = (uint64_t)fe.scale, p2 = (uint64_t)fe.s, p3 = (uint64_t)fe.rank_idx,
             p4 = (uint64_t)fe.scale_s;
    asm volatile("" : "+s"(p0), "+s"(p1), "+s"(p2), "+s"(p3), "+s"(p4), "+s"(fe.num_slabs), "+s"(fe.uniform_bits));
    fe.payload = (const uint32_t*)p0;
    fe.scale = (const __half*)p1;
    fe.s = (const __half*)p2;
    fe.rank_idx = (const int32_t*)p3;
    fe.scale_s = (const __half*)p4;
}

// The words of one wavefront's column-block pair for one (slab, tile) block: 2-bit {nb0, nb1};
// 4-bit {nb0 j0, nb0 j1, nb1 j0, nb1 j1}; 3-bit {low nb0, low nb1, high nb0, high nb1}.
// `blk` is wave-uniform, `unit` = pair*64 + lane and `hi_unit` are 32-bit lane offsets.
__device__ __forceinline__ void load_pair_role0(gptr<uint32_t> blk, int bits, uint32_t unit, uint32_t hi_unit, uint32_t (&w)[4]) {
    if (bits == 4) {
        const u32x4 v = *reinterpret_cast<gptr_u32x4>(blk + unit * 4u);
        w[0] = v[0]; w[1] = v[1]; w[2] = v[2]; w[3] = v[3];
    } else {
        const u32x2 v = *reinterpret_cast<gptr_u32x2>(blk + unit * 2u);
        w[0] = v[0]; w[1] = v[1]; w[2] = 0; w[3] = 0;
        if (bits == 3) {
            const u32x2 h = *reinterpret_cast<gptr_u32x2>(blk + 512u + hi_unit);
            w[2] = h[0]; w[3] = h[1];
        }
    }
}

struct Block16 {   // up to 16 payload words of one lane for one (slab, tile) block
    uint32_t w[16];
};

// role 1 loads: 2-bit 8 words [nb][h], 4-bit 16 words [nb][m], 3-bit 13 words (five code pairs each)
template <int W>
__device__ __forceinline__ void load_block_role1(gptr<uint32_t> blk, int lane, Block16& b) {
    gptr_u32x4 p = reinterpret_cast<gptr_u32x4>(blk + (W == 4 ? lane * 16 : W == 3 ? lane * 4 : lane * 8));
    u32x4 v0 = p[0], v1, v2 = {0, 0, 0, 0}, v3 = {0, 0, 0, 0};
    if constexpr (W == 3) {
        v1 = p[64];       // (+256 words)
        v2 = p[128];
        v3[0] = blk[768 + lane];
    } else {
        v1 = p[1];
    }
    if constexpr (W == 4) {
        v2 = p[2];
        v3 = p[3];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        b.w[i] = v0[i];
        b.w[4 + i] = v1[i];
        b.w[8 + i] = v2[i];
        b.w[12 + i] = v3[i];
    }
}

}  // namespace bitsmoe
