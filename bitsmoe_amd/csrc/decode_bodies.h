// Device code shared by the small-batch ("decode") kernels: constants, the wave-parallel searches
// over expert_offsets, the per-block MFMA bodies of the gate/up and down projections, and the two
// item bodies (one gate/up tile walked over slab groups; one down slab per wavefront) that both
// the one-launch-per-projection kernels and the persistent kernel run.
#pragma once

#include <type_traits>
#include <utility>

#include "fast_helpers.h"

#ifndef BITSMOE_TL_DOWN_STAMP
#define BITSMOE_TL_DOWN_STAMP(i) do {} while (0)      // (time stamps of the timeline build, forward_decode.hip)
#endif

namespace bitsmoe {
constexpr int GU_STRIDE = GU_SLABS * SLAB_ROWS + 8;  // 16-bit elements; +8 staggers LDS banks
constexpr int DN_SLABS_PER_WG = 4;                 // one slab per wavefront
constexpr int MAX_A = 16;                          // assignments per MFMA pass
constexpr int ZROWS = 2;                           // assignment rows of G / U the down kernel's z build fetches together
constexpr int ZROWS_WIDE = 6;                      // ... where z is so large that only three workgroups fit a CU anyway
constexpr int ZSUM_STRIDE = 16;                    // tiles per assignment row of the down kernel's z sums (I <= 1920)

// With few assignments most experts are idle; launching a workgroup per (expert, ...) then
// costs more than the work.  The kernels can instead be launched over `slots` and let every
// workgroup find the slot-th ACTIVE expert (non-empty assignment range) itself: one
// wave-parallel pass over expert_offsets.  Returns -1 when fewer experts are active.
__device__ inline int nth_active_expert(const int32_t* __restrict__ expert_offsets, int E, int A, int slot, int lane) {
    int found = -1;
    for (int e0 = 0; e0 < E && found < 0; e0 += 64) {
        const int e = e0 + lane;
        bool active = false;
        if (e < E) active = min(expert_offsets[e + 1], A) > max(expert_offsets[e], 0);
        const uint64_t mask = __ballot(active);
        const int count = __popcll(mask);
        if (slot < count) {
            const int rank = __popcll(mask & ((1ull << lane) - 1ull));
            const uint64_t hit = __ballot(active && rank == slot);
            found = e0 + (int)__builtin_ctzll(hit);
        }
        slot -= count;
    }
    return __builtin_amdgcn_readfirstlane(found);
}

// With many assignments an expert is served in chunks of 16; walking the chunks of a popular
// expert one after the other inside a workgroup makes that expert the long pole of the launch.
// The kernels can instead be launched over chunk slots: slot -> (expert, chunk) in expert order,
// again by one wave-parallel pass over expert_offsets.  Returns expert -1 past the last chunk.
struct ChunkRef {
    int expert, chunk;
};
// v of lane i + (lanes selected by the DPP control whose source lane exists ? v of the source lane : 0)
template <int CTRL, int ROW_MASK = 0xf>
__device__ inline int dpp_add(int v) {
    return v + __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xf, false);
}
// Inclusive prefix sum over the 64 lanes with data-parallel-primitive moves (no LDS round trips):
// shifts by 1, 2, 4, 8 inside the rows of 16 lanes, then the row totals broadcast forward.
__device__ inline int wave_inclusive_scan(int v) {
    v = dpp_add<0x111>(v);          // row_shr:1
    v = dpp_add<0x112>(v);          // row_shr:2
    v = dpp_add<0x114>(v);          // row_shr:4
    v = dpp_add<0x118>(v);          // row_shr:8
    v = dpp_add<0x142, 0xa>(v);     // row_bcast:15 into rows 1 and 3
    v = dpp_add<0x143, 0xc>(v);     // row_bcast:31 into rows 2 and 3
    return v;
}
__device__ inline ChunkRef nth_chunk(const int32_t* __restrict__ expert_offsets, int E, int A, int slot, int lane) {
    int found_e = -1, found_c = 0;
    for (int e0 = 0; e0 < E && found_e < 0; e0 += 64) {
        const int e = e0 + lane;
        int chunks = 0;
        if (e < E) {
            const int b = max(expert_offsets[e], 0), en = min(expert_offsets[e + 1], A);
            chunks = en > b ? (en - b + 15) >> 4 : 0;
        }
        const int incl = wave_inclusive_scan(chunks);
        const int total = __builtin_amdgcn_readlane(incl, 63);
        if (slot < total) {
            const uint64_t hit = __ballot(slot >= incl - chunks && slot < incl);    // exactly one lane
            const int l = (int)__builtin_ctzll(hit);
            found_e = e0 + l;
            found_c = slot - __builtin_amdgcn_readlane(incl - chunks, l);
        }
        slot -= total;
    }
    return ChunkRef{__builtin_amdgcn_readfirstlane(found_e), __builtin_amdgcn_readfirstlane(found_c)};
}

// ------------------------------------------------------------------------- where assignments come from
// The kernels see an expert's assignments through one of two sources.  Tables: the routing tables the
// operator is given (token_indices / route_w in expert-sorted order, an expert's range from expert_offsets);
// assignment a is row a of the [A, I] intermediates.  Inline: the workgroup has found its expert's entries
// among the T * k routed (token, slot) pairs itself (inline_route); assignment j is then flat entry ent[j]
// = token * k + slot, which is also its row of the intermediates -- no routing kernel runs before the
// forward, and gate/up and down workgroups agree on the rows without any table in memory.
struct AssignTables {
    const int32_t* __restrict__ token_indices;
    const float* __restrict__ route_w;
    int A;
    __device__ __forceinline__ int token(int a) const { return token_indices[min(a, A - 1)]; }
    __device__ __forceinline__ int token_if(int a, bool ok) const { return ok ? token_indices[a] : -1; }
    __device__ __forceinline__ float weight_if(int a, bool ok) const { return ok ? route_w[a] : 0.0f; }
    __device__ __forceinline__ int row(int a) const { return a; }
};
constexpr int ROUTE_INLINE_MAX_FLAT = 1024;      // routed entries (tokens x top-k) a workgroup scans itself
constexpr int ROUTE_INLINE_MAX_ROWS = 256;       // assignments of one expert (at most one per token)
struct InlineRouteLds {
    uint16_t tok[ROUTE_INLINE_MAX_ROWS];
    uint16_t ent[ROUTE_INLINE_MAX_ROWS];
    int wave_sum[4];
};
struct AssignInline {
    const uint16_t* tok;       // LDS
    const uint16_t* ent;       // LDS
    const float* __restrict__ weights;      // [T * k] routing weights in entry order
    int n;
    __device__ __forceinline__ int token(int a) const { return tok[min(a, n - 1)]; }
    __device__ __forceinline__ int token_if(int a, bool ok) const { return ok ? (int)tok[a] : -1; }
    __device__ __forceinline__ float weight_if(int a, bool ok) const { return ok ? weights[ent[a]] : 0.0f; }
    __device__ __forceinline__ int row(int a) const { return ent[a]; }
};
__device__ __forceinline__ int routed_id(const void* __restrict__ selected, int ids_are_i64, int i) {
    return ids_are_i64 ? (int)reinterpret_cast<const int64_t*>(selected)[i] : reinterpret_cast<const int32_t*>(selected)[i];
}
// The entries of the expert with global id `gid` among selected[0 .. n_flat) (n_flat <= ROUTE_INLINE_MAX_FLAT,
// ids 32 or 64 bits wide), in entry order -- the order the routing kernel's stable sort gives
// (bitsmoe/models/base_block.py:258-289) -- written to `r`; returns their number (wave-uniform).  All 256
// threads call it; it contains two workgroup barriers.  Ids that belong to no packed expert match nothing.
// In two halves, so that a caller can put the requests for its other tables between the request for the ids and their
// first use (one round trip for all of them): inline_route_request, then inline_route_finish.
struct RouteIds {
    int ids[4];      // entries 4 tid .. 4 tid + 3 (the last entry again past the end)
};
__device__ __forceinline__ RouteIds inline_route_request(const void* __restrict__ selected, int ids_are_i64, int n_flat, int tid) {
    RouteIds q;
    const int base = 4 * tid;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int i = min(base + k, n_flat - 1);
        q.ids[k] = ids_are_i64 ? (int)reinterpret_cast<const int64_t*>(selected)[i] : reinterpret_cast<const int32_t*>(selected)[i];
    }
    return q;
}
// (the ids are in registers from here on, whatever the compiler would have liked to do with their loads)
__device__ __forceinline__ void hold_route_ids(RouteIds& q) {
    asm volatile("" : "+v"(q.ids[0]), "+v"(q.ids[1]), "+v"(q.ids[2]), "+v"(q.ids[3]));
}
__device__ inline int inline_route_finish(const RouteIds& q, int n_flat, int top_k, int gid, InlineRouteLds& r, int tid) {
    const int lane = tid & 63, wave = tid >> 6;
    const int base = 4 * tid;
    int count = 0;
    bool hit[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        hit[k] = base + k < n_flat && q.ids[k] == gid;
        count += hit[k] ? 1 : 0;
    }
    const int incl = wave_inclusive_scan(count);
    if (lane == 63) r.wave_sum[wave] = incl;
    __syncthreads();
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const int s = r.wave_sum[w];
        before += w < wave ? s : 0;
        total += s;
    }
    int pos = before + incl - count;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        if (hit[k] && pos < ROUTE_INLINE_MAX_ROWS) {
            r.tok[pos] = (uint16_t)((base + k) / top_k);
            r.ent[pos] = (uint16_t)(base + k);
        }
        pos += hit[k] ? 1 : 0;
    }
    __syncthreads();
    return __builtin_amdgcn_readfirstlane(min(total, ROUTE_INLINE_MAX_ROWS));
}
__device__ inline int inline_route(const void* __restrict__ selected, int ids_are_i64, int n_flat, int top_k, int gid,
                                   InlineRouteLds& r, int tid) {
    const RouteIds q = inline_route_request(selected, ids_are_i64, n_flat, tid);
    return inline_route_finish(q, n_flat, top_k, gid, r, tid);
}

constexpr int GRID_EXPERTS = 0;   // the expert coordinate of the grid is the expert
constexpr int GRID_ACTIVE = 1;    // ... counts active experts (nth_active_expert)
constexpr int GRID_CHUNKS = 2;    // ... counts 16-assignment chunks (nth_chunk)

// ------------------------------------------------------------------------------ gate / up
// One (slab, tile) block restricted to one column-block pair: 2 column blocks x 2 k-steps,
// plus the two MFMAs that accumulate the constant term.  The decoded registers hold
// 2^W + code / f_i (staggered fields, wave_layout.h); the activations carry f_i.
// CONST_TERM == false leaves the constant term to the caller (the walking kernel sums it while it
// stages the operand).
template <int W, bool CONST_TERM = true>
__device__ __forceinline__ void gateup_pair(const uint32_t (&w)[4], u32x4 a0, u32x4 a1, int upper, f32x4 (&acc)[2], f32x4& corr,
                                            const Masks3* m3 = nullptr) {
    if constexpr (CONST_TERM) {
        const u32x4 bc = offset0_regs<W>();
        corr = mfma16<false>(a0, bc, corr);
        corr = mfma16<false>(a1, bc, corr);
    }
#pragma unroll
    for (int nbl = 0; nbl < 2; ++nbl) {
        u32x4 b0, b1;
        if constexpr (W == 2) {
            b0 = decode0_lo<2>(w[nbl], 0);
            b1 = decode0_lo<2>(w[nbl], 1);
        } else if constexpr (W == 4) {
            b0 = decode0_fields4(w[2 * nbl]);
            b1 = decode0_fields4(w[2 * nbl + 1]);
        } else if (m3) {
            b0 = decode0_fields3(w[nbl], 0, w[2 + nbl], upper, *m3);
            b1 = decode0_fields3(w[nbl], 1, w[2 + nbl], upper, *m3);
        } else {
            b0 = decode0_fields3(w[nbl], 0, w[2 + nbl], upper);
            b1 = decode0_fields3(w[nbl], 1, w[2 + nbl], upper);
        }
        acc[nbl] = mfma16<false>(a0, b0, acc[nbl]);
        acc[nbl] = mfma16<false>(a1, b1, acc[nbl]);
    }
}

// Sum of v over the 64 lanes, valid in lane 63 (the data-parallel-primitive moves of wave_inclusive_scan).
template <int CTRL, int ROW_MASK = 0xf>
__device__ inline float dpp_add_f32(float v) {
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
__device__ inline float wave_sum_lane63(float v) {
    v = dpp_add_f32<0x111>(v);
    v = dpp_add_f32<0x112>(v);
    v = dpp_add_f32<0x114>(v);
    v = dpp_add_f32<0x118>(v);
    v = dpp_add_f32<0x142, 0xa>(v);
    v = dpp_add_f32<0x143, 0xc>(v);
    return v;
}
// sum over a lane's eight staged operands of operand * (what offset0_regs holds for its register)
template <int W>
__device__ __forceinline__ float const_term_partial(u32x4 staged) {
    typedef __fp16 h2v __attribute__((ext_vector_type(2)));
    const u32x4 bc = offset0_regs<W>();
    const uint32_t s0 = staged[0], s1 = staged[1], s2 = staged[2], s3 = staged[3];
    const uint32_t c0 = bc[0], c1 = bc[1], c2 = bc[2], c3 = bc[3];
    float p = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2v, s0), __builtin_bit_cast(h2v, c0), 0.0f, false);
    p = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2v, s1), __builtin_bit_cast(h2v, c1), p, false);
    p = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2v, s2), __builtin_bit_cast(h2v, c2), p, false);
    p = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2v, s3), __builtin_bit_cast(h2v, c3), p, false);
    return p;
}

template <bool BF16>
__device__ __forceinline__ u32x4 scaled_f16x8(u32x4 raw, u32x4 sc) {
    u32x4 out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t v = raw[i];
        if constexpr (BF16) {      // bf16 -> f16 is exact inside the f16 range (8 significant bits into 11)
            typedef __fp16 h2v __attribute__((ext_vector_type(2)));
            const h2v c = __builtin_amdgcn_cvt_pkrtz(__uint_as_float(v << 16), __uint_as_float(v & 0xFFFF0000u));
            v = __builtin_bit_cast(uint32_t, c);
        }
        out[i] = pk_mul_f16(v, sc[i]);
    }
    return out;
}


// ------------------------------------------------------- gate / up, one tile walked over slab groups
// One item of the gate/up projection for sets in which every expert is one affine run of equal-width
// slabs (bitsmoe_matset::all_affine) whose rank_idx maps every aligned run of eight rows to eight
// consecutive ranks (rank_chunked8): ONE 128-column tile `t` of expert matrix (fe, first) for the up to
// 16 assignments a0 .. a0 + n_a - 1, contracted over the slab groups [g_begin, g_end) with the tile's
// accumulators in registers.  256 threads = 4 wavefronts; wavefront p owns columns [32p, 32p+32).
//  * SPLIT == false: the item covers all groups, every output element has exactly one owner: plain
//    stores, no zero fill of G / U beforehand.  SPLIT == true: several items share an output tile
//    (few active experts: the contraction is split to fill the chip) and add with fp32 atomics into
//    cleared outputs.
//  * The payload stream of a wavefront runs on across the group boundaries (the block addresses
//    are affine in group, slab and tile).
//  * The activation operand of a group is built with 16-byte accesses: wavefront w serves the
//    assignments w, w+4, w+8, w+12 of the chunk; its lane l loads rows 8l .. 8l+7 of the group for
//    one assignment as ONE 16-byte load (eight consecutive ranks of the token's row), the eight
//    folded scales as another, multiplies and writes one 16-byte piece of the LDS operand.  Only
//    assignments that exist are touched (an MFMA output row depends on its own operand row
//    only, and rows past the chunk's assignments are never stored).
//  * Nothing a group needs is fetched when the group begins: the rank of a lane's rows arrives
//    two groups ahead, its scales one group ahead, and the activations of the wavefront's first
//    two assignments are requested right after the previous group's operand has been staged, so
//    they return behind that group's MFMAs.
// A token index out of range is clamped for the address: the down projection ignores such an
// assignment, whatever its G / U rows hold.
// `hs_all`: LDS, 2 * MAX_A * GU_STRIDE 16-bit elements; `cterm_lds`: LDS, MAX_A floats.  The caller
// guarantees that no wavefront still reads either when the item begins (a workgroup barrier).
// KEEP: the tile's sums are not stored; `keep[nbl]` receives them (the lane's rows a = 4*kg + j of column
// 32*pair + 16*nbl + n), for a caller that goes on with them in registers.
// MANY: the activations of the wavefront's third and fourth assignment (chunks of more than eight assignments) are
// requested ahead like those of the first two, instead of when they are staged (a memory round trip each, every group).
template <bool BF16, bool IDENT, int W, bool SPLIT, class AS, bool KEEP = false, bool MANY = false>
__device__ __forceinline__ void gateup_walk_item(gptr<uint32_t> payload, gptr<__half> scale_s, gptr<int32_t> rank_idx,
                                                 const FastSlab first, const uint16_t* __restrict__ h, int64_t ld,
                                                 const AS& as, int a0, int n_a, int T,
                                                 int I, int n_tiles, int t, int g_begin, int g_end, float* __restrict__ out,
                                                 uint16_t* __restrict__ hs_all, float* __restrict__ cterm_lds, int tid,
                                                 f32x4* __restrict__ keep = nullptr) {
    const int pair = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform
    const int lane = tid & 63;
    const int n = lane & 15, kg = lane >> 4;
    const uint32_t unit = (uint32_t)(pair * 64 + lane);
    const uint32_t hi_unit = (uint32_t)hi_index0(kg, n, 2 * pair);
    const int slab_words = n_tiles * 256 * W;       // payload words from one slab to the next
    Masks3 m3;
    if constexpr (W == 3) m3 = masks3_role0();
    int item_zero = 0;
    asm volatile("" : "+s"(item_zero));   // keeps this item's address arithmetic out of the caller's loop
    const int pack0 = first.pack_off + t * 256 * W + item_zero;

    uint32_t pw[GU_SLABS][4];   // slab q's block of the current group; refilled for the next group right after use
    auto issue = [&](auto q_c, int g) {
        constexpr int q = decltype(q_c)::value;
        load_pair_role0(payload + (uint32_t)(pack0 + (g * GU_SLABS + q) * slab_words), W, unit, hi_unit, pw[q]);
    };
    // the rows of this wavefront's assignments pair, pair + 4, pair + 8, pair + 12 (wave-uniform)
    // (indices clamped instead of branches, and all four requested before the first is used:
    // scalar loads in flight together)
    int tki[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) tki[i] = as.token(a0 + pair + 4 * i);
    // rows 8*lane .. 8*lane + 7 of group g: first logical rank, the f16 bits of their eight
    // scale * s * stagger factor (folded once when the set was prepared), the activations
    auto rank_at = [&](int g) {
        const int k = first.rank_off + g * (GU_SLABS * SLAB_ROWS) + 8 * lane;
        if constexpr (IDENT) return k;      // rank_idx[k] == k in every expert of both sets
        else return (int)rank_idx[k];
    };
    auto scale_at = [&](int g) {
        return *reinterpret_cast<gptr_u32x4>(
            scale_s + (uint32_t)(first.scale_off + ((g * GU_SLABS + (lane >> 3)) * n_tiles + t) * SLAB_ROWS + 8 * (lane & 7)));
    };
    const uint16_t* trow[4];
    auto act_at = [&](int i, int rank) { return *reinterpret_cast<const u32x4*>(trow[i] + rank); };
    uint16_t* hs = hs_all;
    // The decoded weights are 2^W + code / f, the levels (code - 2^(W-1)) / f: the difference times
    // the operand, summed over all rows, is the same for every column.  The wavefront that
    // stages an assignment sums it on the way (lane 63 holds the wave's total).
    float cterm[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    auto stage = [&](auto i_c, u32x4 raw, u32x4 sc) {
        constexpr int i = decltype(i_c)::value;
        const u32x4 v = scaled_f16x8<BF16>(raw, sc);
        *reinterpret_cast<u32x4*>(&hs[(pair + 4 * i) * GU_STRIDE + 8 * lane]) = v;
        cterm[i] += wave_sum_lane63(const_term_partial<W>(v));
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    int rank_cur = rank_at(g_begin);
    int rank_nxt = g_begin + 1 < g_end ? rank_at(g_begin + 1) : 0;
    u32x4 sc_cur = scale_at(g_begin);
    // (the token indices are first used here, behind the requests that do not depend on them)
#pragma unroll
    for (int i = 0; i < 4; ++i) trow[i] = h + (int64_t)min(max(__builtin_amdgcn_readfirstlane(tki[i]), 0), T - 1) * ld;
    u32x4 raw0 = {0, 0, 0, 0}, raw1 = {0, 0, 0, 0};
    // (requested whether or not the assignments exist -- a row of token 0 otherwise -- so that
    // the number of loads in flight does not depend on the path and the waits can be counted)
    raw0 = act_at(0, rank_cur);
    raw1 = act_at(1, rank_cur);
    [[maybe_unused]] u32x4 raw2 = {0, 0, 0, 0}, raw3 = {0, 0, 0, 0};
    if constexpr (MANY) {
        raw2 = act_at(2, rank_cur);
        raw3 = act_at(3, rank_cur);
    }
    // The payload of the first group is requested only now: loads return in order, so anything
    // requested behind it would be held back until it has arrived from HBM, and the first
    // operand could not be staged in the meantime.
    static_for([&](auto qc) { issue(qc, g_begin); }, std::make_integer_sequence<int, GU_SLABS>{});
    f32x4 acc[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
    f32x4 corr = {0, 0, 0, 0};
    // (MORE: another group follows -- compiled twice, so that the eight blocks of a group are
    // one straight run of code the compiler can schedule across)
    auto group_step = [&](auto more_c, int g) {
        constexpr bool more = decltype(more_c)::value;
        int rank_nxt2 = 0;
        if (g + 2 < g_end) rank_nxt2 = rank_at(g + 2);
        u32x4 sc_nxt = {0, 0, 0, 0};
        if constexpr (more) sc_nxt = scale_at(g + 1);
        // Group g writes copy g mod 2.  Its last readers (group g - 2) are done: every wavefront
        // passed the barrier of group g - 1 after its MFMAs of group g - 2.
        hs = hs_all + (g & 1) * (MAX_A * GU_STRIDE);
        if (pair < n_a) stage(I0{}, raw0, sc_cur);
        if (pair + 4 < n_a) stage(I1{}, raw1, sc_cur);
        if constexpr (MANY) {
            if (pair + 8 < n_a) stage(I2{}, raw2, sc_cur);
            if (pair + 12 < n_a) stage(I3{}, raw3, sc_cur);
        } else {
            if (pair + 8 < n_a) stage(I2{}, act_at(2, rank_cur), sc_cur);      // (fetched here, not ahead)
            if (pair + 12 < n_a) stage(I3{}, act_at(3, rank_cur), sc_cur);
        }
        __syncthreads();   // the operand is complete
        if constexpr (more) {
            raw0 = act_at(0, rank_nxt);
            raw1 = act_at(1, rank_nxt);
            if constexpr (MANY) {
                raw2 = act_at(2, rank_nxt);
                raw3 = act_at(3, rank_nxt);
            }
        }
        // (inside the one-kernel forward the scheduler otherwise sinks these two requests behind the payload
        // requests below -- loads return in order, the next operand would wait for the next group's payload)
        if constexpr (KEEP) __builtin_amdgcn_sched_barrier(0);
        const uint16_t* ap16 = &hs[n * GU_STRIDE + 16 * kg];
        static_for([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            const u32x4 a_lo = *reinterpret_cast<const u32x4*>(ap16 + q * SLAB_ROWS);
            const u32x4 a_hi = *reinterpret_cast<const u32x4*>(ap16 + q * SLAB_ROWS + 8);
            gateup_pair<W, false>(pw[q], a_lo, a_hi, n >> 3, acc, corr, W == 3 ? &m3 : nullptr);
            if constexpr (more) issue(qc, g + 1);
        }, std::make_integer_sequence<int, GU_SLABS>{});
        sc_cur = sc_nxt;
        rank_cur = rank_nxt;
        rank_nxt = rank_nxt2;
    };
    for (int g = g_begin; g + 1 < g_end; ++g) group_step(std::true_type{}, g);
    group_step(std::false_type{}, g_end - 1);
    // the constant terms of the chunk's assignments, from the wavefronts that staged them
    if (lane == 63) {
#pragma unroll
        for (int i = 0; i < 4; ++i) cterm_lds[pair + 4 * i] = cterm[i];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) corr[j] = cterm_lds[4 * kg + j];
    // remove the constant term; lane holds rows a = 4*kg + j of column 32*pair + 16*nbl + n
    if constexpr (KEEP) {
        keep[0] = acc[0] - corr;
        keep[1] = acc[1] - corr;
        return;
    }
#pragma unroll
    for (int nbl = 0; nbl < 2; ++nbl) {
        const int c = t * N_TILE + 32 * pair + 16 * nbl + n;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int a = 4 * kg + j;
            if (a < n_a && c < I) {
                const int64_t row = as.row(a0 + a);
                if constexpr (SPLIT)
                    atomicAdd(&out[row * I + c], acc[nbl][j] - corr[j]);
                else
                    out[row * I + c] = acc[nbl][j] - corr[j];
            }
        }
    }
}

// ------------------------------------- the same walk for experts whose slab groups differ in width
// An expert of a compressed checkpoint mixes widths (the leading ranks 4 bits, then 3, the bulk 2:
// bitsmoe/quant/packer.py:566-589); the prepared copy stores every group of GU_SLABS slabs at ONE width, so
// the walk only has to switch the decode between groups.  Everything but the payload is laid out alike
// for all widths (row g*512 + 8*lane of the rank table, scale row (g*8 + q) * n_tiles * 64): only the
// payload address and the field decode depend on the group's width.
// `grp_tab[g]` (LDS) = (width, payload word offset of the group's first slab) for g < n_groups; the caller
// fills it and puts a workgroup barrier behind it.
constexpr int WALK_MAX_GROUPS = 32;      // 16384 contraction rows
template <bool BF16, bool IDENT, bool SPLIT, class AS>
__device__ __forceinline__ void gateup_walk_item_mixed(gptr<uint32_t> payload, gptr<__half> scale_s, gptr<int32_t> rank_idx,
                                                       const int2* __restrict__ grp_tab, const uint16_t* __restrict__ h,
                                                       int64_t ld, const AS& as, int a0, int n_a,
                                                       int T, int I, int n_tiles, int t, int g_begin, int g_end,
                                                       float* __restrict__ out, uint16_t* __restrict__ hs_all,
                                                       float* __restrict__ cterm_lds, int tid) {
    const int pair = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform
    // (`lane` is given an opaque copy per group below: what a group's body derives from it -- block
    // offsets, LDS addresses, masks -- is then computed inside that body instead of being hoisted out of
    // the loop over groups for all nine bodies at once, which costs more registers than there are)
    int lane = tid & 63;
    int n = lane & 15, kg = lane >> 4;
    uint32_t unit = (uint32_t)(pair * 64 + lane);
    uint32_t hi_unit = (uint32_t)hi_index0(kg, n, 2 * pair);
    int item_zero = 0;
    asm volatile("" : "+s"(item_zero));   // keeps this item's address arithmetic out of the caller's loop
    auto group_rec = [&](int g) {      // (width, payload word offset of slab 8 g's block of tile t)
        const int2 v = grp_tab[g];
        const int w = __builtin_amdgcn_readfirstlane(v.x);
        return int2{w, __builtin_amdgcn_readfirstlane(v.y) + t * 256 * w + item_zero};
    };

    uint32_t pw[GU_SLABS][4];   // slab q's block of the current group; refilled for the next group right after use
    // slab q of a group of width w whose first block starts at word pack0
    auto issue_at = [&](auto q_c, int w, int pack0) {
        constexpr int q = decltype(q_c)::value;
        load_pair_role0(payload + (uint32_t)(pack0 + q * (n_tiles * 256 * w)), w, unit, hi_unit, pw[q]);
    };
    int tki[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) tki[i] = as.token(a0 + pair + 4 * i);
    auto rank_at = [&](int g) {
        const int k = g * (GU_SLABS * SLAB_ROWS) + 8 * lane;
        if constexpr (IDENT) return k;
        else return (int)rank_idx[k];
    };
    auto scale_at = [&](int g) {
        return *reinterpret_cast<gptr_u32x4>(
            scale_s + (uint32_t)(((g * GU_SLABS + (lane >> 3)) * n_tiles + t) * SLAB_ROWS + 8 * (lane & 7)));
    };
    const uint16_t* trow[4];
    auto act_at = [&](int i, int rank) { return *reinterpret_cast<const u32x4*>(trow[i] + rank); };
    uint16_t* hs = hs_all;
    float cterm[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    int rank_cur = rank_at(g_begin);
    int rank_nxt = g_begin + 1 < g_end ? rank_at(g_begin + 1) : 0;
    u32x4 sc_cur = scale_at(g_begin);
#pragma unroll
    for (int i = 0; i < 4; ++i) trow[i] = h + (int64_t)min(max(__builtin_amdgcn_readfirstlane(tki[i]), 0), T - 1) * ld;
    u32x4 raw0 = act_at(0, rank_cur);
    u32x4 raw1 = act_at(1, rank_cur);
    int2 rec = group_rec(g_begin);
    f32x4 acc[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
    f32x4 corr = {0, 0, 0, 0};
    // W: this group's width.  SAME: the next group exists and has this width (its payload is requested between
    // this group's blocks); MORE: a next group exists (its ranks, scales and activations are requested).
    auto group_step = [&](auto w_c, auto same_c, auto more_c, int g, int pack0) {
        constexpr int W = decltype(w_c)::value;
        constexpr bool same = decltype(same_c)::value, more = decltype(more_c)::value;
        Masks3 m3;
        if constexpr (W == 3) m3 = masks3_role0();
        int rank_nxt2 = 0;
        if (g + 2 < g_end) rank_nxt2 = rank_at(g + 2);
        u32x4 sc_nxt = {0, 0, 0, 0};
        if constexpr (more) sc_nxt = scale_at(g + 1);
        hs = hs_all + (g & 1) * (MAX_A * GU_STRIDE);
        auto stage = [&](auto i_c, u32x4 raw) {
            constexpr int i = decltype(i_c)::value;
            const u32x4 v = scaled_f16x8<BF16>(raw, sc_cur);
            *reinterpret_cast<u32x4*>(&hs[(pair + 4 * i) * GU_STRIDE + 8 * lane]) = v;
            cterm[i] += wave_sum_lane63(const_term_partial<W>(v));
        };
        if (pair < n_a) stage(I0{}, raw0);
        if (pair + 4 < n_a) stage(I1{}, raw1);
        if (pair + 8 < n_a) stage(I2{}, act_at(2, rank_cur));
        if (pair + 12 < n_a) stage(I3{}, act_at(3, rank_cur));
        __syncthreads();   // the operand is complete
        if constexpr (more) {
            raw0 = act_at(0, rank_nxt);
            raw1 = act_at(1, rank_nxt);
        }
        const uint16_t* ap16 = &hs[n * GU_STRIDE + 16 * kg];
        static_for([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            const u32x4 a_lo = *reinterpret_cast<const u32x4*>(ap16 + q * SLAB_ROWS);
            const u32x4 a_hi = *reinterpret_cast<const u32x4*>(ap16 + q * SLAB_ROWS + 8);
            gateup_pair<W, false>(pw[q], a_lo, a_hi, n >> 3, acc, corr, W == 3 ? &m3 : nullptr);
            if constexpr (same) issue_at(qc, W, pack0 + GU_SLABS * (n_tiles * 256 * W));
        }, std::make_integer_sequence<int, GU_SLABS>{});
        sc_cur = sc_nxt;
        rank_cur = rank_nxt;
        rank_nxt = rank_nxt2;
    };
    // Runs of groups of one width, each walked by a loop compiled for that width.  A run requests its own
    // first payload (no block registers are live from one run to the next), behind the activations and
    // scales of its first group, which were requested one group earlier.
    for (int g = g_begin; g < g_end;) {
        lane = tid & 63;
        asm volatile("" : "+v"(lane));
        n = lane & 15;
        kg = lane >> 4;
        unit = (uint32_t)(pair * 64 + lane);
        hi_unit = (uint32_t)hi_index0(kg, n, 2 * pair);
        int g1 = g + 1;
        while (g1 < g_end && __builtin_amdgcn_readfirstlane(grp_tab[g1].x) == rec.x) ++g1;
        const int2 next = g1 < g_end ? group_rec(g1) : int2{0, 0};
        auto run = [&](auto w_c) {
            constexpr int W = decltype(w_c)::value;
            int pack0 = rec.y;
            static_for([&](auto qc) { issue_at(qc, W, pack0); }, std::make_integer_sequence<int, GU_SLABS>{});
            for (; g + 1 < g1; ++g, pack0 += GU_SLABS * (n_tiles * 256 * W))
                group_step(w_c, std::true_type{}, std::true_type{}, g, pack0);
            if (g1 < g_end)
                group_step(w_c, std::false_type{}, std::true_type{}, g, pack0);
            else
                group_step(w_c, std::false_type{}, std::false_type{}, g, pack0);
            ++g;
        };
        if (rec.x == 2)
            run(std::integral_constant<int, 2>{});
        else if (rec.x == 3)
            run(std::integral_constant<int, 3>{});
        else
            run(std::integral_constant<int, 4>{});
        rec = next;
    }
    // the constant terms of the chunk's assignments, from the wavefronts that staged them
    if (lane == 63) {
#pragma unroll
        for (int i = 0; i < 4; ++i) cterm_lds[pair + 4 * i] = cterm[i];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) corr[j] = cterm_lds[4 * kg + j];
#pragma unroll
    for (int nbl = 0; nbl < 2; ++nbl) {
        const int c = t * N_TILE + 32 * pair + 16 * nbl + n;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int a = 4 * kg + j;
            if (a < n_a && c < I) {
                const int64_t row = as.row(a0 + a);
                if constexpr (SPLIT)
                    atomicAdd(&out[row * I + c], acc[nbl][j] - corr[j]);
                else
                    out[row * I + c] = acc[nbl][j] - corr[j];
            }
        }
    }
}

// ------------------------------------------------ gate AND up of one tile, z = silu(G) * U out
// The same walk for BOTH projections of one expert, one after the other in one workgroup (first all
// slab groups of the gate matrix, then all of the up matrix; the payload stream of a wavefront runs on
// from the one into the other), for sets in which the two matrices of every expert share one bit-width
// and one slab count.  The tile's gate sums stay in registers while the up sums are formed, and the item
// writes what the down projection needs, ready-made:
//     Z[a, c]      = f16(silu(G[a, c]) * U[a, c])                    (16-bit MFMA operand, [A, I])
//     Zsum[a, t]   = sum over the tile's 128 columns of Z as rounded  ([A, n_tiles] fp32; the constant term
//                                                                      of the down projection's decode)
// so the fp32 G / U round trip (8 bytes per element written, then read by every slab group of the expert)
// and the SiLU leave the down kernel, and the gate/up launch is one round of (expert, tile) workgroups
// instead of two rounds of (expert, tile, projection) ones.
// `cterm_lds`: 2 * MAX_A floats, `zs_lds`: 4 * MAX_A floats (LDS).
struct WalkMatrix {     // one projection's operands (wave-uniform)
    gptr<uint32_t> payload;
    gptr<__half> scale_s;
    gptr<int32_t> rank_idx;
    FastSlab first;
    const uint16_t* h;
    int64_t ld;
};

template <bool BF16, bool IDENT, int W>
__device__ __forceinline__ void gateup_walk_z_item(const WalkMatrix& mg, const WalkMatrix& mu,
                                                   const int32_t* __restrict__ token_indices, int a0, int n_a, int A, int T,
                                                   int I, int n_tiles, int t, int n_groups, uint16_t* __restrict__ Z,
                                                   float* __restrict__ Zsum, uint16_t* __restrict__ hs_all,
                                                   float* __restrict__ cterm_lds, float* __restrict__ zs_lds, int tid) {
    const int pair = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform
    const int lane = tid & 63;
    const int n = lane & 15, kg = lane >> 4;
    const uint32_t unit = (uint32_t)(pair * 64 + lane);
    const uint32_t hi_unit = (uint32_t)hi_index0(kg, n, 2 * pair);
    const int slab_words = n_tiles * 256 * W;       // payload words from one slab to the next
    Masks3 m3;
    if constexpr (W == 3) m3 = masks3_role0();
    int item_zero = 0;
    asm volatile("" : "+s"(item_zero));   // keeps this item's address arithmetic out of the caller's loop
    const int pack0_g = mg.first.pack_off + t * 256 * W + item_zero;
    const int pack0_u = mu.first.pack_off + t * 256 * W + item_zero;
    const int n_vg = 2 * n_groups;       // "virtual" groups: the gate matrix's, then the up matrix's

    uint32_t pw[GU_SLABS][4];   // slab q's block of the current group; refilled for the next group right after use
    auto issue = [&](auto q_c, int vg) {
        constexpr int q = decltype(q_c)::value;
        const bool up = vg >= n_groups;
        const int g = up ? vg - n_groups : vg;
        gptr<uint32_t> base = up ? mu.payload : mg.payload;
        load_pair_role0(base + (uint32_t)((up ? pack0_u : pack0_g) + (g * GU_SLABS + q) * slab_words), W, unit, hi_unit, pw[q]);
    };
    int tki[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) tki[i] = token_indices[min(a0 + pair + 4 * i, A - 1)];
    auto rank_at = [&](int vg) {
        const bool up = vg >= n_groups;
        const int g = up ? vg - n_groups : vg;
        const int k = (up ? mu.first.rank_off : mg.first.rank_off) + g * (GU_SLABS * SLAB_ROWS) + 8 * lane;
        if constexpr (IDENT) return k;      // rank_idx[k] == k in every expert of both sets
        else return (int)(up ? mu.rank_idx : mg.rank_idx)[k];
    };
    auto scale_at = [&](int vg) {
        const bool up = vg >= n_groups;
        const int g = up ? vg - n_groups : vg;
        gptr<__half> base = up ? mu.scale_s : mg.scale_s;
        return *reinterpret_cast<gptr_u32x4>(
            base + (uint32_t)((up ? mu.first.scale_off : mg.first.scale_off) +
                              ((g * GU_SLABS + (lane >> 3)) * n_tiles + t) * SLAB_ROWS + 8 * (lane & 7)));
    };
    const uint16_t* trow_g[4];
    const uint16_t* trow_u[4];
    auto act_at = [&](int i, int rank, bool up) {
        return *reinterpret_cast<const u32x4*>((up ? trow_u[i] : trow_g[i]) + rank);
    };
    uint16_t* hs = hs_all;
    float cterm_g[4] = {0.0f, 0.0f, 0.0f, 0.0f}, cterm_u[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    auto stage = [&](auto i_c, u32x4 raw, u32x4 sc, bool up) {
        constexpr int i = decltype(i_c)::value;
        const u32x4 v = scaled_f16x8<BF16>(raw, sc);
        *reinterpret_cast<u32x4*>(&hs[(pair + 4 * i) * GU_STRIDE + 8 * lane]) = v;
        const float part = wave_sum_lane63(const_term_partial<W>(v));
        if (up)
            cterm_u[i] += part;
        else
            cterm_g[i] += part;
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    int rank_cur = rank_at(0);
    int rank_nxt = rank_at(1);      // (n_vg >= 2)
    u32x4 sc_cur = scale_at(0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t tk = min(max(__builtin_amdgcn_readfirstlane(tki[i]), 0), T - 1);
        trow_g[i] = mg.h + tk * mg.ld;
        trow_u[i] = mu.h + tk * mu.ld;
    }
    u32x4 raw0 = act_at(0, rank_cur, false);
    u32x4 raw1 = act_at(1, rank_cur, false);
    static_for([&](auto qc) { issue(qc, 0); }, std::make_integer_sequence<int, GU_SLABS>{});
    f32x4 acc[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
    f32x4 acc_g[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
    f32x4 corr = {0, 0, 0, 0};
    auto group_step = [&](auto more_c, int vg) {
        constexpr bool more = decltype(more_c)::value;
        const bool up = vg >= n_groups;
        int rank_nxt2 = 0;
        if (vg + 2 < n_vg) rank_nxt2 = rank_at(vg + 2);
        u32x4 sc_nxt = {0, 0, 0, 0};
        if constexpr (more) sc_nxt = scale_at(vg + 1);
        if (vg == n_groups) {      // the gate sums are complete: keep them, start the up sums
            acc_g[0] = acc[0];
            acc_g[1] = acc[1];
            acc[0] = f32x4{0, 0, 0, 0};
            acc[1] = f32x4{0, 0, 0, 0};
        }
        hs = hs_all + (vg & 1) * (MAX_A * GU_STRIDE);
        if (pair < n_a) stage(I0{}, raw0, sc_cur, up);
        if (pair + 4 < n_a) stage(I1{}, raw1, sc_cur, up);
        if (pair + 8 < n_a) stage(I2{}, act_at(2, rank_cur, up), sc_cur, up);
        if (pair + 12 < n_a) stage(I3{}, act_at(3, rank_cur, up), sc_cur, up);
        __syncthreads();   // the operand is complete
        if constexpr (more) {
            const bool up_nxt = vg + 1 >= n_groups;
            raw0 = act_at(0, rank_nxt, up_nxt);
            raw1 = act_at(1, rank_nxt, up_nxt);
        }
        const uint16_t* ap16 = &hs[n * GU_STRIDE + 16 * kg];
        static_for([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            const u32x4 a_lo = *reinterpret_cast<const u32x4*>(ap16 + q * SLAB_ROWS);
            const u32x4 a_hi = *reinterpret_cast<const u32x4*>(ap16 + q * SLAB_ROWS + 8);
            gateup_pair<W, false>(pw[q], a_lo, a_hi, n >> 3, acc, corr, W == 3 ? &m3 : nullptr);
            if constexpr (more) issue(qc, vg + 1);
        }, std::make_integer_sequence<int, GU_SLABS>{});
        sc_cur = sc_nxt;
        rank_cur = rank_nxt;
        rank_nxt = rank_nxt2;
    };
    for (int vg = 0; vg + 1 < n_vg; ++vg) group_step(std::true_type{}, vg);
    group_step(std::false_type{}, n_vg - 1);
    // the constant terms of the chunk's assignments, from the wavefronts that staged them
    if (lane == 63) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            cterm_lds[pair + 4 * i] = cterm_g[i];
            cterm_lds[MAX_A + pair + 4 * i] = cterm_u[i];
        }
    }
    __syncthreads();
    // lane holds rows a = 4*kg + j of columns 32*pair + 16*nbl + n
    float zpart[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int a = 4 * kg + j;
        const float cg = cterm_lds[a], cu = cterm_lds[MAX_A + a];
#pragma unroll
        for (int nbl = 0; nbl < 2; ++nbl) {
            const int c = t * N_TILE + 32 * pair + 16 * nbl + n;
            const uint16_t zb = z_operand(acc_g[nbl][j] - cg, acc[nbl][j] - cu);
            if (a < n_a && c < I) Z[(int64_t)(a0 + a) * I + c] = zb;
            zpart[j] += __half2float(__ushort_as_half(zb));
        }
    }
    // row sums over this wavefront's 32 columns: the 16 lanes that share kg (one DPP row) hold one row
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float v = zpart[j];
        v = dpp_add_f32<0x111>(v);
        v = dpp_add_f32<0x112>(v);
        v = dpp_add_f32<0x114>(v);
        v = dpp_add_f32<0x118>(v);
        if (n == 15) zs_lds[pair * MAX_A + 4 * kg + j] = v;
    }
    __syncthreads();
    if (tid < n_a)
        Zsum[(int64_t)(a0 + tid) * n_tiles + t] = zs_lds[tid] + zs_lds[MAX_A + tid] + zs_lds[2 * MAX_A + tid] + zs_lds[3 * MAX_A + tid];
}

// ----------------------------------------------------------------------------------- down
// One (slab, tile) block of a down matrix: 4 row blocks x 4 k-steps (micro-tiles).
// `corr`: 1.5 * 2^W times the sum of the tile's z over its 128 columns, per assignment row of the
// lane (the constant term of the decoded operands 2^W + code; the z rows are summed once, when z
// is built, instead of by four more MFMAs per block).
template <int W>
__device__ __forceinline__ void down_block(const Block16& b, const u32x4 (&az)[4], const float (&sc)[4], f32x4 corr, f32x4 (&acc)[4]) {
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
        f32x4 t = {0, 0, 0, 0};
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            u32x4 bw;
            if constexpr (W == 2)
                bw = decode_fields2<2, false>(b.w[nb * 2 + (m >> 1)], 8 * (m & 1));
            else if constexpr (W == 4)
                bw = decode_fields4<false>(b.w[nb * 4 + m]);
            else
                bw = decode_r1w3<false>(b.w, nb, m);
            t = mfma16<false>(az[m], bw, t);
        }
        acc[nb] += (t - corr) * sc[nb];
    }
}

// Everything one wavefront of the down kernel does after the metadata has arrived, compiled
// per bit-width of the wavefront's slab (W == 0: no slab, the wavefront only helps to build z).
// The payload of the first tile is requested BEFORE z is built, so that weights are in flight
// while G and U are read and SiLU is evaluated -- of ONE tile: loads return in the order they
// were asked for, so the rows of G and U wait behind whatever payload was requested first, and
// every workgroup of the launch is at this point at the same time (two tiles ahead of z: the down
// kernel 5 to 7 % slower on 128 experts at 8 and 64 tokens and on 64 experts at 16 tokens, 3 % on
// 512 experts at 256 tokens; none: 2 to 6 % slower).  The second tile is requested when z is
// done; afterwards the tiles stream through two register buffers, one tile ahead of the one
// being computed.  The register budget is 128, so that all four
// workgroups of a CU -- on the 64-token benchmark layer the whole grid -- are resident at once:
// what only the epilogue needs (rank and multiplier of the rows, token and weight of the
// assignments) waits in LDS, and z is built two assignment rows at a time.
// ZREADY: `G` holds Z (16-bit operands, [A, I]) and `U` holds Zsum ([A, n_tiles] fp32) as written by
// gateup_walk_z_item: the z phase is a copy into LDS instead of two fp32 reads and a SiLU per element.
// Otherwise G and U are the first of `n_part` partial results, part_stride floats apart, that are added up.
// ZR: assignment rows whose G / U loads are in flight together while z is built (one memory round trip per ZR
// rows: the pass is latency-bound; more rows need more registers).
// ZBY: z is built a row per wavefront (see there); a variant of its own, chosen by the launcher for batches of several
// assignments per expert -- in one kernel with the column-wise form either is slowed down by the other's registers.
template <int W, bool ZREADY, int ZR, bool ZBY, class AS>
__device__ __forceinline__ void down_wave(gptr<uint32_t> payload, gptr<__half> scale, gptr<__half> svec, gptr<int32_t> rank_idx,
                                 const FastSlab fs, const float* __restrict__ G, const float* __restrict__ U, int n_part,
                                 int64_t part_stride, const AS& as,
                                 int a_begin, int a_end, int T, int I, int tb, int nt, int rank_out,
                                 float* __restrict__ rank_accum, uint16_t* __restrict__ z, int z_stride, float* __restrict__ zsum,
                                 int2* __restrict__ rows, int2* __restrict__ assigns, int tid, int lane) {
    const int n = lane & 15, kg = lane >> 4, g4 = kg * 4;
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    constexpr int WL = W == 0 ? 2 : W;
    for (int a0 = a_begin; a0 < a_end; a0 += MAX_A) {
        const int n_a = min(MAX_A, a_end - a0);
        int chunk_zero = 0;
        asm volatile("" : "+s"(chunk_zero));   // keeps this chunk's address arithmetic inside the loop
        Block16 buf[2];
        float sc[2][4];
        f32x4 acc[4];
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) acc[nb] = f32x4{0, 0, 0, 0};
        // the workgroup's tiles are tb .. tb + nt - 1; `i` counts from 0
        auto issue = [&](auto b_c, int i) {
            constexpr int B = decltype(b_c)::value;
            const int t = tb + i;
            load_block_role1<WL>(payload + (uint32_t)(fs.pack_off + (t + chunk_zero) * (WL == 3 ? R1W3_BLOCK_WORDS : 256 * WL)), lane,
                                 buf[B]);
            gptr<__half> sp = scale + (uint32_t)(fs.scale_off + t * SLAB_ROWS + n);
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) sc[B][nb] = gload_half(sp + 16 * nb);
        };
        auto compute = [&](auto b_c, int i) {
            constexpr int B = decltype(b_c)::value;
            u32x4 az[4];
            const uint16_t* zp = z + n * z_stride + i * N_TILE + 8 * kg;      // (z holds this workgroup's tiles only)
#pragma unroll
            for (int m = 0; m < 4; ++m) az[m] = *reinterpret_cast<const u32x4*>(zp + 32 * m);
            f32x4 corr;
#pragma unroll
            for (int j = 0; j < 4; ++j) corr[j] = zsum[(g4 + j) * ZSUM_STRIDE + tb + i] * (1.5f * (float)(1 << WL));
            down_block<WL>(buf[B], az, sc[B], corr, acc);
        };
        // logical rank and multiplier of the slab's row `lane`: needed by the epilogue only, kept
        // in LDS until then (one wavefront's own 64 entries: no barrier involved)
        int row_rank = -1;
        float row_s = 0.0f;
        if constexpr (W != 0) {
            issue(I0{}, 0);      // (ONE tile ahead of z: see above)
            row_rank = rank_idx[fs.rank_off + lane];
            row_s = gload_half(svec + fs.rank_off + lane);
        }
        // token ids and routing weights of the chunk (lane a holds assignment a): for the epilogue,
        // kept in LDS until then (every wavefront writes the same sixteen entries)
        const int tok_lane = as.token_if(a0 + lane, lane < n_a);
        const float rw_lane = as.weight_if(a0 + lane, lane < n_a);
        __syncthreads();   // the previous chunk is done with z
        if constexpr (ZREADY) {
            const uint16_t* __restrict__ Zg = reinterpret_cast<const uint16_t*>(G);
            const int pieces = nt * (N_TILE / 8);          // 16-byte pieces per row of this workgroup's tiles
            const int total = n_a * pieces;
            for (int idx0 = tid; idx0 < total; idx0 += 3 * 256) {      // (three loads in flight per thread)
                u32x4 v[3];
                int dst[3];
#pragma unroll
                for (int k = 0; k < 3; ++k) {
                    const int idx = min(idx0 + 256 * k, total - 1);
                    const int a = idx / pieces, p = idx - a * pieces;
                    const int c = tb * N_TILE + 8 * p;
                    v[k] = *reinterpret_cast<const u32x4*>(Zg + (int64_t)(a0 + a) * I + c);
                    dst[k] = a * z_stride + 8 * p;
                }
#pragma unroll
                for (int k = 0; k < 3; ++k)
                    if (idx0 + 256 * k < total) *reinterpret_cast<u32x4*>(z + dst[k]) = v[k];
            }
            if (tid < n_a * nt) {
                const int a = tid / nt, i = tid - a * nt;
                zsum[a * ZSUM_STRIDE + tb + i] = U[(int64_t)(a0 + a) * (((I + N_TILE - 1) / N_TILE)) + tb + i];
            }
        } else if constexpr (ZBY) {
            // z[a][c] = silu(G) * U as 16-bit operands for the rows a < n_a (other rows feed output rows that are never
            // stored).  A wavefront takes whole rows -- w, w + 4, ... -- and a lane four neighbouring columns of each 256
            // of the row, ZP such pieces of G and of U requested together: the rows of a chunk are ceil(n_a / 4) memory
            // round trips, where four columns per thread over all rows, two at a time, were ceil(n_a / 2).
            constexpr int ZP = ZR > ZROWS ? 6 : 3;
            const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
            const int c_begin = tb * N_TILE, c_end = min((tb + nt) * N_TILE, I);
            for (int a = wv; a < n_a; a += 4) {
                const int64_t row_off = (int64_t)as.row(a0 + a) * I;
                for (int p0 = c_begin; p0 < c_end; p0 += 256 * ZP) {
                    f32x4 gv[ZP], uv[ZP];
#pragma unroll
                    for (int p = 0; p < ZP; ++p) {
                        const int c = min(p0 + 256 * p + 4 * lane, c_end - 4);      // (a piece past the end repeats the last)
                        gv[p] = *reinterpret_cast<const f32x4*>(G + row_off + c);
                        uv[p] = *reinterpret_cast<const f32x4*>(U + row_off + c);
                    }
                    for (int q = 1; q < n_part; ++q) {
#pragma unroll
                        for (int p = 0; p < ZP; ++p) {
                            const int c = min(p0 + 256 * p + 4 * lane, c_end - 4);
                            gv[p] += *reinterpret_cast<const f32x4*>(G + row_off + c + q * part_stride);
                            uv[p] += *reinterpret_cast<const f32x4*>(U + row_off + c + q * part_stride);
                        }
                    }
#pragma unroll
                    for (int p = 0; p < ZP; ++p) {
                        const int c = p0 + 256 * p + 4 * lane;
                        if (p0 + 256 * p >= c_end) break;      // (wave-uniform)
                        const bool live = c < c_end;
                        uint16_t zb[4];
                        float part = 0.0f;      // sum of the four operands as rounded
#pragma unroll
                        for (int x = 0; x < 4; ++x) {
                            zb[x] = z_operand(gv[p][x], uv[p][x]);
                            part += __half2float(__ushort_as_half(zb[x]));
                        }
                        part = live ? part : 0.0f;
                        if (live) {
                            u32x2 packed;
                            packed[0] = (uint32_t)zb[0] | ((uint32_t)zb[1] << 16);
                            packed[1] = (uint32_t)zb[2] | ((uint32_t)zb[3] << 16);
                            *reinterpret_cast<u32x2*>(z + a * z_stride + c - c_begin) = packed;
                        }
                        // the 32 lanes of a half wavefront hold one tile's 128 columns: their sum arrives in lanes 31 and 63
                        part = dpp_add_f32<0x111>(part);
                        part = dpp_add_f32<0x112>(part);
                        part = dpp_add_f32<0x114>(part);
                        part = dpp_add_f32<0x118>(part);
                        part = dpp_add_f32<0x142, 0xa>(part);
                        const int c_tile = p0 + 256 * p + 4 * (lane & 32);      // first column of this half's tile
                        if ((lane & 31) == 31 && c_tile < c_end) zsum[a * ZSUM_STRIDE + c_tile / N_TILE] = part;
                    }
                }
            }
        } else
        // z[a][c] = silu(G) * U as 16-bit operands for the rows a < n_a (other rows feed
        // output rows that are never stored).  Each thread owns four neighbouring columns
        // and walks the assignments ZR at a time, their vector loads issued together.
        for (int c = tb * N_TILE + tid * 4; c < min((tb + nt) * N_TILE, I); c += 1024) {
            for (int ab = 0; ab < n_a; ab += ZR) {
                f32x4 gv[ZR], uv[ZR];
#pragma unroll
                for (int j = 0; j < ZR; ++j) {
                    const int a = min(ab + j, n_a - 1);
                    const int64_t gi = (int64_t)as.row(a0 + a) * I + c;
                    gv[j] = *reinterpret_cast<const f32x4*>(G + gi);
                    uv[j] = *reinterpret_cast<const f32x4*>(U + gi);
                }
                // (the gate/up kernel split the contraction: the sums are totals of partial results)
                for (int p = 1; p < n_part; ++p) {
#pragma unroll
                    for (int j = 0; j < ZR; ++j) {
                        const int a = min(ab + j, n_a - 1);
                        const int64_t gi = (int64_t)as.row(a0 + a) * I + c + p * part_stride;
                        gv[j] += *reinterpret_cast<const f32x4*>(G + gi);
                        uv[j] += *reinterpret_cast<const f32x4*>(U + gi);
                    }
                }
#pragma unroll
                for (int j = 0; j < ZR; ++j) {
                    if (ab + j < n_a) {
                        uint16_t zb[4];
                        float part = 0.0f;      // sum of the four operands as rounded
#pragma unroll
                        for (int x = 0; x < 4; ++x) {
                            zb[x] = z_operand(gv[j][x], uv[j][x]);
                            part += __half2float(__ushort_as_half(zb[x]));
                        }
                        u32x2 packed;
                        packed[0] = (uint32_t)zb[0] | ((uint32_t)zb[1] << 16);
                        packed[1] = (uint32_t)zb[2] | ((uint32_t)zb[3] << 16);
                        *reinterpret_cast<u32x2*>(z + (ab + j) * z_stride + c - tb * N_TILE) = packed;
                        // the 32 lanes of a half wavefront hold one tile's 128 columns: their sum
                        // arrives in lanes 31 and 63 (whole rows of 16 lanes are active or not)
                        part = dpp_add_f32<0x111>(part);
                        part = dpp_add_f32<0x112>(part);
                        part = dpp_add_f32<0x114>(part);
                        part = dpp_add_f32<0x118>(part);
                        part = dpp_add_f32<0x142, 0xa>(part);
                        if ((lane & 31) == 31) zsum[(ab + j) * ZSUM_STRIDE + c / N_TILE] = part;
                    }
                }
            }
        }
        if constexpr (W != 0) rows[lane] = int2{row_rank, __float_as_int(row_s)};
        if (lane < MAX_A) assigns[lane] = int2{tok_lane, __float_as_int(rw_lane)};
        __syncthreads();
        if (a0 == a_begin) BITSMOE_TL_DOWN_STAMP(2);
        if constexpr (W != 0) {
            if (nt > 1) issue(I1{}, 1);
        }
        if constexpr (W != 0) {
            // two buffers, one tile ahead of the one being computed (two ahead through three buffers: 3 to 5 % slower at 8
            // to 256 tokens on 64, 128 and 512 experts, 1 % faster at 64 tokens on 128)
            for (int i = 0; i < nt; i += 2) {
                compute(I0{}, i);
                if (i + 1 < nt) {
                    if (i + 2 < nt) issue(I0{}, i + 2);
                    compute(I1{}, i + 1);
                    if (i + 3 < nt) issue(I1{}, i + 3);
                }
            }
        }
        if (a0 == a_begin) BITSMOE_TL_DOWN_STAMP(3);
        if constexpr (W != 0) {
            // combine: rows of this slab are distinct output ranks; lane holds assignments 4*kg + j
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) {
                const int2 rs = rows[16 * nb + n];
                const int lr = rs.x;
                const float sv = __int_as_float(rs.y);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int a = g4 + j;
                    const int2 tr = assigns[a];
                    const int tk = tr.x;
                    const float rw = __int_as_float(tr.y);
                    if (lr >= 0 && lr < rank_out && a < n_a && tk >= 0 && tk < T)
                        atomicAdd(&rank_accum[(int64_t)tk * rank_out + lr], acc[nb][j] * sv * rw);
                }
            }
        }
        if (a0 == a_begin) BITSMOE_TL_DOWN_STAMP(4);
    }
}

}  // namespace bitsmoe
