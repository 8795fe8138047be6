// Small-batch ("decode") kernels of the routed-expert forward: HBM-bound streaming of the
// prepared payload, field decode in registers, 16x16x32 MFMA against up to 16 assignments
// of one expert.  See wave_layout.h for the layout and the (2^w + code) operand trick.
//
//   k_gateup_walk     G[a,c] / U[a,c]  = sum_k  hs'[a,k] * level[k,c]   (one workgroup per expert,
//                     projection and 128-column tile over all rows k: plain stores; the default)
//   k_gateup_decode   G[a,c] / U[a,c] += sum_k  hs'[a,k] * level[k,c]   (split over groups of 512 rows,
//                     fp32 atomics into cleared outputs: sets the walking kernel cannot take)
//                     hs'[a,k] = h[tok_a, rank_idx[k]] * s[k] * scale[tile(c), k]  (f16 operand,
//                     times the power of two by which the staggered field decode shrinks the code)
//   k_down_decode     rank_accum[tok_a, rank_idx[r]] += route_w[a] * s[r] *
//                         sum_tiles scale[tile, r] * sum_{c in tile} level[r,c] * z[a,c]
//                     z = silu(G) * U  (f16 operand)
//
// MFMA operands: A = activations (row index = assignment), B = weights (column index =
// output column / output rank row); D[4*(lane/16)+j][lane%16].
//
// The kernels are latency-engineered rather than compute-engineered: one memory round
// trip costs 1-2 us on a loaded MI355X, so (1) all metadata a workgroup needs is
// addressable from its block index (FastExpert / FastSlab tables: one round trip, not a
// chain of five), (2) every workgroup keeps the payload of its next step in flight while it
// computes the current one, (3) requests are ordered by when their data is needed: loads
// return in order, so a small request behind a large one waits for the large one.
// ---- optional in-kernel time stamps (builds with -DBITSMOE_TIMELINE only: `python -m bitsmoe_amd.build --timeline`)
// Thread 0 of every workgroup of k_gateup_walk / k_down_decode writes the 100 MHz wall clock at its phase boundaries
// (first assignment chunk) into a device array that bitsmoe_timeline_read_decode copies out.
// gate/up: 0 entry, 1 tables and routed entries at hand, 2 first chunk's tile stored, 6 exit.
// down:    0 entry, 1 tables and routed entries at hand, 2 z built (barrier passed), 3 tiles multiplied, 4 atomics issued, 6 exit.
#ifdef BITSMOE_TIMELINE
#include <hip/hip_runtime.h>
namespace bitsmoe {
constexpr int TL_STAMPS = 8;
constexpr int TL_MAX_WG = 8192;
__device__ unsigned long long g_tl_walk[TL_MAX_WG * TL_STAMPS];
__device__ unsigned long long g_tl_down[TL_MAX_WG * TL_STAMPS];
}  // namespace bitsmoe
#define BITSMOE_TL(arr, i)                                                          \
    do {                                                                            \
        if (threadIdx.x == 0 && blockIdx.x < ::bitsmoe::TL_MAX_WG)                  \
            ::bitsmoe::arr[blockIdx.x * ::bitsmoe::TL_STAMPS + (i)] = wall_clock64(); \
    } while (0)
#define BITSMOE_TL_DOWN_STAMP(i) BITSMOE_TL(g_tl_down, i)
#else
#define BITSMOE_TL(arr, i) do {} while (0)
#endif
#include "decode_bodies.h"
#include "decode_launch.h"

#include <cstdlib>

namespace bitsmoe {

// grid.x = E * n_groups * n_tchunks, grid.y = 2 (gate, up); 256 threads = 4 wavefronts.
// A workgroup takes one expert, one projection, up to 8 slabs (512 contraction rows) and a
// run of 128-column tiles [t0, t1).  Wavefront p owns columns [32p, 32p+32) of every tile,
// so partial sums never cross wavefronts; they go to G / U with fp32 atomics (the slab
// groups of one tile add into the same outputs).  The gather h[tok, rank_idx[k]] is done
// once per workgroup and kept in registers; per tile only the scale changes.
// Every wavefront walks the (tile, slab) blocks of its column pair as one sequence and
// keeps the payload of the next three blocks in flight (four rotating register buffers).
// GENERAL == false: only the width-specialised bodies (groups of eight equal-width slabs that
// follow each other in the payload); GENERAL == true: only the groups those skip.  Two kernels
// instead of one keep the register budget of the common case free of the general body.
// MODE: what the expert coordinate of the grid counts (GRID_*).
// (Four workgroups per CU: at 128 registers a fourth workgroup's round trips hide behind the other
// three; measured 41 -> 37.5 us on the 64-token case against three workgroups at 140 registers.)
template <bool BF16, bool GENERAL, int MODE>
__global__ __launch_bounds__(256, 4) void k_gateup_decode(
    const FastExpert* __restrict__ gate_fe, const FastSlab* __restrict__ gate_fs, int gate_max_slabs,
    const FastExpert* __restrict__ up_fe, const FastSlab* __restrict__ up_fs, int up_max_slabs,
    const uint16_t* __restrict__ h_gate, const uint16_t* __restrict__ h_up, int Rg, int Ru, int64_t ldg, int64_t ldu,
    const int32_t* __restrict__ token_indices, const int32_t* __restrict__ expert_offsets, int T, int A, int I,
    int E, int n_tiles, int n_groups, int n_tchunks, int tiles_per_wg, float* __restrict__ G, float* __restrict__ U,
    const ExpertOrder gate_order, const ExpertOrder up_order) {
    const int mt = blockIdx.y;
    // (consecutive workgroups land on different XCDs: that spreads experts of different cost)
    const int bid = blockIdx.x;
    const int tchunk = bid % n_tchunks;
    const int grp = (bid / n_tchunks) % n_groups;
    const int tid = threadIdx.x;
    int e = bid / (n_tchunks * n_groups);
    int chunk = -1;
    if constexpr (MODE == GRID_EXPERTS) {      // expensive experts first (the identity when there is no order)
        if (E <= EXPERT_ORDER_MAX) e = mt ? up_order.at(e) : gate_order.at(e);
    } else if constexpr (MODE == GRID_ACTIVE) {
        e = nth_active_expert(expert_offsets, E, A, e, tid & 63);
        if (e < 0) return;
    } else if constexpr (MODE == GRID_CHUNKS) {
        const ChunkRef ref = nth_chunk(expert_offsets, E, A, e, tid & 63);
        e = ref.expert;
        chunk = ref.chunk;
        if (e < 0) return;
    }
    const int pair = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform
    const int lane = tid & 63;
    const int n = lane & 15, kg = lane >> 4;

    // one round trip: assignment range, expert record, the group's slab records
    int a_begin = max(expert_offsets[e], 0);
    int a_end = min(expert_offsets[e + 1], A);
    if (chunk >= 0) {      // this workgroup's chunk only
        a_begin += MAX_A * chunk;
        a_end = min(a_end, a_begin + MAX_A);
    }
    const FastExpert* __restrict__ fe_tab = mt ? up_fe : gate_fe;
    const FastSlab* __restrict__ fs_tab = mt ? up_fs : gate_fs;
    const int max_slabs = mt ? up_max_slabs : gate_max_slabs;
    const int s0 = grp * GU_SLABS;
    if (s0 >= max_slabs) return;
    const FastExpert fe = fe_tab[e];
    int sbits[GU_SLABS], spack[GU_SLABS];
#pragma unroll
    for (int q = 0; q < GU_SLABS; ++q) {
        sbits[q] = 0;
        spack[q] = 0;
        if (s0 + q < max_slabs) {
            const FastSlab fs = load_fast_slab(fs_tab, e * max_slabs + s0 + q);
            sbits[q] = fs.bits;
            spack[q] = fs.pack_off;
        }
    }
    // the two slabs whose rows this wavefront converts (lane = row)
    FastSlab mine[2];
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        mine[it] = FastSlab{0, 0, 0, 0};
        if (s0 + pair + 4 * it < max_slabs) mine[it] = load_fast_slab(fs_tab, e * max_slabs + s0 + pair + 4 * it);
    }
    if (a_end <= a_begin || sbits[0] == 0) return;

    gptr<uint32_t> payload = as_global(fe.payload);
    gptr<__half> scale = as_global(fe.scale);
    gptr<__half> svec = as_global(fe.s);
    gptr<int32_t> rank_idx = as_global(fe.rank_idx);
    const uint16_t* __restrict__ h = mt ? h_up : h_gate;
    const int R = mt ? Ru : Rg;
    const int64_t ld = mt ? ldu : ldg;      // elements from one activation row to the next
    float* __restrict__ out = mt ? U : G;
    const int t0_wg = tchunk * tiles_per_wg;
    const int t1 = min(t0_wg + tiles_per_wg, n_tiles);
    const uint32_t unit = (uint32_t)(pair * 64 + lane);
    const uint32_t hi_unit = (uint32_t)hi_index0(kg, n, 2 * pair);

    __shared__ __attribute__((aligned(16))) uint16_t hs[MAX_A * GU_STRIDE];

    // A group whose eight slabs share one bit-width and follow each other in the payload
    // (the usual case) runs a body compiled for that width: no per-slab branches, affine
    // block addresses.  WG == 0 is the general body with run-time widths.
    bool uniform8 = true;
#pragma unroll
    for (int q = 1; q < GU_SLABS; ++q)
        uniform8 = uniform8 && sbits[q] == sbits[0] && spack[q] == spack[0] + q * n_tiles * 256 * sbits[0];

    auto body = [&](auto wg_c) {
    constexpr int WG = decltype(wg_c)::value;
    const int slab_words = n_tiles * 256 * WG;       // payload words from one slab to the next (WG != 0)
    auto q_bits = [&](int q) { return WG != 0 ? WG : sbits[q]; };
    auto q_pack = [&](int q) { return WG != 0 ? spack[0] + q * slab_words : spack[q]; };
    for (int a0 = a_begin; a0 < a_end; a0 += MAX_A) {
        const int n_a = min(MAX_A, a_end - a0);
        // an opaque zero keeps the address arithmetic of this chunk inside the loop body
        int chunk_zero = 0;
        asm volatile("" : "+s"(chunk_zero));
        const int t0 = t0_wg + chunk_zero;

        uint32_t pw[GU_SLABS][4];   // slab q's block of the current tile; refilled for the next tile right after use
        auto issue = [&](auto buf_c, int t, int q_bits, int q_pack) {
            constexpr int B = decltype(buf_c)::value;
            load_pair_role0(payload + (uint32_t)(q_pack + t * 256 * q_bits), q_bits, unit, hi_unit, pw[B]);
        };
        // prologue: every block of the first tile
        static_for([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            if (q_bits(q) != 0) issue(qc, t0, q_bits(q), q_pack(q));
        }, std::make_integer_sequence<int, GU_SLABS>{});
        // token ids of the chunk: one vector load, broadcast later with readlane
        const int tok_lane = (lane < n_a) ? token_indices[a0 + lane] : -1;

        // rows of this lane: logical rank, per-row multiplier, scale of the first tile
        int rk[2];
        float srow[2], sc_cur[2], sc_nxt[2] = {0.0f, 0.0f};
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            rk[it] = -1;
            srow[it] = 0.0f;
            sc_cur[it] = 0.0f;
            if (mine[it].bits != 0) {
                const int k = mine[it].rank_off + lane;
                const int r = rank_idx[k];
                rk[it] = (r >= 0 && r < R) ? r : -1;
                srow[it] = gload_half(svec + k);
                sc_cur[it] = gload_half(scale + mine[it].scale_off + t0 * SLAB_ROWS + lane);
            }
        }
        // gather the activations of the chunk's assignments for both rows (raw 16-bit, two per
        // register).  Loads are issued in two branch-free groups of eight assignments (clamped
        // addresses, results masked afterwards) so that their round trips overlap.
        uint32_t hp[2][MAX_A / 2];
        const int rkc[2] = {max(rk[0], 0), max(rk[1], 0)};
#pragma unroll
        for (int g = 0; g < 2; ++g) {
#pragma unroll
            for (int ap = 4 * g; ap < 4 * g + 4; ++ap) {
                hp[0][ap] = 0;
                hp[1][ap] = 0;
            }
            if (8 * g < n_a) {
                uint32_t raw[2][8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int tk = __builtin_amdgcn_readlane(tok_lane, 8 * g + j);
                    const int tkc = min(max(tk, 0), T - 1);
#pragma unroll
                    for (int it = 0; it < 2; ++it) raw[it][j] = h[(int64_t)tkc * ld + rkc[it]];
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int tk = __builtin_amdgcn_readlane(tok_lane, 8 * g + j);
                    const bool tk_ok = tk >= 0 && tk < T;
#pragma unroll
                    for (int it = 0; it < 2; ++it)
                        if (!(tk_ok && rk[it] >= 0)) raw[it][j] = 0;
                }
                if constexpr (BF16) {      // the MFMA operands are f16 whatever the activations are
#pragma unroll
                    for (int j = 0; j < 8; ++j)
#pragma unroll
                        for (int it = 0; it < 2; ++it)
                            raw[it][j] = __builtin_bit_cast(uint16_t, (_Float16)__uint_as_float(raw[it][j] << 16));
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    hp[0][4 * g + j] = raw[0][2 * j] | (raw[0][2 * j + 1] << 16);
                    hp[1][4 * g + j] = raw[1][2 * j] | (raw[1][2 * j + 1] << 16);
                }
            }
        }

        for (int t = t0; t < t1; ++t) {
            const bool more = t + 1 < t1;
            if (more) {
#pragma unroll
                for (int it = 0; it < 2; ++it)
                    if (mine[it].bits != 0)
                        sc_nxt[it] = gload_half(scale + mine[it].scale_off + (t + 1) * SLAB_ROWS + lane);
            }
            __syncthreads();   // every wavefront is done reading hs'(t-1)
#pragma unroll
            for (int it = 0; it < 2; ++it) {
                if (mine[it].bits == 0) continue;
                // two assignments per packed multiply; rows without an assignment hold zeros
                // (times the stagger factor of the row: the decoded weight carries its inverse)
                const float fac = (float)stagger_factor(mine[it].bits, lane);
                const uint32_t sv = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)(srow[it] * sc_cur[it] * fac)) * 0x10001u;
                uint16_t* dst = &hs[(pair + 4 * it) * SLAB_ROWS + lane];
#pragma unroll
                for (int ap = 0; ap < MAX_A / 2; ++ap) {
                    const uint32_t v = pk_mul_f16(hp[it][ap], sv);
                    dst[(2 * ap) * GU_STRIDE] = (uint16_t)(v & 0xFFFFu);
                    dst[(2 * ap + 1) * GU_STRIDE] = (uint16_t)(v >> 16);
                }
            }
            __syncthreads();   // hs'(t) is complete
            f32x4 acc[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
            f32x4 corr = {0, 0, 0, 0};
            const uint16_t* ap16 = &hs[n * GU_STRIDE + 16 * kg];
            static_for([&](auto qc) {
                constexpr int q = decltype(qc)::value;
                const int bq = q_bits(q);
                if (bq == 0) return;
                const u32x4 a_lo = *reinterpret_cast<const u32x4*>(ap16 + q * SLAB_ROWS);
                const u32x4 a_hi = *reinterpret_cast<const u32x4*>(ap16 + q * SLAB_ROWS + 8);
                if (bq == 2)
                    gateup_pair<2>(pw[q], a_lo, a_hi, n >> 3, acc, corr);
                else if (bq == 3)
                    gateup_pair<3>(pw[q], a_lo, a_hi, n >> 3, acc, corr);
                else
                    gateup_pair<4>(pw[q], a_lo, a_hi, n >> 3, acc, corr);
                // the buffer is free again: fetch the same slab's block of the next tile
                if (more) issue(qc, t + 1, bq, q_pack(q));
            }, std::make_integer_sequence<int, GU_SLABS>{});
            // remove the constant term and add into G / U: lane holds rows a = 4*kg + j of
            // column 32*pair + 16*nbl + n
#pragma unroll
            for (int nbl = 0; nbl < 2; ++nbl) {
                const int c = t * N_TILE + 32 * pair + 16 * nbl + n;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int a = 4 * kg + j;
                    if (a < n_a && c < I) atomicAdd(&out[(int64_t)(a0 + a) * I + c], acc[nbl][j] - corr[j]);
                }
            }
            sc_cur[0] = sc_nxt[0];
            sc_cur[1] = sc_nxt[1];
        }
    }
    };   // body

    const bool fast = uniform8 && sbits[0] >= 2 && sbits[0] <= 4;
    if constexpr (GENERAL) {
        if (!fast) body(std::integral_constant<int, 0>{});
    } else {
        if (!fast) return;
        if (sbits[0] == 2)
            body(std::integral_constant<int, 2>{});
        else if (sbits[0] == 3)
            body(std::integral_constant<int, 3>{});
        else
            body(std::integral_constant<int, 4>{});
    }
}

// ------------------------------------------------------- gate / up, one workgroup per tile
// gateup_walk_item launched as a grid of its own; 256 threads = 4 wavefronts.  An item is (expert
// coordinate, tile, projection), item = (coordinate * n_tiles + tile) * 2 + projection; an expert with
// more than 16 assignments is served in 16-assignment chunks, one after the other (or one workgroup per
// chunk: GRID_CHUNKS).
// The first `n_unsplit` workgroups take one item each; behind them every item is shared by `split`
// workgroups, each of which contracts over its share of the item's slab groups and stores its sums into
// a partial result of its own: partial p of G / U lies p * part_stride floats behind G / U.  The down
// kernel adds the `n_part` partials up (n_part = split when any item is split, else 1), so a workgroup
// with a whole item stores zeros into the partials 1 .. n_part - 1 of its elements.  The launcher splits
// the items when there are too few of them to fill the chip.
// The kernel also clears `zero_out` (the forward's accumulator, added into by the down kernel).
// MIXED: experts whose slab groups differ in width (gateup_walk_item_mixed); a kernel of its own, so that
// the one-width kernel keeps its registers to itself.
// ROUTED (GRID_EXPERTS or GRID_ACTIVE): there are no routing tables; the workgroup finds its expert's entries among the
// n_flat = T * top_k routed ids itself (inline_route) and row = flat entry index of the intermediates.  With
// GRID_ACTIVE the expert coordinate counts routed ENTRIES: the workgroup of entry s serves the expert that entry
// names if s is that expert's first entry, and exits otherwise -- every active expert is served exactly once.
template <bool BF16, int MODE, bool IDENT, bool MIXED, bool ROUTED>
__global__ __launch_bounds__(256, 4) void k_gateup_walk(
    const FastExpert* __restrict__ gate_fe, const FastSlab* __restrict__ gate_fs, int gate_max_slabs,
    const FastExpert* __restrict__ up_fe, const FastSlab* __restrict__ up_fs, int up_max_slabs,
    const uint16_t* __restrict__ h_gate, const uint16_t* __restrict__ h_up, int64_t ldg, int64_t ldu,
    const int32_t* __restrict__ token_indices, const int32_t* __restrict__ expert_offsets, int T, int A, int I,
    int E, int n_tiles, float* __restrict__ G, float* __restrict__ U, int n_unsplit, int split, int n_part,
    int64_t part_stride, float* __restrict__ zero_out, int64_t zero_n, const ExpertOrder gate_order,
    const ExpertOrder up_order, const void* __restrict__ selected, int ids_are_i64, int n_flat, int top_k,
    const int32_t* __restrict__ local_to_global, const int32_t* __restrict__ global_to_local, int n_global) {
    static_assert(!ROUTED || MODE != GRID_CHUNKS, "inline routing serves whole experts");
    BITSMOE_TL(g_tl_walk, 0);
    const int tid = threadIdx.x;
    // (the routed ids do not depend on the workgroup's expert: requested before anything else, they arrive while the
    // expert's tables are looked up; all of it is waited for together, in front of the scan)
    [[maybe_unused]] RouteIds rid;
    if constexpr (ROUTED && MODE == GRID_EXPERTS) rid = inline_route_request(selected, ids_are_i64, n_flat, tid);
    // (the arguments the start-up goes through, in scalar registers now: one batch of loads from the argument segment
    // and one wait, where the compiler would fetch each in front of its first use, one dependent wait after the other)
    asm volatile("" ::"s"(gate_max_slabs), "s"(up_max_slabs), "s"(E), "s"(n_tiles), "s"(n_unsplit), "s"(split), "s"(top_k));
    {   // this workgroup's share of the accumulator (before any exit)
        const int64_t total = (int64_t)gridDim.x * 256;
        for (int64_t i = (int64_t)blockIdx.x * 256 + tid; i < zero_n; i += total) zero_out[i] = 0.0f;
    }
    int item = blockIdx.x, part = 0, parts = 1;
    if (item >= n_unsplit) {
        const int r = item - n_unsplit;
        item = n_unsplit + r / split;
        part = r % split;
        parts = split;
    }
    const int mt = item & 1;
    const int bid = item >> 1;
    const int t = bid % n_tiles;
    int e = bid / n_tiles;
    int chunk = -1;
    if constexpr (MODE == GRID_EXPERTS) {      // expensive experts first (the identity when there is no order)
        if (E <= EXPERT_ORDER_MAX) e = mt ? up_order.at(e) : gate_order.at(e);
    } else if constexpr (MODE == GRID_ACTIVE && !ROUTED) {
        e = nth_active_expert(expert_offsets, E, A, e, tid & 63);
        if (e < 0) return;
    } else if constexpr (MODE == GRID_CHUNKS) {
        const ChunkRef ref = nth_chunk(expert_offsets, E, A, e, tid & 63);
        e = ref.expert;
        chunk = ref.chunk;
        if (e < 0) return;
    }
    // one round trip: assignment range (or the routed ids), expert record, the record of the expert's first slab
    int a_begin = 0, a_end = 0;
    int gid = -1;
    __shared__ std::conditional_t<ROUTED, InlineRouteLds, int> route_lds;
    const FastExpert* __restrict__ fe_tab = mt ? up_fe : gate_fe;
    const FastSlab* __restrict__ fs_tab = mt ? up_fs : gate_fs;
    const int max_slabs = mt ? up_max_slabs : gate_max_slabs;
    FastExpert fe;
    FastSlab first;
    if constexpr (ROUTED && MODE == GRID_ACTIVE) {
        // `e` is an entry index: serve the expert it names if this is the expert's first entry.  The local id of that
        // expert and its record are asked for as soon as the entry's id is here; the scan of all ids runs meanwhile.
        const int slot = e;
        if (slot >= n_flat) return;
        const RouteIds all = inline_route_request(selected, ids_are_i64, n_flat, tid);
        gid = __builtin_amdgcn_readfirstlane(routed_id(selected, ids_are_i64, slot));
        if (gid < 0 || gid >= n_global) return;
        e = __builtin_amdgcn_readfirstlane(global_to_local[gid]);
        if (e < 0 || e >= E) return;
        fe = fe_tab[e];
        first = load_fast_slab(fs_tab, e * max_slabs);
        a_end = inline_route_finish(all, n_flat, top_k, gid, route_lds, tid);
        hold_fast_expert(fe);
        if (a_end == 0 || route_lds.ent[0] != slot) return;
    } else {
        if constexpr (ROUTED) {
            gid = local_to_global[e];
        } else {
            a_begin = max(expert_offsets[e], 0);
            a_end = min(expert_offsets[e + 1], A);
            if (chunk >= 0) {
                a_begin += MAX_A * chunk;
                a_end = min(a_end, a_begin + MAX_A);
            }
        }
        fe = fe_tab[e];
        first = load_fast_slab(fs_tab, e * max_slabs);
        hold_fast_expert(fe);
    }
    const int fe_num_slabs = fe.num_slabs;
    // the widths and payload offsets of the expert's slab groups (read by the mixed-width walk only, but
    // requested here, together with the expert's record)
    __shared__ int2 grp_tab[MIXED ? WALK_MAX_GROUPS : 1];
    if constexpr (MIXED) {
        if (tid < WALK_MAX_GROUPS && tid * GU_SLABS < max_slabs) {
            const FastSlab gs = fs_tab[(int64_t)e * max_slabs + tid * GU_SLABS];
            grp_tab[tid] = int2{gs.bits, gs.pack_off};
        }
    }
    if constexpr (ROUTED && MODE == GRID_EXPERTS) {
        hold_route_ids(rid);
        a_end = inline_route_finish(rid, n_flat, top_k, gid, route_lds, tid);
    }
    if (a_end <= a_begin || first.bits == 0) return;
    BITSMOE_TL(g_tl_walk, 1);
    const int n_groups = fe_num_slabs / GU_SLABS;
    // this workgroup's share of the slab groups, and the partial result it writes (no division for a whole item)
    int g_begin = 0, g_end = n_groups;
    if (parts > 1) {
        g_begin = part * n_groups / parts;
        g_end = (part + 1) * n_groups / parts;
    }

    gptr<uint32_t> payload = as_global(fe.payload);
    gptr<__half> scale_s = as_global(fe.scale_s);
    gptr<int32_t> rank_idx = as_global(fe.rank_idx);
    const uint16_t* __restrict__ h = mt ? h_up : h_gate;
    const int64_t ld = mt ? ldu : ldg;
    float* __restrict__ out = (mt ? U : G) + part * part_stride;
    auto assignments = [&]() {
        if constexpr (ROUTED)
            return AssignInline{route_lds.tok, route_lds.ent, nullptr, a_end};
        else
            return AssignTables{token_indices, nullptr, A};
    };
    const auto as = assignments();
    // partials nobody else writes for these elements: all but the own one of a share without slab groups,
    // 1 .. n_part - 1 of a whole item
    {
        const int p_first = parts > 1 ? part : 1, p_end = parts > 1 ? (g_begin == g_end ? part + 1 : part) : n_part;
        const int cols = min(N_TILE, I - t * N_TILE);
        for (int p = p_first; p < p_end; ++p) {
            float* __restrict__ zp = (mt ? U : G) + p * part_stride;
            for (int i = tid; i < (a_end - a_begin) * N_TILE; i += 256) {
                const int a = i / N_TILE, c = i - a * N_TILE;
                if (c < cols) zp[(int64_t)as.row(a_begin + a) * I + t * N_TILE + c] = 0.0f;
            }
        }
    }
    if (g_begin == g_end) return;

    // two copies of the operand, used in turn: one workgroup barrier per group instead of two
    __shared__ __attribute__((aligned(16))) uint16_t hs_all[2 * MAX_A * GU_STRIDE];
    __shared__ float cterm_lds[MAX_A];

    if constexpr (MIXED) __syncthreads();        // grp_tab is complete
    for (int a0 = a_begin; a0 < a_end; a0 += MAX_A) {
        const int n_a = min(MAX_A, a_end - a0);
        if (a0 != a_begin) __syncthreads();      // the previous chunk's readers of the operand are done
        if constexpr (MIXED) {
            gateup_walk_item_mixed<BF16, IDENT, false>(payload, scale_s, rank_idx, grp_tab, h, ld, as, a0, n_a, T, I, n_tiles, t,
                                                       g_begin, g_end, out, hs_all, cterm_lds, tid);
        } else {
            auto run = [&](auto w_c) {
                if (n_a > 8)      // (the chunk's wavefronts stage three or four assignments each)
                    gateup_walk_item<BF16, IDENT, decltype(w_c)::value, false, decltype(as), false, true>(
                        payload, scale_s, rank_idx, first, h, ld, as, a0, n_a, T, I, n_tiles, t, g_begin, g_end, out, hs_all,
                        cterm_lds, tid);
                else
                    gateup_walk_item<BF16, IDENT, decltype(w_c)::value, false>(payload, scale_s, rank_idx, first, h, ld, as, a0,
                                                                               n_a, T, I, n_tiles, t, g_begin, g_end, out, hs_all,
                                                                               cterm_lds, tid);
            };
            if (first.bits == 2)
                run(std::integral_constant<int, 2>{});
            else if (first.bits == 3)
                run(std::integral_constant<int, 3>{});
            else if (first.bits == 4)
                run(std::integral_constant<int, 4>{});
        }
        if (a0 == a_begin) BITSMOE_TL(g_tl_walk, 2);
    }
    BITSMOE_TL(g_tl_walk, 6);
}

// gateup_walk_z_item launched as a grid: grid.x = (expert coordinate) * n_tiles; 256 threads.  One
// workgroup forms BOTH projections of its tile and writes Z / Zsum; it also clears `zero_out`.
template <bool BF16, int MODE, bool IDENT>
__global__ __launch_bounds__(256, 4) void k_gateup_walk_z(
    const FastExpert* __restrict__ gate_fe, const FastSlab* __restrict__ gate_fs, const FastExpert* __restrict__ up_fe,
    const FastSlab* __restrict__ up_fs, int max_slabs, const uint16_t* __restrict__ h_gate,
    const uint16_t* __restrict__ h_up, int64_t ldg, int64_t ldu, const int32_t* __restrict__ token_indices,
    const int32_t* __restrict__ expert_offsets, int T, int A, int I, int E, int n_tiles, uint16_t* __restrict__ Z,
    float* __restrict__ Zsum, float* __restrict__ zero_out, int64_t zero_n, const ExpertOrder order) {
    const int bid = blockIdx.x;
    const int tid = threadIdx.x;
    {   // this workgroup's share of the accumulator (before any exit)
        const int64_t total = (int64_t)gridDim.x * 256;
        for (int64_t i = (int64_t)bid * 256 + tid; i < zero_n; i += total) zero_out[i] = 0.0f;
    }
    const int t = bid % n_tiles;
    int e = bid / n_tiles;
    int chunk = -1;
    if constexpr (MODE == GRID_EXPERTS) {      // expensive experts first (the identity when there is no order)
        if (E <= EXPERT_ORDER_MAX) e = order.at(e);
    } else if constexpr (MODE == GRID_ACTIVE) {
        e = nth_active_expert(expert_offsets, E, A, e, tid & 63);
        if (e < 0) return;
    } else if constexpr (MODE == GRID_CHUNKS) {
        const ChunkRef ref = nth_chunk(expert_offsets, E, A, e, tid & 63);
        e = ref.expert;
        chunk = ref.chunk;
        if (e < 0) return;
    }
    int a_begin = max(expert_offsets[e], 0);
    int a_end = min(expert_offsets[e + 1], A);
    if (chunk >= 0) {
        a_begin += MAX_A * chunk;
        a_end = min(a_end, a_begin + MAX_A);
    }
    const FastExpert feg = gate_fe[e];
    const FastExpert feu = up_fe[e];
    const FastSlab first_g = load_fast_slab(gate_fs, e * max_slabs);
    const FastSlab first_u = load_fast_slab(up_fs, e * max_slabs);
    if (a_end <= a_begin || first_g.bits == 0) return;
    const int n_groups = max_slabs / GU_SLABS;
    const WalkMatrix mg{as_global(feg.payload), as_global(feg.scale_s), as_global(feg.rank_idx), first_g, h_gate, ldg};
    const WalkMatrix mu{as_global(feu.payload), as_global(feu.scale_s), as_global(feu.rank_idx), first_u, h_up, ldu};

    __shared__ __attribute__((aligned(16))) uint16_t hs_all[2 * MAX_A * GU_STRIDE];
    __shared__ float cterm_lds[2 * MAX_A];
    __shared__ float zs_lds[4 * MAX_A];

    for (int a0 = a_begin; a0 < a_end; a0 += MAX_A) {
        const int n_a = min(MAX_A, a_end - a0);
        if (a0 != a_begin) __syncthreads();      // the previous chunk's readers of the LDS buffers are done
        auto run = [&](auto w_c) {
            gateup_walk_z_item<BF16, IDENT, decltype(w_c)::value>(mg, mu, token_indices, a0, n_a, A, T, I, n_tiles, t, n_groups, Z,
                                                                  Zsum, hs_all, cterm_lds, zs_lds, tid);
        };
        if (first_g.bits == 2)
            run(std::integral_constant<int, 2>{});
        else if (first_g.bits == 3)
            run(std::integral_constant<int, 3>{});
        else if (first_g.bits == 4)
            run(std::integral_constant<int, 4>{});
    }
}

// grid.x = E * n_groups * n_tchunks; 256 threads; dynamic LDS = z (16 * (n_tiles * 128 + 8) * 2 bytes), the
// per-tile sums of its rows, the epilogue's row and assignment records.
// A workgroup takes four slabs of one expert and a run of tiles; with few active experts the
// tiles are split over several workgroups (their partial sums meet in the atomics of the combine).
// z = silu(G) * U as 16-bit operands [A, I] and the per-tile sums of the rounded operands [A, n_tiles], from the fp32
// gate and up sums (the totals of `n_part` partial results): what the down kernel's workgroups otherwise each form
// for themselves, two rows per memory round trip.  Worth a launch of its own where those workgroups hold full
// 16-assignment chunks and many of them share a chunk.  A thread owns four columns, 32 lanes one tile of one row.
__global__ __launch_bounds__(256) void k_decode_silu(const float* __restrict__ G, const float* __restrict__ U, int n_part,
                                                     int64_t part_stride, int A, int I, int n_tiles,
                                                     uint16_t* __restrict__ Z, float* __restrict__ Zsum) {
    const int64_t unit = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 5;      // (row, tile)
    const int lane32 = threadIdx.x & 31;
    const int a = (int)(unit / n_tiles), t = (int)(unit - (int64_t)a * n_tiles);
    if (a >= A) return;                  // (whole half-wavefronts leave)
    const int c = t * N_TILE + 4 * lane32;
    const bool in = c < I;
    const int64_t gi = (int64_t)a * I + (in ? c : 0);
    f32x4 gv = *reinterpret_cast<const f32x4*>(G + gi), uv = *reinterpret_cast<const f32x4*>(U + gi);
    for (int p = 1; p < n_part; ++p) {
        gv += *reinterpret_cast<const f32x4*>(G + gi + p * part_stride);
        uv += *reinterpret_cast<const f32x4*>(U + gi + p * part_stride);
    }
    uint16_t zb[4];
    float part = 0.0f;      // sum of the four operands as rounded
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        zb[x] = in ? z_operand(gv[x], uv[x]) : (uint16_t)0;
        part += __half2float(__ushort_as_half(zb[x]));
    }
    if (in) {
        u32x2 packed;
        packed[0] = (uint32_t)zb[0] | ((uint32_t)zb[1] << 16);
        packed[1] = (uint32_t)zb[2] | ((uint32_t)zb[3] << 16);
        *reinterpret_cast<u32x2*>(Z + (int64_t)a * I + c) = packed;
    }
    part = dpp_add_f32<0x111>(part);
    part = dpp_add_f32<0x112>(part);
    part = dpp_add_f32<0x114>(part);
    part = dpp_add_f32<0x118>(part);
    part = dpp_add_f32<0x142, 0xa>(part);
    if (lane32 == 31) Zsum[(int64_t)a * n_tiles + t] = part;
}

// ZREADY: G / U hold Z / Zsum written by k_gateup_walk_z instead of the fp32 gate and up sums.  Otherwise the
// sums are the totals of `n_part` partial results part_stride floats apart (k_gateup_walk).
// ROUTED (GRID_EXPERTS or GRID_ACTIVE): no routing tables; the workgroup finds its expert's entries among the routed
// ids itself, as the gate/up kernel did (same rows of the intermediates), and takes the routing weights
// from `sel_weights` in entry order.
// ZR: rows of G / U in flight while z is built; more than the usual two only where z is so large that three
// workgroups fit a CU, which leaves each of them more registers (launch bounds follow).
template <int MODE, bool ZREADY, bool ROUTED, int ZR, bool ZBY = false>
__global__ __launch_bounds__(256, ZR > ZROWS ? 3 : 4) void k_down_decode(
    const FastExpert* __restrict__ down_fe, const FastSlab* __restrict__ down_fs, int max_slabs,
    const float* __restrict__ G, const float* __restrict__ U, int n_part, int64_t part_stride,
    const float* __restrict__ route_w, const int32_t* __restrict__ token_indices,
    const int32_t* __restrict__ expert_offsets, int T, int A, int I, int E, int n_tiles, int n_groups, int n_tchunks,
    int tiles_per_wg, int n_work, int rank_out, float* __restrict__ rank_accum, const void* __restrict__ selected,
    int ids_are_i64, int n_flat, int top_k, const int32_t* __restrict__ local_to_global,
    const float* __restrict__ sel_weights, const int32_t* __restrict__ global_to_local, int n_global) {
    static_assert(!ROUTED || (MODE != GRID_CHUNKS && !ZREADY), "inline routing serves whole experts");
    BITSMOE_TL(g_tl_down, 0);
    // (the routed ids do not depend on the workgroup's expert: requested before anything else)
    [[maybe_unused]] RouteIds rid;
    if constexpr (ROUTED && MODE == GRID_EXPERTS) rid = inline_route_request(selected, ids_are_i64, n_flat, threadIdx.x);
    // (the arguments the start-up goes through, in scalar registers now: one batch of loads from the argument segment)
    asm volatile("" ::"s"(max_slabs), "s"(E), "s"(n_tiles), "s"(n_groups), "s"(n_tchunks), "s"(tiles_per_wg), "s"(n_work),
                 "s"(top_k));
    // Workgroup b runs on XCD b % 8, and every XCD has its own L2: the workgroups of one expert coordinate
    // (which all read the same G / U rows) are given ids of one residue class, so that they share one L2;
    // on the active-expert and the chunk grid coordinate c goes to XCD c % 8, so that the coordinates that have
    // work -- a prefix of them -- spread over all eight (26-layer stack at 32 tokens: 25.3 -> 15.2 us); on the expert
    // grid, where every coordinate may have work, XCD x takes a contiguous eighth (measured 2 % faster there).  The
    // grid holds 8 * ceil(coordinates / 8) * (workgroups per coordinate) ids; coordinates past the last exit.
    const int per_coord = n_tchunks * n_groups;
    const int k_in_xcd = blockIdx.x >> 3;
    const int coords_per_xcd = (int)(gridDim.x >> 3) / per_coord;
    const int e_slot = MODE == GRID_EXPERTS ? (int)(blockIdx.x & 7) * coords_per_xcd + k_in_xcd / per_coord
                                            : 8 * (k_in_xcd / per_coord) + (int)(blockIdx.x & 7);
    if (e_slot * per_coord >= n_work) return;
    const int tchunk = (k_in_xcd % per_coord) % n_tchunks;
    const int grp = (k_in_xcd % per_coord) / n_tchunks;
    const int tid = threadIdx.x;
    int e = e_slot, chunk = -1;
    if constexpr (MODE == GRID_ACTIVE && !ROUTED) {
        e = nth_active_expert(expert_offsets, E, A, e_slot, tid & 63);
    } else if constexpr (MODE == GRID_CHUNKS) {
        const ChunkRef ref = nth_chunk(expert_offsets, E, A, e_slot, tid & 63);
        e = ref.expert;
        chunk = ref.chunk;
    }
    if (e < 0) return;
    const int tb = tchunk * tiles_per_wg;
    const int nt = min(tiles_per_wg, n_tiles - tb);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int si = grp * DN_SLABS_PER_WG + wave;

    int a_begin = 0, a_end = 0, gid = -1;
    __shared__ std::conditional_t<ROUTED, InlineRouteLds, int> route_lds;
    FastExpert fe;
    FastSlab fs = FastSlab{0, 0, 0, 0};
    if constexpr (ROUTED && MODE == GRID_ACTIVE) {
        // `e` is an entry index: serve the expert it names if this is the expert's first entry (its local id and record
        // are asked for as soon as the entry's id is here; the scan of all ids runs meanwhile)
        const int slot = e;
        if (slot >= n_flat) return;
        const RouteIds all = inline_route_request(selected, ids_are_i64, n_flat, tid);
        gid = __builtin_amdgcn_readfirstlane(routed_id(selected, ids_are_i64, slot));
        if (gid < 0 || gid >= n_global) return;
        e = __builtin_amdgcn_readfirstlane(global_to_local[gid]);
        if (e < 0 || e >= E) return;
        fe = down_fe[e];
        if (si < max_slabs) fs = load_fast_slab(down_fs, e * max_slabs + si);
        a_end = inline_route_finish(all, n_flat, top_k, gid, route_lds, tid);
        hold_fast_expert(fe);
        if (a_end == 0 || route_lds.ent[0] != slot) return;
    } else {
        if constexpr (ROUTED) {
            gid = local_to_global[e];
        } else {
            a_begin = max(expert_offsets[e], 0);
            a_end = min(expert_offsets[e + 1], A);
            if (chunk >= 0) {      // this workgroup's chunk only
                a_begin += MAX_A * chunk;
                a_end = min(a_end, a_begin + MAX_A);
            }
        }
        fe = down_fe[e];
        if (si < max_slabs) fs = load_fast_slab(down_fs, e * max_slabs + si);
        hold_fast_expert(fe);
    }
    if constexpr (ROUTED && MODE == GRID_EXPERTS) {
        hold_route_ids(rid);
        a_end = inline_route_finish(rid, n_flat, top_k, gid, route_lds, tid);
    }
    if (a_end <= a_begin || grp * DN_SLABS_PER_WG >= fe.num_slabs) return;
    BITSMOE_TL(g_tl_down, 1);
    auto assignments = [&]() {
        if constexpr (ROUTED)
            return AssignInline{route_lds.tok, route_lds.ent, sel_weights, a_end};
        else
            return AssignTables{token_indices, route_w, A};
    };
    const auto as = assignments();

    gptr<uint32_t> payload = as_global(fe.payload);
    gptr<__half> scale = as_global(fe.scale);
    gptr<__half> svec = as_global(fe.s);
    gptr<int32_t> rank_idx = as_global(fe.rank_idx);
    extern __shared__ __attribute__((aligned(16))) unsigned char dsmem[];
    uint16_t* z = reinterpret_cast<uint16_t*>(dsmem);
    const int z_stride = tiles_per_wg * N_TILE + 8;      // (the workgroup's own tiles)
    float* zsum = reinterpret_cast<float*>(dsmem + (size_t)MAX_A * z_stride * 2);      // [assignment][tile]
    int2* rows = reinterpret_cast<int2*>(zsum + MAX_A * ZSUM_STRIDE) + wave * SLAB_ROWS;     // this wavefront's (rank, multiplier) per row
    int2* assigns = reinterpret_cast<int2*>(zsum + MAX_A * ZSUM_STRIDE) + DN_SLABS_PER_WG * SLAB_ROWS;    // (token, routing weight) per assignment

    // the four wavefronts may run four different instantiations; every one of them executes
    // the same two workgroup barriers per assignment chunk
    if (fs.bits == 2)
        down_wave<2, ZREADY, ZR, ZBY>(payload, scale, svec, rank_idx, fs, G, U, n_part, part_stride, as, a_begin, a_end, T, I, tb, nt,
                           rank_out, rank_accum, z, z_stride, zsum, rows, assigns, tid, lane);
    else if (fs.bits == 3)
        down_wave<3, ZREADY, ZR, ZBY>(payload, scale, svec, rank_idx, fs, G, U, n_part, part_stride, as, a_begin, a_end, T, I, tb, nt,
                           rank_out, rank_accum, z, z_stride, zsum, rows, assigns, tid, lane);
    else if (fs.bits == 4)
        down_wave<4, ZREADY, ZR, ZBY>(payload, scale, svec, rank_idx, fs, G, U, n_part, part_stride, as, a_begin, a_end, T, I, tb, nt,
                           rank_out, rank_accum, z, z_stride, zsum, rows, assigns, tid, lane);
    else
        down_wave<0, ZREADY, ZR, ZBY>(payload, scale, svec, rank_idx, fs, G, U, n_part, part_stride, as, a_begin, a_end, T, I, tb, nt,
                           rank_out, rank_accum, z, z_stride, zsum, rows, assigns, tid, lane);
    BITSMOE_TL(g_tl_down, 6);
}

__global__ void k_fill_zero2(float* __restrict__ p1, int64_t n1, float* __restrict__ p2, int64_t n2) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t i0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (int64_t i = i0; i < n1; i += stride) p1[i] = 0.0f;
    for (int64_t i = i0; i < n2; i += stride) p2[i] = 0.0f;
}

static inline void record(bitsmoe_profile* p, int i, hipStream_t st) {
    if (p) (void)hipEventRecord(p->ev[i], st);
}

bool decode_path_supported(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down, int I) {
    const int n_tiles = (I + N_TILE - 1) / N_TILE;
    const size_t z_bytes = (size_t)MAX_A * (n_tiles * N_TILE + 8) * 2 + MAX_A * ZSUM_STRIDE * 4 + DN_SLABS_PER_WG * SLAB_ROWS * 8 + MAX_A * 8;
    return n_tiles <= ZSUM_STRIDE && gate->role == ROLE_GATE_UP && up->role == ROLE_GATE_UP && down->role == ROLE_DOWN && z_bytes <= 65536;
}

// Can the decode kernels find their assignments among the routed ids themselves (no routing tables)?
bool decode_inline_route_ok(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down, const void* h_gate,
                            const void* h_up, int Rg, int Ru, int64_t ldg, int64_t ldu, int64_t T, int top_k, int I) {
    const int64_t n_flat = T * top_k;
    if (options().route_inline == 0) return false;       // always build routing tables first (experiments)
    if (has_wide_rows(gate) || has_wide_rows(up) || has_wide_rows(down)) return false;      // (their side kernels read the tables)
    if (!(decode_path_supported(gate, up, down, I) && walk_possible(gate, up, h_gate, h_up, Rg, Ru, ldg, ldu) &&
          options().decode_fused_z <= 0 && n_flat > 0 && n_flat <= ROUTE_INLINE_MAX_FLAT &&
          T <= ROUTE_INLINE_MAX_ROWS))
        return false;
    // Where it pays (graph replays, same box, against the routing kernel first).  On the active-expert grid
    // always: 3 to 5 us less per layer.  On the expert grid every expert's workgroups scan the ids, also those of
    // experts nobody chose, which with tables exit after one load: a gain of 1 to 3 us from two entries per
    // expert on average on a 128-expert layer of six tiles, a loss of 1 to 5 us below that, on layers of eleven
    // tiles (more workgroups per expert) and on a 512-expert layer.  The chunk grid keeps its tables.
    const int mode = decode_grid_mode(n_flat, gate->n_experts);
    if (mode == GRID_ACTIVE) return true;
    return mode == GRID_EXPERTS && n_flat >= policy::INLINE_ROUTE_MIN_ENTRIES_PER_EXPERT * (int64_t)gate->n_experts &&
           gate->n_experts <= policy::INLINE_ROUTE_MAX_EXPERTS && gate->n_tiles <= policy::INLINE_ROUTE_MAX_TILES;
}

int launch_forward_decode(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                          const void* h_gate, const void* h_up, int act_dtype, int64_t T, int Rg, int Ru, int64_t ldg,
                          int64_t ldu, const int32_t* tok, const int32_t* off, const float* rw, int64_t A, int rank_out,
                          int I, float* rank_accum, float* G, float* U, int64_t inter_floats, int part_capacity,
                          const DecodeRouted* routed, bitsmoe_profile* prof, hipStream_t st) {
    const int E = gate->n_experts;
    const int n_tiles = gate->n_tiles;
    // Dense experts (every row wide): the 2/3/4-bit kernels would run over padding only.  Clear the sums and the
    // output, then the side kernels alone.
    if (only_wide_rows(gate, up, down) && tok && off && rw) {
        record(prof, 0, st);
        const int64_t n1 = inter_floats + A * (int64_t)I, n2 = T * (int64_t)rank_out;
        hipLaunchKernelGGL(k_fill_zero2, dim3((unsigned)std::min<int64_t>((std::max(n1, n2) + 255) / 256, 2048)), dim3(256), 0, st, G,
                           n1, rank_accum, n2);
        BITSMOE_HIP_TRY(hipGetLastError());
        record(prof, 1, st);
        int rc = launch_wide_gateup(gate, up, h_gate, h_up, act_dtype, Rg, Ru, ldg, ldu, tok, off, A, I, G, U, false, st);
        if (rc != BITSMOE_OK) return rc;
        record(prof, 2, st);
        record(prof, 3, st);
        rc = launch_wide_down(down, G, U, false, 1, 2 * inter_floats, tok, off, rw, A, I, rank_out, rank_accum, st);
        if (rc != BITSMOE_OK) return rc;
        record(prof, 4, st);
        record(prof, 5, st);
        if (prof) prof->recorded = true;
        return BITSMOE_OK;
    }
    // The whole chain in one kernel per (expert, tile) where the sets allow it (option decode_fused = 0 / 1: never /
    // wherever possible).
    if (options().decode_fused != 0 && options().decode_fused_z <= 0 &&
        decode_fused_possible(gate, up, down, h_gate, h_up, Rg, Ru, ldg, ldu, I) &&
        (options().decode_fused > 0 || decode_fused_chosen(gate, A, I)))
        return launch_forward_decode_fused(gate, up, down, h_gate, h_up, act_dtype, T, Rg, Ru, ldg, ldu, tok, off, rw, A, rank_out,
                                           I, rank_accum, routed, prof, st);
    record(prof, 0, st);
    // What the expert coordinate of the grids counts.  Few assignments: the experts that can be
    // active at most, not all of them.  Sixteen or more assignments per expert on average: most
    // experts have several 16-assignment chunks, one workgroup per chunk.  Below that the search
    // of the chunk (one more dependent round trip per workgroup, +10 %) costs more than walking
    // an expert's few chunks in a loop, unless routing is skewed: with at most 64 experts (one
    // search step) the chunk grid is already used from three assignments per expert on average.
    // At most min(E, A) experts can be active.
    const int64_t active_max = std::min<int64_t>(E, A);
    const int mode = decode_grid_mode(A, E);
    const int e_dim = mode == GRID_CHUNKS ? (int)(active_max + A / MAX_A) : mode == GRID_ACTIVE ? (int)active_max : E;
    // (expert, chunk) pairs expected to have work (e_dim is their upper bound in chunk mode)
    const int64_t units = mode == GRID_CHUNKS ? A / MAX_A + active_max / 2 : active_max;
    // Sets of affine single-width experts, enough (expert, tile) pairs to fill the chip: the
    // walking gate/up kernel, which also clears rank_accum and needs no cleared G / U.
    // (its 16-byte activation loads also need rank_idx in runs of eight and aligned rows)
    const bool walk = walk_possible(gate, up, h_gate, h_up, Rg, Ru, ldg, ldu);
    // Both projections in one workgroup, z = silu(G) * U handed to the down kernel ready-made: when the two
    // matrices of every expert share bit-width and slab count, and (expert, tile) pairs alone fill most of
    // the chip.  BITSMOE_DECODE_FUSED_Z=0 / 1 switches it off / on regardless of the size (experiments).
    const int fused_env = options().decode_fused_z;
    const bool wide_gu = has_wide_rows(gate) || has_wide_rows(up);
    const bool fused_possible = walk && gate->all_affine && up->all_affine && gate->prep_max_slabs == up->prep_max_slabs &&
                                gate->expert_bits == up->expert_bits && !wide_gu;
    const bool fused_z = fused_possible && fused_env > 0;
    if (!walk) {
        // G and U are adjacent in the workspace: one range; rank_accum is the second
        const int64_t n1 = inter_floats + A * (int64_t)I;
        const int64_t n2 = T * (int64_t)rank_out;
        const int64_t blocks = std::min<int64_t>((std::max(n1, n2) + 255) / 256, 2048);
        hipLaunchKernelGGL(k_fill_zero2, dim3((unsigned)blocks), dim3(256), 0, st, G, n1, rank_accum, n2);
        BITSMOE_HIP_TRY(hipGetLastError());
    }
    record(prof, 1, st);
    const int max_slabs = std::max(gate->prep_max_slabs, up->prep_max_slabs);
    const int gu_groups = (max_slabs + GU_SLABS - 1) / GU_SLABS;
    // Tiles per workgroup: long runs amortise the start-up round trips, but the grid must
    // still hold a few workgroups per CU (two rounds of three per CU measured best).
    int tiles_per_wg = n_tiles;
    while (tiles_per_wg > 1 &&
           units * 2 * gu_groups * ((n_tiles + tiles_per_wg - 1) / tiles_per_wg) < policy::GATEUP_DECODE_MIN_WORKGROUPS)
        tiles_per_wg = (tiles_per_wg + 1) / 2;
    const int n_tchunks = (n_tiles + tiles_per_wg - 1) / tiles_per_wg;
    dim3 grid((unsigned)(e_dim * gu_groups * n_tchunks), 2);
    // the expert a grid coordinate stands for: by decreasing payload size, or the identity
    auto order_of = [&](const bitsmoe_matset* set) {
        ExpertOrder o{};
        for (int i = 0; i < EXPERT_ORDER_MAX; ++i) o.set(i, set->has_cost_order && i < E ? set->cost_order[i] : (uint16_t)i);
        return o;
    };
    const ExpertOrder gate_order = order_of(gate), up_order = order_of(up);
    auto launch_gateup = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, st, gate->d_fast_experts, gate->d_fast_slabs, gate->prep_max_slabs,
                           up->d_fast_experts, up->d_fast_slabs, up->prep_max_slabs, (const uint16_t*)h_gate,
                           (const uint16_t*)h_up, Rg, Ru, ldg, ldu, tok, off, (int)T, (int)A, I, E, n_tiles, gu_groups, n_tchunks,
                           tiles_per_wg, G, U, gate_order, up_order);
    };
    const bool need_general = !(gate->all_uniform8 && up->all_uniform8);
    const bool bf16 = act_dtype == BITSMOE_DT_BF16;
    auto launch_gateup_mode = [&](auto bf16_c, auto mode_c) {
        constexpr bool B = decltype(bf16_c)::value;
        constexpr int M = decltype(mode_c)::value;
        launch_gateup(k_gateup_decode<B, false, M>);
        if (need_general) launch_gateup(k_gateup_decode<B, true, M>);
    };
    auto with_mode = [&](auto fn, auto bf16_c) {
        if (mode == GRID_CHUNKS)
            fn(bf16_c, std::integral_constant<int, GRID_CHUNKS>{});
        else if (mode == GRID_ACTIVE)
            fn(bf16_c, std::integral_constant<int, GRID_ACTIVE>{});
        else
            fn(bf16_c, std::integral_constant<int, GRID_EXPERTS>{});
    };
    // The walking kernel's workgroups: one per item, unless the items fill less than half of the chip's
    // `slots` (four resident workgroups per CU): then every item is split over `split` workgroups, each of
    // which contracts over a share of the slab groups, and the down kernel adds the `n_part` partial results
    // up.  (Halving only the cheapest items of a grid whose final batch of workgroups is partly empty -- 1536 items on 1024
    // slots -- was measured too: the gate/up kernel gains nothing, the down kernel's SiLU pass reads twice as much.)
    const int64_t n_items = (int64_t)e_dim * n_tiles * 2;
    const int64_t slots = 4 * (int64_t)cu_count();
    const int max_part = (int)std::min<int64_t>(part_capacity, 4);
    int64_t n_unsplit = n_items;
    int split = 1;
    if (walk && !fused_z && n_items * 2 <= slots) {
        while (split * 2 <= max_part && split * 2 <= gu_groups && n_items * split * 2 <= slots) split *= 2;
        if (split > 1) n_unsplit = 0;
    }
    const int n_part = n_unsplit < n_items ? split : 1;
    const int64_t part_stride = 2 * inter_floats;
    auto launch_walk_mode = [&](auto bf16_c, auto mode_c) {
        // (one width per expert in both sets: the kernel compiled for that; else the one that switches per slab group)
        const bool ident = gate->rank_identity && up->rank_identity;
        const bool mixed = !(gate->uniform_experts && up->uniform_experts);
        constexpr bool B = decltype(bf16_c)::value;
        constexpr int M = decltype(mode_c)::value;
        auto kern = mixed ? (ident ? k_gateup_walk<B, M, true, true, false> : k_gateup_walk<B, M, false, true, false>)
                          : (ident ? k_gateup_walk<B, M, true, false, false> : k_gateup_walk<B, M, false, false, false>);
        if constexpr (M != GRID_CHUNKS) {
            if (routed)
                kern = mixed ? (ident ? k_gateup_walk<B, M, true, true, true> : k_gateup_walk<B, M, false, true, true>)
                             : (ident ? k_gateup_walk<B, M, true, false, true> : k_gateup_walk<B, M, false, false, true>);
        }
        hipLaunchKernelGGL(kern, dim3((unsigned)(n_unsplit + (n_items - n_unsplit) * split)), dim3(256), 0, st,
                           gate->d_fast_experts, gate->d_fast_slabs, gate->prep_max_slabs, up->d_fast_experts,
                           up->d_fast_slabs, up->prep_max_slabs, (const uint16_t*)h_gate, (const uint16_t*)h_up, ldg, ldu,
                           tok, off, (int)T, (int)A, I, E, n_tiles, G, U, (int)n_unsplit, split, n_part, part_stride, rank_accum,
                           T * (int64_t)rank_out, gate_order, up_order, routed ? routed->selected : nullptr,
                           routed ? routed->ids_are_i64 : 0, routed ? (int)A : 0, routed ? routed->top_k : 1,
                           routed ? routed->local_to_global : nullptr, routed ? routed->global_to_local : nullptr,
                           routed ? routed->n_global : 0);
    };
    auto launch_walk_z_mode = [&](auto bf16_c, auto mode_c) {
        auto kern = k_gateup_walk_z<decltype(bf16_c)::value, decltype(mode_c)::value, false>;
        if (gate->rank_identity && up->rank_identity) kern = k_gateup_walk_z<decltype(bf16_c)::value, decltype(mode_c)::value, true>;
        // Z takes the place of G in the workspace, Zsum that of U
        hipLaunchKernelGGL(kern, dim3((unsigned)(e_dim * n_tiles)), dim3(256), 0, st, gate->d_fast_experts, gate->d_fast_slabs,
                           up->d_fast_experts, up->d_fast_slabs, gate->prep_max_slabs, (const uint16_t*)h_gate, (const uint16_t*)h_up,
                           ldg, ldu, tok, off, (int)T, (int)A, I, E, n_tiles, (uint16_t*)G, U, rank_accum,
                           T * (int64_t)rank_out, gate_order);
    };
    if (fused_z) {
        if (bf16)
            with_mode(launch_walk_z_mode, std::true_type{});
        else
            with_mode(launch_walk_z_mode, std::false_type{});
    } else if (walk) {
        if (bf16)
            with_mode(launch_walk_mode, std::true_type{});
        else
            with_mode(launch_walk_mode, std::false_type{});
    } else if (bf16) {
        with_mode(launch_gateup_mode, std::true_type{});
    } else {
        with_mode(launch_gateup_mode, std::false_type{});
    }
    BITSMOE_HIP_TRY(hipGetLastError());
    // rows of 6-, 8- and 16-bit slabs: their share of the gate and up sums, added to the first partial result
    if (wide_gu) {
        const int rc = launch_wide_gateup(gate, up, h_gate, h_up, act_dtype, Rg, Ru, ldg, ldu, tok, off, A, I, G, U, false, st);
        if (rc != BITSMOE_OK) return rc;
    }
    record(prof, 2, st);
    // z formed once by a small launch of its own instead of by every down workgroup: on the chunk grid (full
    // 16-assignment chunks: eight dependent round trips of two rows each in every one of the workgroups that share
    // a chunk), when the workspace has a free slot behind the partial results.  option decode_split_z = 0 / 1
    // switches it off / on wherever it is possible (experiments).
    const int split_z_env = options().decode_split_z;
    const bool split_z_possible = !fused_z && !routed && (walk ? n_part : 1) < part_capacity && I % 4 == 0;
    const bool split_z = split_z_possible && (split_z_env >= 0 ? split_z_env > 0 : mode == GRID_CHUNKS);
    const int parts_in = walk && !fused_z ? n_part : 1;
    float* down_g = G;
    float* down_u = U;
    if (split_z) {
        uint16_t* Z = reinterpret_cast<uint16_t*>(G + parts_in * part_stride);
        float* Zsum = U + parts_in * part_stride;
        const int64_t threads = A * (int64_t)n_tiles * 32;
        hipLaunchKernelGGL(k_decode_silu, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, G, U, parts_in, part_stride,
                           (int)A, I, n_tiles, Z, Zsum);
        BITSMOE_HIP_TRY(hipGetLastError());
        down_g = reinterpret_cast<float*>(Z);
        down_u = Zsum;
    }
    record(prof, 3, st);      // (otherwise SiLU happens inside the down kernel)
    const int dn_groups = (down->prep_max_slabs + DN_SLABS_PER_WG - 1) / DN_SLABS_PER_WG;
    int dn_tiles_per_wg = n_tiles;
    // (600 measured best on the 26-layer stack at 32 tokens against 300, 1200 and 2400: the kernel is bound by the
    // instructions a workgroup issues, and more, shorter workgroups add their fixed part)
    while (dn_tiles_per_wg > 1 &&
           units * dn_groups * ((n_tiles + dn_tiles_per_wg - 1) / dn_tiles_per_wg) < policy::DOWN_DECODE_MIN_WORKGROUPS)
        dn_tiles_per_wg = (dn_tiles_per_wg + 1) / 2;
    const size_t z_bytes = (size_t)MAX_A * (dn_tiles_per_wg * N_TILE + 8) * 2 + MAX_A * ZSUM_STRIDE * 4 + DN_SLABS_PER_WG * SLAB_ROWS * 8 + MAX_A * 8;
    const int dn_tchunks = (n_tiles + dn_tiles_per_wg - 1) / dn_tiles_per_wg;
    auto launch_down = [&](auto kernel) {
        const int n_work = e_dim * dn_groups * dn_tchunks;
        hipLaunchKernelGGL(kernel, dim3((unsigned)((e_dim + 7) / 8 * 8 * dn_groups * dn_tchunks)), dim3(256), z_bytes, st, down->d_fast_experts,
                           down->d_fast_slabs, down->prep_max_slabs, down_g, down_u, split_z ? 1 : parts_in, part_stride, rw, tok, off,
                           (int)T, (int)A, I, E, n_tiles, dn_groups, dn_tchunks, dn_tiles_per_wg, n_work, rank_out, rank_accum,
                           routed ? routed->selected : nullptr, routed ? routed->ids_are_i64 : 0, routed ? (int)A : 0,
                           routed ? routed->top_k : 1, routed ? routed->local_to_global : nullptr,
                           routed ? routed->weights : nullptr, routed ? routed->global_to_local : nullptr,
                           routed ? routed->n_global : 0);
    };
    auto launch_down_mode = [&](auto zready_c, auto mode_c) {
        constexpr int M = decltype(mode_c)::value;
        constexpr bool Z = decltype(zready_c)::value;
        // (z beyond 40 KB: at most three workgroups per CU fit the LDS, the kernel compiled for three takes more
        // rows of G / U per round trip)
        const bool wide = !Z && z_bytes > 40 * 1024;
        if constexpr (M != GRID_CHUNKS && !Z) {
            if (routed) {
                if (wide)
                    launch_down(k_down_decode<M, Z, true, ZROWS_WIDE>);
                else
                    launch_down(k_down_decode<M, Z, true, ZROWS>);
                return;
            }
        }
        if constexpr (!Z) {
            if (wide) {
                launch_down(k_down_decode<M, Z, false, ZROWS_WIDE>);
                return;
            }
        }
        // z a row per wavefront: from five assignments per expert on average (512-expert layer, 256 tokens, top-10: the
        // kernel 5 % faster; 128 experts with four per expert: no difference; with one or two: slower)
        if constexpr (!Z && M != GRID_CHUNKS) {
            if (A >= policy::DOWN_Z_BY_ROWS_MIN_PER_EXPERT * (int64_t)E) {
                launch_down(k_down_decode<M, Z, false, ZROWS, true>);
                return;
            }
        }
        launch_down(k_down_decode<M, Z, false, ZROWS>);
    };
    // (G and U are fp32 and the operands f16 whatever the activation type was)
    if (fused_z || split_z)
        with_mode(launch_down_mode, std::true_type{});
    else
        with_mode(launch_down_mode, std::false_type{});
    BITSMOE_HIP_TRY(hipGetLastError());
    if (has_wide_rows(down)) {      // (behind the gate/up kernel, which cleared rank_accum)
        const int rc = launch_wide_down(down, down_g, down_u, split_z, split_z ? 1 : parts_in, part_stride, tok, off, rw, A, I,
                                        rank_out, rank_accum, st);
        if (rc != BITSMOE_OK) return rc;
    }
    record(prof, 4, st);
    record(prof, 5, st);      // (the combine too)
    if (prof) prof->recorded = true;
    return BITSMOE_OK;
}

}  // namespace bitsmoe

#ifdef BITSMOE_TIMELINE
// which: 0 = k_gateup_walk, 1 = k_down_decode
extern "C" int bitsmoe_timeline_read_decode(int which, unsigned long long* host, int n_workgroups) {
    using namespace bitsmoe;
    if (!host || n_workgroups <= 0 || n_workgroups > TL_MAX_WG || which < 0 || which > 1) return BITSMOE_E_INVALID;
    BITSMOE_HIP_TRY(hipDeviceSynchronize());
    const size_t bytes = sizeof(unsigned long long) * TL_STAMPS * n_workgroups;
    if (which == 0)
        BITSMOE_HIP_TRY(hipMemcpyFromSymbol(host, HIP_SYMBOL(g_tl_walk), bytes));
    else
        BITSMOE_HIP_TRY(hipMemcpyFromSymbol(host, HIP_SYMBOL(g_tl_down), bytes));
    return BITSMOE_OK;
}
extern "C" int bitsmoe_timeline_clear_decode(void) {
    using namespace bitsmoe;
    void* p = nullptr;
    BITSMOE_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(g_tl_walk)));
    BITSMOE_HIP_TRY(hipMemset(p, 0, sizeof(unsigned long long) * TL_STAMPS * TL_MAX_WG));
    BITSMOE_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(g_tl_down)));
    BITSMOE_HIP_TRY(hipMemset(p, 0, sizeof(unsigned long long) * TL_STAMPS * TL_MAX_WG));
    return BITSMOE_OK;
}
#endif
