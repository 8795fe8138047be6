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
#include <type_traits>
#include <utility>

#include "fast_helpers.h"

namespace bitsmoe {

constexpr int GU_STRIDE = GU_SLABS * SLAB_ROWS + 8;  // 16-bit elements; +8 staggers LDS banks
constexpr int DN_SLABS_PER_WG = 4;                 // one slab per wavefront
constexpr int MAX_A = 16;                          // assignments per MFMA pass
constexpr int ZROWS = 2;                           // assignment rows of G / U the down kernel's z build fetches together
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
        if (E <= EXPERT_ORDER_MAX) e = mt ? up_order.e[e] : gate_order.e[e];
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
// The same contraction for sets in which every expert is one affine run of equal-width slabs
// (bitsmoe_matset::all_affine) whose rank_idx maps every aligned run of eight rows to eight
// consecutive ranks (rank_chunked8): a workgroup takes one expert, one projection and ONE
// 128-column tile and walks all slab groups, keeping the tile's accumulators in registers.
//  * Every output element has exactly one owner: plain stores instead of fp32 atomics, no zero
//    fill of G / U beforehand.
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
// A token index out of range is clamped for the address: the down kernel ignores such an
// assignment, whatever its G / U rows hold.
// The kernel also clears `zero_out` (the forward's accumulator, added into by the down kernel).
// grid.x = (expert coordinate) * n_tiles, grid.y = 2 (gate, up); 256 threads = 4 wavefronts.
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

template <bool BF16, int MODE, bool IDENT>
__global__ __launch_bounds__(256, 4) void k_gateup_walk(
    const FastExpert* __restrict__ gate_fe, const FastSlab* __restrict__ gate_fs, int gate_max_slabs,
    const FastExpert* __restrict__ up_fe, const FastSlab* __restrict__ up_fs, int up_max_slabs,
    const uint16_t* __restrict__ h_gate, const uint16_t* __restrict__ h_up, int64_t ldg, int64_t ldu,
    const int32_t* __restrict__ token_indices, const int32_t* __restrict__ expert_offsets, int T, int A, int I,
    int E, int n_tiles, float* __restrict__ G, float* __restrict__ U, float* __restrict__ zero_out,
    int64_t zero_n, const ExpertOrder gate_order, const ExpertOrder up_order) {
    const int mt = blockIdx.y;
    const int bid = blockIdx.x;
    const int tid = threadIdx.x;
    {   // this workgroup's share of the accumulator (before any exit)
        const int64_t total = (int64_t)gridDim.x * 2 * 256;
        for (int64_t i = ((int64_t)mt * gridDim.x + bid) * 256 + tid; i < zero_n; i += total) zero_out[i] = 0.0f;
    }
    const int t = bid % n_tiles;
    int e = bid / n_tiles;
    int chunk = -1;
    if constexpr (MODE == GRID_EXPERTS) {      // expensive experts first (the identity when there is no order)
        if (E <= EXPERT_ORDER_MAX) e = mt ? up_order.e[e] : gate_order.e[e];
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

    // one round trip: assignment range, expert record, the record of the expert's first slab
    int a_begin = max(expert_offsets[e], 0);
    int a_end = min(expert_offsets[e + 1], A);
    if (chunk >= 0) {
        a_begin += MAX_A * chunk;
        a_end = min(a_end, a_begin + MAX_A);
    }
    const FastExpert* __restrict__ fe_tab = mt ? up_fe : gate_fe;
    const FastSlab* __restrict__ fs_tab = mt ? up_fs : gate_fs;
    const int max_slabs = mt ? up_max_slabs : gate_max_slabs;
    const FastExpert fe = fe_tab[e];
    const FastSlab first = load_fast_slab(fs_tab, e * max_slabs);
    if (a_end <= a_begin || first.bits == 0) return;
    const int n_groups = max_slabs / GU_SLABS;

    gptr<uint32_t> payload = as_global(fe.payload);
    gptr<__half> scale_s = as_global(fe.scale_s);
    gptr<int32_t> rank_idx = as_global(fe.rank_idx);
    const uint16_t* __restrict__ h = mt ? h_up : h_gate;
    const int64_t ld = mt ? ldu : ldg;
    float* __restrict__ out = mt ? U : G;
    const uint32_t unit = (uint32_t)(pair * 64 + lane);
    const uint32_t hi_unit = (uint32_t)hi_index0(kg, n, 2 * pair);

    // two copies of the operand, used in turn: one workgroup barrier per group instead of two
    __shared__ __attribute__((aligned(16))) uint16_t hs_all[2 * MAX_A * GU_STRIDE];
    __shared__ float cterm_lds[MAX_A];

    auto body = [&](auto w_c) {
    constexpr int W = decltype(w_c)::value;
    const int slab_words = n_tiles * 256 * W;       // payload words from one slab to the next
    Masks3 m3;
    if constexpr (W == 3) m3 = masks3_role0();
    for (int a0 = a_begin; a0 < a_end; a0 += MAX_A) {
        const int n_a = min(MAX_A, a_end - a0);
        int chunk_zero = 0;
        asm volatile("" : "+s"(chunk_zero));   // keeps this chunk's address arithmetic inside the loop
        const int pack0 = first.pack_off + t * 256 * W + chunk_zero;

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
        for (int i = 0; i < 4; ++i) tki[i] = token_indices[min(a0 + pair + 4 * i, A - 1)];
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
        int rank_cur = rank_at(0);
        int rank_nxt = n_groups > 1 ? rank_at(1) : 0;
        u32x4 sc_cur = scale_at(0);
        // (the token indices are first used here, behind the requests that do not depend on them)
#pragma unroll
        for (int i = 0; i < 4; ++i) trow[i] = h + (int64_t)min(max(__builtin_amdgcn_readfirstlane(tki[i]), 0), T - 1) * ld;
        u32x4 raw0 = {0, 0, 0, 0}, raw1 = {0, 0, 0, 0};
        // (requested whether or not the assignments exist -- a row of token 0 otherwise -- so that
        // the number of loads in flight does not depend on the path and the waits can be counted)
        raw0 = act_at(0, rank_cur);
        raw1 = act_at(1, rank_cur);
        // The payload of the first group is requested only now: loads return in order, so anything
        // requested behind it would be held back until it has arrived from HBM, and the first
        // operand could not be staged in the meantime.
        static_for([&](auto qc) { issue(qc, 0); }, std::make_integer_sequence<int, GU_SLABS>{});
        f32x4 acc[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
        f32x4 corr = {0, 0, 0, 0};
        // (MORE: another group follows -- compiled twice, so that the eight blocks of a group are
        // one straight run of code the compiler can schedule across)
        auto group_step = [&](auto more_c, int g) {
            constexpr bool more = decltype(more_c)::value;
            int rank_nxt2 = 0;
            if (g + 2 < n_groups) rank_nxt2 = rank_at(g + 2);
            u32x4 sc_nxt = {0, 0, 0, 0};
            if constexpr (more) sc_nxt = scale_at(g + 1);
            // Group g writes copy g mod 2.  Its last readers (group g - 2) are done: every wavefront
            // passed the barrier of group g - 1 after its MFMAs of group g - 2.  Only a new chunk
            // needs a barrier of its own before the first write.
            hs = hs_all + (g & 1) * (MAX_A * GU_STRIDE);
            if (g == 0) __syncthreads();
            if (pair < n_a) stage(I0{}, raw0, sc_cur);
            if (pair + 4 < n_a) stage(I1{}, raw1, sc_cur);
            if (pair + 8 < n_a) stage(I2{}, act_at(2, rank_cur), sc_cur);      // (rare: fetched here, not ahead)
            if (pair + 12 < n_a) stage(I3{}, act_at(3, rank_cur), sc_cur);
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
                if constexpr (more) issue(qc, g + 1);
            }, std::make_integer_sequence<int, GU_SLABS>{});
            sc_cur = sc_nxt;
            rank_cur = rank_nxt;
            rank_nxt = rank_nxt2;
        };
        for (int g = 0; g + 1 < n_groups; ++g) group_step(std::true_type{}, g);
        group_step(std::false_type{}, n_groups - 1);
        // the constant terms of the chunk's assignments, from the wavefronts that staged them
        if (lane == 63) {
#pragma unroll
            for (int i = 0; i < 4; ++i) cterm_lds[pair + 4 * i] = cterm[i];
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j) corr[j] = cterm_lds[4 * kg + j];
        // remove the constant term; lane holds rows a = 4*kg + j of column 32*pair + 16*nbl + n
#pragma unroll
        for (int nbl = 0; nbl < 2; ++nbl) {
            const int c = t * N_TILE + 32 * pair + 16 * nbl + n;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int a = 4 * kg + j;
                if (a < n_a && c < I) out[(int64_t)(a0 + a) * I + c] = acc[nbl][j] - corr[j];
            }
        }
    }
    };   // body

    if (first.bits == 2)
        body(std::integral_constant<int, 2>{});
    else if (first.bits == 3)
        body(std::integral_constant<int, 3>{});
    else if (first.bits == 4)
        body(std::integral_constant<int, 4>{});
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
                bw = decode_fields3<false>(b.w[nb * 2 + (m >> 1)], 8 * (m & 1), b.w[8 + nb], 4 * m);
            t = mfma16<false>(az[m], bw, t);
        }
        acc[nb] += (t - corr) * sc[nb];
    }
}

// Everything one wavefront of the down kernel does after the metadata has arrived, compiled
// per bit-width of the wavefront's slab (W == 0: no slab, the wavefront only helps to build z).
// The payload of the first two tiles is requested BEFORE z is built, so that the weights
// are in flight while G and U are read and SiLU is evaluated; afterwards the tiles stream
// through three register buffers, two tiles ahead of the one being computed (4-bit slabs, 16
// registers per tile: two buffers, one tile ahead).  The register budget is 128, so that all four
// workgroups of a CU -- on the 64-token benchmark layer the whole grid -- are resident at once:
// what only the epilogue needs (rank and multiplier of the rows, token and weight of the
// assignments) waits in LDS, and z is built two assignment rows at a time.
template <int W>
__device__ __forceinline__ void down_wave(gptr<uint32_t> payload, gptr<__half> scale, gptr<__half> svec, gptr<int32_t> rank_idx,
                                 const FastSlab fs, const float* __restrict__ G, const float* __restrict__ U,
                                 const float* __restrict__ route_w, const int32_t* __restrict__ token_indices,
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
        Block16 buf[3];
        float sc[3][4];
        f32x4 acc[4];
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) acc[nb] = f32x4{0, 0, 0, 0};
        // the workgroup's tiles are tb .. tb + nt - 1; `i` counts from 0
        auto issue = [&](auto b_c, int i) {
            constexpr int B = decltype(b_c)::value;
            const int t = tb + i;
            load_block_role1<WL>(payload + (uint32_t)(fs.pack_off + (t + chunk_zero) * 256 * WL), lane, buf[B]);
            gptr<__half> sp = scale + (uint32_t)(fs.scale_off + t * SLAB_ROWS + n);
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) sc[B][nb] = gload_half(sp + 16 * nb);
        };
        auto compute = [&](auto b_c, int i) {
            constexpr int B = decltype(b_c)::value;
            u32x4 az[4];
            const uint16_t* zp = z + n * z_stride + (tb + i) * N_TILE + 8 * kg;
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
            issue(I0{}, 0);
            if (nt > 1) issue(I1{}, 1);
            row_rank = rank_idx[fs.rank_off + lane];
            row_s = gload_half(svec + fs.rank_off + lane);
        }
        // token ids and routing weights of the chunk (lane a holds assignment a): for the epilogue,
        // kept in LDS until then (every wavefront writes the same sixteen entries)
        const int tok_lane = (lane < n_a) ? token_indices[a0 + lane] : -1;
        const float rw_lane = (lane < n_a) ? route_w[a0 + lane] : 0.0f;
        __syncthreads();   // the previous chunk is done with z
        // z[a][c] = silu(G) * U as 16-bit operands for the rows a < n_a (other rows feed
        // output rows that are never stored).  Each thread owns four neighbouring columns
        // and walks the assignments ZROWS at a time, their vector loads issued together.
        for (int c = tb * N_TILE + tid * 4; c < min((tb + nt) * N_TILE, I); c += 1024) {
            for (int ab = 0; ab < n_a; ab += ZROWS) {
                f32x4 gv[ZROWS], uv[ZROWS];
#pragma unroll
                for (int j = 0; j < ZROWS; ++j) {
                    const int a = min(ab + j, n_a - 1);
                    const int64_t gi = (int64_t)(a0 + a) * I + c;
                    gv[j] = *reinterpret_cast<const f32x4*>(G + gi);
                    uv[j] = *reinterpret_cast<const f32x4*>(U + gi);
                }
#pragma unroll
                for (int j = 0; j < ZROWS; ++j) {
                    if (ab + j < n_a) {
                        uint16_t zb[4];
                        float part = 0.0f;      // sum of the four operands as rounded
#pragma unroll
                        for (int x = 0; x < 4; ++x) {
                            zb[x] = to_operand<false>(silu_f32(gv[j][x]) * uv[j][x]);
                            part += __half2float(__ushort_as_half(zb[x]));
                        }
                        u32x2 packed;
                        packed[0] = (uint32_t)zb[0] | ((uint32_t)zb[1] << 16);
                        packed[1] = (uint32_t)zb[2] | ((uint32_t)zb[3] << 16);
                        *reinterpret_cast<u32x2*>(z + (ab + j) * z_stride + c) = packed;
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
        if constexpr (W == 4) {
            // (16 payload registers per tile: two buffers, one tile ahead)
            for (int i = 0; i < nt; i += 2) {
                compute(I0{}, i);
                if (i + 1 < nt) {
                    if (i + 2 < nt) issue(I0{}, i + 2);
                    compute(I1{}, i + 1);
                    if (i + 3 < nt) issue(I1{}, i + 3);
                }
            }
        } else if constexpr (W != 0) {
            for (int i = 0; i < nt; i += 3) {
                if (i + 2 < nt) issue(I2{}, i + 2);
                compute(I0{}, i);
                if (i + 1 < nt) {
                    if (i + 3 < nt) issue(I0{}, i + 3);
                    compute(I1{}, i + 1);
                }
                if (i + 2 < nt) {
                    if (i + 4 < nt) issue(I1{}, i + 4);
                    compute(I2{}, i + 2);
                }
            }
        }
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
    }
}

// grid.x = E * n_groups * n_tchunks; 256 threads; dynamic LDS = z (16 * (n_tiles * 128 + 8) * 2 bytes), the
// per-tile sums of its rows, the epilogue's row and assignment records.
// A workgroup takes four slabs of one expert and a run of tiles; with few active experts the
// tiles are split over several workgroups (their partial sums meet in the atomics of the combine).
template <int MODE>
__global__ __launch_bounds__(256, 4) void k_down_decode(
    const FastExpert* __restrict__ down_fe, const FastSlab* __restrict__ down_fs, int max_slabs,
    const float* __restrict__ G, const float* __restrict__ U, const float* __restrict__ route_w,
    const int32_t* __restrict__ token_indices, const int32_t* __restrict__ expert_offsets, int T, int A, int I,
    int E, int n_tiles, int n_groups, int n_tchunks, int tiles_per_wg, int n_work, int rank_out,
    float* __restrict__ rank_accum) {
    // Workgroup b runs on XCD b % 8, and every XCD has its own L2: the workgroups of one expert
    // (which all read that expert's G / U rows) are given ids of one residue class, so that they
    // share one L2.  The grid is a multiple of 8; ids past the work exit.
    const int per_xcd = gridDim.x >> 3;
    const int bid = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (bid >= n_work) return;
    const int tchunk = bid % n_tchunks;
    const int grp = (bid / n_tchunks) % n_groups;
    const int e_slot = bid / (n_tchunks * n_groups);
    const int tid = threadIdx.x;
    int e = e_slot, chunk = -1;
    if constexpr (MODE == GRID_ACTIVE) {
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

    int a_begin = max(expert_offsets[e], 0);
    int a_end = min(expert_offsets[e + 1], A);
    if (chunk >= 0) {      // this workgroup's chunk only
        a_begin += MAX_A * chunk;
        a_end = min(a_end, a_begin + MAX_A);
    }
    const FastExpert fe = down_fe[e];
    FastSlab fs = FastSlab{0, 0, 0, 0};
    if (si < max_slabs) fs = load_fast_slab(down_fs, e * max_slabs + si);
    if (a_end <= a_begin || grp * DN_SLABS_PER_WG >= fe.num_slabs) return;

    gptr<uint32_t> payload = as_global(fe.payload);
    gptr<__half> scale = as_global(fe.scale);
    gptr<__half> svec = as_global(fe.s);
    gptr<int32_t> rank_idx = as_global(fe.rank_idx);
    extern __shared__ __attribute__((aligned(16))) unsigned char dsmem[];
    uint16_t* z = reinterpret_cast<uint16_t*>(dsmem);
    const int z_stride = n_tiles * N_TILE + 8;
    float* zsum = reinterpret_cast<float*>(dsmem + (size_t)MAX_A * z_stride * 2);      // [assignment][tile]
    int2* rows = reinterpret_cast<int2*>(zsum + MAX_A * ZSUM_STRIDE) + wave * SLAB_ROWS;     // this wavefront's (rank, multiplier) per row
    int2* assigns = reinterpret_cast<int2*>(zsum + MAX_A * ZSUM_STRIDE) + DN_SLABS_PER_WG * SLAB_ROWS;    // (token, routing weight) per assignment

    // the four wavefronts may run four different instantiations; every one of them executes
    // the same two workgroup barriers per assignment chunk
    if (fs.bits == 2)
        down_wave<2>(payload, scale, svec, rank_idx, fs, G, U, route_w, token_indices, a_begin, a_end, T, I, tb, nt,
                           rank_out, rank_accum, z, z_stride, zsum, rows, assigns, tid, lane);
    else if (fs.bits == 3)
        down_wave<3>(payload, scale, svec, rank_idx, fs, G, U, route_w, token_indices, a_begin, a_end, T, I, tb, nt,
                           rank_out, rank_accum, z, z_stride, zsum, rows, assigns, tid, lane);
    else if (fs.bits == 4)
        down_wave<4>(payload, scale, svec, rank_idx, fs, G, U, route_w, token_indices, a_begin, a_end, T, I, tb, nt,
                           rank_out, rank_accum, z, z_stride, zsum, rows, assigns, tid, lane);
    else
        down_wave<0>(payload, scale, svec, rank_idx, fs, G, U, route_w, token_indices, a_begin, a_end, T, I, tb, nt,
                           rank_out, rank_accum, z, z_stride, zsum, rows, assigns, tid, lane);
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
    return n_tiles <= ZSUM_STRIDE && gate->role == ROLE_GATE_UP && up->role == ROLE_GATE_UP && down->role == ROLE_DOWN && z_bytes <= 65536 &&
           I % N_TILE == 0;
}

int launch_forward_decode(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                          const void* h_gate, const void* h_up, int act_dtype, int64_t T, int Rg, int Ru, int64_t ldg,
                          int64_t ldu, const int32_t* tok, const int32_t* off, const float* rw, int64_t A, int rank_out,
                          int I, float* rank_accum, float* G, float* U, int64_t inter_floats, bitsmoe_profile* prof,
                          hipStream_t st) {
    const int E = gate->n_experts;
    const int n_tiles = gate->n_tiles;
    record(prof, 0, st);
    // What the expert coordinate of the grids counts.  Few assignments: the experts that can be
    // active at most, not all of them.  Sixteen or more assignments per expert on average: most
    // experts have several 16-assignment chunks, one workgroup per chunk.  Below that the search
    // of the chunk (one more dependent round trip per workgroup, +10 %) costs more than walking
    // an expert's few chunks in a loop, unless routing is skewed: with at most 64 experts (one
    // search step) the chunk grid is already used from three assignments per expert on average.
    // At most min(E, A) experts can be active.
    const int64_t active_max = std::min<int64_t>(E, A);
    const int mode = (A >= (int64_t)16 * E || (E <= 64 && A >= (int64_t)3 * E)) ? GRID_CHUNKS : active_max * 2 <= E ? GRID_ACTIVE : GRID_EXPERTS;
    const int e_dim = mode == GRID_CHUNKS ? (int)(active_max + A / MAX_A) : mode == GRID_ACTIVE ? (int)active_max : E;
    // (expert, chunk) pairs expected to have work (e_dim is their upper bound in chunk mode)
    const int64_t units = mode == GRID_CHUNKS ? A / MAX_A + active_max / 2 : active_max;
    // Sets of affine single-width experts, enough (expert, tile) pairs to fill the chip: the
    // walking gate/up kernel, which also clears rank_accum and needs no cleared G / U.
    // (its 16-byte activation loads also need rank_idx in runs of eight and aligned rows)
    auto rows16 = [](const void* p, int64_t ld) { return ((uintptr_t)p & 15) == 0 && ld % 8 == 0; };
    const bool walk = gate->all_affine && up->all_affine && gate->rank_chunked8 && up->rank_chunked8 &&
                   rows16(h_gate, ldg) && rows16(h_up, ldu);
    if (!walk) {
        // G and U are adjacent in the workspace: one range; rank_accum is the second
        const int64_t n1 = inter_floats + A * (int64_t)I;
        const int64_t n2 = T * (int64_t)rank_out;
        const int64_t blocks = std::min<int64_t>((std::max(n1, n2) + 255) / 256, 2048);
        hipLaunchKernelGGL(k_fill_zero2, dim3((unsigned)blocks), dim3(256), 0, st, G, n1, rank_accum, n2);
        BITSMOE_HIP_TRY(hipGetLastError());
    }
    record(prof, 1, st);
    const int max_slabs = std::max(gate->max_slabs, up->max_slabs);
    const int gu_groups = (max_slabs + GU_SLABS - 1) / GU_SLABS;
    // Tiles per workgroup: long runs amortise the start-up round trips, but the grid must
    // still hold a few workgroups per CU (two rounds of three per CU measured best).
    int tiles_per_wg = n_tiles;
    while (tiles_per_wg > 1 && units * 2 * gu_groups * ((n_tiles + tiles_per_wg - 1) / tiles_per_wg) < 1536)
        tiles_per_wg = (tiles_per_wg + 1) / 2;
    const int n_tchunks = (n_tiles + tiles_per_wg - 1) / tiles_per_wg;
    dim3 grid((unsigned)(e_dim * gu_groups * n_tchunks), 2);
    // the expert a grid coordinate stands for: by decreasing payload size, or the identity
    auto order_of = [&](const bitsmoe_matset* set) {
        ExpertOrder o;
        for (int i = 0; i < EXPERT_ORDER_MAX; ++i) o.e[i] = set->has_cost_order && i < E ? set->cost_order[i] : (uint16_t)i;
        return o;
    };
    const ExpertOrder gate_order = order_of(gate), up_order = order_of(up);
    auto launch_gateup = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, st, gate->d_fast_experts, gate->d_fast_slabs, gate->max_slabs,
                           up->d_fast_experts, up->d_fast_slabs, up->max_slabs, (const uint16_t*)h_gate,
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
    auto launch_walk_mode = [&](auto bf16_c, auto mode_c) {
        auto kern = k_gateup_walk<decltype(bf16_c)::value, decltype(mode_c)::value, false>;
        if (gate->rank_identity && up->rank_identity) kern = k_gateup_walk<decltype(bf16_c)::value, decltype(mode_c)::value, true>;
        hipLaunchKernelGGL(kern, dim3((unsigned)(e_dim * n_tiles), 2),
                           dim3(256), 0, st, gate->d_fast_experts, gate->d_fast_slabs, gate->max_slabs, up->d_fast_experts,
                           up->d_fast_slabs, up->max_slabs, (const uint16_t*)h_gate, (const uint16_t*)h_up, ldg, ldu,
                           tok, off, (int)T, (int)A, I, E, n_tiles, G, U, rank_accum, T * (int64_t)rank_out, gate_order,
                           up_order);
    };
    if (walk) {
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
    record(prof, 2, st);
    record(prof, 3, st);      // (SiLU happens inside the down kernel)
    const int dn_groups = (down->max_slabs + DN_SLABS_PER_WG - 1) / DN_SLABS_PER_WG;
    const size_t z_bytes = (size_t)MAX_A * (n_tiles * N_TILE + 8) * 2 + MAX_A * ZSUM_STRIDE * 4 + DN_SLABS_PER_WG * SLAB_ROWS * 8 + MAX_A * 8;
    int dn_tiles_per_wg = n_tiles;
    while (dn_tiles_per_wg > 1 && units * dn_groups * ((n_tiles + dn_tiles_per_wg - 1) / dn_tiles_per_wg) < 600)
        dn_tiles_per_wg = (dn_tiles_per_wg + 1) / 2;
    const int dn_tchunks = (n_tiles + dn_tiles_per_wg - 1) / dn_tiles_per_wg;
    auto launch_down = [&](auto kernel) {
        const int n_work = e_dim * dn_groups * dn_tchunks;
        hipLaunchKernelGGL(kernel, dim3((unsigned)((n_work + 7) / 8 * 8)), dim3(256), z_bytes, st, down->d_fast_experts,
                           down->d_fast_slabs, down->max_slabs, G, U, rw, tok, off, (int)T, (int)A, I, E, n_tiles,
                           dn_groups, dn_tchunks, dn_tiles_per_wg, n_work, rank_out, rank_accum);
    };
    auto launch_down_mode = [&](auto, auto mode_c) { launch_down(k_down_decode<decltype(mode_c)::value>); };
    // (G and U are fp32 and the operands f16 whatever the activation type was)
    with_mode(launch_down_mode, std::false_type{});
    BITSMOE_HIP_TRY(hipGetLastError());
    record(prof, 4, st);
    record(prof, 5, st);      // (the combine too)
    if (prof) prof->recorded = true;
    return BITSMOE_OK;
}

}  // namespace bitsmoe
