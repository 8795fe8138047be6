// The small-batch ("decode") forward as ONE kernel: a workgroup takes one expert (or one 16-assignment chunk of
// it) and ONE 128-column tile of the intermediate dimension and runs the whole chain for it,
//
//     G[:, tile] = hs_gate x gate[:, tile]        (walk over all slab groups, sums stay in registers)
//     U[:, tile] = hs_up   x up[:, tile]          (the same walk; the payload stream runs on)
//     z          = f16(silu(G) * U)               (16 x 128 operand in LDS, never in memory)
//     rank_accum[tok, rank_idx[r]] += route_w * s[r] * scale[tile, r] * sum_{c in tile} level[r, c] * z[:, c]
//                                                 (every slab of the down matrix, this tile's block of it)
//
// The down projection is linear in z, so the partial products of an expert's tiles meet in the fp32 atomics of
// the combine -- n_tiles atomics per (assignment, output rank) instead of one, in exchange for: no fp32 G / U
// round trip through memory, no second kernel (its launch gap, its start-up chain, its own scan of the routed
// ids), no SiLU pass repeated by every slab group of an expert, and one resident batch of workgroups that each
// stream gate, up and down payload back to back.  rank_accum is cleared by a small launch in front (a store
// that clears and an atomic that adds must not race through different L2s inside one kernel).
//
// Reference: bitsmoe/algorithms/cpp/mlp_forward.cu:1043-1206, 1337-1382 (gate/up, small path), 2145-2404 (down,
// small path), 2036-2066 (atomic combine).
#include "decode_launch.h"

namespace bitsmoe {

// ---- optional in-kernel time stamps (builds with -DBITSMOE_TIMELINE only: `python -m bitsmoe_amd.build --timeline`)
// Thread 0 of every workgroup writes the 100 MHz wall clock at the phase boundaries of its FIRST chunk into a
// device array that bitsmoe_timeline_read copies out; stamp 7 holds the XCD and the hardware id of the wavefront.
#ifdef BITSMOE_TIMELINE
constexpr int TIMELINE_STAMPS = 64;      // 0..6 phases, 7 hardware id, 8 + 4 * group + {start, staged, barrier passed, multiplied}
constexpr int TIMELINE_MAX_WG = 4096;
__device__ unsigned long long g_timeline[TIMELINE_MAX_WG * TIMELINE_STAMPS];
#define BITSMOE_STAMP(i)                                                                          \
    do {                                                                                          \
        if (threadIdx.x == 0 && blockIdx.x < TIMELINE_MAX_WG)                                     \
            g_timeline[blockIdx.x * TIMELINE_STAMPS + (i)] = wall_clock64();                      \
    } while (0)
#define BITSMOE_STAMP_HW()                                                                                       \
    do {                                                                                                         \
        if (threadIdx.x == 0 && blockIdx.x < TIMELINE_MAX_WG)                                                    \
            g_timeline[blockIdx.x * TIMELINE_STAMPS + 7] =                                                       \
                ((unsigned long long)__builtin_amdgcn_s_getreg(((4 - 1) << 11) | 20) << 32) |                    \
                (unsigned long long)__builtin_amdgcn_s_getreg(((32 - 1) << 11) | 4);                             \
    } while (0)
#else
#define BITSMOE_STAMP(i) do {} while (0)
#define BITSMOE_STAMP_HW() do {} while (0)
#endif

// A pointer that came out of a table by a vector load is the same in every lane: say so (scalar registers instead of
// a vector register pair per pointer; three matrices' worth of them would not fit beside the payload in flight).
template <class T>
__device__ __forceinline__ gptr<T> uniform_ptr(const T* p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (gptr<T>)(((uint64_t)hi << 32) | lo);
}

constexpr int FZ_STRIDE = N_TILE + 8;          // 16-bit elements per assignment row of z in LDS (+8 staggers banks)
constexpr int FT_STRIDE = SLAB_ROWS + 4;       // floats per assignment row of a wavefront's transposition buffer
constexpr int FUSED_MAX_DOWN_SLABS = 64;       // per expert: 16 per wavefront

// ---- the down phase's payload ring -----------------------------------------------------------------------------
// Wavefront `wave` takes the slabs wave, wave + 4, ... of the expert's down matrix, one (slab, tile) block each;
// NB blocks are in flight at a time (all of a 2-bit matrix of 32 slabs).  The first blocks are requested while the
// up walk's last slab groups are still being multiplied (its payload registers drain as these fill).
template <int WD>
struct DownRing {
    static constexpr int NB = WD == 2 ? 8 : WD == 3 ? 5 : 4;
    static constexpr int BW = WD == 3 ? R1W3_BLOCK_WORDS : 256 * WD;
    // Which ring slot the walk's tail call k = 0 .. 15 fills (-1: none): call k comes when the k-th of the sixteen
    // slab buffers of the walk's last two groups has been multiplied, so the ring fills as those drain -- spread so
    // that the registers of both together stay inside the budget (2-bit: half of the ring per group; wider blocks:
    // during the last group only).
    static constexpr int tail_slot(int k) {
        if (WD == 2) return (k >= 4 && k < 8) ? k - 4 : k >= 12 ? k - 8 : -1;
        if (WD == 3) return k == 15 ? 4 : (k >= 8 && (k & 1) == 0) ? (k - 8) / 2 : -1;
        return (k >= 8 && (k & 1) == 0) ? (k - 8) / 2 : -1;
    }
    Block16 buf[NB];
    uint32_t sc[NB];   // scale[tile, row] of the slab's row `lane`: f16 bits as loaded (converted where they are used:
    uint32_t sv[NB];   // s[row]              a conversion at the request would wait for the request, and for all before it)
    int rk[NB];        // logical rank of the row
};
struct DownSource {      // one expert's down matrix (wave-uniform) and this workgroup's tile
    gptr<uint32_t> payload;
    gptr<__half> scale;
    gptr<__half> svec;
    gptr<int32_t> rank_idx;
    int num_slabs, n_tiles, t;
};
// (unsigned 32-bit lane offsets from wave-uniform bases: the loads take a scalar base and a vector offset, no
// 64-bit address per lane and slot has to be kept)
template <int WD, int B>
__device__ __forceinline__ void down_issue(DownRing<WD>& ring, const DownSource& src, int wave, uint32_t lane, int i) {
    const uint32_t si = (uint32_t)(wave + 4 * i);
    const uint32_t st = si * (uint32_t)src.n_tiles + (uint32_t)src.t;      // (slab, tile) index, wave-uniform
    gptr<uint32_t> blk = src.payload + st * (uint32_t)DownRing<WD>::BW;
    gptr_u32x4 p = reinterpret_cast<gptr_u32x4>(blk + (WD == 4 ? lane * 16u : WD == 3 ? lane * 4u : lane * 8u));
    u32x4 v0 = p[0], v1, v2 = {0, 0, 0, 0}, v3 = {0, 0, 0, 0};
    if constexpr (WD == 3) {
        v1 = p[64];       // (+256 words)
        v2 = p[128];
        v3[0] = blk[768u + lane];
    } else {
        v1 = p[1];
    }
    if constexpr (WD == 4) {
        v2 = p[2];
        v3 = p[3];
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        ring.buf[B].w[x] = v0[x];
        ring.buf[B].w[4 + x] = v1[x];
        ring.buf[B].w[8 + x] = v2[x];
        ring.buf[B].w[12 + x] = v3[x];
    }
    ring.sc[B] = (reinterpret_cast<gptr<uint16_t>>(src.scale) + st * (uint32_t)SLAB_ROWS)[lane];
    ring.sv[B] = (reinterpret_cast<gptr<uint16_t>>(src.svec) + si * (uint32_t)SLAB_ROWS)[lane];
    ring.rk[B] = (src.rank_idx + si * (uint32_t)SLAB_ROWS)[lane];
}

// One (slab, tile) block of a down matrix without its scale: 4 row blocks x 4 k-steps; acc[nb][j] = sum over the
// tile's columns of level[16 nb + n, c] * z[4 kg + j, c] (the constant term of the 2^W + code operands removed).
template <int W>
__device__ __forceinline__ void down_block_raw(const Block16& b, const u32x4 (&az)[4], f32x4 corr, f32x4 (&acc)[4]) {
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
        acc[nb] = t - corr;
    }
}

// z of the workgroup's tile from the gate and up sums in registers, then the down projection of that tile.
//   g, u       the lane's sums: rows a = 4*kg + j of columns 32*wave + 16*nbl + n
//   n_pre      blocks of the ring that have been requested already (by the walk's tail)
//   z_lds      16 x FZ_STRIDE 16-bit; zs_lds 4 x 16 floats; assigns 16 x (token or -1, routing weight)
//   tbuf_all   LDS the gate / up walks are done with: 4 x 16 x FT_STRIDE floats, one buffer per wavefront
// The combine goes through a transposition in LDS: the MFMA leaves a lane with four assignments of four rows; the
// wavefront writes its 16 x 64 block and reads it back with lane = row, so that one atomic instruction per REAL
// assignment adds 64 neighbouring ranks (and rank, s and scale of a row are per-lane values, loaded with the block).
template <int WD, class AS>
__device__ __forceinline__ void fused_z_down(DownRing<WD>& ring, int n_pre, const f32x4 (&g)[2], const f32x4 (&u)[2],
                                             const DownSource& src, const AS& as, int a0, int n_a, int T, int rank_out,
                                             float* __restrict__ rank_accum, uint16_t* __restrict__ z_lds,
                                             float* __restrict__ zs_lds, int2* __restrict__ assigns,
                                             float* __restrict__ tbuf_all, int tid, bool stamp) {
    constexpr int NB = DownRing<WD>::NB;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int lane = tid & 63;
    asm volatile("" : "+v"(lane));      // (what is derived from it is computed here, not in front of the caller's loop)
    const int n = lane & 15, kg = lane >> 4, g4 = 4 * kg;
    const int n_i = (src.num_slabs - wave + 3) >> 2;      // slabs of this wavefront
    float* __restrict__ tbuf = tbuf_all + wave * (MAX_A * FT_STRIDE);

    static_for([&](auto bc) {
        constexpr int B = decltype(bc)::value;
        if (B >= n_pre && B < n_i) down_issue<WD, B>(ring, src, wave, (uint32_t)lane, B);
    }, std::make_integer_sequence<int, NB>{});
    const int tok_lane = as.token_if(a0 + lane, lane < n_a);
    const float rw_lane = as.weight_if(a0 + lane, lane < n_a);

    // z = silu(G) * U as 16-bit operands, and the sums of the rounded operands per assignment row
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int a = g4 + j;
        float v = 0.0f;
#pragma unroll
        for (int nbl = 0; nbl < 2; ++nbl) {
            uint16_t zb = z_operand(g[nbl][j], u[nbl][j]);
            if (a >= n_a) zb = 0;      // (rows without an assignment hold whatever LDS held)
            z_lds[a * FZ_STRIDE + 32 * wave + 16 * nbl + n] = zb;
            v += __half2float(__ushort_as_half(zb));
        }
        v = dpp_add_f32<0x111>(v);
        v = dpp_add_f32<0x112>(v);
        v = dpp_add_f32<0x114>(v);
        v = dpp_add_f32<0x118>(v);
        if (n == 15) zs_lds[wave * MAX_A + a] = v;
    }
    if (tid < MAX_A) assigns[tid] = int2{(tok_lane >= 0 && tok_lane < T) ? tok_lane : -1, __float_as_int(rw_lane)};
    __syncthreads();      // z, its sums and the assignment records are complete
    if (stamp) BITSMOE_STAMP(4);

    // the operand and the constant term are the same for every slab
    u32x4 az[4];
    {
        const uint16_t* zp = z_lds + n * FZ_STRIDE + 8 * kg;
#pragma unroll
        for (int m = 0; m < 4; ++m) az[m] = *reinterpret_cast<const u32x4*>(zp + 32 * m);
    }
    f32x4 corr;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int a = g4 + j;
        corr[j] = (zs_lds[a] + zs_lds[MAX_A + a] + zs_lds[2 * MAX_A + a] + zs_lds[3 * MAX_A + a]) * (1.5f * (float)(1 << WD));
    }
    auto compute = [&](auto b_c) {
        constexpr int B = decltype(b_c)::value;
        f32x4 acc[4];
        down_block_raw<WD>(ring.buf[B], az, corr, acc);
#pragma unroll
        for (int nb = 0; nb < 4; ++nb)
#pragma unroll
            for (int j = 0; j < 4; ++j) tbuf[(g4 + j) * FT_STRIDE + 16 * nb + n] = acc[nb][j];
        const int lr = ring.rk[B];
        const float rs = __half2float(__ushort_as_half((uint16_t)ring.sc[B])) * __half2float(__ushort_as_half((uint16_t)ring.sv[B]));
        const bool row_ok = lr >= 0 && lr < rank_out;
        for (int a = 0; a < n_a; ++a) {
            const int2 tr = assigns[a];        // (one address for the whole wavefront: a broadcast read)
            const float v = tbuf[a * FT_STRIDE + lane];
            if (row_ok && tr.x >= 0) atomicAdd(&rank_accum[(int64_t)tr.x * rank_out + lr], v * rs * __int_as_float(tr.y));
        }
    };
    for (int i0 = 0; i0 < n_i; i0 += NB) {
        static_for([&](auto bc) {
            constexpr int B = decltype(bc)::value;
            if (i0 + B < n_i) {
                compute(bc);
                if (i0 + B + NB < n_i) down_issue<WD, B>(ring, src, wave, (uint32_t)lane, i0 + B + NB);
            }
        }, std::make_integer_sequence<int, NB>{});
    }
}

// ---- gate and up of one tile as ONE walk --------------------------------------------------------------------------
// The slab groups of the gate matrix, then those of the up matrix, as one sequence of "virtual" groups (both matrices
// of the expert have n_groups groups of ONE width W): the payload stream of a wavefront runs on from the one into
// the other, AHEAD groups ahead of the one being multiplied (two: two register buffers used in turn -- what the
// narrow 2-bit blocks leave room for), and while the last AHEAD groups are multiplied the registers they free are
// handed to `tail(index)`, index = 16 - 8 * AHEAD .. 15 -- the caller requests the first blocks of the down matrix there.  Everything else as in gateup_walk_item: operand staged
// by 16-byte accesses into two LDS copies used in turn (one barrier per group), scales one group ahead, ranks two,
// the constant term summed by the staging wavefronts.  g / u receive the tile's sums (the lane's rows
// a = 4*kg + j of column 32*pair + 16*nbl + n).
template <bool BF16, bool IDENT, int W, int AHEAD, class AS, class TAIL>
__device__ __forceinline__ void fused_walk(const WalkMatrix& mg, const WalkMatrix& mu, const AS& as, int a0, int n_a, int T,
                                           int n_tiles, int t, int n_groups, uint16_t* __restrict__ hs_all,
                                           float* __restrict__ cterm_lds, int tid, f32x4 (&g)[2], f32x4 (&u)[2],
                                           TAIL&& tail) {
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
    const int n_vg = 2 * n_groups;       // the gate matrix's groups, then the up matrix's

    static_assert(AHEAD == 1 || AHEAD == 2, "one or two groups ahead");
    uint32_t pw[AHEAD][GU_SLABS][4];   // AHEAD groups in flight; a slab's registers are refilled right after their use
    auto issue = [&](auto b_c, auto q_c, int vg) {
        constexpr int B = decltype(b_c)::value, q = decltype(q_c)::value;
        const bool up = vg >= n_groups;
        const int gg = up ? vg - n_groups : vg;
        gptr<uint32_t> base = up ? mu.payload : mg.payload;
        load_pair_role0(base + (uint32_t)((up ? pack0_u : pack0_g) + (gg * GU_SLABS + q) * slab_words), W, unit, hi_unit, pw[B][q]);
    };
    int tki[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) tki[i] = as.token(a0 + pair + 4 * i);
    auto rank_at = [&](int vg) {
        const bool up = vg >= n_groups;
        const int gg = up ? vg - n_groups : vg;
        const int k = (up ? mu.first.rank_off : mg.first.rank_off) + gg * (GU_SLABS * SLAB_ROWS) + 8 * lane;
        if constexpr (IDENT) return k;      // rank_idx[k] == k in every expert of both sets
        else return (int)(up ? mu.rank_idx : mg.rank_idx)[k];
    };
    auto scale_at = [&](int vg) {
        const bool up = vg >= n_groups;
        const int gg = up ? vg - n_groups : vg;
        gptr<__half> base = up ? mu.scale_s : mg.scale_s;
        return *reinterpret_cast<gptr_u32x4>(
            base + (uint32_t)((up ? mu.first.scale_off : mg.first.scale_off) +
                              ((gg * GU_SLABS + (lane >> 3)) * n_tiles + t) * SLAB_ROWS + 8 * (lane & 7)));
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
    u32x4 raw0 = act_at(0, rank_cur, n_groups == 0);
    u32x4 raw1 = act_at(1, rank_cur, n_groups == 0);
    // (payload behind what the first operand needs: loads return in order)
    static_for([&](auto qc) { issue(I0{}, qc, 0); }, std::make_integer_sequence<int, GU_SLABS>{});
    if constexpr (AHEAD == 2) static_for([&](auto qc) { issue(I1{}, qc, 1); }, std::make_integer_sequence<int, GU_SLABS>{});
    f32x4 acc[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
    f32x4 acc_g[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
    f32x4 corr = {0, 0, 0, 0};
    // B: the register buffer of group vg (= vg mod 2).  MORE: another group follows.  TAILK: 0 = the buffer is
    // refilled with group vg + 2; 1 / 2 = second to last / last group: the freed registers go to tail(0..7) / (8..15).
    auto group_step = [&](auto b_c, auto more_c, auto tail_c, int vg) {
        constexpr bool more = decltype(more_c)::value;
        constexpr int TAILK = decltype(tail_c)::value;
        const bool up = vg >= n_groups;
        if (vg < 12) BITSMOE_STAMP(8 + 4 * vg);
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
        if (vg < 12) BITSMOE_STAMP(8 + 4 * vg + 1);
        __syncthreads();   // the operand is complete
        if (vg < 12) BITSMOE_STAMP(8 + 4 * vg + 2);
        if constexpr (more) {
            const bool up_nxt = vg + 1 >= n_groups;
            raw0 = act_at(0, rank_nxt, up_nxt);
            raw1 = act_at(1, rank_nxt, up_nxt);
        }
        // (these two requests stay HERE, in front of the payload requests below: loads return in order, and the
        // next group's operand must not wait for payload that is two groups away)
        __builtin_amdgcn_sched_barrier(0);
        const uint16_t* ap16 = &hs[n * GU_STRIDE + 16 * kg];
        static_for([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            constexpr int B = decltype(b_c)::value;
            const u32x4 a_lo = *reinterpret_cast<const u32x4*>(ap16 + q * SLAB_ROWS);
            const u32x4 a_hi = *reinterpret_cast<const u32x4*>(ap16 + q * SLAB_ROWS + 8);
            gateup_pair<W, false>(pw[B][q], a_lo, a_hi, n >> 3, acc, corr, W == 3 ? &m3 : nullptr);
            if constexpr (TAILK == 0)
                issue(b_c, qc, vg + AHEAD);
            else
                tail(std::integral_constant<int, (TAILK - 1) * GU_SLABS + q>{});
        }, std::make_integer_sequence<int, GU_SLABS>{});
        if (vg < 12) BITSMOE_STAMP(8 + 4 * vg + 3);
        sc_cur = sc_nxt;
        rank_cur = rank_nxt;
        rank_nxt = rank_nxt2;
    };
    if constexpr (AHEAD == 2) {
        for (int vg = 0; vg + 2 < n_vg; vg += 2) {
            group_step(I0{}, std::true_type{}, I0{}, vg);
            group_step(I1{}, std::true_type{}, I0{}, vg + 1);
        }
        group_step(I0{}, std::true_type{}, I1{}, n_vg - 2);
        group_step(I1{}, std::false_type{}, I2{}, n_vg - 1);
    } else {
        for (int vg = 0; vg + 1 < n_vg; ++vg) group_step(I0{}, std::true_type{}, I0{}, vg);
        group_step(I0{}, std::false_type{}, I2{}, n_vg - 1);
    }
    // the constant terms of the chunk's assignments, from the wavefronts that staged them
    if (lane == 63) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            cterm_lds[pair + 4 * i] = cterm_g[i];
            cterm_lds[MAX_A + pair + 4 * i] = cterm_u[i];
        }
    }
    __syncthreads();
    f32x4 cg, cu;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        cg[j] = cterm_lds[4 * kg + j];
        cu[j] = cterm_lds[MAX_A + 4 * kg + j];
    }
    g[0] = acc_g[0] - cg;
    g[1] = acc_g[1] - cg;
    u[0] = acc[0] - cu;
    u[1] = acc[1] - cu;
}

// grid.x = (expert coordinate) * n_tiles; 256 threads = 4 wavefronts.  MODE: what the expert coordinate counts
// (GRID_*).  ROUTED (GRID_EXPERTS or GRID_ACTIVE): no routing tables; the workgroup finds its expert's entries among
// the n_flat = T * top_k routed ids itself (inline_route) and takes the routing weights in entry order.  Every
// expert of the three sets has ONE bit-width per matrix; where gate, up and down of an expert share it (and gate
// and up their slab count) the single walk runs, otherwise the two projections are walked one after the other and
// the down blocks are requested when z is formed.  The down matrices have at most FUSED_MAX_DOWN_SLABS slabs.
// rank_accum must have been cleared by an earlier launch.
// (The three widths share the kernel's register allocation: what the widest body spills is reloaded in front of
// every body's groups, and every such reload waits for the payload in flight -- loads return in order -- so the wide
// bodies keep one group in flight where the 2-bit body keeps two.)
template <bool BF16, int MODE, bool IDENT, bool ROUTED>
__global__ __launch_bounds__(256, 3) void k_decode_fused(
    const FastExpert* __restrict__ gate_fe, const FastSlab* __restrict__ gate_fs, int gate_max_slabs,
    const FastExpert* __restrict__ up_fe, const FastSlab* __restrict__ up_fs, int up_max_slabs,
    const FastExpert* __restrict__ down_fe, const uint16_t* __restrict__ h_gate, const uint16_t* __restrict__ h_up,
    int64_t ldg, int64_t ldu, const int32_t* __restrict__ token_indices, const int32_t* __restrict__ expert_offsets,
    const float* __restrict__ route_w, int T, int A, int I, int E, int n_tiles, int rank_out,
    float* __restrict__ rank_accum, const ExpertOrder order, const void* __restrict__ selected, int ids_are_i64,
    int n_flat, int top_k, const int32_t* __restrict__ local_to_global, const float* __restrict__ sel_weights,
    const int32_t* __restrict__ global_to_local, int n_global) {
    static_assert(!ROUTED || MODE != GRID_CHUNKS, "inline routing serves whole experts");
    BITSMOE_STAMP(0);
    BITSMOE_STAMP_HW();
    const int tid = threadIdx.x;
    const int bid = blockIdx.x;
    const int t = bid % n_tiles;
    int e = bid / n_tiles;
    int chunk = -1;
    if constexpr (MODE == GRID_EXPERTS) {      // expensive experts first (the identity when there is no order)
        if (E <= EXPERT_ORDER_MAX) e = order.at(e);
    } else if constexpr (MODE == GRID_ACTIVE && !ROUTED) {
        e = nth_active_expert(expert_offsets, E, A, e, tid & 63);
        if (e < 0) return;
    } else if constexpr (MODE == GRID_CHUNKS) {
        const ChunkRef ref = nth_chunk(expert_offsets, E, A, e, tid & 63);
        e = ref.expert;
        chunk = ref.chunk;
        if (e < 0) return;
    }
    int a_begin = 0, a_end = 0;
    int gid = -1;
    __shared__ std::conditional_t<ROUTED, InlineRouteLds, int> route_lds;
    if constexpr (ROUTED && MODE == GRID_ACTIVE) {
        // `e` is an entry index: serve the expert it names if this is the expert's first entry
        const int slot = e;
        if (slot >= n_flat) return;
        gid = routed_id(selected, ids_are_i64, slot);
        a_end = inline_route(selected, ids_are_i64, n_flat, top_k, gid, route_lds, tid);
        if (a_end == 0 || route_lds.ent[0] != slot || gid < 0 || gid >= n_global) return;
        e = global_to_local[gid];
        if (e < 0 || e >= E) return;
    } else if constexpr (ROUTED) {
        gid = local_to_global[e];
    } else {
        a_begin = max(expert_offsets[e], 0);
        a_end = min(expert_offsets[e + 1], A);
        if (chunk >= 0) {
            a_begin += MAX_A * chunk;
            a_end = min(a_end, a_begin + MAX_A);
        }
    }
    const FastExpert feg = gate_fe[e];
    const FastExpert feu = up_fe[e];
    const FastExpert fed = down_fe[e];
    const FastSlab first_g = load_fast_slab(gate_fs, e * gate_max_slabs);
    const FastSlab first_u = load_fast_slab(up_fs, e * up_max_slabs);
    if constexpr (ROUTED && MODE == GRID_EXPERTS) a_end = inline_route(selected, ids_are_i64, n_flat, top_k, gid, route_lds, tid);
    if (a_end <= a_begin || first_g.bits == 0 || first_u.bits == 0) return;
    const int wd = __builtin_amdgcn_readfirstlane(fed.uniform_bits);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lane = (uint32_t)(tid & 63);
    const DownSource dsrc0{uniform_ptr(fed.payload), uniform_ptr(fed.scale), uniform_ptr(fed.s), uniform_ptr(fed.rank_idx),
                           __builtin_amdgcn_readfirstlane(fed.num_slabs), n_tiles, t};
    const int n_i = (dsrc0.num_slabs - wave + 3) >> 2;
    const int gu_groups = __builtin_amdgcn_readfirstlane(feg.num_slabs) / GU_SLABS;
    const int up_groups = __builtin_amdgcn_readfirstlane(feu.num_slabs) / GU_SLABS;
    // gate, up and down of this expert at ONE width, gate and up of one length: the single walk with the down
    // matrix's first blocks requested from its tail
    const bool one_walk = first_g.bits == first_u.bits && first_g.bits == wd && gu_groups == up_groups;

    auto assignments = [&]() {
        if constexpr (ROUTED)
            return AssignInline{route_lds.tok, route_lds.ent, sel_weights, a_end};
        else
            return AssignTables{token_indices, route_w, A};
    };
    const auto as = assignments();

    // (the operand buffers of the gate / up walks; the down phase transposes its results there)
    __shared__ __attribute__((aligned(16))) uint16_t hs_all[2 * MAX_A * GU_STRIDE];
    __shared__ float cterm_lds[2 * MAX_A];
    __shared__ __attribute__((aligned(16))) uint16_t z_lds[MAX_A * FZ_STRIDE];
    __shared__ float zs_lds[4 * MAX_A];
    __shared__ int2 assigns[MAX_A];
    static_assert(sizeof(uint16_t) * 2 * MAX_A * GU_STRIDE >= sizeof(float) * 4 * MAX_A * FT_STRIDE,
                  "the down phase's transposition buffers must fit the operand buffers");
    float* tbuf_all = reinterpret_cast<float*>(hs_all);
    const WalkMatrix mg{uniform_ptr(feg.payload), uniform_ptr(feg.scale_s), uniform_ptr(feg.rank_idx), first_g, h_gate, ldg};
    const WalkMatrix mu{uniform_ptr(feu.payload), uniform_ptr(feu.scale_s), uniform_ptr(feu.rank_idx), first_u, h_up, ldu};

    BITSMOE_STAMP(1);
    for (int a0 = a_begin; a0 < a_end; a0 += MAX_A) {
        const int n_a = min(MAX_A, a_end - a0);
        const bool first_chunk = a0 == a_begin;
        if (!first_chunk) __syncthreads();      // the previous chunk's down phase is done with the LDS buffers
        // (an opaque zero and an opaque lane keep the address arithmetic of the down blocks inside this loop body,
        // where it is cheap scalar work, instead of hoisted in front of the loop and held in registers for every
        // slot of every width)
        int chunk_zero = 0;
        asm volatile("" : "+s"(chunk_zero));
        const DownSource dsrc{dsrc0.payload, dsrc0.scale, dsrc0.svec, dsrc0.rank_idx, dsrc0.num_slabs, n_tiles, t + chunk_zero};
        uint32_t lane_c = lane;
        asm volatile("" : "+v"(lane_c));
        int tid_c = tid, tile_c = t + chunk_zero;
        asm volatile("" : "+v"(tid_c));
        f32x4 g[2], u[2];
        if (one_walk) {
            auto run = [&](auto w_c) {
                constexpr int W = decltype(w_c)::value;
                DownRing<W> ring;
                fused_walk<BF16, IDENT, W, (W == 2 ? 2 : 1)>(mg, mu, as, a0, n_a, T, n_tiles, tile_c, gu_groups, hs_all, cterm_lds, tid_c,
                                                             g, u, [&](auto kc) {
                                                                 constexpr int i = DownRing<W>::tail_slot(decltype(kc)::value);
                                                                 if constexpr (i >= 0) {
                                                                     if (i < n_i) down_issue<W, i>(ring, dsrc, wave, lane_c, i);
                                                                 }
                                                             });
                if (first_chunk) BITSMOE_STAMP(3);
                fused_z_down<W>(ring, DownRing<W>::NB, g, u, dsrc, as, a0, n_a, T, rank_out, rank_accum, z_lds, zs_lds,
                                assigns, tbuf_all, tid_c, first_chunk);
            };
            if (wd == 2)
                run(std::integral_constant<int, 2>{});
            else if (wd == 3)
                run(std::integral_constant<int, 3>{});
            else if (wd == 4)
                run(std::integral_constant<int, 4>{});
        } else {
            auto walk = [&](auto w_c, const WalkMatrix& m, int n_groups, f32x4* keep) {
                gateup_walk_item<BF16, IDENT, decltype(w_c)::value, false, decltype(as), true>(
                    m.payload, m.scale_s, m.rank_idx, m.first, m.h, m.ld, as, a0, n_a, T, I, n_tiles, tile_c, 0, n_groups, nullptr,
                    hs_all, cterm_lds, tid_c, keep);
            };
            auto walk_any = [&](const WalkMatrix& m, int n_groups, f32x4* keep) {
                if (m.first.bits == 2)
                    walk(std::integral_constant<int, 2>{}, m, n_groups, keep);
                else if (m.first.bits == 3)
                    walk(std::integral_constant<int, 3>{}, m, n_groups, keep);
                else
                    walk(std::integral_constant<int, 4>{}, m, n_groups, keep);
            };
            walk_any(mg, gu_groups, g);
            if (first_chunk) BITSMOE_STAMP(2);
            // (every wavefront has passed the walk's closing barrier behind its last operand reads: the buffers are free)
            walk_any(mu, up_groups, u);
            if (first_chunk) BITSMOE_STAMP(3);
            auto down = [&](auto w_c) {
                constexpr int WD = decltype(w_c)::value;
                DownRing<WD> ring;
                fused_z_down<WD>(ring, 0, g, u, dsrc, as, a0, n_a, T, rank_out, rank_accum, z_lds, zs_lds, assigns, tbuf_all, tid_c,
                                 first_chunk);
            };
            if (wd == 2)
                down(std::integral_constant<int, 2>{});
            else if (wd == 3)
                down(std::integral_constant<int, 3>{});
            else if (wd == 4)
                down(std::integral_constant<int, 4>{});
        }
        if (first_chunk) BITSMOE_STAMP(5);
    }
    BITSMOE_STAMP(6);
}

#ifdef BITSMOE_TIMELINE
}  // namespace bitsmoe
extern "C" int bitsmoe_timeline_read(unsigned long long* host, int n_workgroups) {
    using namespace bitsmoe;
    if (!host || n_workgroups <= 0 || n_workgroups > TIMELINE_MAX_WG) return BITSMOE_E_INVALID;
    BITSMOE_HIP_TRY(hipDeviceSynchronize());
    BITSMOE_HIP_TRY(hipMemcpyFromSymbol(host, HIP_SYMBOL(g_timeline), sizeof(unsigned long long) * TIMELINE_STAMPS * n_workgroups));
    return BITSMOE_OK;
}
extern "C" int bitsmoe_timeline_clear(void) {
    using namespace bitsmoe;
    void* p = nullptr;
    BITSMOE_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(g_timeline)));
    BITSMOE_HIP_TRY(hipMemset(p, 0, sizeof(unsigned long long) * TIMELINE_STAMPS * TIMELINE_MAX_WG));
    return BITSMOE_OK;
}
namespace bitsmoe {
#endif

__global__ void k_fused_clear(float* __restrict__ p, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = 0.0f;
}

bool decode_fused_possible(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                           const void* h_gate, const void* h_up, int Rg, int Ru, int64_t ldg, int64_t ldu, int I) {
    return decode_path_supported(gate, up, down, I) && walk_possible(gate, up, h_gate, h_up, Rg, Ru, ldg, ldu) &&
           gate->uniform_experts && up->uniform_experts && down->uniform_experts &&
           down->prep_max_slabs <= FUSED_MAX_DOWN_SLABS &&
           !has_wide_rows(gate) && !has_wide_rows(up) && !has_wide_rows(down);
}

// Measured on one MI355X under graph replay against the two-kernel form (cold weights): 64 tokens on the 128-expert
// layer 62.9 vs 60.0 us, 32 tokens 51.2 vs 54.2, 8 tokens 35.2 vs 30.4, 1 token 24.6 vs 15.7 (the two-kernel form
// splits the contraction of its few items over workgroups, this one cannot), 256 tokens on the 512-expert layer
// 151.5 vs 153.0, the 26-layer stack at 32 tokens 1.55 vs 1.15 ms.  One resident batch of long workgroups ends
// when its slowest member does (in-kernel time stamps: a workgroup lives 45 us on average, the last one 63), which
// eats what the missing intermediates and the second launch save; so it is not chosen by itself anywhere and runs
// where option decode_fused = 1 asks for it.
bool decode_fused_chosen(const bitsmoe_matset* gate, int64_t A, int I) {
    (void)gate;
    (void)A;
    (void)I;
    return false;
}

int launch_forward_decode_fused(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                                const void* h_gate, const void* h_up, int act_dtype, int64_t T, int Rg, int Ru, int64_t ldg,
                                int64_t ldu, const int32_t* tok, const int32_t* off, const float* rw, int64_t A, int rank_out,
                                int I, float* rank_accum, const DecodeRouted* routed, bitsmoe_profile* prof, hipStream_t st) {
    (void)Rg;
    (void)Ru;
    const int E = gate->n_experts;
    const int n_tiles = gate->n_tiles;
    record_phase(prof, 0, st);
    {
        const int64_t n = T * (int64_t)rank_out;
        const int64_t blocks = std::min<int64_t>((n + 1023) / 1024, 1024);
        hipLaunchKernelGGL(k_fused_clear, dim3((unsigned)std::max<int64_t>(blocks, 1)), dim3(256), 0, st, rank_accum, n);
        BITSMOE_HIP_TRY(hipGetLastError());
    }
    record_phase(prof, 1, st);
    const int64_t active_max = std::min<int64_t>(E, A);
    const int mode = decode_grid_mode(A, E);
    const int e_dim = mode == GRID_CHUNKS ? (int)(active_max + A / MAX_A) : mode == GRID_ACTIVE ? (int)active_max : E;
    const ExpertOrder order = expert_order_of(gate);
    const bool bf16 = act_dtype == BITSMOE_DT_BF16;
    const bool ident = gate->rank_identity && up->rank_identity;
    auto launch = [&](auto kern) {
        hipLaunchKernelGGL(kern, dim3((unsigned)(e_dim * n_tiles)), dim3(256), 0, st, gate->d_fast_experts, gate->d_fast_slabs,
                           gate->prep_max_slabs, up->d_fast_experts, up->d_fast_slabs, up->prep_max_slabs,
                           down->d_fast_experts, (const uint16_t*)h_gate, (const uint16_t*)h_up, ldg, ldu, tok, off, rw, (int)T,
                           (int)A, I, E, n_tiles, rank_out, rank_accum, order, routed ? routed->selected : nullptr,
                           routed ? routed->ids_are_i64 : 0, routed ? (int)A : 0, routed ? routed->top_k : 1,
                           routed ? routed->local_to_global : nullptr, routed ? routed->weights : nullptr,
                           routed ? routed->global_to_local : nullptr, routed ? routed->n_global : 0);
    };
    auto with_flags = [&](auto bf16_c, auto ident_c) {
        constexpr bool B = decltype(bf16_c)::value, ID = decltype(ident_c)::value;
        if (mode == GRID_CHUNKS) {
            launch(k_decode_fused<B, GRID_CHUNKS, ID, false>);
        } else if (mode == GRID_ACTIVE) {
            if (routed)
                launch(k_decode_fused<B, GRID_ACTIVE, ID, true>);
            else
                launch(k_decode_fused<B, GRID_ACTIVE, ID, false>);
        } else {
            if (routed)
                launch(k_decode_fused<B, GRID_EXPERTS, ID, true>);
            else
                launch(k_decode_fused<B, GRID_EXPERTS, ID, false>);
        }
    };
    if (bf16) {
        if (ident) with_flags(std::true_type{}, std::true_type{});
        else with_flags(std::true_type{}, std::false_type{});
    } else {
        if (ident) with_flags(std::false_type{}, std::true_type{});
        else with_flags(std::false_type{}, std::false_type{});
    }
    BITSMOE_HIP_TRY(hipGetLastError());
    for (int i = 2; i <= BITSMOE_PROFILE_PHASES; ++i) record_phase(prof, i, st);      // (one kernel: the other phases are empty)
    if (prof) prof->recorded = true;
    return BITSMOE_OK;
}

}  // namespace bitsmoe
