// Small-batch ("decode") kernels of the routed-expert forward: HBM-bound streaming of the
// prepared payload, field decode in registers, 16x16x32 MFMA against up to 16 assignments
// of one expert.  See wave_layout.h for the layout and the (2^w + code) operand trick.
//
//   k_gateup_decode   G[a,c] / U[a,c] += sum_k  hs'[a,k] * level[k,c]
//                     hs'[a,k] = h[tok_a, rank_idx[k]] * s[k] * scale[tile(c), k]  (16-bit operand)
//   k_down_decode     rank_accum[tok_a, rank_idx[r]] += route_w[a] * s[r] *
//                         sum_tiles scale[tile, r] * sum_{c in tile} level[r,c] * z[a,c]
//                     z = silu(G) * U  (16-bit operand)
//
// MFMA operands: A = activations (row index = assignment), B = weights (column index =
// output column / output rank row); D[4*(lane/16)+j][lane%16].
#include "wave_layout.h"

namespace bitsmoe {

constexpr int GU_SLABS_PER_WG = 8;                    // slabs (64 rows each) staged per workgroup
constexpr int GU_ROWS = GU_SLABS_PER_WG * SLAB_ROWS;  // contraction rows staged per workgroup
constexpr int GU_STRIDE = GU_ROWS + 8;                // 16-bit elements; +8 staggers LDS banks
constexpr int DN_SLABS_PER_WG = 4;                    // one slab per wavefront
constexpr int MAX_A = 16;                             // assignments per MFMA pass

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef const u32x2 __attribute__((address_space(1)))* gptr_u32x2;

// A packed matrix with every pointer in the global address space.
struct GView {
    gptr<uint32_t> payload;
    gptr<int32_t> rank_idx;
    gptr<int32_t> tile_meta;
    gptr<int32_t> slab_meta;
    gptr<__half> scale;
    gptr<__half> s;
    int num_slabs;
};

__device__ inline GView load_view(const MatView* __restrict__ views, int e) {
    const MatView mv = views[e];
    GView g;
    g.payload = as_global(mv.payload);
    g.rank_idx = as_global(mv.rank_idx);
    g.tile_meta = as_global(mv.tile_meta);
    g.slab_meta = as_global(mv.slab_meta);
    g.scale = as_global(mv.scale);
    g.s = as_global(mv.s);
    g.num_slabs = mv.num_slabs;
    return g;
}

__device__ inline float gload_half(gptr<__half> p) {
    const uint16_t bits = *reinterpret_cast<gptr<uint16_t>>(p);
    return __half2float(__ushort_as_half(bits));
}

template <int W, bool BF16>
__device__ inline u32x4 corr_operand() {
    const uint32_t c = Codec<W, BF16>::CORR;
    u32x4 r = {c, c, c, c};
    return r;
}

// Keeps a value's computation inside the loop iteration it is written in (the decode of
// the payload does not depend on the assignment chunk, and hoisting it out of the chunk
// loop would park every decoded operand in registers).
__device__ inline void pin(uint32_t& v) { asm volatile("" : "+v"(v)); }

// ------------------------------------------------------------------------------ gate / up
// The words of one wavefront's column-block pair for one (slab, tile) block: 2-bit {nb0, nb1};
// 4-bit {nb0 j0, nb0 j1, nb1 j0, nb1 j1}; 3-bit {low nb0, low nb1, high nb0, high nb1}.
__device__ inline void load_pair_role0(gptr<uint32_t> blk, int bits, int pair, int lane, uint32_t (&w)[4]) {
    if (bits == 4) {
        const u32x4 v = *reinterpret_cast<gptr_u32x4>(blk + (pair * 64 + lane) * 4);
        w[0] = v[0]; w[1] = v[1]; w[2] = v[2]; w[3] = v[3];
    } else {
        const u32x2 v = *reinterpret_cast<gptr_u32x2>(blk + (pair * 64 + lane) * 2);
        w[0] = v[0]; w[1] = v[1]; w[2] = 0; w[3] = 0;
        if (bits == 3) {
            const u32x2 h = *reinterpret_cast<gptr_u32x2>(blk + 512 + hi_index0(lane >> 4, lane & 15, 2 * pair));
            w[2] = h[0]; w[3] = h[1];
        }
    }
}

// One (slab, tile) block restricted to one column-block pair: 2 column blocks x 2 k-steps,
// plus the two MFMAs that accumulate the constant term.
template <int W, bool BF16>
__device__ inline void gateup_pair(const uint32_t (&w)[4], u32x4 a0, u32x4 a1, int upper, f32x4 (&acc)[2], f32x4& corr) {
    const u32x4 bc = corr_operand<W, BF16>();
    corr = mfma16<BF16>(a0, bc, corr);
    corr = mfma16<BF16>(a1, bc, corr);
#pragma unroll
    for (int nbl = 0; nbl < 2; ++nbl) {
        u32x4 b0, b1;
        if constexpr (W == 2) {
            b0 = decode_fields2<2, BF16>(w[nbl], 0);
            b1 = decode_fields2<2, BF16>(w[nbl], 8);
        } else if constexpr (W == 4) {
            b0 = decode_fields4<BF16>(w[2 * nbl]);
            b1 = decode_fields4<BF16>(w[2 * nbl + 1]);
        } else {
            b0 = decode_fields3<BF16>(w[nbl], 0, w[2 + nbl], 8 * upper);
            b1 = decode_fields3<BF16>(w[nbl], 8, w[2 + nbl], 8 * upper + 4);
        }
        acc[nbl] = mfma16<BF16>(a0, b0, acc[nbl]);
        acc[nbl] = mfma16<BF16>(a1, b1, acc[nbl]);
    }
}

// grid.x = E * n_tiles * n_groups, grid.y = 2 (gate, up); 256 threads = 4 wavefronts.
// A workgroup takes one expert, one projection, one 128-column tile and up to 8 slabs
// (512 contraction rows).  Wavefront p owns columns [32p, 32p+32) of the tile for all of the
// workgroup's slabs, so partial sums never cross wavefronts; they go to G / U with fp32
// atomics (the slab groups of one tile add into the same outputs).
template <typename HT, bool BF16>
__global__ __launch_bounds__(256) void k_gateup_decode(
    const MatView* __restrict__ gate, const MatView* __restrict__ up, const HT* __restrict__ h_gate,
    const HT* __restrict__ h_up, int Rg, int Ru, const int32_t* __restrict__ token_indices,
    const int32_t* __restrict__ expert_offsets, int T, int A, int I, int n_tiles, int n_groups,
    float* __restrict__ G, float* __restrict__ U) {
    const int mt = blockIdx.y;
    const int bid = blockIdx.x;
    const int grp = bid % n_groups;
    const int tile = (bid / n_groups) % n_tiles;
    const int e = bid / (n_groups * n_tiles);
    const int a_begin = max(expert_offsets[e], 0);
    const int a_end = min(expert_offsets[e + 1], A);
    if (a_end <= a_begin) return;
    const GView mv = load_view(mt ? up : gate, e);
    const int s0 = grp * GU_SLABS_PER_WG;
    const int s1 = min(s0 + GU_SLABS_PER_WG, mv.num_slabs);
    if (s0 >= s1) return;
    const HT* __restrict__ h = mt ? h_up : h_gate;
    const int R = mt ? Ru : Rg;
    float* __restrict__ out = mt ? U : G;

    __shared__ __attribute__((aligned(16))) uint16_t hs[MAX_A * GU_STRIDE];
    __shared__ int tok_sh[MAX_A];

    const int tid = threadIdx.x;
    const int pair = tid >> 6, lane = tid & 63;
    const int n = lane & 15, kg = lane >> 4;

    // 1. issue every payload load of this wavefront before anything else
    uint32_t pw[GU_SLABS_PER_WG][4];
    int bits_s[GU_SLABS_PER_WG];
#pragma unroll
    for (int q = 0; q < GU_SLABS_PER_WG; ++q) {
        const int s = s0 + q;
        bits_s[q] = 0;
        if (s < s1) {
            bits_s[q] = mv.slab_meta[s * 4 + 0];
            const int t = mv.slab_meta[s * 4 + 3] + tile;
            load_pair_role0(mv.payload + mv.tile_meta[t * 3 + 0], bits_s[q], pair, lane, pw[q]);
        }
    }

    for (int a0 = a_begin; a0 < a_end; a0 += MAX_A) {
        const int n_a = min(MAX_A, a_end - a0);
        __syncthreads();
        if (tid < MAX_A) tok_sh[tid] = (tid < n_a) ? token_indices[a0 + tid] : -1;
        __syncthreads();
        // 2. hs'[a][k] for the rows of slabs [s0, s1), the scale of this tile folded in.
        //    Rows a >= n_a are left as they are: MFMA rows are independent and those
        //    output rows are never stored.
        const int n_rows = (s1 - s0) * SLAB_ROWS;
        for (int idx = tid; idx < n_rows; idx += 256) {
            const int s = s0 + (idx >> 6);
            const int row = idx & 63;
            const int k = mv.slab_meta[s * 4 + 2] + row;
            const int t = mv.slab_meta[s * 4 + 3] + tile;
            const int rk = mv.rank_idx[k];
            const float sv = gload_half(mv.s + k) * gload_half(mv.scale + mv.tile_meta[t * 3 + 1] + row);
            const bool rk_ok = rk >= 0 && rk < R;
            for (int a = 0; a < n_a; ++a) {
                const int tk = tok_sh[a];
                float v = 0.0f;
                if (rk_ok && tk >= 0 && tk < T) v = to_f32<HT>(h[(int64_t)tk * R + rk]) * sv;
                hs[a * GU_STRIDE + idx] = to_operand<BF16>(v);
            }
        }
        __syncthreads();
        // 3. decode + MFMA over the slabs
        f32x4 acc[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
        f32x4 corr = {0, 0, 0, 0};
        const uint16_t* ap = hs + n * GU_STRIDE + 16 * kg;
#pragma unroll
        for (int q = 0; q < GU_SLABS_PER_WG; ++q) {
            if (bits_s[q] == 0) continue;
#pragma unroll
            for (int i = 0; i < 4; ++i) pin(pw[q][i]);
            const u32x4 a_lo = *reinterpret_cast<const u32x4*>(ap + q * SLAB_ROWS);
            const u32x4 a_hi = *reinterpret_cast<const u32x4*>(ap + q * SLAB_ROWS + 8);
            if (bits_s[q] == 2)
                gateup_pair<2, BF16>(pw[q], a_lo, a_hi, n >> 3, acc, corr);
            else if (bits_s[q] == 3)
                gateup_pair<3, BF16>(pw[q], a_lo, a_hi, n >> 3, acc, corr);
            else
                gateup_pair<4, BF16>(pw[q], a_lo, a_hi, n >> 3, acc, corr);
        }
        // 4. remove the constant term and add into G / U: lane holds rows a = 4*kg + j of
        //    column 32*pair + 16*nbl + n
#pragma unroll
        for (int nbl = 0; nbl < 2; ++nbl) {
            const int c = tile * N_TILE + 32 * pair + 16 * nbl + n;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int a = 4 * kg + j;
                if (a < n_a && c < I) atomicAdd(&out[(int64_t)(a0 + a) * I + c], acc[nbl][j] - corr[j]);
            }
        }
    }
}

// ----------------------------------------------------------------------------------- down
struct Block16 {   // up to 16 payload words of one lane for one (slab, tile) block
    uint32_t w[16];
};

// role 1 loads: 2-bit 8 words [nb][h], 4-bit 16 words [nb][m], 3-bit 8 low words + 4 high words [nb]
template <int W>
__device__ inline void load_block_role1(gptr<uint32_t> blk, int lane, Block16& b) {
    gptr_u32x4 p = reinterpret_cast<gptr_u32x4>(blk + (W == 4 ? lane * 16 : lane * 8));
    u32x4 v0 = p[0], v1 = p[1], v2 = {0, 0, 0, 0}, v3 = {0, 0, 0, 0};
    if constexpr (W == 4) {
        v2 = p[2];
        v3 = p[3];
    } else if constexpr (W == 3) {
        v2 = *reinterpret_cast<gptr_u32x4>(blk + 512 + lane * 4);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        b.w[i] = v0[i];
        b.w[4 + i] = v1[i];
        b.w[8 + i] = v2[i];
        b.w[12 + i] = v3[i];
    }
}

// One (slab, tile) block of a down matrix: 4 row blocks x 4 k-steps (micro-tiles).
template <int W, bool BF16>
__device__ inline void down_block(const Block16& b, const u32x4 (&az)[4], const float (&sc)[4], f32x4 (&acc)[4]) {
    const u32x4 bc = corr_operand<W, BF16>();
    f32x4 corr = {0, 0, 0, 0};
#pragma unroll
    for (int m = 0; m < 4; ++m) corr = mfma16<BF16>(az[m], bc, corr);
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
        f32x4 t = {0, 0, 0, 0};
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            u32x4 bw;
            if constexpr (W == 2)
                bw = decode_fields2<2, BF16>(b.w[nb * 2 + (m >> 1)], 8 * (m & 1));
            else if constexpr (W == 4)
                bw = decode_fields4<BF16>(b.w[nb * 4 + m]);
            else
                bw = decode_fields3<BF16>(b.w[nb * 2 + (m >> 1)], 8 * (m & 1), b.w[8 + nb], 4 * m);
            t = mfma16<BF16>(az[m], bw, t);
        }
        acc[nb] += (t - corr) * sc[nb];
    }
}

template <int W, bool BF16>
__device__ inline void down_slab(const GView& mv, int si, int n_tiles, int lane, const uint16_t* __restrict__ z,
                                 int z_stride, f32x4 (&acc)[4]) {
    const int n = lane & 15, kg = lane >> 4;
    const int tile_off = mv.slab_meta[si * 4 + 3];
    Block16 cur, nxt;
    float sc_cur[4], sc_nxt[4];
    auto issue = [&](int t, Block16& b, float (&sc)[4]) {
        const int tm = (tile_off + t) * 3;
        load_block_role1<W>(mv.payload + mv.tile_meta[tm + 0], lane, b);
        gptr<__half> sp = mv.scale + mv.tile_meta[tm + 1] + n;
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) sc[nb] = gload_half(sp + 16 * nb);
    };
    issue(0, cur, sc_cur);
    for (int t = 0; t < n_tiles; ++t) {
        if (t + 1 < n_tiles) issue(t + 1, nxt, sc_nxt);
        u32x4 az[4];
        const uint16_t* zp = z + n * z_stride + t * N_TILE + 8 * kg;
#pragma unroll
        for (int m = 0; m < 4; ++m) az[m] = *reinterpret_cast<const u32x4*>(zp + 32 * m);
        down_block<W, BF16>(cur, az, sc_cur, acc);
        cur = nxt;
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) sc_cur[nb] = sc_nxt[nb];
    }
}

// grid.x = E * n_groups; 256 threads; dynamic LDS = 16 * (n_tiles * 128 + 8) * 2 bytes.
template <bool BF16>
__global__ __launch_bounds__(256) void k_down_decode(
    const MatView* __restrict__ down, const float* __restrict__ G, const float* __restrict__ U,
    const float* __restrict__ route_w, const int32_t* __restrict__ token_indices,
    const int32_t* __restrict__ expert_offsets, int T, int A, int I, int n_tiles, int n_groups, int rank_out,
    float* __restrict__ rank_accum) {
    const int grp = blockIdx.x % n_groups;
    const int e = blockIdx.x / n_groups;
    const int a_begin = max(expert_offsets[e], 0);
    const int a_end = min(expert_offsets[e + 1], A);
    if (a_end <= a_begin) return;
    const GView mv = load_view(down, e);
    if (grp * DN_SLABS_PER_WG >= mv.num_slabs) return;

    extern __shared__ __attribute__((aligned(16))) unsigned char dsmem[];
    uint16_t* z = reinterpret_cast<uint16_t*>(dsmem);
    __shared__ int tok_sh[MAX_A];
    __shared__ float rw_sh[MAX_A];
    const int z_stride = n_tiles * N_TILE + 8;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int n = lane & 15, g4 = (lane >> 4) * 4;
    const int si = grp * DN_SLABS_PER_WG + wave;
    const bool active = si < mv.num_slabs;
    const int bits = active ? mv.slab_meta[si * 4 + 0] : 0;

    for (int a0 = a_begin; a0 < a_end; a0 += MAX_A) {
        const int n_a = min(MAX_A, a_end - a0);
        __syncthreads();
        if (tid < MAX_A) {
            tok_sh[tid] = (tid < n_a) ? token_indices[a0 + tid] : -1;
            rw_sh[tid] = (tid < n_a) ? route_w[a0 + tid] : 0.0f;
        }
        // z[a][c] = silu(G) * U as 16-bit operands for the rows a < n_a (other rows feed
        // output rows that are never stored)
        for (int idx = tid; idx < n_a * I; idx += 256) {
            const int a = idx / I, c = idx - a * I;
            const int64_t gi = (int64_t)(a0 + a) * I + c;
            z[a * z_stride + c] = to_operand<BF16>(silu_f32(G[gi]) * U[gi]);
        }
        __syncthreads();
        if (active) {
            f32x4 acc[4];
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) acc[nb] = f32x4{0, 0, 0, 0};
            if (bits == 2)
                down_slab<2, BF16>(mv, si, n_tiles, lane, z, z_stride, acc);
            else if (bits == 3)
                down_slab<3, BF16>(mv, si, n_tiles, lane, z, z_stride, acc);
            else
                down_slab<4, BF16>(mv, si, n_tiles, lane, z, z_stride, acc);
            // combine: rows of this slab are distinct output ranks
            const int rank_off = mv.slab_meta[si * 4 + 2];
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) {
                const int row = rank_off + 16 * nb + n;
                const int lr = mv.rank_idx[row];
                const float sv = gload_half(mv.s + row);
                if (lr < 0 || lr >= rank_out) continue;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int a = g4 + j;
                    const int tk = tok_sh[a];
                    if (a < n_a && tk >= 0 && tk < T)
                        atomicAdd(&rank_accum[(int64_t)tk * rank_out + lr], acc[nb][j] * sv * rw_sh[a]);
                }
            }
        }
    }
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
    const size_t z_bytes = (size_t)MAX_A * (n_tiles * N_TILE + 8) * 2;
    return gate->role == ROLE_GATE_UP && up->role == ROLE_GATE_UP && down->role == ROLE_DOWN && z_bytes <= 65536 &&
           I % N_TILE == 0;
}

int launch_forward_decode(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                          const void* h_gate, const void* h_up, int act_dtype, int64_t T, int Rg, int Ru,
                          const int32_t* tok, const int32_t* off, const float* rw, int64_t A, int rank_out, int I,
                          float* rank_accum, float* G, float* U, int64_t inter_floats, bitsmoe_profile* prof,
                          hipStream_t st) {
    const int E = gate->n_experts;
    const int n_tiles = gate->n_tiles;
    record(prof, 0, st);
    {
        // G and U are adjacent in the workspace: one range; rank_accum is the second
        const int64_t n1 = inter_floats + A * (int64_t)I;
        const int64_t n2 = T * (int64_t)rank_out;
        const int64_t blocks = std::min<int64_t>((std::max(n1, n2) + 255) / 256, 2048);
        hipLaunchKernelGGL(k_fill_zero2, dim3((unsigned)blocks), dim3(256), 0, st, G, n1, rank_accum, n2);
        BITSMOE_HIP_TRY(hipGetLastError());
    }
    record(prof, 1, st);
    const int max_slabs = std::max(gate->max_slabs, up->max_slabs);
    const int gu_groups = (max_slabs + GU_SLABS_PER_WG - 1) / GU_SLABS_PER_WG;
    dim3 grid((unsigned)(E * n_tiles * gu_groups), 2);
    if (act_dtype == BITSMOE_DT_BF16) {
        hipLaunchKernelGGL((k_gateup_decode<__hip_bfloat16, true>), grid, dim3(256), 0, st, gate->d_views_prepared,
                           up->d_views_prepared, (const __hip_bfloat16*)h_gate, (const __hip_bfloat16*)h_up, Rg, Ru,
                           tok, off, (int)T, (int)A, I, n_tiles, gu_groups, G, U);
    } else {
        hipLaunchKernelGGL((k_gateup_decode<__half, false>), grid, dim3(256), 0, st, gate->d_views_prepared,
                           up->d_views_prepared, (const __half*)h_gate, (const __half*)h_up, Rg, Ru, tok, off, (int)T,
                           (int)A, I, n_tiles, gu_groups, G, U);
    }
    BITSMOE_HIP_TRY(hipGetLastError());
    record(prof, 2, st);
    const int dn_groups = (down->max_slabs + DN_SLABS_PER_WG - 1) / DN_SLABS_PER_WG;
    const size_t z_bytes = (size_t)MAX_A * (n_tiles * N_TILE + 8) * 2;
    if (act_dtype == BITSMOE_DT_BF16) {
        hipLaunchKernelGGL((k_down_decode<true>), dim3((unsigned)(E * dn_groups)), dim3(256), z_bytes, st,
                           down->d_views_prepared, G, U, rw, tok, off, (int)T, (int)A, I, n_tiles, dn_groups, rank_out,
                           rank_accum);
    } else {
        hipLaunchKernelGGL((k_down_decode<false>), dim3((unsigned)(E * dn_groups)), dim3(256), z_bytes, st,
                           down->d_views_prepared, G, U, rw, tok, off, (int)T, (int)A, I, n_tiles, dn_groups, rank_out,
                           rank_accum);
    }
    BITSMOE_HIP_TRY(hipGetLastError());
    record(prof, 3, st);
    if (prof) prof->recorded = true;
    return BITSMOE_OK;
}

}  // namespace bitsmoe
