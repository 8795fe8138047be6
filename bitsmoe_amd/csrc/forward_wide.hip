// Side kernels for the wide rows of prepared matrix sets: rows of 6-, 8- and 16-bit slabs (dense "super"
// experts are all such rows: bitsmoe/models/base_block.py:291-307 runs them as modules; a bit allocation may
// put such a bucket into any matrix: bitsmoe/quant/packer.py:566-589).  They are stored as f16 weights in
// MFMA operand order (wide_layout.h) -- nothing to decode -- and these kernels add their share to what the
// fast kernels compute from the 2/3/4-bit rows: contraction rows in gate/up (the sums are linear in the rows),
// output rows in down (every row is an output rank of its own).  Work is proportional to the assignments of the
// experts that have such rows; both kernels need the routing tables.
#include "wide_layout.h"

#include <algorithm>

namespace bitsmoe {

constexpr int WD_M = 64;             // assignments per block of rows
constexpr int WD_A_LD = 64 + 8;      // halves per row of the staged activation piece (64 contraction rows)
constexpr int WD_Z_LD = N_TILE + 8;  // halves per row of the staged z piece (one tile)

struct WideSet {
    const int32_t* first;      // [E + 1]
    const int32_t* experts;    // experts with wide rows
    int n_experts;
    const int32_t* rank;       // [slabs * 64]
    const __half* s;           // [slabs * 64]
    const __half* weights;     // [slabs][n_tiles][WIDE_BLOCK]
};
bool has_wide_rows(const bitsmoe_matset* set) { return set->wide_slabs > 0; }
bool only_wide_rows(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down) {
    return has_wide_rows(gate) && has_wide_rows(up) && has_wide_rows(down) && gate->narrow_rows == 0 && up->narrow_rows == 0 &&
           down->narrow_rows == 0;
}
static WideSet wide_set_of(const bitsmoe_matset* set) {
    return WideSet{set->d_wide_first, set->d_wide_experts, set->n_wide_experts, set->d_wide_rank, set->d_wide_s, set->d_wide};
}

template <bool BF16>
__device__ inline float act_f32(uint16_t bits) {
    if constexpr (BF16)
        return __uint_as_float((uint32_t)bits << 16);
    else
        return __half2float(__ushort_as_half(bits));
}

// grid.x = (expert of the projection's list, tile, chunk of `chunk` wide slabs, row slot), grid.y = projection.
// A workgroup contracts its chunk of wide slabs for the rows m0 = 64 * slot, 64 * (slot + n_slots), ... of its
// expert: wavefront w owns the 16-column blocks 2w and 2w + 1 of the tile.  F16SUMS: the sums are f16 and this
// workgroup is the only one that adds to its elements (chunk = all slabs): read, add, write.  Otherwise fp32
// atomics.
template <bool BF16, bool F16SUMS>
__global__ __launch_bounds__(256) void k_wide_gateup(WideSet gate, WideSet up, const uint16_t* __restrict__ h_gate,
                                                     const uint16_t* __restrict__ h_up, int Rg, int Ru, int64_t ldg, int64_t ldu,
                                                     const int32_t* __restrict__ tok, const int32_t* __restrict__ off, int I,
                                                     int n_tiles, int chunk, int n_chunks, int n_slots, void* __restrict__ G,
                                                     void* __restrict__ U) {
    __shared__ __attribute__((aligned(16))) uint16_t sA[WD_M * WD_A_LD];
    const bool is_up = blockIdx.y != 0;
    const WideSet ws_tab = is_up ? up : gate;
    int x = blockIdx.x;
    const int slot = x % n_slots;
    x /= n_slots;
    const int ch = x % n_chunks;
    x /= n_chunks;
    const int t = x % n_tiles;
    x /= n_tiles;
    if (x >= ws_tab.n_experts) return;
    const int e = ws_tab.experts[x];
    const int a0 = off[e], na = off[e + 1] - a0;
    const int s0 = ws_tab.first[e] + ch * chunk, s1 = min(ws_tab.first[e + 1], s0 + chunk);
    if (slot * WD_M >= na || s0 >= s1) return;
    const uint16_t* __restrict__ h = is_up ? h_up : h_gate;
    const int R = is_up ? Ru : Rg;
    const int64_t ld = is_up ? ldu : ldg;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int srow = tid >> 2, sk0 = (tid & 3) * 16;      // the staging thread's row and first contraction row
    for (int m0 = slot * WD_M; m0 < na; m0 += n_slots * WD_M) {
        const int my_a = m0 + srow < na ? a0 + m0 + srow : -1;
        const int my_tok = my_a >= 0 ? tok[my_a] : -1;
        f32x4 acc[4][2];
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
            acc[mb][0] = acc[mb][1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        for (int sl = s0; sl < s1; ++sl) {
            // the wavefront's weight operands of this slab: [ks][n]
            u32x4 b[2][2];
            const __half* __restrict__ blk = ws_tab.weights + ((int64_t)sl * n_tiles + t) * WIDE_BLOCK;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int n = 0; n < 2; ++n)
                    b[ks][n] = *reinterpret_cast<const u32x4*>(blk + (((ks * 8 + 2 * wave + n) * 64) + lane) * 8);
            // activation piece: f16(h[tok, rank'[k]] * s'[k]), 64 rows x 64 contraction rows
            uint16_t vals[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int k = sl * SLAB_ROWS + sk0 + j;
                const int rk = ws_tab.rank[k];
                float v = 0.0f;
                if (my_tok >= 0 && rk >= 0 && rk < R) v = act_f32<BF16>(h[(int64_t)my_tok * ld + rk]) * __half2float(ws_tab.s[k]);
                vals[j] = to_operand<false>(v);
            }
            __syncthreads();      // (the previous slab's operand reads are done)
#pragma unroll
            for (int j = 0; j < 16; j += 8) {
                u32x4 p;
#pragma unroll
                for (int q = 0; q < 4; ++q) p[q] = (uint32_t)vals[j + 2 * q] | ((uint32_t)vals[j + 2 * q + 1] << 16);
                *reinterpret_cast<u32x4*>(&sA[srow * WD_A_LD + sk0 + j]) = p;
            }
            __syncthreads();
#pragma unroll
            for (int mb = 0; mb < 4; ++mb) {
                if (m0 + mb * 16 >= na) break;
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const u32x4 a = *reinterpret_cast<const u32x4*>(&sA[(mb * 16 + (lane & 15)) * WD_A_LD + ks * 32 + (lane >> 4) * 8]);
                    acc[mb][0] = mfma16<false>(a, b[ks][0], acc[mb][0]);
                    acc[mb][1] = mfma16<false>(a, b[ks][1], acc[mb][1]);
                }
            }
        }
        // lane holds rows 16 mb + 4 (lane / 16) + j of column lane % 16 of its two column blocks
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int n = 0; n < 2; ++n)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int row = m0 + mb * 16 + (lane >> 4) * 4 + j;
                    if (row >= na) continue;
                    const int64_t at = (int64_t)(a0 + row) * I + t * N_TILE + (2 * wave + n) * 16 + (lane & 15);
                    if constexpr (F16SUMS) {
                        _Float16* p = reinterpret_cast<_Float16*>(is_up ? U : G) + at;
                        *p = (_Float16)((float)*p + acc[mb][n][j]);
                    } else {
                        atomicAdd(reinterpret_cast<float*>(is_up ? U : G) + at, acc[mb][n][j]);
                    }
                }
    }
}

// grid.x = (expert of the list, wide slab of the expert, row slot).  A workgroup computes one wide slab (64 output
// rows: wavefront w owns rows 16w .. 16w + 15) for the rows m0 = 64 * slot, ... of its expert, contracting over
// all columns tile by tile, and adds s'[r] * route_w[a] * sum into rank_accum[tok[a], rank'[r]] by atomics.
// ZF16: `g` holds z = silu(G) * U as f16 [A, I]; otherwise g / u hold n_part fp32 partial sums part_stride apart.
template <bool ZF16>
__global__ __launch_bounds__(256) void k_wide_down(WideSet down, int max_slabs, const void* __restrict__ g,
                                                   const float* __restrict__ u, int n_part, int64_t part_stride,
                                                   const int32_t* __restrict__ tok, const int32_t* __restrict__ off,
                                                   const float* __restrict__ route_w, int I, int n_tiles, int n_slots,
                                                   int rank_out, float* __restrict__ rank_accum) {
    __shared__ __attribute__((aligned(16))) uint16_t sZ[WD_M * WD_Z_LD];
    int x = blockIdx.x;
    const int slot = x % n_slots;
    x /= n_slots;
    const int j_slab = x % max_slabs;
    x /= max_slabs;
    if (x >= down.n_experts) return;
    const int e = down.experts[x];
    const int sl = down.first[e] + j_slab;
    const int a0 = off[e], na = off[e + 1] - a0;
    if (sl >= down.first[e + 1] || slot * WD_M >= na) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int srow = tid >> 2, sc0 = (tid & 3) * 32;      // the staging thread's row and first column of the tile
    const int out_row = sl * SLAB_ROWS + wave * 16 + (lane & 15);
    const int rk = down.rank[out_row];
    const float sv = __half2float(down.s[out_row]);
    for (int m0 = slot * WD_M; m0 < na; m0 += n_slots * WD_M) {
        const int my_a = m0 + srow < na ? a0 + m0 + srow : -1;
        f32x4 acc[4];
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) acc[mb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        for (int t = 0; t < n_tiles; ++t) {
            u32x4 b[4];
            const __half* __restrict__ blk = down.weights + ((int64_t)sl * n_tiles + t) * WIDE_BLOCK;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) b[ks] = *reinterpret_cast<const u32x4*>(blk + (((ks * 4 + wave) * 64) + lane) * 8);
            // z piece: 64 rows x 128 columns, 32 columns per thread
            u32x4 zp[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) zp[q] = u32x4{0u, 0u, 0u, 0u};
            if (my_a >= 0) {
                const int64_t at = (int64_t)my_a * I + t * N_TILE + sc0;
                if constexpr (ZF16) {
                    const u32x4* src = reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(g) + at);
#pragma unroll
                    for (int q = 0; q < 4; ++q) zp[q] = src[q];
                } else {
                    const float* gp = reinterpret_cast<const float*>(g) + at;
                    const float* up = u + at;
#pragma unroll
                    for (int q = 0; q < 4; ++q)
#pragma unroll
                        for (int hv = 0; hv < 2; ++hv) {      // four columns at a time
                            f32x4 gv = *reinterpret_cast<const f32x4*>(gp + q * 8 + hv * 4);
                            f32x4 uv = *reinterpret_cast<const f32x4*>(up + q * 8 + hv * 4);
                            for (int p = 1; p < n_part; ++p) {
                                gv += *reinterpret_cast<const f32x4*>(gp + p * part_stride + q * 8 + hv * 4);
                                uv += *reinterpret_cast<const f32x4*>(up + p * part_stride + q * 8 + hv * 4);
                            }
                            zp[q][2 * hv] = (uint32_t)to_operand<false>(silu_f32(gv[0]) * uv[0]) |
                                            ((uint32_t)to_operand<false>(silu_f32(gv[1]) * uv[1]) << 16);
                            zp[q][2 * hv + 1] = (uint32_t)to_operand<false>(silu_f32(gv[2]) * uv[2]) |
                                                ((uint32_t)to_operand<false>(silu_f32(gv[3]) * uv[3]) << 16);
                        }
                }
            }
            __syncthreads();      // (the previous tile's operand reads are done)
#pragma unroll
            for (int q = 0; q < 4; ++q) *reinterpret_cast<u32x4*>(&sZ[srow * WD_Z_LD + sc0 + q * 8]) = zp[q];
            __syncthreads();
#pragma unroll
            for (int mb = 0; mb < 4; ++mb) {
                if (m0 + mb * 16 >= na) break;
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    const u32x4 a = *reinterpret_cast<const u32x4*>(&sZ[(mb * 16 + (lane & 15)) * WD_Z_LD + ks * 32 + (lane >> 4) * 8]);
                    acc[mb] = mfma16<false>(a, b[ks], acc[mb]);
                }
            }
        }
        if (rk < 0 || rk >= rank_out) continue;
        // lane holds assignments 16 mb + 4 (lane / 16) + j of its output row
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int row = m0 + mb * 16 + (lane >> 4) * 4 + j;
                if (row >= na) continue;
                const int a = a0 + row;
                atomicAdd(&rank_accum[(int64_t)tok[a] * rank_out + rk], acc[mb][j] * sv * route_w[a]);
            }
    }
}

// Row slots: workgroups that share (expert, tile, chunk) and take every n-th block of 64 rows.  Enough of them
// that the launch has a few workgroups per CU when every assignment went to experts with wide rows, no more
// than the blocks of rows there can be.
static int row_slots(int64_t A, int64_t units) {
    const int64_t blocks = std::max<int64_t>((A + WD_M - 1) / WD_M, 1);
    const int64_t want = std::max<int64_t>(1024 / std::max<int64_t>(units, 1), 1);
    return (int)std::min<int64_t>(std::min<int64_t>(blocks, want), 64);
}

int launch_wide_gateup(const bitsmoe_matset* gate, const bitsmoe_matset* up, const void* h_gate, const void* h_up,
                       int act_dtype, int Rg, int Ru, int64_t ldg, int64_t ldu, const int32_t* tok, const int32_t* off,
                       int64_t A, int I, void* G, void* U, bool sums_f16, hipStream_t st) {
    if ((!has_wide_rows(gate) && !has_wide_rows(up)) || A <= 0) return BITSMOE_OK;
    BITSMOE_REQUIRE(tok && off, "the wide rows of these matrix sets need the routing tables");
    const int n_tiles = gate->n_tiles;
    const int n_exp = std::max(gate->n_wide_experts, up->n_wide_experts);
    int max_slabs = 0;
    for (const bitsmoe_matset* set : {gate, up})
        for (int e = 0; e < set->n_experts && has_wide_rows(set); ++e)
            max_slabs = std::max(max_slabs, set->wide_first_host[e + 1] - set->wide_first_host[e]);
    // f16 sums: one workgroup per element (all slabs in one chunk); fp32 sums: chunks of four slabs
    const int chunk = sums_f16 ? max_slabs : 4;
    const int n_chunks = (max_slabs + chunk - 1) / chunk;
    const int n_slots = row_slots(A, (int64_t)n_exp * n_tiles * n_chunks * 2);
    const dim3 grid((unsigned)((int64_t)n_exp * n_tiles * n_chunks * n_slots), 2);
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, st, wide_set_of(gate), wide_set_of(up), (const uint16_t*)h_gate,
                           (const uint16_t*)h_up, Rg, Ru, ldg, ldu, tok, off, I, n_tiles, chunk, n_chunks, n_slots, G, U);
    };
    const bool bf16 = act_dtype == BITSMOE_DT_BF16;
    if (sums_f16) {
        if (bf16) launch(k_wide_gateup<true, true>); else launch(k_wide_gateup<false, true>);
    } else {
        if (bf16) launch(k_wide_gateup<true, false>); else launch(k_wide_gateup<false, false>);
    }
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}

int launch_wide_down(const bitsmoe_matset* down, const void* g_or_z, const float* u, bool z_f16, int n_part,
                     int64_t part_stride, const int32_t* tok, const int32_t* off, const float* rw, int64_t A, int I,
                     int rank_out, float* rank_accum, hipStream_t st) {
    if (!has_wide_rows(down) || A <= 0) return BITSMOE_OK;
    BITSMOE_REQUIRE(tok && off && rw, "the wide rows of this matrix set need the routing tables");
    int max_slabs = 0;
    for (int e = 0; e < down->n_experts; ++e) max_slabs = std::max(max_slabs, down->wide_first_host[e + 1] - down->wide_first_host[e]);
    const int n_slots = row_slots(A, (int64_t)down->n_wide_experts * max_slabs);
    const dim3 grid((unsigned)((int64_t)down->n_wide_experts * max_slabs * n_slots));
    if (z_f16)
        hipLaunchKernelGGL(k_wide_down<true>, grid, dim3(256), 0, st, wide_set_of(down), max_slabs, g_or_z, u, 1, (int64_t)0, tok, off,
                           rw, I, down->n_tiles, n_slots, rank_out, rank_accum);
    else
        hipLaunchKernelGGL(k_wide_down<false>, grid, dim3(256), 0, st, wide_set_of(down), max_slabs, g_or_z, u, n_part, part_stride,
                           tok, off, rw, I, down->n_tiles, n_slots, rank_out, rank_accum);
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}

}  // namespace bitsmoe
