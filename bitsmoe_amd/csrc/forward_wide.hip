// Side kernels for the wide rows of prepared matrix sets: rows of 6-, 8- and 16-bit slabs (dense "super"
// experts are all such rows: bitsmoe/models/base_block.py:291-307 runs them as modules; a bit allocation may
// put such a bucket into any matrix: bitsmoe/quant/packer.py:566-589).  They are stored as f16 weights in
// MFMA operand order (wide_layout.h) -- nothing to decode -- and these kernels add their share to what the
// fast kernels compute from the 2/3/4-bit rows: contraction rows in gate/up (the sums are linear in the rows),
// output rows in down (every row is an output rank of its own).  Work is proportional to the assignments of the
// experts that have such rows.  Sets of dense experts only (every row wide) run these kernels alone; for small
// batches of those the kernels find their assignments among the routed ids themselves, as the decode kernels do.
#include "decode_bodies.h"
#include "wide_layout.h"

#include <algorithm>

namespace bitsmoe {

constexpr int WD_M = 64;             // assignments per block of rows
constexpr int WD_CH = 4;             // wide slabs whose operands a gate/up workgroup holds at a time
constexpr int WD_TC = 2;             // column tiles whose operands a down workgroup holds at a time
constexpr int WD_A_LD = 64 + 8;      // halves per row of a staged activation piece (64 contraction rows)
constexpr int WD_Z_LD = WD_TC * N_TILE + 8;      // halves per row of the staged z piece

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

// Where a workgroup's assignments come from.  Tables: expert e owns rows [off[e], off[e + 1]) of the routing tables,
// which are also its rows of the intermediates.  Routed (sets of dense experts, at most ROUTE_INLINE_MAX_FLAT
// routed entries): the workgroup scans the routed ids for its expert's entries itself; its j-th entry is row
// x * rows_per_expert + j of the intermediates, x the expert's position in the list of wide experts.
struct WideRouted {
    const void* selected;
    int ids_are_i64;
    int n_flat, top_k;
    const int32_t* local_to_global;
    const float* weights;      // [T * k]
    int rows_per_expert;
};

template <bool BF16>
__device__ inline float act_f32(uint16_t bits) {
    if constexpr (BF16)
        return __uint_as_float((uint32_t)bits << 16);
    else
        return __half2float(__ushort_as_half(bits));
}

// grid.x = (expert of the projection's list, tile, chunk of `chunk` wide slabs, row slot), grid.y = projection.
// A workgroup contracts its chunk of wide slabs, WD_CH at a time (their operands requested together, before the
// assignments are known), for the rows m0 = 64 * slot, 64 * (slot + n_slots), ... of its expert: wavefront w
// owns the 16-column blocks 2w and 2w + 1 of the tile.  F16SUMS: the sums are f16 and this workgroup is the only
// one that adds to its elements (chunk = all slabs): read, add, write.  Otherwise fp32 atomics.
// IDENT: rank'[k] = k and 16-byte aligned activation rows: the activations of a slab quarter are two 16-byte loads.
// `clear`: n_clear floats every workgroup clears a share of (the output of a forward that no other kernel clears).
template <bool BF16, bool F16SUMS, bool ROUTED, bool IDENT>
__global__ __launch_bounds__(256) void k_wide_gateup(WideSet gate, WideSet up, const uint16_t* __restrict__ h_gate,
                                                     const uint16_t* __restrict__ h_up, int Rg, int Ru, int64_t ldg, int64_t ldu,
                                                     const int32_t* __restrict__ tok, const int32_t* __restrict__ off, WideRouted ra,
                                                     int I, int n_tiles, int chunk, int n_chunks, int n_slots, int uniform_slabs,
                                                     void* __restrict__ G, void* __restrict__ U, float* __restrict__ clear,
                                                     int64_t n_clear) {
    __shared__ __attribute__((aligned(16))) uint16_t sA[WD_CH * WD_M * WD_A_LD];
    __shared__ InlineRouteLds route_lds;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (clear) {
        const int64_t n4 = n_clear >> 2, stride = (int64_t)gridDim.x * gridDim.y * 256;
        for (int64_t i = ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * 256 + tid; i < n4; i += stride)
            reinterpret_cast<f32x4*>(clear)[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        if (blockIdx.x == 0 && blockIdx.y == 0 && tid < (int)(n_clear & 3)) clear[(n4 << 2) + tid] = 0.0f;
    }
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
    // (uniform_slabs > 0: every expert of the set has that many wide slabs and the list holds every expert)
    const int e = uniform_slabs > 0 ? x : ws_tab.experts[x];
    const int first = uniform_slabs > 0 ? x * uniform_slabs : ws_tab.first[e];
    const int last = uniform_slabs > 0 ? first + uniform_slabs : ws_tab.first[e + 1];
    const int s0 = first + ch * chunk, s1 = min(last, s0 + chunk);
    // the wavefront's weight operands of up to WD_CH slabs: [slab][ks][n]
    u32x4 b[WD_CH][2][2];
    auto request_weights = [&](int sb) {
#pragma unroll
        for (int q = 0; q < WD_CH; ++q) {
            const __half* __restrict__ blk = ws_tab.weights + ((int64_t)min(sb + q, s1 - 1) * n_tiles + t) * WIDE_BLOCK;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int n = 0; n < 2; ++n)
                    b[q][ks][n] = *reinterpret_cast<const u32x4*>(blk + (((ks * 8 + 2 * wave + n) * 64) + lane) * 8);
        }
    };
    const bool early = uniform_slabs > 0 && s0 < s1;
    if (early) request_weights(s0);      // (in flight while the assignments are found)
    int a0 = 0, na;
    if constexpr (ROUTED) {
        na = inline_route(ra.selected, ra.ids_are_i64, ra.n_flat, ra.top_k, ra.local_to_global[e], route_lds, tid);
        a0 = x * ra.rows_per_expert;
    } else {
        a0 = off[e];
        na = off[e + 1] - a0;
    }
    if (slot * WD_M >= na || s0 >= s1) return;
    const uint16_t* __restrict__ h = is_up ? h_up : h_gate;
    const int R = is_up ? Ru : Rg;
    const int64_t ld = is_up ? ldu : ldg;
    const int srow = tid >> 2, sk0 = (tid & 3) * 16;      // the staging thread's row and first contraction row of a slab
    for (int m0 = slot * WD_M; m0 < na; m0 += n_slots * WD_M) {
        int my_tok = -1;
        if (m0 + srow < na) {
            if constexpr (ROUTED)
                my_tok = route_lds.tok[m0 + srow];
            else
                my_tok = tok[a0 + m0 + srow];
        }
        f32x4 acc[4][2];
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) acc[mb][0] = acc[mb][1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        for (int sb = s0; sb < s1; sb += WD_CH) {
            if (!(early && sb == s0 && m0 == slot * WD_M)) request_weights(sb);
            // activation pieces: f16(h[tok, rank'[k]] * s'[k]), 64 rows x 64 contraction rows per slab
            u32x4 piece[WD_CH][2];
#pragma unroll
            for (int q = 0; q < WD_CH; ++q) {
                piece[q][0] = piece[q][1] = u32x4{0u, 0u, 0u, 0u};
                if (sb + q >= s1 || my_tok < 0) continue;
                const int k0 = (sb + q) * SLAB_ROWS + sk0;
                if constexpr (IDENT) {
                    const int col = (sb + q - first) * SLAB_ROWS + sk0;      // rank'[k0 + j] = col + j
                    if (col + 16 <= R) {
                        const u32x4* hp = reinterpret_cast<const u32x4*>(h + (int64_t)my_tok * ld + col);
                        const u32x4* sp = reinterpret_cast<const u32x4*>(ws_tab.s + k0);
#pragma unroll
                        for (int hf = 0; hf < 2; ++hf) {
                            const u32x4 hv = hp[hf], sv = sp[hf];
#pragma unroll
                            for (int i = 0; i < 4; ++i) {
                                const float lo = act_f32<BF16>((uint16_t)(hv[i] & 0xFFFFu)) *
                                                 __half2float(__ushort_as_half((uint16_t)(sv[i] & 0xFFFFu)));
                                const float hi = act_f32<BF16>((uint16_t)(hv[i] >> 16)) *
                                                 __half2float(__ushort_as_half((uint16_t)(sv[i] >> 16)));
                                piece[q][hf][i] = (uint32_t)to_operand<false>(lo) | ((uint32_t)to_operand<false>(hi) << 16);
                            }
                        }
                        continue;
                    }
                }
                uint16_t vals[16];
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const int rk = ws_tab.rank[k0 + j];
                    float v = 0.0f;
                    if (rk >= 0 && rk < R) v = act_f32<BF16>(h[(int64_t)my_tok * ld + rk]) * __half2float(ws_tab.s[k0 + j]);
                    vals[j] = to_operand<false>(v);
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) piece[q][j >> 2][j & 3] = (uint32_t)vals[2 * j] | ((uint32_t)vals[2 * j + 1] << 16);
            }
            __syncthreads();      // (the previous pieces' operand reads are done)
#pragma unroll
            for (int q = 0; q < WD_CH; ++q) {
                *reinterpret_cast<u32x4*>(&sA[(q * WD_M + srow) * WD_A_LD + sk0]) = piece[q][0];
                *reinterpret_cast<u32x4*>(&sA[(q * WD_M + srow) * WD_A_LD + sk0 + 8]) = piece[q][1];
            }
            __syncthreads();
#pragma unroll
            for (int q = 0; q < WD_CH; ++q) {
                if (sb + q >= s1) break;
#pragma unroll
                for (int mb = 0; mb < 4; ++mb) {
                    if (m0 + mb * 16 >= na) break;
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) {
                        const u32x4 a = *reinterpret_cast<const u32x4*>(
                            &sA[(q * WD_M + mb * 16 + (lane & 15)) * WD_A_LD + ks * 32 + (lane >> 4) * 8]);
                        acc[mb][0] = mfma16<false>(a, b[q][ks][0], acc[mb][0]);
                        acc[mb][1] = mfma16<false>(a, b[q][ks][1], acc[mb][1]);
                    }
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

// grid.x = (expert of the list, wide slab of the expert, chunk of tiles, row slot).  A workgroup computes one wide
// slab (64 output rows: wavefront w owns rows 16w .. 16w + 15) for the rows m0 = 64 * slot, ... of its expert,
// contracting over its chunk of column tiles, WD_TC tiles at a time, and adds s'[r] * route_w[a] * sum into
// rank_accum[tok[a], rank'[r]] by atomics.
// ZF16: `g` holds z = silu(G) * U as f16 [A, I]; otherwise g / u hold n_part fp32 partial sums part_stride apart.
template <bool ZF16, bool ROUTED>
__global__ __launch_bounds__(256) void k_wide_down(WideSet down, int max_slabs, const void* __restrict__ g,
                                                   const float* __restrict__ u, int n_part, int64_t part_stride,
                                                   const int32_t* __restrict__ tok, const int32_t* __restrict__ off,
                                                   const float* __restrict__ route_w, WideRouted ra, int I, int n_tiles,
                                                   int tiles_per_wg, int n_tchunks, int n_slots, int uniform_slabs, int rank_out,
                                                   float* __restrict__ rank_accum) {
    __shared__ __attribute__((aligned(16))) uint16_t sZ[WD_M * WD_Z_LD];
    __shared__ InlineRouteLds route_lds;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int x = blockIdx.x;
    const int slot = x % n_slots;
    x /= n_slots;
    const int tc = x % n_tchunks;
    x /= n_tchunks;
    const int j_slab = x % max_slabs;
    x /= max_slabs;
    if (x >= down.n_experts) return;
    const int e = uniform_slabs > 0 ? x : down.experts[x];
    const int first = uniform_slabs > 0 ? x * uniform_slabs : down.first[e];
    const int last = uniform_slabs > 0 ? first + uniform_slabs : down.first[e + 1];
    const int sl = first + j_slab;
    const int t0 = tc * tiles_per_wg, t1 = min(n_tiles, t0 + tiles_per_wg);
    u32x4 b[WD_TC][4];
    auto request_weights = [&](int tb) {
#pragma unroll
        for (int q = 0; q < WD_TC; ++q) {
            const __half* __restrict__ blk = down.weights + ((int64_t)sl * n_tiles + min(tb + q, t1 - 1)) * WIDE_BLOCK;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) b[q][ks] = *reinterpret_cast<const u32x4*>(blk + (((ks * 4 + wave) * 64) + lane) * 8);
        }
    };
    const bool early = uniform_slabs > 0 && t0 < t1;      // (sl < last by construction: max_slabs == uniform_slabs)
    if (early) request_weights(t0);
    int a0 = 0, na;
    if constexpr (ROUTED) {
        na = inline_route(ra.selected, ra.ids_are_i64, ra.n_flat, ra.top_k, ra.local_to_global[e], route_lds, tid);
        a0 = x * ra.rows_per_expert;
    } else {
        a0 = off[e];
        na = off[e + 1] - a0;
    }
    if (sl >= last || slot * WD_M >= na || t0 >= t1) return;
    const int srow = tid >> 2, sc0 = (tid & 3) * 32;      // the staging thread's row and first column of a tile
    const int out_row = sl * SLAB_ROWS + wave * 16 + (lane & 15);
    const int rk = down.rank[out_row];
    const float sv = __half2float(down.s[out_row]);
    for (int m0 = slot * WD_M; m0 < na; m0 += n_slots * WD_M) {
        const int my_a = m0 + srow < na ? a0 + m0 + srow : -1;
        f32x4 acc[4];
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) acc[mb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        for (int tb = t0; tb < t1; tb += WD_TC) {
            if (!(early && tb == t0 && m0 == slot * WD_M)) request_weights(tb);
            // z pieces: 64 rows x 128 columns per tile, 32 columns per thread and tile
            u32x4 zp[WD_TC][4];
#pragma unroll
            for (int q = 0; q < WD_TC; ++q) {
#pragma unroll
                for (int c = 0; c < 4; ++c) zp[q][c] = u32x4{0u, 0u, 0u, 0u};
                if (my_a < 0 || tb + q >= t1) continue;
                const int64_t at = (int64_t)my_a * I + (tb + q) * N_TILE + sc0;
                if constexpr (ZF16) {
                    const u32x4* src = reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(g) + at);
#pragma unroll
                    for (int c = 0; c < 4; ++c) zp[q][c] = src[c];
                } else {
                    const float* gp = reinterpret_cast<const float*>(g) + at;
                    const float* up = u + at;
#pragma unroll
                    for (int c = 0; c < 4; ++c)
#pragma unroll
                        for (int hv = 0; hv < 2; ++hv) {      // four columns at a time
                            f32x4 gv = *reinterpret_cast<const f32x4*>(gp + c * 8 + hv * 4);
                            f32x4 uv = *reinterpret_cast<const f32x4*>(up + c * 8 + hv * 4);
                            for (int p = 1; p < n_part; ++p) {
                                gv += *reinterpret_cast<const f32x4*>(gp + p * part_stride + c * 8 + hv * 4);
                                uv += *reinterpret_cast<const f32x4*>(up + p * part_stride + c * 8 + hv * 4);
                            }
                            zp[q][c][2 * hv] = (uint32_t)z_operand(gv[0], uv[0]) |
                                               ((uint32_t)z_operand(gv[1], uv[1]) << 16);
                            zp[q][c][2 * hv + 1] = (uint32_t)z_operand(gv[2], uv[2]) |
                                                   ((uint32_t)z_operand(gv[3], uv[3]) << 16);
                        }
                }
            }
            __syncthreads();      // (the previous pieces' operand reads are done)
#pragma unroll
            for (int q = 0; q < WD_TC; ++q)
#pragma unroll
                for (int c = 0; c < 4; ++c) *reinterpret_cast<u32x4*>(&sZ[srow * WD_Z_LD + q * N_TILE + sc0 + c * 8]) = zp[q][c];
            __syncthreads();
#pragma unroll
            for (int q = 0; q < WD_TC; ++q) {
                if (tb + q >= t1) break;
#pragma unroll
                for (int mb = 0; mb < 4; ++mb) {
                    if (m0 + mb * 16 >= na) break;
#pragma unroll
                    for (int ks = 0; ks < 4; ++ks) {
                        const u32x4 a = *reinterpret_cast<const u32x4*>(
                            &sZ[(mb * 16 + (lane & 15)) * WD_Z_LD + q * N_TILE + ks * 32 + (lane >> 4) * 8]);
                        acc[mb] = mfma16<false>(a, b[q][ks], acc[mb]);
                    }
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
                int tk;
                float w;
                if constexpr (ROUTED) {
                    tk = route_lds.tok[row];
                    w = ra.weights[route_lds.ent[row]];
                } else {
                    tk = tok[a0 + row];
                    w = route_w[a0 + row];
                }
                atomicAdd(&rank_accum[(int64_t)tk * rank_out + rk], acc[mb][j] * sv * w);
            }
    }
}

__global__ __launch_bounds__(256) void k_wide_clear2(float* __restrict__ p1, float* __restrict__ p2, int64_t n4) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
        reinterpret_cast<f32x4*>(p1)[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        reinterpret_cast<f32x4*>(p2)[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
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
// the wide slabs every expert of the set has, if all have the same number and all have some; else 0
static int uniform_wide_slabs(const bitsmoe_matset* set) {
    if (!has_wide_rows(set) || set->n_wide_experts != set->n_experts) return 0;
    const int n = set->wide_first_host[1] - set->wide_first_host[0];
    for (int e = 1; e < set->n_experts; ++e)
        if (set->wide_first_host[e + 1] - set->wide_first_host[e] != n) return 0;
    return n;
}
static int max_wide_slabs(const bitsmoe_matset* set) {
    int m = 0;
    for (int e = 0; e < set->n_experts && has_wide_rows(set); ++e)
        m = std::max(m, set->wide_first_host[e + 1] - set->wide_first_host[e]);
    return m;
}
// activations of a slab quarter as two 16-byte loads: rank' is the identity, wide rows only, aligned rows
static bool ident_wide(const bitsmoe_matset* set, const void* h, int64_t ld) {
    if (!has_wide_rows(set) || set->narrow_rows != 0 || ((uintptr_t)h & 15) != 0 || ld % 8 != 0) return false;
    for (int e = 0; e < set->n_experts; ++e) {
        const auto& rk = set->rank_idx_host[e];
        for (size_t k = 0; k < rk.size(); ++k)
            if (rk[k] != (int32_t)k) return false;
    }
    return true;
}

static int wide_gateup_impl(const bitsmoe_matset* gate, const bitsmoe_matset* up, const void* h_gate, const void* h_up,
                            int act_dtype, int Rg, int Ru, int64_t ldg, int64_t ldu, const int32_t* tok, const int32_t* off,
                            const WideRouted* routed, int64_t A, int I, void* G, void* U, bool sums_f16, float* clear,
                            int64_t n_clear, hipStream_t st) {
    const int n_tiles = gate->n_tiles;
    const int n_exp = std::max(gate->n_wide_experts, up->n_wide_experts);
    const int max_slabs = std::max(max_wide_slabs(gate), max_wide_slabs(up));
    const int ug = uniform_wide_slabs(gate), uu = uniform_wide_slabs(up);
    const int uniform = (ug > 0 && ug == uu) ? ug : 0;
    // f16 sums: one workgroup per element (all slabs in one chunk).  fp32 sums: as many chunks of slabs as it
    // takes for a thousand workgroups, whole steps of WD_CH slabs (fewer atomics when the batch is large).
    const int64_t blocks = std::max<int64_t>((A / std::max(n_exp, 1) + WD_M - 1) / WD_M, 1);
    int chunk = max_slabs;
    if (!sums_f16) {
        const int64_t want = std::max<int64_t>(1024 / ((int64_t)n_exp * n_tiles * 2 * blocks), 1);
        chunk = (int)std::max<int64_t>((max_slabs + want - 1) / want, 1);
        chunk = (chunk + WD_CH - 1) / WD_CH * WD_CH;
    }
    const int n_chunks = (max_slabs + chunk - 1) / chunk;
    const int n_slots = routed ? 1 : row_slots(A, (int64_t)n_exp * n_tiles * n_chunks * 2);
    const dim3 grid((unsigned)((int64_t)n_exp * n_tiles * n_chunks * n_slots), 2);
    const WideRouted ra = routed ? *routed : WideRouted{};
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, st, wide_set_of(gate), wide_set_of(up), (const uint16_t*)h_gate,
                           (const uint16_t*)h_up, Rg, Ru, ldg, ldu, tok, off, ra, I, n_tiles, chunk, n_chunks, n_slots, uniform, G, U,
                           clear, n_clear);
    };
    const bool bf16 = act_dtype == BITSMOE_DT_BF16;
    const bool ident = ident_wide(gate, h_gate, ldg) && ident_wide(up, h_up, ldu);
    auto with_flags = [&](auto bf16_c, auto ident_c) {
        constexpr bool B = decltype(bf16_c)::value;
        constexpr bool D = decltype(ident_c)::value;
        if (sums_f16)
            launch(k_wide_gateup<B, true, false, D>);
        else if (routed)
            launch(k_wide_gateup<B, false, true, D>);
        else
            launch(k_wide_gateup<B, false, false, D>);
    };
    if (bf16) {
        if (ident)
            with_flags(std::true_type{}, std::true_type{});
        else
            with_flags(std::true_type{}, std::false_type{});
    } else {
        if (ident)
            with_flags(std::false_type{}, std::true_type{});
        else
            with_flags(std::false_type{}, std::false_type{});
    }
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}

static int wide_down_impl(const bitsmoe_matset* down, const void* g_or_z, const float* u, bool z_f16, int n_part,
                          int64_t part_stride, const int32_t* tok, const int32_t* off, const float* rw, const WideRouted* routed,
                          int64_t A, int I, int rank_out, float* rank_accum, hipStream_t st) {
    const int max_slabs = max_wide_slabs(down);
    const int n_tiles = down->n_tiles;
    const int uniform = uniform_wide_slabs(down);
    // chunks of column tiles: as many as it takes for a thousand workgroups, whole steps of WD_TC tiles
    const int64_t blocks = std::max<int64_t>((A / std::max(down->n_wide_experts, 1) + WD_M - 1) / WD_M, 1);
    const int64_t want = std::max<int64_t>(1024 / ((int64_t)down->n_wide_experts * max_slabs * blocks), 1);
    int tiles_per_wg = (int)std::max<int64_t>((n_tiles + want - 1) / want, 1);
    tiles_per_wg = (tiles_per_wg + WD_TC - 1) / WD_TC * WD_TC;
    const int n_tchunks = (n_tiles + tiles_per_wg - 1) / tiles_per_wg;
    const int n_slots = routed ? 1 : row_slots(A, (int64_t)down->n_wide_experts * max_slabs * n_tchunks);
    const dim3 grid((unsigned)((int64_t)down->n_wide_experts * max_slabs * n_tchunks * n_slots));
    const WideRouted ra = routed ? *routed : WideRouted{};
    auto launch = [&](auto kernel, int parts, int64_t stride) {
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, st, wide_set_of(down), max_slabs, g_or_z, u, parts, stride, tok, off, rw, ra,
                           I, n_tiles, tiles_per_wg, n_tchunks, n_slots, uniform, rank_out, rank_accum);
    };
    if (z_f16)
        launch(k_wide_down<true, false>, 1, (int64_t)0);
    else if (routed)
        launch(k_wide_down<false, true>, n_part, part_stride);
    else
        launch(k_wide_down<false, false>, n_part, part_stride);
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}

int launch_wide_gateup(const bitsmoe_matset* gate, const bitsmoe_matset* up, const void* h_gate, const void* h_up,
                       int act_dtype, int Rg, int Ru, int64_t ldg, int64_t ldu, const int32_t* tok, const int32_t* off,
                       int64_t A, int I, void* G, void* U, bool sums_f16, hipStream_t st) {
    if ((!has_wide_rows(gate) && !has_wide_rows(up)) || A <= 0) return BITSMOE_OK;
    BITSMOE_REQUIRE(tok && off, "the wide rows of these matrix sets need the routing tables");
    return wide_gateup_impl(gate, up, h_gate, h_up, act_dtype, Rg, Ru, ldg, ldu, tok, off, nullptr, A, I, G, U, sums_f16, nullptr,
                            0, st);
}

int launch_wide_down(const bitsmoe_matset* down, const void* g_or_z, const float* u, bool z_f16, int n_part,
                     int64_t part_stride, const int32_t* tok, const int32_t* off, const float* rw, int64_t A, int I,
                     int rank_out, float* rank_accum, hipStream_t st) {
    if (!has_wide_rows(down) || A <= 0) return BITSMOE_OK;
    BITSMOE_REQUIRE(tok && off && rw, "the wide rows of this matrix set need the routing tables");
    return wide_down_impl(down, g_or_z, u, z_f16, n_part, part_stride, tok, off, rw, nullptr, A, I, rank_out, rank_accum, st);
}

bool wide_routed_possible(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down, int64_t T, int top_k) {
    const int64_t n_flat = T * top_k;
    const int u = uniform_wide_slabs(gate);
    return options().route_inline != 0 && only_wide_rows(gate, up, down) && n_flat > 0 && n_flat <= ROUTE_INLINE_MAX_FLAT &&
           T <= ROUTE_INLINE_MAX_ROWS && u > 0 && u == uniform_wide_slabs(up) && uniform_wide_slabs(down) > 0 &&
           (int64_t)gate->n_experts * T <= n_flat;      // (the intermediates are sized for n_flat rows)
}

int launch_forward_wide_routed(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                               const void* h_gate, const void* h_up, int act_dtype, int64_t T, int Rg, int Ru, int64_t ldg,
                               int64_t ldu, const DecodeRouted* routed, int64_t n_flat, int rank_out, int I, float* rank_accum,
                               float* G, float* U, int64_t inter_floats, bitsmoe_profile* prof, hipStream_t st) {
    const WideRouted ra{routed->selected, routed->ids_are_i64, (int)n_flat, routed->top_k, routed->local_to_global, routed->weights,
                        (int)T};
    if (prof) (void)hipEventRecord(prof->ev[0], st);
    // the sums are added to by atomics: their rows in use (rows_per_expert per expert) are cleared first; the
    // gate/up kernel clears the output on its way
    (void)inter_floats;
    const int64_t n4 = (int64_t)gate->n_experts * T * I / 4;      // (I is a multiple of 128)
    hipLaunchKernelGGL(k_wide_clear2, dim3((unsigned)std::min<int64_t>((n4 + 255) / 256, 1024)), dim3(256), 0, st, G, U, n4);
    BITSMOE_HIP_TRY(hipGetLastError());
    if (prof) (void)hipEventRecord(prof->ev[1], st);
    int rc = wide_gateup_impl(gate, up, h_gate, h_up, act_dtype, Rg, Ru, ldg, ldu, nullptr, nullptr, &ra, n_flat, I, G, U, false,
                              rank_accum, T * (int64_t)rank_out, st);
    if (rc != BITSMOE_OK) return rc;
    if (prof) (void)hipEventRecord(prof->ev[2], st);
    if (prof) (void)hipEventRecord(prof->ev[3], st);
    rc = wide_down_impl(down, G, U, false, 1, 0, nullptr, nullptr, nullptr, &ra, n_flat, I, rank_out, rank_accum, st);
    if (rc != BITSMOE_OK) return rc;
    if (prof) {
        (void)hipEventRecord(prof->ev[4], st);
        (void)hipEventRecord(prof->ev[5], st);
        prof->recorded = true;
    }
    return BITSMOE_OK;
}

}  // namespace bitsmoe
