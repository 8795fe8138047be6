// Generic kernels of the routed-expert forward: fp32 FMA, accept every legal layout
// (all seven bit-widths, tail slabs, tail tiles, arbitrary rank_idx).  They are the
// fallback for matrices the fast paths do not take and the first parity target.
#include "common.h"

namespace bitsmoe {

constexpr int AC = 8;  // assignments processed per pass over the weights

// grid.x = E * n_tiles * ksplit, grid.y = 2 (gate, up); 256 threads = 128 columns x 2 row
// parities.  Each workgroup accumulates its slabs' contribution to G (or U) for one
// expert and one 128-column tile and adds it with fp32 atomics (out is zero-filled).
template <typename HT>
__global__ __launch_bounds__(256) void k_gateup_generic(
    const MatView* __restrict__ gate, const MatView* __restrict__ up,
    const HT* __restrict__ h_gate, const HT* __restrict__ h_up, int Rg, int Ru, int64_t ldg, int64_t ldu,
    const int32_t* __restrict__ token_indices, const int32_t* __restrict__ expert_offsets,
    int T, int A, int I, int n_tiles, int ksplit, float* __restrict__ G, float* __restrict__ U) {
    const int mt = blockIdx.y;
    const int bid = blockIdx.x;
    const int ks = bid % ksplit;
    const int tile = (bid / ksplit) % n_tiles;
    const int e = bid / (ksplit * n_tiles);
    const int a_begin = max(expert_offsets[e], 0);
    const int a_end = min(expert_offsets[e + 1], A);
    if (a_end <= a_begin) return;

    const MatView mv = (mt ? up : gate)[e];
    const HT* __restrict__ h = mt ? h_up : h_gate;
    const int R = mt ? Ru : Rg;
    const int64_t ld = mt ? ldu : ldg;      // elements from one activation row to the next
    float* __restrict__ out = mt ? U : G;

    __shared__ uint32_t pk[K_STAGE * MICROS * 16];
    __shared__ float hs[AC][K_STAGE];
    __shared__ float sc[K_STAGE];
    __shared__ float red[AC][N_TILE];

    const int tid = threadIdx.x;
    const int col = tid & (N_TILE - 1);
    const int par = tid >> 7;
    const int micro = col >> 5;
    const int lane = col & 31;
    const int c = tile * N_TILE + col;

    for (int a0 = a_begin; a0 < a_end; a0 += AC) {
        const int na = min(AC, a_end - a0);
        float acc[AC];
#pragma unroll
        for (int a = 0; a < AC; ++a) acc[a] = 0.0f;

        for (int si = ks; si < mv.num_slabs; si += ksplit) {
            const int bits = mv.slab_meta[si * 4 + 0];
            const int k_slab = mv.slab_meta[si * 4 + 1];
            const int rank_off = mv.slab_meta[si * 4 + 2];
            const int tile_off = mv.slab_meta[si * 4 + 3];
            const int tile_end = (si + 1 < mv.num_slabs) ? mv.slab_meta[(si + 1) * 4 + 3] : mv.num_tiles;
            const int t = tile_off + tile;
            if (t >= tile_end) continue;
            const int pack_off = mv.tile_meta[t * 3 + 0];
            const int scale_off = mv.tile_meta[t * 3 + 1];
            const int n_valid = mv.tile_meta[t * 3 + 2];
            const int w = words_per_row(bits);
            const bool col_ok = (col < n_valid) && (c < I);

            for (int g0 = 0; g0 < k_slab; g0 += K_STAGE) {
                const int rows = min(K_STAGE, k_slab - g0);
                const int nwords = rows * MICROS * w;
                __syncthreads();
                const uint32_t* src = mv.payload + pack_off + g0 * MICROS * w;
                for (int i = tid; i < nwords; i += 256) pk[i] = src[i];
                if (tid < K_STAGE)
                    sc[tid] = (tid < rows && bits != 16) ? __half2float(mv.scale[scale_off + g0 + tid]) : 1.0f;
                if (tid < AC * K_STAGE) {
                    const int a = tid / K_STAGE, r = tid % K_STAGE;
                    float v = 0.0f;
                    if (a < na && r < rows) {
                        const int tok = token_indices[a0 + a];
                        const int rk = mv.rank_idx[rank_off + g0 + r];
                        if (tok >= 0 && tok < T && rk >= 0 && rk < R)
                            v = to_f32<HT>(h[(int64_t)tok * ld + rk]) * __half2float(mv.s[rank_off + g0 + r]);
                    }
                    hs[a][r] = v;
                }
                __syncthreads();
                if (col_ok) {
                    for (int r = par; r < rows; r += 2) {
                        const float wv = decode_from_row_words(&pk[micro * rows * w + r * w], bits, lane) * sc[r];
#pragma unroll
                        for (int a = 0; a < AC; ++a) acc[a] += hs[a][r] * wv;
                    }
                }
            }
        }
        __syncthreads();
        if (par == 1) {
#pragma unroll
            for (int a = 0; a < AC; ++a) red[a][col] = acc[a];
        }
        __syncthreads();
        if (par == 0 && c < I) {
#pragma unroll
            for (int a = 0; a < AC; ++a) {
                if (a < na) {
                    const float v = acc[a] + red[a][col];
                    if (v != 0.0f) atomicAdd(&out[(int64_t)(a0 + a) * I + c], v);
                }
            }
        }
    }
}

// grid.x = number of (expert, slab) tasks of the down set; 256 threads = 64 rows x 4
// micro-tiles.  z = silu(G) * U is built on the fly per 128-column tile; each thread dots
// its row's 32 columns against z, applies the per-(row, tile) scale, and the row total
// times s * route_w is added to rank_accum with fp32 atomics.
__global__ __launch_bounds__(256) void k_down_generic(
    const MatView* __restrict__ down, const SlabTask* __restrict__ tasks,
    const float* __restrict__ G, const float* __restrict__ U, const float* __restrict__ route_w,
    const int32_t* __restrict__ token_indices, const int32_t* __restrict__ expert_offsets,
    int T, int A, int I, int rank_out, float* __restrict__ rank_accum) {
    const SlabTask task = tasks[blockIdx.x];
    const int e = task.expert;
    const int si = task.slab;
    const int a_begin = max(expert_offsets[e], 0);
    const int a_end = min(expert_offsets[e + 1], A);
    if (a_end <= a_begin) return;
    const MatView mv = down[e];
    const int bits = mv.slab_meta[si * 4 + 0];
    const int k_slab = mv.slab_meta[si * 4 + 1];
    const int rank_off = mv.slab_meta[si * 4 + 2];
    const int tile_off = mv.slab_meta[si * 4 + 3];
    const int tile_end = (si + 1 < mv.num_slabs) ? mv.slab_meta[(si + 1) * 4 + 3] : mv.num_tiles;
    const int w = words_per_row(bits);

    __shared__ uint32_t pk[K_SLAB * MICROS * 16];
    __shared__ float z[AC][N_TILE];

    const int tid = threadIdx.x;
    const int row = tid >> 2;
    const int micro = tid & 3;
    const bool row_ok = row < k_slab;
    int lr = -1;
    float s_val = 0.0f;
    if (row_ok) {
        lr = mv.rank_idx[rank_off + row];
        s_val = __half2float(mv.s[rank_off + row]);
    }
    const bool row_valid = row_ok && lr >= 0 && lr < rank_out;
    const int stage = row / K_STAGE;
    const int r = row - stage * K_STAGE;
    const int rows_cur = min(K_STAGE, k_slab - stage * K_STAGE);
    const int base = stage * K_STAGE * MICROS * w + micro * rows_cur * w + r * w;

    for (int a0 = a_begin; a0 < a_end; a0 += AC) {
        const int na = min(AC, a_end - a0);
        float racc[AC];
#pragma unroll
        for (int a = 0; a < AC; ++a) racc[a] = 0.0f;
        for (int t = tile_off; t < tile_end; ++t) {
            const int pack_off = mv.tile_meta[t * 3 + 0];
            const int scale_off = mv.tile_meta[t * 3 + 1];
            const int n_valid = mv.tile_meta[t * 3 + 2];
            const int c0 = (t - tile_off) * N_TILE;
            const int nwords = k_slab * MICROS * w;
            __syncthreads();
            for (int i = tid; i < nwords; i += 256) pk[i] = mv.payload[pack_off + i];
            for (int i = tid; i < AC * N_TILE; i += 256) {
                const int a = i / N_TILE, cc = i % N_TILE;
                float v = 0.0f;
                if (a < na && cc < n_valid && c0 + cc < I) {
                    const int64_t idx = (int64_t)(a0 + a) * I + c0 + cc;
                    v = silu_f32(G[idx]) * U[idx];
                }
                z[a][cc] = v;
            }
            __syncthreads();
            if (row_valid) {
                float tacc[AC];
#pragma unroll
                for (int a = 0; a < AC; ++a) tacc[a] = 0.0f;
                for (int l = 0; l < N_MICRO; ++l) {
                    const int cc = micro * N_MICRO + l;
                    if (cc >= n_valid) break;
                    const float wv = decode_from_row_words(&pk[base], bits, l);
#pragma unroll
                    for (int a = 0; a < AC; ++a) tacc[a] += wv * z[a][cc];
                }
                const float scv = (bits == 16) ? 1.0f : __half2float(mv.scale[scale_off + row]);
#pragma unroll
                for (int a = 0; a < AC; ++a) racc[a] += tacc[a] * scv;
            }
        }
#pragma unroll
        for (int a = 0; a < AC; ++a) {
            float v = racc[a];
            v += __shfl_xor(v, 1);
            v += __shfl_xor(v, 2);
            if (micro == 0 && row_valid && a < na) {
                const int tok = token_indices[a0 + a];
                if (tok >= 0 && tok < T && v != 0.0f)
                    atomicAdd(&rank_accum[(int64_t)tok * rank_out + lr], v * s_val * route_w[a0 + a]);
            }
        }
    }
}

static inline void record(bitsmoe_profile* p, int i, hipStream_t st) {
    if (p) (void)hipEventRecord(p->ev[i], st);
}

int launch_forward_generic(const bitsmoe_matset* gate, const bitsmoe_matset* up,
                           const bitsmoe_matset* down, const void* h_gate, const void* h_up,
                           int act_dtype, int64_t T, int Rg, int Ru, int64_t ldg, int64_t ldu, const int32_t* tok,
                           const int32_t* off, const float* rw, int64_t A, int rank_out, int I,
                           float* rank_accum, float* G, float* U, bitsmoe_profile* prof,
                           hipStream_t st) {
    const int E = gate->n_experts;
    const int n_tiles = gate->n_tiles;
    record(prof, 0, st);
    int rc = launch_fill_zero(rank_accum, T * (int64_t)rank_out, st);
    if (rc) return rc;
    rc = launch_fill_zero(G, A * (int64_t)I, st);
    if (rc) return rc;
    rc = launch_fill_zero(U, A * (int64_t)I, st);
    if (rc) return rc;
    record(prof, 1, st);
    // split the slab loop so that a few active experts still fill the chip
    const int max_slabs = gate->max_slabs > up->max_slabs ? gate->max_slabs : up->max_slabs;
    int ksplit = 1;
    if (A <= 1024) {
        ksplit = 8;
        if (ksplit > max_slabs) ksplit = max_slabs > 0 ? max_slabs : 1;
    }
    dim3 grid((unsigned)(E * n_tiles * ksplit), 2);
    if (act_dtype == BITSMOE_DT_F16) {
        hipLaunchKernelGGL(k_gateup_generic<__half>, grid, dim3(256), 0, st, gate->d_views, up->d_views,
                           (const __half*)h_gate, (const __half*)h_up, Rg, Ru, ldg, ldu, tok, off, (int)T, (int)A, I,
                           n_tiles, ksplit, G, U);
    } else {
        hipLaunchKernelGGL(k_gateup_generic<__hip_bfloat16>, grid, dim3(256), 0, st, gate->d_views,
                           up->d_views, (const __hip_bfloat16*)h_gate, (const __hip_bfloat16*)h_up, Rg, Ru,
                           ldg, ldu, tok, off, (int)T, (int)A, I, n_tiles, ksplit, G, U);
    }
    BITSMOE_HIP_TRY(hipGetLastError());
    record(prof, 2, st);
    record(prof, 3, st);
    if (down->total_slabs > 0) {
        hipLaunchKernelGGL(k_down_generic, dim3((unsigned)down->total_slabs), dim3(256), 0, st, down->d_views,
                           down->d_slab_tasks, G, U, rw, tok, off, (int)T, (int)A, I, rank_out, rank_accum);
        BITSMOE_HIP_TRY(hipGetLastError());
    }
    record(prof, 4, st);
    record(prof, 5, st);
    if (prof) prof->recorded = true;
    return BITSMOE_OK;
}

}  // namespace bitsmoe
