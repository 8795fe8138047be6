// Routing / permute: token-to-expert histogram, exclusive scan and STABLE scatter built
// on wave64 ballots.  No host synchronisation; the number of kept assignments stays on
// the device as expert_offsets[n_packed].
#include <algorithm>

#include "common.h"
#include "mtiles.h"

namespace bitsmoe {

constexpr int ROUTE_THREADS = 256;
constexpr int ROUTE_ROUNDS = 4;
constexpr int ROUTE_CHUNK = ROUTE_THREADS * ROUTE_ROUNDS;  // flat entries per workgroup
constexpr int ROUTE_MAX_EXPERTS = 4096;                     // histogram lives in LDS

template <typename IdT>
__device__ inline int load_local_id(const IdT* __restrict__ selected, const int32_t* __restrict__ g2l,
                                    int n_global, int n_packed, int64_t idx, int64_t n_flat) {
    if (idx >= n_flat) return -1;
    const int64_t g = (int64_t)selected[idx];
    if (g < 0 || g >= n_global) return -1;
    const int l = g2l[g];
    return (l >= 0 && l < n_packed) ? l : -1;
}

// Lanes of the wave holding the same non-negative id, found with one ballot per id bit.
__device__ inline uint64_t match_same_id(int id, int id_bits) {
    uint64_t mask = __ballot(id >= 0);
    for (int b = 0; b < id_bits; ++b) {
        const bool bit = (id >> b) & 1;
        const uint64_t bal = __ballot(bit);
        mask &= bit ? bal : ~bal;
    }
    return mask;
}

// Rank of each of this workgroup's entries among the earlier entries of the same expert
// inside the workgroup's chunk (flat order), plus the chunk's histogram in `hist` (LDS).
// Entry order inside a chunk: round-major, then thread id.
template <typename IdT>
__device__ inline void chunk_ranks(const IdT* __restrict__ selected, const int32_t* __restrict__ g2l,
                                   int n_global, int n_packed, int id_bits, int64_t chunk_base,
                                   int64_t n_flat, int* hist, int (&local)[ROUTE_ROUNDS],
                                   int (&rank)[ROUTE_ROUNDS]) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    for (int e = tid; e < n_packed; e += ROUTE_THREADS) hist[e] = 0;
    // all rounds' ids first: their (dependent) loads overlap instead of queueing behind the barriers
#pragma unroll
    for (int j = 0; j < ROUTE_ROUNDS; ++j)
        local[j] = load_local_id<IdT>(selected, g2l, n_global, n_packed, chunk_base + (int64_t)j * ROUTE_THREADS + tid, n_flat);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < ROUTE_ROUNDS; ++j) {
        rank[j] = 0;
        if (chunk_base + (int64_t)j * ROUTE_THREADS >= n_flat) continue;     // (uniform) a round without entries
        const int id = local[j];
        const uint64_t same = match_same_id(id, id_bits);
        const int before = __popcll(same & ((1ull << lane) - 1ull));
        const int count = __popcll(same);
        const bool last = (id >= 0) && (lane == 63 - __clzll((long long)same));
        int old = 0;
        for (int wv = 0; wv < ROUTE_THREADS / 64; ++wv) {
            if (wave == wv && id >= 0) old = hist[id];
            __syncthreads();
            if (wave == wv && last) hist[id] = old + count;
            __syncthreads();
        }
        rank[j] = old + before;
    }
}

// The same result with three barriers instead of two per (round, wavefront): every (round,
// wavefront) pair counts into its own table, then one pass per expert turns the tables into
// "entries of this expert before my (round, wavefront)".  tables: ROUTE_ROUNDS * 4 * n_packed ints.
constexpr int ROUTE_TABLE_MAX_EXPERTS = 512;
constexpr int ROUTE_G2L_LDS_MAX = 4096;      // global expert ids whose map is staged in LDS
template <typename IdT>
__device__ inline void chunk_ranks_tables(const IdT* __restrict__ selected, const int32_t* __restrict__ g2l,
                                          int n_global, int n_packed, int id_bits, int64_t chunk_base,
                                          int64_t n_flat, int* hist, int* tables, int* g2l_lds,
                                          int (&local)[ROUTE_ROUNDS], int (&rank)[ROUTE_ROUNDS]) {
    constexpr int WAVES = ROUTE_THREADS / 64;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int64_t left = n_flat - chunk_base;
    const int rounds = (int)((left < ROUTE_CHUNK ? left : ROUTE_CHUNK) + ROUTE_THREADS - 1) / ROUTE_THREADS;   // uniform
    for (int i = tid; i < rounds * WAVES * n_packed; i += ROUTE_THREADS) tables[i] = 0;
    // the global-to-local map is copied to LDS (g2l_lds != nullptr) while the ids are on their
    // way, so that the look-up is not a second global round trip
    int64_t raw[ROUTE_ROUNDS];
#pragma unroll
    for (int j = 0; j < ROUTE_ROUNDS; ++j) {
        const int64_t idx = chunk_base + (int64_t)j * ROUTE_THREADS + tid;
        raw[j] = idx < n_flat ? (int64_t)selected[idx] : -1;
    }
    if (g2l_lds != nullptr) {
        for (int i = tid; i < n_global; i += ROUTE_THREADS) g2l_lds[i] = g2l[i];
        __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < ROUTE_ROUNDS; ++j) {
        int l = -1;
        if (raw[j] >= 0 && raw[j] < n_global) l = g2l_lds != nullptr ? g2l_lds[raw[j]] : g2l[raw[j]];
        local[j] = (l >= 0 && l < n_packed) ? l : -1;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < ROUTE_ROUNDS; ++j) {
        rank[j] = 0;
        if (j >= rounds) continue;
        const int id = local[j];
        const uint64_t same = match_same_id(id, id_bits);
        rank[j] = __popcll(same & ((1ull << lane) - 1ull));
        if (id >= 0 && lane == 63 - __clzll((long long)same)) tables[(j * WAVES + wave) * n_packed + id] = __popcll(same);
    }
    __syncthreads();
    for (int e = tid; e < n_packed; e += ROUTE_THREADS) {
        int run = 0;
        for (int t = 0; t < rounds * WAVES; ++t) {
            const int c = tables[t * n_packed + e];
            tables[t * n_packed + e] = run;
            run += c;
        }
        hist[e] = run;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < ROUTE_ROUNDS; ++j)
        if (j < rounds && local[j] >= 0) rank[j] += tables[(j * WAVES + wave) * n_packed + local[j]];
}

// Exclusive scan of data[0..n) in LDS by the whole workgroup; returns the total.
__device__ inline int block_exclusive_scan(int* data, int n, int* wave_sums) {
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int per = (n + nthreads - 1) / nthreads;
    const int begin = tid * per;
    int sum = 0;
    for (int i = 0; i < per; ++i)
        if (begin + i < n) sum += data[begin + i];
    int incl = sum;
    for (int d = 1; d < 64; d <<= 1) {
        const int v = __shfl_up(incl, d);
        if (lane >= d) incl += v;
    }
    if (lane == 63) wave_sums[wave] = incl;
    __syncthreads();
    const int nwaves = nthreads >> 6;
    int wave_prefix = 0, total = 0;
    for (int wv = 0; wv < nwaves; ++wv) {
        const int v = wave_sums[wv];
        if (wv < wave) wave_prefix += v;
        total += v;
    }
    int run = wave_prefix + incl - sum;
    for (int i = 0; i < per; ++i) {
        if (begin + i < n) {
            const int v = data[begin + i];
            data[begin + i] = run;
            run += v;
        }
    }
    __syncthreads();
    return total;
}

// Whole routing in one workgroup for n_flat <= ROUTE_CHUNK (decode-size batches).
template <typename IdT>
__global__ __launch_bounds__(ROUTE_THREADS) void k_route_fused(
    const IdT* __restrict__ selected, const float* __restrict__ weights, const int32_t* __restrict__ g2l,
    int n_global, int64_t n_flat, int top_k, int n_packed, int id_bits,
    int32_t* __restrict__ token_indices, int32_t* __restrict__ expert_offsets, float* __restrict__ route_flat) {
    extern __shared__ int lds[];
    int* hist = lds;
    int* wave_sums = lds + n_packed;
    int local[ROUTE_ROUNDS], rank[ROUTE_ROUNDS];
    const int tid = threadIdx.x;
    // the weights are only needed by the scatter: requested first, they arrive while the ranks are built
    float w[ROUTE_ROUNDS];
#pragma unroll
    for (int j = 0; j < ROUTE_ROUNDS; ++j) {
        const int64_t idx = (int64_t)j * ROUTE_THREADS + tid;
        w[j] = idx < n_flat ? weights[idx] : 0.0f;
    }
    if (n_packed <= ROUTE_TABLE_MAX_EXPERTS)
        chunk_ranks_tables<IdT>(selected, g2l, n_global, n_packed, id_bits, 0, n_flat, hist, lds + n_packed + 32,
                                n_global <= ROUTE_G2L_LDS_MAX ? lds + n_packed + 32 + ROUTE_ROUNDS * (ROUTE_THREADS / 64) * n_packed : nullptr,
                                local, rank);
    else
        chunk_ranks<IdT>(selected, g2l, n_global, n_packed, id_bits, 0, n_flat, hist, local, rank);
    const int total = block_exclusive_scan(hist, n_packed, wave_sums);
    for (int e = tid; e < n_packed; e += ROUTE_THREADS) expert_offsets[e] = hist[e];
    if (tid == 0) expert_offsets[n_packed] = total;
#pragma unroll
    for (int j = 0; j < ROUTE_ROUNDS; ++j) {
        if (local[j] >= 0) {
            const int64_t idx = (int64_t)j * ROUTE_THREADS + tid;
            const int pos = hist[local[j]] + rank[j];
            token_indices[pos] = (int32_t)(idx / top_k);
            route_flat[pos] = w[j];
        }
    }
}

// Multi-workgroup version: (1) per-chunk ranks + histograms, (2) scan, (3) scatter.
template <typename IdT>
__global__ __launch_bounds__(ROUTE_THREADS) void k_route_count(
    const IdT* __restrict__ selected, const int32_t* __restrict__ g2l, int n_global, int64_t n_flat,
    int n_packed, int id_bits, int32_t* __restrict__ entry_rank, int32_t* __restrict__ chunk_hist, int n_chunks,
    const RouteSideJobs jobs) {
    extern __shared__ int lds[];
    if ((int)blockIdx.x >= n_chunks) {
        // workgroups past the routing chunks: the f16 copy of the activations, grid-stride over groups of eight
        const int64_t n_g = jobs.T * (jobs.ldg >> 3), n_u = jobs.T * (jobs.ldu >> 3);
        const int64_t step = (int64_t)(gridDim.x - n_chunks) * ROUTE_THREADS;
        for (int64_t i = (int64_t)(blockIdx.x - n_chunks) * ROUTE_THREADS + threadIdx.x; i < n_g + n_u; i += step) {
            if (i < n_g)
                convert_bf16_group(jobs.src_g, jobs.dst_g, jobs.sg, jobs.ldg, i);
            else
                convert_bf16_group(jobs.src_u, jobs.dst_u, jobs.su, jobs.ldu, i - n_g);
        }
        return;
    }
    int* hist = lds;
    int local[ROUTE_ROUNDS], rank[ROUTE_ROUNDS];
    const int64_t chunk_base = (int64_t)blockIdx.x * ROUTE_CHUNK;
    if (n_packed <= ROUTE_TABLE_MAX_EXPERTS)
        chunk_ranks_tables<IdT>(selected, g2l, n_global, n_packed, id_bits, chunk_base, n_flat, hist, lds + n_packed + 32,
                                n_global <= ROUTE_G2L_LDS_MAX ? lds + n_packed + 32 + ROUTE_ROUNDS * (ROUTE_THREADS / 64) * n_packed : nullptr,
                                local, rank);
    else
        chunk_ranks<IdT>(selected, g2l, n_global, n_packed, id_bits, chunk_base, n_flat, hist, local, rank);
    const int tid = threadIdx.x;
#pragma unroll
    for (int j = 0; j < ROUTE_ROUNDS; ++j) {
        const int64_t idx = chunk_base + (int64_t)j * ROUTE_THREADS + tid;
        if (idx < n_flat) entry_rank[idx] = (local[j] >= 0) ? rank[j] : -1;
    }
    for (int e = tid; e < n_packed; e += ROUTE_THREADS) chunk_hist[(int64_t)blockIdx.x * n_packed + e] = hist[e];
}

// One workgroup.  chunk_hist[b][e] (entries of expert e in chunk b) becomes the number of entries of
// e in earlier chunks; expert_offsets the exclusive scan of the per-expert totals.  The chunks of an
// expert are split over `parts` threads (parts * n_packed <= 1024) that first add up their runs.
// With side jobs: the tile list of the grouped-GEMM path from the offsets just made, and token_start[t] = t * top_k.
__global__ __launch_bounds__(1024) void k_route_scan(int32_t* __restrict__ chunk_hist, int n_chunks,
                                                      int n_packed, int32_t* __restrict__ expert_offsets,
                                                      const RouteSideJobs jobs, int n_flat, int top_k) {
    extern __shared__ int lds[];
    __shared__ MTileLds mt_lds;
    int* totals = lds;                       // [n_packed + 1]
    int* wave_sums = lds + n_packed + 1;     // [32]
    int* partial = lds + n_packed + 33;      // [parts][n_packed] when parts > 1
    if (jobs.token_start != nullptr)
        for (int64_t t = threadIdx.x; t <= jobs.T; t += blockDim.x) jobs.token_start[t] = (int32_t)(t * top_k);
    const int tid = threadIdx.x;
    const int parts = n_packed <= 512 ? min(1024 / n_packed, 16) : 1;
    if (parts > 1) {
        const int per = (n_chunks + parts - 1) / parts;
        const int e = tid % n_packed, p = tid / n_packed;
        const bool worker = p < parts;
        const int b0 = min(p * per, n_chunks), b1 = min(b0 + per, n_chunks);
        int sum = 0;
        if (worker) {
            for (int b = b0; b < b1; ++b) sum += chunk_hist[(int64_t)b * n_packed + e];
            partial[p * n_packed + e] = sum;
        }
        __syncthreads();
        if (worker) {
            int run = 0;
            for (int q = 0; q < p; ++q) run += partial[q * n_packed + e];
            if (p == parts - 1) totals[e] = run + sum;
            for (int b = b0; b < b1; ++b) {
                const int64_t i = (int64_t)b * n_packed + e;
                const int c = chunk_hist[i];
                chunk_hist[i] = run;
                run += c;
            }
        }
    } else {
        for (int e = tid; e < n_packed; e += blockDim.x) {
            int run = 0;
            for (int b = 0; b < n_chunks; ++b) {
                const int64_t i = (int64_t)b * n_packed + e;
                const int c = chunk_hist[i];
                chunk_hist[i] = run;  // entries of this expert in earlier chunks
                run += c;
            }
            totals[e] = run;
        }
    }
    __syncthreads();
    const int total = block_exclusive_scan(totals, n_packed, wave_sums);
    for (int e = threadIdx.x; e < n_packed; e += blockDim.x) expert_offsets[e] = totals[e];
    if (threadIdx.x == 0) {
        expert_offsets[n_packed] = total;
        totals[n_packed] = total;
    }
    if (jobs.mtiles != nullptr) {
        __syncthreads();
        build_mtile_list(totals, n_packed, n_flat, jobs.max_mtiles, jobs.mtiles, jobs.n_mtiles, jobs.gate_fe, jobs.up_fe,
                         mt_lds);
    }
}

template <typename IdT>
__global__ __launch_bounds__(ROUTE_THREADS) void k_route_scatter(
    const IdT* __restrict__ selected, const float* __restrict__ weights, const int32_t* __restrict__ g2l,
    int n_global, int64_t n_flat, int top_k, int n_packed, const int32_t* __restrict__ entry_rank,
    const int32_t* __restrict__ chunk_hist, const int32_t* __restrict__ expert_offsets,
    int32_t* __restrict__ token_indices, float* __restrict__ route_flat, int32_t* __restrict__ slot,
    int32_t* __restrict__ token_count) {
    const int64_t idx = (int64_t)blockIdx.x * ROUTE_THREADS + threadIdx.x;
    if (idx >= n_flat) return;
    const int r = entry_rank[idx];
    const int64_t token = idx / top_k;
    int before = 0;      // kept entries of the same token in front of this one (they are neighbours in the flat order)
    if (slot != nullptr) {
        for (int64_t i = token * top_k; i < idx; ++i) before += entry_rank[i] >= 0;
        if (idx == token * top_k + top_k - 1) token_count[token] = before + (r >= 0);
    }
    if (r < 0) return;
    const int id = load_local_id<IdT>(selected, g2l, n_global, n_packed, idx, n_flat);
    const int64_t chunk = idx / ROUTE_CHUNK;
    const int pos = expert_offsets[id] + chunk_hist[chunk * n_packed + id] + r;
    token_indices[pos] = (int32_t)token;
    route_flat[pos] = weights[idx];
    if (slot != nullptr) slot[pos] = before;
}

template <typename IdT>
static int route_impl(const IdT* selected, const float* weights, const int32_t* g2l, int n_global,
                      int64_t n_flat, int top_k, int n_packed, int32_t* token_indices,
                      int32_t* expert_offsets, float* route_flat, void* workspace, const RouteSideJobs* jobs,
                      int* jobs_done, hipStream_t st) {
    if (jobs_done) *jobs_done = 0;
    int id_bits = 0;
    while ((1 << id_bits) < n_packed) ++id_bits;
    const size_t lds_bytes = (size_t)(n_packed + 33) * sizeof(int);
    // histogram + wave sums, and the per-(round, wavefront) tables of the low-barrier variant
    const size_t lds_rank_bytes = lds_bytes + (n_packed <= ROUTE_TABLE_MAX_EXPERTS
                                                   ? ((size_t)ROUTE_ROUNDS * (ROUTE_THREADS / 64) * n_packed +
                                                      (n_global <= ROUTE_G2L_LDS_MAX ? n_global : 0)) * sizeof(int)
                                                   : 0);
    if (n_flat <= ROUTE_CHUNK) {
        hipLaunchKernelGGL(k_route_fused<IdT>, dim3(1), dim3(ROUTE_THREADS), lds_rank_bytes, st, selected, weights,
                           g2l, n_global, n_flat, top_k, n_packed, id_bits, token_indices, expert_offsets,
                           route_flat);
        BITSMOE_HIP_TRY(hipGetLastError());
        return BITSMOE_OK;
    }
    const int64_t n_chunks = (n_flat + ROUTE_CHUNK - 1) / ROUTE_CHUNK;
    int32_t* entry_rank = (int32_t*)workspace;
    int32_t* chunk_hist = entry_rank + ((n_flat + 63) / 64) * 64;
    // side jobs: extra workgroups of the counting launch copy the activations, the scatter writes slots and counts
    RouteSideJobs carried;
    int64_t copy_blocks = 0;
    if (jobs != nullptr) {
        carried = *jobs;
        if (carried.src_g != nullptr) {
            const int64_t groups = carried.T * ((carried.ldg >> 3) + (carried.ldu >> 3));
            copy_blocks = std::min<int64_t>((groups + ROUTE_THREADS * 4 - 1) / (ROUTE_THREADS * 4), 4096);
        }
    }
    hipLaunchKernelGGL(k_route_count<IdT>, dim3((unsigned)(n_chunks + copy_blocks)), dim3(ROUTE_THREADS), lds_rank_bytes, st,
                       selected, g2l, n_global, n_flat, n_packed, id_bits, entry_rank, chunk_hist, (int)n_chunks, carried);
    BITSMOE_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(k_route_scan, dim3(1), dim3(1024), lds_bytes + (n_packed <= 512 ? (size_t)16 * n_packed * sizeof(int) : 0),
                       st, chunk_hist, (int)n_chunks, n_packed, expert_offsets, carried, (int)n_flat, top_k);
    BITSMOE_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(k_route_scatter<IdT>, dim3((unsigned)((n_flat + ROUTE_THREADS - 1) / ROUTE_THREADS)),
                       dim3(ROUTE_THREADS), 0, st, selected, weights, g2l, n_global, n_flat, top_k, n_packed,
                       entry_rank, chunk_hist, expert_offsets, token_indices, route_flat, carried.slot,
                       carried.slot ? carried.token_count : nullptr);
    BITSMOE_HIP_TRY(hipGetLastError());
    if (jobs_done)
        *jobs_done = (copy_blocks > 0 ? MFMA_FRONT_CONVERTED : 0) |
                     (carried.slot && carried.token_start ? MFMA_FRONT_TOKEN_COUNTED : 0) | (carried.mtiles ? MFMA_FRONT_MTILES : 0);
    return BITSMOE_OK;
}

}  // namespace bitsmoe

using namespace bitsmoe;

extern "C" size_t bitsmoe_route_workspace_bytes(int64_t n_flat, int32_t n_packed) {
    if (n_flat <= ROUTE_CHUNK || n_packed <= 0) return 256;
    const int64_t n_chunks = (n_flat + ROUTE_CHUNK - 1) / ROUTE_CHUNK;
    return (size_t)(((n_flat + 63) / 64) * 64 + n_chunks * (int64_t)n_packed) * sizeof(int32_t) + 256;
}

extern "C" int bitsmoe_route(const void* selected, int32_t ids_are_i64, const float* weights,
                             const int32_t* global_to_local, int32_t n_global, int64_t n_tokens,
                             int32_t top_k, int32_t n_packed, int32_t* token_indices,
                             int32_t* expert_offsets, float* route_flat, void* workspace,
                             size_t workspace_bytes, void* stream) {
    return route_with_jobs(selected, ids_are_i64, weights, global_to_local, n_global, n_tokens, top_k, n_packed,
                           token_indices, expert_offsets, route_flat, workspace, workspace_bytes, nullptr, nullptr,
                           (hipStream_t)stream);
}

int bitsmoe::route_with_jobs(const void* selected, int32_t ids_are_i64, const float* weights,
                             const int32_t* global_to_local, int32_t n_global, int64_t n_tokens, int32_t top_k,
                             int32_t n_packed, int32_t* token_indices, int32_t* expert_offsets, float* route_flat,
                             void* workspace, size_t workspace_bytes, const RouteSideJobs* jobs, int* jobs_done,
                             hipStream_t st) {
    if (jobs_done) *jobs_done = 0;
    BITSMOE_REQUIRE(n_tokens >= 0 && top_k > 0, "n_tokens must be >= 0 and top_k > 0");
    BITSMOE_REQUIRE(n_packed >= 0 && n_packed <= ROUTE_MAX_EXPERTS, "n_packed=%d outside [0,%d]", n_packed, ROUTE_MAX_EXPERTS);
    BITSMOE_REQUIRE(n_global >= 0, "n_global must be >= 0");
    BITSMOE_REQUIRE(expert_offsets != nullptr, "expert_offsets must not be null");
    const int64_t n_flat = n_tokens * top_k;
    BITSMOE_REQUIRE(n_flat < ((int64_t)1 << 31), "too many assignments");
    if (n_packed == 0 || n_flat == 0) {
        // all offsets are zero; one tiny fill on the stream keeps the call asynchronous
        return launch_fill_zero((float*)expert_offsets, n_packed + 1, st);
    }
    BITSMOE_REQUIRE(selected && weights && global_to_local && token_indices && route_flat, "null pointer");
    const size_t need = bitsmoe_route_workspace_bytes(n_flat, n_packed);
    if (n_flat > ROUTE_CHUNK && (workspace == nullptr || workspace_bytes < need)) {
        set_error("route workspace too small: need %zu bytes, got %zu", need, workspace_bytes);
        return BITSMOE_E_WORKSPACE;
    }
    if (ids_are_i64)
        return route_impl<int64_t>((const int64_t*)selected, weights, global_to_local, n_global, n_flat, top_k,
                                   n_packed, token_indices, expert_offsets, route_flat, workspace, jobs, jobs_done, st);
    return route_impl<int32_t>((const int32_t*)selected, weights, global_to_local, n_global, n_flat, top_k,
                               n_packed, token_indices, expert_offsets, route_flat, workspace, jobs, jobs_done, st);
}
