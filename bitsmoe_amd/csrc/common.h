// Shared declarations of libbitsmoe_hip: device views of packed expert matrices, the
// bit-plane decode rule, error plumbing.  gfx950 only (wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include "../../include/bitsmoe_hip.h"

namespace bitsmoe {

constexpr int K_SLAB = 64;    // rows per slab (at most)
constexpr int K_STAGE = 16;   // rows per stage inside a slab
constexpr int N_TILE = 128;   // columns per tile
constexpr int N_MICRO = 32;   // columns per plane word
constexpr int MICROS = N_TILE / N_MICRO;

// One packed expert matrix as the kernels see it.
struct MatView {
    const uint32_t* payload;
    const int32_t* rank_idx;
    const int32_t* tile_meta;  // [num_tiles][3] = pack_off, scale_off, n_valid
    const int32_t* slab_meta;  // [num_slabs][4] = bits, k_slab, rank_off, tile_off
    const __half* scale;
    const __half* s;
    int32_t num_slabs;
    int32_t num_tiles;
    int32_t rank_len;
    int32_t flags;             // bit0: regular layout
};

// Flattened tables of a prepared ("regular") matrix set: everything a fast kernel needs
// to find a (slab, tile) block is addressable from the expert index alone, so the loads
// of one workgroup's metadata do not depend on each other.
struct FastExpert {
    const uint32_t* payload;   // prepared (wave-native) payload of this expert
    const __half* scale;
    const __half* s;
    const int32_t* rank_idx;
    int32_t num_slabs;
    int32_t uniform_bits;      // the bit-width every slab of this expert shares, or 0
    const __half* scale_s;     // gate/up sets: scale[tile][row] * s[row], same offsets as `scale`
    int32_t pad[4];            // 64 bytes
};
struct FastSlab {              // tile t of the slab: payload word pack_off + t*256*bits, scale scale_off + t*64
    int32_t bits;              // 0 = no such slab
    int32_t pack_off;
    int32_t scale_off;
    int32_t rank_off;
};

// Kernel argument (by value): the expert a grid coordinate stands for.
constexpr int EXPERT_ORDER_MAX = 512;
struct ExpertOrder {      // (two 16-bit entries per word: a wave-uniform index then reads it with ONE scalar load of the
    uint32_t w[EXPERT_ORDER_MAX / 2];      // kernel-argument segment; a 16-bit array element costs a vector load and its wait)
    __host__ __device__ __forceinline__ int at(int i) const { return (int)((w[i >> 1] >> ((i & 1) * 16)) & 0xFFFFu); }
    __host__ inline void set(int i, uint16_t v) {
        const int sh = (i & 1) * 16;
        w[i >> 1] = (w[i >> 1] & ~(0xFFFFu << sh)) | ((uint32_t)v << sh);
    }
};

struct SlabTask {              // one (expert, slab) unit of the down projection
    int32_t expert;
    int32_t slab;
};

bool decode_path_supported(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down, int I);
// The routed ids and weights of a forward whose kernels find their assignments themselves (no routing tables).
struct DecodeRouted {
    const void* selected;             // [T, top_k] expert ids as the router numbers them
    int ids_are_i64;
    const float* weights;             // [T, top_k]
    int top_k;
    const int32_t* local_to_global;   // [n_experts]: the router's id of every expert of the matrix sets
    const int32_t* global_to_local;   // [n_global]: its inverse, -1 for ids that belong to no expert of the sets
    int n_global;
};
bool decode_inline_route_ok(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down, const void* h_gate,
                            const void* h_up, int Rg, int Ru, int64_t ldg, int64_t ldu, int64_t T, int top_k, int I);
int launch_forward_decode(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                          const void* h_gate, const void* h_up, int act_dtype, int64_t T, int Rg, int Ru, int64_t ldg,
                          int64_t ldu, const int32_t* tok, const int32_t* off, const float* rw, int64_t A, int rank_out,
                          int I, float* rank_accum, float* G, float* U, int64_t inter_floats, int part_capacity,
                          const DecodeRouted* routed, bitsmoe_profile* prof, hipStream_t st);
// The one-kernel decode forward (forward_fused.hip): can it run these sets and activations, and does the
// launcher choose it for this batch?  launch_forward_decode_fused runs it (rank_accum cleared by a small launch
// of its own first, then ONE kernel from the activations to the atomics of the combine).
bool decode_fused_possible(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                           const void* h_gate, const void* h_up, int Rg, int Ru, int64_t ldg, int64_t ldu, int I);
bool decode_fused_chosen(const bitsmoe_matset* gate, int64_t A, int I);
int launch_forward_decode_fused(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                                const void* h_gate, const void* h_up, int act_dtype, int64_t T, int Rg, int Ru, int64_t ldg,
                                int64_t ldu, const int32_t* tok, const int32_t* off, const float* rw, int64_t A, int rank_out,
                                int I, float* rank_accum, const DecodeRouted* routed, bitsmoe_profile* prof, hipStream_t st);

// The side kernels for the wide rows of prepared sets (forward_wide.hip).  Gate/up: adds the wide rows' share to the
// gate and up sums the fast kernel has written -- fp32 sums [A, I] by atomics (part 0 of the decode path's partial
// results), or f16 sums (the grouped-GEMM path) by a plain read-add-write.  Down: reads z = silu(G) * U as f16
// [A, I] (z_f16) or forms it from `n_part` fp32 partial sums, and adds the wide rows' outputs, scaled by the
// routing weight, into rank_accum by atomics: after whatever writes or clears rank_accum.  Both need the routing
// tables.  No-ops for sets without wide rows.
bool has_wide_rows(const bitsmoe_matset* set);
// every row of the three sets is wide (dense experts): the side kernels are the whole forward
bool only_wide_rows(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down);
int launch_wide_gateup(const bitsmoe_matset* gate, const bitsmoe_matset* up, const void* h_gate, const void* h_up,
                       int act_dtype, int Rg, int Ru, int64_t ldg, int64_t ldu, const int32_t* tok, const int32_t* off,
                       int64_t A, int I, void* G, void* U, bool sums_f16, hipStream_t st);
int launch_wide_down(const bitsmoe_matset* down, const void* g_or_z, const float* u, bool z_f16, int n_part,
                     int64_t part_stride, const int32_t* tok, const int32_t* off, const float* rw, int64_t A, int I,
                     int rank_out, float* rank_accum, hipStream_t st);

// Sets of dense experts only, a small batch, from the router's output: the side kernels find their assignments among the
// routed ids themselves (no routing tables); launch_forward_wide_routed clears the sums, then two kernels.
bool wide_routed_possible(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down, int64_t T, int top_k);
int launch_forward_wide_routed(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                               const void* h_gate, const void* h_up, int act_dtype, int64_t T, int Rg, int Ru, int64_t ldg,
                               int64_t ldu, const DecodeRouted* routed, int64_t n_flat, int rank_out, int I, float* rank_accum,
                               float* G, float* U, int64_t inter_floats, bitsmoe_profile* prof, hipStream_t st);

// How many partial results of the two fp32 intermediates the decode path's workspace holds (the gate/up kernel
// may split its contraction over workgroups when there are few assignments).
inline int decode_part_capacity(int64_t n_assign) { return n_assign <= 1024 ? 4 : n_assign <= 4096 ? 2 : 1; }

bool mfma_path_supported(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down, int I);
size_t mfma_workspace_bytes(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down, int64_t T,
                            int64_t A, int I);
// Work of the grouped-GEMM path's front end that the routing launches can carry, so that a forward from the
// router's output needs fewer launches: the f16 copy of bf16 activations rides in extra workgroups of the
// counting launch, the scan also builds the tile list (it has the expert offsets at hand) and the scatter also
// writes every assignment's slot within its token and the per-token counts.  The per-token lists then have a
// fixed stride: token t's list starts at t * top_k (token_start), its length is token_count[t].
struct MTile;
struct RouteSideJobs {
    const uint16_t* src_g = nullptr;     // bf16 activations (rows sg / su elements apart); null: no copy
    const uint16_t* src_u = nullptr;
    int64_t T = 0, sg = 0, su = 0;
    int ldg = 0, ldu = 0;                // columns of the copies (multiples of 8)
    uint16_t* dst_g = nullptr;
    uint16_t* dst_u = nullptr;
    int32_t* slot = nullptr;             // [n_flat], by position in the routing tables; null: not wanted
    int32_t* token_count = nullptr;      // [T]
    int32_t* token_start = nullptr;      // [T + 1]
    MTile* mtiles = nullptr;             // [max_mtiles]; null: not wanted
    int32_t* n_mtiles = nullptr;
    int max_mtiles = 0;
    const FastExpert* gate_fe = nullptr;
    const FastExpert* up_fe = nullptr;
};
constexpr int MFMA_FRONT_CONVERTED = 1;        // the f16 copies are made
constexpr int MFMA_FRONT_TOKEN_COUNTED = 2;    // slot, token_count and token_start (stride top_k) are written
constexpr int MFMA_FRONT_MTILES = 4;           // the tile list is built
// Fills `jobs` for a call of launch_forward_mfma with the same arguments; false: that call needs none of them.
bool mfma_front_jobs(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                     const void* h_gate, const void* h_up, int act_dtype, int64_t T, int Rg, int Ru, int64_t ldg_in,
                     int64_t ldu_in, int64_t A, int I, void* workspace, RouteSideJobs* jobs);
// bitsmoe_route with side jobs; *jobs_done: which of them the launches carried (MFMA_FRONT_* bits).
int route_with_jobs(const void* selected, int32_t ids_are_i64, const float* weights, const int32_t* global_to_local,
                    int32_t n_global, int64_t n_tokens, int32_t top_k, int32_t n_packed, int32_t* token_indices,
                    int32_t* expert_offsets, float* route_flat, void* workspace, size_t workspace_bytes,
                    const RouteSideJobs* jobs, int* jobs_done, hipStream_t st);
// front_done: MFMA_FRONT_* bits of what an earlier launch on the stream has already produced in `workspace`.
int launch_forward_mfma(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                        const void* h_gate, const void* h_up, int act_dtype, int64_t T, int Rg, int Ru, int64_t ldg_in,
                        int64_t ldu_in, const int32_t* tok, const int32_t* off, const float* rw, int64_t A, int rank_out,
                        int I, float* rank_accum, void* workspace, int front_done, bitsmoe_profile* prof, hipStream_t st);

// bf16 -> f16, eight elements at a time: group `i` of `total = T * (ld / 8)` groups of one projection.
__device__ inline void convert_bf16_group(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst, int64_t stride,
                                          int ld, int64_t i) {
    typedef uint32_t v4 __attribute__((ext_vector_type(4)));
    const int per_row = ld >> 3;
    const int64_t row = i / per_row;
    const int c = (int)(i - row * per_row) * 8;
    const v4 v = *reinterpret_cast<const v4*>(src + row * stride + c);
    v4 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t lo = __builtin_bit_cast(uint16_t, (_Float16)__uint_as_float(v[k] << 16));
        const uint32_t hi = __builtin_bit_cast(uint16_t, (_Float16)__uint_as_float(v[k] & 0xFFFF0000u));
        o[k] = lo | (hi << 16);
    }
    *reinterpret_cast<v4*>(dst + row * ld + c) = o;
}

}  // namespace bitsmoe

// The opaque handle of the C ABI.
struct bitsmoe_matset {
    int32_t n_experts = 0;
    int32_t intermediate_size = 0;
    int32_t n_tiles = 0;              // ceil(I / 128)
    int32_t max_slabs = 0;            // largest num_slabs over experts
    int64_t total_slabs = 0;
    int32_t max_rank_plus1 = 0;       // 1 + largest logical rank referenced by rank_idx
    int32_t min_rank = 0;             // smallest logical rank
    bool regular = false;             // every matrix: 2/3/4-bit, k_slab % 16 == 0, full tiles
    bool regular64 = false;           // ... and every slab has exactly 64 rows, payload 16-byte aligned
    bool fast_ok = false;             // every slab spans all column tiles: bitsmoe_matset_prepare can take the set
    int role = -1;                    // -1: not prepared; 0: gate/up layout; 1: down layout
    bool rank_chunked8 = false;       // slab i holds local rows 64*i.., and every aligned run of 8 local rows
                                      // maps to 8 consecutive logical ranks starting at a multiple of 8
    bool rank_identity = false;       // rank_idx[k] == k in every expert
    __half* d_scale_s = nullptr;      // gate/up sets: scale folded with the per-row multiplier s
    bool vector_aligned = false;      // scale / s / rank_idx of every expert start on 16-byte boundaries
    bool all_uniform8 = false;        // role 0: every aligned group of 8 slabs has one width and is contiguous
    bool all_affine = false;          // role 0: every expert has max_slabs slabs of ONE width whose payload, scale and
                                      // rank offsets advance by a whole slab from one slab to the next
    // experts by decreasing payload size (prepared sets of at most EXPERT_ORDER_MAX experts): the
    // decode kernels start the expensive experts' workgroups first
    std::vector<uint8_t> expert_bits;   // prepared sets: the bit-width all slabs of an expert share, or 0
    bool uniform_experts = false;       // prepared sets: no expert mixes widths
    bool has_cost_order = false;
    uint16_t cost_order[512] = {};
    uint32_t* d_prepared = nullptr;   // wave-native copy of every payload (see wave_layout.h), every slab padded to 64 rows
    void* d_prepared_rows = nullptr;  // the prepared copy's row tables: rank_idx', source of each row, s', scale'
    bitsmoe::SlabTask* d_prep_tasks = nullptr;       // (expert, slab) of every slab of the prepared copy
    int32_t prep_max_slabs = 0;       // largest slab count of the prepared copy (row stride of d_fast_slabs)
    int32_t pad_rank_plus1 = 0;       // 1 + largest rank the prepared rank table holds, padding rows included
    std::vector<int64_t> prep_row_offsets;
    const int32_t* d_row_src = nullptr;   // (inside d_prepared_rows)
    std::vector<bitsmoe::FastExpert> fast_experts_host;
    std::vector<std::vector<int32_t>> rank_idx_host;
    bitsmoe::FastExpert* d_fast_experts = nullptr;   // [n_experts]
    bitsmoe::FastSlab* d_fast_slabs = nullptr;       // [n_experts][max_slabs]
    // Rows of 6-, 8- and 16-bit slabs ("wide" rows) are no part of the prepared copy above: they sit in a side
    // table of 64-row slabs of f16 weights (level * scale, or the stored half), laid out as the 16x16x32 MFMA's
    // second operand, and the side kernels of forward_wide.hip add their share to what the fast kernels compute.
    int64_t wide_slabs = 0;               // all experts
    int64_t narrow_rows = 0;              // rows of 1/2/3/4-bit slabs, all experts (0: dense experts, wide rows only)
    std::vector<int32_t> wide_first_host; // [n_experts + 1]: expert e owns wide slabs [wide_first[e], wide_first[e + 1])
    int32_t n_wide_experts = 0;           // experts with at least one wide slab
    int32_t* d_wide_tables = nullptr;     // one allocation: wide_first, wide_experts, rank' and source of every row, s'
    const int32_t* d_wide_first = nullptr;
    const int32_t* d_wide_experts = nullptr;
    const int32_t* d_wide_rank = nullptr; // [wide_slabs * 64], -1 for padding rows
    const int32_t* d_wide_src = nullptr;  // (source slab << 8) | row inside it, -1 for padding rows
    const __half* d_wide_s = nullptr;
    __half* d_wide = nullptr;             // [wide_slabs][n_tiles][8192]
    int device = -1;
    std::vector<bitsmoe_matrix_desc> descs;
    std::vector<std::vector<int32_t>> slab_meta_host;
    std::vector<std::vector<int32_t>> tile_meta_host;
    bitsmoe::MatView* d_views = nullptr;      // [n_experts]
    bitsmoe::SlabTask* d_slab_tasks = nullptr;  // [total_slabs]
};

struct bitsmoe_profile {
    hipEvent_t ev[BITSMOE_PROFILE_PHASES + 1];
    bool recorded = false;
};

namespace bitsmoe {

void set_error(const char* fmt, ...);
int hip_fail(hipError_t e, const char* what);

// Experiment switches of the launchers (-1: the library's own choice).  Read from the environment ONCE, when
// the library is loaded (BITSMOE_ROUTE_INLINE, BITSMOE_ROUTE_JOBS, BITSMOE_DECODE_FUSED_Z, BITSMOE_DECODE_SPLIT_Z,
// BITSMOE_DECODE_FUSED, BITSMOE_PREFILL_SPLIT); afterwards only bitsmoe_set_option changes them.  No launch path reads the environment.
struct Options {
    int route_inline = -1;      // 0: routing kernel first even where the decode kernels could route themselves
    int route_jobs = -1;        // 0: the grouped-GEMM front end by launches of its own
    int decode_fused_z = -1;    // 1: the decode gate/up kernel forms z itself
    int decode_split_z = -1;    // 0 / 1: z by the down workgroups / by a launch of its own wherever possible
    int decode_fused = -1;      // 0 / 1: never / wherever possible the one-kernel decode forward
    int prefill_split = -1;     // 1: gate and up as two launches, SiLU in the second's epilogue (default: one launch and a SiLU pass)
    int router_wide = -1;       // 0: the fused router kernel with four wavefronts per workgroup whatever the hidden size
};
Options& options();

// The current device's copy of the static scratch array (device address), resolved on first use per device;
// nullptr with the error set.  Called when a matrix set is created, so that the forward never has to.
void* static_scratch_of_current_device();

#define BITSMOE_HIP_TRY(expr)                                        \
    do {                                                             \
        hipError_t _e = (expr);                                      \
        if (_e != hipSuccess) return ::bitsmoe::hip_fail(_e, #expr); \
    } while (0)

#define BITSMOE_REQUIRE(cond, ...)           \
    do {                                     \
        if (!(cond)) {                       \
            ::bitsmoe::set_error(__VA_ARGS__); \
            return BITSMOE_E_INVALID;        \
        }                                    \
    } while (0)

__host__ __device__ inline int words_per_row(int bits) { return bits == 16 ? 16 : bits; }

__host__ __device__ inline int level_offset(int bits) {
    // stored code u = level + offset; 1-bit stores (level+1)/2
    switch (bits) {
        case 2: return 2;
        case 3: return 4;
        case 4: return 8;
        case 6: return 32;
        case 8: return 128;
        default: return 0;
    }
}

__host__ inline bool bits_supported(int b) {
    return b == 1 || b == 2 || b == 3 || b == 4 || b == 6 || b == 8 || b == 16;
}

// Decode one element from the words of one (row, micro-tile): `w` points at the first
// plane word of that row; returns the level (low-bit) or the stored half (16-bit) as fp32,
// without the scale.
__device__ inline float decode_from_row_words(const uint32_t* w, int bits, int lane) {
    if (bits == 16) {
        const uint32_t word = w[lane >> 1];
        const uint16_t hb = (lane & 1) ? (uint16_t)(word >> 16) : (uint16_t)(word & 0xFFFFu);
        return __half2float(__ushort_as_half(hb));
    }
    int u = 0;
    for (int p = 0; p < bits; ++p) u |= (int)((w[p] >> lane) & 1u) << p;
    const int q = (bits == 1) ? (2 * u - 1) : (u - level_offset(bits));
    return (float)q;
}

template <typename T>
__device__ inline float to_f32(T v);
template <>
__device__ inline float to_f32<__half>(__half v) { return __half2float(v); }
template <>
__device__ inline float to_f32<__hip_bfloat16>(__hip_bfloat16 v) { return __bfloat162float(v); }

__device__ inline float silu_f32(float x) { return x / (1.0f + __expf(-x)); }

// launchers implemented in the kernel translation units
int launch_fill_zero(float* p, int64_t n, hipStream_t st);
int launch_forward_generic(const bitsmoe_matset* gate, const bitsmoe_matset* up,
                           const bitsmoe_matset* down, const void* h_gate, const void* h_up,
                           int act_dtype, int64_t T, int Rg, int Ru, int64_t ldg, int64_t ldu, const int32_t* tok,
                           const int32_t* off, const float* rw, int64_t A, int rank_out, int I,
                           float* rank_accum, float* G, float* U, bitsmoe_profile* prof,
                           hipStream_t st);

}  // namespace bitsmoe
