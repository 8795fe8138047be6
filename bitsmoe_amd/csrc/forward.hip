// C-ABI entry point of the routed-expert forward: argument checks, workspace carving and
// kernel-path selection.
#include "common.h"
#include "launch_policy.h"

using namespace bitsmoe;

#include <mutex>

// Intermediates of bitsmoe_moe_forward_static: one array per GPU, held until the process ends.
// In host code the array's name is only a stand-in for the symbol; its address on a device comes
// from hipGetSymbolAddress, made once per device with that device current.
static __device__ __align__(256) unsigned char scratch[BITSMOE_STATIC_SCRATCH_BYTES];

static constexpr int MAX_DEVICES = 64;
static void* g_scratch_ptr[MAX_DEVICES] = {};
static std::mutex g_scratch_mutex;

// The current device's copy of `scratch` (device address), or nullptr with the error set.  Every matrix set
// creation calls this, so by the time a forward runs the address of its device is cached.
void* bitsmoe::static_scratch_of_current_device() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        hip_fail(e, "hipGetDevice");
        return nullptr;
    }
    if (dev < 0 || dev >= MAX_DEVICES) {
        set_error("device index %d outside [0, %d)", dev, MAX_DEVICES);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) {
            hip_fail(e, "hipGetSymbolAddress(scratch)");
            return nullptr;
        }
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

extern "C" size_t bitsmoe_forward_workspace_bytes(int64_t n_tokens, int64_t n_assign,
                                                  int32_t intermediate_size, int32_t n_experts,
                                                  int32_t rank_out) {
    (void)n_tokens;
    (void)n_experts;
    (void)rank_out;
    if (n_assign < 0 || intermediate_size < 0) return 0;
    // two fp32 [A, I] intermediates (gate and up outputs), several partial results of them for small batches;
    // the fast kernels keep whole 128-column tiles per row
    const size_t inter = align_up((size_t)n_assign * align_up((size_t)intermediate_size, N_TILE) * sizeof(float), 256);
    return 2 * inter * (size_t)decode_part_capacity(n_assign) + 256;
}

// The path bitsmoe_moe_forward takes for these sets, sizes and `path` request
// (BITSMOE_PATH_*), or a negative error code.
static int resolve_path(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                        int64_t n_assign, int32_t intermediate_size, int32_t path) {
    const bool decode_ok = decode_path_supported(gate, up, down, intermediate_size);
    const bool mfma_ok = mfma_path_supported(gate, up, down, intermediate_size);
    if (path == BITSMOE_PATH_MFMA && !mfma_ok) {
        set_error("MFMA path needs matrix sets prepared with bitsmoe_matset_prepare (gate/up role 0, down role 1)");
        return BITSMOE_E_UNSUPPORTED;
    }
    if (path == BITSMOE_PATH_DECODE && !decode_ok) {
        set_error("decode path needs matrix sets prepared with bitsmoe_matset_prepare (gate/up role 0, down role 1)");
        return BITSMOE_E_UNSUPPORTED;
    }
    if (path != BITSMOE_PATH_AUTO) return path;
    // dense experts (wide rows only): the decode launcher runs the side kernels alone, at any batch size
    if (decode_ok && only_wide_rows(gate, up, down)) return BITSMOE_PATH_DECODE;
    // grouped GEMM from 14 assignments per expert on average (measured crossovers on layers of 64,
    // 128 and 512 experts: 12 to 16; the decode kernels re-stream the payload for every 16
    // assignments, the grouped GEMM pays for a longer launch chain)
    if (mfma_ok && n_assign >= (int64_t)policy::MFMA_MIN_ASSIGN_PER_EXPERT * gate->n_experts) return BITSMOE_PATH_MFMA;
    if (decode_ok) return BITSMOE_PATH_DECODE;
    if (mfma_ok) return BITSMOE_PATH_MFMA;      // (an intermediate size beyond the decode kernels' LDS budget)
    return BITSMOE_PATH_GENERIC;
}

extern "C" size_t bitsmoe_forward_workspace_bytes_sets(const bitsmoe_matset* gate, const bitsmoe_matset* up,
                                                       const bitsmoe_matset* down, int64_t n_tokens,
                                                       int64_t n_assign, int32_t path) {
    if (!gate || !up || !down || n_assign < 0) return 0;
    const int I = gate->intermediate_size;
    const int chosen = resolve_path(gate, up, down, n_assign, I, path);
    if (chosen == BITSMOE_PATH_MFMA) return mfma_workspace_bytes(gate, up, down, n_tokens, n_assign, gate->n_tiles * N_TILE);
    return bitsmoe_forward_workspace_bytes(n_tokens, n_assign, I, gate->n_experts, 0);
}

extern "C" int bitsmoe_moe_forward(const bitsmoe_matset* gate, const bitsmoe_matset* up,
                                   const bitsmoe_matset* down, const void* h_gate, const void* h_up,
                                   int32_t act_dtype, int64_t n_tokens, int32_t rank_gate,
                                   int32_t rank_up, const int32_t* token_indices,
                                   const int32_t* expert_offsets, const float* route_w,
                                   int64_t n_assign, int32_t rank_out, int32_t intermediate_size,
                                   int32_t act_type, int32_t path, float* rank_accum, void* workspace,
                                   size_t workspace_bytes, bitsmoe_profile* profile, void* stream) {
    return bitsmoe_moe_forward_strided(gate, up, down, h_gate, h_up, act_dtype, n_tokens, rank_gate, rank_up, rank_gate,
                                       rank_up, token_indices, expert_offsets, route_w, n_assign, rank_out,
                                       intermediate_size, act_type, path, rank_accum, workspace, workspace_bytes, profile,
                                       stream);
}

// front_done: what an earlier launch on the stream already left in the workspace for the grouped-GEMM path
// (MFMA_FRONT_* bits; 0 for callers that bring nothing).
static int forward_strided_impl(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                                const void* h_gate, const void* h_up, int32_t act_dtype, int64_t n_tokens,
                                int32_t rank_gate, int32_t rank_up, int64_t ld_gate, int64_t ld_up,
                                const int32_t* token_indices, const int32_t* expert_offsets, const float* route_w,
                                int64_t n_assign, int32_t rank_out, int32_t intermediate_size, int32_t act_type,
                                int32_t path, float* rank_accum, void* workspace, size_t workspace_bytes, int front_done,
                                bitsmoe_profile* profile, hipStream_t st);

extern "C" int bitsmoe_moe_forward_strided(const bitsmoe_matset* gate, const bitsmoe_matset* up,
                                           const bitsmoe_matset* down, const void* h_gate, const void* h_up,
                                           int32_t act_dtype, int64_t n_tokens, int32_t rank_gate,
                                           int32_t rank_up, int64_t ld_gate, int64_t ld_up,
                                           const int32_t* token_indices, const int32_t* expert_offsets,
                                           const float* route_w, int64_t n_assign, int32_t rank_out,
                                           int32_t intermediate_size, int32_t act_type, int32_t path,
                                           float* rank_accum, void* workspace, size_t workspace_bytes,
                                           bitsmoe_profile* profile, void* stream) {
    return forward_strided_impl(gate, up, down, h_gate, h_up, act_dtype, n_tokens, rank_gate, rank_up, ld_gate, ld_up,
                                token_indices, expert_offsets, route_w, n_assign, rank_out, intermediate_size, act_type, path,
                                rank_accum, workspace, workspace_bytes, 0, profile, (hipStream_t)stream);
}

static int forward_strided_impl(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                                const void* h_gate, const void* h_up, int32_t act_dtype, int64_t n_tokens,
                                int32_t rank_gate, int32_t rank_up, int64_t ld_gate, int64_t ld_up,
                                const int32_t* token_indices, const int32_t* expert_offsets, const float* route_w,
                                int64_t n_assign, int32_t rank_out, int32_t intermediate_size, int32_t act_type,
                                int32_t path, float* rank_accum, void* workspace, size_t workspace_bytes, int front_done,
                                bitsmoe_profile* profile, hipStream_t st) {
    BITSMOE_REQUIRE(gate && up && down, "matrix sets must not be null");
    BITSMOE_REQUIRE(act_type == 0, "only SiLU act_type=0 is currently supported");
    BITSMOE_REQUIRE(act_dtype == BITSMOE_DT_F16 || act_dtype == BITSMOE_DT_BF16, "act_dtype must be f16 (0) or bf16 (1)");
    BITSMOE_REQUIRE(intermediate_size > 0, "intermediate_size must be > 0");
    BITSMOE_REQUIRE(rank_out > 0, "rank_out must be > 0");
    BITSMOE_REQUIRE(n_tokens >= 0 && n_assign >= 0, "negative token or assignment count");
    BITSMOE_REQUIRE(n_tokens < ((int64_t)1 << 31) && n_assign < ((int64_t)1 << 31), "token/assignment count exceeds int32");
    BITSMOE_REQUIRE(rank_accum != nullptr || n_tokens == 0, "rank_accum must not be null");
    BITSMOE_REQUIRE(gate->n_experts == up->n_experts && gate->n_experts == down->n_experts,
                    "gate/up/down sets hold different expert counts (%d, %d, %d)", gate->n_experts,
                    up->n_experts, down->n_experts);
    BITSMOE_REQUIRE(gate->intermediate_size == intermediate_size && up->intermediate_size == intermediate_size &&
                        down->intermediate_size == intermediate_size,
                    "intermediate_size %d does not match the matrix sets", intermediate_size);
    BITSMOE_REQUIRE(path >= BITSMOE_PATH_AUTO && path <= BITSMOE_PATH_MFMA, "unknown path %d", path);

    if (n_tokens == 0) return BITSMOE_OK;
    if (n_assign == 0 || gate->n_experts == 0) {
        if (profile) {
            for (int i = 0; i <= BITSMOE_PROFILE_PHASES; ++i) (void)hipEventRecord(profile->ev[i], st);
            profile->recorded = true;
        }
        return launch_fill_zero(rank_accum, n_tokens * (int64_t)rank_out, st);
    }
    BITSMOE_REQUIRE(h_gate && h_up && token_indices && expert_offsets && route_w, "null input pointer");
    BITSMOE_REQUIRE(rank_gate > 0 && rank_up > 0, "rank_gate/rank_up must be > 0");
    BITSMOE_REQUIRE(ld_gate >= rank_gate && ld_up >= rank_up, "ld_gate/ld_up must be at least rank_gate/rank_up");
    BITSMOE_REQUIRE(gate->max_rank_plus1 <= rank_gate && gate->min_rank >= 0,
                    "gate rank_idx references rank %d but h_gate has %d columns", gate->max_rank_plus1 - 1, rank_gate);
    BITSMOE_REQUIRE(up->max_rank_plus1 <= rank_up && up->min_rank >= 0,
                    "up rank_idx references rank %d but h_up has %d columns", up->max_rank_plus1 - 1, rank_up);
    // (rows whose rank_idx lies outside [0, rank_out) are skipped by design -- the reference does the same,
    // bitsmoe/algorithms/cpp/mlp_forward.cu:1782 -- but a down set whose EVERY reference is out of range is
    // a rank_out that does not belong to these matrices)
    BITSMOE_REQUIRE(down->total_slabs == 0 || (down->min_rank < rank_out && down->max_rank_plus1 > 0),
                    "down rank_idx references ranks [%d, %d] but rank_out is %d: no row of the down matrices writes "
                    "into rank_accum", down->min_rank, down->max_rank_plus1 - 1, rank_out);
    const int chosen = resolve_path(gate, up, down, n_assign, intermediate_size, path);
    if (chosen < 0) return chosen;
    const size_t need = bitsmoe_forward_workspace_bytes_sets(gate, up, down, n_tokens, n_assign, chosen);
    if (workspace == nullptr || workspace_bytes < need) {
        set_error("workspace too small: need %zu bytes, got %zu", need, workspace_bytes);
        return BITSMOE_E_WORKSPACE;
    }
    BITSMOE_REQUIRE(((uintptr_t)workspace & 255) == 0, "workspace must be 256-byte aligned");

    // The fast kernels work on whole 128-column tiles: their intermediates have `cols` columns per row, and the
    // prepared weights of the columns past the matrices' last one are zeros.
    const int cols = gate->n_tiles * N_TILE;
    if (chosen == BITSMOE_PATH_MFMA)
        return launch_forward_mfma(gate, up, down, h_gate, h_up, act_dtype, n_tokens, rank_gate, rank_up, ld_gate, ld_up,
                                   token_indices, expert_offsets, route_w, n_assign, rank_out, cols, rank_accum,
                                   workspace, front_done, profile, st);
    const size_t inter = align_up((size_t)n_assign * (size_t)cols * sizeof(float), 256);
    float* G = (float*)workspace;
    float* U = (float*)((char*)workspace + inter);
    if (chosen == BITSMOE_PATH_DECODE)
        return launch_forward_decode(gate, up, down, h_gate, h_up, act_dtype, n_tokens, rank_gate, rank_up, ld_gate, ld_up,
                                     token_indices, expert_offsets, route_w, n_assign, rank_out, cols,
                                     rank_accum, G, U, (int64_t)(inter / sizeof(float)), decode_part_capacity(n_assign), nullptr,
                                     profile, st);
    return launch_forward_generic(gate, up, down, h_gate, h_up, act_dtype, n_tokens, rank_gate, rank_up, ld_gate, ld_up,
                                  token_indices, expert_offsets, route_w, n_assign, rank_out,
                                  intermediate_size, rank_accum, G, U, profile, st);
}

// ---- the forward from the router's output: routing inside the kernels where they can, else the routing kernel first
static size_t routing_tables_bytes(int64_t n_flat, int32_t n_experts) {
    return 2 * align_up((size_t)n_flat * 4, 256) + align_up((size_t)(n_experts + 1) * 4, 256) +
           align_up(bitsmoe_route_workspace_bytes(n_flat, n_experts), 256);
}

extern "C" size_t bitsmoe_forward_routed_workspace_bytes(const bitsmoe_matset* gate, const bitsmoe_matset* up,
                                                         const bitsmoe_matset* down, int64_t n_tokens, int32_t top_k,
                                                         int32_t path) {
    if (!gate || !up || !down || n_tokens < 0 || top_k <= 0) return 0;
    const int64_t n_flat = n_tokens * top_k;
    return bitsmoe_forward_workspace_bytes_sets(gate, up, down, n_tokens, n_flat, path) + routing_tables_bytes(n_flat, gate->n_experts);
}

extern "C" int bitsmoe_forward_routed_is_inline(const bitsmoe_matset* gate, const bitsmoe_matset* up,
                                               const bitsmoe_matset* down, const void* h_gate, const void* h_up,
                                               int32_t rank_gate, int32_t rank_up, int64_t ld_gate, int64_t ld_up,
                                               int64_t n_tokens, int32_t top_k, int32_t path) {
    if (!gate || !up || !down || n_tokens <= 0 || top_k <= 0) return 0;
    const int I = gate->intermediate_size;
    if (path != BITSMOE_PATH_AUTO && path != BITSMOE_PATH_DECODE) return 0;
    if (resolve_path(gate, up, down, n_tokens * top_k, I, path) != BITSMOE_PATH_DECODE) return 0;
    if (wide_routed_possible(gate, up, down, n_tokens, top_k)) return 1;
    return decode_inline_route_ok(gate, up, down, h_gate, h_up, rank_gate, rank_up, ld_gate, ld_up, n_tokens, top_k, I) ? 1 : 0;
}

extern "C" int bitsmoe_forward_decode_is_fused(const bitsmoe_matset* gate, const bitsmoe_matset* up,
                                              const bitsmoe_matset* down, const void* h_gate, const void* h_up,
                                              int32_t rank_gate, int32_t rank_up, int64_t ld_gate, int64_t ld_up,
                                              int64_t n_assign, int32_t path) {
    if (!gate || !up || !down || n_assign <= 0) return 0;
    const int I = gate->intermediate_size;
    if (path != BITSMOE_PATH_AUTO && path != BITSMOE_PATH_DECODE) return 0;
    if (resolve_path(gate, up, down, n_assign, I, path) != BITSMOE_PATH_DECODE) return 0;
    return options().decode_fused != 0 && options().decode_fused_z <= 0 &&
                   decode_fused_possible(gate, up, down, h_gate, h_up, rank_gate, rank_up, ld_gate, ld_up, I) &&
                   (options().decode_fused > 0 || decode_fused_chosen(gate, n_assign, I))
               ? 1 : 0;
}

extern "C" int bitsmoe_moe_forward_routed(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                                          const void* h_gate, const void* h_up, int32_t act_dtype, int64_t n_tokens,
                                          int32_t rank_gate, int32_t rank_up, int64_t ld_gate, int64_t ld_up,
                                          const void* selected, int32_t ids_are_i64, const float* weights, int32_t top_k,
                                          const int32_t* global_to_local, int32_t n_global,
                                          const int32_t* local_to_global, int32_t rank_out, int32_t intermediate_size,
                                          int32_t act_type, int32_t path, float* rank_accum, void* workspace,
                                          size_t workspace_bytes, bitsmoe_profile* profile, void* stream) {
    hipStream_t st = (hipStream_t)stream;
    BITSMOE_REQUIRE(gate && up && down, "matrix sets must not be null");
    BITSMOE_REQUIRE(top_k > 0 && n_tokens >= 0, "n_tokens must be >= 0 and top_k > 0");
    BITSMOE_REQUIRE(n_tokens * top_k < ((int64_t)1 << 31), "too many assignments");
    BITSMOE_REQUIRE(act_type == 0, "only SiLU act_type=0 is currently supported");
    BITSMOE_REQUIRE(act_dtype == BITSMOE_DT_F16 || act_dtype == BITSMOE_DT_BF16, "act_dtype must be f16 (0) or bf16 (1)");
    const int64_t n_flat = n_tokens * top_k;
    const int E = gate->n_experts;
    if (n_tokens == 0) return BITSMOE_OK;
    const size_t need = bitsmoe_forward_routed_workspace_bytes(gate, up, down, n_tokens, top_k, path);
    if (workspace == nullptr || workspace_bytes < need) {
        set_error("workspace too small: need %zu bytes, got %zu", need, workspace_bytes);
        return BITSMOE_E_WORKSPACE;
    }
    BITSMOE_REQUIRE(((uintptr_t)workspace & 255) == 0, "workspace must be 256-byte aligned");
    // Routing inside the kernels: the same checks as the table form, then the decode launcher without tables.
    const bool shapes_ok = E > 0 && E == up->n_experts && E == down->n_experts && intermediate_size > 0 && rank_out > 0 &&
                           gate->intermediate_size == intermediate_size && up->intermediate_size == intermediate_size &&
                           down->intermediate_size == intermediate_size && h_gate && h_up && selected && weights &&
                           local_to_global && global_to_local && n_global > 0 && rank_accum && rank_gate > 0 && rank_up > 0 && ld_gate >= rank_gate &&
                           ld_up >= rank_up && gate->max_rank_plus1 <= rank_gate && gate->min_rank >= 0 &&
                           up->max_rank_plus1 <= rank_up && up->min_rank >= 0 &&
                           (down->total_slabs == 0 || (down->min_rank < rank_out && down->max_rank_plus1 > 0)) &&
                           path >= BITSMOE_PATH_AUTO && path <= BITSMOE_PATH_MFMA;
    if (shapes_ok && (path == BITSMOE_PATH_AUTO || path == BITSMOE_PATH_DECODE) &&
        resolve_path(gate, up, down, n_flat, intermediate_size, path) == BITSMOE_PATH_DECODE &&
        wide_routed_possible(gate, up, down, n_tokens, top_k)) {
        // dense experts only: their side kernels scan the routed ids themselves
        const int cols = gate->n_tiles * N_TILE;
        const size_t inter = align_up((size_t)n_flat * (size_t)cols * sizeof(float), 256);
        const DecodeRouted routed = {selected, ids_are_i64, weights, top_k, local_to_global, global_to_local, n_global};
        return launch_forward_wide_routed(gate, up, down, h_gate, h_up, act_dtype, n_tokens, rank_gate, rank_up, ld_gate, ld_up,
                                          &routed, n_flat, rank_out, cols, rank_accum, (float*)workspace,
                                          (float*)((char*)workspace + inter), (int64_t)(inter / sizeof(float)), profile, st);
    }
    if (shapes_ok && (path == BITSMOE_PATH_AUTO || path == BITSMOE_PATH_DECODE) &&
        resolve_path(gate, up, down, n_flat, intermediate_size, path) == BITSMOE_PATH_DECODE &&
        decode_inline_route_ok(gate, up, down, h_gate, h_up, rank_gate, rank_up, ld_gate, ld_up, n_tokens, top_k,
                               intermediate_size)) {
        const int cols = gate->n_tiles * N_TILE;
        const size_t inter = align_up((size_t)n_flat * (size_t)cols * sizeof(float), 256);
        float* G = (float*)workspace;
        float* U = (float*)((char*)workspace + inter);
        const DecodeRouted routed = {selected, ids_are_i64, weights, top_k, local_to_global, global_to_local, n_global};
        return launch_forward_decode(gate, up, down, h_gate, h_up, act_dtype, n_tokens, rank_gate, rank_up, ld_gate, ld_up,
                                     nullptr, nullptr, nullptr, n_flat, rank_out, cols, rank_accum, G, U,
                                     (int64_t)(inter / sizeof(float)), decode_part_capacity(n_flat), &routed, profile, st);
    }
    // Otherwise: routing tables at the end of the workspace, then the table form (which reports what is wrong
    // with the arguments, if anything is).
    BITSMOE_REQUIRE(global_to_local != nullptr, "global_to_local must not be null");
    const size_t fwd = bitsmoe_forward_workspace_bytes_sets(gate, up, down, n_tokens, n_flat, path);
    char* tail = (char*)workspace + align_up(fwd, 256);
    int32_t* tok = (int32_t*)tail;
    float* rw = (float*)(tail + align_up((size_t)n_flat * 4, 256));
    int32_t* off = (int32_t*)(tail + 2 * align_up((size_t)n_flat * 4, 256));
    void* route_ws = tail + 2 * align_up((size_t)n_flat * 4, 256) + align_up((size_t)(E + 1) * 4, 256);
    // The grouped-GEMM path's f16 copy of the activations and its per-token tables ride in the routing launches.
    RouteSideJobs jobs;
    const bool carry = options().route_jobs != 0 && shapes_ok && resolve_path(gate, up, down, n_flat, intermediate_size, path) == BITSMOE_PATH_MFMA &&
                       mfma_front_jobs(gate, up, down, h_gate, h_up, act_dtype, n_tokens, rank_gate, rank_up, ld_gate, ld_up,
                                       n_flat, gate->n_tiles * N_TILE, workspace, &jobs);
    int front_done = 0;
    const int rc = route_with_jobs(selected, ids_are_i64, weights, global_to_local, n_global, n_tokens, top_k, E, tok, off, rw,
                                   route_ws, bitsmoe_route_workspace_bytes(n_flat, E), carry ? &jobs : nullptr, &front_done, st);
    if (rc != BITSMOE_OK) return rc;
    return forward_strided_impl(gate, up, down, h_gate, h_up, act_dtype, n_tokens, rank_gate, rank_up, ld_gate, ld_up, tok, off,
                                rw, n_flat, rank_out, intermediate_size, act_type, path, rank_accum, workspace,
                                align_up(fwd, 256), front_done, profile, st);
}

extern "C" size_t bitsmoe_static_scratch_bytes(void) { return (size_t)BITSMOE_STATIC_SCRATCH_BYTES; }

extern "C" int bitsmoe_moe_forward_static(const bitsmoe_matset* gate, const bitsmoe_matset* up,
                                          const bitsmoe_matset* down, const void* h_gate, const void* h_up,
                                          int32_t act_dtype, int64_t n_tokens, int32_t rank_gate, int32_t rank_up,
                                          int64_t ld_gate, int64_t ld_up, const int32_t* token_indices,
                                          const int32_t* expert_offsets, const float* route_w, int64_t n_assign,
                                          int32_t rank_out, int32_t intermediate_size, int32_t act_type, int32_t path,
                                          float* rank_accum, void* stream) {
    BITSMOE_REQUIRE(gate && up && down, "matrix sets must not be null");
    BITSMOE_REQUIRE(n_assign >= 0 && n_tokens >= 0, "negative token or assignment count");
    BITSMOE_REQUIRE(path >= BITSMOE_PATH_AUTO && path <= BITSMOE_PATH_MFMA, "unknown path %d", path);
    // the size check comes first: a call that cannot be served touches nothing
    const int chosen = resolve_path(gate, up, down, n_assign, gate->intermediate_size, path);
    if (chosen < 0) return chosen;
    const size_t need = bitsmoe_forward_workspace_bytes_sets(gate, up, down, n_tokens, n_assign, chosen);
    if (need > (size_t)BITSMOE_STATIC_SCRATCH_BYTES) {
        set_error("bitsmoe_moe_forward_static: this call needs %zu bytes of intermediates, the static scratch holds %zu "
                  "(use bitsmoe_moe_forward with a caller-owned workspace)", need, (size_t)BITSMOE_STATIC_SCRATCH_BYTES);
        return BITSMOE_E_WORKSPACE;
    }
    void* ptr = static_scratch_of_current_device();
    if (!ptr) return BITSMOE_E_HIP;
    // Every path clears what it needs cleared with its own kernels (the array keeps the previous
    // call's contents), so the shared entry point can run on it as on any workspace.
    return bitsmoe_moe_forward_strided(gate, up, down, h_gate, h_up, act_dtype, n_tokens, rank_gate, rank_up, ld_gate, ld_up,
                                       token_indices, expert_offsets, route_w, n_assign, rank_out, intermediate_size,
                                       act_type, chosen, rank_accum, ptr, (size_t)BITSMOE_STATIC_SCRATCH_BYTES, nullptr,
                                       stream);
}
