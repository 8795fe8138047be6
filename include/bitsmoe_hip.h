/*
 * bitsmoe_hip.h — C ABI of libbitsmoe_hip.so: the mixed-bit MoE routed-expert forward for
 * AMD gfx950 (MI355X).
 *
 * Plain pointers and sizes only; no torch types.  Every pointer named "device" must be
 * device memory on the GPU that is current when the call is made; `stream` is a
 * hipStream_t passed as void* (NULL = the default stream).  All calls return 0 on success
 * or a negative BITSMOE_E_* code; bitsmoe_last_error() returns the message of the last
 * failure on the calling thread.
 *
 * Each entry point names the reference interface it replaces (paths relative to the
 * reference tree).
 */
#ifndef BITSMOE_HIP_H
#define BITSMOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BITSMOE_OK 0
#define BITSMOE_E_INVALID (-1)   /* bad argument (shape, dtype code, null pointer, meta out of range) */
#define BITSMOE_E_HIP (-2)       /* a HIP runtime call failed */
#define BITSMOE_E_WORKSPACE (-3) /* workspace too small */
#define BITSMOE_E_UNSUPPORTED (-4)

/* activation dtype of h_gate / h_up */
#define BITSMOE_DT_F16 0
#define BITSMOE_DT_BF16 1

/* kernel-path selector for bitsmoe_moe_forward (BITSMOE_PATH_AUTO in production) */
#define BITSMOE_PATH_AUTO 0
#define BITSMOE_PATH_GENERIC 1  /* fp32 FMA kernels that accept every legal layout */
#define BITSMOE_PATH_DECODE 2   /* bandwidth-bound small-batch kernels (regular layouts only) */
#define BITSMOE_PATH_MFMA 3     /* MFMA grouped-GEMM kernels (regular layouts only) */

const char* bitsmoe_last_error(void);
const char* bitsmoe_version(void);

/*
 * One packed expert matrix: the six runtime buffers of one (expert, projection).
 * Replaces the per-expert entries of the 18 tensor lists taken by
 * moe_packed_forward (bitsmoe/algorithms/cpp/mlp_forward_binding.cpp:53-79) and the
 * buffer contract of bitsmoe/models/base_mlp.py:96-102.  Offsets inside tile_meta are in
 * uint32 words (payload) and fp16 elements (scale).
 */
typedef struct bitsmoe_matrix_desc {
    const void* payload;   /* device uint32 [payload_words]                                   */
    const void* rank_idx;  /* device int32  [rank_len]: local row -> logical rank             */
    const void* tile_meta; /* device int32  [num_tiles][3] = (pack_off, scale_off, n_valid)   */
    const void* slab_meta; /* device int32  [num_slabs][4] = (bits, k_slab, rank_off, tile_off) */
    const void* scale;     /* device fp16   [scale_len]                                       */
    const void* s;         /* device fp16   [rank_len]: per-row multiplier                    */
    int64_t payload_words;
    int64_t scale_len;
    int32_t rank_len;
    int32_t num_tiles;
    int32_t num_slabs;
    int32_t reserved;
} bitsmoe_matrix_desc;

/*
 * A "matrix set": the packed matrices of all E experts for one projection (gate, up or
 * down) of one layer.  Replaces build_packed_meta_cached / PackedMeta
 * (bitsmoe/algorithms/cpp/mlp_forward.cu:2424-2444, 2529-2697): device pointer tables,
 * per-expert counts and the down work list.  Creation copies the slab/tile/rank_idx
 * tables to the host once, validates every offset against the buffer sizes (so that no
 * kernel can read out of bounds) and uploads the tables; it synchronises `stream`.
 * The set borrows the caller's buffers: they must stay alive and unchanged until
 * bitsmoe_matset_destroy.  Unlike the reference's cache the set is owned by the caller,
 * not keyed on raw pointers.
 */
typedef struct bitsmoe_matset bitsmoe_matset;

int bitsmoe_matset_create(const bitsmoe_matrix_desc* descs, int32_t n_experts,
                          int32_t intermediate_size, void* stream, bitsmoe_matset** out);
void bitsmoe_matset_destroy(bitsmoe_matset* set);
/*
 * One-time re-layout of a set into the wave64-native copy the fast kernels read: the payload as
 * bit FIELDS in MFMA operand order, every slab padded to 64 rows (a bit bucket whose row count is
 * not a multiple of 64 ends in a ragged slab: bitsmoe/quant/packer.py:636-643), with row tables of
 * its own (rank_idx, s, scale padded the same way; padding rows carry zero scales).  The caller's
 * buffers are not modified; the library allocates the copy once and frees it in
 * bitsmoe_matset_destroy.  The copy is a SNAPSHOT: buffers overwritten afterwards need a new set.
 * role 0: gate / up (contraction over rows), role 1: down (contraction over columns).
 * Every width the packer emits is taken (bitsmoe/quant/packer.py:566-589): rows of 1-, 2-, 3- and
 * 4-bit slabs go into the field layout (1-bit levels as 2-bit fields); rows of 6-, 8- and 16-bit
 * slabs go into a side table of f16 weights (level * scale rounded once, or the stored half) in MFMA
 * operand order, which side kernels contract next to the field kernels.  A last column tile of
 * fewer than 128 columns (bitsmoe/quant/packer.py:265-287) is stored as a whole tile whose excess
 * columns are zero weights, whatever the caller's payload holds there.
 * Plays the part of the reference's one-time meta build
 * (bitsmoe/algorithms/cpp/mlp_forward.cu:2529-2697).  Returns BITSMOE_E_UNSUPPORTED for empty sets
 * and for slabs that do not span all column tiles: those run on the generic kernels only.
 * Synchronises `stream`.
 */
int bitsmoe_matset_prepare(bitsmoe_matset* set, int32_t role, void* stream);
/* Dense fp32 dequantisation read back FROM THE PREPARED LAYOUT (parity check of it). */
int bitsmoe_dequant_matrix_prepared(const bitsmoe_matset* set, int32_t expert, float* out_device,
                                    void* stream);

/* info[0]=n_experts, [1]=intermediate_size, [2]=total slabs, [3]=max logical rank + 1,
 * [4]=1 if every matrix has slabs of 16-row multiples, 2/3/4-bit, full tiles,
 * [5]=largest slab count, [6]=smallest logical rank, [7]=bit0: bitsmoe_matset_prepare can take the
 * set (fast kernels applicable), bit1: prepared, bit2: prepared for role 0 and every expert is one
 * run of equal-width slabs whose rows sit in aligned runs of eight ranks (the walking gate/up kernel),
 * bits 8 and up: 64-row slabs in the prepared set's side table of 6/8/16-bit rows */
int bitsmoe_matset_info(const bitsmoe_matset* set, int64_t info[8]);

/*
 * Dense dequantisation of one expert matrix to fp32 [rank_len, intermediate_size]
 * (row-major, local row order).  Restates decode_tile_weight * scale
 * (bitsmoe/algorithms/cpp/mlp_forward.cu:215-265, 746-749); used for bit-exact parity.
 */
int bitsmoe_dequant_matrix(const bitsmoe_matset* set, int32_t expert, float* out_device,
                           void* stream);

/*
 * Routing / permute.  Replaces _get_flat_token_ids + _build_packed_routing
 * (bitsmoe/models/base_block.py:245-289): the flat (token-major) top-k list is mapped
 * through global_to_local (entries < 0 are dropped), counted per packed expert, scanned
 * and scattered STABLY (ascending flat position inside every expert).  No host
 * synchronisation; total kept assignments = expert_offsets[n_packed] on the device.
 *   selected     device int32 or int64 [T*k]   (ids_are_i64 selects)
 *   weights      device fp32 [T*k]
 *   global_to_local device int32 [n_global]
 *   token_indices device int32 [T*k] out, expert_offsets device int32 [n_packed+1] out,
 *   route_flat   device fp32 [T*k] out         (entries past the kept count are untouched)
 */
size_t bitsmoe_route_workspace_bytes(int64_t n_flat, int32_t n_packed);
int bitsmoe_route(const void* selected, int32_t ids_are_i64, const float* weights,
                  const int32_t* global_to_local, int32_t n_global, int64_t n_tokens,
                  int32_t top_k, int32_t n_packed, int32_t* token_indices,
                  int32_t* expert_offsets, float* route_flat, void* workspace,
                  size_t workspace_bytes, void* stream);

/*
 * Router front end in one kernel.  Replaces the framework-op chain of the reference's Qwen
 * blocks (bitsmoe/models/qwen3moe/bitsmoe_block.py:45-51,
 * bitsmoe/models/qwen3next/bitsmoe_block.py:92-98): softmax of the logits in fp32, top-k
 * (descending; ties go to the lower expert index), optional division by the sum of the k
 * probabilities, optional round trip of the weights through fp16 / bf16 (round_dtype -1 / 0 / 1).
 *   logits   device [T, n_experts], logits_dtype 0 fp16 / 1 bf16 / 2 fp32
 *   selected device int32 or int64 [T, top_k] out, weights device fp32 [T, top_k] out
 */
int bitsmoe_router_softmax_topk(const void* logits, int32_t logits_dtype, int64_t n_tokens,
                                int32_t n_experts, int32_t top_k, int32_t renormalize,
                                int32_t round_dtype, void* selected, int32_t ids_are_i64,
                                float* weights, void* stream);
/*
 * The same front end for logits that are a column range of a wider row-major tensor (ld_logits elements from one
 * token's row to the next: the router's logits as a slice of ONE projection GEMM that also yields the shared-basis
 * projections), with the picked weights multiplied by weight_scale after the optional renormalisation -- the
 * softmax -> greedy top-k -> * routed_scaling_factor form of the DeepSeek-V2 gate
 * (bitsmoe/models/deepseekv2/configuration_deepseek.py:125-139, call site bitsmoe/models/deepseekv2/bitsmoe_block.py:72).
 */
int bitsmoe_router_softmax_topk_strided(const void* logits, int32_t logits_dtype, int64_t ld_logits, int64_t n_tokens,
                                        int32_t n_experts, int32_t top_k, int32_t renormalize, float weight_scale,
                                        int32_t round_dtype, void* selected, int32_t ids_are_i64, float* weights, void* stream);
/*
 * The router's linear layer and the front end above in ONE kernel, for gates that compute fp32 logits from 16-bit
 * hidden states and a 16-bit weight (the DeepSeek-V2 gate casts both to fp32 and multiplies; the reference calls
 * the model's own gate module: bitsmoe/models/deepseekv2/bitsmoe_block.py:72-74).  Products of two 16-bit values
 * are exact in fp32, so the MFMA sums equal the module's logits up to summation order; no logits reach memory.
 *   hidden  device f16 / bf16 [T, hidden_size], ld_hidden elements between rows (a multiple of 8), 16-byte aligned
 *   weight  device, the same dtype, [n_experts, hidden_size] contiguous; hidden_size a multiple of 128,
 *           n_experts <= 256; weight_is_prepared = 1: the copy bitsmoe_prepare_linear_weight made of it
 */
int bitsmoe_router_linear_topk(const void* hidden, int32_t dtype, int64_t ld_hidden, const void* weight,
                               int32_t weight_is_prepared, int64_t n_tokens, int32_t hidden_size, int32_t n_experts, int32_t top_k,
                               int32_t renormalize, float weight_scale, int32_t round_dtype, void* selected,
                               int32_t ids_are_i64, float* weights, void* stream);

/*
 * A bias-free linear layer for at most 64 rows: out[T, N] = x[T, K] * W[N, K]^T, 16-bit x / W / out of one dtype, fp32
 * sums in a fixed order.  The two GEMMs around the operator -- shared-basis, router and shared-expert projections in
 * (bitsmoe/models/qwen3moe/bitsmoe_block.py:63-64 and the routers' linear layers), output projections out
 * (bitsmoe/models/base_block.py:414) -- have this shape at decode sizes: tens of MB of weights against a handful of
 * tokens.  W in the framework's [out_features, in_features] layout, contiguous; in_features a multiple of 128,
 * out_features even; x rows ld_x elements apart (a multiple of 8), x and W 16-byte aligned.
 * x_is_f32 = 1: x is fp32 (at most 16 rows, ld_x a multiple of 4) and is rounded to `dtype` on its way into the MFMA:
 * the cast of the operator's fp32 rank_accum in front of the output projection (bitsmoe/models/base_block.py:414)
 * without a pass of its own.
 * weight_is_prepared = 1 (at most 16 rows): `weight` is the copy bitsmoe_prepare_linear_weight made of W, in the order the
 * MFMA takes it ([16-column block][k-step of 32][lane][8 values]; bitsmoe_prepared_linear_weight_elements 16-bit elements):
 * every load of a wavefront is 1 KB of consecutive memory.
 * addend (may be null): fp32 [n_rows, out_features], rows ld_addend elements apart, added to the sums before the one
 * rounding of the result -- the dense experts' share of the block output, which the reference adds in a pass of its own
 * (bitsmoe/models/base_block.py:291-307).
 */
int bitsmoe_skinny_linear(const void* x, int32_t dtype, int32_t x_is_f32, int64_t ld_x, const void* weight,
                          int32_t weight_is_prepared, int64_t n_rows, int32_t in_features, int32_t out_features,
                          void* out, int64_t ld_out, const float* addend, int64_t ld_addend, void* stream);
int64_t bitsmoe_prepared_linear_weight_elements(int32_t in_features, int32_t out_features);
int bitsmoe_prepare_linear_weight(const void* weight, int32_t in_features, int32_t out_features, void* prepared,
                                  void* stream);

/*
 * The block's closing elementwise pass: one row of the operand of the output GEMM in the activation dtype,
 *   out[t, 0 .. rank_out)                      = rank_accum[t, :]  (fp32 -> 16 bit; bitsmoe/models/base_block.py:414 casts
 *                                                 with a framework op)
 *   out[t, rank_out .. + shared_intermediate)  = silu(gate_out[t, c]) * up_out[t, c] * (sigmoid(gate_logit[t]) or 1)
 * so that the routed experts' output projection and the always-on shared expert's down projection
 * (bitsmoe/models/qwen3next/bitsmoe_block.py:144-147, bitsmoe/models/deepseekv2/bitsmoe_block.py:123-124) are one GEMM
 * against the stacked [shared_u_down | shared down_proj].  shared_intermediate may be 0 (then the pass is the cast
 * alone and the shared pointers are ignored); shared_gate_logit may be NULL (no sigmoid gate).  Row strides in
 * elements; rank_out, shared_intermediate, ld_shared and ld_out multiples of 8, pointers 16-byte aligned.
 */
int bitsmoe_block_finish(const float* rank_accum, int64_t n_tokens, int32_t rank_out, const void* shared_gate_out,
                         const void* shared_up_out, int64_t ld_shared, int32_t shared_intermediate,
                         const void* shared_gate_logit, int64_t ld_gate_logit, int32_t act_dtype, void* out, int64_t ld_out,
                         void* stream);

/*
 * The routed-expert forward.  Replaces moe_packed_forward
 * (bitsmoe/algorithms/cpp/mlp_forward_binding.cpp:53-155) ->
 * moe_packed_forward_cuda (bitsmoe/algorithms/cpp/mlp_forward.cu:2701-3074):
 *   G = (h_gate[tok] gathered by rank_idx * s) . W_gate,  U likewise,
 *   Z = silu(G) * U,  acc = W_down . Z,
 *   rank_accum[tok, rank_idx_down[r]] += acc * s_down[r] * route_w[a].
 *   h_gate device [T, rank_gate], h_up device [T, rank_up]  (fp16 or bf16, row-major)
 *   token_indices device int32 [A], expert_offsets device int32 [E+1], route_w fp32 [A]
 *   rank_accum device fp32 [T, rank_out] out (fully overwritten)
 * Never allocates and never synchronises with the host: intermediates live in
 * `workspace` (>= bitsmoe_forward_workspace_bytes_sets for the same sets, count and path).  act_type must be 0 (SiLU).
 * n_assign == 0 or zero experts writes zeros and returns (mlp_forward.cu:2733-2737).
 * `profile`, if not NULL, receives phase timings (see bitsmoe_profile_*).
 */
typedef struct bitsmoe_profile bitsmoe_profile;

size_t bitsmoe_forward_workspace_bytes(int64_t n_tokens, int64_t n_assign,
                                       int32_t intermediate_size, int32_t n_experts,
                                       int32_t rank_out);
/*
 * Workspace size for the kernel path that bitsmoe_moe_forward takes with these sets, this
 * assignment count and this `path` request (BITSMOE_PATH_AUTO chooses by size: the grouped
 * GEMM path stages activations as f16 [n_assign, rows of a matrix] and needs more than the
 * two fp32 [n_assign, intermediate] buffers of the other paths).  Takes the place of the
 * reference's per-call torch allocations (bitsmoe/algorithms/cpp/mlp_forward.cu:2837-2847,
 * 2999-3001).  bitsmoe_forward_workspace_bytes is the size of the generic and decode paths.
 */
size_t bitsmoe_forward_workspace_bytes_sets(const bitsmoe_matset* gate, const bitsmoe_matset* up,
                                            const bitsmoe_matset* down, int64_t n_tokens,
                                            int64_t n_assign, int32_t path);
int bitsmoe_moe_forward(const bitsmoe_matset* gate, const bitsmoe_matset* up,
                        const bitsmoe_matset* down, const void* h_gate, const void* h_up,
                        int32_t act_dtype, int64_t n_tokens, int32_t rank_gate,
                        int32_t rank_up, const int32_t* token_indices,
                        const int32_t* expert_offsets, const float* route_w,
                        int64_t n_assign, int32_t rank_out, int32_t intermediate_size,
                        int32_t act_type, int32_t path, float* rank_accum, void* workspace,
                        size_t workspace_bytes, bitsmoe_profile* profile, void* stream);
/*
 * The same with the activation rows ld_gate / ld_up elements apart (>= rank_gate / rank_up), so
 * that h_gate and h_up may be column ranges of one [T, rank_gate + rank_up] product of the two
 * shared-basis projections (bitsmoe/models/qwen3moe/bitsmoe_block.py:63-64 computes them as two
 * GEMMs; the reference's operator demands contiguous tensors,
 * bitsmoe/algorithms/cpp/mlp_forward_binding.cpp:80-86).  bitsmoe_moe_forward is this call with
 * ld_gate = rank_gate and ld_up = rank_up.
 */
int bitsmoe_moe_forward_strided(const bitsmoe_matset* gate, const bitsmoe_matset* up,
                                const bitsmoe_matset* down, const void* h_gate, const void* h_up,
                                int32_t act_dtype, int64_t n_tokens, int32_t rank_gate,
                                int32_t rank_up, int64_t ld_gate, int64_t ld_up,
                                const int32_t* token_indices, const int32_t* expert_offsets,
                                const float* route_w, int64_t n_assign, int32_t rank_out,
                                int32_t intermediate_size, int32_t act_type, int32_t path,
                                float* rank_accum, void* workspace, size_t workspace_bytes,
                                bitsmoe_profile* profile, void* stream);

/*
 * The forward from the router's output: what the block does between its router and its output
 * projection (bitsmoe/models/base_block.py:258-289 builds the routing tables with framework ops and
 * :381-408 calls the operator) as one call.  selected / weights: [n_tokens, top_k] expert ids (32- or
 * 64-bit, as the router numbers them) and routing weights; global_to_local [n_global] maps a router id
 * to the expert's index in the matrix sets or -1 (ids that belong to no packed expert are dropped),
 * local_to_global [n_experts] is its inverse.  For batches of at most 1024 routed entries and 256
 * tokens, on matrix sets the decode kernels take, no routing kernel runs where that was measured to be
 * faster (few active experts, or at least two entries per expert on layers of up to 256 experts and 8
 * column tiles; bitsmoe_forward_routed_is_inline tells): every workgroup finds its expert's entries among
 * the routed ids itself, and row t * top_k + j of the intermediates belongs to entry (t, j).  Otherwise
 * bitsmoe_route fills tables at the end of the workspace and
 * bitsmoe_moe_forward_strided runs on them.  Results equal those of the two-call form (the order
 * of an expert's assignments is the same; fp32 atomics aside).
 */
size_t bitsmoe_forward_routed_workspace_bytes(const bitsmoe_matset* gate, const bitsmoe_matset* up,
                                              const bitsmoe_matset* down, int64_t n_tokens, int32_t top_k,
                                              int32_t path);
/* 1 if bitsmoe_moe_forward_routed would run these arguments without a routing kernel, else 0. */
int bitsmoe_forward_routed_is_inline(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                                     const void* h_gate, const void* h_up, int32_t rank_gate, int32_t rank_up,
                                     int64_t ld_gate, int64_t ld_up, int64_t n_tokens, int32_t top_k, int32_t path);

/*
 * 1 when a forward of these sets over n_assign assignments would run as ONE kernel per (expert, tile) -- gate, up,
 * SiLU, down and the atomic combine without intermediates in memory (forward_fused.hip) -- instead of a gate/up
 * and a down launch; 0 otherwise.  No reference counterpart (the reference always launches both:
 * bitsmoe/algorithms/cpp/mlp_forward.cu:2967-2991).  For callers that attribute time to kernels.
 */
int bitsmoe_forward_decode_is_fused(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                                    const void* h_gate, const void* h_up, int32_t rank_gate, int32_t rank_up,
                                    int64_t ld_gate, int64_t ld_up, int64_t n_assign, int32_t path);
int bitsmoe_moe_forward_routed(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                               const void* h_gate, const void* h_up, int32_t act_dtype, int64_t n_tokens,
                               int32_t rank_gate, int32_t rank_up, int64_t ld_gate, int64_t ld_up,
                               const void* selected, int32_t ids_are_i64, const float* weights, int32_t top_k,
                               const int32_t* global_to_local, int32_t n_global,
                               const int32_t* local_to_global, int32_t rank_out, int32_t intermediate_size,
                               int32_t act_type, int32_t path, float* rank_accum, void* workspace,
                               size_t workspace_bytes, bitsmoe_profile* profile, void* stream);

/*
 * The forward for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): bitsmoe_moe_forward_strided without the
 * workspace argument.  No counterpart in the reference, whose operator allocates its
 * intermediates from the framework's allocator on every call.  The intermediates live in a
 * static device array of BITSMOE_STATIC_SCRATCH_BYTES that every GPU the library runs on holds
 * until the process ends; the call allocates nothing (no hipMalloc / hipFree, no framework
 * allocator).  A call whose path needs more (bitsmoe_forward_workspace_bytes_sets) fails with
 * BITSMOE_E_WORKSPACE before anything is launched.  All calls on one GPU share that GPU's array:
 * calls that overlap on one GPU (two streams, two threads) race; serialise them.
 */
#define BITSMOE_STATIC_SCRATCH_BYTES (32u << 20)
size_t bitsmoe_static_scratch_bytes(void);
int bitsmoe_moe_forward_static(const bitsmoe_matset* gate, const bitsmoe_matset* up,
                               const bitsmoe_matset* down, const void* h_gate, const void* h_up,
                               int32_t act_dtype, int64_t n_tokens, int32_t rank_gate, int32_t rank_up,
                               int64_t ld_gate, int64_t ld_up, const int32_t* token_indices,
                               const int32_t* expert_offsets, const float* route_w, int64_t n_assign,
                               int32_t rank_out, int32_t intermediate_size, int32_t act_type,
                               int32_t path, float* rank_accum, void* stream);

/*
 * Experiment switches of the launchers (no reference counterpart).  Each is read from the environment once,
 * when the library is loaded (BITSMOE_ROUTE_INLINE, BITSMOE_ROUTE_JOBS, BITSMOE_DECODE_FUSED_Z,
 * BITSMOE_DECODE_SPLIT_Z, BITSMOE_DECODE_FUSED, BITSMOE_PREFILL_SPLIT); no launch path reads the environment.
 * bitsmoe_set_option changes one for the whole process: name = "route_inline" | "route_jobs" | "decode_fused_z" |
 * "decode_split_z" | "decode_fused" | "prefill_split", value 0 / 1, or -1 for the library's own choice.  Not synchronised with forwards that run on
 * other threads at the same time.
 */
int bitsmoe_set_option(const char* name, int32_t value);

/*
 * Phase timing with HIP events recorded on the caller's stream between the kernels of
 * one bitsmoe_moe_forward call (no reference counterpart: the reference has no
 * profiling hooks in the op).  After the stream has been synchronised,
 * bitsmoe_profile_read returns milliseconds for phase i:
 *   0 = preparation (zero fill; grouped GEMM: activation conversion, tile and token lists),
 *   1 = the gate/up kernel, 2 = the SiLU-and-multiply pass (its own launch only on the grouped
 *   GEMM path, else 0), 3 = the down kernel, 4 = the per-token combine (its own launch only on
 *   the grouped GEMM path, else 0).
 */
#define BITSMOE_PROFILE_PHASES 5
int bitsmoe_profile_create(bitsmoe_profile** out);
void bitsmoe_profile_destroy(bitsmoe_profile* p);
int bitsmoe_profile_read(bitsmoe_profile* p, float ms[BITSMOE_PROFILE_PHASES]);

/*
 * Bit-plane pack / unpack of quantised levels.  Replaces pack_int8_{1,2,3,4,6,8}bit and
 * unpack_int8_* (bitsmoe/quant/bitpack/bitpack_cuda_binding.cpp:36-68, kernels
 * bitpack_cuda_kernel.cu:84-196): levels int8 [rows, cols] <-> uint32
 * [rows, ceil(cols/32)*bits], word order [row][32-column group][plane].
 */
int bitsmoe_pack_bitplanes(const int8_t* levels, int64_t rows, int64_t cols, int32_t bits,
                           uint32_t* words_out, void* stream);
int bitsmoe_unpack_bitplanes(const uint32_t* words, int64_t rows, int64_t groups,
                             int32_t bits, int8_t* levels_out, void* stream);

/*
 * The quantiser that defines the payload's contents, one wavefront per (row, 128-column tile).
 * Replaces quantize_symmetric as the packer calls it (bitsmoe/quant/quantizer.py:30-84 through
 * bitsmoe/quant/packer.py:226-246, 273): rows fp32 [k, dim] (row_stride elements apart) ->
 * levels int8 [k, ceil(dim/128)*128] (padding columns 0), scale fp32 [k, ceil(dim/128)].
 * bits 2/3/4: mean-abs start and `iters` least-squares refinements (the reference uses 50);
 * 6/8: absmax; 1: sign and mean-abs.
 */
int bitsmoe_quantize_tiles(const float* rows, int64_t k, int64_t dim, int64_t row_stride, int32_t bits,
                           int32_t iters, int8_t* levels_out, float* scale_out, void* stream);
/*
 * Slab packer for the rows of ONE bit bucket.  Replaces _pack_lowbit_slab_payload_and_scale +
 * _reorder_packed_rows_to_runtime_layout (bitsmoe/quant/packer.py:169-306): levels as written by
 * bitsmoe_quantize_tiles -> payload words [slab of <= 64 rows][tile][stage][micro][row][plane]
 * (k * ceil(dim/128) * 4 * bits words) and fp16 scales [slab][tile][row] (k * ceil(dim/128)).
 */
int bitsmoe_pack_slabs(const int8_t* levels, const float* scale, int64_t k, int64_t dim, int32_t bits,
                       uint32_t* payload_out, void* scale_out_f16, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BITSMOE_HIP_H */
