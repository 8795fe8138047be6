// The constants by which the launchers choose kernels and grids, in one place, each with the measurement that set
// it (one MI355X, bf16 activations, cold weights: a rotation of distinct layers; times per forward under graph
// replay unless said otherwise).  Shapes named: "128-expert layer" = 128 experts, top-8, hidden 2048, intermediate
// 768 (6 column tiles); "64-expert layer" = 64 experts, top-6, intermediate 1408 (11 tiles); "512-expert layer" = 512
// experts, top-10, intermediate 512 (4 tiles).  A = routed assignments of the forward, E = experts of the matrix sets.
// tests/test_gpu_baseline_shapes.py::test_sweep_across_launcher_thresholds runs parity on both sides of every one.
#pragma once

namespace bitsmoe {
namespace policy {

// Grouped GEMM (MFMA path) instead of the decode kernels from this many assignments per expert on average.
// Crossovers measured on the three layers: 12 to 16 (the decode kernels re-stream an expert's payload for every 16
// assignments, the grouped GEMM pays for a longer launch chain: routing, conversion, SiLU pass, combine).
constexpr int MFMA_MIN_ASSIGN_PER_EXPERT = 14;

// Decode grids.  The expert coordinate counts 16-assignment CHUNKS from this many assignments per expert on average
// (most experts then have several chunks; below, the chunk search -- one more dependent round trip per workgroup,
// +10 % -- costs more than walking an expert's few chunks in a loop) ...
constexpr int CHUNK_GRID_MIN_ASSIGN_PER_EXPERT = 16;
// ... and already from this many when the layer has at most CHUNK_GRID_SMALL_LAYER experts (one search step, and
// skewed routing makes single experts long: the 26-layer stack of 64-expert layers at 32 tokens, 1.42 -> 1.17 ms).
constexpr int CHUNK_GRID_SMALL_LAYER = 64;
constexpr int CHUNK_GRID_SMALL_LAYER_MIN_ASSIGN_PER_EXPERT = 3;
// The expert coordinate counts ACTIVE experts while at most half of the experts can be active (A <= E / 2): the
// workgroups of idle experts cost more than the search (128-expert layer at 1 token: 19.1 -> 16.0 us).

// Routing inside the decode kernels (no routing kernel) on the expert grid: from this many routed entries per expert
// (below, the workgroups of experts nobody chose cost more scanning the ids than exiting after one table load:
// 1 to 5 us MORE on the 128-expert layer at 8 tokens) ...
constexpr int INLINE_ROUTE_MIN_ENTRIES_PER_EXPERT = 2;
// ... on layers of at most this many experts (512-expert layer: 1 to 5 us more with inline routing) ...
constexpr int INLINE_ROUTE_MAX_EXPERTS = 256;
// ... and at most this many column tiles (64-expert layer, 11 tiles: more workgroups per expert scan the ids: slower).
constexpr int INLINE_ROUTE_MAX_TILES = 8;
// (On the active-expert grid inline routing always pays: 3 to 5 us less per layer.  The chunk grid keeps tables.)

// k_gateup_decode (sets the walking kernel cannot take): column tiles per workgroup are halved until the grid holds
// this many workgroups (two rounds of three per CU measured best on the 128-expert layer at 64 tokens).
constexpr int GATEUP_DECODE_MIN_WORKGROUPS = 1536;
// k_down_decode: tiles per workgroup are halved until the grid holds this many workgroups (600 measured best on the
// stack at 32 tokens against 300, 1200 and 2400: the kernel is bound by the instructions a workgroup issues; more,
// shorter workgroups add their fixed part).
constexpr int DOWN_DECODE_MIN_WORKGROUPS = 600;
// k_down_decode builds z a row per wavefront (ceil(n_a / 4) memory round trips per chunk instead of ceil(n_a / 2)) from
// this many assignments per expert on average, on the grids that go by routing tables: 512 experts, 256 tokens, top-10
// (five per expert) 55.2 -> 52.4 us; 128 experts with four per expert: no difference; with one or two per expert the
// column-wise form is faster (all threads share a row).
constexpr int DOWN_Z_BY_ROWS_MIN_PER_EXPERT = 5;

}  // namespace policy
}  // namespace bitsmoe
