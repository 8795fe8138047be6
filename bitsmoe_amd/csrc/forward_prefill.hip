// Prefill-sized kernels of the routed-expert forward: every expert sees tens to hundreds of
// assignments, so the work is a grouped GEMM and the weights are decoded once per 128-row
// tile of assignments instead of once per 16.
//
//   k_token_count    slot of every assignment within its token (for the per-token lists)
//   k_build_mtiles   expert_offsets -> list of (expert, first assignment, rows <= 128) tiles;
//                    token_start = exclusive scan of the per-token assignment counts
//   k_bf16_to_f16 /  activations as f16, read through the token index by the GEMM kernel, or
//   k_pregather      Hs[a, k] = f16( h[tok_a, rank_idx[k]] ) in expert-sorted assignment order
//   k_gateup_mfma    G = Hs_gate . W_gate, U = Hs_up . W_up as f16;  k_silu_mul_f16: z = silu(G) * U
//   k_down_mfma      y[a, r] = s[r] * sum_c W_down[r, c] z[a, c] as f16, and the per-token lists
//   k_combine_tokens rank_accum[t, rank_idx[r]] = sum over the assignments of t of route_w * y
//
// Both GEMM kernels use 16x16x32 f16 MFMA with four wavefronts of 128 rows x 64 columns per
// workgroup.  The activation operand is staged through LDS in 128 x 64 pieces (double
// buffered, one barrier per piece); the weight operand never touches LDS: every lane loads
// its words of the prepared payload (wave_layout.h) and expands them to packed f16 pairs
// (2^w + code) with a rotate and an and-or; a packed add and a packed multiply turn the pair
// into (code - 2^(w-1)) * scale (gate/up: scale * s, folded once at prepare time) -- the same
// "weight rounded to half" operand the reference's tensor-core path builds
// (bitsmoe/algorithms/cpp/mlp_forward.cu:691-751, 1554-1694).  The top-k combine is a gather
// per token instead of the reference's fp32 atomics (mlp_forward.cu:2036-2066): its result
// does not depend on the order in which workgroups finish.
// Operands are f16 for f16 and bf16 inputs alike (f16 keeps more mantissa than bf16).
#include <algorithm>
#include <type_traits>

#include "fast_helpers.h"
#include "mtiles.h"

// ---- optional in-kernel time stamps (timeline build: -DBITSMOE_TIMELINE) of k_gateup_mfma / k_down_mfma: thread 0 of a
// workgroup writes the 100 MHz wall clock at: 0 entry, 1 tile record and tables at hand, 2 first pieces landed (before the
// first step), 3 steps done, 6 exit (after the epilogue's stores were issued).
#ifdef BITSMOE_TIMELINE
namespace bitsmoe {
constexpr int TLP_STAMPS = 8;
constexpr int TLP_MAX_WG = 8192;
__device__ unsigned long long g_tl_pf_gateup[TLP_MAX_WG * TLP_STAMPS];
__device__ unsigned long long g_tl_pf_down[TLP_MAX_WG * TLP_STAMPS];
}  // namespace bitsmoe
#define BITSMOE_TLP(arr, i)                                                             \
    do {                                                                                \
        if (threadIdx.x == 0 && blockIdx.x < ::bitsmoe::TLP_MAX_WG)                     \
            ::bitsmoe::arr[blockIdx.x * ::bitsmoe::TLP_STAMPS + (i)] = wall_clock64(); \
    } while (0)
#else
#define BITSMOE_TLP(arr, i) do {} while (0)
#endif

namespace bitsmoe {

// -(1.5 * 2^W) as a packed f16 pair: times the scale it is the constant that turns
// (2^W + code) * scale into (code - 2^(W-1)) * scale.
template <int W>
__device__ inline uint32_t neg_offset_pair() {
    return Codec<W, false>::CORR | 0x80008000u;
}

// ------------------------------------------------------------------------------ schedule
// slot[a] = how many assignments of the same token were counted before a (any order);
// token_count must be zero on entry.  Assignments outside [offsets[0], offsets[E]) belong to
// no expert and are not counted.
__global__ __launch_bounds__(256) void k_token_count(const int32_t* __restrict__ token_indices,
                                                     const int32_t* __restrict__ expert_offsets, int E, int A, int T,
                                                     int32_t* __restrict__ token_count, int32_t* __restrict__ slot) {
    const int a = blockIdx.x * 256 + threadIdx.x;
    if (a >= A) return;
    const int lo = min(max(expert_offsets[0], 0), A), hi = min(max(expert_offsets[E], 0), A);
    const int t = token_indices[a];
    int sl = -1;
    if (a >= lo && a < hi && t >= 0 && t < T) sl = atomicAdd(token_count + t, 1);
    slot[a] = sl;
}

// One workgroup: the list of (expert, first assignment, rows <= 128) tiles from
// expert_offsets (build_mtile_list), then token_start = exclusive scan of token_count (T + 1 entries).
__global__ __launch_bounds__(256) void k_build_mtiles(const int32_t* __restrict__ expert_offsets, int E, int A,
                                                      int max_tiles, MTile* __restrict__ tiles,
                                                      int32_t* __restrict__ n_tiles_out,
                                                      const int32_t* __restrict__ token_count, int T,
                                                      int32_t* __restrict__ token_start,
                                                      const FastExpert* __restrict__ gate_fe,
                                                      const FastExpert* __restrict__ up_fe) {
    __shared__ int scan[256];
    __shared__ MTileLds mt_lds;
    const int tid = threadIdx.x;
    build_mtile_list(expert_offsets, E, A, max_tiles, tiles, n_tiles_out, gate_fe, up_fe, mt_lds);

    if (token_count == nullptr) return;
    // every thread scans one contiguous run of tokens (a multiple of four: 16-byte loads)
    const int per = ((T + 255) / 256 + 3) / 4 * 4;
    const int t0 = min(tid * per, T), t1 = min(t0 + per, T);
    const bool whole = t1 - t0 == per;
    int local = 0;
    if (whole) {
#pragma unroll 4
        for (int t = t0; t < t1; t += 4) {
            const i32x4 v = *reinterpret_cast<const i32x4*>(token_count + t);
            local += v[0] + v[1] + v[2] + v[3];
        }
    } else {
        for (int t = t0; t < t1; ++t) local += token_count[t];
    }
    __syncthreads();
    scan[tid] = local;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {
        const int v = tid >= d ? scan[tid - d] : 0;
        __syncthreads();
        scan[tid] += v;
        __syncthreads();
    }
    int run = scan[tid] - local;
    if (whole) {
#pragma unroll 4
        for (int t = t0; t < t1; t += 4) {
            const i32x4 v = *reinterpret_cast<const i32x4*>(token_count + t);
            i32x4 o;
            o[0] = run;
            o[1] = o[0] + v[0];
            o[2] = o[1] + v[1];
            o[3] = o[2] + v[2];
            run = o[3] + v[3];
            *reinterpret_cast<i32x4*>(token_start + t) = o;
        }
    } else {
        for (int t = t0; t < t1; ++t) {
            token_start[t] = run;
            run += token_count[t];
        }
    }
    if (tid == 255) token_start[T] = scan[255];
}

// ------------------------------------------------------------------------------- gather
template <bool BF16>
__device__ inline float raw_to_f32(uint32_t v) {
    if constexpr (BF16)
        return __uint_as_float(v << 16);
    else
        return __half2float(__ushort_as_half((uint16_t)v));
}

// grid (ceil(A / 4), 2): one wavefront per (assignment, projection).
template <bool BF16>
__global__ __launch_bounds__(256) void k_pregather(const FastExpert* __restrict__ gate_fe,
                                                   const FastExpert* __restrict__ up_fe,
                                                   const uint16_t* __restrict__ h_gate,
                                                   const uint16_t* __restrict__ h_up, int Rg, int Ru, int64_t sg,
                                                   int64_t su, const int32_t* __restrict__ token_indices,
                                                   const int32_t* __restrict__ expert_offsets, int E, int T, int A,
                                                   uint16_t* __restrict__ Hs_g, uint16_t* __restrict__ Hs_u, int ldg,
                                                   int ldu) {
    const int lane = threadIdx.x & 63;
    const int a = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int mt = blockIdx.y;
    if (a >= A) return;
    // the expert of assignment a = number of experts whose range ends at or before a
    int cnt = 0;
    for (int j = lane; j < E; j += 64) cnt += (expert_offsets[j + 1] <= a) ? 1 : 0;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) cnt += __shfl_xor(cnt, d);
    const int e = __builtin_amdgcn_readfirstlane(cnt);
    if (e >= E) return;   // past the last kept assignment
    const FastExpert fe = (mt ? up_fe : gate_fe)[e];
    const uint16_t* __restrict__ h = mt ? h_up : h_gate;
    const int R = mt ? Ru : Rg;
    const int ld = mt ? ldu : ldg;
    uint16_t* __restrict__ out = (mt ? Hs_u : Hs_g) + (int64_t)a * ld;
    const int tok = token_indices[a];
    const bool tok_ok = tok >= 0 && tok < T;
    const int64_t hrow = (int64_t)(tok_ok ? tok : 0) * (mt ? su : sg);      // sg, su: elements between activation rows
    const int K = min(fe.num_slabs * SLAB_ROWS, ld);
    gptr<int32_t> rank_idx = as_global(fe.rank_idx);
    for (int k0 = lane * 8; k0 < K; k0 += 512) {
        const i32x4 r0 = *reinterpret_cast<const i32x4 __attribute__((address_space(1)))*>(rank_idx + k0);
        const i32x4 r1 = *reinterpret_cast<const i32x4 __attribute__((address_space(1)))*>(rank_idx + k0 + 4);
        uint32_t raw[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int r = i < 4 ? r0[i] : r1[i - 4];
            raw[i] = h[hrow + min(max(r, 0), R - 1)];
        }
        u32x4 packed;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int r = i < 4 ? r0[i] : r1[i - 4];
            const float v = (tok_ok && r >= 0 && r < R) ? raw_to_f32<BF16>(raw[i]) : 0.0f;
            const uint32_t hb = __builtin_bit_cast(uint16_t, (_Float16)v);
            if (i & 1)
                packed[i >> 1] |= hb << 16;
            else
                packed[i >> 1] = hb;
        }
        *reinterpret_cast<u32x4*>(out + k0) = packed;
    }
}

// bf16 activations (rows sg / su elements apart) -> f16 [T, ld] (columns < ld); blockIdx.y = 0: gate, 1: up;
// grid-stride over 8-element groups.
__global__ __launch_bounds__(256) void k_bf16_to_f16(const uint16_t* __restrict__ src_g, const uint16_t* __restrict__ src_u,
                                                     int64_t T, int64_t sg, int64_t su, int ldg, int ldu,
                                                     uint16_t* __restrict__ dst_g, uint16_t* __restrict__ dst_u,
                                                     int32_t* __restrict__ zero, int n_zero) {
    // (also clears the per-token counters: one launch less in front of the GEMM)
    if (blockIdx.y == 0)
        for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n_zero; i += gridDim.x * blockDim.x) zero[i] = 0;
    const bool is_up = blockIdx.y != 0;
    const uint16_t* src = is_up ? src_u : src_g;
    uint16_t* dst = is_up ? dst_u : dst_g;
    const int64_t R = is_up ? su : sg;      // elements between source rows
    const int ld = is_up ? ldu : ldg;
    const int per_row = ld >> 3;
    const int64_t total = T * per_row;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row = i / per_row;
        const int c = (int)(i - row * per_row) * 8;
        const u32x4 v = *reinterpret_cast<const u32x4*>(src + row * R + c);
        u32x4 o;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t lo = __builtin_bit_cast(uint16_t, (_Float16)__uint_as_float(v[k] << 16));
            const uint32_t hi = __builtin_bit_cast(uint16_t, (_Float16)__uint_as_float(v[k] & 0xFFFF0000u));
            o[k] = lo | (hi << 16);
        }
        *reinterpret_cast<u32x4*>(dst + row * ld + c) = o;
    }
}

// --------------------------------------------------------------------------- shared GEMM parts
// Workgroup id -> logical work index = tile * units + unit.  Hardware places workgroup b on XCD
// b % 8, and every XCD has its own L2: the `units` workgroups of one assignment tile (which share
// its activations) get ids of one residue class.  The tile list is ordered by decreasing cost; it
// is dealt to the XCDs back and forth (tiles 0..7 to XCDs 0..7, tiles 8..15 to XCDs 7..0, ...), so
// that every XCD gets the same mix and starts its own share in order of decreasing cost.
// The grid holds 32 * ceil(max tiles / 32) * units workgroups; -1: no such tile.
__device__ inline int xcd_logical(int bid, int n_tiles_real, int units) {
    const int slot = bid >> 3, x = bid & 7;
    const int q = slot / units;
    const int tile = q * 8 + ((q & 1) ? 7 - x : x);
    if (tile >= n_tiles_real) return -1;
    return tile * units + slot % units;
}

// 128 x 64 16-bit activation piece: thread i owns rows i/8 + 32*j (j = 0..3), elements 8*(i%8)..+7.
// NJ: how many of the four 32-row groups hold assignments (tiles of at most 32 rows: one).
struct APiece {
    u32x4 v[4];
};
// LDS element offset of the 16-byte chunk c (0..7) of row r of a 128 x 64 stage: rows are 128
// bytes apart without padding, and the chunks of a row are permuted by the row index so that the
// sixteen rows an MFMA operand load touches fall into different banks.  (LDS-direct loads fill
// LDS in lane order, which rules out padded rows.)
__device__ __forceinline__ int dma_chunk_off(int r, int c) { return r * 64 + ((c ^ ((r >> 1) & 7)) << 3); }

// s_waitcnt that only waits for the vector-memory counter: at most `n` operations outstanding
// (the counter is six bits wide, split over the immediate; the other counters are left alone).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | 0x0F70);
}
// s_waitcnt lgkmcnt(0) alone: every LDS read of the wavefront has returned (the vector-memory and
// export counters are left at their maxima).
__device__ __forceinline__ void wait_lds_reads() { __builtin_amdgcn_s_waitcnt(0xC07F); }
// Workgroup barrier without the wait for outstanding loads that __syncthreads implies.  The empty
// asm statements keep the compiler from moving LDS accesses across it (the bare instruction is no
// memory fence for the compiler).
__device__ __forceinline__ void barrier_no_drain() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}
constexpr int DMA_STAGE = PF_M * 64;    // 16-bit elements of one unpadded 128 x 64 activation piece

// LDS-direct load: every active lane fetches 16 bytes from `src`, and the wavefront's data lands in
// LDS at lds_base + 16 * lane (lds_base is wave-uniform).  Issued from an asm statement, so the
// compiler keeps no book on it: it neither waits for these loads before LDS reads it cannot tell
// apart from their destination, nor turns its other waits into waits for everything.  The caller
// counts them (wait_vmcnt) and orders LDS accesses around them (barrier_no_drain).
__device__ __forceinline__ void load_to_lds16(const void* src, void* lds_base) {
    using lvoid = void __attribute__((address_space(3)))*;
    const uint32_t l = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lvoid)lds_base);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(l) : "m0", "memory");
}

// ------------------------------------------------------------------------------ gate / up

// Everything one thread fetches from global memory for one slab.
struct GuFetch {
    APiece a;          // this thread's part of the 128 x 64 activation piece
    u32x4 sc[2];       // scale pairs of the eight contraction rows this lane feeds per k-step (its own tile)
    uint32_t bw[2][4]; // payload words of the wavefront's two column-block pairs (its own tile)
};

// One slab (64 contraction rows, `bits` wide) for a wavefront's (16 * NMB) x 64 tile.  The weight
// operand is (code - 2^(bits-1)) * scale_s rounded once to f16 -- the operand the reference
// builds (bitsmoe/algorithms/cpp/mlp_forward.cu:691-751), with the per-row multiplier s folded
// into the scale -- made from the raw field decode 2^bits + code / f (f: the row's stagger factor,
// a power of two that the scale table carries) by a packed add (exact) and a packed multiply.  (One packed FMA with the constant -1.5 * 2^bits * scale_s would round that
// constant: measured 4.5e-3 of error instead of 5e-4.)
// WU != 0: the width is a compile-time constant (experts whose slabs all share it).
template <int WU, int NMB>
__device__ __forceinline__ void gateup_slab_mfma(int bits, const uint16_t* __restrict__ stage, const uint32_t (&bw)[2][4],
                                                 const u32x4 (&sc)[2], int lane, f32x4 (&acc)[NMB][4]) {
    const int n = lane & 15, kg = lane >> 4;
    const int wb = WU != 0 ? WU : bits;
    // minus (2^w + 2^(w-1) / f_i): leaves (code - 2^(w-1)) / f_i of the staggered decode (wave_layout.h);
    // the scale table carries f_i
    u32x4 neg = wb == 2 ? offset0_regs<2>() : wb == 3 ? offset0_regs<3>() : offset0_regs<4>();
#pragma unroll
    for (int i = 0; i < 4; ++i) neg[i] |= 0x80008000u;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        u32x4 a[NMB];
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb)
            a[mb] = *reinterpret_cast<const u32x4*>(
                stage + dma_chunk_off(16 * mb + n, 2 * kg + ks));
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
            const uint32_t(&w)[4] = bw[nb >> 1];
            const int nbl = nb & 1;
            // WU == 0: the width switch wraps the decode of one operand only, so that the accumulators
            // do not flow through alternative paths (which multiplies the register demand)
            u32x4 b;
            if (WU == 2 || (WU == 0 && bits == 2))
                b = decode0_lo<2>(w[nbl], ks);
            else if (WU == 4 || (WU == 0 && bits == 4))
                b = decode0_fields4(w[2 * nbl + ks]);
            else
                b = decode0_fields3(w[nbl], ks, w[2 + nbl], n >> 3);
#pragma unroll
            for (int i = 0; i < 4; ++i) b[i] = pk_mul_f16(pk_add_f16(b[i], neg[i]), sc[ks][i]);
#pragma unroll
            for (int mb = 0; mb < NMB; ++mb) acc[mb][nb] = mfma16<false>(a[mb], b, acc[mb][nb]);
        }
    }
}

// One workgroup = (assignment tile, projection, PAIR of 128-column tiles):
// out[a, c] = f16 of sum_k A[a, k] * f16(level[k, c] * scale_s[tile(c), k]) over all slabs of the matrix.
// Wavefront (tl, wn) owns all assignments of the tile and columns 64*wn .. +63 of tile t0 + tl: a
// decoded weight operand feeds NMB MFMAs.  The activation piece of a slab (128 x 64) is staged in
// LDS once for both tiles; the loads of slab s + 2 are issued before slab s is multiplied.
//
// DIRECT: the activation rows are read straight from the f16 activations [T, ld] through the
// token index (possible when every aligned run of 8 local rows is 8 consecutive logical ranks);
// otherwise Hs is the pre-gathered [A, ld].  WU: the bit-width shared by every slab of the
// matrix, or 0 (mixed).  NMB: 16-row blocks of the assignment tile that are computed.
template <bool DIRECT, int WU, int NMB>
__device__ __forceinline__ void gateup_tile_body(const FastExpert fe, const FastSlab* __restrict__ fs_row, int nslabs,
                                                 const uint16_t* __restrict__ Hs, int ld,
                                                 const int32_t* __restrict__ token_indices, int T, int I, int n_tiles,
                                                 uint16_t* __restrict__ out, int a_begin, int rows, int t0,
                                                 uint16_t* __restrict__ stage_even, uint16_t* __restrict__ stage_odd,
                                                 bool fuse_silu) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tl = wave >> 1, wn = wave & 1;
    const int n = lane & 15, kg = lane >> 4;
    const bool two_tiles = t0 + 1 < n_tiles;
    const bool active = tl == 0 || two_tiles;        // a wavefront without a tile only helps to stage
    const int t = active ? t0 + tl : t0;             // (it re-reads tile t0: in bounds)

    // this thread's staging rows; DIRECT: their activation rows (invalid tokens read row 0: the
    // combine drops their outputs).  Element offsets: the launcher checks that they fit 32 bits.
    constexpr int NJ = (NMB + 1) / 2;      // 32-row groups that hold assignments
    const int r0 = tid >> 3, kc = (tid & 7) * 8;
    uint32_t rowbase[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int a = a_begin + min(r0 + 32 * j, rows - 1);
        if constexpr (DIRECT) {
            const int tk = token_indices[a];
            rowbase[j] = (uint32_t)((tk >= 0 && tk < T) ? tk : 0) * (uint32_t)ld;
        } else {
            rowbase[j] = (uint32_t)a * (uint32_t)ld + (uint32_t)kc;
        }
    }

    f32x4 acc[NMB][4];
#pragma unroll
    for (int i = 0; i < NMB; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0, 0, 0, 0};
    gptr<uint32_t> payload = as_global(fe.payload);
    gptr<__half> scale = as_global(fe.scale_s);
    gptr<int32_t> rank_idx = as_global(fe.rank_idx);
    GuFetch F;                 // the one slab in flight
    auto slab_rec = [&](int s) { return s < nslabs ? load_fast_slab(fs_row, s) : FastSlab{0, 0, 0, 0}; };
    auto rank_base = [&](int s) { return (DIRECT && s < nslabs) ? rank_idx[s * SLAB_ROWS + kc] : 0; };
    auto issue = [&](GuFetch& dst, const FastSlab& r, int rbase, int s) {
        const int wb = WU != 0 ? WU : r.bits;
        const uint32_t col = DIRECT ? (uint32_t)rbase : (uint32_t)(s * SLAB_ROWS);
#pragma unroll
        for (int j = 0; j < NJ; ++j) dst.a.v[j] = *reinterpret_cast<const u32x4*>(Hs + (rowbase[j] + col));
        // the MFMA operand of k-step ks holds contraction rows 16*kg + 8*ks .. +7 of the slab
        gptr<__half> sp = scale + (uint32_t)(r.scale_off + t * SLAB_ROWS + 16 * kg);
        dst.sc[0] = *reinterpret_cast<gptr_u32x4>(sp);
        dst.sc[1] = *reinterpret_cast<gptr_u32x4>(sp + 8);
        gptr<uint32_t> blk = payload + (uint32_t)(r.pack_off + t * 256 * wb);
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int pair = 2 * wn + p;
            load_pair_role0(blk, wb, (uint32_t)(pair * 64 + lane), (uint32_t)hi_index0(kg, n, 2 * pair), dst.bw[p]);
        }
    };
    auto stage_piece = [&](const GuFetch& src, uint16_t* __restrict__ stage) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) *reinterpret_cast<u32x4*>(stage + dma_chunk_off(r0 + 32 * j, tid & 7)) = src.a.v[j];
    };
    if (nslabs > 0) {
        // prologue: slab 0 is fetched and staged, slab 1 requested
        uint32_t bw[2][4];       // payload words and scales of the slab being multiplied
        u32x4 sc[2];
        FastSlab rec = slab_rec(0);
        FastSlab pending = slab_rec(1);
        int pending_rb = rank_base(1);
        int bits = rec.bits;
        issue(F, rec, rank_base(0), 0);
        stage_piece(F, stage_even);
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            sc[p] = F.sc[p];
#pragma unroll
            for (int i = 0; i < 4; ++i) bw[p][i] = F.bw[p][i];
        }
        int bits_next = pending.bits;
        if (nslabs > 1) {
            issue(F, pending, pending_rb, 1);
            pending = slab_rec(2);
            pending_rb = rank_base(2);
        }
        __syncthreads();
        // step s: slab s is in LDS stage s % 2 with its words in `bw`; slab s + 1 (in flight in F) is
        // staged, slab s + 2 requested, then slab s is multiplied
        for (int s = 0; s < nslabs; ++s) {
            uint32_t bw_next[2][4];
            u32x4 sc_next[2];
            const int bits_after = pending.bits;
            if (s + 1 < nslabs) {
                stage_piece(F, (s & 1) ? stage_even : stage_odd);
#pragma unroll
                for (int p = 0; p < 2; ++p) {
                    sc_next[p] = F.sc[p];
#pragma unroll
                    for (int i = 0; i < 4; ++i) bw_next[p][i] = F.bw[p][i];
                }
                if (s + 2 < nslabs) {
                    issue(F, pending, pending_rb, s + 2);
                    pending = slab_rec(s + 3);
                    pending_rb = rank_base(s + 3);
                }
            }
            if (active && bits != 0)
                gateup_slab_mfma<WU, NMB>(bits, (s & 1) ? stage_odd : stage_even, bw, sc, lane, acc);
            __syncthreads();
            if (s + 1 < nslabs) {
#pragma unroll
                for (int p = 0; p < 2; ++p) {
                    sc[p] = sc_next[p];
#pragma unroll
                    for (int i = 0; i < 4; ++i) bw[p][i] = bw_next[p][i];
                }
                bits = bits_next;
                bits_next = bits_after;
            }
        }
    }
    if (!active) return;
    // lane holds rows 16*mb + 4*kg + j, column 128*t + 64*wn + 16*nb + n
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb) {
        if (16 * mb >= rows) break;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = 16 * mb + 4 * kg + j;
            if (row >= rows) continue;
            uint16_t* dst = out + (int64_t)(a_begin + row) * I + N_TILE * t + 64 * wn + n;
            if (fuse_silu) {
                // `out` holds the gate sums an earlier launch stored: z = silu(gate) * up takes their place
                uint16_t gbits[4];
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) gbits[nb] = dst[16 * nb];
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) {
                    const float g = __half2float(__ushort_as_half(gbits[nb]));
                    dst[16 * nb] = z_operand(g, acc[mb][nb][j]);
                }
                continue;
            }
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) dst[16 * nb] = __builtin_bit_cast(uint16_t, (_Float16)acc[mb][nb][j]);
        }
    }
}

constexpr int DMA_STAGES = 3;
constexpr int DMA_MAX_SLABS = 64;       // per-slab tables in LDS
constexpr int DMA_WSTAGE = 4 * 512;     // 32-bit words: payload of a (slab, tile) block as the four wavefronts fetch it
constexpr int DMA_SSTAGE = 4 * 64;      // 16-bit scales: 64 contraction rows per wavefront

// One stage of the ring: everything a workgroup needs for one slab.
struct DmaStage {
    uint16_t* a;     // [DMA_STAGE]
    uint32_t* w;     // [DMA_WSTAGE]
    uint16_t* sc;    // [DMA_SSTAGE]
};

// The same workgroup job as gateup_tile_body for experts of one bit-width, with EVERYTHING of a
// slab -- activation piece, payload words, scales -- loaded straight from global memory into LDS
// (global_load_lds: no registers, no staging instructions), two slabs ahead of the MFMAs in a ring
// of three stages.  A wavefront's load instruction fills LDS in lane order; which 16-byte chunk of
// its activation row a lane fetches is chosen so that the stage ends up in the bank-friendly order
// of dma_chunk_off.  The loop contains no load into registers: the loads of a wavefront complete in
// order, so "slab s + 1 has landed" is "at most the G loads of slab s + 2 are outstanding", waited
// for with a bare s_waitcnt, and the workgroup barrier is the bare instruction (__syncthreads would
// wait for every outstanding load).  Per-slab offsets come from small LDS tables built up front.
template <bool DIRECT, int WU, int NMB>
__device__ __forceinline__ void gateup_tile_body_dma(const FastExpert fe, const FastSlab* __restrict__ fs_row, int nslabs,
                                                     const uint16_t* __restrict__ Hs, int ld,
                                                     const int32_t* __restrict__ token_indices, int T, int I,
                                                     int n_tiles, uint16_t* __restrict__ out, int a_begin, int rows,
                                                     int t0, const DmaStage st0, const DmaStage st1, const DmaStage st2,
                                                     int32_t* __restrict__ pack_tab, int32_t* __restrict__ scale_tab,
                                                     int32_t* __restrict__ rank_tab, int32_t* __restrict__ bits_tab,
                                                     bool fuse_silu) {
    static_assert(WU == 0 || WU == 2 || WU == 3 || WU == 4, "a bit-width, or 0 for widths that differ from slab to slab");
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tl = wave >> 1, wn = wave & 1;
    const int n = lane & 15, kg = lane >> 4;
    const bool two_tiles = t0 + 1 < n_tiles;
    const bool active = tl == 0 || two_tiles;        // a wavefront without a tile only helps to stage
    const int t = active ? t0 + tl : t0;             // (it re-reads tile t0: in bounds)

    // this lane lands in row r0 + 32*j, chunk position tid % 8 of a stage; it fetches the chunk that
    // belongs there (32*j does not change the permutation).  DIRECT: through the token index.
    constexpr int NJ = (NMB + 1) / 2;      // 32-row groups that hold assignments
    constexpr int NB = WU == 2 ? 1 : 2;    // payload load instructions per slab (mixed widths: always two, so that
                                           // one wait count serves every slab; a 2-bit slab repeats its load)
    constexpr int G = NJ + 1 + NB;         // load instructions per slab and wavefront
    const int r0 = tid >> 3;
    const int cpos = (tid & 7) ^ ((r0 >> 1) & 7);
    uint32_t rowbase[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int a = a_begin + min(r0 + 32 * j, rows - 1);
        if constexpr (DIRECT) {
            const int tk = token_indices[a];
            rowbase[j] = (uint32_t)((tk >= 0 && tk < T) ? tk : 0) * (uint32_t)ld;
        } else {
            rowbase[j] = (uint32_t)a * (uint32_t)ld + (uint32_t)(8 * cpos);
        }
    }
    // per-slab tables (ordinary loads, finished before the first LDS-direct load is issued)
    gptr<int32_t> rank_idx = as_global(fe.rank_idx);
    for (int i = tid; i < nslabs; i += 256) {
        const i32x4 r = *reinterpret_cast<const i32x4*>(fs_row + i);     // {bits, pack_off, scale_off, rank_off}
        pack_tab[i] = r[1];
        scale_tab[i] = r[2];
        if constexpr (WU == 0) bits_tab[i] = r[0];
    }
    if constexpr (DIRECT)
        for (int i = tid; i < nslabs * 8; i += 256) rank_tab[i] = rank_idx[(i >> 3) * SLAB_ROWS + (i & 7) * 8];
    __syncthreads();

    f32x4 acc[NMB][4];
#pragma unroll
    for (int i = 0; i < NMB; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0, 0, 0, 0};
    const uint32_t* __restrict__ payload = fe.payload;
    const __half* __restrict__ scale = fe.scale_s;
    // all loads of slab s into stage `st`: G instructions for every wavefront
    auto request = [&](const DmaStage& st, int s) {
        const uint32_t col = DIRECT ? (uint32_t)rank_tab[s * 8 + cpos] : (uint32_t)(s * SLAB_ROWS);
#pragma unroll
        for (int j = 0; j < NJ; ++j)
            load_to_lds16(Hs + (rowbase[j] + col), st.a + j * 2048 + wave * 512);
        // scales of this wavefront's tile: 64 contraction rows, eight lanes of 16 bytes
        if (lane < 8)
            load_to_lds16(scale + (uint32_t)(scale_tab[s] + t * SLAB_ROWS + lane * 8), st.sc + wave * 64);
        // payload of the wavefront's two column-block pairs, in memory order
        if constexpr (WU == 0) {
            const int W = __builtin_amdgcn_readfirstlane(bits_tab[s]);
            const uint32_t* blk = payload + (uint32_t)(pack_tab[s] + t * 256 * W);
            const uint32_t first = W == 4 ? (uint32_t)((2 * wn * 64 + lane) * 4) : (uint32_t)(2 * wn * 128 + lane * 4);
            const uint32_t second = W == 4 ? first + 256u : W == 3 ? (uint32_t)(512 + 2 * wn * 64 + lane * 4) : first;
            load_to_lds16(blk + first, st.w + wave * 512);
            if (W != 3 || lane < 32) load_to_lds16(blk + second, st.w + wave * 512 + 256);
            return;
        }
        const uint32_t* blk = payload + (uint32_t)(pack_tab[s] + t * 256 * WU);
        if constexpr (WU == 4) {
#pragma unroll
            for (int p = 0; p < 2; ++p)
                load_to_lds16(blk + ((2 * wn + p) * 64 + lane) * 4, st.w + wave * 512 + p * 256);
        } else {
            load_to_lds16(blk + 2 * wn * 128 + lane * 4, st.w + wave * 512);
            if constexpr (WU == 3) {
                if (lane < 32)
                    load_to_lds16(blk + 512 + 2 * wn * 64 + lane * 4, st.w + wave * 512 + 256);
            }
        }
    };
    // payload words and scales of the slab in stage `st`, from LDS to this lane's registers
    auto take = [&](const DmaStage& st, int W, uint32_t (&bw)[2][4], u32x4 (&sc)[2]) {
        const uint32_t* wbase = st.w + wave * 512;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            if (WU == 4 || (WU == 0 && W == 4)) {
                const u32x4 v = *reinterpret_cast<const u32x4*>(wbase + p * 256 + lane * 4);
                bw[p][0] = v[0]; bw[p][1] = v[1]; bw[p][2] = v[2]; bw[p][3] = v[3];
            } else {
                const u32x2 v = *reinterpret_cast<const u32x2*>(wbase + p * 128 + lane * 2);
                bw[p][0] = v[0]; bw[p][1] = v[1]; bw[p][2] = 0; bw[p][3] = 0;
                if (WU == 3 || (WU == 0 && W == 3)) {
                    const u32x2 h = *reinterpret_cast<const u32x2*>(wbase + 256 + (p * 32 + kg * 8 + (n & 7)) * 2);
                    bw[p][2] = h[0]; bw[p][3] = h[1];
                }
            }
        }
        // the MFMA operand of k-step ks holds contraction rows 16*kg + 8*ks .. +7 of the slab
        sc[0] = *reinterpret_cast<const u32x4*>(st.sc + wave * 64 + 16 * kg);
        sc[1] = *reinterpret_cast<const u32x4*>(st.sc + wave * 64 + 16 * kg + 8);
    };
    if (nslabs > 0) {
        request(st0, 0);
        if (nslabs > 1) request(st1, 1);
        if (nslabs > 1)
            wait_vmcnt<G>();
        else
            wait_vmcnt<0>();
        barrier_no_drain();
        BITSMOE_TLP(g_tl_pf_gateup, 2);
        // step s (s % 3 == U): slab s + 2 requested into the stage slab s - 1 used, slab s multiplied
        auto step = [&](auto u_c, int s) {
            constexpr int U = decltype(u_c)::value;
            // (the stages are named statically, so that the compiler can tell the stage being read
            // from the ones being loaded)
            const DmaStage& cur = U == 0 ? st0 : U == 1 ? st1 : st2;
            const DmaStage& nxt = U == 0 ? st2 : U == 1 ? st0 : st1;
            uint32_t bw[2][4];
            u32x4 sc[2];
            const int W = WU != 0 ? WU : __builtin_amdgcn_readfirstlane(bits_tab[s]);
            take(cur, W, bw, sc);
            if (s + 2 < nslabs) request(nxt, s + 2);
            if (active) gateup_slab_mfma<WU, NMB>(W, cur.a, bw, sc, lane, acc);
            asm volatile("" ::: "memory");
            if (s + 2 < nslabs)
                wait_vmcnt<G>();      // slab s + 1 has landed; slab s + 2 may be in flight
            else
                wait_vmcnt<0>();
            barrier_no_drain();
        };
        for (int s0 = 0; s0 < nslabs; s0 += DMA_STAGES) {
            step(std::integral_constant<int, 0>{}, s0);
            if (s0 + 1 < nslabs) step(std::integral_constant<int, 1>{}, s0 + 1);
            if (s0 + 2 < nslabs) step(std::integral_constant<int, 2>{}, s0 + 2);
        }
    }
    BITSMOE_TLP(g_tl_pf_gateup, 3);
    if (!active) return;
    // lane holds rows 16*mb + 4*kg + j, column 128*t + 64*wn + 16*nb + n
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb) {
        if (16 * mb >= rows) break;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = 16 * mb + 4 * kg + j;
            if (row >= rows) continue;
            uint16_t* dst = out + (int64_t)(a_begin + row) * I + N_TILE * t + 64 * wn + n;
            if (fuse_silu) {
                // `out` holds the gate sums an earlier launch stored: z = silu(gate) * up takes their place
                uint16_t gbits[4];
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) gbits[nb] = dst[16 * nb];
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) {
                    const float g = __half2float(__ushort_as_half(gbits[nb]));
                    dst[16 * nb] = z_operand(g, acc[mb][nb][j]);
                }
                continue;
            }
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) dst[16 * nb] = __builtin_bit_cast(uint16_t, (_Float16)acc[mb][nb][j]);
        }
    }
}

// grid.x = 32 * ceil(max_mtiles / 32) * (2 or 1 projections) * ceil(n_tiles / 2), 256 threads; G and U are f16 [A, I].
template <bool DIRECT>
__global__ __launch_bounds__(256, 2) void k_gateup_mfma(
    const FastExpert* __restrict__ gate_fe, const FastSlab* __restrict__ gate_fs, int gate_max_slabs,
    const FastExpert* __restrict__ up_fe, const FastSlab* __restrict__ up_fs, int up_max_slabs,
    const uint16_t* __restrict__ Hs_g, const uint16_t* __restrict__ Hs_u, int ldg, int ldu,
    const int32_t* __restrict__ token_indices, int T,
    const MTile* __restrict__ mtiles, const int32_t* __restrict__ n_mtiles, int I, int n_tiles,
    uint16_t* __restrict__ G, uint16_t* __restrict__ U, int proj_sel, int fuse) {
    // The ring of the LDS-direct bodies; the register-staged body uses two of the activation stages.
    __shared__ __attribute__((aligned(16))) uint16_t sa0[DMA_STAGE], sa1[DMA_STAGE], sa2[DMA_STAGE];
    __shared__ __attribute__((aligned(16))) uint32_t sw0[DMA_WSTAGE], sw1[DMA_WSTAGE], sw2[DMA_WSTAGE];
    __shared__ __attribute__((aligned(16))) uint16_t ss0[DMA_SSTAGE], ss1[DMA_SSTAGE], ss2[DMA_SSTAGE];
    __shared__ int32_t pack_tab[DMA_MAX_SLABS], scale_tab[DMA_MAX_SLABS], rank_tab[DMA_MAX_SLABS * 8], bits_tab[DMA_MAX_SLABS];
    BITSMOE_TLP(g_tl_pf_gateup, 0);
    const int n_tp = (n_tiles + 1) >> 1;
    // proj_sel < 0: both projections in this launch; 0 / 1: the gate / the up projection alone.  fuse (up alone, after
    // a gate launch): the epilogue stores z = silu(gate) * up over the gate sums instead of the up sums.
    const int units = proj_sel < 0 ? 2 * n_tp : n_tp;
    const int logical = xcd_logical(blockIdx.x, __builtin_amdgcn_readfirstlane(*n_mtiles), units);
    if (logical < 0) return;
    // the tile pairs of one (assignment tile, projection) are neighbours: they share the activations
    const int tp = logical % n_tp;
    const int proj = proj_sel < 0 ? (logical / n_tp) & 1 : proj_sel;
    const int mt_i = logical / units;
    const bool fuse_silu = fuse != 0 && proj == 1;
    const i32x4 tv = *reinterpret_cast<const i32x4*>(mtiles + mt_i);
    const int e = __builtin_amdgcn_readfirstlane(tv[0]);
    const int a_begin = __builtin_amdgcn_readfirstlane(tv[1]);
    const int rows = __builtin_amdgcn_readfirstlane(tv[2]);
    if (e < 0 || rows <= 0) return;
    const FastExpert fe = (proj ? up_fe : gate_fe)[e];
    const int max_slabs = proj ? up_max_slabs : gate_max_slabs;
    const FastSlab* __restrict__ fs_row = (proj ? up_fs : gate_fs) + (int64_t)e * max_slabs;
    const int nslabs = __builtin_amdgcn_readfirstlane(min(fe.num_slabs, max_slabs));
    const uint16_t* __restrict__ Hs = proj ? Hs_u : Hs_g;
    const int ld = proj ? ldu : ldg;
    uint16_t* __restrict__ out = (proj && !fuse_silu) ? U : G;
    const int w = __builtin_amdgcn_readfirstlane(fe.uniform_bits);
    // tiles of at most 32 / 64 / 96 assignments (experts that see few tokens, remainders) run a body
    // with a quarter / half / three quarters of the accumulators, MFMAs and staging; complete
    // bodies, so that no accumulator lives across the choice
    const DmaStage st0 = {sa0, sw0, ss0}, st1 = {sa1, sw1, ss1}, st2 = {sa2, sw2, ss2};
    BITSMOE_TLP(g_tl_pf_gateup, 1);
#define BITSMOE_GU_BODY(W)                                                                                           \
    do {                                                                                                             \
        if (rows <= 32)                                                                                              \
            gateup_tile_body_dma<DIRECT, W, 2>(fe, fs_row, nslabs, Hs, ld, token_indices, T, I, n_tiles, out,         \
                                               a_begin, rows, 2 * tp, st0, st1, st2, pack_tab, scale_tab, rank_tab, bits_tab, fuse_silu); \
        else if (rows <= 64)                                                                                         \
            gateup_tile_body_dma<DIRECT, W, 4>(fe, fs_row, nslabs, Hs, ld, token_indices, T, I, n_tiles, out,         \
                                               a_begin, rows, 2 * tp, st0, st1, st2, pack_tab, scale_tab, rank_tab, bits_tab, fuse_silu); \
        else if (rows <= 96)                                                                                         \
            gateup_tile_body_dma<DIRECT, W, 6>(fe, fs_row, nslabs, Hs, ld, token_indices, T, I, n_tiles, out,         \
                                               a_begin, rows, 2 * tp, st0, st1, st2, pack_tab, scale_tab, rank_tab, bits_tab, fuse_silu); \
        else                                                                                                         \
            gateup_tile_body_dma<DIRECT, W, 8>(fe, fs_row, nslabs, Hs, ld, token_indices, T, I, n_tiles, out,         \
                                               a_begin, rows, 2 * tp, st0, st1, st2, pack_tab, scale_tab, rank_tab, bits_tab, fuse_silu); \
    } while (0)
    // experts with more slabs than the tables hold take the register-staged body
#define BITSMOE_GU_BODY_MIXED()                                                                                      \
    do {                                                                                                             \
        if (rows <= 32)                                                                                              \
            gateup_tile_body<DIRECT, 0, 2>(fe, fs_row, nslabs, Hs, ld, token_indices, T, I, n_tiles, out, a_begin,    \
                                           rows, 2 * tp, sa0, sa1, fuse_silu);                                       \
        else                                                                                                         \
            gateup_tile_body<DIRECT, 0, 8>(fe, fs_row, nslabs, Hs, ld, token_indices, T, I, n_tiles, out, a_begin,    \
                                           rows, 2 * tp, sa0, sa1, fuse_silu);                                       \
    } while (0)
    if (nslabs > DMA_MAX_SLABS)
        BITSMOE_GU_BODY_MIXED();
    else if (w == 2)
        BITSMOE_GU_BODY(2);
    else if (w == 3)
        BITSMOE_GU_BODY(3);
    else if (w == 4)
        BITSMOE_GU_BODY(4);
    else
        BITSMOE_GU_BODY(0);
#undef BITSMOE_GU_BODY
#undef BITSMOE_GU_BODY_MIXED
    BITSMOE_TLP(g_tl_pf_gateup, 6);
}

// z = f16( silu(G) * U ), written over G; 8 elements per thread and iteration.
__global__ __launch_bounds__(256) void k_silu_mul_f16(uint16_t* __restrict__ G, const uint16_t* __restrict__ U, int64_t n8) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += (int64_t)gridDim.x * blockDim.x) {
        const u32x4 g = *reinterpret_cast<const u32x4*>(G + i * 8);
        const u32x4 u = *reinterpret_cast<const u32x4*>(U + i * 8);
        u32x4 o;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float g0 = __half2float(__ushort_as_half((uint16_t)(g[k] & 0xFFFFu)));
            const float g1 = __half2float(__ushort_as_half((uint16_t)(g[k] >> 16)));
            const float u0 = __half2float(__ushort_as_half((uint16_t)(u[k] & 0xFFFFu)));
            const float u1 = __half2float(__ushort_as_half((uint16_t)(u[k] >> 16)));
            const uint32_t lo = z_operand(g0, u0);
            const uint32_t hi = z_operand(g1, u1);
            o[k] = lo | (hi << 16);
        }
        *reinterpret_cast<u32x4*>(G + i * 8) = o;
    }
}

// ----------------------------------------------------------------------------------- down
constexpr int DN_SLABS_MFMA = 4;   // slabs (64 output rows each) per workgroup: one per wavefront

// Half a tile (64 columns = micro-tiles 2*HH, 2*HH+1) of one (slab, tile) block for a
// wavefront's 128 assignments x 64 output rows.  scp: this lane's row scale in both halves of a
// pair, per 16-row block.  The weight operand is (code - 2^(W-1)) * scale rounded once to f16,
// the operand the reference builds (bitsmoe/algorithms/cpp/mlp_forward.cu:1554-1694).
template <int HH, int NMB>
__device__ __forceinline__ void down_half_mfma(int bits, const uint16_t* stage, const Block16& blk,
                                      const uint32_t (&scp)[4], int lane, f32x4 (&acc)[NMB][4]) {
    const int n = lane & 15, kg = lane >> 4;
#pragma unroll
    for (int km = 0; km < 2; ++km) {
        const int m = 2 * HH + km;
        u32x4 a[NMB];
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb)
            a[mb] = *reinterpret_cast<const u32x4*>(stage + dma_chunk_off(16 * mb + n, 4 * km + kg));
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
            // the width switch wraps one operand only: accumulators that flow through alternative
            // paths multiply the register demand
            u32x4 b;
            uint32_t off;
            if (bits == 2) {
                b = decode_fields2<2, false>(blk.w[nb * 2 + HH], 8 * km);
                off = neg_offset_pair<2>();
            } else if (bits == 4) {
                b = decode_fields4<false>(blk.w[nb * 4 + m]);
                off = neg_offset_pair<4>();
            } else {
                b = decode_r1w3<false>(blk.w, nb, m);
                off = neg_offset_pair<3>();
            }
            for (int i = 0; i < 4; ++i) b[i] = pk_mul_f16(pk_add_f16(b[i], off), scp[nb]);
#pragma unroll
            for (int mb = 0; mb < NMB; ++mb) acc[mb][nb] = mfma16<false>(a[mb], b, acc[mb][nb]);
        }
    }
}

constexpr int DN_WBUF = 1024;    // 32-bit words: the payload block of one (slab, tile) as its wavefront fetches it
constexpr int DN_SBUF = 64;      // 16-bit scales of one (slab, tile) block

// The column loop of one wavefront (fs.bits == 0: no slab, the wavefront only helps to stage).
// Everything comes straight from global memory into LDS (LDS-direct loads, no registers in
// between): the pieces of z (128 assignments x 64 columns, chunk order of dma_chunk_off) into a
// ring of three stages shared by the workgroup, two pieces ahead of the MFMAs; the payload block
// and scales of the wavefront's next tile into a buffer of its own, from where they are taken
// into registers when the tile begins.  The loads of a wavefront complete in order and every
// wavefront issues the same number per step (four 16-byte payload loads whatever the width:
// narrower blocks repeat an address), so "piece h + 1 has landed" is a count of outstanding
// loads, waited for with a bare s_waitcnt before a bare barrier.
template <int NMB>
__device__ __forceinline__ void down_tile_loop(const uint32_t* __restrict__ payload, const __half* __restrict__ scale,
                                      const FastSlab fs, const uint16_t* __restrict__ z, int I, int n_tiles, int a_begin, int rows,
                                      uint16_t* st0, uint16_t* st1, uint16_t* st2, uint32_t* wbuf_all,
                                      uint16_t* sbuf_all, int tid, int lane, f32x4 (&acc)[NMB][4]) {
    constexpr int NJ = (NMB + 1) / 2;      // 32-row groups that hold assignments
    constexpr int NP = 5;                  // payload and scale load instructions per tile
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;
    const int W = fs.bits;
    uint32_t* wbuf = wbuf_all + wave * DN_WBUF;
    uint16_t* sbuf = sbuf_all + wave * DN_SBUF;
    // this lane lands in row r0 + 32*j, chunk position tid % 8 of a stage and fetches the chunk
    // that belongs there
    const int r0 = tid >> 3;
    const int cpos = (tid & 7) ^ ((r0 >> 1) & 7);
    uint32_t rowbase[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
        rowbase[j] = (uint32_t)(a_begin + min(r0 + 32 * j, rows - 1)) * (uint32_t)I + (uint32_t)(8 * cpos);
    auto request_z = [&](uint16_t* st, int h) {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
            load_to_lds16(z + (rowbase[j] + (uint32_t)(64 * h)), st + j * 2048 + wave * 512);
    };
    // role 1 block: 2-bit 8 words per lane, 4-bit 16, 3-bit 13 (three regions of four words per lane, the
    // thirteenth in a region of its own: four lanes fetch the same 16 bytes and each keeps its word)
    // (fast_helpers.h, wave_layout.h); load i fills words 4i .. 4i+3 of every lane's sixteen
    const uint32_t lane_words = (uint32_t)lane * (W == 4 ? 16u : W == 2 ? 8u : 4u);
    auto request_b = [&](int t) {
        const uint32_t base = W != 0 ? (uint32_t)(fs.pack_off + t * block_words(ROLE_DOWN, W)) : 0u;
        const uint32_t o0 = base + lane_words;
        const uint32_t o1 = W == 3 ? o0 + 256u : W != 0 ? o0 + 4u : o0;
        const uint32_t o2 = W == 4 ? o0 + 8u : W == 3 ? o0 + 512u : o0;
        const uint32_t o3 = W == 4 ? o0 + 12u : W == 3 ? base + 768u + (uint32_t)(lane & ~3) : o0;
        load_to_lds16(payload + o0, wbuf);
        load_to_lds16(payload + o1, wbuf + 256);
        load_to_lds16(payload + o2, wbuf + 512);
        load_to_lds16(payload + o3, wbuf + 768);
        const uint32_t so = W != 0 ? (uint32_t)(fs.scale_off + t * SLAB_ROWS) : 0u;
        if (lane < 8) load_to_lds16(scale + (so + (uint32_t)lane * 8u), sbuf);
    };
    Block16 blk;
    uint32_t scp[4];
    auto take_b = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const u32x4 v = *reinterpret_cast<const u32x4*>(wbuf + i * 256 + lane * 4);
            blk.w[4 * i] = v[0];
            blk.w[4 * i + 1] = v[1];
            blk.w[4 * i + 2] = v[2];
            blk.w[4 * i + 3] = v[3];
        }
        if (W == 3) {      // the thirteenth word: this lane's of the four its load brought
            const int k = lane & 3;
            blk.w[12] = k == 0 ? blk.w[12] : k == 1 ? blk.w[13] : k == 2 ? blk.w[14] : blk.w[15];
        }
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) scp[nb] = (uint32_t)sbuf[16 * nb + n] * 0x10001u;
        // the buffer is requested again right away: its reads must have returned
        wait_lds_reads();
        asm volatile("" ::: "memory");
    };
    const int n_halves = 2 * n_tiles;      // at least two
    request_z(st0, 0);
    request_b(0);
    request_z(st1, 1);
    wait_vmcnt<NJ>();                      // block 0 and piece 0 have landed
    barrier_no_drain();
    BITSMOE_TLP(g_tl_pf_down, 2);
    // step h (h % 3 == U, h % 2 == HH): (first half of a tile) the tile's block taken into
    // registers; piece h + 2 requested into the stage piece h - 1 used, then (first half) the next
    // tile's block; piece h multiplied
    auto step = [&](auto u_c, auto hh_c, int h) {
        constexpr int U = decltype(u_c)::value;
        constexpr int HH = decltype(hh_c)::value;
        // (the stages are named statically, so that the compiler can tell the stage being read
        // from the ones being loaded)
        uint16_t* cur = U == 0 ? st0 : U == 1 ? st1 : st2;
        uint16_t* nxt = U == 0 ? st2 : U == 1 ? st0 : st1;
        const bool more = h + 2 < n_halves;
        if (HH == 0) take_b();
        if (more) {
            request_z(nxt, h + 2);
            if (HH == 0) request_b((h >> 1) + 1);      // h + 2 < n_halves: there is a next tile
        }
        if (W != 0) down_half_mfma<HH, NMB>(W, cur, blk, scp, lane, acc);
        asm volatile("" ::: "memory");
        // piece h + 1 (and, after a second half, the next tile's block) must have landed; what this
        // step requested may still be in flight
        if (!more)
            wait_vmcnt<0>();
        else if (HH == 0)
            wait_vmcnt<NJ + NP>();
        else
            wait_vmcnt<NJ>();
        barrier_no_drain();
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    for (int h0 = 0; h0 < n_halves; h0 += 6) {
        step(I0{}, I0{}, h0);
        step(I1{}, I1{}, h0 + 1);
        if (h0 + 2 < n_halves) {
            step(I2{}, I0{}, h0 + 2);
            step(I0{}, I1{}, h0 + 3);
        }
        if (h0 + 4 < n_halves) {
            step(I1{}, I0{}, h0 + 4);
            step(I2{}, I1{}, h0 + 5);
        }
    }
}

// grid.x = 32 * ceil(max_mtiles / 32) * n_groups; workgroup = (assignment tile, group of four
// slabs): wavefront w = all 128 assignments x the 64 output rows of slab 4*group + w.
// Output: y[a, r] = s[r] * sum_c W_down[r, c] z[a, c] as f16, r in the expert's own row order
// (row `A` of y takes the stores of a tile's unused rows), and the per-token assignment lists
// token_list[token_start[tok_a] + slot[a]] = (a, expert) that k_combine_tokens walks.
__global__ __launch_bounds__(256, 2) void k_down_mfma(const FastExpert* __restrict__ down_fe,
                                                      const FastSlab* __restrict__ down_fs, int max_slabs,
                                                      const uint16_t* __restrict__ z, const MTile* __restrict__ mtiles,
                                                      const int32_t* __restrict__ n_mtiles,
                                                      const int32_t* __restrict__ token_indices,
                                                      const int32_t* __restrict__ slot,
                                                      const int32_t* __restrict__ token_start,
                                                      int2* __restrict__ token_list, int A, int I, int n_tiles,
                                                      int n_groups, _Float16* __restrict__ y, int ldy) {
    __shared__ __attribute__((aligned(16))) uint16_t sz0[DMA_STAGE], sz1[DMA_STAGE], sz2[DMA_STAGE];
    __shared__ __attribute__((aligned(16))) uint32_t wbuf[4 * DN_WBUF];
    __shared__ __attribute__((aligned(16))) uint16_t sbuf[4 * DN_SBUF];
    BITSMOE_TLP(g_tl_pf_down, 0);
    const int logical = xcd_logical(blockIdx.x, __builtin_amdgcn_readfirstlane(*n_mtiles), n_groups);
    if (logical < 0) return;
    const int mt_i = logical / n_groups, grp = logical - mt_i * n_groups;
    const i32x4 tv = *reinterpret_cast<const i32x4*>(mtiles + mt_i);
    const int e = __builtin_amdgcn_readfirstlane(tv[0]);
    const int a_begin = __builtin_amdgcn_readfirstlane(tv[1]);
    const int rows = __builtin_amdgcn_readfirstlane(tv[2]);
    if (e < 0 || rows <= 0) return;
    const int tid = threadIdx.x;
    if (grp == 0 && tid < rows) {
        const int a = a_begin + tid;
        const int sl = slot[a];
        if (sl >= 0) token_list[token_start[token_indices[a]] + sl] = int2{a, e};
    }
    const FastExpert fe = down_fe[e];
    const int nslabs = __builtin_amdgcn_readfirstlane(min(fe.num_slabs, max_slabs));
    if (DN_SLABS_MFMA * grp >= nslabs) return;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, kg = lane >> 4;
    const int si = DN_SLABS_MFMA * grp + wave;
    FastSlab fs = FastSlab{0, 0, 0, 0};
    if (si < nslabs) fs = load_fast_slab(down_fs + (int64_t)e * max_slabs, si);
    BITSMOE_TLP(g_tl_pf_down, 1);

    // tiles of at most 32 / 64 / 96 assignments run a body with a quarter / half / three quarters of
    // the accumulators and MFMAs: complete bodies, so that no accumulator lives across the choice
    auto run = [&](auto nmb_c) {
        constexpr int NMB = decltype(nmb_c)::value;
        f32x4 acc[NMB][4];
#pragma unroll
        for (int i = 0; i < NMB; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0, 0, 0, 0};
        // wavefronts without a slab skip the MFMAs; all execute the same barriers
        down_tile_loop<NMB>(fe.payload, fe.scale, fs, z, I, n_tiles, a_begin, rows, sz0, sz1, sz2, wbuf, sbuf, tid, lane, acc);
        BITSMOE_TLP(g_tl_pf_down, 3);
        if (fs.bits == 0) return;

        // lane holds assignments 16*mb + 4*kg + j, output rows 16*nb + n of the slab; the rows'
        // multipliers s[r] go into y here, so that the combine reads one operand per assignment
        float srow[4];
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) srow[nb] = __half2float(fe.s[fs.rank_off + 16 * nb + n]);
        _Float16* ycol = y + fs.rank_off + n;
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb) {
            if (16 * mb >= rows) break;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int r = 16 * mb + 4 * kg + j;
                _Float16* dst = ycol + (int64_t)(r < rows ? a_begin + r : A) * ldy;
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) dst[16 * nb] = (_Float16)(acc[mb][nb][j] * srow[nb]);
            }
        }
    };
    if (rows <= 32)
        run(std::integral_constant<int, 2>{});
    else if (rows <= 64)
        run(std::integral_constant<int, 4>{});
    else if (rows <= 96)
        run(std::integral_constant<int, 6>{});
    else
        run(std::integral_constant<int, 8>{});
    BITSMOE_TLP(g_tl_pf_down, 6);
}

// ------------------------------------------------------------------------------- combine
constexpr int CB_COLS = 4096;    // output columns one pass of the general form accumulates in LDS
constexpr int CB_SORT = 256;     // list entries ordered at a time

// rank_accum[t, rank_idx_e[r]] = sum over the assignments (a, e) of token t, in ascending a,
// of route_w[a] * y[a, r] (y carries the row multiplier s_e[r]).  One workgroup per token; it writes every column of its
// row, so rank_accum needs no zero fill.  IDENTITY: rank_idx_e[r] == r in every expert, and a
// thread keeps its eight columns in registers; otherwise the row is accumulated in LDS, one
// assignment after the other.
template <bool IDENTITY>
__global__ __launch_bounds__(256) void k_combine_tokens(const FastExpert* __restrict__ down_fe, int max_slabs,
                                                        const _Float16* __restrict__ y, int ldy,
                                                        const int32_t* __restrict__ token_start,
                                                        const int32_t* __restrict__ token_count,
                                                        const int2* __restrict__ token_list,
                                                        const float* __restrict__ route_w, int rank_out,
                                                        float* __restrict__ rank_accum) {
    __shared__ __attribute__((aligned(16))) float out_s[IDENTITY ? 4 : CB_COLS];
    __shared__ int2 raw_s[CB_SORT];
    __shared__ const _Float16* y_s[CB_SORT];
    __shared__ const int32_t* idx_s[CB_SORT];
    __shared__ int nrow_s[CB_SORT];
    __shared__ float rw_s[CB_SORT];
    const int t = blockIdx.x;
    const int tid = threadIdx.x;
    // (token_count given: lists of a fixed stride, only partly filled)
    const int begin = token_start[t], count = token_count ? token_count[t] : token_start[t + 1] - begin;
    float* out_row = rank_accum + (int64_t)t * rank_out;
    constexpr int STEP = IDENTITY ? 256 * 8 : CB_COLS;
    for (int c0 = 0; c0 < rank_out; c0 += STEP) {
        const int cols = min(STEP, rank_out - c0);
        float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        if (!IDENTITY)
            for (int i = tid; i < cols; i += 256) out_s[i] = 0.0f;
        for (int l0 = 0; l0 < count; l0 += CB_SORT) {
            const int nl = min(CB_SORT, count - l0);
            __syncthreads();
            if (tid < nl) raw_s[tid] = token_list[begin + l0 + tid];
            __syncthreads();
            if (tid < nl) {      // the lists were filled in arbitrary order: sort by assignment
                const int2 mine = raw_s[tid];
                int pos = 0;
                for (int i = 0; i < nl; ++i) pos += raw_s[i].x < mine.x;
                const FastExpert fe = down_fe[mine.y];
                y_s[pos] = y + (int64_t)mine.x * ldy;
                idx_s[pos] = fe.rank_idx;
                nrow_s[pos] = min(fe.num_slabs, max_slabs) * SLAB_ROWS;
                rw_s[pos] = route_w[mine.x];
            }
            __syncthreads();
            if (IDENTITY) {
                const int r0 = c0 + tid * 8;
                // eight entries at a time: their loads are in flight together (an entry past
                // the list or past its expert's rows loads from a valid address and is not added)
                constexpr int CB_FLIGHT = 8;
                for (int i0 = 0; i0 < nl; i0 += CB_FLIGHT) {
                    u32x4 yv[CB_FLIGHT];
                    float rw[CB_FLIGHT];
                    bool ok[CB_FLIGHT];
#pragma unroll
                    for (int u = 0; u < CB_FLIGHT; ++u) {
                        const int i = min(i0 + u, nl - 1);
                        ok[u] = i0 + u < nl && r0 < nrow_s[i];
                        const int rr = ok[u] ? r0 : 0;
                        yv[u] = *reinterpret_cast<const u32x4*>(y_s[i] + rr);
                        rw[u] = rw_s[i];
                    }
#pragma unroll
                    for (int u = 0; u < CB_FLIGHT; ++u) {
                        if (!ok[u]) continue;
#pragma unroll
                        for (int k = 0; k < 8; ++k) {
                            const uint32_t yw = yv[u][k >> 1];
                            const h2 yp = __builtin_bit_cast(h2, yw);
                            acc[k] += (float)yp[k & 1] * rw[u];
                        }
                    }
                }
            } else {
                for (int i = 0; i < nl; ++i) {
                    const int nrow = nrow_s[i];
                    const float rw = rw_s[i];
                    gptr<int32_t> rank_idx = as_global(idx_s[i]);
                    const _Float16* yrow = y_s[i];
                    for (int r0 = tid * 8; r0 < nrow; r0 += 256 * 8) {
                        const u32x4 yv = *reinterpret_cast<const u32x4*>(yrow + r0);
                        const i32x4 ia = *reinterpret_cast<gptr<i32x4>>(rank_idx + r0);
                        const i32x4 ib = *reinterpret_cast<gptr<i32x4>>(rank_idx + r0 + 4);
#pragma unroll
                        for (int k = 0; k < 8; ++k) {
                            const uint32_t yw = yv[k >> 1];
                            const h2 yp = __builtin_bit_cast(h2, yw);
                            const int col = (k < 4 ? ia[k & 3] : ib[k & 3]) - c0;
                            if (col >= 0 && col < cols) atomicAdd(out_s + col, (float)yp[k & 1] * rw);
                        }
                    }
                    __syncthreads();    // entries are added one after the other: the sum has one order
                }
            }
        }
        if (IDENTITY) {
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (tid * 8 + k < cols) out_row[c0 + tid * 8 + k] = acc[k];
        } else {
            __syncthreads();
            for (int i = tid; i < cols; i += 256) out_row[c0 + i] = out_s[i];
            __syncthreads();
        }
    }
}

// ---------------------------------------------------------------------------------- host
static inline size_t align256(size_t v) { return (v + 255) / 256 * 256; }
static inline void record(bitsmoe_profile* p, int i, hipStream_t st) {
    if (p) (void)hipEventRecord(p->ev[i], st);
}

bool mfma_path_supported(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down, int I) {
    (void)I;
    return gate->role == ROLE_GATE_UP && up->role == ROLE_GATE_UP && down->role == ROLE_DOWN &&
           gate->vector_aligned && up->vector_aligned && down->vector_aligned;
}

// Can the gate/up kernel read activation rows through the token index (no pre-gather)?
static bool direct_ok(const bitsmoe_matset* gate, const bitsmoe_matset* up) {
    return gate->rank_chunked8 && up->rank_chunked8 && gate->d_scale_s && up->d_scale_s;
}
// (columns of the f16 copy of bf16 activations: every rank the prepared rank table names, padding rows included)
static inline int direct_ld(const bitsmoe_matset* set) { return (set->pad_rank_plus1 + 7) / 8 * 8; }

// Carving of the workspace, shared by the size query and the launcher.
struct MfmaWorkspace {
    size_t mtiles, n_mtiles, token_count, token_start, slot, token_list, acts, z, u, y, total;
};
static MfmaWorkspace mfma_workspace(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                                    int64_t T, int64_t A, int I) {
    const int64_t max_mtiles = A / PF_M + gate->n_experts;
    const size_t direct = align256((size_t)T * direct_ld(gate) * 2) + align256((size_t)T * direct_ld(up) * 2);
    const size_t gathered = align256((size_t)A * gate->prep_max_slabs * SLAB_ROWS * 2) + align256((size_t)A * up->prep_max_slabs * SLAB_ROWS * 2);
    MfmaWorkspace w;
    size_t at = 0;
    auto take = [&](size_t bytes) { const size_t here = at; at += align256(bytes); return here; };
    w.mtiles = take((size_t)max_mtiles * sizeof(MTile));
    w.n_mtiles = take(256);
    w.token_count = take((size_t)(T + 1) * 4);
    w.token_start = take((size_t)(T + 1) * 4);
    w.slot = take((size_t)A * 4);
    w.token_list = take((size_t)A * 8);
    // the direct form falls back to the gathered one when the activation pointers or row
    // lengths do not allow 16-byte loads, which is only known at the call
    w.acts = take(std::max(direct_ok(gate, up) ? direct : 0, gathered));
    w.z = take((size_t)A * I * 2);
    w.u = take((size_t)A * I * 2);
    w.y = take((size_t)(A + 1) * down->prep_max_slabs * SLAB_ROWS * 2);
    w.total = at;
    return w;
}

size_t mfma_workspace_bytes(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down, int64_t T,
                            int64_t A, int I) {
    return mfma_workspace(gate, up, down, T, A, I).total;
}

// How the gate/up kernel gets its activations: `direct`: rows read through the token index (from the caller's f16
// rows, or from an f16 copy of bf16 rows: `convert`), else gathered per assignment; ldg / ldu: elements per row of
// what the kernel reads.
struct ActsPlan {
    bool direct, convert;
    int ldg, ldu;
};
static ActsPlan acts_plan(const bitsmoe_matset* gate, const bitsmoe_matset* up, const void* h_gate, const void* h_up,
                          int act_dtype, int64_t T, int Rg, int Ru, int64_t ldg_in, int64_t ldu_in) {
    // ldg_in / ldu_in: elements between the caller's activation rows (>= Rg / Ru)
    // (padding rows have zero scales but their activations are still read and multiplied: every rank they
    // name has to be a column of h)
    ActsPlan p;
    p.direct = direct_ok(gate, up) && Rg % 8 == 0 && Ru % 8 == 0 && ldg_in % 8 == 0 && ldu_in % 8 == 0 &&
               gate->pad_rank_plus1 <= Rg && up->pad_rank_plus1 <= Ru && (((uintptr_t)h_gate | (uintptr_t)h_up) & 15) == 0 &&
               T * std::max(ldg_in, ldu_in) < ((int64_t)1 << 31);
    p.convert = p.direct && act_dtype == BITSMOE_DT_BF16;
    p.ldg = p.direct ? (p.convert ? direct_ld(gate) : (int)ldg_in) : gate->prep_max_slabs * SLAB_ROWS;
    p.ldu = p.direct ? (p.convert ? direct_ld(up) : (int)ldu_in) : up->prep_max_slabs * SLAB_ROWS;
    return p;
}
static inline size_t acts_up_offset(const bitsmoe_matset* gate, const ActsPlan& p, int64_t T, int64_t A) {
    return p.direct ? align256((size_t)T * direct_ld(gate) * 2) : align256((size_t)A * p.ldg * 2);
}

bool mfma_front_jobs(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                     const void* h_gate, const void* h_up, int act_dtype, int64_t T, int Rg, int Ru, int64_t ldg_in,
                     int64_t ldu_in, int64_t A, int I, void* workspace, RouteSideJobs* jobs) {
    const ActsPlan p = acts_plan(gate, up, h_gate, h_up, act_dtype, T, Rg, Ru, ldg_in, ldu_in);
    const MfmaWorkspace w = mfma_workspace(gate, up, down, T, A, I);
    char* ws = (char*)workspace;
    *jobs = RouteSideJobs{};
    jobs->T = T;
    if (p.convert) {
        jobs->src_g = (const uint16_t*)h_gate;
        jobs->src_u = (const uint16_t*)h_up;
        jobs->sg = ldg_in;
        jobs->su = ldu_in;
        jobs->ldg = p.ldg;
        jobs->ldu = p.ldu;
        jobs->dst_g = (uint16_t*)(ws + w.acts);
        jobs->dst_u = (uint16_t*)(ws + w.acts + acts_up_offset(gate, p, T, A));
    }
    jobs->slot = (int32_t*)(ws + w.slot);
    jobs->token_count = (int32_t*)(ws + w.token_count);
    jobs->token_start = (int32_t*)(ws + w.token_start);
    jobs->mtiles = (MTile*)(ws + w.mtiles);
    jobs->n_mtiles = (int32_t*)(ws + w.n_mtiles);
    jobs->max_mtiles = (int)(A / PF_M + gate->n_experts);
    jobs->gate_fe = gate->d_fast_experts;
    jobs->up_fe = up->d_fast_experts;
    return true;
}

int launch_forward_mfma(const bitsmoe_matset* gate, const bitsmoe_matset* up, const bitsmoe_matset* down,
                        const void* h_gate, const void* h_up, int act_dtype, int64_t T, int Rg, int Ru, int64_t ldg_in,
                        int64_t ldu_in, const int32_t* tok, const int32_t* off, const float* rw, int64_t A, int rank_out,
                        int I, float* rank_accum, void* workspace, int front_done, bitsmoe_profile* prof, hipStream_t st) {
    const int E = gate->n_experts;
    const int n_tiles = gate->n_tiles;
    const int64_t max_mtiles = A / PF_M + E;
    const ActsPlan plan = acts_plan(gate, up, h_gate, h_up, act_dtype, T, Rg, Ru, ldg_in, ldu_in);
    const bool direct = plan.direct;
    const int ldg = plan.ldg, ldu = plan.ldu;
    const MfmaWorkspace w = mfma_workspace(gate, up, down, T, A, I);
    char* ws = (char*)workspace;
    MTile* mtiles = (MTile*)(ws + w.mtiles);
    int32_t* n_mtiles = (int32_t*)(ws + w.n_mtiles);
    int32_t* token_count = (int32_t*)(ws + w.token_count);
    int32_t* token_start = (int32_t*)(ws + w.token_start);
    int32_t* slot = (int32_t*)(ws + w.slot);
    int2* token_list = (int2*)(ws + w.token_list);
    const uint16_t* Hs_g = (const uint16_t*)(ws + w.acts);
    const uint16_t* Hs_u = (const uint16_t*)(ws + w.acts + acts_up_offset(gate, plan, T, A));
    uint16_t* z = (uint16_t*)(ws + w.z);     // gate output, then silu(gate) * up in place
    uint16_t* Ubuf = (uint16_t*)(ws + w.u);
    _Float16* y = (_Float16*)(ws + w.y);
    const int ldy = down->prep_max_slabs * SLAB_ROWS;

    record(prof, 0, st);
    const bool convert = plan.convert;
    // slot, token_count, token_start (fixed stride: the lists' lengths come from token_count) and the tile list are
    // there already
    const bool counted = (front_done & MFMA_FRONT_TOKEN_COUNTED) != 0 && (front_done & MFMA_FRONT_MTILES) != 0;
    if (convert && !(front_done & MFMA_FRONT_CONVERTED)) {      // the conversion pass clears the per-token counters on its way
        const int64_t groups = T * (std::max(ldg, ldu) / 8);
        hipLaunchKernelGGL(k_bf16_to_f16, dim3((unsigned)std::min<int64_t>((groups + 255) / 256, 2048), 2), dim3(256), 0, st,
                           (const uint16_t*)h_gate, (const uint16_t*)h_up, T, ldg_in, ldu_in, ldg, ldu, (uint16_t*)Hs_g,
                           (uint16_t*)Hs_u, token_count, counted ? 0 : (int)(T + 1));
        BITSMOE_HIP_TRY(hipGetLastError());
    } else if (!counted) {
        BITSMOE_REQUIRE(launch_fill_zero((float*)token_count, T + 1, st) == BITSMOE_OK, "zero fill failed");
    }
    if (!counted)
        hipLaunchKernelGGL(k_token_count, dim3((unsigned)((A + 255) / 256)), dim3(256), 0, st, tok, off, E, (int)A, (int)T,
                           token_count, slot);
    if (!counted)
        hipLaunchKernelGGL(k_build_mtiles, dim3(1), dim3(256), 0, st, off, E, (int)A, (int)max_mtiles, mtiles, n_mtiles,
                           token_count, (int)T, token_start, gate->d_fast_experts, up->d_fast_experts);
    BITSMOE_HIP_TRY(hipGetLastError());
    if (direct) {
        if (!convert) {
            Hs_g = (const uint16_t*)h_gate;
            Hs_u = (const uint16_t*)h_up;
        }
    } else {
        dim3 grid((unsigned)((A + 3) / 4), 2);
        if (act_dtype == BITSMOE_DT_BF16)
            hipLaunchKernelGGL((k_pregather<true>), grid, dim3(256), 0, st, gate->d_fast_experts, up->d_fast_experts,
                               (const uint16_t*)h_gate, (const uint16_t*)h_up, Rg, Ru, ldg_in, ldu_in, tok, off, E, (int)T, (int)A,
                               (uint16_t*)Hs_g, (uint16_t*)Hs_u, ldg, ldu);
        else
            hipLaunchKernelGGL((k_pregather<false>), grid, dim3(256), 0, st, gate->d_fast_experts, up->d_fast_experts,
                               (const uint16_t*)h_gate, (const uint16_t*)h_up, Rg, Ru, ldg_in, ldu_in, tok, off, E, (int)T, (int)A,
                               (uint16_t*)Hs_g, (uint16_t*)Hs_u, ldg, ldu);
        BITSMOE_HIP_TRY(hipGetLastError());
    }
    record(prof, 1, st);
    {
        const int n_tp = (n_tiles + 1) / 2;
        // One launch for both projections and a SiLU pass behind it.  Option prefill_split = 1: two launches, gate
        // then up, the up launch's epilogue storing z = silu(gate) * up over the gate sums (the up sums never reach
        // memory, no SiLU pass).  Measured at 4096 tokens on the 128-expert layer: 241 us for the two launches against
        // 202 + 25 us -- two half-size grids end in two tails, and the epilogue waits for the gate sums -- so it is
        // off unless asked for.
        const bool wide_gu = has_wide_rows(gate) || has_wide_rows(up);
        const bool split = options().prefill_split > 0 && !wide_gu;      // (the side kernel adds to the sums before SiLU)
        auto launch = [&](auto kernel, int proj_sel, int fuse) -> hipError_t {
            const int64_t wgs = (max_mtiles + 31) / 32 * 32 * (proj_sel < 0 ? 2 : 1) * n_tp;
            hipLaunchKernelGGL(kernel, dim3((unsigned)wgs), dim3(256), 0, st, gate->d_fast_experts, gate->d_fast_slabs,
                               gate->prep_max_slabs, up->d_fast_experts, up->d_fast_slabs, up->prep_max_slabs, Hs_g, Hs_u, ldg, ldu, tok,
                               (int)T, mtiles, n_mtiles, I, n_tiles, z, Ubuf, proj_sel, fuse);
            return hipGetLastError();
        };
        if (split) {
            BITSMOE_HIP_TRY(direct ? launch(k_gateup_mfma<true>, 0, 0) : launch(k_gateup_mfma<false>, 0, 0));
            BITSMOE_HIP_TRY(direct ? launch(k_gateup_mfma<true>, 1, 1) : launch(k_gateup_mfma<false>, 1, 1));
            record(prof, 2, st);
        } else {
            BITSMOE_HIP_TRY(direct ? launch(k_gateup_mfma<true>, -1, 0) : launch(k_gateup_mfma<false>, -1, 0));
            if (wide_gu) {      // rows of 6-, 8- and 16-bit slabs: their share of the (f16) gate and up sums
                const int rc = launch_wide_gateup(gate, up, h_gate, h_up, act_dtype, Rg, Ru, ldg_in, ldu_in, tok, off, A, I, z, Ubuf,
                                                  true, st);
                if (rc != BITSMOE_OK) return rc;
            }
            record(prof, 2, st);
            const int64_t n8 = A * (int64_t)I / 8;
            hipLaunchKernelGGL(k_silu_mul_f16, dim3((unsigned)std::min<int64_t>((n8 + 255) / 256, 4096)), dim3(256), 0, st, z,
                               Ubuf, n8);
            BITSMOE_HIP_TRY(hipGetLastError());
        }
    }
    record(prof, 3, st);
    {
        const int n_pairs = (down->prep_max_slabs + DN_SLABS_MFMA - 1) / DN_SLABS_MFMA;
        const int64_t wgs = (max_mtiles + 31) / 32 * 32 * n_pairs;
        hipLaunchKernelGGL(k_down_mfma, dim3((unsigned)wgs), dim3(256), 0, st, down->d_fast_experts, down->d_fast_slabs,
                           down->prep_max_slabs, z, mtiles, n_mtiles, tok, slot, token_start, token_list, (int)A, I, n_tiles,
                           n_pairs, y, ldy);
        record(prof, 4, st);
        if (down->rank_identity)
            hipLaunchKernelGGL(k_combine_tokens<true>, dim3((unsigned)T), dim3(256), 0, st, down->d_fast_experts,
                               down->prep_max_slabs, y, ldy, token_start, counted ? token_count : nullptr, token_list, rw,
                               rank_out, rank_accum);
        else
            hipLaunchKernelGGL(k_combine_tokens<false>, dim3((unsigned)T), dim3(256), 0, st, down->d_fast_experts,
                               down->prep_max_slabs, y, ldy, token_start, counted ? token_count : nullptr, token_list, rw,
                               rank_out, rank_accum);
        BITSMOE_HIP_TRY(hipGetLastError());
        if (has_wide_rows(down)) {      // (behind the combine, which writes every element of rank_accum)
            const int rc = launch_wide_down(down, z, nullptr, true, 1, 0, tok, off, rw, A, I, rank_out, rank_accum, st);
            if (rc != BITSMOE_OK) return rc;
        }
    }
    record(prof, 5, st);
    if (prof) prof->recorded = true;
    return BITSMOE_OK;
}

}  // namespace bitsmoe

#ifdef BITSMOE_TIMELINE
// which: 0 = k_gateup_mfma, 1 = k_down_mfma
extern "C" int bitsmoe_timeline_read_prefill(int which, unsigned long long* host, int n_workgroups) {
    using namespace bitsmoe;
    if (!host || n_workgroups <= 0 || n_workgroups > TLP_MAX_WG || which < 0 || which > 1) return BITSMOE_E_INVALID;
    BITSMOE_HIP_TRY(hipDeviceSynchronize());
    const size_t bytes = sizeof(unsigned long long) * TLP_STAMPS * n_workgroups;
    if (which == 0)
        BITSMOE_HIP_TRY(hipMemcpyFromSymbol(host, HIP_SYMBOL(g_tl_pf_gateup), bytes));
    else
        BITSMOE_HIP_TRY(hipMemcpyFromSymbol(host, HIP_SYMBOL(g_tl_pf_down), bytes));
    return BITSMOE_OK;
}
extern "C" int bitsmoe_timeline_clear_prefill(void) {
    using namespace bitsmoe;
    void* p = nullptr;
    BITSMOE_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(g_tl_pf_gateup)));
    BITSMOE_HIP_TRY(hipMemset(p, 0, sizeof(unsigned long long) * TLP_STAMPS * TLP_MAX_WG));
    BITSMOE_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(g_tl_pf_down)));
    BITSMOE_HIP_TRY(hipMemset(p, 0, sizeof(unsigned long long) * TLP_STAMPS * TLP_MAX_WG));
    return BITSMOE_OK;
}
#endif
