// One-time re-layout of a matrix set's payload into the wave64-native field layout
// (wave_layout.h) and the dense dequantiser that reads it back (parity check of the layout).
#include "wave_layout.h"

#include <algorithm>
#include <cstring>

namespace bitsmoe {

// code (unsigned, before the level offset) of element (row, col) of a (slab, tile) block
// in the reference bit-plane layout; `blk` points at the block's first word, rows = 64.
__device__ inline uint32_t ref_code(const uint32_t* __restrict__ blk, int w, int row, int col) {
    const int stage = row >> 4, r = row & 15, micro = col >> 5, lane = col & 31;
    const uint32_t* words = blk + stage * (K_STAGE * MICROS * w) + micro * (K_STAGE * w) + r * w;
    uint32_t u = 0;
    for (int p = 0; p < w; ++p) u |= ((words[p] >> lane) & 1u) << p;
    return u;
}

// (row, col) of contraction index x of the run owned by (nb, kg, n)
__device__ inline void run_element(int role, int nb, int kg, int n, int x, int* row, int* col) {
    if (role == ROLE_GATE_UP) {          // 16 rows 16*kg + x, column 16*nb + n
        *row = 16 * kg + x;
        *col = 16 * nb + n;
    } else {                              // row 16*nb + n, columns 32*(x/8) + 8*kg + x%8
        *row = 16 * nb + n;
        *col = 32 * (x >> 3) + 8 * kg + (x & 7);
    }
}

// grid: (slab tasks, tiles); every thread builds whole output words of one block.
__global__ __launch_bounds__(256) void k_prepack(const MatView* __restrict__ src, const MatView* __restrict__ dst,
                                                 const SlabTask* __restrict__ tasks, int role) {
    const SlabTask task = tasks[blockIdx.x];
    const MatView mv = src[task.expert];
    const int si = task.slab;
    const int w = mv.slab_meta[si * 4 + 0];
    const int tile_off = mv.slab_meta[si * 4 + 3];
    const int t = tile_off + blockIdx.y;
    const int pack_off = mv.tile_meta[t * 3 + 0];
    const uint32_t* __restrict__ in = mv.payload + pack_off;
    uint32_t* __restrict__ out = const_cast<uint32_t*>(dst[task.expert].payload) + pack_off;
    const int nbs = (role == ROLE_GATE_UP) ? 8 : 4;        // output blocks per lane
    const int run = (role == ROLE_GATE_UP) ? 16 : 32;      // contraction indices per (lane, nb)
    const int n_words = 256 * w;
    for (int idx = threadIdx.x; idx < n_words; idx += blockDim.x) {
        uint32_t word = 0;
        if (w == 3 && idx >= 512) {
            // third bit of the 3-bit codes
            const int j = idx - 512;
            if (role == ROLE_GATE_UP) {   // j = hi_index0(kg, n8, nb), shared by lanes n8 and n8 + 8
                const int q = (j >> 1) & 31;
                const int nb = 2 * (j >> 6) + (j & 1), n8 = q & 7, kg = q >> 3;
                for (int upper = 0; upper < 2; ++upper)
                    for (int x = 0; x < 16; ++x) {
                        int row, col;
                        run_element(role, nb, kg, n8 + 8 * upper, x, &row, &col);
                        word |= ((ref_code(in, w, row, col) >> 2) & 1u) << pos1s(x, upper);
                    }
            } else {                      // j = l*4 + nb
                const int nb = j & 3, l = j >> 2, n = l & 15, kg = l >> 4;
                for (int x = 0; x < 32; ++x) {
                    int row, col;
                    run_element(role, nb, kg, n, x, &row, &col);
                    word |= ((ref_code(in, w, row, col) >> 2) & 1u) << pos1(x);
                }
            }
            out[idx] = word;
            continue;
        }
        // two-bit / four-bit field words: words per (lane, nb) = run * fieldbits / 32
        const int fb = (w == 4) ? 4 : 2;
        const int per = run * fb / 32;                   // role0: 1 (w=2,3) or 2 (w=4); role1: 2 or 4
        const int sub = idx % per;
        int nb, l;
        if (role == ROLE_GATE_UP) {      // idx / per = idx2_role0(nb, l)
            const int i2 = idx / per;
            nb = 2 * (i2 >> 7) + (i2 & 1);
            l = (i2 >> 1) & 63;
        } else {
            nb = (idx / per) % nbs;
            l = idx / (per * nbs);
        }
        const int n = l & 15, kg = l >> 4;
        const int codes = 32 / fb;                       // codes per word
        for (int i = 0; i < codes; ++i) {
            const int x = sub * codes + i;
            int row, col;
            run_element(role, nb, kg, n, x, &row, &col);
            const uint32_t u = ref_code(in, w, row, col);
            if (role == ROLE_GATE_UP)      // staggered fields; one may wrap around bit 31
                word |= rotl32(fb == 4 ? (u & 15u) : (u & 3u), fb == 4 ? pos4s(i) : pos2s(w, i));
            else if (fb == 4)
                word |= (u & 15u) << pos4(i);
            else
                word |= (u & 3u) << pos2(i);
        }
        out[idx] = word;
    }
}

// Dense fp32 dequantisation FROM THE PREPARED LAYOUT, written to mirror the decode of the
// hot kernels (fields, not planes); output identical to k_dequant_matrix.
__global__ __launch_bounds__(256) void k_dequant_prepared(MatView mv /* payload = prepared */, int role, int I,
                                                          float* __restrict__ out) {
    const int si = blockIdx.x;
    const int w = mv.slab_meta[si * 4 + 0];
    const int rank_off = mv.slab_meta[si * 4 + 2];
    const int t = mv.slab_meta[si * 4 + 3] + blockIdx.y;
    const int pack_off = mv.tile_meta[t * 3 + 0];
    const int scale_off = mv.tile_meta[t * 3 + 1];
    const uint32_t* __restrict__ blk = mv.payload + pack_off;
    const int nbs = (role == ROLE_GATE_UP) ? 8 : 4;
    const int run = (role == ROLE_GATE_UP) ? 16 : 32;
    for (int idx = threadIdx.x; idx < SLAB_ROWS * N_TILE; idx += blockDim.x) {
        // enumerate (lane, nb, x) instead of (row, col) so the layout is read the way kernels read it
        const int x = idx % run;
        const int nb = (idx / run) % nbs;
        const int l = idx / (run * nbs);
        const int n = l & 15, kg = l >> 4;
        int row, col;
        run_element(role, nb, kg, n, x, &row, &col);
        uint32_t u;
        const int unit = (role == ROLE_GATE_UP) ? idx2_role0(nb, l) : (l * nbs + nb);
        if (w == 4) {
            const int per = run / 8;
            const uint32_t word = blk[unit * per + (x >> 3)];
            u = (role == ROLE_GATE_UP ? rotr32(word, pos4s(x & 7)) : word >> pos4(x & 7)) & 15u;
        } else {
            const int per = run / 16;
            const uint32_t word = blk[unit * per + (x >> 4)];
            u = (role == ROLE_GATE_UP ? rotr32(word, pos2s(w, x & 15)) : word >> pos2(x & 15)) & 3u;
            if (w == 3) {
                uint32_t hi;
                int p;
                if (role == ROLE_GATE_UP) {
                    hi = blk[512 + hi_index0(kg, n, nb)];
                    p = pos1s(x, n >> 3);
                } else {
                    hi = blk[512 + l * 4 + nb];
                    p = pos1(x);
                }
                u |= ((hi >> p) & 1u) << 2;
            }
        }
        const int c = blockIdx.y * N_TILE + col;
        if (c < I) {
            const float q = (float)((int)u - level_offset(w));
            out[(int64_t)(rank_off + row) * I + c] = q * __half2float(mv.scale[scale_off + row]);
        }
    }
}

// scale_s[scale_off(slab, tile) + row] = scale[...] * s[rank_off(slab) + row], rounded once to fp16,
// times the row's stagger factor (a power of two: the decoded weight carries its inverse).
// grid (slab tasks, tiles), 64 threads.
__global__ __launch_bounds__(64) void k_fold_scale_s(const MatView* __restrict__ views, const SlabTask* __restrict__ tasks,
                                                     const int64_t* __restrict__ out_offsets, __half* __restrict__ out) {
    const SlabTask task = tasks[blockIdx.x];
    const MatView mv = views[task.expert];
    const int si = task.slab;
    const int rank_off = mv.slab_meta[si * 4 + 2];
    const int t = mv.slab_meta[si * 4 + 3] + blockIdx.y;
    const int scale_off = mv.tile_meta[t * 3 + 1];
    const int row = threadIdx.x;
    const float v = __half2float(mv.scale[scale_off + row]) * __half2float(mv.s[rank_off + row]);
    const int w = mv.slab_meta[si * 4 + 0];
    out[out_offsets[task.expert] + scale_off + row] = __float2half(v * (float)stagger_factor(w, row));
}

}  // namespace bitsmoe

using namespace bitsmoe;

static int prepare_impl(bitsmoe_matset* set, int32_t role, hipStream_t st);

extern "C" int bitsmoe_matset_prepare(bitsmoe_matset* set, int32_t role, void* stream) {
    BITSMOE_REQUIRE(set != nullptr, "set must not be null");
    BITSMOE_REQUIRE(role == ROLE_GATE_UP || role == ROLE_DOWN, "role must be 0 (gate/up) or 1 (down)");
    if (set->role == role) return BITSMOE_OK;
    BITSMOE_REQUIRE(set->role < 0, "matrix set is already prepared for the other role");
    const int rc = prepare_impl(set, role, (hipStream_t)stream);
    if (rc != BITSMOE_OK) {
        // nothing of a failed attempt stays behind: the set remains usable by the generic kernels
        void** owned[] = {(void**)&set->d_prepared, (void**)&set->d_views_prepared, (void**)&set->d_fast_experts,
                          (void**)&set->d_fast_slabs, (void**)&set->d_scale_s};
        for (void** p : owned) {
            if (*p) (void)hipFree(*p);
            *p = nullptr;
        }
        set->role = -1;
    }
    return rc;
}

static int prepare_impl(bitsmoe_matset* set, int32_t role, hipStream_t st) {
    if (!set->regular64 || set->total_slabs == 0) {
        set_error("matrix set is not regular (every slab 64 rows of 2/3/4 bits, full 128-column tiles): "
                  "only the generic kernels can run it");
        return BITSMOE_E_UNSUPPORTED;
    }
    // the flattened tables assume the tiles of a slab follow each other in payload and scale
    std::vector<FastSlab> fslabs((size_t)set->n_experts * set->max_slabs, FastSlab{0, 0, 0, 0});
    for (int e = 0; e < set->n_experts; ++e) {
        const auto& slab = set->slab_meta_host[e];
        const auto& tile = set->tile_meta_host[e];
        for (int si = 0; si < set->descs[e].num_slabs; ++si) {
            const int bits = slab[si * 4 + 0], tile_off = slab[si * 4 + 3];
            for (int t = 0; t < set->n_tiles; ++t) {
                if (tile[(tile_off + t) * 3 + 0] != tile[tile_off * 3 + 0] + t * 256 * bits ||
                    tile[(tile_off + t) * 3 + 1] != tile[tile_off * 3 + 1] + t * SLAB_ROWS) {
                    set_error("expert %d slab %d: tiles are not contiguous in payload/scale; only the generic "
                              "kernels can run this set", e, si);
                    return BITSMOE_E_UNSUPPORTED;
                }
            }
            fslabs[(size_t)e * set->max_slabs + si] =
                FastSlab{bits, tile[tile_off * 3 + 0], tile[tile_off * 3 + 1], slab[si * 4 + 2]};
        }
    }
    // does every aligned group of GU_SLABS slabs have one width and follow each other in the payload?
    // (the same test the gate/up kernel applies per workgroup)
    bool all_uniform = set->max_slabs % GU_SLABS == 0;
    for (int e = 0; e < set->n_experts && all_uniform; ++e) {
        if (set->descs[e].num_slabs != set->max_slabs) all_uniform = false;
        for (int s0 = 0; s0 < set->descs[e].num_slabs && all_uniform; s0 += GU_SLABS) {
            const FastSlab& first = fslabs[(size_t)e * set->max_slabs + s0];
            for (int q = 1; q < GU_SLABS; ++q) {
                const FastSlab& f = fslabs[(size_t)e * set->max_slabs + s0 + q];
                if (f.bits != first.bits || f.pack_off != first.pack_off + q * set->n_tiles * 256 * first.bits)
                    all_uniform = false;
            }
        }
    }
    set->all_uniform8 = all_uniform;
    // is every expert one affine run of equal-width slabs (what the walking gate/up kernel assumes)?
    bool all_affine = all_uniform;
    for (int e = 0; e < set->n_experts && all_affine; ++e) {
        const FastSlab& first = fslabs[(size_t)e * set->max_slabs];
        for (int si = 1; si < set->max_slabs; ++si) {
            const FastSlab& f = fslabs[(size_t)e * set->max_slabs + si];
            if (f.bits != first.bits || f.pack_off != first.pack_off + si * set->n_tiles * 256 * first.bits ||
                f.scale_off != first.scale_off + si * set->n_tiles * SLAB_ROWS || f.rank_off != first.rank_off + si * SLAB_ROWS)
                all_affine = false;
        }
    }
    set->all_affine = all_affine;
    bool aligned = true;
    for (int e = 0; e < set->n_experts; ++e) {
        const bitsmoe_matrix_desc& d = set->descs[e];
        if ((((uintptr_t)d.scale) | ((uintptr_t)d.s) | ((uintptr_t)d.rank_idx)) & 15) aligned = false;
    }
    set->vector_aligned = aligned;
    int64_t total_words = 0;
    std::vector<int64_t> offs(set->n_experts);
    for (int e = 0; e < set->n_experts; ++e) {
        offs[e] = total_words;
        total_words += (set->descs[e].payload_words + 63) / 64 * 64;    // keep every matrix 256-byte aligned
    }
    BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_prepared, (size_t)total_words * 4));
    std::vector<MatView> views(set->n_experts);
    BITSMOE_HIP_TRY(hipMemcpyAsync(views.data(), set->d_views, sizeof(MatView) * set->n_experts, hipMemcpyDeviceToHost, st));
    BITSMOE_HIP_TRY(hipStreamSynchronize(st));
    for (int e = 0; e < set->n_experts; ++e) views[e].payload = set->d_prepared + offs[e];
    BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_views_prepared, sizeof(MatView) * set->n_experts));
    BITSMOE_HIP_TRY(hipMemcpyAsync(set->d_views_prepared, views.data(), sizeof(MatView) * set->n_experts, hipMemcpyHostToDevice, st));
    // gate/up sets also get a copy of the scales folded with the per-row multiplier
    std::vector<int64_t> sc_offs(set->n_experts, 0);
    if (role == ROLE_GATE_UP) {
        int64_t total_scale = 0;
        for (int e = 0; e < set->n_experts; ++e) {
            sc_offs[e] = total_scale;
            total_scale += (set->descs[e].scale_len + 127) / 128 * 128;    // keep every expert 256-byte aligned
        }
        int64_t* d_offs = nullptr;
        BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_scale_s, (size_t)std::max<int64_t>(total_scale, 1) * 2));
        BITSMOE_HIP_TRY(hipMalloc((void**)&d_offs, sizeof(int64_t) * set->n_experts));
        BITSMOE_HIP_TRY(hipMemcpyAsync(d_offs, sc_offs.data(), sizeof(int64_t) * set->n_experts, hipMemcpyHostToDevice, st));
        hipLaunchKernelGGL(k_fold_scale_s, dim3((unsigned)set->total_slabs, set->n_tiles), dim3(64), 0, st, set->d_views,
                           set->d_slab_tasks, d_offs, set->d_scale_s);
        const hipError_t launch_err = hipGetLastError();
        const hipError_t sync_err = hipStreamSynchronize(st);
        (void)hipFree(d_offs);
        BITSMOE_HIP_TRY(launch_err);
        BITSMOE_HIP_TRY(sync_err);
    }
    std::vector<FastExpert> fexp(set->n_experts);
    set->expert_bits.assign(set->n_experts, 0);
    for (int e = 0; e < set->n_experts; ++e) {
        FastExpert& f = fexp[e];
        memset(&f, 0, sizeof(f));
        f.scale_s = set->d_scale_s ? set->d_scale_s + sc_offs[e] : nullptr;
        f.payload = set->d_prepared + offs[e];
        f.scale = (const __half*)set->descs[e].scale;
        f.s = (const __half*)set->descs[e].s;
        f.rank_idx = (const int32_t*)set->descs[e].rank_idx;
        f.num_slabs = set->descs[e].num_slabs;
        f.uniform_bits = f.num_slabs > 0 ? set->slab_meta_host[e][0] : 0;
        for (int si = 1; si < f.num_slabs; ++si)
            if (set->slab_meta_host[e][si * 4] != f.uniform_bits) f.uniform_bits = 0;
        set->expert_bits[e] = (uint8_t)f.uniform_bits;
    }
    set->has_cost_order = set->n_experts <= EXPERT_ORDER_MAX;
    if (set->has_cost_order) {
        std::vector<int> order(set->n_experts);
        for (int e = 0; e < set->n_experts; ++e) order[e] = e;
        auto words = [&](int e) {       // payload words per tile of expert e
            int64_t w = 0;
            for (int si = 0; si < set->descs[e].num_slabs; ++si) w += set->slab_meta_host[e][si * 4];
            return w;
        };
        std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return words(a) > words(b); });
        for (int e = 0; e < set->n_experts; ++e) set->cost_order[e] = (uint16_t)order[e];
    }
    BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_fast_experts, sizeof(FastExpert) * fexp.size()));
    BITSMOE_HIP_TRY(hipMemcpyAsync(set->d_fast_experts, fexp.data(), sizeof(FastExpert) * fexp.size(), hipMemcpyHostToDevice, st));
    BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_fast_slabs, sizeof(FastSlab) * fslabs.size()));
    BITSMOE_HIP_TRY(hipMemcpyAsync(set->d_fast_slabs, fslabs.data(), sizeof(FastSlab) * fslabs.size(), hipMemcpyHostToDevice, st));
    hipLaunchKernelGGL(k_prepack, dim3((unsigned)set->total_slabs, set->n_tiles), dim3(256), 0, st, set->d_views,
                       set->d_views_prepared, set->d_slab_tasks, role);
    BITSMOE_HIP_TRY(hipGetLastError());
    BITSMOE_HIP_TRY(hipStreamSynchronize(st));
    set->prepared_offsets = offs;
    set->role = role;
    return BITSMOE_OK;
}

extern "C" int bitsmoe_dequant_matrix_prepared(const bitsmoe_matset* set, int32_t expert, float* out_device, void* stream) {
    BITSMOE_REQUIRE(set && out_device, "null argument");
    BITSMOE_REQUIRE(expert >= 0 && expert < set->n_experts, "expert %d out of range", expert);
    BITSMOE_REQUIRE(set->role >= 0, "matrix set is not prepared");
    hipStream_t st = (hipStream_t)stream;
    const bitsmoe_matrix_desc& d = set->descs[expert];
    MatView mv;
    mv.payload = set->d_prepared + set->prepared_offsets[expert];
    mv.rank_idx = (const int32_t*)d.rank_idx;
    mv.tile_meta = (const int32_t*)d.tile_meta;
    mv.slab_meta = (const int32_t*)d.slab_meta;
    mv.scale = (const __half*)d.scale;
    mv.s = (const __half*)d.s;
    mv.num_slabs = d.num_slabs;
    mv.num_tiles = d.num_tiles;
    mv.rank_len = d.rank_len;
    mv.flags = 1;
    hipLaunchKernelGGL(k_dequant_prepared, dim3(d.num_slabs, set->n_tiles), dim3(256), 0, st, mv, set->role,
                       set->intermediate_size, out_device);
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}
