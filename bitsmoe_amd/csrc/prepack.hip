// One-time re-layout of a matrix set's payload into the wave64-native field layout
// (wave_layout.h) and the dense dequantiser that reads it back (parity check of the layout).
#include "wave_layout.h"

#include <algorithm>
#include <cstring>

namespace bitsmoe {

// code (unsigned, before the level offset) of element (row, col) of a (slab, tile) block of `k_slab`
// rows in the reference bit-plane layout; `blk` points at the block's first word.  Rows past
// k_slab (a ragged slab is padded to 64 rows in the prepared copy) read as the code of level zero.
__device__ inline uint32_t ref_code(const uint32_t* __restrict__ blk, int w, int k_slab, int row, int col) {
    if (row >= k_slab) return (uint32_t)level_offset(w);
    const int stage = row >> 4, r = row & 15, micro = col >> 5, lane = col & 31;
    const int rows_cur = min(K_STAGE, k_slab - stage * K_STAGE);
    const uint32_t* words = blk + stage * (K_STAGE * MICROS * w) + micro * (rows_cur * w) + r * w;
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

// grid: (slab tasks, tiles); every thread builds whole output words of one block.  Reads the caller's
// reference layout (through its own tile_meta / slab_meta), writes the prepared copy at the offsets of
// the FastSlab table.
__global__ __launch_bounds__(256) void k_prepack(const MatView* __restrict__ src, const FastExpert* __restrict__ fexp,
                                                 const FastSlab* __restrict__ fslabs, int max_slabs,
                                                 const SlabTask* __restrict__ tasks, int role) {
    const SlabTask task = tasks[blockIdx.x];
    const MatView mv = src[task.expert];
    const int si = task.slab;
    const int w = mv.slab_meta[si * 4 + 0];
    const int k_slab = mv.slab_meta[si * 4 + 1];
    const int tile_off = mv.slab_meta[si * 4 + 3];
    const int t = tile_off + blockIdx.y;
    const uint32_t* __restrict__ in = mv.payload + mv.tile_meta[t * 3 + 0];
    const FastSlab fs = fslabs[(int64_t)task.expert * max_slabs + si];
    uint32_t* __restrict__ out = const_cast<uint32_t*>(fexp[task.expert].payload) + fs.pack_off + (int)blockIdx.y * 256 * w;
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
                        word |= ((ref_code(in, w, k_slab, row, col) >> 2) & 1u) << pos1s(x, upper);
                    }
            } else {                      // j = l*4 + nb
                const int nb = j & 3, l = j >> 2, n = l & 15, kg = l >> 4;
                for (int x = 0; x < 32; ++x) {
                    int row, col;
                    run_element(role, nb, kg, n, x, &row, &col);
                    word |= ((ref_code(in, w, k_slab, row, col) >> 2) & 1u) << pos1(x);
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
            const uint32_t u = ref_code(in, w, k_slab, row, col);
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

// The per-row tables of the prepared copy, every slab padded to 64 rows: s' (multiplier), scale'
// [(slab, tile)][64] and, for gate/up sets, scale_s' = scale * s * stagger factor (a power of two: the
// decoded weight carries its inverse), each rounded once to fp16.  Padding rows get zeros, so whatever
// the kernels read for them contributes nothing.  grid (slab tasks, tiles), 64 threads.
__global__ __launch_bounds__(64) void k_prepare_rows(const MatView* __restrict__ views, const FastExpert* __restrict__ fexp,
                                                     const FastSlab* __restrict__ fslabs, int max_slabs,
                                                     const SlabTask* __restrict__ tasks) {
    const SlabTask task = tasks[blockIdx.x];
    const MatView mv = views[task.expert];
    const FastExpert fe = fexp[task.expert];
    const int si = task.slab;
    const int w = mv.slab_meta[si * 4 + 0];
    const int k_slab = mv.slab_meta[si * 4 + 1];
    const int rank_off = mv.slab_meta[si * 4 + 2];
    const int t = mv.slab_meta[si * 4 + 3] + blockIdx.y;
    const int scale_off = mv.tile_meta[t * 3 + 1];
    const FastSlab fs = fslabs[(int64_t)task.expert * max_slabs + si];
    const int row = threadIdx.x;
    const bool valid = row < k_slab;
    const float sv = valid ? __half2float(mv.s[rank_off + row]) : 0.0f;
    const float sc = valid ? __half2float(mv.scale[scale_off + row]) : 0.0f;
    const int out_sc = fs.scale_off + (int)blockIdx.y * SLAB_ROWS + row;
    const_cast<__half*>(fe.scale)[out_sc] = __float2half(sc);
    if (fe.scale_s) const_cast<__half*>(fe.scale_s)[out_sc] = __float2half(sc * sv * (float)stagger_factor(w, row));
    if (blockIdx.y == 0) const_cast<__half*>(fe.s)[fs.rank_off + row] = __float2half(sv);
}

// Dense fp32 dequantisation FROM THE PREPARED COPY, written to mirror the decode of the hot kernels
// (fields, not planes); rows in the caller's local row order, output identical to k_dequant_matrix.
__global__ __launch_bounds__(256) void k_dequant_prepared(MatView mv /* the caller's tables */, FastExpert fe,
                                                          const FastSlab* __restrict__ fs_row, int role, int I,
                                                          float* __restrict__ out) {
    const int si = blockIdx.x;
    const int w = mv.slab_meta[si * 4 + 0];
    const int k_slab = mv.slab_meta[si * 4 + 1];
    const int rank_off = mv.slab_meta[si * 4 + 2];
    const FastSlab fs = fs_row[si];
    const uint32_t* __restrict__ blk = fe.payload + fs.pack_off + (int)blockIdx.y * 256 * w;
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
        if (c < I && row < k_slab) {
            const float q = (float)((int)u - level_offset(w));
            out[(int64_t)(rank_off + row) * I + c] = q * __half2float(fe.scale[fs.scale_off + (int)blockIdx.y * SLAB_ROWS + row]);
        }
    }
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
        void** owned[] = {(void**)&set->d_prepared, (void**)&set->d_fast_experts, (void**)&set->d_fast_slabs,
                          (void**)&set->d_scale_s, (void**)&set->d_prepared_rows};
        for (void** p : owned) {
            if (*p) (void)hipFree(*p);
            *p = nullptr;
        }
        set->role = -1;
    }
    return rc;
}

static inline int64_t round_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

static int prepare_impl(bitsmoe_matset* set, int32_t role, hipStream_t st) {
    if (!set->fast_ok || set->total_slabs == 0) {
        set_error("matrix set holds slabs of other widths than 2, 3 or 4 bits, or tiles of fewer than 128 columns: "
                  "only the generic kernels can run it");
        return BITSMOE_E_UNSUPPORTED;
    }
    const int E = set->n_experts, n_tiles = set->n_tiles, max_slabs = set->max_slabs;
    // Offsets of the prepared copy: every slab is a full 64-row slab there (a ragged slab of the caller's
    // layout is padded), so slab si of an expert holds local rows [64 si, 64 si + 64), its tiles follow
    // each other in payload' (256 w words each) and in scale' (64 each).
    std::vector<FastSlab> fslabs((size_t)E * max_slabs, FastSlab{0, 0, 0, 0});
    std::vector<int64_t> pay_off(E), row_off(E), sc_off(E);
    int64_t pay_words = 0, rows_total = 0, scale_total = 0;
    for (int e = 0; e < E; ++e) {
        pay_off[e] = pay_words;
        row_off[e] = rows_total;
        sc_off[e] = scale_total;
        const auto& slab = set->slab_meta_host[e];
        int64_t words = 0;
        const int ns = set->descs[e].num_slabs;
        for (int si = 0; si < ns; ++si) {
            const int bits = slab[si * 4 + 0];
            BITSMOE_REQUIRE(words < ((int64_t)1 << 31) - (int64_t)n_tiles * 256 * 4, "expert %d: prepared payload exceeds int32 word offsets", e);
            fslabs[(size_t)e * max_slabs + si] = FastSlab{bits, (int32_t)words, si * n_tiles * SLAB_ROWS, si * SLAB_ROWS};
            words += (int64_t)n_tiles * 256 * bits;
        }
        pay_words += round_up(words, 64);                               // keep every matrix 256-byte aligned
        rows_total += round_up((int64_t)ns * SLAB_ROWS, 64);
        scale_total += round_up((int64_t)ns * n_tiles * SLAB_ROWS, 128);
    }
    // rank_idx' on the host (the kernels' eligibility flags are read off it): a padding row reads rank -1,
    // which every kernel treats as "no such row" -- except whole padded runs of eight rows, which read the
    // ranks 0..7 (their scale is zero) so that they do not break the runs-of-eight property below.
    std::vector<int32_t> rank_rows((size_t)std::max<int64_t>(rows_total, 1), -1);
    for (int e = 0; e < E; ++e) {
        const auto& slab = set->slab_meta_host[e];
        const auto& rk = set->rank_idx_host[e];
        for (int si = 0; si < set->descs[e].num_slabs; ++si) {
            const int k_slab = slab[si * 4 + 1], rank_off = slab[si * 4 + 2];
            int32_t* dst = rank_rows.data() + row_off[e] + (int64_t)si * SLAB_ROWS;
            for (int r = 0; r < SLAB_ROWS; ++r) {
                if (r < k_slab)
                    dst[r] = rk[rank_off + r];
                else if ((r & ~7) >= k_slab && set->max_rank_plus1 >= 8)
                    dst[r] = r & 7;
            }
        }
    }
    // every aligned run of 8 rows = 8 consecutive logical ranks starting at a multiple of 8?  rank'[k] == k?
    bool chunked8 = E > 0, identity = E > 0;
    for (int e = 0; e < E && (chunked8 || identity); ++e) {
        const int64_t n = (int64_t)set->descs[e].num_slabs * SLAB_ROWS;
        const int32_t* r = rank_rows.data() + row_off[e];
        for (int64_t k = 0; k < n; ++k) {
            if (r[k] != (int32_t)k) identity = false;
            if ((k & 7) == 0 ? (r[k] < 0 || (r[k] & 7) != 0) : (r[k] != r[k - 1] + 1)) chunked8 = false;
        }
    }
    set->rank_chunked8 = chunked8;
    set->rank_identity = identity;
    // does every aligned group of GU_SLABS slabs have one width (the same test the split gate/up kernel
    // applies per workgroup), and is every expert ONE run of equal-width slabs (what the walking kernel assumes)?
    bool all_uniform = max_slabs % GU_SLABS == 0, all_affine = max_slabs % GU_SLABS == 0;
    for (int e = 0; e < E && all_uniform; ++e) {
        if (set->descs[e].num_slabs != max_slabs) all_uniform = all_affine = false;
        for (int si = 0; si < set->descs[e].num_slabs && all_uniform; ++si) {
            const int bits = fslabs[(size_t)e * max_slabs + si].bits;
            if (bits != fslabs[(size_t)e * max_slabs + si / GU_SLABS * GU_SLABS].bits) all_uniform = false;
            if (bits != fslabs[(size_t)e * max_slabs].bits) all_affine = false;
        }
    }
    set->all_uniform8 = all_uniform;
    set->all_affine = all_uniform && all_affine;
    set->vector_aligned = true;       // (the prepared tables are the library's own, 256-byte aligned allocations)

    BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_prepared, (size_t)std::max<int64_t>(pay_words, 1) * 4));
    // one allocation for the row tables: rank' (i32), s' (f16), scale' (f16)
    const size_t rows_bytes = (size_t)round_up(rows_total * 4, 256) + (size_t)round_up(rows_total * 2, 256) +
                              (size_t)round_up(scale_total * 2, 256);
    BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_prepared_rows, std::max<size_t>(rows_bytes, 256)));
    int32_t* d_rank = (int32_t*)set->d_prepared_rows;
    __half* d_s = (__half*)((char*)set->d_prepared_rows + round_up(rows_total * 4, 256));
    __half* d_scale = (__half*)((char*)d_s + round_up(rows_total * 2, 256));
    if (role == ROLE_GATE_UP)
        BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_scale_s, (size_t)std::max<int64_t>(scale_total, 1) * 2));
    BITSMOE_HIP_TRY(hipMemcpyAsync(d_rank, rank_rows.data(), (size_t)rows_total * 4, hipMemcpyHostToDevice, st));

    std::vector<FastExpert> fexp(E);
    set->expert_bits.assign(E, 0);
    for (int e = 0; e < E; ++e) {
        FastExpert& f = fexp[e];
        memset(&f, 0, sizeof(f));
        f.payload = set->d_prepared + pay_off[e];
        f.scale = d_scale + sc_off[e];
        f.s = d_s + row_off[e];
        f.rank_idx = d_rank + row_off[e];
        f.scale_s = set->d_scale_s ? set->d_scale_s + sc_off[e] : nullptr;
        f.num_slabs = set->descs[e].num_slabs;
        f.uniform_bits = f.num_slabs > 0 ? set->slab_meta_host[e][0] : 0;
        for (int si = 1; si < f.num_slabs; ++si)
            if (set->slab_meta_host[e][si * 4] != f.uniform_bits) f.uniform_bits = 0;
        set->expert_bits[e] = (uint8_t)f.uniform_bits;
    }
    set->has_cost_order = E <= EXPERT_ORDER_MAX;
    if (set->has_cost_order) {
        std::vector<int> order(E);
        for (int e = 0; e < E; ++e) order[e] = e;
        auto words = [&](int e) {       // payload words per tile of expert e
            int64_t w = 0;
            for (int si = 0; si < set->descs[e].num_slabs; ++si) w += set->slab_meta_host[e][si * 4];
            return w;
        };
        std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return words(a) > words(b); });
        for (int e = 0; e < E; ++e) set->cost_order[e] = (uint16_t)order[e];
    }
    BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_fast_experts, sizeof(FastExpert) * fexp.size()));
    BITSMOE_HIP_TRY(hipMemcpyAsync(set->d_fast_experts, fexp.data(), sizeof(FastExpert) * fexp.size(), hipMemcpyHostToDevice, st));
    BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_fast_slabs, sizeof(FastSlab) * fslabs.size()));
    BITSMOE_HIP_TRY(hipMemcpyAsync(set->d_fast_slabs, fslabs.data(), sizeof(FastSlab) * fslabs.size(), hipMemcpyHostToDevice, st));
    hipLaunchKernelGGL(k_prepare_rows, dim3((unsigned)set->total_slabs, n_tiles), dim3(64), 0, st, set->d_views,
                       set->d_fast_experts, set->d_fast_slabs, max_slabs, set->d_slab_tasks);
    BITSMOE_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(k_prepack, dim3((unsigned)set->total_slabs, n_tiles), dim3(256), 0, st, set->d_views,
                       set->d_fast_experts, set->d_fast_slabs, max_slabs, set->d_slab_tasks, role);
    BITSMOE_HIP_TRY(hipGetLastError());
    BITSMOE_HIP_TRY(hipStreamSynchronize(st));      // (the host vectors above are read by the copies until here)
    set->fast_experts_host = fexp;
    set->role = role;
    return BITSMOE_OK;
}

extern "C" int bitsmoe_dequant_matrix_prepared(const bitsmoe_matset* set, int32_t expert, float* out_device, void* stream) {
    BITSMOE_REQUIRE(set && out_device, "null argument");
    BITSMOE_REQUIRE(expert >= 0 && expert < set->n_experts, "expert %d out of range", expert);
    BITSMOE_REQUIRE(set->role >= 0, "matrix set is not prepared");
    hipStream_t st = (hipStream_t)stream;
    const bitsmoe_matrix_desc& d = set->descs[expert];
    if (d.num_slabs == 0) return BITSMOE_OK;
    MatView mv;
    mv.payload = (const uint32_t*)d.payload;
    mv.rank_idx = (const int32_t*)d.rank_idx;
    mv.tile_meta = (const int32_t*)d.tile_meta;
    mv.slab_meta = (const int32_t*)d.slab_meta;
    mv.scale = (const __half*)d.scale;
    mv.s = (const __half*)d.s;
    mv.num_slabs = d.num_slabs;
    mv.num_tiles = d.num_tiles;
    mv.rank_len = d.rank_len;
    mv.flags = 1;
    hipLaunchKernelGGL(k_dequant_prepared, dim3(d.num_slabs, set->n_tiles), dim3(256), 0, st, mv,
                       set->fast_experts_host[expert], set->d_fast_slabs + (int64_t)expert * set->max_slabs, set->role,
                       set->intermediate_size, out_device);
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}
