// One-time re-layout of a matrix set's payload into the wave64-native field layout
// (wave_layout.h) and the dense dequantiser that reads it back (parity check of the layout).
#include "wave_layout.h"
#include "wide_layout.h"

#include <algorithm>
#include <cstring>

namespace bitsmoe {

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

// Where a row of the prepared copy comes from: (source slab << 8) | row inside that slab, or -1 for a
// padding row.  The prepared copy keeps the caller's local row order but cuts it into slabs of its own:
// rows [64 p, 64 p + 64) whatever bucket they came from, stored at the widest width among them (a narrower
// code is the same LEVEL at a wider width: level = code - 2^(w-1), and the scale stays per row), so that a
// bucket whose row count is no multiple of 64 leaves no gap in the row numbering.
struct PrepSource {
    const int32_t* row_src;      // [rows of the prepared copy], all experts
    const int32_t* rank_base;    // the prepared rank table's first element: an expert's rows start at fe.rank_idx - rank_base
};

// The level (signed) of prepared row `row` of prepared slab `ps`, column `col` of tile `t`.
__device__ inline int source_level(const MatView& mv, const int32_t* __restrict__ row_src, int ps, int row, int t, int col) {
    const int src = row_src[ps * SLAB_ROWS + row];
    if (src < 0) return 0;
    const int s = src >> 8, r = src & 255;
    const int w = mv.slab_meta[s * 4 + 0], k_slab = mv.slab_meta[s * 4 + 1];
    const int32_t* tm = mv.tile_meta + (mv.slab_meta[s * 4 + 3] + t) * 3;
    if (col >= tm[2]) return 0;          // (columns past the matrix's last one: whatever the payload holds there)
    const uint32_t* __restrict__ blk = mv.payload + tm[0];
    const int stage = r >> 4, rr = r & 15, micro = col >> 5, lane = col & 31;
    const int rows_cur = min(K_STAGE, k_slab - stage * K_STAGE);
    const uint32_t* words = blk + stage * (K_STAGE * MICROS * w) + micro * (rows_cur * w) + rr * w;
    int u = 0;
    for (int p = 0; p < w; ++p) u |= (int)((words[p] >> lane) & 1u) << p;
    return w == 1 ? 2 * u - 1 : u - level_offset(w);      // (1-bit codes are the levels -1 / +1)
}

// grid: (prepared slab tasks, tiles); every thread builds whole output words of one block.  Reads the
// caller's reference layout (through its own tile_meta / slab_meta), writes the prepared copy at the
// offsets of the FastSlab table.
__global__ __launch_bounds__(256) void k_prepack(const MatView* __restrict__ src, const FastExpert* __restrict__ fexp,
                                                 const FastSlab* __restrict__ fslabs, int max_slabs,
                                                 const SlabTask* __restrict__ tasks, PrepSource ps_tab, int role) {
    const SlabTask task = tasks[blockIdx.x];
    const MatView mv = src[task.expert];
    const FastExpert fe = fexp[task.expert];
    const int ps = task.slab;
    const int t = blockIdx.y;
    const FastSlab fs = fslabs[(int64_t)task.expert * max_slabs + ps];
    const int w = fs.bits;
    const int32_t* __restrict__ row_src = ps_tab.row_src + (fe.rank_idx - ps_tab.rank_base);
    uint32_t* __restrict__ out = const_cast<uint32_t*>(fe.payload) + fs.pack_off + t * block_words(role, w);
    auto code_at = [&](int row, int col) { return (uint32_t)(source_level(mv, row_src, ps, row, t, col) + level_offset(w)); };
    const int nbs = (role == ROLE_GATE_UP) ? 8 : 4;        // output blocks per lane
    const int run = (role == ROLE_GATE_UP) ? 16 : 32;      // contraction indices per (lane, nb)
    const int n_words = block_words(role, w);
    for (int idx = threadIdx.x; idx < n_words; idx += blockDim.x) {
        uint32_t word = 0;
        if (w == 3 && role == ROLE_DOWN) {
            // whole 3-bit fields, five pairs of neighbouring codes per word (wave_layout.h)
            const int l = idx < 768 ? (idx & 255) >> 2 : idx - 768;
            const int j = idx < 768 ? (idx >> 8) * 4 + (idx & 3) : 12;
            const int n = l & 15, kg = l >> 4;
            for (int sl = 0; sl < 5; ++sl) {
                const int P = 5 * j + sl;
                if (P >= 64) break;
                const int nb = P >> 4, m = (P >> 2) & 3, i = P & 3;
                for (int odd = 0; odd < 2; ++odd) {
                    int row, col;
                    run_element(role, nb, kg, n, 8 * m + 2 * i + odd, &row, &col);
                    word |= (code_at(row, col) & 7u) << (r1w3_slot_pos(sl) + 16 * odd);
                }
            }
            out[idx] = word;
            continue;
        }
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
                        word |= ((code_at(row, col) >> 2) & 1u) << pos1s(x, upper);
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
            const uint32_t u = code_at(row, col);
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

// The per-row tables of the prepared copy: s' (multiplier), scale' [(slab, tile)][64] and, for gate/up
// sets, scale_s' = scale * s * stagger factor of the row at the PREPARED slab's width (a power of two: the
// decoded weight carries its inverse), each rounded once to fp16.  Padding rows get zeros, so whatever
// the kernels read for them contributes nothing.  grid (prepared slab tasks, tiles), 64 threads.
__global__ __launch_bounds__(64) void k_prepare_rows(const MatView* __restrict__ views, const FastExpert* __restrict__ fexp,
                                                     const FastSlab* __restrict__ fslabs, int max_slabs,
                                                     const SlabTask* __restrict__ tasks, PrepSource ps_tab) {
    const SlabTask task = tasks[blockIdx.x];
    const MatView mv = views[task.expert];
    const FastExpert fe = fexp[task.expert];
    const int ps = task.slab;
    const int t = blockIdx.y;
    const FastSlab fs = fslabs[(int64_t)task.expert * max_slabs + ps];
    const int row = threadIdx.x;
    const int src = (ps_tab.row_src + (fe.rank_idx - ps_tab.rank_base))[ps * SLAB_ROWS + row];
    float sv = 0.0f, sc = 0.0f;
    if (src >= 0) {
        const int s = src >> 8, r = src & 255;
        sv = __half2float(mv.s[mv.slab_meta[s * 4 + 2] + r]);
        sc = __half2float(mv.scale[mv.tile_meta[(mv.slab_meta[s * 4 + 3] + t) * 3 + 1] + r]);
    }
    const int out_sc = fs.scale_off + t * SLAB_ROWS + row;
    const_cast<__half*>(fe.scale)[out_sc] = __float2half(sc);
    if (fe.scale_s) const_cast<__half*>(fe.scale_s)[out_sc] = __float2half(sc * sv * (float)stagger_factor(fs.bits, row));
    if (t == 0) const_cast<__half*>(fe.s)[fs.rank_off + row] = __float2half(sv);
}

// The side table of wide rows (wide_layout.h) from the caller's layout.  grid (wide slabs, tiles).
__global__ __launch_bounds__(256) void k_prepack_wide(const MatView* __restrict__ views, const int32_t* __restrict__ slab_expert,
                                                      const int32_t* __restrict__ wide_src, int role, int n_tiles,
                                                      __half* __restrict__ wide, __half* __restrict__ wide_s) {
    const int ws = blockIdx.x, t = blockIdx.y;
    const MatView mv = views[slab_expert[ws]];
    __half* __restrict__ out = wide + ((int64_t)ws * n_tiles + t) * WIDE_BLOCK;
    for (int idx = threadIdx.x; idx < WIDE_BLOCK; idx += blockDim.x) {
        const int row = idx >> 7, col = idx & 127;
        const int src = wide_src[ws * SLAB_ROWS + row];
        float v = 0.0f;
        if (src >= 0) {
            const int s = src >> 8, r = src & 255;
            const int bits = mv.slab_meta[s * 4 + 0], k_slab = mv.slab_meta[s * 4 + 1];
            const int32_t* tm = mv.tile_meta + (mv.slab_meta[s * 4 + 3] + t) * 3;
            if (col < tm[2]) {
                const int w = words_per_row(bits);
                const int stage = r >> 4, rr = r & 15, micro = col >> 5, lane = col & 31;
                const int rows_cur = min(K_STAGE, k_slab - stage * K_STAGE);
                v = decode_from_row_words(mv.payload + tm[0] + stage * (K_STAGE * MICROS * w) + micro * (rows_cur * w) + rr * w, bits, lane);
                if (bits != 16) v *= __half2float(mv.scale[tm[1] + r]);
            }
        }
        out[wide_index(role, row, col)] = __float2half(v);
    }
    if (t == 0 && threadIdx.x < SLAB_ROWS) {
        const int src = wide_src[ws * SLAB_ROWS + threadIdx.x];
        wide_s[ws * SLAB_ROWS + threadIdx.x] = src >= 0 ? mv.s[mv.slab_meta[(src >> 8) * 4 + 2] + (src & 255)] : __float2half(0.0f);
    }
}

// Dense fp32 dequantisation of an expert's wide rows FROM THE SIDE TABLE (rows in the caller's local row order).
// grid (wide slabs of the expert, tiles).
__global__ __launch_bounds__(256) void k_dequant_wide(MatView mv, const __half* __restrict__ wide, const int32_t* __restrict__ wide_src,
                                                      int ws0, int role, int n_tiles, int I, float* __restrict__ out) {
    const int ws = ws0 + blockIdx.x, t = blockIdx.y;
    const __half* __restrict__ blk = wide + ((int64_t)ws * n_tiles + t) * WIDE_BLOCK;
    for (int idx = threadIdx.x; idx < WIDE_BLOCK; idx += blockDim.x) {
        const int row = idx >> 7, col = idx & 127;
        const int src = wide_src[ws * SLAB_ROWS + row];
        const int c = t * N_TILE + col;
        if (src < 0 || c >= I) continue;
        const int local_row = mv.slab_meta[(src >> 8) * 4 + 2] + (src & 255);
        out[(int64_t)local_row * I + c] = __half2float(blk[wide_index(role, row, col)]);
    }
}

// Dense fp32 dequantisation FROM THE PREPARED COPY, written to mirror the decode of the hot kernels
// (fields, not planes); rows in the caller's local row order, output identical to k_dequant_matrix.
// grid (prepared slabs of the expert, tiles).
__global__ __launch_bounds__(256) void k_dequant_prepared(MatView mv /* the caller's tables */, FastExpert fe,
                                                          const FastSlab* __restrict__ fs_row, const int32_t* __restrict__ row_src,
                                                          int role, int I, float* __restrict__ out) {
    const int ps = blockIdx.x;
    const FastSlab fs = fs_row[ps];
    const int w = fs.bits;
    const uint32_t* __restrict__ blk = fe.payload + fs.pack_off + (int)blockIdx.y * block_words(role, w);
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
        if (w == 3 && role == ROLE_DOWN) {
            const int P = 16 * nb + 4 * (x >> 3) + ((x & 7) >> 1);
            u = (blk[r1w3_word_index(l, P / 5)] >> (r1w3_slot_pos(P % 5) + 16 * (x & 1))) & 7u;
        } else if (w == 4) {
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
                hi = blk[512 + hi_index0(kg, n, nb)];      // (role 0: role 1 took the branch above)
                p = pos1s(x, n >> 3);
                u |= ((hi >> p) & 1u) << 2;
            }
        }
        const int c = blockIdx.y * N_TILE + col;
        const int src = row_src[ps * SLAB_ROWS + row];
        if (c < I && src >= 0) {
            const int local_row = mv.slab_meta[(src >> 8) * 4 + 2] + (src & 255);
            const float q = (float)((int)u - level_offset(w));
            out[(int64_t)local_row * I + c] = q * __half2float(fe.scale[fs.scale_off + (int)blockIdx.y * SLAB_ROWS + row]);
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
                          (void**)&set->d_scale_s, (void**)&set->d_prepared_rows, (void**)&set->d_prep_tasks,
                          (void**)&set->d_wide_tables, (void**)&set->d_wide};
        for (void** p : owned) {
            if (*p) (void)hipFree(*p);
            *p = nullptr;
        }
        set->role = -1;
        set->wide_slabs = 0;
        set->n_wide_experts = 0;
    }
    return rc;
}

static inline int64_t round_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

static int prepare_impl(bitsmoe_matset* set, int32_t role, hipStream_t st) {
    if (!set->fast_ok || set->total_slabs == 0) {
        set_error("matrix set is empty or holds a slab that does not span all column tiles: only the generic kernels can run it");
        return BITSMOE_E_UNSUPPORTED;
    }
    const int E = set->n_experts, n_tiles = set->n_tiles;
    // The slabs of the prepared copy: the caller's local rows in their order, cut every 64 rows; gate/up
    // sets in whole groups of GU_SLABS slabs (what one workgroup of the walking kernel contracts over
    // between two barriers), a group stored at ONE width, the widest among its rows.
    // Rows of 6-, 8- and 16-bit slabs are kept out of it: they go to the side table of wide rows (below).
    const int unit = role == ROLE_GATE_UP ? GU_SLABS : 1;
    auto is_wide = [](int bits) { return bits > 4; };
    std::vector<int> n_ps(E);
    std::vector<int32_t> wide_first(E + 1, 0);
    int pms = 0;
    int64_t narrow_rows = 0;
    for (int e = 0; e < E; ++e) {
        int64_t rows = 0, rows_wide = 0;
        for (int si = 0; si < set->descs[e].num_slabs; ++si)
            (is_wide(set->slab_meta_host[e][si * 4 + 0]) ? rows_wide : rows) += set->slab_meta_host[e][si * 4 + 1];
        n_ps[e] = (int)round_up(std::max<int64_t>((rows + SLAB_ROWS - 1) / SLAB_ROWS, 1), unit);
        pms = std::max(pms, n_ps[e]);
        narrow_rows += rows;
        wide_first[e + 1] = wide_first[e] + (int32_t)((rows_wide + SLAB_ROWS - 1) / SLAB_ROWS);
    }
    set->prep_max_slabs = pms;
    std::vector<FastSlab> fslabs((size_t)E * pms, FastSlab{0, 0, 0, 0});
    std::vector<SlabTask> tasks;
    std::vector<int64_t> pay_off(E), row_off(E), sc_off(E);
    int64_t pay_words = 0, rows_total = 0, scale_total = 0;
    for (int e = 0; e < E; ++e) {
        row_off[e] = rows_total;
        sc_off[e] = scale_total;
        rows_total += (int64_t)n_ps[e] * SLAB_ROWS;
        scale_total += round_up((int64_t)n_ps[e] * n_tiles * SLAB_ROWS, 128);
    }
    std::vector<int32_t> rank_rows((size_t)std::max<int64_t>(rows_total, 1), -1), row_src((size_t)std::max<int64_t>(rows_total, 1), -1);
    int pad_rank_plus1 = set->max_rank_plus1;
    for (int e = 0; e < E; ++e) {
        const auto& slab = set->slab_meta_host[e];
        const auto& rk = set->rank_idx_host[e];
        int32_t* rr = rank_rows.data() + row_off[e];
        int32_t* rs = row_src.data() + row_off[e];
        std::vector<int> width(n_ps[e], 0);
        int64_t p = 0;
        for (int si = 0; si < set->descs[e].num_slabs; ++si) {
            const int bits = slab[si * 4 + 0], k_slab = slab[si * 4 + 1], rank_off = slab[si * 4 + 2];
            if (is_wide(bits)) continue;
            for (int r = 0; r < k_slab; ++r, ++p) {
                rr[p] = rk[rank_off + r];
                rs[p] = (si << 8) | r;
                width[p / SLAB_ROWS] = std::max(width[p / SLAB_ROWS], std::max(bits, 2));      // (1-bit levels fit 2-bit fields)
            }
        }
        // Padding rows (zero scales) behind the last row.  When the real rows are the identity (row k holds
        // rank k: what ascending bit buckets without gaps give) the padding rows continue it, so that the set
        // keeps its identity and runs-of-eight properties; kernels skip ranks outside the activations / the
        // output, and pad_rank_plus1 tells the launchers how far the padding reaches.  Otherwise a run of
        // eight that is all padding reads the ranks 0..7, the rest of a run that the last rows begin
        // continues that run, and any other padding row has rank -1 ("no such row" to every kernel).
        const int64_t rows_e = p, rows_p = (int64_t)n_ps[e] * SLAB_ROWS;
        bool ident_e = rows_e > 0;      // (an expert without 2/3/4-bit rows: padding only, which reads the ranks 0..7)
        for (int64_t j = 0; j < rows_e && ident_e; ++j) ident_e = rr[j] == (int32_t)j;
        for (; p < rows_p; ++p) {
            const int64_t run0 = p & ~(int64_t)7;
            if (ident_e) {
                rr[p] = (int32_t)p;
                pad_rank_plus1 = std::max(pad_rank_plus1, rr[p] + 1);
            } else if (run0 >= rows_e) {
                if (set->max_rank_plus1 >= 8) rr[p] = (int32_t)(p & 7);
            } else if (rr[run0] >= 0 && (rr[run0] & 7) == 0) {
                rr[p] = rr[run0] + (int32_t)(p - run0);
                pad_rank_plus1 = std::max(pad_rank_plus1, rr[p] + 1);
            }
        }
        for (int ps = 0; ps < n_ps[e]; ++ps)
            if (width[ps] == 0) width[ps] = ps > 0 ? width[ps - 1] : 2;      // (a slab of padding only)
        if (role == ROLE_GATE_UP)
            for (int g0 = 0; g0 < n_ps[e]; g0 += GU_SLABS) {
                int w = 0;
                for (int q = 0; q < GU_SLABS; ++q) w = std::max(w, width[g0 + q]);
                for (int q = 0; q < GU_SLABS; ++q) width[g0 + q] = w;
            }
        pay_off[e] = pay_words;
        int64_t words = 0;
        for (int ps = 0; ps < n_ps[e]; ++ps) {
            BITSMOE_REQUIRE(words < ((int64_t)1 << 31) - (int64_t)n_tiles * 256 * 4, "expert %d: prepared payload exceeds int32 word offsets", e);
            fslabs[(size_t)e * pms + ps] = FastSlab{width[ps], (int32_t)words, ps * n_tiles * SLAB_ROWS, ps * SLAB_ROWS};
            words += (int64_t)n_tiles * block_words(role, width[ps]);
            tasks.push_back(SlabTask{e, ps});
        }
        pay_words += round_up(words, 64);      // keep every matrix 256-byte aligned
    }
    set->pad_rank_plus1 = pad_rank_plus1;
    // every aligned run of 8 rows = 8 consecutive logical ranks starting at a multiple of 8?  rank'[k] == k?
    bool chunked8 = E > 0, identity = E > 0;
    for (int e = 0; e < E && (chunked8 || identity); ++e) {
        const int64_t n = (int64_t)n_ps[e] * SLAB_ROWS;
        const int32_t* r = rank_rows.data() + row_off[e];
        for (int64_t k = 0; k < n; ++k) {
            if (r[k] != (int32_t)k) identity = false;
            if ((k & 7) == 0 ? (r[k] < 0 || (r[k] & 7) != 0) : (r[k] != r[k - 1] + 1)) chunked8 = false;
        }
    }
    set->rank_chunked8 = chunked8;
    set->rank_identity = identity;
    // one width per expert and the same slab count everywhere (what the kernel that forms both projections in one
    // workgroup still assumes)?  The walking kernel itself only needs whole groups of one width: true by construction.
    bool all_affine = role == ROLE_GATE_UP;
    for (int e = 0; e < E && all_affine; ++e) {
        if (n_ps[e] != pms) all_affine = false;
        for (int ps = 1; ps < n_ps[e] && all_affine; ++ps)
            if (fslabs[(size_t)e * pms + ps].bits != fslabs[(size_t)e * pms].bits) all_affine = false;
    }
    set->all_uniform8 = role == ROLE_GATE_UP;
    set->all_affine = all_affine;
    set->vector_aligned = true;       // (the prepared tables are the library's own, 256-byte aligned allocations)

    BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_prepared, (size_t)std::max<int64_t>(pay_words, 1) * 4));
    // one allocation for the row tables: rank' (i32), source of every row (i32), s' (f16), scale' (f16)
    const size_t rows_bytes = 2 * (size_t)round_up(rows_total * 4, 256) + (size_t)round_up(rows_total * 2, 256) +
                              (size_t)round_up(scale_total * 2, 256);
    BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_prepared_rows, std::max<size_t>(rows_bytes, 256)));
    int32_t* d_rank = (int32_t*)set->d_prepared_rows;
    int32_t* d_src = (int32_t*)((char*)d_rank + round_up(rows_total * 4, 256));
    __half* d_s = (__half*)((char*)d_src + round_up(rows_total * 4, 256));
    __half* d_scale = (__half*)((char*)d_s + round_up(rows_total * 2, 256));
    if (role == ROLE_GATE_UP)
        BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_scale_s, (size_t)std::max<int64_t>(scale_total, 1) * 2));
    BITSMOE_HIP_TRY(hipMemcpyAsync(d_rank, rank_rows.data(), (size_t)rows_total * 4, hipMemcpyHostToDevice, st));
    BITSMOE_HIP_TRY(hipMemcpyAsync(d_src, row_src.data(), (size_t)rows_total * 4, hipMemcpyHostToDevice, st));
    BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_prep_tasks, sizeof(SlabTask) * std::max<size_t>(tasks.size(), 1)));
    BITSMOE_HIP_TRY(hipMemcpyAsync(set->d_prep_tasks, tasks.data(), sizeof(SlabTask) * tasks.size(), hipMemcpyHostToDevice, st));

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
        f.num_slabs = n_ps[e];
        f.uniform_bits = fslabs[(size_t)e * pms].bits;
        for (int ps = 1; ps < n_ps[e]; ++ps)
            if (fslabs[(size_t)e * pms + ps].bits != f.uniform_bits) f.uniform_bits = 0;
        set->expert_bits[e] = (uint8_t)f.uniform_bits;
    }
    set->uniform_experts = true;
    for (int e = 0; e < E; ++e)
        if (set->expert_bits[e] == 0) set->uniform_experts = false;
    set->has_cost_order = E <= EXPERT_ORDER_MAX;
    if (set->has_cost_order) {
        std::vector<int> order(E);
        for (int e = 0; e < E; ++e) order[e] = e;
        auto words = [&](int e) {       // payload words per tile of expert e
            int64_t w = 0;
            for (int ps = 0; ps < n_ps[e]; ++ps) w += fslabs[(size_t)e * pms + ps].bits;
            return w;
        };
        std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return words(a) > words(b); });
        for (int e = 0; e < E; ++e) set->cost_order[e] = (uint16_t)order[e];
    }
    BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_fast_experts, sizeof(FastExpert) * fexp.size()));
    BITSMOE_HIP_TRY(hipMemcpyAsync(set->d_fast_experts, fexp.data(), sizeof(FastExpert) * fexp.size(), hipMemcpyHostToDevice, st));
    BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_fast_slabs, sizeof(FastSlab) * fslabs.size()));
    BITSMOE_HIP_TRY(hipMemcpyAsync(set->d_fast_slabs, fslabs.data(), sizeof(FastSlab) * fslabs.size(), hipMemcpyHostToDevice, st));
    const PrepSource ps_tab{d_src, d_rank};
    hipLaunchKernelGGL(k_prepare_rows, dim3((unsigned)tasks.size(), n_tiles), dim3(64), 0, st, set->d_views,
                       set->d_fast_experts, set->d_fast_slabs, pms, set->d_prep_tasks, ps_tab);
    BITSMOE_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(k_prepack, dim3((unsigned)tasks.size(), n_tiles), dim3(256), 0, st, set->d_views,
                       set->d_fast_experts, set->d_fast_slabs, pms, set->d_prep_tasks, ps_tab, role);
    BITSMOE_HIP_TRY(hipGetLastError());
    // The side table of wide rows: an expert's rows of 6-, 8- and 16-bit slabs in their local order, 64 to a slab.
    const int64_t n_ws = wide_first[E];
    std::vector<int32_t> wide_tab;
    if (n_ws > 0) {
        std::vector<int32_t> wide_experts, slab_expert((size_t)n_ws);
        std::vector<int32_t> wrank((size_t)n_ws * SLAB_ROWS, -1), wsrc((size_t)n_ws * SLAB_ROWS, -1);
        for (int e = 0; e < E; ++e) {
            if (wide_first[e + 1] > wide_first[e]) wide_experts.push_back(e);
            for (int32_t j = wide_first[e]; j < wide_first[e + 1]; ++j) slab_expert[j] = e;
            const auto& slab = set->slab_meta_host[e];
            const auto& rk = set->rank_idx_host[e];
            int64_t p = (int64_t)wide_first[e] * SLAB_ROWS;
            for (int si = 0; si < set->descs[e].num_slabs; ++si) {
                if (!is_wide(slab[si * 4 + 0])) continue;
                for (int r = 0; r < slab[si * 4 + 1]; ++r, ++p) {
                    wrank[p] = rk[slab[si * 4 + 2] + r];
                    wsrc[p] = (si << 8) | r;
                }
            }
        }
        // one allocation: wide_first [E + 1], wide_experts, slab_expert, rank', source (int32 each), then s' (f16)
        const size_t n_int = (size_t)(E + 1) + wide_experts.size() + slab_expert.size() + wrank.size() + wsrc.size();
        const size_t int_bytes = (size_t)round_up((int64_t)n_int * 4, 256);
        BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_wide_tables, int_bytes + (size_t)n_ws * SLAB_ROWS * 2));
        BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_wide, (size_t)n_ws * n_tiles * WIDE_BLOCK * 2));
        wide_tab.reserve(n_int);
        wide_tab.insert(wide_tab.end(), wide_first.begin(), wide_first.end());
        wide_tab.insert(wide_tab.end(), wide_experts.begin(), wide_experts.end());
        wide_tab.insert(wide_tab.end(), slab_expert.begin(), slab_expert.end());
        wide_tab.insert(wide_tab.end(), wrank.begin(), wrank.end());
        wide_tab.insert(wide_tab.end(), wsrc.begin(), wsrc.end());
        BITSMOE_HIP_TRY(hipMemcpyAsync(set->d_wide_tables, wide_tab.data(), n_int * 4, hipMemcpyHostToDevice, st));
        set->d_wide_first = set->d_wide_tables;
        set->d_wide_experts = set->d_wide_first + (E + 1);
        const int32_t* d_slab_expert = set->d_wide_experts + wide_experts.size();
        set->d_wide_rank = d_slab_expert + slab_expert.size();
        set->d_wide_src = set->d_wide_rank + wrank.size();
        set->d_wide_s = (const __half*)((const char*)set->d_wide_tables + int_bytes);
        set->n_wide_experts = (int32_t)wide_experts.size();
        hipLaunchKernelGGL(k_prepack_wide, dim3((unsigned)n_ws, n_tiles), dim3(256), 0, st, set->d_views, d_slab_expert,
                           set->d_wide_src, role, n_tiles, set->d_wide, const_cast<__half*>(set->d_wide_s));
        BITSMOE_HIP_TRY(hipGetLastError());
    }
    set->wide_slabs = n_ws;
    set->narrow_rows = narrow_rows;
    set->wide_first_host = wide_first;
    BITSMOE_HIP_TRY(hipStreamSynchronize(st));      // (the host vectors above are read by the copies until here)
    set->fast_experts_host = fexp;
    set->prep_row_offsets = row_off;
    set->d_row_src = d_src;
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
    const FastExpert& fe = set->fast_experts_host[expert];
    const int32_t* d_src = set->d_row_src + set->prep_row_offsets[expert];
    hipLaunchKernelGGL(k_dequant_prepared, dim3(fe.num_slabs, set->n_tiles), dim3(256), 0, st, mv, fe,
                       set->d_fast_slabs + (int64_t)expert * set->prep_max_slabs, d_src, set->role, set->intermediate_size,
                       out_device);
    BITSMOE_HIP_TRY(hipGetLastError());
    if (set->wide_slabs > 0 && set->wide_first_host[expert + 1] > set->wide_first_host[expert]) {
        const int ws0 = set->wide_first_host[expert];
        hipLaunchKernelGGL(k_dequant_wide, dim3(set->wide_first_host[expert + 1] - ws0, set->n_tiles), dim3(256), 0, st, mv,
                           set->d_wide, set->d_wide_src, ws0, set->role, set->n_tiles, set->intermediate_size, out_device);
        BITSMOE_HIP_TRY(hipGetLastError());
    }
    return BITSMOE_OK;
}
