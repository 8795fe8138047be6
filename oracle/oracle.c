/*
 * oracle.c — plain-C CPU restatement of the reference's mixed-bit MoE routed-expert path.
 *
 * TEST INFRASTRUCTURE ONLY: loaded by tests/, __graft_entry__.smoke() and the cpu_baseline
 * leg of bench.py; never linked into or called by the product library.
 *
 * The reference has no CPU implementation of this path (bitsmoe/models/base_block.py:428-438
 * raises without the CUDA extension), so this file restates the arithmetic of the CUDA
 * kernels for the host:
 *   decode rule        bitsmoe/algorithms/cpp/mlp_forward.cu:215-265 (decode_tile_weight),
 *                      74-84 (bits_offset)
 *   gate / up          mlp_forward.cu:1043-1206 (gate_up_small_warp_accumulate): fp32
 *                      acc += (h * s) * (q * scale)
 *   SiLU * up          mlp_forward.cu:86-88, 2073-2094
 *   down + combine     mlp_forward.cu:2145-2404 (down_small_kernel): per-(row, tile) dot,
 *                      times scale, then acc * s * route_w added to rank_accum
 *   routing            bitsmoe/models/base_block.py:258-289 (stable order inside an expert)
 * It is pinned against oracle/ref_oracle.py (numpy) in tests/test_oracle_c.py, which is in
 * turn pinned by known-answer vectors and closed forms.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define K_STAGE 16
#define N_TILE 128
#define N_MICRO 32
#define MICROS 4

typedef struct oracle_matrix {
    const uint32_t* payload;
    const int32_t* rank_idx;
    const int32_t* tile_meta; /* [num_tiles][3] pack_off, scale_off, n_valid */
    const int32_t* slab_meta; /* [num_slabs][4] bits, k_slab, rank_off, tile_off */
    const uint16_t* scale;    /* fp16 bits */
    const uint16_t* s;        /* fp16 bits */
    int32_t num_slabs;
    int32_t num_tiles;
    int32_t rank_len;
    int32_t pad;
} oracle_matrix;

static float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                man <<= 1;
                ++e;
            } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static int level_offset(int bits) {
    switch (bits) {
        case 2: return 2;
        case 3: return 4;
        case 4: return 8;
        case 6: return 32;
        case 8: return 128;
        default: return 0;
    }
}

/* Decode one row of one tile (128 columns, unscaled levels or stored halves). */
static void decode_row(const uint32_t* tile_words, int bits, int k_slab, int row, float* out128) {
    const int w = bits == 16 ? 16 : bits;
    const int stage = row / K_STAGE;
    const int r = row - stage * K_STAGE;
    int rows_cur = k_slab - stage * K_STAGE;
    if (rows_cur > K_STAGE) rows_cur = K_STAGE;
    const uint32_t* stage_words = tile_words + (size_t)stage * K_STAGE * MICROS * w;
    for (int micro = 0; micro < MICROS; ++micro) {
        const uint32_t* rw = stage_words + (size_t)micro * rows_cur * w + (size_t)r * w;
        float* o = out128 + micro * N_MICRO;
        if (bits == 16) {
            for (int l = 0; l < N_MICRO; ++l) {
                const uint32_t word = rw[l >> 1];
                o[l] = half_to_float((uint16_t)((l & 1) ? (word >> 16) : (word & 0xFFFFu)));
            }
        } else {
            const int off = level_offset(bits);
            for (int l = 0; l < N_MICRO; ++l) {
                int u = 0;
                for (int p = 0; p < bits; ++p) u |= (int)((rw[p] >> l) & 1u) << p;
                o[l] = (float)(bits == 1 ? 2 * u - 1 : u - off);
            }
        }
    }
}

void oracle_dequant_matrix(const oracle_matrix* m, int32_t I, float* out) {
    memset(out, 0, sizeof(float) * (size_t)m->rank_len * (size_t)I);
    for (int si = 0; si < m->num_slabs; ++si) {
        const int bits = m->slab_meta[si * 4 + 0], k_slab = m->slab_meta[si * 4 + 1];
        const int rank_off = m->slab_meta[si * 4 + 2], tile_off = m->slab_meta[si * 4 + 3];
        const int tile_end = (si + 1 < m->num_slabs) ? m->slab_meta[(si + 1) * 4 + 3] : m->num_tiles;
        for (int t = tile_off; t < tile_end; ++t) {
            const int pack_off = m->tile_meta[t * 3 + 0], scale_off = m->tile_meta[t * 3 + 1];
            const int n_valid = m->tile_meta[t * 3 + 2];
            const int c0 = (t - tile_off) * N_TILE;
            float row[N_TILE];
            for (int r = 0; r < k_slab; ++r) {
                decode_row(m->payload + pack_off, bits, k_slab, r, row);
                const float sc = bits == 16 ? 1.0f : half_to_float(m->scale[scale_off + r]);
                for (int c = 0; c < n_valid && c0 + c < I; ++c)
                    out[(size_t)(rank_off + r) * I + c0 + c] = bits == 16 ? row[c] : row[c] * sc;
            }
        }
    }
}

/* out[a - a0][c] (+)= sum_rows (h[tok_a, rank_idx[row]] * s[row]) * (level * scale) for one
 * expert matrix and one 128-column tile. */
static void gate_tile(const oracle_matrix* m, int tile_local, int32_t I, const float* h, int R, int T,
                      const int32_t* tok, int a0, int a1, float* out /* [a1-a0][I] */) {
    float row[N_TILE];
    for (int si = 0; si < m->num_slabs; ++si) {
        const int bits = m->slab_meta[si * 4 + 0], k_slab = m->slab_meta[si * 4 + 1];
        const int rank_off = m->slab_meta[si * 4 + 2], tile_off = m->slab_meta[si * 4 + 3];
        const int tile_end = (si + 1 < m->num_slabs) ? m->slab_meta[(si + 1) * 4 + 3] : m->num_tiles;
        const int t = tile_off + tile_local;
        if (t >= tile_end) continue;
        const int pack_off = m->tile_meta[t * 3 + 0], scale_off = m->tile_meta[t * 3 + 1];
        int n_valid = m->tile_meta[t * 3 + 2];
        const int c0 = tile_local * N_TILE;
        if (c0 + n_valid > I) n_valid = I - c0;
        for (int r = 0; r < k_slab; ++r) {
            decode_row(m->payload + pack_off, bits, k_slab, r, row);
            const float sc = bits == 16 ? 1.0f : half_to_float(m->scale[scale_off + r]);
            const int rk = m->rank_idx[rank_off + r];
            const float sv = half_to_float(m->s[rank_off + r]);
            if (rk < 0 || rk >= R) continue;
            if (bits != 16)
                for (int c = 0; c < n_valid; ++c) row[c] *= sc;
            for (int a = a0; a < a1; ++a) {
                const int tk = tok[a];
                if (tk < 0 || tk >= T) continue;
                const float hs = h[(size_t)tk * R + rk] * sv;
                float* o = out + (size_t)(a - a0) * I + c0;
                for (int c = 0; c < n_valid; ++c) o[c] += hs * row[c];
            }
        }
    }
}

static float silu(float x) { return x / (1.0f + expf(-x)); }

/* rank_accum [T, rank_out] is fully overwritten.  h_gate / h_up are fp32 copies of the
 * (fp16 or bf16) activations.  Returns 0, or -1 when scratch memory cannot be allocated. */
int oracle_moe_forward(const oracle_matrix* gate, const oracle_matrix* up, const oracle_matrix* down,
                       int32_t n_experts, const float* h_gate, const float* h_up, int32_t T, int32_t Rg,
                       int32_t Ru, const int32_t* tok, const int32_t* off, const float* rw, int32_t rank_out,
                       int32_t I, float* rank_accum, int32_t n_threads) {
    memset(rank_accum, 0, sizeof(float) * (size_t)T * (size_t)rank_out);
    const int A = off[n_experts];
    if (A <= 0) return 0;
    float* G = (float*)calloc((size_t)A * I, sizeof(float));
    float* U = (float*)calloc((size_t)A * I, sizeof(float));
    if (!G || !U) {
        free(G);
        free(U);
        return -1;
    }
    const int n_tiles = (I + N_TILE - 1) / N_TILE;
#ifdef _OPENMP
    if (n_threads > 0) omp_set_num_threads(n_threads);
#endif
    /* gate and up: one task per (expert, projection, tile) */
    const long n_tasks = (long)n_experts * 2 * n_tiles;
#pragma omp parallel for schedule(dynamic, 1)
    for (long task = 0; task < n_tasks; ++task) {
        const int e = (int)(task / (2 * n_tiles));
        const int rem = (int)(task % (2 * n_tiles));
        const int mt = rem / n_tiles, tile = rem % n_tiles;
        const int a0 = off[e], a1 = off[e + 1];
        if (a1 <= a0) continue;
        if (mt == 0)
            gate_tile(&gate[e], tile, I, h_gate, Rg, T, tok, a0, a1, G + (size_t)a0 * I);
        else
            gate_tile(&up[e], tile, I, h_up, Ru, T, tok, a0, a1, U + (size_t)a0 * I);
    }
    /* z = silu(G) * U, in place in G */
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)A * I; ++i) G[i] = silu(G[i]) * U[i];
    /* down: one task per (expert, slab); rows of one task are distinct output ranks, tasks
     * of different experts may hit the same (token, rank) -> atomic adds */
    long total_slabs = 0;
    for (int e = 0; e < n_experts; ++e) total_slabs += down[e].num_slabs;
    int32_t* task_e = (int32_t*)malloc(sizeof(int32_t) * (size_t)(total_slabs > 0 ? total_slabs : 1));
    int32_t* task_s = (int32_t*)malloc(sizeof(int32_t) * (size_t)(total_slabs > 0 ? total_slabs : 1));
    if (!task_e || !task_s) {
        free(G); free(U); free(task_e); free(task_s);
        return -1;
    }
    long n = 0;
    for (int e = 0; e < n_experts; ++e)
        for (int s = 0; s < down[e].num_slabs; ++s) {
            task_e[n] = e;
            task_s[n++] = s;
        }
#pragma omp parallel for schedule(dynamic, 1)
    for (long task = 0; task < total_slabs; ++task) {
        const int e = task_e[task], si = task_s[task];
        const int a0 = off[e], a1 = off[e + 1];
        if (a1 <= a0) continue;
        const oracle_matrix* m = &down[e];
        const int bits = m->slab_meta[si * 4 + 0], k_slab = m->slab_meta[si * 4 + 1];
        const int rank_off = m->slab_meta[si * 4 + 2], tile_off = m->slab_meta[si * 4 + 3];
        const int tile_end = (si + 1 < m->num_slabs) ? m->slab_meta[(si + 1) * 4 + 3] : m->num_tiles;
        float row[N_TILE];
        const int n_a = a1 - a0;
        float* accs = (float*)malloc(sizeof(float) * (size_t)n_a);
        if (!accs) continue;
        for (int r = 0; r < k_slab; ++r) {
            const int lr = m->rank_idx[rank_off + r];
            if (lr < 0 || lr >= rank_out) continue;
            const float sv = half_to_float(m->s[rank_off + r]);
            for (int a = 0; a < n_a; ++a) accs[a] = 0.0f;
            for (int t = tile_off; t < tile_end; ++t) {
                const int pack_off = m->tile_meta[t * 3 + 0], scale_off = m->tile_meta[t * 3 + 1];
                int n_valid = m->tile_meta[t * 3 + 2];
                const int c0 = (t - tile_off) * N_TILE;
                if (c0 + n_valid > I) n_valid = I - c0;
                decode_row(m->payload + pack_off, bits, k_slab, r, row);
                const float sc = bits == 16 ? 1.0f : half_to_float(m->scale[scale_off + r]);
                for (int a = 0; a < n_a; ++a) {
                    const float* z = G + (size_t)(a0 + a) * I + c0;
                    float dot = 0.0f;
                    for (int c = 0; c < n_valid; ++c) dot += row[c] * z[c];
                    accs[a] += dot * sc;
                }
            }
            for (int a = 0; a < n_a; ++a) {
                const int tk = tok[a0 + a];
                if (tk < 0 || tk >= T) continue;
                const float v = accs[a] * sv * rw[a0 + a];
#pragma omp atomic
                rank_accum[(size_t)tk * rank_out + lr] += v;
            }
        }
        free(accs);
    }
    free(G);
    free(U);
    free(task_e);
    free(task_s);
    return 0;
}

/* Stable counting sort of the flat (token-major) top-k list by local expert id. */
void oracle_route(const int64_t* selected, const float* weights, const int32_t* g2l, int32_t n_global,
                  int64_t n_tokens, int32_t top_k, int32_t n_packed, int32_t* token_indices,
                  int32_t* expert_offsets, float* route_flat) {
    const int64_t n_flat = n_tokens * top_k;
    for (int e = 0; e <= n_packed; ++e) expert_offsets[e] = 0;
    for (int64_t i = 0; i < n_flat; ++i) {
        const int64_t g = selected[i];
        if (g < 0 || g >= n_global) continue;
        const int l = g2l[g];
        if (l >= 0 && l < n_packed) expert_offsets[l + 1]++;
    }
    for (int e = 0; e < n_packed; ++e) expert_offsets[e + 1] += expert_offsets[e];
    int32_t* cursor = (int32_t*)malloc(sizeof(int32_t) * (size_t)(n_packed > 0 ? n_packed : 1));
    for (int e = 0; e < n_packed; ++e) cursor[e] = expert_offsets[e];
    for (int64_t i = 0; i < n_flat; ++i) {
        const int64_t g = selected[i];
        if (g < 0 || g >= n_global) continue;
        const int l = g2l[g];
        if (l < 0 || l >= n_packed) continue;
        const int pos = cursor[l]++;
        token_indices[pos] = (int32_t)(i / top_k);
        route_flat[pos] = weights[i];
    }
    free(cursor);
}

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
