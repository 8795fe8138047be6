// Matrix sets: validation of the packed layout on the host, device tables, dense dequant.
#include "common.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>

namespace bitsmoe {

static thread_local std::string g_last_error;

void set_error(const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
}

int hip_fail(hipError_t e, const char* what) {
    set_error("HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
    return BITSMOE_E_HIP;
}

// One workgroup per (slab, tile): every thread decodes elements straight from global
// memory.  Parity/debug kernel, not a hot path.
__global__ __launch_bounds__(256) void k_dequant_matrix(MatView mv, int I, float* __restrict__ out) {
    const int si = blockIdx.x;
    const int tile_local = blockIdx.y;
    const int bits = mv.slab_meta[si * 4 + 0];
    const int k_slab = mv.slab_meta[si * 4 + 1];
    const int rank_off = mv.slab_meta[si * 4 + 2];
    const int tile_off = mv.slab_meta[si * 4 + 3];
    const int tile_end = (si + 1 < mv.num_slabs) ? mv.slab_meta[(si + 1) * 4 + 3] : mv.num_tiles;
    const int t = tile_off + tile_local;
    if (t >= tile_end) return;
    const int pack_off = mv.tile_meta[t * 3 + 0];
    const int scale_off = mv.tile_meta[t * 3 + 1];
    const int n_valid = mv.tile_meta[t * 3 + 2];
    const int w = words_per_row(bits);
    for (int idx = threadIdx.x; idx < k_slab * N_TILE; idx += blockDim.x) {
        const int row = idx / N_TILE;
        const int col = idx - row * N_TILE;
        const int c = tile_local * N_TILE + col;
        if (col >= n_valid || c >= I) continue;
        const int stage = row / K_STAGE;
        const int r = row - stage * K_STAGE;
        const int rows_cur = min(K_STAGE, k_slab - stage * K_STAGE);
        const int micro = col / N_MICRO;
        const int lane = col - micro * N_MICRO;
        const uint32_t* words =
            mv.payload + pack_off + stage * K_STAGE * MICROS * w + micro * rows_cur * w + r * w;
        float v = decode_from_row_words(words, bits, lane);
        if (bits != 16) v *= __half2float(mv.scale[scale_off + row]);
        out[(int64_t)(rank_off + row) * I + c] = v;
    }
}

__global__ void k_fill_zero(float* __restrict__ p, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = 0.0f;
}

int launch_fill_zero(float* p, int64_t n, hipStream_t st) {
    if (n <= 0) return BITSMOE_OK;
    const int64_t blocks = std::min<int64_t>((n + 255) / 256, 4096);
    hipLaunchKernelGGL(k_fill_zero, dim3((unsigned)blocks), dim3(256), 0, st, p, n);
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}

}  // namespace bitsmoe

using namespace bitsmoe;

extern "C" const char* bitsmoe_last_error(void) { return g_last_error.c_str(); }

namespace bitsmoe {
static int env_switch(const char* name) {
    const char* v = getenv(name);
    return v && v[0] ? atoi(v) : -1;
}
Options& options() {
    static Options o = [] {
        Options x;
        x.route_inline = env_switch("BITSMOE_ROUTE_INLINE");
        x.route_jobs = env_switch("BITSMOE_ROUTE_JOBS");
        x.decode_fused_z = env_switch("BITSMOE_DECODE_FUSED_Z");
        x.decode_split_z = env_switch("BITSMOE_DECODE_SPLIT_Z");
        x.decode_fused = env_switch("BITSMOE_DECODE_FUSED");
        x.prefill_split = env_switch("BITSMOE_PREFILL_SPLIT");
        x.router_wide = env_switch("BITSMOE_ROUTER_WIDE");
        return x;
    }();
    return o;
}
}  // namespace bitsmoe

extern "C" int bitsmoe_set_option(const char* name, int32_t value) {
    BITSMOE_REQUIRE(name != nullptr, "option name must not be null");
    Options& o = options();
    const std::string n(name);
    int* slot = n == "route_inline" ? &o.route_inline : n == "route_jobs" ? &o.route_jobs
                : n == "decode_fused_z" ? &o.decode_fused_z : n == "decode_split_z" ? &o.decode_split_z
                : n == "decode_fused" ? &o.decode_fused : n == "prefill_split" ? &o.prefill_split
                : n == "router_wide" ? &o.router_wide : nullptr;
    BITSMOE_REQUIRE(slot != nullptr, "unknown option '%s'", name);
    *slot = value < 0 ? -1 : (int)value;
    return BITSMOE_OK;
}
extern "C" const char* bitsmoe_version(void) { return "bitsmoe_hip 0.1 (gfx950)"; }

static int validate_matrix(const bitsmoe_matrix_desc& d, int e, int I,
                           const std::vector<int32_t>& slab, const std::vector<int32_t>& tile,
                           bool* regular, bool* regular64, bool* fast_ok) {
    const int n_tiles_mat = (I + N_TILE - 1) / N_TILE;
    int64_t rows_seen = 0;
    for (int s = 0; s < d.num_slabs; ++s) {
        const int bits = slab[s * 4 + 0], k_slab = slab[s * 4 + 1];
        const int rank_off = slab[s * 4 + 2], tile_off = slab[s * 4 + 3];
        const int tile_end = (s + 1 < d.num_slabs) ? slab[(s + 1) * 4 + 3] : d.num_tiles;
        BITSMOE_REQUIRE(bits_supported(bits), "expert %d slab %d: unsupported bits=%d", e, s, bits);
        BITSMOE_REQUIRE(k_slab >= 1 && k_slab <= K_SLAB, "expert %d slab %d: k_slab=%d outside [1,64]", e, s, k_slab);
        BITSMOE_REQUIRE(rank_off >= 0 && (int64_t)rank_off + k_slab <= d.rank_len,
                        "expert %d slab %d: rows [%d,%d) exceed rank_len=%d", e, s, rank_off, rank_off + k_slab, d.rank_len);
        BITSMOE_REQUIRE(tile_off >= 0 && tile_off <= tile_end && tile_end <= d.num_tiles,
                        "expert %d slab %d: tile range [%d,%d) exceeds num_tiles=%d", e, s, tile_off, tile_end, d.num_tiles);
        BITSMOE_REQUIRE(tile_end - tile_off <= n_tiles_mat,
                        "expert %d slab %d: %d tiles but intermediate_size=%d allows %d", e, s,
                        tile_end - tile_off, I, n_tiles_mat);
        if (!(bits == 2 || bits == 3 || bits == 4) || (k_slab % K_STAGE) != 0 ||
            tile_end - tile_off != n_tiles_mat)
            *regular = false;
        if (tile_end - tile_off != n_tiles_mat) *fast_ok = false;
        if (k_slab != K_SLAB) *regular64 = false;
        const int64_t words_tile = (int64_t)k_slab * MICROS * words_per_row(bits);
        for (int t = tile_off; t < tile_end; ++t) {
            const int64_t pack_off = tile[t * 3 + 0], scale_off = tile[t * 3 + 1];
            const int n_valid = tile[t * 3 + 2];
            BITSMOE_REQUIRE(pack_off >= 0 && pack_off + words_tile <= d.payload_words,
                            "expert %d tile %d: payload words [%lld,%lld) exceed payload size %lld", e, t,
                            (long long)pack_off, (long long)(pack_off + words_tile), (long long)d.payload_words);
            BITSMOE_REQUIRE(scale_off >= 0 && scale_off + k_slab <= d.scale_len,
                            "expert %d tile %d: scale range exceeds scale size %lld", e, t, (long long)d.scale_len);
            BITSMOE_REQUIRE(n_valid >= 1 && n_valid <= N_TILE, "expert %d tile %d: n_valid=%d outside [1,128]", e, t, n_valid);
            if (n_valid != N_TILE || (pack_off & 3) != 0) *regular = false;
            // (the last tile of a slab may be narrower: the matrix's own last columns)
            if (n_valid != N_TILE && !(t == tile_end - 1 && n_valid == I - (n_tiles_mat - 1) * N_TILE)) *fast_ok = false;
        }
        rows_seen += k_slab;
    }
    (void)rows_seen;
    return BITSMOE_OK;
}

extern "C" int bitsmoe_matset_create(const bitsmoe_matrix_desc* descs, int32_t n_experts,
                                     int32_t intermediate_size, void* stream, bitsmoe_matset** out) {
    BITSMOE_REQUIRE(out != nullptr, "out must not be null");
    *out = nullptr;
    BITSMOE_REQUIRE(n_experts >= 0, "n_experts must be >= 0");
    BITSMOE_REQUIRE(intermediate_size > 0, "intermediate_size must be > 0");
    BITSMOE_REQUIRE(descs != nullptr || n_experts == 0, "descs must not be null");
    hipStream_t st = (hipStream_t)stream;

    auto* set = new bitsmoe_matset();
    struct Guard {
        bitsmoe_matset* s;
        ~Guard() { if (s) bitsmoe_matset_destroy(s); }
    } guard{set};

    set->n_experts = n_experts;
    set->intermediate_size = intermediate_size;
    set->n_tiles = (intermediate_size + N_TILE - 1) / N_TILE;
    BITSMOE_HIP_TRY(hipGetDevice(&set->device));
    // the static scratch of this device is located now (a symbol query), so that bitsmoe_moe_forward_static
    // never has to make one -- its first call may come under stream capture
    if (static_scratch_of_current_device() == nullptr) return BITSMOE_E_HIP;
    set->descs.assign(descs, descs + n_experts);
    set->slab_meta_host.resize(n_experts);
    set->tile_meta_host.resize(n_experts);
    set->regular = n_experts > 0;
    set->regular64 = n_experts > 0;
    set->fast_ok = n_experts > 0;
    set->rank_idx_host.resize(n_experts);

    std::vector<MatView> views(n_experts);
    std::vector<SlabTask> tasks;
    std::vector<int32_t> rk;
    int max_rank = -1, min_rank = 0x7fffffff;
    bool chunked8 = n_experts > 0, identity = n_experts > 0;
    for (int e = 0; e < n_experts; ++e) {
        const bitsmoe_matrix_desc& d = descs[e];
        BITSMOE_REQUIRE(d.num_slabs >= 0 && d.num_tiles >= 0 && d.rank_len >= 0 && d.payload_words >= 0 && d.scale_len >= 0,
                        "expert %d: negative size", e);
        BITSMOE_REQUIRE(d.payload_words < (int64_t)1 << 31, "expert %d: payload larger than int32 word offsets allow", e);
        if (d.num_slabs > 0)
            BITSMOE_REQUIRE(d.payload && d.rank_idx && d.tile_meta && d.slab_meta && d.scale && d.s,
                            "expert %d: null buffer pointer", e);
        auto& slab = set->slab_meta_host[e];
        auto& tile = set->tile_meta_host[e];
        slab.resize((size_t)d.num_slabs * 4);
        tile.resize((size_t)d.num_tiles * 3);
        rk.resize((size_t)d.rank_len);
        if (!slab.empty())
            BITSMOE_HIP_TRY(hipMemcpyAsync(slab.data(), d.slab_meta, slab.size() * 4, hipMemcpyDeviceToHost, st));
        if (!tile.empty())
            BITSMOE_HIP_TRY(hipMemcpyAsync(tile.data(), d.tile_meta, tile.size() * 4, hipMemcpyDeviceToHost, st));
        if (!rk.empty())
            BITSMOE_HIP_TRY(hipMemcpyAsync(rk.data(), d.rank_idx, rk.size() * 4, hipMemcpyDeviceToHost, st));
        BITSMOE_HIP_TRY(hipStreamSynchronize(st));
        bool regular = true, regular64 = true, fast_ok = true;
        const int rc = validate_matrix(d, e, intermediate_size, slab, tile, &regular, &regular64, &fast_ok);
        if (rc != BITSMOE_OK) return rc;
        if (!fast_ok || d.num_slabs == 0) set->fast_ok = false;
        set->rank_idx_host[e] = rk;
        if (!regular || d.num_slabs == 0) set->regular = false;
        if (!regular || !regular64 || d.num_slabs == 0 || ((uintptr_t)d.payload & 15) != 0) set->regular64 = false;
        for (int32_t v : rk) {
            max_rank = std::max(max_rank, v);
            min_rank = std::min(min_rank, v);
        }
        for (size_t k = 0; k < rk.size() && identity; ++k) identity = rk[k] == (int32_t)k;
        for (int si = 0; si < d.num_slabs && chunked8; ++si)
            if (slab[si * 4 + 2] != si * K_SLAB) chunked8 = false;
        if (d.rank_len % 8 != 0) chunked8 = false;
        for (size_t k0 = 0; k0 + 8 <= rk.size() && chunked8; k0 += 8) {
            if (rk[k0] < 0 || rk[k0] % 8 != 0) chunked8 = false;
            for (int i = 1; i < 8; ++i)
                if (rk[k0 + i] != rk[k0] + i) chunked8 = false;
        }
        MatView& mv = views[e];
        mv.payload = (const uint32_t*)d.payload;
        mv.rank_idx = (const int32_t*)d.rank_idx;
        mv.tile_meta = (const int32_t*)d.tile_meta;
        mv.slab_meta = (const int32_t*)d.slab_meta;
        mv.scale = (const __half*)d.scale;
        mv.s = (const __half*)d.s;
        mv.num_slabs = d.num_slabs;
        mv.num_tiles = d.num_tiles;
        mv.rank_len = d.rank_len;
        mv.flags = regular ? 1 : 0;
        set->max_slabs = std::max(set->max_slabs, d.num_slabs);
        for (int s = 0; s < d.num_slabs; ++s) tasks.push_back(SlabTask{e, s});
    }
    set->rank_chunked8 = chunked8;
    set->rank_identity = identity;
    set->total_slabs = (int64_t)tasks.size();
    set->max_rank_plus1 = max_rank + 1;
    set->min_rank = (min_rank == 0x7fffffff) ? 0 : min_rank;

    if (n_experts > 0) {
        BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_views, sizeof(MatView) * n_experts));
        BITSMOE_HIP_TRY(hipMemcpyAsync(set->d_views, views.data(), sizeof(MatView) * n_experts, hipMemcpyHostToDevice, st));
    }
    if (!tasks.empty()) {
        BITSMOE_HIP_TRY(hipMalloc((void**)&set->d_slab_tasks, sizeof(SlabTask) * tasks.size()));
        BITSMOE_HIP_TRY(hipMemcpyAsync(set->d_slab_tasks, tasks.data(), sizeof(SlabTask) * tasks.size(), hipMemcpyHostToDevice, st));
    }
    BITSMOE_HIP_TRY(hipStreamSynchronize(st));
    guard.s = nullptr;
    *out = set;
    return BITSMOE_OK;
}

extern "C" void bitsmoe_matset_destroy(bitsmoe_matset* set) {
    if (!set) return;
    if (set->d_views) (void)hipFree(set->d_views);
    if (set->d_slab_tasks) (void)hipFree(set->d_slab_tasks);
    if (set->d_prepared) (void)hipFree(set->d_prepared);
    if (set->d_scale_s) (void)hipFree(set->d_scale_s);
    if (set->d_prepared_rows) (void)hipFree(set->d_prepared_rows);
    if (set->d_prep_tasks) (void)hipFree(set->d_prep_tasks);
    if (set->d_fast_experts) (void)hipFree(set->d_fast_experts);
    if (set->d_fast_slabs) (void)hipFree(set->d_fast_slabs);
    if (set->d_wide_tables) (void)hipFree(set->d_wide_tables);
    if (set->d_wide) (void)hipFree(set->d_wide);
    delete set;
}

extern "C" int bitsmoe_matset_info(const bitsmoe_matset* set, int64_t info[8]) {
    BITSMOE_REQUIRE(set && info, "null argument");
    info[0] = set->n_experts;
    info[1] = set->intermediate_size;
    info[2] = set->total_slabs;
    info[3] = set->max_rank_plus1;
    info[4] = set->regular ? 1 : 0;
    info[5] = set->max_slabs;
    info[6] = set->min_rank;
    info[7] = (set->fast_ok ? 1 : 0) | (set->role >= 0 ? 2 : 0) | (set->role == 0 && set->all_affine && set->rank_chunked8 ? 4 : 0) |
              (set->wide_slabs << 8);
    return BITSMOE_OK;
}

extern "C" int bitsmoe_dequant_matrix(const bitsmoe_matset* set, int32_t expert, float* out_device, void* stream) {
    BITSMOE_REQUIRE(set && out_device, "null argument");
    BITSMOE_REQUIRE(expert >= 0 && expert < set->n_experts, "expert %d out of range", expert);
    hipStream_t st = (hipStream_t)stream;
    const bitsmoe_matrix_desc& d = set->descs[expert];
    const int I = set->intermediate_size;
    int rc = launch_fill_zero(out_device, (int64_t)d.rank_len * I, st);
    if (rc != BITSMOE_OK) return rc;
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
    mv.flags = 0;
    hipLaunchKernelGGL(k_dequant_matrix, dim3(d.num_slabs, set->n_tiles), dim3(256), 0, st, mv, I, out_device);
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}

extern "C" int bitsmoe_profile_create(bitsmoe_profile** out) {
    BITSMOE_REQUIRE(out, "null argument");
    auto* p = new bitsmoe_profile();
    for (int i = 0; i <= BITSMOE_PROFILE_PHASES; ++i) {
        hipError_t e = hipEventCreate(&p->ev[i]);
        if (e != hipSuccess) {
            for (int j = 0; j < i; ++j) (void)hipEventDestroy(p->ev[j]);
            delete p;
            return hip_fail(e, "hipEventCreate");
        }
    }
    *out = p;
    return BITSMOE_OK;
}

extern "C" void bitsmoe_profile_destroy(bitsmoe_profile* p) {
    if (!p) return;
    for (int i = 0; i <= BITSMOE_PROFILE_PHASES; ++i) (void)hipEventDestroy(p->ev[i]);
    delete p;
}

extern "C" int bitsmoe_profile_read(bitsmoe_profile* p, float ms[BITSMOE_PROFILE_PHASES]) {
    BITSMOE_REQUIRE(p && ms, "null argument");
    BITSMOE_REQUIRE(p->recorded, "profile holds no recorded forward");
    for (int i = 0; i < BITSMOE_PROFILE_PHASES; ++i)
        BITSMOE_HIP_TRY(hipEventElapsedTime(&ms[i], p->ev[i], p->ev[i + 1]));
    return BITSMOE_OK;
}
