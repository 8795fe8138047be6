// The quantiser that defines the payload's contents and the slab packer, as kernels.
//
//   k_quantize_tiles   one wavefront per (row, 128-column tile): the symmetric quantiser of
//                      bitsmoe/quant/quantizer.py:30-84 -- 2/3/4 bits: scale_0 = mean|x|, then `iters` times
//                      { q = clamp(round_half_even(x / scale)); scale = max(mean(x q) / (mean(q q) + eps), eps) }
//                      with the means over the tile's real columns; 6/8 bits: absmax; 1 bit: sign, mean|x|.
//                      The levels returned are those of the last pass, the scale the one fitted to them.
//   k_pack_slabs       levels of one bit bucket -> payload words in the runtime order
//                      [slab of <= 64 rows][tile][stage of 16 rows][micro of 32 columns][row][plane]
//                      (bitsmoe/quant/packer.py:169-306) and scales in [slab][tile][row] order; the plane
//                      words come from wave64 ballots, two 32-column micro-tiles per wavefront.
//
// Sums run over a wavefront in a fixed order that differs from the framework's reduction order, so a
// scale can differ from the CPU restatement's in its last bit and a level with it where x / scale sits
// on a rounding tie; given equal levels the words are identical.
#include "common.h"

namespace bitsmoe {

__device__ inline float wave_sum_all(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
    return v;
}
__device__ inline float wave_max_all(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v = fmaxf(v, __shfl_xor(v, d));
    return v;
}

// grid-stride over (row, tile) units, one wavefront each; lane l holds columns l and l + 64 of the tile.
__global__ __launch_bounds__(256) void k_quantize_tiles(const float* __restrict__ rows, int64_t k, int64_t dim,
                                                        int64_t row_stride, int n_tiles, int bits, int iters, float eps,
                                                        int8_t* __restrict__ levels, float* __restrict__ scale_out) {
    const int lane = threadIdx.x & 63;
    const int64_t n_units = k * n_tiles;
    const int64_t wave0 = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t n_waves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    const float lo = (bits == 1) ? -1.0f : -(float)(1 << (bits - 1));
    const float hi = (bits == 1) ? 1.0f : (float)((1 << (bits - 1)) - 1);
    for (int64_t unit = wave0; unit < n_units; unit += n_waves) {
        const int64_t row = unit / n_tiles;
        const int t = (int)(unit - row * n_tiles);
        const int n_valid = (int)min((int64_t)N_TILE, dim - (int64_t)t * N_TILE);
        const float* src = rows + row * row_stride + (int64_t)t * N_TILE;
        const bool v0 = lane < n_valid, v1 = lane + 64 < n_valid;
        const float x0 = v0 ? src[lane] : 0.0f, x1 = v1 ? src[lane + 64] : 0.0f;
        const float inv_n = 1.0f / (float)n_valid;
        float q0 = 0.0f, q1 = 0.0f, scale;
        if (bits == 1) {
            scale = fmaxf(wave_sum_all(fabsf(x0) + fabsf(x1)) * inv_n, eps);
            q0 = x0 < 0.0f ? -1.0f : 1.0f;
            q1 = x1 < 0.0f ? -1.0f : 1.0f;
        } else if (bits <= 4) {
            scale = fmaxf(wave_sum_all(fabsf(x0) + fabsf(x1)) * inv_n, eps);
            for (int it = 0; it < iters; ++it) {
                q0 = fminf(fmaxf(rintf(x0 / scale), lo), hi);
                q1 = fminf(fmaxf(rintf(x1 / scale), lo), hi);
                if (!v0) q0 = 0.0f;
                if (!v1) q1 = 0.0f;
                const float xq = wave_sum_all(x0 * q0 + x1 * q1) * inv_n;
                const float qq = wave_sum_all(q0 * q0 + q1 * q1) * inv_n;
                scale = fmaxf(xq / (qq + eps), eps);
            }
        } else {
            scale = fmaxf(wave_max_all(fmaxf(fabsf(x0), fabsf(x1))) / hi, eps);
            q0 = fminf(fmaxf(rintf(x0 / scale), lo), hi);
            q1 = fminf(fmaxf(rintf(x1 / scale), lo), hi);
        }
        // levels are stored over whole tiles: padding columns hold level 0
        int8_t* dst = levels + (row * n_tiles + t) * N_TILE;
        dst[lane] = v0 ? (int8_t)q0 : (int8_t)0;
        dst[lane + 64] = v1 ? (int8_t)q1 : (int8_t)0;
        if (lane == 0) scale_out[row * n_tiles + t] = scale;
    }
}

__device__ inline unsigned code_of_level(int q, int bits) {
    return (bits == 1) ? (unsigned)((q + 1) >> 1) : (unsigned)(q + level_offset(bits));
}

// levels int8 [k, n_tiles * 128] of ONE bit bucket (rows in bucket order), scale fp32 [k, n_tiles] ->
// payload words and fp16 scales of the bucket's slabs (slab i = rows [64 i, 64 i + 64), the last one ragged).
// One wavefront per (row, tile, micro pair).
__global__ __launch_bounds__(256) void k_pack_slabs(const int8_t* __restrict__ levels, const float* __restrict__ scale,
                                                    int64_t k, int n_tiles, int bits, uint32_t* __restrict__ payload,
                                                    __half* __restrict__ scale_out) {
    const int lane = threadIdx.x & 63;
    const int64_t n_units = k * n_tiles * 2;
    const int64_t wave0 = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t n_waves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    const int w = bits;
    for (int64_t unit = wave0; unit < n_units; unit += n_waves) {
        const int half = (int)(unit & 1);
        const int64_t rt = unit >> 1;
        const int64_t row = rt / n_tiles;
        const int t = (int)(rt - row * n_tiles);
        const int64_t slab = row / K_SLAB;
        const int r_in = (int)(row - slab * K_SLAB);
        const int k_slab = (int)min((int64_t)K_SLAB, k - slab * K_SLAB);
        const int stage = r_in / K_STAGE, rr = r_in - stage * K_STAGE;
        const int rows_cur = min(K_STAGE, k_slab - stage * K_STAGE);
        // words before this slab: full slabs of 64 rows; inside: tile, stage, micro, row, plane
        const int64_t slab_base = slab * (int64_t)K_SLAB * n_tiles * MICROS * w;
        const int64_t tile_base = slab_base + (int64_t)t * k_slab * MICROS * w + (int64_t)stage * K_STAGE * MICROS * w;
        const unsigned code = code_of_level((int)levels[(row * n_tiles + t) * N_TILE + half * 64 + lane], bits) & 0xFFu;
        for (int p = 0; p < w; ++p) {
            const uint64_t bal = __ballot((code >> p) & 1u);
            if (lane == 0) {
                const int m0 = half * 2;
                payload[tile_base + (int64_t)m0 * rows_cur * w + rr * w + p] = (uint32_t)(bal & 0xFFFFFFFFull);
                payload[tile_base + (int64_t)(m0 + 1) * rows_cur * w + rr * w + p] = (uint32_t)(bal >> 32);
            }
        }
        if (half == 0 && lane == 0)
            scale_out[slab * (int64_t)K_SLAB * n_tiles + (int64_t)t * k_slab + r_in] = __float2half(scale[row * n_tiles + t]);
    }
}

}  // namespace bitsmoe

using namespace bitsmoe;

static bool quant_bits_ok(int bits) { return bits == 1 || bits == 2 || bits == 3 || bits == 4 || bits == 6 || bits == 8; }

extern "C" int bitsmoe_quantize_tiles(const float* rows, int64_t k, int64_t dim, int64_t row_stride, int32_t bits,
                                      int32_t iters, int8_t* levels_out, float* scale_out, void* stream) {
    BITSMOE_REQUIRE(quant_bits_ok(bits), "Unsupported bit width: %d", bits);
    BITSMOE_REQUIRE(k >= 0 && dim >= 0 && row_stride >= dim && iters >= 1, "invalid shape");
    if (k == 0 || dim == 0) return BITSMOE_OK;
    BITSMOE_REQUIRE(rows && levels_out && scale_out, "null pointer");
    const int64_t n_tiles = (dim + N_TILE - 1) / N_TILE;
    BITSMOE_REQUIRE(n_tiles < ((int64_t)1 << 24), "too many columns");
    const int64_t units = k * n_tiles;
    const int64_t blocks = std::min<int64_t>((units + 3) / 4, 65535);
    hipLaunchKernelGGL(k_quantize_tiles, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, rows, k, dim, row_stride,
                       (int)n_tiles, bits, iters, 1e-8f, levels_out, scale_out);
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}

extern "C" int bitsmoe_pack_slabs(const int8_t* levels, const float* scale, int64_t k, int64_t dim, int32_t bits,
                                  uint32_t* payload_out, void* scale_out_f16, void* stream) {
    BITSMOE_REQUIRE(quant_bits_ok(bits), "Unsupported bit width: %d", bits);
    BITSMOE_REQUIRE(k >= 0 && dim >= 0, "invalid shape");
    if (k == 0 || dim == 0) return BITSMOE_OK;
    BITSMOE_REQUIRE(levels && scale && payload_out && scale_out_f16, "null pointer");
    const int64_t n_tiles = (dim + N_TILE - 1) / N_TILE;
    BITSMOE_REQUIRE(n_tiles < ((int64_t)1 << 24), "too many columns");
    const int64_t units = k * n_tiles * 2;
    const int64_t blocks = std::min<int64_t>((units + 3) / 4, 65535);
    hipLaunchKernelGGL(k_pack_slabs, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, levels, scale, k, (int)n_tiles,
                       bits, payload_out, (__half*)scale_out_f16);
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}
