// Bit-plane pack / unpack of quantised levels with wave64 ballots: one wavefront turns 64
// consecutive columns of one row into the plane words of two 32-column groups.
#include "common.h"

namespace bitsmoe {

__device__ inline unsigned code_from_level(int q, int bits) {
    return (bits == 1) ? (unsigned)((q + 1) >> 1) : (unsigned)(q + level_offset(bits));
}

__global__ __launch_bounds__(256) void k_pack_bitplanes(const int8_t* __restrict__ levels, int64_t rows,
                                                         int64_t cols, int groups, int bits,
                                                         uint32_t* __restrict__ words) {
    const int lane = threadIdx.x & 63;
    const int pairs = (groups + 1) / 2;
    const int64_t n_units = rows * pairs;
    const int64_t wave0 = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t n_waves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    for (int64_t unit = wave0; unit < n_units; unit += n_waves) {
        const int64_t row = unit / pairs;
        const int pair = (int)(unit - row * pairs);
        const int64_t col = (int64_t)pair * 64 + lane;
        unsigned code = 0;
        if (col < cols) code = code_from_level((int)levels[row * cols + col], bits) & 0xFFu;
        for (int p = 0; p < bits; ++p) {
            const uint64_t bal = __ballot((code >> p) & 1u);
            if (lane == 0) {
                const int g0 = pair * 2;
                words[(row * groups + g0) * bits + p] = (uint32_t)(bal & 0xFFFFFFFFull);
                if (g0 + 1 < groups) words[(row * groups + g0 + 1) * bits + p] = (uint32_t)(bal >> 32);
            }
        }
    }
}

__global__ __launch_bounds__(256) void k_unpack_bitplanes(const uint32_t* __restrict__ words, int64_t rows,
                                                           int groups, int bits, int8_t* __restrict__ levels) {
    const int64_t n = rows * groups * 32;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const int64_t rg = i >> 5;  // (row, group)
        const int lane = (int)(i & 31);
        const uint32_t* w = words + rg * bits;
        int u = 0;
        for (int p = 0; p < bits; ++p) u |= (int)((w[p] >> lane) & 1u) << p;
        levels[i] = (int8_t)((bits == 1) ? (2 * u - 1) : (u - level_offset(bits)));
    }
}

}  // namespace bitsmoe

using namespace bitsmoe;

static bool pack_bits_ok(int bits) { return bits == 1 || bits == 2 || bits == 3 || bits == 4 || bits == 6 || bits == 8; }

extern "C" int bitsmoe_pack_bitplanes(const int8_t* levels, int64_t rows, int64_t cols, int32_t bits,
                                      uint32_t* words_out, void* stream) {
    BITSMOE_REQUIRE(pack_bits_ok(bits), "Unsupported bit width: %d", bits);
    BITSMOE_REQUIRE(rows >= 0 && cols >= 0, "invalid shape");
    if (rows == 0 || cols == 0) return BITSMOE_OK;
    BITSMOE_REQUIRE(levels && words_out, "null pointer");
    const int64_t groups = (cols + 31) / 32;
    BITSMOE_REQUIRE(groups < ((int64_t)1 << 30), "too many columns");
    const int64_t units = rows * ((groups + 1) / 2);
    const int64_t blocks = std::min<int64_t>((units + 3) / 4, 65535);
    hipLaunchKernelGGL(k_pack_bitplanes, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, levels, rows,
                       cols, (int)groups, bits, words_out);
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}

extern "C" int bitsmoe_unpack_bitplanes(const uint32_t* words, int64_t rows, int64_t groups, int32_t bits,
                                        int8_t* levels_out, void* stream) {
    BITSMOE_REQUIRE(pack_bits_ok(bits), "Unsupported bit width: %d", bits);
    BITSMOE_REQUIRE(rows >= 0 && groups >= 0 && groups < ((int64_t)1 << 30), "invalid shape");
    if (rows == 0 || groups == 0) return BITSMOE_OK;
    BITSMOE_REQUIRE(words && levels_out, "null pointer");
    const int64_t n = rows * groups * 32;
    const int64_t blocks = std::min<int64_t>((n + 255) / 256, 65535);
    hipLaunchKernelGGL(k_unpack_bitplanes, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, words, rows,
                       (int)groups, bits, levels_out);
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}
