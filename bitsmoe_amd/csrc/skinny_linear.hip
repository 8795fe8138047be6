// A bias-free linear layer for a FEW rows: out[T, N] = x[T, K] * W[N, K]^T with T <= 64, 16-bit x / W / out, fp32 sums.
// The two GEMMs around the routed-expert operator (the row-stacked shared-basis / router / shared-expert projections
// in, the column-stacked output projections out: bitsmoe/models/qwen3moe/bitsmoe_block.py:63-64,
// bitsmoe/models/base_block.py:414) are this shape at decode sizes: tens of MB of weights against a handful of tokens,
// i.e. a stream of W at HBM speed, which general GEMM kernels tiled for square problems reach a fraction of.
// W stays in the framework's [out_features, in_features] layout: a lane's 16 bytes of a weight row are eight
// consecutive contraction indices, which is what the 16x16x32 MFMA takes as its second operand.
// A workgroup owns 16 * NBW output columns; its four wavefronts contract a quarter of K each, two batches of four
// k-steps in flight (every load of a batch is out before the previous batch's MFMAs run), and add up in LDS.
#include "common.h"

#include <algorithm>

namespace bitsmoe {

typedef float sk_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t sk_u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 sk_f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 sk_bf16x8 __attribute__((ext_vector_type(8)));

constexpr int SK_U = 4;      // k-steps per batch of loads

// XF32: x is fp32 and is rounded to the 16-bit type on its way into the MFMA (the cast of the operator's fp32 output in
// front of the output projection, bitsmoe/models/base_block.py:414, without a pass of its own); one 16-row block only.
// PREP: W was re-laid out once (bitsmoe_prepare_linear_weight) into the order the MFMA takes it: [16-column block]
// [k-step of 32][lane][8 values], so that a wavefront's load is 1 KB of consecutive memory instead of sixteen 64-byte
// pieces of sixteen rows.
template <bool BF16, int NMB, int NBW, bool XF32 = false, bool PREP = false>
__global__ __launch_bounds__(256) void k_skinny_linear(const void* __restrict__ x_any, int64_t ld_x, const uint16_t* __restrict__ w,
                                                       int T, int K, int N, uint16_t* __restrict__ out, int64_t ld_out,
                                                       const float* __restrict__ addend, int64_t ld_add) {
    static_assert(!XF32 || NMB == 1, "fp32 rows: one block of 16 rows");
    const uint16_t* __restrict__ x = reinterpret_cast<const uint16_t*>(x_any);
    const float* __restrict__ xf = reinterpret_cast<const float*>(x_any);
    __shared__ float part[4][NMB * 16][NBW * 16 + 1];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int n0 = blockIdx.x * (NBW * 16);
    const int kq = K >> 2;                       // contraction range of this wavefront (a multiple of 32)
    const int kbase = wv * kq + (lane >> 4) * 8;
    const uint16_t* xp[NMB];
    const uint16_t* wp[NBW];
    const float* xfp = xf + (int64_t)min(lane & 15, T - 1) * ld_x + kbase;
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb) xp[mb] = x + (int64_t)min(mb * 16 + (lane & 15), T - 1) * ld_x + kbase;
#pragma unroll
    for (int nb = 0; nb < NBW; ++nb) {
        if constexpr (PREP)      // (N is a multiple of 16 * NBW there; step ks of this wavefront: + (ks / 32) * 512 elements)
            wp[nb] = w + ((int64_t)(blockIdx.x * NBW + nb) * (K >> 5) + wv * (kq >> 5)) * 512 + lane * 8;
        else
            wp[nb] = w + (int64_t)min(n0 + nb * 16 + (lane & 15), N - 1) * K + kbase;
    }
    sk_f32x4 acc[NMB][NBW];
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) acc[mb][nb] = sk_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    sk_u32x4 a[2][SK_U][NMB], b[2][SK_U][NBW];
    sk_f32x4 af[2][SK_U][XF32 ? 2 : 1];      // (fp32 rows as loaded: eight values per lane and k-step)
    auto request = [&](auto buf_c, int s0) {
        constexpr int B = decltype(buf_c)::value;
#pragma unroll
        for (int u = 0; u < SK_U; ++u) {
            const int ks = min(s0 + 32 * u, kq - 32);      // (a short last batch repeats its final step: masked below)
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb)
                b[B][u][nb] = *reinterpret_cast<const sk_u32x4*>(wp[nb] + (PREP ? ks * 16 : ks));
            if constexpr (XF32) {
                af[B][u][0] = *reinterpret_cast<const sk_f32x4*>(xfp + ks);
                af[B][u][1] = *reinterpret_cast<const sk_f32x4*>(xfp + ks + 4);
            } else {
#pragma unroll
                for (int mb = 0; mb < NMB; ++mb) a[B][u][mb] = *reinterpret_cast<const sk_u32x4*>(xp[mb] + ks);
            }
        }
    };
    auto round16 = [](float v) -> uint32_t {
        if constexpr (BF16)
            return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)v);
        else
            return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)v);
    };
    auto multiply = [&](auto buf_c, int s0) {
        constexpr int B = decltype(buf_c)::value;
#pragma unroll
        for (int u = 0; u < SK_U; ++u) {
            const bool live = s0 + 32 * u < kq;      // (no branch between the steps: a step past the end contributes zeros)
            if constexpr (XF32) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const sk_f32x4 v = af[B][u][c >> 1];
                    a[B][u][0][c] = round16(v[2 * (c & 1)]) | (round16(v[2 * (c & 1) + 1]) << 16);
                }
            }
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb) {
                sk_u32x4 bv = b[B][u][nb];
#pragma unroll
                for (int c = 0; c < 4; ++c) bv[c] = live ? bv[c] : 0u;
#pragma unroll
                for (int mb = 0; mb < NMB; ++mb) {
                    if constexpr (BF16)
                        acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(sk_bf16x8, a[B][u][mb]),
                                                                              __builtin_bit_cast(sk_bf16x8, bv), acc[mb][nb], 0, 0, 0);
                    else
                        acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(sk_f16x8, a[B][u][mb]),
                                                                             __builtin_bit_cast(sk_f16x8, bv), acc[mb][nb], 0, 0, 0);
                }
            }
        }
    };
    using B0 = std::integral_constant<int, 0>;
    using B1 = std::integral_constant<int, 1>;
    constexpr int STEP = 32 * SK_U;
    request(B0{}, 0);
    for (int s0 = 0; s0 < kq; s0 += 2 * STEP) {
        if (s0 + STEP < kq) request(B1{}, s0 + STEP);
        __builtin_amdgcn_sched_barrier(0);
        multiply(B0{}, s0);
        if (s0 + STEP < kq) {
            if (s0 + 2 * STEP < kq) request(B0{}, s0 + 2 * STEP);
            __builtin_amdgcn_sched_barrier(0);
            multiply(B1{}, s0 + STEP);
        }
    }
    // lane holds rows 16 mb + 4 (lane / 16) + j, column 16 nb + lane % 16
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb)
#pragma unroll
            for (int j = 0; j < 4; ++j) part[wv][mb * 16 + 4 * (lane >> 4) + j][nb * 16 + (lane & 15)] = acc[mb][nb][j];
    __syncthreads();
    // the four partial sums in a fixed order, two neighbouring columns per thread
    constexpr int PAIRS = NMB * 16 * NBW * 8;
    for (int i = threadIdx.x; i < PAIRS; i += 256) {
        const int row = i / (NBW * 8), c = (i - row * (NBW * 8)) * 2;
        if (row >= T || n0 + c >= N) continue;
        float v0 = part[0][row][c] + part[1][row][c] + part[2][row][c] + part[3][row][c];
        float v1 = part[0][row][c + 1] + part[1][row][c + 1] + part[2][row][c + 1] + part[3][row][c + 1];
        if (addend) {      // (fp32 [T, N] added to the sums before the one rounding of the result)
            v0 += addend[(int64_t)row * ld_add + n0 + c];
            v1 += addend[(int64_t)row * ld_add + n0 + c + 1];
        }
        uint32_t packed;
        if constexpr (BF16)
            packed = (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)v0) | ((uint32_t)__builtin_bit_cast(uint16_t, (__bf16)v1) << 16);
        else
            packed = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)v0) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)v1) << 16);
        *reinterpret_cast<uint32_t*>(out + (int64_t)row * ld_out + n0 + c) = packed;
    }
}

// W [N, K] -> [ceil(N / 16)][K / 32][64 lanes][8]: lane = 16 * (k % 32 / 8) + n % 16 holds W[n][32 ks + 8 (lane / 16) .. + 7];
// rows past N are zeros.  One thread per 16-byte piece.
__global__ __launch_bounds__(256) void k_prepare_linear_weight(const uint16_t* __restrict__ w, int N, int K, uint16_t* __restrict__ out,
                                                               int64_t pieces) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= pieces) return;
    const int lane = (int)(i & 63);
    const int64_t blk = i >> 6;
    const int ksteps = K >> 5;
    const int ks = (int)(blk % ksteps), nb = (int)(blk / ksteps);
    const int n = nb * 16 + (lane & 15), k = ks * 32 + (lane >> 4) * 8;
    sk_u32x4 v = {0u, 0u, 0u, 0u};
    if (n < N) v = *reinterpret_cast<const sk_u32x4*>(w + (int64_t)n * K + k);
    *reinterpret_cast<sk_u32x4*>(out + i * 8) = v;
}

}  // namespace bitsmoe

using namespace bitsmoe;

extern "C" int64_t bitsmoe_prepared_linear_weight_elements(int32_t in_features, int32_t out_features) {
    if (in_features <= 0 || out_features <= 0) return 0;
    return (int64_t)((out_features + 15) / 16) * 16 * in_features;
}

extern "C" int bitsmoe_prepare_linear_weight(const void* weight, int32_t in_features, int32_t out_features, void* prepared,
                                             void* stream) {
    BITSMOE_REQUIRE(in_features >= 128 && in_features % 128 == 0, "in_features must be a positive multiple of 128");
    BITSMOE_REQUIRE(out_features >= 1, "out_features must be positive");
    BITSMOE_REQUIRE(weight && prepared, "null pointer");
    BITSMOE_REQUIRE((((uintptr_t)weight | (uintptr_t)prepared) & 15) == 0, "weight and prepared must be 16-byte aligned");
    const int64_t pieces = bitsmoe_prepared_linear_weight_elements(in_features, out_features) / 8;
    hipLaunchKernelGGL(k_prepare_linear_weight, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t*)weight, out_features, in_features, (uint16_t*)prepared, pieces);
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}

extern "C" int bitsmoe_skinny_linear(const void* x, int32_t dtype, int32_t x_is_f32, int64_t ld_x, const void* weight,
                                     int32_t weight_is_prepared, int64_t n_rows, int32_t in_features, int32_t out_features,
                                     void* out, int64_t ld_out, const float* addend, int64_t ld_addend, void* stream) {
    BITSMOE_REQUIRE(dtype == BITSMOE_DT_F16 || dtype == BITSMOE_DT_BF16, "dtype must be f16 (0) or bf16 (1)");
    BITSMOE_REQUIRE(n_rows >= 0 && n_rows <= (x_is_f32 ? 16 : 64), "n_rows must be in [0, 64] (fp32 rows: [0, 16])");
    BITSMOE_REQUIRE(in_features >= 128 && in_features % 128 == 0, "in_features must be a positive multiple of 128");
    BITSMOE_REQUIRE(out_features >= 2 && out_features % 2 == 0, "out_features must be even");
    BITSMOE_REQUIRE(ld_x >= in_features && ld_x % (x_is_f32 ? 4 : 8) == 0,
                    "ld_x must be at least in_features and a multiple of 8 (fp32 rows: of 4)");
    BITSMOE_REQUIRE(ld_out >= out_features && ld_out % 2 == 0, "ld_out must be at least out_features and even");
    BITSMOE_REQUIRE(addend == nullptr || ld_addend >= out_features, "ld_addend must be at least out_features");
    if (n_rows == 0) return BITSMOE_OK;
    BITSMOE_REQUIRE(x && weight && out, "null pointer");
    BITSMOE_REQUIRE((((uintptr_t)x | (uintptr_t)weight) & 15) == 0 && ((uintptr_t)out & 3) == 0,
                    "x and weight must be 16-byte aligned, out 4-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const bool bf16 = dtype == BITSMOE_DT_BF16;
    // two 16-column blocks per wavefront once that still leaves a workgroup per CU and more (half the re-reads of x)
    const bool two = out_features >= 32 * 512;
    const int nmb = (int)((n_rows + 15) / 16);
    const unsigned grid = (unsigned)((out_features + (two ? 32 : 16) - 1) / (two ? 32 : 16));
#define BITSMOE_SKINNY(B, NMB, NBW)                                                                                     \
    hipLaunchKernelGGL((k_skinny_linear<B, NMB, NBW>), dim3(grid), dim3(256), 0, st, x, ld_x,           \
                       (const uint16_t*)weight, (int)n_rows, in_features, out_features, (uint16_t*)out, ld_out, (const float*)addend, ld_addend)
#define BITSMOE_SKINNY_M(B, NBW)                                      \
    do {                                                              \
        if (nmb == 1) BITSMOE_SKINNY(B, 1, NBW);                      \
        else if (nmb == 2) BITSMOE_SKINNY(B, 2, NBW);                 \
        else if (nmb == 3) BITSMOE_SKINNY(B, 3, NBW);                 \
        else BITSMOE_SKINNY(B, 4, NBW);                               \
    } while (0)
    if (x_is_f32 || weight_is_prepared) {
        // (the forms the block uses at a few tokens: one column block per wavefront)
        BITSMOE_REQUIRE(!x_is_f32 || n_rows <= 16, "fp32 rows: at most 16 rows");
        const dim3 g1((unsigned)((out_features + 15) / 16));
        const int nmb1 = (int)((n_rows + 15) / 16);
#define BITSMOE_SKINNY_1(B, NMB, XF, PR)                                                                                   \
        hipLaunchKernelGGL((k_skinny_linear<B, NMB, 1, XF, PR>), g1, dim3(256), 0, st, x, ld_x, (const uint16_t*)weight,   \
                           (int)n_rows, in_features, out_features, (uint16_t*)out, ld_out, (const float*)addend, ld_addend)
#define BITSMOE_SKINNY_P(B)                                                                  \
        do {                                                                                 \
            if (x_is_f32 && weight_is_prepared) BITSMOE_SKINNY_1(B, 1, true, true);          \
            else if (x_is_f32) BITSMOE_SKINNY_1(B, 1, true, false);                          \
            else if (nmb1 == 1) BITSMOE_SKINNY_1(B, 1, false, true);                         \
            else if (nmb1 == 2) BITSMOE_SKINNY_1(B, 2, false, true);                         \
            else if (nmb1 == 3) BITSMOE_SKINNY_1(B, 3, false, true);                         \
            else BITSMOE_SKINNY_1(B, 4, false, true);                                        \
        } while (0)
        if (bf16) BITSMOE_SKINNY_P(true); else BITSMOE_SKINNY_P(false);
#undef BITSMOE_SKINNY_P
#undef BITSMOE_SKINNY_1
    } else if (bf16) {
        if (two) BITSMOE_SKINNY_M(true, 2); else BITSMOE_SKINNY_M(true, 1);
    } else {
        if (two) BITSMOE_SKINNY_M(false, 2); else BITSMOE_SKINNY_M(false, 1);
    }
#undef BITSMOE_SKINNY_M
#undef BITSMOE_SKINNY
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}
