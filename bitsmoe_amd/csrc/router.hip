// Router front end in one kernel: softmax over the expert logits in fp32, top-k, optional
// renormalisation of the k probabilities, optional round trip of the weights through a 16-bit
// type.  Replaces the chain of framework ops of the reference's Qwen blocks
// (bitsmoe/models/qwen3moe/bitsmoe_block.py:45-51, bitsmoe/models/qwen3next/bitsmoe_block.py:92-98):
//     p = softmax(logits.float());  w, idx = topk(p, k);  w /= w.sum();  w = w.to(act dtype)
// One wavefront per token; a lane holds the logits of experts lane, lane + 64, ...
#include "common.h"

#include <algorithm>

namespace bitsmoe {

constexpr int ROUTER_MAX_PER_LANE = 16;   // experts <= 1024

template <int DT>   // 0: fp16, 1: bf16, 2: fp32 logits
__device__ inline float load_logit(const void* __restrict__ base, int64_t idx) {
    if constexpr (DT == 2) {
        return reinterpret_cast<const float*>(base)[idx];
    } else if constexpr (DT == 1) {
        return __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(base)[idx] << 16);
    } else {
        return __half2float(reinterpret_cast<const __half*>(base)[idx]);
    }
}

__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
    return v;
}

// grid = ceil(T / 4), 256 threads (four tokens per workgroup)
template <int DT>
__global__ __launch_bounds__(256) void k_router_softmax_topk(const void* __restrict__ logits, int64_t ld, float wscale,
                                                             int T, int E, int k,
                                                             int renorm, int round_dt, int32_t* __restrict__ sel32,
                                                             int64_t* __restrict__ sel64, float* __restrict__ weights) {
    const int lane = threadIdx.x & 63;
    const int tkn = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tkn >= T) return;
    const int per = (E + 63) >> 6;
    float v[ROUTER_MAX_PER_LANE];
    float vmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < ROUTER_MAX_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        v[i] = (i < per && e < E) ? load_logit<DT>(logits, (int64_t)tkn * ld + e) : -INFINITY;
        vmax = fmaxf(vmax, v[i]);
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) vmax = fmaxf(vmax, __shfl_xor(vmax, d));
    float part = 0.0f;
#pragma unroll
    for (int i = 0; i < ROUTER_MAX_PER_LANE; ++i)
        if (i < per) part += (v[i] == -INFINITY) ? 0.0f : expf(v[i] - vmax);
    const float denom = wave_sum(part);

    // k rounds of arg-max over what is left; ties go to the lower expert index
    float my_w = 0.0f;      // lane j < k keeps the j-th pick
    int my_e = 0;
    float picked_sum = 0.0f;
    for (int j = 0; j < k; ++j) {
        float best = -INFINITY;
        int best_e = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < ROUTER_MAX_PER_LANE; ++i) {
            const int e = lane + 64 * i;
            if (i < per && (v[i] > best)) {      // ascending e inside a lane: strict > keeps the lower index
                best = v[i];
                best_e = e;
            }
        }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            const float ob = __shfl_xor(best, d);
            const int oe = __shfl_xor(best_e, d);
            if (ob > best || (ob == best && oe < best_e)) {
                best = ob;
                best_e = oe;
            }
        }
        // remove the pick from its owner
#pragma unroll
        for (int i = 0; i < ROUTER_MAX_PER_LANE; ++i)
            if (lane + 64 * i == best_e) v[i] = -INFINITY;
        const float p = (best == -INFINITY) ? 0.0f : expf(best - vmax) / denom;
        picked_sum += p;
        if (lane == j) {
            my_w = p;
            my_e = best_e < E ? best_e : 0;
        }
    }
    if (lane < k) {
        float w = (renorm ? my_w / picked_sum : my_w) * wscale;
        if (round_dt == BITSMOE_DT_F16)
            w = __half2float(__float2half(w));
        else if (round_dt == BITSMOE_DT_BF16)
            w = __bfloat162float(__float2bfloat16(w));
        const int64_t o = (int64_t)tkn * k + lane;
        if (sel32) sel32[o] = my_e;
        if (sel64) sel64[o] = my_e;
        weights[o] = w;
    }
}

// The same result for at most 256 experts without the k dependent arg-max rounds: every lane
// counts, for each of its (up to four) logits, how many of the token's logits precede it in
// the order (value descending, expert index ascending); that count is the position of the
// expert in the top-k list.  The logits of a token sit in LDS and are read as broadcasts.
// grid = ceil(T / 4), 256 threads (one wavefront per token).
constexpr int ROUTER_RANK_PER_LANE = 4;
template <int NW>      // wavefronts per workgroup
struct RankTopkLds {
    // sort key of a logit: the float mapped to an unsigned integer of the same order, above the
    // complemented expert index, so that one 64-bit comparison is "precedes in the top-k order"
    uint64_t keys[NW][64 * ROUTER_RANK_PER_LANE];
    float picked[NW][64];
};
// One token by one wavefront (`wv` of its workgroup): v[i] is the logit of expert lane + 64 i (-inf past E).
// LIVE: logits per lane that can exist (E <= 64 LIVE); the counting loop, which is most of the work, runs over those only.
template <int LIVE, int NW>
__device__ inline void rank_topk_live(float (&v)[ROUTER_RANK_PER_LANE], RankTopkLds<NW>& lds, int wv, int lane, int tkn, float wscale,
                                      int E, int k, int renorm, int round_dt, int32_t* __restrict__ sel32,
                                      int64_t* __restrict__ sel64, float* __restrict__ weights) {
    const int e2 = (E + 1) & ~1;
    uint64_t mine[LIVE];
    float vmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < LIVE; ++i) {
        const int e = lane + 64 * i;
        vmax = fmaxf(vmax, v[i]);
        const uint32_t bits = __float_as_uint(v[i] + 0.0f);      // (-0 and +0 are one value)
        const uint32_t ordered = bits ^ ((bits >> 31) ? 0xFFFFFFFFu : 0x80000000u);
        mine[i] = e < E ? ((uint64_t)ordered << 32) | (uint32_t)(0xFFFFFFFFu - (uint32_t)e) : 0ull;   // padding sorts last
        lds.keys[wv][e] = mine[i];
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) vmax = fmaxf(vmax, __shfl_xor(vmax, d));
    float pr[LIVE];
    float part = 0.0f;
#pragma unroll
    for (int i = 0; i < LIVE; ++i) {
        pr[i] = (v[i] == -INFINITY) ? 0.0f : expf(v[i] - vmax);
        part += pr[i];
    }
    const float denom = wave_sum(part);
    // the other lanes' keys are read below: order the LDS writes above before those reads whatever
    // the compiler's schedule (one wavefront: a wave-scope fence and a wave barrier, no s_barrier)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    int rank[LIVE] = {};
#pragma unroll 4
    for (int o = 0; o < e2; o += 2) {
        const uint64_t q0 = lds.keys[wv][o], q1 = lds.keys[wv][o + 1];
#pragma unroll
        for (int i = 0; i < LIVE; ++i) rank[i] += (int)(q0 > mine[i]) + (int)(q1 > mine[i]);
    }
#pragma unroll
    for (int i = 0; i < LIVE; ++i)
        if (lane + 64 * i < E && rank[i] < k) lds.picked[wv][rank[i]] = pr[i] / denom;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    float picked_sum = 0.0f;
    for (int j = 0; j < k; ++j) picked_sum += lds.picked[wv][j];
#pragma unroll
    for (int i = 0; i < LIVE; ++i) {
        if (lane + 64 * i < E && rank[i] < k) {
            float w = pr[i] / denom;
            if (renorm) w /= picked_sum;
            w *= wscale;
            if (round_dt == BITSMOE_DT_F16)
                w = __half2float(__float2half(w));
            else if (round_dt == BITSMOE_DT_BF16)
                w = __bfloat162float(__float2bfloat16(w));
            const int64_t o = (int64_t)tkn * k + rank[i];
            if (sel32) sel32[o] = lane + 64 * i;
            if (sel64) sel64[o] = lane + 64 * i;
            weights[o] = w;
        }
    }
    // (the next token of this wavefront overwrites keys / picked: its reads above are done first)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int NW>
__device__ inline void rank_topk_token(float (&v)[ROUTER_RANK_PER_LANE], RankTopkLds<NW>& lds, int wv, int lane, int tkn, float wscale,
                                       int E, int k, int renorm, int round_dt, int32_t* __restrict__ sel32,
                                       int64_t* __restrict__ sel64, float* __restrict__ weights) {
    if (E <= 64)
        rank_topk_live<1>(v, lds, wv, lane, tkn, wscale, E, k, renorm, round_dt, sel32, sel64, weights);
    else if (E <= 128)
        rank_topk_live<2>(v, lds, wv, lane, tkn, wscale, E, k, renorm, round_dt, sel32, sel64, weights);
    else
        rank_topk_live<ROUTER_RANK_PER_LANE>(v, lds, wv, lane, tkn, wscale, E, k, renorm, round_dt, sel32, sel64, weights);
}

template <int DT>
__global__ __launch_bounds__(256) void k_router_rank_topk(const void* __restrict__ logits, int64_t ld, float wscale, int T,
                                                          int E, int k,
                                                          int renorm, int round_dt, int32_t* __restrict__ sel32,
                                                          int64_t* __restrict__ sel64, float* __restrict__ weights) {
    __shared__ __attribute__((aligned(16))) RankTopkLds<4> lds;
    const int lane = threadIdx.x & 63;
    const int wv = threadIdx.x >> 6;
    const int tkn = blockIdx.x * 4 + wv;
    if (tkn >= T) return;            // (no workgroup barrier below: a wavefront only reads what it wrote)
    float v[ROUTER_RANK_PER_LANE];
#pragma unroll
    for (int i = 0; i < ROUTER_RANK_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        v[i] = e < E ? load_logit<DT>(logits, (int64_t)tkn * ld + e) : -INFINITY;
    }
    rank_topk_token(v, lds, wv, lane, tkn, wscale, E, k, renorm, round_dt, sel32, sel64, weights);
}

// The router's linear layer and the top-k in ONE kernel, for gates that compute their logits in fp32 from 16-bit
// hidden states and a 16-bit weight (DeepSeek-V2's gate: bitsmoe/models/deepseekv2/configuration_deepseek.py:125-139
// names its form; the reference calls the model's own gate module, bitsmoe/models/deepseekv2/bitsmoe_block.py:74):
// the products of 16-bit values are exact in fp32, so MFMA sums in fp32 are the module's logits up to summation
// order.  A workgroup of NW wavefronts takes 16 tokens: wavefront w contracts over the w-th part of the hidden size
// for all experts (NB 16-expert blocks; sixteen wavefronts: all its operands of a 2048-wide layer are ONE batch of
// loads), the partial sums meet in LDS (a tree in a fixed order: the same logits whenever the inputs are the same), then
// the wavefronts rank the tokens, 16 / NW each.
// x [T, K] and weight [E, K] are read as MFMA operands straight from memory (16 bytes per lane).
// PREP: the weight in MFMA operand order ([16-expert block][k-step of 32][lane][8 values]: bitsmoe_prepare_linear_weight):
// a wavefront's load is 1 KB of consecutive memory.
template <bool BF16, int NB, int NW, bool PREP>
__global__ __launch_bounds__(NW * 64) void k_router_linear_topk(const uint16_t* __restrict__ x, int64_t ld_x,
                                                                const uint16_t* __restrict__ weight, int T, int K, int E, int k,
                                                                float wscale, int renorm, int round_dt,
                                                                int32_t* __restrict__ sel32, int64_t* __restrict__ sel64,
                                                                float* __restrict__ weights) {
    constexpr int U = NB <= 4 ? 4 : NB <= 8 ? 2 : 1;      // k-steps whose operands are requested together
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
    typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
    constexpr int LD = NB * 16 + 1;
    // DIRECT: every wavefront's partial sums fit the LDS side by side and the ranking wavefront adds them up itself (one
    // barrier); otherwise a tree over half as many slots (slot 0 ends as the total).  Both add in a fixed order.
    constexpr bool DIRECT = NW * 16 * LD * 4 + sizeof(RankTopkLds<NW>) <= 160 * 1024;
    __shared__ float part[(DIRECT ? NW : NW / 2) * 16 * LD];
    __shared__ __attribute__((aligned(16))) RankTopkLds<NW> lds;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int t0 = blockIdx.x * 16;
    const int row = t0 + (lane & 15);
    const int kq = K / NW;                       // contraction range of this wavefront (a multiple of 32)
    const int kbase = wv * kq + (lane >> 4) * 8;
    f32x4 acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const uint16_t* __restrict__ xp = x + (int64_t)min(row, T - 1) * ld_x + kbase;
    for (int s0 = 0; s0 < kq; s0 += 32 * U) {
        u32x4 a[U], b[U][NB];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ks = min(s0 + 32 * u, kq - 32);      // (a short last group repeats its final step: masked below)
            a[u] = *reinterpret_cast<const u32x4*>(xp + ks);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                if constexpr (PREP) {
                    const int blk = min(nb, (E - 1) >> 4);      // (blocks past the last expert repeat it: masked below)
                    b[u][nb] = *reinterpret_cast<const u32x4*>(weight + (((int64_t)blk * (K >> 5) + ((wv * kq + ks) >> 5)) * 64 + lane) * 8);
                } else {
                    const int e = min(nb * 16 + (lane & 15), E - 1);
                    b[u][nb] = *reinterpret_cast<const u32x4*>(weight + (int64_t)e * K + kbase + ks);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);      // (every request of the group is out before its first MFMA)
#pragma unroll
        for (int u = 0; u < U; ++u) {
            // (no branch between the steps: a step past the end contributes zeros)
            const bool live = s0 + 32 * u < kq;
#pragma unroll
            for (int c = 0; c < 4; ++c) a[u][c] = live ? a[u][c] : 0u;
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                if constexpr (BF16)
                    acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[u]), __builtin_bit_cast(bf16x8, b[u][nb]),
                                                                      acc[nb], 0, 0, 0);
                else
                    acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a[u]), __builtin_bit_cast(f16x8, b[u][nb]),
                                                                     acc[nb], 0, 0, 0);
            }
        }
    }
    // lane holds tokens 4 (lane / 16) + j, expert 16 nb + lane % 16
    auto slot_of = [&](int w, int nb, int j) -> float& { return part[(w * 16 + 4 * (lane >> 4) + j) * LD + nb * 16 + (lane & 15)]; };
    if constexpr (DIRECT) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int j = 0; j < 4; ++j) slot_of(wv, nb, j) = acc[nb][j];
    }
    for (int half = DIRECT ? 0 : NW / 2; half >= 1; half >>= 1) {      // wavefronts [half, 2 half) hand their sums to [0, half)
        if (wv >= half && wv < 2 * half) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int j = 0; j < 4; ++j) slot_of(wv - half, nb, j) = acc[nb][j];
        }
        __syncthreads();
        if (wv < half) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[nb][j] += slot_of(wv, nb, j);
        }
        __syncthreads();
    }
    if (!DIRECT && wv == 0) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int j = 0; j < 4; ++j) slot_of(0, nb, j) = acc[nb][j];
    }
    __syncthreads();
    constexpr int PER = 16 / NW > 0 ? 16 / NW : 1;
    for (int i = 0; i < PER; ++i) {
        const int tl = wv * PER + i, tkn = t0 + tl;
        if (tl >= 16 || tkn >= T) break;       // (wave-uniform; no workgroup barrier below)
        float v[ROUTER_RANK_PER_LANE];
#pragma unroll
        for (int q = 0; q < ROUTER_RANK_PER_LANE; ++q) {
            const int e = lane + 64 * q;
            float sum = -INFINITY;
            if (e < E && e < NB * 16) {
                sum = part[tl * LD + e];
                if constexpr (DIRECT) {
#pragma unroll
                    for (int w = 1; w < NW; ++w) sum += part[(w * 16 + tl) * LD + e];
                }
            }
            v[q] = sum;
        }
        rank_topk_token(v, lds, wv, lane, tkn, wscale, E, k, renorm, round_dt, sel32, sel64, weights);
    }
}

}  // namespace bitsmoe

using namespace bitsmoe;

extern "C" int bitsmoe_router_softmax_topk_strided(const void* logits, int32_t logits_dtype, int64_t ld_logits, int64_t n_tokens,
                                                   int32_t n_experts, int32_t top_k, int32_t renormalize, float weight_scale,
                                                   int32_t round_dtype, void* selected, int32_t ids_are_i64, float* weights,
                                                   void* stream) {
    BITSMOE_REQUIRE(n_tokens >= 0 && n_tokens < ((int64_t)1 << 31), "token count out of range");
    BITSMOE_REQUIRE(n_experts >= 1 && n_experts <= 64 * ROUTER_MAX_PER_LANE, "n_experts must be in [1, %d]",
                    64 * ROUTER_MAX_PER_LANE);
    BITSMOE_REQUIRE(top_k >= 1 && top_k <= 64 && top_k <= n_experts, "top_k must be in [1, min(64, n_experts)]");
    BITSMOE_REQUIRE(logits_dtype >= 0 && logits_dtype <= 2, "logits_dtype must be 0 (fp16), 1 (bf16) or 2 (fp32)");
    BITSMOE_REQUIRE(round_dtype >= -1 && round_dtype <= 1, "round_dtype must be -1 (none), 0 (fp16) or 1 (bf16)");
    BITSMOE_REQUIRE(ld_logits >= n_experts, "ld_logits must be at least n_experts");
    if (n_tokens == 0) return BITSMOE_OK;
    BITSMOE_REQUIRE(logits && selected && weights, "null pointer");
    hipStream_t st = (hipStream_t)stream;
    int32_t* s32 = ids_are_i64 ? nullptr : (int32_t*)selected;
    int64_t* s64 = ids_are_i64 ? (int64_t*)selected : nullptr;
    const dim3 grid((unsigned)((n_tokens + 3) / 4));
    const bool by_rank = n_experts <= 64 * ROUTER_RANK_PER_LANE;
#define BITSMOE_ROUTER_LAUNCH(KERNEL)                                                                              \
    hipLaunchKernelGGL(KERNEL, grid, dim3(256), 0, st, logits, ld_logits, weight_scale, (int)n_tokens, n_experts, top_k, \
                       renormalize, round_dtype, s32, s64, weights)
    if (logits_dtype == 0) {
        if (by_rank) BITSMOE_ROUTER_LAUNCH(k_router_rank_topk<0>); else BITSMOE_ROUTER_LAUNCH(k_router_softmax_topk<0>);
    } else if (logits_dtype == 1) {
        if (by_rank) BITSMOE_ROUTER_LAUNCH(k_router_rank_topk<1>); else BITSMOE_ROUTER_LAUNCH(k_router_softmax_topk<1>);
    } else {
        if (by_rank) BITSMOE_ROUTER_LAUNCH(k_router_rank_topk<2>); else BITSMOE_ROUTER_LAUNCH(k_router_softmax_topk<2>);
    }
#undef BITSMOE_ROUTER_LAUNCH
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}

extern "C" int bitsmoe_router_softmax_topk(const void* logits, int32_t logits_dtype, int64_t n_tokens, int32_t n_experts,
                                           int32_t top_k, int32_t renormalize, int32_t round_dtype, void* selected,
                                           int32_t ids_are_i64, float* weights, void* stream) {
    return bitsmoe_router_softmax_topk_strided(logits, logits_dtype, n_experts, n_tokens, n_experts, top_k, renormalize, 1.0f,
                                               round_dtype, selected, ids_are_i64, weights, stream);
}

extern "C" int bitsmoe_router_linear_topk(const void* hidden, int32_t dtype, int64_t ld_hidden, const void* weight,
                                          int32_t weight_is_prepared, int64_t n_tokens, int32_t hidden_size, int32_t n_experts, int32_t top_k,
                                          int32_t renormalize, float weight_scale, int32_t round_dtype, void* selected,
                                          int32_t ids_are_i64, float* weights, void* stream) {
    BITSMOE_REQUIRE(n_tokens >= 0 && n_tokens < ((int64_t)1 << 31), "token count out of range");
    BITSMOE_REQUIRE(dtype == BITSMOE_DT_F16 || dtype == BITSMOE_DT_BF16, "dtype must be f16 (0) or bf16 (1)");
    BITSMOE_REQUIRE(n_experts >= 1 && n_experts <= 64 * ROUTER_RANK_PER_LANE, "n_experts must be in [1, %d]", 64 * ROUTER_RANK_PER_LANE);
    BITSMOE_REQUIRE(top_k >= 1 && top_k <= 64 && top_k <= n_experts, "top_k must be in [1, min(64, n_experts)]");
    BITSMOE_REQUIRE(hidden_size >= 128 && hidden_size % 128 == 0, "hidden_size must be a positive multiple of 128");
    // (option router_wide = 0: four wavefronts per workgroup whatever the hidden size; experiments)
    const bool wide_wg = hidden_size % 512 == 0 && options().router_wide != 0;      // sixteen wavefronts, a sixteenth of the contraction each
    BITSMOE_REQUIRE(ld_hidden >= hidden_size && ld_hidden % 8 == 0, "ld_hidden must be at least hidden_size and a multiple of 8");
    BITSMOE_REQUIRE(round_dtype >= -1 && round_dtype <= 1, "round_dtype must be -1 (none), 0 (fp16) or 1 (bf16)");
    if (n_tokens == 0) return BITSMOE_OK;
    BITSMOE_REQUIRE(hidden && weight && selected && weights, "null pointer");
    BITSMOE_REQUIRE((((uintptr_t)hidden | (uintptr_t)weight) & 15) == 0, "hidden and weight must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    int32_t* s32 = ids_are_i64 ? nullptr : (int32_t*)selected;
    int64_t* s64 = ids_are_i64 ? (int64_t*)selected : nullptr;
    const dim3 grid((unsigned)((n_tokens + 15) / 16));
    const bool bf16 = dtype == BITSMOE_DT_BF16;
#define BITSMOE_ROUTER_LINEAR_P(B, NB, NWIDE, PR)                                                                             \
    do {                                                                                                                     \
        if (wide_wg)                                                                                                         \
            hipLaunchKernelGGL((k_router_linear_topk<B, NB, NWIDE, PR>), grid, dim3(NWIDE * 64), 0, st,                      \
                               (const uint16_t*)hidden, ld_hidden, (const uint16_t*)weight, (int)n_tokens, hidden_size,      \
                               n_experts, top_k, weight_scale, renormalize, round_dtype, s32, s64, weights);                 \
        else                                                                                                                 \
            hipLaunchKernelGGL((k_router_linear_topk<B, NB, 4, PR>), grid, dim3(256), 0, st, (const uint16_t*)hidden,        \
                               ld_hidden, (const uint16_t*)weight, (int)n_tokens, hidden_size, n_experts, top_k,             \
                               weight_scale, renormalize, round_dtype, s32, s64, weights);                                   \
    } while (0)
#define BITSMOE_ROUTER_LINEAR(B, NB, NWIDE)                                                      \
    do {                                                                                         \
        if (weight_is_prepared) BITSMOE_ROUTER_LINEAR_P(B, NB, NWIDE, true);                     \
        else BITSMOE_ROUTER_LINEAR_P(B, NB, NWIDE, false);                                       \
    } while (0)
    // (more than 128 experts: eight wavefronts, the partial sums of sixteen would not fit the LDS)
    if (n_experts <= 64) {
        if (bf16) BITSMOE_ROUTER_LINEAR(true, 4, 16); else BITSMOE_ROUTER_LINEAR(false, 4, 16);
    } else if (n_experts <= 128) {
        if (bf16) BITSMOE_ROUTER_LINEAR(true, 8, 16); else BITSMOE_ROUTER_LINEAR(false, 8, 16);
    } else {
        if (bf16) BITSMOE_ROUTER_LINEAR(true, 16, 8); else BITSMOE_ROUTER_LINEAR(false, 16, 8);
    }
#undef BITSMOE_ROUTER_LINEAR
#undef BITSMOE_ROUTER_LINEAR_P
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}

// ---- the block's closing elementwise pass ---------------------------------------------------------------------------
// One row of the operand of the block's output GEMM, in the activation dtype:
//     out[t, 0 .. R)        = rank_accum[t, :]                                   (fp32 -> 16 bit)
//     out[t, R .. R + I_sh) = silu(a[t, c]) * b[t, c] * (g ? sigmoid(g[t]) : 1)   (the always-on shared expert's z)
// so that the routed experts' output projection and the shared expert's down projection are ONE GEMM against
// the stacked [U_down | W_down_shared] (bitsmoe/models/base_block.py:414, bitsmoe/models/qwen3next/bitsmoe_block.py:144-147,
// bitsmoe/models/deepseekv2/bitsmoe_block.py:123-124 run them as separate modules and add).  Eight elements per thread.
template <bool BF16>
__global__ __launch_bounds__(256) void k_block_finish(const float* __restrict__ rank_accum, int64_t T, int R,
                                                      const uint16_t* __restrict__ a, const uint16_t* __restrict__ b,
                                                      int64_t ld_ab, int I_sh, const uint16_t* __restrict__ g, int64_t ld_g,
                                                      uint16_t* __restrict__ out, int64_t ld_out) {
    const int per_row = (R + I_sh) >> 3;
    const int64_t total = T * per_row;
    auto to_f32 = [](uint16_t v) {
        if constexpr (BF16) return __uint_as_float((uint32_t)v << 16);
        else return __half2float(__ushort_as_half(v));
    };
    auto to_16 = [](float v) -> uint16_t {
        if constexpr (BF16) return __builtin_bit_cast(uint16_t, (__bf16)v);
        else return __builtin_bit_cast(uint16_t, (_Float16)v);
    };
    typedef uint32_t v4 __attribute__((ext_vector_type(4)));
    typedef float f4 __attribute__((ext_vector_type(4)));
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t t = i / per_row;
        const int c = (int)(i - t * per_row) * 8;
        uint16_t o[8];
        if (c < R) {
            const f4 lo = *reinterpret_cast<const f4*>(rank_accum + t * R + c);
            const f4 hi = *reinterpret_cast<const f4*>(rank_accum + t * R + c + 4);
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                o[x] = to_16(lo[x]);
                o[4 + x] = to_16(hi[x]);
            }
        } else {
            const int cs = c - R;
            const v4 av = *reinterpret_cast<const v4*>(a + t * ld_ab + cs);
            const v4 bv = *reinterpret_cast<const v4*>(b + t * ld_ab + cs);
            float gate = 1.0f;
            if (g) gate = 1.0f / (1.0f + __expf(-to_f32(g[t * ld_g])));
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const float a0 = to_f32((uint16_t)(av[x] & 0xFFFFu)), a1 = to_f32((uint16_t)(av[x] >> 16));
                const float b0 = to_f32((uint16_t)(bv[x] & 0xFFFFu)), b1 = to_f32((uint16_t)(bv[x] >> 16));
                // (rounded as the modules round: silu in the activation dtype, the product, the gate's scaling)
                o[2 * x] = to_16(to_f32(to_16(to_f32(to_16(a0 / (1.0f + __expf(-a0)))) * b0)) * gate);
                o[2 * x + 1] = to_16(to_f32(to_16(to_f32(to_16(a1 / (1.0f + __expf(-a1)))) * b1)) * gate);
            }
        }
        v4 packed;
#pragma unroll
        for (int x = 0; x < 4; ++x) packed[x] = (uint32_t)o[2 * x] | ((uint32_t)o[2 * x + 1] << 16);
        *reinterpret_cast<v4*>(out + t * ld_out + c) = packed;
    }
}

extern "C" int bitsmoe_block_finish(const float* rank_accum, int64_t n_tokens, int32_t rank_out, const void* shared_gate_out,
                                    const void* shared_up_out, int64_t ld_shared, int32_t shared_intermediate,
                                    const void* shared_gate_logit, int64_t ld_gate_logit, int32_t act_dtype, void* out,
                                    int64_t ld_out, void* stream) {
    BITSMOE_REQUIRE(n_tokens >= 0 && rank_out > 0 && shared_intermediate >= 0, "negative size");
    BITSMOE_REQUIRE(rank_out % 8 == 0 && shared_intermediate % 8 == 0, "rank_out and shared_intermediate must be multiples of 8");
    BITSMOE_REQUIRE(act_dtype == BITSMOE_DT_F16 || act_dtype == BITSMOE_DT_BF16, "act_dtype must be f16 (0) or bf16 (1)");
    BITSMOE_REQUIRE(ld_out >= rank_out + shared_intermediate && ld_out % 8 == 0, "ld_out too small or not a multiple of 8");
    if (n_tokens == 0) return BITSMOE_OK;
    BITSMOE_REQUIRE(rank_accum && out, "null pointer");
    BITSMOE_REQUIRE(((uintptr_t)rank_accum & 15) == 0 && ((uintptr_t)out & 15) == 0, "rank_accum and out must be 16-byte aligned");
    if (shared_intermediate > 0) {
        BITSMOE_REQUIRE(shared_gate_out && shared_up_out && ld_shared >= shared_intermediate && ld_shared % 8 == 0,
                        "shared expert operands missing, or their row stride is not a multiple of 8");
        BITSMOE_REQUIRE(((uintptr_t)shared_gate_out & 15) == 0 && ((uintptr_t)shared_up_out & 15) == 0,
                        "shared expert operands must be 16-byte aligned");
    }
    hipStream_t st = (hipStream_t)stream;
    const int64_t total = n_tokens * ((rank_out + shared_intermediate) / 8);
    const unsigned blocks = (unsigned)std::min<int64_t>((total + 255) / 256, 4096);
    if (act_dtype == BITSMOE_DT_BF16)
        hipLaunchKernelGGL(k_block_finish<true>, dim3(blocks), dim3(256), 0, st, rank_accum, n_tokens, rank_out,
                           (const uint16_t*)shared_gate_out, (const uint16_t*)shared_up_out, ld_shared, shared_intermediate,
                           (const uint16_t*)shared_gate_logit, ld_gate_logit, (uint16_t*)out, ld_out);
    else
        hipLaunchKernelGGL(k_block_finish<false>, dim3(blocks), dim3(256), 0, st, rank_accum, n_tokens, rank_out,
                           (const uint16_t*)shared_gate_out, (const uint16_t*)shared_up_out, ld_shared, shared_intermediate,
                           (const uint16_t*)shared_gate_logit, ld_gate_logit, (uint16_t*)out, ld_out);
    BITSMOE_HIP_TRY(hipGetLastError());
    return BITSMOE_OK;
}
