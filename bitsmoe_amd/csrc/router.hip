// Router front end in one kernel: softmax over the expert logits in fp32, top-k, optional
// renormalisation of the k probabilities, optional round trip of the weights through a 16-bit
// type.  Replaces the chain of framework ops of the reference's Qwen blocks
// (bitsmoe/models/qwen3moe/bitsmoe_block.py:45-51, bitsmoe/models/qwen3next/bitsmoe_block.py:92-98):
//     p = softmax(logits.float());  w, idx = topk(p, k);  w /= w.sum();  w = w.to(act dtype)
// One wavefront per token; a lane holds the logits of experts lane, lane + 64, ...
#include "common.h"

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
__global__ __launch_bounds__(256) void k_router_softmax_topk(const void* __restrict__ logits, int T, int E, int k,
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
        v[i] = (i < per && e < E) ? load_logit<DT>(logits, (int64_t)tkn * E + e) : -INFINITY;
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
        float w = renorm ? my_w / picked_sum : my_w;
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
template <int DT>
__global__ __launch_bounds__(256) void k_router_rank_topk(const void* __restrict__ logits, int T, int E, int k,
                                                          int renorm, int round_dt, int32_t* __restrict__ sel32,
                                                          int64_t* __restrict__ sel64, float* __restrict__ weights) {
    // sort key of a logit: the float mapped to an unsigned integer of the same order, above the
    // complemented expert index, so that one 64-bit comparison is "precedes in the top-k order"
    __shared__ __attribute__((aligned(16))) uint64_t keys[4][64 * ROUTER_RANK_PER_LANE];
    __shared__ float picked[4][64];
    const int lane = threadIdx.x & 63;
    const int wv = threadIdx.x >> 6;
    const int tkn = blockIdx.x * 4 + wv;
    if (tkn >= T) return;            // (no workgroup barrier below: a wavefront only reads what it wrote)
    const int e2 = (E + 1) & ~1;
    float v[ROUTER_RANK_PER_LANE];
    uint64_t mine[ROUTER_RANK_PER_LANE];
    float vmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < ROUTER_RANK_PER_LANE; ++i) {
        const int e = lane + 64 * i;
        v[i] = e < E ? load_logit<DT>(logits, (int64_t)tkn * E + e) : -INFINITY;
        vmax = fmaxf(vmax, v[i]);
        const uint32_t bits = __float_as_uint(v[i] + 0.0f);      // (-0 and +0 are one value)
        const uint32_t ordered = bits ^ ((bits >> 31) ? 0xFFFFFFFFu : 0x80000000u);
        mine[i] = e < E ? ((uint64_t)ordered << 32) | (uint32_t)(0xFFFFFFFFu - (uint32_t)e) : 0ull;   // padding sorts last
        keys[wv][e] = mine[i];
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) vmax = fmaxf(vmax, __shfl_xor(vmax, d));
    float pr[ROUTER_RANK_PER_LANE];
    float part = 0.0f;
#pragma unroll
    for (int i = 0; i < ROUTER_RANK_PER_LANE; ++i) {
        pr[i] = (v[i] == -INFINITY) ? 0.0f : expf(v[i] - vmax);
        part += pr[i];
    }
    const float denom = wave_sum(part);
    // the other lanes' keys are read below: order the LDS writes above before those reads whatever
    // the compiler's schedule (one wavefront: a wave-scope fence and a wave barrier, no s_barrier)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    int rank[ROUTER_RANK_PER_LANE] = {0, 0, 0, 0};
#pragma unroll 4
    for (int o = 0; o < e2; o += 2) {
        const uint64_t q0 = keys[wv][o], q1 = keys[wv][o + 1];
#pragma unroll
        for (int i = 0; i < ROUTER_RANK_PER_LANE; ++i) rank[i] += (int)(q0 > mine[i]) + (int)(q1 > mine[i]);
    }
#pragma unroll
    for (int i = 0; i < ROUTER_RANK_PER_LANE; ++i)
        if (lane + 64 * i < E && rank[i] < k) picked[wv][rank[i]] = pr[i] / denom;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    float picked_sum = 0.0f;
    for (int j = 0; j < k; ++j) picked_sum += picked[wv][j];
#pragma unroll
    for (int i = 0; i < ROUTER_RANK_PER_LANE; ++i) {
        if (lane + 64 * i < E && rank[i] < k) {
            float w = pr[i] / denom;
            if (renorm) w /= picked_sum;
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
}

}  // namespace bitsmoe

using namespace bitsmoe;

extern "C" int bitsmoe_router_softmax_topk(const void* logits, int32_t logits_dtype, int64_t n_tokens, int32_t n_experts,
                                           int32_t top_k, int32_t renormalize, int32_t round_dtype, void* selected,
                                           int32_t ids_are_i64, float* weights, void* stream) {
    BITSMOE_REQUIRE(n_tokens >= 0 && n_tokens < ((int64_t)1 << 31), "token count out of range");
    BITSMOE_REQUIRE(n_experts >= 1 && n_experts <= 64 * ROUTER_MAX_PER_LANE, "n_experts must be in [1, %d]",
                    64 * ROUTER_MAX_PER_LANE);
    BITSMOE_REQUIRE(top_k >= 1 && top_k <= 64 && top_k <= n_experts, "top_k must be in [1, min(64, n_experts)]");
    BITSMOE_REQUIRE(logits_dtype >= 0 && logits_dtype <= 2, "logits_dtype must be 0 (fp16), 1 (bf16) or 2 (fp32)");
    BITSMOE_REQUIRE(round_dtype >= -1 && round_dtype <= 1, "round_dtype must be -1 (none), 0 (fp16) or 1 (bf16)");
    if (n_tokens == 0) return BITSMOE_OK;
    BITSMOE_REQUIRE(logits && selected && weights, "null pointer");
    hipStream_t st = (hipStream_t)stream;
    int32_t* s32 = ids_are_i64 ? nullptr : (int32_t*)selected;
    int64_t* s64 = ids_are_i64 ? (int64_t*)selected : nullptr;
    const dim3 grid((unsigned)((n_tokens + 3) / 4));
    const bool by_rank = n_experts <= 64 * ROUTER_RANK_PER_LANE;
#define BITSMOE_ROUTER_LAUNCH(KERNEL)                                                                              \
    hipLaunchKernelGGL(KERNEL, grid, dim3(256), 0, st, logits, (int)n_tokens, n_experts, top_k, renormalize, \
                       round_dtype, s32, s64, weights)
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
