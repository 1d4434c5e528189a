#pragma once
// The router behind the reference's own names (src/architecture/deepseek_v4/kernels/
// moe_router.hpp:17-189): softplus_sqrt, cpu_moe_router and moe_router_kernel, for callers that
// launch the kernel with <<<num_tokens, 64>>> themselves (v4_layer_body_moe.hpp:143-157).
//
// Same contract: score = sqrt(softplus(logit)); the choice adds the optional per-expert bias;
// the top_k experts are taken by descending choice, ties to the lower index; the weights are
// the unbiased scores, renormalised over the picks (sum + 1e-20) when asked, times the routed
// scaling factor; with a hash table and token ids the picks are the table's row instead.
//
// One wave64 per token. Selection is by rank, not by a serial scan: every lane counts, for each
// of its experts, how many experts beat it under the total order (choice descending, index
// ascending); rank r < top_k is the r-th pick. Scores are computed in fp64 so that two choices
// an fp32 rounding apart are still ordered by value. The batched library call for the same
// step is aeon_moe_router (include/aeon_mi355.h).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <vector>

namespace aeon::kernel {

__host__ __device__ inline double router_sqrt_softplus(double x) {
    if (x > 20.0) return sqrt(x);
    if (x < -20.0) return sqrt(exp(x));
    return sqrt(log1p(exp(x)));
}

__device__ inline float softplus_sqrt(float x) { return static_cast<float>(router_sqrt_softplus(x)); }

// Host statement of the same rule, one token at a time.
inline void cpu_moe_router(const float* router_logits, const float* bias, const int64_t* hash_table,
                           const int32_t* token_ids, float* topk_weights, int32_t* topk_indices,
                           int num_tokens, int n_routed_experts = 256, int top_k = 6,
                           float routed_scaling_factor = 1.5f, bool renormalize = true) {
    std::vector<double> score(n_routed_experts), choice(n_routed_experts);
    std::vector<int> order(n_routed_experts);
    for (int t = 0; t < num_tokens; ++t) {
        const float* logits = router_logits + static_cast<size_t>(t) * n_routed_experts;
        for (int e = 0; e < n_routed_experts; ++e) {
            score[e] = router_sqrt_softplus(static_cast<double>(logits[e]));
            choice[e] = score[e] + (bias != nullptr ? static_cast<double>(bias[e]) : 0.0);
            order[e] = e;
        }
        int32_t* ids = topk_indices + static_cast<size_t>(t) * top_k;
        float* weights = topk_weights + static_cast<size_t>(t) * top_k;
        if (hash_table != nullptr && token_ids != nullptr) {
            for (int k = 0; k < top_k; ++k) {
                ids[k] = static_cast<int32_t>(hash_table[static_cast<size_t>(token_ids[t]) * top_k + k]);
            }
        } else {
            std::stable_sort(order.begin(), order.end(),
                             [&](int a, int b) { return choice[a] > choice[b]; });
            for (int k = 0; k < top_k; ++k) ids[k] = order[k];
        }
        double sum = 0.0;
        for (int k = 0; k < top_k; ++k) sum += score[ids[k]];
        for (int k = 0; k < top_k; ++k) {
            double w = score[ids[k]];
            if (renormalize) w /= sum + 1e-20;
            weights[k] = static_cast<float>(w * static_cast<double>(routed_scaling_factor));
        }
    }
}

constexpr int kShimRouterMaxExperts = 1024;
constexpr int kShimRouterMaxTopK = 64;

__global__ void __launch_bounds__(64) moe_router_kernel(
    const float* __restrict__ router_logits, const float* __restrict__ bias,
    const int64_t* __restrict__ hash_table, const int32_t* __restrict__ token_ids,
    float* __restrict__ topk_weights, int32_t* __restrict__ topk_indices, int n_routed_experts,
    int top_k, float routed_scaling_factor, bool renormalize) {
    __shared__ double score[kShimRouterMaxExperts];
    __shared__ double choice[kShimRouterMaxExperts];
    __shared__ int picked[kShimRouterMaxTopK];
    const int token = blockIdx.x;
    const int lane = threadIdx.x;
    const float* logits = router_logits + static_cast<size_t>(token) * n_routed_experts;
    for (int e = lane; e < n_routed_experts; e += 64) {
        const double s = router_sqrt_softplus(static_cast<double>(logits[e]));
        score[e] = s;
        choice[e] = s + (bias != nullptr ? static_cast<double>(bias[e]) : 0.0);
    }
    __syncthreads();
    if (hash_table != nullptr && token_ids != nullptr) {
        if (lane < top_k) {
            picked[lane] = static_cast<int>(hash_table[static_cast<size_t>(token_ids[token]) * top_k + lane]);
        }
    } else {
        for (int e = lane; e < n_routed_experts; e += 64) {
            const double mine = choice[e];
            int rank = 0;
            for (int f = 0; f < n_routed_experts; ++f) {
                const double other = choice[f];
                rank += (other > mine || (other == mine && f < e)) ? 1 : 0;
            }
            if (rank < top_k) picked[rank] = e;
        }
    }
    __syncthreads();
    if (lane < top_k) {
        double sum = 0.0;
        for (int k = 0; k < top_k; ++k) sum += score[picked[k]];
        double w = score[picked[lane]];
        if (renormalize) w /= sum + 1e-20;
        topk_indices[static_cast<size_t>(token) * top_k + lane] = picked[lane];
        topk_weights[static_cast<size_t>(token) * top_k + lane] =
            static_cast<float>(w * static_cast<double>(routed_scaling_factor));
    }
}

}  // namespace aeon::kernel
