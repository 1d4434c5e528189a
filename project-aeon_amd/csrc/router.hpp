// Internal launch interface of the router kernels.
#pragma once

#include "common.hpp"

namespace aeon355 {

int router_logits_chunks(int tokens, int hidden);
// partial[c][t][e], c < router_logits_chunks(): per-chunk sums of x[t][h] * Wr[h][e]
int launch_router_partials(const void* d_x, int x_stride, const float* d_router_weight,
                           float* partial, int tokens, int hidden, int experts, hipStream_t stream);
// With `partial` the kernel first reduces the chunks (ascending) into `logits`; without, it
// reads `logits`. Then score, biased top-k, renormalised weights.
int launch_router_topk(const float* partial, int chunks, float* logits, const float* bias,
                       const int64_t* hash_table, const int32_t* token_ids, float* topk_weights,
                       int32_t* topk_indices, int tokens, int experts, int top_k, float scaling,
                       int renormalize, int score_kind, hipStream_t stream);

}  // namespace aeon355
