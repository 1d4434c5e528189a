#pragma once
// run_moe_grouped_expert_batch and MoeGroupedBatchScratch under the reference's names and
// signatures (src/architecture/deepseek_v4/moe/moe_grouped_batch.hpp:34-147): a chunk's routing
// goes through the token -> expert permutation, the grouped gate/up and W2 launches and the
// slot-ordered reduce that folds in what the caller already stored in each token's output row.
//
// What the contract fixes: the Filler is told every expert's draw count, so the per-expert bounds
// are read back once per call (one stream synchronisation, as at :80-83), a weight table holds
// kAeonSwizzledMaxExperts experts, and an expert wider than the scratch is refused (:90-93).
// What is done differently here:
//   * the grouped launches read the permutation's own device-side bounds (the table of a launch
//     is a window of perm_offsets, positions stay absolute), so nothing is re-based on the host
//     and no bounds are copied back to the device; `batch_offsets` of the scratch is unused;
//   * a window with no draws costs no launch and no Filler call;
//   * the reduce is one launch over all tokens of the chunk, not one per token.
// The resident-expert path (aeon_moe_layer_routed) needs none of this: it has no read-back.
#include "architecture/deepseek_v4/kernels/moe_grouped_dispatch.hpp"
#include "infrastructure/hip_check.hpp"
#include "platform/ops/expert_permutation.hpp"
#include "platform/ops/moe_accumulate.hpp"

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <vector>

namespace aeon::core {

struct MoeGroupedBatchScratch {
    int* perm_offsets{nullptr};     // [expert_count + 1]
    int* perm_tokens{nullptr};      // [token_count * slots]
    int* perm_draws{nullptr};       // [token_count * slots]
    float* perm_weights{nullptr};   // [token_count * slots]
    int* batch_offsets{nullptr};    // [kAeonSwizzledMaxExperts + 1], kept for the signature
    half* chunk_hidden{nullptr};    // [kAeonSwizzledMaxExperts, hidden_tokens, intermediate]
    float* chunk_contrib{nullptr};  // [token_count * slots, hidden]
    int intermediate{0};
    int hidden{0};
    int hidden_tokens{0};  // rows of chunk_hidden per expert
};

// fill(expert, j, count, w13, w2) puts expert `expert`, which owns `count` draws, at position j
// of the two weight tables; an expert with count 0 may leave its position empty.
template <class Filler>
void run_moe_grouped_expert_batch(const half* batch_input, int input_stride, const int* batch_ids,
                                  const float* batch_weights, uint32_t token_count, int slots,
                                  int expert_count, float swiglu_limit,
                                  const MoeGroupedBatchScratch& scratch, Filler&& fill,
                                  half* batch_output, int output_stride, hipStream_t stream = 0) {
    if (token_count == 0) return;
    const int tokens = static_cast<int>(token_count);
    kernel::dispatch_expert_permutation(batch_ids, tokens, slots, expert_count,
                                        scratch.perm_offsets, scratch.perm_tokens,
                                        scratch.perm_draws, batch_weights, scratch.perm_weights,
                                        stream);

    std::vector<int> bound(static_cast<size_t>(expert_count) + 1);
    CHECK_HIP(hipMemcpyAsync(bound.data(), scratch.perm_offsets, bound.size() * sizeof(int),
                             hipMemcpyDeviceToHost, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    auto draws_of = [&](int expert) { return bound[expert + 1] - bound[expert]; };

    int widest = 1;
    for (int expert = 0; expert < expert_count; ++expert) {
        if (draws_of(expert) > widest) widest = draws_of(expert);
    }
    if (widest > scratch.hidden_tokens) {
        throw std::invalid_argument(
            "run_moe_grouped_expert_batch: the chunk's widest expert exceeds the scratch");
    }

    constexpr int kTable = kernel::kAeonSwizzledMaxExperts;
    for (int window = 0; window < expert_count; window += kTable) {
        const int in_window = expert_count - window < kTable ? expert_count - window : kTable;
        if (bound[window + in_window] == bound[window]) continue;
        kernel::SwizzledW13ExpertPtrs gate_up{};
        kernel::SwizzledW2ExpertPtrs down{};
        for (int j = 0; j < in_window; ++j) fill(window + j, j, draws_of(window + j), gate_up, down);
        const int* device_bounds = scratch.perm_offsets + window;  // absolute positions
        kernel::dispatch_aeon_moe_grouped_w13_swiglu_wmma<4, 4, 8, kernel::kMoeGroupedMTiles>(
            batch_input, device_bounds, scratch.perm_tokens, gate_up, scratch.chunk_hidden, in_window,
            widest, scratch.intermediate, scratch.hidden, swiglu_limit, input_stride, stream);
        kernel::dispatch_aeon_moe_grouped_w2_wmma<4, 8, 4, kernel::kMoeGroupedMTiles>(
            scratch.chunk_hidden, device_bounds, scratch.perm_draws, scratch.perm_weights, down,
            scratch.chunk_contrib, in_window, widest, scratch.hidden, scratch.intermediate, stream);
    }

    aeon355::throw_on_error(aeon_moe_accumulate_fixed_order_tokens(
        scratch.chunk_contrib, tokens, slots, batch_output, output_stride, scratch.hidden, stream));
}

}  // namespace aeon::core
