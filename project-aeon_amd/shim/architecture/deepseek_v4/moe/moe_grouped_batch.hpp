#pragma once
// run_moe_grouped_expert_batch and MoeGroupedBatchScratch with the reference's signatures
// (src/architecture/deepseek_v4/moe/moe_grouped_batch.hpp:34-147): permutation, grouped gate/up
// and W2 per range of at most kAeonSwizzledMaxExperts experts, then the per-token slot-ordered
// reduce folding in whatever the caller already stored in each token's output row.
//
// The Filler contract hands the host each expert's draw count, so the expert offsets are read
// back and the stream synchronised once per call, as the reference does (:80-83); the
// resident-expert path (aeon_moe_layer_routed) has no such read-back.
#include "architecture/deepseek_v4/kernels/moe_grouped_dispatch.hpp"
#include "infrastructure/hip_check.hpp"
#include "platform/ops/expert_permutation.hpp"
#include "platform/ops/moe_accumulate.hpp"

#include <algorithm>
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
    int* batch_offsets{nullptr};    // [kAeonSwizzledMaxExperts + 1]
    half* chunk_hidden{nullptr};    // [kAeonSwizzledMaxExperts, hidden_tokens, intermediate]
    float* chunk_contrib{nullptr};  // [token_count * slots, hidden]
    int intermediate{0};
    int hidden{0};
    int hidden_tokens{0};  // rows of chunk_hidden per expert; a wider expert is refused
};

// fill(expert, j, count, w13, w2) sets table position j for expert `expert`, which owns `count`
// draws (0 = never read).
template <class Filler>
void run_moe_grouped_expert_batch(const half* batch_input, int input_stride, const int* batch_ids,
                                  const float* batch_weights, uint32_t token_count, int slots,
                                  int expert_count, float swiglu_limit,
                                  const MoeGroupedBatchScratch& scratch, Filler&& fill,
                                  half* batch_output, int output_stride, hipStream_t stream = 0) {
    if (token_count == 0) return;
    kernel::dispatch_expert_permutation(batch_ids, static_cast<int>(token_count), slots,
                                        expert_count, scratch.perm_offsets, scratch.perm_tokens,
                                        scratch.perm_draws, batch_weights, scratch.perm_weights,
                                        stream);
    std::vector<int> offsets(static_cast<size_t>(expert_count) + 1);
    CHECK_HIP(hipMemcpyAsync(offsets.data(), scratch.perm_offsets, offsets.size() * sizeof(int),
                             hipMemcpyDeviceToHost, stream));
    CHECK_HIP(hipStreamSynchronize(stream));

    int widest = 1;
    for (int e = 0; e < expert_count; ++e) widest = std::max(widest, offsets[e + 1] - offsets[e]);
    if (widest > scratch.hidden_tokens) {
        throw std::invalid_argument(
            "run_moe_grouped_expert_batch: the chunk's widest expert exceeds the scratch");
    }

    const int per_launch = kernel::kAeonSwizzledMaxExperts;
    for (int base = 0; base < expert_count; base += per_launch) {
        const int batch_count = std::min(per_launch, expert_count - base);
        if (offsets[base] == offsets[base + batch_count]) continue;  // no draws in this range
        const int first_draw = offsets[base];
        kernel::SwizzledW13ExpertPtrs w13{};
        kernel::SwizzledW2ExpertPtrs w2{};
        std::vector<int> rebased(static_cast<size_t>(batch_count) + 1);
        for (int j = 0; j < batch_count; ++j) {
            const int expert = base + j;
            rebased[j] = offsets[expert] - first_draw;
            fill(expert, j, offsets[expert + 1] - offsets[expert], w13, w2);
        }
        rebased[batch_count] = offsets[base + batch_count] - first_draw;
        // pageable host memory: the copy is complete, as far as the host buffer goes, on return
        CHECK_HIP(hipMemcpyAsync(scratch.batch_offsets, rebased.data(), rebased.size() * sizeof(int),
                                 hipMemcpyHostToDevice, stream));
        kernel::dispatch_aeon_moe_grouped_w13_swiglu_wmma<4, 4, 8, kernel::kMoeGroupedMTiles>(
            batch_input, scratch.batch_offsets, scratch.perm_tokens + first_draw, w13,
            scratch.chunk_hidden, batch_count, widest, scratch.intermediate, scratch.hidden,
            swiglu_limit, input_stride, stream);
        kernel::dispatch_aeon_moe_grouped_w2_wmma<4, 8, 4, kernel::kMoeGroupedMTiles>(
            scratch.chunk_hidden, scratch.batch_offsets, scratch.perm_draws + first_draw,
            scratch.perm_weights + first_draw, w2, scratch.chunk_contrib, batch_count, widest,
            scratch.hidden, scratch.intermediate, stream);
    }

    constexpr int kThreads = 256;
    for (uint32_t token = 0; token < token_count; ++token) {
        half* accum = batch_output + static_cast<size_t>(token) * output_stride;
        kernel::moe_accumulate_fixed_order_kernel<<<(scratch.hidden + kThreads - 1) / kThreads,
                                                    kThreads, 0, stream>>>(
            scratch.chunk_contrib + static_cast<size_t>(token) * slots * scratch.hidden, slots, accum,
            accum, scratch.hidden);
    }
}

}  // namespace aeon::core
