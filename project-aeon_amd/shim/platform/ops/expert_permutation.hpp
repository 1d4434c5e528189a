#pragma once
// dispatch_expert_permutation with the reference's signature and argument checks
// (src/platform/ops/expert_permutation.hpp:130-175).
#include "aeon355/status.hpp"

#include <hip/hip_runtime.h>

#include <stdexcept>

namespace aeon::kernel {

inline constexpr int kMaxPermutationExperts = 1024;

inline void dispatch_expert_permutation(const int* topk_indices, int token_count, int slots,
                                        int expert_count, int* expert_offsets, int* token_indices,
                                        int* draw_indices, const float* weights_by_draw = nullptr,
                                        float* weights_by_position = nullptr,
                                        hipStream_t stream = 0) {
    if (topk_indices == nullptr || expert_offsets == nullptr || token_indices == nullptr ||
        draw_indices == nullptr) {
        throw std::invalid_argument("dispatch_expert_permutation: null buffer");
    }
    if (token_count < 0 || slots <= 0) {
        throw std::invalid_argument("dispatch_expert_permutation: bad draw shape");
    }
    if (expert_count <= 0 || expert_count > kMaxPermutationExperts) {
        throw std::invalid_argument("dispatch_expert_permutation: expert count out of range");
    }
    if ((weights_by_draw == nullptr) != (weights_by_position == nullptr)) {
        throw std::invalid_argument(
            "dispatch_expert_permutation: weights need both a source and a destination");
    }
    aeon355::throw_on_error(aeon_expert_permutation(topk_indices, token_count, slots, expert_count,
                                                    expert_offsets, token_indices, draw_indices,
                                                    weights_by_draw, weights_by_position, stream));
}

}  // namespace aeon::kernel
