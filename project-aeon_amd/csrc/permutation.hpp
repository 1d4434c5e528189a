// Internal launch interface of the token -> expert permutation.
#pragma once

#include "common.hpp"

namespace aeon355 {

// One thread per expert list in the scan: the reference primitive's own bound
// (kMaxPermutationExperts, src/platform/ops/expert_permutation.hpp:46-47), which here has to
// include the always-on expert's list when there is one.
constexpr int kMaxPermutationExperts = 1024;

struct PermutationArgs {
    const int32_t* ids;  // [draws] expert of draw token*slots+slot
    int draws;
    int slots;
    unsigned slots_reciprocal;  // filled by launch_permutation
    int experts;         // routed experts
    int shared_tokens;   // > 0: append one more list holding tokens 0..shared_tokens-1
    int32_t* offsets;    // [lists + 1]
    int32_t* token_indices;  // [positions]
    int32_t* draw_indices;   // [positions]; the appended list gets rows draws..draws+tokens-1
    const float* weights_by_draw;  // nullable together with weights_by_position
    float* weights_by_position;
    // optional segment list: each list cut into runs of at most seg_tokens positions
    int32_t* seg_expert;
    int32_t* seg_first;
    int32_t* seg_count;
    int32_t* seg_total;
    int seg_tokens;
    int seg_capacity;
    int32_t* seg_alone = nullptr;  // optional [seg_capacity]: 1 where a list has a single segment
};

int launch_permutation(const PermutationArgs& a, hipStream_t stream);

}  // namespace aeon355
