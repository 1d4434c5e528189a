#pragma once
// SwizzledW2ExpertPtrs and dispatch_aeon_moe_fused_w2_contrib (aeon_moe_fused_w2.hpp:12-15,
// 231-256): contrib[e*N + row] = topk_w[e] * (W2_e . hidden_e)[row], one writer per element.
// dispatch_aeon_moe_fused_w2_accum (:144-174), a superseded control in the reference, keeps its
// signature; the sum behind it runs in slot order in one workgroup per row block instead of
// through atomicAdd, and the completion counters are left as the caller set them.
#include "backend/swizzled_w4a16/kernels/aeon_moe_fused_w13.hpp"

namespace aeon::kernel {

struct SwizzledW2ExpertPtrs {
    const uint4* w2[kAeonSwizzledMaxExperts];
    const half* s2[kAeonSwizzledMaxExperts];
};
static_assert(sizeof(SwizzledW2ExpertPtrs) == sizeof(aeon_w2_table),
              "the table is handed to the C ABI by layout");

template <int WAVES, int RPW, int LPR, int ITERS>
inline void dispatch_aeon_moe_fused_w2_contrib(const half* expert_hidden,
                                               const SwizzledW2ExpertPtrs& weights,
                                               const float* topk_weights, float* contrib,
                                               int expert_count, int N, int K,
                                               hipStream_t stream = 0) {
    static_assert(RPW * LPR == 32, "RPW and LPR must describe one 32-slot storage tile");
    if (expert_count <= 0 || expert_count > kAeonSwizzledMaxExperts || N <= 0 ||
        K != ITERS * LPR * 32 || N % RPW != 0 || contrib == nullptr) {
        throw std::invalid_argument(
            "dispatch_aeon_moe_fused_w2_contrib: incompatible expert or N/K shape");
    }
    aeon_w2_table table;
    std::memcpy(&table, &weights, sizeof table);
    aeon355::throw_on_error(aeon_moe_fused_w2_contrib(expert_hidden, &table, topk_weights, contrib,
                                                      expert_count, N, K, RPW, LPR, stream));
}

template <int WAVES, int RPW, int LPR, int ITERS>
inline void dispatch_aeon_moe_fused_w2_accum(const half* expert_hidden,
                                             const SwizzledW2ExpertPtrs& weights,
                                             const float* topk_weights, const half* initial_output,
                                             float* output_f32, half* output_f16, int* counters,
                                             int expert_count, int N, int K,
                                             hipStream_t stream = 0) {
    static_assert(RPW * LPR == 32, "RPW and LPR must describe one 32-slot storage tile");
    (void)counters;
    if (expert_count <= 0 || expert_count > kAeonSwizzledMaxExperts || N <= 0 ||
        K != ITERS * LPR * 32 || N % RPW != 0) {
        throw std::invalid_argument(
            "dispatch_aeon_moe_fused_w2_accum: incompatible expert or N/K shape");
    }
    aeon_w2_table table;
    std::memcpy(&table, &weights, sizeof table);
    aeon355::throw_on_error(aeon_moe_fused_w2_accum(expert_hidden, &table, topk_weights,
                                                    initial_output, output_f32, output_f16,
                                                    expert_count, N, K, RPW, LPR, stream));
}

}  // namespace aeon::kernel
