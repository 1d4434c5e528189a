#pragma once
// dispatch_aeon_moe_grouped_{w13_swiglu,w2}_wmma (moe_grouped_dispatch.hpp:40-88) with the
// reference's signatures. The names keep their `_wmma` suffix because callers spell them so;
// behind them is the gfx950 MFMA kernel. WAVES and MTILES were tuning knobs of the wave32 WMMA
// kernel and are ignored.
#include "architecture/deepseek_v4/kernels/moe_grouped_epilogue.hpp"
#include "backend/swizzled_w4a16/kernels/aeon_moe_fused_w2.hpp"

namespace aeon::kernel {

inline constexpr int kMoeGroupedMTiles = 4;

template <int WAVES, int RPW, int LPR, int MTILES>
inline void dispatch_aeon_moe_grouped_w13_swiglu_wmma(
    const half* activation, const int* expert_offsets, const int* token_indices,
    const SwizzledW13ExpertPtrs& weights, half* expert_hidden, int expert_count,
    int expert_hidden_tokens, int N, int K, float swiglu_limit, int activation_stride = 0,
    hipStream_t stream = 0) {
    aeon_w13_table table;
    std::memcpy(&table, &weights, sizeof table);
    aeon355::throw_on_error(aeon_moe_grouped_w13_swiglu(
        activation, expert_offsets, token_indices, &table, expert_hidden, expert_count,
        expert_hidden_tokens, N, K, RPW, LPR, swiglu_limit, activation_stride, stream));
}

template <int WAVES, int RPW, int LPR, int MTILES>
inline void dispatch_aeon_moe_grouped_w2_wmma(const half* expert_hidden, const int* expert_offsets,
                                              const int* draw_indices, const float* draw_weights,
                                              const SwizzledW2ExpertPtrs& weights, float* contrib,
                                              int expert_count, int expert_hidden_tokens, int N,
                                              int K, hipStream_t stream = 0) {
    aeon_w2_table table;
    std::memcpy(&table, &weights, sizeof table);
    aeon355::throw_on_error(aeon_moe_grouped_w2(expert_hidden, expert_offsets, draw_indices,
                                                draw_weights, &table, contrib, expert_count,
                                                expert_hidden_tokens, N, K, RPW, LPR, stream));
}

}  // namespace aeon::kernel
