#pragma once
// dispatch_dsv4_moe_gemv_w13_swiglu (moe_gemv_dispatch.hpp:28-45): the per-token gate/up pair
// with the model's clamped SwiGLU. Including this header brings both weight-table types, as
// the reference's does.
#include "architecture/deepseek_v4/kernels/moe_grouped_epilogue.hpp"
#include "backend/swizzled_w4a16/kernels/aeon_moe_fused_w13.hpp"
#include "backend/swizzled_w4a16/kernels/aeon_moe_fused_w2.hpp"

namespace aeon::kernel {

template <int WAVES, int RPW, int LPR, int ITERS>
inline void dispatch_dsv4_moe_gemv_w13_swiglu(const half* activation,
                                              const SwizzledW13ExpertPtrs& weights,
                                              half* expert_hidden, float* output_f32,
                                              int output_dim, int expert_count, int N, int K,
                                              float swiglu_limit, hipStream_t stream = 0) {
    dispatch_aeon_moe_fused_gate_up<WAVES, RPW, LPR, ITERS>(
        activation, weights, expert_hidden, output_f32, output_dim, expert_count, N, K,
        Dsv4ClampedSwiGLUEpilogue{swiglu_limit}, stream);
}

}  // namespace aeon::kernel
