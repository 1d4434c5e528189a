#pragma once
// The model-named entry point of the per-token expert pair,
// dispatch_dsv4_moe_gemv_w13_swiglu (moe_gemv_dispatch.hpp:28-45). A caller that includes this
// header gets both weight-table types with it, as with the reference's. The library has the
// model's clamped SwiGLU built into its gate/up launch, so the call goes straight to the C ABI
// with the clamp limit as a number.
#include "backend/swizzled_w4a16/kernels/aeon_moe_fused_w2.hpp"
#include "backend/swizzled_w4a16/kernels/aeon_moe_fused_w13.hpp"
#include "architecture/deepseek_v4/kernels/moe_grouped_epilogue.hpp"

namespace aeon::kernel {

template <int WAVES, int RPW, int LPR, int ITERS>
inline void dispatch_dsv4_moe_gemv_w13_swiglu(const half* activation,
                                              const SwizzledW13ExpertPtrs& weights,
                                              half* expert_hidden, float* output_f32,
                                              int output_dim, int expert_count, int N, int K,
                                              float swiglu_limit, hipStream_t stream = 0) {
    static_assert(RPW * LPR == 32, "RPW and LPR must describe one 32-slot storage tile");
    const bool shape_ok = N > 0 && N % RPW == 0 && K == ITERS * LPR * 32;
    const bool count_ok = expert_count >= 1 && expert_count <= kAeonSwizzledMaxExperts;
    if (!shape_ok || !count_ok) {
        throw std::invalid_argument(
            "dispatch_dsv4_moe_gemv_w13_swiglu: incompatible expert or N/K shape");
    }
    aeon_w13_table by_layout;
    std::memcpy(&by_layout, &weights, sizeof by_layout);
    const int status = aeon_moe_gemv_w13_swiglu(activation, &by_layout, expert_hidden, output_f32,
                                                output_dim, expert_count, N, K, RPW, LPR,
                                                swiglu_limit, stream);
    aeon355::throw_on_error(status);
}

}  // namespace aeon::kernel
