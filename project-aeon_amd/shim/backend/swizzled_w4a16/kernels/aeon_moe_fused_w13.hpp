#pragma once
// SwizzledW13ExpertPtrs and dispatch_aeon_moe_fused_gate_up (aeon_moe_fused_w13.hpp:13-141).
#include "architecture/deepseek_v4/kernels/moe_grouped_epilogue.hpp"
#include "backend/swizzled_w4a16/kernels/aeon_w4a16_swizzled_gemv.hpp"

#include <cstring>
#include <type_traits>

namespace aeon::kernel {

constexpr int kAeonSwizzledMaxExperts = AEON_SWIZZLED_MAX_EXPERTS;

struct SwizzledW13ExpertPtrs {
    const uint4* w1[kAeonSwizzledMaxExperts];
    const half* s1[kAeonSwizzledMaxExperts];
    const uint4* w3[kAeonSwizzledMaxExperts];
    const half* s3[kAeonSwizzledMaxExperts];
};
static_assert(sizeof(SwizzledW13ExpertPtrs) == sizeof(aeon_w13_table),
              "the table is handed to the C ABI by layout");

// The gate/up pair. `Epilogue` is a template parameter as in the reference (:113); the library
// behind this call implements the model's clamped SwiGLU, so that is the one policy accepted --
// any other is refused when the call is compiled, not computed with the wrong rule.
template <int WAVES, int RPW, int LPR, int ITERS, class Epilogue>
inline void dispatch_aeon_moe_fused_gate_up(const half* activation,
                                            const SwizzledW13ExpertPtrs& weights,
                                            half* expert_hidden, float* output_f32, int output_dim,
                                            int expert_count, int N, int K,
                                            Epilogue epilogue, hipStream_t stream = 0) {
    static_assert(std::is_same_v<Epilogue, Dsv4ClampedSwiGLUEpilogue>,
                  "the gfx950 gate/up kernels implement Dsv4ClampedSwiGLUEpilogue only");
    static_assert(RPW * LPR == 32, "RPW and LPR must describe one 32-slot storage tile");
    if (expert_count <= 0 || expert_count > kAeonSwizzledMaxExperts || N <= 0 ||
        K != ITERS * LPR * 32 || N % RPW != 0) {
        throw std::invalid_argument(
            "dispatch_aeon_moe_fused_gate_up: incompatible expert or N/K shape");
    }
    aeon_w13_table table;
    std::memcpy(&table, &weights, sizeof table);
    aeon355::throw_on_error(aeon_moe_gemv_w13_swiglu(activation, &table, expert_hidden, output_f32,
                                                     output_dim, expert_count, N, K, RPW, LPR,
                                                     epilogue.limit, stream));
}

}  // namespace aeon::kernel
