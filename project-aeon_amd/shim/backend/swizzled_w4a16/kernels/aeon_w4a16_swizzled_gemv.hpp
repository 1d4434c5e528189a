#pragma once
// dispatch_aeon_w4a16_swizzled_{gemv,dual_gemv} with the reference's signatures
// (aeon_w4a16_swizzled_gemv.hpp:166-222), forwarding to the gfx950 library. The template
// arguments describe the payload's wave32 storage geometry; they are validated exactly as the
// reference does (K == ITERS*LPR*32, N % RPW == 0 -> std::invalid_argument) and passed on as
// runtime values. WAVES was a launch-shape tuning knob of the wave32 kernel and has no meaning
// for the wave64 one. Launch errors are left for the caller's hipGetLastError, as before.
#include "aeon355/status.hpp"
#include "backend/swizzled_w4a16/kernels/aeon_w4a16_swizzle.hpp"

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>
#include <stdexcept>

namespace aeon::kernel {

template <int WAVES, int RPW, int LPR, int ITERS>
inline void dispatch_aeon_w4a16_swizzled_gemv(const half* activation, const uint32_t* packed,
                                              const half* scale, half* output, int N, int K,
                                              hipStream_t stream = 0) {
    static_assert(RPW * LPR == 32, "RPW and LPR must describe one 32-slot storage tile");
    if (N <= 0 || K != ITERS * LPR * 32 || N % RPW != 0) {
        throw std::invalid_argument("dispatch_aeon_w4a16_swizzled_gemv: incompatible N/K shape");
    }
    aeon355::throw_on_error(
        aeon_w4a16_swizzled_gemv(activation, packed, scale, output, N, K, RPW, LPR, stream));
}

template <int WAVES, int RPW, int LPR, int ITERS>
inline void dispatch_aeon_w4a16_swizzled_dual_gemv(const half* activation, const uint32_t* packed_a,
                                                   const half* scale_a, const uint32_t* packed_b,
                                                   const half* scale_b, half* output_a,
                                                   half* output_b, int N, int K,
                                                   hipStream_t stream = 0) {
    static_assert(RPW * LPR == 32, "RPW and LPR must describe one 32-slot storage tile");
    if (N <= 0 || K != ITERS * LPR * 32 || N % RPW != 0) {
        throw std::invalid_argument("dispatch_aeon_w4a16_swizzled_dual_gemv: incompatible N/K shape");
    }
    aeon355::throw_on_error(aeon_w4a16_swizzled_dual_gemv(activation, packed_a, scale_a, packed_b,
                                                          scale_b, output_a, output_b, N, K, RPW,
                                                          LPR, stream));
}

}  // namespace aeon::kernel
