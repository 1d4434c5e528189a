#pragma once
// The model's two epilogue policies (moe_grouped_epilogue.hpp:29-47). The reference injects them
// into its kernels as device functors; the kernels behind the C ABI implement exactly these two
// rules, so a dispatcher here only reads `limit` out of the value it is handed. The device
// members are kept so that code written against the reference's types (a caller's own kernel, an
// explicit instantiation) still compiles and computes the same thing.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

namespace aeon::kernel {

// fp16( silu(min(gate, limit)) * clamp(up, -limit, +limit) ): the gate is bounded from above only
struct Dsv4ClampedSwiGLUEpilogue {
    float limit;

    __device__ half gate_up(float gate, float up) const {
        const float g = fminf(gate, limit);
        const float u = fmaxf(-limit, fminf(up, limit));
        return __float2half(g / (1.0f + expf(-g)) * u);
    }
};

// contribution = routing weight * accumulator
struct Dsv4RoutingWeightEpilogue {
    __device__ float down(float accumulator, float weight) const { return weight * accumulator; }
};

}  // namespace aeon::kernel
