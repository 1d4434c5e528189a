#pragma once
// The model's two epilogue choices, as plain host-side values (the reference passes them as
// device functors, moe_grouped_epilogue.hpp:29-47; here the kernels behind the C ABI implement
// exactly these two rules, so the types only carry the parameter).
namespace aeon::kernel {

// silu(min(gate, limit)) * clamp(up, -limit, +limit), stored as fp16
struct Dsv4ClampedSwiGLUEpilogue {
    float limit;
};

// contribution = routing weight * accumulator
struct Dsv4RoutingWeightEpilogue {};

}  // namespace aeon::kernel
