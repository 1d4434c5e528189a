#pragma once
// The model's clamped SwiGLU as an element-wise kernel under the reference's name
// (src/architecture/deepseek_v4/kernels/v4_swiglu_clamp.hpp:18-34), for callers that launch it
// with <<<>>> themselves (v4_layer_body_moe.hpp:242, the shared-expert path):
// out = silu(min(gate, limit)) * clamp(up, -limit, +limit) in fp32, one fp16 rounding. The gate
// is bounded only from above. The fused kernels apply the same function inside the gate/up
// launch; the library call for a standalone pass is aeon_swiglu_clamp (include/aeon_mi355.h).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

namespace aeon::kernel {

__global__ inline void v4_swiglu_clamp_kernel(const half* __restrict__ gate,
                                              const half* __restrict__ up, half* __restrict__ out,
                                              int total_elements, float limit) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total_elements) return;
    const float g = fminf(__half2float(gate[i]), limit);
    const float u = fminf(fmaxf(__half2float(up[i]), -limit), limit);
    out[i] = __float2half((g / (1.0f + expf(-g))) * u);
}

}  // namespace aeon::kernel
