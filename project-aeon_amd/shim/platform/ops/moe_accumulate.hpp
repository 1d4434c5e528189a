#pragma once
// moe_accumulate_fixed_order_kernel with the reference's name and signature
// (src/platform/ops/moe_accumulate.hpp:73-92), because its callers launch it with <<<>>>
// directly: out[i] = half(float(shared[i]) + sum of contrib[e][i] for e ascending), fp32,
// one rounding; `shared_output` may be null and may alias `out`.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

namespace aeon::kernel {

// The fp16-chain control (src/platform/ops/moe_accumulate.hpp:32-44), superseded in the
// reference and kept there for gates only: accum = half(float(accum) + weight * float(expert)),
// one fp16 rounding per expert.
__global__ inline void moe_accumulate_expert_kernel(half* __restrict__ accum_out,
                                                    const half* __restrict__ expert_out,
                                                    float weight, int hidden_dim) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < hidden_dim) {
        accum_out[i] = __float2half(__half2float(accum_out[i]) + weight * __half2float(expert_out[i]));
    }
}

__global__ inline void moe_accumulate_fixed_order_kernel(const float* __restrict__ contrib,
                                                         int expert_count,
                                                         const half* shared_output, half* out,
                                                         int hidden_dim) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < hidden_dim) {
        float acc = shared_output != nullptr ? __half2float(shared_output[i]) : 0.0f;
        for (int e = 0; e < expert_count; ++e) acc += contrib[static_cast<size_t>(e) * hidden_dim + i];
        out[i] = __float2half(acc);
    }
}

}  // namespace aeon::kernel
