#pragma once
// The hyper-connection kernels behind the reference's own names and launch shapes
// (src/architecture/deepseek_v4/kernels/hc_sinkhorn.hpp:22-290), for callers that launch them
// with <<<>>> themselves:
//   hc_project_kernel            <<<dim3(24, tokens), 256>>>   mixes[t][m] = rsqrt(mean(r^2) + eps) * (r . fn[m])
//   hc_sinkhorn_normalize_kernel <<<tokens, 32>>>              pre/post gates and the 4x4 comb matrix
//   hc_pre_combine_kernel        <<<dim3(ceil(hidden/4/256), tokens), 256>>>  layer_input = sum_j pre[j] * r[j]
//   hc_post_kernel               <<<dim3(ceil(hidden/block), tokens), block>>> out[j] = post[j]*y + sum_i comb[i][j]*r[i]
// The residual is fp32 [tokens][hc_mult][hidden] for the first and third, fp16 for the last,
// as in the reference. The batched library calls for the same steps are aeon_hc_project,
// aeon_hc_sinkhorn_normalize, aeon_hc_pre_combine and aeon_hc_post (include/aeon_mi355.h).
//
// Written for 64-wide waves: the projection reduces over whole waves and sums the workgroup's
// partials in wave order (fixed order, no atomics); the 4x4 normalisation runs in the registers
// of one lane per token, which a 32-thread block (half a wave) carries as well as a full one.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

namespace aeon::kernel {

__global__ void __launch_bounds__(256) hc_project_kernel(const float* __restrict__ residual_in,
                                                         const float* __restrict__ fn,
                                                         float* __restrict__ mixes, int hidden_size,
                                                         int hc_mult, float rms_eps) {
    const int mix = blockIdx.x;
    const int token = blockIdx.y;
    const int width = hc_mult * hidden_size;
    const float* r = residual_in + static_cast<size_t>(token) * width;
    const float* f = fn + static_cast<size_t>(mix) * width;
    float squares = 0.0f, dot = 0.0f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float v = r[i];
        squares += v * v;
        dot += v * f[i];
    }
    for (int offset = 32; offset > 0; offset >>= 1) {
        squares += __shfl_xor(squares, offset, 64);
        dot += __shfl_xor(dot, offset, 64);
    }
    __shared__ float wave_squares[16], wave_dot[16];
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
        wave_squares[wave] = squares;
        wave_dot[wave] = dot;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float s = 0.0f, d = 0.0f;
        for (int w = 0; w < static_cast<int>(blockDim.x + 63) / 64; ++w) {
            s += wave_squares[w];
            d += wave_dot[w];
        }
        mixes[static_cast<size_t>(token) * 24 + mix] = d * rsqrtf(s / static_cast<float>(width) + rms_eps);
    }
}

__global__ void __launch_bounds__(256) hc_pre_combine_kernel(const float* __restrict__ residual_in,
                                                             const float* __restrict__ pre_mix,
                                                             __half* __restrict__ layer_input,
                                                             int hidden_size, int hc_mult) {
    const int token = blockIdx.y;
    const int column = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (column >= hidden_size) return;
    const float* r = residual_in + static_cast<size_t>(token) * hc_mult * hidden_size + column;
    const float* p = pre_mix + static_cast<size_t>(token) * 4;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int j = 0; j < hc_mult; ++j) {
        const float4 v = *reinterpret_cast<const float4*>(r + static_cast<size_t>(j) * hidden_size);
        acc[0] += p[j] * v.x;
        acc[1] += p[j] * v.y;
        acc[2] += p[j] * v.z;
        acc[3] += p[j] * v.w;
    }
    __half2* out = reinterpret_cast<__half2*>(layer_input + static_cast<size_t>(token) * hidden_size + column);
    out[0] = __floats2half2_rn(acc[0], acc[1]);
    out[1] = __floats2half2_rn(acc[2], acc[3]);
}

__global__ void __launch_bounds__(64) hc_sinkhorn_normalize_kernel(
    const float* __restrict__ mixes, const float* __restrict__ hc_scale,
    const float* __restrict__ hc_base, float* __restrict__ pre_mix, float* __restrict__ post_mix,
    float* __restrict__ comb_mix, float hc_pre_eps, float hc_sinkhorn_eps, float hc_post_alpha,
    int sinkhorn_iters) {
    if (threadIdx.x != 0) return;
    const int token = blockIdx.x;
    const float* m = mixes + static_cast<size_t>(token) * 24;
    for (int j = 0; j < 4; ++j) {
        const float a = m[j] * hc_scale[0] + hc_base[j];
        pre_mix[token * 4 + j] = 1.0f / (1.0f + expf(-a)) + hc_pre_eps;
        const float b = m[j + 4] * hc_scale[1] + hc_base[j + 4];
        post_mix[token * 4 + j] = (1.0f / (1.0f + expf(-b))) * hc_post_alpha;
    }
    float c[4][4];
    for (int i = 0; i < 4; ++i) {
        float row[4];
        for (int j = 0; j < 4; ++j) row[j] = m[8 + i * 4 + j] * hc_scale[2] + hc_base[8 + i * 4 + j];
        const float top = fmaxf(fmaxf(row[0], row[1]), fmaxf(row[2], row[3]));
        float e[4];
        for (int j = 0; j < 4; ++j) e[j] = expf(row[j] - top);
        const float sum = e[0] + e[1] + e[2] + e[3];
        for (int j = 0; j < 4; ++j) c[i][j] = e[j] / sum + hc_sinkhorn_eps;
    }
    // softmax rows, then columns, then (iters - 1) x (rows, columns)
    for (int pass = 0; pass < 2 * sinkhorn_iters - 1; ++pass) {
        if ((pass & 1) == 0) {
            for (int j = 0; j < 4; ++j) {
                const float inv = 1.0f / (c[0][j] + c[1][j] + c[2][j] + c[3][j] + hc_sinkhorn_eps);
                for (int i = 0; i < 4; ++i) c[i][j] *= inv;
            }
        } else {
            for (int i = 0; i < 4; ++i) {
                const float inv = 1.0f / (c[i][0] + c[i][1] + c[i][2] + c[i][3] + hc_sinkhorn_eps);
                for (int j = 0; j < 4; ++j) c[i][j] *= inv;
            }
        }
    }
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j) comb_mix[token * 16 + i * 4 + j] = c[i][j];
}

__global__ void hc_post_kernel(const __half* __restrict__ layer_out,
                               const __half* __restrict__ residual_in,
                               const float* __restrict__ post_mix,
                               const float* __restrict__ comb_mix,
                               __half* __restrict__ residual_out, int hidden_size) {
    const int token = blockIdx.y;
    const int h = blockIdx.x * blockDim.x + threadIdx.x;
    if (h >= hidden_size) return;
    const size_t base = static_cast<size_t>(token) * 4 * hidden_size + h;
    const float y = __half2float(layer_out[static_cast<size_t>(token) * hidden_size + h]);
    float r[4];
    for (int i = 0; i < 4; ++i) r[i] = __half2float(residual_in[base + static_cast<size_t>(i) * hidden_size]);
    const float* post = post_mix + static_cast<size_t>(token) * 4;
    const float* comb = comb_mix + static_cast<size_t>(token) * 16;
    for (int j = 0; j < 4; ++j) {
        float v = post[j] * y;
        for (int i = 0; i < 4; ++i) v += comb[i * 4 + j] * r[i];
        residual_out[base + static_cast<size_t>(j) * hidden_size] = __float2half(v);
    }
}

}  // namespace aeon::kernel
