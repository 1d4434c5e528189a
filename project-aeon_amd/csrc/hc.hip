// Hyper-connection mixing around the MoE: the Sinkhorn-normalised 4x4 stream mix and the
// pre-combine / post expansion over the four residual streams (hc_mult = 4).
//
// Conventions kept from the reference kernels: comb[i*4 + j] with i the contraction stream and
// j the output stream; the softmax runs over j, the first normalisation over i, then
// (iters - 1) x (over j, over i); every denominator carries the Sinkhorn eps; pre carries
// +eps, post is x post_alpha with no eps. All arithmetic in fp32, streams in fp16.
#include "common.hpp"

namespace aeon355 {

constexpr int kHc = 4;

__global__ __launch_bounds__(64) void hc_sinkhorn_kernel(
    const float* __restrict__ mixes, const float* __restrict__ hc_scale,
    const float* __restrict__ hc_base, float* __restrict__ pre, float* __restrict__ post,
    float* __restrict__ comb, int tokens, float pre_eps, float sinkhorn_eps, float post_alpha,
    int iters) {
    // one thread per token: the matrix is 4x4 and lives in registers
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= tokens) return;
    const float* m = mixes + static_cast<size_t>(t) * 24;
#pragma unroll
    for (int j = 0; j < kHc; ++j) {
        const float a = m[j] * hc_scale[0] + hc_base[j];
        pre[t * 4 + j] = 1.0f / (1.0f + expf(-a)) + pre_eps;
        const float b = m[j + 4] * hc_scale[1] + hc_base[j + 4];
        post[t * 4 + j] = (1.0f / (1.0f + expf(-b))) * post_alpha;
    }
    float c[kHc][kHc];
#pragma unroll
    for (int i = 0; i < kHc; ++i) {
        float row[kHc];
#pragma unroll
        for (int j = 0; j < kHc; ++j) row[j] = m[8 + i * 4 + j] * hc_scale[2] + hc_base[8 + i * 4 + j];
        const float mx = fmaxf(fmaxf(row[0], row[1]), fmaxf(row[2], row[3]));
        float e[kHc];
        float sum = 0.0f;
#pragma unroll
        for (int j = 0; j < kHc; ++j) {
            e[j] = expf(row[j] - mx);
        }
        sum = e[0] + e[1] + e[2] + e[3];
#pragma unroll
        for (int j = 0; j < kHc; ++j) c[i][j] = e[j] / sum + sinkhorn_eps;
    }
    for (int pass = 0; pass < 2 * iters - 1; ++pass) {
        if ((pass & 1) == 0) {
#pragma unroll
            for (int j = 0; j < kHc; ++j) {
                const float inv = 1.0f / (c[0][j] + c[1][j] + c[2][j] + c[3][j] + sinkhorn_eps);
#pragma unroll
                for (int i = 0; i < kHc; ++i) c[i][j] *= inv;
            }
        } else {
#pragma unroll
            for (int i = 0; i < kHc; ++i) {
                const float inv = 1.0f / (c[i][0] + c[i][1] + c[i][2] + c[i][3] + sinkhorn_eps);
#pragma unroll
                for (int j = 0; j < kHc; ++j) c[i][j] *= inv;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < kHc; ++i)
#pragma unroll
        for (int j = 0; j < kHc; ++j) comb[t * 16 + i * 4 + j] = c[i][j];
}

// layer_input[t][h] = sum_j pre[j] * residual[t][j][h], eight columns per thread.
template <bool F32>
__global__ __launch_bounds__(256) void hc_pre_combine_kernel(
    const void* __restrict__ residual, long token_stride, long stream_stride,
    const float* __restrict__ pre, int pre_token_stride, uint16_t* __restrict__ out, long out_stride,
    int hidden) {
    const int t = blockIdx.y;
    const int h = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (h >= hidden) return;
    const float* p = pre + static_cast<size_t>(t) * pre_token_stride;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < kHc; ++j) {
        const float pj = p[j];
        if (F32) {
            const float* r = static_cast<const float*>(residual) + t * token_stride + j * stream_stride + h;
            const float4_t a = *reinterpret_cast<const float4_t*>(r);
            const float4_t b = *reinterpret_cast<const float4_t*>(r + 4);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                acc[q] += pj * a[q];
                acc[4 + q] += pj * b[q];
            }
        } else {
            const uint16_t* r = static_cast<const uint16_t*>(residual) + t * token_stride + j * stream_stride + h;
            const half8_t v = *reinterpret_cast<const half8_t*>(r);
#pragma unroll
            for (int q = 0; q < 8; ++q) acc[q] += pj * static_cast<float>(v[q]);
        }
    }
    half8_t o;
#pragma unroll
    for (int q = 0; q < 8; ++q) o[q] = static_cast<half_t>(acc[q]);
    *reinterpret_cast<half8_t*>(out + t * out_stride + h) = o;
}

// out[t][j][h] = post[j] * layer_out[t][h] + sum_i comb[i*4+j] * residual[t][i][h]
__global__ __launch_bounds__(256) void hc_post_kernel(
    const uint16_t* __restrict__ layer_out, long layer_out_stride,
    const uint16_t* __restrict__ residual_in, long token_stride, long stream_stride,
    const float* __restrict__ post, const float* __restrict__ comb, int mix_token_stride,
    uint16_t* __restrict__ residual_out, int hidden) {
    const int t = blockIdx.y;
    const int h = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (h >= hidden) return;
    const float* pm = post + static_cast<size_t>(t) * mix_token_stride * 4;
    const float* cm = comb + static_cast<size_t>(t) * mix_token_stride * 16;
    const half8_t lo = *reinterpret_cast<const half8_t*>(layer_out + t * layer_out_stride + h);
    half8_t r[kHc];
#pragma unroll
    for (int i = 0; i < kHc; ++i) {
        r[i] = *reinterpret_cast<const half8_t*>(residual_in + t * token_stride + i * stream_stride + h);
    }
#pragma unroll
    for (int j = 0; j < kHc; ++j) {
        half8_t o;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            float v = pm[j] * static_cast<float>(lo[q]);
#pragma unroll
            for (int i = 0; i < kHc; ++i) v += cm[i * 4 + j] * static_cast<float>(r[i][q]);
            o[q] = static_cast<half_t>(v);
        }
        *reinterpret_cast<half8_t*>(residual_out + t * token_stride + j * stream_stride + h) = o;
    }
}

}  // namespace aeon355

using namespace aeon355;

extern "C" int aeon_hc_sinkhorn_normalize(const float* d_mixes, const float* d_hc_scale,
                                          const float* d_hc_base, float* d_pre_mix,
                                          float* d_post_mix, float* d_comb_mix, int tokens,
                                          float hc_pre_eps, float hc_sinkhorn_eps,
                                          float hc_post_alpha, int sinkhorn_iters, void* stream) {
    const char* who = "aeon_hc_sinkhorn_normalize";
    AEON_REQUIRE(d_mixes && d_hc_scale && d_hc_base && d_pre_mix && d_post_mix && d_comb_mix,
                 AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    AEON_REQUIRE(tokens >= 0 && sinkhorn_iters >= 1, AEON_ERR_INVALID_ARGUMENT,
                 "%s: bad shape (tokens=%d iters=%d)", who, tokens, sinkhorn_iters);
    if (tokens == 0) return AEON_OK;
    hc_sinkhorn_kernel<<<(tokens + 63) / 64, 64, 0, as_stream(stream)>>>(
        d_mixes, d_hc_scale, d_hc_base, d_pre_mix, d_post_mix, d_comb_mix, tokens, hc_pre_eps,
        hc_sinkhorn_eps, hc_post_alpha, sinkhorn_iters);
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

extern "C" int aeon_hc_pre_combine(const void* d_residual, int residual_is_f32, long token_stride,
                                   long stream_stride, const float* d_pre_mix,
                                   int pre_token_stride, void* d_layer_input, long out_stride,
                                   int tokens, int hidden, void* stream) {
    const char* who = "aeon_hc_pre_combine";
    AEON_REQUIRE(d_residual && d_pre_mix && d_layer_input, AEON_ERR_INVALID_ARGUMENT,
                 "%s: null buffer", who);
    AEON_REQUIRE(tokens >= 0 && hidden > 0 && hidden % 8 == 0 && token_stride % 8 == 0 &&
                     stream_stride % 8 == 0 && out_stride % 8 == 0 && out_stride >= hidden &&
                     (pre_token_stride == 0 || pre_token_stride == 4),
                 AEON_ERR_INVALID_ARGUMENT, "%s: bad shape or pitch", who);
    if (tokens == 0) return AEON_OK;
    const dim3 grid((hidden / 8 + 255) / 256, tokens);
    if (residual_is_f32) {
        hc_pre_combine_kernel<true><<<grid, 256, 0, as_stream(stream)>>>(
            d_residual, token_stride, stream_stride, d_pre_mix, pre_token_stride,
            static_cast<uint16_t*>(d_layer_input), out_stride, hidden);
    } else {
        hc_pre_combine_kernel<false><<<grid, 256, 0, as_stream(stream)>>>(
            d_residual, token_stride, stream_stride, d_pre_mix, pre_token_stride,
            static_cast<uint16_t*>(d_layer_input), out_stride, hidden);
    }
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

namespace aeon355 {

// mixes[t][m] = rsqrt(mean(r^2) + eps) * sum_k r[k] * fn[m][k] over the token's flattened
// hc_mult x hidden residual r. One workgroup per token reads the residual once and carries all
// 24 dot products plus the sum of squares (the reference launches one block per (mix, token),
// reading the residual 24 times); fn (24 rows of hc_mult*hidden floats) is shared by every
// token and stays in L2. Thread partials are combined in a fixed order -- xor butterfly inside
// a wave, then waves 0..3 in sequence -- so a run is reproducible bit for bit.
constexpr int kHcMixes = kHc * (2 + kHc);

template <bool RESIDUAL_F32>
__global__ __launch_bounds__(256) void hc_project_kernel(
    const void* __restrict__ residual, long token_stride, long stream_stride,
    const float* __restrict__ fn, float* __restrict__ mixes, int hidden, float rms_eps) {
    const int token = blockIdx.x;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    float dot[kHcMixes];
#pragma unroll
    for (int m = 0; m < kHcMixes; ++m) dot[m] = 0.0f;
    float sum_sq = 0.0f;
    const size_t flat = static_cast<size_t>(kHc) * hidden;
    for (int j = 0; j < kHc; ++j) {
        for (int h = threadIdx.x * 4; h < hidden; h += 256 * 4) {
            float r[4];
            const size_t at = static_cast<size_t>(token) * token_stride + j * stream_stride + h;
            if (RESIDUAL_F32) {
                const float4 v = *reinterpret_cast<const float4*>(static_cast<const float*>(residual) + at);
                r[0] = v.x; r[1] = v.y; r[2] = v.z; r[3] = v.w;
            } else {
                const uint2 v = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(residual) + at);
                r[0] = half_bits_to_float(static_cast<uint16_t>(v.x & 0xFFFFu));
                r[1] = half_bits_to_float(static_cast<uint16_t>(v.x >> 16));
                r[2] = half_bits_to_float(static_cast<uint16_t>(v.y & 0xFFFFu));
                r[3] = half_bits_to_float(static_cast<uint16_t>(v.y >> 16));
            }
            sum_sq += r[0] * r[0] + r[1] * r[1] + r[2] * r[2] + r[3] * r[3];
            const float* f = fn + static_cast<size_t>(j) * hidden + h;
#pragma unroll
            for (int m = 0; m < kHcMixes; ++m) {
                const float4 w = *reinterpret_cast<const float4*>(f + m * flat);
                dot[m] += r[0] * w.x + r[1] * w.y + r[2] * w.z + r[3] * w.w;
            }
        }
    }
    __shared__ float partial[4][kHcMixes + 1];
#pragma unroll
    for (int m = 0; m < kHcMixes; ++m) {
        const float v = wave_xor_sum(dot[m], 63);
        if (lane == 0) partial[wave][m] = v;
    }
    const float sq = wave_xor_sum(sum_sq, 63);
    if (lane == 0) partial[wave][kHcMixes] = sq;
    __syncthreads();
    if (threadIdx.x < kHcMixes) {
        const float total_sq = ((partial[0][kHcMixes] + partial[1][kHcMixes]) + partial[2][kHcMixes]) +
                               partial[3][kHcMixes];
        const float total = ((partial[0][threadIdx.x] + partial[1][threadIdx.x]) + partial[2][threadIdx.x]) +
                            partial[3][threadIdx.x];
        mixes[static_cast<size_t>(token) * kHcMixes + threadIdx.x] =
            total * rsqrtf(total_sq / static_cast<float>(flat) + rms_eps);
    }
}

// out[t][i] = half(x[t][i] * rsqrt(mean(x[t]^2) + eps) * weight[i]); fp32 arithmetic, fp16 in and
// out, fp16 weight (null = the weightless form). One workgroup per token; the sum of squares is
// combined in the same fixed order as above.
// VEC: rows and pitches are multiples of 8 elements and 16-byte aligned, so a thread moves eight
// values at a time and keeps its share of the row (up to kRmsHeld x 8 values) in registers
// between the two passes; otherwise one value at a time, the row read twice.
constexpr int kRmsHeld = 4;  // 256 threads x 8 x 4 = rows of up to 8192 stay in registers
template <bool VEC>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const uint16_t* __restrict__ x, long x_stride,
                                                      const uint16_t* __restrict__ weight,
                                                      uint16_t* __restrict__ out, long out_stride,
                                                      int dim, float eps) {
    const int token = blockIdx.x;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const uint16_t* row = x + static_cast<size_t>(token) * x_stride;
    float sum_sq = 0.0f;
    half8_t held[kRmsHeld];
    if (VEC) {
#pragma unroll
        for (int r = 0; r < kRmsHeld; ++r) {
            const int i = (r * 256 + threadIdx.x) * 8;
            if (i < dim) {
                held[r] = *reinterpret_cast<const half8_t*>(row + i);
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    const float v = static_cast<float>(held[r][q]);
                    sum_sq += v * v;
                }
            }
        }
        for (int i = (kRmsHeld * 256 + threadIdx.x) * 8; i < dim; i += 256 * 8) {
            const half8_t v8 = *reinterpret_cast<const half8_t*>(row + i);
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const float v = static_cast<float>(v8[q]);
                sum_sq += v * v;
            }
        }
    } else {
        for (int i = threadIdx.x; i < dim; i += 256) {
            const float v = half_bits_to_float(row[i]);
            sum_sq += v * v;
        }
    }
    __shared__ float partial[4];
    const float sq = wave_xor_sum(sum_sq, 63);
    if (lane == 0) partial[wave] = sq;
    __syncthreads();
    const float inv_rms =
        rsqrtf((((partial[0] + partial[1]) + partial[2]) + partial[3]) / static_cast<float>(dim) + eps);
    uint16_t* dst = out + static_cast<size_t>(token) * out_stride;
    if (VEC) {
        auto scaled = [&](const half8_t& v8, int i) {
            half8_t w8;
            if (weight != nullptr) w8 = *reinterpret_cast<const half8_t*>(weight + i);
            half8_t o;
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const float w = weight != nullptr ? static_cast<float>(w8[q]) : 1.0f;
                o[q] = static_cast<half_t>(static_cast<float>(v8[q]) * inv_rms * w);
            }
            *reinterpret_cast<half8_t*>(dst + i) = o;
        };
#pragma unroll
        for (int r = 0; r < kRmsHeld; ++r) {
            const int i = (r * 256 + threadIdx.x) * 8;
            if (i < dim) scaled(held[r], i);
        }
        for (int i = (kRmsHeld * 256 + threadIdx.x) * 8; i < dim; i += 256 * 8) {
            scaled(*reinterpret_cast<const half8_t*>(row + i), i);
        }
    } else {
        for (int i = threadIdx.x; i < dim; i += 256) {
            const float w = weight != nullptr ? half_bits_to_float(weight[i]) : 1.0f;
            dst[i] = float_to_half_bits(half_bits_to_float(row[i]) * inv_rms * w);
        }
    }
}

}  // namespace aeon355

using namespace aeon355;

extern "C" int aeon_hc_project(const void* d_residual, int residual_is_f32, long token_stride,
                               long stream_stride, const float* d_fn, float* d_mixes, int tokens,
                               int hidden, float rms_eps, void* stream) {
    const char* who = "aeon_hc_project";
    AEON_REQUIRE(d_residual && d_fn && d_mixes, AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    AEON_REQUIRE(tokens >= 0 && hidden > 0 && hidden % 4 == 0 && token_stride % 4 == 0 &&
                     stream_stride % 4 == 0,
                 AEON_ERR_INVALID_ARGUMENT, "%s: bad shape or pitch (hidden=%d)", who, hidden);
    if (tokens == 0) return AEON_OK;
    if (residual_is_f32) {
        hc_project_kernel<true><<<tokens, 256, 0, as_stream(stream)>>>(
            d_residual, token_stride, stream_stride, d_fn, d_mixes, hidden, rms_eps);
    } else {
        hc_project_kernel<false><<<tokens, 256, 0, as_stream(stream)>>>(
            d_residual, token_stride, stream_stride, d_fn, d_mixes, hidden, rms_eps);
    }
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

extern "C" int aeon_rmsnorm(const void* d_x, long x_stride, const void* d_weight, void* d_out,
                            long out_stride, int tokens, int dim, float eps, void* stream) {
    const char* who = "aeon_rmsnorm";
    AEON_REQUIRE(d_x && d_out, AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    AEON_REQUIRE(tokens >= 0 && dim > 0 && x_stride >= dim && out_stride >= dim,
                 AEON_ERR_INVALID_ARGUMENT, "%s: bad shape or pitch (dim=%d)", who, dim);
    if (tokens == 0) return AEON_OK;
    const bool vec = dim % 8 == 0 && x_stride % 8 == 0 && out_stride % 8 == 0 &&
                     ((reinterpret_cast<uintptr_t>(d_x) | reinterpret_cast<uintptr_t>(d_out) |
                       reinterpret_cast<uintptr_t>(d_weight)) & 15) == 0;
    if (vec) {
        rmsnorm_kernel<true><<<tokens, 256, 0, as_stream(stream)>>>(
            static_cast<const uint16_t*>(d_x), x_stride, static_cast<const uint16_t*>(d_weight),
            static_cast<uint16_t*>(d_out), out_stride, dim, eps);
    } else {
        rmsnorm_kernel<false><<<tokens, 256, 0, as_stream(stream)>>>(
            static_cast<const uint16_t*>(d_x), x_stride, static_cast<const uint16_t*>(d_weight),
            static_cast<uint16_t*>(d_out), out_stride, dim, eps);
    }
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

extern "C" int aeon_hc_post(const void* d_layer_out, long layer_out_stride,
                            const void* d_residual_in, long token_stride, long stream_stride,
                            const float* d_post_mix, const float* d_comb_mix, int mix_per_token,
                            void* d_residual_out, int tokens, int hidden, void* stream) {
    const char* who = "aeon_hc_post";
    AEON_REQUIRE(d_layer_out && d_residual_in && d_post_mix && d_comb_mix && d_residual_out,
                 AEON_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    AEON_REQUIRE(tokens >= 0 && hidden > 0 && hidden % 8 == 0 && token_stride % 8 == 0 &&
                     stream_stride % 8 == 0 && layer_out_stride % 8 == 0 &&
                     layer_out_stride >= hidden,
                 AEON_ERR_INVALID_ARGUMENT, "%s: bad shape or pitch", who);
    AEON_REQUIRE(d_residual_in != d_residual_out, AEON_ERR_INVALID_ARGUMENT,
                 "%s: every output stream reads all four input streams; in-place is not defined",
                 who);
    if (tokens == 0) return AEON_OK;
    hc_post_kernel<<<dim3((hidden / 8 + 255) / 256, tokens), 256, 0, as_stream(stream)>>>(
        static_cast<const uint16_t*>(d_layer_out), layer_out_stride,
        static_cast<const uint16_t*>(d_residual_in), token_stride, stream_stride, d_post_mix,
        d_comb_mix, mix_per_token ? 1 : 0, static_cast<uint16_t*>(d_residual_out), hidden);
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}
