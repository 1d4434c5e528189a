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
