// MoE router: fp32 logits = x . Wr, then score, biased top-k selection and renormalised weights.
//
// Selection runs in fp64 on the device. The specification the results are held to is an fp64
// host computation (descending biased score, ties to the lower index); two experts whose
// biased scores differ by less than an fp32 rounding would otherwise be ordered by rounding
// noise, and the routed ids have to match the host bit for bit.
#include "common.hpp"

namespace aeon355 {

constexpr int kRouterTokenTile = 16;
constexpr int kRouterMaxExperts = 1024;

// partial[c][t][e] = sum over the rows h of chunk c of x[t][h] * Wr[h][e].
// One workgroup = (chunk, tile of 16 tokens), four waves. A wave takes every fourth row of the
// chunk and reads it as one coalesced float4-per-lane load (64 lanes x 4 experts = 256 experts
// per pass), eight rows in flight; the four waves' sums meet in LDS in wave order, so the
// result does not depend on timing.
__global__ __launch_bounds__(256) void router_logits_partial_kernel(
    const uint16_t* __restrict__ x, long x_stride, const float* __restrict__ wr,
    float* __restrict__ partial, int tokens, int hidden, int experts, int chunk_rows) {
    const int chunk = blockIdx.x;
    const int t0 = blockIdx.y * kRouterTokenTile;
    const int h0 = chunk * chunk_rows;
    const int h1 = min(hidden, h0 + chunk_rows);
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    extern __shared__ float lds[];
    float* xs = lds;                                  // [chunk_rows][kRouterTokenTile]
    float* sums = lds + chunk_rows * kRouterTokenTile;  // [3][kRouterTokenTile][256]: waves 1..3
    for (int i = threadIdx.x; i < kRouterTokenTile * chunk_rows; i += blockDim.x) {
        const int t = i % kRouterTokenTile;
        const int h = h0 + i / kRouterTokenTile;
        xs[i] = (t0 + t < tokens && h < h1) ? half_bits_to_float(x[(t0 + t) * x_stride + h]) : 0.0f;
    }
    __syncthreads();
    for (int e0 = 0; e0 < experts; e0 += 256) {
        const int e = e0 + lane * 4;
        float4_t acc[kRouterTokenTile];
#pragma unroll
        for (int t = 0; t < kRouterTokenTile; ++t) acc[t] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        constexpr int kRows = 8;
        for (int hb = h0 + wave; hb < h1; hb += 4 * kRows) {
            float4_t w[kRows];
#pragma unroll
            for (int j = 0; j < kRows; ++j) {
                const int h = hb + 4 * j;
                w[j] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
                if (h < h1 && e + 3 < experts) {
                    w[j] = *reinterpret_cast<const float4_t*>(wr + static_cast<size_t>(h) * experts + e);
                } else if (h < h1) {
                    for (int q = 0; q < 4; ++q) {
                        if (e + q < experts) w[j][q] = wr[static_cast<size_t>(h) * experts + e + q];
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < kRows; ++j) {
                const int h = hb + 4 * j;
                if (h < h1) {
                    const float* xrow = xs + (h - h0) * kRouterTokenTile;
#pragma unroll
                    for (int t = 0; t < kRouterTokenTile; ++t) acc[t] += xrow[t] * w[j];
                }
            }
        }
        if (wave > 0) {
#pragma unroll
            for (int t = 0; t < kRouterTokenTile; ++t) {
                *reinterpret_cast<float4_t*>(sums + ((wave - 1) * kRouterTokenTile + t) * 256 +
                                             lane * 4) = acc[t];
            }
        }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int t = 0; t < kRouterTokenTile; ++t) {
                float4_t v = acc[t];
#pragma unroll
                for (int w2 = 0; w2 < 3; ++w2) {
                    v += *reinterpret_cast<const float4_t*>(sums + (w2 * kRouterTokenTile + t) * 256 +
                                                            lane * 4);
                }
                if (t0 + t < tokens) {
                    float* dst = partial + (static_cast<size_t>(chunk) * tokens + t0 + t) * experts + e;
                    for (int q = 0; q < 4; ++q) {
                        if (e + q < experts) dst[q] = v[q];
                    }
                }
            }
        }
        __syncthreads();
    }
}

// logits[i] = sum over chunks, ascending (eight loads in flight).
__global__ __launch_bounds__(256) void router_logits_reduce_kernel(
    const float* __restrict__ partial, float* __restrict__ logits, int chunks, size_t count) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float acc = 0.0f;
    for (int c0 = 0; c0 < chunks; c0 += 8) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = c0 + j < chunks ? partial[static_cast<size_t>(c0 + j) * count + i] : 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) acc += v[j];
    }
    logits[i] = acc;
}

__device__ __forceinline__ double router_score(double logit, int score_kind) {
    if (score_kind == AEON_ROUTER_SCORE_SIGMOID) return 1.0 / (1.0 + exp(-logit));
    const double softplus = logit > 20.0 ? logit : log1p(exp(logit));
    return sqrt(softplus);
}

// One wave per token. Lane l owns experts l, l+64, ...; each of the k rounds is a lane-local
// scan in ascending index followed by a wave arg-max whose ties go to the lower index.
template <int kPerLane>
__global__ __launch_bounds__(64) void router_topk_kernel(
    const float* __restrict__ logits, const float* __restrict__ bias,
    const int64_t* __restrict__ hash_table, const int32_t* __restrict__ token_ids,
    float* __restrict__ topk_weights, int32_t* __restrict__ topk_indices, int experts, int top_k,
    float scaling, int renormalize, int score_kind) {
    const int token = blockIdx.x;
    const int lane = threadIdx.x;
    const float* row = logits + static_cast<size_t>(token) * experts;

    double score[kPerLane];
    double choice[kPerLane];
#pragma unroll
    for (int j = 0; j < kPerLane; ++j) {
        const int e = lane + 64 * j;
        if (e < experts) {
            score[j] = router_score(static_cast<double>(row[e]), score_kind);
            choice[j] = bias != nullptr ? score[j] + static_cast<double>(bias[e]) : score[j];
        } else {
            score[j] = 0.0;
            choice[j] = -1.0e300;
        }
    }

    __shared__ double picked_score[64];
    __shared__ int picked_id[64];
    const bool hashed = hash_table != nullptr && token_ids != nullptr;
    for (int k = 0; k < top_k; ++k) {
        int best_e;
        if (hashed) {
            best_e = static_cast<int>(hash_table[static_cast<size_t>(token_ids[token]) * top_k + k]);
        } else {
            double best_v = -1.0e300;
            best_e = 0x7FFFFFFF;
#pragma unroll
            for (int j = 0; j < kPerLane; ++j) {
                const int e = lane + 64 * j;
                if (e < experts && choice[j] > best_v) {
                    best_v = choice[j];
                    best_e = e;
                }
            }
#pragma unroll
            for (int offset = 32; offset > 0; offset >>= 1) {
                const double other_v = __shfl_xor(best_v, offset, 64);
                const int other_e = __shfl_xor(best_e, offset, 64);
                if (other_v > best_v || (other_v == best_v && other_e < best_e)) {
                    best_v = other_v;
                    best_e = other_e;
                }
            }
        }
        // the owner publishes the unbiased score and retires the expert
        if ((best_e & 63) == lane) {
            const int j = best_e >> 6;
            double s = 0.0;
#pragma unroll
            for (int jj = 0; jj < kPerLane; ++jj) {
                if (jj == j) {
                    s = score[jj];
                    if (!hashed) choice[jj] = -1.0e300;
                }
            }
            picked_score[k] = s;
            picked_id[k] = best_e;
        }
    }
    __syncthreads();
    if (lane < top_k) {
        double sum = 0.0;
        for (int k = 0; k < top_k; ++k) sum += picked_score[k];
        double w = picked_score[lane];
        if (renormalize) w = w / (sum + 1e-20);
        w *= static_cast<double>(scaling);
        topk_indices[static_cast<size_t>(token) * top_k + lane] = picked_id[lane];
        topk_weights[static_cast<size_t>(token) * top_k + lane] = static_cast<float>(w);
    }
}

int router_logits_chunks(int tokens, int hidden) {
    // about 256 workgroups: many short chunks for a decode batch, few for a prefill chunk
    const int tiles = (tokens + kRouterTokenTile - 1) / kRouterTokenTile;
    int chunks = 256 / (tiles > 0 ? tiles : 1);
    if (chunks > 64) chunks = 64;
    if (chunks < 1) chunks = 1;
    const int max_chunks = (hidden + 31) / 32;
    if (chunks > max_chunks) chunks = max_chunks;
    const int min_chunks = (hidden + 127) / 128;  // a chunk's activations must fit in LDS
    if (chunks < min_chunks) chunks = min_chunks;
    return chunks;
}

}  // namespace aeon355

using namespace aeon355;

extern "C" size_t aeon_router_logits_workspace_bytes(int tokens, int hidden, int experts) {
    if (tokens <= 0 || hidden <= 0 || experts <= 0) return 0;
    return static_cast<size_t>(router_logits_chunks(tokens, hidden)) * tokens * experts * sizeof(float);
}

extern "C" int aeon_router_logits(const void* d_x, int x_stride, const float* d_router_weight,
                                  float* d_logits, int tokens, int hidden, int experts,
                                  void* d_workspace, size_t workspace_bytes, void* stream) {
    const char* who = "aeon_router_logits";
    AEON_REQUIRE(d_x && d_router_weight && d_logits && d_workspace, AEON_ERR_INVALID_ARGUMENT,
                 "%s: null buffer", who);
    AEON_REQUIRE(tokens >= 0 && hidden > 0 && experts > 0 && x_stride >= hidden,
                 AEON_ERR_INVALID_ARGUMENT, "%s: bad shape (tokens=%d hidden=%d experts=%d pitch=%d)",
                 who, tokens, hidden, experts, x_stride);
    if (tokens == 0) return AEON_OK;
    AEON_REQUIRE(workspace_bytes >= aeon_router_logits_workspace_bytes(tokens, hidden, experts),
                 AEON_ERR_INVALID_ARGUMENT, "%s: workspace of %zu bytes is too small", who,
                 workspace_bytes);
    const int chunks = router_logits_chunks(tokens, hidden);
    const int chunk_rows = (hidden + chunks - 1) / chunks;
    const int tiles = (tokens + kRouterTokenTile - 1) / kRouterTokenTile;
    const size_t lds = static_cast<size_t>(kRouterTokenTile) * (chunk_rows + 3 * 256) * sizeof(float);
    AEON_REQUIRE(lds <= 64 * 1024, AEON_ERR_INVALID_ARGUMENT,
                 "%s: hidden=%d needs %zu bytes of LDS per chunk", who, hidden, lds);
    hipStream_t s = as_stream(stream);
    float* partial = static_cast<float*>(d_workspace);
    router_logits_partial_kernel<<<dim3(chunks, tiles), 256, lds, s>>>(
        static_cast<const uint16_t*>(d_x), x_stride, d_router_weight, partial, tokens, hidden,
        experts, chunk_rows);
    AEON_LAUNCH_CHECK();
    const size_t count = static_cast<size_t>(tokens) * experts;
    router_logits_reduce_kernel<<<static_cast<unsigned>((count + 255) / 256), 256, 0, s>>>(
        partial, d_logits, chunks, count);
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

extern "C" int aeon_moe_router(const float* d_logits, const float* d_bias,
                               const int64_t* d_hash_table, const int32_t* d_token_ids,
                               float* d_topk_weights, int32_t* d_topk_indices, int tokens,
                               int experts, int top_k, float routed_scaling_factor, int renormalize,
                               int score_kind, void* stream) {
    const char* who = "aeon_moe_router";
    AEON_REQUIRE(d_logits && d_topk_weights && d_topk_indices, AEON_ERR_INVALID_ARGUMENT,
                 "%s: null buffer", who);
    AEON_REQUIRE(tokens >= 0 && experts > 0 && experts <= kRouterMaxExperts && top_k > 0 &&
                     top_k <= 64 && top_k <= experts,
                 AEON_ERR_INVALID_ARGUMENT, "%s: bad shape (tokens=%d experts=%d top_k=%d)", who,
                 tokens, experts, top_k);
    AEON_REQUIRE(score_kind == AEON_ROUTER_SCORE_SQRT_SOFTPLUS || score_kind == AEON_ROUTER_SCORE_SIGMOID,
                 AEON_ERR_INVALID_ARGUMENT, "%s: unknown score kind %d", who, score_kind);
    AEON_REQUIRE((d_hash_table == nullptr) == (d_token_ids == nullptr), AEON_ERR_INVALID_ARGUMENT,
                 "%s: the hash branch needs both the table and the token ids", who);
    if (tokens == 0) return AEON_OK;
    if (experts <= 256) {
        router_topk_kernel<4><<<tokens, 64, 0, as_stream(stream)>>>(
            d_logits, d_bias, d_hash_table, d_token_ids, d_topk_weights, d_topk_indices, experts,
            top_k, routed_scaling_factor, renormalize, score_kind);
    } else {
        router_topk_kernel<kRouterMaxExperts / 64><<<tokens, 64, 0, as_stream(stream)>>>(
            d_logits, d_bias, d_hash_table, d_token_ids, d_topk_weights, d_topk_indices, experts,
            top_k, routed_scaling_factor, renormalize, score_kind);
    }
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}
