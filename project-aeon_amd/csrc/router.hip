// MoE router: fp32 logits = x . Wr, then score, biased top-k selection and renormalised weights.
//
// Selection runs in fp64 on the device. The specification the results are held to is an fp64
// host computation (descending biased score, ties to the lower index); two experts whose
// biased scores differ by less than an fp32 rounding would otherwise be ordered by rounding
// noise, and the routed ids have to match the host bit for bit.
#include "router.hpp"

namespace aeon355 {

constexpr int kRouterTokenTile = 16;   // tokens per workgroup: the M of the fp32 MFMA
constexpr int kRouterWaves = 4;        // waves per workgroup, each with its own slice of rows
constexpr int kRouterWaveRows = 112;   // rows of Wr per wave (7 MFMA passes of 16 rows)
constexpr int kRouterChunkRows = kRouterWaves * kRouterWaveRows;  // rows per workgroup
constexpr int kRouterMaxExperts = 1024;

// partial[c][t][e] = sum over the rows h of chunk c of x[t][h] * Wr[h][e], on the fp32 matrix
// cores (v_mfma_f32_16x16x4_f32: full fp32 operands and accumulate).
// One workgroup = (chunk of 448 rows, 16 tokens, 64 experts). Each of its four waves takes 112
// rows; per 16 rows a lane reads 4 activations (8 bytes) and four float4 of Wr (row
// 4*(l/16)+s, experts 4*(l%16)..+3 of the block -- 256 contiguous bytes per row), which feed
// 16 MFMAs: component j of the float4 is the B operand of the tile holding experts 4n+j. The
// waves' tiles are added through LDS in wave order, so the result does not depend on timing.
__global__ __launch_bounds__(kRouterWaves * 64) void router_logits_partial_kernel(
    const uint16_t* __restrict__ x, long x_stride, const float* __restrict__ wr,
    float* __restrict__ partial, int tokens, int hidden, int experts) {
    const int chunk = blockIdx.x;
    const int t0 = blockIdx.y * kRouterTokenTile;
    const int e0 = blockIdx.z * 64;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 15;
    const int kq = lane >> 4;
    const int h_begin = chunk * kRouterChunkRows + wave * kRouterWaveRows;
    const int token = min(t0 + n, tokens - 1);  // a padded row repeats a live token, never stored
    const uint16_t* xrow = x + token * x_stride;
    const int e = e0 + 4 * n;

    float4_t acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    // every load of the wave's 112 rows is issued before the first MFMA: the kernel is a few
    // microseconds long, so one round trip to HBM is all it can afford
    constexpr int kSteps = kRouterWaveRows / 16;
    uint2 xa[kSteps];
    float4_t b[kSteps][4];
    // the fast path reads 16 bytes of a weight row at column e and 8 bytes of an activation row:
    // both must be aligned, which an expert count that is not a multiple of four (rows of the
    // weight then start at 4-byte offsets) or an odd base pointer would break
    const bool whole = (e + 3 < experts) && (experts % 4 == 0) && (h_begin + kRouterWaveRows <= hidden) &&
                       (x_stride % 4 == 0) && ((reinterpret_cast<uintptr_t>(wr) & 15) == 0) &&
                       ((reinterpret_cast<uintptr_t>(x) & 7) == 0);
    if (whole) {
#pragma unroll
        for (int step = 0; step < kSteps; ++step) {
            const int h = h_begin + step * 16 + 4 * kq;
            xa[step] = *reinterpret_cast<const uint2*>(xrow + h);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                b[step][r] = *reinterpret_cast<const float4_t*>(wr + static_cast<size_t>(h + r) * experts + e);
            }
        }
    } else {
#pragma unroll
        for (int step = 0; step < kSteps; ++step) {
            const int h = h_begin + step * 16 + 4 * kq;
            uint16_t xv[4] = {0, 0, 0, 0};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                b[step][r] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
                if (h + r < hidden) {
                    xv[r] = xrow[h + r];
                    for (int q = 0; q < 4; ++q) {
                        if (e + q < experts) b[step][r][q] = wr[static_cast<size_t>(h + r) * experts + e + q];
                    }
                }
            }
            xa[step] = make_uint2(xv[0] | (static_cast<uint32_t>(xv[1]) << 16),
                                  xv[2] | (static_cast<uint32_t>(xv[3]) << 16));
        }
    }
#pragma unroll
    for (int step = 0; step < kSteps; ++step) {
        const float a[4] = {half_bits_to_float(static_cast<uint16_t>(xa[step].x & 0xFFFFu)),
                            half_bits_to_float(static_cast<uint16_t>(xa[step].x >> 16)),
                            half_bits_to_float(static_cast<uint16_t>(xa[step].y & 0xFFFFu)),
                            half_bits_to_float(static_cast<uint16_t>(xa[step].y >> 16))};
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[r], b[step][r][j], acc[j], 0, 0, 0);
            }
    }

    __shared__ float4_t sums[kRouterWaves - 1][4][64];
    if (wave > 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) sums[wave - 1][j][lane] = acc[j];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float4_t v = acc[j];
#pragma unroll
            for (int w = 0; w < kRouterWaves - 1; ++w) v += sums[w][j][lane];
            // lane holds tokens 4*kq + i (i = 0..3) of expert e0 + 4*n + j
            const int ee = e0 + 4 * n + j;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int t = t0 + 4 * kq + i;
                if (t < tokens && ee < experts) {
                    partial[(static_cast<size_t>(chunk) * tokens + t) * experts + ee] = v[i];
                }
            }
        }
    }
}

// logits[i] = sum over chunks, ascending (sixteen loads in flight).
__global__ __launch_bounds__(256) void router_logits_reduce_kernel(
    const float* __restrict__ partial, float* __restrict__ logits, int chunks, size_t count) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float acc = 0.0f;
    for (int c0 = 0; c0 < chunks; c0 += 16) {
        float v[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) v[j] = c0 + j < chunks ? partial[static_cast<size_t>(c0 + j) * count + i] : 0.0f;
#pragma unroll
        for (int j = 0; j < 16; ++j) acc += v[j];
    }
    logits[i] = acc;
}

__device__ __forceinline__ double router_score(double logit, int score_kind) {
    if (score_kind == AEON_ROUTER_SCORE_SIGMOID) return 1.0 / (1.0 + exp(-logit));
    const double softplus = logit > 20.0 ? logit : log1p(exp(logit));
    return sqrt(softplus);
}

// One workgroup of 256 x kParts threads per token. When `partial` is given the first 256 threads
// sum the token's logits over the chunks (ascending) into `logits` and score their experts in
// fp64. Each expert's rank under the total order (biased score descending, index ascending) is
// then counted against all experts held in LDS, the candidates split into kParts ranges whose
// counts (integers, so the order of the adds does not matter) meet in LDS: rank r < top_k is the
// r-th pick. No serial scan and no cross-lane argmax, and the order -- ties to the lower index
// included -- is exactly the specification's.
template <int kPerThread, int kParts>
__global__ __launch_bounds__(256 * kParts) void router_topk_kernel(
    const float* __restrict__ partial, int chunks, int tokens, float* __restrict__ logits,
    const float* __restrict__ bias, const int64_t* __restrict__ hash_table,
    const int32_t* __restrict__ token_ids, float* __restrict__ topk_weights,
    int32_t* __restrict__ topk_indices, int experts, int top_k, float scaling, int renormalize,
    int score_kind) {
    const int token = blockIdx.x;
    __shared__ double choice_lds[kPerThread * 256];
    __shared__ double score_lds[kPerThread * 256];
    __shared__ double picked_score[64];
    __shared__ int picked_id[64];
    __shared__ int rank_lds[kPerThread * 256];
    float* out_row = logits + static_cast<size_t>(token) * experts;
    const int lane_expert = threadIdx.x % 256;
    const int part = threadIdx.x / 256;
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
        const int e = lane_expert + 256 * j;
        if (part == 0 && e < experts) {
            float acc;
            if (partial != nullptr) {
                acc = 0.0f;
                const size_t count = static_cast<size_t>(tokens) * experts;
                const float* p = partial + static_cast<size_t>(token) * experts + e;
                for (int c0 = 0; c0 < chunks; c0 += 16) {
                    float v[16];
#pragma unroll
                    for (int q = 0; q < 16; ++q) v[q] = c0 + q < chunks ? p[static_cast<size_t>(c0 + q) * count] : 0.0f;
#pragma unroll
                    for (int q = 0; q < 16; ++q) acc += v[q];
                }
                out_row[e] = acc;
            } else {
                acc = out_row[e];
            }
            const double sc = router_score(static_cast<double>(acc), score_kind);
            score_lds[e] = sc;
            choice_lds[e] = bias != nullptr ? sc + static_cast<double>(bias[e]) : sc;
            rank_lds[e] = 0;
        }
    }
    __syncthreads();

    const bool hashed = hash_table != nullptr && token_ids != nullptr;
    if (hashed) {
        if (static_cast<int>(threadIdx.x) < top_k) {
            const int e = static_cast<int>(
                hash_table[static_cast<size_t>(token_ids[token]) * top_k + threadIdx.x]);
            picked_id[threadIdx.x] = e;
            picked_score[threadIdx.x] = score_lds[e];
        }
    } else {
        const int span = (experts + kParts - 1) / kParts;
        const int first = part * span;
        const int last = first + span < experts ? first + span : experts;
#pragma unroll
        for (int j = 0; j < kPerThread; ++j) {
            const int e = lane_expert + 256 * j;
            if (e < experts) {
                int rank = 0;
                const double mine = choice_lds[e];
                // A candidate f beats e when its score is higher, or equal with f < e. The wave's
                // experts are 64 consecutive indices: for the candidates below all of them the
                // test is one >=, for those above all of them one >, and only the 64 candidates
                // in between need the index (the three loops' bounds are the same for the wave).
                const int wave_lo = e - static_cast<int>(threadIdx.x & 63);
                const int begin = min(first, last);   // a part past the last expert has no range
                const int below_end = min(last, max(begin, wave_lo));
                const int above_begin = max(below_end, min(last, wave_lo + 64));
                for (int f = begin; f < below_end; ++f) rank += choice_lds[f] >= mine ? 1 : 0;
                for (int f = below_end; f < above_begin; ++f) {
                    const double other = choice_lds[f];
                    rank += (other > mine || (other == mine && f < e)) ? 1 : 0;
                }
                for (int f = above_begin; f < last; ++f) rank += choice_lds[f] > mine ? 1 : 0;
                if (kParts > 1) atomicAdd(&rank_lds[e], rank);
                else rank_lds[e] = rank;
            }
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < kPerThread; ++j) {
            const int e = lane_expert + 256 * j;
            if (part == 0 && e < experts && rank_lds[e] < top_k) {
                picked_id[rank_lds[e]] = e;
                picked_score[rank_lds[e]] = score_lds[e];
            }
        }
    }
    __syncthreads();
    if (static_cast<int>(threadIdx.x) < top_k) {
        double sum = 0.0;
        for (int k = 0; k < top_k; ++k) sum += picked_score[k];
        double w = picked_score[threadIdx.x];
        if (renormalize) w = w / (sum + 1e-20);
        w *= static_cast<double>(scaling);
        topk_indices[static_cast<size_t>(token) * top_k + threadIdx.x] = picked_id[threadIdx.x];
        topk_weights[static_cast<size_t>(token) * top_k + threadIdx.x] = static_cast<float>(w);
    }
}

int router_logits_chunks(int tokens, int hidden) {
    (void)tokens;
    return (hidden + kRouterChunkRows - 1) / kRouterChunkRows;
}

// Launches the partial-sum kernel; the chunk sums are left for the caller's reduce.
int launch_router_partials(const void* d_x, int x_stride, const float* d_router_weight,
                           float* partial, int tokens, int hidden, int experts,
                           hipStream_t stream) {
    const int chunks = router_logits_chunks(tokens, hidden);
    const int tiles = (tokens + kRouterTokenTile - 1) / kRouterTokenTile;
    router_logits_partial_kernel<<<dim3(chunks, tiles, (experts + 63) / 64), kRouterWaves * 64, 0,
                                   stream>>>(static_cast<const uint16_t*>(d_x), x_stride,
                                             d_router_weight, partial, tokens, hidden, experts);
    AEON_LAUNCH_CHECK();
    return AEON_OK;
}

int launch_router_topk(const float* partial, int chunks, float* logits, const float* bias,
                       const int64_t* hash_table, const int32_t* token_ids, float* topk_weights,
                       int32_t* topk_indices, int tokens, int experts, int top_k, float scaling,
                       int renormalize, int score_kind, hipStream_t stream) {
    if (experts <= 256) {
        router_topk_kernel<1, 4><<<tokens, 1024, 0, stream>>>(
            partial, chunks, tokens, logits, bias, hash_table, token_ids, topk_weights,
            topk_indices, experts, top_k, scaling, renormalize, score_kind);
    } else {
        router_topk_kernel<kRouterMaxExperts / 256, 1><<<tokens, 256, 0, stream>>>(
            partial, chunks, tokens, logits, bias, hash_table, token_ids, topk_weights,
            topk_indices, experts, top_k, scaling, renormalize, score_kind);
    }
    AEON_LAUNCH_CHECK();
    return AEON_OK;
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
    hipStream_t s = as_stream(stream);
    float* partial = static_cast<float*>(d_workspace);
    if (int rc = launch_router_partials(d_x, x_stride, d_router_weight, partial, tokens, hidden,
                                        experts, s)) {
        return rc;
    }
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
    // with no partial sums the kernel only reads `logits`
    return launch_router_topk(nullptr, 0, const_cast<float*>(d_logits), d_bias, d_hash_table,
                              d_token_ids, d_topk_weights, d_topk_indices, tokens, experts, top_k,
                              routed_scaling_factor, renormalize, score_kind, as_stream(stream));
}

